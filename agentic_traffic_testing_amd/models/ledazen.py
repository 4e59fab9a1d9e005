"""Ledazen decoder over the mixer op layer (``ops.mixers``).

Layer = one RMS norm (weight stored around zero) whose output feeds the sequence mixer and a
squared-ReLU feed-forward side by side; both are added to an fp32 residual stream.  Mixers:

* ``delta``    - gated delta rule (short convolutions on q / k / v, unit-length q and k, one
  decay per head, SiLU output gate);
* ``parallel`` - softmax attention (q/k norm, interleaved rotary positions, sink) next to a
  gated delta rule with one decay per head and key channel (low-rank decay and sigmoid gate
  projections); the branches are mixed with two configured weights.

MI355X layout: every projection that reads the layer's normed input is one row of blocks in a
single fused weight (one library GEMM per layer instead of ten), each block padded to 8 rows
so the slices the mixer kernels read stay 16-byte aligned; the three output projections are
library GEMMs whose products one kernel adds into the residual while it computes the next
layer's norm.  Softmax keys / values live in the paged pool, recurrent state, convolution
tails and the previous token in per-sequence state slots (``engine.state_cache``).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from pathlib import Path

import torch
import torch.nn.functional as F

from ..config import LedazenConfig
from ..engine.state_cache import HybridCache, LayerCacheSpec
from ..ops import mixers as mx


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


@dataclass
class HybridLayerWeights:
    norm: torch.Tensor
    w_in: torch.Tensor                    # fused input projections [sum of padded blocks, width]
    seg: dict = field(default_factory=dict)   # block name -> (column offset, width)
    # softmax branch
    q_norm: torch.Tensor | None = None
    k_norm: torch.Tensor | None = None
    inv_freq: torch.Tensor | None = None
    attn_o: torch.Tensor | None = None
    # delta branch
    conv_w: torch.Tensor | None = None        # [2 * G * d + H * dv, taps] (q, k, v channels)
    a_log: torch.Tensor | None = None         # fp32 [H]
    dt_bias: torch.Tensor | None = None       # fp32 [H] or [H * d]
    a2: torch.Tensor | None = None            # low-rank decay, second factor
    g2: torch.Tensor | None = None            # low-rank gate, second factor
    out_norm: torch.Tensor | None = None
    delta_o: torch.Tensor | None = None
    # feed-forward
    down: torch.Tensor | None = None


class LedazenModel:
    family = "ledazen"
    has_state = True

    def __init__(self, cfg: LedazenConfig, dtype=torch.bfloat16, device="cuda", tp_rank: int = 0,
                 tp_size: int = 1, tp_group=None, quantization: str = ""):
        if tp_size != 1:
            raise ValueError("Ledazen runs on one GPU per replica (tensor_parallel_size 1)")
        if quantization:
            raise ValueError("Ledazen weights are 16-bit or 32-bit; no quantization")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Ledazen activations are bfloat16 or float32")
        self.cfg = cfg
        self.dtype = dtype
        self.device = torch.device(device)
        self.tp_rank, self.tp_size, self.tp_group = 0, 1, None
        self.layers: list[HybridLayerWeights] = []
        self.embed = self.pair_table = self.final_norm = self.head = None
        self.vocab_shard = cfg.vocab_size
        if self.dtype == torch.float32 and self.device.type == "cuda":
            # fp32 serving is exact fp32: no reduced-precision matrix mode
            torch.backends.cuda.matmul.allow_tf32 = False
            torch.backends.cudnn.allow_tf32 = False

    # ---------------------------------------------------------------------------------
    def tensor_shapes(self, decay_rank: int | None = None, gate_rank: int | None = None) -> dict:
        """Checkpoint tensor name -> shape for this configuration."""
        c = self.cfg
        W = c.hidden_size
        out = {"embed": (c.vocab_size, W), "bigram": (c.pair_buckets + 1, W),
               "final.norm": (W,), "head": (c.vocab_size, W)}

        def delta(pre, m):
            qk, vv = m.kv_heads * m.dim, m.heads * m.vdim
            out.update({pre + "q": (qk, W), pre + "q.conv": (qk, m.conv), pre + "k": (qk, W),
                        pre + "k.conv": (qk, m.conv), pre + "v": (vv, W),
                        pre + "v.conv": (vv, m.conv), pre + "b": (m.heads, W),
                        pre + "A_log": (m.heads,), pre + "norm": (m.vdim,), pre + "o": (W, vv)})
            if m.channel_decay:
                ra = decay_rank or m.decay_rank or 16
                rg = gate_rank or m.gate_rank or 16
                out.update({pre + "a1": (ra, W), pre + "a2": (m.heads * m.dim, ra),
                            pre + "dt_bias": (m.heads * m.dim,), pre + "g1": (rg, W),
                            pre + "g2": (vv, rg)})
            else:
                out.update({pre + "a": (m.heads, W), pre + "dt_bias": (m.heads,),
                            pre + "g": (vv, W)})

        for i, L in enumerate(c.layers):
            p = f"l{i}."
            out[p + "norm1"] = (W,)
            if L.kind == "parallel":
                s = L.softmax
                out.update({p + "mix.left.q": (s.heads * s.dim, W),
                            p + "mix.left.k": (s.kv_heads * s.dim, W),
                            p + "mix.left.v": (s.kv_heads * s.vdim, W),
                            p + "mix.left.q.norm": (s.dim,), p + "mix.left.k.norm": (s.dim,),
                            p + "mix.left.o": (W, s.heads * s.vdim)})
                delta(p + "mix.right.", L.delta)
            else:
                delta(p + "mix.", L.delta)
            if L.ff:
                out.update({p + "mlp.up": (L.ff, W), p + "mlp.down": (W, L.ff)})
        return out

    def random_state(self, seed: int = 0) -> dict:
        """Seeded random tensors under the checkpoint's names (bf16-representable values)."""
        g = torch.Generator().manual_seed(1234567 + seed)
        st = {}
        for name, shape in self.tensor_shapes().items():
            r = torch.randn(shape, generator=g)
            leaf = name.split(".")[-1]
            if name in ("embed", "bigram"):
                t = r
            elif leaf in ("norm1",) or name == "final.norm":
                t = 0.1 * r
            elif leaf == "norm":          # plain-weight norms (q / k / output)
                t = 1.0 + 0.1 * r
            elif leaf == "conv":
                t = 0.5 * r
            elif leaf == "A_log":
                t = torch.log(0.25 + 2.0 * torch.rand(shape, generator=g))
            elif leaf == "dt_bias":
                t = r - 1.0
            else:
                t = r / math.sqrt(shape[-1])
            st[name] = t.to(torch.bfloat16)
        return st

    def init_random(self, seed: int = 0):
        return self.load_state(self.random_state(seed))

    def load_safetensors(self, path: str):
        from safetensors import safe_open

        files = sorted(Path(path).glob("*.safetensors"))
        if not files:
            raise FileNotFoundError(f"no safetensors in {path}")
        st = {}
        for f in files:
            with safe_open(str(f), framework="pt") as sf:
                for k in sf.keys():
                    st[k] = sf.get_tensor(k)
        return self.load_state(st)

    def load_state(self, st: dict):
        """Build the fused device weights from checkpoint-named tensors."""
        c, dev, dt = self.cfg, self.device, self.dtype
        W = c.hidden_size

        def act(name, shape=None):
            t = st[name]
            if shape is not None and tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, configuration wants {shape}")
            return t.to(dt).to(dev).contiguous()

        def f32(name, shape=None):
            t = st[name]
            if shape is not None and tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, configuration wants {shape}")
            return t.float().to(dev).contiguous()

        self.embed = act("embed", (c.vocab_size, W))
        self.pair_table = act("bigram", (c.pair_buckets + 1, W))
        self.final_norm = act("final.norm", (W,))
        self.head = act("head", (c.vocab_size, W))
        self.layers = []
        for i, L in enumerate(c.layers):
            p = f"l{i}."
            blocks = []     # (name, tensor [n, W])
            lw = HybridLayerWeights(norm=act(p + "norm1", (W,)), w_in=None)
            if L.kind == "parallel":
                s = L.softmax
                blocks += [("sq", act(p + "mix.left.q", (s.heads * s.dim, W))),
                           ("sk", act(p + "mix.left.k", (s.kv_heads * s.dim, W))),
                           ("sv", act(p + "mix.left.v", (s.kv_heads * s.vdim, W)))]
                lw.q_norm = act(p + "mix.left.q.norm", (s.dim,))
                lw.k_norm = act(p + "mix.left.k.norm", (s.dim,))
                lw.inv_freq = mx.inv_freq(s.rot_dims, s.rot_base, dev)
                lw.attn_o = act(p + "mix.left.o", (W, s.heads * s.vdim))
                d = p + "mix.right."
            elif L.kind == "delta":
                d = p + "mix."
            else:
                raise ValueError(L.kind)
            m = L.delta
            qk, vv = m.kv_heads * m.dim, m.heads * m.vdim
            # q, k, v of the delta branch stay adjacent: one convolution launch covers them
            qkv = torch.cat([act(d + "q", (qk, W)), act(d + "k", (qk, W)), act(d + "v", (vv, W))])
            blocks.append(("dqkv", qkv))
            lw.conv_w = torch.cat([act(d + "q.conv", (qk, m.conv)), act(d + "k.conv", (qk, m.conv)),
                                   act(d + "v.conv", (vv, m.conv))]).contiguous()
            blocks.append(("beta", act(d + "b", (m.heads, W))))
            lw.a_log = f32(d + "A_log", (m.heads,))
            lw.out_norm = act(d + "norm", (m.vdim,))
            lw.delta_o = act(d + "o", (W, vv))
            if m.channel_decay:
                blocks += [("a1", act(d + "a1")), ("g1", act(d + "g1"))]
                lw.a2 = act(d + "a2")
                lw.g2 = act(d + "g2")
                if lw.a2.shape != (m.heads * m.dim, blocks[-2][1].shape[0]) or \
                        lw.g2.shape != (vv, blocks[-1][1].shape[0]):
                    raise ValueError(f"{d}a2 / g2: low-rank factors do not fit each other")
                lw.dt_bias = f32(d + "dt_bias", (m.heads * m.dim,))
            else:
                blocks += [("a", act(d + "a", (m.heads, W))), ("gate", act(d + "g", (vv, W)))]
                lw.dt_bias = f32(d + "dt_bias", (m.heads,))
            if L.ff:
                blocks.append(("up", act(p + "mlp.up", (L.ff, W))))
                lw.down = act(p + "mlp.down", (W, L.ff))
            rows, off = [], 0
            for name, t in blocks:
                n = t.shape[0]
                lw.seg[name] = (off, n)
                rows.append(t)
                if _pad8(n) != n:
                    rows.append(torch.zeros(_pad8(n) - n, W, dtype=dt, device=dev))
                off += _pad8(n)
            lw.w_in = torch.cat(rows).contiguous()
            self.layers.append(lw)
        return self

    def prepare_decode_weights(self):
        return self

    def decode_copy_bytes(self) -> int:
        return 0

    def weight_bytes(self) -> int:
        ts = [self.embed, self.pair_table, self.final_norm, self.head]
        for L in self.layers:
            ts += [L.norm, L.w_in, L.q_norm, L.k_norm, L.attn_o, L.conv_w, L.a_log, L.dt_bias, L.a2,
                   L.g2, L.out_norm, L.delta_o, L.down]
        return sum(t.numel() * t.element_size() for t in ts if t is not None)

    # ---------------------------------------------------------------------------------
    def cache_specs(self) -> list[LayerCacheSpec]:
        specs = []
        for L in self.cfg.layers:
            m = L.delta
            kw = dict(state_heads=m.heads, state_dim=m.dim, state_vdim=m.vdim,
                      conv_channels=2 * m.kv_heads * m.dim + m.heads * m.vdim, conv_taps=m.conv)
            if L.softmax is not None:
                s = L.softmax
                kw.update(kv_heads=s.kv_heads, kdim=s.dim, vdim=s.vdim)
            specs.append(LayerCacheSpec(**kw))
        return specs

    @property
    def attn_tile_tokens(self) -> int:
        return mx.ATTN_TILE_TOKENS

    # ---------------------------------------------------------------------------------
    def _delta_branch(self, P, lw, m, md, lc):
        """Gated delta rule on the slices of the fused projection ``P``; returns the gated,
        normed head outputs [T, heads * vdim] (before the output projection)."""
        eps = self.cfg.rms_norm_eps
        o, n = lw.seg["dqkv"]
        qkv = mx.short_conv_silu(P[:, o:o + n], lw.conv_w, lc.conv, md.positions, md.seq_qstart,
                                 md.seq_slot)
        o, n = lw.seg["beta"]
        beta = P[:, o:o + n]
        if m.channel_decay:
            o, n = lw.seg["a1"]
            decay = F.linear(P[:, o:o + n], lw.a2)
            o, n = lw.seg["g1"]
            gate = F.linear(P[:, o:o + n], lw.g2)
        else:
            o, n = lw.seg["a"]
            decay = P[:, o:o + n]
            o, n = lw.seg["gate"]
            gate = P[:, o:o + n]
        out = mx.gated_delta_rule(qkv, beta, decay, lw.a_log, lw.dt_bias, lc.state, md.positions,
                                  md.seq_qstart, md.seq_slot, m.heads, m.kv_heads, m.dim, m.vdim)
        return mx.gated_rms_norm(out, gate, lw.out_norm, eps,
                                 "sigmoid" if m.channel_decay else "silu", self.dtype)

    def _softmax_branch(self, P, lw, s, md, lc, tables):
        eps = self.cfg.rms_norm_eps
        key = (s.rot_dims, s.rot_base)
        if key not in tables:   # cos / sin of the step's positions, once per rotary setting
            tables[key] = mx.rotary_table(md.positions, lw.inv_freq)
        oq, nq = lw.seg["sq"]
        ok, nk = lw.seg["sk"]
        ov, nv = lw.seg["sv"]
        q = mx.qk_norm_rope_cache(P[:, oq:oq + nq], P[:, ok:ok + nk], P[:, ov:ov + nv], lw.q_norm,
                                  lw.k_norm, eps, md.positions, md.slot_mapping, tables[key], lc.k,
                                  lc.v, s.heads, s.kv_heads, s.dim, s.vdim)
        a = mx.sink_attention(q, lc.k, lc.v, md.block_tables, md.seq_kvlen, md.seq_qstart,
                              md.tile_seq, md.tile_qoff, s.scale, s.sink, md.num_decode,
                              md.max_decode_kv)
        return a.view(a.shape[0], s.heads * s.vdim)

    def forward(self, input_ids, md, cache: HybridCache, rows=None, layer_out=None):
        """One step over a decode-first batch of portions; returns the final-normed hidden rows
        (all, or ``rows``).  ``layer_out``: a list that receives a copy of the fp32 residual
        stream after every layer (debugging / tests)."""
        c = self.cfg
        eps = c.rms_norm_eps
        x = mx.embed_pair(self.embed, self.pair_table, input_ids, md.positions, md.seq_qstart,
                          md.seq_slot, cache.prev_token, c.pair_mul_prev, c.pair_mul_cur,
                          c.pair_buckets)
        h = mx.rms_norm_f32(x, self.layers[0].norm, eps, True, self.dtype) if self.layers else None
        last = len(self.layers) - 1
        tables = {}
        for li, (L, lw) in enumerate(zip(c.layers, self.layers)):
            lc = cache.layers[li]
            P = F.linear(h, lw.w_in)
            ff = None
            if L.ff:
                o, n = lw.seg["up"]
                ff = F.linear(mx.relu_sq(P[:, o:o + n]), lw.down)
            d = F.linear(self._delta_branch(P, lw, L.delta, md, lc), lw.delta_o)
            if L.kind == "parallel":
                a = F.linear(self._softmax_branch(P, lw, L.softmax, md, lc, tables), lw.attn_o)
                br = (a, L.softmax_scale, d, L.delta_scale, ff)
            else:
                br = (d, 1.0, None, 1.0, ff)
            if li < last:   # residual sum and the next layer's norm in one kernel
                h = mx.add_norm(x, *br, self.layers[li + 1].norm, eps, True, self.dtype)
            else:
                mx.residual_add(x, *br)
            if layer_out is not None:
                layer_out.append(x.clone())
        if rows is not None:
            x = x.index_select(0, rows)
        return mx.rms_norm_f32(x, self.final_norm, eps, True, self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.head).float()
