"""Soselix decoder over the mixer op layer (``ops.mixers``).

Pre-norm layers on an fp32 residual stream: ``x += m * mixer(norm1(x))`` then
``x += m * ff(norm2(x))`` with one-number RMS norms and a biased xIELU feed-forward.  Mixers:

* ``latent_attention`` - softmax attention over ONE cached latent per token (plus a rotated
  key part shared by the heads), queries through a latent of their own, a learned sink score per
  head, a sigmoid output gate per head; a layer may read an earlier layer's cache;
* ``hgrn2``  - linear attention whose per-channel forget gate is also the write gate;
* ``mamba2`` - state-space recurrence behind a short causal convolution, gated group norm.

MI355X layout: the projections that read a mixer's normed input are one fused library GEMM
(blocks padded to 8 rows so the kernels read 16-byte aligned slices in place).  Latent
attention runs in absorbed form - the key up-projection is applied to the queries, the value
up-projection to the attention output (two batched GEMMs per layer) - so prefill and decode
are multi-query attention over the compressed pages: a page holds ``kv_rank + rot_dim`` key
channels and ``kv_rank`` value channels per token for all heads.  The residual sum and the
next norm are one kernel; both recurrences run in one scan kernel with fp32 state in
per-sequence slots (``engine.state_cache``).  The one-number norm weights are expanded to
rows at load time so the fused norm kernels serve them unchanged.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from pathlib import Path

import torch
import torch.nn.functional as F

from ..config import Hgrn2Config, LatentAttentionConfig, Mamba2Config, SoselixConfig
from ..engine.state_cache import HybridCache, LayerCacheSpec
from ..ops import mixers as mx


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


@dataclass
class SoselixLayerWeights:
    norm1: torch.Tensor
    w_in: torch.Tensor                         # fused projections of the mixer's input
    seg: dict = field(default_factory=dict)    # block name -> (column offset, width)
    w_o: torch.Tensor | None = None
    # latent attention
    dq_norm: torch.Tensor | None = None
    uq: torch.Tensor | None = None
    dkv_norm: torch.Tensor | None = None
    uk: torch.Tensor | None = None             # [H, dim, kv_rank]
    uv_t: torch.Tensor | None = None           # [H, kv_rank, vdim]
    sink: torch.Tensor | None = None           # fp32 [H]
    inv_freq: torch.Tensor | None = None
    # recurrences
    p0: torch.Tensor | None = None             # fp32: hgrn2 gate bias / mamba2 dt bias
    p1: torch.Tensor | None = None             # fp32: hgrn2 lower bound / mamba2 A_log
    p2: torch.Tensor | None = None             # fp32: mamba2 D
    out_norm: torch.Tensor | None = None
    conv_w: torch.Tensor | None = None
    conv_b: torch.Tensor | None = None
    # feed-forward
    norm2: torch.Tensor | None = None
    up: torch.Tensor | None = None
    up_b: torch.Tensor | None = None
    down: torch.Tensor | None = None
    down_b: torch.Tensor | None = None
    act_p: float = 0.0                         # softplus of the two activation numbers
    act_q: float = 0.0


def _softplus(x: float) -> float:
    return max(x, 0.0) + math.log1p(math.exp(-abs(x)))


class SoselixModel:
    family = "soselix"
    has_state = True

    def __init__(self, cfg: SoselixConfig, dtype=torch.bfloat16, device="cuda", tp_rank: int = 0,
                 tp_size: int = 1, tp_group=None, quantization: str = ""):
        if tp_size != 1:
            raise ValueError("Soselix runs on one GPU per replica (tensor_parallel_size 1)")
        if quantization:
            raise ValueError("Soselix weights are 16-bit or 32-bit; no quantization")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Soselix activations are bfloat16 or float32")
        self.cfg = cfg
        self.dtype = dtype
        self.device = torch.device(device)
        self.tp_rank, self.tp_size, self.tp_group = 0, 1, None
        self.layers: list[SoselixLayerWeights] = []
        self.embed = self.final_norm = self.head = None
        self.vocab_shard = cfg.vocab_size
        if self.dtype == torch.float32 and self.device.type == "cuda":
            # fp32 serving is exact fp32: no reduced-precision matrix mode
            torch.backends.cuda.matmul.allow_tf32 = False
            torch.backends.cudnn.allow_tf32 = False

    # ---------------------------------------------------------------------------------
    def tensor_shapes(self) -> dict:
        """Checkpoint tensor name -> shape for this configuration."""
        c = self.cfg
        W = c.hidden_size
        out = {"embed": (c.vocab_size, W), "final.norm": (), "head": (c.vocab_size, W)}
        for i, L in enumerate(c.layers):
            p, m = f"l{i}.", L.mixer
            out[p + "norm1"] = ()
            x = p + "mix."
            if L.kind == "latent_attention":
                qr = m.q_rank or max(8, W // 2)
                out.update({x + "dq": (qr, W), x + "dq.norm": (qr,),
                            x + "uq": (m.heads * (m.dim + m.rot_dim), qr),
                            x + "uk": (m.heads * m.dim, m.kv_rank),
                            x + "uv": (m.heads * m.vdim, m.kv_rank), x + "sink": (m.heads,),
                            x + "g": (m.heads, W), x + "o": (W, m.heads * m.vdim)})
                if m.kv_from < 0:
                    out.update({x + "dkv": (m.kv_rank + m.rot_dim, W), x + "dkv.norm": (m.kv_rank,)})
            elif L.kind == "hgrn2":
                qk, vv = m.heads * m.dim, m.heads * m.vdim
                out.update({x + "q": (qk, W), x + "f": (qk, W), x + "f.b": (qk,),
                            x + "lower": (qk,), x + "v": (vv, W), x + "norm": (m.vdim,),
                            x + "o": (W, vv)})
            else:
                out.update({x + "in": (2 * m.inner + 2 * m.groups * m.state + m.heads, W),
                            x + "conv": (m.conv_channels, m.conv), x + "conv.b": (m.conv_channels,),
                            x + "dt_bias": (m.heads,), x + "A_log": (m.heads,), x + "D": (m.heads,),
                            x + "norm": (m.inner,), x + "o": (W, m.inner)})
            if L.ff:
                out.update({p + "norm2": (), p + "mlp.up": (L.ff, W), p + "mlp.up.b": (L.ff,),
                            p + "mlp.down": (W, L.ff), p + "mlp.down.b": (W,), p + "mlp.act": (2,)})
        return out

    def random_state(self, seed: int = 0) -> dict:
        """Seeded random tensors under the checkpoint's names (bf16-representable values)."""
        g = torch.Generator().manual_seed(7654321 + seed)
        st = {}
        for name, shape in self.tensor_shapes().items():
            r = torch.randn(shape, generator=g)
            leaf = name.split(".")[-1]
            if name == "embed":
                t = r
            elif leaf in ("norm1", "norm2") or name == "final.norm":
                t = 1.0 + 0.1 * r
            elif leaf == "norm":
                t = 1.0 + 0.1 * r
            elif leaf == "conv":
                t = 0.5 * r
            elif leaf == "b":
                t = 0.1 * r
            elif leaf == "A_log":
                t = torch.log(0.25 + 2.0 * torch.rand(shape, generator=g))
            elif leaf == "dt_bias":
                t = r - 1.0
            elif leaf == "D":
                t = 1.0 + 0.1 * r
            elif leaf == "lower":
                t = 0.9 * torch.rand(shape, generator=g)
            elif leaf in ("sink", "act"):
                t = 0.5 * r
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

        def get(name, shape):
            t = st[name]
            if shape is not None and tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, configuration wants {shape}")
            return t

        def act(name, shape=None):
            return get(name, shape).to(dt).to(dev).contiguous()

        def f32(name, shape=None):
            return get(name, shape).float().to(dev).contiguous()

        def one(name):   # a one-number norm weight as a row for the fused norm kernels
            return get(name, ()).to(dt).reshape(1).expand(W).to(dev).contiguous()

        def fuse(lw, blocks):
            rows, off = [], 0
            for name, t in blocks:
                n = t.shape[0]
                lw.seg[name] = (off, n)
                rows.append(t)
                if _pad8(n) != n:
                    rows.append(torch.zeros(_pad8(n) - n, W, dtype=dt, device=dev))
                off += _pad8(n)
            lw.w_in = torch.cat(rows).contiguous()

        self.embed = act("embed", (c.vocab_size, W))
        self.final_norm = one("final.norm")
        self.head = act("head", (c.vocab_size, W))
        self.layers = []
        for i, L in enumerate(c.layers):
            p, m = f"l{i}.", L.mixer
            x = p + "mix."
            lw = SoselixLayerWeights(norm1=one(p + "norm1"), w_in=None)
            if L.kind == "latent_attention":
                qr = st[x + "dq"].shape[0]
                if m.q_rank and m.q_rank != qr:
                    raise ValueError(f"{x}dq: {qr} rows, configuration says q_rank {m.q_rank}")
                blocks = [("dq", act(x + "dq", (qr, W)))]
                if m.kv_from < 0:
                    blocks.append(("dkv", act(x + "dkv", (m.kv_rank + m.rot_dim, W))))
                    lw.dkv_norm = act(x + "dkv.norm", (m.kv_rank,))
                blocks.append(("gate", act(x + "g", (m.heads, W))))
                fuse(lw, blocks)
                lw.dq_norm = act(x + "dq.norm", (qr,))
                lw.uq = act(x + "uq", (m.heads * (m.dim + m.rot_dim), qr))
                lw.uk = act(x + "uk", (m.heads * m.dim, m.kv_rank)).view(
                    m.heads, m.dim, m.kv_rank).contiguous()
                lw.uv_t = act(x + "uv", (m.heads * m.vdim, m.kv_rank)).view(
                    m.heads, m.vdim, m.kv_rank).transpose(1, 2).contiguous()
                lw.sink = f32(x + "sink", (m.heads,))
                lw.inv_freq = mx.inv_freq(m.rot_dims, m.rot_base, dev)
                lw.w_o = act(x + "o", (W, m.heads * m.vdim))
            elif L.kind == "hgrn2":
                qk, vv = m.heads * m.dim, m.heads * m.vdim
                fuse(lw, [("q", act(x + "q", (qk, W))), ("f", act(x + "f", (qk, W))),
                          ("v", act(x + "v", (vv, W)))])
                lw.p0 = f32(x + "f.b", (qk,))
                lw.p1 = f32(x + "lower", (qk,))
                lw.out_norm = act(x + "norm", (m.vdim,))
                lw.w_o = act(x + "o", (W, vv))
            elif L.kind == "mamba2":
                gn = m.groups * m.state
                w = act(x + "in", (2 * m.inner + 2 * gn + m.heads, W))
                # z | x B C (one convolution over the adjacent block) | dt
                fuse(lw, [("z", w[:m.inner]), ("xbc", w[m.inner:2 * m.inner + 2 * gn]),
                          ("dt", w[2 * m.inner + 2 * gn:])])
                lw.conv_w = act(x + "conv", (m.conv_channels, m.conv))
                lw.conv_b = act(x + "conv.b", (m.conv_channels,))
                lw.p0 = f32(x + "dt_bias", (m.heads,))
                lw.p1 = f32(x + "A_log", (m.heads,))
                lw.p2 = f32(x + "D", (m.heads,))
                lw.out_norm = act(x + "norm", (m.inner,))
                lw.w_o = act(x + "o", (W, m.inner))
            else:
                raise ValueError(L.kind)
            if L.ff:
                lw.norm2 = one(p + "norm2")
                lw.up = act(p + "mlp.up", (L.ff, W))
                lw.up_b = act(p + "mlp.up.b", (L.ff,))
                lw.down = act(p + "mlp.down", (W, L.ff))
                lw.down_b = act(p + "mlp.down.b", (W,))
                a = get(p + "mlp.act", (2,)).double()
                lw.act_p, lw.act_q = _softplus(float(a[0])), _softplus(float(a[1]))
            self.layers.append(lw)
        return self

    def prepare_decode_weights(self):
        return self

    def decode_copy_bytes(self) -> int:
        return 0

    def weight_bytes(self) -> int:
        ts = [self.embed, self.final_norm, self.head]
        for L in self.layers:
            ts += [v for v in vars(L).values() if isinstance(v, torch.Tensor)]
        return sum(t.numel() * t.element_size() for t in ts if t is not None)

    # ---------------------------------------------------------------------------------
    def cache_specs(self) -> list[LayerCacheSpec]:
        specs = []
        for L in self.cfg.layers:
            m = L.mixer
            if isinstance(m, LatentAttentionConfig):
                specs.append(LayerCacheSpec(kv_heads=1, kdim=m.kv_rank + m.rot_dim, vdim=m.kv_rank,
                                            kv_from=m.kv_from))
            elif isinstance(m, Hgrn2Config):
                specs.append(LayerCacheSpec(state_heads=m.heads, state_dim=m.dim,
                                            state_vdim=m.vdim))
            elif isinstance(m, Mamba2Config):
                specs.append(LayerCacheSpec(state_heads=m.heads, state_dim=m.state,
                                            state_vdim=m.vdim, conv_channels=m.conv_channels,
                                            conv_taps=m.conv))
        return specs

    @property
    def attn_tile_tokens(self) -> int:
        return mx.ATTN_TILE_TOKENS

    # ---------------------------------------------------------------------------------
    def _latent_attention(self, h, lw, m, md, lc, tables):
        eps = self.cfg.rms_norm_eps
        T = h.shape[0]
        P = F.linear(h, lw.w_in)
        key = (m.rot_dims, m.rot_base)
        if key not in tables:   # cos / sin of the step's positions, once per rotary setting
            tables[key] = mx.rotary_table(md.positions, lw.inv_freq)
        o, n = lw.seg["dq"]
        q = F.linear(mx.rms_norm_rows(P[:, o:o + n], lw.dq_norm, eps), lw.uq)
        q = q.view(T, m.heads, m.dim + m.rot_dim)
        # absorbed queries: q_unrotated W_uk per head, then [ . | rotated part ]
        q_lat = torch.bmm(q[:, :, :m.dim].transpose(0, 1), lw.uk)
        kvx = None
        if m.kv_from < 0:
            o, n = lw.seg["dkv"]
            kvx = P[:, o:o + n]
        qa = mx.latent_rope_cache(q_lat, q, kvx, lw.dkv_norm, eps, md.slot_mapping, tables[key],
                                  lc.k, lc.v)
        a = mx.sink_attention(qa, lc.k, lc.v, md.block_tables, md.seq_kvlen, md.seq_qstart,
                              md.tile_seq, md.tile_qoff, m.scale, True, md.num_decode,
                              md.max_decode_kv, sink_values=lw.sink)
        ov = torch.bmm(a.transpose(0, 1), lw.uv_t)          # [H, T, vdim]
        o, n = lw.seg["gate"]
        return F.linear(mx.head_gate(ov.contiguous(), P[:, o:o + n]), lw.w_o)

    def _hgrn2(self, h, lw, m, md, lc):
        P = F.linear(h, lw.w_in)
        (oq, nq), (of, nf), (ov, nv) = lw.seg["q"], lw.seg["f"], lw.seg["v"]
        o = mx.forget_gate_scan(P[:, oq:oq + nq], P[:, of:of + nf], P[:, ov:ov + nv], lw.p0, lw.p1,
                                lc.state, md.positions, md.seq_qstart, md.seq_slot, m.heads, m.dim,
                                m.vdim)
        y = mx.group_rms_norm(o.view(o.shape[0], m.heads * m.vdim), None, lw.out_norm, m.heads,
                              self.cfg.rms_norm_eps, self.dtype)
        return F.linear(y, lw.w_o)

    def _mamba2(self, h, lw, m, md, lc):
        P = F.linear(h, lw.w_in)
        (oz, nz), (ox, nx), (od, nd) = lw.seg["z"], lw.seg["xbc"], lw.seg["dt"]
        xbc = mx.short_conv_silu(P[:, ox:ox + nx], lw.conv_w, lc.conv, md.positions, md.seq_qstart,
                                 md.seq_slot, bias=lw.conv_b)
        gn = m.groups * m.state
        y = mx.state_space_scan(xbc[:, :m.inner], xbc[:, m.inner:m.inner + gn],
                                xbc[:, m.inner + gn:], P[:, od:od + nd], lw.p0, lw.p1, lw.p2,
                                lc.state, md.positions, md.seq_qstart, md.seq_slot, m.heads,
                                m.groups, m.state, m.vdim)
        y = mx.group_rms_norm(y.view(y.shape[0], m.inner), P[:, oz:oz + nz], lw.out_norm,
                              m.norm_groups, self.cfg.rms_norm_eps, self.dtype)
        return F.linear(y, lw.w_o)

    def forward(self, input_ids, md, cache: HybridCache, rows=None, layer_out=None):
        """One step over a decode-first batch of portions; returns the final-normed hidden rows
        (all, or ``rows``).  ``layer_out``: a list that receives a copy of the fp32 residual
        stream after every layer (debugging / tests)."""
        c = self.cfg
        eps, mult = c.rms_norm_eps, c.residual_mult
        x = mx.embed_scale(self.embed, input_ids, c.embed_scale)
        h = mx.rms_norm_f32(x, self.layers[0].norm1, eps, False, self.dtype) if self.layers else None
        last = len(self.layers) - 1
        tables = {}
        for li, (L, lw) in enumerate(zip(c.layers, self.layers)):
            lc = cache.layers[li]
            if L.kind == "latent_attention":
                y = self._latent_attention(h, lw, L.mixer, md, lc, tables)
            elif L.kind == "hgrn2":
                y = self._hgrn2(h, lw, L.mixer, md, lc)
            else:
                y = self._mamba2(h, lw, L.mixer, md, lc)
            if L.ff:   # residual sum and the feed-forward's norm in one kernel
                h2 = mx.add_norm(x, y, mult, None, 1.0, None, lw.norm2, eps, False, self.dtype)
                u = mx.xielu_bias(F.linear(h2, lw.up), lw.up_b, lw.act_p, lw.act_q)
                y = F.linear(u, lw.down, lw.down_b)
            if li < last:
                h = mx.add_norm(x, y, mult, None, 1.0, None, self.layers[li + 1].norm1, eps, False,
                                self.dtype)
            else:
                mx.residual_add(x, y, mult)
            if layer_out is not None:
                layer_out.append(x.clone())
        if rows is not None:
            x = x.index_select(0, rows)
        return mx.rms_norm_f32(x, self.final_norm, eps, False, self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.head).float()
