"""Sequence-mixer op layer: softmax attention with q/k norm, interleaved rotary positions and
an optional sink (score 0 or one learned score per head); latent attention's front end
(absorbed queries, rotate-half positions, compressed K / V pages) and per-head output gate;
short causal convolutions with carried tails; the gated delta rule and the gated linear
recurrence (forget-gate and state-space forms) with per-sequence fp32 state; the fp32-residual
norms, sums and activations around them.

Same device-strict dispatch as ``ops``: GPU tensors run the HIP kernels of
``ops/csrc/mixers`` (library ``_atta_mixers.so``, operators ``torch.ops.atta_mix.*``; built on
its own so a model that needs only these does not wait for the GEMM / GEMV library), CPU
tensors run ``mixers_reference``.  Activations are bf16 or fp32; the residual stream,
recurrent state, scores, norms, decays and gates are fp32 in both.
"""
from __future__ import annotations

import os
from pathlib import Path

import torch

from . import mixers_reference as mref

_LIB = Path(__file__).resolve().parent / "_atta_mixers.so"
_loaded = False
_load_error: str | None = None


class MixerKernelsUnavailable(RuntimeError):
    pass


def load_native(build_if_missing: bool = True) -> bool:
    global _loaded, _load_error
    if _loaded:
        return True
    try:
        from . import build

        want = build.mixer_source_hash()
        try:
            embeds = want.encode() in _LIB.read_bytes()
        except OSError:
            embeds = False
        if not embeds:
            if not build_if_missing:
                raise RuntimeError(f"{_LIB} missing or built from other sources")
            build.build_mixers()
        torch.ops.load_library(str(_LIB))
        _loaded, _load_error = True, None
    except Exception as e:  # pragma: no cover - depends on environment
        _load_error = f"{type(e).__name__}: {e}"
    return _loaded


def native_available() -> bool:
    return load_native(build_if_missing=os.environ.get("ATTA_NO_BUILD", "0") != "1")


def _native():
    if not native_available():
        raise MixerKernelsUnavailable(
            f"mixer HIP kernels not loadable from {_LIB}: {_load_error}. "
            "Run `python -m agentic_traffic_testing_amd.ops.build`.")
    return torch.ops.atta_mix


ATTN_TILE_TOKENS = 64     # query tokens per prefill attention tile (the block manager tiles by it)
DECODE_PART_TOKENS = 128  # keys per decode-attention partition
ATTENTION_MFMA = os.environ.get("ATTA_MIX_ATTENTION_MFMA", "1") != "0"
ACT_SILU, ACT_SIGMOID = 0, 1


def inv_freq(rot_dims: int, base: float, device) -> torch.Tensor:
    """fp32 table base^(-2i / rot_dims), i < rot_dims / 2 (computed in float64, rounded once)."""
    i = torch.arange(rot_dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / rot_dims).to(
        torch.float32).to(device)


def embed_pair(table, pair_table, ids, positions, seq_qstart, seq_slot, prev_token, mul_prev,
               mul_cur, buckets):
    if not table.is_cuda:
        return mref.embed_pair(table, pair_table, ids, positions, seq_qstart, seq_slot,
                               prev_token, mul_prev, mul_cur, buckets)
    out = torch.empty(ids.shape[0], table.shape[1], dtype=torch.float32, device=table.device)
    _native().embed_pair(out, table, pair_table, ids, positions, seq_qstart, seq_slot, prev_token,
                         mul_prev, mul_cur, buckets)
    return out


def rms_norm_f32(x, w, eps, one_plus=True, dtype=torch.bfloat16, out=None):
    if not x.is_cuda:
        return mref.rms_norm_f32(x, w, eps, one_plus, dtype)
    out = torch.empty(x.shape, dtype=dtype, device=x.device) if out is None else out
    _native().rms_norm_f32(out, x, w, eps, one_plus)
    return out


def rotary_table(positions, inv_freq_t):
    """fp32 [T, 2 n]: cos | sin of position * inv_freq[i]; one per step and rotary setting,
    shared by every layer that uses it."""
    if not positions.is_cuda:
        return mref.rotary_table(positions, inv_freq_t)
    out = torch.empty(positions.shape[0], 2 * inv_freq_t.shape[0], dtype=torch.float32,
                      device=positions.device)
    _native().rotary_table(out, positions, inv_freq_t)
    return out


def qk_norm_rope_cache(qx, kx, vx, q_norm, k_norm, eps, positions, slot_mapping, cos_sin,
                       k_cache, v_cache, heads, kv_heads, dim, vdim):
    """qx / kx / vx: row-strided [T, heads * dim] / [T, kv_heads * dim] / [T, kv_heads * vdim];
    cos_sin: ``rotary_table`` of the step's positions."""
    if not qx.is_cuda:
        return mref.qk_norm_rope_cache(qx, kx, vx, q_norm, k_norm, eps, positions, slot_mapping,
                                       cos_sin, k_cache, v_cache, heads, kv_heads, dim, vdim)
    q = torch.empty(qx.shape[0], heads, dim, dtype=qx.dtype, device=qx.device)
    _native().qk_norm_rope_cache(q, qx, kx, vx, q_norm, k_norm, eps, positions, slot_mapping,
                                 cos_sin, k_cache, v_cache)
    return q


def mfma_attention_ok(q, k_cache, v_cache) -> bool:
    """Can the matrix-core prefill kernel take these shapes (else the rows kernel does)?"""
    dim, vdim, bs = q.shape[2], v_cache.shape[2], k_cache.shape[2]
    return (q.dtype == torch.bfloat16 and dim % 16 == 0 and vdim % 32 == 0 and dim <= 256
            and vdim <= 256 and bs >= 8 and bs & (bs - 1) == 0 and ATTENTION_MFMA)


def sink_attention(q, k_cache, v_cache, block_tables, seq_kvlen, seq_qstart, tile_seq, tile_qoff,
                   scale, sink=True, num_decode=0, max_decode_kv=0, sink_values=None):
    """Causal attention of every portion's rows over its sequence's pages
    (k_cache [nb, G, BS, d], v_cache [nb, G, dv, BS]).  Sequences [0, num_decode) have one
    query row each and go through the partitioned decode kernel (``max_decode_kv``: their
    longest context, for the grid); ``tile_seq`` / ``tile_qoff`` hold one entry per
    ATTN_TILE_TOKENS query rows of every other portion (sequence index, row offset in it).
    ``sink_values``: fp32 [H], the sink's (unscaled) score per query head instead of 0."""
    if not q.is_cuda:
        return mref.sink_attention(q, k_cache, v_cache, block_tables, seq_kvlen, seq_qstart,
                                   scale, sink, sink_values)
    out = torch.empty(q.shape[0], q.shape[1], v_cache.shape[2], dtype=q.dtype, device=q.device)
    part = None
    if num_decode > 0:
        parts = max(1, -(-int(max_decode_kv) // DECODE_PART_TOKENS))
        part = torch.empty(num_decode, q.shape[1], parts, v_cache.shape[2] + 2,
                           dtype=torch.float32, device=q.device)
    if tile_seq.shape[0] > 0 or num_decode > 0:
        _native().sink_attention(out, q, k_cache, v_cache, block_tables, seq_kvlen, seq_qstart,
                                 tile_seq, tile_qoff, scale, sink, num_decode,
                                 max(1, int(max_decode_kv)), part,
                                 mfma_attention_ok(q, k_cache, v_cache), sink_values)
    return out


def short_conv_silu(x, w, conv_state, positions, seq_qstart, seq_slot, bias=None):
    """x: row-strided [T, C]; conv_state [slots, taps - 1, C] is advanced in place; ``bias``
    [C] is added before the SiLU."""
    if not x.is_cuda:
        return mref.short_conv_silu(x, w, conv_state, positions, seq_qstart, seq_slot, bias)
    out = torch.empty(x.shape[0], w.shape[0], dtype=x.dtype, device=x.device)
    if conv_state is None:  # one tap: nothing is carried
        conv_state = x.new_zeros(1, 0, w.shape[0])
    _native().short_conv_silu(out, x, w, conv_state, positions, seq_qstart, seq_slot, bias)
    return out


def gated_delta_rule(qkv, beta_logit, decay_logit, a_log, dt_bias, state, positions, seq_qstart,
                     seq_slot, heads, kv_heads, dim, vdim):
    if not qkv.is_cuda:
        return mref.gated_delta_rule(qkv, beta_logit, decay_logit, a_log, dt_bias, state,
                                     positions, seq_qstart, seq_slot, heads, kv_heads, dim, vdim)
    out = torch.empty(qkv.shape[0], heads, vdim, dtype=torch.float32, device=qkv.device)
    _native().gated_delta_rule(out, qkv, beta_logit, decay_logit, a_log, dt_bias, state, positions,
                               seq_qstart, seq_slot, heads, kv_heads, dim, vdim)
    return out


def gated_rms_norm(o, gate, w, eps, act="silu", dtype=torch.bfloat16):
    if not o.is_cuda:
        return mref.gated_rms_norm(o, gate, w, eps, act, dtype)
    T, H, dv = o.shape
    out = torch.empty(T, H * dv, dtype=dtype, device=o.device)
    _native().gated_rms_norm(out, o, gate, w, eps, ACT_SIGMOID if act == "sigmoid" else ACT_SILU)
    return out


def relu_sq(x):
    if not x.is_cuda:
        return mref.relu_sq(x)
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    _native().relu_sq(out, x)
    return out


def residual_add(x, a, sa=1.0, b=None, sb=1.0, c=None):
    if not x.is_cuda:
        return mref.residual_add(x, a, sa, b, sb, c)
    _native().residual_add(x, a, float(sa), b, float(sb), c)
    return x


def add_norm(x, a, sa, b, sb, c, w, eps, one_plus=True, dtype=torch.bfloat16):
    """Layer boundary fused: x (fp32, in place) += sa * a [+ sb * b] [+ c]; returns the RMS norm
    of the new x with weight ``w`` (1 + w when ``one_plus``) in ``dtype``."""
    if not x.is_cuda:
        mref.residual_add(x, a, sa, b, sb, c)
        return mref.rms_norm_f32(x, w, eps, one_plus, dtype)
    h = torch.empty(x.shape, dtype=dtype, device=x.device)
    _native().add_norm(h, x, a, float(sa), b, float(sb), c, w, eps, one_plus)
    return h


def embed_scale(table, ids, scale):
    """fp32 rows table[id] * scale."""
    if not table.is_cuda:
        return mref.embed_scale(table, ids, scale)
    out = torch.empty(ids.shape[0], table.shape[1], dtype=torch.float32, device=table.device)
    _native().embed_scale(out, table, ids, float(scale))
    return out


def rms_norm_rows(x, w, eps):
    """RMS norm with a plain weight over row-strided activation rows [T, N]."""
    if not x.is_cuda:
        return mref.rms_norm_rows(x, w, eps)
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    _native().rms_norm_rows(out, x, w, eps)
    return out


def xielu_bias(x, bias, ap, aq):
    """xIELU of x + bias (row-strided x [T, N]): z > 0: ap z^2 + z / 2, else
    (1/2 + aq)(exp(z) - 1 - z) + z / 2; ap, aq are the softplus of the layer's two numbers."""
    if not x.is_cuda:
        return mref.xielu_bias(x, bias, ap, aq)
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    _native().xielu_bias(out, x, bias, float(ap), float(aq))
    return out


def group_rms_norm(y, gate, w, n_groups, eps, dtype=torch.bfloat16):
    """y fp32 [T, N] (times silu(gate) first, when a gate [T, N] is given) RMS-normed in
    ``n_groups`` equal parts, times w ([N / n_groups] shared by the parts, or [N])."""
    if not y.is_cuda:
        return mref.group_rms_norm(y, gate, w, n_groups, eps, dtype)
    out = torch.empty(y.shape, dtype=dtype, device=y.device)
    _native().group_rms_norm(out, y, gate, w, n_groups, eps)
    return out


def head_gate(o, gate):
    """o [H, T, dv] (head-major) times sigmoid(gate [T, H]) -> [T, H * dv]."""
    if not o.is_cuda:
        return mref.head_gate(o, gate)
    H, T, dv = o.shape
    out = torch.empty(T, H * dv, dtype=o.dtype, device=o.device)
    _native().head_gate(out, o, gate)
    return out


def latent_rope_cache(q_lat, qx, kvx, c_norm, eps, slot_mapping, cos_sin, k_cache, v_cache):
    """Front end of latent attention over one shared compressed K / V head.  q_lat [H, T, rank]:
    queries times the key up-projection; qx [T, H, qdim + rot]: its last ``rot`` channels are
    rotated (rotate-half pairs, table ``cos_sin``); returns the absorbed queries
    [T, H, rank + rot].  kvx [T, rank + rot] (or None for a layer that reads another layer's
    pages): the first ``rank`` channels are RMS-normed with weight ``c_norm``, the rest rotated;
    [latent | rotated key] goes to k_cache [nb, 1, BS, rank + rot], the latent to the
    channel-major v_cache [nb, 1, rank, BS]."""
    if not qx.is_cuda:
        return mref.latent_rope_cache(q_lat, qx, kvx, c_norm, eps, slot_mapping, cos_sin, k_cache,
                                      v_cache)
    H, T, rank = q_lat.shape
    rot = k_cache.shape[3] - rank
    q = torch.empty(T, H, rank + rot, dtype=qx.dtype, device=qx.device)
    c_out = torch.empty(T if kvx is not None else 0, rank, dtype=qx.dtype, device=qx.device)
    _native().latent_rope_cache(q, q_lat, qx, kvx, c_norm, eps, slot_mapping, cos_sin, k_cache,
                                v_cache, c_out)
    return q


def forget_gate_scan(q, f, v, f_bias, lower, state, positions, seq_qstart, seq_slot, heads, dim,
                     vdim):
    """HGRN2 recurrence: per head S = diag(a) S + (1 - a) v^T, o = S^T silu(q) with
    a = lower + (1 - lower) sigmoid(f + f_bias).  q, f [T, heads * dim], v [T, heads * vdim]
    (row-strided); state fp32 [slots, heads, dim, vdim] advanced in place; returns fp32
    [T, heads, vdim]."""
    if not v.is_cuda:
        return mref.forget_gate_scan(q, f, v, f_bias, lower, state, positions, seq_qstart,
                                     seq_slot, heads, dim, vdim)
    out = torch.empty(v.shape[0], heads, vdim, dtype=torch.float32, device=v.device)
    _native().gated_linear_scan(out, state, q, f, v, None, f_bias, lower, None, positions,
                                seq_qstart, seq_slot, heads, heads, dim, vdim, 0)
    return out


def state_space_scan(x, B, C, dt, dt_bias, a_log, skip, state, positions, seq_qstart, seq_slot,
                     heads, groups, n_state, vdim):
    """Mamba-2 recurrence: dt = softplus(dt + dt_bias); per head S = exp(-exp(a_log) dt) S +
    dt B x^T, y = S^T C + skip x, B / C [T, groups * n_state] shared by the heads of a group.
    state fp32 [slots, heads, n_state, vdim] advanced in place; returns fp32 [T, heads, vdim]."""
    if not x.is_cuda:
        return mref.state_space_scan(x, B, C, dt, dt_bias, a_log, skip, state, positions,
                                     seq_qstart, seq_slot, heads, groups, n_state, vdim)
    out = torch.empty(x.shape[0], heads, vdim, dtype=torch.float32, device=x.device)
    _native().gated_linear_scan(out, state, C, B, x, dt, dt_bias, a_log, skip, positions,
                                seq_qstart, seq_slot, heads, groups, n_state, vdim, 1)
    return out
