"""Sequence-mixer op layer: softmax attention with q/k norm, interleaved rotary positions and
an optional sink (score 0 or one learned score per head); latent attention's front end
(absorbed queries, rotate-half positions, compressed K / V pages) and per-head output gate;
short causal convolutions with carried tails; the gated delta rule and the gated linear
recurrence (forget-gate and state-space forms) with per-sequence fp32 state; the fp32-residual
norms, sums and activations around them; hyper-connection streams, token shift, the minGRU
recurrence, element-wise gates, GELU, and routed clamped-GLU or SiLU-GLU experts (grouped matrix
products over rows sorted by expert; sigmoid or softmax routing, optionally with a choice
correction and group-limited choice; identity experts), the sandwich-norm layer boundary (layer
norm or RMS norm of a branch added to the fp32 residual, then the next norm), q / k norms over
a whole projection, and scaled, soft-capped logits.

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
ACT_SILU, ACT_SIGMOID, ACT_GELU_TANH = 0, 1, 2
_ACT_CODES = {"silu": ACT_SILU, "sigmoid": ACT_SIGMOID, "gelu_tanh": ACT_GELU_TANH}


def inv_freq(rot_dims: int, base: float, device) -> torch.Tensor:
    """fp32 table base^(-2i / rot_dims), i < rot_dims / 2 (computed in float64, rounded once)."""
    i = torch.arange(rot_dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / rot_dims).to(
        torch.float32).to(device)


def scaled_inv_freq(rot_dims: int, base: float, scaling, device) -> torch.Tensor:
    """``inv_freq`` with wavelength-dependent scaling ``(factor, low, high, original)``: a
    frequency whose wavelength 2 pi / f is shorter than original / high is kept, longer than
    original / low is divided by factor, between them blended linearly in original / wavelength.
    float64, rounded once to fp32."""
    i = torch.arange(rot_dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / rot_dims)
    if scaling is not None:
        factor, low, high, original = (float(v) for v in scaling)
        wave = 2.0 * torch.pi / f
        smooth = (original / wave - low) / (high - low) if high != low else torch.ones_like(f)
        mid = (1.0 - smooth) * f / factor + smooth * f
        f = torch.where(wave < original / high, f, torch.where(wave > original / low, f / factor,
                                                              mid))
    return f.to(torch.float32).to(device)


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
                       k_cache, v_cache, heads, kv_heads, dim, vdim, rotate_half_pairs=False,
                       norm_last=False, whole_norm=False):
    """qx / kx / vx: row-strided [T, heads * dim] / [T, kv_heads * dim] / [T, kv_heads * vdim];
    cos_sin: ``rotary_table`` of the step's positions.  ``q_norm`` / ``k_norm`` None: the norm
    has no weight; ``rotate_half_pairs``: channel i pairs with i + n_freq instead of
    (2i, 2i + 1); ``norm_last``: rotate first, then norm; ``whole_norm``: q (and k) are normed
    over the whole projection, all heads at once, with weights [heads * dim] ([kv_heads * dim]) -
    a one-wave-per-row kernel computes the two inverse root mean squares of every row first."""
    if not qx.is_cuda:
        return mref.qk_norm_rope_cache(qx, kx, vx, q_norm, k_norm, eps, positions, slot_mapping,
                                       cos_sin, k_cache, v_cache, heads, kv_heads, dim, vdim,
                                       rotate_half_pairs, norm_last, whole_norm)
    if whole_norm and norm_last:
        raise ValueError("a norm over the whole projection precedes the rotation")
    q = torch.empty(qx.shape[0], heads, dim, dtype=qx.dtype, device=qx.device)
    row_inv = None
    if whole_norm:
        row_inv = torch.empty(qx.shape[0], 2, dtype=torch.float32, device=qx.device)
        _native().proj_inv_rms(row_inv, qx, kx, eps)
    _native().qk_norm_rope_cache(q, qx, kx, vx, q_norm, k_norm, eps, positions, slot_mapping,
                                 cos_sin, k_cache, v_cache, rotate_half_pairs, norm_last, row_inv)
    return q


def mfma_attention_ok(q, k_cache, v_cache) -> bool:
    """Can the matrix-core prefill kernel take these shapes (else the rows kernel does)?"""
    dim, vdim, bs = q.shape[2], v_cache.shape[2], k_cache.shape[2]
    return (q.dtype == torch.bfloat16 and dim % 16 == 0 and vdim % 32 == 0 and dim <= 256
            and vdim <= 256 and bs >= 8 and bs & (bs - 1) == 0 and ATTENTION_MFMA)


def sink_attention(q, k_cache, v_cache, block_tables, seq_kvlen, seq_qstart, tile_seq, tile_qoff,
                   scale, sink=True, num_decode=0, max_decode_kv=0, sink_values=None, window=0):
    """Causal attention of every portion's rows over its sequence's pages
    (k_cache [nb, G, BS, d], v_cache [nb, G, dv, BS]).  Sequences [0, num_decode) have one
    query row each and go through the partitioned decode kernel (``max_decode_kv``: their
    longest context, for the grid); ``tile_seq`` / ``tile_qoff`` hold one entry per
    ATTN_TILE_TOKENS query rows of every other portion (sequence index, row offset in it).
    ``sink_values``: fp32 [H], the sink's (unscaled) score per query head instead of 0.
    ``window`` > 0: a row at position i sees keys j with 0 <= i - j < window (decode then runs
    only the partitions that overlap the window)."""
    window = int(window)
    if not q.is_cuda:
        return mref.sink_attention(q, k_cache, v_cache, block_tables, seq_kvlen, seq_qstart,
                                   scale, sink, sink_values, window)
    out = torch.empty(q.shape[0], q.shape[1], v_cache.shape[2], dtype=q.dtype, device=q.device)
    part = None
    if num_decode > 0:
        parts = max(1, -(-int(max_decode_kv) // DECODE_PART_TOKENS))
        if window > 0:   # the window touches at most this many partitions
            parts = min(parts, -(-window // DECODE_PART_TOKENS) + 1)
        part = torch.empty(num_decode, q.shape[1], parts, v_cache.shape[2] + 2,
                           dtype=torch.float32, device=q.device)
    if tile_seq.shape[0] > 0 or num_decode > 0:
        _native().sink_attention(out, q, k_cache, v_cache, block_tables, seq_kvlen, seq_qstart,
                                 tile_seq, tile_qoff, scale, sink, num_decode,
                                 max(1, int(max_decode_kv)), part,
                                 mfma_attention_ok(q, k_cache, v_cache), sink_values, window)
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


def embed_scale(table, ids, scale, copies=0):
    """fp32 rows table[id] * scale [T, W]; ``copies`` > 0: [T, copies, W], the row that many
    times (the streams of a multi-stream residual)."""
    if not table.is_cuda:
        return mref.embed_scale(table, ids, scale, copies)
    shape = (ids.shape[0], copies, table.shape[1]) if copies else (ids.shape[0], table.shape[1])
    out = torch.empty(shape, dtype=torch.float32, device=table.device)
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



def hyper_norm(xs, w_in, w, eps, dtype=torch.bfloat16):
    """xs fp32 [T, s, W] (the residual streams): RMS norm with weight ``w`` of
    u = sum_s w_in[s] xs[:, s] -> [T, W] of ``dtype``.  w_in fp32 [s]."""
    if not xs.is_cuda:
        return mref.hyper_norm(xs, w_in, w, eps, dtype)
    out = torch.empty(xs.shape[0], xs.shape[2], dtype=dtype, device=xs.device)
    _native().hyper_update_norm(out, xs, None, None, None, w_in, w, eps)
    return out


def hyper_update_norm(xs, y, mix, w_out, w_in_next, w_next, eps, dtype=torch.bfloat16):
    """Layer boundary of a multi-stream residual in one pass: every stream at once from the old
    ones, xs[:, t] = sum_s mix[s, t] xs[:, s] + w_out[t] y (fp32, in place), then (unless
    ``w_next`` is None) the next sub-layer's ``hyper_norm`` of the new streams."""
    if not xs.is_cuda:
        mref.hyper_update(xs, y, mix, w_out)
        return mref.hyper_norm(xs, w_in_next, w_next, eps, dtype) if w_next is not None else None
    out = (torch.empty(xs.shape[0], xs.shape[2], dtype=dtype, device=xs.device)
           if w_next is not None else None)
    _native().hyper_update_norm(out, xs, y, mix, w_out, w_in_next, w_next, eps)
    return out


def token_shift(n, mu, shift_state, positions, seq_qstart, seq_slot, dtype=torch.bfloat16):
    """h = n + (n_prev - n) * mu with n_prev the previous token's row of n (fp32 [T, W]); the
    row before a portion is ``shift_state[slot]`` (zeros before position 0), which then takes the
    portion's last row."""
    if not n.is_cuda:
        return mref.token_shift(n, mu, shift_state, positions, seq_qstart, seq_slot, dtype)
    out = torch.empty(n.shape, dtype=dtype, device=n.device)
    _native().token_shift(out, n, mu, shift_state, positions, seq_qstart, seq_slot)
    return out


def gate_mul(a, gate, act="sigmoid"):
    """a [T, N] times sigmoid / SiLU / tanh-form GELU of the gate [T, N]; both may be row-strided
    slices of a fused projection (a GLU is ``gate_mul(up, gate, act)``)."""
    code = _ACT_CODES[act]
    if not a.is_cuda:
        return mref.gate_mul(a, gate, code)
    out = torch.empty(a.shape, dtype=a.dtype, device=a.device)
    _native().gate_mul(out, a, gate, code)
    return out


def mingru_scan(z, x, g, state, positions, seq_qstart, seq_slot, dtype=torch.bfloat16):
    """minGRU over every portion: S = S + sigmoid(z) (c - S), c = x + 1/2 (x >= 0) or sigmoid(x),
    output S * silu(g) in ``dtype``.  z, x, g row-strided [T, C]; state fp32 [slots, ..., C]
    advanced in place (zero before position 0)."""
    if not z.is_cuda:
        return mref.mingru_scan(z, x, g, state, positions, seq_qstart, seq_slot, dtype)
    out = torch.empty(z.shape, dtype=dtype, device=z.device)
    _native().mingru_scan(out, state, z, x, g, positions, seq_qstart, seq_slot)
    return out


def gelu(x, tanh_form=False):
    if not x.is_cuda:
        return mref.gelu(x, tanh_form)
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    _native().gelu(out, x, bool(tanh_form))
    return out


MOE_TILE_ROWS = 64         # rows of one expert per grouped-product tile ...
MOE_BIG_TILE_ROWS = 128    # ... and for prefill-sized steps on the matrix-core kernel
MOE_BIG_TILE_PAIRS = 1024  # (row, choice) pairs from which the large tiles are used
# floating-point operations of a step's expert products (6 pairs ff W) from which the library
# path runs them (0: never): below it the grouped kernels finish before a host round trip and
# three launches per expert would
MOE_LIBRARY_FLOPS = float(os.environ.get("ATTA_MIX_MOE_LIBRARY_FLOPS", "8e11"))


def _pair_sum(y, T, k, dtype=None):
    """y [T * k, W] (a row's k summands adjacent; ``dtype`` or fp32) -> their fp32 sum per row in
    ``dtype`` (y's own by default)."""
    dtype = dtype or y.dtype
    if k == 1 and y.dtype == dtype:
        return y
    out = torch.empty(T, y.shape[1], dtype=dtype, device=y.device)
    _native().pair_sum(out, y.view(T, k, y.shape[1]))
    return out


def clamped_glu(gu, wts, limit, alpha=1.702):
    """[gate | up] products [R, 2 ff] with the rows' router weights [R] -> activation [R, ff]."""
    if not gu.is_cuda:
        return mref.clamped_glu(gu, wts, limit, alpha)
    out = torch.empty(gu.shape[0], gu.shape[1] // 2, dtype=gu.dtype, device=gu.device)
    _native().clamped_glu(out, gu, wts, float(limit), float(alpha))
    return out


def _moe_combine(y, idx, wts, h, addend, E, split):
    """out[t] = sum_j wts[t, j] * (y[t, j] summed over its ``split`` partial rows, or h[t] for an
    identity expert idx[t, j] >= E) (+ addend[t]), in fp32, stored in h's dtype."""
    out = torch.empty_like(h)
    _native().moe_combine(out, y, idx, wts, h, addend, E, split)
    return out


def _moe_experts_library(h, idx, wts, w_gu, w_down, limit, alpha, silu_glu=False, addend=None):
    """Prefill-sized steps: rows sorted by expert, then per expert one library product with the
    stacked [gate; up] matrix, the activation kernel and one library product with the down
    matrix.  The per-expert row counts come to the host (one synchronisation per call), so this
    path is not taken while a graph is being recorded."""
    T, W = h.shape
    k = idx.shape[1]
    E, ff = w_gu.shape[0], w_gu.shape[1] // 2
    flat = idx.flatten().long()
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=E).tolist()
    xs = h.index_select(0, torch.div(order, k, rounding_mode="floor"))
    ws = wts.flatten().index_select(0, order)
    ys = torch.empty(T * k, W, dtype=h.dtype, device=h.device)
    off = 0
    for e, c in enumerate(counts[:E]):     # indices >= E are identity experts: no product
        if c:
            gu = torch.nn.functional.linear(xs[off:off + c], w_gu[e])
            a = (gate_mul(gu[:, ff:], gu[:, :ff], "silu") if silu_glu else
                 clamped_glu(gu, ws[off:off + c], limit, alpha))
            torch.mm(a, w_down[e].t(), out=ys[off:off + c])
            off += c
    y = torch.empty_like(ys)
    y.index_copy_(0, order, ys)
    if silu_glu:
        return _moe_combine(y, idx, wts, h, addend, E, 1)
    return _pair_sum(y, T, k)


def moe_route(logits, top, score="sigmoid", correction=None, groups=1, keep=1, renorm=False):
    """fp32 router logits [T, E] -> (expert index int32 [T, top], score fp32 [T, top]) of every
    row's ``top`` largest scores (ties: lowest index).  ``score``: "sigmoid", or "softmax" over
    the row.  ``correction`` fp32 [E] is added to the scores for the choice only (the returned
    weights are the plain scores).  ``groups`` > 1: the experts form that many equal runs of
    neighbours, a group's score is its largest choice score, and only experts of the ``keep``
    best groups can be chosen.  ``renorm``: the chosen scores are divided by their sum + 1e-20."""
    E = logits.shape[1]
    if groups < 1 or E % groups or not 1 <= keep <= groups or top > keep * (E // groups):
        raise ValueError("moe_route: groups must split the experts evenly and hold `top` of them")
    if not logits.is_cuda:
        return mref.moe_route(logits, top, score == "softmax", correction, groups, keep, renorm)
    T = logits.shape[0]
    idx = torch.empty(T, top, dtype=torch.int32, device=logits.device)
    wts = torch.empty(T, top, dtype=torch.float32, device=logits.device)
    _native().moe_route(idx, wts, logits, score == "softmax", correction, groups, keep, renorm)
    return idx, wts


def moe_experts(h, idx, wts, w_gu, w_down, limit=0.0, alpha=1.702, glu="clamped", addend=None):
    """Routed GLU experts over a row's chosen (e, w) = (idx[t, j], wts[t, j]); w_gu [E, 2 ff, W]
    stacks every expert's gate rows on its up rows; w_down [E, W, ff].

    ``glu`` "clamped": out[t] = sum_j W_down[e] act(W_gate[e] (w h_t), W_up[e] (w h_t)) - the
    weight scales the expert's INPUT - with act(g, u) = g' sigmoid(alpha g') (u' + 1),
    g' = min(g, limit), u' = clamp(u, -limit, limit).
    ``glu`` "silu": out[t] = sum_j w expert_e(h_t) (+ ``addend``[t], e.g. a shared expert) - the
    weight scales the expert's OUTPUT, in fp32 - with expert_e(x) = W_down[e] (silu(W_gate[e] x) *
    (W_up[e] x)); an index e >= E is an identity expert, expert_e(x) = x, without weights.

    On the GPU: one planning kernel sorts the (row, choice) pairs by expert into tiles of
    MOE_TILE_ROWS (or MOE_BIG_TILE_ROWS), then two grouped matrix products (gate | up with the
    activation in the epilogue; down) run over the tiles - no host synchronisation, so the step
    can be captured in a graph.  Steps whose expert products reach MOE_LIBRARY_FLOPS run library
    products per expert instead (outside a capture)."""
    silu_glu = glu == "silu"
    if not silu_glu and (glu != "clamped" or addend is not None):
        raise ValueError("moe_experts: glu is 'clamped' or 'silu'; an addend goes with 'silu'")
    if not h.is_cuda:
        return mref.moe_experts(h, idx, wts, w_gu, w_down, limit, alpha, silu_glu, addend)
    T, W = h.shape
    E, ff = w_gu.shape[0], w_gu.shape[1] // 2
    k = idx.shape[1]
    P = T * k
    if 0 < MOE_LIBRARY_FLOPS <= 6.0 * P * ff * W and not torch.cuda.is_current_stream_capturing():
        return _moe_experts_library(h, idx, wts, w_gu, w_down, limit, alpha, silu_glu, addend)
    big = (h.dtype == torch.bfloat16 and W % 8 == 0 and ff % 8 == 0 and P >= MOE_BIG_TILE_PAIRS)
    rows = MOE_BIG_TILE_ROWS if big else MOE_TILE_ROWS
    max_tiles = P // rows + min(E, P)
    dev = h.device
    # few tiles (a decode step): the down product's long K range is cut over `split` workgroups
    # per tile so the launch fills the chip; the fp32 partials are summed with the row's choices
    split = 1
    groups = max_tiles * -(-W // MOE_TILE_ROWS)
    if h.dtype == torch.bfloat16 and W % 8 == 0 and ff % 8 == 0 and not big and groups < 1024:
        split = max(1, min(8, 2048 // groups, ff // 256))
    plan = torch.empty(2 + 3 * max_tiles + P, dtype=torch.int32, device=dev)
    act = torch.empty(P, ff, dtype=h.dtype, device=dev)
    y = torch.empty(P * split, W, dtype=torch.float32 if split > 1 else h.dtype, device=dev)
    _native().moe_experts(y, act, plan, h, idx, wts, w_gu[:, :ff], w_gu[:, ff:], w_down,
                          float(limit), float(alpha), max_tiles, rows, split, int(silu_glu))
    if silu_glu:
        return _moe_combine(y, idx, wts, h, addend, E, split)
    return _pair_sum(y, T, k * split, h.dtype)


def norm_add_norm(x, y, w_post, w_next, eps, kind="layer", dtype=torch.bfloat16):
    """Layer boundary of a sandwich-norm residual in one pass: x (fp32 [T, W], in place) +=
    norm(y) * w_post (y None: nothing is added), then returns norm(x) * w_next in ``dtype``
    (None when ``w_next`` is None).  ``kind`` "layer": (v - mean) / sqrt(var + eps) with var the
    mean squared deviation; "rms": v / sqrt(mean(v^2) + eps).  Sums and statistics in fp32."""
    if kind not in ("layer", "rms"):
        raise ValueError(kind)
    if not x.is_cuda:
        return mref.norm_add_norm(x, y, w_post, w_next, eps, kind == "layer", dtype)
    h = torch.empty(x.shape, dtype=dtype, device=x.device) if w_next is not None else None
    _native().norm_add_norm(h, x, y, w_post, w_next, eps, kind == "layer")
    return h


def scale_softcap(logits, scale=1.0, cap=0.0):
    """fp32 cap * tanh(logits * scale / cap) of activation-dtype logits (cap 0: logits * scale)."""
    if not logits.is_cuda:
        return mref.scale_softcap(logits, float(scale), float(cap))
    out = torch.empty(logits.shape, dtype=torch.float32, device=logits.device)
    _native().scale_softcap(out, logits, float(scale), float(cap))
    return out
