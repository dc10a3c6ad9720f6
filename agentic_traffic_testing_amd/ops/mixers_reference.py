"""Plain-PyTorch definitions of the sequence-mixer ops (``ops/mixers.py``): the numerics
reference the GPU tests compare ``csrc/mixers/*.hip`` against, and the implementation the
engine runs on CPU tensors (the CPU test tier).  Values are rounded to the activation dtype
where the kernels round them; everything the kernels keep in fp32 is fp32 here.

Batch metadata (all int32): ``positions`` [T] position of each row in its sequence,
``seq_qstart`` [S+1] first row of each sequence's portion, ``seq_slot`` [S] state slot of each
sequence (-1: padding, skipped), ``slot_mapping`` [T] KV-cache token slot of each row (-1:
skipped), ``block_tables`` [S, W], ``seq_kvlen`` [S].  A portion whose first position is 0
starts from the zero state whatever its slot holds.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def _portions(seq_qstart, seq_slot):
    qs = seq_qstart.tolist()
    for s, slot in enumerate(seq_slot.tolist()):
        if slot >= 0 and qs[s + 1] > qs[s]:
            yield s, slot, qs[s], qs[s + 1]


def embed_pair(table, pair_table, ids, positions, seq_qstart, seq_slot, prev_token, mul_prev,
               mul_cur, buckets):
    """fp32 rows table[id] + pair_table[(prev * mul_prev + id * mul_cur) % buckets] (row
    ``buckets`` at position 0).  The token before a portion's first row comes from
    ``prev_token[slot]``, which is then set to the portion's last token."""
    T = ids.shape[0]
    out = torch.zeros(T, table.shape[1], dtype=torch.float32, device=table.device)
    idl = ids.long()
    for s, slot, a, b in _portions(seq_qstart, seq_slot):
        cur = idl[a:b]
        prev = torch.cat([prev_token[slot:slot + 1].long(), cur[:-1]])
        row = (prev * mul_prev + cur * mul_cur) % buckets
        row = torch.where(positions[a:b].long() == 0, torch.full_like(row, buckets), row)
        out[a:b] = table[cur].float() + pair_table[row].float()
        prev_token[slot] = int(cur[-1])
    return out


def rms_norm_f32(x, w, eps, one_plus, dtype):
    """fp32 rows in, rows of ``dtype`` out: x / sqrt(mean(x^2) + eps) * (w or 1 + w)."""
    xf = x.float()
    g = w.float() + 1.0 if one_plus else w.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * g).to(dtype)


def rotary_table(positions, inv_freq):
    """fp32 [T, 2 n]: cos | sin of position * inv_freq[i] (fp32 angles)."""
    ang = positions.float()[:, None] * inv_freq.float()[None, :]
    return torch.cat([torch.cos(ang), torch.sin(ang)], 1)


def rotate_interleaved(x, cos_sin):
    """x [T, H, d] fp32: pairs (2i, 2i+1) for i < n rotate by the angles of cos_sin [T, 2 n]."""
    n = cos_sin.shape[1] // 2
    T = x.shape[0]
    c, s = cos_sin[:T, None, :n], cos_sin[:T, None, n:]
    out = x.clone()
    u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
    out[..., 0:2 * n:2] = u * c - v * s
    out[..., 1:2 * n:2] = v * c + u * s
    return out


def qk_norm_rope_cache(qx, kx, vx, q_norm, k_norm, eps, positions, slot_mapping, cos_sin,
                       k_cache, v_cache, heads, kv_heads, dim, vdim, rotate_half_pairs=False,
                       norm_last=False, whole_norm=False):
    """Per-head RMS norm (plain weight, or none when ``q_norm`` / ``k_norm`` is None; with
    ``whole_norm`` one norm over all heads of the projection with weights [heads * dim]) and rotary
    positions on q [T, heads * dim] and k [T, kv_heads * dim] (row-strided views); returns
    q [T, heads, dim] and writes k and v [T, kv_heads * vdim] into the paged caches
    k_cache [nb, kv_heads, BS, dim], v_cache [nb, kv_heads, vdim, BS] (channel-major pages).
    ``rotate_half_pairs``: channel i pairs with i + n instead of (2i, 2i + 1); ``norm_last``: the
    norm follows the rotation instead of preceding it."""
    T = qx.shape[0]
    dt = qx.dtype
    q = qx.reshape(T, heads, dim).float()
    k = kx.reshape(T, kv_heads, dim).float()
    v = vx.reshape(T, kv_heads, vdim)

    def nrm(x, w):
        if whole_norm:
            y = x * torch.rsqrt(x.pow(2).mean((-2, -1), keepdim=True) + eps)
            return y * w.float().view(x.shape[1], x.shape[2]) if w is not None else y
        y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
        return y * w.float() if w is not None else y

    rot = rotate_half if rotate_half_pairs else rotate_interleaved
    if norm_last:
        q, k = nrm(rot(q, cos_sin), q_norm).to(dt), nrm(rot(k, cos_sin), k_norm).to(dt)
    else:
        q, k = rot(nrm(q, q_norm), cos_sin).to(dt), rot(nrm(k, k_norm), cos_sin).to(dt)
    bs = k_cache.shape[2]
    sm = slot_mapping.long()
    ok = sm >= 0
    if bool(ok.any()):
        s = sm[ok]
        k_cache[s // bs, :, s % bs, :] = k[ok]
        v_cache[s // bs, :, :, s % bs] = v[ok].to(v_cache.dtype)
    return q


def sink_attention(q, k_cache, v_cache, block_tables, seq_kvlen, seq_qstart, scale, sink,
                   sink_values=None, window=0):
    """Causal paged attention of every portion's rows over its sequence's cached keys; fp32
    scores and weights; ``sink`` adds exp(s - max) to each denominator, s = 0 or the head's
    entry of ``sink_values`` [H]; ``window`` > 0: a row at position i sees keys j with
    0 <= i - j < window.  q [T, H, d] -> [T, H, dv]."""
    T, H, _ = q.shape
    G, bs, dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[2]
    out = torch.zeros(T, H, dv, dtype=q.dtype, device=q.device)
    qs = seq_qstart.tolist()
    for s, kvlen in enumerate(seq_kvlen.tolist()):
        a, b = qs[s], qs[s + 1]
        if kvlen <= 0 or b <= a:
            continue
        nblk = (kvlen + bs - 1) // bs
        pages = block_tables[s, :nblk].long()
        k = k_cache[pages].permute(1, 0, 2, 3).reshape(G, nblk * bs, -1)[:, :kvlen].float()
        v = v_cache[pages].permute(1, 0, 3, 2).reshape(G, nblk * bs, dv)[:, :kvlen].float()
        k = k.repeat_interleave(H // G, 0)
        v = v.repeat_interleave(H // G, 0)
        n = b - a
        sc = torch.einsum("qhd,hkd->hqk", q[a:b].float(), k) * scale
        qpos = torch.arange(kvlen - n, kvlen, device=q.device)
        kpos = torch.arange(kvlen, device=q.device)
        mask = kpos[None, :] > qpos[:, None]
        if window > 0:
            mask = mask | (kpos[None, :] <= qpos[:, None] - window)
        sc = sc.masked_fill(mask[None], float("-inf"))
        m = sc.amax(-1, keepdim=True)
        if sink:
            sv = (sink_values.float().view(H, 1, 1) if sink_values is not None
                  else torch.zeros(H, 1, 1, device=q.device))
            m = torch.maximum(m, sv)
        e = torch.exp(sc - m)
        den = e.sum(-1, keepdim=True)
        if sink:
            den = den + torch.exp(sv - m)
        out[a:b] = torch.einsum("hqk,hkd->qhd", e / den, v).to(q.dtype)
    return out


def short_conv_silu(x, w, conv_state, positions, seq_qstart, seq_slot, bias=None):
    """Causal per-channel convolution over time (w [C, taps], last tap = current row) of
    x [T, C] (a row-strided view) followed by SiLU; rows before a portion come from
    conv_state [slots, taps - 1, C] (zeros before position 0), which is then advanced."""
    T = x.shape[0]
    C, taps = w.shape
    dt = x.dtype
    out = torch.zeros(T, C, dtype=dt, device=x.device)
    wf = w.float()
    for s, slot, a, b in _portions(seq_qstart, seq_slot):
        tail = (conv_state[slot].float() if taps > 1 and conv_state is not None
                else torch.zeros(0, C, device=x.device))
        if int(positions[a]) == 0:
            tail = torch.zeros_like(tail)
        full = torch.cat([tail, x[a:b].float()], 0)          # [taps - 1 + n, C]
        acc = torch.zeros(b - a, C, dtype=torch.float32, device=x.device)
        if bias is not None:
            acc += bias.float()
        for j in range(taps):
            acc += full[j:j + b - a] * wf[:, j]
        out[a:b] = (acc / (1.0 + torch.exp(-acc))).to(dt)
        if taps > 1:
            conv_state[slot] = full[-(taps - 1):].to(conv_state.dtype)
    return out


def gated_delta_rule(qkv, beta_logit, decay_logit, a_log, dt_bias, state, positions, seq_qstart,
                     seq_slot, heads, kv_heads, dim, vdim):
    """qkv [T, 2 * kv_heads * dim + heads * vdim] (after convolution and SiLU); beta_logit
    [T, heads]; decay_logit [T, heads] or [T, heads * dim]; state fp32 [slots, heads, dim, vdim].
    Per head: unit-length q (times dim^-1/2) and k, beta = sigmoid, decay =
    exp(-exp(a_log) * softplus(logit + dt_bias)); S = decay * S; u = beta (v - S^T k);
    S += k u^T; o = S^T q.  Returns o fp32 [T, heads, vdim]; all of it in fp32."""
    T = qkv.shape[0]
    H, G = heads, kv_heads
    rep = H // G
    q = qkv[:, :G * dim].reshape(T, G, dim).float()
    k = qkv[:, G * dim:2 * G * dim].reshape(T, G, dim).float()
    v = qkv[:, 2 * G * dim:].reshape(T, H, vdim).float()
    q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    q = q.repeat_interleave(rep, 1)
    k = k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(beta_logit.float())
    per_channel = decay_logit.shape[1] == H * dim
    z = decay_logit.float() + dt_bias.float()
    rate = torch.exp(a_log.float())
    if per_channel:
        decay = torch.exp(-rate[None, :, None] * F.softplus(z.view(T, H, dim)))
    else:
        decay = torch.exp(-rate[None, :] * F.softplus(z))[:, :, None].expand(T, H, dim)
    out = torch.zeros(T, H, vdim, dtype=torch.float32, device=qkv.device)
    for s, slot, a, b in _portions(seq_qstart, seq_slot):
        S = state[slot].clone()
        if int(positions[a]) == 0:
            S.zero_()
        for t in range(a, b):
            S = S * decay[t][:, :, None]
            u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
            S = S + k[t][:, :, None] * u[:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[slot] = S
    return out


def gated_rms_norm(o, gate, w, eps, act, dtype):
    """o fp32 [T, H, dv] / rms over dv * w [dv] * act(gate [T, H * dv]) -> [T, H * dv]."""
    T, H, dv = o.shape
    g = gate.float().view(T, H, dv)
    g = torch.sigmoid(g) if act == "sigmoid" else g * torch.sigmoid(g)
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * w.float() * g
    return y.to(dtype).view(T, H * dv)


def relu_sq(x):
    r = torch.relu(x.float())
    return (r * r).to(x.dtype)


def residual_add(x, a, sa, b=None, sb=1.0, c=None):
    """x (fp32, in place) += sa * a [+ sb * b] [+ c]."""
    y = a.float() * sa
    if b is not None:
        y = y + b.float() * sb
    if c is not None:
        y = y + c.float()
    x += y
    return x


def embed_scale(table, ids, scale, copies=0):
    x = table[ids.long()].float() * scale
    return x.unsqueeze(1).repeat(1, copies, 1) if copies else x


def rms_norm_rows(x, w, eps):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(x.dtype)


def xielu_bias(x, bias, ap, aq):
    z = x.float()
    if bias is not None:
        z = z + bias.float()
    pos = ap * z * z + 0.5 * z
    neg = (0.5 + aq) * (torch.expm1(z.clamp_max(0.0)) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg).to(x.dtype)


def group_rms_norm(y, gate, w, n_groups, eps, dtype):
    T, N = y.shape
    u = y.float()
    if gate is not None:
        g = gate.float()
        u = u * (g * torch.sigmoid(g))
    u = u.view(T, n_groups, N // n_groups)
    u = u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps)
    wf = w.float().view(n_groups, -1) if w.numel() == N else w.float()
    return (u * wf).to(dtype).view(T, N)


def head_gate(o, gate):
    H, T, dv = o.shape
    g = torch.sigmoid(gate.float())                       # [T, H]
    return (o.float().permute(1, 0, 2) * g[:, :, None]).to(o.dtype).reshape(T, H * dv)


def rotate_half(x, cos_sin):
    """x [T, ..., r] fp32: channel i pairs with i + n over the first 2 n channels."""
    n = cos_sin.shape[1] // 2
    T = x.shape[0]
    shape = [T] + [1] * (x.dim() - 2) + [n]
    c, s = cos_sin[:T, :n].view(shape), cos_sin[:T, n:].view(shape)
    u, v = x[..., :n], x[..., n:2 * n]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * n:]], -1)


def latent_rope_cache(q_lat, qx, kvx, c_norm, eps, slot_mapping, cos_sin, k_cache, v_cache):
    H, T, rank = q_lat.shape
    rot = k_cache.shape[3] - rank
    dt = qx.dtype
    qr = rotate_half(qx[..., qx.shape[2] - rot:].float(), cos_sin).to(dt)
    q = torch.cat([q_lat.permute(1, 0, 2), qr], -1).contiguous()
    if kvx is not None:
        kv = kvx.float()
        c = kv[:, :rank]
        c = (c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * c_norm.float()).to(dt)
        kr = rotate_half(kv[:, rank:], cos_sin).to(dt)
        bs = k_cache.shape[2]
        sm = slot_mapping.long()
        ok = sm >= 0
        if bool(ok.any()):
            s = sm[ok]
            k_cache[s // bs, 0, s % bs, :] = torch.cat([c, kr], -1)[ok]
            v_cache[s // bs, 0, :, s % bs] = c[ok]
    return q


def forget_gate_scan(q, f, v, f_bias, lower, state, positions, seq_qstart, seq_slot, heads, dim,
                     vdim):
    T = v.shape[0]
    lo = lower.float()
    a = (lo + (1.0 - lo) * torch.sigmoid(f.float() + f_bias.float())).view(T, heads, dim)
    qq = q.float()
    qq = (qq * torch.sigmoid(qq)).view(T, heads, dim)
    vv = v.float().reshape(T, heads, vdim)
    out = torch.zeros(T, heads, vdim, dtype=torch.float32, device=v.device)
    for s, slot, b0, b1 in _portions(seq_qstart, seq_slot):
        S = state[slot].clone()
        if int(positions[b0]) == 0:
            S.zero_()
        for t in range(b0, b1):
            S = a[t][:, :, None] * S + (1.0 - a[t])[:, :, None] * vv[t][:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, qq[t])
        state[slot] = S
    return out


def state_space_scan(x, B, C, dt, dt_bias, a_log, skip, state, positions, seq_qstart, seq_slot,
                     heads, groups, n_state, vdim):
    T = x.shape[0]
    rep = heads // groups
    xx = x.float().reshape(T, heads, vdim)
    Bf = B.float().reshape(T, groups, n_state).repeat_interleave(rep, 1)
    Cf = C.float().reshape(T, groups, n_state).repeat_interleave(rep, 1)
    d = F.softplus(dt.float() + dt_bias.float())                       # [T, H]
    dec = torch.exp(-torch.exp(a_log.float())[None] * d)
    out = torch.zeros(T, heads, vdim, dtype=torch.float32, device=x.device)
    for s, slot, b0, b1 in _portions(seq_qstart, seq_slot):
        S = state[slot].clone()
        if int(positions[b0]) == 0:
            S.zero_()
        for t in range(b0, b1):
            S = dec[t][:, None, None] * S + (d[t][:, None] * Bf[t])[:, :, None] * xx[t][:, None, :]
            out[t] = torch.einsum("hnv,hn->hv", S, Cf[t]) + skip.float()[:, None] * xx[t]
        state[slot] = S
    return out


# ---- hyper-connections, token shift, minGRU, gates, GELU, expert routing -----------------------

def hyper_norm(xs, w_in, w, eps, dtype):
    """xs fp32 [T, s, W] residual streams: RMS norm (weight w) of u = sum_s w_in[s] xs[:, s]."""
    u = (xs.float() * w_in.float()[None, :, None]).sum(1)
    return (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(dtype)


def hyper_update(xs, y, mix, w_out):
    """All streams at once from the old ones: xs[:, t] = sum_s mix[s, t] xs[:, s] + w_out[t] y."""
    new = torch.einsum("tsw,sr->trw", xs.float(), mix.float()) + \
        w_out.float()[None, :, None] * y.float()[:, None, :]
    xs.copy_(new)
    return xs


def token_shift(n, mu, shift_state, positions, seq_qstart, seq_slot, dtype):
    """h = n + (n_prev - n) * mu per channel, n_prev the previous token's row of n (zeros before
    position 0, ``shift_state[slot]`` before a later portion's first row); the portion's last row
    of n becomes the new ``shift_state[slot]``.  n fp32 [T, W] -> [T, W] of ``dtype``."""
    out = torch.zeros(n.shape, dtype=dtype, device=n.device)
    nf = n.float()
    for s, slot, a, b in _portions(seq_qstart, seq_slot):
        first = shift_state[slot].float().clone()
        if int(positions[a]) == 0:
            first.zero_()
        prev = torch.cat([first[None], nf[a:b - 1]], 0)
        out[a:b] = (nf[a:b] + (prev - nf[a:b]) * mu.float()).to(dtype)
        shift_state[slot] = nf[b - 1]
    return out


def gate_mul(a, gate, act):
    """a [T, N] times sigmoid (act 1), SiLU (act 0) or tanh-form GELU (act 2) of gate [T, N]
    (both row-strided)."""
    g = gate.float()
    if act == 2:
        g = 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g * g * g)))
    else:
        g = torch.sigmoid(g) if act == 1 else g * torch.sigmoid(g)
    return (a.float() * g).to(a.dtype)


def mingru_scan(z, x, g, state, positions, seq_qstart, seq_slot, dtype):
    """minGRU: gate sigmoid(z), candidate x + 1/2 (x >= 0) or sigmoid(x) (x < 0),
    S = (1 - gate) S + gate * candidate per channel, output S * silu(g).  z, x, g [T, C]
    (row-strided); state fp32 [slots, C] advanced in place; all of it in fp32."""
    T, C = z.shape
    gate = torch.sigmoid(z.float())
    xf = x.float()
    cand = torch.where(xf >= 0, xf + 0.5, torch.sigmoid(xf))
    gf = g.float()
    og = gf * torch.sigmoid(gf)
    out = torch.zeros(T, C, dtype=dtype, device=z.device)
    st = state.view(state.shape[0], C)
    for s, slot, a, b in _portions(seq_qstart, seq_slot):
        S = st[slot].clone()
        if int(positions[a]) == 0:
            S.zero_()
        for t in range(a, b):
            S = S + gate[t] * (cand[t] - S)
            out[t] = (S * og[t]).to(dtype)
        st[slot] = S
    return out


def gelu(x, tanh_form=False):
    return F.gelu(x.float(), approximate="tanh" if tanh_form else "none").to(x.dtype)


def moe_route(logits, top, softmax=False, correction=None, groups=1, keep=1, renorm=False):
    """Scores (sigmoid, or softmax over the row) of fp32 router logits [T, E]; the ``top`` largest
    per row (ties: lowest index) -> (int32 [T, top], fp32 [T, top]).  ``correction`` [E] is added
    to the scores for the choice only; with ``groups`` > 1 only experts of the ``keep`` groups (equal
    runs of neighbours) with the largest best choice score can be chosen; ``renorm``: the chosen
    scores are divided by their sum + 1e-20."""
    z = logits.float()
    s = torch.softmax(z, 1) if softmax else torch.sigmoid(z)
    c = s + correction.float() if correction is not None else s.clone()
    T, E = s.shape
    if groups > 1:
        best = c.view(T, groups, E // groups).amax(2)
        kept = torch.argsort(best, dim=1, descending=True, stable=True)[:, :keep]
        allow = torch.zeros(T, groups, dtype=torch.bool, device=s.device)
        allow.scatter_(1, kept, True)
        c = c.masked_fill(~allow.repeat_interleave(E // groups, 1), float("-inf"))
    order = torch.argsort(c, dim=1, descending=True, stable=True)[:, :top]
    w = torch.gather(s, 1, order)
    if renorm:
        w = w / (w.sum(1, keepdim=True) + 1e-20)
    return order.to(torch.int32), w


def moe_experts(h, idx, wts, w_gu, w_down, limit, alpha, silu_glu=False, addend=None):
    """``silu_glu``: see ``moe_experts_silu``.  Otherwise:
    sum over a row's chosen experts of W_down act(W_gate (w h), W_up (w h)) with
    act(g, u) = g' sigmoid(alpha g') (u' + 1), g' = min(g, limit), u' = clamp(u, -limit, limit).
    h [T, W]; idx / wts [T, k]; w_gu [E, 2 ff, W] (gate rows, then up rows); w_down [E, W, ff].
    fp32 accumulation, the activation rounded to h's dtype between the two products like the
    kernels do."""
    if silu_glu:
        return moe_experts_silu(h, idx, wts, w_gu, w_down, addend)
    T, W = h.shape
    out = torch.zeros(T, W, dtype=torch.float32, device=h.device)
    hf = h.float()
    for j in range(idx.shape[1]):
        for e in torch.unique(idx[:, j]).tolist():
            rows = (idx[:, j] == e).nonzero().flatten()
            a = clamped_glu(hf[rows] @ w_gu[e].float().T, wts[rows, j], limit, alpha).to(h.dtype)
            out[rows] += (a.float() @ w_down[e].float().T).to(h.dtype).float()
    return out.to(h.dtype)


def moe_experts_silu(h, idx, wts, w_gu, w_down, addend=None):
    """out[t] = sum_j w[t, j] expert_{idx[t, j]}(h_t) (+ addend[t]) with
    expert_e(x) = W_down[e] (silu(W_gate[e] x) * (W_up[e] x)) for e < E and expert_e(x) = x for the
    identity experts e >= E.  The weights multiply the experts' outputs in fp32; the activation
    and each expert's output are rounded to h's dtype like the kernels do."""
    T, W = h.shape
    E, ff = w_gu.shape[0], w_gu.shape[1] // 2
    out = torch.zeros(T, W, dtype=torch.float32, device=h.device)
    hf = h.float()
    for j in range(idx.shape[1]):
        for e in torch.unique(idx[:, j]).tolist():
            rows = (idx[:, j] == e).nonzero().flatten()
            w = wts[rows, j].float()[:, None]
            if e >= E:
                out[rows] += w * hf[rows]
                continue
            gu = hf[rows] @ w_gu[e].float().T
            a = (gu[:, :ff] * torch.sigmoid(gu[:, :ff]) * gu[:, ff:]).to(h.dtype)
            out[rows] += w * (a.float() @ w_down[e].float().T).to(h.dtype).float()
    if addend is not None:
        out += addend.float()
    return out.to(h.dtype)


def norm_add_norm(x, y, w_post, w_next, eps, layer, dtype):
    """x (fp32 [T, W], in place) += norm(y) * w_post (nothing when y is None); returns
    norm(x) * w_next in ``dtype`` (None when w_next is None).  norm: the layer norm
    (x - mean) / sqrt(var + eps) when ``layer``, else x / sqrt(mean(x^2) + eps); all in fp32."""
    def nrm(v, w):
        v = v.float()
        if layer:
            v = v - v.mean(-1, keepdim=True)
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w.float()

    if y is not None:
        x += nrm(y, w_post)
    return nrm(x, w_next).to(dtype) if w_next is not None else None


def scale_softcap(logits, scale, cap):
    """fp32 cap * tanh(logits * scale / cap) (cap 0: logits * scale)."""
    z = logits.float() * scale
    return cap * torch.tanh(z / cap) if cap > 0 else z


def clamped_glu(gu, wts, limit, alpha):
    """Rows of [gate | up] products [R, 2 ff] and their router weights [R] -> the clamped GLU
    activation [R, ff] (see ``moe_experts``)."""
    ff = gu.shape[1] // 2
    w = wts.float()[:, None]
    g = (gu[:, :ff].float() * w).clamp(max=limit)
    u = (gu[:, ff:].float() * w).clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)
