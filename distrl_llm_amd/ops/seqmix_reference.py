"""Plain torch forms of the sequence-mixing ops (``ops/seqmix.py``).

They define the numerics of the HIP kernels in ``csrc_seqmix`` (each
kernel is tested against the function of the same name here) and are the
execution path of CPU runs. Everything the kernels keep in fp32 is fp32
here: norms, positions and angles, scores and softmax, recurrent state,
router logits and the residual sum.

Flat-batch conventions: a step holds ``T`` tokens of ``B`` sequences,
row ``b`` owning tokens ``cu[b]:cu[b+1]``; ``tok_seq[t]`` is the row of
token ``t``, ``positions[t]`` its position in its sequence, ``slots[b]``
the row's recurrent-state slot.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def offset_rmsnorm(x, w, eps, out_dtype, offset=1.0, groups=1):
    """x / sqrt(mean(x^2) + eps) * (offset + w) in fp32 -> (fp32, out_dtype);
    with ``groups`` > 1 the mean is taken separately over that many equal
    consecutive parts of the row."""
    x = x.float()
    xg = x.view(x.shape[0], groups, -1)
    h = (xg * torch.rsqrt(xg.pow(2).mean(-1, keepdim=True) + eps)).view_as(x)
    h = h * (offset + w.float())
    return h, h.to(out_dtype)


def causal_tap_conv(h, w, tails, cu, slots, out_dtype):
    """out_t = h_t + sum_j w[:, j] * h_(t - taps + 1 + j) per sequence, with
    the taps-1 inputs before the portion taken from ``tails[slot]``, which
    is then advanced to the portion's end. h fp32 [T, D]; w fp32 [D, taps];
    tails fp32 [slots, taps-1, D]."""
    taps = w.shape[1]
    out = torch.empty_like(h)
    cu_l, slots_l = cu.tolist(), slots.tolist()
    for b, s in enumerate(slots_l):
        a, e = cu_l[b], cu_l[b + 1]
        if e == a:
            continue
        ext = torch.cat([tails[s], h[a:e]], 0)          # [taps-1 + n, D]
        acc = h[a:e].clone()
        n = e - a
        for j in range(taps):
            acc += w[:, j] * ext[j:j + n]
        out[a:e] = acc
        if taps > 1:
            tails[s] = ext[ext.shape[0] - (taps - 1):]
    return out.to(out_dtype)


def _rotate_half(v, positions, base, dims):
    """Rotate the first ``dims`` entries of the last axis (fp32 in/out).
    v [T, ..., n]; positions [T]."""
    half = dims // 2
    i = torch.arange(half, device=v.device, dtype=torch.float32)
    freq = torch.exp2(i * (-2.0 / dims) * torch.log2(
        torch.tensor(float(base), device=v.device)))
    ang = positions.to(torch.float32)[:, None] * freq[None, :]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., dims:]], -1)


def _rotate_table(v, positions, freqs, mag, pairs):
    """Rotate the first 2 * len(freqs) entries of the last axis by the
    angles position * freqs, cos and sin scaled by ``mag``; pairs (2i, 2i+1)
    or (i, i + half). v fp32 [T, ..., n]."""
    half = freqs.numel()
    if half == 0:
        return v
    dims = 2 * half
    ang = positions.to(torch.float32)[:, None] * freqs.float()[None, :]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    c, s = (torch.cos(ang) * mag).view(shape), (torch.sin(ang) * mag).view(shape)
    if pairs:
        a, b = v[..., 0:dims:2], v[..., 1:dims:2]
        rot = torch.stack([a * c - b * s, b * c + a * s], -1).flatten(-2)
        return torch.cat([rot, v[..., dims:]], -1)
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., dims:]], -1)


def latent_prepare(q, dkv, heads, dim, rot_dim, kv_rank, norm_w, eps,
                   positions, rope_base, rope_dims, page_slot, cache,
                   freqs=None, mag=1.0, pairs=False):
    """q [T, heads * (dim + rot_dim)] query rows, dkv [T, kv_rank + rot_dim]
    (None for a layer that reads another layer's cache): write the normed
    latent and the rotated shared key part into ``cache`` rows
    ``page_slot`` and return the rotated query part [T, heads, rot_dim] in
    fp32. ``freqs`` (fp32 [rope_dims / 2]) replaces base^(-2i/dims); ``mag``
    scales cos and sin; ``pairs`` rotates entries (2i, 2i+1) instead of
    (i, i + dims/2)."""
    T = q.shape[0]

    def rot(v):
        if freqs is None:
            return _rotate_half(v, positions, rope_base, rope_dims)
        return _rotate_table(v, positions, freqs, mag, pairs)

    q = q.reshape(T, heads, dim + rot_dim)
    q_rot = rot(q[..., dim:].float())
    if dkv is not None:
        d = dkv.float()
        c = d[:, :kv_rank]
        c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
        kr = rot(d[:, kv_rank:kv_rank + rot_dim])
        cache[page_slot.long()] = torch.cat([c, kr], -1).to(cache.dtype)
    return q_rot


def latent_window_attention(q_lat, q_rot, cache, kv_rank, block_tables,
                            block_size, cu, positions, window, scale,
                            out_dtype, sink=None, gate=None):
    """Softmax attention in latent space over a paged cache.

    q_lat [H, T, kv_rank] (the query already folded through the key
    up-projection), q_rot fp32 [T, H, rot_dim], cache rows
    [c (kv_rank) | k_rot]. Token at position p sees positions j with
    0 <= p - j < window (window 0: all j <= p). ``sink`` (fp32 [H]) adds
    exp(sink[h]) to the softmax denominator; ``gate`` ([T, H]
    pre-activations) multiplies head h's result by sigmoid(gate[t, h]).
    Returns sum_j p_j c_j, [H, T, kv_rank]."""
    H, T, r = q_lat.shape
    out = torch.zeros(H, T, r, dtype=torch.float32, device=q_lat.device)
    cu_l = cu.tolist()
    pos_l = positions.tolist()
    for b in range(len(cu_l) - 1):
        a, e = cu_l[b], cu_l[b + 1]
        if e == a:
            continue
        p0, p1 = pos_l[a], pos_l[e - 1]
        lo = 0 if window <= 0 else max(0, p0 - window + 1)
        j = torch.arange(lo, p1 + 1, device=cache.device)
        rows = block_tables[b].long()[j // block_size] * block_size + j % block_size
        kv = cache[rows].float()
        c, kr = kv[:, :kv_rank], kv[:, kv_rank:]
        s = torch.einsum("htr,jr->htj", q_lat[:, a:e].float(), c)
        s = s + torch.einsum("thd,jd->htj", q_rot[a:e].float(), kr)
        s = s * scale
        p = positions[a:e].long()[:, None]
        ok = j[None, :] <= p
        if window > 0:
            ok = ok & (p - j[None, :] < window)
        s = s.masked_fill(~ok[None], float("-inf"))
        if sink is not None:
            s = torch.cat([s, sink.float()[:, None, None].expand(-1, e - a, 1)], -1)
        w = torch.softmax(s, -1)[..., :j.numel()]
        out[:, a:e] = torch.einsum("htj,jr->htr", w, c)
    if gate is not None:
        out = out * torch.sigmoid(gate.float()).t()[:, :, None]
    return out.to(out_dtype)


def mingru_scan(zxg, bias, state, cu, slots, out_dtype):
    """zxg [T, 3n] = [z | x | g] pre-activations (bias [3n] fp32 still to
    add); state fp32 [slots, n], advanced in place. Returns S_t * silu(g_t)."""
    n = zxg.shape[1] // 3
    v = zxg.float() + bias.float()
    z = torch.sigmoid(v[:, :n])
    u = v[:, n:2 * n]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = v[:, 2 * n:]
    gate = g * torch.sigmoid(g)
    out = torch.empty(zxg.shape[0], n, dtype=torch.float32, device=zxg.device)
    cu_l, slots_l = cu.tolist(), slots.tolist()
    for b, s in enumerate(slots_l):
        S = state[s]
        for t in range(cu_l[b], cu_l[b + 1]):
            S = (1.0 - z[t]) * S + z[t] * cand[t]
            out[t] = S * gate[t]
        state[s] = S
    return out.to(out_dtype)


def moe_route(h, router_w, router_b, top):
    """fp32 router: logits = W h + b; the ``top`` largest (ties: lowest
    index first); weights = softmax over the chosen logits."""
    z = F.linear(h.float(), router_w.float(), router_b.float())
    val, idx = torch.sort(z, dim=-1, descending=True, stable=True)
    val, idx = val[:, :top], idx[:, :top]
    return idx.to(torch.int32), torch.softmax(val, -1)


def moe_experts(h, idx, wts, exp_gu, exp_down):
    """sum_k wts[t,k] * down_e(silu(gate_e h) * up_e h), e = idx[t,k].
    exp_gu [E, 2ff, D] = per expert [gate; up]; exp_down [E, D, ff].
    Returns fp32 [T, D]."""
    T, D = h.shape
    E, ff2, _ = exp_gu.shape
    ff = ff2 // 2
    out = torch.zeros(T, D, dtype=torch.float32, device=h.device)
    for e in range(E):
        hit = idx == e
        rows = hit.any(-1).nonzero().flatten()
        if rows.numel() == 0:
            continue
        gu = F.linear(h[rows], exp_gu[e])
        g = gu[:, :ff].float()
        act = (g * torch.sigmoid(g) * gu[:, ff:].float()).to(h.dtype)
        y = F.linear(act, exp_down[e]).float()
        w = (wts[rows] * hit[rows]).sum(-1, keepdim=True)
        out[rows] += w * y
    return out


def gated_residual_add(x, mix, ff, gates, gate_b, mult):
    """x += mult * (mix * sigmoid(g1) + ff * sigmoid(g2)) on the fp32
    residual, in place. gates [T, D or 2D] pre-bias; ff None when the
    layer has no feed-forward."""
    D = x.shape[1]
    g = torch.sigmoid(gates.float() + gate_b.float())
    acc = mix.float() * g[:, :D]
    if ff is not None:
        acc = acc + ff.float() * g[:, D:2 * D]
    x.add_(acc, alpha=mult)
    return x


# ------------------------------------------------- sandwich-block mechanisms

def sandwich_residual_norm(x, y, y2, post_w, next_w, eps, out_dtype,
                           offset=1.0, y_scale=1.0, y2_scale=1.0,
                           cast_next=False, groups=1):
    """x += rms_unit(y_scale y [+ y2_scale y2]) * (offset + post_w) on the
    fp32 residual, in place (``post_w`` None: the sum is added as it is);
    with ``next_w`` also returns the next offset RMS norm of the new residual
    (over ``groups`` parts) in ``out_dtype``; with ``cast_next`` the new
    residual itself in ``out_dtype``; else None."""
    s = y.float() * y_scale
    if y2 is not None:
        s = s + y2.float() * y2_scale
    if post_w is None:                  # no closing norm: the plain sum
        x.add_(s)
    else:
        x.add_(s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + eps)
               * (offset + post_w.float()))
    if next_w is not None:
        return offset_rmsnorm(x, next_w, eps, out_dtype, offset, groups)[1]
    return x.to(out_dtype) if cast_next else None


def _rotate_pairs(v, positions, base, dims):
    """Rotate entries (2i, 2i+1) of the first ``dims`` of the last axis by
    position * base^(-2i/dims) (fp32 in/out). v [T, heads, n]."""
    if dims == 0:
        return v
    half = dims // 2
    i = torch.arange(half, device=v.device, dtype=torch.float32)
    freq = torch.exp2(i * (-2.0 / dims) * torch.log2(
        torch.tensor(float(base), device=v.device)))
    ang = positions.to(torch.float32)[:, None] * freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    rot = torch.stack([a * c - b * s, b * c + a * s], -1).flatten(-2)
    return torch.cat([rot, v[..., dims:]], -1)


def rope_kv_write(proj, heads, kv_heads, dim, vdim, positions, rope_base,
                  rope_dims, page_slot, cache, vmix, v_first):
    """From packed [q | k | v] projection rows: rotate q and k, blend v with
    ``v_first`` ((1 - vmix) v + vmix v_first, when given) and write
    [k | v] into ``cache`` rows ``page_slot``. Returns the rotated queries
    [T, heads, dim] in the projection's dtype."""
    T = proj.shape[0]
    nq, nk = heads * dim, kv_heads * dim
    q = _rotate_pairs(proj[:, :nq].float().view(T, heads, dim), positions,
                      rope_base, rope_dims)
    k = _rotate_pairs(proj[:, nq:nq + nk].float().view(T, kv_heads, dim),
                      positions, rope_base, rope_dims)
    v = proj[:, nq + nk:].float()
    if v_first is not None:
        lam = vmix.float().reshape(())
        v = (1.0 - lam) * v + lam * v_first.float()
    cache[page_slot.long()] = torch.cat([k.reshape(T, nk), v], -1).to(cache.dtype)
    return q.to(proj.dtype)


def sink_attention(q, cache, heads, kv_heads, dim, vdim, block_tables,
                   block_size, cu, positions, scale, softcap, sink, talk,
                   out_dtype):
    """Causal grouped-query softmax attention over paged [k | v] rows.

    score = q.k * scale, then softcap * tanh(score / softcap) when softcap
    > 0; the softmax denominator also holds exp(sink[h]) (sink None: plain
    softmax); the heads' weights are mixed by ``talk`` [H, H]
    (w_h <- sum_g talk[h, g] w_g) before head h reads the values of its own
    kv head. q [T, H, dim] -> [T, H * vdim]."""
    T = q.shape[0]
    rep = heads // kv_heads
    nk = kv_heads * dim
    out = torch.zeros(T, heads, vdim, dtype=torch.float32, device=q.device)
    cu_l, pos_l = cu.tolist(), positions.tolist()
    for b in range(len(cu_l) - 1):
        a, e = cu_l[b], cu_l[b + 1]
        if e == a:
            continue
        j = torch.arange(0, pos_l[e - 1] + 1, device=cache.device)
        rows = block_tables[b].long()[j // block_size] * block_size + j % block_size
        kv = cache[rows].float()
        k = kv[:, :nk].view(-1, kv_heads, dim).repeat_interleave(rep, 1)
        v = kv[:, nk:].view(-1, kv_heads, vdim).repeat_interleave(rep, 1)
        s = torch.einsum("thd,jhd->htj", q[a:e].float(), k) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        ok = j[None, :] <= positions[a:e].long()[:, None]
        s = s.masked_fill(~ok[None], float("-inf"))
        if sink is not None:
            s = torch.cat([s, sink.float()[:, None, None].expand(-1, e - a, 1)], -1)
        w = torch.softmax(s, -1)[..., :j.numel()]
        if talk is not None:
            w = torch.einsum("hg,gtj->htj", talk.float(), w)
        out[a:e] = torch.einsum("htj,jhd->thd", w, v)
    return out.reshape(T, heads * vdim).to(out_dtype)


def tap_conv_silu(x, w, tails, cu, slots, out_dtype):
    """silu(sum_j w[:, j] * x_(t - taps + 1 + j)) per channel and sequence;
    inputs before the portion come from ``tails[slot]`` (fp32
    [slots, taps-1, C]), which is advanced to the portion's end."""
    taps = w.shape[1]
    x = x.float()
    out = torch.empty_like(x)
    cu_l, slots_l = cu.tolist(), slots.tolist()
    for b, s in enumerate(slots_l):
        a, e = cu_l[b], cu_l[b + 1]
        if e == a:
            continue
        ext = torch.cat([tails[s], x[a:e]], 0)
        n = e - a
        acc = torch.zeros_like(x[a:e])
        for j in range(taps):
            acc += w[:, j] * ext[j:j + n]
        out[a:e] = acc * torch.sigmoid(acc)
        if taps > 1:
            tails[s] = ext[ext.shape[0] - (taps - 1):]
    return out.to(out_dtype)


def gated_delta_rule(qkv, gate, ab, a_log, dt_bias, onorm_w, eps, state, cu,
                     slots, heads, kv_heads, dim, vdim, out_dtype,
                     decay_up=None, gate_sigmoid=False):
    """Gated delta rule over a flat batch.

    qkv [T, 2 G dim + H vdim] (after convolution and SiLU), gate [T, H vdim]
    pre-activation, ab fp32 [T, 2H] = [write strength | step] pre-activations.
    Per head: q, k -> unit vectors (q also / sqrt(dim));
    beta = sigmoid(b); decay = exp(-exp(a_log) softplus(a + dt_bias));
    S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q;
    out = o / rms(o) * onorm_w * silu(gate). state fp32
    [slots, H * vdim * dim] (per head value-major: S^T), advanced in place.
    With ``decay_up`` (fp32 [H dim, R]) the decay is per head and key
    channel: ab = [write strength (H) | low-rank decay input (R)], the step
    is softplus(decay_up a + dt_bias) with dt_bias [H dim], and the decay
    multiplies the state's key rows. ``gate_sigmoid``: the output gate is
    sigmoid(gate) instead of silu(gate)."""
    T = qkv.shape[0]
    H, G = heads, kv_heads
    rep = H // G
    n = G * dim
    x = qkv.float()
    q = x[:, :n].view(T, G, dim)
    k = x[:, n:2 * n].view(T, G, dim)
    v = x[:, 2 * n:].view(T, H, vdim)
    q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(ab[:, :H].float())
    if decay_up is None:
        decay = torch.exp(-torch.exp(a_log.float())
                          * F.softplus(ab[:, H:].float() + dt_bias.float()))
        decay = decay[:, :, None]                       # [T, H, 1]
    else:
        step = F.softplus(F.linear(ab[:, H:].float(), decay_up.float())
                          + dt_bias.float()).view(T, H, dim)
        decay = torch.exp(-torch.exp(a_log.float())[None, :, None] * step)
    o = torch.empty(T, H, vdim, dtype=torch.float32, device=qkv.device)
    cu_l, slots_l = cu.tolist(), slots.tolist()
    for b, s in enumerate(slots_l):
        S = state[s].view(H, vdim, dim).transpose(1, 2).clone()
        for t in range(cu_l[b], cu_l[b + 1]):
            S = decay[t][:, :, None] * S
            u = beta[t][:, None] * (v[t] - torch.einsum("hkv,hk->hv", S, k[t]))
            S = S + k[t][:, :, None] * u[:, None, :]
            o[t] = torch.einsum("hkv,hk->hv", S, q[t])
        state[s] = S.transpose(1, 2).reshape(-1)
    o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * onorm_w.float()
    g = gate.float().view(T, H, vdim)
    act = torch.sigmoid(g) if gate_sigmoid else g * torch.sigmoid(g)
    return (o * act).reshape(T, H * vdim).to(out_dtype)


def capped_glu(gu, limit):
    """gu [T, 2ff] = [gate | up]: g = min(gate, limit), u = clamp(up,
    +-limit); g * sigmoid(1.702 g) * (u + 1), in gu's dtype."""
    ff = gu.shape[1] // 2
    g = gu[:, :ff].float().clamp(max=limit)
    u = gu[:, ff:].float().clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)).to(gu.dtype)


def silu_glu(gu):
    """gu [T, 2ff] = [gate | up]: silu(gate) * up, in gu's dtype."""
    ff = gu.shape[1] // 2
    g = gu[:, :ff].float()
    return (g * torch.sigmoid(g) * gu[:, ff:].float()).to(gu.dtype)


def qk_norm_kv_write(proj, heads, kv_heads, dim, vdim, q_norm_w, k_norm_w, eps,
                     page_slot, cache):
    """From packed [q | k | v] projection rows: RMS-norm every q and k head
    over ``dim`` with the shared plain weights, write [k | v] into ``cache``
    rows ``page_slot``; returns the normed queries [T, heads, dim] in the
    projection's dtype."""
    T = proj.shape[0]
    nq, nk = heads * dim, kv_heads * dim
    q = proj[:, :nq].float().view(T, heads, dim)
    k = proj[:, nq:nq + nk].float().view(T, kv_heads, dim)
    q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_norm_w.float()
    k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_norm_w.float()
    v = proj[:, nq + nk:nq + nk + kv_heads * vdim].float()
    cache[page_slot.long()] = torch.cat([k.reshape(T, nk), v], -1).to(cache.dtype)
    return q.to(proj.dtype)


def sigmoid_attention(q, cache, heads, kv_heads, dim, vdim, block_tables,
                      block_size, cu, positions, scale, window, keep_first,
                      slopes, pos_bias, out_dtype):
    """Grouped-query attention with sigmoid weights over paged [k | v] rows.

    weight(i, j) = sigmoid(q_i . k_j * scale - slopes[h] (i - j) + pos_bias[h])
    for the visible keys j <= i with i - j < window or j < keep_first
    (window 0: all j <= i); weights are not normalised.
    q [T, H, dim] -> [T, H * vdim]."""
    T = q.shape[0]
    rep = heads // kv_heads
    nk = kv_heads * dim
    out = torch.zeros(T, heads, vdim, dtype=torch.float32, device=q.device)
    cu_l, pos_l = cu.tolist(), positions.tolist()
    sl = slopes.float()[:, None, None]
    for b in range(len(cu_l) - 1):
        a, e = cu_l[b], cu_l[b + 1]
        if e == a:
            continue
        j = torch.arange(0, pos_l[e - 1] + 1, device=cache.device)
        rows = block_tables[b].long()[j // block_size] * block_size + j % block_size
        kv = cache[rows].float()
        k = kv[:, :nk].view(-1, kv_heads, dim).repeat_interleave(rep, 1)
        v = kv[:, nk:].view(-1, kv_heads, vdim).repeat_interleave(rep, 1)
        p = positions[a:e].long()[:, None]
        dist = (p - j[None, :]).float()
        s = torch.einsum("thd,jhd->htj", q[a:e].float(), k) * scale
        s = s - sl * dist[None] + pos_bias.float()[:, None, None]
        ok = j[None, :] <= p
        if window > 0:
            ok = ok & ((p - j[None, :] < window) | (j[None, :] < keep_first))
        w = torch.sigmoid(s) * ok[None]
        out[a:e] = torch.einsum("htj,jhd->thd", w, v)
    return out.reshape(T, heads * vdim).to(out_dtype)


def moe_route_all(h, router_w, correction, top, scale):
    """fp32 router over every output: s = softmax(W h); the ``top`` largest
    s + correction are chosen (ties: lowest index first); weights =
    s[chosen] * scale, not renormalised."""
    s = torch.softmax(F.linear(h.float(), router_w.float()), -1)
    c = s if correction is None else s + correction.float()
    _, idx = torch.sort(c, dim=-1, descending=True, stable=True)
    idx = idx[:, :top]
    return idx.to(torch.int32), torch.gather(s, 1, idx) * scale


def moe_experts_glu(h, idx, wts, exp_gu, exp_down, limit):
    """Mixture of clamped-GLU experts; indices >= the number of expert
    weight sets name identity experts whose output is the input itself."""
    T, D = h.shape
    E = exp_gu.shape[0]
    out = torch.zeros(T, D, dtype=torch.float32, device=h.device)
    for e in range(E):
        hit = idx == e
        rows = hit.any(-1).nonzero().flatten()
        if rows.numel() == 0:
            continue
        act = capped_glu(F.linear(h[rows], exp_gu[e]), limit)
        y = F.linear(act, exp_down[e]).float()
        out[rows] += (wts[rows] * hit[rows]).sum(-1, keepdim=True) * y
    ident = (wts * (idx >= E)).sum(-1, keepdim=True)
    return out + ident * h.float()


# ------------------------------------------- windowed softmax attention, MLP

def qk_prepare_kv_write(proj, heads, kv_heads, dim, vdim, q_norm_w, k_norm_w,
                        eps, positions, freqs, mag, mix, page_slot, cache):
    """From packed [q | k | v | ...] projection rows: optional RMS norm of
    every q and k head (plain shared weights), optional half-layout rotation
    of their first 2 len(freqs) entries by position * freqs with cos and sin
    scaled by ``mag``, page write of [k | v]. Returns the queries in the
    projection's dtype: [T, heads, dim], or with ``mix`` (fp32 [H, H])
    [T, heads, kv_heads * dim], where row h holds, in the columns of kv head
    c, sum over the heads g of c of mix[h, g] q_g: its product with a whole
    key row is the score of head h mixed over all heads."""
    T = proj.shape[0]
    nq, nk = heads * dim, kv_heads * dim
    q = proj[:, :nq].float().view(T, heads, dim)
    k = proj[:, nq:nq + nk].float().view(T, kv_heads, dim)
    if q_norm_w is not None:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_norm_w.float()
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_norm_w.float()
    if freqs is not None and freqs.numel():
        q = _rotate_table(q, positions, freqs, mag, False)
        k = _rotate_table(k, positions, freqs, mag, False)
    v = proj[:, nq + nk:nq + nk + kv_heads * vdim].float()
    cache[page_slot.long()] = torch.cat([k.reshape(T, nk), v], -1).to(cache.dtype)
    if mix is not None:
        rep = heads // kv_heads
        m = mix.float().view(heads, kv_heads, rep)
        q = torch.einsum("hcr,tcrd->thcd", m, q.view(T, kv_heads, rep, dim))
        q = q.reshape(T, heads, nk)
    return q.to(proj.dtype)


def window_attention(q, cache, heads, kv_heads, dim, vdim, whole_key,
                     block_tables, block_size, cu, positions, scale, window,
                     keep_first, r1, r2, gate, out_dtype):
    """Grouped-query softmax attention over paged [k | v] rows.

    Query i sees the keys j <= i with i - j < window or j < keep_first
    (window 0: all j <= i). score = q . k * scale, where head h meets the
    keys of its own kv head, or with ``whole_key`` (q rows of kv_heads * dim
    entries) the whole key row; ``r1``/``r2`` (fp32 [H]) take
    r1 ln(1 + r2 (i - j)) off the score; ``gate`` ([T, H] pre-activations)
    scales head h's result by its sigmoid. -> [T, H * vdim]."""
    T = q.shape[0]
    rep = heads // kv_heads
    nk = kv_heads * dim
    out = torch.zeros(T, heads, vdim, dtype=torch.float32, device=q.device)
    cu_l, pos_l = cu.tolist(), positions.tolist()
    for b in range(len(cu_l) - 1):
        a, e = cu_l[b], cu_l[b + 1]
        if e == a:
            continue
        j = torch.arange(0, pos_l[e - 1] + 1, device=cache.device)
        rows = block_tables[b].long()[j // block_size] * block_size + j % block_size
        kv = cache[rows].float()
        v = kv[:, nk:].view(-1, kv_heads, vdim).repeat_interleave(rep, 1)
        if whole_key:
            s = torch.einsum("thd,jd->htj", q[a:e].float(), kv[:, :nk]) * scale
        else:
            k = kv[:, :nk].view(-1, kv_heads, dim).repeat_interleave(rep, 1)
            s = torch.einsum("thd,jhd->htj", q[a:e].float(), k) * scale
        p = positions[a:e].long()[:, None]
        if r1 is not None:
            dist = (p - j[None, :]).clamp(min=0).float()
            s = s - r1.float()[:, None, None] * torch.log1p(
                r2.float()[:, None, None] * dist[None])
        ok = j[None, :] <= p
        if window > 0:
            ok = ok & ((p - j[None, :] < window) | (j[None, :] < keep_first))
        s = s.masked_fill(~ok[None], float("-inf"))
        out[a:e] = torch.einsum("htj,jhd->thd", torch.softmax(s, -1), v)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[:, :, None]
    return out.reshape(T, heads * vdim).to(out_dtype)


def gelu_tanh(x):
    """0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))) in x's dtype."""
    z = x.float()
    return (0.5 * z * (1.0 + torch.tanh(0.7978845608028654
                                        * (z + 0.044715 * z * z * z)))).to(x.dtype)


def moe_route_sigmoid(h, router_w, top):
    """fp32 router: scores = sigmoid(W h); the ``top`` largest (ties: lowest
    index first); weights = the chosen scores, not renormalised."""
    s = torch.sigmoid(F.linear(h.float(), router_w.float()))
    _, idx = torch.sort(s, dim=-1, descending=True, stable=True)
    idx = idx[:, :top]
    return idx.to(torch.int32), torch.gather(s, 1, idx)


def moe_experts_scaled_input(h, idx, wts, exp_gu, exp_down):
    """sum_k down_e(silu(gate_e (w h)) * up_e (w h)), e = idx[t, k],
    w = wts[t, k]: the weight multiplies the expert's input. The products
    gate_e h and up_e h are scaled by w in fp32 before the activation.
    Returns fp32 [T, D]."""
    T, D = h.shape
    E, ff2, _ = exp_gu.shape
    ff = ff2 // 2
    out = torch.zeros(T, D, dtype=torch.float32, device=h.device)
    for k in range(idx.shape[1]):
        for e in range(E):
            rows = (idx[:, k] == e).nonzero().flatten()
            if rows.numel() == 0:
                continue
            gu = F.linear(h[rows], exp_gu[e]).float() * wts[rows, k:k + 1]
            g = gu[:, :ff]
            act = (g * torch.sigmoid(g) * gu[:, ff:]).to(h.dtype)
            out[rows] += F.linear(act, exp_down[e]).float()
    return out
