"""Plain float64 implementation of the Kakilorn design, one function per
mechanism, written position by position from the design's equations. It
shares no code with the package: tests compare the engine against it.

``cfg`` is the design's ``config.json`` as a dict, ``w`` maps checkpoint
tensor names to tensors. Every function takes one whole sequence.
"""

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def rotary_table(rot):
    """Per-pair frequencies and the common factor on cos and sin."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def turn_dim(turns):
            return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

        lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
        hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
        for i in range(half):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / factor * ramp + f[i] * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    return f, mag


def rotate_interleaved(v, pos, rot):
    """v [..., n] at position pos: pairs (2i, 2i+1) of the first dims."""
    f, mag = rotary_table(rot)
    out = v.clone()
    for i, fi in enumerate(f):
        a = pos * fi
        c, s = math.cos(a) * mag, math.sin(a) * mag
        u, w_ = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = u * c - w_ * s
        out[..., 2 * i + 1] = w_ * c + u * s
    return out


def short_conv_silu(x, taps_w):
    """x [T, C], taps_w [C, taps]; last column meets the current token."""
    T, C = x.shape
    taps = taps_w.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        acc = torch.zeros(C, dtype=F64)
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                acc = acc + taps_w[:, j] * x[s]
        out[t] = silu(acc)
    return out


def delta_walk(q, k, v, beta, decay):
    """q, k [T, H, dk] (already unit vectors), v [T, H, dv], beta [T, H],
    decay [T, H, dk] (a per-head decay is repeated over dk). Returns o."""
    T, H, dk = k.shape
    dv = v.shape[-1]
    S = torch.zeros(H, dk, dv, dtype=F64)
    o = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        S = decay[t][:, :, None] * S
        read = torch.einsum("hkv,hk->hv", S, k[t])
        u = beta[t][:, None] * (v[t] - read)
        S = S + k[t][:, :, None] * u[:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return o


def _delta_inputs(h, w, p, mc):
    H, G, dk, dv = int(mc["heads"]), int(mc["kv_heads"]), int(mc["dim"]), int(mc["vdim"])
    T = h.shape[0]
    q = short_conv_silu(h @ w[p + "q"].T, w[p + "q.conv"]).view(T, G, dk)
    k = short_conv_silu(h @ w[p + "k"].T, w[p + "k.conv"]).view(T, G, dk)
    v = short_conv_silu(h @ w[p + "v"].T, w[p + "v.conv"]).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(h @ w[p + "b"].T)
    return q, k, v, beta


def head_delta(h, w, p, mc, eps):
    """Gated delta rule with one decay per head and a SiLU output gate."""
    H, dk, dv = int(mc["heads"]), int(mc["dim"]), int(mc["vdim"])
    T = h.shape[0]
    q, k, v, beta = _delta_inputs(h, w, p, mc)
    step = torch.nn.functional.softplus(h @ w[p + "a"].T + w[p + "dt_bias"])
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * step)            # [T, H]
    o = delta_walk(q, k, v, beta, decay[:, :, None].expand(T, H, dk))
    o = unit_rms(o, eps) * w[p + "norm"] * silu(h @ w[p + "g"].T).view(T, H, dv)
    return o.reshape(T, H * dv) @ w[p + "o"].T


def channel_delta(h, w, p, mc, eps):
    """Gated delta rule with a decay per head and key channel (low-rank
    input) and a low-rank sigmoid output gate."""
    H, dk, dv = int(mc["heads"]), int(mc["dim"]), int(mc["vdim"])
    T = h.shape[0]
    q, k, v, beta = _delta_inputs(h, w, p, mc)
    step = torch.nn.functional.softplus(
        (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).view(T, H, dk)
    decay = torch.exp(-torch.exp(w[p + "A_log"])[None, :, None] * step)
    o = delta_walk(q, k, v, beta, decay)
    gate = torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).view(T, H, dv)
    o = unit_rms(o, eps) * w[p + "norm"] * gate
    return o.reshape(T, H * dv) @ w[p + "o"].T


def sigmoid_window_attention(h, w, p, mc, eps):
    """Grouped-query attention without softmax: sigmoid weights, a linear
    distance penalty per head, a sliding window that keeps the first
    tokens, RMS-normed queries and keys."""
    H, G, dk, dv = int(mc["heads"]), int(mc["kv_heads"]), int(mc["dim"]), int(mc["vdim"])
    T = h.shape[0]
    mask = mc.get("mask") or {}
    size, keep = int(mask.get("size") or 0), int(mask.get("keep_first") or 0)
    q = unit_rms((h @ w[p + "q"].T).view(T, H, dk), eps) * w[p + "q.norm"]
    k = unit_rms((h @ w[p + "k"].T).view(T, G, dk), eps) * w[p + "k.norm"]
    v = (h @ w[p + "v"].T).view(T, G, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for a in range(H):
        g = a // (H // G)
        slope = 2.0 ** (-8.0 * (a + 1) / H)
        for i in range(T):
            j = torch.arange(i + 1)
            seen = torch.ones(i + 1, dtype=torch.bool)
            if size > 0:
                seen = (i - j < size) | (j < keep)
            s = (k[:i + 1, g] @ q[i, a]) * float(mc["scale"]) - slope * (i - j).to(F64)
            wt = torch.sigmoid(s + w[p + "pb"][a]) * seen.to(F64)
            out[i, a] = wt @ v[:i + 1, g]
    return out.reshape(T, H * dv) @ w[p + "o"].T


def parallel_mixer(h, w, p, mc, eps):
    left = sigmoid_window_attention(h, w, p + "left.", mc["left"], eps)
    right = head_delta(h, w, p + "right.", mc["right"], eps)
    return float(mc["left_scale"]) * left + float(mc["right_scale"]) * right


def latent_attention(h, w, p, mc, eps):
    """Low-rank queries and a shared key/value latent; rotated part shared
    by the heads; causal softmax with a per-head sink; per-head output gate."""
    H, dn, dr, dv = int(mc["heads"]), int(mc["dim"]), int(mc["rot_dim"]), int(mc["vdim"])
    r = int(mc["kv_rank"])
    T = h.shape[0]
    cq = unit_rms(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (cq @ w[p + "uq"].T).view(T, H, dn + dr)
    dkv = h @ w[p + "dkv"].T
    c = unit_rms(dkv[:, :r], eps) * w[p + "dkv.norm"]
    kr = dkv[:, r:r + dr]
    kn = (c @ w[p + "uk"].T).view(T, H, dn)
    v = (c @ w[p + "uv"].T).view(T, H, dv)
    qr = torch.stack([rotate_interleaved(q[t, :, dn:], t, mc["rot"]) for t in range(T)])
    kr = torch.stack([rotate_interleaved(kr[t], t, mc["rot"]) for t in range(T)])
    gate = torch.sigmoid(h @ w[p + "g"].T)                        # [T, H]
    out = torch.zeros(T, H, dv, dtype=F64)
    for a in range(H):
        for i in range(T):
            s = (kn[:i + 1, a] @ q[i, a, :dn] + kr[:i + 1] @ qr[i, a]) * float(mc["scale"])
            m = max(float(s.max()), float(w[p + "sink"][a]))
            e = torch.exp(s - m)
            den = e.sum() + math.exp(float(w[p + "sink"][a]) - m)
            out[i, a] = (e / den) @ v[:i + 1, a] * gate[i, a]
    return out.reshape(T, H * dv) @ w[p + "o"].T


def dense_ff(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


MIXERS = {"channel_delta": channel_delta, "latent_attention": latent_attention,
          "parallel": parallel_mixer}


def forward(cfg, w, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out`` (a list) receives
    the residual stream after every layer."""
    w = {k: v.to(F64) for k, v in w.items()}
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens)] * float(cfg["embedding"]["scale"])
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = MIXERS[lc["type"]](x, w, p + "mix.", lc["mixer"], eps)
        x = x + unit_rms(y, eps) * w[p + "norm1"]
        if lc.get("mlp") is not None:
            x = x + unit_rms(dense_ff(x, w, p + "mlp."), eps) * w[p + "norm2"]
        if layers_out is not None:
            layers_out.append(x.clone())
    hid = unit_rms(x, eps) * w["final.norm"]
    return hid @ w["embed"].T * float(cfg["logit_scale"])
