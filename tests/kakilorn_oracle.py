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


# ------------------------------------------------ configurations and weights

def latent_layer(heads=2, dim=4, rot_dim=4, vdim=5, kv_rank=6, q_rank=7, scale=0.4,
                 base=100.0, rot_dims=None, scaling=None, mlp=8):
    rot = {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"type": "latent_attention", "mlp": _mlp(mlp),
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
                      "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale, "rot": rot}}


def channel_layer(heads=2, kv_heads=2, dim=8, vdim=6, conv=3, mlp=None, ranks=(3, 5)):
    return {"type": "channel_delta", "mlp": _mlp(mlp), "ranks": ranks,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                      "conv": conv}}


def parallel_layer(heads=4, kv_heads=2, dim=6, vdim=5, scale=0.5, window=5, keep=2,
                   r_heads=2, r_kv_heads=1, r_dim=8, r_vdim=6, conv=2, left_scale=0.8,
                   right_scale=1.3, mlp=8):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        left["mask"] = {"size": window, "keep_first": keep}
    return {"type": "parallel", "mlp": _mlp(mlp),
            "mixer": {"left": left, "left_scale": left_scale, "right_scale": right_scale,
                      "right": {"heads": r_heads, "kv_heads": r_kv_heads, "dim": r_dim,
                                "vdim": r_vdim, "conv": conv}}}


def _mlp(ff):
    return None if ff is None else {"kind": "dense", "ff": ff}


def make_cfg(layers, width=16, vocab=29, eps=1e-5, embed_scale=0.7, logit_scale=0.4):
    """(config dict, {layer index: (decay rank, gate rank)})."""
    ranks = {i: l["ranks"] for i, l in enumerate(layers) if "ranks" in l}
    layers = [{k: v for k, v in l.items() if k != "ranks"} for l in layers]
    return {"architecture": "Kakilorn", "embedding": {"scale": embed_scale},
            "layers": layers, "logit_scale": logit_scale, "norm": {"eps": eps},
            "vocab": vocab, "width": width}, ranks


def random_weights(cfg, ranks, seed=0):
    """Random bf16-representable tensors under the design's names."""
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]
    w = {}

    def mat(name, rows, cols, s=None):
        w[name] = torch.randn(rows, cols, generator=g) * (s if s is not None else cols ** -0.5)

    def vec(name, n, mean=0.0, s=0.3):
        w[name] = mean + s * torch.randn(n, generator=g)

    def delta(x, mc, chan, rk=None):
        H, G, dk, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        for nm, rows in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
            mat(x + nm, rows, D, 1.5 * D ** -0.5)
            mat(x + nm + ".conv", rows, mc["conv"], 0.6)
        mat(x + "b", H, D)
        vec(x + "A_log", H, -0.5, 0.5)
        vec(x + "norm", dv, 1.0, 0.2)
        if chan:
            mat(x + "a1", rk[0], D)
            mat(x + "a2", H * dk, rk[0])
            vec(x + "dt_bias", H * dk, -1.0, 1.0)
            mat(x + "g1", rk[1], D)
            mat(x + "g2", H * dv, rk[1])
        else:
            mat(x + "a", H, D)
            vec(x + "dt_bias", H, -1.0, 1.0)
            mat(x + "g", H * dv, D)
        mat(x + "o", D, H * dv)

    mat("embed", cfg["vocab"], D, 1.0)
    vec("final.norm", D, 1.0, 0.2)
    for i, lc in enumerate(cfg["layers"]):
        p, mc = f"l{i}.", lc["mixer"]
        x = p + "mix."
        vec(p + "norm1", D, 1.0, 0.2)
        if lc["type"] == "latent_attention":
            H, dn, dr, dv = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"]
            r, rq = mc["kv_rank"], mc["q_rank"]
            mat(x + "dq", rq, D)
            vec(x + "dq.norm", rq, 1.0, 0.2)
            mat(x + "uq", H * (dn + dr), rq, 2.0 * rq ** -0.5)
            mat(x + "dkv", r + dr, D)
            vec(x + "dkv.norm", r, 1.0, 0.2)
            mat(x + "uk", H * dn, r, 2.0 * r ** -0.5)
            mat(x + "uv", H * dv, r)
            vec(x + "sink", H, 0.5, 1.0)
            mat(x + "g", H, D)
            mat(x + "o", D, H * dv)
        elif lc["type"] == "channel_delta":
            delta(x, mc, True, ranks[i])
        else:
            a = mc["left"]
            H, G, dk, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            mat(x + "left.q", H * dk, D)
            mat(x + "left.k", G * dk, D)
            mat(x + "left.v", G * dv, D)
            vec(x + "left.q.norm", dk, 1.0, 0.3)
            vec(x + "left.k.norm", dk, 1.0, 0.3)
            vec(x + "left.pb", H, -0.5, 0.7)
            mat(x + "left.o", D, H * dv)
            delta(x + "right.", mc["right"], False)
        if lc.get("mlp") is not None:
            ff = lc["mlp"]["ff"]
            vec(p + "norm2", D, 1.0, 0.2)
            mat(p + "mlp.gate", ff, D)
            mat(p + "mlp.up", ff, D)
            mat(p + "mlp.down", D, ff)
    return {k: v.bfloat16().float() for k, v in w.items()}
