"""Plain float64 implementation of the Legilix design, one function per
mechanism, written position by position from the design's equations. It
shares no code with the package: tests compare the engine against it.

``cfg`` is the design's ``config.json`` as a dict, ``w`` maps checkpoint
tensor names to tensors. Every function takes one whole sequence.
"""

import math

import torch

F64 = torch.float64


def group_norm(x, weight, groups, eps):
    """x [..., D] cut into ``groups`` consecutive parts; each part divided by
    its own root mean square, the whole times ``weight``."""
    D = x.shape[-1]
    n = D // groups
    out = torch.empty_like(x)
    for g in range(groups):
        part = x[..., g * n:(g + 1) * n]
        out[..., g * n:(g + 1) * n] = part / torch.sqrt(
            (part * part).mean(-1, keepdim=True) + eps)
    return out * weight


def head_norm(x, weight, eps):
    """RMS norm over the last axis with a plain weight."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rotary_table(rot):
    """Per-pair frequencies and the common factor on cos and sin."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def where(turns):
            return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

        lo = max(math.floor(where(float(sc["fast"]))), 0)
        hi = min(math.ceil(where(float(sc["slow"]))), dims - 1)
        for i in range(len(f)):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / factor * ramp + f[i] * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    return f, mag


def rotate_halves(v, pos, rot):
    """v [..., n] at position pos: entry i pairs with entry i + dims/2."""
    if not rot or not int(rot.get("dims") or 0):
        return v
    f, mag = rotary_table(rot)
    half = len(f)
    out = v.clone()
    for i, fi in enumerate(f):
        a = pos * fi
        c, s = math.cos(a) * mag, math.sin(a) * mag
        u, w_ = v[..., i], v[..., i + half]
        out[..., i] = u * c - w_ * s
        out[..., i + half] = w_ * c + u * s
    return out


def visible(i, mask):
    """Positions that position i sees under a sliding window that may keep
    the first tokens."""
    size = int(mask.get("size") or 0)
    keep = int(mask.get("keep_first") or 0)
    return [j for j in range(i + 1)
            if size <= 0 or i - j < size or j < keep]


def _lin(w, name, h):
    y = h @ w[name].to(F64).t()
    if name + ".b" in w:
        y = y + w[name + ".b"].to(F64)
    return y


def rotary_attention(mc, w, p, h, eps):
    """The 'attention' mixer: q/k norm, rotation, scores mixed across heads
    before the softmax, window with kept first tokens."""
    T = h.shape[0]
    H, G, dk, dv = int(mc["heads"]), int(mc["kv_heads"]), int(mc["dim"]), int(mc["vdim"])
    rep = H // G
    q = _lin(w, p + "q", h).view(T, H, dk)
    k = _lin(w, p + "k", h).view(T, G, dk)
    v = _lin(w, p + "v", h).view(T, G, dv)
    q = head_norm(q, w[p + "q.norm"].to(F64), eps)
    k = head_norm(k, w[p + "k.norm"].to(F64), eps)
    rot = mc.get("rot")
    q = torch.stack([rotate_halves(q[t], t, rot) for t in range(T)])
    k = torch.stack([rotate_halves(k[t], t, rot) for t in range(T)])
    talk = w[p + "talk"].to(F64)
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        js = visible(i, mc.get("mask") or {})
        kk = k[js]                                   # [n, G, dk]
        s = torch.stack([kk[:, a // rep] @ q[i, a] for a in range(H)]) * float(mc["scale"])
        s = talk @ s                                 # [H, n]
        wt = torch.softmax(s, -1)
        for a in range(H):
            out[i, a] = wt[a] @ v[js][:, a // rep]
    return out.reshape(T, H * dv) @ w[p + "o"].to(F64).t()


def distance_attention(mc, w, p, h):
    """The 'attention_2' mixer: no rotation, a logarithmic distance bias,
    plain window, sigmoid gate per head on the output."""
    T = h.shape[0]
    H, G, dk, dv = int(mc["heads"]), int(mc["kv_heads"]), int(mc["dim"]), int(mc["vdim"])
    rep = H // G
    q = _lin(w, p + "q", h).view(T, H, dk)
    k = _lin(w, p + "k", h).view(T, G, dk)
    v = _lin(w, p + "v", h).view(T, G, dv)
    r1, r2 = w[p + "r1"].to(F64), w[p + "r2"].to(F64)
    gate = torch.sigmoid(h @ w[p + "g"].to(F64).t())     # [T, H]
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        js = visible(i, mc.get("mask") or {})
        dist = torch.tensor([float(i - j) for j in js], dtype=F64)
        for a in range(H):
            s = (k[js][:, a // rep] @ q[i, a]) * float(mc["scale"])
            s = s - r1[a] * torch.log(1.0 + r2[a] * dist)
            out[i, a] = (torch.softmax(s, -1) @ v[js][:, a // rep]) * gate[i, a]
    return out.reshape(T, H * dv) @ w[p + "o"].to(F64).t()


def dense_ff(w, p, h):
    return gelu_tanh(h @ w[p + "up"].to(F64).t()) @ w[p + "down"].to(F64).t()


def expert(w, p, h):
    return (silu(h @ w[p + "gate"].to(F64).t()) * (h @ w[p + "up"].to(F64).t())
            ) @ w[p + "down"].to(F64).t()


def route(w, p, h, top):
    """Chosen experts and their weights for one token."""
    s = torch.sigmoid(w[p + "router"].to(F64) @ h)
    order = sorted(range(s.numel()), key=lambda e: (-float(s[e]), e))[:top]
    return order, [s[e] for e in order]


def moe_ff(fc, w, p, h):
    top = int(fc["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        idx, wt = route(w, p, h[t], top)
        for e, g in zip(idx, wt):
            out[t] = out[t] + expert(w, f"{p}e{e}.", g * h[t])
    return out


def forward(cfg, w, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out`` (a list) receives
    the residual stream after every layer."""
    eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"].get("groups") or 1)
    E = w["embed"].to(F64)
    x = E[torch.tensor(tokens)] * float(cfg["embedding"]["scale"])
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = group_norm(x, w[p + "norm1"].to(F64), groups, eps)
        if lc["type"] == "attention":
            x = x + rotary_attention(lc["mixer"], w, p + "mix.", h, eps)
        elif lc["type"] == "attention_2":
            x = x + distance_attention(lc["mixer"], w, p + "mix.", h)
        else:
            raise ValueError(lc["type"])
        fc = lc.get("mlp")
        if fc is not None:
            h = group_norm(x, w[p + "norm2"].to(F64), groups, eps)
            if fc["kind"] == "dense":
                x = x + dense_ff(w, p + "mlp.", h)
            else:
                x = x + moe_ff(fc, w, p + "mlp.", h)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = group_norm(x, w["final.norm"].to(F64), groups, eps)
    return (x @ E.t()) * float(cfg["logit_scale"])
