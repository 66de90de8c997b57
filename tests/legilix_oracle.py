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


# ------------------------------------------------- small configs for tests

def rotary_layer(heads=4, kv_heads=2, dim=8, vdim=6, window=7, keep=2, rot_dims=4,
                 base=100.0, scaling=(4.0, 16, 2.0, 0.5), scale=None, mlp=12):
    """An 'attention' layer; ``mlp`` an int (dense ff), a tuple (experts,
    top, ff) or None."""
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    mask = {"size": window, "keep_first": keep} if window else {}
    mc = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
          "mask": mask, "rot": rot, "scale": scale if scale is not None else dim ** -0.5}
    return {"type": "attention", "mixer": mc, "mlp": _mlp(mlp)}


def distance_layer(heads=4, kv_heads=2, dim=8, vdim=6, window=7, scale=None, mlp=12):
    """An 'attention_2' layer."""
    mc = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
          "mask": {"size": window} if window else {},
          "scale": scale if scale is not None else dim ** -0.5}
    return {"type": "attention_2", "mixer": mc, "mlp": _mlp(mlp)}


def _mlp(m):
    if m is None:
        return None
    if isinstance(m, int):
        return {"kind": "dense", "ff": m}
    experts, top, ff = m
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def make_cfg(layers, width=24, vocab=37, groups=3, eps=1e-5, embed_scale=3.0,
             logit_scale=0.5):
    return {"architecture": "Legilix", "embedding": {"scale": embed_scale},
            "layers": layers, "logit_scale": logit_scale,
            "norm": {"eps": eps, "groups": groups}, "vocab": vocab, "width": width}


def random_weights(cfg, seed=0):
    """Checkpoint tensors of a configuration, rounded to bfloat16 as a
    checkpoint file holds them."""
    g = torch.Generator().manual_seed(seed)
    D = int(cfg["width"])
    w = {}

    def mat(name, rows, cols):
        w[name] = torch.randn(rows, cols, generator=g) / math.sqrt(cols)

    def vec(name, n, mean=0.0, std=0.1):
        w[name] = mean + std * torch.randn(n, generator=g)

    w["embed"] = torch.randn(int(cfg["vocab"]), D, generator=g) * 0.5
    vec("final.norm", D, 1.0)
    for i, lc in enumerate(cfg["layers"]):
        p, mc = f"l{i}.", lc["mixer"]
        H, G, dk, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        vec(p + "norm1", D, 1.0)
        for nm, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
            mat(p + "mix." + nm, rows, D)
            vec(p + "mix." + nm + ".b", rows, 0.0, 0.3)
        if lc["type"] == "attention":
            vec(p + "mix.q.norm", dk, 1.0, 0.2)
            vec(p + "mix.k.norm", dk, 1.0, 0.2)
            w[p + "mix.talk"] = torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)
        else:
            vec(p + "mix.r1", H, 0.6, 0.3)
            w[p + "mix.r2"] = 0.2 + torch.rand(H, generator=g)
            mat(p + "mix.g", H, D)
        mat(p + "mix.o", D, H * dv)
        fc = lc.get("mlp")
        if fc is None:
            continue
        vec(p + "norm2", D, 1.0)
        if fc["kind"] == "dense":
            mat(p + "mlp.up", fc["ff"], D)
            mat(p + "mlp.down", D, fc["ff"])
        else:
            ff = fc["expert"]["ff"]
            mat(p + "mlp.router", fc["router"]["experts"], D)
            for e in range(fc["router"]["experts"]):
                mat(f"{p}mlp.e{e}.gate", ff, D)
                mat(f"{p}mlp.e{e}.up", ff, D)
                mat(f"{p}mlp.e{e}.down", D, ff)
    return {k: v.to(torch.bfloat16).float() for k, v in w.items()}
