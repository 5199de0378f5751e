"""A plain float64 implementation of the Nukizen design, written from its equations: whole sequences, no cache, no
batching, one function per mechanism.  It shares no code with the package; the tests compare the engine with it.

``tensors``: checkpoint name -> tensor; ``config``: the config.json dictionary.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def silu(z):
    return z * torch.sigmoid(z)


# ----------------------------------------------------------------------------- positions
def rotary_frequencies(rot):
    """(frequency of every pair [dims / 2], factor on cos and sin)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn(t):     # the pair index whose wave makes t turns over the original length
        return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turn(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, rot):
    """x [T, heads, dim]: pairs (i, i + dims / 2) of the first dims dimensions turn by position * frequency."""
    if not rot or not rot.get("dims"):
        return x
    dims = int(rot["dims"])
    half = dims // 2
    f, m = rotary_frequencies(rot)
    ang = torch.arange(x.shape[0], dtype=F64)[:, None] * f[None, :]
    c, s = (torch.cos(ang) * m)[:, None, :], (torch.sin(ang) * m)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], -1)


def visible(T, mask):
    """[T, T] bool: query i sees key j."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if mask and mask.get("size"):
        n = int(mask["size"])
        ok = ok & (i // n == j // n)
    return ok


# ----------------------------------------------------------------------------- mixers
def project_kv(h, m, w, eps):
    """Rotated keys [T, G, dim] and values [T, G, vdim] of an attention mixer that has projections of its own."""
    T = h.shape[0]
    G, D, V = int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    k = h @ w("k").T
    if w("k.norm", None) is not None:
        k = rms_unit(k, eps) * w("k.norm")
    return rotate(k.view(T, G, D), m.get("rot")), (h @ w("v").T).view(T, G, V)


def attention(h, m, w, eps, kv=None):
    """Softmax attention of one mixer; ``kv``: keys and values of another layer to use instead of own ones."""
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = h @ w("q").T
    if w("q.norm", None) is not None:
        q = rms_unit(q, eps) * w("q.norm")
    q = rotate(q.view(T, H, D), m.get("rot"))
    k, v = kv if kv is not None else project_kv(h, m, w, eps)
    ok = visible(T, m.get("mask"))
    out = torch.zeros(T, H, V, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * float(m["scale"])
        if m.get("softcap"):
            cap = float(m["softcap"])
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~ok, -math.inf)
        e = torch.exp(s - s.max(-1, keepdim=True).values)
        den = e.sum(-1, keepdim=True)
        if w("sink", None) is not None:
            den = den + torch.exp(w("sink")[hd] - s.max(-1, keepdim=True).values)
        out[:, hd] = (e / den) @ v[:, g]
    if w("g", None) is not None:
        out = out * torch.sigmoid(h @ w("g").T)[:, :, None]
    return out.reshape(T, H * V) @ w("o").T


def causal_conv(x, taps, bias=None):
    """x [T, C], taps [C, n]: y_t = sum_j taps[:, n - 1 - j] x_(t - j), zeros before the start."""
    T, C = x.shape
    n = taps.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for j in range(n):
        y[j:] += taps[:, n - 1 - j] * x[:T - j]
    return y if bias is None else y + bias


def rglru(h, m, w):
    T = h.shape[0]
    C, B = int(m["width"]), int(m["blocks"])
    y = gelu_tanh(h @ w("y").T + w("y.b"))
    u = causal_conv(h @ w("x").T + w("x.b"), w("conv"), w("conv.b"))
    ub = u.view(T, B, C // B)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w("ra")) + w("ra.b")).reshape(T, C)
    i = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w("ri")) + w("ri.b")).reshape(T, C)
    a = torch.exp(-8.0 * r * softplus(w("lam")))
    S = torch.zeros(C, dtype=F64)
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return (out * y) @ w("o").T


def delta_rule(h, m, w, eps):
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(causal_conv(h @ w("q").T, w("q.conv"))).view(T, G, D)
    k = silu(causal_conv(h @ w("k").T, w("k.conv"))).view(T, G, D)
    v = silu(causal_conv(h @ w("v").T, w("v.conv"))).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w("b").T)
    decay = torch.exp(-torch.exp(w("A_log")) * softplus(h @ w("a").T + w("dt_bias")))
    out = torch.zeros(T, H, V, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(D, V, dtype=F64)
        for t in range(T):
            S = decay[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, hd] = S.T @ q[t, g]
    out = rms_unit(out, eps) * w("norm") * silu(h @ w("g").T).view(T, H, V)
    return out.reshape(T, H * V) @ w("o").T


def gated_ff(h, w):
    return (torch.relu(h @ w("gate").T) * (h @ w("up").T)) @ w("down").T


# ----------------------------------------------------------------------------- model
def forward(tensors, config, tokens):
    """(logits [T, vocab], the residual stream after every layer [layers, T, width]), float64."""
    eps = float(config["norm"]["eps"])

    def scope(prefix):
        def w(name, *default):
            t = tensors.get(prefix + name)
            if t is None:
                if default:
                    return default[0]
                raise KeyError(prefix + name)
            return t.to(F64)
        return w

    x = tensors["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)]
    kv = {}
    after = []
    for i, L in enumerate(config["layers"]):
        h = rms_unit(x, eps) * tensors[f"l{i}.norm1"].to(F64)
        m, w = L["mixer"], scope(f"l{i}.mix.")
        if L["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kv[i] = project_kv(h, m, w, eps)
            y = attention(h, m, w, eps, kv[i if src is None else int(src)])
        elif L["type"] == "rglru":
            y = rglru(h, m, w)
        elif L["type"] == "parallel":
            left = attention(h, m["left"], scope(f"l{i}.mix.left."), eps)
            right = delta_rule(h, m["right"], scope(f"l{i}.mix.right."), eps)
            y = 0.5 * (rms_unit(left, eps) * w("left.out") + rms_unit(right, eps) * w("right.out"))
        else:
            raise ValueError(L["type"])
        if L.get("mlp"):
            y = y + gated_ff(h, scope(f"l{i}.mlp."))
        x = x + y
        after.append(x)
    z = (rms_unit(x, eps) * tensors["final.norm"].to(F64)) @ tensors["head"].to(F64).T
    cap = config.get("logit_softcap")
    if cap:
        z = float(cap) * torch.tanh(z / float(cap))
    return z, torch.stack(after)


def greedy(tensors, config, tokens, n):
    """n tokens generated greedily after ``tokens`` (the whole sequence is run again for every token)."""
    toks = list(tokens)
    out = []
    for _ in range(n):
        z, _ = forward(tensors, config, toks)
        out.append(int(torch.argmax(z[-1])))
        toks.append(out[-1])
    return out
