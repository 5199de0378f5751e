"""A plain float64 implementation of the Semanex design, written from its equations: whole sequences, no cache, no
batching, one function per mechanism.  It shares no code with the package; the tests compare the engine with it.

``tensors``: checkpoint name -> tensor; ``config``: the config.json dictionary.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def silu(z):
    return z * torch.sigmoid(z)


def causal_conv(x, taps, bias=None):
    """x [T, C], taps [C, n]: y_t = sum_j taps[:, j] x_(t - n + 1 + j), zeros before the start."""
    T, C = x.shape
    n = taps.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for j in range(n):
        back = n - 1 - j
        if back < T:
            y[back:] += taps[:, j] * x[:T - back]
    return y if bias is None else y + bias


def rotate_pairs(x, rot):
    """x [T, heads, dim]: the pairs (2i, 2i + 1) of the first ``dims`` dimensions turn by position * base^(-2i/dims)."""
    if not rot or not rot.get("dims"):
        return x
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    ang = torch.arange(x.shape[0], dtype=F64)[:, None] * (base ** (-2.0 * i / dims))[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def softmax_rows(s, sink=None):
    """Causal softmax over the rows of s [T, T]; ``sink``: one more term e^sink in every denominator."""
    T = s.shape[0]
    s = s.masked_fill(torch.arange(T)[None, :] > torch.arange(T)[:, None], -math.inf)
    mx = s.max(-1, keepdim=True).values
    if sink is not None:
        mx = torch.maximum(mx, sink.reshape(1, 1))
    e = torch.exp(s - mx)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink - mx)
    return e / den


# ----------------------------------------------------------------------------- mixers
def latent_attention(h, m, w, eps):
    """Keys and values are up-projections of one normed low-rank row per token; one rotated key part is shared by the
    heads; queries come from a normed low-rank row as well."""
    T = h.shape[0]
    H, D, R, V, C = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    rot = m["rot"]
    cq = rms_unit(h @ w("dq").T, eps) * w("dq.norm")
    q = (cq @ w("uq").T).view(T, H, D + R)
    qn, qr = q[..., :D], rotate_pairs(q[..., D:], rot)
    dkv = h @ w("dkv").T
    c = rms_unit(dkv[:, :C], eps) * w("dkv.norm")
    kr = rotate_pairs(dkv[:, C:].view(T, 1, R), rot)[:, 0]
    kn = (c @ w("uk").T).view(T, H, D)
    v = (c @ w("uv").T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=F64)
    for hd in range(H):
        s = (qn[:, hd] @ kn[:, hd].T + qr[:, hd] @ kr.T) * float(m["scale"])
        out[:, hd] = softmax_rows(s, w("sink")[hd]) @ v[:, hd]
    y = out.reshape(T, H * V) * torch.sigmoid(h @ w("g").T)
    return y @ w("o").T


def capped_attention(h, m, w, eps):
    """Grouped-query attention without positions: per-head normed queries and keys, capped scores, gated output."""
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = rms_unit((h @ w("q").T).view(T, H, D), eps) * w("q.norm")
    k = rms_unit((h @ w("k").T).view(T, G, D), eps) * w("k.norm")
    v = (h @ w("v").T).view(T, G, V)
    cap = float(m["softcap"])
    out = torch.zeros(T, H, V, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * float(m["scale"])
        out[:, hd] = softmax_rows(cap * torch.tanh(s / cap)) @ v[:, g]
    y = out.reshape(T, H * V) * torch.sigmoid(h @ w("g").T)
    return y @ w("o").T


def ssd(h, m, w, eps):
    """State-space recurrence with a scalar decay per head and token."""
    T = h.shape[0]
    H, V, N, G, ng = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["norm_groups"])
    inner = H * V
    p = h @ w("in").T
    z, xbc, dt = p[:, :inner], p[:, inner:2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w("conv"), w("conv.b")))
    x = xbc[:, :inner].view(T, H, V)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w("dt_bias"))
    decay = torch.exp(-torch.exp(w("A_log")) * dt)                       # [T, H]
    y = torch.zeros(T, H, V, dtype=F64)
    S = torch.zeros(H, N, V, dtype=F64)
    of = torch.arange(H) // (H // G)                                     # the group of every head
    for t in range(T):
        S = decay[t, :, None, None] * S + dt[t, :, None, None] * B[t, of][:, :, None] * x[t][:, None, :]
        y[t] = torch.einsum("hnv,hn->hv", S, Cm[t, of]) + w("D")[:, None] * x[t]
    y = y.reshape(T, inner) * silu(z)
    y = rms_unit(y.view(T, ng, inner // ng), eps).reshape(T, inner) * w("norm")
    return y @ w("o").T


def mixer(kind, h, m, w, eps):
    if kind == "latent_attention":
        return latent_attention(h, m, w, eps)
    if kind == "parallel":
        left = capped_attention(h, m["left"], lambda n, *d: w("left." + n, *d), eps)
        right = ssd(h, m["right"], lambda n, *d: w("right." + n, *d), eps)
        return float(m["left_scale"]) * left + float(m["right_scale"]) * right
    raise ValueError(kind)


# ----------------------------------------------------------------------------- model
def forward(tensors, config, tokens, after=None):
    """Logits [T, vocab] of one sequence; ``after`` (a list) receives the residual stream after every layer."""
    get = lambda name: tensors[name].to(F64)
    eps = float(config["norm"]["eps"])
    alpha = float(config["postln_alpha"])
    x = get("embed")[torch.as_tensor(tokens, dtype=torch.long)] * float(config["embedding"]["scale"])
    for i, L in enumerate(config["layers"]):
        p = f"l{i}."

        def w(name, *default, p=p):
            if default and p + "mix." + name not in tensors:
                return default[0]
            return get(p + "mix." + name)

        h = x
        if p + "canon1" in tensors:
            h = h + causal_conv(h, get(p + "canon1"))
        x = rms_unit(alpha * x + mixer(L["type"], h, L["mixer"], w, eps), eps) * get(p + "norm1")
        if L.get("mlp"):
            f = gelu_erf(x @ get(p + "mlp.up").T) @ get(p + "mlp.down").T
            x = rms_unit(alpha * x + f, eps) * get(p + "norm2")
        elif p + "norm2" in tensors:                                       # a second norm without a feed-forward
            x = rms_unit(alpha * x, eps) * get(p + "norm2")
        if after is not None:
            after.append(x.clone())
    x = rms_unit(x, eps) * get("final.norm")
    return x @ get("head").T


def greedy(tensors, config, prompt, n):
    """n tokens, each the arg-max of the last position's logits (lowest index on a tie)."""
    toks = list(prompt)
    out = []
    for _ in range(n):
        t = int(torch.argmax(forward(tensors, config, toks)[-1]))
        out.append(t)
        toks.append(t)
    return out
