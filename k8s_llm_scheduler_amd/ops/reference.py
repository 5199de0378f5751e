"""Plain-PyTorch fp32 reference implementations of every HIP kernel.

They define the semantics the kernels are tested against (T3 numerics tests compare a kernel
with the function of the same name here) and they run the model on CPU for the multi-process
``gloo`` tests (TP=k vs TP=1).  They are never used for CUDA tensors: the wrappers in
``ops/__init__.py`` refuse to fall back on a GPU.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch

U32 = 0xFFFFFFFF


# ----------------------------------------------------------------------------- hashing / RNG
def _fmix32(h: torch.Tensor) -> torch.Tensor:
    h = h & U32
    h = h ^ (h >> 16)
    h = (h * 0x85EBCA6B) & U32
    h = h ^ (h >> 13)
    h = (h * 0xC2B2AE35) & U32
    h = h ^ (h >> 16)
    return h


def hash3(a, b, c: torch.Tensor) -> torch.Tensor:
    """Same bits as common.h hash3 (int64 tensors holding uint32 values)."""
    c = torch.as_tensor(c, dtype=torch.int64)
    b = torch.as_tensor(b, dtype=torch.int64, device=c.device)
    a = torch.as_tensor(a, dtype=torch.int64, device=c.device)
    inner = _fmix32((c + 0x7F4A7C15) & U32)
    mid = _fmix32((((b + 0x9E3779B9) & U32) ^ inner) & U32)
    return _fmix32((a ^ mid) & U32)


def u01(h: torch.Tensor) -> torch.Tensor:
    return ((h >> 8).to(torch.float64) + 0.5) * (1.0 / 16777216.0)


def hash_init(rows: int, cols: int, gcols: int, row0: int, col0: int, seed: int, tensor_id: int,
              scale: float, shift: float, dtype=torch.bfloat16, device="cpu") -> torch.Tensor:
    r = torch.arange(rows, dtype=torch.int64, device=device).unsqueeze(1) + row0
    c = torch.arange(cols, dtype=torch.int64, device=device).unsqueeze(0) + col0
    flat = (r * gcols + c) & U32
    u = u01(hash3(seed, tensor_id, flat)).to(torch.float32)
    return ((2.0 * u - 1.0) * scale + shift).to(dtype)


# ----------------------------------------------------------------------------- layers
def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float,
            residual: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    if residual is not None:
        r = (x.float() + residual.float()).to(x.dtype)
        residual.copy_(r)
        x = r
    xf = x.float()
    out = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return out.to(x.dtype), residual


def rope_table(head_dim: int, max_pos: int, theta: float, scaling: Optional[dict] = None) -> torch.Tensor:
    """[max_pos, head_dim] fp32: cos in [:, :D/2], sin in [:, D/2:] (llama3, linear or yarn scaling if given; linear:
    every frequency divided by ``factor``; yarn: the frequencies between the pairs that make ``fast`` and ``slow``
    turns over ``original`` positions go over linearly from unscaled to divided by ``factor``, and cos and sin are
    multiplied by 0.1 ln(factor) + 1).  Angles are formed in float64."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    mag = 1.0
    if scaling and scaling.get("rope_type", scaling.get("type")) == "yarn":
        factor, orig = float(scaling["factor"]), float(scaling["original"])
        turn = lambda t: head_dim * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(theta))
        lo = max(math.floor(turn(float(scaling["fast"]))), 0)
        hi = min(math.ceil(turn(float(scaling["slow"]))), head_dim - 1)
        ramp = ((torch.arange(head_dim // 2, dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        inv = inv / factor * ramp + inv * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    if scaling and scaling.get("rope_type", scaling.get("type")) == "linear":
        inv = inv / float(scaling["factor"])
    if scaling and scaling.get("rope_type", scaling.get("type")) == "llama3":
        factor = scaling["factor"]
        lo, hi = scaling["low_freq_factor"], scaling["high_freq_factor"]
        old = scaling["original_max_position_embeddings"]
        lo_wl, hi_wl = old / lo, old / hi
        wl = 2 * math.pi / inv
        inv_l = torch.where(wl > lo_wl, inv / factor, inv)
        smooth = (old / wl - lo) / (hi - lo)
        smoothed = (1 - smooth) * inv_l / factor + smooth * inv_l
        medium = (wl >= hi_wl) & (wl <= lo_wl)
        inv = torch.where(medium, smoothed, inv_l)
    pos = torch.arange(max_pos, dtype=torch.float64)
    f = torch.outer(pos, inv)
    return (torch.cat([f.cos(), f.sin()], dim=-1) * mag).float()


def _rotate(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    # x [..., D] fp32, cs [..., D] (cos | sin)
    h = x.shape[-1] // 2
    c, s = cs[..., :h], cs[..., h:]
    x1, x2 = x[..., :h], x[..., h:]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)


def rope_kv_write(qkv: torch.Tensor, cos_sin: torch.Tensor, positions: torch.Tensor, slot_mapping: torch.Tensor,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, nq: int, nkv: int, D: int) -> torch.Tensor:
    T = qkv.shape[0]
    x = qkv.view(T, nq + 2 * nkv, D).float()
    cs = cos_sin[positions.long()].unsqueeze(1)
    q = _rotate(x[:, :nq], cs).to(qkv.dtype)
    k = _rotate(x[:, nq:nq + nkv], cs).to(qkv.dtype)
    v = x[:, nq + nkv:].to(qkv.dtype)
    keep = slot_mapping >= 0
    sl = slot_mapping[keep].long()
    k_cache.view(-1, nkv, D)[sl] = k[keep]
    v_cache.view(-1, nkv, D)[sl] = v[keep]
    return q.contiguous()


def decode_positions(context_lens: torch.Tensor, block_tables: torch.Tensor, block_size: int):
    pos = (context_lens - 1).clamp(min=0).long()
    blk = block_tables.long().gather(1, (pos // block_size).unsqueeze(1)).squeeze(1)
    slots = blk * block_size + pos % block_size
    slots = torch.where(context_lens > 0, slots, torch.full_like(slots, -1))
    return pos.int(), slots.int()


def _gather_kv(cache: torch.Tensor, bt_row: torch.Tensor, n: int, block_size: int, kvh: int) -> torch.Tensor:
    idx = torch.arange(n, device=cache.device)
    slots = bt_row.long()[idx // block_size] * block_size + idx % block_size
    return cache.view(-1, cache.shape[-2], cache.shape[-1])[slots, kvh].float()   # [n, D]


def paged_decode_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                           context_lens: torch.Tensor, scale: float, block_size: int) -> torch.Tensor:
    B, nq, D = q.shape
    nkv = k_cache.shape[-2]
    G = nq // nkv
    out = torch.zeros_like(q)
    for b in range(B):
        n = int(context_lens[b])
        if n <= 0:
            continue
        for kvh in range(nkv):
            K = _gather_kv(k_cache, block_tables[b], n, block_size, kvh)
            V = _gather_kv(v_cache, block_tables[b], n, block_size, kvh)
            qq = q[b, kvh * G:(kvh + 1) * G].float()
            p = torch.softmax(qq @ K.T * scale, dim=-1)
            out[b, kvh * G:(kvh + 1) * G] = (p @ V).to(q.dtype)
    return out


def paged_prefill_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, cu_q: torch.Tensor,
                            context_lens: torch.Tensor, block_tables: torch.Tensor, scale: float,
                            block_size: int) -> torch.Tensor:
    T, nq, D = q.shape
    nkv = k_cache.shape[-2]
    G = nq // nkv
    out = torch.zeros_like(q)
    cu = cu_q.tolist()
    for s in range(len(cu) - 1):
        q0, q1 = cu[s], cu[s + 1]
        qlen = q1 - q0
        if qlen == 0:
            continue
        ctx = int(context_lens[s])
        qpos = torch.arange(ctx - qlen, ctx, device=q.device)
        kpos = torch.arange(ctx, device=q.device)
        mask = kpos[None, :] <= qpos[:, None]
        for kvh in range(nkv):
            K = _gather_kv(k_cache, block_tables[s], ctx, block_size, kvh)
            V = _gather_kv(v_cache, block_tables[s], ctx, block_size, kvh)
            for g in range(G):
                h = kvh * G + g
                sc = (q[q0:q1, h].float() @ K.T) * scale
                sc = sc.masked_fill(~mask, float("-inf"))
                out[q0:q1, h] = (torch.softmax(sc, -1) @ V).to(q.dtype)
    return out


FP8_MAX = 448.0


def quantize_fp8(w: torch.Tensor):
    """Row-scaled OCP e4m3: returns (q [N, K] uint8 bit patterns, scale [N] fp32) with
    w ~= e4m3(q) * scale[:, None] (same recipe as fp8.hip)."""
    wf = w.float()
    amax = wf.abs().amax(dim=1)
    scale = torch.where(amax > 0, amax / FP8_MAX, torch.ones_like(amax))
    q = (wf * (1.0 / scale)[:, None]).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q.view(torch.uint8), scale


def dequant_fp8(q: torch.Tensor, scale: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    return (q.view(torch.float8_e4m3fn).float() * scale.float()[:, None]).to(dtype)


MX_BLOCK = 32


def quantize_mx(x: torch.Tensor):
    """OCP MX e4m3 (fp8.hip quantize_act_mx_kernel): every 32 consecutive values of a row share the E8M0 scale
    e = the smallest power of two >= max|block| / 448 (byte 127 + log2; 127 for an all-zero block, clamped to
    [1, 253]).  Returns (q [M, K] uint8 e4m3 bit patterns, e [M, K / 32] uint8)."""
    M, K = x.shape
    xf = x.float().reshape(M, K // MX_BLOCK, MX_BLOCK)
    amax = xf.abs().amax(dim=-1)
    bits = (amax * (1.0 / FP8_MAX)).contiguous().view(torch.int32)
    e = (bits >> 23) + ((bits & 0x7FFFFF) != 0).to(torch.int32)
    e = torch.where(amax == 0, torch.full_like(e, 127), e).clamp(1, 253)
    inv = torch.ldexp(torch.ones_like(amax), (127 - e).float())
    q = (xf * inv[..., None]).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q.view(torch.uint8).reshape(M, K), e.to(torch.uint8)


def mx_scales_to_device_layout(e: torch.Tensor) -> torch.Tensor:
    """[M, K / 32] E8M0 -> the kernels' layout [K / 128, M, 4] (csrc/kernels/common.h mx_scale_off)."""
    M, KB = e.shape
    return e.reshape(M, KB // 4, 4).permute(1, 0, 2).contiguous()


def mx_scales_from_device_layout(e: torch.Tensor) -> torch.Tensor:
    """[K / 128, M, 4] -> [M, K / 32]."""
    KT, M, _ = e.shape
    return e.permute(1, 0, 2).reshape(M, KT * 4)


def dequant_mx(q: torch.Tensor, e: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    """``e``: [M, K / 32] (logical) or the kernels' [K / 128, M, 4]."""
    if e.dim() == 3:
        e = mx_scales_from_device_layout(e)
    M, K = q.shape
    s = torch.ldexp(torch.ones(e.shape, dtype=torch.float32, device=q.device), e.float() - 127)
    v = q.view(torch.float8_e4m3fn).float().reshape(M, K // MX_BLOCK, MX_BLOCK) * s[..., None]
    return v.reshape(M, K).to(dtype)


def _wf(w) -> torch.Tensor:
    """fp32 view of a weight: a plain tensor or an ops.Fp8Weight (duck-typed: .q / .scale)."""
    if hasattr(w, "scale") and hasattr(w, "q"):
        return dequant_fp8(w.q, w.scale)
    return w.float()


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype=None) -> torch.Tensor:
    y = x.float() @ _wf(w).T
    return y.to(out_dtype or x.dtype)


def silu_mul(gu: torch.Tensor) -> torch.Tensor:
    I = gu.shape[-1] // 2
    g, u = gu[..., :I].float(), gu[..., I:].float()
    return (torch.nn.functional.silu(g) * u).to(gu.dtype)


def linear_swiglu(x: torch.Tensor, w_gate_up: torch.Tensor) -> torch.Tensor:
    gu = x.float() @ _wf(w_gate_up).T
    I = gu.shape[-1] // 2
    return (torch.nn.functional.silu(gu[..., :I]) * gu[..., I:]).to(x.dtype)


def embedding(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    return table[ids.long().clamp(0, table.shape[0] - 1)]


def _ord_key(l: torch.Tensor) -> torch.Tensor:
    u = l.float().contiguous().view(torch.int32).to(torch.int64) & U32
    neg = (u & 0x80000000) != 0
    return torch.where(neg, (~u) & U32, u | 0x80000000)


NUC_FS = float(np.float32(65536.0 / 28.0))   # sampler.hip NUC_FS


def nucleus_fine_mass(l: torch.Tensor, M: float, T: float):
    """Per token of an fp32 logits row: fine bin f = floor((M - l) / T * 65536/28) (65536 = none beyond 28) and the
    integer mass floor(exp((l - M) / T) * 2^40) (0 for none), as sampler.hip computes them for row max M."""
    l = l.float().cpu()
    invT = torch.tensor(1.0, dtype=torch.float32) / torch.tensor(T, dtype=torch.float32)
    M = torch.tensor(M, dtype=torch.float32)
    x = ((M - l) * invT) * torch.tensor(NUC_FS, dtype=torch.float32)
    valid = x < 65536.0
    f = torch.where(valid, x, torch.zeros_like(x)).to(torch.int64)
    f = torch.where(valid, f, torch.full_like(f, 65536))
    mass = (torch.exp((l - M) * invT) * 1099511627776.0).to(torch.int64)
    return f, torch.where(valid, mass, torch.zeros_like(mass))


def nucleus_coarse_hist(f: torch.Tensor, mass: torch.Tensor) -> torch.Tensor:
    return torch.zeros(257, dtype=torch.int64).index_add_(0, torch.clamp(f >> 8, max=256), mass)[:256]


def nucleus_fine_hist(f: torch.Tensor, mass: torch.Tensor, bstar: int) -> torch.Tensor:
    inb = (f >> 8) == bstar
    return torch.zeros(256, dtype=torch.int64).index_add_(0, (f & 255)[inb], mass[inb])


def nucleus_pick(hist: torch.Tensor, target: int, above: int = 0):
    """(first bin where above + the cumulative mass reaches target -- 255 if none --, mass before that bin)."""
    cum = above + torch.cumsum(hist, 0)
    hit = ((cum >= target) & (hist != 0)).nonzero()
    b = int(hit[0]) if len(hit) else 255
    return b, int(cum[b] - hist[b])


def nucleus_target(coarse: torch.Tensor, P: float) -> int:
    return int(float(int(coarse.sum())) * float(np.float32(P)))


def nucleus_mask(l: torch.Tensor, T: float, P: float) -> torch.Tensor:
    """The nucleus of sampler.hip for one row of fp32 logits: fine bin f = floor((M - l) / T * 65536/28)
    (none beyond 28), mass = floor(exp((l - M) / T) * 2^40) as an integer, target = floor(Z * P); the
    smallest f* with mass{f <= f*} >= target is found coarse (f >> 8) then fine (f & 255); keep f <= f*."""
    l = l.float().cpu()
    f, mass = nucleus_fine_mass(l, float(l.max()), T)
    coarse = nucleus_coarse_hist(f, mass)
    target = nucleus_target(coarse, P)
    bstar, above = nucleus_pick(coarse, target)
    fstar = bstar * 256 + nucleus_pick(nucleus_fine_hist(f, mass, bstar), target, above)[0]
    return f <= fstar


def sample_key(l: torch.Tensor, T: float, seed: int, ctr: int, id0: int, keep=None):
    """(score, global id) of the best token of one logits row whose token ids start at ``id0`` (a vocab shard):
    greedy (T <= 0) or Gumbel-max over ``keep``; ties to the lowest id, like sampler.hip's packed keys.  None if
    ``keep`` leaves no token."""
    l = l.float()
    vid = torch.arange(l.numel(), dtype=torch.int64, device=l.device) + id0
    if T <= 0:
        score = l
    else:
        u = u01(hash3(int(seed), int(ctr), vid)).float()
        score = l / T - torch.log(-torch.log(u))
    if keep is not None:
        score = torch.where(keep.to(score.device), score, torch.full_like(score, float("-inf")))
        if not bool(keep.any()):
            return None
    m = score.max()
    i = int((score == m).nonzero()[0])
    return float(m), int(vid[i])


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, seeds: torch.Tensor,
           counter: torch.Tensor) -> torch.Tensor:
    """logits [B, V] fp32 -> tokens [B] int32, bit-compatible with sampler.hip (up to fp rounding
    of the Gumbel scores and of the per-token masses at a nucleus boundary)."""
    B, V = logits.shape
    out = torch.empty(B, dtype=torch.int32, device=logits.device)
    for b in range(B):
        l = logits[b].float()
        T, P = float(temperature[b]), float(top_p[b])
        keep = nucleus_mask(l, T, P) if T > 0 and P < 1.0 else None
        out[b] = sample_key(l, T, int(seeds[b]), int(counter[b]), 0, keep)[1]
    return out


def sample_vocab_parallel(local: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, seeds: torch.Tensor,
                          counter: torch.Tensor, rank: int, gather) -> torch.Tensor:
    """Vocab-parallel form of :func:`sample` (sampler.hip's TP path, on CPU): ``local`` [B, Vs] is this rank's vocab
    shard (global ids rank * Vs ..), ``gather(t)`` all-gathers a tensor over the ranks ([world, *t.shape]).  Nucleus
    rows combine the row max and the two integer bin histograms over the ranks, then every rank's best (score, id)
    is gathered and the best of them taken: the tokens of :func:`sample` over the concatenated shards."""
    B, Vs = local.shape
    id0 = rank * Vs
    nuc = [float(temperature[b]) > 0 and float(top_p[b]) < 1.0 for b in range(B)]
    keep = [None] * B
    if any(nuc):
        M = gather(local.float().max(dim=1).values).max(dim=0).values
        fm = [nucleus_fine_mass(local[b], float(M[b]), float(temperature[b])) if nuc[b] else None for b in range(B)]
        z = torch.zeros(256, dtype=torch.int64)
        coarse = gather(torch.stack([nucleus_coarse_hist(*fm[b]) if nuc[b] else z for b in range(B)])).sum(0)
        sel = {}
        for b in range(B):
            if nuc[b]:
                target = nucleus_target(coarse[b], float(top_p[b]))
                sel[b] = (target,) + nucleus_pick(coarse[b], target)
        fine = gather(torch.stack([nucleus_fine_hist(*fm[b], sel[b][1]) if nuc[b] else z for b in range(B)])).sum(0)
        for b in range(B):
            if nuc[b]:
                target, bstar, above = sel[b]
                keep[b] = fm[b][0] <= bstar * 256 + nucleus_pick(fine[b], target, above)[0]
    best = torch.full((B, 2), float("-inf"), dtype=torch.float64)
    for b in range(B):
        k = sample_key(local[b], float(temperature[b]), int(seeds[b]), int(counter[b]), id0, keep[b])
        if k is not None:
            best[b, 0], best[b, 1] = k[0], -k[1]
    g = gather(best)                                  # [world, B, 2]: (score, -id); max = best score, lowest id
    out = torch.empty(B, dtype=torch.int32)
    for b in range(B):
        cand = [tuple(g[r, b].tolist()) for r in range(g.shape[0])]
        out[b] = int(-max(cand)[1])
    return out


# ----------------------------------------------------------------------------- device-side stop detection (oracle)
def token_stop_classes(texts, eos_ids, vocab: int) -> torch.Tensor:
    """Per-token class words of sampler.hip's stop detection, [vocab, 2] int32, from each token's decoded text
    (``texts[i]`` for token i; missing / special tokens: no braces).  x = eos | net brace delta << 8 | min running
    depth relative to the entry << 16; y = has '{' | depth at the end counted from the token's first '{' << 8 |
    min depth after that '{' << 16 (int8 fields)."""
    def i8(v: int) -> int:
        return max(-128, min(127, v)) & 0xFF

    out = torch.zeros(vocab, 2, dtype=torch.int32)
    xs, ys = [0] * vocab, [0] * vocab
    for i, t in enumerate(texts[:vocab]):
        if not t or ("{" not in t and "}" not in t):
            continue
        d = m = 0
        for ch in t:
            if ch == "{":
                d += 1
            elif ch == "}":
                d -= 1
                m = min(m, d)
        xs[i] = (i8(d) << 8) | (i8(m) << 16)
        k = t.find("{")
        if k >= 0:
            d2, m2 = 1, 1
            for ch in t[k + 1:]:
                if ch == "{":
                    d2 += 1
                elif ch == "}":
                    d2 -= 1
                    m2 = min(m2, d2)
            ys[i] = 1 | (i8(d2) << 8) | (i8(m2) << 16)
    for e in eos_ids:
        if 0 <= e < vocab:
            xs[e] |= 1
    out[:, 0] = torch.tensor(xs, dtype=torch.int64).to(torch.int32)
    out[:, 1] = torch.tensor(ys, dtype=torch.int64).to(torch.int32)
    return out


def _i8(v: int) -> int:
    v &= 0xFF
    return v - 256 if v >= 128 else v


def json_step(state: int, cx: int, cy: int):
    """(new state, closed) -- sampler.hip json_step."""
    if state >= 1:
        amin, adelta = _i8(cx >> 16), _i8(cx >> 8)
        if state + amin <= 0:
            return 0, True
        return state + adelta, False
    if cy & 1:
        bmin, bend = _i8(cy >> 16), _i8(cy >> 8)
        if bmin <= 0:
            return 0, True
        return bend, False
    return state, False


def write_token_stop(s: int, tok: int, tokens, ctx_inc, hist, steps, stop) -> None:
    """sampler.hip write_token with stop detection, for state slot s (CPU reference of the decode graphs)."""
    st = int(steps[s])
    fin = False
    cls, cfg = stop["cls"], int(stop["cfg"][s])
    max_new = cfg >> 8
    state = int(stop["json"][s])
    if state == -2:
        t0 = int(hist[s, 0])
        state = -1
        if (cfg & 1) and (int(cls[t0, 0]) & 1):
            fin = True
        elif cfg & 2:
            state, fin = json_step(state, int(cls[t0, 0]), int(cls[t0, 1]))
        if not fin and st >= max_new:
            fin = True
        if fin:
            stop["json"][s] = state
            ctx_inc[s] = 0
            stop["done"][s] = 1
            return
    forced, flen = stop.get("forced"), stop.get("forced_len")
    if forced is not None and int(flen[s]) >= 0:
        tok = int(forced[s, st]) if st < int(flen[s]) else int(stop["eos_tok"])
    cx, cy = int(cls[tok, 0]), int(cls[tok, 1])
    if (cfg & 1) and (cx & 1):
        fin = True
    else:
        if cfg & 2:
            state, fin = json_step(state, cx, cy)
        if st + 1 >= max_new:
            fin = True
    stop["json"][s] = state
    tokens[s] = tok
    if st < hist.shape[1]:
        hist[s, st] = tok
    steps[s] = st + 1
    ctx_inc[s] = 0 if fin else int(ctx_inc[s]) + 1
    if fin:
        stop["done"][s] = 1


# ----------------------------------------------------------------------------- fp32 residual stream, gated activations
ACT_GELU_TANH, ACT_SWISH_CLAMP, ACT_TANH, ACT_SILU, ACT_GELU_ERF, ACT_RELU, ACT_SOFTCAP = 0, 1, 2, 3, 4, 5, 6


def embed_rows(ids: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """fp32 rows of the embedding table times ``scale`` (the residual stream starts in fp32)."""
    return table.index_select(0, ids.long()).float() * scale


def resnorm(x: torch.Tensor, branch, mult: float, rowvec, w, offset: float, eps: float, out_dtype, groups: int = 1,
            branch2=None):
    """x (fp32, in place) += mult * (branch + branch2) + rowvec; returns x / sqrt(mean(x^2) + eps) * (offset + w) or
    None, the mean taken over each of ``groups`` equal consecutive parts of a row by itself."""
    if branch is not None and branch2 is not None:
        x.add_((branch.float() + branch2.float()) * mult)
    elif branch is not None:
        x.add_(branch.float() * mult)
    if rowvec is not None:
        x.add_(rowvec.float())
    if w is None:
        return None
    T, W = x.shape
    xg = x.view(T, groups, W // groups)
    y = (xg * torch.rsqrt(xg.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, W) * (offset + w.float())
    return y.to(out_dtype)


def postnorm(x: torch.Tensor, branch, branch2, alpha: float, c1: float, c2: float, gain: float, eps: float, out_dtype):
    """x (fp32, in place) <- v / sqrt(mean(v^2) + eps) * gain with v = alpha x + c1 branch + c2 branch2; returns the new
    rows in ``out_dtype`` (None: nothing)."""
    v = alpha * x
    if branch is not None:
        v = v + c1 * branch.float()
    if branch2 is not None:
        v = v + c2 * branch2.float()
    x.copy_(v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * gain)
    return x.to(out_dtype) if out_dtype is not None else None


GATE_SIGMOID, GATE_SILU = 0, 1


def gate_mul(y: torch.Tensor, gate: torch.Tensor, kind: int) -> torch.Tensor:
    """y * sigmoid(gate), or y * silu(gate), in the gate's type."""
    g = gate.float()
    f = torch.sigmoid(g)
    if kind == GATE_SILU:
        f = f * g
    return (y.float() * f).to(gate.dtype)


def act(x: torch.Tensor, kind: int, limit: float = 0.0, alpha: float = 1.0, row_scale=None, row_map=None) -> torch.Tensor:
    """Gated kinds (ACT_GELU_TANH, ACT_SWISH_CLAMP, ACT_RELU: relu(g) u) take [T, 2F] = [gate | up] and return [T, F];
    ACT_TANH / ACT_SILU / ACT_GELU_ERF / ACT_SOFTCAP (limit tanh(x / limit)) are elementwise and take a factor per row:
    logical row i is row ``row_map[i]`` (or i), its input times ``row_scale[i]``."""
    if kind == ACT_SOFTCAP:
        return (limit * torch.tanh(x.float() / limit)).to(x.dtype)
    if kind in (ACT_TANH, ACT_SILU, ACT_GELU_ERF):
        f = x.float()
        if row_scale is not None:
            sc = row_scale.float()
            if row_map is not None:
                sc = torch.zeros(x.shape[0]).index_copy_(0, row_map.long(), sc)
            f = f * sc.unsqueeze(-1)
        if kind == ACT_GELU_ERF:
            return (0.5 * f * (1.0 + torch.erf(f / math.sqrt(2.0)))).to(x.dtype)
        return (torch.tanh(f) if kind == ACT_TANH else f * torch.sigmoid(f)).to(x.dtype)
    F = x.shape[-1] // 2
    g, u = x[..., :F].float(), x[..., F:].float()
    if kind == ACT_GELU_TANH:
        y = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g * g * g))) * u
    elif kind == ACT_RELU:
        y = torch.relu(g) * u
    else:
        if limit > 0:
            g = g.clamp(max=limit)
            u = u.clamp(-limit, limit)
        y = g * torch.sigmoid(alpha * g) * (u + 1.0)
    return y.to(x.dtype)


def gemm_any(a: torch.Tensor, w: torch.Tensor, out_dtype, a_rows=None, tiles=None, seg=None) -> torch.Tensor:
    """a [M, K] @ w [N, K]^T, or batched a [G, M, K] (any strides) @ w [G, N, K]^T -> [G, M, N]; grouped
    (``seg`` [G + 1] row offsets into the gathered rows ``a[a_rows]``): rows seg[g] .. seg[g + 1] use w[g]."""
    if seg is not None:
        rows = a.index_select(0, a_rows.long()).float() if a_rows is not None else a.float()
        out = torch.zeros(rows.shape[0], w.shape[1], dtype=torch.float32)
        s = seg.tolist()
        for g in range(len(s) - 1):
            if s[g + 1] > s[g]:
                out[s[g]:s[g + 1]] = rows[s[g]:s[g + 1]] @ w[g].float().T
        return out.to(out_dtype)
    return (a.float() @ w.float().transpose(-1, -2)).to(out_dtype)


# ----------------------------------------------------------------------------- recurrent mixer (token shift + wkv)
def token_shift(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor, seq_slots: torch.Tensor,
                positions: torch.Tensor) -> torch.Tensor:
    """out[s, t] = h[t] + (prev[t] - h[t]) * mu[s]; prev is the previous token of the same sequence: h[t - 1]
    inside a portion, the slot's saved row at a portion's start, zeros at position 0.  Rows with position < 0 are
    skipped (zeros).  [n, T, W]."""
    T, W = h.shape
    hf = h.float()
    prev = torch.zeros(T, W)
    cu = cu_q.tolist()
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if b <= a or int(positions[a]) < 0:
            continue
        prev[a + 1:b] = hf[a:b - 1]
        if int(positions[a]) > 0:
            prev[a] = state[int(seq_slots[s])].float()
    out = hf.unsqueeze(0) + (prev - hf).unsqueeze(0) * mu.float().unsqueeze(1)
    return out.to(h.dtype)


def shift_save(state: torch.Tensor, h: torch.Tensor, cu_q: torch.Tensor, seq_slots: torch.Tensor,
               positions: torch.Tensor) -> None:
    cu = cu_q.tolist()
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if b > a and int(positions[a]) >= 0:
            state[int(seq_slots[s])] = h[b - 1]


def wkv_scan(r, k, v, g, z, w0, u, lnw, state, cu_q, seq_slots, positions, H: int, D: int, eps: float, out_dtype):
    """Per head: o_t = (S + diag(u) k_t v_t^T)^T r_t, S <- diag(w_t) S + k_t v_t^T with w = exp(-exp(z + w0));
    the head's o / rms(o) * lnw * silu(g).  ``state`` [slots, H, D, D] fp32 carries S between calls (zero at
    position 0)."""
    T = r.shape[0]
    out = torch.zeros(T, H * D)
    w = torch.exp(-torch.exp(z.float() + w0.float()))
    rf, kf, vf, gf = (t.float().view(T, H, D) for t in (r, k, v, g))
    w = w.view(T, H, D)
    uf = u.float().view(H, D)
    cu = cu_q.tolist()
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if b <= a or int(positions[a]) < 0:
            continue
        slot = int(seq_slots[s])
        S = torch.zeros(H, D, D) if int(positions[a]) == 0 else state[slot].clone()
        for t in range(a, b):
            kv = kf[t].unsqueeze(2) * vf[t].unsqueeze(1)                   # [H, D, D]
            o = torch.einsum("hi,hij->hj", rf[t], S + uf.unsqueeze(2) * kv)
            S = w[t].unsqueeze(2) * S + kv
            o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
            out[t] = o.reshape(-1)
        state[slot] = S
    g2 = gf.reshape(T, H * D)
    return (out * lnw.float() * g2 * torch.sigmoid(g2)).to(out_dtype)


# ----------------------------------------------------------------------------- latent attention
def latent_kv_write(cache, dkv, normw, q, cos_sin, positions, slot_mapping, C: int, R: int, H: int, Dn: int,
                    rot_dims: int, eps: float, interleaved: bool = False) -> None:
    """cache[slot] = [rms(dkv[:C]) * normw | rope(dkv[C:])]; q's rotated part ([T, H, Dn + R], last R of each head)
    is rotated in place (pairs (i, i + rot_dims / 2), or (2i, 2i + 1) when ``interleaved``).  Rows with a negative
    slot are not written."""
    T = dkv.shape[0]
    d = dkv.float()
    c = d[:, :C] * torch.rsqrt(d[:, :C].pow(2).mean(-1, keepdim=True) + eps) * normw.float()
    half = rot_dims // 2
    cs = cos_sin[positions.long().clamp(min=0)]
    cos, sin = cs[:, :half], cs[:, half:]

    def rot(x, cos, sin):
        if interleaved:
            y = x.clone()
            a, b = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
            y[..., 0:rot_dims:2], y[..., 1:rot_dims:2] = a * cos - b * sin, b * cos + a * sin
            return y
        a, b = x[..., :half], x[..., half:rot_dims]
        return torch.cat([a * cos - b * sin, b * cos + a * sin, x[..., rot_dims:]], -1)

    kr = rot(d[:, C:], cos, sin)
    row = torch.cat([c, kr], -1).to(cache.dtype)
    ok = slot_mapping >= 0
    cache[slot_mapping[ok].long()] = row[ok]
    qv = q.view(T, H, Dn + R)
    qv[..., Dn:] = rot(qv[..., Dn:].float(), cos.unsqueeze(1), sin.unsqueeze(1)).to(q.dtype)


def latent_attention(q_abs, q, cache, block_tables, tok_seq, positions, C: int, R: int, H: int, Dn: int,
                     window: int, scale: float, block_size: int, out_dtype, sinks=None):
    """Token t of sequence tok_seq[t] at position p attends the cached rows of positions max(0, p - window + 1) .. p
    (window <= 0: all): score = (q_abs . c + q_rot . k_rot) * scale, softmax (``sinks`` [H]: one more term e^sinks[h]
    in head h's denominator), returns sum p c  [T, H, C]."""
    T = q_abs.shape[0]
    out = torch.zeros(T, H, C)
    qa = q_abs.float().view(T, H, C)
    qr = q.float().view(T, H, Dn + R)[..., Dn:]
    for t in range(T):
        p = int(positions[t])
        if p < 0:
            continue
        lo = 0 if window <= 0 else max(0, p - window + 1)
        js = torch.arange(lo, p + 1)
        bt = block_tables[int(tok_seq[t])].long()
        rows = cache[bt[js // block_size] * block_size + js % block_size].float()
        s = (qa[t] @ rows[:, :C].T + qr[t] @ rows[:, C:].T) * scale
        if sinks is not None:
            mx = torch.maximum(s.max(-1, keepdim=True).values, sinks.float().view(H, 1))
            e = torch.exp(s - mx)
            out[t] = (e / (e.sum(-1, keepdim=True) + torch.exp(sinks.float().view(H, 1) - mx))) @ rows[:, :C]
            continue
        out[t] = torch.softmax(s, -1) @ rows[:, :C]
    return out.to(out_dtype)


# ----------------------------------------------------------------------------- mixture of experts
def moe_route(logits: torch.Tensor, E: int, top: int, scale: float, score: str = "softmax"):
    """Scores over the first E columns, the ``top`` largest (ties: lowest index).  "softmax": weights
    s / (sum of the chosen s + 1e-20) * scale; "sigmoid": weights s * scale, not renormalised."""
    z = logits[:, :E].float()
    s = torch.sigmoid(z) if score == "sigmoid" else torch.softmax(z, -1)
    w, idx = torch.sort(s, dim=-1, descending=True, stable=True)
    w, idx = w[:, :top], idx[:, :top]
    if score != "sigmoid":
        w = w / (w.sum(-1, keepdim=True) + 1e-20)
    return idx.int().contiguous(), (w * scale).contiguous()


def moe_align(topk_idx: torch.Tensor, E: int, BM: int):
    """Sort the (token, choice) pairs by expert.  Returns sorted_tok [P] (token of each sorted row), pos_of_pair [P]
    (sorted row of pair t * top + k), seg [E + 1] and the row tiles [(expert, row0, rows)] padded with expert -1."""
    T, top = topk_idx.shape
    flat = topk_idx.reshape(-1).long()
    order = torch.sort(flat, stable=True).indices
    pos = torch.empty_like(order)
    pos[order] = torch.arange(order.numel())
    cnt = torch.bincount(flat, minlength=E)
    seg = torch.zeros(E + 1, dtype=torch.int32)
    seg[1:] = cnt.cumsum(0)
    ntiles = (T * top + BM - 1) // BM + E
    tiles = torch.full((ntiles, 3), -1, dtype=torch.int32)
    i = 0
    for e in range(E):
        for r0 in range(int(seg[e]), int(seg[e + 1]), BM):
            tiles[i] = torch.tensor([e, r0, min(BM, int(seg[e + 1]) - r0)])
            i += 1
    return (order // top).int(), pos.int(), seg, tiles


def moe_combine(D, pos_of_pair, topk_w, shared, logits, sg_col: int, out_dtype, top: int = 0):
    """z[t] = sum_k w[t, k] D[pos[t, k]] + sigmoid(logits[t, sg_col]) * shared[t]  (topk_w None: plain sum)."""
    top = topk_w.shape[1] if topk_w is not None else top
    T = pos_of_pair.numel() // top
    rows = D.float()[pos_of_pair.long().view(T, top)]
    z = (rows * topk_w.unsqueeze(-1) if topk_w is not None else rows).sum(1)
    if shared is not None:
        gate = torch.sigmoid(logits[:, sg_col].float()).unsqueeze(-1) if sg_col >= 0 else 1.0
        z = z + gate * shared.float()
    return z.to(out_dtype)


# ----------------------------------------------------------------------------- windowed attention with pooled blocks
def pool_entry(bt_row, b: int, P: int, bs: int) -> int:
    """Entry of pooled block b: it lives with the page that holds its first token; a page has ceil(bs / P) entries."""
    ppb = -(-bs // P)
    page = b * P // bs
    first = -(-(page * bs) // P)
    return int(bt_row[page]) * ppb + (b - first)


def window_kv_write(kcache, vcache, qkv, koff: int, voff: int, qb, kb, vb, cos_sin, positions, slot_mapping, vfirst_in,
                    vfirst_out, lam: float, H: int, G: int, D: int, V: int, dims: int, eps: float, unit: bool,
                    half_layout: bool = False, qnw=None, knw=None, head_qnw=None, head_knw=None) -> None:
    """Per token: q (first H D columns of qkv, rewritten in place) and k (at koff) get their bias, (``qnw`` / ``knw``)
    the RMS norm over the whole projection (all heads at once) with that weight, the rotation of the pairs
    (2i, 2i + 1) -- ``half_layout``: (i, i + dims / 2) --, i < dims / 2, by cos_sin[pos] = [cos | sin], and (``unit``)
    x / sqrt(mean(x^2) + eps) per head; ``head_qnw`` / ``head_knw`` [D]: before the rotation every head is divided by
    its own root mean square and multiplied by that weight; v (at voff) gets its bias and (``vfirst_in``) becomes (1 - lam) v + lam
    vfirst_in; ``vfirst_out`` receives v in fp32.  k, v go to kcache [slots, G, D] / vcache [slots, G, V] at the tokens'
    slots (negative: not written); ``kcache`` None: queries only.  Rows with a negative position are skipped."""
    T = qkv.shape[0]
    live = positions >= 0
    half = dims // 2
    cs = cos_sin[positions.long().clamp(min=0)] if dims else None

    def prep(x, bias, n, nw, hnw):
        x = x.float().reshape(T, n, D)
        if bias is not None:
            x = x + bias.float().view(n, D)
        if nw is not None:
            x = x * torch.rsqrt(x.pow(2).mean((-2, -1), keepdim=True) + eps) * nw.float().view(n, D)
        if hnw is not None:
            x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * hnw.float().view(D)
        if dims:
            c, s = cs[:, None, :half], cs[:, None, half:]
            x = x.clone()
            if half_layout:
                a, b = x[..., :half].clone(), x[..., half:dims].clone()
                x[..., :half], x[..., half:dims] = a * c - b * s, b * c + a * s
            else:
                a, b = x[..., 0:dims:2], x[..., 1:dims:2]
                x[..., 0:dims:2], x[..., 1:dims:2] = a * c - b * s, b * c + a * s
        if unit:
            x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
        return x

    q = prep(qkv[:, :H * D], qb, H, qnw, head_qnw).reshape(T, H * D)
    qkv[live, :H * D] = q[live].to(qkv.dtype)
    if kcache is None:
        return
    k = prep(qkv[:, koff:koff + G * D], kb, G, knw, head_knw)
    v = qkv[:, voff:voff + G * V].float()
    if vb is not None:
        v = v + vb.float()
    if vfirst_in is not None:
        v = (1.0 - lam) * v + lam * vfirst_in
    if vfirst_out is not None:
        vfirst_out[live] = v[live]
    ok = live & (slot_mapping >= 0)
    kcache[slot_mapping[ok].long()] = k[ok].to(kcache.dtype)
    vcache[slot_mapping[ok].long()] = v[ok].view(-1, G, V).to(vcache.dtype)


def window_pool(kpool, vpool, kcache, vcache, block_tables, tok_seq, positions, P: int, bs: int) -> None:
    """For every token that ends a block of P tokens: the fp32 mean of the block's cached keys / values."""
    for t in range(positions.shape[0]):
        p = int(positions[t])
        if p < 0 or (p + 1) % P:
            continue
        b = p // P
        bt = block_tables[int(tok_seq[t])].long()
        js = torch.arange(b * P, b * P + P)
        slots = bt[js // bs] * bs + js % bs
        e = pool_entry(bt, b, P, bs)
        kpool[e] = kcache[slots].float().mean(0)
        vpool[e] = vcache[slots].float().mean(0)


def window_attention(q, gate, kcache, vcache, kpool, vpool, block_tables, tok_seq, positions, H: int, G: int, D: int,
                     V: int, window: int, P: int, scale: float, sink: bool, bs: int, out_dtype, chunk: int = 0,
                     softcap: float = 0.0, sinks=None, gate_per_head: bool = False):
    """Token t at position p attends the cached tokens max(0, p - window + 1) .. p (window <= 0: all; ``chunk`` > 0
    instead: the tokens of its own chunk, p - p % chunk .. p) and the pooled blocks b with b P + P - 1 <= p - window,
    in one softmax (``sink``: one more term e^sinks[h], or one unit, in the denominator); scores q . k * scale, then
    (``softcap`` > 0) softcap tanh(score / softcap); query head h uses key / value head h // (H / G).  The result times
    sigmoid(gate) if given ([T, H V], or [T, H] with ``gate_per_head``).  [T, H V]."""
    T = q.shape[0]
    out = torch.zeros(T, H, V)
    qf = q.float().reshape(T, -1)[:, :H * D].view(T, H, D)
    R = H // G
    for t in range(T):
        p = int(positions[t])
        if p < 0:
            continue
        lo = 0 if window <= 0 else max(0, p - window + 1)
        if chunk > 0:
            lo = p - p % chunk
        nb = (p - window + 1) // P if (window > 0 and P > 0 and p - window + 1 >= P) else 0
        bt = block_tables[int(tok_seq[t])].long()
        js = torch.arange(lo, p + 1)
        slots = bt[js // bs] * bs + js % bs
        K, Vv = kcache[slots].float(), vcache[slots].float()
        if nb:
            es = torch.tensor([pool_entry(bt, b, P, bs) for b in range(nb)])
            K, Vv = torch.cat([kpool[es], K]), torch.cat([vpool[es], Vv])
        for h in range(H):
            g = h // R
            s = (K[:, g] @ qf[t, h]) * scale
            if softcap > 0:
                s = softcap * torch.tanh(s / softcap)
            s0 = (sinks[h].float() if sinks is not None else torch.zeros(())) if sink else None
            mx = torch.maximum(s.max(), s0) if sink else s.max()
            e = torch.exp(s - mx)
            den = e.sum() + (torch.exp(s0 - mx) if sink else 0.0)
            out[t, h] = (e / den) @ Vv[:, g]
    if gate is not None and gate_per_head:
        out = out * torch.sigmoid(gate.float()).unsqueeze(-1)
    out = out.reshape(T, H * V)
    if gate is not None and not gate_per_head:
        out = out * torch.sigmoid(gate.float())
    return out.to(out_dtype)


# ----------------------------------------------------------------------------- gated matrix-state recurrences
SCAN_HGRN2, SCAN_MLSTM, SCAN_SSD = 0, 1, 2


def gated_scan_record(kind: int, D: int, V: int) -> int:
    return D * V + (D + 1 if kind == SCAN_MLSTM else 0)


def ssd_scan(proj, cols: dict, aux, head_params, state, cu_q, seq_slots, positions, H: int, G: int, D: int, V: int):
    """``proj`` fp32 holds x (H V, at cols v), B and C (G D each, at cols k and q); ``aux`` fp32 holds the step-size
    logits (H, at cols f) and the gate (H V, at cols g); ``head_params`` [3, H] = neg_a, dt_bias, skip.  Per head h with
    the B, C of group h // (H / G): dt = softplus(f + dt_bias), S <- exp(neg_a dt) S + dt B x^T (S [D, V]),
    y = (S^T C + skip x) * silu(g).  fp32 [T, H V]; ``state`` [slots, H, D V] fp32."""
    T = proj.shape[0]
    pf, af = proj.float(), aux.float()
    x = pf[:, cols["v"]:cols["v"] + H * V].view(T, H, V)
    B = pf[:, cols["k"]:cols["k"] + G * D].view(T, G, D).repeat_interleave(H // G, 1)
    C = pf[:, cols["q"]:cols["q"] + G * D].view(T, G, D).repeat_interleave(H // G, 1)
    neg_a, dt_bias, skip = head_params.float()
    dt = torch.nn.functional.softplus(af[:, cols["f"]:cols["f"] + H] + dt_bias, threshold=1e9)
    decay = torch.exp(neg_a * dt)
    gate = af[:, cols["g"]:cols["g"] + H * V]
    out = torch.zeros(T, H, V)
    cu = cu_q.tolist()
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if b <= a or int(positions[a]) < 0:
            continue
        slot = int(seq_slots[s])
        S = torch.zeros(H, D, V) if int(positions[a]) == 0 else state[slot].view(H, D, V).clone()
        for t in range(a, b):
            S = decay[t].view(H, 1, 1) * S + (dt[t].view(H, 1) * B[t]).unsqueeze(2) * x[t].unsqueeze(1)
            out[t] = torch.einsum("hdv,hd->hv", S, C[t]) + skip.view(H, 1) * x[t]
        state[slot] = S.reshape(H, D * V)
    return out.reshape(T, H * V) * gate * torch.sigmoid(gate)


def gated_scan(proj, kind: int, cols: dict, fbias, ibias, lower, normw, state, cu_q, seq_slots, positions, H: int,
               D: int, V: int, eps: float, cap: float, out_dtype, aux=None, head_params=None, groups: int = 0):
    """``proj`` fp32 [T, ld] holds the parts at the column offsets ``cols``; ``state`` [slots, H, record] fp32.
    SCAN_HGRN2: f = low + (1 - low) sigmoid(zf + bf), S <- diag(f) S + (1 - f) v^T, o = S^T silu(zq),
    y = o / rms(o) * normw [V].  SCAN_MLSTM: i = cap tanh((zi + bi) / cap), f = logsigmoid(cap tanh((zf + bf) / cap)),
    m' = max(f + m, i), S <- e^(f + m - m') S + e^(i - m') k v^T, n likewise, o = S^T q / (max(|n . q|, e^(-m')) + 1e-6)
    with q = zq / sqrt(D), y = o / rms(o) * normw [H V] * sigmoid(zg).  A portion at position 0 starts from zero."""
    if kind == SCAN_SSD:
        return ssd_scan(proj, cols, aux, head_params, state, cu_q, seq_slots, positions, H, groups, D, V)
    T = proj.shape[0]
    pf = proj.float()
    out = torch.zeros(T, H, V)
    cu = cu_q.tolist()
    part = lambda key, n: pf[:, cols[key]:cols[key] + H * n].view(T, H, n)
    v = part("v", V)
    if kind == SCAN_HGRN2:
        zq = part("q", D)
        q = zq * torch.sigmoid(zq)
        low = lower.float().view(H, D)
        zf = part("f", D) + (fbias.float().view(H, D) if fbias is not None else 0.0)
        f = low + (1.0 - low) * torch.sigmoid(zf)
    else:
        q = part("q", D) / math.sqrt(D)
        k = part("k", D)
        zi = pf[:, cols["i"]:cols["i"] + H] + (ibias.float() if ibias is not None else 0.0)
        zf = pf[:, cols["f"]:cols["f"] + H] + (fbias.float() if fbias is not None else 0.0)
        ig = cap * torch.tanh(zi / cap)
        fg = torch.nn.functional.logsigmoid(cap * torch.tanh(zf / cap))
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if b <= a or int(positions[a]) < 0:
            continue
        slot = int(seq_slots[s])
        rec = torch.zeros(H, gated_scan_record(kind, D, V)) if int(positions[a]) == 0 else state[slot].clone()
        S = rec[:, :D * V].reshape(H, D, V).clone()
        if kind == SCAN_MLSTM:
            n, m = rec[:, D * V:D * V + D].clone(), rec[:, D * V + D].clone()
        for t in range(a, b):
            if kind == SCAN_HGRN2:
                S = f[t].unsqueeze(2) * S + (1.0 - f[t]).unsqueeze(2) * v[t].unsqueeze(1)
                o = torch.einsum("hdv,hd->hv", S, q[t])
            else:
                mn = torch.maximum(fg[t] + m, ig[t])
                ka, kb = torch.exp(fg[t] + m - mn), torch.exp(ig[t] - mn)
                m = mn
                S = ka[:, None, None] * S + kb[:, None, None] * k[t].unsqueeze(2) * v[t].unsqueeze(1)
                n = ka[:, None] * n + kb[:, None] * k[t]
                den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
                o = torch.einsum("hdv,hd->hv", S, q[t]) / den[:, None]
            out[t] = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
        state[slot, :, :D * V] = S.reshape(H, D * V)
        if kind == SCAN_MLSTM:
            state[slot, :, D * V:D * V + D] = n
            state[slot, :, D * V + D] = m
    if kind == SCAN_HGRN2:
        y = (out * normw.float().view(1, 1, V)).reshape(T, H * V)
    else:
        y = out.reshape(T, H * V) * normw.float() * torch.sigmoid(pf[:, cols["g"]:cols["g"] + H * V])
    return y.to(out_dtype)


# ----------------------------------------------------------------------------- short convolutions, delta rule, RG-LRU
CONV_NONE, CONV_SILU = 0, 1


def short_conv(x, w, state, cu_q, seq_slots, positions, in_bias, out_bias, act: int, unit_cols: int, unit_dim: int,
               scale_cols: int, scale: float, unit_eps: float, residual: bool = False):
    """Causal convolution over time per channel, over a varlen batch.  ``x`` [T, C] (any row stride), ``w`` [C, taps]
    (the last tap is the current token's), inputs x + in_bias, zeros before position 0; the taps - 1 inputs before a
    portion come from ``state`` [slots, taps - 1, C] fp32, which then receives the portion's last ones.  Then out_bias,
    the activation, and for the first ``unit_cols`` channels, in groups of ``unit_dim``: v / sqrt(sum(v^2) + unit_eps);
    the first ``scale_cols`` channels times ``scale``.  Returns fp32 [T, C]."""
    T, C = x.shape
    n = w.shape[1]
    wf = w.float()
    out = torch.zeros(T, C)
    cu = cu_q.tolist()
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if b <= a or int(positions[a]) < 0:
            continue
        slot, p0 = int(seq_slots[s]), int(positions[a])
        xin = x[a:b].float()
        if in_bias is not None:
            xin = xin + in_bias.float()
        hist = state[slot].clone() if n > 1 else torch.zeros(0, C)
        for r in range(n - 1):
            if p0 - (n - 1) + r < 0:
                hist[r] = 0.0
        full = torch.cat([hist, xin])
        y = torch.zeros(b - a, C)
        for j in range(n):
            y += wf[:, j] * full[j:j + b - a]
        out[a:b] = y
        if n > 1:
            state[slot] = full[-(n - 1):]
    if out_bias is not None:
        out = out + out_bias.float()
    if act == CONV_SILU:
        out = out * torch.sigmoid(out)
    if residual:                      # rows of idle sequences stay zero
        live = torch.zeros(T, dtype=torch.bool)
        for s in range(len(cu) - 1):
            if cu[s + 1] > cu[s] and int(positions[cu[s]]) >= 0:
                live[cu[s]:cu[s + 1]] = True
        xin = x.float() + (in_bias.float() if in_bias is not None else 0.0)
        out = torch.where(live[:, None], out + xin, out)
    if unit_cols:
        u = out[:, :unit_cols].reshape(T, unit_cols // unit_dim, unit_dim)
        out[:, :unit_cols] = (u * torch.rsqrt(u.pow(2).sum(-1, keepdim=True) + unit_eps)).reshape(T, unit_cols)
    if scale_cols:
        out[:, :scale_cols] *= scale
    return out


def delta_scan(qkv, proj, cols: dict, neg_a, dt_bias, normw, state, cu_q, seq_slots, positions, H: int, G: int, D: int,
               V: int, eps: float, out_dtype):
    """Gated delta rule.  ``qkv`` fp32 [T, G D | G D | H V] (prepared queries, keys, values), ``proj`` fp32 with the
    columns b (H), a (H) and g (H V) at ``cols``; per head h (queries / keys of head h // (H / G)):
    decay = exp(neg_a[h] softplus(a + dt_bias[h])), beta = sigmoid(b), S <- decay S, u = beta (v - S^T k),
    S <- S + k u^T, o = S^T q; y = o / rms(o) * normw [V] * silu(g).  ``state`` [slots, H, D V] fp32."""
    T = qkv.shape[0]
    q = qkv[:, :G * D].float().view(T, G, D)
    k = qkv[:, G * D:2 * G * D].float().view(T, G, D)
    v = qkv[:, 2 * G * D:2 * G * D + H * V].float().view(T, H, V)
    pf = proj.float()
    beta = torch.sigmoid(pf[:, cols["b"]:cols["b"] + H])
    decay = torch.exp(neg_a.float() * torch.nn.functional.softplus(pf[:, cols["a"]:cols["a"] + H] + dt_bias.float()))
    gate = pf[:, cols["g"]:cols["g"] + H * V]
    out = torch.zeros(T, H, V)
    R = H // G
    cu = cu_q.tolist()
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if b <= a or int(positions[a]) < 0:
            continue
        slot = int(seq_slots[s])
        S = torch.zeros(H, D, V) if int(positions[a]) == 0 else state[slot].view(H, D, V).clone()
        for t in range(a, b):
            kk = k[t].repeat_interleave(R, 0)                              # [H, D]
            qq = q[t].repeat_interleave(R, 0)
            S = decay[t].view(H, 1, 1) * S
            u = beta[t].view(H, 1) * (v[t] - torch.einsum("hdv,hd->hv", S, kk))
            S = S + kk.unsqueeze(2) * u.unsqueeze(1)
            out[t] = torch.einsum("hdv,hd->hv", S, qq)
        state[slot] = S.reshape(H, D * V)
    y = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps) * normw.float()
    y = y.reshape(T, H * V) * gate * torch.sigmoid(gate)
    return y.to(out_dtype)


def rglru_scan(u, gates, gate_bias, decay_rate, proj, ycol: int, ybias, state, cu_q, seq_slots, positions, C: int,
               blocks: int, out_dtype):
    """Real-gated linear recurrent unit per channel.  ``u`` fp32 [T, C]; ``gates`` fp32 [T, blocks, 2 C / blocks]: per
    block the logits of the recurrence gate then of the input gate, ``gate_bias`` [blocks, 2 C / blocks] added;
    r, i = sigmoid of them; a = exp(decay_rate r) (``decay_rate`` [C] <= 0), S <- a S + sqrt(1 - a^2) i u;
    out = S gelu_tanh(proj[:, ycol + c] + ybias).  ``state`` [slots, C] fp32."""
    T = u.shape[0]
    bw = C // blocks
    z = gates.float().view(T, blocks, 2 * bw) + gate_bias.float().view(blocks, 2 * bw)
    r = torch.sigmoid(z[..., :bw]).reshape(T, C)
    i = torch.sigmoid(z[..., bw:]).reshape(T, C)
    la = decay_rate.float() * r
    a = torch.exp(la)
    w = torch.sqrt(-torch.expm1(2.0 * la)) * i * u.float()
    out = torch.zeros(T, C)
    cu = cu_q.tolist()
    for s in range(len(cu) - 1):
        lo, hi = cu[s], cu[s + 1]
        if hi <= lo or int(positions[lo]) < 0:
            continue
        slot = int(seq_slots[s])
        S = torch.zeros(C) if int(positions[lo]) == 0 else state[slot].clone()
        for t in range(lo, hi):
            S = a[t] * S + w[t]
            out[t] = S
        state[slot] = S
    g = proj[:, ycol:ycol + C].float() + ybias.float()
    y = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g * g * g)))
    return (out * y).to(out_dtype)


def norm_mix(a, wa, b, wb, eps: float, ca: float, cb: float, out_dtype, groups: int = 1):
    """ca * a / rms(a) * wa + cb * b / rms(b) * wb  (rows; ``b`` may be None); ``groups`` > 1: the root mean square of
    each of that many equal consecutive parts of a row by itself."""
    af = a.float()
    if groups > 1:
        ag = af.reshape(af.shape[0], groups, -1)
        y = ca * (ag * torch.rsqrt(ag.pow(2).mean(-1, keepdim=True) + eps)).reshape(af.shape) * wa.float()
        return y.to(out_dtype)
    y = ca * af * torch.rsqrt(af.pow(2).mean(-1, keepdim=True) + eps) * wa.float()
    if b is not None:
        bf = b.float()
        y = y + cb * bf * torch.rsqrt(bf.pow(2).mean(-1, keepdim=True) + eps) * wb.float()
    return y.to(out_dtype)
