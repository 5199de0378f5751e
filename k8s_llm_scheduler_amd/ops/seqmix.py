"""Ops of models with an fp32 residual stream, recurrent / windowed- or latent-attention mixers and mixtures of experts.

Same dispatch rule as the rest of :mod:`..ops`: CUDA (= HIP) tensors always run the gfx950 kernels
(``stream32.hip``, ``mixers.hip``, ``window_attn.hip``, ``gated_scan.hip``, ``delta_scan.hip``, ``moe.hip``) and raise when the extension is missing; CPU tensors run the fp32
reference in :mod:`.reference` (the CPU test-suite).  Every op takes bf16 or true-fp32 activations / weights (the
``f32`` flag of the kernels); what a design computes in fp32 regardless (residual sum, recurrent state, decays, router,
attention scores) is fp32 in both.
"""

from __future__ import annotations

import os
from typing import Optional

import torch

from . import reference as ref
from .reference import ACT_GELU_ERF, ACT_GELU_TANH, ACT_RELU, ACT_SILU, ACT_SOFTCAP, ACT_SWISH_CLAMP, ACT_TANH  # noqa: F401
from .reference import CONV_NONE, CONV_SILU  # noqa: F401
from .reference import GATE_SIGMOID, GATE_SILU  # noqa: F401
from .reference import SCAN_HGRN2, SCAN_MLSTM, SCAN_SSD  # noqa: F401

BF16, F32, I32 = torch.bfloat16, torch.float32, torch.int32
GROUP_BM = 64   # row-tile height of the grouped GEMM (gemm_any_kernel's BM)


def _native():
    from . import native

    return native()


def _gpu(*ts) -> bool:
    cuda = [t.is_cuda for t in ts if t is not None]
    if any(cuda) and not all(cuda):
        raise ValueError("mixed CPU/GPU tensors")
    return bool(cuda) and cuda[0]


def _p(t: Optional[torch.Tensor], dtype=None, name: str = "tensor") -> int:
    if t is None:
        return 0
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: must be contiguous")
    return t.data_ptr()


def _f32(dtype) -> int:
    if dtype == F32:
        return 1
    if dtype == BF16:
        return 0
    raise TypeError(f"activations must be bfloat16 or float32, got {dtype}")


# ----------------------------------------------------------------------------- residual stream
def embed_rows(ids: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """fp32 [T, W] rows of ``table`` (bf16 or fp32) times ``scale``."""
    if not _gpu(ids, table):
        return ref.embed_rows(ids, table, scale)
    T, W = ids.shape[0], table.shape[1]
    out = torch.empty(T, W, dtype=F32, device=table.device)
    _native().embed_rows(out.data_ptr(), _p(ids, I32, "ids"), _p(table), T, W, table.shape[0], float(scale),
                         _f32(table.dtype), -1)
    return out


def resnorm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float, *, branch: Optional[torch.Tensor] = None,
            mult: float = 1.0, rowvec: Optional[torch.Tensor] = None, offset: float = 0.0,
            out_dtype=BF16, groups: int = 1, branch2: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``x`` (fp32 [T, W], updated in place) += mult * (branch + branch2) + rowvec (two sublayers that read one norm
    leave two branches); returns rms-norm(x) * (offset + w) in
    ``out_dtype``, or None when ``w`` is None (add only).  ``groups`` > 1: every one of that many equal consecutive
    parts of a row is divided by its own root mean square."""
    if x.dtype != F32:
        raise TypeError("the residual stream is fp32")
    T, W = x.shape
    if groups < 1 or W % groups:
        raise ValueError(f"resnorm: {groups} groups do not divide the width {W}")
    if branch is None and branch2 is not None:
        branch, branch2 = branch2, None
    if not _gpu(x, w, branch, rowvec, branch2):
        return ref.resnorm(x, branch, mult, rowvec, w, offset, eps, out_dtype, groups, branch2)
    out = torch.empty(T, W, dtype=out_dtype, device=x.device) if w is not None else None
    f32 = _f32(out_dtype)
    for t, n in ((branch, "branch"), (branch2, "branch2"), (rowvec, "rowvec"), (w, "w")):
        if t is not None and t.dtype != out_dtype:
            raise TypeError(f"{n}: expected {out_dtype}, got {t.dtype}")
    _native().resnorm(_p(x), _p(branch), _p(branch2), float(mult), _p(rowvec), _p(w), float(offset), float(eps),
                      _p(out), T, W, int(groups), f32, -1)
    return out


def norm_mix(a: torch.Tensor, wa: torch.Tensor, b: Optional[torch.Tensor], wb: Optional[torch.Tensor], eps: float,
             ca: float = 1.0, cb: float = 1.0, out_dtype=None, groups: int = 1) -> torch.Tensor:
    """ca * rms-norm(a) * wa + cb * rms-norm(b) * wb over rows [T, W] (norms in fp32; ``b`` None: the first term
    only): the outputs of two mixers that run side by side, each normed, joined.  ``a`` may be a column slice of a
    wider tensor (row stride free).  ``groups`` > 1 (``a`` alone): every one of that many equal consecutive parts of a
    row is divided by its own root mean square."""
    out_dtype = out_dtype or a.dtype
    T, W = a.shape
    if groups < 1 or W % groups or (groups > 1 and b is not None):
        raise ValueError(f"norm_mix: {groups} groups must divide the width {W} and go with one input")
    if not _gpu(a, wa, b, wb):
        return ref.norm_mix(a, wa, b, wb, eps, ca, cb, out_dtype, groups)
    if a.stride(1) != 1:
        raise ValueError("norm_mix: rows must be contiguous")
    if b is not None and (b.shape != a.shape or b.dtype != a.dtype or wb is None):
        raise ValueError("norm_mix: the two inputs must agree in shape and dtype")
    out = torch.empty(T, W, dtype=out_dtype, device=a.device)
    _native().norm_mix(out.data_ptr(), a.data_ptr(), a.stride(0), _p(wa, a.dtype, "wa"), _p(b), _p(wb, a.dtype, "wb"),
                       float(eps), float(ca), float(cb), T, W, int(groups), _f32(a.dtype), _f32(out_dtype), -1)
    return out


def postnorm(x: torch.Tensor, branch: Optional[torch.Tensor], alpha: float, gain: float, eps: float, *,
             branch2: Optional[torch.Tensor] = None, c1: float = 1.0, c2: float = 1.0,
             out_dtype=None) -> Optional[torch.Tensor]:
    """Norm after the sum: ``x`` (fp32 [T, W], updated in place) <- rms-norm(alpha x + c1 branch + c2 branch2) * gain
    with one ``gain`` for the whole row, so the stream itself stays normed.  With ``out_dtype`` the new rows are also
    returned in that type (the input of the sublayer that reads them next)."""
    if x.dtype != F32 or not x.is_contiguous():
        raise TypeError("the residual stream is contiguous fp32")
    if branch is None and branch2 is not None:
        branch, branch2, c1, c2 = branch2, None, c2, c1
    if not _gpu(x, branch, branch2):
        return ref.postnorm(x, branch, branch2, alpha, c1, c2, gain, eps, out_dtype)
    T, W = x.shape
    bt = branch.dtype if branch is not None else out_dtype
    for t, n in ((branch, "branch"), (branch2, "branch2")):
        if t is not None and (t.dtype != bt or t.shape != x.shape):
            raise TypeError(f"postnorm: {n} must be [T, W] of one activation type")
    if out_dtype is not None and bt is not None and out_dtype != bt:
        raise TypeError("postnorm: the returned rows take the branches' type")
    out = torch.empty(T, W, dtype=out_dtype, device=x.device) if out_dtype is not None else None
    _native().postnorm(_p(x), _p(branch), _p(branch2), float(alpha), float(c1), float(c2), float(gain), float(eps),
                       _p(out), T, W, _f32(bt or F32), -1)
    return out


def gate_mul(y: torch.Tensor, gate: torch.Tensor, kind: int = GATE_SIGMOID) -> torch.Tensor:
    """y * sigmoid(gate) (GATE_SIGMOID) or y * silu(gate) (GATE_SILU), element by element; ``y`` [T, F] (the gate's
    type, or fp32) and ``gate`` [T, F] may be column slices of wider tensors.  Returns [T, F] of the gate's type."""
    if y.shape != gate.shape or y.dim() != 2:
        raise ValueError("gate_mul: y and gate must be [T, F]")
    if not _gpu(y, gate):
        return ref.gate_mul(y, gate, kind)
    if y.stride(1) != 1 or gate.stride(1) != 1 or y.dtype not in (gate.dtype, F32):
        raise ValueError("gate_mul: rows must be contiguous; y is of the gate's type or fp32")
    T, F = y.shape
    out = torch.empty(T, F, dtype=gate.dtype, device=y.device)
    _native().gate_mul(out.data_ptr(), y.data_ptr(), y.stride(0), gate.data_ptr(), gate.stride(0), T, F, int(kind),
                       int(y.dtype == F32), _f32(gate.dtype), -1)
    return out


def act(x: torch.Tensor, kind: int, limit: float = 0.0, alpha: float = 1.0, *,
        row_scale: Optional[torch.Tensor] = None, row_map: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Gated kinds (ACT_GELU_TANH, ACT_SWISH_CLAMP, ACT_RELU = relu(g) u): [T, 2F] = [gate | up] -> [T, F]; ACT_TANH /
    ACT_SILU / ACT_GELU_ERF (exact gelu) / ACT_SOFTCAP (limit tanh(x / limit)): elementwise.  Elementwise kinds take an
    fp32 factor per row, ``row_scale`` [T]: logical row i is row ``row_map[i]`` (a permutation; default i) and its
    input is multiplied by ``row_scale[i]`` before the function."""
    gated = kind in (ACT_GELU_TANH, ACT_SWISH_CLAMP, ACT_RELU)
    if kind == ACT_SOFTCAP and not limit > 0:
        raise ValueError("act: a soft cap needs a positive limit")
    if gated and (row_scale is not None or row_map is not None):
        raise ValueError("act: row factors go with the elementwise kinds")
    if not _gpu(x, row_scale, row_map):
        return ref.act(x, kind, limit, alpha, row_scale, row_map)
    T = x.shape[0]
    F = x.shape[1] // 2 if gated else x.shape[1]
    for t, n in ((row_scale, "row_scale"), (row_map, "row_map")):
        if t is not None and t.numel() != T:
            raise ValueError(f"act: {n} must have one entry per row")
    out = torch.empty(T, F, dtype=x.dtype, device=x.device)
    _native().act(out.data_ptr(), _p(x), T, F, kind, float(limit or 0.0), float(alpha), _p(row_scale, F32, "row_scale"),
                  _p(row_map, I32, "row_map"), _f32(x.dtype), -1)
    return out


def _route_fast(a: torch.Tensor, w: torch.Tensor, out_dtype) -> bool:
    """bf16 products of production size whose shape the framework's tuned GEMV / MFMA GEMM kernels take (128-byte
    k steps, N % 16 == 0, at least 1024 x 512 weights: the sizes their plan tables and heuristics were tuned and
    tested on).  Smaller products are launch-bound and stay on the any-shape kernel."""
    from . import GEMM_BACKEND, LEAN

    if LEAN:
        return False
    if a.dtype != BF16 or w.dtype != BF16 or out_dtype not in (BF16, F32) or a.dim() != 2 or w.dim() != 2:
        return False
    if GEMM_BACKEND == "library" or not a.is_contiguous() or not w.is_contiguous():
        return False
    N, K = w.shape
    return K % 64 == 0 and N % 16 == 0 and K * N >= 512 * 1024 and K >= 128 and N >= 128


# route fitting bf16 shapes to ops.linear (K8S_SEQMIX_FAST_GEMM=0: every product on the any-shape kernel)
FAST_GEMM = os.environ.get("K8S_SEQMIX_FAST_GEMM", "1") != "0"


def linear(a: torch.Tensor, w: torch.Tensor, out_dtype=None) -> torch.Tensor:
    """a [M, K] @ w [N, K]^T for any shape, bf16 or fp32 operands (fp32: plain fp32 FMAs, no reduced-precision
    matrix mode), fp32 accumulation.  Shapes that fit the tuned bf16 kernels go there."""
    out_dtype = out_dtype or a.dtype
    if not _gpu(a, w):
        return ref.gemm_any(a, w, out_dtype)
    if FAST_GEMM and _route_fast(a, w, out_dtype):
        from . import NoKernelForShape, linear as tuned

        try:
            return tuned(a, w, out_dtype=F32 if out_dtype == F32 else None)
        except NoKernelForShape:
            pass
    return gemm(a, w, out_dtype)


def gemm(a: torch.Tensor, w: torch.Tensor, out_dtype=None, *, a_rows: Optional[torch.Tensor] = None,
         tiles: Optional[torch.Tensor] = None, rows: Optional[int] = None,
         seg: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The any-shape GEMM.  2-D: a [M, K] (row stride free) @ w [N, K]^T.  3-D: batched over dim 0 (a [G, M, K] with
    any strides whose last is 1, w [G, N, K]) -> [G, M, N]; ``out``: a [G, M, N] view with any batch / row strides.
    Grouped (``tiles`` [n, 3] from :func:`moe_align`, w [G, N, K]): ``rows`` compact rows, row r = a[a_rows[r]] (or
    a[r]), the rows of tile (g, r0, n) use w[g] -> [rows, N] (``seg``: the groups' row offsets, read by the CPU
    reference only)."""
    out_dtype = out_dtype or a.dtype
    if a.dtype != w.dtype:
        raise TypeError(f"gemm operands differ in dtype: {a.dtype} and {w.dtype}")
    if a.stride(-1) != 1 or w.stride(-1) != 1:
        raise ValueError("gemm: the k dimension must be contiguous")
    if tiles is not None:
        G, N, K = w.shape
        if a.shape[-1] != K:
            raise ValueError("gemm: k mismatch")
        if not _gpu(a, w):
            return ref.gemm_any(a, w, out_dtype, a_rows, tiles, seg)
        out = torch.empty(rows, N, dtype=out_dtype, device=a.device)
        _native().gemm_any(out.data_ptr(), a.data_ptr(), _p(w), rows, N, K, a.stride(0), K, N, 1, 0, N * K, 0,
                           _p(a_rows, I32, "a_rows"), _p(tiles, I32, "tiles"), tiles.shape[0], _f32(a.dtype),
                           _f32(out_dtype), -1)
        return out
    if a.shape[-1] != w.shape[-1]:
        raise ValueError(f"gemm: k mismatch {tuple(a.shape)} x {tuple(w.shape)}")
    if not _gpu(a, w):
        y = ref.gemm_any(a, w, out_dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y
    if a.dim() == 2:
        M, K = a.shape
        N = w.shape[0]
        out = torch.empty(M, N, dtype=out_dtype, device=a.device)
        _native().gemm_any(out.data_ptr(), a.data_ptr(), w.data_ptr(), M, N, K, a.stride(0), w.stride(0), N, 1, 0, 0,
                           0, 0, 0, 0, _f32(a.dtype), _f32(out_dtype), -1)
        return out
    G, M, K = a.shape
    N = w.shape[1]
    if out is None:
        out = torch.empty(G, M, N, dtype=out_dtype, device=a.device)
    elif out.shape != (G, M, N) or out.stride(2) != 1 or out.dtype != out_dtype:
        raise ValueError("gemm: out must be a [G, M, N] view of the output dtype with contiguous rows")
    _native().gemm_any(out.data_ptr(), a.data_ptr(), w.data_ptr(), M, N, K, a.stride(1), w.stride(1), out.stride(1), G,
                       a.stride(0), w.stride(0), out.stride(0), 0, 0, 0, _f32(a.dtype), _f32(out_dtype), -1)
    return out


# ----------------------------------------------------------------------------- recurrent mixer
def token_shift(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor, tok_seq: torch.Tensor,
                seq_slots: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
    """[n, T, W]: h + (previous token's h - h) * mu[s]; the previous token of a portion's first token is the slot's
    row of ``state`` (zeros at position 0)."""
    if not _gpu(h, mu, state):
        return ref.token_shift(h, mu, state, cu_q, seq_slots, positions)
    T, W = h.shape
    n = mu.shape[0]
    out = torch.empty(n, T, W, dtype=h.dtype, device=h.device)
    _native().token_shift(out.data_ptr(), _p(h), _p(mu, h.dtype, "mu"), _p(state, h.dtype, "state"),
                          _p(cu_q, I32, "cu_q"), _p(tok_seq, I32, "tok_seq"), _p(seq_slots, I32, "seq_slots"),
                          _p(positions, I32, "positions"), n, T, W, _f32(h.dtype), -1)
    return out


def shift_save(state: torch.Tensor, h: torch.Tensor, cu_q: torch.Tensor, seq_slots: torch.Tensor,
               positions: torch.Tensor) -> None:
    """state[slot of s] = h[last token of sequence s]."""
    if not _gpu(h, state):
        return ref.shift_save(state, h, cu_q, seq_slots, positions)
    _native().shift_save(_p(state, h.dtype, "state"), _p(h), _p(cu_q, I32), _p(seq_slots, I32), _p(positions, I32),
                         cu_q.shape[0] - 1, h.shape[1], _f32(h.dtype), -1)


def wkv_max_dim() -> int:
    return 128


# Batches of at least WKV_CHUNK_MIN tokens run the recurrence as three passes over chunks of WKV_CHUNK tokens (parallel
# over chunks); shorter ones (decoding, short portions) as one workgroup per sequence.
WKV_CHUNK = int(os.environ.get("K8S_WKV_CHUNK", "64"))
WKV_CHUNK_MIN = int(os.environ.get("K8S_WKV_CHUNK_MIN", "256"))


def wkv_scan(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, z: torch.Tensor, w0: torch.Tensor,
             u: torch.Tensor, lnw: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor, seq_slots: torch.Tensor,
             positions: torch.Tensor, H: int, D: int, eps: float, chunk: Optional[int] = None) -> torch.Tensor:
    """The recurrence with its per-head unit norm, norm weight and silu gate; r, k, v, g [T, H D] (one row stride),
    z [T, H D] fp32 decay logits (w = exp(-exp(z + w0))), ``state`` [slots, H, D, D] fp32 updated in place."""
    T = r.shape[0]
    if z.dtype != F32 or state.dtype != F32:
        raise TypeError("decay logits and recurrent state are fp32")
    if not _gpu(r, state):
        return ref.wkv_scan(r, k, v, g, z, w0, u, lnw, state, cu_q, seq_slots, positions, H, D, eps, r.dtype)
    if D > wkv_max_dim():
        raise ValueError(f"wkv_scan: head dimension {D} exceeds the kernel's {wkv_max_dim()}")
    ld = r.stride(0)
    for t in (r, k, v, g):
        if t.stride(0) != ld or t.stride(1) != 1 or t.dtype != r.dtype:
            raise ValueError("wkv_scan: r, k, v, g must share dtype and row stride")
    out = torch.empty(T, H * D, dtype=r.dtype, device=r.device)
    nseq = cu_q.shape[0] - 1
    Lc = (WKV_CHUNK if T >= WKV_CHUNK_MIN else 0) if chunk is None else int(chunk)
    ws = torch.empty(_native().wkv_workspace(T, nseq, H, D, Lc), dtype=F32, device=r.device) if Lc > 0 else None
    _native().wkv_scan(out.data_ptr(), r.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), ld, _p(z),
                       _p(w0, r.dtype, "w0"), _p(u, r.dtype, "u"), _p(lnw, r.dtype, "lnw"), _p(state),
                       _p(cu_q, I32), _p(seq_slots, I32), _p(positions, I32), nseq, H, D, float(eps),
                       _f32(r.dtype), T, Lc, _p(ws), -1)
    return out


# ----------------------------------------------------------------------------- latent attention
def latent_kv_write(cache: torch.Tensor, dkv: torch.Tensor, normw: torch.Tensor, q: torch.Tensor,
                    cos_sin: torch.Tensor, positions: torch.Tensor, slot_mapping: torch.Tensor, C: int, R: int, H: int,
                    Dn: int, rot_dims: int, eps: float, interleaved: bool = False) -> None:
    """cache[slot] = [rms-norm(dkv[:, :C]) * normw | rotated dkv[:, C:]]; rotates the last R of every head of q
    ([T, H (Dn + R)]) in place.  ``cos_sin`` [positions, rot_dims] = [cos | sin] fp32.  The rotation pairs dimension i
    with i + rot_dims / 2, or (``interleaved``) dimension 2i with 2i + 1.  ``dkv`` [T, C + R] may be a column slice of
    a wider projection."""
    if dkv.dim() != 2 or dkv.shape[1] != C + R:
        raise ValueError("latent_kv_write: dkv must be [T, C + R]")
    if not _gpu(cache, dkv, q):
        return ref.latent_kv_write(cache, dkv, normw, q, cos_sin, positions, slot_mapping, C, R, H, Dn, rot_dims, eps,
                                   interleaved)
    dt = dkv.dtype
    if dkv.stride(1) != 1:
        raise ValueError("latent_kv_write: rows must be contiguous")
    _native().latent_kv_write(_p(cache, dt, "cache"), dkv.data_ptr(), _p(normw, dt, "normw"), _p(q, dt, "q"),
                              _p(cos_sin, F32, "cos_sin"), _p(positions, I32), _p(slot_mapping, I32), dkv.shape[0], C,
                              R, H, Dn, rot_dims, float(eps), _f32(dt), dkv.stride(0), int(bool(interleaved)), -1)


LATENT_MFMA = os.environ.get("K8S_LATENT_MFMA", "1") != "0"   # 0: always the plain-FMA attention kernel


def latent_splits(T: int, H: int, max_keys: int) -> int:
    """Key splits of the MFMA latent attention: one when the (token, 16-head group) grid fills the chip by itself
    (prefill), else enough splits of at least one 32-key step each for about 256 workgroups (decoding)."""
    groups = T * ((H + 15) // 16)
    if groups >= 128:
        return 1
    return max(1, min(256 // groups, (max(1, max_keys) + 31) // 32, 32))


def latent_attention(q_abs: torch.Tensor, q: torch.Tensor, cache: torch.Tensor, block_tables: torch.Tensor,
                     tok_seq: torch.Tensor, positions: torch.Tensor, C: int, R: int, H: int, Dn: int, window: int,
                     scale: float, block_size: int, max_keys: int = 0, cu_q: Optional[torch.Tensor] = None,
                     max_qlen: int = 0, sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Sliding-window attention in the latent space over the paged cache; returns softmax-weighted latents [T, H, C].
    ``max_keys``: an upper bound of the keys any token sees (sizes the key splits; 0: the table's capacity).
    ``cu_q`` / ``max_qlen`` (the sequences' query offsets and longest portion): portions of prompts run four
    consecutive tokens per workgroup, sharing the staged cache rows.
    ``sinks`` [H] fp32: the softmax denominator of head h holds one more term e^sinks[h] (no key, no value).
    bf16 with 16-byte-aligned parts runs on the matrix cores; fp32 and other sizes on the plain-FMA kernel."""
    if sinks is not None and (sinks.dtype != F32 or sinks.numel() != H):
        raise ValueError("latent_attention: sinks are fp32 [H]")
    if not _gpu(q_abs, q, cache, sinks):
        return ref.latent_attention(q_abs, q, cache, block_tables, tok_seq, positions, C, R, H, Dn, window, scale,
                                    block_size, q.dtype, sinks)
    T = q.shape[0]
    dt = q.dtype
    out = torch.empty(T, H, C, dtype=dt, device=q.device)
    nat = _native()
    args = (_p(q_abs, dt, "q_abs"), _p(q), _p(cache, dt, "cache"), _p(block_tables, I32, "block_tables"),
            block_tables.shape[1], _p(tok_seq, I32), _p(positions, I32), T, C, R, H, Dn, int(window), float(scale),
            block_size)
    if LATENT_MFMA and dt == BF16 and nat.latent_mfma_ok(C, R, Dn):
        cap = block_tables.shape[1] * block_size
        bound = min(max_keys or cap, window or cap, cap)
        ns = latent_splits(T, H, bound)
        pacc = pml = None
        if ns > 1:
            HP = (H + 15) // 16 * 16
            pacc = torch.empty(T * HP * ns * C, dtype=F32, device=q.device)
            pml = torch.empty(T * HP * ns * 2, dtype=F32, device=q.device)
        nseq = cu_q.shape[0] - 1 if cu_q is not None else 0
        nat.latent_attention_mfma(out.data_ptr(), _p(pacc), _p(pml), *args, ns, _p(cu_q, I32, "cu_q"), nseq,
                                  int(max_qlen), _p(sinks), -1)
    else:
        nat.latent_attention(out.data_ptr(), *args, _f32(dt), _p(sinks), -1)
    return out


# ----------------------------------------------------------------------------- mixture of experts
def moe_route(logits: torch.Tensor, E: int, top: int, scale: float, score: str = "softmax"):
    """fp32 router logits [T, >= E] -> (expert ids int32 [T, top], weights fp32 [T, top]).  ``score``: "softmax"
    (weights renormalised over the chosen experts) or "sigmoid" (the chosen experts' scores as they are)."""
    if logits.dtype != F32:
        raise TypeError("router logits are fp32")
    if score not in ("softmax", "sigmoid"):
        raise ValueError(f"moe_route: unknown score {score!r}")
    if not _gpu(logits):
        return ref.moe_route(logits, E, top, scale, score)
    T = logits.shape[0]
    idx = torch.empty(T, top, dtype=I32, device=logits.device)
    w = torch.empty(T, top, dtype=F32, device=logits.device)
    _native().moe_route(idx.data_ptr(), w.data_ptr(), _p(logits), logits.stride(0), T, E, top, float(scale),
                        int(score == "sigmoid"), -1)
    return idx, w


def moe_align(topk_idx: torch.Tensor, E: int):
    """(sorted_tok [P], pos_of_pair [P], seg [E + 1], tiles [n, 3]) for the grouped GEMMs; no host sync."""
    if not _gpu(topk_idx):
        return ref.moe_align(topk_idx, E, GROUP_BM)
    T, top = topk_idx.shape
    P = T * top
    ntiles = (P + GROUP_BM - 1) // GROUP_BM + E
    dev = topk_idx.device
    sorted_tok = torch.empty(P, dtype=I32, device=dev)
    pos = torch.empty(P, dtype=I32, device=dev)
    seg = torch.empty(E + 1, dtype=I32, device=dev)
    tiles = torch.empty(ntiles, 3, dtype=I32, device=dev)
    _native().moe_align(sorted_tok.data_ptr(), pos.data_ptr(), seg.data_ptr(), tiles.data_ptr(), ntiles,
                        _p(topk_idx, I32, "topk_idx"), P, top, E, GROUP_BM, -1)
    return sorted_tok, pos, seg, tiles


def moe_combine(D: torch.Tensor, pos_of_pair: torch.Tensor, topk_w: Optional[torch.Tensor],
                shared: Optional[torch.Tensor], logits: Optional[torch.Tensor], sg_col: int, top: int = 0) -> torch.Tensor:
    """z[t] = sum_k w[t, k] D[pos[t, k]] + sigmoid(logits[t, sg_col]) * shared[t]  (sg_col < 0: ungated).
    ``topk_w`` None (with ``top`` given): a plain sum, for experts whose weight scaled their input."""
    top = topk_w.shape[1] if topk_w is not None else int(top)
    if top <= 0 or pos_of_pair.numel() % top:
        raise ValueError("moe_combine: the choices per token are needed")
    if sg_col >= 0 and logits is None:
        raise ValueError("moe_combine: a gated shared expert needs the router logits")
    if not _gpu(D, topk_w, shared):
        return ref.moe_combine(D, pos_of_pair, topk_w, shared, logits, sg_col, D.dtype, top)
    T = pos_of_pair.numel() // top
    W = D.shape[1]
    z = torch.empty(T, W, dtype=D.dtype, device=D.device)
    _native().moe_combine(z.data_ptr(), _p(D), _p(pos_of_pair, I32), _p(topk_w, F32), _p(shared, D.dtype, "shared"),
                          _p(logits, F32), logits.stride(0) if logits is not None else 0, sg_col, T, W, top,
                          _f32(D.dtype), -1)
    return z


# ----------------------------------------------------------------------------- windowed attention with pooled blocks
def pool_entries_per_page(block_size: int, P: int) -> int:
    """Pooled blocks of P tokens that can start inside one cache page."""
    return -(-block_size // P) if P > 0 else 0


def window_kv_write(kcache: torch.Tensor, vcache: torch.Tensor, qkv: torch.Tensor, koff: int, voff: int,
                    qb: Optional[torch.Tensor], kb: Optional[torch.Tensor], vb: Optional[torch.Tensor],
                    cos_sin: Optional[torch.Tensor], positions: torch.Tensor, slot_mapping: torch.Tensor, H: int, G: int,
                    D: int, V: int, dims: int, eps: float, unit: bool = True, *,
                    vfirst_in: Optional[torch.Tensor] = None, vfirst_out: Optional[torch.Tensor] = None,
                    lam: float = 0.0, half_layout: bool = False, qnw: Optional[torch.Tensor] = None,
                    knw: Optional[torch.Tensor] = None, head_qnw: Optional[torch.Tensor] = None,
                    head_knw: Optional[torch.Tensor] = None) -> None:
    """Prepares a projected row [q (H D) | ... k (G D at ``koff``) ... v (G V at ``voff``) ...] of every token: biases,
    rotation of the dimension pairs (2i, 2i + 1), i < dims / 2, by ``cos_sin[pos]`` = [cos | sin] (fp32), unit RMS per
    head of q and k (``unit``), value mixing v <- (1 - lam) v + lam ``vfirst_in`` [T, G V] fp32; the first mixing layer
    leaves its v in ``vfirst_out``.  q is rewritten in place; k and v go to the paged caches [slots, G, D] / [slots, G, V].
    ``half_layout``: the rotation pairs dimension i with i + dims / 2 instead.  ``qnw`` [H D] / ``knw`` [G D]: before the
    rotation the whole projection (all heads at once) is divided by its root mean square and multiplied by the weight.
    ``head_qnw`` / ``head_knw`` [D]: before the rotation every head is divided by its own root mean square and
    multiplied by the weight, which all heads share.
    ``kcache`` None (a layer that attends another layer's cache): only the queries are prepared."""
    dt = qkv.dtype
    if kcache is None:
        vcache, G, koff, voff = None, 0, 0, 0
    if qkv.dim() != 2 or qkv.stride(1) != 1:
        raise ValueError("window_kv_write: the projected rows must be contiguous")
    if koff + G * D > qkv.shape[1] or voff + G * V > qkv.shape[1] or H * D > qkv.shape[1]:
        raise ValueError("window_kv_write: part offsets exceed the projected row")
    if not _gpu(kcache, vcache, qkv):
        return ref.window_kv_write(kcache, vcache, qkv, koff, voff, qb, kb, vb, cos_sin, positions, slot_mapping,
                                   vfirst_in, vfirst_out, lam, H, G, D, V, dims, eps, unit, half_layout, qnw, knw,
                                   head_qnw, head_knw)
    T = qkv.shape[0]
    if cos_sin is not None and (cos_sin.shape[1] != dims or cos_sin.dtype != F32):
        raise ValueError("window_kv_write: the angle table must be fp32 [positions, dims]")
    for t in (vfirst_in, vfirst_out):
        if t is not None and (t.shape != (T, G * V) or t.dtype != F32):
            raise ValueError("window_kv_write: mixed values are fp32 [T, G V]")
    for t in (head_qnw, head_knw):
        if t is not None and t.numel() != D:
            raise ValueError("window_kv_write: per-head norm weights are [D]")
    _native().window_kv_write(_p(kcache, dt, "kcache"), _p(vcache, dt, "vcache"), qkv.data_ptr(), qkv.stride(0), koff,
                              voff, _p(qb, dt, "qb"), _p(kb, dt, "kb"), _p(vb, dt, "vb"), _p(cos_sin),
                              _p(positions, I32), _p(slot_mapping, I32), _p(vfirst_in), _p(vfirst_out), float(lam), T, H,
                              G, D, V, dims, float(eps), int(bool(unit)), int(bool(half_layout)), _p(qnw, dt, "qnw"),
                              _p(knw, dt, "knw"), _p(head_qnw, dt, "head_qnw"), _p(head_knw, dt, "head_knw"),
                              _f32(dt), -1)


def window_pool(kpool: torch.Tensor, vpool: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                block_tables: torch.Tensor, tok_seq: torch.Tensor, positions: torch.Tensor, P: int,
                block_size: int) -> None:
    """For every token of the batch that ends a block of P tokens ((pos + 1) % P == 0): the fp32 mean of the block's
    cached keys / values -> kpool / vpool [pages * ceil(block_size / P), G, D or V] (the block's entry lives with the
    page of its first token).  Call after :func:`window_kv_write` of the same batch."""
    if P <= 0:
        return
    if kpool.dtype != F32 or vpool.dtype != F32:
        raise TypeError("pooled keys / values are fp32")
    if not _gpu(kpool, vpool, kcache, vcache):
        return ref.window_pool(kpool, vpool, kcache, vcache, block_tables, tok_seq, positions, P, block_size)
    G, D, V = kcache.shape[1], kcache.shape[2], vcache.shape[2]
    _native().window_pool(_p(kpool), _p(vpool), _p(kcache), _p(vcache, kcache.dtype, "vcache"),
                          _p(block_tables, I32, "block_tables"), block_tables.shape[1], _p(tok_seq, I32),
                          _p(positions, I32), positions.shape[0], G, D, V, P, block_size, _f32(kcache.dtype), -1)


WINDOW_MFMA = os.environ.get("K8S_WINDOW_MFMA", "1") != "0"   # 0: always the plain-FMA attention kernel


def window_splits(T: int, G: int, window: int, P: int, max_pos: int, tile_rows: int) -> int:
    """Key splits of the plain windowed attention: one when the (token, key head) grid fills the chip several times over
    by itself, else enough splits of at least one tile each for about 1024 workgroups (a workgroup walks its tiles one
    after the other, so decoding wants them spread).  ``max_pos``: positions a token can have."""
    groups = T * G
    if groups >= 1024 or tile_rows <= 0:
        return 1
    keys = max_pos if window <= 0 else min(max_pos, window + (max_pos // P if P > 0 else 0))
    return max(1, min(-(-1024 // groups), -(-max(1, keys) // tile_rows), 16))


def window_attention(q: torch.Tensor, gate: Optional[torch.Tensor], kcache: torch.Tensor, vcache: torch.Tensor,
                     kpool: Optional[torch.Tensor], vpool: Optional[torch.Tensor], block_tables: torch.Tensor,
                     tok_seq: torch.Tensor, positions: torch.Tensor, H: int, window: int, P: int, scale: float,
                     sink: bool, block_size: int, cu_q: Optional[torch.Tensor] = None, max_qlen: int = 0,
                     max_keys: int = 0, *, chunk: int = 0, softcap: float = 0.0, sinks: Optional[torch.Tensor] = None,
                     gate_per_head: bool = False) -> torch.Tensor:
    """Grouped-query attention over the paged caches [slots, G, D] / [slots, G, V]: the token at position p sees the
    tokens max(0, p - window + 1) .. p (``window`` <= 0: all) and, with ``P`` > 0, the pooled blocks that lie wholly
    before the window (b P + P - 1 <= p - window), all in one softmax; ``sink``: one more unit in the denominator.
    ``q`` [T, >= H D] (row stride free, the prepared queries first), ``gate`` [T, H V] (row stride free): the result is
    multiplied by sigmoid(gate); ``gate_per_head``: ``gate`` is [T, H], one number per head.  Returns [T, H V].
    ``chunk`` > 0 (instead of a window): positions are cut into chunks of that many, counted from 0, and a token sees
    the tokens of its own chunk up to itself.  ``softcap`` > 0: scores become softcap tanh(score / softcap).  ``sinks``
    [H] fp32 (with ``sink``): the extra term of head h is e^sinks[h] instead of 1.
    ``cu_q`` / ``max_qlen`` (the sequences' query offsets and longest portion): bf16 portions of prompts whose sizes
    fit run on the matrix cores, tiles of consecutive tokens sharing the staged keys; anything else (fp32, single
    tokens, other sizes) on the plain-FMA kernel, which splits the keys of few tokens over several workgroups
    (``max_keys``: an upper bound of the positions any token sees, 0: the block tables' capacity)."""
    G, D, V = kcache.shape[1], kcache.shape[2], vcache.shape[2]
    if H % G:
        raise ValueError(f"window_attention: {H} query heads over {G} key heads")
    if chunk > 0 and window > 0:
        raise ValueError("window_attention: a window or chunks, not both")
    if window <= 0:
        P = 0
    if sinks is not None and (not sink or sinks.dtype != F32 or sinks.numel() != H):
        raise ValueError("window_attention: sinks are fp32 [H] and go with sink=True")
    if not _gpu(q, kcache, vcache):
        return ref.window_attention(q, gate, kcache, vcache, kpool, vpool, block_tables, tok_seq, positions, H, G, D, V,
                                    window, P, scale, sink, block_size, q.dtype, chunk, softcap, sinks, gate_per_head)
    T = q.shape[0]
    dt = q.dtype
    if q.stride(1) != 1 or (gate is not None and (gate.stride(1) != 1 or gate.dtype != dt)):
        raise ValueError("window_attention: q and gate rows must be contiguous and of one dtype")
    out = torch.empty(T, H * V, dtype=dt, device=q.device)
    nat = _native()
    if (WINDOW_MFMA and dt == BF16 and cu_q is not None and max_qlen > 1 and nat.window_mfma_ok(H, G, D, V)
            and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0):
        nat.window_attention_mfma(out.data_ptr(), q.data_ptr(), q.stride(0), gate.data_ptr() if gate is not None else 0,
                                  gate.stride(0) if gate is not None else 0, _p(kcache, dt, "kcache"),
                                  _p(vcache, dt, "vcache"), _p(kpool, F32, "kpool"), _p(vpool, F32, "vpool"),
                                  _p(block_tables, I32, "block_tables"), block_tables.shape[1], _p(cu_q, I32, "cu_q"),
                                  _p(positions, I32), cu_q.shape[0] - 1, int(max_qlen), H, G, D, V, int(window), int(P),
                                  float(scale), int(bool(sink)), block_size, int(chunk), float(softcap), _p(sinks),
                                  int(bool(gate_per_head)), -1)
        return out
    ns = window_splits(T, G, window if chunk <= 0 else chunk, P, max_keys or block_tables.shape[1] * block_size,
                       nat.window_tile_rows(H, G, D, V))
    pacc = pml = None
    if ns > 1:
        pacc = torch.empty(T * H * ns * V, dtype=F32, device=q.device)
        pml = torch.empty(T * H * ns * 2, dtype=F32, device=q.device)
    nat.window_attention(out.data_ptr(), _p(pacc), _p(pml), q.data_ptr(), q.stride(0),
                         gate.data_ptr() if gate is not None else 0, gate.stride(0) if gate is not None else 0,
                         _p(kcache, dt, "kcache"), _p(vcache, dt, "vcache"), _p(kpool, F32, "kpool"),
                         _p(vpool, F32, "vpool"), _p(block_tables, I32, "block_tables"), block_tables.shape[1],
                         _p(tok_seq, I32), _p(positions, I32), T, H, G, D, V, int(window), int(P), float(scale),
                         int(bool(sink)), block_size, ns, int(chunk), float(softcap), _p(sinks), int(bool(gate_per_head)),
                         _f32(dt), -1)
    return out


# ----------------------------------------------------------------------------- gated matrix-state recurrences
def gated_scan_max_dim() -> int:
    return 256


def gated_scan_record(kind: int, D: int, V: int) -> int:
    """fp32 values of one (slot, head) state record: S [D, V] (SCAN_MLSTM: then n [D] and the running maximum)."""
    return ref.gated_scan_record(kind, D, V)


# Batches of at least SCAN_CHUNK_MIN tokens run the recurrences as three passes over chunks of SCAN_CHUNK tokens (parallel
# over chunks); shorter ones (decoding, short portions) as one workgroup per sequence.
SCAN_CHUNK = int(os.environ.get("K8S_SCAN_CHUNK", "64"))
SCAN_CHUNK_MIN = int(os.environ.get("K8S_SCAN_CHUNK_MIN", "256"))


def gated_scan(proj: torch.Tensor, kind: int, cols: dict, normw: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor,
               seq_slots: torch.Tensor, positions: torch.Tensor, H: int, D: int, V: int, eps: float, out_dtype, *,
               fbias: Optional[torch.Tensor] = None, ibias: Optional[torch.Tensor] = None,
               lower: Optional[torch.Tensor] = None, cap: float = 0.0, chunk: Optional[int] = None,
               aux: Optional[torch.Tensor] = None, head_params: Optional[torch.Tensor] = None,
               groups: int = 0) -> torch.Tensor:
    """A gated linear recurrence with a matrix state per head over a varlen batch; ``proj`` fp32 [T, ld] is the fused
    input projection with its parts at the column offsets ``cols``; ``state`` [slots, H, record] fp32 is updated in
    place (a portion at position 0 starts from zero).  Returns the normed (and, SCAN_MLSTM, gated) outputs [T, H V].
    SCAN_HGRN2: cols q, f, v; ``lower`` [H D], ``fbias`` [H D], ``normw`` [V].
    SCAN_MLSTM: cols q, k, v, i, f, g; ``ibias`` / ``fbias`` [H], ``cap`` > 0, ``normw`` [H V].
    SCAN_SSD (a scalar decay per head and token, set by a step size): ``proj`` holds v (the heads' inputs x, H V),
    k (B) and q (C) (``groups`` D each; head h uses group h // (H / groups)); ``aux`` fp32 [T, lda] holds f (the step
    size logits, H) and g (the output gate, H V) at ``cols``; ``head_params`` fp32 [3, H] = -exp(A_log), dt_bias, skip.
    dt = softplus(f + dt_bias); S <- exp(-exp(A_log) dt) S + dt B x^T; y = (S^T C + skip x) silu(g), returned in fp32
    without a norm (``normw`` None, ``out_dtype`` fp32)."""
    if proj.dtype != F32 or state.dtype != F32:
        raise TypeError("the recurrence's inputs and state are fp32")
    if proj.dim() != 2 or proj.stride(1) != 1:
        raise ValueError("gated_scan: projected rows must be contiguous")
    need = {SCAN_HGRN2: ("q", "f", "v"), SCAN_MLSTM: ("q", "k", "v", "i", "f", "g"),
            SCAN_SSD: ("q", "k", "v", "f", "g")}[kind]
    G = int(groups) if kind == SCAN_SSD else H
    width = {"q": G * D, "k": G * D, "v": H * V, "g": H * V, "i": H, "f": H * D if kind == SCAN_HGRN2 else H}
    if kind == SCAN_SSD:
        if aux is None or head_params is None or G <= 0 or H % G:
            raise ValueError("gated_scan: SCAN_SSD needs aux, head_params and groups that divide the heads")
        if aux.dtype != F32 or aux.stride(1) != 1 or aux.shape[0] != proj.shape[0]:
            raise TypeError("gated_scan: aux is fp32 [T, lda] with contiguous rows")
        if head_params.dtype != F32 or head_params.shape != (3, H) or not head_params.is_contiguous():
            raise TypeError("gated_scan: head_params is contiguous fp32 [3, H]")
        if out_dtype != F32:
            raise TypeError("gated_scan: SCAN_SSD returns fp32")
    for key in need:
        src = aux if kind == SCAN_SSD and key in ("f", "g") else proj
        if cols[key] < 0 or cols[key] + width[key] > src.shape[1]:
            raise ValueError(f"gated_scan: part {key!r} exceeds the projected row")
    if state.shape[1:] != (H, gated_scan_record(kind, D, V)):
        raise ValueError("gated_scan: state must be [slots, H, record]")
    if not _gpu(proj, state):
        return ref.gated_scan(proj, kind, cols, fbias, ibias, lower, normw, state, cu_q, seq_slots, positions, H, D, V,
                              eps, cap, out_dtype, aux, head_params, G)
    if max(D, V) > gated_scan_max_dim():
        raise ValueError(f"gated_scan: head sizes {D} x {V} exceed the kernel's {gated_scan_max_dim()}")
    T = proj.shape[0]
    out = torch.empty(T, H * V, dtype=out_dtype, device=proj.device)
    c = lambda key: int(cols.get(key, 0))
    nseq = cu_q.shape[0] - 1
    Lc = (SCAN_CHUNK if T >= SCAN_CHUNK_MIN else 0) if chunk is None else int(chunk)
    ws = torch.empty(_native().gated_scan_workspace(T, nseq, H, D, V, Lc), dtype=F32, device=proj.device) if Lc > 0 \
        else None
    _native().gated_scan(out.data_ptr(), _p(proj), proj.stride(0), kind, c("q"), c("k"), c("v"), c("i"), c("f"), c("g"),
                         _p(fbias, out_dtype, "fbias"), _p(ibias, out_dtype, "ibias"), _p(lower, out_dtype, "lower"),
                         _p(normw, out_dtype, "normw"), _p(state), _p(cu_q, I32), _p(seq_slots, I32),
                         _p(positions, I32), nseq, H, D, V, float(eps), float(cap), _f32(out_dtype), T, Lc, _p(ws),
                         aux.data_ptr() if aux is not None else 0, aux.stride(0) if aux is not None else 0,
                         _p(head_params), H // G, -1)
    return out


# ----------------------------------------------------------------------------- short convolutions, delta rule, RG-LRU
CONV_MAX_TAPS = 16


def short_conv(x: torch.Tensor, w: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor, tok_seq: torch.Tensor,
               seq_slots: torch.Tensor, positions: torch.Tensor, *, in_bias: Optional[torch.Tensor] = None,
               out_bias: Optional[torch.Tensor] = None, act: int = CONV_NONE, unit_cols: int = 0, unit_dim: int = 0,
               scale_cols: int = 0, scale: float = 1.0, unit_eps: float = 1e-6, residual: bool = False,
               out_dtype=F32) -> torch.Tensor:
    """Causal convolution over time per channel over a varlen batch, in fp32.  ``x`` fp32 [T, C] (row stride free),
    ``w`` fp32 [C, taps] (the last tap is the current token's); inputs are x + in_bias, zeros before position 0; the
    taps - 1 inputs before a portion come from ``state`` [slots, taps - 1, C] fp32, which then receives the portion's
    last inputs (a portion at position 0 starts from zeros).  Then out_bias, the activation (CONV_SILU), and, for the
    first ``unit_cols`` channels in groups of ``unit_dim``, v / sqrt(sum(v^2) + unit_eps); the first ``scale_cols``
    channels times ``scale``.  ``residual``: the token's own input is added to the result (x + conv(x)).  Returns
    [T, C] in ``out_dtype`` (fp32, or bf16 for a result that feeds a bf16 projection)."""
    T, C = x.shape
    taps = w.shape[1]
    if x.dtype != F32 or w.dtype != F32 or state.dtype != F32 or x.stride(1) != 1:
        raise TypeError("short_conv: inputs, taps and state are fp32 with contiguous rows")
    if w.shape[0] != C or taps < 1 or taps > CONV_MAX_TAPS or state.shape[1:] != (max(taps - 1, 0), C):
        raise ValueError("short_conv: taps [C, n] and state [slots, n - 1, C] must fit the input")
    if unit_cols and (unit_dim <= 0 or unit_cols % unit_dim or unit_cols > C or unit_dim > 256):
        raise ValueError("short_conv: unit groups must tile the leading channels")
    if scale_cols > C:
        raise ValueError("short_conv: scale_cols exceeds the channels")
    if not _gpu(x, w, state):
        return ref.short_conv(x, w, state, cu_q, seq_slots, positions, in_bias, out_bias, act, unit_cols, unit_dim,
                              scale_cols, scale, unit_eps, residual).to(out_dtype)
    out = torch.empty(T, C, dtype=out_dtype, device=x.device)
    _native().short_conv(out.data_ptr(), x.data_ptr(), x.stride(0), _p(w), _p(state), _p(cu_q, I32, "cu_q"),
                         _p(tok_seq, I32, "tok_seq"), _p(seq_slots, I32, "seq_slots"), _p(positions, I32, "positions"),
                         _p(in_bias, F32, "in_bias"), _p(out_bias, F32, "out_bias"), int(act), T, C, taps,
                         cu_q.shape[0] - 1, int(unit_cols), int(unit_dim), int(scale_cols), float(scale),
                         float(unit_eps), int(bool(residual)), _f32(out_dtype), -1)
    return out


def delta_scan_max_dim() -> int:
    return 256


def delta_scan(qkv: torch.Tensor, proj: torch.Tensor, cols: dict, neg_a: torch.Tensor, dt_bias: torch.Tensor,
               normw: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor, seq_slots: torch.Tensor,
               positions: torch.Tensor, H: int, G: int, D: int, V: int, eps: float, out_dtype,
               chunk: Optional[int] = None) -> torch.Tensor:
    """The gated delta rule with a matrix state per head over a varlen batch.  ``qkv`` fp32 [T, G D | G D | H V]: the
    prepared queries (unit vectors times D^-1/2), keys (unit vectors) and values; ``proj`` fp32 [T, ld] holds the
    columns ``cols`` b (H: beta = sigmoid), a (H: decay = exp(neg_a softplus(a + dt_bias))) and g (H V: output gate,
    silu); ``neg_a`` / ``dt_bias`` / ``normw`` fp32 [H] / [H] / [V].  Per head, with the queries / keys of head
    h // (H / G): S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q; y = o / rms(o) * normw * silu(g).
    ``state`` [slots, H, D V] fp32 is updated in place (a portion at position 0 starts from zero).  [T, H V].
    Batches of at least SCAN_CHUNK_MIN tokens run as three passes over chunks of SCAN_CHUNK tokens, parallel over chunks
    (``chunk``: another chunk length, 0: one workgroup per sequence)."""
    T = qkv.shape[0]
    for t, n in ((qkv, "qkv"), (proj, "proj"), (state, "state"), (neg_a, "neg_a"), (dt_bias, "dt_bias"),
                 (normw, "normw")):
        if t.dtype != F32:
            raise TypeError(f"delta_scan: {n} is fp32")
    if H % G or qkv.shape[1] != 2 * G * D + H * V or not qkv.is_contiguous() or proj.stride(1) != 1:
        raise ValueError("delta_scan: qkv must be contiguous [T, G D | G D | H V]")
    for key, wd in (("b", H), ("a", H), ("g", H * V)):
        if cols[key] < 0 or cols[key] + wd > proj.shape[1]:
            raise ValueError(f"delta_scan: part {key!r} exceeds the projected row")
    if state.shape[1:] != (H, D * V):
        raise ValueError("delta_scan: state must be [slots, H, D V]")
    if not _gpu(qkv, proj, state):
        return ref.delta_scan(qkv, proj, cols, neg_a, dt_bias, normw, state, cu_q, seq_slots, positions, H, G, D, V, eps,
                              out_dtype)
    if max(D, V) > delta_scan_max_dim():
        raise ValueError(f"delta_scan: head sizes {D} x {V} exceed the kernel's {delta_scan_max_dim()}")
    out = torch.empty(T, H * V, dtype=out_dtype, device=qkv.device)
    nat = _native()
    nseq = cu_q.shape[0] - 1
    Lc = (SCAN_CHUNK if T >= SCAN_CHUNK_MIN else 0) if chunk is None else int(chunk)
    if Lc > 0 and not nat.delta_scan_chunks_ok(D, V):
        Lc = 0
    ws = torch.empty(nat.delta_scan_workspace(T, nseq, H, D, V, Lc), dtype=F32, device=qkv.device) if Lc > 0 else None
    nat.delta_scan(out.data_ptr(), _p(qkv), _p(proj), proj.stride(0), int(cols["b"]), int(cols["a"]), int(cols["g"]),
                   _p(neg_a), _p(dt_bias), _p(normw), _p(state), _p(cu_q, I32), _p(seq_slots, I32), _p(positions, I32),
                   nseq, H, G, D, V, float(eps), _f32(out_dtype), T, Lc, _p(ws), -1)
    return out


def rglru_scan(u: torch.Tensor, gates: torch.Tensor, gate_bias: torch.Tensor, decay_rate: torch.Tensor,
               proj: torch.Tensor, ycol: int, ybias: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor,
               seq_slots: torch.Tensor, positions: torch.Tensor, blocks: int, out_dtype, max_qlen: int = 0
               ) -> torch.Tensor:
    """The real-gated linear recurrent unit per channel over a varlen batch.  ``u`` fp32 [T, C] (the convolved
    branch); ``gates`` fp32 [T, blocks, 2 C / blocks]: per block the logits of the recurrence gate r, then of the
    input gate i (``gate_bias`` [blocks, 2 C / blocks] added, sigmoid); a = exp(decay_rate r) with ``decay_rate``
    [C] <= 0; S <- a S + sqrt(1 - a^2) i u; out = S gelu_tanh(proj[:, ycol + c] + ybias[c]).  ``state`` [slots, C]
    fp32 is updated in place (a portion at position 0 starts from zero).  ``max_qlen``: the longest portion (long
    portions are cut into time slices that run side by side and are joined exactly)."""
    T, C = u.shape
    for t, n in ((u, "u"), (gates, "gates"), (gate_bias, "gate_bias"), (decay_rate, "decay_rate"), (proj, "proj"),
                 (ybias, "ybias"), (state, "state")):
        if t.dtype != F32:
            raise TypeError(f"rglru_scan: {n} is fp32")
    if C % blocks or gates.numel() != T * 2 * C or not gates.is_contiguous() or not u.is_contiguous():
        raise ValueError("rglru_scan: gates must be contiguous [T, blocks, 2 C / blocks]")
    if ycol < 0 or ycol + C > proj.shape[1] or proj.stride(1) != 1 or state.shape[1:] != (C,):
        raise ValueError("rglru_scan: the gate branch exceeds the projected row, or state is not [slots, C]")
    if not _gpu(u, gates, state):
        return ref.rglru_scan(u, gates, gate_bias, decay_rate, proj, ycol, ybias, state, cu_q, seq_slots, positions, C,
                              blocks, out_dtype)
    out = torch.empty(T, C, dtype=out_dtype, device=u.device)
    _native().rglru_scan(out.data_ptr(), _p(u), _p(gates), _p(gate_bias), _p(decay_rate), _p(proj), proj.stride(0),
                         int(ycol), _p(ybias), _p(state), _p(cu_q, I32), _p(seq_slots, I32), _p(positions, I32),
                         cu_q.shape[0] - 1, C, blocks, int(max_qlen or T), _f32(out_dtype), -1)
    return out
