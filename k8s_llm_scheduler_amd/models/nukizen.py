"""Nukizen: a decoder with an fp32 residual stream and parallel blocks, ``h = norm(x); x += mixer(h) + ff(h)`` (one
RMS norm per layer, read by both sublayers), a dense feed-forward ``W_down (relu(W_gate h) * W_up h)`` and three mixers
in any order the config lists:

* ``attention``: grouped-query attention without biases; rotary positions in the half layout (dimension i turns with
  i + dims / 2) on the first ``rot.dims`` dimensions of each head, frequencies ``base^(-2i / dims)``; scores
  ``q . k * scale`` soft-capped to ``cap tanh(s / cap)``; a chunked mask (positions are cut into chunks of ``mask.size``
  counted from 0, a token sees its own chunk up to itself); a sigmoid output gate of one number per head.  With
  ``kv_from: j`` the layer has no key / value projections and attends layer j's cache with its own queries.
* ``rglru``: two branches of ``width`` channels, ``y = gelu_tanh(W_y h + b)`` and ``u = conv(W_x h + b)`` (a short
  causal convolution per channel); block-diagonal gates ``r, i = sigmoid(W_b u_b + b)``; ``a = exp(-8 r softplus(lam))``,
  ``S <- a S + sqrt(1 - a^2) i u``; output ``W_o (S y)``.
* ``parallel``: two mixers side by side on the same input, each output RMS-normed over the model width with its own
  weight, half their sum.  Left: attention as above with an RMS norm over the whole query / key projection before the
  rotation, YaRN-scaled frequencies (``rot.scaling``), no soft cap, and a learned sink per head in the softmax's
  denominator (``e^sink``, no value).  Right: the gated delta rule -- q, k, v pass a short causal convolution and
  silu; q, k become unit vectors per head (q times ``dim^(-1/2)``); ``beta = sigmoid(W_b h)``,
  ``g = exp(-exp(A_log) softplus(W_a h + dt_bias))``; ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``;
  each head's output RMS-normed with a weight shared by the heads, times ``silu(W_g h)``.

The logits are soft-capped (``logit_softcap``).  Every optional part is keyed by the config or by the presence of its
tensor: no mask means every earlier token, no ``rot`` no rotation, no ``softcap`` none, no ``.g`` / ``.sink`` /
``.q.norm`` tensor none of that.

The model presents the engine's interface through :class:`~.stream.StreamModel`; caches: per attention mixer with
projections of its own a paged K / V cache (layers with ``kv_from`` read another mixer's), per recurrent mixer fp32
records per request slot (the recurrent state and the convolutions' last inputs).  Every op is a kernel of
:mod:`..ops.seqmix`; ``dtype=float32`` runs everything in true fp32.  Single rank (TP = 1).
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from pathlib import Path
from typing import Dict, List, Optional

import torch

from ..ops import reference as ref
from ..ops import seqmix as sm
from ..parallel import TPGroup
from . import stream
from .stream import StreamModel

ARCHITECTURE = "Nukizen"
MIXERS = ("attention", "rglru", "parallel")
F32 = torch.float32
DECAY_RATE = -8.0        # log a = DECAY_RATE * r * softplus(lam)
UNIT_EPS = 1e-6          # unit vectors of the delta rule: x / sqrt(sum(x^2) + UNIT_EPS)


# ----------------------------------------------------------------------------- configuration
@dataclass
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int = 0               # 0: every earlier token is seen
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: Optional[dict] = None   # {"factor", "original", "fast", "slow"}
    softcap: float = 0.0
    kv_from: Optional[int] = None
    qk_norm: bool = False        # RMS norm over the whole q / k projection (tensors q.norm, k.norm)
    sink: bool = False           # a learned term per head in the softmax's denominator (tensor sink)
    gate: bool = False           # sigmoid output gate, one number per head (tensor g)


@dataclass
class DeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass
class RglruConfig:
    width: int
    blocks: int
    conv: int


@dataclass
class LayerConfig:
    type: str
    mixer: object                # AttentionConfig | RglruConfig | (AttentionConfig, DeltaConfig)
    ff: int = 0                  # 0: no feed-forward


@dataclass
class NukizenConfig:
    name: str
    vocab: int
    hidden: int
    layers: List[LayerConfig]
    rms_eps: float = 1e-6
    logit_softcap: float = 0.0
    max_position: int = 1 << 20
    bos_id: int = 0
    eos_ids: tuple = ()
    extra: dict = field(default_factory=dict)
    token_ids_only = True    # checkpoints of this design ship no tokenizer: requests are token ids

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def validate_tp(self, tp: int) -> None:
        if tp != 1:
            raise ValueError(f"{self.name}: this design runs on one rank (tp={tp})")


def _attention_from(d: dict, side: bool) -> AttentionConfig:
    """``side``: the attention of a ``parallel`` mixer (whole-projection norms and a sink); else gated heads."""
    rot, mask = d.get("rot") or {}, d.get("mask") or {}
    dim = int(d["dim"])
    kv_from = d.get("kv_from")
    return AttentionConfig(heads=int(d["heads"]), kv_heads=int(d.get("kv_heads") or d["heads"]), dim=dim,
                           vdim=int(d.get("vdim") or dim), scale=float(d.get("scale", 1.0 / math.sqrt(dim))),
                           chunk=int(mask.get("size") or 0), rot_dims=int(rot.get("dims") or 0),
                           rot_base=float(rot.get("base", 10000.0)), rot_scaling=dict(rot["scaling"]) if rot.get("scaling") else None,
                           softcap=float(d.get("softcap") or 0.0), kv_from=None if kv_from is None else int(kv_from),
                           qk_norm=bool(d.get("qk_norm", side)), sink=bool(d.get("sink", side)),
                           gate=bool(d.get("gate", not side)))


def _layer_from(l: dict) -> LayerConfig:
    kind, d = l["type"], l["mixer"]
    if kind == "attention":
        mixer: object = _attention_from(d, False)
    elif kind == "rglru":
        mixer = RglruConfig(int(d["width"]), int(d.get("blocks") or 1), int(d.get("conv") or 1))
    elif kind == "parallel":
        r = d["right"]
        mixer = (_attention_from(d["left"], True),
                 DeltaConfig(int(r["heads"]), int(r.get("kv_heads") or r["heads"]), int(r["dim"]),
                             int(r.get("vdim") or r["dim"]), int(r.get("conv") or 1)))
    else:
        raise ValueError(f"unknown mixer type {kind!r} (known: {', '.join(MIXERS)})")
    mlp = l.get("mlp")
    if mlp is not None and mlp.get("kind", "dense") != "dense":
        raise ValueError(f"unknown mlp kind {mlp['kind']!r}")
    return LayerConfig(kind, mixer, int(mlp["ff"]) if mlp else 0)


def config_from_json(c: dict, name: str = "nukizen") -> NukizenConfig:
    return NukizenConfig(name=name, vocab=int(c["vocab"]), hidden=int(c["width"]),
                         layers=[_layer_from(l) for l in c["layers"]],
                         rms_eps=float((c.get("norm") or {}).get("eps", 1e-6)),
                         logit_softcap=float(c.get("logit_softcap") or 0.0))


def _attention_json(a: AttentionConfig, side: bool) -> dict:
    d: dict = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale}
    if a.chunk:
        d["mask"] = {"size": a.chunk}
    if a.rot_dims:
        d["rot"] = {"dims": a.rot_dims, "base": a.rot_base, **({"scaling": a.rot_scaling} if a.rot_scaling else {})}
    if a.softcap:
        d["softcap"] = a.softcap
    if a.kv_from is not None:
        d["kv_from"] = a.kv_from
    for key, val, default in (("qk_norm", a.qk_norm, side), ("sink", a.sink, side), ("gate", a.gate, not side)):
        if val != default:
            d[key] = val
    return d


def config_to_json(cfg: NukizenConfig) -> dict:
    layers = []
    for L in cfg.layers:
        m = L.mixer
        if L.type == "attention":
            mixer = _attention_json(m, False)
        elif L.type == "rglru":
            mixer = {"width": m.width, "blocks": m.blocks, "conv": m.conv}
        else:
            r = m[1]
            mixer = {"left": _attention_json(m[0], True),
                     "right": {"heads": r.heads, "kv_heads": r.kv_heads, "dim": r.dim, "vdim": r.vdim, "conv": r.conv}}
        layers.append({"type": L.type, "mixer": mixer, "mlp": {"kind": "dense", "ff": L.ff} if L.ff else None})
    out = {"architecture": ARCHITECTURE, "vocab": cfg.vocab, "width": cfg.hidden, "layers": layers,
           "norm": {"eps": cfg.rms_eps}}
    if cfg.logit_softcap:
        out["logit_softcap"] = cfg.logit_softcap
    return out


def _attention_shapes(t: Dict[str, tuple], p: str, a: AttentionConfig, W: int) -> None:
    H, G, D, V = a.heads, a.kv_heads, a.dim, a.vdim
    t[p + "q"] = (H * D, W)
    if a.kv_from is None:
        t.update({p + "k": (G * D, W), p + "v": (G * V, W)})
    if a.qk_norm:
        t[p + "q.norm"] = (H * D,)
        if a.kv_from is None:
            t[p + "k.norm"] = (G * D,)
    if a.sink:
        t[p + "sink"] = (H,)
    if a.gate:
        t[p + "g"] = (H, W)
    t[p + "o"] = (W, H * V)


def tensor_shapes(cfg: NukizenConfig) -> Dict[str, tuple]:
    """Checkpoint tensor names and shapes of a configuration."""
    W = cfg.hidden
    t: Dict[str, tuple] = {"embed": (cfg.vocab, W), "final.norm": (W,), "head": (cfg.vocab, W)}
    for i, L in enumerate(cfg.layers):
        p = f"l{i}."
        t[p + "norm1"] = (W,)
        if L.type == "attention":
            _attention_shapes(t, p + "mix.", L.mixer, W)
        elif L.type == "rglru":
            m = L.mixer
            C, B = m.width, m.blocks
            t.update({p + "mix.y": (C, W), p + "mix.y.b": (C,), p + "mix.x": (C, W), p + "mix.x.b": (C,),
                      p + "mix.conv": (C, m.conv), p + "mix.conv.b": (C,), p + "mix.ra": (B, C // B, C // B),
                      p + "mix.ra.b": (B, C // B), p + "mix.ri": (B, C // B, C // B), p + "mix.ri.b": (B, C // B),
                      p + "mix.lam": (C,), p + "mix.o": (W, C)})
        else:
            a, r = L.mixer
            _attention_shapes(t, p + "mix.left.", a, W)
            q = p + "mix.right."
            H, G, D, V = r.heads, r.kv_heads, r.dim, r.vdim
            t.update({q + "q": (G * D, W), q + "q.conv": (G * D, r.conv), q + "k": (G * D, W),
                      q + "k.conv": (G * D, r.conv), q + "v": (H * V, W), q + "v.conv": (H * V, r.conv),
                      q + "b": (H, W), q + "A_log": (H,), q + "norm": (V,), q + "a": (H, W), q + "dt_bias": (H,),
                      q + "g": (H * V, W), q + "o": (W, H * V), p + "mix.left.out": (W,), p + "mix.right.out": (W,)})
        if L.ff:
            t.update({p + "mlp.gate": (L.ff, W), p + "mlp.up": (L.ff, W), p + "mlp.down": (W, L.ff)})
    return t


def random_tensors(cfg: NukizenConfig, seed: int = 0, device="cpu") -> Dict[str, torch.Tensor]:
    """Random bf16 weights of a configuration (benchmarks and tests): projections ~ N(0, 1 / fan_in), norm weights
    around one, biases and sinks of order one, convolution taps of order 1 / sqrt(taps)."""
    g = torch.Generator(device=device).manual_seed(seed)
    out: Dict[str, torch.Tensor] = {}
    randn = lambda shape: torch.randn(shape, generator=g, device=device)
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm", "norm1", "out"):
            t = 1.0 + randn(shape) * 0.1
        elif leaf in ("b", "dt_bias", "sink", "A_log", "lam") and len(shape) == 1 or name.endswith(("ra.b", "ri.b")):
            t = randn(shape) * 0.5
        elif leaf == "conv":
            t = randn(shape) / math.sqrt(shape[-1])
        else:
            t = randn(shape) / math.sqrt(shape[-1])
        out[name] = t.to(torch.bfloat16)
    return out


def save_checkpoint(cfg: NukizenConfig, tensors: Dict[str, torch.Tensor], path: Path) -> None:
    stream.save_checkpoint(config_to_json(cfg), tensors, path)


def preset(name: str, width: int, vocab: int, repeats: int, *, heads: int, kv_heads: int, dim: int, vdim: int, chunk: int,
           rot_dims: int, side_heads: int, side_kv_heads: int, side_dim: int, side_chunk: int, delta_heads: int,
           delta_kv_heads: int, delta_dim: int, delta_vdim: int, lru_width: int, lru_blocks: int, ff: int,
           order=("attention", "parallel", "rglru", "shared", "parallel")) -> NukizenConfig:
    """``repeats`` x ``order``; ``shared``: an attention layer on the keys and values of the group's first."""
    layers: List[LayerConfig] = []
    for _ in range(repeats):
        first = None
        for kind in order:
            if kind in ("attention", "shared"):
                src = first if kind == "shared" else None
                if src is None:
                    first = len(layers)
                mixer: object = AttentionConfig(heads, kv_heads, dim, vdim, 1.0 / math.sqrt(dim), chunk=chunk,
                                                rot_dims=rot_dims, rot_base=10000.0, softcap=50.0, kv_from=src, gate=True)
                layers.append(LayerConfig("attention", mixer, ff))
            elif kind == "rglru":
                layers.append(LayerConfig("rglru", RglruConfig(lru_width, lru_blocks, 4), ff))
            else:
                left = AttentionConfig(side_heads, side_kv_heads, side_dim, side_dim, 1.0 / math.sqrt(side_dim),
                                       chunk=side_chunk, rot_dims=side_dim, rot_base=10000.0,
                                       rot_scaling={"factor": 8.0, "original": 2048, "fast": 16.0, "slow": 2.0},
                                       qk_norm=True, sink=True)
                layers.append(LayerConfig("parallel", (left, DeltaConfig(delta_heads, delta_kv_heads, delta_dim,
                                                                         delta_vdim, 3)), ff))
    return NukizenConfig(name, vocab, width, layers, rms_eps=1e-6, logit_softcap=40.0)


PRESETS = {
    # runs on the CPU in tests: every mixer, a shared-cache layer, chunks shorter than the prompts
    "nukizen-tiny": preset("nukizen-tiny", 96, 320, 1, heads=6, kv_heads=2, dim=16, vdim=24, chunk=24, rot_dims=8,
                           side_heads=4, side_kv_heads=2, side_dim=16, side_chunk=40, delta_heads=4, delta_kv_heads=2,
                           delta_dim=16, delta_vdim=24, lru_width=64, lru_blocks=4, ff=128),
    # layer shapes of a ~1B-class model (benchmarks, random weights)
    "nukizen-1b": preset("nukizen-1b", 2048, 32768, 2, heads=16, kv_heads=4, dim=128, vdim=128, chunk=1024,
                         rot_dims=64, side_heads=16, side_kv_heads=4, side_dim=128, side_chunk=1024, delta_heads=16,
                         delta_kv_heads=8, delta_dim=64, delta_vdim=128, lru_width=2560, lru_blocks=10, ff=4096,
                         order=("attention", "parallel", "rglru", "shared")),
}


# ----------------------------------------------------------------------------- weights
@dataclass
class _Attention:
    cfg: AttentionConfig
    w_in: torch.Tensor                  # [H D (+ G D + G V) (+ H), W]: q | k | v | gate, rows padded to a multiple of 16
    o: torch.Tensor                     # [W, H V]
    cos_sin: Optional[torch.Tensor]     # [positions, rot_dims] fp32
    koff: int = 0
    voff: int = 0
    goff: int = 0
    qnw: Optional[torch.Tensor] = None
    knw: Optional[torch.Tensor] = None
    sinks: Optional[torch.Tensor] = None   # fp32 [H]
    cache: int = -1                     # index into kv_cache: its own, or the one of the layer it reads


@dataclass
class _Delta:
    cfg: DeltaConfig
    w_in: torch.Tensor                  # q | k | v | b | a | g
    cols: Dict[str, int]
    taps: torch.Tensor                  # fp32 [2 G D + H V, conv]
    neg_a: torch.Tensor                 # fp32 [H]: -exp(A_log)
    dt_bias: torch.Tensor               # fp32 [H]
    norm: torch.Tensor                  # fp32 [V]
    o: torch.Tensor
    state: int = -1                     # index into states: (conv inputs, S)


@dataclass
class _Rglru:
    cfg: RglruConfig
    w_in: torch.Tensor                  # y | x
    yb: torch.Tensor                    # fp32 [C]
    xb: torch.Tensor                    # fp32 [C]
    taps: torch.Tensor                  # fp32 [C, conv]
    conv_b: torch.Tensor                # fp32 [C]
    w_gate: torch.Tensor                # fp32 [blocks, 2 C / blocks, C / blocks]: per block ra rows, then ri rows
    gate_b: torch.Tensor                # fp32 [blocks, 2 C / blocks]
    rate: torch.Tensor                  # fp32 [C]: DECAY_RATE * softplus(lam)
    o: torch.Tensor
    state: int = -1


@dataclass
class _Side:
    left: _Attention
    right: _Delta
    left_out: torch.Tensor
    right_out: torch.Tensor


@dataclass
class _Layer:
    n1: torch.Tensor
    mixer: object
    w_gu: Optional[torch.Tensor]        # [2 F, W]: gate | up
    w_down: Optional[torch.Tensor]      # [W, F]


def _columns(parts) -> Dict[str, int]:
    cols, at = {}, 0
    for key, n in parts:
        cols[key] = at
        at += n
    return cols


class NukizenModel(StreamModel):
    def __init__(self, cfg: NukizenConfig, tp: Optional[TPGroup] = None, device="cpu", dtype=torch.bfloat16,
                 seed: int = 0, weights: Optional[str] = None, tensors: Optional[Dict[str, torch.Tensor]] = None,
                 max_model_len: int = 8192, weight_dtype: str = "bf16"):
        super().__init__(cfg, tp, device, dtype, seed, max_model_len, weight_dtype)
        self._rope: Dict[tuple, torch.Tensor] = {}
        if tensors is None:
            tensors = self._open(Path(weights)) if weights else random_tensors(cfg, seed, self.device)
        get = tensors if callable(tensors) else tensors.__getitem__
        self._build(get)

    # ------------------------------------------------------------------ weights
    def _f(self, t: torch.Tensor) -> torch.Tensor:
        """Small constants that enter fp32 arithmetic are kept in fp32."""
        return t.to(F32).to(self.device).contiguous()

    @staticmethod
    def _has(get, name: str) -> bool:
        try:
            get(name)
            return True
        except KeyError:
            return False

    def _rope_table(self, a: AttentionConfig) -> Optional[torch.Tensor]:
        if not a.rot_dims:
            return None
        sc = a.rot_scaling
        key = (a.rot_dims, a.rot_base, tuple(sorted(sc.items())) if sc else None)
        if key not in self._rope:
            self._rope[key] = ref.rope_table(a.rot_dims, self.max_model_len, a.rot_base,
                                             {"type": "yarn", **sc} if sc else None).to(self.device).contiguous()
        return self._rope[key]

    def _build_attention(self, get, p: str, a: AttentionConfig, where: str) -> _Attention:
        t = self._t
        H, G, D, V = a.heads, a.kv_heads, a.dim, a.vdim
        if H % G:
            raise ValueError(f"{where}: {H} query heads over {G} key / value heads")
        if a.rot_dims > D or a.rot_dims % 2:
            raise ValueError(f"{where}: rot.dims {a.rot_dims} must be even and at most dim {D}")
        own = a.kv_from is None
        # a checkpoint settles the optional parts by the tensors it holds
        has = lambda name: self._has(get, p + name)
        a.gate, a.sink, a.qk_norm = has("g"), has("sink"), has("q.norm")
        parts = [("q", H * D)] + ([("k", G * D), ("v", G * V)] if own else []) + ([("g", H)] if a.gate else [])
        cols = _columns(parts)
        rows = [get(p + key) for key, _ in parts]
        n = sum(r.shape[0] for r in rows)
        if n % 16:                       # 16-byte aligned output rows for the matrix-core kernels
            rows.append(torch.zeros(16 - n % 16, rows[0].shape[1], dtype=rows[0].dtype))
        w = _Attention(a, t(torch.cat(rows)), t(get(p + "o")), self._rope_table(a), cols.get("k", 0), cols.get("v", 0),
                       cols.get("g", 0))
        if a.qk_norm:
            w.qnw = t(get(p + "q.norm"))
            w.knw = t(get(p + "k.norm")) if own else None
        if a.sink:
            w.sinks = self._f(get(p + "sink"))
        return w

    def _build(self, get) -> None:
        c, t, f = self.cfg, self._t, self._f
        self.embed = t(get("embed"))
        self.final_norm = t(get("final.norm"))
        self.lm_head = t(get("head"))
        self.layers: List[_Layer] = []
        self._kv_owners: List[_Attention] = []
        self._recurrent: List[object] = []
        own_of: Dict[int, _Attention] = {}

        def attention(i: int, p: str, a: AttentionConfig) -> _Attention:
            w = self._build_attention(get, p, a, f"layer {i}")
            if a.kv_from is None:
                w.cache = len(self._kv_owners)
                self._kv_owners.append(w)
            return w

        for i, L in enumerate(c.layers):
            p = f"l{i}.mix."
            if L.type == "attention":
                mixer: object = attention(i, p, L.mixer)
                if L.mixer.kv_from is None:
                    own_of[i] = mixer
            elif L.type == "rglru":
                m = L.mixer
                C, B = m.width, m.blocks
                if C % B:
                    raise ValueError(f"layer {i}: {B} blocks do not divide the width {C}")
                if m.conv > sm.CONV_MAX_TAPS:
                    raise ValueError(f"layer {i}: {m.conv} convolution taps exceed {sm.CONV_MAX_TAPS}")
                lam = get(p + "lam").double()
                mixer = _Rglru(m, t(torch.cat([get(p + "y"), get(p + "x")])), f(get(p + "y.b")), f(get(p + "x.b")),
                               f(get(p + "conv")), f(get(p + "conv.b")),
                               f(torch.cat([get(p + "ra"), get(p + "ri")], 1)),
                               f(torch.cat([get(p + "ra.b"), get(p + "ri.b")], 1)),
                               f(DECAY_RATE * torch.nn.functional.softplus(lam)), t(get(p + "o")),
                               state=len(self._recurrent))
                self._recurrent.append(mixer)
            else:
                a, r = L.mixer
                left = attention(i, p + "left.", a)
                H, G, D, V = r.heads, r.kv_heads, r.dim, r.vdim
                if H % G:
                    raise ValueError(f"layer {i}: {H} delta-rule heads over {G} query / key heads")
                if max(D, V) > sm.delta_scan_max_dim() or r.conv > sm.CONV_MAX_TAPS:
                    raise ValueError(f"layer {i}: delta-rule head sizes {D} x {V} or {r.conv} taps exceed the kernels'")
                q = p + "right."
                cols = _columns((("q", G * D), ("k", G * D), ("v", H * V), ("b", H), ("a", H), ("g", H * V)))
                right = _Delta(r, t(torch.cat([get(q + s) for s in ("q", "k", "v", "b", "a", "g")])), cols,
                               f(torch.cat([get(q + s + ".conv") for s in ("q", "k", "v")])),
                               f(-torch.exp(get(q + "A_log").double())), f(get(q + "dt_bias")), f(get(q + "norm")),
                               t(get(q + "o")), state=len(self._recurrent))
                self._recurrent.append(right)
                mixer = _Side(left, right, t(get(p + "left.out")), t(get(p + "right.out")))
                if a.kv_from is None:
                    own_of[i] = left
            w_gu = w_down = None
            if L.ff:
                w_gu = t(torch.cat([get(f"l{i}.mlp.gate"), get(f"l{i}.mlp.up")]))
                w_down = t(get(f"l{i}.mlp.down"))
            self.layers.append(_Layer(t(get(f"l{i}.norm1")), mixer, w_gu, w_down))
        for i, L in enumerate(c.layers):       # layers that read another layer's keys and values
            a = L.mixer if L.type == "attention" else L.mixer[0] if L.type == "parallel" else None
            if a is None or a.kv_from is None:
                continue
            src = own_of.get(a.kv_from)
            if src is None or a.kv_from >= i:
                raise ValueError(f"layer {i}: kv_from {a.kv_from} must name an earlier attention layer with projections")
            s = src.cfg
            if (s.kv_heads, s.dim, s.vdim) != (a.kv_heads, a.dim, a.vdim):
                raise ValueError(f"layer {i}: head sizes differ from layer {a.kv_from}'s, whose cache it reads")
            w = self.layers[i].mixer
            (w if isinstance(w, _Attention) else w.left).cache = src.cache

    def _weight_roots(self) -> tuple:
        return (self.embed, self.final_norm, self.lm_head, *self.layers)

    # ------------------------------------------------------------------ cache and state
    def _needs_state(self) -> bool:
        return bool(self._recurrent)

    def allocate_kv(self, num_blocks: int, block_size: int):
        """Per attention mixer with projections of its own: paged keys [slots, G, D] and values [slots, G, V]."""
        self.block_size = block_size
        n = num_blocks * block_size
        self.kv_cache = [(torch.zeros(n, a.cfg.kv_heads, a.cfg.dim, dtype=self.dtype, device=self.device),
                          torch.zeros(n, a.cfg.kv_heads, a.cfg.vdim, dtype=self.dtype, device=self.device))
                         for a in self._kv_owners]
        return self.kv_cache

    def kv_bytes_per_block(self, block_size: int) -> int:
        eb = torch.finfo(self.dtype).bits // 8
        return max(1, sum(block_size * a.cfg.kv_heads * (a.cfg.dim + a.cfg.vdim) * eb for a in self._kv_owners))

    def _state_shapes(self, w) -> tuple:
        """(convolution inputs [taps - 1, channels], recurrent state) of one recurrent mixer, per request slot."""
        m = w.cfg
        if isinstance(w, _Rglru):
            return (max(m.conv - 1, 0), m.width), (m.width,)
        return (max(m.conv - 1, 0), 2 * m.kv_heads * m.dim + m.heads * m.vdim), (m.heads, m.dim * m.vdim)

    def allocate_state(self, slots: int) -> None:
        """Per recurrent mixer and request slot, fp32: the convolutions' last inputs and the recurrent state."""
        self.state_slots = slots
        z = lambda shape: torch.zeros(slots, *shape, dtype=F32, device=self.device)
        self.states = [tuple(z(s) for s in self._state_shapes(w)) for w in self._recurrent]

    def state_bytes_per_slot(self) -> int:
        return sum(4 * math.prod(s) for w in self._recurrent for s in self._state_shapes(w))

    # ------------------------------------------------------------------ layers
    def _attention(self, w: _Attention, h, b) -> torch.Tensor:
        a = w.cfg
        H, G, D, V = a.heads, a.kv_heads, a.dim, a.vdim
        kc, vc = self.kv_cache[w.cache]
        own = a.kv_from is None
        proj = sm.linear(h, w.w_in)                                        # [T, q | k | v | gate]
        sm.window_kv_write(kc if own else None, vc if own else None, proj, w.koff, w.voff, None, None, None, w.cos_sin,
                           b["positions"], b["slot_mapping"], H, G, D, V, a.rot_dims, self.cfg.rms_eps, False,
                           half_layout=True, qnw=w.qnw, knw=w.knw)
        y = sm.window_attention(proj, proj[:, w.goff:w.goff + H] if a.gate else None, kc, vc, None, None,
                                b["block_tables"], b["tok_seq"], b["positions"], H, 0, 0, a.scale, a.sink,
                                self.block_size, b["cu_q"], b.get("max_qlen", 0), b.get("max_keys", 0), chunk=a.chunk,
                                softcap=a.softcap, sinks=w.sinks, gate_per_head=True)
        return y

    def _delta(self, w: _Delta, h, b) -> torch.Tensor:
        m = w.cfg
        H, G, D, V = m.heads, m.kv_heads, m.dim, m.vdim
        conv_state, S = self.states[w.state]
        proj = sm.linear(h, w.w_in, out_dtype=F32)                         # what enters the recurrence stays fp32
        n = 2 * G * D + H * V
        qkv = sm.short_conv(proj[:, :n], w.taps, conv_state, b["cu_q"], b["tok_seq"], b["seq_slots"], b["positions"],
                            act=sm.CONV_SILU, unit_cols=2 * G * D, unit_dim=D, scale_cols=G * D, scale=D ** -0.5,
                            unit_eps=UNIT_EPS)
        return sm.delta_scan(qkv, proj, w.cols, w.neg_a, w.dt_bias, w.norm, S, b["cu_q"], b["seq_slots"],
                             b["positions"], H, G, D, V, self.cfg.rms_eps, self.dtype)

    def _rglru(self, w: _Rglru, h, b) -> torch.Tensor:
        m = w.cfg
        C, B = m.width, m.blocks
        conv_state, S = self.states[w.state]
        proj = sm.linear(h, w.w_in, out_dtype=F32)                         # [T, y | x]
        u = sm.short_conv(proj[:, C:2 * C], w.taps, conv_state, b["cu_q"], b["tok_seq"], b["seq_slots"], b["positions"],
                          in_bias=w.xb, out_bias=w.conv_b)
        T = u.shape[0]
        gates = torch.empty(T, B, 2 * C // B, dtype=F32, device=u.device)
        sm.gemm(u.view(T, B, C // B).transpose(0, 1), w.w_gate, F32, out=gates.transpose(0, 1))
        return sm.rglru_scan(u, gates, w.gate_b, w.rate, proj, 0, w.yb, S, b["cu_q"], b["seq_slots"], b["positions"], B,
                             self.dtype, b.get("max_qlen", 1))

    def _mixer(self, L: _Layer, h, b) -> torch.Tensor:
        w = L.mixer
        if isinstance(w, _Attention):
            return sm.linear(self._attention(w, h, b), w.o)
        if isinstance(w, _Rglru):
            return sm.linear(self._rglru(w, h, b), w.o)
        left = sm.linear(self._attention(w.left, h, b), w.left.o)
        right = sm.linear(self._delta(w.right, h, b), w.right.o)
        return sm.norm_mix(left, w.left_out, right, w.right_out, self.cfg.rms_eps, 0.5, 0.5)

    def _blocks(self, ids, b, after=None):
        """The residual stream before the last layer's branches are added: (x, mixer branch, feed-forward branch)."""
        c, dt = self.cfg, self.dtype
        x = sm.embed_rows(ids, self.embed)
        mix = ff = None                   # branch outputs not yet added: the next norm adds them in fp32
        for L in self.layers:
            h = sm.resnorm(x, L.n1, c.rms_eps, branch=mix, branch2=ff, out_dtype=dt)
            mix = self._mixer(L, h, b)
            ff = sm.linear(sm.act(sm.linear(h, L.w_gu), sm.ACT_RELU), L.w_down) if L.w_gu is not None else None
            if after is not None:
                sm.resnorm(x, None, c.rms_eps, branch=mix, branch2=ff, out_dtype=dt)
                mix = ff = None
                after.append(x.clone())
        return x, mix, ff

    def _forward(self, ids, b, rows) -> torch.Tensor:
        c = self.cfg
        x, mix, ff = self._blocks(ids, b)
        pick = lambda t: t.index_select(0, rows) if t is not None else None
        hf = sm.resnorm(x.index_select(0, rows), self.final_norm, c.rms_eps, branch=pick(mix), branch2=pick(ff),
                        out_dtype=self.dtype)
        z = sm.linear(hf, self.lm_head, out_dtype=F32)
        if c.logit_softcap > 0:
            z = sm.act(z, sm.ACT_SOFTCAP, limit=c.logit_softcap)
        return z.unsqueeze(0)                                              # [1, S, vocab]

    def residual_after_runs(self, ids, b) -> List[torch.Tensor]:
        """(debugging / tests) the fp32 residual stream after every layer."""
        after: List[torch.Tensor] = []
        self._blocks(ids, b, after)
        return after
