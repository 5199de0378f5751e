"""Semanex: a decoder whose fp32 residual stream is normed *after* every sum,
``x <- norm1(alpha x + mixer(x)); x <- norm2(alpha x + ff(x))`` (RMS norms with a single gain; the sublayers read the
normed stream itself), a dense feed-forward ``W_down gelu(W_up x)`` (exact gelu) and two mixers in any order the config
lists.  What a mixer reads first passes a short causal convolution over time per channel, ``h = x + conv(x)``
(``canon.taps`` taps, no bias); the last taps - 1 inputs are part of a sequence's state in every layer.

* ``latent_attention``: keys and values are up-projections (``W_uk``, ``W_uv``) of one cached low-rank row per token,
  ``c = rmsnorm(W_dkv h)[:kv_rank]``, beside one rotated key part shared by the heads; queries come from a normed
  low-rank row as well, ``q = W_uq rmsnorm(W_dq h)``, each head laid out as [dim unrotated | rot_dim rotated]; the
  rotation turns the pairs (2i, 2i + 1) by ``pos * base^(-2i / dims)``; causal softmax of
  ``(q_n . k_n + q_r . k_r) * scale`` with a learned sink per head in the denominator (``e^sink``, no key, no value);
  the heads' outputs times ``sigmoid(W_g h)`` element by element, then ``W_o``.  Queries are absorbed into the latent
  space (``q_n W_uk``), so the cache is attended as it is stored and ``W_uv`` follows the softmax.
* ``parallel``: two mixers side by side on the same input, ``left_scale * left + right_scale * right``.  Left:
  grouped-query attention without positions; queries and keys RMS-normed per head with a weight of ``dim`` numbers that
  the heads share; scores ``q . k * scale`` capped to ``cap tanh(s / cap)``; causal softmax; output times
  ``sigmoid(W_g h)`` before ``W_o``.  Right: a state-space recurrence with a scalar decay per head (the Mamba-2 layer
  of "Transformers are SSMs", Dao and Gu): ``W_in h = [z | x | B | C | dt]``; x, B, C pass a short causal convolution
  with bias and silu; ``dt = softplus(dt + dt_bias)``; per head (B, C of its group) ``S <- exp(-exp(A_log) dt) S + dt B x^T``,
  ``y = S^T C + D x``; ``y silu(z)`` is RMS-normed in ``norm_groups`` equal parts, times a weight, then ``W_o``.

The model presents the engine's interface through :class:`~.stream.StreamModel`; caches: per latent attention a paged
``[slots, kv_rank + rot_dim]`` cache, per left attention paged keys / values, per layer the convolution's last inputs
and per recurrence its convolution inputs and state, fp32 records per request slot.  Every op is a kernel of
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

ARCHITECTURE = "Semanex"
MIXERS = ("latent_attention", "parallel")
F32 = torch.float32


# ----------------------------------------------------------------------------- configuration
@dataclass
class LatentConfig:
    heads: int
    dim: int                 # unrotated query / key dimensions per head
    rot_dim: int             # rotated dimensions per head (one key part shared by the heads)
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_base: float = 10000.0
    rot_dims: int = -1       # dimensions of the rotated part that turn (the first ones); -1: all of it

    def __post_init__(self):
        if self.rot_dims < 0:
            self.rot_dims = self.rot_dim


@dataclass
class CappedConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float = 0.0


@dataclass
class SsdConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    conv: int

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass
class ParallelConfig:
    left: CappedConfig
    right: SsdConfig
    left_scale: float = 1.0
    right_scale: float = 1.0


@dataclass
class LayerConfig:
    type: str
    mixer: object            # LatentConfig | ParallelConfig
    ff: int = 0              # 0: no feed-forward


@dataclass
class SemanexConfig:
    name: str
    vocab: int
    hidden: int
    layers: List[LayerConfig]
    rms_eps: float = 1e-6
    alpha: float = 1.0               # x <- norm(alpha x + branch)
    embed_scale: float = 1.0
    canon_taps: int = 0              # 0: the mixers read the stream as it is
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


def _layer_from(l: dict) -> LayerConfig:
    kind, d = l["type"], l["mixer"]
    if kind == "latent_attention":
        rot = d.get("rot") or {}
        dim, rot_dim = int(d["dim"]), int(d["rot_dim"])
        mixer: object = LatentConfig(int(d["heads"]), dim, rot_dim, int(d["vdim"]), int(d["kv_rank"]), int(d["q_rank"]),
                                     float(d.get("scale", 1.0 / math.sqrt(dim + rot_dim))),
                                     float(rot.get("base", 10000.0)), int(rot.get("dims", rot_dim)))
    elif kind == "parallel":
        a, r = d["left"], d["right"]
        dim = int(a["dim"])
        left = CappedConfig(int(a["heads"]), int(a.get("kv_heads") or a["heads"]), dim, int(a.get("vdim") or dim),
                            float(a.get("scale", 1.0 / math.sqrt(dim))), float(a.get("softcap") or 0.0))
        right = SsdConfig(int(r["heads"]), int(r["vdim"]), int(r["state"]), int(r.get("groups") or 1),
                          int(r.get("norm_groups") or 1), int(r.get("conv") or 1))
        mixer = ParallelConfig(left, right, float(d.get("left_scale", 1.0)), float(d.get("right_scale", 1.0)))
    else:
        raise ValueError(f"unknown mixer type {kind!r} (known: {', '.join(MIXERS)})")
    mlp = l.get("mlp")
    if mlp is not None and mlp.get("kind", "dense") != "dense":
        raise ValueError(f"unknown mlp kind {mlp['kind']!r}")
    return LayerConfig(kind, mixer, int(mlp["ff"]) if mlp else 0)


def config_from_json(c: dict, name: str = "semanex") -> SemanexConfig:
    return SemanexConfig(name=name, vocab=int(c["vocab"]), hidden=int(c["width"]),
                         layers=[_layer_from(l) for l in c["layers"]],
                         rms_eps=float((c.get("norm") or {}).get("eps", 1e-6)),
                         alpha=float(c.get("postln_alpha", 1.0)),
                         embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                         canon_taps=int((c.get("canon") or {}).get("taps") or 0))


def config_to_json(cfg: SemanexConfig) -> dict:
    layers = []
    for L in cfg.layers:
        m = L.mixer
        if L.type == "latent_attention":
            mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                     "q_rank": m.q_rank, "scale": m.scale, "rot": {"dims": m.rot_dims, "base": m.rot_base}}
        else:
            a, r = m.left, m.right
            mixer = {"left": {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                              "softcap": a.softcap},
                     "right": {"heads": r.heads, "vdim": r.vdim, "state": r.state, "groups": r.groups,
                               "norm_groups": r.norm_groups, "conv": r.conv},
                     "left_scale": m.left_scale, "right_scale": m.right_scale}
        layers.append({"type": L.type, "mixer": mixer, "mlp": {"kind": "dense", "ff": L.ff} if L.ff else None})
    out = {"architecture": ARCHITECTURE, "vocab": cfg.vocab, "width": cfg.hidden, "layers": layers,
           "norm": {"eps": cfg.rms_eps}, "postln_alpha": cfg.alpha, "embedding": {"scale": cfg.embed_scale}}
    if cfg.canon_taps:
        out["canon"] = {"taps": cfg.canon_taps}
    return out


def tensor_shapes(cfg: SemanexConfig) -> Dict[str, tuple]:
    """Checkpoint tensor names and shapes of a configuration."""
    W = cfg.hidden
    t: Dict[str, tuple] = {"embed": (cfg.vocab, W), "final.norm": (), "head": (cfg.vocab, W)}
    for i, L in enumerate(cfg.layers):
        p = f"l{i}."
        t[p + "norm1"] = ()
        if cfg.canon_taps:
            t[p + "canon1"] = (W, cfg.canon_taps)
        m = L.mixer
        if L.type == "latent_attention":
            q = p + "mix."
            H = m.heads
            t.update({q + "dq": (m.q_rank, W), q + "dq.norm": (m.q_rank,), q + "uq": (H * (m.dim + m.rot_dim), m.q_rank),
                      q + "dkv": (m.kv_rank + m.rot_dim, W), q + "dkv.norm": (m.kv_rank,),
                      q + "uk": (H * m.dim, m.kv_rank), q + "uv": (H * m.vdim, m.kv_rank), q + "sink": (H,),
                      q + "g": (H * m.vdim, W), q + "o": (W, H * m.vdim)})
        else:
            a, r = m.left, m.right
            q = p + "mix.left."
            t.update({q + "q": (a.heads * a.dim, W), q + "k": (a.kv_heads * a.dim, W), q + "v": (a.kv_heads * a.vdim, W),
                      q + "q.norm": (a.dim,), q + "k.norm": (a.dim,), q + "g": (a.heads * a.vdim, W),
                      q + "o": (W, a.heads * a.vdim)})
            q = p + "mix.right."
            t.update({q + "in": (2 * r.inner + 2 * r.groups * r.state + r.heads, W),
                      q + "conv": (r.conv_channels, r.conv), q + "conv.b": (r.conv_channels,),
                      q + "dt_bias": (r.heads,), q + "A_log": (r.heads,), q + "D": (r.heads,), q + "norm": (r.inner,),
                      q + "o": (W, r.inner)})
        if L.ff:
            t.update({p + "norm2": (), p + "mlp.up": (L.ff, W), p + "mlp.down": (W, L.ff)})
    return t


def random_tensors(cfg: SemanexConfig, seed: int = 0, device="cpu") -> Dict[str, torch.Tensor]:
    """Random bf16 weights of a configuration (benchmarks and tests): projections ~ N(0, 1 / fan_in), norm weights and
    gains around one, biases, sinks and skips of order one, convolution taps of order 1 / sqrt(taps)."""
    g = torch.Generator(device=device).manual_seed(seed)
    out: Dict[str, torch.Tensor] = {}
    randn = lambda shape: torch.randn(shape, generator=g, device=device)
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm", "norm1", "norm2"):
            t = 1.0 + randn(shape) * 0.1
        elif leaf in ("b", "dt_bias", "sink", "A_log", "D"):
            t = randn(shape) * 0.5
        elif leaf == "embed":
            t = randn(shape) / math.sqrt(shape[-1])
        else:
            t = randn(shape) / math.sqrt(shape[-1])
        out[name] = t.to(torch.bfloat16)
    return out


def save_checkpoint(cfg: SemanexConfig, tensors: Dict[str, torch.Tensor], path: Path) -> None:
    stream.save_checkpoint(config_to_json(cfg), tensors, path)


def preset(name: str, width: int, vocab: int, repeats: int, *, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
           q_rank: int, side_heads: int, side_kv_heads: int, side_dim: int, side_vdim: int, ssd_heads: int,
           ssd_vdim: int, ssd_state: int, ssd_groups: int, norm_groups: int, ff: int, taps: int = 4,
           order=("latent_attention", "latent_attention", "parallel", "latent_attention")) -> SemanexConfig:
    """``repeats`` x ``order``, every layer with a feed-forward; alpha grows with the depth as (2 layers)^(1/4)."""
    layers: List[LayerConfig] = []
    for _ in range(repeats):
        for kind in order:
            if kind == "latent_attention":
                mixer: object = LatentConfig(heads, dim, rot_dim, vdim, kv_rank, q_rank, 1.0 / math.sqrt(dim + rot_dim),
                                             10000.0)
            else:
                mixer = ParallelConfig(CappedConfig(side_heads, side_kv_heads, side_dim, side_vdim,
                                                    1.0 / math.sqrt(side_dim), 30.0),
                                       SsdConfig(ssd_heads, ssd_vdim, ssd_state, ssd_groups, norm_groups, 4), 1.0, 1.0)
            layers.append(LayerConfig(kind, mixer, ff))
    return SemanexConfig(name, vocab, width, layers, rms_eps=1e-6, alpha=(2.0 * len(layers)) ** 0.25,
                         embed_scale=math.sqrt(width), canon_taps=taps)


PRESETS = {
    # runs on the CPU in tests: both mixers, odd sizes
    "semanex-tiny": preset("semanex-tiny", 96, 320, 1, heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=32, q_rank=40,
                           side_heads=4, side_kv_heads=2, side_dim=16, side_vdim=24, ssd_heads=4, ssd_vdim=12,
                           ssd_state=16, ssd_groups=2, norm_groups=2, ff=128,
                           order=("latent_attention", "parallel")),
    # layer shapes of a ~1B-class model (benchmarks, random weights)
    "semanex-1b": preset("semanex-1b", 2048, 32768, 2, heads=16, dim=128, rot_dim=64, vdim=128, kv_rank=512,
                         q_rank=1536, side_heads=16, side_kv_heads=4, side_dim=128, side_vdim=128, ssd_heads=32,
                         ssd_vdim=64, ssd_state=128, ssd_groups=4, norm_groups=4, ff=4096),
}


# ----------------------------------------------------------------------------- weights
@dataclass
class _Latent:
    cfg: LatentConfig
    w_in: torch.Tensor                  # [q_rank | kv_rank + rot_dim | H V (gate), W], parts padded to multiples of 16 rows
    cols: Dict[str, int]
    dq_norm: torch.Tensor               # [q_rank]
    uq: torch.Tensor                    # [H (Dn + R), q_rank]
    dkv_norm: torch.Tensor              # [kv_rank]
    uk_t: torch.Tensor                  # [H, kv_rank, Dn]: per head W_uk^T (absorbs the query into the latent space)
    uv: torch.Tensor                    # [H, V, kv_rank]
    sinks: torch.Tensor                 # fp32 [H]
    o: torch.Tensor                     # [W, H V]
    cos_sin: torch.Tensor               # [positions, rot_dim] fp32
    cache: int = -1                     # index into kv_cache


@dataclass
class _Capped:
    cfg: CappedConfig
    w_in: torch.Tensor                  # q | k | v | gate
    cols: Dict[str, int]
    qnw: torch.Tensor                   # [D]
    knw: torch.Tensor                   # [D]
    o: torch.Tensor
    cache: int = -1


@dataclass
class _Ssd:
    cfg: SsdConfig
    w_in: torch.Tensor                  # z | x | B | C | dt
    taps: torch.Tensor                  # fp32 [inner + 2 G N, conv]
    conv_b: torch.Tensor                # fp32
    head_params: torch.Tensor           # fp32 [3, H]: -exp(A_log), dt_bias, D
    norm: torch.Tensor                  # fp32 [inner]
    o: torch.Tensor
    state: int = -1                     # index into states: (conv inputs, S)


@dataclass
class _Side:
    cfg: ParallelConfig
    left: _Capped
    right: _Ssd


@dataclass
class _Layer:
    gain1: float
    mixer: object
    taps: Optional[torch.Tensor]        # fp32 [W, taps]: the convolution ahead of the mixer
    canon: int = -1                     # index into states: the convolution's last inputs
    gain2: float = 1.0
    post2: bool = False                 # a second norm (with or without a feed-forward ahead of it)
    w_up: Optional[torch.Tensor] = None
    w_down: Optional[torch.Tensor] = None


def _stack(parts, align: int = 16):
    """Rows of several projections of one input, every part padded to a multiple of ``align`` rows (16-byte aligned
    column offsets in the product): (weight, column offset of every part)."""
    rows, cols, at = [], {}, 0
    for key, w in parts:
        cols[key] = at
        rows.append(w)
        pad = (-w.shape[0]) % align
        if pad:
            rows.append(torch.zeros(pad, w.shape[1], dtype=w.dtype))
        at += w.shape[0] + pad
    return torch.cat(rows), cols


class SemanexModel(StreamModel):
    def __init__(self, cfg: SemanexConfig, tp: Optional[TPGroup] = None, device="cpu", dtype=torch.bfloat16,
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

    def _rope_table(self, dims: int, base: float) -> torch.Tensor:
        if (dims, base) not in self._rope:
            self._rope[(dims, base)] = ref.rope_table(dims, self.max_model_len, base).to(self.device).contiguous()
        return self._rope[(dims, base)]

    def _build_latent(self, get, p: str, m: LatentConfig, where: str) -> _Latent:
        t = self._t
        H, Dn, R, V, C = m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank
        if m.rot_dims % 2 or not 0 < m.rot_dims <= R:
            raise ValueError(f"{where}: rot.dims {m.rot_dims} must be even, positive and at most rot_dim {R}")
        w_in, cols = _stack((("dq", get(p + "dq").cpu()), ("dkv", get(p + "dkv").cpu()), ("g", get(p + "g").cpu())))
        return _Latent(m, t(w_in), cols, t(get(p + "dq.norm")), t(get(p + "uq")), t(get(p + "dkv.norm")),
                       t(get(p + "uk").view(H, Dn, C).transpose(1, 2)), t(get(p + "uv").view(H, V, C)),
                       self._f(get(p + "sink")), t(get(p + "o")), self._rope_table(m.rot_dims, m.rot_base))

    def _build_side(self, get, p: str, m: ParallelConfig, where: str) -> _Side:
        t, f = self._t, self._f
        a, r = m.left, m.right
        if a.heads % a.kv_heads:
            raise ValueError(f"{where}: {a.heads} query heads over {a.kv_heads} key / value heads")
        if r.heads % r.groups or r.inner % r.norm_groups:
            raise ValueError(f"{where}: {r.groups} groups / {r.norm_groups} norm groups do not divide the {r.heads} heads")
        if max(r.state, r.vdim) > sm.gated_scan_max_dim():
            raise ValueError(f"{where}: state {r.state} x {r.vdim} exceeds the kernels' {sm.gated_scan_max_dim()}")
        q = p + "left."
        w_in, cols = _stack(tuple((s, get(q + s).cpu()) for s in ("q", "k", "v", "g")))
        left = _Capped(a, t(w_in), cols, t(get(q + "q.norm")), t(get(q + "k.norm")), t(get(q + "o")))
        q = p + "right."
        r.conv = int(get(q + "conv").shape[1])                 # the taps are what the checkpoint holds
        if r.conv > sm.CONV_MAX_TAPS:
            raise ValueError(f"{where}: {r.conv} convolution taps exceed {sm.CONV_MAX_TAPS}")
        hp = torch.stack([-torch.exp(get(q + "A_log").double()), get(q + "dt_bias").double(), get(q + "D").double()])
        right = _Ssd(r, t(get(q + "in")), f(get(q + "conv")), f(get(q + "conv.b")), f(hp), f(get(q + "norm")),
                     t(get(q + "o")))
        return _Side(m, left, right)

    def _build(self, get) -> None:
        c, t, f = self.cfg, self._t, self._f
        if c.canon_taps > sm.CONV_MAX_TAPS:
            raise ValueError(f"{c.canon_taps} convolution taps exceed {sm.CONV_MAX_TAPS}")
        self.embed = t(get("embed"))
        self.final_gain = float(get("final.norm").float())
        self.lm_head = t(get("head"))
        self.layers: List[_Layer] = []
        self._latents: List[_Latent] = []
        self._capped: List[_Capped] = []
        self._state_shapes: List[tuple] = []      # per state record pair: (conv inputs [taps - 1, C], state or None)
        for i, L in enumerate(c.layers):
            p = f"l{i}."
            if L.type == "latent_attention":
                mixer: object = self._build_latent(get, p + "mix.", L.mixer, f"layer {i}")
                self._latents.append(mixer)
            else:
                mixer = self._build_side(get, p + "mix.", L.mixer, f"layer {i}")
                self._capped.append(mixer.left)
                r = L.mixer.right
                mixer.right.state = len(self._state_shapes)
                self._state_shapes.append(((max(r.conv - 1, 0), r.conv_channels), (r.heads, r.state * r.vdim)))
            lay = _Layer(float(get(p + "norm1").float()), mixer, None)
            if self._has(get, p + "canon1"):      # a checkpoint settles optional parts by its tensors, taps included
                lay.taps = f(get(p + "canon1"))
                if lay.taps.shape[1] > sm.CONV_MAX_TAPS:
                    raise ValueError(f"layer {i}: {lay.taps.shape[1]} convolution taps exceed {sm.CONV_MAX_TAPS}")
                lay.canon = len(self._state_shapes)
                self._state_shapes.append(((lay.taps.shape[1] - 1, c.hidden), None))
            if L.ff:
                lay.w_up, lay.w_down = t(get(p + "mlp.up")), t(get(p + "mlp.down"))
            if L.ff or self._has(get, p + "norm2"):
                lay.post2, lay.gain2 = True, float(get(p + "norm2").float())
            self.layers.append(lay)
        # caches: latent attentions first, then the left attentions of the parallel mixers
        for n, w in enumerate(self._latents):
            w.cache = n
        for n, w in enumerate(self._capped):
            w.cache = len(self._latents) + n

    def _weight_roots(self) -> tuple:
        return (self.embed, self.lm_head, *self.layers)

    # ------------------------------------------------------------------ cache and state
    def _needs_state(self) -> bool:
        return bool(self._state_shapes)

    def allocate_kv(self, num_blocks: int, block_size: int):
        """Per latent attention one paged cache [slots, kv_rank + rot_dim]; per left attention paged keys
        [slots, G, D] and values [slots, G, V]."""
        self.block_size = block_size
        n = num_blocks * block_size
        z = lambda *shape: torch.zeros(n, *shape, dtype=self.dtype, device=self.device)
        self.kv_cache = [z(w.cfg.kv_rank + w.cfg.rot_dim) for w in self._latents]
        self.kv_cache += [(z(w.cfg.kv_heads, w.cfg.dim), z(w.cfg.kv_heads, w.cfg.vdim)) for w in self._capped]
        return self.kv_cache

    def kv_bytes_per_block(self, block_size: int) -> int:
        eb = torch.finfo(self.dtype).bits // 8
        per_token = sum(w.cfg.kv_rank + w.cfg.rot_dim for w in self._latents)
        per_token += sum(w.cfg.kv_heads * (w.cfg.dim + w.cfg.vdim) for w in self._capped)
        return max(1, block_size * per_token * eb)

    def allocate_state(self, slots: int) -> None:
        """fp32 records per request slot: every layer's last convolution inputs; per recurrence its convolution
        inputs and state."""
        self.state_slots = slots
        z = lambda shape: torch.zeros(slots, *shape, dtype=F32, device=self.device) if shape is not None else None
        self.states = [(z(a), z(b)) for a, b in self._state_shapes]

    def state_bytes_per_slot(self) -> int:
        return sum(4 * math.prod(s) for pair in self._state_shapes for s in pair if s is not None)

    # ------------------------------------------------------------------ layers
    def _latent(self, w: _Latent, h, b) -> torch.Tensor:
        m = w.cfg
        T = h.shape[0]
        H, Dn, R, C, V = m.heads, m.dim, m.rot_dim, m.kv_rank, m.vdim
        eps = self.cfg.rms_eps
        cache = self.kv_cache[w.cache]
        proj = sm.linear(h, w.w_in)                                        # [T, dq | dkv | gate]
        cq = sm.norm_mix(proj[:, w.cols["dq"]:w.cols["dq"] + m.q_rank], w.dq_norm, None, None, eps)
        q = sm.linear(cq, w.uq)                                            # [T, H (Dn + R)]
        sm.latent_kv_write(cache, proj[:, w.cols["dkv"]:w.cols["dkv"] + C + R], w.dkv_norm, q, w.cos_sin,
                           b["positions"], b["slot_mapping"], C, R, H, Dn, m.rot_dims, eps, interleaved=True)
        q_abs = torch.empty(T, H, C, dtype=self.dtype, device=h.device)
        sm.gemm(q.view(T, H, Dn + R)[:, :, :Dn].permute(1, 0, 2), w.uk_t, out=q_abs.permute(1, 0, 2))
        lat = sm.latent_attention(q_abs, q, cache, b["block_tables"], b["tok_seq"], b["positions"], C, R, H, Dn, 0,
                                  m.scale, self.block_size, b.get("max_keys", 0), b["cu_q"], b.get("max_qlen", 0),
                                  sinks=w.sinks)                           # [T, H, C]
        a = torch.empty(T, H, V, dtype=self.dtype, device=h.device)
        sm.gemm(lat.permute(1, 0, 2), w.uv, out=a.permute(1, 0, 2))
        y = sm.gate_mul(a.view(T, H * V), proj[:, w.cols["g"]:w.cols["g"] + H * V], sm.GATE_SIGMOID)
        return sm.linear(y, w.o)

    def _capped_attention(self, w: _Capped, h, b) -> torch.Tensor:
        a = w.cfg
        H, G, D, V = a.heads, a.kv_heads, a.dim, a.vdim
        kc, vc = self.kv_cache[w.cache]
        proj = sm.linear(h, w.w_in)                                        # [T, q | k | v | gate]
        sm.window_kv_write(kc, vc, proj, w.cols["k"], w.cols["v"], None, None, None, None, b["positions"],
                           b["slot_mapping"], H, G, D, V, 0, self.cfg.rms_eps, False, head_qnw=w.qnw, head_knw=w.knw)
        y = sm.window_attention(proj, proj[:, w.cols["g"]:w.cols["g"] + H * V], kc, vc, None, None, b["block_tables"],
                                b["tok_seq"], b["positions"], H, 0, 0, a.scale, False, self.block_size, b["cu_q"],
                                b.get("max_qlen", 0), b.get("max_keys", 0), softcap=a.softcap)
        return sm.linear(y, w.o)

    def _ssd(self, w: _Ssd, h, b) -> torch.Tensor:
        m = w.cfg
        H, V, N, G = m.heads, m.vdim, m.state, m.groups
        inner, n = m.inner, m.conv_channels
        conv_state, S = self.states[w.state]
        proj = sm.linear(h, w.w_in, out_dtype=F32)                         # what enters the recurrence stays fp32
        xbc = sm.short_conv(proj[:, inner:inner + n], w.taps, conv_state, b["cu_q"], b["tok_seq"], b["seq_slots"],
                            b["positions"], out_bias=w.conv_b, act=sm.CONV_SILU)
        cols = {"v": 0, "k": inner, "q": inner + G * N, "g": 0, "f": inner + n}
        y = sm.gated_scan(xbc, sm.SCAN_SSD, cols, None, S, b["cu_q"], b["seq_slots"], b["positions"], H, N, V,
                          self.cfg.rms_eps, F32, aux=proj, head_params=w.head_params, groups=G)
        y = sm.norm_mix(y, w.norm, None, None, self.cfg.rms_eps, out_dtype=self.dtype, groups=m.norm_groups)
        return sm.linear(y, w.o)

    def _blocks(self, ids, b, after=None) -> torch.Tensor:
        """The residual stream after the last layer (normed: every layer ends with a norm)."""
        c, dt = self.cfg, self.dtype
        x = sm.embed_rows(ids, self.embed, c.embed_scale)
        for L in self.layers:
            if L.taps is not None:
                h = sm.short_conv(x, L.taps, self.states[L.canon][0], b["cu_q"], b["tok_seq"], b["seq_slots"],
                                  b["positions"], residual=True, out_dtype=dt)
            else:
                h = x.to(dt)
            w = L.mixer
            if isinstance(w, _Latent):
                h2 = sm.postnorm(x, self._latent(w, h, b), c.alpha, L.gain1, c.rms_eps, out_dtype=dt)
            else:
                h2 = sm.postnorm(x, self._capped_attention(w.left, h, b), c.alpha, L.gain1, c.rms_eps,
                                 branch2=self._ssd(w.right, h, b), c1=w.cfg.left_scale, c2=w.cfg.right_scale,
                                 out_dtype=dt)
            if L.post2:
                f = sm.linear(sm.act(sm.linear(h2, L.w_up), sm.ACT_GELU_ERF), L.w_down) if L.w_up is not None else None
                sm.postnorm(x, f, c.alpha, L.gain2, c.rms_eps)
            if after is not None:
                after.append(x.clone())
        return x

    def _forward(self, ids, b, rows) -> torch.Tensor:
        c = self.cfg
        x = self._blocks(ids, b)
        hf = sm.postnorm(x.index_select(0, rows), None, 1.0, self.final_gain, c.rms_eps, out_dtype=self.dtype)
        return sm.linear(hf, self.lm_head, out_dtype=F32).unsqueeze(0)     # [1, S, vocab]

    def residual_after_runs(self, ids, b) -> List[torch.Tensor]:
        """(debugging / tests) the fp32 residual stream after every layer."""
        after: List[torch.Tensor] = []
        self._blocks(ids, b, after)
        return after
