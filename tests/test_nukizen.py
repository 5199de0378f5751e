"""Nukizen through the engine (checkpoint loader, registry, slots, paged caches shared between layers, recurrent and
convolution state, replay and generation entry points) against the plain float64 oracle in nukizen_oracle.py.  Every
test runs on the CPU (reference ops: model, cache, state and scheduler logic) and, marked gpu, on the HIP kernels.
Small own configurations, random weights; where random weights would hide a fault the weights are shaped so that it
shows."""

import copy

import pytest
import torch

import nukizen_oracle as oracle
from k8s_llm_scheduler_amd.engine import SamplingParams, build_engine
from k8s_llm_scheduler_amd.models import load_config, model_class
from k8s_llm_scheduler_amd.models.nukizen import (NukizenModel, config_from_json, config_to_json, random_tensors,
                                                  save_checkpoint)

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
TOL = {"float32": 3e-4, "bfloat16": 6e-2}
YARN = {"factor": 3.0, "original": 48, "fast": 6.0, "slow": 1.5}


def att(heads=4, kv_heads=2, dim=12, vdim=10, chunk=7, dims=8, base=5000.0, scale=0.4, softcap=5.0, kv_from=None,
        scaling=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if dims:
        m["rot"] = {"dims": dims, "base": base, **({"scaling": scaling} if scaling else {})}
    if chunk:
        m["mask"] = {"size": chunk}
    if softcap:
        m["softcap"] = softcap
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def attention(ff=0, **kw):
    return {"type": "attention", "mixer": att(**kw), "mlp": {"kind": "dense", "ff": ff} if ff else None}


def rglru(width=24, blocks=3, conv=4, ff=0):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def delta(heads=4, kv_heads=2, dim=8, vdim=12, conv=3):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def parallel(ff=0, right=None, **left):
    left.setdefault("softcap", 0.0)
    left.setdefault("scaling", YARN)
    left.setdefault("chunk", 9)
    return {"type": "parallel", "mixer": {"left": att(**left), "right": right or delta()},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=48, vocab=90, eps=1e-5, cap=12.0):
    c = {"architecture": "Nukizen", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps}}
    if cap:
        c["logit_softcap"] = cap
    return c


FULL = config([attention(ff=40), parallel(ff=56), rglru(ff=40), attention(ff=24, kv_from=0, chunk=11, heads=2),
               parallel(chunk=13, heads=2, kv_heads=1, dim=16, vdim=16, dims=16, right=delta(heads=2, kv_heads=2, dim=12, vdim=6, conv=2))])


def make(tmp_path, cfg, device, dtype, seed=0, max_tokens=256, slots=4, graphs=False, edit=None):
    pc = config_from_json(cfg, "case")
    tensors = random_tensors(pc, seed)
    if edit:
        edit(tensors)
    save_checkpoint(pc, tensors, tmp_path / "ckpt")
    eng = build_engine(weights=str(tmp_path / "ckpt"), device=device, dtype=dtype, max_batch=slots, block_size=16,
                       num_blocks=max_tokens // 16, max_model_len=max_tokens, cuda_graphs=graphs, capture=graphs)
    assert isinstance(eng.model, NukizenModel)
    return eng, tensors


def expect(cfg, tensors, toks, streams=False):
    logits, after = oracle.forward(tensors, cfg, toks)
    return (logits, after) if streams else logits


def row_errs(got, want):
    """Per row: rms of the difference (its mean taken off) over the rms of the centred expected row."""
    got, want = got.double(), want.double()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def rel_err(got, want):
    return row_errs(got, want).max().item()


def close(got, want, dtype):
    """float32: every row within rounding.  bfloat16: models this small amplify the rounding of single rows (a
    48-wide norm, a head's output divided by its own small root mean square) -- nine rows in ten (all but one of a
    short request) must be tight, none far off."""
    e = row_errs(got, want)
    if dtype == "float32":
        return e.max().item() < TOL[dtype]
    return int((e >= TOL[dtype]).sum()) <= max(1, e.numel() // 10) and e.max().item() < 0.3


def tokens(n, vocab, seed, avoid=()):
    g = torch.Generator().manual_seed(seed)
    out = torch.randint(0, vocab, (n,), generator=g).tolist()
    return [t if t not in avoid else (t + 1) % vocab for t in out]


def whole(eng, key, toks):
    return eng.replay_step([(key, toks, list(range(len(toks))))], [key])


def stepwise(eng, key, toks, first):
    """The first ``first`` tokens as one portion, the rest one by one."""
    rows = [eng.replay_step([(key, toks[:first], list(range(first)))])] if first else []
    rows += [eng.replay_step([(key, [t], [0])]) for t in toks[first:]]
    return torch.cat(rows)


# ----------------------------------------------------------------------------- registry, configuration, loader
def test_registry_and_config_roundtrip(tmp_path):
    pc = config_from_json(FULL, "x")
    assert config_from_json(config_to_json(pc), "x") == pc
    save_checkpoint(pc, random_tensors(pc, 1), tmp_path / "m")
    got = load_config(str(tmp_path / "m"))
    assert model_class(got) is NukizenModel and got.layers == pc.layers
    assert (got.rms_eps, got.logit_softcap) == (1e-5, 12.0)
    a = got.layers[3].mixer
    assert (a.chunk, a.kv_from, a.rot_dims, a.softcap, a.heads, a.gate, a.sink) == (11, 0, 8, 5.0, 2, True, False)
    left, right = got.layers[1].mixer
    assert (left.rot_scaling, left.sink, left.qk_norm, left.gate, right.conv) == (YARN, True, True, False, 3)
    assert model_class(load_config("nukizen-tiny")) is NukizenModel
    assert model_class(load_config("rupatar-tiny")).__name__ == "RupatarModel"
    assert model_class(load_config("tiny")).__name__ == "LlamaModel"


def test_yarn_table_matches_the_oracle():
    """The angle table of the scaled rotation, per pair, against the oracle's frequencies and magnitude."""
    from k8s_llm_scheduler_amd.ops import reference as ref

    for dims, base, sc in ((16, 5000.0, YARN), (8, 100.0, {"factor": 8.0, "original": 20, "fast": 3.0, "slow": 0.5}),
                           (12, 1e6, {"factor": 1.5, "original": 4096, "fast": 32.0, "slow": 1.0})):
        f, m = oracle.rotary_frequencies({"dims": dims, "base": base, "scaling": sc})
        table = ref.rope_table(dims, 70, base, {"type": "yarn", **sc}).double()
        ang = torch.arange(70, dtype=torch.float64)[:, None] * f[None, :]
        assert torch.allclose(table, torch.cat([ang.cos() * m, ang.sin() * m], -1), atol=1e-6)
        plain, _ = oracle.rotary_frequencies({"dims": dims, "base": base})
        assert not torch.allclose(f, plain)                     # the scaling changes some pair


# ----------------------------------------------------------------------------- each mechanism alone
MECHANISMS = {
    "attention_chunked_capped_gated": config([attention()]),
    "attention_no_mask": config([attention(chunk=0)]),
    "attention_chunk_of_one": config([attention(chunk=1)]),
    "attention_chunk_is_a_page": config([attention(chunk=16)]),
    "attention_full_rotation": config([attention(dims=12)]),
    "attention_no_rotation_no_cap": config([attention(dims=0, softcap=0.0)]),
    "attention_one_kv_head": config([attention(heads=3, kv_heads=1)]),
    "attention_all_kv_heads": config([attention(heads=3, kv_heads=3)]),
    "attention_tight_cap": config([attention(softcap=0.3, scale=2.0)]),
    "shared_cache": config([attention(), rglru(), attention(kv_from=0, chunk=5, heads=6, softcap=0.0),
                            attention(kv_from=0, chunk=0, dims=8)]),
    "feed_forward": config([attention(ff=36)]),
    "rglru": config([rglru()]),
    "rglru_one_block_no_history": config([rglru(width=20, blocks=1, conv=1)]),
    "rglru_block_per_channel_long_taps": config([rglru(width=7, blocks=7, conv=9)]),
    "parallel": config([parallel()]),
    "parallel_plain_frequencies": config([parallel(scaling=None, dims=4)]),
    "parallel_no_mask": config([parallel(chunk=0, right=delta(heads=2, kv_heads=2, conv=1))]),
    "parallel_one_head_each": config([parallel(heads=1, kv_heads=1, right=delta(heads=1, kv_heads=1, dim=5, vdim=3, conv=5))]),
    "no_logit_cap": config([rglru(ff=12)], cap=0.0),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_mechanism_alone(tmp_path, device, name):
    cfg = MECHANISMS[name]
    eng, tensors = make(tmp_path, cfg, device, "float32")
    toks = tokens(45, cfg["vocab"], 3)
    assert rel_err(whole(eng, "a", toks), expect(cfg, tensors, toks)) < TOL["float32"]


def test_mechanisms_move_the_output():
    """The premise of the tests above, on the oracle: every constant and optional part changes the logits by far more
    than the tolerance -- a chunk one token longer or shorter, the cap, the sink, the gate, the scaled rotation, the
    layer whose cache is read, the convolution's taps, the decay."""
    toks = tokens(45, 90, 3)

    def moved(cfg, other, edit=None, seed=0):
        t = random_tensors(config_from_json(cfg, "a"), seed)
        t2 = dict(t)
        if edit:
            edit(t2)
        return rel_err(expect(other, t2, toks), expect(cfg, t, toks))

    base = config([attention()])
    for change in (dict(chunk=6), dict(chunk=8), dict(softcap=4.0), dict(softcap=0.0), dict(scale=0.5), dict(dims=6),
                   dict(base=4000.0)):
        assert moved(base, config([attention(**change)])) > 0.01, change
    assert moved(base, base, lambda t: t.pop("l0.mix.g")) > 0.01
    side = config([parallel()])
    for change in (dict(chunk=8), dict(scaling=None), dict(scaling={**YARN, "factor": 2.0}), dict(scaling={**YARN, "slow": 0.1})):
        assert moved(side, config([parallel(**change)])) > 0.003, change
    for name in ("l0.mix.left.sink", "l0.mix.left.q.norm", "l0.mix.left.k.norm"):
        assert moved(side, side, lambda t: t.pop(name)) > 0.003, name
    assert moved(side, side, lambda t: t.update({"l0.mix.right.A_log": t["l0.mix.right.A_log"] + 1.0})) > 0.003
    assert moved(side, side, lambda t: t.update({"l0.mix.right.k.conv": t["l0.mix.right.k.conv"].flip(1)})) > 0.003
    shared = config([attention(), attention(chunk=0), attention(kv_from=0, chunk=0)])
    other = copy.deepcopy(shared)
    other["layers"][2]["mixer"]["kv_from"] = 1
    assert moved(shared, other) > 0.01
    lru = config([rglru()])
    assert moved(lru, lru, lambda t: t.update({"l0.mix.lam": t["l0.mix.lam"] + 1.0})) > 0.003
    assert moved(lru, lru, lambda t: t.update({"l0.mix.conv": t["l0.mix.conv"].flip(1)})) > 0.003
    assert moved(lru, lru, lambda t: t.update({"l0.mix.ra": t["l0.mix.ra"].flip(0)})) > 0.003


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_full_model_and_layer_streams(tmp_path, device, dtype):
    eng, tensors = make(tmp_path, FULL, device, dtype)
    toks = tokens(45, FULL["vocab"], 4)
    want, streams = expect(FULL, tensors, toks, streams=True)
    assert close(whole(eng, "a", toks), want, dtype)
    m, dev = eng.model, eng.device
    T = len(toks)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    b = m.batch_meta(i32(list(range(T))), i32(list(range(T))), i32([0, T]), i32([list(range(16))]), i32([0]))
    b["max_qlen"] = T
    got = m.residual_after_runs(i32(toks), b)
    assert len(got) == len(streams) == len(FULL["layers"])
    for g, w in zip(got, streams):
        assert close(g.cpu(), w, dtype)


# ----------------------------------------------------------------------------- cutting, batching, reuse
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_against_token_by_token(tmp_path, device, dtype):
    eng, tensors = make(tmp_path, FULL, device, dtype)
    toks = tokens(40, FULL["vocab"], 5)
    want = expect(FULL, tensors, toks)
    rows = [eng.replay_step([("s", [t], [0])], ["s"] if i == len(toks) - 1 else []) for i, t in enumerate(toks)]
    assert close(torch.cat(rows), want, dtype)
    assert len(eng.free_slots) == eng.max_batch and eng.allocator.num_free == eng.num_blocks


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2, 2, 2, 3, 1, 1, 29], [17, 16, 1, 6], [1, 15, 16, 8], [39, 1], [5] * 8])
def test_portions(tmp_path, device, sizes):
    """Portions down to two tokens and single tokens: shorter than the convolutions' taps, across chunk and page
    borders."""
    eng, tensors = make(tmp_path, FULL, device, "float32")
    toks = tokens(sum(sizes), FULL["vocab"], 6)
    want = expect(FULL, tensors, toks)
    rows, at = [], 0
    for n in sizes:
        rows.append(eng.replay_step([("p", toks[at:at + n], list(range(n)))]))
        at += n
    assert rel_err(torch.cat(rows), want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batch_against_each_alone_with_reuse(tmp_path, device, dtype):
    """Four slots and 96 cache tokens for six requests of unequal length: portions of some beside single tokens of
    others, requests left out of steps, slots and blocks taken again by later requests."""
    eng, tensors = make(tmp_path, FULL, device, dtype, max_tokens=96, slots=4)
    V = FULL["vocab"]
    seqs = {k: tokens(n, V, 10 + i) for i, (k, n) in enumerate([("a", 30), ("b", 7), ("c", 18), ("d", 1), ("e", 33),
                                                                 ("f", 20)])}
    want = {k: expect(FULL, tensors, v) for k, v in seqs.items()}
    plan = [  # (key, count) per step
        [("a", 11), ("b", 3)],
        [("a", 1), ("b", 2), ("c", 9), ("d", 1)],            # d ends: its slot is free again
        [("a", 1), ("c", 2)],                                 # b left out
        [("a", 1), ("b", 1), ("c", 1), ("e", 5)],             # e takes d's slot
        [("a", 16), ("b", 1), ("c", 6), ("e", 2)],            # a, b, c end
        [("e", 1), ("f", 20)],                                # f in a freed slot and freed blocks
        [("e", 25)],
    ]
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    for step in plan:
        entries, end = [], []
        for k, n in step:
            entries.append((k, seqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(seqs[k]):
                end.append(k)
        rows = eng.replay_step(entries, end)
        o = 0
        for k, n in step:
            got[k].append(rows[o:o + n])
            o += n
    assert at == {k: len(v) for k, v in seqs.items()}
    for k in seqs:
        assert close(torch.cat(got[k]), want[k], dtype), k
    assert len(eng.free_slots) == 4 and eng.allocator.num_free == eng.num_blocks


@pytest.mark.parametrize("device", DEVICES)
def test_reused_slot_and_pages_start_clean(tmp_path, device):
    """One slot, one request after another: the second must not see the first's recurrent states, saved convolution
    inputs or cached rows."""
    cfg = config([rglru(), parallel(chunk=0), attention(chunk=0), attention(kv_from=2, chunk=0)])
    eng, tensors = make(tmp_path, cfg, device, "float32", max_tokens=32, slots=1)
    a, b = tokens(30, cfg["vocab"], 1), tokens(25, cfg["vocab"], 2)
    whole(eng, "a", a)
    got = [eng.replay_step([("b", b[:1], [0])]), eng.replay_step([("b", b[1:9], list(range(8)))]),
           eng.replay_step([("b", b[9:], list(range(16)))], ["b"])]
    assert rel_err(torch.cat(got), expect(cfg, tensors, b)) < TOL["float32"]


# ----------------------------------------------------------------------------- chunk edges, far keys
LOUD, DIM_U = 7, 10


def loud_weights(cfg):
    """One token is made loud: width coordinate 0 is set for it only and coordinate 1 for every token; every key head
    maps coordinate 0 onto the unrotated head dimension DIM_U and every query head coordinate 1, so the loud token's
    key dominates every softmax it is part of (in the first layer; later layers inherit what it leaves)."""
    def edit(t):
        t["embed"][:, 0] = 0
        t["embed"][:, 1] = 1.0
        t["embed"][LOUD] = 0
        t["embed"][LOUD, 0] = 8.0
        t["embed"][LOUD, 1] = 1.0
        for i, L in enumerate(cfg["layers"]):
            for p, m in ((f"l{i}.mix.", L["mixer"]),) if L["type"] == "attention" else \
                    ((f"l{i}.mix.left.", L["mixer"]["left"]),) if L["type"] == "parallel" else ():
                D = m["dim"]
                if p + "k" in t:
                    for g in range(m["kv_heads"]):
                        t[p + "k"][g * D + DIM_U, 0] = 4.0
                for h in range(m["heads"]):
                    t[p + "q"][h * D + DIM_U, 1] = 6.0
    return edit


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("chunk,side", [(1, 2), (2, 3), (16, 17), (17, 15), (5, 32), (21, 9)])
def test_chunk_edges_in_prompt_and_decoding(tmp_path, device, chunk, side):
    """The loud token is seen by the rest of its chunk and by nobody in the next one: placed first, last and inside
    chunks, in a prompt portion and among tokens decoded one by one, across page borders (pages of 16); a capped
    attention layer, the attention of a parallel layer with a sink and a layer on the first one's cache."""
    cfg = config([attention(chunk=chunk, dim=16, dims=6, scale=1.0, heads=2, kv_heads=1, softcap=20.0),
                  parallel(chunk=side, dim=16, vdim=16, dims=8, scale=0.5, heads=2, kv_heads=2, ff=24),
                  attention(chunk=chunk + 2, kv_from=0, dim=16, dims=6, scale=1.0, heads=3, kv_heads=1, softcap=9.0)], vocab=60)
    eng, tensors = make(tmp_path, cfg, device, "float32", edit=loud_weights(cfg))
    toks = tokens(90, 60, 8, avoid=(LOUD,))
    places = (3, 14, 31, 40, 52, 63, 64)
    for p in places:
        toks[p] = LOUD
    want = expect(cfg, tensors, toks)
    quiet = expect(cfg, tensors, [8 if t == LOUD else t for t in toks])
    assert rel_err(quiet, want) > 0.05                     # the loud token matters
    got = stepwise(eng, "w", toks, 36)
    assert rel_err(got, want) < TOL["float32"]
    for p in places:                                        # the rows around each edge, one by one
        for n in (chunk, side, chunk + 2):
            last = p // n * n + n - 1                       # the last query that sees p; the next one does not
            for i in (last, last + 1):
                if i < len(toks):
                    assert rel_err(got[i:i + 1], want[i:i + 1]) < TOL["float32"], (p, n, i)


@pytest.mark.parametrize("device", DEVICES)
def test_far_keys_and_long_decoding(tmp_path, device):
    """Unmasked attention, a long chunk and both recurrences: position 200+ still depends on the first tokens (checked
    on the oracle), over many page borders, with 90 tokens decoded one by one."""
    cfg = config([attention(chunk=0, dim=16, dims=6, scale=1.0, heads=2, kv_heads=1), rglru(width=16, blocks=2),
                  parallel(chunk=150, dim=16, vdim=8, dims=16, heads=2, kv_heads=2, ff=16,
                           scaling={"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}),
                  attention(chunk=0, kv_from=0, dim=16, dims=6, heads=4, kv_heads=1)], width=32, vocab=50)
    eng, tensors = make(tmp_path, cfg, device, "float32", max_tokens=256, edit=loud_weights(cfg))
    toks = tokens(215, 50, 9, avoid=(LOUD,))
    toks[1] = toks[64] = LOUD
    want = expect(cfg, tensors, toks)
    other = expect(cfg, tensors, [toks[0], 8] + toks[2:])
    assert rel_err(other[-1:], want[-1:]) > 1e-3            # the end sees position 1
    rows = [eng.replay_step([("f", toks[:100], list(range(100)))]), eng.replay_step([("f", toks[100:125], list(range(25)))])]
    rows += [eng.replay_step([("f", [t], [0])]) for t in toks[125:]]
    assert rel_err(torch.cat(rows), want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_among_hundreds(tmp_path, device):
    """One unmasked attention layer: the loud token lies hundreds of positions back; the last rows change by far more
    than the tolerance when it is silenced, and the engine follows the oracle."""
    cfg = config([attention(chunk=0, dim=16, dims=6, scale=1.0, heads=2, kv_heads=1, softcap=25.0)], width=32, vocab=50)
    eng, tensors = make(tmp_path, cfg, device, "float32", max_tokens=320, edit=loud_weights(cfg))
    toks = tokens(300, 50, 11, avoid=(LOUD,))
    toks[20] = LOUD
    want = expect(cfg, tensors, toks)
    other = expect(cfg, tensors, toks[:20] + [8] + toks[21:])
    assert rel_err(other[-3:], want[-3:]) > 0.005
    got = torch.cat([eng.replay_step([("g", toks[:250], list(range(250)))]), stepwise(eng, "g", toks[250:], 0)])
    assert rel_err(got, want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_a_large_sink_takes_its_share(tmp_path, device):
    """Sinks as large as the scores: heads give most of their weight away; left out, the rows would be far off."""
    cfg = config([parallel(chunk=6)])

    def edit(t):
        t["l0.mix.left.sink"] = torch.tensor([4.0, -3.0, 2.0, 0.5]).to(torch.bfloat16)

    eng, tensors = make(tmp_path, cfg, device, "float32", edit=edit)
    toks = tokens(40, cfg["vocab"], 12)
    want = expect(cfg, tensors, toks)
    without = dict(tensors)
    without.pop("l0.mix.left.sink")
    assert rel_err(expect(cfg, without, toks), want) > 0.02
    assert rel_err(stepwise(eng, "s", toks, 25), want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(tmp_path, device):
    eng, tensors = make(tmp_path, FULL, device, "float32")
    for n in (1, 2, 3):
        toks = tokens(n, FULL["vocab"], 20 + n)
        assert rel_err(whole(eng, f"s{n}", toks), expect(FULL, tensors, toks)) < TOL["float32"]
    toks = tokens(4, FULL["vocab"], 30)
    got = [eng.replay_step([("x", toks[:1], [0])]), eng.replay_step([("x", toks[1:2], [0])]),
           eng.replay_step([("x", toks[2:], [0, 1])], ["x"])]
    assert rel_err(torch.cat(got), expect(FULL, tensors, toks)) < TOL["float32"]


# ----------------------------------------------------------------------------- other sizes
OTHER_SIZES = [
    # head sizes above one wave, many query heads per key head (more than the waves of a workgroup), long taps
    config([attention(heads=20, kv_heads=2, dim=72, vdim=80, chunk=40, dims=70, scale=0.11, ff=30),
            parallel(heads=6, kv_heads=3, dim=80, vdim=72, chunk=33, dims=40, scale=0.1,
                     right=delta(heads=2, kv_heads=1, dim=72, vdim=96, conv=6)),
            rglru(width=130, blocks=2, conv=7, ff=20)], width=40, vocab=77, eps=1e-6),
    # odd sizes everywhere
    config([attention(heads=5, kv_heads=5, dim=7, vdim=9, chunk=11, dims=6, base=100.0, scale=0.6, ff=13),
            rglru(width=15, blocks=5, conv=2),
            parallel(heads=3, kv_heads=1, dim=10, vdim=3, chunk=7, dims=6, right=delta(heads=3, kv_heads=3, dim=5, vdim=13, conv=4), ff=7),
            attention(heads=5, kv_heads=5, dim=7, vdim=9, chunk=2, dims=2, scale=0.3, kv_from=0)], width=37, vocab=53),
    # one of everything: one head, one channel per block, value size one, chunks longer than the sequence
    config([attention(heads=1, kv_heads=1, dim=4, vdim=1, chunk=500, dims=4, scale=1.0, ff=1),
            rglru(width=1, blocks=1, conv=1), parallel(heads=1, kv_heads=1, dim=2, vdim=1, chunk=500, dims=2,
                                                       right=delta(heads=1, kv_heads=1, dim=2, vdim=1, conv=1))], width=8, vocab=11),
    # delta-rule heads wider than two waves: key channels in groups of 32 and 64
    config([parallel(right=delta(heads=1, kv_heads=1, dim=40, vdim=200, conv=3)),
            parallel(right=delta(heads=2, kv_heads=1, dim=144, vdim=136, conv=2), ff=16),
            parallel(right=delta(heads=2, kv_heads=2, dim=250, vdim=24, conv=4))], width=48, vocab=31),
    # aligned sizes, mixers of different widths in one model, two cache owners with readers of each
    config([attention(heads=8, kv_heads=4, dim=32, vdim=16, chunk=33, dims=32, scale=0.18, ff=64),
            attention(heads=8, kv_heads=2, dim=64, vdim=16, chunk=64, dims=16, scale=0.125),
            rglru(width=64, blocks=4), attention(heads=4, kv_heads=4, dim=32, vdim=16, chunk=0, dims=32, kv_from=0),
            parallel(heads=4, kv_heads=2, dim=32, vdim=32, dims=32, chunk=48, right=delta(heads=4, kv_heads=2, dim=32, vdim=64), ff=32),
            attention(heads=2, kv_heads=2, dim=64, vdim=16, chunk=20, dims=16, kv_from=1)], width=64, vocab=80),
]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("case", range(len(OTHER_SIZES)))
def test_other_sizes(tmp_path, device, case):
    cfg = OTHER_SIZES[case]
    eng, tensors = make(tmp_path, cfg, device, "float32")
    toks = tokens(70, cfg["vocab"], 40 + case)
    assert rel_err(stepwise(eng, "o", toks, 45), expect(cfg, tensors, toks)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_bfloat16_aligned_sizes_long_context(tmp_path, device):
    """Sizes whose rows are 16-byte aligned (on the GPU: the matrix-core kernels) in bfloat16: a prompt in portions,
    then 70 tokens one by one, chunks across many pages."""
    cfg = config([attention(heads=4, kv_heads=2, dim=16, vdim=16, chunk=0, dims=8, scale=0.25, ff=32),
                  parallel(heads=16, kv_heads=2, dim=32, vdim=16, chunk=37, dims=16, scale=0.18,
                           right=delta(heads=2, kv_heads=1, dim=32, vdim=32)),
                  rglru(width=64, blocks=2, ff=32), attention(heads=8, kv_heads=2, dim=16, vdim=16, chunk=50, dims=8, kv_from=0)],
                 width=64, vocab=80)
    eng, tensors = make(tmp_path, cfg, device, "bfloat16", max_tokens=256)
    toks = tokens(190, 80, 12)
    want = expect(cfg, tensors, toks)
    rows = [eng.replay_step([("m", toks[:90], list(range(90)))]), eng.replay_step([("m", toks[90:120], list(range(30)))])]
    rows += [eng.replay_step([("m", [t], [0])]) for t in toks[120:]]
    assert close(torch.cat(rows), want, "bfloat16")


@pytest.mark.parametrize("device", DEVICES)
def test_long_portion_of_the_recurrences(tmp_path, device):
    """A portion long enough for the time-sliced scan, then a short one and single tokens from the state it left."""
    cfg = config([rglru(width=40, blocks=2, conv=4), parallel(chunk=64, ff=16)], width=32, vocab=50)
    eng, tensors = make(tmp_path, cfg, device, "float32", max_tokens=320)
    toks = tokens(300, 50, 14)
    want = expect(cfg, tensors, toks)
    got = torch.cat([eng.replay_step([("l", toks[:280], list(range(280)))]),
                     eng.replay_step([("l", toks[280:295], list(range(15)))]), stepwise(eng, "l", toks[295:], 0)])
    assert rel_err(got, want) < TOL["float32"]


# ----------------------------------------------------------------------------- generation entry point
@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(tmp_path, device):
    """engine.generate: admission, chunked prefill, mixed steps and (on the GPU) the captured decode graphs; three
    prompts of unequal length on two slots, so the third waits for a slot and reuses it."""
    eng, tensors = make(tmp_path, FULL, device, "float32", max_tokens=192, slots=2, graphs=device == "cuda", seed=3)
    prompts = [tokens(n, FULL["vocab"], 50 + n) for n in (21, 5, 34)]
    sp = SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True, stop_on_json_close=False)
    outs = eng.generate(prompts, sp)
    for p, o in zip(prompts, outs):
        assert o.finish_reason == "length" and o.token_ids == oracle.greedy(tensors, FULL, p, 12)
    if device == "cuda":
        assert eng.stats["graph_replays"] > 0
    assert len(eng.free_slots) == 2 and eng.allocator.num_free == eng.num_blocks


# ----------------------------------------------------------------------------- command line
def test_replay_and_generate_command_line(tmp_path):
    """The replay runner as a user starts it: steps on standard input, one logits file per step that wants rows,
    `done <step>` after every step; and `generate` on token ids."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parent.parent
    cfg = config([attention(ff=20), parallel(), rglru(ff=12), attention(kv_from=0)])
    pc = config_from_json(cfg, "cli")
    tensors = random_tensors(pc, 5)
    save_checkpoint(pc, tensors, tmp_path / "ckpt")
    a, b = tokens(21, cfg["vocab"], 70), tokens(9, cfg["vocab"], 71)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[17:18], "want": []}, {"id": "b", "tokens": b, "want": [8]}],
              "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[18:], "want": [2]}], "end": ["a"]}]
    out = tmp_path / "out"
    r = subprocess.run([str(root / "bin" / "trace_run"), "--model", str(tmp_path / "ckpt"), "--dtype", "float32", "--out",
                        str(out), "--max-tokens", "64", "--device", "cpu"], input="\n".join(map(json.dumps, steps)) + "\n",
                       capture_output=True, text=True, timeout=300, cwd=str(root))
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert sorted(p.name for p in out.iterdir()) == ["0.f32", "1.f32", "2.f32"]
    wa, wb = expect(cfg, tensors, a), expect(cfg, tensors, b)
    V = cfg["vocab"]
    got = {i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V)) for i in range(3)}
    assert rel_err(got[0], wa[[0, 16]]) < TOL["float32"]
    assert rel_err(got[1], wb[[8]]) < TOL["float32"]
    assert rel_err(got[2], wa[[20]]) < TOL["float32"]
    g = subprocess.run([sys.executable, "-m", "k8s_llm_scheduler_amd", "generate", "--model", str(tmp_path / "ckpt"),
                        "--dtype", "float32", "--prompt", " ".join(map(str, b)), "--max-new", "5", "--device", "cpu",
                        "--no-graphs"], capture_output=True, text=True, timeout=300, cwd=str(root))
    assert g.returncode == 0, g.stderr[-2000:]
    line = json.loads([l for l in g.stdout.splitlines() if l.startswith("{")][-1])
    assert line["token_ids"] == oracle.greedy(tensors, cfg, b, 5)


# ----------------------------------------------------------------------------- random configurations
def random_config(seed):
    """A random small model: 2-5 layers of any mixer in any order, with or without feed-forward, sizes that are and are
    not multiples of 8 / 16, chunks from 1 to beyond the sequence, layers that read an earlier layer's cache."""
    import random

    rng = random.Random(seed)
    aligned = rng.random() < 0.5
    pick = lambda xs: rng.choice(xs)
    width = pick([32, 64, 96]) if aligned else pick([24, 36, 52, 72])
    layers, owners = [], []
    for i in range(rng.randint(2, 5)):
        ff = pick([0, 16, 32]) if aligned else pick([0, 5, 12])
        r = rng.random()
        if r < 0.25:
            bw = pick([8, 16]) if aligned else pick([1, 5, 12])
            blocks = pick([1, 2, 4])
            layers.append(rglru(width=bw * blocks, blocks=blocks, conv=pick([1, 2, 4, 5]), ff=ff))
            continue
        kv = pick([1, 2, 3])
        dim = pick([8, 16, 24]) if aligned else pick([6, 10, 12])
        vdim = pick([16, 32]) if aligned else pick([5, 9])
        kw = dict(heads=kv * pick([1, 2, 5]), kv_heads=kv, dim=dim, vdim=vdim, chunk=pick([0, 1, 2, 7, 31, 32, 33, 50, 500]),
                  dims=pick([0, 2, dim // 2 * 2, dim // 4 * 2]), base=pick([100.0, 10000.0, 1e6]), scale=pick([0.1, 0.25, 0.5]))
        if r < 0.6:
            kw["softcap"] = pick([0.0, 2.0, 30.0])
            if owners and rng.random() < 0.4:
                j, okv, odim, ovdim, odims, obase = pick(owners)
                kw.update(kv_from=j, kv_heads=okv, heads=okv * pick([1, 2, 3]), dim=odim, vdim=ovdim, dims=odims, base=obase)
            else:
                owners.append((i, kv, dim, vdim, kw["dims"], kw["base"]))
            layers.append(attention(ff=ff, **kw))
        else:
            if kw["dims"]:
                kw["scaling"] = pick([None, {"factor": pick([2.0, 8.0]), "original": pick([16, 64]), "fast": pick([4.0, 32.0]),
                                             "slow": pick([0.5, 1.0])}])
            else:
                kw["scaling"] = None
            g = pick([1, 2])
            layers.append(parallel(ff=ff, right=delta(heads=g * pick([1, 2]), kv_heads=g,
                                                      dim=pick([8, 16, 32]) if aligned else pick([5, 12, 33]),
                                                      vdim=pick([8, 32]) if aligned else pick([6, 21]), conv=pick([1, 2, 3, 4])), **kw))
    return config(layers, width=width, vocab=pick([40, 64, 101]), eps=pick([1e-6, 1e-5]), cap=pick([0.0, 8.0, 30.0]))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, device, seed):
    """A prompt in two portions, a second request beside its decoded tokens, then tokens one by one."""
    cfg = random_config(seed)
    eng, tensors = make(tmp_path, cfg, device, "float32", seed=seed, max_tokens=160, slots=2)
    V = cfg["vocab"]
    a, b = tokens(75, V, 100 + seed), tokens(28, V, 200 + seed)
    wa, wb = expect(cfg, tensors, a), expect(cfg, tensors, b)
    ga = [eng.replay_step([("a", a[:40], list(range(40)))]), eng.replay_step([("a", a[40:43], [0, 1, 2])])]
    gb = []
    for i in range(43, 75):
        if i == 50:
            rows = eng.replay_step([("a", [a[i]], [0]), ("b", b[:20], list(range(20)))])
            gb.append(rows[1:])
        elif 50 < i <= 58:
            rows = eng.replay_step([("a", [a[i]], [0]), ("b", [b[20 + i - 51]], [0])], ["b"] if i == 58 else [])
            gb.append(rows[1:])
        else:
            rows = eng.replay_step([("a", [a[i]], [0])])
        ga.append(rows[:1])
    assert rel_err(torch.cat(ga), wa) < TOL["float32"], cfg
    assert rel_err(torch.cat(gb), wb) < TOL["float32"], cfg
