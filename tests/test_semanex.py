"""Semanex through the engine (checkpoint loader, registry, slots, paged caches, convolution and recurrent state, replay
and generation entry points) against the plain float64 oracle in semanex_oracle.py.  Every test runs on the CPU
(reference ops: model, cache, state and scheduler logic) and, marked gpu, on the HIP kernels.  Small own
configurations, random weights; where random weights would hide a fault the weights are shaped so that it shows."""

import pytest
import torch

import semanex_oracle as oracle
from k8s_llm_scheduler_amd.engine import SamplingParams, build_engine
from k8s_llm_scheduler_amd.models import load_config, model_class
from k8s_llm_scheduler_amd.models.semanex import (SemanexModel, config_from_json, config_to_json, random_tensors,
                                                  save_checkpoint)

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
TOL = {"float32": 3e-4, "bfloat16": 6e-2}


def latent(ff=0, heads=3, dim=12, rot_dim=8, vdim=10, kv_rank=20, q_rank=28, scale=0.3, base=5000.0, dims=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale, "rot": {"dims": rot_dim if dims is None else dims, "base": base}}
    return {"type": "latent_attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def capped(heads=4, kv_heads=2, dim=12, vdim=10, scale=0.4, softcap=5.0):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap}


def ssd(heads=4, vdim=6, state=10, groups=2, norm_groups=3, conv=4):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}


def parallel(ff=0, left=None, right=None, left_scale=1.3, right_scale=0.7):
    return {"type": "parallel", "mixer": {"left": left or capped(), "right": right or ssd(), "left_scale": left_scale,
                                          "right_scale": right_scale},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=48, vocab=90, eps=1e-5, alpha=1.5, taps=3, scale=5.0):
    c = {"architecture": "Semanex", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
         "postln_alpha": alpha, "embedding": {"scale": scale}}
    if taps:
        c["canon"] = {"taps": taps}
    return c


FULL = config([latent(ff=40), parallel(ff=56), latent(ff=24, heads=2, kv_rank=12, q_rank=9, rot_dim=4, base=100.0),
               parallel(left=capped(heads=2, kv_heads=1, dim=16, vdim=16, softcap=2.0),
                        right=ssd(heads=2, vdim=9, state=7, groups=1, norm_groups=1, conv=2)), latent()])


def make(tmp_path, cfg, device, dtype, seed=0, max_tokens=256, slots=4, graphs=False, edit=None):
    pc = config_from_json(cfg, "case")
    tensors = random_tensors(pc, seed)
    if edit:
        edit(tensors)
    save_checkpoint(pc, tensors, tmp_path / "ckpt")
    eng = build_engine(weights=str(tmp_path / "ckpt"), device=device, dtype=dtype, max_batch=slots, block_size=16,
                       num_blocks=max_tokens // 16, max_model_len=max_tokens, cuda_graphs=graphs, capture=graphs)
    assert isinstance(eng.model, SemanexModel)
    return eng, tensors


def expect(cfg, tensors, toks, streams=False):
    after = []
    logits = oracle.forward(tensors, cfg, toks, after)
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
    """float32: every row within rounding.  bfloat16: models this small amplify the rounding of single rows -- nine
    rows in ten (all but one of a short request) must be tight, none far off."""
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
    assert model_class(got) is SemanexModel and got.layers == pc.layers
    assert (got.rms_eps, got.alpha, got.embed_scale, got.canon_taps) == (1e-5, 1.5, 5.0, 3)
    a = got.layers[2].mixer
    assert (a.heads, a.kv_rank, a.q_rank, a.rot_dim, a.rot_dims, a.rot_base) == (2, 12, 9, 4, 4, 100.0)
    side = got.layers[3].mixer
    assert (side.left.softcap, side.left.kv_heads, side.right.groups, side.right.norm_groups, side.right.conv,
            side.left_scale, side.right_scale) == (2.0, 1, 1, 1, 2, 1.3, 0.7)
    assert model_class(load_config("semanex-tiny")) is SemanexModel
    assert model_class(load_config("nukizen-tiny")).__name__ == "NukizenModel"
    assert model_class(load_config("tiny")).__name__ == "LlamaModel"


# ----------------------------------------------------------------------------- each mechanism alone
MECHANISMS = {
    "latent": config([latent()]),
    "latent_one_head": config([latent(heads=1)]),
    "latent_partly_rotated": config([latent(rot_dim=8, dims=4)]),
    "latent_small_base": config([latent(base=20.0)]),
    "latent_rank_above_the_heads": config([latent(kv_rank=40, q_rank=7)]),
    "latent_feed_forward": config([latent(ff=36)]),
    "latent_no_input_convolution": config([latent(ff=12)], taps=0),
    "latent_one_tap": config([latent()], taps=1),
    "latent_five_taps": config([latent()], taps=5),
    "latent_alpha_one_no_scale": config([latent(ff=20)], alpha=1.0, scale=1.0),
    "parallel": config([parallel()]),
    "parallel_feed_forward": config([parallel(ff=30)]),
    "parallel_one_kv_head": config([parallel(left=capped(heads=3, kv_heads=1))]),
    "parallel_all_kv_heads": config([parallel(left=capped(heads=3, kv_heads=3))]),
    "parallel_tight_cap": config([parallel(left=capped(softcap=0.3, scale=2.0))]),
    "parallel_one_group": config([parallel(right=ssd(groups=1, norm_groups=1))]),
    "parallel_group_per_head": config([parallel(right=ssd(groups=4, norm_groups=4))]),
    "parallel_norm_group_per_channel": config([parallel(right=ssd(heads=2, vdim=3, norm_groups=6))]),
    "parallel_no_history": config([parallel(right=ssd(conv=1))], taps=1),
    "parallel_long_taps": config([parallel(right=ssd(conv=7))], taps=6),
    "parallel_left_only": config([parallel(right_scale=0.0)]),
    "parallel_right_only": config([parallel(left_scale=0.0)]),
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
    than the tolerance -- the sink, the gate, the cap, the pair layout of the rotation, the base, alpha, the taps of
    both convolutions, the decay, the skip, the step-size bias, the norm groups, the two scales, the norms' weights."""
    toks = tokens(45, 90, 3)

    def moved(cfg, other, edit=None, seed=0):
        t = random_tensors(config_from_json(cfg, "a"), seed)
        t2 = dict(t)
        if edit:
            edit(t2)
        return rel_err(expect(other, t2, toks), expect(cfg, t, toks))

    def bump(name, by=1.0):
        return lambda t: t.update({name: t[name] + by})

    base = config([latent()])
    for change in (dict(scale=0.4), dict(base=4000.0), dict(dims=6)):
        assert moved(base, config([latent(**change)])) > 0.003, change
    for other in (config([latent()], alpha=1.0), config([latent()], scale=4.0), config([latent()], eps=1e-2)):
        assert moved(base, other) > 0.003
    for name in ("l0.mix.sink", "l0.mix.dq.norm", "l0.mix.dkv.norm", "final.norm"):
        assert moved(base, base, bump(name)) > 0.003, name
    two = config([latent(ff=20), latent()])             # a gain matters to the sublayer that reads the normed stream
    for name in ("l0.norm1", "l0.norm2"):
        assert moved(two, two, bump(name)) > 0.003, name
    assert moved(base, base, lambda t: t.update({"l0.mix.g": t["l0.mix.g"] * 0})) > 0.01
    assert moved(base, base, lambda t: t.update({"l0.canon1": t["l0.canon1"].flip(1)})) > 0.01
    # the half layout instead of interleaved pairs: swap the roles of the rotated dimensions in q and k alike
    half = [0, 2, 4, 6, 1, 3, 5, 7]

    def relayout(t):
        uq = t["l0.mix.uq"].clone().view(3, 20, -1)
        uq[:, 12:] = uq[:, 12:][:, half]
        t["l0.mix.uq"] = uq.view(60, -1)
        dkv = t["l0.mix.dkv"].clone()
        dkv[20:] = dkv[20:][half]
        t["l0.mix.dkv"] = dkv

    assert moved(base, base, relayout) > 0.003
    side = config([parallel()])
    for change in (dict(left_scale=0.5), dict(right_scale=0.2), dict(left=capped(softcap=1.0)), dict(left=capped(scale=0.3)),
                   dict(right=ssd(norm_groups=1))):
        assert moved(side, config([parallel(**change)])) > 0.003, change
    for name in ("l0.mix.right.A_log", "l0.mix.right.D", "l0.mix.right.dt_bias", "l0.mix.right.conv.b",
                 "l0.mix.left.q.norm", "l0.mix.left.k.norm", "l0.mix.right.norm"):
        assert moved(side, side, bump(name)) > 0.003, name
    assert moved(side, side, lambda t: t.update({"l0.mix.right.conv": t["l0.mix.right.conv"].flip(1)})) > 0.003
    assert moved(side, side, lambda t: t.update({"l0.mix.left.g": t["l0.mix.left.g"] * 0})) > 0.003


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
    """Portions down to two tokens and single tokens: shorter than the convolutions' taps, across page borders."""
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
    """One slot, one request after another: the second must not see the first's recurrent state, the saved inputs of
    any convolution or the cached rows."""
    cfg = config([parallel(right=ssd(conv=5)), latent(), parallel()], taps=4)
    eng, tensors = make(tmp_path, cfg, device, "float32", max_tokens=32, slots=1)
    a, b = tokens(30, cfg["vocab"], 1), tokens(25, cfg["vocab"], 2)
    whole(eng, "a", a)
    got = [eng.replay_step([("b", b[:1], [0])]), eng.replay_step([("b", b[1:9], list(range(8)))]),
           eng.replay_step([("b", b[9:], list(range(16)))], ["b"])]
    assert rel_err(torch.cat(got), expect(cfg, tensors, b)) < TOL["float32"]


# ----------------------------------------------------------------------------- far keys, sinks, long memory
LOUD, DIM_U = 7, 10


def loud_weights(cfg):
    """One token is made loud: width coordinate 0 is set for it only and coordinate 1 for every token, and neither
    passes the input convolutions.  Left attentions: every key head maps coordinate 0 onto head dimension DIM_U and
    every query head coordinate 1 (per-head norms keep the directions).  Latent attentions: the shared rotated key part
    is not normed, so coordinate 0 is mapped, large, onto its slowest-turning pair; the query latent takes coordinate 1
    into its first channel, and from there into the same pair of every head.  The loud token's key then dominates
    every softmax it is part of (in the first layer; later layers inherit what it leaves)."""
    def edit(t):
        t["embed"][:, 0] = 0
        t["embed"][:, 1] = 1.0
        t["embed"][LOUD] = 0
        t["embed"][LOUD, 0] = 3.0
        t["embed"][LOUD, 1] = 1.0
        for i, L in enumerate(cfg["layers"]):
            if f"l{i}.canon1" in t:
                t[f"l{i}.canon1"][:2] = 0
            m = L["mixer"]
            if L["type"] == "parallel":
                p, a = f"l{i}.mix.left.", m["left"]
                D = a["dim"]
                for g in range(a["kv_heads"]):
                    t[p + "k"][g * D + DIM_U, 0] = 4.0
                for h in range(a["heads"]):
                    t[p + "q"][h * D + DIM_U, 1] = 6.0
            else:
                p = f"l{i}.mix."
                C, R, D = m["kv_rank"], m["rot_dim"], m["dim"]
                t[p + "dkv"][C + R - 2, 0] = 4.0
                t[p + "dq"][0, 1] = 6.0
                for h in range(m["heads"]):
                    t[p + "uq"][h * (D + R) + D + R - 2, 0] = 3.0
    return edit


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_among_hundreds(tmp_path, device):
    """The loud token lies hundreds of positions back, in a latent attention and in a capped attention: the last rows
    change by far more than the tolerance when it is silenced, and the engine follows the oracle through a long
    portion, a short one and single tokens."""
    for n, layer in enumerate((latent(dim=16, rot_dim=8, scale=0.5, base=1e6),
                               parallel(left=capped(heads=2, kv_heads=1, dim=16, vdim=8, scale=1.0, softcap=25.0),
                                        right_scale=0.1))):
        cfg = config([layer], width=32, vocab=50)
        eng, tensors = make(tmp_path / str(n), cfg, device, "float32", max_tokens=320, edit=loud_weights(cfg))
        toks = tokens(300, 50, 11, avoid=(LOUD,))
        toks[20] = LOUD
        want = expect(cfg, tensors, toks)
        other = expect(cfg, tensors, toks[:20] + [8] + toks[21:])
        assert rel_err(other[-3:], want[-3:]) > 0.005, n
        got = torch.cat([eng.replay_step([("g", toks[:250], list(range(250)))]),
                         eng.replay_step([("g", toks[250:263], list(range(13)))]), stepwise(eng, "g", toks[263:], 0)])
        assert rel_err(got, want) < TOL["float32"], n


@pytest.mark.parametrize("device", DEVICES)
def test_loud_keys_at_page_borders_and_long_decoding(tmp_path, device):
    """Loud tokens on both sides of page borders (pages of 16), in a prompt portion and among 90 tokens decoded one by
    one; all mixers; every row after a loud token depends on it."""
    cfg = config([latent(dim=16, rot_dim=8, scale=0.5, base=1e6, ff=16),
                  parallel(left=capped(heads=2, kv_heads=2, dim=16, vdim=8, scale=1.0, softcap=20.0), ff=24),
                  latent(heads=2, dim=16, rot_dim=4, scale=0.4)], width=32, vocab=60)
    eng, tensors = make(tmp_path, cfg, device, "float32", edit=loud_weights(cfg))
    toks = tokens(126, 60, 8, avoid=(LOUD,))
    places = (0, 15, 16, 31, 47, 48, 63, 64, 80, 95, 96)
    for p in places:
        toks[p] = LOUD
    want = expect(cfg, tensors, toks)
    quiet = expect(cfg, tensors, [8 if t == LOUD else t for t in toks])
    assert rel_err(quiet, want) > 0.05                     # the loud tokens matter
    got = stepwise(eng, "w", toks, 36)
    assert rel_err(got, want) < TOL["float32"]
    for p in places:                                        # the rows at and after each loud token, one by one
        for i in (p, p + 1, p + 2):
            assert rel_err(got[i:i + 1], want[i:i + 1]) < TOL["float32"], (p, i)


@pytest.mark.parametrize("device", DEVICES)
def test_a_large_sink_takes_its_share(tmp_path, device):
    """Sinks as large as the scores, and larger than any of them: heads give most of their weight away; left out, the
    rows would be far off."""
    cfg = config([latent(heads=4)])

    def edit(t):
        t["l0.mix.sink"] = torch.tensor([4.0, -3.0, 12.0, 0.5]).to(torch.bfloat16)

    eng, tensors = make(tmp_path, cfg, device, "float32", edit=edit)
    toks = tokens(40, cfg["vocab"], 12)
    want = expect(cfg, tensors, toks)
    without = dict(tensors)
    without["l0.mix.sink"] = torch.full((4,), -30.0)
    assert rel_err(expect(cfg, without, toks), want) > 0.02
    assert rel_err(stepwise(eng, "s", toks, 25), want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_recurrent_state_remembers_far_tokens(tmp_path, device):
    """The recurrence alone (the attention beside it switched off), with slow decays: the last rows still depend on the
    second token 280 positions back; a portion long enough for the chunk-parallel form, a short one, single tokens."""
    cfg = config([parallel(left_scale=0.0, right=ssd(heads=2, vdim=8, state=12, groups=1, norm_groups=2))], width=32,
                 vocab=50, taps=2)

    def edit(t):
        t["l0.mix.right.A_log"] = torch.tensor([-6.0, -4.5]).to(torch.bfloat16)

    eng, tensors = make(tmp_path, cfg, device, "float32", max_tokens=320, edit=edit)
    toks = tokens(300, 50, 14)
    want = expect(cfg, tensors, toks)
    other = expect(cfg, tensors, [toks[0], (toks[1] + 1) % 50] + toks[2:])
    assert rel_err(other[-3:], want[-3:]) > 0.003
    got = torch.cat([eng.replay_step([("l", toks[:270], list(range(270)))]),
                     eng.replay_step([("l", toks[270:285], list(range(15)))]), stepwise(eng, "l", toks[285:], 0)])
    assert rel_err(got, want) < TOL["float32"]


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
    # head sizes above one wave, more heads than one matrix tile's columns, state wider than two waves, long taps
    config([latent(heads=20, dim=72, rot_dim=40, vdim=80, kv_rank=96, q_rank=50, scale=0.1, ff=30),
            parallel(left=capped(heads=6, kv_heads=3, dim=80, vdim=72, scale=0.1, softcap=8.0),
                     right=ssd(heads=3, vdim=200, state=40, groups=1, norm_groups=5, conv=6)),
            parallel(left=capped(heads=20, kv_heads=2, dim=72, vdim=24, scale=0.11),
                     right=ssd(heads=4, vdim=24, state=144, groups=2, norm_groups=1, conv=2), ff=20)],
           width=40, vocab=77, eps=1e-6, taps=7),
    # odd sizes everywhere
    config([latent(heads=5, dim=7, rot_dim=6, vdim=9, kv_rank=11, q_rank=13, scale=0.6, base=100.0, ff=13),
            parallel(left=capped(heads=3, kv_heads=1, dim=10, vdim=3), right=ssd(heads=3, vdim=5, state=13, groups=3,
                                                                               norm_groups=5, conv=3), ff=7),
            latent(heads=7, dim=3, rot_dim=2, vdim=5, kv_rank=9, q_rank=4, scale=0.3)], width=37, vocab=53, taps=2),
    # one of everything: one head, one group, one state channel, value size one, one tap
    config([latent(heads=1, dim=2, rot_dim=2, vdim=1, kv_rank=1, q_rank=1, scale=1.0, ff=1),
            parallel(left=capped(heads=1, kv_heads=1, dim=2, vdim=1), right=ssd(heads=1, vdim=1, state=1, groups=1,
                                                                              norm_groups=1, conv=1))],
           width=8, vocab=11, taps=1),
    # aligned sizes (rows of 16 bytes in bfloat16), mixers of different widths in one model
    config([latent(heads=8, dim=32, rot_dim=16, vdim=32, kv_rank=64, q_rank=48, scale=0.15, ff=64),
            latent(heads=17, dim=16, rot_dim=8, vdim=16, kv_rank=32, q_rank=32, scale=0.2),
            parallel(left=capped(heads=8, kv_heads=2, dim=32, vdim=16, scale=0.18, softcap=15.0),
                     right=ssd(heads=4, vdim=32, state=64, groups=2, norm_groups=2), ff=32),
            parallel(left=capped(heads=4, kv_heads=4, dim=64, vdim=32, scale=0.125, softcap=50.0),
                     right=ssd(heads=8, vdim=16, state=16, groups=8, norm_groups=4, conv=3))], width=64, vocab=80),
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
    then 70 tokens one by one, across many pages."""
    cfg = OTHER_SIZES[3]
    eng, tensors = make(tmp_path, cfg, device, "bfloat16", max_tokens=256)
    toks = tokens(190, 80, 12)
    want = expect(cfg, tensors, toks)
    rows = [eng.replay_step([("m", toks[:90], list(range(90)))]), eng.replay_step([("m", toks[90:120], list(range(30)))])]
    rows += [eng.replay_step([("m", [t], [0])]) for t in toks[120:]]
    assert close(torch.cat(rows), want, "bfloat16")


@pytest.mark.parametrize("device", DEVICES)
def test_a_second_norm_without_feed_forward(tmp_path, device):
    """A checkpoint that holds a second norm for a layer without a feed-forward: the norm still applies."""
    cfg = config([latent(), parallel()])

    def edit(t):
        t["l0.norm2"] = torch.tensor(0.7).to(torch.bfloat16)

    eng, tensors = make(tmp_path, cfg, device, "float32", edit=edit)
    toks = tokens(30, cfg["vocab"], 15)
    want = expect(cfg, tensors, toks)
    without = dict(tensors)
    without.pop("l0.norm2")
    assert rel_err(expect(cfg, without, toks), want) > 0.003
    assert rel_err(stepwise(eng, "n", toks, 20), want) < TOL["float32"]


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
    cfg = config([latent(ff=20), parallel(), latent()])
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
    """A random small model: 2-5 layers of either mixer in any order, with or without feed-forward, sizes that are and
    are not multiples of 8 / 16, any number of taps."""
    import random

    rng = random.Random(seed)
    aligned = rng.random() < 0.5
    pick = lambda xs: rng.choice(xs)
    width = pick([32, 64, 96]) if aligned else pick([24, 36, 52, 72])
    layers = []
    for _ in range(rng.randint(2, 5)):
        ff = pick([0, 16, 32]) if aligned else pick([0, 5, 12])
        if rng.random() < 0.5:
            rot = pick([8, 16]) if aligned else pick([2, 6, 10])
            layers.append(latent(ff=ff, heads=pick([1, 2, 5, 18]), dim=pick([8, 16, 24]) if aligned else pick([3, 10, 12]),
                                 rot_dim=rot, dims=pick([rot, rot, 2]), vdim=pick([16, 32]) if aligned else pick([5, 9]),
                                 kv_rank=pick([16, 48]) if aligned else pick([7, 20]),
                                 q_rank=pick([16, 24]) if aligned else pick([5, 30]), scale=pick([0.1, 0.25, 0.5]),
                                 base=pick([100.0, 10000.0, 1e6])))
        else:
            kv, g = pick([1, 2, 3]), pick([1, 2])
            heads = g * pick([1, 2, 3])
            vdim = pick([8, 32]) if aligned else pick([6, 21])
            layers.append(parallel(ff=ff, left=capped(heads=kv * pick([1, 2, 5]), kv_heads=kv,
                                                      dim=pick([8, 16, 32]) if aligned else pick([6, 10, 12]),
                                                      vdim=pick([16, 32]) if aligned else pick([5, 9]),
                                                      scale=pick([0.1, 0.25, 0.5]), softcap=pick([2.0, 30.0])),
                                   right=ssd(heads=heads, vdim=vdim, state=pick([8, 16, 64]) if aligned else pick([5, 12, 33]),
                                             groups=g, norm_groups=pick([1, heads, vdim]), conv=pick([1, 2, 3, 4])),
                                   left_scale=pick([0.5, 1.0, 1.2]), right_scale=pick([0.4, 1.0])))
    return config(layers, width=width, vocab=pick([40, 64, 101]), eps=pick([1e-6, 1e-5]), alpha=pick([1.0, 2.0, 3.0]),
                  taps=pick([0, 1, 2, 3, 4]), scale=pick([1.0, 6.0]))


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


def mid_config(seed):
    """A random model of a few hundred channels: up to 24 heads, latent ranks up to 160, recurrent states up to 128
    channels, feed-forwards of one to two widths -- the sizes at which the matrix-core kernels and the tuned products
    take over."""
    import random

    rng = random.Random(seed)
    pick = lambda xs: rng.choice(xs)
    width = pick([128, 192, 256, 320, 384])
    layers = []
    for _ in range(rng.randint(2, 4)):
        ff = pick([0, width, 2 * width, 3 * width // 2])
        if rng.random() < 0.55:
            layers.append(latent(ff=ff, heads=pick([2, 4, 6, 12, 16, 24]), dim=pick([16, 32, 48, 96]),
                                 rot_dim=pick([8, 16, 64]), vdim=pick([16, 32, 64, 128]),
                                 kv_rank=pick([32, 48, 96, 128, 160]), q_rank=pick([48, 64, 192]),
                                 scale=pick([0.08, 0.1, 0.15]), base=pick([1e4, 1e6, 5e5])))
        else:
            kv, g = pick([1, 2, 4]), pick([1, 2, 4])
            heads = g * pick([1, 2, 4])
            layers.append(parallel(ff=ff, left=capped(heads=kv * pick([1, 2, 4]), kv_heads=kv, dim=pick([32, 64, 128]),
                                                      vdim=pick([32, 64, 128]), scale=pick([0.09, 0.125]),
                                                      softcap=pick([10.0, 50.0])),
                                   right=ssd(heads=heads, vdim=pick([16, 32, 48, 64]), state=pick([16, 32, 64, 128]),
                                             groups=g, norm_groups=pick([1, 2, heads]), conv=pick([2, 3, 4])),
                                   left_scale=pick([0.8, 1.2]), right_scale=pick([0.7, 1.0])))
    return config(layers, width=width, vocab=pick([300, 512, 1000]), eps=1e-6, alpha=pick([1.7, 2.0, 2.5]),
                  taps=pick([2, 3, 5]), scale=width ** 0.5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(6))
def test_mid_size_configurations_on_the_kernels(tmp_path, dtype, seed):
    """A 290-token prompt (long enough for the chunk-parallel recurrence), a short portion, a second request beside
    decoded tokens.  bfloat16: nine rows in ten within the tolerance (single rows of random networks amplify rounding)."""
    cfg = mid_config(seed)
    eng, tensors = make(tmp_path, cfg, "cuda", dtype, seed=seed, max_tokens=448, slots=4)
    V = cfg["vocab"]
    a, b = tokens(320, V, 100 + seed), tokens(50, V, 200 + seed)
    wa, wb = expect(cfg, tensors, a), expect(cfg, tensors, b)
    ga = [eng.replay_step([("a", a[:290], list(range(290)))]), eng.replay_step([("a", a[290:293], [0, 1, 2])])]
    gb = []
    for i in range(293, 320):
        if i == 300:
            rows = eng.replay_step([("a", [a[i]], [0]), ("b", b[:40], list(range(40)))])
            gb.append(rows[1:])
        elif 300 < i <= 310:
            rows = eng.replay_step([("a", [a[i]], [0]), ("b", [b[40 + i - 301]], [0])], ["b"] if i == 310 else [])
            gb.append(rows[1:])
        else:
            rows = eng.replay_step([("a", [a[i]], [0])])
        ga.append(rows[:1])
    for got, want in ((torch.cat(ga), wa), (torch.cat(gb), wb)):
        e = row_errs(got, want)
        if dtype == "float32":
            assert e.max().item() < TOL[dtype], cfg
        else:
            assert int((e >= TOL[dtype]).sum()) <= e.numel() // 10 and e.median().item() < 2e-2, cfg
