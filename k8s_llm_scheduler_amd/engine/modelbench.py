"""Prefill and decode throughput of the registered model designs at equal layer sizes (``bench.py --model-bench``).

For every size a Putulorn (dense feed-forwards), a Putulorn with experts, a Rupatar (experts in every layer), a Nukizen
(dense feed-forward beside every mixer), a Semanex (dense feed-forward after every mixer) and a Llama of the same width, depth, feed-forward / expert size and vocabulary are built with random weights and driven through the
same engine entry points:

* prefill: one whole prompt of ``T`` tokens in one step (``LLMEngine.replay_step``, the varlen forward), tokens/s;
* decode: ``B`` requests generated together (``LLMEngine.generate``: captured decode graphs), new tokens/s from the
  engine's GPU-event decode time.
"""

from __future__ import annotations

import time
from typing import Dict, List

SIZES = {
    # width: (layer pairs, ff, wkv head dim, latent heads, expert ff, experts)
    2048: (4, 8192, 64, 16, 2048, 8),
    4096: (2, 14336, 64, 32, 3584, 8),
}
VOCAB = 32768


def _register(width: int) -> Dict[str, str]:
    from ..models import nukizen, putulorn, rupatar, semanex
    from ..models.config import PRESETS, LlamaConfig

    pairs, ff, wd, heads, eff, experts = SIZES[width]
    names = {"putulorn-dense": f"putulorn-w{width}-dense", "putulorn-moe": f"putulorn-w{width}-moe",
             "rupatar": f"rupatar-w{width}", "nukizen": f"nukizen-w{width}", "semanex": f"semanex-w{width}",
             "llama": f"llama-w{width}"}
    # Semanex: 2 x pairs layers in the order latent, latent, parallel (capped attention + state-space recurrence),
    # latent; latent attention shaped like Putulorn's (rank 512 + 64 rotated, 128-wide heads) with a query latent of
    # 3 / 4 of the width, the side attention like Rupatar's (4 query heads per key head, 128-wide), recurrent heads of
    # 128 state channels x 64 values filling the width, the feed-forward size of the Putulorn-dense layers
    semanex.PRESETS[names["semanex"]] = semanex.preset(
        names["semanex"], width, VOCAB, max(1, pairs // 2), heads=heads, dim=128, rot_dim=64, vdim=128, kv_rank=512,
        q_rank=width * 3 // 4, side_heads=heads, side_kv_heads=heads // 4, side_dim=128, side_vdim=128,
        ssd_heads=width // wd, ssd_vdim=wd, ssd_state=128, ssd_groups=max(1, width // wd // 8), norm_groups=4, ff=ff)
    # Nukizen: 2 x pairs layers in the order attention, parallel (attention + delta rule), rglru, attention on the first
    # layer's cache; attention shaped like Rupatar's (4 query heads per key head, 128-wide, chunks of 1024), delta-rule
    # heads of 64 x 64 like the wkv heads, a recurrent unit 5 / 4 of the width in 10 blocks, the dense feed-forward of
    # the Putulorn-dense layers beside every mixer
    nukizen.PRESETS[names["nukizen"]] = nukizen.preset(
        names["nukizen"], width, VOCAB, max(1, pairs // 2), heads=heads, kv_heads=heads // 4, dim=128, vdim=128,
        chunk=1024, rot_dims=64, side_heads=heads, side_kv_heads=heads // 4, side_dim=128, side_chunk=1024,
        delta_heads=width // wd, delta_kv_heads=width // wd // 2, delta_dim=wd, delta_vdim=wd, lru_width=width * 5 // 4,
        lru_blocks=10, ff=ff, order=("attention", "parallel", "rglru", "shared"))
    # Rupatar: 2 x pairs layers in the order attention, hgrn2, attention, mlstm (windowed attention with 4 query heads
    # per key head, window 1024, pooled blocks of 16; recurrences of head size 64 x 64 like the wkv heads), every layer
    # with the experts of the Putulorn-moe layers and a shared expert of the same size
    rupatar.PRESETS[names["rupatar"]] = rupatar.preset(
        names["rupatar"], width, VOCAB, max(1, pairs // 2), heads=heads, kv_heads=heads // 4, dim=128, vdim=128,
        window=1024, pool=16, rot_dims=64, scan_heads=width // wd, scan_dim=wd, scan_vdim=wd, experts=experts, top=2,
        expert_ff=eff, shared_ff=eff)
    kw = dict(heads=heads, wkv_dim=wd, dim=128, rot_dim=64, vdim=128, kv_rank=512, window=1024, ff=ff)
    putulorn.PRESETS[names["putulorn-dense"]] = putulorn.preset(names["putulorn-dense"], width, VOCAB, pairs, **kw)
    putulorn.PRESETS[names["putulorn-moe"]] = putulorn.preset(names["putulorn-moe"], width, VOCAB, pairs, experts=experts,
                                                            top=2, expert_ff=eff, **kw)
    PRESETS[names["llama"]] = LlamaConfig(names["llama"], 2 * pairs, width, width // 128, max(1, width // 512), 128, ff,
                                          VOCAB, bos_id=VOCAB - 256, eos_ids=(VOCAB - 255,), max_position=8192)
    return names


def run(widths=(2048, 4096), prefill_tokens=(512, 2048), decode_batches=(1, 8, 32), context: int = 512,
        new_tokens: int = 32, repeats: int = 3, progress=print, models=None) -> List[dict]:
    import torch

    from . import build_engine
    from .sampling import SamplingParams

    rows = []
    for width in widths:
        for kind, name in _register(width).items():
            if models and kind not in models:
                continue
            maxb = max(decode_batches)
            mml = max(max(prefill_tokens), context + new_tokens + 16)
            eng = build_engine(name, max_batch=maxb, block_size=16, num_blocks=maxb * (mml // 16 + 1),
                               max_model_len=mml, prefix_caching=False, max_prefill_tokens=max(prefill_tokens))
            row = {"model": kind, "width": width, "layers": eng.model.cfg.num_layers,
                   "weight_gb": round(eng.model.weight_bytes() / 1e9, 2)}
            g = torch.Generator().manual_seed(0)
            for T in prefill_tokens:
                toks = torch.randint(0, VOCAB - 512, (T,), generator=g).tolist()
                best = 1e9
                for i in range(repeats + 1):
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    eng.replay_step([("p", toks, [T - 1])], ["p"])
                    torch.cuda.synchronize()
                    if i:
                        best = min(best, time.perf_counter() - t0)
                row[f"prefill_tok_s@{T}"] = round(T / best)
            sp = SamplingParams(max_tokens=new_tokens, temperature=0.0, ignore_eos=True, stop_on_json_close=False)
            for B in decode_batches:
                prompts = [torch.randint(0, VOCAB - 512, (context,), generator=g).tolist() for _ in range(B)]
                best = 0.0
                for i in range(2):
                    eng.stats["decode_time"], eng.stats["decode_tokens"] = 0.0, 0
                    eng.generate(prompts, sp)
                    best = max(best, eng.stats["decode_tokens"] / max(eng.stats["decode_time"], 1e-9))
                row[f"decode_tok_s@B{B}"] = round(best)
            progress(row)
            rows.append(row)
            del eng
            torch.cuda.empty_cache()
    return rows
