"""Niresun configurations drawn at random (layers of every kind in any order and number; head sizes, widths, states,
ranks, taps, chunks and page sizes that are no powers of two and no multiples of what the kernels' tiles like) through
the engine, whole, in portions and mixed, in float32 and in bfloat16, against the plain implementation."""
import random

import pytest
import torch

from helpers import random_tokens, replay_in_process, trace_bulk_then_single, trace_mixed, trace_portions, trace_whole
from niresun_helpers import SCALING, attn, dense, make_model, mamba, pair, plain_logits
from test_niresun_gpu import check

pytestmark = pytest.mark.gpu


def draw_config(seed):
    rng = random.Random(seed)
    pick = rng.choice

    def mlp():
        return dense(pick([24, 100, 172, 256])) if rng.random() < 0.6 else None

    def layer():
        kind = pick(["mamba1", "attention", "parallel"])
        if kind == "mamba1":
            return mamba(pick([24, 50, 96, 130]), pick([1, 3, 16, 17, 33, 64]), pick([1, 7, 16]), pick([1, 2, 3, 4, 6]), mlp())
        kv = pick([1, 2, 3])
        heads = kv * pick([1, 2, 4])
        dim = pick([8, 12, 20, 24, 40, 64, 72])
        if kind == "attention":
            rot = pick([0, 2, dim // 2 // 2 * 2, dim // 2 * 2])
            return attn(heads, kv, dim, pick([8, 12, 24, 40, 80]), pick([None, 5, 16, 37, 64, 130]), rot,
                        base=pick([100.0, 10000.0, 1e6]), scaling=pick([None, SCALING]) if rot else None,
                        scale=pick([None, 0.2]), mlp=mlp())
        return pair(heads, kv, dim, pick([8, 20, 24, 48]), pick([1, 2, 3, 5]), pick([None, (0.6, 7), (2.0, 50)]),
                    pick([1, 2, 3]), pick([8, 20, 48]), pick([8, 12, 40, 80]), pick([2.0, 14.0, 50.0]), mlp=mlp())

    cfg = {"architecture": "Niresun", "vocab": pick([41, 97, 256, 331]), "width": pick([40, 72, 100, 136, 256]),
           "norm": {"eps": pick([1e-5, 1e-6])}, "layers": [layer() for _ in range(pick([2, 3, 4, 5]))]}
    return cfg, pick([4, 8, 16, 32]), [pick([1, 2, 5, 17, 40, 77, 130, 200, 300]) for _ in range(5)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10])
def test_a_configuration_drawn_at_random(tmp_path, seed, dtype):
    from lmsf_amd.engine import load_engine_core
    cfg, page, lens = draw_config(seed)
    folder, cfg, w = make_model(tmp_path, cfg, seed)
    reqs = {"r%d" % i: random_tokens(n, cfg["vocab"], 50 + i) for i, n in enumerate(lens)}
    refs = {rid: plain_logits(cfg, w, toks) for rid, toks in reqs.items()}
    alone = -(-max(lens) // page) + 1
    for what, steps, pages in (("whole", trace_whole(reqs), alone),
                               ("bulk then single", trace_bulk_then_single(reqs, tail=8), alone),
                               ("portions", trace_portions(reqs, seed=seed), alone),
                               ("mixed", trace_mixed(reqs, 512, seed=seed), 512 // page)):
        core = load_engine_core(folder, dtype=dtype, block_size=page, num_pages=pages, max_model_len=pages * page,
                                max_num_seqs=4)
        got = replay_in_process(core.executor, steps)
        for rid in reqs:
            assert torch.isfinite(got[rid]).all(), (what, rid, cfg)
            check(got[rid], refs[rid], dtype, (what, rid, cfg, page), (cfg, w, reqs[rid]))
        core.storage.manager.check_invariants()
        assert core.storage.manager.num_free_state_slots() == 4
        del core
