"""Takosun through the engine's host side (configuration, weights by name, schedule with borrowed caches, cache
manager, batching, scheduler, sampling) on the CPU, with torch stand-ins for the kernels, against the plain
implementation. The kernels themselves are tested on the GPU (test_takosun_gpu.py)."""
import copy
import random

import pytest
import torch

from plain_takosun import t_forward
from takosun_helpers import CONFIGS, make_model, plain_logits, rel_err, replay
from torch_ops import TorchOps

from lmsf_amd.config import ConfigError, resolve_architecture
from lmsf_amd.engine import EngineArgs, LLMEngine, StepEntry, load_engine_core
from lmsf_amd.sampling import SamplingParams
from lmsf_amd.weights.loader import WeightsError

TOL = 2e-5


def build(tmp_path, which, pages=24, block=8, seed=0, **kw):
    folder, cfg, w = make_model(tmp_path, which, seed)
    core = load_engine_core(folder, dtype="float32", block_size=block, num_pages=pages, max_model_len=pages * block,
                            device="cpu", ops=TorchOps(), max_num_seqs=4, **kw)
    return core, cfg, w


def tokens(n, vocab, seed):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def test_the_architecture_is_found_by_its_name():
    assert resolve_architecture({"architecture": "Takosun"}).name == "Takosun"


@pytest.mark.parametrize("which", sorted(k for k in CONFIGS if k != "M"))   # (M: sizes for the GPU kernels)
def test_whole_prompt(tmp_path, which):
    core, cfg, w = build(tmp_path, which)
    toks = tokens(45, cfg["vocab"], 1)
    out = core.executor.step([StepEntry("a", toks, list(range(len(toks))))])
    assert rel_err(out, plain_logits(cfg, w, toks)) < TOL


@pytest.mark.parametrize("which", sorted(k for k in CONFIGS if k != "M"))   # (M: sizes for the GPU kernels)
def test_portions_down_to_two_tokens_then_one_by_one(tmp_path, which):
    core, cfg, w = build(tmp_path, which)
    toks = tokens(61, cfg["vocab"], 2)
    cuts = [3, 2, 8, 7, 2, 16, 9] + [1] * 14          # portions that end inside and on the edges of pages of 8
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", c)] for c in cuts])["a"]
    assert rel_err(got, plain_logits(cfg, w, toks)) < TOL
    core.storage.manager.check_invariants()


@pytest.mark.parametrize("which", sorted(k for k in CONFIGS if k != "M"))   # (M: sizes for the GPU kernels)
def test_token_by_token_from_the_first(tmp_path, which):
    core, cfg, w = build(tmp_path, which)
    toks = tokens(20, cfg["vocab"], 3)
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", 1)] for _ in toks])["a"]
    assert rel_err(got, plain_logits(cfg, w, toks)) < TOL


@pytest.mark.parametrize("which", sorted(k for k in CONFIGS if k != "M"))   # (M: sizes for the GPU kernels)
def test_unequal_requests_together_with_pages_used_again(tmp_path, which):
    core, cfg, w = build(tmp_path, which, pages=20)     # 160 tokens of room: the third request needs pages given back
    V = cfg["vocab"]
    reqs = {"a": tokens(70, V, 4), "b": tokens(1, V, 5), "c": tokens(33, V, 6), "d": tokens(90, V, 7)}
    steps = [[("a", 30), ("b", 1), ("c", 2)], [("a", 1), ("c", 17)], [("c", 14), ("a", 38)], [("a", 1)],
             [("d", 50)], [("d", 39)], [("d", 1)]]
    got = replay(core.executor, StepEntry, reqs, steps)
    for k, t in reqs.items():
        assert rel_err(got[k], plain_logits(cfg, w, t)) < TOL, k
    core.storage.manager.check_invariants()
    assert core.storage.manager.num_free_pages(0) == 20


def test_greedy_generation_through_the_engine(tmp_path):
    folder, cfg, w = make_model(tmp_path, "P", seed=3)
    args = EngineArgs(model=folder, dtype="float32", block_size=8, device="cpu", num_gpu_blocks_override=40,
                      max_num_seqs=4, max_model_len=200, prefill_chunk_size=16, max_num_batched_tokens=24)
    engine = LLMEngine(args, ops=TorchOps())
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (1, 9, 40)]
    for i, p in enumerate(prompts):
        engine.add_request(i, p, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))
    done = {}
    while engine.has_unfinished_requests():
        for out in engine.step():
            if out.finished:
                done[out.request_id] = out
    for i, p in enumerate(prompts):
        seq = list(p)
        for _ in range(6):
            seq.append(int(t_forward(cfg, w, seq, dtype=torch.float64)[-1].argmax()))
        assert done[i].outputs[0].token_ids == seq[len(p):], i


def test_a_wrong_configuration_is_refused_by_key(tmp_path):
    bad = copy.deepcopy(CONFIGS["P"])
    bad["layers"][2]["mixer"]["kv_from"] = 2
    with pytest.raises(ConfigError, match="kv_from"):
        resolve_architecture(bad).config_class.from_dict(bad)
    bad = copy.deepcopy(CONFIGS["P"])
    bad["layers"][2]["mixer"]["kv_rank"] = 16            # not the size of the latent it reads
    with pytest.raises(ConfigError, match="differ"):
        resolve_architecture(bad).config_class.from_dict(bad)
    bad = copy.deepcopy(CONFIGS["P"])
    del bad["norm"]["groups"]
    with pytest.raises(ConfigError, match="groups"):
        resolve_architecture(bad).config_class.from_dict(bad)


def test_missing_and_misshapen_tensors_are_listed(tmp_path):
    from takosun_helpers import make_weights, write_model
    cfg = CONFIGS["R"]
    w = make_weights(cfg, 0)
    del w["l1.mix.uk"]
    w["l0.mlp.table"] = w["l0.mlp.table"][:10]
    folder = write_model(str(tmp_path / "broken"), cfg, w)
    with pytest.raises(WeightsError) as e:
        load_engine_core(folder, dtype="float32", block_size=8, num_pages=4, device="cpu", ops=TorchOps())
    assert "l1.mix.uk" in e.value.missing and any(n == "l0.mlp.table" for n, _, _ in e.value.wrong_shape)
