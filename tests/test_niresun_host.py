"""Niresun through the engine's host side (configuration, weights by name, state slots and pages, batching, scheduler,
sampling) on the CPU, with torch stand-ins for the kernels, against the plain implementation. The kernels themselves
are tested on the GPU (test_niresun_gpu.py)."""
import copy
import random

import pytest
import torch

from niresun_helpers import CONFIGS, make_model, make_weights, plain_logits, write_model
from takosun_helpers import rel_err, replay
from torch_ops import TorchOps

from lmsf_amd.config import ConfigError, resolve_architecture
from lmsf_amd.engine import EngineArgs, LLMEngine, StepEntry, load_engine_core
from lmsf_amd.sampling import SamplingParams
from lmsf_amd.weights.loader import WeightsError

TOL = 3e-5
SMALL = ("A", "B", "C")


def build(tmp_path, which, pages=24, block=8, seed=0, **kw):
    folder, cfg, w = make_model(tmp_path, which, seed)
    core = load_engine_core(folder, dtype="float32", block_size=block, num_pages=pages, max_model_len=pages * block,
                            device="cpu", ops=TorchOps(), max_num_seqs=kw.pop("slots", 4), **kw)
    return core, cfg, w


def tokens(n, vocab, seed):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def test_the_architecture_is_found_by_its_name():
    assert resolve_architecture({"architecture": "Niresun"}).name == "Niresun"


@pytest.mark.parametrize("which", SMALL)
def test_whole_prompt(tmp_path, which):
    core, cfg, w = build(tmp_path, which)
    toks = tokens(45, cfg["vocab"], 1)
    out = core.executor.step([StepEntry("a", toks, list(range(len(toks))))])
    assert rel_err(out, plain_logits(cfg, w, toks)) < TOL


@pytest.mark.parametrize("which", SMALL)
def test_portions_down_to_two_tokens_then_one_by_one(tmp_path, which):
    core, cfg, w = build(tmp_path, which)
    toks = tokens(61, cfg["vocab"], 2)
    cuts = [3, 2, 8, 7, 2, 16, 9] + [1] * 14          # portions that end inside and on the edges of pages and chunks
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", c)] for c in cuts])["a"]
    assert rel_err(got, plain_logits(cfg, w, toks)) < TOL
    core.storage.manager.check_invariants()


@pytest.mark.parametrize("which", SMALL)
def test_token_by_token_from_the_first(tmp_path, which):
    core, cfg, w = build(tmp_path, which)
    toks = tokens(24, cfg["vocab"], 3)
    got = replay(core.executor, StepEntry, {"a": toks}, [[("a", 1)] for _ in toks])["a"]
    assert rel_err(got, plain_logits(cfg, w, toks)) < TOL


@pytest.mark.parametrize("which", SMALL)
def test_unequal_requests_together_with_pages_and_slots_used_again(tmp_path, which):
    core, cfg, w = build(tmp_path, which, pages=20, slots=3)     # 160 tokens of room, three state slots
    V = cfg["vocab"]
    reqs = {"a": tokens(70, V, 4), "b": tokens(1, V, 5), "c": tokens(33, V, 6), "d": tokens(90, V, 7),
            "e": tokens(5, V, 8)}
    steps = [[("a", 30), ("b", 1), ("c", 2)], [("a", 1), ("c", 17), ("e", 2)], [("c", 14), ("a", 38)], [("a", 1), ("e", 3)],
             [("d", 50)], [("d", 39)], [("d", 1)]]
    got = replay(core.executor, StepEntry, reqs, steps)
    for k, t in reqs.items():
        assert rel_err(got[k], plain_logits(cfg, w, t)) < TOL, k
    core.storage.manager.check_invariants()
    assert core.storage.manager.num_free_pages(0) == 20 and core.storage.manager.num_free_state_slots() == 3


def test_a_request_takes_a_slot_that_another_has_left(tmp_path):
    core, cfg, w = build(tmp_path, "A", slots=1)
    V = cfg["vocab"]
    for name, n in (("first", 30), ("second", 19)):                 # the second finds the first one's state cleared
        toks = tokens(n, V, n)
        got = replay(core.executor, StepEntry, {name: toks}, [[(name, n - 4)]] + [[(name, 1)]] * 4)[name]
        assert rel_err(got, plain_logits(cfg, w, toks)) < TOL, name


def test_greedy_generation_through_the_engine(tmp_path):
    folder, cfg, w = make_model(tmp_path, "A", seed=3)
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
            seq.append(int(plain_logits(cfg, w, seq)[-1].argmax()))
        assert done[i].outputs[0].token_ids == seq[len(p):], i


def test_a_wrong_configuration_is_refused_by_key():
    def parse(c):
        return resolve_architecture(c).config_class.from_dict(c)

    bad = copy.deepcopy(CONFIGS["A"])
    bad["layers"][0]["type"] = "mamba7"
    with pytest.raises(ConfigError, match="mamba7"):
        parse(bad)
    bad = copy.deepcopy(CONFIGS["A"])
    del bad["layers"][0]["mixer"]["dt_rank"]
    with pytest.raises(ConfigError, match="dt_rank"):
        parse(bad)
    bad = copy.deepcopy(CONFIGS["A"])
    bad["layers"][1]["mixer"]["kv_heads"] = 3
    with pytest.raises(ConfigError, match="kv_heads"):
        parse(bad)
    bad = copy.deepcopy(CONFIGS["A"])
    bad["layers"][1]["mixer"]["rot"]["dims"] = 7
    with pytest.raises(ConfigError, match="dims"):
        parse(bad)
    bad = copy.deepcopy(CONFIGS["A"])
    del bad["layers"][2]["mixer"]["right"]["gate_cap"]
    with pytest.raises(ConfigError, match="gate_cap"):
        parse(bad)
    bad = copy.deepcopy(CONFIGS["A"])
    bad["layers"][3]["mlp"]["kind"] = "sparse"
    with pytest.raises(ConfigError, match="sparse"):
        parse(bad)


def test_missing_and_misshapen_tensors_are_listed(tmp_path):
    cfg = CONFIGS["C"]
    w = make_weights(cfg, 0)
    del w["l1.mix.A_log"]
    w["l0.mix.q.b"] = w["l0.mix.q.b"][:10]
    folder = write_model(str(tmp_path / "broken"), cfg, w)
    with pytest.raises(WeightsError) as e:
        load_engine_core(folder, dtype="float32", block_size=8, num_pages=4, device="cpu", ops=TorchOps())
    assert "l1.mix.A_log" in e.value.missing and any(n == "l0.mix.q.b" for n, _, _ in e.value.wrong_shape)
