"""Takosun on the GPU: every new kernel alone against the plain implementation's function of the same mechanism,
then the model through the engine's step function in float32 and bfloat16 under the four ways of cutting a
request into steps, with a far key that matters, long decoding from graphs, and generation through the entry
point."""
import math
import random

import pytest
import torch

from plain_takosun import (t_depth_average, t_forward, t_gated_ff, t_group_rms_norm, t_rms_norm, t_rotate,
                           t_table_moe)
from takosun_helpers import (CONFIGS, bfloat16_limits, make_model, plain_logits, rel_err, replay, row_err, row_errs,
                             within)

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
TOL_F32 = 3e-5


def check(got, ref, dtype, cfg, w, toks, what=""):
    """float32: the largest difference of any logit, relative to the logits' spread. bfloat16: every position
    within what rounding may cost there (rounding has outliers at positions whose logits hang on small
    differences; a fault moves rows that rounding leaves alone)."""
    if dtype == "float32":
        assert rel_err(got, ref) < TOL_F32, what
    else:
        ok, worst = within(got, ref, bfloat16_limits(cfg, w, toks, ref))
        assert ok, (what, worst)
        # and over all positions no worse than the plain implementation rounded to bfloat16 throughout
        everywhere = t_forward(cfg, w, toks, dtype=torch.bfloat16)
        assert float(row_errs(got, ref).pow(2).mean()) <= float(row_errs(everywhere, ref).pow(2).mean()), what


def ops():
    from lmsf_amd.ops import get_ops
    return get_ops()


def close(got, ref, dtype, scale=1.0):
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    err = float((got.double().cpu() - ref.double().cpu()).abs().max())
    assert err <= tol * scale * max(1.0, float(ref.abs().max())), err


def rotary_table(max_pos, rot, base):
    i = torch.arange(rot // 2, dtype=torch.float64)
    freq = (float(base) ** (-2.0 * i / rot)).to(torch.float32)
    ang = torch.arange(max_pos, dtype=torch.float32)[:, None] * freq[None, :]
    return torch.cat([torch.cos(ang), torch.sin(ang)], dim=1).contiguous()


# --------------------------------------------------------------------------- kernels alone


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W,groups", [(64, 1), (120, 4), (96, 3), (4096, 2), (10, 10)])
def test_group_norm_in_every_arrangement(dtype, W, groups):
    o = ops()
    g = torch.Generator().manual_seed(W + groups)
    N, L = 7, 4
    x = (torch.randn((N, W + 8), generator=g) * 3).to(dtype)
    res = torch.randn((N, W), generator=g)
    wa, wb = 1 + 0.3 * torch.randn(W, generator=g), 1 + 0.3 * torch.randn(W, generator=g)
    hist = torch.randn((L, N, W), generator=g)
    mix = torch.rand(L, generator=g)
    xv = x.cuda()[:, 3:3 + W] if dtype == torch.float32 else x.cuda()[:, 8:8 + W]     # a view into wider rows
    xr = xv.cpu().float()
    # the norm of the stream, at chosen rows
    rows = torch.tensor([5, 0, 5], dtype=torch.int32)
    got = o.group_norm(residual=res.cuda(), out_weight=wa.cuda(), groups=groups, out_eps=1e-5, out_dtype=dtype,
                       rows=rows.cuda())
    close(got, t_group_rms_norm(res[rows.long()], wa, 1e-5, groups), dtype)
    # the norm of activations alone
    got = o.group_norm(x=xv, x_weight=wa.cuda(), groups=groups, x_eps=1e-3, out_dtype=dtype)
    close(got, t_group_rms_norm(xr, wa, 1e-3, groups), dtype)
    # stream += norm(branch), then the next norm of the sum
    r = res.clone().cuda()
    got = o.group_norm(x=xv, x_weight=wa.cuda(), residual=r, out_weight=wb.cuda(), groups=groups, x_eps=1e-5,
                       out_eps=1e-6, out_dtype=dtype)
    s = res + t_group_rms_norm(xr, wa, 1e-5, groups)
    close(r, s, torch.float32)
    close(got, t_group_rms_norm(s, wb, 1e-6, groups), dtype)
    # the same with the sum stored as result 2 and the stream replaced by the average of results 0..2
    r, h = res.clone().cuda(), hist.clone().cuda()
    assert o.group_norm(x=xv, x_weight=wa.cuda(), residual=r, groups=groups, history=h, index=2, mix=mix.cuda(),
                        want_out=False) is None
    close(h[2], s, torch.float32)
    close(h[3], hist[3], torch.float32, 0)
    close(r, t_depth_average([hist[0], hist[1], s], mix), torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,O,K,xh,oh", [(2, 32, 16, 24, 48), (5, 40, 24, 40, 56), (1, 300, 7, 7, 300), (3, 8, 513, 520, 8),
                                         (4, 40, 64, 96, 48), (3, 224, 32, 40, 256), (2, 70, 96, 96, 72)])
def test_per_head_products_with_and_without_gate(dtype, H, O, K, xh, oh):
    o = ops()
    g = torch.Generator().manual_seed(H * O + K)
    for N in (1, 8, 19, 70, 200):          # from 32 tokens on, bfloat16 products with K a multiple of 32 use the matrix cores
        x = torch.randn((N, H * xh + 4), generator=g).to(dtype)
        W = (torch.randn((H, O, K), generator=g) / math.sqrt(K)).to(dtype)
        gate = torch.randn((N, H + 3), generator=g).to(dtype)
        for use_gate in (False, True):
            out = torch.full((N, H * oh), 7.0, dtype=dtype).cuda()
            o.head_linear(x.cuda()[:, 4:] if dtype == torch.float32 else x.cuda(), xh, W.cuda(), out, oh,
                          gate=gate.cuda()[:, 1:1 + H] if use_gate else None)
            xs = (x[:, 4:] if dtype == torch.float32 else x).float()
            for h in range(H):
                ref = xs[:, h * xh:h * xh + K] @ W[h].float().t()
                if use_gate:
                    ref = ref * torch.sigmoid(gate[:, 1 + h:2 + h].float())
                close(out[:, h * oh:h * oh + O], ref, dtype, 2.0)
                assert (out[:, h * oh + O:(h + 1) * oh] == 7.0).all()      # nothing written beside a head's outputs


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("R,dr,rot,D,ps", [(32, 8, 8, 48, 8), (40, 16, 16, 64, 16), (12, 4, 4, 16, 4), (24, 32, 16, 64, 32)])
def test_latent_rows_and_rotated_query_parts(dtype, R, dr, rot, D, ps):
    o = ops()
    g = torch.Generator().manual_seed(R + dr)
    N, pages, base = 11, 6, 777.0
    table = rotary_table(64, rot, base)
    x = torch.randn((N, R + dr + 5), generator=g).to(dtype)
    w = 1 + 0.3 * torch.randn(R, generator=g)
    pos = torch.tensor([0, 1, 7, 8, 9, 31, 32, 33, 63, 5, 2], dtype=torch.int32)
    slots = torch.tensor([0, 1, ps - 1, ps, 3 * ps + 1, -1, 5 * ps + ps - 1, 2 * ps, 4 * ps, -1, 2], dtype=torch.int32)
    k = torch.full((pages, 1, ps, D), 9.0, dtype=dtype).cuda()
    v = torch.full((pages, 1, D, ps), 9.0, dtype=dtype).cuda()
    o.latent_cache_write(x.cuda(), w.cuda(), 1e-5, R, dr, pos.cuda(), table.cuda(), slots.cuda(), k, v)
    c = t_rms_norm(x[:, :R].float(), w, 1e-5)
    r = t_rotate(x[:, R:R + dr].float(), pos, base, rot)
    kk, vv = k.float().cpu().reshape(pages * ps, D), v.float().cpu().permute(0, 1, 3, 2).reshape(pages * ps, D)
    written = set()
    for n in range(N):
        s = int(slots[n])
        if s < 0:
            continue
        written.add(s)
        for page in (kk, vv):
            close(page[s, :R], c[n], dtype)
            close(page[s, R:R + dr], r[n], dtype)
            assert (page[s, R + dr:] == 0).all()
    untouched = [s for s in range(pages * ps) if s not in written]
    assert (kk[untouched] == 9.0).all() and (vv[untouched] == 9.0).all()
    # the rotated part of every head's query, into a wider row, with the rest behind it zeroed
    H, dn = 3, 10
    q = torch.randn((N, H * (dn + dr)), generator=g).to(dtype)
    qa = torch.full((N, H * D), 5.0, dtype=dtype).cuda()
    o.rope_tail(q.cuda(), dn + dr, dn, qa, D, R, H, dr, pos.cuda(), table.cuda())
    qf = q.float().reshape(N, H, dn + dr)
    ref = t_rotate(qf[..., dn:], pos, base, rot)
    got = qa.float().cpu().reshape(N, H, D)
    close(got[..., R:R + dr], ref, dtype)
    assert (got[..., :R] == 5.0).all() and (got[..., R + dr:] == 0).all()
    # the same from the launch of the per-head products, which fill the columns before it
    for n_tok in (N, 3):
        Wk = (torch.randn((H, R, dn), generator=g) / math.sqrt(dn)).to(dtype)
        qa = torch.full((n_tok, H * D), 5.0, dtype=dtype).cuda()
        o.head_linear(q[:n_tok].cuda(), dn + dr, Wk.cuda(), qa, D, rope_tail=(dn, R, dr, pos[:n_tok].cuda(), table.cuda()))
        got = qa.float().cpu().reshape(n_tok, H, D)
        close(got[..., R:R + dr], ref[:n_tok], dtype)
        close(got[..., :R], torch.einsum("nhd,hrd->nhr", qf[:n_tok, :, :dn], Wk.float()), dtype, 2.0)
        assert (got[..., R + dr:] == 0).all()
    # the norm of another part of the same rows from the cache write's launch
    x2 = torch.randn((N, 7 + R + dr), generator=g).to(dtype)
    w2 = 1 + 0.3 * torch.randn(7, generator=g)
    got = o.latent_cache_write(x2.cuda()[:, 7:], w.cuda(), 1e-5, R, dr, pos.cuda(), table.cuda(), slots.cuda(), k, v,
                               also_norm=x2.cuda()[:, :7], also_weight=w2.cuda())
    close(got, t_rms_norm(x2[:, :7].float(), w2, 1e-5), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N", [13, 150, 333])      # few tokens stream the experts' rows; many are grouped by expert
@pytest.mark.parametrize("W,F,E,top,shared", [(64, 32, 3, 2, True), (120, 24, 5, 1, False), (32, 16, 6, 6, True),
                                              (256, 100, 4, 3, False), (128, 96, 7, 2, True), (96, 64, 70, 1, False)])
def test_experts_assigned_by_a_table(dtype, W, F, E, top, shared, N):
    o = ops()
    g = torch.Generator().manual_seed(W + F + E)
    V = 37
    w = {}
    for e in range(E):
        w["m.e%d.gate" % e] = (torch.randn((F, W), generator=g) / math.sqrt(W)).to(dtype).float()
        w["m.e%d.up" % e] = (torch.randn((F, W), generator=g) / math.sqrt(W)).to(dtype).float()
        w["m.e%d.down" % e] = (torch.randn((W, F), generator=g) / math.sqrt(F)).to(dtype).float()
    w["m.table"] = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(V)]).to(torch.int32)
    h = torch.randn((N, W), generator=g).to(dtype)
    ids = torch.randint(0, V, (N,), generator=g).to(torch.int32)
    base = torch.randn((N, W), generator=g).to(dtype) if shared else None
    gu = torch.stack([torch.cat([w["m.e%d.gate" % e], w["m.e%d.up" % e]]) for e in range(E)]).to(dtype).cuda()
    dn = torch.stack([w["m.e%d.down" % e] for e in range(E)]).to(dtype).cuda()
    got = o.table_moe(h.cuda(), gu, dn, ids.cuda(), w["m.table"].cuda(), 1.0 / top, base=base.cuda() if shared else None)
    ref = t_table_moe(h.float(), ids, w, "m", {"router": {"top": top}})
    if shared:
        ref = ref + base.float()
    close(got, ref, dtype, 2.0)


# --------------------------------------------------------------------------- the model through the step function


def build(tmp_path, which, dtype, pages=48, block=16, seed=0, spread=1.0, eager=False):
    from lmsf_amd.engine import load_engine_core
    folder, cfg, w = make_model(tmp_path, which, seed, spread)
    core = load_engine_core(folder, dtype=dtype, block_size=block, num_pages=pages, max_model_len=pages * block,
                            max_num_seqs=4, enforce_eager=eager)
    return core, cfg, w


def tokens(n, vocab, seed):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", sorted(k for k in CONFIGS if k != "M"))
def test_four_ways_of_cutting_give_the_plain_logits(tmp_path, which, dtype):
    from lmsf_amd.engine import StepEntry
    core, cfg, w = build(tmp_path, which, dtype)
    V = cfg["vocab"]
    ex = core.executor
    a, b, c, d = tokens(150, V, 1), tokens(1, V, 2), tokens(67, V, 3), tokens(200, V, 4)
    ref = {k: plain_logits(cfg, w, t) for k, t in (("a", a), ("b", b), ("c", c), ("d", d))}
    # whole
    for k, t in (("a", a), ("b", b)):
        check(replay(ex, StepEntry, {k: t}, [[(k, len(t))]])[k], ref[k], dtype, cfg, w, t, (k, "whole"))
    # most of it at once, the last 40 one by one (over two page borders)
    got = replay(ex, StepEntry, {"a": a}, [[("a", 110)]] + [[("a", 1)]] * 40)["a"]
    check(got, ref["a"], dtype, cfg, w, a, "decode")
    # portions of changing size, some of two tokens, ending on and beside page borders
    cuts = [15, 1, 2, 30, 16, 2, 33, 17, 19] + [1] * 15
    assert sum(cuts) == 150
    got = replay(ex, StepEntry, {"a": a}, [[("a", n)] for n in cuts])["a"]
    check(got, ref["a"], dtype, cfg, w, a, "portions")
    # unequal requests together; d starts in pages that a and c have given back
    steps = [[("a", 64), ("b", 1), ("c", 3)], [("c", 2), ("a", 1)], [("a", 85), ("c", 61)], [("c", 1)],
             [("d", 2)], [("d", 197)], [("d", 1)]]
    got = replay(ex, StepEntry, {"a": a, "b": b, "c": c, "d": d}, steps)
    for k, t in (("a", a), ("b", b), ("c", c), ("d", d)):
        check(got[k], ref[k], dtype, cfg, w, t, (k, "mixed"))
    core.storage.manager.check_invariants()
    assert core.storage.manager.num_free_pages(0) == 48


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_at_which_the_matrix_core_forms_run(tmp_path, dtype):
    """Width 1,024: per-head products and grouped experts on the matrix cores, the 17-and-more-rows and many-rows
    products, attention over a cached row of 256 entries; a prompt in two portions, a second request beside it, then
    single tokens of both."""
    from lmsf_amd.engine import StepEntry
    core, cfg, w = build(tmp_path, "M", dtype, pages=40)
    V = cfg["vocab"]
    a, b = tokens(330, V, 21), tokens(70, V, 22)
    steps = [[("a", 280)], [("a", 40), ("b", 60)]] + [[("a", 1), ("b", 1)]] * 10
    got = replay(core.executor, StepEntry, {"a": a, "b": b}, steps)
    for k, t in (("a", a), ("b", b)):
        check(got[k], plain_logits(cfg, w, t), dtype, cfg, w, t, k)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_that_decides_the_logits(tmp_path, dtype):
    """Peaked attention (wide query and key up-projections): changing one token far back changes the last logits
    by much more than the tolerance, in a prompt portion and in decoding alike, so a lost or misplaced key shows."""
    from lmsf_amd.engine import StepEntry
    core, cfg, w = build(tmp_path, "P", dtype, spread=2.5)
    V = cfg["vocab"]
    t = tokens(330, V, 9)
    ref = plain_logits(cfg, w, t)
    limits = bfloat16_limits(cfg, w, t, ref) if dtype == "bfloat16" else torch.full((len(t),), TOL_F32)
    for j in (16, 100):          # a page's first slot, and a key far inside
        moved = row_errs(plain_logits(cfg, w, t[:j] + [(t[j] + 1) % V] + t[j + 1:]), ref)[-8:]
        assert (moved > 6 * limits[-8:]).any(), (j, moved / limits[-8:])      # twice what no position may reach
    ex = core.executor
    got = replay(ex, StepEntry, {"a": t}, [[("a", 300)], [("a", 22)]] + [[("a", 1)]] * 8)["a"]
    check(got, ref, dtype, cfg, w, t)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_graphs_equals_eager(tmp_path, dtype):
    from lmsf_amd.engine import StepEntry
    outs = []
    for eager in (False, True):
        core, cfg, w = build(tmp_path, "Q", dtype, eager=eager)
        V = cfg["vocab"]
        a, b = tokens(200, V, 11), tokens(140, V, 12)
        steps = [[("a", 20), ("b", 3)]] + [[("a", 1), ("b", 1)]] * 137 + [[("a", 1)]] * 43
        outs.append(replay(core.executor, StepEntry, {"a": a, "b": b}, steps))
        assert core.executor.use_graphs == (not eager)
    ref = {"a": plain_logits(cfg, w, a), "b": plain_logits(cfg, w, b)}
    for k in ref:
        assert torch.equal(outs[0][k], outs[1][k]), k
        check(outs[0][k], ref[k], dtype, cfg, w, {"a": a, "b": b}[k], k)


def test_greedy_generation_through_the_entry_point(tmp_path):
    from lmsf_amd.engine import LLM
    from lmsf_amd.sampling import SamplingParams
    folder, cfg, w = make_model(tmp_path, "R", seed=5)
    llm = LLM(folder, dtype="float32", block_size=8, num_gpu_blocks_override=64, max_num_seqs=4, max_model_len=256,
              prefill_chunk_size=16, max_num_batched_tokens=32)
    prompts = [tokens(n, cfg["vocab"], 30 + n) for n in (1, 5, 37, 70)]
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    for p, out in zip(prompts, outs):
        seq = list(p)
        for _ in range(12):
            seq.append(int(t_forward(cfg, w, seq, dtype=torch.float64)[-1].argmax()))
        assert out.outputs[0].token_ids == seq[len(p):]
