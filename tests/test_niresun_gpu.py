"""Niresun on the GPU: the new kernels alone against the plain implementation's function of the same mechanism, every
kind of layer alone and the whole model through the engine's step function in float32 and bfloat16 under the ways of
cutting a request into steps, keys at the edges of chunks and pages and far away made to decide the logits, state
slots used again, long decoding from graphs, and generation through the entry point."""
import math
import random

import pytest
import torch

import plain_niresun as P
from niresun_helpers import (CONFIGS, bfloat16_limits, make_model, make_weights, plain_logits, row_errs, single_layer,
                             within)
from takosun_helpers import rel_err, replay

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
TOL_F32 = 3e-5
# bfloat16 without a model to measure rounding on: products and activations between kernels are rounded to 8 bits of
# mantissa; per position the error's root mean square over the vocabulary, relative to the logits' spread. A lost key,
# a chunk one token off or a state that is not carried moves rows by several tenths (the tests of edges check that
# with the plain implementation).
TOL_BF16 = 0.06


def ops():
    from lmsf_amd.ops import get_ops
    return get_ops()


def check(got, ref, dtype, what="", model=None):
    """``model`` = (configuration, weights, tokens): float32 then may differ by three times what float32 rounding
    costs the plain implementation itself on these tokens, where that is more than TOL_F32 (a configuration whose
    logits hang on small differences)."""
    if dtype == "float32":
        tol = TOL_F32
        if model is not None:
            tol = max(tol, 3 * rel_err(plain_logits(model[0], model[1], model[2], dtype=torch.float32), ref))
        assert rel_err(got, ref) < tol, (what, rel_err(got, ref), tol)
    elif model is not None:
        # per position, three times what rounding costs the plain implementation when it rounds what may be kept in
        # 16 bits (a fault moves rows that rounding leaves alone)
        ok, worst = within(got, ref, bfloat16_limits(model[0], model[1], model[2], ref))
        assert ok, (what, worst)
    else:
        # (rounding has outliers at positions whose logits hang on small differences: one position in fifty, or one,
        # may pass the limit, none three times the limit; a fault moves many rows, and by more)
        e = row_errs(got, ref)
        over = int((e > TOL_BF16).sum())
        assert over <= max(1, e.numel() // 50) and float(e.max()) < 3 * TOL_BF16 and float(e.median()) < TOL_BF16 / 3, \
            (what, over, float(e.max()), float(e.median()))


def close(got, ref, dtype, scale=1.0):
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    err = float((got.double().cpu() - ref.double().cpu()).abs().max())
    assert err <= tol * scale * max(1.0, float(ref.abs().max())), err


class Step:
    """The part of a step's description that the state-carrying kernels read."""

    def __init__(self, lens, slots):
        starts = [0]
        for n in lens:
            starts.append(starts[-1] + n)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
        self.n_segments = len(lens)
        self.seg_starts, self.state_slots = i32(starts), i32(slots)
        self.seg_of_token = i32([s for s, n in enumerate(lens) for _ in range(n)])


# --------------------------------------------------------------------------- kernels alone


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [48, 321, 4096, 10])
def test_dynamic_tanh_with_and_without_the_addition(dtype, H):
    o = ops()
    g = torch.Generator().manual_seed(H)
    N = 9
    branch = (torch.randn((N, H), generator=g) * 2).to(dtype)
    res = torch.randn((N, H), generator=g) * 3
    w, b = 1 + 0.3 * torch.randn(H, generator=g), 0.2 * torch.randn(H, generator=g)
    alpha = torch.tensor([0.37])
    dev = lambda t: t.cuda()
    r = res.clone().cuda()
    got = o.dyt_norm(dev(branch), r, dev(w), dev(b), dev(alpha), dtype)
    total = res + branch.float()
    close(r, total, torch.float32)
    close(got, P.dyt(total, w, b, alpha), dtype)
    rows = torch.tensor([4, 0, 4, 8], dtype=torch.int32)
    r2 = res.clone().cuda()
    got = o.dyt_norm(dev(branch), r2, dev(w), dev(b), dev(alpha), dtype, rows=dev(rows))
    close(got, P.dyt(total[rows.long()], w, b, alpha), dtype)
    assert torch.equal(r2.cpu(), res)                        # chosen rows: the stream stays as it was
    close(o.dyt_norm(None, dev(res), dev(w), dev(b), dev(alpha), dtype), P.dyt(res, w, b, alpha), dtype)
    close(o.dyt_norm(dev(branch), None, dev(w), dev(b), dev(alpha), dtype), P.dyt(branch.float(), w, b, alpha), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_activation_in_the_tanh_form(dtype):
    g = torch.Generator().manual_seed(1)
    gu = (torch.randn((5, 2 * 72), generator=g) * 3).to(dtype)
    got = ops().gated_act(gu.cuda(), "gelu_tanh")
    close(got, P.gelu_tanh(gu[:, :72].double()) * gu[:, 72:].double(), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 2, 8, 16, 40, 300])
def test_gated_product_with_the_tanh_form(dtype, rows):
    """One and few rows: the activation is the product's epilogue; more rows: the product, then the activation kernel."""
    g = torch.Generator().manual_seed(rows)
    K, I = 256, 136
    x = torch.randn((rows, K), generator=g).to(dtype)
    w = (torch.randn((2 * I, K), generator=g) / 16).to(dtype)
    got = ops().linear_gated(x.cuda(), w.cuda(), None, "gelu_tanh")
    gate, up = (x.double() @ w[:I].double().T).to(dtype).double(), (x.double() @ w[I:].double().T).to(dtype).double()
    close(got, P.gelu_tanh(gate) * up, dtype, scale=2.0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,taps,act,off", [(24, 3, None, 2), (300, 4, "silu", 2), (8, 2, None, 8), (40, 7, "silu", 8),
                                            (16, 1, None, 2), (512, 4, "silu", 8), (72, 3, None, 8)])
def test_short_convolution_over_cut_requests(dtype, C, taps, act, off):
    """Three requests; their tokens arrive in steps of unequal portions (down to one token, shorter than the filter),
    in slots that do not follow their order; every output equals the convolution over the whole request. The operand
    is a view into wider rows, beginning on a 16-byte border (off 8) or not (off 2)."""
    o = ops()
    g = torch.Generator().manual_seed(C * taps)
    lens = {"a": 23, "b": 1, "c": 9}
    u = {k: (torch.randn((n, C + 16), generator=g)).to(dtype) for k, n in lens.items()}
    w = (torch.randn((C, taps), generator=g) * 0.5).to(dtype)
    bias = (torch.randn(C, generator=g) * 0.1).to(dtype) if act else None
    state = torch.zeros((4, C * max(taps - 1, 1) + 3), dtype=torch.float32, device="cuda")
    slot = {"a": 2, "b": 0, "c": 3}
    steps = [[("a", 5), ("b", 1), ("c", 1)], [("c", 1), ("a", 1)], [("a", 2), ("c", 7)], [("a", 15)]]
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    for step in steps:
        x = torch.cat([u[k][at[k]:at[k] + n] for k, n in step]).cuda()[:, off:off + C]   # a view into wider rows
        y = o.short_conv(x, w.cuda(), None if bias is None else bias.cuda(), state[:, 3:] if taps > 1 else None,
                         Step([n for _, n in step], [slot[k] for k, _ in step]), act)
        row = 0
        for k, n in step:
            got[k].append(y[row:row + n].cpu())
            row += n
            at[k] += n
    for k in lens:
        ref = P.causal_conv(u[k][:, off:off + C].double(), w.double(), None if bias is None else bias.double())
        close(torch.cat(got[k]), P.silu(ref) if act else ref, dtype, scale=2.0)
    assert float(state[1].abs().max()) == 0.0 and float(state[:, :3].abs().max()) == 0.0     # nobody else's memory


def rotary_table(max_pos, rot, base, scaling=None):
    f = P.rotary_frequencies(rot, base, scaling).to(torch.float32)
    ang = torch.arange(max_pos, dtype=torch.float32)[:, None] * f[None, :]
    return torch.cat([torch.cos(ang), torch.sin(ang)], dim=1).contiguous()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,dim,vdim,rot,norm,temp,ps", [(4, 2, 16, 24, 8, False, None, 8), (3, 3, 40, 8, 0, True, (0.5, 4), 16),
                                                          (6, 2, 64, 72, 32, False, None, 16), (2, 1, 24, 24, 24, True, (1.5, 64), 4)])
def test_queries_keys_and_values_made_ready(dtype, H, G, dim, vdim, rot, norm, temp, ps):
    o = ops()
    g = torch.Generator().manual_seed(H * dim + vdim)
    N, pages, D = 21, 6, (max(dim, vdim) + 15) // 16 * 16
    buf = (torch.randn((N, (H + G) * dim + G * vdim + 4), generator=g) * 2).to(dtype)
    q, k, v = buf[:, :H * dim], buf[:, H * dim:(H + G) * dim], buf[:, (H + G) * dim:(H + G) * dim + G * vdim]
    pos = torch.randint(0, 300, (N,), generator=g).to(torch.int32)
    slots = torch.randperm(pages * ps, generator=g)[:N].to(torch.int32)
    slots[5] = -1
    table = rotary_table(512, rot, 10000.0) if rot else None
    kp = torch.full((pages, G, ps, D), 7.0, dtype=dtype, device="cuda")
    vp = torch.full((pages, G, D, ps), 7.0, dtype=dtype, device="cuda")
    b = buf.cuda()
    qa = o.attn_prepare(b[:, :H * dim], b[:, H * dim:(H + G) * dim], b[:, (H + G) * dim:], H, G, dim, vdim, D, pos.cuda(),
                        slots.cuda(), kp, vp, table=None if table is None else table.cuda(),
                        unit_norm_eps=1e-5 if norm else None, temp_coef=temp[0] if temp else 0.0,
                        temp_every=temp[1] if temp else 0)
    qr, kr = q.double().reshape(N, H, dim), k.double().reshape(N, G, dim)
    if norm:
        qr, kr = P.unit_rms(qr, 1e-5), P.unit_rms(kr, 1e-5)
    if rot:
        qr, kr = P.rotate(qr, pos.long(), rot, 10000.0, None), P.rotate(kr, pos.long(), rot, 10000.0, None)
    if temp:
        qr = qr * (1.0 + temp[0] * torch.log(torch.floor((pos.double() + 1) / temp[1]) + 1.0))[:, None, None]
    qa = qa.reshape(N, H, D).cpu()
    close(qa[..., :dim], qr, dtype, scale=2.0)
    assert float(qa[..., dim:].abs().max()) == 0.0 if D > dim else True
    kp, vp = kp.cpu(), vp.cpu()
    for t in range(N):
        s = int(slots[t])
        if s < 0:
            continue
        close(kp[s // ps, :, s % ps, :dim], kr[t], dtype, scale=2.0)
        close(vp[s // ps, :, :vdim, s % ps], v[t].double().reshape(G, vdim), dtype)
        assert float(kp[s // ps, :, s % ps, dim:].abs().sum()) == 0.0 and float(vp[s // ps, :, vdim:, s % ps].abs().sum()) == 0.0
    used = set(int(s) for s in slots if s >= 0)
    free = [s for s in range(pages * ps) if s not in used]
    assert all(float(kp[s // ps, 0, s % ps, 0]) == 7.0 for s in free)                    # untouched slots stay


@pytest.mark.parametrize("kernel", ["generic", "mfma"])
@pytest.mark.parametrize("chunk,ps", [(20, 16), (80, 16), (7, 8), (64, 32), (33, 4)])
def test_attention_within_chunks_of_positions(kernel, chunk, ps):
    """A prompt's portion that begins inside a chunk and runs over two chunk edges, and single tokens on both sides of
    an edge; one key just inside the chunk and one just outside are made to stand out, so that an edge one token
    off moves the result."""
    o = ops()
    dtype = torch.bfloat16 if kernel == "mfma" else torch.float32
    g = torch.Generator().manual_seed(chunk)
    H, G, d = 4, 2, 32
    T = 3 * chunk + 5
    k = torch.randn((T, G, d), generator=g)
    v = torch.randn((T, G, d), generator=g)
    for edge in (chunk, 2 * chunk, 3 * chunk):
        k[edge] *= 4.0
        k[edge - 1] *= 4.0                                  # the last key of the chunk before: never seen from behind the edge
    q = torch.randn((T, H, d), generator=g) * 2
    k, v, q = k.to(dtype), v.to(dtype), q.to(dtype)
    pages = -(-T // ps)
    order = torch.randperm(pages, generator=g)
    kp = torch.zeros((pages, G, ps, d), dtype=dtype)
    vp = torch.zeros((pages, G, d, ps), dtype=dtype)
    for t in range(T):
        kp[order[t // ps], :, t % ps] = k[t]
        vp[order[t // ps], :, :, t % ps] = v[t]
    ref = P.masked_softmax_attention(q.double(), k.double(), v.double(), 0.3, lambda i, j: j <= i and i // chunk == j // chunk)
    bt = order.to(torch.int32)[None, :].contiguous().cuda()
    first = chunk - 3
    for rows in ([*range(first, T)], [chunk - 1], [chunk], [2 * chunk + 1], [T - 1]):
        n = len(rows)
        got = o.paged_attention(q[rows].reshape(n, H * d).cuda(), kp.cuda(), vp.cuda(), bt,
                                torch.zeros(n, dtype=torch.int32, device="cuda"),
                                torch.tensor(rows, dtype=torch.int32, device="cuda"), H, G, d, 0.3, kernel=kernel, chunk=chunk)
        close(got.reshape(n, H, d), ref[rows], dtype, scale=3.0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_heads_gated_and_unpadded_and_two_branches_joined(dtype):
    o = ops()
    g = torch.Generator().manual_seed(3)
    N, H, D, dv, W = 6, 3, 32, 24, 80
    x = torch.randn((N, H * D), generator=g).to(dtype)
    gate = torch.randn((N, H * dv + 8), generator=g).to(dtype)
    ref = x.double().reshape(N, H, D)[..., :dv].reshape(N, H * dv)
    close(o.head_gate(x.cuda(), D, H, dv), ref, dtype)
    close(o.head_gate(x.cuda(), D, H, dv, gate=gate.cuda()[:, 8:]), ref * torch.sigmoid(gate[:, 8:].double()), dtype)
    a, b = (torch.randn((N, W), generator=g) * 3).to(dtype), (torch.randn((N, W), generator=g) * 0.1).to(dtype)
    wa, wb = 1 + 0.3 * torch.randn(W, generator=g), 1 + 0.3 * torch.randn(W, generator=g)
    ref = 0.5 * (P.unit_rms(a.double(), 1e-5) * wa + P.unit_rms(b.double(), 1e-5) * wb)
    close(o.rms_pair(a.cuda(), b.cuda(), wa.cuda(), wb.cuda(), 1e-5, 0.5), ref, dtype)


# --------------------------------------------------------------------------- through the engine


def build(tmp_path, which, dtype, pages=48, block=8, seed=0, spread=1.0, eager=False, slots=4, weights=None):
    from lmsf_amd.engine import load_engine_core
    folder, cfg, w = make_model(tmp_path, which, seed, spread, weights=weights)
    core = load_engine_core(folder, dtype=dtype, block_size=block, num_pages=pages, max_model_len=pages * block,
                            max_num_seqs=slots, enforce_eager=eager)
    return core, cfg, w


def tokens(n, vocab, seed):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


LAYERS_ALONE = [("A", 0), ("A", 1), ("A", 2), ("B", 0), ("B", 1), ("B", 2), ("B", 3), ("B", 4), ("C", 0), ("C", 2), ("C", 3),
                ("M", 2), ("M", 3)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which,index", LAYERS_ALONE)
def test_every_kind_of_layer_alone(tmp_path, which, index, dtype):
    """One layer between the embedding and the head: whole, then in portions down to two tokens with single tokens
    behind them, beside a second request."""
    from lmsf_amd.engine import StepEntry
    cfg = single_layer(which, index)
    core, cfg, w = build(tmp_path, cfg, dtype, seed=index)
    V = cfg["vocab"]
    a, b = tokens(75, V, 1), tokens(30, V, 2)
    ref = {"a": plain_logits(cfg, w, a), "b": plain_logits(cfg, w, b)}
    check(replay(core.executor, StepEntry, {"a": a}, [[("a", 75)]])["a"], ref["a"], dtype, "whole", (cfg, w, a))
    steps = [[("a", 7), ("b", 2)], [("a", 2)], [("b", 20), ("a", 33)], [("a", 1), ("b", 1)], [("a", 22), ("b", 1)]] + \
            [[("a", 1), ("b", 1)]] * 6 + [[("a", 1)]] * 4
    got = replay(core.executor, StepEntry, {"a": a, "b": b}, steps)
    for k in ref:
        check(got[k], ref[k], dtype, k, (cfg, w, {"a": a, "b": b}[k]))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which,index,chunk", [("A", 0, 32), ("B", 2, 16), ("M", 3, 128), ("A", 2, 0), ("B", 4, 0), ("M", 2, 0)])
def test_long_portions_take_the_forms_that_work_on_chunks(tmp_path, which, index, chunk, dtype):
    """A scan or a matrix memory alone under prompts' portions of hundreds of tokens: the selective scan cuts them into
    chunks that run side by side (here also with small chunks, so that there are many), the matrix memory works on a
    chunk of tokens at once; a second request's short portions and single tokens beside them take the other forms,
    and the state goes from one form to the other and back."""
    from lmsf_amd.engine import StepEntry
    cfg = single_layer(which, index)
    core, cfg, w = build(tmp_path, cfg, dtype, seed=7, pages=64, block=16)
    o = ops()
    keep = o.scan_chunk_tokens
    try:
        if chunk:
            o.scan_chunk_tokens = chunk
        V = cfg["vocab"]
        a, b = tokens(700, V, 5), tokens(60, V, 6)
        steps = [[("a", 301), ("b", 3)], [("a", 1), ("b", 1)], [("b", 40), ("a", 333)], [("a", 1)], [("a", 60), ("b", 16)]] + \
                [[("a", 1)]] * 4
        got = replay(core.executor, StepEntry, {"a": a, "b": b}, steps)
        for k, t in (("a", a), ("b", b)):
            check(got[k], plain_logits(cfg, w, t), dtype, k, (cfg, w, t))
    finally:
        o.scan_chunk_tokens = keep


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_four_ways_of_cutting_give_the_plain_logits(tmp_path, which, dtype):
    from lmsf_amd.engine import StepEntry
    core, cfg, w = build(tmp_path, which, dtype, slots=3)
    V = cfg["vocab"]
    ex = core.executor
    a, b, c, d = tokens(150, V, 1), tokens(1, V, 2), tokens(67, V, 3), tokens(200, V, 4)
    ref = {k: plain_logits(cfg, w, t) for k, t in (("a", a), ("b", b), ("c", c), ("d", d))}
    toks = {"a": a, "b": b, "c": c, "d": d}
    for k, t in (("a", a), ("b", b)):
        check(replay(ex, StepEntry, {k: t}, [[(k, len(t))]])[k], ref[k], dtype, (k, "whole"), (cfg, w, t))
    got = replay(ex, StepEntry, {"a": a}, [[("a", 110)]] + [[("a", 1)]] * 40)["a"]
    check(got, ref["a"], dtype, "decode", (cfg, w, a))
    cuts = [15, 1, 2, 30, 16, 2, 33, 17, 19] + [1] * 15
    got = replay(ex, StepEntry, {"a": a}, [[("a", n)] for n in cuts])["a"]
    check(got, ref["a"], dtype, "portions", (cfg, w, a))
    # unequal requests together, three state slots for four requests; d starts in pages and a slot that were given back
    steps = [[("a", 64), ("b", 1), ("c", 3)], [("c", 2), ("a", 1)], [("a", 85), ("c", 61)], [("c", 1)],
             [("d", 2)], [("d", 197)], [("d", 1)]]
    got = replay(ex, StepEntry, {"a": a, "b": b, "c": c, "d": d}, steps)
    for k in ref:
        check(got[k], ref[k], dtype, (k, "mixed"), (cfg, w, toks[k]))
    core.storage.manager.check_invariants()
    assert core.storage.manager.num_free_pages(0) == 48 and core.storage.manager.num_free_state_slots() == 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_at_which_the_matrix_core_kernels_run(tmp_path, dtype):
    from lmsf_amd.engine import StepEntry
    core, cfg, w = build(tmp_path, "M", dtype, pages=40, block=16)
    V = cfg["vocab"]
    a, b = tokens(330, V, 21), tokens(70, V, 22)
    steps = [[("a", 280)], [("a", 40), ("b", 60)]] + [[("a", 1), ("b", 1)]] * 10
    got = replay(core.executor, StepEntry, {"a": a, "b": b}, steps)
    for k, t in (("a", a), ("b", b)):
        check(got[k], plain_logits(cfg, w, t), dtype, k, (cfg, w, t))


def peaked(cfg, seed, kind):
    """Weights and constants with which the layer's attention is peaked, so that single keys decide: queries and
    keys scaled up where their size matters, the score's scale where they are normed."""
    w = make_weights(cfg, seed)
    if kind == "attention":
        for x in ("q", "k"):
            w["l0.mix." + x] = (w["l0.mix." + x] * 3.0).to(torch.bfloat16).to(torch.float32)
    else:
        cfg["layers"][0]["mixer"]["left"]["scale"] = 1.0
    return w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["attention", "parallel"])
def test_keys_at_edges_and_far_away_decide(tmp_path, kind, dtype):
    """Peaked attention in one layer. The plain implementation names a far token whose change moves the last logits
    by much more than the tolerance (attention in chunks: the far tokens of the last chunk, its first key among
    them; the parallel layer: the first hundred tokens), and says that the last token before the chunk moves
    nothing. The engine must then give the plain logits from a prompt in two portions and single tokens behind."""
    import copy
    from lmsf_amd.engine import StepEntry
    cfg = copy.deepcopy(single_layer("A", 1 if kind == "attention" else 2))
    w = peaked(cfg, 5, kind)
    core, cfg, w = build(tmp_path, cfg, dtype, weights=w)
    V = cfg["vocab"]
    t = tokens(187, V, 9)
    ref = plain_logits(cfg, w, t)
    tol = TOL_F32 if dtype == "float32" else TOL_BF16
    chunk = cfg["layers"][0]["mixer"].get("mask", {}).get("size")
    first = 186 - 186 % chunk if chunk else 0
    far = range(first, first + 4) if chunk else range(0, 100, 3)

    def moved(j):
        return float(row_errs(plain_logits(cfg, w, t[:j] + [(t[j] + 1) % V] + t[j + 1:]), ref)[-5:].max())

    effects = {j: moved(j) for j in far}
    assert max(effects.values()) > 4 * tol, effects
    if chunk:
        assert moved(first) > tol and moved(first - 1) < 1e-9          # the chunk's first key is seen, the one before is not
    got = replay(core.executor, StepEntry, {"a": t}, [[("a", 150)], [("a", 29)]] + [[("a", 1)]] * 8)["a"]
    check(got, ref, dtype, "", (cfg, w, t))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_graphs_equals_eager(tmp_path, dtype):
    from lmsf_amd.engine import StepEntry
    outs = []
    for eager in (False, True):
        core, cfg, w = build(tmp_path, "A", dtype, eager=eager)
        V = cfg["vocab"]
        a, b = tokens(200, V, 11), tokens(140, V, 12)
        steps = [[("a", 20), ("b", 3)]] + [[("a", 1), ("b", 1)]] * 137 + [[("a", 1)]] * 43
        outs.append(replay(core.executor, StepEntry, {"a": a, "b": b}, steps))
        assert core.executor.use_graphs == (not eager)
    ref = {"a": plain_logits(cfg, w, a), "b": plain_logits(cfg, w, b)}
    for k in ref:
        assert torch.equal(outs[0][k], outs[1][k]), k
        check(outs[0][k], ref[k], dtype, k, (cfg, w, {"a": a, "b": b}[k]))


def test_greedy_generation_through_the_entry_point(tmp_path):
    from lmsf_amd.engine import LLM
    from lmsf_amd.sampling import SamplingParams
    folder, cfg, w = make_model(tmp_path, "B", seed=5)
    llm = LLM(folder, dtype="float32", block_size=8, num_gpu_blocks_override=64, max_num_seqs=4, max_model_len=256,
              prefill_chunk_size=16, max_num_batched_tokens=32)
    prompts = [tokens(n, cfg["vocab"], 30 + n) for n in (1, 5, 37, 70)]
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    for p, out in zip(prompts, outs):
        seq = list(p)
        for _ in range(12):
            seq.append(int(plain_logits(cfg, w, seq)[-1].argmax()))
        assert out.outputs[0].token_ids == seq[len(p):]
