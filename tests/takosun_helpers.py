"""Shared by the Takosun tests: small configurations that differ from one another in every size, weights made
here (by checkpoint name, with no help from the package) and the comparison with the plain implementation."""
import json
import math
import os

import torch
from safetensors.torch import save_file

from plain_takosun import t_forward


def mixer(heads, dim, rot_dim, vdim, kv_rank, q_rank, base=10000.0, kv_from=None, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "rot": {"base": base, "dims": rot_dim}, "scale": scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim)}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, shared=None):
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def layer(m, mlp):
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


# P: two heads, values wider than keys, two experts of three per token, a borrowed latent two layers back, one
# norm group; S: sizes that are multiples of 4 at most, with a latent wider than the matrix-core attention's heads;
# Q: five heads, sizes that are no powers of two, a layer without feed-forward, experts without a
# shared one, four norm groups; R: one head, a single expert per token, three layers on one latent.
CONFIGS = {
    "P": {"architecture": "Takosun", "vocab": 97, "width": 64, "norm": {"eps": 1e-5, "groups": 1}, "layers": [
        layer(mixer(2, 16, 8, 24, 32, 40), dense(96)),
        layer(mixer(2, 16, 8, 24, 48, 24, base=777.0), moe(32, 3, 2, shared=48)),
        layer(mixer(2, 16, 8, 24, 32, 40, kv_from=0), moe(40, 4, 3)),
    ]},
    "Q": {"architecture": "Takosun", "vocab": 211, "width": 120, "norm": {"eps": 1e-6, "groups": 4}, "layers": [
        layer(mixer(5, 24, 16, 8, 40, 56, base=50000.0, scale=0.21), None),
        layer(mixer(5, 24, 16, 8, 40, 56, base=50000.0, kv_from=0, scale=0.3), moe(24, 5, 1)),
        layer(mixer(3, 8, 32, 40, 24, 16), dense(72)),
        layer(mixer(3, 8, 32, 40, 24, 16, kv_from=2), dense(200)),
    ]},
    "S": {"architecture": "Takosun", "vocab": 61, "width": 36, "norm": {"eps": 1e-5, "groups": 3}, "layers": [
        layer(mixer(3, 12, 20, 6, 300, 20), moe(10, 3, 2, shared=50)),
        layer(mixer(2, 4, 20, 28, 300, 44, kv_from=0), dense(52)),
    ]},
    # M: sizes at which the matrix-core forms of the per-head products and of the grouped experts run, the cached row
    # as wide as the matrix-core attention takes (224 + 32), products of many rows and columns
    "M": {"architecture": "Takosun", "vocab": 300, "width": 1024, "norm": {"eps": 1e-5, "groups": 2}, "layers": [
        layer(mixer(8, 64, 32, 96, 224, 384, base=50000.0), dense(2048)),
        layer(mixer(8, 64, 32, 96, 224, 384, base=50000.0, kv_from=0), moe(512, 4, 2, shared=512)),
    ]},
    "R": {"architecture": "Takosun", "vocab": 50, "width": 32, "norm": {"eps": 1e-5, "groups": 2}, "layers": [
        layer(mixer(1, 32, 4, 16, 12, 8), moe(16, 2, 1, shared=8)),
        layer(mixer(1, 32, 4, 16, 12, 8, kv_from=0), dense(64)),
        layer(mixer(1, 32, 4, 16, 12, 8, kv_from=0), moe(16, 6, 2, shared=16)),
    ]},
}


def make_weights(cfg, seed, spread=1.0):
    """Random weights by checkpoint name. Matrices N(0, spread^2 / inputs), so that activations keep their size and
    ``spread`` sets how peaked the attention is; norm weights around 1; averaging weights positive and unequal;
    every table row distinct experts."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    w = {}

    def mat(name, rows, cols, s=1.0):
        w[name] = torch.randn((rows, cols), generator=g) * (s / math.sqrt(cols))

    def vec(name, n):
        w[name] = 1.0 + 0.2 * torch.randn((n,), generator=g)

    w["embed"] = torch.randn((V, W), generator=g)
    for i, lay in enumerate(cfg["layers"]):
        p, m, mlp = "l%d" % i, lay["mixer"], lay["mlp"]
        H, dn, dr, dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        vec(p + ".norm1", W), vec(p + ".norm1b", W)
        mat(p + ".mix.dq", Q, W), vec(p + ".mix.dq.norm", Q), mat(p + ".mix.uq", H * (dn + dr), Q, spread * 2.0)
        if m.get("kv_from") is None:
            mat(p + ".mix.dkv", R + dr, W), vec(p + ".mix.dkv.norm", R)
        mat(p + ".mix.uk", H * dn, R, spread * 2.0), mat(p + ".mix.uv", H * dv, R), mat(p + ".mix.g", H, W)
        mat(p + ".mix.o", W, H * dv)
        if mlp is not None:
            vec(p + ".norm2", W), vec(p + ".norm2b", W)
            if mlp["kind"] == "dense":
                mat(p + ".mlp.gate", mlp["ff"], W), mat(p + ".mlp.up", mlp["ff"], W), mat(p + ".mlp.down", W, mlp["ff"])
            else:
                E, top, F = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"]
                for e in range(E):
                    q = "%s.mlp.e%d" % (p, e)
                    mat(q + ".gate", F, W), mat(q + ".up", F, W), mat(q + ".down", W, F)
                w[p + ".mlp.table"] = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(V)]).to(torch.int32)
                if mlp.get("shared"):
                    S = mlp["shared"]["ff"]
                    mat(p + ".mlp.shared.gate", S, W), mat(p + ".mlp.shared.up", S, W), mat(p + ".mlp.shared.down", W, S)
        w[p + ".dwa"] = 0.15 + torch.rand((i + 2,), generator=g) * 0.5
    vec("final.norm", W)
    mat("head", V, W)
    # the values a bfloat16 checkpoint would hold, so that every run sees the same numbers
    return {k: (v.to(torch.bfloat16).to(torch.float32) if v.dtype.is_floating_point else v) for k, v in w.items()}


def write_model(folder, cfg, weights):
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: (v.to(torch.bfloat16) if v.dtype.is_floating_point else v).contiguous() for k, v in weights.items()},
              os.path.join(folder, "model.safetensors"))
    return folder


def make_model(tmp_path, which, seed=0, spread=1.0):
    cfg = CONFIGS[which]
    weights = make_weights(cfg, seed, spread)
    folder = write_model(os.path.join(str(tmp_path), "takosun_%s_%d_%g" % (which, seed, spread)), cfg, weights)
    return folder, cfg, weights


def plain_logits(cfg, weights, tokens):
    return t_forward(cfg, weights, tokens, dtype=torch.float64).to(torch.float32)


def rel_err(got, ref):
    """The largest difference, relative to the spread of the reference logits."""
    return float((got.double().cpu() - ref.double()).abs().max() / ref.double().std())


def replay(executor, StepEntry, requests, steps):
    """Runs ``steps`` (lists of (request, count)) over ``requests`` (name -> tokens), wanting every position;
    a request is released when its tokens are used up. Returns name -> logits [T, V]."""
    at = {k: 0 for k in requests}
    got = {k: [] for k in requests}
    for step in steps:
        entries = []
        for k, n in step:
            entries.append(StepEntry(k, requests[k][at[k]:at[k] + n], list(range(n))))
        out = executor.step(entries)
        row = 0
        for k, n in step:
            got[k].append(out[row:row + n].float().cpu())
            row += n
            at[k] += n
            if at[k] == len(requests[k]):
                executor.release(k)
    return {k: torch.cat(v) for k, v in got.items() if v}


def row_err(got, ref):
    """Per position: the root mean square over the vocabulary of the difference (its mean taken off), relative to
    the spread of the reference logits; the largest over the positions. Rounding in bfloat16 spreads over a row,
    a wrong key moves the whole row."""
    d = got.double().cpu() - ref.double()
    d = d - d.mean(dim=-1, keepdim=True)
    return float(d.pow(2).mean(dim=-1).sqrt().max() / ref.double().std())


def row_errs(got, ref):
    """``row_err`` for every position."""
    d = got.double().cpu() - ref.double()
    d = d - d.mean(dim=-1, keepdim=True)
    return d.pow(2).mean(dim=-1).sqrt() / ref.double().std()


def bfloat16_limits(cfg, weights, tokens, ref):
    """What rounding to bfloat16 may cost at every position: three times what it costs the plain implementation run
    in bfloat16 throughout (norms and softmax too, which the engine keeps in float32), but no less than three times
    the median of that over the positions. Positions whose logits hang on small differences have large limits,
    the others small ones."""
    e = row_errs(t_forward(cfg, weights, tokens, dtype=torch.bfloat16), ref)
    return 3.0 * torch.maximum(e, e.median())


def within(got, ref, limits):
    """Whether ``got`` differs from ``ref`` by rounding only: at most 4 % of the positions (or one) over their limit,
    none over three times its limit. (One sample of rounding per position is a rough measure, hence the allowance.)
    Returns (verdict, the worst ratio)."""
    ratio = row_errs(got, ref) / limits
    over = int((ratio > 1.0).sum())
    return bool(over <= max(1, 0.04 * ratio.numel()) and (ratio <= 3.0).all()), float(ratio.max())
