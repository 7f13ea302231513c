"""Small Niresun configurations and random weights by checkpoint name, made without the package's help, for the
tests that compare the engine with the plain implementation (plain_niresun.py)."""
import json
import math
import os

import torch
from safetensors.torch import save_file

import plain_niresun as P


def mamba(inner, state, rank, conv, mlp=None):
    return {"type": "mamba1", "mixer": {"inner": inner, "state": state, "dt_rank": rank, "conv": conv}, "mlp": mlp}


def attn(heads, kv, dim, vdim, chunk, rot_dims, base=10000.0, scaling=None, scale=None, mlp=None):
    rot = None if not rot_dims else {"base": base, "dims": rot_dims}
    if rot is not None and scaling:
        rot["scaling"] = scaling
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5}
    if rot is not None:
        m["rot"] = rot
    if chunk:
        m["mask"] = {"size": chunk}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def pair(heads, kv, dim, vdim, conv, temp, rheads, rdim, rvdim, cap, scale=None, mlp=None):
    left = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale or dim ** -0.5}
    if temp:
        left["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": rheads, "dim": rdim, "vdim": rvdim,
                                                                  "gate_cap": cap}}, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


SCALING = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}

# Sizes differ between the configurations and from one another inside each: values wider and narrower than keys,
# one to six heads, kv heads equal to the heads and fewer, one to five taps, states of 4 to 40 entries (more than 16 a
# lane group, and not a power of two), chunks that are no multiple of a page, layers in several orders, with and
# without a feed-forward, rotation over a whole head and over part of it, with and without frequency scaling.
CONFIGS = {
    "A": {"architecture": "Niresun", "vocab": 61, "width": 48, "norm": {"eps": 1e-5}, "layers": [
        mamba(72, 8, 5, 4),
        attn(4, 2, 16, 24, 20, 8, scaling=SCALING, mlp=dense(96)),
        pair(4, 2, 16, 16, 3, (0.4, 8), 2, 24, 16, 12.0, mlp=dense(64)),
        mamba(72, 8, 5, 4, mlp=dense(80)),
    ]},
    "B": {"architecture": "Niresun", "vocab": 77, "width": 64, "norm": {"eps": 1e-6}, "layers": [
        pair(6, 6, 8, 24, 2, None, 3, 8, 40, 4.0, mlp=None),
        attn(3, 1, 32, 16, 7, 32, base=500.0),
        mamba(40, 40, 3, 2),
        attn(2, 2, 24, 24, None, None, scale=0.3, mlp=dense(48)),
        pair(1, 1, 32, 8, 5, (1.5, 3), 1, 40, 24, 30.0),
    ]},
    "C": {"architecture": "Niresun", "vocab": 40, "width": 32, "norm": {"eps": 1e-5}, "layers": [
        attn(1, 1, 48, 64, 33, 16, scaling={"factor": 2.0, "low": 2.0, "high": 8.0, "original": 32}),
        mamba(32, 4, 1, 3, mlp=dense(32)),
        pair(2, 1, 16, 8, 1, (0.25, 1), 2, 8, 8, 2.0),          # filters of one tap: no state of the convolution
        mamba(24, 20, 2, 1),
    ]},
    # sizes at which the matrix-core attention kernels and the wider state tiles run (GPU tests)
    "M": {"architecture": "Niresun", "vocab": 300, "width": 256, "norm": {"eps": 1e-5}, "layers": [
        mamba(512, 16, 16, 4),
        attn(8, 2, 64, 96, 48, 32, scaling=SCALING, mlp=dense(512)),
        pair(8, 4, 64, 64, 4, (0.3, 16), 4, 64, 128, 10.0, mlp=dense(384)),
        mamba(512, 72, 16, 4),
    ]},
}


def make_weights(cfg, seed, spread=1.0):
    """Matrices N(0, spread^2 / inputs); Dynamic Tanh weights around 1 with small offsets and alpha around 0.7;
    convolution filters of order 1; decays exp(A_log) between about 0.3 and 3; gate biases that keep some memory."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    w = {}

    def mat(name, rows, cols, s=1.0):
        w[name] = torch.randn((rows, cols), generator=g) * (s / math.sqrt(cols))

    def around(name, n, centre=1.0, dev=0.2):
        w[name] = centre + dev * torch.randn((n,), generator=g)

    def dyt(name):
        around(name, W), around(name + ".b", W, 0.0, 0.1)
        w[name + ".alpha"] = torch.tensor(0.5 + 0.4 * float(torch.rand((), generator=g)))

    w["embed"] = torch.randn((V, W), generator=g)
    for i, lay in enumerate(cfg["layers"]):
        p, m = "l%d" % i, lay["mixer"]
        dyt(p + ".norm1")
        q = p + ".mix"
        if lay["type"] == "mamba1":
            I, n, r, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
            mat(q + ".in", 2 * I, W), mat(q + ".x", r + 2 * n, I), mat(q + ".dt", I, r), mat(q + ".o", W, I)
            w[q + ".conv"] = torch.randn((I, taps), generator=g) * 0.5
            around(q + ".conv.b", I, 0.0, 0.1), around(q + ".dt.b", I, -1.0, 0.5), around(q + ".D", I)
            w[q + ".A_log"] = torch.randn((I, n), generator=g) * 0.6
        elif lay["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            mat(q + ".q", H * d, W, spread * 2.0), mat(q + ".k", G * d, W, spread * 2.0), mat(q + ".v", G * dv, W)
            around(q + ".q.b", H * d, 0.0, 0.1), around(q + ".k.b", G * d, 0.0, 0.1), around(q + ".v.b", G * dv, 0.0, 0.1)
            mat(q + ".g", H * dv, W), mat(q + ".o", W, H * dv)
        else:
            lf, rt = m["left"], m["right"]
            H, G, d, dv, taps = lf["heads"], lf["kv_heads"], lf["dim"], lf["vdim"], lf["conv"]
            mat(q + ".left.q", H * d, W, spread), mat(q + ".left.k", G * d, W, spread), mat(q + ".left.v", G * dv, W)
            for x, n in (("q", H * d), ("k", G * d), ("v", G * dv)):
                w["%s.left.%s.conv" % (q, x)] = torch.randn((n, taps), generator=g) * 0.5
            mat(q + ".left.o", W, H * dv), around(q + ".left.out", W)
            H, d, dv = rt["heads"], rt["dim"], rt["vdim"]
            mat(q + ".right.q", H * d, W), mat(q + ".right.k", H * d, W), mat(q + ".right.v", H * dv, W)
            mat(q + ".right.g", H * dv, W), mat(q + ".right.o", W, H * dv), around(q + ".right.norm", H * dv)
            mat(q + ".right.i", H, W, 2.0), mat(q + ".right.f", H, W, 2.0)
            around(q + ".right.i.b", H, 0.0, 1.0), around(q + ".right.f.b", H, 2.0, 1.0), around(q + ".right.out", W)
        if lay["mlp"] is not None:
            dyt(p + ".norm2")
            F = lay["mlp"]["ff"]
            mat(p + ".mlp.gate", F, W), mat(p + ".mlp.up", F, W), mat(p + ".mlp.down", W, F)
    dyt("final.norm")
    mat("head", V, W)
    # the values a bfloat16 checkpoint would hold, so that every run sees the same numbers
    return {k: v.to(torch.bfloat16).to(torch.float32) for k, v in w.items()}


def write_model(folder, cfg, weights):
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def make_model(tmp_path, which, seed=0, spread=1.0, weights=None):
    cfg = CONFIGS[which] if isinstance(which, str) else which
    weights = weights if weights is not None else make_weights(cfg, seed, spread)
    tag = which if isinstance(which, str) else "custom"
    folder = write_model(os.path.join(str(tmp_path), "niresun_%s_%d_%g" % (tag, seed, spread)), cfg, weights)
    return folder, cfg, weights


def plain_logits(cfg, weights, tokens, dtype=torch.float64):
    return P.forward(cfg, {k: v.to(dtype) for k, v in weights.items()}, tokens).to(torch.float32)


def row_errs(got, ref):
    """Per position: the root mean square over the vocabulary of the difference (its mean taken off), relative to
    the spread of the reference logits."""
    d = got.double().cpu() - ref.double()
    d = d - d.mean(dim=-1, keepdim=True)
    return d.pow(2).mean(dim=-1).sqrt() / ref.double().std()


def single_layer(which, index, vocab=53):
    """The configuration of one layer of ``which`` alone (a mechanism on its own)."""
    cfg = CONFIGS[which]
    return {"architecture": "Niresun", "vocab": vocab, "width": cfg["width"], "norm": cfg["norm"],
            "layers": [cfg["layers"][index]]}


def bfloat16_limits(cfg, weights, tokens, ref):
    """What rounding to bfloat16 may cost at every position: three times what it costs the plain implementation when
    it rounds what an engine may keep in 16 bits (plain_niresun.storage), but no less than three times the median
    of that over the positions."""
    with P.storage(torch.bfloat16):
        e = row_errs(plain_logits(cfg, weights, tokens), ref)
    return 3.0 * torch.maximum(e, e.median())


def within(got, ref, limits):
    """Whether ``got`` differs from ``ref`` by rounding only: at most 4 % of the positions (or one) over their limit,
    none over three times its limit. (One sample of rounding per position is a rough measure, hence the allowance.)
    Returns (verdict, the worst ratio)."""
    ratio = row_errs(got, ref) / limits
    over = int((ratio > 1.0).sum())
    return bool(over <= max(1, 0.04 * ratio.numel()) and (ratio <= 3.0).all()), float(ratio.max())
