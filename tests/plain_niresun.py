"""A plain, slow Niresun: whole sequences, no cache, no batches, one function per mechanism.

Written from the design's equations only; it shares nothing with the package. A model is (config dict, dict
of tensors by checkpoint name). Everything runs in the dtype of the tensors handed in (the tests use float64
or float32), token by token where the mechanism is a recurrence.

``with storage(torch.bfloat16):`` makes it round what an engine may keep in 16 bits (the operands and results of the
projections, the convolutions and activations behind them, queries, keys and values, what a mixer or feed-forward
hands back) while everything else stays as exact as the tensors' dtype: what rounding alone costs, for the tests'
limits.
"""
import contextlib
import math

import torch

_STORAGE = [None]


@contextlib.contextmanager
def storage(dtype):
    _STORAGE[0] = dtype
    try:
        yield
    finally:
        _STORAGE[0] = None


def kept(x):
    """x as a 16-bit engine would hold it between two operations."""
    return x if _STORAGE[0] is None else x.to(_STORAGE[0]).to(x.dtype)


def lin(h, w, b=None, wide=False):
    """h w^T (+ b); ``wide``: the result stays in 32 bits (it enters a recurrence, or is the logits)."""
    y = kept(h) @ w.T
    if b is not None:
        y = y + b
    return y if wide else kept(y)


def dyt(x, w, b, alpha):
    """tanh(alpha x) w + b."""
    return kept(torch.tanh(alpha * x) * w + b)


def unit_rms(x, eps):
    """x divided by its root mean square over the last dimension."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def causal_conv(u, w, bias=None):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], 0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + pad[j:j + T] * w[:, j]
    return y if bias is None else y + bias


def rotary_frequencies(dims, base, scaling, dtype=torch.float64):
    i = torch.arange(dims // 2, dtype=dtype)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f
    factor, low, high, orig = scaling["factor"], scaling["low"], scaling["high"], scaling["original"]
    out = []
    for fi in f.tolist():
        lam = 2 * math.pi / fi
        if lam < orig / high:
            out.append(fi)
        elif lam > orig / low:
            out.append(fi / factor)
        else:
            s = (orig / lam - low) / (high - low)
            out.append((1 - s) * fi / factor + s * fi)
    return torch.tensor(out, dtype=dtype)


def rotate(x, positions, dims, base, scaling):
    """x [T, heads, d]: the first ``dims`` entries of every head in pairs (i, i + dims/2)."""
    f = rotary_frequencies(dims, base, scaling, x.dtype)
    a = positions.to(x.dtype)[:, None] * f[None, :]                 # [T, dims/2]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def masked_softmax_attention(q, k, v, scale, visible):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; visible(i, j) says whether query i sees key j."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        mask = torch.tensor([[visible(i, j) for j in range(T)] for i in range(T)])
        s = s.masked_fill(~mask, float("-inf"))
        out[:, h] = torch.softmax(s, -1) @ v[:, g]
    return out


def mamba1(h, W, p, m):
    """Selective scan. h [T, width]; W name -> tensor; p the layer's prefix with '.mix'."""
    inner, state, rank = m["inner"], m["state"], m["dt_rank"]
    xz = lin(h, W[p + ".in"])
    x, z = xz[:, :inner], xz[:, inner:]
    x = kept(silu(causal_conv(x, W[p + ".conv"], W[p + ".conv.b"])))
    low = lin(x, W[p + ".x"])
    dt = softplus(lin(low[:, :rank], W[p + ".dt"], W[p + ".dt.b"], wide=True))
    B, C = low[:, rank:rank + state], low[:, rank + state:rank + 2 * state]
    A = -torch.exp(W[p + ".A_log"])
    S = torch.zeros(inner, state, dtype=h.dtype)
    ys = []
    for t in range(h.shape[0]):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        ys.append(S @ C[t] + W[p + ".D"] * x[t])
    y = kept(torch.stack(ys) * silu(z))
    return lin(y, W[p + ".o"])


def attention(h, W, p, m, eps):
    """Rotary, chunked, gated softmax attention with biases."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = lin(h, W[p + ".q"], W[p + ".q.b"]).view(T, H, d)
    k = lin(h, W[p + ".k"], W[p + ".k.b"]).view(T, G, d)
    v = lin(h, W[p + ".v"], W[p + ".v.b"]).view(T, G, dv)
    pos = torch.arange(T)
    rot = m.get("rot")               # (a configuration may leave the rotation or the chunks out)
    if rot:
        q = kept(rotate(q, pos, rot["dims"], rot["base"], rot.get("scaling")))
        k = kept(rotate(k, pos, rot["dims"], rot["base"], rot.get("scaling")))
    size = m["mask"]["size"] if m.get("mask") else 1 << 30
    o = kept(masked_softmax_attention(q, k, v, m["scale"], lambda i, j: j <= i and i // size == j // size))
    o = kept(o.reshape(T, H * dv) * torch.sigmoid(lin(h, W[p + ".g"])))
    return lin(o, W[p + ".o"])


def conv_attention(h, W, p, m, eps):
    """The left half of a parallel mixer: short convolutions, unit-norm q and k, query temperature, causal."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = kept(causal_conv(lin(h, W[p + ".q"]), W[p + ".q.conv"])).view(T, H, d)
    k = kept(causal_conv(lin(h, W[p + ".k"]), W[p + ".k.conv"])).view(T, G, d)
    v = kept(causal_conv(lin(h, W[p + ".v"]), W[p + ".v.conv"])).view(T, G, dv)
    q, k = unit_rms(q, eps), kept(unit_rms(k, eps))
    pos = torch.arange(T)
    if m.get("q_temp"):              # (a configuration may leave the temperature out)
        temp = 1.0 + m["q_temp"]["coef"] * torch.log(torch.floor((pos + 1) / m["q_temp"]["every"]).to(h.dtype) + 1.0)
        q = q * temp[:, None, None]
    o = kept(masked_softmax_attention(kept(q), k, v, m["scale"], lambda i, j: j <= i))
    return lin(o.reshape(T, H * dv), W[p + ".o"])


def mlstm(h, W, p, m, eps):
    """The right half: a matrix memory per head with capped log gates and a running maximum that starts at 0."""
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = lin(h, W[p + ".q"]).view(T, H, d) * d ** -0.5
    k = lin(h, W[p + ".k"]).view(T, H, d)
    v = lin(h, W[p + ".v"]).view(T, H, dv)
    gi = cap * torch.tanh(lin(h, W[p + ".i"], W[p + ".i.b"], wide=True) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh(lin(h, W[p + ".f"], W[p + ".f.b"], wide=True) / cap))
    S = torch.zeros(H, d, dv, dtype=h.dtype)
    n = torch.zeros(H, d, dtype=h.dtype)
    mx = torch.zeros(H, dtype=h.dtype)
    outs = []
    for t in range(T):
        m_new = torch.maximum(gf[t] + mx, gi[t])
        keep, take = torch.exp(gf[t] + mx - m_new), torch.exp(gi[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        mx = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        outs.append(num / den[:, None])
    o = unit_rms(torch.stack(outs), eps).reshape(T, H * dv) * W[p + ".norm"]
    o = kept(o * torch.sigmoid(lin(h, W[p + ".g"])))
    return lin(o, W[p + ".o"])


def parallel(h, W, p, m, eps):
    a = unit_rms(conv_attention(h, W, p + ".left", m["left"], eps), eps) * W[p + ".left.out"]
    b = unit_rms(mlstm(h, W, p + ".right", m["right"], eps), eps) * W[p + ".right.out"]
    return kept(0.5 * (a + b))


def dense_ffn(h, W, p):
    return lin(kept(gelu_tanh(lin(h, W[p + ".gate"])) * lin(h, W[p + ".up"])), W[p + ".down"])


MIXERS = {"mamba1": lambda h, W, p, m, eps: mamba1(h, W, p, m), "attention": attention, "parallel": parallel}


def forward(config, W, tokens, want_layers=False):
    """Logits [T, vocab] of one sequence; with ``want_layers`` also the stream after every layer [L, T, width]."""
    eps = config["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    after = []
    for i, layer in enumerate(config["layers"]):
        p = "l%d" % i
        h = dyt(x, W[p + ".norm1"], W[p + ".norm1.b"], W[p + ".norm1.alpha"])
        x = x + MIXERS[layer["type"]](h, W, p + ".mix", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            h = dyt(x, W[p + ".norm2"], W[p + ".norm2.b"], W[p + ".norm2.alpha"])
            x = x + dense_ffn(h, W, p + ".mlp")
        after.append(x)
    logits = lin(dyt(x, W["final.norm"], W["final.norm.b"], W["final.norm.alpha"]), W["head"], wide=True)
    return (logits, torch.stack(after)) if want_layers else logits
