"""Plain, slow implementation of the Takosun decoder: whole sequences, no cache, no batching, float32 (or
float64) on the CPU, one function per mechanism. It reads the configuration as a plain dict and the weights
as a dict of tensors by checkpoint name, and shares no code with the package under test.

Notation: T tokens, W the model's width, H heads, dn / dr unrotated / rotated query-key sizes of a head,
dv a head's value size, R the latent's size.

The keys and values are formed for every head from the latent (k_h = [U_k,h c | rot(r)], v_h = U_v,h c): the
direct form, not the one with the up-projections folded into the queries.
"""
import math

import torch


def t_group_rms_norm(x, weight, eps, groups):
    """The vector in ``groups`` equal consecutive parts; each part over the root of its own mean square plus
    eps; the whole times w."""
    shape = x.shape
    n = shape[-1]
    assert n % groups == 0
    parts = x.reshape(shape[:-1] + (groups, n // groups))
    ms = (parts * parts).mean(dim=-1, keepdim=True)
    return (parts / torch.sqrt(ms + eps)).reshape(shape) * weight


def t_rms_norm(x, weight, eps):
    return t_group_rms_norm(x, weight, eps, 1)


def t_rotate(x, positions, base, dims):
    """Rotation of the first ``dims`` entries of the last axis: entry i pairs with i + dims/2,
    (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = position * base^(-2i/dims). x: [T, ..., >= dims]."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    freq = (float(base) ** (-2.0 * i / dims)).to(torch.float32)
    ang = positions.to(torch.float32)[:, None] * freq[None, :]            # float32 angles
    cos, sin = torch.cos(ang).to(x.dtype), torch.sin(ang).to(x.dtype)
    while cos.dim() < x.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def t_latent_kv(h, positions, w, prefix, m, eps):
    """What a layer with a down-projection of its own keeps per token: the normed latent [T, R] and the one
    rotated key part [T, dr]."""
    R, dr = m["kv_rank"], m["rot_dim"]
    ckv = h @ w[prefix + ".mix.dkv"].T
    c = t_rms_norm(ckv[:, :R], w[prefix + ".mix.dkv.norm"], eps)
    r = t_rotate(ckv[:, R:R + dr], positions, m["rot"]["base"], m["rot"]["dims"])
    return c, r


def t_latent_attention(h, positions, w, prefix, m, eps, latent):
    """h [T, W] -> [T, W]. ``latent`` = (c, r) of this layer or of the layer it borrows from."""
    H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    c, r = latent
    cq = t_rms_norm(h @ w[prefix + ".mix.dq"].T, w[prefix + ".mix.dq.norm"], eps)
    q = (cq @ w[prefix + ".mix.uq"].T).reshape(T, H, dn + dr)
    q_n = q[..., :dn]
    q_r = t_rotate(q[..., dn:], positions, m["rot"]["base"], m["rot"]["dims"])
    k_n = (c @ w[prefix + ".mix.uk"].T).reshape(T, H, dn)
    v = (c @ w[prefix + ".mix.uv"].T).reshape(T, H, dv)
    s = (torch.einsum("thd,jhd->htj", q_n, k_n) + torch.einsum("thd,jd->htj", q_r, r)) * m["scale"]
    visible = positions[None, :] <= positions[:, None]                      # [t, j]
    s = s.masked_fill(~visible[None], -math.inf)
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("htj,jhd->thd", p, v)
    gate = torch.sigmoid(h @ w[prefix + ".mix.g"].T)                         # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * dv) @ w[prefix + ".mix.o"].T


def t_silu(z):
    return z * torch.sigmoid(z)


def t_gated_ff(h, w, prefix):
    return (t_silu(h @ w[prefix + ".gate"].T) * (h @ w[prefix + ".up"].T)) @ w[prefix + ".down"].T


def t_table_moe(h, tokens, w, prefix, mlp):
    """Every token's experts come from a table row of its id; each weighs 1/top; a shared expert is added."""
    top = mlp["router"]["top"]
    table = w[prefix + ".table"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(top):
            e = int(table[int(tokens[t]), k])
            out[t] += t_gated_ff(h[t:t + 1], w, "%s.e%d" % (prefix, e))[0] / top
    if mlp.get("shared"):
        out = out + t_gated_ff(h, w, prefix + ".shared")
    return out


def t_feed_forward(h, tokens, w, prefix, mlp):
    if mlp["kind"] == "dense":
        return t_gated_ff(h, w, prefix)
    if mlp["kind"] == "moe":
        return t_table_moe(h, tokens, w, prefix, mlp)
    raise ValueError(mlp["kind"])


def t_depth_average(history, weights):
    """sum_j weights[j] * history[j]."""
    return sum(weights[j] * x for j, x in enumerate(history))


def t_forward(config, weights, tokens, dtype=torch.float32, return_layers=False):
    """Logits [T, V] of one whole sequence. With ``return_layers`` also the stream after every layer (after the
    depth average)."""
    w = {k: (v.to(dtype) if v.dtype.is_floating_point else v) for k, v in weights.items()}
    eps, groups = config["norm"]["eps"], config["norm"]["groups"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.shape[0])
    x = w["embed"][tokens]
    history = [x]
    latents = {}
    after = []
    for i, layer in enumerate(config["layers"]):
        p = "l%d" % i
        m = layer["mixer"]
        if layer["type"] != "latent_attention":
            raise ValueError(layer["type"])
        h = t_group_rms_norm(x, w[p + ".norm1"], eps, groups)
        if m.get("kv_from") is None:
            latents[i] = t_latent_kv(h, positions, w, p, m, eps)
            latent = latents[i]
        else:
            latent = latents[m["kv_from"]]
        a = t_latent_attention(h, positions, w, p, m, eps, latent)
        x = x + t_group_rms_norm(a, w[p + ".norm1b"], eps, groups)
        if layer.get("mlp") is not None:
            f = t_feed_forward(t_group_rms_norm(x, w[p + ".norm2"], eps, groups), tokens, w, p + ".mlp", layer["mlp"])
            x = x + t_group_rms_norm(f, w[p + ".norm2b"], eps, groups)
        history.append(x)
        x = t_depth_average(history, w[p + ".dwa"])
        after.append(x)
    logits = t_group_rms_norm(x, w["final.norm"], eps, groups) @ w["head"].T
    if return_layers:
        return logits, torch.stack(after)
    return logits
