"""Nogidra, the slow way: every mechanism of the design as one plain function over a whole sequence.

Double precision on the CPU, full score matrices, recurrences walked token by token, experts row by row.  Shares
nothing with the package: it is what the package's parts and kernels are held against.

A model is ``(config, weights)``: the config.json mapping and name -> tensor.  A layer's tensors start with
``l<i>.``; a mixer's with ``l<i>.mix.``, a feed-forward's with ``l<i>.mlp.``; linear weights are ``[out, in]``.
"""
import math

import torch

F = torch.float64


def unit_rms(x, eps):
    """x over its root mean square along the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """The layers' norm: the stored weight lies around zero and one is added to it."""
    return unit_rms(x, eps) * (1.0 + w)


def plain_norm(x, w, eps):
    return unit_rms(x, eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def short_convolution(u, taps_weight, bias=None):
    """y[t] = sum_j w[:, j] * u[t - taps + 1 + j] (+ bias): the last column meets the current token, and what lies
    before the sequence's start counts as zero.  ``u`` [steps, channels], ``taps_weight`` [channels, taps]."""
    steps, taps = u.shape[0], taps_weight.shape[1]
    out = torch.zeros_like(u)
    for t in range(steps):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += taps_weight[:, j] * u[s]
    return out if bias is None else out + bias


def angles(positions, dims, base):
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)
    return torch.tensor(positions, dtype=F)[:, None] * freq[None, :]


def rotate_halves(x, positions, dims, base):
    """x [steps, heads, size]: element i turns together with element i + dims/2; what lies beyond ``dims`` stays."""
    a = angles(positions, dims, base)
    cos, sin = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def rotate_neighbours(x, positions, dims, base):
    """x [steps, heads, size]: element 2i turns together with element 2i + 1; what lies beyond ``dims`` stays."""
    a = angles(positions, dims, base)
    cos, sin = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    turned = torch.stack([u * cos - v * sin, v * cos + u * sin], dim=-1).reshape(*x.shape[:-1], dims)
    return torch.cat([turned, x[..., dims:]], dim=-1)


def visible(steps, mask):
    """[i, j] true where position i sees position j: j <= i, and with a window i - j < size."""
    i, j = torch.arange(steps)[:, None], torch.arange(steps)[None, :]
    see = j <= i
    if mask:
        see = see & (i - j < int(mask["size"]))
    return see


def softmax_heads(q, k, v, scale, see, per_kv, bias=None):
    """q [steps, H, d], k [steps, G, d], v [steps, G, e]; query head h reads key/value head h // per_kv.
    ``bias`` [H, steps, steps] is taken off the scaled scores.  -> [steps, H, e]."""
    steps, heads = q.shape[0], q.shape[1]
    out = torch.zeros(steps, heads, v.shape[-1], dtype=F)
    for h in range(heads):
        g = h // per_kv
        score = (q[:, h] @ k[:, g].T) * scale
        if bias is not None:
            score = score - bias[h]
        out[:, h] = torch.softmax(score.masked_fill(~see, float("-inf")), dim=-1) @ v[:, g]
    return out


def distance_slopes(heads):
    return [2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)]


def query_temperature(positions, q_temp):
    """The factor on the queries of every position: 1 + coef * ln(floor((p + 1) / every) + 1)."""
    coef, every = float(q_temp["coef"]), int(q_temp["every"])
    return torch.tensor([1.0 + coef * math.log((p + 1) // every + 1) for p in positions], dtype=F)


def biased_attention(h, m, w, p):
    """The 'attention' mixer: q, k, v each through a short convolution of its own, no rotation, queries that grow
    with the position, scores lowered by slope * distance, a window, a sigmoid gate a head."""
    steps = h.shape[0]
    heads, kv_heads, dim, vdim = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    positions = list(range(steps))
    q, k, v = (h @ w[p + n].T for n in ("q", "k", "v"))
    if m.get("conv"):
        q, k, v = (short_convolution(u, w[p + n + ".conv"]) for u, n in ((q, "q"), (k, "k"), (v, "v")))
    if m.get("q_temp"):
        q = q * query_temperature(positions, m["q_temp"])[:, None]
    i, j = torch.arange(steps, dtype=F)[:, None], torch.arange(steps, dtype=F)[None, :]
    bias = torch.stack([s * (i - j) for s in distance_slopes(heads)])
    out = softmax_heads(q.view(steps, heads, dim), k.view(steps, kv_heads, dim), v.view(steps, kv_heads, vdim),
                        float(m["scale"]), visible(steps, m.get("mask")), heads // kv_heads, bias)
    out = out * torch.sigmoid(h @ w[p + "g"].T)[:, :, None]
    return out.reshape(steps, heads * vdim) @ w[p + "o"].T


def latent_attention(h, m, w, p, eps):
    """Keys and values out of one normed latent a token, plus one rotated key part that all heads share."""
    steps = h.shape[0]
    heads, dim, rot_dim, vdim, rank = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
    positions = list(range(steps))
    dims, base = int(m["rot"]["dims"]), float(m["rot"]["base"])
    q = (h @ w[p + "q"].T).view(steps, heads, dim + rot_dim)
    q_plain, q_turned = q[..., :dim], rotate_halves(q[..., dim:], positions, dims, base)
    down = h @ w[p + "dkv"].T
    latent = plain_norm(down[:, :rank], w[p + "dkv.norm"], eps)
    shared = rotate_halves(down[:, None, rank:], positions, dims, base)[:, 0]
    k_plain = (latent @ w[p + "uk"].T).view(steps, heads, dim)
    values = (latent @ w[p + "uv"].T).view(steps, heads, vdim)
    see = visible(steps, m.get("mask"))
    out = torch.zeros(steps, heads, vdim, dtype=F)
    for head in range(heads):
        score = (q_plain[:, head] @ k_plain[:, head].T + q_turned[:, head] @ shared.T) * float(m["scale"])
        out[:, head] = torch.softmax(score.masked_fill(~see, float("-inf")), dim=-1) @ values[:, head]
    return out.reshape(steps, heads * vdim) @ w[p + "o"].T


def wide_norm_attention(h, m, w, p, eps):
    """The left branch: projections with biases, q and k each normed over the whole projection (all heads at once),
    neighbouring pairs rotated on the first ``rot.dims`` elements of a head, a window."""
    steps = h.shape[0]
    heads, kv_heads, dim, vdim = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    positions = list(range(steps))
    q, k, v = (h @ w[p + n].T + w[p + n + ".b"] for n in ("q", "k", "v"))
    q = plain_norm(q, w[p + "q.norm"], eps).view(steps, heads, dim)
    k = plain_norm(k, w[p + "k.norm"], eps).view(steps, kv_heads, dim)
    dims, base = int(m["rot"]["dims"]), float(m["rot"]["base"])
    q, k = rotate_neighbours(q, positions, dims, base), rotate_neighbours(k, positions, dims, base)
    out = softmax_heads(q, k, v.view(steps, kv_heads, vdim), float(m["scale"]), visible(steps, m.get("mask")),
                        heads // kv_heads)
    return out.reshape(steps, heads * vdim) @ w[p + "o"].T


def state_space(h, m, w, p, eps):
    """The right branch (Mamba-2): per head S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x, from S = 0;
    y times silu(z), normed in equal parts, output projection."""
    steps = h.shape[0]
    heads, vdim, n, groups, parts = (int(m[k]) for k in ("heads", "vdim", "state", "groups", "norm_groups"))
    inner = heads * vdim
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * groups * n], proj[:, 2 * inner + 2 * groups * n:]
    xbc = silu(short_convolution(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].view(steps, heads, vdim)
    B = xbc[:, inner:inner + groups * n].view(steps, groups, n)
    C = xbc[:, inner + groups * n:].view(steps, groups, n)
    dt = softplus(dt + w[p + "dt_bias"])
    rate = torch.exp(w[p + "A_log"])
    S = torch.zeros(heads, n, vdim, dtype=F)
    y = torch.zeros(steps, heads, vdim, dtype=F)
    for t in range(steps):
        for head in range(heads):
            g = head // (heads // groups)
            S[head] = torch.exp(-rate[head] * dt[t, head]) * S[head] + dt[t, head] * torch.outer(B[t, g], x[t, head])
            y[t, head] = S[head].T @ C[t, g] + w[p + "D"][head] * x[t, head]
    y = y.reshape(steps, inner) * silu(z)
    y = unit_rms(y.view(steps, parts, inner // parts), eps).reshape(steps, inner) * w[p + "norm"]
    return y @ w[p + "o"].T


def side_by_side(h, m, w, p, eps):
    return float(m["left_scale"]) * wide_norm_attention(h, m["left"], w, p + "left.", eps) + \
        float(m["right_scale"]) * state_space(h, m["right"], w, p + "right.", eps)


def dense_feed_forward(h, w, p):
    return (silu(h @ w[p + "gate"].T + w[p + "gate.b"]) * (h @ w[p + "up"].T + w[p + "up.b"])) @ w[p + "down"].T + w[p + "down.b"]


def expert(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, router, top):
    """For every row the experts with the largest router outputs, weighted by the softmax over those alone."""
    logits = h @ router.T
    best = torch.topk(logits, top, dim=-1)
    return best.indices, torch.softmax(best.values, dim=-1)


def mixture(h, mlp, w, p):
    chosen, weight = route(h, w[p + "router"], int(mlp["router"]["top"]))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weight[t]):
            out[t] += a * expert(h[t:t + 1], w, f"{p}e{e}.")[0]
    return out


def mixer(kind, h, m, w, p, eps):
    if kind == "attention":
        return biased_attention(h, m, w, p)
    if kind == "latent_attention":
        return latent_attention(h, m, w, p, eps)
    if kind == "parallel":
        return side_by_side(h, m, w, p, eps)
    raise ValueError(f"unknown layer type {kind!r}")


def forward(config, weights, tokens, layers_out=None):
    """Logits [steps, vocab] of one sequence from position 0; ``layers_out`` (a list) receives the stream after
    every layer."""
    w = {k: v.to(F) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        x = x + mixer(layer["type"], offset_norm(x, w[p + "norm1"], eps), layer["mixer"], w, p + "mix.", eps)
        mlp = layer.get("mlp")
        if mlp:
            h = offset_norm(x, w[p + "norm2"], eps)
            x = x + (mixture(h, mlp, w, p + "mlp.") if mlp["kind"] == "moe" else dense_feed_forward(h, w, p + "mlp."))
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = offset_norm(x, w["final.norm"], eps) @ w["head"].T
    cap = config.get("logit_softcap")
    return float(cap) * torch.tanh(logits / float(cap)) if cap else logits
