"""Fosulix, the slow way: every mechanism of the design as one plain function over a whole sequence.

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


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def input_convolution(h, taps_weight):
    """h + conv(h): conv(h)[t] = sum_j w[:, j] * h[t - taps + 1 + j], zeros before the sequence's start.
    ``h`` [steps, width], ``taps_weight`` [width, taps]."""
    steps, taps = h.shape[0], taps_weight.shape[1]
    out = h.clone()
    for t in range(steps):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += taps_weight[:, j] * h[s]
    return out


def rotary_frequencies(dims, base, scaling=None):
    """The frequency of every pair and the factor on cos and sin.  With ``scaling`` (factor, original, fast, slow):
    pairs that turn often within the original length keep their frequency, pairs that turn rarely are slowed by
    ``factor``, a linear ramp over the pair index between; cos and sin grow by 0.1 ln(factor) + 1."""
    freq = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return freq, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pair_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
    out = []
    for i, f in enumerate(freq):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_adjacent(x, positions, rot):
    """x [steps, heads, size]: elements 2i and 2i+1 (below rot.dims) turn together by position * frequency_i;
    elements from ``dims`` on are left alone."""
    dims = int(rot["dims"])
    freq, grow = rotary_frequencies(dims, float(rot["base"]), rot.get("scaling"))
    angle = torch.tensor(positions, dtype=F)[:, None] * torch.tensor(freq, dtype=F)[None, :]
    cos, sin = (torch.cos(angle) * grow)[:, None, :], (torch.sin(angle) * grow)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    turned = torch.stack([u * cos - v * sin, v * cos + u * sin], dim=-1).reshape(*x.shape[:-1], dims)
    return torch.cat([turned, x[..., dims:]], dim=-1)


def latent_keys(h, m, w, p, eps, positions):
    """What a latent-attention layer caches: the normed latent [steps, kv_rank] and the rotated key part
    [steps, rot_dim] that all heads share."""
    rank = int(m["kv_rank"])
    down = h @ w[p + "dkv"].T
    latent = rms_norm(down[:, :rank], w[p + "dkv.norm"], eps)
    shared = rotate_adjacent(down[:, None, rank:], positions, m["rot"])[:, 0]
    return latent, shared


def latent_attention(h, m, w, p, eps, positions, cached):
    """The mixer on input ``h`` [steps, width]; ``cached`` = (latent, rotated key part), its own or another layer's."""
    steps = h.shape[0]
    heads, dim, rot_dim, vdim = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    q = (rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps) @ w[p + "uq"].T).view(steps, heads, dim + rot_dim)
    q_plain, q_turned = q[..., :dim], rotate_adjacent(q[..., dim:], positions, m["rot"])
    latent, shared = cached
    k_plain = (latent @ w[p + "uk"].T).view(steps, heads, dim)
    values = (latent @ w[p + "uv"].T).view(steps, heads, vdim)
    i, j = torch.arange(steps)[:, None], torch.arange(steps)[None, :]
    see = (j <= i) & (i - j < int(m["mask"]["size"])) if m.get("mask") else (j <= i)
    out = torch.zeros(steps, heads, vdim, dtype=F)
    for head in range(heads):
        score = (q_plain[:, head] @ k_plain[:, head].T + q_turned[:, head] @ shared.T) * float(m["scale"])
        out[:, head] = torch.softmax(score.masked_fill(~see, float("-inf")), dim=-1) @ values[:, head]
    return out.reshape(steps, heads * vdim) @ w[p + "o"].T


def forget_gate(h, w, p):
    """Per head and key channel: lower + (1 - lower) * sigmoid(W_f h + b)."""
    lower = w[p + "lower"]
    return lower + (1.0 - lower) * torch.sigmoid(h @ w[p + "f"].T + w[p + "f.b"])


def gated_memory(h, m, w, p, eps):
    """Linear attention whose forget gate also says what is written: per head S <- diag(f) S + (1 - f) v^T,
    o = S^T q, from S = 0; o over its root mean square times a gain shared by the heads; output projection."""
    steps = h.shape[0]
    heads, dim, vdim = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    pre = h @ w[p + "q"].T
    q = (pre * torch.sigmoid(pre)).view(steps, heads, dim)
    f = forget_gate(h, w, p).view(steps, heads, dim)
    v = (h @ w[p + "v"].T).view(steps, heads, vdim)
    S = torch.zeros(heads, dim, vdim, dtype=F)
    out = torch.zeros(steps, heads, vdim, dtype=F)
    for t in range(steps):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return rms_norm(out, w[p + "norm"], eps).reshape(steps, heads * vdim) @ w[p + "o"].T


def expert(h, w, p, limit):
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def route(h, router, r):
    """For every row: the chosen experts and their weights.  Scores sigmoid(router h); experts in equal groups of
    neighbours, a group's score the sum of its two best scores, only the best groups stay open; the best open
    scores win and weigh in with their score times the router's scale."""
    total, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(h @ router.T)
    choice = s.clone()
    groups = r.get("groups")
    if groups and int(groups["count"]) > 1:
        count, keep = int(groups["count"]), int(groups["keep"])
        size = total // count
        grouped = choice.view(-1, count, size)
        group_score = torch.topk(grouped, min(2, size), dim=-1).values.sum(dim=-1)
        kept = torch.topk(group_score, keep, dim=-1).indices
        allowed = torch.zeros_like(group_score, dtype=torch.bool).scatter_(1, kept, True)
        allowed = allowed[:, :, None].expand(-1, -1, size).reshape(-1, total)
        choice = choice.masked_fill(~allowed, float("-inf"))
    chosen = torch.topk(choice, top, dim=-1).indices
    return chosen, torch.gather(s, 1, chosen) * float(r["scale"])


def mixture(h, mlp, w, p):
    chosen, weight = route(h, w[p + "router"], mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weight[t]):
            out[t] += a * expert(h[t:t + 1], w, f"{p}e{e}.", float(mlp["expert"]["limit"]))[0]
    return out


def forward(config, weights, tokens, layers_out=None):
    """Logits [steps, vocab] of one sequence from position 0; ``layers_out`` (a list) receives the stream
    after every layer (after the average over depth)."""
    w = {k: v.to(F) for k, v in weights.items()}
    eps, mult = float(config["norm"]["eps"]), float(config["residual_mult"])
    positions = list(range(len(tokens)))
    x = w["embed"][torch.tensor(tokens)] * float(config["embedding"]["scale"])
    results = [x]                                   # the embedding output, then every layer's own result
    caches = {}
    for i, layer in enumerate(config["layers"]):
        m, p = layer["mixer"], f"l{i}."
        h = input_convolution(rms_norm(x, w[p + "norm1"], eps), w[p + "canon1"])
        if layer["type"] == "latent_attention":
            source = m.get("kv_from")
            if source is None:
                caches[i] = latent_keys(h, m, w, p + "mix.", eps, positions)
            mixed = latent_attention(h, m, w, p + "mix.", eps, positions, caches[i if source is None else int(source)])
        elif layer["type"] == "hgrn2":
            mixed = gated_memory(h, m, w, p + "mix.", eps)
        else:
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        x = x + mult * mixed
        if layer.get("mlp"):
            x = x + mult * mixture(rms_norm(x, w[p + "norm2"], eps), layer["mlp"], w, p + "mlp.")
        results.append(x)
        x = sum(w[p + "dwa"][j] * results[j] for j in range(len(results)))
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T
