"""Plain, slow Salopel used only as the oracle of the tests.

Whole sequences, no cache, one sequence at a time, one function per mechanism, written from the
design's equations and sharing no code with the product path.  Weights are a dict of torch
tensors under the checkpoint's own names (linear maps stored [out, in]).  Everything is evaluated
in ``dtype`` (float64 unless asked otherwise); recurrences run token by token.

Notation: h [T, width] is a sublayer's input, rms(v) = sqrt(mean(v^2) + eps) over the last axis.
"""

import math

import torch


def rms(v, eps):
    return torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    """x / rms(x) * (1 + w): the scale is stored as its distance from one."""
    return x / rms(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    """x / rms(x) * w."""
    return x / rms(x, eps) * w


def silu(v):
    return v * torch.sigmoid(v)


def softplus(v):
    return torch.where(v > 30.0, v, torch.log1p(torch.exp(torch.clamp(v, max=30.0))))


def causal_conv(u, taps, bias):
    """out[t, c] = bias[c] + sum_j taps[c, j] * u[t - (J - 1 - j), c]: the last column of ``taps``
    meets the current token, inputs before the sequence are zeros.  u [T, C], taps [C, J]."""
    tokens, channels = u.shape
    width = taps.shape[1]
    padded = torch.cat([u.new_zeros(width - 1, channels), u])
    out = bias.expand(tokens, channels).clone()
    for j in range(width):
        out = out + padded[j:j + tokens] * taps[:, j]
    return out


def poly_norm(z, coefficients, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e with N(v) = v / rms(v) over a token's whole vector."""
    a, b, c, e = [coefficients[i] for i in range(4)]
    unit = lambda v: v / rms(v, eps)
    return a * unit(z) + b * unit(z * z) + c * unit(z * z * z) + e


def feed_forward(h, w, prefix, eps):
    return poly_norm(h @ w[prefix + "up"].T, w[prefix + "act"], eps) @ w[prefix + "down"].T


def latent_attention(h, w, prefix, sizes, eps):
    """Queries and keys/values both come through a normalised low-rank latent; no positions."""
    heads, dim, vdim, scale = sizes["heads"], sizes["dim"], sizes["vdim"], sizes["scale"]
    tokens = h.shape[0]
    c_q = norm_plain(h @ w[prefix + "dq"].T, w[prefix + "dq.norm"], eps)
    q = (c_q @ w[prefix + "uq"].T).reshape(tokens, heads, dim)
    c = norm_plain(h @ w[prefix + "dkv"].T, w[prefix + "dkv.norm"], eps)
    k = (c @ w[prefix + "uk"].T).reshape(tokens, heads, dim)
    v = (c @ w[prefix + "uv"].T).reshape(tokens, heads, vdim)
    scores = torch.einsum("ihd,jhd->hij", q, k) * scale
    future = torch.arange(tokens).unsqueeze(0) > torch.arange(tokens).unsqueeze(1)
    scores = scores.masked_fill(future.unsqueeze(0), float("-inf"))
    weights = torch.softmax(scores, dim=-1)
    mixed = torch.einsum("hij,jhd->ihd", weights, v).reshape(tokens, heads * vdim)
    gate = torch.sigmoid(h @ w[prefix + "g"].T)
    return (mixed * gate) @ w[prefix + "o"].T


def mamba1(h, w, prefix, sizes):
    """Selective scan, one state row per channel: S[c, :] <- exp(dt_c A[c, :]) S[c, :] + dt_c x_c B,
    y_c = S[c, :] . C + D_c x_c."""
    inner, state, dt_rank = sizes["inner"], sizes["state"], sizes["dt_rank"]
    tokens = h.shape[0]
    xz = h @ w[prefix + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, w[prefix + "conv"], w[prefix + "conv.b"]))
    low = x @ w[prefix + "x"].T
    dt_low, B, C = low[:, :dt_rank], low[:, dt_rank:dt_rank + state], low[:, dt_rank + state:]
    dt = softplus(dt_low @ w[prefix + "dt"].T + w[prefix + "dt.b"])
    A = -torch.exp(w[prefix + "A_log"])
    S = h.new_zeros(inner, state)
    ys = []
    for t in range(tokens):
        S = torch.exp(dt[t].unsqueeze(1) * A) * S + (dt[t] * x[t]).unsqueeze(1) * B[t].unsqueeze(0)
        ys.append(S @ C[t] + w[prefix + "D"] * x[t])
    y = torch.stack(ys)
    return (y * silu(z)) @ w[prefix + "o"].T


def mamba2(h, w, prefix, sizes, eps):
    """One decay per head: S_h <- exp(-exp(A_log_h) dt_h) S_h + dt_h B x^T (S_h is [state, vdim]),
    y = S_h^T C + D_h x; gate, then a norm in equal parts."""
    heads, vdim, state, groups = sizes["heads"], sizes["vdim"], sizes["state"], sizes["groups"]
    parts = sizes["norm_groups"]
    inner, gn = heads * vdim, groups * state
    tokens = h.shape[0]
    proj = h @ w[prefix + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * gn], proj[:, 2 * inner + 2 * gn:]
    xbc = silu(causal_conv(xbc, w[prefix + "conv"], w[prefix + "conv.b"]))
    x = xbc[:, :inner].reshape(tokens, heads, vdim)
    B = xbc[:, inner:inner + gn].reshape(tokens, groups, state)
    C = xbc[:, inner + gn:].reshape(tokens, groups, state)
    dt = softplus(dt + w[prefix + "dt_bias"])
    decay_rate = torch.exp(w[prefix + "A_log"])
    per_group = heads // groups
    S = h.new_zeros(heads, state, vdim)
    ys = []
    for t in range(tokens):
        row = []
        for head in range(heads):
            g = head // per_group
            S[head] = math.exp(-float(decay_rate[head]) * float(dt[t, head])) * S[head] \
                + dt[t, head] * B[t, g].unsqueeze(1) * x[t, head].unsqueeze(0)
            row.append(S[head].T @ C[t, g] + w[prefix + "D"][head] * x[t, head])
        ys.append(torch.cat(row))
    y = torch.stack(ys) * silu(z)
    y = y.reshape(tokens, parts, inner // parts)
    y = (y / rms(y, eps)).reshape(tokens, inner) * w[prefix + "norm"]
    return y @ w[prefix + "o"].T


def mixer(h, w, layer, entry, eps):
    prefix = f"l{layer}.mix."
    if entry["type"] == "latent_attention":
        return latent_attention(h, w, prefix, entry["mixer"], eps)
    if entry["type"] == "mamba1":
        return mamba1(h, w, prefix, entry["mixer"])
    if entry["type"] == "mamba2":
        return mamba2(h, w, prefix, entry["mixer"], eps)
    raise ValueError(entry["type"])


def forward(ids, weights, config, dtype=torch.float64, layers_out=None):
    """Logits [len(ids), vocab] of one sequence that starts at position 0.  ``layers_out``: a list
    that receives the residual stream after every layer run."""
    w = {k: v.to(dtype) for k, v in weights.items()}
    eps, mult = config["norm"]["eps"], config["residual_mult"]
    x = norm_around_zero(w["embed"][torch.as_tensor(ids, dtype=torch.long)], w["embed.norm"], eps)
    for index, entry in enumerate(config["layers"]):
        layer = index
        while config["layers"][layer].get("weights_of") is not None:      # a borrower runs its owner's tensors
            layer = config["layers"][layer]["weights_of"]
        x = x + mult * norm_around_zero(mixer(x, w, layer, entry, eps), w[f"l{layer}.norm1"], eps)
        if entry.get("mlp") is not None:
            x = x + mult * norm_around_zero(feed_forward(x, w, f"l{layer}.mlp.", eps), w[f"l{layer}.norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = norm_around_zero(x, w["final.norm"], eps)
    return x @ w["embed"].T


def greedy(ids, weights, config, steps, dtype=torch.float64):
    """Greedy continuation: the whole sequence is recomputed for every new token; ties go to the
    lowest index."""
    ids, out = list(ids), []
    for _ in range(steps):
        token = int(torch.argmax(forward(ids, weights, config, dtype)[-1]))
        out.append(token)
        ids.append(token)
    return out
