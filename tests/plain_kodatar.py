"""A plain, slow Kodatar in float64: whole sequences, no cache, one function per mechanism.

It shares no code with the package: configuration is read from the config.json dictionary as it
is, tensors by their checkpoint names.  Notation: x the residual stream [T, width], p the position
of a token in its sequence (from 0), H query heads on G key/value heads.
"""

import math

import torch

F64 = torch.float64


def layer_norm(x, scale, shift, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * scale + shift


def unit_rms(x, scale, eps):
    """x over its root mean square (eps inside the root), times a scale over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * scale


def frequencies(rot):
    """f_i = base^(-2i/dims), i < dims/2; with `scaling`, long wavelengths are slowed by `factor`, short
    ones kept, and those between original/high and original/low blended linearly in original/wavelength."""
    dims = rot["dims"]
    out = []
    for i in range(dims // 2):
        f = rot["base"] ** (-2.0 * i / dims)
        s = rot.get("scaling")
        if s:
            wavelength = 2.0 * math.pi / f
            if wavelength > s["original"] / s["low"]:
                f = f / s["factor"]
            elif wavelength >= s["original"] / s["high"]:
                t = (s["original"] / wavelength - s["low"]) / (s["high"] - s["low"])
                f = (1.0 - t) * f / s["factor"] + t * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def turn(x, positions, rot):
    """x [T, heads, dim]: channel i < dims/2 and channel i + dims/2 of every head form a pair that is
    rotated by the angle p * f_i; channels from dims on stay."""
    if not rot or not rot.get("dims"):
        return x
    dims, half = rot["dims"], rot["dims"] // 2
    angle = positions.to(F64)[:, None] * frequencies(rot)[None, :]            # [T, half]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    first, second = x[..., :half], x[..., half:dims]
    return torch.cat([first * cos - second * sin, second * cos + first * sin, x[..., dims:]], dim=-1)


def visible(positions, mask):
    """[T, T] bool: query i sees key j if j <= i and, with a chunk size, both lie in the same chunk
    counted from position 0."""
    i, j = positions[:, None], positions[None, :]
    seen = j <= i
    if mask and mask.get("size"):
        seen = seen & (torch.div(i, mask["size"], rounding_mode="floor") == torch.div(j, mask["size"], rounding_mode="floor"))
    return seen


def attention(h, w, prefix, sizes, eps):
    T = h.shape[0]
    H, G, D, V = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    positions = torch.arange(T)
    q = (h @ w[prefix + "q"].T).view(T, H, D)
    k = (h @ w[prefix + "k"].T).view(T, G, D)
    v = (h @ w[prefix + "v"].T).view(T, G, V)
    q = turn(unit_rms(q, w[prefix + "q.norm"], eps), positions, sizes.get("rot"))
    k = turn(unit_rms(k, w[prefix + "k.norm"], eps), positions, sizes.get("rot"))
    seen = visible(positions, sizes.get("mask"))
    out = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        shared = head // (H // G)
        scores = (q[:, head] @ k[:, shared].T) * sizes["scale"]
        scores = scores.masked_fill(~seen, float("-inf"))
        out[:, head] = torch.softmax(scores, dim=-1) @ v[:, shared]
    return out.reshape(T, H * V) @ w[prefix + "o"].T


def gated_expert(h, w, prefix):
    gate, up = h @ w[prefix + "gate"].T, h @ w[prefix + "up"].T
    return (gate * torch.sigmoid(gate) * up) @ w[prefix + "down"].T


def route(h, w, prefix, router):
    """(chosen [T, top], weights [T, top]): softmax over all router outputs; the choice is made on
    score + correction among the experts of the best `keep` groups (a group's rank is its best
    corrected score), the weights are the plain scores of the chosen, normalised to sum one."""
    scores = torch.softmax(h @ w[prefix + "router"].T, dim=-1)
    ranked = scores + w[prefix + "correction"]
    groups = router.get("groups")
    if groups:
        T, n = ranked.shape
        per = n // groups["count"]
        best = ranked.view(T, groups["count"], per).max(-1).values
        shut = torch.ones(T, groups["count"], dtype=torch.bool)
        shut.scatter_(1, best.topk(groups["keep"], dim=-1).indices, False)
        ranked = ranked.masked_fill(shut[:, :, None].expand(T, groups["count"], per).reshape(T, n), float("-inf"))
    chosen = ranked.topk(router["top"], dim=-1).indices
    weights = scores.gather(1, chosen)
    return chosen, weights / (weights.sum(-1, keepdim=True) + 1e-20)


def experts(h, w, prefix, mlp):
    router = mlp["router"]
    chosen, weights = route(h, w, prefix, router)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, weight in zip(chosen[t].tolist(), weights[t]):
            if e >= router["experts"]:                       # an identity expert: its output is its input
                out[t] += weight * h[t]
            else:
                out[t] += weight * gated_expert(h[t:t + 1], w, f"{prefix}e{e}.")[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ w[prefix + "shared.sg"].T) * gated_expert(h, w, prefix + "shared.")
    return out


def layer(x, w, index, entry, eps):
    p = f"l{index}."
    norm = lambda name, v: layer_norm(v, w[p + name], w[p + name + ".b"], eps)
    x = x + norm("norm1b", attention(norm("norm1", x), w, p + "mix.", entry["mixer"], eps))
    if entry.get("mlp"):
        x = x + norm("norm2b", experts(norm("norm2", x), w, p + "mlp.", entry["mlp"]))
    return x


def order_of_runs(config):
    """[(layer, number of the pass it opens or None)]."""
    n, loop = len(config["layers"]), config.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for number in range(loop["times"]):
        runs += [(i, number if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n)]


def forward(ids, weights, config, residuals=None):
    """float64 logits [T, vocab] of one sequence; ``residuals``: a list that receives x after every run of a layer."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    x0 = w["embed"][torch.tensor(ids)] * config["embedding"]["scale"]
    x = x0
    for index, opens in order_of_runs(config):
        if opens is not None:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T + w["loop.step"][opens]
        x = layer(x, w, index, config["layers"][index], eps)
        if residuals is not None:
            residuals.append(x)
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return x @ w["embed"].T * config["logit_scale"]


def greedy(ids, weights, config, new_tokens):
    ids, out = list(ids), []
    for _ in range(new_tokens):
        out.append(int(forward(ids, weights, config)[-1].argmax()))
        ids.append(out[-1])
    return out
