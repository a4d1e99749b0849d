"""The kernels that came with Kodatar's mechanisms, each alone against float64: head norms with
rotation into the cache, the router, the gated experts' activation, the layer norm of a sublayer's
output, joined rows, the scaled embedding, and attention whose keys are seen in chunks (every
attention kernel, with one dominant key placed just inside and just outside a chunk)."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

from burn_transformers_amd.kernels import library as K  # noqa: E402
from kernel_helpers import PagedCase  # noqa: E402

DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def rel_err(got, want):
    got = got.detach().cpu().double()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,rot,norm", [(4, 2, 16, 32, 8, True), (3, 3, 24, 10, 24, True),
                                                              (6, 1, 8, 8, 0, True), (2, 2, 40, 48, 20, False),
                                                              (5, 5, 130, 70, 64, True)])
def test_head_norms_and_rotation_into_the_cache(dtype, heads, kv_heads, dim, vdim, rot, norm):
    dt = DTYPES[dtype]
    hd = (max(dim, vdim) + 15) // 16 * 16
    totals, counts = [70, 5, 131], [70, 2, 3]
    case = PagedCase(totals, counts, kv_heads, hd, dt, DEV, seed=1)
    gen = torch.Generator().manual_seed(2)
    cols = (heads + kv_heads) * dim + kv_heads * vdim
    fused = torch.randn(case.n_tokens, cols + 3, generator=gen)
    q_gamma, k_gamma = torch.randn(dim, generator=gen) + 1.0, torch.randn(dim, generator=gen) + 1.0
    inv_freq = (1000.0 ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / max(rot, 1))).float()
    q_out = torch.full((case.n_tokens, heads * hd), float("nan"), dtype=dt, device=DEV)
    K.head_rotary(fused.to(DEV)[:, :cols], heads, kv_heads, dim, vdim, rot, inv_freq.to(DEV) if rot else None,
                  q_gamma.to(DEV) if norm else None, k_gamma.to(DEV) if norm else None, 1e-3, q_out,
                  case.tok_seq, case.tok_pos, case.view(), dt)
    x = fused.double()
    pos = case.tok_pos.cpu().double()

    def heads_of(first, count, size, gamma):
        rows = x[:, first:first + count * size].reshape(-1, count, size)
        if gamma is not None and norm:
            rows = rows / torch.sqrt((rows * rows).mean(-1, keepdim=True) + 1e-3) * gamma.double()
        if gamma is not None and rot:
            half = rot // 2
            angle = (pos[:, None].float() * inv_freq[None, :]).double()          # the angle itself is a 32-bit product
            cos, sin = torch.cos(angle)[:, None], torch.sin(angle)[:, None]
            a, b = rows[..., :half], rows[..., half:rot]
            rows = torch.cat([a * cos - b * sin, b * cos + a * sin, rows[..., rot:]], dim=-1)
        out = torch.zeros(rows.shape[0], count, hd, dtype=torch.float64)
        out[..., :size] = rows
        return out.reshape(rows.shape[0], count * hd)

    bound = 2e-6 if dtype == "float32" else 6e-3
    assert rel_err(q_out, heads_of(0, heads, dim, q_gamma)) < bound
    k_all, v_all = case.read_back()
    step_rows = []
    at = 0
    for total, count in zip(totals, counts):
        step_rows += list(range(at + total - count, at + total))
        at += total
    assert rel_err(k_all[step_rows], heads_of(heads * dim, kv_heads, dim, k_gamma)) < bound
    assert rel_err(v_all[step_rows], heads_of((heads + kv_heads) * dim, kv_heads, vdim, None)) < bound


def plain_route(h, router, correction, top, groups, keep):
    scores = torch.softmax(h.double() @ router.double().T, dim=-1)
    ranked = scores + (correction.double() if correction is not None else 0.0)
    rows, n = ranked.shape
    if groups > 1:
        per = n // groups
        best = ranked.view(rows, groups, per).max(-1).values
        shut = torch.ones(rows, groups, dtype=torch.bool)
        shut.scatter_(1, best.topk(keep, dim=-1).indices, False)
        ranked = ranked.masked_fill(shut[:, :, None].expand(rows, groups, per).reshape(rows, n), float("-inf"))
    chosen = ranked.topk(top, dim=-1).indices
    weights = torch.zeros(rows, n, dtype=torch.float64)
    picked = scores.gather(1, chosen)
    weights.scatter_(1, chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20))
    return weights


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("experts,top,groups,keep,width", [(8, 3, 4, 2, 64), (5, 1, 1, 1, 40), (4, 4, 2, 2, 32),
                                                           (12, 3, 3, 1, 96), (64, 6, 8, 3, 128), (7, 2, 0, 0, 24)])
def test_router(dtype, experts, top, groups, keep, width):
    dt = DTYPES[dtype]
    gen = torch.Generator().manual_seed(experts)
    h = torch.randn(37, width, generator=gen).to(dt)
    router = torch.randn(experts, width, generator=gen) * (2.0 / math.sqrt(width))
    correction = torch.randn(experts, generator=gen) * 0.3 - 0.4            # corrected scores are mostly negative
    gate_w = torch.randn(width, generator=gen) / math.sqrt(width)
    weights = torch.full((37, experts), float("nan"), device=DEV)
    gate = torch.full((37, 1), float("nan"), device=DEV)
    K.route(h.to(DEV), router.to(DEV), correction.to(DEV), top, groups, keep, weights, gate_w.to(DEV), gate)
    want = plain_route(h.float(), router, correction, top, groups, keep)
    assert torch.equal(weights.cpu() != 0, want != 0), "another expert was chosen"
    assert float((weights.cpu().double() - want).abs().max()) < 2e-6
    assert float((gate.cpu().double()[:, 0] - torch.sigmoid(h.double() @ gate_w.double())).abs().max()) < 2e-6


def test_router_shuts_groups_out_and_corrections_only_choose():
    """Made so that each rule shows: the best single expert sits in a group that loses (its group's
    best corrected score is lower than two other groups'), a correction lifts an expert into the
    choice without entering its weight, and shut-out experts stay out although every open expert's
    corrected score is negative."""
    width, experts = 8, 6                      # three groups of two, two stay open
    h = torch.zeros(1, width)
    h[0, 0] = 1.0
    router = torch.zeros(experts, width)
    router[:, 0] = torch.tensor([2.0, 0.0, 1.0, 0.5, 1.5, 1.4])
    correction = torch.tensor([-5.0, -5.0, -1.0, -1.3, -1.2, -1.2])
    weights = torch.empty(1, experts, device=DEV)
    K.route(h.to(DEV), router.to(DEV), correction.to(DEV), 3, 3, 2, weights)
    scores = torch.softmax(router[:, 0].double(), 0)
    chosen = [2, 4, 5]                         # expert 0 has the best score but its group is shut; 3 loses to 4 and 5
    want = torch.zeros(experts, dtype=torch.float64)
    want[chosen] = scores[chosen] / scores[chosen].sum()
    assert float((weights.cpu().double()[0] - want).abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("experts,ff,shared,identity", [(4, 8, 16, 2), (3, 5, 0, 0), (6, 12, 7, 1)])
def test_gated_experts_activation(dtype, experts, ff, shared, identity):
    dt = DTYPES[dtype]
    gen = torch.Generator().manual_seed(ff)
    rows, width = 19, 24
    inner = experts * ff + shared
    gu = torch.randn(rows, 2 * inner, generator=gen).to(dt)
    h = torch.randn(rows, width, generator=gen).to(dt)
    weights = torch.rand(rows, experts + identity, generator=gen)
    weights[torch.rand(rows, experts + identity, generator=gen) < 0.5] = 0.0
    gate = torch.rand(rows, 1, generator=gen)
    cols = (inner + 7) // 8 * 8
    hidden = torch.full((rows, cols), float("nan"), dtype=dt, device=DEV)
    identity_out = torch.full((rows, width), float("nan"), device=DEV) if identity else None
    K.gated_experts(gu.to(DEV), weights.to(DEV), gate.to(DEV) if shared else None, experts, ff, shared, identity, hidden,
                    h=h.to(DEV) if identity else None, identity_out=identity_out)
    g = gu.double()
    want = torch.zeros(rows, cols, dtype=torch.float64)
    for e in range(experts):
        a, b = g[:, 2 * e * ff:2 * e * ff + ff], g[:, 2 * e * ff + ff:2 * (e + 1) * ff]
        want[:, e * ff:(e + 1) * ff] = weights[:, e:e + 1].double() * a * torch.sigmoid(a) * b
    if shared:
        a, b = g[:, 2 * experts * ff:2 * experts * ff + shared], g[:, 2 * experts * ff + shared:]
        want[:, experts * ff:inner] = gate.double() * a * torch.sigmoid(a) * b
    assert rel_err(hidden, want) < (2e-6 if dtype == "float32" else 5e-3)
    if identity:
        total = weights[:, experts:].double().sum(-1, keepdim=True)
        assert rel_err(identity_out, total * h.double()) < 2e-6


@pytest.mark.parametrize("rows", [9, 70])          # a wave a row up to 64 rows, a work-group a row beyond
@pytest.mark.parametrize("width", [40, 256, 1500, 2600])
@pytest.mark.parametrize("kind", ["layer_norm", "rms_norm"])
def test_norm_of_a_sublayers_output(width, kind, rows):
    gen = torch.Generator().manual_seed(width)
    x = torch.randn(rows, width, generator=gen)
    delta = torch.randn(3, rows, width, generator=gen) + 0.7
    bias = torch.randn(width, generator=gen)
    gamma, beta = torch.randn(width, generator=gen), torch.randn(width, generator=gen)
    stream = x.clone().to(DEV)
    K.output_norm(stream, gamma.to(DEV), 1e-4, 0.8, delta=delta.to(DEV), bias=bias.to(DEV), kind=kind,
                  beta=beta.to(DEV) if kind == "layer_norm" else None)
    v = delta.double().sum(0) + bias.double()
    if kind == "layer_norm":
        mean = v.mean(-1, keepdim=True)
        normed = (v - mean) / torch.sqrt(((v - mean) ** 2).mean(-1, keepdim=True) + 1e-4) * gamma.double() + beta.double()
    else:
        normed = v / torch.sqrt((v * v).mean(-1, keepdim=True) + 1e-4) * gamma.double()
    assert rel_err(stream, x.double() + 0.8 * normed) < 3e-6
    # the same with the norm that reads the stream next done in the same pass
    for then_kind, dt in (("layer_norm", torch.float32), ("rms_norm", torch.bfloat16), ("layer_norm", torch.bfloat16)):
        stream = x.clone().to(DEV)
        out = torch.full((rows, width + 8), float("nan"), dtype=dt, device=DEV)[:, :width]
        g2, b2 = torch.randn(width, generator=gen), torch.randn(width, generator=gen)
        K.output_norm(stream, gamma.to(DEV), 1e-4, 0.8, delta=delta.to(DEV), bias=bias.to(DEV), kind=kind,
                      beta=beta.to(DEV) if kind == "layer_norm" else None,
                      then=(then_kind, g2.to(DEV), b2.to(DEV) if then_kind == "layer_norm" else None, 1e-3, out))
        y = x.double() + 0.8 * normed
        assert rel_err(stream, y) < 3e-6
        if then_kind == "layer_norm":
            mean = y.mean(-1, keepdim=True)
            want = (y - mean) / torch.sqrt(((y - mean) ** 2).mean(-1, keepdim=True) + 1e-3) * g2.double() + b2.double()
        else:
            want = y / torch.sqrt((y * y).mean(-1, keepdim=True) + 1e-3) * g2.double()
        assert rel_err(out, want) < (3e-6 if dt == torch.float32 else 5e-3)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_joined_rows_and_scaled_embedding(dtype):
    dt = DTYPES[dtype]
    gen = torch.Generator().manual_seed(3)
    x, y = torch.randn(13, 20, generator=gen), torch.randn(13, 20, generator=gen)
    out = torch.full((13, 48), float("nan"), dtype=dt, device=DEV)
    K.join_rows(x.to(DEV), y.to(DEV), out)
    want = torch.cat([x, y, torch.zeros(13, 8)], dim=1).to(dt)
    assert torch.equal(out.cpu(), want)
    table = torch.randn(50, 20, generator=gen).to(dt)
    ids = torch.randint(0, 50, (13,), generator=gen, dtype=torch.int32)
    rows, copy = torch.empty(13, 20, device=DEV), torch.empty(13, 20, device=DEV)
    K.embed(ids.to(DEV), None, table.to(DEV), None, rows, scale=3.5, copy=copy)
    assert torch.equal(rows.cpu(), table[ids.long()].float() * 3.5) and torch.equal(rows, copy)


def chunked_reference(case, q, q_heads, scale, chunk, window=0):
    """float64 attention of the step's queries over the keys of their own chunk (CPU)."""
    hd, group = case.head_dim, q_heads // case.kv_heads
    out = torch.zeros(case.n_tokens, q_heads * hd, dtype=torch.float64)
    q = q.detach().cpu().double()
    row = 0
    for s, (total, count) in enumerate(zip(case.totals, case.counts)):
        k = case.k_rows[s].double().view(total, case.kv_heads, hd)
        v = case.v_rows[s].double().view(total, case.kv_heads, hd)
        for i in range(count):
            pos = total - count + i
            lo = max(pos - pos % chunk, pos - window + 1 if window else 0)
            for h in range(q_heads):
                scores = (k[lo:pos + 1, h // group] @ q[row, h * hd:(h + 1) * hd]) * scale
                out[row, h * hd:(h + 1) * hd] = torch.softmax(scores, dim=0) @ v[lo:pos + 1, h // group]
            row += 1
    return out


IMPLS = {"float32": ["plain", "tiled"], "bfloat16": ["plain", "mfma"]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("q_heads,kv_heads,hd,chunk,window", [(4, 2, 32, 24, 0), (2, 2, 64, 64, 0), (3, 1, 48, 100, 0),
                                                              (2, 1, 128, 7, 0), (4, 4, 16, 200, 30), (2, 2, 64, 1, 0), (2, 1, 128, 448, 0), (4, 2, 48, 448, 0)])
def test_attention_in_chunks(dtype, q_heads, kv_heads, hd, chunk, window):
    """Prompts, portions that start inside a chunk, and single tokens, on every attention kernel."""
    dt = DTYPES[dtype]
    scale = 0.4 / math.sqrt(hd)
    for totals, counts in (([130, 5, 300], [130, 5, 300]), ([250, 64, 201], [50, 3, 200]), ([257, 24, 100, 449], [1, 1, 1, 1])) + \
            ((([940, 600], [940, 152]), ([940, 897], [1, 1])) if chunk > 150 else ()):
        case = PagedCase(totals, counts, kv_heads, hd, dt, DEV, seed=4, poison=True)
        gen = torch.Generator().manual_seed(7)
        q = torch.randn(case.n_tokens, q_heads * hd, generator=gen).to(dt).to(DEV)
        want = chunked_reference(case, q, q_heads, scale, chunk, window)
        for impl in IMPLS[dtype]:
            for decode in ([False, True] if max(counts) == 1 and impl != "plain" else [max(counts) == 1]):
                out = torch.full((case.n_tokens, q_heads * hd), float("nan"), dtype=dt, device=DEV)
                args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                                        q_heads, len(totals), max(counts), scale, window, chunk=chunk)
                K.attention(args, dt, decode=decode, impl=impl)
                assert rel_err(out, want) < (4e-6 if dtype == "float32" else 1.2e-2), (impl, decode, totals, counts)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("chunk", [48, 64, 96])
def test_one_dominant_key_just_inside_and_just_outside_a_chunk(dtype, chunk):
    """One key is made to take all the weight.  Placed at the first position of the query's chunk it
    must be found (the output is its value row); placed one position earlier it must not be seen at
    all (the output is what the chunk's own keys give)."""
    dt, hd, total = DTYPES[dtype], 64, 5 * chunk + 11
    start = total - 1 - (total - 1) % chunk                     # first position of the last query's chunk
    for target, found in ((start, True), (start - 1, False), (total - 1, True), (0, False)):
        for counts in ([1], [total - start + 5], [total]):
            case = PagedCase([total], counts, 1, hd, dt, DEV, seed=target)
            case.k_rows[0][:] *= 0.05
            case.k_rows[0][target, 3] = 8.0
            seq = torch.zeros(total, dtype=torch.int32, device=DEV)
            pos = torch.arange(total, dtype=torch.int32, device=DEV)
            K.kv_copy(case.k_rows[0].to(DEV), case.v_rows[0].to(DEV), seq, pos, case.view(), True)
            q = torch.zeros(case.n_tokens, hd)
            q[-1, 3] = 8.0                                       # the last query looks for the key; the others look nowhere
            q = q.to(dt).to(DEV)
            want = chunked_reference(case, q, 1, 1.0, chunk)
            hit = float((want[-1] - case.v_rows[0][target].double()).abs().max()) < 1e-3
            assert hit == found
            for impl in IMPLS[dtype]:
                out = torch.empty(case.n_tokens, hd, dtype=dt, device=DEV)
                args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                                        1, 1, max(counts), 1.0, 0, chunk=chunk)
                K.attention(args, dt, decode=max(counts) == 1, impl=impl)
                assert rel_err(out[-1:], want[-1:]) < (1e-5 if dtype == "float32" else 1e-2), (target, counts, impl)
