"""The kernels that Salopel's parts brought, each alone against the plain implementation's function
of the same mechanism, at sizes that divide nothing."""

import pytest
import torch

pytestmark = pytest.mark.gpu

import plain_salopel as plain  # noqa: E402
from burn_transformers_amd.kernels import library as K  # noqa: E402
from step_helpers import make_step  # noqa: E402

DEVICE = "cuda:0"


def rand(*shape, seed=0, scale=1.0):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_poly_norm(out_dtype):
    z = rand(7, 45, seed=1, scale=1.7)
    coefficients = torch.tensor([0.7, -0.3, 0.2, 0.05])
    padded = torch.zeros(7, 48)
    padded[:, :45] = z
    out = torch.full((7, 48), 9.0, dtype=out_dtype, device=DEVICE)
    K.poly_norm(padded.to(DEVICE), 45, coefficients.to(DEVICE), 1e-5, out)
    want = plain.poly_norm(z.double(), coefficients.double(), 1e-5)
    bound = 1e-5 if out_dtype == torch.float32 else 2e-2
    assert float((out[:, :45].cpu().double() - want).abs().max()) < bound
    assert float(out[:, 45:].float().abs().max()) == 0.0


def test_output_norm_adds_the_scaled_norm_of_partial_sums():
    x, parts, bias, gamma = rand(5, 37, seed=2), rand(3, 5, 37, seed=3), rand(37, seed=4), rand(37, seed=5)
    xd = x.to(DEVICE)
    cast = torch.full((5, 40), 7.0, dtype=torch.bfloat16, device=DEVICE)
    K.output_norm(xd, gamma.to(DEVICE), 1e-4, 0.6, delta=parts.to(DEVICE), bias=bias.to(DEVICE), cast=cast)
    v = parts.double().sum(0) + bias.double()
    want = x.double() + 0.6 * plain.norm_plain(v, gamma.double(), 1e-4)
    assert float((xd.cpu().double() - want).abs().max()) < 1e-5
    assert float((cast[:, :37].float().cpu().double() - want).abs().max()) < 3e-2
    assert float(cast[:, 37:].float().abs().max()) == 0.0
    K.output_norm(xd, gamma.to(DEVICE), 1e-4, 1.0, accumulate=False)          # the rows themselves, in place
    assert float((xd.cpu().double() - plain.norm_plain(want, gamma.double(), 1e-4)).abs().max()) < 1e-5


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_causal_conv_in_portions_of_two_sequences(taps):
    """Two sequences of different lengths in the same steps, each cut into portions, a portion shorter
    than the taps included; the state carries the inputs between the steps."""
    channels = 13
    weight, bias = rand(channels, taps, seed=6), rand(channels, seed=7)
    u = [rand(11, channels, seed=8), rand(6, channels, seed=9)]
    want = [plain.silu(plain.causal_conv(s.double(), weight.double(), bias.double())) for s in u]
    state = torch.zeros(4, max(1, (taps - 1) * channels) + 3, device=DEVICE)       # rows longer than needed: a pitch
    got = [[], []]
    cuts = [[(0, 1), (1, 3), (3, 11)], [(0, 2), (2, 3), (3, 6)]]
    for part in range(3):
        spans = [cuts[0][part], cuts[1][part]]
        counts = [b - a for a, b in spans]
        step = make_step(torch.float32, counts, starts=[a for a, _ in spans], slots=[2, 0])
        rows = torch.cat([u[i][a:b] for i, (a, b) in enumerate(spans)]).to(DEVICE)
        out = torch.empty(sum(counts), channels, device=DEVICE)
        cast = torch.full((sum(counts), 16), 5.0, dtype=torch.bfloat16, device=DEVICE)
        K.causal_conv(rows, weight.to(DEVICE), bias.to(DEVICE), out, state[:, :max(1, (taps - 1) * channels)], step, cast=cast)
        got[0].append(out[:counts[0]].cpu())
        got[1].append(out[counts[0]:].cpu())
        assert float(cast[:, channels:].float().abs().max()) == 0.0
        assert float((cast[:, :channels].float() - out).abs().max()) < 2e-2
    for i in range(2):
        assert float((torch.cat(got[i]).double() - want[i]).abs().max()) < 1e-5
    assert float(state[1].abs().max()) == 0.0 and float(state[3].abs().max()) == 0.0      # other slots untouched


def test_head_project_with_gate():
    heads, vdim, rank, pitch, tokens = 3, 5, 22, 32, 19
    ctx, weight, gate = rand(tokens, heads * pitch, seed=10), rand(heads * vdim, rank, seed=11), rand(tokens, heads * vdim + 2, seed=12)
    out = torch.full((tokens, 16), 3.0, device=DEVICE)
    K.head_project(ctx.to(DEVICE), weight.to(DEVICE), heads, vdim, rank, pitch, out, gate=gate.to(DEVICE)[:, 2:])
    per_head = ctx.double().view(tokens, heads, pitch)[:, :, :rank]
    want = torch.einsum("thr,hvr->thv", per_head, weight.double().view(heads, vdim, rank)).reshape(tokens, heads * vdim)
    want = want * torch.sigmoid(gate.double()[:, 2:])
    assert float((out[:, :15].cpu().double() - want).abs().max()) < 1e-5
    assert float(out[:, 15:].abs().max()) == 0.0
