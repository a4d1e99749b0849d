"""Kodatar without a GPU: configuration, plan, contract, the cache ledger's chunks, and pins of the
plain implementation the GPU tests compare with."""

import copy
import math

import pytest
import torch

import burn_transformers_amd as bt
import plain_kodatar as plain
from burn_transformers_amd.cache.ledger import BLOCK, RELEASED, CacheLedger
from burn_transformers_amd.config import ConfigError, KodatarConfig, resolve_family
from burn_transformers_amd.parts.rotary_attention import rotary_frequencies
from kodatar_helpers import BASIC, CONFIGS, ODD, layer, mixer, model_config, moe, prompts_for, weights_for


def test_configuration_round_trip_and_family():
    for config, _ in CONFIGS.values():
        typed = KodatarConfig.from_dict(config)
        assert KodatarConfig.from_dict(typed.to_dict()) == typed
        assert resolve_family(config).name == "kodatar"
    typed = KodatarConfig.from_dict(BASIC)
    assert typed.layers[0].mixer.chunk == 24 and typed.layers[2].mixer.chunk == 0
    assert typed.layers[0].mlp.groups == 4 and typed.layers[1].mlp.groups == 0 and typed.layers[1].mlp.shared_ff == 0
    assert KodatarConfig.from_dict(ODD).layers[0].mlp is None


@pytest.mark.parametrize("path,value,field", [
    (("width",), None, "width"), (("norm", "eps"), 0.0, "norm.eps"), (("layers", 0, "type"), "conv", "layers[0].type"),
    (("layers", 0, "mixer", "kv_heads"), 3, "layers[0].mixer.kv_heads"), (("layers", 0, "mixer", "rot", "dims"), 18, "layers[0].mixer.rot.dims"),
    (("layers", 0, "mlp", "router", "top"), 9, "layers[0].mlp.router.top"), (("layers", 0, "mlp", "router", "groups", "count"), 3, "layers[0].mlp.router.groups.count"),
    (("layers", 0, "mlp", "router", "groups", "keep"), 1, "layers[0].mlp.router.groups.keep"), (("layers", 0, "mlp", "kind"), "dense", "layers[0].mlp.kind"),
    (("loop", "stop"), 7, "loop"), (("embedding", "scale"), None, "embedding.scale")])
def test_configuration_errors_name_the_field(path, value, field):
    config = copy.deepcopy(BASIC)
    at = config
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ConfigError) as error:
        KodatarConfig.from_dict(config)
    assert error.value.field == field


def test_plan_runs_the_loop_with_a_cache_entry_per_run_and_an_entry_part_per_pass():
    family = resolve_family(BASIC)
    plan = family.plan(KodatarConfig.from_dict(BASIC))
    kinds = [plan.layers[entry.layer].block for entry in plan.schedule]
    assert kinds == ["transform", "sandwich_norm", "sandwich_norm"] * 3 + ["sandwich_norm"]
    assert [entry.cache for entry in plan.schedule if entry.cache is not None] == list(range(7))
    assert [entry.layer for entry in plan.schedule if entry.cache is not None] == [0, 1, 0, 1, 0, 1, 2]
    rows = [plan.layers[entry.layer].parts["transform"].params["row"] for entry in plan.schedule if entry.cache is None]
    assert rows == [0, 1, 2]
    # a loop that starts late: the layers before it run once, before the first pass
    late = family.plan(KodatarConfig.from_dict(ODD))
    assert [late.layers[entry.layer].block for entry in late.schedule] == \
        ["sandwich_norm", "transform", "sandwich_norm", "transform", "sandwich_norm", "sandwich_norm"]
    assert "ff" not in late.layers[0].parts
    # without a loop nothing is kept of the embedding and no part stands between the layers
    flat = family.plan(KodatarConfig.from_dict(model_config([layer(mixer(2, 1, 8, 8, 0.3))], width=16, vocab=11)))
    assert [flat.layers[entry.layer].block for entry in flat.schedule] == ["sandwich_norm"]
    assert not flat.embedding.params["keep_origin"]


def test_contract_and_random_weights_fit():
    family = resolve_family(BASIC)
    typed = KodatarConfig.from_dict(BASIC)
    names = {spec.name: spec for spec in family.contract(typed).tensors}
    assert names["l0.mlp.router"].shape == (8, 64) and names["l0.mlp.router"].layout == "vector"     # 32-bit
    assert names["l0.mlp.e5.down"].shape == (64, 24) and names["l0.mlp.shared.sg"].shape == (1, 64)
    assert "l1.mlp.shared.gate" not in names and names["loop.step"].shape == (3, 64)
    assert names["l0.mix.v"].shape == (2 * 32, 64) and names["l0.mix.q.norm"].shape == (16,)
    _, tensors = bt.random_tensors(BASIC, 0)
    assert set(tensors) == set(names) and all(tuple(tensors[n].shape) == names[n].shape for n in names)


def test_ledger_gives_back_what_lies_before_the_chunk_of_the_next_token():
    ledger = CacheLedger(2, 64, 4, 32, windows=[0, 0], chunks=[0, 150])
    slot = ledger.acquire()
    for length in (100, 149, 150, 299, 300, 700):
        ledger.check_growth({slot: length})
        ledger.reserve(slot, length)
        ledger.commit(slot, length)
        ledger.check()
        first = (length - length % 150) // BLOCK
        held = ledger.held_blocks[1][slot]
        assert all(block == RELEASED for block in held[:first]) and RELEASED not in held[first:]
        assert RELEASED not in ledger.held_blocks[0][slot]
    with pytest.raises(ValueError):
        ledger.truncate(slot, 500)            # position 500's chunk starts at 450, in a block that went back
    ledger.truncate(slot, 650)
    ledger.release(slot)
    ledger.check()
    assert ledger.blocks[1].available() == 64


def test_rescaled_frequencies():
    scaling = {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 64}
    for dims, base in ((8, 500.0), (64, 10000.0), (40, 300000.0)):
        rot = {"dims": dims, "base": base, "scaling": scaling}
        got, want = rotary_frequencies(dims, base, scaling), plain.frequencies(rot)
        assert float((got / want - 1).abs().max()) < 1e-12
        plain_f = plain.frequencies({"dims": dims, "base": base})
        ratio = want / plain_f
        assert float(ratio.max()) <= 1.0 + 1e-12 and float(ratio.min()) >= 0.25 - 1e-12
        long_waves = 2 * math.pi / plain_f > 64
        assert torch.allclose(ratio[long_waves], torch.full_like(ratio[long_waves], 0.25))
        assert torch.allclose(ratio[2 * math.pi / plain_f < 64 / 3], torch.ones_like(ratio[2 * math.pi / plain_f < 64 / 3]))


def test_plain_a_token_sees_its_own_chunk_only():
    config, ids = CONFIGS["attention"][0], prompts_for("attention", [150], seed=1)[0]
    weights = weights_for("attention")
    base = plain.forward(ids, weights, config)
    changed = list(ids)
    changed[10] = (changed[10] + 1) % config["vocab"]
    moved = plain.forward(changed, weights, config)
    differs = (base - moved).abs().max(dim=1).values > 1e-9
    assert differs[10:64].all() and not differs[:10].any() and not differs[64:].any()       # chunks of 64


def test_plain_rotation_depends_on_distance_only_and_leaves_the_rest():
    rot = {"dims": 8, "base": 50.0}
    gen = torch.Generator().manual_seed(0)
    q, k = torch.randn(1, 1, 12, generator=gen, dtype=torch.float64), torch.randn(1, 1, 12, generator=gen, dtype=torch.float64)
    def score(pq, pk):
        return float((plain.turn(q, torch.tensor([pq]), rot) * plain.turn(k, torch.tensor([pk]), rot)).sum())
    assert abs(score(5, 2) - score(105, 102)) < 1e-9 and abs(score(5, 2) - score(5, 3)) > 1e-3
    assert torch.equal(plain.turn(q, torch.tensor([9]), rot)[..., 8:], q[..., 8:])
    assert torch.equal(plain.turn(q, torch.tensor([0]), rot), q)


def test_plain_router_by_hand():
    """Three groups of two of which two stay open; the best single expert is in the group that loses."""
    w = {"r.router": torch.tensor([[2.0], [0.0], [1.0], [0.5], [1.5], [1.4]], dtype=torch.float64),
         "r.correction": torch.tensor([-5.0, -5.0, -1.0, -1.3, -1.2, -1.2], dtype=torch.float64)}
    chosen, weights = plain.route(torch.ones(1, 1, dtype=torch.float64), w, "r.",
                                  {"experts": 6, "top": 3, "groups": {"count": 3, "keep": 2}})
    assert sorted(chosen[0].tolist()) == [2, 4, 5] and abs(float(weights.sum()) - 1.0) < 1e-12
    scores = torch.softmax(w["r.router"][:, 0], 0)
    assert abs(float(weights[0][chosen[0].tolist().index(2)]) - float(scores[2] / scores[[2, 4, 5]].sum())) < 1e-12


def test_plain_identity_experts_and_passes():
    config = model_config([layer(mixer(1, 1, 8, 8, 0.3), moe(1, 8, 2, identity=1))], width=16, vocab=13, loop=(0, 1, 2))
    _, weights = bt.random_tensors(config, 0)
    ids = [1, 2, 3]
    runs = []
    plain.forward(ids, weights, config, residuals=runs)
    assert len(runs) == 2
    # both the expert and the identity expert are always chosen: zeroing the expert leaves weight * h
    w = {k: v.double() for k, v in weights.items()}
    h = torch.randn(2, 16, dtype=torch.float64)
    w["l0.mlp.e0.down"] = torch.zeros_like(w["l0.mlp.e0.down"])
    out = plain.experts(h, w, "l0.mlp.", config["layers"][0]["mlp"])
    scores = torch.softmax(h @ w["l0.mlp.router"].T, -1)
    assert torch.allclose(out, scores[:, 1:2] / scores.sum(-1, keepdim=True) * h)
