"""Salopel's configuration, registry entry, plan and checkpoint contract (no GPU)."""

import copy

import pytest
import torch

import burn_transformers_amd as bt
import plain_salopel as plain
from burn_transformers_amd.config.salopel import SalopelConfig
from salopel_helpers import CONFIGS, MIXED, ODD, latent, mamba1, mamba2, model_config


def test_the_registry_finds_the_family_by_the_singular_key():
    family = bt.resolve_family(MIXED)
    assert family.name == "salopel" and family is bt.resolve_family({"model_type": "salopel"})
    assert family.config_class is SalopelConfig


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_configuration_round_trip(name):
    config = CONFIGS[name][0]
    assert SalopelConfig.from_dict(config).to_dict() == config


@pytest.mark.parametrize("change,field", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c["norm"].pop("eps"), "norm.eps"),
    (lambda c: c.update(residual_mult="x"), "residual_mult"),
    (lambda c: c.update(layers=[]), "layers"),
    (lambda c: c["layers"][0].update(type="rotary_attention"), "layers[0].type"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "layers[0].mixer.kv_rank"),
    (lambda c: c["layers"][1]["mixer"].update(groups=4), "layers[1].mixer.groups"),
    (lambda c: c["layers"][1]["mixer"].update(norm_groups=5), "layers[1].mixer.norm_groups"),
    (lambda c: c["layers"][1]["mlp"].update(kind="experts"), "layers[1].mlp.kind"),
    (lambda c: c["layers"][3].update(weights_of=3), "layers[3].weights_of"),
    (lambda c: c["layers"][3].update(weights_of=1), "layers[3].weights_of"),
    (lambda c: c["layers"][3].update(weights_of=9), "layers[3].weights_of"),
    (lambda c: (c["layers"][0].update(weights_of=3), c["layers"][3].update(weights_of=0)), "layers[0].weights_of"),
])
def test_each_bad_field_is_named(change, field):
    config = copy.deepcopy(MIXED)
    change(config)
    with pytest.raises(bt.ConfigError) as info:
        SalopelConfig.from_dict(config)
    assert info.value.field == field, str(info.value)


def test_plan_runs_a_borrowed_layer_as_a_second_run_of_its_owner():
    family = bt.resolve_family(MIXED)
    config = family.config_class.from_dict(MIXED)
    plan = family.plan(config)
    assert len(plan.layers) == 3                                     # three layers have tensors
    assert [(e.layer, e.cache, e.writes) for e in plan.schedule] == [(0, 0, True), (1, 1, True), (2, 2, True),
                                                                     (0, 3, True), (2, 4, True)]
    assert [sorted(layer.parts) for layer in plan.layers] == [["ff", "ff_norm", "mixer", "mixer_norm"]] * 2 + \
        [["mixer", "mixer_norm"]]
    assert all(layer.block == "output_norm" and layer.params == {"mult": 0.5} for layer in plan.layers)
    assert [layer.parts["mixer"].kind for layer in plan.layers] == ["latent_attention", "head_scan", "selective_scan"]
    names = {spec.name for spec in family.contract(config).tensors}
    assert not any(name.startswith(("l3.", "l4.")) for name in names)
    used = {name for layer in plan.layers for part in layer.parts.values() for name in part.tensors.values()}
    used |= set(plan.embedding.tensors.values()) | set(plan.final_norm.tensors.values()) | set(plan.readout.tensors.values())
    assert used == names                                             # every tensor has a part, every part its tensors


def test_contract_shapes_follow_the_sizes():
    family = bt.resolve_family(ODD)
    shapes = {spec.name: spec.shape for spec in family.contract(family.config_class.from_dict(ODD)).tensors}
    assert shapes["l0.mix.in"] == (60 + 60 + 2 * 200 + 5, 96) and shapes["l0.mix.conv"] == (460, 1)
    assert shapes["l1.mix.uk"] == (160, 20) and shapes["l1.mix.uv"] == (80, 20) and shapes["l1.mix.o"] == (96, 80)
    assert shapes["l2.mix.x"] == (2 + 140, 76) and shapes["l2.mix.dt"] == (76, 2) and shapes["l2.mix.A_log"] == (76, 70)
    assert shapes["l1.mlp.act"] == (4,) and "l0.norm2" not in shapes and "l1.norm2" in shapes


def test_a_checkpoint_that_does_not_fit_is_refused_with_every_fault(tmp_path):
    from burn_transformers_amd.weights.contract import check
    family = bt.resolve_family(MIXED)
    config, tensors = bt.random_tensors(MIXED, 0)

    class Held:
        def __init__(self, t):
            self.shape, self.dtype = tuple(t.shape), "BF16"
    entries = {k: Held(v) for k, v in tensors.items()}
    del entries["l1.mix.D"]
    entries["l3.norm1"] = Held(torch.zeros(64))                        # a borrower has no tensors
    entries["l0.mix.uq"] = Held(torch.zeros(48, 41))
    with pytest.raises(bt.WeightError) as info:
        check(entries, family.contract(config), "test")
    assert info.value.missing == ["l1.mix.D"] and info.value.unexpected == ["l3.norm1"]
    assert len(info.value.mismatched) == 1 and "l0.mix.uq" in info.value.mismatched[0]


def test_the_plain_implementation_is_causal_and_carries_state():
    """The oracle's own pins: a later token changes nothing before it, and the recurrences' outputs
    at a position do depend on tokens far back (state is carried, not dropped)."""
    config = model_config([mamba1(24, 4, 2, 3), mamba2(2, 8, 4, 1, 1, 2), latent(2, 8, 8, 8, 8, 0.5, ff=16)], width=16, vocab=29)
    _, tensors = bt.random_tensors(config, 3)
    ids = torch.randint(0, 29, (40,), generator=torch.Generator().manual_seed(1)).tolist()
    base = plain.forward(ids, tensors, config)
    changed = list(ids)
    changed[25] = (changed[25] + 1) % 29
    after = plain.forward(changed, tensors, config)
    assert torch.equal(base[:25], after[:25]) and not torch.allclose(base[25:], after[25:])
    changed = list(ids)
    changed[0] = (changed[0] + 1) % 29
    assert float((plain.forward(changed, tensors, config)[-1] - base[-1]).abs().max()) > 1e-9


def test_the_plain_convolution_and_polynorm():
    u = torch.arange(12, dtype=torch.float64).reshape(4, 3)
    taps = torch.tensor([[1.0, 10.0], [0.0, 1.0], [2.0, 0.0]], dtype=torch.float64)
    out = plain.causal_conv(u, taps, torch.tensor([0.5, 0.0, 0.0], dtype=torch.float64))
    assert out[0].tolist() == [0.5, 1.0, 0.0]                          # nothing before the first token
    assert out[2].tolist() == [3.0 + 60.0 + 0.5, 7.0, 2 * 5.0]         # last column: the current token
    z = torch.tensor([[3.0, -4.0]], dtype=torch.float64)
    got = plain.poly_norm(z, torch.tensor([1.0, 0.0, 0.0, 0.25], dtype=torch.float64), 0.0)
    assert torch.allclose(got, z / (12.5 ** 0.5) + 0.25)
    got = plain.poly_norm(z, torch.tensor([0.0, 2.0, 0.0, 0.0], dtype=torch.float64), 0.0)
    assert torch.allclose(got, 2 * z * z / ((81 + 256) / 2) ** 0.5)


def test_a_borrower_may_come_before_its_owner_or_name_another_borrower():
    layers = [latent(2, 8, 8, 8, 16, 0.5, ff=24, weights_of=2), mamba1(24, 4, 2, 3), latent(2, 8, 8, 8, 16, 0.5, ff=24),
              mamba1(24, 4, 2, 3, weights_of=1), mamba1(24, 4, 2, 3, weights_of=3)]
    config_json = model_config(layers, width=16, vocab=29)
    family = bt.resolve_family(config_json)
    config = family.config_class.from_dict(config_json)
    assert [config.owner(i) for i in range(5)] == [2, 1, 2, 1, 1]
    plan = family.plan(config)
    assert [(e.layer, e.cache) for e in plan.schedule] == [(1, 0), (0, 1), (1, 2), (0, 3), (0, 4)]
    names = {spec.name for spec in family.contract(config).tensors}
    assert any(n.startswith("l1.") for n in names) and any(n.startswith("l2.") for n in names)
    assert not any(n.startswith(("l0.", "l3.", "l4.")) for n in names)
    _, tensors = bt.random_tensors(config_json, 0)
    logits = plain.forward([1, 2, 3, 4], tensors, config_json)
    assert logits.shape == (4, 29) and torch.isfinite(logits).all()
