"""Salopel as a family: its plan, its checkpoint contract and its random initialisation.

This is the only file that knows Salopel's wiring and tensor names.
  plan      token table, then an RMS norm (every norm of the layers' outputs, of the embedding and
            before the readout multiplies by 1 + weight); layers of the kinds config.json lists, each
            an ``output_norm`` block: x += m * norm1(mixer(x)), then x += m * norm2(ff(x)) where the
            layer has a feed-forward; mixers ``latent_attention``, ``selective_scan`` (config type
            mamba1) and ``head_scan`` (mamba2); dense feed-forward with the poly_norm activation;
            readout tied to the token table.  A layer with ``weights_of`` is a second run of its
            owner's parts with a cache entry of its own.
  contract  tensor names ('l<i>.mix.*', 'l<i>.mlp.*', 'l<i>.norm1' ...), shapes; matrices [out, in]
  init      random weights for tests and benchmarks
"""

import math

import torch

from ..config.registry import Family, register_family
from ..config.salopel import SalopelConfig
from ..engine.plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from ..weights.contract import Contract, TensorSpec

NORM_OFFSET = 1.0         # the scales of the layer, embedding and final norms are stored around zero


def _mixer_tensors(kind, sizes, width):
    """[(name below '<layer>.mix.', shape, layout, role in the part)] of a mixer."""
    if kind == "latent_attention":
        heads, dim, vdim, q_rank, kv_rank = (sizes[k] for k in ("heads", "dim", "vdim", "q_rank", "kv_rank"))
        return [("dq", (q_rank, width), "out_in", "down_q"), ("dq.norm", (q_rank,), "vector", "q_norm"),
                ("uq", (heads * dim, q_rank), "out_in", "up_q"), ("dkv", (kv_rank, width), "out_in", "down_kv"),
                ("dkv.norm", (kv_rank,), "vector", "kv_norm"), ("uk", (heads * dim, kv_rank), "out_in", "up_k"),
                ("uv", (heads * vdim, kv_rank), "out_in", "up_v"), ("g", (heads * vdim, width), "out_in", "gate"),
                ("o", (width, heads * vdim), "out_in", "out_weight")]
    if kind == "mamba1":
        inner, state, dt_rank, taps = (sizes[k] for k in ("inner", "state", "dt_rank", "conv"))
        return [("in", (2 * inner, width), "out_in", "in_weight"), ("conv", (inner, taps), "vector", "conv_weight"),
                ("conv.b", (inner,), "vector", "conv_bias"), ("x", (dt_rank + 2 * state, inner), "out_in", "x_weight"),
                ("dt", (inner, dt_rank), "out_in", "dt_weight"), ("dt.b", (inner,), "vector", "dt_bias"),
                ("A_log", (inner, state), "vector", "A_log"), ("D", (inner,), "vector", "D"),
                ("o", (width, inner), "out_in", "out_weight")]
    heads, vdim, state, groups, taps = (sizes[k] for k in ("heads", "vdim", "state", "groups", "conv"))
    inner, channels = heads * vdim, heads * vdim + 2 * groups * state
    return [("in", (inner + channels + heads, width), "out_in", "in_weight"),
            ("conv", (channels, taps), "vector", "conv_weight"), ("conv.b", (channels,), "vector", "conv_bias"),
            ("dt_bias", (heads,), "vector", "dt_bias"), ("A_log", (heads,), "vector", "A_log"),
            ("D", (heads,), "vector", "D"), ("norm", (inner,), "vector", "norm_weight"),
            ("o", (width, inner), "out_in", "out_weight")]


def _mixer_spec(layer, index, config):
    sizes, width = layer.sizes, config.width
    tensors = {role: f"l{index}.mix.{name}" for name, _, _, role in _mixer_tensors(layer.type, sizes, width)}
    if layer.type == "latent_attention":
        params = {"width": width, "eps": config.norm_eps, **{k: sizes[k] for k in ("heads", "dim", "vdim", "q_rank", "kv_rank", "scale")}}
        return PartSpec("latent_attention", params, tensors)
    if layer.type == "mamba1":
        params = {"width": width, "inner": sizes["inner"], "state": sizes["state"], "dt_rank": sizes["dt_rank"], "taps": sizes["conv"]}
        return PartSpec("selective_scan", params, tensors)
    params = {"width": width, "eps": config.norm_eps, "taps": sizes["conv"],
              **{k: sizes[k] for k in ("heads", "vdim", "state", "groups", "norm_groups")}}
    return PartSpec("head_scan", params, tensors)


def plan(config: SalopelConfig) -> ModelPlan:
    width, eps = config.width, config.norm_eps

    def norm(name):
        return PartSpec("rms_norm", {"width": width, "eps": eps, "offset": NORM_OFFSET}, {"weight": name})

    layers, number = [], {}
    for index, layer in enumerate(config.layers):
        if layer.weights_of is not None:
            continue
        parts = {"mixer": _mixer_spec(layer, index, config), "mixer_norm": norm(f"l{index}.norm1")}
        if layer.ff is not None:
            parts["ff"] = PartSpec("dense", {"width": width, "inner": layer.ff, "activation": "poly_norm", "eps": eps},
                                   {"up_weight": f"l{index}.mlp.up", "down_weight": f"l{index}.mlp.down",
                                    "act_coefficients": f"l{index}.mlp.act"})
            parts["ff_norm"] = norm(f"l{index}.norm2")
        number[index] = len(layers)
        layers.append(LayerPlan("output_norm", parts, {"mult": config.residual_mult}))
    return ModelPlan(
        width=width, vocab_size=config.vocab, max_positions=2 ** 31 - 1,      # no position is encoded anywhere
        embedding=PartSpec("normalized_tokens", {"width": width, "vocab_size": config.vocab, "eps": eps,
                                                 "offset": NORM_OFFSET},
                           {"tokens": "embed", "norm_weight": "embed.norm"}),
        layers=layers,
        # every run of a layer has a cache entry (keys and values, or state) of its own
        schedule=[ScheduleEntry(layer=number[config.owner(i)], cache=i) for i in range(len(config.layers))],
        final_norm=norm("final.norm"),
        readout=PartSpec("linear_readout", {"width": width, "vocab_size": config.vocab}, {"weight": "embed"}))


def contract(config: SalopelConfig) -> Contract:
    width = config.width
    tensors = [TensorSpec("embed", (config.vocab, width), "table"), TensorSpec("embed.norm", (width,), "vector")]
    for index, layer in enumerate(config.layers):
        if layer.weights_of is not None:
            continue
        tensors.append(TensorSpec(f"l{index}.norm1", (width,), "vector"))
        if layer.ff is not None:
            tensors.append(TensorSpec(f"l{index}.norm2", (width,), "vector"))
        tensors += [TensorSpec(f"l{index}.mix.{name}", shape, layout)
                    for name, shape, layout, _ in _mixer_tensors(layer.type, layer.sizes, width)]
        if layer.ff is not None:
            tensors += [TensorSpec(f"l{index}.mlp.up", (layer.ff, width), "out_in"),
                        TensorSpec(f"l{index}.mlp.down", (width, layer.ff), "out_in"),
                        TensorSpec(f"l{index}.mlp.act", (4,), "vector")]
    tensors.append(TensorSpec("final.norm", (width,), "vector"))
    return Contract(tensors=tensors, prefixes=("",), anchor="embed")


def init(config: SalopelConfig, generator):
    """Matrices N(0, 1/in); norm scales near zero (they are distances from one); the recurrences'
    constants in the ranges such layers are usually started in (decay rates 1..state, step sizes of
    a few hundredths to a tenth)."""

    def normal(shape, std, mean=0.0):
        return torch.randn(shape, generator=generator, dtype=torch.float32) * std + mean

    def uniform(shape, low, high):
        return torch.rand(shape, generator=generator, dtype=torch.float32) * (high - low) + low

    tensors = {}
    for spec in contract(config).tensors:
        name, shape = spec.name, spec.shape
        leaf = name.split(".", 1)[1] if "." in name else name
        if name == "embed":
            tensors[name] = normal(shape, 1.0)
        elif leaf in ("norm", "norm1", "norm2"):                         # around zero: the norm adds one
            tensors[name] = normal(shape, 0.1)
        elif leaf in ("mix.dq.norm", "mix.dkv.norm", "mix.norm"):        # plain scales
            tensors[name] = normal(shape, 0.1, 1.0)
        elif leaf == "mlp.act":
            tensors[name] = torch.tensor([0.6, 0.3, 0.2, 0.05]) + normal(shape, 0.05)
        elif leaf == "mix.conv":
            tensors[name] = normal(shape, 1.0 / math.sqrt(shape[1]))
        elif leaf in ("mix.conv.b", "mix.D"):
            tensors[name] = normal(shape, 0.3, 1.0 if leaf == "mix.D" else 0.0)
        elif leaf == "mix.A_log":
            tensors[name] = torch.log(uniform(shape, 1.0, 8.0))
        elif leaf in ("mix.dt.b", "mix.dt_bias"):                          # softplus^-1 of a step size in 0.01 .. 0.2
            step = torch.exp(uniform(shape, math.log(0.01), math.log(0.2)))
            tensors[name] = step + torch.log(-torch.expm1(-step))
        else:
            tensors[name] = normal(shape, 1.0 / math.sqrt(shape[-1]))
    return tensors


FAMILY = register_family(Family(
    name="salopel", architectures=("Salopel",), model_types=("salopel",),
    config_class=SalopelConfig, plan=plan, contract=contract, init=init))
