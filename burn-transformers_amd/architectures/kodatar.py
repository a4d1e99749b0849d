"""Kodatar as a family: its plan, its checkpoint contract and its random initialisation.

This is the only file that knows Kodatar's wiring and tensor names.
  plan      token table times a scale (kept beside the stream as x0); layers as config.json lists
            them, each a ``sandwich_norm`` block with four layer norms (scale and shift):
            x += norm1b(mixer(norm1(x))), then, where the layer has a feed-forward,
            x += norm2b(ff(norm2(x))); mixer ``rotary_attention`` (head norms, partial rotation with
            rescaled frequencies, grouped heads, keys seen in chunks); feed-forward
            ``routed_experts``.  With ``loop``, layers start .. stop - 1 run ``times`` times with the same
            tensors and a cache entry per run; every pass is entered through a ``joined_projection``
            x <- W [x; x0] + step[pass].  Final layer norm, readout tied to the token table, the
            logits' scale folded into the final norm's scale and shift.
  contract  tensor names ('l<i>.mix.*', 'l<i>.mlp.*', 'l<i>.norm1' ..., 'loop.in', 'loop.step'), shapes
  init      random weights for tests and benchmarks
"""

import math

import torch

from ..config.kodatar import KodatarConfig
from ..config.registry import Family, register_family
from ..engine.plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from ..weights.contract import Contract, TensorSpec

NORMS = ("norm1", "norm1b", "norm2", "norm2b")


def _expert_tensors(prefix, experts):
    """[(checkpoint name, shape kind, role in the part)] of a layer's feed-forward."""
    names = [(f"{prefix}router", "router", "router"), (f"{prefix}correction", "correction", "correction")]
    for e in range(experts.experts):
        names += [(f"{prefix}e{e}.gate", "in", f"gate_{e}"), (f"{prefix}e{e}.up", "in", f"up_{e}"),
                  (f"{prefix}e{e}.down", "out", f"down_{e}")]
    if experts.shared_ff:
        names += [(f"{prefix}shared.gate", "shared_in", "shared_gate"), (f"{prefix}shared.up", "shared_in", "shared_up"),
                  (f"{prefix}shared.down", "shared_out", "shared_down"), (f"{prefix}shared.sg", "mix", "shared_mix")]
    return names


def plan(config: KodatarConfig) -> ModelPlan:
    width, eps = config.width, config.norm_eps

    def norm(name, gain=1.0):
        params = {"width": width, "eps": eps}
        if gain != 1.0:
            params["gain"] = gain
        return PartSpec("layer_norm", params, {"weight": name, "bias": name + ".b"})

    layers = []
    for index, layer in enumerate(config.layers):
        m, p = layer.mixer, f"l{index}."
        mixer = PartSpec("rotary_attention",
                         {"width": width, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
                          "scale": m.scale, "eps": eps, "head_norm": True, "rot_dims": m.rot_dims, "rot_base": m.rot_base,
                          "rot_scaling": m.rot_scaling.to_dict() if m.rot_scaling else None, "chunk": m.chunk},
                         {"q_weight": p + "mix.q", "k_weight": p + "mix.k", "v_weight": p + "mix.v",
                          "q_norm": p + "mix.q.norm", "k_norm": p + "mix.k.norm", "out_weight": p + "mix.o"})
        parts = {"mixer_norm": norm(p + "norm1"), "mixer": mixer, "mixer_post": norm(p + "norm1b")}
        if layer.mlp is not None:
            e = layer.mlp
            parts["ff_norm"], parts["ff_post"] = norm(p + "norm2"), norm(p + "norm2b")
            parts["ff"] = PartSpec("routed_experts",
                                   {"width": width, "experts": e.experts, "ff": e.ff, "identity": e.identity, "top": e.top,
                                    "groups": e.groups, "keep": e.keep, "shared_ff": e.shared_ff},
                                   {role: name for name, _, role in _expert_tensors(p + "mlp.", e)})
        layers.append(LayerPlan("sandwich_norm", parts))
    # a pass of the loop is entered through a part of its own (the same matrix, its own row of the shift)
    entry = {}
    if config.loop is not None:
        for number in range(config.loop.times):
            entry[number] = len(layers)
            layers.append(LayerPlan("transform", {"transform": PartSpec(
                "joined_projection", {"width": width, "row": number}, {"weight": "loop.in", "shift": "loop.step"})}))
    schedule = []
    for index, opens in config.runs():
        if opens is not None:
            schedule.append(ScheduleEntry(layer=entry[opens], cache=None))
        schedule.append(ScheduleEntry(layer=index, cache=sum(1 for s in schedule if s.cache is not None)))
    return ModelPlan(
        width=width, vocab_size=config.vocab, max_positions=2 ** 31 - 1,      # positions are angles: no table bounds them
        embedding=PartSpec("token_only", {"width": width, "vocab_size": config.vocab, "scale": config.embedding_scale,
                                          "keep_origin": config.loop is not None}, {"tokens": "embed"}),
        layers=layers, schedule=schedule, final_norm=norm("final.norm", config.logit_scale),
        readout=PartSpec("linear_readout", {"width": width, "vocab_size": config.vocab}, {"weight": "embed"}))


def contract(config: KodatarConfig) -> Contract:
    width = config.width
    tensors = [TensorSpec("embed", (config.vocab, width), "table")]
    if config.loop is not None:
        tensors += [TensorSpec("loop.in", (width, 2 * width), "out_in"),
                    TensorSpec("loop.step", (config.loop.times, width), "vector")]
    for index, layer in enumerate(config.layers):
        m, p = layer.mixer, f"l{index}."
        for name in NORMS if layer.mlp is not None else NORMS[:2]:
            tensors += [TensorSpec(p + name, (width,), "vector"), TensorSpec(p + name + ".b", (width,), "vector")]
        tensors += [TensorSpec(p + "mix.q", (m.heads * m.dim, width), "out_in"),
                    TensorSpec(p + "mix.k", (m.kv_heads * m.dim, width), "out_in"),
                    TensorSpec(p + "mix.v", (m.kv_heads * m.vdim, width), "out_in"),
                    TensorSpec(p + "mix.q.norm", (m.dim,), "vector"), TensorSpec(p + "mix.k.norm", (m.dim,), "vector"),
                    TensorSpec(p + "mix.o", (width, m.heads * m.vdim), "out_in")]
        if layer.mlp is not None:
            e = layer.mlp
            shapes = {"router": ((e.experts + e.identity, width), "vector"),       # routers are 32-bit: held as stored, widened
                      "correction": ((e.experts + e.identity,), "vector"),
                      "in": ((e.ff, width), "out_in"), "out": ((width, e.ff), "out_in"),
                      "shared_in": ((e.shared_ff, width), "out_in"), "shared_out": ((width, e.shared_ff), "out_in"),
                      "mix": ((1, width), "vector")}
            tensors += [TensorSpec(name, *shapes[kind]) for name, kind, _ in _expert_tensors(p + "mlp.", e)]
    tensors += [TensorSpec("final.norm", (width,), "vector"), TensorSpec("final.norm.b", (width,), "vector")]
    return Contract(tensors=tensors, prefixes=("",), anchor="embed")


def init(config: KodatarConfig, generator):
    """Matrices N(0, 1/in); norm scales around one, shifts and corrections small."""

    def normal(shape, std, mean=0.0):
        return torch.randn(shape, generator=generator, dtype=torch.float32) * std + mean

    tensors = {}
    for spec in contract(config).tensors:
        name, shape = spec.name, spec.shape
        if name == "embed":
            tensors[name] = normal(shape, 1.0)
        elif name == "loop.step" or name.endswith(".b"):
            tensors[name] = normal(shape, 0.1)
        elif name.endswith(".correction"):
            tensors[name] = normal(shape, 0.02)
        elif spec.layout == "vector" and len(shape) == 1:              # scales of norms
            tensors[name] = normal(shape, 0.1, 1.0)
        else:
            tensors[name] = normal(shape, 1.0 / math.sqrt(shape[-1]))
    return tensors


FAMILY = register_family(Family(
    name="kodatar", architectures=("Kodatar",), model_types=("kodatar",),
    config_class=KodatarConfig, plan=plan, contract=contract, init=init))
