"""Tiny Kodatar configurations and helpers shared by the tests of that family."""

import torch

import burn_transformers_amd as bt
import plain_kodatar as plain


def mixer(heads, kv_heads, dim, vdim, scale, rot_dims=None, base=10000.0, scaling=None, chunk=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
            "rot": {"dims": rot_dims, "base": base, "scaling": scaling} if rot_dims else None,
            "mask": {"size": chunk} if chunk else None}


def moe(experts, ff, top, identity=0, groups=None, shared=None):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "identity": identity,
                       "groups": {"count": groups[0], "keep": groups[1]} if groups else None},
            "shared": {"ff": shared} if shared else None}


def layer(mix, mlp=None):
    return {"type": "attention", "mixer": mix, "mlp": mlp}


def model_config(layers, width=64, vocab=211, loop=None, embed_scale=2.0, logit_scale=0.5, eps=1e-5):
    config = {"architecture": "Kodatar", "vocab": vocab, "width": width, "embedding": {"scale": embed_scale},
              "logit_scale": logit_scale, "norm": {"eps": eps}, "layers": layers}
    if loop:
        config["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return config


SCALING = {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 64}
# values wider than queries, part of a head turned with rescaled frequencies, chunks that are no multiple
# of a tile, experts in four groups of which two stay open, identity experts, a shared expert; the first two
# layers run three times
BASIC = model_config([layer(mixer(4, 2, 16, 32, 0.25, rot_dims=8, base=500.0, scaling=SCALING, chunk=24),
                            moe(6, 24, 3, identity=2, groups=(4, 2), shared=40)),
                      layer(mixer(4, 4, 32, 16, 0.2, rot_dims=32, chunk=40), moe(4, 16, 2)),
                      layer(mixer(2, 1, 16, 16, 0.3, rot_dims=16, base=50.0), moe(8, 8, 2, groups=(2, 1), shared=24))],
                     loop=(0, 2, 3))
# sizes the kernels do not divide, layers that differ, a layer without a feed-forward, no rotation in
# one layer, one expert a token (its weight is then one), every expert chosen, a loop that starts late
ODD = model_config([layer(mixer(3, 3, 24, 10, 0.2, rot_dims=24, base=100.0)),
                    layer(mixer(6, 1, 8, 8, 0.4, chunk=7), moe(5, 12, 1)),
                    layer(mixer(2, 2, 40, 48, 0.15, rot_dims=20, chunk=100), moe(3, 20, 4, identity=1, groups=(2, 2)))],
                   width=40, vocab=97, loop=(1, 2, 2), embed_scale=0.5, logit_scale=2.0, eps=1e-3)
ATTENTION_ONLY = model_config([layer(mixer(4, 2, 32, 32, 0.18, rot_dims=16, base=1000.0, chunk=64))], width=64, vocab=101)
FULL_CAUSAL = model_config([layer(mixer(2, 1, 64, 32, 0.125, rot_dims=64, base=10000.0))], width=32, vocab=101)
EXPERTS_PLAIN = model_config([layer(mixer(1, 1, 16, 16, 0.25), moe(6, 16, 2))], width=32, vocab=61)
EXPERTS_FULL = model_config([layer(mixer(1, 1, 16, 16, 0.25), moe(9, 8, 3, identity=3, groups=(3, 2), shared=16))],
                            width=32, vocab=61)
LOOP_ONLY = model_config([layer(mixer(2, 2, 16, 16, 0.25, rot_dims=8))], width=32, vocab=61, loop=(0, 1, 4))
# heads of 128, chunks that span several blocks: keys far back and at block borders
LONG = model_config([layer(mixer(2, 1, 128, 64, 0.09, rot_dims=64, base=300000.0, scaling={"factor": 6.0, "low": 1.0,
                                                                                           "high": 5.0, "original": 256},
                                 chunk=448), moe(4, 32, 2, shared=32)),
                     layer(mixer(4, 2, 48, 48, 0.14, rot_dims=48, base=10000.0), moe(4, 32, 1, identity=1))],
                    width=96, vocab=151, loop=(0, 2, 2))
# more query heads on a cached head than a decode tile takes, and one cached head for all
MANY_HEADS = model_config([layer(mixer(20, 1, 16, 16, 0.25, rot_dims=16, chunk=48), moe(2, 16, 1, shared=8))], width=48, vocab=71)
# heads wider than any MFMA attention kernel's (the plain attention kernel runs them), an odd feed-forward
WIDE_HEADS = model_config([layer(mixer(2, 1, 144, 20, 0.08, rot_dims=100, chunk=30), moe(3, 5, 2, shared=3))], width=32, vocab=53)
CONFIGS = {"wide_heads": (WIDE_HEADS, 10), "many_heads": (MANY_HEADS, 9), "basic": (BASIC, 1), "odd": (ODD, 2), "attention": (ATTENTION_ONLY, 3), "causal": (FULL_CAUSAL, 4),
           "experts": (EXPERTS_PLAIN, 5), "experts_full": (EXPERTS_FULL, 6), "loop": (LOOP_ONLY, 7), "long": (LONG, 8)}

_weights, _models = {}, {}


def weights_for(name, sharpen=1.0, dtype="float32"):
    """float32 weights as a load will see them (rounded to bfloat16).  ``sharpen`` multiplies the
    queries' head scale, so that attention puts its weight on few keys and a lost key shows.
    For bfloat16 runs the routers' corrections are spread out (steps of 1.5, in a shuffled order of the
    experts), so that which experts a token uses does not hang on a close call: with operands rounded
    to 8 bits a near tie between two experts' scores falls the other way now and then, the token's
    whole feed-forward output is then another, and no bound on rounding holds.  The weights of the
    chosen experts still differ from token to token; the choice itself varies in the float32 runs,
    which go through the same steps."""
    key = (name, sharpen, dtype == "bfloat16")
    if key not in _weights:
        config, seed = CONFIGS[name]
        _, tensors = bt.random_tensors(config, seed)
        if sharpen != 1.0:
            tensors = {k: (v * sharpen if k.endswith(".mix.q.norm") else v) for k, v in tensors.items()}
        if dtype == "bfloat16":
            gen = torch.Generator().manual_seed(seed)
            for k in sorted(tensors):
                if k.endswith(".mlp.correction"):
                    n = tensors[k].numel()
                    tensors[k] = tensors[k] + 1.5 * torch.randperm(n, generator=gen).float()
        _weights[key] = {k: v.to(torch.bfloat16).float() for k, v in tensors.items()}
    return _weights[key]


def model_for(name, dtype, sharpen=1.0):
    key = (name, dtype, sharpen)
    if key not in _models:
        stored = {k: v.to(torch.bfloat16) for k, v in weights_for(name, sharpen, dtype).items()}
        _models[key] = bt.model_from_tensors(CONFIGS[name][0], stored, dtype, "cuda:0")
    return _models[key]


def engine_for(name, dtype, max_tokens=4096, sharpen=1.0, **options):
    return bt.Engine(model_for(name, dtype, sharpen), max_tokens=max_tokens, **options)


def plain_logits(name, ids, sharpen=1.0, dtype="float32"):
    return plain.forward(ids, weights_for(name, sharpen, dtype), CONFIGS[name][0])


def prompts_for(name, lengths, seed=0):
    gen = torch.Generator().manual_seed(seed)
    return [torch.randint(0, CONFIGS[name][0]["vocab"], (n,), generator=gen).tolist() for n in lengths]


def tolerance(dtype, reference):
    """Largest allowed absolute error of logits: float32 differs from float64 by the rounding of sums;
    bfloat16 rounds the operands of every product to 8 bits."""
    scale = float(reference.abs().max())
    return 2e-5 + 3e-5 * scale if dtype == "float32" else 3e-2 * scale
