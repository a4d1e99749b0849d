"""Tiny Salopel configurations and helpers shared by the tests of that family."""

import torch

import burn_transformers_amd as bt
import plain_salopel as plain


def latent(heads, dim, vdim, q_rank, kv_rank, scale, ff=None, weights_of=None):
    entry = {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank,
                                                   "kv_rank": kv_rank, "scale": scale},
             "mlp": {"kind": "dense", "ff": ff} if ff else None}
    if weights_of is not None:
        entry["weights_of"] = weights_of
    return entry


def mamba1(inner, state, dt_rank, conv, ff=None, weights_of=None):
    entry = {"type": "mamba1", "mixer": {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv},
             "mlp": {"kind": "dense", "ff": ff} if ff else None}
    if weights_of is not None:
        entry["weights_of"] = weights_of
    return entry


def mamba2(heads, vdim, state, groups, norm_groups, conv, ff=None, weights_of=None):
    entry = {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups,
                                         "norm_groups": norm_groups, "conv": conv},
             "mlp": {"kind": "dense", "ff": ff} if ff else None}
    if weights_of is not None:
        entry["weights_of"] = weights_of
    return entry


def model_config(layers, width=64, vocab=257, mult=0.5, eps=1e-6):
    return {"architecture": "Salopel", "vocab": vocab, "width": width, "residual_mult": mult, "norm": {"eps": eps},
            "layers": layers}


# every kind of layer, with and without a feed-forward, two layers run twice; query/key and value
# sizes differ, the latent is no multiple of 16, groups of several heads, one part of the norm
MIXED = model_config([latent(3, 16, 24, 40, 48, 0.3, ff=100),
                      mamba2(6, 8, 16, 3, 1, 2, ff=72),
                      mamba1(96, 5, 3, 4),
                      latent(3, 16, 24, 40, 48, 0.3, ff=100, weights_of=0),
                      mamba1(96, 5, 3, 4, weights_of=2)])
# sizes the kernels do not divide: more heads than a decode tile takes, ranks and inner widths that
# are no multiple of eight, a state longer than one register per lane, no convolution state (one
# tap), every head a group and a part of the norm of its own
ODD = model_config([mamba2(5, 12, 40, 5, 5, 1),
                    latent(20, 8, 4, 12, 20, 0.5, ff=52),
                    mamba1(76, 70, 2, 5, ff=36),
                    mamba2(2, 20, 3, 1, 2, 3)], width=96, vocab=131, mult=0.8, eps=1e-3)
# sizes of one: a single head, a single state element, a rank-one step size (every channel's step
# then hangs on one number, which no rounding to 8 bits survives: float32 only), one tap
ONES = model_config([latent(1, 4, 4, 4, 4, 0.7), mamba1(24, 1, 1, 1), mamba2(1, 16, 1, 1, 1, 2, ff=8),
                     mamba1(20, 3, 1, 2, ff=12)], width=16, vocab=37, mult=1.0, eps=1e-5)
ATTENTION_ONLY = model_config([latent(4, 32, 16, 24, 64, 0.25), latent(2, 16, 48, 56, 32, 0.4, ff=96)], width=64, vocab=211)
SCAN_ONLY = model_config([mamba1(64, 16, 4, 3)], width=32, vocab=101, mult=0.7)
HEADS_ONLY = model_config([mamba2(4, 16, 32, 2, 2, 4)], width=32, vocab=101, mult=0.7)
FEED_FORWARD = model_config([latent(1, 8, 8, 8, 16, 1.0, ff=40)], width=32, vocab=61, mult=2.0)
# a latent wider than any MFMA attention kernel's head: the plain attention kernel runs it
WIDE_LATENT = model_config([latent(2, 8, 8, 16, 136, 0.3)], width=32, vocab=53)
# the first layer runs the third's tensors, the last one the second's: a borrower before and behind its owner
LOOPED = model_config([latent(2, 16, 8, 24, 32, 0.3, ff=40, weights_of=2), mamba1(48, 8, 4, 3),
                       latent(2, 16, 8, 24, 32, 0.3, ff=40), mamba1(48, 8, 4, 3, weights_of=1)], width=48, vocab=89)
# odd numbers everywhere a kernel counts in fours, eights or sixteens: head sizes 6 and 10, values of 5,
# ranks 7 and 9, 3 heads in 3 groups, 30 and 18 inner channels, a feed-forward of 37
RAGGED = model_config([mamba2(3, 6, 9, 3, 1, 2, ff=37), latent(3, 6, 5, 7, 9, 0.4), mamba1(30, 3, 5, 2),
                       mamba2(1, 10, 17, 1, 2, 3), latent(5, 3, 7, 9, 11, 0.6, ff=19)], width=40, vocab=71, mult=0.9)
CONFIGS = {"ragged": (RAGGED, 10), "looped": (LOOPED, 9), "wide": (WIDE_LATENT, 8), "mixed": (MIXED, 1), "odd": (ODD, 2), "attention": (ATTENTION_ONLY, 3), "scan": (SCAN_ONLY, 4),
           "heads": (HEADS_ONLY, 5), "ff": (FEED_FORWARD, 6), "ones": (ONES, 7)}

_weights, _models = {}, {}


def weights_for(name, sharpen=1.0):
    """float32 weights as a load will see them (rounded to bfloat16).  ``sharpen`` multiplies the
    queries' up-projection, so that attention puts its weight on few keys and a lost key shows."""
    key = (name, sharpen)
    if key not in _weights:
        config, seed = CONFIGS[name]
        _, tensors = bt.random_tensors(config, seed)
        if sharpen != 1.0:
            tensors = {k: (v * sharpen if k.endswith(".mix.uq") else v) for k, v in tensors.items()}
        _weights[key] = {k: v.to(torch.bfloat16).float() for k, v in tensors.items()}
    return _weights[key]


def model_for(name, dtype, sharpen=1.0):
    key = (name, dtype, sharpen)
    if key not in _models:
        stored = {k: v.to(torch.bfloat16) for k, v in weights_for(name, sharpen).items()}
        _models[key] = bt.model_from_tensors(CONFIGS[name][0], stored, dtype, "cuda:0")
    return _models[key]


def engine_for(name, dtype, max_tokens=2048, sharpen=1.0, **options):
    return bt.Engine(model_for(name, dtype, sharpen), max_tokens=max_tokens, **options)


def plain_logits(name, ids, sharpen=1.0):
    return plain.forward(ids, weights_for(name, sharpen), CONFIGS[name][0])


def prompts_for(name, lengths, seed=0):
    gen = torch.Generator().manual_seed(seed)
    return [torch.randint(0, CONFIGS[name][0]["vocab"], (n,), generator=gen).tolist() for n in lengths]


def tolerance(dtype, reference):
    """Largest allowed absolute error of logits: float32 differs from float64 by rounding of sums and
    of the recurrences' exponentials; bfloat16 rounds the operands of every product to 8 bits (measured:
    up to 1.5e-2 of the largest logit where a layer's output is scaled up before it joins the stream)."""
    scale = float(reference.abs().max())
    return 2e-5 + 2e-5 * scale if dtype == "float32" else 2.5e-2 * scale
