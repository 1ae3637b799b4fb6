"""Small Givizen configurations for the tests and weights that make faults show.

Random weights of one small scale would hide most faults: every softmax nearly uniform, every sink negligible, every
clamp idle.  ``make_weights`` draws bolder ones: queries and keys large enough for peaked attention, sinks that take
a visible share, projections into the experts large enough to reach their limits, norm weights away from zero.
Everything is rounded to bfloat16 once, so that both precisions run the same model.

``exact_router=True`` makes the routers' choices safe from rounding: a router then reads only a few *marker*
coordinates of the stream, which hold small integers from the embedding and which no branch writes to (the rows of
every output projection that feed them are zero), through weights that are small dyadic numbers; every router logit
is then exact in bfloat16 as in float64, and a last marker that is 1 for every token separates equal logits.  Without
it a bfloat16 engine and a float64 yardstick would now and then choose different experts for a token whose two best
scores lie close, which is no fault of either.
"""

from __future__ import annotations

import math

import torch

from polosun_util import Fixed, make_runner, spread  # noqa: F401  (architecture-neutral helpers)

MOE_A = {"kind": "moe", "router": {"experts": 6, "top": 2}, "expert": {"ff": 40, "limit": 1.25},
         "shared": {"ff": 48, "limit": 1.75}}

# every size differs from its neighbours'; head sizes for keys and values differ; a layer without feed-forward and
# one without a shared expert; all experts chosen somewhere; windows from 2 tokens up; periods that the positions pass
SMALL_A = {
    "architecture": "Givizen", "vocab": 96, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 0.75},
    "logit_softcap": 12.0,
    "layers": [
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.3, "mask": {"size": 20},
                   "q_temp": {"coef": 0.4, "every": 8}},
         "mlp": MOE_A},
        {"type": "attention_2",
         "mixer": {"heads": 6, "kv_heads": 3, "dim": 8, "vdim": 8, "scale": 0.5, "softcap": 4.0, "mask": {"size": 7},
                   "q_temp": {"coef": 0.25, "every": 5}},
         "mlp": {"kind": "moe", "router": {"experts": 3, "top": 3}, "expert": {"ff": 24, "limit": 2.0}}},
        {"type": "attention",
         "mixer": {"heads": 3, "kv_heads": 1, "dim": 40, "vdim": 16, "scale": 0.15, "mask": {"size": 33},
                   "q_temp": {"coef": 0.6, "every": 16}},
         "mlp": None},
        {"type": "attention_2",
         "mixer": {"heads": 2, "kv_heads": 2, "dim": 24, "vdim": 72, "scale": 0.2, "softcap": 9.0, "mask": {"size": 2},
                   "q_temp": {"coef": 0.1, "every": 3}},
         "mlp": {"kind": "moe", "router": {"experts": 12, "top": 1}, "expert": {"ff": 16, "limit": 0.75},
                 "shared": {"ff": 8, "limit": 3.0}}},
    ],
}

# a width and expert sizes that are no multiples of 8, twenty query heads on one key head, a head wider than the
# matrix-core attention takes, a window longer than any test sequence
SMALL_B = {
    "architecture": "Givizen", "vocab": 130, "width": 50, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.5},
    "logit_softcap": 30.0,
    "layers": [
        {"type": "attention_2",
         "mixer": {"heads": 5, "kv_heads": 1, "dim": 12, "vdim": 20, "scale": 0.4, "softcap": 6.0, "mask": {"size": 64},
                   "q_temp": {"coef": 0.5, "every": 32}},
         "mlp": {"kind": "moe", "router": {"experts": 10, "top": 4}, "expert": {"ff": 30, "limit": 1.0},
                 "shared": {"ff": 22, "limit": 1.5}}},
        {"type": "attention",
         "mixer": {"heads": 20, "kv_heads": 1, "dim": 64, "vdim": 32, "scale": 0.06, "mask": {"size": 1000},
                   "q_temp": {"coef": 0.2, "every": 50}},
         "mlp": {"kind": "moe", "router": {"experts": 5, "top": 2}, "expert": {"ff": 18, "limit": 2.5}}},
        {"type": "attention",
         "mixer": {"heads": 2, "kv_heads": 2, "dim": 136, "vdim": 8, "scale": 0.05, "mask": {"size": 16},
                   "q_temp": {"coef": 0.3, "every": 4}},
         "mlp": None},
    ],
}

SMALL = {"A": SMALL_A, "B": SMALL_B}

MARKERS = 5  # stream coordinates 0..3 hold a token's small integers, coordinate 4 holds 1


def single(layer: dict, width: int = 32, vocab: int = 50, cap=None) -> dict:
    """A model of one layer: a mechanism alone."""
    out = {"architecture": "Givizen", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "embedding": {"scale": 0.5},
           "layers": [layer]}
    if cap:
        out["logit_softcap"] = cap
    return out


def make_weights(raw: dict, seed: int, sharp: float = 1.0, exact_router: bool = False) -> dict[str, torch.Tensor]:
    """Float32 tensors (bfloat16-representable values) for every name the configuration's model expects."""
    from cie_amd.config import config_from_dict
    from cie_amd.parts.model import expected_tensors

    expected = expected_tensors(config_from_dict(raw).model_spec())
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in expected.items():
        if spec.optional:
            continue
        shape = tuple(spec.shape)
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        fan_in = shape[-1] if len(shape) >= 2 else 1
        if leaf in ("norm1", "norm2") or name == "final.norm":
            t = 0.4 * torch.randn(shape, generator=g)              # stored around zero
        elif leaf in ("mix.q.norm", "mix.k.norm"):
            t = 0.5 + torch.rand(shape, generator=g)
        elif leaf == "mix.sink":
            t = torch.linspace(-1.0, 3.0, shape[0])[torch.randperm(shape[0], generator=g)]
        elif leaf in ("mix.q", "mix.k"):
            t = torch.randn(shape, generator=g) * (2.0 * sharp / math.sqrt(fan_in))
        elif leaf == "mix.g":
            t = torch.randn(shape, generator=g) * (3.0 / math.sqrt(fan_in))
        elif leaf.endswith(".gate") or leaf.endswith(".up"):
            t = torch.randn(shape, generator=g) * (2.0 / math.sqrt(fan_in))   # reaches the limits now and then
        elif leaf == "mlp.router":
            t = torch.randn(shape, generator=g) * (2.0 / math.sqrt(fan_in))
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.0 / math.sqrt(fan_in))
        out[name] = t
    if exact_router:
        vocab = out["embed"].shape[0]
        marks = torch.randint(-3, 4, (vocab, MARKERS - 1), generator=g).float()
        out["embed"][:, : MARKERS - 1] = marks
        out["embed"][:, MARKERS - 1] = 1.0
        for name in list(out):
            leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
            if leaf == "mix.o" or leaf.endswith(".down"):
                out[name][:MARKERS] = 0.0                         # no branch writes to the markers
            if leaf == "mlp.router":
                experts = out[name].shape[0]
                router = torch.zeros_like(out[name])
                router[:, : MARKERS - 1] = torch.randint(-2, 3, (experts, MARKERS - 1), generator=g).float() * 0.5
                # no two experts' logits are equal: the other coordinates move a logit in steps of 0.5 markers,
                # this one by less than that in all (and stays exact in bfloat16 up to 128 experts)
                steps = 4 << max(experts - 1, 1).bit_length()
                router[:, MARKERS - 1] = torch.arange(experts).float() / steps
                out[name] = router
    return {name: t.to(torch.bfloat16).float() for name, t in out.items()}
