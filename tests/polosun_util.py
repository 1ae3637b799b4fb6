"""Small Polosun configurations for the tests and weights that make faults show.

Random weights of one small scale would hide most faults: every softmax nearly uniform, every gate near one half,
every decay the same.  ``make_weights`` therefore draws bolder ones: projections large enough for peaked attention
and gates that open and close, decays' parameters spread over their range, depth averages that weigh every earlier
layer, gains away from one.  Everything is rounded to bfloat16 once, so that both precisions run the same model.
"""

from __future__ import annotations

import math

import torch

ROT_SCALED = {"base": 10000.0, "dims": 8, "scaling": {"factor": 4.0, "fast": 16.0, "original": 64, "slow": 1.0}}

# every size differs from its neighbours'; widths that are no powers of two; a layer without feed-forward; one head,
# one block and one tap somewhere; a rotation over a part of the head only, and none at all
SMALL_A = {
    "architecture": "Polosun", "vocab": 96, "width": 64, "residual_mult": 0.5, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "rglru", "mixer": {"width": 48, "blocks": 3, "conv": 4}, "mlp": {"kind": "dense", "ff": 80}},
        {"type": "latent_attention",
         "mixer": {"heads": 3, "dim": 16, "rot_dim": 8, "vdim": 24, "kv_rank": 40, "scale": 0.6, "rot": ROT_SCALED},
         "mlp": {"kind": "dense", "ff": 72}},
        {"type": "retention",
         "mixer": {"heads": 3, "dim": 16, "vdim": 8, "decay": [0.5, 0.96875, 0.998046875], "rot": {"base": 500.0, "dims": 8}},
         "mlp": None},
        {"type": "latent_attention",
         "mixer": {"heads": 1, "dim": 24, "rot_dim": 16, "vdim": 8, "kv_rank": 16, "scale": 0.45,
                   "rot": {"base": 100.0, "dims": 16}},
         "mlp": {"kind": "dense", "ff": 40}},
        {"type": "retention", "mixer": {"heads": 1, "dim": 8, "vdim": 40, "decay": [0.9375]},
         "mlp": {"kind": "dense", "ff": 56}},
        {"type": "rglru", "mixer": {"width": 24, "blocks": 1, "conv": 1}, "mlp": None},
    ],
}

SMALL_B = {
    "architecture": "Polosun", "vocab": 130, "width": 48, "residual_mult": 1.25, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "retention",
         "mixer": {"heads": 2, "dim": 24, "vdim": 24, "decay": [0.75, 0.9921875], "rot": {"base": 50.0, "dims": 24}},
         "mlp": {"kind": "dense", "ff": 64}},
        {"type": "rglru", "mixer": {"width": 80, "blocks": 5, "conv": 2}, "mlp": {"kind": "dense", "ff": 96}},
        {"type": "latent_attention",
         "mixer": {"heads": 5, "dim": 8, "rot_dim": 4, "vdim": 16, "kv_rank": 88, "scale": 1.1,
                   "rot": {"base": 30.0, "dims": 4}},
         "mlp": None},
    ],
}

SMALL = {"A": SMALL_A, "B": SMALL_B}


def single(layer: dict, width: int = 32, vocab: int = 50) -> dict:
    """A model of one layer (without feed-forward unless the layer has one): a mechanism alone."""
    return {"architecture": "Polosun", "vocab": vocab, "width": width, "residual_mult": 0.8, "norm": {"eps": 1e-6},
            "layers": [layer]}


def make_weights(raw: dict, seed: int, sharp: float = 1.0) -> dict[str, torch.Tensor]:
    """Float32 tensors (bfloat16-representable values) for every name the configuration's model expects."""
    from cie_amd.config import config_from_dict
    from cie_amd.parts.model import expected_tensors

    expected = expected_tensors(config_from_dict(raw).model_spec())
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in expected.items():
        shape = tuple(spec.shape)
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        fan_in = shape[-1] if len(shape) >= 2 else 1
        if leaf in ("norm1", "norm2") or name == "final.norm":
            t = 0.6 + 0.8 * torch.rand(shape, generator=g)
        elif leaf == "dwa":
            t = torch.randn(shape, generator=g) * 0.3
            t[-1] += 1.0
        elif leaf == "mix.dkv.norm":
            t = 0.5 + torch.rand(shape, generator=g)
        elif leaf == "mix.lam":
            t = torch.linspace(-6.0, 2.0, shape[0])[torch.randperm(shape[0], generator=g)]
        elif leaf in ("mix.ra", "mix.ri"):
            t = torch.randn(shape, generator=g) * (2.5 / math.sqrt(fan_in))
        elif leaf.endswith(".b"):
            t = torch.randn(shape, generator=g) * 0.5
        elif leaf == "mix.conv":
            t = torch.randn(shape, generator=g) * 0.6
        elif leaf in ("mix.q", "mix.k", "mix.uk", "mix.dkv"):
            t = torch.randn(shape, generator=g) * (1.6 * sharp / math.sqrt(fan_in))
        elif name in ("embed", "head"):
            t = torch.randn(shape, generator=g) * (1.0 if name == "embed" else 1.0 / math.sqrt(fan_in))
        else:
            t = torch.randn(shape, generator=g) * (1.0 / math.sqrt(fan_in))
        if not spec.optional:
            out[name] = t.to(torch.bfloat16).float()
    return out


class Fixed:
    """A weight source that hands out given tensors."""

    def __init__(self, tensors):
        self.tensors = tensors

    def load(self, expected, dtype, device, tied_optional=None):
        target = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
        return {name: self.tensors[name].to(target).to(device) for name in expected if name in self.tensors}


def make_runner(raw, weights, dtype, kv_tokens, page_size=16, max_running=4, max_model_len=None, graph_decode=False):
    from cie_amd.config import build_engine_config, config_from_dict
    from cie_amd.engine import Runner
    from cie_amd.engine.loading import build_model

    model = build_model(config_from_dict(raw))
    model.load(Fixed(weights), dtype, "cuda:0")
    engine_config = build_engine_config(dtype=dtype, page_size=page_size, kv_tokens=kv_tokens, max_running=max_running,
                                        max_model_len=max_model_len or kv_tokens, prefix_cache_pages=0, graph_decode=graph_decode)
    return Runner(model, engine_config, "cuda:0")


def spread(rows: dict, plain: dict) -> tuple[float, float]:
    """(worst, root mean square) difference of the logits with each row's mean taken off, as a share of the plain
    logits' own spread."""
    import numpy as np

    worst, square, count, scale_sq, scale_n = 0.0, 0.0, 0, 0.0, 0
    for rid, by_pos in rows.items():
        for pos, got in by_pos.items():
            want = plain[rid][pos].double().numpy()
            d = got.astype(np.float64) - want
            d = d - d.mean()
            w = want - want.mean()
            scale_sq += float((w ** 2).sum())
            scale_n += w.size
            e = float(np.sqrt((d ** 2).mean()))
            worst = max(worst, e)
            square += e * e
            count += 1
    scale = math.sqrt(scale_sq / scale_n)
    return worst / scale, math.sqrt(square / count) / scale
