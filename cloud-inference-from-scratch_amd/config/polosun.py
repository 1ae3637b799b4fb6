"""Configuration of the Polosun decoder, read from its ``config.json``.

The file lists the layers one by one: ``layers[i] = {"type", "mixer", "mlp"}`` with ``type`` one of
``latent_attention``, ``rglru`` and ``retention``, ``mixer`` that mixer's sizes and constants, and ``mlp`` either
``{"kind": "dense", "ff": n}`` or ``null`` (a layer without feed-forward).  Beside them ``vocab``, ``width``,
``residual_mult`` and ``norm.eps``.  Every size and constant comes from the file; nothing is fixed here but the
design's own formulas.  The model has no longest position: rotation tables grow with the context.

Layers are arranged as ``parallel_depth_average`` blocks (``parts/block.py``); tensors are named ``embed``,
``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.norm2``, ``l<i>.mlp.*``, ``l<i>.dwa``, ``final.norm`` and ``head``.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any

from .specs import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec

MIXER_TYPES = ("latent_attention", "rglru", "retention")


def _need(table: dict, keys: tuple, where: str) -> None:
    missing = [key for key in keys if key not in table]
    if missing:
        raise ConfigError(f"{where}: missing {missing}")


def _positive_int(table: dict, key: str, where: str) -> int:
    value = table[key]
    if isinstance(value, bool) or not isinstance(value, int) or value < 1:
        raise ConfigError(f"{where}: {key} must be a positive integer, got {value!r}")
    return value


@dataclass(frozen=True)
class PolosunConfig:
    raw: dict = field(compare=False)

    architecture = "Polosun"

    # -- reading ---------------------------------------------------------------------------
    @classmethod
    def from_hf_config(cls, raw: dict[str, Any]) -> "PolosunConfig":
        _need(raw, ("layers", "norm", "residual_mult", "vocab", "width"), "config")
        if not isinstance(raw["layers"], list) or not raw["layers"]:
            raise ConfigError("config: layers must be a list with at least one layer")
        if not isinstance(raw["norm"], dict) or not float(raw["norm"].get("eps", 0)) > 0:
            raise ConfigError("config: norm.eps must be positive")
        for key in ("vocab", "width"):
            _positive_int(raw, key, "config")
        config = cls(copy.deepcopy(raw))
        spec = config.model_spec()  # (everything else is checked where it is read ...
        from ..parts.model import expected_tensors  # ... or by the parts themselves, built once here)

        try:
            expected_tensors(spec)
        except (KeyError, TypeError, ValueError) as error:
            if isinstance(error, ConfigError):
                raise
            raise ConfigError(f"config: {error}") from error
        return config

    def to_hf_config(self) -> dict[str, Any]:
        out = copy.deepcopy(self.raw)
        out["architecture"] = self.architecture
        return out

    # -- plain properties --------------------------------------------------------------------
    @property
    def hidden_size(self) -> int:
        return int(self.raw["width"])

    @property
    def vocab_size(self) -> int:
        return int(self.raw["vocab"])

    @property
    def eps(self) -> float:
        return float(self.raw["norm"]["eps"])

    # -- what the engine builds from -----------------------------------------------------------
    def _position(self, rot: Any, head_dim: int, where: str) -> PartSpec:
        if not rot:
            return PartSpec.of("none", head_dim=head_dim)
        _need(rot, ("base", "dims"), where + ".rot")
        dims = _positive_int(rot, "dims", where + ".rot")
        if dims % 2 or dims > head_dim:
            raise ConfigError(f"{where}.rot: dims must be even and at most {head_dim}, got {dims}")
        scaling = rot.get("scaling")
        if scaling:
            _need(scaling, ("factor", "original", "fast", "slow"), where + ".rot.scaling")
            scaling = tuple(float(scaling[key]) for key in ("factor", "original", "fast", "slow"))
        return PartSpec.of("rotary_half", head_dim=head_dim, theta=float(rot["base"]), max_position=None,
                           rotary_dim=dims, scaling=scaling or None)

    def _mixer(self, kind: str, sizes: dict, where: str) -> PartSpec:
        width = self.hidden_size
        if kind == "latent_attention":
            _need(sizes, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale"), where)
            rot_dim = int(sizes["rot_dim"])
            rot = sizes.get("rot")
            if rot and int(rot.get("dims", rot_dim)) != rot_dim:
                raise ConfigError(f"{where}: the turned part of a head ({rot_dim}) and rot.dims ({rot.get('dims')}) differ")
            return PartSpec.of(
                "latent_attention", hidden_size=width, num_heads=_positive_int(sizes, "heads", where),
                head_dim=_positive_int(sizes, "dim", where), rot_dim=rot_dim,
                value_dim=_positive_int(sizes, "vdim", where), kv_rank=_positive_int(sizes, "kv_rank", where),
                scale=float(sizes["scale"]), eps=self.eps,
                position=self._position(rot, rot_dim, where) if rot_dim else PartSpec.of("none", head_dim=0))
        if kind == "rglru":
            _need(sizes, ("width", "blocks", "conv"), where)
            return PartSpec.of("gated_linear_recurrence", hidden_size=width, width=_positive_int(sizes, "width", where),
                               blocks=_positive_int(sizes, "blocks", where), taps=_positive_int(sizes, "conv", where))
        if kind == "retention":
            _need(sizes, ("heads", "dim", "vdim", "decay"), where)
            dim = _positive_int(sizes, "dim", where)
            return PartSpec.of("retention", hidden_size=width, num_heads=_positive_int(sizes, "heads", where),
                               head_dim=dim, value_dim=_positive_int(sizes, "vdim", where),
                               decay=tuple(float(d) for d in sizes["decay"]), eps=self.eps,
                               position=self._position(sizes.get("rot"), dim, where))
        raise ConfigError(f"{where}: unknown layer type {kind!r}; known: {MIXER_TYPES}")

    def _feed_forward(self, mlp: Any, where: str) -> PartSpec:
        if mlp is None:
            return PartSpec.of("none", hidden_size=self.hidden_size)
        _need(mlp, ("kind", "ff"), where + ".mlp")
        if mlp["kind"] != "dense":
            raise ConfigError(f"{where}.mlp: unknown kind {mlp['kind']!r}; known: ('dense',)")
        return PartSpec.of("gated_mlp", hidden_size=self.hidden_size,
                           intermediate_size=_positive_int(mlp, "ff", where + ".mlp"), activation="silu",
                           names=("gate", "up", "down"))

    def model_spec(self) -> ModelSpec:
        norm = PartSpec.of("rms_norm_scalar", size=self.hidden_size, eps=self.eps)
        layers = []
        for index, layer in enumerate(self.raw["layers"]):
            where = f"layers[{index}]"
            if not isinstance(layer, dict):
                raise ConfigError(f"{where}: must be a table")
            _need(layer, ("type", "mixer"), where)
            try:
                layers.append(LayerSpec(
                    mixer=self._mixer(layer["type"], layer["mixer"], where),
                    feed_forward=self._feed_forward(layer.get("mlp"), where),
                    norm1=norm, norm2=norm, block="parallel_depth_average",
                    names=(("norm1", "norm1"), ("mixer", "mix"), ("norm2", "norm2"), ("feed_forward", "mlp")),
                    options=(("average_name", "dwa"), ("depth", index), ("mult", float(self.raw["residual_mult"]))),
                ))
            except (TypeError, ValueError) as error:
                if isinstance(error, ConfigError):
                    raise
                raise ConfigError(f"{where}: {error}") from error
        count = len(layers)
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.hidden_size,
            layers=tuple(layers), order=tuple(LayerCall(layer=i, cache=i, writes=True) for i in range(count)),
            final_norm=norm, tie_word_embeddings=False, max_position=1 << 30,
            eos_token_id=self.raw.get("eos_token_id"), embedding_name="embed", final_norm_name="final.norm",
            head_name="head", layer_prefix="l{index}.",
        )
