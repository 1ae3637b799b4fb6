"""Configuration of the Givizen decoder, read from its ``config.json``.

The file lists the layers one by one: ``layers[i] = {"type", "mixer", "mlp"}``.  ``type`` is ``attention`` (queries
and keys normed per head with a weight, a sink in the softmax) or ``attention_2`` (queries and keys brought to unit
RMS, scores capped, every head's output gated); both see a window (``mixer.mask.size``), scale their queries by the
position (``mixer.q_temp``), take a bias by the distance off the scores and know no rotation.  ``mlp`` is
``{"kind": "moe", "router": {experts, top}, "expert": {ff, limit}, "shared": {ff, limit}}`` or ``null``.  Beside the
layers: ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``, ``logit_softcap``.  Every size and every constant
that the file gives is read from it; what the design itself fixes (the slopes' base 8, the unit's 1.702 and + 1) is
handed to the parts as parameters here.

Layers are ``branch_norm`` blocks (``parts/block.py``); tensors are named ``embed``, ``l<i>.norm1``, ``l<i>.mix.*``,
``l<i>.norm2``, ``l<i>.mlp.*``, ``final.norm`` and ``head``.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any

from .specs import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec

MIXER_TYPES = ("attention", "attention_2")
SLOPE_BASE = 8.0      # head h of H loses 2^(-8 (h + 1) / H) per token of distance
UNIT_ALPHA = 1.702    # the experts' unit: g * sigmoid(1.702 g) * (u + 1)
UNIT_OFFSET = 1.0


def _need(table: Any, keys: tuple, where: str) -> None:
    if not isinstance(table, dict):
        raise ConfigError(f"{where}: must be a table")
    missing = [key for key in keys if key not in table]
    if missing:
        raise ConfigError(f"{where}: missing {missing}")


def _positive_int(table: dict, key: str, where: str) -> int:
    value = table[key]
    if isinstance(value, bool) or not isinstance(value, int) or value < 1:
        raise ConfigError(f"{where}: {key} must be a positive integer, got {value!r}")
    return value


def _positive(table: dict, key: str, where: str) -> float:
    value = table[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not value > 0:
        raise ConfigError(f"{where}: {key} must be a positive number, got {value!r}")
    return float(value)


@dataclass(frozen=True)
class GivizenConfig:
    raw: dict = field(compare=False)

    architecture = "Givizen"

    @classmethod
    def from_hf_config(cls, raw: dict[str, Any]) -> "GivizenConfig":
        _need(raw, ("layers", "norm", "vocab", "width"), "config")
        if not isinstance(raw["layers"], list) or not raw["layers"]:
            raise ConfigError("config: layers must be a list with at least one layer")
        _need(raw["norm"], ("eps",), "config.norm")
        _positive(raw["norm"], "eps", "config.norm")
        for key in ("vocab", "width"):
            _positive_int(raw, key, "config")
        if raw.get("embedding") is not None:
            _need(raw["embedding"], ("scale",), "config.embedding")
        if raw.get("logit_softcap") is not None:
            _positive(raw, "logit_softcap", "config")
        config = cls(copy.deepcopy(raw))
        spec = config.model_spec()
        from ..parts.model import expected_tensors  # (the parts are built once here: what one refuses is a ConfigError)

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

    @property
    def hidden_size(self) -> int:
        return int(self.raw["width"])

    @property
    def vocab_size(self) -> int:
        return int(self.raw["vocab"])

    @property
    def eps(self) -> float:
        return float(self.raw["norm"]["eps"])

    def _mixer(self, kind: str, sizes: Any, where: str) -> PartSpec:
        if kind not in MIXER_TYPES:
            raise ConfigError(f"{where}: unknown layer type {kind!r}; known: {MIXER_TYPES}")
        _need(sizes, ("heads", "kv_heads", "dim", "vdim", "scale"), where)
        window = None
        if sizes.get("mask") is not None:
            _need(sizes["mask"], ("size",), where + ".mask")
            window = _positive_int(sizes["mask"], "size", where + ".mask")
        temperature = None
        if sizes.get("q_temp") is not None:
            _need(sizes["q_temp"], ("coef", "every"), where + ".q_temp")
            temperature = (float(sizes["q_temp"]["coef"]), _positive_int(sizes["q_temp"], "every", where + ".q_temp"))
        second = kind == "attention_2"
        softcap = None
        if second:
            _need(sizes, ("softcap",), where)
            softcap = _positive(sizes, "softcap", where)
        return PartSpec.of(
            "scored_attention", hidden_size=self.hidden_size, num_heads=_positive_int(sizes, "heads", where),
            num_kv_heads=_positive_int(sizes, "kv_heads", where), head_dim=_positive_int(sizes, "dim", where),
            value_dim=_positive_int(sizes, "vdim", where), scale=float(sizes["scale"]), eps=self.eps, window=window,
            qk_norm="unit" if second else "weight", q_temperature=temperature, softcap=softcap,
            slope_base=SLOPE_BASE, sink=not second, head_gate=second)

    def _feed_forward(self, mlp: Any, where: str) -> PartSpec:
        if mlp is None:
            return PartSpec.of("none", hidden_size=self.hidden_size)
        _need(mlp, ("kind", "router", "expert"), where)
        if mlp["kind"] != "moe":
            raise ConfigError(f"{where}: unknown kind {mlp['kind']!r}; known: ('moe',)")
        _need(mlp["router"], ("experts", "top"), where + ".router")
        _need(mlp["expert"], ("ff", "limit"), where + ".expert")
        shared = mlp.get("shared")
        if shared is not None:
            _need(shared, ("ff", "limit"), where + ".shared")
        return PartSpec.of(
            "routed_experts", hidden_size=self.hidden_size,
            experts=_positive_int(mlp["router"], "experts", where + ".router"),
            top=_positive_int(mlp["router"], "top", where + ".router"),
            expert_ff=_positive_int(mlp["expert"], "ff", where + ".expert"),
            expert_limit=_positive(mlp["expert"], "limit", where + ".expert"),
            shared_ff=_positive_int(shared, "ff", where + ".shared") if shared is not None else None,
            shared_limit=_positive(shared, "limit", where + ".shared") if shared is not None else None,
            alpha=UNIT_ALPHA, offset=UNIT_OFFSET)

    def model_spec(self) -> ModelSpec:
        norm = PartSpec.of("rms_norm_one_plus", size=self.hidden_size, eps=self.eps)
        layers = []
        for index, layer in enumerate(self.raw["layers"]):
            where = f"layers[{index}]"
            _need(layer, ("type", "mixer"), where)
            try:
                layers.append(LayerSpec(
                    mixer=self._mixer(layer["type"], layer["mixer"], where + ".mixer"),
                    feed_forward=self._feed_forward(layer.get("mlp"), where + ".mlp"),
                    norm1=norm, norm2=norm, block="branch_norm",
                    names=(("norm1", "norm1"), ("mixer", "mix"), ("norm2", "norm2"), ("feed_forward", "mlp")),
                ))
            except (TypeError, ValueError) as error:
                if isinstance(error, ConfigError):
                    raise
                raise ConfigError(f"{where}: {error}") from error
        embedding = self.raw.get("embedding") or {}
        cap = self.raw.get("logit_softcap")
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.hidden_size,
            layers=tuple(layers), order=tuple(LayerCall(layer=i, cache=i, writes=True) for i in range(len(layers))),
            final_norm=norm, tie_word_embeddings=False, max_position=1 << 30,
            eos_token_id=self.raw.get("eos_token_id"), embedding_name="embed", final_norm_name="final.norm",
            head_name="head", layer_prefix="l{index}.", embedding_scale=float(embedding.get("scale", 1.0)),
            logit_softcap=float(cap) if cap is not None else None,
        )
