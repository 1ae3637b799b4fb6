"""CPU: what pins the plain Givizen implementation (tests/plain_givizen.py) and the configuration's reading."""

from __future__ import annotations

import copy
import math

import pytest
import torch
import torch.nn.functional as F

import givizen_util as gu
import plain_givizen as pg
from conftest import random_tokens


def test_norm_is_the_library_norm_with_one_added_to_the_weight():
    x = torch.randn(5, 24, dtype=torch.float64)
    w = torch.randn(24, dtype=torch.float64) * 0.3
    assert torch.allclose(pg.norm_one_plus(x, w, 1e-5), F.rms_norm(x, (24,), 1.0 + w, 1e-5))
    assert torch.allclose(pg.norm_one_plus(x, torch.zeros(24, dtype=torch.float64), 1e-5), x / pg.rms(x, 1e-5))


def test_temperature_steps_with_the_position():
    t = pg.query_temperature(torch.arange(0, 20), {"coef": 0.5, "every": 8})
    assert torch.all(t[:7] == 1.0)                               # floor((p + 1) / 8) = 0 up to p = 6
    assert torch.allclose(t[7:15], torch.full((8,), 1.0 + 0.5 * math.log(2.0), dtype=torch.float64))
    assert torch.allclose(t[15:], torch.full((5,), 1.0 + 0.5 * math.log(3.0), dtype=torch.float64))


def test_slopes_halve_their_exponent_with_the_head():
    s = pg.slopes(8)
    assert s[0] == 0.5 and s[7] == 2.0 ** -8 and torch.allclose(s[1:] / s[:-1], torch.full((7,), 0.5, dtype=torch.float64))
    assert pg.slopes(2)[0] == 2.0 ** -4


@pytest.mark.parametrize("kind", ["attention", "attention_2"])
def test_scores_are_the_library_attention_with_a_bias(kind):
    """Without sink and cap, the weights are the softmax of library attention under an additive mask that holds the
    window and the distance bias; with them, the same by hand."""
    T, H, G, D = 30, 4, 2, 8
    p = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": 0.4, "mask": {"size": 9}}
    if kind == "attention_2":
        p["softcap"] = 1e9                                        # (so large that it changes nothing)
    q = torch.randn(T, H, D, dtype=torch.float64)
    k = torch.randn(T, G, D, dtype=torch.float64)
    v = torch.randn(T, G, D, dtype=torch.float64)
    pos = torch.arange(T)
    s = pg.attention_scores(kind, p, q, k, pos, pos)
    a = pg.attention_weights(kind, s, torch.full((H,), -1e9, dtype=torch.float64))
    distance = (pos[:, None] - pos[None, :]).double()
    bias = -pg.slopes(H)[:, None, None] * distance[None]
    bias = bias.masked_fill(((distance < 0) | (distance >= 9))[None], float("-inf"))
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.repeat_interleave(2, 1).transpose(0, 1)[None],
                                          v.repeat_interleave(2, 1).transpose(0, 1)[None], attn_mask=bias[None], scale=0.4)
    got = torch.einsum("hts,shv->htv", a, v.repeat_interleave(2, 1))
    assert torch.allclose(got, want[0], atol=1e-12)
    # a sink takes its share of every row and of nothing else
    sink = torch.tensor([0.5, -1.0, 2.0, 0.0], dtype=torch.float64)
    with_sink = pg.attention_weights("attention", s, sink)
    share = 1.0 - with_sink.sum(-1)
    e = torch.exp(s - s.max(-1, keepdim=True).values)
    by_hand = torch.exp(sink[:, None] - s.max(-1).values) / (e.sum(-1) + torch.exp(sink[:, None] - s.max(-1).values))
    assert torch.allclose(share, by_hand, atol=1e-12) and bool((share > 0).all())
    # the cap bounds a score before the bias, never after it
    p["softcap"] = 0.5
    capped = pg.attention_scores("attention_2", p, q * 50, k, pos, pos)
    seen = torch.isfinite(capped)
    assert bool(((capped + pg.slopes(H)[:, None, None] * distance[None])[seen].abs() <= 0.5 + 1e-12).all())


def test_an_expert_and_the_router():
    g = torch.Generator().manual_seed(0)
    w = {"gate": torch.randn(6, 10, generator=g, dtype=torch.float64), "up": torch.randn(6, 10, generator=g, dtype=torch.float64),
         "down": torch.randn(10, 6, generator=g, dtype=torch.float64), "router": torch.randn(5, 10, generator=g, dtype=torch.float64)}
    y = torch.randn(3, 10, generator=g, dtype=torch.float64) * 3
    gate = (y @ w["gate"].T).clamp(max=1.5)
    up = (y @ w["up"].T).clamp(-1.5, 1.5)
    assert torch.allclose(pg.expert(w, "", y, 1.5), (gate * torch.sigmoid(1.702 * gate) * (up + 1)) @ w["down"].T)
    assert float(gate.max()) == 1.5 and float(gate.min()) < -1.5  # (the gate is bounded above only)
    chosen, weights = pg.router_choice(w, "", y, 2)
    scores = torch.sigmoid(y @ w["router"].T)
    assert torch.equal(chosen, scores.argsort(dim=1, descending=True)[:, :2])
    assert torch.allclose(weights, scores.gather(1, chosen)) and not torch.allclose(weights.sum(1), torch.ones(3, dtype=torch.float64))
    # the weight is on the input: not the same as on the output
    mlp = {"router": {"experts": 1, "top": 1}, "expert": {"ff": 6, "limit": 1.5}}
    one = {"e0.gate": w["gate"], "e0.up": w["up"], "e0.down": w["down"], "router": w["router"][:1]}
    s = torch.sigmoid(y @ one["router"].T)
    assert torch.allclose(pg.feed_forward(mlp, one, "", y), pg.expert(w, "", s * y, 1.5))
    assert not torch.allclose(pg.feed_forward(mlp, one, "", y), s * pg.expert(w, "", y, 1.5))


@pytest.mark.parametrize("name", sorted(gu.SMALL))
def test_pieces_give_what_the_whole_gives(name):
    raw = gu.SMALL[name]
    w = gu.make_weights(raw, 5)
    tokens = random_tokens(70, raw["vocab"], 3)
    whole = pg.forward(raw, w, tokens)
    stepper = pg.Stepper(raw, w)
    pieces = torch.cat([stepper.feed(tokens[a:b]) for a, b in ((0, 1), (1, 3), (3, 40), (40, 41), (41, 70))])
    assert torch.allclose(whole, pieces, atol=1e-10)
    assert float(whole.abs().max()) < raw["logit_softcap"]


def test_a_layer_adds_the_norm_of_what_its_sublayers_make_of_the_stream_itself():
    raw = gu.single(copy.deepcopy(gu.SMALL_A["layers"][0]), width=64, vocab=96)
    w = gu.make_weights(raw, 2)
    tokens = random_tokens(12, 96, 1)
    layers = []
    pg.forward(raw, w, tokens, layers_out=layers)
    x0 = w["embed"].double()[torch.tensor(tokens)] * 0.5
    mixed, _ = pg.attention_mixer("attention", raw["layers"][0]["mixer"], pg.cast(w, torch.float64), "l0.mix.", x0,
                                  torch.arange(12), 1e-6)
    x1 = x0 + F.rms_norm(mixed, (64,), 1.0 + w["l0.norm1"].double(), 1e-6)
    fed = pg.feed_forward(raw["layers"][0]["mlp"], pg.cast(w, torch.float64), "l0.mlp.", x1)
    assert torch.allclose(layers[0], x1 + F.rms_norm(fed, (64,), 1.0 + w["l0.norm2"].double(), 1e-6), atol=1e-12)


def test_the_configuration_reads_every_size_and_constant():
    from cie_amd.config import ConfigError, GivizenConfig, config_from_dict

    config = config_from_dict(gu.SMALL_A)
    assert isinstance(config, GivizenConfig)
    spec = config.model_spec()
    assert spec.embedding_scale == 0.75 and spec.logit_softcap == 12.0 and spec.vocab_size == 96
    first, second = spec.layers[0].mixer.as_dict(), spec.layers[1].mixer.as_dict()
    assert (first["num_heads"], first["num_kv_heads"], first["head_dim"], first["value_dim"]) == (4, 2, 16, 24)
    assert first["window"] == 20 and first["q_temperature"] == (0.4, 8) and first["sink"] and not first["head_gate"]
    assert first["qk_norm"] == "weight" and first["softcap"] is None and first["slope_base"] == 8.0
    assert second["qk_norm"] == "unit" and second["softcap"] == 4.0 and second["head_gate"] and not second["sink"]
    experts = spec.layers[0].feed_forward.as_dict()
    assert (experts["experts"], experts["top"], experts["expert_ff"], experts["expert_limit"]) == (6, 2, 40, 1.25)
    assert (experts["shared_ff"], experts["shared_limit"]) == (48, 1.75)
    assert spec.layers[1].feed_forward.as_dict()["shared_ff"] is None and spec.layers[2].feed_forward.kind == "none"
    from cie_amd.parts.model import expected_tensors

    names = expected_tensors(spec)
    assert "l0.mix.sink" in names and "l1.mix.g" in names and "l0.mix.g" not in names and "l1.mix.q.norm" not in names
    assert names["l0.mlp.e5.down"].shape == (64, 40) and "l1.mlp.shared.gate" not in names and names["l2.norm2"].optional
    for broken, text in (({"layers": [dict(gu.SMALL_A["layers"][0], type="attention_3")]}, "unknown layer type"),
                         ({"layers": [dict(gu.SMALL_A["layers"][1], mixer={k: v for k, v in gu.SMALL_A["layers"][1]["mixer"].items()
                                                                           if k != "softcap"})]}, "softcap"),
                         ({"norm": {}}, "eps"), ({"width": 0}, "width")):
        with pytest.raises(ConfigError, match=text):
            config_from_dict({**gu.SMALL_A, **broken})
