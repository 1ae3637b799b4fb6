"""No GPU: the Polosun configuration reader, the tensors it expects, the rotation tables, and what pins the plain
implementation (each mechanism in a second, independent formulation)."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import plain_polosun as plain
import polosun_util as pu


def test_configuration_names_every_tensor_and_reads_every_size():
    from cie_amd.config import ConfigError, PolosunConfig, config_from_dict
    from cie_amd.parts.model import expected_tensors

    config = config_from_dict(pu.SMALL_A)
    assert isinstance(config, PolosunConfig) and config.to_hf_config()["architecture"] == "Polosun"
    assert config_from_dict(config.to_hf_config()).to_hf_config() == config.to_hf_config()
    spec = config.model_spec()
    assert [layer.mixer.kind for layer in spec.layers] == [
        "gated_linear_recurrence", "latent_attention", "retention", "latent_attention", "retention", "gated_linear_recurrence"]
    expected = expected_tensors(spec)
    assert tuple(expected["embed"].shape) == (96, 64) and tuple(expected["head"].shape) == (96, 64)
    assert tuple(expected["final.norm"].shape) == () and tuple(expected["l0.norm1"].shape) == ()
    assert tuple(expected["l0.mix.ra"].shape) == (3, 16, 16) and tuple(expected["l0.mix.conv"].shape) == (48, 4)
    assert tuple(expected["l1.mix.q"].shape) == (3 * 24, 64) and tuple(expected["l1.mix.dkv"].shape) == (48, 64)
    assert tuple(expected["l1.mix.uk"].shape) == (48, 40) and tuple(expected["l1.mix.uv"].shape) == (72, 40)
    assert tuple(expected["l2.mix.v"].shape) == (24, 64) and tuple(expected["l4.mix.g"].shape) == (40, 64)
    assert [tuple(expected[f"l{i}.dwa"].shape) for i in range(6)] == [(i + 2,) for i in range(6)]
    # a layer without feed-forward has no feed-forward tensors; a second norm is tolerated, not asked for
    assert "l2.mlp.gate" not in expected and expected["l2.norm2"].optional and not expected["l1.norm2"].optional
    for damage, message in (
            (lambda raw: raw["layers"][0].update(type="window"), "unknown layer type"),
            (lambda raw: raw["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
            (lambda raw: raw["layers"][2]["mixer"].update(decay=[0.5]), "one decay per head"),
            (lambda raw: raw["layers"][0]["mixer"].update(blocks=5), "blocks"),
            (lambda raw: raw["layers"][3]["mlp"].update(kind="routed"), "unknown kind"),
            (lambda raw: raw.pop("residual_mult"), "residual_mult"),
            (lambda raw: raw["layers"][1]["mixer"]["rot"].update(dims=6), "differ")):
        raw = copy.deepcopy(pu.SMALL_A)
        damage(raw)
        with pytest.raises(ConfigError, match=message):
            config_from_dict(raw)


def test_a_folder_round_trip_and_an_extra_second_norm(tmp_path):
    from cie_amd.config import load_config
    from cie_amd.parts.model import expected_tensors
    from cie_amd.weights import SafetensorsSource, WeightError, write_tensors

    weights = pu.make_weights(pu.SMALL_B, seed=1)
    folder = write_tensors(tmp_path / "m", pu.SMALL_B, {k: v.to(torch.bfloat16) for k, v in weights.items()})
    expected = expected_tensors(load_config(folder).model_spec())
    loaded = SafetensorsSource(folder).load(expected, "float32", "cpu")
    assert set(loaded) == set(weights) and all(torch.equal(loaded[k], weights[k]) for k in weights)
    extra = dict(weights, **{"l2.norm2": torch.tensor(1.0)})
    folder = write_tensors(tmp_path / "n", pu.SMALL_B, {k: v.to(torch.bfloat16) for k, v in extra.items()})
    assert "l2.norm2" in SafetensorsSource(folder).load(expected, "float32", "cpu")
    del extra["l1.norm2"]
    folder = write_tensors(tmp_path / "o", pu.SMALL_B, {k: v.to(torch.bfloat16) for k, v in extra.items()})
    with pytest.raises(WeightError, match="l1.norm2"):
        SafetensorsSource(folder).load(expected, "float32", "cpu")


@pytest.mark.parametrize("rot", [pu.ROT_SCALED, {"base": 500000.0, "dims": 24},
                                 {"base": 1000.0, "dims": 16, "scaling": {"factor": 8.0, "fast": 8.0, "original": 32, "slow": 0.5}}])
def test_rotation_tables_grow_and_follow_the_frequencies(rot):
    from cie_amd.parts.position import RotaryHalf

    scaling = rot.get("scaling")
    part = RotaryHalf(rot["dims"] + 8, rot["base"], None, rot["dims"],
                      tuple(scaling[k] for k in ("factor", "original", "fast", "slow")) if scaling else None)
    cos, sin = part.tables("cpu", 10)
    first = cos.shape[0]
    cos, sin = part.tables("cpu", first + 1)
    assert cos.shape[0] == 2 * first and part.tables("cpu", 5)[0].shape[0] == 2 * first
    f, gain = plain.frequencies(rot)
    positions = torch.tensor([0, 1, 7, first + 1, 2 * first - 1], dtype=torch.float64)
    angle = positions[:, None] * f[None, :]
    # float32 angles: an error of position * 2^-24 of the angle
    assert torch.allclose(cos[positions.long()].double(), angle.cos() * gain, atol=2e-3 * gain)
    assert torch.allclose(sin[positions.long()].double(), angle.sin() * gain, atol=2e-3 * gain)
    assert torch.allclose(cos[:8].double(), (torch.arange(8.0, dtype=torch.float64)[:, None] * f[None, :]).cos() * gain, atol=1e-6)
    if scaling:
        plainf = rot["base"] ** (-2.0 * torch.arange(rot["dims"] // 2, dtype=torch.float64) / rot["dims"])
        assert float(f[0]) == pytest.approx(float(plainf[0])) and float(f[-1]) == pytest.approx(float(plainf[-1]) / scaling["factor"])
        assert gain == pytest.approx(0.1 * math.log(scaling["factor"]) + 1.0)


# ---------------------------------------------------------------- what pins the plain implementation
def _one_layer(kind, mixer):
    raw = pu.single({"type": kind, "mlp": None, "mixer": mixer})
    return raw, {k: v.double() for k, v in pu.make_weights(raw, seed=5).items()}


def test_plain_retention_equals_its_sum_over_the_past():
    """o_t = sum_{j <= t} decay^(t - j) (q_t . k_j) v_j, normed: the recurrence unrolled."""
    p = {"heads": 2, "dim": 6, "vdim": 5, "decay": [0.9, 0.5], "rot": {"base": 100.0, "dims": 4}}
    raw, w = _one_layer("retention", p)
    hs = torch.randn(9, 32, dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    state = plain.RetentionState(2, 6, 5, torch.float64)
    got = torch.stack([plain.retention_token(p, w, "l0.mix.", 1e-6, h, t, state) for t, h in enumerate(hs)])
    pos = torch.arange(9)
    q = plain.rotate((hs @ w["l0.mix.q"].T).reshape(9, 2, 6), pos, p["rot"])
    k = plain.rotate((hs @ w["l0.mix.k"].T).reshape(9, 2, 6), pos, p["rot"]) / math.sqrt(6)
    v = (hs @ w["l0.mix.v"].T).reshape(9, 2, 5)
    for t in range(9):
        o = torch.zeros(2, 5, dtype=torch.float64)
        for j in range(t + 1):
            for h in range(2):
                o[h] += p["decay"][h] ** (t - j) * (q[t, h] @ k[j, h]) * v[j, h]
        o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-6)
        want = w["l0.mix.o"] @ (o.reshape(-1) * torch.nn.functional.silu(w["l0.mix.g"] @ hs[t]))
        assert torch.allclose(got[t], want, atol=1e-10)
    # the rotation makes q . k depend on the distance only
    a = plain.rotate(torch.ones(1, 1, 6, dtype=torch.float64), torch.tensor([3]), p["rot"])
    b = plain.rotate(torch.ones(1, 1, 6, dtype=torch.float64), torch.tensor([10]), p["rot"])
    c = plain.rotate(torch.ones(1, 1, 6, dtype=torch.float64), torch.tensor([13]), p["rot"])
    d = plain.rotate(torch.ones(1, 1, 6, dtype=torch.float64), torch.tensor([20]), p["rot"])
    assert torch.allclose((a * b).sum(), (c * d).sum(), atol=1e-12)


def test_plain_latent_attention_equals_its_folded_form():
    """Queries folded into the latent space and the value expansion applied after the sum give the same output as
    keys and values expanded per head."""
    p = {"heads": 3, "dim": 4, "rot_dim": 2, "vdim": 5, "kv_rank": 7, "scale": 0.8, "rot": {"base": 10.0, "dims": 2}}
    raw, w = _one_layer("latent_attention", p)
    hs = torch.randn(6, 32, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    state = plain.LatentAttentionState()
    got = torch.stack([plain.latent_attention_token(p, w, "l0.mix.", 1e-6, h, t, state) for t, h in enumerate(hs)])
    c = torch.stack(state.latents)
    kr = torch.stack(state.shared)
    uk = w["l0.mix.uk"].reshape(3, 4, 7)
    uv = w["l0.mix.uv"].reshape(3, 5, 7)
    for t in range(6):
        q = (w["l0.mix.q"] @ hs[t]).reshape(3, 6)
        qr = plain.rotate(q[None, :, 4:], torch.tensor([t]), p["rot"])[0]
        folded = torch.einsum("hd,hdc->hc", q[:, :4], uk)
        scores = (folded @ c[: t + 1].T + qr @ kr[: t + 1].T) * 0.8
        mixed = torch.einsum("hc,hvc->hv", torch.softmax(scores, -1) @ c[: t + 1], uv).reshape(-1)
        want = w["l0.mix.o"] @ (mixed * torch.sigmoid(w["l0.mix.g"] @ hs[t]))
        assert torch.allclose(got[t], want, atol=1e-10)


def test_plain_recurrence_and_convolution_against_library_routines():
    p = {"width": 12, "blocks": 3, "conv": 4}
    raw, w = _one_layer("rglru", p)
    hs = torch.randn(10, 32, dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    state = plain.RglruState(12, 4, torch.float64)
    got = torch.stack([plain.rglru_token(p, w, "l0.mix.", h, state) for h in hs])
    x = hs @ w["l0.mix.x"].T + w["l0.mix.x.b"]
    u = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (3, 0)), w["l0.mix.conv"][:, None, :],
                                   w["l0.mix.conv.b"], groups=12)[0].T
    y = torch.nn.functional.gelu(hs @ w["l0.mix.y"].T + w["l0.mix.y.b"], approximate="tanh")
    r = torch.sigmoid(u @ torch.block_diag(*w["l0.mix.ra"]).T + w["l0.mix.ra.b"].reshape(-1))
    i = torch.sigmoid(u @ torch.block_diag(*w["l0.mix.ri"]).T + w["l0.mix.ri.b"].reshape(-1))
    a = torch.exp(-8.0 * r * torch.nn.functional.softplus(w["l0.mix.lam"]))
    s = torch.zeros(12, dtype=torch.float64)
    for t in range(10):
        s = a[t] * s + torch.sqrt(1 - a[t] ** 2) * i[t] * u[t]
        assert torch.allclose(got[t], w["l0.mix.o"] @ (s * y[t]), atol=1e-10)


def test_plain_model_composes_branches_and_depth_average():
    """Two layers by hand from the mechanisms: both branches read the same normed stream, their sum is weighed by the
    multiplier, and each layer's input is the weighted sum of the embedding and all earlier layers' results."""
    raw = copy.deepcopy(pu.SMALL_B)
    raw["layers"] = raw["layers"][:2]
    w = {k: v.double() for k, v in pu.make_weights(raw, seed=2).items()}
    tokens = [3, 100, 7, 7, 52]
    streams = []
    got = plain.forward(raw, w, tokens, streams=streams)
    norm = lambda x, g: x / torch.sqrt((x * x).mean() + 1e-6) * g
    s0 = plain.RetentionState(2, 24, 24, torch.float64)
    s1 = plain.RglruState(80, 2, torch.float64)
    for t, token in enumerate(tokens):
        x0 = w["embed"][token]
        b0 = plain.retention_token(raw["layers"][0]["mixer"], w, "l0.mix.", 1e-6, norm(x0, w["l0.norm1"]), t, s0) \
            + plain.dense_feed_forward(w, "l0.mlp.", norm(x0, w["l0.norm2"]))
        x1 = x0 + 1.25 * b0
        in1 = w["l0.dwa"][0] * x0 + w["l0.dwa"][1] * x1
        b1 = plain.rglru_token(raw["layers"][1]["mixer"], w, "l1.mix.", norm(in1, w["l1.norm1"]), s1) \
            + plain.dense_feed_forward(w, "l1.mlp.", norm(in1, w["l1.norm2"]))
        x2 = in1 + 1.25 * b1
        out = w["l1.dwa"][0] * x0 + w["l1.dwa"][1] * x1 + w["l1.dwa"][2] * x2
        assert torch.allclose(streams[t][0], in1, atol=1e-12) and torch.allclose(streams[t][1], out, atol=1e-12)
        assert torch.allclose(got[t], w["head"] @ norm(out, w["final.norm"]), atol=1e-10)


def test_retention_kernel_plan_fits_its_limits():
    from cie_amd.kernels import ops

    for dim, vdim in ((32, 64), (8, 40), (128, 256), (256, 64), (4, 72), (32, 1024), (512, 512), (3, 5), (1024, 64)):
        for units in (1, 8, 64, 1000):
            rows, groups, parts, piece, chunk = ops.plan_retention(dim, vdim, units)
            assert rows in ops.RETENTION_ROWS and rows * groups * parts >= dim and piece <= min(vdim, 64)
            threads = -(-piece * groups // 64) * 64
            assert threads <= 512 and (parts - 1) * rows * groups < dim
            assert chunk >= 1 and chunk * (2 * rows * groups + piece + groups * piece) <= ops.RETENTION_LDS_FLOATS
            assert chunk * 2 * rows * groups // 4 <= 6 * threads and chunk * piece <= 12 * threads


def test_the_command_line_writes_a_model_folder_of_this_design(tmp_path, capsys):
    import json

    from cie_amd import cli
    from cie_amd.config import load_config

    config_file = tmp_path / "config.json"
    config_file.write_text(json.dumps(pu.SMALL_B))
    assert cli.main(["init-model", "--config", str(config_file), "--out", str(tmp_path / "model"), "--seed", "3"]) == 0
    assert load_config(tmp_path / "model").to_hf_config()["layers"][2]["type"] == "latent_attention"
    from safetensors import safe_open

    with safe_open(str(tmp_path / "model" / "model.safetensors"), framework="pt") as handle:
        names = set(handle.keys())
    assert "l2.mix.dkv.norm" in names and "l2.norm2" not in names and "l1.norm2" in names
    assert cli.main(["models"]) == 0
    assert "Polosun" in capsys.readouterr().out
