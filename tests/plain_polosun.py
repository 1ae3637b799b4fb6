"""A plain, slow Polosun: one function per mechanism, written from the design's equations with torch tensor
arithmetic only, token by token where the design has a recurrence.  It shares no code with the package; the tests
compare the engine with it.

A model is ``(raw, weights)``: ``raw`` the dictionary a ``config.json`` of this design holds, ``weights`` a
name -> tensor dictionary.  Everything runs in ``dtype`` (float64 by default, the yardstick; float32 to see what 32
bits alone cost).  ``forward`` runs whole sequences; ``Stepper`` keeps what a sequence needs from token to token
(latents, states, the convolution's last inputs) and is fed any number of tokens at a time.
"""

from __future__ import annotations

import math

import torch


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def unit_rms(x, eps):
    """x over the root of (its mean square + eps), along the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


# ---------------------------------------------------------------- rotation
def frequencies(rot, dtype=torch.float64):
    """One frequency per rotated pair and the factor on cos and sin: base^(-2i/n), stretched pair by pair where
    the configuration has a ``scaling``."""
    n = int(rot["dims"])
    i = torch.arange(n // 2, dtype=torch.float64)
    f = float(rot["base"]) ** (-2.0 * i / n)
    gain = 1.0
    s = rot.get("scaling")
    if s:
        def turn(t):  # the (fractional) pair index that makes t turns over the original length
            return n * math.log(float(s["original"]) / (2.0 * math.pi * t)) / (2.0 * math.log(float(rot["base"])))
        lo = max(math.floor(turn(float(s["fast"]))), 0)
        hi = min(math.ceil(turn(float(s["slow"]))), n - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / float(s["factor"]) * ramp + f * (1.0 - ramp)
        gain = 0.1 * math.log(float(s["factor"])) + 1.0
    return f.to(dtype), gain


def rotate(x, positions, rot, dtype=None):
    """x [T, heads, D]: the first ``dims`` numbers of every head turn, pair (i, i + dims/2) by position * f_i."""
    if not rot:
        return x
    dtype = dtype or x.dtype
    n = int(rot["dims"])
    f, gain = frequencies(rot, torch.float32 if dtype == torch.float32 else torch.float64)
    angle = positions.to(f.dtype)[:, None] * f[None, :]
    cos = (angle.cos() * gain).to(x.dtype)[:, None, :]
    sin = (angle.sin() * gain).to(x.dtype)[:, None, :]
    u, v, rest = x[..., : n // 2], x[..., n // 2: n], x[..., n:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, rest], dim=-1)


# ---------------------------------------------------------------- mixers, one token at a time
class LatentAttentionState:
    def __init__(self):
        self.latents = []   # per token: the normed latent
        self.shared = []    # per token: the rotated key part that all heads share


def latent_attention_token(p, w, pre, eps, h, position, state):
    """One token of the attention over compressed keys.  h [width]."""
    heads, dim, rot_dim, vdim, rank = (int(p[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
    pos = torch.tensor([position])
    q = (w[pre + "q"] @ h).reshape(heads, dim + rot_dim)
    q_plain, q_turned = q[:, :dim], rotate(q[None, :, dim:], pos, p.get("rot"))[0]
    down = w[pre + "dkv"] @ h
    latent = unit_rms(down[:rank], eps) * w[pre + "dkv.norm"]
    shared = rotate(down[None, None, rank:], pos, p.get("rot"))[0, 0]
    state.latents.append(latent)
    state.shared.append(shared)
    c = torch.stack(state.latents)                       # [n, rank]
    kr = torch.stack(state.shared)                       # [n, rot_dim]
    keys = (c @ w[pre + "uk"].T).reshape(-1, heads, dim)     # [n, heads, dim]
    values = (c @ w[pre + "uv"].T).reshape(-1, heads, vdim)
    scores = (torch.einsum("hd,nhd->hn", q_plain, keys) + q_turned @ kr.T) * float(p["scale"])
    weights = torch.softmax(scores, dim=-1)
    mixed = torch.einsum("hn,nhv->hv", weights, values).reshape(-1)
    return w[pre + "o"] @ (mixed * torch.sigmoid(w[pre + "g"] @ h))


class RglruState:
    def __init__(self, width, taps, dtype):
        self.s = torch.zeros(width, dtype=dtype)
        self.inputs = torch.zeros(max(taps - 1, 0), width, dtype=dtype)   # the convolution's last inputs, oldest first


def rglru_token(p, w, pre, h, state):
    """One token of the gated linear recurrence with its short convolution.  h [width of the model]."""
    width, blocks = int(p["width"]), int(p["blocks"])
    y = gelu_tanh(w[pre + "y"] @ h + w[pre + "y.b"])
    x = w[pre + "x"] @ h + w[pre + "x.b"]
    window = torch.cat([state.inputs, x[None, :]], dim=0)        # [taps, width], the last row is this token's
    u = (window * w[pre + "conv"].T).sum(dim=0) + w[pre + "conv.b"]
    state.inputs = window[1:]
    part = u.reshape(blocks, width // blocks)
    r = torch.sigmoid(torch.einsum("boi,bi->bo", w[pre + "ra"], part) + w[pre + "ra.b"]).reshape(-1)
    i = torch.sigmoid(torch.einsum("boi,bi->bo", w[pre + "ri"], part) + w[pre + "ri.b"]).reshape(-1)
    log_a = -8.0 * r * torch.nn.functional.softplus(w[pre + "lam"])
    a = torch.exp(log_a)
    state.s = a * state.s + torch.sqrt(1.0 - a * a) * i * u
    return w[pre + "o"] @ (state.s * y)


class RetentionState:
    def __init__(self, heads, dim, vdim, dtype):
        self.s = torch.zeros(heads, dim, vdim, dtype=dtype)


def retention_token(p, w, pre, eps, h, position, state):
    """One token of the decayed outer-product memory."""
    heads, dim, vdim = int(p["heads"]), int(p["dim"]), int(p["vdim"])
    pos = torch.tensor([position])
    q = rotate((w[pre + "q"] @ h).reshape(1, heads, dim), pos, p.get("rot"))[0]
    k = rotate((w[pre + "k"] @ h).reshape(1, heads, dim), pos, p.get("rot"))[0] * dim ** -0.5
    v = (w[pre + "v"] @ h).reshape(heads, vdim)
    decay = torch.tensor([float(d) for d in p["decay"]], dtype=h.dtype)
    state.s = decay[:, None, None] * state.s + k[:, :, None] * v[:, None, :]
    out = torch.einsum("hdv,hd->hv", state.s, q)
    out = unit_rms(out, eps).reshape(-1)
    return w[pre + "o"] @ (out * silu(w[pre + "g"] @ h))


def dense_feed_forward(w, pre, h):
    return w[pre + "down"] @ (silu(w[pre + "gate"] @ h) * (w[pre + "up"] @ h))


# ---------------------------------------------------------------- the model
class Stepper:
    """One sequence, fed token by token."""

    def __init__(self, raw, weights, dtype=torch.float64):
        self.raw = raw
        self.dtype = dtype
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
        self.position = 0
        self.eps = float(raw["norm"]["eps"])
        self.states = []
        for layer in raw["layers"]:
            p = layer["mixer"]
            if layer["type"] == "latent_attention":
                self.states.append(LatentAttentionState())
            elif layer["type"] == "rglru":
                self.states.append(RglruState(int(p["width"]), int(p["conv"]), dtype))
            elif layer["type"] == "retention":
                self.states.append(RetentionState(int(p["heads"]), int(p["dim"]), int(p["vdim"]), dtype))
            else:
                raise ValueError(layer["type"])

    def norm(self, name, x):
        return unit_rms(x, self.eps) * self.w[name]

    def token(self, token_id, streams=None):
        """Logits after this token.  ``streams``, a list, receives the stream after every layer."""
        w, m = self.w, float(self.raw["residual_mult"])
        x = w["embed"][token_id]
        outputs = [x]                       # what the embedding and every layer so far left, before any averaging
        for index, layer in enumerate(self.raw["layers"]):
            pre = f"l{index}."
            h = self.norm(pre + "norm1", x)
            kind, p, state = layer["type"], layer["mixer"], self.states[index]
            if kind == "latent_attention":
                branch = latent_attention_token(p, w, pre + "mix.", self.eps, h, self.position, state)
            elif kind == "rglru":
                branch = rglru_token(p, w, pre + "mix.", h, state)
            else:
                branch = retention_token(p, w, pre + "mix.", self.eps, h, self.position, state)
            if layer.get("mlp"):
                branch = branch + dense_feed_forward(w, pre + "mlp.", self.norm(pre + "norm2", x))
            outputs.append(x + m * branch)
            x = sum(w[pre + "dwa"][j] * outputs[j] for j in range(index + 2))
            if streams is not None:
                streams.append(x)
        self.position += 1
        return w["head"] @ self.norm("final.norm", x)


def forward(raw, weights, tokens, dtype=torch.float64, streams=None):
    """Logits [len(tokens), vocab] of one sequence.  ``streams`` (a list) receives [layers, width] per token."""
    stepper = Stepper(raw, weights, dtype)
    rows = []
    for token in tokens:
        per_layer = [] if streams is not None else None
        rows.append(stepper.token(int(token), per_layer))
        if streams is not None:
            streams.append(torch.stack(per_layer))
    return torch.stack(rows)


def generate_greedy(raw, weights, prompt, steps, dtype=torch.float64):
    stepper = Stepper(raw, weights, dtype)
    logits = None
    for token in prompt:
        logits = stepper.token(int(token))
    out = []
    for _ in range(steps):
        out.append(int(torch.argmax(logits)))
        logits = stepper.token(out[-1])
    return out
