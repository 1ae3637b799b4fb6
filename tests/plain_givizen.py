"""A plain, slow Givizen: one function per mechanism, written from the design's equations with torch tensor
arithmetic only.  It shares no code with the package; the tests compare the engine with it.

A model is ``(raw, weights)``: ``raw`` the dictionary a ``config.json`` of this design holds, ``weights`` a
name -> tensor dictionary.  Everything runs in ``dtype`` (float64 by default, the yardstick).  ``forward`` runs a
whole sequence and can hand back the stream after every layer; ``Stepper`` keeps a sequence's keys and values from
call to call and is fed any number of tokens at a time.

The design in this file's notation (t a token at position p, h the stream at a sublayer's input):

    x_0 = E[token] * c_embed
    x <- x + N1(mix(x)),  x <- x + N2(ff(x))          N(y) = y / rms(y) * (1 + w);  rms(y) = sqrt(mean(y^2) + eps)
    logits = cap_L(H N_final(x)),  cap_c(z) = c tanh(z / c)

    attention, query head a of H on key head floor(a / (H / G)):
      q, k = per-head norm of W_q h, W_k h   (kind 'attention': y / rms(y) * w;  'attention_2': y / rms(y))
      q <- q * (1 + coef * ln(floor((p + 1) / every) + 1))
      s_ij = (q_i . k_j) * scale          ('attention_2': s <- cap_c(s))
      s_ij <- s_ij - 2^(-8 (a + 1) / H) * (i - j)          for 0 <= i - j < window, nothing else is seen
      'attention':   o_i = sum_j e^(s_ij) v_j / (e^(sink_a) + sum_j e^(s_ij))
      'attention_2': o_i = softmax_j(s_ij) v_j * sigmoid(W_g h)_a
      out = W_o concat(o)

    feed-forward: z = W_r h, s = sigmoid(z), the `top` largest s chosen;
      out = sum_chosen expert_e(s_e h) + shared(h)
      expert(y): g = min(W_gate y, L), u = clamp(W_up y, -L, L); W_down (g sigmoid(1.702 g) (u + 1))
"""

from __future__ import annotations

import math

import torch


def rms(x, eps):
    return torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """RMS norm whose stored weight lies around zero."""
    return x / rms(x, eps) * (1.0 + w)


def soft_cap(z, cap):
    return cap * torch.tanh(z / cap)


def slopes(heads: int, dtype=torch.float64):
    return torch.tensor([2.0 ** (-8.0 * (a + 1) / heads) for a in range(heads)], dtype=dtype)


def query_temperature(positions, q_temp, dtype=torch.float64):
    """1 + coef ln(floor((p + 1) / every) + 1) for integer positions."""
    if not q_temp:
        return torch.ones(len(positions), dtype=dtype)
    steps = torch.div(positions + 1, int(q_temp["every"]), rounding_mode="floor")
    return 1.0 + float(q_temp["coef"]) * torch.log(steps.to(dtype) + 1.0)


def head_norms(kind, p, w, pre, q, k, eps):
    """q [T, H, D], k [T, G, D] after the per-head norm of the layer's kind."""
    if kind == "attention":
        return q / rms(q, eps) * w[pre + "q.norm"], k / rms(k, eps) * w[pre + "k.norm"]
    return q / rms(q, eps), k / rms(k, eps)


def attention_scores(kind, p, q, keys, q_pos, k_pos):
    """Scores of queries q [T, H, D] at positions q_pos against keys [S, G, D] at k_pos: [H, T, S], hidden pairs
    at -inf.  The cap comes before the distance bias; the bias is on the distance itself."""
    heads, groups = q.shape[1], keys.shape[1]
    each = heads // groups
    k_full = keys.repeat_interleave(each, dim=1)                      # [S, H, D]
    s = torch.einsum("thd,shd->hts", q, k_full) * float(p["scale"])
    if kind == "attention_2" and p.get("softcap"):
        s = soft_cap(s, float(p["softcap"]))
    distance = (q_pos[:, None] - k_pos[None, :])                          # [T, S]
    s = s - slopes(heads, s.dtype)[:, None, None] * distance.to(s.dtype)[None]
    seen = distance >= 0
    if p.get("mask"):
        seen = seen & (distance < int(p["mask"]["size"]))
    return s.masked_fill(~seen[None], float("-inf"))


def attention_weights(kind, s, sink):
    """Softmax over the last axis; with a sink the denominator holds exp(sink) once more (per head)."""
    m = s.max(dim=-1, keepdim=True).values
    if kind == "attention":
        m = torch.maximum(m, sink[:, None, None])
    e = torch.exp(s - m)
    total = e.sum(dim=-1, keepdim=True)
    if kind == "attention":
        total = total + torch.exp(sink[:, None, None] - m)
    return e / total


def attention_mixer(kind, p, w, pre, h, positions, eps, past=None):
    """h [T, width] at ``positions``; ``past`` = (keys, values, their positions) of earlier tokens or None.
    Returns the output [T, width] and the new (keys, values, positions)."""
    heads, groups, dim, vdim = (int(p[n]) for n in ("heads", "kv_heads", "dim", "vdim"))
    T = h.shape[0]
    q = (h @ w[pre + "q"].T).reshape(T, heads, dim)
    k = (h @ w[pre + "k"].T).reshape(T, groups, dim)
    v = (h @ w[pre + "v"].T).reshape(T, groups, vdim)
    q, k = head_norms(kind, p, w, pre, q, k, eps)
    q = q * query_temperature(positions, p.get("q_temp"), h.dtype)[:, None, None]
    if past is not None:
        k, v, k_pos = torch.cat([past[0], k]), torch.cat([past[1], v]), torch.cat([past[2], positions])
    else:
        k_pos = positions
    s = attention_scores(kind, p, q, k, positions, k_pos)
    a = attention_weights(kind, s, w[pre + "sink"] if kind == "attention" else None)
    v_full = v.repeat_interleave(heads // groups, dim=1)               # [S, H, V]
    o = torch.einsum("hts,shv->thv", a, v_full)
    if kind == "attention_2":
        o = o * torch.sigmoid(h @ w[pre + "g"].T)[:, :, None]
    return o.reshape(T, heads * vdim) @ w[pre + "o"].T, (k, v, k_pos)


def expert(w, pre, y, limit):
    g = torch.clamp(y @ w[pre + "gate"].T, max=limit)
    u = torch.clamp(y @ w[pre + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


def router_choice(w, pre, h, top):
    """(indices [T, top], weights [T, top]): the experts with the largest sigmoid scores, scores as they are."""
    s = torch.sigmoid(h @ w[pre + "router"].T)
    weights, chosen = torch.topk(s, top, dim=-1)
    return chosen, weights


def feed_forward(mlp, w, pre, h):
    out = torch.zeros_like(h)
    chosen, weights = router_choice(w, pre, h, int(mlp["router"]["top"]))
    limit = float(mlp["expert"]["limit"])
    for t in range(h.shape[0]):
        for e, s in zip(chosen[t].tolist(), weights[t]):
            out[t] += expert(w, f"{pre}e{e}.", s * h[t], limit)      # the weight is on the expert's input
    if mlp.get("shared"):
        out = out + expert(w, pre + "shared.", h, float(mlp["shared"]["limit"]))
    return out


def cast(weights, dtype):
    return {name: (t.to(dtype) if t.is_floating_point() else t) for name, t in weights.items()}


class Stepper:
    """One sequence, fed in pieces."""

    def __init__(self, raw, weights, dtype=torch.float64):
        self.raw, self.w, self.dtype = raw, cast(weights, dtype), dtype
        self.past = [None] * len(raw["layers"])
        self.length = 0

    def feed(self, tokens, layers_out=None):
        """Logits [len(tokens), vocab] of the next tokens."""
        raw, w = self.raw, self.w
        eps = float(raw["norm"]["eps"])
        positions = torch.arange(self.length, self.length + len(tokens))
        x = w["embed"][torch.tensor(tokens)] * float(raw["embedding"]["scale"])
        for i, layer in enumerate(raw["layers"]):
            pre = f"l{i}."
            mixed, self.past[i] = attention_mixer(layer["type"], layer["mixer"], w, pre + "mix.", x, positions, eps,
                                                  self.past[i])
            x = x + norm_one_plus(mixed, w[pre + "norm1"], eps)
            if layer.get("mlp"):
                x = x + norm_one_plus(feed_forward(layer["mlp"], w, pre + "mlp.", x), w[pre + "norm2"], eps)
            if layers_out is not None:
                layers_out.append(x.clone())
        self.length += len(tokens)
        logits = norm_one_plus(x, w["final.norm"], eps) @ w["head"].T
        cap = raw.get("logit_softcap")
        return soft_cap(logits, float(cap)) if cap else logits


def forward(raw, weights, tokens, dtype=torch.float64, layers_out=None):
    return Stepper(raw, weights, dtype).feed(tokens, layers_out)
