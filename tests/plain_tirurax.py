"""A plain, slow implementation of the Tirurax decoder used only as the oracle of the tests.

Whole sequences from position 0, no cache, token-by-token recurrences, one function per
mechanism, float64 arithmetic on the CPU.  Nothing here imports the product package.  A
model is a dictionary `cfg` (the content of its config.json) and a dictionary of tensors
under their checkpoint names.

Notation: T tokens, W the model's width; matrices are stored [out, in].
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def f64(t):
    return t.to(F64)


def rms_norm(x, weight, eps):
    """y = x / sqrt(mean(x^2) + eps) * w over the last axis."""
    x = f64(x)
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * f64(weight)


def rms_scale(x, eps):
    """x / sqrt(mean(x^2) + eps), no weight."""
    x = f64(x)
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def linear(x, weight, bias=None):
    y = f64(x) @ f64(weight).T
    return y if bias is None else y + f64(bias)


def silu(x):
    return x / (1.0 + torch.exp(-x))


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def short_conv(x, taps_weight):
    """Causal convolution over time, per channel: y[t, c] = sum_j w[c, j] x[t - (J-1) + j, c]
    with x = 0 before the sequence starts; the last tap multiplies the current token."""
    x, w = f64(x), f64(taps_weight)
    T, C = x.shape
    J = w.shape[1]
    padded = torch.cat([torch.zeros(J - 1, C, dtype=F64), x], dim=0)
    y = torch.zeros(T, C, dtype=F64)
    for j in range(J):
        y += padded[j:j + T] * w[:, j]
    return y


def unit_vectors(x, eps=1e-6):
    """x / sqrt(sum(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + eps)


def delta_recurrence(q, k, v, beta, decay):
    """Gated delta rule, one head: q, k [T, d], v [T, e], beta, decay [T].
    S_t = g_t S_{t-1};  u_t = beta_t (v_t - S_t^T k_t);  S_t += k_t u_t^T;  o_t = S_t^T q_t."""
    T, d = q.shape
    e = v.shape[1]
    S = torch.zeros(d, e, dtype=F64)
    out = torch.zeros(T, e, dtype=F64)
    for t in range(T):
        S = decay[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def delta_mixer(h, p, m, eps):
    """The 'delta' mixer on a whole sequence.  `p`: its tensors by short name, `m`: its sizes."""
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(short_conv(linear(h, p["q"]), p["q.conv"])).reshape(T, G, d)
    k = silu(short_conv(linear(h, p["k"]), p["k.conv"])).reshape(T, G, d)
    v = silu(short_conv(linear(h, p["v"]), p["v.conv"])).reshape(T, H, e)
    q = unit_vectors(q) * d ** -0.5
    k = unit_vectors(k)
    beta = torch.sigmoid(linear(h, p["b"]))                               # [T, H]
    decay = torch.exp(-torch.exp(f64(p["A_log"])) * softplus(linear(h, p["a"]) + f64(p["dt_bias"])))
    gate = silu(linear(h, p["g"])).reshape(T, H, e)
    out = torch.zeros(T, H, e, dtype=F64)
    for head in range(H):
        shared = head // (H // G)
        out[:, head] = delta_recurrence(q[:, shared], k[:, shared], v[:, head], beta[:, head],
                                        decay[:, head])
    out = rms_scale(out, eps) * f64(p["norm"]) * gate
    return linear(out.reshape(T, H * e), p["o"])


def distance_slopes(heads):
    return [2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)]


def attention_mixer(h, p, m, eps):
    """The 'attention' mixer on a whole sequence starting at position 0."""
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = rms_norm(linear(h, p["q"], p["q.b"]), p["q.norm"], eps).reshape(T, H, d)
    k = rms_norm(linear(h, p["k"], p["k.b"]), p["k.norm"], eps).reshape(T, G, d)
    v = linear(h, p["v"], p["v.b"]).reshape(T, G, e)
    chunk = (m.get("mask") or {}).get("size")
    slopes = distance_slopes(H)
    out = torch.zeros(T, H, e, dtype=F64)
    for head in range(H):
        shared = head // (H // G)
        for i in range(T):
            first = 0 if chunk is None else (i // chunk) * chunk
            keys = torch.arange(first, i + 1)
            score = (k[first:i + 1, shared] @ q[i, head]) * m["scale"]
            score = score - slopes[head] * (i - keys).to(F64)
            top = max(score.max().item(), float(p["sink"][head]))
            weight = torch.exp(score - top)
            total = weight.sum() + math.exp(float(p["sink"][head]) - top)
            out[i, head] = (weight / total) @ v[first:i + 1, shared]
    return linear(out.reshape(T, H * e), p["o"])


def dense_feed_forward(h, p):
    """down(relu(up h)^2)."""
    return linear(torch.relu(linear(h, p["up"])) ** 2, p["down"])


def sub_tensors(tensors, prefix):
    return {name[len(prefix):]: t for name, t in tensors.items() if name.startswith(prefix)}


def layer(x, index, cfg, tensors):
    """x + norm1(mixer(x)), then x + norm2(ff(x)): the norms sit on the sublayers' outputs."""
    spec = cfg["layers"][index]
    eps = cfg["norm"]["eps"]
    mix = sub_tensors(tensors, f"l{index}.mix.")
    mixer = {"delta": delta_mixer, "attention": attention_mixer}[spec["type"]]
    x = x + rms_norm(mixer(x, mix, spec["mixer"], eps), tensors[f"l{index}.norm1"], eps)
    if spec.get("mlp") is not None:
        ff = dense_feed_forward(x, sub_tensors(tensors, f"l{index}.mlp."))
        x = x + rms_norm(ff, tensors[f"l{index}.norm2"], eps)
    return x


def forward(cfg, tensors, ids, keep_layers=False):
    """float64 logits [T, vocab] of a whole sequence (and the residual stream after every
    layer, when asked)."""
    x = f64(tensors["embed"])[torch.as_tensor(ids, dtype=torch.long)]
    kept = []
    for index in range(len(cfg["layers"])):
        x = layer(x, index, cfg, tensors)
        kept.append(x)
    logits = linear(rms_norm(x, tensors["final.norm"], cfg["norm"]["eps"]), tensors["head"])
    return (logits, torch.stack(kept)) if keep_layers else logits
