"""A plain, slow implementation of the Zadenex decoder used only as the oracle of the tests.

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


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def log_sigmoid(x):
    """log(1 / (1 + e^-x)) without overflow on either side."""
    return torch.where(x < 0, x - torch.log1p(torch.exp(torch.clamp(x, max=0.0))),
                       -torch.log1p(torch.exp(-torch.clamp(x, min=0.0))))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def soft_cap(x, cap):
    return cap * torch.tanh(x / cap)


# ---------------------------------------------------------------------------
def rotate_neighbours(x, positions, base, dims):
    """x [T, ..., d]: elements (2i, 2i + 1), i < dims / 2, of the last axis turn by the angle
    position * base^(-2i / dims); elements from `dims` on stay."""
    x = f64(x)
    out = x.clone()
    half = dims // 2
    freq = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    angle = f64(positions)[:, None] * freq[None, :]                   # [T, half]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    cos, sin = torch.cos(angle).reshape(shape), torch.sin(angle).reshape(shape)
    even, odd = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = even * cos - odd * sin
    out[..., 1:dims:2] = odd * cos + even * sin
    return out


def matrix_memory(q, k, v, log_in, log_forget):
    """One head of the stabilised matrix memory: q, k [T, d], v [T, e], log gates [T].
    m_t = max(f_t + m_{t-1}, i_t), m_0 = 0;
    S_t = e^(f_t + m_{t-1} - m_t) S_{t-1} + e^(i_t - m_t) k_t v_t^T, n_t alike with k_t alone;
    o_t = S_t^T q_t / (max(|n_t . q_t|, e^(-m_t)) + 1e-6)."""
    T, d = q.shape
    e = v.shape[1]
    S = torch.zeros(d, e, dtype=F64)
    n = torch.zeros(d, dtype=F64)
    m = torch.zeros((), dtype=F64)
    out = torch.zeros(T, e, dtype=F64)
    for t in range(T):
        m_new = torch.maximum(log_forget[t] + m, log_in[t])
        keep, take = torch.exp(log_forget[t] + m - m_new), torch.exp(log_in[t] - m_new)
        S = keep * S + take * torch.outer(k[t], v[t])
        n = keep * n + take * k[t]
        m = m_new
        bottom = torch.maximum(torch.abs(n @ q[t]), torch.exp(-m)) + 1e-6
        out[t] = (S.T @ q[t]) / bottom
    return out


def mlstm_mixer(h, p, m, eps):
    heads, d, e, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    T = h.shape[0]
    q = linear(h, p["q"]).reshape(T, heads, d) * d ** -0.5
    k = linear(h, p["k"]).reshape(T, heads, d)
    v = linear(h, p["v"]).reshape(T, heads, e)
    log_in = soft_cap(linear(h, p["i"], p["i.b"]), cap)                       # [T, heads]
    log_forget = log_sigmoid(soft_cap(linear(h, p["f"], p["f.b"]), cap))
    read = torch.stack([matrix_memory(q[:, a], k[:, a], v[:, a], log_in[:, a], log_forget[:, a])
                        for a in range(heads)], dim=1)                        # [T, heads, e]
    read = rms_scale(read, eps).reshape(T, heads * e) * f64(p["norm"])
    return linear(read * sigmoid(linear(h, p["g"])), p["o"])


def latent_attention_mixer(h, p, m, eps):
    heads, d, r, e, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    positions = torch.arange(T)
    q = linear(rms_norm(linear(h, p["dq"]), p["dq.norm"], eps), p["uq"]).reshape(T, heads, d + r)
    q_plain, q_turn = q[..., :d], q[..., d:]
    down = linear(h, p["dkv"])
    latent = rms_norm(down[:, :rank], p["dkv.norm"], eps)                     # [T, rank]
    k_turn = down[:, rank:]                                                    # [T, r], all heads
    k_plain = linear(latent, p["uk"]).reshape(T, heads, d)
    v = linear(latent, p["uv"]).reshape(T, heads, e)
    rot = m["rot"]
    q_turn = rotate_neighbours(q_turn, positions, rot["base"], rot["dims"])
    k_turn = rotate_neighbours(k_turn, positions, rot["base"], rot["dims"])
    scores = (torch.einsum("iad,jad->aij", q_plain, k_plain)
              + torch.einsum("iar,jr->aij", q_turn, k_turn)) * float(m["scale"])
    visible = positions[None, :] <= positions[:, None]
    scores = scores.masked_fill(~visible[None], -math.inf)
    top = torch.maximum(scores.max(dim=-1).values, f64(p["sink"])[:, None])   # [heads, T]
    weight = torch.exp(scores - top[..., None])
    bottom = weight.sum(dim=-1) + torch.exp(f64(p["sink"])[:, None] - top)
    out = torch.einsum("aij,jae->iae", weight / bottom[..., None], v)         # [T, heads, e]
    out = out * sigmoid(linear(h, p["g"]))[..., None]
    return linear(out.reshape(T, heads * e), p["o"])


def talking_attention_mixer(h, p, m):
    heads, groups, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = linear(h, p["q"], p["q.b"]).reshape(T, heads, d)
    k = linear(h, p["k"], p["k.b"]).reshape(T, groups, d)
    v = linear(h, p["v"], p["v.b"]).reshape(T, groups, e)
    share = heads // groups
    k = k.repeat_interleave(share, dim=1)
    v = v.repeat_interleave(share, dim=1)
    scores = torch.einsum("iad,jad->aij", q, k) * float(m["scale"])
    scores = torch.einsum("ab,bij->aij", f64(p["talk"]), scores)
    positions = torch.arange(T)
    distance = positions[:, None] - positions[None, :]
    visible = distance >= 0
    if m.get("mask") is not None:
        visible = visible & (distance < int(m["mask"]["size"]))
    scores = scores.masked_fill(~visible[None], -math.inf)
    top = torch.clamp(scores.max(dim=-1).values, min=0.0)                     # the 1 is e^0
    weight = torch.exp(scores - top[..., None])
    bottom = weight.sum(dim=-1) + torch.exp(-top)
    out = torch.einsum("aij,jae->iae", weight / bottom[..., None], v)
    return linear(out.reshape(T, heads * e), p["o"], p["o.b"])


def gated_feed_forward(h, p):
    inner = gelu_tanh(linear(h, p["gate"], p["gate.b"])) * linear(h, p["up"], p["up.b"])
    return linear(inner, p["down"], p["down.b"])


# ---------------------------------------------------------------------------
def sub_tensors(tensors, prefix):
    return {name[len(prefix):]: t for name, t in tensors.items() if name.startswith(prefix)}


def mixer(h, kind, p, m, eps):
    if kind == "mlstm":
        return mlstm_mixer(h, p, m, eps)
    if kind == "latent_attention":
        return latent_attention_mixer(h, p, m, eps)
    if kind == "attention":
        return talking_attention_mixer(h, p, m)
    raise ValueError(f"unknown mixer '{kind}'")


def layer(x, index, cfg, tensors):
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    spec, pre = cfg["layers"][index], f"l{index}."
    mixed = mixer(rms_norm(x, tensors[pre + "norm1"], eps), spec["type"],
                  sub_tensors(tensors, pre + "mix."), spec["mixer"], eps)
    x = x + mult * rms_norm(mixed, tensors[pre + "norm1b"], eps)
    if spec.get("mlp") is not None:
        fed = gated_feed_forward(rms_norm(x, tensors[pre + "norm2"], eps),
                                 sub_tensors(tensors, pre + "mlp."))
        x = x + mult * rms_norm(fed, tensors[pre + "norm2b"], eps)
    return x


def layer_runs(cfg):
    """(layer, pass number or None) in the order in which the layers run."""
    count = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(count)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, None) for i in range(start)]
    for t in range(times):
        runs += [(i, t) for i in range(start, stop)]
    return runs + [(i, None) for i in range(stop, count)]


def forward(cfg, tensors, ids, keep_layers=False):
    """Logits [T, vocab] of one sequence (and the stream after every layer run)."""
    ids = torch.as_tensor(ids, dtype=torch.long)
    x0 = f64(tensors["embed"])[ids] * float(cfg["embedding"]["scale"])
    x = x0
    loop = cfg.get("loop")
    kept = []
    for index, turn in layer_runs(cfg):
        if turn is not None and index == int(loop["start"]):
            x = linear(torch.cat([x, x0], dim=-1), tensors["loop.in"]) + f64(tensors["loop.step"])[turn]
        x = layer(x, index, cfg, tensors)
        kept.append(x)
    logits = linear(rms_norm(x, tensors["final.norm"], float(cfg["norm"]["eps"])), tensors["head"])
    return (logits, torch.stack(kept)) if keep_layers else logits


def generate(cfg, tensors, prompt, new_tokens):
    ids = list(prompt)
    for _ in range(new_tokens):
        ids.append(int(torch.argmax(forward(cfg, tensors, ids)[-1])))
    return ids[len(prompt):]


def read_folder(path):
    """(cfg, tensors) of a model folder; safetensors read by hand (8-byte length, JSON
    header, data)."""
    import json
    import struct
    from pathlib import Path
    import numpy as np
    path = Path(path)
    cfg = json.loads((path / "config.json").read_text())
    raw = (path / "model.safetensors").read_bytes()
    (length,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + length])
    data = raw[8 + length:]
    tensors = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        lo, hi = info["data_offsets"]
        piece = bytearray(data[lo:hi])
        if info["dtype"] == "BF16":
            t = torch.frombuffer(piece, dtype=torch.bfloat16)
        elif info["dtype"] == "F32":
            t = torch.frombuffer(piece, dtype=torch.float32)
        elif info["dtype"] == "I32":
            t = torch.frombuffer(piece, dtype=torch.int32)
        else:
            raise ValueError(f"tensor '{name}' has the unsupported type {info['dtype']}")
        tensors[name] = t.reshape(info["shape"]).clone()
    return cfg, tensors
