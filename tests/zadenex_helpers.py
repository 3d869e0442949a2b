"""Small Zadenex configurations and weights for the tests.

The configurations differ from each other in every size and option: key and value head
sizes that differ, group ratios 1, 2 and 4, one head, windows below, at and just above the
cache's page of 64 tokens (and none at all), rotated parts of 2 to 16 elements, latents
narrower and wider than the heads, key sizes of the matrix memory that are no multiple of 8,
layers without a feed-forward, every mixer first, loops over the first layers, the last ones,
all of them and none, embedding scale and residual multiplier of 1 and other values.  The
weights are drawn so that signals are of order one (N(0, 0.02) matrices would make every
softmax flat and every state tiny, and hide a wrong key or a lost state); they are rounded to
bfloat16, so that both precisions and the oracle see the same numbers.
"""
import json
from pathlib import Path

import torch


def _mlp(ff):
    return None if ff is None else {"kind": "dense", "ff": ff}


def mlstm(heads, dim, vdim, cap, ff):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap},
            "mlp": _mlp(ff)}


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base, ff):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
                      "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
                      "rot": {"base": base, "dims": rot_dim}},
            "mlp": _mlp(ff)}


def attention(heads, kv_heads, dim, vdim, scale, window, ff):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer, "mlp": _mlp(ff)}


def model(vocab, width, eps, scale, mult, loop, layers):
    return {"architecture": "Zadenex", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": scale}, "residual_mult": mult,
            "loop": None if loop is None else dict(zip(("start", "stop", "times"), loop)),
            "layers": layers}


CONFIG_A = model(211, 64, 1e-5, 2.0, 0.5, (1, 3, 3), [
    attention(6, 3, 16, 24, 0.3, 20, 96),
    latent(3, 16, 8, 24, 40, 24, 0.2, 10000.0, 80),
    mlstm(3, 24, 16, 10.0, None),
    latent(5, 8, 2, 8, 16, 48, 0.35, 500.0, None)])
CONFIG_B = model(97, 96, 1e-6, 1.0, 1.0, None, [
    mlstm(1, 40, 72, 15.0, 128),
    attention(4, 4, 8, 48, 0.5, 100, None),
    latent(1, 32, 16, 40, 24, 56, 0.15, 1e6, 64),
    attention(8, 2, 16, 16, 0.25, None, 40),
    mlstm(4, 8, 8, 4.0, 72)])
# a loop over every layer; windows of exactly a page and of one token more; one kv head
CONFIG_C = model(150, 128, 1e-6, 0.7, 0.25, (0, 3, 2), [
    attention(4, 1, 32, 32, 0.18, 64, 160),
    mlstm(2, 20, 36, 30.0, 96),
    attention(2, 2, 64, 16, 0.125, 65, None)])
# a loop over the last layers, run once; 20 heads over a latent wider than a head
CONFIG_D = model(120, 48, 1e-5, 1.5, 0.8, (1, 2, 1), [
    latent(20, 8, 4, 8, 72, 16, 0.3, 20000.0, 64),
    attention(2, 1, 24, 40, 0.2, 3, 56)])
# sizes that the matrix-core attention kernel for wide keys takes in bfloat16
CONFIG_E = model(180, 64, 1e-6, 1.2, 0.6, (1, 3, 2), [
    attention(8, 2, 16, 32, 0.25, 50, 96),
    latent(4, 16, 16, 16, 48, 32, 0.2, 10000.0, 64),
    mlstm(2, 16, 32, 12.0, 48)])
# sizes that are multiples of nothing: no vector kernel and no few-rows product applies
CONFIG_F = model(101, 50, 1e-5, 0.9, 0.7, (0, 2, 2), [
    latent(3, 10, 6, 6, 22, 14, 0.3, 3000.0, 30),
    attention(6, 3, 12, 10, 0.3, 7, None),
    mlstm(3, 12, 5, 8.0, 26)])
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C, "D": CONFIG_D, "E": CONFIG_E,
           "F": CONFIG_F}


def tensor_shapes(cfg):
    """name -> (shape, law) of every tensor of a model of `cfg`."""
    w = cfg["width"]
    out = {"embed": ((cfg["vocab"], w), "table"), "final.norm": ((w,), "norm"),
           "head": ((cfg["vocab"], w), "matrix")}
    if cfg.get("loop"):
        out["loop.in"] = ((w, 2 * w), "matrix")
        out["loop.step"] = ((cfg["loop"]["times"], w), "bias")
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}."
        for name in ("norm1", "norm1b", "norm2", "norm2b"):
            out[p + name] = ((w,), "norm")
        if layer["type"] == "mlstm":
            qk, v = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            out[p + "mix.q"] = ((qk, w), "matrix")
            out[p + "mix.k"] = ((qk, w), "matrix")
            out[p + "mix.v"] = ((v, w), "matrix")
            out[p + "mix.g"] = ((v, w), "matrix")
            out[p + "mix.i"] = ((m["heads"], w), "matrix")
            out[p + "mix.i.b"] = ((m["heads"],), "in_bias")
            out[p + "mix.f"] = ((m["heads"], w), "matrix")
            out[p + "mix.f.b"] = ((m["heads"],), "forget_bias")
            out[p + "mix.norm"] = ((v,), "norm")
            out[p + "mix.o"] = ((w, v), "matrix")
        elif layer["type"] == "latent_attention":
            h, d, r = m["heads"], m["dim"], m["rot_dim"]
            out[p + "mix.dq"] = ((m["q_rank"], w), "matrix")
            out[p + "mix.dq.norm"] = ((m["q_rank"],), "norm")
            out[p + "mix.uq"] = ((h * (d + r), m["q_rank"]), "wide")
            out[p + "mix.dkv"] = ((m["kv_rank"] + r, w), "matrix")
            out[p + "mix.dkv.norm"] = ((m["kv_rank"],), "norm")
            out[p + "mix.uk"] = ((h * d, m["kv_rank"]), "wide")
            out[p + "mix.uv"] = ((h * m["vdim"], m["kv_rank"]), "matrix")
            out[p + "mix.sink"] = ((h,), "sink")
            out[p + "mix.g"] = ((h, w), "matrix")
            out[p + "mix.o"] = ((w, h * m["vdim"]), "matrix")
        else:
            q, k, v = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            out[p + "mix.q"] = ((q, w), "wide")
            out[p + "mix.q.b"] = ((q,), "bias")
            out[p + "mix.k"] = ((k, w), "wide")
            out[p + "mix.k.b"] = ((k,), "bias")
            out[p + "mix.v"] = ((v, w), "matrix")
            out[p + "mix.v.b"] = ((v,), "bias")
            out[p + "mix.talk"] = ((m["heads"], m["heads"]), "talk")
            out[p + "mix.o"] = ((w, m["heads"] * m["vdim"]), "matrix")
            out[p + "mix.o.b"] = ((w,), "bias")
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            for name, shape in (("gate", (ff, w)), ("up", (ff, w)), ("down", (w, ff))):
                out[p + f"mlp.{name}"] = (shape, "matrix")
                out[p + f"mlp.{name}.b"] = ((shape[0],), "bias")
    return out


def sharp_weights(cfg, seed, long_memory=False):
    """Tensors of order-one signal, bfloat16.  `long_memory`: the matrix memories forget
    slowly (forget gates close to 1), so that a token far back still shows in the logits."""
    g = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, (shape, law) in tensor_shapes(cfg).items():
        if law == "matrix":
            value = torch.randn(shape, generator=g) / shape[1] ** 0.5
        elif law == "wide":       # queries and keys: scores of order one and more
            value = torch.randn(shape, generator=g) * 1.6 / shape[1] ** 0.5
        elif law == "table":
            value = torch.randn(shape, generator=g)
        elif law == "norm":
            value = 1.0 + (torch.rand(shape, generator=g) * 0.4 - 0.2)
        elif law == "bias":
            value = torch.randn(shape, generator=g) * 0.3
        elif law == "sink":
            value = torch.rand(shape, generator=g) * 3.0 - 1.0
        elif law == "talk":
            value = torch.eye(shape[0]) + torch.randn(shape, generator=g) * 0.3
        elif law == "in_bias":
            value = torch.randn(shape, generator=g)
        elif law == "forget_bias":
            value = (torch.rand(shape, generator=g) * 1.0 + 6.0 if long_memory
                     else torch.rand(shape, generator=g) * 3.0 + 0.5)
        tensors[name] = value.to(torch.bfloat16)
    return tensors


def write_folder(path, cfg, tensors):
    from safetensors.torch import save_file
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg, indent=1))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(path / "model.safetensors"))
    return path


def ids(vocab, count, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=g).tolist()
