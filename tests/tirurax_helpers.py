"""Small Tirurax configurations and weights for the tests.

The configurations differ from each other in every size and option: key and value head
sizes that differ, group ratios 1, 3 and 4, chunks that are no multiple of the cache's page
of 64 tokens (and none at all), 1 to 5 convolution taps, key sizes that are no multiple of
8 and above 128, layers without a feed-forward, both layer kinds first, and (C) attention
with head sizes 64 and 128 and values as wide as keys, which in bfloat16 runs on the
matrix-core kernels.  The weights are
drawn so that signals are of order one (N(0, 0.02) matrices would make every softmax flat
and every state tiny, and hide a wrong key or a lost state); they are rounded to bfloat16,
so that both precisions and the oracle see the same numbers.
"""
import json
from pathlib import Path

import torch


def delta(heads, kv_heads, dim, vdim, conv, ff):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                                       "vdim": vdim, "conv": conv},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def attention(heads, kv_heads, dim, vdim, scale, chunk, ff):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk is not None:
        mixer["mask"] = {"size": chunk}
    return {"type": "attention", "mixer": mixer,
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


CONFIG_A = {"architecture": "Tirurax", "vocab": 211, "width": 64, "norm": {"eps": 1e-5},
            "layers": [attention(6, 2, 16, 24, 0.3, 24, 96), delta(4, 4, 16, 8, 3, None),
                       delta(4, 1, 24, 16, 2, 80), attention(2, 2, 32, 32, 0.2, None, 72)]}
CONFIG_B = {"architecture": "Tirurax", "vocab": 97, "width": 96, "norm": {"eps": 1e-6},
            "layers": [delta(2, 1, 40, 20, 5, 128), attention(3, 3, 8, 48, 0.5, 100, None),
                       delta(1, 1, 160, 12, 1, 64), attention(8, 2, 16, 16, 0.25, 7, 40)]}
# head sizes 64 and 128 with values as wide as keys: what the matrix-core attention kernels take
CONFIG_C = {"architecture": "Tirurax", "vocab": 150, "width": 128, "norm": {"eps": 1e-6},
            "layers": [attention(6, 2, 64, 64, 0.15, 48, 160), delta(2, 2, 32, 64, 4, 96),
                       attention(3, 3, 128, 128, 0.1, 200, None),
                       attention(8, 2, 64, 64, 0.125, None, 64)]}
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C}


def tensor_shapes(cfg):
    """name -> (shape, law) of every tensor of a model of `cfg`."""
    w = cfg["width"]
    out = {"embed": ((cfg["vocab"], w), "table"), "final.norm": ((w,), "norm"),
           "head": ((cfg["vocab"], w), "matrix")}
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}."
        out[p + "norm1"] = ((w,), "norm")
        if layer["type"] == "delta":
            qk, v = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
            for name, rows in (("q", qk), ("k", qk), ("v", v)):
                out[p + f"mix.{name}"] = ((rows, w), "matrix")
                out[p + f"mix.{name}.conv"] = ((rows, m["conv"]), "conv")
            out[p + "mix.b"] = ((m["heads"], w), "matrix")
            out[p + "mix.a"] = ((m["heads"], w), "matrix")
            out[p + "mix.A_log"] = ((m["heads"],), "rate")
            out[p + "mix.dt_bias"] = ((m["heads"],), "rate_bias")
            out[p + "mix.norm"] = ((m["vdim"],), "norm")
            out[p + "mix.g"] = ((v, w), "matrix")
            out[p + "mix.o"] = ((w, v), "matrix")
        else:
            q, k, v = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            for name, rows in (("q", q), ("k", k), ("v", v)):
                out[p + f"mix.{name}"] = ((rows, w), "matrix")
                out[p + f"mix.{name}.b"] = ((rows,), "bias")
            out[p + "mix.q.norm"] = ((q,), "norm")
            out[p + "mix.k.norm"] = ((k,), "norm")
            out[p + "mix.sink"] = ((m["heads"],), "sink")
            out[p + "mix.o"] = ((w, m["heads"] * m["vdim"]), "matrix")
        if layer["mlp"] is not None:
            out[p + "norm2"] = ((w,), "norm")
            out[p + "mlp.up"] = ((layer["mlp"]["ff"], w), "matrix")
            out[p + "mlp.down"] = ((w, layer["mlp"]["ff"]), "matrix")
    return out


def sharp_weights(cfg, seed, slow_decay=False):
    """Tensors of order-one signal, bfloat16.  `slow_decay`: the delta layers forget slowly
    (decay close to 1), so that a token far back still shows in the logits."""
    g = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, (shape, law) in tensor_shapes(cfg).items():
        if law == "matrix":
            value = torch.randn(shape, generator=g) / shape[1] ** 0.5
        elif law == "table":
            value = torch.randn(shape, generator=g)
        elif law == "conv":
            value = torch.randn(shape, generator=g) * 0.6
        elif law == "norm":
            value = 1.0 + (torch.rand(shape, generator=g) * 0.4 - 0.2)
        elif law == "bias":
            value = torch.randn(shape, generator=g) * 0.3
        elif law == "sink":
            value = torch.rand(shape, generator=g) * 3.0 - 1.0
        elif law == "rate":
            value = (torch.rand(shape, generator=g) * 1.0 - 7.0 if slow_decay
                     else torch.rand(shape, generator=g) * 2.5 - 2.0)
        elif law == "rate_bias":
            value = torch.rand(shape, generator=g) * 3.0 - 3.0
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
