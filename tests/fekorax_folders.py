"""Small Fekorax model folders for the tests, written without the engine's code (config.json and a safetensors file made by
`model_folders.write_safetensors_by_hand`), so that the engine's loader reads files it did not write.

Matrices are 0.2 * N(0, 1), which makes scores and logits of order one; norm weights 1 + 0.1 * N(0, 1); the gates' biases and the
sinks are of order one so that leaving one out shows.  The configurations differ from one another in every size and option:
value heads smaller and larger than key heads, one and several key/value heads, rotations of a part of the head and of all of
it, with and without stretched frequencies, chunks shorter than a page and no multiple of one, layers with and without a
feed-forward, readers of other layers' keys with the same and with another chunk, memories whose value heads are no multiple of
the kernel's tiles, key heads that are no multiple of 4, and one configuration whose sizes are multiples of nothing."""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch

from model_folders import write_safetensors_by_hand


def _attention(heads, kv_heads, dim, vdim, scale, rot=None, chunk=None, kv_from=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if rot is not None:
        m["rot"] = rot
    if chunk is not None:
        m["mask"] = dict(size=chunk)
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _layer(kind, mixer, ff=None):
    return dict(type=kind, mixer=mixer, mlp=None if ff is None else dict(kind="dense", ff=ff))


_ROT_A = dict(dims=8, base=100.0, scaling=dict(factor=4.0, low=1.0, high=2.0, original=16))
FEKORAX_A = dict(architecture="Fekorax", vocab=320, width=64, embedding=dict(scale=3.0), norm=dict(eps=1e-5), layers=[
    _layer("attention", _attention(4, 2, 32, 16, 0.2, _ROT_A, chunk=24), ff=96),
    _layer("mlstm", dict(heads=2, dim=24, vdim=40, gate_cap=10.0), ff=80),
    _layer("attention", _attention(4, 2, 32, 16, 0.15, _ROT_A, chunk=24, kv_from=0)),
    _layer("mlstm", dict(heads=4, dim=16, vdim=16, gate_cap=6.0)),
])
FEKORAX_B = dict(architecture="Fekorax", vocab=257, width=96, embedding=dict(scale=0.7), norm=dict(eps=1e-6), layers=[
    _layer("mlstm", dict(heads=3, dim=20, vdim=72, gate_cap=14.0)),
    _layer("attention", _attention(3, 3, 16, 48, 0.3, dict(dims=16, base=50.0), chunk=7), ff=64),
    _layer("attention", _attention(6, 3, 16, 48, 0.25, dict(dims=16, base=50.0), chunk=13, kv_from=1), ff=48),
    _layer("attention", _attention(2, 1, 24, 24, 0.4)),
    _layer("mlstm", dict(heads=1, dim=36, vdim=128, gate_cap=8.0), ff=72),
])
# Heads of 64 channels, keys and values alike, a chunk that is a multiple of the page: sizes the matrix-core attention kernels take.
FEKORAX_C = dict(architecture="Fekorax", vocab=512, width=128, embedding=dict(scale=5.0), norm=dict(eps=1e-5), layers=[
    _layer("attention", _attention(4, 2, 64, 64, 0.125, dict(dims=32, base=10000.0), chunk=64), ff=256),
    _layer("mlstm", dict(heads=2, dim=64, vdim=64, gate_cap=12.0)),
    _layer("attention", _attention(4, 2, 64, 64, 0.11, dict(dims=32, base=10000.0), chunk=64, kv_from=0)),
    _layer("attention", _attention(2, 2, 64, 64, 0.125, dict(dims=64, base=500.0), chunk=80), ff=128),
])
# Sizes that are multiples of nothing: rows of 50 numbers, heads of 6 and 3 channels, five heads, a chunk of 5 positions.
FEKORAX_D = dict(architecture="Fekorax", vocab=211, width=50, embedding=dict(scale=1.0), norm=dict(eps=1e-4), layers=[
    _layer("mlstm", dict(heads=5, dim=3, vdim=5, gate_cap=4.0), ff=30),
    _layer("attention", _attention(5, 5, 6, 10, 0.5, dict(dims=2, base=7.0, scaling=dict(factor=2.0, low=1.0, high=3.0, original=8)), chunk=5)),
    _layer("attention", _attention(5, 1, 10, 6, 0.3, dict(dims=6, base=9.0)), ff=22),
])
CONFIGS = {"A": FEKORAX_A, "B": FEKORAX_B, "C": FEKORAX_C, "D": FEKORAX_D}
PAGE_SIZE = {"A": 4, "B": 8, "C": 16, "D": 16}


def tensor_layout(cfg):
    d, out = cfg["width"], [("embed", (cfg["vocab"], cfg["width"])), ("final.norm", (cfg["width"],))]
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out += [(p + "norm1", (d,)), (p + "norm1b", (d,))]
        x = p + "mix."
        if layer["type"] == "mlstm":
            qk, vv, h = m["heads"] * m["dim"], m["heads"] * m["vdim"], m["heads"]
            out += [(x + "q", (qk, d)), (x + "k", (qk, d)), (x + "v", (vv, d)), (x + "g", (vv, d)), (x + "o", (d, vv)), (x + "norm", (vv,)),
                    (x + "i", (h, d)), (x + "i.b", (h,)), (x + "f", (h, d)), (x + "f.b", (h,))]
        else:
            out += [(x + "q", (m["heads"] * m["dim"], d)), (x + "q.norm", (m["dim"],)), (x + "sink", (m["heads"],)), (x + "g", (m["heads"], d)),
                    (x + "o", (d, m["heads"] * m["vdim"]))]
            if m.get("kv_from") is None:
                out += [(x + "k", (m["kv_heads"] * m["dim"], d)), (x + "v", (m["kv_heads"] * m["vdim"], d)), (x + "k.norm", (m["dim"],))]
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            out += [(p + "norm2", (d,)), (p + "norm2b", (d,)), (p + "mlp.gate", (ff, d)), (p + "mlp.up", (ff, d)), (p + "mlp.down", (d, ff))]
    return out


def random_weights(cfg, seed, std=0.2):
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in tensor_layout(cfg):
        z = rng.standard_normal(shape)
        if "norm" in name.split(".")[-1] or name.endswith(".norm"):
            w[name] = torch.from_numpy((1.0 + 0.1 * z).astype(np.float32))
        elif name.endswith((".i.b", ".f.b", ".sink")):
            w[name] = torch.from_numpy((1.0 * z).astype(np.float32))
        else:
            w[name] = torch.from_numpy((std * z).astype(np.float32))
    return w


def write_model(folder, cfg, seed=0, dtype=torch.bfloat16, std=0.2, weights=None):
    """Writes the folder; returns the float32 weights before rounding to the storage dtype."""
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg, indent=2))
    w = weights if weights is not None else random_weights(cfg, seed, std)
    write_safetensors_by_hand(folder / "model.safetensors", {n: t.to(dtype) for n, t in w.items()}, shuffle_seed=seed + 5)
    return w
