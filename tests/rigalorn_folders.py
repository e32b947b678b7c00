"""Small Rigalorn model folders for the tests, written without the engine's code (config.json and a safetensors file made by
`model_folders.write_safetensors_by_hand`), so that the engine's loader reads files it did not write.

Matrices are 0.2 * N(0, 1), which makes scores and logits of order one; norm weights 1 + 0.1 * N(0, 1); biases, the decays'
parameters, the activation's two numbers and the blends' weights are of order one so that leaving one out shows.  The
configurations differ from one another in every size and option: value heads smaller and larger than key heads, one and several
key/value heads, rotations of a part of the head and of all of it, with and without stretched frequencies, windows shorter than a
page, no multiple of one, of one position, and none at all; layers with and without a feed-forward; blended values in two, three
and no layers, the first of the family first or late in the model; convolutions of one to five taps; memories whose value heads
are no multiple of the kernel's tiles; latents longer and shorter than the heads; one configuration whose sizes are multiples of
nothing, one of the sizes the matrix-core kernels take, and one without a single page."""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch

from model_folders import write_safetensors_by_hand


def _attention(heads, kv_heads, dim, vdim, scale, rot=None, window=None, v_mix=False):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if rot is not None:
        m["rot"] = rot
    if window is not None:
        m["mask"] = dict(size=window)
    if v_mix:
        m["v_mix"] = True
    return m


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, window=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank, scale=scale, rot=dict(dims=rot_dim, base=base))
    if window is not None:
        m["mask"] = dict(size=window)
    return m


def _delta(heads, kv_heads, dim, vdim, conv):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv)


def _layer(kind, mixer, ff=None):
    return dict(type=kind, mixer=mixer, mlp=None if ff is None else dict(kind="dense", ff=ff))


_YARN_A = dict(dims=16, base=100.0, scaling=dict(factor=4.0, original=32, fast=4.0, slow=1.0))
RIGALORN_A = dict(architecture="Rigalorn", vocab=320, width=64, embedding=dict(scale=3.0), norm=dict(eps=1e-5), layers=[
    _layer("delta", _delta(4, 2, 16, 24, 4), ff=96),
    _layer("latent_attention", _latent(4, 16, 8, 24, 40, 32, 0.2, 1000.0, window=20), ff=80),
    _layer("attention", _attention(4, 2, 32, 16, 0.2, _YARN_A, window=12, v_mix=True), ff=72),
    _layer("delta", _delta(2, 2, 24, 18, 2)),
    _layer("attention", _attention(2, 2, 24, 16, 0.25, dict(dims=8, base=50.0), window=9, v_mix=True), ff=64),
])
RIGALORN_B = dict(architecture="Rigalorn", vocab=257, width=96, embedding=dict(scale=0.7), norm=dict(eps=1e-6), layers=[
    _layer("attention", _attention(6, 3, 16, 48, 0.3, dict(dims=16, base=50.0), window=7, v_mix=True), ff=64),
    _layer("attention", _attention(3, 3, 16, 24, 0.25, dict(dims=4, base=20.0, scaling=dict(factor=2.0, original=8, fast=2.0, slow=0.5)))),
    _layer("latent_attention", _latent(3, 20, 4, 12, 24, 56, 0.22, 30.0), ff=48),
    _layer("attention", _attention(3, 3, 8, 48, 0.4, None, window=33, v_mix=True), ff=72),
    _layer("delta", _delta(3, 1, 20, 72, 5), ff=40),
    _layer("attention", _attention(6, 3, 24, 48, 0.2, dict(dims=24, base=80.0), window=5, v_mix=True)),
])
# Heads of 64 channels, keys and values alike, windows that are multiples of the page: sizes the matrix-core attention kernels take.
RIGALORN_C = dict(architecture="Rigalorn", vocab=512, width=128, embedding=dict(scale=5.0), norm=dict(eps=1e-5), layers=[
    _layer("attention", _attention(4, 2, 64, 64, 0.125, dict(dims=32, base=10000.0), window=64), ff=256),
    _layer("delta", _delta(2, 2, 64, 64, 4), ff=128),
    _layer("latent_attention", _latent(4, 32, 16, 32, 64, 64, 0.14, 10000.0, window=48)),
    _layer("attention", _attention(2, 2, 64, 64, 0.125, dict(dims=64, base=500.0, scaling=dict(factor=8.0, original=64, fast=8.0, slow=1.0)), window=80), ff=128),
])
# Sizes that are multiples of nothing: rows of 50 numbers, heads of 3 to 10 channels, five heads, windows of 1 and 5 positions, a single tap.
RIGALORN_D = dict(architecture="Rigalorn", vocab=211, width=50, embedding=dict(scale=1.0), norm=dict(eps=1e-4), layers=[
    _layer("delta", _delta(5, 5, 3, 5, 3), ff=30),
    _layer("attention", _attention(5, 1, 10, 6, 0.5, dict(dims=2, base=7.0), window=1)),
    _layer("latent_attention", _latent(3, 6, 2, 5, 7, 9, 0.4, 9.0, window=5), ff=22),
    _layer("delta", _delta(1, 1, 7, 9, 1)),
])
# No page anywhere: memories only.
RIGALORN_E = dict(architecture="Rigalorn", vocab=128, width=48, embedding=dict(scale=2.0), norm=dict(eps=1e-5), layers=[
    _layer("delta", _delta(2, 1, 40, 12, 3), ff=64),
    _layer("delta", _delta(3, 3, 8, 32, 4)),
])
CONFIGS = {"A": RIGALORN_A, "B": RIGALORN_B, "C": RIGALORN_C, "D": RIGALORN_D, "E": RIGALORN_E}
PAGE_SIZE = {"A": 4, "B": 8, "C": 16, "D": 16, "E": 4}


def tensor_layout(cfg):
    d, out = cfg["width"], [("embed", (cfg["vocab"], cfg["width"])), ("final.norm", (cfg["width"],)), ("head", (cfg["vocab"], cfg["width"]))]
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out.append((p + "norm1", (d,)))
        x = p + "mix."
        if layer["type"] == "delta":
            qk, vv, h, n = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"], m["heads"], m["conv"]
            out += [(x + "q", (qk, d)), (x + "q.conv", (qk, n)), (x + "k", (qk, d)), (x + "k.conv", (qk, n)), (x + "v", (vv, d)), (x + "v.conv", (vv, n)),
                    (x + "b", (h, d)), (x + "A_log", (h,)), (x + "norm", (m["vdim"],)), (x + "a", (h, d)), (x + "dt_bias", (h,)), (x + "g", (vv, d)), (x + "o", (d, vv))]
        elif layer["type"] == "attention":
            a, kv, kvv = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            out += [(x + "q", (a, d)), (x + "q.b", (a,)), (x + "k", (kv, d)), (x + "k.b", (kv,)), (x + "v", (kvv, d)), (x + "v.b", (kvv,)),
                    (x + "o", (d, m["heads"] * m["vdim"]))]
            if m.get("v_mix"):
                out.append((x + "vmix", ()))
        else:
            H, r = m["heads"], m["rot_dim"]
            out += [(x + "dq", (m["q_rank"], d)), (x + "dq.norm", (m["q_rank"],)), (x + "uq", (H * (m["dim"] + r), m["q_rank"])), (x + "dkv", (m["kv_rank"] + r, d)),
                    (x + "dkv.norm", (m["kv_rank"],)), (x + "uk", (H * m["dim"], m["kv_rank"])), (x + "uv", (H * m["vdim"], m["kv_rank"])), (x + "o", (d, H * m["vdim"]))]
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            out += [(p + "mlp.up", (ff, d)), (p + "mlp.down", (d, ff)), (p + "mlp.act", (2,))]
    return out


def random_weights(cfg, seed, std=0.2):
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in tensor_layout(cfg):
        z = rng.standard_normal(shape)
        last = name.split(".")[-1]
        if last in ("norm", "norm1"):
            t = 1.0 + 0.1 * z
        elif last in ("b", "act", "dt_bias") and len(shape) == 1:          # biases of projections, the activation's numbers, the step sizes' bias
            t = 0.5 * z
        elif last == "A_log":                                             # decays between about 0.2 and 0.95 a token
            t = -1.0 + 0.8 * z
        elif last == "vmix":
            t = 0.3 + 0.2 * rng.random()
        elif last == "conv":
            t = 0.5 * z
        else:
            t = std * z
        w[name] = torch.from_numpy(np.asarray(t, dtype=np.float32))
    return w


def write_model(folder, cfg, seed=0, dtype=torch.bfloat16, std=0.2, weights=None):
    """Writes the folder; returns the float32 weights before rounding to the storage dtype."""
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg, indent=2))
    w = weights if weights is not None else random_weights(cfg, seed, std)
    write_safetensors_by_hand(folder / "model.safetensors", {n: t.to(dtype) for n, t in w.items()}, shuffle_seed=seed + 5)
    return w


def stored_weights(folder):
    """The folder's tensors as the file holds them (read with the safetensors package, not the engine's reader)."""
    from safetensors.torch import load_file
    return load_file(str(Path(folder) / "model.safetensors"))
