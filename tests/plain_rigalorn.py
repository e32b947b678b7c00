"""A plain, slow statement of the Rigalorn decoder on the CPU, one function per mechanism, for the tests to hold the engine
against.  It shares no code with the engine: every function takes tensors and numbers, works on one whole sequence (rows =
positions 0 .. T-1) in the dtype of its inputs (the tests use float64), and keeps no cache.

A Rigalorn layer is "parallel": with h = norm(x), x <- x + mixer(h) + feed_forward(h).  The mixer is one of
  attention          grouped heads, biases on q, k, v, a rotation of the first channels of a head (pairs i, i + r/2) whose
                     frequencies may be blended between stretched and plain ones (YaRN) and whose cosines and sines are then
                     scaled, a sliding window, and values blended with those of the first such layer;
  delta              the gated delta rule: a memory S per head that decays, is corrected towards the new value along the new
                     key, and is read with the query, behind short causal convolutions;
  latent_attention   queries and keys/values through low-rank latents; one rotated key part shared by all heads (pairs 2i,
                     2i + 1), a sliding window.
The feed-forward is down(act(up(h))) with a two-parameter activation that is quadratic on the right and exponential on the left.

`store`, where a function takes it, is applied to what an engine that computes in bfloat16 would keep in bfloat16 (rows that go
into a matrix product, cached keys and values); the identity by default.  It serves to measure what such rounding alone does.
"""
from __future__ import annotations

import math

import torch


def rms_norm(x, weight, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight


def softplus(z):
    return torch.where(z > 20, z, torch.log1p(torch.exp(torch.clamp(z, max=20))))


def xielu(z, p, q):
    """With a = softplus(p) and b = 1/2 + softplus(q): z/2 + a z^2 on the right of zero, z/2 + b (e^z - 1 - z) on the left."""
    right = softplus(p) * z * z + z / 2
    left = (0.5 + softplus(q)) * (torch.expm1(torch.clamp(z, max=0)) - z) + z / 2
    return torch.where(z > 0, right, left)


def same(x):
    return x


def to_bfloat16_and_back(x):
    return x.to(torch.bfloat16).to(x.dtype)


def dense_mlp(h, up, down, act, store=same):
    return store(xielu(h @ up.T, act[0], act[1])) @ down.T


def rotary_frequencies(dims, base, scaling=None):
    """(frequencies [dims/2], what cosines and sines are multiplied by).  scaling = dict(factor, original, fast, slow)."""
    f = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if scaling is None:
        return f, 1.0
    def turns_to_index(t):
        return dims * math.log(scaling["original"] / (2 * math.pi * t)) / (2 * math.log(base))
    lo = max(math.floor(turns_to_index(scaling["fast"])), 0)
    hi = min(math.ceil(turns_to_index(scaling["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / scaling["factor"] * ramp + fi * (1 - ramp))
    return out, 0.1 * math.log(scaling["factor"]) + 1.0


def _angles(T, frequencies, dtype):
    pos = torch.arange(T, dtype=torch.float64)
    a = pos[:, None] * torch.tensor(frequencies, dtype=torch.float64)[None, :]
    return torch.cos(a).to(dtype), torch.sin(a).to(dtype)


def rotate_half_split(x, frequencies, magnitude=1.0):
    """x [T, heads, channels]: the first 2*len(frequencies) channels of every head are turned, pair (i, i + r/2)."""
    half = len(frequencies)
    cos, sin = _angles(x.shape[0], frequencies, x.dtype)
    cos, sin = (cos * magnitude)[:, None, :], (sin * magnitude)[:, None, :]
    u, v, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, rest], dim=-1)


def rotate_interleaved(x, frequencies):
    """x [T, heads, channels]: the first 2*len(frequencies) channels of every head are turned, pair (2i, 2i + 1)."""
    half = len(frequencies)
    cos, sin = _angles(x.shape[0], frequencies, x.dtype)
    cos, sin = cos[:, None, :], sin[:, None, :]
    turned = x[..., :2 * half].reshape(*x.shape[:-1], half, 2)
    u, v = turned[..., 0], turned[..., 1]
    out = torch.stack([u * cos - v * sin, v * cos + u * sin], dim=-1).reshape(*x.shape[:-1], 2 * half)
    return torch.cat([out, x[..., 2 * half:]], dim=-1)


def window_mask(T, window):
    """[T, T] True where row i sees column j: j <= i and, with a window, i - j < window."""
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    seen = j <= i
    if window is not None:
        seen &= (i - j) < window
    return seen


def softmax_attention(q, k, v, scale, window):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; query head h reads key/value head h // (H/G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    k, v = k.repeat_interleave(H // G, dim=1), v.repeat_interleave(H // G, dim=1)
    scores = torch.einsum("thd,shd->hts", q, k) * scale
    scores = scores.masked_fill(~window_mask(T, window)[None], float("-inf"))
    return torch.einsum("hts,shd->thd", torch.softmax(scores, dim=-1), v)


def attention(h, w, m, v_first=None, store=same):
    """m: the layer's `mixer` entry of config.json; w: its tensors by their short names.  Returns (output, the values it used
    before blending if it is the first blending layer, else None)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T + w["q.b"]).view(T, H, d)
    k = (h @ w["k"].T + w["k.b"]).view(T, G, d)
    v = (h @ w["v"].T + w["v.b"]).view(T, G, dv)
    if m.get("rot"):
        f, mag = rotary_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
        q, k = rotate_half_split(q, f, mag), rotate_half_split(k, f, mag)
    own = None
    if m.get("v_mix"):
        if v_first is None:
            own = v
        else:
            lam = w["vmix"]
            v = (1 - lam) * v + lam * v_first
    window = m["mask"]["size"] if m.get("mask") else None
    o = softmax_attention(store(q), store(k), store(v), m["scale"], window)
    return store(o.reshape(T, H * dv)) @ w["o"].T, own


def latent_attention(h, w, m, eps, store=same):
    T = h.shape[0]
    H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = store(rms_norm(h @ w["dq"].T, w["dq.norm"], eps))
    q = (cq @ w["uq"].T).view(T, H, d + r)
    down = h @ w["dkv"].T
    c = store(rms_norm(down[:, :rank], w["dkv.norm"], eps))
    f, _ = rotary_frequencies(r, m["rot"]["base"])
    k_rot = store(rotate_interleaved(down[:, None, rank:], f))              # [T, 1, r], one for all heads
    q_rot = store(rotate_interleaved(q[..., d:], f))
    k = torch.cat([(c @ w["uk"].T).view(T, H, d), k_rot.expand(T, H, r)], dim=-1)
    v = (c @ w["uv"].T).view(T, H, dv)
    window = m["mask"]["size"] if m.get("mask") else None
    o = softmax_attention(torch.cat([store(q[..., :d]), q_rot], dim=-1), k, v, m["scale"], window)
    return store(o.reshape(T, H * dv)) @ w["o"].T


def short_conv_silu(x, taps):
    """x [T, channels], taps [channels, n]: y_t = silu(sum_j taps[:, j] x_(t - (n-1) + j)), zeros before the start."""
    n = taps.shape[1]
    padded = torch.cat([x.new_zeros(n - 1, x.shape[1]), x], dim=0)
    y = sum(padded[j:j + x.shape[0]] * taps[:, j] for j in range(n))
    return y * torch.sigmoid(y)


def delta_rule(q, k, v, beta, g):
    """One head.  q, k [T, dk], v [T, dv], beta (step sizes), g (decays) [T].  The memory starts at zero; a token lets it decay, moves
    what it holds along the token's key towards the token's value by the step size, and is read with the query."""
    S = q.new_zeros(q.shape[1], v.shape[1])
    out = []
    for t in range(q.shape[0]):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out)


def delta(h, w, m, eps, store=same):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv_silu(h @ w["q"].T, w["q.conv"]).view(T, G, dk)
    k = short_conv_silu(h @ w["k"].T, w["k.conv"]).view(T, G, dk)
    v = short_conv_silu(h @ w["v"].T, w["v.conv"]).view(T, H, dv)
    unit = lambda x: x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + 1e-6)
    q, k = unit(q) * dk ** -0.5, unit(k)
    beta = torch.sigmoid(h @ w["b"].T)
    g = torch.exp(-torch.exp(w["A_log"]) * softplus(h @ w["a"].T + w["dt_bias"]))
    heads = []
    for i in range(H):
        j = i // (H // G)
        o = delta_rule(q[:, j], k[:, j], v[:, i], beta[:, i], g[:, i])
        heads.append(o / torch.sqrt((o * o).mean(dim=-1, keepdim=True) + eps) * w["norm"])
    gate = h @ w["g"].T
    return store(torch.cat(heads, dim=-1) * (gate * torch.sigmoid(gate))) @ w["o"].T


def forward(config, tensors, tokens, dtype=torch.float64, layer_outputs=None, store=same):
    """Logits [T, vocab] of a whole sequence.  config: config.json as a dict; tensors: by name.  layer_outputs: a list that
    gets the residual stream after every layer."""
    t = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)] * config["embedding"]["scale"]
    v_first = None
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        w = {k[len(p) + 4:]: v for k, v in t.items() if k.startswith(p + "mix.")}
        h = store(rms_norm(x, t[p + "norm1"], eps))
        kind, m = layer["type"], layer["mixer"]
        if kind == "attention":
            mixed, own = attention(h, w, m, v_first, store)
            v_first = own if own is not None else v_first
        elif kind == "latent_attention":
            mixed = latent_attention(h, w, m, eps, store)
        elif kind == "delta":
            mixed = delta(h, w, m, eps, store)
        else:
            raise ValueError(f"unknown layer type {kind!r}")
        if layer.get("mlp") is not None:
            mixed = mixed + dense_mlp(h, t[p + "mlp.up"], t[p + "mlp.down"], t[p + "mlp.act"], store)
        x = x + mixed
        if layer_outputs is not None:
            layer_outputs.append(x)
    return store(rms_norm(x, t["final.norm"], eps)) @ t["head"].T


def greedy(config, tensors, prompt, n, dtype=torch.float64):
    """The n tokens that follow `prompt` when the likeliest is taken every time (the lowest index on ties)."""
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(torch.argmax(forward(config, tensors, tokens, dtype)[-1])))
    return tokens[len(prompt):]
