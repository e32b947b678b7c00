"""A plain, slow Fekorax decoder: whole sequences, no cache, no state carried between calls, one function for each mechanism.

It is the answer key for the Fekorax tests and shares no code with the engine: it reads a model folder with the few lines of
safetensors parsing of `plain_llama.read_model_folder` and computes everything with ordinary torch operations on the CPU, in
float64 unless told otherwise.  `store` (identity, or a rounding to bfloat16) is applied wherever the engine keeps an activation
as an input of a matrix product, so that the same code also tells how much rounding alone moves the logits.

Notation: T tokens, H heads, G key/value heads, dk / dv channels of a key / value head, p the position of a token in its sequence.
"""
from __future__ import annotations

import math

import torch

from plain_llama import read_model_folder


def unit_rms(x, eps):
    """x divided by its root mean square over the last axis, eps under the root."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z.pow(3))))


def scaled_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2.  With scaling {factor, low, high, original}: a wavelength 2 pi / f shorter than
    original/high keeps f, one longer than original/low gets f/factor, and between the two f is blended linearly in
    original/wavelength."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling is not None:
            wavelength, original = 2.0 * math.pi / f, float(scaling["original"])
            if wavelength > original / scaling["low"]:
                f = f / scaling["factor"]
            elif wavelength >= original / scaling["high"]:
                s = (original / wavelength - scaling["low"]) / (scaling["high"] - scaling["low"])
                f = (1.0 - s) * f / scaling["factor"] + s * f
        out.append(f)
    return out


def turn_first_channels(x, positions, dims, frequencies):
    """x [T, heads, d]: channel i < dims/2 and channel i + dims/2 form a pair (u, v) that becomes
    (u cos a - v sin a, v cos a + u sin a), a = p f_i; channels from `dims` on are left alone."""
    f = torch.tensor(frequencies, dtype=torch.float64)
    angle = positions.to(torch.float64)[:, None] * f[None, :]
    c, s = torch.cos(angle).to(x.dtype)[:, None, :], torch.sin(angle).to(x.dtype)[:, None, :]
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def visible(positions_q, positions_k, chunk=None):
    """[Tq, Tk] booleans: key j is seen from i if j <= i and, with chunks, both lie in the same chunk counted from position 0."""
    i, j = positions_q[:, None], positions_k[None, :]
    ok = j <= i
    if chunk is not None:
        ok = ok & (torch.div(i, chunk, rounding_mode="floor") == torch.div(j, chunk, rounding_mode="floor"))
    return ok


def sink_attention(q, k, v, mask, scale, sinks):
    """q [Tq, H, dk], k [Tk, G, dk], v [Tk, G, dv] -> [Tq, H, dv].  Query head h reads key/value head h // (H/G).  The softmax's
    denominator holds one more term per head, exp(sinks[h]), which brings no value."""
    H, G = q.shape[1], k.shape[1]
    out = torch.zeros(q.shape[0], H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        score = (q[:, h, :] @ k[:, g, :].T) * scale
        score = score.masked_fill(~mask, -math.inf)
        top = torch.maximum(score.max(dim=-1).values, sinks[h].expand(score.shape[0]))
        weight = torch.exp(score - top[:, None])
        total = weight.sum(dim=-1) + torch.exp(sinks[h] - top)
        out[:, h, :] = (weight / total[:, None]) @ v[:, g, :]
    return out


def matrix_memory(q, k, v, log_in, log_forget):
    """One sequence from its start.  q, k [T, H, dk] (q already scaled), v [T, H, dv], the gates' logarithms [T, H].
    Per head: m_t = max(lf_t + m_(t-1), li_t);  S_t = e^(lf_t + m_(t-1) - m_t) S_(t-1) + e^(li_t - m_t) k_t v_t^T, n_t likewise
    with k_t;  o_t = S_t^T q_t / (max(|n_t . q_t|, e^(-m_t)) + 1e-6).  S_0 = 0, n_0 = 0, m_0 = 0."""
    T, H, dk = q.shape
    dv = v.shape[2]
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for h in range(H):
        S, n, m = torch.zeros(dk, dv, dtype=q.dtype), torch.zeros(dk, dtype=q.dtype), torch.zeros((), dtype=q.dtype)
        for t in range(T):
            m_next = torch.maximum(log_forget[t, h] + m, log_in[t, h])
            keep, take = torch.exp(log_forget[t, h] + m - m_next), torch.exp(log_in[t, h] - m_next)
            S = keep * S + take * torch.outer(k[t, h], v[t, h])
            n = keep * n + take * k[t, h]
            m = m_next
            out[t, h] = (S.T @ q[t, h]) / (torch.maximum((n @ q[t, h]).abs(), torch.exp(-m)) + 1e-6)
    return out


def capped(x, cap):
    return cap * torch.tanh(x / cap)


class PlainFekorax:
    def __init__(self, folder, dtype=torch.float64, store=None):
        self.cfg, tensors = read_model_folder(folder)
        self.w = {name: t.to(dtype) for name, t in tensors.items()}
        self.dtype, self.eps = dtype, float(self.cfg["norm"]["eps"])
        self.store = store if store is not None else (lambda x: x)

    def norm(self, x, name):
        return unit_rms(x, self.eps) * self.w[name]

    # ---------------------------------------------------------------------------------- mixers
    def mlstm(self, h, prefix, m):
        T, H, dk, dv, cap = h.shape[0], m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
        w = lambda name: self.w[prefix + name]
        q = (h @ w("q").T).view(T, H, dk) * dk ** -0.5
        k = (h @ w("k").T).view(T, H, dk)
        v = (h @ w("v").T).view(T, H, dv)
        log_in = capped(h @ w("i").T + w("i.b"), cap)
        log_forget = torch.nn.functional.logsigmoid(capped(h @ w("f").T + w("f.b"), cap))
        o = unit_rms(matrix_memory(q, k, v, log_in, log_forget), self.eps).reshape(T, H * dv)
        return self.store(o * w("norm") * torch.sigmoid(h @ w("g").T)) @ w("o").T

    def keys_and_values(self, h, prefix, m, positions):
        T, G, dk, dv = h.shape[0], m["kv_heads"], m["dim"], m["vdim"]
        k = unit_rms((h @ self.w[prefix + "k"].T).view(T, G, dk), self.eps) * self.w[prefix + "k.norm"]
        v = (h @ self.w[prefix + "v"].T).view(T, G, dv)
        return self.store(self.turned(k, positions, m)), self.store(v)

    def turned(self, x, positions, m):
        rot = m.get("rot")
        if not rot:
            return x
        return turn_first_channels(x, positions, rot["dims"], scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling")))

    def attention(self, h, prefix, m, positions, kv):
        T, H, dk = h.shape[0], m["heads"], m["dim"]
        q = unit_rms((h @ self.w[prefix + "q"].T).view(T, H, dk), self.eps) * self.w[prefix + "q.norm"]
        q = self.store(self.turned(q, positions, m))
        k, v = kv
        mask = visible(positions, positions, (m.get("mask") or {}).get("size"))
        o = sink_attention(q, k, v, mask, float(m["scale"]), self.w[prefix + "sink"])
        o = o * torch.sigmoid(h @ self.w[prefix + "g"].T)[:, :, None]
        return self.store(o.reshape(T, -1)) @ self.w[prefix + "o"].T

    # ------------------------------------------------------------------------------- whole model
    def residual_streams(self, tokens):
        """The residual stream [T, width] after every layer, for one sequence from its start."""
        tokens = torch.as_tensor(tokens, dtype=torch.long)
        positions = torch.arange(len(tokens))
        x = self.w["embed"][tokens] * float(self.cfg["embedding"]["scale"])
        kept, streams = {}, []
        for i, layer in enumerate(self.cfg["layers"]):
            p, m = f"l{i}.", layer["mixer"]
            h = self.store(self.norm(x, p + "norm1"))
            if layer["type"] == "mlstm":
                y = self.mlstm(h, p + "mix.", m)
            else:
                source = m.get("kv_from")
                if source is None:
                    kept[i] = self.keys_and_values(h, p + "mix.", m, positions)
                y = self.attention(h, p + "mix.", m, positions, kept[i if source is None else source])
            x = x + self.norm(y, p + "norm1b")
            if layer.get("mlp") is not None:
                h = self.store(self.norm(x, p + "norm2"))
                inner = self.store(gelu_tanh(h @ self.w[p + "mlp.gate"].T) * (h @ self.w[p + "mlp.up"].T))
                x = x + self.norm(inner @ self.w[p + "mlp.down"].T, p + "norm2b")
            streams.append(x)
        return streams

    def logits(self, tokens):
        """[T, vocab]: the output norm, then the token table itself (without the embedding's scale)."""
        x = self.residual_streams(tokens)[-1]
        return self.store(self.norm(x, "final.norm")) @ self.w["embed"].T

    def greedy(self, prompt, n_new):
        tokens, out = list(prompt), []
        for _ in range(n_new):
            out.append(int(torch.argmax(self.logits(tokens)[-1])))
            tokens.append(out[-1])
        return out


def to_bfloat16_and_back(x):
    return x.to(torch.bfloat16).to(x.dtype)
