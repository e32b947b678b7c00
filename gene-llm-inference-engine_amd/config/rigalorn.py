"""Typed configuration of the Rigalorn decoder, read from its own config.json keys.

A Rigalorn model is a list of layers of three kinds, in any order.  Every layer is "parallel": one norm, whose rows both the
mixer and the feed-forward (if the layer has one) read, and both results join the residual stream.  The mixer is
  attention          grouped-query attention with biases on q, k and v, a rotation of the first channels of a head (half-split
                     pairs) whose frequencies may be blended between stretched and plain ones with the cosines and sines
                     lengthened (YaRN), a sliding window, and, in layers that say `v_mix`, values blended with those of the
                     first such layer;
  delta              the gated delta rule behind short convolutions;
  latent_attention   attention through low-rank latents with one rotated key part for all heads (neighbouring pairs) and a
                     sliding window.
The feed-forward has no gate: down(xielu(up(h))), the activation's two numbers in a tensor.  The token table is scaled on the
way in; the head is a matrix of its own.

config.json:
    architecture  "Rigalorn"
    vocab, width  sizes of the token table
    embedding     {scale}
    norm          {eps}: every RMS norm of the model
    layers        [{type: "attention" | "delta" | "latent_attention", mixer: {...}, mlp: null | {kind: "dense", ff}}]
      attention mixer         {heads, kv_heads, dim, vdim, scale, rot: {dims, base, scaling: {factor, original, fast, slow}},
                               mask: {size}, v_mix}       (rot, rot.scaling, mask and v_mix may be absent, null or false)
      delta mixer             {heads, kv_heads, dim, vdim, conv}
      latent_attention mixer  {heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot: {dims, base}, mask: {size}}
    max_positions optional: the longest sequence (default 131072)
Tensors: embed, final.norm, head, and per layer i under "l<i>.": norm1, mix.*, (mlp.up, mlp.down, mlp.act).
"""
from __future__ import annotations

import math
import re
from dataclasses import dataclass
from typing import Optional, Tuple

from .errors import ConfigError
from .fekorax import _int, _number
from .registry import register_architecture
from .spec import (AttentionSpec, DenseMlpSpec, GatedDeltaSpec, InterleavedRotarySpec, LatentAttentionSpec, LayerSpec, ModelSpec, PartialRotarySpec,
                   RmsNormSpec, RotarySpec, RunEntry, ScaleSpec)


@dataclass(frozen=True)
class YarnScaling:
    """Frequencies blended between plain ones (pairs that turn fast) and ones divided by `factor` (pairs that turn slowly), by a
    ramp over the pair's index between the indices whose pairs make `fast` and `slow` turns over `original` positions."""
    factor: float
    original: int
    fast: float
    slow: float

    def magnitude(self) -> float:
        return 0.1 * math.log(self.factor) + 1.0


def yarn_frequencies(dims: int, base: float, scaling: YarnScaling):
    """The dims/2 frequencies.  Pair i turns at base^(-2i/dims); the pair that makes exactly t turns over the original context is the
    (fractional) one at index(t) = dims ln(original / (2 pi t)) / (2 ln base).  Pairs up to lo = floor(index(fast)) keep their
    frequency, pairs from hi = ceil(index(slow)) on turn `factor` times slower, and between the two the share r_i of the slow
    frequency climbs linearly from 0 to 1: f_i (1 - r_i) + (f_i / factor) r_i."""
    index = lambda turns: dims * math.log(scaling.original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(index(scaling.fast)), 0)
    hi = min(math.ceil(index(scaling.slow)), dims - 1)
    out = []
    for i in range(dims // 2):
        f = math.pow(float(base), -2.0 * i / dims)
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / scaling.factor * ramp + f * (1.0 - ramp))
    return tuple(out)


@dataclass(frozen=True)
class RigalornRotation:
    dims: int
    base: float
    scaling: Optional[YarnScaling] = None


@dataclass(frozen=True)
class RigalornAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[RigalornRotation] = None
    window: Optional[int] = None
    v_mix: bool = False


@dataclass(frozen=True)
class RigalornDelta:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass(frozen=True)
class RigalornLatentAttention:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    window: Optional[int] = None


@dataclass(frozen=True)
class RigalornLayer:
    mixer: object                        # RigalornAttention, RigalornDelta or RigalornLatentAttention
    ff: Optional[int] = None             # the feed-forward's inner size, or None for a layer without one


def _window(m, where) -> Optional[int]:
    if m.get("mask") is None:
        return None
    if not isinstance(m["mask"], dict) or m["mask"].get("kind", "window") not in ("window", "sliding", "sliding_window"):
        raise ConfigError(f"config.json: {where} has a mask of an unknown kind")
    return _int(m["mask"], "size", where + ", mask")


@dataclass(frozen=True)
class RigalornConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[RigalornLayer, ...]
    max_positions: int = 131072
    architecture: str = "Rigalorn"

    # ------------------------------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, cfg: dict) -> "RigalornConfig":
        if not isinstance(cfg.get("layers"), list) or not cfg["layers"]:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(cfg["layers"]):
            where = f"layer {i}"
            if not isinstance(entry, dict) or not isinstance(entry.get("mixer"), dict):
                raise ConfigError(f"config.json: {where} needs a 'type' and a 'mixer'")
            m, kind = entry["mixer"], entry.get("type")
            if kind == "attention":
                mixer = cls._attention(m, where)
            elif kind == "delta":
                mixer = RigalornDelta(_int(m, "heads", where), _int(m, "kv_heads", where), _int(m, "dim", where), _int(m, "vdim", where), _int(m, "conv", where))
                if mixer.heads % mixer.kv_heads:
                    raise ConfigError(f"config.json: {where}: 'heads' must be a multiple of 'kv_heads'")
            elif kind == "latent_attention":
                mixer = cls._latent(m, where)
            else:
                raise ConfigError(f"config.json: {where} has the unknown type {kind!r} (attention, delta or latent_attention)")
            mlp, ff = entry.get("mlp"), None
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"config.json: {where} has a feed-forward of an unknown kind (dense, or null for none)")
                ff = _int(mlp, "ff", where + ", mlp")
            layers.append(RigalornLayer(mixer, ff))
        blended = [l.mixer for l in layers if isinstance(l.mixer, RigalornAttention) and l.mixer.v_mix]
        if any((b.kv_heads, b.vdim) != (blended[0].kv_heads, blended[0].vdim) for b in blended):
            raise ConfigError("config.json: the layers that blend their values (v_mix) must have the same number and size of value heads")
        max_positions = cfg.get("max_positions")
        return cls(vocab=_int(cfg, "vocab", "the model"), width=_int(cfg, "width", "the model"),
                   embedding_scale=_number(cfg.get("embedding"), "scale", "'embedding'"), norm_eps=_number(cfg.get("norm"), "eps", "'norm'"),
                   layers=tuple(layers), max_positions=131072 if max_positions is None else _int(cfg, "max_positions", "the model"))

    @staticmethod
    def _attention(m, where) -> RigalornAttention:
        heads, kv_heads = _int(m, "heads", where), _int(m, "kv_heads", where)
        if heads % kv_heads:
            raise ConfigError(f"config.json: {where}: 'heads' must be a multiple of 'kv_heads'")
        dim = _int(m, "dim", where)
        rot = None
        if m.get("rot") is not None:
            r = m["rot"]
            dims = _int(r, "dims", where + ", rot", least=2)
            if dims % 2 or dims > dim:
                raise ConfigError(f"config.json: {where}: rot.dims must be even and at most 'dim'")
            base = _number(r, "base", where + ", rot")
            if base == 1.0:
                raise ConfigError(f"config.json: {where}: rot.base must differ from 1")
            scaling = None
            if r.get("scaling") is not None:
                s, w = r["scaling"], where + ", rot.scaling"
                scaling = YarnScaling(_number(s, "factor", w), _int(s, "original", w), _number(s, "fast", w), _number(s, "slow", w))
            rot = RigalornRotation(dims, base, scaling)
        return RigalornAttention(heads, kv_heads, dim, _int(m, "vdim", where), _number(m, "scale", where), rot, _window(m, where), bool(m.get("v_mix")))

    @staticmethod
    def _latent(m, where) -> RigalornLatentAttention:
        rot_dim = _int(m, "rot_dim", where, least=2)
        r = m.get("rot")
        if not isinstance(r, dict):
            raise ConfigError(f"config.json: {where} needs 'rot' with 'dims' and 'base'")
        if rot_dim % 2 or _int(r, "dims", where + ", rot", least=2) != rot_dim:
            raise ConfigError(f"config.json: {where}: rot.dims must equal 'rot_dim', an even number")
        return RigalornLatentAttention(_int(m, "heads", where), _int(m, "dim", where), rot_dim, _int(m, "vdim", where), _int(m, "q_rank", where),
                                       _int(m, "kv_rank", where), _number(m, "scale", where), _number(r, "base", where + ", rot"), _window(m, where))

    def to_dict(self) -> dict:
        """config.json content that `from_dict` reads back to an equal configuration."""
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, RigalornAttention):
                mixer, kind = dict(heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale), "attention"
                if m.rot is not None:
                    mixer["rot"] = dict(dims=m.rot.dims, base=m.rot.base)
                    if m.rot.scaling is not None:
                        s = m.rot.scaling
                        mixer["rot"]["scaling"] = dict(factor=s.factor, original=s.original, fast=s.fast, slow=s.slow)
                if m.window is not None:
                    mixer["mask"] = dict(size=m.window)
                if m.v_mix:
                    mixer["v_mix"] = True
            elif isinstance(m, RigalornDelta):
                mixer, kind = dict(heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, conv=m.conv), "delta"
            else:
                mixer, kind = dict(heads=m.heads, dim=m.dim, rot_dim=m.rot_dim, vdim=m.vdim, q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale,
                                   rot=dict(dims=m.rot_dim, base=m.rot_base)), "latent_attention"
                if m.window is not None:
                    mixer["mask"] = dict(size=m.window)
            layers.append(dict(type=kind, mixer=mixer, mlp=None if layer.ff is None else dict(kind="dense", ff=layer.ff)))
        return dict(architecture=self.architecture, vocab=self.vocab, width=self.width, embedding=dict(scale=self.embedding_scale),
                    norm=dict(eps=self.norm_eps), layers=layers, max_positions=self.max_positions)

    # ------------------------------------------------------------------------------------ as parts
    def model_spec(self) -> ModelSpec:
        eps, width = self.norm_eps, self.width
        specs, unused = [], []
        first_blender = next((i for i, l in enumerate(self.layers) if isinstance(l.mixer, RigalornAttention) and l.mixer.v_mix), None)
        for i, layer in enumerate(self.layers):
            p, m = f"l{i}.", layer.mixer
            x = p + "mix."
            if isinstance(m, RigalornAttention):
                position = None
                if m.rot is not None:
                    frequencies = None if m.rot.scaling is None else yarn_frequencies(m.rot.dims, m.rot.base, m.rot.scaling)
                    magnitude = 1.0 if m.rot.scaling is None else m.rot.scaling.magnitude()
                    position = (RotarySpec(m.dim, m.rot.base, frequencies, magnitude) if m.rot.dims == m.dim
                                else PartialRotarySpec(m.dim, m.rot.dims, m.rot.base, frequencies, magnitude))
                if m.v_mix and i == first_blender:
                    unused.append(re.escape(x + "vmix"))          # the family's first layer blends nothing: its weight is in the file and is not read
                mixer = AttentionSpec(hidden_size=width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, q_proj=x + "q", k_proj=x + "k",
                                      v_proj=x + "v", o_proj=x + "o", position=position, window=m.window, value_dim=m.vdim, scale=m.scale,
                                      q_bias=x + "q.b", k_bias=x + "k.b", v_bias=x + "v.b", value_family="v_mix" if m.v_mix else None,
                                      value_blend=x + "vmix" if m.v_mix and i != first_blender else None)
            elif isinstance(m, RigalornDelta):
                mixer = GatedDeltaSpec(hidden_size=width, n_heads=m.heads, n_kv_heads=m.kv_heads, key_dim=m.dim, value_dim=m.vdim, conv_taps=m.conv,
                                       norm_eps=eps, q_proj=x + "q", k_proj=x + "k", v_proj=x + "v", q_conv=x + "q.conv", k_conv=x + "k.conv",
                                       v_conv=x + "v.conv", a_proj=x + "a", a_log=x + "A_log", dt_bias=x + "dt_bias", b_proj=x + "b", gate_proj=x + "g",
                                       out_norm=x + "norm", o_proj=x + "o")
            else:
                mixer = LatentAttentionSpec(hidden_size=width, n_heads=m.heads, head_dim=m.dim, rotary_dim=m.rot_dim, value_dim=m.vdim, q_rank=m.q_rank,
                                            kv_rank=m.kv_rank, scale=m.scale, norm_eps=eps, dq_proj=x + "dq", dq_norm=x + "dq.norm", uq_proj=x + "uq",
                                            dkv_proj=x + "dkv", dkv_norm=x + "dkv.norm", uk_proj=x + "uk", uv_proj=x + "uv", o_proj=x + "o",
                                            position=InterleavedRotarySpec(m.rot_dim, m.rot_base), window=m.window)
            ff = None if layer.ff is None else DenseMlpSpec(hidden_size=width, intermediate_size=layer.ff, up_proj=p + "mlp.up", down_proj=p + "mlp.down",
                                                            activation="xielu", activation_params=p + "mlp.act")
            specs.append(LayerSpec(mixer=mixer, feed_forward=ff, mixer_norm=RmsNormSpec(width, eps, p + "norm1"), feed_forward_norm=None, block="parallel"))
        return ModelSpec(architecture=self.architecture, vocab_size=self.vocab, hidden_size=width, max_positions=self.max_positions,
                         embedding="embed", final_norm=RmsNormSpec(width, eps, "final.norm"), lm_head="head", layers=tuple(specs),
                         run_order=tuple(RunEntry(i) for i in range(len(self.layers))), ignorable_tensors=tuple(unused),
                         after_embedding=(ScaleSpec(self.embedding_scale),))


register_architecture(RigalornConfig.architecture, RigalornConfig, model_type="rigalorn")
