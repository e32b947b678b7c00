"""Typed configuration of the Fekorax decoder, read from its own config.json keys.

A Fekorax model is a list of layers of two kinds, in any order.  Every layer is a "sandwich": a norm before and a norm
after its mixer, and the same around its feed-forward if it has one.  The mixer is either a matrix memory with exponential
gates (`mlstm`) or grouped-query attention (`attention`) with a norm on every query and key head, a rotation of the first
channels of a head, a mask cut into chunks, a learned sink in the softmax and a gate per head on the output; an attention
layer may read the keys and values of an earlier one (`kv_from`) instead of making its own.  The feed-forward is gated with
the tanh form of GELU.  The token table is scaled on the way in and serves unscaled as the output head.

config.json:
    architecture  "Fekorax"
    vocab, width  sizes of the token table
    embedding     {scale}
    norm          {eps}: every RMS norm of the model
    layers        [{type: "mlstm" | "attention", mixer: {...}, mlp: null | {kind: "dense", ff}}]
      mlstm mixer      {heads, dim, vdim, gate_cap}
      attention mixer  {heads, kv_heads, dim, vdim, scale, rot: {dims, base, scaling: {factor, low, high, original}},
                        mask: {size}, kv_from}      (rot, rot.scaling, mask and kv_from may be absent or null)
    max_positions optional: the longest sequence (default 131072)
Tensors: embed, final.norm, and per layer i under "l<i>.": norm1, norm1b, (norm2, norm2b,) mix.*, (mlp.gate, mlp.up, mlp.down).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .errors import ConfigError
from .llama import Llama3Scaling, rotary_frequencies
from .registry import register_architecture
from .spec import (AttentionSpec, LayerSpec, MlstmSpec, ModelSpec, PartialRotarySpec, RmsNormSpec, RotarySpec, RunEntry, ScaleSpec,
                   SwiGluSpec)


def _int(d, key, where, least=1):
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, float) and v == int(v):
        v = int(v)
    if isinstance(v, bool) or not isinstance(v, int) or v < least:
        raise ConfigError(f"config.json: {where} needs an integer '{key}' of at least {least}")
    return v


def _number(d, key, where, positive=True):
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (positive and not v > 0):
        raise ConfigError(f"config.json: {where} needs a {'positive ' if positive else ''}number '{key}'")
    return float(v)


@dataclass(frozen=True)
class FekoraxRotation:
    dims: int
    base: float
    scaling: Optional[Llama3Scaling] = None


@dataclass(frozen=True)
class FekoraxMlstm:
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class FekoraxAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[FekoraxRotation] = None
    chunk: Optional[int] = None
    kv_from: Optional[int] = None


@dataclass(frozen=True)
class FekoraxLayer:
    mixer: object                        # FekoraxMlstm or FekoraxAttention
    ff: Optional[int] = None             # the feed-forward's inner size, or None for a layer without one


@dataclass(frozen=True)
class FekoraxConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[FekoraxLayer, ...]
    max_positions: int = 131072
    architecture: str = "Fekorax"

    # ------------------------------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, cfg: dict) -> "FekoraxConfig":
        if not isinstance(cfg.get("layers"), list) or not cfg["layers"]:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(cfg["layers"]):
            where = f"layer {i}"
            if not isinstance(entry, dict) or not isinstance(entry.get("mixer"), dict):
                raise ConfigError(f"config.json: {where} needs a 'type' and a 'mixer'")
            m, kind = entry["mixer"], entry.get("type")
            if kind == "mlstm":
                mixer = FekoraxMlstm(_int(m, "heads", where), _int(m, "dim", where), _int(m, "vdim", where), _number(m, "gate_cap", where))
            elif kind == "attention":
                mixer = cls._attention(m, i, layers, where)
            else:
                raise ConfigError(f"config.json: {where} has the unknown type {kind!r} (mlstm or attention)")
            mlp, ff = entry.get("mlp"), None
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"config.json: {where} has a feed-forward of an unknown kind (dense, or null for none)")
                ff = _int(mlp, "ff", where + ", mlp")
            layers.append(FekoraxLayer(mixer, ff))
        max_positions = cfg.get("max_positions")
        return cls(vocab=_int(cfg, "vocab", "the model"), width=_int(cfg, "width", "the model"),
                   embedding_scale=_number(cfg.get("embedding"), "scale", "'embedding'"), norm_eps=_number(cfg.get("norm"), "eps", "'norm'"),
                   layers=tuple(layers), max_positions=131072 if max_positions is None else _int(cfg, "max_positions", "the model"))

    @staticmethod
    def _attention(m, i, earlier, where):
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
            scaling = None
            if isinstance(r, dict) and r.get("scaling") is not None:
                s, w = r["scaling"], where + ", rot.scaling"
                scaling = Llama3Scaling(_number(s, "factor", w), _number(s, "low", w), _number(s, "high", w), _int(s, "original", w))
                if scaling.high_freq_factor == scaling.low_freq_factor:
                    raise ConfigError(f"config.json: {w}: 'low' and 'high' must differ")
            rot = FekoraxRotation(dims, _number(r, "base", where + ", rot"), scaling)
        chunk = None
        if m.get("mask") is not None:
            if not isinstance(m["mask"], dict) or m["mask"].get("kind", "chunk") not in ("chunk", "chunked"):
                raise ConfigError(f"config.json: {where} has a mask of an unknown kind")
            chunk = _int(m["mask"], "size", where + ", mask")
        kv_from = m.get("kv_from")
        mixer = FekoraxAttention(heads, kv_heads, dim, _int(m, "vdim", where), _number(m, "scale", where), rot, chunk,
                                 None if kv_from is None else _int(m, "kv_from", where, least=0))
        if kv_from is not None:
            src = earlier[kv_from].mixer if kv_from < i else None
            if not isinstance(src, FekoraxAttention) or src.kv_from is not None:
                raise ConfigError(f"config.json: {where} takes its keys and values from layer {kv_from}, which is no earlier attention layer with projections of its own")
            if (src.kv_heads, src.dim, src.vdim, src.rot) != (kv_heads, dim, mixer.vdim, rot):
                raise ConfigError(f"config.json: {where} takes its keys and values from layer {kv_from}, whose head counts, sizes or rotation differ")
        return mixer

    def to_dict(self) -> dict:
        """config.json content that `from_dict` reads back to an equal configuration."""
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, FekoraxMlstm):
                mixer, kind = dict(heads=m.heads, dim=m.dim, vdim=m.vdim, gate_cap=m.gate_cap), "mlstm"
            else:
                mixer, kind = dict(heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale), "attention"
                if m.rot is not None:
                    mixer["rot"] = dict(dims=m.rot.dims, base=m.rot.base)
                    if m.rot.scaling is not None:
                        s = m.rot.scaling
                        mixer["rot"]["scaling"] = dict(factor=s.factor, low=s.low_freq_factor, high=s.high_freq_factor, original=s.original_max_position_embeddings)
                if m.chunk is not None:
                    mixer["mask"] = dict(size=m.chunk)
                if m.kv_from is not None:
                    mixer["kv_from"] = m.kv_from
            layers.append(dict(type=kind, mixer=mixer, mlp=None if layer.ff is None else dict(kind="dense", ff=layer.ff)))
        return dict(architecture=self.architecture, vocab=self.vocab, width=self.width, embedding=dict(scale=self.embedding_scale),
                    norm=dict(eps=self.norm_eps), layers=layers, max_positions=self.max_positions)

    # ------------------------------------------------------------------------------------ as parts
    def model_spec(self) -> ModelSpec:
        eps, width = self.norm_eps, self.width
        norm = lambda name: RmsNormSpec(width, eps, name)
        specs = []
        for i, layer in enumerate(self.layers):
            p, m = f"l{i}.", layer.mixer
            if isinstance(m, FekoraxMlstm):
                x = p + "mix."
                mixer = MlstmSpec(hidden_size=width, n_heads=m.heads, key_dim=m.dim, value_dim=m.vdim, gate_cap=m.gate_cap, norm_eps=eps,
                                  q_proj=x + "q", k_proj=x + "k", v_proj=x + "v", gate_proj=x + "g", o_proj=x + "o", out_norm=x + "norm",
                                  i_proj=x + "i", i_bias=x + "i.b", f_proj=x + "f", f_bias=x + "f.b")
            else:
                mixer = self._attention_spec(i, m)
            ff = None if layer.ff is None else SwiGluSpec(hidden_size=width, intermediate_size=layer.ff, gate_proj=p + "mlp.gate",
                                                          up_proj=p + "mlp.up", down_proj=p + "mlp.down", activation="gelu_tanh")
            specs.append(LayerSpec(mixer=mixer, feed_forward=ff, mixer_norm=norm(p + "norm1"), feed_forward_norm=None if ff is None else norm(p + "norm2"),
                                   block="sandwich", mixer_post_norm=norm(p + "norm1b"), feed_forward_post_norm=None if ff is None else norm(p + "norm2b")))
        return ModelSpec(architecture=self.architecture, vocab_size=self.vocab, hidden_size=width, max_positions=self.max_positions,
                         embedding="embed", final_norm=norm("final.norm"), lm_head="embed", layers=tuple(specs),
                         run_order=tuple(RunEntry(i, getattr(l.mixer, "kv_from", None)) for i, l in enumerate(self.layers)),
                         after_embedding=(ScaleSpec(self.embedding_scale),))

    def _attention_spec(self, i: int, m: FekoraxAttention) -> AttentionSpec:
        x = f"l{i}.mix."
        position = None
        if m.rot is not None:
            frequencies = None if m.rot.scaling is None else rotary_frequencies(m.rot.dims, m.rot.base, m.rot.scaling)
            position = (RotarySpec(m.dim, m.rot.base, frequencies) if m.rot.dims == m.dim
                        else PartialRotarySpec(m.dim, m.rot.dims, m.rot.base, frequencies))
        # Pages of chunks gone by can be given back where the owner of the pages and all who read them cut their masks alike.
        owner = i if m.kv_from is None else m.kv_from
        family = [l.mixer for j, l in enumerate(self.layers) if isinstance(l.mixer, FekoraxAttention) and (j == owner or l.mixer.kv_from == owner)]
        keep_chunk = m.chunk if m.chunk is not None and all(f.chunk == m.chunk for f in family) else None
        own = m.kv_from is None
        return AttentionSpec(hidden_size=self.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, q_proj=x + "q",
                             k_proj=x + "k" if own else None, v_proj=x + "v" if own else None, o_proj=x + "o", position=position,
                             value_dim=m.vdim, scale=m.scale, chunk=m.chunk, sinks=x + "sink", q_norm=x + "q.norm",
                             k_norm=x + "k.norm" if own else None, qk_norm_eps=self.norm_eps, head_gate=x + "g", keep_chunk=keep_chunk)


register_architecture(FekoraxConfig.architecture, FekoraxConfig, model_type="fekorax")
