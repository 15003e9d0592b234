"""Danonex: a decoder whose layers are listed one by one in config.json, each with a mixer of its
own kind and sizes and an optional plain feed-forward.

config.json keys (every size and every constant that may differ between models is read from here):

    architecture      "Danonex"
    vocab, width      vocabulary and residual width
    norm.eps          eps of every RMS norm of the model
    residual_mult     m: a branch joins the stream as x <- x + m * norm(branch(x))
    logit_scale       the logits are multiplied by this; the head is the embedding matrix
    layers[i]         type: "attention" | "delta"; mixer: that mixer's sizes; mlp: {kind: "dense", ff} or null
      attention       heads, kv_heads, dim (query/key width), vdim (value width), scale, softcap,
                      rot {base, dims, scaling {factor, original, fast, slow} or null}
      delta           heads, kv_heads, dim, vdim, conv (taps of the short convolutions)

Fixed by the design, so constants of this file: the norm sits on a branch's output and the
branches read the stream itself; query and key are RMS-normed over their whole projection before
the rotation; the rotation pairs features (2i, 2i + 1); every attention head has a sink in its
softmax; the delta rule's unit vectors carry 1e-6 inside their root; the feed-forward is
W_down gelu(W_up x) with the exact (erf) gelu; no biases anywhere.  Tensor names: `embed`,
`final.norm`, and below `l<i>.`: `norm1`, `norm2`, `mix.<q|k|v|o>`, `mix.q.norm`, `mix.k.norm`,
`mix.sink` (attention), `mix.<q|k|v>.conv`, `mix.b`, `mix.a`, `mix.g`, `mix.A_log`, `mix.dt_bias`,
`mix.norm` (delta), `mlp.up`, `mlp.down`.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from ..config.model_config import (ConfigError, DeltaMixerSpec, FeedForwardSpec, FrequencyRamp, LayerSpec, MixerSpec,
                                   ModelPlan, NormSpec, PositionSpec, ScheduleEntry, positive, require)
from ..config.registry import register_architecture

ARCHITECTURE = "Danonex"
DELTA_UNIT_EPS = 1e-6


def _section(cfg: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = cfg.get(key)
    if not isinstance(value, Mapping):
        raise ConfigError(f"{where} lacks the section '{key}'")
    return value


@dataclass(frozen=True)
class DanonexLayer:
    kind: str                       # "attention" or "delta"
    mixer: Tuple[Tuple[str, Any], ...]   # the mixer's keys as read, kept in order for `to_json_dict`
    ff: Optional[int]               # width of the feed-forward, None: the layer has none

    def get(self, key: str, default=None):
        return dict(self.mixer).get(key, default)


def _freeze(value):
    if isinstance(value, Mapping):
        return tuple((k, _freeze(v)) for k, v in value.items())
    return value


def _thaw(value):
    if isinstance(value, tuple) and all(isinstance(item, tuple) and len(item) == 2 and isinstance(item[0], str)
                                        for item in value):
        return {k: _thaw(v) for k, v in value}
    return value


@dataclass(frozen=True)
class DanonexConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    logit_scale: float
    layers: Tuple[DanonexLayer, ...]
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any]) -> "DanonexConfig":
        layers = cfg.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json lacks the list 'layers'")
        read = []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            kind = layer.get("type")
            if kind not in ("attention", "delta"):
                raise ConfigError(f"{where}: unknown mixer type {kind!r} (known: attention, delta)")
            mixer = _section(layer, "mixer", where)
            for key in ("heads", "kv_heads", "dim", "vdim") + (("conv",) if kind == "delta" else ("scale",)):
                if mixer.get(key) is None:
                    raise ConfigError(f"{where}.mixer lacks the key '{key}'")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"{where}.mlp: unknown kind {mlp.get('kind')!r} (known: dense)")
                positive(f"{where}.mlp.ff", require(mlp, "ff"))
            read.append(DanonexLayer(kind, _freeze(mixer), None if mlp is None else int(mlp["ff"])))
        out = cls(vocab=require(cfg, "vocab"), width=require(cfg, "width"),
                  eps=require(_section(cfg, "norm", "config.json"), "eps", float),
                  residual_mult=require(cfg, "residual_mult", float), logit_scale=require(cfg, "logit_scale", float),
                  layers=tuple(read), torch_dtype=str(cfg.get("torch_dtype", cfg.get("dtype", "bfloat16"))))
        out.validate()
        return out

    def validate(self) -> None:
        positive("vocab", self.vocab)
        positive("width", self.width)
        if not self.eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {self.eps}")
        for i, layer in enumerate(self.layers):
            heads, kv = int(layer.get("heads")), int(layer.get("kv_heads"))
            for key in ("heads", "kv_heads", "dim", "vdim"):
                positive(f"layers[{i}].mixer.{key}", int(layer.get(key)))
            if heads % kv:
                raise ConfigError(f"layers[{i}]: {heads} heads are not a multiple of {kv} kv_heads")
            if layer.kind == "delta":
                positive(f"layers[{i}].mixer.conv", int(layer.get("conv")))
            rot = _thaw(layer.get("rot")) if layer.kind == "attention" else None
            if rot:
                dims = int(rot.get("dims", 0))
                if dims % 2 or not 0 <= dims <= int(layer.get("dim")):
                    raise ConfigError(f"layers[{i}]: rot.dims {dims} must be even and at most dim {layer.get('dim')}")
                if dims and not float(rot.get("base", 0)) > 0:
                    raise ConfigError(f"layers[{i}]: rot.base must be positive")

    def to_json_dict(self) -> dict:
        return {
            "architecture": ARCHITECTURE,
            "vocab": self.vocab,
            "width": self.width,
            "norm": {"eps": self.eps},
            "residual_mult": self.residual_mult,
            "logit_scale": self.logit_scale,
            "torch_dtype": self.torch_dtype,
            "layers": [{"type": layer.kind, "mixer": _thaw(layer.mixer),
                        "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}}
                       for layer in self.layers],
        }

    def _mixer_spec(self, layer: DanonexLayer):
        heads, kv, dim, vdim = (int(layer.get(k)) for k in ("heads", "kv_heads", "dim", "vdim"))
        if layer.kind == "delta":
            return DeltaMixerSpec(hidden_size=self.width, num_heads=heads, num_kv_heads=kv, key_dim=dim, value_dim=vdim,
                                  conv_taps=int(layer.get("conv")), norm_eps=self.eps, unit_eps=DELTA_UNIT_EPS)
        rot = _thaw(layer.get("rot"))
        position = None
        if rot and int(rot.get("dims", 0)):
            scaling = rot.get("scaling")
            ramp = None
            if scaling:
                ramp = FrequencyRamp(factor=float(scaling["factor"]), original=float(scaling["original"]),
                                     fast=float(scaling["fast"]), slow=float(scaling["slow"]))
            position = PositionSpec(kind="interleaved_rope", rotary_dim=int(rot["dims"]), theta=float(rot["base"]),
                                    ramp=ramp)
        cap = layer.get("softcap")
        return MixerSpec(hidden_size=self.width, num_heads=heads, num_kv_heads=kv, head_dim=dim, value_dim=vdim,
                         scale=float(layer.get("scale")), qkv_bias=False, out_bias=False, position=position,
                         softcap=float(cap) if cap else None, sinks=True, sink_name="sink",
                         qk_norm="projection", qk_norm_eps=self.eps, q_norm_name="q.norm", k_norm_name="k.norm",
                         q_name="q", k_name="k", v_name="v", o_name="o", weight_suffix="")

    def plan(self) -> ModelPlan:
        layers = []
        for i, layer in enumerate(self.layers):
            norm1 = NormSpec(size=self.width, eps=self.eps, weight_name="norm1")
            ffn = norm2 = None
            if layer.ff is not None:
                ffn = FeedForwardSpec(kind="dense", hidden_size=self.width, intermediate_size=layer.ff,
                                      activation="gelu", up_name="up", down_name="down", weight_suffix="")
                norm2 = NormSpec(size=self.width, eps=self.eps, weight_name="norm2")
            layers.append(LayerSpec(prefix=f"l{i}.", mixer=self._mixer_spec(layer), feed_forward=ffn, mixer_norm=norm1,
                                    feed_forward_norm=norm2, mixer_prefix="mix.", feed_forward_prefix="mlp.",
                                    mixer_norm_prefix="", feed_forward_norm_prefix="", arrangement="branchnorm",
                                    residual_scale=self.residual_mult))
        return ModelPlan(
            architecture=ARCHITECTURE, hidden_size=self.width, vocab_size=self.vocab, layers=tuple(layers),
            schedule=tuple(ScheduleEntry(layer=i) for i in range(len(layers))),
            final_norm=NormSpec(size=self.width, eps=self.eps, weight_name="final.norm"),
            embedding_name="embed", head_name=None, final_norm_prefix="", logit_scale=self.logit_scale)


register_architecture(ARCHITECTURE, DanonexConfig.from_dict)
