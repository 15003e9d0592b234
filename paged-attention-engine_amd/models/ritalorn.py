"""Ritalorn: a decoder whose layers are listed one by one in config.json, whose residual stream is kept
in several copies joined by hyper-connections, and whose mixers are two kinds of attention.

config.json keys (every size and every constant that may differ between models is read from here):

    architecture      "Ritalorn"
    vocab, width      vocabulary and residual width
    norm.eps          eps of every RMS norm of the model (inside the root)
    streams           S, the copies the stream is kept in
    logit_softcap     c: logits <- c tanh(logits / c)
    layers[i]         type: "attention" | "latent_attention"; mixer: that mixer's sizes; mlp: {kind: "dense", ff} or null
      attention         heads, kv_heads, dim (query/key width), vdim (value width), scale, conv (taps of the
                        short convolutions), mask {size} (chunk length), kv_from (optional: the layer whose
                        keys and values this layer reads instead of having its own)
      latent_attention  heads, dim (unrotated query/key width), rot_dim (rotated width), vdim, kv_rank,
                        scale, rot {base, dims}, mask {size} (sliding window)

Fixed by the design, so constants of this file: pre-norm layers, x_t <- sum_s mix[s, t] x_s + out[t] y
with y the sublayer's output times a per-feature scale (`ls1`, `ls2`) and u = sum_s in[s] x_s its input,
the model's output norm on the sum of the copies; in "attention": biases on q, k, v and o, a causal
convolution over time on q, k and v right after the projection, q and k divided by their root mean
square per head without a weight, no rotation but score -= 2^(-8 (h + 1) / H) (i - j), a mask in chunks
whose borders are multiples of the chunk length in the token's own sequence, a gate sigmoid(W_g x) on the heads before W_o; in "latent_attention": the latent
RMS-normed with a weight, the rotated parts turned in pairs (2i, 2i + 1) by p * base^(-2i / dims), a
sliding window that includes the token itself; the feed-forward W_down(gelu_tanh(W_gate x) * W_up x);
a head of its own.  A mixer without "mask" sees every earlier token.
Tensor names: `embed`, `final.norm`, `head`, and below `l<i>.`: `norm1`, `norm2`, `ls1`, `ls2`,
`hc1.in|out|mix`, `hc2.in|out|mix`, `mix.q|k|v|o` with `.b` and (q, k, v) `.conv`, `mix.g` (attention),
`mix.q`, `mix.dkv`, `mix.dkv.norm`, `mix.uk`, `mix.uv`, `mix.o` (latent attention), `mlp.gate|up|down`.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from ..config.model_config import (ConfigError, FeedForwardSpec, LatentMixerSpec, LayerSpec, MixerSpec, ModelPlan,
                                   NormSpec, PositionSpec, ScheduleEntry, positive, require)
from ..config.registry import register_architecture

ARCHITECTURE = "Ritalorn"
DISTANCE_SLOPE_BASE = 8.0
MIXERS = ("attention", "latent_attention")
_NEEDED = {"attention": ("heads", "kv_heads", "dim", "vdim", "scale", "conv"),
           "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale")}


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
class RitalornLayer:
    kind: str                            # one of MIXERS
    mixer: Tuple[Tuple[str, Any], ...]   # the mixer's keys as read, kept in order for `to_json_dict`
    ff: Optional[int]                    # width of the feed-forward, None: the layer has none

    def get(self, key: str, default=None):
        return _thaw(dict(self.mixer).get(key, default))

    @property
    def mask_size(self) -> Optional[int]:
        mask = self.get("mask")
        return int(mask["size"]) if mask and mask.get("size") else None


@dataclass(frozen=True)
class RitalornConfig:
    vocab: int
    width: int
    eps: float
    streams: int
    logit_softcap: Optional[float]
    layers: Tuple[RitalornLayer, ...]
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any]) -> "RitalornConfig":
        layers = cfg.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json lacks the list 'layers'")
        read = []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            kind = layer.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"{where}: unknown mixer type {kind!r} (known: {', '.join(MIXERS)})")
            mixer = layer.get("mixer")
            if not isinstance(mixer, Mapping):
                raise ConfigError(f"{where} lacks the section 'mixer'")
            for key in _NEEDED[kind]:
                if mixer.get(key) is None:
                    raise ConfigError(f"{where}.mixer lacks the key '{key}'")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"{where}.mlp: unknown kind {mlp.get('kind')!r} (known: dense)")
                positive(f"{where}.mlp.ff", require(mlp, "ff"))
            read.append(RitalornLayer(kind, _freeze(mixer), None if mlp is None else int(mlp["ff"])))
        norm = cfg.get("norm")
        if not isinstance(norm, Mapping):
            raise ConfigError("config.json lacks the section 'norm'")
        cap = cfg.get("logit_softcap")
        out = cls(vocab=require(cfg, "vocab"), width=require(cfg, "width"), eps=require(norm, "eps", float),
                  streams=require(cfg, "streams"), logit_softcap=float(cap) if cap else None, layers=tuple(read),
                  torch_dtype=str(cfg.get("torch_dtype", cfg.get("dtype", "bfloat16"))))
        out.validate()
        return out

    def validate(self) -> None:
        positive("vocab", self.vocab)
        positive("width", self.width)
        positive("streams", self.streams)
        if self.streams > 8:
            raise ConfigError(f"streams = {self.streams}: the stream's kernels keep up to 8 copies")
        if not self.eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {self.eps}")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}].mixer"
            for key in _NEEDED[layer.kind]:
                if key != "scale":
                    positive(f"{where}.{key}", int(layer.get(key)))
            if layer.mask_size is not None:
                positive(f"{where}.mask.size", layer.mask_size)
            if layer.kind == "attention":
                heads, kv = int(layer.get("heads")), int(layer.get("kv_heads"))
                if heads % kv:
                    raise ConfigError(f"layers[{i}]: {heads} heads are not a multiple of {kv} kv_heads")
                source = layer.get("kv_from")
                if source is not None:
                    source = int(source)
                    if not 0 <= source < i:
                        raise ConfigError(f"layers[{i}]: kv_from {source} does not name an earlier layer")
                    other = self.layers[source]
                    if other.kind != "attention" or other.get("kv_from") is not None:
                        raise ConfigError(f"layers[{i}]: kv_from {source} is not an attention layer with keys and values of its own")
                    for key in ("kv_heads", "dim", "vdim"):
                        if int(other.get(key)) != int(layer.get(key)):
                            raise ConfigError(f"layers[{i}]: its {key} differs from that of layer {source}, whose keys and values it reads")
            else:
                rot = layer.get("rot")
                dims = int(rot.get("dims", 0)) if rot else 0
                if dims % 2 or not 0 <= dims <= int(layer.get("rot_dim")):
                    raise ConfigError(f"layers[{i}]: rot.dims {dims} must be even and at most rot_dim {layer.get('rot_dim')}")
                if dims and not float(rot.get("base", 0)) > 0:
                    raise ConfigError(f"layers[{i}]: rot.base must be positive")

    def to_json_dict(self) -> dict:
        return {
            "architecture": ARCHITECTURE,
            "vocab": self.vocab,
            "width": self.width,
            "norm": {"eps": self.eps},
            "streams": self.streams,
            "logit_softcap": self.logit_softcap,
            "torch_dtype": self.torch_dtype,
            "layers": [{"type": layer.kind, "mixer": _thaw(layer.mixer),
                        "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}}
                       for layer in self.layers],
        }

    def _mixer_spec(self, layer: RitalornLayer):
        if layer.kind == "attention":
            return MixerSpec(hidden_size=self.width, num_heads=int(layer.get("heads")), num_kv_heads=int(layer.get("kv_heads")),
                             head_dim=int(layer.get("dim")), value_dim=int(layer.get("vdim")), scale=float(layer.get("scale")),
                             qkv_bias=True, out_bias=True, window=layer.mask_size,
                             mask="chunk" if layer.mask_size else "window", position=None, qk_norm="head",
                             qk_norm_eps=self.eps, conv_taps=int(layer.get("conv")), conv_suffix=".conv",
                             distance_slope_base=DISTANCE_SLOPE_BASE, gate_name="g", bias_suffix=".b",
                             own_kv=layer.get("kv_from") is None, q_name="q", k_name="k", v_name="v", o_name="o",
                             weight_suffix="")
        rot = layer.get("rot")
        position = None
        if rot and int(rot.get("dims", 0)):
            position = PositionSpec(kind="interleaved_rope", rotary_dim=int(rot["dims"]), theta=float(rot["base"]))
        return LatentMixerSpec(hidden_size=self.width, num_heads=int(layer.get("heads")), nope_dim=int(layer.get("dim")),
                               rope_dim=int(layer.get("rot_dim")), value_dim=int(layer.get("vdim")),
                               kv_rank=int(layer.get("kv_rank")), scale=float(layer.get("scale")), window=layer.mask_size,
                               mask="window", position=position, norm_eps=self.eps)

    def plan(self) -> ModelPlan:
        layers, schedule = [], []
        for i, layer in enumerate(self.layers):
            norm1 = NormSpec(size=self.width, eps=self.eps, weight_name="norm1")
            ffn = norm2 = None
            if layer.ff is not None:
                ffn = FeedForwardSpec(kind="swiglu", hidden_size=self.width, intermediate_size=layer.ff,
                                      activation="gelu_tanh", gate_name="gate", up_name="up", down_name="down",
                                      weight_suffix="")
                norm2 = NormSpec(size=self.width, eps=self.eps, weight_name="norm2")
            layers.append(LayerSpec(prefix=f"l{i}.", mixer=self._mixer_spec(layer), feed_forward=ffn, mixer_norm=norm1,
                                    feed_forward_norm=norm2, mixer_prefix="mix.", feed_forward_prefix="mlp.",
                                    mixer_norm_prefix="", feed_forward_norm_prefix="", arrangement="hyper",
                                    streams=self.streams, connection_prefixes=("hc1.", "hc2."),
                                    layer_scale_names=("ls1", "ls2")))
            source = layer.get("kv_from") if layer.kind == "attention" else None
            schedule.append(ScheduleEntry(layer=i, cache_from=None if source is None else int(source)))
        return ModelPlan(
            architecture=ARCHITECTURE, hidden_size=self.width, vocab_size=self.vocab, layers=tuple(layers),
            schedule=tuple(schedule), final_norm=NormSpec(size=self.width, eps=self.eps, weight_name="final.norm"),
            embedding_name="embed", head_name="head", final_norm_prefix="", logit_softcap=self.logit_softcap,
            streams=self.streams)


register_architecture(ARCHITECTURE, RitalornConfig.from_dict)
