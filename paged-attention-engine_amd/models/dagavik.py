"""Dagavik: a decoder whose layers are listed one by one in config.json, each with two branches that read the
same stream, a mixer of one of three kinds and a feed-forward of routed experts.

config.json keys (every size and every constant that may differ between models is read from here):

    architecture      "Dagavik"
    vocab, width      vocabulary and residual width
    norm.eps          eps of every RMS norm of the model (inside the root)
    embedding.bigram  {buckets, mul_prev, mul_cur}: the table `bigram` of buckets + 1 rows added to the embedding
    layers[i]         type: "parallel" | "latent_attention" | "channel_delta"; mixer: that mixer's sizes;
                      mlp: {kind: "moe", expert {ff}, router {experts, top, scale, groups {count, keep}}} or null
      parallel          left {heads, kv_heads, dim, vdim, scale, mask {size}, rot {base, dims}},
                        right {heads, dim, vdim, gate_cap}, left_scale, right_scale
      latent_attention  heads, dim, vdim, kv_rank, scale, kv_from (optional: the layer whose cached rows this one reads)
      channel_delta     heads, kv_heads, dim, vdim, conv (taps); the widths between its two pairs of narrow
                        products are the rows of the tensors `a1` and `g1` (or the keys decay_rank, gate_rank)

Fixed by the design, so constants of this file: x <- x + mixer(norm1(x)) + mlp(norm2(x)) with both norms of
the same x; norm weights stored around zero (the weight is 1 + w); a sequence's first token takes the bigram
table's last row.  In "parallel": the left mixer is softmax attention with biases on q, k and v, a rotation
of the pairs (i, i + dims/2) of each head's first `dims` features and a sliding window that includes the
token itself; the right one a matrix memory with exponential gates (q times dim^-1/2, gates capped by
c tanh(z / c), 1e-6 added to the read-out's denominator, a norm per head without eps of its own, a weight per head
and feature, a sigmoid output gate).  In "latent_attention": no positions, the latent RMS-normed with a
plain weight, causal, a sink per head.  In "channel_delta": the gated delta rule with a decay per head and key
channel, 1e-6 inside the unit vectors' root, a sigmoid gate.  Experts are W_down (silu(W_gate h) * W_up h).
Tensor names: `embed`, `bigram`, `final.norm`, `head`, and below `l<i>.`: `norm1`, `norm2`,
`mix.left.q|k|v` with `.b`, `mix.left.o`, `mix.right.q|k|v|g|o|norm`, `mix.right.i|f` with `.b` (parallel);
`mix.q|dkv|dkv.norm|uk|uv|sink|o` (latent attention); `mix.q|k|v` with `.conv`, `mix.b|A_log|dt_bias|norm|a1|a2|g1|g2|o`
(channel delta); `mlp.router`, `mlp.e<j>.gate|up|down`.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from ..config.model_config import (ConfigError, DeltaMixerSpec, ExpertsSpec, LatentMixerSpec, LayerSpec, MatrixMemorySpec,
                                   MixerSpec, ModelPlan, NormSpec, PairEmbeddingSpec, PositionSpec, ScheduleEntry,
                                   SideBySideSpec, positive, require)
from ..config.registry import register_architecture

ARCHITECTURE = "Dagavik"
MIXERS = ("parallel", "latent_attention", "channel_delta")
DELTA_UNIT_EPS = 1e-6
READOUT_FLOOR = 1e-6
_NEEDED = {"latent_attention": ("heads", "dim", "vdim", "kv_rank", "scale"),
           "channel_delta": ("heads", "kv_heads", "dim", "vdim", "conv"),
           "parallel": ("left", "right", "left_scale", "right_scale")}
_NEEDED_LEFT = ("heads", "kv_heads", "dim", "vdim", "scale")
_NEEDED_RIGHT = ("heads", "dim", "vdim", "gate_cap")


def _freeze(value):
    if isinstance(value, Mapping):
        return tuple((k, _freeze(v)) for k, v in value.items())
    return value


def _thaw(value):
    if isinstance(value, tuple) and all(isinstance(item, tuple) and len(item) == 2 and isinstance(item[0], str)
                                        for item in value):
        return {k: _thaw(v) for k, v in value}
    return value


def _section(cfg: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = cfg.get(key)
    if not isinstance(value, Mapping):
        raise ConfigError(f"{where} lacks the section '{key}'")
    return value


@dataclass(frozen=True)
class DagavikLayer:
    kind: str                            # one of MIXERS
    mixer: Tuple[Tuple[str, Any], ...]   # the mixer's keys as read, kept in order for `to_json_dict`
    mlp: Optional[Tuple[Tuple[str, Any], ...]]  # the feed-forward's keys as read; None: the layer has none
    decay_rank: Optional[int] = None     # channel_delta: features between W_a1 and W_a2 ...
    gate_rank: Optional[int] = None      # ... and between W_g1 and W_g2

    def get(self, key: str, default=None):
        return _thaw(dict(self.mixer).get(key, default))

    @property
    def feed_forward(self) -> Optional[dict]:
        return None if self.mlp is None else _thaw(self.mlp)


@dataclass(frozen=True)
class DagavikConfig:
    vocab: int
    width: int
    eps: float
    bigram: Optional[Tuple[int, int, int]]   # (buckets, mul_prev, mul_cur); None: no such table
    layers: Tuple[DagavikLayer, ...]
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], shapes: Optional[Mapping[str, Tuple[int, ...]]] = None) -> "DagavikConfig":
        layers = cfg.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json lacks the list 'layers'")
        read = []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            kind = layer.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"{where}: unknown mixer type {kind!r} (known: {', '.join(MIXERS)})")
            mixer = _section(layer, "mixer", where)
            for key in _NEEDED[kind]:
                if mixer.get(key) is None:
                    raise ConfigError(f"{where}.mixer lacks the key '{key}'")
            if kind == "parallel":
                for side, needed in (("left", _NEEDED_LEFT), ("right", _NEEDED_RIGHT)):
                    for key in needed:
                        if _section(mixer, side, f"{where}.mixer").get(key) is None:
                            raise ConfigError(f"{where}.mixer.{side} lacks the key '{key}'")
            ranks = [None, None]
            if kind == "channel_delta":
                for slot, (key, tensor) in enumerate((("decay_rank", "a1"), ("gate_rank", "g1"))):
                    if mixer.get(key) is not None:
                        ranks[slot] = int(mixer[key])
                    elif shapes is not None and f"l{i}.mix.{tensor}" in shapes:
                        ranks[slot] = int(shapes[f"l{i}.mix.{tensor}"][0])
                    else:
                        raise ConfigError(f"{where}.mixer: neither the key '{key}' nor the tensor l{i}.mix.{tensor} "
                                          "says how wide the narrow product is")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "moe":
                    raise ConfigError(f"{where}.mlp: unknown kind {mlp.get('kind')!r} (known: moe)")
                require(_section(mlp, "expert", f"{where}.mlp"), "ff")
                router = _section(mlp, "router", f"{where}.mlp")
                for key in ("experts", "top"):
                    require(router, key)
                require(router, "scale", float)
            read.append(DagavikLayer(kind, _freeze(mixer), None if mlp is None else _freeze(mlp), *ranks))
        bigram = (cfg.get("embedding") or {}).get("bigram")
        if bigram is not None:
            bigram = tuple(require(bigram, key) for key in ("buckets", "mul_prev", "mul_cur"))
        out = cls(vocab=require(cfg, "vocab"), width=require(cfg, "width"),
                  eps=require(_section(cfg, "norm", "config.json"), "eps", float), bigram=bigram, layers=tuple(read),
                  torch_dtype=str(cfg.get("torch_dtype", cfg.get("dtype", "bfloat16"))))
        out.validate()
        return out

    def validate(self) -> None:
        positive("vocab", self.vocab)
        positive("width", self.width)
        if not self.eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {self.eps}")
        if self.bigram is not None:
            positive("embedding.bigram.buckets", self.bigram[0])
            if min(self.bigram[1:]) < 0:
                raise ConfigError("embedding.bigram: the multipliers must not be negative")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}].mixer"
            if layer.kind == "parallel":
                left, right = layer.get("left"), layer.get("right")
                for key in ("heads", "kv_heads", "dim", "vdim"):
                    positive(f"{where}.left.{key}", int(left[key]))
                for key in ("heads", "dim", "vdim"):
                    positive(f"{where}.right.{key}", int(right[key]))
                if int(left["heads"]) % int(left["kv_heads"]):
                    raise ConfigError(f"layers[{i}]: {left['heads']} heads are not a multiple of {left['kv_heads']} kv_heads")
                if not float(right["gate_cap"]) > 0:
                    raise ConfigError(f"{where}.right.gate_cap must be positive")
                rot = left.get("rot") or {}
                dims = int(rot.get("dims", 0))
                if dims % 2 or not 0 <= dims <= int(left["dim"]):
                    raise ConfigError(f"layers[{i}]: rot.dims {dims} must be even and at most dim {left['dim']}")
                if dims and not float(rot.get("base", 0)) > 0:
                    raise ConfigError(f"layers[{i}]: rot.base must be positive")
                size = (left.get("mask") or {}).get("size")
                if size is not None:
                    positive(f"{where}.left.mask.size", int(size))
            else:
                for key in _NEEDED[layer.kind]:
                    if key != "scale":
                        positive(f"{where}.{key}", int(layer.get(key)))
            if layer.kind == "channel_delta":
                if int(layer.get("heads")) % int(layer.get("kv_heads")):
                    raise ConfigError(f"layers[{i}]: {layer.get('heads')} heads are not a multiple of "
                                      f"{layer.get('kv_heads')} kv_heads")
                positive(f"{where}.decay_rank", layer.decay_rank)
                positive(f"{where}.gate_rank", layer.gate_rank)
            if layer.kind == "latent_attention" and layer.get("kv_from") is not None:
                source = int(layer.get("kv_from"))
                if not 0 <= source < i:
                    raise ConfigError(f"layers[{i}]: kv_from {source} does not name an earlier layer")
                other = self.layers[source]
                if other.kind != "latent_attention" or other.get("kv_from") is not None:
                    raise ConfigError(f"layers[{i}]: kv_from {source} is not a latent attention layer with a down "
                                      "projection of its own")
                if int(other.get("kv_rank")) != int(layer.get("kv_rank")):
                    raise ConfigError(f"layers[{i}]: its kv_rank differs from that of layer {source}, whose rows it reads")
            mlp = layer.feed_forward
            if mlp is not None:
                router = mlp["router"]
                experts, top = int(router["experts"]), int(router["top"])
                groups = router.get("groups") or {}
                count, keep = int(groups.get("count", 1)), int(groups.get("keep", 1))
                positive(f"layers[{i}].mlp.expert.ff", int(mlp["expert"]["ff"]))
                positive(f"layers[{i}].mlp.router.experts", experts)
                positive(f"layers[{i}].mlp.router.top", top)
                if count <= 0 or experts % count or not 0 < keep <= count:
                    raise ConfigError(f"layers[{i}].mlp.router: {experts} experts in {count} groups, {keep} kept")
                if top > keep * (experts // count):
                    raise ConfigError(f"layers[{i}].mlp.router: top {top} exceeds the {keep * (experts // count)} "
                                      "experts of the groups that are kept")

    def to_json_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            mixer = _thaw(layer.mixer)
            if layer.kind == "channel_delta":  # a config that stands alone names the sizes a checkpoint's shapes would give
                mixer = {**mixer, "decay_rank": layer.decay_rank, "gate_rank": layer.gate_rank}
            layers.append({"type": layer.kind, "mixer": mixer, "mlp": layer.feed_forward})
        out = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
               "torch_dtype": self.torch_dtype, "layers": layers}
        if self.bigram is not None:
            out["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), self.bigram))}
        return out

    # ------------------------------------------------------------------ specs
    def _left_spec(self, left: Mapping[str, Any]) -> MixerSpec:
        rot = left.get("rot") or {}
        position = None
        if int(rot.get("dims", 0)):
            position = PositionSpec(kind="neox_rope", rotary_dim=int(rot["dims"]), theta=float(rot["base"]))
        size = (left.get("mask") or {}).get("size")
        return MixerSpec(hidden_size=self.width, num_heads=int(left["heads"]), num_kv_heads=int(left["kv_heads"]),
                         head_dim=int(left["dim"]), value_dim=int(left["vdim"]), scale=float(left["scale"]), qkv_bias=True,
                         out_bias=False, window=int(size) if size else None, position=position, q_name="q", k_name="k",
                         v_name="v", o_name="o", weight_suffix="", bias_suffix=".b")

    def _mixer_spec(self, layer: DagavikLayer):
        if layer.kind == "parallel":
            right = layer.get("right")
            memory = MatrixMemorySpec(hidden_size=self.width, num_heads=int(right["heads"]), key_dim=int(right["dim"]),
                                      value_dim=int(right["vdim"]), gate_cap=float(right["gate_cap"]), norm_eps=self.eps,
                                      readout_floor=READOUT_FLOOR)
            return SideBySideSpec(left=self._left_spec(layer.get("left")), right=memory,
                                  left_scale=float(layer.get("left_scale")), right_scale=float(layer.get("right_scale")))
        if layer.kind == "latent_attention":
            return LatentMixerSpec(hidden_size=self.width, num_heads=int(layer.get("heads")), nope_dim=int(layer.get("dim")),
                                   rope_dim=0, value_dim=int(layer.get("vdim")), kv_rank=int(layer.get("kv_rank")),
                                   scale=float(layer.get("scale")), window=None, position=None, norm_eps=self.eps,
                                   sinks=True, own_kv=layer.get("kv_from") is None)
        return DeltaMixerSpec(hidden_size=self.width, num_heads=int(layer.get("heads")), num_kv_heads=int(layer.get("kv_heads")),
                              key_dim=int(layer.get("dim")), value_dim=int(layer.get("vdim")), conv_taps=int(layer.get("conv")),
                              norm_eps=self.eps, unit_eps=DELTA_UNIT_EPS, decay="channel", decay_rank=layer.decay_rank,
                              gate_rank=layer.gate_rank, gate_activation="sigmoid")

    def _feed_forward_spec(self, layer: DagavikLayer) -> Optional[ExpertsSpec]:
        mlp = layer.feed_forward
        if mlp is None:
            return None
        router = mlp["router"]
        groups = router.get("groups") or {}
        return ExpertsSpec(hidden_size=self.width, intermediate_size=int(mlp["expert"]["ff"]), num_experts=int(router["experts"]),
                           top=int(router["top"]), groups=int(groups.get("count", 1)), groups_kept=int(groups.get("keep", 1)),
                           route_scale=float(router["scale"]), activation="silu")

    def plan(self) -> ModelPlan:
        layers, schedule = [], []
        for i, layer in enumerate(self.layers):
            ffn = self._feed_forward_spec(layer)
            norm1 = NormSpec(size=self.width, eps=self.eps, weight_name="norm1", weight_offset=1.0)
            norm2 = NormSpec(size=self.width, eps=self.eps, weight_name="norm2", weight_offset=1.0) if ffn is not None else None
            layers.append(LayerSpec(prefix=f"l{i}.", mixer=self._mixer_spec(layer), feed_forward=ffn, mixer_norm=norm1,
                                    feed_forward_norm=norm2, mixer_prefix="mix.", feed_forward_prefix="mlp.",
                                    mixer_norm_prefix="", feed_forward_norm_prefix="", arrangement="parallel"))
            source = layer.get("kv_from") if layer.kind == "latent_attention" else None
            schedule.append(ScheduleEntry(layer=i, cache_from=None if source is None else int(source)))
        pairs = None
        if self.bigram is not None:
            pairs = PairEmbeddingSpec(name="bigram", buckets=self.bigram[0], mul_prev=self.bigram[1], mul_cur=self.bigram[2])
        return ModelPlan(
            architecture=ARCHITECTURE, hidden_size=self.width, vocab_size=self.vocab, layers=tuple(layers),
            schedule=tuple(schedule),
            final_norm=NormSpec(size=self.width, eps=self.eps, weight_name="final.norm", weight_offset=1.0),
            embedding_name="embed", head_name="head", final_norm_prefix="", pair_embedding=pairs)


register_architecture(ARCHITECTURE, DagavikConfig.from_dict, sizes_from_tensors=True)
