"""Zikezen: a decoder whose layers are listed one by one in config.json, some of them run several times over,
each with a norm before and after every sublayer, two mixers side by side and a dense or routed feed-forward.

config.json keys (every size and every constant that may differ between models is read from here):

    architecture      "Zikezen"
    vocab, width      vocabulary and residual width
    max_positions     rows of the table `pos` of learned positions
    embedding.scale   multiplier of the embedding row (the position's row is added unscaled)
    norm.eps          eps of every RMS norm of the model (inside the root)
    layers[i]         type: "parallel"; mixer: {left {...}, right {...}, left_scale, right_scale};
                      mlp: {kind: "dense", ff} | {kind: "moe", expert {ff}, router {experts, top}} | null
      left              heads, kv_heads, dim, vdim, scale, mask {size}, rot {base, dims, scaling {factor, low, high, original}}
      right             heads, dim, vdim, tau; the width between its two narrow products is the rows of the tensor
                        `a1` (or the key decay_rank)
    loop              {start, stop, times}: layers start .. stop - 1 run `times` times in a row with the same weights
    token_side.dim    columns of the table `side.embed` that each layer reads (layer i: [i dim, (i + 1) dim))
    logit_softcap     c: logits become c tanh(logits / c)

Fixed by the design, so constants of this file: x <- x + norm1b(mixer(norm1(x))), then x <- x + norm2b(mlp(norm2(x))),
then the token's input x <- x + side.norm(side.proj(gelu_tanh(side.gate x) * side.embed[token] columns)); all norms
RMS with plain weights; every pass over the looped layers has a cache and state of its own, and before every pass but
the first the embedding's output joins the stream again.  Left mixer: softmax attention with biases on q, k and v,
an RMS norm of every q and k head with one weight shared by the heads (before the rotation), a rotation of the pairs
(2i, 2i + 1) of each head's first `dims` features with frequencies stretched by wavelength, a sliding window that
includes the token itself, and a sink of score 0 without a value in every head's softmax.  Right mixer: gated linear
attention (q times dim^-1/2, a decay sigmoid(.)^(1 / tau) per key channel through two narrow products and a bias, a
norm per head with a weight shared by the heads, a SiLU gate).  Feed-forwards are W_down (silu(W_gate h) * W_up h),
dense or as experts chosen by softmax score plus a stored correction and weighted by the score alone.
Tensor names: `embed`, `pos`, `side.embed`, `final.norm`, `head`, and below `l<i>.`: `norm1`, `norm1b`, `norm2`,
`norm2b`, `mix.left.q|k|v` with `.b`, `mix.left.q.norm`, `mix.left.k.norm`, `mix.left.o`,
`mix.right.q|k|v|g|o|norm|a1|a2`, `mix.right.a2.b`, `mlp.gate|up|down` (dense), `mlp.router`, `mlp.correction`,
`mlp.e<j>.gate|up|down` (moe), `side.gate`, `side.proj`, `side.norm`.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from ..config.model_config import (ConfigError, ExpertsSpec, FeedForwardSpec, LayerSpec, LinearAttentionSpec, MixerSpec,
                                   ModelPlan, NormSpec, PositionSpec, ScheduleEntry, SideBySideSpec, TokenSideSpec,
                                   WavelengthRamp, positive, require)
from ..config.registry import register_architecture

ARCHITECTURE = "Zikezen"
SINK_SCORE = 0.0            # every head's softmax holds one more term, exp(0), that has no value
SIDE_ACTIVATION = "gelu_tanh"
_NEEDED_LEFT = ("heads", "kv_heads", "dim", "vdim", "scale")
_NEEDED_RIGHT = ("heads", "dim", "vdim", "tau")


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
class ZikezenLayer:
    mixer: Tuple[Tuple[str, Any], ...]            # the mixer's keys as read, kept in order for `to_json_dict`
    mlp: Optional[Tuple[Tuple[str, Any], ...]]    # the feed-forward's keys as read; None: the layer has none
    decay_rank: int                               # features between the right mixer's two narrow products

    def get(self, key: str, default=None):
        return _thaw(dict(self.mixer).get(key, default))

    @property
    def feed_forward(self) -> Optional[dict]:
        return None if self.mlp is None else _thaw(self.mlp)


@dataclass(frozen=True)
class ZikezenConfig:
    vocab: int
    width: int
    max_positions: int
    eps: float
    embedding_scale: float
    layers: Tuple[ZikezenLayer, ...]
    loop: Optional[Tuple[int, int, int]]   # (start, stop, times); None: every layer runs once
    side_dim: Optional[int]                # columns of the second token table a layer reads; None: no such table
    logit_softcap: Optional[float]
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], shapes: Optional[Mapping[str, Tuple[int, ...]]] = None) -> "ZikezenConfig":
        layers = cfg.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json lacks the list 'layers'")
        read = []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            if layer.get("type") != "parallel":
                raise ConfigError(f"{where}: unknown layer type {layer.get('type')!r} (known: parallel)")
            mixer = _section(layer, "mixer", where)
            for key in ("left_scale", "right_scale"):
                require(mixer, key, float)
            for side, needed in (("left", _NEEDED_LEFT), ("right", _NEEDED_RIGHT)):
                for key in needed:
                    if _section(mixer, side, f"{where}.mixer").get(key) is None:
                        raise ConfigError(f"{where}.mixer.{side} lacks the key '{key}'")
            right = mixer["right"]
            if right.get("decay_rank") is not None:
                rank = int(right["decay_rank"])
            elif shapes is not None and f"l{i}.mix.right.a1" in shapes:
                rank = int(shapes[f"l{i}.mix.right.a1"][0])
            else:
                raise ConfigError(f"{where}.mixer.right: neither the key 'decay_rank' nor the tensor l{i}.mix.right.a1 "
                                  "says how wide the narrow product is")
            mlp = layer.get("mlp")
            if mlp is not None:
                kind = mlp.get("kind")
                if kind == "dense":
                    require(mlp, "ff")
                elif kind == "moe":
                    require(_section(mlp, "expert", f"{where}.mlp"), "ff")
                    router = _section(mlp, "router", f"{where}.mlp")
                    for key in ("experts", "top"):
                        require(router, key)
                else:
                    raise ConfigError(f"{where}.mlp: unknown kind {kind!r} (known: dense, moe)")
            # the rank is kept beside the mixer's keys, so that a config reads the same with the key and without it
            kept = {**mixer, "right": {k: v for k, v in right.items() if k != "decay_rank"}}
            read.append(ZikezenLayer(_freeze(kept), None if mlp is None else _freeze(mlp), rank))
        loop = cfg.get("loop")
        if loop is not None:
            loop = tuple(require(loop, key) for key in ("start", "stop", "times"))
        side = cfg.get("token_side")
        cap = cfg.get("logit_softcap")
        out = cls(vocab=require(cfg, "vocab"), width=require(cfg, "width"), max_positions=require(cfg, "max_positions"),
                  eps=require(_section(cfg, "norm", "config.json"), "eps", float),
                  embedding_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)), layers=tuple(read), loop=loop,
                  side_dim=None if not side else require(side, "dim"), logit_softcap=None if not cap else float(cap),
                  torch_dtype=str(cfg.get("torch_dtype", cfg.get("dtype", "bfloat16"))))
        out.validate()
        return out

    def validate(self) -> None:
        positive("vocab", self.vocab)
        positive("width", self.width)
        positive("max_positions", self.max_positions)
        if not self.eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {self.eps}")
        if self.side_dim is not None:
            positive("token_side.dim", self.side_dim)
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ConfigError(f"logit_softcap must be positive, got {self.logit_softcap}")
        if self.loop is not None:
            start, stop, times = self.loop
            if not 0 <= start < stop <= len(self.layers) or times < 1:
                raise ConfigError(f"loop: layers {start} .. {stop - 1} of {len(self.layers)}, {times} times")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}].mixer"
            left, right = layer.get("left"), layer.get("right")
            for key in ("heads", "kv_heads", "dim", "vdim"):
                positive(f"{where}.left.{key}", int(left[key]))
            for key in ("heads", "dim", "vdim"):
                positive(f"{where}.right.{key}", int(right[key]))
            positive(f"{where}.right.decay_rank", layer.decay_rank)
            if int(left["heads"]) % int(left["kv_heads"]):
                raise ConfigError(f"layers[{i}]: {left['heads']} heads are not a multiple of {left['kv_heads']} kv_heads")
            if not float(right["tau"]) > 0:
                raise ConfigError(f"{where}.right.tau must be positive")
            rot = left.get("rot") or {}
            dims = int(rot.get("dims", 0))
            if dims % 2 or not 0 <= dims <= int(left["dim"]):
                raise ConfigError(f"layers[{i}]: rot.dims {dims} must be even and at most dim {left['dim']}")
            if dims and not float(rot.get("base", 0)) > 0:
                raise ConfigError(f"layers[{i}]: rot.base must be positive")
            scaling = rot.get("scaling")
            if dims and scaling:
                for key in ("factor", "low", "high", "original"):
                    if not float(scaling.get(key) or 0) > 0:
                        raise ConfigError(f"layers[{i}]: rot.scaling.{key} must be positive")
            size = (left.get("mask") or {}).get("size")
            if size is not None:
                positive(f"{where}.left.mask.size", int(size))
            mlp = layer.feed_forward
            if mlp is not None and mlp["kind"] == "dense":
                positive(f"layers[{i}].mlp.ff", int(mlp["ff"]))
            elif mlp is not None:
                experts, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
                positive(f"layers[{i}].mlp.expert.ff", int(mlp["expert"]["ff"]))
                if not 0 < top <= experts:
                    raise ConfigError(f"layers[{i}].mlp.router: top {top} of {experts} experts")

    def to_json_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            mixer = _thaw(layer.mixer)
            # a config that stands alone names the size a checkpoint's shapes would give
            mixer = {**mixer, "right": {**mixer["right"], "decay_rank": layer.decay_rank}}
            layers.append({"type": "parallel", "mixer": mixer, "mlp": layer.feed_forward})
        out = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "max_positions": self.max_positions,
               "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.eps}, "torch_dtype": self.torch_dtype,
               "layers": layers}
        if self.loop is not None:
            out["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        if self.side_dim is not None:
            out["token_side"] = {"dim": self.side_dim}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        return out

    # ------------------------------------------------------------------ specs
    def _left_spec(self, left: Mapping[str, Any]) -> MixerSpec:
        rot = left.get("rot") or {}
        position = None
        if int(rot.get("dims", 0)):
            scaling = rot.get("scaling")
            ramp = None
            if scaling:
                ramp = WavelengthRamp(factor=float(scaling["factor"]), original=float(scaling["original"]),
                                      low=float(scaling["low"]), high=float(scaling["high"]))
            position = PositionSpec(kind="interleaved_rope", rotary_dim=int(rot["dims"]), theta=float(rot["base"]), ramp=ramp)
        size = (left.get("mask") or {}).get("size")
        return MixerSpec(hidden_size=self.width, num_heads=int(left["heads"]), num_kv_heads=int(left["kv_heads"]),
                         head_dim=int(left["dim"]), value_dim=int(left["vdim"]), scale=float(left["scale"]), qkv_bias=True,
                         out_bias=False, window=int(size) if size else None, position=position, q_name="q", k_name="k",
                         v_name="v", o_name="o", weight_suffix="", bias_suffix=".b", fixed_sink=SINK_SCORE,
                         qk_norm="per_head", qk_norm_eps=self.eps, q_norm_name="q.norm", k_norm_name="k.norm")

    def _mixer_spec(self, layer: ZikezenLayer) -> SideBySideSpec:
        right = layer.get("right")
        linear = LinearAttentionSpec(hidden_size=self.width, num_heads=int(right["heads"]), key_dim=int(right["dim"]),
                                     value_dim=int(right["vdim"]), decay_rank=layer.decay_rank,
                                     decay_temperature=float(right["tau"]), norm_eps=self.eps, gate_activation="silu")
        return SideBySideSpec(left=self._left_spec(layer.get("left")), right=linear,
                              left_scale=float(layer.get("left_scale")), right_scale=float(layer.get("right_scale")))

    def _feed_forward_spec(self, layer: ZikezenLayer):
        mlp = layer.feed_forward
        if mlp is None:
            return None
        if mlp["kind"] == "dense":
            return FeedForwardSpec(hidden_size=self.width, intermediate_size=int(mlp["ff"]), activation="silu",
                                   gate_name="gate", up_name="up", down_name="down", weight_suffix="")
        router = mlp["router"]
        return ExpertsSpec(hidden_size=self.width, intermediate_size=int(mlp["expert"]["ff"]),
                           num_experts=int(router["experts"]), top=int(router["top"]), groups=1, groups_kept=1,
                           route_scale=1.0, activation="silu", choice_bias_name="correction")

    def layer_runs(self):
        """[(layer, does the embedding's output join the stream before it?)] in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        start, stop, times = self.loop
        runs = [(i, False) for i in range(start)]
        for turn in range(times):
            runs += [(i, turn > 0 and i == start) for i in range(start, stop)]
        return runs + [(i, False) for i in range(stop, n)]

    def plan(self) -> ModelPlan:
        layers, optional = [], []
        norm = lambda name: NormSpec(size=self.width, eps=self.eps, weight_name=name)
        for i, layer in enumerate(self.layers):
            ffn = self._feed_forward_spec(layer)
            side = None
            if self.side_dim is not None:
                side = TokenSideSpec(table_name="side.embed", table_width=self.side_dim * len(self.layers),
                                     first_column=i * self.side_dim, dim=self.side_dim, vocab_size=self.vocab, eps=self.eps,
                                     activation=SIDE_ACTIVATION)
            layers.append(LayerSpec(prefix=f"l{i}.", mixer=self._mixer_spec(layer), feed_forward=ffn, mixer_norm=norm("norm1"),
                                    feed_forward_norm=norm("norm2") if ffn is not None else None,
                                    mixer_out_norm=norm("norm1b"),
                                    feed_forward_out_norm=norm("norm2b") if ffn is not None else None, mixer_prefix="mix.",
                                    feed_forward_prefix="mlp.", mixer_norm_prefix="", feed_forward_norm_prefix="",
                                    arrangement="sandwich", token_side=side))
            if ffn is None:  # a checkpoint may still hold the norms of the feed-forward the layer does not have
                optional += [f"l{i}.norm2", f"l{i}.norm2b"]
        schedule = tuple(ScheduleEntry(layer=i, add_embedding=joins) for i, joins in self.layer_runs())
        return ModelPlan(
            architecture=ARCHITECTURE, hidden_size=self.width, vocab_size=self.vocab, layers=tuple(layers),
            schedule=schedule, final_norm=norm("final.norm"), embedding_name="embed", head_name="head",
            final_norm_prefix="", max_positions=self.max_positions, optional_names=tuple(optional),
            embedding_scale=self.embedding_scale, logit_softcap=self.logit_softcap, position_table_name="pos")


register_architecture(ARCHITECTURE, ZikezenConfig.from_dict, sizes_from_tensors=True)
