"""Dipisun as a ``ModelSpec``.

A decoder whose sub-layers read the residual stream itself and whose norms stand on the sub-layers' OUTPUTS:
``x <- x + m * norm1(mixer(x))``, ``x <- x + m * norm2(ff(x))`` (``parts.block.OutputNormBlock``).  The embeddings get a
sinusoidal position vector.  ``config.json`` lists the layers one by one, each with its kind of mixer, the mixer's sizes
and its feed-forward (or none), so layers may differ in everything.  Two kinds of mixer, both ``parts.normed_attention``:

``attention``    queries and keys normed over the whole projection, a query temperature by position, a learned bias by
                 bucket of distance added to the scaled scores;
``attention_2``  queries and keys normed per head with one weight for all heads, no positions at all.

Layers whose mixer says ``v_mix`` blend their values with those that the first such layer made for the same token.  The
feed-forward is a mixture of experts: softmax over all router outputs, a correction added for the choice only, weights
that are the chosen scores as they are and scale the expert's output, clamped gated units, and identity experts behind
the real ones.  There is no position limit in the configuration, so ``max_position`` is the caller's.

Tensor names: ``embed``, ``head``, ``final.norm``, and per layer ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.{q,k,v,o,q.norm,k.norm,rel,vmix}``, ``l<i>.mlp.{router,correction,e<k>.gate,e<k>.up,e<k>.down}``.  What the
design fixes is fixed here: the sinusoid's base, the slope 1.702 inside the units' sigmoid and the one added to their
up branch.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.model_config import ConfigError, ModelConfig, require
from ..config.registry import architecture_name, register_architecture
from ..parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

# positions an engine is given when its caller names no limit (the configuration has none)
DEFAULT_MAX_POSITION = 1 << 17
SINUSOID_BASE = 10000.0
UNIT_SLOPE = 1.702  # g * sigmoid(1.702 g)
UNIT_SHIFT = 1.0    # ... * (u + 1)

_MIXER_NAMES = (("q", "q"), ("k", "k"), ("v", "v"), ("o", "o"), ("q_norm", "q.norm"), ("k_norm", "k.norm"), ("rel", "rel"), ("mix", "vmix"))
_MIXER_KINDS = ("attention", "attention_2")


def _section(raw: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    value = raw.get(key)
    if not isinstance(value, dict):
        raise ConfigError(f"config.json: {where}{key!r} must be an object")
    return value


@dataclass
class DipisunConfig(ModelConfig):
    width: int = 0
    vocab: int = 0
    norm_eps: float = 0.0
    residual_mult: float = 1.0
    layers: List[Dict[str, Any]] = field(default_factory=list)  # validated copies of the configuration's entries

    @staticmethod
    def from_dict(raw: Dict[str, Any]) -> "DipisunConfig":
        width, vocab = require(raw, "width", int), require(raw, "vocab", int)
        eps = require(_section(raw, "norm", ""), "eps", float)
        mult = float(raw.get("residual_mult", 1.0))
        if width <= 0 or vocab <= 0 or eps <= 0:
            raise ConfigError("width, vocab and norm.eps must be positive")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        layers: List[Dict[str, Any]] = []
        blended_size: Optional[int] = None
        for index, entry in enumerate(listed):
            where = f"layers[{index}]."
            kind = entry.get("type")
            if kind not in _MIXER_KINDS:
                raise ConfigError(f"{where}type={kind!r} is not a layer of this design ({', '.join(_MIXER_KINDS)})")
            mixer = _section(entry, "mixer", where)
            sizes = {key: require(mixer, key, int) for key in ("heads", "kv_heads", "dim", "vdim")}
            if min(sizes.values()) <= 0 or sizes["heads"] % sizes["kv_heads"]:
                raise ConfigError(f"{where}mixer: heads, kv_heads, dim and vdim must be positive and heads a multiple of kv_heads")
            scale = require(mixer, "scale", float)
            if not scale > 0:
                raise ConfigError(f"{where}mixer.scale must be positive")
            temperature = bias_far = None
            if kind == "attention":
                if mixer.get("q_temp") is not None:
                    temp = _section(mixer, "q_temp", where + "mixer.")
                    temperature = (require(temp, "coef", float), require(temp, "every", int))
                    if temperature[1] < 1:
                        raise ConfigError(f"{where}mixer.q_temp.every must be at least 1")
                bias_far = require(mixer, "bias_max", float)
                if not bias_far > 0:
                    raise ConfigError(f"{where}mixer.bias_max must be positive")
            blends = bool(mixer.get("v_mix", False))
            if blends:
                size = sizes["kv_heads"] * sizes["vdim"]
                if blended_size is not None and size != blended_size:
                    raise ConfigError(f"{where}mixer: layers that blend values need values of one size (kv_heads * vdim = {blended_size}), got {size}")
                blended_size = size
            mlp = entry.get("mlp")
            feed_forward: Optional[Dict[str, Any]] = None
            if mlp is not None:
                if mlp.get("kind") != "moe":
                    raise ConfigError(f"{where}mlp.kind={mlp.get('kind')!r} is not a feed-forward of this design (only 'moe')")
                router = _section(mlp, "router", where + "mlp.")
                expert = _section(mlp, "expert", where + "mlp.")
                feed_forward = {"ff": require(expert, "ff", int), "limit": require(expert, "limit", float), "experts": require(router, "experts", int),
                                "identity": int(router.get("identity", 0) or 0), "top": require(router, "top", int)}
                if feed_forward["ff"] <= 0 or feed_forward["experts"] < 1 or feed_forward["identity"] < 0 or not feed_forward["limit"] > 0:
                    raise ConfigError(f"{where}mlp: ff, experts and limit must be positive, identity not negative")
                if not 1 <= feed_forward["top"] <= feed_forward["experts"] + feed_forward["identity"]:
                    raise ConfigError(f"{where}mlp.router: top={feed_forward['top']} must lie between 1 and the number of router outputs")
            layers.append({"kind": kind, "sizes": sizes, "scale": scale, "q_temp": temperature, "bias_far": bias_far, "v_mix": blends, "mlp": feed_forward})
        return DipisunConfig(architecture=architecture_name(raw), raw=dict(raw), width=width, vocab=vocab, norm_eps=eps, residual_mult=mult, layers=layers)

    def to_json_dict(self) -> Dict[str, Any]:
        return {key: value for key, value in self.raw.items() if key != "tensor_shapes"}


def dipisun_spec(config: DipisunConfig, max_position: Optional[int] = None) -> ModelSpec:
    max_position = int(max_position or DEFAULT_MAX_POSITION)
    width = config.width
    norm = PartSpec.of("rmsnorm", hidden_size=width, eps=config.norm_eps, weight_name="")
    layers: List[LayerSpec] = []
    schedule: List[ScheduleEntry] = []
    seen_blend = False
    for index, layer in enumerate(config.layers):
        sizes = layer["sizes"]
        value_mix = None
        if layer["v_mix"]:
            value_mix, seen_blend = ("blend" if seen_blend else "first"), True
        biased = layer["kind"] == "attention"
        buckets = None
        if biased:
            buckets = _bias_buckets(config, index)
        mixer = PartSpec.of("normed_attention", hidden_size=width, num_heads=sizes["heads"], num_kv_heads=sizes["kv_heads"], dim=sizes["dim"], vdim=sizes["vdim"],
                            scale=layer["scale"], norm_eps=config.norm_eps, qk_norm="whole" if biased else "per_head", q_temp=layer["q_temp"],
                            distance_bias=(buckets, layer["bias_far"]) if biased else None, value_mix=value_mix, names=_MIXER_NAMES)
        mlp = layer["mlp"]
        if mlp is None:
            feed_forward = PartSpec.of("none")
        else:
            feed_forward = PartSpec.of("routed_experts", hidden_size=width, intermediate_size=mlp["ff"], num_experts=mlp["experts"], top=mlp["top"],
                                       score="softmax", renormalize=False, scale_input=False, expert_names=("e{e}.gate", "e{e}.up", "e{e}.down"),
                                       router_name="router", unit=(UNIT_SLOPE, mlp["limit"], UNIT_SHIFT), identity_experts=mlp["identity"],
                                       correction_name="correction")
        layers.append(LayerSpec(prefix=f"l{index}.", mixer=mixer, feed_forward=feed_forward, mixer_norm=norm, ff_norm=norm, arrangement="output_norm",
                                arrangement_args=(("residual_mult", config.residual_mult),), mixer_prefix="mix.", feed_forward_prefix="mlp.",
                                mixer_norm_prefix="norm1", ff_norm_prefix="norm2"))
        schedule.append(ScheduleEntry(index))
    return ModelSpec(vocab_size=config.vocab, hidden_size=width, max_position=max_position, layers=layers, schedule=schedule, final_norm=norm,
                     positions={"sinusoid": PartSpec.of("sinusoidal", width=width, base=SINUSOID_BASE)}, embedding_position="sinusoid", tie_head=False,
                     embed_name="embed", head_name="head", final_norm_prefix="final.norm", eos_token_ids=())


def _bias_buckets(config: DipisunConfig, index: int) -> int:
    """Rows of layer ``index``'s table of biases: a size that only the tensor's shape gives.  A folder's reader notes the
    shapes under ``tensor_shapes`` of the configuration; a configuration without them says ``bias_buckets`` per mixer."""
    name = f"l{index}.mix.rel"
    shapes = config.raw.get("tensor_shapes") or {}
    if name in shapes:
        return int(shapes[name][0])
    stated = config.raw["layers"][index]["mixer"].get("bias_buckets")
    if stated is None:
        raise ConfigError(f"layers[{index}].mixer: the number of distance buckets is the first size of tensor {name!r}; "
                          "read the configuration from a model folder or state 'bias_buckets'")
    return int(stated)


register_architecture("Dipisun", DipisunConfig.from_dict, dipisun_spec, reads_tensor_shapes=True)
