"""Tiverax as a ``ModelSpec``.

A decoder in which every layer reads ONE RMS norm with both sub-layers (``x += mixer(n) + ff(n)``), the mixer is
attention over a cached latent (``parts.latent_attention``) with an interleaved, stretched rotation and a sigmoid
gate, and the feed-forward is dense, a mixture of experts with a shared expert, or absent.  ``config.json`` lists
the layers one by one, each with the sizes of its mixer and feed-forward, so layers may differ in everything; a
mixer with ``kv_from: j`` has no down-projection and reads the cache of layer ``j``.  The embedding is scaled; there
is no position limit in the configuration, so ``max_position`` is the caller's (the tables are built for it).

Tensor names: ``embed``, ``head``, ``final.norm``, and per layer ``l<i>.norm1``, ``l<i>.mix.{q,dkv,dkv.norm,uk,uv,g,o}``,
``l<i>.mlp.{gate,up,down}`` (dense) or ``l<i>.mlp.{router, e<k>.gate, e<k>.up, e<k>.down, shared.gate, shared.up,
shared.down}``.  What the design fixes is fixed here: SiLU in every gated unit, sigmoid scores that are not
renormalised and scale the expert's input, a gate on the heads, softmax over all keys at or before the query.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.model_config import ConfigError, ModelConfig, require
from ..config.registry import architecture_name, register_architecture
from ..parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

# positions an engine is given when its caller names no limit (the configuration has none)
DEFAULT_MAX_POSITION = 1 << 17

_MIXER_NAMES = (("q", "q"), ("down", "dkv"), ("down_norm", "dkv.norm"), ("up_k", "uk"), ("up_v", "uv"), ("gate", "g"), ("out", "o"))
_UNIT_NAMES = ("gate", "up", "down")


def _section(raw: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    value = raw.get(key)
    if not isinstance(value, dict):
        raise ConfigError(f"config.json: {where}{key!r} must be an object")
    return value


@dataclass
class TiveraxConfig(ModelConfig):
    width: int = 0
    vocab: int = 0
    norm_eps: float = 0.0
    embedding_scale: float = 1.0
    layers: List[Dict[str, Any]] = field(default_factory=list)  # validated copies of the configuration's entries

    @staticmethod
    def from_dict(raw: Dict[str, Any]) -> "TiveraxConfig":
        width, vocab = require(raw, "width", int), require(raw, "vocab", int)
        eps = require(_section(raw, "norm", ""), "eps", float)
        scale = float(_section(raw, "embedding", "").get("scale", 1.0)) if raw.get("embedding") is not None else 1.0
        if width <= 0 or vocab <= 0 or eps <= 0:
            raise ConfigError("width, vocab and norm.eps must be positive")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        layers: List[Dict[str, Any]] = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]."
            if entry.get("type") != "latent_attention":
                raise ConfigError(f"{where}type={entry.get('type')!r} is not a layer of this design (only 'latent_attention')")
            mixer = _section(entry, "mixer", where)
            sizes = {key: require(mixer, key, int) for key in ("heads", "dim", "rot_dim", "vdim", "kv_rank")}
            if min(sizes.values()) <= 0:
                raise ConfigError(f"{where}mixer: heads, dim, rot_dim, vdim and kv_rank must be positive")
            rot = _section(mixer, "rot", where + "mixer.")
            rotation = {"dims": require(rot, "dims", int), "base": require(rot, "base", float), "stretch": None}
            if rotation["dims"] <= 0 or rotation["dims"] % 2 or rotation["dims"] > sizes["rot_dim"] or rotation["base"] <= 0:
                raise ConfigError(f"{where}mixer.rot: dims={rotation['dims']} must be even, positive and at most rot_dim={sizes['rot_dim']}; base must be positive")
            if rot.get("scaling") is not None:
                scaling = rot["scaling"]
                rotation["stretch"] = tuple(require(scaling, key, float) for key in ("factor", "original", "fast", "slow"))
                if min(rotation["stretch"]) <= 0:
                    raise ConfigError(f"{where}mixer.rot.scaling: factor, original, fast and slow must be positive")
            source = mixer.get("kv_from")
            if source is not None:
                source = int(source)
                if not 0 <= source < index or layers[source]["kv_from"] is not None:
                    raise ConfigError(f"{where}mixer.kv_from={source} must name an earlier layer that has a down-projection of its own")
                theirs = layers[source]
                if (theirs["sizes"]["kv_rank"], theirs["sizes"]["rot_dim"], theirs["rotation"]) != (sizes["kv_rank"], sizes["rot_dim"], rotation):
                    raise ConfigError(f"{where}mixer: kv_rank, rot_dim and the rotation must equal those of layer {source}, whose cache it reads")
            mlp = entry.get("mlp")
            feed_forward: Optional[Dict[str, Any]] = None
            if mlp is not None:
                kind = mlp.get("kind")
                if kind == "dense":
                    feed_forward = {"kind": "dense", "ff": require(mlp, "ff", int)}
                elif kind == "moe":
                    router = _section(mlp, "router", where + "mlp.")
                    feed_forward = {"kind": "moe", "ff": require(_section(mlp, "expert", where + "mlp."), "ff", int),
                                    "experts": require(router, "experts", int), "top": require(router, "top", int),
                                    "shared_ff": require(mlp["shared"], "ff", int) if mlp.get("shared") else None}
                    if not 1 <= feed_forward["top"] <= feed_forward["experts"]:
                        raise ConfigError(f"{where}mlp.router: top={feed_forward['top']} must lie between 1 and experts={feed_forward['experts']}")
                else:
                    raise ConfigError(f"{where}mlp.kind={kind!r} is not implemented ('dense' or 'moe')")
                if feed_forward["ff"] <= 0 or (feed_forward.get("shared_ff") or 1) <= 0:
                    raise ConfigError(f"{where}mlp: ff sizes must be positive")
            layers.append({"sizes": sizes, "scale": require(mixer, "scale", float), "rotation": rotation, "kv_from": source, "mlp": feed_forward})
            if layers[-1]["scale"] <= 0:
                raise ConfigError(f"{where}mixer.scale must be positive")
        return TiveraxConfig(architecture=architecture_name(raw), raw=dict(raw), width=width, vocab=vocab, norm_eps=eps, embedding_scale=scale, layers=layers)

    def to_json_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def tiverax_spec(config: TiveraxConfig, max_position: Optional[int] = None) -> ModelSpec:
    max_position = int(max_position or DEFAULT_MAX_POSITION)
    width = config.width
    norm = PartSpec.of("rmsnorm", hidden_size=width, eps=config.norm_eps, weight_name="")
    positions: Dict[str, PartSpec] = {}
    key_of: Dict[tuple, str] = {}
    layers: List[LayerSpec] = []
    schedule: List[ScheduleEntry] = []
    for index, layer in enumerate(config.layers):
        rotation = layer["rotation"]
        identity = (rotation["dims"], rotation["base"], rotation["stretch"])
        if identity not in key_of:  # layers with the same rotation share its tables
            key_of[identity] = f"rotation{len(key_of)}"
            positions[key_of[identity]] = PartSpec.of("rotary", rotary_dim=rotation["dims"], theta=rotation["base"], max_position=max_position,
                                                      layout="interleaved", stretch=rotation["stretch"])
        sizes = layer["sizes"]
        mixer = PartSpec.of("latent_attention", hidden_size=width, num_heads=sizes["heads"], dim=sizes["dim"], rot_dim=sizes["rot_dim"], vdim=sizes["vdim"],
                            kv_rank=sizes["kv_rank"], scale=layer["scale"], norm_eps=config.norm_eps, gate=True, own_latent=layer["kv_from"] is None,
                            names=_MIXER_NAMES)
        mlp = layer["mlp"]
        if mlp is None:
            feed_forward = PartSpec.of("none")
        elif mlp["kind"] == "dense":
            feed_forward = PartSpec.of("gated_mlp", hidden_size=width, intermediate_size=mlp["ff"], activation="silu", names=_UNIT_NAMES)
        else:
            feed_forward = PartSpec.of("routed_experts", hidden_size=width, intermediate_size=mlp["ff"], num_experts=mlp["experts"], top=mlp["top"],
                                       score="sigmoid", renormalize=False, scale_input=True, shared_intermediate_size=mlp["shared_ff"],
                                       expert_names=("e{e}.gate", "e{e}.up", "e{e}.down"), router_name="router", shared_prefix="shared.",
                                       shared_names=_UNIT_NAMES)
        layers.append(LayerSpec(prefix=f"l{index}.", mixer=mixer, feed_forward=feed_forward, mixer_norm=norm, ff_norm=norm, position=key_of[identity],
                                arrangement="parallel", mixer_prefix="mix.", feed_forward_prefix="mlp.", mixer_norm_prefix="norm1"))
        schedule.append(ScheduleEntry(index, cache_from=layer["kv_from"]))
    return ModelSpec(vocab_size=config.vocab, hidden_size=width, max_position=max_position, layers=layers, schedule=schedule, final_norm=norm,
                     positions=positions, tie_head=False, embed_name="embed", head_name="head", final_norm_prefix="final.norm",
                     eos_token_ids=(), embedding=PartSpec.of("table", scale=config.embedding_scale))


register_architecture("Tiverax", TiveraxConfig.from_dict, tiverax_spec)
