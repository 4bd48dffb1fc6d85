"""Small Dipisun configurations and weights for the tests, written here from the design's tensor names and shapes
(not from the framework's tables, so that a wrong name or shape there shows), with weights sharp enough that
attention is peaked, the bias by distance matters, the correction changes which experts are chosen and the
units' clamps are reached: a key that is lost, a bucket that is one off or a blend that is left out then changes
the logits by far more than any tolerance."""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import torch
from safetensors.torch import save_file


def biased(heads, kv_heads, dim, vdim, scale, buckets, far, temp=None, v_mix=False) -> dict:
    """A layer of type ``attention``; ``buckets`` is the first size of its bias table (``bias_buckets`` in the
    configuration stands for it where no folder with tensors is at hand)."""
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "bias_max": far, "bias_buckets": buckets}
    if temp is not None:
        mixer["q_temp"] = {"coef": temp[0], "every": temp[1]}
    if v_mix:
        mixer["v_mix"] = True
    return {"type": "attention", "mixer": mixer}


def plain(heads, kv_heads, dim, vdim, scale, v_mix=False) -> dict:
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if v_mix:
        mixer["v_mix"] = True
    return {"type": "attention_2", "mixer": mixer}


def moe(experts, identity, top, ff, limit) -> dict:
    return {"kind": "moe", "router": {"experts": experts, "identity": identity, "top": top}, "expert": {"ff": ff, "limit": limit}}


def layer(mix: dict, mlp: Optional[dict]) -> dict:
    return dict(mix, mlp=mlp)


# Sizes that differ wherever two could be told apart: query/key heads wider and narrower than value heads, heads that are
# no multiple of 16, a blending layer before which a layer does not blend, a layer without a feed-forward, bias tables of
# 8 and 6 rows reaching 24 and 10 positions back, a temperature that changes every 8 positions, one to three experts per
# token with none, one or two identity experts.
CONFIG_A = {
    "architecture": "Dipisun", "vocab": 97, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 0.7,
    "layers": [
        layer(plain(4, 2, 16, 8, 0.6), moe(4, 1, 2, 24, 1.0)),
        layer(biased(4, 1, 12, 20, 0.5, 8, 24, temp=(0.4, 8), v_mix=True), None),
        layer(plain(2, 2, 24, 10, 0.45, v_mix=True), moe(3, 0, 1, 16, 2.0)),
        layer(biased(3, 1, 8, 20, 0.7, 6, 10, v_mix=True), moe(5, 2, 3, 20, 0.75)),
    ],
}
# Nothing a multiple of 4, 8 or 16 where it need not be: rows of 2 x 86 bytes, an odd number of buckets, as many
# key/value heads as query heads, a far end that is no integer.
CONFIG_B = {
    "architecture": "Dipisun", "vocab": 131, "width": 86, "norm": {"eps": 3e-6}, "residual_mult": 1.3,
    "layers": [
        layer(biased(3, 3, 10, 6, 0.6, 7, 33.5, temp=(1.1, 5), v_mix=True), moe(6, 1, 3, 22, 1.5)),
        layer(plain(5, 1, 6, 18, 0.8, v_mix=True), moe(3, 3, 2, 10, 0.5)),
    ],
}
# Sizes the kernels for decode-sized bfloat16 batches and the matrix cores take (multiples of 64 and 8).
CONFIG_C = {
    "architecture": "Dipisun", "vocab": 160, "width": 128, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
    "layers": [
        layer(biased(4, 2, 32, 64, 0.3, 12, 100, temp=(0.3, 64), v_mix=True), moe(8, 2, 2, 64, 1.25)),
        layer(plain(8, 2, 64, 64, 0.22, v_mix=True), moe(8, 0, 3, 32, 3.0)),
        layer(plain(4, 4, 32, 16, 0.3), None),
        layer(biased(8, 1, 16, 128, 0.4, 32, 70, v_mix=True), moe(4, 1, 1, 64, 1.0)),
    ],
}
# What other configurations make differ is equal or 1 here: one factor of 1 on the residual, one head, one expert per
# token, a temperature that changes at every position, no identity experts, no blending, two buckets.
CONFIG_D = {
    "architecture": "Dipisun", "vocab": 64, "width": 48, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
    "layers": [
        layer(biased(1, 1, 16, 16, 0.5, 2, 3, temp=(0.25, 1)), moe(2, 0, 1, 48, 1.0)),
        layer(plain(1, 1, 48, 48, 0.3), moe(1, 0, 1, 8, 4.0)),
    ],
}
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C, "D": CONFIG_D}
PAGE_SIZE = {"A": 4, "B": 8, "C": 16, "D": 16}


def tensor_shapes(config: dict) -> Dict[str, tuple]:
    width = config["width"]
    shapes = {"embed": (config["vocab"], width), "final.norm": (width,), "head": (config["vocab"], width)}
    for i, entry in enumerate(config["layers"]):
        m, p = entry["mixer"], f"l{i}."
        whole = entry["type"] == "attention"
        shapes[p + "norm1"] = (width,)
        shapes[p + "mix.q"] = (m["heads"] * m["dim"], width)
        shapes[p + "mix.k"] = (m["kv_heads"] * m["dim"], width)
        shapes[p + "mix.v"] = (m["kv_heads"] * m["vdim"], width)
        shapes[p + "mix.q.norm"] = (m["heads"] * m["dim"] if whole else m["dim"],)
        shapes[p + "mix.k.norm"] = (m["kv_heads"] * m["dim"] if whole else m["dim"],)
        if whole:
            shapes[p + "mix.rel"] = (m["bias_buckets"], m["heads"])
        if m.get("v_mix"):
            shapes[p + "mix.vmix"] = ()
        shapes[p + "mix.o"] = (width, m["heads"] * m["vdim"])
        mlp = entry["mlp"]
        if mlp is None:
            continue
        shapes[p + "norm2"] = (width,)
        outputs = mlp["router"]["experts"] + mlp["router"]["identity"]
        shapes[p + "mlp.router"] = (outputs, width)
        shapes[p + "mlp.correction"] = (outputs,)
        for e in range(mlp["router"]["experts"]):
            q, ff = f"{p}mlp.e{e}.", mlp["expert"]["ff"]
            shapes[q + "gate"], shapes[q + "up"], shapes[q + "down"] = (ff, width), (ff, width), (width, ff)
    return shapes


def random_weights(config: dict, seed: int) -> Dict[str, torch.Tensor]:
    """float32 tensors: matrices N(0, 1 / fan-in) (the units' and the routers' larger, so that clamps are reached and
    routers decide), q/k norm weights around 1.5, bias tables N(0, 1.5), corrections N(0, 0.15), blends in (0.2, 0.8),
    other norm weights 1 + N(0, 0.1), the embedding N(0, 1)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        if name.endswith(".vmix"):
            out[name] = 0.2 + 0.6 * torch.rand((), generator=g)
        elif name.endswith(".rel"):
            out[name] = 1.5 * torch.randn(shape, generator=g)
        elif name.endswith(".correction"):
            out[name] = 0.15 * torch.randn(shape, generator=g)
        elif name.endswith((".q.norm", ".k.norm")):
            out[name] = 1.5 + 0.3 * torch.randn(shape, generator=g)
        elif len(shape) == 1:
            out[name] = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif name == "embed":
            out[name] = torch.randn(shape, generator=g)
        else:
            gain = 2.5 if name.endswith((".router", ".gate", ".up")) else 1.0
            out[name] = torch.randn(shape, generator=g) * (gain / shape[1] ** 0.5)
    return out


def write_folder(path, config: dict, seed: int, dtype: str = "float32", weights: Optional[Dict[str, torch.Tensor]] = None, strip: bool = True) -> str:
    """``strip``: the written configuration does not say ``bias_buckets``, as a folder from elsewhere would not: the
    reader has to take it from the tensor's shape."""
    path = str(path)
    os.makedirs(path, exist_ok=True)
    weights = weights if weights is not None else random_weights(config, seed)
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    save_file({name: t.to(storage).contiguous() for name, t in weights.items()}, os.path.join(path, "model.safetensors"))
    written = json.loads(json.dumps(config))
    if strip:
        for entry in written["layers"]:
            entry["mixer"].pop("bias_buckets", None)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(written, handle)
    return path


def prompts(vocab: int, lengths, seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}
