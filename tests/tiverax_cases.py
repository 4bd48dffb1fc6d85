"""Small Tiverax configurations and weights for the tests, written here from the design's tensor names and shapes
(not from the framework's tables, so that a wrong name or shape there shows), with weights large enough that
attention is peaked and routers decide clearly: a key that is lost, read from a wrong page or rotated by a wrong
angle then changes the logits by far more than any tolerance."""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import torch
from safetensors.torch import save_file


def mixer(heads, dim, rot_dim, vdim, kv_rank, scale, dims=None, base=10000.0, scaling=None, kv_from=None) -> dict:
    out = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
           "rot": {"dims": dims if dims is not None else rot_dim, "base": base}}
    if scaling is not None:
        out["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if kv_from is not None:
        out["kv_from"] = kv_from
    return out


def dense(ff) -> dict:
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None) -> dict:
    out = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def layer(mix, mlp) -> dict:
    return {"type": "latent_attention", "mixer": mix, "mlp": mlp}


# Sizes that differ from one another wherever two could be told apart: heads, plain / rotated / value channels, the
# latent's rank, a rotation over fewer channels than the rotated part has, two experts per token, a layer without a
# feed-forward, borrowers whose heads and sizes are not their lender's, cached vectors of 28 and 56 channels (padded
# to 32 and 64), a stretch whose ramp lies inside the rotation and an original length below the tests' prompts.
_STRETCH_A = (4.0, 24, 8.0, 1.0)
CONFIG_A = {
    "architecture": "Tiverax", "vocab": 97, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.75},
    "layers": [
        layer(mixer(2, 16, 8, 24, 20, 0.2, scaling=_STRETCH_A), dense(96)),
        layer(mixer(3, 8, 8, 12, 20, 0.3, scaling=_STRETCH_A, kv_from=0), moe(4, 2, 32, shared=48)),
        layer(mixer(3, 12, 16, 8, 40, 0.25, dims=12, base=500.0), None),
        layer(mixer(1, 20, 16, 16, 40, 0.2, dims=12, base=500.0, kv_from=2), moe(5, 1, 24)),
        layer(mixer(2, 16, 8, 8, 20, 0.2, scaling=_STRETCH_A, kv_from=0), dense(40)),
    ],
}
# One layer of each feed-forward kind, no stretch, no embedding scale, three experts per token, widths that are no
# multiple of 64 or 16.
CONFIG_B = {
    "architecture": "Tiverax", "vocab": 131, "width": 88, "norm": {"eps": 3e-6},
    "layers": [
        layer(mixer(4, 8, 4, 8, 12, 0.35, base=100.0), moe(6, 3, 20, shared=28)),
        layer(mixer(2, 24, 4, 20, 12, 0.2, base=100.0, kv_from=0), dense(72)),
    ],
}
# Sizes the kernels for decode-sized bfloat16 batches take (widths that are multiples of 64).
CONFIG_C = {
    "architecture": "Tiverax", "vocab": 160, "width": 128, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
    "layers": [
        layer(mixer(4, 32, 16, 32, 48, 0.15, scaling=(2.0, 32, 16.0, 1.0)), moe(8, 2, 64, shared=64)),
        layer(mixer(4, 32, 16, 16, 48, 0.15, scaling=(2.0, 32, 16.0, 1.0), kv_from=0), dense(192)),
        layer(mixer(2, 64, 32, 64, 96, 0.1), dense(128)),
    ],
}
# Nothing a multiple of 4, 8 or 16: rows of 200 bytes, odd heads, a cached vector of 24 channels, three experts of twelve.
CONFIG_D = {
    "architecture": "Tiverax", "vocab": 77, "width": 100, "norm": {"eps": 1e-5}, "embedding": {"scale": 0.5},
    "layers": [
        layer(mixer(3, 10, 6, 14, 18, 0.3, base=50.0, scaling=(3.0, 16, 4.0, 0.5)), moe(3, 2, 12, shared=20)),
        layer(mixer(5, 6, 6, 2, 18, 0.4, base=50.0, scaling=(3.0, 16, 4.0, 0.5), kv_from=0), dense(36)),
    ],
}
# A latent so wide that the cached vector (260 + 12 channels) is beyond the tiled attention kernels' 256.
CONFIG_E = {
    "architecture": "Tiverax", "vocab": 90, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0},
    "layers": [
        layer(mixer(2, 8, 12, 8, 260, 0.3, base=1000.0), dense(48)),
        layer(mixer(3, 4, 12, 4, 260, 0.3, base=1000.0, kv_from=0), None),
    ],
}
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C, "D": CONFIG_D, "E": CONFIG_E}
PAGE_SIZE = {"A": 4, "B": 8, "C": 16, "D": 16, "E": 8}


def tensor_shapes(config: dict) -> Dict[str, tuple]:
    width = config["width"]
    shapes = {"embed": (config["vocab"], width), "final.norm": (width,), "head": (config["vocab"], width)}
    for i, entry in enumerate(config["layers"]):
        m, p = entry["mixer"], f"l{i}."
        shapes[p + "norm1"] = (width,)
        shapes[p + "mix.q"] = (m["heads"] * (m["dim"] + m["rot_dim"]), width)
        if "kv_from" not in m:
            shapes[p + "mix.dkv"] = (m["kv_rank"] + m["rot_dim"], width)
            shapes[p + "mix.dkv.norm"] = (m["kv_rank"],)
        shapes[p + "mix.uk"] = (m["heads"] * m["dim"], m["kv_rank"])
        shapes[p + "mix.uv"] = (m["heads"] * m["vdim"], m["kv_rank"])
        shapes[p + "mix.g"] = (m["heads"] * m["vdim"], width)
        shapes[p + "mix.o"] = (width, m["heads"] * m["vdim"])
        mlp = entry["mlp"]
        if mlp is None:
            continue

        def unit(q, ff):
            shapes[q + "gate"], shapes[q + "up"], shapes[q + "down"] = (ff, width), (ff, width), (width, ff)

        if mlp["kind"] == "dense":
            unit(p + "mlp.", mlp["ff"])
        else:
            shapes[p + "mlp.router"] = (mlp["router"]["experts"], width)
            for e in range(mlp["router"]["experts"]):
                unit(f"{p}mlp.e{e}.", mlp["expert"]["ff"])
            if mlp.get("shared"):
                unit(p + "mlp.shared.", mlp["shared"]["ff"])
    return shapes


def random_weights(config: dict, seed: int, sharp: float = 3.0) -> Dict[str, torch.Tensor]:
    """float32 tensors: matrices N(0, 1 / fan-in), queries, latents and routers ``sharp`` times larger, norm weights
    1 + N(0, 0.1), the embedding N(0, 1) over the configuration's scale."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    scale = float(config.get("embedding", {}).get("scale", 1.0))
    for name, shape in tensor_shapes(config).items():
        if len(shape) == 1:
            out[name] = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif name == "embed":
            out[name] = torch.randn(shape, generator=g) / scale
        else:
            gain = sharp if name.endswith((".q", ".dkv", ".router")) else 1.0
            out[name] = torch.randn(shape, generator=g) * (gain / shape[1] ** 0.5)
    return out


def write_folder(path, config: dict, seed: int, dtype: str = "float32", weights: Optional[Dict[str, torch.Tensor]] = None) -> str:
    path = str(path)
    os.makedirs(path, exist_ok=True)
    weights = weights if weights is not None else random_weights(config, seed)
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    save_file({name: t.to(storage).contiguous() for name, t in weights.items()}, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(config, handle)
    return path


def prompts(vocab: int, lengths, seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}
