"""A plain, slow Tiverax forward: whole sequences, no cache, no batching, one function per mechanism,
on the CPU in float32 or float64, sharing no code with ``velox_amd``.

Tiverax is a decoder whose layers read ONE RMS norm with both sub-layers (``x += mixer(n) + ff(n)``), whose
mixer is attention over a cached low-rank latent (keys and values are expanded from it per head; one small
rotated key part is shared by all heads), with an interleaved rotation whose frequencies are stretched
(YaRN), a sigmoid gate on the concatenated heads, and whose feed-forward is either dense or a mixture of
experts with sigmoid scores that scale the expert's INPUT, plus a shared expert.  A layer may read the
latent and rotated key of an earlier layer instead of making its own.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch
from safetensors.torch import load_file


def read_folder(model_dir: str, dtype: torch.dtype = torch.float32):
    with open(os.path.join(model_dir, "config.json"), "r", encoding="utf-8") as handle:
        config = json.load(handle)
    weights = {name: (t.to(dtype) if t.is_floating_point() else t) for name, t in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return config, weights


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps), eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * weight


def stretched_frequencies(dims: int, base: float, scaling: Optional[dict], dtype=torch.float64) -> (torch.Tensor, float):
    """The rotation's frequencies f_i, i < dims/2, and the factor both cos and sin are multiplied with.

    Plain: f_i = base^(-2i/dims), factor 1.  Stretched (YaRN): with d(t) = dims ln(original / (2 pi t)) / (2 ln base),
    lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), dims - 1), r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1):
    f_i <- f_i / factor * r_i + f_i (1 - r_i), and the magnitude factor is 0.1 ln(factor) + 1."""
    i = torch.arange(dims // 2, dtype=dtype)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor, magnitude: float, dims: int) -> torch.Tensor:
    """Rotates the first ``dims`` entries of the last axis of ``x`` [T, ..., d]: (x[2i], x[2i+1]) at position p becomes
    (u cos a - v sin a, v cos a + u sin a) with a = p f_i; the rest passes unchanged."""
    angles = positions.to(freqs.dtype)[:, None] * freqs[None, :]
    cos = (angles.cos() * magnitude).to(x.dtype)
    sin = (angles.sin() * magnitude).to(x.dtype)
    while cos.dim() < x.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def latent_and_shared_key(n: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mixer: dict, eps: float, positions, freqs, magnitude):
    """What a layer with a down-projection of its own leaves for attention (and for later layers that borrow it):
    the normed latent c [T, kv_rank] and the rotated key part [T, rot_dim] that every head shares."""
    rank, rot = int(mixer["kv_rank"]), int(mixer["rot_dim"])
    down = n @ w[p + "dkv"].T
    c = rms_norm(down[:, :rank], w[p + "dkv.norm"], eps)
    shared = rotate_pairs(down[:, rank:rank + rot], positions, freqs, magnitude, int(mixer["rot"]["dims"]))
    return c, shared


def latent_attention(n: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mixer: dict, c: torch.Tensor, shared: torch.Tensor, positions, freqs, magnitude):
    """Causal softmax attention of every head over keys [W_uk c ; shared rotated part] and values W_uv c, a sigmoid gate
    on the concatenated heads, and the output product."""
    t = n.shape[0]
    heads, dim, rot, vdim = int(mixer["heads"]), int(mixer["dim"]), int(mixer["rot_dim"]), int(mixer["vdim"])
    q = (n @ w[p + "q"].T).view(t, heads, dim + rot)
    q_plain = q[..., :dim]
    q_turned = rotate_pairs(q[..., dim:], positions, freqs, magnitude, int(mixer["rot"]["dims"]))
    k_plain = (c @ w[p + "uk"].T).view(t, heads, dim)
    values = (c @ w[p + "uv"].T).view(t, heads, vdim)
    seen = positions[:, None] >= positions[None, :]
    out = torch.empty((t, heads, vdim), dtype=n.dtype)
    for h in range(heads):
        scores = (q_plain[:, h] @ k_plain[:, h].T + q_turned[:, h] @ shared.T) * float(mixer["scale"])
        weights = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1)
        out[:, h] = weights @ values[:, h]
    gated = out.reshape(t, heads * vdim) * torch.sigmoid(n @ w[p + "g"].T)
    return gated @ w[p + "o"].T


def gated_unit(x: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    """W_down (silu(W_gate x) * (W_up x))."""
    gate = x @ w[p + "gate"].T
    return (gate * torch.sigmoid(gate) * (x @ w[p + "up"].T)) @ w[p + "down"].T


def routed_experts(n: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    """Scores sigmoid(W_router n); the ``top`` largest choose the experts; the score scales the expert's input;
    a shared expert, if the layer has one, runs for every token."""
    experts, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    scores = torch.sigmoid(n @ w[p + "router"].T)
    chosen = scores.topk(top, dim=-1).indices
    out = torch.zeros_like(n)
    for e in range(experts):
        rows = (chosen == e).any(dim=-1).nonzero().flatten()
        if rows.numel():
            out[rows] += gated_unit(n[rows] * scores[rows, e:e + 1], w, f"{p}e{e}.")
    if mlp.get("shared"):
        out = out + gated_unit(n, w, p + "shared.")
    return out


def feed_forward(n: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mlp: Optional[dict]) -> torch.Tensor:
    if mlp is None:
        return torch.zeros_like(n)
    if mlp["kind"] == "dense":
        return gated_unit(n, w, p)
    if mlp["kind"] == "moe":
        return routed_experts(n, w, p, mlp)
    raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")


def tiverax_logits(config: dict, weights: Dict[str, torch.Tensor], token_ids, dtype: torch.dtype = torch.float32, residuals: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits at every position of one whole sequence, [T, vocab].  ``residuals``: a list that receives the residual
    stream after every layer."""
    w = {name: (t.to(dtype) if t.is_floating_point() else t) for name, t in weights.items()}
    ids = torch.as_tensor(list(token_ids), dtype=torch.long)
    positions = torch.arange(ids.shape[0])
    eps = float(config["norm"]["eps"])
    x = w["embed"][ids] * float((config.get("embedding") or {}).get("scale", 1.0))
    kept = {}
    for index, layer in enumerate(config["layers"]):
        if layer["type"] != "latent_attention":
            raise ValueError(f"unknown layer type {layer['type']!r}")
        mixer = layer["mixer"]
        p = f"l{index}."
        n = rms_norm(x, w[p + "norm1"], eps)
        freqs, magnitude = stretched_frequencies(int(mixer["rot"]["dims"]), float(mixer["rot"]["base"]), mixer["rot"].get("scaling"), dtype)
        source = mixer.get("kv_from")
        if source is None:
            kept[index] = latent_and_shared_key(n, w, p + "mix.", mixer, eps, positions, freqs, magnitude)
            source = index
        c, shared = kept[source]
        mixed = latent_attention(n, w, p + "mix.", mixer, c, shared, positions, freqs, magnitude)
        x = x + (mixed + feed_forward(n, w, p + "mlp.", layer.get("mlp")))
        if residuals is not None:
            residuals.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T
