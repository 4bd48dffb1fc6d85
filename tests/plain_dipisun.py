"""A plain, slow Dipisun forward: whole sequences, no cache, no batching, one function per mechanism,
on the CPU in float32 or float64, sharing no code with ``velox_amd``.

Dipisun is a decoder in which a sub-layer reads the residual stream ``x`` itself and only its OUTPUT is
normed: ``x <- x + m * norm1(mixer(x))``, then ``x <- x + m * norm2(ff(x))``.  Token embeddings get a
sinusoidal position vector.  Two mixers: causal softmax attention whose queries and keys are RMS-normed
over the whole projection, with a query temperature that grows with the position and a learned bias
per head and bucket of distance; and causal softmax attention with a per-head query/key norm and no
positions at all.  Both may blend their values with the values that the first blending layer made for
the same token.  The feed-forward is a mixture of experts with softmax scores, a correction that only
steers the choice, clamped gated units, and identity experts that hand their input through.
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


def sinusoid(positions: torch.Tensor, width: int, dtype) -> torch.Tensor:
    """[T, width]: entry 2i = sin(p * 10000^(-2i/width)), entry 2i+1 = cos of the same angle."""
    out = torch.zeros((positions.shape[0], width), dtype=dtype)
    for i in range((width + 1) // 2):
        angle = positions.to(dtype) * (10000.0 ** (-2.0 * i / width))
        out[:, 2 * i] = torch.sin(angle)
        if 2 * i + 1 < width:
            out[:, 2 * i + 1] = torch.cos(angle)
    return out


def distance_bucket(n: int, buckets: int, far: float) -> int:
    """Distances below half the buckets have a bucket each; beyond, buckets grow logarithmically up to ``far``."""
    near = buckets // 2
    if n < near:
        return n
    if near == 0 or far <= near:  # (no logarithmic part to speak of: everything else is the last bucket)
        return buckets - 1
    return min(buckets - 1, near + int(math.floor(math.log(n / near) / math.log(far / near) * (buckets - near))))


def query_temperature(position: int, coef: float, every: int) -> float:
    return 1.0 + coef * math.log(math.floor((position + 1) / every) + 1)


def causal_softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv], bias [H, T, T] or None -> [T, H * dv]; query head h reads key/value head h // (H/G)."""
    t, heads, _ = q.shape
    group = heads // k.shape[1]
    out = torch.zeros((t, heads, v.shape[2]), dtype=q.dtype)
    for h in range(heads):
        g = h // group
        for i in range(t):
            scores = (k[: i + 1, g] @ q[i, h]) * scale
            if bias is not None:
                scores = scores + bias[h, i, : i + 1]
            out[i, h] = torch.softmax(scores, dim=0) @ v[: i + 1, g]
    return out.reshape(t, -1)


def blended_values(v: torch.Tensor, first: Optional[torch.Tensor], lam) -> torch.Tensor:
    return v if first is None else (1.0 - lam) * v + lam * first


def mixer_biased(x, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float, positions, first_values):
    """Attention with a whole-projection q/k norm, a query temperature and a bias by distance.  Returns (output, values)."""
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    t = x.shape[0]
    q = rms_unit(x @ w[p + "q"].T, eps) * w[p + "q.norm"]
    k = rms_unit(x @ w[p + "k"].T, eps) * w[p + "k.norm"]
    v = x @ w[p + "v"].T
    if m.get("q_temp"):
        temp = torch.tensor([query_temperature(int(pos), m["q_temp"]["coef"], m["q_temp"]["every"]) for pos in positions], dtype=x.dtype)
        q = q * temp[:, None]
    table = w[p + "rel"]
    bias = torch.zeros((heads, t, t), dtype=x.dtype)
    for i in range(t):
        for j in range(i + 1):
            bias[:, i, j] = table[distance_bucket(int(positions[i] - positions[j]), table.shape[0], m["bias_max"])]
    if m.get("v_mix") and first_values is not None:
        v = blended_values(v, first_values, w[p + "vmix"])
    out = causal_softmax_attention(q.view(t, heads, dim), k.view(t, groups, dim), v.view(t, groups, vdim), m["scale"], bias)
    return out @ w[p + "o"].T, v


def mixer_plain(x, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float, positions, first_values):
    """Attention with a per-head q/k norm (one weight of the head's size for all heads) and no positions."""
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    t = x.shape[0]
    q = rms_unit((x @ w[p + "q"].T).view(t, heads, dim), eps) * w[p + "q.norm"]
    k = rms_unit((x @ w[p + "k"].T).view(t, groups, dim), eps) * w[p + "k.norm"]
    v = x @ w[p + "v"].T
    if m.get("v_mix") and first_values is not None:
        v = blended_values(v, first_values, w[p + "vmix"])
    out = causal_softmax_attention(q, k, v.view(t, groups, vdim), m["scale"], None)
    return out @ w[p + "o"].T, v


def clamped_unit(h, gate_w, up_w, down_w, limit: float):
    g = torch.clamp(h @ gate_w.T, max=limit)
    u = torch.clamp(h @ up_w.T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down_w.T


def mixture(x, w: Dict[str, torch.Tensor], p: str, mlp: dict):
    """Softmax over all router outputs; the choice adds a correction, the weights do not; the last outputs are identity experts."""
    router = mlp["router"]
    experts, identity, top = router["experts"], router.get("identity", 0), router["top"]
    scores = torch.softmax(x @ w[p + "router"].T, dim=-1)
    steer = scores + w[p + "correction"] if (p + "correction") in w else scores
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        order = sorted(range(experts + identity), key=lambda e: (-float(steer[t, e]), e))[:top]
        for e in order:
            if e >= experts:
                out[t] += scores[t, e] * x[t]
            else:
                q = f"{p}e{e}."
                out[t] += scores[t, e] * clamped_unit(x[t], w[q + "gate"], w[q + "up"], w[q + "down"], mlp["expert"]["limit"])
    return out


def dipisun_forward(config: dict, w: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float32, keep_layers: bool = False):
    """Logits [T, vocab]; with ``keep_layers`` also the residual stream after every layer, [layers, T, width]."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps, mult, width = config["norm"]["eps"], config["residual_mult"], config["width"]
    positions = torch.arange(len(tokens))
    x = w["embed"][torch.tensor(tokens)] + sinusoid(positions, width, dtype)
    first_values = None
    seen_blend = False
    kept = []
    for index, layer in enumerate(config["layers"]):
        p = f"l{index}."
        m = layer["mixer"]
        fn = {"attention": mixer_biased, "attention_2": mixer_plain}[layer["type"]]
        mixed, values = fn(x, w, p + "mix.", m, eps, positions, first_values if seen_blend else None)
        if m.get("v_mix") and not seen_blend:
            first_values, seen_blend = values, True
        x = x + mult * rms_unit(mixed, eps) * w[p + "norm1"]
        if layer.get("mlp") is not None:
            x = x + mult * rms_unit(mixture(x, w, p + "mlp.", layer["mlp"]), eps) * w[p + "norm2"]
        kept.append(x.clone())
    logits = (rms_unit(x, eps) * w["final.norm"]) @ w["head"].T
    return (logits, torch.stack(kept)) if keep_layers else logits
