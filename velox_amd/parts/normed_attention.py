"""Grouped-query softmax attention with normed queries and keys, over the paged cache.

Beside ``parts.attention`` (rotated queries and keys of one size for keys and values), this mixer has

* queries and keys that pass an RMS norm before the dot product, either over the whole projection at once
  (``qk_norm="whole"``: one weight of ``heads * dim`` and one of ``kv_heads * dim`` entries) or per head
  (``"per_head"``: one weight of ``dim`` entries for all query heads, one for all key heads);
* its own sizes for query/key heads (``dim``) and value heads (``vdim``);
* optionally a query temperature, ``q <- q * (1 + coef * ln(floor((p + 1) / every) + 1))`` at position ``p``;
* optionally a learned bias by distance, added to the scaled score: ``rel[bucket(i - j), head]`` with ``B`` buckets of
  which the first ``B // 2`` hold one distance each and the others grow logarithmically up to distance ``far``:
  ``bucket(n) = n`` below ``B // 2``, else ``min(B - 1, B // 2 + floor(ln(n / (B // 2)) / ln(far / (B // 2)) * (B - B // 2)))``;
* optionally blended values: the first layer that blends publishes its values of the step's tokens under
  ``value_mix_key``; every later one caches ``(1 - lambda) v + lambda v_first`` with its own learned ``lambda``.

There is no rotation: positions enter through the temperature and the bias only, or not at all.

How it meets the kernels: the tiled attention kernels take one head size for keys and values, a multiple of 16, so
the cache holds heads of ``D = ceil16(max(dim, vdim))`` channels whose padding is zero (zero key channels add nothing
to a dot product, zero value channels come out as zeros), the queries are written at that size by the same kernel
that norms them and writes the cache, and the output product reads a copy of its weight with zero columns at the
padding's places.  The bias is handed to the kernels as a table by distance, ``[heads, L]`` float32, where ``L - 1`` is
the first distance of the last bucket: every farther key reads the last column.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Sequence, Tuple

import torch

from .attention import SHORT_CONTEXT_KEYS, kv_pages
from .base import Mixer, Param, fused_rows, register_part, single


def distance_bucket(n: int, buckets: int, far: float) -> int:
    near = buckets // 2
    if n < near:
        return n
    if near < 1 or far <= near:
        return buckets - 1
    return min(buckets - 1, near + int(math.floor(math.log(n / near) / math.log(far / near) * (buckets - near))))


def bias_by_distance(rel: torch.Tensor, far: float) -> torch.Tensor:
    """``rel`` [B, heads] -> float32 [heads, L]: column ``n`` holds the bias of distance ``n``, the last column that of
    every distance from ``L - 1`` on."""
    buckets = rel.shape[0]
    columns = []
    n = 0
    while True:
        b = distance_bucket(n, buckets, far)
        columns.append(b)
        if b >= buckets - 1:
            break
        n += 1
    index = torch.tensor(columns, dtype=torch.long, device=rel.device)
    return rel.float()[index].t().contiguous()


class NormedAttentionMixer(Mixer):
    def __init__(
        self,
        prefix: str,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        dim: int,
        vdim: int,
        scale: float,
        norm_eps: float,
        qk_norm: str = "per_head",
        q_temp: Optional[Sequence[float]] = None,
        distance_bias: Optional[Sequence[float]] = None,
        value_mix: Optional[str] = None,
        value_mix_key: str = "first_values",
        has_mix_weight: Optional[bool] = None,
        names: Tuple[Tuple[str, str], ...] = (),
    ) -> None:
        """``q_temp = (coef, every)``; ``distance_bias = (buckets, far)``; ``value_mix``: None, ``"first"`` (publishes its
        values) or ``"blend"`` (blends with the published ones); ``has_mix_weight``: whether the checkpoint holds the
        blending weight for this layer (default: whenever ``value_mix`` is set; the publishing layer's is not used);
        ``names``: pairs (tensor, name below the prefix) that replace the default names."""
        super().__init__(prefix)
        if num_heads % num_kv_heads != 0:
            raise ValueError(f"num_heads={num_heads} must be a multiple of num_kv_heads={num_kv_heads}")
        if qk_norm not in ("whole", "per_head"):
            raise ValueError(f"qk_norm must be 'whole' or 'per_head', got {qk_norm!r}")
        if value_mix not in (None, "first", "blend"):
            raise ValueError(f"value_mix must be None, 'first' or 'blend', got {value_mix!r}")
        if min(int(dim), int(vdim)) < 1 or not float(scale) > 0:
            raise ValueError("dim and vdim must be positive, and so must the scale")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.dim = int(dim)
        self.vdim = int(vdim)
        self.cached_dim = (max(self.dim, self.vdim) + 15) // 16 * 16  # one head in the cache and in the kernels
        self.scale = float(scale)
        self.norm_eps = float(norm_eps)
        self.qk_norm = qk_norm
        self.q_temp = (float(q_temp[0]), int(q_temp[1])) if q_temp is not None else None
        if self.q_temp is not None and self.q_temp[1] < 1:
            raise ValueError("q_temp: 'every' must be at least 1")
        self.distance_bias = (int(distance_bias[0]), float(distance_bias[1])) if distance_bias is not None else None
        if self.distance_bias is not None and (self.distance_bias[0] < 1 or not self.distance_bias[1] > 0):
            raise ValueError("distance_bias: at least one bucket and a positive 'far'")
        self.value_mix = value_mix
        self.value_mix_key = value_mix_key
        self.has_mix_weight = (value_mix is not None) if has_mix_weight is None else bool(has_mix_weight)
        self.names = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight", "q_norm": "q_norm.weight",
                      "k_norm": "k_norm.weight", "rel": "distance_bias", "mix": "value_mix"}
        self.names.update(dict(names))
        self.q_size = self.num_heads * self.dim
        self.k_size = self.num_kv_heads * self.dim
        self.v_size = self.num_kv_heads * self.vdim
        self.qkv_weight: Optional[torch.Tensor] = None
        self.o_weight: Optional[torch.Tensor] = None
        self.q_norm_weight: Optional[torch.Tensor] = None
        self.k_norm_weight: Optional[torch.Tensor] = None
        self.rel: Optional[torch.Tensor] = None
        self.mix_weight: Optional[torch.Tensor] = None
        self.bias_table: Optional[torch.Tensor] = None
        self.o_padded: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        h, names = self.hidden_size, self.names
        whole = self.qk_norm == "whole"
        out = {
            "qkv_weight": fused_rows((names["q"], names["k"], names["v"]), ((self.q_size, h), (self.k_size, h), (self.v_size, h))),
            "q_norm_weight": single(names["q_norm"], (self.q_size if whole else self.dim,), role="vector", init="one_plus_normal"),
            "k_norm_weight": single(names["k_norm"], (self.k_size if whole else self.dim,), role="vector", init="one_plus_normal"),
        }
        if self.distance_bias is not None:
            out["rel"] = single(names["rel"], (self.distance_bias[0], self.num_heads), role="vector")
        if self.has_mix_weight:
            out["mix_weight"] = single(names["mix"], (), role="vector")
        out["o_weight"] = single(names["o"], (h, self.num_heads * self.vdim))
        return out

    def cache_need(self):
        return kv_pages(self.num_kv_heads, self.cached_dim)

    def finalize(self, device, dtype) -> None:
        self.refresh_derived()

    def refresh_derived(self) -> None:
        """What is derived from the bound tensors: the bias by distance and the output weight at the kernels' head size.
        To be called again after a tensor was bound anew."""
        if self.distance_bias is not None and self.rel is not None:
            self.bias_table = bias_by_distance(self.rel, self.distance_bias[1])
        self.o_padded = None
        if self.o_weight is not None and self.cached_dim != self.vdim:
            wide = torch.zeros((self.hidden_size, self.num_heads, self.cached_dim), dtype=self.o_weight.dtype, device=self.o_weight.device)
            wide[:, :, : self.vdim] = self.o_weight.view(self.hidden_size, self.num_heads, self.vdim)
            self.o_padded = wide.view(self.hidden_size, self.num_heads * self.cached_dim)
        self._prepared.pop("o_padded", None)

    def prepare_kernels(self, ops) -> None:
        load = getattr(ops, "attention_library", None)
        if load is not None and self.cached_dim <= getattr(ops, "MAX_TILED_HEAD_DIM", self.cached_dim):
            load(self.cached_dim, self.distance_bias is not None)
        self.prepare_weight(ops, "qkv_weight")
        self.prepare_weight(ops, "o_padded" if self.o_padded is not None else "o_weight")

    def capture_key_bounds(self, ops, batch: int, max_model_len: int):
        choose = getattr(ops, "choose_splits", None)
        if choose is None or max_model_len <= SHORT_CONTEXT_KEYS:
            return ()
        differs = choose(batch, self.num_kv_heads, 1, max_model_len, True) != choose(batch, self.num_kv_heads, 1, SHORT_CONTEXT_KEYS, True)
        return (SHORT_CONTEXT_KEYS,) if differs else ()

    def workspace_needs(self, ops, limits):
        sizes = getattr(ops, "attention_scratch_elems", None)
        if sizes is None:
            return {}
        partial_out, partial_lse = sizes(self.num_heads, self.num_kv_heads, self.cached_dim, limits.max_num_tokens, limits.max_num_seqs, limits.max_model_len)
        return {"attention_partial_out": partial_out, "attention_partial_lse": partial_lse}

    def forward(self, x, ctx, cache, owns_cache: bool = True):
        ops = ctx.ops
        meta = cache.batch
        qkv = ops.linear(x, self.operand("qkv_weight"), None, ctx.dtype)
        first = None
        if self.value_mix == "blend":
            first = ctx.shared.get(self.value_mix_key)
            if first is None:
                raise RuntimeError(f"{self.prefix}: no earlier layer of this step has published {self.value_mix_key!r}")
        q = ops.qk_norm_write(
            qkv, self.num_heads, self.num_kv_heads, self.dim, self.vdim, self.cached_dim,
            self.q_norm_weight, self.k_norm_weight, self.qk_norm == "whole", self.norm_eps,
            self.q_temp, ctx.positions, first, self.mix_weight if first is not None else None,
            meta.slot_mapping, cache.tensors["k"], cache.tensors["v"], cache.block_size, write_kv=owns_cache,
        )
        if self.value_mix == "first":
            # (this layer's values as the product left them: the rows of qkv behind the queries and keys)
            ctx.shared[self.value_mix_key] = (qkv, self.q_size + self.k_size)
        attn = ops.paged_attention(
            q, self.num_heads, self.num_kv_heads, self.cached_dim,
            cache.tensors["k"], cache.tensors["v"], cache.block_size,
            meta.block_tables, ctx.cu_q, meta.kv_lens,
            ctx.max_q_len, meta.max_kv_len, self.scale, None,
            ctx.all_decode, ctx.workspace,
            decode_prefix=getattr(ctx, "decode_prefix", 0), portions_max_kv_len=getattr(meta, "max_kv_len_of_portions", 0) or None,
            distance_bias=self.bias_table,
        )
        return ops.linear(attn, self.operand("o_padded" if self.o_padded is not None else "o_weight"), None, ctx.dtype)


register_part("mixer", "normed_attention", NormedAttentionMixer)
