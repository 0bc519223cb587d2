"""Operator layer of the LFM2 decode/prefill step on MI355X.

Each function keeps the name, argument meaning and error behaviour of the reference function it
stands in for (cited per function, paths under the reference's src/climbing_gym/inference/), and
launches the hand-written gfx950 kernel behind the C ABI.  Outputs are fresh tensors from torch's
caching allocator unless stated, everything is ordered on the current stream and can be captured
into a HIP graph.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib
from ._lib import DTYPE_CODE, call, query
from ._checks import reject

FP8 = torch.float8_e4m3fn


def _code(dtype: torch.dtype) -> int:
    try:
        return DTYPE_CODE[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype}") from None


def _rows(x: torch.Tensor) -> int:
    return x.numel() // x.size(-1)


def _check(*tensors):
    for t in tensors:
        if t is None:
            continue
        reject(not t.is_cuda, "HIP kernels require GPU tensors")
        reject(not t.is_contiguous(), "HIP kernels require contiguous tensors")


# ----------------------------------------------------------------------------------- embedding / norms
def embedding(tokens: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """F.embedding of lfm25_cuda.py:134 for int64 token ids."""
    _check(tokens, table)
    flat = tokens.reshape(-1).to(torch.long)
    out = torch.empty((flat.numel(), table.size(1)), device=table.device, dtype=table.dtype)
    call("lfm2_embedding", out, table, flat, flat.numel(), table.size(1), table.size(0), _code(table.dtype))
    return out.view(*tokens.shape, table.size(1))


def embedding_rms_norm(tokens: torch.Tensor, table: torch.Tensor, weight: torch.Tensor, eps: float, *, fp8: bool):
    """`embedding` followed by the step's first norm, which has no residual (lfm25_cuda.py:134-137), as one launch:
    returns (norm output, hidden) or, with `fp8`, ((e4m3 rows, scales), hidden); `hidden` is the embedding itself."""
    _check(tokens, table, weight)
    flat = tokens.reshape(-1).to(torch.long)
    rows, width = flat.numel(), table.size(1)
    hidden = torch.empty((rows, width), device=table.device, dtype=table.dtype)
    if fp8:
        q = torch.empty((rows, width), device=table.device, dtype=FP8)
        scales = torch.empty(rows, device=table.device, dtype=torch.float32)
        call("lfm2_embedding_rms_norm", None, q, scales, hidden, table, flat, weight, rows, width, table.size(0), float(eps),
             _code(table.dtype))
        return (q, scales), hidden
    out = torch.empty_like(hidden)
    call("lfm2_embedding_rms_norm", out, None, None, hidden, table, flat, weight, rows, width, table.size(0), float(eps),
         _code(table.dtype))
    return out, hidden


def rms_norm(x, weight: torch.Tensor, eps: float, residual: torch.Tensor | None = None):
    """lfm25_cuda_kernels.py:47-55: returns (norm(x+residual)*w, x+residual); `summed is x` without residual.
    `x` may be a `SplitProduct` (then a residual is required and the projection's reduce pass runs inside the norm)."""
    if isinstance(x, SplitProduct):
        _check(weight, residual)
        reject(residual is None, "a deferred projection can only feed a norm that adds a residual")
        rows, width = x.shape
        out = torch.empty((rows, width), device=weight.device, dtype=x.dtype)
        summed = torch.empty_like(out)
        call("lfm2_rms_norm_split", out, summed, x.partials, x.partials.size(0), x.a_scales, x.w_scales, weight, residual,
             rows, width, float(eps), _code(x.dtype))
        return out, summed
    _check(x, weight, residual)
    out = torch.empty_like(x)
    summed = torch.empty_like(x) if residual is not None else x
    call("lfm2_rms_norm", out, summed if residual is not None else None, x, weight, residual,
         _rows(x), x.size(-1), float(eps), _code(x.dtype))
    return out, summed


@dataclass
class SplitProduct:
    """A projection left as split-K partial sums (`PackedFP8Weight.linear_quantized(..., defer_reduce=True)`,
    `linear(..., defer_reduce=True)`): the value is round((sum of partials) * a_scales[m] * w_scales[n]) in `dtype`,
    without the scales for a bf16 product.  `rms_norm_fp8` and `rms_norm` fold that reduction into their own pass;
    `materialize()` gives the ordinary tensor."""
    partials: torch.Tensor   # [splits, M, N] fp32
    a_scales: Optional[torch.Tensor]
    w_scales: Optional[torch.Tensor]
    dtype: torch.dtype

    @property
    def shape(self):
        return self.partials.shape[1:]

    def materialize(self) -> torch.Tensor:
        total = self.partials[0].clone()
        for part in self.partials[1:]:
            total += part
        if self.a_scales is None:
            return total.to(self.dtype)
        return ((total * self.a_scales[:, None]) * self.w_scales[None, :]).to(self.dtype)


def rms_norm_fp8(x, weight, eps, residual=None):
    """lfm25_fp8.py:57-64: (e4m3 rows, per-row scales, x+residual).  `x` may be a `SplitProduct`."""
    if isinstance(x, SplitProduct):
        _check(weight, residual)
        rows, width = x.shape
        q = torch.empty((rows, width), device=weight.device, dtype=FP8)
        scales = torch.empty(rows, device=weight.device, dtype=torch.float32)
        reject(residual is None, "a deferred projection can only feed a norm that adds a residual")
        summed = torch.empty((rows, width), device=weight.device, dtype=x.dtype)
        call("lfm2_rms_norm_fp8_split", q, scales, summed, x.partials, x.partials.size(0), x.a_scales, x.w_scales, weight,
             residual, rows, width, float(eps), _code(x.dtype))
        return q, scales, summed
    _check(x, weight, residual)
    q = torch.empty(x.shape, device=x.device, dtype=FP8)
    scales = torch.empty(_rows(x), device=x.device, dtype=torch.float32)
    summed = torch.empty_like(x) if residual is not None else x
    call("lfm2_rms_norm_fp8", q, scales, summed if residual is not None else None, x, weight, residual,
         _rows(x), x.size(-1), float(eps), _code(x.dtype))
    return q, scales, summed


def swiglu(x: torch.Tensor) -> torch.Tensor:
    """lfm25_cuda_kernels.py:68-72: silu(gate) * up on [M, 2I] with the gate half first."""
    _check(x)
    width = x.size(-1) // 2
    out = torch.empty((x.size(0), width), device=x.device, dtype=x.dtype)
    call("lfm2_swiglu", out, x, x.size(0), width, _code(x.dtype))
    return out


def swiglu_fp8(x: torch.Tensor):
    """lfm25_fp8.py:67-73."""
    _check(x)
    width = x.size(1) // 2
    q = torch.empty((x.size(0), width), device=x.device, dtype=FP8)
    scales = torch.empty(x.size(0), device=x.device, dtype=torch.float32)
    call("lfm2_swiglu_fp8", q, scales, x, x.size(0), width, _code(x.dtype))
    return q, scales


def quantize_rows(x: torch.Tensor, *, out: tuple[torch.Tensor, torch.Tensor] | None = None):
    """lfm25_fp8.py:108-117, including its argument errors."""
    reject(x.ndim != 2 or not x.is_cuda or not x.is_contiguous() or x.dtype not in (torch.bfloat16, torch.float16),
           "FP8 quantization requires a contiguous 2D CUDA BF16/FP16 tensor")
    reject(min(x.shape) <= 0 or x.size(1) > 32768, "FP8 row width must be in [1, 32768]")
    if out is None:
        out = (torch.empty(x.shape, device=x.device, dtype=FP8),
               torch.empty(x.size(0), device=x.device, dtype=torch.float32))
    call("lfm2_quantize_rows", out[0], out[1], x, x.size(0), x.size(1), _code(x.dtype))
    return out


def conv_update(bcx, weight, state, active=None, slot_ids=None):
    """lfm25_cuda_kernels.py:103-110: one gated short-conv step; `state` [slots,H,3] is updated in place."""
    _check(bcx, weight, state, active, slot_ids)
    width = weight.size(0)
    out = torch.empty((bcx.size(0), width), device=bcx.device, dtype=bcx.dtype)
    call("lfm2_conv_update", out, bcx, weight, state, active, slot_ids, bcx.size(0), width, state.size(0),
         _code(bcx.dtype))
    return out


def conv_update_fp8(bcx, weight, state, active=None, slot_ids=None):
    """`conv_update` followed by `quantize_rows` of its output (lfm25_cuda.py:146-149 in front of an FP8 out
    projection) as one launch; returns (e4m3 rows, per-row scales)."""
    _check(bcx, weight, state, active, slot_ids)
    width = weight.size(0)
    q = torch.empty((bcx.size(0), width), device=bcx.device, dtype=FP8)
    scales = torch.empty(bcx.size(0), device=bcx.device, dtype=torch.float32)
    call("lfm2_conv_update_fp8", q, scales, bcx, weight, state, active, slot_ids, bcx.size(0), width, state.size(0),
         _code(bcx.dtype))
    return q, scales


def prepare_qkv_store(x, q_weight, k_weight, cos, sin, positions, q_heads: int, kv_heads: int, head_dim: int, eps: float,
                      k_cache, v_cache, k_scales=None, v_scales=None, *, active=None, slot_ids=None):
    """`prepare_qkv` (lfm25_cuda_kernels.py:143-151) fused with the decode-step KV append (`store_kv` of
    lfm25_fp8_kv.py:58-69 when scale tensors are given, `append_bf16_kv` of lfm25_batching.py:66-69 otherwise):
    returns q [M,1,QH,D]; keys and values go straight into the cache views at `positions`."""
    _check(x, q_weight, k_weight, cos, sin, positions, active, slot_ids)
    reject(positions.dtype != torch.int32, "positions must be int32")
    m = x.size(0)
    q = torch.empty((m, 1, q_heads, head_dim), device=x.device, dtype=x.dtype)
    c0, c1, c2 = _cache_strides(k_cache)
    call("lfm2_prepare_qkv_store", q, x, q_weight, k_weight, cos, sin, positions, k_cache, v_cache, k_scales, v_scales,
         active, slot_ids, m, q_heads, kv_heads, head_dim, cos.size(0), float(eps), c0, c1, c2,
         int(k_scales is not None), _code(x.dtype))
    return q


def qkv_project_store_supported(packed, head_dim: int, dtype, k_cache) -> bool:
    """Whether `qkv_project_store` covers the shape: an e4m3 weight, head_dim 64, bf16, K a multiple of 128 and cache
    strides that keep a head's 16-byte pieces aligned."""
    return (packed is not None and head_dim == 64 and dtype == torch.bfloat16 and packed.values.size(1) % 128 == 0
            and all(stride % 16 == 0 for stride in _cache_strides(k_cache)))


def qkv_project_store(xq, x_scales, packed, q_weight, k_weight, cos, sin, positions, q_heads: int, kv_heads: int,
                      head_dim: int, eps: float, k_cache, v_cache, k_scales=None, v_scales=None, *, active=None, slot_ids=None):
    """The W8A8 QKV projection (`PackedFP8Weight.linear_quantized`, lfm25_fp8.py:141-168) with `prepare_qkv_store` as
    its epilogue: quantised rows in, q [M,1,QH,D] out, keys and values appended to the cache.  Same bytes as the two
    calls."""
    _check(xq, x_scales, q_weight, k_weight, cos, sin, positions, active, slot_ids)
    reject(positions.dtype != torch.int32, "positions must be int32")
    m, width = xq.shape
    reject(packed.values.shape != ((q_heads + 2 * kv_heads) * head_dim, width),
           "QKV weight does not match the activation width and head counts")
    q = torch.empty((m, 1, q_heads, head_dim), device=xq.device, dtype=q_weight.dtype)
    c0, c1, c2 = _cache_strides(k_cache)
    call("lfm2_fp8_gemm_qkv_store", q, xq, x_scales, packed.values, packed.scales, q_weight, k_weight, cos, sin, positions,
         k_cache, v_cache, k_scales, v_scales, active, slot_ids, m, q_heads, kv_heads, head_dim, width, cos.size(0),
         float(eps), c0, c1, c2, int(k_scales is not None), _code(q_weight.dtype))
    return q


def prepare_qkv(x, q_weight, k_weight, cos, sin, positions, q_heads: int, kv_heads: int, head_dim: int, eps: float):
    """lfm25_cuda_kernels.py:143-151: QK RMSNorm + rotate-half RoPE + split; q/k/v come back as [M,1,heads,D]."""
    _check(x, q_weight, k_weight, cos, sin, positions)
    reject(positions.dtype != torch.int32, "positions must be int32")
    m = x.size(0)
    q = torch.empty((m, 1, q_heads, head_dim), device=x.device, dtype=x.dtype)
    k = torch.empty((m, 1, kv_heads, head_dim), device=x.device, dtype=x.dtype)
    v = torch.empty_like(k)
    call("lfm2_prepare_qkv", q, k, v, x, q_weight, k_weight, cos, sin, positions, m, q_heads, kv_heads, head_dim,
         cos.size(0), float(eps), _code(x.dtype))
    return q, k, v


def conv_prefill(bcx, weight, state, cu_seqlens, seq_of_token, slots):
    """Packed-batch form of lfm25_engine.py:1478-1511: causal depthwise conv over each sequence of a varlen
    batch, gate, and the last three b*x of every sequence into `state[slots[seq]]`."""
    _check(bcx, weight, state, cu_seqlens, seq_of_token, slots)
    width = weight.size(0)
    out = torch.empty((bcx.size(0), width), device=bcx.device, dtype=bcx.dtype)
    call("lfm2_conv_prefill", out, state, bcx, weight, cu_seqlens, seq_of_token, slots, bcx.size(0),
         cu_seqlens.numel() - 1, width, state.size(0), _code(bcx.dtype))
    return out


def conv_prefill_fp8(bcx, weight, state, cu_seqlens, seq_of_token, slots):
    """`quantize_rows(conv_prefill(...))` (lfm25_engine.py:1478-1511, then lfm25_fp8.py:108-117): (e4m3 rows, per-token
    scales), the same bits, in one launch where a workgroup can hold whole rows (16-bit dtype, width a multiple of 8
    up to 2048) and in the two launches otherwise."""
    _check(bcx, weight, state, cu_seqlens, seq_of_token, slots)
    width = weight.size(0)
    if width % 8 or width > 2048 or bcx.dtype not in (torch.bfloat16, torch.float16):
        return quantize_rows(conv_prefill(bcx, weight, state, cu_seqlens, seq_of_token, slots))
    q = torch.empty((bcx.size(0), width), device=bcx.device, dtype=FP8)
    scales = torch.empty(bcx.size(0), device=bcx.device, dtype=torch.float32)
    call("lfm2_conv_prefill_fp8", q, scales, state, bcx, weight, cu_seqlens, seq_of_token, slots, bcx.size(0),
         cu_seqlens.numel() - 1, width, state.size(0), _code(bcx.dtype))
    return q, scales


# ----------------------------------------------------------------------------------- GEMMs
@dataclass
class RowPlacement:
    """Where a product's rows go: row m is written to `out[slots[m]]` (`out[m]` without slots) when `active[m]`
    (always without a mask) and the slot is in range; the other rows of `out` keep their contents.  This is
    `_scatter_logits` of lfm25_batching.py:25-32 done by the producing GEMM."""
    out: torch.Tensor
    slots: Optional[torch.Tensor] = None
    active: Optional[torch.Tensor] = None

    def check(self, rows: int, columns: int, dtype) -> None:
        out = self.out
        reject(out.ndim != 2 or out.size(1) != columns or out.dtype != dtype or not out.is_contiguous(),
               "placed rows need a contiguous [slots, columns] destination of the product's dtype")
        reject(self.slots is None and rows > out.size(0), "more product rows than destination rows")
        reject(self.slots is not None and (self.slots.dtype != torch.int32 or self.slots.numel() != rows),
               "slots must be int32, one per product row")
        reject(self.active is not None and (self.active.dtype not in (torch.bool, torch.uint8) or self.active.numel() != rows),
               "active must be a bool mask, one per product row")


def linear(x: torch.Tensor, weight: torch.Tensor, *, tile: int = -1, split_k: int = 0,
           place: Optional[RowPlacement] = None, defer_reduce: bool = False):
    """lfm25_cuda_kernels.py:19-29: y = x W^T on the bf16 MFMA kernel of this package; any other dtype is refused
    (there is no vendor-library path).  With `place`, rows land in `place.out`.  With `defer_reduce`, a product the
    plan splits along K comes back as a `SplitProduct` for `rms_norm` to reduce."""
    reject(x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16,
           "linear runs in bfloat16 only: this package has no GEMM for other dtypes")
    _check(x, weight)
    m, k = _rows(x), x.size(-1)
    n = weight.size(0)
    reject(weight.size(1) != k, "activation and weight widths differ")
    if place is not None:
        place.check(m, n, x.dtype)
        call("lfm2_bf16_gemm_rows", place.out, x, weight, place.slots, place.active, place.out.size(0), m, n, k, tile)
        return place.out
    if defer_reduce and x.ndim == 2:
        splits = query("lfm2_bf16_gemm_default_splits", m, n, k) if split_k == 0 else split_k
        if splits > 1:
            partials = torch.empty((splits, m, n), device=x.device, dtype=torch.float32)
            call("lfm2_bf16_gemm_partials", partials, x, weight, m, n, k, tile, splits)
            return SplitProduct(partials, None, None, x.dtype)
    out = torch.empty((*x.shape[:-1], n), device=x.device, dtype=x.dtype)
    need = query("lfm2_bf16_gemm_workspace", m, n, k) if split_k == 0 else max(split_k, 1) * m * n
    ws = torch.empty(need, device=x.device, dtype=torch.float32) if need and split_k != 1 else None
    call("lfm2_bf16_gemm", out, x, weight, ws, m, n, k, tile, split_k)
    return out


def linear_swiglu(x: torch.Tensor, weight: torch.Tensor):
    """`swiglu(linear(x, weight))` for the packed gate+up weight [2I, K] (lfm25_cuda_kernels.py:19-29 then :58-72),
    the same bits, in one launch where the product's shape has the fused form and in the two launches otherwise."""
    reject(x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16,
           "linear runs in bfloat16 only: this package has no GEMM for other dtypes")
    _check(x, weight)
    m, k, n = _rows(x), x.size(-1), weight.size(0)
    reject(weight.size(1) != k or n % 2,
           "activation and weight widths differ, or the packed gate+up weight has an odd row count")
    if x.ndim != 2 or not query("lfm2_gemm_swiglu_fits", m, n, k, 2):
        return swiglu(linear(x, weight))
    out = torch.empty((m, n // 2), device=x.device, dtype=x.dtype)
    call("lfm2_bf16_gemm_swiglu", out, x, weight, m, n, k)
    return out


def _conv_rows(rows: int, state, active, slot_ids):
    reject(state.ndim != 3 or state.size(2) != 3 or not state.is_contiguous(), "conv state must be a contiguous [slots, H, 3] tensor")
    reject(slot_ids is None and rows > state.size(0), "more rows than conv state slots")


def linear_conv_update(x: torch.Tensor, weight: torch.Tensor, conv_weight, state, active=None, slot_ids=None):
    """`conv_update(linear(x, weight), conv_weight, state, active, slot_ids)` for the packed in-projection weight [3H, K]
    (lfm25_cuda_kernels.py:19-29 then :103-110) in one launch, the same bits, where the product's shape has the fused
    form; None otherwise (the caller runs the two launches)."""
    reject(x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16, "linear runs in bfloat16 only: this package has no GEMM for other dtypes")
    _check(x, weight, conv_weight)
    m, k, n = _rows(x), x.size(-1), weight.size(0)
    reject(weight.size(1) != k or n % 3 or conv_weight.shape != (n // 3, 3), "in-projection, conv weight and activation shapes differ")
    if x.ndim != 2 or not query("lfm2_gemm_conv_fits", m, n, k, 2):
        return None
    _conv_rows(m, state, active, slot_ids)
    out = torch.empty((m, n // 3), device=x.device, dtype=x.dtype)
    call("lfm2_bf16_gemm_conv_update", out, x, weight, conv_weight, state, active, slot_ids, m, n, k, state.size(0))
    return out


@dataclass
class PackedFP8Weight:
    """lfm25_fp8.py:120-168: per-output-channel e4m3 copy of a weight.  `refresh()` re-quantises into the
    same buffers so captured graphs keep seeing current weights."""
    original: torch.Tensor
    values: torch.Tensor
    scales: torch.Tensor

    @classmethod
    def from_weight(cls, weight: torch.Tensor):
        values, scales = quantize_rows(weight)
        return cls(weight, values, scales)

    def refresh(self):
        quantize_rows(self.original, out=(self.values, self.scales))

    def linear(self, x: torch.Tensor, *, config=None):
        values, scales = quantize_rows(x)
        return self.linear_quantized(values, scales, dtype=x.dtype, config=config)

    def linear_quantized(self, x, scales, *, dtype=torch.bfloat16, config=None, defer_reduce=False, place=None):
        """config = (tile index, split_k) overrides the default tile choice.  With `defer_reduce`, a product the
        plan (default or `config`) splits along K comes back as a `SplitProduct` for `rms_norm_fp8` to reduce.
        With `place` (a `RowPlacement`) the rows land in `place.out`."""
        batch, width = x.shape
        rows = self.values.size(0)
        reject(width != self.values.size(1), "FP8 activation and weight widths differ")
        tile, split_k = (-1, 0) if config is None else (int(config[0]), int(config[1]) if len(config) > 1 else 0)
        if place is not None:
            place.check(batch, rows, dtype)
            call("lfm2_fp8_gemm_rows", place.out, x, scales, self.values, self.scales, place.slots, place.active,
                 place.out.size(0), batch, rows, width, _code(dtype), tile)
            return place.out
        if defer_reduce:
            splits = query("lfm2_fp8_gemm_default_splits", batch, rows, width) if split_k == 0 else split_k
            if splits > 1:
                partials = torch.empty((splits, batch, rows), device=x.device, dtype=torch.float32)
                call("lfm2_fp8_gemm_partials", partials, x, self.values, batch, rows, width, tile, splits)
                return SplitProduct(partials, scales, self.scales, dtype)
        out = torch.empty((batch, rows), device=x.device, dtype=dtype)
        need = query("lfm2_fp8_gemm_workspace", batch, rows, width) if split_k == 0 else max(split_k, 1) * batch * rows
        ws = torch.empty(need, device=x.device, dtype=torch.float32) if need and split_k != 1 else None
        call("lfm2_fp8_gemm", out, x, scales, self.values, self.scales, ws, batch, rows, width, _code(dtype), tile, split_k)
        return out

    def linear_conv_update(self, x, scales, conv_weight, state, active=None, slot_ids=None, *, dtype=torch.bfloat16):
        """For the packed conv in-projection weight: `conv_update(self.linear_quantized(x, scales), conv_weight, state,
        active, slot_ids)` (lfm25_fp8.py:141-168 then lfm25_cuda_kernels.py:103-110) in one launch, the same bits,
        where the product's shape has the fused form; None otherwise."""
        batch, width = x.shape
        rows = self.values.size(0)
        reject(width != self.values.size(1) or rows % 3 or conv_weight.shape != (rows // 3, 3),
               "in-projection, conv weight and activation shapes differ")
        if not query("lfm2_gemm_conv_fits", batch, rows, width, 1):
            return None
        _conv_rows(batch, state, active, slot_ids)
        out = torch.empty((batch, rows // 3), device=x.device, dtype=dtype)
        call("lfm2_fp8_gemm_conv_update", out, x, scales, self.values, self.scales, conv_weight, state, active, slot_ids,
             batch, rows, width, state.size(0), _code(dtype))
        return out

    def linear_swiglu_quantized(self, x, scales, *, dtype=torch.bfloat16):
        """For the packed gate+up weight: `swiglu_fp8(self.linear_quantized(x, scales))` (lfm25_fp8.py:141-168 then
        :67-73) as (e4m3 rows, row scales), the same bits; where the product's shape has the fused form the SwiGLU runs
        in the projection's epilogue and only [M, I] is written and quantised, otherwise the two launches run."""
        batch, width = x.shape
        rows = self.values.size(0)
        reject(width != self.values.size(1) or rows % 2,
               "FP8 activation and weight widths differ, or the packed gate+up weight has an odd row count")
        if not query("lfm2_gemm_swiglu_fits", batch, rows, width, 1):
            return swiglu_fp8(self.linear_quantized(x, scales, dtype=dtype))
        hidden = torch.empty((batch, rows // 2), device=x.device, dtype=dtype)
        call("lfm2_fp8_gemm_swiglu", hidden, x, scales, self.values, self.scales, batch, rows, width, _code(dtype))
        return quantize_rows(hidden)


# ----------------------------------------------------------------------------------- KV cache + attention
def _cache_strides(cache: torch.Tensor):
    reject(cache.ndim != 4 or cache.stride(3) != 1,
           "cache views must be [slots, positions, heads, dim] with a contiguous last dimension")
    return cache.stride(0), cache.stride(1), cache.stride(2)


def store_kv(k, v, k_cache, v_cache, k_scales, v_scales, *, positions=None, active=None, slot_ids=None):
    """lfm25_fp8_kv.py:58-69: write [batch, tokens, KV heads, dim] as e4m3 rows with fp32 scales into (possibly
    strided) cache views; append mode when `positions` is given."""
    batch, tokens, heads, dim = k.shape
    reject(k.stride(3) != 1 or v.stride(3) != 1, "k and v need a contiguous head dimension")
    c0, c1, c2 = _cache_strides(k_cache)
    call("lfm2_store_kv_fp8", k, v, k_cache, v_cache, k_scales, v_scales, positions, active, slot_ids, batch, tokens,
         heads, dim, *k.stride()[:3], *v.stride()[:3], c0, c1, c2, _code(k.dtype))


def append_bf16_kv(k, v, k_cache, v_cache, positions, slots, active):
    """lfm25_batching.py:66-69 (also the in-kernel append of flash_attn_with_kvcache); slots/active may be None."""
    _check(k, v)
    c0, c1, c2 = _cache_strides(k_cache)
    call("lfm2_append_kv", k, v, k_cache, v_cache, positions, slots, active, k.size(0), k.size(-2), k.size(-1),
         c0, c1, c2, _code(k.dtype))


def store_kv_packed(k, v, k_cache, v_cache, k_scales, v_scales, cu_seqlens, seq_of_token, slots):
    """Cache write of a varlen prefill batch (LFM25HybridCache.store_prefill, lfm25_engine.py:387-398):
    k, v are [tokens, KV heads, dim] packed by cu_seqlens; sequence i goes to cache slot slots[i]."""
    _check(k, v)
    c0, c1, c2 = _cache_strides(k_cache)
    call("lfm2_store_kv_packed", k, v, k_cache, v_cache, k_scales, v_scales, cu_seqlens, seq_of_token, slots,
         k.size(0), k.size(1), k.size(2), c0, c1, c2, int(k_scales is not None), _code(k.dtype))


def decode_schedule(positions, active=None, slot_ids=None, *, capacity: int):
    """Work list of the persistent decode-attention kernel for the rows' current lengths; one list serves every
    attention layer of a decode step (pass it to `attend(..., schedule=...)`)."""
    rows = positions.numel()
    schedule = torch.empty(query("lfm2_decode_schedule_size", rows, int(capacity)), device=positions.device, dtype=torch.int32)
    call("lfm2_decode_schedule", schedule, positions, active, slot_ids, rows)
    return schedule


def decode_begin(lengths, active=None, *, capacity: int, gather=None):
    """The head of a decode step in one launch: returns (positions, schedule) where `positions` is a snapshot of the
    rows' cache lengths for the step's layers and `schedule` the attention work list; the lengths of the rows that take
    part are advanced by one (nothing else of the step reads them).  `gather` = (input tokens [slots], activity
    flags [slots], slot map int32 [rows], tokens out int64 [rows], positions out int32 [rows], mask out bool [rows])
    makes the rows a compact batch over the slots (`gather_inputs` of lfm25_batching.py:11-22 in the same launch)."""
    if gather is None:
        rows = lengths.numel()
        positions = torch.empty(rows, device=lengths.device, dtype=torch.int32)
        schedule = torch.empty(query("lfm2_decode_schedule_size", rows, int(capacity)), device=lengths.device, dtype=torch.int32)
        call("lfm2_decode_begin", schedule, positions, None, None, lengths, None, active, None, rows)
        return positions, schedule
    input_tokens, slot_active, slots, tokens, positions, mask = gather
    rows = slots.numel()
    schedule = torch.empty(query("lfm2_decode_schedule_size", rows, int(capacity)), device=lengths.device, dtype=torch.int32)
    call("lfm2_decode_begin", schedule, positions, tokens, mask, lengths, input_tokens, slot_active, slots, rows)
    return positions, schedule


def attend(q, k_cache, v_cache, k_scales, v_scales, positions, *, active=None, scale=None, config=None,
           slot_ids=None, window=0, block_table=None, page=16, schedule=None, quantized=False):
    """lfm25_fp8_kv.py:138-167 (e4m3 history + scales) and flash_attn_with_kvcache of lfm25_cuda.py:156-165
    (`k_scales is None`: history in the model dtype).  Attends over positions [0, positions[b]]; inactive rows
    return zeros.  With `block_table` the caches are page pools [pages, page, KV heads, dim]."""
    reject(window, "sliding windows belong to LFM3 and are not part of this path")
    batch, _, query_heads, dim = q.shape
    _check(q, positions)
    heads = k_cache.size(2)
    c0, c1, c2 = _cache_strides(k_cache)
    capacity = k_cache.size(1) if block_table is None else block_table.size(1) * page
    ws = torch.empty(query("lfm2_decode_attention_workspace", batch, query_heads, dim, capacity),
                     device=q.device, dtype=torch.float32)
    if quantized:  # rows come back as (e4m3 [B, QH*D], per-row scales), ready for an FP8 out projection
        out = None
        out_q = torch.empty((batch, query_heads * dim), device=q.device, dtype=FP8)
        out_scales = torch.empty(batch, device=q.device, dtype=torch.float32)
    else:
        out, out_q, out_scales = torch.empty_like(q), None, None
    call("lfm2_decode_attention", out, q, k_cache, v_cache, k_scales, v_scales, positions, active, slot_ids,
         block_table, 0 if block_table is None else block_table.size(1), page, schedule, ws, batch, query_heads, heads, dim,
         capacity, c0, c1, c2, float(scale if scale is not None else dim ** -0.5), int(k_scales is not None),
         _code(q.dtype), out_q, out_scales)
    return (out_q, out_scales) if quantized else out


def decode(q, k, v, k_cache, v_cache, k_scales, v_scales, positions, *, active=None, scale=None, slot_ids=None, window=0,
           schedule=None):
    """lfm25_fp8_kv.py:170-172: append the new token, then attend."""
    store_kv(k, v, k_cache, v_cache, k_scales, v_scales, positions=positions, active=active, slot_ids=slot_ids)
    return attend(q, k_cache, v_cache, k_scales, v_scales, positions, active=active, scale=scale, slot_ids=slot_ids,
                  window=window, schedule=schedule)


def prefill_attention(q, k, v, cu_seqlens, max_seqlen: int, scale: float | None = None):
    """Varlen causal GQA attention (flash_attn_func of lfm25_engine.py:1415-1417 on a packed batch):
    q [tokens, QH, D], k/v [tokens, KH, D], cu_seqlens int32."""
    _check(q, k, v, cu_seqlens)
    out = torch.empty_like(q)
    call("lfm2_prefill_attention", out, q, k, v, cu_seqlens, cu_seqlens.numel() - 1, int(max_seqlen), q.size(1),
         k.size(1), q.size(2), float(scale if scale is not None else q.size(2) ** -0.5), _code(q.dtype))
    return out


# ----------------------------------------------------------------------------------- batch metadata
def build_token_map(cu_seqlens: torch.Tensor, total: int):
    """Device-side expansion of cu_seqlens into (sequence index, position) per packed token."""
    seq = torch.empty(total, device=cu_seqlens.device, dtype=torch.int32)
    pos = torch.empty_like(seq)
    call("lfm2_build_token_map", seq, pos, cu_seqlens, cu_seqlens.numel() - 1, total)
    return seq, pos


def gather_inputs(tokens, positions, mask, input_tokens, lengths, active, slots):
    """lfm25_batching.py:11-22 (writes into the three preallocated row buffers)."""
    call("lfm2_gather_inputs", tokens, positions, mask, input_tokens, lengths, active, slots, slots.numel())


def scatter_logits(saved, logits, slots, active):
    """lfm25_batching.py:25-32; `slots=None` is `where(active[:,None], logits, saved)` of lfm25_cuda.py:243."""
    call("lfm2_scatter_logits", saved, logits, slots, active, logits.size(0), logits.size(1), _code(logits.dtype))


def advance_positions(lengths, positions, slots, active):
    """lfm25_batching.py:44-46; `slots=None` advances row i itself (lfm25_cuda.py:185-186)."""
    call("lfm2_advance_positions", lengths, positions, slots, active, positions.numel())


# ----------------------------------------------------------------------------------- sampling
def _check_row_output(tensor, batch: int, dtype, device, name: str) -> None:
    """A caller-provided per-row output the kernels write through a raw pointer: right type, size and place, or None."""
    reject(tensor is not None and (not tensor.is_cuda or tensor.device != device or tensor.dtype != dtype
                                   or tensor.numel() != batch or not tensor.is_contiguous()),
           f"{name} must be a contiguous {dtype} tensor with one entry per row on the logits' device")


def _sample_scratch(batch: int, vocab: int, device):
    return torch.empty(batch * ((vocab + 4095) // 4096) * 4, device=device, dtype=torch.float32)


def sample_logits(logits: torch.Tensor, *, temperature: float, seed: int, step: int, return_logprobs: bool,
                  sampling_logprobs: torch.Tensor | None = None):
    """lfm25_sampling.py:61-92: greedy (first maximum) or a categorical draw from softmax(logits / T) over the
    full support (one uniform number per row through the inverse cumulative distribution: the same law as the
    reference's Gumbel-max); log-probabilities are the raw log-softmax of the chosen token.  Deterministic in
    (seed, step).  `sampling_logprobs` (fp32 [batch], optional) receives the draw's log-probability under
    softmax(logits / T), the third value of lfm25_engine.py:1574-1609."""
    reject(logits.ndim != 2 or not logits.is_cuda or logits.dtype not in (torch.bfloat16, torch.float16, torch.float32),
           "sampling requires a 2D CUDA BF16/FP16/FP32 logits tensor")
    logits = logits.contiguous()
    batch, vocab = logits.shape
    reject(batch == 0 or vocab == 0 or temperature < 0, "sampling requires nonempty logits and nonnegative temperature")
    tokens = torch.empty(batch, device=logits.device, dtype=torch.long)
    logprobs = torch.empty(batch, device=logits.device, dtype=torch.float32) if return_logprobs else None
    _check_row_output(sampling_logprobs, batch, torch.float32, logits.device, "sampling_logprobs")
    call("lfm2_sample", tokens, logprobs, sampling_logprobs, logits, _sample_scratch(batch, vocab, logits.device), None, None, None,
         int(seed) & 0x7FFFFFFFFFFFFFFF, int(step), float(temperature), batch, vocab, _code(logits.dtype))
    return tokens, logprobs


def sample_logits_static(logits: torch.Tensor, tokens: torch.Tensor, logprobs: torch.Tensor | None, *, temperature: float,
                         seed: int, step: int):
    """`sample_logits` into caller-provided outputs with no device allocation at all: the sampler's tile statistics
    live in a fixed 256 KiB array inside the library (at most 16384 row-tiles of 4096 logits per call; calls that
    overlap on one GPU race on it).  For callers that must not allocate; no counterpart in the reference."""
    reject(logits.ndim != 2 or not logits.is_cuda or not logits.is_contiguous()
           or logits.dtype not in (torch.bfloat16, torch.float16, torch.float32),
           "sampling requires a contiguous 2D GPU BF16/FP16/FP32 logits tensor")
    batch, vocab = logits.shape
    reject(batch == 0 or vocab == 0 or temperature < 0, "sampling requires nonempty logits and nonnegative temperature")
    reject(tokens is None, "tokens must be a contiguous torch.int64 tensor with one entry per row on the logits' device")
    _check_row_output(tokens, batch, torch.long, logits.device, "tokens")
    _check_row_output(logprobs, batch, torch.float32, logits.device, "logprobs")
    call("lfm2_sample_static", tokens, logprobs, logits, None, None, None, int(seed) & 0x7FFFFFFFFFFFFFFF, int(step),
         float(temperature), batch, vocab, _code(logits.dtype))
    return tokens, logprobs


class RowSampler:
    """lfm25_sampling.py:95-123: per-row seeds/steps/temperatures; returns buffers that are reused."""

    def __init__(self, logits):
        self.batch, self.vocab = logits.shape
        self.scratch = _sample_scratch(self.batch, self.vocab, logits.device)
        # zeros, not empty: a caller that draws only some rows into these buffers still hands valid token ids on
        self.tokens = torch.zeros(self.batch, device=logits.device, dtype=torch.long)
        self.logprobs = torch.zeros(self.batch, device=logits.device, dtype=torch.float32)

    def sample(self, logits, seeds, steps, temperatures):
        call("lfm2_sample", self.tokens, self.logprobs, None, logits, self.scratch, seeds, steps, temperatures, 0, 0, 1.0,
             self.batch, self.vocab, _code(logits.dtype))
        return self.tokens, self.logprobs


def sample_and_record(sampler: RowSampler, logits, table, input_tokens, stop_table, eos: int, cap: int):
    """`RowSampler.sample` with the session's per-row seeds, positions and temperatures followed by `record_sample` of
    the draw (lfm25_session.py:469-482), the record done by the sampler's last launch.  `table` owns the per-row state
    columns; returns the sampler's reused (tokens, logprobs) buffers."""
    call("lfm2_sample_record", sampler.tokens, sampler.logprobs, logits, sampler.scratch, table.seeds, table.rng_positions,
         table.temperatures, table.tokens, table.logprobs, table.lengths, table.limits, table.reasons, table.alive,
         table.pending, input_tokens, table.stop_states, table.stop_offsets, stop_table, table.ignore_eos,
         table.rng_positions, int(eos), int(cap), sampler.batch, sampler.vocab, _code(logits.dtype))
    return sampler.tokens, sampler.logprobs


def sample_filtered(logits, *, temperature: float = 1.0, top_k: int = 0, top_p: float = 1.0, seed: int = 0, step: int = 0,
                    seeds=None, steps=None, temperatures=None, top_ks=None, top_ps=None, return_kept: bool = False, out=None,
                    sampling_logprobs: torch.Tensor | None = None):
    """Device form of `_sample` + `_apply_top_k_top_p` (lfm25_engine.py:1574-1609, 1759-1774) for temperature > 0:
    returns (tokens, raw log-probabilities[, survivors per row]).  With per-row `temperatures`, `top_ks` (int32) and
    `top_ps` every row has its own parameters, and rows that ask for no filter or for greedy decoding are left as `out`
    holds them.  `sampling_logprobs` (fp32 [batch], optional) receives the draw's log-probability under the tempered,
    filtered distribution (lfm25_engine.py:1605-1608)."""
    reject(logits.ndim != 2 or not logits.is_cuda, "sampling requires a 2D GPU logits tensor")
    logits = logits.contiguous()
    batch, vocab = logits.shape
    tokens, logprobs = out if out is not None else (
        torch.empty(batch, device=logits.device, dtype=torch.long),
        torch.empty(batch, device=logits.device, dtype=torch.float32))
    kept = torch.empty(batch, device=logits.device, dtype=torch.int32) if return_kept else None
    _check_row_output(tokens, batch, torch.long, logits.device, "tokens")
    _check_row_output(logprobs, batch, torch.float32, logits.device, "logprobs")
    _check_row_output(sampling_logprobs, batch, torch.float32, logits.device, "sampling_logprobs")
    call("lfm2_sample_filtered", tokens, logprobs, sampling_logprobs, kept, logits, seeds, steps, temperatures, top_ks, top_ps,
         int(seed) & 0x7FFFFFFFFFFFFFFF, int(step), float(temperature), int(top_k), float(top_p), batch, vocab,
         _code(logits.dtype))
    return (tokens, logprobs, kept) if return_kept else (tokens, logprobs)


def behavior_topk(logits, selected, logprobs, k):
    """lfm25_sampling.py:137-149: top-k ids with log-probabilities that reuse the sampler's normaliser."""
    reject(not 0 < k <= min(logits.size(1), 128), 'Behavior head exceeds the vocabulary or supported size')
    values, ids = torch.topk(logits, k, dim=-1, sorted=True)
    probs = torch.empty(values.shape, dtype=torch.float32, device=logits.device)
    call("lfm2_head_logprobs", probs, logits, selected, logprobs, values.contiguous(), logits.size(0), logits.size(1),
         k, _code(logits.dtype))
    return ids, probs


def record_sample(sampled, logp, tokens, logprobs, lengths, limits, reasons, alive, pending, input_tokens,
                  stop_states, stop_offsets, stop_table, ignore_eos, rng_positions, eos: int, vocab: int, cap: int):
    """lfm25_session.py:34-56."""
    call("lfm2_record_sample", sampled, logp, tokens, logprobs, lengths, limits, reasons, alive, pending, input_tokens,
         stop_states, stop_offsets, stop_table, ignore_eos, rng_positions, int(eos), int(vocab), int(cap),
         sampled.numel())


def configure_rows(specs, table) -> None:
    """Per-row session state of newly admitted requests in one launch (lfm25_session.py:150-165, 244-262): `specs` is
    int64 [count, 8] on the device (see `lfm2_configure_rows`), `table` the object that owns the state columns."""
    call("lfm2_configure_rows", specs, specs.size(0), table.lengths.numel(), table.lengths, table.limits, table.reasons,
         table.alive, table.pending, table.ignore_eos, table.temperatures, table.top_ks, table.top_ps, table.seeds,
         table.rng_positions, table.stop_states, table.stop_offsets)


def record_head(ids, probs, out_ids, out_probs, lengths, alive, k: int, cap: int):
    """lfm25_session.py:22-31."""
    call("lfm2_record_head", ids.contiguous(), probs.contiguous(), out_ids, out_probs, lengths, alive, int(k),
         int(cap), lengths.numel())


# ----------------------------------------------------------------------------------- measurement
def hbm_stream_read(buffer: torch.Tensor, sink: torch.Tensor, *, workgroups: int, layout: int = 0) -> int:
    """Launch the loads-only streaming read of `buffer` (`lfm2_hbm_stream_read`); returns the bytes the launch reads.
    `sink` is an int32 tensor of at least workgroups * 256 entries."""
    reject(not buffer.is_cuda or not buffer.is_contiguous() or not sink.is_cuda or sink.dtype != torch.int32
           or sink.numel() < workgroups * 256, "hbm_stream_read needs a contiguous GPU buffer and an int32 sink of workgroups * 256")
    size = buffer.numel() * buffer.element_size()
    call("lfm2_hbm_stream_read", buffer, size, sink, int(workgroups), int(layout))
    return (size // 4096 // workgroups) * workgroups * 4096


def mfma_fp8_peak(sink: torch.Tensor, clock, *, workgroups: int, waves: int, iterations: int) -> int:
    """Launch the register-operand fp8 MFMA loop (`lfm2_mfma_fp8_peak`); returns the flops of the launch.  `sink` is a
    float32 tensor of at least workgroups * waves * 64 entries, `clock` None or an int64 tensor of 2 * workgroups."""
    reject(not sink.is_cuda or sink.dtype != torch.float32 or sink.numel() < workgroups * waves * 64,
           "mfma_fp8_peak needs a float32 GPU sink of workgroups * waves * 64")
    reject(clock is not None and (not clock.is_cuda or clock.dtype != torch.int64 or clock.numel() < 2 * workgroups),
           "mfma_fp8_peak's clock output is an int64 GPU tensor of 2 * workgroups")
    call("lfm2_mfma_fp8_peak", sink, clock, int(workgroups), int(waves), int(iterations))
    return workgroups * waves * iterations * 8 * (2 * 16 * 16 * 128)


def timestamp(out: torch.Tensor) -> None:
    """Store the device wall clock into the int64 element `out` points at, in stream order (`lfm2_timestamp`)."""
    reject(not out.is_cuda or out.dtype != torch.int64 or out.numel() < 1, "timestamp needs an int64 GPU element")
    call("lfm2_timestamp", out)


def timestamp_rate_hz() -> float:
    rate = query("lfm2_timestamp_rate_khz")
    reject(rate <= 0, "the device's wall-clock rate cannot be read", RuntimeError)
    return rate * 1000.0
