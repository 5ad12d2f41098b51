"""Typed Python entry points of the HIP kernels.

Every function checks its operands on the host (device, dtype, layout, sizes)
before the launch, because a kernel that reads outside its buffers can take the
GPU down.  Nothing here computes on the CPU and nothing falls back to another
implementation: without a GPU or without the compiled library a call raises.
"""

from __future__ import annotations

import threading
from ctypes import c_float, c_int, c_longlong, c_void_p

import numpy as np
import torch
from torch import Tensor

from . import library

FE_F32 = 0
FE_BF16 = 1
_STATUS = {1: "bad argument", 2: "launch failed"}
_DTYPE_CODE = {torch.float32: FE_F32, torch.bfloat16: FE_BF16}
_SAMPLE_PARAMS = np.dtype([("temperature", "<f4"), ("top_k", "<i4"), ("top_p", "<f4"), ("min_p", "<f4"),
                           ("seed", "<u8"), ("draw", "<u8")])


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or failed to launch."""


def _code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dtype}") from None


def _gpu(tensor: Tensor, name: str, dtype=None, contiguous: bool = True) -> Tensor:
    if not isinstance(tensor, Tensor):
        raise KernelError(f"{name} must be a tensor")
    if tensor.device.type != "cuda":
        raise KernelError(f"{name} must live on the GPU (got {tensor.device}); there is no CPU path")
    if dtype is not None and tensor.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {tensor.dtype}")
    if contiguous and not tensor.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    return tensor


def _ptr(tensor: Tensor | None) -> c_void_p:
    return c_void_p(0 if tensor is None else tensor.data_ptr())


def _stream() -> c_void_p:
    # the raw handle of the current stream of the current device (a plain C call; building a
    # torch.cuda.Stream object for every launch costs more than the launch)
    return c_void_p(torch._C._cuda_getCurrentRawStream(torch.cuda.current_device()))


def _call(lib_name: str, fn_name: str, *args) -> None:
    fn = getattr(library.load(lib_name), fn_name)
    fn.restype = c_int
    status = fn(*args)
    if status != 0:
        raise KernelError(f"{fn_name}: {_STATUS.get(status, status)}")


# ------------------------------------------------------------------ row-wise

def embed_rows(ids: Tensor, table: Tensor, out: Tensor, scale: float = 1.0) -> Tensor:
    """out[t] = float32(table[ids[t]]) * scale; ids int32 [T], table [V, H], out float32 [T, H]."""
    _gpu(ids, "ids", torch.int32)
    _gpu(table, "table")
    _gpu(out, "out", torch.float32)
    tokens = ids.numel()
    vocab, hidden = table.shape
    if out.shape != (tokens, hidden):
        raise KernelError(f"out must be [{tokens}, {hidden}], got {tuple(out.shape)}")
    _call("rowwise", "fe_embed_rows", _ptr(ids), _ptr(table), c_int(_code(table.dtype)), _ptr(out),
          c_int(tokens), c_int(hidden), c_int(vocab), c_float(scale), _stream())
    return out


def add_rmsnorm(h: Tensor, delta: Tensor | None, weight: Tensor, eps: float, out: Tensor,
                rows: Tensor | None = None, store_sum: bool = True) -> Tensor:
    """sum = h[s] + delta[s] (float32, written back to h if store_sum);
    out[r] = sum * rsqrt(mean(sum^2) + eps) * weight, s = rows[r] or r.
    delta may be [parts, rows, hidden]: the parts are added up in order first."""
    _gpu(h, "h", torch.float32)
    _gpu(weight, "weight", torch.float32)
    _gpu(out, "out")
    total_rows, hidden = h.shape
    if weight.shape != (hidden,):
        raise KernelError(f"weight must be [{hidden}], got {tuple(weight.shape)}")
    parts = 1
    if delta is not None:
        _gpu(delta, "delta")
        parts = _delta_parts(h, delta)
    n_rows = total_rows
    if rows is not None:
        _gpu(rows, "rows", torch.int32)
        n_rows = rows.numel()
        if store_sum and delta is not None:
            raise KernelError("store_sum with a row list is not allowed (rows may repeat)")
    if out.shape != (n_rows, hidden):
        raise KernelError(f"out must be [{n_rows}, {hidden}], got {tuple(out.shape)}")
    if not eps > 0.0:
        raise KernelError("eps must be positive")
    _call("rowwise", "fe_add_rmsnorm", _ptr(h), _ptr(delta),
          c_int(_code(delta.dtype) if delta is not None else FE_F32), _ptr(weight), _ptr(out),
          c_int(_code(out.dtype)), _ptr(rows), c_int(n_rows), c_int(hidden), c_float(eps),
          c_int(1 if (store_sum and delta is not None) else 0), c_int(parts), c_longlong(h.numel()), _stream())
    return out


def _delta_parts(h: Tensor, delta: Tensor) -> int:
    if delta.shape == h.shape:
        return 1
    if delta.dim() == 3 and delta.shape[1:] == h.shape and 1 <= delta.shape[0] <= 64:
        return delta.shape[0]
    raise KernelError(f"delta must be {tuple(h.shape)} or [parts <= 64, {h.shape[0]}, {h.shape[1]}], got {tuple(delta.shape)}")


def add_rows(h: Tensor, delta: Tensor) -> Tensor:
    """h += delta, in float32; delta may be [parts, rows, hidden] (added up in order)."""
    _gpu(h, "h", torch.float32)
    _gpu(delta, "delta")
    parts = _delta_parts(h, delta)
    _call("rowwise", "fe_add_rows", _ptr(h), _ptr(delta), c_int(_code(delta.dtype)),
          c_longlong(h.numel()), c_int(parts), c_longlong(h.numel()), _stream())
    return h


def swiglu(gate_up: Tensor, out: Tensor) -> Tensor:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i]."""
    _gpu(gate_up, "gate_up")
    _gpu(out, "out", gate_up.dtype)
    tokens, two_inter = gate_up.shape
    if two_inter % 2 or out.shape != (tokens, two_inter // 2):
        raise KernelError(f"out must be [{tokens}, {two_inter // 2}], got {tuple(out.shape)}")
    _call("rowwise", "fe_swiglu", _ptr(gate_up), _ptr(out), c_int(_code(out.dtype)), c_int(tokens),
          c_int(two_inter // 2), _stream())
    return out


def stream_read(data: Tensor, sink: Tensor) -> None:
    """Read every byte of ``data`` once and do nothing else (a measurement of what the memory
    delivers); ``sink`` is one float32 that is never really written."""
    _gpu(data, "data")
    _gpu(sink, "sink", torch.float32)
    size = data.numel() * data.element_size()
    if size % 16:
        raise KernelError("the buffer's size must be a multiple of 16 bytes")
    _call("rowwise", "fe_stream_read", _ptr(data), c_longlong(size), _ptr(sink), _stream())


# ------------------------------------------------------------ matrix products

def gemm_nt_f32(a: Tensor, b: Tensor, bias: Tensor | None = None, out: Tensor | None = None) -> Tensor:
    """out[M, N] = a[M, K] @ b[N, K]^T (+ bias), true float32 (FMA, no matrix cores)."""
    _gpu(a, "a", torch.float32, contiguous=False)
    _gpu(b, "b", torch.float32, contiguous=False)
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise KernelError(f"shapes {tuple(a.shape)} x {tuple(b.shape)}^T do not match")
    if a.stride(1) != 1 or b.stride(1) != 1:
        raise KernelError("both operands must be contiguous along K")
    m, k = a.shape
    n = b.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=a.device)
    _gpu(out, "out", torch.float32)
    if out.shape != (m, n):
        raise KernelError(f"out must be [{m}, {n}], got {tuple(out.shape)}")
    if bias is not None:
        _gpu(bias, "bias", torch.float32)
        if bias.shape != (n,):
            raise KernelError(f"bias must be [{n}]")
    lda = a.stride(0) if m > 1 else max(k, a.stride(0))
    ldb = b.stride(0) if n > 1 else max(k, b.stride(0))
    _call("gemm_f32", "fe_gemm_nt_f32", _ptr(a), _ptr(b), _ptr(bias), _ptr(out), c_int(m), c_int(n),
          c_int(k), c_longlong(lda), c_longlong(ldb), c_longlong(n), _stream())
    return out


# The weight-streaming kernel takes up to 64 rows; measured on MI355X it beats the matrix library up
# to 16 rows (one MFMA row tile) and loses beyond, so the policy below stops there.
SKINNY_KERNEL_ROWS = 64
SKINNY_MAX_ROWS = 16
_EPI_F32, _EPI_BF16, _EPI_SWIGLU = 0, 1, 2


def _skinny_fits(x: Tensor, weight: Tensor, rows: int = SKINNY_MAX_ROWS) -> bool:
    return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.dim() == 2
            and x.shape[0] <= rows and x.is_contiguous() and x.shape[1] % 8 == 0
            and weight.stride(1) == 1 and weight.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def gemm_skinny(x: Tensor, weight: Tensor, epilogue: str = "bf16", tiles: int = 0, waves: int = 0,
                splits: int = 1) -> Tensor:
    """y = x @ weight^T for up to 64 rows of bfloat16 x, float32 accumulation.

    epilogue ``f32``/``bf16``: y [M, N] in that dtype; ``swiglu``: weight is
    [2I, K] with the gate rows first and y = silu(x Wg^T) * (x Wu^T) in bfloat16.
    ``splits`` > 1 (``f32`` only): K is summed in that many parts by blocks of their own
    and the result is the parts [splits, M, N], to be added up by the consumer."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(weight, "weight", torch.bfloat16, contiguous=False)
    if not _skinny_fits(x, weight, SKINNY_KERNEL_ROWS):
        raise KernelError("the skinny product takes at most 64 contiguous bfloat16 rows with K a multiple of 8")
    m, k = x.shape
    rows = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"shapes {tuple(x.shape)} x {tuple(weight.shape)}^T do not match")
    code = {"f32": _EPI_F32, "bf16": _EPI_BF16, "swiglu": _EPI_SWIGLU}[epilogue]
    if code == _EPI_SWIGLU and rows % 2:
        raise KernelError("a gated weight needs an even number of rows")
    n = rows // 2 if code == _EPI_SWIGLU else rows
    if splits != 1 and (code != _EPI_F32 or not 1 <= splits <= 16):
        raise KernelError("parts of K need the float32 epilogue and at most 16 parts")
    shape = (m, n) if splits == 1 else (splits, m, n)
    out = torch.empty(shape, dtype=torch.float32 if code == _EPI_F32 else torch.bfloat16, device=x.device)
    _call("gemm_skinny", "fe_gemm_skinny", _ptr(x), _ptr(weight), _ptr(out), c_int(m), c_int(n), c_int(k),
          c_longlong(weight.stride(0)), c_longlong(n), c_int(code), c_int(tiles), c_int(waves), c_int(splits),
          c_longlong(m * n), _stream())
    return out


# Which kernel takes a product of up to 16 rows, measured in the decode step at the sizes of Qwen3-4B, 8B and 32B
# (hidden 2560 / 4096 / 5120; milliseconds a step before -> after at the batch named).  The kernels for up to 16
# rows (`fe_gemm_skinny`) were shaped at 8 rows of the 4B sizes; the product for portions (`fe_gemm_wide`: a tile
# of 16 rows of x in LDS, 64 weight rows a block, K in the parts that fill the CUs) turned out faster for:
# * updates of the stream (output and down projections) from 4 rows (4B, batch 8: 2.83 -> 2.79, batch 16: 3.35 ->
#   3.17; 8B, batch 8: 4.15 -> 3.96; 32B, batch 16: 18.2 -> 16.3), and faster than the library there (8B, batch 16:
#   4.39 against 4.45); with up to 3 rows the K-split kernel stays (4B, batch 1: 2.50 against 2.51);
# * gate/up at K up to 3072, with gate and up rows paired in a wave, at every row count (4B: 2.50 -> 2.48 at batch 1,
#   2.83 -> 2.79 at batch 8, 3.35 -> 3.28 at batch 16); at K = 4096 the kernel whose blocks keep x in registers wins
#   (8B, batch 8: 3.94 against 4.15); a weight of more than 40,000 rows goes to the library from 2 rows (32B: 13.86
#   -> 13.50 at batch 2, 14.75 -> 14.27 at batch 8, 16.35 -> 15.85 at batch 16; a weight of 34,816 rows at the same
#   K does not: 72 against 78 us at 8 rows);
# * q/k/v: from 5 rows, in up to four parts that the attention launch adds up (4B, batch 8: 2.74 -> 2.71, batch 16:
#   3.35 -> 3.31; 8B, batch 16: 4.84 -> 4.70); a weight of more than 64 MB goes to the library from 5 rows (14B,
#   batch 8: 6.70 -> 6.61; 32B, batch 16: 15.85 -> 15.00 with the other two in place).
FEW_ROWS = 8                        # q/k/v where the product for portions does not fit: up to here the kernel for up to 16 rows
FEW_ROWS_IN_PARTS = 4               # q/k/v: up to here the kernel for up to 16 rows, then the product for portions in parts
FEW_ROWS_UPDATE = 3                 # updates of the stream: up to here
GATE_HALF_FEW_ROWS_MAX_K = 3072     # gate/up in the product that pairs gate and up rows at every row count: K up to here
GATE_LIBRARY_WEIGHT_ROWS = 40000    # gate/up through a weight of more rows than this: the library from 2 rows


IN_PARTS_MAX_WEIGHT_BYTES = 64 << 20   # q/k/v from 5 rows: a larger weight than this goes to the library (the 14B sizes'
                                       # 7168 x 5120, 73 MB: 6.70 -> 6.61 ms a step at batch 8, 7.15 -> 7.05 at 16; the 8B
                                       # sizes' 6144 x 4096, 50 MB, stays: 3.89 against 3.93)


def _few_rows_to_library(x: Tensor, weight: Tensor) -> bool:
    """A product that stores bfloat16 (q/k/v), 5 to 16 rows, a weight too large for the kernels of
    few rows to win: the matrix library."""
    return (FEW_ROWS_IN_PARTS < x.shape[0] <= SKINNY_MAX_ROWS
            and weight.shape[0] * weight.shape[1] * weight.element_size() > IN_PARTS_MAX_WEIGHT_BYTES)


def linear(x: Tensor, weight: Tensor, bias: Tensor | None = None, out_dtype=None) -> Tensor:
    """y = x @ weight^T (+ bias) for a weight in [out, in] layout; float32
    accumulation; y in ``out_dtype`` (default: x's dtype).

    float32 weights go through the true float32 kernel (a weight stored in
    32-bit stays 32-bit even in a bfloat16 model; the activation is widened).
    bfloat16: up to 16 rows take the weight-streaming kernel and up to 256 rows the
    product for portions, where the measurements above and below say they win; the
    rest is the platform's matrix library's, which the reference uses for every
    projection (its nn.Linear calls, qwen3.py:115-122,215-223).
    """
    _gpu(x, "x")
    _gpu(weight, "weight", contiguous=False)
    out_dtype = x.dtype if out_dtype is None else out_dtype
    if weight.dtype == torch.float32:
        y = gemm_nt_f32(x if x.dtype == torch.float32 else x.float(), weight, bias)
        return y if out_dtype == torch.float32 else y.to(out_dtype)
    if x.dtype != weight.dtype:
        raise KernelError(f"activation {x.dtype} does not match weight {weight.dtype}")
    if (bias is None and _skinny_fits(x, weight) and out_dtype in (torch.float32, torch.bfloat16)
            and not (out_dtype == torch.bfloat16 and _few_rows_to_library(x, weight))):
        return gemm_skinny(x, weight, "f32" if out_dtype == torch.float32 else "bf16")
    if (bias is None and out_dtype == torch.bfloat16 and _wide_fits(x, weight, WIDE_STORE_MAX_ROWS, SKINNY_MAX_ROWS + 1)
            and _wide_store_pays(x.shape[0], weight.shape[0], weight.shape[1])):
        rows = x.shape[0]        # up to 64 rows: blocks of 32 weight rows, so that the launch has twice the blocks
        return gemm_wide(x, weight, "bf16", row_tile=64 if rows <= 128 else 128, block_rows=32 if rows <= 64 else 64)
    if out_dtype == torch.float32:
        y = torch.mm(x, weight.t(), out_dtype=torch.float32)
    else:
        y = torch.matmul(x, weight.t())
    if bias is not None:
        y += bias.to(y.dtype)
    return y


# Measured on MI355X: a weight with few row tiles and a long K (the output and down projections: 160
# tiles, K = 4096 and 9728) leaves CUs idle; parts of K of about twelve 128-steps each (three and
# six parts), of equal length, summed by blocks of four waves, take 6.9 instead of 9.0 us and 13.1
# instead of 18.4 us at 8 rows.  The consumer (add_rmsnorm, add_rows) adds the parts in order; more
# parts make the product no faster and the norm slower (3.1 us behind three parts, 3.8 behind eight).
UPDATE_SPLIT_MAX_TILES = 384       # hidden sizes up to 6144 (160 tiles at 2560, 320 at 5120: both measured)
UPDATE_SPLIT_MIN_STEPS = 32
UPDATE_SPLIT_STEPS = 12        # 128-steps a part: fewer, longer parts cost the product little and save the norm reads
UPDATE_SPLIT_MAX = 16
UPDATE_SPLIT_BLOCKS = 1536     # blocks of four waves aimed at: all resident at once, parts of equal length


# Between 17 and 64 rows the product is still bound by the weight's bytes; the matrix library needs
# 21 us for each of the two projections back to the hidden size at 64 rows (1 to 2.4 TB/s).  The
# kernel below splits K over blocks of 64 weight rows, aiming at this many blocks (measured at 64
# rows: output 8.0, down 14.8, q/k/v 11.8 us; more parts make shorter pipelines and are slower).
MID_ROWS = 64
MID_TARGET_BLOCKS = 240


def _mid_parts(steps: int, blocks: int, most: int = 16) -> int:
    """Parts of K for the 17-64-row product: about MID_TARGET_BLOCKS blocks in all, at least four
    128-steps a part (the kernel fetches two steps ahead), no part without steps."""
    parts = max(1, min(most, MID_TARGET_BLOCKS // blocks, steps // 4))
    return -(-steps // -(-steps // parts))


def _mid_fits(x: Tensor, weight: Tensor) -> bool:
    return _skinny_fits(x, weight, MID_ROWS) and weight.shape[1] % 128 == 0


def gemm_mid_parts(x: Tensor, weight: Tensor, parts: int) -> Tensor:
    """Partial sums [parts, M, N] (float32) of x @ weight^T over ``parts`` runs of whole 128-steps
    of K, for up to 64 rows of bfloat16 x."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(weight, "weight", torch.bfloat16, contiguous=False)
    if not _mid_fits(x, weight) or weight.shape[1] != x.shape[1] or not 1 <= parts <= 64:
        raise KernelError("the product in parts takes at most 64 contiguous bfloat16 rows, K a multiple of 128, at most 64 parts")
    m, k = x.shape
    n = weight.shape[0]
    out = torch.empty((parts, m, n), dtype=torch.float32, device=x.device)
    _call("gemm_mid", "fe_gemm_mid_parts", _ptr(x), _ptr(weight), _ptr(out), c_int(m), c_int(n), c_int(k),
          c_longlong(weight.stride(0)), c_longlong(n), c_int(parts), c_longlong(m * n), _stream())
    return out


# Measured on MI355X at Qwen3-4B's sizes against the matrix library, per call: the products back to the
# hidden size (2560 weight rows; K = 4096 / 9728) in parts of K take 10 / 20 us at 128 rows (library 28 / 53),
# 14 / 30 us at 256 rows (25 / 46), 18 / 41 at 384 (24 / 47) and lose from 512 rows on; the q/k/v product
# (6144 weight rows) takes 18 - 20 us at 96 and 128 rows in row tiles of 64 and 23 - 26 us at 192 and 256 rows
# in tiles of 128 (library 24 and 27 - 33), 15 - 16 us at 32 and 64 rows in blocks of 32 weight rows (library
# 20 - 23); the gate/up product (19456 weight rows) is the library's at every row count above 64 (55 against
# 52 us at 256 rows).
WIDE_UPDATE_MAX_ROWS = 384     # most rows of x for which a product in parts of K beats the matrix library ...
WIDE_UPDATE_SURE_ROWS = 256    # ... for weights of up to WIDE_UPDATE_FEW_WEIGHT_ROWS rows; up to this many rows it does for every
WIDE_UPDATE_FEW_WEIGHT_ROWS = 3072   # weight measured (hidden sizes 2560, 4096, 5120 at 256 rows: output projection 14 / 21 / 45 us
                                     # against 25 / 26 / 73, down projection 30 / 55 / 146 against 46 / 59 / 178); at 384 rows the
                                     # hidden sizes 4096 and 5120 are the library's by a tenth
WIDE_STORE_MAX_ROWS = 256      # ... and a product that stores bfloat16
WIDE_STORE_MIN_BLOCKS = 140    # ... with more than 64 rows, if its launch has at least this many blocks (row tiles x 64 weight
                               # rows): q/k/v of 6144 rows 18-26 against 24-33 us and of 4608 to 5120 rows level with the library,
                               # but of 4096 rows (K = 2048, 128 blocks) 13-17 against 10-12 us
WIDE_MAX_WEIGHT_ROWS = 8192    # weights with more rows fill the chip in the library's large tiles
WIDE_GATE_MAX_K = 4096         # the gate/up product for 17 to 64 rows: beyond this K the matrix library is faster
WIDE_CUS = 256                 # the product's blocks run one a CU, round after round: the parts of K are chosen to fill the rounds


def _wide_store_pays(rows: int, weight_rows: int, k: int = 0) -> bool:
    """Whether the product for portions that stores bfloat16 beats the library: up to 64 rows unless the
    weight is large (8192 x 6144, 100 MB: 32-35 against 25-28 us), beyond if it has the blocks to fill the chip."""
    if rows <= MID_ROWS:
        return weight_rows * k * 2 <= MID_IN_PARTS_MAX_WEIGHT_BYTES
    return -(-weight_rows // 64) * -(-rows // (64 if rows <= 128 else 128)) >= WIDE_STORE_MIN_BLOCKS


def _wide_fits(x: Tensor, weight: Tensor, most_rows: int, least_rows: int = MID_ROWS + 1) -> bool:
    return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.dim() == 2 and x.is_contiguous()
            and least_rows <= x.shape[0] <= most_rows and weight.dim() == 2 and weight.stride(1) == 1
            and weight.shape[0] <= WIDE_MAX_WEIGHT_ROWS
            and weight.shape[1] == x.shape[1] and x.shape[1] % 64 == 0 and weight.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def gemm_wide(x: Tensor, weight: Tensor, ending: str = "bf16", parts: int = 1, row_tile: int = 0,
              block_rows: int = 64) -> Tensor:
    """x @ weight^T for a few dozen to a few hundred bfloat16 rows: ``"parts"`` float32 partial sums
    [parts, M, N] over runs of whole 64-steps of K, ``"bf16"`` [M, N], or ``"swiglu"``: silu(gate) * up
    [M, N / 2] for a fused gate/up weight (gate rows first)."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(weight, "weight", torch.bfloat16, contiguous=False)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k or k % 64 or weight.stride(1) != 1 or weight.stride(0) % 8 or not 1 <= parts <= 64:
        raise KernelError("the product for portions takes contiguous bfloat16 rows, K a multiple of 64, at most 64 parts")
    if ending == "parts":
        out = torch.empty((parts, m, n), dtype=torch.float32, device=x.device)
        code, cols = 0, n
    elif ending in ("bf16", "swiglu", "swiglu_half") and parts == 1 and (ending == "bf16" or n % 2 == 0):
        cols = n if ending == "bf16" else n // 2
        out = torch.empty((m, cols), dtype=torch.bfloat16, device=x.device)
        code = {"bf16": 1, "swiglu": 2, "swiglu_half": 3}[ending]
    else:
        raise KernelError(f"no ending {ending!r} with {parts} parts")
    _call("gemm_wide", "fe_gemm_wide", _ptr(x), _ptr(weight), _ptr(out), c_int(m), c_int(cols), c_int(k),
          c_longlong(weight.stride(0)), c_longlong(cols), c_int(code), c_int(parts), c_longlong(m * cols),
          c_int(row_tile or (16 if m <= 16 else 64 if m <= 64 else 128)), c_int(block_rows), _stream())
    return out


def _wide_parts(m: int, n: int, k: int, block_rows: int = 64, most: int = 16) -> int:
    """Parts of K for the product above.  Its blocks run one a CU in rounds, so the count of parts is
    the one whose blocks fill their rounds best (measured at 40 to 160 blocks a part: 240 blocks beat
    280 and 320, 480 beat 160 and 320), the smaller of near equals (every part writes and the consumer
    reads a partial sum of the whole result), at least eight 64-steps a part, no part without steps."""
    steps = k // 64
    base = -(-n // block_rows) * -(-m // (64 if m <= 64 else 128))
    best, best_fill = 1, 0.0
    for parts in range(1, max(1, min(most, steps // 8)) + 1):
        blocks = base * parts
        fill = blocks / (-(-blocks // WIDE_CUS) * WIDE_CUS) - 0.02 * parts
        if fill > best_fill + 1e-9:
            best, best_fill = parts, fill
    return -(-steps // -(-steps // best))


def linear_update(x: Tensor, weight: Tensor, bias: Tensor | None = None, stream: Tensor | None = None) -> Tensor | None:
    """The float32 product x @ weight^T (+ bias) as an update of the residual stream: [M, N], or
    partial sums [parts, M, N] that ``add_rmsnorm`` / ``add_rows`` add up.  Given the float32
    ``stream`` [M, N] itself, the matrix library's product (more than 64 rows) adds into it as it
    stores, which saves the next norm the update's bytes, and None is returned: the same float32
    sum in the same order, stream + (x @ weight^T)."""
    _gpu(x, "x")
    _gpu(weight, "weight", contiguous=False)
    plain_bf16 = bias is None and weight.dtype == torch.bfloat16 and x.dtype == torch.bfloat16
    if plain_bf16 and FEW_ROWS_UPDATE < x.shape[0] <= SKINNY_MAX_ROWS and _wide_fits(x, weight, SKINNY_MAX_ROWS, 1):
        # a tile of 16 rows of x: a tile's rows beyond M are fetched and multiplied like the others (with tiles of
        # 64 rows: 4B, batch 16: 3.05 -> 3.00 ms; 32B: 15.4 -> 14.9; tiles of 32 rows for 17 to 32 rows lose 2 to 6 %)
        return gemm_wide(x, weight, "parts", _wide_parts(x.shape[0], weight.shape[0], weight.shape[1]), row_tile=16)
    if (plain_bf16 and _skinny_fits(x, weight)
            and -(-weight.shape[0] // 16) <= UPDATE_SPLIT_MAX_TILES
            and -(-weight.shape[1] // 128) >= UPDATE_SPLIT_MIN_STEPS):
        steps, tiles = -(-weight.shape[1] // 128), -(-weight.shape[0] // 16)
        splits = max(1, min(UPDATE_SPLIT_MAX, (steps + UPDATE_SPLIT_STEPS // 2) // UPDATE_SPLIT_STEPS,
                            UPDATE_SPLIT_BLOCKS // tiles))
        splits = -(-steps // -(-steps // splits))        # parts of equal length, none empty
        return gemm_skinny(x, weight, "f32", tiles=1, waves=4, splits=splits)
    if plain_bf16 and _wide_fits(x, weight, MID_ROWS, SKINNY_MAX_ROWS + 1):
        # 17 to 64 rows: one tile of x a block, the parts of K that fill the CUs; measured at 64 rows against
        # the product below: output projection 9.2 against 11.1 us (hidden size 4096: 10.6 against 12.5),
        # down projection 15.1 against 15.3 us (25.0 against 30.2)
        return gemm_wide(x, weight, "parts", _wide_parts(x.shape[0], weight.shape[0], weight.shape[1]), row_tile=64)
    if plain_bf16 and x.shape[0] > SKINNY_MAX_ROWS and _mid_fits(x, weight):
        steps = -(-weight.shape[1] // 128)
        blocks = -(-weight.shape[0] // 64)
        return gemm_mid_parts(x, weight, _mid_parts(steps, blocks))
    if plain_bf16 and _wide_fits(x, weight, WIDE_UPDATE_MAX_ROWS if weight.shape[0] <= WIDE_UPDATE_FEW_WEIGHT_ROWS
                                 else WIDE_UPDATE_SURE_ROWS):
        # a long K beside more than 128 rows: blocks of eight waves (128 weight rows share a tile of x) in twice the
        # parts; measured at K = 9728: 29 against 32 us at 256 rows, 38 against 43 at 384 (at K = 4096 nothing)
        block_rows = 128 if x.shape[0] > 128 and weight.shape[1] >= 8192 else 64
        parts = _wide_parts(x.shape[0], weight.shape[0], weight.shape[1], block_rows)
        return gemm_wide(x, weight, "parts", parts, block_rows=block_rows)
    if (plain_bf16 and stream is not None and x.shape[0] > SKINNY_MAX_ROWS and stream.dtype == torch.float32
            and stream.shape == (x.shape[0], weight.shape[0]) and stream.is_contiguous()):
        torch.addmm(stream, x, weight.t(), out_dtype=torch.float32, out=stream)
        return None
    return linear(x, weight, bias, out_dtype=torch.float32)


# Measured on MI355X for the q/k/v projection of Qwen3-4B (6144 x 2560): two parts of K at up to 16
# rows take 10.1 instead of 12.0 us, two parts at 64 rows 11.8 instead of the library's 15.8.
IN_PARTS_MIN_STEPS = 8
IN_PARTS_FEW_ROWS = 2
MID_IN_PARTS_MAX_WEIGHT_BYTES = 80 << 20   # 17 to 64 rows in parts of K: a larger weight than this is the library's


def linear_in_parts(x: Tensor, weight: Tensor) -> Tensor | None:
    """x @ weight^T as float32 partial sums [parts <= 4, M, N] over parts of K, for a consumer that
    adds them up itself (the decode attention kernel that prepares its own queries and keys);
    None where the plain product is the better choice or the sizes do not fit."""
    _gpu(x, "x")
    _gpu(weight, "weight", contiguous=False)
    steps = -(-weight.shape[1] // 128)
    if not (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and steps >= IN_PARTS_MIN_STEPS):
        return None
    rows = x.shape[0]
    if _few_rows_to_library(x, weight):
        return None
    if FEW_ROWS_IN_PARTS < rows <= SKINNY_MAX_ROWS and _wide_fits(x, weight, SKINNY_MAX_ROWS, 1):
        # blocks of 32 weight rows in up to four parts of K (768 blocks for 6144 weight rows): 1 % of the step
        # at 6 to 16 rows against the kernels below (4B, batch 8: 2.74 -> 2.71 ms; 8B: 3.93 -> 3.89)
        parts = _wide_parts(rows, weight.shape[0], weight.shape[1], 32, most=4)
        return gemm_wide(x, weight, "parts", parts, row_tile=16, block_rows=32)
    if _skinny_fits(x, weight) and rows <= FEW_ROWS:
        return gemm_skinny(x, weight, "f32", tiles=1, waves=4, splits=IN_PARTS_FEW_ROWS)
    if (_mid_fits(x, weight) and weight.shape[0] <= WIDE_MAX_WEIGHT_ROWS
            and weight.shape[0] * weight.shape[1] * weight.element_size() <= MID_IN_PARTS_MAX_WEIGHT_BYTES):
        # (a weight of 10240 rows, K = 5120: 30 us at 32 rows against the library's 26; 7168 rows: 18 against 20;
        # 8192 rows at K = 6144, 100 MB: 35-41 against 25-27)
        return gemm_mid_parts(x, weight, _mid_parts(steps, -(-weight.shape[0] // 64), most=4))
    return None


def gemm_gated(x: Tensor, gate_up_weight: Tensor, shape: int = 0) -> Tensor:
    """silu(x Wg^T) * (x Wu^T) for the fused weight [2I, K] (gate rows first) and any number of
    bfloat16 rows: blocks keep a tile of rows of x in LDS and their accumulators in registers over
    the whole of K; the intermediate [M, 2I] never exists.  ``shape``: the block's tile, see
    ``fe_gemm_gated``."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(gate_up_weight, "gate_up_weight", torch.bfloat16, contiguous=False)
    m, k = x.shape
    rows = gate_up_weight.shape[0]
    if (gate_up_weight.dim() != 2 or gate_up_weight.shape[1] != k or k % 64 or rows % 2 or gate_up_weight.stride(1) != 1
            or gate_up_weight.stride(0) % 8 or x.data_ptr() % 16 or gate_up_weight.data_ptr() % 16):
        raise KernelError("the gated product takes contiguous bfloat16 rows, K a multiple of 64, an even number of weight rows")
    out = torch.empty((m, rows // 2), dtype=torch.bfloat16, device=x.device)
    _call("gemm_tile", "fe_gemm_gated", _ptr(x), _ptr(gate_up_weight), _ptr(out), c_int(m), c_int(rows // 2), c_int(k),
          c_longlong(gate_up_weight.stride(0)), c_longlong(rows // 2), c_int(shape), _stream())
    return out


def _gate_block_columns(columns: int) -> int:
    """Output columns a block of the gate/up product for 17 to 64 rows takes (8 a wave, four to eight
    waves): the count whose blocks fill rounds of one a CU best, the larger of equals (x is read once a
    block)."""
    def fill(width: int) -> float:
        blocks = -(-columns // width)
        return blocks / (-(-blocks // WIDE_CUS) * WIDE_CUS)
    return max((32, 40, 48, 56, 64), key=lambda width: (round(fill(width), 3), width))


# The gate/up product with its SwiGLU ending in one kernel (`fe_gemm_gated`, tiles of 256 rows of x in LDS)
# against the matrix library followed by `fe_swiglu`, microseconds at Qwen3-4B's widths (K = 2560, 9728 columns):
# 1,024 rows 134 / 126, 1,536: 157 / 148, 2,048: 199 / 224, 2,560: 264 / 310, 3,072: 297 / 272, 4,096: 377 / 438,
# 8,192: 793 / 755; at K = 4096 (12,288 columns) the library wins at every row count but one (2,048: 329 / 306,
# 4,096: 683 / 590).  So: a short K, and the row counts of a prompt portion of 2,048 to 4,096 tokens.
GATED_TILE_MIN_ROWS = 2048
GATED_TILE_MAX_ROWS = 4096
GATED_TILE_MAX_K = 3072


def linear_swiglu(x: Tensor, gate_up_weight: Tensor) -> Tensor:
    """silu(x Wg^T) * (x Wu^T) for the fused weight [2I, K] (gate rows first)."""
    _gpu(x, "x")
    _gpu(gate_up_weight, "gate_up_weight")
    rows = x.shape[0]
    if (GATED_TILE_MIN_ROWS <= rows <= GATED_TILE_MAX_ROWS and x.dtype == torch.bfloat16 and gate_up_weight.dtype == torch.bfloat16
            and x.is_contiguous() and x.shape[1] % 64 == 0 and x.shape[1] <= GATED_TILE_MAX_K and gate_up_weight.shape[0] % 2 == 0
            and gate_up_weight.dim() == 2 and gate_up_weight.stride(1) == 1 and gate_up_weight.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and gate_up_weight.data_ptr() % 16 == 0
            and gate_up_weight.shape[0] * gate_up_weight.stride(0) < 2 ** 32 and rows * x.shape[1] < 2 ** 32):
        return gemm_gated(x, gate_up_weight, shape=3)
    to_library = (2 <= rows <= SKINNY_MAX_ROWS and gate_up_weight.shape[0] > GATE_LIBRARY_WEIGHT_ROWS
                  and x.dtype == torch.bfloat16 and gate_up_weight.dtype == torch.bfloat16)
    paired_fits = (rows <= MID_ROWS and x.dtype == torch.bfloat16 and gate_up_weight.dtype == torch.bfloat16
                   and x.is_contiguous() and gate_up_weight.is_contiguous() and x.shape[1] % 64 == 0
                   and x.shape[1] <= WIDE_GATE_MAX_K and gate_up_weight.shape[0] % 2 == 0
                   and x.data_ptr() % 16 == 0 and gate_up_weight.data_ptr() % 16 == 0)
    if paired_fits and not to_library and (rows > SKINNY_MAX_ROWS or x.shape[1] <= GATE_HALF_FEW_ROWS_MAX_K):
        # gate and up rows paired in a wave.  17 to 64 rows (many requests decoding), measured at 32 rows against the
        # matrix library with the gate kernel behind it: 24 against 28 us at 9728 columns of K = 2560, 46 against 50 at
        # 12288 of K = 4096; at K = 5120 the library wins (17408 columns: 85 against 82 us, 25600 columns: 111 against
        # 96), and from 96 rows on at every size.  Up to 16 rows: see FEW_ROWS above.
        return gemm_wide(x, gate_up_weight, "swiglu_half", block_rows=_gate_block_columns(gate_up_weight.shape[0] // 2))
    if _skinny_fits(x, gate_up_weight) and not to_library:
        return gemm_skinny(x, gate_up_weight, "swiglu")
    gate_up = torch.matmul(x, gate_up_weight.t()) if to_library else linear(x, gate_up_weight)
    out = torch.empty((x.shape[0], gate_up_weight.shape[0] // 2), dtype=gate_up.dtype, device=x.device)
    return swiglu(gate_up, out)


# ------------------------------------------------------------------ attention

def qk_norm_rope_write(qkv: Tensor, q_weight: Tensor | None, k_weight: Tensor | None,
                       inv_freq: Tensor | None, positions: Tensor, token_seq: Tensor,
                       block_table: Tensor, key_pages: Tensor, value_pages: Tensor, *, q_heads: int,
                       kv_heads: int, head_dim: int, rotary_dim: int, eps: float,
                       write_kv: bool = True) -> None:
    """Per-head RMSNorm of q and k, rotation, and the write of k, v into pages.

    qkv [T, (Hq + 2 Hkv) D] is changed in place (q part); pages are
    keys [blocks, Hkv, block_size, D], values transposed [blocks, Hkv, D, block_size];
    block_table [B, max_blocks] int32.
    """
    _gpu(qkv, "qkv")
    tokens = qkv.shape[0]
    width = (q_heads + (2 * kv_heads if write_kv else 0)) * head_dim  # q only when nothing is written
    if qkv.dim() != 2 or qkv.shape[1] != width:
        raise KernelError(f"qkv must be [T, {width}], got {tuple(qkv.shape)}")
    for name, w in (("q_weight", q_weight), ("k_weight", k_weight)):
        if w is not None:
            _gpu(w, name, torch.float32)
            if w.shape != (head_dim,):
                raise KernelError(f"{name} must be [{head_dim}]")
    if rotary_dim:
        _gpu(inv_freq, "inv_freq", torch.float32)
        if inv_freq.shape != (rotary_dim // 2,):
            raise KernelError(f"inv_freq must be [{rotary_dim // 2}]")
    _gpu(positions, "positions", torch.int32)
    _gpu(token_seq, "token_seq", torch.int32)
    if positions.numel() != tokens or token_seq.numel() != tokens:
        raise KernelError("positions and token_seq must have one entry per token")
    _gpu(block_table, "block_table", torch.int32)
    _gpu(key_pages, "key_pages", qkv.dtype)
    _gpu(value_pages, "value_pages", qkv.dtype)
    if key_pages.dim() != 4 or key_pages.shape[1] != kv_heads or key_pages.shape[3] != head_dim:
        raise KernelError(f"pages must be [blocks, {kv_heads}, block_size, {head_dim}], got {tuple(key_pages.shape)}")
    num_blocks, _, block_size, _ = key_pages.shape
    if value_pages.shape != (num_blocks, kv_heads, head_dim, block_size):
        raise KernelError(f"value pages are transposed: [blocks, {kv_heads}, {head_dim}, block_size], got {tuple(value_pages.shape)}")
    if block_table.dim() != 2:
        raise KernelError("block_table must be [sequences, max_blocks]")
    _call("qk_rope", "fe_qk_norm_rope_write", _ptr(qkv), c_int(_code(qkv.dtype)), _ptr(q_weight),
          _ptr(k_weight), _ptr(inv_freq if rotary_dim else None), _ptr(positions), _ptr(token_seq),
          _ptr(block_table), c_int(block_table.stride(0)), _ptr(key_pages), _ptr(value_pages),
          c_int(tokens), c_int(q_heads), c_int(kv_heads if write_kv else 0), c_int(head_dim), c_int(rotary_dim),
          c_int(block_size), c_int(num_blocks), c_float(eps), c_int(1 if write_kv else 0), _stream())


DECODE_TARGET_BLOCKS = 256     # blocks aimed at (measured: at 8 sequences x 8 kv heads four key splits beat eight)


class Workspace:
    """Device memory that kernels share between launches and that must survive them: the arrival
    counters of the decode kernel's key splits, one per (sequence, kv head), zero between launches
    (the kernel leaves them so).  Launches that share counters must not overlap, so whoever runs
    steps on a stream of its own (a ``ModelRunner``) owns a workspace of its own and makes it
    current around its launches (``use_workspace``); calls outside any take the one of their
    (device, stream).  A counter buffer is never given back while the workspace lives: a captured
    graph keeps the address it was recorded with, so a larger buffer is added beside the old one,
    never in its place."""

    def __init__(self) -> None:
        self._counters: dict = {}
        self._retired: list[Tensor] = []

    def split_counters(self, device: torch.device, count: int) -> Tensor:
        key = (device.type, device.index)
        have = self._counters.get(key)
        if have is None or have.numel() < count:
            if have is not None:
                self._retired.append(have)      # launches already recorded keep using it
            have = torch.zeros(max(count, 4096, 2 * (have.numel() if have is not None else 0)),
                               dtype=torch.int32, device=device)
            self._counters[key] = have
        return have


_WORKSPACES = threading.local()
_STREAM_WORKSPACES: dict = {}


class use_workspace:
    """Make ``workspace`` the one that this thread's kernel calls draw from."""

    def __init__(self, workspace: Workspace) -> None:
        self.workspace = workspace

    def __enter__(self) -> Workspace:
        self.before = getattr(_WORKSPACES, "current", None)
        _WORKSPACES.current = self.workspace
        return self.workspace

    def __exit__(self, *exc) -> None:
        _WORKSPACES.current = self.before


def _split_counters(device, count: int) -> Tensor:
    current = getattr(_WORKSPACES, "current", None)
    if current is None:
        stream = torch._C._cuda_getCurrentRawStream(device.index if device.index is not None else torch.cuda.current_device()) \
            if device.type == "cuda" else 0
        current = _STREAM_WORKSPACES.setdefault((device.type, device.index, stream), Workspace())
    return current.split_counters(device, count)


def decode_splits(num_decode: int, kv_heads: int, max_ctx: int) -> int:
    """Key splits per (sequence, kv head) for the decode kernel: enough blocks to
    fill the chip, at least four 32-key blocks of work (one per wave) in each."""
    want = -(-DECODE_TARGET_BLOCKS // max(1, num_decode * kv_heads))
    most = max(1, -(-max_ctx // 32) // 4)
    return max(1, min(want, most, 64))


PREFILL_KEY_GROUPS = 0         # 0: the prefill attention launch chooses its blocks' key groups (1 or 2 force them)
PREFILL_ROW_SETS = 0           # 0: ... and how many sets of 16 query rows a wave takes (1 or 2 force them)
GENERIC_TARGET_BLOCKS = 512    # blocks the general attention kernel aims at before it stops cutting the keys into runs


def generic_splits(num_seqs: int, kv_heads: int, groups: int, max_q_len: int, head_dim: int, max_ctx: int | None) -> int:
    """Runs that the general attention kernel cuts every row's keys into: 1 when the step already
    fills the chip or the context is not known, else enough for about GENERIC_TARGET_BLOCKS
    blocks, each with at least four of the kernel's key tiles."""
    if max_ctx is None:
        return 1
    blocks = -(-max(1, max_q_len) * groups // 16) * kv_heads * num_seqs
    key_tile = 64 if head_dim <= 64 else (32 if head_dim <= 128 else 16)
    return max(1, min(-(-GENERIC_TARGET_BLOCKS // blocks), max_ctx // (4 * key_tile), 64))


ROWS_TARGET_BLOCKS = 1024      # blocks the vector-ALU decode attention aims at (four resident a CU)


def rows_splits(num_decode: int, kv_heads: int, groups: int, head_dim: int, max_ctx: int | None) -> int:
    """Runs that the vector-ALU decode attention cuts every sequence's keys into: enough for about
    ROWS_TARGET_BLOCKS blocks, each with at least two of the kernel's key tiles."""
    if max_ctx is None:
        return 1
    blocks = -(-groups // (4 if groups <= 4 else 8)) * kv_heads * max(1, num_decode)
    key_tile = 64 if head_dim <= 64 else (32 if head_dim <= 128 else 16)
    return max(1, min(-(-ROWS_TARGET_BLOCKS // blocks), max_ctx // (2 * key_tile), 64))


def paged_attention(q: Tensor, key_pages: Tensor, value_pages: Tensor, out: Tensor, cu_q: Tensor,
                    ctx_len: Tensor, block_table: Tensor, *, num_seqs: int, max_q_len: int,
                    q_heads: int, kv_heads: int, head_dim: int, scale: float,
                    window: int | None = None, num_decode: int | None = None,
                    max_ctx: int | None = None, splits: int | None = None, chunk: int | None = None,
                    sink: Tensor | None = None, softcap: float | None = None, slopes: Tensor | None = None,
                    dist_bias: Tensor | None = None) -> Tensor:
    """Attention of every query token of a mixed batch over its paged keys.

    ``chunk`` (a token reads keys of its own run of that many positions only), ``sink``
    (float32 [Hq]: exp(sink_h) joins head h's softmax denominator), ``softcap`` (scores, after
    the scale, become cap * tanh(score / cap)) and ``slopes`` (float32 [Hq]: head h's score of key j
    loses slopes[h] * (position - j); not together with a cap) are served by the two
    matrix-core kernels alone: a call that brings either for sizes those do not take is refused
    (``masked_attention`` routes such sizes to the vector-ALU kernel that knows both).

    q: [T, >= Hq*D] (row stride may exceed Hq*D: the q part of a fused qkv
    buffer); out [T, Hq*D]; cu_q int32 [B+1]; ctx_len int32 [B] (keys after the
    step, the step's own included); block_table int32 [B, max_blocks].
    ``num_decode`` (how many sequences bring exactly one token) and ``max_ctx``
    are host-side hints: with them, single-token sequences of a bfloat16 cache
    go to the streaming decode kernel and the others to the general kernel.
    """
    _gpu(q, "q", contiguous=False)
    _gpu(out, "out", q.dtype)
    _gpu(key_pages, "key_pages", q.dtype)
    _gpu(value_pages, "value_pages", q.dtype)
    _gpu(cu_q, "cu_q", torch.int32)
    _gpu(ctx_len, "ctx_len", torch.int32)
    _gpu(block_table, "block_table", torch.int32)
    tokens = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < q_heads * head_dim:
        raise KernelError(f"q must be [T, >= {q_heads * head_dim}] with unit inner stride")
    if out.shape != (tokens, q_heads * head_dim):
        raise KernelError(f"out must be [{tokens}, {q_heads * head_dim}], got {tuple(out.shape)}")
    if q_heads % kv_heads:
        raise KernelError("query heads must be a multiple of kv heads")
    if head_dim % 2 or not 2 <= head_dim <= 256:
        raise KernelError(f"head size {head_dim} is not an even number in [2, 256]")
    if key_pages.dim() != 4 or key_pages.shape[1] != kv_heads or key_pages.shape[3] != head_dim:
        raise KernelError(f"pages must be [blocks, {kv_heads}, block_size, {head_dim}], got {tuple(key_pages.shape)}")
    if value_pages.shape != (key_pages.shape[0], kv_heads, head_dim, key_pages.shape[2]):
        raise KernelError(f"value pages are transposed: [blocks, {kv_heads}, {head_dim}, block_size], got {tuple(value_pages.shape)}")
    if cu_q.numel() != num_seqs + 1 or ctx_len.numel() != num_seqs or block_table.shape[0] < num_seqs:
        raise KernelError("cu_q, ctx_len and block_table do not match the number of sequences")
    if block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("block_table must be [sequences, max_blocks] with unit inner stride")
    num_blocks, _, block_size, _ = key_pages.shape
    groups = q_heads // kv_heads
    q_stride = q.stride(0) if tokens > 1 else q.shape[1]
    if num_decode is None:   # unknown: single-token sequences may sit beside longer ones
        any_single, any_longer, num_decode = True, max_q_len > 1, num_seqs
    else:
        any_single, any_longer = num_decode > 0, num_decode < num_seqs
    bf16_pages = (q.dtype == torch.bfloat16 and block_size >= 16 and block_size & (block_size - 1) == 0
                  and q.data_ptr() % 16 == 0 and q_stride % 8 == 0)      # the fast kernels read 16 bytes at a time
    fast_decode = bf16_pages and head_dim in (64, 128, 256) and groups <= 8
    fast_prefill = bf16_pages and head_dim in (64, 128)
    masked = chunk is not None or sink is not None or softcap is not None or slopes is not None or dist_bias is not None
    if masked:
        if dist_bias is not None:     # a table of biases by distance, float32 [Hq, span]: entry min(position - j, span - 1) joins the score
            _gpu(dist_bias, "dist_bias", torch.float32)
            if dist_bias.dim() != 2 or dist_bias.shape[0] != q_heads or dist_bias.shape[1] < 1 or slopes is not None or softcap is not None \
                    or not scale > 0.0:
                raise KernelError(f"dist_bias must be [{q_heads}, span], with a positive scale and without slopes or a soft cap")
        if slopes is not None:
            _gpu(slopes, "slopes", torch.float32)
            if slopes.shape != (q_heads,) or softcap is not None or not scale > 0.0:
                raise KernelError(f"slopes must be [{q_heads}], with a positive scale and without a soft cap")
        if (any_single and not fast_decode) or (any_longer and not fast_prefill):
            raise KernelError("chunks, sinks and soft caps are served by the matrix-core attention kernels only")
        if softcap is not None and not (softcap > 0.0 and scale > 0.0):
            raise KernelError("softcap and scale must be positive")
        if sink is not None:
            _gpu(sink, "sink", torch.float32)
            if sink.shape != (q_heads,):
                raise KernelError(f"sink must be [{q_heads}]")
        if chunk is not None and chunk < 1:
            raise KernelError("chunk must be positive")

    def general(min_q: int, max_q: int) -> None:
        runs = generic_splits(num_seqs, kv_heads, groups, min(max_q, max_q_len), head_dim, max_ctx)
        part_acc = part_ml = None
        if runs > 1:
            part_acc = torch.empty((runs, tokens, q_heads * head_dim), dtype=torch.float32, device=q.device)
            part_ml = torch.empty((runs, tokens, q_heads, 2), dtype=torch.float32, device=q.device)
        _call("attention_generic", "fe_paged_attention_generic", _ptr(q), c_longlong(q_stride),
              _ptr(key_pages), _ptr(value_pages), _ptr(out), c_longlong(out.stride(0)),
              c_int(_code(q.dtype)), _ptr(cu_q), _ptr(ctx_len), _ptr(block_table),
              c_int(block_table.stride(0)), c_int(num_seqs), c_int(max_q_len), c_int(kv_heads),
              c_int(groups), c_int(head_dim), c_int(block_size), c_int(num_blocks),
              c_int(window or 0), c_float(scale), c_int(min_q), c_int(max_q), c_int(runs), _ptr(part_acc),
              _ptr(part_ml), c_int(tokens), _stream())

    if any_single and fast_decode:
        if splits is None:
            reach = max_ctx if max_ctx is not None else 16 * 4 * 8
            splits = decode_splits(num_decode, kv_heads, reach if chunk is None else min(reach, chunk))
        part_o = part_ml = counters = None
        if splits > 1:
            part_o = torch.empty(num_seqs * kv_heads * splits * groups * head_dim, dtype=torch.float32, device=q.device)
            part_ml = torch.empty(num_seqs * kv_heads * splits * groups * 2, dtype=torch.float32, device=q.device)
            counters = _split_counters(q.device, num_seqs * kv_heads)
        mask = (c_int(chunk or 0), _ptr(sink)) + ((_ptr(slopes),) if slopes is not None else ()) if masked else ()
        if dist_bias is not None:
            mask = (c_int(chunk or 0), _ptr(sink), _ptr(dist_bias), c_int(dist_bias.shape[1]))
        cap = (c_float(softcap),) if softcap is not None else ()
        name = ("fe_paged_attention_decode_biased" if dist_bias is not None else "fe_paged_attention_decode_sloped" if slopes is not None else "fe_paged_attention_decode_capped" if cap
                else "fe_paged_attention_decode_masked" if masked else "fe_paged_attention_decode")
        _call("attention_decode", name, _ptr(q), c_longlong(q_stride),
              _ptr(key_pages), _ptr(value_pages), _ptr(out), c_longlong(out.stride(0)), _ptr(part_o),
              _ptr(part_ml), _ptr(counters), _ptr(cu_q), _ptr(ctx_len), _ptr(block_table), c_int(block_table.stride(0)),
              c_int(num_seqs), c_int(kv_heads), c_int(groups), c_int(head_dim), c_int(block_size),
              c_int(num_blocks), c_int(window or 0), *mask, c_float(scale), *cap, c_int(splits), _stream())
    if any_longer and fast_prefill:
        mask = (c_int(chunk or 0), _ptr(sink)) + ((_ptr(slopes),) if slopes is not None else ()) if masked else ()
        if dist_bias is not None:
            mask = (c_int(chunk or 0), _ptr(sink), _ptr(dist_bias), c_int(dist_bias.shape[1]))
        cap = (c_float(softcap),) if softcap is not None else ()
        name = ("fe_paged_attention_prefill_biased" if dist_bias is not None else "fe_paged_attention_prefill_sloped" if slopes is not None else "fe_paged_attention_prefill_capped" if cap
                else "fe_paged_attention_prefill_masked" if masked else "fe_paged_attention_prefill")
        _call("attention_prefill", name, _ptr(q), c_longlong(q_stride),
              _ptr(key_pages), _ptr(value_pages), _ptr(out), c_longlong(out.stride(0)), _ptr(cu_q),
              _ptr(ctx_len), _ptr(block_table), c_int(block_table.stride(0)), c_int(num_seqs),
              c_int(max_q_len), c_int(kv_heads), c_int(groups), c_int(head_dim), c_int(block_size),
              c_int(num_blocks), c_int(window or 0), *mask, c_float(scale), *cap, c_int(PREFILL_KEY_GROUPS), c_int(PREFILL_ROW_SETS),
              c_int(tokens), _stream())
    # whatever the two fast kernels did not take: single tokens go to the vector-ALU decode kernel where
    # it can read four elements at a time, the rest to the general kernel
    single_left = any_single and not fast_decode
    longer_left = any_longer and not fast_prefill
    item = q.element_size()
    if (single_left and head_dim % 4 == 0 and block_size % 4 == 0 and q_stride % 4 == 0
            and q.data_ptr() % (4 * item) == 0 and key_pages.data_ptr() % (4 * item) == 0
            and value_pages.data_ptr() % (4 * item) == 0):
        runs = rows_splits(num_decode, kv_heads, groups, head_dim, max_ctx)
        part_acc = part_ml = None
        if runs > 1:
            part_acc = torch.empty((runs, tokens, q_heads * head_dim), dtype=torch.float32, device=q.device)
            part_ml = torch.empty((runs, tokens, q_heads, 2), dtype=torch.float32, device=q.device)
        _call("attention_generic", "fe_paged_attention_rows", _ptr(q), c_longlong(q_stride),
              _ptr(key_pages), _ptr(value_pages), _ptr(out), c_longlong(out.stride(0)),
              c_int(_code(q.dtype)), _ptr(cu_q), _ptr(ctx_len), _ptr(block_table),
              c_int(block_table.stride(0)), c_int(num_seqs), c_int(kv_heads), c_int(groups), c_int(head_dim),
              c_int(block_size), c_int(num_blocks), c_int(window or 0), c_float(scale), c_int(runs),
              _ptr(part_acc), _ptr(part_ml), c_int(tokens), _stream())
        single_left = False
    if single_left or longer_left:
        general(1 if single_left else 2, max_q_len if longer_left else 1)
    return out


def decode_prepare_supported(dtype, *, q_heads: int, kv_heads: int, head_dim: int, rotary_dim: int,
                             block_size: int) -> bool:
    """Whether ``decode_attention_prepare`` serves these sizes: a bfloat16 cache, heads of 64,
    128 or 256 elements rotated whole, at most eight query heads per kv head."""
    return (dtype == torch.bfloat16 and head_dim in (64, 128, 256) and rotary_dim == head_dim
            and q_heads % kv_heads == 0 and q_heads // kv_heads <= 8
            and block_size >= 16 and block_size & (block_size - 1) == 0)


def decode_attention_prepare(qkv: Tensor, q_weight: Tensor | None, k_weight: Tensor | None, inv_freq: Tensor,
                             key_pages: Tensor, value_pages: Tensor, out: Tensor, cu_q: Tensor, ctx_len: Tensor,
                             block_table: Tensor, *, q_heads: int, kv_heads: int, head_dim: int, eps: float,
                             scale: float, window: int | None = None, max_ctx: int | None = None,
                             splits: int | None = None) -> Tensor:
    """A step of single tokens only, from the fused projection's output to the attention's
    output in one launch: what ``qk_norm_rope_write`` followed by ``paged_attention`` does for
    such a batch (same bits in the cache; qkv is left as it is).

    qkv [B, (Hq + 2 Hkv) D] bfloat16, one row per sequence, or float32 [parts <= 4, B, ...]:
    partial sums of the projection (``linear_in_parts``), added up in order and rounded to
    bfloat16 inside the kernel.  ctx_len counts the new token, whose position is ctx_len - 1."""
    width = (q_heads + 2 * kv_heads) * head_dim
    if isinstance(qkv, Tensor) and qkv.dtype == torch.float32:
        _gpu(qkv, "qkv", torch.float32)
        if qkv.dim() != 3 or not 1 <= qkv.shape[0] <= 4 or qkv.shape[2] != width:
            raise KernelError(f"qkv in parts must be [parts <= 4, B, {width}], got {tuple(qkv.shape)}")
        sums, num_seqs = qkv.shape[0], qkv.shape[1]
    else:
        _gpu(qkv, "qkv", torch.bfloat16)
        if qkv.dim() != 2 or qkv.shape[1] != width:
            raise KernelError(f"qkv must be [B, {width}], got {tuple(qkv.shape)}")
        sums, num_seqs = 0, qkv.shape[0]
    _gpu(key_pages, "key_pages", torch.bfloat16)
    _gpu(value_pages, "value_pages", torch.bfloat16)
    if key_pages.dim() != 4 or key_pages.shape[1] != kv_heads or key_pages.shape[3] != head_dim:
        raise KernelError(f"pages must be [blocks, {kv_heads}, block_size, {head_dim}], got {tuple(key_pages.shape)}")
    num_blocks, _, block_size, _ = key_pages.shape
    if value_pages.shape != (num_blocks, kv_heads, head_dim, block_size):
        raise KernelError(f"value pages are transposed: [blocks, {kv_heads}, {head_dim}, block_size], got {tuple(value_pages.shape)}")
    if not decode_prepare_supported(key_pages.dtype, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
                                    rotary_dim=2 * inv_freq.numel() if inv_freq is not None else 0,
                                    block_size=block_size):
        raise KernelError("these sizes are not served by the fused decode kernel: heads of 64, 128 or 256 "
                          "elements rotated whole, at most 8 query heads per kv head, pages of a power of two >= 16")
    if (q_weight is None) != (k_weight is None):
        raise KernelError("q and k are normalised both or neither")
    for name, w in (("q_weight", q_weight), ("k_weight", k_weight)):
        if w is not None:
            _gpu(w, name, torch.float32)
            if w.shape != (head_dim,):
                raise KernelError(f"{name} must be [{head_dim}]")
    _gpu(inv_freq, "inv_freq", torch.float32)
    _gpu(out, "out", torch.bfloat16)
    if out.shape != (num_seqs, q_heads * head_dim):
        raise KernelError(f"out must be [{num_seqs}, {q_heads * head_dim}], got {tuple(out.shape)}")
    _gpu(cu_q, "cu_q", torch.int32)
    _gpu(ctx_len, "ctx_len", torch.int32)
    _gpu(block_table, "block_table", torch.int32)
    if cu_q.numel() != num_seqs + 1 or ctx_len.numel() != num_seqs or block_table.shape[0] < num_seqs:
        raise KernelError("cu_q, ctx_len and block_table do not match the number of sequences")
    if block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("block_table must be [sequences, max_blocks] with unit inner stride")
    groups = q_heads // kv_heads
    if splits is None:
        splits = decode_splits(num_seqs, kv_heads, max_ctx if max_ctx is not None else 16 * 4 * 8)
    part_o = part_ml = counters = None
    if splits > 1:
        part_o = torch.empty(num_seqs * kv_heads * splits * groups * head_dim, dtype=torch.float32, device=qkv.device)
        part_ml = torch.empty(num_seqs * kv_heads * splits * groups * 2, dtype=torch.float32, device=qkv.device)
        counters = _split_counters(qkv.device, num_seqs * kv_heads)
    _call("attention_decode", "fe_paged_attention_decode_prepare", _ptr(qkv), c_int(sums),
          c_longlong(num_seqs * width), c_longlong(width), _ptr(q_weight),
          _ptr(k_weight), _ptr(inv_freq), c_float(eps), _ptr(key_pages), _ptr(value_pages), _ptr(out),
          c_longlong(out.stride(0)), _ptr(part_o), _ptr(part_ml), _ptr(counters), _ptr(cu_q), _ptr(ctx_len),
          _ptr(block_table), c_int(block_table.stride(0)), c_int(num_seqs), c_int(kv_heads), c_int(groups),
          c_int(head_dim), c_int(block_size), c_int(num_blocks), c_int(window or 0), c_float(scale),
          c_int(splits), _stream())
    return out


# ------------------------------------------------------------------- sampling

def argmax_rows(logits: Tensor, tokens: Tensor, status: Tensor) -> None:
    """tokens[r] = argmax(logits[r]) (lowest index on ties); status bits: 1 NaN, 2 +inf, 4 no finite entry."""
    _gpu(logits, "logits", torch.float32)
    _gpu(tokens, "tokens", torch.int32)
    _gpu(status, "status", torch.int32)
    rows, vocab = logits.shape
    if tokens.numel() != rows or status.numel() != rows:
        raise KernelError("tokens and status need one entry per row")
    scratch = torch.empty(rows * 32 * 3, dtype=torch.int32, device=logits.device)
    _call("sample", "fe_argmax_rows", _ptr(logits), c_longlong(logits.stride(0)), c_int(rows),
          c_int(vocab), _ptr(tokens), _ptr(status), _ptr(scratch), _stream())


ARGMAX_STATIC_MAX_ROWS = 1024   # FE_ARGMAX_STATIC_MAX_ROWS of csrc/sample_api.h


def argmax_rows_static(logits: Tensor, tokens: Tensor, status: Tensor) -> None:
    """``argmax_rows`` without any allocation: the partial maxima live in an array inside the
    library's device image, shared by every call on the GPU (calls that overlap there race;
    calls on one stream do not).  At most ``ARGMAX_STATIC_MAX_ROWS`` rows."""
    _gpu(logits, "logits", torch.float32)
    _gpu(tokens, "tokens", torch.int32)
    _gpu(status, "status", torch.int32)
    rows, vocab = logits.shape
    if tokens.numel() != rows or status.numel() != rows:
        raise KernelError("tokens and status need one entry per row")
    if rows > ARGMAX_STATIC_MAX_ROWS:
        raise KernelError(f"the arg-max without allocation takes at most {ARGMAX_STATIC_MAX_ROWS} rows, got {rows}")
    _call("sample", "fe_argmax_rows_static", _ptr(logits), c_longlong(logits.stride(0)), c_int(rows),
          c_int(vocab), _ptr(tokens), _ptr(status), _stream())


SAMPLE_PARAM_WORDS = 8      # per row: temperature, top_k, top_p, min_p (four-byte words), seed, draw index (eight bytes each)


def pack_sample_params(rows) -> Tensor:
    """int32 [rows, SAMPLE_PARAM_WORDS] on the host for ``sample_filtered_rows`` from tuples
    (temperature, top_k or None, top_p, min_p, seed, draw index); temperature 0 asks for the arg-max."""
    packed = np.zeros(len(rows), dtype=_SAMPLE_PARAMS)
    for i, (temperature, top_k, top_p, min_p, seed, draw) in enumerate(rows):
        packed[i] = (temperature, min(top_k or 0, 2**31 - 1), top_p, min_p, seed & (2**64 - 1), draw & (2**64 - 1))
    return torch.from_numpy(packed.view(np.int32).reshape(len(rows), SAMPLE_PARAM_WORDS))


SAMPLE_MAX_SPLIT = 32                # most slices of a row, a block each
SAMPLE_SCRATCH_BYTES_PER_ROW = 76800
SAMPLE_TARGET_BLOCKS = 1024          # slices of all rows together: four blocks of 256 threads a CU


def sample_filtered_rows(logits: Tensor, params: Tensor, tokens: Tensor, status: Tensor,
                         any_top_k: bool = True, any_top_p: bool = True) -> None:
    """tokens[r]: the arg-max of logits[r], or a draw from softmax(logits[r] / temperature) after
    top-k, top-p and min-p (in the order of the reference, src/forge_engine/sampling.py:83-140) with
    the uniform philox(counter=draw index, key=seed); ``params`` as ``pack_sample_params`` lays
    them out, on the device.  status[r]: bit 0 NaN, bit 1 +inf, bit 2 no finite entry.
    ``any_top_k`` / ``any_top_p``: whether any row limits by top-k / top-p (each search is up to
    four launches that rows without it sit out; saying no where a row does ask leaves that row
    unfinished, which raises)."""
    _gpu(logits, "logits", torch.float32, contiguous=False)
    _gpu(params, "params", torch.int32)
    _gpu(tokens, "tokens", torch.int32)
    _gpu(status, "status", torch.int32)
    rows, vocab = logits.shape
    if logits.stride(1) != 1 or logits.stride(0) < vocab:
        raise KernelError("logits rows must be contiguous")
    if params.shape != (rows, SAMPLE_PARAM_WORDS) or params.data_ptr() % 8:
        raise KernelError(f"params must be int32 [rows, {SAMPLE_PARAM_WORDS}], 8-byte aligned")
    if tokens.numel() != rows or status.numel() != rows:
        raise KernelError("tokens and status need one entry per row")
    if rows == 0:
        return
    # slices of at least 4,096 entries, about SAMPLE_TARGET_BLOCKS blocks in all
    split = max(1, min(SAMPLE_MAX_SPLIT, -(-SAMPLE_TARGET_BLOCKS // rows), vocab // 4096))
    scratch = torch.empty(rows * SAMPLE_SCRATCH_BYTES_PER_ROW, dtype=torch.uint8, device=logits.device)
    launches = 3 + (4 if any_top_k else 0) + (4 if any_top_p else 0)
    _call("sample", "fe_sample_filtered_rows", _ptr(logits), c_longlong(logits.stride(0)), c_int(rows),
          c_int(vocab), _ptr(params), _ptr(tokens), _ptr(status), _ptr(scratch), c_int(split), c_int(launches),
          _stream())


LIBRARIES = ("rowwise", "gemm_f32", "gemm_skinny", "gemm_mid", "gemm_wide", "gemm_tile", "qk_rope", "attention_generic", "attention_decode", "attention_prefill", "sample")


# ------------------------------------------------- ops on the stream, beside the matrix products

def cast_rows(h: Tensor, dtype) -> Tensor:
    """The stream in the compute dtype (itself when that is float32)."""
    _gpu(h, "h")
    return h if h.dtype == dtype else h.to(dtype)


def _sequences(cu_q: Tensor, state_slots: Tensor, num_seqs: int) -> None:
    _gpu(cu_q, "cu_q", torch.int32)
    _gpu(state_slots, "state_slots", torch.int32)
    if num_seqs < 1 or cu_q.numel() != num_seqs + 1 or state_slots.numel() != num_seqs:
        raise KernelError("cu_q and state_slots do not match the number of sequences")


def _parts_of(update: Tensor, rows: int, width: int, name: str) -> int:
    _gpu(update, name, torch.float32)
    if update.shape == (rows, width):
        return 1
    if update.dim() == 3 and update.shape[1:] == (rows, width) and 1 <= update.shape[0] <= 64:
        return update.shape[0]
    raise KernelError(f"{name} must be [{rows}, {width}] or [parts <= 64, {rows}, {width}], got {tuple(update.shape)}")


def token_shift(x: Tensor, weights: Tensor, state: Tensor, cu_q: Tensor, token_seq: Tensor, state_slots: Tensor, *,
                num_seqs: int, out_dtype) -> Tensor:
    """out[s, t] = x[t] + (x'[t] - x[t]) * weights[s]: x' is the row before within the token's
    sequence, and for a sequence's first token of the step the row that ``state`` keeps for its slot
    (zeros for a request's first token); afterwards ``state`` holds every sequence's last row.
    x [T, W] float32 or bfloat16, weights float32 [n, W], state float32 [slots, W]; out [n, T, W]."""
    _gpu(x, "x")
    _gpu(weights, "weights", torch.float32)
    _gpu(state, "state", torch.float32)
    _gpu(token_seq, "token_seq", torch.int32)
    _sequences(cu_q, state_slots, num_seqs)
    tokens, width = x.shape
    if weights.dim() != 2 or weights.shape[1] != width or not 1 <= weights.shape[0] <= 8:
        raise KernelError(f"weights must be [1..8, {width}], got {tuple(weights.shape)}")
    if state.dim() != 2 or state.shape[1] != width or token_seq.numel() != tokens:
        raise KernelError("state must be [slots, width] and token_seq hold one entry per token")
    out = torch.empty((weights.shape[0], tokens, width), dtype=out_dtype, device=x.device)
    _call("stream_ops", "fe_token_shift", _ptr(x), c_int(_code(x.dtype)), _ptr(weights), _ptr(state), _ptr(cu_q),
          _ptr(token_seq), _ptr(state_slots), _ptr(out), c_int(_code(out.dtype)), c_int(tokens), c_int(width),
          c_int(weights.shape[0]), c_int(state.shape[0]), _stream())
    _call("stream_ops", "fe_save_last_rows", _ptr(x), c_int(_code(x.dtype)), _ptr(state), _ptr(cu_q), _ptr(state_slots),
          c_int(num_seqs), c_int(width), c_int(state.shape[0]), c_int(tokens), _stream())
    return out


def rmsnorm_update(h: Tensor, update: Tensor, weight: Tensor, eps: float, out: Tensor | None = None) -> Tensor | None:
    """h += u * rsqrt(mean(u^2) + eps) * weight, u the update (float32, [parts, T, W] added up in
    order first); all float32.  ``out`` (compute dtype [T, W]) receives the new h as well."""
    _gpu(h, "h", torch.float32)
    _gpu(weight, "weight", torch.float32)
    rows, width = h.shape
    parts = _parts_of(update, rows, width, "update")
    if weight.shape != (width,):
        raise KernelError(f"weight must be [{width}]")
    if out is not None:
        _gpu(out, "out")
        if out.shape != h.shape:
            raise KernelError("out must have the stream's shape")
    if not eps > 0.0:
        raise KernelError("eps must be positive")
    _call("stream_ops", "fe_rmsnorm_update", _ptr(h), _ptr(update), c_int(parts), c_longlong(h.numel()), _ptr(weight),
          c_float(eps), _ptr(out), c_int(_code(out.dtype) if out is not None else -1), c_int(rows), c_int(width), _stream())
    return out


def layernorm_update(h: Tensor, update: Tensor, weight: Tensor, eps: float, factor: float = 1.0,
                     out: Tensor | None = None) -> Tensor | None:
    """h += factor * (u - mean(u)) * rsqrt(var(u) + eps) * weight, u the update (float32, [parts, T, W] added up
    in order first), var the mean of the squared deviations; all float32.  ``out`` (compute dtype [T, W])
    receives the new h as well."""
    _gpu(h, "h", torch.float32)
    _gpu(weight, "weight", torch.float32)
    rows, width = h.shape
    parts = _parts_of(update, rows, width, "update")
    if weight.shape != (width,):
        raise KernelError(f"weight must be [{width}]")
    if out is not None:
        _gpu(out, "out")
        if out.shape != h.shape:
            raise KernelError("out must have the stream's shape")
    if not eps > 0.0:
        raise KernelError("eps must be positive")
    _call("stream_ops", "fe_layernorm_update", _ptr(h), _ptr(update), c_int(parts), c_longlong(h.numel()), _ptr(weight),
          c_float(eps), c_float(factor), _ptr(out), c_int(_code(out.dtype) if out is not None else -1), c_int(rows),
          c_int(width), _stream())
    return out


FUSED_NORMS_MAX_WIDTH = 8192       # 8 elements a thread at 1,024 threads a row


def rmsnorm_update_norm(h: Tensor, update: Tensor, weight: Tensor, eps: float, next_weight: Tensor, next_eps: float, out: Tensor,
                        rows: Tensor | None = None) -> Tensor:
    """A norm behind a sublayer and the norm before the next one: ``v = h[s] + u * rsqrt(mean(u^2) + eps) * weight``
    (u the update, float32, [parts, T, W] added up in order first), ``out[r] = v * rsqrt(mean(v^2) + next_eps) *
    next_weight``, s = rows[r] or r; all float32 with one rounding at the store.  Without ``rows`` v is written back to
    h; with them h stays as it is.  One kernel for rows up to FUSED_NORMS_MAX_WIDTH wide, two otherwise."""
    _gpu(h, "h", torch.float32)
    _gpu(weight, "weight", torch.float32)
    _gpu(next_weight, "next_weight", torch.float32)
    _gpu(out, "out")
    total, width = h.shape
    parts = _parts_of(update, total, width, "update")
    count = total
    if rows is not None:
        _gpu(rows, "rows", torch.int32)
        count = rows.numel()
    if weight.shape != (width,) or next_weight.shape != (width,) or out.shape != (count, width):
        raise KernelError(f"weights must be [{width}] and out [{count}, {width}]")
    if not (eps > 0.0 and next_eps > 0.0):
        raise KernelError("eps must be positive")
    if width > FUSED_NORMS_MAX_WIDTH:
        if rows is not None:      # the chosen rows alone, and the stream stays as it is: on a copy of those rows
            picked = h.index_select(0, rows.long())
            chosen = update.index_select(update.dim() - 2, rows.long())
            rmsnorm_update(picked, chosen, weight, eps, None)
            return add_rmsnorm(picked, None, next_weight, next_eps, out)
        rmsnorm_update(h, update, weight, eps, None)
        return add_rmsnorm(h, None, next_weight, next_eps, out)
    _call("stream_ops", "fe_rmsnorm_update_norm", _ptr(h), _ptr(update), c_int(parts), c_longlong(h.numel()), _ptr(weight),
          c_float(eps), _ptr(next_weight), c_float(next_eps), _ptr(out), c_int(_code(out.dtype)), _ptr(rows),
          c_int(0 if rows is not None else 1), c_int(count), c_int(width), _stream())
    return out


def rmsnorm_mean(updates, weights: Tensor, eps: float, out: Tensor) -> Tensor:
    """out = mean over b of u_b * rsqrt(mean(u_b^2) + eps) * weights[b]; float32 (an update may
    come as [parts, T, W])."""
    _gpu(out, "out", torch.float32)
    _gpu(weights, "weights", torch.float32)
    rows, width = out.shape
    count = len(updates)
    if not 1 <= count <= 4 or weights.shape != (count, width):
        raise KernelError(f"one to four updates with weights [{count}, {width}]")
    parts = [_parts_of(u, rows, width, f"update {i}") for i, u in enumerate(updates)]
    pointers = [_ptr(updates[i]) if i < count else _ptr(None) for i in range(4)]
    counts = [c_int(parts[i] if i < count else 0) for i in range(4)]
    _call("stream_ops", "fe_rmsnorm_mean", *pointers, *counts, c_int(count), c_longlong(out.numel()), _ptr(weights),
          c_float(eps), _ptr(out), c_int(rows), c_int(width), _stream())
    return out


def polynorm(z: Tensor, coefficients: Tensor, eps: float, out: Tensor) -> Tensor:
    """out = a N(z) + b N(z^2) + c N(z^3) + e, N(y) = y * rsqrt(mean(y^2) + eps) over a row; the
    four numbers float32 on the device; float32 inside."""
    _gpu(z, "z")
    _gpu(out, "out", z.dtype)
    _gpu(coefficients, "coefficients", torch.float32)
    if z.dim() != 2 or out.shape != z.shape or coefficients.numel() != 4:
        raise KernelError("z and out must be [T, F] and the coefficients four numbers")
    _call("stream_ops", "fe_polynorm", _ptr(z), c_int(_code(z.dtype)), _ptr(coefficients), c_float(eps), _ptr(out),
          c_int(z.shape[0]), c_int(z.shape[1]), _stream())
    return out


def add_bias(update: Tensor, bias: Tensor) -> Tensor:
    """update += bias along the rows, for a float32 update [T, W]; of an update in parts
    [parts, T, W] the first part takes it (the parts are added up by whoever reads them)."""
    _gpu(update, "update", torch.float32)
    _gpu(bias, "bias", torch.float32)
    if update.dim() not in (2, 3) or bias.shape != (update.shape[-1],):
        raise KernelError(f"update must be [T, W] or [parts, T, W] and bias [W], got {tuple(update.shape)} and {tuple(bias.shape)}")
    _call("stream_ops", "fe_add_bias", _ptr(update), _ptr(bias), c_int(update.shape[-2]), c_int(update.shape[-1]), _stream())
    return update


def tanh_rows(x: Tensor) -> Tensor:
    """tanh of every element, in place (float32 inside)."""
    _gpu(x, "x")
    _call("stream_ops", "fe_tanh_rows", _ptr(x), c_int(_code(x.dtype)), c_longlong(x.numel()), _stream())
    return x


_ACTS = {"none": 0, "silu": 1, "sigmoid": 2}


def _strided_rows(t: Tensor, name: str, width: int) -> int:
    _gpu(t, name, contiguous=False)
    if t.dim() != 2 or t.shape[1] != width or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{name} must be [T, {width}] with unit inner stride, got {tuple(t.shape)}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), width)


def head_norm_gate(o: Tensor, weight: Tensor | None, gate: Tensor | None, out: Tensor, *, heads: int, dim: int,
                   eps: float, act: str = "none", extra: int = 0, floor: Tensor | None = None) -> Tensor:
    """out[t, h] = o[t, h, :dim] / rms * weight * act(gate[t, h]) per head, rms over dim (epsilon
    inside the root).  o float32 [T, heads, dim + extra]; with ``extra`` = 1 the last column is a
    normaliser n and the head is first divided by max(|n|, floor[t, h]) + 1e-6.  weight float32
    of heads * dim entries, or of dim entries shared by the heads; gate [T, heads * dim] rows of
    any stride, in the compute dtype."""
    _gpu(o, "o", torch.float32)
    _gpu(out, "out")
    tokens = o.shape[0]
    if o.shape != (tokens, heads, dim + extra) or extra not in (0, 1) or out.shape != (tokens, heads * dim):
        raise KernelError(f"o must be [T, {heads}, {dim + extra}] and out [T, {heads * dim}]")
    if act not in _ACTS:
        raise KernelError(f"unknown gate activation '{act}'")
    weight_len = 0
    if weight is not None:
        _gpu(weight, "weight", torch.float32)
        weight_len = weight.numel()
        if weight_len not in (dim, heads * dim):
            raise KernelError(f"weight must hold {dim} or {heads * dim} entries")
    gate_stride = 0
    if gate is not None:
        gate_stride = _strided_rows(gate, "gate", heads * dim)
        if gate.dtype != out.dtype:
            raise KernelError("gate must be in the output's dtype")
    if extra:
        _gpu(floor, "floor", torch.float32)
        if floor.shape != (tokens, heads):
            raise KernelError(f"floor must be [T, {heads}]")
    _call("stream_ops", "fe_head_norm_gate", _ptr(o), _ptr(weight), c_int(weight_len), _ptr(gate), c_longlong(gate_stride),
          _ptr(out), c_int(_code(out.dtype)), _ptr(floor if extra else None), c_int(tokens), c_int(heads), c_int(dim),
          c_int(extra), c_float(eps), c_int(_ACTS[act]), _stream())
    return out


# ------------------------------------------------- short convolution, rotation, unit norm, page write

def conv_rope_norm_write(qkv: Tensor, bias: Tensor | None, conv_weight: Tensor | None, conv_state: Tensor | None, inv_freq: Tensor | None,
                         positions: Tensor, token_seq: Tensor, cu_q: Tensor, state_slots: Tensor, block_table: Tensor,
                         key_pages: Tensor, value_pages: Tensor, q_out: Tensor, *, num_seqs: int, q_heads: int,
                         kv_heads: int, head_dim: int, value_dim: int, rotary_dim: int, unit_norm_eps: float | None,
                         taps: int, v_from: Tensor | None = None, v_mix: float = 0.0, v_keep: Tensor | None = None,
                         norm_weight_q: Tensor | None = None, norm_weight_k: Tensor | None = None,
                         norm_first: bool = False) -> None:
    """From the projection's output to queries and cached keys and values in one kernel: a short
    projection's bias (float32 [channels] or None: the product before has none), a short causal
    convolution over time on every q, k and v channel (``taps`` > 0: y_t = sum_j c[:, j] *
    u_(t - taps + 1 + j), rows before the step from ``conv_state`` [slots, taps - 1, channels],
    which afterwards holds every sequence's last taps - 1 projected rows; one tap needs no state); rotation of the first
    ``rotary_dim`` dims of q and k heads (dim i pairs with i + rotary_dim / 2); then q and k heads
    divided by their root mean square (``unit_norm_eps`` not None); q into ``q_out`` [T, Hq * D],
    k and v into their pages (values transposed).  float32 inside, one rounding at the stores.
    qkv [T, >= channels] with any row stride.  ``v_from`` ([T, kv_heads * value_dim], another layer's values of
    the same tokens): the values become ``(1 - v_mix) v + v_mix v_from`` before they are stored; ``v_keep`` (same
    shape) receives the values as stored, for layers that lean on this one's.  ``norm_weight_q`` / ``norm_weight_k``
    (float32 [head_dim], shared by the heads): the unit norm's result times a weight per dim, an RMS norm;
    ``norm_first``: the norm comes before the rotation instead of behind it."""
    channels = (q_heads + kv_heads) * head_dim + kv_heads * value_dim
    for name, w in (("norm_weight_q", norm_weight_q), ("norm_weight_k", norm_weight_k)):
        if w is not None:
            _gpu(w, name, torch.float32)
            if w.shape != (head_dim,) or unit_norm_eps is None:
                raise KernelError(f"{name} must be [{head_dim}] and comes with a unit norm")
    if norm_first and unit_norm_eps is None:
        raise KernelError("norm_first comes with a unit norm")
    _gpu(qkv, "qkv", contiguous=False)
    tokens = qkv.shape[0]
    if qkv.dim() != 2 or qkv.shape[1] < channels or qkv.stride(1) != 1:
        raise KernelError(f"qkv must be [T, >= {channels}] with unit inner stride")
    _gpu(q_out, "q_out", qkv.dtype)
    if q_out.shape != (tokens, q_heads * head_dim):
        raise KernelError(f"q_out must be [{tokens}, {q_heads * head_dim}]")
    if bias is not None:
        _gpu(bias, "bias", torch.float32)
        if bias.shape != (channels,):
            raise KernelError(f"bias must be [{channels}]")
    if taps:
        _gpu(conv_weight, "conv_weight", torch.float32)
        if conv_weight.shape != (channels, taps) or not 1 <= taps <= 8:
            raise KernelError(f"conv_weight must be [{channels}, taps in 1..8]")
    if taps > 1:
        _gpu(conv_state, "conv_state", torch.float32)
        if conv_state.dim() != 3 or conv_state.shape[1:] != (taps - 1, channels):
            raise KernelError(f"conv_state must be [slots, {taps - 1}, {channels}]")
    if rotary_dim:
        _gpu(inv_freq, "inv_freq", torch.float32)
        if inv_freq.shape != (rotary_dim // 2,) or rotary_dim % 2 or rotary_dim > head_dim:
            raise KernelError(f"inv_freq must be [{rotary_dim // 2}] for an even rotary_dim <= head_dim")
    if head_dim > 256 or value_dim > 256:
        raise KernelError("head sizes up to 256")
    _gpu(positions, "positions", torch.int32)
    _gpu(token_seq, "token_seq", torch.int32)
    _sequences(cu_q, state_slots, num_seqs)
    if positions.numel() != tokens or token_seq.numel() != tokens:
        raise KernelError("positions and token_seq must have one entry per token")
    _gpu(block_table, "block_table", torch.int32)
    _gpu(key_pages, "key_pages", qkv.dtype)
    _gpu(value_pages, "value_pages", qkv.dtype)
    if key_pages.dim() != 4 or key_pages.shape[1] != kv_heads or key_pages.shape[3] != head_dim:
        raise KernelError(f"key pages must be [blocks, {kv_heads}, block_size, {head_dim}], got {tuple(key_pages.shape)}")
    num_blocks, _, block_size, _ = key_pages.shape
    if value_pages.shape != (num_blocks, kv_heads, value_dim, block_size):
        raise KernelError(f"value pages are transposed: [blocks, {kv_heads}, {value_dim}, block_size], got {tuple(value_pages.shape)}")
    if block_table.dim() != 2 or block_table.stride(1) != 1 or block_table.shape[0] < num_seqs:
        raise KernelError("block_table must be [sequences, max_blocks] with unit inner stride")
    for name, dense in (("v_from", v_from), ("v_keep", v_keep)):
        if dense is not None:
            _gpu(dense, name, qkv.dtype)
            if dense.shape != (tokens, kv_heads * value_dim):
                raise KernelError(f"{name} must be [{tokens}, {kv_heads * value_dim}], got {tuple(dense.shape)}")
    stride = qkv.stride(0) if tokens > 1 else max(qkv.stride(0), qkv.shape[1])
    slots = conv_state.shape[0] if taps > 1 else 0
    _call("conv_rope", "fe_conv_rope_norm_write", _ptr(qkv), c_int(_code(qkv.dtype)), c_longlong(stride), _ptr(bias),
          _ptr(conv_weight if taps else None), _ptr(conv_state if taps > 1 else None), _ptr(inv_freq if rotary_dim else None),
          _ptr(positions), _ptr(token_seq), _ptr(cu_q), _ptr(state_slots), _ptr(block_table), c_int(block_table.stride(0)),
          _ptr(key_pages), _ptr(value_pages), _ptr(q_out), c_int(tokens), c_int(q_heads), c_int(kv_heads), c_int(head_dim),
          c_int(value_dim), c_int(rotary_dim), c_float(unit_norm_eps if unit_norm_eps is not None else 0.0),
          c_int(1 if unit_norm_eps is not None else 0), c_int(taps), c_int(block_size), c_int(num_blocks), c_int(slots),
          _ptr(v_from), c_float(v_mix), _ptr(v_keep), _ptr(norm_weight_q), _ptr(norm_weight_k), c_int(1 if norm_first else 0),
          _stream())
    if taps > 1:
        _call("conv_rope", "fe_conv_state_update", _ptr(qkv), c_int(_code(qkv.dtype)), c_longlong(stride), _ptr(bias), _ptr(conv_state),
              _ptr(cu_q), _ptr(state_slots), c_int(num_seqs), c_int(channels), c_int(taps), c_int(slots), c_int(tokens),
              _stream())


def masked_attention(q: Tensor, key_pages: Tensor, value_pages: Tensor | None, out: Tensor, cu_q: Tensor, ctx_len: Tensor,
                     block_table: Tensor, *, num_seqs: int, max_q_len: int, q_heads: int, kv_heads: int, head_dim: int,
                     value_dim: int, scale: float, window: int | None = None, chunk: int | None = None,
                     sink: Tensor | None = None, gate: Tensor | None = None, num_decode: int | None = None,
                     max_ctx: int | None = None, softcap: float | None = None, head_gate: bool = False,
                     slopes: Tensor | None = None, dist_bias: Tensor | None = None) -> Tensor:
    """Paged grouped-query attention with the masks and softmax forms beyond the causal one: the
    query at position p reads keys j <= p with j > p - window (``window``) and j >= p - p % chunk
    (``chunk``); ``sink`` (float32 [Hq]) adds exp(sink_h) to head h's softmax denominator, with
    no key and no value; values may be of another width than keys; ``gate`` ([T, Hq * Dv] rows of
    any stride; with ``head_gate`` [T, Hq], one number a head) multiplies the result by sigmoid(gate);
    ``softcap``: scores, after the scale, become cap * tanh(score / cap); ``slopes`` (float32 [Hq]): head h's score
    of key j loses slopes[h] * (p - j); ``dist_bias`` (float32 [Hq, span]): head h's score of key j gains
    dist_bias[h, min(p - j, span - 1)] (after the scale, which does not multiply it); ``value_pages`` None: a key's
    first ``value_dim`` dims are its value (a cache of keys only).  out [T, Hq * Dv].  Scores and softmax
    float32.  A bfloat16 cache with keys and values of 64 or 128 elements, groups up to 8 and pages of
    a power of two >= 16 goes to the matrix-core kernels of ``paged_attention`` (single tokens and
    portions each to its own), with the gate in a small kernel behind them; everything else, and
    the float32 mode, to the vector-ALU kernel that does all of it in one launch."""
    _gpu(q, "q", contiguous=False)
    _gpu(out, "out", q.dtype)
    _gpu(key_pages, "key_pages", q.dtype)
    if value_pages is not None:
        _gpu(value_pages, "value_pages", q.dtype)
    _gpu(cu_q, "cu_q", torch.int32)
    _gpu(ctx_len, "ctx_len", torch.int32)
    _gpu(block_table, "block_table", torch.int32)
    tokens = q.shape[0]
    q_stride = _strided_rows(q, "q", q_heads * head_dim)
    if out.shape != (tokens, q_heads * value_dim):
        raise KernelError(f"out must be [{tokens}, {q_heads * value_dim}], got {tuple(out.shape)}")
    if q_heads % kv_heads or not 1 <= head_dim <= MASKED_MAX_KEY_DIM or not 1 <= value_dim <= MASKED_MAX_VALUE_DIM:
        raise KernelError(f"query heads must be a multiple of kv heads, keys of up to {MASKED_MAX_KEY_DIM} and values of up to {MASKED_MAX_VALUE_DIM} dims")
    if value_pages is None and value_dim > head_dim:
        raise KernelError("values that are the keys' own dims cannot be wider than the keys")
    if key_pages.dim() != 4 or key_pages.shape[1] != kv_heads or key_pages.shape[3] != head_dim:
        raise KernelError(f"key pages must be [blocks, {kv_heads}, block_size, {head_dim}], got {tuple(key_pages.shape)}")
    num_blocks, _, block_size, _ = key_pages.shape
    if value_pages is not None and value_pages.shape != (num_blocks, kv_heads, value_dim, block_size):
        raise KernelError(f"value pages are transposed: [blocks, {kv_heads}, {value_dim}, block_size]")
    if cu_q.numel() != num_seqs + 1 or ctx_len.numel() != num_seqs or block_table.shape[0] < num_seqs:
        raise KernelError("cu_q, ctx_len and block_table do not match the number of sequences")
    if block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("block_table must be [sequences, max_blocks] with unit inner stride")
    if sink is not None:
        _gpu(sink, "sink", torch.float32)
        if sink.shape != (q_heads,):
            raise KernelError(f"sink must be [{q_heads}]")
    if slopes is not None:
        _gpu(slopes, "slopes", torch.float32)
        if slopes.shape != (q_heads,):
            raise KernelError(f"slopes must be [{q_heads}]")
    span = 0
    if dist_bias is not None:
        _gpu(dist_bias, "dist_bias", torch.float32)
        if dist_bias.dim() != 2 or dist_bias.shape[0] != q_heads or dist_bias.shape[1] < 1:
            raise KernelError(f"dist_bias must be [{q_heads}, span >= 1], got {tuple(dist_bias.shape)}")
        span = dist_bias.shape[1]
    gate_stride = 0
    if gate is not None:
        gate_stride = _strided_rows(gate, "gate", q_heads if head_gate else q_heads * value_dim)
        if gate.dtype != q.dtype:
            raise KernelError("gate must be in q's dtype")
    if softcap is not None and not softcap > 0.0:
        raise KernelError("softcap must be positive")
    if (window is not None and window < 1) or (chunk is not None and chunk < 1) or max_q_len < 1:
        raise KernelError("window, chunk and max_q_len must be positive")
    if (q.dtype == torch.bfloat16 and head_dim == value_dim and head_dim in (64, 128) and q_heads // kv_heads <= 8
            and not (slopes is not None and softcap is not None) and value_pages is not None
            and not (dist_bias is not None and (slopes is not None or softcap is not None))
            and block_size >= 16 and block_size & (block_size - 1) == 0 and q.data_ptr() % 16 == 0 and q_stride % 8 == 0):
        paged_attention(q, key_pages, value_pages, out, cu_q, ctx_len, block_table, num_seqs=num_seqs, max_q_len=max_q_len,
                        q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, scale=scale, window=window,
                        num_decode=num_decode, max_ctx=max_ctx, chunk=chunk, sink=sink, softcap=softcap, slopes=slopes,
                        dist_bias=dist_bias)
        if gate is not None:
            _call("stream_ops", "fe_sigmoid_gate", _ptr(out), _ptr(gate), c_longlong(gate_stride), c_int(_code(out.dtype)),
                  c_int(tokens), c_int(q_heads * value_dim), c_int(value_dim if head_gate else 1), _stream())
        return out
    _call("attention_masked", "fe_masked_attention", _ptr(q), c_int(_code(q.dtype)), c_longlong(q_stride), _ptr(key_pages),
          _ptr(value_pages), _ptr(out), _ptr(gate), c_longlong(gate_stride), _ptr(sink), _ptr(cu_q), _ptr(ctx_len),
          _ptr(block_table), c_int(block_table.stride(0)), c_int(num_seqs), c_int(max_q_len), c_int(q_heads),
          c_int(kv_heads), c_int(head_dim), c_int(value_dim), c_int(block_size), c_int(num_blocks),
          c_int(window or 0), c_int(chunk or 0), c_float(scale), c_float(softcap or 0.0), c_int(1 if head_gate else 0),
          c_int(tokens), _ptr(slopes), _ptr(dist_bias), c_int(span), _stream())
    return out


MASKED_MAX_KEY_DIM = 640        # what the vector-ALU attention kernel holds of a key tile in LDS
MASKED_MAX_VALUE_DIM = 512


# ------------------------------------------------- attention through a latent

def latent_norm_rope_write(x: Tensor, q_weight: Tensor, kv_weight: Tensor | None, inv_freq: Tensor | None, positions: Tensor,
                           token_seq: Tensor, block_table: Tensor | None, key_pages: Tensor | None, value_pages: Tensor | None,
                           cq_out: Tensor, *, q_rank: int, kv_rank: int, rot_dim: int, rotary_dim: int, eps: float,
                           write_kv: bool) -> Tensor:
    """From a token's fused down-projections x = [a | b | r] (float32 [T, >= q_rank (+ kv_rank + rot_dim)], any
    row stride): ``cq_out`` [T, q_rank] = a / rms(a) * q_weight, and with ``write_kv`` the token's cache row
    [b / rms(b) * kv_weight | rotate(r)] into ``key_pages`` [blocks, 1, block_size, kv_rank + rot_dim] and, if the
    cache keeps values (``value_pages`` [blocks, 1, kv_rank, block_size], transposed), its first kv_rank numbers
    there as well.  The rotation turns the first ``rotary_dim`` dims of r, dim i with dim i + rotary_dim / 2, by
    position * inv_freq[i].  Norms and angles float32 (epsilon inside the root), one rounding at the stores."""
    _gpu(x, "x", torch.float32, contiguous=False)
    _gpu(q_weight, "q_weight", torch.float32)
    _gpu(cq_out, "cq_out")
    tokens = x.shape[0]
    need = q_rank + (kv_rank + rot_dim if write_kv else 0)
    if x.dim() != 2 or x.shape[1] < need or (x.shape[1] > 1 and x.stride(1) != 1):
        raise KernelError(f"x must be [T, >= {need}] with unit inner stride, got {tuple(x.shape)}")
    if q_weight.shape != (q_rank,) or cq_out.shape != (tokens, q_rank) or not eps > 0.0:
        raise KernelError(f"q_weight must be [{q_rank}], cq_out [{tokens}, {q_rank}] and eps positive")
    if rotary_dim % 2 or not 0 <= rotary_dim <= rot_dim:
        raise KernelError("rotary_dim must be even and at most rot_dim")
    block_size = num_blocks = table_stride = 0
    if write_kv:
        _gpu(kv_weight, "kv_weight", torch.float32)
        _gpu(key_pages, "key_pages", cq_out.dtype)
        _gpu(block_table, "block_table", torch.int32)
        _gpu(positions, "positions", torch.int32)
        _gpu(token_seq, "token_seq", torch.int32)
        if kv_weight.shape != (kv_rank,) or positions.numel() != tokens or token_seq.numel() != tokens:
            raise KernelError(f"kv_weight must be [{kv_rank}], positions and token_seq hold one entry per token")
        if key_pages.dim() != 4 or key_pages.shape[1] != 1 or key_pages.shape[3] != kv_rank + rot_dim:
            raise KernelError(f"key pages must be [blocks, 1, block_size, {kv_rank + rot_dim}], got {tuple(key_pages.shape)}")
        if block_table.dim() != 2 or block_table.stride(1) != 1:
            raise KernelError("block_table must be [sequences, max_blocks] with unit inner stride")
        if rotary_dim:
            _gpu(inv_freq, "inv_freq", torch.float32)
            if inv_freq.shape != (rotary_dim // 2,):
                raise KernelError(f"inv_freq must be [{rotary_dim // 2}]")
        num_blocks, _, block_size, _ = key_pages.shape
        table_stride = block_table.stride(0)
        if value_pages is not None:
            _gpu(value_pages, "value_pages", cq_out.dtype)
            if value_pages.shape != (num_blocks, 1, kv_rank, block_size):
                raise KernelError(f"value pages are transposed: [blocks, 1, {kv_rank}, block_size], got {tuple(value_pages.shape)}")
    stride = x.stride(0) if tokens > 1 else max(x.stride(0), x.shape[1])
    _call("latent", "fe_latent_norm_rope_write", _ptr(x), c_longlong(stride), c_int(q_rank), c_int(kv_rank), c_int(rot_dim),
          c_int(rotary_dim), _ptr(q_weight), _ptr(kv_weight if write_kv else None), _ptr(inv_freq if write_kv and rotary_dim else None),
          _ptr(positions if write_kv else None), _ptr(token_seq if write_kv else None), _ptr(block_table if write_kv else None),
          c_int(table_stride), _ptr(key_pages if write_kv else None), _ptr(value_pages if write_kv else None), _ptr(cq_out),
          c_int(_code(cq_out.dtype)), c_float(eps),
          c_int(tokens), c_int(block_size), c_int(num_blocks), c_int(1 if write_kv else 0), _stream())
    return cq_out


def latent_query_pack(q: Tensor, qa: Tensor, inv_freq: Tensor | None, positions: Tensor, out: Tensor, *, heads: int, dim: int,
                      rot_dim: int, rotary_dim: int, kv_rank: int) -> Tensor:
    """The attention's query rows ``out`` [T, heads, kv_rank + rot_dim]: head h's first kv_rank dims are
    ``qa[h, t]`` (qa [heads, T, kv_rank]: the queries taken through the keys' up-projection), the rest the
    last rot_dim dims of head h of ``q`` [T, heads * (dim + rot_dim)], their first ``rotary_dim`` rotated
    (dim i with dim i + rotary_dim / 2, angle position * inv_freq[i], float32)."""
    _gpu(q, "q", contiguous=False)
    _gpu(qa, "qa", q.dtype)
    _gpu(out, "out", q.dtype)
    _gpu(positions, "positions", torch.int32)
    tokens = q.shape[0]
    q_stride = _strided_rows(q, "q", heads * (dim + rot_dim))
    if qa.shape != (heads, tokens, kv_rank) or out.shape != (tokens, heads, kv_rank + rot_dim) or positions.numel() != tokens:
        raise KernelError(f"qa must be [{heads}, {tokens}, {kv_rank}] and out [{tokens}, {heads}, {kv_rank + rot_dim}]")
    if rotary_dim % 2 or not 0 <= rotary_dim <= rot_dim:
        raise KernelError("rotary_dim must be even and at most rot_dim")
    if rotary_dim:
        _gpu(inv_freq, "inv_freq", torch.float32)
        if inv_freq.shape != (rotary_dim // 2,):
            raise KernelError(f"inv_freq must be [{rotary_dim // 2}]")
    _call("latent", "fe_latent_query_pack", _ptr(q), c_longlong(q_stride), _ptr(qa), _ptr(inv_freq if rotary_dim else None),
          _ptr(positions), _ptr(out), c_int(_code(q.dtype)), c_int(tokens), c_int(heads), c_int(dim), c_int(rot_dim),
          c_int(rotary_dim), c_int(kv_rank), _stream())
    return out


LATENT_TARGET_BLOCKS = 512      # blocks the matrix-core attention over a latent aims at before it stops cutting the keys into runs
LATENT_MIN_TILES = 2            # ... and the fewest tiles a run may have (8 sequences at 1,024 keys, 16 heads, rows of 576, us a call with the
                                # merge, in a captured graph: 1 run 110, 2 runs 62, 4 runs 36, 8 runs 24, 16 runs 21, 32 runs 25)


def latent_splits(num_seqs: int, max_q_len: int, heads: int, max_ctx: int | None) -> int:
    """Runs that the matrix-core attention over a latent cuts every block's keys into: 1 when the step fills
    the chip or the context is not known, else enough for about LATENT_TARGET_BLOCKS blocks with at least
    LATENT_MIN_TILES tiles of 32 keys each."""
    if max_ctx is None:
        return 1
    blocks = -(-max(1, max_q_len) * heads // 64) * max(1, num_seqs)
    return max(1, min(-(-LATENT_TARGET_BLOCKS // blocks), max_ctx // (32 * LATENT_MIN_TILES), 32))


def latent_attention_supported(dtype, row_dim: int, value_dim: int, block_size: int) -> bool:
    """Whether the matrix-core kernel takes these sizes (else the vector-ALU kernel does)."""
    if dtype != torch.bfloat16 or block_size < 8 or block_size & (block_size - 1):      # pages of a power of two, eight slots or more
        return False
    fn = library.load("attention_latent").fe_latent_attention_supported
    fn.restype = c_int
    return bool(fn(c_int(row_dim), c_int(value_dim)))


def latent_attention(q: Tensor, key_pages: Tensor, value_pages: Tensor | None, out: Tensor, cu_q: Tensor, ctx_len: Tensor,
                     block_table: Tensor, *, num_seqs: int, max_q_len: int, heads: int, row_dim: int, value_dim: int,
                     scale: float, num_decode: int | None = None, max_ctx: int | None = None, splits: int | None = None) -> Tensor:
    """Causal attention of ``heads`` query heads over one shared cache of rows, ``key_pages`` [blocks, 1,
    block_size, row_dim]: a row is the key of every head and its first ``value_dim`` dims are the value, which
    ``value_pages`` [blocks, 1, value_dim, block_size] holds a second time, transposed (None: a cache of keys
    only, read by the vector-ALU kernel).  q [T, heads * row_dim], out [T, heads * value_dim]; scores and
    softmax float32.  bfloat16 at the sizes the matrix-core kernel is compiled for goes there (``splits``: its
    key runs, chosen here if None); everything else, and the float32 mode, to the vector-ALU kernel."""
    _gpu(q, "q")
    _gpu(key_pages, "key_pages", q.dtype)
    block_size = key_pages.shape[2] if key_pages.dim() == 4 else 0
    if value_pages is None or not latent_attention_supported(q.dtype, row_dim, value_dim, block_size) or q.data_ptr() % 16:
        return masked_attention(q, key_pages, value_pages, out, cu_q, ctx_len, block_table, num_seqs=num_seqs, max_q_len=max_q_len,
                                q_heads=heads, kv_heads=1, head_dim=row_dim, value_dim=value_dim, scale=scale,
                                num_decode=num_decode, max_ctx=max_ctx)
    _gpu(value_pages, "value_pages", q.dtype)
    _gpu(out, "out", q.dtype)
    _gpu(cu_q, "cu_q", torch.int32)
    _gpu(ctx_len, "ctx_len", torch.int32)
    _gpu(block_table, "block_table", torch.int32)
    tokens = q.shape[0]
    if q.shape != (tokens, heads * row_dim) or out.shape != (tokens, heads * value_dim):
        raise KernelError(f"q must be [T, {heads * row_dim}] and out [T, {heads * value_dim}], got {tuple(q.shape)} and {tuple(out.shape)}")
    if key_pages.dim() != 4 or key_pages.shape[1] != 1 or key_pages.shape[3] != row_dim:
        raise KernelError(f"key pages must be [blocks, 1, block_size, {row_dim}], got {tuple(key_pages.shape)}")
    num_blocks = key_pages.shape[0]
    if value_pages.shape != (num_blocks, 1, value_dim, block_size):
        raise KernelError(f"value pages are transposed: [blocks, 1, {value_dim}, block_size], got {tuple(value_pages.shape)}")
    if cu_q.numel() != num_seqs + 1 or ctx_len.numel() != num_seqs or block_table.dim() != 2 or block_table.shape[0] < num_seqs \
            or block_table.stride(1) != 1 or max_q_len < 1:
        raise KernelError("cu_q, ctx_len and block_table do not match the number of sequences")
    if splits is None:
        splits = latent_splits(num_seqs, max_q_len, heads, max_ctx)
    if not 1 <= splits <= 64:
        raise KernelError("between 1 and 64 key runs")
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty((splits, tokens * heads, value_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((splits, tokens * heads, 2), dtype=torch.float32, device=q.device)
    _call("attention_latent", "fe_latent_attention", _ptr(q), c_longlong(q.stride(0)), _ptr(key_pages), _ptr(value_pages), _ptr(out),
          _ptr(part_o), _ptr(part_ml), _ptr(cu_q), _ptr(ctx_len), _ptr(block_table), c_int(block_table.stride(0)), c_int(num_seqs),
          c_int(max_q_len), c_int(heads), c_int(row_dim), c_int(value_dim), c_int(block_size), c_int(num_blocks), c_float(scale),
          c_int(splits), c_int(tokens), _stream())
    return out


def heads_product(x: Tensor, weight: Tensor) -> Tensor:
    """A product per head: x [T, heads, K] (rows and heads of any stride, unit inner stride) times weight
    [heads, K, N] gives [heads, T, N] in x's dtype, accumulated in float32 (true float32 products for
    float32 operands).  The platform's batched matrix product."""
    _gpu(x, "x", contiguous=False)
    _gpu(weight, "weight", x.dtype, contiguous=False)
    if x.dim() != 3 or weight.dim() != 3 or weight.shape[0] != x.shape[1] or weight.shape[1] != x.shape[2]:
        raise KernelError(f"x must be [T, heads, K] and weight [heads, K, N], got {tuple(x.shape)} and {tuple(weight.shape)}")
    return torch.bmm(x.transpose(0, 1), weight)


# ------------------------------------------------- linear recurrences over a matrix state

_DECAY_KINDS = {"none": 0, "exp_neg_exp": 1, "sigmoid_root": 2}


def linear_recurrence(q: Tensor, k: Tensor, v: Tensor, out: Tensor, state: Tensor, cu_q: Tensor, state_slots: Tensor, *,
                      num_seqs: int, max_q_len: int, heads: int, key_dim: int, value_dim: int,
                      decay: Tensor | None = None, decay_kind: str = "none", decay_bias: Tensor | None = None,
                      tau: float = 1.0, head_decay: Tensor | None = None, in_scale: Tensor | None = None,
                      q_scale: float = 1.0, bonus: Tensor | None = None, ones_column: bool = False) -> Tensor:
    """Per sequence and head, token after token:  S <- diag(a_t) S + b_t k_t v_t^T,  o_t = S^T (q_t *
    q_scale), with S [key_dim, value_dim] float32 carried in ``state`` [slots, heads, value_dim (+1),
    key_dim] (value-major) between steps.

    a_t per key channel from ``decay`` (float32 [T, heads * key_dim], before its bias):
    ``exp_neg_exp`` a = exp(-exp(d + bias)), ``sigmoid_root`` a = sigmoid(d + bias)^(1 / tau); or per
    head from ``head_decay`` (float32 [T, heads]; not both); b_t = ``in_scale`` [T, heads] or 1.
    ``bonus`` (float32 [heads * key_dim]): the query reads the state before the token's update plus
    diag(bonus) k_t v_t^T instead.  ``ones_column``: one more value column fed by v = 1 (a
    normaliser).  ``decay`` is overwritten with the decays a_t (its transform runs in place, in a
    kernel of its own over the whole step, before the walk).  q, k [T, heads * key_dim] and v [T, heads * value_dim] rows of any stride, in the
    compute dtype; out float32 [T, heads, value_dim (+1)]."""
    columns = value_dim + (1 if ones_column else 0)
    tokens = q.shape[0]
    strides = [_strided_rows(q, "q", heads * key_dim), _strided_rows(k, "k", heads * key_dim),
               _strided_rows(v, "v", heads * value_dim)]
    if k.dtype != q.dtype or v.dtype != q.dtype or k.shape[0] != tokens or v.shape[0] != tokens:
        raise KernelError("q, k and v must share dtype and token count")
    _gpu(out, "out", torch.float32)
    _gpu(state, "state", torch.float32)
    _sequences(cu_q, state_slots, num_seqs)
    if out.shape != (tokens, heads, columns):
        raise KernelError(f"out must be [{tokens}, {heads}, {columns}], got {tuple(out.shape)}")
    if state.dim() != 4 or state.shape[1:] != (heads, columns, key_dim):
        raise KernelError(f"state must be [slots, {heads}, {columns}, {key_dim}], got {tuple(state.shape)}")
    if not 1 <= key_dim <= 256:
        raise KernelError("key sizes up to 256")
    if decay_kind not in _DECAY_KINDS or (decay is None) != (decay_kind == "none"):
        raise KernelError("decay and decay_kind go together")
    for name, t, shape in (("decay", decay, (tokens, heads * key_dim)), ("decay_bias", decay_bias, (heads * key_dim,)),
                           ("head_decay", head_decay, (tokens, heads)), ("in_scale", in_scale, (tokens, heads)),
                           ("bonus", bonus, None)):
        if t is not None:
            _gpu(t, name, torch.float32)
            if shape is not None and tuple(t.shape) != shape:
                raise KernelError(f"{name} must be {shape}, got {tuple(t.shape)}")
    if bonus is not None and bonus.numel() != heads * key_dim:
        raise KernelError(f"bonus must hold {heads * key_dim} entries")
    if decay is not None and decay_bias is None:
        raise KernelError("a decay comes with its bias")
    if decay is not None and head_decay is not None:
        raise KernelError("the decay comes per key channel or per head, not both")
    if max_q_len < 1 or not tau > 0.0:
        raise KernelError("max_q_len and tau must be positive")
    _call("linear_recurrence", "fe_linear_recurrence", _ptr(q), _ptr(k), _ptr(v), c_int(_code(q.dtype)),
          c_longlong(strides[0]), c_longlong(strides[1]), c_longlong(strides[2]), _ptr(decay), c_int(_DECAY_KINDS[decay_kind]),
          _ptr(decay_bias), c_float(tau), _ptr(head_decay), _ptr(in_scale), c_float(q_scale), _ptr(bonus),
          c_int(1 if ones_column else 0), _ptr(state), c_int(state.shape[0]), _ptr(out), _ptr(cu_q), _ptr(state_slots),
          c_int(num_seqs), c_int(max_q_len), c_int(heads), c_int(key_dim), c_int(value_dim), c_int(tokens), _stream())
    return out


def mlstm_gate_scan(gates: Tensor, bias: Tensor, cap: float, maximum: Tensor, cu_q: Tensor, state_slots: Tensor,
                    out: Tensor, *, num_seqs: int, heads: int) -> Tensor:
    """The stabilised gates of an mLSTM, per sequence and head along the tokens: with i = cap tanh((g_i +
    b_i) / cap), f = logsigmoid(cap tanh((g_f + b_f) / cap)) and the running maximum m_t = max(f + m_(t-1),
    i) (``maximum`` [slots, heads] keeps m between steps, 0 for a new request): out[0] = exp(f + m_(t-1) -
    m_t), out[1] = exp(i - m_t), out[2] = exp(-m_t).  gates float32 [T, 2 heads] (input gates, then forget
    gates), bias float32 [2 heads], out float32 [3, T, heads]."""
    _gpu(gates, "gates", torch.float32)
    _gpu(bias, "bias", torch.float32)
    _gpu(maximum, "maximum", torch.float32)
    _gpu(out, "out", torch.float32)
    _sequences(cu_q, state_slots, num_seqs)
    tokens = gates.shape[0]
    if gates.shape != (tokens, 2 * heads) or bias.shape != (2 * heads,) or out.shape != (3, tokens, heads):
        raise KernelError(f"gates [T, {2 * heads}], bias [{2 * heads}], out [3, T, {heads}]")
    if maximum.dim() != 2 or maximum.shape[1] != heads or not cap > 0.0:
        raise KernelError(f"maximum must be [slots, {heads}] and cap positive")
    _call("linear_recurrence", "fe_mlstm_gate_scan", _ptr(gates), _ptr(bias), c_float(cap), _ptr(maximum),
          c_int(maximum.shape[0]), _ptr(cu_q), _ptr(state_slots), _ptr(out), c_int(tokens), c_int(num_seqs), c_int(heads),
          _stream())
    return out


# ------------------------------------------------- several residual streams, token pairs, a factor on the logits

def hyper_norm(streams: Tensor, update: Tensor | None, mix: Tensor | None, share: Tensor | None, read: Tensor | None,
               weight: Tensor | None, bias: Tensor | None, eps: float, out: Tensor | None, rows: Tensor | None = None,
               store: bool = True, rms: bool = False) -> Tensor | None:
    """The norm over S residual streams [S, T, W] (float32; S = 1: one plain stream), fused with the
    pending update (float32 [T, W] or [parts, T, W], added up in order):
    ``x_t <- sum_s mix[s, t] x_s + share[t] * update`` (mix None: the identity, share None: ones; written
    back unless ``store`` is False), ``u = sum_t read[t] x_t`` (None: the plain sum), and ``out`` =
    the layer norm of u with weight and bias (``rms``: the RMS norm, no mean, bias optional), of the
    rows listed in ``rows`` if given.  ``out`` None: the update is applied and nothing else."""
    _gpu(streams, "streams", torch.float32)
    if streams.dim() != 3 or not 1 <= streams.shape[0] <= 8:
        raise KernelError(f"streams must be [1..8, T, W], got {tuple(streams.shape)}")
    count, total_rows, width = streams.shape
    if width > 16384:
        raise KernelError("rows of up to 16,384 elements")
    parts = 0
    if update is not None:
        parts = _parts_of(update, total_rows, width, "update")
    elif out is None:
        raise KernelError("nothing to do: neither an update nor an output")
    for name, t, shape in (("mix", mix, (count, count)), ("share", share, (count,)), ("read", read, (count,)),
                           ("weight", weight, (width,)), ("bias", bias, (width,))):
        if t is not None:
            _gpu(t, name, torch.float32)
            if tuple(t.shape) != shape:
                raise KernelError(f"{name} must be {shape}, got {tuple(t.shape)}")
    n_rows = total_rows
    if rows is not None:
        _gpu(rows, "rows", torch.int32)
        n_rows = rows.numel()
        if store and update is not None:
            raise KernelError("store with a row list is not allowed (rows may repeat)")
    if out is not None:
        _gpu(out, "out")
        if out.shape != (n_rows, width) or weight is None or not eps > 0.0:
            raise KernelError(f"out must be [{n_rows}, {width}] and come with a weight and a positive eps")
    _call("hyper", "fe_hyper_norm", _ptr(streams), c_longlong(total_rows * width), c_int(count), _ptr(update), c_int(parts),
          c_longlong(total_rows * width), _ptr(mix), _ptr(share), _ptr(read), _ptr(weight), _ptr(bias), c_float(eps),
          c_int(1 if rms else 0), _ptr(out), c_int(_code(out.dtype) if out is not None else FE_F32), _ptr(rows),
          c_int(n_rows), c_int(width), c_int(1 if (store and update is not None) else 0), _stream())
    return out


def embed_token_pairs(ids: Tensor, table: Tensor, pair_table: Tensor, positions: Tensor, token_seq: Tensor, cu_q: Tensor,
                      state_slots: Tensor, previous: Tensor, out: Tensor, *, num_seqs: int, buckets: int, mul_prev: int,
                      mul_cur: int) -> Tensor:
    """out[t] = float32(table[ids[t]]) + float32(pair_table[r]) with r = (prev * mul_prev + ids[t] * mul_cur)
    mod buckets, prev the token before t in its sequence: the row before within the step, or, for a
    sequence's first token of the step, what ``previous`` [slots, 1] (int32) keeps for its slot; a token at
    position 0 takes row ``buckets`` (the table's last).  Afterwards ``previous`` holds every
    sequence's last token."""
    for name, t in (("ids", ids), ("positions", positions), ("token_seq", token_seq), ("previous", previous)):
        _gpu(t, name, torch.int32)
    _sequences(cu_q, state_slots, num_seqs)
    _gpu(table, "table")
    _gpu(pair_table, "pair_table", table.dtype)
    _gpu(out, "out", torch.float32)
    tokens = ids.numel()
    vocab, hidden = table.shape
    if pair_table.shape != (buckets + 1, hidden) or buckets < 1 or mul_prev < 0 or mul_cur < 0:
        raise KernelError(f"pair_table must be [{buckets + 1}, {hidden}], got {tuple(pair_table.shape)}")
    if out.shape != (tokens, hidden) or positions.numel() != tokens or token_seq.numel() != tokens:
        raise KernelError("out must be [T, hidden]; positions and token_seq hold one entry per token")
    if previous.dim() != 2 or previous.shape[1] != 1:
        raise KernelError("previous must be [slots, 1]")
    _call("hyper", "fe_embed_token_pairs", _ptr(ids), _ptr(table), _ptr(pair_table), c_int(_code(table.dtype)), _ptr(positions),
          _ptr(token_seq), _ptr(cu_q), _ptr(state_slots), _ptr(previous), _ptr(out), c_int(tokens), c_int(hidden), c_int(vocab),
          c_longlong(buckets), c_longlong(mul_prev), c_longlong(mul_cur), c_int(num_seqs), c_int(previous.shape[0]), _stream())
    return out


def scale_rows(x: Tensor, factor: float) -> Tensor:
    """x *= factor, in place (float32)."""
    _gpu(x, "x", torch.float32)
    _call("hyper", "fe_scale_rows", _ptr(x), c_float(factor), c_longlong(x.numel()), _stream())
    return x


# ------------------------------------------------- a norm over the whole projection, rotation, page write

def whole_norm_rope_write(qkv: Tensor, q_weight: Tensor, k_weight: Tensor | None, inv_freq: Tensor | None, positions: Tensor,
                          token_seq: Tensor, block_table: Tensor, key_pages: Tensor, value_pages: Tensor, q_out: Tensor, *,
                          q_heads: int, kv_heads: int, head_dim: int, value_dim: int, rotary_dim: int, eps: float,
                          magnitude: float = 1.0, write_kv: bool = True) -> None:
    """q (and k) divided by the root mean square over the whole projection (all heads at once, epsilon
    inside the root) times a weight of that length; then the first ``rotary_dim`` dims of every head turn
    (dim i pairs with i + rotary_dim / 2, cosines and sines times ``magnitude``); q into ``q_out``
    [T, Hq * D], k and v into their pages (values transposed).  qkv [T, >= q | k | v] with any row stride;
    with ``write_kv`` False it holds q alone and the pages are left as they are.  float32 inside."""
    q_size, kv_size, v_size = q_heads * head_dim, kv_heads * head_dim, kv_heads * value_dim
    need = q_size + (kv_size + v_size if write_kv else 0)
    _gpu(qkv, "qkv", contiguous=False)
    tokens = qkv.shape[0]
    if qkv.dim() != 2 or qkv.shape[1] < need or qkv.stride(1) != 1:
        raise KernelError(f"qkv must be [T, >= {need}] with unit inner stride")
    _gpu(q_out, "q_out", qkv.dtype)
    if q_out.shape != (tokens, q_size):
        raise KernelError(f"q_out must be [{tokens}, {q_size}]")
    _gpu(q_weight, "q_weight", torch.float32)
    if q_weight.shape != (q_size,):
        raise KernelError(f"q_weight must be [{q_size}]")
    if rotary_dim:
        _gpu(inv_freq, "inv_freq", torch.float32)
        if inv_freq.shape != (rotary_dim // 2,) or rotary_dim % 2 or rotary_dim > head_dim or rotary_dim > 256:
            raise KernelError(f"inv_freq must be [{rotary_dim // 2}] for an even rotary_dim <= head_dim and <= 256")
    _gpu(positions, "positions", torch.int32)
    _gpu(token_seq, "token_seq", torch.int32)
    if positions.numel() != tokens or token_seq.numel() != tokens:
        raise KernelError("positions and token_seq must have one entry per token")
    block_size = num_blocks = table_stride = 0
    if write_kv:
        _gpu(k_weight, "k_weight", torch.float32)
        if k_weight.shape != (kv_size,):
            raise KernelError(f"k_weight must be [{kv_size}]")
        _gpu(block_table, "block_table", torch.int32)
        _gpu(key_pages, "key_pages", qkv.dtype)
        _gpu(value_pages, "value_pages", qkv.dtype)
        if key_pages.dim() != 4 or key_pages.shape[1] != kv_heads or key_pages.shape[3] != head_dim:
            raise KernelError(f"key pages must be [blocks, {kv_heads}, block_size, {head_dim}], got {tuple(key_pages.shape)}")
        num_blocks, _, block_size, _ = key_pages.shape
        if value_pages.shape != (num_blocks, kv_heads, value_dim, block_size):
            raise KernelError(f"value pages are transposed: [blocks, {kv_heads}, {value_dim}, block_size], got {tuple(value_pages.shape)}")
        if block_table.dim() != 2 or block_table.stride(1) != 1:
            raise KernelError("block_table must be [sequences, max_blocks] with unit inner stride")
        table_stride = block_table.stride(0)
    if not eps > 0.0:
        raise KernelError("eps must be positive")
    stride = qkv.stride(0) if tokens > 1 else max(qkv.stride(0), qkv.shape[1])
    _call("whole_norm_rope", "fe_whole_norm_rope_write", _ptr(qkv), c_int(_code(qkv.dtype)), c_longlong(stride), _ptr(q_weight),
          _ptr(k_weight if write_kv else None), _ptr(inv_freq if rotary_dim else None), _ptr(positions), _ptr(token_seq),
          _ptr(block_table if write_kv else None), c_int(table_stride), _ptr(key_pages if write_kv else None),
          _ptr(value_pages if write_kv else None), _ptr(q_out), c_int(tokens), c_int(q_heads), c_int(kv_heads), c_int(head_dim),
          c_int(value_dim), c_int(rotary_dim), c_float(eps), c_float(magnitude), c_int(1 if write_kv else 0), c_int(block_size),
          c_int(num_blocks), _stream())


# ------------------------------------------------- a mixture of experts

_SCORINGS = {"softmax": 0, "sigmoid": 1}
_GATED_FORMS = {"bounded": 0, "silu": 1}


def moe_route(x: Tensor, router_weight: Tensor, router_bias: Tensor | None, top: int, scoring: str = "softmax") -> tuple[Tensor, Tensor]:
    """Router logits ``x W^T + b`` in float32; for every token the ``top`` experts with the largest logits
    (int32 [T, top], largest first, the lowest index among equals) and their weights (float32 [T, top]): the
    softmax over the chosen logits alone, or (``scoring`` "sigmoid") each chosen logit's own sigmoid."""
    _gpu(x, "x")
    _gpu(router_weight, "router_weight", x.dtype)
    tokens, hidden = x.shape
    experts = router_weight.shape[0]
    if router_weight.shape != (experts, hidden) or not 1 <= top <= min(experts, 16) or experts > 1024:
        raise KernelError(f"router_weight must be [experts <= 1024, {hidden}] and top between 1 and min(experts, 16)")
    if router_bias is not None:
        _gpu(router_bias, "router_bias", torch.float32)
        if router_bias.shape != (experts,):
            raise KernelError(f"router_bias must be [{experts}]")
    logits = linear(x, router_weight, out_dtype=torch.float32)     # float32 accumulation, float32 logits
    chosen = torch.empty((tokens, top), dtype=torch.int32, device=x.device)
    weights = torch.empty((tokens, top), dtype=torch.float32, device=x.device)
    _call("moe", "fe_moe_select", _ptr(logits), _ptr(router_bias), _ptr(chosen), _ptr(weights), c_int(tokens), c_int(experts),
          c_int(top), c_int(_SCORINGS[scoring]), _stream())
    return chosen, weights


def moe_route_grouped(x: Tensor, router_weight: Tensor, correction: Tensor | None, *, experts: int, top: int, groups: int = 1,
                      keep: int = 1, scale: float = 1.0) -> tuple[Tensor, Tensor, Tensor]:
    """Router logits ``x W^T`` in float32 (W may hold rows beyond the ``experts`` first, a gate's say: their logits
    come back with the others); scores s = softmax over the experts' logits; an expert's choice score is
    ``s + correction``; the experts form ``groups`` equal runs of neighbours, a run's score is its largest
    choice score, and only experts of the ``keep`` best runs can be chosen; the ``top`` largest choice scores
    are chosen (int32 [T, top], largest first, the lowest index among equals) and their weights (float32
    [T, top]) are their own s over the sum of the chosen s (+ 1e-20), times ``scale``.  Returns (chosen,
    weights, logits [T, rows of W])."""
    _gpu(x, "x")
    _gpu(router_weight, "router_weight", x.dtype)
    tokens, hidden = x.shape
    if router_weight.dim() != 2 or router_weight.shape[1] != hidden or router_weight.shape[0] < experts:
        raise KernelError(f"router_weight must be [>= {experts}, {hidden}], got {tuple(router_weight.shape)}")
    if not 1 <= experts <= 1024 or not 1 <= groups <= 64 or experts % groups or not 1 <= keep <= groups:
        raise KernelError("up to 1,024 experts in up to 64 equal groups, of which between one and all are kept")
    if not 1 <= top <= min(16, experts // groups * keep):
        raise KernelError(f"top must lie between 1 and min(16, experts of the kept groups), got {top}")
    if correction is not None:
        _gpu(correction, "correction", torch.float32)
        if correction.shape != (experts,):
            raise KernelError(f"correction must be [{experts}]")
    logits = linear(x, router_weight, out_dtype=torch.float32)
    chosen = torch.empty((tokens, top), dtype=torch.int32, device=x.device)
    weights = torch.empty((tokens, top), dtype=torch.float32, device=x.device)
    _call("moe", "fe_moe_select_grouped", _ptr(logits), c_longlong(logits.shape[1]), _ptr(correction), _ptr(chosen), _ptr(weights),
          c_int(tokens), c_int(experts), c_int(top), c_int(groups), c_int(keep), c_float(scale), _stream())
    return chosen, weights, logits


def moe_experts(x: Tensor, chosen: Tensor, weights: Tensor, gate_up: Tensor, down: Tensor, out: Tensor, *, limit: float = 0.0,
                alpha: float = 1.0, extra: Tensor | None = None, form: str = "bounded", weight_input: bool = False) -> Tensor:
    """out[k, t] = weights[t, k] * down[e] @ act, e = chosen[t, k], with ``act = min(g, limit) *
    sigmoid(alpha * min(g, limit)) * (clamp(u, -limit, limit) + 1)``, ``g = gate_up[e, :F] @ x[t]``,
    ``u = gate_up[e, F:] @ x[t]``.  x [T, H]; gate_up [E, 2F, H]; down [E, H, F]; out float32 [top, T, H]
    (one part per choice).  ``extra`` (float32 [T, H] or [parts, T, H], added up in order): what every
    token gets beside its experts; it joins the first choice's part.  ``form`` "silu": ``act = silu(g) * u``, no
    bounds.  ``weight_input``: the routing weight scales the expert's input instead of its output (g and u are
    multiplied by it before the activation, which is the same as multiplying x).  The pairs are sorted by
    expert on the device and two grouped products run over the sorted rows."""
    _gpu(x, "x")
    _gpu(chosen, "chosen", torch.int32)
    _gpu(weights, "weights", torch.float32)
    _gpu(gate_up, "gate_up", x.dtype)
    _gpu(down, "down", x.dtype)
    _gpu(out, "out", torch.float32)
    tokens, hidden = x.shape
    top = chosen.shape[1] if chosen.dim() == 2 else 0
    if gate_up.dim() != 3 or gate_up.shape[2] != hidden or gate_up.shape[1] % 2:
        raise KernelError(f"gate_up must be [experts, 2F, {hidden}], got {tuple(gate_up.shape)}")
    experts, inner = gate_up.shape[0], gate_up.shape[1] // 2
    if down.shape != (experts, hidden, inner):
        raise KernelError(f"down must be [{experts}, {hidden}, {inner}], got {tuple(down.shape)}")
    if chosen.shape != (tokens, top) or weights.shape != (tokens, top) or not 1 <= top <= 16 or experts > 1024:
        raise KernelError("chosen and weights must be [T, top <= 16] and experts at most 1,024")
    if out.shape != (top, tokens, hidden):
        raise KernelError(f"out must be [{top}, {tokens}, {hidden}], got {tuple(out.shape)}")
    if form not in _GATED_FORMS or (form == "bounded" and not limit > 0.0):
        raise KernelError("the bounded activation needs a positive limit; forms: " + ", ".join(_GATED_FORMS))
    extra_parts = 0 if extra is None else _parts_of(extra, tokens, hidden, "extra")
    pairs = tokens * top
    offsets = torch.empty(experts + 1, dtype=torch.int32, device=x.device)
    order = torch.empty(pairs, dtype=torch.int32, device=x.device)
    act = torch.empty((pairs, inner), dtype=x.dtype, device=x.device)
    code = c_int(_code(x.dtype))
    _call("moe", "fe_moe_plan", _ptr(chosen), c_int(pairs), c_int(experts), _ptr(offsets), _ptr(order), _stream())
    _call("moe", "fe_moe_gate_up", _ptr(x), _ptr(gate_up), code, _ptr(offsets), _ptr(order), _ptr(act), c_int(tokens), c_int(top),
          c_int(experts), c_int(hidden), c_int(inner), c_float(limit), c_float(alpha), c_int(_GATED_FORMS[form]),
          _ptr(weights if weight_input else None), _stream())
    _call("moe", "fe_moe_down", _ptr(act), _ptr(down), code, _ptr(offsets), _ptr(order), _ptr(None if weight_input else weights), _ptr(out), c_int(tokens),
          c_int(top), c_int(experts), c_int(hidden), c_int(inner), _ptr(extra), c_int(extra_parts), _stream())
    return out


def linear_gated(x: Tensor, gate_up_weight: Tensor, *, limit: float, alpha: float) -> Tensor:
    """``min(g, limit) * sigmoid(alpha * min(g, limit)) * (clamp(u, -limit, limit) + 1)`` with g and u the two
    halves of ``x @ gate_up_weight^T`` ([2F, H]: gate rows first); the result [T, F] in x's dtype."""
    gate_up = linear(x, gate_up_weight)
    tokens, width = gate_up.shape
    if width % 2 or not limit > 0.0:
        raise KernelError("a gated weight needs an even number of rows and a positive limit")
    out = torch.empty((tokens, width // 2), dtype=gate_up.dtype, device=gate_up.device)
    _call("moe", "fe_gated_act", _ptr(gate_up), _ptr(out), c_int(_code(gate_up.dtype)), c_int(tokens), c_int(width // 2),
          c_float(limit), c_float(alpha), _stream())
    return out


# ------------------------------------------------- dense activations, short convolutions, selective scans

def relu_squared(x: Tensor) -> Tensor:
    """max(x, 0)^2 of every element, into a new tensor of x's dtype (float32 inside)."""
    _gpu(x, "x")
    out = torch.empty_like(x)
    _call("stream_ops", "fe_relu_squared", _ptr(x), _ptr(out), c_int(_code(x.dtype)), c_longlong(x.numel()), _stream())
    return out


ACTIVATIONS = {"relu_squared": 0, "gelu": 1, "gelu_tanh": 2}


def activate(x: Tensor, kind: str) -> Tensor:
    """An activation of every element, into a new tensor of x's dtype (float32 inside): ``relu_squared``,
    ``gelu`` (0.5 z (1 + erf(z / sqrt 2))) or ``gelu_tanh`` (0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))))."""
    _gpu(x, "x")
    if kind not in ACTIVATIONS:
        raise KernelError(f"unknown activation '{kind}' (known: {', '.join(ACTIVATIONS)})")
    out = torch.empty_like(x)
    _call("stream_ops", "fe_activate", _ptr(x), _ptr(out), c_int(_code(x.dtype)), c_longlong(x.numel()), c_int(ACTIVATIONS[kind]),
          _stream())
    return out


def gate_rows(update: Tensor, logits: Tensor, column: int) -> Tensor:
    """update[..., t, :] *= sigmoid(logits[t, column]), in place: one gate a token over a float32 update
    [T, W] or [parts, T, W]; logits float32 [T, n]."""
    _gpu(update, "update", torch.float32)
    _gpu(logits, "logits", torch.float32)
    if update.dim() not in (2, 3) or logits.dim() != 2 or logits.shape[0] != update.shape[-2] or not 0 <= column < logits.shape[1]:
        raise KernelError(f"update must be [T, W] or [parts, T, W] and logits [T, > {column}], got {tuple(update.shape)} and {tuple(logits.shape)}")
    parts = update.shape[0] if update.dim() == 3 else 1
    _call("stream_ops", "fe_gate_rows", _ptr(update), c_int(parts), c_void_p(logits.data_ptr() + 4 * column), c_longlong(logits.shape[1]),
          c_int(update.shape[-2]), c_int(update.shape[-1]), _stream())
    return update


def causal_conv_act(u: Tensor, weight: Tensor, bias: Tensor | None, state: Tensor | None, token_seq: Tensor, cu_q: Tensor,
                    state_slots: Tensor, *, num_seqs: int, act: str = "silu") -> Tensor:
    """A short causal convolution over time on every channel, then the activation: ``y_t = act(b + sum_j
    w[:, j] * u_(t - taps + 1 + j))``.  u [T, >= channels] with any row stride (its first ``channels`` columns
    are read); weight float32 [channels, taps], the last column the token's own; bias float32 [channels] or
    None; state float32 [slots, taps - 1, channels]: every sequence's last taps - 1 rows of u, read for the
    rows before the step and moved on afterwards (None with one tap).  Returns [T, channels] in u's dtype."""
    _gpu(u, "u", contiguous=False)
    _gpu(weight, "weight", torch.float32)
    if weight.dim() != 2 or not 1 <= weight.shape[1] <= 8:
        raise KernelError("weight must be [channels, taps in 1..8]")
    channels, taps = weight.shape
    tokens = u.shape[0]
    stride = _strided_rows(u, "u", channels)
    if bias is not None:
        _gpu(bias, "bias", torch.float32)
        if bias.shape != (channels,):
            raise KernelError(f"bias must be [{channels}]")
    if taps > 1:
        _gpu(state, "state", torch.float32)
        if state.dim() != 3 or state.shape[1:] != (taps - 1, channels):
            raise KernelError(f"state must be [slots, {taps - 1}, {channels}]")
    _gpu(token_seq, "token_seq", torch.int32)
    if token_seq.numel() != tokens:
        raise KernelError("token_seq must have one entry per token")
    _sequences(cu_q, state_slots, num_seqs)
    if act not in _ACTS or _ACTS[act] > 1:
        raise KernelError("act must be none or silu")
    slots = state.shape[0] if taps > 1 else 0
    out = torch.empty((tokens, channels), dtype=u.dtype, device=u.device)
    code = c_int(_code(u.dtype))
    _call("selective_scan", "fe_causal_conv_act", _ptr(u), code, c_longlong(stride), _ptr(weight), _ptr(bias),
          _ptr(state if taps > 1 else None), _ptr(token_seq), _ptr(cu_q), _ptr(state_slots), _ptr(out), c_int(tokens),
          c_int(channels), c_int(taps), c_int(slots), c_int(_ACTS[act]), _stream())
    if taps > 1:
        _call("conv_rope", "fe_conv_state_update", _ptr(u), code, c_longlong(stride), _ptr(None), _ptr(state), _ptr(cu_q),
              _ptr(state_slots), c_int(num_seqs), c_int(channels), c_int(taps), c_int(slots), c_int(tokens), _stream())
    return out


_SCAN_SHAPES = ((4, 4), (8, 4), (16, 1), (16, 2), (16, 4), (16, 8), (16, 16))   # (lanes a channel, states a lane)
SCAN_TARGET_BLOCKS = 512
SCAN_SEGMENT = 64              # tokens a segment when a step's sequences are cut up (a multiple of 16)
SCAN_SEGMENT_MIN_TOKENS = 128  # ... which happens when a sequence of the step may be this much longer than one token


def scan_shape(channels: int, states: int, blocks_each: int) -> tuple[int, int]:
    """How many lanes share a channel and how many states each holds: the fewest lanes whose launch still has
    about two blocks a CU (``blocks_each`` blocks work on every channel: sequences, or segments), else the
    most; then the fewest states a lane that hold them all."""
    fitting = [(lanes, per) for lanes, per in _SCAN_SHAPES if lanes * per >= states]
    if not fitting:
        raise KernelError(f"up to 256 states a channel, not {states}")
    by_lanes: dict[int, int] = {}
    for lanes, per in fitting:
        by_lanes[lanes] = min(per, by_lanes.get(lanes, per))
    for lanes in sorted(by_lanes):
        if -(-channels * lanes // 256) * blocks_each >= SCAN_TARGET_BLOCKS:
            return lanes, by_lanes[lanes]
    lanes = max(by_lanes)
    return lanes, by_lanes[lanes]


def scan_segment(tokens: int, num_seqs: int) -> int:
    """Tokens a segment, or 0 for one block a sequence and channel group.  The lengths themselves are on the
    device: a step is cut up when one of its sequences can be long enough for it to pay (a sequence that fits
    one segment costs two launches whose blocks leave at once; measured at 2,048 tokens, 4,096 channels of
    16 states: 453 us in one walk, 186 us in segments of 64 or 128, 199 us in segments of 256)."""
    if SCAN_SEGMENT <= 0 or tokens - num_seqs < SCAN_SEGMENT_MIN_TOKENS:
        return 0
    return SCAN_SEGMENT


def selective_scan(x: Tensor, dt_lin: Tensor, dt_bias: Tensor, a: Tensor, bc: Tensor, d: Tensor, z: Tensor, state: Tensor,
                   cu_q: Tensor, state_slots: Tensor, *, num_seqs: int) -> Tensor:
    """The selective state-space recurrence, per sequence, channel c and state n, token after token:
    ``dt = softplus(dt_lin[t, c] + dt_bias[c])``, ``S[c, n] <- exp(dt a[c, n]) S[c, n] + dt x[t, c] B[t, n]``,
    ``y[t, c] = (sum_n S[c, n] C[t, n] + d[c] x[t, c]) * silu(z[t, c])``.  x [T, C]; dt_lin float32 [T, C];
    dt_bias, d float32 [C]; a float32 [C, N] (negative); bc float32 [T, >= 2N] (B, then C) and z [T, >= C] with
    any row stride; state float32 [slots, C, N], read at the step's start and written at its end.  Returns
    [T, C] in x's dtype; everything inside is float32."""
    _gpu(x, "x")
    tokens, channels = x.shape
    _gpu(dt_lin, "dt_lin", torch.float32)
    _gpu(dt_bias, "dt_bias", torch.float32)
    _gpu(a, "a", torch.float32)
    _gpu(d, "d", torch.float32)
    _gpu(bc, "bc", torch.float32, contiguous=False)
    _gpu(z, "z", x.dtype, contiguous=False)
    _gpu(state, "state", torch.float32)
    if a.dim() != 2 or a.shape[0] != channels:
        raise KernelError(f"a must be [{channels}, states]")
    states = a.shape[1]
    if dt_lin.shape != (tokens, channels) or dt_bias.shape != (channels,) or d.shape != (channels,):
        raise KernelError("dt_lin must be [T, C], dt_bias and d [C]")
    if state.dim() != 3 or state.shape[1:] != (channels, states):
        raise KernelError(f"state must be [slots, {channels}, {states}], got {tuple(state.shape)}")
    if bc.shape[0] != tokens or z.shape[0] != tokens:
        raise KernelError("bc and z must have one row per token")
    bc_stride = _strided_rows(bc, "bc", 2 * states)
    z_stride = _strided_rows(z, "z", channels)
    _sequences(cu_q, state_slots, num_seqs)
    segment = scan_segment(tokens, num_seqs)
    lanes, per_lane = scan_shape(channels, states, max(num_seqs, -(-tokens // segment)) if segment else num_seqs)
    out = torch.empty((tokens, channels), dtype=x.dtype, device=x.device)
    rows = tokens // segment + num_seqs + 1 if segment else 0
    seg_start = torch.empty((rows, channels, states), dtype=torch.float32, device=x.device) if segment else None
    seg_dt = torch.empty((rows, channels), dtype=torch.float32, device=x.device) if segment else None
    _call("selective_scan", "fe_selective_scan", _ptr(x), c_int(_code(x.dtype)), _ptr(dt_lin), _ptr(dt_bias), _ptr(a), _ptr(bc),
          c_longlong(bc_stride), _ptr(d), _ptr(z), c_longlong(z_stride), _ptr(state), _ptr(cu_q), _ptr(state_slots), _ptr(out),
          c_int(tokens), c_int(num_seqs), c_int(channels), c_int(states), c_int(state.shape[0]), c_int(lanes), c_int(per_lane),
          c_int(segment), _ptr(seg_start), _ptr(seg_dt), c_int(rows), _stream())
    return out
