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

def embed_rows(ids: Tensor, table: Tensor, out: Tensor) -> Tensor:
    """out[t] = float32(table[ids[t]]); ids int32 [T], table [V, H], out float32 [T, H]."""
    _gpu(ids, "ids", torch.int32)
    _gpu(table, "table")
    _gpu(out, "out", torch.float32)
    tokens = ids.numel()
    vocab, hidden = table.shape
    if out.shape != (tokens, hidden):
        raise KernelError(f"out must be [{tokens}, {hidden}], got {tuple(out.shape)}")
    _call("rowwise", "fe_embed_rows", _ptr(ids), _ptr(table), c_int(_code(table.dtype)), _ptr(out),
          c_int(tokens), c_int(hidden), c_int(vocab), _stream())
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
                    max_ctx: int | None = None, splits: int | None = None) -> Tensor:
    """Attention of every query token of a mixed batch over its paged keys.

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
            splits = decode_splits(num_decode, kv_heads, max_ctx if max_ctx is not None else 16 * 4 * 8)
        part_o = part_ml = counters = None
        if splits > 1:
            part_o = torch.empty(num_seqs * kv_heads * splits * groups * head_dim, dtype=torch.float32, device=q.device)
            part_ml = torch.empty(num_seqs * kv_heads * splits * groups * 2, dtype=torch.float32, device=q.device)
            counters = _split_counters(q.device, num_seqs * kv_heads)
        _call("attention_decode", "fe_paged_attention_decode", _ptr(q), c_longlong(q_stride),
              _ptr(key_pages), _ptr(value_pages), _ptr(out), c_longlong(out.stride(0)), _ptr(part_o),
              _ptr(part_ml), _ptr(counters), _ptr(cu_q), _ptr(ctx_len), _ptr(block_table), c_int(block_table.stride(0)),
              c_int(num_seqs), c_int(kv_heads), c_int(groups), c_int(head_dim), c_int(block_size),
              c_int(num_blocks), c_int(window or 0), c_float(scale), c_int(splits), _stream())
    if any_longer and fast_prefill:
        _call("attention_prefill", "fe_paged_attention_prefill", _ptr(q), c_longlong(q_stride),
              _ptr(key_pages), _ptr(value_pages), _ptr(out), c_longlong(out.stride(0)), _ptr(cu_q),
              _ptr(ctx_len), _ptr(block_table), c_int(block_table.stride(0)), c_int(num_seqs),
              c_int(max_q_len), c_int(kv_heads), c_int(groups), c_int(head_dim), c_int(block_size),
              c_int(num_blocks), c_int(window or 0), c_float(scale), c_int(PREFILL_KEY_GROUPS), c_int(PREFILL_ROW_SETS),
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
