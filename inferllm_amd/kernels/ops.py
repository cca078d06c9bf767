"""The kernel library as Python functions over torch tensors.

Every function checks on the host that shapes, dtypes and devices are what its
kernel and launch grid assume, then launches on torch's current HIP stream.
Tensors must live on the GPU: there is no CPU path, and a missing or unbuildable
library raises (`kernels.build.KernelLibraryError`).  Parts call these through the
module (`ops.add_rmsnorm(...)`).

Matrix products: float32 operands always go to the library's own float32 kernel
(plain fused multiply-adds, fixed summation order).  bfloat16 operands go to the
MFMA kernels of this library when the shape fits them (few rows: decoding), and
to the vendor GEMM through `torch.matmul` otherwise, which is where the reference
uses a vendor GEMM too (cublasSgemm, src/kern/gpu/kernel_gpu.cu:420-435).

Five things ride on the products.  `Weight`: a matrix with a second copy in the
kernels' own tile order (`decode_weight`).  `linear_add` / `NormedRows`: the
residual add in the product's epilogue and the RMS norm that follows it taken by
the next product (up to 16 rows).  `linear_planes`: the product of up to 128 rows (from
17, or from fewer where the plan says that pays) with a long thin matrix, K cut into
ranges whose float32 planes `add_rmsnorm` adds.  `linear_rows`, and `qkv_rope_store` and
`gate_up_silu` from 17 rows on (from fewer where the plan says): products of up to 64 (128)
rows with the wide matrices, X shared by a block's waves through LDS, with the rotation and
cache store or the SiLU-multiply in the same kernel (csrc/gemm_rows.hip).
`_planned_matmul`: products of many rows whole or cut along the output columns, as the
current plan's table says for the shape (`kernels.plan`: fixed tables by default, so that
nothing depends on a stopwatch).
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional

import torch

from . import build
from .plan import NEVER_BELOW, Plan, Rules

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}
_ERRORS = {1: "sizes or dtypes the kernel does not take", 2: "the HIP runtime refused the launch",
           3: "the call needs more of the library's own scratch memory than it holds"}


class KernelError(RuntimeError):
    pass


def _lib():
    return build.library()


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"dtype {t.dtype} is not served (float32 and bfloat16 are)") from None


def _p(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current stream of the current device as a handle for the library (every op calls
    this: the raw lookup costs a fraction of `torch.cuda.current_stream()`)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel operands must be on the GPU (there is no CPU path)")
            _need(t.is_contiguous(), "kernel operands must be contiguous")


def _i32(t: Optional[torch.Tensor], n: Optional[int] = None) -> None:
    if t is not None:
        _need(t.dtype == torch.int32, "index tensors must be int32")
        if n is not None:
            _need(t.numel() >= n, f"index tensor has {t.numel()} entries, {n} needed")


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise KernelError(f"{what}: {_ERRORS.get(rc, rc)}")


# ------------------------------------------------------------------ rows
def embed(tokens: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """float32 [T, E] rows of `table` [V, E] at int32 `tokens` [T]."""
    _gpu(tokens, table)
    _i32(tokens)
    _need(table.dim() == 2 and tokens.dim() == 1, "embed: tokens [T], table [V, E]")
    T, (V, E) = tokens.numel(), table.shape
    out = torch.empty((T, E), dtype=torch.float32, device=table.device)
    _check(_lib().illm_embed(_p(tokens), _p(table), _code(table), _p(out), T, E, V, _stream()),
           "embed")
    return out


def add_rmsnorm(x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, row_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMS norm of the float32 residual rows `x` [T, E] after adding `delta` to them.

    Without `row_idx` the sum is written back to `x`.  With `row_idx` only those
    rows are normed (and `x` is left as it is).  `delta` may be [S, T, E]: the planes of a
    product whose K was split (`linear_planes`), added in order.
    """
    _gpu(x, delta, weight, row_idx)
    _i32(row_idx)
    _need(x.dtype == torch.float32 and x.dim() == 2, "add_rmsnorm: x must be float32 [T, E]")
    T, E = x.shape
    _need(weight.shape == (E,), f"add_rmsnorm: weight {tuple(weight.shape)} for width {E}")
    planes = 1
    if delta is not None:
        if delta.dim() == 3:
            planes = delta.shape[0]
            _need(planes >= 1 and E % 4 == 0, "add_rmsnorm: planes need a width that is a multiple of 4")
        _need(delta.shape[-2:] == x.shape, "add_rmsnorm: delta must have x's shape")
    rows = T if row_idx is None else row_idx.numel()
    out = torch.empty((rows, E), dtype=out_dtype, device=x.device)
    _check(_lib().illm_add_rmsnorm(
        _p(x), _p(delta), _code(delta) if delta is not None else 0, planes,
        ctypes.c_size_t(T * E), _p(weight), _code(weight),
        _p(out), _code(out), _p(row_idx), rows, E, ctypes.c_float(eps), _stream()), "add_rmsnorm")
    return out


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up from rows [gate (F) | up (F)]."""
    _gpu(gate_up)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "silu_mul: rows of [gate | up]")
    T, F2 = gate_up.shape
    out = torch.empty((T, F2 // 2), dtype=gate_up.dtype, device=gate_up.device)
    _check(_lib().illm_silu_mul(_p(gate_up), _p(out), _code(gate_up), T, F2 // 2, _stream()),
           "silu_mul")
    return out


def rope_store(qkv: torch.Tensor, cos_sin: Optional[torch.Tensor], rot: int, pairing: int,
               row_pos: torch.Tensor, row_slot: Optional[torch.Tensor],
               slot_len: Optional[torch.Tensor], kcache: Optional[torch.Tensor],
               vcache: Optional[torch.Tensor], page_table: Optional[torch.Tensor],
               page_size: int, ring: int, nh: int, nkv: int, hd: int) -> None:
    """Rotate q and k of packed rows in place; store k and v in the paged cache.

    qkv [T, (nh + 2 nkv) hd]; cos_sin float32 [max_pos, rot/2, 2] or None (no rotation);
    kcache / vcache [pages, nkv, page_size, hd] or None (nothing stored);
    page_table int32 [slots, pages per sequence].
    """
    _gpu(qkv, cos_sin, row_pos, row_slot, slot_len, kcache, vcache, page_table)
    _i32(row_pos, qkv.shape[0]); _i32(row_slot, qkv.shape[0]); _i32(slot_len); _i32(page_table)
    T = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] == (nh + 2 * nkv) * hd,
          f"rope_store: rows of {qkv.shape[1]} for {nh}+2*{nkv} heads of {hd}")
    max_pos = 0
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 3 and
              cos_sin.shape[1] * 2 == rot and cos_sin.shape[2] == 2,
              "rope_store: angle table must be float32 [max_pos, rot/2, 2]")
        max_pos = cos_sin.shape[0]
    stride = 1
    if kcache is not None:
        _need(vcache is not None and page_table is not None and row_slot is not None,
              "rope_store: a cache needs vcache, page_table and row_slot")
        _need(kcache.dtype == qkv.dtype and vcache.dtype == qkv.dtype,
              "rope_store: cache dtype differs from the activations'")
        _need(kcache.shape[1:] == (nkv, page_size, hd) and vcache.shape == kcache.shape,
              f"rope_store: cache shape {tuple(kcache.shape)} vs (pages, {nkv}, {page_size}, {hd})")
        _need(page_table.dim() == 2, "rope_store: page_table [slots, pages]")
        stride = page_table.shape[1]
    _check(_lib().illm_rope_store(
        _p(qkv), _code(qkv), _p(cos_sin), max_pos, rot, pairing, _p(row_pos), _p(row_slot),
        _p(slot_len), _p(kcache), _p(vcache), _p(page_table), stride, page_size, ring, T, nh, nkv,
        hd, _stream()), "rope_store")


# ------------------------------------------------------------------ products
def gemm_generic(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """x [M, K] . w [N, K]^T by the library's float32 multiply-add kernel."""
    _gpu(x, w)
    _need(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1],
          f"linear: x {tuple(x.shape)} against w {tuple(w.shape)}")
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _check(_lib().illm_gemm_generic(_p(x), _code(x), _p(w), _code(w), _p(y), _code(y), M, N, K,
                                    _stream()), "gemm_generic")
    return y


def gemm_f32_mfma_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.dtype == torch.float32 and w.dtype == torch.float32 and x.dim() == 2 and w.dim() == 2
            and x.shape[0] >= 1 and x.shape[1] == w.shape[1] and x.shape[1] % 16 == 0
            and x.is_contiguous() and w.is_contiguous())


def gemm_f32_mfma(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """x [M, K] . w [N, K]^T, both float32, on the matrix cores' float32 instruction (float32
    operands, products and sums; no shorter type anywhere).  For many rows."""
    _gpu(x, w)
    _need(gemm_f32_mfma_fits(x, w), "gemm_f32_mfma: operands not taken")
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _check(_lib().illm_gemm_f32_mfma(_p(x), _p(w), _p(y), _code(y), M, N, K, _stream()),
           "gemm_f32_mfma")
    return y


class Weight:
    """A matrix [N, K] of a product with, optionally, a second copy laid out for the few-rows
    kernels (`tile_weight`).  Wherever the ops take a weight they take this or a plain tensor."""
    __slots__ = ("plain", "tiled", "mode")

    def __init__(self, plain: torch.Tensor, tiled: Optional[torch.Tensor] = None, mode: str = "plain"):
        # mode: which kernel's tiles the copy follows (`tile_rows`); only that kernel may read it
        self.plain, self.tiled, self.mode = plain, tiled, mode

    @property
    def shape(self):
        return self.plain.shape

    @property
    def dtype(self):
        return self.plain.dtype


def _w(w, mode: str = "plain"):
    """(plain tensor, pointer of the tiled copy or None) of a weight argument, for the kernel
    whose tiles are `mode`; a copy made for another kernel's tiles is not used."""
    if isinstance(w, Weight):
        return w.plain, (_p(w.tiled) if w.tiled is not None and w.mode == mode else None)
    return w, None


def plain_weight(w) -> torch.Tensor:
    return w.plain if isinstance(w, Weight) else w


def tile_rows(N: int, mode: str = "plain", nh: int = 0, nkv: int = 0, hd: int = 0) -> torch.Tensor:
    """Row numbers (int64 [tiles, 16], -1 = a zero row) of the tiles the few-rows kernels work on.
    "plain": 16 consecutive rows.  "gate_up" (N = 2F rows [gate | up]): 8 gate rows and the same
    8 up rows.  "qkv" (rows [q heads | k heads | v heads]): 8 rows of a q or k head and their
    rotation partners hd/2 further, then 16 consecutive rows of v."""
    if mode == "plain":
        t = torch.arange(((N + 15) // 16) * 16).view(-1, 16)
        return torch.where(t < N, t, torch.full_like(t, -1))
    if mode == "gate_up":
        F = N // 2
        lo = torch.arange(((F + 7) // 8) * 8).view(-1, 8)
        ok = lo < F
        return torch.cat([torch.where(ok, lo, torch.full_like(lo, -1)),
                          torch.where(ok, lo + F, torch.full_like(lo, -1))], dim=1)
    if mode == "qkv":
        heads = torch.arange(nh + nkv).view(-1, 1, 1) * hd
        j = torch.arange(hd // 16).view(1, -1, 1) * 8
        i = torch.arange(8).view(1, 1, -1)
        lo = (heads + j + i).view(-1, 8)
        rot = torch.cat([lo, lo + hd // 2], dim=1)
        v = ((nh + nkv) * hd + torch.arange(nkv * hd)).view(-1, 16)
        return torch.cat([rot, v], dim=0)
    raise ValueError(f"unknown tile mode {mode!r}")


def tile_weight(w: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    """The copy [tiles][K / 32][16][32] of w [N, K] for the given tiles of rows (K % 32 == 0)."""
    N, K = w.shape
    _need(K % 32 == 0 and w.dtype == torch.bfloat16, "tile_weight: bfloat16 with K a multiple of 32")
    rows = rows.to(w.device)
    picked = w[rows.clamp(min=0).view(-1)]
    picked[(rows < 0).view(-1)] = 0
    return picked.view(rows.shape[0], 16, K // 32, 32).permute(0, 2, 1, 3).contiguous()


def decode_weight(w: torch.Tensor, mode: str = "plain", copies=False, **geometry):
    """The weight as the parts keep it: with a tiled copy for the few-rows kernels if the engine
    asked for decode copies and the matrix allows it, else the tensor itself.  `copies`: False,
    True (of every matrix) or "thin" (only of matrices with K >= 2 N, the down projections:
    where the vendor GEMM is weakest at 17 to 64 rows and `linear_planes` needs the copy; for
    models whose copies do not all fit)."""
    if (copies and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] % 32 == 0
            and w.is_cuda and (mode != "qkv" or geometry.get("hd", 0) % 16 == 0)
            and (copies != "thin" or (mode == "plain" and w.shape[1] >= 2 * w.shape[0]))):
        return Weight(w, tile_weight(w, tile_rows(w.shape[0], mode, **geometry)), mode)
    return w


class NormedRows:
    """Residual rows whose RMS norm the next product takes itself (few rows, bfloat16).

    Left by `linear_add(..., norm=)`: `x` the float32 residual rows (the sum already in them),
    `xb` = bfloat16(x * weight), `ssq[m][p]` partial sums of x^2.  A product of few rows reads
    `xb` and scales row m of its result by 1 / sqrt(sum_p ssq[m][p] / K + eps), which is the
    product of the normed rows since the scale is common to a row; anything else asks `rows()`
    for the normed rows."""

    def __init__(self, x: torch.Tensor, weight: torch.Tensor, eps: float, act_dtype: torch.dtype,
                 xb: torch.Tensor, ssq: torch.Tensor):
        self.x, self.weight, self.eps, self.dtype = x, weight, float(eps), act_dtype
        self.xb, self.ssq = xb, ssq
        self.shape = x.shape
        self._rows: Optional[torch.Tensor] = None

    def rows(self) -> torch.Tensor:
        if self._rows is None:
            self._rows = add_rmsnorm(self.x, None, self.weight, self.eps, self.dtype)
        return self._rows

    def made_for(self, weight: torch.Tensor, eps: float) -> bool:
        return weight is self.weight and float(eps) == self.eps


def _operand(x):
    """(tensor the kernel reads, ssq pointer, parts, eps) of a few-rows product's input."""
    if isinstance(x, NormedRows):
        return x.xb, _p(x.ssq), x.ssq.shape[1], ctypes.c_float(x.eps)
    return x, None, 0, ctypes.c_float(0.0)


GEMV_F32_MAX_ROWS = 128    # up to here 16 rows at a time, W read once for each 16, beat the
                           # multiply-add tile, whose blocks each walk all of K (measured at the
                           # 7B shape: a decode step of 64 rows 146 -> 45 ms); where K is a
                           # multiple of 32 `gemm_rows_f32_mfma` takes these rows instead


def gemv_rows_f32_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.dtype == torch.float32 and w.dtype == torch.float32 and x.dim() == 2 and w.dim() == 2
            and 1 <= x.shape[0] <= GEMV_F32_MAX_ROWS and x.shape[1] % 4 == 0
            and x.shape[1] == w.shape[1] and x.is_contiguous() and w.is_contiguous())


def gemv_rows_f32(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """x [M <= 128, K] . w [N, K]^T, both float32, plain float32 multiply-adds, W read once for
    every 16 rows.  A row's sum does not depend on the other rows or on their number."""
    _gpu(x, w)
    _need(gemv_rows_f32_fits(x, w), "gemv_rows_f32: operands not taken")
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    for m0 in range(0, M, 16):
        rows = min(16, M - m0)
        _check(_lib().illm_gemv_rows_f32(_p(x[m0:m0 + rows]), _p(w), _p(y[m0:m0 + rows]), _code(y),
                                         rows, N, K, _stream()), "gemv_rows_f32")
    return y


ROWS_F32_MFMA_FROM = 9     # measured streaming over many matrices of the 7B shapes: up to 8 rows
                           # `gemv_rows_f32` reads W at 4.5 to 5.5 TB/s against 3.2 to 4.0; at 16 rows
                           # it is 2.4 to 2.9 against 3.1 to 3.4, at 64 rows 0.7 against 1.4 to 1.8


def gemm_rows_f32_mfma_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.dtype == torch.float32 and w.dtype == torch.float32 and x.dim() == 2 and w.dim() == 2
            and 1 <= x.shape[0] <= 128 and x.shape[1] % 32 == 0
            and x.shape[1] == w.shape[1] and x.is_contiguous() and w.is_contiguous())


def gemm_rows_f32_mfma(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """x [M <= 128, K] . w [N, K]^T, both float32, W read once, on the matrix cores' float32
    instruction.  A row's sum does not depend on the other rows or on their number."""
    _gpu(x, w)
    _need(gemm_rows_f32_mfma_fits(x, w), "gemm_rows_f32_mfma: operands not taken")
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _check(_lib().illm_gemm_rows_f32_mfma(_p(x), _p(w), _p(y), _code(y), M, N, K, _stream()),
           "gemm_rows_f32_mfma")
    return y


def linear_add_fits(x, w, into: torch.Tensor) -> bool:
    """Whether `linear_add` takes these operands (few bfloat16 rows into float32 rows)."""
    w = plain_weight(w)
    return (isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and x.dim() == 2 and w.dim() == 2 and into.dtype == torch.float32 and
            into.is_contiguous() and 1 <= x.shape[0] <= SKINNY_BEST_ROWS and x.shape[1] % 8 == 0
            and w.shape[1] == x.shape[1] and into.shape == (x.shape[0], w.shape[0]))


def linear_add(x: torch.Tensor, w, into: torch.Tensor, norm=None,
               act_dtype: torch.dtype = torch.bfloat16) -> Optional[NormedRows]:
    """into += x . w^T in the product's kernel: the residual add of a block's output projection,
    each element added by the one thread that owns it.  norm = (weight [N], eps) of the RMS norm
    that follows: the kernel also leaves what the next few-rows product needs to take that norm
    itself, returned as `NormedRows` (only if N % 8 == 0, else None as without `norm`)."""
    _need(linear_add_fits(x, w, into), "linear_add: operands not taken")
    w, wt = _w(w)
    _gpu(x, w, into)
    M, K = x.shape
    N = w.shape[0]
    if norm is not None and (N % 8 or norm[0].dtype not in _CODES or act_dtype != torch.bfloat16
                             or norm[0].shape != (N,)):
        norm = None
    if norm is None:
        _check(_lib().illm_gemm_skinny_add(_p(x), _p(w), wt, _p(into), M, N, K, None, BF16, None,
                                           None, PLAIN_WAVES, _stream()), "linear_add")
        return None
    weight, eps = norm
    _gpu(weight)
    xb = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    ssq = torch.empty((M, (N + 15) // 16), dtype=torch.float32, device=x.device)
    _check(_lib().illm_gemm_skinny_add(_p(x), _p(w), wt, _p(into), M, N, K, _p(weight),
                                       _code(weight), _p(xb), _p(ssq), PLAIN_WAVES, _stream()),
           "linear_add")
    return NormedRows(into, weight, eps, act_dtype, xb, ssq)


MID_MAX_ROWS = 128       # rows a launch of csrc/gemm_mid.hip takes (a limit of the kernel; the break-even
                         # points of the ways are the plan's: `kernels.plan.Rules` and its tables)

# The tables that products with more than one way are dispatched by (`kernels.plan`).  An engine
# makes its own current at the start of each of its steps; nothing is timed unless the plan asks.
_plan: Plan = Plan.fixed()


def use_plan(plan: Plan) -> None:
    global _plan
    _plan = plan


def current_plan() -> Plan:
    return _plan


def linear_planes_fits(x, w) -> bool:
    """Whether `linear_planes` takes these operands: up to 128 bfloat16 rows and a matrix with a
    decode copy in plain tile order that has few rows for its length (K >= 2 N; from 17 rows on
    K >= N)."""
    return (isinstance(w, Weight) and w.tiled is not None and w.mode == "plain"
            and isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16 and x.dim() == 2
            and 1 <= x.shape[0] <= MID_MAX_ROWS and x.shape[1] == w.plain.shape[1]
            and w.plain.shape[0] % 4 == 0 and w.plain.shape[0] <= _plan.rules.planes_most_cols
            and w.plain.shape[1] >= (2 if x.shape[0] <= SKINNY_BEST_ROWS else 1) * w.plain.shape[0])


_flush: Dict[int, torch.Tensor] = {}


def _flush_buffer() -> torch.Tensor:
    """512 MB of zeros on the current device, larger than its last-level cache; kept while the
    process measures (a plan that measures nothing never asks for it)."""
    dev = torch.cuda.current_device()
    if dev not in _flush:
        _flush[dev] = torch.zeros(1 << 28, dtype=torch.int16, device=dev)
    return _flush[dev]


def _cold_time(fn, reps: int = 5) -> float:
    """Median milliseconds of `fn` with the last-level cache flushed before every run: a decode
    step streams gigabytes between two uses of a matrix, so its products always run cold, and a
    matrix of tens of megabytes timed back to back would be served from the cache.  The flush
    reads: after a fill the cache is full of lines to be written back, which costs a kernel
    whose loads allocate in it tens of microseconds that it does not pay in a step (measured
    against streaming over many copies of a matrix, which the reading flush agrees with)."""
    flush = _flush_buffer()
    fn()
    times = []
    for _ in range(reps):
        flush.sum()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        end.synchronize()
        times.append(start.elapsed_time(end))
    return sorted(times)[len(times) // 2]


def measure_planes_from(w: "Weight") -> int:
    """Fewest rows from which `linear_planes` and the norm that adds its planes take less time
    than `linear_add` (whose norm the next product takes), measured at 16, 12, 8 and 4 rows."""
    N, K = w.plain.shape
    if N * K < _plan.rules.planes_min_elements:
        return NEVER_BELOW
    dev = w.plain.device
    x = torch.zeros((SKINNY_BEST_ROWS, K), dtype=torch.bfloat16, device=dev)
    into = torch.zeros((SKINNY_BEST_ROWS, N), dtype=torch.float32, device=dev)
    nw = torch.ones(N, dtype=torch.bfloat16, device=dev)

    timed = _cold_time

    first = NEVER_BELOW
    for rows in (16, 12, 8, 4):
        xs, dst = x[:rows], into[:rows]
        t_add = timed(lambda: linear_add(xs, w, dst, (nw, 1e-5)))
        t_planes = timed(lambda: add_rmsnorm(dst, linear_planes(xs, w), nw, 1e-5, torch.bfloat16))
        if t_planes >= 0.97 * t_add:              # the planes have to pay clearly
            break
        first = rows - 3
    return first


def tune_product(plan: Plan, kind: str, w, votes: int = 1, **geometry) -> Optional[tuple]:
    """Time what the plan's tables lack for one product a part lists (`Part.tunables`) and enter
    it: for a thin "plain" matrix from how few rows the planes pay, for a fused "qkv" or
    "gate_up" matrix from how few rows the kernels that share X do.  The median of `votes`
    measurements.  Returns (table, key, value) of the new entry, or None if nothing was timed
    (no decode copy, a shape the kernels do not take, an entry that is there)."""
    if not (isinstance(w, Weight) and w.tiled is not None and w.mode == kind):
        return None
    N, K = w.shape
    if kind == "plain":
        key, table = (N, K), plan.planes_from
        fits = K >= 2 * N and N <= plan.rules.planes_most_cols and N % 4 == 0
        measure = lambda: measure_planes_from(w)
    elif kind == "qkv":
        key, table = ("qkv", N, K), plan.rows_from
        fits = K % 64 == 0
        measure = lambda: measure_rows_from_qkv(w, geometry["nh"], geometry["nkv"], geometry["hd"])
    elif kind == "gate_up":
        key, table = ("gate_up", N, K), plan.rows_from
        fits = K % 64 == 0
        measure = lambda: measure_rows_from_gate_up(w)
    else:
        raise ValueError(f"unknown kind of product {kind!r}")
    if not fits or key in table:
        return None
    saved, current = _plan, plan
    use_plan(current)
    try:
        runs = sorted(measure() for _ in range(max(1, votes)))
    finally:
        use_plan(saved)
    table[key] = runs[len(runs) // 2]
    return ("planes_from" if kind == "plain" else "rows_from"), key, table[key]


def linear_planes_pays(x, w) -> bool:
    """Whether the planes are the faster way for these operands (which `linear_planes_fits`).
    From 17 to 64 rows always.  Up to 16 rows `linear_add` reads X once per
    block of W rows, so its time grows with the rows, and a matrix whose tiles do not fill the
    chip evenly is slow at any (measured: LLaMA-2-7B's down projection 23.3 against 21.7 us at
    16 rows, the 70B's 105 against 77, a 5120 x 13824 one 34 against 30 at 4 rows): by the
    plan's table; a plan that measures times a shape it lacks once, outside graph capture."""
    rows = x.shape[0]
    if rows > SKINNY_BEST_ROWS:
        # (65 to 128 rows, one launch, product and the norm that adds its planes against the
        # vendor GEMM and its norm: the 7B down projection 28 to 33 us against 38 to 64, the 70B
        # one 86 to 101 against 134 to 221, 4096 x 4096 18 to 22 against 20 to 29; 17 to 64 rows
        # of 4096 x 4096 15 to 18 against 17 to 19, of 5120 x 5120 17 to 22 against 21 to 31)
        return True
    key = tuple(w.plain.shape)
    first = _plan.planes_from.get(key)
    if first is None:
        if not _plan.measure or torch.cuda.is_current_stream_capturing():
            return rows >= NEVER_BELOW
        first = _plan.planes_from[key] = measure_planes_from(w)
    return rows >= first


def linear_planes(x: torch.Tensor, w: "Weight", splits: int = 0) -> torch.Tensor:
    """x . w^T as float32 planes [S, M, N] whose sum over S is the product: K is cut into S
    ranges so that a matrix with few rows fills the chip (csrc/gemm_mid.hip).  The planes go to
    `add_rmsnorm` as `delta`, which adds them in order."""
    _need(linear_planes_fits(x, w), "linear_planes: operands not taken")
    x = x.contiguous()
    _gpu(x, w.plain)
    M, K = x.shape
    N = w.plain.shape[0]
    S = splits or _lib().illm_gemm_mid_splits(N, K)
    y = torch.empty((S, M, N), dtype=torch.float32, device=x.device)
    _check(_lib().illm_gemm_mid_bf16(_p(x), _p(w.tiled), _p(y), F32, M, N, K, S, _stream()),
           "linear_planes")
    return y


def linear(x, w, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """y = x . w^T, w stored [out, in] (src/kern/naive/naive.cpp:363-379).  x may be
    `NormedRows`, w a `Weight`."""
    if isinstance(x, NormedRows):
        if w.dtype == torch.bfloat16:
            return gemm_skinny_bf16(x, w, out_dtype or x.dtype)
        x = x.rows()
    out_dtype = out_dtype or x.dtype
    if (isinstance(w, Weight) and out_dtype == torch.float32 and rows_fits(x, w, "plain")
            and x.shape[0] >= rows_from("plain", w)):
        return linear_rows(x, w, out_dtype)              # logits of 17 to 128 rows
    if isinstance(w, Weight) and not (x.dtype == torch.bfloat16 and 1 <= x.shape[0] <= SKINNY_BEST_ROWS):
        w = w.plain                                      # only the few-rows kernel reads the copy
    if x.dtype == torch.float32 or w.dtype == torch.float32:
        if x.shape[0] >= ROWS_F32_MFMA_FROM and gemm_rows_f32_mfma_fits(x, w):
            return gemm_rows_f32_mfma(x, w, out_dtype)
        if gemv_rows_f32_fits(x, w):
            return gemv_rows_f32(x, w, out_dtype)
        if gemm_f32_mfma_fits(x, w):
            return gemm_f32_mfma(x, w, out_dtype)
        return gemm_generic(x, w, out_dtype)
    M, K = x.shape
    if M == 0:
        return torch.empty((0, w.shape[0]), dtype=out_dtype, device=x.device)
    if skinny_fits(M, w.shape[0], K) and (M <= SKINNY_BEST_ROWS or out_dtype == torch.float32):
        return gemm_skinny_bf16(x, w, out_dtype)
    if out_dtype == torch.float32 and K % 8 == 0:
        # float32 results (logits) keep the accumulator's precision: 64 rows at a time
        return torch.cat([gemm_skinny_bf16(x[i:i + SKINNY_MAX_ROWS], w, out_dtype)
                          for i in range(0, M, SKINNY_MAX_ROWS)], dim=0)
    if out_dtype == torch.float32:
        return gemm_generic(x, w, out_dtype)
    _gpu(x, w)
    return _planned_matmul(x, w)


# The vendor GEMM's own choice of kernel is now and then a poor one for a shape (measured on
# MI355X: 2048 x 22016 x 4096 takes 408 us whole and 253 us as 8192 + 13824 columns; most shapes
# gain nothing).  So products of many rows are planned per shape: the whole product or a cut of
# the output columns, each part written into its slice of one result, as the current plan's
# table says (`kernels.plan`; a plan that measures times the candidates for a shape it lacks).
# Every output element is still one kernel's sum; plans differ in rounding only.
# (from how many rows and columns a cut or a filling-up is a candidate: `kernels.plan.Rules`)


def _split_candidates(N: int, M: int = 0):
    """Plans to measure: () whole, (c,) cut of the output columns at c, ("rows", n) the rows in n
    equal parts (2048 x 12288 x 4096 runs 6 % faster as two products of 1024 rows)."""
    cuts = {(N // 8192) * 8192, (N // 4096) * 4096, (N // 2 // 256) * 256, 8192, 12288, 16384,
            ((2 * N // 3) // 4096) * 4096, ((3 * N // 4) // 4096) * 4096}
    plans = [()] + [(c,) for c in sorted(cuts) if 2048 <= c <= N - 1024]
    if M >= 2048 and M % 512 == 0:
        plans.append(("rows", 2))
    return plans


def _run_plan(x: torch.Tensor, w: torch.Tensor, plan, out: Optional[torch.Tensor] = None):
    if not plan:
        return torch.matmul(x, w.t(), out=out) if out is not None else torch.matmul(x, w.t())
    if plan[0] == "pad":
        # rows filled up to plan[1]; what the added rows hold does not matter, rows are independent
        xp = torch.empty((plan[1], x.shape[1]), dtype=x.dtype, device=x.device)
        xp[:x.shape[0]].copy_(x)
        y = torch.matmul(xp, w.t())[:x.shape[0]]
        if out is not None:
            out.copy_(y)
            return out
        return y
    if out is None:
        out = torch.empty((x.shape[0], w.shape[0]), dtype=x.dtype, device=x.device)
    if plan[0] == "rows":
        step = x.shape[0] // plan[1]
        for a in range(0, x.shape[0], step):
            torch.matmul(x[a:a + step], w.t(), out=out[a:a + step])
        return out
    edges = (0,) + tuple(plan) + (w.shape[0],)
    for a, b in zip(edges[:-1], edges[1:]):
        torch.matmul(x, w[a:b].t(), out=out[:, a:b])
    return out


def measure_plan(x: torch.Tensor, w: torch.Tensor, candidates=None, margin: float = 0.97):
    """The fastest of the candidate plans for x . w^T; a plan replaces the best so far only if
    it takes less than `margin` of its time (a cut has to pay clearly)."""
    out = torch.empty((x.shape[0], w.shape[0]), dtype=x.dtype, device=x.device)
    best, best_t = (), None
    for plan in candidates or _split_candidates(w.shape[0], x.shape[0]):
        # cold, as in a step, where gigabytes pass between two uses of a matrix: run back to
        # back on one matrix the whole product of 2048 x 12288 x 4096 looks as fast as its cut
        # at 8192 columns, over matrices that come from memory it takes 193 against 159 us
        t = _cold_time(lambda: _run_plan(x, w, plan, out), reps=3)
        if best_t is None or t < margin * best_t:
            best, best_t = plan, t
    return best


def _planned_matmul(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    M, K = x.shape
    N = w.shape[0]
    capturing = torch.cuda.is_current_stream_capturing()
    rules = _plan.rules
    if rules.pad_rows_above < M < rules.pad_rows_to:
        # the vendor GEMM takes 65 to 255 rows of some shapes slower than 256 (measured: 4096 x
        # 11008 at 192 rows 82 us, at 256 rows 51): whole or filled up to 256, per shape and
        # 32 rows
        key = ("pad", -(-M // 32), N, K)
        plan = _plan.cuts.get(key)
        if plan is None:
            if not _plan.measure or capturing:
                return torch.matmul(x, w.t())
            plan = _plan.cuts[key] = measure_plan(x, w, [(), ("pad", rules.pad_rows_to)])
        return _run_plan(x, w, plan)
    if M < rules.cut_min_rows or N < rules.cut_min_cols:
        return torch.matmul(x, w.t())
    key = (-(-M // 256), N, K)
    plan = _plan.cuts.get(key)
    if plan is None:
        if not _plan.measure or capturing:
            return torch.matmul(x, w.t())
        plan = _plan.cuts[key] = measure_plan(x, w)
    if plan and plan[0] == "rows" and M % (256 * plan[1]):
        plan = ()                                # measured at the class's full size; M is ragged
    return _run_plan(x, w, plan)


ROWS_MAX = 128           # rows the products of csrc/gemm_rows.hip take, all in one launch (a limit of
                         # the kernel; measured against the vendor GEMM with the elementwise kernel
                         # behind it at 80 / 96 / 128 rows: gate|up of the 7B shape 39 / 40 / 44 against
                         # 50 / 50 / 49 us, of the 8B shape 46 / 48 / 52 against 73 / 59 / 61; in two
                         # launches of 64 rows they lost)


def rows_from(mode: str, w) -> int:
    """Fewest rows from which the product with `w` in tile order `mode` goes to
    csrc/gemm_rows.hip: the plan's entry for the shape, else the plan's rule."""
    return _plan.rows_from.get((mode,) + tuple(w.shape), _plan.rules.rows_from)


def rows_most(mode: str, w) -> int:
    """Most rows for which it does: the plan's entry for the shape, else all a launch takes."""
    return min(ROWS_MAX, _plan.rows_most.get((mode,) + tuple(w.shape), ROWS_MAX))


def rows_fits(x, w, mode: str) -> bool:
    """Whether the products of csrc/gemm_rows.hip take these operands: bfloat16 rows (or
    `NormedRows`, up to 16) and a weight with a decode copy in `mode`'s tile order."""
    xt = x.xb if isinstance(x, NormedRows) else x
    if not (isinstance(w, Weight) and w.tiled is not None and w.mode == mode):
        return False
    most = 16 if isinstance(x, NormedRows) else rows_most(mode, w)
    return (isinstance(w, Weight) and w.tiled is not None and w.mode == mode
            and isinstance(xt, torch.Tensor) and xt.dtype == torch.bfloat16 and xt.dim() == 2
            and 1 <= xt.shape[0] <= most
            and xt.shape[1] == w.plain.shape[1] and xt.shape[1] % 64 == 0)


def linear_rows(x, w: "Weight", out_dtype: torch.dtype) -> torch.Tensor:
    """x [M <= 128, K] . w^T from the plain decode copy, X shared by a block's waves through LDS
    and K cut inside the block: the product of 17 to 128 rows with a wide matrix."""
    _need(rows_fits(x, w, "plain"), "linear_rows: operands not taken")
    xt, ssq, parts, eps = _operand(x)
    xt = xt.contiguous()
    _gpu(xt, w.tiled)
    M, K = xt.shape
    N = w.plain.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=xt.device)
    _check(_lib().illm_gemm_rows_bf16(_p(xt), _p(w.tiled), _p(y), _code(y), M, N, K, ssq, parts,
                                      eps, _stream()), "linear_rows")
    return y


SKINNY_MAX_ROWS = 64     # rows the few-rows kernel takes
SKINNY_BEST_ROWS = 16    # up to here it beats the vendor GEMM (measured at the 7B shapes)


def skinny_fits(M: int, N: int, K: int) -> bool:
    """Shapes the few-rows MFMA kernel takes (csrc/gemm_skinny.hip)."""
    return 1 <= M <= SKINNY_MAX_ROWS and K % 8 == 0


def gemm_skinny_bf16(x, w, out_dtype: torch.dtype) -> torch.Tensor:
    """x [M <= 64, K] . w [N, K]^T, both bfloat16, float32 accumulation on the matrix cores; or
    x `NormedRows`: the product of the normed rows."""
    xt, ssq, parts, eps = _operand(x)
    w, wt = _w(w)
    _gpu(xt, w)
    _need(xt.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny: bfloat16 operands")
    _need(xt.dim() == 2 and w.dim() == 2 and xt.shape[1] == w.shape[1],
          f"linear: x {tuple(xt.shape)} against w {tuple(w.shape)}")
    M, K = xt.shape
    N = w.shape[0]
    _need(skinny_fits(M, N, K), f"gemm_skinny: M={M} K={K} not taken")
    y = torch.empty((M, N), dtype=out_dtype, device=xt.device)
    _check(_lib().illm_gemm_skinny_bf16(_p(xt), _p(w), wt, _p(y), _code(y), M, N, K, ssq, parts,
                                        eps, PLAIN_WAVES, _stream()), "gemm_skinny")
    return y


QKV_ROPE_WAVES = 0       # waves per block of the fused kernel; 0: the kernel's own choice
GATE_UP_WAVES = 0        # the same for the fused gate|up product
PLAIN_WAVES = 0          # and for the plain few-rows product


def qkv_rope_store_fits(x, w_qkv, hd: int) -> bool:
    """Whether the one-kernel q|k|v product + rotation + cache store takes these operands: up to
    16 rows always, up to 128 (96 for small matrices) with a decode copy of the matrix in q|k|v
    tile order."""
    if not (x.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16 and hd % 16 == 0):
        return False
    if 1 <= x.shape[0] <= SKINNY_BEST_ROWS and x.shape[1] % 8 == 0:
        return True
    return rows_fits(x, w_qkv, "qkv")


def measure_rows_from_gate_up(w_gate_up: "Weight") -> int:
    """Fewest rows (1, 5, 9, 13 or 17) from which the fused gate|up product of csrc/gemm_rows.hip
    takes less time than the few-rows one (for the tuner; times both at 16, 12, 8 and 4 rows)."""
    F2, K = w_gate_up.plain.shape
    x = torch.zeros((16, K), dtype=torch.bfloat16, device=w_gate_up.plain.device)
    saved, key = dict(_plan.rows_from), ("gate_up", F2, K)

    def timed(rows: int, threshold: int) -> float:
        _plan.rows_from[key] = threshold
        return _cold_time(lambda: gate_up_silu(x[:rows], w_gate_up))

    first = _plan.rules.rows_from
    try:
        for rows in (16, 12, 8, 4):
            if timed(rows, 1) >= 0.97 * timed(rows, _plan.rules.rows_from):
                break
            first = rows - 3
    finally:
        _plan.rows_from.clear()
        _plan.rows_from.update(saved)
    return first


def measure_rows_from_qkv(w_qkv: "Weight", nh: int, nkv: int, hd: int) -> int:
    """Fewest rows (1, 5, 9, 13 or 17) from which the fused q|k|v product of csrc/gemm_rows.hip
    takes less time than the few-rows one (for the tuner; times both at 16, 12, 8 and 4 rows)."""
    N, K = w_qkv.plain.shape
    dev = w_qkv.plain.device
    x = torch.zeros((16, K), dtype=torch.bfloat16, device=dev)
    table = torch.zeros((16, hd // 2, 2), dtype=torch.float32, device=dev)
    pos = torch.arange(16, dtype=torch.int32, device=dev)
    pages = torch.arange(16, dtype=torch.int32, device=dev).view(16, 1).contiguous()
    kc = torch.zeros((16, nkv, 64, hd), dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    saved, key = dict(_plan.rows_from), ("qkv", N, K)

    def timed(rows: int, threshold: int) -> float:
        _plan.rows_from[key] = threshold
        return _cold_time(lambda: qkv_rope_store(x[:rows], w_qkv, table, pos[:rows], pos[:rows], kc,
                                                 vc, pages, 64, 0, nh, nkv, hd))

    first = _plan.rules.rows_from
    try:
        for rows in (16, 12, 8, 4):
            if timed(rows, 1) >= 0.97 * timed(rows, _plan.rules.rows_from):
                break
            first = rows - 3
    finally:
        _plan.rows_from.clear()
        _plan.rows_from.update(saved)
    return first


def qkv_rope_store(x, w_qkv, cos_sin: torch.Tensor,
                   row_pos: torch.Tensor, row_slot: torch.Tensor, kcache: torch.Tensor,
                   vcache: torch.Tensor, page_table: torch.Tensor, page_size: int, ring: int,
                   nh: int, nkv: int, hd: int) -> torch.Tensor:
    """Decode only: x . Wqkv^T, q and k rotated (pairs (i, i + hd/2), all dims) at row_pos, q
    returned in rows [q | k | v] whose k and v parts are NOT filled, k and v stored in the cache.
    x may be `NormedRows`."""
    xt, ssq, parts, eps = _operand(x)
    _need(qkv_rope_store_fits(x, w_qkv, hd), "qkv_rope_store: operands not taken")
    w_qkv, wt = _w(w_qkv, "qkv")
    _gpu(xt, w_qkv, cos_sin, row_pos, row_slot, kcache, vcache, page_table)
    _i32(row_pos, x.shape[0]); _i32(row_slot, x.shape[0]); _i32(page_table)
    M, K = x.shape
    N = (nh + 2 * nkv) * hd
    _need(w_qkv.shape == (N, K), f"qkv_rope_store: weight {tuple(w_qkv.shape)} vs ({N}, {K})")
    _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 3 and cos_sin.shape[1] * 2 == hd and
          cos_sin.shape[2] == 2, "qkv_rope_store: angle table must be float32 [max_pos, hd/2, 2]")
    _need(kcache.dtype == torch.bfloat16 and kcache.shape[1:] == (nkv, page_size, hd) and
          vcache.shape == kcache.shape and vcache.dtype == torch.bfloat16 and page_table.dim() == 2,
          "qkv_rope_store: cache shape or dtype")
    y = torch.empty((M, N), dtype=torch.bfloat16, device=xt.device)
    if wt is not None and K % 64 == 0 and M >= rows_from("qkv", w_qkv):
        _check(_lib().illm_qkv_rope_store_rows(
            _p(xt), wt, _p(y), M, K, _p(cos_sin), cos_sin.shape[0], _p(row_pos), _p(row_slot),
            _p(kcache), _p(vcache), _p(page_table), page_table.shape[1], page_size, ring, nh, nkv,
            hd, ssq, parts, eps, _stream()), "qkv_rope_store (rows)")
        return y
    _check(_lib().illm_qkv_rope_store_skinny(
        _p(xt), _p(w_qkv), wt, _p(y), M, K, _p(cos_sin), cos_sin.shape[0], _p(row_pos), _p(row_slot),
        _p(kcache), _p(vcache), _p(page_table), page_table.shape[1], page_size, ring, nh, nkv, hd,
        ssq, parts, eps, QKV_ROPE_WAVES, _stream()), "qkv_rope_store")
    return y


def gate_up_silu(x, w_gate_up) -> torch.Tensor:
    """silu(x . Wg^T) * (x . Wu^T) for w_gate_up = [Wg | Wu] stacked as [2F, K].

    Few bfloat16 rows: one fused MFMA kernel.  Otherwise the product and `silu_mul`.
    x may be `NormedRows`."""
    if isinstance(x, NormedRows) and (w_gate_up.dtype != torch.bfloat16 or w_gate_up.shape[0] % 2):
        x = x.rows()
    M, K = x.shape
    F2 = w_gate_up.shape[0]
    if F2 % 2 == 0 and rows_fits(x, w_gate_up, "gate_up") and M >= rows_from("gate_up", w_gate_up):
        xt, ssq, parts, eps = _operand(x)
        xt = xt.contiguous()
        _gpu(xt, w_gate_up.tiled)
        y = torch.empty((M, F2 // 2), dtype=x.dtype, device=xt.device)
        _check(_lib().illm_gemm_rows_gateup_silu(_p(xt), _p(w_gate_up.tiled), _p(y), _code(y), M,
                                                 F2 // 2, K, ssq, parts, eps, _stream()),
               "gate_up_silu (rows)")
        return y
    if (x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and F2 % 2 == 0
            and 1 <= M <= SKINNY_BEST_ROWS and K % 8 == 0):
        xt, ssq, parts, eps = _operand(x)
        wp, wt = _w(w_gate_up, "gate_up")
        _gpu(xt, wp)
        _need(wp.dim() == 2 and wp.shape[1] == K, "gate_up_silu: shapes")
        y = torch.empty((M, F2 // 2), dtype=x.dtype, device=xt.device)
        _check(_lib().illm_gemm_skinny_gateup_silu(_p(xt), _p(wp), wt, _p(y), _code(y), M,
                                                   F2 // 2, K, ssq, parts, eps, GATE_UP_WAVES,
                                                   _stream()), "gate_up_silu")
        return y
    if isinstance(x, NormedRows):
        x = x.rows()
    return silu_mul(linear(x, plain_weight(w_gate_up)))


# ------------------------------------------------------------------ attention
def attn_prefill(qkv: torch.Tensor, cu_seqlens: torch.Tensor, n_seqs: int, max_len: int, nh: int,
                 nkv: int, hd: int, scale: float, window: int) -> torch.Tensor:
    """Causal attention of whole prompts over packed rows; returns [T, nh * hd]."""
    _gpu(qkv, cu_seqlens)
    _i32(cu_seqlens, n_seqs + 1)
    T = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] == (nh + 2 * nkv) * hd, "attn_prefill: packed qkv rows")
    _need(nh % nkv == 0, "attn_prefill: heads must be a multiple of kv heads")
    out = torch.empty((T, nh * hd), dtype=qkv.dtype, device=qkv.device)
    if qkv.dtype == torch.bfloat16 and hd % 16 == 0:
        _check(_lib().illm_attn_prefill_bf16(
            _p(qkv), _p(out), _p(cu_seqlens), n_seqs, max_len, nh, nkv, hd,
            ctypes.c_float(scale), window, _stream()), f"attn_prefill_bf16 (head_dim {hd})")
        return out
    _check(_lib().illm_attn_prefill_generic(
        _p(qkv), _p(out), _code(qkv), _p(cu_seqlens), n_seqs, max_len, nh, nkv, hd,
        ctypes.c_float(scale), window, _stream()), f"attn_prefill (head_dim {hd})")
    return out


def attn_prefill_paged(qkv: torch.Tensor, cu_seqlens: torch.Tensor, seq_slot: torch.Tensor,
                       seq_start: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                       page_table: torch.Tensor, page_size: int, ring: int, n_seqs: int,
                       max_len: int, nh: int, nkv: int, hd: int, scale: float,
                       window: int) -> torch.Tensor:
    """Causal attention of a step's packed rows that go on from tokens the cache already holds:
    row r of sequence b stands at position seq_start[b] + r and attends over the keys 0 .. its
    position of the paged cache, which must hold the step's own keys and values too by now.
    `max_len`: the most rows a sequence brings.  Returns [T, nh * hd]."""
    _gpu(qkv, cu_seqlens, seq_slot, seq_start, kcache, vcache, page_table)
    _i32(cu_seqlens, n_seqs + 1); _i32(seq_slot, n_seqs); _i32(seq_start, n_seqs); _i32(page_table)
    T = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] >= nh * hd, "attn_prefill_paged: packed rows [q | ...]")
    _need(nh % nkv == 0, "attn_prefill_paged: heads must be a multiple of kv heads")
    _need(kcache.dtype == qkv.dtype and vcache.shape == kcache.shape and
          kcache.shape[1:] == (nkv, page_size, hd) and page_table.dim() == 2,
          "attn_prefill_paged: cache shape or dtype")
    _need(qkv.shape[1] == (nh + 2 * nkv) * hd, "attn_prefill_paged: packed qkv rows")
    out = torch.empty((T, nh * hd), dtype=qkv.dtype, device=qkv.device)
    if qkv.dtype == torch.bfloat16 and hd % 16 == 0 and page_size % 64 == 0:
        _check(_lib().illm_attn_prefill_paged_bf16(
            _p(qkv), _p(out), _p(cu_seqlens), _p(seq_slot), _p(seq_start), _p(kcache), _p(vcache),
            _p(page_table), page_table.shape[1], page_size, ring, n_seqs, max_len, nh, nkv, hd,
            ctypes.c_float(scale), window, _stream()), f"attn_prefill_paged_bf16 (head_dim {hd})")
        return out
    _check(_lib().illm_attn_prefill_paged_generic(
        _p(qkv), _p(out), _code(qkv), _p(cu_seqlens), _p(seq_slot), _p(seq_start), _p(kcache),
        _p(vcache), _p(page_table), page_table.shape[1], page_size, ring, n_seqs, max_len, nh, nkv,
        hd, ctypes.c_float(scale), window, _stream()), f"attn_prefill_paged (head_dim {hd})")
    return out


def decode_splits(B: int, nkv: int, max_len: int, nh: int = 0, hd: int = 0, ragged: bool = False):
    """(nsplit, waves): how to cut the keys of a decode step among blocks (`nsplit` ranges per
    sequence, combined by a merge kernel) and among the waves of a block (combined in LDS).
    Measured on MI355X at head size 128, 32/32, 32/8 and 64/8 heads, 1 to 64 sequences of 650
    to 4000 keys: about as many blocks as the chip has compute units (256) is best or within a
    microsecond of it, in at most 16 ranges; 8 waves a block (idle ones cost nothing) until
    there are 512 blocks, then 4.  `ragged` (the lengths differ widely, the longest has 1,024
    keys or more): every sequence has the same number of ranges, so the long sequences' blocks
    outlast the others'; the ranges are doubled, up to 8, while that makes no more than 1,024
    blocks (16 sequences of 64 to 4,096 keys, 32/8 heads: 30.5 -> 26.3 us, 32/32 heads: 80 -> 74;
    one of 4,000 among 15 of 200: 27.7 -> 21.7 and 51.5 -> 40.7; beyond 1,024 blocks more ranges
    cost more than they even out: one of 2,000 among 63 of 100, 32/32 heads, 34 us whole, 88 in
    8 ranges)."""
    base = max(1, B * nkv)
    if nh > nkv > 0 and hd % 32 == 0 and 0 < hd <= 128:
        base *= -(-(nh // nkv) // 16)          # the grouped kernel takes 16 heads a block
    tiles = max(1, (max_len + 63) // 64)
    nsplit = max(1, min(-(-256 // base), 16, tiles))
    if ragged and tiles >= 16:
        while nsplit < 8 and base * nsplit * 2 <= 1024:
            nsplit *= 2
    return nsplit, (8 if base * nsplit < 512 else 4)


def attn_decode(qkv: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                page_table: torch.Tensor, page_size: int, ring: int, seq_slot: torch.Tensor,
                seq_len: torch.Tensor, nh: int, nkv: int, hd: int, scale: float, window: int,
                nsplit: int, waves: int = 1) -> torch.Tensor:
    """One new token per sequence against the paged cache; returns [B, nh * hd].
    seq_len[b]: keys of sequence b, the new one included.  The keys of a sequence are cut
    into `nsplit` ranges (blocks, combined by a merge kernel) and each range is shared by
    `waves` waves of a block (combined in LDS; the bfloat16 kernels only)."""
    _gpu(qkv, kcache, vcache, page_table, seq_slot, seq_len)
    _i32(page_table); _i32(seq_slot, qkv.shape[0]); _i32(seq_len, qkv.shape[0])
    B = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] == (nh + 2 * nkv) * hd, "attn_decode: packed qkv rows")
    _need(kcache.dtype == qkv.dtype and vcache.shape == kcache.shape and
          kcache.shape[1:] == (nkv, page_size, hd), "attn_decode: cache shape or dtype")
    _need(nh % nkv == 0, "attn_decode: heads must be a multiple of kv heads")
    out = torch.empty((B, nh * hd), dtype=qkv.dtype, device=qkv.device)
    if qkv.dtype == torch.bfloat16 and hd % 8 == 0 and page_size % 64 == 0:
        partial = (torch.empty((B, nh, nsplit, hd + 2), dtype=torch.float32, device=qkv.device)
                   if nsplit > 1 else None)
        _check(_lib().illm_attn_decode_bf16(
            _p(qkv), _p(out), _p(kcache), _p(vcache), _p(page_table), page_table.shape[1],
            page_size, ring, _p(seq_slot), _p(seq_len), _p(partial), nsplit, waves, B, nh, nkv, hd,
            ctypes.c_float(scale), window, _stream()), f"attn_decode_bf16 (head_dim {hd})")
        return out
    partial = torch.empty((B, nh, nsplit, hd + 2), dtype=torch.float32, device=qkv.device)
    _check(_lib().illm_attn_decode_generic(
        _p(qkv), _p(out), _code(qkv), _p(kcache), _p(vcache), _p(page_table), page_table.shape[1],
        page_size, ring, _p(seq_slot), _p(seq_len), _p(partial), nsplit, B, nh, nkv, hd,
        ctypes.c_float(scale), window, _stream()), f"attn_decode (head_dim {hd})")
    return out


# ------------------------------------------------------------------ sampling
def argmax(logits: torch.Tensor) -> torch.Tensor:
    _gpu(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "argmax: float32 [B, V]")
    B, V = logits.shape
    out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    # a row in parts of 2,048 ids or more, about 512 blocks in all: one block a row walks a long
    # row alone (128,256 ids: 56 us whatever the batch)
    parts = max(1, min(64, V // 2048, 512 // max(B, 1)))
    scratch = torch.empty((2, B, parts), dtype=torch.int32, device=logits.device) if parts > 1 else None
    _check(_lib().illm_argmax(_p(logits), _p(out), _p(scratch), B, V, parts, _stream()), "argmax")
    return out


SAMPLE_LONG_FROM = 16384          # ids from which a row without top_k is sampled by several blocks
_sample_long_row_bytes = 0        # ILLM_SAMPLE_LONG_ROW_BYTES of csrc/api.h, asked of the library at first use


def sample(logits: torch.Tensor, temperature: float, top_k: int, top_p: float,
           repeat_penalty: float, last_tokens: Optional[torch.Tensor], seeds: torch.Tensor,
           counters: torch.Tensor) -> torch.Tensor:
    """One draw per row; see csrc/sampling.hip.  seeds: int64 [B] (bit pattern used), counters int32 [B]."""
    _gpu(logits, last_tokens, seeds, counters)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "sample: float32 [B, V]")
    B, V = logits.shape
    _need(seeds.dtype == torch.int64 and seeds.numel() >= B, "sample: seeds int64 [B]")
    _i32(counters, B); _i32(last_tokens)
    n_last = 0
    if last_tokens is not None:
        _need(last_tokens.dim() == 2 and last_tokens.shape[0] == B, "sample: last_tokens [B, n]")
        n_last = last_tokens.shape[1]
    _need(temperature > 0 and top_p > 0 and repeat_penalty > 0 and n_last <= 256,
          "sample: temperature, top_p and repeat_penalty must be positive, window <= 256")
    out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    scratch = torch.empty((2, B, V), dtype=torch.float32, device=logits.device)
    if (top_k <= 0 or top_k >= V) and V >= SAMPLE_LONG_FROM and B <= 65535:
        # a long row without top_k: several blocks a row (one block walks 32,000 ids in 54 us for
        # temperature alone and 109 us with top_p, 128,256 in 134 and 395 us)
        global _sample_long_row_bytes
        if not _sample_long_row_bytes:
            _sample_long_row_bytes = int(_lib().illm_sample_long_row_bytes())
        rows = torch.empty((B, (_sample_long_row_bytes + 7) // 8), dtype=torch.int64, device=logits.device)
        _check(_lib().illm_sample_long(
            _p(logits), _p(scratch), _p(rows), _p(out), B, V, ctypes.c_float(temperature),
            ctypes.c_float(top_p), ctypes.c_float(repeat_penalty), _p(last_tokens), n_last, _p(seeds),
            _p(counters), _stream()), "sample_long")
        return out
    _check(_lib().illm_sample(
        _p(logits), _p(scratch), _p(out), B, V, ctypes.c_float(temperature), int(top_k),
        ctypes.c_float(top_p), ctypes.c_float(repeat_penalty), _p(last_tokens), n_last, _p(seeds),
        _p(counters), _stream()), "sample")
    return out
