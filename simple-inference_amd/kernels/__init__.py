"""The device kernels, as an object the parts call.

``HipKernels`` loads the compiled HIP libraries and launches their entry points on
torch's current stream, with torch tensors as buffers.  It checks on the host that
operand shapes, dtypes and devices are what the kernels and their grids assume, and
raises before a launch that would not fit.  There is no other implementation in this
package: without a GPU or without ``hipcc`` to build a missing library it raises.
Matrix products of the bfloat16 path with more than 16 rows go to the vendor's BLAS library
(called directly, or through ``torch`` where that way is not available), as the reference's
go to its vendor's (``ops/attention.py:128-130``, ``ops/mlp.py:117,128``); products of fewer
rows and the whole 32-bit path use this package's own kernels.
"""

from __future__ import annotations

import contextlib
import ctypes
from typing import Dict, Optional

import torch

from . import build

_DT = {torch.float32: 0, torch.bfloat16: 1}

_c_int, _c_float, _c_ptr, _c_ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong

_SIGNATURES = {
    "sia_embed": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "sia_add_rmsnorm": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "sia_swiglu": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "sia_cast": [_c_ptr, _c_ptr, _c_ll, _c_int, _c_ptr],
    "sia_rope_kv_write": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr,
                          _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_attention_generic": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr,
                              _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr],
    "sia_attention_max_head_dim": [],
    "sia_gemm_generic": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_prenorm_block": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr],
    "sia_sample": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "sia_sample_workspace_bytes": [_c_int],
    "sia_sample_static": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "sia_sample_static_max_rows": [],
    "sia_sample_static_init": [],
    "sia_gemm_skinny": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_gemm_skinny_max_rows": [],
    "sia_gemm_skinny_residual_blocks": [_c_int],
    "sia_gemm_skinny_swiglu": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_float, _c_ptr],
    "sia_gemm_skinny_rope": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int,
                             _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_float, _c_ptr],
    "sia_gemm_skinny_residual": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "sia_gemm_skinny_residual_tiled": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "sia_gemm_skinny_tile_height": [_c_int],
    "sia_place_tokens": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr],
    "sia_scale_rows": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_float, _c_ptr],
    "sia_stream_read": [_c_ptr, _c_ll, _c_ptr, _c_ptr],
}


_ATTN_SIGNATURES = {
    "sia_attn_decode": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                        _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr],
    "sia_attn_prefill": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr,
                         _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int,
                         _c_ptr],
    "sia_attn_decode_max_splits": [_c_int, _c_int],
    "sia_attn_decode_workspace": [_c_int, _c_int, _c_int, _c_int, _c_int],
    "sia_attn_decode_mode": [_c_int, _c_int, _c_int, _c_int],
    "sia_attn_prefill_rows": [],
    "sia_attn_prefill_rows_split": [],
    "sia_attn_prefill_rows_long": [],
    "sia_attn_mfma_head_dim": [],
}


def attention_library_spec(head_dim: int):
    """(name, sources, defines) of the matrix-core attention library for one head size."""
    return (f"attn_mfma_d{head_dim}", ("attention_mfma.hip",), (f"SIA_HEAD_DIM={head_dim}",))


class KernelError(RuntimeError):
    pass


class PendingProduct:
    """A part's output that is still to be computed: ``x @ w^T``.  A residual stream takes it for a delta; the norm
    that follows may hand it to ``linear_into_residual``, anybody else gets the tensor from ``compute()``."""

    __slots__ = ("x", "w", "kernels")

    def __init__(self, x, w, kernels):
        self.x, self.w, self.kernels = x, w, kernels

    def compute(self):
        return self.kernels.linear(self.x, self.w)


class ScaledRows:
    """Rows of an RMS norm that are multiplied by the gain but not yet divided by their root mean square:
    ``norm(x) = rows * rsqrt(sum_p partials[p, m] / width + eps)``.  ``linear``, ``gated_linear`` and ``qkv_to_cache``
    take them in place of a tensor and scale the rows of their result instead, which is the same product."""

    __slots__ = ("rows", "partials", "eps")

    def __init__(self, rows, partials, eps):
        self.rows, self.partials, self.eps = rows, partials, eps

    shape = property(lambda self: self.rows.shape)
    dtype = property(lambda self: self.rows.dtype)
    device = property(lambda self: self.rows.device)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


class _BlockOwn(ctypes.Structure):
    """``SiaBlockOwn`` of csrc/block.hip."""
    _fields_ = ([(n, ctypes.c_void_p) for n in ("mixer_norm_gain", "w_qkv", "w_o", "feed_forward_norm_gain", "w_gate_up",
                                               "w_down", "cos_table", "sin_table")]
                + [(n, ctypes.c_float) for n in ("mixer_norm_eps", "feed_forward_norm_eps", "scale")]
                + [(n, ctypes.c_int) for n in ("hidden", "n_heads", "n_kv", "head_dim", "rotary_dim", "inter", "window")])


class _BlockStep(ctypes.Structure):
    """``SiaBlockStep`` of csrc/block.hip."""
    _fields_ = ([(n, ctypes.c_void_p) for n in ("product", "attend_single", "attend_runs", "residual", "normed", "qkv",
                                               "attended", "mixed", "gate_up", "activated", "fed", "positions",
                                               "seq_of_token", "cu_q", "kv_len", "ws_acc", "ws_ml")]
                + [(n, ctypes.c_int) for n in ("n_tokens", "n_seqs", "n_single", "max_splits", "n_tiles", "n_tiles_split",
                                               "n_tiles_long", "q_bound", "kv_bound")])


def _bind(lib, signatures):
    for name, argtypes in signatures.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int


class HipKernels:
    name = "hip-gfx950"

    def __init__(self, device="cuda:0"):
        if not torch.cuda.is_available():
            raise KernelError(
                "simple-inference_amd needs an AMD GPU: torch sees no device, and the engine has no "
                "other implementation of its kernels")
        self.device = torch.device(device)
        self.core = build.load_library("core")
        _bind(self.core, _SIGNATURES)
        self.core.sia_sample_workspace_bytes.restype = ctypes.c_longlong
        self._attn_libs = {}
        # the short way to the current stream's handle, where this torch has it (a few microseconds less a launch)
        self._raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        self._device_index = torch.device(device).index or 0
        self.use_mfma_attention = True   # tests switch it off to reach the plain kernel in bfloat16
        self.tiled_weights = True        # tests switch it off to compare with the product that reads W as it is
        self.use_skinny_gemm = True      # few-row bfloat16 products by this package's kernel, not the library
        self.fuse_norms = True           # few rows: residual add in the product before a norm, row scale in the one after
        self.fuse_rope = True            # few rows: rotation and cache write in the q/k/v product
        self.whole_blocks = True         # many rows: a block's launches in one call (``prenorm_block``)
        self._products_known: Dict[tuple, bool] = {}
        self._skinny_rows = self.core.sia_gemm_skinny_max_rows()
        self.blas = self._load_blas()    # the BLAS library called directly; None: its products go through torch

    def _load_blas(self):
        """The direct way to the vendor's BLAS library, which spares the host most of what a product through torch
        costs it.  It is a convenience, not a kernel of this package: if it cannot be built, loaded or initialised
        the products go through torch, to the same library."""
        try:
            lib = build.load_library("blas")
            lib.sia_blas_init.argtypes, lib.sia_blas_init.restype = [], ctypes.c_int
            lib.sia_blas_mm.argtypes = [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr]
            lib.sia_blas_mm.restype = ctypes.c_int
            lib.sia_blas_try_out.argtypes, lib.sia_blas_try_out.restype = [_c_int], ctypes.c_int
            lib.sia_blas_can.argtypes, lib.sia_blas_can.restype = [_c_int, _c_int, _c_int, _c_int], ctypes.c_int
            with torch.cuda.device(self.device):
                if lib.sia_blas_init() != 0:
                    return None
            return lib
        except (build.KernelBuildError, OSError, AttributeError):
            return None

    @contextlib.contextmanager
    def recurring_shapes(self):
        """Inside, the products that go to the BLAS library have the library's candidate algorithms timed on their
        own operands when their shape is first met (few rows only), and the fastest kept, for use inside this context
        only: products outside it keep the library's first choice.  For runs whose shapes will recur many times: the
        eager runs before a graph is captured, and the capture itself (which times nothing and records what those
        runs chose).  Which candidate wins is decided by the clock, so the last bits of a replayed step's products
        can differ from one process to the next; within a process a graph, once captured, never changes."""
        if self.blas is None:
            yield
            return
        with torch.cuda.device(self.device):
            self.blas.sia_blas_try_out(1)
        try:
            yield
        finally:
            with torch.cuda.device(self.device):
                self.blas.sia_blas_try_out(0)

    def _library_product(self, x, w, out_float32):
        """``x @ w^T`` for bfloat16 operands by the BLAS library, float accumulation."""
        if self.blas is not None:
            M, K = x.shape
            N = w.shape[0]
            y = torch.empty((M, N), dtype=torch.float32 if out_float32 else torch.bfloat16, device=x.device)
            if self.blas.sia_blas_mm(_ptr(x), _ptr(w), _ptr(y), M, N, K, int(out_float32), self._stream()) == 0:
                return y
        y = torch.mm(x, w.t())
        return self.cast(y, torch.float32) if out_float32 else y

    def _attn_lib(self, head_dim: int):
        """The matrix-core attention kernels for this head size, compiled at first use."""
        lib = self._attn_libs.get(head_dim)
        if lib is None:
            name, sources, defines = attention_library_spec(head_dim)
            lib = build.load_library(name, sources, defines)
            _bind(lib, _ATTN_SIGNATURES)
            lib.sia_attn_decode_workspace.restype = ctypes.c_longlong
            if lib.sia_attn_mfma_head_dim() != head_dim:
                raise KernelError(f"library {name} was built for another head size")
            self._attn_libs[head_dim] = lib
        return lib

    # -- helpers -------------------------------------------------------------
    def _stream(self):
        """Handle of torch's current stream on the device (during graph capture: the capturing stream)."""
        if self._raw_stream is not None:
            return self._raw_stream(self._device_index)
        return torch.cuda.current_stream(self.device).cuda_stream

    def _check(self, code: int, what: str):
        if code != 0:
            if code == 10001:
                raise KernelError(f"{what}: the kernel refused its arguments (sizes or types it does not take)")
            raise KernelError(f"{what}: HIP error {code}")

    def _want(self, t: torch.Tensor, what: str, dtype=None, shape=None):
        if t.device.type != "cuda":
            raise KernelError(f"{what} must be on the GPU, is on {t.device}")
        if not t.is_contiguous():
            raise KernelError(f"{what} must be contiguous")
        if dtype is not None and t.dtype != dtype:
            raise KernelError(f"{what} must be {dtype}, is {t.dtype}")
        if shape is not None and tuple(t.shape) != tuple(shape):
            raise KernelError(f"{what} must have shape {tuple(shape)}, has {tuple(t.shape)}")

    # -- measurement -----------------------------------------------------------
    def measured_read_bandwidth(self, megabytes: int = 2048, repeats: int = 5) -> float:
        """GB/s that a plain streaming read of a buffer far larger than the caches reaches on this card (the best
        of ``repeats``): the ceiling a decode step's reads can be priced against beside the published one."""
        n = int(megabytes) * (1 << 20)
        buf = torch.empty(n, dtype=torch.uint8, device=self.device)
        buf.zero_()
        sink = torch.zeros(1, dtype=torch.int32, device=self.device)
        best = 0.0
        for _ in range(repeats + 1):   # the first run warms up
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            self._check(self.core.sia_stream_read(_ptr(buf), n, _ptr(sink), self._stream()), "stream_read")
            end.record()
            end.synchronize()
            best = max(best, n / (start.elapsed_time(end) * 1e-3) / 1e9)
        return best

    # -- embedding -------------------------------------------------------------
    def place_tokens(self, token_ids, dst_rows, src_tokens, src_rows):
        """``token_ids[dst_rows[i]] = src_tokens[src_rows[i]]`` (all int32, on the device)."""
        for t, what in ((token_ids, "token ids"), (dst_rows, "destination rows"), (src_tokens, "source tokens"),
                        (src_rows, "source rows")):
            self._want(t, what, torch.int32)
        if dst_rows.numel() != src_rows.numel():
            raise KernelError(f"{dst_rows.numel()} destination rows for {src_rows.numel()} source rows")
        self._check(self.core.sia_place_tokens(_ptr(token_ids), _ptr(dst_rows), _ptr(src_tokens), _ptr(src_rows),
                                               dst_rows.numel(), self._stream()), "place_tokens")

    def embed(self, token_ids, table):
        self._want(token_ids, "token_ids", torch.int32)
        self._want(table, "embedding table")
        if table.dtype not in _DT or table.dim() != 2:
            raise KernelError(f"embedding table must be a float32 or bfloat16 matrix, is {table.dtype} {tuple(table.shape)}")
        n, hidden = token_ids.numel(), table.shape[1]
        out = torch.empty((n, hidden), dtype=torch.float32, device=table.device)
        self._check(self.core.sia_embed(_ptr(token_ids), _ptr(table), _ptr(out), n, hidden, _DT[table.dtype],
                                        self._stream()), "embed")
        return out

    # -- residual add + rms norm ---------------------------------------------
    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype, rows=None):
        n, hidden = residual.shape
        self._want(residual, "residual", torch.float32)
        self._want(weight, "norm weight", torch.float32, (hidden,))
        if out_dtype not in _DT:
            raise KernelError(f"norm output dtype {out_dtype} is not float32 or bfloat16")
        if delta is not None:
            self._want(delta, "delta", out_dtype, (n, hidden))
        n_out = n
        if rows is not None:
            self._want(rows, "rows", torch.int32)
            n_out = rows.numel()
        out = torch.empty((n_out, hidden), dtype=out_dtype, device=residual.device)
        self._check(self.core.sia_add_rmsnorm(_ptr(residual), _ptr(delta), _ptr(weight), _ptr(out), _ptr(rows),
                                              n_out, hidden, float(eps), _DT[out_dtype], self._stream()),
                    "add_rmsnorm")
        return out

    # -- matrix product --------------------------------------------------------
    def linear(self, x, w, out_float32=False):
        """``x [M, K] @ w [N, K]^T`` with float accumulation."""
        x = self.finish_rows(x)
        self._want(x, "linear input")
        self._want(w, "linear weight")
        if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
            raise KernelError(f"linear shapes do not fit: x {tuple(x.shape)}, w {tuple(w.shape)}")
        if x.dtype not in _DT or w.dtype not in _DT:
            raise KernelError(f"linear takes float32 or bfloat16, got {x.dtype} and {w.dtype}")
        M, K = x.shape
        N = w.shape[0]
        if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
            # up to 16 rows: this package's kernel, whose sums do not depend on the number of rows
            if self.use_skinny_gemm and M <= self._skinny_rows and K % 64 == 0:
                y = torch.empty((M, N), dtype=torch.float32 if out_float32 else torch.bfloat16, device=x.device)
                self._check(self.core.sia_gemm_skinny(_ptr(x), _ptr(w), _ptr(y), M, N, K, int(out_float32),
                                                      self._stream()), "gemm_skinny")
                return y
            return self._library_product(x, w, out_float32)
        # True 32-bit product.  A float32-stored matrix meeting bfloat16 activations widens them.
        back = None
        if x.dtype == torch.bfloat16:
            back = torch.bfloat16
            x = self.cast(x, torch.float32)
        if w.dtype == torch.bfloat16:
            w = self.cast(w, torch.float32)
        y = torch.empty((M, N), dtype=torch.float32, device=x.device)
        self._check(self.core.sia_gemm_generic(_ptr(x), _ptr(w), _ptr(y), M, N, K, 0, 1, self._stream()),
                    "gemm_generic")
        if back is not None and not out_float32:
            y = self.cast(y, back)
        return y

    def gated_linear(self, x, w_gate_up):
        """``silu(x Wg^T) * (x Wu^T)`` for ``w_gate_up = [Wg; Wu]``: one kernel for few rows, else product + SwiGLU."""
        self._want(w_gate_up, "gate/up weight")
        M, K = x.shape
        two_i = w_gate_up.shape[0]
        if (self.use_skinny_gemm and x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16
                and M <= self._skinny_rows and two_i % 2 == 0 and K % 64 == 0 and w_gate_up.shape[1] == K):
            rows, partials, n_partials, eps = self._scaled(x)
            self._want(rows, "gated linear input")
            y = torch.empty((M, two_i // 2), dtype=torch.bfloat16, device=rows.device)
            self._check(self.core.sia_gemm_skinny_swiglu(_ptr(rows), _ptr(w_gate_up), _ptr(y), M, two_i // 2, K,
                                                         _ptr(partials), n_partials, eps, self._stream()),
                        "gemm_skinny_swiglu")
            return y
        return self.swiglu(self.linear(x, w_gate_up))

    # -- a product whose result goes into the residual, and the norm after it ---------
    def pending_linear(self, x, w):
        """``linear(x, w)`` as the last product of a part.  For few rows in bfloat16 it is not computed yet: the norm
        that follows has it computed by ``linear_into_residual``, which saves the norm's own kernel."""
        if (self.use_skinny_gemm and self.fuse_norms and isinstance(x, torch.Tensor) and x.dim() == 2 and w.dim() == 2
                and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.shape[1] == w.shape[1]
                and 0 < x.shape[0] <= self._skinny_rows and w.shape[1] % 64 == 0):
            return PendingProduct(x, w, self)
        return self.linear(x, w)

    def linear_into_residual(self, pending, residual, gain, eps):
        """``residual += x @ w^T`` (the product rounded to bfloat16 first, as ``linear`` rounds it) and the rows of
        the RMS norm of the sum as ``ScaledRows``."""
        x, w = pending.x, pending.w
        self._want(x, "linear input", torch.bfloat16)
        self._want(w, "linear weight", torch.bfloat16)
        self._want(residual, "residual", torch.float32)
        self._want(gain, "norm weight", torch.float32)
        M, K = x.shape
        N = w.shape[0]
        if (w.shape[1] != K or tuple(residual.shape) != (M, N) or tuple(gain.shape) != (N,) or M > self._skinny_rows
                or K % 64):
            raise KernelError(f"product into the residual does not fit: x {tuple(x.shape)}, w {tuple(w.shape)}, "
                              f"residual {tuple(residual.shape)}, gain {tuple(gain.shape)}")
        rows = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
        partials = torch.empty((self.core.sia_gemm_skinny_residual_blocks(N), 16), dtype=torch.float32, device=x.device)
        tiled = self._tiled_copy(w)
        if tiled is not None:
            self._check(self.core.sia_gemm_skinny_residual_tiled(_ptr(x), _ptr(tiled), M, N, K, _ptr(residual),
                                                                 _ptr(gain), _ptr(rows), _ptr(partials), self._stream()),
                        "gemm_skinny_residual_tiled")
        else:
            self._check(self.core.sia_gemm_skinny_residual(_ptr(x), _ptr(w), M, N, K, _ptr(residual), _ptr(gain),
                                                           _ptr(rows), _ptr(partials), self._stream()),
                        "gemm_skinny_residual")
        return ScaledRows(rows, partials, float(eps))

    # A weight whose product goes into the residual in steps of few rows may have a second copy, laid out in the
    # order in which that kernel's workgroups read it (every load instruction one run of memory: the o and down
    # products of a decode step take 10 to 15 % less).  The copy hangs on the weight tensor itself, so it lives as long
    # as the weight does, and remembers the version of the tensor it was made from: a weight changed in place since
    # is read as it is.  Steps of more rows, which go to the library, read the weight as it is anyway.
    def prepare_pending_weight(self, w) -> bool:
        """Makes the tiled copy of a weight that ``pending_linear`` will be given; True if one was made."""
        if (not self.tiled_weights or not isinstance(w, torch.Tensor) or w.dim() != 2 or w.dtype != torch.bfloat16
                or not w.is_cuda or not w.is_contiguous() or w.shape[1] % 64 or torch.cuda.is_current_stream_capturing()):
            return False
        N, K = w.shape
        height = self.core.sia_gemm_skinny_tile_height(N)
        if height <= 0:
            return False
        blocks = -(-N // height)
        rows = torch.arange(blocks * height, device=w.device).clamp_(max=N - 1)   # the last block repeats the last row
        # element (block, step, half, row, lane group, e) = W[block * height + row][64 step + 16 group + 8 half + e]
        tiled = w[rows].view(blocks, height, K // 64, 4, 2, 8).permute(0, 2, 4, 1, 3, 5).contiguous()
        w._sia_tiled = (tiled, w._version)
        return True

    def _tiled_copy(self, w):
        kept = getattr(w, "_sia_tiled", None) if self.tiled_weights else None
        if kept is None or kept[1] != w._version:
            return None
        return kept[0]

    @staticmethod
    def _scaled(x):
        """(rows, partials, n_partials, eps) of an input that may be ``ScaledRows``."""
        if isinstance(x, ScaledRows):
            return x.rows, x.partials, x.partials.shape[0], x.eps
        return x, None, 0, 0.0

    def finish_rows(self, x):
        """The tensor that ``ScaledRows`` stand for (a tensor is returned as it is)."""
        if not isinstance(x, ScaledRows):
            return x
        out = torch.empty_like(x.rows)
        self._check(self.core.sia_scale_rows(_ptr(x.rows), _ptr(x.partials), _ptr(out), x.rows.shape[0],
                                             x.rows.shape[1], x.partials.shape[0], x.eps, self._stream()),
                    "scale_rows")
        return out

    def gemm_generic(self, x, w, out_float32=False):
        """The plain kernel for either dtype (tests compare it with the library product)."""
        self._want(x, "gemm input")
        self._want(w, "gemm weight", x.dtype)
        M, K = x.shape
        N = w.shape[0]
        out_dtype = torch.float32 if (out_float32 or x.dtype == torch.float32) else x.dtype
        y = torch.empty((M, N), dtype=out_dtype, device=x.device)
        self._check(self.core.sia_gemm_generic(_ptr(x), _ptr(w), _ptr(y), M, N, K, _DT[x.dtype],
                                               int(out_dtype == torch.float32), self._stream()), "gemm_generic")
        return y

    def cast(self, x, dtype):
        self._want(x, "cast input")
        if x.dtype == dtype:
            return x
        if {x.dtype, dtype} != {torch.float32, torch.bfloat16}:
            raise KernelError(f"cast is between float32 and bfloat16 only, got {x.dtype} -> {dtype}")
        out = torch.empty(x.shape, dtype=dtype, device=x.device)
        self._check(self.core.sia_cast(_ptr(x), _ptr(out), x.numel(), _DT[x.dtype], self._stream()), "cast")
        return out

    # -- feed-forward activation ---------------------------------------------
    def swiglu(self, gu):
        self._want(gu, "swiglu input")
        if gu.dtype not in _DT or gu.dim() != 2 or gu.shape[1] % 2:
            raise KernelError(f"swiglu takes a [tokens, 2*intermediate] float32/bfloat16 matrix, got {gu.dtype} {tuple(gu.shape)}")
        n, two_i = gu.shape
        out = torch.empty((n, two_i // 2), dtype=gu.dtype, device=gu.device)
        for n0 in range(0, n, 65535):  # grid.y limit
            n1 = min(n, n0 + 65535)
            self._check(self.core.sia_swiglu(_ptr(gu[n0:n1]), _ptr(out[n0:n1]), n1 - n0, two_i // 2,
                                             _DT[gu.dtype], self._stream()), "swiglu")
        return out

    # -- rotation + cache write ------------------------------------------------
    def rope_kv_write(self, qkv, n_heads, n_kv_written, head_dim, rotary_dim, cos, sin, ctx, cache):
        self._want(qkv, "qkv")
        n, width = qkv.shape
        if qkv.dtype not in _DT:
            raise KernelError(f"qkv must be float32 or bfloat16, is {qkv.dtype}")
        if width != (n_heads + 2 * n_kv_written) * head_dim:
            raise KernelError(f"qkv row of {width} does not hold {n_heads} + 2*{n_kv_written} heads of {head_dim}")
        if n != ctx.n_tokens:
            raise KernelError(f"qkv has {n} rows, the step {ctx.n_tokens} tokens")
        if rotary_dim:
            for t, what in ((cos, "cos table"), (sin, "sin table")):
                self._want(t, what, torch.float32)
                if t.shape[1] != rotary_dim // 2 or t.shape[0] <= ctx.max_kv_len - 1:
                    raise KernelError(f"{what} {tuple(t.shape)} does not cover position {ctx.max_kv_len - 1} "
                                      f"with {rotary_dim // 2} pairs")
        table = table_w = k_pages = v_pages = None
        page_size = 0
        if n_kv_written:
            k_pages, v_pages, table, page_size = cache.k_pages, cache.v_pages, cache.block_table, cache.page_size
            self._check_pages(k_pages, v_pages, table, page_size, n_kv_written, head_dim, qkv.dtype, ctx)
        table_w = table.shape[1] if table is not None else 0
        self._check(self.core.sia_rope_kv_write(
            _ptr(qkv), width, _ptr(cos) if rotary_dim else None, _ptr(sin) if rotary_dim else None,
            _ptr(ctx.positions), _ptr(ctx.seq_of_token), _ptr(table), table_w, _ptr(k_pages), _ptr(v_pages),
            n, n_heads, n_kv_written, head_dim, rotary_dim, page_size, _DT[qkv.dtype], self._stream()),
            "rope_kv_write")

    def qkv_to_cache(self, x, w_qkv, n_heads, n_kv_written, head_dim, rotary_dim, cos, sin, ctx, cache):
        """The q/k/v product, the rotation of q and k and the write of k and v into the pages.  Returns the
        ``[tokens, (n_heads + 2 n_kv_written) head_dim]`` matrix whose q columns hold the rotated queries; its
        k and v columns are not to be read (for few rows one kernel does all three and never writes them)."""
        M, K = x.shape
        if (self.use_skinny_gemm and self.fuse_rope and n_kv_written and x.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16
                and M <= self._skinny_rows and rotary_dim == head_dim and head_dim % 2 == 0 and K % 64 == 0):
            x, partials, n_partials, norm_eps = self._scaled(x)
            self._want(x, "q/k/v input")
            self._want(w_qkv, "q/k/v weight")
            width = (n_heads + 2 * n_kv_written) * head_dim
            if tuple(w_qkv.shape) != (width, K):
                raise KernelError(f"q/k/v weight {tuple(w_qkv.shape)} is not [{width}, {K}]")
            if M != ctx.n_tokens:
                raise KernelError(f"q/k/v input has {M} rows, the step {ctx.n_tokens} tokens")
            for t, what in ((cos, "cos table"), (sin, "sin table")):
                self._want(t, what, torch.float32)
                if t.shape[1] != rotary_dim // 2 or t.shape[0] <= ctx.max_kv_len - 1:
                    raise KernelError(f"{what} {tuple(t.shape)} does not cover position {ctx.max_kv_len - 1} "
                                      f"with {rotary_dim // 2} pairs")
            self._check_pages(cache.k_pages, cache.v_pages, cache.block_table, cache.page_size, n_kv_written,
                              head_dim, x.dtype, ctx)
            qkv = torch.empty((M, width), dtype=torch.bfloat16, device=x.device)
            self._check(self.core.sia_gemm_skinny_rope(
                _ptr(x), _ptr(w_qkv), _ptr(qkv), M, K, _ptr(cos), _ptr(sin), _ptr(ctx.positions),
                _ptr(ctx.seq_of_token), _ptr(cache.block_table), cache.block_table.shape[1], _ptr(cache.k_pages),
                _ptr(cache.v_pages), n_heads, n_kv_written, head_dim, cache.page_size, _ptr(partials), n_partials,
                norm_eps, self._stream()),
                "gemm_skinny_rope")
            return qkv
        qkv = self.linear(x, w_qkv)
        self.rope_kv_write(qkv, n_heads, n_kv_written, head_dim, rotary_dim, cos, sin, ctx, cache)
        return qkv

    def _check_pages(self, k_pages, v_pages, table, page_size, n_kv, head_dim, dtype, ctx):
        self._want(k_pages, "key pages", dtype)
        self._want(v_pages, "value pages", dtype)
        pages = k_pages.shape[0]
        if tuple(k_pages.shape) != (pages, n_kv, page_size, head_dim):
            raise KernelError(f"key pages {tuple(k_pages.shape)} are not [pages, {n_kv}, {page_size}, {head_dim}]")
        if tuple(v_pages.shape) != (pages, n_kv, head_dim, page_size):
            raise KernelError(f"value pages {tuple(v_pages.shape)} are not [pages, {n_kv}, {head_dim}, {page_size}]")
        self._want(table, "block table", torch.int32)
        if table.dim() != 2 or table.shape[0] != ctx.n_seqs or table.shape[1] * page_size < ctx.max_kv_len:
            raise KernelError(f"block table {tuple(table.shape)} does not cover {ctx.n_seqs} sequences of up to "
                              f"{ctx.max_kv_len} positions with pages of {page_size}")

    # -- attention ---------------------------------------------------------------
    def check_attention_geometry(self, n_heads: int, n_kv_heads: int, head_dim: int) -> None:
        """Raises for head counts and sizes that no attention kernel here takes.  A mixer calls it when the model is
        built, so that such a model is refused before it is loaded, not at its first step."""
        limit = self.core.sia_attention_max_head_dim()
        if not 0 < head_dim <= limit:
            raise KernelError(f"head size {head_dim} is outside what the attention kernels take (1 to {limit})")
        if n_kv_heads <= 0 or n_heads <= 0 or n_heads % n_kv_heads:
            raise KernelError(f"{n_heads} query heads cannot share {n_kv_heads} key/value heads evenly")
        if n_heads > 65535:
            raise KernelError(f"{n_heads} query heads exceed the kernels' grids (65,535)")

    def paged_attention(self, qkv, n_heads, n_kv_heads, head_dim, scale, window, ctx, cache):
        self._want(qkv, "qkv")
        n, width = qkv.shape
        if width < n_heads * head_dim or n != ctx.n_tokens:
            raise KernelError(f"qkv {tuple(qkv.shape)} does not hold {ctx.n_tokens} rows of {n_heads} heads of {head_dim}")
        self._check_pages(cache.k_pages, cache.v_pages, cache.block_table, cache.page_size, n_kv_heads, head_dim,
                          qkv.dtype, ctx)
        out = torch.empty((n, n_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
        page = cache.page_size
        if (self.use_mfma_attention and qkv.dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 256
                and page >= 8 and width % 8 == 0 and scale > 0):
            self._mfma_attention(qkv, out, n_heads, n_kv_heads, head_dim, scale, int(window or 0), ctx, cache)
            return out
        self._check(self.core.sia_attention_generic(
            _ptr(qkv), width, _ptr(cache.k_pages), _ptr(cache.v_pages), _ptr(cache.block_table),
            cache.block_table.shape[1], _ptr(ctx.seq_of_token), _ptr(ctx.positions), _ptr(out), n, n_heads,
            n_kv_heads, head_dim, page, float(scale), int(window or 0), _DT[qkv.dtype],
            self._stream()), "attention_generic")
        return out

    def _attention_plan(self, lib, device, n_heads, n_kv_heads, head_dim, window, ctx):
        """What the attention launches of a step need beside the tensors: the same for every layer with this
        geometry, so it is worked out once per step and kept with the step's context (workspaces included: a step's
        layers run one after the other)."""
        key = (n_heads, n_kv_heads, head_dim, window)
        plans = getattr(ctx, "attention_plans", None)
        if plans is not None and key in plans:
            return plans[key]
        group = n_heads // n_kv_heads
        n_dec = ctx.n_decode_seqs if group <= 16 and 4 * group * (head_dim + 2) * 4 <= 65536 else 0
        max_splits, ws_acc, ws_ml = 1, None, None
        if n_dec:
            # How many workgroups share a (sequence, kv head) is the kernel's decision, from that sequence's own
            # length; the step's longest possible sequence only sizes the grid and the workspaces.
            max_splits = lib.sia_attn_decode_max_splits(int(ctx.kv_bound or ctx.max_kv_len), window)
            ws_acc, ws_ml = (
                torch.empty((floats,), dtype=torch.float32, device=device) if floats else None
                for floats in (lib.sia_attn_decode_workspace(n_dec, n_heads, n_kv_heads, max_splits, which)
                               for which in (0, 1)))
        tiles = (0, 0, 0, 0, 0)
        if n_dec < ctx.n_seqs:
            # row tiles at each of the kernel's workgroup sizes, and what bounds a sequence's tokens and keys in this
            # step: a portion over a long past takes another workgroup shape than a prompt from its start
            tiles = tuple(sum(-(-q // rows) for q in ctx.q_lens[n_dec:]) if rows else 0
                          for rows in (lib.sia_attn_prefill_rows(), lib.sia_attn_prefill_rows_split(),
                                       lib.sia_attn_prefill_rows_long()))
            tiles += (int(max(ctx.q_lens[n_dec:])), int(getattr(ctx, "max_run_kv_len", 0) or ctx.max_kv_len))
        plan = (n_dec, max_splits, ws_acc, ws_ml, tiles)
        if plans is None:
            try:
                ctx.attention_plans = plans = {}
            except AttributeError:      # a context that takes no further attributes: nothing is kept
                return plan
        plans[key] = plan
        return plan

    def _mfma_attention(self, qkv, out, n_heads, n_kv_heads, head_dim, scale, window, ctx, cache):
        lib = self._attn_lib(head_dim)
        width = qkv.shape[1]
        table = cache.block_table
        n_dec, max_splits, ws_acc, ws_ml, (n_tiles, n_tiles_split, n_tiles_long, q_bound, kv_bound) = \
            self._attention_plan(lib, qkv.device, n_heads, n_kv_heads, head_dim, window, ctx)
        if n_dec:
            self._check(lib.sia_attn_decode(
                _ptr(qkv), width, _ptr(cache.k_pages), _ptr(cache.v_pages), _ptr(table), table.shape[1],
                _ptr(ctx.cu_q), _ptr(ctx.kv_len), _ptr(out), _ptr(ws_acc), _ptr(ws_ml), n_dec, n_heads,
                n_kv_heads, cache.page_size, float(scale), window, max_splits, self._stream()),
                "attn_decode")
        if n_dec < ctx.n_seqs:
            self._check(lib.sia_attn_prefill(
                _ptr(qkv), width, _ptr(cache.k_pages), _ptr(cache.v_pages), _ptr(table), table.shape[1],
                _ptr(ctx.cu_q), _ptr(ctx.kv_len), _ptr(out), n_dec, ctx.n_seqs, n_tiles, n_tiles_split, n_tiles_long,
                q_bound, kv_bound, n_heads, n_kv_heads, cache.page_size, float(scale), window, self._stream()),
                "attn_prefill")

    # -- a whole block in one call -------------------------------------------------
    def _library_can(self, M, N, K) -> bool:
        key = (M, N, K)
        known = self._products_known.get(key)
        if known is None:
            with torch.cuda.device(self.device):
                known = self._products_known[key] = self.blas.sia_blas_can(M, N, K, 0) == 0
        return known

    def _block_own(self, block):
        """The block as the one-call form takes it (a structure of pointers and constants, with the tensors it points
        into), or False if its parts are not of the kinds that form covers.  Made once and kept with the block."""
        forms = block.plain_forms
        if forms is not None:
            return forms
        block.plain_forms = False
        # the block says what it is: its kind and its parts' own descriptions.  The one-call form exists for a
        # pre-norm block of an RMS norm, paged attention, an RMS norm and a SwiGLU feed-forward.
        whole = getattr(block, "plain_form", lambda: None)()
        if not whole or whole.get("kind") != "prenorm":
            return False
        parts = [whole.get(name) for name in ("mixer_norm", "mixer", "feed_forward_norm", "feed_forward")]
        if any(f is None for f in parts) or [f["kind"] for f in parts] != ["rmsnorm", "paged_attention", "rmsnorm", "swiglu"]:
            return False
        n1, at, n2, ff = parts
        H, nh, nkv, D, I = at["hidden"], at["n_heads"], at["n_kv_heads"], at["head_dim"], ff["inter"]
        bf, f32 = torch.bfloat16, torch.float32
        wanted = ((n1["weight"], f32, (H,)), (n2["weight"], f32, (H,)), (at["w_qkv"], bf, ((nh + 2 * nkv) * D, H)),
                  (at["w_o"], bf, (H, nh * D)), (ff["w_gate_up"], bf, (2 * I, H)), (ff["w_down"], bf, (H, I)))
        rd = at["rotary_dim"]
        if rd:
            wanted += ((at["cos"], f32, None), (at["sin"], f32, None))
        for t, dtype, shape in wanted:
            if (not isinstance(t, torch.Tensor) or t.device.type != "cuda" or t.dtype != dtype or not t.is_contiguous()
                    or (shape is not None and tuple(t.shape) != shape)):
                return False
        if (ff["hidden"] != H or n1["size"] != H or n2["size"] != H or D % 16 or D > 256 or not at["scale"] > 0
                or (rd and (at["cos"].shape[1] != rd // 2 or at["sin"].shape != at["cos"].shape))):
            return False
        own = _BlockOwn(_ptr(n1["weight"]), _ptr(at["w_qkv"]), _ptr(at["w_o"]), _ptr(n2["weight"]), _ptr(ff["w_gate_up"]),
                        _ptr(ff["w_down"]), _ptr(at["cos"]) if rd else None, _ptr(at["sin"]) if rd else None,
                        float(n1["eps"]), float(n2["eps"]), float(at["scale"]), H, nh, nkv, D, rd, I, int(at["window"] or 0))
        block.plain_forms = (own, [t for t, _, _ in wanted], at["cos"].shape[0] if rd else None)
        return block.plain_forms

    def _block_step(self, own, ctx, device):
        """What a step brings to the one-call form of its blocks of this geometry: buffers, metadata, the attention
        plan.  Made once per step and geometry and kept with the step's context; None if the library has no
        algorithm for one of the products at this number of rows."""
        key = (own.hidden, own.n_heads, own.n_kv, own.head_dim, own.inter, own.window)
        steps = getattr(ctx, "block_steps", None)
        if steps is None:
            try:
                ctx.block_steps = steps = {}
            except AttributeError:
                return None
        if key in steps:
            return steps[key]
        M, H, Q, I = ctx.n_tokens, own.hidden, own.n_heads * own.head_dim, own.inter
        width = (own.n_heads + 2 * own.n_kv) * own.head_dim
        steps[key] = None
        if not all(self._library_can(M, n, k) for n, k in ((width, H), (H, Q), (2 * I, H), (H, I))):
            return None
        lib = self._attn_lib(own.head_dim)
        n_dec, max_splits, ws_acc, ws_ml, tiles = self._attention_plan(lib, device, own.n_heads, own.n_kv, own.head_dim,
                                                                       own.window, ctx)
        new = lambda n: torch.empty((M, n), dtype=torch.bfloat16, device=device)
        buffers = [new(H), new(width), new(Q), new(H), new(2 * I), new(I), new(H)]
        fn = lambda f: ctypes.cast(f, ctypes.c_void_p).value
        step = _BlockStep(fn(self.blas.sia_blas_mm), fn(lib.sia_attn_decode), fn(lib.sia_attn_prefill), None,
                          *[_ptr(b) for b in buffers], _ptr(ctx.positions), _ptr(ctx.seq_of_token), _ptr(ctx.cu_q),
                          _ptr(ctx.kv_len), _ptr(ws_acc), _ptr(ws_ml), M, ctx.n_seqs, n_dec, max_splits, *tiles)
        steps[key] = (step, buffers)
        return steps[key]

    def prenorm_block(self, block, stream, ctx, cache) -> bool:
        """Runs a pre-norm block of RMS norms, paged attention and SwiGLU on a step of many rows with one call into
        the library (the same launches, in the same order, as the parts' own calls make); False, with nothing done,
        where that form does not apply: the caller then goes part by part."""
        if not self.whole_blocks or self.blas is None or not self.use_mfma_attention:
            return False
        residual = stream.residual
        M = ctx.n_tokens
        if (M <= self._skinny_rows or M > 65535 or getattr(ctx, "extra", None)
                or residual.dtype != torch.float32 or cache.k_pages is None or cache.page_size < 8):
            return False
        made = self._block_own(block)
        if not made:
            return False
        own, _, positions_covered = made
        if (tuple(residual.shape) != (M, own.hidden) or not residual.is_contiguous() or cache.k_pages.dtype != torch.bfloat16
                or (positions_covered is not None and positions_covered <= ctx.max_kv_len - 1)):
            return False
        step = self._block_step(own, ctx, residual.device)
        if step is None:
            return False
        delta = stream.delta    # computes it if it is a product not yet computed
        if delta is not None and (delta.dtype != torch.bfloat16 or tuple(delta.shape) != (M, own.hidden)
                                  or not delta.is_contiguous()):
            return False
        self._check_pages(cache.k_pages, cache.v_pages, cache.block_table, cache.page_size, own.n_kv, own.head_dim,
                          torch.bfloat16, ctx)
        step_struct, buffers = step
        step_struct.residual = _ptr(residual)
        self._check(self.core.sia_prenorm_block(
            ctypes.addressof(own), ctypes.addressof(step_struct), _ptr(delta), _ptr(cache.block_table),
            cache.block_table.shape[1], _ptr(cache.k_pages), _ptr(cache.v_pages), cache.page_size, self._stream()),
            "prenorm_block")
        stream.delta = buffers[-1]
        return True

    # -- sampling ------------------------------------------------------------------
    def sample(self, logits, temperature, top_k, top_p, uniform, all_greedy=False, filters=None):
        """One token per row.  What the caller knows on the host spares launches: ``all_greedy`` (every
        temperature is 0; the parameter tensors may then be None), or ``filters``, the sum of 1 if some row
        may have a top-k filter and 2 if some row may have a top-p filter below 1 (None: both)."""
        rows, vocab = logits.shape
        self._want(logits, "logits", torch.float32)
        if all_greedy:
            filters = 0
            temperature = top_k = top_p = uniform = None
        else:
            filters = 4 | (3 if filters is None else int(filters) & 3)
            self._want(temperature, "temperature", torch.float32, (rows,))
            self._want(top_k, "top_k", torch.int32, (rows,))
            self._want(top_p, "top_p", torch.float32, (rows,))
            self._want(uniform, "uniform", torch.float32, (rows,))
        out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
        # One workspace, kept and grown as needed: the kernels set to zero what they need at zero, and calls follow
        # one another on the stream.  (Callers on several streams at once need a kernels object each.)
        need = self.core.sia_sample_workspace_bytes(rows)
        workspace = getattr(self, "_sample_workspace", None)
        if workspace is None or workspace.numel() < need or workspace.device != logits.device:
            workspace = self._sample_workspace = torch.empty((need,), dtype=torch.uint8, device=logits.device)
        self._check(self.core.sia_sample(_ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(uniform),
                                         _ptr(out), _ptr(workspace), rows, vocab, filters, self._stream()), "sample")
        return out
