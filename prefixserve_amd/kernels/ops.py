"""Python face of the kernel library: checks shapes on the host, then launches the
hand-written HIP kernels on torch's current stream with raw pointers.

There is no other implementation behind these calls: without a GPU or without the
compiled library, constructing ``HipOps`` raises. The only library routine on the path is
the matrix product ``torch.matmul`` (hipBLASLt) for bfloat16 products with more than 64
rows, where the reference's engine also calls a library (prefixserve/model/llama.py:113-126);
every 32-bit product and every product with at most 64 rows is a kernel of this package.
"""

from __future__ import annotations

import contextlib
import ctypes
import logging
import os
from typing import Any, Sequence

import torch

from prefixserve_amd.build import ensure_kernels
from prefixserve_amd.parts.base import NormedRows

_F32, _BF16 = 0, 1
_vp, _i32, _i64, _f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float


class KernelError(RuntimeError):
    pass


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _F32
    if dtype == torch.bfloat16:
        return _BF16
    raise KernelError(f"kernels take float32 or bfloat16, got {dtype}")


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


logger = logging.getLogger(__name__)

_SIGNATURES = {
    "psamd_embed": [_vp, _vp, _vp, _i32, _vp, _i64, _i32, _i32],
    "psamd_add_rmsnorm": [_vp, _vp, _vp, _i32, _i32, _i64, _vp, _vp, _i32, _f32, _vp, _i32, _i64, _i32],
    "psamd_swiglu": [_vp, _vp, _vp, _i32, _i64, _i32],
    "psamd_rope_kv_append": [_vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp, _vp, _vp, _vp],
    "psamd_linear": [_vp, _vp, _i32, _vp, _i32, _vp, _i32, _i64, _i32, _i32],
    "psamd_gemm_lt": [_vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _i32],
    "psamd_linear_skinny": [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32],
    "psamd_linear_skinny_ksplit": [_i32, _i32, _i32],
    "psamd_qkv_rope_append": [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp],
    "psamd_normed_supports": [_i32, _i32],
    "psamd_linear_skinny_add": [_vp, _vp, _vp, _vp, _i32, _i32, _i32],
    "psamd_linear_normed": [_vp, _vp, _vp, _vp, _i32, _f32, _vp, _vp, _i32, _i32, _i32, _i32, _i32],
    "psamd_qkv_rope_append_normed": [_vp, _vp, _vp, _i32, _f32, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp],
    "psamd_attention_generic": [_vp, _vp, _i32, _vp, _vp, _i32, _i64, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _f32, _i32],
    "psamd_attention_mfma_supports": [_i32, _i32, _i32],
    "psamd_attention_prefill_nsplit": [_i32, _i32, _i32, _i32, _i32],
    "psamd_attention_prefill_part_rows": [_i32, _i32, _i32],
    "psamd_attention_decode_skewed": [_i32, _i32, _i64],
    "psamd_attention_decode_plan": [_i32, _i32, _i32, _i32, _i32, _vp, _vp],
    "psamd_attention_decode_max_parts": [_i32],
    "psamd_attention_prefill": [_vp, _vp, _i32, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _vp, _vp, _vp, _i32, _i32, _i32,
                                _f32, _i32, _vp, _vp, _i32],
    "psamd_attention_decode": [_vp, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _vp, _i32, _i32, _i32,
                               _i32, _f32, _i32, _i32],
    "psamd_sample": [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32],
}


class HipOps:
    PREFILL_TILE_Q = 32    # queries per workgroup of the prefill attention kernel (its 4 waves split the keys)
    SKINNY_MAX_ROWS = 64
    FUSED_SWIGLU_MAX_ROWS = 32      # above it (to SKINNY_MAX_ROWS) gate/up goes to the library, where there is one
    LIBRARY_ADD_MIN_ROWS = 1024     # from here on a product that feeds the residual stream adds into it in the library
    name = "hip"

    def __init__(self, device: torch.device | str, workspace: Any = None) -> None:
        self.device = torch.device(device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise KernelError("prefixserve_amd runs on a GPU only: no device kernels can run on "
                              f"{self.device} and there is no CPU implementation to fall back to")
        self.lib = ensure_kernels()
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(self.lib, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        self.lib.psamd_last_error.restype = ctypes.c_char_p
        self.lib.psamd_sample_scratch_floats.argtypes = [ctypes.c_int]
        self.lib.psamd_sample_scratch_floats.restype = ctypes.c_int64
        self.ws = workspace
        self._sample_scratch: torch.Tensor | None = None
        self._step_stream: int | None = None
        self._plans: dict[tuple, tuple[int, int]] = {}
        self._bounds: dict[Any, int] = {}                # sizes of the attention's partial-result buffers, from the library
        self._fuses: dict[tuple[int, int], bool] = {}
        self._slice_views: dict[tuple, tuple] = {}      # (name, slices, rows) -> (buffer, its [slices, rows, N] view)
        # The library for large bfloat16 products, called directly if it can be (it sets itself up
        # here, outside any capture); through torch.mm otherwise.
        self.lib.psamd_gemm_lt_available.argtypes = []
        with torch.cuda.device(self.device):
            self._direct_library = bool(self.lib.psamd_gemm_lt_available())
        # Set while a step is run for, or under, graph capture: the key length that grids and
        # LDS tables are sized by instead of the step's own, and no product with a workspace.
        self.fixed_kv_len: int | None = None
        self.fixed_skew = False      # with fixed_kv_len: whether the step's context lengths count as skewed

    # ---------------------------------------------------------------- helpers

    def _stream(self) -> int:
        if self._step_stream is not None:
            return self._step_stream
        return torch.cuda.current_stream(self.device).cuda_stream

    @contextlib.contextmanager
    def step_scope(self):
        """All calls inside go to the stream that is current now: a step runs on one stream,
        and asking torch for it costs as much as launching a small kernel."""
        outer = self._step_stream
        self._step_stream = torch.cuda.current_stream(self.device).cuda_stream
        try:
            yield
        finally:
            self._step_stream = outer

    def _ok(self, rc: int) -> None:
        if rc != 0:
            raise KernelError(self.lib.psamd_last_error().decode())

    # ------------------------------------------------- kernels a part brings itself

    def load_extension(self, path: "str | os.PathLike[str]", signatures: dict[str, list]) -> ctypes.CDLL:
        """Loads a library of device kernels built with ``build.build_extension`` and declares
        its entry points (``name -> ctypes argument types``; each returns 0 or an error code):
        how a part with a kernel of its own gets at it without a change to this file. The part
        calls ``lib.entry(ops.stream_pointer(), tensor.data_ptr(), ...)`` and hands the result to
        ``ops.check``; the stream is the step's, so the call may be captured like any other."""
        try:
            lib = ctypes.CDLL(os.fspath(path))
        except OSError as e:
            raise KernelError(f"cannot load the kernel library {path}: {e}") from None
        for name, argtypes in signatures.items():
            try:
                fn = getattr(lib, name)
            except AttributeError:
                raise KernelError(f"{path} has no entry point {name}") from None
            fn.argtypes = list(argtypes)
            fn.restype = ctypes.c_int
        return lib

    def stream_pointer(self) -> int:
        """The stream this step's kernels are launched on, as a kernel library takes it."""
        return self._stream()

    @staticmethod
    def check(rc: int, what: str) -> None:
        """Raises if an entry point of an extension returned an error code."""
        if rc != 0:
            raise KernelError(f"{what} failed with code {rc}")

    @staticmethod
    def _need(cond: bool, msg: str) -> None:
        if not cond:
            raise KernelError(msg)

    def fuses_norm(self, count: int, width: int, dtype: torch.dtype) -> bool:
        """Whether a bfloat16 step of ``count`` tokens of this width runs without norm kernels:
        the products that read the normalized residual stream normalize its rows themselves
        (``NormedRows`` for x), and ``linear_to_residual`` adds into the stream."""
        if dtype != torch.bfloat16:
            return False
        key = (int(count), int(width))
        ok = self._fuses.get(key)
        if ok is None:
            ok = self._fuses[key] = bool(self.lib.psamd_normed_supports(*key))
        return ok

    def normed(self, x: "torch.Tensor | NormedRows", name: str = "normed.x") -> torch.Tensor:
        """x as a tensor: rows handed over with their norm still to be applied go through the
        norm kernel now (for a consumer whose kernel does not normalize its tokens itself)."""
        if not isinstance(x, NormedRows):
            return x
        out = self.ws.get(name, x.shape, x.dtype)
        if x.rows is None:
            self.add_rmsnorm(x.residual, None, x.weight, x.eps, out)
        else:
            self.add_rmsnorm_rows(x.residual, None, x.rows, x.weight, x.eps, out)
        return out

    def _normed_args(self, x: NormedRows, k: int) -> tuple:
        self._need(x.residual.dtype == torch.float32 and x.residual.is_contiguous() and x.residual.shape[1] == k,
                   "rows to normalize must be float32 [T, K]")
        self._need(x.weight.numel() == k and x.weight.is_contiguous(), "the norm's weight must be [K]")
        if x.rows is not None:
            self._need(x.rows.dtype == torch.int32 and x.rows.is_contiguous(), "rows must be int32")
        return x.residual.data_ptr(), _ptr(x.rows), x.weight.data_ptr(), _code(x.weight.dtype), float(x.eps)

    def prepare_matrix(self, w: torch.Tensor, rt: Any) -> torch.Tensor:
        """A weight matrix on the device in the activation dtype (bfloat16 values widen to
        float32 exactly on the 32-bit path)."""
        return w.to(device=rt.device, dtype=rt.dtype).contiguous()

    # ------------------------------------------------------------ elementwise

    def embed(self, ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> None:
        t, h = out.shape
        self._need(ids.dtype == torch.int32 and ids.numel() == t, "embed: ids must be int32 [T]")
        self._need(table.shape[1] == h and out.dtype == torch.float32 and out.is_contiguous(), "embed: bad output")
        self._ok(self.lib.psamd_embed(self._stream(), ids.data_ptr(), table.data_ptr(), _code(table.dtype),
                                      out.data_ptr(), t, h, table.shape[0]))

    def _delta_args(self, delta, t: int, h: int, out_dtype: torch.dtype) -> tuple:
        """(pointer, dtype code, slices, stride) of a delta: [T, H] in the activation dtype, or
        [S, T, H] float32 partial sums of a K-split product."""
        if delta is None:
            return None, _F32, 0, 0
        self._need(delta.is_contiguous(), "delta must be contiguous")
        if delta.dim() == 3:
            self._need(delta.dtype == torch.float32 and delta.shape[1:] == (t, h), "partial sums must be float32 [S, T, H]")
            return delta.data_ptr(), _F32, delta.shape[0], t * h
        self._need(delta.shape == (t, h) and delta.dtype == out_dtype, "delta must match the output")
        return delta.data_ptr(), _code(delta.dtype), 1, 0

    def add_rmsnorm(self, residual, delta, weight, eps: float, out) -> None:
        t, h = residual.shape
        self._need(residual.dtype == torch.float32 and residual.is_contiguous(), "add_rmsnorm: residual must be float32")
        self._need(out.shape == (t, h) and out.is_contiguous(), "add_rmsnorm: bad output shape")
        self._need(weight.numel() == h, "add_rmsnorm: weight size")
        dptr, dcode, slices, stride = self._delta_args(delta, t, h, out.dtype)
        self._ok(self.lib.psamd_add_rmsnorm(self._stream(), residual.data_ptr(), dptr, dcode, slices, stride, None,
                                            weight.data_ptr(), _code(weight.dtype), eps, out.data_ptr(),
                                            _code(out.dtype), t, h))

    def add_rmsnorm_rows(self, residual, delta, rows, weight, eps: float, out) -> None:
        t, h = residual.shape
        s = rows.numel()
        self._need(residual.dtype == torch.float32 and rows.dtype == torch.int32, "add_rmsnorm_rows: dtypes")
        self._need(out.shape == (s, h) and out.is_contiguous(), "add_rmsnorm_rows: bad output shape")
        dptr, dcode, slices, stride = self._delta_args(delta, t, h, out.dtype)
        self._ok(self.lib.psamd_add_rmsnorm(self._stream(), residual.data_ptr(), dptr, dcode, slices, stride,
                                            rows.data_ptr(), weight.data_ptr(), _code(weight.dtype), eps,
                                            out.data_ptr(), _code(out.dtype), s, h))

    def swiglu(self, gate_up, out) -> None:
        t, inter = out.shape
        self._need(gate_up.shape == (t, 2 * inter) and gate_up.dtype == out.dtype, "swiglu: shapes")
        self._ok(self.lib.psamd_swiglu(self._stream(), gate_up.data_ptr(), out.data_ptr(), _code(out.dtype), t, inter))

    def rope_kv_append(self, qkv, hq: int, hkv: int, d: int, positions, table, kv, write_slot) -> None:
        t = qkv.shape[0]
        self._need(qkv.shape[1] == (hq + 2 * hkv) * d and qkv.is_contiguous(), "rope_kv_append: qkv shape")
        self._need(positions.dtype == torch.int32 and positions.numel() == t, "rope_kv_append: positions")
        if table is not None:
            self._need(table.dtype == torch.float32 and table.shape[1:] == (d // 2, 2) and table.is_contiguous(),
                       "rope_kv_append: table must be float32 [positions, D/2, 2]")
        if kv is not None:
            self._need(kv.dtype == qkv.dtype and kv.shape[1:] == (2, hkv, 16 * d) and kv.is_contiguous(),
                       "rope_kv_append: cache must be [blocks, 2, kv_heads, 16*D] in the activation dtype")
            self._need(write_slot.dtype == torch.int32 and write_slot.numel() == t, "rope_kv_append: write slots")
        self._ok(self.lib.psamd_rope_kv_append(self._stream(), qkv.data_ptr(), _code(qkv.dtype), t, hq, hkv, d,
                                               positions.data_ptr(), _ptr(table), _ptr(kv),
                                               None if kv is None else write_slot.data_ptr()))

    def qkv_rope_append(self, x, w_qkv, qkv, hq: int, hkv: int, d: int, positions, table, kv, write_slot) -> None:
        """qkv = x @ w_qkv^T, q and k rotated, k and v written to their pages. One kernel for a
        bfloat16 step of at most 64 tokens; otherwise the product followed by ``rope_kv_append``."""
        m, k = x.shape
        if isinstance(x, NormedRows):
            if (x.rows is None and d % 16 == 0 and qkv.dtype == torch.bfloat16 and self.fuses_norm(m, k, x.dtype)):
                resid, _rows, nw, nw_code, eps = self._normed_args(x, k)
                self._need(w_qkv.shape == ((hq + 2 * hkv) * d, k) and qkv.shape == (m, (hq + 2 * hkv) * d), "qkv: shapes")
                self._need(w_qkv.is_contiguous() and qkv.is_contiguous() and w_qkv.dtype == torch.bfloat16, "qkv: operands")
                self._need(positions.dtype == torch.int32 and positions.numel() == m, "qkv: positions")
                if table is not None:
                    self._need(table.dtype == torch.float32 and table.shape[1:] == (d // 2, 2) and table.is_contiguous(),
                               "qkv: table must be float32 [positions, D/2, 2]")
                if kv is not None:
                    self._need(kv.dtype == qkv.dtype and kv.shape[1:] == (2, hkv, 16 * d) and kv.is_contiguous(),
                               "qkv: cache must be [blocks, 2, kv_heads, 16*D] in the activation dtype")
                    self._need(write_slot.dtype == torch.int32 and write_slot.numel() == m, "qkv: write slots")
                self._ok(self.lib.psamd_qkv_rope_append_normed(
                    self._stream(), resid, nw, nw_code, eps, w_qkv.data_ptr(), qkv.data_ptr(), m, k, hq, hkv, d,
                    positions.data_ptr(), _ptr(table), _ptr(kv), None if kv is None else write_slot.data_ptr()))
                return
            x = self.normed(x)
        if (x.dtype == torch.bfloat16 and 0 < m <= self.SKINNY_MAX_ROWS and k % 8 == 0 and d % 16 == 0):
            self._need(w_qkv.shape == ((hq + 2 * hkv) * d, k) and qkv.shape == (m, (hq + 2 * hkv) * d), "qkv: shapes")
            self._need(x.is_contiguous() and w_qkv.is_contiguous() and qkv.is_contiguous(), "qkv: contiguous operands")
            self._need(positions.dtype == torch.int32 and positions.numel() == m, "qkv: positions")
            if table is not None:
                self._need(table.dtype == torch.float32 and table.shape[1:] == (d // 2, 2) and table.is_contiguous(),
                           "qkv: table must be float32 [positions, D/2, 2]")
            if kv is not None:
                self._need(kv.dtype == qkv.dtype and kv.shape[1:] == (2, hkv, 16 * d) and kv.is_contiguous(),
                           "qkv: cache must be [blocks, 2, kv_heads, 16*D] in the activation dtype")
                self._need(write_slot.dtype == torch.int32 and write_slot.numel() == m, "qkv: write slots")
            self._ok(self.lib.psamd_qkv_rope_append(self._stream(), x.data_ptr(), w_qkv.data_ptr(), qkv.data_ptr(), m, k,
                                                    hq, hkv, d, positions.data_ptr(), _ptr(table), _ptr(kv),
                                                    None if kv is None else write_slot.data_ptr()))
            return
        self.linear(x, w_qkv, qkv)
        self.rope_kv_append(qkv, hq, hkv, d, positions, table, kv, write_slot)

    # ---------------------------------------------------------------- products

    def linear(self, x, w, out) -> None:
        m, k = x.shape
        n = w.shape[0]
        if isinstance(x, NormedRows):
            if m > 0 and w.dtype == torch.bfloat16 and self.fuses_norm(m, k, x.dtype):
                resid, rows, nw, nw_code, eps = self._normed_args(x, k)
                self._need(w.shape[1] == k and out.shape == (m, n) and w.is_contiguous() and out.is_contiguous(), "linear: operands")
                self._ok(self.lib.psamd_linear_normed(self._stream(), resid, rows, nw, nw_code, eps, w.data_ptr(), out.data_ptr(),
                                                      _code(out.dtype), m, n, k, 0))
                return
            x = self.normed(x)
        self._need(w.shape[1] == k and out.shape == (m, n), f"linear: shapes {tuple(x.shape)} x {tuple(w.shape)}")
        self._need(x.is_contiguous() and w.is_contiguous() and out.is_contiguous(), "linear: contiguous operands")
        self._need(x.dtype == w.dtype, "linear: x and w must have one dtype")
        if m == 0:
            return
        if x.dtype == torch.bfloat16 and k % 8 == 0:
            if m > self.SKINNY_MAX_ROWS and self._direct_library:
                # Library product, as in the reference (float32 output for more than 64 rows of logits).
                rc = self.lib.psamd_gemm_lt(self._stream(), x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out.dtype),
                                            m, n, k, 0 if self.fixed_kv_len else 1, 0)
                if rc != 2:                      # 2: no algorithm for this shape (without a workspace): the paths below
                    self._ok(rc)
                    return
            if m <= self.SKINNY_MAX_ROWS or out.dtype == torch.float32:
                for r0 in range(0, m, self.SKINNY_MAX_ROWS):
                    r1 = min(m, r0 + self.SKINNY_MAX_ROWS)
                    self._ok(self.lib.psamd_linear_skinny(self._stream(), x[r0:r1].data_ptr(), w.data_ptr(),
                                                          out[r0:r1].data_ptr(), _code(out.dtype), r1 - r0, n, k, 0, 1))
                return
            if out.dtype == torch.bfloat16:
                torch.matmul(x, w.t(), out=out)
                return
        self._ok(self.lib.psamd_linear(self._stream(), x.data_ptr(), _code(x.dtype), w.data_ptr(), _code(w.dtype),
                                       out.data_ptr(), _code(out.dtype), m, n, k))

    def linear_to_residual(self, x, w, name: str, residual: torch.Tensor | None = None) -> torch.Tensor | None:
        """x @ w^T for a consumer that adds it to the residual stream (the fused add+norm).
        Returns [T, N] in the activation dtype or, for a small bfloat16 step whose product has
        few output columns, [S, T, N] float32 partial sums of a K-split, which the consumer adds
        up: splitting K over workgroups is what lets such a product use the whole chip. With the
        stream itself given as ``residual`` (float32 [T, N]), a step small enough to run without
        norm kernels adds the product into it here, K-slice by K-slice, and returns None."""
        m, k = x.shape
        n = w.shape[0]
        if (residual is not None and 0 < m and x.dtype == torch.bfloat16 and k % 8 == 0 and residual.shape == (m, n)
                and self.fuses_norm(m, n, x.dtype)):
            self._need(residual.dtype == torch.float32 and residual.is_contiguous(), "the residual stream is float32")
            self._need(w.shape[1] == k and x.is_contiguous() and w.is_contiguous(), "linear_to_residual: operands")
            self._ok(self.lib.psamd_linear_skinny_add(self._stream(), x.data_ptr(), w.data_ptr(), residual.data_ptr(), m, n, k))
            return None
        if (residual is not None and m >= self.LIBRARY_ADD_MIN_ROWS and x.dtype == torch.bfloat16 and k % 8 == 0
                and residual.shape == (m, n) and residual.dtype == torch.float32 and self._direct_library):
            # A large step: the library's product adds into the float32 stream itself (out = x w^T + out),
            # so the sum is not rounded to bfloat16 on its way there and the norm that follows reads the
            # stream alone (2,048 rows of the 1B shape: o + norm 32.9 -> 30.2 us, down + norm 78.5 -> 76.7;
            # at 512 rows down lost, 37.3 -> 40.7, hence the bound).
            self._need(w.shape[1] == k and x.is_contiguous() and w.is_contiguous() and residual.is_contiguous(),
                       "linear_to_residual: operands")
            rc = self.lib.psamd_gemm_lt(self._stream(), x.data_ptr(), w.data_ptr(), residual.data_ptr(), _F32, m, n, k,
                                        0 if self.fixed_kv_len else 1, 1)
            if rc != 2:                          # 2: no algorithm for this shape: the ways below
                self._ok(rc)
                return None
        if x.dtype == torch.bfloat16 and k % 8 == 0 and 0 < m <= self.SKINNY_MAX_ROWS:
            ksplit = self.lib.psamd_linear_skinny_ksplit(m, n, k)
            if ksplit > 1:
                self._need(w.shape[1] == k and x.is_contiguous() and w.is_contiguous(), "linear_to_residual: operands")
                # Room for the most slices of the most rows, so that the buffer never grows.
                self._need(ksplit <= 8, "linear_to_residual: more slices than there is room for")
                room = self.ws.get(name + ".slices", (8 * self.SKINNY_MAX_ROWS * n,), torch.float32)
                kept = self._slice_views.get((name, ksplit, m))
                if kept is None or kept[0] is not room:
                    kept = self._slice_views[(name, ksplit, m)] = (room, room[:ksplit * m * n].view(ksplit, m, n))
                out = kept[1]
                self._ok(self.lib.psamd_linear_skinny(self._stream(), x.data_ptr(), w.data_ptr(), out.data_ptr(),
                                                      _F32, m, n, k, 0, ksplit))
                return out
        out = self.ws.get(name, (m, n), x.dtype)
        self.linear(x, w, out)
        return out

    def linear_swiglu(self, x, w_gate_up, out) -> None:
        m, k = x.shape
        inter = out.shape[1]
        self._need(w_gate_up.shape == (2 * inter, k) and out.shape[0] == m, "linear_swiglu: shapes")
        if m == 0:
            return
        if isinstance(x, NormedRows):
            if w_gate_up.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and self.fuses_norm(m, k, x.dtype):
                resid, rows, nw, nw_code, eps = self._normed_args(x, k)
                self._need(w_gate_up.is_contiguous() and out.is_contiguous(), "linear_swiglu: operands")
                self._ok(self.lib.psamd_linear_normed(self._stream(), resid, rows, nw, nw_code, eps, w_gate_up.data_ptr(),
                                                      out.data_ptr(), _BF16, m, inter, k, 1))
                return
            x = self.normed(x)
        self._need(x.is_contiguous() and w_gate_up.is_contiguous() and out.is_contiguous(), "linear_swiglu: contiguous operands")
        small = x.dtype == torch.bfloat16 and k % 8 == 0 and m <= self.SKINNY_MAX_ROWS
        if small and m > self.FUSED_SWIGLU_MAX_ROWS and self._direct_library:
            # Between these row counts the library's product and the activation kernel behind it
            # take less time than the fused form, which streams the weights with too few rows a wave.
            gu = self.ws.get("mlp.gate_up", (m, 2 * inter), x.dtype)
            rc = self.lib.psamd_gemm_lt(self._stream(), x.data_ptr(), w_gate_up.data_ptr(), gu.data_ptr(), _BF16,
                                        m, 2 * inter, k, 0 if self.fixed_kv_len else 1, 0)
            if rc != 2:                          # 2: no algorithm for this shape: the fused form below
                self._ok(rc)
                self.swiglu(gu, out)
                return
        if small:
            self._ok(self.lib.psamd_linear_skinny(self._stream(), x.data_ptr(), w_gate_up.data_ptr(), out.data_ptr(),
                                                  _BF16, m, inter, k, 1, 1))
            return
        gu = self.ws.get("mlp.gate_up", (m, 2 * inter), x.dtype)
        self.linear(x, w_gate_up, gu)
        self.swiglu(gu, out)

    # --------------------------------------------------------------- attention

    def decode_is_skewed(self, count: int, longest: int, total: int) -> bool:
        """The library's rule for when the single-token items of a step have one context far
        longer than the rest (it then cuts every request's keys into long runs, as many as the
        longest needs). A captured decode step is keyed by it."""
        return bool(self.lib.psamd_attention_decode_skewed(int(count), int(longest), int(total)))

    def decode_plan(self, count: int, kv_len: int, skewed: bool, hkv: int, window: int) -> tuple[int, int]:
        """(runs per request, shortest run in keys) for a step of ``count`` single-token items."""
        plan = self._plans.get((count, kv_len, skewed, hkv, window))
        if plan is None:
            nsplit, min_run = ctypes.c_int(0), ctypes.c_int(0)
            self._ok(self.lib.psamd_attention_decode_plan(count, kv_len, int(skewed), hkv, window, ctypes.byref(nsplit),
                                                          ctypes.byref(min_run)))
            if len(self._plans) > 4096:
                self._plans.clear()
            plan = self._plans[(count, kv_len, skewed, hkv, window)] = (nsplit.value, min_run.value)
        return plan

    def mfma_attention_supported(self, hq: int, hkv: int, d: int) -> bool:
        return bool(self.lib.psamd_attention_mfma_supports(hq, hkv, d))

    def paged_attention(self, qkv, out, kv, ctx, group: int, hq: int, hkv: int, d: int, scale: float,
                        window: int | None) -> None:
        t = qkv.shape[0]
        g = ctx.groups[group]
        self._need(out.shape == (t, hq * d) and out.is_contiguous() and out.dtype == qkv.dtype, "attention: output")
        self._need(kv.dtype == qkv.dtype and kv.shape[1:] == (2, hkv, 16 * d) and kv.is_contiguous(),
                   "attention: cache must be [blocks, 2, kv_heads, 16*D] in the activation dtype")
        self._need(t == ctx.num_tokens, "attention: token count differs from the step batch")
        win = int(window) if window is not None else 0
        stride = qkv.shape[1]
        s = self._stream()
        if qkv.dtype == torch.bfloat16 and stride % 8 == 0 and self.mfma_attention_supported(hq, hkv, d):
            if ctx.num_prefill_tiles:
                kv_len = self.fixed_kv_len or ctx.max_kv_len
                # Few query tiles on a long context: the kernel deals their keys out to several
                # workgroups, whose partial results pass through these buffers. They are kept at
                # the most rows any step of this shape can need (the library says how many), so
                # they never grow.
                nsplit = self.lib.psamd_attention_prefill_nsplit(ctx.num_prefill_tiles, kv_len, hq, hkv, d)
                rows = self._bounds.get((hq, hkv, d))
                if rows is None:
                    rows = self._bounds[(hq, hkv, d)] = int(self.lib.psamd_attention_prefill_part_rows(hq, hkv, d))
                part_o = self.ws.get("attn.prefill_part_o", (rows * hq * d,), torch.float32)
                part_ml = self.ws.get("attn.prefill_part_ml", (rows * hq * 2,), torch.float32)
                if nsplit > 1:
                    self._need(32 * ctx.num_prefill_tiles * nsplit <= rows, "attention: more split tiles than planned for")
                self._ok(self.lib.psamd_attention_prefill(
                    s, qkv.data_ptr(), stride, out.data_ptr(), kv.data_ptr(), ctx.pf_tiles.data_ptr(),
                    ctx.num_prefill_tiles, ctx.pf_blocks.data_ptr(), ctx.num_prefill_blocks, kv_len,
                    ctx.item_start.data_ptr(), ctx.item_pos0.data_ptr(),
                    g.table_off.data_ptr(), g.block_ids.data_ptr(), hq, hkv, d, scale, win,
                    part_o.data_ptr() if nsplit > 1 else None, part_ml.data_ptr() if nsplit > 1 else None, nsplit))
            if ctx.num_decode:
                kv_len = self.fixed_kv_len or ctx.max_kv_len
                skewed = self.fixed_skew if self.fixed_kv_len else ctx.decode_skewed
                nsplit, min_run = self.decode_plan(ctx.num_decode, kv_len, skewed, hkv, win)
                # Room for the (request, run) pairs of any plan: asked for once, never grown.
                parts = self._bounds.get(ctx.num_decode)
                if parts is None:
                    parts = self._bounds[ctx.num_decode] = int(self.lib.psamd_attention_decode_max_parts(ctx.num_decode))
                self._need(ctx.num_decode * nsplit <= parts, "attention: more (request, run) pairs than planned for")
                part_o = self.ws.get("attn.part_o", (parts * hq * d,), torch.float32)
                part_ml = self.ws.get("attn.part_ml", (parts * hq * 2,), torch.float32)
                self._ok(self.lib.psamd_attention_decode(
                    s, qkv.data_ptr(), stride, out.data_ptr(), kv.data_ptr(), part_o.data_ptr(), part_ml.data_ptr(),
                    ctx.dec_items.data_ptr(), ctx.num_decode, ctx.item_start.data_ptr(),
                    ctx.item_end.data_ptr(), g.table_off.data_ptr(), g.block_ids.data_ptr(), hq, hkv, d, nsplit, scale,
                    win, min_run))
            return
        self._ok(self.lib.psamd_attention_generic(
            s, qkv.data_ptr(), stride, out.data_ptr(), kv.data_ptr(), _code(qkv.dtype), t, ctx.positions.data_ptr(),
            ctx.tok_item.data_ptr(), g.table_off.data_ptr(), g.block_ids.data_ptr(), hq, hkv, d, scale, win))

    # ---------------------------------------------------------------- sampling

    def sample(self, logits, temperatures, uniforms, out) -> None:
        rows, vocab = logits.shape
        self._need(logits.dtype == torch.float32 and logits.is_contiguous(), "sample: logits must be float32")
        self._need(temperatures.dtype == torch.float32 and uniforms.dtype == torch.float32 and
                   temperatures.numel() == rows and uniforms.numel() == rows, "sample: one temperature and uniform per row")
        self._need(out.dtype == torch.int32 and out.numel() == rows, "sample: output must be int32 [rows]")
        need = int(self.lib.psamd_sample_scratch_floats(rows))
        if self._sample_scratch is None or self._sample_scratch.numel() < need:
            # Kept apart from the workspace: growing it must not drop captured graphs.
            self._sample_scratch = torch.empty(max(need, 64 * 128), dtype=torch.float32, device=self.device)
        self._ok(self.lib.psamd_sample(self._stream(), logits.data_ptr(), temperatures.data_ptr(), uniforms.data_ptr(),
                                       out.data_ptr(), self._sample_scratch.data_ptr(), rows, vocab))

    def argmax(self, logits, out) -> None:
        rows = logits.shape[0]
        zeros = self.ws.get("sample.zeros", (rows,), torch.float32)
        zeros.zero_()
        self.sample(logits, zeros, zeros, out)
