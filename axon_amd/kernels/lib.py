"""The kernel library as Python calls: tensors in, launches on the current HIP stream.

`kernels(dtype)` loads (compiling at first use) the library of one compute dtype and wraps
each C entry point.  Wrappers check what the C side cannot see (dtypes, devices, contiguity)
and raise `KernelError` with the library's own message when a call is refused.  There is no
other implementation behind these calls: without the library they fail.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_void_p
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from . import build

MODE_STORE, MODE_ADD_F32, MODE_STORE_F32, MODE_SWIGLU = 0, 1, 2, 3


class KernelError(RuntimeError):
    pass


def _ptr(t: Optional[torch.Tensor]) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


def _stream() -> c_void_p:
    return c_void_p(torch.cuda.current_stream().cuda_stream)


# for the callers of `Kernels.call`: a tensor's (or a packed matrix's) address, the current stream
ptr, current_stream = _ptr, _stream
register_kernel_source = build.register_kernel_source


_SIGNATURES = {
    "axk_embed": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p],
    "axk_rmsnorm": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_void_p],
    "axk_rope_table": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "axk_rope_kv_write": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int,
                          c_int, c_int, c_int, c_int, c_int, c_void_p],
    "axk_gemm_qkv_rope_ok": [c_int, c_int, c_int, c_int, c_int],
    "axk_gemm_qkv_rope": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int,
                          c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                          c_int, c_void_p, ctypes.c_long, c_void_p],
    "axk_gemm_normed_ok": [c_int, c_int, c_int, c_int],
    "axk_gemm_normed_glu": [c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                            c_void_p],
    "axk_gemm_normed_qkv_rope": [c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int, c_void_p, c_int,
                                 c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int,
                                 c_int, c_int, c_int, c_int, c_void_p],
    "axk_attention": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int,
                      c_int, c_int, c_int, c_int, c_float, c_void_p],
    "axk_attention_prefill": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                              c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p],
    "axk_attention_decode": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                             c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                             c_float, c_void_p],
    "axk_attention_fast_ok": [c_int, c_int, c_int, c_int],
    "axk_gemm": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p,
                 ctypes.c_long, c_void_p],
    "axk_pack_ok": [c_int, c_int, c_int],
    "axk_pack_matrix": [c_void_p, c_void_p, c_int, c_int, c_void_p],
    "axk_gemm_segments": [c_int, c_int, c_int],
    "axk_gemm_then_norm_ok": [c_int, c_int, c_int],
    "axk_gemm_then_norm": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int,
                           c_float, c_void_p, c_void_p, ctypes.c_long, c_void_p],
    "axk_swiglu": [c_void_p, c_void_p, c_int, c_int, c_void_p],
    "axk_argmax": [c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_void_p],
    "axk_topk": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                 c_void_p, c_void_p],
    "axk_topk_workspace": [c_int, c_int, c_int],
    "axk_fill_i32": [c_void_p, c_int, c_int, c_void_p],
    "axk_fill_f32": [c_void_p, c_float, c_int, c_void_p],
}


class PackedMatrix:
    """A [rows, cols] matrix in the layout the matrix-core products read: blocks of 16 rows x 32
    columns, each 1 KB in the order in which a wave holds them as an MFMA operand, ordered
    [row tile][column block]; rows padded with zeros to a multiple of 16.  `data` is the flat
    storage.  A leading slice of whole row tiles is a view."""

    def __init__(self, data: torch.Tensor, rows: int, cols: int):
        self.data, self.rows, self.cols = data, rows, cols

    @property
    def shape(self):
        return (self.rows, self.cols)

    @property
    def dtype(self):
        return self.data.dtype

    def data_ptr(self) -> int:
        return self.data.data_ptr()

    def __getitem__(self, rows) -> "PackedMatrix":
        if not isinstance(rows, slice) or rows.start not in (None, 0) or rows.step not in (None, 1):
            raise KernelError("a packed matrix gives only its leading rows")
        n = self.rows if rows.stop is None else int(rows.stop)
        if not 0 < n <= self.rows or (n % 16 and n != self.rows):
            raise KernelError(f"a packed matrix of {self.rows} rows is cut at multiples of 16, not at {n}")
        return PackedMatrix(self.data[:-(-n // 16) * 16 * self.cols], n, self.cols)


class Kernels:
    """One loaded kernel library.  `dtype` is the torch dtype of `elem` tensors."""

    def __init__(self, dtype_name: str):
        self.dtype_name = dtype_name
        self.dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype_name]
        self.path = build.build_kernels(dtype_name)
        self.lib = ctypes.CDLL(self.path, mode=ctypes.RTLD_LOCAL)
        self.lib.axk_last_error.restype = c_char_p
        for name, args in _SIGNATURES.items():
            fn = getattr(self.lib, name)
            fn.argtypes = args
            fn.restype = c_int
        self.lib.axk_attention_decode_workspace.argtypes = [c_int, c_int, c_int, c_int]
        self.lib.axk_attention_decode_workspace.restype = ctypes.c_long
        self.lib.axk_packed_elems.argtypes = [c_int, c_int]
        self.lib.axk_packed_elems.restype = ctypes.c_long
        self.lib.axk_gemm_workspace.argtypes = [c_int, c_int, c_int, c_int]
        self.lib.axk_gemm_workspace.restype = ctypes.c_long
        self.lib.axk_topk_workspace.restype = ctypes.c_long
        self.lib.axk_argmax_workspace.argtypes = [c_int, c_int]
        self.lib.axk_argmax_workspace.restype = ctypes.c_long
        self.lib.axk_instances.argtypes = [c_char_p, ctypes.c_long, c_int]
        self.lib.axk_instances.restype = ctypes.c_long
        self.lib.axk_instances_reset.argtypes = []
        self.lib.axk_instances_reset.restype = None
        if bool(self.lib.axk_is_bf16()) != (dtype_name == "bfloat16"):
            raise KernelError(f"{self.path} was not built for {dtype_name}")
        self._extensions: Dict[str, ctypes.CDLL] = {}      # a registered source's path -> its library
        self._chunk_factor = None

    # ------------------------------------------------------------------ a part's own kernels
    def call(self, name: str, *args) -> None:
        """Call the entry point `name` of a kernel source that a part registered
        (`register_kernel_source(path, {name: argument types})`); its library is compiled for this
        compute dtype and loaded at the first call.  Arguments as ctypes takes them (`ptr(tensor)`,
        `current_stream()`, ints, floats).  A refusal raises `KernelError` with the library's message."""
        for path, signatures in build.registered_kernel_sources().items():
            if name in signatures:
                break
        else:
            raise KernelError(f"no registered kernel source has an entry point '{name}'")
        lib = self._extensions.get(path)
        if lib is None:
            lib = ctypes.CDLL(build.build_extension(path, self.dtype_name), mode=ctypes.RTLD_LOCAL)
            lib.axk_last_error.restype = c_char_p
            if bool(lib.axk_is_bf16()) != (self.dtype_name == "bfloat16"):
                raise KernelError(f"the library of {path} was not built for {self.dtype_name}")
            for entry, argtypes in signatures.items():
                fn = getattr(lib, entry)
                fn.argtypes, fn.restype = list(argtypes), c_int
            self._extensions[path] = lib
        if getattr(lib, name)(*args) != 0:
            raise KernelError(lib.axk_last_error().decode())

    # ------------------------------------------------------------------ helpers
    def _check(self, rc: int) -> None:
        if rc != 0:
            raise KernelError(self.lib.axk_last_error().decode())

    def instances(self, launched: bool = False) -> List[str]:
        """The kernel instances compiled into the library (the instances of the templates that the
        dispatches choose from), or those `launched` since `reset_instances`."""
        need = self.lib.axk_instances(None, 0, 1 if launched else 0)
        buf = ctypes.create_string_buffer(need)
        self.lib.axk_instances(buf, need, 1 if launched else 0)
        return [n for n in buf.value.decode().split("\n") if n]

    def reset_instances(self) -> None:
        self.lib.axk_instances_reset()

    # what launches kernels: wrapped while a step is profiled
    _LAUNCHING = ("embed", "rmsnorm", "rope_table", "rope_kv_write", "gemm_qkv_rope", "attention", "attention_prefill",
                  "attention_decode", "gemm", "gemm_normed_glu", "gemm_normed_qkv_rope", "swiglu", "argmax", "topk",
                  "fill_i32", "fill_f32", "call")
    _MATRIX_AT = {"gemm": 1, "gemm_qkv_rope": 1, "gemm_normed_glu": 3, "gemm_normed_qkv_rope": 3}   # which argument is W

    def set_launch_hook(self, hook) -> None:
        """`hook(name, matrix_bytes)` is told of every call that has launched kernels, with the
        bytes of the weight matrix it read (0 if none), as the reference's launch sites tell
        theirs (src/cuda/qwen2.rs:2294, 2361-2449); None: off."""
        for name in self._LAUNCHING:
            self.__dict__.pop(name, None)
        if hook is None:
            return
        for name in self._LAUNCHING:
            plain = getattr(type(self), name)

            def told(*a, _plain=plain, _name=name, **kw):
                out = _plain(self, *a, **kw)
                label, nbytes = (str(a[0]) if _name == "call" else _name), 0
                if _name in self._MATRIX_AT:
                    w = a[self._MATRIX_AT[_name]]
                    data = w.data if isinstance(w, PackedMatrix) else w
                    nbytes = data.numel() * data.element_size()
                    label = f"{_name} {w.shape[0]}x{w.shape[1]}"
                hook(label, nbytes)
                return out
            self.__dict__[name] = told

    def _elem(self, t: torch.Tensor, what: str) -> None:
        if t.dtype != self.dtype or not t.is_cuda:
            raise KernelError(f"{what}: expected a {self.dtype_name} device tensor, got {t.dtype} on {t.device}")

    @staticmethod
    def _f32(t: torch.Tensor, what: str) -> None:
        if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous():
            raise KernelError(f"{what}: expected a contiguous float32 device tensor, got {t.dtype} on {t.device}")

    @staticmethod
    def _i32(t: torch.Tensor, what: str) -> None:
        if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
            raise KernelError(f"{what}: expected a contiguous int32 device tensor, got {t.dtype} on {t.device}")

    @staticmethod
    def _vec_flag(v: Optional[torch.Tensor], what: str) -> int:
        if v is None:
            return 1
        if v.dtype not in (torch.float32, torch.bfloat16) or not v.is_cuda or not v.is_contiguous():
            raise KernelError(f"{what}: a vector must be float32 or bfloat16 on the device, got {v.dtype}")
        return 1 if v.dtype == torch.float32 else 0

    def _check_caches(self, k_cache, v_cache, n_kv_heads, page_size, head_dim) -> None:
        """Keys are [pages, kv heads, page_size, head_dim]; values are kept position-contiguous:
        [pages, kv heads, head_dim, page_size]."""
        self._elem(k_cache, "k cache"); self._elem(v_cache, "v cache")
        if (k_cache.dim() != 4 or tuple(k_cache.shape[1:]) != (n_kv_heads, page_size, head_dim)
                or not k_cache.is_contiguous()):
            raise KernelError(f"key cache {tuple(k_cache.shape)} is not [pages, {n_kv_heads}, {page_size}, {head_dim}]")
        if (v_cache.dim() != 4 or tuple(v_cache.shape[1:]) != (n_kv_heads, head_dim, page_size)
                or not v_cache.is_contiguous() or v_cache.shape[0] != k_cache.shape[0]):
            raise KernelError(f"value cache {tuple(v_cache.shape)} is not [pages, {n_kv_heads}, {head_dim}, {page_size}]")

    # ------------------------------------------------------------------ ops
    def embed(self, tokens: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        packed = isinstance(table, PackedMatrix)
        self._i32(tokens, "embed tokens"); self._elem(table.data if packed else table, "embed table")
        self._f32(out, "embed out")
        vocab, dim = table.shape
        if out.shape != (tokens.numel(), dim) or not (packed or table.is_contiguous()):
            raise KernelError(f"embed: out {tuple(out.shape)} does not fit {tokens.numel()} tokens of width {dim}")
        self._check(self.lib.axk_embed(_ptr(tokens), _ptr(table), 1 if packed else 0, _ptr(out), tokens.numel(), dim,
                                       vocab, _stream()))
        return out

    def rmsnorm(self, x: torch.Tensor, gain: torch.Tensor, eps: float, out: torch.Tensor,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        self._f32(x, "rmsnorm x"); self._elem(out, "rmsnorm out")
        dim = x.shape[-1]
        n = out.shape[0]
        if rows is not None:
            self._i32(rows, "rmsnorm rows")
            if rows.numel() != n:
                raise KernelError(f"rmsnorm: {rows.numel()} row indices for {n} output rows")
        elif x.shape[0] != n:
            raise KernelError(f"rmsnorm: {x.shape[0]} rows in, {n} rows out")
        if gain.numel() != dim or out.shape[-1] != dim or not out.is_contiguous():
            raise KernelError(f"rmsnorm: width {dim}, gain {gain.numel()}, out {tuple(out.shape)}")
        self._check(self.lib.axk_rmsnorm(_ptr(x), _ptr(rows), _ptr(gain), self._vec_flag(gain, "rmsnorm gain"),
                                         _ptr(out), n, dim, float(eps), _stream()))
        return out

    def rope_table(self, positions: torch.Tensor, freqs: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        self._i32(positions, "rope positions"); self._f32(out, "rope table")
        if freqs.dtype != torch.float64 or not freqs.is_cuda:
            raise KernelError("rope_table: frequencies must be float64 on the device")
        if out.shape != (positions.numel(), freqs.numel(), 2):
            raise KernelError(f"rope_table: table {tuple(out.shape)} for {positions.numel()} x {freqs.numel()} pairs")
        self._check(self.lib.axk_rope_table(_ptr(positions), _ptr(freqs), _ptr(out), positions.numel(), freqs.numel(),
                                            _stream()))
        return out

    def rope_kv_write(self, qkv, table, positions, seq_rows, block_table, k_cache, v_cache, n_heads, n_kv_heads,
                      head_dim, rotary_dim, page_size, write_kv=True) -> None:
        self._elem(qkv, "rope qkv"); self._f32(table, "rope table")
        self._i32(positions, "positions"); self._i32(seq_rows, "seq_rows"); self._i32(block_table, "block_table")
        T = positions.numel()
        width = (n_heads + 2 * n_kv_heads) * head_dim
        if qkv.shape != (T, width) or not qkv.is_contiguous():
            raise KernelError(f"rope_kv_write: qkv {tuple(qkv.shape)} is not [{T}, {width}] contiguous")
        if table.shape != (T, rotary_dim // 2, 2):
            raise KernelError(f"rope_kv_write: table {tuple(table.shape)} for rotary_dim {rotary_dim}")
        if write_kv:
            self._check_caches(k_cache, v_cache, n_kv_heads, page_size, head_dim)
        self._check(self.lib.axk_rope_kv_write(
            _ptr(qkv), _ptr(table), _ptr(positions), _ptr(seq_rows), _ptr(block_table), block_table.shape[-1],
            _ptr(k_cache if write_kv else None), _ptr(v_cache if write_kv else None), T, n_heads, n_kv_heads, head_dim,
            rotary_dim, page_size, 1 if write_kv else 0, _stream()))

    def gemm_qkv_rope_ok(self, m: int, n: int, k: int, head_dim: int, rotary_dim: int) -> bool:
        """Whether `gemm_qkv_rope` takes a step of m tokens and a matrix of n rows of these sizes."""
        return bool(self.lib.axk_gemm_qkv_rope_ok(m, n, k, head_dim, rotary_dim))

    def gemm_qkv_rope(self, x, w, bias, qkv, table, positions, seq_rows, block_table, k_cache, v_cache, n_heads,
                      n_kv_heads, head_dim, page_size, write_kv=True) -> None:
        """The [q; k; v] product, the rotary encoding and the store into the pages in one launch
        (up to 16 tokens) or with the kernel that adds a product's segments doing the rest:
        the same bits as `gemm` into qkv followed by `rope_kv_write`.  q lands in qkv[:, :n_heads *
        head_dim]; the k and v columns of qkv are not written.  Without write_kv, w holds the q
        rows only."""
        if not isinstance(w, PackedMatrix):
            raise KernelError("gemm_qkv_rope: needs a packed matrix")
        self._elem(x, "qkv x"); self._elem(w.data, "qkv w"); self._elem(qkv, "qkv out"); self._f32(table, "rope table")
        self._i32(positions, "positions"); self._i32(seq_rows, "seq_rows"); self._i32(block_table, "block_table")
        M, K = x.shape
        rows = (n_heads + (2 * n_kv_heads if write_kv else 0)) * head_dim
        if w.shape != (rows, K) or x.stride(1) != 1:
            raise KernelError(f"gemm_qkv_rope: x {tuple(x.shape)} w {tuple(w.shape)}, expected w [{rows}, {K}]")
        if qkv.shape[0] != M or qkv.shape[1] < n_heads * head_dim or qkv.stride(1) != 1:
            raise KernelError(f"gemm_qkv_rope: qkv {tuple(qkv.shape)} does not hold [{M}, {n_heads * head_dim}]")
        if table.shape != (M, head_dim // 2, 2) or positions.numel() != M or seq_rows.numel() != M:
            raise KernelError(f"gemm_qkv_rope: table {tuple(table.shape)} or positions do not fit {M} tokens")
        if bias is not None and bias.numel() != rows:
            raise KernelError(f"gemm_qkv_rope: bias of {bias.numel()} for {rows} rows")
        if write_kv:
            self._check_caches(k_cache, v_cache, n_kv_heads, page_size, head_dim)
        need = self.lib.axk_gemm_workspace(M, rows, K, MODE_STORE)
        work = torch.empty(need // 4, dtype=torch.float32, device=x.device) if need > 0 else None
        self._check(self.lib.axk_gemm_qkv_rope(
            _ptr(x), x.stride(0), _ptr(w), _ptr(bias), self._vec_flag(bias, "qkv bias"), _ptr(qkv), qkv.stride(0), M, K,
            _ptr(table), _ptr(positions), _ptr(seq_rows), _ptr(block_table),
            block_table.shape[-1], _ptr(k_cache if write_kv else None), _ptr(v_cache if write_kv else None), n_heads,
            n_kv_heads, head_dim, page_size, 1 if write_kv else 0, _ptr(work), need, _stream()))

    def gemm_normed_ok(self, m: int, n: int, k: int, gated: bool = False, gain=None) -> bool:
        """Whether the product of m rows with a packed [n, k] matrix (gated: [gate; up] of 2 n rows)
        takes the RMS norm of its operand inside (`gemm_normed_glu`, `gemm_normed_qkv_rope`); with
        `gain`, also whether that gain is one the kernels take (bfloat16)."""
        if gain is not None and gain.dtype != torch.bfloat16:
            return False
        return bool(self.lib.axk_gemm_normed_ok(m, n, k, 1 if gated else 0))

    def _normed_rows(self, rows, gain, K, what):
        if rows.dtype != torch.float32 or not rows.is_cuda:
            raise KernelError(f"{what}: the rows must be float32 on the device, got {rows.dtype} on {rows.device}")
        if rows.dim() != 2 or rows.shape[1] != K or rows.stride(1) != 1 or gain.numel() != K or not gain.is_contiguous():
            raise KernelError(f"{what}: rows {tuple(rows.shape)} or a gain of {gain.numel()} do not fit K={K}")

    def gemm_normed_glu(self, rows, gain, eps, w, out) -> torch.Tensor:
        """out = silu(X Wg^T) * (X Wu^T) with X = rmsnorm(rows, gain, eps) worked out inside the
        kernel (few rows; `gemm_normed_ok`): the same bits as `rmsnorm` followed by `gemm` in the
        gated mode."""
        if not isinstance(w, PackedMatrix):
            raise KernelError("gemm_normed_glu: needs a packed matrix")
        M, K = rows.shape
        N = w.shape[0] // 2
        self._normed_rows(rows, gain, K, "gemm_normed_glu")
        self._elem(w.data, "gate|up w"); self._elem(out, "gate|up out")
        if w.shape != (2 * N, K) or out.shape != (M, N) or out.stride(1) != 1:
            raise KernelError(f"gemm_normed_glu: w {tuple(w.shape)} out {tuple(out.shape)} for rows {tuple(rows.shape)}")
        self._check(self.lib.axk_gemm_normed_glu(_ptr(rows), rows.stride(0), _ptr(gain), self._vec_flag(gain, "norm gain"),
                                                 float(eps), _ptr(w), _ptr(out), out.stride(0), M, N, K, _stream()))
        return out

    def gemm_normed_qkv_rope(self, rows, gain, eps, w, bias, qkv, table, positions, seq_rows, block_table, k_cache, v_cache,
                             n_heads, n_kv_heads, head_dim, page_size, write_kv=True) -> None:
        """`gemm_qkv_rope` of X = rmsnorm(rows, gain, eps), X worked out inside the kernel (few
        rows; `gemm_normed_ok`): the same bits as `rmsnorm` followed by `gemm_qkv_rope`."""
        if not isinstance(w, PackedMatrix):
            raise KernelError("gemm_normed_qkv_rope: needs a packed matrix")
        M, K = rows.shape
        self._normed_rows(rows, gain, K, "gemm_normed_qkv_rope")
        self._elem(w.data, "qkv w"); self._elem(qkv, "qkv out"); self._f32(table, "rope table")
        self._i32(positions, "positions"); self._i32(seq_rows, "seq_rows"); self._i32(block_table, "block_table")
        n = (n_heads + (2 * n_kv_heads if write_kv else 0)) * head_dim
        if w.shape != (n, K):
            raise KernelError(f"gemm_normed_qkv_rope: w {tuple(w.shape)}, expected [{n}, {K}]")
        if qkv.shape[0] != M or qkv.shape[1] < n_heads * head_dim or qkv.stride(1) != 1:
            raise KernelError(f"gemm_normed_qkv_rope: qkv {tuple(qkv.shape)} does not hold [{M}, {n_heads * head_dim}]")
        if table.shape != (M, head_dim // 2, 2) or positions.numel() != M or seq_rows.numel() != M:
            raise KernelError(f"gemm_normed_qkv_rope: table {tuple(table.shape)} or positions do not fit {M} tokens")
        if bias is not None and bias.numel() != n:
            raise KernelError(f"gemm_normed_qkv_rope: bias of {bias.numel()} for {n} rows")
        if write_kv:
            self._check_caches(k_cache, v_cache, n_kv_heads, page_size, head_dim)
        self._check(self.lib.axk_gemm_normed_qkv_rope(
            _ptr(rows), rows.stride(0), _ptr(gain), self._vec_flag(gain, "norm gain"), float(eps), _ptr(w), _ptr(bias),
            self._vec_flag(bias, "qkv bias"), _ptr(qkv), qkv.stride(0), M, K, _ptr(table), _ptr(positions), _ptr(seq_rows),
            _ptr(block_table), block_table.shape[-1], _ptr(k_cache if write_kv else None),
            _ptr(v_cache if write_kv else None), n_heads, n_kv_heads, head_dim, page_size, 1 if write_kv else 0, _stream()))

    def attention(self, q, q_stride, k_cache, v_cache, block_table, positions, seq_rows, out, n_heads, n_kv_heads,
                  head_dim, page_size, window, scale) -> torch.Tensor:
        self._elem(q, "attention q"); self._elem(k_cache, "k cache"); self._elem(v_cache, "v cache")
        self._elem(out, "attention out")
        self._i32(positions, "positions"); self._i32(seq_rows, "seq_rows"); self._i32(block_table, "block_table")
        T = positions.numel()
        if out.shape != (T, n_heads * head_dim) or not out.is_contiguous():
            raise KernelError(f"attention: out {tuple(out.shape)} is not [{T}, {n_heads * head_dim}]")
        self._check_caches(k_cache, v_cache, n_kv_heads, page_size, head_dim)
        self._check(self.lib.axk_attention(
            _ptr(q), q_stride, _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[-1], _ptr(positions),
            _ptr(seq_rows), _ptr(out), T, n_heads, n_kv_heads, head_dim, page_size, window, float(scale), _stream()))
        return out

    def attention_fast_ok(self, head_dim: int, page_size: int, n_heads: int, n_kv_heads: int) -> bool:
        """Whether the matrix-core attention kernels take these sizes (never in float32)."""
        return bool(self.lib.axk_attention_fast_ok(head_dim, page_size, n_heads, n_kv_heads))

    def attention_prefill(self, q, q_stride, k_cache, v_cache, block_table, positions, seq_rows, out, tiles, n_heads,
                          n_kv_heads, head_dim, page_size, window, scale) -> torch.Tensor:
        """Attention of prompt portions: tiles [n, 4] int32 = (first token, count <= 128) twice, the
        two runs of tokens one block takes one after the other (second count 0: none); [n, 2]
        is taken as one run a block.  `pair_tiles` pairs runs so that blocks get equal work."""
        self._elem(q, "attention q"); self._elem(out, "attention out")
        self._check_caches(k_cache, v_cache, n_kv_heads, page_size, head_dim)
        self._i32(positions, "positions"); self._i32(seq_rows, "seq_rows"); self._i32(block_table, "block_table")
        self._i32(tiles, "tiles")
        if tiles.dim() == 2 and tiles.shape[1] == 2:
            tiles = torch.cat([tiles, torch.zeros_like(tiles)], dim=1).contiguous()
        if (out.shape[1] != n_heads * head_dim or not out.is_contiguous() or tiles.dim() != 2 or tiles.shape[1] != 4
                or not tiles.is_contiguous()):
            raise KernelError(f"attention_prefill: out {tuple(out.shape)}, tiles {tuple(tiles.shape)}")
        self._check(self.lib.axk_attention_prefill(
            _ptr(q), q_stride, _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[-1], _ptr(positions),
            _ptr(seq_rows), _ptr(out), _ptr(tiles), tiles.shape[0], n_heads, n_kv_heads, head_dim, page_size, window,
            float(scale), _stream()))
        return out

    @property
    def attention_prefill_tile(self) -> int:
        """The most consecutive tokens of one request in a run of `attention_prefill`'s tiles."""
        return int(self.lib.axk_attention_prefill_tile())

    def _decode_chunk_and_factor(self):
        if self._chunk_factor is None:
            self._chunk_factor = (int(self.lib.axk_attention_decode_chunk()), int(self.lib.axk_attention_decode_item_factor()))
        return self._chunk_factor

    @property
    def attention_decode_chunk(self) -> int:
        """Positions of one chunk of the decoding kernel: a token's range (from the chunk that
        holds the window's first position, or 0) is cut into chunks of this size."""
        return int(self.lib.axk_attention_decode_chunk())

    @property
    def attention_decode_max_context(self) -> int:
        """The longest context the decoding kernel's work list can name."""
        return self.attention_decode_chunk * int(self.lib.axk_attention_decode_item_factor())

    def attention_decode_workspace(self, n_tokens: int, n_heads: int, head_dim: int, max_chunks: int) -> int:
        return int(self.lib.axk_attention_decode_workspace(n_tokens, n_heads, head_dim, max_chunks))

    def attention_decode_work(self, positions: Sequence[int], window: int, pad_to: int = 0) -> List[int]:
        """The work list of the decoding kernel for single tokens at `positions` (in the order
        of their slots): one item per (token, chunk), slot * factor + chunk, a token's chunks
        side by side; padded with -1 to `pad_to` items."""
        chunk, factor = self._decode_chunk_and_factor()
        pos = np.asarray(positions, dtype=np.int64)
        lo = np.maximum(0, pos + 1 - window) if window > 0 else np.zeros_like(pos)
        n = (pos - lo // chunk * chunk) // chunk + 1
        if n.size and int(n.max()) > factor:
            raise KernelError(f"attention_decode: a context of {int(pos.max()) + 1} positions is more than {factor} chunks")
        total = int(n.sum())
        first = np.cumsum(n) - n                                   # where each token's items start
        items = np.repeat(np.arange(pos.size, dtype=np.int64) * factor - first, n) + np.arange(total, dtype=np.int64)
        out = np.full(max(total, pad_to), -1, dtype=np.int32)
        out[:total] = items
        return out.tolist()

    def attention_decode(self, q, q_stride, k_cache, v_cache, block_table, positions, seq_rows, out, token_index,
                         partial, max_chunks, n_heads, n_kv_heads, head_dim, page_size, window, scale,
                         work: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Attention of single decoding tokens named by token_index (int32), or of the first
        `token_index` tokens of the step if that is a number.  `work` (int32, on the device):
        the chunks to compute, as `attention_decode_work` lists them; None: made here from the
        positions, which waits for the device."""
        self._elem(q, "attention q"); self._elem(out, "attention out")
        self._check_caches(k_cache, v_cache, n_kv_heads, page_size, head_dim)
        self._i32(positions, "positions"); self._i32(seq_rows, "seq_rows"); self._i32(block_table, "block_table")
        if isinstance(token_index, int):
            n, token_index = token_index, None
        else:
            self._i32(token_index, "token_index")
            n = token_index.numel()
        if n > q.shape[0]:
            raise KernelError(f"attention_decode: {n} tokens, q has {q.shape[0]} rows")
        if out.shape[1] != n_heads * head_dim or not out.is_contiguous():
            raise KernelError(f"attention_decode: out {tuple(out.shape)}")
        self._f32(partial, "attention partial")
        if partial.numel() < self.attention_decode_workspace(n, n_heads, head_dim, max_chunks):
            raise KernelError(f"attention_decode: workspace of {partial.numel()} floats is too small")
        if work is None:
            at = positions[:n] if token_index is None else positions[token_index.long()]
            work = torch.tensor(self.attention_decode_work(at.tolist(), window), dtype=torch.int32).to(q.device)
        self._i32(work, "attention work list")
        if work.dim() != 1 or not work.is_contiguous():
            raise KernelError(f"attention_decode: work list {tuple(work.shape)}")
        self._check(self.lib.axk_attention_decode(
            _ptr(q), q_stride, _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[-1], _ptr(positions),
            _ptr(seq_rows), _ptr(out), _ptr(token_index), n, _ptr(work), work.numel(),
            _ptr(partial), max_chunks, n_heads, n_kv_heads, head_dim, page_size, window,
            float(scale), _stream()))
        return out

    def pack_ok(self, rows: int, cols: int, gated: bool = False) -> bool:
        """Whether a [rows, cols] matrix can be packed for the matrix-core products (gated: a
        [gate; up] matrix for the SwiGLU epilogue).  Never in the float32 build."""
        return bool(self.lib.axk_pack_ok(rows, cols, 1 if gated else 0))

    def pack_matrix(self, w: torch.Tensor) -> PackedMatrix:
        self._elem(w, "pack_matrix")
        if w.dim() != 2 or not w.is_contiguous() or not self.pack_ok(w.shape[0], w.shape[1]):
            raise KernelError(f"pack_matrix: {tuple(w.shape)} cannot be packed")
        rows, cols = w.shape
        out = torch.empty(self.lib.axk_packed_elems(rows, cols), dtype=w.dtype, device=w.device)
        self._check(self.lib.axk_pack_matrix(_ptr(w), _ptr(out), rows, cols, _stream()))
        return PackedMatrix(out, rows, cols)

    def prepare_weight(self, w: torch.Tensor, gated: bool = False):
        """A weight matrix as the products want it: packed where that is possible (then the
        row-major tensor is no longer needed), else as it is."""
        if isinstance(w, torch.Tensor) and w.dim() == 2 and self.pack_ok(w.shape[0], w.shape[1], gated):
            return self.pack_matrix(w.contiguous())
        return w

    def gemm_then_norm_ok(self, m: int, n: int, k: int) -> bool:
        """Whether the product that adds into [m, n] float32 rows can also write the RMS norm of
        the new rows (see `gemm`: `following_norm`)."""
        return bool(self.lib.axk_gemm_then_norm_ok(m, n, k))

    def gemm_segments(self, n: int, k: int, gated: bool = False) -> int:
        """The number of contiguous segments of K whose sums a product with a packed [n, k]
        matrix adds in ascending order (gated: a [gate; up] matrix for n output columns).  It
        depends on the matrix alone: a row's bits do not depend on the other rows of a step."""
        return int(self.lib.axk_gemm_segments(n, k, 1 if gated else 0))

    def gemm(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None,
             mode: int = MODE_STORE, following_norm=None) -> torch.Tensor:
        """out = epilogue(x . w^T + bias); x [M, K] (rows may be strided), w [N, K] contiguous or
        a PackedMatrix (the matrix-core kernels; a row-major w goes to the 32-bit FMA kernel).
        MODE_SWIGLU: w is [2 N, K], gate rows then up rows; out [M, N] = silu(x gate^T) * (x up^T).

        `following_norm` = (gain, values [M, N], eps) with MODE_ADD_F32, where `gemm_then_norm_ok`:
        the kernel that finishes the product also writes the RMS norm of the new rows,
        values = out / sqrt(mean(out^2) + eps) * gain, the same bits as `rmsnorm` after it."""
        packed = isinstance(w, PackedMatrix)
        self._elem(x, "gemm x"); self._elem(w.data if packed else w, "gemm w")
        M, K = x.shape
        N = w.shape[0]
        if mode == MODE_SWIGLU:
            if N % 2 or bias is not None:
                raise KernelError("gemm: the gated epilogue needs gate and up rows and takes no bias")
            N //= 2
        if w.shape[1] != K or not (packed or w.is_contiguous()) or x.stride(1) != 1 or out.stride(1) != 1:
            raise KernelError(f"gemm: x {tuple(x.shape)} w {tuple(w.shape)} do not multiply, or are not row-major")
        if out.shape != (M, N) or not out.is_cuda:
            raise KernelError(f"gemm: out {tuple(out.shape)} is not [{M}, {N}]")
        want = self.dtype if mode in (MODE_STORE, MODE_SWIGLU) else torch.float32
        if out.dtype != want:
            raise KernelError(f"gemm: mode {mode} writes {want}, out is {out.dtype}")
        if bias is not None and bias.numel() != N:
            raise KernelError(f"gemm: bias of {bias.numel()} for {N} columns")
        need = self.lib.axk_gemm_workspace(M, N, K, mode) if packed else 0
        work = torch.empty(need // 4, dtype=torch.float32, device=x.device) if need > 0 else None
        if following_norm is None:
            self._check(self.lib.axk_gemm(_ptr(x), x.stride(0), _ptr(w), 1 if packed else 0, _ptr(bias),
                                          self._vec_flag(bias, "gemm bias"), _ptr(out), out.stride(0), M, N, K, mode,
                                          _ptr(work), need, _stream()))
            return out
        gain, values, norm_eps = following_norm
        self._elem(values, "gemm norm values")
        if not packed or mode != MODE_ADD_F32:
            raise KernelError("gemm: a norm follows only the product with a packed matrix that adds into float32 rows")
        if gain.numel() != N or values.shape != (M, N) or not values.is_contiguous():
            raise KernelError(f"gemm: the following norm's gain {tuple(gain.shape)} or values "
                              f"{tuple(values.shape)} do not fit [{M}, {N}]")
        self._check(self.lib.axk_gemm_then_norm(
            _ptr(x), x.stride(0), _ptr(w), _ptr(bias), self._vec_flag(bias, "gemm bias"), _ptr(out), out.stride(0),
            M, N, K, _ptr(gain), self._vec_flag(gain, "gemm norm gain"), float(norm_eps), _ptr(values), _ptr(work),
            need, _stream()))
        return out

    def swiglu(self, gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        self._elem(gate_up, "swiglu in"); self._elem(out, "swiglu out")
        T, F = out.shape
        if gate_up.shape != (T, 2 * F) or not gate_up.is_contiguous() or not out.is_contiguous():
            raise KernelError(f"swiglu: in {tuple(gate_up.shape)} out {tuple(out.shape)}")
        self._check(self.lib.axk_swiglu(_ptr(gate_up), _ptr(out), T, F, _stream()))
        return out

    def argmax(self, logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        self._i32(out, "argmax out")
        if logits.dtype != torch.float32 or not logits.is_cuda or logits.stride(1) != 1 or out.numel() != logits.shape[0]:
            raise KernelError(f"argmax: logits {tuple(logits.shape)} {logits.dtype}, picks {out.numel()}")
        rows, n = logits.shape
        work = torch.empty(max(1, self.lib.axk_argmax_workspace(rows, n) // 8), dtype=torch.int64, device=logits.device)
        self._check(self.lib.axk_argmax(_ptr(logits), logits.stride(0), _ptr(out), rows, n, _ptr(work), _stream()))
        return out

    def topk(self, logits, recent, n_recent, penalty, k_of_row, cands, k_max: Optional[int] = None) -> torch.Tensor:
        """`k_max`: the largest of k_of_row, where the caller knows it (else it is read back from
        the device, which waits for it)."""
        self._i32(recent, "topk recent"); self._i32(n_recent, "topk n_recent"); self._i32(k_of_row, "topk k")
        self._f32(penalty, "topk penalty")
        rows, n = logits.shape
        if (logits.dtype != torch.float32 or not logits.is_cuda or logits.stride(1) != 1 or cands.dtype != torch.int64
                or cands.shape[0] != rows or not cands.is_contiguous() or recent.shape[0] != rows):
            raise KernelError(f"topk: logits {tuple(logits.shape)} cands {tuple(cands.shape)} {cands.dtype}")
        if k_max is None:
            k_max = int(k_of_row.max())
        if k_max > cands.shape[1]:
            raise KernelError(f"topk: k up to {k_max} for {cands.shape[1]} candidate places")
        need = self.lib.axk_topk_workspace(rows, n, cands.shape[1])
        work = torch.empty(max(need, 8) // 8, dtype=torch.int64, device=logits.device)
        self._check(self.lib.axk_topk(_ptr(logits), logits.stride(0), _ptr(recent), recent.shape[1], _ptr(n_recent),
                                      _ptr(penalty), _ptr(k_of_row), _ptr(cands), cands.shape[1], rows, n, _ptr(work),
                                      _stream()))
        return cands

    def fill_i32(self, dst: torch.Tensor, value: int) -> None:
        self._i32(dst, "fill")
        self._check(self.lib.axk_fill_i32(_ptr(dst), int(value), dst.numel(), _stream()))

    def fill_f32(self, dst: torch.Tensor, value: float) -> None:
        self._f32(dst, "fill")
        self._check(self.lib.axk_fill_f32(_ptr(dst), float(value), dst.numel(), _stream()))


_LOADED: Dict[str, Kernels] = {}


def kernels(dtype_name: str) -> Kernels:
    """The kernel library for "bfloat16" or "float32" (loaded once per process)."""
    if dtype_name not in _LOADED:
        _LOADED[dtype_name] = Kernels(dtype_name)
    return _LOADED[dtype_name]
