"""The kernel library as Python calls: tensors in, launches on the current HIP stream.

`kernels(dtype)` loads (compiling at first use) the library of one compute dtype and wraps
each C entry point.  Wrappers check what the C side cannot see (dtypes, devices, contiguity)
and raise `KernelError` with the library's own message when a call is refused.  There is no
other implementation behind these calls: without the library they fail.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_long, c_void_p
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
    "axk_embed_scaled": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_void_p],
    "axk_norm_add": [c_void_p, c_void_p, c_int, c_float, c_float, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "axk_round_rows": [c_void_p, c_void_p, c_long, c_void_p],
    "axk_activation": [c_void_p, c_long, c_int, c_void_p],
    "axk_clamped_glu": [c_void_p, c_void_p, c_int, c_int, c_float, c_float, c_void_p],
    "axk_grouped_gemm_uses_mfma": [c_int, c_int, c_long, c_long],
    "axk_grouped_gemm": [c_void_p, c_int, c_long, c_long, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_long, c_long,
                         c_void_p, c_void_p, c_long, c_int, c_void_p, c_int, c_float, c_float, c_float, c_void_p, c_void_p, c_int, c_int,
                         c_int, c_int, c_int, c_int, c_void_p],
    "axk_route_topk": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p],
    "axk_route_scored": [c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_void_p, c_void_p],
    "axk_route_max_tiles": [c_int, c_int, c_int],
    "axk_route_sort": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    "axk_route_combine": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_long, c_void_p],
    "axk_gather_rows": [c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "axk_causal_conv": [c_void_p, c_long, c_void_p, c_void_p, c_int, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_int,
                        c_int, c_void_p],
    "axk_gated_scan": [c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_long, c_void_p, c_int, c_float, c_void_p, c_long,
                       c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p],
    "axk_state_conv": [c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_void_p, c_long, c_long, c_long, c_void_p, c_void_p,
                       c_void_p, c_int, c_int, c_int, c_void_p, c_long, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p],
    "axk_state_space_scan": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_long, c_long, c_long, c_void_p, c_int, c_void_p,
                             c_void_p, c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int, c_void_p,
                             c_void_p, c_void_p, c_void_p],
    "axk_gated_group_norm": [c_void_p, c_void_p, c_long, c_void_p, c_int, c_float, c_void_p, c_int, c_int, c_int, c_void_p],
    "axk_latent_prepare": [c_void_p, c_long, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p, c_int, c_void_p, c_int,
                           c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    "axk_latent_query_rope": [c_void_p, c_long, c_int, c_int, c_int, c_int, c_float, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "axk_latent_attention": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                             c_int, c_int, c_int, c_float, c_void_p, c_void_p, c_long, c_void_p],
    "axk_sum_norm": [c_void_p, c_float, c_void_p, c_int, c_float, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "axk_layernorm": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_void_p],
    "axk_softcap": [c_void_p, c_long, c_int, c_int, c_float, c_void_p],
    "axk_scale_rows": [c_void_p, c_long, c_int, c_int, c_float, c_void_p],
    "axk_add_scaled": [c_void_p, c_void_p, c_float, c_long, c_void_p],
    "axk_heads_prepare": [c_void_p, c_long, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_float,
                          c_int, c_int, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                          c_int, c_float, c_int, c_void_p],
    "axk_masked_attention_uses_mfma": [c_int, c_int, c_int, c_int, c_int, c_int],
    "axk_masked_attention": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_int, c_int,
                             c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_float, c_float, c_float,
                             c_void_p, c_int, c_void_p, c_long, c_float, c_int, c_int, c_void_p],
    "axk_concat_round": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p],
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
        self.lib.axk_latent_attention_workspace.argtypes = [c_int, c_int, c_int, c_int, c_int, c_int, c_int]
        self.lib.axk_latent_attention_workspace.restype = ctypes.c_long
        self.lib.axk_masked_attention_workspace.argtypes = [c_int] * 10
        self.lib.axk_masked_attention_workspace.restype = ctypes.c_long
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
                  "fill_i32", "fill_f32", "call", "norm_add", "round_rows", "activation", "clamped_glu", "grouped_gemm",
                  "route_topk", "route_sort", "route_combine", "gather_rows", "causal_conv", "gated_scan", "latent_prepare",
                  "latent_query_rope", "latent_attention", "heads_prepare", "masked_attention", "concat_round", "scale_rows",
                  "add_scaled", "state_conv", "state_space_scan", "gated_group_norm", "route_scored", "sum_norm", "layernorm",
                  "softcap")
    _MATRIX_AT = {"gemm": 1, "gemm_qkv_rope": 1, "gemm_normed_glu": 3, "gemm_normed_qkv_rope": 3, "grouped_gemm": 1}   # which argument is W

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
                    label = f"{_name} {'x'.join(str(n) for n in w.shape)}"
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
    def _f32_rows(t: torch.Tensor, what: str) -> None:
        """float32 rows that may lie apart (a view into the columns of a wider product's rows)."""
        if t.dtype != torch.float32 or not t.is_cuda or t.dim() != 2 or t.stride(1) != 1:
            raise KernelError(f"{what}: expected float32 rows on the device, got {t.dtype} {tuple(t.shape)} with strides {t.stride()}")

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
    def embed(self, tokens: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        packed = isinstance(table, PackedMatrix)
        self._i32(tokens, "embed tokens"); self._elem(table.data if packed else table, "embed table")
        self._f32(out, "embed out")
        vocab, dim = table.shape
        if out.shape != (tokens.numel(), dim) or not (packed or table.is_contiguous()):
            raise KernelError(f"embed: out {tuple(out.shape)} does not fit {tokens.numel()} tokens of width {dim}")
        self._check(self.lib.axk_embed_scaled(_ptr(tokens), _ptr(table), 1 if packed else 0, _ptr(out), tokens.numel(), dim,
                                              vocab, float(scale), _stream()))
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

    # ------------------------------------------------------------------ a norm on a sublayer's output, roundings, activations
    def norm_add(self, y: torch.Tensor, gain: torch.Tensor, eps: float, mult: float, x: torch.Tensor,
                 rounded: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x += mult * rmsnorm(y, gain, eps), row by row; `rounded` also gets the new x in the compute dtype."""
        self._f32(y, "norm_add y"); self._f32(x, "norm_add x")
        if y.shape != x.shape or y.dim() != 2 or gain.numel() != x.shape[1]:
            raise KernelError(f"norm_add: y {tuple(y.shape)}, x {tuple(x.shape)}, a gain of {gain.numel()}")
        if rounded is not None:
            self._elem(rounded, "norm_add rounded")
            if rounded.shape != x.shape or not rounded.is_contiguous():
                raise KernelError(f"norm_add: rounded {tuple(rounded.shape)} is not {tuple(x.shape)} contiguous")
        self._check(self.lib.axk_norm_add(_ptr(y), _ptr(gain), self._vec_flag(gain, "norm_add gain"), float(eps), float(mult),
                                          _ptr(x), _ptr(rounded), x.shape[0], x.shape[1], _stream()))
        return x

    NORM_KINDS = {"rms": 0, "layer": 1}

    def sum_norm(self, y: torch.Tensor, alpha: float, gain: torch.Tensor, eps: float, kind: str, x: torch.Tensor,
                 rounded: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x = norm(alpha x + y) * gain, row by row (kind "rms" or "layer"); `rounded` also gets the new x in
        the compute dtype."""
        self._f32(y, "sum_norm y"); self._f32(x, "sum_norm x")
        if y.shape != x.shape or y.dim() != 2 or gain.numel() != x.shape[1] or kind not in self.NORM_KINDS:
            raise KernelError(f"sum_norm: y {tuple(y.shape)}, x {tuple(x.shape)}, a gain of {gain.numel()}, kind '{kind}'")
        if rounded is not None:
            self._elem(rounded, "sum_norm rounded")
            if rounded.shape != x.shape or not rounded.is_contiguous():
                raise KernelError(f"sum_norm: rounded {tuple(rounded.shape)} is not {tuple(x.shape)} contiguous")
        self._check(self.lib.axk_sum_norm(_ptr(y), float(alpha), _ptr(gain), self._vec_flag(gain, "sum_norm gain"), float(eps),
                                          self.NORM_KINDS[kind], _ptr(x), _ptr(rounded), x.shape[0], x.shape[1], _stream()))
        return x

    def layernorm(self, x: torch.Tensor, gain: torch.Tensor, eps: float, out: torch.Tensor,
                  rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """out = (x - mean) / sqrt(var + eps) * gain of float32 rows (`rows`: which of them)."""
        self._f32(x, "layernorm x"); self._elem(out, "layernorm out")
        n = x.shape[0]
        if rows is not None:
            self._i32(rows, "layernorm rows")
            n = rows.numel()
        if x.dim() != 2 or out.shape != (n, x.shape[1]) or not out.is_contiguous() or gain.numel() != x.shape[1]:
            raise KernelError(f"layernorm: x {tuple(x.shape)}, out {tuple(out.shape)}, a gain of {gain.numel()}")
        self._check(self.lib.axk_layernorm(_ptr(x), _ptr(rows), _ptr(gain), self._vec_flag(gain, "layernorm gain"), _ptr(out), n,
                                           x.shape[1], float(eps), _stream()))
        return out

    def softcap(self, v: torch.Tensor, cap: float) -> torch.Tensor:
        """v = cap tanh(v / cap) in place on float32 rows."""
        if v.dtype != torch.float32 or not v.is_cuda or v.dim() != 2 or v.stride(1) != 1:
            raise KernelError(f"softcap: {tuple(v.shape)} {v.dtype} with strides {v.stride()}")
        self._check(self.lib.axk_softcap(_ptr(v), v.stride(0), v.shape[0], v.shape[1], float(cap), _stream()))
        return v

    def scale_rows(self, v: torch.Tensor, factor: float) -> torch.Tensor:
        """v *= factor in place on float32 rows."""
        if v.dtype != torch.float32 or not v.is_cuda or v.dim() != 2 or v.stride(1) != 1:
            raise KernelError(f"scale_rows: {tuple(v.shape)} {v.dtype} with strides {v.stride()}")
        self._check(self.lib.axk_scale_rows(_ptr(v), v.stride(0), v.shape[0], v.shape[1], float(factor), _stream()))
        return v

    def add_scaled(self, x: torch.Tensor, y: torch.Tensor, factor: float = 1.0) -> torch.Tensor:
        """x += factor * y on float32 tensors of one shape."""
        self._f32(x, "add_scaled x"); self._f32(y, "add_scaled y")
        if x.shape != y.shape or not x.is_contiguous() or not y.is_contiguous():
            raise KernelError(f"add_scaled: {tuple(x.shape)} and {tuple(y.shape)}")
        self._check(self.lib.axk_add_scaled(_ptr(x), _ptr(y), float(factor), x.numel(), _stream()))
        return x

    def round_rows(self, x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        self._f32(x, "round_rows x"); self._elem(out, "round_rows out")
        if out.numel() != x.numel() or not out.is_contiguous():
            raise KernelError(f"round_rows: {tuple(x.shape)} into {tuple(out.shape)}")
        self._check(self.lib.axk_round_rows(_ptr(x), _ptr(out), x.numel(), _stream()))
        return out

    ACTIVATIONS = {"gelu_tanh": 0, "gelu_erf": 1}

    def activation(self, v: torch.Tensor, kind: str = "gelu_tanh") -> torch.Tensor:
        self._elem(v, "activation")
        if kind not in self.ACTIVATIONS or not v.is_contiguous():
            raise KernelError(f"activation: '{kind}' on a tensor of strides {v.stride()}")
        self._check(self.lib.axk_activation(_ptr(v), v.numel(), self.ACTIVATIONS[kind], _stream()))
        return v

    def concat_round(self, a: torch.Tensor, b: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """out = [a | b] row by row, rounded to the compute dtype."""
        self._f32(a, "concat_round a"); self._f32(b, "concat_round b"); self._elem(out, "concat_round out")
        if a.dim() != 2 or b.dim() != 2 or a.shape[0] != b.shape[0] or out.shape != (a.shape[0], a.shape[1] + b.shape[1]) \
                or not out.is_contiguous():
            raise KernelError(f"concat_round: {tuple(a.shape)} and {tuple(b.shape)} into {tuple(out.shape)}")
        self._check(self.lib.axk_concat_round(_ptr(a), a.shape[1], _ptr(b), b.shape[1], _ptr(out), a.shape[0], _stream()))
        return out

    def clamped_glu(self, gate_up: torch.Tensor, out: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
        self._elem(gate_up, "clamped_glu in"); self._elem(out, "clamped_glu out")
        T, F = out.shape
        if gate_up.shape != (T, 2 * F) or not gate_up.is_contiguous() or not out.is_contiguous():
            raise KernelError(f"clamped_glu: in {tuple(gate_up.shape)} out {tuple(out.shape)}")
        self._check(self.lib.axk_clamped_glu(_ptr(gate_up), _ptr(out), T, F, float(limit), float(alpha), _stream()))
        return out

    # ------------------------------------------------------------------ grouped products
    def grouped_gemm(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, *, x_group_stride: int, out_group_stride: int,
                     bias: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None, glu=None, routed=None,
                     rows: Optional[int] = None, gate_per_group: bool = False, row_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
        """out[orow(r), g ogs + n] = epilogue(sum_k x[xrow(r), g xgs + k] w[g, n, k] + bias[g, n]).

        x [rows, >= g xgs + K] float32 or compute dtype, rows may be strided; w [G, N, K] (with `glu`
        = (limit, alpha[, shift]): [G, 2 N, K], gate rows then up rows; out = g sigmoid(alpha g) (u + shift) with g
        and u clamped by limit, shift 1 unless given; (inf, 1, 0) is silu(gate) up) in the compute dtype; out float32 or
        compute dtype.  Block-diagonal: every row meets every group.  `routed` = (tiles, n_tiles,
        max_tiles, x_rows, out_rows[, tile_rows]), int32 on the device: the listed rows (`rows` of them at
        most) meet the group their tile names; tile_rows (16, or 64: many rows a group) is what the list
        was made for.  `gate` (float32, out's shape): out is multiplied
        by its sigmoid; with `gate_per_group` the gate holds one number a group, [rows, >= G].  `row_scale`
        (float32, one number an out row): the sums are multiplied by it before bias and epilogue, as if the
        row of x had been."""
        G, NW, K = w.shape
        N = NW // 2 if glu else NW
        self._elem(w, "grouped w")
        if not w.is_contiguous() or x.stride(-1) != 1 or out.stride(-1) != 1 or x.dim() != 2 or out.dim() != 2:
            raise KernelError("grouped_gemm: w must be contiguous, x and out row-major matrices")
        for t, what in ((x, "x"), (out, "out")):
            if t.dtype not in (torch.float32, self.dtype) or not t.is_cuda:
                raise KernelError(f"grouped_gemm: {what} is {t.dtype} on {t.device}")
        M = x.shape[0] if rows is None else int(rows)
        if x.shape[1] < (G - 1) * x_group_stride + K and routed is None or out.shape[1] < (G - 1) * out_group_stride + N and routed is None:
            raise KernelError(f"grouped_gemm: x {tuple(x.shape)} / out {tuple(out.shape)} do not hold {G} groups of {K} -> {N}")
        if routed is None and out.shape[0] != M:
            raise KernelError(f"grouped_gemm: {M} rows in, {out.shape[0]} out")
        if bias is not None and bias.numel() != G * NW:
            raise KernelError(f"grouped_gemm: a bias of {bias.numel()} for {G} x {NW}")
        if gate is not None:
            if gate.dtype != torch.float32 or not gate.is_cuda or gate.dim() != 2 or gate.shape[0] != out.shape[0] or gate.stride(-1) != 1 \
                    or (gate_per_group and gate.shape[1] < G):
                raise KernelError(f"grouped_gemm: gate {tuple(gate.shape)} for out {tuple(out.shape)} in {G} groups")
        tiles = n_tiles = x_rows = out_rows = None
        max_tiles, tile_rows = 0, 16
        if routed is not None:
            tiles, n_tiles, max_tiles, x_rows, out_rows = routed[:5]
            tile_rows = routed[5] if len(routed) > 5 else 16
            for t in (tiles, n_tiles, x_rows, out_rows):
                if t is not None:
                    self._i32(t, "grouped_gemm routing")
            if x.shape[1] < K or out.shape[1] < N:
                raise KernelError(f"grouped_gemm: x {tuple(x.shape)} / out {tuple(out.shape)} for {K} -> {N}")
        if row_scale is not None:
            self._f32(row_scale, "grouped_gemm row_scale")
            if not row_scale.is_contiguous() or row_scale.numel() < (M if routed is not None else out.shape[0]):
                raise KernelError(f"grouped_gemm: {row_scale.numel()} row factors for {M} rows")
        limit, alpha, shift = (tuple(glu) + (1.0,))[:3] if glu else (0.0, 0.0, 0.0)
        self._check(self.lib.axk_grouped_gemm(
            _ptr(x), 1 if x.dtype == torch.float32 else 0, x.stride(0), x_group_stride, _ptr(x_rows), _ptr(w), _ptr(bias),
            self._vec_flag(bias, "grouped bias"), _ptr(out), 1 if out.dtype == torch.float32 else 0, out.stride(0),
            out_group_stride, _ptr(out_rows), _ptr(gate), 0 if gate is None else gate.stride(0), 1 if gate_per_group else 0,
            _ptr(row_scale), 1 if glu else 0, float(limit), float(alpha), float(shift), _ptr(tiles), _ptr(n_tiles), int(max_tiles), int(tile_rows), M, N, K, G, _stream()))
        return out

    # ------------------------------------------------------------------ routing
    def route_topk(self, logits: torch.Tensor, top: int, experts: torch.Tensor, weights: torch.Tensor) -> None:
        self._f32(logits, "router logits"); self._i32(experts, "chosen experts"); self._f32(weights, "router weights")
        T, E = logits.shape
        if experts.shape != (T, top) or weights.shape != (T, top):
            raise KernelError(f"route_topk: {tuple(experts.shape)} / {tuple(weights.shape)} for {T} x {top}")
        self._check(self.lib.axk_route_topk(_ptr(logits), T, E, top, _ptr(experts), _ptr(weights), _stream()))

    def route_scored(self, logits: torch.Tensor, correction: Optional[torch.Tensor], top: int, groups: int, keep: int, scale: float,
                     experts: torch.Tensor, weights: torch.Tensor, normalize: bool = True, n_experts: Optional[int] = None) -> None:
        """Sigmoid scores, the choice by score + correction among the `keep` best of `groups` groups of
        neighbouring experts, weights the chosen scores over their sum (without `normalize`: the scores
        themselves), times scale (axk_route_scored).  `n_experts`: the leading columns of `logits` that
        are router logits (all, unless given)."""
        self._f32(logits, "router logits"); self._i32(experts, "chosen experts"); self._f32(weights, "router weights")
        T, E = logits.shape
        if n_experts is not None:
            if not 0 < n_experts <= E:
                raise KernelError(f"route_scored: {n_experts} experts in rows of {E} logits")
            E = int(n_experts)
        if experts.shape != (T, top) or weights.shape != (T, top) or logits.stride(1) != 1:
            raise KernelError(f"route_scored: {tuple(experts.shape)} / {tuple(weights.shape)} for {T} x {top}")
        if correction is not None:
            self._f32(correction, "router correction")
            if correction.numel() != E:
                raise KernelError(f"route_scored: a correction of {correction.numel()} for {E} experts")
        self._check(self.lib.axk_route_scored(_ptr(logits), logits.stride(0), _ptr(correction), T, E, top, int(groups), int(keep),
                                              float(scale), 1 if normalize else 0, _ptr(experts), _ptr(weights), _stream()))

    def route_max_tiles(self, n_pairs: int, n_experts: int, tile_rows: int = 16) -> int:
        return int(self.lib.axk_route_max_tiles(n_pairs, n_experts, tile_rows))

    def route_sort(self, experts: torch.Tensor, n_experts: int, sorted_pairs, sorted_tokens, tiles, n_tiles, place_of=None,
                   first_of=None, tile_rows: int = 16) -> None:
        """The pairs in expert order, their tokens, the grouped product's tiles; optionally where each
        pair stands (place_of [pairs]) and where each expert's pairs start (first_of [experts + 1])."""
        for t in (experts, sorted_pairs, sorted_tokens, tiles, n_tiles) + tuple(t for t in (place_of, first_of) if t is not None):
            self._i32(t, "route_sort")
        if (place_of is not None and place_of.numel() < experts.numel()) or (first_of is not None and first_of.numel() < n_experts + 1):
            raise KernelError("route_sort: place_of or first_of is too short")
        P = experts.numel()
        if sorted_pairs.numel() < P or sorted_tokens.numel() < P or tiles.numel() < 3 * self.route_max_tiles(P, n_experts, tile_rows):
            raise KernelError(f"route_sort: lists too short for {P} pairs of {n_experts} experts")
        self._check(self.lib.axk_route_sort(_ptr(experts), P, n_experts, experts.shape[-1], _ptr(sorted_pairs), _ptr(sorted_tokens),
                                            _ptr(tiles), _ptr(n_tiles), _ptr(place_of), _ptr(first_of), int(tile_rows), _stream()))

    def gather_rows(self, x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        self._elem(x, "gather x"); self._elem(out, "gather out"); self._i32(rows, "gather rows")
        if out.shape != (rows.numel(), x.shape[1]) or x.stride(1) != 1 or not out.is_contiguous():
            raise KernelError(f"gather_rows: {rows.numel()} rows of {tuple(x.shape)} into {tuple(out.shape)}")
        self._check(self.lib.axk_gather_rows(_ptr(x), x.stride(0), _ptr(rows), _ptr(out), rows.numel(), x.shape[1], _stream()))
        return out

    def route_combine(self, rows: torch.Tensor, weights: Optional[torch.Tensor], y: torch.Tensor, accumulate: bool = False,
                      place_of: Optional[torch.Tensor] = None, top: Optional[int] = None, extra: Optional[torch.Tensor] = None,
                      extra_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """y[t] (+)= sum_k weights[t, k] rows[t top + k] (weights None: all 1, `top` then says how many rows a
        token) + extra[t] sigmoid(extra_gate[t]) (extra: float32 like y; extra_gate: a float32 column, one logit a
        token, rows may be strided; None: no gate)."""
        self._f32(rows, "expert rows"); self._f32(y, "combine y")
        if place_of is not None:
            self._i32(place_of, "combine place_of")
        T = y.shape[0]
        if weights is not None:
            self._f32(weights, "router weights")
            if weights.shape[0] != T or not weights.is_contiguous():
                raise KernelError(f"route_combine: weights {tuple(weights.shape)} for {T} tokens")
            top = weights.shape[1]
        if top is None or rows.shape != (T * top, y.shape[1]) or not rows.is_contiguous() or not y.is_contiguous():
            raise KernelError(f"route_combine: rows {tuple(rows.shape)}, {top} a token, y {tuple(y.shape)}")
        gate_stride = 0
        if extra is not None:
            self._f32(extra, "combine extra")
            if extra.shape != y.shape or not extra.is_contiguous():
                raise KernelError(f"route_combine: extra {tuple(extra.shape)} beside y {tuple(y.shape)}")
            if extra_gate is not None:
                self._f32_rows(extra_gate, "combine extra gate")
                if extra_gate.shape != (T, 1):
                    raise KernelError(f"route_combine: a gate of {tuple(extra_gate.shape)} for {T} tokens")
                gate_stride = extra_gate.stride(0)
        elif extra_gate is not None:
            raise KernelError("route_combine: a gate without the rows it gates")
        self._check(self.lib.axk_route_combine(_ptr(rows), _ptr(weights), _ptr(y), T, top, y.shape[1], 1 if accumulate else 0,
                                               _ptr(place_of), _ptr(extra), _ptr(extra_gate), gate_stride, _stream()))
        return y

    # ------------------------------------------------------------------ convolution and recurrence with per-request state
    def causal_conv(self, x: torch.Tensor, w: torch.Tensor, bias, state: torch.Tensor, positions: torch.Tensor,
                    seq_rows: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
        """u[t, c] = bias[c] + sum_k w[c, k] x(t - (taps - 1 - k)); x [T, C] in the compute dtype (rows may
        be strided), inputs before the step from the float32 state rows [slots, >= 2 taps C] (two copies,
        the one behind position p at p & 1: see csrc/recurrent.hip)."""
        self._elem(x, "conv x"); self._elem(w, "conv w"); self._f32(state, "conv state"); self._f32(u, "conv u")
        self._i32(seq_rows, "seq_rows"); self._i32(positions, "positions")
        T, C = u.shape
        if x.shape != (T, C) or x.stride(1) != 1 or w.dim() != 2 or w.shape[0] != C or not w.is_contiguous() or seq_rows.numel() != T:
            raise KernelError(f"causal_conv: x {tuple(x.shape)}, w {tuple(w.shape)}, u {tuple(u.shape)}")
        if bias is not None and bias.numel() != C:
            raise KernelError(f"causal_conv: a bias of {bias.numel()} for {C} channels")
        self._check(self.lib.axk_causal_conv(_ptr(x), x.stride(0), _ptr(w), _ptr(bias), self._vec_flag(bias, "conv bias"),
                                             _ptr(state), state.stride(0), _ptr(positions), _ptr(seq_rows), _ptr(u), T, C,
                                             w.shape[1], _stream()))
        return u

    def gated_scan(self, gates, u, y, x, lam, decay: float, state, spans, positions, seq_rows, out, block_width: int, taps: int):
        """The gated linear recurrence over each request's tokens (see csrc/recurrent.hip): gates
        [T, C / block_width, 2 block_width] and u [T, C] float32; y, x [T, C] compute dtype (rows may be
        strided); state float32 [slots, >= 2 taps C]; spans int32 [n, 3] = (slot, first token, tokens) or
        None (each token a request of its own in slot seq_rows[t]); out [T, C] compute dtype."""
        self._f32(gates, "scan gates"); self._f32(u, "scan u"); self._elem(y, "scan y"); self._elem(x, "scan x")
        self._f32(state, "scan state"); self._elem(out, "scan out"); self._i32(seq_rows, "seq_rows"); self._i32(positions, "positions")
        T, C = u.shape
        if (gates.shape != (T, 2 * C) and gates.numel() != T * 2 * C) or y.shape != (T, C) or x.shape != (T, C) or out.shape != (T, C) \
                or y.stride(1) != 1 or x.stride(1) != 1 or not out.is_contiguous() or lam.numel() != C or seq_rows.numel() != T:
            raise KernelError(f"gated_scan: gates {tuple(gates.shape)}, u {tuple(u.shape)}, y {tuple(y.shape)}, out {tuple(out.shape)}")
        terms = None
        if spans is not None:
            self._i32(spans, "scan spans")
            n = spans.shape[0]
            if T > 4 * n:            # stretches of tokens: the state-free terms for all tokens at once, then a lean walk
                terms = torch.empty((T, 3, C), dtype=torch.float32, device=u.device)
        else:
            n = T
        self._check(self.lib.axk_gated_scan(_ptr(gates), _ptr(u), _ptr(y), y.stride(0), _ptr(x), x.stride(0), _ptr(lam),
                                            self._vec_flag(lam, "scan lam"), float(decay), _ptr(state), state.stride(0),
                                            _ptr(spans), n, _ptr(positions), _ptr(seq_rows), _ptr(out), C, int(block_width),
                                            int(taps), _ptr(terms), T, _stream()))
        return out

    # ------------------------------------------------------------------ a state-space mixer with per-request state
    def state_conv(self, x, w, bias, state, copy_elems: int, tail_at: int, positions, seq_rows, u, silu: bool = True,
                   raw=None, dt_bias=None, a_log=None, terms=None) -> torch.Tensor:
        """u[t, c] = act(bias[c] + sum_k w[c, k] x(t - (taps - 1 - k))) over float32 rows x [T, C] (a view whose
        rows may be strided), inputs before the step from the float32 state rows (two copies of `copy_elems`
        floats, the kept inputs from `tail_at`: see csrc/state_space.hip).  With `raw` [T, heads] (float32, a
        view), `dt_bias`, `a_log` and `terms` [T, heads, 2]: the heads' (dt, a) as well."""
        self._f32_rows(x, "conv x"); self._elem(w, "conv w"); self._f32(state, "conv state"); self._f32(u, "conv u")
        self._i32(seq_rows, "seq_rows"); self._i32(positions, "positions")
        T, C = u.shape
        if x.shape != (T, C) or w.dim() != 2 or w.shape[0] != C or not w.is_contiguous() or seq_rows.numel() != T:
            raise KernelError(f"state_conv: x {tuple(x.shape)}, w {tuple(w.shape)}, u {tuple(u.shape)}")
        if bias is not None and bias.numel() != C:
            raise KernelError(f"state_conv: a bias of {bias.numel()} for {C} channels")
        heads = 0
        if raw is not None:
            self._f32_rows(raw, "conv raw"); self._f32(terms, "conv terms")
            heads = raw.shape[1]
            if raw.shape[0] != T or raw.stride(1) != 1 or terms.shape != (T, heads, 2) or not terms.is_contiguous() \
                    or dt_bias.numel() != heads or a_log.numel() != heads:
                raise KernelError(f"state_conv: raw {tuple(raw.shape)}, terms {tuple(terms.shape)} for {heads} heads")
        self._check(self.lib.axk_state_conv(
            _ptr(x), x.stride(0), _ptr(w), _ptr(bias), self._vec_flag(bias, "conv bias"), 1 if silu else 0, _ptr(state),
            state.stride(0), int(copy_elems), int(tail_at), _ptr(positions), _ptr(seq_rows), _ptr(u), T, C, w.shape[1],
            _ptr(raw), 0 if raw is None else raw.stride(0), _ptr(dt_bias), self._vec_flag(dt_bias, "dt bias"), _ptr(a_log),
            self._vec_flag(a_log, "A_log"), _ptr(terms), heads, _stream()))
        return u

    def state_space_scan(self, u, terms, d_skip, state, copy_elems: int, tail_at: int, spans, positions, seq_rows, conv_in, y,
                         heads: int, groups: int, vdim: int, n_state: int, taps: int, segments=None) -> torch.Tensor:
        """The state-space recurrence over each request's tokens (see csrc/state_space.hip): u [T, heads vdim +
        2 groups n_state] and terms [T, heads, 2] float32; spans int32 [n, 3] = (slot, first token, tokens) or None
        (each token a request of its own in slot seq_rows[t]); conv_in: the convolution's inputs (float32, rows may
        be strided), kept for the next step; y [T, heads vdim] float32.  `segments` = (segs int32 [n, 4]: slot,
        first token, tokens, whether the request's first; spans5 int32 [requests, 5]: slot, first token, tokens,
        first segment, segments; the longest segment's tokens): long stretches run in segments side by side and are folded (sums in another
        order, by rounding)."""
        for t, what in ((u, "scan u"), (terms, "scan terms"), (state, "scan state"), (y, "scan y")):
            self._f32(t, what)
        self._f32_rows(conv_in, "scan conv_in")
        self._i32(seq_rows, "seq_rows"); self._i32(positions, "positions")
        T, C = u.shape
        if C != heads * vdim + 2 * groups * n_state or not u.is_contiguous() or terms.shape != (T, heads, 2) \
                or not terms.is_contiguous() or y.shape != (T, heads * vdim) or not y.is_contiguous() \
                or conv_in.shape != (T, C) or conv_in.stride(1) != 1 or d_skip.numel() != heads or seq_rows.numel() != T:
            raise KernelError(f"state_space_scan: u {tuple(u.shape)}, terms {tuple(terms.shape)}, y {tuple(y.shape)}")
        if spans is not None:
            self._i32(spans, "scan spans")
            n = spans.shape[0]
        else:
            n = T
        segs = spans5 = ends = cum = None
        n_segs = longest = 0
        if segments is not None:
            segs, spans5, longest = segments
            self._i32(segs, "scan segments"); self._i32(spans5, "scan requests")
            n_segs = segs.shape[0]
            if spans is None or segs.dim() != 2 or segs.shape[1] != 4 or spans5.shape != (n, 5):
                raise KernelError(f"state_space_scan: segments {tuple(segs.shape)} of requests {tuple(spans5.shape)} for {n} requests")
            ends = torch.empty((n_segs, heads, n_state, vdim), dtype=torch.float32, device=u.device)
            cum = torch.empty((T, heads), dtype=torch.float32, device=u.device)
        self._check(self.lib.axk_state_space_scan(
            _ptr(u), _ptr(terms), _ptr(d_skip), self._vec_flag(d_skip, "D"), _ptr(state), state.stride(0), int(copy_elems),
            int(tail_at), _ptr(spans), n, _ptr(positions), _ptr(seq_rows), _ptr(conv_in), conv_in.stride(0), _ptr(y), heads,
            groups, vdim, n_state, taps, _ptr(segs), n_segs, int(longest), _ptr(spans5), _ptr(ends), _ptr(cum), _stream()))
        return y

    def gated_group_norm(self, y, z, gain, eps: float, out, parts: int) -> torch.Tensor:
        """out = rms in `parts` equal parts of (y silu(z)), times gain: y float32 [T, W], z float32 [T, W] (rows
        may be strided), out [T, W] in the compute dtype."""
        self._f32(y, "group norm y"); self._f32_rows(z, "group norm z"); self._elem(out, "group norm out")
        T, W = y.shape
        if z.shape != (T, W) or z.stride(1) != 1 or out.shape != (T, W) or not y.is_contiguous() or not out.is_contiguous() \
                or gain.numel() != W or parts < 1 or W % parts:
            raise KernelError(f"gated_group_norm: y {tuple(y.shape)}, z {tuple(z.shape)}, out {tuple(out.shape)}, {parts} parts")
        self._check(self.lib.axk_gated_group_norm(_ptr(y), _ptr(z), z.stride(0), _ptr(gain), self._vec_flag(gain, "group norm gain"),
                                                  float(eps), _ptr(out), T, W, int(parts), _stream()))
        return out

    # ------------------------------------------------------------------ attention over a latent cache
    def latent_prepare(self, fused, q_at, q_rank, kv_at, rank, rot, rot_dims, q_gain, kv_gain, eps, table, positions, seq_rows,
                       block_table, cache, page_size, cq, write_kv=True, neighbours=False, magnitude=1.0) -> None:
        self._f32(fused, "latent fused"); self._f32(table, "rope table"); self._i32(positions, "positions")
        self._i32(seq_rows, "seq_rows"); self._i32(block_table, "block_table"); self._elem(cache, "latent cache")
        T = positions.numel()
        if fused.shape[0] != T or (rot_dims and table.shape != (T, rot_dims // 2, 2)) or seq_rows.numel() != T:
            raise KernelError(f"latent_prepare: fused {tuple(fused.shape)}, table {tuple(table.shape)} for {T} tokens")
        if cache.dim() != 4 or tuple(cache.shape[1:]) != (1, page_size, 2 * rank + rot) or not cache.is_contiguous():
            raise KernelError(f"latent_prepare: cache {tuple(cache.shape)} is not [pages, 1, {page_size}, {2 * rank + rot}]")
        if q_rank:
            self._elem(cq, "latent cq")
            if cq.shape != (T, q_rank) or not cq.is_contiguous() or q_gain.numel() != q_rank:
                raise KernelError(f"latent_prepare: cq {tuple(cq.shape)} for a query latent of {q_rank}")
        if kv_gain.numel() != rank:
            raise KernelError(f"latent_prepare: a gain of {kv_gain.numel()} for a latent of {rank}")
        self._check(self.lib.axk_latent_prepare(
            _ptr(fused), fused.stride(0), q_at, q_rank, kv_at, rank, rot, rot_dims, 1 if neighbours else 0, float(magnitude),
            _ptr(q_gain if q_rank else None), self._vec_flag(q_gain if q_rank else None, "q gain"),
            _ptr(kv_gain), self._vec_flag(kv_gain, "kv gain"), float(eps), _ptr(table), _ptr(positions), _ptr(seq_rows),
            _ptr(block_table), block_table.shape[-1], _ptr(cache), page_size, _ptr(cq if q_rank else None), T,
            1 if write_kv else 0, _stream()))

    def latent_query_rope(self, q, dim, rot, rot_dims, table, q_full, rank, heads, neighbours=False, magnitude=1.0) -> None:
        """q: float32 [T, >= heads (dim + rot)], rows may be strided (a view into a wider product's rows)."""
        self._f32(q_full, "latent q_full"); self._f32(table, "rope table")
        T = q.shape[0]
        if q.dtype != torch.float32 or not q.is_cuda or q.dim() != 2 or q.shape[1] < heads * (dim + rot) or q.stride(1) != 1 or q_full.shape != (T, heads * (rank + rot)) \
                or not q_full.is_contiguous():
            raise KernelError(f"latent_query_rope: q {tuple(q.shape)}, q_full {tuple(q_full.shape)}")
        self._check(self.lib.axk_latent_query_rope(_ptr(q), q.stride(0), dim, rot, rot_dims, 1 if neighbours else 0, float(magnitude),
                                                   _ptr(table), _ptr(q_full), rank, heads, T, _stream()))

    def latent_attention(self, q_full, cache, block_table, positions, seq_rows, o_lat, heads, rank, rot, page_size, window,
                         scale, sink=None, span: int = 0) -> torch.Tensor:
        """`sink`: float32 [heads], a number a head whose exponential the softmax's denominator also holds;
        `span`: the most positions a row of this step sees, where the caller knows it (attention without a
        window then lets the blocks of a token's positions run side by side in steps of few tokens)."""
        self._f32(q_full, "latent q_full"); self._f32(o_lat, "latent o_lat"); self._elem(cache, "latent cache")
        self._i32(positions, "positions"); self._i32(seq_rows, "seq_rows"); self._i32(block_table, "block_table")
        T = positions.numel()
        if q_full.shape != (T, heads * (rank + rot)) or o_lat.shape != (T, heads * rank) or seq_rows.numel() != T:
            raise KernelError(f"latent_attention: q_full {tuple(q_full.shape)}, o_lat {tuple(o_lat.shape)} for {T} tokens")
        if cache.dim() != 4 or tuple(cache.shape[1:]) != (1, page_size, 2 * rank + rot) or not cache.is_contiguous():
            raise KernelError(f"latent_attention: cache {tuple(cache.shape)} is not [pages, 1, {page_size}, {2 * rank + rot}]")
        if sink is not None:
            self._f32(sink, "latent sink")
            if sink.numel() != heads:
                raise KernelError(f"latent_attention: {sink.numel()} sinks for {heads} heads")
        need = int(self.lib.axk_latent_attention_workspace(T, heads, rank, rot, page_size, int(window), int(span)))
        partial = torch.empty(need, dtype=torch.float32, device=o_lat.device) if need else None
        self._check(self.lib.axk_latent_attention(_ptr(q_full), _ptr(cache), _ptr(block_table), block_table.shape[-1],
                                                  _ptr(positions), _ptr(seq_rows), _ptr(o_lat), T, heads, rank, rot, page_size,
                                                  int(window), int(span), float(scale), _ptr(sink), _ptr(partial), need, _stream()))
        return o_lat

    # ------------------------------------------------------------------ attention with maps, masks and bent scores
    MASKS = {"causal": 0, "window": 1, "chunk": 2}

    def _check_heads_cache(self, cache, page_size, row, what) -> None:
        self._elem(cache, what + " cache")
        if cache.dim() != 4 or tuple(cache.shape[1:]) != (1, page_size, row) or not cache.is_contiguous():
            raise KernelError(f"{what}: cache {tuple(cache.shape)} is not [pages, 1, {page_size}, {row}]")

    def heads_prepare(self, proj, q_at, n_q, k_at, n_k, v_at, v_width, dim, q_gain, k_gain, eps, rot, neighbours, magnitude,
                      table, positions, seq_rows, block_table, cache, page_size, q_out, write_kv=True, q_temp=None) -> None:
        """The projections' float32 rows into queries (q_out) and the page's keys and values: see
        axk_heads_prepare in csrc/api.h.  `q_temp` = (coef, every): a query's temperature by its position."""
        self._f32(proj, "heads proj"); self._f32(table, "rope table"); self._i32(positions, "positions")
        self._i32(seq_rows, "seq_rows"); self._i32(block_table, "block_table"); self._elem(q_out, "heads q_out")
        T = positions.numel()
        if proj.dim() != 2 or proj.shape[0] != T or (rot and table.shape != (T, rot // 2, 2)) or seq_rows.numel() != T:
            raise KernelError(f"heads_prepare: proj {tuple(proj.shape)}, table {tuple(table.shape)} for {T} tokens")
        self._check_heads_cache(cache, page_size, n_k * dim + v_width, "heads_prepare")
        if q_out.shape != (T, n_q * dim) or not q_out.is_contiguous():
            raise KernelError(f"heads_prepare: q_out {tuple(q_out.shape)} is not [{T}, {n_q * dim}]")
        for gain in (q_gain, k_gain):
            if gain is not None and gain.numel() != dim:
                raise KernelError(f"heads_prepare: a gain of {gain.numel()} for units of {dim}")
        self._check(self.lib.axk_heads_prepare(
            _ptr(proj), proj.stride(0), q_at, n_q, k_at, n_k, v_at, v_width, dim, _ptr(q_gain), self._vec_flag(q_gain, "q gain"),
            _ptr(k_gain), self._vec_flag(k_gain, "k gain"), float(eps), rot, 1 if neighbours else 0, float(magnitude), _ptr(table),
            _ptr(positions), _ptr(seq_rows), _ptr(block_table), block_table.shape[-1], _ptr(cache), page_size, _ptr(q_out), T,
            1 if write_kv else 0, float(q_temp[0]) if q_temp else 0.0, int(q_temp[1]) if q_temp else 0, _stream()))

    def masked_attention_uses_mfma(self, heads, kv_heads, maps, dim, vdim, page_size) -> bool:
        return bool(self.lib.axk_masked_attention_uses_mfma(heads, kv_heads, maps, dim, vdim, page_size))

    def masked_attention(self, q, cache, block_table, positions, seq_rows, out, heads, kv_heads, maps, dim, vdim, page_size,
                         mask, mask_size, scale, softcap=0.0, lam=0.0, out_scale=1.0, eps=0.0, gate=None, tiles=None,
                         sink=None, gate_per_head=False, span=0) -> torch.Tensor:
        """q [T, heads maps dim] -> out [T, heads vdim] (compute dtype): see axk_masked_attention in csrc/api.h.
        `gate`: float32 rows (a view whose rows may be strided) of heads vdim gate logits (of heads logits with
        `gate_per_head`), or None.  `sink`: the score of a key without a value in every softmax, or None.  `span`
        (causal masks): the positions the step's longest row sees, so that a step of few tokens can run a token's
        blocks of positions side by side; 0: a wave walks them."""
        self._elem(q, "attention q"); self._elem(out, "attention out")
        self._i32(positions, "positions"); self._i32(seq_rows, "seq_rows"); self._i32(block_table, "block_table")
        T = positions.numel()
        if q.shape != (T, heads * maps * dim) or out.shape != (T, heads * vdim) or seq_rows.numel() != T \
                or not q.is_contiguous() or not out.is_contiguous():
            raise KernelError(f"masked_attention: q {tuple(q.shape)}, out {tuple(out.shape)} for {T} tokens")
        self._check_heads_cache(cache, page_size, kv_heads * (maps * dim + vdim), "masked_attention")
        if mask not in self.MASKS:
            raise KernelError(f"masked_attention: mask '{mask}' is not known ({', '.join(self.MASKS)})")
        gate_stride = 0
        if gate is not None:
            gw = heads if gate_per_head else heads * vdim
            if gate.dtype != torch.float32 or gate.shape != (T, gw) or gate.stride(1) != 1:
                raise KernelError(f"masked_attention: gate {tuple(gate.shape)} {gate.dtype} is not float32 [{T}, {gw}]")
            gate_stride = gate.stride(0)
        n_tiles = 0
        if tiles is not None:
            self._i32(tiles, "attention tiles")
            n_tiles = tiles.shape[0]
        need = int(self.lib.axk_masked_attention_workspace(T, heads, kv_heads, maps, dim, vdim, page_size, self.MASKS[mask],
                                                           int(mask_size), int(span)))
        partial = torch.empty(need, dtype=torch.float32, device=out.device) if need else None
        self._check(self.lib.axk_masked_attention(
            _ptr(q), _ptr(cache), _ptr(block_table), block_table.shape[-1], _ptr(positions), _ptr(seq_rows), _ptr(gate),
            gate_stride, _ptr(out), T, heads, kv_heads, maps, dim, vdim, page_size, self.MASKS[mask], int(mask_size), float(scale),
            float(softcap), float(lam), float(out_scale), float(eps), _ptr(tiles), n_tiles, _ptr(partial), need,
            float("-inf") if sink is None else float(sink), 1 if gate_per_head else 0, int(span), _stream()))
        return out

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
