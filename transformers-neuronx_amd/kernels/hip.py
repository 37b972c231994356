"""The product kernel backend: hand-written HIP for gfx950 behind a C interface.

Each call checks shapes and dtypes on the host, launches on torch's current
stream and raises with the library's message if the library refuses. torch is
the allocator and nothing else here. A missing library is compiled at first use;
if that fails the call fails: there is no other path.
"""
import ctypes
from typing import Dict, Optional

import numpy as np
import torch

from . import build
from .attention_plan import QUERY_TILE
from .. import debug

_F32, _BF16 = 0, 1
_ACT = {None: 0, "none": 0, "relu": 1, "gelu": 2, "gelu_new": 3, "relu2": 5}
_GATE_ACT = {"gelu_new": 3, "silu": 4, "clamped_swiglu": 6}     # what a gated expert's kernels take
_LIBS: Dict[str, ctypes.CDLL] = {}

_c_void_p, _c_int, _c_float, _c_ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_longlong

_SIGNATURES = {
    "elementwise": {
        "tnx_gather_rows": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_int, _c_void_p],
        "tnx_copy_ints": [_c_void_p, _c_void_p, _c_int, _c_void_p],
        "tnx_device_pointer": [_c_void_p, _c_void_p],
        "tnx_add_positions": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p,
                              _c_int, _c_int, _c_int, _c_float, _c_void_p],
        "tnx_cast": [_c_void_p, _c_int, _c_void_p, _c_int, _c_ll, _c_void_p],
        "tnx_epilogue": [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_layernorm": [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                          _c_int, _c_void_p],
    },
    "gemm": {
        "tnx_gemm_f32": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                         _c_int, _c_void_p],
        "tnx_gemm_bf16": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                          _c_int, _c_int, _c_int, _c_void_p],
        "tnx_gemm_bf16_qkv": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p,
                              _c_void_p, _c_void_p, _c_void_p, _c_float, _c_int, _c_int, _c_int, _c_int, _c_int,
                              _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
        "tnx_gemm_skinny_tiles_per_block": [_c_int, _c_int],
        "tnx_gemm_bf16_mid": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                              _c_int, _c_void_p, ctypes.c_size_t, _c_int, _c_int, _c_void_p],
        "tnx_gemm_library": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                             _c_int, _c_void_p, ctypes.c_size_t, _c_void_p, ctypes.c_size_t, _c_int, _c_void_p],
        "tnx_gemm_bf16_normed": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_void_p, _c_int,
                                 _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_gemm_bf16_qkv_normed": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_int,
                                     _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_int, _c_int,
                                     _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                                     _c_int, _c_void_p],
    },
    "attention": {
        "tnx_qkv_write": [_c_void_p, _c_int, _c_void_p, _c_float, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                          _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p,
                          _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_int,
                          _c_void_p],
        "tnx_attention_any": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                              _c_int, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_attention_prefill_scored": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                                         _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_ll, _c_float,
                                         _c_void_p, _c_ll, _c_void_p, _c_int, _c_float, _c_int, _c_int, _c_int, _c_int,
                                         _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_attention_prefill": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                                  _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                                  _c_int, _c_int, _c_int, _c_void_p],
        "tnx_attention_decode": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                                 _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                                 _c_int, _c_int, _c_int, _c_void_p, _c_int, _c_void_p],
        "tnx_attention_decode_static": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                                        _c_int, _c_int, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                                        _c_int, _c_int, _c_void_p, _c_void_p],
    },
    "sampling": {
        "tnx_ban_tokens": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
        "tnx_ban_pairs": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_argmax": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
        "tnx_store_tokens": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p,
                             _c_void_p],
        "tnx_sample": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                       _c_int, _c_void_p],
    },
    "stream": {
        "tnx_embed_pairs": [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_ll, _c_ll,
                            _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                            _c_void_p],
        "tnx_norm_add": [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_int, _c_void_p, _c_float, _c_void_p, _c_void_p,
                         _c_int, _c_int, _c_int, _c_void_p],
        "tnx_rows_fit": [_c_int],
        "tnx_join_norm_conv": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_float, _c_void_p, _c_void_p,
                               _c_void_p, _c_int, _c_float, _c_void_p, _c_void_p, _c_ll, _c_int, _c_void_p, _c_void_p,
                               _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                               _c_void_p],
        "tnx_input_conv": [_c_void_p, _c_void_p, _c_void_p, _c_ll, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                           _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_poly_norm": [_c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_mul_columns": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_int, _c_void_p],
        "tnx_weighted_sum": [_c_void_p, _c_void_p, _c_int, _c_ll, _c_void_p, _c_ll, _c_void_p],
    },
    "latent": {
        "tnx_latent_norms": [_c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int,
                             _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_ll, _c_ll,
                             _c_int, _c_int, _c_void_p, _c_ll, _c_int, _c_void_p],
        "tnx_latent_attention_mfma": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                                      _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_int, _c_void_p,
                                      _c_void_p, _c_void_p, _c_ll, _c_ll, _c_ll, _c_void_p, _c_int, _c_float, _c_int,
                                      _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_void_p,
                                      _c_void_p, _c_ll, _c_void_p],
        "tnx_batched_linear": [_c_void_p, _c_int, _c_ll, _c_ll, _c_void_p, _c_int, _c_void_p, _c_int, _c_float, _c_int,
                               _c_int, _c_int, _c_int, _c_void_p],
        "tnx_latent_gather": [_c_void_p, _c_void_p, _c_ll, _c_ll, _c_int, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p,
                              _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_expanded_attention": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                                   _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_ll, _c_void_p, _c_int, _c_float,
                                   _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_ll, _c_void_p],
        "tnx_latent_attention_any": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                                     _c_int, _c_int, _c_void_p, _c_void_p, _c_ll, _c_ll, _c_void_p, _c_int, _c_float,
                                     _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_ll,
                                     _c_void_p],
    },
    "prepare": {
        "tnx_qkv_prepare": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_int, _c_void_p,
                            _c_float, _c_void_p, _c_void_p, _c_ll, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                            _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                            _c_int, _c_void_p, _c_void_p],
    },
    "memory": {
        "tnx_matrix_memory": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                              _c_int, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                              _c_int, _c_float, _c_void_p],
    },
    "experts": {
        "tnx_route": [_c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_float,
                      _c_void_p],
        "tnx_expert_mixture": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                               _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                               _c_int, _c_int, _c_float, _c_void_p],
        "tnx_gated_activation": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_float, _c_void_p],
        "tnx_expert_order": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                             _c_void_p, _c_void_p],
        "tnx_expert_combine": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    },
    "hyper": {
        "tnx_add_sinusoid": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                             _c_float, _c_void_p],
        "tnx_hyper_step": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p,
                           _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    },
    "recurrent": {
        "tnx_min_gru": [_c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_ll, _c_int,
                        _c_float, _c_int, _c_int, _c_void_p],
        "tnx_channel_conv": [_c_void_p, _c_ll, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p,
                             _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p],
        "tnx_gated_linear_recurrence": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_ll, _c_void_p, _c_void_p,
                                        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_ll, _c_int, _c_float, _c_int,
                                        _c_int, _c_int, _c_int, _c_void_p],
    },
    "scored": {
        "tnx_attention_scored_mfma": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                                      _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_int, _c_void_p, _c_ll,
                                      _c_float, _c_void_p, _c_ll, _c_void_p, _c_int, _c_float, _c_int, _c_int, _c_int,
                                      _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_int, _c_void_p],
        "tnx_attention_scored": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                                 _c_int, _c_void_p, _c_ll, _c_float, _c_void_p, _c_ll, _c_void_p, _c_int, _c_float,
                                 _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    },
    "probe": {
        "tnx_probe_stream_read": [_c_void_p, ctypes.c_size_t, _c_void_p, _c_int, _c_void_p],
        "tnx_probe_mfma_loop": [_c_int, _c_int, _c_void_p, _c_void_p],
    },
}


def register_signatures(module: str, signatures: Dict[str, list]) -> None:
    """The C entry points (name -> ctypes argument types, all returning int) of a kernel module registered
    with `build.register_module`."""
    _SIGNATURES.setdefault(module, {}).update(signatures)


class PreparedWeight:
    """A `[out, in]` matrix as the kernels want it: the tensor itself, and beside it (bfloat16, `out` a
    multiple of 16, `in` of 128) a copy in the order the few-rows kernel streams it,
    `[out/16][in/128][4][16][4][8]`: each block then reads one contiguous run of memory. The copy doubles
    the memory of the matrices; it is what decoding reads, the plain tensor is what prompts read."""

    __slots__ = ("tensor", "tiles", "folded", "inner")

    def __init__(self, tensor: torch.Tensor, tiles: Optional[torch.Tensor], inner: Optional[int] = None):
        self.tensor, self.tiles = tensor, tiles
        self.folded: Optional["FoldedNorm"] = None
        # the matrix's own inner size where `tensor` carries columns of zeros after it (bfloat16 rows are
        # read 16 bytes at a time: an inner size that is no multiple of 8 is filled up once, here, and the
        # rows that meet it are filled up as they come)
        self.inner = tensor.shape[1] if inner is None else inner

    @property
    def shape(self):
        return torch.Size((self.tensor.shape[0], self.inner))

    @property
    def dtype(self):
        return self.tensor.dtype


class FoldedNorm:
    """A matrix with the LayerNorm in front of it folded in, for the few-rows kernel: `tiles` is
    W diag(gamma) in tile order, `c` its row sums (of the rounded values, which are what is multiplied),
    `d` = W beta; `key` names the norm's tensors it was made from."""

    __slots__ = ("tiles", "c", "d", "key", "_with_bias")

    def __init__(self, tiles, c, d, key):
        self.tiles, self.c, self.d, self.key = tiles, c, d, key
        self._with_bias = {}

    def d_with(self, bias):
        """`d + bias`: what a plain product of the folded copy with rows that are normalised but not yet
        scaled adds (made once a bias vector)."""
        if bias is None:
            return self.d
        k = bias.data_ptr()
        if k not in self._with_bias:
            self._with_bias[k] = (self.d + bias).contiguous()
        return self._with_bias[k]


class DeferredNorm:
    """The input of a LayerNorm whose output only a matrix product reads: the product of few rows applies the
    norm itself (`HipOps.linear`, `HipOps.qkv_project`); whoever else gets one calls `materialize()`."""

    __slots__ = ("ops", "x", "weight", "bias", "eps", "dtype", "center")

    def __init__(self, ops, x, weight, bias, eps, dtype, center=True):
        self.ops, self.x, self.weight, self.bias, self.eps, self.dtype = ops, x, weight, bias, eps, dtype
        self.center = center

    @property
    def shape(self):
        return self.x.shape

    @property
    def key(self):
        return (self.weight.data_ptr() if self.weight is not None else 0,
                self.bias.data_ptr() if self.bias is not None else 0, bool(self.center))

    def materialize(self):
        return self.ops.layernorm(self.x, self.weight, self.bias, self.eps, self.dtype, False, True, self.center)[1]

    def normalised(self):
        """`(x - mean) rstd` alone, for a product with a folded copy."""
        return self.ops.layernorm(self.x, None, None, self.eps, self.dtype, False, True, self.center)[1]


def tile_order(w: torch.Tensor) -> torch.Tensor:
    """`w[n, k]` -> `[n/16][k/128][s][r][g][e]` with n = 16*nt + r and k = 128*kt + 32*s + 8*g + e."""
    n, k = w.shape
    return w.view(n // 16, 16, k // 128, 4, 4, 8).permute(0, 2, 3, 1, 4, 5).contiguous()


def library(module: str) -> ctypes.CDLL:
    """The compiled library of a kernel module, compiled now if it is not there."""
    lib = _LIBS.get(module)
    if lib is None:
        path = build.find_library(module) or build.compile_module(module)
        lib = ctypes.CDLL(path)
        lib.tnx_last_error.restype = ctypes.c_char_p
        for name, argtypes in _SIGNATURES[module].items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _c_int
        _LIBS[module] = lib
    return lib


def loaded_libraries() -> Dict[str, str]:
    return {m: lib._name for m, lib in _LIBS.items()}


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _F32
    if dtype == torch.bfloat16:
        return _BF16
    raise TypeError(f"the kernels take float32 and bfloat16, not {dtype}")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _want(t: torch.Tensor, name: str, dtype=None, shape=None):
    if not t.is_cuda:
        raise ValueError(f"{name} must be on the GPU")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    return t


class HipOps:
    name = "hip"

    def __init__(self, dtype: torch.dtype, device="cuda:0"):
        self.dtype = dtype
        self.device = torch.device(device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise RuntimeError("the HIP kernels need a GPU; none is visible to torch")
        _code(dtype)
        self.compute_units = torch.cuda.get_device_properties(self.device).multi_processor_count
        self._bias_copies = {}
        self._conv_copies = {}
        self._later = []
        self._tiles_per_block = {}
        self._landing, self._landing_turn = [None, None], 0
        self._ints, self._ints_done, self._ints_turn = [None, None], [None, None], 0

    def _call(self, module: str, fn: str, *args, work=None):
        """`work` = (what, bytes, flops) names the launch for a kernel timer: what it is (its sizes), what it has
        to read and write once, and its multiply-adds times two."""
        lib = library(module)
        timer = debug.timer()
        end = None
        if timer is not None:
            end = timer.start(fn, 0, 0) if work is None else timer.start(f"{fn} {work[0]}", work[1], work[2])
        rc = getattr(lib, fn)(*args)
        if end is not None:
            end.record()
        if rc != 0:
            raise RuntimeError(f"{fn}: {lib.tnx_last_error().decode()}")

    def call(self, module: str, fn: str, *args) -> None:
        """An entry point of any registered kernel module (also one a part brought itself); `stream()` and
        `pointer()` give what such entry points take."""
        self._call(module, fn, *args)

    stream = staticmethod(_stream)
    pointer = staticmethod(_ptr)

    @staticmethod
    def _product_work(m, n, k, item=2, x_item=2, out_item=2, residual=False):
        """What a product out[m, n] = x[m, k] w[n, k]^T is for a kernel timer: its sizes, the bytes it has to move
        (the matrix, the rows, the result, the residual) and its flops."""
        return (f"{m}x{n}x{k}", n * k * item + m * k * x_item + m * n * (out_item + (4 if residual else 0)), 2.0 * m * n * k)

    @staticmethod
    def _attention_work(ctx, which, num_heads, num_kv_heads, head_size, window, item):
        """The same for the attention of a step's decoding runs (`which` "decode": bytes of the keys and values
        they read) or of its longer runs ("prompt": flops of scores and weighted values under the causal mask)."""
        lens, cached = ctx.run_lens_host.astype(np.float64), ctx.cached_lens_host.astype(np.float64)
        pick = lens == 1 if which == "decode" else lens > 1
        seen = cached[pick] + (lens[pick] + 1) / 2                     # keys a query of the run sees on average
        if window:
            seen = np.minimum(seen, window)
        keys = float((lens[pick] * seen).sum())
        nbytes = float((np.minimum(cached[pick] + lens[pick], window or 1e18)).sum()) * 2 * num_kv_heads * head_size * item
        return (f"{which} {int(pick.sum())} runs", nbytes, 4.0 * num_heads * head_size * keys)

    # ---------------------------------------------------------------- input end

    def gather_rows(self, x, rows, indirect=None):
        """`x[rows]`; a row number -1 - k stands for `indirect[k]` (int32, on the device)."""
        _want(x, "x")
        _want(rows, "rows", torch.int32)
        if x.dim() != 2:
            raise ValueError("gather_rows takes a matrix")
        if indirect is not None:
            _want(indirect, "indirect rows", torch.int32)
        out = torch.empty(rows.numel(), x.shape[1], dtype=x.dtype, device=x.device)
        self._call("elementwise", "tnx_gather_rows", _ptr(x), _ptr(rows), _ptr(out), rows.numel(),
                   x.shape[1] * x.element_size(), x.shape[0], _ptr(indirect),
                   indirect.numel() if indirect is not None else 0, _stream())
        return out

    def embed(self, token_ids, table, dtype=None, kept_tokens=None):
        """Rows of the token table; an id -1 - k is the token kept in `kept_tokens[k]`."""
        return self.gather_rows(table, token_ids, kept_tokens)

    def pinned_ints(self, n: int):
        """`n` int32 in pinned host memory, and the address under which kernels reach them."""
        host = torch.empty(n, dtype=torch.int32, pin_memory=True)
        address = ctypes.c_void_p()
        self._call("elementwise", "tnx_device_pointer", ctypes.c_void_p(host.data_ptr()), ctypes.byref(address))
        return host, address

    def copy_ints(self, dst, pinned, n=None) -> None:
        """`dst[:n] = host[:n]` for what `pinned_ints` returned, by a kernel on the current stream."""
        host, address = pinned
        n = host.numel() if n is None else n
        _want(dst, "dst", torch.int32)
        if n > host.numel() or n > dst.numel():
            raise ValueError(f"copy_ints: {n} integers from {host.numel()} into {dst.numel()}")
        self._call("elementwise", "tnx_copy_ints", address, _ptr(dst), n, _stream())

    def send_ints(self, flat):
        """A host array of int32 as a device tensor, through pinned memory and a copy kernel (two buffers
        in turn; one is written again only when the copy that read it has run)."""
        n = flat.size
        self._ints_turn ^= 1
        i = self._ints_turn
        if self._ints_done[i] is not None:
            self._ints_done[i].synchronize()   # also before a buffer is replaced: its copy may still read it
        if self._ints[i] is None or self._ints[i][0].numel() < n:
            self._ints[i] = self.pinned_ints(max(2 * n, 1024))
        self._ints[i][0].numpy()[:n] = flat
        dst = torch.empty(n, dtype=torch.int32, device=self.device)
        self.copy_ints(dst, self._ints[i], n)
        if self._ints_done[i] is None:
            self._ints_done[i] = torch.cuda.Event()
        self._ints_done[i].record()
        return dst

    def send_tokens(self, tokens, kept, ctx):
        """Leave the chosen tokens for the next step (`kept[slot]`, see `store_tokens`) and write them into
        pinned host memory by the same kernel. Returns what `receive_tokens` takes."""
        n = tokens.numel()
        self._landing_turn ^= 1
        pinned = self._landing[self._landing_turn]
        if pinned is None or pinned[0].numel() < n:
            pinned = self._landing[self._landing_turn] = self.pinned_ints(max(2 * n, 256))
        self.store_tokens(kept, tokens, ctx, pinned[1])
        landed = torch.cuda.Event()
        landed.record()
        return pinned[0], n, landed

    def receive_tokens(self, sent):
        host, n, landed = sent
        landed.synchronize()
        return host[:n].tolist()

    def store_tokens(self, kept, tokens, ctx, landing=None):
        """`kept[slot]` = the token chosen for the request in that slot; `tokens[i]` belongs to the
        request of the step's i-th wanted row. `landing`: an address in pinned host memory that gets
        the tokens too."""
        _want(kept, "kept tokens", torch.int32)
        _want(tokens, "tokens", torch.int32, (ctx.logits_rows.numel(),))
        self._call("sampling", "tnx_store_tokens", _ptr(tokens), _ptr(ctx.logits_rows), _ptr(ctx.token_request),
                   _ptr(ctx.slots), tokens.numel(), _ptr(kept), kept.numel(), landing, _stream())

    def add_positions(self, src, positions, table, offset, dtype, want_compute, scale=1.0):
        _want(src, "src")
        t, width = src.shape
        _want(positions, "positions", torch.int32, (t,))
        _want(table, "position table")
        if table.shape[1] != width:
            raise ValueError(f"position table is {table.shape[1]} wide, the tokens {width}")
        out = torch.empty(t, width, dtype=torch.float32, device=src.device)
        cd = torch.empty(t, width, dtype=dtype, device=src.device) if want_compute and dtype != torch.float32 else None
        self._call("elementwise", "tnx_add_positions", _ptr(src), _code(src.dtype), _ptr(positions), _ptr(table),
                   _code(table.dtype), table.shape[0], offset, _ptr(out), _ptr(cd), _code(dtype), t, width, float(scale),
                   _stream())
        return out, ((cd if cd is not None else out) if want_compute else None)

    def to_stream(self, src, dtype, want_compute, scale=1.0):
        _want(src, "src")
        t, width = src.shape
        out = torch.empty(t, width, dtype=torch.float32, device=src.device)
        cd = torch.empty(t, width, dtype=dtype, device=src.device) if want_compute and dtype != torch.float32 else None
        self._call("elementwise", "tnx_add_positions", _ptr(src), _code(src.dtype), None, None, 0, 0, 0, _ptr(out),
                   _ptr(cd), _code(dtype), t, width, float(scale), _stream())
        return out, ((cd if cd is not None else out) if want_compute else None)

    def cast(self, x, dtype):
        _want(x, "x")
        if x.dtype == dtype:
            return x
        out = torch.empty_like(x, dtype=dtype)
        self._call("elementwise", "tnx_cast", _ptr(x), _code(x.dtype), _ptr(out), _code(dtype), x.numel(), _stream())
        return out

    # ---------------------------------------------------------------- norms

    def layernorm(self, x, weight, bias, eps, dtype, want_f32, want_compute, center=True):
        """`center=False`: the norm that only scales, x / sqrt(mean(x^2) + eps) (times weight, plus bias)."""
        _want(x, "x", torch.float32)
        t, width = x.shape
        if weight is not None:
            _want(weight, "norm weight", torch.float32, (width,))
        if bias is not None:
            _want(bias, "norm bias", torch.float32, (width,))
        same = dtype == torch.float32
        out_f32 = torch.empty_like(x) if (want_f32 or (want_compute and same)) else None
        out_cd = torch.empty(t, width, dtype=dtype, device=x.device) if (want_compute and not same) else None
        self._call("elementwise", "tnx_layernorm", _ptr(x), _ptr(weight), _ptr(bias), float(eps), _ptr(out_f32),
                   _ptr(out_cd), _code(dtype), t, width, int(bool(center)), _stream(),
                   work=(f"{t}x{width}", t * width * (4 + (4 if out_f32 is not None else 0) + (2 if out_cd is not None else 0)), 0.0))
        return (out_f32 if want_f32 else None), ((out_f32 if same else out_cd) if want_compute else None)

    # Steps of few rows: a LayerNorm that only a matrix product reads is done by that product (`fold_norm`,
    # `layernorm_deferred`). Up to `fuse_norm_rows` rows the few-rows kernel reads the float32 rows itself
    # (measured at 4,096 -> 12,288: 23.0 us against 24.4 for norm and product at 8 rows, but 25.8 against 25.2 at
    # 16 and twice the time at 32: every block reads all rows, and these are float32); beyond that, as far as
    # the few-rows kernel goes, the norm's kernel normalises and the folded copy does the rest.
    # Where the blocks take one tile of weight rows each (what `tnx_gemm_skinny_tiles_per_block` says), every
    # 32 bytes of weight come with 64 of float32 rows and the norm's own kernel is the cheaper way again
    # (9,216 -> 27,648 at 8 rows: 120 us against 10 + 91). And where the blocks between them read more than
    # `fuse_norm_bytes` of rows: 4,096 -> 16,384, 512 blocks of two tiles, is 0.3 to 0.6 us quicker with the norm
    # inside up to 4 rows, as quick at 6 (50 MB of rows) and 0.8 us slower at 8 (28.1 against 27.3 us), while
    # 4,096 -> 12,288, 256 blocks of three, stays 0.6 us quicker at 8 rows (34 MB); 9,216 -> 36,864 at 8 rows
    # (226 MB): 111.1 us against 106.3.
    fuse_norm = True
    fuse_norm_rows = 8
    fuse_norm_bytes = 40 << 20

    def _norm_in_the_product(self, m, n, k) -> bool:
        if m > self.fuse_norm_rows:
            return False
        key = (m, n)
        if key not in self._tiles_per_block:
            self._tiles_per_block[key] = library("gemm").tnx_gemm_skinny_tiles_per_block(m, n)
        tiles = self._tiles_per_block[key]
        blocks = -(-(n // 16) // tiles)
        return tiles >= 2 and blocks * m * k * 4 <= self.fuse_norm_bytes
    few_rows = 32           # the few-rows kernel takes up to this many rows

    def fold_norm(self, w, weight, bias, center=True) -> bool:
        """Called once when a layer has its tensors, for a matrix `w` that reads a LayerNorm's output and
        nothing else does: keeps, in the place of its tile-ordered copy, the copy with the norm's weight
        folded in and the two vectors that go with it (see `FoldedNorm`). False if this matrix has no such
        copy (then the norm stays a kernel of its own)."""
        if not (self.fuse_norm and self.dtype == torch.bfloat16 and isinstance(w, PreparedWeight)
                and w.tiles is not None and w.tensor.dtype == torch.bfloat16):
            return False
        full = w.tensor.float()
        scaled = (full * weight.float()[None, :] if weight is not None else full).to(torch.bfloat16)
        c = scaled.float().sum(dim=1).contiguous()
        d = (full @ bias.float() if bias is not None else torch.zeros_like(c)).contiguous()
        key = (weight.data_ptr() if weight is not None else 0, bias.data_ptr() if bias is not None else 0, bool(center))
        w.folded = FoldedNorm(tile_order(scaled), c, d, key)
        w.tiles = None          # the few-rows steps read the folded copy; the memory stays what it was
        return True

    def layernorm_deferred(self, x, weight, bias, eps, dtype, center=True):
        """The compute-dtype output of the norm, or, in steps of few rows, a `DeferredNorm`."""
        if self.fuse_norm and dtype == torch.bfloat16 and self.dtype == torch.bfloat16 \
                and x.shape[0] <= self.few_rows and x.shape[1] % 128 == 0 and not debug.tapping():
            return DeferredNorm(self, x, weight, bias, eps, dtype, center)
        return self.layernorm(x, weight, bias, eps, dtype, False, True, center)[1]

    def _folded_for(self, h, w):
        """The folded copy of `w` that fits the deferred norm `h`, or None."""
        if isinstance(w, PreparedWeight) and w.folded is not None and w.folded.key == h.key:
            return w.folded
        return None

    # ---------------------------------------------------------------- matrix products

    # Keep a tile-ordered copy of every matrix for the few-rows kernel: True, False, or "later", when they do
    # not all fit: then `finish_weights` makes those a number of bytes allows, once everything else is loaded.
    decode_copies = True

    def prepare_weight(self, w: torch.Tensor) -> PreparedWeight:
        """Called once per matrix when a part receives its tensors."""
        tiles = None
        fits = (self.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 2
                and w.shape[0] % 16 == 0 and w.shape[1] % 128 == 0)
        if fits and self.decode_copies == "later":
            pw = PreparedWeight(w, None)
            self._later.append(pw)
            return pw
        if fits and self.decode_copies:
            tiles = tile_order(w)
        if self.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] % 8:
            inner = w.shape[1]
            return PreparedWeight(torch.nn.functional.pad(w, (0, 8 - inner % 8)).contiguous(), None, inner)
        return PreparedWeight(w, tiles)

    def finish_weights(self, budget_bytes: int) -> int:
        """The tile-ordered copies that `budget_bytes` allow, of the matrices that waited for them: those
        with the fewest rows first (measured at OPT-66B sizes, 8 rows: the copy saves 5 us of 37 for
        9,216 x 9,216, 20 of 134 for 9,216 x 36,864, 14 of 105 for 27,648 x 9,216 and 6 of 121 for
        36,864 x 9,216, that is 29, 29, 28 and 8 us a GB). Returns the bytes taken."""
        taken = 0
        waiting, self._later = self._later, []
        for pw in sorted(waiting, key=lambda pw: pw.tensor.shape[0]):      # (stable: layer order within a size)
            size = pw.tensor.numel() * pw.tensor.element_size()
            if pw.tiles is None and taken + size <= budget_bytes:
                pw.tiles = tile_order(pw.tensor)
                taken += size
        return taken

    def linear(self, x, w, bias=None, act=None, residual=None, out_f32=False, force_tiled=False, f32_by_library=False,
               into=None):
        """`f32_by_library`: a float32 result without a residual may come from the vendor library too (many rows);
        left False such a product (the head's) stays on our kernel. `into`: where such a float32 result goes (rows
        of a larger tensor), instead of a tensor of its own."""
        if isinstance(x, DeferredNorm):
            folded = self._folded_for(x, w) if (residual is None and not out_f32 and force_tiled != 1) else None
            if folded is not None and self._library_product(x.shape[0], w.tensor.shape[0], w.tensor.shape[1],
                                                              w.tensor, force_tiled):
                folded = None
            if folded is None:
                x = x.materialize()
            elif not self._norm_in_the_product(x.shape[0], w.tensor.shape[0], w.tensor.shape[1]):
                # the norm's kernel without weight and bias, then the plain product of the folded copy
                m, k = x.shape
                n = w.tensor.shape[0]
                out = torch.empty(m, n, dtype=self.dtype, device=x.x.device)
                rows, shift = x.normalised(), folded.d_with(bias)     # held until the launch is made
                self._call("gemm", "tnx_gemm_bf16", _ptr(rows), _ptr(w.tensor), _ptr(folded.tiles), _ptr(shift), None,
                           _ptr(out), _code(self.dtype), _ACT[act], m, n, k, int(force_tiled), _stream(),
                           work=self._product_work(m, n, k))
                return out
            else:
                if act not in _ACT:
                    raise ValueError(f"unknown activation {act!r}")
                m, k = x.shape
                n = w.tensor.shape[0]
                if bias is not None:
                    _want(bias, "bias", torch.float32, (n,))
                out = torch.empty(m, n, dtype=self.dtype, device=x.x.device)
                self._call("gemm", "tnx_gemm_bf16_normed", _ptr(x.x), _ptr(folded.tiles), _ptr(folded.c),
                           _ptr(folded.d), float(x.eps), _ptr(bias), _ptr(out), _code(self.dtype), _ACT[act], m, n, k,
                           int(force_tiled), int(bool(x.center)), _stream(), work=self._product_work(m, n, k, x_item=4))
                return out
        tiles = None
        if isinstance(w, PreparedWeight):
            if w.inner != w.tensor.shape[1] and x.shape[1] == w.inner:
                x = torch.nn.functional.pad(x, (0, w.tensor.shape[1] - w.inner))
            w, tiles = w.tensor, w.tiles
        _want(x, "x")
        _want(w, "w")
        if act not in _ACT:
            raise ValueError(f"unknown activation {act!r}")
        m, k = x.shape
        n, kw = w.shape
        if kw != k:
            raise ValueError(f"x is {k} wide, w takes {kw}")
        if bias is not None:
            _want(bias, "bias", torch.float32, (n,))
        if residual is not None:
            _want(residual, "residual", torch.float32, (m, n))
        out_dtype = torch.float32 if out_f32 else self.dtype
        if self._some_rows_product(m, n, k, w, tiles, residual, out_f32, force_tiled):
            # decode batches of 33 to 128 requests, a float32 result: our kernel for some rows
            out = torch.empty(m, n, dtype=out_dtype, device=x.device)
            space = self._library_workspace(x.device)
            self._call("gemm", "tnx_gemm_bf16_mid", _ptr(self.cast(x, torch.bfloat16)), _ptr(tiles), _ptr(bias),
                       _ptr(residual), _ptr(out), _code(out_dtype), _ACT[act], m, n, k, _ptr(space), space.numel() // 4,
                       0, 0, _stream(), work=self._product_work(m, n, k, out_item=4, residual=residual is not None))
            return out
        if (self._library_product(m, n, k, w, force_tiled) and (residual is not None or not out_f32)):
            # Many rows: the product goes to the vendor library (hipBLASLt), with what follows it where the
            # library can do that itself: bias and ReLU before it rounds a bfloat16 result, or bias and the
            # residual added to its float32 sums for a float32 result. The float32 head keeps our kernel.
            xa = self.cast(x, torch.bfloat16)
            # (its ReLU comes after everything it adds, so a product with both ReLU and a residual is not its)
            plain_act = act in (None, "none")
            if self.library_direct and (plain_act or (act == "relu" and residual is None)) \
                    and (residual is None or out_f32):
                out = torch.empty(m, n, dtype=out_dtype, device=x.device)
                if self._library_call(xa, w, bias, residual, out, act, m, n, k):
                    return out
            # Not to be had that way (another activation, no library to be found, no algorithm that fits):
            # the product through torch, and one kernel of ours for what follows it.
            if bias is not None and residual is None and not out_f32:
                b16 = self._bias_bf16(bias)
                if act == "relu":
                    return torch._addmm_activation(b16, xa, w.t(), use_gelu=False)
                y = torch.addmm(b16, xa, w.t())
                bias = None
            else:
                y = torch.mm(xa, w.t())
            out = torch.empty(m, n, dtype=out_dtype, device=x.device) if out_f32 else y
            if bias is not None or residual is not None or (act not in (None, "none")) or out_f32:
                self._call("elementwise", "tnx_epilogue", _ptr(y), _ptr(bias), _ACT[act], _ptr(residual), _ptr(out),
                           _code(out_dtype), m, n, _stream())
            return out
        out = torch.empty(m, n, dtype=out_dtype, device=x.device) if into is None else _want(into, "into", out_dtype, (m, n))
        if (f32_by_library and out_f32 and residual is None and act in (None, "none") and self.library_direct
                and self._library_product(m, n, k, w, force_tiled)
                and self._library_call(self.cast(x, torch.bfloat16), w, bias, None, out, act, m, n, k)):
            return out
        if w.dtype == torch.float32:
            xa = self.cast(x, torch.float32)
            self._call("gemm", "tnx_gemm_f32", _ptr(xa), _ptr(w), _ptr(bias), _ptr(residual), _ptr(out),
                       _code(out_dtype), _ACT[act], m, n, k, _stream(),
                       work=self._product_work(m, n, k, 4, 4, out.element_size(), residual is not None))
        else:
            xa = self.cast(x, torch.bfloat16)
            self._call("gemm", "tnx_gemm_bf16", _ptr(xa), _ptr(w), _ptr(tiles), _ptr(bias), _ptr(residual),
                       _ptr(out), _code(out_dtype), _ACT[act], m, n, k, int(force_tiled), _stream(),
                       work=self._product_work(m, n, k, out_item=out.element_size(), residual=residual is not None))
        return out

    library_direct = True   # many-rows products as calls of the vendor library itself, with what follows them
    library_tune = 1        # and its algorithms timed once: 1, for products of few rows; 2, for every product
    _workspaces: Dict[str, torch.Tensor] = {}

    def _library_call(self, xa, w, bias, residual, out, act, m, n, k) -> bool:
        """`out = act(xa w^T + bias) + residual` by the vendor library; False where that is not to be had."""
        lib = library("gemm")
        space = self._library_workspace(xa.device)

        def call(flush, tune):
            return lib.tnx_gemm_library(_ptr(xa), _ptr(w), _ptr(bias), _ptr(residual), _ptr(out), _code(out.dtype),
                                        _ACT[act], m, n, k, _ptr(space), space.numel(), _ptr(flush),
                                        flush.numel() if flush is not None else 0, int(tune), _stream())
        timer = debug.timer()
        end = None
        if timer is not None:
            what, nbytes, flops = self._product_work(m, n, k, out_item=out.element_size(), residual=residual is not None)
            end = timer.start(f"tnx_gemm_library {what}", nbytes, flops)
        rc = call(None, self.library_tune)
        if end is not None:
            end.record()
        if rc == 3:
            # the algorithms for this size are timed now, once: with memory to push the operands out of the
            # caches, as large as the last-level cache; without it, if the device has no room, nothing is timed
            try:
                flush = torch.empty(256 << 20, dtype=torch.uint8, device=xa.device)
            except torch.OutOfMemoryError:
                flush = None
            rc = call(flush, int(self.library_tune) if flush is not None else 0)
        if rc == 1:
            raise RuntimeError(f"tnx_gemm_library: {lib.tnx_last_error().decode()}")
        return rc == 0

    @classmethod
    def _library_workspace(cls, device) -> torch.Tensor:
        """Memory the library's algorithms may ask for (those that split the inner dimension over blocks keep
        partial sums there, as does our kernel for some rows), one block per device, made at the first product
        and kept. Products on different streams of one device would share it: the engine runs its steps on
        one stream."""
        key = str(device)
        if key not in cls._workspaces:
            cls._workspaces[key] = torch.empty(32 << 20, dtype=torch.uint8, device=device)
        return cls._workspaces[key]

    # From this many rows on, plain bfloat16 products go to the vendor library (0: never). Up to 16 rows our
    # own kernel streams the weight as fast as the library does and fuses what follows the product.
    library_rows = 17

    def _bias_bf16(self, bias):
        """The bfloat16 copy of a float32 bias that the library's epilogue takes, made once. The original
        is held with it, so that its address names no other tensor while the copy is kept."""
        kept = self._bias_copies.get(bias.data_ptr())
        if kept is None or kept[0] is not bias:
            kept = (bias, bias.to(torch.bfloat16))
            self._bias_copies[bias.data_ptr()] = kept
        return kept[1]

    # Products of 17 to 128 rows with a float32 result (those that end in the residual sum, and the head): the
    # vendor library's kernels for such sizes leave much of the memory's rate unused (4,096 columns, K of
    # 16,384, 64 rows: 41 us against 31 here; 5,120 columns, K of 20,480, 32 rows: 68 against 41). Our kernel
    # gives a block 64 columns and shares K out until every compute unit has a block at most, so it is taken
    # where that leaves three units in four with one (9,216 columns make 144 blocks on 256 units, and there
    # the library is as good or better: 147 us against 195 at K of 36,864 and 64 rows), for matrices small
    # enough that the launches count and not the bytes, and for the head up to 64 rows (50,272 columns, more
    # column blocks than units; at 128 rows every block's reading of all rows costs more than it saves). Up to
    # 32 rows a small matrix stays with the few-rows kernel, one launch.
    some_rows = True

    def _some_rows_product(self, m, n, k, w, tiles, residual, out_f32, force_tiled) -> bool:
        if not (self.some_rows and tiles is not None and 16 < m <= 128 and out_f32 and not force_tiled
                and self.dtype == torch.bfloat16 and w.dtype == torch.bfloat16):
            return False
        small = n * k <= self.small_matrix
        if m <= self.few_rows and small:
            return False
        column_blocks = -(-n // 64)
        if column_blocks > self.compute_units:
            return residual is None and m <= 64
        shares = max(1, min(self.compute_units // column_blocks, k // 512))     # as the kernel shares K out
        return small or 4 * column_blocks * shares >= 3 * self.compute_units

    def _library_product(self, m, n, k, w, force_tiled) -> bool:
        if not (self.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and self.library_rows > 0
                and m >= self.library_rows and not force_tiled and n % 8 == 0 and k % 8 == 0):
            return False
        # small matrices at up to 32 rows: one launch of ours (5 to 10 us with its epilogue) beats the
        # library's product and the epilogue after it (11 to 15 us)
        return not (m <= 32 and n * k <= self.small_matrix)

    small_matrix = 1 << 23

    # ---------------------------------------------------------------- attention

    def _check_pages(self, k_pages, v_pages, num_kv, head_size, page_size):
        """The number of pages. A page's own elements lie together; from page to page there may be more than a
        page's elements, the same for keys and values (`_page_pad`: how many more)."""
        n = k_pages.shape[0]
        for t, name, shape in ((k_pages, "key pages", (n, num_kv, page_size, head_size)),
                               (v_pages, "value pages", (n, num_kv, head_size, page_size))):
            if not t.is_cuda or t.dtype != self.dtype:
                raise TypeError(f"{name} must be {self.dtype} on the GPU, got {t.dtype} on {t.device}")
            if tuple(t.shape) != shape:
                raise ValueError(f"{name} have shape {tuple(t.shape)}, expected {shape}")
            inner = (shape[2] * shape[3], shape[3], 1)
            if tuple(t.stride()[1:]) != inner or t.stride(0) < num_kv * inner[0] or (t.stride(0) - num_kv * inner[0]) % 8:
                raise ValueError(f"{name} must hold each page's elements together, pages a multiple of 8 elements "
                                 f"apart; strides {tuple(t.stride())}")
        if k_pages.stride(0) != v_pages.stride(0):
            raise ValueError("key and value pages must lie equally far apart")
        return n

    @staticmethod
    def _page_pad(pages, num_kv, head_size, page_size) -> int:
        return int(pages.stride(0) - num_kv * head_size * page_size) if pages is not None else 0

    @staticmethod
    def _turn_args(turn, head_size, ctx):
        """(a, b, positions, rows) of pair-turning tables as the entry points take them; all None / 0 without."""
        if turn is None:
            return None, None, None, 0
        a, b = turn
        _want(a, "turn a", torch.float32)
        _want(b, "turn b", torch.float32, tuple(a.shape))
        if a.dim() != 2 or a.shape[1] != head_size or head_size % 2:
            raise ValueError(f"pair-turning tables are [positions, head_size] with an even head size, got {tuple(a.shape)} "
                             f"for a head of {head_size}")
        return a, b, ctx.positions, a.shape[0]

    def qkv_project(self, h, w, bias, num_heads, num_kv_write, head_size, scale, ctx, view, k_pages, v_pages,
                    force_tiled=0, turn=None):
        """Queries, keys and values of the step's tokens: one matrix product whose epilogue scales the
        queries and stores keys and values in their pages (bfloat16), or product and `qkv_write` apart.
        `turn` = (a, b), float32 `[positions, head_size]`: element d of every query and key head of a token at
        position p becomes a[p, d] x[d] + b[p, d] x[d ^ 1] (bias added, before the scale), in the same launch."""
        turn_a, turn_b, turn_pos, turn_rows = self._turn_args(turn, head_size, ctx)
        if isinstance(h, DeferredNorm):
            folded = self._folded_for(h, w) if force_tiled != 1 else None
            if folded is not None and (ctx.num_tokens >= 128 or self._library_product(
                    ctx.num_tokens, w.tensor.shape[0], w.tensor.shape[1], w.tensor, force_tiled)):
                folded = None
            if folded is None:
                h = h.materialize()
            elif not self._norm_in_the_product(h.shape[0], w.tensor.shape[0], w.tensor.shape[1]):
                # the norm's kernel without weight and bias, then the fused projection of the folded copy
                h, w, bias = h.normalised(), PreparedWeight(w.tensor, folded.tiles), folded.d_with(bias)
            else:
                t = ctx.num_tokens
                total = (num_heads + 2 * num_kv_write) * head_size
                _want(h.x, "x", torch.float32, (t, w.tensor.shape[1]))
                if tuple(w.tensor.shape) != (total, h.x.shape[1]):
                    raise ValueError(f"w is {tuple(w.tensor.shape)}, the projections need {(total, h.x.shape[1])}")
                if bias is not None:
                    _want(bias, "qkv bias", torch.float32, (total,))
                num_pages = 0
                if num_kv_write:
                    num_pages = self._check_pages(k_pages, v_pages, num_kv_write, head_size, view.page_size)
                _want(view.token_page, "token pages", torch.int32, (t,))
                _want(view.token_offset, "token offsets", torch.int32, (t,))
                q = torch.empty(t, num_heads * head_size, dtype=self.dtype, device=h.x.device)
                self._call("gemm", "tnx_gemm_bf16_qkv_normed", _ptr(h.x), _ptr(folded.tiles), _ptr(folded.c),
                           _ptr(folded.d), float(h.eps), _ptr(bias), t, h.x.shape[1], _ptr(view.token_page),
                           _ptr(view.token_offset), _ptr(q), _ptr(k_pages) if num_kv_write else None,
                           _ptr(v_pages) if num_kv_write else None, float(scale), num_heads, num_kv_write, head_size,
                           view.page_size, num_pages, int(force_tiled), _ptr(turn_a), _ptr(turn_b), _ptr(turn_pos),
                           turn_rows, self._page_pad(k_pages if num_kv_write else None, num_kv_write, head_size,
                                                     view.page_size), int(bool(h.center)), _stream(),
                           work=self._product_work(t, total, h.x.shape[1], x_item=4))
                return q
        tiles = None
        if isinstance(w, PreparedWeight):
            w, tiles = w.tensor, w.tiles
        many = ctx.num_tokens >= 128 and w.shape[1] % 64 == 0 and w.shape[0] % 8 == 0 and not force_tiled
        if self.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and (many or self._library_product(
                ctx.num_tokens, w.shape[0], w.shape[1], w, force_tiled)):
            # many rows (the vendor library, or our wide-tile kernel where sizes allow): the bias joins the
            # product's float32 sums before they are rounded, once, as in the fused kernel below, so that keys
            # and values are cached with the same rounding whichever path a token took; the queries are
            # scaled after that
            return self.qkv_write(self.linear(h, w, bias), None, num_heads, num_kv_write, head_size, scale, ctx,
                                  view, k_pages, v_pages, turn)
        if self.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
            return self.qkv_write(self.linear(h, w, None), bias, num_heads, num_kv_write, head_size, scale, ctx,
                                  view, k_pages, v_pages, turn)
        t = ctx.num_tokens
        total = (num_heads + 2 * num_kv_write) * head_size
        _want(h, "h", torch.bfloat16, (t, w.shape[1]))
        _want(w, "w", torch.bfloat16, (total, h.shape[1]))
        if bias is not None:
            _want(bias, "qkv bias", torch.float32, (total,))
        num_pages = 0
        if num_kv_write:
            num_pages = self._check_pages(k_pages, v_pages, num_kv_write, head_size, view.page_size)
        _want(view.token_page, "token pages", torch.int32, (t,))
        _want(view.token_offset, "token offsets", torch.int32, (t,))
        q = torch.empty(t, num_heads * head_size, dtype=self.dtype, device=h.device)
        self._call("gemm", "tnx_gemm_bf16_qkv", _ptr(h), _ptr(w), _ptr(tiles), _ptr(bias), t, h.shape[1],
                   _ptr(view.token_page), _ptr(view.token_offset), _ptr(q),
                   _ptr(k_pages) if num_kv_write else None, _ptr(v_pages) if num_kv_write else None, float(scale),
                   num_heads, num_kv_write, head_size, view.page_size, num_pages, int(force_tiled), _ptr(turn_a),
                   _ptr(turn_b), _ptr(turn_pos), turn_rows,
                   self._page_pad(k_pages if num_kv_write else None, num_kv_write, head_size, view.page_size), _stream(),
                   work=self._product_work(t, total, h.shape[1]))
        return q

    def qkv_write(self, qkv, bias, num_heads, num_kv_write, head_size, scale, ctx, view, k_pages, v_pages, turn=None):
        turn_a, turn_b, _, turn_rows = self._turn_args(turn, head_size, ctx)
        t = ctx.num_tokens
        total = (num_heads + 2 * num_kv_write) * head_size
        _want(qkv, "qkv", self.dtype, (t, total))
        if bias is not None:
            _want(bias, "qkv bias", torch.float32, (total,))
        num_pages = 0
        if num_kv_write:
            num_pages = self._check_pages(k_pages, v_pages, num_kv_write, head_size, view.page_size)
        _want(view.block_table, "block table", torch.int32, (ctx.num_requests, view.width))
        q = torch.empty(t, num_heads * head_size, dtype=self.dtype, device=qkv.device)
        # the values of runs of several tokens are written by tiles (8 positions by 8 elements a thread, 16 bytes a store)
        by_tiles = (self.dtype == torch.bfloat16 and self.value_tiles and num_kv_write
                    and ctx.plan.get("tile_run") is not None and ctx.plan["tile_run"].numel() > 0)
        self._call("attention", "tnx_qkv_write", _ptr(qkv), _code(self.dtype), _ptr(bias), float(scale),
                   _ptr(ctx.positions), _ptr(ctx.token_request), _ptr(view.block_table), view.width, view.page_size,
                   num_pages, _ptr(q), _ptr(k_pages) if num_kv_write else None,
                   _ptr(v_pages) if num_kv_write else None, t, num_heads, num_kv_write, head_size,
                   _ptr(ctx.run_start), _ptr(ctx.cached_lens), _ptr(ctx.plan["tile_run"]), _ptr(ctx.plan["tile_start"]),
                   ctx.plan["tile_run"].numel() if by_tiles else 0, QUERY_TILE, _ptr(turn_a), _ptr(turn_b), turn_rows,
                   self._page_pad(k_pages if num_kv_write else None, num_kv_write, head_size, view.page_size), _stream())
        return q

    def attention(self, q, num_heads, num_kv_heads, head_size, ctx, view, k_pages, v_pages, window=None):
        t = ctx.num_tokens
        _want(q, "q", self.dtype, (t, num_heads * head_size))
        num_pages = self._check_pages(k_pages, v_pages, num_kv_heads, head_size, view.page_size)
        _want(view.block_table, "block table", torch.int32, (ctx.num_requests, view.width))
        if ctx.max_total > view.width * view.page_size:
            raise ValueError("a request is longer than its block table")
        out = torch.empty_like(q)
        window = int(window or 0)
        pad = self._page_pad(k_pages, num_kv_heads, head_size, view.page_size)
        fast = (self.dtype == torch.bfloat16 and not self.force_plain_attention
                and (ctx.plan["decode_runs"].numel() == 0
                     or view.page_size & (view.page_size - 1) == 0))
        if self.dtype == torch.bfloat16 and not fast and not self.force_plain_attention and not HipOps._warned_page_size:
            HipOps._warned_page_size = True
            build._log(f"a page size of {view.page_size} is no power of two: steps with decoding requests run on the "
                       "general attention kernel (one wave a query), several times slower than the matrix-unit "
                       "kernels that pages of 16, 32, 64, ... tokens get")
        if not fast:
            self._call("attention", "tnx_attention_any", _ptr(q), _code(self.dtype), _ptr(k_pages), _ptr(v_pages),
                       _ptr(ctx.positions), _ptr(ctx.token_request), _ptr(view.block_table), view.width,
                       view.page_size, num_pages, _ptr(out), t, num_heads, num_kv_heads, head_size, window, pad,
                       _stream())
            return out
        if ctx.plan["tile_run"].numel():
            self._call("attention", "tnx_attention_prefill", _ptr(q), _ptr(k_pages), _ptr(v_pages),
                       _ptr(ctx.run_start), _ptr(ctx.cached_lens), _ptr(view.block_table), view.width,
                       view.page_size, num_pages, _ptr(ctx.plan["tile_run"]), _ptr(ctx.plan["tile_start"]), ctx.plan["tile_run"].numel(),
                       _ptr(out), num_heads, num_kv_heads, head_size, window,
                       int(self.prefill_direct) or self._prefill_sets(ctx, num_heads, window), QUERY_TILE, pad,
                       _stream(), work=self._attention_work(ctx, "prompt", num_heads, num_kv_heads, head_size, window, 2)
                       if debug.timer() is not None else None)
        n_dec = ctx.plan["decode_runs"].numel()
        if n_dec:
            splits, waves = self._decode_splits(ctx, n_dec * self._decode_blocks(num_heads, num_kv_heads, head_size),
                                                window, head_size)
            part_o = part_ml = None
            if splits > 1:
                part_o = torch.empty(n_dec * num_heads * splits * head_size, dtype=torch.float32, device=q.device)
                part_ml = torch.empty(n_dec * num_heads * splits * 2, dtype=torch.float32, device=q.device)
            self._call("attention", "tnx_attention_decode", _ptr(q), _ptr(k_pages), _ptr(v_pages),
                       _ptr(ctx.run_start), _ptr(ctx.cached_lens), _ptr(view.block_table), view.width,
                       view.page_size, num_pages, _ptr(ctx.plan["decode_runs"]), n_dec, _ptr(out), _ptr(part_o),
                       _ptr(part_ml), num_heads, num_kv_heads, head_size, window, splits, waves,
                       _ptr(ctx.plan["longest_decode"]), pad,
                       _stream(), work=self._attention_work(ctx, "decode", num_heads, num_kv_heads, head_size, window, 2)
                       if debug.timer() is not None else None)
        return out

    # What the choice between one and two sets of waves a block rests on: the time of one 64-key step of a
    # block, in microseconds, measured on an MI355X at head size 128 (a block alone on its compute unit, two
    # blocks that share one, a block of two sets, and what a second round of blocks adds). Only the ratios
    # matter; another chip or head size changes which of two close estimates wins, not the results.
    prefill_step_cost = dict(alone=2.6, shared=3.9, two_sets=4.1, second_round=7.0)

    def _prefill_sets(self, ctx, num_heads, window) -> int:
        """How the staged prompt kernel runs this step: 0, two sets of four waves a block that halve a tile's
        keys between them, or 2, one set. One set lets two blocks share a compute unit and overlap each other's
        waits; two sets halve the time of the tile that sees the most keys, which the launch waits for when the
        blocks are few or uneven. The choice compares two estimates made from `prefill_step_cost`."""
        plan = ctx.plans.get(("prefill_sets", window))
        if plan is None:
            cost = self.prefill_step_cost
            lens, cached = ctx.run_lens_host, ctx.cached_lens_host
            steps = []
            for i in np.nonzero(lens > 1)[0]:
                for q0 in range(0, int(lens[i]), QUERY_TILE):
                    last = int(cached[i]) + min(q0 + QUERY_TILE, int(lens[i]))      # keys the tile's last query sees
                    first = max(0, int(cached[i]) + q0 - window + 1) // 64 if window > 0 else 0
                    steps.append(-(-last // 64) - first)
            steps = np.array(steps)
            halves = (steps + 1) // 2
            units = self.compute_units
            one = max(steps.max() * cost["alone"], steps.sum() * num_heads / units * cost["shared"] / 2)
            two = max(halves.max() * cost["two_sets"], halves.sum() * num_heads / units * cost["two_sets"])
            if len(steps) * num_heads > units:
                two += cost["second_round"]
            plan = ctx.plans[("prefill_sets", window)] = 0 if two < one else 2
        return plan

    _warned_page_size = False         # said once a process
    value_tiles = True                # tests clear it to write every value token by token
    prefill_direct = False            # tests set it: True, the prompt kernel that reads pages without LDS staging;
                                      # 2, the staged one with one set of four waves a block; 3, with two
    force_plain_attention = False     # tests set it to run the one-wave-per-query kernel in bfloat16 too
    decode_waves = 4                  # waves of a decode attention block (8 is kept for head sizes up to 128)
    decode_blocks_wanted = None       # the keys of decoding requests are split until about this many blocks run;
                                      # None: one block a compute unit

    @staticmethod
    def _decode_blocks(num_heads: int, num_kv_heads: int, head_size: int) -> int:
        """Blocks of the decode attention a request and a share of its keys: one a head, or, where heads share
        keys and values, one for every 16 heads of a group (8 at head sizes beyond 128), which read them once."""
        group = num_heads // num_kv_heads
        if group == 1:
            return num_heads
        return num_kv_heads * -(-group // (16 if head_size <= 128 else 8))

    def _decode_splits(self, ctx, pairs: int, window: int, head_size: int = 128):
        """(splits, waves): how many blocks share the keys of one decoding (request, head), and how many
        waves a block has. Blocks of four waves: with the products on the matrix unit a wave keeps the
        next tile's keys and values in flight by itself, and more waves bought nothing (measured at head
        size 128 and a context of 2,048: one request 8 x 4 waves 15.6 us against 16.9 for 4 x 8; eight
        requests 49.7 against 50.9; 64 requests 369 against 376).
        No block gets less than 256 keys of the longest request (a 64-key tile a wave). Requests about as
        long as one another are cut into as many blocks as that allows, up to 8: small blocks spread evenly
        over the compute units whatever the number of pairs (32 heads at 2,048 tokens, tokens a second: 9
        requests 1,582 -> 1,801, 20: 2,388 -> 2,545, 33: 3,067 -> 3,150, 128: 4,398 -> 4,487), except
        where the pairs alone give 0.7 to 1 block a compute unit (7 and 8 requests: whole requests, 1,548
        against 1,520 and 1,675 against 1,654) or a whole number of blocks each, within a twentieth (16, 24,
        32, 48, 64 requests: the many small blocks and the kernel that merges them cost 2 to 3 % there and
        have nothing to even out). Requests of very different lengths are not cut beyond what
        gives every compute unit a block: most blocks of a short request would be empty (64 requests of 16
        to 1,280 tokens: 6,430 tokens a second whole, 4,760 in eight blocks each). A recorded step is sized
        by the same two facts, which are part of what it is recorded under."""
        longest = ctx.length_bound if ctx.length_bound is not None else ctx.plan_host["longest_decode"]
        fills, alike = ctx.plan_host.get("decode_shape", (0, False))
        return self._splits_for(longest, fills, alike, pairs, window, head_size)

    def _splits_for(self, longest: int, fills: int, alike: bool, pairs: int, window: int, head_size: int):
        if not alike:
            fills = min(8, -(-longest // 256))
        if window:
            longest = min(longest, window + 64)
            fills = min(fills, -(-longest // 256))
        waves = 8 if self.decode_waves == 8 and head_size <= 128 else 4
        units = self.decode_blocks_wanted or self.compute_units
        if self.decode_blocks_wanted:                  # told how many blocks to make (measurements and tests)
            return max(1, min(-(-units // pairs), -(-longest // 256))), waves
        if 0.7 * units <= pairs <= units:
            return 1, waves
        fill_the_chip = max(1, min(-(-units // pairs), fills))
        if pairs > units and -(-pairs // units) * units <= 1.05 * pairs:
            alike = False         # whole requests already come out even over the compute units
        return (max(fill_the_chip, fills) if alike else fill_the_chip), waves

    def attention_launch_shape(self, step, num_heads: int, window, head_size: int, num_kv_heads: Optional[int] = None):
        """What the decode attention's launch in a recorded step is sized by beyond the number of requests: the
        blocks that share a request's keys (and their waves), for a `PackedStep` about to be replayed. A
        recorded step is sized for the longest request the model allows; how requests about as long as one
        another are cut depends on how long they are now, so a batch that grows is recorded again only when
        that changes the launch (8 requests of 32 heads: never; 9: at every 256 keys up to eight blocks)."""
        n_dec = int((step.run_lens == 1).sum())
        if n_dec == 0 or self.dtype != torch.bfloat16:
            return None
        fills, alike = step.plan_host.get("decode_shape", (0, False))
        blocks = self._decode_blocks(num_heads, num_kv_heads or num_heads, head_size)
        return ("decode", blocks, head_size) + self._splits_for(step.length_bound, fills, alike, n_dec * blocks,
                                                                int(window or 0), head_size)

    # ---------------------------------------------------------------- parts of other designs

    def embed_pairs(self, token_ids, table, pairs, buckets, mul_prev, mul_cur, ctx, last_token, kept_tokens=None):
        """See `ReferenceOps.embed_pairs`."""
        t = token_ids.numel()
        _want(token_ids, "token ids", torch.int32)
        _want(table, "token table")
        _want(pairs, "pair table", table.dtype, (buckets + 1, table.shape[1]))
        _want(last_token, "last tokens", torch.int32)
        if last_token.dim() != 2 or last_token.shape[1] != 2:
            raise ValueError(f"last tokens are [slots, 2], got {tuple(last_token.shape)}")
        if kept_tokens is not None:
            _want(kept_tokens, "kept tokens", torch.int32)
        out = torch.empty(t, table.shape[1], dtype=torch.float32, device=table.device)
        self._call("stream", "tnx_embed_pairs", _ptr(token_ids), _ptr(kept_tokens),
                   kept_tokens.numel() if kept_tokens is not None else 0, _ptr(table), _ptr(pairs), _code(table.dtype),
                   table.shape[0], buckets, mul_prev, mul_cur, _ptr(ctx.positions), _ptr(ctx.token_request),
                   _ptr(ctx.run_start), _ptr(ctx.slots), _ptr(last_token), _ptr(out), t, table.shape[1],
                   ctx.num_requests, _stream(), work=(f"{t}x{table.shape[1]}", t * table.shape[1] * (4 + 2 * table.element_size()), 0.0))
        return out

    def norm_add(self, y, weight, bias, eps, center, residual, mult=1.0, out=None, want_compute=False):
        """float32 `residual + mult * norm(y)`; `center` as in `layernorm`. With `want_compute` the pair (result,
        its copy in the compute dtype)."""
        _want(y, "y", torch.float32)
        t, width = y.shape
        _want(residual, "residual", torch.float32, (t, width))
        if weight is not None:
            _want(weight, "norm weight", torch.float32, (width,))
        if bias is not None:
            _want(bias, "norm bias", torch.float32, (width,))
        if out is None:
            out = torch.empty_like(y)
        else:
            _want(out, "out", torch.float32, (t, width))
        copy = None
        if want_compute and self.dtype != torch.float32 and self.rows_fit(width):
            copy = torch.empty(t, width, dtype=self.dtype, device=y.device)
        self._call("stream", "tnx_norm_add", _ptr(y), _ptr(weight), _ptr(bias), float(eps), int(bool(center)),
                   _ptr(residual), float(mult), _ptr(out), _ptr(copy), _code(self.dtype), t, width, _stream(),
                   work=(f"{t}x{width}", t * width * (12 + (2 if copy is not None else 0)), 0.0))
        if not want_compute:
            return out
        return out, (copy if copy is not None else self.cast(out, self.dtype))

    fuse_rows = 64       # up to this many rows the join, the norm and the convolution are one launch

    @staticmethod
    def rows_fit(width: int) -> bool:
        """Whether the kernels that hold a row in registers take this width."""
        return bool(library("stream").tnx_rows_fit(int(width)))

    def join_norm_conv(self, x, join, pre, conv_w, state, which, ctx, dtype):
        """What a part reads, in one launch where the width allows: `h = pre_norm(x')`, the result `h + conv(h)`
        as `input_conv` makes it, with `x' = x`, or for `join` = (y, weight, bias, center, mult),
        `x' = x + mult * post_norm(y)`. `pre` = (weight, bias, center, eps), one eps for both norms. Returns
        (x', the result in `dtype`)."""
        t, width = x.shape
        taps = conv_w.shape[1]
        pw, pb, pc, eps = pre
        # Many rows: a token's block makes the rows of the taps - 1 tokens before it again, which costs more than
        # the launches it saves (2,048 rows of 4,096, four taps: 149 us in one launch, 81 in three).
        if not self.rows_fit(width) or t > self.fuse_rows:
            if join is not None:
                x = self.norm_add(join[0], join[1], join[2], eps, join[3], x, join[4])
            h = self.layernorm(x, pw, pb, eps, torch.float32, True, False, pc)[0]
            return x, self.input_conv(h, conv_w, state, which, ctx, dtype)
        _want(x, "x", torch.float32)
        _want(conv_w, "convolution weights", torch.float32, (width, taps))
        conv_w = self._taps_first(conv_w)
        mine, stride = None, 0
        if taps > 1:
            _want(state, "convolution state", torch.float32)
            if state.dim() != 4 or tuple(state.shape[2:]) != (taps, width) or not 0 <= which < state.shape[1]:
                raise ValueError(f"convolution state is [slots, parts, {taps}, {width}], got {tuple(state.shape)}")
            mine, stride = state.data_ptr() + which * taps * width * 4, state.stride(0)
        y = jw = jb = x_out = None
        jc, mult = 1, 1.0
        if join is not None:
            y, jw, jb, jc, mult = join
            _want(y, "y", torch.float32, (t, width))
            x_out = torch.empty_like(x)
        single = bool(ctx.run_lens_host.max() == 1)
        keep = torch.empty(t, width, dtype=torch.float32, device=x.device) if taps > 1 and not single else None
        out = torch.empty(t, width, dtype=dtype, device=x.device)
        self._call("stream", "tnx_join_norm_conv", _ptr(x), _ptr(y), _ptr(jw), _ptr(jb), int(bool(jc)), float(mult),
                   _ptr(x_out), _ptr(pw), _ptr(pb), int(bool(pc)), float(eps), _ptr(conv_w), mine, stride, taps,
                   _ptr(ctx.positions), _ptr(ctx.token_request), _ptr(ctx.run_start), _ptr(ctx.slots), _ptr(out),
                   _code(dtype), _ptr(keep), int(single), t, width, ctx.num_requests, _stream(),
                   work=(f"{t}x{width}{' joined' if join is not None else ''}",
                         t * width * (4 + out.element_size() + (8 if join is not None else 0)), 0.0))
        return (x_out if join is not None else x), out

    def _taps_first(self, weight):
        """The `[width, taps]` weights of a convolution as the kernels read them, `[taps, width]` (made once a
        tensor; the original is held with the copy, so that its address names no other tensor meanwhile)."""
        kept = self._conv_copies.get(weight.data_ptr())
        if kept is None or kept[0] is not weight:
            kept = (weight, weight.t().contiguous())
            self._conv_copies[weight.data_ptr()] = kept
        return kept[1]

    def input_conv(self, h, weight, state, which, ctx, dtype):
        """See `ReferenceOps.input_conv`."""
        _want(h, "h", torch.float32)
        t, width = h.shape
        taps = weight.shape[1]
        _want(weight, "convolution weights", torch.float32, (width, taps))
        weight = self._taps_first(weight)
        mine, stride = None, 0
        if taps > 1:
            _want(state, "convolution state", torch.float32)
            if state.dim() != 4 or tuple(state.shape[2:]) != (taps, width) or not 0 <= which < state.shape[1]:
                raise ValueError(f"convolution state is [slots, parts, {taps}, {width}], got {tuple(state.shape)}")
            mine, stride = state.data_ptr() + which * taps * width * 4, state.stride(0)
        out = torch.empty(t, width, dtype=dtype, device=h.device)
        self._call("stream", "tnx_input_conv", _ptr(h), _ptr(weight), mine, stride, taps, _ptr(ctx.positions),
                   _ptr(ctx.token_request), _ptr(ctx.run_start), _ptr(ctx.slots), _ptr(out), _code(dtype), t, width, ctx.num_requests, _stream(),
                   work=(f"{t}x{width}", t * width * (4 + out.element_size()), 0.0))
        return out

    def poly_norm(self, z, coeffs, eps):
        """See `ReferenceOps.poly_norm`."""
        _want(z, "z", torch.float32)
        _want(coeffs, "coefficients", torch.float32, (4,))
        out = torch.empty(z.shape, dtype=self.dtype, device=z.device)
        self._call("stream", "tnx_poly_norm", _ptr(z), _ptr(coeffs), float(eps), _ptr(out), _code(self.dtype),
                   z.shape[0], z.shape[1], _stream(), work=(f"{z.shape[0]}x{z.shape[1]}", z.numel() * (4 + out.element_size()), 0.0))
        return out

    def mul_columns(self, g, rows, offset):
        _want(g, "g", self.dtype)
        _want(rows, "rows", self.dtype)
        if rows.shape[0] != g.shape[0]:
            raise ValueError(f"{g.shape[0]} rows of g, {rows.shape[0]} rows of the table")
        out = torch.empty_like(g)
        self._call("stream", "tnx_mul_columns", _ptr(g), _ptr(rows), _code(self.dtype), int(offset), g.shape[1],
                   rows.shape[1], _ptr(out), g.shape[0], _stream())
        return out

    def weighted_sum(self, history, weights, count):
        _want(history, "history", torch.float32)
        _want(weights, "weights", torch.float32)
        if not 1 <= count <= history.shape[0] or weights.numel() < count:
            raise ValueError(f"weighted_sum of {count} slots: {history.shape[0]} are there, {weights.numel()} weights")
        out = torch.empty_like(history[0])
        self._call("stream", "tnx_weighted_sum", _ptr(history), _ptr(weights), count, history.stride(0), _ptr(out),
                   out.numel(), _stream(), work=(f"{count}x{out.numel()}", (count + 1) * out.numel() * 4, 0.0))
        return out

    def _latent_pages(self, latent_pages, rotated_pages, kv_rank, rot, page_size, across_pages=None):
        if across_pages is not None:
            a = across_pages
            if not a.is_cuda or a.dtype != self.dtype or a.dim() != 3 or tuple(a.shape) != (latent_pages.shape[0], kv_rank, page_size) \
                    or tuple(a.stride()[1:]) != (page_size, 1) or a.stride(0) < kv_rank * page_size:
                raise ValueError(f"the latents with a page's tokens side by side are [pages, {kv_rank}, {page_size}] in "
                                 f"{self.dtype}, got {tuple(a.shape)} {a.dtype} with strides {tuple(a.stride())}")
        for pages, name, last in ((latent_pages, "latent pages", kv_rank), (rotated_pages, "rotated pages", rot)):
            if not pages.is_cuda or pages.dtype != self.dtype:
                raise TypeError(f"{name} must be {self.dtype} on the GPU, got {pages.dtype} on {pages.device}")
            if pages.dim() != 3 or tuple(pages.shape[1:]) != (page_size, last) or tuple(pages.stride()[1:]) != (last, 1) \
                    or pages.stride(0) < page_size * last:
                raise ValueError(f"{name} are [pages, {page_size}, {last}] with a page's elements together, got "
                                 f"{tuple(pages.shape)} with strides {tuple(pages.stride())}")
        if latent_pages.shape[0] != rotated_pages.shape[0]:
            raise ValueError("latent and rotated pages differ in number")
        return latent_pages.shape[0]

    def latent_norms(self, down, q_rank, kv_rank, rot, q_weight, kv_weight, eps, freqs, ctx, view, latent_pages,
                     rotated_pages, across_pages=None):
        """See `ReferenceOps.latent_norms`."""
        t = ctx.num_tokens
        _want(down, "down", torch.float32)
        if down.dim() != 2 or down.shape[0] != t or down.shape[1] < q_rank + kv_rank + (rot if kv_rank else 0):
            raise ValueError(f"down must be [{t}, {q_rank + kv_rank + rot} or more], got {tuple(down.shape)}")
        if q_rank:
            _want(q_weight, "query latent norm", torch.float32, (q_rank,))
        _want(freqs, "frequencies", torch.float32)
        num_pages = 0
        if kv_rank:
            _want(kv_weight, "key/value latent norm", torch.float32, (kv_rank,))
            num_pages = self._latent_pages(latent_pages, rotated_pages, kv_rank, rot, view.page_size, across_pages)
            _want(view.token_page, "token pages", torch.int32, (t,))
            _want(view.token_offset, "token offsets", torch.int32, (t,))
        c_q = torch.empty(t, q_rank, dtype=self.dtype, device=down.device) if q_rank else None
        self._call("latent", "tnx_latent_norms", _ptr(down), down.shape[1], q_rank, kv_rank, rot,
                   _ptr(q_weight) if q_rank else None, _ptr(kv_weight),
                   float(eps), _ptr(freqs), freqs.numel(), _ptr(ctx.positions), _ptr(view.token_page),
                   _ptr(view.token_offset), _ptr(c_q), _code(self.dtype), _ptr(latent_pages) if kv_rank else None,
                   _ptr(rotated_pages) if kv_rank else None, latent_pages.stride(0) if kv_rank else 0,
                   rotated_pages.stride(0) if kv_rank else 0, num_pages, view.page_size,
                   _ptr(across_pages) if kv_rank and across_pages is not None else None,
                   across_pages.stride(0) if kv_rank and across_pages is not None else 0, t, _stream(),
                   work=(f"{t}x{q_rank}+{kv_rank}+{rot}", t * ((q_rank + kv_rank + rot) * 4 + (q_rank + 2 * kv_rank + rot) * 2), 0.0))
        return c_q

    batched_library_rows = 64      # from this many rows on a bfloat16 product per head goes to the vendor library (0: never)

    def batched_linear(self, x, w, alpha=1.0, out_f32=False):
        """`out[t, h, :] = alpha * w[h] x[t, h, :]`: x `[T, H, K]` (a view whose last axis is dense), w `[H, N, K]`."""
        if x.dim() != 3 or w.dim() != 3 or x.shape[1] != w.shape[0] or x.shape[2] != w.shape[2]:
            raise ValueError(f"batched_linear: x {tuple(x.shape)} does not fit w {tuple(w.shape)}")
        if not x.is_cuda or x.stride(2) != 1:
            raise ValueError("batched_linear: x must be on the GPU with a dense last axis")
        _want(w, "w")
        t, heads, k = x.shape
        n = w.shape[1]
        if (self.dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and not out_f32
                and alpha == 1.0 and t >= self.batched_library_rows > 0):
            # many rows: the vendor library's batched product, as the plain products of many rows go to it
            timer = debug.timer()
            end = timer.start(f"library batched product {t}x{heads}x{n}x{k}", heads * n * k * 2 + t * heads * (k + n) * 2,
                              2.0 * t * heads * n * k) if timer is not None else None
            out = torch.bmm(x.transpose(0, 1), w.transpose(1, 2)).transpose(0, 1).contiguous()
            if end is not None:
                end.record()
            return out
        out = torch.empty(t, heads, n, dtype=torch.float32 if out_f32 else self.dtype, device=x.device)
        self._call("latent", "tnx_batched_linear", _ptr(x), _code(x.dtype), x.stride(0), x.stride(1), _ptr(w),
                   _code(w.dtype), _ptr(out), _code(out.dtype), float(alpha), t, heads, n, k, _stream(),
                   work=(f"{t}x{heads}x{n}x{k}", heads * n * k * w.element_size() + t * heads * (k + n) * 2,
                         2.0 * t * heads * n * k))
        return out

    # Steps that are prompts' runs only, of this many tokens or more: the keys and values of the tokens a run can
    # see are made from the cached latents once a step (library products) and attention runs on them; a (query,
    # key) pair then costs 2 (n + r + v) multiply-adds a head instead of the 2 (2 R + r) of the form that reads the
    # latents as they lie, which is the one for decoding. 0: never.
    expand_rows = 128

    def latent_expands(self, ctx, head_size, rot, value_size, kv_rank) -> bool:
        """Whether `latent_attention_expanded` takes this step."""
        return bool(self.dtype == torch.bfloat16 and self.latent_matrix_unit and self.expand_rows > 0
                    and ctx.num_tokens >= self.expand_rows and "decode_runs" in ctx.plan
                    and ctx.plan["decode_runs"].numel() == 0 and head_size % 8 == 0 and rot % 8 == 0
                    and head_size + rot <= 256 and value_size % 16 == 0 and value_size <= 256 and kv_rank % 8 == 0)

    def latent_attention_expanded(self, q, w_uk, w_uv, num_heads, head_size, rot, value_size, kv_rank, freqs, scale, ctx,
                                  view, latent_pages, rotated_pages, window=None, sink=None, gate=None):
        """Attention of a step of prompts' runs with expanded keys and values: `[T, H * value_size]`, what
        `latent_attention` and the product with W_uv give. `w_uk` `[H * head_size, kv_rank]` and `w_uv`
        `[H * value_size, kv_rank]` are the whole matrices."""
        t = ctx.num_tokens
        _want(q, "q", self.dtype, (t, num_heads * (head_size + rot)))
        num_pages = self._latent_pages(latent_pages, rotated_pages, kv_rank, rot, view.page_size)
        _want(view.block_table, "block table", torch.int32, (ctx.num_requests, view.width))
        lens, cached = ctx.run_lens_host.astype(np.int64), ctx.cached_lens_host.astype(np.int64)
        # what a run can see: from the first key of its first query's window (down to a multiple of 64) to its end,
        # in dense rows that begin at a multiple of 64
        base = (np.maximum(0, cached - window + 1) if window else np.zeros_like(cached)) // 64 * 64
        count = cached + lens - base
        padded = -(-count // 64) * 64
        start = np.concatenate([[0], np.cumsum(padded)[:-1]])
        rows = int(padded.sum())
        row_run = np.repeat(np.arange(len(lens)), padded)
        within = np.arange(rows) - np.repeat(start, padded)
        row_pos = np.where(within < np.repeat(count, padded), np.repeat(base, padded) + within, -1)
        ints = self.send_ints(np.concatenate([row_run, row_pos, start, base]).astype(np.int32))
        row_run_d, row_pos_d = ints[:rows], ints[rows:2 * rows]
        start_d, base_d = ints[2 * rows:2 * rows + len(lens)], ints[2 * rows + len(lens):]
        c_dense = torch.empty(rows, kv_rank, dtype=self.dtype, device=q.device)
        r_dense = torch.empty(rows, max(rot, 1), dtype=self.dtype, device=q.device)
        self._call("latent", "tnx_latent_gather", _ptr(latent_pages), _ptr(rotated_pages), latent_pages.stride(0),
                   rotated_pages.stride(0), view.page_size, num_pages, _ptr(view.block_table), view.width,
                   _ptr(row_run_d), _ptr(row_pos_d), _ptr(c_dense), _ptr(r_dense), kv_rank, rot, rows, _stream(),
                   work=(f"{rows}x{kv_rank}+{rot}", rows * (kv_rank + rot) * 4, 0.0))
        k_n = self.linear(c_dense, w_uk, None)                                   # [rows, H * n]
        uv = w_uv.tensor if isinstance(w_uv, PreparedWeight) else w_uv
        v_t = self.linear(uv, c_dense, None)                                     # [H * v, rows]: tokens side by side
        out = torch.empty(t, num_heads * value_size, dtype=self.dtype, device=q.device)
        tiles = ctx.plan["tile_run"].numel()
        seen = np.minimum(cached + (lens + 1) / 2, window or 1 << 30)
        self._call("latent", "tnx_expanded_attention", _ptr(q), _ptr(k_n), _ptr(r_dense), _ptr(v_t), _ptr(out),
                   _ptr(ctx.run_start), _ptr(ctx.cached_lens), _ptr(start_d), _ptr(base_d), _ptr(ctx.plan["tile_run"]),
                   _ptr(ctx.plan["tile_start"]), tiles, QUERY_TILE, rows, _ptr(freqs), freqs.numel(), float(scale),
                   num_heads, head_size, rot, value_size, int(window or 0), *self._sink_and_gate(sink, gate, t, num_heads),
                   _stream(),
                   work=(f"{tiles} tiles", rows * num_heads * (head_size + value_size) * 2.0,
                         2.0 * num_heads * (head_size + rot + value_size) * float((lens * seen).sum())))
        return out

    def _sink_and_gate(self, sink, gate, t, num_heads):
        """(sink pointer, gate pointer, the gate's row distance) for the latent-attention kernels."""
        if sink is not None:
            _want(sink, "sinks", torch.float32, (num_heads,))
        gate_ld = self._rows_apart(gate, "the gate", torch.float32, t, num_heads) if gate is not None else 0
        return _ptr(sink), _ptr(gate), gate_ld

    latent_matrix_unit = True      # tests clear it to run the any-sizes kernel in bfloat16 too
    latent_prompt_kind = 0         # tests set 1: the prompt kernel whose waves each walk the keys for their own queries

    def latent_attention(self, q, q_lat, num_heads, head_size, rot, kv_rank, freqs, scale, ctx, view, latent_pages,
                         rotated_pages, across_pages=None, window=None, sink=None, gate=None):
        """See `ReferenceOps.latent_attention`. bfloat16 with a latent of a multiple of 16 up to 512 elements, a
        rotated part of a multiple of 8 up to 64 and head sizes in 8s runs on the matrix unit (and reads
        `across_pages`); everything else, and float32, on the kernel for any sizes."""
        t = ctx.num_tokens
        _want(q, "q", self.dtype, (t, num_heads * (head_size + rot)))
        _want(q_lat, "q_lat", self.dtype, (t, num_heads, kv_rank))
        _want(freqs, "frequencies", torch.float32)
        num_pages = self._latent_pages(latent_pages, rotated_pages, kv_rank, rot, view.page_size, across_pages)
        _want(view.block_table, "block table", torch.int32, (ctx.num_requests, view.width))
        if ctx.max_total > view.width * view.page_size:
            raise ValueError("a request is longer than its block table")
        out = torch.empty(t, num_heads, kv_rank, dtype=self.dtype, device=q.device)
        finish = self._sink_and_gate(sink, gate, t, num_heads)
        fast = (self.dtype == torch.bfloat16 and self.latent_matrix_unit and across_pages is not None
                and kv_rank % 16 == 0 and kv_rank <= 512 and rot % 8 == 0 and rot <= 64 and head_size % 8 == 0
                and "tile_run" in ctx.plan and latent_pages.stride(0) % 8 == 0 and rotated_pages.stride(0) % 8 == 0
                and across_pages.stride(0) % 8 == 0)
        if fast:
            tiles, decodes = ctx.plan["tile_run"].numel(), ctx.plan["decode_runs"].numel()
            part, splits, per_split = None, 1, 1
            if decodes:
                # The keys of the decoding requests are shared out over blocks until there is about one a compute
                # unit: a block is 16 heads of a request. A recorded step is sized for the longest request there
                # can be (a window bounds what any request reads).
                longest = ctx.length_bound if ctx.length_bound is not None else ctx.plan_host["longest_decode"]
                key_tiles = (longest - 1) // 64 + 1
                if window:
                    key_tiles = min(key_tiles, (window - 1) // 64 + 2)
                blocks = decodes * -(-num_heads // 16)
                splits = max(1, min(key_tiles, self.compute_units // blocks, 32))
                per_split = -(-key_tiles // splits)
                splits = -(-key_tiles // per_split)
                if splits > 1:
                    part = torch.empty(decodes * num_heads * splits * (kv_rank + 2), dtype=torch.float32, device=q.device)
            seen = float(np.minimum(ctx.cached_lens_host + ctx.run_lens_host, window or 1 << 30).sum())
            self._call("latent", "tnx_latent_attention_mfma", _ptr(q), _ptr(q_lat), _ptr(out), _ptr(ctx.run_start),
                       _ptr(ctx.cached_lens), _ptr(view.block_table), view.width, view.page_size, num_pages,
                       _ptr(ctx.plan["tile_run"]), _ptr(ctx.plan["tile_start"]), tiles, QUERY_TILE,
                       _ptr(ctx.plan["decode_runs"]), decodes, _ptr(latent_pages), _ptr(rotated_pages),
                       _ptr(across_pages), latent_pages.stride(0), rotated_pages.stride(0), across_pages.stride(0),
                       _ptr(freqs), freqs.numel(), float(scale), num_heads, head_size, rot, kv_rank, int(window or 0),
                       _ptr(part), splits, per_split, int(self.latent_prompt_kind), *finish, _stream(),
                       work=(f"{tiles} tiles {decodes} decodes", seen * (2 * kv_rank + rot) * 2,
                             2.0 * num_heads * (2 * kv_rank + rot) * float(
                                 (ctx.run_lens_host * np.minimum(ctx.cached_lens_host + (ctx.run_lens_host + 1) / 2,
                                                                 window or 1 << 30)).sum()))
                       if debug.timer() is not None else None)
            return out
        self._call("latent", "tnx_latent_attention_any", _ptr(q), _code(self.dtype), _ptr(q_lat), _ptr(out),
                   _ptr(ctx.positions), _ptr(ctx.token_request), _ptr(view.block_table), view.width, view.page_size,
                   num_pages, _ptr(latent_pages), _ptr(rotated_pages), latent_pages.stride(0), rotated_pages.stride(0),
                   _ptr(freqs), freqs.numel(), float(scale), num_heads, head_size, rot, kv_rank, int(window or 0), t,
                   *finish, _stream())
        return out


    # ---------------------------------------------------------------- normed, turned and blended projections

    def qkv_prepare(self, proj, num_heads, num_kv, head_size, value_size, cache_head, q_weight, k_weight, eps, freqs,
                    interleaved, scale, mix_weight, first_values, ctx, view, k_pages, v_pages, per_head=False,
                    values_at=None, head_scale=None):
        """See `ReferenceOps.qkv_prepare`. The rows of `proj` may hold more behind the values."""
        t = ctx.num_tokens
        need = num_heads * head_size + num_kv * head_size
        need = max(need, (need if values_at is None else int(values_at)) + num_kv * value_size)
        if head_scale is not None:
            _want(head_scale, "head scales", torch.float32, (num_heads,))
        _want(proj, "projections", torch.float32)
        if proj.dim() != 2 or proj.shape[0] != t or proj.shape[1] < need:
            raise ValueError(f"projections must be [{t}, {need} or more], got {tuple(proj.shape)}")
        total = proj.shape[1]
        if q_weight is not None:
            _want(q_weight, "query norm", torch.float32, (num_heads * head_size,))
            _want(k_weight, "key norm", torch.float32, (num_kv * head_size,))
        if freqs is not None:
            _want(freqs, "frequencies", torch.float32)
        first_ld = 0
        if first_values is not None:
            _want(mix_weight, "blending weight", torch.float32, (1,))
            if (not first_values.is_cuda or first_values.dtype != torch.float32 or first_values.dim() != 2
                    or tuple(first_values.shape) != (t, num_kv * value_size) or first_values.stride(1) != 1):
                raise ValueError(f"the values to blend with are float32 [{t}, {num_kv * value_size}] with dense rows, got "
                                 f"{tuple(first_values.shape)} {first_values.dtype}")
            first_ld = first_values.stride(0)
        num_pages = self._check_pages(k_pages, v_pages, num_kv, cache_head, view.page_size)
        _want(view.token_page, "token pages", torch.int32, (t,))
        _want(view.token_offset, "token offsets", torch.int32, (t,))
        q = torch.empty(t, num_heads * cache_head, dtype=self.dtype, device=proj.device)
        self._call("prepare", "tnx_qkv_prepare", _ptr(proj), total, _ptr(q_weight), _ptr(k_weight), float(eps),
                   _ptr(freqs), freqs.numel() if freqs is not None else 0, int(bool(interleaved)), _ptr(ctx.positions),
                   float(scale), _ptr(mix_weight) if first_values is not None else None, _ptr(first_values), first_ld,
                   _ptr(view.token_page), _ptr(view.token_offset), _ptr(q), _ptr(k_pages), _ptr(v_pages),
                   k_pages.stride(0), num_pages, view.page_size, _code(self.dtype), t, num_heads, num_kv, head_size,
                   value_size, cache_head, int(bool(per_head)), -1 if values_at is None else int(values_at),
                   _ptr(head_scale), _stream(),
                   work=(f"{t}x{total}", t * (total * 4 + (num_heads + 2 * num_kv) * cache_head * q.element_size()), 0.0))
        return q

    # ---------------------------------------------------------------- several copies of the stream

    def add_sinusoid(self, src, positions, freqs, dtype, want_compute, scale=1.0):
        """See `ReferenceOps.add_sinusoid`."""
        _want(src, "src")
        t, width = src.shape
        _want(positions, "positions", torch.int32, (t,))
        _want(freqs, "frequencies", torch.float32, (width // 2,))
        out = torch.empty(t, width, dtype=torch.float32, device=src.device)
        cd = torch.empty(t, width, dtype=dtype, device=src.device) if want_compute and dtype != torch.float32 else None
        self._call("hyper", "tnx_add_sinusoid", _ptr(src), _code(src.dtype), _ptr(positions), _ptr(freqs), _ptr(out),
                   _ptr(cd), _code(dtype), t, width, float(scale), _stream(),
                   work=(f"{t}x{width}", t * width * (4 + src.element_size()), 0.0))
        return out, ((cd if cd is not None else out) if want_compute else None)

    def _hyper(self, copies, pending, read, norm_weight, eps, h32, hcd, total):
        _want(copies, "copies of the stream", torch.float32)
        s, t, width = copies.shape
        y = mix = out_w = None
        if pending is not None:
            y, mix, out_w = pending
            _want(y, "the result to join", torch.float32, (t, width))
            _want(mix, "mix", torch.float32, (s, s))
            _want(out_w, "out", torch.float32, (s,))
        if read is not None:
            _want(read, "in", torch.float32, (s,))
            _want(norm_weight, "norm weight", torch.float32, (width,))
        moved = s * t * width * 4.0 * (2 if pending is not None else 1) + (t * width * 4.0 if pending is not None else 0)
        self._call("hyper", "tnx_hyper_step", _ptr(copies), _ptr(y), _ptr(mix), _ptr(out_w), _ptr(read), _ptr(norm_weight),
                   float(eps), _ptr(h32), _ptr(hcd), _code(hcd.dtype) if hcd is not None else 0, _ptr(total), s, t, width,
                   _stream(), work=(f"{s}x{t}x{width}", moved + t * width * 4.0, 0.0))

    def hyper_step(self, copies, pending, read, norm_weight, eps, dtype, want_f32, want_compute):
        """See `ReferenceOps.hyper_step`."""
        _, t, width = copies.shape
        same = dtype == torch.float32
        h32 = torch.empty(t, width, dtype=torch.float32, device=copies.device) if (want_f32 or (want_compute and same)) else None
        hcd = torch.empty(t, width, dtype=dtype, device=copies.device) if (want_compute and not same) else None
        self._hyper(copies, pending, read, norm_weight, eps, h32, hcd, None)
        return (h32 if want_f32 else None), ((h32 if same else hcd) if want_compute else None)

    def hyper_sum(self, copies, pending):
        """See `ReferenceOps.hyper_sum`."""
        _, t, width = copies.shape
        total = torch.empty(t, width, dtype=torch.float32, device=copies.device)
        self._hyper(copies, pending, None, None, 0.0, None, None, total)
        return total

    # ---------------------------------------------------------------- scores that are not the plain ones

    @staticmethod
    def _rows_apart(x, name, dtype, t, width):
        """A `[t, width]` tensor whose rows may lie apart (a slice of columns): its row distance in elements."""
        if (not x.is_cuda or x.dtype != dtype or x.dim() != 2 or tuple(x.shape) != (t, width)
                or (width > 1 and x.stride(1) != 1)):
            raise ValueError(f"{name} must be {dtype} [{t}, {width}] with dense rows on the GPU, got {tuple(x.shape)} {x.dtype}")
        return x.stride(0) if t > 1 else max(x.stride(0), width)

    def attention_scored(self, q, num_heads, num_kv_heads, head_size, ctx, view, k_pages, v_pages, window=None,
                         chunk=None, softcap=None, distance_bias=None, gate=None, value_size=None, out=None,
                         out_scale=1.0, gate_per_head=False):
        """See `ReferenceOps.attention_scored`."""
        t = ctx.num_tokens
        value_size = head_size if value_size is None else value_size
        _want(q, "q", self.dtype, (t, num_heads * head_size))
        num_pages = self._check_pages(k_pages, v_pages, num_kv_heads, head_size, view.page_size)
        _want(view.block_table, "block table", torch.int32, (ctx.num_requests, view.width))
        if ctx.max_total > view.width * view.page_size:
            raise ValueError("a request is longer than its block table")
        if out is None:
            out = torch.empty_like(q)
        out_ld = self._rows_apart(out, "the result", self.dtype, t, num_heads * head_size)
        gate_head = 1 if gate_per_head else value_size
        gate_ld = self._rows_apart(gate, "the gate", torch.float32, t, num_heads * gate_head) if gate is not None else 0
        far = 0
        if distance_bias is not None:
            _want(distance_bias, "bias by distance", torch.float32)
            if distance_bias.dim() != 2 or distance_bias.shape[0] != num_heads:
                raise ValueError(f"the bias by distance is [heads, distances], got {tuple(distance_bias.shape)}")
            far = distance_bias.shape[1] - 1
        pad = self._page_pad(k_pages, num_kv_heads, head_size, view.page_size)
        work = (self._scored_work(ctx, num_heads, num_kv_heads, head_size, window, chunk, q.element_size())
                if debug.timer() is not None else None)
        if self.dtype == torch.bfloat16 and not self.force_plain_attention and "tile_run" in ctx.plan:
            # on the matrix unit: the runs of several tokens by tiles of queries (through LDS where the pages are a
            # power of two of keys), the runs of one token by key/value head
            tiles, single = ctx.plan["tile_run"], ctx.plan["decode_runs"]
            staged = tiles.numel() > 0 and view.page_size & (view.page_size - 1) == 0
            if staged:
                sets = 1 if (int(self.prefill_direct) or self._prefill_sets(ctx, num_heads, int(window or chunk or 0))) == 2 else 2
                self._call("attention", "tnx_attention_prefill_scored", _ptr(q), _ptr(k_pages), _ptr(v_pages),
                           _ptr(ctx.run_start), _ptr(ctx.cached_lens), _ptr(view.block_table), view.width, view.page_size,
                           num_pages, _ptr(tiles), _ptr(ctx.plan["tile_start"]), tiles.numel(), QUERY_TILE, _ptr(out), out_ld,
                           float(out_scale), _ptr(gate), gate_ld, _ptr(distance_bias), far, float(softcap or 0.0),
                           int(window or 0), int(chunk or 0), num_heads, num_kv_heads, head_size, value_size, sets, pad,
                           gate_head, _stream(), work=work)
            if not staged or single.numel():
                splits, partial = self._scored_splits(ctx, single.numel(), num_heads, num_kv_heads, head_size, window, chunk)
                self._call("scored", "tnx_attention_scored_mfma", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(ctx.run_start),
                           _ptr(ctx.cached_lens), _ptr(view.block_table), view.width, view.page_size, num_pages, _ptr(tiles),
                           _ptr(ctx.plan["tile_start"]), 0 if staged else tiles.numel(), QUERY_TILE, _ptr(single),
                           single.numel(), _ptr(out), out_ld, float(out_scale), _ptr(gate), gate_ld, _ptr(distance_bias), far,
                           float(softcap or 0.0), int(window or 0), int(chunk or 0), num_heads, num_kv_heads, head_size,
                           value_size, pad, splits, _ptr(partial), gate_head, _stream(), work=None if staged else work)
            return out
        self._call("scored", "tnx_attention_scored", _ptr(q), _code(self.dtype), _ptr(k_pages), _ptr(v_pages),
                   _ptr(ctx.positions), _ptr(ctx.token_request), _ptr(view.block_table), view.width, view.page_size,
                   num_pages, _ptr(out), out_ld, float(out_scale), _ptr(gate), gate_ld, _ptr(distance_bias), far,
                   float(softcap or 0.0), int(window or 0), int(chunk or 0), t, num_heads, num_kv_heads, head_size,
                   value_size, pad, gate_head, _stream(), work=work)
        return out

    scored_decode_splits = None       # tests set it: the blocks that share a decoded token's keys

    def _scored_splits(self, ctx, singles, num_heads, num_kv_heads, head_size, window, chunk):
        """(splits, workspace): how many blocks share the keys of a decoded token's (request, key/value head). A
        token's time is the latency of a wave's chain of loads (measured: a wave lives some 9 us whether it takes
        one tile or two, and a compute unit holds one or two such blocks), so the tiles the longest request can see
        are spread until a wave has one (eight waves a block), as long as every block finds a compute unit free. The result
        does not depend on the number beyond rounding: a recorded step keeps the one it was recorded with."""
        if not singles:
            return 1, None
        longest = ctx.length_bound if ctx.length_bound is not None else ctx.plan_host.get("longest_decode", 0)
        seen = min(longest, (window or longest) + 63, (chunk or longest) + 63)
        tiles = seen // 64 + 1
        splits = self.scored_decode_splits or max(1, min(8, -(-tiles // 8), self.compute_units // max(1, singles * num_kv_heads * -(-(num_heads // num_kv_heads) // 16))))
        if splits == 1:
            return 1, None
        return splits, torch.empty(singles * num_heads * splits * (head_size + 4), dtype=torch.float32, device=self.device)

    @staticmethod
    def _scored_work(ctx, num_heads, num_kv_heads, head_size, window, chunk, item):
        """For a kernel timer: the keys the step's queries see (a query at position p sees p + 1, cut by the window
        and by the chunk it lies in), the bytes of keys and values its runs must read once, the flops."""
        lens, cached = ctx.run_lens_host.astype(np.int64), ctx.cached_lens_host.astype(np.int64)
        pairs, span = 0.0, 0.0
        for n, have in zip(lens, cached):
            p = np.arange(have, have + n, dtype=np.int64)
            seen = p + 1
            if window:
                seen = np.minimum(seen, window)
            if chunk:
                seen = np.minimum(seen, p % chunk + 1)
            pairs += float(seen.sum())
            first = int((p - seen + 1).min()) if n else 0
            span += float(have + n - first)
        return (f"{len(lens)} runs {int(lens.sum())} tokens", span * 2 * num_kv_heads * head_size * item,
                4.0 * num_heads * head_size * pairs)

    # ---------------------------------------------------------------- recurrences

    def min_gru(self, proj, inner, ctx, carried, out=None, out_scale=1.0):
        """See `ReferenceOps.min_gru`."""
        t = ctx.num_tokens
        _want(proj, "projections", torch.float32, (t, 3 * inner))
        _want(carried, "carried state", torch.float32, (carried.shape[0], 2, inner))
        if out is None:
            out = torch.empty(t, inner, dtype=self.dtype, device=proj.device)
        out_ld = self._rows_apart(out, "the result", self.dtype, t, inner)
        self._call("recurrent", "tnx_min_gru", _ptr(proj), 3 * inner, inner, _ptr(ctx.positions), _ptr(ctx.run_start),
                   _ptr(ctx.slots), _ptr(carried), _ptr(out), out_ld, _code(self.dtype), float(out_scale), t,
                   ctx.num_requests, _stream(), work=(f"{t}x{inner}", t * inner * (12.0 + out.element_size()), 0.0))
        return out

    def channel_conv(self, x, weight, bias, ctx, state):
        """See `ReferenceOps.channel_conv`."""
        t = ctx.num_tokens
        channels, taps = weight.shape
        ld = self._rows_apart(x, "the convolution's input", torch.float32, t, channels)
        _want(weight, "convolution weights", torch.float32, (channels, taps))
        _want(bias, "convolution bias", torch.float32, (channels,))
        if taps > 1:
            _want(state, "convolution state", torch.float32, (state.shape[0], taps, channels))
        out = torch.empty(t, channels, dtype=torch.float32, device=x.device)
        cd = torch.empty(t, channels, dtype=self.dtype, device=x.device) if self.dtype != torch.float32 else None
        self._call("recurrent", "tnx_channel_conv", _ptr(x), ld, _ptr(self._taps_first(weight)), _ptr(bias),
                   _ptr(state) if taps > 1 else None, taps, _ptr(ctx.positions), _ptr(ctx.token_request),
                   _ptr(ctx.run_start), _ptr(ctx.slots), _ptr(out), _ptr(cd), _code(self.dtype), t, channels,
                   ctx.num_requests, _stream(), work=(f"{t}x{channels}", t * channels * 10.0, 0.0))
        return out, (cd if cd is not None else out)

    def gated_linear_recurrence(self, gates, gate_bias, u, y, rate, ctx, carried, out=None, out_scale=1.0):
        """See `ReferenceOps.gated_linear_recurrence`."""
        t = ctx.num_tokens
        _want(gates, "gates", torch.float32)
        if gates.dim() != 3 or gates.shape[0] != t or gates.shape[2] % 2:
            raise ValueError(f"gates must be [{t}, blocks, 2 w], got {tuple(gates.shape)}")
        blocks, w = gates.shape[1], gates.shape[2] // 2
        channels = blocks * w
        _want(gate_bias, "gate biases", torch.float32, (blocks, 2 * w))
        _want(u, "u", torch.float32, (t, channels))
        _want(rate, "rate", torch.float32, (channels,))
        _want(carried, "carried state", torch.float32, (carried.shape[0], 2, channels))
        y_ld = self._rows_apart(y, "y", torch.float32, t, channels)
        if out is None:
            out = torch.empty(t, channels, dtype=self.dtype, device=u.device)
        out_ld = self._rows_apart(out, "the result", self.dtype, t, channels)
        self._call("recurrent", "tnx_gated_linear_recurrence", _ptr(gates), _ptr(gate_bias), _ptr(u), _ptr(y), y_ld,
                   _ptr(rate), _ptr(ctx.positions), _ptr(ctx.run_start), _ptr(ctx.slots), _ptr(carried), _ptr(out), out_ld,
                   _code(self.dtype), float(out_scale), t, ctx.num_requests, blocks, w, _stream(),
                   work=(f"{t}x{channels}", t * channels * (16.0 + out.element_size()), 0.0))
        return out

    # ---------------------------------------------------------------- the matrix memory

    def matrix_memory(self, proj, num_heads, head_size, value_size, gate_cap, eps, norm_weight, ctx, memory, normalizer,
                      peak):
        """See `ReferenceOps.matrix_memory`."""
        t = ctx.num_tokens
        h, n, v = num_heads, head_size, value_size
        total = 2 * h * n + 2 * h * v + 2 * h
        _want(proj, "projections", torch.float32, (t, total))
        _want(norm_weight, "norm weight", torch.float32, (h * v,))
        slots = memory.shape[0]
        _want(memory, "memory", torch.float32, (slots, 2, h, v, n))
        _want(normalizer, "normalizer", torch.float32, (slots, 2, h, n))
        _want(peak, "peak", torch.float32, (slots, 2, h))
        raw = torch.empty(t, h * v, dtype=torch.float32, device=proj.device)
        # two factors and a floor a token, and the normalizer every run begins with
        gates = torch.empty(3 * t * h + ctx.num_requests * h * n, dtype=torch.float32, device=proj.device)
        out = torch.empty(t, h * v, dtype=self.dtype, device=proj.device)
        state = float(ctx.num_requests) * h * n * v * 8
        self._call("memory", "tnx_matrix_memory", _ptr(proj), total, _ptr(ctx.run_start), _ptr(ctx.cached_lens),
                   _ptr(ctx.slots), _ptr(memory), _ptr(normalizer), _ptr(peak), slots, _ptr(raw), _ptr(gates), _ptr(norm_weight),
                   float(eps), _ptr(out), _code(self.dtype), t, ctx.num_requests, h, n, v, float(gate_cap), _stream(),
                   work=(f"{t} tokens {ctx.num_requests} runs", state + t * total * 4.0, 4.0 * t * h * n * v))
        return out

    # ---------------------------------------------------------------- experts

    def route(self, z, top, score="sigmoid", renormalize=False, correction=None, scale=1.0):
        """See `ReferenceOps.route`."""
        _want(z, "router logits", torch.float32)
        t, experts = z.shape
        if score not in ("sigmoid", "softmax"):
            raise ValueError(f"unknown router score {score!r}")
        chosen = torch.empty(t, top, dtype=torch.int32, device=z.device)
        weights = torch.empty(t, top, dtype=torch.float32, device=z.device)
        if correction is not None:
            _want(correction, "the choice's correction", torch.float32, (experts,))
        self._call("experts", "tnx_route", _ptr(z), t, experts, top, int(score == "softmax"), int(bool(renormalize)),
                   _ptr(chosen), _ptr(weights), _ptr(correction), float(scale), _stream())
        return chosen, weights

    def gated_activation(self, gate_up, activation, row_weights=None, limit=None):
        """See `ReferenceOps.gated_activation`."""
        _want(gate_up, "gate and up", torch.float32)
        t, two_f = gate_up.shape
        if two_f % 2 or activation not in _GATE_ACT:
            raise ValueError(f"gated_activation: rows of {two_f}, activation {activation!r}")
        if row_weights is not None:
            _want(row_weights, "row weights", torch.float32, (t,))
        out = torch.empty(t, two_f // 2, dtype=self.dtype, device=gate_up.device)
        self._call("experts", "tnx_gated_activation", _ptr(gate_up), _ptr(out), _code(self.dtype), t, two_f // 2,
                   _GATE_ACT[activation], _ptr(row_weights), float(limit or 0.0), _stream(),
                   work=(f"{t}x{two_f // 2}", t * two_f * 4.0 + out.numel() * out.element_size(), 0.0))
        return out

    # A step of this many (token, choice) pairs an expert or more, bfloat16, that is not being recorded: the host
    # reads where each expert's pairs begin (one small copy that waits for the device) and every expert's two
    # products go to the vendor library over its own rows, as the many-rows products of the other parts do. Below
    # that, and in recorded steps, one launch of ours takes all experts and the host reads nothing. 0: never.
    expert_library_rows = 96
    expert_row_step = 128
    expert_plain_products = False      # tests set it: the kernel without the matrix unit in bfloat16 too

    def expert_mixture(self, h, chosen, weights, w_gate_up, w_down, activation, weight_on, residual=None, may_wait=False,
                       limit=None):
        """See `ReferenceOps.expert_mixture`. `may_wait`: the step is not being recorded, so the host may read
        what the device has made."""
        t, top = chosen.shape
        experts, two_f, width = w_gate_up.shape
        f = two_f // 2
        if activation not in _GATE_ACT or weight_on not in ("input", "output"):
            raise ValueError(f"expert_mixture: activation {activation!r}, weight_on {weight_on!r}")
        _want(h, "h", w_gate_up.dtype, (t, width))
        _want(chosen, "chosen experts", torch.int32)
        _want(weights, "weights", torch.float32, (t, top))
        _want(w_gate_up, "gate and up matrices")
        _want(w_down, "down matrices", w_gate_up.dtype, (experts, width, f))
        if residual is not None:
            _want(residual, "residual", torch.float32, (t, width))
        dev = h.device
        pairs = t * top
        out = torch.empty(t, width, dtype=torch.float32, device=dev)
        if (may_wait and self.expert_library_rows > 0 and pairs >= self.expert_library_rows * experts
                and self.dtype == torch.bfloat16 and h.dtype == torch.bfloat16 and width % 8 == 0 and f % 8 == 0
                and self.library_direct and not debug.tapping()):
            step = self.expert_row_step
            ints = torch.zeros(experts + 1 + 3 * pairs + step, dtype=torch.int32, device=dev)
            first, order = ints[:experts + 1], ints[experts + 1:experts + 1 + pairs]
            place, token = ints[experts + 1 + pairs:experts + 1 + 2 * pairs], ints[experts + 1 + 2 * pairs:]
            sorted_weights = torch.zeros(pairs + step, dtype=torch.float32, device=dev)      # zeros behind the pairs
            self._call("experts", "tnx_expert_order", _ptr(chosen), _ptr(weights), t, experts, top, _ptr(first), _ptr(order),
                       _ptr(place), _ptr(token), _ptr(sorted_weights), _stream())
            # An expert's products run over its rows filled up to a multiple of `expert_row_step`, so that the
            # library's choice for a size is made once and found again: the rows behind an expert's own are the next
            # expert's, whose products come later on the stream and write over what these left there.
            step = self.expert_row_step
            rows = self.gather_rows(h, token)                               # the pairs' tokens' rows, expert by expert
            begins = first.tolist()                                         # the host waits here for the device
            y = torch.empty(pairs + step, width, dtype=torch.float32, device=dev)
            scale = sorted_weights
            on_input = weight_on == "input"
            for e in range(experts):
                a, b = begins[e], begins[e + 1]
                if b == a:
                    continue
                b = a + -(-(b - a) // step) * step
                gu = self.linear(rows[a:b], w_gate_up[e], None, out_f32=True, f32_by_library=True)
                inner = self.gated_activation(gu, activation, scale[a:b] if on_input else None, limit=limit)
                self.linear(inner, w_down[e], None, out_f32=True, f32_by_library=True, into=y[a:b])
            self._call("experts", "tnx_expert_combine", _ptr(y), _ptr(place), None if on_input else _ptr(weights),
                       _ptr(residual), _ptr(out), t, top, width, _stream(),
                       work=(f"{t}x{top}x{width}", (pairs + 2.0 * t) * width * 4, 0.0))
            return out
        ints = torch.empty(experts + 1 + pairs, dtype=torch.int32, device=dev)
        inner = torch.empty(pairs, f, dtype=h.dtype, device=dev)
        rows = torch.empty(pairs, width, dtype=torch.float32, device=dev) if top > 1 else None
        item = h.element_size()
        used = min(experts, pairs)
        self._call("experts", "tnx_expert_mixture", _ptr(h), _ptr(chosen), _ptr(weights), _ptr(w_gate_up), _ptr(w_down),
                   _ptr(ints[:experts + 1]), _ptr(ints[experts + 1:]), _ptr(inner), _ptr(rows), _ptr(residual), _ptr(out),
                   _code(h.dtype), t, experts, top, width, f, _GATE_ACT[activation], int(weight_on == "input"),
                   int(bool(self.expert_plain_products)), float(limit or 0.0), _stream(),
                   work=(f"{t}x{top} of {experts}", used * 3.0 * f * width * item + t * width * (item + 8.0),
                         6.0 * t * top * f * width))
        return out

    # ---------------------------------------------------------------- output end

    def ban_tokens(self, logits, tokens):
        """In place: `logits[i, tokens[i]] = -inf` where `tokens[i] >= 0`."""
        _want(logits, "logits", torch.float32)
        _want(tokens, "tokens", torch.int32, (logits.shape[0],))
        self._call("sampling", "tnx_ban_tokens", _ptr(logits), _ptr(tokens), logits.shape[0], logits.shape[1],
                   _stream())
        return logits

    def ban_pairs(self, logits, rows, tokens):
        """In place: `logits[rows[i], tokens[i]] = -inf` for every pair."""
        _want(logits, "logits", torch.float32)
        _want(rows, "rows", torch.int32)
        _want(tokens, "tokens", torch.int32, (rows.numel(),))
        self._call("sampling", "tnx_ban_pairs", _ptr(logits), _ptr(rows), _ptr(tokens), rows.numel(), logits.shape[0],
                   logits.shape[1], _stream())
        return logits

    def argmax(self, logits):
        _want(logits, "logits", torch.float32)
        out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
        self._call("sampling", "tnx_argmax", _ptr(logits), _ptr(out), logits.shape[0], logits.shape[1], _stream())
        return out

    def sample(self, logits, temperature, top_k, top_p, seeds, counters, min_keep=None):
        """See `ReferenceOps.sample`."""
        _want(logits, "logits", torch.float32)
        m = logits.shape[0]
        _want(temperature, "temperature", torch.float32, (m,))
        _want(top_k, "top_k", torch.int32, (m,))
        _want(top_p, "top_p", torch.float32, (m,))
        _want(seeds, "seeds", torch.int64, (m,))
        _want(counters, "counters", torch.int64, (m,))
        if min_keep is not None:
            _want(min_keep, "min_keep", torch.int32, (m,))
        out = torch.empty(m, dtype=torch.int32, device=logits.device)
        self._call("sampling", "tnx_sample", _ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(seeds),
                   _ptr(counters), _ptr(min_keep), _ptr(out), m, logits.shape[1], _stream())
        return out

    def synchronize(self):
        torch.cuda.synchronize(self.device)
