"""ctypes binding of libsubspec_hip.so (the C ABI declared in include/subspec_hip.h).

The library is built in-tree by ``python -m subspec_amd.build`` (or ``__graft_entry__.build()``).
There is no CPU fallback: if the library is missing, ``lib()`` raises.
"""
from __future__ import annotations

import ctypes as C
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libsubspec_hip.so")
HEADER = os.path.join(os.path.dirname(HERE), "include", "subspec_hip.h")

F32, F16, BF16 = 0, 1, 2
VERIFY_EXACT, VERIFY_LOSSY = 0, 1
GATE_ENTROPY, GATE_PROB = 0, 1
ENTROPY_GUARD, ENTROPY_ALWAYS = 0, 1
MAX_TREE_NODES = 512
TREE_VERIFY_STATIC_MAX_ROWS = 2048

_lib = None

_p, _i32, _i64, _f64, _sz = C.c_void_p, C.c_int32, C.c_int64, C.c_double, C.c_size_t


class DecoderLayerDims(C.Structure):
    """subspec_decoder_layer_dims"""
    _fields_ = [("dtype", C.c_int32), ("reserved", C.c_int32),
                ("n_rows", _i64), ("hidden", _i64), ("intermediate", _i64), ("n_q_heads", _i64), ("n_kv_heads", _i64),
                ("head_dim", _i64), ("kv_seq_stride", _i64), ("prefix_len", _i64), ("n_tree_slots", _i64),
                ("rms_eps", C.c_float), ("rope_theta", C.c_float), ("rope_inv_freq", C.c_void_p),
                ("prefix_len_dev", C.c_void_p), ("page_indices", C.c_void_p), ("n_pages", _i64), ("max_pages", _i64),
                ("page_len", _i64)]


class DecoderLayerWeights(C.Structure):
    """subspec_decoder_layer_weights"""
    _fields_ = [(n, _p) for n in ("input_norm", "post_norm", "qkv_wq", "qkv_sz", "qkv_bias", "o_wq", "o_sz",
                                  "gate_up_wq", "gate_up_sz", "down_wq", "down_sz")]


class DenseLayerWeights(C.Structure):
    """subspec_dense_layer_weights"""
    _fields_ = [(n, _p) for n in ("input_norm", "post_norm", "qkv_w", "qkv_bias", "o_w", "gate_up_w", "down_w")]


_SIGNATURES = {
    "subspec_abi_version": (C.c_int, []),
    "subspec_last_error": (C.c_char_p, []),
    "subspec_profile_enable": (C.c_int, [C.c_int]),
    "subspec_profile_count": (C.c_int, []),
    "subspec_profile_read_ms": (C.c_float, [C.c_int]),
    "subspec_tree_verify_workspace": (_sz, [_i64, _i64, _i64, C.c_int]),
    "subspec_tree_verify": (C.c_int, [_p, C.c_int, _i64, _i64, _i64, _p, _p, _i64, _i32, _i32, _i64,
                                      C.c_int, C.c_int, _f64, _i32, C.c_int, _p, _sz,
                                      _p, _p, _p, _p, _p, _p, _p]),
    "subspec_tree_verify_static": (C.c_int, [_p, C.c_int, _i64, _i64, _i64, _p, _p, _i64, _i32, _i32, _i64,
                                             C.c_int, C.c_int, _f64, _i32, C.c_int,
                                             _p, _p, _p, _p, _p, _p, _p]),
    "subspec_tree_verify_sample": (C.c_int, [_p, C.c_int, _i64, _i64, _i64, _p, _p, _i64, _i32, _i32, _i64,
                                             C.c_int, C.c_int, _f64, _i32, C.c_int, C.c_float, C.c_uint64, C.c_uint64,
                                             _p, _sz, _p, _p, _p, _p, _p, _p, _p]),
    "subspec_topk_expand_workspace": (_sz, [_i64, _i64, _i64, _i32]),
    "subspec_topk_expand": (C.c_int, [_p, _p, C.c_int, _i64, _i64, _i64, _i32, _p, _sz, _p, _p, _p, _p]),
    "subspec_tree_attention_workspace": (_sz, [_i64, _i64, _i64, _i64, _i64, _i64]),
    "subspec_tree_attention": (C.c_int, [_p, _p, _p, _p, C.c_int, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _p, _i64,
                                         C.c_float, _p, _sz, _p]),
    "subspec_tree_attention_paged": (C.c_int, [_p, _p, _p, _i64, _i64, _i64, _p, C.c_int, _i64, _i64, _i64, _i64, _i64, _i64, _p,
                                               C.c_float, _p, _sz, _p]),
    "subspec_kv_compact_paged": (C.c_int, [_p, _i64, _i64, _i64, _i64, _p, _i64, _i64, _p, _p, _i32, _i32, _p]),
    "subspec_softmax_temperature_workspace": (_sz, [_i64, _i64]),
    "subspec_softmax_temperature": (C.c_int, [_p, _p, C.c_int, _i64, _i64, C.c_float, _p, _sz, _p]),
    "subspec_temperature_warp": (C.c_int, [_p, _p, C.c_int, _i64, C.c_float, _p]),
    "subspec_int4_linear_workspace": (_sz, [_i64, _i64, _i64]),
    "subspec_int4_linear": (C.c_int, [_p, _p, _p, _p, _p, C.c_int, _i64, _i64, _i64, _i64, _p, _sz, _p]),
    "subspec_int4_gate_up_silu": (C.c_int, [_p, _p, _p, _p, _p, C.c_int, _i64, _i64, _i64, _p]),
    "subspec_dense_gate_up_silu": (C.c_int, [_p, _p, _p, _p, C.c_int, _i64, _i64, _i64, _p]),
    "subspec_int4_decoder_layer_workspace": (_sz, [C.POINTER(DecoderLayerDims)]),
    "subspec_int4_decoder_layer": (C.c_int, [C.POINTER(DecoderLayerDims), C.POINTER(DecoderLayerWeights), _p, _p, _p, _p,
                                             _p, _p, _p, _sz, _p]),
    "subspec_dense_linear_workspace": (_sz, [_i64, _i64, _i64]),
    "subspec_dense_linear": (C.c_int, [_p, _p, _p, _p, C.c_int, _i64, _i64, _i64, _p, _sz, _p]),
    "subspec_dense_decoder_layer": (C.c_int, [C.POINTER(DecoderLayerDims), C.POINTER(DenseLayerWeights), _p, _p, _p, _p,
                                              _p, _p, _p, _sz, _p]),
    "subspec_rms_norm": (C.c_int, [_p, _p, _p, C.c_int, _i64, _i64, C.c_float, _p]),
    "subspec_stream_copy_h2d": (C.c_int, [_p, _p, _sz, _p]),
    "subspec_kv_compact": (C.c_int, [_p, _p, _i64, _i64, _i64, _i64, _i64, _p, _p, _i32, _i32, _p]),
}


class SubspecHipError(RuntimeError):
    pass


def declared_symbols():
    """Names of all functions declared in include/subspec_hip.h."""
    with open(HEADER) as f:
        text = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    return sorted(set(re.findall(r"\b(subspec_[a-z0-9_]+)\s*\(", text)))


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise SubspecHipError(
                f"{LIB_PATH} not found: build it with `python -m subspec_amd.build` "
                "(hipcc, gfx950). There is no CPU fallback.")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = lib().subspec_last_error().decode("utf-8", "replace")
        kind = ValueError if code in (-1, -4) else SubspecHipError
        raise kind(f"{what}: {msg} (code {code})")
