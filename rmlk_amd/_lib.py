"""ctypes binding of librmlk_hip.so (the C ABI declared in include/rmlk_hip.h)."""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_int32, c_int64, c_size_t, c_void_p

MAX_RANK = 8

_HERE = os.path.dirname(os.path.abspath(__file__))


class LibraryNotBuilt(RuntimeError):
    """librmlk_hip.so is missing: build it with `make -C rmlk_amd/csrc` (or __graft_entry__.build)."""


class RmlkError(RuntimeError):
    """A C-ABI entry point returned a non-zero status."""

    def __init__(self, status: int, message: str, where: str):
        super().__init__(f"{where}: {message} (status {status})")
        self.status = status
        self.message = message


class Dims(ctypes.Structure):
    """struct rmlk_dims"""
    _fields_ = [("rank", c_int32), ("v", c_int64 * MAX_RANK)]

    @staticmethod
    def of(values) -> "Dims":
        values = [int(v) for v in values]
        if len(values) > MAX_RANK:
            raise RmlkError(-1, "rank outside 1..8", "rmlk_dims")
        d = Dims()
        d.rank = len(values)
        for i, v in enumerate(values):
            d.v[i] = v
        return d


class RowStream(ctypes.Structure):
    """struct rmlk_row_stream"""
    _fields_ = [("shape", Dims), ("x_stride", Dims), ("x", c_void_p), ("cos", c_void_p),
                ("sin", c_void_p), ("cos_stride", Dims), ("sin_stride", Dims), ("out", c_void_p),
                ("idx", c_void_p), ("tuple_size", c_int32), ("data_shape", Dims),
                ("partials", c_int32), ("partial_stride", c_int64)]


class DeviceInfo(ctypes.Structure):
    """struct rmlk_device_info"""
    _fields_ = [("name", ctypes.c_char * 128), ("arch", ctypes.c_char * 64),
                ("compute_units", c_int32), ("wavefront_size", c_int32),
                ("lds_bytes_per_block", c_int32), ("clock_khz", c_int32),
                ("total_mem_bytes", c_int64)]


def library_path() -> str:
    """In-tree build output, or the file RMLK_HIP_LIBRARY names."""
    return os.environ.get("RMLK_HIP_LIBRARY") or os.path.join(_HERE, "lib", "librmlk_hip.so")


# name -> (restype, argtypes); every symbol include/rmlk_hip.h declares
_PD = POINTER(Dims)
SIGNATURES = {
    "rmlk_hip_binary": (c_int32, [c_void_p, c_int32, c_int32, c_int32, _PD, _PD, _PD, c_void_p,
                                  c_void_p, c_void_p]),
    "rmlk_hip_where": (c_int32, [c_void_p, c_int32, _PD, _PD, _PD, _PD, c_void_p, c_void_p,
                                 c_void_p, c_void_p]),
    "rmlk_hip_unary": (c_int32, [c_void_p, c_int32, c_int32, c_int64, c_void_p, c_void_p]),
    "rmlk_hip_cast": (c_int32, [c_void_p, c_int32, c_int32, c_int64, c_void_p, c_void_p]),
    "rmlk_hip_reduce_mean": (c_int32, [c_void_p, c_int32, _PD, POINTER(c_int64), c_int32, c_void_p,
                                       c_void_p]),
    "rmlk_hip_softmax": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_void_p,
                                   c_void_p]),
    "rmlk_hip_matmul": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_void_p,
                                  c_int64, c_int64, c_int32, c_void_p, c_int64, c_int64, c_int32,
                                  c_void_p, c_int64, c_int64, c_void_p, c_size_t]),
    "rmlk_hip_matmul_noalloc": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_void_p,
                                          c_int64, c_int64, c_int32, c_void_p, c_int64, c_int64, c_int32,
                                          c_void_p, c_int64, c_int64]),
    "rmlk_hip_matmul_workspace_size": (c_size_t, [c_int32, c_int64, c_int64, c_int64, c_int64]),
    "rmlk_hip_matmul_describe": (c_int32, [c_int32, c_int64, c_int64, c_int64, c_int64, c_char_p,
                                           c_int32]),
    "rmlk_hip_transpose": (c_int32, [c_void_p, c_int32, _PD, POINTER(c_int64), c_void_p,
                                     c_void_p]),
    "rmlk_hip_expand": (c_int32, [c_void_p, c_int32, _PD, _PD, c_void_p, c_void_p]),
    "rmlk_hip_slice": (c_int32, [c_void_p, c_int32, _PD, _PD, _PD, _PD, c_void_p, c_void_p]),
    "rmlk_hip_concat": (c_int32, [c_void_p, c_int32, _PD, _PD, c_int32, c_int64, c_void_p,
                                  c_void_p]),
    "rmlk_hip_gather": (c_int32, [c_void_p, c_int32, c_int32, _PD, c_int32, c_int64, c_void_p,
                                  c_void_p, c_void_p, c_void_p]),
    "rmlk_hip_concat_many": (c_int32, [c_void_p, c_int32, c_int32, c_void_p, c_void_p, _PD, c_int32,
                                       c_void_p]),
    "rmlk_hip_scatter_nd_copy": (c_int32, [c_void_p, c_int32, _PD, c_int64, c_int32, c_void_p, c_void_p,
                                           c_void_p, c_void_p, c_void_p]),
    "rmlk_hip_scatter_nd": (c_int32, [c_void_p, c_int32, c_int32, _PD, c_int64, c_int32, c_void_p,
                                      c_void_p, c_void_p, c_void_p]),
    "rmlk_hip_trilu": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int32, c_int64,
                                 c_void_p, c_void_p]),
    "rmlk_hip_rmsnorm": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_void_p, c_void_p,
                                   ctypes.c_float, c_int32, c_void_p]),
    "rmlk_hip_add_rmsnorm": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_void_p, c_void_p,
                                       c_void_p, ctypes.c_float, c_int32, c_void_p, c_void_p]),
    "rmlk_hip_scale_mask_softmax": (c_int32, [c_void_p, c_int32, _PD, _PD, c_int32, ctypes.c_float,
                                              c_void_p, c_void_p, c_void_p]),
    "rmlk_hip_swiglu": (c_int32, [c_void_p, c_int32, c_int64, c_void_p, c_void_p, c_void_p]),
    "rmlk_hip_gemv_partials_workspace_size": (c_size_t, [c_int32, c_int64, c_int64]),
    "rmlk_hip_gemv_partials": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_void_p, c_void_p,
                                         c_int64, c_void_p, c_size_t, POINTER(c_int32)]),
    "rmlk_hip_splitk_swiglu": (c_int32, [c_void_p, c_int32, c_int64, c_void_p, c_int32, c_int64,
                                         c_int64, c_int64, c_void_p]),
    "rmlk_hip_matmul_partials_workspace_size": (c_size_t, [c_int32, c_int64, c_int64, c_int64]),
    "rmlk_hip_matmul_partials": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_void_p,
                                           c_int64, c_int32, c_void_p, c_int64, c_int32, c_void_p, c_size_t,
                                           POINTER(c_int32)]),
    "rmlk_hip_splitk_add_rmsnorm": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_void_p, c_int32,
                                              c_int64, c_void_p, c_void_p, ctypes.c_float, c_int32,
                                              c_void_p, c_void_p]),
    "rmlk_hip_bf16x3_pieces_size": (c_size_t, [c_int64, c_int64]),
    "rmlk_hip_bf16x3_split": (c_int32, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_void_p]),
    "rmlk_hip_bf16x3_splits": (c_int32, [c_int64, c_int64, c_int64]),
    "rmlk_hip_matmul_bf16x3": (c_int32, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int64,
                                         c_int32, c_void_p, c_int64, c_int64]),
    "rmlk_hip_rmsnorm_pieces": (c_int32, [c_void_p, c_int64, c_int64, c_void_p, c_int32, c_int64, c_void_p, c_void_p,
                                          ctypes.c_float, c_int32, c_void_p, c_void_p, c_void_p]),
    "rmlk_hip_matmul_bf16x3_grouped": (c_int32, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_int32,
                                                 POINTER(c_int64), POINTER(c_void_p)]),
    "rmlk_hip_matmul_bf16x3_swiglu": (c_int32, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                                c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p]),
    "rmlk_hip_store_weights": (c_int32, [c_void_p, c_int32, c_int64, c_void_p, c_void_p]),
    "rmlk_hip_weights_fit": (c_int32, [c_void_p, c_int32, c_int64, c_void_p, c_void_p]),
    "rmlk_hip_gemv_kmajor": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_void_p, c_int32, c_void_p,
                                       c_int64, c_void_p]),
    "rmlk_hip_gemv_kmajor_swiglu": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_void_p, c_int32,
                                              c_void_p, c_int64, c_int64, c_int64, c_void_p]),
    "rmlk_hip_gemv_kmajor_add": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_void_p, c_int32, c_void_p,
                                           c_int64, c_void_p, c_void_p]),
    "rmlk_hip_gemv_kmajor_normed": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_void_p, c_void_p,
                                              ctypes.c_float, c_int32, c_int32, c_void_p, c_int64,
                                              c_void_p]),
    "rmlk_hip_gemv_kmajor_swiglu_normed": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_void_p, c_void_p,
                                                     ctypes.c_float, c_int32, c_int32, c_void_p, c_int64,
                                                     c_int64, c_int64, c_void_p]),
    "rmlk_hip_attention": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_int64,
                                     c_int64, c_void_p, c_void_p, c_void_p, c_void_p, _PD, c_int32,
                                     ctypes.c_float, c_int32, c_void_p]),
    "rmlk_hip_attention_workspace_size": (c_size_t, [c_int32, c_int64, c_int64, c_int64, c_int64, c_int64,
                                                     c_int64, _PD]),
    "rmlk_hip_attention_ws": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_int64,
                                        c_int64, c_void_p, c_void_p, c_void_p, c_void_p, _PD, c_int32,
                                        ctypes.c_float, c_int32, c_void_p, c_size_t, c_void_p]),
    "rmlk_hip_attention_map_size": (c_size_t, [c_int32, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, _PD]),
    "rmlk_hip_attention_map": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_int64,
                                         c_int64, c_void_p, _PD, c_void_p, c_size_t]),
    "rmlk_hip_attention_mapped": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_int64,
                                            c_int64, c_void_p, c_void_p, c_void_p, c_void_p, _PD, c_int32,
                                            ctypes.c_float, c_int32, c_void_p, c_size_t, c_void_p]),
    "rmlk_hip_attention_mapped_pieces": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_int64,
                                                   c_int64, c_void_p, c_void_p, c_void_p, c_void_p, _PD, c_int32,
                                                   ctypes.c_float, c_void_p, c_size_t, c_void_p, c_void_p]),
    "rmlk_hip_attention_ws_pieces": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_int64,
                                               c_int64, c_void_p, c_void_p, c_void_p, c_void_p, _PD, c_int32,
                                               ctypes.c_float, c_void_p, c_size_t, c_void_p, c_void_p]),
    "rmlk_hip_attention_few_rows_workspace_size": (c_size_t, [c_int32, c_int64, c_int64, c_int64, c_int64,
                                                              c_int64, c_int64]),
    "rmlk_hip_attention_few_rows": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64,
                                              c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                                              _PD, c_int32, ctypes.c_float, c_int32, c_void_p, c_size_t,
                                              c_void_p]),
    "rmlk_hip_attention_few_rows_one_launch": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64,
                                                         c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                                         c_void_p, c_void_p, _PD, c_int32, ctypes.c_float,
                                                         c_int32, c_void_p, c_size_t, c_void_p, c_void_p]),
    "rmlk_hip_matmul_grouped_workspace_size": (c_size_t, [c_int32, c_int64, c_int64, c_int32,
                                                          POINTER(c_int64)]),
    "rmlk_hip_matmul_grouped": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_void_p, c_int64,
                                          c_int32, c_void_p, c_int64, c_int32, c_int32, POINTER(c_int64),
                                          POINTER(c_void_p), c_void_p, c_size_t]),
    "rmlk_hip_matmul_swiglu": (c_int32, [c_void_p, c_int32, c_int64, c_int64, c_int64, c_void_p,
                                         c_int64, c_int32, c_void_p, c_int64, c_int32, c_int64, c_int64,
                                         c_void_p, c_int64]),
    "rmlk_hip_rotary": (c_int32, [c_void_p, c_int32, _PD, _PD, _PD, _PD, c_void_p, c_void_p,
                                  c_void_p, c_void_p]),
    "rmlk_hip_head_rows": (c_int32, [c_void_p, c_int32, c_int32, POINTER(RowStream), c_void_p]),
    "rmlk_hip_gemv_kmajor_head_rows": (c_int32, [c_void_p, c_int32, c_int64, c_void_p, c_void_p, ctypes.c_float,
                                                 c_int32, c_int32, c_void_p, c_int64, c_int32, c_void_p,
                                                 c_void_p, c_void_p]),
    "rmlk_hip_batch_begin": (c_int32, [c_void_p]),
    "rmlk_hip_batch_flush": (c_int32, [c_void_p]),
    "rmlk_hip_batch_end": (c_int32, [c_void_p]),
    "rmlk_hip_batch_collects": (c_int32, [_PD, c_int32, _PD]),
    "rmlk_hip_fill": (c_int32, [c_void_p, c_int32, c_int64, c_void_p, c_void_p]),
    "rmlk_hip_range": (c_int32, [c_void_p, c_int32, c_int64, c_void_p, c_void_p, c_void_p]),
    "rmlk_hip_stream_yardstick": (c_int32, [c_void_p, c_int32, c_size_t, c_void_p, c_void_p, c_void_p]),
    "rmlk_hip_issue_yardstick": (c_int32, [c_void_p, c_int32, c_int32, c_int32, c_int32, c_void_p]),
    "rmlk_hip_write_small": (c_int32, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "rmlk_hip_malloc": (c_int32, [POINTER(c_void_p), c_size_t]),
    "rmlk_hip_free": (c_int32, [c_void_p]),
    "rmlk_hip_memcpy_htod": (c_int32, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "rmlk_hip_memcpy_dtoh": (c_int32, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "rmlk_hip_memcpy_dtod": (c_int32, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "rmlk_hip_memcpy_dtod_many": (c_int32, [c_void_p, c_int32, POINTER(c_void_p), POINTER(c_void_p),
                                            POINTER(c_size_t)]),
    "rmlk_hip_memset": (c_int32, [c_void_p, c_void_p, c_int32, c_size_t]),
    "rmlk_hip_stream_sync": (c_int32, [c_void_p]),
    "rmlk_hip_device_info": (c_int32, [c_int32, POINTER(DeviceInfo)]),
    "rmlk_hip_status_string": (c_char_p, [c_int32]),
    "rmlk_hip_version": (c_char_p, []),
    # include/rmlk_runtime.h
    "rmlk_last_error": (c_char_p, []),
    "rmlk_graph_create": (c_int32, [POINTER(c_void_p)]),
    "rmlk_graph_destroy": (None, [c_void_p]),
    "rmlk_graph_input": (c_int32, [c_void_p, c_char_p, c_int32, POINTER(c_int64), c_int32]),
    "rmlk_graph_constant": (c_int32, [c_void_p, c_char_p, c_int32, POINTER(c_int64), c_int32,
                                      c_void_p]),
    "rmlk_graph_op": (c_int32, [c_void_p, c_char_p, POINTER(c_char_p), c_int32, POINTER(c_char_p),
                                c_int32]),
    "rmlk_graph_attr_int": (c_int32, [c_void_p, c_int32, c_char_p, c_int64]),
    "rmlk_graph_attr_float": (c_int32, [c_void_p, c_int32, c_char_p, ctypes.c_float]),
    "rmlk_graph_attr_ints": (c_int32, [c_void_p, c_int32, c_char_p, POINTER(c_int64), c_int32]),
    "rmlk_graph_attr_floats": (c_int32, [c_void_p, c_int32, c_char_p, POINTER(ctypes.c_float),
                                         c_int32]),
    "rmlk_graph_attr_string": (c_int32, [c_void_p, c_int32, c_char_p, c_char_p]),
    "rmlk_graph_attr_tensor": (c_int32, [c_void_p, c_int32, c_char_p, c_int32, POINTER(c_int64),
                                         c_int32, c_void_p]),
    "rmlk_graph_output": (c_int32, [c_void_p, c_char_p]),
    "rmlk_graph_load_onnx": (c_int32, [c_void_p, c_size_t, c_char_p, POINTER(c_void_p)]),
    "rmlk_graph_load_onnx_file": (c_int32, [c_char_p, POINTER(c_void_p)]),
    "rmlk_graph_describe": (c_int64, [c_void_p, c_char_p, c_int64]),
    "rmlk_session_create": (c_int32, [c_void_p, c_int32, POINTER(c_void_p)]),
    "rmlk_session_create_ex": (c_int32, [c_void_p, c_int32, ctypes.c_uint32, POINTER(c_void_p)]),
    "rmlk_session_fused_nodes": (c_int32, [c_void_p]),
    "rmlk_session_weights_16bit": (c_int32, [c_void_p]),
    "rmlk_session_products_bf16_pieces": (c_int32, [c_void_p]),
    "rmlk_session_destroy": (None, [c_void_p]),
    "rmlk_session_set_input": (c_int32, [c_void_p, c_char_p, c_int32, POINTER(c_int64), c_int32,
                                         c_void_p]),
    "rmlk_session_bind_input": (c_int32, [c_void_p, c_char_p, c_int32, POINTER(c_int64), c_int32,
                                          c_void_p, c_int32]),
    "rmlk_session_feed_output": (c_int32, [c_void_p, c_char_p, c_char_p]),
    "rmlk_session_run": (c_int32, [c_void_p]),
    "rmlk_session_output_info": (c_int32, [c_void_p, c_char_p, POINTER(c_int32), POINTER(c_int64),
                                           POINTER(c_int32), POINTER(c_void_p)]),
    "rmlk_session_read_output": (c_int32, [c_void_p, c_char_p, c_void_p, c_size_t]),
    "rmlk_session_capture": (c_int32, [c_void_p]),
    "rmlk_session_replay": (c_int32, [c_void_p]),
    "rmlk_session_replay_enqueue": (c_int32, [c_void_p]),
    "rmlk_session_check": (c_int32, [c_void_p]),
    "rmlk_session_sync": (c_int32, [c_void_p]),
    "rmlk_session_stream": (c_void_p, [c_void_p]),
    "rmlk_session_set_profiling": (c_int32, [c_void_p, c_int32]),
    "rmlk_session_node_count": (c_int32, [c_void_p]),
    "rmlk_session_node_info": (c_int32, [c_void_p, c_int32, POINTER(c_char_p),
                                         POINTER(ctypes.c_double), POINTER(ctypes.c_double),
                                         POINTER(ctypes.c_double)]),
    "rmlk_session_memory_stats": (c_int32, [c_void_p, POINTER(c_int64), POINTER(c_int64),
                                            POINTER(c_int64)]),
}

_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library; raises LibraryNotBuilt when the HIP extension has not been built."""
    global _lib
    if _lib is None:
        path = library_path()
        if not os.path.exists(path):
            raise LibraryNotBuilt(f"{path} not found; there is no CPU fallback")
        handle = ctypes.CDLL(path)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(status: int, where: str) -> None:
    if status != 0:
        msg = lib().rmlk_hip_status_string(status)
        raise RmlkError(status, msg.decode() if msg else "unknown", where)
