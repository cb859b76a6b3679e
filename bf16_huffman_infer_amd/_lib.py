"""ctypes binding of libbhi_hip.so (the C ABI declared in include/bhi.h).

The library is built in-tree by ``python -m bf16_huffman_infer_amd.csrc.build``.  There
is no fallback: if it is missing every op of this package raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libbhi_hip.so")

_vp, _i64, _i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int


class GemvMember(ctypes.Structure):
    """``bhi_gemv_member`` of include/bhi.h: one weight of a grouped GEMV launch."""
    _fields_ = [("A_rem", _vp), ("A_exp", _vp), ("exp_words", _i64), ("Y", _vp), ("offsets", _vp),
                ("table", _vp), ("table_bytes", _i64), ("header", _vp), ("bias", _vp), ("M", ctypes.c_int32),
                ("reserved", ctypes.c_int32), ("residual", _vp)]


_grouped = (_i32, [ctypes.POINTER(GemvMember), _i32, _vp, _i32, _i32, _i32, _vp])

_SIGNATURES = {
    "bhi_constants": (_i32, [ctypes.POINTER(ctypes.c_int32), _i32]),
    "bhi_chunks_per_group": (_i32, [_i32, _i32, _i32]),
    "bhi_last_error_string": (ctypes.c_char_p, []),
    "bhi_stream_read": (_i64, [_vp, _i64, _i32, _i32, _vp, _vp]),
    "bhi_decode_attention": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, ctypes.c_float, ctypes.c_float, _vp]),
    "bhi_gemv_bf16_huffman": (_i32, [_vp, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp,
                                     _i32, _i32, _i32, _i32, _vp]),
    "bhi_huffman_decode": (_i32, [_vp, _vp, _i64, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp,
                                  _i32, _i32, _i32, _vp]),
    "bhi_huffman_encode": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i64, _vp]),
    "bhi_encode_capacity": (_i64, [_i32]),
    "bhi_gemv_bf16_ans": (_i32, [_vp, _vp, _i64, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp]),
    "bhi_ans_decode": (_i32, [_vp, _vp, _i64, _vp, _vp, _vp, _i32, _i32, _i32, _vp]),
    "bhi_ans_encode": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i64, _vp]),
    "bhi_ans_encode_capacity": (_i64, [_i32]),
    "bhi_gemv_bf16_nibble": (_i32, [_vp, _vp, _i64, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp]),
    "bhi_nibble_decode": (_i32, [_vp, _vp, _i64, _vp, _vp, _vp, _i32, _i32, _i32, _vp]),
    "bhi_nibble_encode": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i64, _vp]),
    "bhi_nibble_encode_capacity": (_i64, [_i32]),
    "bhi_gemv_bf16_huffman_grouped": _grouped,
    "bhi_gemv_bf16_ans_grouped": _grouped,
    "bhi_gemv_bf16_nibble_grouped": _grouped,
    "bhi_gemv_bf16_huffman_grouped_x": (_i32, [ctypes.POINTER(GemvMember), _i32, _vp, _i32, _i32, _i32, _i32, _vp,
                                               ctypes.c_float, _vp]),
    "bhi_gemv_bf16_ans_grouped_x": (_i32, [ctypes.POINTER(GemvMember), _i32, _vp, _i32, _i32, _i32, _i32, _vp,
                                           ctypes.c_float, _vp]),
    "bhi_rms_norm": (_i32, [_vp, _vp, _vp, _i32, _i32, ctypes.c_float, _vp]),
    "bhi_silu_mul": (_i32, [_vp, _vp, _vp, _i64, _vp]),
    "bhi_gemm_bf16_huffman": (_i32, [ctypes.POINTER(GemvMember), _vp, _i32, _i32, _i32, _vp, _i64, _vp]),
    "bhi_gemm_bf16_ans": (_i32, [ctypes.POINTER(GemvMember), _vp, _i32, _i32, _i32, _vp, _i64, _vp]),
    "bhi_gemm_bf16_huffman_grouped": (_i32, [ctypes.POINTER(GemvMember), _i32, _vp, _i32, _i32, _i32, _vp]),
    "bhi_gemm_bf16_ans_grouped": (_i32, [ctypes.POINTER(GemvMember), _i32, _vp, _i32, _i32, _i32, _vp]),
    "bhi_gemm_workspace_bytes": (_i64, [_i32, _i32, _i32, _i32]),
    "bhi_gemm_bf16_huffman_static": (_i32, [ctypes.POINTER(GemvMember), _vp, _i32, _i32, _i32, _vp]),
    "bhi_gemm_static_workspace_bytes": (_i64, []),
    "bhi_device_init": (_i32, []),
    "bhi_gemm_workspace_reset": (_i32, [_vp, _i64, _vp]),
    "bhi_reference_huffman_decode": (_i32, [_vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _vp]),
    "bhi_reference_ans_decode": (_i32, [_vp, _vp, _i64, _vp, _vp, _vp, _i32, _i32, _i32, _vp]),
}

_CONST_NAMES = (
    "format_version", "lanes", "group_rows", "step_cols", "table_bits", "window_words",
    "header_bits", "max_batch", "ans_precision", "align_words", "tail_pad_words",
    "target_tasks", "max_task_steps", "member_bytes",
)

EXPORTS = tuple(_SIGNATURES)

_lib = None


def load() -> ctypes.CDLL:
    """Returns the loaded library; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP extension first "
                "(python -m bf16_huffman_infer_amd.csrc.build). There is no CPU fallback.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        buf = (ctypes.c_int32 * len(_CONST_NAMES))()
        if lib.bhi_constants(buf, len(_CONST_NAMES)) != len(_CONST_NAMES):
            raise RuntimeError("constant table of the library and of the binding differ: rebuild the library")
        if buf[_CONST_NAMES.index("member_bytes")] != ctypes.sizeof(GemvMember):
            raise RuntimeError("bhi_gemv_member of the library and of the binding differ: rebuild the library")
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().bhi_last_error_string().decode()
        raise RuntimeError(f"{what} failed (code {rc}): {msg}")


def constants() -> dict:
    lib = load()
    buf = (ctypes.c_int32 * len(_CONST_NAMES))()
    n = lib.bhi_constants(buf, len(_CONST_NAMES))
    assert n == len(_CONST_NAMES), "constant table of the library and of the binding differ"
    return dict(zip(_CONST_NAMES, buf))
