"""ctypes binding of libmi_attn.so (declarations mirror include/mi_attn.h).

The library is loaded from the package directory only; there is no fallback:
if it has not been built (python -m tritonops_amd.build) loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi_attn.so")

MI_ATTN_ABI_VERSION = 8
MI_DECODE_STATIC_SCRATCH_BYTES = 32 << 20
MI_KV_BATCHED, MI_KV_PACKED, MI_KV_PAGED = 0, 1, 2
MI_ATTN_BLOCK = 64
MI_DENSE_FORM_AUTO, MI_DENSE_FORM_256_ROWS, MI_DENSE_FORM_128_ROWS = 0, 1, 2
MI_DTYPE_F32 = 2
MI_DTYPE_BF16 = 0
MI_DTYPE_F16 = 1

STATUS = {
    0: "MI_OK",
    -1: "MI_ERR_NULL_POINTER",
    -2: "MI_ERR_STRUCT_SIZE",
    -3: "MI_ERR_DTYPE",
    -4: "MI_ERR_HEAD_DIM",
    -5: "MI_ERR_GQA",
    -6: "MI_ERR_SHAPE",
    -7: "MI_ERR_STRIDE",
    -8: "MI_ERR_ALIGNMENT",
    -9: "MI_ERR_SCALE",
    -10: "MI_ERR_WORKSPACE",
    -11: "MI_ERR_SPARSE_LAYOUT",
    -12: "MI_ERR_LAUNCH",
    -13: "MI_ERR_NO_DEVICE",
}

_i32, _i64, _u32, _f32, _vp, _sz = C.c_int32, C.c_int64, C.c_uint32, C.c_float, C.c_void_p, C.c_size_t


class AttnFwdArgs(C.Structure):
    _fields_ = [
        ("struct_size", _u32), ("dtype", _i32),
        ("q", _vp), ("k", _vp), ("v", _vp), ("o", _vp), ("lse", _vp),
        ("q_stride_b", _i64), ("q_stride_s", _i64), ("q_stride_h", _i64),
        ("k_stride_b", _i64), ("k_stride_s", _i64), ("k_stride_h", _i64),
        ("v_stride_b", _i64), ("v_stride_s", _i64), ("v_stride_h", _i64),
        ("o_stride_b", _i64), ("o_stride_s", _i64), ("o_stride_h", _i64),
        ("lse_stride_b", _i64), ("lse_stride_s", _i64), ("lse_stride_h", _i64),
        ("cu_seqlens", _vp),
        ("batch", _i32), ("heads_q", _i32), ("heads_kv", _i32),
        ("max_seqlen", _i32), ("head_dim", _i32), ("causal", _i32),
        ("scale_log2", _f32), ("total_rows", _i32), ("dense_form", _i32),
    ]


class AttnSparseArgs(C.Structure):
    _fields_ = [
        ("struct_size", _u32), ("dtype", _i32),
        ("q", _vp), ("k", _vp), ("v", _vp), ("o", _vp), ("lse", _vp),
        ("q_stride_b", _i64), ("q_stride_s", _i64), ("q_stride_h", _i64),
        ("k_stride_b", _i64), ("k_stride_s", _i64), ("k_stride_h", _i64),
        ("v_stride_b", _i64), ("v_stride_s", _i64), ("v_stride_h", _i64),
        ("o_stride_b", _i64), ("o_stride_s", _i64), ("o_stride_h", _i64),
        ("lse_stride_b", _i64), ("lse_stride_s", _i64), ("lse_stride_h", _i64),
        ("cu_seqlens", _vp), ("row_ptr", _vp), ("col_idx", _vp),
        ("row_ptr_stride_b", _i64), ("row_ptr_stride_h", _i64),
        ("col_idx_stride_b", _i64), ("col_idx_stride_h", _i64),
        ("batch", _i32), ("heads_q", _i32), ("heads_kv", _i32),
        ("max_seqlen", _i32), ("head_dim", _i32), ("block_size", _i32),
        ("window_local", _i32), ("window_global", _i32),
        ("scale_log2", _f32), ("total_rows", _i32),
    ]


class AttnBwdArgs(C.Structure):
    _fields_ = (
        [("struct_size", _u32), ("dtype", _i32),
         ("q", _vp), ("k", _vp), ("v", _vp), ("o", _vp), ("dout", _vp), ("lse", _vp),
         ("dq", _vp), ("dk", _vp), ("dv", _vp)]
        + [("%s_stride_%s" % (t, d), _i64) for t in ("q", "k", "v", "o", "dout", "dq", "dk", "dv", "lse")
           for d in ("b", "s", "h")]
        + [("cu_seqlens", _vp),
           ("batch", _i32), ("heads_q", _i32), ("heads_kv", _i32),
           ("max_seqlen", _i32), ("head_dim", _i32), ("causal", _i32),
           ("scale_log2", _f32),
           ("workspace", _vp), ("workspace_bytes", _sz), ("total_rows", _i32)]
    )


class RmsNormArgs(C.Structure):
    _fields_ = [
        ("struct_size", _u32), ("x_dtype", _i32), ("w_dtype", _i32), ("dim", _i32),
        ("rows", _i64),
        ("x", _vp), ("w", _vp), ("y", _vp), ("rsqrt", _vp), ("dy", _vp), ("dx", _vp), ("dw", _vp),
        ("x_stride", _i64), ("y_stride", _i64), ("dy_stride", _i64), ("dx_stride", _i64),
        ("eps", _f32),
        ("workspace", _vp), ("workspace_bytes", _sz),
    ]


class XentArgs(C.Structure):
    _fields_ = [
        ("struct_size", _u32), ("dtype", _i32),
        ("tokens", _i32), ("dim", _i32), ("vocab", _i32), ("labels_i64", _i32),
        ("x", _vp), ("w", _vp), ("y", _vp),
        ("x_stride", _i64), ("w_stride", _i64),
        ("lse", _vp), ("loss", _vp),
        ("workspace", _vp), ("workspace_bytes", _sz),
    ]


class XentBwdArgs(C.Structure):
    _fields_ = [
        ("struct_size", _u32), ("dtype", _i32),
        ("tokens", _i32), ("dim", _i32), ("vocab", _i32), ("labels_i64", _i32),
        ("x", _vp), ("w", _vp), ("y", _vp),
        ("x_stride", _i64), ("w_stride", _i64),
        ("lse", _vp), ("dloss", _vp),
        ("dlogits", _vp), ("ld", _i64),
    ]


class XentGradArgs(C.Structure):
    _fields_ = [
        ("struct_size", _u32), ("dtype", _i32), ("vocab", _i32), ("labels_i64", _i32),
        ("rows", _i64), ("ld", _i64),
        ("logits", _vp), ("lse", _vp), ("dloss", _vp), ("y", _vp),
    ]


class DecodeArgs(C.Structure):
    _fields_ = [
        ("struct_size", _u32), ("dtype", _i32),
        ("q", _vp), ("k", _vp), ("v", _vp), ("o", _vp), ("lse", _vp),
        ("q_stride_b", _i64), ("q_stride_h", _i64),
        ("k_stride_b", _i64), ("k_stride_s", _i64), ("k_stride_h", _i64),
        ("v_stride_b", _i64), ("v_stride_s", _i64), ("v_stride_h", _i64),
        ("o_stride_b", _i64), ("o_stride_h", _i64),
        ("seq_lens", _vp), ("cu_seqlens", _vp),
        ("batch", _i32), ("heads_q", _i32), ("heads_kv", _i32),
        ("max_seqlen", _i32), ("head_dim", _i32),
        ("scale_log2", _f32),
        ("split_tokens", _i32),
        ("workspace", _vp), ("workspace_bytes", _sz),
        ("block_idx", _vp), ("block_cnt", _vp),
        ("block_idx_stride_b", _i64), ("block_idx_stride_h", _i64),
        ("max_blocks", _i32), ("block_size", _i32), ("split_blocks", _i32),
        ("window_local", _i32), ("window_global", _i32),
        ("include_last_block", _i32),
        ("kv_layout", _i32), ("page_size", _i32),
        ("page_table", _vp), ("page_table_stride_b", _i64),
        ("window_form", _i32),
    ]


# name -> (restype, argtypes); every symbol include/mi_attn.h declares
EXPORTS = {
    "mi_attn_fwd": (C.c_int, [C.POINTER(AttnFwdArgs), _vp]),
    "mi_attn_fwd_blocksparse": (C.c_int, [C.POINTER(AttnSparseArgs), _vp]),
    "mi_attn_bwd": (C.c_int, [C.POINTER(AttnBwdArgs), _vp]),
    "mi_attn_bwd_workspace_bytes": (_sz, [C.POINTER(AttnBwdArgs)]),
    "mi_attn_bwd_validate": (C.c_int, [C.POINTER(AttnBwdArgs)]),
    "mi_rmsnorm_fwd": (C.c_int, [C.POINTER(RmsNormArgs), _vp]),
    "mi_rmsnorm_bwd": (C.c_int, [C.POINTER(RmsNormArgs), _vp]),
    "mi_rmsnorm_bwd_workspace_bytes": (_sz, [C.POINTER(RmsNormArgs)]),
    "mi_xent_fwd": (C.c_int, [C.POINTER(XentArgs), _vp]),
    "mi_xent_fwd_workspace_bytes": (_sz, [C.POINTER(XentArgs)]),
    "mi_xent_dlogits": (C.c_int, [C.POINTER(XentGradArgs), _vp]),
    "mi_xent_bwd_dlogits": (C.c_int, [C.POINTER(XentBwdArgs), _vp]),
    "mi_decode_num_splits": (C.c_int, [C.POINTER(DecodeArgs)]),
    "mi_decode_workspace_bytes": (_sz, [C.POINTER(DecodeArgs)]),
    "mi_decode_choose_split_tokens": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int]),
    "mi_decode_choose_split_blocks": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int]),
    "mi_decode_splitkv": (C.c_int, [C.POINTER(DecodeArgs), _vp]),
    "mi_decode_merge": (C.c_int, [C.POINTER(DecodeArgs), _vp]),
    "mi_decode": (C.c_int, [C.POINTER(DecodeArgs), _vp]),
    "mi_abi_version": (C.c_int, []),
    "mi_last_error": (C.c_char_p, []),
    "mi_status_name": (C.c_char_p, [C.c_int]),
    "mi_attn_fwd_validate": (C.c_int, [C.POINTER(AttnFwdArgs)]),
    "mi_attn_fwd_blocksparse_validate": (C.c_int, [C.POINTER(AttnSparseArgs)]),
    "mi_decode_validate": (C.c_int, [C.POINTER(DecodeArgs)]),
    "mi_decode_noalloc": (C.c_int, [C.POINTER(DecodeArgs), _vp]),
    "mi_device_cu_count": (C.c_int, []),
    # include/mi_attn_bench.h
    "mi_time_launches": (C.c_int, [C.c_int, _vp, C.c_int, _sz, _vp, C.c_int, C.c_int, C.POINTER(C.c_float)]),
}


class MiAttnError(RuntimeError):
    def __init__(self, status, message):
        self.status = status
        super().__init__("%s (%d): %s" % (STATUS.get(status, "MI_ERR_UNKNOWN"), status, message))


_lib = None


def load():
    """Load the shared library (once) and declare every exported symbol."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s is missing: build it with `python -m tritonops_amd.build` "
            "(there is no fallback implementation)" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in EXPORTS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.mi_abi_version() != MI_ATTN_ABI_VERSION:
        raise ImportError("libmi_attn.so ABI %d != binding ABI %d" % (lib.mi_abi_version(), MI_ATTN_ABI_VERSION))
    _lib = lib
    return lib


def check(status):
    if status != 0:
        raise MiAttnError(status, load().mi_last_error().decode())
