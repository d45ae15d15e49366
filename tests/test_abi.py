"""CPU-only checks of the C ABI: the library loads, exports every symbol that
include/mi_attn.h declares, the ctypes structs match the C layout, and every
validation error is reported before anything touches a device."""
import ctypes as C
import os
import re
import subprocess

import pytest

from tritonops_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", n) for n in ("mi_attn.h", "mi_attn_bench.h")]


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def test_every_declared_symbol_is_exported(lib):
    text = "".join(open(h).read() for h in HEADERS)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = set(re.findall(r"\b(mi_[a-z_0-9]+)\s*\(", text))
    assert declared, "no prototypes found in the header"
    assert declared == set(_lib.EXPORTS), "ctypes table and header disagree: %s" % (declared ^ set(_lib.EXPORTS))
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.mi_abi_version() == _lib.MI_ATTN_ABI_VERSION == 8


def test_struct_layout_matches_the_c_compiler(tmp_path):
    src = tmp_path / "sz.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "mi_attn.h"\nint main(){printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu\\n",'
                   "sizeof(mi_attn_fwd_args),sizeof(mi_attn_sparse_args),sizeof(mi_decode_args),"
                   "offsetof(mi_attn_fwd_args,scale_log2),offsetof(mi_attn_sparse_args,scale_log2),"
                   "offsetof(mi_decode_args,page_table),"
                   "sizeof(mi_attn_bwd_args),offsetof(mi_attn_bwd_args,workspace),"
                   "sizeof(mi_rmsnorm_args),offsetof(mi_rmsnorm_args,eps),"
                   "sizeof(mi_xent_args),offsetof(mi_xent_args,workspace),"
                   "sizeof(mi_xent_grad_args),offsetof(mi_xent_grad_args,y),"
                   "sizeof(mi_xent_bwd_args),offsetof(mi_xent_bwd_args,ld));return 0;}\n")
    exe = tmp_path / "sz"
    subprocess.check_call(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    got = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    want = [C.sizeof(_lib.AttnFwdArgs), C.sizeof(_lib.AttnSparseArgs), C.sizeof(_lib.DecodeArgs),
            _lib.AttnFwdArgs.scale_log2.offset, _lib.AttnSparseArgs.scale_log2.offset,
            _lib.DecodeArgs.page_table.offset,
            C.sizeof(_lib.AttnBwdArgs), _lib.AttnBwdArgs.workspace.offset,
            C.sizeof(_lib.RmsNormArgs), _lib.RmsNormArgs.eps.offset,
            C.sizeof(_lib.XentArgs), _lib.XentArgs.workspace.offset,
            C.sizeof(_lib.XentGradArgs), _lib.XentGradArgs.y.offset,
            C.sizeof(_lib.XentBwdArgs), _lib.XentBwdArgs.ld.offset]
    assert got == want


def _good_fwd():
    a = _lib.AttnFwdArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = 0
    a.q = a.k = a.v = a.o = 0x1000
    for n in "qkvo":
        setattr(a, n + "_stride_s", 128 * 4)
        setattr(a, n + "_stride_h", 128)
        setattr(a, n + "_stride_b", 128 * 4 * 64)
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim, a.causal = 2, 4, 2, 64, 128, 1
    a.scale_log2 = 0.1275
    return a


def _err(lib):
    return lib.mi_last_error().decode()


def test_fwd_validation(lib):
    a = _good_fwd()
    assert lib.mi_attn_fwd_validate(C.byref(a)) == 0
    cases = [
        (lambda a: setattr(a, "struct_size", 8), "MI_ERR_STRUCT_SIZE"),
        (lambda a: setattr(a, "dtype", 7), "MI_ERR_DTYPE"),
        (lambda a: setattr(a, "head_dim", 80), "MI_ERR_HEAD_DIM"),
        (lambda a: setattr(a, "heads_kv", 3), "MI_ERR_GQA"),
        (lambda a: setattr(a, "heads_q", 0), "MI_ERR_GQA"),
        (lambda a: setattr(a, "batch", 0), "MI_ERR_SHAPE"),
        (lambda a: setattr(a, "max_seqlen", -1), "MI_ERR_SHAPE"),
        (lambda a: setattr(a, "causal", 2), "MI_ERR_SHAPE"),
        (lambda a: setattr(a, "scale_log2", 0.0), "MI_ERR_SCALE"),
        (lambda a: setattr(a, "scale_log2", float("nan")), "MI_ERR_SCALE"),
        (lambda a: setattr(a, "q", None), "MI_ERR_NULL_POINTER"),
        (lambda a: setattr(a, "k", 0x1004), "MI_ERR_ALIGNMENT"),
        (lambda a: setattr(a, "v_stride_s", 100), "MI_ERR_STRIDE"),
        (lambda a: setattr(a, "o_stride_b", 4), "MI_ERR_STRIDE"),
        (lambda a: setattr(a, "total_rows", -1), "MI_ERR_SHAPE"),
        (lambda a: setattr(a, "total_rows", 64), "MI_ERR_SHAPE"),       # batched form: there are no rows outside the sequences
        (lambda a: setattr(a, "dense_form", 3), "MI_ERR_SHAPE"),
        (lambda a: setattr(a, "dense_form", -1), "MI_ERR_SHAPE"),
    ]
    for mutate, want in cases:
        a = _good_fwd()
        mutate(a)
        rc = lib.mi_attn_fwd_validate(C.byref(a))
        assert rc < 0 and lib.mi_status_name(rc).decode() == want == _lib.STATUS[rc], (want, rc)
        assert _err(lib)
        # the launch entry point refuses the same way, before any HIP call
        assert lib.mi_attn_fwd(C.byref(a), None) == rc
    assert lib.mi_attn_fwd_validate(None) == -1
    # packed mode ignores batch strides
    a = _good_fwd()
    a.cu_seqlens = 0x2000
    a.o_stride_b = 4
    a.total_rows = 4096
    assert lib.mi_attn_fwd_validate(C.byref(a)) == 0
    for form in (_lib.MI_DENSE_FORM_AUTO, _lib.MI_DENSE_FORM_256_ROWS, _lib.MI_DENSE_FORM_128_ROWS):
        a.dense_form = form
        assert lib.mi_attn_fwd_validate(C.byref(a)) == 0


def _good_sparse():
    a = _lib.AttnSparseArgs()
    a.struct_size = C.sizeof(a)
    a.q = a.k = a.v = a.o = 0x1000
    a.row_ptr = a.col_idx = 0x3000
    for n in "qkvo":
        setattr(a, n + "_stride_s", 256)
        setattr(a, n + "_stride_h", 128)
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim = 1, 2, 2, 640, 128
    a.block_size, a.window_local, a.window_global = 64, -1, -1
    a.scale_log2 = 0.1
    return a


def test_sparse_validation(lib):
    assert lib.mi_attn_fwd_blocksparse_validate(C.byref(_good_sparse())) == 0
    for mutate, want in [
        (lambda a: setattr(a, "block_size", 128), "MI_ERR_SPARSE_LAYOUT"),
        (lambda a: setattr(a, "row_ptr", None), "MI_ERR_NULL_POINTER"),
        (lambda a: setattr(a, "window_local", 5), "MI_ERR_SPARSE_LAYOUT"),
        (lambda a: setattr(a, "col_idx_stride_h", -1), "MI_ERR_SPARSE_LAYOUT"),
        (lambda a: setattr(a, "head_dim", 256), "MI_ERR_HEAD_DIM"),
    ]:
        a = _good_sparse()
        mutate(a)
        rc = lib.mi_attn_fwd_blocksparse_validate(C.byref(a))
        assert lib.mi_status_name(rc).decode() == want
        assert lib.mi_attn_fwd_blocksparse(C.byref(a), None) == rc
    # no lists at all: the token-window form, which needs both windows and a local one of at least a token
    a = _good_sparse()
    a.row_ptr = a.col_idx = None
    for wl, wg, rc in ((-1, -1, -1), (0, 64, -1), (1, 0, 0), (4096, 128, 0), (2 ** 31 - 1, 2 ** 31 - 1, 0)):
        a.window_local, a.window_global = wl, wg
        assert lib.mi_attn_fwd_blocksparse_validate(C.byref(a)) == rc, (wl, wg)
        assert rc == 0 or "window_local >= 1" in _err(lib)


def _good_decode():
    a = _lib.DecodeArgs()
    a.struct_size = C.sizeof(a)
    a.q = a.k = a.v = a.o = 0x1000
    a.seq_lens = 0x2000
    a.q_stride_b, a.q_stride_h = 32 * 128, 128
    a.k_stride_b, a.k_stride_s, a.k_stride_h = 8 * 4096 * 128, 128, 4096 * 128
    a.v_stride_b, a.v_stride_s, a.v_stride_h = 8 * 4096 * 128, 128, 4096 * 128
    a.o_stride_b, a.o_stride_h = 32 * 128, 128
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim = 4, 32, 8, 4096, 128
    a.scale_log2 = 0.1
    a.split_tokens = 512
    a.workspace, a.workspace_bytes = 0x4000, 1 << 30
    return a


def test_decode_geometry_and_validation(lib):
    a = _good_decode()
    assert lib.mi_decode_num_splits(C.byref(a)) == 8
    assert lib.mi_decode_workspace_bytes(C.byref(a)) == 4 * 32 * 8 * 129 * 4
    assert lib.mi_decode_validate(C.byref(a)) == 0
    for mutate, want in [
        (lambda a: setattr(a, "split_tokens", 100), "MI_ERR_WORKSPACE"),
        (lambda a: setattr(a, "workspace_bytes", 16), "MI_ERR_WORKSPACE"),
        (lambda a: setattr(a, "workspace", None), "MI_ERR_NULL_POINTER"),
        (lambda a: setattr(a, "cu_seqlens", 0x2000), "MI_ERR_NULL_POINTER"),     # both given
        (lambda a: setattr(a, "seq_lens", None), "MI_ERR_NULL_POINTER"),         # none given
        (lambda a: setattr(a, "heads_kv", 0), "MI_ERR_GQA"),
        (lambda a: (setattr(a, "heads_q", 66), setattr(a, "heads_kv", 4)), "MI_ERR_GQA"),   # not a multiple
        (lambda a: setattr(a, "window_form", 2), "MI_ERR_SPARSE_LAYOUT"),
        (lambda a: setattr(a, "k_stride_s", 12), "MI_ERR_STRIDE"),
        # a tile is addressed with 32-bit byte offsets: negative or huge row strides would wrap
        (lambda a: setattr(a, "k_stride_s", -128), "MI_ERR_STRIDE"),
        (lambda a: setattr(a, "v_stride_s", 1 << 24), "MI_ERR_STRIDE"),
        (lambda a: setattr(a, "head_dim", 32), "MI_ERR_HEAD_DIM"),
    ]:
        a = _good_decode()
        mutate(a)
        rc = lib.mi_decode_validate(C.byref(a))
        assert lib.mi_status_name(rc).decode() == want, (want, rc, _err(lib))
        assert lib.mi_decode(C.byref(a), None) == rc
    a = _good_decode()
    a.k_stride_s = a.v_stride_s = (1 << 24) - 8
    assert lib.mi_decode_validate(C.byref(a)) == 0
    # a GQA group of more than 32 query heads is walked in slices of 32
    a = _good_decode()
    a.heads_q, a.heads_kv = 66, 2
    assert lib.mi_decode_validate(C.byref(a)) == 0
    assert lib.mi_decode_workspace_bytes(C.byref(a)) == 4 * 66 * 8 * 129 * 4
    # window form: the list is derived in the kernel, block_idx may be NULL
    a = _good_decode()
    a.window_form, a.block_size, a.split_blocks = 1, 64, 4
    a.window_global, a.window_local = 256, 1000
    a.max_blocks = 4 + 16 + 1
    assert lib.mi_decode_validate(C.byref(a)) == 0 and lib.mi_decode_num_splits(C.byref(a)) == 6
    a.include_last_block = 1     # ignored in the window form
    assert lib.mi_decode_num_splits(C.byref(a)) == 6
    for mutate in (lambda a: setattr(a, "max_blocks", 20), lambda a: setattr(a, "window_local", -1),
                   lambda a: setattr(a, "split_blocks", 0), lambda a: setattr(a, "block_size", 32)):
        b = _lib.DecodeArgs.from_buffer_copy(a)
        mutate(b)
        assert lib.mi_status_name(lib.mi_decode_validate(C.byref(b))).decode() == "MI_ERR_SPARSE_LAYOUT", _err(lib)
    # sparse form
    a = _good_decode()
    a.block_idx = 0x5000
    a.max_blocks, a.block_size, a.split_blocks = 129, 64, 8
    a.window_local = a.window_global = -1
    assert lib.mi_decode_num_splits(C.byref(a)) == 17
    assert lib.mi_decode_validate(C.byref(a)) == 0
    a.block_size = 32
    assert lib.mi_status_name(lib.mi_decode_validate(C.byref(a))).decode() == "MI_ERR_SPARSE_LAYOUT"
    # an empty list is valid exactly when the implicit last block is attended
    a.block_size, a.max_blocks, a.include_last_block = 64, 0, 1
    assert lib.mi_decode_validate(C.byref(a)) == 0 and lib.mi_decode_num_splits(C.byref(a)) == 1
    a.include_last_block = 0
    assert lib.mi_status_name(lib.mi_decode_validate(C.byref(a))).decode() == "MI_ERR_SPARSE_LAYOUT"
    a.max_blocks = -1
    a.include_last_block = 1
    assert lib.mi_status_name(lib.mi_decode_validate(C.byref(a))).decode() == "MI_ERR_SPARSE_LAYOUT"


def test_decode_noalloc_validation(lib):
    """The entry point that allocates nothing ignores the workspace fields and
    refuses, before any HIP call, a launch whose partials exceed its buffer."""
    a = _good_decode()
    a.workspace, a.workspace_bytes = None, 0
    a.head_dim = 32                                   # every other check still runs first
    assert lib.mi_status_name(lib.mi_decode_noalloc(C.byref(a), None)).decode() == "MI_ERR_HEAD_DIM"
    a = _good_decode()
    a.workspace, a.workspace_bytes = None, 0
    a.batch, a.max_seqlen, a.split_tokens = 64, 1 << 20, 64      # 64 * 32 * 16384 * 129 * 4 bytes of partials
    assert lib.mi_decode_workspace_bytes(C.byref(a)) > _lib.MI_DECODE_STATIC_SCRATCH_BYTES
    rc = lib.mi_decode_noalloc(C.byref(a), None)
    assert lib.mi_status_name(rc).decode() == "MI_ERR_WORKSPACE" and "static buffer" in _err(lib)
    text = open(HEADERS[0]).read()
    assert re.search(r"#define MI_DECODE_STATIC_SCRATCH_BYTES \(32u << 20\)", text)


def test_decode_kv_layout_validation(lib):
    a = _good_decode()
    a.kv_layout = 7
    assert lib.mi_status_name(lib.mi_decode_validate(C.byref(a))).decode() == "MI_ERR_SHAPE"
    a = _good_decode()
    a.kv_layout = 2                                   # paged
    a.page_size, a.page_table = 48, 0x6000
    assert lib.mi_status_name(lib.mi_decode_validate(C.byref(a))).decode() == "MI_ERR_SHAPE"   # not a multiple of 32
    a.page_size, a.page_table = 64, None
    assert lib.mi_status_name(lib.mi_decode_validate(C.byref(a))).decode() == "MI_ERR_NULL_POINTER"
    a.page_table = 0x6000
    assert lib.mi_decode_validate(C.byref(a)) == 0
    a = _good_decode()
    a.kv_layout = 1                                   # packed: offsets come from cu_seqlens
    if a.cu_seqlens:
        assert lib.mi_decode_validate(C.byref(a)) == 0
        a.seq_lens, a.cu_seqlens = a.cu_seqlens, None
    assert lib.mi_status_name(lib.mi_decode_validate(C.byref(a))).decode() == "MI_ERR_NULL_POINTER"


def test_split_heuristic(lib):
    f = lib.mi_decode_choose_split_tokens
    for args in [(64, 8, 32768, 256), (1, 1, 100, 256), (1, 8, 131072, 256), (512, 8, 4096, 256), (0, 0, 0, 0)]:
        t = f(*args)
        assert t % 64 == 0 and 64 <= t <= 2048
    assert f(64, 8, 32768, 256) == 2048          # plenty of work: the longest chunk
    assert f(1, 8, 32768, 256) == 512            # little work: the shortest chunk worth a partial result
    assert f(1, 8, 8192, 256) == 256             # ... which is shorter where a sequence still makes at most 32 chunks
    assert f(4, 8, 8192, 256) == 256
    assert f(8, 8, 8192, 256) == 512
    assert f(1, 8, 12288, 256) == 384
    assert f(4, 8, 32768, 256) == 1024           # in between: about half a resident round's share
    assert f(1, 1, 1 << 20, 256) == 1024


def test_backward_and_rmsnorm_validation(lib):
    a = _lib.AttnBwdArgs()
    a.struct_size = C.sizeof(a)
    a.dtype, a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim, a.causal = 0, 1, 4, 2, 128, 128, 1
    a.scale_log2 = 0.1
    for n in ("q", "k", "v", "o", "dout", "lse", "dq", "dk", "dv"):
        setattr(a, n, 0x1000)
        for d in ("b", "s", "h"):
            setattr(a, "%s_stride_%s" % (n, d), 1024)
    assert lib.mi_attn_bwd_workspace_bytes(C.byref(a)) == 1 * 4 * 128 * 4
    assert lib.mi_status_name(lib.mi_attn_bwd_validate(C.byref(a))).decode() == "MI_ERR_WORKSPACE"
    a.workspace, a.workspace_bytes = 0x2000, 4096
    assert lib.mi_attn_bwd_validate(C.byref(a)) == 0
    a.dk = None
    assert lib.mi_status_name(lib.mi_attn_bwd_validate(C.byref(a))).decode() == "MI_ERR_NULL_POINTER"
    a.dk = 0x1000
    for field in ("q_stride_s", "dout_stride_s", "lse_stride_s"):      # streamed tiles use 32-bit lane offsets
        for bad in (-1024, 1 << 24):
            setattr(a, field, bad)
            assert lib.mi_status_name(lib.mi_attn_bwd_validate(C.byref(a))).decode() == "MI_ERR_STRIDE", field
        setattr(a, field, 1024)
    assert lib.mi_attn_bwd_validate(C.byref(a)) == 0
    a.dk, a.heads_kv = 0x1000, 3
    assert lib.mi_status_name(lib.mi_attn_bwd_validate(C.byref(a))).decode() == "MI_ERR_GQA"
    a.heads_kv, a.struct_size = 2, 8
    assert lib.mi_attn_bwd(C.byref(a), None) == -2

    r = _lib.RmsNormArgs()
    r.struct_size = C.sizeof(r)
    r.x_dtype, r.w_dtype, r.dim, r.rows = 0, 2, 255, 10
    r.x = r.w = r.y = r.rsqrt = 0x1000
    r.x_stride = r.y_stride = 255
    r.eps = 1e-6
    # a launch would follow a clean validation, so only the failing cases are called here
    r.w_dtype = 1
    assert lib.mi_status_name(lib.mi_rmsnorm_fwd(C.byref(r), None)).decode() == "MI_ERR_DTYPE"
    r.w_dtype, r.x_stride = 2, 100
    assert lib.mi_status_name(lib.mi_rmsnorm_fwd(C.byref(r), None)).decode() == "MI_ERR_STRIDE"
    r.x_stride, r.dim = 255, 0
    assert lib.mi_status_name(lib.mi_rmsnorm_fwd(C.byref(r), None)).decode() == "MI_ERR_SHAPE"
    r.dim = 255
    assert lib.mi_status_name(lib.mi_rmsnorm_bwd(C.byref(r), None)).decode() == "MI_ERR_NULL_POINTER"
    assert lib.mi_rmsnorm_bwd_workspace_bytes(C.byref(r)) == (12 + 32) * 255 * 4  # 10 rows -> 12 partial rows + 32 stage rows
    r.rows = 0
    assert lib.mi_rmsnorm_fwd(C.byref(r), None) == 0 and lib.mi_rmsnorm_bwd(C.byref(r), None) == 0


def test_fused_cross_entropy_validation(lib):
    a = _lib.XentArgs()
    a.struct_size = C.sizeof(a)
    a.dtype, a.tokens, a.dim, a.vocab, a.labels_i64 = 0, 8192, 4096, 128256, 1
    a.x = a.w = a.y = a.lse = a.loss = 0x1000
    a.x_stride = a.w_stride = 4096
    # 32 token tiles of 256 -> 8 vocabulary ranges fill 256 CUs; two fp32 per token and range
    assert lib.mi_xent_fwd_workspace_bytes(C.byref(a)) == 8192 * 8 * 2 * 4
    # a launch would follow a clean validation, so only the failing cases are called here
    assert lib.mi_status_name(lib.mi_xent_fwd(C.byref(a), None)).decode() == "MI_ERR_WORKSPACE"
    a.workspace, a.workspace_bytes = 0x2000, 1 << 20
    a.dim = 4000
    assert lib.mi_status_name(lib.mi_xent_fwd(C.byref(a), None)).decode() == "MI_ERR_SHAPE"
    a.dim, a.x_stride = 4096, 4000
    assert lib.mi_status_name(lib.mi_xent_fwd(C.byref(a), None)).decode() == "MI_ERR_STRIDE"
    a.x_stride, a.dtype = 4096, 2
    assert lib.mi_status_name(lib.mi_xent_fwd(C.byref(a), None)).decode() == "MI_ERR_DTYPE"
    a.dtype, a.x = 0, 0x1008
    assert lib.mi_status_name(lib.mi_xent_fwd(C.byref(a), None)).decode() == "MI_ERR_ALIGNMENT"
    a.x, a.loss = 0x1000, None
    assert lib.mi_status_name(lib.mi_xent_fwd(C.byref(a), None)).decode() == "MI_ERR_NULL_POINTER"
    a.tokens = 0
    assert lib.mi_xent_fwd(C.byref(a), None) == 0
    # few tokens: one token tile, as many ranges as CUs, never more than vocabulary tiles
    a.tokens, a.vocab = 100, 1000
    assert lib.mi_xent_fwd_workspace_bytes(C.byref(a)) == 100 * 4 * 2 * 4

    b = _lib.XentBwdArgs()
    b.struct_size = C.sizeof(b)
    b.dtype, b.tokens, b.dim, b.vocab, b.labels_i64 = 0, 512, 1024, 32000, 0
    b.x = b.w = b.y = b.lse = b.dloss = b.dlogits = 0x1000
    b.x_stride = b.w_stride = 1024
    b.ld = 31999
    assert lib.mi_status_name(lib.mi_xent_bwd_dlogits(C.byref(b), None)).decode() == "MI_ERR_STRIDE"
    b.ld, b.dim = 32000, 1000
    assert lib.mi_status_name(lib.mi_xent_bwd_dlogits(C.byref(b), None)).decode() == "MI_ERR_SHAPE"
    b.dim, b.dloss = 1024, None
    assert lib.mi_status_name(lib.mi_xent_bwd_dlogits(C.byref(b), None)).decode() == "MI_ERR_NULL_POINTER"
    b.tokens = 0
    assert lib.mi_xent_bwd_dlogits(C.byref(b), None) == 0

    g = _lib.XentGradArgs()
    g.struct_size = C.sizeof(g)
    g.dtype, g.vocab, g.labels_i64, g.rows, g.ld = 0, 1000, 1, 16, 900
    g.logits = g.lse = g.dloss = g.y = 0x1000
    assert lib.mi_status_name(lib.mi_xent_dlogits(C.byref(g), None)).decode() == "MI_ERR_STRIDE"
    g.ld, g.y = 1000, None
    assert lib.mi_status_name(lib.mi_xent_dlogits(C.byref(g), None)).decode() == "MI_ERR_NULL_POINTER"
    g.rows = 0
    assert lib.mi_xent_dlogits(C.byref(g), None) == 0
    g.struct_size = 4
    assert lib.mi_xent_dlogits(C.byref(g), None) == -2


def test_split_blocks_heuristic(lib):
    f = lib.mi_decode_choose_split_blocks
    # 32 sequences x 8 kv-heads on 256 CUs: 2048 resident wavefronts / 256 units = 8 chunks of 129 blocks
    assert f(32, 8, 129, 256) == 17
    assert f(4096, 8, 129, 256) == 129           # more units than wavefront slots: one chunk each
    assert f(1, 1, 129, 256) == 1                # one unit: a chunk per block
    assert f(0, 0, 0, 0) == 1
    for args in [(32, 8, 129, 256), (3, 5, 77, 256), (64, 8, 2048, 304)]:
        sb = f(*args)
        chunks = -(-args[2] // sb)
        assert 1 <= sb <= args[2] and chunks * args[0] * args[1] <= max(8 * args[3], args[0] * args[1])


def test_time_launches_rejects_bad_arguments(lib):
    ms = C.c_float()
    assert lib.mi_time_launches(0, None, 1, 0, None, 0, 1, C.byref(ms)) == -1
    assert "non-NULL" in _err(lib)
    a = _good_fwd()
    assert lib.mi_time_launches(12, C.cast(C.byref(a), C.c_void_p), 1, 0, None, 0, 1, C.byref(ms)) == -6
    assert "kind" in _err(lib)
    assert lib.mi_time_launches(0, C.cast(C.byref(a), C.c_void_p), 0, 0, None, 0, 1, C.byref(ms)) == -6
    a.head_dim = 5
    assert lib.mi_time_launches(0, C.cast(C.byref(a), C.c_void_p), 1, 0, None, 1, 1, C.byref(ms)) == -4


def test_python_wrappers_refuse_cpu_tensors():
    import torch

    import tritonops_amd as ta

    q = torch.zeros(1, 4, 2, 64, dtype=torch.bfloat16)
    cu = torch.tensor([0, 4], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="GPU only"):
        ta.flash_attention(q, q, q, cu)
    with pytest.raises(RuntimeError, match="GPU only"):
        ta.flash_attention_decoding(q[:, 0], q, q, cu)


def test_python_wrappers_check_extents_before_any_launch():
    """The kernels take every extent from q: a shorter k / v, a mis-shaped do or
    lse, or a wrong index tensor must be refused on the host (no GPU needed)."""
    import torch

    import tritonops_amd as ta
    from tritonops_amd import ops

    bf = torch.bfloat16
    q = torch.zeros(1, 16, 4, 64, dtype=bf)
    k = torch.zeros(1, 16, 2, 64, dtype=bf)
    cu = torch.tensor([0, 16], dtype=torch.int32)
    lse = torch.zeros(1, 16, 4)
    for bad_k, bad_v in ((k[:, :8], k), (k, k[:, :8]), (k, k[:, :, :1]), (k.float(), k), (k[..., :32], k[..., :32]),
                         (torch.zeros(1, 16, 3, 64, dtype=bf),) * 2):
        with pytest.raises(ValueError):
            ta.flash_attention(q, bad_k, bad_v, cu)
        with pytest.raises(ValueError):
            ta.flash_attn_sparse_triton(q, bad_k, bad_v, cu, None, 64, 64)
        with pytest.raises(ValueError):
            ta.flash_attn_triton_bwd(q, bad_k, bad_v, q, q, lse, cu, 0.1)
    with pytest.raises(ValueError):                      # batched form: [B, H, S, D]
        ta.flash_attention(q.transpose(1, 2), k.transpose(1, 2)[:, :, :8], k.transpose(1, 2)[:, :, :8])
    for o, do, l in ((q[:, :8], q, lse), (q, q[:, :8], lse), (q, q, lse[:, :8]), (q, q, lse.double()),
                     (q, q.float(), lse), (q, lse, q)):     # the last one: do and lse swapped
        with pytest.raises(ValueError):
            ta.flash_attn_triton_bwd(q, k, k, o, do, l, cu, 0.1)
    # all extents right: the call gets as far as the device check
    with pytest.raises(RuntimeError, match="GPU only"):
        ta.flash_attn_triton_bwd(q, k, k, q, q, lse, cu, 0.1)

    qd = torch.zeros(2, 4, 64, dtype=bf)
    kd = torch.zeros(2, 128, 2, 64, dtype=bf)
    cu2 = torch.tensor([0, 100, 228], dtype=torch.int32)
    with pytest.raises(ValueError):
        ta.flash_attention_decoding(qd, kd, kd[:, :64], cu2)
    with pytest.raises(ValueError):
        ta.flash_attention_decoding(qd, kd, kd.half(), cu2)
    with pytest.raises(ValueError):
        ta.flash_attention_decoding(qd, kd, kd, cu2[:2])
    with pytest.raises(ValueError):
        ta.flash_attention_decoding(qd, kd, kd, None, seq_lens=torch.tensor([1.0, 2.0]))
    with pytest.raises(ValueError):
        ta.flash_attention_decoding(qd, kd, kd, cu2, kv_layout="paged", page_table=torch.zeros(2, 2), page_size=128)
    for idx in (torch.zeros(2, 2, 3), torch.zeros(2, 3, dtype=torch.int32), torch.zeros(1, 2, 3, dtype=torch.int32)):
        with pytest.raises(ValueError):
            ta.flash_attention_sparse_decoding(qd, kd, kd, cu2, block_indices=idx)
    with pytest.raises(ValueError):
        ta.flash_attention_sparse_decoding(qd, kd, kd, cu2, block_indices=torch.zeros(2, 2, 1, dtype=torch.int32),
                                           block_counts=torch.zeros(2, 3, dtype=torch.int32))
    with pytest.raises(ValueError):
        ta.flash_attention_sparse_decoding(qd, kd, kd, cu2, block_indices=torch.zeros(2, 2, 0, dtype=torch.int32),
                                           include_last_block=False)
    with pytest.raises(RuntimeError, match="GPU only"):
        ta.flash_attention_decoding(qd, kd, kd, cu2)


def test_window_csr_is_built_once():
    from tritonops_amd import masks

    a = masks.window_csr(40, 200, 128, "cpu")
    b = masks.window_csr(40, 200, 128, "cpu")
    assert a[0] is b[0] and a[1] is b[1]
    want = masks.block_mask_to_csr(masks.window_block_mask(40, 200, 128), "cpu")
    assert (a[0] == want[0]).all() and (a[1] == want[1]).all() and a[2] == want[2]


def test_host_knowledge_of_cu_seq_lens_follows_the_tensor():
    """The drop-ins keep what one host read of a cu_seq_lens tensor told them (longest
    sequence, first and last entry) for as long as that tensor object is unmodified, and
    decide from it whether any row of a packed output lies outside every sequence."""
    import torch

    from tritonops_amd import ops

    cu = torch.tensor([0, 200, 512], dtype=torch.int32)
    assert ops._rows_to_cover(cu, 512, 512) == 512          # nothing on file yet: the library looks for such rows
    assert ops._max_len(cu, None) == 312                    # the host read
    assert ops._rows_to_cover(cu, 312, 512) == 0            # the sequences tile [0, 512) and none is cut
    assert ops._rows_to_cover(cu, 311, 512) == 512          # the longer sequence would be cut
    assert ops._rows_to_cover(cu, 312, 600) == 600          # padding rows behind the last sequence
    assert ops._max_len(cu, 100) == 100                     # a hint is taken as it is
    cu[2] = 400                                             # in place: the version counter moves
    assert ops._rows_to_cover(cu, 512, 512) == 512
    assert ops._max_len(cu, None) == 200 and ops._rows_to_cover(cu, 200, 400) == 0
    lead = torch.tensor([64, 200, 512], dtype=torch.int32)
    assert ops._max_len(lead, None) == 312 and ops._rows_to_cover(lead, 312, 512) == 512   # rows in front of the first sequence
    assert ops._max_len(torch.tensor([0], dtype=torch.int32), None) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    """No fallback: with the shared library absent every entry point raises."""
    import torch

    import tritonops_amd as ta

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libmi_attn.so"))
    with pytest.raises(ImportError):
        _lib.load()
    x = torch.zeros((2, 128), dtype=torch.bfloat16)
    for call in (lambda: ta.rmsnorm_fwd(x, torch.ones(128), 1e-6),
                 lambda: ta.cross_entropy_fused_fwd(x, x, torch.zeros(2, dtype=torch.int64)),
                 lambda: ta.flash_attention(x.view(1, 2, 1, 128), x.view(1, 2, 1, 128), x.view(1, 2, 1, 128),
                                            torch.tensor([0, 2], dtype=torch.int32))):
        with pytest.raises((ImportError, RuntimeError, TypeError, ValueError)):
            call()


def test_product_package_never_imports_the_oracle():
    """The oracle is test infrastructure: nothing under tritonops_amd/ (nor the
    C sources) may import, include or mention a path into oracle/."""
    import re

    pkg = os.path.join(ROOT, "tritonops_amd")
    pat = re.compile(r"^\s*(from|import)\s+oracle\b|oracle/|from\s+\.\.?oracle", re.M)
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, f), encoding="utf-8", errors="ignore").read()
                assert not pat.search(text), os.path.join(dirpath, f)


def test_bench_names_kernels_that_exist_in_the_library():
    """bench.py reports, per workload, the device symbol its roofline figure is
    about; every such symbol must be in the built library."""
    import importlib.util

    spec = importlib.util.spec_from_file_location("bench", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    blob = open(_lib.LIB_PATH, "rb").read()
    assert set(bench.KERNELS) == set(bench.WORKLOADS)
    for workload, names in bench.KERNELS.items():
        for name in names.split(" + "):
            assert name.encode() in blob, (workload, name)
