// C ABI of the library: host-side validation, launch geometry, error text.
// Nothing in this file touches the device except the final kernel launches.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "../../include/mi_attn.h"
#include "kernels.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// packed outputs [row][head][head_dim] (+ fp32 lse [row][head]) -> fill descriptors
mi::RowFillTensor fill_of(void* base, int64_t stride_s, int64_t stride_h, int heads, int elem_bytes, int row_elems) {
  mi::RowFillTensor t;
  t.base = base;
  t.row_stride = stride_s * elem_bytes;
  t.head_stride = stride_h * elem_bytes;
  t.heads = heads;
  t.bytes = row_elems * elem_bytes;
  return t;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
bool mult8(int64_t s) { return (s % 8) == 0; }

int check_common(int dtype, int head_dim, int batch, int hq, int hkv, int max_seqlen, float scale) {
  if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_F16) return fail(MI_ERR_DTYPE, "dtype %d is not bf16(0)/f16(1)", dtype);
  if (head_dim != 64 && head_dim != 96 && head_dim != 128)
    return fail(MI_ERR_HEAD_DIM, "head_dim %d not in {64, 96, 128}", head_dim);
  if (hq <= 0 || hkv <= 0 || hq % hkv != 0)
    return fail(MI_ERR_GQA, "heads_q %d must be a positive multiple of heads_kv %d", hq, hkv);
  if (batch <= 0) return fail(MI_ERR_SHAPE, "batch %d must be positive", batch);
  if (max_seqlen < 0) return fail(MI_ERR_SHAPE, "max_seqlen %d is negative", max_seqlen);
  if (!std::isfinite(scale) || scale <= 0.f) return fail(MI_ERR_SCALE, "scale_log2 %g must be finite and > 0", (double)scale);
  return MI_OK;
}

template <typename A>
int check_qkvo(const A* a) {
  if (!a->q || !a->k || !a->v || !a->o) return fail(MI_ERR_NULL_POINTER, "q, k, v and o must be non-NULL");
  if (!aligned16(a->q) || !aligned16(a->k) || !aligned16(a->v) || !aligned16(a->o))
    return fail(MI_ERR_ALIGNMENT, "q, k, v and o must be 16-byte aligned");
  return MI_OK;
}

template <typename A>
int check_prefill_strides(const A* a) {
  const int64_t s[] = {a->q_stride_s, a->q_stride_h, a->k_stride_s, a->k_stride_h,
                       a->v_stride_s, a->v_stride_h, a->o_stride_s, a->o_stride_h};
  for (int64_t x : s)
    if (!mult8(x)) return fail(MI_ERR_STRIDE, "q/k/v/o strides must be multiples of 8 elements (got %lld)", (long long)x);
  // the tile loads address a 64-key tile as scalar base + 32-bit lane offset
  if (a->k_stride_s < 0 || a->v_stride_s < 0 || a->k_stride_s >= (1 << 24) || a->v_stride_s >= (1 << 24))
    return fail(MI_ERR_STRIDE, "k/v sequence strides must be in [0, 2^24) elements (got %lld, %lld)",
                (long long)a->k_stride_s, (long long)a->v_stride_s);
  if (!a->cu_seqlens) {
    const int64_t sb[] = {a->q_stride_b, a->k_stride_b, a->v_stride_b, a->o_stride_b};
    for (int64_t x : sb)
      if (!mult8(x)) return fail(MI_ERR_STRIDE, "batch strides must be multiples of 8 elements (got %lld)", (long long)x);
  }
  return MI_OK;
}

template <typename A>
void fill_prefill(const A* a, mi::PrefillParams& p, int rows_per_wg) {
  std::memset(&p, 0, sizeof(p));
  p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o; p.lse = a->lse;
  p.q_sb = a->q_stride_b; p.q_ss = a->q_stride_s; p.q_sh = a->q_stride_h;
  p.k_sb = a->k_stride_b; p.k_ss = a->k_stride_s; p.k_sh = a->k_stride_h;
  p.v_sb = a->v_stride_b; p.v_ss = a->v_stride_s; p.v_sh = a->v_stride_h;
  p.o_sb = a->o_stride_b; p.o_ss = a->o_stride_s; p.o_sh = a->o_stride_h;
  p.lse_sb = a->lse_stride_b; p.lse_ss = a->lse_stride_s; p.lse_sh = a->lse_stride_h;
  p.cu = a->cu_seqlens;
  p.batch = a->batch; p.hq = a->heads_q; p.hkv = a->heads_kv; p.max_seqlen = a->max_seqlen;
  p.n_qtiles = (int)(((long long)a->max_seqlen + rows_per_wg - 1) / rows_per_wg);
  p.scale = a->scale_log2;
  p.win_local = -1; p.win_global = -1;
}

bool decode_listed(const mi_decode_args* a) { return a->block_idx != nullptr || a->window_form == 1; }

int decode_splits(const mi_decode_args* a) {
  if (decode_listed(a)) return (a->max_blocks + ((a->include_last_block && a->window_form != 1) ? 1 : 0) + a->split_blocks - 1) / a->split_blocks;
  return (a->max_seqlen + a->split_tokens - 1) / a->split_tokens;
}

void fill_decode(const mi_decode_args* a, mi::DecodeParams& p) {
  std::memset(&p, 0, sizeof(p));
  p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o; p.lse = a->lse;
  p.q_sb = a->q_stride_b; p.q_sh = a->q_stride_h;
  p.k_sb = a->k_stride_b; p.k_ss = a->k_stride_s; p.k_sh = a->k_stride_h;
  p.v_sb = a->v_stride_b; p.v_ss = a->v_stride_s; p.v_sh = a->v_stride_h;
  p.o_sb = a->o_stride_b; p.o_sh = a->o_stride_h;
  p.seq_lens = a->seq_lens; p.cu = a->cu_seqlens;
  p.batch = a->batch; p.hq = a->heads_q; p.hkv = a->heads_kv; p.max_seqlen = a->max_seqlen;
  p.scale = a->scale_log2;
  p.split_tokens = a->split_tokens;
  p.n_splits = decode_splits(a);
  p.part_o = static_cast<float*>(a->workspace);
  p.part_lse = p.part_o + (size_t)a->batch * a->heads_q * p.n_splits * a->head_dim;
  p.gslices = (a->heads_q / a->heads_kv + 31) / 32;
  const bool listed = decode_listed(a);
  p.list_mode = a->window_form == 1 ? 2 : (a->block_idx ? 1 : 0);
  p.block_idx = a->block_idx; p.block_cnt = a->block_cnt;
  p.bi_sb = a->block_idx_stride_b; p.bi_sh = a->block_idx_stride_h;
  p.max_blocks = a->max_blocks; p.split_blocks = a->split_blocks;
  p.win_local = listed ? a->window_local : -1;
  p.win_global = listed ? a->window_global : -1;
  p.add_last = (p.list_mode == 1 && a->include_last_block) ? 1 : 0;
  if (!listed) { p.max_blocks = 0; p.split_blocks = 1; }
  p.kv_layout = a->kv_layout; p.page_size = a->page_size;
  p.page_table = a->page_table; p.pt_sb = a->page_table_stride_b;
}

int launch_status(int hip_err, const char* what) {
  if (hip_err == 0) return MI_OK;
  return fail(MI_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(static_cast<hipError_t>(hip_err)));
}

// total_rows > 0: zero the rows of o and lse that belong to no sequence
template <typename A>
int zero_uncovered(const A* a, hipStream_t s) {
  if (a->total_rows <= 0) return MI_OK;
  mi::RowFillParams f;
  std::memset(&f, 0, sizeof(f));
  f.cu = a->cu_seqlens; f.batch = a->batch; f.total_rows = a->total_rows; f.max_seqlen = a->max_seqlen;
  f.t[f.n_tensors++] = fill_of(a->o, a->o_stride_s, a->o_stride_h, a->heads_q, 2, a->head_dim);
  if (a->lse) f.t[f.n_tensors++] = fill_of(a->lse, a->lse_stride_s, a->lse_stride_h, a->heads_q, 4, 1);
  return launch_status(mi::launch_zero_uncovered_rows(f, s), "zero fill of rows outside every sequence");
}

}  // namespace

namespace mi {
int set_error(int code, const char* msg) { return fail(code, "%s", msg); }
}  // namespace mi

extern "C" {

int mi_abi_version(void) { return MI_ATTN_ABI_VERSION; }
const char* mi_last_error(void) { return g_err; }

const char* mi_status_name(int status) {
  switch (status) {
    case MI_OK: return "MI_OK";
    case MI_ERR_NULL_POINTER: return "MI_ERR_NULL_POINTER";
    case MI_ERR_STRUCT_SIZE: return "MI_ERR_STRUCT_SIZE";
    case MI_ERR_DTYPE: return "MI_ERR_DTYPE";
    case MI_ERR_HEAD_DIM: return "MI_ERR_HEAD_DIM";
    case MI_ERR_GQA: return "MI_ERR_GQA";
    case MI_ERR_SHAPE: return "MI_ERR_SHAPE";
    case MI_ERR_STRIDE: return "MI_ERR_STRIDE";
    case MI_ERR_ALIGNMENT: return "MI_ERR_ALIGNMENT";
    case MI_ERR_SCALE: return "MI_ERR_SCALE";
    case MI_ERR_WORKSPACE: return "MI_ERR_WORKSPACE";
    case MI_ERR_SPARSE_LAYOUT: return "MI_ERR_SPARSE_LAYOUT";
    case MI_ERR_LAUNCH: return "MI_ERR_LAUNCH";
    case MI_ERR_NO_DEVICE: return "MI_ERR_NO_DEVICE";
  }
  return "MI_ERR_UNKNOWN";
}

int mi_attn_fwd_validate(const mi_attn_fwd_args* a) {
  if (!a) return fail(MI_ERR_NULL_POINTER, "args is NULL");
  if (a->struct_size != sizeof(mi_attn_fwd_args))
    return fail(MI_ERR_STRUCT_SIZE, "mi_attn_fwd_args.struct_size %u != %zu", a->struct_size, sizeof(mi_attn_fwd_args));
  int rc = check_common(a->dtype, a->head_dim, a->batch, a->heads_q, a->heads_kv, a->max_seqlen, a->scale_log2);
  if (rc) return rc;
  if ((rc = check_qkvo(a))) return rc;
  if ((rc = check_prefill_strides(a))) return rc;
  if (a->causal != 0 && a->causal != 1) return fail(MI_ERR_SHAPE, "causal must be 0 or 1");
  if (a->total_rows < 0) return fail(MI_ERR_SHAPE, "total_rows %d is negative", a->total_rows);
  if (a->total_rows > 0 && !a->cu_seqlens) return fail(MI_ERR_SHAPE, "total_rows is for the packed form (cu_seqlens != NULL)");
  if (a->dense_form < MI_DENSE_FORM_AUTO || a->dense_form > MI_DENSE_FORM_128_ROWS)
    return fail(MI_ERR_SHAPE, "dense_form %d is none of MI_DENSE_FORM_AUTO / _256_ROWS / _128_ROWS", a->dense_form);
  // (work item ids are 32-bit and the persistent kernels step them by their grid size)
  const long long wgs = (((long long)a->max_seqlen + mi::kShortRows - 1) / mi::kShortRows) * a->heads_q * a->batch;
  if (wgs > 0x3fffffffLL) return fail(MI_ERR_SHAPE, "%lld work items are too many", wgs);
  return MI_OK;
}

static int rms_elem_bytes(int dt) { return dt == MI_DTYPE_F32 ? 4 : 2; }

static int rms_validate(const mi_rmsnorm_args* a, bool backward) {
  if (!a) return fail(MI_ERR_NULL_POINTER, "args is NULL");
  if (a->struct_size != sizeof(mi_rmsnorm_args))
    return fail(MI_ERR_STRUCT_SIZE, "mi_rmsnorm_args.struct_size %u != %zu", a->struct_size, sizeof(mi_rmsnorm_args));
  if (a->x_dtype != MI_DTYPE_BF16 && a->x_dtype != MI_DTYPE_F16 && a->x_dtype != MI_DTYPE_F32)
    return fail(MI_ERR_DTYPE, "x_dtype %d is not bf16 / f16 / f32", a->x_dtype);
  if (a->w_dtype != a->x_dtype && a->w_dtype != MI_DTYPE_F32)
    return fail(MI_ERR_DTYPE, "w_dtype %d must equal x_dtype or be f32", a->w_dtype);
  if (a->dim <= 0 || a->rows < 0) return fail(MI_ERR_SHAPE, "dim %d must be positive, rows %lld non-negative", a->dim, (long long)a->rows);
  if (!(a->eps >= 0.f) || !std::isfinite(a->eps)) return fail(MI_ERR_SCALE, "eps must be finite and >= 0");
  if (a->rows == 0) return MI_OK;
  if (a->rows > 0x7fffffffLL * 4) return fail(MI_ERR_SHAPE, "too many rows");
  if (!a->x || !a->w || !a->rsqrt) return fail(MI_ERR_NULL_POINTER, "x, w and rsqrt must be non-NULL");
  if (a->x_stride < a->dim) return fail(MI_ERR_STRIDE, "x row stride %lld < dim", (long long)a->x_stride);
  if (!backward) {
    if (!a->y) return fail(MI_ERR_NULL_POINTER, "y must be non-NULL");
    if (a->y_stride < a->dim) return fail(MI_ERR_STRIDE, "y row stride %lld < dim", (long long)a->y_stride);
  } else {
    if (!a->dy || !a->dx || !a->dw) return fail(MI_ERR_NULL_POINTER, "dy, dx and dw must be non-NULL");
    if (a->dy_stride < a->dim || a->dx_stride < a->dim) return fail(MI_ERR_STRIDE, "dy / dx row stride < dim");
    if (!a->workspace || a->workspace_bytes < mi_rmsnorm_bwd_workspace_bytes(a))
      return fail(MI_ERR_WORKSPACE, "workspace of %zu bytes needed", mi_rmsnorm_bwd_workspace_bytes(a));
  }
  return MI_OK;
}

// 16-byte chunk path: dim and row strides multiples of the chunk, 16-byte aligned bases, <= 16 chunks per lane
static bool rms_vec_ok(const mi_rmsnorm_args* a, bool backward) {
  const int epc = 16 / rms_elem_bytes(a->x_dtype);
  // chunks per row: 16 per thread of a workgroup; 8 in the backward pass, whose
  // per-position dw sums share the registers
  if (a->dim % epc || a->dim / epc > 256 * (backward ? 8 : 16)) return false;
  if (!aligned16(a->x) || a->x_stride % epc) return false;
  if (!backward) return aligned16(a->y) && a->y_stride % epc == 0;
  return aligned16(a->dy) && aligned16(a->dx) && a->dy_stride % epc == 0 && a->dx_stride % epc == 0;
}

static void rms_fill(const mi_rmsnorm_args* a, mi::RmsParams& p) {
  std::memset(&p, 0, sizeof(p));
  p.x = a->x; p.w = a->w; p.dy = a->dy; p.y = a->y; p.dx = a->dx; p.dw = a->dw;
  p.rsqrt = a->rsqrt; p.dw_part = static_cast<float*>(a->workspace);
  p.x_st = a->x_stride; p.y_st = a->y_stride; p.dy_st = a->dy_stride; p.dx_st = a->dx_stride;
  p.rows = a->rows; p.dim = a->dim; p.eps = a->eps;
}

int mi_rmsnorm_fwd(const mi_rmsnorm_args* a, void* stream) {
  int rc = rms_validate(a, false);
  if (rc) return rc;
  if (a->rows == 0) return MI_OK;
  mi::RmsParams p;
  rms_fill(a, p);
  return launch_status(mi::launch_rms_fwd(p, a->x_dtype, a->w_dtype, rms_vec_ok(a, false), mi::rms_partial_rows(a->rows, 256),
                                          static_cast<hipStream_t>(stream)),
                       "mi_rmsnorm_fwd");
}

size_t mi_rmsnorm_bwd_workspace_bytes(const mi_rmsnorm_args* a) {
  if (!a || a->dim <= 0 || a->rows <= 0) return 0;
  return (size_t)(mi::rms_partial_rows(a->rows, 256) + mi::kRmsStageRows) * (size_t)a->dim * sizeof(float);
}

int mi_rmsnorm_bwd(const mi_rmsnorm_args* a, void* stream) {
  int rc = rms_validate(a, true);
  if (rc) return rc;
  if (a->rows == 0) return MI_OK;   // dw of an empty batch is left to the caller
  mi::RmsParams p;
  rms_fill(a, p);
  return launch_status(mi::launch_rms_bwd(p, a->x_dtype, a->w_dtype, rms_vec_ok(a, true), mi::rms_partial_rows(a->rows, 256),
                                          static_cast<hipStream_t>(stream)),
                       "mi_rmsnorm_bwd");
}

static int xent_validate(const mi_xent_args* a) {
  if (!a) return fail(MI_ERR_NULL_POINTER, "args is NULL");
  if (a->struct_size != sizeof(mi_xent_args))
    return fail(MI_ERR_STRUCT_SIZE, "mi_xent_args.struct_size %u != %zu", a->struct_size, sizeof(mi_xent_args));
  if (a->dtype != MI_DTYPE_BF16 && a->dtype != MI_DTYPE_F16) return fail(MI_ERR_DTYPE, "dtype %d is not bf16 / f16", a->dtype);
  if (a->tokens < 0 || a->dim <= 0 || a->vocab <= 0)
    return fail(MI_ERR_SHAPE, "tokens %d must be >= 0, dim %d and vocab %d positive", a->tokens, a->dim, a->vocab);
  if (a->dim % 128) return fail(MI_ERR_SHAPE, "dim %d must be a multiple of 128 (pad with zero columns)", a->dim);
  if (a->labels_i64 != 0 && a->labels_i64 != 1) return fail(MI_ERR_SHAPE, "labels_i64 must be 0 or 1");
  if (a->tokens == 0) return MI_OK;
  if (!a->x || !a->w || !a->y || !a->lse || !a->loss)
    return fail(MI_ERR_NULL_POINTER, "x, w, y, lse and loss must be non-NULL");
  if (!aligned16(a->x) || !aligned16(a->w)) return fail(MI_ERR_ALIGNMENT, "x and w must be 16-byte aligned");
  if (a->x_stride < a->dim || a->w_stride < a->dim || a->x_stride % 8 || a->w_stride % 8)
    return fail(MI_ERR_STRIDE, "row strides must be >= dim and multiples of 8 elements");
  // per-lane row offsets inside a 256-row slab are 32-bit
  if (a->x_stride > (1 << 22) || a->w_stride > (1 << 22)) return fail(MI_ERR_STRIDE, "row stride beyond 2^22 elements");
  if (!a->workspace || a->workspace_bytes < mi_xent_fwd_workspace_bytes(a))
    return fail(MI_ERR_WORKSPACE, "workspace of %zu bytes needed", mi_xent_fwd_workspace_bytes(a));
  return MI_OK;
}

size_t mi_xent_fwd_workspace_bytes(const mi_xent_args* a) {
  if (!a || a->tokens <= 0 || a->vocab <= 0) return 0;
  return (size_t)a->tokens * (size_t)mi::xent_choose_splits(a->tokens, a->vocab, 256) * 2 * sizeof(float);
}

int mi_xent_fwd(const mi_xent_args* a, void* stream) {
  int rc = xent_validate(a);
  if (rc) return rc;
  if (a->tokens == 0) return MI_OK;
  mi::XentParams p;
  std::memset(&p, 0, sizeof(p));
  p.x = a->x; p.w = a->w; p.y = a->y; p.y_is_i64 = a->labels_i64;
  p.x_st = a->x_stride; p.w_st = a->w_stride;
  p.T = a->tokens; p.D = a->dim; p.N = a->vocab;
  p.n_split = mi::xent_choose_splits(a->tokens, a->vocab, 256);
  p.lse_part = static_cast<float*>(a->workspace);
  p.tgt_part = p.lse_part + (size_t)a->tokens * p.n_split;
  p.lse = a->lse; p.loss = a->loss;
  return launch_status(mi::launch_xent_fwd(p, a->dtype, false, static_cast<hipStream_t>(stream)), "mi_xent_fwd");
}

int mi_xent_bwd_dlogits(const mi_xent_bwd_args* a, void* stream) {
  if (!a) return fail(MI_ERR_NULL_POINTER, "args is NULL");
  if (a->struct_size != sizeof(mi_xent_bwd_args))
    return fail(MI_ERR_STRUCT_SIZE, "mi_xent_bwd_args.struct_size %u != %zu", a->struct_size, sizeof(mi_xent_bwd_args));
  if (a->dtype != MI_DTYPE_BF16 && a->dtype != MI_DTYPE_F16) return fail(MI_ERR_DTYPE, "dtype %d is not bf16 / f16", a->dtype);
  if (a->tokens < 0 || a->dim <= 0 || a->vocab <= 0)
    return fail(MI_ERR_SHAPE, "tokens %d must be >= 0, dim %d and vocab %d positive", a->tokens, a->dim, a->vocab);
  if (a->dim % 128) return fail(MI_ERR_SHAPE, "dim %d must be a multiple of 128 (pad with zero columns)", a->dim);
  if (a->labels_i64 != 0 && a->labels_i64 != 1) return fail(MI_ERR_SHAPE, "labels_i64 must be 0 or 1");
  if (a->tokens == 0) return MI_OK;
  if (!a->x || !a->w || !a->y || !a->lse || !a->dloss || !a->dlogits)
    return fail(MI_ERR_NULL_POINTER, "x, w, y, lse, dloss and dlogits must be non-NULL");
  if (!aligned16(a->x) || !aligned16(a->w)) return fail(MI_ERR_ALIGNMENT, "x and w must be 16-byte aligned");
  if (a->x_stride < a->dim || a->w_stride < a->dim || a->x_stride % 8 || a->w_stride % 8)
    return fail(MI_ERR_STRIDE, "row strides must be >= dim and multiples of 8 elements");
  if (a->x_stride > (1 << 22) || a->w_stride > (1 << 22)) return fail(MI_ERR_STRIDE, "row stride beyond 2^22 elements");
  if (a->ld < a->vocab) return fail(MI_ERR_STRIDE, "ld %lld < vocab", (long long)a->ld);
  mi::XentParams p;
  std::memset(&p, 0, sizeof(p));
  p.x = a->x; p.w = a->w; p.y = a->y; p.y_is_i64 = a->labels_i64;
  p.x_st = a->x_stride; p.w_st = a->w_stride;
  p.T = a->tokens; p.D = a->dim; p.N = a->vocab;
  p.n_split = mi::xent_choose_splits(a->tokens, a->vocab, 256);
  p.lse = const_cast<float*>(a->lse); p.dloss = a->dloss;
  p.dlogits = a->dlogits; p.dl_ld = a->ld;
  p.dl_vec = aligned16(a->dlogits) && a->ld % 8 == 0;
  return launch_status(mi::launch_xent_fwd(p, a->dtype, true, static_cast<hipStream_t>(stream)), "mi_xent_bwd_dlogits");
}

int mi_xent_dlogits(const mi_xent_grad_args* a, void* stream) {
  if (!a) return fail(MI_ERR_NULL_POINTER, "args is NULL");
  if (a->struct_size != sizeof(mi_xent_grad_args))
    return fail(MI_ERR_STRUCT_SIZE, "mi_xent_grad_args.struct_size %u != %zu", a->struct_size, sizeof(mi_xent_grad_args));
  if (a->dtype != MI_DTYPE_BF16 && a->dtype != MI_DTYPE_F16) return fail(MI_ERR_DTYPE, "dtype %d is not bf16 / f16", a->dtype);
  if (a->rows < 0 || a->vocab <= 0 || a->rows > 0x7fffffffLL)
    return fail(MI_ERR_SHAPE, "rows %lld must be in [0, 2^31), vocab %d positive", (long long)a->rows, a->vocab);
  if (a->labels_i64 != 0 && a->labels_i64 != 1) return fail(MI_ERR_SHAPE, "labels_i64 must be 0 or 1");
  if (a->rows == 0) return MI_OK;
  if (!a->logits || !a->lse || !a->dloss || !a->y) return fail(MI_ERR_NULL_POINTER, "logits, lse, dloss and y must be non-NULL");
  if (a->ld < a->vocab) return fail(MI_ERR_STRIDE, "ld %lld < vocab", (long long)a->ld);
  mi::XentGradParams p;
  std::memset(&p, 0, sizeof(p));
  p.logits = a->logits; p.lse = a->lse; p.dloss = a->dloss; p.y = a->y;
  p.ld = a->ld; p.rows = a->rows; p.N = a->vocab; p.y_is_i64 = a->labels_i64;
  p.vec = aligned16(a->logits) && a->ld % 8 == 0;
  return launch_status(mi::launch_xent_dlogits(p, a->dtype, static_cast<hipStream_t>(stream)), "mi_xent_dlogits");
}

int mi_attn_bwd_validate(const mi_attn_bwd_args* a) {
  if (!a) return fail(MI_ERR_NULL_POINTER, "args is NULL");
  if (a->struct_size != sizeof(mi_attn_bwd_args))
    return fail(MI_ERR_STRUCT_SIZE, "mi_attn_bwd_args.struct_size %u != %zu", a->struct_size, sizeof(mi_attn_bwd_args));
  int rc = check_common(a->dtype, a->head_dim, a->batch, a->heads_q, a->heads_kv, a->max_seqlen, a->scale_log2);
  if (rc) return rc;
  if (a->total_rows < 0) return fail(MI_ERR_SHAPE, "total_rows %d is negative", a->total_rows);
  if (a->total_rows > 0 && !a->cu_seqlens) return fail(MI_ERR_SHAPE, "total_rows is for the packed form (cu_seqlens != NULL)");
  if (a->max_seqlen == 0 && a->total_rows == 0) return MI_OK;
  const void* ptrs[] = {a->q, a->k, a->v, a->o, a->dout, a->lse, a->dq, a->dk, a->dv};
  for (const void* x : ptrs)
    if (!x) return fail(MI_ERR_NULL_POINTER, "q, k, v, o, dout, lse, dq, dk and dv must be non-NULL");
  const void* al[] = {a->q, a->k, a->v, a->o, a->dout, a->dq, a->dk, a->dv};
  for (const void* x : al)
    if (!aligned16(x)) return fail(MI_ERR_ALIGNMENT, "q, k, v, o, dout, dq, dk and dv must be 16-byte aligned");
  const int64_t st[] = {a->q_stride_s, a->q_stride_h, a->k_stride_s, a->k_stride_h, a->v_stride_s, a->v_stride_h,
                        a->o_stride_s, a->o_stride_h, a->dout_stride_s, a->dout_stride_h, a->dq_stride_s,
                        a->dq_stride_h, a->dk_stride_s, a->dk_stride_h, a->dv_stride_s, a->dv_stride_h};
  for (int64_t x : st)
    if (!mult8(x)) return fail(MI_ERR_STRIDE, "tensor strides must be multiples of 8 elements (got %lld)", (long long)x);
  // a streamed 64-row tile is addressed as uniform base + 32-bit byte offset per lane
  const int64_t ss[] = {a->q_stride_s, a->k_stride_s, a->v_stride_s, a->dout_stride_s, a->lse_stride_s};
  for (int64_t x : ss)
    if (x < 0 || x >= (1 << 24))
      return fail(MI_ERR_STRIDE, "q/k/v/dout/lse sequence strides must be in [0, 2^24) elements (got %lld)", (long long)x);
  if (!a->cu_seqlens) {
    const int64_t sb[] = {a->q_stride_b, a->k_stride_b, a->v_stride_b, a->o_stride_b, a->dout_stride_b,
                          a->dq_stride_b, a->dk_stride_b, a->dv_stride_b};
    for (int64_t x : sb)
      if (!mult8(x)) return fail(MI_ERR_STRIDE, "batch strides must be multiples of 8 elements (got %lld)", (long long)x);
  }
  if (a->causal != 0 && a->causal != 1) return fail(MI_ERR_SHAPE, "causal must be 0 or 1");
  const long long wgs = (long long)((a->max_seqlen + 255) / 256) * a->heads_q * a->batch;
  if (wgs > 0x7fffffffLL || a->heads_q > 65535 || a->batch > 65535)
    return fail(MI_ERR_SHAPE, "launch grid too large");
  if (a->max_seqlen > 0) {
    if (!a->workspace || a->workspace_bytes < mi_attn_bwd_workspace_bytes(a))
      return fail(MI_ERR_WORKSPACE, "workspace of %zu bytes needed", mi_attn_bwd_workspace_bytes(a));
    if (!aligned16(a->workspace)) return fail(MI_ERR_ALIGNMENT, "workspace must be 16-byte aligned");
  }
  return MI_OK;
}

size_t mi_attn_bwd_workspace_bytes(const mi_attn_bwd_args* a) {
  if (!a || a->batch <= 0 || a->heads_q <= 0 || a->max_seqlen <= 0) return 0;
  return (size_t)a->batch * a->heads_q * (size_t)a->max_seqlen * sizeof(float);
}

int mi_attn_bwd(const mi_attn_bwd_args* a, void* stream) {
  int rc = mi_attn_bwd_validate(a);
  if (rc) return rc;
  if (a->total_rows > 0) {
    mi::RowFillParams f;
    std::memset(&f, 0, sizeof(f));
    f.cu = a->cu_seqlens; f.batch = a->batch; f.total_rows = a->total_rows; f.max_seqlen = a->max_seqlen;
    f.t[f.n_tensors++] = fill_of(a->dq, a->dq_stride_s, a->dq_stride_h, a->heads_q, 2, a->head_dim);
    f.t[f.n_tensors++] = fill_of(a->dk, a->dk_stride_s, a->dk_stride_h, a->heads_kv, 2, a->head_dim);
    f.t[f.n_tensors++] = fill_of(a->dv, a->dv_stride_s, a->dv_stride_h, a->heads_kv, 2, a->head_dim);
    if ((rc = launch_status(mi::launch_zero_uncovered_rows(f, static_cast<hipStream_t>(stream)),
                            "zero fill of rows outside every sequence")))
      return rc;
  }
  if (a->max_seqlen == 0) return MI_OK;
  mi::BwdParams p;
  std::memset(&p, 0, sizeof(p));
  p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o; p.dout = a->dout; p.lse = a->lse;
  p.delta = static_cast<float*>(a->workspace);
  p.dq = a->dq; p.dk = a->dk; p.dv = a->dv;
  p.q_sb = a->q_stride_b; p.q_ss = a->q_stride_s; p.q_sh = a->q_stride_h;
  p.k_sb = a->k_stride_b; p.k_ss = a->k_stride_s; p.k_sh = a->k_stride_h;
  p.v_sb = a->v_stride_b; p.v_ss = a->v_stride_s; p.v_sh = a->v_stride_h;
  p.o_sb = a->o_stride_b; p.o_ss = a->o_stride_s; p.o_sh = a->o_stride_h;
  p.do_sb = a->dout_stride_b; p.do_ss = a->dout_stride_s; p.do_sh = a->dout_stride_h;
  p.dq_sb = a->dq_stride_b; p.dq_ss = a->dq_stride_s; p.dq_sh = a->dq_stride_h;
  p.dk_sb = a->dk_stride_b; p.dk_ss = a->dk_stride_s; p.dk_sh = a->dk_stride_h;
  p.dv_sb = a->dv_stride_b; p.dv_ss = a->dv_stride_s; p.dv_sh = a->dv_stride_h;
  p.lse_sb = a->lse_stride_b; p.lse_ss = a->lse_stride_s; p.lse_sh = a->lse_stride_h;
  p.dl_sh = a->max_seqlen; p.dl_sb = (int64_t)a->heads_q * a->max_seqlen;
  p.cu = a->cu_seqlens;
  p.batch = a->batch; p.hq = a->heads_q; p.hkv = a->heads_kv; p.max_seqlen = a->max_seqlen;
  p.n_rtiles = (a->max_seqlen + 255) / 256;
  p.causal = a->causal;
  p.scale = a->scale_log2;
  p.scale_nat = a->scale_log2 * 0.6931471805599453f;
  return launch_status(mi::launch_attn_bwd(p, a->dtype, a->head_dim, static_cast<hipStream_t>(stream)), "mi_attn_bwd");
}

int mi_attn_fwd(const mi_attn_fwd_args* a, void* stream) {
  int rc = mi_attn_fwd_validate(a);
  if (rc) return rc;
  if ((rc = zero_uncovered(a, static_cast<hipStream_t>(stream)))) return rc;
  if (a->max_seqlen == 0) return MI_OK;
  mi::PrefillParams p;
  fill_prefill(a, p, mi::kDenseRows);
  p.causal = a->causal;
  p.dense_form = a->dense_form;
  return launch_status(mi::launch_prefill_dense(p, a->dtype, a->head_dim, static_cast<hipStream_t>(stream)), "mi_attn_fwd");
}

int mi_attn_fwd_blocksparse_validate(const mi_attn_sparse_args* a) {
  if (!a) return fail(MI_ERR_NULL_POINTER, "args is NULL");
  if (a->struct_size != sizeof(mi_attn_sparse_args))
    return fail(MI_ERR_STRUCT_SIZE, "mi_attn_sparse_args.struct_size %u != %zu", a->struct_size, sizeof(mi_attn_sparse_args));
  int rc = check_common(a->dtype, a->head_dim, a->batch, a->heads_q, a->heads_kv, a->max_seqlen, a->scale_log2);
  if (rc) return rc;
  if ((rc = check_qkvo(a))) return rc;
  if ((rc = check_prefill_strides(a))) return rc;
  if ((a->row_ptr == nullptr) != (a->col_idx == nullptr))
    return fail(MI_ERR_NULL_POINTER, "row_ptr and col_idx must both be given or both be NULL");
  if (a->block_size != MI_ATTN_BLOCK) return fail(MI_ERR_SPARSE_LAYOUT, "block_size %d must be %d", a->block_size, MI_ATTN_BLOCK);
  if (a->row_ptr_stride_b < 0 || a->row_ptr_stride_h < 0 || a->col_idx_stride_b < 0 || a->col_idx_stride_h < 0)
    return fail(MI_ERR_SPARSE_LAYOUT, "mask strides must be >= 0");
  if ((a->window_local < 0) != (a->window_global < 0) || a->window_local < -1 || a->window_global < -1)
    return fail(MI_ERR_SPARSE_LAYOUT, "window_local/window_global must both be -1 or both be >= 0");
  // no lists: the token-window form, whose blocks follow from the two windows
  if (!a->row_ptr && (a->window_local < 1 || a->window_global < 0))
    return fail(MI_ERR_NULL_POINTER, "without row_ptr / col_idx the call needs window_local >= 1 and window_global >= 0 (got %d, %d)",
                a->window_local, a->window_global);
  if (a->total_rows < 0) return fail(MI_ERR_SHAPE, "total_rows %d is negative", a->total_rows);
  if (a->total_rows > 0 && !a->cu_seqlens) return fail(MI_ERR_SHAPE, "total_rows is for the packed form (cu_seqlens != NULL)");
  const long long wgs = (((long long)a->max_seqlen + mi::kSparseRows - 1) / mi::kSparseRows) * a->heads_q * a->batch;
  if (wgs > 0x7fffffffLL) return fail(MI_ERR_SHAPE, "grid of %lld workgroups is too large", wgs);
  return MI_OK;
}

int mi_attn_fwd_blocksparse(const mi_attn_sparse_args* a, void* stream) {
  int rc = mi_attn_fwd_blocksparse_validate(a);
  if (rc) return rc;
  if ((rc = zero_uncovered(a, static_cast<hipStream_t>(stream)))) return rc;
  if (a->max_seqlen == 0) return MI_OK;
  mi::PrefillParams p;
  if (!a->row_ptr) {
    fill_prefill(a, p, mi::kShortRows);
    p.causal = 1;
    // (a window as long as the longest sequence already is the whole sequence)
    p.win_local = std::min(a->window_local, a->max_seqlen); p.win_global = std::min(a->window_global, a->max_seqlen);
    return launch_status(mi::launch_prefill_window(p, a->dtype, a->head_dim, static_cast<hipStream_t>(stream)), "mi_attn_fwd_blocksparse");
  }
  fill_prefill(a, p, mi::kSparseRows);
  p.causal = 1;
  p.row_ptr = a->row_ptr; p.col_idx = a->col_idx;
  p.rp_sb = a->row_ptr_stride_b; p.rp_sh = a->row_ptr_stride_h;
  p.ci_sb = a->col_idx_stride_b; p.ci_sh = a->col_idx_stride_h;
  // (-1 stays -1; a window as long as the longest sequence already is the whole sequence)
  p.win_local = std::min(a->window_local, a->max_seqlen); p.win_global = std::min(a->window_global, a->max_seqlen);
  return launch_status(mi::launch_prefill_sparse(p, a->dtype, a->head_dim, static_cast<hipStream_t>(stream)), "mi_attn_fwd_blocksparse");
}

static_assert(mi::kDecodeScratchBytes == MI_DECODE_STATIC_SCRATCH_BYTES, "header and kernel disagree on the static buffer");

static int decode_validate_shape(const mi_decode_args* a) {
  if (!a) return fail(MI_ERR_NULL_POINTER, "args is NULL");
  if (a->struct_size != sizeof(mi_decode_args))
    return fail(MI_ERR_STRUCT_SIZE, "mi_decode_args.struct_size %u != %zu", a->struct_size, sizeof(mi_decode_args));
  int rc = check_common(a->dtype, a->head_dim, a->batch, a->heads_q, a->heads_kv, a->max_seqlen, a->scale_log2);
  if (rc) return rc;
  if (a->window_form != 0 && a->window_form != 1) return fail(MI_ERR_SPARSE_LAYOUT, "window_form must be 0 or 1");
  if (a->window_form == 1) {
    if (a->block_size != MI_ATTN_BLOCK) return fail(MI_ERR_SPARSE_LAYOUT, "block_size %d must be %d", a->block_size, MI_ATTN_BLOCK);
    if (a->window_local < 0 || a->window_global < 0)
      return fail(MI_ERR_SPARSE_LAYOUT, "the window form needs window_local and window_global >= 0");
    const long long need = ((long long)a->window_global + 63) / 64 + ((long long)a->window_local + 63) / 64 + 1;
    if (a->max_blocks < need || a->split_blocks <= 0)
      return fail(MI_ERR_SPARSE_LAYOUT, "the window form needs max_blocks >= %lld (got %d) and split_blocks > 0 (got %d)",
                  need, a->max_blocks, a->split_blocks);
  } else if (a->block_idx) {
    if (a->block_size != MI_ATTN_BLOCK) return fail(MI_ERR_SPARSE_LAYOUT, "block_size %d must be %d", a->block_size, MI_ATTN_BLOCK);
    if (a->include_last_block != 0 && a->include_last_block != 1)
      return fail(MI_ERR_SPARSE_LAYOUT, "include_last_block must be 0 or 1");
    // an empty list is a valid one when the implicit last block is attended
    if (a->max_blocks < 0 || a->max_blocks + a->include_last_block <= 0 || a->split_blocks <= 0)
      return fail(MI_ERR_SPARSE_LAYOUT, "max_blocks %d (+ the implicit last block) and split_blocks %d must be positive",
                  a->max_blocks, a->split_blocks);
    if (a->block_idx_stride_b < 0 || a->block_idx_stride_h < 0)
      return fail(MI_ERR_SPARSE_LAYOUT, "block_idx strides must be >= 0");
    if ((a->window_local < 0) != (a->window_global < 0) || a->window_local < -1 || a->window_global < -1)
      return fail(MI_ERR_SPARSE_LAYOUT, "window_local/window_global must both be -1 or both be >= 0");
  } else {
    if (a->split_tokens <= 0 || a->split_tokens % 64 != 0)
      return fail(MI_ERR_WORKSPACE, "split_tokens %d must be a positive multiple of 64", a->split_tokens);
  }
  if (a->kv_layout != MI_KV_BATCHED && a->kv_layout != MI_KV_PACKED && a->kv_layout != MI_KV_PAGED)
    return fail(MI_ERR_SHAPE, "kv_layout %d is not MI_KV_BATCHED / MI_KV_PACKED / MI_KV_PAGED", a->kv_layout);
  if (a->kv_layout == MI_KV_PAGED && (a->page_size <= 0 || a->page_size % 32 != 0 || a->page_table_stride_b < 0))
    return fail(MI_ERR_SHAPE, "paged KV needs page_size a positive multiple of 32 (got %d) and a page table stride >= 0",
                a->page_size);
  if (decode_splits(a) > 65535) return fail(MI_ERR_WORKSPACE, "more than 65535 splits per sequence");
  if ((long long)a->heads_kv * ((a->heads_q / a->heads_kv + 31) / 32) > 65535 || a->batch > 65535 || a->heads_q > 0x7fffffff / 2)
    return fail(MI_ERR_SHAPE, "batch / head count exceeds the launch grid limits");
  return MI_OK;
}

int mi_decode_num_splits(const mi_decode_args* a) {
  int rc = decode_validate_shape(a);
  if (rc) return rc;
  return decode_splits(a);
}

size_t mi_decode_workspace_bytes(const mi_decode_args* a) {
  if (decode_validate_shape(a)) return 0;
  return (size_t)a->batch * a->heads_q * decode_splits(a) * (a->head_dim + 1) * sizeof(float);
}

int mi_decode_choose_split_tokens(int batch, int heads_kv, int max_seqlen, int num_cus) {
  // The dense kernel deals the live chunks to one resident round of wavefronts
  // (8 per CU).  Chunks of about half a round's share keep every wavefront's
  // fixed costs (first tile, partial results, merge) small against its stream;
  // beyond 2048 tokens nothing is gained, and the shortest chunk worth a
  // partial result is 512 tokens, or 256 where that still leaves a sequence in
  // no more than 32 chunks for the merge (measured on 1 to 64 sequences of 8k,
  // 32k and 128k tokens: 1 to 4 sequences of 8k take 29 to 36 us with chunks of
  // 256 tokens against 36 to 43 us with 512, one sequence of 32k 63 against 55).
  if (batch <= 0 || heads_kv <= 0 || max_seqlen <= 0) return 64;
  if (num_cus <= 0) num_cus = 256;
  const long long work = (long long)batch * heads_kv * max_seqlen;  // tokens x kv-heads
  long long tokens = 2 * work / (8LL * num_cus);
  tokens = (tokens + 63) / 64 * 64;
  long long shortest = (long long)max_seqlen / 32 / 64 * 64;
  shortest = shortest < 256 ? 256 : (shortest > 512 ? 512 : shortest);
  if (tokens < shortest) tokens = shortest;
  if (tokens > 2048) tokens = 2048;
  return (int)tokens;
}

int mi_decode_choose_split_blocks(int batch, int heads_kv, int total_blocks, int num_cus) {
  // One wavefront per (chunk, kv-head, sequence), 8 wavefronts resident per
  // compute unit: use as many chunks as fit in one resident round.
  if (batch <= 0 || heads_kv <= 0 || total_blocks <= 0) return 1;
  if (num_cus <= 0) num_cus = 256;
  const long long units = (long long)batch * heads_kv;
  long long chunks = 8LL * num_cus / units;
  if (chunks < 1) chunks = 1;
  if (chunks > total_blocks) chunks = total_blocks;
  return (int)((total_blocks + chunks - 1) / chunks);
}

// everything but the workspace
static int decode_validate_args(const mi_decode_args* a) {
  int rc = decode_validate_shape(a);
  if (rc) return rc;
  if (!a->q || !a->k || !a->v || !a->o) return fail(MI_ERR_NULL_POINTER, "q, k, v and o must be non-NULL");
  if (!aligned16(a->q) || !aligned16(a->k) || !aligned16(a->v))
    return fail(MI_ERR_ALIGNMENT, "q, k and v must be 16-byte aligned");
  if ((a->seq_lens == nullptr) == (a->cu_seqlens == nullptr))
    return fail(MI_ERR_NULL_POINTER, "exactly one of seq_lens / cu_seqlens must be non-NULL");
  if (a->kv_layout == MI_KV_PACKED && !a->cu_seqlens)
    return fail(MI_ERR_NULL_POINTER, "packed KV takes the row offsets from cu_seqlens");
  if (a->kv_layout == MI_KV_PAGED && !a->page_table)
    return fail(MI_ERR_NULL_POINTER, "paged KV needs page_table");
  const int64_t s[] = {a->q_stride_b, a->q_stride_h, a->k_stride_b, a->k_stride_s, a->k_stride_h,
                       a->v_stride_b, a->v_stride_s, a->v_stride_h};
  for (int64_t x : s)
    if (!mult8(x)) return fail(MI_ERR_STRIDE, "q/k/v strides must be multiples of 8 elements (got %lld)", (long long)x);
  // a 32-key tile is addressed as scalar base + 32-bit byte offset per lane
  if (a->k_stride_s < 0 || a->v_stride_s < 0 || a->k_stride_s >= (1 << 24) || a->v_stride_s >= (1 << 24))
    return fail(MI_ERR_STRIDE, "k/v sequence strides must be in [0, 2^24) elements (got %lld, %lld)",
                (long long)a->k_stride_s, (long long)a->v_stride_s);
  return MI_OK;
}

int mi_decode_validate(const mi_decode_args* a) {
  int rc = decode_validate_args(a);
  if (rc) return rc;
  if (!a->workspace) return fail(MI_ERR_NULL_POINTER, "workspace is NULL");
  if (!aligned16(a->workspace)) return fail(MI_ERR_ALIGNMENT, "workspace must be 16-byte aligned");
  const size_t need = mi_decode_workspace_bytes(a);
  if (a->workspace_bytes < need)
    return fail(MI_ERR_WORKSPACE, "workspace_bytes %zu < required %zu", a->workspace_bytes, need);
  return MI_OK;
}

int mi_decode_splitkv(const mi_decode_args* a, void* stream) {
  int rc = mi_decode_validate(a);
  if (rc) return rc;
  if (a->max_seqlen == 0) return MI_OK;
  mi::DecodeParams p;
  fill_decode(a, p);
  return launch_status(mi::launch_decode_splitkv(p, a->dtype, a->head_dim, static_cast<hipStream_t>(stream)), "mi_decode_splitkv");
}

int mi_decode_merge(const mi_decode_args* a, void* stream) {
  int rc = mi_decode_validate(a);
  if (rc) return rc;
  mi::DecodeParams p;
  fill_decode(a, p);
  if (a->max_seqlen == 0) p.n_splits = 0;
  return launch_status(mi::launch_decode_merge(p, a->dtype, a->head_dim, static_cast<hipStream_t>(stream)), "mi_decode_merge");
}

int mi_decode(const mi_decode_args* a, void* stream) {
  int rc = mi_decode_splitkv(a, stream);
  if (rc) return rc;
  return mi_decode_merge(a, stream);
}

int mi_decode_noalloc(const mi_decode_args* a, void* stream) {
  int rc = decode_validate_args(a);
  if (rc) return rc;
  const size_t need = mi_decode_workspace_bytes(a);
  if (need > MI_DECODE_STATIC_SCRATCH_BYTES)
    return fail(MI_ERR_WORKSPACE,
                "the split-KV partials of this call take %zu bytes, the static buffer of mi_decode_noalloc holds %u: "
                "use larger split_tokens / split_blocks or mi_decode with a workspace",
                need, (unsigned)MI_DECODE_STATIC_SCRATCH_BYTES);
  void* buf = nullptr;
  const int e = mi::decode_static_scratch(&buf);
  if (e != 0) return fail(MI_ERR_NO_DEVICE, "device address of the static decode buffer: %s",
                          hipGetErrorString(static_cast<hipError_t>(e)));
  mi_decode_args b = *a;
  b.workspace = buf;
  b.workspace_bytes = MI_DECODE_STATIC_SCRATCH_BYTES;
  return mi_decode(&b, stream);
}

int mi_device_cu_count(void) { return mi::device_cu_count(); }

}  // extern "C"
