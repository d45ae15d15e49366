// Host-visible launch interface between the C ABI layer (api.cpp) and the HIP
// translation units.  Everything here is already validated by the caller.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace mi {

struct PrefillParams {
  const void *q, *k, *v;
  void* o;
  float* lse;  // may be null
  int64_t q_sb, q_ss, q_sh;
  int64_t k_sb, k_ss, k_sh;
  int64_t v_sb, v_ss, v_sh;
  int64_t o_sb, o_ss, o_sh;
  int64_t lse_sb, lse_ss, lse_sh;
  const int32_t* cu;  // null => batched
  // block-sparse only
  const int32_t* row_ptr;
  const int32_t* col_idx;
  int64_t rp_sb, rp_sh, ci_sb, ci_sh;
  int32_t batch, hq, hkv, max_seqlen;
  int32_t n_qtiles;  // ceil(max_seqlen / rows per workgroup)
  int32_t n_items;   // logical workgroups = n_qtiles * hq * batch (set by the launcher)
  int32_t causal;
  int32_t dense_form;             // dense only: 0 chosen per launch, 1 256-row items, 2 128-row items
  int32_t win_local, win_global;  // -1 => off
  float scale;                    // log2 domain
};

struct DecodeParams {
  const void *q, *k, *v;
  void* o;
  float* lse;  // may be null
  int64_t q_sb, q_sh;
  int64_t k_sb, k_ss, k_sh;
  int64_t v_sb, v_ss, v_sh;
  int64_t o_sb, o_sh;
  const int32_t* seq_lens;  // one of the two
  const int32_t* cu;
  int32_t batch, hq, hkv, max_seqlen;
  float scale;
  int32_t split_tokens;  // dense chunk, multiple of 64
  int32_t n_splits;      // chunks per sequence (grid.x)
  float* part_o;         // [batch][hq][n_splits][D]
  float* part_lse;       // [batch][hq][n_splits]
  int32_t gslices;       // slices of 32 query heads per GQA group = ceil((hq / hkv) / 32)
  // block-sparse
  int32_t list_mode;         // 0 dense, 1 block list read from block_idx, 2 list derived from the two windows
  const int32_t* block_idx;  // list_mode 1
  const int32_t* block_cnt;
  int64_t bi_sb, bi_sh;
  int32_t max_blocks, split_blocks;
  int32_t win_local, win_global;
  int32_t add_last;  // implicit extra entry: the block of token len-1
  // KV-cache layout: 0 batched, 1 packed (rows of sequence b start at cu[b]), 2 paged
  int32_t kv_layout;
  int32_t page_size;
  const int32_t* page_table;
  int64_t pt_sb;
};

struct BwdParams {
  const void *q, *k, *v, *o, *dout;
  const float* lse;  // base-2 row log-sum-exp of the forward pass
  float* delta;      // workspace [batch][hq][max_seqlen] fp32
  void *dq, *dk, *dv;
  int64_t q_sb, q_ss, q_sh;
  int64_t k_sb, k_ss, k_sh;
  int64_t v_sb, v_ss, v_sh;
  int64_t o_sb, o_ss, o_sh;
  int64_t do_sb, do_ss, do_sh;
  int64_t dq_sb, dq_ss, dq_sh;
  int64_t dk_sb, dk_ss, dk_sh;
  int64_t dv_sb, dv_ss, dv_sh;
  int64_t lse_sb, lse_ss, lse_sh;
  int64_t dl_sb, dl_sh;
  const int32_t* cu;  // null => batched
  int32_t batch, hq, hkv, max_seqlen;
  int32_t n_rtiles;   // ceil(max_seqlen / 256): resident tiles of the dQ kernel
  int32_t causal;
  float scale;        // log2 domain
  float scale_nat;    // natural base (= scale * ln 2)
};

struct RmsParams {
  const void *x, *w, *dy;
  void *y, *dx, *dw;
  float* rsqrt;    // [rows] fp32: written by the forward, read by the backward
  float* dw_part;  // workspace [partial rows][dim] fp32
  int64_t x_st, y_st, dy_st, dx_st;  // row strides, elements
  int64_t rows;
  int32_t dim;
  float eps;
};

struct XentParams {
  const void *x, *w;   // [T, D], [N, D] row-major, row strides in elements
  const void* y;       // [T] int32 or int64 labels
  float* lse_part;     // workspace [T][n_split]
  float* tgt_part;     // workspace [T][n_split]
  float *lse, *loss;   // [T]: outputs of the forward; lse is an input of the gradient launch
  const float* dloss;  // [T], gradient launch
  void* dlogits;       // [T, N] row stride dl_ld (elements), gradient launch
  int64_t dl_ld;
  int32_t dl_vec;      // dlogits rows can be written in 16-byte pieces
  int64_t x_st, w_st;
  int32_t T, D, N;
  int32_t y_is_i64;
  int32_t n_split;           // vocabulary ranges (xent_choose_splits)
  int32_t tiles_t, block_t;  // set by the launcher
};

struct XentGradParams {
  void* logits;        // [rows, N] in / dlogits out, row stride ld (elements)
  const float* lse;    // [rows]
  const float* dloss;  // [rows]
  const void* y;
  int64_t ld, rows;
  int32_t N;
  int32_t y_is_i64;
  int32_t vec;         // rows can be accessed in 16-byte chunks
};

// CUs of the current device (cached per device; 0 if the query fails).
int device_cu_count();

// Stores `msg` as this thread's mi_last_error() text and returns `code`
// (for the host translation units other than api.cpp).
int set_error(int code, const char* msg);

// Raises a kernel's dynamic-LDS limit to `bytes`, once per (kernel, device):
// `st` is a state object that belongs to one kernel (a function-local static of
// its launcher).  Every launch after the first on a device costs one
// hipGetDevice and records nothing but the kernel launch itself.  Returns
// hipError_t as int.
constexpr int kMaxDevices = 64;
struct LdsLimitOnce {
  std::atomic<unsigned char> done[kMaxDevices];
};
inline int raise_lds_limit(LdsLimitOnce& st, const void* kern, int bytes) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  const bool slot = dev >= 0 && dev < kMaxDevices;
  if (slot && st.done[dev].load(std::memory_order_acquire)) return 0;
  e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return (int)e;
  if (slot) st.done[dev].store(1, std::memory_order_release);
  return 0;
}

// Zero-fill of the rows of packed outputs that belong to no sequence: rows of
// [0, total_rows) behind cu[batch], and rows behind the first max_seqlen tokens
// of their sequence.  Up to three tensors [row][head][bytes] per call.
struct RowFillTensor {
  void* base;
  int64_t row_stride, head_stride;  // bytes
  int32_t heads, bytes;             // bytes per (row, head): a multiple of 4
};
struct RowFillParams {
  const int32_t* cu;
  int32_t batch, total_rows, max_seqlen, n_tensors;
  RowFillTensor t[3];
};
int launch_zero_uncovered_rows(const RowFillParams& p, hipStream_t s);

// dtype: 0 bf16, 1 f16.  head_dim in {64, 96, 128}.  Return hipError_t as int.
int launch_prefill_dense(const PrefillParams& p, int dtype, int head_dim, hipStream_t s);
int launch_prefill_sparse(const PrefillParams& p, int dtype, int head_dim, hipStream_t s);
// token-window form without block lists (win_local >= 1, win_global >= 0, causal): the 128-row form of the
// dense walk over the sink tiles and the band of each item
int launch_prefill_window(const PrefillParams& p, int dtype, int head_dim, hipStream_t s);
int launch_decode_splitkv(const DecodeParams& p, int dtype, int head_dim, hipStream_t s);
int launch_decode_merge(const DecodeParams& p, int dtype, int head_dim, hipStream_t s);
// Bytes of the static device buffer behind mi_decode_noalloc
// (= MI_DECODE_STATIC_SCRATCH_BYTES) and its device address on the current
// device (hipError_t as int; no allocation).
constexpr unsigned kDecodeScratchBytes = 32u << 20;
int decode_static_scratch(void** ptr);
// the dQ kernel (which also writes Delta), then the dK + dV kernel
int launch_attn_bwd(const BwdParams& p, int dtype, int head_dim, hipStream_t s);
// RMSNorm.  x_dtype: 0 bf16, 1 f16, 2 f32; w_dtype: x_dtype or 2.  `vec`: rows
// can be read in 16-byte chunks (dim a multiple of the chunk, aligned rows,
// at most 4096 chunks).  `n_waves` = rms_partial_rows(): wavefronts of the
// launch and upper bound of the partial dw rows the backward pass writes.
// The backward workspace holds rms_partial_rows() + kRmsStageRows fp32 rows of `dim`.
constexpr int kRmsStageRows = 32;
int rms_partial_rows(long long rows, int num_cus);
int launch_rms_fwd(const RmsParams& p, int x_dtype, int w_dtype, bool vec, int n_waves, hipStream_t s);
int launch_rms_bwd(const RmsParams& p, int x_dtype, int w_dtype, bool vec, int n_waves, hipStream_t s);

// Fused linear + cross-entropy.  D a multiple of 64, rows 16-byte aligned.
int xent_choose_splits(long long tokens, int vocab, int num_cus);
int launch_xent_fwd(const XentParams& p, int dtype, bool grad, hipStream_t s);  // forward: partials + combine
int launch_xent_dlogits(const XentGradParams& p, int dtype, hipStream_t s);

// Query rows per workgroup of the two prefill kernels.
constexpr int kDenseRows = 256;
constexpr int kSparseRows = 64;
// The short form of the dense kernel: query rows per workgroup, LDS stages,
// keys per tile, workgroups resident per CU (three at head_dim 64, whose waves
// need 163 registers; two otherwise).
constexpr int kShortRows = 128;
constexpr int kShortStages = 5;
constexpr int kShortTileKeys = 32;
constexpr int kShortPerCu = 3;
constexpr int short_per_cu(int head_dim) { return head_dim == 64 ? kShortPerCu : 2; }
// LDS stages of the two prefill kernels: KV tiles resident per workgroup
// (dense), K tiles and V tiles resident per workgroup (block-sparse: the K
// ring runs one tile ahead of the V ring).
constexpr int kDenseStages = 4;
constexpr int kSparseStages = 2;
// Keys per LDS tile of the block-sparse kernel: a 64-key block is walked as two
// 32-key tiles so that four 2-wave workgroups (8 waves) fit one CU's LDS.
constexpr int kSparseTileKeys = 32;

}  // namespace mi
