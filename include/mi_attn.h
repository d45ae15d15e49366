/*
 * mi_attn.h - C ABI of the MI355X (gfx950) attention forward library.
 *
 * The upstream project (rookie-joe/TritonOps) has no FFI of its own: its
 * boundary is a set of Python launchers that hand torch tensors to Triton
 * kernels.  Every entry point below replaces one such launcher + kernel pair;
 * the citation names the reference interface it stands in for (paths relative
 * to the reference checkout).
 *
 * Conventions shared by all entry points
 *   - plain C structs of pointers, element strides and sizes; no torch types;
 *   - every struct starts with `struct_size` (sizeof the struct as the caller
 *     compiled it) so the library can reject a mismatched caller;
 *   - device pointers are raw HIP device addresses, `stream` is a hipStream_t
 *     passed as void* (NULL = the null stream);
 *   - the innermost (head_dim) axis of q/k/v/o must be contiguous and every
 *     row must start on a 16-byte boundary (strides are in ELEMENTS);
 *   - return value: MI_OK (0) or a negative mi_status; nothing throws, nothing
 *     allocates or frees device memory, nothing synchronises the device (the
 *     blocking timing helper for benchmarks lives in mi_attn_bench.h);
 *   - all argument validation happens on the host before any HIP call, so it
 *     can be exercised on a machine without a GPU;
 *   - log-sum-exp values are base 2 of the scaled scores, fp32:
 *       lse2 = log2( sum_j 2^(q.k_j * scale_log2) ),  scale_log2 = scale*log2(e)
 *     exactly as flash_attn_triton/flash_attn_triton.py:163,170,180,839;
 *   - q-head h reads kv-head h / (heads_q / heads_kv)
 *     (flash_attn_triton/flash_attn_triton.py:86-87,616).
 */
#ifndef MI_ATTN_H
#define MI_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI_ATTN_ABI_VERSION 8

/* KV tile edge (tokens) of the prefill kernels and block edge of the block
 * sparse layouts; fixed at build time. */
#define MI_ATTN_BLOCK 64

typedef enum mi_dtype {
  MI_DTYPE_BF16 = 0,
  MI_DTYPE_F16 = 1,
  MI_DTYPE_F32 = 2            /* mi_rmsnorm_* only                             */
} mi_dtype;

typedef enum mi_status {
  MI_OK = 0,
  MI_ERR_NULL_POINTER = -1,   /* a required pointer is NULL                    */
  MI_ERR_STRUCT_SIZE = -2,    /* struct_size does not match this library       */
  MI_ERR_DTYPE = -3,          /* dtype is not MI_DTYPE_BF16 / MI_DTYPE_F16     */
  MI_ERR_HEAD_DIM = -4,       /* head_dim not in {64, 96, 128}                 */
  MI_ERR_GQA = -5,            /* heads_q % heads_kv != 0 or a count <= 0       */
  MI_ERR_SHAPE = -6,          /* negative / zero / overflowing extent          */
  MI_ERR_STRIDE = -7,         /* stride not a multiple of 8 elements (16 B)    */
  MI_ERR_ALIGNMENT = -8,      /* base pointer not 16-byte aligned              */
  MI_ERR_SCALE = -9,          /* scale_log2 not finite or <= 0                 */
  MI_ERR_WORKSPACE = -10,     /* workspace too small / splits out of range     */
  MI_ERR_SPARSE_LAYOUT = -11, /* block size / index list arguments invalid     */
  MI_ERR_LAUNCH = -12,        /* hipLaunchKernel reported an error             */
  MI_ERR_NO_DEVICE = -13      /* no HIP device / wrong architecture            */
} mi_status;

/* ------------------------------------------------------------------------- */
/* Dense forward.
 * Replaces flash_attn_triton_fwd + flash_attn_fwd_kernel
 * (flash_attn_triton/flash_attn_triton.py:595-658, :52-180) for the packed
 * var-len causal GQA form, and the [B,H,N,D] kernels of
 * tutorial/4.3.multi_head_attention.py:45-194 (non-causal) and
 * tutorial/4.4.causal_attention.py:133-180 (causal) for the batched form.
 *
 * Two addressing modes, one kernel:
 *   cu_seqlens != NULL : packed. Token t of sequence b lives at row
 *                        cu_seqlens[b]+t; *_stride_b is ignored.
 *   cu_seqlens == NULL : batched. Every sequence has max_seqlen tokens and
 *                        sequence b starts at b * *_stride_b.
 * Rows whose sequence has length 0 are never written.  In the packed form
 * max_seqlen must bound every length: a longer sequence is cut at max_seqlen
 * (its later rows are neither read nor written).
 * total_rows (packed form only): the reference launcher zero-fills o and lse
 * before its kernel runs (flash_attn_triton.py:608-609), so rows that belong to
 * no sequence come back as zeros.  With total_rows > 0 the call does the same
 * for exactly those rows - rows of [0, total_rows) that lie behind
 * cu_seqlens[batch], or behind the first max_seqlen tokens of their sequence -
 * with one small extra launch, so the caller can hand in uninitialised
 * outputs.  0 leaves such rows untouched.
 * dense_form: the kernel comes in two forms that give the same bits - work
 * items of 256 query rows on workgroups of eight wavefronts, one to a compute
 * unit, and work items of 128 rows on workgroups of four wavefronts, two to a
 * compute unit (three at head_dim 64).  MI_DENSE_FORM_AUTO lets the library
 * pick per launch from the number of work items (the short form when every
 * work item has a compute unit to itself; at head_dim 64 also where three
 * workgroups per unit outrun one); the other two values are for tests and for
 * callers who have measured their own shapes.
 */
enum { MI_DENSE_FORM_AUTO = 0, MI_DENSE_FORM_256_ROWS = 1, MI_DENSE_FORM_128_ROWS = 2 };

typedef struct mi_attn_fwd_args {
  uint32_t struct_size;
  int32_t dtype;                 /* mi_dtype of q, k, v, o                     */
  const void *q, *k, *v;         /* device                                     */
  void *o;                       /* device, dtype as q                         */
  float *lse;                    /* device, fp32 base-2 LSE; may be NULL       */
  int64_t q_stride_b, q_stride_s, q_stride_h;
  int64_t k_stride_b, k_stride_s, k_stride_h;
  int64_t v_stride_b, v_stride_s, v_stride_h;
  int64_t o_stride_b, o_stride_s, o_stride_h;
  int64_t lse_stride_b, lse_stride_s, lse_stride_h;
  const int32_t *cu_seqlens;     /* device [batch+1] or NULL                   */
  int32_t batch, heads_q, heads_kv;
  int32_t max_seqlen;            /* upper bound of every sequence length       */
  int32_t head_dim;              /* 64, 96 or 128 (q, k and v alike)           */
  int32_t causal;                /* 0 / 1                                      */
  float scale_log2;              /* softmax scale * log2(e), > 0               */
  int32_t total_rows;            /* packed: rows of o / lse to cover, or 0     */
  int32_t dense_form;            /* MI_DENSE_FORM_*                            */
} mi_attn_fwd_args;

int mi_attn_fwd(const mi_attn_fwd_args *args, void *stream);

/* ------------------------------------------------------------------------- */
/* Dense backward.
 * Replaces flash_attn_triton_bwd and its three kernels
 * (flash_attn_triton/flash_attn_triton.py:661-813, :183-593): given q, k, v,
 * the forward's o and base-2 lse, and dout = d(loss)/d(o), writes dq, dk, dv
 * (dtype as q; dk/dv have heads_kv heads: the query heads of a GQA group are
 * summed inside the kernel).  Addressing modes, causal flag and scale as in
 * mi_attn_fwd.  The workspace holds
 * Delta = rowsum(o * dout) in fp32.  Two launches on `stream`.
 * total_rows as in mi_attn_fwd: with a value > 0 (packed form) the rows of dq,
 * dk and dv that belong to no sequence are zero-filled by one more launch.
 */
typedef struct mi_attn_bwd_args {
  uint32_t struct_size;
  int32_t dtype;
  const void *q, *k, *v, *o, *dout;  /* device                                 */
  const float *lse;                  /* device, as written by mi_attn_fwd      */
  void *dq, *dk, *dv;                /* device, fully written for rows < len   */
  int64_t q_stride_b, q_stride_s, q_stride_h;
  int64_t k_stride_b, k_stride_s, k_stride_h;
  int64_t v_stride_b, v_stride_s, v_stride_h;
  int64_t o_stride_b, o_stride_s, o_stride_h;
  int64_t dout_stride_b, dout_stride_s, dout_stride_h;
  int64_t dq_stride_b, dq_stride_s, dq_stride_h;
  int64_t dk_stride_b, dk_stride_s, dk_stride_h;
  int64_t dv_stride_b, dv_stride_s, dv_stride_h;
  int64_t lse_stride_b, lse_stride_s, lse_stride_h;
  const int32_t *cu_seqlens;         /* device [batch+1] or NULL               */
  int32_t batch, heads_q, heads_kv;
  int32_t max_seqlen;
  int32_t head_dim;                  /* 64, 96 or 128                          */
  int32_t causal;
  float scale_log2;                  /* the value the forward pass was given   */
  void *workspace;                   /* device, mi_attn_bwd_workspace_bytes()  */
  size_t workspace_bytes;
  int32_t total_rows;                /* packed: rows of dq/dk/dv to cover, or 0 */
} mi_attn_bwd_args;

size_t mi_attn_bwd_workspace_bytes(const mi_attn_bwd_args *args);
int mi_attn_bwd(const mi_attn_bwd_args *args, void *stream);

/* ------------------------------------------------------------------------- */
/* Block-sparse forward (always token-causal).
 * Replaces the sparse launcher + kernel of
 * flash_attn_triton/flash_attn_sparse_attn_triton.py:237-326, :47-234, whose
 * mask (oracle :422-433) is  k <= q  and  (q < k + local_window or
 * k < global_window); generalised to an arbitrary list of live 64x64 blocks.
 *
 * Layout: CSR over query blocks of MI_ATTN_BLOCK tokens (block coordinates are
 * relative to each sequence's first token).  Query block i of (batch b, head
 * h) walks  col_idx[ off + row_ptr[i] .. off + row_ptr[i+1] )  with
 *   row_ptr taken at   row_ptr + b*row_ptr_stride_b + h*row_ptr_stride_h
 *   col_idx taken at   col_idx + b*col_idx_stride_b + h*col_idx_stride_h
 * (strides of 0 broadcast one mask over batch and/or heads).  Column indices
 * must be ascending, unique and <= i.  Inside a live block, keys beyond the
 * query (causal) or beyond the sequence are masked per token.
 *
 * window_local / window_global: when window_local >= 0 the reference's token
 * window is applied on top of the block list inside every live block:
 *   allowed(q,k) = k <= q and (q - k < window_local or k < window_global).
 * Pass -1 / -1 for a pure block mask.
 * The window form needs no lists: with row_ptr = col_idx = NULL (both), and
 * window_local >= 1 and window_global >= 0, the blocks follow from the two
 * windows (the reference's launcher takes nothing else, :237-326): every 128
 * query rows walk the tiles of the first window_global keys and the band of
 * tiles that ends at their diagonal, on the dense kernel's pipeline.  Same
 * results as the call with the window's lists up to summation order; faster
 * than it for local windows of 2048 tokens or more at head_dim 96 / 128,
 * slower for short windows and at head_dim 64 (the lists are then the better
 * call).  window_local = 0 (not even the diagonal is visible) takes lists.
 * A query row with no allowed key yields o = 0 and lse = -inf.
 * total_rows as in mi_attn_fwd (the reference launcher zero-fills both outputs,
 * flash_attn_sparse_attn_triton.py:274-275).
 */
typedef struct mi_attn_sparse_args {
  uint32_t struct_size;
  int32_t dtype;
  const void *q, *k, *v;
  void *o;
  float *lse;                    /* may be NULL                                */
  int64_t q_stride_b, q_stride_s, q_stride_h;
  int64_t k_stride_b, k_stride_s, k_stride_h;
  int64_t v_stride_b, v_stride_s, v_stride_h;
  int64_t o_stride_b, o_stride_s, o_stride_h;
  int64_t lse_stride_b, lse_stride_s, lse_stride_h;
  const int32_t *cu_seqlens;     /* device [batch+1] or NULL (batched)         */
  const int32_t *row_ptr;        /* device [n_q_blocks+1] per (b,h) slice, or  */
  const int32_t *col_idx;        /* device; both NULL: the window form         */
  int64_t row_ptr_stride_b, row_ptr_stride_h;
  int64_t col_idx_stride_b, col_idx_stride_h;
  int32_t batch, heads_q, heads_kv;
  int32_t max_seqlen;
  int32_t head_dim;
  int32_t block_size;            /* must equal MI_ATTN_BLOCK                   */
  int32_t window_local;          /* tokens, or -1                              */
  int32_t window_global;         /* tokens, or -1                              */
  float scale_log2;
  int32_t total_rows;            /* packed: rows of o / lse to cover, or 0     */
} mi_attn_sparse_args;

int mi_attn_fwd_blocksparse(const mi_attn_sparse_args *args, void *stream);

/* ------------------------------------------------------------------------- */
/* Single-query decoding, dense and block-sparse.
 * Replaces flash_attention_decoding (flash_attn_triton/flash_attn_decoding.py
 * :213-336: pass 1 kernel :9-122, merge kernel :126-210) and
 * flash_attention_sparse_decoding (flash_attn_triton/
 * flash_attn_decoding_sparse.py:222-365: pass 1 :10-127, merge :131-219).
 *
 * q [batch, heads_q, head_dim]; k, v padded per sequence: token t of sequence
 * b, kv-head h at  b*stride_b + t*stride_s + h*stride_h ; only the first
 * seq_lens[b] tokens are read (flash_attn_decoding.py:46-48,80).  The G =
 * heads_q/heads_kv query heads of one kv-head are processed together, 32 to a
 * wavefront, so every K/V byte is fetched once per 32 query heads (the
 * reference fetches it once per query head, flash_attn_decoding.py:42-45,
 * 264-268); any ratio G is accepted.
 *
 * Pass 1 splits each sequence into chunks of `split_tokens` tokens (dense) or
 * `split_blocks` listed blocks (sparse); one workgroup per (chunk, kv-head,
 * batch) writes an un-normalised fp32 partial output and its base-2 LSE into
 * the workspace.  Pass 2 merges the partials (flash_attn_decoding.py:171-208).
 * seq_lens[b] == 0 gives an all-zero output row (flash_attn_decoding.py:49-50,
 * 151,197-210).
 *
 * Sparse form (block_idx != NULL): kv-head h of batch b reads the token blocks
 *   block_idx[b*block_idx_stride_b + h*block_idx_stride_h + i],
 *   i < (block_cnt ? block_cnt[b*heads_kv + h] : max_blocks),
 * each `block_size` (64) tokens; indices must be unique and in range
 * [0, ceil(seq_len/block_size)); tokens >= seq_len are masked.  With
 * include_last_block the block of the newest token is attended as well; if it
 * is also listed it still counts once.  On top of the
 * list an optional token window reproduces flash_attn_decoding_sparse.py
 * :391-396:  allowed(k) = k < window_global or k >= seq_len - window_local
 * (pass -1/-1 to disable).
 *
 * Window form (window_form = 1, block_idx ignored): the list is not read from
 * memory but derived per sequence from (seq_len, window_global, window_local),
 * which is all the reference's sparse decoder attends (flash_attn_decoding_
 * sparse.py:391-396): the blocks of the first window_global tokens, then the
 * blocks from token max(seq_len - window_local, 0) to the last one, each once,
 * with the token window applied inside them.  max_blocks must be at least
 *   ceil(window_global / 64) + ceil(window_local / 64) + 1
 * (it sizes the chunks and the workspace); block_cnt and include_last_block
 * are ignored.
 */
/* Where token t of sequence b lives in k / v (element strides as given):
 *   MI_KV_BATCHED  k + b*k_stride_b + t*k_stride_s            ([batch, max_seqlen, heads_kv, D] view; the
 *                  layout flash_attention_decoding takes, flash_attn_decoding.py:283-290)
 *   MI_KV_PACKED   k + (cu_seqlens[b] + t)*k_stride_s          (one [total_tokens, heads_kv, D] buffer, the
 *                  layout the reference's decode oracle consumes, flash_attn_decoding.py:357-359;
 *                  needs cu_seqlens, k_stride_b is ignored)
 *   MI_KV_PAGED    k + page_table[b][t / page_size]*k_stride_b + (t % page_size)*k_stride_s
 *                  (a pool of pages [num_pages, page_size, heads_kv, D]; k_stride_b is the page stride).
 * No counterpart of the paged form exists in the reference; it is the cache
 * layout of a serving loop around this call. */
#define MI_KV_BATCHED 0
#define MI_KV_PACKED 1
#define MI_KV_PAGED 2

typedef struct mi_decode_args {
  uint32_t struct_size;
  int32_t dtype;
  const void *q, *k, *v;
  void *o;                       /* [batch, heads_q, head_dim], dtype as q     */
  float *lse;                    /* [batch, heads_q] fp32 base-2; may be NULL  */
  int64_t q_stride_b, q_stride_h;
  int64_t k_stride_b, k_stride_s, k_stride_h;
  int64_t v_stride_b, v_stride_s, v_stride_h;
  int64_t o_stride_b, o_stride_h;
  const int32_t *seq_lens;       /* device [batch]; or                         */
  const int32_t *cu_seqlens;     /* device [batch+1] (lengths = differences);  */
                                 /* exactly one of the two is non-NULL         */
  int32_t batch, heads_q, heads_kv;
  int32_t max_seqlen;            /* upper bound of every length (grid size)    */
  int32_t head_dim;              /* 64, 96 or 128                              */
  float scale_log2;
  /* split-KV */
  int32_t split_tokens;          /* dense: tokens per workgroup, multiple of 64*/
  void *workspace;               /* device, mi_decode_workspace_bytes() bytes  */
  size_t workspace_bytes;
  /* block-sparse (all ignored when block_idx == NULL) */
  const int32_t *block_idx;      /* device                                     */
  const int32_t *block_cnt;      /* device [batch*heads_kv] or NULL            */
  int64_t block_idx_stride_b, block_idx_stride_h;
  int32_t max_blocks;            /* list capacity per (b, kv-head)             */
  int32_t block_size;            /* must equal MI_ATTN_BLOCK                   */
  int32_t split_blocks;          /* sparse: listed blocks per workgroup        */
  int32_t window_local;          /* tokens, or -1                              */
  int32_t window_global;         /* tokens, or -1                              */
  int32_t include_last_block;    /* 1: also attend the block holding token     */
                                 /* seq_len-1 (listed or not, counted once)    */
  /* KV-cache layout (see MI_KV_* above) */
  int32_t kv_layout;             /* MI_KV_BATCHED, MI_KV_PACKED or MI_KV_PAGED */
  int32_t page_size;             /* paged: tokens per page, multiple of 32     */
  const int32_t *page_table;     /* paged: device; physical page of logical    */
                                 /* page p of sequence b at [b*stride_b + p]   */
  int64_t page_table_stride_b;
  int32_t window_form;           /* 1: block list derived from the two windows */
} mi_decode_args;

/* Number of pass-1 chunks per sequence for these arguments (host only). */
int mi_decode_num_splits(const mi_decode_args *args);
/* Bytes of workspace the two passes need: fp32 partial o + fp32 lse2. */
size_t mi_decode_workspace_bytes(const mi_decode_args *args);
/* Heuristic chunk length (tokens, multiple of 64) that fills `num_cus` compute
 * units for the given problem; host only. */
int mi_decode_choose_split_tokens(int batch, int heads_kv, int max_seqlen,
                                  int num_cus);
/* Heuristic chunk length in listed blocks for the block-list form: the largest
 * number of chunks per (sequence, kv-head) whose wavefronts are all resident
 * at once on `num_cus` compute units (a second, partly filled round of
 * wavefronts costs more than longer chunks do); host only.  `total_blocks`
 * counts the implicit last block when include_last_block is set. */
int mi_decode_choose_split_blocks(int batch, int heads_kv, int total_blocks,
                                  int num_cus);

/* Pass 1 only: partials into the workspace. */
int mi_decode_splitkv(const mi_decode_args *args, void *stream);
/* Pass 2 only: merge the workspace into o (and lse). */
int mi_decode_merge(const mi_decode_args *args, void *stream);
/* Both passes back to back on `stream`. */
int mi_decode(const mi_decode_args *args, void *stream);

/* mi_decode for callers that cannot allocate device memory.
 * No counterpart in the reference (its launcher allocates the partial results
 * with torch on every call, flash_attn_decoding.py:249-261).  It is for callers
 * that cannot call hipMalloc or size and carry a workspace: code under HIP
 * graph capture, tight serving loops, harnesses that forbid allocation.
 * Same arguments and results (bit for bit) as mi_decode, except that
 * args->workspace / workspace_bytes are ignored: the split-KV partials go to a
 * buffer of MI_DECODE_STATIC_SCRATCH_BYTES that the library holds in device
 * memory, one per GPU, from load time until the process ends.  A call whose
 * mi_decode_workspace_bytes() exceeds that size fails with MI_ERR_WORKSPACE
 * before anything is launched (pick larger split_tokens / split_blocks).
 * The call allocates and frees nothing and records only kernel launches; the
 * FIRST call on a device also asks the runtime for the buffer's device address
 * (hipGetSymbolAddress, which may load the code object), so make one call per
 * device outside capture before recording it into a graph.
 * Every call on one GPU uses the same buffer: calls that overlap on one GPU
 * (different streams, or graphs replayed concurrently) race; serialise them.
 * The buffer keeps the previous call's partials; nothing in it needs to start
 * at zero, because pass 2 reads only the slots pass 1 of the same call wrote. */
#define MI_DECODE_STATIC_SCRATCH_BYTES (32u << 20)
int mi_decode_noalloc(const mi_decode_args *args, void *stream);

/* ------------------------------------------------------------------------- */
/* RMSNorm forward / backward over rows of `dim` elements.
 * Replaces RMSNormTritonFunction.forward / .backward and their kernels
 * (common/rms.py:221-355, :8-218):
 *   rsqrt[t] = 1 / sqrt(eps + mean_d x[t,d]^2)         fp32, saved for backward
 *   y[t,d]   = x[t,d] * rsqrt[t] * w[d]
 *   dx[t,d]  = dy[t,d] w[d] rsqrt[t] - x[t,d] rsqrt[t]^3 (sum_d dy w x) / dim
 *   dw[d]    = sum_t dy[t,d] x[t,d] rsqrt[t]
 * x, y, dy, dx share one dtype (MI_DTYPE_BF16, MI_DTYPE_F16 or MI_DTYPE_F32),
 * rows contiguous with the given row strides (elements); w and dw have the
 * same dtype as x or are fp32.  Any dim >= 1 (the reference's test uses 255).
 * The backward needs mi_rmsnorm_bwd_workspace_bytes() of device workspace for
 * the partial dw rows (no atomics: results are deterministic).
 */
typedef struct mi_rmsnorm_args {
  uint32_t struct_size;
  int32_t x_dtype;               /* of x, y, dy, dx                            */
  int32_t w_dtype;               /* of w, dw: x_dtype or MI_DTYPE_F32          */
  int32_t dim;
  int64_t rows;
  const void *x, *w;             /* device                                     */
  void *y;                       /* forward output                             */
  float *rsqrt;                  /* [rows]: forward output, backward input     */
  const void *dy;                /* backward input                             */
  void *dx, *dw;                 /* backward outputs                           */
  int64_t x_stride, y_stride, dy_stride, dx_stride;  /* row strides            */
  float eps;
  void *workspace;               /* backward only                              */
  size_t workspace_bytes;
} mi_rmsnorm_args;

int mi_rmsnorm_fwd(const mi_rmsnorm_args *args, void *stream);
size_t mi_rmsnorm_bwd_workspace_bytes(const mi_rmsnorm_args *args);
int mi_rmsnorm_bwd(const mi_rmsnorm_args *args, void *stream);

/* ------------------------------------------------------------------------- */
/* Fused linear + cross-entropy.
 *
 * Replaces CrossEntropyFusedFunction.forward and its kernel
 * cross_entropy_fused_fwd_lse_kernel (cross_entropy_triton/cross_entropy.py:
 * 276-352, :43-183) and the element-wise kernel of its backward
 * (cross_entropy_fused_bwd_kernel, :185-266):
 *   logits[t,n] = sum_d x[t,d] w[n,d]             (never written by the forward)
 *   lse[t]      = log sum_n exp(logits[t,n])       fp32, saved for the backward
 *   loss[t]     = lse[t] - logits[t, y[t]]         fp32
 *   dlogits[t,n] = dloss[t] (exp(logits[t,n] - lse[t]) - [n == y[t]])
 * x [tokens, dim] and w [vocab, dim] are bf16 or f16, row-major with row
 * strides in elements (multiples of 8, bases 16-byte aligned); dim must be a
 * multiple of 128 (pad x and w with zero columns otherwise).  Labels are int32
 * or int64; a label outside [0, vocab) contributes no target logit
 * (loss = lse).  The forward needs mi_xent_fwd_workspace_bytes() of device
 * workspace for the per-range partial results.
 */
typedef struct mi_xent_args {
  uint32_t struct_size;
  int32_t dtype;                 /* of x and w                                 */
  int32_t tokens, dim, vocab;
  int32_t labels_i64;            /* 1: y is int64, 0: int32                    */
  const void *x, *w;             /* device                                     */
  const void *y;                 /* [tokens] labels                            */
  int64_t x_stride, w_stride;    /* row strides, elements                      */
  float *lse, *loss;             /* [tokens] fp32 outputs                      */
  void *workspace;
  size_t workspace_bytes;
} mi_xent_args;

size_t mi_xent_fwd_workspace_bytes(const mi_xent_args *args);
int mi_xent_fwd(const mi_xent_args *args, void *stream);

/* Backward, first step: dlogits[t,n] = dloss[t] (exp(logits[t,n] - lse[t]) -
 * [n == y[t]]) for a block of tokens, computed by the forward's GEMM kernel
 * with this epilogue on the fp32 accumulators and written once, in the dtype
 * of x.  Replaces `xw_partial = torch.mm(x_partial, w^T)` plus
 * cross_entropy_fused_bwd_kernel (cross_entropy.py:374, :185-266), which round
 * the logits to the storage dtype before the exponential.  The two gradient
 * GEMMs (grad_x = dlogits w, grad_w = dlogits^T x, :407-415) stay with the
 * caller's BLAS.  x / w / y as for mi_xent_fwd; no workspace. */
typedef struct mi_xent_bwd_args {
  uint32_t struct_size;
  int32_t dtype;                 /* of x, w and dlogits                        */
  int32_t tokens, dim, vocab;
  int32_t labels_i64;
  const void *x, *w;             /* device                                     */
  const void *y;                 /* [tokens] labels                            */
  int64_t x_stride, w_stride;    /* row strides, elements                      */
  const float *lse, *dloss;      /* [tokens] fp32                              */
  void *dlogits;                 /* [tokens, vocab], row stride ld (elements)  */
  int64_t ld;
} mi_xent_bwd_args;

int mi_xent_bwd_dlogits(const mi_xent_bwd_args *args, void *stream);

/* In place over a block of logits [rows, vocab] (row stride ld, elements):
 * logits[t,n] <- dloss[t] (exp(logits[t,n] - lse[t]) - [n == y[t]]), the
 * operand of the two gradient GEMMs (cross_entropy.py:255-266, :369-415). */
typedef struct mi_xent_grad_args {
  uint32_t struct_size;
  int32_t dtype;                 /* of logits                                  */
  int32_t vocab;
  int32_t labels_i64;
  int64_t rows, ld;
  void *logits;                  /* device, in / out                           */
  const float *lse, *dloss;      /* [rows] fp32                                */
  const void *y;                 /* [rows] labels                              */
} mi_xent_grad_args;

int mi_xent_dlogits(const mi_xent_grad_args *args, void *stream);

/* ------------------------------------------------------------------------- */
/* Introspection (host only). */
int mi_abi_version(void);
/* Message of the last failing call on this thread ("" if none). */
const char *mi_last_error(void);
/* Name of a status code. */
const char *mi_status_name(int status);
/* Compute units of the current HIP device, the figure the library's own
 * launches and the mi_decode_choose_* heuristics are sized with (0 when no
 * device can be queried; the heuristics then assume 256). */
int mi_device_cu_count(void);
/* Validate without launching (what the launch entry points run first). */
int mi_attn_fwd_validate(const mi_attn_fwd_args *args);
int mi_attn_fwd_blocksparse_validate(const mi_attn_sparse_args *args);
int mi_decode_validate(const mi_decode_args *args);
int mi_attn_bwd_validate(const mi_attn_bwd_args *args);

#ifdef __cplusplus
}
#endif
#endif /* MI_ATTN_H */
