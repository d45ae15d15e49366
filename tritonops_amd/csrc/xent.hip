// Fused linear + cross-entropy for gfx950.
//
// Replaces cross_entropy_fused_fwd_lse_kernel and cross_entropy_fused_bwd_kernel
// of cross_entropy_triton/cross_entropy.py:43-183, :185-266 and the host
// combine in CrossEntropyFusedFunction.forward (:337-339):
//   logits[t, n] = sum_d x[t, d] w[n, d]        never written to memory
//   lse[t]  = log sum_n exp(logits[t, n])
//   loss[t] = lse[t] - logits[t, y[t]]
//   dlogits[t, n] = do[t] (exp(logits[t, n] - lse[t]) - [n == y[t]])   (:255-265)
//
// Forward (MFMA-bound).  A workgroup of 8 wavefronts owns 256 tokens and a
// range of 256-row vocabulary tiles; per tile it runs the D loop of
// logits^T = W X^T in 64-element steps (D is a multiple of 128): both 256 x 64 slabs are fetched with
// direct-to-LDS loads into a two-stage ring (rows of 128 bytes, 16-byte chunk c
// of row r stored in slot c ^ ((r >> 1) & 7), which makes the 16-byte fragment
// reads of 16 neighbouring rows conflict-free), one barrier per step.  A
// wavefront accumulates a 128 (vocabulary) x 64 (tokens) block in eight 32x32
// MFMA accumulators.  W is the A operand, so the 16 values a lane holds per
// accumulator belong to ONE token: the per-token maximum and exponential sum
// of a tile are in-lane arithmetic plus one exchange between the lane halves.
// The running (max, sum) pair and the target logit of every token stay in
// registers across the tiles; the two wavefronts that share tokens meet in LDS
// at the end and the workgroup writes one partial (lse, target logit) per token
// and vocabulary range.  A second kernel merges the ranges.
//
// Workgroup ids are dealt round-robin to the 8 XCDs; the id is remapped so
// that the 32 workgroups that run together on one XCD form a block of token
// tiles x vocabulary ranges and share their slabs in that XCD's L2.
#include <type_traits>

#include "kernels.h"
#include "tile_core.h"

namespace mi {
namespace {

constexpr int waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

extern __shared__ __attribute__((aligned(1024))) unsigned char xsmem[];

constexpr int kXTileT = 256;   // tokens per workgroup
constexpr int kXTileN = 256;   // vocabulary rows per tile
constexpr int kXStepK = 64;    // elements of D per step
constexpr int kXSlabB = 256 * kXStepK * 2;  // one slab: 32 KiB
constexpr int kXLdsBytes = 4 * kXSlabB;     // W stage 0, W stage 1, X stage 0, X stage 1
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// GRAD = false: forward (partial lse and target logit per token and range).
// GRAD = true: the same product with the epilogue of the backward pass: every
// tile of logits is turned into dloss[t] (exp(logit - lse[t]) - [n == y[t]])
// straight from the fp32 accumulators and written to dlogits[t, n] in the
// storage dtype (the reference rounds the logits to the storage dtype first,
// cross_entropy.py:374,255-265, which costs accuracy when logits are large).
template <typename T, bool GRAD>
__global__ void __launch_bounds__(512) xent_gemm_kernel(const XentParams p) {
  typedef __attribute__((address_space(3))) const i32x4 lds_i32x4;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lq = lane & 31, lh = lane >> 5;
  const int wv = wave >> 2;  // vocabulary half of the tile
  const int wt = wave & 3;   // 64-token quarter of the workgroup's tokens

  // ---- workgroup id -> (token tile, vocabulary range)
  int t_tile, split;
  {
    const int id = blockIdx.x;
    const int xcd = id & 7, slot = id >> 3;
    const int L = ((slot >> 5) << 8) + (xcd << 5) + (slot & 31);
    const int bt = p.block_t, bs = 32 / p.block_t;  // block shape, bt a power of two
    const int blocks_t = (p.tiles_t + bt - 1) / bt;
    const int blk = L >> 5, in = L & 31;
    t_tile = (blk % blocks_t) * bt + (in & (bt - 1));
    split = (blk / blocks_t) * bs + in / bt;
    if (t_tile >= p.tiles_t || split >= p.n_split) return;
  }
  const int t0 = t_tile * kXTileT;
  // vocabulary tiles of this range
  const int nt_all = (p.N + kXTileN - 1) / kXTileN;
  const int nt_base = nt_all / p.n_split, nt_rem = nt_all % p.n_split;
  const int tile_first = split * nt_base + min(split, nt_rem);
  const int tile_cnt = nt_base + (split < nt_rem ? 1 : 0);
  const int nk = p.D / kXStepK;
  const int total = tile_cnt * nk;

  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)xsmem);
  auto uniform64 = [](uint64_t v) __attribute__((always_inline)) -> uint64_t {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
  };
  const uint64_t w_base = uniform64((uint64_t)(uintptr_t)p.w);
  const uint64_t x_base = uniform64((uint64_t)(uintptr_t)p.x);
  const uint32_t w_pitch = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(p.w_st * 2));
  const uint32_t x_pitch = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(p.x_st * 2));

  // ---- loads: wavefront `wave` fills rows [32 wave, 32 wave + 32) of both
  // slabs with four instructions each; instruction q covers 8 rows, lane i
  // fills slot i % 8 of row 8 q + i / 8.
  const int ld_row = lane >> 3;   // row inside the instruction's 8 rows
  const int ld_slot = lane & 7;
  uint32_t xoff[4], woff[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int r = 32 * wave + 8 * q + ld_row;
    const int c = ld_slot ^ ((r >> 1) & 7);
    const int tok = min(t0 + r, p.T - 1);  // rows past the end re-read the last token
    xoff[q] = (uint32_t)(tok - t0) * x_pitch + c * 16;
  }
  auto set_woff = [&](int n0) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = 32 * wave + 8 * q + ld_row;
      const int c = ld_slot ^ ((r >> 1) & 7);
      const int rr = min(r, p.N - 1 - n0);  // rows past the vocabulary re-read its last row
      woff[q] = (uint32_t)rr * w_pitch + c * 16;
    }
  };
  int iss_k = 0, iss_n0 = tile_first * kXTileN;
  set_woff(iss_n0);
  // The eight loads of a step (four of W, four of X per wavefront) are sent one
  // at a time behind the first MFMAs of the step before: sent together right
  // after the barrier, 64 KiB of requests queue up in the memory pipeline and a
  // wavefront reaches its MFMAs only when its own requests have been accepted.
  // arm() fixes the wave-uniform slab addresses, drip(k) sends load k, next()
  // moves on; a load whose mask is 0 is a no-op (all 64 lanes are active and
  // control flow is wave-uniform here, so exec is restored to all ones).
  uint64_t drip_on = 0, drip_wb = 0, drip_xb = 0;
  uint32_t drip_sw = 0, drip_sx = 0;
  auto arm = [&](int stage, bool on) __attribute__((always_inline)) {
    drip_on = uniform64(on ? ~0ull : 0ull);
    drip_wb = uniform64(w_base + (uint64_t)iss_n0 * w_pitch + (uint32_t)(iss_k * kXStepK * 2));
    drip_xb = uniform64(x_base + (uint64_t)t0 * x_pitch + (uint32_t)(iss_k * kXStepK * 2));
    drip_sw = lds0 + stage * kXSlabB + wave * 4096;
    drip_sx = lds0 + (2 + stage) * kXSlabB + wave * 4096;
  };
  auto drip = [&](int k) __attribute__((always_inline)) {
    const int q = k >> 1;
    const uint64_t base = (k & 1) ? drip_xb : drip_wb;
    const uint32_t off = (k & 1) ? xoff[q] : woff[q];
    const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(((k & 1) ? drip_sx : drip_sw) + q * 1024);
    asm volatile("s_mov_b32 m0, %3\n\ts_mov_b64 exec, %0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, -1"
                 :
                 : "s"(drip_on), "v"(off), "s"(base), "s"(slab)
                 : "memory");
  };
  auto next = [&]() __attribute__((always_inline)) {
    if (++iss_k == nk) {
      iss_k = 0;
      iss_n0 += kXTileN;
      if (iss_n0 < p.N) set_woff(iss_n0);
    }
  };

  // ---- fragment reads: row lq of a 32-row block, chunk 2 s + lh
  uint32_t a_addr[4], b_addr[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const uint32_t lo = lq * 128 + (((2 * s + lh) ^ ((lq >> 1) & 7)) << 4);
    a_addr[s] = lds0 + wv * 16384 + lo;
    b_addr[s] = lds0 + 2 * kXSlabB + wt * 8192 + lo;
    asm volatile("" : "+v"(a_addr[s]), "+v"(b_addr[s]));
  }

  f32x16 acc[4][2];
#pragma unroll
  for (int rb = 0; rb < 4; ++rb)
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) acc[rb][cb] = (f32x16){0};

  // One step = four 16-element sub-steps of 8 MFMAs.  The fragments of sub-step
  // s + 1 are read while the MFMAs of sub-step s issue; sched_barrier(0) pins
  // the slices (two reads, two MFMAs) so that the reads stay spread out.
  auto compute = [&](int stage) __attribute__((always_inline)) {
    i32x4 af[2][4], bf[2][2];
    auto read_a = [&](int s, int rb) __attribute__((always_inline)) {
      af[s & 1][rb] = *(lds_i32x4*)(uintptr_t)(a_addr[s] + stage * kXSlabB + rb * 4096);
    };
    auto read_b = [&](int s, int cb) __attribute__((always_inline)) {
      bf[s & 1][cb] = *(lds_i32x4*)(uintptr_t)(b_addr[s] + stage * kXSlabB + cb * 4096);
    };
    read_b(0, 0);
    read_b(0, 1);
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) read_a(0, rb);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
#pragma unroll
      for (int rb = 0; rb < 4; ++rb) {
        if (s + 1 < 4) {
          if (rb == 0) {
            read_b(s + 1, 0);
            read_b(s + 1, 1);
          } else if (rb == 1) {
            read_a(s + 1, 0);
            read_a(s + 1, 1);
          } else if (rb == 2) {
            read_a(s + 1, 2);
            read_a(s + 1, 3);
          }
        }
        acc[rb][0] = Elem<T>::mfma(af[s & 1][rb], bf[s & 1][0], acc[rb][0]);
        acc[rb][1] = Elem<T>::mfma(af[s & 1][rb], bf[s & 1][1], acc[rb][1]);
        if (4 * s + rb < 8) drip(4 * s + rb);   // the first eight slices carry one load each
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // ---- per-token state: tokens t0 + 64 wt + 32 cb + lq
  float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f}, tgt[2] = {0.f, 0.f};
  long long yv[2] = {0, 0};
  if (!GRAD) {
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
      const int tok = min(t0 + 64 * wt + 32 * cb + lq, p.T - 1);
      yv[cb] = p.y_is_i64 ? reinterpret_cast<const long long*>(p.y)[tok]
                          : (long long)reinterpret_cast<const int*>(p.y)[tok];
    }
  }

  // accumulators hold logits of vocabulary rows n0 + 128 wv + 32 rb + 8 (i / 4) + 4 lh + i % 4
  auto finish_tile = [&](int n0) __attribute__((always_inline)) {
    const int nw = n0 + 128 * wv;
    if (GRAD) {
      // The tile is transposed through LDS so that it leaves in 16-byte pieces
      // of whole 256-byte rows.  The slabs of the step just finished (stage 1:
      // a tile ends on an odd step) are free until the next step refills them;
      // each wavefront stages 32 tokens x 128 rows at a time in its own 8 KiB.
      __syncthreads();  // every wavefront is done reading stage 1
      typedef __attribute__((address_space(3))) i32x2 lds_w_i32x2;
      // (opaque copies: the row addresses below must be formed here, not hoisted
      // out of the main loop into registers that the loop cannot spare)
      int t0v = t0, ldv = (int)p.dl_ld;
      asm volatile("" : "+s"(t0v), "+s"(ldv));
      // per-token inputs are fetched here, once per tile, rather than kept in
      // registers through the main loop
      float lse2[2], gl[2];
      long long yt[2];
#pragma unroll
      for (int cb = 0; cb < 2; ++cb) {
        const int tok = min(t0v + 64 * wt + 32 * cb + lq, p.T - 1);
        lse2[cb] = p.lse[tok] * kLog2e;
        gl[cb] = p.dloss[tok];
        yt[cb] = p.y_is_i64 ? reinterpret_cast<const long long*>(p.y)[tok]
                            : (long long)reinterpret_cast<const int*>(p.y)[tok];
      }
      const uint32_t stg = lds0 + (wave < 4 ? 1 : 3) * kXSlabB + (wave & 3) * 8192;
#pragma unroll
      for (int cb = 0; cb < 2; ++cb) {
        // position of the label inside this wavefront's 128 rows, -1 if elsewhere
        const long long rel64 = yt[cb] - nw;
        const int rel = rel64 >= 0 && rel64 < 128 ? (int)rel64 : -1;
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) {
            const int nl = 32 * rb + 8 * g4 + 4 * lh;  // first of this lane's 4 consecutive rows
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const float pr = exp2f(acc[rb][cb][4 * g4 + j] * kLog2e - lse2[cb]);
              v[j] = gl[cb] * (pr - (rel == nl + j ? 1.f : 0.f));
            }
            const i32x2 pk = {(int)Elem<T>::pack2(v[0], v[1]), (int)Elem<T>::pack2(v[2], v[3])};
            // 8-byte slot nl / 4 of token row lq, slot pairs swizzled by the row
            const uint32_t slot = (uint32_t)(nl >> 2) ^ ((lq & 15) << 1);
            *(lds_w_i32x2*)(uintptr_t)(stg + lq * 256 + slot * 8) = pk;
            __builtin_amdgcn_sched_barrier(0);  // keeps the register need of this rare block small
          }
        // read back: 16 lanes per row
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int r = 4 * i + (lane >> 4), ch = lane & 15;  // token row, 16-byte chunk (8 vocabulary rows)
          const uint32_t slot = (uint32_t)(2 * ch) ^ ((r & 15) << 1);
          const i32x4 val = *(lds_i32x4*)(uintptr_t)(stg + r * 256 + slot * 8);
          const int tok = t0v + 64 * wt + 32 * cb + r;
          const int n = nw + 8 * ch;
          if (tok < p.T && n < p.N) {
            T* dst = reinterpret_cast<T*>(p.dlogits) + (int64_t)tok * ldv + n;
            if (p.dl_vec && n + 8 <= p.N) {
              __builtin_nontemporal_store(val, reinterpret_cast<i32x4*>(dst));
            } else {
              const T* e = reinterpret_cast<const T*>(&val);
#pragma unroll
              for (int j = 0; j < 8; ++j)
                if (n + j < p.N) dst[j] = e[j];
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    } else if (nw < p.N) {
      if (nw + 128 > p.N) {  // the tile that crosses the end of the vocabulary
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const bool dead = nw + 32 * rb + 8 * (i >> 2) + 4 * lh + (i & 3) >= p.N;
#pragma unroll
            for (int cb = 0; cb < 2; ++cb)
              if (dead) acc[rb][cb][i] = -INFINITY;
          }
      }
#pragma unroll
      for (int cb = 0; cb < 2; ++cb) {
        float mx = acc[0][cb][0];
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
          for (int i = 0; i < 16; ++i) mx = fmaxf(mx, acc[rb][cb][i]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run[cb], mx);  // finite: row nw is alive
        const float mb = m_new * kLog2e;
        float sum = 0.f;
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
          for (int i = 0; i < 16; ++i) sum += exp2f(acc[rb][cb][i] * kLog2e - mb);
        l_run[cb] = l_run[cb] * exp2f((m_run[cb] - m_new) * kLog2e) + sum;
        m_run[cb] = m_new;
        const long long rel = yv[cb] - nw;
        const bool mine = rel >= 0 && rel < 128 && (((int)rel >> 2) & 1) == lh;
        if (__builtin_amdgcn_ballot_w64(mine)) {
          const int rl = (int)rel;
#pragma unroll
          for (int rb = 0; rb < 4; ++rb)
#pragma unroll
            for (int i = 0; i < 16; ++i)
              if (mine && rl == 32 * rb + 8 * (i >> 2) + 4 * lh + (i & 3)) tgt[cb] = acc[rb][cb][i];
        }
      }
    }
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int cb = 0; cb < 2; ++cb) acc[rb][cb] = (f32x16){0};
  };

  // ---- main loop: one barrier per step; the loads of step it + 1 fly during
  // the products of step it.  D is a multiple of 128, so a tile is a whole
  // number of step pairs.
  int ck = 0, cn0 = tile_first * kXTileN;
  int it = 0;
  arm(0, total > 0);
#pragma unroll
  for (int k = 0; k < 8; ++k) drip(k);
  next();
  auto step = [&](int stage) __attribute__((always_inline)) {
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __syncthreads();
    const bool more = ++it < total;
    arm(stage ^ 1, more);
    compute(stage);
    if (more) next();
  };
  while (it < total) {
    step(0);
    step(1);
    ck += 2;
    if (ck == nk) {
      finish_tile(cn0);
      ck = 0;
      cn0 += kXTileN;
    }
  }

  if (GRAD) return;
  // ---- lane halves, then the two wavefronts that share tokens
#pragma unroll
  for (int cb = 0; cb < 2; ++cb) {
    l_run[cb] += __shfl_xor(l_run[cb], 32, 64);
    tgt[cb] += __shfl_xor(tgt[cb], 32, 64);
  }
  __syncthreads();  // every wavefront is done with the slabs
  float* ex = reinterpret_cast<float*>(xsmem);  // [2 halves][256 tokens][3]
  if (lh == 0) {
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
      float* e = ex + ((wv * 256) + 64 * wt + 32 * cb + lq) * 3;
      e[0] = m_run[cb];
      e[1] = l_run[cb];
      e[2] = tgt[cb];
    }
  }
  __syncthreads();
  if (tid < 256 && t0 + tid < p.T) {
    const float* e0 = ex + tid * 3;
    const float* e1 = ex + (256 + tid) * 3;
    const float M = fmaxf(e0[0], e1[0]);
    const float Lsum = e0[1] * exp2f((e0[0] - M) * kLog2e) + e1[1] * exp2f((e1[0] - M) * kLog2e);
    const int64_t o = (int64_t)(t0 + tid) * p.n_split + split;
    p.lse_part[o] = M + log2f(Lsum) * kLn2;
    p.tgt_part[o] = e0[2] + e1[2];
  }
}

// lse[t] = log sum over the ranges of exp(lse_part), loss[t] = lse[t] - target logit
__global__ void __launch_bounds__(256) xent_combine_kernel(const XentParams p) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= p.T) return;
  const float* lp = p.lse_part + (int64_t)t * p.n_split;
  const float* tp = p.tgt_part + (int64_t)t * p.n_split;
  float M = -INFINITY;
  for (int s = 0; s < p.n_split; ++s) M = fmaxf(M, lp[s]);
  float sum = 0.f, tg = 0.f;
  for (int s = 0; s < p.n_split; ++s) {
    sum += exp2f((lp[s] - M) * kLog2e);
    tg += tp[s];
  }
  const float lse = M + log2f(sum) * kLn2;
  p.lse[t] = lse;
  p.loss[t] = lse - tg;
}

// In place over a [rows, N] block of logits: g = do[t] (exp(logit - lse[t]) - [n == y[t]]).
// One workgroup per (row, 2048-column segment): blockIdx.x = row.
template <typename T>
__global__ void __launch_bounds__(256) xent_dlogits_kernel(const XentGradParams p) {
  const int64_t t = blockIdx.x;
  const int n0 = blockIdx.y * 2048 + threadIdx.x * 8;
  T* row = reinterpret_cast<T*>(p.logits) + t * p.ld;
  const float lse = p.lse[t] * kLog2e, g = p.dloss[t];
  const long long y = p.y_is_i64 ? reinterpret_cast<const long long*>(p.y)[t]
                                 : (long long)reinterpret_cast<const int*>(p.y)[t];
  if (p.vec && n0 + 8 <= p.N) {
    i32x4 raw = *reinterpret_cast<const i32x4*>(row + n0);
    T* e = reinterpret_cast<T*>(&raw);
#pragma unroll
    for (int i = 0; i < 8; ++i)
      e[i] = (T)(g * (exp2f((float)e[i] * kLog2e - lse) - (n0 + i == y ? 1.f : 0.f)));
    *reinterpret_cast<i32x4*>(row + n0) = raw;
  } else {
    for (int i = 0; i < 8 && n0 + i < p.N; ++i)
      row[n0 + i] = (T)(g * (exp2f((float)row[n0 + i] * kLog2e - lse) - (n0 + i == y ? 1.f : 0.f)));
  }
}

}  // namespace

// Vocabulary ranges for `tokens` rows: as many as keep one round of workgroups
// (one per CU) busy, never more than there are 256-row vocabulary tiles.
int xent_choose_splits(long long tokens, int vocab, int num_cus) {
  const long long tiles_t = (tokens + kXTileT - 1) / kXTileT;
  const int tiles_n = (vocab + kXTileN - 1) / kXTileN;
  long long s = (num_cus > 0 ? num_cus : 256) / (tiles_t > 0 ? tiles_t : 1);
  if (s < 1) s = 1;
  if (s > tiles_n) s = tiles_n;
  return (int)s;
}

namespace {
template <typename T, bool GRAD>
int launch_gemm(const XentParams& p, unsigned grid, hipStream_t s) {
  auto kern = xent_gemm_kernel<T, GRAD>;
  static LdsLimitOnce lds_once;
  if (const int e = raise_lds_limit(lds_once, reinterpret_cast<const void*>(kern), kXLdsBytes)) return e;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), kXLdsBytes, s, p);
  return (int)hipGetLastError();
}
}  // namespace

// grad: the launch writes dlogits instead of the partial lse / target logit
int launch_xent_fwd(const XentParams& p0, int dtype, bool grad, hipStream_t s) {
  XentParams p = p0;
  p.tiles_t = (p.T + kXTileT - 1) / kXTileT;
  p.block_t = p.tiles_t >= 8 ? 8 : p.tiles_t >= 4 ? 4 : p.tiles_t >= 2 ? 2 : 1;
  const int bs = 32 / p.block_t;
  const long long blocks = (long long)((p.tiles_t + p.block_t - 1) / p.block_t) * ((p.n_split + bs - 1) / bs);
  const unsigned grid = (unsigned)((blocks * 32 + 255) / 256 * 256);
  int rc;
  if (dtype == 0)
    rc = grad ? launch_gemm<__bf16, true>(p, grid, s) : launch_gemm<__bf16, false>(p, grid, s);
  else
    rc = grad ? launch_gemm<_Float16, true>(p, grid, s) : launch_gemm<_Float16, false>(p, grid, s);
  if (rc || grad) return rc;
  hipLaunchKernelGGL(xent_combine_kernel, dim3((unsigned)((p.T + 255) / 256)), dim3(256), 0, s, p);
  return (int)hipGetLastError();
}

int launch_xent_dlogits(const XentGradParams& p, int dtype, hipStream_t s) {
  const dim3 grid((unsigned)p.rows, (unsigned)((p.N + 2047) / 2048));
  if (dtype == 0)
    hipLaunchKernelGGL(xent_dlogits_kernel<__bf16>, grid, dim3(256), 0, s, p);
  else
    hipLaunchKernelGGL(xent_dlogits_kernel<_Float16>, grid, dim3(256), 0, s, p);
  return (int)hipGetLastError();
}

}  // namespace mi
