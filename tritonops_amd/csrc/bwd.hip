// Dense attention backward for gfx950: dq, dk, dv from q, k, v, o, do and the
// base-2 row log-sum-exp the forward pass returns.
//
// Replaces flash_attn_bwd_D_kernel, flash_attn_bwd_dq_kernel and
// flash_attn_bwd_dkdv_kernel (flash_attn_triton/flash_attn_triton.py:183-593)
// and their launcher flash_attn_triton_bwd (:661-813).  Math, with
// S2 = q.k * scale_log2, P = 2^(S2 - lse2), Delta_i = sum_d o_id do_id:
//   dV = P^T dO,   dP = dO V^T,   dS = P o (dP - Delta),
//   dQ = dS K * scale,   dK = dS^T Q * scale      (scale in the natural base).
// Delta is kept in fp32 (the reference rounds it to the input dtype, :677),
// P and dS are rounded to the input dtype before their second product as the
// reference does (in the dK + dV kernel dS is formed from the rounded P), the
// GQA members of a kv-head are accumulated in registers
// (the reference materialises one dk/dv per member and sums, :687-692,813).
//
// Two kernels on the forward pass's tile engine.  A wavefront keeps 32
// "resident" rows (their B operands) in registers and streams 64-row tiles of
// the other side through a three-stage LDS ring (direct-to-LDS loads).
//   dQ     : resident q, do rows; streams K, V.
//            S^T = K Q^T, dP^T = V dO^T, dQ^T += K^T dS^T
//            It also forms Delta of its resident rows (one pass over the o
//            rows) and stores it for the second kernel, which runs after it.
//   dK + dV: resident k, v rows; streams Q, dO (all query heads of the GQA
//            group in turn).  The work of a 32-row group is split between two
//            wavefronts that share a SIMD: one forms S, P and dV^T += dO^T P,
//            the other dP, dS and dK^T += Q^T dS (see bwd_dkdv_item).
// In every first product 16 streamed rows of ONE resident row land in each
// lane, and the rounded, pairwise packed result already is the B operand of
// the accumulating product; its A operand is a streamed tile read through the
// transposing LDS load.  Every streamed tile uses one layout that serves both
// the row-fragment read and the transposing read (UniFrags).
#include <type_traits>

#include "kernels.h"
#include "tile_core.h"

namespace mi {
namespace {

template <int V>
using ic = std::integral_constant<int, V>;

// f(ic<B>{}), f(ic<B + 1>{}), ..., f(ic<E - 1>{})
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(ic<B>{});
    static_for<B + 1, E>(f);
  }
}

// vmcnt(N) expcnt(7) lgkmcnt(15) for s_waitcnt on gfx9-family encodings
constexpr int waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }
// vmcnt(63) expcnt(7) lgkmcnt(N)
constexpr int waitcnt_lgkm(int n) { return 0xF | (3 << 14) | (7 << 4) | ((n & 0xF) << 8); }

// 256-byte rows (head_dim 64 and 96 leave the tail of a row unused), 16-byte
// chunks XOR-swizzled per row with a pattern
// that is free of bank conflicts for BOTH access patterns: a row-fragment read
// takes one chunk from 16 rows whose low four row bits are all different, a
// transposing read takes four consecutive chunks from four consecutive rows.
template <int D>
struct UniFrags {
  using G = RowGeom<D>;
  static constexpr int ROWB = 256;
  static constexpr int SLOTS = 16;
  static __device__ __forceinline__ int swz(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }
  int lq, lh;
  uint32_t r_a[G::KSTEPS];  // absolute LDS address of row fragment step c, block 0 of tile 0
  uint32_t t_a[G::NDB][2];  // same for the transposing read of (d block, first/second half)

  __device__ __forceinline__ void init(int lane, uint32_t lds_base) {
    lq = lane & 31;
    lh = lane >> 5;
    const int krow = key_perm(lq);
#pragma unroll
    for (int c = 0; c < G::KSTEPS; ++c) {
      r_a[c] = lds_base + krow * ROWB + (((2 * c + lh) ^ swz(krow)) << 4);
      asm volatile("" : "+v"(r_a[c]));
    }
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int r = 8 * lh + 4 * e + ((lane & 15) >> 2);
#pragma unroll
      for (int db = 0; db < G::NDB; ++db) {
        const int ch = 4 * db + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
        t_a[db][e] = lds_base + r * ROWB + ((ch ^ swz(r)) << 4) + (lane & 1) * 8;
        asm volatile("" : "+v"(t_a[db][e]));
      }
    }
  }
  // swz is invariant under row += 16, so blocks are plain immediates
  __device__ __forceinline__ i32x4 rows(uint32_t tile_off, int blk, int c) const {
    typedef __attribute__((address_space(3))) const i32x4 lds_i32x4;
    return *(lds_i32x4*)(uintptr_t)(r_a[c] + tile_off + blk * 32 * ROWB);
  }
  __device__ __forceinline__ i32x4 tr(uint32_t tile_off, int kk, int db) const {
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(uintptr_t)(t_a[db][0] + tile_off + kk * 16 * ROWB));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(uintptr_t)(t_a[db][1] + tile_off + kk * 16 * ROWB));
    i32x2 l2 = __builtin_bit_cast(i32x2, lo);
    i32x2 h2 = __builtin_bit_cast(i32x2, hi);
    i32x4 out = {l2[0], l2[1], h2[0], h2[1]};
    return out;
  }
};

extern __shared__ __attribute__((aligned(1024))) unsigned char smem_bwd[];

constexpr int kBwdStages = 3;  // streamed tile pairs resident in LDS (4 measured the same)

// dQ: resident q, do rows; streams K, V.
//   S^T = K Q^T,  dP^T = V dO^T,  dS = P o (dP - Delta),  dQ^T += K^T dS^T
template <typename T, int D>
__device__ __forceinline__ void bwd_dq_item(const BwdParams& p, const int bid) {
  using G = RowGeom<D>;
  using F = UniFrags<D>;
  constexpr int NW = 8, BM = 32 * NW, TN = 64, NS = kBwdStages;
  constexpr int TILEB = TN * F::ROWB;             // one streamed tile
  constexpr int STAGEB = 2 * TILEB + 1024;        // tile 0, tile 1, lse[64] and delta[64] (fp32)
  constexpr int RPI = 1024 / F::ROWB;             // tile rows per direct-to-LDS instruction
  constexpr int IPW = TN / RPI / NW;              // such instructions per tile and wave
  constexpr int IPT = 2 * IPW;                    // loads per streamed tile and wave
  constexpr int OROWB = D * 2 + 16;               // epilogue staging row

  const int tid = threadIdx.x;
  int lane = tid & 63;
  // An opaque copy per item: what is derived from the lane id (fragment
  // addresses, load offsets) is then recomputed for every item instead of
  // being held in registers across the whole item loop, where it was spilled.
  asm volatile("" : "+v"(lane));
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int heads_r = p.hq;
  const int gqa = p.hq / p.hkv;
  // Work item -> (sequence, resident head, resident tile).  Consecutive ids go
  // round-robin to the 8 XCDs (private L2 each): give every XCD whole
  // (sequence, head) units so the streamed tensors of a unit stay in one L2,
  // and walk a unit's tiles from the one that streams most to the one that
  // streams least (causal: the last q tile).
  const int n_units = p.batch * heads_r;
  int unit, slot;
  {
    if ((n_units & 7) == 0) {
      const int sl = bid >> 3;
      unit = (sl / p.n_rtiles) * 8 + (bid & 7);
      slot = sl % p.n_rtiles;
    } else {
      unit = bid / p.n_rtiles;
      slot = bid % p.n_rtiles;
    }
  }
  const int rt = p.n_rtiles - 1 - slot;
  const int hr = unit % heads_r;
  const int b = unit / heads_r;

  int len;
  int64_t start;  // first row of the sequence in packed tensors
  if (p.cu) {
    start = p.cu[b];
    // never beyond the bound the workspace and the grid were sized for
    len = min(p.cu[b + 1] - (int)start, p.max_seqlen);
  } else {
    start = 0;
    len = p.max_seqlen;
  }
  const int64_t bsel = p.cu ? 0 : b;
  const int r0 = rt * BM;
  if (r0 >= len) return;

  F fr;
  const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem_bwd);
  fr.init(lane, lds0);
  const int r0w = r0 + 32 * wave;
  const int rrow = r0w + fr.lq;                 // resident row of this lane
  const int rclamp = min(rrow, len - 1);

  // ---- resident B operands: lane (row lq, half lh) holds d = 16c + 8lh .. +7
  const T* xp = reinterpret_cast<const T*>(p.q) + bsel * p.q_sb + (start + rclamp) * p.q_ss + hr * p.q_sh;
  const T* yp = reinterpret_cast<const T*>(p.dout) + bsel * p.do_sb + (start + rclamp) * p.do_ss + hr * p.do_sh;
  const T* op = reinterpret_cast<const T*>(p.o) + bsel * p.o_sb + (start + rclamp) * p.o_ss + hr * p.o_sh;
  i32x4 Xf[G::KSTEPS], Yf[G::KSTEPS];
  // Delta[row] = sum_d o[row][d] * do[row][d] (fp32) is formed here, from the
  // resident do rows and one pass over the o rows, and stored for the dK + dV
  // kernel, which runs after this one.
  float delta_l = 0.f;
#pragma unroll
  for (int c = 0; c < G::KSTEPS; ++c) {
    Xf[c] = *reinterpret_cast<const i32x4*>(xp + 8 * fr.lh + 16 * c);
    Yf[c] = *reinterpret_cast<const i32x4*>(yp + 8 * fr.lh + 16 * c);
    const i32x4 Of = *reinterpret_cast<const i32x4*>(op + 8 * fr.lh + 16 * c);
    const T* oe = reinterpret_cast<const T*>(&Of);
    const T* de = reinterpret_cast<const T*>(&Yf[c]);
#pragma unroll
    for (int i = 0; i < 8; ++i) delta_l += (float)oe[i] * (float)de[i];
  }
  delta_l += __shfl_xor(delta_l, 32);
  if (fr.lh == 0 && rrow < len) p.delta[(int64_t)b * p.dl_sb + (int64_t)hr * p.dl_sh + rrow] = delta_l;
  const float lse_l = p.lse[bsel * p.lse_sb + (start + rclamp) * p.lse_ss + hr * p.lse_sh];

  f32x16 acc[G::NDB];
#pragma unroll
  for (int db = 0; db < G::NDB; ++db) acc[db] = (f32x16){0};

  // ---- streamed tiles: which rows, for which heads
  const int n_all = (len + TN - 1) / TN;
  const int n_stream = p.causal ? min(n_all, (r0 + BM + TN - 1) / TN) : n_all;  // key tiles 0 .. n_stream - 1

  // ---- direct-to-LDS loads (inline assembly: see the note in prefill.hip)
  const int drow = lane / F::SLOTS, dslot = lane % F::SLOTS;
  auto uniform64 = [](uint64_t x) __attribute__((always_inline)) -> uint64_t {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)x);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
    return ((uint64_t)hi << 32) | lo;
  };
  // a load of the lanes in `mask` in straight-line code (all lanes are active
  // and control flow is wave-uniform here: exec is restored to all ones)
  auto dma_masked = [&](uint64_t mask, uint64_t base, uint32_t off, uint32_t slab) __attribute__((always_inline)) {
    asm volatile("s_mov_b32 m0, %3\n\ts_mov_b64 exec, %0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, -1"
                 : : "s"(mask), "v"(off), "s"(base), "s"(slab) : "memory");
  };
  // Streamed tensors: K feeds the first product and, transposed, the last; V
  // the second.  Wave w sends slabs w and w + 8 (1 KiB = four rows) of either
  // tile; the swizzle of a lane's chunk depends on the slab only through
  // slab % 4, so one lane offset per tensor serves both and the slab moves the
  // scalar base.  The tile addresses are running, wave-uniform values.
  const int64_t pitch0 = p.k_ss * 2, pitch1 = p.v_ss * 2;
  const int hs = hr / gqa;
  const char* h0 = reinterpret_cast<const char*>(reinterpret_cast<const T*>(p.k) + bsel * p.k_sb + start * p.k_ss + hs * p.k_sh);
  const char* h1 = reinterpret_cast<const char*>(reinterpret_cast<const T*>(p.v) + bsel * p.v_sb + start * p.v_ss + hs * p.v_sh);
  uint64_t a0 = uniform64((uint64_t)(uintptr_t)h0), a1 = uniform64((uint64_t)(uintptr_t)h1);
  const uint64_t step0 = uniform64((uint64_t)(TN * pitch0)), step1 = uniform64((uint64_t)(TN * pitch1));
  const uint64_t slab0 = uniform64((uint64_t)(NW * RPI * pitch0)), slab1 = uniform64((uint64_t)(NW * RPI * pitch1));
  uint32_t off0, off1;
  uint64_t lane_mask;
  {
    const int r = RPI * wave + drow;
    const int c = dslot ^ F::swz(r);
    off0 = (uint32_t)r * (uint32_t)pitch0 + c * 16;
    off1 = (uint32_t)r * (uint32_t)pitch1 + c * 16;
    lane_mask = __builtin_amdgcn_ballot_w64(G::NCH == 16 || c < G::NCH);
  }
  static_assert(IPT == 4, "compute_fast() places four loads");
  int iss_s0 = 0;            // first row of the next request
  int iss_st = 0;            // its stage
  uint32_t iss_base = lds0;  // and the stage's LDS address
  uint64_t drip_on = 0;      // all ones while the loads of a request are still to be sent by a compute step
  // request(): a tile that reaches past the sequence end is loaded at once,
  // row by row with clamped row numbers (masked later); a whole tile only arms
  // drip(), and the compute step sends the four loads between its MFMAs.
  auto request = [&]() __attribute__((always_inline)) {
    if (iss_s0 + TN <= len) {
      drip_on = ~0ull;
    } else {
      drip_on = 0;
      const int last = len - 1 - iss_s0;  // >= 0
#pragma unroll
      for (int t = 0; t < IPW; ++t) {
        const int inst = wave + NW * t;
        const int r = RPI * inst + drow;
        const int c = dslot ^ F::swz(r);
        const int64_t rr = min(r, last);
        const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(iss_base + inst * 1024);
        if (G::NCH == 16 || c < G::NCH) {
          asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                       : : "v"((const char*)a0 + rr * pitch0 + c * 16), "s"(slab) : "memory");
          asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                       : : "v"((const char*)a1 + rr * pitch1 + c * 16), "s"(slab + TILEB) : "memory");
        }
      }
    }
  };
  // load k of a request: k & 1 = tensor, k >> 1 = slab
  auto drip = [&](int k) __attribute__((always_inline)) {
    const int t = k >> 1;
    const int inst = wave + NW * t;
    if (k & 1)
      dma_masked(drip_on & lane_mask, a1 + t * slab1, off1, iss_base + TILEB + inst * 1024);
    else
      dma_masked(drip_on & lane_mask, a0 + t * slab0, off0, iss_base + inst * 1024);
  };
  auto drip_all = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int k = 0; k < IPT; ++k) drip(k);
  };
  auto advance = [&]() __attribute__((always_inline)) {
    drip_on = 0;
    iss_s0 += TN;
    a0 += step0;
    a1 += step1;
    const bool last_st = iss_st == NS - 1;
    iss_st = last_st ? 0 : iss_st + 1;
    iss_base = last_st ? lds0 : iss_base + STAGEB;
  };

  const float scale = p.scale;
  const int causal = p.causal;

  // ---- this wave's view of the tile it works on: LDS addresses that move
  // from stage to stage (one add per address register and step; every read is
  // then "register + immediate": absolute stage offsets exceed the 16-bit
  // immediate of an LDS instruction)
  int cmp_st = 0;
  auto rotate = [&]() __attribute__((always_inline)) {
    const bool last_st = cmp_st == NS - 1;
    const int d = last_st ? -(NS - 1) * STAGEB : STAGEB;
    cmp_st = last_st ? 0 : cmp_st + 1;
#pragma unroll
    for (int c = 0; c < G::KSTEPS; ++c) fr.r_a[c] += d;
#pragma unroll
    for (int db = 0; db < G::NDB; ++db) {
      fr.t_a[db][0] += d;
      fr.t_a[db][1] += d;
    }
  };

  constexpr int kPrefetch = 4;
  constexpr int K = G::KSTEPS;
  // slice of block 0's S chain behind which the n-th of a tile's four loads goes
  auto drip_slice = [](int n) constexpr { return K == 8 ? 2 * n + 1 : K == 6 ? n + 1 + (n >= 2) : n; };
  i32x4 f[kPrefetch];   // row fragments of the first two products, read ahead
  // One 32-row block of the streamed tile as one pinned instruction stream
  // (sched_barrier(0) after every slice): the S chain; the dP chain with the
  // exponentials of S behind its MFMAs; the first half of dS; the last product
  // with the second half of dS behind its first MFMAs.  Row fragments are read
  // four steps ahead, transposed fragments two.  Register r of this lane is
  // streamed row  sblk + 16*(r/8) + 8*lh + r%8.
  auto block = [&](auto sb_c, auto masked_c, const int sblk, const bool f_ready) __attribute__((always_inline)) {
    constexpr int sb = decltype(sb_c)::value;
    constexpr bool masked = decltype(masked_c)::value != 0;
    constexpr int NSTEP = 2 * K;
    f32x16 S = (f32x16){0}, dP = (f32x16){0};
    auto frag = [&](int st) __attribute__((always_inline)) -> i32x4 {
      return st < K ? fr.rows(0, sb, st) : fr.rows(TILEB, sb, st - K);
    };
    auto prob = [&](int r) __attribute__((always_inline)) {   // S[r] <- P[r]
      S[r] = fast_exp2(fmaf(S[r], scale, -lse_l));
    };
    auto dsv = [&](int r) __attribute__((always_inline)) -> float {
      return S[r] * (dP[r] - delta_l);
    };
    if (!f_ready) {
#pragma unroll
      for (int st = 0; st < kPrefetch; ++st) f[st] = frag(st);
    }
    // Issue priority: highest while the wave feeds the accumulators (the last
    // product, 2*NDB MFMAs over NDB independent chains), low during the two
    // serial chains S and dP; the two waves of a SIMD then fall out of step
    // instead of competing with the same kind of work (measured 3 %).
    __builtin_amdgcn_s_setprio(1);
    static_for<0, K>([&](auto st_c) __attribute__((always_inline)) {
      constexpr int st = decltype(st_c)::value;
      S = Elem<T>::mfma(f[st % kPrefetch], Xf[st], S);
      if (st + kPrefetch < NSTEP) f[st % kPrefetch] = frag(st + kPrefetch);
      if (sb == 0 && !masked)
        static_for<0, IPT>([&](auto n_c) __attribute__((always_inline)) {
          if (st == drip_slice(decltype(n_c)::value)) drip(decltype(n_c)::value);
        });
      __builtin_amdgcn_sched_barrier(0);
    });
    if (masked) {
      // rows / columns that do not exist or lie above the diagonal give P = 0
      bool need_mask = sblk + 32 > len;
      if (causal) need_mask = need_mask || sblk + 31 > r0w;
      if (need_mask) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int srow = sblk + 16 * (r >> 3) + 8 * fr.lh + (r & 7);
          const bool ok = srow < len && (!causal || srow <= rrow);
          S[r] = ok ? S[r] : -INFINITY;
        }
      }
    }
    i32x4 tf[2];
    uint32_t W[8];
#pragma unroll
    for (int c = 0; c < K; ++c) {
      const int st = K + c;
      dP = Elem<T>::mfma(f[st % kPrefetch], Yf[c], dP);
      if (st + kPrefetch < NSTEP) f[st % kPrefetch] = frag(st + kPrefetch);
      if (c >= K - 2) tf[c - (K - 2)] = fr.tr(0, 2 * sb, c - (K - 2));
      // 16 exponentials spread over the K slices
#pragma unroll
      for (int r = 16 * c / K; r < 16 * (c + 1) / K; ++r) prob(r);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) W[i] = Elem<T>::pack2(dsv(2 * i), dsv(2 * i + 1));
    __builtin_amdgcn_sched_barrier(0);
    // last product: 2*NDB MFMAs, fragment (kk, db) = step kk*NDB + db
    constexpr int NACC = 2 * G::NDB;
    __builtin_amdgcn_s_setprio(3);
#pragma unroll
    for (int i = 0; i < NACC; ++i) {
      const int kk = i / G::NDB, db = i % G::NDB;
      const i32x4 wf = {(int)W[4 * kk], (int)W[4 * kk + 1], (int)W[4 * kk + 2], (int)W[4 * kk + 3]};
      acc[db] = Elem<T>::mfma(tf[i & 1], wf, acc[db]);
      if (i + 2 < NACC) tf[i & 1] = fr.tr(0, 2 * sb + (i + 2) / G::NDB, (i + 2) % G::NDB);
      // the ring is idle now: fetch the first fragments of the tile's second block
      if (sb == 0 && i >= NACC - kPrefetch) f[i - (NACC - kPrefetch)] = fr.rows(0, 1, i - (NACC - kPrefetch));
      if (i < G::NDB) {
        // second half of dS (8 values) spread over the first NDB slices
#pragma unroll
        for (int q = 4 * i / G::NDB; q < 4 * (i + 1) / G::NDB; ++q)
          W[4 + q] = Elem<T>::pack2(dsv(8 + 2 * q), dsv(9 + 2 * q));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // a tile whose 64 keys all exist and lie at or before this wave's first query
  auto compute_fast = [&](int s0) __attribute__((always_inline)) {
    block(ic<0>{}, ic<0>{}, s0, false);
    block(ic<1>{}, ic<0>{}, s0 + 32, true);
  };
  // a tile on the diagonal or at the sequence end
  auto compute_slow = [&](int s0) __attribute__((always_inline)) {
    drip_all();
    bool f_ready = false;
    if (s0 < len && !(causal && s0 > r0w + 31)) {
      block(ic<0>{}, ic<1>{}, s0, false);
      f_ready = true;
    }
    if (s0 + 32 < len && !(causal && s0 + 32 > r0w + 31)) block(ic<1>{}, ic<1>{}, s0 + 32, f_ready);
  };

  // tiles 0 .. NS-2 are requested up front; step u requests tile u + NS - 1
  // into the stage that tile u - 1 has left
#pragma unroll
  for (int u = 0; u < NS - 1; ++u)
    if (u < n_stream) {
      request();
      drip_all();
      advance();
    }
  // resident operands and tile 0 are needed now; the full wait also tells the
  // compiler that no register load is pending inside the loop
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
  __syncthreads();
  // Each loop below holds ONE kind of step (with the masked and the unmasked
  // path in one loop body the accumulators were copied between two register
  // sets on every trip); every step ends in the workgroup's barrier, so the
  // waves may split the tiles differently.
  int n_fast = min(n_stream, len / TN);
  if (causal) n_fast = min(n_fast, (r0w + 1) / TN);
  auto step = [&](auto fast_c, int u) __attribute__((always_inline)) {
    const bool refill = u + NS - 1 < n_stream;
    if (refill) request();
    if (decltype(fast_c)::value)
      compute_fast(u * TN);
    else
      compute_slow(u * TN);
    rotate();
    if (refill) advance();
    // the next tile must have landed (this wave's loads retire in order: only
    // the tile requested in this step may still fly) and everyone is done with this one
    if (refill)
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(IPT));
    else
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __syncthreads();
  };
  for (int u = 0; u < n_fast; ++u) step(ic<1>{}, u);
  for (int u = n_fast; u < n_stream; ++u) step(ic<0>{}, u);
  __builtin_amdgcn_s_setprio(0);
  __syncthreads();

  // ---- epilogue: scale, transpose through LDS, coalesced 16-byte stores
  const float oscale = p.scale_nat;
  T* outp = reinterpret_cast<T*>(p.dq) + bsel * p.dq_sb + start * p.dq_ss + hr * p.dq_sh;
  const int64_t o_ss = p.dq_ss;
  unsigned char* stage = smem_bwd + wave * 32 * OROWB;
#pragma unroll
  for (int db = 0; db < G::NDB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = 32 * db + 8 * g + 4 * fr.lh;
      i32x2 w;
      w[0] = (int)Elem<T>::pack2(acc[db][4 * g] * oscale, acc[db][4 * g + 1] * oscale);
      w[1] = (int)Elem<T>::pack2(acc[db][4 * g + 2] * oscale, acc[db][4 * g + 3] * oscale);
      *reinterpret_cast<i32x2*>(stage + fr.lq * OROWB + d * 2) = w;
    }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < (32 * G::NCH + 63) / 64; ++i) {
    const int idx = lane + 64 * i;
    const int row = idx / G::NCH, ch = idx % G::NCH;
    if (((32 * G::NCH) % 64 == 0 || idx < 32 * G::NCH) && r0w + row < len) {
      const i32x4 val = *reinterpret_cast<const i32x4*>(stage + row * OROWB + ch * 16);
      *reinterpret_cast<i32x4*>(outp + (int64_t)(r0w + row) * o_ss + ch * 8) = val;
    }
  }
}

// ---------------------------------------------------------------------------
// dK and dV in one pass (replaces flash_attn_bwd_dkdv_kernel,
// flash_attn_triton/flash_attn_triton.py:413-592, which also forms both in one
// kernel).  Both accumulators of 32 resident k / v rows (2 x 64 registers at
// head_dim 128) plus the two resident B operands do not fit one wavefront at
// two wavefronts per SIMD, so the work of a 32-row group is split between TWO
// wavefronts that share a SIMD (waves w and w + 4):
//   score wave:  S = Q K^T -> P = 2^(S scale - lse),   dV^T += dO^T P
//   grad wave :  dP = dO V^T, dS = P o (dP - Delta),   dK^T += Q^T dS
// Each holds one resident operand (k or v), one accumulator, and runs half of
// the MFMAs; S and P are computed once for both gradients and Q / dO are
// streamed once.  P travels from the score wave to the grad wave through LDS,
// rounded to the storage dtype (the operand of dV; the reference forms dS from
// the fp32 P, :578): the score wave works one streamed tile AHEAD of the grad
// wave, so the barrier that ends a tile step is the only synchronisation.
template <typename T, int D>
__device__ __forceinline__ void bwd_dkdv_item(const BwdParams& p, const int bid, const int n_rt) {
  using G = RowGeom<D>;
  using F = UniFrags<D>;
  constexpr int NP = 4, BM = 32 * NP, TN = 64, NS = kBwdStages;
  static_assert(NS == 3, "stage reuse below assumes three stages");
  constexpr int TILEB = TN * F::ROWB;
  constexpr int STAGEB = 2 * TILEB + 1024;
  constexpr int RPI = 1024 / F::ROWB;
  constexpr int OROWB = D * 2 + 16;
  constexpr uint32_t PBUF = NS * STAGEB;       // P exchange: [2 tile slots][NP pairs][2 blocks][2 KiB]
  constexpr uint32_t PSLOT = NP * 2 * 2048;

  const int tid = threadIdx.x;
  int lane = tid & 63;
  asm volatile("" : "+v"(lane));
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pr = wave & 3;            // 32-row group of the item
  const bool grad = wave >= 4;        // role of this wave

  const int gqa = p.hq / p.hkv;
  const int n_units = p.batch * p.hkv;
  int unit, slot;
  if ((n_units & 7) == 0) {
    const int sl = bid >> 3;
    unit = (sl / n_rt) * 8 + (bid & 7);
    slot = sl % n_rt;
  } else {
    unit = bid / n_rt;
    slot = bid % n_rt;
  }
  const int rt = slot;  // causal: the first key tile streams most
  const int hr = unit % p.hkv;
  const int b = unit / p.hkv;

  int len;
  int64_t start;
  if (p.cu) {
    start = p.cu[b];
    // never beyond the bound the workspace and the grid were sized for
    len = min(p.cu[b + 1] - (int)start, p.max_seqlen);
  } else {
    start = 0;
    len = p.max_seqlen;
  }
  const int64_t bsel = p.cu ? 0 : b;
  const int r0 = rt * BM;
  if (r0 >= len) return;

  F fr;
  const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem_bwd);
  fr.init(lane, lds0);
  const int r0w = r0 + 32 * pr;
  const int rrow = r0w + fr.lq;
  const int rclamp = min(rrow, len - 1);

  // resident B operand: k rows (score wave) or v rows (grad wave)
  const T* xp = grad ? reinterpret_cast<const T*>(p.v) + bsel * p.v_sb + (start + rclamp) * p.v_ss + hr * p.v_sh
                     : reinterpret_cast<const T*>(p.k) + bsel * p.k_sb + (start + rclamp) * p.k_ss + hr * p.k_sh;
  i32x4 Xf[G::KSTEPS];
#pragma unroll
  for (int c = 0; c < G::KSTEPS; ++c) Xf[c] = *reinterpret_cast<const i32x4*>(xp + 8 * fr.lh + 16 * c);

  f32x16 acc[G::NDB];
#pragma unroll
  for (int db = 0; db < G::NDB; ++db) acc[db] = (f32x16){0};

  const int n_all = (len + TN - 1) / TN;
  const int j0 = p.causal ? r0 / TN : 0;
  const int nj = n_all - j0;
  const int n_stream = nj * gqa;

  const int drow = lane / F::SLOTS, dslot = lane % F::SLOTS;
  auto uniform64 = [](uint64_t x) __attribute__((always_inline)) -> uint64_t {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)x);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
    return ((uint64_t)hi << 32) | lo;
  };
  // A direct-to-LDS load of the lanes in `mask` (all 64 lanes are active and
  // control flow is wave-uniform wherever this is called, so exec is restored
  // to all ones).  Switching a load off through the exec mask keeps it in
  // straight-line code: a branch around it would end the basic block and let
  // the compiler move the arithmetic that is meant to sit behind the MFMAs.
  auto dma_masked = [&](uint64_t mask, uint64_t base, uint32_t off, uint32_t slab, auto wide_c) __attribute__((always_inline)) {
    if (decltype(wide_c)::value)
      asm volatile("s_mov_b32 m0, %3\n\ts_mov_b64 exec, %0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, -1"
                   : : "s"(mask), "v"(off), "s"(base), "s"(slab) : "memory");
    else
      asm volatile("s_mov_b32 m0, %3\n\ts_mov_b64 exec, %0\n\tglobal_load_lds_dword %1, %2\n\ts_mov_b64 exec, -1"
                   : : "s"(mask), "v"(off), "s"(base), "s"(slab) : "memory");
  };

  // ---- streamed tiles.  Per tile and wavefront: four loads of 1 KiB (two of
  // Q, two of dO); wavefronts 0 and 1 also fetch the tile's 64 lse / Delta
  // values.  The addresses are running, wave-uniform values: they advance by
  // one tile per request and jump to the next query head of the group when a
  // head's tiles are through (one add each per step; the item's scalar
  // bookkeeping is issued by the same wavefronts that feed the MFMAs, one
  // instruction per four cycles, so every instruction saved per step counts).
  const int64_t pitch0 = p.q_ss * 2, pitch1 = p.do_ss * 2;
  const char* h0 = reinterpret_cast<const char*>(reinterpret_cast<const T*>(p.q) + bsel * p.q_sb + (start + j0 * TN) * p.q_ss + hr * gqa * p.q_sh);
  const char* h1 = reinterpret_cast<const char*>(reinterpret_cast<const T*>(p.dout) + bsel * p.do_sb + (start + j0 * TN) * p.do_ss + hr * gqa * p.do_sh);
  const char* hl = wave == 0
      ? reinterpret_cast<const char*>(p.lse + bsel * p.lse_sb + (start + j0 * TN) * p.lse_ss + hr * gqa * p.lse_sh)
      : reinterpret_cast<const char*>(p.delta + (int64_t)b * p.dl_sb + (int64_t)hr * gqa * p.dl_sh + j0 * TN);
  const int64_t pitchl = wave == 0 ? p.lse_ss * 4 : 4;
  uint64_t a0 = uniform64((uint64_t)(uintptr_t)h0), a1 = uniform64((uint64_t)(uintptr_t)h1), al = uniform64((uint64_t)(uintptr_t)hl);
  const uint64_t step0 = uniform64((uint64_t)(TN * pitch0)), step1 = uniform64((uint64_t)(TN * pitch1));
  const uint64_t stepl = uniform64((uint64_t)(TN * pitchl));
  const uint64_t wrap0 = uniform64((uint64_t)(p.q_sh * 2 - (int64_t)(nj - 1) * TN * pitch0));
  const uint64_t wrap1 = uniform64((uint64_t)(p.do_sh * 2 - (int64_t)(nj - 1) * TN * pitch1));
  const uint64_t wrapl = uniform64((uint64_t)((wave == 0 ? p.lse_sh * 4 : p.dl_sh * 4) - (int64_t)(nj - 1) * TN * pitchl));
  // The four score wavefronts send the loads (the grad wavefronts carry more
  // arithmetic per tile): wave pr sends slabs pr, pr + 4, pr + 8, pr + 12 of
  // the Q tile and of the dO tile (1 KiB = four rows each).  The swizzle of a
  // lane's chunk depends on the slab only through slab % 4, so one lane offset
  // per tensor serves all four slabs; the slab moves the scalar base.
  constexpr int kSlabs = TN / RPI / NP;      // slabs per tensor, tile and score wave
  constexpr int kDrips = 2 * kSlabs;
  static_assert(kDrips == 8, "compute_fast() places eight loads");
  uint32_t off0, off1;
  uint64_t lane_mask;
  {
    const int r = RPI * pr + drow;
    const int c = dslot ^ F::swz(r);
    off0 = (uint32_t)r * (uint32_t)pitch0 + c * 16;
    off1 = (uint32_t)r * (uint32_t)pitch1 + c * 16;
    lane_mask = __builtin_amdgcn_ballot_w64(G::NCH == 16 || c < G::NCH);
  }
  const uint64_t slab0 = uniform64((uint64_t)(NP * RPI * pitch0)), slab1 = uniform64((uint64_t)(NP * RPI * pitch1));
  const uint32_t lv_off = (uint32_t)lane * (uint32_t)pitchl;
  const uint64_t lv_mask = wave < 2 ? ~0ull : 0ull;
  int iss_left = nj;        // tiles of the current head still to request
  int iss_s0 = j0 * TN;     // first row of the next request
  int iss_st = 0;           // its stage
  uint32_t iss_base = lds0; // and the stage's LDS address
  uint64_t drip_on = 0;     // all ones while the loads of a request are still to be sent by compute_fast()
  // request(): a tile that reaches past the sequence end is loaded at once,
  // row by row with clamped row numbers (masked later); a full tile only arms
  // drip(), and compute_fast() sends the loads between its MFMAs: wavefronts
  // that send their loads together right after the barrier stand in the
  // memory pipeline's queue before any of them starts its arithmetic.
  auto request = [&]() __attribute__((always_inline)) {
    if (iss_s0 + TN <= len) {
      drip_on = ~0ull;
    } else {
      drip_on = 0;
      if (grad) return;
      const int last = len - 1 - iss_s0;  // >= 0
#pragma unroll
      for (int t = 0; t < kSlabs; ++t) {
        const int inst = pr + NP * t;
        const int r = RPI * inst + drow;
        const int c = dslot ^ F::swz(r);
        const int64_t rr = min(r, last);
        const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(iss_base + inst * 1024);
        if (G::NCH == 16 || c < G::NCH) {
          asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                       : : "v"((const char*)a0 + rr * pitch0 + c * 16), "s"(slab) : "memory");
          asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                       : : "v"((const char*)a1 + rr * pitch1 + c * 16), "s"(slab + TILEB) : "memory");
        }
      }
      if (wave < 2) {
        const int64_t rr = min(lane, last);
        const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(iss_base + 2 * TILEB + (wave == 0 ? 0 : 256));
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
                     : : "v"((const char*)al + rr * pitchl), "s"(slab) : "memory");
      }
    }
  };
  // load k of a request (score waves): k & 1 = tensor, k >> 1 = slab
  auto drip = [&](int k) __attribute__((always_inline)) {
    const int t = k >> 1;
    const int inst = pr + NP * t;
    if (k & 1)
      dma_masked(drip_on & lane_mask, a1 + t * slab1, off1, iss_base + TILEB + inst * 1024, ic<1>{});
    else
      dma_masked(drip_on & lane_mask, a0 + t * slab0, off0, iss_base + inst * 1024, ic<1>{});
    if (k == 0) dma_masked(drip_on & lv_mask, al, lv_off, iss_base + 2 * TILEB + (wave == 0 ? 0 : 256), ic<0>{});
  };
  auto drip_all = [&]() __attribute__((always_inline)) {
    if (grad) return;
#pragma unroll
    for (int k = 0; k < kDrips; ++k) drip(k);
  };
  // after the loads of a request are out: the next request's addresses
  auto advance = [&]() __attribute__((always_inline)) {
    drip_on = 0;
    if (--iss_left == 0) {
      iss_left = nj;
      iss_s0 = j0 * TN;
      a0 += wrap0;
      a1 += wrap1;
      al += wrapl;
    } else {
      iss_s0 += TN;
      a0 += step0;
      a1 += step1;
      al += stepl;
    }
    const bool last_st = iss_st == NS - 1;
    iss_st = last_st ? 0 : iss_st + 1;
    iss_base = last_st ? lds0 : iss_base + STAGEB;
  };

  const float scale = p.scale;
  const int causal = p.causal;
  typedef __attribute__((address_space(3))) i32x4 lds_i32x4;
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) const f32x4 lds_f4;

  // ---- this wave's view of the tile it works on: LDS addresses that move
  // from stage to stage (one add per address register and step, every read
  // then is "register + immediate"; absolute stage offsets exceed the 16-bit
  // immediate of an LDS instruction)
  {
    const uint32_t tro = grad ? TILEB : 0;   // tile read as row fragments: dO (grad) / Q (score)
    const uint32_t tto = grad ? 0 : TILEB;   // tile read transposed for the accumulating product
#pragma unroll
    for (int c = 0; c < G::KSTEPS; ++c) fr.r_a[c] += tro;
#pragma unroll
    for (int db = 0; db < G::NDB; ++db) {
      fr.t_a[db][0] += tto;
      fr.t_a[db][1] += tto;
    }
  }
  uint32_t lva = lds0 + 2 * TILEB + (grad ? 256u : 0u) + 8 * fr.lh * 4;   // lse (score) / Delta (grad) of the tile's rows
  uint32_t pbv = lds0 + PBUF + (uint32_t)pr * 4096 + (uint32_t)lane * 16;   // P exchange slot of this 32-row group
  int pb_step = (int)PSLOT;
  int cmp_st = 0, cmp_left = nj, cmp_s0 = j0 * TN;
  const bool rows_full = r0w + 32 <= len;
  auto rotate = [&]() __attribute__((always_inline)) {
    const bool last_st = cmp_st == NS - 1;
    const int d = last_st ? -(NS - 1) * STAGEB : STAGEB;
    cmp_st = last_st ? 0 : cmp_st + 1;
#pragma unroll
    for (int c = 0; c < G::KSTEPS; ++c) fr.r_a[c] += d;
#pragma unroll
    for (int db = 0; db < G::NDB; ++db) {
      fr.t_a[db][0] += d;
      fr.t_a[db][1] += d;
    }
    lva += d;
    pbv += pb_step;
    pb_step = -pb_step;
    if (--cmp_left == 0) {
      cmp_left = nj;
      cmp_s0 = j0 * TN;
    } else {
      cmp_s0 += TN;
    }
  };

  constexpr int kPrefetch = 4;
  constexpr int NACC = 2 * G::NDB;
  // One streamed tile for this wave's role, common case: all 64 streamed rows
  // and all 32 resident rows exist and no pair is masked.  The two 32-row
  // blocks of the tile are worked on as one software pipeline, so that the
  // wave's vector arithmetic sits behind its own MFMAs:
  //   1. chain(0)                          3. accumulate(0)  + arithmetic(1)
  //   2. chain(1)  + arithmetic(0)         4. accumulate(1)
  auto compute_fast = [&](auto role_c) __attribute__((always_inline)) {
    constexpr bool grad = decltype(role_c)::value != 0;
    {
      // Slots of the pipeline: phase 1 is slots 0 .. K-1, phase 2 K .. 2K-1,
      // phase 3 2K .. 2K+NACC-1.  Pair i of block 0 is formed in phase 2,
      // pair j of block 1 in phase 3; the lse / Delta values (four per LDS
      // read) and the packed P a pair needs are read two slots earlier, so
      // that only a few of them are live at a time (registers).
      constexpr int K = G::KSTEPS;
      // slice of a chain phase behind which the n-th of its four loads goes
      auto drip_slice = [](int n) constexpr { return K == 8 ? 2 * n + 1 : K == 6 ? n + 1 + (n >= 2) : n; };
      auto slice_of = [](int i, int n) constexpr { int st = 0; while ((st + 1) * 8 / n <= i) ++st; return st; };
      auto use_slot = [&](int sb, int i) constexpr { return sb == 0 ? K + slice_of(i, K) : 2 * K + slice_of(i, NACC); };
      float lv[2][16];
      i32x4 pp[2][2];  // grad wave: packed P of the two blocks
      auto load_lv = [&](int sb, int q) __attribute__((always_inline)) {
        const f32x4 v4 = *(lds_f4*)(uintptr_t)(lva + (32 * sb + 16 * (q >> 1) + 4 * (q & 1)) * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) lv[sb][4 * q + e] = v4[e];
      };
      // reads due at `slot` (or, for slot 0, everything due at or before it)
      auto side_reads = [&](auto slot_c) __attribute__((always_inline)) {
        constexpr int slot = decltype(slot_c)::value;
#pragma unroll
        for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int due = use_slot(sb, 2 * q) - 2;
            if (due == slot || (slot == 0 && due < 0)) load_lv(sb, q);
          }
          if (grad) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              const int due = use_slot(sb, 4 * h) - 2;
              if (due == slot || (slot == 0 && due < 0)) pp[sb][h] = *(lds_i32x4*)(uintptr_t)(pbv + sb * 2048 + h * 1024);
            }
          }
        }
      };
      f32x16 S0 = (f32x16){0}, S1 = (f32x16){0};
      uint32_t W0[8], W1[8];
      // pair i of a block: P (score wave) or dS (grad wave), rounded and packed
      auto pair = [&](const f32x16& S, const float* lvb, const i32x4* ppb, int i) __attribute__((always_inline)) -> uint32_t {
        if (!grad) {
          return Elem<T>::pack2(fast_exp2(fmaf(S[2 * i], scale, -lvb[2 * i])),
                                fast_exp2(fmaf(S[2 * i + 1], scale, -lvb[2 * i + 1])));
        } else {
          const uint32_t pk = (uint32_t)(i < 4 ? ppb[0][i] : ppb[1][i - 4]);
          float plo, phi;
          if (std::is_same<T, __bf16>::value) {
            plo = __builtin_bit_cast(float, pk << 16);
            phi = __builtin_bit_cast(float, pk & 0xffff0000u);
          } else {
            const f16x2 h2 = __builtin_bit_cast(f16x2, pk);
            plo = (float)h2[0];
            phi = (float)h2[1];
          }
          return Elem<T>::pack2(plo * (S[2 * i] - lvb[2 * i]), phi * (S[2 * i + 1] - lvb[2 * i + 1]));
        }
      };
      i32x4 f[kPrefetch];
#pragma unroll
      for (int st = 0; st < kPrefetch; ++st) f[st] = st < K ? fr.rows(0, 0, st) : fr.rows(0, 1, st - K);
      __builtin_amdgcn_s_setprio(1);
      // 1. chain of block 0
      static_for<0, K>([&](auto st_c) __attribute__((always_inline)) {
        constexpr int st = decltype(st_c)::value;
        S0 = Elem<T>::mfma(f[st % kPrefetch], Xf[st], S0);
        constexpr int nx = st + kPrefetch;
        f[st % kPrefetch] = nx < K ? fr.rows(0, 0, nx) : fr.rows(0, 1, nx - K);
        side_reads(ic<st>{});
        if (!grad)
          static_for<0, 4>([&](auto n_c) __attribute__((always_inline)) {
            if (st == drip_slice(decltype(n_c)::value)) drip(decltype(n_c)::value);
          });
        __builtin_amdgcn_sched_barrier(0);
      });
      // 2. chain of block 1, arithmetic of block 0
      i32x4 tf[2];
      tf[0] = fr.tr(0, 0, 0);
      tf[1] = fr.tr(0, 0, 1);
      static_for<0, K>([&](auto st_c) __attribute__((always_inline)) {
        constexpr int st = decltype(st_c)::value;
        S1 = Elem<T>::mfma(f[(st + K) % kPrefetch], Xf[st], S1);
        constexpr int nx = st + kPrefetch;
        if (nx < K) f[(st + K) % kPrefetch] = fr.rows(0, 1, nx);
        side_reads(ic<K + st>{});
#pragma unroll
        for (int i = st * 8 / K; i < (st + 1) * 8 / K; ++i) {
          W0[i] = pair(S0, lv[0], pp[0], i);
          asm volatile("" : "+v"(W0[i]));  // computed here, behind this MFMA
        }
        if (!grad)
          static_for<0, 4>([&](auto n_c) __attribute__((always_inline)) {
            if (st == drip_slice(decltype(n_c)::value)) drip(4 + decltype(n_c)::value);
          });
        __builtin_amdgcn_sched_barrier(0);
      });
      if (!grad) {
        *(lds_i32x4*)(uintptr_t)(pbv) = (i32x4){(int)W0[0], (int)W0[1], (int)W0[2], (int)W0[3]};
        *(lds_i32x4*)(uintptr_t)(pbv + 1024) = (i32x4){(int)W0[4], (int)W0[5], (int)W0[6], (int)W0[7]};
      }
      __builtin_amdgcn_s_setprio(3);
      // 3. accumulating product of block 0, arithmetic of block 1
      static_for<0, NACC>([&](auto i_c) __attribute__((always_inline)) {
        constexpr int i = decltype(i_c)::value;
        constexpr int kk = i / G::NDB, db = i % G::NDB;
        const i32x4 wf = {(int)W0[4 * kk], (int)W0[4 * kk + 1], (int)W0[4 * kk + 2], (int)W0[4 * kk + 3]};
        acc[db] = Elem<T>::mfma(tf[i & 1], wf, acc[db]);
        constexpr int nx = i + 2;
        tf[i & 1] = nx < NACC ? fr.tr(0, nx / G::NDB, nx % G::NDB) : fr.tr(0, 2 + (nx - NACC) / G::NDB, (nx - NACC) % G::NDB);
        side_reads(ic<2 * K + i>{});
#pragma unroll
        for (int j = i * 8 / NACC; j < (i + 1) * 8 / NACC; ++j) {
          W1[j] = pair(S1, lv[1], pp[1], j);
          asm volatile("" : "+v"(W1[j]));
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      if (!grad) {
        *(lds_i32x4*)(uintptr_t)(pbv + 2048) = (i32x4){(int)W1[0], (int)W1[1], (int)W1[2], (int)W1[3]};
        *(lds_i32x4*)(uintptr_t)(pbv + 2048 + 1024) = (i32x4){(int)W1[4], (int)W1[5], (int)W1[6], (int)W1[7]};
      }
      // 4. accumulating product of block 1
#pragma unroll
      for (int i = 0; i < NACC; ++i) {
        const int kk = i / G::NDB, db = i % G::NDB;
        const i32x4 wf = {(int)W1[4 * kk], (int)W1[4 * kk + 1], (int)W1[4 * kk + 2], (int)W1[4 * kk + 3]};
        acc[db] = Elem<T>::mfma(tf[i & 1], wf, acc[db]);
        if (i + 2 < NACC) tf[i & 1] = fr.tr(0, 2 + (i + 2) / G::NDB, (i + 2) % G::NDB);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  // Tiles on the diagonal or at the sequence end: block by block, with masks.
  auto compute_slow = [&](auto role_c) __attribute__((always_inline)) {
    constexpr bool grad = decltype(role_c)::value != 0;
    const int s0 = cmp_s0;
    drip_all();
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      const int sblk = s0 + 32 * sb;
      if (sblk >= len) continue;
      if (causal && sblk + 31 < r0w) continue;  // queries before this group's first key
      // per streamed row: lse (score wave) or Delta (grad wave); register r of
      // this lane is streamed row  sblk + 16*(r/8) + 8*lh + r%8
      float vec_r[16];
#pragma unroll
      for (int g2 = 0; g2 < 2; ++g2)
#pragma unroll
        for (int q4 = 0; q4 < 2; ++q4) {
          const f32x4 v4 = *(lds_f4*)(uintptr_t)(lva + (32 * sb + 16 * g2 + 4 * q4) * 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) vec_r[8 * g2 + 4 * q4 + e] = v4[e];
        }
      // first product: rows of Q (score) / dO (grad) against the resident operand
      f32x16 S = (f32x16){0};
      i32x4 f[kPrefetch];
#pragma unroll
      for (int st = 0; st < kPrefetch; ++st) f[st] = fr.rows(0, sb, st);
      __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int st = 0; st < G::KSTEPS; ++st) {
        S = Elem<T>::mfma(f[st % kPrefetch], Xf[st], S);
        if (st + kPrefetch < G::KSTEPS) f[st % kPrefetch] = fr.rows(0, sb, st + kPrefetch);
        __builtin_amdgcn_sched_barrier(0);
      }
      i32x4 tf[2];
      tf[0] = fr.tr(0, 2 * sb, 0);
      tf[1] = fr.tr(0, 2 * sb, 1);
      uint32_t W[8];
      if (!grad) {
        // rows / columns that do not exist or lie above the diagonal give P = 0
        bool need_mask = sblk + 32 > len || !rows_full;
        if (causal) need_mask = need_mask || sblk < r0w + 31;
        if (need_mask) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int srow = sblk + 16 * (r >> 3) + 8 * fr.lh + (r & 7);
            const bool ok = srow < len && rrow < len && (!causal || rrow <= srow);
            S[r] = ok ? S[r] : -INFINITY;
          }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
          W[i] = Elem<T>::pack2(fast_exp2(fmaf(S[2 * i], scale, -vec_r[2 * i])),
                                fast_exp2(fmaf(S[2 * i + 1], scale, -vec_r[2 * i + 1])));
        // P for the grad wave of this group (it reads it in the next tile step)
        *(lds_i32x4*)(uintptr_t)(pbv + sb * 2048) = (i32x4){(int)W[0], (int)W[1], (int)W[2], (int)W[3]};
        *(lds_i32x4*)(uintptr_t)(pbv + sb * 2048 + 1024) = (i32x4){(int)W[4], (int)W[5], (int)W[6], (int)W[7]};
      } else {
        const i32x4 p0 = *(lds_i32x4*)(uintptr_t)(pbv + sb * 2048);
        const i32x4 p1 = *(lds_i32x4*)(uintptr_t)(pbv + sb * 2048 + 1024);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const uint32_t pk = (uint32_t)(i < 4 ? p0[i] : p1[i - 4]);
          float plo, phi;
          if (std::is_same<T, __bf16>::value) {
            plo = __builtin_bit_cast(float, pk << 16);
            phi = __builtin_bit_cast(float, pk & 0xffff0000u);
          } else {
            const f16x2 h2 = __builtin_bit_cast(f16x2, pk);
            plo = (float)h2[0];
            phi = (float)h2[1];
          }
          W[i] = Elem<T>::pack2(plo * (S[2 * i] - vec_r[2 * i]), phi * (S[2 * i + 1] - vec_r[2 * i + 1]));
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      // accumulating product: dV^T += dO^T P  /  dK^T += Q^T dS
      __builtin_amdgcn_s_setprio(3);
#pragma unroll
      for (int i = 0; i < NACC; ++i) {
        const int kk = i / G::NDB, db = i % G::NDB;
        const i32x4 wf = {(int)W[4 * kk], (int)W[4 * kk + 1], (int)W[4 * kk + 2], (int)W[4 * kk + 3]};
        acc[db] = Elem<T>::mfma(tf[i & 1], wf, acc[db]);
        if (i + 2 < NACC) tf[i & 1] = fr.tr(0, 2 * sb + (i + 2) / G::NDB, (i + 2) % G::NDB);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // step i: the score waves work on tile i, the grad waves on tile i - 1, and
  // tile i + 1 is on its way into the stage that tile i - 2 has left
  if (n_stream > 0) {
    request();
    drip_all();
    advance();
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
  __syncthreads();
  auto sync_step = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __syncthreads();
  };
  // Tiles of a head that need masks: the first ones of a causal item (keys of
  // this group against queries at or before them) and a last, partial one.
  int n_pre = causal ? (32 * pr + 31 + TN - 1) / TN : 0;
  int n_post = (len % TN) != 0 ? 1 : 0;
  if (!rows_full) n_pre = nj;
  n_pre = min(n_pre, nj);
  n_post = min(n_post, nj - n_pre);
  int req_left = n_stream - 1;  // requests still to make (the first one is out)
  // Each loop below holds ONE kind of step: with the masked path and the
  // pipelined path in one loop body the accumulators were copied between two
  // register sets on every trip.
  auto run = [&](auto role_c) __attribute__((always_inline)) {
    constexpr bool gr = decltype(role_c)::value != 0;
    auto step = [&](auto fast_c) __attribute__((always_inline)) {
      const bool more = req_left > 0;
      if (more) request();
      if (decltype(fast_c)::value)
        compute_fast(role_c);
      else
        compute_slow(role_c);
      rotate();
      if (more) advance();
      --req_left;
      sync_step();
    };
    if (gr) {  // step 0: nothing to work on yet
      if (req_left > 0) {
        request();
        drip_all();
        advance();
      }
      --req_left;
      sync_step();
    }
    for (int g = 0; g < gqa; ++g) {
      for (int jj = 0; jj < n_pre; ++jj) step(ic<0>{});
      for (int jj = n_pre; jj < nj - n_post; ++jj) step(ic<1>{});
      for (int jj = nj - n_post; jj < nj; ++jj) step(ic<0>{});
    }
    if (!gr) sync_step();  // the grad waves' last tile
  };
  if (!grad)
    run(ic<0>{});
  else
    run(ic<1>{});

  // ---- epilogue: dV from the score waves, dK from the grad waves
  const float oscale = grad ? p.scale_nat : 1.f;
  T* outp = grad ? reinterpret_cast<T*>(p.dk) + bsel * p.dk_sb + start * p.dk_ss + hr * p.dk_sh
                 : reinterpret_cast<T*>(p.dv) + bsel * p.dv_sb + start * p.dv_ss + hr * p.dv_sh;
  const int64_t o_ss = grad ? p.dk_ss : p.dv_ss;
  unsigned char* stg = smem_bwd + wave * 32 * OROWB;
#pragma unroll
  for (int db = 0; db < G::NDB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = 32 * db + 8 * g + 4 * fr.lh;
      i32x2 w;
      w[0] = (int)Elem<T>::pack2(acc[db][4 * g] * oscale, acc[db][4 * g + 1] * oscale);
      w[1] = (int)Elem<T>::pack2(acc[db][4 * g + 2] * oscale, acc[db][4 * g + 3] * oscale);
      *reinterpret_cast<i32x2*>(stg + fr.lq * OROWB + d * 2) = w;
    }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < (32 * G::NCH + 63) / 64; ++i) {
    const int idx = lane + 64 * i;
    const int row = idx / G::NCH, ch = idx % G::NCH;
    if (((32 * G::NCH) % 64 == 0 || idx < 32 * G::NCH) && r0w + row < len) {
      const i32x4 val = *reinterpret_cast<const i32x4*>(stg + row * OROWB + ch * 16);
      *reinterpret_cast<i32x4*>(outp + (int64_t)(r0w + row) * o_ss + ch * 8) = val;
    }
  }
}

template <typename T, int D>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2)))
bwd_dkdv_kernel(const BwdParams p, const int n_items, const int n_rt) {
  const int grid = gridDim.x;
  int round = 0;
  for (int base = 0; base < n_items; base += grid, ++round) {
    int w = blockIdx.x;
    if ((round & 1) && (grid & 7) == 0) w = (((grid >> 3) - 1 - (w >> 3)) << 3) | (w & 7);
    const int bid = base + w;
    if (bid < n_items) bwd_dkdv_item<T, D>(p, bid, n_rt);
    if (base + grid < n_items) __syncthreads();
  }
}

// Persistent launch, as in the forward pass: at most one workgroup per CU, each
// walking the work item ids id, id + grid, ... (a fresh 512-thread workgroup
// with this much LDS starts several microseconds after its predecessor ends);
// odd rounds run back to front within an XCD so that a workgroup that drew an
// item that streams many tiles draws one that streams few next.
template <typename T, int D>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2)))
bwd_dq_kernel(const BwdParams p, const int n_items) {
  const int grid = gridDim.x;
  int round = 0;
  for (int base = 0; base < n_items; base += grid, ++round) {
    int w = blockIdx.x;
    if ((round & 1) && (grid & 7) == 0) w = (((grid >> 3) - 1 - (w >> 3)) << 3) | (w & 7);
    const int bid = base + w;
    if (bid < n_items) bwd_dq_item<T, D>(p, bid);
    if (base + grid < n_items) __syncthreads();  // the next item's tiles overwrite the staging area
  }
}

template <typename T, int D>
int launch_dq(const BwdParams& p, hipStream_t s) {
  constexpr size_t lds = kBwdStages * (2 * 64 * 256 + 1024);
  static_assert(lds >= 8 * 32 * (D * 2 + 16), "epilogue staging must fit the tile ring");
  auto kern = bwd_dq_kernel<T, D>;
  static LdsLimitOnce lds_once;
  if (const int e = raise_lds_limit(lds_once, reinterpret_cast<const void*>(kern), (int)lds)) return e;
  const long long items = (long long)p.n_rtiles * p.hq * p.batch;
  long long grid = items;
  const int cus = device_cu_count();
  if (cus > 0 && grid > cus) grid = cus;  // one workgroup per CU is resident (LDS)
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), lds, s, p, (int)items);
  return (int)hipGetLastError();
}

template <typename T, int D>
int launch_dkdv(const BwdParams& p, hipStream_t s) {
  constexpr size_t lds = kBwdStages * (2 * 64 * 256 + 1024) + 2 * 4 * 2 * 2048;  // tile ring + P exchange
  static_assert(lds >= 8 * 32 * (D * 2 + 16), "epilogue staging must fit");
  auto kern = bwd_dkdv_kernel<T, D>;
  static LdsLimitOnce lds_once;
  if (const int e = raise_lds_limit(lds_once, reinterpret_cast<const void*>(kern), (int)lds)) return e;
  const int n_rt = (p.max_seqlen + 127) / 128;
  const long long items = (long long)n_rt * p.hkv * p.batch;
  long long grid = items;
  const int cus = device_cu_count();
  if (cus > 0 && grid > cus) grid = cus;  // one workgroup per CU is resident (LDS)
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), lds, s, p, (int)items, n_rt);
  return (int)hipGetLastError();
}

template <typename T, int D>
int launch_all(const BwdParams& p, hipStream_t s) {
  // dQ first: it also writes Delta, which the dK + dV kernel reads
  int rc;
  if ((rc = launch_dq<T, D>(p, s))) return rc;
  return launch_dkdv<T, D>(p, s);
}

}  // namespace

int launch_attn_bwd(const BwdParams& p, int dtype, int head_dim, hipStream_t s) {
  if (dtype == 0) {
    if (head_dim == 64) return launch_all<__bf16, 64>(p, s);
    if (head_dim == 96) return launch_all<__bf16, 96>(p, s);
    if (head_dim == 128) return launch_all<__bf16, 128>(p, s);
  } else {
    if (head_dim == 64) return launch_all<_Float16, 64>(p, s);
    if (head_dim == 96) return launch_all<_Float16, 96>(p, s);
    if (head_dim == 128) return launch_all<_Float16, 128>(p, s);
  }
  return (int)hipErrorInvalidValue;
}

}  // namespace mi
