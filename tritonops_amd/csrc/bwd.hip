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
    len = p.cu[b + 1] - (int)start;
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
  i32x4 Xf[G::KSTEPS], Yf[G::KSTEPS];
#pragma unroll
  for (int c = 0; c < G::KSTEPS; ++c) {
    Xf[c] = *reinterpret_cast<const i32x4*>(xp + 8 * fr.lh + 16 * c);
    Yf[c] = *reinterpret_cast<const i32x4*>(yp + 8 * fr.lh + 16 * c);
  }
  const float lse_l = p.lse[bsel * p.lse_sb + (start + rclamp) * p.lse_ss + hr * p.lse_sh];
  const float delta_l = p.delta[(int64_t)b * p.dl_sb + (int64_t)hr * p.dl_sh + rclamp];

  f32x16 acc[G::NDB];
#pragma unroll
  for (int db = 0; db < G::NDB; ++db) acc[db] = (f32x16){0};

  // ---- streamed tiles: which rows, for which heads
  const int n_all = (len + TN - 1) / TN;
  const int n_stream = p.causal ? min(n_all, (r0 + BM + TN - 1) / TN) : n_all;  // key tiles 0 .. n_stream - 1

  // ---- direct-to-LDS loads (inline assembly: see the note in prefill.hip)
  const int drow = lane / F::SLOTS, dslot = lane % F::SLOTS;
  auto dma16 = [&](const char* g, uint32_t slab_u) __attribute__((always_inline)) {
    const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(slab_u);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(slab) : "memory");
  };
  // the same with the address as "uniform 64-bit base + 32-bit lane offset":
  // no vector arithmetic per load
  auto dma16s = [&](uint64_t base, uint32_t off, uint32_t slab_u) __attribute__((always_inline)) {
    const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(slab_u);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(off), "s"(base), "s"(slab) : "memory");
  };
  auto uniform64 = [](uint64_t x) __attribute__((always_inline)) -> uint64_t {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)x);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
    return ((uint64_t)hi << 32) | lo;
  };
  // Streamed tensors: K feeds the first product and, transposed, the last; V
  // the second.  Their row pitches and this lane's offsets inside a tile are
  // fixed for the item.
  const int64_t pitch0 = p.k_ss * 2, pitch1 = p.v_ss * 2;
  const int hs = hr / gqa;
  const char* h0 = reinterpret_cast<const char*>(reinterpret_cast<const T*>(p.k) + bsel * p.k_sb + start * p.k_ss + hs * p.k_sh);
  const char* h1 = reinterpret_cast<const char*>(reinterpret_cast<const T*>(p.v) + bsel * p.v_sb + start * p.v_ss + hs * p.v_sh);
  uint32_t off0[IPW], off1[IPW];
#pragma unroll
  for (int t = 0; t < IPW; ++t) {
    const int r = RPI * (wave + NW * t) + drow;
    const int c = dslot ^ F::swz(r);
    off0[t] = (uint32_t)r * (uint32_t)pitch0 + c * 16;
    off1[t] = (uint32_t)r * (uint32_t)pitch1 + c * 16;
  }
  // key tile u into stage ST
  auto issue = [&](int u, auto stage_c) __attribute__((always_inline)) {
    constexpr int ST = decltype(stage_c)::value;
    const int s0 = u * TN;
    const uint32_t base = lds0 + ST * STAGEB;
    if (s0 + TN <= len) {
      const uint64_t a0 = uniform64((uint64_t)(uintptr_t)(h0 + s0 * pitch0));
      const uint64_t a1 = uniform64((uint64_t)(uintptr_t)(h1 + s0 * pitch1));
#pragma unroll
      for (int t = 0; t < IPW; ++t) {
        const int inst = wave + NW * t;
        const int c = dslot ^ F::swz(RPI * inst + drow);
        if (G::NCH == 16 || c < G::NCH) {
          dma16s(a0, off0[t], base + inst * 1024);
          dma16s(a1, off1[t], base + TILEB + inst * 1024);
        }
      }
    } else {
#pragma unroll
      for (int t = 0; t < IPW; ++t) {
        const int inst = wave + NW * t;
        const int r = RPI * inst + drow;
        const int c = dslot ^ F::swz(r);
        const int64_t rr = min(s0 + r, len - 1);  // rows past the end re-read the last row (masked later)
        if (G::NCH == 16 || c < G::NCH) {
          dma16(h0 + rr * pitch0 + c * 16, base + inst * 1024);
          dma16(h1 + rr * pitch1 + c * 16, base + TILEB + inst * 1024);
        }
      }
    }
  };

  const float scale = p.scale;
  const int causal = p.causal;

  auto compute = [&](int u, auto stage_c) __attribute__((always_inline)) {
    constexpr int ST = decltype(stage_c)::value;
    constexpr uint32_t T0 = ST * STAGEB, T1 = ST * STAGEB + TILEB;
    const int s0 = u * TN;
    constexpr int kPrefetch = 4;
    i32x4 f[kPrefetch];   // row fragments of the first product, read ahead
    bool f_ready = false; // block 0 has already fetched the first fragments of block 1
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      const int sblk = s0 + 32 * sb;
      if (sblk >= len) continue;
      if (causal && sblk > r0w + 31) continue;  // keys past this wave's last query
      // register r of this lane is streamed row  sblk + 16*(r/8) + 8*lh + r%8
      // The block as one pinned instruction stream (sched_barrier(0) after every
      // slice): the S chain; the dP chain with the exponentials of S behind its
      // MFMAs; the first half of dS; the last product with the second half of
      // dS behind its first MFMAs.  Row fragments are read four steps ahead,
      // transposed fragments two.
      constexpr int NSTEP = 2 * G::KSTEPS;
      constexpr uint32_t TT = T0;  // tile whose transpose is the A operand of the last product
      f32x16 S = (f32x16){0}, dP = (f32x16){0};
      auto frag = [&](int st) __attribute__((always_inline)) -> i32x4 {
        return st < G::KSTEPS ? fr.rows(T0, sb, st) : fr.rows(T1, sb, st - G::KSTEPS);
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
#pragma unroll
      for (int st = 0; st < G::KSTEPS; ++st) {
        S = Elem<T>::mfma(f[st % kPrefetch], Xf[st], S);
        if (st + kPrefetch < NSTEP) f[st % kPrefetch] = frag(st + kPrefetch);
        __builtin_amdgcn_sched_barrier(0);
      }
      // rare: rows / columns that do not exist or lie above the diagonal give P = 0
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
      i32x4 tf[2];
      uint32_t W[8];
#pragma unroll
      for (int c = 0; c < G::KSTEPS; ++c) {
        const int st = G::KSTEPS + c;
        dP = Elem<T>::mfma(f[st % kPrefetch], Yf[c], dP);
        if (st + kPrefetch < NSTEP) f[st % kPrefetch] = frag(st + kPrefetch);
        if (c >= G::KSTEPS - 2) tf[c - (G::KSTEPS - 2)] = fr.tr(TT, 2 * sb, c - (G::KSTEPS - 2));
        // 16 exponentials spread over the KSTEPS slices
#pragma unroll
        for (int r = 16 * c / G::KSTEPS; r < 16 * (c + 1) / G::KSTEPS; ++r) prob(r);
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
        if (i + 2 < NACC) tf[i & 1] = fr.tr(TT, 2 * sb + (i + 2) / G::NDB, (i + 2) % G::NDB);
        // the ring is idle now: fetch the first fragments of the tile's second block
        if (sb == 0 && i >= NACC - kPrefetch) f[i - (NACC - kPrefetch)] = fr.rows(T0, 1, i - (NACC - kPrefetch));
        if (i < G::NDB) {
          // second half of dS (8 values) spread over the first NDB slices
#pragma unroll
          for (int q = 4 * i / G::NDB; q < 4 * (i + 1) / G::NDB; ++q)
            W[4 + q] = Elem<T>::pack2(dsv(8 + 2 * q), dsv(9 + 2 * q));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      f_ready = sb == 0;
    }
  };

  auto step = [&](auto stage_c, int u) __attribute__((always_inline)) {
    constexpr int ST = decltype(stage_c)::value;
    const bool refill = u + NS - 1 < n_stream;
    if (refill) issue(u + NS - 1, ic<(ST + NS - 1) % NS>{});
    compute(u, stage_c);
    // the next tile must have landed (this wave's loads retire in order: only
    // the tiles requested after it may still fly) and everyone is done with this one
    const int younger = min(n_stream - 1, u + NS - 1) - (u + 1);
    if (younger >= 2)
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(2 * IPT));
    else if (younger == 1)
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(IPT));
    else
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __syncthreads();
  };

  if (n_stream > 0) issue(0, ic<0>{});
  if (n_stream > 1) issue(1, ic<1>{});
  if (NS > 3 && n_stream > 2) issue(2, ic<2 % NS>{});
  // resident operands and tile 0 are needed now; the full wait also tells the
  // compiler that no register load is pending inside the loop
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
  __syncthreads();
  for (int u = 0; u < n_stream; u += NS) {
    step(ic<0>{}, u);
    if (u + 1 >= n_stream) break;
    step(ic<1>{}, u + 1);
    if (u + 2 >= n_stream) break;
    step(ic<2>{}, u + 2);
    if (NS > 3) {
      if (u + 3 >= n_stream) break;
      step(ic<3 % NS>{}, u + 3);
    }
  }
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
  constexpr int NW = 8, NP = 4, BM = 32 * NP, TN = 64, NS = kBwdStages;
  static_assert(NS == 3, "stage reuse below assumes three stages");
  constexpr int TILEB = TN * F::ROWB;
  constexpr int STAGEB = 2 * TILEB + 1024;
  constexpr int RPI = 1024 / F::ROWB;
  constexpr int IPW = TN / RPI / NW;
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
    len = p.cu[b + 1] - (int)start;
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
  auto dma16 = [&](const char* g, uint32_t slab_u) __attribute__((always_inline)) {
    const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(slab_u);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(slab) : "memory");
  };
  auto dma4 = [&](const char* g, uint32_t slab_u) __attribute__((always_inline)) {
    const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(slab_u);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" : : "v"(g), "s"(slab) : "memory");
  };
  auto dma16s = [&](uint64_t base, uint32_t off, uint32_t slab_u) __attribute__((always_inline)) {
    const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(slab_u);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(off), "s"(base), "s"(slab) : "memory");
  };
  auto dma4s = [&](uint64_t base, uint32_t off, uint32_t slab_u) __attribute__((always_inline)) {
    const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(slab_u);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" : : "v"(off), "s"(base), "s"(slab) : "memory");
  };
  auto uniform64 = [](uint64_t x) __attribute__((always_inline)) -> uint64_t {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)x);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
    return ((uint64_t)hi << 32) | lo;
  };
  // streamed tensors of the first query head of the group, first row of the sequence
  const int64_t pitch0 = p.q_ss * 2, pitch1 = p.do_ss * 2;
  const char* h0 = reinterpret_cast<const char*>(reinterpret_cast<const T*>(p.q) + bsel * p.q_sb + start * p.q_ss + hr * gqa * p.q_sh);
  const char* h1 = reinterpret_cast<const char*>(reinterpret_cast<const T*>(p.dout) + bsel * p.do_sb + start * p.do_ss + hr * gqa * p.do_sh);
  const char* lv0 = reinterpret_cast<const char*>(p.lse + bsel * p.lse_sb + start * p.lse_ss + hr * gqa * p.lse_sh);
  const char* dv0 = reinterpret_cast<const char*>(p.delta + (int64_t)b * p.dl_sb + (int64_t)hr * gqa * p.dl_sh);
  uint32_t off0[IPW], off1[IPW];
#pragma unroll
  for (int t = 0; t < IPW; ++t) {
    const int r = RPI * (wave + NW * t) + drow;
    const int c = dslot ^ F::swz(r);
    off0[t] = (uint32_t)r * (uint32_t)pitch0 + c * 16;
    off1[t] = (uint32_t)r * (uint32_t)pitch1 + c * 16;
  }
  const uint32_t lv_off = (uint32_t)lane * (uint32_t)(p.lse_ss * 4);
  // streamed tiles are requested in order: (head, tile, stage) of the next
  // request; Q rows, dO rows, lse and Delta of the rows
  int iss_g = 0, iss_j = j0, iss_st = 0;
  auto issue = [&]() __attribute__((always_inline)) {
    const int s0 = iss_j * TN;
    const uint32_t base = lds0 + (uint32_t)iss_st * STAGEB;
    const char* t0 = h0 + iss_g * (p.q_sh * 2);
    const char* t1 = h1 + iss_g * (p.do_sh * 2);
    const char* lp = lv0 + iss_g * (p.lse_sh * 4);
    const char* dp = dv0 + (int64_t)iss_g * p.dl_sh * 4;
    if (s0 + TN <= len) {
      const uint64_t a0 = uniform64((uint64_t)(uintptr_t)(t0 + s0 * pitch0));
      const uint64_t a1 = uniform64((uint64_t)(uintptr_t)(t1 + s0 * pitch1));
#pragma unroll
      for (int t = 0; t < IPW; ++t) {
        const int inst = wave + NW * t;
        const int c = dslot ^ F::swz(RPI * inst + drow);
        if (G::NCH == 16 || c < G::NCH) {
          dma16s(a0, off0[t], base + inst * 1024);
          dma16s(a1, off1[t], base + TILEB + inst * 1024);
        }
      }
      if (wave == 0) dma4s(uniform64((uint64_t)(uintptr_t)(lp + s0 * (p.lse_ss * 4))), lv_off, base + 2 * TILEB);
      if (wave == 1) dma4s(uniform64((uint64_t)(uintptr_t)(dp + s0 * 4)), (uint32_t)lane * 4u, base + 2 * TILEB + 256);
    } else {
#pragma unroll
      for (int t = 0; t < IPW; ++t) {
        const int inst = wave + NW * t;
        const int r = RPI * inst + drow;
        const int c = dslot ^ F::swz(r);
        const int64_t rr = min(s0 + r, len - 1);  // rows past the end re-read the last row (masked later)
        if (G::NCH == 16 || c < G::NCH) {
          dma16(t0 + rr * pitch0 + c * 16, base + inst * 1024);
          dma16(t1 + rr * pitch1 + c * 16, base + TILEB + inst * 1024);
        }
      }
      const int64_t rr = min(s0 + lane, len - 1);
      if (wave == 0) dma4(lp + rr * (p.lse_ss * 4), base + 2 * TILEB);
      if (wave == 1) dma4(dp + rr * 4, base + 2 * TILEB + 256);
    }
    if (++iss_j == j0 + nj) {
      iss_j = j0;
      ++iss_g;
    }
    iss_st = iss_st == NS - 1 ? 0 : iss_st + 1;
  };

  const float scale = p.scale;
  const int causal = p.causal;
  typedef __attribute__((address_space(3))) i32x4 lds_i32x4;
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) const f32x4 lds_f4;

  // One streamed tile for this wave's role.  Both roles walk the same blocks.
  int cmp_j = j0, cmp_slot = 0;  // tile and P slot of this wave's next compute() call
  // (role and stage are compile-time: every LDS address below is a lane register plus an immediate)
  auto compute = [&](auto role_c, auto stage_c) __attribute__((always_inline)) {
    constexpr bool grad = decltype(role_c)::value != 0;
    constexpr uint32_t stage = decltype(stage_c)::value * STAGEB;
    constexpr uint32_t T0 = stage, T1 = stage + TILEB, LV = stage + 2 * TILEB;
    const uint32_t pb = lds0 + PBUF + (uint32_t)cmp_slot * PSLOT + (uint32_t)pr * 4096 + (uint32_t)lane * 16;
    const int s0 = cmp_j * TN;
    if (++cmp_j == j0 + nj) cmp_j = j0;
    cmp_slot ^= 1;
    constexpr int kPrefetch = 4;
    constexpr int NACC = 2 * G::NDB;
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
          const uint32_t a = lds0 + LV + (grad ? 256u : 0u) + (32 * sb + 16 * g2 + 8 * fr.lh + 4 * q4) * 4;
          const f32x4 lv = *(lds_f4*)(uintptr_t)a;
#pragma unroll
          for (int e = 0; e < 4; ++e) vec_r[8 * g2 + 4 * q4 + e] = lv[e];
        }
      // first product: rows of Q (score) / dO (grad) against the resident operand
      constexpr uint32_t TR = grad ? T1 : T0;   // tile read as row fragments
      constexpr uint32_t TT = grad ? T0 : T1;   // tile read transposed for the accumulating product
      f32x16 S = (f32x16){0};
      i32x4 f[kPrefetch];
#pragma unroll
      for (int st = 0; st < kPrefetch; ++st) f[st] = fr.rows(TR, sb, st);
      // Issue priority: low during the serial chain and the arithmetic behind
      // it, high while the wave feeds its accumulators (NDB independent chains),
      // so that the two waves of a SIMD fall out of step.
      __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int st = 0; st < G::KSTEPS; ++st) {
        S = Elem<T>::mfma(f[st % kPrefetch], Xf[st], S);
        if (st + kPrefetch < G::KSTEPS) f[st % kPrefetch] = fr.rows(TR, sb, st + kPrefetch);
        __builtin_amdgcn_sched_barrier(0);
      }
      i32x4 tf[2];
      tf[0] = fr.tr(TT, 2 * sb, 0);
      tf[1] = fr.tr(TT, 2 * sb, 1);
      uint32_t W[8];
      if (!grad) {
        // rare: rows / columns that do not exist or lie above the diagonal give P = 0
        bool need_mask = sblk + 32 > len || r0w + 32 > len;
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
        *(lds_i32x4*)(uintptr_t)(pb + sb * 2048) = (i32x4){(int)W[0], (int)W[1], (int)W[2], (int)W[3]};
        *(lds_i32x4*)(uintptr_t)(pb + sb * 2048 + 1024) = (i32x4){(int)W[4], (int)W[5], (int)W[6], (int)W[7]};
      } else {
        const i32x4 p0 = *(lds_i32x4*)(uintptr_t)(pb + sb * 2048);
        const i32x4 p1 = *(lds_i32x4*)(uintptr_t)(pb + sb * 2048 + 1024);
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
        if (i + 2 < NACC) tf[i & 1] = fr.tr(TT, 2 * sb + (i + 2) / G::NDB, (i + 2) % G::NDB);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // step i: the score waves work on tile i, the grad waves on tile i - 1, and
  // tile i + 1 is on its way into the stage that tile i - 2 has left
  if (n_stream > 0) issue();
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
  __syncthreads();
  auto step = [&](auto role_c, auto stage_c, int i) __attribute__((always_inline)) {
    if (i + 1 < n_stream) issue();
    if (decltype(role_c)::value ? i >= 1 : i < n_stream) compute(role_c, stage_c);
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __syncthreads();
  };
  if (!grad) {
    for (int i = 0; i <= n_stream; i += NS) {
      step(ic<0>{}, ic<0>{}, i);
      if (i + 1 > n_stream) break;
      step(ic<0>{}, ic<1>{}, i + 1);
      if (i + 2 > n_stream) break;
      step(ic<0>{}, ic<2>{}, i + 2);
    }
  } else {
    step(ic<1>{}, ic<0>{}, 0);  // nothing to work on yet
    for (int i = 1; i <= n_stream; i += NS) {
      step(ic<1>{}, ic<0>{}, i);
      if (i + 1 > n_stream) break;
      step(ic<1>{}, ic<1>{}, i + 1);
      if (i + 2 > n_stream) break;
      step(ic<1>{}, ic<2>{}, i + 2);
    }
  }

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

// Delta[b][h][s] = sum_d o[s][d] * do[s][d], fp32.  16 lanes per row (one 16-byte
// chunk each), 16 rows per 256-thread workgroup.
template <typename T>
__global__ void __launch_bounds__(256) bwd_delta_kernel(const BwdParams p, int head_dim) {
  const int ch = threadIdx.x & 15;
  const int row = blockIdx.x * 16 + (threadIdx.x >> 4);
  const int h = blockIdx.y, b = blockIdx.z;
  int len;
  int64_t start;
  if (p.cu) {
    start = p.cu[b];
    len = p.cu[b + 1] - (int)start;
  } else {
    start = 0;
    len = p.max_seqlen;
  }
  const int64_t bsel = p.cu ? 0 : b;
  float s = 0.f;
  if (row < len && ch * 8 < head_dim) {
    const T* op = reinterpret_cast<const T*>(p.o) + bsel * p.o_sb + (start + row) * p.o_ss + h * p.o_sh + ch * 8;
    const T* dp = reinterpret_cast<const T*>(p.dout) + bsel * p.do_sb + (start + row) * p.do_ss + h * p.do_sh + ch * 8;
    const i32x4 ov = *reinterpret_cast<const i32x4*>(op);
    const i32x4 dv = *reinterpret_cast<const i32x4*>(dp);
    const T* oe = reinterpret_cast<const T*>(&ov);
    const T* de = reinterpret_cast<const T*>(&dv);
#pragma unroll
    for (int i = 0; i < 8; ++i) s += (float)oe[i] * (float)de[i];
  }
#pragma unroll
  for (int m = 8; m >= 1; m >>= 1) s += __shfl_xor(s, m, 16);
  if (ch == 0 && row < len) p.delta[(int64_t)b * p.dl_sb + (int64_t)h * p.dl_sh + row] = s;
}

template <typename T, int D>
int launch_dq(const BwdParams& p, hipStream_t s) {
  constexpr size_t lds = kBwdStages * (2 * 64 * 256 + 1024);
  static_assert(lds >= 8 * 32 * (D * 2 + 16), "epilogue staging must fit the tile ring");
  auto kern = bwd_dq_kernel<T, D>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
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
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
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
  dim3 grid((p.max_seqlen + 15) / 16, p.hq, p.batch);
  hipLaunchKernelGGL((bwd_delta_kernel<T>), grid, dim3(256), 0, s, p, D);
  int rc = (int)hipGetLastError();
  if (rc) return rc;
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
