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
// reference does, the GQA members of a kv-head are accumulated in registers
// (the reference materialises one dk/dv per member and sums, :687-692,813).
//
// One kernel template, three modes, all on the forward pass's tile engine: a
// wavefront keeps 32 "resident" rows (and their two B operands) in registers
// and streams 64-row tiles of the other side through LDS.
//   DQ: resident q, do rows;  streams K, V.   S^T = K Q^T, dP^T = V dO^T, dQ^T += K^T dS^T
//   DK: resident k, v rows;   streams Q, dO.  S = Q K^T,   dP = dO V^T,   dK^T += Q^T dS
//   DV: resident k rows;      streams Q, dO.  S = Q K^T,                  dV^T += dO^T P
// In every mode the first product puts 16 streamed rows of ONE resident row
// into each lane, and the rounded, pairwise packed result already is the B
// operand of the last product; its A operand is a streamed tile read through
// the transposing LDS load.  Every streamed tile uses one layout that serves
// both the row-fragment read and the transposing read (UniFrags).
#include "kernels.h"
#include "tile_core.h"

namespace mi {
namespace {

template <int V>
using ic = std::integral_constant<int, V>;

// vmcnt(N) expcnt(7) lgkmcnt(15) for s_waitcnt on gfx9-family encodings
constexpr int waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

enum { kDQ = 0, kDK = 1, kDV = 2 };

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

template <typename T, int D, int MODE>
__device__ __forceinline__ void bwd_item(const BwdParams& p, const int bid) {
  using G = RowGeom<D>;
  using F = UniFrags<D>;
  constexpr int NW = 8, BM = 32 * NW, TN = 64, NS = kBwdStages;
  constexpr int TILEB = TN * F::ROWB;             // one streamed tile
  constexpr int STAGEB = 2 * TILEB + 1024;        // tile 0, tile 1, lse[64] and delta[64] (fp32)
  constexpr int RPI = 1024 / F::ROWB;             // tile rows per direct-to-LDS instruction
  constexpr int IPW = TN / RPI / NW;              // such instructions per tile and wave
  constexpr bool ROWVEC = MODE != kDQ;            // lse / delta belong to the streamed rows
  constexpr int IPT = 2 * IPW + (ROWVEC ? 2 : 0); // loads per streamed tile and wave
  constexpr int OROWB = D * 2 + 16;               // epilogue staging row

  const int tid = threadIdx.x;
  int lane = tid & 63;
  // An opaque copy per item: what is derived from the lane id (fragment
  // addresses, load offsets) is then recomputed for every item instead of
  // being held in registers across the whole item loop, where it was spilled.
  asm volatile("" : "+v"(lane));
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int heads_r = MODE == kDQ ? p.hq : p.hkv;
  const int gqa = p.hq / p.hkv;
  // Work item -> (sequence, resident head, resident tile).  Consecutive ids go
  // round-robin to the 8 XCDs (private L2 each): give every XCD whole
  // (sequence, head) units so the streamed tensors of a unit stay in one L2,
  // and walk a unit's tiles from the one that streams most to the one that
  // streams least (causal: the last q tile for DQ, the first key tile for DK/DV).
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
  const int rt = MODE == kDQ ? p.n_rtiles - 1 - slot : slot;
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
  const T* xp;
  const T* yp = nullptr;
  if (MODE == kDQ) {
    xp = reinterpret_cast<const T*>(p.q) + bsel * p.q_sb + (start + rclamp) * p.q_ss + hr * p.q_sh;
    yp = reinterpret_cast<const T*>(p.dout) + bsel * p.do_sb + (start + rclamp) * p.do_ss + hr * p.do_sh;
  } else {
    xp = reinterpret_cast<const T*>(p.k) + bsel * p.k_sb + (start + rclamp) * p.k_ss + hr * p.k_sh;
    if (MODE == kDK) yp = reinterpret_cast<const T*>(p.v) + bsel * p.v_sb + (start + rclamp) * p.v_ss + hr * p.v_sh;
  }
  i32x4 Xf[G::KSTEPS], Yf[G::KSTEPS];
#pragma unroll
  for (int c = 0; c < G::KSTEPS; ++c) {
    Xf[c] = *reinterpret_cast<const i32x4*>(xp + 8 * fr.lh + 16 * c);
    if (MODE != kDV) Yf[c] = *reinterpret_cast<const i32x4*>(yp + 8 * fr.lh + 16 * c);
  }
  float lse_l = 0.f, delta_l = 0.f;
  if (MODE == kDQ) {
    lse_l = p.lse[bsel * p.lse_sb + (start + rclamp) * p.lse_ss + hr * p.lse_sh];
    delta_l = p.delta[(int64_t)b * p.dl_sb + (int64_t)hr * p.dl_sh + rclamp];
  }

  f32x16 acc[G::NDB];
#pragma unroll
  for (int db = 0; db < G::NDB; ++db) acc[db] = (f32x16){0};

  // ---- streamed tiles: which rows, for which heads
  int j0, nj;  // first streamed tile and number of tiles per head
  {
    const int n_all = (len + TN - 1) / TN;
    if (MODE == kDQ) {
      j0 = 0;
      nj = p.causal ? min(n_all, (r0 + BM + TN - 1) / TN) : n_all;
    } else {
      j0 = p.causal ? r0 / TN : 0;
      nj = n_all - j0;
    }
  }
  const int n_heads_s = MODE == kDQ ? 1 : gqa;
  const int n_stream = nj * n_heads_s;

  // ---- direct-to-LDS loads (inline assembly: see the note in prefill.hip)
  const int drow = lane / F::SLOTS, dslot = lane % F::SLOTS;
  auto dma16 = [&](const char* g, uint32_t slab_u) __attribute__((always_inline)) {
    const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(slab_u);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(slab) : "memory");
  };
  auto dma4 = [&](const char* g, uint32_t slab_u) __attribute__((always_inline)) {
    const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(slab_u);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" : : "v"(g), "s"(slab) : "memory");
  };
  // tile 0 feeds the first product (row fragments), tile 1 the second one
  // (row fragments; in DV mode the transposing read)
  auto issue = [&](int u, auto stage_c) __attribute__((always_inline)) {
    constexpr int ST = decltype(stage_c)::value;
    const int g = u / nj, j = j0 + u % nj;
    const int s0 = j * TN;
    const char *t0, *t1;
    int64_t pitch0, pitch1;
    int hs;
    if (MODE == kDQ) {
      hs = hr / gqa;
      t0 = reinterpret_cast<const char*>(reinterpret_cast<const T*>(p.k) + bsel * p.k_sb + start * p.k_ss + hs * p.k_sh);
      t1 = reinterpret_cast<const char*>(reinterpret_cast<const T*>(p.v) + bsel * p.v_sb + start * p.v_ss + hs * p.v_sh);
      pitch0 = p.k_ss * 2;
      pitch1 = p.v_ss * 2;
    } else {
      hs = hr * gqa + g;
      t0 = reinterpret_cast<const char*>(reinterpret_cast<const T*>(p.q) + bsel * p.q_sb + start * p.q_ss + hs * p.q_sh);
      t1 = reinterpret_cast<const char*>(reinterpret_cast<const T*>(p.dout) + bsel * p.do_sb + start * p.do_ss + hs * p.do_sh);
      pitch0 = p.q_ss * 2;
      pitch1 = p.do_ss * 2;
    }
    const uint32_t base = lds0 + ST * STAGEB;
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
    if (ROWVEC) {
      const int64_t rr = min(s0 + lane, len - 1);
      const float* lp = p.lse + bsel * p.lse_sb + (start + rr) * p.lse_ss + hs * p.lse_sh;
      const float* dp = p.delta + (int64_t)b * p.dl_sb + (int64_t)hs * p.dl_sh + rr;
      dma4(reinterpret_cast<const char*>(lp), base + 2 * TILEB);
      dma4(reinterpret_cast<const char*>(dp), base + 2 * TILEB + 256);
    }
  };

  const float scale = p.scale;
  const int causal = p.causal;

  auto compute = [&](int u, auto stage_c) __attribute__((always_inline)) {
    constexpr int ST = decltype(stage_c)::value;
    constexpr uint32_t T0 = ST * STAGEB, T1 = ST * STAGEB + TILEB, LV = ST * STAGEB + 2 * TILEB;
    const int s0 = (j0 + u % nj) * TN;
    constexpr int kPrefetch = 4;
    i32x4 f[kPrefetch];   // row fragments of the first product, read ahead
    bool f_ready = false; // block 0 has already fetched the first fragments of block 1
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      const int sblk = s0 + 32 * sb;
      if (sblk >= len) continue;
      if (causal) {
        // DQ: keys past this wave's last query; DK/DV: queries before this wave's first key
        if (MODE == kDQ ? (sblk > r0w + 31) : (sblk + 31 < r0w)) continue;
      }
      // register r of this lane is streamed row  sblk + 16*(r/8) + 8*lh + r%8
      float lse_r[16], dl_r[16];
      if (ROWVEC) {
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        typedef __attribute__((address_space(3))) const f32x4 lds_f4;
#pragma unroll
        for (int g2 = 0; g2 < 2; ++g2)
#pragma unroll
          for (int q4 = 0; q4 < 2; ++q4) {
            const uint32_t a = lds0 + LV + (32 * sb + 16 * g2 + 8 * fr.lh + 4 * q4) * 4;
            const f32x4 lv = *(lds_f4*)(uintptr_t)a;
            lse_r[8 * g2 + 4 * q4 + 0] = lv[0]; lse_r[8 * g2 + 4 * q4 + 1] = lv[1];
            lse_r[8 * g2 + 4 * q4 + 2] = lv[2]; lse_r[8 * g2 + 4 * q4 + 3] = lv[3];
            if (MODE == kDK) {
              const f32x4 dv = *(lds_f4*)(uintptr_t)(a + 256);
              dl_r[8 * g2 + 4 * q4 + 0] = dv[0]; dl_r[8 * g2 + 4 * q4 + 1] = dv[1];
              dl_r[8 * g2 + 4 * q4 + 2] = dv[2]; dl_r[8 * g2 + 4 * q4 + 3] = dv[3];
            }
          }
      }
      // The block as one pinned instruction stream (sched_barrier(0) after every
      // slice): the S chain; the dP chain with the exponentials of S behind its
      // MFMAs; the first half of dS; the last product with the second half of
      // dS behind its first MFMAs.  Row fragments are read four steps ahead,
      // transposed fragments two.
      constexpr bool TWO = MODE != kDV;
      constexpr int NSTEP = (TWO ? 2 : 1) * G::KSTEPS;
      constexpr uint32_t TT = MODE == kDV ? T1 : T0;  // tile whose transpose is the A operand
      f32x16 S = (f32x16){0}, dP = (f32x16){0};
      auto frag = [&](int st) __attribute__((always_inline)) -> i32x4 {
        return st < G::KSTEPS ? fr.rows(T0, sb, st) : fr.rows(T1, sb, st - G::KSTEPS);
      };
      auto prob = [&](int r) __attribute__((always_inline)) {   // S[r] <- P[r]
        S[r] = fast_exp2(fmaf(S[r], scale, -(ROWVEC ? lse_r[r] : lse_l)));
      };
      auto dsv = [&](int r) __attribute__((always_inline)) -> float {
        return MODE == kDV ? S[r] : S[r] * (dP[r] - (ROWVEC ? dl_r[r] : delta_l));
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
      if (MODE != kDQ) need_mask = need_mask || r0w + 32 > len;
      if (causal) need_mask = need_mask || (MODE == kDQ ? (sblk + 31 > r0w) : (sblk < r0w + 31));
      if (need_mask) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int srow = sblk + 16 * (r >> 3) + 8 * fr.lh + (r & 7);
          bool ok;
          if (MODE == kDQ)
            ok = srow < len && (!causal || srow <= rrow);
          else
            ok = srow < len && rrow < len && (!causal || rrow <= srow);
          S[r] = ok ? S[r] : -INFINITY;
        }
      }
      i32x4 tf[2];
      uint32_t W[8];
      if (TWO) {
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
      } else {
        tf[0] = fr.tr(TT, 2 * sb, 0);
        tf[1] = fr.tr(TT, 2 * sb, 1);
#pragma unroll
        for (int r = 0; r < 8; ++r) prob(r);
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
          for (int q = 4 * i / G::NDB; q < 4 * (i + 1) / G::NDB; ++q) {
            if (!TWO) {
              prob(8 + 2 * q);
              prob(9 + 2 * q);
            }
            W[4 + q] = Elem<T>::pack2(dsv(8 + 2 * q), dsv(9 + 2 * q));
          }
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
  const float oscale = MODE == kDV ? 1.f : p.scale_nat;
  T* outp;
  int64_t o_ss;
  if (MODE == kDQ) {
    outp = reinterpret_cast<T*>(p.dq) + bsel * p.dq_sb + start * p.dq_ss + hr * p.dq_sh;
    o_ss = p.dq_ss;
  } else if (MODE == kDK) {
    outp = reinterpret_cast<T*>(p.dk) + bsel * p.dk_sb + start * p.dk_ss + hr * p.dk_sh;
    o_ss = p.dk_ss;
  } else {
    outp = reinterpret_cast<T*>(p.dv) + bsel * p.dv_sb + start * p.dv_ss + hr * p.dv_sh;
    o_ss = p.dv_ss;
  }
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

// Persistent launch, as in the forward pass: at most one workgroup per CU, each
// walking the work item ids id, id + grid, ... (a fresh 512-thread workgroup
// with this much LDS starts several microseconds after its predecessor ends);
// odd rounds run back to front within an XCD so that a workgroup that drew an
// item that streams many tiles draws one that streams few next.
template <typename T, int D, int MODE>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2)))
bwd_kernel(const BwdParams p, const int n_items) {
  const int grid = gridDim.x;
  int round = 0;
  for (int base = 0; base < n_items; base += grid, ++round) {
    int w = blockIdx.x;
    if ((round & 1) && (grid & 7) == 0) w = (((grid >> 3) - 1 - (w >> 3)) << 3) | (w & 7);
    const int bid = base + w;
    if (bid < n_items) bwd_item<T, D, MODE>(p, bid);
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

template <typename T, int D, int MODE>
int launch_mode(const BwdParams& p, hipStream_t s) {
  constexpr size_t lds = kBwdStages * (2 * 64 * 256 + 1024);
  static_assert(lds >= 8 * 32 * (D * 2 + 16), "epilogue staging must fit the tile ring");
  auto kern = bwd_kernel<T, D, MODE>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
  const long long items = (long long)p.n_rtiles * (MODE == kDQ ? p.hq : p.hkv) * p.batch;
  long long grid = items;
  const int cus = device_cu_count();
  if (cus > 0 && grid > cus) grid = cus;  // one workgroup per CU is resident (LDS)
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), lds, s, p, (int)items);
  return (int)hipGetLastError();
}

template <typename T, int D>
int launch_all(const BwdParams& p, hipStream_t s) {
  dim3 grid((p.max_seqlen + 15) / 16, p.hq, p.batch);
  hipLaunchKernelGGL((bwd_delta_kernel<T>), grid, dim3(256), 0, s, p, D);
  int rc = (int)hipGetLastError();
  if (rc) return rc;
  if ((rc = launch_mode<T, D, kDQ>(p, s))) return rc;
  if ((rc = launch_mode<T, D, kDK>(p, s))) return rc;
  return launch_mode<T, D, kDV>(p, s);
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
