// Device-side building blocks shared by the prefill and the decoding kernels
// (gfx950 / CDNA4 only, wave64).
//
// Formulation.  One wavefront owns 32 query rows.  Per KV tile it computes the
// TRANSPOSED score block  S^T = K . Q^T  with v_mfma_f32_32x32x16 (A = K rows
// from LDS, B = Q^T kept in registers for the whole kernel), so that after the
// MFMA every lane holds scores of ONE query (column = lane % 32) against 16 of
// the 32 keys of the block.  Consequences:
//   * row max / row sum of the online softmax are in-lane reductions plus one
//     exchange between lane l and lane l^32 (v_permlane32_swap);
//   * the rescale factor of the output accumulator is a per-lane scalar;
//   * the probabilities, converted to 16-bit and packed pairwise, already ARE
//     the B operand (P^T) of the second product  O^T = V^T . P^T, no LDS trip.
// The K rows are fetched in a permuted order (key_perm) chosen so that the 8
// accumulator registers feeding one PV MFMA are 8 CONSECUTIVE keys; V^T then
// comes out of a row-major V tile with two ds_read_b64_tr_b16 per operand.
//
// Two LDS tile layouts (both row-major [key][head_dim], both free of bank
// conflicts for the two access patterns: a K fragment read takes one 16 B
// chunk from 16 consecutive rows per quarter wave, a V transposing read takes
// 64 B from each of 4 consecutive rows per half wave):
//   PaddedFrags   - rows padded (K +16 B, V +64 B); every fragment address is a
//                   lane base + immediate.  Filled with ds_write from registers
//                   (decoding kernel).
//   SwizzledFrags - unpadded rows, 16-byte chunks XOR-swizzled per row, so that
//                   a global_load_lds_dwordx4 (64 lanes x 16 B, contiguous in
//                   LDS) can fill 1 KiB of a tile directly; the XOR is applied
//                   on the global-address side.  Fragment addresses are
//                   precomputed per lane (prefill kernel).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

constexpr int kTileN = 64;  // keys per prefill KV tile (two 32-key MFMA blocks)

template <typename T>
struct Elem;

template <>
struct Elem<__bf16> {
  static __device__ __forceinline__ f32x16 mfma(i32x4 a, i32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    bf16x2 r = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(uint32_t, r);
  }
};

template <>
struct Elem<_Float16> {
  static __device__ __forceinline__ f32x16 mfma(i32x4 a, i32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    f16x2 r = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, r);
  }
};

// Compile-time geometry of a tile row for head_dim D.
template <int D>
struct RowGeom {
  static_assert(D == 64 || D == 96 || D == 128, "head_dim");
  static constexpr int DP = (D == 64) ? 64 : 128;  // row padded to a power of two, elements
  static constexpr int NCH = D / 8;                // real 16-byte chunks per row
  static constexpr int KSTEPS = D / 16;            // QK^T MFMA steps (k = 16)
  static constexpr int NDB = D / 32;               // 32-row blocks of O^T
};

// Accumulator row rho of the 32x32 MFMA (rho = 8*(reg/4) + 4*(lane/32) + reg%4)
// is fed from key key_perm(rho), which makes register r of lane-half h hold
// key  16*(r/8) + 8*h + r%8  of the 32-key block.
__device__ __forceinline__ int key_perm(int rho) {
  const int g = rho >> 3, hh = (rho >> 2) & 1, t = rho & 3;
  return 16 * (g >> 1) + 8 * hh + 4 * (g & 1) + t;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// max / sum of x over lanes l and l^32.
__device__ __forceinline__ float max_with_other_half(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
}
__device__ __forceinline__ float sum_with_other_half(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
}

__device__ __forceinline__ i32x4 read_tr_pair(const unsigned char* a0, const unsigned char* a1) {
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)a0);
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)a1);
  i32x2 l2 = __builtin_bit_cast(i32x2, lo);
  i32x2 h2 = __builtin_bit_cast(i32x2, hi);
  i32x4 out = {l2[0], l2[1], h2[0], h2[1]};
  return out;
}

// ---------------------------------------------------------------------------
// Layout policy 1: padded rows.
template <int D>
struct PaddedFrags {
  using G = RowGeom<D>;
  static constexpr int KROWB = G::DP * 2 + 16;
  static constexpr int VROWB = G::DP * 2 + 64;
  int lq;     // query column of this lane (lane % 32)
  int lh;     // lane half (lane / 32)
  int k_off;  // byte offset of this lane's K fragment inside a 32-key block, chunk 0
  int v_off;  // byte offset of this lane's V^T fragment for kk = 0, db = 0, first read

  __device__ __forceinline__ void init(int lane) {
    lq = lane & 31;
    lh = lane >> 5;
    k_off = key_perm(lq) * KROWB + lh * 16;
    // transposing read: lane j of a 16-lane group addresses row j/4, 8 bytes at
    // element 4*(j%4) of the group's 16 columns; groups 0/1 (2/3) are the two
    // column halves of lane half 0 (1), which starts 8 rows further down.
    v_off = (8 * lh + ((lane & 15) >> 2)) * VROWB + (2 * ((lane >> 4) & 1) + ((lane & 3) >> 1)) * 16 +
            (lane & 1) * 8;
  }
  // A operand of S^T: K[32*kb + key_perm(lane%32)][16c + 8*(lane/32) .. +7]
  __device__ __forceinline__ i32x4 load_k(const unsigned char* sK, int kb, int c) const {
    return *reinterpret_cast<const i32x4*>(sK + k_off + kb * 32 * KROWB + 32 * c);
  }
  // A operand of O^T: V[16*kk + 8*(lane/32) + 0..7][32*db + lane%32]
  __device__ __forceinline__ i32x4 load_v(const unsigned char* sV, int kk, int db) const {
    const unsigned char* a0 = sV + v_off + (16 * kk) * VROWB + db * 64;
    return read_tr_pair(a0, a0 + 4 * VROWB);
  }
  static __device__ __forceinline__ void store_k(unsigned char* tile, int row, int ch, i32x4 val) {
    *reinterpret_cast<i32x4*>(tile + row * KROWB + (ch << 4)) = val;
  }
  static __device__ __forceinline__ void store_v(unsigned char* tile, int row, int ch, i32x4 val) {
    *reinterpret_cast<i32x4*>(tile + row * VROWB + (ch << 4)) = val;
  }
};

// ---------------------------------------------------------------------------
// Layout policy 2: XOR-swizzled 16-byte chunks, unpadded rows of DP*2 bytes.
// LDS slot s of row r holds logical chunk s ^ swz(r).
template <int D>
struct SwizzledFrags {
  using G = RowGeom<D>;
  static constexpr int ROWB = G::DP * 2;
  static constexpr int SLOTS = ROWB / 16;  // 16-byte slots per row
  static __device__ __forceinline__ int swz_k(int row) {
    return G::DP == 128 ? (row & 15) : ((row >> 1) & 7);
  }
  static __device__ __forceinline__ int swz_v(int row) {
    return G::DP == 128 ? (((row & 3) << 2) | ((row >> 2) & 3)) : (((row >> 1) & 1) << 2);
  }
  int lq, lh;
  uint32_t k_a[G::KSTEPS];  // byte offset of chunk step c inside a 32-key block
  uint32_t v_a[G::NDB][2];  // byte offset of (d block, first/second read) inside a 16-key group

  // The lane registers hold absolute LDS addresses: lds_base is the address of
  // the first K tile, lds_base + v_bias that of the first V tile (the V tiles
  // may then live beyond the 64 KiB reach of a DS immediate while every read
  // still is "lane register + immediate" with the tile offset of its K tile).
  // Each address is pinned in a register of its own (empty asm): the compiler
  // would otherwise re-derive them with vector adds inside the loop, or fold
  // the bias into the immediates and push those past 64 KiB.
  __device__ __forceinline__ void init(int lane, uint32_t lds_base, int v_bias) {
    lq = lane & 31;
    lh = lane >> 5;
    v_bias += (int)lds_base;
    asm volatile("" : "+v"(v_bias));
    const int krow = key_perm(lq);
#pragma unroll
    for (int c = 0; c < G::KSTEPS; ++c) {
      k_a[c] = lds_base + krow * ROWB + (((2 * c + lh) ^ swz_k(krow)) << 4);
      asm volatile("" : "+v"(k_a[c]));
    }
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int r = 8 * lh + 4 * e + ((lane & 15) >> 2);
#pragma unroll
      for (int db = 0; db < G::NDB; ++db) {
        const int ch = 4 * db + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
        v_a[db][e] = v_bias + r * ROWB + ((ch ^ swz_v(r)) << 4) + (lane & 1) * 8;
        asm volatile("" : "+v"(v_a[db][e]));
      }
    }
  }
  // swz_k is invariant under row += 32, swz_v under row += 16
  // tile_off: byte offset of the stage's K tile from the first K tile (the V
  // tile of the same stage sits at the same offset from the first V tile)
  __device__ __forceinline__ i32x4 load_k(uint32_t tile_off, int kb, int c) const {
    typedef __attribute__((address_space(3))) const i32x4 lds_i32x4;
    return *(lds_i32x4*)(uintptr_t)(k_a[c] + tile_off + kb * 32 * ROWB);
  }
  __device__ __forceinline__ i32x4 load_v(uint32_t tile_off, int kk, int db) const {
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(uintptr_t)(v_a[db][0] + tile_off + kk * 16 * ROWB));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(uintptr_t)(v_a[db][1] + tile_off + kk * 16 * ROWB));
    i32x2 l2 = __builtin_bit_cast(i32x2, lo);
    i32x2 h2 = __builtin_bit_cast(i32x2, hi);
    i32x4 out = {l2[0], l2[1], h2[0], h2[1]};
    return out;
  }
};

// The running max may lag behind the true row max by up to this many binades
// before the accumulators are rescaled: probabilities then reach 2^8 at most,
// far inside the range of the 16-bit formats and of the fp32 sums, and the
// final o = O / l and lse = m + log2(l) do not depend on which m was used.
constexpr float kRescaleSlack = 8.0f;

// S^T = K Q^T for a tile of NKB 32-key blocks: NKB independent accumulator
// chains stepped alternately, K fragments fetched kPrefetch steps ahead of the
// MFMA that uses them.
template <typename T, int D, int NKB, typename Frags, typename Tile>
__device__ __forceinline__ void qk_scores(Tile sK, const Frags& fr,
                                          const i32x4 (&Qf)[RowGeom<D>::KSTEPS], f32x16 (&S)[NKB]) {
  using G = RowGeom<D>;
  constexpr int NSTEP = NKB * G::KSTEPS;
  constexpr int kPrefetch = 4;
  i32x4 kf[kPrefetch];
#pragma unroll
  for (int s = 0; s < kPrefetch; ++s) kf[s] = fr.load_k(sK, s % NKB, s / NKB);
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb) S[kb] = (f32x16){0};
#pragma unroll
  for (int s = 0; s < NSTEP; ++s) {
    S[s % NKB] = Elem<T>::mfma(kf[s % kPrefetch], Qf[s / NKB], S[s % NKB]);
    if (s + kPrefetch < NSTEP) kf[s % kPrefetch] = fr.load_k(sK, (s + kPrefetch) % NKB, (s + kPrefetch) / NKB);
  }
  // Pin that order for the instruction scheduler (it otherwise sinks every LDS
  // read to just before its MFMA and exposes the LDS latency at every step):
  // kPrefetch reads, then one MFMA + one read per step, then the MFMA tail.
  __builtin_amdgcn_sched_group_barrier(0x100, kPrefetch, 0);
#pragma unroll
  for (int s = 0; s < NSTEP - kPrefetch; ++s) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
  }
  __builtin_amdgcn_sched_group_barrier(0x008, kPrefetch, 0);
}

// Online-softmax step on the scores of one tile.  On return P holds the packed
// 16-bit probabilities (P[kb][i] = keys 2i, 2i+1 of the lane's 16 keys in block
// kb), l has this lane's share of the row sum added, and O / l / m have been
// rescaled if the row max outgrew the slack.
template <typename T, int D, int NKB, typename MaskF>
__device__ __forceinline__ void softmax_tile(f32x16 (&S)[NKB], int lh, f32x16 (&O)[RowGeom<D>::NDB], float& m,
                                             float& l, float scale, bool need_mask, MaskF allowed,
                                             uint32_t (&P)[NKB][8]) {
  using G = RowGeom<D>;
  if (need_mask) {
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = kb * 32 + 16 * (r >> 3) + 8 * lh + (r & 7);
        if (!allowed(key)) S[kb][r] = -INFINITY;
      }
  }

  float mx = S[0][0];
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
    for (int r = 0; r < 16; ++r) mx = fmaxf(mx, S[kb][r]);
  mx = max_with_other_half(mx);

  // Lazy rescale: keep exponentiating against the old max while the new one
  // is at most kRescaleSlack above it (wave-uniform branch, rarely taken after
  // the first tiles).
  const float m_new = fmaxf(m, mx * scale);
  if (__builtin_amdgcn_ballot_w64(m_new > m + kRescaleSlack) != 0) {
    // a lane whose keys were all masked so far has m = m_new = -inf: factor 0
    const float alpha = fast_exp2(m - ((m_new == -INFINITY) ? 0.f : m_new));
    l *= alpha;
#pragma unroll
    for (int db = 0; db < G::NDB; ++db) O[db] *= alpha;
    m = m_new;
  }
  const float m_use = (m == -INFINITY) ? 0.f : m;  // nothing but masked keys so far

  float rs = 0.f;
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const float p0 = fast_exp2(fmaf(S[kb][r], scale, -m_use));
      const float p1 = fast_exp2(fmaf(S[kb][r + 1], scale, -m_use));
      rs += p0 + p1;
      P[kb][r >> 1] = Elem<T>::pack2(p0, p1);
    }
  l += rs;
}

// O^T += V^T P^T for one tile.
template <typename T, int D, int NKB, typename Frags, typename Tile>
__device__ __forceinline__ void pv_accumulate(Tile sV, const Frags& fr,
                                              const uint32_t (&P)[NKB][8], f32x16 (&O)[RowGeom<D>::NDB]) {
  using G = RowGeom<D>;
#pragma unroll
  for (int kk = 0; kk < 2 * NKB; ++kk) {
    const int kb = kk >> 1, o4 = (kk & 1) * 4;
    const i32x4 pf = {(int)P[kb][o4], (int)P[kb][o4 + 1], (int)P[kb][o4 + 2], (int)P[kb][o4 + 3]};
#pragma unroll
    for (int db = 0; db < G::NDB; ++db) {
      const i32x4 vf = fr.load_v(sV, kk, db);
      O[db] = Elem<T>::mfma(vf, pf, O[db]);
    }
  }
}

// One KV tile of NKB*32 keys against the wave's 32 queries.
//   sK, sV : LDS tiles holding the keys of this tile, in the layout of Frags
//            (pointers for PaddedFrags, byte offsets for SwizzledFrags)
//   Qf     : B operands of Q^T, chunk c covers d = 16c .. 16c+15
//   O      : O^T accumulators, block db covers d = 32db .. 32db+31
//   m      : reference max of the exponent, scaled base-2 domain (-inf at
//            start); within kRescaleSlack of the true running max
//   l      : this lane's share of the running row sum (the other half of the
//            sum lives in lane l^32; add them at the end)
//   allowed(key_in_tile) is consulted only when need_mask is true.
template <typename T, int D, int NKB, typename Frags, typename Tile, typename MaskF>
__device__ __forceinline__ void compute_tile(Tile sK, Tile sV, const Frags& fr, const i32x4 (&Qf)[RowGeom<D>::KSTEPS],
                                             f32x16 (&O)[RowGeom<D>::NDB], float& m, float& l,
                                             float scale, bool need_mask, MaskF allowed) {
  f32x16 S[NKB];
  uint32_t P[NKB][8];
  qk_scores<T, D, NKB>(sK, fr, Qf, S);
  softmax_tile<T, D, NKB>(S, fr.lh, O, m, l, scale, need_mask, allowed, P);
  pv_accumulate<T, D, NKB>(sV, fr, P, O);
}

}  // namespace mi
