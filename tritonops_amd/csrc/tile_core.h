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
// LDS tile layout: row-major [key][head_dim], rows padded so that the access
// patterns below are bank-conflict free and every fragment address is a
// per-lane base plus a compile-time immediate: K rows carry 16 pad bytes (a
// fragment read takes one 16 B chunk from 16 consecutive rows per quarter
// wave), V rows 64 pad bytes (a transposing read takes 64 B from each of 4
// consecutive rows per half wave).
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
  static constexpr int DP = (D == 64) ? 64 : 128;  // padded row, elements
  static constexpr int KROWB = DP * 2 + 16;        // LDS bytes per K row
  static constexpr int VROWB = DP * 2 + 64;        // LDS bytes per V row
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

// Value held by lane l^32.
__device__ __forceinline__ float other_half(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  // r[0]: both halves see the lower half's value; r[1]: the upper half's.
  const unsigned lo = r[0], hi = r[1];
  return __builtin_bit_cast(float, (threadIdx.x & 32) ? lo : hi);
}
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

// Per-lane constants of the fragment addressing, computed once per kernel.
template <int D>
struct LaneCtx {
  int lq;     // query column of this lane (lane % 32)
  int lh;     // lane half (lane / 32)
  int k_off;  // byte offset of this lane's K fragment inside a 32-key block, chunk 0
  int v_off;  // byte offset of this lane's V^T fragment for kk = 0, db = 0, first read

  __device__ __forceinline__ void init(int lane) {
    using G = RowGeom<D>;
    lq = lane & 31;
    lh = lane >> 5;
    k_off = key_perm(lq) * G::KROWB + lh * 16;
    // transposing read: lane j of a 16-lane group addresses row j/4, 8 bytes at
    // element 4*(j%4) of the group's 16 columns; groups 0/1 (2/3) are the two
    // column halves of lane half 0 (1), which starts 8 rows further down.
    v_off = (8 * lh + ((lane & 15) >> 2)) * G::VROWB + (2 * ((lane >> 4) & 1) + ((lane & 3) >> 1)) * 16 +
            (lane & 1) * 8;
  }
};

// Store one 16-byte chunk of a K / V row into its LDS slot.
template <int D>
__device__ __forceinline__ void lds_store_k(unsigned char* tile, int row, int ch, i32x4 val) {
  *reinterpret_cast<i32x4*>(tile + row * RowGeom<D>::KROWB + (ch << 4)) = val;
}
template <int D>
__device__ __forceinline__ void lds_store_v(unsigned char* tile, int row, int ch, i32x4 val) {
  *reinterpret_cast<i32x4*>(tile + row * RowGeom<D>::VROWB + (ch << 4)) = val;
}

// A operand of O^T += V^T P^T for 16-key group kk and 32-wide d block db:
// lane (d = 32*db + lane%32) receives V[16*kk + 8*(lane/32) + 0..7][d].
template <int D>
__device__ __forceinline__ i32x4 load_vt_frag(const unsigned char* sV, const LaneCtx<D>& lc, int kk,
                                              int db) {
  using G = RowGeom<D>;
  const unsigned char* a0 = sV + lc.v_off + (16 * kk) * G::VROWB + db * 64;
  const unsigned char* a1 = a0 + 4 * G::VROWB;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)a0);
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)a1);
  i32x2 l2 = __builtin_bit_cast(i32x2, lo);
  i32x2 h2 = __builtin_bit_cast(i32x2, hi);
  i32x4 out = {l2[0], l2[1], h2[0], h2[1]};
  return out;
}

// The running max may lag behind the true row max by up to this many binades
// before the accumulators are rescaled: probabilities then reach 2^8 at most,
// far inside the range of the 16-bit formats and of the fp32 sums, and the
// final o = O / l and lse = m + log2(l) do not depend on which m was used.
constexpr float kRescaleSlack = 8.0f;

// One KV tile of NKB*32 keys against the wave's 32 queries.
//   sK, sV : LDS tiles (row-major, swizzled) holding the keys of this tile
//   Qf     : B operands of Q^T, chunk c covers d = 16c .. 16c+15
//   O      : O^T accumulators, block db covers d = 32db .. 32db+31
//   m      : reference max of the exponent, scaled base-2 domain (-inf at
//            start); within kRescaleSlack of the true running max
//   l      : this lane's share of the running row sum (the other half of the
//            sum lives in lane l^32; add them at the end)
//   allowed(key_in_tile) is consulted only when need_mask is true.
template <typename T, int D, int NKB, typename MaskF>
__device__ __forceinline__ void compute_tile(const unsigned char* sK, const unsigned char* sV,
                                             const LaneCtx<D>& lc,
                                             const i32x4 (&Qf)[RowGeom<D>::KSTEPS],
                                             f32x16 (&O)[RowGeom<D>::NDB], float& m, float& l,
                                             float scale, bool need_mask, MaskF allowed) {
  using G = RowGeom<D>;
  // S^T = K Q^T: NKB independent accumulator chains, stepped alternately, with
  // the K fragments fetched kPrefetch steps ahead of the MFMA that uses them.
  f32x16 S[NKB];
  {
    constexpr int NSTEP = NKB * G::KSTEPS;
    constexpr int kPrefetch = 4;
    auto frag = [&](int s) -> i32x4 {
      const int kb = s % NKB, c = s / NKB;
      return *reinterpret_cast<const i32x4*>(sK + lc.k_off + kb * 32 * G::KROWB + 32 * c);
    };
    i32x4 kf[kPrefetch];
#pragma unroll
    for (int s = 0; s < kPrefetch; ++s) kf[s] = frag(s);
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) S[kb] = (f32x16){0};
#pragma unroll
    for (int s = 0; s < NSTEP; ++s) {
      S[s % NKB] = Elem<T>::mfma(kf[s % kPrefetch], Qf[s / NKB], S[s % NKB]);
      if (s + kPrefetch < NSTEP) kf[s % kPrefetch] = frag(s + kPrefetch);
    }
    // Pin that order for the instruction scheduler (it otherwise sinks every
    // LDS read to just before its MFMA and exposes the LDS latency 16 times):
    // kPrefetch reads, then one MFMA + one read per step, then the MFMA tail.
    __builtin_amdgcn_sched_group_barrier(0x100, kPrefetch, 0);
#pragma unroll
    for (int s = 0; s < NSTEP - kPrefetch; ++s) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kPrefetch, 0);
  }

  if (need_mask) {
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = kb * 32 + 16 * (r >> 3) + 8 * lc.lh + (r & 7);
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

  uint32_t P[NKB][8];
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

#pragma unroll
  for (int kk = 0; kk < 2 * NKB; ++kk) {
    const int kb = kk >> 1, o4 = (kk & 1) * 4;
    const i32x4 pf = {(int)P[kb][o4], (int)P[kb][o4 + 1], (int)P[kb][o4 + 2], (int)P[kb][o4 + 3]};
#pragma unroll
    for (int db = 0; db < G::NDB; ++db) {
      const i32x4 vf = load_vt_frag<D>(sV, lc, kk, db);
      O[db] = Elem<T>::mfma(vf, pf, O[db]);
    }
  }
}

}  // namespace mi
