// Prefill (many-query) attention forward for gfx950: dense causal / non-causal
// and block-sparse, packed var-len or batched, GQA.
//
// Work decomposition: one workgroup = NW wavefronts = 32*NW consecutive query
// rows of one (sequence, q-head); KV is walked in tiles of 64 keys that the
// whole workgroup stages through LDS (double buffered, one barrier per tile);
// each wavefront then runs compute_tile() on its own 32 rows.
//
// Replaces flash_attn_fwd_kernel of flash_attn_triton/flash_attn_triton.py
// :52-180 (dense) and flash_attn_triton/flash_attn_sparse_attn_triton.py
// :47-234 (sparse).  Differences from the reference on purpose: the softmax
// carries (max, sum) and forms the base-2 LSE once at the end instead of an
// exp2+log2 pair per tile (:170); masks are built only for tiles that cross
// the diagonal, the sequence end or a window edge (:148-154 builds one for
// every tile); Q is read once (:155 re-reads it per tile).
#include "kernels.h"
#include "tile_core.h"

namespace mi {
namespace {

template <typename T, int D, int NW, bool SPARSE>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2)))
prefill_kernel(const PrefillParams p) {
  using G = RowGeom<D>;
  constexpr int BM = 32 * NW;
  constexpr int NT = 64 * NW;
  constexpr int KTILEB = kTileN * G::KROWB;
  constexpr int VTILEB = kTileN * G::VROWB;
  constexpr int STAGEB = KTILEB + VTILEB;
  constexpr int NCHUNK = kTileN * G::NCH;            // 16-byte chunks per tile
  constexpr int LOADS = (NCHUNK + NT - 1) / NT;      // per thread, per tensor
  constexpr int OROWB = D * 2 + 16;                  // epilogue staging row

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;

  // ---- workgroup -> (sequence, head, q tile).  Consecutive workgroup ids are
  // dealt round-robin to the 8 XCDs, each with a private L2: give every XCD
  // whole (sequence, kv-head) units so their K/V stay in one L2, and walk the
  // q tiles of a unit from the longest (last) to the shortest.
  const int gqa = p.hq / p.hkv;
  const int per_unit = p.n_qtiles * gqa;
  const int n_units = p.batch * p.hkv;
  int unit, s;
  {
    const int bid = blockIdx.x;
    if ((n_units & 7) == 0) {
      const int xcd = bid & 7, slot = bid >> 3;
      unit = (slot / per_unit) * 8 + xcd;
      s = slot % per_unit;
    } else {
      unit = bid / per_unit;
      s = bid % per_unit;
    }
  }
  const int qt = p.n_qtiles - 1 - s / gqa;
  const int b = unit / p.hkv;
  const int kvh = unit % p.hkv;
  const int h = kvh * gqa + s % gqa;

  int len;
  int64_t q_off, k_off, v_off, o_off, lse_off;
  if (p.cu) {
    const int start = p.cu[b];
    len = p.cu[b + 1] - start;
    q_off = start * p.q_ss;
    k_off = start * p.k_ss;
    v_off = start * p.v_ss;
    o_off = start * p.o_ss;
    lse_off = start * p.lse_ss;
  } else {
    len = p.max_seqlen;
    q_off = b * p.q_sb;
    k_off = b * p.k_sb;
    v_off = b * p.v_sb;
    o_off = b * p.o_sb;
    lse_off = b * p.lse_sb;
  }
  const int q0 = qt * BM;
  if (q0 >= len) return;

  const T* qp = reinterpret_cast<const T*>(p.q) + q_off + h * p.q_sh;
  const T* kp = reinterpret_cast<const T*>(p.k) + k_off + kvh * p.k_sh;
  const T* vp = reinterpret_cast<const T*>(p.v) + v_off + kvh * p.v_sh;
  T* op = reinterpret_cast<T*>(p.o) + o_off + h * p.o_sh;

  LaneCtx<D> lc;
  lc.init(lane);
  const int q0w = q0 + 32 * wave;
  const int qrow = q0w + lc.lq;

  // ---- tile list
  int n_tiles;
  const int32_t* cols = nullptr;
  if constexpr (SPARSE) {
    const int32_t* rp = p.row_ptr + b * p.rp_sb + h * p.rp_sh;
    const int beg = rp[qt];
    n_tiles = rp[qt + 1] - beg;
    cols = p.col_idx + b * p.ci_sb + h * p.ci_sh + beg;
  } else {
    n_tiles = (len + kTileN - 1) / kTileN;
    if (p.causal) n_tiles = min(n_tiles, (q0 + BM + kTileN - 1) / kTileN);
  }

  // ---- Q^T operands: lane (query lq, half lh) holds d = 16c + 8lh .. +7
  i32x4 Qf[G::KSTEPS];
  {
    const T* qr = qp + (int64_t)min(qrow, len - 1) * p.q_ss + 8 * lc.lh;
#pragma unroll
    for (int c = 0; c < G::KSTEPS; ++c) Qf[c] = *reinterpret_cast<const i32x4*>(qr + 16 * c);
  }

  f32x16 O[G::NDB];
#pragma unroll
  for (int db = 0; db < G::NDB; ++db) O[db] = (f32x16){0};
  float m = -INFINITY, l = 0.f;

  // ---- global -> register -> LDS staging of one K and one V tile
  i32x4 kreg[LOADS], vreg[LOADS];
  auto gload = [&](int col) {
    const int k0 = col * kTileN;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int idx = tid + i * NT;
      if (NCHUNK % NT == 0 || idx < NCHUNK) {
        const int row = idx / G::NCH, ch = idx % G::NCH;
        const int64_t kr = min(k0 + row, len - 1);  // clamp: masked later
        kreg[i] = *reinterpret_cast<const i32x4*>(kp + kr * p.k_ss + ch * 8);
        vreg[i] = *reinterpret_cast<const i32x4*>(vp + kr * p.v_ss + ch * 8);
      }
    }
  };
  auto lstore = [&](int stage) {
    unsigned char* sK = smem + stage * STAGEB;
    unsigned char* sV = sK + KTILEB;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int idx = tid + i * NT;
      if (NCHUNK % NT == 0 || idx < NCHUNK) {
        const int row = idx / G::NCH, ch = idx % G::NCH;
        lds_store_k<D>(sK, row, ch, kreg[i]);
        lds_store_v<D>(sV, row, ch, vreg[i]);
      }
    }
  };

  if (n_tiles > 0) {
    gload(SPARSE ? cols[0] : 0);
    lstore(0);
  }
  // Drain every outstanding global load (the Q fragments) here, so that inside
  // the loop the only loads in flight are the next tile's and no MFMA has to
  // wait on a vector-memory counter.  s_waitcnt vmcnt(0) expcnt(7) lgkmcnt(15).
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();

  for (int it = 0; it < n_tiles; ++it) {
    const int col = SPARSE ? cols[it] : it;
    const bool more = it + 1 < n_tiles;
    if (more) gload(SPARSE ? cols[it + 1] : it + 1);

    const int k0 = col * kTileN;
    // whole tile above the diagonal for this wave: nothing to add
    const bool skip = p.causal && k0 > q0w + 31;
    if (!skip) {
      bool need_mask = (k0 + kTileN > len) || (p.causal && k0 + kTileN - 1 > q0w);
      const int wl = p.win_local, wg = p.win_global;
      if (SPARSE && wl >= 0) need_mask = need_mask || !((k0 + kTileN - 1 < wg) || (q0w + 31 - k0 < wl));
      const int causal = p.causal;
      auto allowed = [&](int key_in_tile) -> bool {
        const int key = k0 + key_in_tile;
        bool ok = key < len && (!causal || key <= qrow);
        if (SPARSE && wl >= 0) ok = ok && ((qrow - key < wl) || (key < wg));
        return ok;
      };
      const unsigned char* sK = smem + (it & 1) * STAGEB;
      compute_tile<T, D, 2>(sK, sK + KTILEB, lc, Qf, O, m, l, p.scale, need_mask, allowed);
    }
    if (more) lstore((it + 1) & 1);
    __syncthreads();
  }

  // ---- epilogue: normalise, transpose through LDS, coalesced 16-byte stores
  const float l_tot = sum_with_other_half(l);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (p.lse && lc.lh == 0 && qrow < len) {
    float* lp = p.lse + lse_off + h * p.lse_sh;
    lp[(int64_t)qrow * p.lse_ss] = l_tot > 0.f ? m + fast_log2(l_tot) : -INFINITY;
  }
  unsigned char* stage = smem + wave * 32 * OROWB;
#pragma unroll
  for (int db = 0; db < G::NDB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = 32 * db + 8 * g + 4 * lc.lh;
      i32x2 w;
      w[0] = (int)Elem<T>::pack2(O[db][4 * g] * inv, O[db][4 * g + 1] * inv);
      w[1] = (int)Elem<T>::pack2(O[db][4 * g + 2] * inv, O[db][4 * g + 3] * inv);
      *reinterpret_cast<i32x2*>(stage + lc.lq * OROWB + d * 2) = w;
    }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < (32 * G::NCH + 63) / 64; ++i) {
    const int idx = lane + 64 * i;
    const int row = idx / G::NCH, ch = idx % G::NCH;
    if (((32 * G::NCH) % 64 == 0 || idx < 32 * G::NCH) && q0w + row < len) {
      const i32x4 val = *reinterpret_cast<const i32x4*>(stage + row * OROWB + ch * 16);
      *reinterpret_cast<i32x4*>(op + (int64_t)(q0w + row) * p.o_ss + ch * 8) = val;
    }
  }
}

template <int D, int NW>
constexpr size_t prefill_lds_bytes() {
  const size_t pipe = 2 * kTileN * (RowGeom<D>::KROWB + RowGeom<D>::VROWB);
  const size_t epi = (size_t)NW * 32 * (D * 2 + 16);
  return pipe > epi ? pipe : epi;
}

template <typename T, int D, int NW, bool SPARSE>
int launch_one(const PrefillParams& p, hipStream_t s) {
  auto kern = prefill_kernel<T, D, NW, SPARSE>;
  constexpr size_t lds = prefill_lds_bytes<D, NW>();
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
  const long long grid = (long long)p.n_qtiles * p.hq * p.batch;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NW * 64), lds, s, p);
  return (int)hipGetLastError();
}

template <int NW, bool SPARSE>
int dispatch(const PrefillParams& p, int dtype, int head_dim, hipStream_t s) {
  if (dtype == 0) {
    switch (head_dim) {
      case 64: return launch_one<__bf16, 64, NW, SPARSE>(p, s);
      case 96: return launch_one<__bf16, 96, NW, SPARSE>(p, s);
      case 128: return launch_one<__bf16, 128, NW, SPARSE>(p, s);
    }
  } else {
    switch (head_dim) {
      case 64: return launch_one<_Float16, 64, NW, SPARSE>(p, s);
      case 96: return launch_one<_Float16, 96, NW, SPARSE>(p, s);
      case 128: return launch_one<_Float16, 128, NW, SPARSE>(p, s);
    }
  }
  return (int)hipErrorInvalidValue;
}

}  // namespace

int launch_prefill_dense(const PrefillParams& p, int dtype, int head_dim, hipStream_t s) {
  return dispatch<kDenseRows / 32, false>(p, dtype, head_dim, s);
}
int launch_prefill_sparse(const PrefillParams& p, int dtype, int head_dim, hipStream_t s) {
  return dispatch<kSparseRows / 32, true>(p, dtype, head_dim, s);
}

}  // namespace mi
