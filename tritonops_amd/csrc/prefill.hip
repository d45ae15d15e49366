// Prefill (many-query) attention forward for gfx950: dense causal / non-causal
// and block-sparse, packed var-len or batched, GQA.
//
// Work decomposition: one workgroup = NW wavefronts = 32*NW consecutive query
// rows of one (sequence, q-head); KV is walked in tiles of 64 keys that the
// whole workgroup brings into LDS with direct-to-LDS loads
// (global_load_lds_dwordx4: no staging registers, no ds_write), double
// buffered, one barrier per tile; each wavefront then runs compute_tile() on
// its own 32 rows.
//
// Replaces flash_attn_fwd_kernel of flash_attn_triton/flash_attn_triton.py
// :52-180 (dense) and flash_attn_triton/flash_attn_sparse_attn_triton.py
// :47-234 (sparse).  Differences from the reference on purpose: the softmax
// carries (max, sum) and forms the base-2 LSE once at the end instead of an
// exp2+log2 pair per tile (:170); masks are built only for tiles that cross
// the diagonal, the sequence end or a window edge (:148-154 builds one for
// every tile); Q is read once (:155 re-reads it per tile).
#include <type_traits>

#include "kernels.h"
#include "tile_core.h"

namespace mi {
namespace {

typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void glb_void;

template <int V>
using ic = std::integral_constant<int, V>;

// vmcnt(N) expcnt(7) lgkmcnt(15) for s_waitcnt on gfx9-family encodings
constexpr int waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

// NW wavefronts per workgroup, NS LDS stages (tiles in flight + the one in
// use), TN keys per tile (64, or 32 so that more workgroups fit one CU's LDS).
template <typename T, int D, int NW, int NS, int TN, bool SPARSE>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2)))
prefill_kernel(const PrefillParams p) {
  using G = RowGeom<D>;
  using F = SwizzledFrags<D>;
  constexpr int BM = 32 * NW;
  constexpr int TILEB = TN * F::ROWB;   // one K or V tile
  constexpr int VBASE = NS * TILEB;         // LDS: NS K tiles, then NS V tiles
  constexpr int RPI = 1024 / F::ROWB;       // tile rows filled by one direct-to-LDS instruction
  constexpr int NINST = TN / RPI;       // such instructions per tensor per tile
  constexpr int IPW = NINST / NW;           // ... per wavefront
  static_assert(NINST % NW == 0, "tile rows must split evenly over the waves");
  constexpr int OROWB = D * 2 + 16;         // epilogue staging row

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

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

  F fr;
  fr.init(lane, VBASE);
  const int q0w = q0 + 32 * wave;
  const int qrow = q0w + fr.lq;

  // ---- tile list
  int n_tiles;
  const int32_t* cols = nullptr;
  if constexpr (SPARSE) {
    const int32_t* rp = p.row_ptr + b * p.rp_sb + h * p.rp_sh;
    const int beg = rp[qt];
    n_tiles = (rp[qt + 1] - beg) * (kTileN / TN);  // a 64-key block is TN-key tiles
    cols = p.col_idx + b * p.ci_sb + h * p.ci_sh + beg;
  } else {
    static_assert(SPARSE || TN == kTileN, "dense kernel walks 64-key tiles");
    n_tiles = (len + TN - 1) / TN;
    if (p.causal) n_tiles = min(n_tiles, (q0 + BM + TN - 1) / TN);
  }

  // ---- Q^T operands: lane (query lq, half lh) holds d = 16c + 8lh .. +7
  i32x4 Qf[G::KSTEPS];
  {
    const T* qr = qp + (int64_t)min(qrow, len - 1) * p.q_ss + 8 * fr.lh;
#pragma unroll
    for (int c = 0; c < G::KSTEPS; ++c) Qf[c] = *reinterpret_cast<const i32x4*>(qr + 16 * c);
  }

  f32x16 O[G::NDB];
#pragma unroll
  for (int db = 0; db < G::NDB; ++db) O[db] = (f32x16){0};
  float m = -INFINITY, l = 0.f;

  // ---- direct-to-LDS tile loads.  Instruction t of this wave fills the 1 KiB
  // of LDS that holds tile rows RPI*(wave + NW*t) .. +RPI-1: lane i's 16 bytes
  // land in slot i of that KiB, i.e. row drow = i / SLOTS, slot dslot = i %
  // SLOTS, which must receive logical chunk dslot ^ swz(row) of that row.
  const int drow = lane / F::SLOTS, dslot = lane % F::SLOTS;
  const int64_t k_rowb = p.k_ss * 2, v_rowb = p.v_ss * 2;  // bytes between keys
  // first key of tile `it` of this workgroup's list
  auto tile_k0 = [&](int it) -> int {
    if (!SPARSE) return it * TN;
    constexpr int PER = kTileN / TN;
    return cols[it / PER] * kTileN + (it % PER) * TN;
  };
  auto dma_tile = [&](int k0, auto stage_c) {
    constexpr int ST = decltype(stage_c)::value;
    const char* kt = reinterpret_cast<const char*>(kp) + k0 * k_rowb;
    const char* vt = reinterpret_cast<const char*>(vp) + k0 * v_rowb;
    unsigned char* sK = smem + ST * TILEB;
    unsigned char* sV = smem + VBASE + ST * TILEB;
    if (k0 + TN <= len) {
      // whole tile inside the sequence: uniform base + 32-bit lane offset
#pragma unroll
      for (int t = 0; t < IPW; ++t) {
        const int inst = wave + NW * t;
        const int r = RPI * inst + drow;
        const int kc = dslot ^ F::swz_k(r), vc = dslot ^ F::swz_v(r);
        const uint32_t kl = (uint32_t)drow * (uint32_t)k_rowb + (uint32_t)kc * 16u;
        const uint32_t vl = (uint32_t)drow * (uint32_t)v_rowb + (uint32_t)vc * 16u;
        if (D != 96 || kc < G::NCH)
          __builtin_amdgcn_global_load_lds((glb_void*)(kt + (RPI * inst) * k_rowb + kl),
                                           (lds_void*)(sK + inst * 1024), 16, 0, 0);
        if (D != 96 || vc < G::NCH)
          __builtin_amdgcn_global_load_lds((glb_void*)(vt + (RPI * inst) * v_rowb + vl),
                                           (lds_void*)(sV + inst * 1024), 16, 0, 0);
      }
    } else {
      // rows past the sequence end re-read its last row (masked later)
#pragma unroll
      for (int t = 0; t < IPW; ++t) {
        const int inst = wave + NW * t;
        const int r = RPI * inst + drow;
        const int kc = dslot ^ F::swz_k(r), vc = dslot ^ F::swz_v(r);
        const int64_t rr = min(k0 + r, len - 1) - k0;
        if (D != 96 || kc < G::NCH)
          __builtin_amdgcn_global_load_lds((glb_void*)(kt + rr * k_rowb + kc * 16), (lds_void*)(sK + inst * 1024),
                                           16, 0, 0);
        if (D != 96 || vc < G::NCH)
          __builtin_amdgcn_global_load_lds((glb_void*)(vt + rr * v_rowb + vc * 16), (lds_void*)(sV + inst * 1024),
                                           16, 0, 0);
      }
    }
  };

  auto step = [&](auto stage_c, int it) {
    constexpr int ST = decltype(stage_c)::value;
    // refill the stage that was read in the previous iteration
    const bool refill = it + NS - 1 < n_tiles;
    if (refill) dma_tile(tile_k0(it + NS - 1), ic<(ST + NS - 1) % NS>{});

    const int k0 = tile_k0(it);
    // whole tile above the diagonal for this wave: nothing to add
    const bool skip = p.causal && k0 > q0w + 31;
    if (!skip) {
      bool need_mask = (k0 + TN > len) || (p.causal && k0 + TN - 1 > q0w);
      const int wl = p.win_local, wg = p.win_global;
      if (SPARSE && wl >= 0) need_mask = need_mask || !((k0 + TN - 1 < wg) || (q0w + 31 - k0 < wl));
      const int causal = p.causal;
      auto allowed = [&](int key_in_tile) -> bool {
        const int key = k0 + key_in_tile;
        bool ok = key < len && (!causal || key <= qrow);
        if (SPARSE && wl >= 0) ok = ok && ((qrow - key < wl) || (key < wg));
        return ok;
      };
      // V addresses carry VBASE inside the lane offsets (see fr.init)
      compute_tile<T, D, TN / 32>(smem + ST * TILEB, smem + ST * TILEB, fr, Qf, O, m, l, p.scale, need_mask, allowed);
    }
    // The next tile must have landed and everyone must be done with this one.
    // This wave's loads complete in order, so it is enough that at most the
    // loads of the NS-2 younger tiles are still in flight (2*IPW each).
    if (refill)
      __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 2) * 2 * IPW));
    else
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __syncthreads();
  };

#pragma unroll
  for (int s0 = 0; s0 < NS - 1; ++s0)
    if (s0 < n_tiles) {
      if (s0 == 0) dma_tile(tile_k0(0), ic<0>{});
      if (s0 == 1) dma_tile(tile_k0(1), ic<1 % NS>{});
      if (s0 == 2) dma_tile(tile_k0(2), ic<2 % NS>{});
    }
  // tile 0 (and the Q loads issued before it) must be complete
  if (n_tiles >= NS - 1)
    __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 2) * 2 * IPW));
  else
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
  __syncthreads();

  int it = 0;
  for (; it + NS <= n_tiles; it += NS) {
    step(ic<0>{}, it);
    step(ic<1 % NS>{}, it + 1);
    if (NS > 2) step(ic<2 % NS>{}, it + 2);
    if (NS > 3) step(ic<3 % NS>{}, it + 3);
  }
  if (it < n_tiles) step(ic<0>{}, it++);
  if (it < n_tiles) step(ic<1 % NS>{}, it++);
  if (NS > 3 && it < n_tiles) step(ic<2 % NS>{}, it++);

  // ---- epilogue: normalise, transpose through LDS, coalesced 16-byte stores
  const float l_tot = sum_with_other_half(l);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (p.lse && fr.lh == 0 && qrow < len) {
    float* lp = p.lse + lse_off + h * p.lse_sh;
    lp[(int64_t)qrow * p.lse_ss] = l_tot > 0.f ? m + fast_log2(l_tot) : -INFINITY;
  }
  unsigned char* stage = smem + wave * 32 * OROWB;
#pragma unroll
  for (int db = 0; db < G::NDB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = 32 * db + 8 * g + 4 * fr.lh;
      i32x2 w;
      w[0] = (int)Elem<T>::pack2(O[db][4 * g] * inv, O[db][4 * g + 1] * inv);
      w[1] = (int)Elem<T>::pack2(O[db][4 * g + 2] * inv, O[db][4 * g + 3] * inv);
      *reinterpret_cast<i32x2*>(stage + fr.lq * OROWB + d * 2) = w;
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

template <int D, int NW, int NS, int TN>
constexpr size_t prefill_lds_bytes() {
  const size_t pipe = (size_t)NS * 2 * TN * SwizzledFrags<D>::ROWB;
  const size_t epi = (size_t)NW * 32 * (D * 2 + 16);
  return pipe > epi ? pipe : epi;
}

template <typename T, int D, int NW, bool SPARSE>
int launch_one(const PrefillParams& p, hipStream_t s) {
  constexpr int NS = SPARSE ? kSparseStages : kDenseStages;
  constexpr int TN = SPARSE ? kSparseTileKeys : kTileN;
  auto kern = prefill_kernel<T, D, NW, NS, TN, SPARSE>;
  constexpr size_t lds = prefill_lds_bytes<D, NW, NS, TN>();
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
