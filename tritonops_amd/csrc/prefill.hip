// Prefill (many-query) attention forward for gfx950: dense causal / non-causal
// and block-sparse, packed var-len or batched, GQA.
//
// Work decomposition: one work item = NW wavefronts x 32 consecutive query
// rows of one (sequence, q-head); KV is walked in tiles that the whole
// workgroup brings into an LDS ring with direct-to-LDS loads
// (global_load_lds_dwordx4: no staging registers, no ds_write), one barrier
// per tile.  Dense: 64-key tiles, four stages, a persistent grid that walks the
// items and requests the first tiles of its next item while it writes out the
// current one, and a software pipeline over half tiles inside each wavefront
// (see dense_kernel).  Block-sparse: the same pipeline over 32-key tiles of
// the listed blocks, two stages per tensor, one launch per item.  The sparse
// launcher's two-window form also runs without lists: the 128-row form of the
// dense walk over each item's sink tiles and band (dense_short_kernel, WIN).
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

template <int V>
using ic = std::integral_constant<int, V>;

// vmcnt(N) expcnt(7) lgkmcnt(15) for s_waitcnt on gfx9-family encodings
constexpr int waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

// Where one work item lives: (sequence, heads, q tile), the sequence length and
// the element offsets of the sequence's first token in each tensor.
struct ItemGeo {
  int b, kvh, h, qt, len;
  int64_t q_off, k_off, v_off, o_off, lse_off;
};

// Work item id -> geometry; false when the q tile (BM rows) starts past the end
// of its sequence.  Consecutive ids are dealt round-robin to the 8 XCDs, each
// with a private L2: give every XCD whole (sequence, kv-head) units so their
// K/V stay in one L2, and walk the q tiles of a unit from the longest (last)
// to the shortest.
template <int BM>
__device__ __forceinline__ bool item_geo(const PrefillParams& p, const int bid, ItemGeo& g) {
  const int gqa = p.hq / p.hkv;
  const int per_unit = p.n_qtiles * gqa;
  const int n_units = p.batch * p.hkv;
  int unit, s;
  if ((n_units & 7) == 0) {
    const int xcd = bid & 7, slot = bid >> 3;
    unit = (slot / per_unit) * 8 + xcd;
    s = slot % per_unit;
  } else {
    unit = bid / per_unit;
    s = bid % per_unit;
  }
  g.qt = p.n_qtiles - 1 - s / gqa;
  g.b = unit / p.hkv;
  g.kvh = unit % p.hkv;
  g.h = g.kvh * gqa + s % gqa;
  if (p.cu) {
    const int start = p.cu[g.b];
    // (a sequence longer than the caller's bound is cut at the bound: the grid covers no row beyond it)
    g.len = min(p.cu[g.b + 1] - start, p.max_seqlen);
    g.q_off = start * p.q_ss;
    g.k_off = start * p.k_ss;
    g.v_off = start * p.v_ss;
    g.o_off = start * p.o_ss;
    g.lse_off = start * p.lse_ss;
  } else {
    g.len = p.max_seqlen;
    g.q_off = g.b * p.q_sb;
    g.k_off = g.b * p.k_sb;
    g.v_off = g.b * p.v_sb;
    g.o_off = g.b * p.o_sb;
    g.lse_off = g.b * p.lse_sb;
  }
  return g.qt * BM < g.len;
}

// K and V of one (sequence, kv-head): first token, as pointers and as 64-bit
// values the compiler knows to be wave-uniform, and the sequence length.
template <typename T>
struct KvSrc {
  const T *kp, *vp;
  uint64_t k_base, v_base;
  int len;
};

// Direct-to-LDS loads of KV tiles.  NW wavefronts share a tile of TN keys; the
// ring has NS stages (NS K tiles, then NS V tiles).  Instruction t of a wave
// fills the 1 KiB of LDS that holds tile rows RPI*(wave + NW*t) .. +RPI-1:
// lane i's 16 bytes land in slot i of that KiB, i.e. row drow = i / SLOTS, slot
// dslot = i % SLOTS, which must receive logical chunk dslot ^ swz(row) of that
// row.
template <typename T, int D, int NW, int NS, int TN>
struct TileDma {
  using G = RowGeom<D>;
  using F = SwizzledFrags<D>;
  static constexpr int TILEB = TN * F::ROWB;  // one K or V tile
  static constexpr int VBASE = NS * TILEB;    // first V tile
  static constexpr int RPI = 1024 / F::ROWB;  // tile rows filled by one instruction
  static constexpr int NINST = TN / RPI;      // instructions per tensor per tile
  static constexpr int IPW = NINST / NW;      // ... per wavefront
  static_assert(NINST % NW == 0, "tile rows must split evenly over the waves");

  uint32_t lds0;
  int wave, lane;
  int64_t k_rowb, v_rowb;      // bytes between keys
  uint32_t k_pitch, v_pitch;   // the same, wave-uniform
  uint32_t koff[IPW], voff[IPW];

  static __device__ __forceinline__ uint64_t uniform64(uint64_t x) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)x);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
    return ((uint64_t)hi << 32) | lo;
  }
  // The load is issued from inline assembly on purpose: the compiler then does
  // not know that LDS writes are in flight.  When it knows, it makes every
  // transposing LDS read wait for ALL outstanding loads (vmcnt(0)), the tile
  // requested a moment ago included, which turns the multi-stage pipeline into
  // a synchronous copy.  Completion is tracked by hand instead: a wave's loads
  // retire in order, so "at most n younger loads outstanding" (counted vmcnt
  // waits) followed by the workgroup barrier publishes a tile.  M0 carries the
  // LDS byte address of the 1 KiB slab.
  static __device__ __forceinline__ void dma16(const char* g, uint32_t slab_u) {
    const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(slab_u);  // uniform by construction
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(g), "s"(slab)
                 : "memory");
  }

  // The same with the address as "uniform 64-bit base + 32-bit lane offset"
  // (no vector arithmetic per load).
  static __device__ __forceinline__ void dma16s(uint64_t base, uint32_t off, uint32_t slab_u) {
    const uint32_t slab = (uint32_t)__builtin_amdgcn_readfirstlane(slab_u);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(off), "s"(base), "s"(slab)
                 : "memory");
  }

  // A load of the lanes in `mask`, for straight-line code between MFMAs
  // (all 64 lanes are active and control flow is wave-uniform where it is
  // used, so exec is restored to all ones; a branch around the load would end
  // the basic block and the pinned instruction order with it).
  static __device__ __forceinline__ void dma16m(uint64_t mask, uint64_t base, uint32_t off, uint32_t slab) {
    asm volatile("s_mov_b32 m0, %3\n\ts_mov_b64 exec, %0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, -1"
                 :
                 : "s"(mask), "v"(off), "s"(base), "s"(slab)
                 : "memory");
  }

  // Loads of one whole tile, sent one at a time: arm() fixes the tile
  // (wave-uniform bases), one(k) sends load k of 2*IPW (K and V alternate).
  struct Drip {
    uint64_t on;  // all ones when armed, 0: the loads are no-ops
    uint64_t kt, vt;
    uint32_t sK, sV;
  };
  template <int ST>
  __device__ __forceinline__ Drip arm(const KvSrc<T>& s, int k0, bool on) const {
    Drip d;
    const uint32_t k0u = (uint32_t)__builtin_amdgcn_readfirstlane(k0);
    d.on = uniform64(on ? ~0ull : 0ull);
    d.kt = uniform64(s.k_base + (uint64_t)k0u * k_pitch);
    d.vt = uniform64(s.v_base + (uint64_t)k0u * v_pitch);
    d.sK = lds0 + ST * TILEB;
    d.sV = lds0 + VBASE + ST * TILEB;
    return d;
  }
  // the same for a tile whose loads are all on (no exec mask; not for D = 96,
  // whose rows have dead chunks)
  __device__ __forceinline__ void one_on(const Drip& d, int k) const {
    const int t = k >> 1;
    const int inst = wave + NW * t;
    if (k & 1)
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff[t]), "s"(d.vt), "s"(d.sV + inst * 1024) : "memory");
    else
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(koff[t]), "s"(d.kt), "s"(d.sK + inst * 1024) : "memory");
  }
  // Contiguous rows (pitch = ROWB, e.g. a [B,H,S,D] tensor): the slabs of a
  // tile are then 1 KiB apart in memory exactly as they are in LDS, and a
  // load's immediate offset moves both addresses.  M0 is written once per
  // tensor and tile (pointing kFastMid bytes into the wave's first slab, so
  // that the offsets of all IPW loads fit the signed 13-bit immediate); loads
  // t and t + 2 land 16 rows apart, where the swizzle repeats, and share one
  // lane offset (kfast / vfast).  Load k of 2*IPW: the K loads first, then V.
  static constexpr int kFastMid = NW * 1024 * (IPW - 1) / 2;
  static constexpr bool kFastOk = D == 128 && IPW == 4 && NW == 2;
  uint32_t kfast[2], vfast[2];
  template <int K>
  __device__ __forceinline__ void one_fast(const Drip& d) const {
    constexpr int t = K % IPW;
    constexpr int imm = NW * 1024 * t - kFastMid;
    static_assert(imm >= -4096 && imm <= 4095, "immediate offset of a global load");
    if constexpr (K < IPW) {
      if constexpr (t == 0)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3" : : "v"(kfast[t & 1]), "s"(d.kt), "s"(d.sK + wave * 1024 + kFastMid), "n"(imm) : "memory");
      else
        asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(kfast[t & 1]), "s"(d.kt), "n"(imm) : "memory");
    } else {
      if constexpr (t == 0)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3" : : "v"(vfast[t & 1]), "s"(d.vt), "s"(d.sV + wave * 1024 + kFastMid), "n"(imm) : "memory");
      else
        asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(vfast[t & 1]), "s"(d.vt), "n"(imm) : "memory");
    }
  }
  __device__ __forceinline__ void one(const Drip& d, int k) const {
    const int t = k >> 1;
    const int inst = wave + NW * t;
    uint64_t mask = d.on;
    if (D == 96) {
      int ln = lane;
      const int drow = ln / F::SLOTS, dslot = ln % F::SLOTS;
      const int r = RPI * inst + drow;
      const int c = dslot ^ ((k & 1) ? F::swz_v(r) : F::swz_k(r));
      mask = uniform64(mask & __builtin_amdgcn_ballot_w64(c < G::NCH));
    }
    if (k & 1)
      dma16m(mask, d.vt, voff[t], d.sV + inst * 1024);
    else
      dma16m(mask, d.kt, koff[t], d.sK + inst * 1024);
  }

  __device__ __forceinline__ void init(const PrefillParams& p, int lane_, int wave_) {
    lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem);
    wave = wave_;
    lane = lane_;
    const int drow = lane / F::SLOTS, dslot = lane % F::SLOTS;
    k_rowb = p.k_ss * 2;
    v_rowb = p.v_ss * 2;
    k_pitch = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)k_rowb);
    v_pitch = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)v_rowb);
    // A tile load address is (uniform tensor base + uniform tile offset), both
    // kept in scalar registers, plus a per-lane 32-bit offset that is fixed for
    // the whole launch: two vector instructions per load instead of a 64-bit
    // multiply-add chain.
#pragma unroll
    for (int t = 0; t < IPW; ++t) {
      const int r = RPI * (wave + NW * t) + drow;
      koff[t] = (uint32_t)r * k_pitch + (uint32_t)(dslot ^ F::swz_k(r)) * 16u;
      voff[t] = (uint32_t)r * v_pitch + (uint32_t)(dslot ^ F::swz_v(r)) * 16u;
    }
    if constexpr (kFastOk) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        kfast[t] = koff[t] + (uint32_t)(kFastMid - NW * 1024 * t);
        vfast[t] = voff[t] + (uint32_t)(kFastMid - NW * 1024 * t);
      }
    }
  }
  // do the rows of K and of V follow one another without a gap?
  __device__ __forceinline__ bool rows_contiguous() const { return k_pitch == F::ROWB && v_pitch == F::ROWB; }

  static __device__ __forceinline__ KvSrc<T> source(const T* kp, const T* vp, int len) {
    KvSrc<T> s;
    s.kp = kp;
    s.vp = vp;
    s.k_base = uniform64((uint64_t)(uintptr_t)kp);
    s.v_base = uniform64((uint64_t)(uintptr_t)vp);
    s.len = len;
    return s;
  }

  // keys k0 .. k0+TN-1 of K (or of V) into stage ST, rows past the sequence
  // end re-reading its last row
  template <int ST, bool IS_V>
  __device__ __forceinline__ void tensor_tile(const KvSrc<T>& s, int k0) const {
    const uint32_t sB = lds0 + (IS_V ? VBASE : 0) + ST * TILEB;
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int drow = ln / F::SLOTS, dslot = ln % F::SLOTS;
    const int64_t rowb = IS_V ? v_rowb : k_rowb;
    const char* bt = reinterpret_cast<const char*>(IS_V ? s.vp : s.kp) + k0 * rowb;
#pragma unroll
    for (int t = 0; t < IPW; ++t) {
      const int inst = wave + NW * t;
      const int r = RPI * inst + drow;
      const int c = dslot ^ (IS_V ? F::swz_v(r) : F::swz_k(r));
      const int64_t rr = min(k0 + r, s.len - 1) - k0;
      if (D != 96 || c < G::NCH) dma16(bt + rr * rowb + c * 16, sB + inst * 1024);
    }
  }

  // keys k0 .. k0+TN-1 of `s` into stage ST
  template <int ST>
  __device__ __forceinline__ void tile(const KvSrc<T>& s, int k0) const {
    const uint32_t sK = lds0 + ST * TILEB;
    const uint32_t sV = lds0 + VBASE + ST * TILEB;
    // (lane coordinates from an opaque copy: nothing derived from them is
    // worth a register across the tile loop)
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int drow = ln / F::SLOTS, dslot = ln % F::SLOTS;
    if (k0 + TN <= s.len) {
      // whole tile inside the sequence
      const uint32_t k0u = (uint32_t)__builtin_amdgcn_readfirstlane(k0);
      // (scalar base + lane offset pays in the dense kernels; the block-sparse one,
      // whose base changes with every listed block, measured faster with the sum in vector registers)
      constexpr bool kScalarBase = NW >= 4;
      const uint64_t kt_u = s.k_base + (uint64_t)k0u * k_pitch, vt_u = s.v_base + (uint64_t)k0u * v_pitch;
      const uint64_t kt_s = kScalarBase ? uniform64(kt_u) : 0, vt_s = kScalarBase ? uniform64(vt_u) : 0;
#pragma unroll
      for (int t = 0; t < IPW; ++t) {
        const int inst = wave + NW * t;
        const int r = RPI * inst + drow;
        const int kc = dslot ^ F::swz_k(r), vc = dslot ^ F::swz_v(r);
        if (kScalarBase) {
          if (D != 96 || kc < G::NCH) dma16s(kt_s, koff[t], sK + inst * 1024);
          if (D != 96 || vc < G::NCH) dma16s(vt_s, voff[t], sV + inst * 1024);
        } else {
          if (D != 96 || kc < G::NCH) dma16(reinterpret_cast<const char*>(kt_u + koff[t]), sK + inst * 1024);
          if (D != 96 || vc < G::NCH) dma16(reinterpret_cast<const char*>(vt_u + voff[t]), sV + inst * 1024);
        }
      }
    } else {
      // rows past the sequence end re-read its last row (masked later)
      const char* kt = reinterpret_cast<const char*>(s.kp) + k0 * k_rowb;
      const char* vt = reinterpret_cast<const char*>(s.vp) + k0 * v_rowb;
#pragma unroll
      for (int t = 0; t < IPW; ++t) {
        const int inst = wave + NW * t;
        const int r = RPI * inst + drow;
        const int kc = dslot ^ F::swz_k(r), vc = dslot ^ F::swz_v(r);
        const int64_t rr = min(k0 + r, s.len - 1) - k0;
        if (D != 96 || kc < G::NCH) dma16(kt + rr * k_rowb + kc * 16, sK + inst * 1024);
        if (D != 96 || vc < G::NCH) dma16(vt + rr * v_rowb + vc * 16, sV + inst * 1024);
      }
    }
  }
};

// ---------------------------------------------------------------------------
// Block-sparse: one workgroup of two wavefronts per 64-row block row, four
// workgroups per CU, the dense kernel's software pipeline (see dense_kernel
// below) over the 32-key tiles of the listed blocks.  At position h a wave runs
//   block A: [MFMAs of S(h+1) = K(h+1) Q^T]  with [exp2 / sum / pack of the last 8 keys of S(h)]
//                                             and the loads of K(h+2) and V(h+1), one per MFMA
//   check  : row sums sane? else exact_fix (rare); mask S(h+1) if its tile needs one
//   block B: [MFMAs of O += V(h)^T P(h)^T]   with [exp2 / sum / pack of the first 8 keys of S(h+1)]
// K tiles live one position ahead of V tiles, so each tensor has a ring of its
// own two stages: K(h+2) replaces K(h), which was scored in position h-1, and
// V(h+1) replaces V(h-1).  One wait and one barrier per position publish both.
// The loads sit in block A, whose MFMAs form one serial chain and leave the
// wave time to queue them; behind the four independent chains of block B they
// measured 6 % slower.  Probabilities are taken against the reference point
// the row already has (no row maximum in the common path, as in the dense
// kernel); a row that has not met a visible key yet takes the exact path.
// The block list is kept in registers, 64 entries at a time (lane l holds
// entry 64 * chunk + l; the chunk being walked and the one behind it), and
// read with v_readlane: a memory load inside the tile loop would have to be
// waited for with vmcnt(0), which also drains the tiles requested a moment
// ago.  A block's two tiles share one list lookup and one address product.
// When every listed block ends inside the sequence (the usual case: lengths
// that are multiples of the block size) the walk runs in a copy of the loop
// whose loads carry no exec mask and that has no path for clamped tiles.
template <typename T, int D>
__global__ void __launch_bounds__(kSparseRows * 2) __attribute__((amdgpu_waves_per_eu(D == 64 ? 3 : 2)))
sparse_kernel(const PrefillParams p) {
  constexpr int NW = kSparseRows / 32, NS = kSparseStages, TN = kSparseTileKeys;
  static_assert(NW == 2 && NS == 2 && TN == 32 && kTileN == 64, "a listed block is two tiles; two stages per tensor");
  using G = RowGeom<D>;
  using F = SwizzledFrags<D>;
  using DMA = TileDma<T, D, NW, NS, TN>;
  constexpr int BM = 32 * NW;
  constexpr int TILEB = DMA::TILEB, VBASE = DMA::VBASE, IPW = DMA::IPW;
  constexpr int OROWB = D * 2 + 16;  // epilogue staging row

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  ItemGeo g;
  if (!item_geo<BM>(p, blockIdx.x, g)) return;
  const int len = g.len, qt = g.qt, hd = g.h;
  const int q0 = qt * BM;
  const T* qp = reinterpret_cast<const T*>(p.q) + g.q_off + hd * p.q_sh;
  T* op = reinterpret_cast<T*>(p.o) + g.o_off + hd * p.o_sh;

  F fr;
  fr.init(lane, (uint32_t)(uintptr_t)smem, VBASE);
  DMA dma;
  dma.init(p, lane, wave);
  const KvSrc<T> kv = DMA::source(reinterpret_cast<const T*>(p.k) + g.k_off + g.kvh * p.k_sh,
                                  reinterpret_cast<const T*>(p.v) + g.v_off + g.kvh * p.v_sh, len);
  const int q0w = q0 + 32 * wave;
  const int qrow = q0w + fr.lq;

  // ---- tile list: 64 entries at a time in registers
  const int32_t* rp = p.row_ptr + g.b * p.rp_sb + hd * p.rp_sh;
  const int beg = __builtin_amdgcn_readfirstlane(rp[qt]);
  const int n_blk = __builtin_amdgcn_readfirstlane(rp[qt + 1] - beg);
  const int n_tiles = n_blk * 2;
  const int32_t* cols = p.col_idx + g.b * p.ci_sb + hd * p.ci_sh + beg;
  auto load_cols = [&](int chunk) __attribute__((always_inline)) -> int {
    const int idx = chunk * 64 + lane;
    return idx < n_blk ? cols[idx] : 0;
  };
  int col_chunk = 0;
  int col_cur = load_cols(0), col_nxt = load_cols(1);
  // does every listed block end inside the sequence?  (A list may name blocks
  // past the end of a short sequence: their rows are clamped and masked.)
  bool all_inside;
  {
    int mx = max(col_cur, col_nxt);
    for (int c = 2; c * 64 < n_blk; ++c) mx = max(mx, load_cols(c));
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mx = max(mx, __shfl_xor(mx, off));
    all_inside = (__builtin_amdgcn_readfirstlane(mx) + 1) * kTileN <= len;
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
  float m = -INFINITY, m_neg = 0.f, l = 0.f;
  const float scale = p.scale;
  const int causal = p.causal;
  const int wl = p.win_local, wg = p.win_global;

  // keys of the tile at k0 that this lane's query must not see -> -inf.
  // Register r of a score block is key k0 + 8 lh + e(r), e(r) = 16 (r / 8) + r % 8:
  // every test is "e(r) against a per-lane bound", branch-free.
  const int lim_row = min(len - 1, causal ? qrow : 0x3fffffff) - 8 * fr.lh;  // largest visible key, less the lane's offset
  auto mask_tile = [&](int k0, f32x16& Sx) __attribute__((always_inline)) {
    bool need = (k0 + TN > len) || (causal && k0 + TN - 1 > q0w);
    if (wl >= 0) need = need || !((k0 + TN - 1 < wg) || (q0w + 31 - k0 < wl));
    if (need) {
      const int hi = lim_row - k0;                    // e(r) <= hi
      const int lo = qrow - wl - 8 * fr.lh - k0;      // window: e(r) > lo ...
      const int gl = wg - 8 * fr.lh - k0;             // ... or e(r) < gl
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int e = 16 * (r >> 3) + (r & 7);
        bool ok = e <= hi;
        if (wl >= 0) ok = ok & ((e > lo) | (e < gl));
        Sx[r] = ok ? Sx[r] : -INFINITY;
      }
    }
  };

  constexpr float kRowSumLimit = 4096.f;
  f32x16 S[2];
  uint32_t Pb[2][8];
  float rsv[2];
  float e_p0, e_u1;
  auto exp_first = [&](const f32x16& Sx, int i) __attribute__((always_inline)) {
    e_p0 = fast_exp2(fmaf(Sx[2 * i], scale, m_neg));
    e_u1 = fmaf(Sx[2 * i + 1], scale, m_neg);
  };
  auto exp_second = [&](int i, uint32_t (&Pd)[8], float& rs) __attribute__((always_inline)) {
    const float p1 = fast_exp2(e_u1);
    rs = i == 0 ? e_p0 + p1 : rs + (e_p0 + p1);
    Pd[i] = Elem<T>::pack2(e_p0, p1);
  };
  // rare: bring m to the exact running maximum including the tile in Sx,
  // rescale l and O, and redo the probabilities of that tile
  auto exact_fix = [&](const f32x16& Sx, uint32_t (&Pd)[8], float& rs) __attribute__((always_inline)) {
    float mx = Sx[0];
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(mx, Sx[r]);
    mx = max_with_other_half(mx);
    const float m_new = fmaxf(m, mx * scale);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fast_exp2(m - m_safe);
    l *= alpha;
#pragma unroll
    for (int db = 0; db < G::NDB; ++db) O[db] *= alpha;
    m = m_new;
    m_neg = -m_safe;
    rs = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float p0 = fast_exp2(fmaf(Sx[2 * i], scale, -m_safe));
      const float p1 = fast_exp2(fmaf(Sx[2 * i + 1], scale, -m_safe));
      rs += p0 + p1;
      Pd[i] = Elem<T>::pack2(p0, p1);
    }
  };

  // K fragments kept in flight ahead of their MFMA.  At head_dim 64 two instead of four bring a wave to 168 registers,
  // so that three waves fit a SIMD (six workgroups per CU): 5 to 9 % faster on the benchmark's mask at that head_dim
  constexpr int KR = D == 64 ? 2 : (G::KSTEPS < 4 ? G::KSTEPS : 4);
  // first key and tile addresses of the listed blocks being walked (wave-uniform)
  int c0C = 0, c0N = 0;
  uint64_t bvC = 0, bkN = 0, bvN = 0;
  bool hasN = false;
  auto position = [&](auto j_c, auto last_c, auto steady_c, int h) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value;  // h % 2
    // both requested tiles exist and lie inside the sequence: loads without a mask;
    // level 2: rows are contiguous as well, M0 is written once per tensor (TileDma::one_fast)
    constexpr bool STEADY = decltype(steady_c)::value != 0 && D != 96;
    constexpr bool FAST = decltype(steady_c)::value == 2 && DMA::kFastOk;
    constexpr bool LAST = decltype(last_c)::value != 0;  // no tile h+1: only the second half of block A's arithmetic and block B's MFMAs
    constexpr uint32_t KOFF = (J ^ 1) * TILEB, VOFF = J * TILEB;  // K of tile h+1, V of tile h
    f32x16& Sc = S[J];
    f32x16& Sn = S[J ^ 1];
    uint32_t (&Pc)[8] = Pb[J];
    uint32_t (&Pn)[8] = Pb[J ^ 1];
    // Tiles 2q and 2q+1 are the halves of listed block q.  An even position
    // (h = 2q) looks up block q+1 ("N"); block q ("C") was looked up two
    // positions ago.  Requests: even h: K of N's first half, V of C's second
    // half; odd h: K of N's second half, V of N's first half.
    if constexpr (J == 0) {
      const int bn = (h >> 1) + 1;
      hasN = bn < n_blk;
      if (hasN) {
        if ((bn >> 6) != col_chunk) {  // walked into the next 64 entries of the list
          ++col_chunk;
          col_cur = col_nxt;
          col_nxt = load_cols(col_chunk + 1);
        }
        c0N = __builtin_amdgcn_readlane(col_cur, bn & 63) * kTileN;
        bkN = kv.k_base + (uint64_t)(uint32_t)c0N * dma.k_pitch;
        bvN = kv.v_base + (uint64_t)(uint32_t)c0N * dma.v_pitch;
      }
    }
    const bool has1 = J == 0 ? true : hasN, has2 = hasN;
    const int k0n = J == 0 ? c0C + TN : c0N;  // the tile scored here, whose V is requested here
    const int k0r = J == 0 ? c0N : c0N + TN;  // the tile whose K is requested here
    typename DMA::Drip dK, dV;
    dK.on = dV.on = ~0ull;
    if constexpr (!STEADY) {
      // a tile that reaches past the sequence end at once (clamped rows), a
      // whole tile one load at a time behind the MFMAs below
      const bool kwhole = k0r + TN <= len, vwhole = k0n + TN <= len;
      if (!LAST) {
        if (has2 && !kwhole) dma.template tensor_tile<J, false>(kv, k0r);
        if (has1 && !vwhole) dma.template tensor_tile<J ^ 1, true>(kv, k0n);
      }
      dK.on = DMA::uniform64((has2 && kwhole) ? ~0ull : 0ull);
      dV.on = DMA::uniform64((has1 && vwhole) ? ~0ull : 0ull);
    }
    dK.kt = J == 0 ? bkN : bkN + (uint64_t)(TN * dma.k_pitch);
    dK.sK = dma.lds0 + J * TILEB;
    dV.vt = J == 0 ? bvC + (uint64_t)(TN * dma.v_pitch) : bvN;
    dV.sV = dma.lds0 + VBASE + (J ^ 1) * TILEB;
    dK.vt = 0; dK.sV = 0; dV.kt = 0; dV.sK = 0;

    i32x4 kf[KR], vf[G::NDB];
    __builtin_amdgcn_s_setprio(3);
    if (!LAST) {
#pragma unroll
      for (int c = 0; c < KR; ++c) kf[c] = fr.load_k(KOFF, 0, c);
    }
    // the K fragments were requested a moment ago (their tile was published by
    // the barrier just passed): the first pair of exponentials goes in front of
    // the first MFMA, and the last two MFMAs have no arithmetic behind them
    exp_first(Sc, 4);
    exp_second(4, Pc, rsv[J]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      if (c < G::KSTEPS && !LAST) {
        const f32x16 acc = (c == 0) ? (f32x16){0} : Sn;
        Sn = Elem<T>::mfma(kf[c % KR], Qf[c], acc);
        if (c + KR < G::KSTEPS) kf[c % KR] = fr.load_k(KOFF, 0, c + KR);
      }
      if (c >= 8 - G::NDB) vf[c - (8 - G::NDB)] = fr.load_v(VOFF, 0, c - (8 - G::NDB));
      if (!LAST) {
        if constexpr (FAST) {
          static_assert(2 * IPW == 8, "one load per MFMA slice");
          if (c == 0) dma.template one_fast<0>(dK);
          if (c == 1) dma.template one_fast<1>(dK);
          if (c == 2) dma.template one_fast<2>(dK);
          if (c == 3) dma.template one_fast<3>(dK);
          if (c == 4) dma.template one_fast<4>(dV);
          if (c == 5) dma.template one_fast<5>(dV);
          if (c == 6) dma.template one_fast<6>(dV);
          if (c == 7) dma.template one_fast<7>(dV);
        } else {
#pragma unroll
          for (int k = c * 2 * IPW / 8; k < (c + 1) * 2 * IPW / 8; ++k) {
            if constexpr (STEADY)
              dma.one_on((k & 1) ? dV : dK, k);
            else
              dma.one((k & 1) ? dV : dK, k);
          }
        }
      }
      if (c < 6) {
        if ((c & 1) == 0)
          exp_first(Sc, 5 + c / 2);
        else
          exp_second(5 + c / 2, Pc, rsv[J]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("" : "+v"(Pc[4]), "+v"(Pc[5]), "+v"(Pc[6]), "+v"(Pc[7]), "+v"(rsv[J]));
    // a row that has not met a visible key yet has no reference point: exact path
    if (__builtin_amdgcn_ballot_w64(!(rsv[J] <= kRowSumLimit) || m == -INFINITY) != 0) exact_fix(Sc, Pc, rsv[J]);
    l += rsv[J];
    if (!LAST) mask_tile(k0n, Sn);
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int sl = 0; sl < 8; ++sl) {
      if (sl < 2 * G::NDB) {
        const int kk = sl / G::NDB, db = sl % G::NDB;
        const i32x4 pf = {(int)Pc[4 * kk], (int)Pc[4 * kk + 1], (int)Pc[4 * kk + 2], (int)Pc[4 * kk + 3]};
        O[db] = Elem<T>::mfma(vf[db], pf, O[db]);
        if (kk == 0) vf[db] = fr.load_v(VOFF, 1, db);
      }
      if (!LAST) {
        if ((sl & 1) == 0)
          exp_first(Sn, sl / 2);
        else
          exp_second(sl / 2, Pn, rsv[J ^ 1]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (!LAST) {
      asm volatile("" : "+v"(Pn[0]), "+v"(Pn[1]), "+v"(Pn[2]), "+v"(Pn[3]), "+v"(rsv[J ^ 1]));
      // K(h+2) and V(h+1) must have landed and everyone must be done with K(h+1) and V(h)
      if constexpr (J == 1) {
        c0C = c0N;
        bvC = bvN;
      }
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
      __syncthreads();
    }
  };

  if (n_tiles > 0) {
    c0C = __builtin_amdgcn_readlane(col_cur, 0) * kTileN;
    bvC = kv.v_base + (uint64_t)(uint32_t)c0C * dma.v_pitch;
    dma.template tile<0>(kv, c0C);
    dma.template tensor_tile<1, false>(kv, c0C + TN);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __syncthreads();
    {
      // scores of tile 0, its exact row maximum as the first reference point,
      // the probabilities of its first 8 keys
      f32x16 acc = (f32x16){0};
#pragma unroll
      for (int c = 0; c < G::KSTEPS; ++c) acc = Elem<T>::mfma(fr.load_k(0u, 0, c), Qf[c], acc);
      S[0] = acc;
      mask_tile(c0C, S[0]);
      exact_fix(S[0], Pb[0], rsv[0]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        exp_first(S[0], i);
        exp_second(i, Pb[0], rsv[0]);
      }
    }
    __syncthreads();  // position 0 requests K(2) into the stage of K(0), which the other wave may still be reading
    int h = 0;
    if (all_inside && DMA::kFastOk && dma.rows_contiguous()) {
      // ... and the rows of K and V are contiguous: one M0 write per tensor and tile
      for (; h + 2 < n_tiles; h += 2) {
        position(ic<0>{}, ic<0>{}, ic<2>{}, h);
        position(ic<1>{}, ic<0>{}, ic<2>{}, h + 1);
      }
    } else if (all_inside) {
      // every listed block lies inside the sequence: the loop whose loads carry no mask
      for (; h + 2 < n_tiles; h += 2) {
        position(ic<0>{}, ic<0>{}, ic<1>{}, h);
        position(ic<1>{}, ic<0>{}, ic<1>{}, h + 1);
      }
    } else {
      for (; h + 2 < n_tiles; h += 2) {
        position(ic<0>{}, ic<0>{}, ic<0>{}, h);
        position(ic<1>{}, ic<0>{}, ic<0>{}, h + 1);
      }
    }
    position(ic<0>{}, ic<0>{}, ic<0>{}, h);
    position(ic<1>{}, ic<1>{}, ic<0>{}, h + 1);
    __builtin_amdgcn_s_setprio(0);
    __syncthreads();  // every wave is done with the tiles: the staging below reuses them
  }

  // ---- epilogue: normalise, transpose through LDS, coalesced 16-byte stores
  const float l_tot = sum_with_other_half(l);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (p.lse && fr.lh == 0 && qrow < len) {
    float* lp = p.lse + g.lse_off + hd * p.lse_sh;
    lp[(int64_t)qrow * p.lse_ss] = l_tot > 0.f ? m + fast_log2(l_tot) : -INFINITY;
  }
  unsigned char* stage = smem + wave * 32 * OROWB;
#pragma unroll
  for (int db = 0; db < G::NDB; ++db)
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const int d = 32 * db + 8 * gq + 4 * fr.lh;
      i32x2 w;
      w[0] = (int)Elem<T>::pack2(O[db][4 * gq] * inv, O[db][4 * gq + 1] * inv);
      w[1] = (int)Elem<T>::pack2(O[db][4 * gq + 2] * inv, O[db][4 * gq + 3] * inv);
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

// ---------------------------------------------------------------------------
// Dense: persistent workgroups of 8 wavefronts (256 query rows per item).
//
// The grid holds at most as many workgroups as the device runs at once, and
// each walks the work item ids id, id + grid, ...: a fresh workgroup launch
// left the CU idle for several microseconds (measured ~12 us between the end
// of one 512-thread, 128 KiB-LDS workgroup and the first instruction of the
// next).  Odd rounds are walked back to front within each XCD (id & 7 is
// kept): ids run from the longest q tile of a unit to the shortest, so the
// workgroup that drew a long tile in one round draws a short one in the next,
// which balances causal work without a shared counter.
//
// Item boundary: once every wave is done with the tiles of an item, the
// workgroup requests Q and the first NS-1 tiles of its NEXT item (stages
// 0..NS-2) while it normalises and writes out the current one, staging the
// output through the last stage: Q and tile 0 go out first, tiles 1 and 2
// after the first and the second pass of output stores, so the requests queue
// in the vector-memory pipeline while the waves do the arithmetic of the
// write-out instead of in front of it; one barrier separates the two items.
//
// Inner loop: a software pipeline over HALF tiles (32 keys) inside each wave.
// MFMA and softmax arithmetic overlap best when one wave's instruction stream
// interleaves them, so at position h the wave runs two straight-line blocks:
// the 8 MFMAs of S[h+1] = K Q^T together with half of the exp2 / sum / convert
// work of S[h], then the 8 MFMAs of O += V^T P[h]^T together with the first
// half of that work for S[h+1].  K of half h+1 must be in LDS while half h is
// being finished: tile t+1 has to be visible before position 2t+1, which the
// barrier at the top of tile t guarantees.
template <typename T, int D>
__global__ void __launch_bounds__(kDenseRows * 2) __attribute__((amdgpu_waves_per_eu(2)))
dense_kernel(const PrefillParams p) {
  constexpr int NW = kDenseRows / 32, NS = kDenseStages, TN = kTileN;
  static_assert(NW == 8 && NS == 4 && TN == 64, "stage use at the item boundary assumes this shape");
  using G = RowGeom<D>;
  using F = SwizzledFrags<D>;
  using DMA = TileDma<T, D, NW, NS, TN>;
  constexpr int BM = 32 * NW;
  constexpr int TILEB = DMA::TILEB, VBASE = DMA::VBASE, IPW = DMA::IPW;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // 32-row block of the item that this wave owns.  Waves w and w + 4 share a
  // SIMD; in the diagonal block of a causal item row block r has r + 1 halves
  // to do, so pairing blocks (r, 7 - r) gives every SIMD the same nine.
  const int rblk = wave < 4 ? wave : 11 - wave;
  F fr;
  fr.init(lane, (uint32_t)(uintptr_t)smem, VBASE);
  DMA dma;
  dma.init(p, lane, wave);
  const int causal = p.causal;
  const float scale = p.scale;

  // ---- the items of this workgroup
  struct Item {
    int len, q0, n_tiles;
    const T* qp;
    T* op;
    float* lp;  // LSE row of this head, or null
    KvSrc<T> kv;
  };
  const int grid = gridDim.x;
  int round = 0, base = 0;
  // advance to the next item of this workgroup that has rows; false when there is none
  auto next_item = [&](Item& it) __attribute__((always_inline)) -> bool {
    while (base < p.n_items) {
      int w = blockIdx.x;
      if ((round & 1) && (grid & 7) == 0) w = (((grid >> 3) - 1 - (w >> 3)) << 3) | (w & 7);
      const int bid = base + w;
      base += grid;
      ++round;
      ItemGeo g;
      if (bid < p.n_items && item_geo<BM>(p, bid, g)) {
        it.len = g.len;
        it.q0 = g.qt * BM;
        it.n_tiles = (g.len + TN - 1) / TN;
        if (causal) it.n_tiles = min(it.n_tiles, (it.q0 + BM + TN - 1) / TN);
        it.qp = reinterpret_cast<const T*>(p.q) + g.q_off + g.h * p.q_sh;
        it.op = reinterpret_cast<T*>(p.o) + g.o_off + g.h * p.o_sh;
        it.lp = p.lse ? p.lse + g.lse_off + g.h * p.lse_sh : nullptr;
        it.kv = DMA::source(reinterpret_cast<const T*>(p.k) + g.k_off + g.kvh * p.k_sh,
                            reinterpret_cast<const T*>(p.v) + g.v_off + g.kvh * p.v_sh, g.len);
        return true;
      }
    }
    return false;
  };
  // Q^T operands of an item (lane (query lq, half lh) holds d = 16c + 8lh .. +7)
  // and its first tile (tiles 1 and 2 follow from request_tile1 / 2); nothing waits here
  auto request_item = [&](const Item& it, i32x4 (&Q)[G::KSTEPS]) __attribute__((always_inline)) {
    const int row = min(it.q0 + 32 * rblk + fr.lq, it.len - 1);
    const T* qr = it.qp + (int64_t)row * p.q_ss + 8 * fr.lh;
    // Issued from inline assembly like the tile loads, and for the same reason:
    // a load the compiler knows about is guarded by a counted wait at its first
    // use, and that wait would also cover the output stores issued after it.
    // The registers are complete after the wait at the top of the item.
#pragma unroll
    for (int c = 0; c < G::KSTEPS; ++c)
      asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "=v"(Q[c]) : "v"(qr), "n"(32 * c));
    if (0 < it.n_tiles) dma.template tile<0>(it.kv, 0);
  };
  auto request_tile1 = [&](const Item& it) __attribute__((always_inline)) {
    if (1 < it.n_tiles) dma.template tile<1>(it.kv, TN);
  };
  auto request_tile2 = [&](const Item& it) __attribute__((always_inline)) {
    if (2 < it.n_tiles) dma.template tile<2>(it.kv, 2 * TN);
  };

  // ---- state of the item being computed
  Item cur;
  i32x4 Qf[G::KSTEPS];
  f32x16 O[G::NDB];
  float m, l;
  float m_neg;  // -m, or 0 while m is still -inf: the addend of every exponent (changes only in exact_fix)
  int len, n_tiles, q0w, qrow, row_lim, H_w;
  int tail_t;  // first tile (> 0) at whose top no further tile is requested
  f32x16 S[2];
  constexpr int KR = G::KSTEPS < 4 ? G::KSTEPS : 4;  // K fragments kept in flight
  i32x4 kf[KR];  // fragments 0..KR-1 of the half that is scored next, read one block ahead

  // keys of half hh that this lane's query must not see -> -inf (rare)
  auto mask_half = [&](int hh, f32x16& Sx) __attribute__((always_inline)) {
    const int k0h = hh * 32;
    if ((k0h + 32 > len) || (causal && k0h + 31 > q0w)) {
      const int t = row_lim - k0h - 8 * fr.lh;
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (16 * (r >> 3) + (r & 7) > t) Sx[r] = -INFINITY;
    }
  };

  // Probabilities of a half are taken against the reference point m the row
  // already has; m is only moved (exactly, to the true running maximum) when
  // a lane's partial row sum of a half passes kRowSumLimit or is not finite.
  // Any reference point gives the same o and lse, so the common path needs
  // no row maximum at all: 7 vector instructions per pair of scores.
  constexpr float kRowSumLimit = 4096.f;  // probabilities stay below 2^12: far inside bf16 / fp32 range
  uint32_t Pb[2][8];  // packed probabilities of the half in S[0] / S[1]
  float rsv[2];       // their partial row sums (this lane's 16 keys)
  float e_p0, e_u1;   // first element done, second element scaled: carried between two slices
  auto exp_first = [&](const f32x16& Sx, int i, float m_neg) __attribute__((always_inline)) {
    e_p0 = fast_exp2(fmaf(Sx[2 * i], scale, m_neg));
    e_u1 = fmaf(Sx[2 * i + 1], scale, m_neg);
  };
  auto exp_second = [&](int i, uint32_t (&Pd)[8], float& rs) __attribute__((always_inline)) {
    const float p1 = fast_exp2(e_u1);
    rs = i == 0 ? e_p0 + p1 : rs + (e_p0 + p1);  // pair 0 opens the row sum of its half
    Pd[i] = Elem<T>::pack2(e_p0, p1);
  };
  // The same work for four pairs (i0 .. i0 + 3) spread over the eight slices of
  // a block as a pipeline in which no instruction uses the result of its
  // predecessor: the scaled exponents of a pair are formed a slice before its
  // exponentials, and its sum and packed pair a slice after them.
  float su0[2], su1[2], sp0[2], sp1[2], st;
  auto soft_slice = [&](int c, const f32x16& Sx, int i0, uint32_t (&Pd)[8], float& rs, float mn) __attribute__((always_inline)) {
    const int j = (c + 1) / 2;      // pair whose exponents are formed in an odd slice / whose first exponential runs in an even one
    if (c == 0) {
      su0[0] = fmaf(Sx[2 * i0], scale, mn);
      su1[0] = fmaf(Sx[2 * i0 + 1], scale, mn);
      sp0[0] = fast_exp2(su0[0]);
      return;
    }
    if (c & 1) {
      // odd slice: second exponential of pair (c - 1) / 2, row sum of the pair before it, exponents of the next pair
      const int k = (c - 1) / 2, sl = k & 1;
      sp1[sl] = fast_exp2(su1[sl]);
      if (k > 0) rs = (i0 == 0 && k == 1) ? st : rs + st;
      if (k < 3) {
        su0[sl ^ 1] = fmaf(Sx[2 * (i0 + k + 1)], scale, mn);
        su1[sl ^ 1] = fmaf(Sx[2 * (i0 + k + 1) + 1], scale, mn);
      } else {
        const float t2 = sp0[sl] + sp1[sl];
        Pd[i0 + 3] = Elem<T>::pack2(sp0[sl], sp1[sl]);
        rs += t2;
      }
    } else {
      // even slice c = 2 j: first exponential of pair j, sum and packed pair of pair j - 1
      const int sl = j & 1;
      sp0[sl] = fast_exp2(su0[sl]);
      st = sp0[sl ^ 1] + sp1[sl ^ 1];
      Pd[i0 + j - 1] = Elem<T>::pack2(sp0[sl ^ 1], sp1[sl ^ 1]);
    }
  };
  // rare: bring m to the exact running maximum including the half in Sx,
  // rescale l and O, and redo the probabilities of that half
  auto exact_fix = [&](const f32x16& Sx, uint32_t (&Pd)[8], float& rs) __attribute__((always_inline)) {
    float mx = Sx[0];
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(mx, Sx[r]);
    mx = max_with_other_half(mx);
    const float m_new = fmaxf(m, mx * scale);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;  // no key seen yet: l and O are 0
    const float alpha = fast_exp2(m - m_safe);
    l *= alpha;
#pragma unroll
    for (int db = 0; db < G::NDB; ++db) O[db] *= alpha;
    m = m_new;
    m_neg = -m_safe;
    rs = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float p0 = fast_exp2(fmaf(Sx[2 * i], scale, -m_safe));
      const float p1 = fast_exp2(fmaf(Sx[2 * i + 1], scale, -m_safe));
      rs += p0 + p1;
      Pd[i] = Elem<T>::pack2(p0, p1);
    }
  };

  // Position h.  Entry state: S[h&1] holds the scores of half h and the
  // probabilities of its first 8 keys per lane are done; kf holds the first
  // K fragments of half h+1.
  //   block A: [MFMAs of S(h+1) = K Q^T]      with [exp2 / sum / pack of the last 8 keys of S(h)]
  //   check  : row sums sane? else exact_fix (rare)
  //   block B: [MFMAs of O += V^T P(h)^T]    with [exp2 / sum / pack of the first 8 keys of S(h+1)]
  // so every MFMA has three or four vector instructions behind it.
  // sched_barrier(0) after each slice pins the interleaving: one MFMA, the
  // LDS reads for a slice four positions ahead, and those vector instructions.
  auto half_step = [&](auto j_c, int h) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value;  // h % (2 NS)
    if (h >= H_w) return;
    constexpr int TS = J / 2, KB = J & 1;    // stage of tile h/2, which half of it
    constexpr int KS = KB == 0 ? TS : (TS + 1) % NS;      // stage holding K of half h+1
    constexpr uint32_t KOFF = KS * TILEB, VOFF = TS * TILEB;
    constexpr uint32_t K2OFF = ((TS + 1) % NS) * TILEB;   // stage holding K of half h+2
    f32x16& Sc = S[KB];
    f32x16& Sn = S[KB ^ 1];
    uint32_t (&Pc)[8] = Pb[KB];
    uint32_t (&Pn)[8] = Pb[KB ^ 1];
    // Block A carries the serial chain of the eight S MFMAs: a raised issue
    // priority while a wave is in it (and a lower one in block B, whose MFMAs
    // form four independent chains) lets the two waves of a SIMD fall out of
    // step, one in A while the other is in B; measured 1 % on the launch.
    __builtin_amdgcn_s_setprio(3);
    i32x4 vf[G::NDB];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      if (c < G::KSTEPS) {
        const f32x16 acc = (c == 0) ? (f32x16){0} : Sn;
        Sn = Elem<T>::mfma(kf[c % KR], Qf[c], acc);
        if (c + KR < G::KSTEPS) kf[c % KR] = fr.load_k(KOFF, KB ^ 1, c + KR);
      }
      if (c >= 8 - G::NDB) vf[c - (8 - G::NDB)] = fr.load_v(VOFF, 2 * KB, c - (8 - G::NDB));
      soft_slice(c, Sc, 4, Pc, rsv[KB], m_neg);
      __builtin_amdgcn_sched_barrier(0);
    }
    // keep the exponentials in this block (they would otherwise sink below
    // the branches that follow, away from the MFMAs they are meant to overlap)
    asm volatile("" : "+v"(Pc[4]), "+v"(Pc[5]), "+v"(Pc[6]), "+v"(Pc[7]), "+v"(rsv[KB]));
    if (__builtin_amdgcn_ballot_w64(!(rsv[KB] <= kRowSumLimit)) != 0) exact_fix(Sc, Pc, rsv[KB]);
    l += rsv[KB];
    mask_half(h + 1, Sn);
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int sl = 0; sl < 8; ++sl) {
      if (sl < 2 * G::NDB) {
        const int kk = sl / G::NDB, db = sl % G::NDB;
        const i32x4 pf = {(int)Pc[4 * kk], (int)Pc[4 * kk + 1], (int)Pc[4 * kk + 2], (int)Pc[4 * kk + 3]};
        O[db] = Elem<T>::mfma(vf[db], pf, O[db]);
        if (kk == 0) vf[db] = fr.load_v(VOFF, 2 * KB + 1, db);
      }
      if (sl >= 4 && sl - 4 < KR) kf[sl - 4] = fr.load_k(K2OFF, KB, sl - 4);
      // (for the last half of a wave Sn holds scores of stale LDS contents: the results are never used)
      soft_slice(sl, Sn, 0, Pn, rsv[KB ^ 1], m_neg);
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("" : "+v"(Pn[0]), "+v"(Pn[1]), "+v"(Pn[2]), "+v"(Pn[3]), "+v"(rsv[KB ^ 1]));
  };

  // tile t: barrier (tile t+1 visible, stage of tile t-1 free), refill, two halves.
  // (Tile 0: the item's first barrier has done all of that.)
  auto tile_iter = [&](auto ts_c, int t) __attribute__((always_inline)) {
    constexpr int TS = decltype(ts_c)::value;
    if (t + NS - 1 < n_tiles) {
      if (t > 0) {
        // tile t+1 was requested NS-2 iterations ago; the younger tile t+2 may still fly
        __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 3) * 2 * IPW));
        __syncthreads();
        dma.template tile<(TS + NS - 1) % NS>(cur.kv, (t + NS - 1) * TN);
      }
    } else if (t == tail_t) {
      // Nothing is left to request: every remaining tile is in the ring or on
      // its way.  One full wait and one barrier publish them all, and the waves
      // then run to the end of the item without meeting again - in the diagonal
      // block of a causal item each wave has its own number of halves to do.
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
      __syncthreads();
    }
    half_step(ic<2 * TS>{}, 2 * t);
    half_step(ic<2 * TS + 1>{}, 2 * t + 1);
  };

  // ---- normalise, transpose through LDS, coalesced 16-byte stores; LSE from
  // half the lanes.  The staging area is the LAST stage (first four waves in
  // its K tile, the others in its V tile) because the other stages are being
  // filled for the next item; a wave stages and stores its 32 rows in two
  // passes of up to 64 columns.  Only the wave itself reads what it staged and
  // a wave's LDS accesses execute in order, so no barrier is needed.
  constexpr int DBP = (G::NDB + 1) / 2;  // 32-column blocks of O per pass
  constexpr int SROW = DBP * 64;         // bytes of a staged row
  constexpr int CH = SROW / 16;          // 16-byte chunks of a staged row
  // 16-byte store instructions a wave issues for 32 rows that all exist; they
  // are the last vector-memory instructions of an item
  constexpr int kOutStores = 2 * (32 * CH / 64);
  auto write_out = [&](auto&& after_pass0, auto&& after_pass1) __attribute__((always_inline)) {
    static_assert(4 * 32 * SROW <= TILEB, "four waves stage inside one tile");
    auto sswz = [](int row) { return SROW == 128 ? ((row >> 1) & 7) : ((row >> 2) & 3); };
    // Lane coordinates through an opaque copy: the staging and output offsets
    // below would otherwise be computed once, ahead of the item loop, and sit
    // in (spilled) registers across the tile loop.
    int lane_o = lane, lq_o = fr.lq, lh_o = fr.lh;
    asm volatile("" : "+v"(lane_o), "+v"(lq_o), "+v"(lh_o));
    const float l_tot = sum_with_other_half(l);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (cur.lp && lh_o == 0 && qrow < len)
      cur.lp[(int64_t)qrow * p.lse_ss] = l_tot > 0.f ? m + fast_log2(l_tot) : -INFINITY;
    unsigned char* stage = smem + (wave < 4 ? 0 : VBASE) + (NS - 1) * TILEB + (wave & 3) * 32 * SROW;
#pragma unroll
    for (int ps = 0; ps < 2; ++ps) {
#pragma unroll
      for (int dl = 0; dl < DBP; ++dl) {
        const int db = ps * DBP + dl;
        if (db < G::NDB) {
#pragma unroll
          for (int gq = 0; gq < 4; ++gq) {
            const int c = 4 * dl + gq;  // chunk of the staged row: columns 8c + 4lh .. +3 of this pass
            i32x2 w;
            w[0] = (int)Elem<T>::pack2(O[db][4 * gq] * inv, O[db][4 * gq + 1] * inv);
            w[1] = (int)Elem<T>::pack2(O[db][4 * gq + 2] * inv, O[db][4 * gq + 3] * inv);
            *reinterpret_cast<i32x2*>(stage + lq_o * SROW + ((c ^ sswz(lq_o)) << 4) + 8 * lh_o) = w;
          }
        }
      }
      asm volatile("" ::: "memory");
#pragma unroll
      for (int i = 0; i < 32 * CH / 64; ++i) {
        const int idx = lane_o + 64 * i;
        const int row = idx / CH, ch = idx % CH;
        const int och = ps * CH + ch;  // chunk of the output row
        if (och < G::NCH && q0w + row < len) {
          const i32x4 val = *reinterpret_cast<const i32x4*>(stage + row * SROW + ((ch ^ sswz(row)) << 4));
          // One store instruction per statement, whatever the compiler would
          // have made of a plain assignment: the wait at the top of the next
          // item counts on exactly kOutStores of them behind the loads that
          // request_item() issued.  The s_nop covers the wait states a store
          // of more than 8 bytes needs before its data registers may be
          // overwritten (the compiler pads its own stores, not this one).
          T* dst = cur.op + (int64_t)(q0w + row) * p.o_ss + och * 8;
          asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1" : : "v"(dst), "v"(val) : "memory");
        }
      }
      asm volatile("" ::: "memory");
      if (ps == 0)
        after_pass0();
      else
        after_pass1();
    }
  };

  bool have = next_item(cur);
  if (have) {
    request_item(cur, Qf);
    request_tile1(cur);
    request_tile2(cur);
  }
  int out_stores = 0;  // output stores of the previous item that may still be in flight
  while (have) {
    len = cur.len;
    n_tiles = cur.n_tiles;
    q0w = cur.q0 + 32 * rblk;
    qrow = q0w + fr.lq;
    row_lim = causal ? min(qrow, len - 1) : len - 1;  // largest key this lane may see
    H_w = (len + 31) / 32;                            // halves this wave works on
    if (causal) H_w = min(H_w, q0w / 32 + 1);         // nothing above its own diagonal block
    H_w = min(H_w, 2 * n_tiles);
    if (q0w >= len) H_w = 0;                          // all rows past the sequence end
    tail_t = max(1, n_tiles - (NS - 1));
#pragma unroll
    for (int db = 0; db < G::NDB; ++db) O[db] = (f32x16){0};
    m = -INFINITY;
    m_neg = 0.f;
    l = 0.f;

    // The Q operands and tiles 0 and 1 must have landed (K of tile 1 is read
    // while tile 0 is finished).  At an item boundary the requests and the
    // previous item's output stores were issued in the order
    //   Q, tile 0, stores of pass 0, tile 1, stores of pass 1, tile 2
    // so that the loads queue behind one another while the wave works on the
    // write-out.  vmcnt retires loads and stores in issue order: the stores of
    // pass 1 and the loads of tile 2 may stay in flight when both were issued
    // in full (out_stores says so); otherwise everything is waited for.  The
    // barrier publishes the tiles and separates the previous item's staging
    // reads from the refill of the last stage, which follows at once.
    if (out_stores == kOutStores)
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(kOutStores / 2 + 2 * IPW));
    else
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    // The Q registers were written by loads the compiler cannot see.  Passing
    // them through an empty statement HERE makes every use of them depend on a
    // point behind the wait, so no read of them can be scheduled above it.
#pragma unroll
    for (int c = 0; c < G::KSTEPS; ++c) asm volatile("" : "+v"(Qf[c]));
    __syncthreads();
    if (NS - 1 < n_tiles) dma.template tile<NS - 1>(cur.kv, (NS - 1) * TN);
    if (H_w > 0) {
      // scores of half 0, its exact row maximum as the first reference point,
      // the probabilities of its first 8 keys, then the first fragments of half 1
      f32x16 acc = (f32x16){0};
#pragma unroll
      for (int c = 0; c < G::KSTEPS; ++c) acc = Elem<T>::mfma(fr.load_k(0u, 0, c), Qf[c], acc);
      S[0] = acc;
      mask_half(0, S[0]);
      exact_fix(S[0], Pb[0], rsv[0]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        exp_first(S[0], i, m_neg);
        exp_second(i, Pb[0], rsv[0]);
      }
#pragma unroll
      for (int c = 0; c < KR; ++c) kf[c] = fr.load_k(0u, 1, c);
    }

    for (int t = 0; t < n_tiles; t += NS) {
      tile_iter(ic<0>{}, t);
      if (t + 1 >= n_tiles) break;
      tile_iter(ic<1 % NS>{}, t + 1);
      if (t + 2 >= n_tiles) break;
      tile_iter(ic<2 % NS>{}, t + 2);
      if (NS > 3) {
        if (t + 3 >= n_tiles) break;
        tile_iter(ic<3 % NS>{}, t + 3);
      }
    }
    __builtin_amdgcn_s_setprio(0);
    __syncthreads();  // every wave is done with the tiles

    Item nxt = cur;
    const bool more = next_item(nxt);
    if (more) request_item(nxt, Qf);  // (Qf is dead by now; no copy may sit between a load and its wait)
    write_out([&]() __attribute__((always_inline)) { if (more) request_tile1(nxt); },
              [&]() __attribute__((always_inline)) { if (more) request_tile2(nxt); });
    // every store instruction had live lanes and tile 2 was requested behind them
    out_stores = (q0w + 32 <= len && more && 2 < nxt.n_tiles) ? kOutStores : 0;
    cur = nxt;
    have = more;
  }
}

// ---------------------------------------------------------------------------
// Dense, short form: workgroups of 4 wavefronts (128 query rows per item), KV
// tiles of 32 keys in a ring of five stages (80 KiB of LDS per workgroup, 40 at
// head_dim 64), two workgroups to a CU, three at head_dim 64.
//
// dense_kernel keeps one 8-wave workgroup per CU, two wavefronts per SIMD, and
// a work item is one chain of latencies (geometry, Q and first tiles, the exact
// first half, the tile loop, normalise, stage, store).  Two uses:
//  - launches with at most one 128-row item per CU (short prompts, few heads):
//    twice as many CUs work, each on a chain half as long.  10 to 17 % faster
//    than dense_kernel at head_dim 128 on every such launch measured (1 to 4
//    sequences of 256 to 4096 tokens, 8 and 32 heads, causal and not); with
//    more items than CUs the two forms are within 5 % of each other at head_dim
//    96 and 128 (two waves per SIMD either way) and dense_kernel stays ahead.
//  - head_dim 64: the softmax arithmetic outweighs the matrix work there (56
//    vector instructions against 8 MFMAs per 32 x 32 block of scores) and a
//    wave's registers (O, S, Q^T, P: 163 in all) leave room for a third
//    wavefront per SIMD, which fills issue slots that two leave empty.  3 to 8 %
//    faster than dense_kernel on launches of eight rounds or more (4 x 8192
//    tokens, 32 heads: 1158 against 1190 us), 6 to 11 % on 16 sequences of 2048
//    / 512 tokens; slower where the item count is a round and a bit (1024 items
//    on 768 slots) while dense_kernel's rounds come out even, which the launcher
//    works out per launch (short_form_pays).
// The price is twice the tile traffic from the L2s per query row.
//
//
// The same half-tile software pipeline as dense_kernel, a tile now being one
// half: at position h a wave forms S(h+1) = K(h+1) Q^T together with the second
// half of the exponentials of S(h), then O += V(h)^T P(h)^T together with the
// first half of those of S(h+1), and reads the first K fragments of tile h+2
// along the way.  Tile j is requested at the top of position j - 4 into stage
// j % 5, the stage of tile j - 5, which every wave has left by then (barrier);
// at the top of position h tiles up to h+2 must have landed, tile h+3 may still
// be in flight (counted wait, loads retire in issue order).  Score registers
// alternate with the position's parity and the ring has five stages, so the
// tile loop is unrolled ten times.
//
// WIN: the token-window form (causal, key > query - win_local or key <
// win_global) without block lists.  The keys a 128-row item can see are the
// tiles of the first win_global keys (the sink tiles) and a band of tiles that
// ends at its diagonal block, so the walk is the dense one over a shorter
// sequence of tiles: position j is tile j when j < n_sink and tile j + skip
// otherwise.  The window's lower edge is masked per key like the diagonal.
// With win_global == 0 the first positions of an item lie below the window of
// its later rows: a row that has not met a visible key has no reference point
// yet and takes the exact path until it has one.
template <typename T, int D, bool WIN>
__global__ void __launch_bounds__(kShortRows * 2) __attribute__((amdgpu_waves_per_eu(short_per_cu(D))))
dense_short_kernel(const PrefillParams p) {
  constexpr int NW = kShortRows / 32, NS = kShortStages, TN = kShortTileKeys;
  static_assert(NW == 4 && NS == 5 && TN == 32, "stage use at the item boundary assumes this shape");
  using G = RowGeom<D>;
  using F = SwizzledFrags<D>;
  using DMA = TileDma<T, D, NW, NS, TN>;
  constexpr int BM = 32 * NW;
  constexpr int TILEB = DMA::TILEB, VBASE = DMA::VBASE, IPW = DMA::IPW;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  F fr;
  fr.init(lane, (uint32_t)(uintptr_t)smem, VBASE);
  DMA dma;
  dma.init(p, lane, wave);
  const int causal = p.causal;
  const float scale = p.scale;

  struct Item {
    int len, q0, n_tiles;
    int n_sink, skip;  // WIN: positions below n_sink are tiles of their own number, the others lie `skip` tiles further on
    const T* qp;
    T* op;
    float* lp;
    KvSrc<T> kv;
  };
  // first key of the tile at position j of an item's walk
  auto key_of = [](const Item& it, int j) __attribute__((always_inline)) -> int {
    return WIN ? (j + (j >= it.n_sink ? it.skip : 0)) * TN : j * TN;
  };
  const int grid = gridDim.x;
  const int wl = p.win_local, wg = p.win_global;
  int round = 0, base = 0;
  auto next_item = [&](Item& it) __attribute__((always_inline)) -> bool {
    while (base < p.n_items) {
      int w = blockIdx.x;
      if ((round & 1) && (grid & 7) == 0) w = (((grid >> 3) - 1 - (w >> 3)) << 3) | (w & 7);
      const int bid = base + w;
      base += grid;
      ++round;
      ItemGeo g;
      if (bid < p.n_items && item_geo<BM>(p, bid, g)) {
        it.len = g.len;
        it.q0 = g.qt * BM;
        it.n_tiles = (g.len + TN - 1) / TN;
        if (causal) it.n_tiles = min(it.n_tiles, (it.q0 + BM + TN - 1) / TN);
        it.n_sink = it.skip = 0;
        if (WIN) {
          const int t0 = max(it.q0 - wl + 1, 0) / TN;  // tile of the first key inside the local window of the item's first row
          it.n_sink = min((wg + TN - 1) / TN, t0);
          it.skip = t0 - it.n_sink;
          it.n_tiles -= it.skip;
        }
        it.qp = reinterpret_cast<const T*>(p.q) + g.q_off + g.h * p.q_sh;
        it.op = reinterpret_cast<T*>(p.o) + g.o_off + g.h * p.o_sh;
        it.lp = p.lse ? p.lse + g.lse_off + g.h * p.lse_sh : nullptr;
        it.kv = DMA::source(reinterpret_cast<const T*>(p.k) + g.k_off + g.kvh * p.k_sh,
                            reinterpret_cast<const T*>(p.v) + g.v_off + g.kvh * p.v_sh, g.len);
        return true;
      }
    }
    return false;
  };
  // Q^T operands of an item and its first tile; tiles 1 to 3 follow from
  // request_tile<1..3>.  Nothing waits here (loads from inline assembly, see dense_kernel).
  auto request_item = [&](const Item& it, i32x4 (&Q)[G::KSTEPS]) __attribute__((always_inline)) {
    const int row = min(it.q0 + 32 * wave + fr.lq, it.len - 1);
    const T* qr = it.qp + (int64_t)row * p.q_ss + 8 * fr.lh;
#pragma unroll
    for (int c = 0; c < G::KSTEPS; ++c)
      asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "=v"(Q[c]) : "v"(qr), "n"(32 * c));
    if (0 < it.n_tiles) dma.template tile<0>(it.kv, key_of(it, 0));
  };
  auto request_tile = [&](auto j_c, const Item& it) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value;
    if (J < it.n_tiles) dma.template tile<J>(it.kv, key_of(it, J));
  };

  Item cur;
  i32x4 Qf[G::KSTEPS];
  f32x16 O[G::NDB];
  float m, l, m_neg;
  int len, n_tiles, q0w, qrow, row_lim, H_w;
  int tail_h;  // first position (> 0) at whose top no further tile is requested
  f32x16 S[2];
  constexpr int KR = G::KSTEPS < 4 ? G::KSTEPS : 4;
  i32x4 kf[KR];

  auto mask_half = [&](int hh, f32x16& Sx) __attribute__((always_inline)) {
    const int k0h = WIN ? key_of(cur, hh) : hh * 32;
    bool edge = (k0h + 32 > len) || (causal && k0h + 31 > q0w);
    // WIN: some key of the tile may lie below the local window of some row of the wave and outside the global one
    if (WIN) edge = edge || (k0h <= q0w + 31 - wl && k0h + 31 >= wg);
    if (edge) {
      const int t = row_lim - k0h - 8 * fr.lh;
      const int below = t - wl;               // WIN: offsets up to here are at or below query - win_local ...
      const int sink = wg - k0h - 8 * fr.lh;  // ... and are masked unless they are below this one (inside the global window)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kk = 16 * (r >> 3) + (r & 7);
        if (kk > t || (WIN && kk <= below && kk >= sink)) Sx[r] = -INFINITY;
      }
    }
  };

  constexpr float kRowSumLimit = 4096.f;
  uint32_t Pb[2][8];
  float rsv[2];
  float e_p0, e_u1;
  auto exp_first = [&](const f32x16& Sx, int i, float mn) __attribute__((always_inline)) {
    e_p0 = fast_exp2(fmaf(Sx[2 * i], scale, mn));
    e_u1 = fmaf(Sx[2 * i + 1], scale, mn);
  };
  auto exp_second = [&](int i, uint32_t (&Pd)[8], float& rs) __attribute__((always_inline)) {
    const float p1 = fast_exp2(e_u1);
    rs = i == 0 ? e_p0 + p1 : rs + (e_p0 + p1);
    Pd[i] = Elem<T>::pack2(e_p0, p1);
  };
  float su0[2], su1[2], sp0[2], sp1[2], st;
  auto soft_slice = [&](int c, const f32x16& Sx, int i0, uint32_t (&Pd)[8], float& rs, float mn) __attribute__((always_inline)) {
    const int j = (c + 1) / 2;
    if (c == 0) {
      su0[0] = fmaf(Sx[2 * i0], scale, mn);
      su1[0] = fmaf(Sx[2 * i0 + 1], scale, mn);
      sp0[0] = fast_exp2(su0[0]);
      return;
    }
    if (c & 1) {
      const int k = (c - 1) / 2, sl = k & 1;
      sp1[sl] = fast_exp2(su1[sl]);
      if (k > 0) rs = (i0 == 0 && k == 1) ? st : rs + st;
      if (k < 3) {
        su0[sl ^ 1] = fmaf(Sx[2 * (i0 + k + 1)], scale, mn);
        su1[sl ^ 1] = fmaf(Sx[2 * (i0 + k + 1) + 1], scale, mn);
      } else {
        const float t2 = sp0[sl] + sp1[sl];
        Pd[i0 + 3] = Elem<T>::pack2(sp0[sl], sp1[sl]);
        rs += t2;
      }
    } else {
      const int sl = j & 1;
      sp0[sl] = fast_exp2(su0[sl]);
      st = sp0[sl ^ 1] + sp1[sl ^ 1];
      Pd[i0 + j - 1] = Elem<T>::pack2(sp0[sl ^ 1], sp1[sl ^ 1]);
    }
  };
  auto exact_fix = [&](const f32x16& Sx, uint32_t (&Pd)[8], float& rs) __attribute__((always_inline)) {
    float mx = Sx[0];
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(mx, Sx[r]);
    mx = max_with_other_half(mx);
    const float m_new = fmaxf(m, mx * scale);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fast_exp2(m - m_safe);
    l *= alpha;
#pragma unroll
    for (int db = 0; db < G::NDB; ++db) O[db] *= alpha;
    m = m_new;
    m_neg = -m_safe;
    rs = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float p0 = fast_exp2(fmaf(Sx[2 * i], scale, -m_safe));
      const float p1 = fast_exp2(fmaf(Sx[2 * i + 1], scale, -m_safe));
      rs += p0 + p1;
      Pd[i] = Elem<T>::pack2(p0, p1);
    }
  };

  // position h; J = h % 10: stage J % 5, score registers S[J & 1]
  auto half_step = [&](auto j_c, int h) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value;
    if (h >= H_w) return;
    constexpr int TS = J % NS, KB = J & 1;
    constexpr uint32_t KOFF = ((TS + 1) % NS) * TILEB, VOFF = TS * TILEB, K2OFF = ((TS + 2) % NS) * TILEB;
    f32x16& Sc = S[KB];
    f32x16& Sn = S[KB ^ 1];
    uint32_t (&Pc)[8] = Pb[KB];
    uint32_t (&Pn)[8] = Pb[KB ^ 1];
    __builtin_amdgcn_s_setprio(3);
    i32x4 vf[G::NDB];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      if (c < G::KSTEPS) {
        const f32x16 acc = (c == 0) ? (f32x16){0} : Sn;
        Sn = Elem<T>::mfma(kf[c % KR], Qf[c], acc);
        if (c + KR < G::KSTEPS) kf[c % KR] = fr.load_k(KOFF, 0, c + KR);
      }
      if (c >= 8 - G::NDB) vf[c - (8 - G::NDB)] = fr.load_v(VOFF, 0, c - (8 - G::NDB));
      soft_slice(c, Sc, 4, Pc, rsv[KB], m_neg);
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("" : "+v"(Pc[4]), "+v"(Pc[5]), "+v"(Pc[6]), "+v"(Pc[7]), "+v"(rsv[KB]));
    if (__builtin_amdgcn_ballot_w64(!(rsv[KB] <= kRowSumLimit) || (WIN && m == -INFINITY)) != 0) exact_fix(Sc, Pc, rsv[KB]);
    l += rsv[KB];
    mask_half(h + 1, Sn);
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int sl = 0; sl < 8; ++sl) {
      if (sl < 2 * G::NDB) {
        const int kk = sl / G::NDB, db = sl % G::NDB;
        const i32x4 pf = {(int)Pc[4 * kk], (int)Pc[4 * kk + 1], (int)Pc[4 * kk + 2], (int)Pc[4 * kk + 3]};
        O[db] = Elem<T>::mfma(vf[db], pf, O[db]);
        if (kk == 0) vf[db] = fr.load_v(VOFF, 1, db);
      }
      if (sl >= 4 && sl - 4 < KR) kf[sl - 4] = fr.load_k(K2OFF, 0, sl - 4);
      // (for the last position of a wave Sn holds scores of stale LDS contents: the results are never used)
      soft_slice(sl, Sn, 0, Pn, rsv[KB ^ 1], m_neg);
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("" : "+v"(Pn[0]), "+v"(Pn[1]), "+v"(Pn[2]), "+v"(Pn[3]), "+v"(rsv[KB ^ 1]));
  };

  // top of position h (> 0), then the position
  auto pos = [&](auto j_c, int h) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value;
    if (h + NS - 1 < n_tiles) {
      // tiles up to h+2 landed (requested at least two positions ago); tile h+3 may still fly
      __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 4) * 2 * IPW));
      __syncthreads();
      dma.template tile<(J + NS - 1) % NS>(cur.kv, key_of(cur, h + NS - 1));
    } else if (h == tail_h) {
      // nothing left to request: one full wait and one barrier publish what is
      // still on its way, and the waves run to the end of the item on their own
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
      __syncthreads();
    }
    half_step(j_c, h);
  };

  // ---- normalise, transpose through LDS, coalesced 16-byte stores (as in
  // dense_kernel; the staging area is the last stage: waves 0, 1 in its K tile,
  // waves 2, 3 in its V tile)
  constexpr int DBP = (G::NDB + 1) / 2;
  constexpr int SROW = DBP * 64;
  constexpr int CH = SROW / 16;
  auto write_out = [&](auto&& after_pass0, auto&& after_pass1) __attribute__((always_inline)) {
    static_assert(2 * 32 * SROW <= TILEB, "two waves stage inside one tile");
    auto sswz = [](int row) { return SROW == 128 ? ((row >> 1) & 7) : ((row >> 2) & 3); };
    int lane_o = lane, lq_o = fr.lq, lh_o = fr.lh;
    asm volatile("" : "+v"(lane_o), "+v"(lq_o), "+v"(lh_o));
    const float l_tot = sum_with_other_half(l);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (cur.lp && lh_o == 0 && qrow < len)
      cur.lp[(int64_t)qrow * p.lse_ss] = l_tot > 0.f ? m + fast_log2(l_tot) : -INFINITY;
    unsigned char* stage = smem + (wave < 2 ? 0 : VBASE) + (NS - 1) * TILEB + (wave & 1) * 32 * SROW;
#pragma unroll
    for (int ps = 0; ps < 2; ++ps) {
#pragma unroll
      for (int dl = 0; dl < DBP; ++dl) {
        const int db = ps * DBP + dl;
        if (db < G::NDB) {
#pragma unroll
          for (int gq = 0; gq < 4; ++gq) {
            const int c = 4 * dl + gq;
            i32x2 w;
            w[0] = (int)Elem<T>::pack2(O[db][4 * gq] * inv, O[db][4 * gq + 1] * inv);
            w[1] = (int)Elem<T>::pack2(O[db][4 * gq + 2] * inv, O[db][4 * gq + 3] * inv);
            *reinterpret_cast<i32x2*>(stage + lq_o * SROW + ((c ^ sswz(lq_o)) << 4) + 8 * lh_o) = w;
          }
        }
      }
      asm volatile("" ::: "memory");
#pragma unroll
      for (int i = 0; i < 32 * CH / 64; ++i) {
        const int idx = lane_o + 64 * i;
        const int row = idx / CH, ch = idx % CH;
        const int och = ps * CH + ch;
        if (och < G::NCH && q0w + row < len) {
          const i32x4 val = *reinterpret_cast<const i32x4*>(stage + row * SROW + ((ch ^ sswz(row)) << 4));
          T* dst = cur.op + (int64_t)(q0w + row) * p.o_ss + och * 8;
          // (from assembly, so that no counted wait of the compiler's sits between these stores and the tile requests around them)
          asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1" : : "v"(dst), "v"(val) : "memory");
        }
      }
      asm volatile("" ::: "memory");
      if (ps == 0)
        after_pass0();
      else
        after_pass1();
    }
  };

  bool have = next_item(cur);
  if (have) {
    request_item(cur, Qf);
    request_tile(ic<1>{}, cur);
    request_tile(ic<2>{}, cur);
    request_tile(ic<3>{}, cur);
  }
  while (have) {
    len = cur.len;
    n_tiles = cur.n_tiles;
    q0w = cur.q0 + 32 * wave;
    qrow = q0w + fr.lq;
    row_lim = causal ? min(qrow, len - 1) : len - 1;
    H_w = (len + 31) / 32;
    if (causal) H_w = min(H_w, q0w / 32 + 1);
    if (WIN) H_w -= cur.skip;  // (positions, not keys: the diagonal lies in the band)
    H_w = min(H_w, n_tiles);
    if (q0w >= len) H_w = 0;
    tail_h = max(1, n_tiles - (NS - 1));
#pragma unroll
    for (int db = 0; db < G::NDB; ++db) O[db] = (f32x16){0};
    m = -INFINITY;
    m_neg = 0.f;
    l = 0.f;

    // Q and tiles 0 to 2 must have landed (position 0 reads K of tiles 1 and
    // 2).  They were requested in the order Q, tile 0, [stores], tile 1,
    // [stores], tile 2, tile 3, and everything retires in that order: when tile
    // 3 exists its loads are the youngest and may stay in flight.
    if (NS - 2 < n_tiles)
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(2 * IPW));
    else
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
#pragma unroll
    for (int c = 0; c < G::KSTEPS; ++c) asm volatile("" : "+v"(Qf[c]));
    __syncthreads();
    if (NS - 1 < n_tiles) dma.template tile<NS - 1>(cur.kv, key_of(cur, NS - 1));
    if (H_w > 0) {
      f32x16 acc = (f32x16){0};
#pragma unroll
      for (int c = 0; c < G::KSTEPS; ++c) acc = Elem<T>::mfma(fr.load_k(0u, 0, c), Qf[c], acc);
      S[0] = acc;
      mask_half(0, S[0]);
      exact_fix(S[0], Pb[0], rsv[0]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        exp_first(S[0], i, m_neg);
        exp_second(i, Pb[0], rsv[0]);
      }
#pragma unroll
      for (int c = 0; c < KR; ++c) kf[c] = fr.load_k(1u * TILEB, 0, c);
    }

    half_step(ic<0>{}, 0);
    for (int h = 1; h < n_tiles; h += 10) {
      pos(ic<1>{}, h);
      if (h + 1 >= n_tiles) break;
      pos(ic<2>{}, h + 1);
      if (h + 2 >= n_tiles) break;
      pos(ic<3>{}, h + 2);
      if (h + 3 >= n_tiles) break;
      pos(ic<4>{}, h + 3);
      if (h + 4 >= n_tiles) break;
      pos(ic<5>{}, h + 4);
      if (h + 5 >= n_tiles) break;
      pos(ic<6>{}, h + 5);
      if (h + 6 >= n_tiles) break;
      pos(ic<7>{}, h + 6);
      if (h + 7 >= n_tiles) break;
      pos(ic<8>{}, h + 7);
      if (h + 8 >= n_tiles) break;
      pos(ic<9>{}, h + 8);
      if (h + 9 >= n_tiles) break;
      pos(ic<0>{}, h + 9);
    }
    __builtin_amdgcn_s_setprio(0);
    __syncthreads();  // every wave is done with the tiles

    Item nxt = cur;
    const bool more = next_item(nxt);
    if (more) request_item(nxt, Qf);
    write_out([&]() __attribute__((always_inline)) { if (more) request_tile(ic<1>{}, nxt); },
              [&]() __attribute__((always_inline)) {
                if (more) {
                  request_tile(ic<2>{}, nxt);
                  request_tile(ic<3>{}, nxt);
                }
              });
    cur = nxt;
    have = more;
  }
}

template <int D, int NW, int NS, int TN>
constexpr size_t prefill_lds_bytes() {
  const size_t pipe = (size_t)NS * 2 * TN * SwizzledFrags<D>::ROWB;
  const size_t epi = (size_t)NW * 32 * (D * 2 + 16);
  return pipe > epi ? pipe : epi;
}

// Which form for a head_dim-64 launch?  A model of how long the busiest CU
// works, in units of one 128-row item at full occupancy.  Short form: the grid
// is kShortPerCu workgroups per CU, workgroup w sits on CU w % cus and walks
// items w, w + grid, ...; the first n % grid workgroups have one item more than
// the others.  Three resident workgroups keep a CU busy; when the ones with
// fewer items have finished, two run at 0.7 and a lone one at 0.4 of that rate.
// Long form: one 256-row item after another per CU, each worth 2.3 items of the
// short form (twice the rows at about 13 % less per row).  The three constants
// are fitted to HIP-event timings of both forms on 1 to 48 sequences of 256 to
// 8192 tokens with 12, 20 and 32 heads, causal and not: against the faster
// form of each launch the choice costs 0.7 % in the geometric mean (always the
// long form: 8.5 %, always the short form: 2.5 %).
inline double short_form_cost(long long n, int cus) {
  const long long grid = (long long)kShortPerCu * cus;
  const long long q = n / grid, r = n % grid;
  static_assert(kShortPerCu == 3, "the rates below are those of one, two and three workgroups");
  const double rate[kShortPerCu + 1] = {0.0, 0.4, 0.7, 1.0};
  double worst = 0.0;
  for (const int c : {0, cus - 1}) {   // items per workgroup fall with the workgroup id: the ends of the range suffice
    long long items[kShortPerCu];
    for (int k = 0; k < kShortPerCu; ++k) items[k] = q + ((long long)c + (long long)k * cus < r ? 1 : 0);
    // (items[0] >= items[1] >= items[2]) phases: all three until the shortest is done, then two, then one
    double t = 0.0;
    long long done = 0;
    for (int live = kShortPerCu; live >= 1; --live) {
      const long long upto = items[live - 1];
      if (upto > done) {
        t += (double)(upto - done) * live / rate[live];
        done = upto;
      }
    }
    worst = t > worst ? t : worst;
  }
  return worst;
}
inline bool short_form_pays(long long n128, long long n256, int cus) {
  if (cus <= 0) return false;
  if (n128 <= cus) return true;   // a CU per workgroup: twice as many CUs busy as with 256-row items
  return short_form_cost(n128, cus) < 2.3 * (double)((n256 + cus - 1) / cus);
}

template <typename T, int D, bool WIN = false>
int launch_short(const PrefillParams& p, long long items, int cus, hipStream_t s) {
  auto kern = dense_short_kernel<T, D, WIN>;
  constexpr size_t lds = prefill_lds_bytes<D, kShortRows / 32, kShortStages, kShortTileKeys>();
  constexpr int per_cu = short_per_cu(D);
  static_assert(per_cu * lds <= 160 * 1024, "that many workgroups share a CU's LDS");
  static LdsLimitOnce lds_once;
  if (const int e = raise_lds_limit(lds_once, reinterpret_cast<const void*>(kern), (int)lds)) return e;
  PrefillParams pp = p;
  pp.n_qtiles = (p.max_seqlen + kShortRows - 1) / kShortRows;
  pp.n_items = (int)items;
  long long grid = items;
  if (cus > 0 && grid > (long long)per_cu * cus) grid = (long long)per_cu * cus;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kShortRows * 2), lds, s, pp);
  return (int)hipGetLastError();
}

template <typename T, int D, bool SPARSE>
int launch_one(const PrefillParams& p, hipStream_t s) {
  if constexpr (!SPARSE) {
    const int cus = device_cu_count();
    const long long n = (long long)((p.max_seqlen + kShortRows - 1) / kShortRows) * p.hq * p.batch;
    bool short_form = p.dense_form == 2;
    if (p.dense_form == 0) {
      if (D == 64)
        short_form = short_form_pays(n, (long long)p.n_qtiles * p.hq * p.batch, cus);
      else
        short_form = cus > 0 && n <= cus;   // a CU per 128-row item
    }
    if (short_form) return launch_short<T, D>(p, n, cus, s);
  }
  constexpr int NW = (SPARSE ? kSparseRows : kDenseRows) / 32;
  constexpr int NS = SPARSE ? kSparseStages : kDenseStages;
  constexpr int TN = SPARSE ? kSparseTileKeys : kTileN;
  void (*kern)(const PrefillParams);
  if constexpr (SPARSE)
    kern = sparse_kernel<T, D>;
  else
    kern = dense_kernel<T, D>;
  constexpr size_t lds = prefill_lds_bytes<D, NW, NS, TN>();
  static LdsLimitOnce lds_once;
  if (const int e = raise_lds_limit(lds_once, reinterpret_cast<const void*>(kern), (int)lds)) return e;
  PrefillParams pp = p;
  const long long items = (long long)p.n_qtiles * p.hq * p.batch;
  pp.n_items = (int)items;
  long long grid = items;
  if (!SPARSE) {
    // One workgroup per CU is resident (LDS); more ids than that are walked
    // in-kernel.  (The sparse kernel keeps one launch per q tile: four small
    // workgroups share a CU and cover each other's start-up, and walking ids
    // in-kernel measured slower there.)
    const int cus = device_cu_count();
    if (cus > 0 && grid > cus) grid = cus;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NW * 64), lds, s, pp);
  return (int)hipGetLastError();
}

// The token-window form without block lists: the 128-row form of the dense walk over each item's sink tiles and band.
template <typename T, int D>
int launch_window(const PrefillParams& p, hipStream_t s) {
  const long long n = (long long)((p.max_seqlen + kShortRows - 1) / kShortRows) * p.hq * p.batch;
  return launch_short<T, D, true>(p, n, device_cu_count(), s);
}

template <bool SPARSE>
int dispatch(const PrefillParams& p, int dtype, int head_dim, hipStream_t s) {
  if (dtype == 0) {
    switch (head_dim) {
      case 64: return launch_one<__bf16, 64, SPARSE>(p, s);
      case 96: return launch_one<__bf16, 96, SPARSE>(p, s);
      case 128: return launch_one<__bf16, 128, SPARSE>(p, s);
    }
  } else {
    switch (head_dim) {
      case 64: return launch_one<_Float16, 64, SPARSE>(p, s);
      case 96: return launch_one<_Float16, 96, SPARSE>(p, s);
      case 128: return launch_one<_Float16, 128, SPARSE>(p, s);
    }
  }
  return (int)hipErrorInvalidValue;
}

// Rows of packed outputs that no work item writes.  A workgroup looks at 64
// consecutive rows: lane i finds the sequence of row r0 + i by bisection of cu
// (non-decreasing) and the workgroup leaves at once when all 64 are covered,
// which is the usual case; otherwise its threads zero the uncovered rows.
__global__ void __launch_bounds__(256) zero_uncovered_rows_kernel(const RowFillParams p) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 64 + lane;
  bool uncovered = false;
  if (row < p.total_rows) {
    // last b in [0, batch] with cu[b] <= row
    int lo = 0, hi = p.batch;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (p.cu[mid] <= row) lo = mid; else hi = mid - 1;
    }
    uncovered = lo >= p.batch || row < p.cu[0] || row - p.cu[lo] >= p.max_seqlen;
  }
  const unsigned long long todo = __builtin_amdgcn_ballot_w64(uncovered);
  if (todo == 0) return;
  for (int i = 0; i < 64; ++i) {
    if (!((todo >> i) & 1)) continue;
    const int64_t r = (int64_t)blockIdx.x * 64 + i;
    for (int k = 0; k < p.n_tensors; ++k) {
      const RowFillTensor& t = p.t[k];
      const int words = t.bytes >> 2;
      for (int j = threadIdx.x; j < t.heads * words; j += blockDim.x) {
        const int h = j / words, w = j % words;
        *reinterpret_cast<uint32_t*>(static_cast<char*>(t.base) + r * t.row_stride + h * t.head_stride + 4 * w) = 0u;
      }
    }
  }
}

}  // namespace

int launch_zero_uncovered_rows(const RowFillParams& p, hipStream_t s) {
  if (p.total_rows <= 0 || p.n_tensors <= 0) return 0;
  hipLaunchKernelGGL(zero_uncovered_rows_kernel, dim3((unsigned)((p.total_rows + 63) / 64)), dim3(256), 0, s, p);
  return (int)hipGetLastError();
}

// CUs of the current device (cached per device; 0 if the query fails)
int device_cu_count() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
    cached[dev] = n > 0 ? n : -1;
  }
  return cached[dev] > 0 ? cached[dev] : 0;
}

int launch_prefill_dense(const PrefillParams& p, int dtype, int head_dim, hipStream_t s) {
  return dispatch<false>(p, dtype, head_dim, s);
}
int launch_prefill_sparse(const PrefillParams& p, int dtype, int head_dim, hipStream_t s) {
  return dispatch<true>(p, dtype, head_dim, s);
}
int launch_prefill_window(const PrefillParams& p, int dtype, int head_dim, hipStream_t s) {
  if (dtype == 0) {
    switch (head_dim) {
      case 64: return launch_window<__bf16, 64>(p, s);
      case 96: return launch_window<__bf16, 96>(p, s);
      case 128: return launch_window<__bf16, 128>(p, s);
    }
  } else {
    switch (head_dim) {
      case 64: return launch_window<_Float16, 64>(p, s);
      case 96: return launch_window<_Float16, 96>(p, s);
      case 128: return launch_window<_Float16, 128>(p, s);
    }
  }
  return (int)hipErrorInvalidValue;
}

}  // namespace mi
