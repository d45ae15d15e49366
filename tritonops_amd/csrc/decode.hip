// Single-query (decoding) attention for gfx950: split-KV pass + LSE merge pass,
// dense and block-sparse.
//
// Replaces flash_attn_decoding_kernel / flash_attn_decoding_correction_kernel
// of flash_attn_triton/flash_attn_decoding.py:9-122,:126-210 and their sparse
// twins in flash_attn_triton/flash_attn_decoding_sparse.py:10-127,:131-219.
//
// Pass 1: one wavefront (= one workgroup) per (chunk, kv-head, sequence).  The
// G = hq/hkv query heads that share the kv-head sit in the first G of the 32
// query columns of the same S^T = K.Q^T / O^T = V^T.P^T MFMA pipeline the
// prefill kernel uses, so each K/V byte is fetched once for the whole group
// (the reference launches one program per q-head and re-reads KV G times,
// flash_attn_decoding.py:42-45,264-268) and the dot products cost no VALU
// work.  KV streams global -> registers -> wave-private LDS in 32-key tiles
// with fully coalesced 16-byte loads; no barriers are needed because a single
// wave's LDS operations execute in order.  Partials are fp32 (the reference
// rounds them to the input dtype, :249-251).
// Pass 2: per (sequence, q-head) merge  o = sum_c o_c 2^(lse_c - lse).
#include "kernels.h"
#include "tile_core.h"

namespace mi {
namespace {

constexpr int kDecTile = 32;

template <typename T, int D>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2)))
decode_splitkv_kernel(const DecodeParams p) {
  using G = RowGeom<D>;
  using F = PaddedFrags<D>;
  constexpr int KTILEB = kDecTile * F::KROWB;
  constexpr int VTILEB = kDecTile * F::VROWB;
  constexpr int NCHUNK = kDecTile * G::NCH;
  constexpr int LOADS = (NCHUNK + 63) / 64;

  __shared__ __attribute__((aligned(16))) unsigned char smem[KTILEB + VTILEB];
  unsigned char* sK = smem;
  unsigned char* sV = smem + KTILEB;

  const int lane = threadIdx.x;
  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int len = p.seq_lens ? p.seq_lens[b] : p.cu[b + 1] - p.cu[b];
  const int gqa = p.hq / p.hkv;
  const bool sparse = p.block_idx != nullptr;

  int n_tiles, t_begin = 0;
  const int32_t* blist = nullptr;
  int n_listed = 0;  // listed entries that fall into this chunk
  const int last_blk = (len - 1) / 64;
  if (sparse) {
    const int cnt = p.block_cnt ? min(p.block_cnt[b * p.hkv + kvh], p.max_blocks) : p.max_blocks;
    const int total = cnt + p.add_last;  // the implicit last block sits behind the list
    const int b0 = split * p.split_blocks;
    if (b0 >= total || len <= 0) return;
    blist = p.block_idx + b * p.bi_sb + kvh * p.bi_sh + b0;
    n_tiles = 2 * min(total - b0, p.split_blocks);
    n_listed = max(0, min(cnt - b0, p.split_blocks));
  } else {
    t_begin = split * p.split_tokens;
    if (t_begin >= len) return;
    n_tiles = (min(len, t_begin + p.split_tokens) - t_begin + kDecTile - 1) / kDecTile;
  }
  // sparse: entry i/2 of the chunk; entries behind the listed ones are the
  // implicit last block, and a LISTED last block is dropped when the implicit
  // one exists (base -1 => the whole tile is masked)
  auto tile_base = [&](int i) -> int {
    if (!sparse) return t_begin + i * kDecTile;
    const int e = i >> 1;
    const int blk = e < n_listed ? blist[e] : last_blk;
    if (p.add_last && e < n_listed && blk == last_blk) return -1;
    return blk * 64 + (i & 1) * kDecTile;
  };

  // Start of this sequence's rows: batch stride, row offset cu[b] of a packed
  // buffer, or (paged) the pool itself with the page looked up per tile.
  const int64_t seq0 = p.kv_layout == 1 ? (int64_t)p.cu[b] : 0;
  const int64_t bsel = p.kv_layout == 0 ? b : 0;
  const T* kp = reinterpret_cast<const T*>(p.k) + bsel * p.k_sb + seq0 * p.k_ss + kvh * p.k_sh;
  const T* vp = reinterpret_cast<const T*>(p.v) + bsel * p.v_sb + seq0 * p.v_ss + kvh * p.v_sh;
  const bool paged = p.kv_layout == 2;
  const int32_t* ptab = paged ? p.page_table + b * p.pt_sb : nullptr;
  // Paged: a 32-token tile never straddles a page (page_size % 32 == 0).  The
  // returned element offset moves token `tb` of the flat addressing below onto
  // its place in the physical page.
  auto page_shift = [&](int tb, int64_t page_stride, int64_t row_stride) -> int64_t {
    if (!paged) return 0;
    const int lp = tb / p.page_size;
    const int64_t phys = ptab[lp];
    return phys * page_stride - (int64_t)lp * p.page_size * row_stride;
  };

  F lc;
  lc.init(lane);

  // Q^T operand: column lq is q-head kvh*gqa + lq, columns >= gqa are zero.
  i32x4 Qf[G::KSTEPS];
  {
    const T* qr = reinterpret_cast<const T*>(p.q) + b * p.q_sb +
                  (int64_t)(kvh * gqa + min(lc.lq, gqa - 1)) * p.q_sh + 8 * lc.lh;
#pragma unroll
    for (int c = 0; c < G::KSTEPS; ++c) {
      i32x4 t = *reinterpret_cast<const i32x4*>(qr + 16 * c);
      Qf[c] = lc.lq < gqa ? t : (i32x4){0, 0, 0, 0};
    }
  }

  f32x16 O[G::NDB];
#pragma unroll
  for (int db = 0; db < G::NDB; ++db) O[db] = (f32x16){0};
  float m = -INFINITY, l = 0.f;

  // The loads of tile t + 1 fly while tile t is worked on.  (Registers for a
  // second tile in flight do not exist: the occupancy of this kernel is bounded
  // by LDS, one private tile per wave, at 256 registers per wave, and O, Q and
  // one K/V set already take 240 of them at head_dim 128.)
  i32x4 kreg[LOADS], vreg[LOADS];
  // First token a tile is fetched from.  A tile that is masked as a whole (a
  // dropped duplicate, base -1, or the second half of the last block when the
  // sequence ends in its first half) is fetched from the tile of the last
  // token instead, so that no row outside [0, len) and no page beyond the
  // sequence is ever touched.
  const int last_tile = ((len - 1) / kDecTile) * kDecTile;
  auto addr_base = [&](int base) -> int { return min(max(base, 0), last_tile); };
  // Load i of a lane covers chunk lane % NCH of row lane / NCH + i * (64 / NCH)
  // when NCH divides 64 (head_dim 64 and 128): the address is then a uniform
  // base that advances by a fixed step per load plus one 32-bit lane offset.
  constexpr bool kUniformRows = 64 % G::NCH == 0;
  typedef __attribute__((address_space(1))) const i32x4 g_i32x4;  // global memory, not generic
  typedef __attribute__((address_space(1))) const char g_char;
  auto uniform64 = [](uint64_t x) __attribute__((always_inline)) -> uint64_t {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)x);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
    return ((uint64_t)hi << 32) | lo;
  };
  // pins a uniform address in a scalar register pair, so that the load keeps
  // the form "scalar base + 32-bit lane offset" (the optimiser would otherwise
  // fold the lane offset into a 64-bit vector address per load)
  auto scalar_ptr = [](uint64_t a) __attribute__((always_inline)) -> g_char* {
    uint32_t lo = (uint32_t)a, hi = (uint32_t)(a >> 32);
    asm volatile("" : "+s"(lo), "+s"(hi));
    return (g_char*)(((uint64_t)hi << 32) | lo);
  };
  const uint32_t k_step = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)((64 / G::NCH) * p.k_ss * 2));
  const uint32_t v_step = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)((64 / G::NCH) * p.v_ss * 2));
  const uint32_t k_lane = (uint32_t)((lane / G::NCH) * p.k_ss * 2 + (lane % G::NCH) * 16);
  const uint32_t v_lane = (uint32_t)((lane / G::NCH) * p.v_ss * 2 + (lane % G::NCH) * 16);
  // shift: page_shift() of the tile (0 unless paged)
  const uint32_t k_rowb = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(p.k_ss * 2));
  const uint32_t v_rowb = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(p.v_ss * 2));
  // regs[i] <- chunk (lane + 64 i) of the tile at `tile` (uniform address of
  // its first row); rows beyond row_max re-read row row_max (the last token:
  // same tile, hence same page)
  auto load_tile = [&](i32x4 (&regs)[LOADS], uint64_t tile, int row_max, uint32_t rowb, uint32_t step,
                       uint32_t lane_off) __attribute__((always_inline)) {
    if (kUniformRows && row_max >= kDecTile - 1) {
#pragma unroll
      for (int i = 0; i < LOADS; ++i)
        regs[i] = __builtin_nontemporal_load((g_i32x4*)(scalar_ptr(tile + (uint64_t)i * step) + lane_off));
      return;
    }
    g_char* base = scalar_ptr(tile);
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int idx = lane + i * 64;
      if (NCHUNK % 64 == 0 || idx < NCHUNK) {
        const int row = idx / G::NCH, ch = idx % G::NCH;
        const uint32_t off = (uint32_t)min(row, row_max) * rowb + ch * 16;
        regs[i] = __builtin_nontemporal_load((g_i32x4*)(base + off));
      }
    }
  };
  auto gload = [&](int base, int64_t kshift, int64_t vshift) __attribute__((always_inline)) {
    const int tb = addr_base(base);
    load_tile(kreg, uniform64((uint64_t)(uintptr_t)(kp + kshift + (int64_t)tb * p.k_ss)), len - 1 - tb, k_rowb, k_step,
              k_lane);
    load_tile(vreg, uniform64((uint64_t)(uintptr_t)(vp + vshift + (int64_t)tb * p.v_ss)), len - 1 - tb, v_rowb, v_step,
              v_lane);
  };
  auto lstore = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int idx = lane + i * 64;
      if (NCHUNK % 64 == 0 || idx < NCHUNK) {
        const int row = idx / G::NCH, ch = idx % G::NCH;
        F::store_k(sK, row, ch, kreg[i]);
        F::store_v(sV, row, ch, vreg[i]);
      }
    }
  };

  const int wl = p.win_local, wg = p.win_global;
  // tile bases and page look-ups run one tile ahead of the loads that use
  // them, which run one tile ahead of the compute
  auto shift_k = [&](int base) -> int64_t { return page_shift(addr_base(base), p.k_sb, p.k_ss); };
  auto shift_v = [&](int base) -> int64_t { return page_shift(addr_base(base), p.v_sb, p.v_ss); };
  int base_cur = tile_base(0);
  gload(base_cur, shift_k(base_cur), shift_v(base_cur));
  int base_nxt = n_tiles > 1 ? tile_base(1) : 0;
  int64_t ks_nxt = shift_k(base_nxt), vs_nxt = shift_v(base_nxt);
  lstore();
  for (int it = 0; it < n_tiles; ++it) {
    const int base = base_cur;
    const bool more = it + 1 < n_tiles;
    if (more) gload(base_nxt, ks_nxt, vs_nxt);
    base_cur = base_nxt;
    if (it + 2 < n_tiles) {
      base_nxt = tile_base(it + 2);
      ks_nxt = shift_k(base_nxt);
      vs_nxt = shift_v(base_nxt);
    }
    bool need_mask = base + kDecTile > len || base < 0;
    if (wl >= 0) need_mask = need_mask || !((base + kDecTile - 1 < wg) || (base >= len - wl));
    auto allowed = [&](int key_in_tile) -> bool {
      const int key = base + key_in_tile;
      bool ok = key < len && base >= 0;
      if (wl >= 0) ok = ok && (key < wg || key >= len - wl);
      return ok;
    };
    compute_tile<T, D, 1>(sK, sV, lc, Qf, O, m, l, p.scale, need_mask, allowed);
    if (more) lstore();
  }

  const float l_tot = sum_with_other_half(l);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (lc.lq < gqa) {
    const int h = kvh * gqa + lc.lq;
    const int64_t slot = ((int64_t)b * p.hq + h) * p.n_splits + split;
    if (lc.lh == 0) p.part_lse[slot] = l_tot > 0.f ? m + fast_log2(l_tot) : -INFINITY;
    float* po = p.part_o + slot * D;
#pragma unroll
    for (int db = 0; db < G::NDB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float4 w = {O[db][4 * g] * inv, O[db][4 * g + 1] * inv, O[db][4 * g + 2] * inv,
                    O[db][4 * g + 3] * inv};
        *reinterpret_cast<float4*>(po + 32 * db + 8 * g + 4 * lc.lh) = w;
      }
  }
}

template <typename T>
__global__ void __launch_bounds__(128)
decode_merge_kernel(const DecodeParams p, int D) {
  const int h = blockIdx.x, b = blockIdx.y;
  const int d = threadIdx.x;
  const int len = p.seq_lens ? p.seq_lens[b] : p.cu[b + 1] - p.cu[b];
  int nvalid;
  if (p.block_idx) {
    const int kvh = h / (p.hq / p.hkv);
    const int cnt = p.block_cnt ? min(p.block_cnt[b * p.hkv + kvh], p.max_blocks) : p.max_blocks;
    nvalid = len > 0 ? (cnt + p.add_last + p.split_blocks - 1) / p.split_blocks : 0;
  } else {
    nvalid = (len + p.split_tokens - 1) / p.split_tokens;
  }
  nvalid = max(0, min(nvalid, p.n_splits));
  const int64_t slot0 = ((int64_t)b * p.hq + h) * p.n_splits;
  const float* pl = p.part_lse + slot0;

  float M = -INFINITY;
  for (int c = 0; c < nvalid; ++c) M = fmaxf(M, pl[c]);
  float den = 0.f, acc = 0.f;
  if (M > -INFINITY && d < D) {
    const float* po = p.part_o + slot0 * D + d;
    for (int c = 0; c < nvalid; ++c) {
      const float w = fast_exp2(pl[c] - M);
      den += w;
      acc += w * po[(int64_t)c * D];
    }
  }
  if (d < D) {
    T* op = reinterpret_cast<T*>(p.o) + b * p.o_sb + h * p.o_sh;
    op[d] = (T)(den > 0.f ? acc / den : 0.f);
  }
  if (d == 0 && p.lse) p.lse[(int64_t)b * p.hq + h] = den > 0.f ? M + fast_log2(den) : -INFINITY;
}

template <typename T, int D>
int launch_split(const DecodeParams& p, hipStream_t s) {
  dim3 grid(p.n_splits, p.hkv, p.batch);
  hipLaunchKernelGGL((decode_splitkv_kernel<T, D>), grid, dim3(64), 0, s, p);
  return (int)hipGetLastError();
}

}  // namespace

int launch_decode_splitkv(const DecodeParams& p, int dtype, int head_dim, hipStream_t s) {
  if (dtype == 0) {
    switch (head_dim) {
      case 64: return launch_split<__bf16, 64>(p, s);
      case 96: return launch_split<__bf16, 96>(p, s);
      case 128: return launch_split<__bf16, 128>(p, s);
    }
  } else {
    switch (head_dim) {
      case 64: return launch_split<_Float16, 64>(p, s);
      case 96: return launch_split<_Float16, 96>(p, s);
      case 128: return launch_split<_Float16, 128>(p, s);
    }
  }
  return (int)hipErrorInvalidValue;
}

int launch_decode_merge(const DecodeParams& p, int dtype, int head_dim, hipStream_t s) {
  dim3 grid(p.hq, p.batch);
  if (dtype == 0)
    hipLaunchKernelGGL((decode_merge_kernel<__bf16>), grid, dim3(128), 0, s, p, head_dim);
  else
    hipLaunchKernelGGL((decode_merge_kernel<_Float16>), grid, dim3(128), 0, s, p, head_dim);
  return (int)hipGetLastError();
}

}  // namespace mi
