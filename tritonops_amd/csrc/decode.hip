// Single-query (decoding) attention for gfx950: split-KV pass + LSE merge pass,
// dense and block-sparse.
//
// Replaces flash_attn_decoding_kernel / flash_attn_decoding_correction_kernel
// of flash_attn_triton/flash_attn_decoding.py:9-122,:126-210 and their sparse
// twins in flash_attn_triton/flash_attn_decoding_sparse.py:10-127,:131-219.
//
// Pass 1: a work item is a (chunk, kv-head, sequence) triple and is handled
// by one wavefront (= one workgroup).  The block-list form launches one
// wavefront per item; the dense form launches one resident round of wavefronts
// (8 per CU) and deals the live chunks of a ragged batch to them round-robin.
// The G = hq/hkv query heads that share the kv-head sit in the first G of the 32
// query columns of the same S^T = K.Q^T / O^T = V^T.P^T MFMA pipeline the
// prefill kernel uses, so each K/V byte is fetched once for the whole group
// (the reference launches one program per q-head and re-reads KV G times,
// flash_attn_decoding.py:42-45,264-268) and the dot products cost no VALU
// work.  A group of more than 32 heads is split into slices of 32, each a work
// item of its own: KV is then fetched once per slice.  KV streams global -> registers -> wave-private LDS in 32-key tiles
// with fully coalesced 16-byte loads (non-temporal: every byte is used once);
// as soon as a tile has arrived, each register is written to LDS and refilled
// with its part of the tile after next.  No barriers are needed because a
// single wave's LDS operations execute in order.  Partials are fp32 (the reference
// rounds them to the input dtype, :249-251).
// Pass 2: per (sequence, q-head) merge  o = sum_c o_c 2^(lse_c - lse).
#include <atomic>

#include "kernels.h"
#include "tile_core.h"

// Split-KV partials of mi_decode_noalloc: device memory the library holds from
// load time on, one copy per GPU.  Host code must not use this name as an
// address (it is a host-side stand-in); decode_static_scratch() below asks the
// runtime for the device address, per device, and everything else uses that.
static __device__ __align__(256) unsigned char scratch[mi::kDecodeScratchBytes];

namespace mi {
namespace {

constexpr int kDecTile = 32;

// The block list of the window form, which is arithmetic: the blocks of the
// first `wg` tokens (entries 0 .. n_sink-1), then the blocks from token
// max(len - wl, 0) to the last one (entries n_sink .. cnt-1, starting at block
// tail0), every block once.
struct WindowList {
  int n_sink, tail0, cnt;
  __device__ __forceinline__ int block(int e) const { return e < n_sink ? e : tail0 + (e - n_sink); }
};
__device__ __forceinline__ WindowList window_list(int len, int wg, int wl) {
  const int nblk = (len + 63) / 64;
  WindowList w;
  w.n_sink = min((wg + 63) / 64, nblk);
  w.tail0 = max(max(len - wl, 0) / 64, w.n_sink);
  w.cnt = w.n_sink + max(nblk - w.tail0, 0);
  return w;
}

// One work item: chunk `split` of (sequence b, kv-head kvh) for the 32 query
// heads of the group that start at head g0 of it (slice kvs % gslices; a group
// of up to 32 heads is one slice).
template <typename T, int D>
__device__ __forceinline__ void decode_item(const DecodeParams& p, unsigned char* smem, const int split, const int kvs,
                                            const int b) {
  const int kvh = kvs / p.gslices;
  const int g0 = (kvs % p.gslices) * 32;
  using G = RowGeom<D>;
  using F = PaddedFrags<D>;
  constexpr int KTILEB = kDecTile * F::KROWB;
  constexpr int NCHUNK = kDecTile * G::NCH;
  constexpr int LOADS = (NCHUNK + 63) / 64;

  unsigned char* sK = smem;
  unsigned char* sV = smem + KTILEB;

  const int lane = threadIdx.x;
  const int len = p.seq_lens ? p.seq_lens[b] : p.cu[b + 1] - p.cu[b];
  const int gqa_all = p.hq / p.hkv;
  const int gqa = min(32, gqa_all - g0);  // query heads of this slice
  const bool sparse = p.list_mode != 0;
  const bool derived = p.list_mode == 2;

  int n_tiles, t_begin = 0;
  const int32_t* blist = nullptr;
  WindowList wlist = {0, 0, 0};
  int n_listed = 0;  // listed entries that fall into this chunk
  int b0 = 0;        // first entry of this chunk
  const int last_blk = (len - 1) / 64;
  if (sparse) {
    int cnt;
    if (derived) {
      wlist = window_list(len, p.win_global, p.win_local);
      cnt = min(wlist.cnt, p.max_blocks);
    } else {
      cnt = p.block_cnt ? min(p.block_cnt[b * p.hkv + kvh], p.max_blocks) : p.max_blocks;
    }
    const int total = cnt + p.add_last;  // the implicit last block sits behind the list
    b0 = split * p.split_blocks;
    if (b0 >= total || len <= 0) return;
    if (!derived) blist = p.block_idx + b * p.bi_sb + kvh * p.bi_sh + b0;
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
    const int blk = e < n_listed ? (derived ? wlist.block(b0 + e) : blist[e]) : last_blk;
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
                  (int64_t)(kvh * gqa_all + g0 + min(lc.lq, gqa - 1)) * p.q_sh + 8 * lc.lh;
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
  const uint32_t k_rowb = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(p.k_ss * 2));
  const uint32_t v_rowb = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(p.v_ss * 2));
  // reg <- chunk (lane + 64 i) of the tile at `tile` (uniform address of its
  // first row); rows beyond row_max re-read row row_max (the last token: same
  // tile, hence same page)
  auto load_one = [&](i32x4& reg, int i, uint64_t tile, int row_max, uint32_t rowb, uint32_t step,
                      uint32_t lane_off) __attribute__((always_inline)) {
    const int idx = lane + i * 64;
    if (NCHUNK % 64 != 0 && idx >= NCHUNK) return;
    if (kUniformRows && row_max >= kDecTile - 1) {
      reg = __builtin_nontemporal_load((g_i32x4*)(scalar_ptr(tile + (uint64_t)i * step) + lane_off));
    } else {
      const int row = idx / G::NCH, ch = idx % G::NCH;
      const uint32_t off = (uint32_t)min(row, row_max) * rowb + ch * 16;
      reg = __builtin_nontemporal_load((g_i32x4*)(scalar_ptr(tile) + off));
    }
  };
  auto store_one = [&](int i) __attribute__((always_inline)) {
    const int idx = lane + i * 64;
    if (NCHUNK % 64 != 0 && idx >= NCHUNK) return;
    const int row = idx / G::NCH, ch = idx % G::NCH;
    F::store_k(sK, row, ch, kreg[i]);
    F::store_v(sV, row, ch, vreg[i]);
  };
  // where a tile comes from: uniform addresses of its first K / V row and the
  // last row that may be read
  struct TileSrc {
    uint64_t k, v;
    int row_max;
  };
  auto tile_src = [&](int base) __attribute__((always_inline)) -> TileSrc {
    const int tb = addr_base(base);
    TileSrc t;
    t.k = uniform64((uint64_t)(uintptr_t)(kp + page_shift(tb, p.k_sb, p.k_ss) + (int64_t)tb * p.k_ss));
    t.v = uniform64((uint64_t)(uintptr_t)(vp + page_shift(tb, p.v_sb, p.v_ss) + (int64_t)tb * p.v_ss));
    t.row_max = len - 1 - tb;
    return t;
  };
  auto load_pair = [&](int i, const TileSrc& t) __attribute__((always_inline)) {
    load_one(kreg[i], i, t.k, t.row_max, k_rowb, k_step, k_lane);
    load_one(vreg[i], i, t.v, t.row_max, v_rowb, v_step, v_lane);
  };

  const int wl = p.win_local, wg = p.win_global;
  // Tile t is worked on from LDS while tile t + 1 is in flight into the
  // registers.  When it has arrived, every register is written to LDS and
  // refilled at once with its part of tile t + 2, so that the next loads leave
  // as early as possible; the address of tile t + 2 (block list and page
  // look-ups) is prepared before tile t is worked on.
  int base_cur = tile_base(0);
  {
    const TileSrc t0 = tile_src(base_cur);
#pragma unroll
    for (int i = 0; i < LOADS; ++i) load_pair(i, t0);
  }
  int base_nxt = n_tiles > 1 ? tile_base(1) : 0;
  TileSrc src = tile_src(base_nxt);  // tile 1, then the tile two ahead of the compute
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    store_one(i);
    if (n_tiles > 1) load_pair(i, src);
  }
  for (int it = 0; it < n_tiles; ++it) {
    const int base = base_cur;
    base_cur = base_nxt;
    const bool refill = it + 2 < n_tiles;
    if (refill) {
      base_nxt = tile_base(it + 2);
      src = tile_src(base_nxt);
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
    if (it + 1 < n_tiles) {
#pragma unroll
      for (int i = 0; i < LOADS; ++i) {
        store_one(i);
        if (refill) load_pair(i, src);
      }
    }
  }

  const float l_tot = sum_with_other_half(l);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (lc.lq < gqa) {
    const int h = kvh * gqa_all + g0 + lc.lq;
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

// Block-list form: one wavefront per (chunk, kv-head, sequence), grid
// (n_splits, hkv, batch).  Dense form: the live chunks of all sequences (a
// sequence of length L has ceil(L / split_tokens) of them) are numbered
// consecutively and dealt round-robin to gridDim.x wavefronts, one resident
// round of the chip, so that ragged batches leave no tail of half-empty rounds:
// every wavefront gets the same number of chunks, give or take one.
template <typename T, int D>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2)))
decode_splitkv_kernel(const DecodeParams p) {
  using F = PaddedFrags<D>;
  __shared__ __attribute__((aligned(16))) unsigned char smem[kDecTile * (F::KROWB + F::VROWB)];
  if (p.list_mode != 0) {
    decode_item<T, D>(p, smem, blockIdx.x, blockIdx.y, blockIdx.z);
    return;
  }
  const int lane = threadIdx.x;
  auto chunks_of = [&](int b) -> int {
    if (b >= p.batch) return 0;
    const int len = p.seq_lens ? p.seq_lens[b] : p.cu[b + 1] - p.cu[b];
    return max(0, min((len + p.split_tokens - 1) / p.split_tokens, p.n_splits));
  };
  // chunks of all sequences (wave-wide sum, 64 sequences per step)
  int total = 0;
  for (int b0 = 0; b0 < p.batch; b0 += 64) {
    int c = chunks_of(b0 + lane);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) c += __shfl_xor(c, m, 64);
    total += c;
  }
  total = __builtin_amdgcn_readfirstlane(total);
  const int kv_slices = p.hkv * p.gslices;  // (kv-head, 32-head slice of its group) pairs
  const long long items = (long long)total * kv_slices;
  for (long long g = blockIdx.x; g < items; g += gridDim.x) {
    const int t = (int)(g / kv_slices), kvh = (int)(g % kv_slices);
    // sequence that owns live chunk t: inclusive scan over the chunk counts
    int b = 0, first = 0;
    for (int b0 = 0, seen = 0; b0 < p.batch; b0 += 64) {
      const int c = chunks_of(b0 + lane);
      int incl = c;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
      }
      const int before = seen + incl - c;  // live chunks ahead of this lane's sequence
      const unsigned long long hit = __builtin_amdgcn_ballot_w64(c > 0 && t >= before && t < before + c);
      if (hit) {
        const int src = __builtin_ctzll(hit);
        b = b0 + src;
        first = __shfl(before, src, 64);
        break;
      }
      seen += __shfl(incl, 63, 64);
    }
    b = __builtin_amdgcn_readfirstlane(b);
    first = __builtin_amdgcn_readfirstlane(first);
    decode_item<T, D>(p, smem, t - first, kvh, b);
  }
}

template <typename T>
__global__ void __launch_bounds__(128)
decode_merge_kernel(const DecodeParams p, int D) {
  const int h = blockIdx.x, b = blockIdx.y;
  const int d = threadIdx.x;
  const int len = p.seq_lens ? p.seq_lens[b] : p.cu[b + 1] - p.cu[b];
  int nvalid;
  if (p.list_mode != 0) {
    const int kvh = h / (p.hq / p.hkv);
    int cnt;
    if (p.list_mode == 2)
      cnt = min(window_list(len, p.win_global, p.win_local).cnt, p.max_blocks);
    else
      cnt = p.block_cnt ? min(p.block_cnt[b * p.hkv + kvh], p.max_blocks) : p.max_blocks;
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
  dim3 grid(p.n_splits, p.hkv * p.gslices, p.batch);
  if (p.list_mode == 0) {
    // dense: one resident round (8 wavefronts per CU), fewer when there are fewer chunks
    const long long slots = (long long)p.n_splits * p.hkv * p.gslices * p.batch;
    const int cus = device_cu_count();
    const long long resident = 8LL * (cus > 0 ? cus : 256);
    grid = dim3((unsigned)(slots < resident ? slots : resident), 1, 1);
  }
  hipLaunchKernelGGL((decode_splitkv_kernel<T, D>), grid, dim3(64), 0, s, p);
  return (int)hipGetLastError();
}

}  // namespace

// Device address of `scratch` on the current device.  Looked up once per device
// with that device current (each GPU holds its own copy at its own address);
// the lookup allocates nothing.  Two threads racing on the first call both
// look it up and store the same value.
int decode_static_scratch(void** ptr) {
  constexpr int kMaxDev = 64;
  static std::atomic<void*> addr[kMaxDev];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDev) return (int)hipErrorInvalidDevice;
  void* a = addr[dev].load(std::memory_order_acquire);
  if (a == nullptr) {
    e = hipGetSymbolAddress(&a, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (a == nullptr) return (int)hipErrorInvalidSymbol;
    addr[dev].store(a, std::memory_order_release);
  }
  *ptr = a;
  return (int)hipSuccess;
}

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
