// RMSNorm forward and backward for gfx950 (HBM-bound).
//
// Replaces rmsnorm_fwd_kernel / rmsnorm_bwd_kernel of common/rms.py:8-88,
// :90-218 and their launchers in RMSNormTritonFunction (:221-355):
//   r_t  = 1 / sqrt(eps + mean_d x_td^2)          (saved, fp32, :67-68,88)
//   y_td = x_td * r_t * w_d                       (:81)
//   dx_td = dy_td w_d r_t - x_td r_t^3 (sum_d dy_td w_d x_td) / D   (:199-212)
//   dw_d  = sum_t dy_td x_td r_t                  (:213; the reference adds
//           per-tile sums with atomics, :215)
// A row is owned by one wavefront (short rows) or by the four wavefronts of a
// workgroup (long rows) and is read once, with 16-byte loads, into registers;
// the owners walk the rows with a fixed stride and request the next row before
// they work on the current one.  The backward pass keeps the dw sums of each
// thread's element positions in registers over all its rows; dw is reduced in
// two deterministic stages (every workgroup writes one fp32 partial row, a
// second kernel adds the partial rows).  Rows that cannot be read in 16-byte
// chunks (dim not a multiple of the chunk, unaligned rows, more than 4096
// chunks) take an element-wise path with one partial row per wavefront.
#include <type_traits>

#include "kernels.h"
#include "tile_core.h"

namespace mi {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

// element type tags: 0 bf16, 1 f16, 2 f32
constexpr int kMaxJ = 16;  // 16-byte chunks a lane keeps in registers per row

// EPC elements per 16-byte chunk
template <typename T>
struct Chunk {
  static constexpr int EPC = 16 / sizeof(T);
  i32x4 raw;
  __device__ __forceinline__ float at(int e) const { return (float)reinterpret_cast<const T*>(&raw)[e]; }
  __device__ __forceinline__ void set(int e, float v) { reinterpret_cast<T*>(&raw)[e] = (T)v; }
};

// One row's 16-byte chunks of a thread: chunk j is row chunk t + GROUP*j, where
// GROUP threads (one wavefront, or the four of a workgroup) share the row.
template <typename T, int J, int GROUP>
struct RowRegs {
  static constexpr int EPC = Chunk<T>::EPC;
  Chunk<T> c[J];
  // STREAM: the row is not read again soon (non-temporal hint)
  template <bool STREAM = false>
  __device__ __forceinline__ void load(const T* row, int t, int nch) {
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const int ch = t + GROUP * j;
      if (ch < nch) {
        const i32x4* src = reinterpret_cast<const i32x4*>(row + ch * EPC);
        c[j].raw = STREAM ? __builtin_nontemporal_load(src) : *src;
      }
    }
  }
};

// Sum over the GROUP threads that share a row.  WPR == 4: the wavefront sums
// meet in LDS; `xs` is double-buffered by row parity, so one barrier per row is
// enough (a wavefront can only overwrite a slot after every other wavefront
// has passed the barrier of the row in between).
template <int WPR>
__device__ __forceinline__ float group_sum(float v, float (*xs)[4], int& par, int wave, int lane) {
  v = wave_sum(v);
  if (WPR > 1) {
    if (lane == 0) xs[par][wave] = v;
    __syncthreads();
    v = (xs[par][0] + xs[par][1]) + (xs[par][2] + xs[par][3]);
    par ^= 1;
  }
  return v;
}

// ---------------------------------------------------------------- forward
// WPR wavefronts (1 or 4) own a row at a time and walk rows slot, slot +
// n_slots, ...; the next row is requested before the current one is reduced
// and scaled (J <= 8: two rows fit in registers).
template <typename T, typename TW, int J, int WPR>
__global__ void __launch_bounds__(256) rms_fwd_vec_kernel(const RmsParams p) {
  constexpr int EPC = Chunk<T>::EPC;
  constexpr int GROUP = 64 * WPR;
  constexpr bool PF = J <= 8;
  __shared__ float xs[2][4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t = WPR == 1 ? lane : (int)threadIdx.x;
  const int slot = WPR == 1 ? blockIdx.x * 4 + wave : (int)blockIdx.x;
  const int n_slots = WPR == 1 ? gridDim.x * 4 : (int)gridDim.x;
  const TW* w = reinterpret_cast<const TW*>(p.w);
  const int D = p.dim;
  const int nch = D / EPC;
  const T* xb = reinterpret_cast<const T*>(p.x);
  int par = 0;
  RowRegs<T, J, GROUP> cur, nxt;
  if (PF && slot < p.rows) cur.load(xb + (int64_t)slot * p.x_st, t, nch);
  for (int64_t row = slot; row < p.rows; row += n_slots) {
    if (PF) {
      if (row + n_slots < p.rows) nxt.load(xb + (row + n_slots) * p.x_st, t, nch);
    } else {
      cur.load(xb + row * p.x_st, t, nch);
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < J; ++j)
      if (t + GROUP * j < nch) {
#pragma unroll
        for (int e = 0; e < EPC; ++e) ss += cur.c[j].at(e) * cur.c[j].at(e);
      }
    ss = group_sum<WPR>(ss, xs, par, wave, lane);
    const float r = 1.0f / sqrtf(p.eps + ss / (float)D);
    T* y = reinterpret_cast<T*>(p.y) + row * p.y_st;
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const int ch = t + GROUP * j;
      if (ch < nch) {
        Chunk<T> o;
#pragma unroll
        for (int e = 0; e < EPC; ++e) o.set(e, cur.c[j].at(e) * r * (float)w[ch * EPC + e]);
        __builtin_nontemporal_store(o.raw, reinterpret_cast<i32x4*>(y + ch * EPC));
      }
    }
    if (t == 0) p.rsqrt[row] = r;
    if (PF) cur = nxt;
  }
}

// element-wise path: any dim, any alignment
template <typename T, typename TW>
__global__ void __launch_bounds__(256) rms_fwd_elem_kernel(const RmsParams p) {
  const int lane = threadIdx.x & 63;
  const int wid = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int n_waves = gridDim.x * 4;
  const TW* w = reinterpret_cast<const TW*>(p.w);
  const int D = p.dim;
  for (int64_t row = wid; row < p.rows; row += n_waves) {
    const T* x = reinterpret_cast<const T*>(p.x) + row * p.x_st;
    T* y = reinterpret_cast<T*>(p.y) + row * p.y_st;
    float ss = 0.f;
    for (int i = lane; i < D; i += 64) {
      const float v = (float)x[i];
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(p.eps + ss / (float)D);
    for (int i = lane; i < D; i += 64) y[i] = (T)((float)x[i] * r * (float)w[i]);
    if (lane == 0) p.rsqrt[row] = r;
  }
}

// --------------------------------------------------------------- backward
// WPR wavefronts (1 or 4) own a row at a time and walk rows slot, slot +
// n_slots, ...; every thread keeps the dw contributions of its element
// positions in registers and the workgroup writes ONE fp32 partial row (WPR ==
// 1: the four wavefronts cover the same positions and add theirs through LDS).
template <typename T, typename TW, int J, int WPR>
__global__ void __launch_bounds__(256) rms_bwd_vec_kernel(const RmsParams p) {
  constexpr int EPC = Chunk<T>::EPC;
  constexpr int GROUP = 64 * WPR;
  constexpr bool PF = J <= 4;  // two (x, dy) row pairs in registers
  __shared__ float xs[2][4];
  __shared__ float red[WPR == 1 ? 4 : 1][64][EPC + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t = WPR == 1 ? lane : (int)threadIdx.x;
  const int slot = WPR == 1 ? blockIdx.x * 4 + wave : (int)blockIdx.x;
  const int n_slots = WPR == 1 ? gridDim.x * 4 : (int)gridDim.x;
  const TW* w = reinterpret_cast<const TW*>(p.w);
  const int D = p.dim;
  const int nch = D / EPC;
  const T* xb = reinterpret_cast<const T*>(p.x);
  const T* db = reinterpret_cast<const T*>(p.dy);
  int par = 0;
  float dwacc[J][EPC];
#pragma unroll
  for (int j = 0; j < J; ++j)
#pragma unroll
    for (int e = 0; e < EPC; ++e) dwacc[j][e] = 0.f;
  RowRegs<T, J, GROUP> cx, cd, nx, nd;
  if (PF && slot < p.rows) {
    cx.template load<true>(xb + (int64_t)slot * p.x_st, t, nch);
    cd.template load<true>(db + (int64_t)slot * p.dy_st, t, nch);
  }
  for (int64_t row = slot; row < p.rows; row += n_slots) {
    if (PF) {
      if (row + n_slots < p.rows) {
        nx.template load<true>(xb + (row + n_slots) * p.x_st, t, nch);
        nd.template load<true>(db + (row + n_slots) * p.dy_st, t, nch);
      }
    } else {
      cx.template load<true>(xb + row * p.x_st, t, nch);
      cd.template load<true>(db + row * p.dy_st, t, nch);
    }
    T* dx = reinterpret_cast<T*>(p.dx) + row * p.dx_st;
    const float r = p.rsqrt[row];
    float dot = 0.f;
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const int ch = t + GROUP * j;
      if (ch < nch) {
#pragma unroll
        for (int e = 0; e < EPC; ++e) dot += cd.c[j].at(e) * (float)w[ch * EPC + e] * cx.c[j].at(e);
      }
    }
    dot = group_sum<WPR>(dot, xs, par, wave, lane);
    const float k = r * r * r * dot / (float)D;
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const int ch = t + GROUP * j;
      if (ch < nch) {
        Chunk<T> o;
#pragma unroll
        for (int e = 0; e < EPC; ++e) {
          const float xv = cx.c[j].at(e), dv = cd.c[j].at(e);
          o.set(e, dv * (float)w[ch * EPC + e] * r - xv * k);
          dwacc[j][e] += dv * xv * r;
        }
        __builtin_nontemporal_store(o.raw, reinterpret_cast<i32x4*>(dx + ch * EPC));
      }
    }
    if (PF) {
      cx = nx;
      cd = nd;
    }
  }
  float* part = p.dw_part + (int64_t)blockIdx.x * D;
  if (WPR > 1) {
    // every thread owns its positions of the workgroup's partial row
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const int ch = t + GROUP * j;
      if (ch < nch) {
#pragma unroll
        for (int e = 0; e < EPC; ++e) part[ch * EPC + e] = dwacc[j][e];
      }
    }
  } else {
    // the four wavefronts cover the same positions: add through LDS, one chunk position at a time
#pragma unroll
    for (int j = 0; j < J; ++j) {
#pragma unroll
      for (int e = 0; e < EPC; ++e) red[wave][lane][e] = dwacc[j][e];
      __syncthreads();
      if (wave == 0) {
        const int ch = lane + 64 * j;
        if (ch < nch) {
#pragma unroll
          for (int e = 0; e < EPC; ++e)
            part[ch * EPC + e] = red[0][lane][e] + red[1][lane][e] + red[2][lane][e] + red[3][lane][e];
        }
      }
      __syncthreads();
    }
  }
}

// element-wise path: any dim, any alignment
template <typename T, typename TW>
__global__ void __launch_bounds__(256) rms_bwd_elem_kernel(const RmsParams p) {
  const int lane = threadIdx.x & 63;
  const int wid = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int n_waves = gridDim.x * 4;
  const TW* w = reinterpret_cast<const TW*>(p.w);
  const int D = p.dim;
  float* part = p.dw_part + (int64_t)wid * D;
  for (int i = lane; i < D; i += 64) part[i] = 0.f;
  for (int64_t row = wid; row < p.rows; row += n_waves) {
    const T* x = reinterpret_cast<const T*>(p.x) + row * p.x_st;
    const T* dy = reinterpret_cast<const T*>(p.dy) + row * p.dy_st;
    T* dx = reinterpret_cast<T*>(p.dx) + row * p.dx_st;
    const float r = p.rsqrt[row];
    float dot = 0.f;
    for (int i = lane; i < D; i += 64) dot += (float)dy[i] * (float)w[i] * (float)x[i];
    dot = wave_sum(dot);
    const float k = r * r * r * dot / (float)D;
    for (int i = lane; i < D; i += 64) {
      const float xv = (float)x[i], dv = (float)dy[i];
      dx[i] = (T)(dv * (float)w[i] * r - xv * k);
      part[i] += dv * xv * r;  // element i of the partial row belongs to lane i % 64 alone
    }
  }
}

// First stage of the dw sum: out[y][d] = sum of the rows i = y (mod gridDim.y)
// of in[n_in][D].  A workgroup covers 64 x V columns with 4 row slices.
template <int V>
__global__ void __launch_bounds__(256) rms_dw_stage_kernel(const float* in, float* out, int n_in, int D) {
  __shared__ float red[4][64][V + 1];
  const int lane = threadIdx.x & 63, slice = threadIdx.x >> 6;
  const int col = (blockIdx.x * 64 + lane) * V;
  float acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = 0.f;
  if (col < D) {
    for (int i = blockIdx.y + gridDim.y * slice; i < n_in; i += gridDim.y * 4) {
      const float* src = in + (int64_t)i * D + col;
      if (V == 4) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(src);
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] += v[e];
      } else {
        acc[0] += src[0];
      }
    }
  }
#pragma unroll
  for (int e = 0; e < V; ++e) red[slice][lane][e] = acc[e];
  __syncthreads();
  if (slice == 0 && col < D) {
#pragma unroll
    for (int e = 0; e < V; ++e)
      out[(int64_t)blockIdx.y * D + col + e] = (red[0][lane][e] + red[1][lane][e]) + (red[2][lane][e] + red[3][lane][e]);
  }
}

// Last stage: dw[d] = sum of in[n_in][D] over the rows, 64 columns x 4 row slices per workgroup
template <typename TW>
__global__ void __launch_bounds__(256) rms_dw_reduce_kernel(const float* in, TW* dw, int n_in, int D) {
  __shared__ float red[4][64];
  const int col = threadIdx.x & 63, slice = threadIdx.x >> 6;
  const int d = blockIdx.x * 64 + col;
  float s = 0.f;
  if (d < D)
    for (int i = slice; i < n_in; i += 4) s += in[(int64_t)i * D + d];
  red[slice][col] = s;
  __syncthreads();
  if (slice == 0 && d < D) dw[d] = (TW)((red[0][col] + red[1][col]) + (red[2][col] + red[3][col]));
}

// Adds n_parts partial rows at p.dw_part into p.dw; more than kStageRows of
// them go through kStageRows intermediate rows kept behind the `max_parts`
// rows of the workspace.
template <typename TW>
int reduce_dw(const RmsParams& p, int n_parts, int max_parts, hipStream_t s) {
  const float* in = p.dw_part;
  if (n_parts > kRmsStageRows) {
    float* mid = p.dw_part + (int64_t)max_parts * p.dim;
    const bool v4 = p.dim % 4 == 0 && reinterpret_cast<uintptr_t>(p.dw_part) % 16 == 0;
    const dim3 grid((unsigned)((p.dim + (v4 ? 255 : 63)) / (v4 ? 256 : 64)), kRmsStageRows);
    if (v4)
      hipLaunchKernelGGL((rms_dw_stage_kernel<4>), grid, dim3(256), 0, s, in, mid, n_parts, p.dim);
    else
      hipLaunchKernelGGL((rms_dw_stage_kernel<1>), grid, dim3(256), 0, s, in, mid, n_parts, p.dim);
    int rc = (int)hipGetLastError();
    if (rc) return rc;
    in = mid;
    n_parts = kRmsStageRows;
  }
  hipLaunchKernelGGL((rms_dw_reduce_kernel<TW>), dim3((unsigned)((p.dim + 63) / 64)), dim3(256), 0, s, in,
                     reinterpret_cast<TW*>(p.dw), n_parts, p.dim);
  return (int)hipGetLastError();
}

// Shape of the 16-byte path: rows of up to 128 chunks are owned by one
// wavefront (1 or 2 chunks per lane), longer ones by a workgroup of four.
constexpr int kWaveRowChunks = 128;
constexpr int kMaxRowWorkgroups = 1024;

template <typename F>
void by_shape(int nch, F&& f) {
  using std::integral_constant;
  if (nch <= 64)
    f(integral_constant<int, 1>{}, integral_constant<int, 1>{});
  else if (nch <= kWaveRowChunks)
    f(integral_constant<int, 2>{}, integral_constant<int, 1>{});
  else if (nch <= 256)
    f(integral_constant<int, 1>{}, integral_constant<int, 4>{});
  else if (nch <= 512)
    f(integral_constant<int, 2>{}, integral_constant<int, 4>{});
  else if (nch <= 1024)
    f(integral_constant<int, 4>{}, integral_constant<int, 4>{});
  else if (nch <= 2048)
    f(integral_constant<int, 8>{}, integral_constant<int, 4>{});
  else
    f(integral_constant<int, kMaxJ>{}, integral_constant<int, 4>{});
}

// workgroups of the 16-byte path (= partial dw rows of the backward pass)
inline unsigned vec_grid(const RmsParams& p, int nch, int n_waves) {
  if (nch <= kWaveRowChunks) return (unsigned)(n_waves / 4);
  return (unsigned)(p.rows < kMaxRowWorkgroups ? p.rows : kMaxRowWorkgroups);
}

template <typename T, typename TW>
int launch_fwd_t(const RmsParams& p, bool vec, int n_waves, hipStream_t s) {
  if (vec) {
    const int nch = p.dim / Chunk<T>::EPC;
    by_shape(nch, [&](auto jc, auto wc) {
      hipLaunchKernelGGL((rms_fwd_vec_kernel<T, TW, decltype(jc)::value, decltype(wc)::value>),
                         dim3(vec_grid(p, nch, n_waves)), dim3(256), 0, s, p);
    });
  } else {
    hipLaunchKernelGGL((rms_fwd_elem_kernel<T, TW>), dim3((unsigned)(n_waves / 4)), dim3(256), 0, s, p);
  }
  return (int)hipGetLastError();
}

// Partial dw rows: one per workgroup (16-byte path) or one per wavefront; never more than n_waves.
template <typename T, typename TW>
int launch_bwd_t(const RmsParams& p, bool vec, int n_waves, hipStream_t s) {
  int n_parts = n_waves;
  if (vec) {
    const int nch = p.dim / Chunk<T>::EPC;
    const unsigned grid = vec_grid(p, nch, n_waves);
    n_parts = (int)grid;
    by_shape(nch, [&](auto jc, auto wc) {
      hipLaunchKernelGGL((rms_bwd_vec_kernel<T, TW, decltype(jc)::value, decltype(wc)::value>), dim3(grid),
                         dim3(256), 0, s, p);
    });
  } else {
    hipLaunchKernelGGL((rms_bwd_elem_kernel<T, TW>), dim3((unsigned)(n_waves / 4)), dim3(256), 0, s, p);
  }
  int rc = (int)hipGetLastError();
  if (rc) return rc;
  return reduce_dw<TW>(p, n_parts, n_waves, s);
}

template <typename F>
int dispatch2(int xt, int wt, F&& f) {
  // w is either of x's type or fp32 (an fp32 parameter under 16-bit activations)
  if (xt == 0) return wt == 0 ? f((__bf16*)nullptr, (__bf16*)nullptr) : f((__bf16*)nullptr, (float*)nullptr);
  if (xt == 1) return wt == 1 ? f((_Float16*)nullptr, (_Float16*)nullptr) : f((_Float16*)nullptr, (float*)nullptr);
  return f((float*)nullptr, (float*)nullptr);
}

}  // namespace

int rms_partial_rows(long long rows, int num_cus) {
  // wavefronts of a pass (and upper bound of the partial dw rows): enough to
  // fill the chip (16 wavefronts per CU), never more than one per row, a multiple of 4
  long long w = (long long)(num_cus > 0 ? num_cus : 256) * 16;
  if (w > rows) w = rows;
  w = (w + 3) / 4 * 4;
  return (int)(w < 4 ? 4 : w);
}

int launch_rms_fwd(const RmsParams& p, int x_dtype, int w_dtype, bool vec, int n_waves, hipStream_t s) {
  return dispatch2(x_dtype, w_dtype, [&](auto* tx, auto* tw) {
    using T = std::remove_pointer_t<decltype(tx)>;
    using TW = std::remove_pointer_t<decltype(tw)>;
    return launch_fwd_t<T, TW>(p, vec, n_waves, s);
  });
}

int launch_rms_bwd(const RmsParams& p, int x_dtype, int w_dtype, bool vec, int n_waves, hipStream_t s) {
  return dispatch2(x_dtype, w_dtype, [&](auto* tx, auto* tw) {
    using T = std::remove_pointer_t<decltype(tx)>;
    using TW = std::remove_pointer_t<decltype(tw)>;
    return launch_bwd_t<T, TW>(p, vec, n_waves, s);
  });
}

}  // namespace mi
