// Timing helper for benchmarks (include/mi_attn_bench.h).  Kept out of api.cpp:
// it is the one exported call that creates HIP events and blocks.
#include <hip/hip_runtime.h>

#include "../../include/mi_attn_bench.h"
#include "kernels.h"

extern "C" int mi_time_launches(int kind, const void* args, int n_args, size_t arg_stride, void* stream, int warmup,
                                int iters, float* ms_per_launch) {
  if (!args || !ms_per_launch) return mi::set_error(MI_ERR_NULL_POINTER, "mi_time_launches: args and ms_per_launch must be non-NULL");
  if (n_args <= 0 || iters <= 0 || warmup < 0 || kind < 0 || kind > 11)
    return mi::set_error(MI_ERR_SHAPE, "mi_time_launches: n_args and iters must be positive, warmup >= 0, kind in [0, 11]");
  const char* base = static_cast<const char*>(args);
  int n = 0;
  auto once = [&]() -> int {
    const void* a = base + (size_t)(n++ % n_args) * arg_stride;
    switch (kind) {
      case 0: return mi_attn_fwd(static_cast<const mi_attn_fwd_args*>(a), stream);
      case 1: return mi_attn_fwd_blocksparse(static_cast<const mi_attn_sparse_args*>(a), stream);
      case 2: return mi_decode(static_cast<const mi_decode_args*>(a), stream);
      case 3: return mi_decode_splitkv(static_cast<const mi_decode_args*>(a), stream);
      case 4: return mi_decode_merge(static_cast<const mi_decode_args*>(a), stream);
      case 5: return mi_attn_bwd(static_cast<const mi_attn_bwd_args*>(a), stream);
      case 6: return mi_rmsnorm_fwd(static_cast<const mi_rmsnorm_args*>(a), stream);
      case 7: return mi_rmsnorm_bwd(static_cast<const mi_rmsnorm_args*>(a), stream);
      case 8: return mi_xent_fwd(static_cast<const mi_xent_args*>(a), stream);
      case 9: return mi_xent_dlogits(static_cast<const mi_xent_grad_args*>(a), stream);
      case 10: return mi_xent_bwd_dlogits(static_cast<const mi_xent_bwd_args*>(a), stream);
      default: return mi_decode_noalloc(static_cast<const mi_decode_args*>(a), stream);
    }
  };
  hipStream_t s = static_cast<hipStream_t>(stream);
  for (int i = 0; i < warmup; ++i) {
    const int rc = once();
    if (rc) return rc;
  }
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess) return mi::set_error(MI_ERR_NO_DEVICE, "mi_time_launches: hipEventCreate failed");
  if (hipEventCreate(&e1) != hipSuccess) {
    (void)hipEventDestroy(e0);
    return mi::set_error(MI_ERR_NO_DEVICE, "mi_time_launches: hipEventCreate failed");
  }
  int rc = MI_OK;
  (void)hipEventRecord(e0, s);
  for (int i = 0; i < iters && rc == MI_OK; ++i) rc = once();
  (void)hipEventRecord(e1, s);
  hipError_t e = hipEventSynchronize(e1);
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc) return rc;  // the entry point that failed has set the message
  if (e != hipSuccess) return mi::set_error(MI_ERR_LAUNCH, hipGetErrorString(e));
  *ms_per_launch = ms / iters;
  return MI_OK;
}
