// Interface between the recon stage-1 dispatcher and its MFMA-bound fast path (recon_fast.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace xkv {

struct FastParams {
  const void* q; const void* kA; const void* Bp;   // Bp: kB re-packed into MFMA operand order (caller workspace)
  int64_t sAb, sAl, sBpb;
  float* partial; float* lse;
  void* scores; int scores_dtype;               // scores != NULL: write [batch, hq, kv_len] scaled scores, no softmax / P.A
  const int32_t* num_splits; const int32_t* kv_lens;
  int hq, hkv, kv_len, max_splits, total_wg;
  float sm_scale;
  const float* inv_freq; int64_t pos_offset;
  const void* vA; int64_t sVb, sVl;             // separate value basis (recon_duo kernels only)
};

int launch_recon_fast(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                      hipStream_t st);

// The 8-wave kernels (recon_duo_impl.h) for key ranks 256 / 384 / 512 with scores only (mode 0), the key basis reused as
// the value basis (mode 1) or a separate value basis of rank rv (mode 2).  Each translation unit serves the shapes it
// instantiates and returns DUO_NOT_MINE for the others.
constexpr int DUO_NOT_MINE = -1000;
int launch_recon_duo_a(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                       int mode, int rk, int rv, hipStream_t st);
int launch_recon_duo_b(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                       int mode, int rk, int rv, hipStream_t st);
int launch_recon_duo_c(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                       int mode, int rk, int rv, hipStream_t st);

}  // namespace xkv
