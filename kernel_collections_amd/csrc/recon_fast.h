// Interface between the recon stage-1 dispatcher and its MFMA-bound fast paths (recon_fast_*.hip, recon_duo_*.hip).
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

// The 4-wave kernel (recon_fast_impl.h): scores only, or the key basis reused as the value basis.  Instantiated at rank 256,
// where its scores-only form fits a CU twice.
int launch_recon_fast_256(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                          hipStream_t st);
// The wave-specialised 8-wave kernel (recon_spec_impl.h), one translation unit per key rank: the same shapes and arguments.
int launch_recon_spec_512(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                          hipStream_t st);
int launch_recon_spec_384(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                          hipStream_t st);
int launch_recon_spec_256(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                          hipStream_t st);
inline int launch_recon_spec(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                             int rank, hipStream_t st) {
  return rank == 512   ? launch_recon_spec_512(p, kB, sBb, sBh, sBr, batch, dtype, st)
         : rank == 384 ? launch_recon_spec_384(p, kB, sBb, sBh, sBr, batch, dtype, st)
                       : launch_recon_spec_256(p, kB, sBb, sBh, sBr, batch, dtype, st);
}

// The 8-wave kernels (recon_duo_impl.h) for key ranks 256 / 384 / 512 with a separate value basis of rank rv (mode 2; the
// kernel template also has a scores-only mode 0 and a shared-basis mode 1, which the 4-wave kernel above now serves).  Each
// translation unit serves the shapes it instantiates and returns DUO_NOT_MINE for the others.
constexpr int DUO_NOT_MINE = -1000;
int launch_recon_duo_b(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                       int mode, int rk, int rv, hipStream_t st);
int launch_recon_duo_c(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                       int mode, int rk, int rv, hipStream_t st);

}  // namespace xkv
