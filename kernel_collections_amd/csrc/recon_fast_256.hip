// The 4-wave fused RoPE reconstruction kernel (recon_fast_impl.h) at rank 256.
#include "recon_fast_impl.h"

namespace xkv {

int launch_recon_fast_256(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                          hipStream_t st) {
  return fast::launch_recon_fast_rank<256>(p, kB, sBb, sBh, sBr, batch, dtype, st);
}

}  // namespace xkv
