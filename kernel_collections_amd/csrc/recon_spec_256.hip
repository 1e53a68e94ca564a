// The wave-specialised fused RoPE reconstruction kernel (recon_spec_impl.h) at rank 256.
#include "recon_spec_impl.h"

namespace xkv {

int launch_recon_spec_256(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                          hipStream_t st) {
  return spec::launch_recon_spec_rank<256>(p, kB, sBb, sBh, sBr, batch, dtype, st);
}

}  // namespace xkv
