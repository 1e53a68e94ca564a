// Shapes of the 8-wave fused RoPE reconstruction kernel built in this translation unit: scores only at rank 384, shared key / value basis at ranks 384 and 256.
#include "recon_duo_impl.h"

namespace xkv {

int launch_recon_duo_a(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                       int mode, int rk, int rv, hipStream_t st) {
  using namespace duo;
#define XKV_DUO_CASE(MODE, RK, RV) \
  if (mode == MODE && rk == RK && (MODE != DUO_VDISTINCT || rv == RV)) return launch_duo<RK, RV, MODE>(p, kB, sBb, sBh, sBr, batch, dtype, st);
  XKV_DUO_CASE(DUO_SCORES, 384, 384)   // at rank 256 the register-staged kernel is the faster scores kernel
  XKV_DUO_CASE(DUO_VSHARED, 384, 384) XKV_DUO_CASE(DUO_VSHARED, 256, 256)
#undef XKV_DUO_CASE
  return DUO_NOT_MINE;
}

}  // namespace xkv
