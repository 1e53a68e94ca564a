// Shapes of the 8-wave fused RoPE reconstruction kernel built in this translation unit: separate value basis, key rank / value rank 256 / 256, 256 / 512.
#include "recon_duo_impl.h"

namespace xkv {

int launch_recon_duo_c(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                       int mode, int rk, int rv, hipStream_t st) {
  using namespace duo;
#define XKV_DUO_CASE(MODE, RK, RV) \
  if (mode == MODE && rk == RK && (MODE != DUO_VDISTINCT || rv == RV)) return launch_duo<RK, RV, MODE>(p, kB, sBb, sBh, sBr, batch, dtype, st);
  XKV_DUO_CASE(DUO_VDISTINCT, 256, 256) XKV_DUO_CASE(DUO_VDISTINCT, 256, 512)
#undef XKV_DUO_CASE
  return DUO_NOT_MINE;
}

}  // namespace xkv
