// Shared device helpers for the xKV decode kernels (gfx950 / CDNA4 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>

#include "../../include/xkv_hip.h"

namespace xkv {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16;

constexpr int WAVE = 64;
constexpr int MIN_BLOCK_KV = 32;  // split granularity, flash_decoding/gqa.py:38 of the reference
constexpr float NEG_INF = -__builtin_huge_valf();

// 16-bit operand type traits.  A "packet" is 8 consecutive elements = 16 bytes =
// one lane's share of a 16x16x32 (or 32x32x16) MFMA operand.
template <typename T> struct Elem;
template <> struct Elem<__bf16> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Elem<_Float16> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

template <typename T> __device__ __forceinline__ float to_f32(T x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f32(float x) { return (T)x; }

// The reconstruction kernels hand the rotated key tile and the query to the q-dot MFMA as fp16 WHATEVER the operand type.
// The reference's kernels do the same (`.to(tl.float16)` before the dot, flash_recontruction/qAB/v1.py:73-74), and it
// matters for parity: a key rounded to bf16 (8 mantissa bits) puts ~1e-3 * |s| of noise on every score, which at
// sm_scale = 1 on unit-variance inputs (logit sigma 7 - 11, the reference scripts' regime) moves attention outputs by
// 3e-2 .. 9e-2; fp16's 11 bits keep that below 1e-2.  Like the reference this assumes |K'| and |q| stay below 65504.
typedef _Float16 sc_t;
typedef f16x8 sc_vec8;

__device__ __forceinline__ u16 bits_of(__bf16 x) { return __builtin_bit_cast(u16, x); }
__device__ __forceinline__ u16 bits_of(_Float16 x) { return __builtin_bit_cast(u16, x); }

// 16-byte packet load/store through a generic pointer (global or LDS)
template <typename V> __device__ __forceinline__ V ld16(const void* p) {
  return __builtin_bit_cast(V, *reinterpret_cast<const u32x4*>(p));
}
template <typename V> __device__ __forceinline__ void st16(void* p, V v) {
  *reinterpret_cast<u32x4*>(p) = __builtin_bit_cast(u32x4, v);
}

__host__ __device__ __forceinline__ int cdiv(int a, int b) { return (a + b - 1) / b; }

// Token range of one KV split; identical integer arithmetic to the reference's
// flash_decoding/gqa.py:95-99 (stage 1) and :273-281 (stage 2).
__host__ __device__ __forceinline__ void split_bounds(int kv_len, int num_splits, int split_id,
                                                       int& start, int& end) {
  int per = cdiv(cdiv(kv_len, num_splits), MIN_BLOCK_KV) * MIN_BLOCK_KV;
  start = per * split_id;
  int e = start + per;
  end = e < kv_len ? e : kv_len;
}

// Split count a sequence is scanned with: the caller's, or more when `cap_tokens` > 0 and the caller's splits would be longer
// than that (one split per cap_tokens tokens at least).  Stage 1 and the merge evaluate it from the same two device
// integers, so they agree without any exchange; split-K is exact under the merge, so the result does not depend on it.
__host__ __device__ __forceinline__ int effective_splits(int kv_len, int num_splits, int cap_tokens) {
  if (cap_tokens > 0) {
    const int need = cdiv(kv_len, cap_tokens);
    return need > num_splits ? need : num_splits;
  }
  return num_splits;
}

// The cap in force: the host's value, raised by the one a planning kernel left in the first word of its plan (if any).
__device__ __forceinline__ int split_cap_in_force(int cap_tokens, const int32_t* plan) {
  if (!plan) return cap_tokens;
  const int d = plan[0];
  return d > cap_tokens ? d : cap_tokens;
}

// Reductions over the 4 lane groups {n, n+16, n+32, n+48} that share a column
// index in the 16x16 MFMA result layout.
__device__ __forceinline__ float group4_max(float v) {
  v = fmaxf(v, __shfl_xor(v, 16));
  v = fmaxf(v, __shfl_xor(v, 32));
  return v;
}
__device__ __forceinline__ float group4_sum(float v) {
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 32);
  return v;
}

// max / sum over each aligned group of WIDTH (8 or 16) consecutive lanes, result in every lane of the group
// (DPP butterflies inside a 16-lane row: no LDS traffic, unlike __shfl_xor)
template <bool IS_MAX, int WIDTH> __device__ __forceinline__ float row_reduce(float x) {
  static_assert(WIDTH == 8 || WIDTH == 16, "row_reduce width");
#define XKV_DPP_STEP(ctrl)                                                                                       \
  {                                                                                                              \
    const float y = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), ctrl, 0xf, 0xf, false)); \
    x = IS_MAX ? fmaxf(x, y) : x + y;                                                                            \
  }
  XKV_DPP_STEP(0xB1)   // quad_perm [1,0,3,2]
  XKV_DPP_STEP(0x4E)   // quad_perm [2,3,0,1]
  XKV_DPP_STEP(0x141)  // row_half_mirror
  if (WIDTH == 16) XKV_DPP_STEP(0x140)  // row_mirror
#undef XKV_DPP_STEP
  return x;
}

// Workgroups are dealt round-robin over the 8 XCDs (one L2 each) by linear id.  `cluster` consecutive logical ids read the
// same token rows, so a cluster must sit on one XCD; the clusters themselves go round-robin over the XCDs, which keeps
// ragged batches (long and short sequences, dead splits) balanced across the chip.  Grid size: xcd_grid(total, cluster).
__device__ __forceinline__ int xcd_cluster_remap(int id, int cluster) {
  const int xcd = id & 7, j = id >> 3;
  return ((j / cluster) * 8 + xcd) * cluster + (j % cluster);
}
inline int xcd_grid(int total_wg, int cluster) { return ((total_wg / cluster + 7) & ~7) * cluster; }

// hipFuncSetAttribute costs host microseconds on every call: a launcher asks for a kernel's dynamic LDS size once per device
// (again only if a later call needs more).  One DynLds per kernel instantiation, as a function-local static.
struct DynLds {
  std::atomic<int> bytes[16];
  DynLds() { for (auto& b : bytes) b.store(0, std::memory_order_relaxed); }
};
// `hand_tracked`: the kernel issues loads in asm and tracks their completion by hand (s_waitcnt counts, registers that
// stay in flight across instructions).  That bookkeeping only holds while the compiler adds no memory traffic of its own to
// the kernel: a build whose register allocation spills (another compiler, other flags) is refused with XKV_ETOOLCHAIN
// instead of computing on stale registers.  Returns XKV_OK, XKV_ETOOLCHAIN or a positive hipError_t.
inline int ensure_dynamic_lds(DynLds& st, const void* kernel, int bytes, bool hand_tracked = false) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev >= 0 && dev < 16 && st.bytes[dev].load(std::memory_order_acquire) >= bytes) return XKV_OK;
  if (hand_tracked) {
    hipFuncAttributes attr;
    e = hipFuncGetAttributes(&attr, kernel);
    if (e != hipSuccess) return (int)e;
    if (attr.localSizeBytes != 0) return XKV_ETOOLCHAIN;
  }
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && dev >= 0 && dev < 16) st.bytes[dev].store(bytes, std::memory_order_release);
  return (int)e;
}

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? XKV_OK : (int)e;
}

}  // namespace xkv
