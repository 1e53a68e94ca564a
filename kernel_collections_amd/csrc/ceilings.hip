// Measurement and test aids, not part of the decode path.  Two ceilings: what this GPU sustains with NOTHING but the instruction a
// kernel is bound by.  (1) v_mfma_f32_32x32x16 on register operands, every wave of every CU; (2) an HBM read
// stream, into registers or straight into LDS (global_load_lds_dwordx4), with no use of the data.  The scan and
// reconstruction kernels are judged against the published peaks; these two figures say how much of the distance
// to those peaks any kernel on this part could close.
#include "xkv_common.h"

namespace xkv {

// ---- (1) matrix pipe ---------------------------------------------------------------------------------------------
// 4 independent accumulator chains per wave so that back-to-back MFMAs never wait for a result.
template <typename T>
__global__ __launch_bounds__(256) void ceiling_mfma_kernel(float* __restrict__ out, int iters) {
  typedef typename Elem<T>::vec8 vec8;
  const int lane = threadIdx.x & 63;
  vec8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      // pseudo-random operands in (-1, 1): the clock the matrix pipe sustains depends on how many operand bits toggle,
      // so regular data would flatter the figure
      unsigned ha = (unsigned)(lane * 8 + e + 512 * i) * 2654435761u, hb = (unsigned)(lane * 8 + e + 512 * i + 7) * 2246822519u;
      ha ^= ha >> 15; hb ^= hb >> 13;
      a[i][e] = from_f32<T>((float)(int)(ha >> 8 & 0xffff) * (1.f / 32768.f) - 1.f);
      b[i][e] = from_f32<T>((float)(int)(hb >> 8 & 0xffff) * (1.f / 32768.f) - 1.f);
    }
  f32x16 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < 32; ++m) acc[m & 3] = Elem<T>::mfma32(a[m & 3], b[(m >> 2) & 3], acc[m & 3]);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) s += acc[i][0] + acc[i][15];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

// ---- (2) HBM read stream ---------------------------------------------------------------------------------------------
// Workgroup w reads the w-th contiguous share of the buffer, wave by wave in 8 KiB steps (8 instructions of 1 KiB).
// TO_LDS: global_load_lds_dwordx4 into a per-wave ring of DEPTH steps, never read; at most DEPTH - 1 steps stay in flight.
// Otherwise 16-byte loads into registers, folded into one value so the compiler keeps them.
template <bool TO_LDS, int DEPTH>
__global__ __launch_bounds__(256) void ceiling_stream_kernel(const unsigned char* __restrict__ src, int64_t steps_per_wave,
                                                             float* __restrict__ out) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t wave_id = (int64_t)blockIdx.x * 4 + wave;
  const unsigned char* base = src + wave_id * steps_per_wave * 8192;
  unsigned fold = 0;
  if (TO_LDS) {
    const unsigned ring = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)smem + wave * (DEPTH * 8192);
    const unsigned lane_off = lane * 16;
    for (int64_t s = 0; s < steps_per_wave; ++s) {
      const unsigned dst = ring + (unsigned)(s % DEPTH) * 8192;
      const unsigned char* row = base + s * 8192;
#pragma unroll
      for (int r = 0; r < 8; ++r)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst + r * 1024), "v"(lane_off), "s"(row + r * 1024)
                     : "memory", "m0");
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(8 * (DEPTH - 1)) : "memory");
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  } else {
    for (int64_t s = 0; s < steps_per_wave; ++s) {
      const u32x4* row = reinterpret_cast<const u32x4*>(base + s * 8192) + lane;
      u32x4 v[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) v[r] = __builtin_nontemporal_load(row + r * 64);
#pragma unroll
      for (int r = 0; r < 8; ++r) fold ^= v[r][0] ^ v[r][3];
    }
  }
  if (fold == 0x12345678u || blockIdx.x == 0) out[threadIdx.x] = (float)fold;
}

// The third path: 16-byte loads into a register queue DEPTH steps deep (so DEPTH x 8 KiB per wave are in flight whatever the
// LDS holds), each step written on to a small per-wave LDS buffer with ds_write_b128 once it has landed - what a loader wave
// does when registers, not LDS slots, are the landing zone.
template <int DEPTH>
__global__ __launch_bounds__(256) void ceiling_stream_regs_to_lds_kernel(const unsigned char* __restrict__ src, int64_t steps_per_wave,
                                                                         float* __restrict__ out) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t wave_id = (int64_t)blockIdx.x * 4 + wave;
  const u32x4* base = reinterpret_cast<const u32x4*>(src + wave_id * steps_per_wave * 8192) + lane;
  u32x4* buf = reinterpret_cast<u32x4*>(smem + wave * 2 * 8192) + lane;   // two 8 KiB buffers per wave
  u32x4 v[DEPTH][8];
  unsigned seen = 0;   // 16-byte packets handed on (their first and last words agree in a buffer filled with one byte value)
  const int64_t rounds = steps_per_wave / DEPTH;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
#pragma unroll
    for (int r = 0; r < 8; ++r) v[d][r] = __builtin_nontemporal_load(base + (int64_t)d * 512 + r * 64);
  for (int64_t k = 0; k < rounds; ++k) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      u32x4* dst = buf + (d & 1) * 512;
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        dst[r * 64] = v[d][r];     // the oldest step has landed: hand it on
        seen += v[d][r][0] == v[d][r][3] ? 1u : 0u;
      }
      if (k + 1 < rounds) {
#pragma unroll
        for (int r = 0; r < 8; ++r) v[d][r] = __builtin_nontemporal_load(base + ((k + 1) * DEPTH + d) * 512 + r * 64);
      }
    }
  }
  __syncthreads();
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = (float)seen;   // host check: the sum is bytes / 16
}

template <bool TO_LDS, int DEPTH>
static int launch_stream(const void* src, int64_t bytes, int wgs, float* out, hipStream_t st) {
  const int64_t steps = bytes / ((int64_t)wgs * 4 * 8192);
  if (steps <= 0) return XKV_EINVAL;
  const size_t shm = TO_LDS ? (size_t)4 * DEPTH * 8192 : 0;
  auto kern = ceiling_stream_kernel<TO_LDS, DEPTH>;
  if (TO_LDS) {
    static DynLds lds;
    const int e = ensure_dynamic_lds(lds, reinterpret_cast<const void*>(kern), (int)shm);
    if (e != XKV_OK) return e;
  }
  kern<<<dim3(wgs), dim3(256), shm, st>>>(reinterpret_cast<const unsigned char*>(src), steps, out);
  return launch_status();
}

}  // namespace xkv

using namespace xkv;

// ---- (3) a test aid: LDS is not cleared between kernels, so a kernel that reads a part of its LDS before anything of its own
// has landed there computes on whatever the previous kernel on that CU left.  poison_lds_kernel leaves a pattern that is a NaN
// as fp16, bf16 and fp32 in all 160 KiB of every CU (one workgroup fills a CU's LDS, so no two of them share one; four per CU
// so that every CU gets one), and count_lds_kernel reports how much of a fresh workgroup's LDS still holds it.
constexpr int POISON_LDS_BYTES = 160 * 1024;
__global__ __launch_bounds__(1024) void poison_lds_kernel(unsigned pattern) {
  extern __shared__ __attribute__((aligned(16))) unsigned lds_words[];
  for (int i = threadIdx.x; i < POISON_LDS_BYTES / 4; i += 1024) lds_words[i] = pattern;
  __syncthreads();
  const unsigned back = lds_words[(threadIdx.x * 37) % (POISON_LDS_BYTES / 4)];
  asm volatile("" ::"v"(back));   // a use of the LDS contents: keeps the stores alive
}
__global__ __launch_bounds__(1024) void count_lds_kernel(unsigned pattern, int32_t* __restrict__ seen) {
  extern __shared__ __attribute__((aligned(16))) unsigned lds_words[];
  int n = 0;
  for (int i = threadIdx.x; i < POISON_LDS_BYTES / 4; i += 1024) n += lds_words[i] == pattern;
  atomicAdd(&seen[0], n);
  if (threadIdx.x == 0) atomicAdd(&seen[1], POISON_LDS_BYTES / 4);
}

extern "C" int xkv_poison_lds(uint32_t pattern, int32_t* seen, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return (int)e;
  static DynLds lds[2];
  if (!seen) {
    const int rc = ensure_dynamic_lds(lds[0], reinterpret_cast<const void*>(poison_lds_kernel), POISON_LDS_BYTES);
    if (rc != XKV_OK) return rc;
    poison_lds_kernel<<<dim3(4 * cus), dim3(1024), POISON_LDS_BYTES, st>>>(pattern);
  } else {
    const int rc = ensure_dynamic_lds(lds[1], reinterpret_cast<const void*>(count_lds_kernel), POISON_LDS_BYTES);
    if (rc != XKV_OK) return rc;
    count_lds_kernel<<<dim3(cus), dim3(1024), POISON_LDS_BYTES, st>>>(pattern, seen);
  }
  return launch_status();
}

extern "C" int xkv_ceiling_mfma(float* out, int workgroups, int iters, int dtype, void* stream) {
  if (!out || workgroups <= 0 || iters <= 0) return XKV_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == XKV_BF16) ceiling_mfma_kernel<__bf16><<<dim3(workgroups), dim3(256), 0, st>>>(out, iters);
  else if (dtype == XKV_F16) ceiling_mfma_kernel<_Float16><<<dim3(workgroups), dim3(256), 0, st>>>(out, iters);
  else return XKV_EDTYPE;
  return launch_status();
}

extern "C" int xkv_ceiling_stream(const void* src, int64_t bytes, int workgroups, int to_lds, int depth, float* out,
                                  void* stream) {
  if (!src || !out || bytes <= 0 || workgroups <= 0) return XKV_EINVAL;
  if (reinterpret_cast<uintptr_t>(src) & 15) return XKV_EALIGN;
  hipStream_t st = (hipStream_t)stream;
  if (!to_lds) return launch_stream<false, 1>(src, bytes, workgroups, out, st);
  if (to_lds == 2) {   // register queue of `depth` steps, then ds_write
    const int64_t steps = bytes / ((int64_t)workgroups * 4 * 8192) / (depth > 0 ? depth : 1) * (depth > 0 ? depth : 1);
    if (steps <= 0) return XKV_EINVAL;
    const unsigned char* s8 = reinterpret_cast<const unsigned char*>(src);
    switch (depth) {
      case 2: ceiling_stream_regs_to_lds_kernel<2><<<dim3(workgroups), dim3(256), 4 * 2 * 8192, st>>>(s8, steps, out); break;
      case 4: ceiling_stream_regs_to_lds_kernel<4><<<dim3(workgroups), dim3(256), 4 * 2 * 8192, st>>>(s8, steps, out); break;
      case 6: ceiling_stream_regs_to_lds_kernel<6><<<dim3(workgroups), dim3(256), 4 * 2 * 8192, st>>>(s8, steps, out); break;
      default: return XKV_EUNSUPPORTED;
    }
    return launch_status();
  }
  switch (depth) {
    case 2: return launch_stream<true, 2>(src, bytes, workgroups, out, st);
    case 3: return launch_stream<true, 3>(src, bytes, workgroups, out, st);
    case 4: return launch_stream<true, 4>(src, bytes, workgroups, out, st);
    default: return XKV_EUNSUPPORTED;
  }
}
