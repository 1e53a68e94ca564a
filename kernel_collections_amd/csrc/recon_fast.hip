// Fast path of the fused reconstruct + RoPE + softmax + P.A stage 1 (rank 512, head_dim 128, the
// token basis shared by K and V): the MFMA-bound headline kernel.
//
// Work split.  One workgroup = one (batch, kv head, split); its 4 wavefronts form a 2 x 2 grid over
// (rank half kq, feature half dq): wave (kq, dq) keeps B[kh][256 kq .. +256][{32 dq .. +32} u {64 + 32 dq .. +32}]
// stationary in 128 VGPRs (both members of every rotate-half pair) and multiplies it, on
// v_mfma_f32_32x32x16, with its rank half of the 32-token tile.  Every element of the tile is therefore read
// from LDS by two waves, not four - LDS read bandwidth (128 B/clk/CU), not MFMA, bounds the 4-way split.
// RoPE, the rounding to the operand type and the q-dot are all linear in K, so each wave rotates and dots its
// PARTIAL key tile (partial over its rank half and its feature half) and only 4 x [G x 32] fp32 partial scores
// are summed through LDS.
//
// Rotation.  R(pos) = R(tile base) R(offset in tile).  The in-tile part is a per-lane constant table (32
// VGPRs); the base part is moved to the query: q^ = R(-base) q is recomputed per tile by the workgroup
// (one thread per pair index, incremental rotation re-seeded with a range-reduced sincosf every 32 tiles)
// and read back as the B operand of the q-dot MFMA.
//
// Pipeline.  The tile ring (4 x 32 tokens x 1040 B) is filled by direct-to-LDS loads issued two tiles ahead.
// Softmax and P.A of tile t-1 run in the same barrier interval as the reconstruction of tile t, so there is ONE
// workgroup barrier per tile.  The direct-to-LDS loads are inline asm so that the compiler's wait-count pass does
// not serialise them against every LDS read; completion is tracked by hand (s_waitcnt vmcnt(8): the 8 loads of
// the next tile may still be in flight).
#include "xkv_common.h"
#include "recon_fast.h"

namespace xkv {


typedef short s16x4f __attribute__((ext_vector_type(4)));
typedef short s16x8f __attribute__((ext_vector_type(8)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int FT = 32;              // tokens per tile
constexpr int FROW = 1040;          // LDS bytes per tile row (1024 + 16 pad: 16 rows hit 16 distinct bank groups)
constexpr int FTILE = FT * FROW;    // 33280
constexpr int FRING = 4;
constexpr int FSP_ROW = FT + 4;     // partial-score row stride (floats)

// The LDS destination of a direct-to-LDS load is M0 + lane * 16.  A SALU write of M0 needs one wait state
// before an instruction that reads M0 (the compiler schedules around this for its own code; here it is explicit).
__device__ __forceinline__ void async_row16(const void* gsrc, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(gsrc) : "memory", "m0");
}
template <int N> __device__ __forceinline__ void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// ---------------------------------------------------------------------------------------------------------------
// kB [hkv][512][128] (strided) -> Bp [hkv][wave 4][ks 16][blk 2][lane 64][8]: the 16-byte packet lane l of wave
// (kq, dq) feeds to MFMA (ks, blk) as the A operand: B[256 kq + 16 ks + 8 (l / 32) + e][64 blk + 32 dq + l % 32].
// ---------------------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void pack_b_kernel(const T* __restrict__ kB, T* __restrict__ Bp, int64_t sBb, int64_t sBh,
                                                      int64_t sBr, int hkv) {
  const int kh = blockIdx.x, b = blockIdx.y;
  const T* Bh = kB + b * sBb + kh * sBh;
  T* out = Bp + ((int64_t)b * hkv + kh) * (512 * 128);
  for (int idx = threadIdx.x; idx < 4 * 16 * 2 * 64; idx += 256) {
    const int l = idx & 63, blk = (idx >> 6) & 1, ks = (idx >> 7) & 15, w = idx >> 11;
    const int kq = w >> 1, dq = w & 1;
    const int col = 64 * blk + 32 * dq + (l & 31);
    const int row0 = 256 * kq + 16 * ks + 8 * (l >> 5);
    typename Elem<T>::vec8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = Bh[(int64_t)(row0 + e) * sBr + col];
    st16(out + (int64_t)idx * 8, v);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void recon_fast_kernel(const FastParams p) {
  typedef typename Elem<T>::vec8 vec8;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kq = wave >> 1, dq = wave & 1;
  const int n32 = lane & 31, g2 = lane >> 5;
  const int n16 = lane & 15, g4 = lane >> 4;

  const int total8 = gridDim.x;
  int wg = (blockIdx.x & 7) * (total8 >> 3) + (blockIdx.x >> 3);   // XCD-aware: the 8 kv heads of a tile stream share an L2
  if (wg >= p.total_wg) return;
  const int kh = wg % p.hkv;
  const int split = (wg / p.hkv) % p.max_splits;
  const int b = wg / (p.hkv * p.max_splits);
  const int L = p.kv_lens ? p.kv_lens[b] : p.kv_len;
  int start, end;
  split_bounds(L, p.num_splits[b], split, start, end);
  if (end <= start) return;
  const int G = p.hq / p.hkv, h0 = kh * G;
  const int ntiles = (end - start + FT - 1) / FT;
  const int last = end - 1;

  // ---- LDS carve-up ---------------------------------------------------------------------------------------------
  unsigned char* ring = smem;                                              // FRING * FTILE
  float* s_part = reinterpret_cast<float*>(smem + FRING * FTILE);          // [2][4 waves][8 heads][FSP_ROW]
  T* qhat = reinterpret_cast<T*>(s_part + 2 * 4 * 8 * FSP_ROW);            // [2][8 heads][128]
  const unsigned ring_lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)ring;

  // ---- async tile loads: wave w brings rows 8w .. 8w+7, one 1 KiB row per instruction ------------------------------
  const unsigned char* Ab = reinterpret_cast<const unsigned char*>(p.kA) + b * p.sAb * 2 + lane * 16;
  const int64_t row_bytes = p.sAl * 2;
  auto issue_tile = [&](int t) {
    const unsigned dst = ring_lds + (unsigned)(t & (FRING - 1)) * FTILE + (unsigned)(wave * 8) * FROW;
    const int tok0 = start + t * FT + wave * 8;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      int tok = tok0 + r;
      tok = tok < last ? tok : last;   // rows past the split end are masked in the softmax; keep the read in bounds
      async_row16(Ab + (int64_t)tok * row_bytes, dst + r * FROW);
    }
  };
  issue_tile(0);
  issue_tile(1);

  // ---- stationary B operands: 16 k-steps x 2 feature blocks ---------------------------------------------------------
  vec8 breg[16][2];
  {
    const T* bp = reinterpret_cast<const T*>(p.Bp) + b * p.sBpb + (int64_t)kh * (512 * 128) + ((int64_t)wave * 2048 + lane) * 8;
#pragma unroll
    for (int ks = 0; ks < 16; ++ks)
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) breg[ks][blk] = ld16<vec8>(bp + (ks * 2 + blk) * 512);
  }

  // ---- in-tile rotation table: accumulator register r of lane (token n32, g2) is pair j = 32 dq + 8 (r/4) + 4 g2 + r%4 --
  float ci[16], si[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int j = 32 * dq + 8 * (r >> 2) + 4 * g2 + (r & 3);
    sincosf((float)n32 * p.inv_freq[j], &si[r], &ci[r]);
  }

  // ---- query-side base rotation: thread -> pair j = tid % 64, head slots 4 (tid / 64) .. +3 ---------------------------
  const int qj = tid & 63, qh0 = (tid >> 6) * 4;
  float q0[4], q1[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int h = qh0 + i;
    if (h < G) {
      const T* qrow = reinterpret_cast<const T*>(p.q) + ((int64_t)b * p.hq + h0 + h) * 128;
      q0[i] = to_f32(qrow[qj]);
      q1[i] = to_f32(qrow[qj + 64]);
    } else {
      q0[i] = 0.f; q1[i] = 0.f;
    }
  }
  const float qinv = p.inv_freq[qj];
  float qc32, qs32, qcb = 1.f, qsb = 0.f;
  sincosf((float)FT * qinv, &qs32, &qc32);
  auto prep_qhat = [&](int t) {   // q^ for tile t: rotate q by minus the tile's base position
    if (t >= ntiles) return;
    if ((t & 31) == 0) {
      sincosf((float)(p.pos_offset + start + (int64_t)t * FT) * qinv, &qsb, &qcb);
    } else {
      const float c = qcb * qc32 - qsb * qs32, s = qsb * qc32 + qcb * qs32;
      qcb = c; qsb = s;
    }
    if (qh0 < 8) {
      T* dst = qhat + (t & 1) * (8 * 128);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        dst[(qh0 + i) * 128 + qj] = from_f32<T>(q0[i] * qcb + q1[i] * qsb);
        dst[(qh0 + i) * 128 + qj + 64] = from_f32<T>(q1[i] * qcb - q0[i] * qsb);
      }
    }
  };
  prep_qhat(0);

  // ---- running softmax state (replicated: every wave tracks all heads) and P.A accumulators --------------------------
  float m_run = NEG_INF, l_run = 0.f;
  f32x4 acc[8];
#pragma unroll
  for (int mb = 0; mb < 8; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int hrow = n16 < G ? n16 : G - 1;   // lanes beyond the real heads recompute the last one; never stored

  auto softmax_pv = [&](int t) {   // tile t: partial scores -> P -> acc += V^T P^T
    const float* sp = s_part + (t & 1) * (4 * 8 * FSP_ROW) + hrow * FSP_ROW + 8 * g4;
    f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      lo += *reinterpret_cast<const f32x4*>(sp + w * 8 * FSP_ROW);
      hi += *reinterpret_cast<const f32x4*>(sp + w * 8 * FSP_ROW + 4);
    }
    float sv[8];
    const int tok0 = start + t * FT + 8 * g4;
    float mx = NEG_INF;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float s = (e < 4 ? lo[e] : hi[e - 4]) * p.sm_scale;
      sv[e] = (tok0 + e < end) ? s : NEG_INF;
      mx = fmaxf(mx, sv[e]);
    }
    mx = group4_max(mx);
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __expf(m_run - m_new);
    float sum = 0.f;
    vec8 pb;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float ex = __expf(sv[e] - m_new);
      sum += ex;
      pb[e] = from_f32<T>(ex);
    }
    sum = group4_sum(sum);
    l_run = l_run * alpha + sum;
    m_run = m_new;
    const unsigned char* vt = ring + (t & (FRING - 1)) * FTILE + (8 * g4 + (n16 >> 2)) * FROW + (wave * 128 + 4 * (n16 & 3)) * 2;
#pragma unroll
    for (int mb = 0; mb < 8; ++mb) {
      s16x4f a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4f*)(vt + mb * 32));
      s16x4f a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4f*)(vt + mb * 32 + 4 * FROW));
      vec8 a = __builtin_bit_cast(vec8, (s16x8f)__builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7));
      acc[mb] = Elem<T>::mfma16(a, pb, acc[mb] * alpha);
    }
  };

  // ---- main loop: one barrier per tile ------------------------------------------------------------------------------------
  for (int t = 0; t < ntiles; ++t) {
    wait_vmcnt<8>();        // this wave's rows of tile t have landed (tile t+1's 8 loads may be in flight)
    __syncthreads();        // tile t, q^(t) and the partial scores of tile t-1 are complete for every wave
    issue_tile(t + 2);
    prep_qhat(t + 1);

    // reconstruct this wave's partial key tile: [32 low features | 32 partner features] x 32 tokens
    f32x16 k0, k1;
#pragma unroll
    for (int r = 0; r < 16; ++r) { k0[r] = 0.f; k1[r] = 0.f; }
    const unsigned char* arow = ring + (t & (FRING - 1)) * FTILE + n32 * FROW + (256 * kq + 8 * g2) * 2;
#pragma unroll
    for (int ks = 0; ks < 16; ++ks) {
      const vec8 at = ld16<vec8>(arow + ks * 32);
      k0 = Elem<T>::mfma32(breg[ks][0], at, k0);
      k1 = Elem<T>::mfma32(breg[ks][1], at, k1);
    }
    // rotate by the in-tile offset, round to the operand type, dot with q^ (4 contraction chunks of 16 features)
    f32x16 sacc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
    const T* qrow = qhat + (t & 1) * (8 * 128) + (n32 < G ? n32 : G - 1) * 128 + 32 * dq + 4 * g2;
#pragma unroll
    for (int o = 0; o < 4; ++o) {
      vec8 kop, qop;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int r = 4 * o + e;
        kop[e] = from_f32<T>(k0[r] * ci[r] - k1[r] * si[r]);
        kop[4 + e] = from_f32<T>(k1[r] * ci[r] + k0[r] * si[r]);
      }
      const u32x2 ql = *reinterpret_cast<const u32x2*>(qrow + 8 * o);
      const u32x2 qh = *reinterpret_cast<const u32x2*>(qrow + 64 + 8 * o);
      const u32x4 qq = {ql[0], ql[1], qh[0], qh[1]};
      qop = __builtin_bit_cast(vec8, qq);
      sacc = Elem<T>::mfma32(kop, qop, sacc);
    }
    // lane (n32 = head, g2): register r = token 8 (r/4) + 4 g2 + r%4
    if (n32 < G) {
      float* dst = s_part + (t & 1) * (4 * 8 * FSP_ROW) + (wave * 8 + n32) * FSP_ROW + 4 * g2;
#pragma unroll
      for (int qd = 0; qd < 4; ++qd)
        *reinterpret_cast<f32x4*>(dst + 8 * qd) = f32x4{sacc[4 * qd], sacc[4 * qd + 1], sacc[4 * qd + 2], sacc[4 * qd + 3]};
    }
    if (t > 0) softmax_pv(t - 1);
  }
  wait_vmcnt<0>();
  __syncthreads();
  softmax_pv(ntiles - 1);

  // ---- epilogue ----------------------------------------------------------------------------------------------------------
  if (n16 < G) {
    const float inv = 1.f / l_run;
    const int64_t ph = ((int64_t)b * p.hq + h0 + n16) * p.max_splits + split;
    float* dst = p.partial + ph * 512 + wave * 128 + 4 * g4;
#pragma unroll
    for (int mb = 0; mb < 8; ++mb) *reinterpret_cast<f32x4*>(dst + mb * 16) = acc[mb] * inv;
    if (wave == 0 && g4 == 0) p.lse[ph] = m_run + __logf(l_run);
  }
}

constexpr size_t FAST_SHM = (size_t)FRING * FTILE + 2 * 4 * 8 * FSP_ROW * 4 + 2 * 8 * 128 * 2;

template <typename T>
int launch_recon_fast_t(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, hipStream_t st) {
  const int nb = sBb == 0 ? 1 : batch;   // one packed copy when the factor is shared by the batch
  pack_b_kernel<T><<<dim3(p.hkv, nb), dim3(256), 0, st>>>((const T*)kB, (T*)p.Bp, sBb, sBh, sBr, p.hkv);
  auto kern = recon_fast_kernel<T>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)FAST_SHM);
  if (e != hipSuccess) return (int)e;
  const int total = batch * p.hkv * p.max_splits;
  kern<<<dim3((total + 7) & ~7), dim3(256), FAST_SHM, st>>>(p);
  return launch_status();
}

int launch_recon_fast(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                      hipStream_t st) {
  return dtype == XKV_BF16 ? launch_recon_fast_t<__bf16>(p, kB, sBb, sBh, sBr, batch, st)
                           : launch_recon_fast_t<_Float16>(p, kB, sBb, sBh, sBr, batch, st);
}

}  // namespace xkv
