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
#include <type_traits>

namespace xkv {


typedef short s16x4f __attribute__((ext_vector_type(4)));
typedef short s16x8f __attribute__((ext_vector_type(8)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

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

// max / sum over each row of 16 lanes, result in every lane of the row (DPP butterflies, no LDS traffic)
template <bool IS_MAX> __device__ __forceinline__ float row16_reduce(float x) {
#define XKV_DPP_STEP(ctrl)                                                                                       \
  {                                                                                                              \
    const float y = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), ctrl, 0xf, 0xf, false)); \
    x = IS_MAX ? fmaxf(x, y) : x + y;                                                                            \
  }
  XKV_DPP_STEP(0xB1)   // quad_perm [1,0,3,2]
  XKV_DPP_STEP(0x4E)   // quad_perm [2,3,0,1]
  XKV_DPP_STEP(0x141)  // row_half_mirror
  XKV_DPP_STEP(0x140)  // row_mirror
#undef XKV_DPP_STEP
  return x;
}

constexpr int FP_ROW = FT + 8;       // P row stride (elements)
constexpr float LAZY_RESCALE = 16.f; // the softmax reference only moves when a tile maximum exceeds it by this much

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
  float* s_part = reinterpret_cast<float*>(smem + FRING * FTILE);          // [4 waves][8 heads][FSP_ROW]
  T* qhat = reinterpret_cast<T*>(s_part + 4 * 8 * FSP_ROW);                // [2][8 heads][128]
  T* p_lds = qhat + 2 * 8 * 128;                                           // [16 head slots][FP_ROW]
  float* alpha_lds = reinterpret_cast<float*>(p_lds + 16 * FP_ROW);        // [16]
  float* ml_lds = alpha_lds + 16;                                          // [8][2]
  const unsigned ring_lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)ring;
  for (int i = tid; i < 16 * FP_ROW; i += 256) p_lds[i] = from_f32<T>(0.f);   // slots of absent heads stay zero
  if (tid < 16) alpha_lds[tid] = 1.f;

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

  // ---- stationary B operands: 16 k-steps x 2 feature blocks, kept in accumulation registers ---------------------------
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

  // ---- query-side base rotation: thread -> pair j = lane, head slots wave and wave + 4 ---------------------------------
  float q0[2], q1[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int h = wave + 4 * i;
    if (h < G) {
      const T* qrow = reinterpret_cast<const T*>(p.q) + ((int64_t)b * p.hq + h0 + h) * 128;
      q0[i] = to_f32(qrow[lane]);
      q1[i] = to_f32(qrow[lane + 64]);
    } else {
      q0[i] = 0.f; q1[i] = 0.f;
    }
  }
  const float qinv = p.inv_freq[lane];
  float qc32, qs32, qcb = 1.f, qsb = 0.f;
  sincosf((float)FT * qinv, &qs32, &qc32);
  auto seed_base = [&](int t) { sincosf((float)(p.pos_offset + start + (int64_t)t * FT) * qinv, &qsb, &qcb); };
  auto step_base = [&]() {
    const float c = qcb * qc32 - qsb * qs32, s = qsb * qc32 + qcb * qs32;
    qcb = c; qsb = s;
  };
  auto write_qhat = [&](int t) {   // q^ for tile t = R(-base(t)) q, base held in (qcb, qsb)
    T* dst = qhat + (t & 1) * (8 * 128) + wave * 128 + lane;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      dst[i * 512] = from_f32<T>(q0[i] * qcb + q1[i] * qsb);
      dst[i * 512 + 64] = from_f32<T>(q1[i] * qcb - q0[i] * qsb);
    }
  };

  // ---- softmax role: lanes 0..15 of wave w own head w, lanes 16..31 head w + 4; two tokens per lane ---------------------
  const int sm_head = wave + 4 * ((lane >> 4) & 1);
  const int sm_row = sm_head < G ? sm_head : G - 1;
  const bool sm_valid = sm_head < G;   // lanes 32..63 duplicate lanes 0..31 (same values, same addresses)
  float m_ref = NEG_INF, l_run = 0.f;
#ifdef XKV_DEBUG_SCORES
  float dbg0 = 0.f, dbg1 = 0.f;
#endif
  auto softmax_tile = [&](int t) {   // scores of tile t -> P (operand type) and the rescale factor, through LDS
    const float* sp = s_part + sm_row * FSP_ROW + 2 * n16;
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const f32x2 v = *reinterpret_cast<const f32x2*>(sp + w * 8 * FSP_ROW);
      s0 += v[0];
      s1 += v[1];
    }
    const int tok = start + t * FT + 2 * n16;
    s0 = tok < end ? s0 * p.sm_scale : NEG_INF;
    s1 = tok + 1 < end ? s1 * p.sm_scale : NEG_INF;
#ifdef XKV_DEBUG_SCORES
    dbg0 = s0; dbg1 = s1;
#endif
    const float mx = row16_reduce<true>(fmaxf(s0, s1));
    const float m_new = mx > m_ref + LAZY_RESCALE ? mx : m_ref;
    const float alpha = __expf(m_ref - m_new);
    const float e0 = __expf(s0 - m_new), e1 = __expf(s1 - m_new);
    l_run = l_run * alpha + row16_reduce<false>(e0 + e1);
    m_ref = m_new;
    T* pd = p_lds + sm_head * FP_ROW + 2 * n16;
    pd[0] = from_f32<T>(sm_valid ? e0 : 0.f);
    pd[1] = from_f32<T>(sm_valid ? e1 : 0.f);
    alpha_lds[sm_head] = alpha;
  };

  // ---- P.A accumulators: wave w owns latent features 128 w .. +128 -----------------------------------------------------
  f32x4 acc[8];
#pragma unroll
  for (int mb = 0; mb < 8; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto pv_tile = [&](int t) {
    const float al = alpha_lds[n16];
    if (__builtin_amdgcn_ballot_w64(al != 1.f)) {   // rare: the softmax reference moved
#pragma unroll
      for (int mb = 0; mb < 8; ++mb) acc[mb] *= al;
    }
    const vec8 pb = ld16<vec8>(p_lds + n16 * FP_ROW + 8 * g4);
    const unsigned char* vt = ring + (t & (FRING - 1)) * FTILE + (8 * g4 + (n16 >> 2)) * FROW + (wave * 128 + 4 * (n16 & 3)) * 2;
#pragma unroll
    for (int mb = 0; mb < 8; ++mb) {
      s16x4f a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4f*)(vt + mb * 32));
      s16x4f a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4f*)(vt + mb * 32 + 4 * FROW));
      vec8 a = __builtin_bit_cast(vec8, (s16x8f)__builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7));
      acc[mb] = Elem<T>::mfma16(a, pb, acc[mb]);
    }
  };

  // ---- reconstruction of this wave's partial key tile, k-steps [KS0, KS1) -----------------------------------------------
  f32x16 k0, k1;
  auto recon_steps = [&](int t, auto ks0, auto ks1) {
    const unsigned char* arow = ring + (t & (FRING - 1)) * FTILE + n32 * FROW + (256 * kq + 8 * g2) * 2;
#pragma unroll
    for (int ks = decltype(ks0)::value; ks < decltype(ks1)::value; ++ks) {
      const vec8 at = ld16<vec8>(arow + ks * 32);
      k0 = Elem<T>::mfma32(breg[ks][0], at, k0);
      k1 = Elem<T>::mfma32(breg[ks][1], at, k1);
    }
  };
  // rotate by the in-tile offset, round to the operand type, dot with q^ (4 contraction chunks of 16 features), store
  auto rope_qdot = [&](int t) {
    f32x16 sacc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
    const T* qrow = qhat + (t & 1) * (8 * 128) + (n32 < G ? n32 : G - 1) * 128 + 32 * dq + 4 * g2;
#pragma unroll
    for (int o = 0; o < 4; ++o) {
      vec8 kop;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int r = 4 * o + e;
        kop[e] = from_f32<T>(k0[r] * ci[r] - k1[r] * si[r]);
        kop[4 + e] = from_f32<T>(k1[r] * ci[r] + k0[r] * si[r]);
      }
      const u32x2 ql = *reinterpret_cast<const u32x2*>(qrow + 8 * o);
      const u32x2 qh = *reinterpret_cast<const u32x2*>(qrow + 64 + 8 * o);
      const u32x4 qq = {ql[0], ql[1], qh[0], qh[1]};
      sacc = Elem<T>::mfma32(kop, __builtin_bit_cast(vec8, qq), sacc);
    }
    // lane (n32 = head, g2): register r = token 8 (r/4) + 4 g2 + r%4
    if (n32 < G) {
      float* dst = s_part + (wave * 8 + n32) * FSP_ROW + 4 * g2;
#pragma unroll
      for (int qd = 0; qd < 4; ++qd)
        *reinterpret_cast<f32x4*>(dst + 8 * qd) = f32x4{sacc[4 * qd], sacc[4 * qd + 1], sacc[4 * qd + 2], sacc[4 * qd + 3]};
    }
  };
  auto zero_k = [&]() {
#pragma unroll
    for (int r = 0; r < 16; ++r) { k0[r] = 0.f; k1[r] = 0.f; }
  };
  typedef std::integral_constant<int, 0> I0;
  typedef std::integral_constant<int, 8> I8;
  typedef std::integral_constant<int, 16> I16;

  // ---- tile 0: no predecessor to finish ---------------------------------------------------------------------------------
  seed_base(0);
  write_qhat(0);
  step_base();              // (qcb, qsb) always holds the base of the next tile whose q^ is to be written
  wait_vmcnt<8>();
  __syncthreads();
  issue_tile(2);
  zero_k();
  recon_steps(0, I0(), I16());
  rope_qdot(0);

  // ---- steady state: tile t is reconstructed while tile t-1 goes through softmax and P.A ------------------------------------
  int t = 1;
  while (t < ntiles) {
    const int chunk_end = (t | 31) + 1 < ntiles ? (t | 31) + 1 : ntiles;
    if ((t & 31) == 0) seed_base(t);   // re-seed the base angle with a full-range sincos every 32 tiles
    for (; t < chunk_end; ++t) {
#pragma unroll
      for (int ks = 0; ks < 16; ++ks) {
#ifndef XKV_NO_PIN
        asm volatile("" : "+a"(breg[ks][0]));
        asm volatile("" : "+a"(breg[ks][1]));
#endif
      }
      wait_vmcnt<8>();        // this wave's rows of tile t have landed (tile t+1's 8 loads may be in flight)
      __syncthreads();        // B1: tile t and the partial scores of tile t-1 are complete for every wave
      issue_tile(t + 2);
      write_qhat(t);
      step_base();
      zero_k();
      softmax_tile(t - 1);
      recon_steps(t, I0(), I8());
      __syncthreads();        // B2: P and the rescale factors of tile t-1 are visible
      recon_steps(t, I8(), I16());
      pv_tile(t - 1);
      rope_qdot(t);
    }
  }
  wait_vmcnt<0>();
  __syncthreads();
  softmax_tile(ntiles - 1);
  if (sm_valid && n16 == 0) { ml_lds[2 * sm_head] = m_ref; ml_lds[2 * sm_head + 1] = l_run; }
  __syncthreads();
  pv_tile(ntiles - 1);

  // ---- epilogue ----------------------------------------------------------------------------------------------------------
  if (n16 < G) {
    const float m = ml_lds[2 * n16], l = ml_lds[2 * n16 + 1];
    const float inv = 1.f / l;
    const int64_t ph = ((int64_t)b * p.hq + h0 + n16) * p.max_splits + split;
    float* dst = p.partial + ph * 512 + wave * 128 + 4 * g4;
#pragma unroll
    for (int mb = 0; mb < 8; ++mb) *reinterpret_cast<f32x4*>(dst + mb * 16) = acc[mb] * inv;
    if (wave == 0 && g4 == 0) p.lse[ph] = m + __logf(l);
  }
#ifdef XKV_DEBUG_SCORES
  __syncthreads();
  if (sm_valid && lane < 16) {   // last tile's scaled scores of head sm_head into the first 32 partial columns
    float* dst = p.partial + (((int64_t)b * p.hq + h0 + sm_head) * p.max_splits + split) * 512 + 2 * n16;
    dst[0] = dbg0; dst[1] = dbg1;
  }
#endif
}

constexpr size_t FAST_SHM = (size_t)FRING * FTILE + 4 * 8 * FSP_ROW * 4 + 2 * 8 * 128 * 2 + 16 * FP_ROW * 2 + 16 * 4 + 16 * 4;

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
