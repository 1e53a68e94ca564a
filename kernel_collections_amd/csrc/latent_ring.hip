// Split-K flash-decoding stage 1 for WIDE latent rows (512 or 1024 features, optionally + 64 RoPE features):
// the bandwidth-bound scans of the path (absorbed no-PE xKV scores and decode, MLA over c_kv | k_pe).
//
// Same arithmetic as latent_stage1.hip; what differs is how bytes move.  A CU has to keep roughly
// (HBM latency x its share of 8 TB/s) = 60-100 KB of loads in flight to stream at full rate, which a
// register-staged double buffer cannot hold.  Here the token rows go HBM -> LDS directly
// (global_load_lds_dwordx4, no VGPRs involved) into a ring of RSLOT tiles of RTN tokens, RSLOT-1 tiles always in
// flight per workgroup, two workgroups per CU (one's barrier waits overlap the other's work), and the query
// operands live in registers for the whole kernel, so the per-tile work is
//   A:  wait for tile t, barrier, issue tile t+RSLOT-1 into the slot PV(t-1) just released
//   QK: wave (tb, kh) multiplies token block tb by its k-range kh of q on v_mfma_f32_16x16x32 -> partial scores in LDS
//   B:  barrier; softmax threads add the k-range partials, update the running max / sum, publish P and alpha
//   C:  barrier; PV: each wave owns a quarter of the value features, token-major operand via ds_read_b64_tr_b16.
// Scores-only mode (qAB without PE) stops after B and writes the summed scores.
//
// LDS tile layout: C rows are row-major with a 16-byte pad (conflict-free ds_read_b128 over 16 rows and
// conflict-free transposed reads); the 128-byte RoPE-key rows are stored chunk-major ([8 chunks][TN rows][16 B]),
// which the per-lane global addresses of the direct-to-LDS load make free.
#include "xkv_common.h"
#include "latent_ring.h"

namespace xkv {

typedef short s16x4r __attribute__((ext_vector_type(4)));
typedef short s16x8r __attribute__((ext_vector_type(8)));

// LDS destination of a direct-to-LDS load = M0 + lane * 16; a SALU write of M0 needs one wait state before its use.
__device__ __forceinline__ void ring_load16(const void* sbase, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase)
               : "memory", "m0");
}
template <int N> __device__ __forceinline__ void ring_wait() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

template <typename V8>
__device__ __forceinline__ V8 ring_tr_operand(const unsigned char* p0, const unsigned char* p1) {
  s16x4r a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4r*)p0);
  s16x4r b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4r*)p1);
  s16x8r r = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(V8, r);
}

constexpr int RTN = 32;            // tokens per tile
constexpr int RSLOT = 2;           // ring slots: two workgroups share a CU, each keeps one tile in flight
constexpr int RSP = RTN + 4;       // partial-score row stride (floats)
constexpr int RLDP = RTN + 8;      // P row stride (elements)

// T: operand type; NHB: 16-row head blocks; LO: q has a low-order part; DN: latent width; HAS_R: 64 RoPE features follow;
// SCORES: write scores, no softmax / PV.  V is the first DV = 512 features of the row (shared-tile mode only).
template <typename T, int NHB, bool LO, int DN, bool HAS_R, bool SCORES>
__global__ __launch_bounds__(256) void latent_ring_kernel(const RingParams p) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int HB = 16 * NHB;
  constexpr int NKS_N = DN / 32, NKS = NKS_N + (HAS_R ? 2 : 0);
  constexpr int KS_W = (NKS + 1) / 2;             // k-steps per wave (two k-ranges)
  constexpr int CROW = DN * 2 + 16;               // padded C row (bytes)
  constexpr int CBYTES = RTN * CROW;
  constexpr int SLOT = CBYTES + (HAS_R ? RTN * 128 : 0);
  constexpr int IPR = DN / 512;                   // 1 KiB load instructions per C row
  constexpr int LPT = 8 * IPR + (HAS_R ? 1 : 0);  // loads per wave per tile
  constexpr int DV = 512, NVB = DV / 64;          // value features, 16-feature blocks per wave
  constexpr int TPH = 256 / HB, TPT = RTN / TPH;  // softmax threads per head row, tokens per thread

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n16 = lane & 15, g4 = lane >> 4;
  const int tb = wave & 1, kh = wave >> 1;

  int wg = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);   // XCD-aware: neighbours in (group, split) share an L2
  if (wg >= p.total_wg) return;
  const int group = wg % p.groups;
  const int split = (wg / p.groups) % p.max_splits;
  const int b = wg / (p.groups * p.max_splits);
  const int L = p.kv_lens ? p.kv_lens[b] : p.kv_len;
  int start, end;
  split_bounds(L, p.num_splits[b], split, start, end);
  if (end <= start) return;
  const int hg = p.hq / p.groups, h0 = group * hg;
  const int ntiles = (end - start + RTN - 1) / RTN;
  const int last = end - 1;

  // ---- LDS carve-up -------------------------------------------------------------------------------------------
  unsigned char* ring = smem;
  float* s_part = reinterpret_cast<float*>(smem + RSLOT * SLOT);   // [2 k-ranges][HB][RSP]
  T* p_lds = reinterpret_cast<T*>(s_part + 2 * HB * RSP);          // [HB][RLDP]
  float* alpha_lds = reinterpret_cast<float*>(p_lds + HB * RLDP);  // [HB]
  float* ml_lds = alpha_lds + HB;                                  // [HB][2]
  const unsigned ring_lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)ring;

  // ---- tile loads: wave w brings C rows 8w .. 8w+7 and RoPE-key chunks 2w, 2w+1 of every row ---------------------
  const unsigned char* Cb = reinterpret_cast<const unsigned char*>(p.C) + (b * p.sCb + group * p.sCh) * 2;
  const unsigned char* Rb = HAS_R ? reinterpret_cast<const unsigned char*>(p.R) + (b * p.sRb + group * p.sRh) * 2 : nullptr;
  const int64_t crow_bytes = p.sCl * 2, rrow_bytes = p.sRl * 2;
  const unsigned lane_off = lane * 16;
  const int r_row = lane & 31, r_chunk = 2 * wave + (lane >> 5);
  auto issue_tile = [&](int t) {
    const unsigned slot = ring_lds + (unsigned)(t & (RSLOT - 1)) * SLOT;
    const int base = start + t * RTN;
    const int tok0 = base + wave * 8;
    if (base + RTN <= end) {           // whole tile inside the split: row pointers advance by adds
      const unsigned char* row = Cb + (int64_t)tok0 * crow_bytes;
#pragma unroll
      for (int r = 0; r < 8; ++r) {
#pragma unroll
        for (int c = 0; c < IPR; ++c) ring_load16(row + c * 1024, lane_off, slot + (wave * 8 + r) * CROW + c * 1024);
        row += crow_bytes;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        int tok = tok0 + r;
        tok = tok < last ? tok : last;   // rows past the split end are masked in the softmax; keep the read in bounds
        const unsigned char* row = Cb + (int64_t)tok * crow_bytes;
#pragma unroll
        for (int c = 0; c < IPR; ++c) ring_load16(row + c * 1024, lane_off, slot + (wave * 8 + r) * CROW + c * 1024);
      }
    }
    if (HAS_R) {
      int tok = base + r_row;
      tok = tok < last ? tok : last;
      ring_load16(Rb, (unsigned)tok * (unsigned)rrow_bytes + r_chunk * 16, slot + CBYTES + wave * 1024);
    }
  };
#pragma unroll
  for (int t = 0; t < RSLOT - 1; ++t) issue_tile(t);

  // ---- query operands in registers: lane (n16 = head row, g4) holds q[head][32 ks + 8 g4 .. +8] for its k-range ----
  vec8 qreg[KS_W][NHB], qlo[LO ? KS_W : 1][NHB];
  const int ks0 = kh * KS_W;
#pragma unroll
  for (int k = 0; k < KS_W; ++k) {
    const int ks = ks0 + k;
#pragma unroll
    for (int hb = 0; hb < NHB; ++hb) {
      const int row = hb * 16 + n16;
      vec8 v = {0, 0, 0, 0, 0, 0, 0, 0}, vl = {0, 0, 0, 0, 0, 0, 0, 0};
      if (row < hg && ks < NKS) {
        const int64_t qh = (int64_t)b * p.hq + h0 + row;
        if (ks < NKS_N) {
          v = ld16<vec8>(reinterpret_cast<const T*>(p.qn) + qh * DN + ks * 32 + 8 * g4);
          if (LO) vl = ld16<vec8>(reinterpret_cast<const T*>(p.qn_lo) + qh * DN + ks * 32 + 8 * g4);
        } else {
          v = ld16<vec8>(reinterpret_cast<const T*>(p.qr) + qh * 64 + (ks - NKS_N) * 32 + 8 * g4);
        }
      }
      qreg[k][hb] = v;
      if (LO) qlo[k][hb] = vl;
    }
  }

  // ---- running state ---------------------------------------------------------------------------------------------
  const int srow = tid / TPH, ssub = tid % TPH;
  float m_run = NEG_INF, l_run = 0.f;
  f32x4 acc[SCORES ? 1 : NVB][NHB];
#pragma unroll
  for (int mb = 0; mb < (SCORES ? 1 : NVB); ++mb)
#pragma unroll
    for (int hb = 0; hb < NHB; ++hb) acc[mb][hb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int vcol0 = wave * (DV / 4);

  for (int t = 0; t < ntiles; ++t) {
    ring_wait<(RSLOT - 2) * LPT>();   // this wave's rows of tile t have landed (RSLOT-2 younger tiles may be in flight)
    __syncthreads();                  // A: tile t complete for every wave; every wave is past PV / score write of tile t-1
    issue_tile(t + RSLOT - 1);        // into the slot of tile t-1 (past the end: clamped rows, never used)
    const unsigned char* slot = ring + (t & (RSLOT - 1)) * SLOT;
    const int base = start + t * RTN;

    // ---- QK: partial scores of token block tb over this wave's k-range -------------------------------------------
    {
      f32x4 sacc[NHB];
#pragma unroll
      for (int hb = 0; hb < NHB; ++hb) sacc[hb] = f32x4{0.f, 0.f, 0.f, 0.f};
      const unsigned char* arow = slot + (tb * 16 + n16) * CROW + g4 * 16;
      const unsigned char* rrow = slot + CBYTES + (g4 * RTN + tb * 16 + n16) * 16;
#pragma unroll
      for (int k = 0; k < KS_W; ++k) {
        const int ks = ks0 + k;
        if (ks < NKS) {
          const unsigned char* ap = (!HAS_R || ks < NKS_N) ? arow + ks * 64 : rrow + (ks - NKS_N) * (4 * RTN * 16);
          const vec8 a = ld16<vec8>(ap);
#pragma unroll
          for (int hb = 0; hb < NHB; ++hb) {
            sacc[hb] = Elem<T>::mfma16(a, qreg[k][hb], sacc[hb]);
            if (LO) sacc[hb] = Elem<T>::mfma16(a, qlo[k][hb], sacc[hb]);
          }
        }
      }
      // lane (n16 = head row, g4): tokens tb*16 + 4 g4 + r
#pragma unroll
      for (int hb = 0; hb < NHB; ++hb)
        *reinterpret_cast<f32x4*>(s_part + (kh * HB + hb * 16 + n16) * RSP + tb * 16 + 4 * g4) = sacc[hb];
    }
    __syncthreads();                  // B: both k-range partials of every head row are visible

    if (SCORES) {
      // thread -> head row tid / 4, tokens 8 (tid % 4) .. +8: a 32-byte piece of a 128-byte score row
      const int row = tid >> 2, c0 = (tid & 3) * 8;
      if (row < hg) {
        const int64_t o = ((int64_t)b * p.hq + h0 + row) * p.kv_len + base + c0;
        float s[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          s[j] = (s_part[row * RSP + c0 + j] + s_part[(HB + row) * RSP + c0 + j]) * p.sm_scale;
          if (p.logit_cap > 0.f) s[j] = p.logit_cap * tanhf(s[j] / p.logit_cap);
        }
        if (p.scores_dtype == XKV_F32 && (p.kv_len & 3) == 0 && base + c0 + 8 <= end) {
          float* dst = reinterpret_cast<float*>(p.scores) + o;
          *reinterpret_cast<f32x4*>(dst) = f32x4{s[0], s[1], s[2], s[3]};
          *reinterpret_cast<f32x4*>(dst + 4) = f32x4{s[4], s[5], s[6], s[7]};
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (base + c0 + j < end) {
              if (p.scores_dtype == XKV_F32) reinterpret_cast<float*>(p.scores)[o + j] = s[j];
              else reinterpret_cast<T*>(p.scores)[o + j] = from_f32<T>(s[j]);
            }
        }
      }
      continue;
    }

    // ---- online softmax: TPH threads per head row, TPT tokens each ----------------------------------------------
    {
      float sv[TPT];
      float mx = NEG_INF;
#pragma unroll
      for (int i = 0; i < TPT; ++i) {
        const int c = ssub * TPT + i;
        float s = (s_part[srow * RSP + c] + s_part[(HB + srow) * RSP + c]) * p.sm_scale;
        if (p.logit_cap > 0.f) s = p.logit_cap * tanhf(s / p.logit_cap);
        sv[i] = base + c < end ? s : NEG_INF;
        mx = fmaxf(mx, sv[i]);
      }
      mx = row_reduce<true, TPH>(mx);
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __expf(m_run - m_new);
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < TPT; ++i) {
        const float e = __expf(sv[i] - m_new);
        sum += e;
        p_lds[srow * RLDP + ssub * TPT + i] = from_f32<T>(e);
      }
      sum = row_reduce<false, TPH>(sum);
      l_run = l_run * alpha + sum;
      m_run = m_new;
      if (ssub == 0) alpha_lds[srow] = alpha;
    }
    __syncthreads();                  // C: P and alpha of tile t are visible

    // ---- PV: acc^T[feature, head] += V^T P^T, this wave's quarter of the value features -----------------------------
    {
      float al[NHB];
      vec8 pb[NHB];
#pragma unroll
      for (int hb = 0; hb < NHB; ++hb) {
        al[hb] = alpha_lds[hb * 16 + n16];
        pb[hb] = ld16<vec8>(p_lds + (hb * 16 + n16) * RLDP + 8 * g4);
      }
      const unsigned char* vrow = slot + (8 * g4 + (n16 >> 2)) * CROW + (vcol0 + 4 * (n16 & 3)) * 2;
#pragma unroll
      for (int mb = 0; mb < NVB; ++mb) {
        const vec8 a = ring_tr_operand<vec8>(vrow + mb * 32, vrow + mb * 32 + 4 * CROW);
#pragma unroll
        for (int hb = 0; hb < NHB; ++hb) acc[mb][hb] = Elem<T>::mfma16(a, pb[hb], acc[mb][hb] * al[hb]);
      }
    }
  }
  ring_wait<0>();                     // drain the clamped look-ahead loads before the workgroup's LDS is released
  if (SCORES) return;

  // ---- epilogue: normalise, write partial + lse --------------------------------------------------------------------
  if (ssub == 0) { ml_lds[2 * srow] = m_run; ml_lds[2 * srow + 1] = l_run; }
  __syncthreads();
#pragma unroll
  for (int hb = 0; hb < NHB; ++hb) {
    const int hrow = hb * 16 + n16;
    if (hrow < hg) {
      const float m = ml_lds[2 * hrow], l = ml_lds[2 * hrow + 1];
      const float inv = 1.f / l;
      const int64_t ph = ((int64_t)b * p.hq + h0 + hrow) * p.max_splits + split;
      float* dst = p.partial + ph * DV + vcol0 + 4 * g4;
#pragma unroll
      for (int mb = 0; mb < NVB; ++mb) *reinterpret_cast<f32x4*>(dst + mb * 16) = acc[mb][hb] * inv;
      if (wave == 0 && g4 == 0) p.lse[ph] = m + __logf(l);
    }
  }
}

template <typename T, int NHB, bool LO, int DN, bool HAS_R, bool SCORES>
static int launch_ring_t(const RingParams& p, int batch, hipStream_t st) {
  constexpr int HB = 16 * NHB;
  constexpr size_t SLOT = (size_t)RTN * (DN * 2 + 16) + (HAS_R ? RTN * 128 : 0);
  constexpr size_t SHM = RSLOT * SLOT + 2 * HB * RSP * 4 + HB * RLDP * 2 + HB * 4 + HB * 8;
  static_assert(SHM <= 160 * 1024, "ring does not fit the LDS");
  auto kern = latent_ring_kernel<T, NHB, LO, DN, HAS_R, SCORES>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)SHM);
  if (e != hipSuccess) return (int)e;
  const int total = batch * p.groups * p.max_splits;
  kern<<<dim3((total + 7) & ~7), dim3(256), SHM, st>>>(p);
  return launch_status();
}

template <typename T>
static int launch_ring_dt(const RingParams& p, int batch, hipStream_t st) {
  const int hg = p.hq / p.groups;
  const bool lo = p.qn_lo != nullptr, r = p.R != nullptr, sc = p.scores != nullptr;
  if (p.dn != 512) return XKV_EUNSUPPORTED;
#define XKV_RING_CASE(NHB, LO, HAS_R, SC) \
  if ((hg <= 16) == (NHB == 1) && lo == LO && r == HAS_R && sc == SC) return launch_ring_t<T, NHB, LO, 512, HAS_R, SC>(p, batch, st);
  XKV_RING_CASE(1, false, false, false) XKV_RING_CASE(1, false, true, false)
  XKV_RING_CASE(2, false, false, false) XKV_RING_CASE(2, false, true, false)
  XKV_RING_CASE(1, true, false, false)  XKV_RING_CASE(2, true, false, false)
  XKV_RING_CASE(1, true, false, true)   XKV_RING_CASE(2, true, false, true)
  XKV_RING_CASE(1, false, false, true)  XKV_RING_CASE(2, false, false, true)
#undef XKV_RING_CASE
  return XKV_EUNSUPPORTED;
}

bool ring_eligible(const RingParams& p, bool vshared) {
  const int hg = p.hq / p.groups;
  if (hg > 32 || p.dn != 512) return false;
  if (p.R && p.dr != 64) return false;
  if (p.R && p.qn_lo) return false;
  if (!p.scores && (!vshared || p.dv != 512)) return false;
  if (p.scores && p.R) return false;
  if (p.sCl < p.dn || (p.R && p.sRl < 64)) return false;
  // the RoPE-key load addresses rows with a 32-bit byte offset from the sequence's first row
  if (p.R && (int64_t)p.kv_len * p.sRl * 2 >= (int64_t)1 << 31) return false;
  return true;
}

int launch_ring(const RingParams& p, int batch, int dtype, hipStream_t st) {
  return dtype == XKV_BF16 ? launch_ring_dt<__bf16>(p, batch, st) : launch_ring_dt<_Float16>(p, batch, st);
}

}  // namespace xkv
