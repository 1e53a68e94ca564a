// Split-K stage 1 with fused key reconstruction and RoPE:
//   K = kA @ kB[kh]  ->  rotate-half RoPE in registers  ->  q_pe . K'  ->  online softmax  ->  P @ vA
// K never exists outside registers.
//
// One workgroup (4 wavefronts) owns one (batch, kv head, split).  The kv head's factor
// kB[kh] (rank x 128) is STATIONARY IN REGISTERS for the whole workgroup: wave w holds the
// columns {16w..16w+15} and {64+16w..64+16w+15} - both members of every rotate-half pair -
// as MFMA A operands (rank/32 x 2 packets).  The shared token basis kA streams through LDS
// in 32-token tiles and is the B operand, so each v_mfma_f32_16x16x32 yields
// K^T[16 features x 16 tokens] with a lane holding 4 features j..j+3 AND their partners
// j+64.. of one token: the rotation is lane-local.  The rotated tile, rounded to the operand
// type, is directly the A operand of the q-dot MFMA (contraction index = the lane's 8
// features), so scores need no LDS round trip either; only the 4 per-wave partial score
// blocks (a quarter of head_dim each) are summed through LDS.
//
// cos/sin of the absolute position come from angle addition: per-lane constants for the
// in-tile offset (0..31) times a per-tile base rotation that is re-seeded with a fully
// range-reduced sincosf every 32 tiles and advanced by a constant rotation in between.
#include "xkv_common.h"
#include "recon_fast.h"
#include <mutex>

namespace xkv {

struct ReconParams {
  const void* q; const void* kA; const void* kB; const void* vA;
  int64_t sAb, sAl, sBb, sBh, sBr, sVb, sVl;
  int rank, dv;
  float* partial; float* lse; void* scores; int scores_dtype;
  const int32_t* num_splits; const int32_t* kv_lens;
  int hq, hkv, kv_len, max_splits, total_wg;
  float sm_scale;
  int rope; const float* inv_freq; int64_t pos_offset;
  const void* sin_cos; int64_t sSCl;
};


typedef short s16x4r __attribute__((ext_vector_type(4)));
typedef short s16x8r __attribute__((ext_vector_type(8)));
template <typename V8>
__device__ __forceinline__ V8 tr_operand_r(const void* p0, const void* p1) {
  s16x4r a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4r*)p0);
  s16x4r b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4r*)p1);
  s16x8r r = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(V8, r);
}

constexpr int RTN = 32;  // tokens per tile

template <typename T, int NKS, bool EXACT, int NVB_MAX, bool VSHARED, bool SCORES_ONLY>
__global__ __launch_bounds__(256) void recon_stage1_kernel(const ReconParams p) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int NPK_A = (RTN * NKS * 4) / 256;                 // 16-byte packets of an A tile per thread
  constexpr int NPK_V = (VSHARED || SCORES_ONLY) ? 0 : (RTN * NVB_MAX * 8) / 256;
  constexpr int LDS_S = RTN + 4;
  constexpr int LDP = RTN + 8;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n16 = lane & 15, g4 = lane >> 4;

  const int wg = xcd_cluster_remap(blockIdx.x, p.hkv);   // the kv heads of one (sequence, split) share an L2
  if (wg >= p.total_wg) return;
  const int kh = wg % p.hkv;
  const int split = (wg / p.hkv) % p.max_splits;
  const int b = wg / (p.hkv * p.max_splits);
  const int L = p.kv_lens ? p.kv_lens[b] : p.kv_len;
  int start, end;
  split_bounds(L, p.num_splits[b], split, start, end);
  if (end <= start) return;

  const int G = p.hq / p.hkv, h0 = kh * G;
  const int nks = EXACT ? NKS : (p.rank >> 5);
  const int lda = p.rank + 8, ldv = VSHARED ? lda : p.dv + 8;

  T* atile = reinterpret_cast<T*>(smem);
  T* vtile = (VSHARED || SCORES_ONLY) ? atile : atile + RTN * lda;
  float* s_part = reinterpret_cast<float*>(vtile + ((VSHARED || SCORES_ONLY) ? RTN * lda : RTN * ldv));  // [4][16][LDS_S]
  T* p_lds = reinterpret_cast<T*>(s_part + 4 * 16 * LDS_S);
  float* alpha_lds = reinterpret_cast<float*>(p_lds + 16 * LDP);
  float* ml_lds = alpha_lds + 16;

  // ---- stationary operands -------------------------------------------------------------------
  // feature index of this lane's r-th accumulator row in column block mblk: mblk*64 + 16*wave + 4*g4 + r
  const T* Bh = reinterpret_cast<const T*>(p.kB) + b * p.sBb + kh * p.sBh;
  vec8 breg[NKS][2];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      vec8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (EXACT || ks < nks) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = Bh[(int64_t)(ks * 32 + 8 * g4 + e) * p.sBr + mb * 64 + 16 * wave + n16];
      }
      breg[ks][mb] = v;
    }
  // q operand of the q-dot: lane (n16 = head, g4) holds q[head][4 low features | 4 partner features]
  sc_vec8 qop = {0, 0, 0, 0, 0, 0, 0, 0};
  if (n16 < G) {
    const T* qh = reinterpret_cast<const T*>(p.q) + ((int64_t)b * p.hq + h0 + n16) * 128;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      qop[e] = from_f32<sc_t>(to_f32(qh[16 * wave + 4 * g4 + e]));
      qop[4 + e] = from_f32<sc_t>(to_f32(qh[64 + 16 * wave + 4 * g4 + e]));
    }
  }
  // RoPE constants for this lane's 4 pair indices j = 16*wave + 4*g4 + r
  float invf[4], ci[2][4], si[2][4], c32[4], s32[4], cb[4], sb[4];
  const bool computed_rope = p.rope && !p.sin_cos;
  if (computed_rope) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      invf[r] = p.inv_freq[16 * wave + 4 * g4 + r];
#pragma unroll
      for (int tb = 0; tb < 2; ++tb) sincosf((float)(tb * 16 + n16) * invf[r], &si[tb][r], &ci[tb][r]);
      sincosf((float)RTN * invf[r], &s32[r], &c32[r]);
    }
  }

  // ---- tile staging ---------------------------------------------------------------------------
  const T* Ab = reinterpret_cast<const T*>(p.kA) + b * p.sAb;
  const T* Vb = NPK_V ? reinterpret_cast<const T*>(p.vA) + b * p.sVb : nullptr;
  int a_row[NPK_A], a_col[NPK_A];
  int v_row[NPK_V > 0 ? NPK_V : 1], v_col[NPK_V > 0 ? NPK_V : 1];
  const int ppr_a = p.rank >> 3, ppr_v = p.dv >> 3;
#pragma unroll
  for (int k = 0; k < NPK_A; ++k) {
    int i = tid + 256 * k;
    a_row[k] = i / ppr_a;
    a_col[k] = (i - a_row[k] * ppr_a) << 3;
    if (a_row[k] >= RTN) a_row[k] = -1;
  }
#pragma unroll
  for (int k = 0; k < NPK_V; ++k) {
    int i = tid + 256 * k;
    v_row[k] = i / ppr_v;
    v_col[k] = (i - v_row[k] * ppr_v) << 3;
    if (v_row[k] >= RTN) v_row[k] = -1;
  }
  vec8 a_reg[NPK_A], v_reg[NPK_V > 0 ? NPK_V : 1];
  const int last = end - 1;
  auto issue_loads = [&](int base) {
#pragma unroll
    for (int k = 0; k < NPK_A; ++k)
      if (a_row[k] >= 0) {
        int t = base + a_row[k];
        t = t < last ? t : last;
        a_reg[k] = ld16<vec8>(Ab + (int64_t)t * p.sAl + a_col[k]);
      }
#pragma unroll
    for (int k = 0; k < NPK_V; ++k)
      if (v_row[k] >= 0) {
        int t = base + v_row[k];
        t = t < last ? t : last;
        v_reg[k] = ld16<vec8>(Vb + (int64_t)t * p.sVl + v_col[k]);
      }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int k = 0; k < NPK_A; ++k)
      if (a_row[k] >= 0) st16(atile + a_row[k] * lda + a_col[k], a_reg[k]);
#pragma unroll
    for (int k = 0; k < NPK_V; ++k)
      if (v_row[k] >= 0) st16(vtile + v_row[k] * ldv + v_col[k], v_reg[k]);
  };

  // ---- running state ---------------------------------------------------------------------------
  const int srow = tid >> 4, ssub = tid & 15;  // softmax role: 16 threads per head row, 2 tokens each
  float m_run = NEG_INF, l_run = 0.f;
  f32x4 acc[SCORES_ONLY ? 1 : NVB_MAX];
#pragma unroll
  for (int mb = 0; mb < (SCORES_ONLY ? 1 : NVB_MAX); ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int nvb = p.dv >> 6;
  const int vcol0 = wave * (p.dv >> 2);

  issue_loads(start);
  int tile_idx = 0;
  for (int base = start; base < end; base += RTN, ++tile_idx) {
    store_tile();
    __syncthreads();
    if (base + RTN < end) issue_loads(base + RTN);

    // ---- base rotation of this tile -------------------------------------------------------------
    if (computed_rope) {
      if ((tile_idx & 31) == 0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) sincosf((float)(p.pos_offset + base) * invf[r], &sb[r], &cb[r]);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float c = cb[r] * c32[r] - sb[r] * s32[r];
          float s = sb[r] * c32[r] + cb[r] * s32[r];
          cb[r] = c; sb[r] = s;
        }
      }
    }

    // ---- reconstruct -> rotate -> q-dot, per 16-token block -------------------------------------
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
      f32x4 k0 = {0.f, 0.f, 0.f, 0.f}, k1 = {0.f, 0.f, 0.f, 0.f};
      const T* trow = atile + (tb * 16 + n16) * lda + 8 * g4;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks)
        if (EXACT || ks < nks) {
          vec8 at = ld16<vec8>(trow + ks * 32);
          k0 = Elem<T>::mfma16(breg[ks][0], at, k0);
          k1 = Elem<T>::mfma16(breg[ks][1], at, k1);
        }
      // lane (n16 = token, g4): k0[r] = K[token][16w+4g+r], k1[r] = K[token][64+16w+4g+r]
      sc_vec8 kop;
      if (p.rope) {
        float c[4], s[4];
        if (computed_rope) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            c[r] = cb[r] * ci[tb][r] - sb[r] * si[tb][r];
            s[r] = sb[r] * ci[tb][r] + cb[r] * si[tb][r];
          }
        } else {
          int t = base + tb * 16 + n16;
          t = t < last ? t : last;
          const T* sc = reinterpret_cast<const T*>(p.sin_cos) + (int64_t)t * p.sSCl + 16 * wave + 4 * g4;
#pragma unroll
          for (int r = 0; r < 4; ++r) { s[r] = to_f32(sc[r]); c[r] = to_f32(sc[64 + r]); }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          kop[r] = from_f32<sc_t>(k0[r] * c[r] - k1[r] * s[r]);
          kop[4 + r] = from_f32<sc_t>(k1[r] * c[r] + k0[r] * s[r]);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) { kop[r] = from_f32<sc_t>(k0[r]); kop[4 + r] = from_f32<sc_t>(k1[r]); }
      }
      f32x4 sp = {0.f, 0.f, 0.f, 0.f};
      sp = Elem<sc_t>::mfma16(kop, qop, sp);  // lane (n16 = head, g4): tokens tb*16 + 4*g4 + r
      *reinterpret_cast<f32x4*>(s_part + (wave * 16 + n16) * LDS_S + tb * 16 + 4 * g4) = sp;
    }
    __syncthreads();

    if (SCORES_ONLY) {
      // 16 head rows x 32 tokens; thread -> (head = tid/32 (+8), token = tid%32)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int head = (tid >> 5) + 8 * hh, tok = tid & 31;
        if (head < G && base + tok < end) {
          float s = 0.f;
#pragma unroll
          for (int w = 0; w < 4; ++w) s += s_part[(w * 16 + head) * LDS_S + tok];
          s *= p.sm_scale;
          const int64_t o = ((int64_t)b * p.hq + h0 + head) * p.kv_len + base + tok;
          if (p.scores_dtype == XKV_F32) reinterpret_cast<float*>(p.scores)[o] = s;
          else reinterpret_cast<T*>(p.scores)[o] = from_f32<T>(s);
        }
      }
      __syncthreads();
      continue;
    }

    // ---- online softmax ---------------------------------------------------------------------------
    {
      float sv[2];
      float mx = NEG_INF;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int tok = ssub * 2 + i;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) s += s_part[(w * 16 + srow) * LDS_S + tok];
        s *= p.sm_scale;
        sv[i] = (base + tok < end) ? s : NEG_INF;
        mx = fmaxf(mx, sv[i]);
      }
#pragma unroll
      for (int o = 1; o < 16; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __expf(m_run - m_new);
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        float e = __expf(sv[i] - m_new);
        sum += e;
        p_lds[srow * LDP + ssub * 2 + i] = from_f32<T>(e);
      }
#pragma unroll
      for (int o = 1; o < 16; o <<= 1) sum += __shfl_xor(sum, o);
      l_run = l_run * alpha + sum;
      m_run = m_new;
      if (ssub == 0) alpha_lds[srow] = alpha;
    }
    __syncthreads();

    // ---- PV in rank space --------------------------------------------------------------------------
    {
      const float al = alpha_lds[n16];
      vec8 pb = ld16<vec8>(p_lds + n16 * LDP + 8 * g4);
      const T* vrow = vtile + (8 * g4 + (n16 >> 2)) * ldv + vcol0 + 4 * (n16 & 3);
#pragma unroll
      for (int mb = 0; mb < NVB_MAX; ++mb)
        if (mb < nvb) {
          vec8 a = tr_operand_r<vec8>(vrow + mb * 16, vrow + mb * 16 + 4 * ldv);
          acc[mb] = Elem<T>::mfma16(a, pb, acc[mb] * al);
        }
    }
    __syncthreads();
  }
  if (SCORES_ONLY) return;

  if (ssub == 0) { ml_lds[2 * srow] = m_run; ml_lds[2 * srow + 1] = l_run; }
  __syncthreads();
  if (n16 < G) {
    const float m = ml_lds[2 * n16], l = ml_lds[2 * n16 + 1];
    const float inv = 1.f / l;
    const int64_t ph = ((int64_t)b * p.hq + h0 + n16) * p.max_splits + split;
    float* dst = p.partial + ph * p.dv + vcol0 + 4 * g4;
#pragma unroll
    for (int mb = 0; mb < NVB_MAX; ++mb)
      if (mb < nvb) *reinterpret_cast<f32x4*>(dst + mb * 16) = acc[mb] * inv;
    if (wave == 0 && g4 == 0) p.lse[ph] = m + __logf(l);
  }
}

template <typename T, int NKS, bool EXACT, int NVB_MAX, bool VSHARED, bool SCORES_ONLY>
static int launch_recon(const ReconParams& p, int batch, hipStream_t st) {
  const int lda = p.rank + 8, ldv = VSHARED ? lda : p.dv + 8;
  size_t shm = (size_t)RTN * lda * 2;
  if (!VSHARED && !SCORES_ONLY) shm += (size_t)RTN * ldv * 2;
  shm += 4 * 16 * (RTN + 4) * 4 + 16 * (RTN + 8) * 2 + 16 * 4 + 16 * 8;
  auto kern = recon_stage1_kernel<T, NKS, EXACT, NVB_MAX, VSHARED, SCORES_ONLY>;
  static DynLds lds;
  const int e = ensure_dynamic_lds(lds, reinterpret_cast<const void*>(kern), (int)shm);
  if (e != XKV_OK) return e;
  const int total = batch * p.hkv * p.max_splits;
  kern<<<dim3(xcd_grid(total, p.hkv)), dim3(256), shm, st>>>(p);
  return launch_status();
}

template <typename T>
static int dispatch_recon(const ReconParams& p, int batch, bool vshared, hipStream_t st) {
  const bool so = p.scores != nullptr;
  if (p.rank == 512) {
    if (so) return launch_recon<T, 16, true, 8, true, true>(p, batch, st);
    return vshared ? launch_recon<T, 16, true, 8, true, false>(p, batch, st)
                   : launch_recon<T, 16, true, 8, false, false>(p, batch, st);
  }
#define XKV_RECON_RANK(R)                                                                      \
  if (p.rank == R) {                                                                           \
    if (so) return launch_recon<T, R / 32, true, 8, true, true>(p, batch, st);                 \
    return vshared ? launch_recon<T, R / 32, true, 8, true, false>(p, batch, st)               \
                   : launch_recon<T, R / 32, true, 8, false, false>(p, batch, st);             \
  }
  // exact instantiations (no per-k-step bound checks, registers sized to the rank) for the common ranks
  XKV_RECON_RANK(384) XKV_RECON_RANK(256) XKV_RECON_RANK(192) XKV_RECON_RANK(128)
#undef XKV_RECON_RANK
  if (so) return launch_recon<T, 16, false, 8, true, true>(p, batch, st);
  return vshared ? launch_recon<T, 16, false, 8, true, false>(p, batch, st)
                 : launch_recon<T, 16, false, 8, false, false>(p, batch, st);
}

}  // namespace xkv

using namespace xkv;

extern "C" int64_t xkv_recon_workspace_bytes(int batch, int hkv, int rank, int64_t stride_kB_b) {
  if (rank != 512 && rank != 384 && rank != 256) return 0;
  return (int64_t)(stride_kB_b == 0 ? 1 : batch) * hkv * rank * 128 * 2;
}

extern "C" int xkv_recon_stage1(const void* q_pe, xkv_kv_operand kA, const void* kB, int64_t sBb, int64_t sBh,
                                int64_t sBr, xkv_kv_operand vA, float* partial, float* lse, void* scores_out,
                                int scores_dtype, const int32_t* num_kv_splits, const int32_t* kv_lens, int batch,
                                int hq, int hkv, int kv_len, int max_splits, float sm_scale, int rope,
                                const float* inv_freq, int64_t pos_offset, const void* sin_cos, int64_t sc_stride_l,
                                void* workspace, int64_t workspace_bytes, int dtype, void* stream) {
  if (!q_pe || !kA.ptr || !kB || !num_kv_splits || batch <= 0 || hq <= 0 || hkv <= 0 || kv_len <= 0 || max_splits <= 0)
    return XKV_EINVAL;
  const bool so = scores_out != nullptr;
  if (!so && (!vA.ptr || !partial || !lse)) return XKV_EINVAL;
  if (rope && !inv_freq && !sin_cos) return XKV_EINVAL;
  if (dtype != XKV_BF16 && dtype != XKV_F16) return XKV_EDTYPE;
  if (so && scores_dtype != XKV_F32 && scores_dtype != dtype) return XKV_EDTYPE;
  if (hq % hkv || hq / hkv > 16) return XKV_EUNSUPPORTED;
  const int rank = kA.dim;
  if (rank <= 0 || rank % 32 || rank > 512) return XKV_EUNSUPPORTED;
  if (!so && (vA.dim <= 0 || vA.dim % 64 || vA.dim > 512)) return XKV_EUNSUPPORTED;
  if ((kA.stride_b & 7) || (kA.stride_l & 7) || (reinterpret_cast<uintptr_t>(kA.ptr) & 15)) return XKV_EALIGN;
  if (!so && ((vA.stride_b & 7) || (vA.stride_l & 7) || (reinterpret_cast<uintptr_t>(vA.ptr) & 15))) return XKV_EALIGN;

  ReconParams p;
  p.q = q_pe; p.kA = kA.ptr; p.kB = kB; p.vA = vA.ptr;
  p.sAb = kA.stride_b; p.sAl = kA.stride_l; p.sBb = sBb; p.sBh = sBh; p.sBr = sBr;
  p.sVb = vA.stride_b; p.sVl = vA.stride_l;
  p.rank = rank; p.dv = so ? 64 : vA.dim;
  p.partial = partial; p.lse = lse; p.scores = scores_out; p.scores_dtype = scores_dtype;
  p.num_splits = num_kv_splits; p.kv_lens = kv_lens;
  p.hq = hq; p.hkv = hkv; p.kv_len = kv_len; p.max_splits = max_splits; p.total_wg = batch * hkv * max_splits;
  p.sm_scale = sm_scale; p.rope = rope; p.inv_freq = inv_freq; p.pos_offset = pos_offset;
  p.sin_cos = sin_cos; p.sSCl = sc_stride_l;
  const bool vshared = !so && vA.ptr == kA.ptr && vA.stride_b == kA.stride_b && vA.stride_l == kA.stride_l &&
                       vA.dim == kA.dim;
  hipStream_t st = (hipStream_t)stream;
  // MFMA-bound fast path: rank 512 / 384 / 256, scores only or a basis shared by K and V, computed RoPE angles, at most 8 query heads
  // per kv head
  const int64_t need = xkv_recon_workspace_bytes(batch, hkv, rank, sBb);
  if ((so || vshared) && rope && !sin_cos && (rank == 512 || rank == 384 || rank == 256) && hq / hkv <= 8 && workspace && need > 0 &&
      workspace_bytes >= need && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0) {
    FastParams f;
    f.q = q_pe; f.kA = kA.ptr; f.Bp = workspace;
    f.sAb = kA.stride_b; f.sAl = kA.stride_l; f.sBpb = sBb == 0 ? 0 : (int64_t)hkv * rank * 128;
    f.partial = partial; f.lse = lse; f.scores = scores_out; f.scores_dtype = scores_dtype;
    f.num_splits = num_kv_splits; f.kv_lens = kv_lens;
    f.hq = hq; f.hkv = hkv; f.kv_len = kv_len; f.max_splits = max_splits; f.total_wg = batch * hkv * max_splits;
    f.sm_scale = sm_scale; f.inv_freq = inv_freq; f.pos_offset = pos_offset;
    // Scores only at rank 256: the 4-wave kernel, the one instantiation small enough for two workgroups per CU (measured
    // 10 - 15 % ahead there).  Everything else: the wave-specialised kernel (8 - 13 % ahead of the 4-wave kernel).
    if (!(so && rank == 256)) return launch_recon_spec(f, kB, sBb, sBh, sBr, batch, dtype, rank, st);
    return launch_recon_fast_256(f, kB, sBb, sBh, sBr, batch, dtype, st);
  }
  // 8-wave kernels: a value basis of its own beside key ranks 256 / 384 / 512
  if (!so && !vshared && rope && !sin_cos && hq / hkv <= 8 && workspace && need > 0 && workspace_bytes >= need &&
      (reinterpret_cast<uintptr_t>(workspace) & 15) == 0 && (int64_t)kA.stride_l * 2 * 3 < ((int64_t)1 << 31) &&
      (int64_t)vA.stride_l * 2 * 3 < ((int64_t)1 << 31)) {
    FastParams f;
    f.q = q_pe; f.kA = kA.ptr; f.Bp = workspace;
    f.sAb = kA.stride_b; f.sAl = kA.stride_l; f.sBpb = sBb == 0 ? 0 : (int64_t)hkv * rank * 128;
    f.partial = partial; f.lse = lse; f.scores = nullptr; f.scores_dtype = scores_dtype;
    f.num_splits = num_kv_splits; f.kv_lens = kv_lens;
    f.hq = hq; f.hkv = hkv; f.kv_len = kv_len; f.max_splits = max_splits; f.total_wg = batch * hkv * max_splits;
    f.sm_scale = sm_scale; f.inv_freq = inv_freq; f.pos_offset = pos_offset;
    f.vA = vA.ptr; f.sVb = vA.stride_b; f.sVl = vA.stride_l;
    int rc = launch_recon_duo_b(f, kB, sBb, sBh, sBr, batch, dtype, 2, rank, vA.dim, st);
    if (rc == DUO_NOT_MINE) rc = launch_recon_duo_c(f, kB, sBb, sBh, sBr, batch, dtype, 2, rank, vA.dim, st);
    if (rc != DUO_NOT_MINE) return rc;
  }
  return dtype == XKV_BF16 ? dispatch_recon<__bf16>(p, batch, vshared, st) : dispatch_recon<_Float16>(p, batch, vshared, st);
}

// ---------------------------------------------------------------------------------------------------------------------
// The same stage 1 for callers that cannot allocate: the packed copy of kB lives in a file-scope device array instead of
// a caller workspace.  Every GPU holds its own copy of the array at its own address; the address is looked up once per
// device (first call with that device current) and kept.  The array's NAME is only a host-side handle for that lookup:
// kernels and copies always get the looked-up pointer.
// ---------------------------------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[XKV_STATIC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
void* scratch_ptr[MAX_DEVICES];   // device address of `scratch` on each GPU, NULL until looked up

int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= MAX_DEVICES) return XKV_EUNSUPPORTED;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return (int)hipErrorInvalidSymbol;
    scratch_ptr[dev] = ptr;
  }
  *out = scratch_ptr[dev];
  return XKV_OK;
}
}  // namespace

extern "C" int xkv_recon_stage1_static(const void* q_pe, xkv_kv_operand kA, const void* kB, int64_t sBb, int64_t sBh,
                                       int64_t sBr, xkv_kv_operand vA, float* partial, float* lse, void* scores_out,
                                       int scores_dtype, const int32_t* num_kv_splits, const int32_t* kv_lens,
                                       int batch, int hq, int hkv, int kv_len, int max_splits, float sm_scale, int rope,
                                       const float* inv_freq, int64_t pos_offset, const void* sin_cos,
                                       int64_t sc_stride_l, int dtype, void* stream) {
  if (batch <= 0 || hkv <= 0) return XKV_EINVAL;
  int64_t need = xkv_recon_workspace_bytes(batch, hkv, kA.dim, sBb);
  // only the MFMA-bound paths (generated angles, at most 8 query heads per kv head) pack kB; every other shape runs the
  // generic kernel, which needs no scratch
  if (!(rope && !sin_cos && hq > 0 && hq % hkv == 0 && hq / hkv <= 8)) need = 0;
  if (need > (int64_t)XKV_STATIC_SCRATCH_BYTES) return XKV_ESCRATCH;   // nothing is launched
  void* ws = nullptr;
  if (need > 0) {
    const int rc = static_scratch(&ws);
    if (rc != XKV_OK) return rc;
  }
  return xkv_recon_stage1(q_pe, kA, kB, sBb, sBh, sBr, vA, partial, lse, scores_out, scores_dtype, num_kv_splits, kv_lens,
                          batch, hq, hkv, kv_len, max_splits, sm_scale, rope, inv_freq, pos_offset, sin_cos, sc_stride_l,
                          ws, need, dtype, stream);
}
