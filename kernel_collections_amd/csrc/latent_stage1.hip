// Split-K flash-decoding stage 1 over dot-product scores:  s = sm_scale * q . C_l,  partial = softmax(s) V.
//
// One workgroup (4 wavefronts) owns one (batch, kv group, split) and walks its token range in
// tiles of TN tokens.  Per tile:
//   load   C (and R, and V when it is a different tensor) rows global -> registers -> LDS, the
//          next tile's loads being issued before this tile's math (the registers are the
//          second buffer, so HBM latency overlaps the MFMA work);
//   QK     S^T[token, head] on v_mfma_f32_16x16x32: A operand = tile rows straight from LDS
//          (8 consecutive features per lane), B operand = the query rows kept in LDS;
//   softmax running max / sum per head, P written to LDS in the operand type;
//   PV     acc^T[feature, head] += V^T P^T on the same MFMA, each wave owning a quarter of the
//          V features; the token-major operand comes from the row-major tile through
//          ds_read_b64_tr_b16 (4 tokens x 16 features transposed per 16 lanes).
// When V is the same tensor as C (MLA latent, xKV with a basis shared by K and V) the tile is
// loaded once and used for both products.
#include "xkv_common.h"
#include "latent_ring.h"

namespace xkv {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

// 4 tokens x 16 features transposed: lane j of each 16-lane group passes the address of
// tile[t0 + j/4][c0 + 4*(j%4)] and receives tile[t0 .. t0+3][c0 + j].
template <typename V8>
__device__ __forceinline__ V8 tr_operand(const void* p0, const void* p1) {
  s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p0);
  s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p1);
  s16x8 r = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(V8, r);
}

template <typename T, int NHB, int TN, int NVB_MAX, int NPK_C, int NPK_R, int NPK_V, bool VSHARED, bool SCORES_ONLY>
__global__ __launch_bounds__(256) void latent_stage1_kernel(const LatentParams p) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int HB = 16 * NHB;       // head rows held (zero padded)
  constexpr int NTB = TN / 16;       // 16-token blocks per tile (one per wave)
  constexpr int TPH = 256 / HB;      // softmax threads per head
  constexpr int TPT = TN / TPH;      // tokens per softmax thread
  constexpr int LDS_S = TN + 4;      // fp32 score row stride
  constexpr int LDP = TN + 8;        // P row stride (elements)
  static_assert(TPT >= 1 && NTB <= 4, "tile shape");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n16 = lane & 15, g4 = lane >> 4;

  const int wg = xcd_cluster_remap(blockIdx.x, p.groups);   // the kv groups of one (sequence, split) share an L2
  if (wg >= p.total_wg) return;
  const int group = wg % p.groups;
  int split = (wg / p.groups) % p.max_splits;
  int b = wg / (p.groups * p.max_splits);
  if (p.split_plan) {   // job list: the live (sequence, split) pairs come first in the grid
    const int job = wg / p.groups;
    if (job >= p.split_plan[1]) return;
    b = p.split_plan[2 + 2 * job];
    split = p.split_plan[3 + 2 * job];
  }

  const int L = p.kv_lens ? p.kv_lens[b] : p.kv_len;
  int start, end;
  split_bounds(L, effective_splits(L, p.num_splits[b], split_cap_in_force(p.split_cap, p.split_plan)), split, start, end);
  if (end <= start) return;

  const int hg = p.hq / p.groups;  // heads of this kv group
  const int h0 = group * hg;
  const int dtot = p.dn + p.dr;
  const int ldc = dtot + 8;        // tile row stride (elements), +16 B so 16 rows hit distinct banks
  const int ldv = VSHARED ? ldc : p.dv + 8;

  // ---- LDS carve-up ------------------------------------------------------------------------
  T* ctile = reinterpret_cast<T*>(smem);
  T* vtile = VSHARED ? ctile : ctile + TN * ldc;
  T* qs = vtile + (VSHARED ? TN * ldc : TN * ldv);
  T* qlo = qs + HB * ldc;
  unsigned char* after_q = reinterpret_cast<unsigned char*>(qlo + (p.qn_lo ? HB * ldc : 0));
  float* s_lds = reinterpret_cast<float*>(after_q);
  T* p_lds = reinterpret_cast<T*>(s_lds + HB * LDS_S);
  float* alpha_lds = reinterpret_cast<float*>(p_lds + HB * LDP);
  float* ml_lds = alpha_lds + HB;

  // ---- query rows -> LDS ([qn | qr], zero rows above hg) -----------------------------------
  {
    const int ppr = dtot >> 3;
    for (int i = tid; i < HB * ppr; i += 256) {
      const int row = i / ppr, cp = (i - row * ppr) << 3;
      vec8 v = {0, 0, 0, 0, 0, 0, 0, 0}, vl = {0, 0, 0, 0, 0, 0, 0, 0};
      if (row < hg) {
        const int64_t qh = (int64_t)b * p.hq + h0 + row;
        if (cp < p.dn) {
          v = ld16<vec8>(reinterpret_cast<const T*>(p.qn) + qh * p.dn + cp);
          if (p.qn_lo) vl = ld16<vec8>(reinterpret_cast<const T*>(p.qn_lo) + qh * p.dn + cp);
        } else {
          v = ld16<vec8>(reinterpret_cast<const T*>(p.qr) + qh * p.dr + (cp - p.dn));
        }
      }
      st16(qs + row * ldc + cp, v);
      if (p.qn_lo) st16(qlo + row * ldc + cp, vl);
    }
  }

  // ---- per-thread packet plan (same for every tile; division only here) ---------------------
  const T* Cb = reinterpret_cast<const T*>(p.C) + b * p.sCb + group * p.sCh;
  const T* Rb = p.dr ? reinterpret_cast<const T*>(p.R) + b * p.sRb + group * p.sRh : nullptr;
  const T* Vb = (!VSHARED && !SCORES_ONLY) ? reinterpret_cast<const T*>(p.V) + b * p.sVb + group * p.sVh : nullptr;
  int c_row[NPK_C > 0 ? NPK_C : 1], c_col[NPK_C > 0 ? NPK_C : 1];
  int r_row[NPK_R > 0 ? NPK_R : 1], r_col[NPK_R > 0 ? NPK_R : 1];
  int v_row[NPK_V > 0 ? NPK_V : 1], v_col[NPK_V > 0 ? NPK_V : 1];
  const int ppr_c = p.dn >> 3, ppr_r = p.dr >> 3, ppr_v = p.dv >> 3;
#pragma unroll
  for (int k = 0; k < NPK_C; ++k) {
    int i = tid + 256 * k;
    c_row[k] = i / ppr_c;
    c_col[k] = (i - c_row[k] * ppr_c) << 3;
    if (c_row[k] >= TN) c_row[k] = -1;
  }
#pragma unroll
  for (int k = 0; k < NPK_R; ++k) {
    int i = tid + 256 * k;
    r_row[k] = ppr_r ? i / ppr_r : TN;
    r_col[k] = ppr_r ? (i - r_row[k] * ppr_r) << 3 : 0;
    if (r_row[k] >= TN) r_row[k] = -1;
  }
#pragma unroll
  for (int k = 0; k < NPK_V; ++k) {
    int i = tid + 256 * k;
    v_row[k] = i / ppr_v;
    v_col[k] = (i - v_row[k] * ppr_v) << 3;
    if (v_row[k] >= TN) v_row[k] = -1;
  }

  vec8 c_reg[NPK_C > 0 ? NPK_C : 1], r_reg[NPK_R > 0 ? NPK_R : 1], v_reg[NPK_V > 0 ? NPK_V : 1];
  const int last = end - 1;
  auto issue_loads = [&](int base) {
#pragma unroll
    for (int k = 0; k < NPK_C; ++k)
      if (c_row[k] >= 0) {
        int t = base + c_row[k];
        t = t < last ? t : last;  // rows past the split end are masked later; keep the read in bounds
        c_reg[k] = ld16<vec8>(Cb + (int64_t)t * p.sCl + c_col[k]);
      }
#pragma unroll
    for (int k = 0; k < NPK_R; ++k)
      if (r_row[k] >= 0) {
        int t = base + r_row[k];
        t = t < last ? t : last;
        r_reg[k] = ld16<vec8>(Rb + (int64_t)t * p.sRl + r_col[k]);
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
    for (int k = 0; k < NPK_C; ++k)
      if (c_row[k] >= 0) st16(ctile + c_row[k] * ldc + c_col[k], c_reg[k]);
#pragma unroll
    for (int k = 0; k < NPK_R; ++k)
      if (r_row[k] >= 0) st16(ctile + r_row[k] * ldc + p.dn + r_col[k], r_reg[k]);
#pragma unroll
    for (int k = 0; k < NPK_V; ++k)
      if (v_row[k] >= 0) st16(vtile + v_row[k] * ldv + v_col[k], v_reg[k]);
  };

  // ---- running state ---------------------------------------------------------------------
  const int srow = tid / TPH, ssub = tid % TPH;  // softmax role
  float m_run = NEG_INF, l_run = 0.f;
  f32x4 acc[SCORES_ONLY ? 1 : NVB_MAX][NHB];
#pragma unroll
  for (int mb = 0; mb < (SCORES_ONLY ? 1 : NVB_MAX); ++mb)
#pragma unroll
    for (int hb = 0; hb < NHB; ++hb) acc[mb][hb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int nvb = p.dv >> 6;          // 16-feature blocks per wave (dv / 4 / 16)
  const int vcol0 = wave * (p.dv >> 2);
  const int nks = dtot >> 5, nks_n = p.dn >> 5;
  const bool has_lo = p.qn_lo != nullptr;

  issue_loads(start);
  for (int base = start; base < end; base += TN) {
    store_tile();
    __syncthreads();
    if (base + TN < end) issue_loads(base + TN);

    // ---- QK ------------------------------------------------------------------------------
    if (wave < NTB) {
      f32x4 sacc[NHB], sacc_lo[NHB];
#pragma unroll
      for (int hb = 0; hb < NHB; ++hb) { sacc[hb] = f32x4{0.f, 0.f, 0.f, 0.f}; sacc_lo[hb] = f32x4{0.f, 0.f, 0.f, 0.f}; }
      const T* arow = ctile + (wave * 16 + n16) * ldc + 8 * g4;
      const T* qrow = qs + n16 * ldc + 8 * g4;
      const T* lrow = qlo + n16 * ldc + 8 * g4;
      for (int ks = 0; ks < nks; ++ks) {
        vec8 a = ld16<vec8>(arow + ks * 32);
#pragma unroll
        for (int hb = 0; hb < NHB; ++hb) {
          vec8 bq = ld16<vec8>(qrow + hb * 16 * ldc + ks * 32);
          sacc[hb] = Elem<T>::mfma16(a, bq, sacc[hb]);
        }
        if (has_lo && ks < nks_n) {
#pragma unroll
          for (int hb = 0; hb < NHB; ++hb) {
            vec8 bq = ld16<vec8>(lrow + hb * 16 * ldc + ks * 32);
            sacc_lo[hb] = Elem<T>::mfma16(a, bq, sacc_lo[hb]);
          }
        }
      }
      // lane (n16 = head, g4): tokens wave*16 + 4*g4 + r
      const int tok0 = base + wave * 16 + 4 * g4;
#pragma unroll
      for (int hb = 0; hb < NHB; ++hb) {
        f32x4 sv;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float s = (sacc[hb][r] + sacc_lo[hb][r]) * p.sm_scale;
          if (p.logit_cap > 0.f) s = p.logit_cap * tanhf(s / p.logit_cap);
          sv[r] = (tok0 + r < end) ? s : NEG_INF;
        }
        const int hrow = hb * 16 + n16;
        if (SCORES_ONLY) {
          if (hrow < hg) {
            const int64_t o = ((int64_t)b * p.hq + h0 + hrow) * p.kv_len + tok0;
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (tok0 + r < end) {
                if (p.scores_dtype == XKV_F32) reinterpret_cast<float*>(p.scores)[o + r] = sv[r];
                else reinterpret_cast<T*>(p.scores)[o + r] = from_f32<T>(sv[r]);
              }
          }
        } else {
          *reinterpret_cast<f32x4*>(s_lds + hrow * LDS_S + wave * 16 + 4 * g4) = sv;
        }
      }
    }
    if (SCORES_ONLY) {
      __syncthreads();  // tile fully consumed before the next store_tile
      continue;
    }
    __syncthreads();

    // ---- online softmax (TPH threads per head row) ------------------------------------------
    {
      float sv[TPT];
      float mx = NEG_INF;
#pragma unroll
      for (int i = 0; i < TPT; ++i) { sv[i] = s_lds[srow * LDS_S + ssub * TPT + i]; mx = fmaxf(mx, sv[i]); }
#pragma unroll
      for (int o = 1; o < TPH; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __expf(m_run - m_new);
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < TPT; ++i) {
        float e = __expf(sv[i] - m_new);
        sum += e;
        p_lds[srow * LDP + ssub * TPT + i] = from_f32<T>(e);
      }
#pragma unroll
      for (int o = 1; o < TPH; o <<= 1) sum += __shfl_xor(sum, o);
      l_run = l_run * alpha + sum;
      m_run = m_new;
      if (ssub == 0) alpha_lds[srow] = alpha;
    }
    __syncthreads();

    // ---- PV --------------------------------------------------------------------------------
    {
      float al[NHB];
#pragma unroll
      for (int hb = 0; hb < NHB; ++hb) al[hb] = alpha_lds[hb * 16 + n16];
#pragma unroll
      for (int mb = 0; mb < NVB_MAX; ++mb)
        if (mb < nvb) {
#pragma unroll
          for (int hb = 0; hb < NHB; ++hb) acc[mb][hb] *= al[hb];
        }
#pragma unroll
      for (int kk = 0; kk < TN / 32; ++kk) {
        vec8 pb[NHB];
#pragma unroll
        for (int hb = 0; hb < NHB; ++hb) pb[hb] = ld16<vec8>(p_lds + (hb * 16 + n16) * LDP + kk * 32 + 8 * g4);
        const T* vrow = vtile + (kk * 32 + 8 * g4 + (n16 >> 2)) * ldv + vcol0 + 4 * (n16 & 3);
#pragma unroll
        for (int mb = 0; mb < NVB_MAX; ++mb)
          if (mb < nvb) {
            vec8 a = tr_operand<vec8>(vrow + mb * 16, vrow + mb * 16 + 4 * ldv);
#pragma unroll
            for (int hb = 0; hb < NHB; ++hb) acc[mb][hb] = Elem<T>::mfma16(a, pb[hb], acc[mb][hb]);
          }
      }
    }
    __syncthreads();
  }
  if (SCORES_ONLY) return;

  // ---- epilogue: normalise, write partial + lse --------------------------------------------
  if (ssub == 0) { ml_lds[2 * srow] = m_run; ml_lds[2 * srow + 1] = l_run; }
  __syncthreads();
#pragma unroll
  for (int hb = 0; hb < NHB; ++hb) {
    const int hrow = hb * 16 + n16;
    if (hrow < hg) {
      const float m = ml_lds[2 * hrow], l = ml_lds[2 * hrow + 1];
      const float inv = 1.f / l;
      const int64_t ph = ((int64_t)b * p.hq + h0 + hrow) * p.max_splits + split;
      float* dst = p.partial + ph * p.dv + vcol0 + 4 * g4;
#pragma unroll
      for (int mb = 0; mb < NVB_MAX; ++mb)
        if (mb < nvb) *reinterpret_cast<f32x4*>(dst + mb * 16) = acc[mb][hb] * inv;
      if (wave == 0 && g4 == 0) p.lse[ph] = m + __logf(l);
    }
  }
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
template <typename T, int NHB, int TN, int NVB_MAX, int NPK_C, int NPK_R, int NPK_V, bool VSHARED, bool SCORES_ONLY>
static int launch_latent(const LatentParams& p, int batch, hipStream_t st) {
  constexpr int HB = 16 * NHB;
  const int dtot = p.dn + p.dr, ldc = dtot + 8, ldv = VSHARED ? ldc : p.dv + 8;
  // operands must fit the per-thread packet plan of this instantiation
  if (TN * (p.dn >> 3) > NPK_C * 256) return XKV_EUNSUPPORTED;
  if (TN * (p.dr >> 3) > NPK_R * 256) return XKV_EUNSUPPORTED;
  if (!VSHARED && !SCORES_ONLY && TN * (p.dv >> 3) > NPK_V * 256) return XKV_EUNSUPPORTED;
  if (!SCORES_ONLY && (p.dv >> 6) > NVB_MAX) return XKV_EUNSUPPORTED;
  size_t shm = (size_t)TN * ldc * 2;
  if (!VSHARED && !SCORES_ONLY) shm += (size_t)TN * ldv * 2;
  shm += (size_t)HB * ldc * 2 * (p.qn_lo ? 2 : 1);
  shm += (size_t)HB * (TN + 4) * 4 + (size_t)HB * (TN + 8) * 2 + HB * 4 + HB * 8;
  if (shm > 160 * 1024) return XKV_EUNSUPPORTED;
  auto kern = latent_stage1_kernel<T, NHB, TN, NVB_MAX, NPK_C, NPK_R, NPK_V, VSHARED, SCORES_ONLY>;
  static DynLds lds;
  const int e = ensure_dynamic_lds(lds, reinterpret_cast<const void*>(kern), (int)shm);
  if (e != XKV_OK) return e;
  const int total = batch * p.groups * p.max_splits;
  const int grid = xcd_grid(total, p.groups);
  kern<<<dim3(grid), dim3(256), shm, st>>>(p);
  return launch_status();
}

template <typename T, int NHB>
static int dispatch_latent(const LatentParams& p, int batch, bool vshared, hipStream_t st) {
  if (p.scores) return launch_latent<T, NHB, 64, 1, 16, 4, 0, true, true>(p, batch, st);
  if (vshared) return launch_latent<T, NHB, 64, 8, 16, 4, 0, true, false>(p, batch, st);
  // distinct V: small operands (plain GQA heads) keep 64-token tiles, wide ones drop to 32
  if (p.dn <= 256 && p.dr == 0 && p.dv <= 128) return launch_latent<T, NHB, 64, 2, 8, 0, 4, false, false>(p, batch, st);
  return launch_latent<T, NHB, 32, 8, 16, 2, 8, false, false>(p, batch, st);
}

}  // namespace xkv

using namespace xkv;

static bool aligned8(int64_t s) { return (s & 7) == 0; }
static bool ptr16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

extern "C" int xkv_latent_stage1(xkv_q_operand qn, const void* qn_lo, xkv_q_operand qr, xkv_kv_operand C,
                                 xkv_kv_operand R, xkv_kv_operand V, float* partial, float* lse, void* scores_out,
                                 int scores_dtype, const int32_t* num_kv_splits, const int32_t* kv_lens, int batch,
                                 int hq, int n_kv_groups, int kv_len, int max_splits, int split_cap_tokens,
                                 const int32_t* split_plan, float sm_scale,
                                 float logit_cap,
                                 int dtype, void* stream) {
  if (!qn.ptr || !C.ptr || !num_kv_splits || batch <= 0 || hq <= 0 || n_kv_groups <= 0 || kv_len <= 0 ||
      max_splits <= 0)
    return XKV_EINVAL;
  // with a cap the longest sequence may need cdiv(kv_len, cap) splits: the workspace must have a row for each
  if (split_cap_tokens < 0 || (split_cap_tokens > 0 && max_splits < cdiv(kv_len, split_cap_tokens))) return XKV_EINVAL;
  if (split_plan && split_cap_tokens <= 0) return XKV_EINVAL;   // the host value is what bounds the workspaces
  const bool scores_only = scores_out != nullptr;
  if (!scores_only && (!V.ptr || !partial || !lse)) return XKV_EINVAL;
  if (dtype != XKV_BF16 && dtype != XKV_F16) return XKV_EDTYPE;
  if (scores_only && scores_dtype != XKV_F32 && scores_dtype != dtype) return XKV_EDTYPE;
  if (hq % n_kv_groups) return XKV_EUNSUPPORTED;
  const int hg = hq / n_kv_groups;
  if (hg > 32) return XKV_EUNSUPPORTED;
  if (qn.dim != C.dim || C.dim <= 0 || C.dim % 32 || C.dim > 1024) return XKV_EUNSUPPORTED;
  const int dr = (qr.ptr && R.ptr) ? R.dim : 0;
  if ((qr.ptr != nullptr) != (R.ptr != nullptr)) return XKV_EINVAL;
  if (dr && (qr.dim != R.dim || dr % 32 || dr > 128)) return XKV_EUNSUPPORTED;
  if (!scores_only && (V.dim <= 0 || V.dim % 64 || V.dim > 512)) return XKV_EUNSUPPORTED;
  if (!aligned8(C.stride_b) || !aligned8(C.stride_l) || !aligned8(C.stride_h) || !ptr16(C.ptr) || !ptr16(qn.ptr))
    return XKV_EALIGN;
  if (dr && (!aligned8(R.stride_b) || !aligned8(R.stride_l) || !aligned8(R.stride_h) || !ptr16(R.ptr) || !ptr16(qr.ptr)))
    return XKV_EALIGN;
  if (!scores_only && (!aligned8(V.stride_b) || !aligned8(V.stride_l) || !aligned8(V.stride_h) || !ptr16(V.ptr)))
    return XKV_EALIGN;
  if (qn_lo && !ptr16(qn_lo)) return XKV_EALIGN;

  LatentParams p;
  p.qn = qn.ptr; p.qn_lo = qn_lo; p.qr = dr ? qr.ptr : nullptr;
  p.C = C.ptr; p.R = dr ? R.ptr : nullptr; p.V = V.ptr;
  p.sCb = C.stride_b; p.sCl = C.stride_l; p.sCh = C.stride_h;
  p.sRb = R.stride_b; p.sRl = R.stride_l; p.sRh = R.stride_h;
  p.sVb = V.stride_b; p.sVl = V.stride_l; p.sVh = V.stride_h;
  p.dn = C.dim; p.dr = dr; p.dv = scores_only ? 64 : V.dim;
  p.partial = partial; p.lse = lse; p.scores = scores_out; p.scores_dtype = scores_dtype;
  p.num_splits = num_kv_splits; p.kv_lens = kv_lens;
  p.hq = hq; p.groups = n_kv_groups; p.kv_len = kv_len; p.max_splits = max_splits; p.split_cap = split_cap_tokens;
  p.split_plan = split_plan;
  p.total_wg = batch * n_kv_groups * max_splits;
  p.sm_scale = sm_scale; p.logit_cap = logit_cap;
  p.heads_in_row = 0;
  const bool vshared = !scores_only && V.ptr == C.ptr && V.stride_b == C.stride_b && V.stride_l == C.stride_l &&
                       V.stride_h == C.stride_h && V.dim == C.dim;
  hipStream_t st = (hipStream_t)stream;
  // Plain keys of 8 kv heads x 128 side by side in a token row, values either laid out the same way or one shared
  // 256 .. 512-wide row (V = v_A): one workgroup serves every head of a split.  A token's keys are then one 1024-wide row
  // against a block-diagonal query (which the kernel builds from the compact rows), so whole 2 KiB rows stream through
  // the LDS ring and the shared value row is read once per token instead of once per kv head.
  if (!scores_only && !qn_lo && !dr && C.dim == 128 && n_kv_groups == 8 && C.stride_h == 128 && C.stride_l >= 1024 &&
      hq <= 32) {
    const bool v_heads = V.dim == 128 && V.stride_h == 128 && V.stride_l >= 1024;
    const bool v_shared_row = V.stride_h == 0 && (V.dim == 256 || V.dim == 384 || V.dim == 512) && V.stride_l >= V.dim;
    if (v_heads || v_shared_row) {
      LatentParams w = p;
      w.dn = 1024; w.sCh = 0; w.heads_in_row = 8;
      if (v_shared_row) { w.groups = 1; w.total_wg = batch * max_splits; }
      if (ring_eligible(w, false)) return launch_ring(w, batch, false, dtype, st);
    }
  }
  if (ring_eligible(p, vshared)) return launch_ring(p, batch, vshared, dtype, st);
  if (dtype == XKV_BF16)
    return hg <= 16 ? dispatch_latent<__bf16, 1>(p, batch, vshared, st) : dispatch_latent<__bf16, 2>(p, batch, vshared, st);
  return hg <= 16 ? dispatch_latent<_Float16, 1>(p, batch, vshared, st) : dispatch_latent<_Float16, 2>(p, batch, vshared, st);
}

extern "C" int xkv_softmax_pv_stage1(const float* scores, xkv_kv_operand V, float* partial, float* lse,
                                     const int32_t* num_kv_splits, const int32_t* kv_lens, int batch, int hq, int kv_len,
                                     int max_splits, int split_cap_tokens, const int32_t* split_plan, int dtype, void* stream) {
  if (!scores || !V.ptr || !partial || !lse || !num_kv_splits || batch <= 0 || hq <= 0 || kv_len <= 0 || max_splits <= 0)
    return XKV_EINVAL;
  if (split_cap_tokens < 0 || (split_cap_tokens > 0 && max_splits < cdiv(kv_len, split_cap_tokens))) return XKV_EINVAL;
  if (split_plan && split_cap_tokens <= 0) return XKV_EINVAL;
  if (dtype != XKV_BF16 && dtype != XKV_F16) return XKV_EDTYPE;
  if (hq > 32 || (V.dim != 512 && V.dim != 384 && V.dim != 256) || V.stride_h != 0 || V.stride_l < V.dim || (kv_len & 3))
    return XKV_EUNSUPPORTED;
  if (!aligned8(V.stride_b) || !aligned8(V.stride_l) || !ptr16(V.ptr) || !ptr16(scores)) return XKV_EALIGN;
  LatentParams p;
  p.qn = nullptr; p.qn_lo = nullptr; p.qr = nullptr;
  p.C = V.ptr; p.R = nullptr; p.V = V.ptr;
  p.sCb = V.stride_b; p.sCl = V.stride_l; p.sCh = 0;
  p.sRb = p.sRl = p.sRh = 0;
  p.sVb = V.stride_b; p.sVl = V.stride_l; p.sVh = 0;
  p.dn = V.dim; p.dr = 0; p.dv = V.dim;
  p.partial = partial; p.lse = lse; p.scores = const_cast<float*>(scores); p.scores_dtype = XKV_F32;
  p.num_splits = num_kv_splits; p.kv_lens = kv_lens;
  p.hq = hq; p.groups = 1; p.kv_len = kv_len; p.max_splits = max_splits; p.split_cap = split_cap_tokens;
  p.split_plan = split_plan;
  p.total_wg = batch * max_splits;
  p.sm_scale = 1.f; p.logit_cap = 0.f;
  p.heads_in_row = 0;
  return launch_ring_given(p, batch, dtype, (hipStream_t)stream);
}
