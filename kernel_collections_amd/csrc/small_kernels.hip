// RoPE table, query absorption and the stage-2 merge: the small kernels around the scans.
#include "xkv_common.h"

namespace xkv {

// ----------------------------------------------------------------------------------------------
// RoPE table.  angle = float(pos) * inv_freq[j] in fp32 (one rounding), then sincosf with full
// range reduction - the eager closed form of the reference (rope/rope_ref.py:3-9), not the
// fast-math pow/sin/cos of its Triton table kernel.
// ----------------------------------------------------------------------------------------------
template <typename O>
__global__ void rope_table_kernel(O* __restrict__ sin_out, O* __restrict__ cos_out,
                                  const float* __restrict__ inv_freq, int64_t seqlen, int64_t start,
                                  int half_dim) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= seqlen * half_dim) return;
  int j = (int)(idx % half_dim);
  int64_t l = idx / half_dim;
  float ang = (float)(start + l) * inv_freq[j];
  float s, c;
  sincosf(ang, &s, &c);
  sin_out[idx] = (O)s;
  cos_out[idx] = (O)c;
}

// ----------------------------------------------------------------------------------------------
// Rotate-half RoPE applied to rows x[b, r, h, :] at position (positions ? positions[b] : pos0) + r: one thread per pair
// (j, j + dim/2), fp32 angle float(pos) * inv_freq[j] and fp32 arithmetic as in the eager form (rope/rope_ref.py:3-20).
// ----------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void rope_apply_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                          const float* __restrict__ inv_freq,
                                                          const int64_t* __restrict__ positions, int64_t pos0, int64_t total,
                                                          int rows, int heads, int half, int64_t sxb, int64_t sxr, int64_t sxh,
                                                          int64_t sob, int64_t sor, int64_t soh) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int j = (int)(idx % half);
  int64_t t = idx / half;
  const int h = (int)(t % heads);
  t /= heads;
  const int r = (int)(t % rows);
  const int64_t b = t / rows;
  const int64_t pos = (positions ? positions[b] : pos0) + r;
  float s, c;
  sincosf((float)pos * inv_freq[j], &s, &c);
  const T* xi = x + b * sxb + r * sxr + h * sxh;
  T* oi = out + b * sob + r * sor + h * soh;
  const float x0 = (float)xi[j], x1 = (float)xi[j + half];
  oi[j] = (T)(x0 * c - x1 * s);
  oi[j + half] = (T)(x1 * c + x0 * s);
}

// ----------------------------------------------------------------------------------------------
// qt[b,h,rho] = sum_d q[b,h,d] * B[b,h/G,rho,d]; one workgroup per (kv head, batch), one thread
// per rho (strided), the G query rows of the kv head held in LDS as fp32.
// ----------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void absorb_q_kernel(
    const T* __restrict__ q, const T* __restrict__ B, T* __restrict__ qt_hi, T* __restrict__ qt_lo,
    int hq, int hkv, int d, int rank, int64_t sBb, int64_t sBh, int64_t sBr) {
  typedef typename Elem<T>::vec8 vec8;
  __shared__ float qs[32 * 256];
  const int kh = blockIdx.x, b = blockIdx.y, Gall = hq / hkv;
  const int HC = 8192 / d < 32 ? 8192 / d : 32;   // heads whose query rows fit the LDS buffer at a time
  const T* Bh = B + b * sBb + kh * sBh;
  for (int gc = 0; gc < Gall; gc += HC) {
  const int G = Gall - gc < HC ? Gall - gc : HC;
  const T* qb = q + ((int64_t)b * hq + (int64_t)kh * Gall + gc) * d;
  __syncthreads();
  for (int i = threadIdx.x; i < G * d; i += blockDim.x) qs[i] = to_f32(qb[i]);
  __syncthreads();
  for (int rho = blockIdx.z * blockDim.x + threadIdx.x; rho < rank; rho += blockDim.x * gridDim.z) {
    const T* row = Bh + rho * sBr;
    for (int g0 = 0; g0 < G; g0 += 4) {
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
      for (int c = 0; c < d; c += 8) {
        vec8 v = ld16<vec8>(row + c);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float x = to_f32(v[e]);
#pragma unroll
          for (int gi = 0; gi < 4; ++gi)
            if (g0 + gi < G) acc[gi] += x * qs[(g0 + gi) * d + c + e];
        }
      }
#pragma unroll
      for (int gi = 0; gi < 4; ++gi)
        if (g0 + gi < G) {
          int64_t o = ((int64_t)b * hq + (int64_t)kh * Gall + gc + g0 + gi) * rank + rho;
          T hi = from_f32<T>(acc[gi]);
          qt_hi[o] = hi;
          if (qt_lo) qt_lo[o] = from_f32<T>(acc[gi] - to_f32(hi));
        }
    }
  }
  }
}

// Same product for head_dim 64 / 128 / 256 / 512 with coalesced reads: TPR = d / 8 consecutive lanes cover one row of B
// (16 bytes each), 256 / TPR rows per pass; the per-row dot products are finished by a lane reduction.  A workgroup
// takes ABS_ROWS rows of B and up to ABS_HEADS query heads of one kv head (their rows sit in LDS as fp32), so that
// even a single sequence with one kv head spreads over tens of CUs.
constexpr int ABS_ROWS = 16, ABS_HEADS = 8;
template <typename T, int TPR>
__global__ __launch_bounds__(256) void absorb_q_rows_kernel(
    const T* __restrict__ q, const T* __restrict__ B, T* __restrict__ qt_hi, T* __restrict__ qt_lo,
    int hq, int hkv, int rank, int64_t sBb, int64_t sBh, int64_t sBr, int nhc) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int D = TPR * 8, RPP = 256 / TPR;
  __shared__ float qs[ABS_HEADS * D];
  const int kh = blockIdx.x / nhc, g0 = (blockIdx.x % nhc) * ABS_HEADS, b = blockIdx.y, G = hq / hkv;
  const int gn = G - g0 < ABS_HEADS ? G - g0 : ABS_HEADS;
  const int sub = threadIdx.x % TPR, rr = threadIdx.x / TPR;
  const T* Bh = B + b * sBb + kh * sBh;
  const T* qb = q + ((int64_t)b * hq + (int64_t)kh * G + g0) * D;
  for (int i = threadIdx.x; i < gn * D; i += 256) qs[i] = to_f32(qb[i]);
  __syncthreads();
  for (int r0 = 0; r0 < ABS_ROWS; r0 += RPP) {
    const int rho = blockIdx.z * ABS_ROWS + r0 + rr;
    const bool live = rho < rank && rr < ABS_ROWS;
    float x[8];
    {
      vec8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (live) v = ld16<vec8>(Bh + (int64_t)rho * sBr + sub * 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = to_f32(v[e]);
    }
    for (int g = 0; g < gn; ++g) {
      const f32x4 qa = *reinterpret_cast<const f32x4*>(qs + g * D + sub * 8);
      const f32x4 qb4 = *reinterpret_cast<const f32x4*>(qs + g * D + sub * 8 + 4);
      float a = x[0] * qa[0] + x[1] * qa[1] + x[2] * qa[2] + x[3] * qa[3] + x[4] * qb4[0] + x[5] * qb4[1] +
                x[6] * qb4[2] + x[7] * qb4[3];
      a = row_reduce<false, (TPR < 16 ? TPR : 16)>(a);
      if (TPR >= 32) a += __shfl_xor(a, 16);
      if (TPR >= 64) a += __shfl_xor(a, 32);
      if (live && sub == (g % TPR)) {
        const int64_t o = ((int64_t)b * hq + (int64_t)kh * G + g0 + g) * rank + rho;
        const T hi = from_f32<T>(a);
        qt_hi[o] = hi;
        if (qt_lo) qt_lo[o] = from_f32<T>(a - to_f32(hi));
      }
    }
  }
}

// ----------------------------------------------------------------------------------------------
// Block-diagonal query: out[b, h, kh * d + c] = q[b, h, c] if kh == h / G else 0.  With it the per-head keys of a token,
// stored side by side ([batch, kv_len, hkv * d]), act as ONE wide row shared by every head, so a single workgroup can
// serve all query heads of a sequence (and read a value basis shared by the heads once instead of once per kv head).
// ----------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void blockdiag_q_kernel(const T* __restrict__ q, T* __restrict__ out, int hq, int hkv, int d,
                                                          int64_t total8) {
  typedef typename Elem<T>::vec8 vec8;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;   // one 8-element packet of out
  if (i >= total8) return;
  const int ppr = hkv * d / 8, dp = d / 8;
  const int64_t row = i / ppr;            // b * hq + h
  const int pk = (int)(i - row * ppr);
  const int kh = pk / dp, c = (pk - kh * dp) * 8;
  const int h = (int)(row % hq), G = hq / hkv;
  vec8 v = {0, 0, 0, 0, 0, 0, 0, 0};
  if (kh == h / G) v = ld16<vec8>(q + row * d + c);
  st16(out + i * 8, v);
}

// ----------------------------------------------------------------------------------------------
// Stage 2.  One workgroup per (kv head, batch), or per (query head, batch) when there are many splits: merges the live splits of its query heads
// (reference order: increasing split id, running max of lse), then optionally multiplies the
// merged rank-space rows by vB[b, kh] (read once for the G heads).
// ----------------------------------------------------------------------------------------------
constexpr int MERGE_RED_FLOATS = 32 * 4 * 64, MERGE_FIN_FLOATS = 4 * 512;   // the kernel's static LDS (the launcher counts it)
template <typename O, typename TB>
__global__ __launch_bounds__(256) void merge_stage2_kernel(
    const float* __restrict__ partial, const float* __restrict__ lse, O* __restrict__ out,
    const TB* __restrict__ vB, int64_t sVb, int64_t sVh, int64_t sVr, int d_out,
    const int32_t* __restrict__ num_kv_splits, const int32_t* __restrict__ kv_lens,
    int hq, int hkv, int kv_len, int max_splits, int dv, int64_t sOb, int64_t sOh, int hpw,
    float* __restrict__ lse_out, int64_t sLb, int64_t sLh, int d_blk, int split_cap, const int32_t* __restrict__ split_plan) {
  extern __shared__ float merged[];  // [G][dv], then the split weights [G][max_splits]
  __shared__ float fin[MERGE_FIN_FLOATS];     // per-head-block totals of the up-projection
  // this workgroup: heads hfirst .. hfirst + G - 1 of sequence b, all of kv head kh (G = hpw divides the GQA group size)
  const int G = hpw, hfirst = blockIdx.x * hpw, kh = hfirst / (hq / hkv), b = blockIdx.y;
  // blockIdx.z: a block of d_blk output columns of the up-projection (every block repeats the merge: when the grid is
  // small the partial rows are read from more CUs at once, which is what bounds a single long sequence)
  if (blockIdx.z > 0) {
    const int cz = blockIdx.z * d_blk;
    vB += cz;
    out += cz;
    d_out = d_out - cz < d_blk ? d_out - cz : d_blk;
    lse_out = nullptr;
  } else if (d_blk < d_out) {
    d_out = d_blk;
  }
  const int L = kv_lens ? kv_lens[b] : kv_len;
  const int ns = effective_splits(L, num_kv_splits[b], split_cap_in_force(split_cap, split_plan));
  float* wts = merged + G * dv;
  int nlive = 0;
  {
    const int per = ns > 0 ? cdiv(cdiv(L, ns), MIN_BLOCK_KV) * MIN_BLOCK_KV : 0;
    nlive = per > 0 ? cdiv(L, per) : 0;
    nlive = nlive < max_splits ? nlive : max_splits;
  }
  // weights of the live splits, w_i = exp(lse_i - max lse) / sum: one wave per head, lanes stride over the splits
  {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int gi = wave; gi < G; gi += 4) {
      const float* pl = lse + ((int64_t)b * hq + hfirst + gi) * max_splits;
      float mx = NEG_INF;
      for (int i = lane; i < max_splits; i += 64) {
        int s0, e0;
        split_bounds(L, ns, i, s0, e0);
        const float v = e0 > s0 ? pl[i] : NEG_INF;   // dead splits were never written
        wts[gi * max_splits + i] = v;
        mx = fmaxf(mx, v);
      }
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
      float sum = 0.f;
      for (int i = lane; i < max_splits; i += 64) {
        const float v = wts[gi * max_splits + i];
        const float w = v == NEG_INF ? 0.f : __expf(v - mx);
        wts[gi * max_splits + i] = w;
        sum += w;
      }
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) sum += __shfl_xor(sum, o);
      const float inv = 1.f / sum;
      for (int i = lane; i < max_splits; i += 64) wts[gi * max_splits + i] *= inv;
      if (lse_out && lane == 0) lse_out[b * sLb + (hfirst + gi) * sLh] = mx + __logf(sum);   // log-sum-exp of the merged range
    }
  }
  __syncthreads();
  // weighted sum of the live splits (a prefix of the split range: split i is live iff per * i < L), 16 bytes per load.
  // Work item = 4 consecutive features of one head; when there are fewer items than threads the threads form split
  // groups (split i goes to group i % nsg) whose sums meet in LDS, so that a single long sequence still has 256 loads
  // in flight per workgroup.
  if ((dv & 3) == 0 && (reinterpret_cast<uintptr_t>(partial) & 15) == 0) {
    const int items = G * dv / 4;
    const int lanes_per = items < 256 ? items : 256;
    const int nsg = 256 / lanes_per, sg = threadIdx.x / lanes_per;
    for (int item = threadIdx.x % lanes_per; item < items && sg < nsg; item += lanes_per) {
      const int gi = (item * 4) / dv, c = item * 4 - gi * dv;
      const int h = hfirst + gi;
      const float* pp = partial + ((int64_t)b * hq + h) * max_splits * (int64_t)dv + c;
      const float* w = wts + gi * max_splits;
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
      for (int i = sg; i < nlive; i += nsg) acc += w[i] * *reinterpret_cast<const f32x4*>(pp + (int64_t)i * dv);
      if (nsg == 1) {
        if (vB) {
          *reinterpret_cast<f32x4*>(merged + item * 4) = acc;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) out[b * sOb + h * sOh + c + e] = (O)acc[e];
        }
      } else {
        *reinterpret_cast<f32x4*>(fin + (sg * items + item) * 4) = acc;   // nsg * items * 4 <= 1024 floats
      }
    }
    if (nsg > 1) {
      __syncthreads();
      for (int idx = threadIdx.x; idx < G * dv; idx += blockDim.x) {
        const int gi = idx / dv, c = idx - gi * dv;
        float acc = 0.f;
        for (int k = 0; k < nsg; ++k) acc += fin[k * items * 4 + idx];
        if (vB)
          merged[idx] = acc;
        else
          out[b * sOb + (hfirst + gi) * sOh + c] = (O)acc;
      }
      __syncthreads();   // fin is reused by the up-projection
    }
  } else {
    for (int idx = threadIdx.x; idx < G * dv; idx += blockDim.x) {
      const int gi = idx / dv, c = idx - gi * dv;
      const int h = hfirst + gi;
      const float* pp = partial + ((int64_t)b * hq + h) * max_splits * (int64_t)dv + c;
      const float* w = wts + gi * max_splits;
      float acc = 0.f;
#pragma unroll 8
      for (int i = 0; i < nlive; ++i) acc += w[i] * pp[(int64_t)i * dv];
      if (vB)
        merged[idx] = acc;
      else
        out[b * sOb + h * sOh + c] = (O)acc;
    }
  }
  if (!vB) return;
  __syncthreads();
  // out[g][c] = sum_rho merged[g][rho] * vB[rho][c].  Thread -> (8 output columns, one of 256/ncb rank groups): 16-byte
  // loads of vB, several in flight, then a reduction over the rank groups through LDS.
  typedef typename Elem<TB>::vec8 vec8;
  const TB* Bh = vB + b * sVb + kh * sVh;
  __shared__ float red[MERGE_RED_FLOATS];            // [rank group][4 heads][columns of the block]: 32 KiB
  const int ncb = (d_out + 7) >> 3;                  // 8-column blocks (d_out <= 512 -> <= 64)
  const int ngrp = 256 / ncb;                        // rank groups
  const int cb = threadIdx.x % ncb, grp = threadIdx.x / ncb;
  const bool active = grp < ngrp && cb * 8 + 8 <= d_out;
  for (int g0 = 0; g0 < G; g0 += 4) {
    float acc[4][8];
#pragma unroll
    for (int gi = 0; gi < 4; ++gi)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[gi][e] = 0.f;
    if (active) {
#pragma unroll 4
      for (int rho = grp; rho < dv; rho += ngrp) {
        const vec8 w = ld16<vec8>(Bh + rho * sVr + cb * 8);
#pragma unroll
        for (int gi = 0; gi < 4; ++gi) {
          const float m = g0 + gi < G ? merged[(g0 + gi) * dv + rho] : 0.f;
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[gi][e] += m * to_f32(w[e]);
        }
      }
    }
    // reduce over the rank groups through LDS, `chunk` groups per pass (as many as fit `red`)
    const int cols = ncb * 8;                        // <= 512
    const int gstride = 4 * cols;                    // a rank group's 4 x cols floats
    const int chunk = MERGE_RED_FLOATS / gstride;    // groups per pass (>= 4): what fits `red`
    for (int base = 0; base < ngrp; base += chunk) {
      __syncthreads();
      if (active && grp >= base && grp < base + chunk) {
#pragma unroll
        for (int gi = 0; gi < 4; ++gi)
#pragma unroll
          for (int e = 0; e < 8; ++e) red[(grp - base) * gstride + gi * cols + cb * 8 + e] = acc[gi][e];
      }
      __syncthreads();
      const int n_here = (ngrp - base) < chunk ? (ngrp - base) : chunk;
      const int nout = 4 * d_out;
      if (nout <= 128 && ngrp <= chunk) {
        // a narrow column block: fewer totals than threads and many rank groups (one pass).  256 / nout threads share a total's
        // groups, so that nobody walks 64 LDS words one after the other; their sums meet in `fin`.
        const int parts = 256 / nout, o = threadIdx.x % nout, part = threadIdx.x / nout;
        const int gi = o / d_out, c = o - gi * d_out;
        float sacc = 0.f;
        if (part < parts) {
#pragma unroll 8
          for (int k = part; k < n_here; k += parts) sacc += red[k * gstride + gi * cols + c];
          fin[part * nout + o] = sacc;
        }
        __syncthreads();
        if (threadIdx.x < nout) {
          float tot = fin[threadIdx.x];
          for (int q = 1; q < parts; ++q) tot += fin[q * nout + threadIdx.x];
          fin[threadIdx.x] = tot;
        }
      } else {
        for (int idx = threadIdx.x; idx < nout; idx += blockDim.x) {
          const int gi = idx / d_out, c = idx - gi * d_out;
          if (g0 + gi < G) {
            float sacc = 0.f;
#pragma unroll 8
            for (int k = 0; k < n_here; ++k) sacc += red[k * gstride + gi * cols + c];
            fin[idx] = (base == 0 ? 0.f : fin[idx]) + sacc;
          }
        }
      }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < 4 * d_out; idx += blockDim.x) {
      const int gi = idx / d_out, c = idx - gi * d_out;
      if (g0 + gi < G) out[b * sOb + (hfirst + g0 + gi) * sOh + c] = (O)fin[idx];
    }
  }
}

template <typename O>
static int launch_rope(void* s, void* c, const float* inv, int64_t seqlen, int64_t start, int half_dim,
                       hipStream_t st) {
  int64_t n = seqlen * half_dim;
  rope_table_kernel<O><<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st>>>((O*)s, (O*)c, inv, seqlen, start,
                                                                               half_dim);
  return launch_status();
}

template <typename O, typename TB>
static int launch_merge(const float* partial, const float* lse, void* out, const void* vB, int64_t sVb, int64_t sVh,
                        int64_t sVr, int d_out, const int32_t* ns, const int32_t* kl, int batch, int hq, int hkv,
                        int kv_len, int max_splits, int dv, int64_t sOb, int64_t sOh, float* lse_out, int64_t sLb, int64_t sLh,
                        int split_cap, const int32_t* split_plan, hipStream_t st) {
  // few splits: one workgroup per kv head (vB read once for its heads); many splits: one per query head, so that the
  // partial rows of a long sequence are spread over more CUs - unless the kv heads alone fill half the device and there
  // is an up-projection, whose vB rows then weigh more than the partial rows
  const int g = hq / hkv;
  const bool enough_wgs = vB && (int64_t)hkv * batch >= 128;   // vB costs more than the partial rows: keep it read once per kv head
  int hpw = (g > 16 || (max_splits > 16 && !enough_wgs)) ? 1 : g;
  if (!vB) hpw = 1;   // nothing is shared by the heads of a kv head without an up-projection: one workgroup per head
  // dynamic LDS beside the kernel's static LDS (the up-projection's reduction buffers): the default limit of 64 KiB per
  // workgroup must hold both; a group of heads that does not fit is merged one head per workgroup, and a single head that
  // does not fit is refused
  constexpr size_t LDS_LIMIT = 64 * 1024, STATIC_LDS = (MERGE_RED_FLOATS + MERGE_FIN_FLOATS) * sizeof(float);
  auto dyn_lds = [&](int heads) { return (size_t)heads * (dv + max_splits) * sizeof(float); };
  while (hpw > 1 && (g % hpw != 0 || dyn_lds(hpw) + STATIC_LDS > LDS_LIMIT)) --hpw;   // the largest group of heads that fits
  const size_t shm = dyn_lds(hpw);
  if (shm + STATIC_LDS > LDS_LIMIT) return XKV_EUNSUPPORTED;
  // a small grid over many splits is bound by the latency of its partial-row loads: split the up-projection's columns
  // over more workgroups
  int zb = 1;
  if (vB && (hq / hpw) * batch < 128 && max_splits >= 64 && d_out % 32 == 0) zb = d_out >= 512 ? 4 : d_out >= 256 ? 2 : 1;
  // few splits: the merge itself is cheap to repeat, and what is left is the latency of the vB rows a thread reads one after
  // the other - column blocks of >= 32 until the grid has 512 workgroups (a thread then reads dv / 64 rows instead of dv / 16)
  if (vB && max_splits <= 16)
    while ((int64_t)(hq / hpw) * batch * zb < 512 && d_out % (zb * 2 * 8) == 0 && d_out / (zb * 2) >= 32) zb *= 2;
  merge_stage2_kernel<O, TB><<<dim3(hq / hpw, batch, zb), dim3(256), shm, st>>>(partial, lse, (O*)out, (const TB*)vB, sVb, sVh,
                                                                               sVr, d_out, ns, kl, hq, hkv, kv_len, max_splits,
                                                                               dv, sOb, sOh, hpw, lse_out, sLb, sLh, d_out / zb, split_cap, split_plan);
  return launch_status();
}

// plan[0]: smallest multiple of 32 >= floor_tokens with sum_b ceil(len_b / cap) <= target_jobs, by a 256-ary search over
// cap / 32 (the job count falls monotonically as the cap grows).  Then the job list: sequence b has n_b = effective_splits(len_b,
// num_splits[b], cap) splits of which the live ones are a prefix; whole splits first (sequence-major), every sequence's last
// live split - the short one - after them.  One workgroup; thread t handles sequences t, t + 256, ...
__global__ __launch_bounds__(256) void plan_splits_kernel(const int32_t* __restrict__ kv_lens, const int32_t* __restrict__ num_splits,
                                                          int batch, int max_splits, int floor_tokens, int target_jobs,
                                                          int32_t* __restrict__ plan) {
  __shared__ int red[4];
  __shared__ int carry;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  auto block_reduce = [&](int v, bool take_max) {
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int w = __shfl_xor(v, o);
      v = take_max ? (w > v ? w : v) : v + w;
    }
    __syncthreads();            // red is free again
    if (lane == 0) red[wave] = v;
    __syncthreads();
    int r = red[0];
#pragma unroll
    for (int i = 1; i < 4; ++i) r = take_max ? (red[i] > r ? red[i] : r) : r + red[i];
    return r;
  };
  int lm = 0;
  for (int b = threadIdx.x; b < batch; b += 256) lm = kv_lens[b] > lm ? kv_lens[b] : lm;
  lm = block_reduce(lm, true);
  int lo = cdiv(floor_tokens > 32 ? floor_tokens : 32, 32), hi = cdiv(lm > 32 ? lm : 32, 32);   // in units of 32 tokens
  if (hi < lo) hi = lo;
  // 256-ary search over [lo, hi]: the range is cut into 256 blocks and thread t tests the LAST cap of block t; the answer
  // lies in the first block whose last cap fits.  If nothing fits - even one job per sequence is too many - it is hi, the
  // longest length.
  __shared__ int first_fit[4];
  while (lo < hi) {
    const int stride = cdiv(hi - lo + 1, 256);
    const int blk_lo = lo + threadIdx.x * stride;
    int blk_hi = blk_lo + stride - 1;
    blk_hi = blk_hi < hi ? blk_hi : hi;
    bool fits = false;
    if (blk_lo <= hi) {
      const int cap = blk_hi * 32;
      int jobs = 0;
      for (int b = 0; b < batch; ++b) jobs += cdiv(kv_lens[b] > 0 ? kv_lens[b] : 0, cap);
      fits = jobs <= target_jobs;
    }
    const unsigned long long m = __builtin_amdgcn_ballot_w64(fits);
    __syncthreads();            // first_fit is free again
    if (lane == 0) first_fit[wave] = m ? wave * 64 + (int)__builtin_ctzll(m) : 1 << 30;
    __syncthreads();
    int t = first_fit[0];
#pragma unroll
    for (int i = 1; i < 4; ++i) t = first_fit[i] < t ? first_fit[i] : t;
    if (t == 1 << 30) { lo = hi; break; }
    const int new_lo = lo + t * stride;
    int new_hi = new_lo + stride - 1;
    new_hi = new_hi < hi ? new_hi : hi;
    lo = new_lo;
    hi = new_hi;                // fits; with stride 1 this ends the search
  }
  const int cap = lo * 32;
  // live splits of a sequence, in the arithmetic of split_bounds
  auto live_of = [&](int b) {
    const int L = kv_lens[b];
    if (L <= 0) return 0;
    const int n = effective_splits(L, num_splits[b], cap);
    const int per = cdiv(cdiv(L, n), MIN_BLOCK_KV) * MIN_BLOCK_KV;
    const int live = cdiv(L, per);
    return live < max_splits ? live : max_splits;
  };
  // exclusive prefix sums over the sequences, 256 at a time: first of (live - 1) whole splits, then of the last splits
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int pass = 0; pass < 2; ++pass) {
    for (int b0 = 0; b0 < batch; b0 += 256) {
      const int b = b0 + threadIdx.x;
      const int live = b < batch ? live_of(b) : 0;
      const int mine = pass == 0 ? (live > 0 ? live - 1 : 0) : (live > 0 ? 1 : 0);
      // inclusive scan within the wave, then across the four waves
      int incl = mine;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int w = __shfl_up(incl, o);
        if (lane >= o) incl += w;
      }
      __syncthreads();
      if (lane == 63) red[wave] = incl;
      __syncthreads();
      int before = carry;
      for (int i = 0; i < wave; ++i) before += red[i];
      const int start = before + incl - mine;
      if (pass == 0) {
        for (int s2 = 0; s2 < mine; ++s2) { plan[2 + 2 * (start + s2)] = b; plan[3 + 2 * (start + s2)] = s2; }
      } else if (mine) {
        plan[2 + 2 * start] = b; plan[3 + 2 * start] = live - 1;
      }
      __syncthreads();
      if (threadIdx.x == 255) carry = start + mine;
      __syncthreads();
    }
  }
  if (threadIdx.x == 0) { plan[0] = cap; plan[1] = carry; }
}

}  // namespace xkv

using namespace xkv;

extern "C" int xkv_plan_splits(const int32_t* kv_lens, const int32_t* num_kv_splits, int batch, int max_splits, int floor_tokens,
                               int target_jobs, int32_t* plan, void* stream) {
  if (!kv_lens || !num_kv_splits || !plan || batch <= 0 || max_splits <= 0 || floor_tokens <= 0 || target_jobs <= 0) return XKV_EINVAL;
  plan_splits_kernel<<<dim3(1), dim3(256), 0, (hipStream_t)stream>>>(kv_lens, num_kv_splits, batch, max_splits, floor_tokens,
                                                                     target_jobs, plan);
  return launch_status();
}

extern "C" int xkv_abi_version(void) { return XKV_ABI_VERSION; }

extern "C" const char* xkv_error_string(int code) {
  switch (code) {
    case XKV_OK: return "ok";
    case XKV_EINVAL: return "invalid argument (null pointer or non-positive size)";
    case XKV_EUNSUPPORTED: return "shape outside the built envelope";
    case XKV_EALIGN: return "pointer or stride not 16-byte aligned";
    case XKV_EDTYPE: return "unsupported dtype code";
    case XKV_ESCRATCH: return "the call needs more scratch than the library's static device array holds";
    case XKV_ETOOLCHAIN: return "a kernel that tracks its own loads was built with register spills: rebuild with the validated compiler";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown xkv error";
  }
}

extern "C" int xkv_rope_table(void* sin_out, void* cos_out, const float* inv_freq, int64_t seqlen, int64_t start,
                              int half_dim, int out_dtype, void* stream) {
  if (!sin_out || !cos_out || !inv_freq || seqlen < 0 || half_dim <= 0) return XKV_EINVAL;
  if (seqlen == 0) return XKV_OK;
  hipStream_t st = (hipStream_t)stream;
  switch (out_dtype) {
    case XKV_F32: return launch_rope<float>(sin_out, cos_out, inv_freq, seqlen, start, half_dim, st);
    case XKV_F16: return launch_rope<_Float16>(sin_out, cos_out, inv_freq, seqlen, start, half_dim, st);
    case XKV_BF16: return launch_rope<__bf16>(sin_out, cos_out, inv_freq, seqlen, start, half_dim, st);
    default: return XKV_EDTYPE;
  }
}

template <typename T>
static int launch_rope_apply(const void* x, void* out, const float* inv_freq, const int64_t* positions, int64_t pos0,
                             int batch, int rows, int heads, int dim, int64_t sxb, int64_t sxr, int64_t sxh, int64_t sob,
                             int64_t sor, int64_t soh, hipStream_t st) {
  const int64_t total = (int64_t)batch * rows * heads * (dim / 2);
  const int64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffff) return XKV_EUNSUPPORTED;
  rope_apply_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, st>>>((const T*)x, (T*)out, inv_freq, positions, pos0, total, rows,
                                                                      heads, dim / 2, sxb, sxr, sxh, sob, sor, soh);
  return launch_status();
}

extern "C" int xkv_rope_apply(const void* x, void* out, const float* inv_freq, const int64_t* positions, int64_t pos0,
                              int batch, int rows, int heads, int dim, int64_t sxb, int64_t sxr, int64_t sxh,
                              int64_t sob, int64_t sor, int64_t soh, int dtype, void* stream) {
  if (!x || !out || !inv_freq || batch < 0 || rows < 0 || heads <= 0 || dim <= 0) return XKV_EINVAL;
  if (dim % 2) return XKV_EUNSUPPORTED;
  if (batch == 0 || rows == 0) return XKV_OK;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case XKV_F32: return launch_rope_apply<float>(x, out, inv_freq, positions, pos0, batch, rows, heads, dim, sxb, sxr, sxh, sob, sor, soh, st);
    case XKV_F16: return launch_rope_apply<_Float16>(x, out, inv_freq, positions, pos0, batch, rows, heads, dim, sxb, sxr, sxh, sob, sor, soh, st);
    case XKV_BF16: return launch_rope_apply<__bf16>(x, out, inv_freq, positions, pos0, batch, rows, heads, dim, sxb, sxr, sxh, sob, sor, soh, st);
    default: return XKV_EDTYPE;
  }
}

extern "C" int xkv_absorb_q(const void* q, const void* B, void* qt_hi, void* qt_lo, int batch, int hq, int hkv, int d,
                            int rank, int64_t sBb, int64_t sBh, int64_t sBr, int dtype, void* stream) {
  if (!q || !B || !qt_hi || batch <= 0 || hq <= 0 || hkv <= 0 || d <= 0 || rank <= 0) return XKV_EINVAL;
  if (hq % hkv || hq / hkv > 32 || d > 512 || d % 8) return XKV_EUNSUPPORTED;
  if (sBr % 8 || sBh % 8 || sBb % 8 || ((uintptr_t)B & 15)) return XKV_EALIGN;
  hipStream_t st = (hipStream_t)stream;
  if (dtype != XKV_BF16 && dtype != XKV_F16) return XKV_EDTYPE;
  const dim3 block(256);
  const int nhc = (hq / hkv + ABS_HEADS - 1) / ABS_HEADS;   // head chunks per kv head
#define XKV_ABSORB(T)                                                                                                         \
  if (d == 128)                                                                                                               \
    absorb_q_rows_kernel<T, 16><<<dim3(hkv * nhc, batch, (rank + ABS_ROWS - 1) / ABS_ROWS), block, 0, st>>>((const T*)q, (const T*)B, (T*)qt_hi,    \
                                                                                        (T*)qt_lo, hq, hkv, rank, sBb, sBh, sBr, nhc); \
  else if (d == 512)                                                                                                          \
    absorb_q_rows_kernel<T, 64><<<dim3(hkv * nhc, batch, (rank + ABS_ROWS - 1) / ABS_ROWS), block, 0, st>>>((const T*)q, (const T*)B, (T*)qt_hi,    \
                                                                                        (T*)qt_lo, hq, hkv, rank, sBb, sBh, sBr, nhc); \
  else if (d == 256)                                                                                                          \
    absorb_q_rows_kernel<T, 32><<<dim3(hkv * nhc, batch, (rank + ABS_ROWS - 1) / ABS_ROWS), block, 0, st>>>((const T*)q, (const T*)B, (T*)qt_hi,    \
                                                                                        (T*)qt_lo, hq, hkv, rank, sBb, sBh, sBr, nhc); \
  else if (d == 64)                                                                                                           \
    absorb_q_rows_kernel<T, 8><<<dim3(hkv * nhc, batch, (rank + ABS_ROWS - 1) / ABS_ROWS), block, 0, st>>>((const T*)q, (const T*)B, (T*)qt_hi,     \
                                                                                       (T*)qt_lo, hq, hkv, rank, sBb, sBh, sBr, nhc); \
  else                                                                                                                        \
    absorb_q_kernel<T><<<dim3(hkv, batch, (rank + 255) / 256), block, 0, st>>>((const T*)q, (const T*)B, (T*)qt_hi, (T*)qt_lo, \
                                                                                 hq, hkv, d, rank, sBb, sBh, sBr);
  if (dtype == XKV_BF16) { XKV_ABSORB(__bf16) } else { XKV_ABSORB(_Float16) }
#undef XKV_ABSORB
  return launch_status();
}

extern "C" int xkv_blockdiag_q(const void* q, void* out, int batch, int hq, int hkv, int d, int dtype, void* stream) {
  if (!q || !out || batch <= 0 || hq <= 0 || hkv <= 0 || d <= 0) return XKV_EINVAL;
  if (hq % hkv || d % 8) return XKV_EUNSUPPORTED;
  if (((uintptr_t)q & 15) || ((uintptr_t)out & 15)) return XKV_EALIGN;
  const int64_t total8 = (int64_t)batch * hq * hkv * d / 8;
  const dim3 grid((unsigned)((total8 + 255) / 256)), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == XKV_BF16) blockdiag_q_kernel<__bf16><<<grid, block, 0, st>>>((const __bf16*)q, (__bf16*)out, hq, hkv, d, total8);
  else if (dtype == XKV_F16) blockdiag_q_kernel<_Float16><<<grid, block, 0, st>>>((const _Float16*)q, (_Float16*)out, hq, hkv, d, total8);
  else return XKV_EDTYPE;
  return launch_status();
}

extern "C" int xkv_merge_stage2(const float* partial, const float* lse, void* out, const void* vB, int64_t sVb,
                                int64_t sVh, int64_t sVr, int d_out, int vB_dtype, const int32_t* ns,
                                const int32_t* kl, int batch, int hq, int hkv, int kv_len, int max_splits,
                                int split_cap_tokens, const int32_t* split_plan, int dv, int64_t sOb, int64_t sOh, int out_dtype, float* lse_out,
                                int64_t sLb, int64_t sLh, void* stream) {
  if (!partial || !lse || !out || !ns || batch <= 0 || hq <= 0 || hkv <= 0 || max_splits <= 0 || dv <= 0)
    return XKV_EINVAL;
  if (split_cap_tokens < 0 || (split_cap_tokens > 0 && (kv_len <= 0 || max_splits < cdiv(kv_len, split_cap_tokens)))) return XKV_EINVAL;
  if (split_plan && split_cap_tokens <= 0) return XKV_EINVAL;
  if (hq % hkv || hq / hkv > 32 || dv > 512) return XKV_EUNSUPPORTED;
  if (vB && (d_out <= 0 || d_out > 512 || d_out % 8)) return XKV_EUNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
#define XKV_MERGE(O, TB) \
  return launch_merge<O, TB>(partial, lse, out, vB, sVb, sVh, sVr, d_out, ns, kl, batch, hq, hkv, kv_len, max_splits, dv, sOb, sOh, lse_out, sLb, sLh, split_cap_tokens, split_plan, st)
  const int bt = vB ? vB_dtype : XKV_BF16;
  if (bt != XKV_BF16 && bt != XKV_F16) return XKV_EDTYPE;
  switch (out_dtype) {
    case XKV_F32: if (bt == XKV_BF16) XKV_MERGE(float, __bf16); else XKV_MERGE(float, _Float16);
    case XKV_F16: if (bt == XKV_BF16) XKV_MERGE(_Float16, __bf16); else XKV_MERGE(_Float16, _Float16);
    case XKV_BF16: if (bt == XKV_BF16) XKV_MERGE(__bf16, __bf16); else XKV_MERGE(__bf16, _Float16);
    default: return XKV_EDTYPE;
  }
#undef XKV_MERGE
}
