// Fast path of the fused reconstruct + RoPE + softmax + P.A stage 1 (rank RK = 512 / 384 / 256, head_dim 128, the
// token basis shared by K and V): the MFMA-bound headline kernel.  Included by one translation unit per rank.
// (Figures in the comments below are those of rank 512: 16 k-steps per wave, split 5 / 6 / 5 over the three parts.)
//
// Work split.  One workgroup = one (batch, kv head, split); its 4 wavefronts form a 2 x 2 grid over
// (rank half kq, feature half dq): wave (kq, dq) keeps B[kh][RK/2 kq .. +RK/2][{32 dq .. +32} u {64 + 32 dq .. +32}]
// stationary in RK/4 accumulation registers (both members of every rotate-half pair) and multiplies it, on
// v_mfma_f32_32x32x16, with its rank half of the 32-token tile.  Every element of the tile is therefore read
// from LDS by two waves, not four - LDS reads, not MFMA, bound a 4-way feature split.
// RoPE, the rounding to the operand type and the q-dot are all linear in K, so each wave rotates and dots its
// PARTIAL key tile (partial over its rank half and its feature half) and only 4 x [G x 32] fp32 partial scores
// are summed through LDS.
//
// Rotation.  R(pos) = R(base) R(offset).  The base is that of an even tile and is moved to the query: q^ = R(-base) q
// is recomputed once per two tiles by the workgroup (one thread per pair index, incremental rotation re-seeded with a
// range-reduced sincosf every 32 tiles) and read back as the B operand of the q-dot MFMA; the offset part (0..31 for
// the even tile, 32..63 for the odd one) is two per-lane constant tables in fp16 (32 VGPRs).
//
// Pipeline.  A wave issues instructions in order, so MFMA time and VALU time only overlap when independent
// work is interleaved in its instruction stream.  Iteration i therefore runs the 16 reconstruction MFMA steps of
// tile i (accumulating into one of two key-accumulator sets) in three parts, interleaved with what tile i-1 still
// needs: part 1 (steps 0..4) rotates tile i-1's partial keys (the other accumulator set) in packed fp16, dots them
// with q^ on v_mfma_f32_16x16x32 and stores the partial scores; barrier; part 2 (steps 5..10) runs the softmax of
// tile i-1 (one owner lane group per head: no redundant work), publishes P and the rescale factor through LDS and
// reads tile i-1 transposed for P.A; barrier; part 3 (steps 11..15) accumulates P.A for tile i-1, each wave owning
// RK/4 latent features, issues the loads of tile i+3 into the slot tile i-1 has left (one load behind each MFMA),
// writes q^ for the next pair of tiles and prefetches the first LDS operands of tile i+1.  Two barriers per tile separate the parts.
// The softmax reference only moves when a tile maximum exceeds it by 16 (8 for fp16 operands: lazy rescaling), so the
// P.A accumulators are almost never rescaled.
//
// Tiles stream through a 4-slot LDS ring filled by direct-to-LDS loads issued three tiles ahead.  Those loads
// are inline asm so that the compiler's wait-count pass does not serialise them against every LDS read;
// completion is tracked by hand (s_waitcnt vmcnt(8): the 8 loads of the next tile but one may still be in flight).
#pragma once
#include "xkv_common.h"
#include "recon_fast.h"
#include <type_traits>

namespace xkv {
namespace fast {

typedef short s16x4f __attribute__((ext_vector_type(4)));
typedef short s16x8f __attribute__((ext_vector_type(8)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int FT = 32;              // tokens per tile
constexpr int FRING = 4;
// Per rank: LDS tile geometry and the split of a wave's NKS k-steps (16 ranks each) over the three parts of an iteration.
template <int RK, bool SCORES> struct FastShape {
  static_assert(RK == 512 || RK == 384 || RK == 256, "rank");
  static constexpr int FROW = RK * 2 + 16;     // LDS bytes per tile row (16 pad: 16 rows hit 16 distinct bank groups)
  static constexpr int FTILE = FT * FROW;
  static constexpr int NKS = RK / 32;
  // measured, the best of the splits tried at each rank: 5+6+5, 5+5+2, and at rank 256 3+4+1 (fused) / 3+3+2 (scores only:
  // the split that keeps that instantiation small enough for two workgroups per CU)
  static constexpr int P1 = RK == 512 ? 5 : RK == 384 ? 5 : 3;
  static constexpr int P2 = RK == 512 ? 6 : RK == 384 ? 5 : SCORES ? 3 : 4;
  static constexpr int P3 = NKS - P1 - P2;
  static_assert(P3 <= 5 && P1 >= 1 && P2 >= 1, "part 3 has five groups, one k-step each");
  static constexpr int NMB = RK / 64;          // 16-feature blocks of the RK / 4 latent features a wave owns in P.A
  static_assert(3 * FROW < 4096, "instruction offset field");
  // part 1, group o (0..3): reconstruction MFMA m (0 .. 2 P1 - 1) and the read of fragment P1 + j (j < P2)
  static constexpr int p1_group_of_mfma(int m) { return m * 2 / P1; }
  static constexpr int p1_group_of_read(int j) { return j < 3 ? j : 3; }
  // part 2, group g (0..3): k-step P1 + s (s < P2), the read of fragment P1 + P2 + j (j < P3), transposed read pair mb
  static constexpr int p2_group_of_step(int s) { return P2 == 5 ? (s < 3 ? s : s - 1) : s * 4 / P2; }
  static constexpr int p2_group_of_read(int j) { return P3 == 5 ? (j < 1 ? 0 : j < 3 ? 1 : j - 1) : j * 4 / P3; }
  static constexpr int p2_group_of_tr(int mb) { return mb < (NMB + 2) / 4 ? 1 : mb < 2 * ((NMB + 2) / 4) ? 2 : 3; }
  // part 3, group u (0..4): the k-step (the last P3 groups hold one each), P.A block mb, the read of fragment j (j < P1) of
  // the next tile, and the tile loads issued in the group (8 per tile)
  static constexpr int p3_step(int u) { return u >= 5 - P3 ? P1 + P2 + u - (5 - P3) : -1; }
  static constexpr int p3_group_of_pv(int mb) { return 1 + mb * 4 / NMB; }
  static constexpr int p3_group_of_read(int j) { return j < 4 ? j : 4; }
  static constexpr int p3_loads(int u) { return P3 == 5 ? (u == 0 || u == 4 ? 1 : 2) : (u == 0 ? 0 : 2); }
  static constexpr int p3_first_load(int u) { return P3 == 5 ? (u == 0 ? 0 : 2 * u - 1) : 2 * u - 2; }
  static constexpr size_t SHM = (size_t)FRING * FTILE + 4 * 8 * (FT + 4) * 4 + 2 * 8 * 128 * 2 + 16 * (FT + 8) * 2 + 16 * 4 + 16 * 4 + 128 * 2;
};
constexpr int FSP_ROW = FT + 4;     // partial-score row stride (floats)
constexpr int FP_ROW = FT + 8;      // P row stride (elements)
// The softmax reference only moves when a tile maximum exceeds it by this much.  P = exp(s - reference) is stored in the
// operand type, so the bound must keep exp(bound) finite there: e^16 = 8.9e6 fits bf16's exponent range, but fp16 ends
// at 65504 = e^11.09, hence 8 (e^8 = 2981) for fp16.
template <typename T> constexpr float lazy_rescale() { return std::is_same<T, _Float16>::value ? 8.f : 16.f; }

// The LDS destination of a direct-to-LDS load is M0 + lane * 16.  A SALU write of M0 needs one wait state
// before an instruction that reads M0 (the compiler schedules around this for its own code; here it is explicit).
// Address = scalar row base + per-lane byte offset.
__device__ __forceinline__ void async_row16(const void* row_base, unsigned lane_off, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(lane_off), "s"(row_base)
               : "memory", "m0");
}
// The instruction offset moves the LDS address AND the global address: with base = (first row of a group of four) - 128
// bytes and per-row lane offsets voff[r] = lane * 16 + 128 + r * (row_bytes - FROW), the instruction offset r * FROW puts
// global row r at tile row r, so the four rows of a group share one scalar base and one M0 value.  (FROW must stay below
// 4096 / 3 for the 13-bit offset field.)
template <int OFF>
__device__ __forceinline__ void async_row_off(const void* base_m128, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3"
               ::"s"(lds_addr), "v"(voff), "s"(base_m128), "n"(OFF) : "memory", "m0");
}
template <int N> __device__ __forceinline__ void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// ---------------------------------------------------------------------------------------------------------------
// kB [hkv][RK][128] (strided) -> Bp [hkv][wave 4][ks RK/32][blk 2][lane 64][8]: the 16-byte packet lane l of wave
// (kq, dq) feeds to MFMA (ks, blk) as the A operand: B[RK/2 kq + 16 ks + 8 (l / 32) + e][64 blk + 32 dq + l % 32].
// ---------------------------------------------------------------------------------------------------------------
template <typename T, int RK>
__global__ __launch_bounds__(256) void pack_b_kernel(const T* __restrict__ kB, T* __restrict__ Bp, int64_t sBb, int64_t sBh,
                                                      int64_t sBr, int hkv) {
  const int kh = blockIdx.x, b = blockIdx.y;
  const T* Bh = kB + b * sBb + kh * sBh;
  constexpr int NKS = RK / 32;
  T* out = Bp + ((int64_t)b * hkv + kh) * (RK * 128);
  for (int idx = blockIdx.z * 256 + threadIdx.x; idx < 4 * NKS * 2 * 64; idx += 256 * gridDim.z) {
    const int l = idx & 63, blk = (idx >> 6) & 1, ks = (idx >> 7) % NKS, w = idx / (128 * NKS);
    const int kq = w >> 1, dq = w & 1;
    const int col = 64 * blk + 32 * dq + (l & 31);
    const int row0 = (RK / 2) * kq + 16 * ks + 8 * (l >> 5);
    typename Elem<T>::vec8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = Bh[(int64_t)(row0 + e) * sBr + col];
    st16(out + (int64_t)idx * 8, v);
  }
}

template <int V> using IC = std::integral_constant<int, V>;
#define XKV_FENCE() __builtin_amdgcn_sched_barrier(0)

// SCORES: write the scaled scores (the qAB-with-RoPE form) instead of running softmax and P.A
template <typename T, bool SCORES, int RK>
__global__ __launch_bounds__(256) void recon_fast_kernel(const FastParams p) {
  typedef typename Elem<T>::vec8 vec8;
  typedef FastShape<RK, SCORES> S;
  constexpr int FROW = S::FROW, FTILE = S::FTILE, NKS = S::NKS, P1 = S::P1, P2 = S::P2, P3 = S::P3, NMB = S::NMB;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kq = wave >> 1, dq = wave & 1;
  const int n32 = lane & 31, g2 = lane >> 5;
  const int n16 = lane & 15, g4 = lane >> 4;

  const int wg = xcd_cluster_remap(blockIdx.x, p.hkv);   // the kv heads of one (sequence, split) stream the same rows: one L2
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
  sc_t* qhat = reinterpret_cast<sc_t*>(s_part + 4 * 8 * FSP_ROW);          // [2][8 heads][128]
  T* p_lds = reinterpret_cast<T*>(qhat + 2 * 8 * 128);                                          // [16 head slots][FP_ROW]
  float* alpha_lds = reinterpret_cast<float*>(p_lds + 16 * FP_ROW);        // [16]
  float* ml_lds = alpha_lds + 16;                                          // [8][2]
  sc_t* qzero = reinterpret_cast<sc_t*>(ml_lds + 16);                      // [128] zeros: the q-dot operand of masked lanes
  const unsigned ring_lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)ring;
  for (int i = tid; i < 16 * FP_ROW; i += 256) p_lds[i] = from_f32<T>(0.f);   // slots of absent heads stay zero
  if (tid < 16) alpha_lds[tid] = 1.f;
  if (tid < 128) qzero[tid] = from_f32<sc_t>(0.f);

  // ---- async tile loads: wave w brings rows 8w .. 8w+7, one row (RK * 2 bytes: lanes 0 .. RK/8 - 1) per instruction -----
  // Scalar row pointers advance by adds only; the clamped form is needed only where a tile crosses the split end.
  const unsigned char* Ab = reinterpret_cast<const unsigned char*>(p.kA) + b * p.sAb * 2;
  const int64_t row_bytes = p.sAl * 2;
  const unsigned lane_off = lane * 16;
  unsigned voff4[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) voff4[r] = lane_off + 128u + (unsigned)(r * ((int)row_bytes - FROW));
  // One row per call: in the loop every load sits behind an MFMA of its own (a burst of loads holds the wave's issue for
  // about 20 cycles per instruction).  full_c: the caller knows the whole tile lies inside the split.
  auto issue_one = [&](int t, auto r_c, auto full_c) {
    constexpr int R = decltype(r_c)::value;
    const int tok0 = start + t * FT + wave * 8;
    const bool live = RK == 512 || lane < RK / 8;   // scalar addresses are formed outside this lane predicate
    if (decltype(full_c)::value) {
      const unsigned dst = ring_lds + (unsigned)(t & (FRING - 1)) * FTILE + (unsigned)(wave * 8 + (R & ~3)) * FROW;
      const unsigned char* base = Ab + (int64_t)(tok0 + (R & ~3)) * row_bytes - 128;
      if (live) async_row_off<(R & 3) * FROW>(base, voff4[R & 3], dst);
    } else {
      int tok = tok0 + R;
      tok = tok < last ? tok : last;   // rows past the split end are masked in the softmax; keep the read in bounds
      const unsigned char* rowp = Ab + (int64_t)tok * row_bytes;
      const unsigned dst = ring_lds + (unsigned)(t & (FRING - 1)) * FTILE + (unsigned)(wave * 8 + R) * FROW;
      if (live) async_row16(rowp, lane_off, dst);
    }
  };
  auto issue_tile = [&](int t) {
    issue_one(t, IC<0>(), IC<0>()); issue_one(t, IC<1>(), IC<0>()); issue_one(t, IC<2>(), IC<0>()); issue_one(t, IC<3>(), IC<0>());
    issue_one(t, IC<4>(), IC<0>()); issue_one(t, IC<5>(), IC<0>()); issue_one(t, IC<6>(), IC<0>()); issue_one(t, IC<7>(), IC<0>());
  };
  issue_tile(0);
  issue_tile(1);
  issue_tile(2);

  // ---- stationary B operands: NKS k-steps x 2 feature blocks, kept in accumulation registers --------------------------
  vec8 breg[NKS][2];
  {
    const T* bp = reinterpret_cast<const T*>(p.Bp) + b * p.sBpb + (int64_t)kh * (RK * 128) + ((int64_t)wave * (128 * NKS) + lane) * 8;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) breg[ks][blk] = ld16<vec8>(bp + (ks * 2 + blk) * 512);
  }

  // ---- in-tile rotation table: accumulator register r of lane (token n32, g2) is pair j = 32 dq + 8 (r/4) + 4 g2 + r%4 --
  typedef _Float16 rot2 __attribute__((ext_vector_type(2)));
  // Two tables: the query-side base is that of an EVEN tile and serves the odd tile after it too, whose offsets are 32 .. 63.
  rot2 ch[2][8], sh[2][8];     // [tile parity]: cos / sin of registers 2k, 2k+1, in fp16 (16 + 16 VGPRs)
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      float c0, s0, c1, s1;
      __sincosf((float)(n32 + 32 * h) * p.inv_freq[32 * dq + 8 * (r >> 2) + 4 * g2 + (r & 3)], &s0, &c0);
      __sincosf((float)(n32 + 32 * h) * p.inv_freq[32 * dq + 8 * ((r + 1) >> 2) + 4 * g2 + ((r + 1) & 3)], &s1, &c1);
      ch[h][r >> 1] = rot2{(_Float16)c0, (_Float16)c1};
      sh[h][r >> 1] = rot2{(_Float16)s0, (_Float16)s1};
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
  // q^ is kept in q-dot operand order: pair j = 32 dq' + 8 o + 4 g' + e sits at [o][dq'][g'][e] (partner at e + 4), so that
  // a lane's 8 contraction values of chunk o are one 16-byte read
  const int qpos = ((((lane >> 3) & 3) * 2 + (lane >> 5)) * 2 + ((lane >> 2) & 1)) * 8 + (lane & 3);
  float qc32, qs32, qcb = 1.f, qsb = 0.f;   // (qcb, qsb): base rotation of the tile whose q^ is written next
  sincosf((float)(2 * FT) * qinv, &qs32, &qc32);   // the base advances two tiles at a time
  // The base advances by angle addition; every 32 tiles it is replaced by a freshly range-reduced value (the seed),
  // computed outside the pipeline's inner loop and swapped in with a select so that write_qhat stays branch-free.
  int seed_t = 0;
  float seed_c, seed_s;
  auto make_seed = [&](int t) {
    seed_t = t;
    sincosf((float)(p.pos_offset + start + (int64_t)t * FT) * qinv, &seed_s, &seed_c);
  };
  auto write_qhat = [&](int t) {   // q^ for the even tile t and the odd one after it = R(-base(t)) q, into buffer (t / 2) & 1
    const bool sd = t == seed_t;
    qcb = sd ? seed_c : qcb;
    qsb = sd ? seed_s : qsb;
    sc_t* dst = qhat + ((t >> 1) & 1) * (8 * 128) + wave * 128 + qpos;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (i == 1 && G <= 4) break;   // head slots 4..7 are absent: nothing reads their rows
      dst[i * 512] = from_f32<sc_t>(q0[i] * qcb + q1[i] * qsb);
      dst[i * 512 + 4] = from_f32<sc_t>(q1[i] * qcb - q0[i] * qsb);
    }
    const float c = qcb * qc32 - qsb * qs32, s = qsb * qc32 + qcb * qs32;
    qcb = c; qsb = s;
  };
  make_seed(0);
  write_qhat(0);

  // ---- softmax role: lanes 0..15 of wave w own head w, lanes 16..31 head w + 4 (lanes 32..63 mirror them) --------------
  const int sm_head = wave + 4 * ((lane >> 4) & 1);
  const int sm_row = sm_head < G ? sm_head : G - 1;
  const bool sm_valid = sm_head < G;
  float m_ref = NEG_INF, l_run = 0.f;   // reference maximum of the lane's head; this lane's share of the head's row sum
  f32x2 sp_v[4];
  auto softmax_read = [&]() {   // the four waves' partial scores of this lane's two tokens
    const float* sp = s_part + sm_row * FSP_ROW + 2 * n16;
#pragma unroll
    for (int w = 0; w < 4; ++w) sp_v[w] = *reinterpret_cast<const f32x2*>(sp + w * 8 * FSP_ROW);
  };
  auto softmax_tile = [&](int t) {   // scores of tile t -> P (operand type) and the rescale factor, through LDS
    float s0 = (sp_v[0][0] + sp_v[1][0]) + (sp_v[2][0] + sp_v[3][0]);
    float s1 = (sp_v[0][1] + sp_v[1][1]) + (sp_v[2][1] + sp_v[3][1]);
    const int tok = start + t * FT + 2 * n16;
    if (SCORES) {   // lanes 0..31 of wave w hold heads w and w + 4, two tokens each
      if (sm_valid && lane < 32) {
        const int64_t o = ((int64_t)b * p.hq + h0 + sm_head) * p.kv_len + tok;
        s0 *= p.sm_scale;
        s1 *= p.sm_scale;
        if (p.scores_dtype == XKV_F32) {
          float* dst = reinterpret_cast<float*>(p.scores) + o;
          if (tok < end) dst[0] = s0;
          if (tok + 1 < end) dst[1] = s1;
        } else {
          T* dst = reinterpret_cast<T*>(p.scores) + o;
          if (tok < end) dst[0] = from_f32<T>(s0);
          if (tok + 1 < end) dst[1] = from_f32<T>(s1);
        }
      }
      return;
    }
    s0 = tok < end ? s0 * p.sm_scale : NEG_INF;
    s1 = tok + 1 < end ? s1 * p.sm_scale : NEG_INF;
    // the reference maximum only moves when the tile maximum exceeds it by lazy_rescale<T>(); the reduction that finds the
    // maximum runs only then, so the usual path from scores to P has no cross-lane step
    float alpha = 1.f;
    if (__builtin_amdgcn_ballot_w64(fmaxf(s0, s1) > m_ref + lazy_rescale<T>())) {   // rare: some head's maximum moves
      const float mx = row_reduce<true, 16>(fmaxf(s0, s1));
      const float m_new = mx > m_ref + lazy_rescale<T>() ? mx : m_ref;
      alpha = __expf(m_ref - m_new);
      m_ref = m_new;
    }
    const float e0 = __expf(s0 - m_ref), e1 = __expf(s1 - m_ref);
    l_run = l_run * alpha + (e0 + e1);   // per lane (alpha is the head's, the same in all 16): summed over the lanes once, at the end
    T* pd = p_lds + sm_head * FP_ROW + 2 * n16;
    pd[0] = from_f32<T>(sm_valid ? e0 : 0.f);
    pd[1] = from_f32<T>(sm_valid ? e1 : 0.f);
    alpha_lds[sm_head] = alpha;
  };

  // ---- q-dot B operand source: lanes whose token half (lane bit 4) matches their column's (lane bit 3) read q^ of head
  // lane % 8 (absent heads: the last one; their columns are not stored), the others read zeros ------------------------------
  const bool q_live = ((lane >> 4) & 1) == ((lane >> 3) & 1);
  const sc_t* qsrc = q_live ? qhat + ((lane & 7) < G ? (lane & 7) : G - 1) * 128 + (dq * 2 + g2) * 8 : qzero;
  const int qpar = q_live ? 8 * 128 : 0;   // q^ is double-buffered by tile parity, the zeros are not

  // ---- accumulators and loop-carried operand registers ---------------------------------------------------------------------
  f32x4 acc[NMB];        // P.A: wave w owns latent features RK/4 w .. + RK/4
#pragma unroll
  for (int mb = 0; mb < NMB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
  f32x16 ka[2][2];       // two sets of partial key accumulators [set][low | partner feature block]
  vec8 at[NKS];          // this wave's rank chunks of the tile being reconstructed (read one part ahead of their use)
  sc_vec8 qop[4];        // q^ operands of the tile being rotated

  auto tile_frag = [&](int t, int ks) -> vec8 {
    return ld16<vec8>(ring + (t & (FRING - 1)) * FTILE + n32 * FROW + ((RK / 2) * kq + 8 * g2) * 2 + ks * 32);
  };

  // One pipeline iteration.  PAR: accumulator set written by the reconstruction of tile i; tile i-1 lives in set PAR^1.
  // Interval structure (two barriers per iteration):
  //   part 1 [after B_c of i-1]  R(i) k-steps 0..P1-1       ||  rotate tile i-1, q-dot, publish partial scores
  //   B_b
  //   part 2                     R(i) k-steps P1..P1+P2-1   ||  softmax of tile i-1; wait for tile i+1
  //   B_c
  //   part 3                     R(i) the last P3 k-steps   ||  acc += V^T P^T for tile i-1; issue tile i+3; write q^(i+1)
  // Which group of a part holds which MFMA, LDS read and tile load: FastShape.
  // Every LDS operand is read one part before the MFMAs that consume it.  FULL: tile i+3 lies wholly inside the split.
  auto iteration = [&](int i, auto par_c, auto do_r_c, auto do_prev_c, auto full_c) {
    constexpr int PAR = decltype(par_c)::value;
    constexpr bool DO_R = decltype(do_r_c)::value != 0, DO_PREV = decltype(do_prev_c)::value != 0;
    f32x16& k0 = ka[PAR][0];
    f32x16& k1 = ka[PAR][1];
    const f32x16& j0 = ka[PAR ^ 1][0];
    const f32x16& j1 = ka[PAR ^ 1][1];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      asm volatile("" : "+a"(breg[ks][0]));
      asm volatile("" : "+a"(breg[ks][1]));
    }
    // Groups of instructions between XKV_FENCE() are scheduled by the compiler on their own and stay in source order:
    // LDS reads and the tile loads are dealt out among the MFMAs instead of being hoisted into bursts that make the four
    // waves queue on the LDS pipe right after every barrier.
    // ---- part 1 ----------------------------------------------------------------------------------------------------------
    {
      f32x4 sacc;
#pragma unroll
      for (int o = 0; o < 4; ++o) {
        if (DO_R) {
#pragma unroll
          for (int j = 0; j < P2; ++j)
            if (S::p1_group_of_read(j) == o) at[P1 + j] = tile_frag(i, P1 + j);
#pragma unroll
          for (int m = 0; m < 2 * P1; ++m) {
            if (S::p1_group_of_mfma(m) != o) continue;
            const int ks = m >> 1;
            if (ks == 0) {
              const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
              if ((m & 1) == 0) k0 = Elem<T>::mfma32(breg[0][0], at[0], z); else k1 = Elem<T>::mfma32(breg[0][1], at[0], z);
            } else {
              if ((m & 1) == 0) k0 = Elem<T>::mfma32(breg[ks][0], at[ks], k0); else k1 = Elem<T>::mfma32(breg[ks][1], at[ks], k1);
            }
          }
        }
        if (DO_PREV) {
          // The rotation runs in packed fp16, two pairs per instruction (v_pk_mul_f16 / v_pk_fma_f16): the partial key sums
          // and the in-tile cos / sin are rounded to fp16 first, as the reference does (fp16 accumulators and fp16 cos / sin,
          // flash_recontruction/qAB/v1.py:59-77).  8 VALU instructions fewer per 8 rotated values than the fp32 form.
          typedef _Float16 h2 __attribute__((ext_vector_type(2)));
          h2 lo2[2], hi2[2];
#pragma unroll
          for (int e2 = 0; e2 < 2; ++e2) {
            const int r = 4 * o + 2 * e2;
            const h2 a = {(_Float16)j0[r], (_Float16)j0[r + 1]}, bb = {(_Float16)j1[r], (_Float16)j1[r + 1]};
            lo2[e2] = a * ch[PAR ^ 1][2 * o + e2] - bb * sh[PAR ^ 1][2 * o + e2];   // tile i-1: parity PAR ^ 1
            hi2[e2] = bb * ch[PAR ^ 1][2 * o + e2] + a * sh[PAR ^ 1][2 * o + e2];
          }
          const sc_vec8 kop = {lo2[0][0], lo2[0][1], lo2[1][0], lo2[1][1], hi2[0][0], hi2[0][1], hi2[1][0], hi2[1][1]};
          // q-dot on v_mfma_f32_16x16x32: as its A operand, lane (n32, g2) is row n32 % 16 and k-group (n32 / 16) + 2 g2, so
          // the two token halves of the tile land in the same 16 rows as different k-groups; the B operand keeps them apart:
          // column c holds q^ of head c % 8 in the k-groups of token half c / 8 and zeros in the other two.  Result: lane
          // (c, g4), register r = score of token 16 (c / 8) + 4 g4 + r for head c % 8.
          sacc = Elem<sc_t>::mfma16(kop, qop[o], o == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : sacc);
        }
        XKV_FENCE();
      }
      if (DO_PREV && (n16 & 7) < G)
        *reinterpret_cast<f32x4*>(s_part + (wave * 8 + (n16 & 7)) * FSP_ROW + 16 * (n16 >> 3) + 4 * g4) = sacc;
    }
    __syncthreads();        // B_b: partial scores of tile i-1 are visible
    // ---- part 2 ----------------------------------------------------------------------------------------------------------
    s16x4f tr[2 * NMB];
    const unsigned char* vt =
        ring + ((i - 1) & (FRING - 1)) * FTILE + (8 * g4 + (n16 >> 2)) * FROW + (wave * (RK / 4) + 4 * (n16 & 3)) * 2;
    auto tr_read = [&](int mb) {
      if (SCORES) return;
      tr[2 * mb] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4f*)(vt + mb * 32));
      tr[2 * mb + 1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4f*)(vt + mb * 32 + 4 * FROW));
    };
    auto recon_step = [&](int ks) {
      k0 = Elem<T>::mfma32(breg[ks][0], at[ks], k0);
      k1 = Elem<T>::mfma32(breg[ks][1], at[ks], k1);
    };
    auto part2_group = [&](auto g_c) {   // the LDS reads and k-steps FastShape assigns to group g of part 2
      constexpr int g = decltype(g_c)::value;
      if (DO_PREV) {
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb)
          if (S::p2_group_of_tr(mb) == g) tr_read(mb);   // every transposed read of tile i-1 precedes B_c
      }
      if (DO_R) {
#pragma unroll
        for (int j = 0; j < P3; ++j)
          if (S::p2_group_of_read(j) == g) at[P1 + P2 + j] = tile_frag(i, P1 + P2 + j);
#pragma unroll
        for (int s2 = 0; s2 < P2; ++s2)
          if (S::p2_group_of_step(s2) == g) recon_step(P1 + s2);
      }
    };
    if (DO_PREV) softmax_read();
    part2_group(IC<0>());
    XKV_FENCE();
    part2_group(IC<1>());
    XKV_FENCE();
    if (DO_PREV) softmax_tile(i - 1);
    part2_group(IC<2>());
    XKV_FENCE();
    part2_group(IC<3>());
    if (DO_R) {
      wait_vmcnt<8>();      // this wave's rows of tile i+1 have landed (the 8 loads of tile i+2 may be in flight)
    } else {
      wait_vmcnt<0>();
      if (!SCORES) {        // final state for the epilogue
        const float l_head = row_reduce<false, 16>(l_run);
        if (sm_valid && n16 == 0) { ml_lds[2 * sm_head] = m_ref; ml_lds[2 * sm_head + 1] = l_head; }
      }
    }
    __syncthreads();        // B_c: P and rescale factors of tile i-1 are visible; tile i+1 is complete for every wave;
                            // the transposed reads of tile i-1 have returned, so its ring slot is free
    // ---- part 3 ----------------------------------------------------------------------------------------------------------
    vec8 pb;
    vec8 at_next[P1];
    sc_vec8 qop_next[4];
    const sc_t* qrow = qsrc + ((i >> 1) & 1) * qpar;   // q^ of the pair of tiles i (even) opens
    auto pv_step = [&](int mb) {
      if (SCORES) return;
      vec8 a = __builtin_bit_cast(vec8, (s16x8f)__builtin_shufflevector(tr[2 * mb], tr[2 * mb + 1], 0, 1, 2, 3, 4, 5, 6, 7));
      acc[mb] = Elem<T>::mfma16(a, pb, acc[mb]);
    };
    float al = 1.f;
    if (DO_PREV && !SCORES) {
      al = alpha_lds[n16];
      pb = ld16<vec8>(p_lds + n16 * FP_ROW + 8 * g4);
    }
    // Group u of part 3: the P.A blocks, the k-step, the reads of the next tile's first fragments and of q^, and the tile
    // loads FastShape assigns to it; every load sits behind an MFMA of its own where the group has one.
    auto grp = [&](auto u_c) {
      constexpr int u = decltype(u_c)::value;
      constexpr int ks = S::p3_step(u), nl = S::p3_loads(u), l0 = S::p3_first_load(u);
      if (DO_PREV && u >= 1) {
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb)
          if (S::p3_group_of_pv(mb) == u) pv_step(mb);
      }
      if (DO_R) {
#pragma unroll
        for (int j = 0; j < P1; ++j)
          if (S::p3_group_of_read(j) == u) at_next[j] = tile_frag(i + 1, j);
        if (u >= 1 && PAR == 0) qop_next[u >= 1 ? u - 1 : 0] = ld16<sc_vec8>(qrow + (u - 1) * 32);   // an odd tile keeps its predecessor's
        if (ks >= 0) {
          constexpr int kk = ks >= 0 ? ks : 0;
          k0 = Elem<T>::mfma32(breg[kk][0], at[kk], k0);
          if (nl >= 1) {
            XKV_FENCE();
            issue_one(i + 3, IC<l0>(), full_c);        // into the ring slot of tile i-1, whose readers are done
            XKV_FENCE();
          }
          k1 = Elem<T>::mfma32(breg[kk][1], at[kk], k1);
          if (nl >= 2) {
            XKV_FENCE();
            issue_one(i + 3, IC<l0 + 1>(), full_c);
          }
        } else if (nl > 0) {
          XKV_FENCE();
          issue_one(i + 3, IC<l0>(), full_c);
          if (nl >= 2) issue_one(i + 3, IC<(nl >= 2 ? l0 + 1 : l0)>(), full_c);
        }
        if (u == 4 && PAR == 1) write_qhat(i + 1);   // buffer ((i+1)/2)&1 was last read in part 3 of iteration i-3
      }
      XKV_FENCE();
      if (u == 0 && DO_PREV && !SCORES) {   // the MFMAs above cover the LDS latency of the rescale factor this branch waits for
        if (__builtin_amdgcn_ballot_w64(al != 1.f)) {   // rare: the softmax reference moved
#pragma unroll
          for (int mb = 0; mb < NMB; ++mb) acc[mb] *= al;
        }
      }
    };
    grp(IC<0>()); grp(IC<1>()); grp(IC<2>()); grp(IC<3>()); grp(IC<4>());
    if (DO_R) {
#pragma unroll
      for (int ks = 0; ks < P1; ++ks) at[ks] = at_next[ks];
#pragma unroll
      for (int o = 0; o < 4; ++o)
        if (PAR == 0) qop[o] = qop_next[o];
    }
  };

  // ---- pipeline: R(0) | {R(i), prev(i-1)} for i = 1 .. ntiles-1 | prev(ntiles-1) -------------------------------------------------
  wait_vmcnt<0>();          // tiles 0..2 and the B operands
  __syncthreads();
#pragma unroll
  for (int ks = 0; ks < P1; ++ks) at[ks] = tile_frag(0, ks);
  const int nfull = (end - start) / FT;
  iteration(0, IC<0>(), IC<1>(), IC<0>(), IC<0>());
  int i = 1;
  // pairs of iterations in chunks that end where q^ is re-seeded; `fast` pairs know that tiles i+3 and i+4 are full
  auto pairs = [&](auto full_c) {
    while (i + 1 < ntiles && (!decltype(full_c)::value || i + 5 <= nfull)) {
      make_seed((i + 32) & ~31);
      for (; i < seed_t && i + 1 < ntiles && (!decltype(full_c)::value || i + 5 <= nfull); i += 2) {
        iteration(i, IC<1>(), IC<1>(), IC<1>(), full_c);
        iteration(i + 1, IC<0>(), IC<1>(), IC<1>(), full_c);
      }
    }
  };
  pairs(IC<1>());
  pairs(IC<0>());
  if (i < ntiles) {
    iteration(i, IC<1>(), IC<1>(), IC<1>(), IC<0>());
    ++i;
  }
  if (ntiles & 1) iteration(ntiles, IC<1>(), IC<0>(), IC<1>(), IC<0>());
  else iteration(ntiles, IC<0>(), IC<0>(), IC<1>(), IC<0>());
  __syncthreads();
  if (SCORES) return;

  // ---- epilogue ----------------------------------------------------------------------------------------------------------
  if (n16 < G) {
    const float m = ml_lds[2 * n16], l = ml_lds[2 * n16 + 1];
    const float inv = 1.f / l;
    const int64_t ph = ((int64_t)b * p.hq + h0 + n16) * p.max_splits + split;
    float* dst = p.partial + ph * RK + wave * (RK / 4) + 4 * g4;
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) *reinterpret_cast<f32x4*>(dst + mb * 16) = acc[mb] * inv;
    if (wave == 0 && g4 == 0) p.lse[ph] = m + __logf(l);
  }
}

template <typename T, int RK>
int launch_recon_fast_t(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, hipStream_t st) {
  typedef FastShape<RK, false> S;   // the LDS footprint does not depend on the mode
  const int nb = sBb == 0 ? 1 : batch;   // one packed copy when the factor is shared by the batch
  pack_b_kernel<T, RK><<<dim3(p.hkv, nb, 32), dim3(256), 0, st>>>((const T*)kB, (T*)p.Bp, sBb, sBh, sBr, p.hkv);
  auto kern = p.scores ? recon_fast_kernel<T, true, RK> : recon_fast_kernel<T, false, RK>;
  static DynLds lds[2];
  const int e = ensure_dynamic_lds(lds[p.scores ? 1 : 0], reinterpret_cast<const void*>(kern), (int)S::SHM, true);
  if (e != XKV_OK) return e;
  const int total = batch * p.hkv * p.max_splits;
  kern<<<dim3(xcd_grid(total, p.hkv)), dim3(256), S::SHM, st>>>(p);
  return launch_status();
}

template <int RK>
int launch_recon_fast_rank(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                           hipStream_t st) {
  return dtype == XKV_BF16 ? launch_recon_fast_t<__bf16, RK>(p, kB, sBb, sBh, sBr, batch, st)
                           : launch_recon_fast_t<_Float16, RK>(p, kB, sBb, sBh, sBr, batch, st);
}

}  // namespace fast
}  // namespace xkv
