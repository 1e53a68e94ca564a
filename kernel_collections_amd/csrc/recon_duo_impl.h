// Fused reconstruct + RoPE + softmax + P.A stage 1 with a SEPARATE value basis (a second row stream), which the 4-wave
// kernel (recon_fast_impl.h) is not built for: key rank 256 / 384 / 512, value rank 256 / 384 / 512, head_dim 128, computed
// RoPE angles.  (The template also has a scores-only and a shared-basis mode; the 4-wave kernel is the faster one there and
// the dispatcher sends those shapes to it.)  Included by the recon_duo_*.hip translation units, which instantiate the shapes.
//
// Work split.  One workgroup = one (batch, kv head, split), 8 wavefronts = two per SIMD.  The waves form a 2 x 4 grid
// over (rank half kq, feature quarter dq): wave (kq, dq) keeps B[kh][RK/2 kq .. +RK/2][{16 dq .. +16} u {64 + 16 dq .. +16}]
// stationary in RK/8 registers - one 32-row MFMA block holds 16 features AND their 16 rotate-half partners - and
// multiplies it, on v_mfma_f32_32x32x16, with its rank half of the 32-token tile.  Accumulator registers r and r + 8 of a
// lane are then the two members of one RoPE pair, so the rotation needs no exchange and no wave rotates anything twice.
// RoPE, the rounding to the operand type and the q-dot are all linear in K, so each wave rotates and dots its PARTIAL key
// tile (partial over its rank half and its feature quarter) and only 8 x [G x 32] fp32 partial scores are summed through LDS.
//
// Rotation.  R(pos) = R(tile base) R(offset in tile).  The in-tile part is a per-lane constant table (16 VGPRs); the
// base part is moved to the query: q^ = R(-base) q is recomputed per tile by the workgroup (thread = (head, pair),
// incremental rotation re-seeded with a range-reduced sincosf every 32 tiles) and read back as the B operand of the
// q-dot MFMA.
//
// Pipeline.  Iteration t (accumulator generation t & 1 holds tile t's partial keys), two barriers:
//   I1: rotate / q-dot tile t -> partial scores  ||  first half of the reconstruction of tile t+1 (other generation);
//       issue the loads that the slots freed at the last barrier allow; q^ of tile t+1 (double-buffered)
//   I2: acc += P.A of tile t-1 (operands already in registers)  ||  softmax of tile t (wave w owns head w) -> P, rescale
//       factor (double-buffered)  ||  the rest of tile t+1  ||  transposed value operands of tile t -> registers
// The loop body is straight-line: past the last tile the reconstruction runs on the clamped look-ahead rows (never
// used), and the first P.A multiplies zeros.  The softmax reference only moves when a tile maximum exceeds it by 16 (lazy
// rescaling).  Key tiles (and value tiles) stream through LDS rings filled by direct-to-LDS loads; those loads are inline
// asm, invisible to the compiler's wait-count pass, and completion is tracked by hand with s_waitcnt vmcnt.
#pragma once
#include "xkv_common.h"
#include "recon_fast.h"
#include <type_traits>

namespace xkv {
namespace duo {

typedef short s16x4d __attribute__((ext_vector_type(4)));
typedef short s16x8d __attribute__((ext_vector_type(8)));
typedef float f32x2d __attribute__((ext_vector_type(2)));

enum { DUO_SCORES = 0, DUO_VSHARED = 1, DUO_VDISTINCT = 2 };

constexpr int FT = 32;              // tokens per tile
constexpr int NW = 8;               // wavefronts per workgroup
constexpr int FSP_ROW = FT + 4;     // partial-score row stride (floats)
constexpr int FP_ROW = FT + 8;      // P row stride (elements)
// The softmax reference only moves when a tile maximum exceeds it by this much.  P = exp(s - reference) is stored in the
// operand type, so the bound must keep exp(bound) finite there: e^16 = 8.9e6 fits bf16's exponent range, but fp16 ends
// at 65504 = e^11.09, hence 8 (e^8 = 2981) for fp16.
template <typename T> constexpr float lazy_rescale() { return std::is_same<T, _Float16>::value ? 8.f : 16.f; }
#define XKV_DUO_FENCE() __builtin_amdgcn_sched_barrier(0)
#define XKV_DUO_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)   // 0x8 MFMA, 0x2 VALU, 0x100 LDS read, 0x200 LDS write

// LDS budget: everything but the tile rings
constexpr int DUO_TAIL = NW * 8 * FSP_ROW * 4 + 2 * 8 * 128 * 2 + 2 * 16 * FP_ROW * 2 + 32 * 4 + 16 * 4 + 32 * 2;

template <int RK, int RV, int MODE>
struct DuoShape {
  static constexpr bool V2 = MODE == DUO_VDISTINCT;
  static constexpr int KROW = RK * 2 + 16;                 // padded key-tile row: 16 rows hit 16 distinct bank groups
  static constexpr int VROW = RV * 2 + 16;
  static constexpr int KTILE = FT * KROW, VTILE = V2 ? FT * VROW : 0;
  static constexpr int ROOM = 160 * 1024 - DUO_TAIL;
  // one stream: as many slots as fit, at most 6.  Two streams: 2 value slots, and 3 key slots when they fit (else 2)
  static constexpr int NSV = V2 ? 2 : 0;
  static constexpr int NSK_FIT = (ROOM - NSV * VTILE) / KTILE;
  static constexpr int NSK = V2 ? (NSK_FIT >= 3 ? 3 : 2) : (NSK_FIT > 6 ? 6 : NSK_FIT);
  static constexpr int SHM = NSK * KTILE + NSV * VTILE + DUO_TAIL;
  static_assert(NSK >= 2 && (V2 || NSK >= 4), "ring too short");
  static_assert(SHM <= 160 * 1024, "LDS budget");
  // key tile t + KAHEAD and (two streams) value tile t + VAHEAD are issued at the start of iteration t
  static constexpr int KAHEAD = V2 ? NSK : NSK - 1;
  static constexpr int VAHEAD = NSV - 1;
  static constexpr int LPT = V2 ? 8 : 4;                   // loads per wave and iteration
  // loads that may still be in flight where tile t+2's keys must have landed (end of I2 of iteration t) ...
  static constexpr int WAIT_K = V2 ? 4 + 8 * (NSK - 2) : 4 * (NSK - 3);
  // ... and where tile t's values must have landed (end of I1 of iteration t)
  static constexpr int WAIT_V = 8 * VAHEAD;
  static_assert(WAIT_K < 64 && WAIT_V < 64, "vmcnt holds 6 bits");
};

// The LDS destination of a direct-to-LDS load is M0 + lane * 16.  A SALU write of M0 needs one wait state before an
// instruction that reads M0.  Address = scalar row base + per-lane byte offset.
__device__ __forceinline__ void duo_row16(const void* row_base, unsigned lane_off, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(lane_off), "s"(row_base)
               : "memory", "m0");
}
// Four rows with one M0 / base pair: the instruction offset r * ROW moves the LDS address AND the global address, so the
// per-row lane offsets voff[r] = lane * 16 + 128 + r * (row_bytes - ROW) (base = first row - 128 bytes) put row r of the
// tile at global row r.  (ROW must stay below 4096 / 3 for the 13-bit offset field.)
template <int ROW>
__device__ __forceinline__ void duo_rows4(const void* base_m128, unsigned v0, unsigned v1, unsigned v2, unsigned v3,
                                          unsigned lds_addr) {
  static_assert(3 * ROW < 4096, "instruction offset field");
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
               "global_load_lds_dwordx4 %1, %5\n\t"
               "global_load_lds_dwordx4 %2, %5 offset:%6\n\t"
               "global_load_lds_dwordx4 %3, %5 offset:%7\n\t"
               "global_load_lds_dwordx4 %4, %5 offset:%8"
               ::"s"(lds_addr), "v"(v0), "v"(v1), "v"(v2), "v"(v3), "s"(base_m128), "n"(ROW), "n"(2 * ROW), "n"(3 * ROW)
               : "memory", "m0");
}
template <int N> __device__ __forceinline__ void duo_wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// One row stream: this wave's 4 rows of every tile, HBM -> its LDS ring, advancing by adds only.
template <int WIDTH, int ROW, int NS>
struct DuoStream {
  const unsigned char* base;   // first row of the sequence
  const unsigned char* ptr;    // this wave's first row of the next tile, minus 128 bytes
  int64_t row_bytes;
  int tok;                     // first token of the next tile
  unsigned dst, dst_end;       // LDS address of this wave's rows in the next slot / one past the ring
  unsigned voff[4];
  __device__ __forceinline__ void init(const void* rows, int64_t stride_elems, int start, int wave, int lane, unsigned ring_lds) {
    base = reinterpret_cast<const unsigned char*>(rows);
    row_bytes = stride_elems * 2;
    ptr = base + (int64_t)(start + wave * 4) * row_bytes - 128;
    tok = start;
    dst = ring_lds + (unsigned)(wave * 4) * ROW;
    dst_end = dst + NS * FT * ROW;
#pragma unroll
    for (int r = 0; r < 4; ++r) voff[r] = lane * 16 + 128u + (unsigned)(r * ((int)row_bytes - ROW));
  }
  __device__ __forceinline__ void issue(int end, int last, int wave, int lane) {
    if (WIDTH >= 512 || lane < WIDTH / 8) {   // a row narrower than 1 KiB fills only part of a load instruction
      if (tok + FT <= end) {                  // the whole tile lies inside the split
        duo_rows4<ROW>(ptr, voff[0], voff[1], voff[2], voff[3], dst);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          int tk = tok + wave * 4 + r;
          tk = tk < last ? tk : last;         // rows past the split end are masked in the softmax; keep the read in bounds
          duo_row16(base + (int64_t)tk * row_bytes, lane * 16, dst + r * ROW);
        }
      }
    }
    tok += FT;
    ptr += FT * row_bytes;
    dst += FT * ROW;
    dst = dst == dst_end ? dst - NS * FT * ROW : dst;
  }
};

// ---------------------------------------------------------------------------------------------------------------
// kB [hkv][RK][128] (strided) -> Bp [hkv][wave 8][ks RK/32][lane 64][8]: the 16-byte packet lane l = (n32, g2) of wave
// (kq, dq) feeds to MFMA ks as the A operand: B[RK/2 kq + 16 ks + 8 g2 + e][feature], feature = 16 dq + n32 for the low
// half of the block (n32 < 16) and 64 + 16 dq + n32 - 16 (the rotate-half partner) for the upper half.
// ---------------------------------------------------------------------------------------------------------------
template <typename T, int RK>
__global__ __launch_bounds__(256) void duo_pack_b_kernel(const T* __restrict__ kB, T* __restrict__ Bp, int64_t sBb, int64_t sBh,
                                                          int64_t sBr, int hkv) {
  constexpr int NKS = RK / 32;
  const int kh = blockIdx.x, b = blockIdx.y;
  const T* Bh = kB + b * sBb + kh * sBh;
  T* out = Bp + ((int64_t)b * hkv + kh) * (RK * 128);
  for (int idx = blockIdx.z * 256 + threadIdx.x; idx < NW * NKS * 64; idx += 256 * gridDim.z) {
    const int l = idx & 63, ks = (idx >> 6) % NKS, w = idx / (64 * NKS);
    const int kq = w >> 2, dq = w & 3, n32 = l & 31;
    const int col = n32 < 16 ? 16 * dq + n32 : 64 + 16 * dq + n32 - 16;
    const int row0 = (RK / 2) * kq + 16 * ks + 8 * (l >> 5);
    typename Elem<T>::vec8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = Bh[(int64_t)(row0 + e) * sBr + col];
    st16(out + (int64_t)idx * 8, v);
  }
}

template <typename T, int RK, int RV, int MODE>
__global__ __launch_bounds__(64 * NW) void recon_duo_kernel(const FastParams p) {
  typedef typename Elem<T>::vec8 vec8;
  typedef DuoShape<RK, RV, MODE> S;
  constexpr bool SCORES = MODE == DUO_SCORES, V2 = MODE == DUO_VDISTINCT;
  constexpr int KROW = S::KROW, KTILE = S::KTILE, NSK = S::NSK, VROW = S::VROW, VTILE = S::VTILE, NSV = S::NSV;
  constexpr int NKS = RK / 32;        // k-steps (16 ranks each) of a wave's rank half
  constexpr int KA = NKS / 2;         // k-steps of tile t+1 that run in I1 (beside the rotation of tile t)
  constexpr int PF = 2;               // tile fragments read ahead of the MFMA that consumes them
  constexpr int DV = V2 ? RV : RK;    // value features
  constexpr int NMB = DV / 128;       // 16-feature blocks of the DV / 8 value features a wave owns
  static_assert(RK % 128 == 0 && DV % 128 == 0 && KA >= 4, "shape");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kq = wave >> 2, dq = wave & 3;
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
  unsigned char* kring = smem;                                             // NSK * KTILE
  unsigned char* vring = V2 ? smem + NSK * KTILE : smem;                   // NSV * VTILE (one stream: the key ring)
  float* s_part = reinterpret_cast<float*>(smem + NSK * KTILE + NSV * VTILE);   // [8 waves][8 heads][FSP_ROW]
  sc_t* qhat = reinterpret_cast<sc_t*>(s_part + NW * 8 * FSP_ROW);         // [2][8 heads][128]
  T* p_lds = reinterpret_cast<T*>(qhat + 2 * 8 * 128);                                          // [2][16 head slots][FP_ROW]
  float* alpha_lds = reinterpret_cast<float*>(p_lds + 2 * 16 * FP_ROW);    // [2][16]
  float* ml_lds = alpha_lds + 32;                                          // [8][2]
  sc_t* qzero = reinterpret_cast<sc_t*>(ml_lds + 16);                      // [32] zeros: the q-dot operand of masked lanes
  const unsigned smem_lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)smem;
  for (int i = tid; i < 2 * 16 * FP_ROW; i += 64 * NW) p_lds[i] = from_f32<T>(0.f);   // slots of absent heads stay zero
  if (tid < 32) alpha_lds[tid] = 1.f;
  if (tid < 32) qzero[tid] = from_f32<sc_t>(0.f);

  // ---- async tile loads: wave w brings rows 4w .. 4w+3 of every tile ---------------------------------------------
  DuoStream<RK, KROW, NSK> ks_;
  ks_.init(reinterpret_cast<const unsigned char*>(p.kA) + b * p.sAb * 2, p.sAl, start, wave, lane, smem_lds);
  DuoStream<V2 ? RV : RK, V2 ? VROW : KROW, V2 ? NSV : NSK> vs_;
  if (V2) vs_.init(reinterpret_cast<const unsigned char*>(p.vA) + b * p.sVb * 2, p.sVl, start, wave, lane, smem_lds + NSK * KTILE);
#pragma unroll
  for (int i = 0; i < S::KAHEAD; ++i) ks_.issue(end, last, wave, lane);
  if (V2) {
#pragma unroll
    for (int i = 0; i < S::VAHEAD; ++i) vs_.issue(end, last, wave, lane);
  }

  // ---- stationary B operands: NKS k-steps of one 32-feature block (16 low features + their 16 partners) ----------
  vec8 breg[NKS];
  {
    const T* bp = reinterpret_cast<const T*>(p.Bp) + b * p.sBpb + (int64_t)kh * (RK * 128) + ((int64_t)wave * (64 * NKS) + lane) * 8;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) breg[ks] = ld16<vec8>(bp + ks * 512);
  }

  // ---- in-tile rotation table: accumulator registers r and r + 8 of lane (token n32, g2) are the two members of pair
  // j = 16 dq + 8 (r / 4) + 4 g2 + r % 4 ---------------------------------------------------------------------------------
  // kept in fp16, two registers per VGPR: the rotation runs in packed fp16 (see there)
  typedef _Float16 rot2 __attribute__((ext_vector_type(2)));
  rot2 ch[4], sh[4];
#pragma unroll
  for (int r = 0; r < 8; r += 2) {
    float c0, s0, c1, s1;
    __sincosf((float)n32 * p.inv_freq[16 * dq + 8 * (r >> 2) + 4 * g2 + (r & 3)], &s0, &c0);
    __sincosf((float)n32 * p.inv_freq[16 * dq + 8 * ((r + 1) >> 2) + 4 * g2 + ((r + 1) & 3)], &s1, &c1);
    ch[r >> 1] = rot2{(_Float16)c0, (_Float16)c1};
    sh[r >> 1] = rot2{(_Float16)s0, (_Float16)s1};
  }

  // ---- query-side base rotation: thread -> (head slot = wave, pair j = lane) -------------------------------------------
  float q0 = 0.f, q1 = 0.f;
  if (wave < G) {
    const T* qrow = reinterpret_cast<const T*>(p.q) + ((int64_t)b * p.hq + h0 + wave) * 128;
    q0 = to_f32(qrow[lane]);
    q1 = to_f32(qrow[lane + 64]);
  }
  const float qinv = p.inv_freq[lane];
  // q^ is kept in q-dot operand order: pair j = 16 dq' + 8 o + 4 g' + e sits at [dq'][o][g'][e] (partner at e + 4), so
  // that a lane's 8 contraction values are one 16-byte read
  const int qpos = (lane >> 2) * 8 + (lane & 3);
  float qc32, qs32, qcb = 1.f, qsb = 0.f;   // (qcb, qsb): base rotation of the tile whose q^ is written next
  sincosf((float)FT * qinv, &qs32, &qc32);
  auto write_qhat = [&](int t) {   // q^ for tile t = R(-base(t)) q, into buffer t & 1
    if (wave >= G) return;         // absent head slot: nothing reads its row
    if ((t & 31) == 0)             // the base advances by angle addition; every 32 tiles it is range-reduced afresh
      sincosf((float)(p.pos_offset + start + (int64_t)t * FT) * qinv, &qsb, &qcb);
    sc_t* dst = qhat + (t & 1) * (8 * 128) + wave * 128 + qpos;
    dst[0] = from_f32<sc_t>(q0 * qcb + q1 * qsb);
    dst[4] = from_f32<sc_t>(q1 * qcb - q0 * qsb);
    const float c = qcb * qc32 - qsb * qs32, s = qsb * qc32 + qcb * qs32;
    qcb = c; qsb = s;
  };

  // ---- softmax role: lanes (l & 15) of wave w own tokens 2 (l & 15), +1 of head w (the four 16-lane groups mirror) ----
  const bool sm_valid = wave < G;
  const int sm_row = sm_valid ? wave : G - 1;
  float m_ref = NEG_INF, l_run = 0.f;
  // ---- accumulators ---------------------------------------------------------------------------------------------------
  f32x4 acc[NMB];        // P.A: wave w owns value features DV/8 w .. + DV/8
#pragma unroll
  for (int mb = 0; mb < NMB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
  f32x16 ka[2];          // two generations of the partial key tile: 32 tokens x [16 low | 16 partner] features
  s16x4d tr[2 * NMB];    // transposed value operands of the tile whose P is being computed
#pragma unroll
  for (int i = 0; i < 2 * NMB; ++i) tr[i] = s16x4d{0, 0, 0, 0};

  auto tile_frag = [&](int t, int ks) -> vec8 {
    return ld16<vec8>(kring + (t % NSK) * KTILE + n32 * KROW + ((RK / 2) * kq + 8 * g2) * 2 + ks * 32);
  };
  // q-dot on v_mfma_f32_16x16x32: as its A operand, lane (n32, g2) is row n32 % 16 and k-group (n32 / 16) + 2 g2, so the two
  // token halves of the tile land in the same 16 rows as different k-groups; the B operand keeps them apart: column c holds
  // q^ of head c % 8 in the k-groups of token half c / 8 (lanes whose bit 4 equals bit 3) and zeros in the other two.
  // Result: lane (c, g4), register r = score of token 16 (c / 8) + 4 g4 + r for head c % 8.
  const bool q_live = ((lane >> 4) & 1) == ((lane >> 3) & 1);
  const sc_t* qrow = q_live ? qhat + ((lane & 7) < G ? (lane & 7) : G - 1) * 128 + (dq * 4 + g2) * 8 : qzero;
  const int qpar = q_live ? 8 * 128 : 0;   // q^ is double-buffered by tile parity, the zeros are not
  auto tr_read = [&](int t) {   // this wave's DV/8 value features of tile t, token-major
    if (SCORES) return;
    constexpr int VR = V2 ? VROW : KROW;
    const unsigned char* vt = (V2 ? vring + (t % NSV) * VTILE : kring + (t % NSK) * KTILE) + (8 * g4 + (n16 >> 2)) * VR +
                              (wave * (DV / 8) + 4 * (n16 & 3)) * 2;
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) {
      tr[2 * mb] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4d*)(vt + mb * 32));
      tr[2 * mb + 1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4d*)(vt + mb * 32 + 4 * VR));
    }
  };
  auto pv = [&](int buf) {      // acc^T[feature, head] += V^T P^T over the tile held in tr, P and rescale factors from buffer buf
    if (SCORES) return;
    const float al = alpha_lds[buf * 16 + n16];
    const vec8 pb = ld16<vec8>(p_lds + buf * (16 * FP_ROW) + n16 * FP_ROW + 8 * g4);
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) {
      const vec8 a = __builtin_bit_cast(vec8, (s16x8d)__builtin_shufflevector(tr[2 * mb], tr[2 * mb + 1], 0, 1, 2, 3, 4, 5, 6, 7));
      acc[mb] = Elem<T>::mfma16(a, pb, acc[mb] * al);
    }
  };

  // ---- pipeline ------------------------------------------------------------------------------------------------------------
  const f32x16 z16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  write_qhat(0);
  duo_wait_vmcnt<0>();      // the first tiles and the B operands
  // the compiler cannot see the direct-to-LDS loads: make it finish its own loads here, not inside the loop
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) asm volatile("" : "+v"(breg[ks]));
  __syncthreads();
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) ka[0] = Elem<T>::mfma32(breg[ks], tile_frag(0, ks), ks == 0 ? z16 : ka[0]);
  __syncthreads();          // every wave has read tile 0: with two streams its slot is refilled in the first iteration
  auto iteration = [&](int t, auto par_c) {
    constexpr int PAR = decltype(par_c)::value;
    f32x16& kn = ka[PAR ^ 1];          // tile t+1 (being reconstructed)
    const f32x16& kc = ka[PAR];        // tile t (being rotated)
    // ---- I1 ----
    vec8 fr[NKS];
#pragma unroll
    for (int i = 0; i < PF; ++i) fr[i] = tile_frag(t + 1, i);
    const sc_t* qr = qrow + PAR * qpar;
    const sc_vec8 qop0 = ld16<sc_vec8>(qr), qop1 = ld16<sc_vec8>(qr + 16);
    sc_vec8 kop[2];
    f32x4 sacc;
#pragma unroll
    for (int ks = 0; ks < KA; ++ks) {
      if (ks < 4) {              // two pairs of the rotation per group: registers r, r + 1 and their partners r + 8, r + 9
        // packed fp16 (v_pk_mul_f16 / v_pk_fma_f16): partial key sums and cos / sin rounded to fp16 first, as the
        // reference does (fp16 accumulators and fp16 cos / sin, flash_recontruction/qAB/v1.py:59-77)
        const int r = 2 * ks, o = r >> 2, e = r & 3;
        const rot2 a = {(_Float16)kc[r], (_Float16)kc[r + 1]}, bb = {(_Float16)kc[r + 8], (_Float16)kc[r + 9]};
        const rot2 lo2 = a * ch[ks] - bb * sh[ks], hi2 = bb * ch[ks] + a * sh[ks];
        kop[o][e] = lo2[0]; kop[o][e + 1] = lo2[1];
        kop[o][4 + e] = hi2[0]; kop[o][5 + e] = hi2[1];
      }
      if (ks + PF < NKS) fr[ks + PF] = tile_frag(t + 1, ks + PF);
      kn = Elem<T>::mfma32(breg[ks], fr[ks], ks == 0 ? z16 : kn);
      if (ks == 1) sacc = Elem<sc_t>::mfma16(kop[0], qop0, f32x4{0.f, 0.f, 0.f, 0.f});
      if (ks == 3) sacc = Elem<sc_t>::mfma16(kop[1], qop1, sacc);
      if (ks == 2) {             // scalar address work and the load issue run under the MFMAs already in the pipe
        XKV_DUO_FENCE();
        ks_.issue(end, last, wave, lane);          // key tile t + KAHEAD, into the slot freed at the last barrier
        if (V2) vs_.issue(end, last, wave, lane);  // value tile t + VAHEAD
      }
      if (ks == (KA > 5 ? 5 : KA - 1)) {
        if ((n16 & 7) < G)
          *reinterpret_cast<f32x4*>(s_part + (wave * 8 + (n16 & 7)) * FSP_ROW + 16 * (n16 >> 3) + 4 * g4) = sacc;
      }
      XKV_DUO_FENCE();
    }
    write_qhat(t + 1);       // into the buffer tile t does not read
    if (V2) duo_wait_vmcnt<S::WAIT_V>();   // this wave's rows of value tile t have landed
    __syncthreads();         // B1: partial scores of tile t, q^(t+1) visible; value tile t complete
    // ---- I2 ----
    // The softmax is a chain of dependent steps (LDS reads, adds, two cross-lane reductions, exponentials).  It is written
    // out in four stages, each led by its share of the remaining reconstruction MFMAs, so that the chain runs under them.
    constexpr int NI2 = NKS - KA, PER = (NI2 + 3) / 4;
    auto mfmas = [&](auto stage_c) {
      constexpr int S0 = KA + decltype(stage_c)::value * PER;
#pragma unroll
      for (int ks = S0; ks < S0 + PER; ++ks) {
        if (ks < NKS) {
          if (ks + PF < NKS) fr[ks + PF] = tile_frag(t + 1, ks + PF);
          kn = Elem<T>::mfma32(breg[ks], fr[ks], kn);
        }
      }
    };
    float al = 1.f;
    vec8 pb;
    if (!SCORES) {     // P and the rescale factors of tile t-1 were published before the last barrier
      al = alpha_lds[(PAR ^ 1) * 16 + n16];
      pb = ld16<vec8>(p_lds + (PAR ^ 1) * (16 * FP_ROW) + n16 * FP_ROW + 8 * g4);
    }
    f32x2d v[NW];
    {
      const float* sp = s_part + sm_row * FSP_ROW + 2 * n16;
#pragma unroll
      for (int w = 0; w < NW; ++w) v[w] = *reinterpret_cast<const f32x2d*>(sp + w * 8 * FSP_ROW);
    }
    const int tok = start + t * FT + 2 * n16;
    XKV_DUO_FENCE();
    // stage 0: sum the eight partial scores, scale, mask
    mfmas(std::integral_constant<int, 0>());
    float s0 = ((v[0][0] + v[1][0]) + (v[2][0] + v[3][0])) + ((v[4][0] + v[5][0]) + (v[6][0] + v[7][0]));
    float s1 = ((v[0][1] + v[1][1]) + (v[2][1] + v[3][1])) + ((v[4][1] + v[5][1]) + (v[6][1] + v[7][1]));
    float e0 = 0.f, e1 = 0.f, alpha = 1.f;
    if (SCORES) {
      if (sm_valid && lane < 16) {
        const int64_t o = ((int64_t)b * p.hq + h0 + wave) * p.kv_len + tok;
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
      XKV_DUO_FENCE();
      mfmas(std::integral_constant<int, 1>());
      mfmas(std::integral_constant<int, 2>());
      mfmas(std::integral_constant<int, 3>());
    } else {
      s0 = s0 * p.sm_scale + (tok < end ? 0.f : NEG_INF);       // (finite) - inf = -inf: masked without a branch
      s1 = s1 * p.sm_scale + (tok + 1 < end ? 0.f : NEG_INF);
      XKV_DUO_FENCE();
      // stage 1: the tile maximum of this head; the reference only moves when it exceeds it by lazy_rescale<T>()
      mfmas(std::integral_constant<int, 1>());
      const float mx = row_reduce<true, 16>(fmaxf(s0, s1));
      const float m_new = mx > m_ref + lazy_rescale<T>() ? mx : m_ref;
      XKV_DUO_FENCE();
      // stage 2: exponentials, P and the rescale factor -> LDS (buffer t & 1; absent heads keep zeros)
      mfmas(std::integral_constant<int, 2>());
      alpha = __expf(m_ref - m_new);
      m_ref = m_new;
      e0 = __expf(s0 - m_ref);
      e1 = __expf(s1 - m_ref);
      T* pd = p_lds + PAR * (16 * FP_ROW) + wave * FP_ROW + 2 * n16;   // the four 16-lane groups store the same values
      pd[0] = from_f32<T>(sm_valid ? e0 : 0.f);
      pd[1] = from_f32<T>(sm_valid ? e1 : 0.f);
      alpha_lds[PAR * 16 + wave] = sm_valid ? alpha : 1.f;
      XKV_DUO_FENCE();
      // stage 3: acc += P.A of tile t-1 from the operands in registers, then tile t's operands replace them
      mfmas(std::integral_constant<int, 3>());
#pragma unroll
      for (int mb = 0; mb < NMB; ++mb) {
        const vec8 a = __builtin_bit_cast(vec8, (s16x8d)__builtin_shufflevector(tr[2 * mb], tr[2 * mb + 1], 0, 1, 2, 3, 4, 5, 6, 7));
        acc[mb] = Elem<T>::mfma16(a, pb, acc[mb] * al);
      }
      XKV_DUO_FENCE();
      tr_read(t);
      l_run = l_run * alpha + row_reduce<false, 16>(e0 + e1);
    }
    XKV_DUO_FENCE();
    duo_wait_vmcnt<S::WAIT_K>();   // this wave's rows of key tile t+2 have landed
    __syncthreads();         // B2: P, rescale factors of tile t visible; key tile t+2 complete; the slots read in this
                             // iteration are free
  };
  for (int t = 0; t < ntiles; t += 2) {
    iteration(t, std::integral_constant<int, 0>());
    if (t + 1 < ntiles) iteration(t + 1, std::integral_constant<int, 1>());
  }
  pv((ntiles - 1) & 1);      // P.A of the last tile
  duo_wait_vmcnt<0>();       // the clamped look-ahead loads must land before the LDS is released
  if (SCORES) return;
  if (sm_valid && lane == 0) { ml_lds[2 * wave] = m_ref; ml_lds[2 * wave + 1] = l_run; }
  __syncthreads();

  // ---- epilogue ----------------------------------------------------------------------------------------------------------
  if (n16 < G) {
    const float m = ml_lds[2 * n16], l = ml_lds[2 * n16 + 1];
    const float inv = 1.f / l;
    const int64_t ph = ((int64_t)b * p.hq + h0 + n16) * p.max_splits + split;
    float* dst = p.partial + ph * DV + wave * (DV / 8) + 4 * g4;
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) *reinterpret_cast<f32x4*>(dst + mb * 16) = acc[mb] * inv;
    if (wave == 0 && g4 == 0) p.lse[ph] = m + __logf(l);
  }
}

template <typename T, int RK, int RV, int MODE>
int launch_duo_t(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, hipStream_t st) {
  typedef DuoShape<RK, RV, MODE> S;
  const int nb = sBb == 0 ? 1 : batch;   // one packed copy when the factor is shared by the batch
  duo_pack_b_kernel<T, RK><<<dim3(p.hkv, nb, 16), dim3(256), 0, st>>>((const T*)kB, (T*)p.Bp, sBb, sBh, sBr, p.hkv);
  auto kern = recon_duo_kernel<T, RK, RV, MODE>;
  static DynLds lds;
  const int e = ensure_dynamic_lds(lds, reinterpret_cast<const void*>(kern), S::SHM, true);
  if (e != XKV_OK) return e;
  const int total = batch * p.hkv * p.max_splits;
  kern<<<dim3(xcd_grid(total, p.hkv)), dim3(64 * NW), S::SHM, st>>>(p);
  return launch_status();
}

template <int RK, int RV, int MODE>
int launch_duo(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype, hipStream_t st) {
  return dtype == XKV_BF16 ? launch_duo_t<__bf16, RK, RV, MODE>(p, kB, sBb, sBh, sBr, batch, st)
                           : launch_duo_t<_Float16, RK, RV, MODE>(p, kB, sBb, sBh, sBr, batch, st);
}

}  // namespace duo
}  // namespace xkv
