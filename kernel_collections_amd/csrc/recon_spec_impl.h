// Wave-specialised form of the fused reconstruct + RoPE + softmax + P.A stage 1 (rank RK = 512 / 384 / 256, head_dim 128,
// the token basis shared by K and V): 8 wavefronts per workgroup, two per SIMD, with different jobs.
//
// Reconstruction waves (0..3) form the 2 x 2 grid over (rank half kq, feature half dq) of recon_fast_impl.h: wave (kq, dq)
// keeps its quarter of B_h stationary in RK / 4 accumulation registers and issues nothing but the v_mfma_f32_32x32x16 of the
// 32-token tile, the LDS reads of its operands, and the hand-over of the finished partial key tile - rounded to fp16, 16 KB
// per tile - to the consumer waves through a double-buffered LDS area.  Their instruction stream is 32 MFMAs against ~40
// other instructions per tile, so the matrix pipe of the SIMD stays fed.
// Consumer waves (4..7; consumer c owns pairs 32 (c / 2) + 16 (c % 2) .. + 16 of the rotate-half pairs and RK / 4 latent
// features of P.A) do everything else, each step one workgroup barrier behind the one before it:
//   period p:  tile loads of tile p+2 (direct to LDS, ring of 3 slots)
//              softmax + P.A of tile p-3 (scores summed from the four consumers' partial scores; the softmax is computed by
//                every consumer for all heads, so P goes from registers straight into the MFMA operand)
//              transposed reads of tile p for its P.A, kept in accumulation registers until period p+3 (3 sets of RK / 16)
//              rotation + q-dot of tile p-2 (adds the two rank halves, rotates in packed fp16, v_mfma_f32_16x16x32)
//              q^ for the next pair of tiles (even p)
// One barrier per period is the only synchronisation: everything a period reads was written at least one barrier earlier, and
// the four activities of a consumer period do not depend on each other.  A tile stays in the LDS ring for one period only
// (both its readers, the reconstruction and the transposed reads, run in period p), which is what makes 3 slots enough.
#pragma once
#include "recon_fast_impl.h"
#include <utility>


namespace xkv {
namespace spec {
using namespace fast;

constexpr int SRING = 3;
template <int RK> struct SpecShape {
  static_assert(RK == 512 || RK == 384 || RK == 256, "rank");
  static constexpr int FROW = RK * 2 + 16;     // LDS bytes per tile row
  static constexpr int FTILE = FT * FROW;
  static constexpr int NKS = RK / 32;          // k-steps of a reconstruction wave (16 ranks each)
  static constexpr int NMB = RK / 64;          // 16-feature blocks of the RK / 4 latent features a consumer owns in P.A
  static constexpr int KB_BYTES = 16 * 1024;   // one key buffer: [kq 2][dq 2][part 2][blk 2][lane 64] x 16 bytes of fp16
  static constexpr int SP_FLOATS = 4 * 8 * FSP_ROW;   // one buffer of partial scores: [consumer 4][head 8][FSP_ROW]
  static constexpr int LATE = NKS / 4;         // k-steps of a tile that run after the barrier that ends its period
  static constexpr int EARLY = 2;              // operand reads are issued this many slots before the uniform one-per-slot rate
  static constexpr int NLR = 2;                // rows of a wave pair's eight that the reconstruction wave loads (measured: 0, 2, 4, 6, 8)
  // slot of a reconstruction period in which hand-over unit un (0..3) of the previous tile is converted and written
  static constexpr int unit_step(int un) { return LATE + 2 + un * (NKS - LATE - 3) / 4; }
  static constexpr size_t SHM = (size_t)SRING * FTILE + 2 * KB_BYTES + 2 * SP_FLOATS * 4 + 2 * 8 * 128 * 2 + 128 * 2;
};

typedef _Float16 h2 __attribute__((ext_vector_type(2)));

template <int CTRL> __device__ __forceinline__ unsigned dpp_u32(unsigned x) {
  return (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xf, 0xf, true);
}
// The consumer's accumulation registers are managed by hand, by register number, in asm statements: a[0 .. RK/16) hold the P.A
// accumulators (block mb in a[4 mb .. 4 mb + 3]), a[RK/16 .. RK/4) three sets of transposed tile reads (set s, block mb in
// a[RK/16 (1 + s) + 4 mb .. + 3]).  The compiler must not manage them: the reads are in flight for a period (a register copy
// it inserted would copy stale contents), and it picks one register class for all MFMA results of a kernel.  Its own code
// in the consumer branch uses no accumulation register (the build checks the consumer's ordinary registers do not spill).
// Nothing reads an accumulator sooner than a barrier after the MFMA that wrote it, so no wait states are needed there.
// The first MFMA of a tile follows the VALU instructions that formed pb; as asm it gets no hazard handling from the compiler,
// so the wait states a VALU result needs before an MFMA may read it are part of the statement.
template <typename T, int ACC, int A> __device__ __forceinline__ void pa_mfma_at(u32x4 pb) {
  if constexpr (std::is_same<T, __bf16>::value) {
    if constexpr (ACC == 0)
      asm volatile("s_nop 7\n\tv_mfma_f32_16x16x32_bf16 a[%1:%2], a[%3:%4], %0, a[%1:%2]" ::"v"(pb), "n"(ACC), "n"(ACC + 3), "n"(A), "n"(A + 3));
    else
      asm volatile("v_mfma_f32_16x16x32_bf16 a[%1:%2], a[%3:%4], %0, a[%1:%2]" ::"v"(pb), "n"(ACC), "n"(ACC + 3), "n"(A), "n"(A + 3));
  } else {
    if constexpr (ACC == 0)
      asm volatile("s_nop 7\n\tv_mfma_f32_16x16x32_f16 a[%1:%2], a[%3:%4], %0, a[%1:%2]" ::"v"(pb), "n"(ACC), "n"(ACC + 3), "n"(A), "n"(A + 3));
    else
      asm volatile("v_mfma_f32_16x16x32_f16 a[%1:%2], a[%3:%4], %0, a[%1:%2]" ::"v"(pb), "n"(ACC), "n"(ACC + 3), "n"(A), "n"(A + 3));
  }
}
template <int R, int OFF> __device__ __forceinline__ void tr_read_at(unsigned addr) {
  asm volatile("ds_read_b64_tr_b16 a[%1:%2], %0 offset:%3" ::"v"(addr), "n"(R), "n"(R + 1), "n"(OFF) : "memory");
}
template <int R> __device__ __forceinline__ void acc_set_at(float x) { asm volatile("v_accvgpr_write_b32 a%1, %0" ::"v"(x), "n"(R)); }
template <int R> __device__ __forceinline__ float acc_get_at() {
  float x;
  asm volatile("v_accvgpr_read_b32 %0, a%1" : "=v"(x) : "n"(R));
  return x;
}
template <int... I, typename F> __device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(IC<I>()), ...);
}
template <int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>(), f);
}
template <typename T> __device__ __forceinline__ unsigned pack_pair(float a, float b) {
  typedef T t2 __attribute__((ext_vector_type(2)));
  const t2 v = {from_f32<T>(a), from_f32<T>(b)};
  return __builtin_bit_cast(unsigned, v);
}

// GP: head slots of a kv head rounded up to 4 or 8 (softmax lane layout).  SCORES: write the scaled scores only.
template <typename T, bool SCORES, int RK, int GP>
__global__ __launch_bounds__(512) void recon_spec_kernel(const FastParams p) {
  typedef typename Elem<T>::vec8 vec8;
  typedef SpecShape<RK> S;
  constexpr int FROW = S::FROW, FTILE = S::FTILE, NKS = S::NKS, NMB = S::NMB, KB_BYTES = S::KB_BYTES, SP_FLOATS = S::SP_FLOATS;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
  const int nfull = (end - start) / FT;
  const int last = end - 1;
  const int NP6 = (ntiles + 3 + 5) / 6 * 6;   // periods (one barrier each); the last tile's P.A runs in period ntiles + 2

  // ---- LDS carve-up ---------------------------------------------------------------------------------------------
  unsigned char* ring = smem;                                              // SRING * FTILE
  unsigned char* keybuf = smem + SRING * FTILE;                            // 2 * KB_BYTES
  float* s_part = reinterpret_cast<float*>(keybuf + 2 * KB_BYTES);         // [2][4 consumers][8 heads][FSP_ROW]
  sc_t* qhat = reinterpret_cast<sc_t*>(s_part + 2 * SP_FLOATS);            // [2][8 heads][128]
  sc_t* qzero = qhat + 2 * 8 * 128;                                        // [128] zeros: the q-dot operand of masked lanes
  const unsigned ring_lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)ring;
  if (tid < 128) qzero[tid] = from_f32<sc_t>(0.f);

  // ---- async tile loads: rows 8 wq .. 8 wq + 7 of a tile belong to reconstruction wave wq (the first NLR of them, one behind
  // each of its first MFMA slots) and consumer wq (the rest); one row (RK * 2 bytes: lanes 0 .. RK/8 - 1) per instruction ----
  const int wq = wave & 3;
  constexpr int NLR = S::NLR;
  const unsigned char* Ab = reinterpret_cast<const unsigned char*>(p.kA) + b * p.sAb * 2;
  const int64_t row_bytes = p.sAl * 2;
  const unsigned lane_off = lane * 16;
  unsigned voff4[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) voff4[r] = lane_off + 128u + (unsigned)(r * ((int)row_bytes - FROW));
  auto issue_one = [&](int t, auto slot_c, auto r_c, auto full_c) {
    constexpr int R = decltype(r_c)::value, SLOT = decltype(slot_c)::value;
    const int tok0 = start + t * FT + wq * 8;
    const bool live = RK == 512 || lane < RK / 8;   // scalar addresses are formed outside this lane predicate
    if (decltype(full_c)::value) {
      const unsigned dst = ring_lds + (unsigned)SLOT * FTILE + (unsigned)(wq * 8 + (R & ~3)) * FROW;
      const unsigned char* base = Ab + (int64_t)(tok0 + (R & ~3)) * row_bytes - 128;
      if (live) async_row_off<(R & 3) * FROW>(base, voff4[R & 3], dst);
    } else {
      int tok = tok0 + R;
      tok = tok < last ? tok : last;   // rows past the split end are masked in the softmax; keep the read in bounds
      const unsigned char* rowp = Ab + (int64_t)tok * row_bytes;
      const unsigned dst = ring_lds + (unsigned)SLOT * FTILE + (unsigned)(wq * 8 + R) * FROW;
      if (live) async_row16(rowp, lane_off, dst);
    }
  };
  auto issue_rows = [&](int t, auto slot_c, auto full_c, auto r0_c, auto r1_c) {   // rows [R0, R1) of this wave's eight
    constexpr int R0 = decltype(r0_c)::value, R1 = decltype(r1_c)::value;
    static_for<R1 - R0>([&](auto i_c) { issue_one(t, slot_c, IC<R0 + decltype(i_c)::value>(), full_c); });
  };
  if (wave < 4) {
    // =================================================================================================================
    // reconstruction wave (kq, dq)
    // =================================================================================================================
    const int kq = wave >> 1, dq = wave & 1;
    // B operands go from memory straight into accumulation registers (no transit through the 128 ordinary registers the
    // kernel may use): the loads are asm, and so is the wait for them.
    vec8 breg[NKS][2];
    {
      const T* bp = reinterpret_cast<const T*>(p.Bp) + b * p.sBpb + (int64_t)kh * (RK * 128) + (int64_t)wave * (128 * NKS) * 8;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
          asm volatile("global_load_dwordx4 %0, %1, %2" : "=a"(breg[ks][blk]) : "v"((unsigned)(lane * 16 + (ks * 2 + blk) * 1024)), "s"(bp) : "memory");
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    f32x16 ka[2][2];       // two sets of partial key accumulators [set][low | partner feature block]
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int k = 0; k < 2; ++k)
#pragma unroll
        for (int r = 0; r < 16; ++r) ka[s][k][r] = 0.f;
    const unsigned char* fr0 = ring + n32 * FROW + ((RK / 2) * kq + 8 * g2) * 2;
    unsigned char* kw0 = keybuf + ((kq * 2 + dq) * 4) * 1024 + lane * 16;
    __syncthreads();        // the consumers' prologue: tiles 0 and 1 and q^(0) are in the LDS

    // Period pp: the last LATE k-steps of tile pp-1 (accumulator set (pp-1) % 2; their operands were read before the barrier,
    // so the matrix pipe has work while the first operands of tile pp travel from the LDS), then the first NKS - LATE k-steps
    // of tile pp (set pp % 2), with the hand-over of tile pp-1 through key buffer (pp-1) % 2 dealt out among them.
    // u = pp % 6 fixes every register and slot index at compile time.
    constexpr int LATE = S::LATE, EARLY = S::EARLY;
    vec8 carry[LATE];      // operands of the previous tile's last LATE k-steps
#pragma unroll
    for (int v = 0; v < LATE; ++v) carry[v] = ld16<vec8>(fr0 + v * 32);
    auto period = [&](int pp, auto u_c) {
      constexpr int u = decltype(u_c)::value, PAR = u & 1, SLOT = u % 3;
      f32x16& k0 = ka[PAR][0];
      f32x16& k1 = ka[PAR][1];
      f32x16& j0 = ka[PAR ^ 1][0];
      f32x16& j1 = ka[PAR ^ 1][1];
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        asm volatile("" : "+a"(breg[ks][0]));
        asm volatile("" : "+a"(breg[ks][1]));
      }
      const unsigned char* fr = fr0 + SLOT * FTILE;
      unsigned char* kw = kw0 + (PAR ^ 1) * KB_BYTES;
      // hand-over unit un: registers 8 part .. + 8 of block blk, i.e. what consumer (dq, part) rotates, as 8 fp16
      auto write_unit = [&](auto un_c) {
        constexpr int un = decltype(un_c)::value, part = un >> 1, blk = un & 1;
        const f32x16& src = blk ? j1 : j0;
        const h2 v0 = {(_Float16)src[8 * part + 0], (_Float16)src[8 * part + 1]};
        const h2 v1 = {(_Float16)src[8 * part + 2], (_Float16)src[8 * part + 3]};
        const h2 v2 = {(_Float16)src[8 * part + 4], (_Float16)src[8 * part + 5]};
        const h2 v3 = {(_Float16)src[8 * part + 6], (_Float16)src[8 * part + 7]};
        const f16x8 pk = {v0[0], v0[1], v1[0], v1[1], v2[0], v2[1], v3[0], v3[1]};
        st16(kw + (part * 2 + blk) * 1024, pk);
      };
      // Past the last tile (and in period 0, which finishes and hands over a tile that does not exist) the same code runs on
      // whatever the LDS holds: nothing downstream uses those results, and one code path keeps the loop a single block.
      if (pp <= ntiles) {
        vec8 at[NKS];
        static_for<NKS>([&](auto v_c) {   // slot v of the period: one k-step = two MFMAs
          constexpr int v = decltype(v_c)::value;
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks)
            if ((ks > EARLY ? ks - EARLY : 0) == v) at[ks] = ld16<vec8>(fr + ks * 32);   // read EARLY + LATE slots ahead of use
          if constexpr (v < LATE) {
            constexpr int ksl = NKS - LATE + v;
            j0 = Elem<T>::mfma32(breg[ksl][0], carry[v], j0);
            j1 = Elem<T>::mfma32(breg[ksl][1], carry[v], j1);
          } else if constexpr (v == LATE) {
            const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            k0 = Elem<T>::mfma32(breg[0][0], at[0], z);
            k1 = Elem<T>::mfma32(breg[0][1], at[0], z);
          } else {
            k0 = Elem<T>::mfma32(breg[v - LATE][0], at[v - LATE], k0);
            k1 = Elem<T>::mfma32(breg[v - LATE][1], at[v - LATE], k1);
          }
          // this wave's share of the loads of tile pp+2, spread evenly over the period: the CU's address unit takes 16 clocks
          // per 1 KiB load, and a wave that issues into a full queue stalls
          constexpr int LSTEP = NKS / (NLR > 0 ? NLR : 1);
          if constexpr (NLR > 0 && v % LSTEP == LSTEP / 2 && v / LSTEP < NLR) {
            XKV_FENCE();
            issue_one(pp + 2, IC<(u + 2) % 3>(), IC<v / LSTEP>(), IC<0>());   // (row clamped to the split: one code path)
            XKV_FENCE();
          }
          if (S::unit_step(0) == v) write_unit(IC<0>());
          if (S::unit_step(1) == v) write_unit(IC<1>());
          if (S::unit_step(2) == v) write_unit(IC<2>());
          if (S::unit_step(3) == v) write_unit(IC<3>());
          XKV_FENCE();
        });
#pragma unroll
        for (int v = 0; v < LATE; ++v) carry[v] = at[NKS - LATE + v];
        if (NLR > 0) wait_vmcnt<NLR>();   // this wave's rows of tile pp+1 have landed
      }
      __syncthreads();
    };
    for (int pb = 0; pb < NP6; pb += 6) {
      period(pb, IC<0>()); period(pb + 1, IC<1>()); period(pb + 2, IC<2>());
      period(pb + 3, IC<3>()); period(pb + 4, IC<4>()); period(pb + 5, IC<5>());
    }
    wait_vmcnt<0>();
    return;
  }

  // ===================================================================================================================
  // consumer wave c
  // ===================================================================================================================
  const int c = wave - 4, dq = c >> 1, part = c & 1;

  issue_rows(0, IC<0>(), IC<0>(), IC<0>(), IC<8>());   // the first two tiles: all eight rows from the consumer
  issue_rows(1, IC<1>(), IC<0>(), IC<0>(), IC<8>());

  // ---- in-tile rotation tables: this consumer's 8 pairs per lane (token n32, g2): r = 8 part + 2k, + 1 -------------------
  // pair index j = 32 dq + 8 (r / 4) + 4 g2 + r % 4; two tables: the query-side base is that of an EVEN tile and serves the
  // odd tile after it too, whose offsets are 32 .. 63.
  h2 ch[2][4], sh[2][4];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int r = 8 * part + 2 * k;
      float c0, s0, c1, s1;
      __sincosf((float)(n32 + 32 * h) * p.inv_freq[32 * dq + 8 * (r >> 2) + 4 * g2 + (r & 3)], &s0, &c0);
      __sincosf((float)(n32 + 32 * h) * p.inv_freq[32 * dq + 8 * ((r + 1) >> 2) + 4 * g2 + ((r + 1) & 3)], &s1, &c1);
      ch[h][k] = h2{(_Float16)c0, (_Float16)c1};
      sh[h][k] = h2{(_Float16)s0, (_Float16)s1};
    }

  // ---- query-side base rotation: thread -> pair j = lane, head slots c and c + 4 ------------------------------------------
  float q0[2], q1[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int h = c + 4 * i;
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
  float qc32, qs32, qcb, qsb;   // (qcb, qsb): base rotation of the tile whose q^ is written next
  sincosf((float)(2 * FT) * qinv, &qs32, &qc32);   // the base advances two tiles at a time
  // The base advances by angle addition and is replaced by a freshly range-reduced value every 30 tiles
  auto seed_qhat = [&](int t) { sincosf((float)(p.pos_offset + start + (int64_t)t * FT) * qinv, &qsb, &qcb); };
  seed_qhat(0);
  auto write_qhat = [&](int t) {   // q^ for the even tile t and the odd one after it = R(-base(t)) q, into buffer (t / 2) & 1
    sc_t* dst = qhat + ((t >> 1) & 1) * (8 * 128) + c * 128 + qpos;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (i == 1 && GP <= 4) break;   // head slots 4..7 are absent: nothing reads their rows
      dst[i * 512] = from_f32<sc_t>(q0[i] * qcb + q1[i] * qsb);
      dst[i * 512 + 4] = from_f32<sc_t>(q1[i] * qcb - q0[i] * qsb);
    }
    const float cc = qcb * qc32 - qsb * qs32, ss = qsb * qc32 + qcb * qs32;
    qcb = cc; qsb = ss;
  };
  write_qhat(0);

  // ---- q-dot B operand source: lanes whose token half (lane bit 4) matches their column's (lane bit 3) read q^ of head
  // lane % 8 (absent heads: the last one; their columns are not stored), the others read zeros ------------------------------
  const bool q_live = ((lane >> 4) & 1) == ((lane >> 3) & 1);
  const sc_t* qsrc = q_live ? qhat + ((lane & 7) < G ? (lane & 7) : G - 1) * 128 + (dq * 2 + g2) * 8 : qzero;
  const int qpar = q_live ? 8 * 128 : 0;   // q^ is double-buffered by tile pair, the zeros are not

  // ---- softmax role: every consumer computes P of all heads; lane (n16, g4) holds head n16 % GP, tokens 8 g4 + TPL (n16 / GP) ..
  constexpr int TPL = GP / 2;   // tokens per lane
  const int sm_head = n16 & (GP - 1);
  const int sm_row = sm_head < G ? sm_head : G - 1;
  const int sm_tok = 8 * g4 + TPL * (n16 / GP);
  float m_ref = NEG_INF, l_run = 0.f;   // reference maximum of the lane's head (base-2 domain); this lane's share of its row sum
  const float scale2 = p.sm_scale * 1.44269504088896f, lazy2 = lazy_rescale<T>() * 1.44269504088896f;
  // P.A accumulators (consumer c owns latent features RK/4 c .. + RK/4; column n16 = head slot) and the transposed tile reads
  // of three tiles live in accumulation registers a[0 .. RK/4), by number (see pa_mfma_at)
  constexpr int TR0 = 4 * NMB, TRSET = 4 * NMB;
  static_for<4 * NMB>([&](auto r_c) { acc_set_at<decltype(r_c)::value>(0.f); });
  if constexpr (RK == 512) asm volatile("" ::: "a127");   // the kernel owns a[0 .. RK/4) whatever the reconstruction branch pins
  else if constexpr (RK == 384) asm volatile("" ::: "a95");
  else asm volatile("" ::: "a63");

  wait_vmcnt<0>();          // tiles 0 and 1
  __syncthreads();

  // Transposed reads: a 16-lane group reads a block of 4 rows x 16 columns, lanes 4 j .. 4 j + 3 supplying row j, and lane i
  // receives column i (4 values, one per row).  Rows 2 j (first read) and 2 j + 1 (second read) of the group's 8 tokens: with
  // the 16-byte row padding, rows two apart start 8 banks apart, so the 32-byte pieces of a read do not overlap (adjacent rows
  // would, by half).  Element e of the lane's 8 contraction values is therefore token 8 g4 + 2 e (e < 4) or 8 g4 + 2 (e - 4) + 1.
  const unsigned tr_base = ring_lds + (unsigned)((8 * g4 + 2 * (n16 >> 2)) * FROW + (c * (RK / 4) + 4 * (n16 & 3)) * 2);
  const unsigned char* kr0 = keybuf + (dq * 4 + part * 2) * 1024 + lane * 16;

  // rotation + q-dot of tile t: partial scores (over this consumer's 16 pairs) for all heads and the 32 tokens.  The LDS reads
  // are a step of their own so that a period can issue all its reads first and compute while they travel.
  struct S1In { f16x8 k[4]; sc_vec8 q[2]; };
  auto stage1_load = [&](int t, auto kbuf_c) {
    constexpr int KBUF = decltype(kbuf_c)::value;
    const unsigned char* kr = kr0 + KBUF * KB_BYTES;
    const sc_t* qrow = qsrc + ((t >> 1) & 1) * qpar + (2 * part) * 32;
    S1In in;
    in.k[0] = ld16<f16x8>(kr); in.k[1] = ld16<f16x8>(kr + 8192);                  // rank halves kq = 0, 1 of the low block
    in.k[2] = ld16<f16x8>(kr + 1024); in.k[3] = ld16<f16x8>(kr + 1024 + 8192);    // ... of the partner block
    in.q[0] = ld16<sc_vec8>(qrow); in.q[1] = ld16<sc_vec8>(qrow + 32);
    return in;
  };
  struct S1Rot { sc_vec8 kop[2]; };
  auto stage1_rotate = [&](const S1In& in, auto tpar_c) {   // adds the rank halves and rotates: the q-dot's A operands
    constexpr int TPAR = decltype(tpar_c)::value;
    const f16x8 lo = in.k[0] + in.k[1], hi = in.k[2] + in.k[3];
    S1Rot r;
#pragma unroll
    for (int oo = 0; oo < 2; ++oo) {
      h2 lo2[2], hi2[2];
#pragma unroll
      for (int e2 = 0; e2 < 2; ++e2) {
        const h2 a = {lo[4 * oo + 2 * e2], lo[4 * oo + 2 * e2 + 1]}, bb = {hi[4 * oo + 2 * e2], hi[4 * oo + 2 * e2 + 1]};
        lo2[e2] = a * ch[TPAR][2 * oo + e2] - bb * sh[TPAR][2 * oo + e2];
        hi2[e2] = bb * ch[TPAR][2 * oo + e2] + a * sh[TPAR][2 * oo + e2];
      }
      r.kop[oo] = sc_vec8{lo2[0][0], lo2[0][1], lo2[1][0], lo2[1][1], hi2[0][0], hi2[0][1], hi2[1][0], hi2[1][1]};
    }
    return r;
  };
  auto stage1_dot = [&](const S1Rot& r, const S1In& in, auto tpar_c) {
    constexpr int TPAR = decltype(tpar_c)::value;
    // as the A operand of v_mfma_f32_16x16x32, lane (n32, g2) is row n32 % 16 and k-group (n32 / 16) + 2 g2; the B operand
    // keeps the token halves apart (column c' holds q^ of head c' % 8 in the k-groups of token half c' / 8, zeros elsewhere).
    // Result: lane (c', g4), register r = score of token 16 (c' / 8) + 4 g4 + r for head c' % 8.
    f32x4 sacc = Elem<sc_t>::mfma16(r.kop[0], in.q[0], f32x4{0.f, 0.f, 0.f, 0.f});
    sacc = Elem<sc_t>::mfma16(r.kop[1], in.q[1], sacc);
    if ((n16 & 7) < G)
      *reinterpret_cast<f32x4*>(s_part + TPAR * SP_FLOATS + (c * 8 + (n16 & 7)) * FSP_ROW + 16 * (n16 >> 3) + 4 * g4) = sacc;
  };

  // softmax and P.A of tile t (partial scores in buffer t % 2, transposed tile in register set t % 3)
  typedef float fv __attribute__((ext_vector_type(TPL)));
  struct S23In { fv a[4]; };
  auto stage23_load = [&](auto tpar_c) {
    constexpr int TPAR = decltype(tpar_c)::value;
    S23In in;
    if (!SCORES) {
      const float* sp = s_part + TPAR * SP_FLOATS + sm_row * FSP_ROW + sm_tok;
#pragma unroll
      for (int w = 0; w < 4; ++w) in.a[w] = *reinterpret_cast<const fv*>(sp + w * 8 * FSP_ROW);
    }
    return in;
  };
  // (FULL: the tile lies wholly inside the split, no token is masked.)  The softmax runs in the base-2 domain: scores are
  // scaled by sm_scale * log2(e) in one multiplication and the reference maximum is kept in that domain, so that P is one
  // subtraction and one v_exp_f32 per score.
  auto stage23 = [&](int t, const S23In& in, auto ts_c, auto tpar_c, auto full_c) {
    constexpr int TS = decltype(ts_c)::value, TPAR = decltype(tpar_c)::value;
    constexpr bool FULL = decltype(full_c)::value != 0;
    if (SCORES) {   // consumer c writes heads c and c + 4: lane -> (head c + 4 (lane / 32), token lane % 32)
      const int head = c + 4 * g2;
      const float* sp = s_part + TPAR * SP_FLOATS + (head < G ? head : G - 1) * FSP_ROW + n32;
      const float s = ((sp[0] + sp[8 * FSP_ROW]) + (sp[2 * 8 * FSP_ROW] + sp[3 * 8 * FSP_ROW])) * p.sm_scale;
      const int tok = start + t * FT + n32;
      if (head < G && tok < end) {
        const int64_t o = ((int64_t)b * p.hq + h0 + head) * p.kv_len + tok;
        if (p.scores_dtype == XKV_F32) reinterpret_cast<float*>(p.scores)[o] = s;
        else reinterpret_cast<T*>(p.scores)[o] = from_f32<T>(s);
      }
      return;
    }
    float s[TPL];
    {
      const fv sum = (in.a[0] + in.a[1]) + (in.a[2] + in.a[3]);
#pragma unroll
      for (int e = 0; e < TPL; ++e) s[e] = sum[e];
    }
    const int tok = start + t * FT + sm_tok;
    float mxl = NEG_INF;
#pragma unroll
    for (int e = 0; e < TPL; ++e) {
      s[e] = (FULL || tok + e < end) ? s[e] * scale2 : NEG_INF;
      mxl = fmaxf(mxl, s[e]);
    }
    // the reference maximum only moves when the tile maximum exceeds it by the lazy bound; the cross-lane reduction that
    // finds the maximum runs only then.  Every consumer sees the same scores, so all four keep the same reference.
    if (__builtin_amdgcn_ballot_w64(mxl > m_ref + lazy2)) {   // rare: some head's maximum moves
      float mx = mxl;
#pragma unroll
      for (int m = GP; m < 64; m <<= 1) mx = fmaxf(mx, __shfl_xor(mx, m));
      const float m_new = mx > m_ref + lazy2 ? mx : m_ref;
      const float alpha = __builtin_amdgcn_exp2f(m_ref - m_new);
      m_ref = m_new;
      l_run *= alpha;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {   // column n16 < GP of the accumulators is this lane's head
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
        static_for<4 * NMB>([&](auto r_c) { acc_set_at<decltype(r_c)::value>(acc_get_at<decltype(r_c)::value>() * alpha); });
        asm volatile("s_nop 7" ::: "memory");
      }
    }
    float e[TPL];
    float esum = 0.f;
#pragma unroll
    for (int k = 0; k < TPL; ++k) {
      e[k] = __builtin_amdgcn_exp2f(s[k] - m_ref);
      esum += e[k];
    }
    l_run += esum;
    // P as the B operand of v_mfma_f32_16x16x32: lane (column n16 = head, g4) holds its head's tokens 8 g4 .. + 8 in the order
    // of the transposed reads (even tokens, then odd ones); lanes n16 < GP gather the other token groups of their head from
    // lanes n16 + GP, ... of the same 16-lane row (columns >= GP are unused)
    u32x4 pbu;
    if (GP == 4) {   // this lane: tokens 2 tq, 2 tq + 1; lane + 4: the next two
      const float y0 = __builtin_bit_cast(float, dpp_u32<0x104>(__builtin_bit_cast(unsigned, e[0])));
      const float y1 = __builtin_bit_cast(float, dpp_u32<0x104>(__builtin_bit_cast(unsigned, e[1])));
      const unsigned ev = pack_pair<T>(e[0], y0), od = pack_pair<T>(e[1], y1);   // (2 tq, 2 tq + 2), (2 tq + 1, 2 tq + 3)
      pbu = u32x4{ev, dpp_u32<0x108>(ev), od, dpp_u32<0x108>(od)};
    } else {         // this lane: tokens 4 tq .. + 4
      const unsigned ev = pack_pair<T>(e[0], e[TPL > 2 ? 2 : 0]), od = pack_pair<T>(e[1], e[TPL > 2 ? 3 : 1]);
      pbu = u32x4{ev, dpp_u32<0x108>(ev), od, dpp_u32<0x108>(od)};
    }
    static_for<NMB>([&](auto mb_c) {
      constexpr int mb = decltype(mb_c)::value;
      pa_mfma_at<T, 4 * mb, TR0 + TS * TRSET + 4 * mb>(pbu);
    });
  };

  // transposed reads of the tile in ring slot SLOT into register set TS; completion is awaited before the period's barrier
  auto trread = [&](auto ts_c, auto slot_c) {
    constexpr int TS = decltype(ts_c)::value, SLOT = decltype(slot_c)::value;
    const unsigned vt = tr_base + (unsigned)SLOT * FTILE;
    static_for<NMB>([&](auto mb_c) {
      constexpr int mb = decltype(mb_c)::value;
      tr_read_at<TR0 + TS * TRSET + 4 * mb, mb * 32>(vt);
      tr_read_at<TR0 + TS * TRSET + 4 * mb + 2, mb * 32 + FROW>(vt);
    });
  };

  // STEADY: tiles pp-3 .. pp+2 all exist and tile pp+2 lies wholly inside the split.  Otherwise only the softmax + P.A step is
  // guarded (it must not touch its state for a tile that does not exist); the other steps run on whatever the LDS holds
  // (loads clamp their rows to the split), and nothing uses their results.
  // The consumer's share of the tile loads is dealt out over the period in four portions: the CU's address unit takes 16
  // clocks per 1 KiB load, and a wave that issues into a full queue stalls.
  auto period = [&](int pp, auto u_c, auto steady_c) {
    constexpr int u = decltype(u_c)::value;
    constexpr bool STEADY = decltype(steady_c)::value != 0;
    constexpr int NLC = 8 - NLR, LC1 = NLR + (NLC + 3) / 4, LC2 = NLR + (2 * NLC + 3) / 4, LC3 = NLR + (3 * NLC + 3) / 4;
    const int t_pv = pp - 3;
    const bool pv_live = STEADY || (t_pv >= 0 && t_pv < ntiles);
    if (STEADY || pp < ntiles + 3) {
      // all LDS reads of the period first; the first tile loads are issued while they travel
      const S1In in1 = stage1_load(pp - 2, IC<u & 1>());
      const S23In in23 = stage23_load(IC<(u + 1) & 1>());
      XKV_FENCE();
      issue_rows(pp + 2, IC<(u + 2) % 3>(), steady_c, IC<NLR>(), IC<LC1>());
      XKV_FENCE();
      // the rotation's VALU work next to the softmax's (independent chains); the q-dot follows the transposed reads
      const S1Rot rot1 = stage1_rotate(in1, IC<u & 1>());
      if (!SCORES && pv_live) stage23(t_pv, in23, IC<u % 3>(), IC<(u + 1) & 1>(), steady_c);
      issue_rows(pp + 2, IC<(u + 2) % 3>(), steady_c, IC<LC1>(), IC<LC2>());
      XKV_FENCE();
      // The compiler does not know of the transposed reads: a wait it placed after them for LDS data it read earlier would
      // wait for them too.  Using that data here makes it wait now, and the q-dot below overlaps the transposed reads.
      asm volatile("" ::"v"(in1.q[0]), "v"(in1.q[1]), "v"(rot1.kop[0]), "v"(rot1.kop[1]));
      if (!SCORES) trread(IC<u % 3>(), IC<u % 3>());
      issue_rows(pp + 2, IC<(u + 2) % 3>(), steady_c, IC<LC2>(), IC<LC3>());
      XKV_FENCE();
      stage1_dot(rot1, in1, IC<u & 1>());
      issue_rows(pp + 2, IC<(u + 2) % 3>(), steady_c, IC<LC3>(), IC<8>());
      XKV_FENCE();
      if ((u & 1) == 0 && pp >= 2) write_qhat(pp);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the transposed reads
      wait_vmcnt<8 - NLR>();      // this wave's rows of tile pp+1 have landed; its loads of tile pp+2 may be in flight
      // Scores mode stores to memory, and stores count in vmcnt like loads: they are issued after the wait, so that they have
      // a whole period to complete before the next one (which cannot tell them from the loads it waits for)
      if (SCORES && pv_live) stage23(t_pv, in23, IC<u % 3>(), IC<(u + 1) & 1>(), steady_c);
    }
    __syncthreads();
  };
  for (int pb = 0; pb < NP6; pb += 6) {
    if (pb > 0 && pb % 30 == 0) seed_qhat(pb);   // period pb writes q^ of tile pb next
    if (pb >= 6 && pb + 7 < nfull) {
      period(pb, IC<0>(), IC<1>()); period(pb + 1, IC<1>(), IC<1>()); period(pb + 2, IC<2>(), IC<1>());
      period(pb + 3, IC<3>(), IC<1>()); period(pb + 4, IC<4>(), IC<1>()); period(pb + 5, IC<5>(), IC<1>());
    } else {
      period(pb, IC<0>(), IC<0>()); period(pb + 1, IC<1>(), IC<0>()); period(pb + 2, IC<2>(), IC<0>());
      period(pb + 3, IC<3>(), IC<0>()); period(pb + 4, IC<4>(), IC<0>()); period(pb + 5, IC<5>(), IC<0>());
    }
  }
  wait_vmcnt<0>();
  if (SCORES) return;

  // ---- epilogue: every consumer holds every head's (reference, row sum); it normalises and writes its RK / 4 features ---------
  float l_head = l_run;
#pragma unroll
  for (int m = GP; m < 64; m <<= 1) l_head += __shfl_xor(l_head, m);
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  f32x4 acc[NMB];
  static_for<4 * NMB>([&](auto r_c) { constexpr int r = decltype(r_c)::value; acc[r >> 2][r & 3] = acc_get_at<r>(); });
  if (n16 < G) {
    const float inv = 1.f / l_head;
    const int64_t ph = ((int64_t)b * p.hq + h0 + n16) * p.max_splits + split;
    float* dst = p.partial + ph * RK + c * (RK / 4) + 4 * g4;
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) *reinterpret_cast<f32x4*>(dst + mb * 16) = acc[mb] * inv;
    if (c == 0 && g4 == 0) p.lse[ph] = m_ref * 0.6931471805599453f + __logf(l_head);
  }
}

template <typename T, int RK>
int launch_recon_spec_t(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, hipStream_t st) {
  typedef SpecShape<RK> S;
  const int nb = sBb == 0 ? 1 : batch;   // one packed copy when the factor is shared by the batch
  pack_b_kernel<T, RK><<<dim3(p.hkv, nb, 32), dim3(256), 0, st>>>((const T*)kB, (T*)p.Bp, sBb, sBh, sBr, p.hkv);
  const bool gp4 = p.hq / p.hkv <= 4;
  auto kern = p.scores ? (gp4 ? recon_spec_kernel<T, true, RK, 4> : recon_spec_kernel<T, true, RK, 8>)
                       : (gp4 ? recon_spec_kernel<T, false, RK, 4> : recon_spec_kernel<T, false, RK, 8>);
  static DynLds lds[4];
  const int e = ensure_dynamic_lds(lds[(p.scores ? 2 : 0) + (gp4 ? 1 : 0)], reinterpret_cast<const void*>(kern), (int)S::SHM, true);
  if (e != XKV_OK) return e;
  const int total = batch * p.hkv * p.max_splits;
  kern<<<dim3(xcd_grid(total, p.hkv)), dim3(512), S::SHM, st>>>(p);
  return launch_status();
}

template <int RK>
int launch_recon_spec_rank(const FastParams& p, const void* kB, int64_t sBb, int64_t sBh, int64_t sBr, int batch, int dtype,
                           hipStream_t st) {
  return dtype == XKV_BF16 ? launch_recon_spec_t<__bf16, RK>(p, kB, sBb, sBh, sBr, batch, st)
                           : launch_recon_spec_t<_Float16, RK>(p, kB, sBb, sBh, sBr, batch, st);
}

}  // namespace spec
}  // namespace xkv
