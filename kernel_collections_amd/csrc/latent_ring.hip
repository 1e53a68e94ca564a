// Split-K flash-decoding stage 1 for WIDE latent rows (256 .. 1024 features, optionally + 64 RoPE features):
// the bandwidth-bound scans of the path (absorbed no-PE xKV scores and decode, MLA over c_kv | k_pe, V-only
// factorised decode with the per-head keys viewed as one 1024-wide row against a block-diagonal query).
//
// Same arithmetic as latent_stage1.hip; what differs is how bytes move.  A CU has to keep roughly
// (HBM latency x its share of the HBM rate) = 60-100 KB of loads in flight to stream at full rate.  Here four extra
// wavefronts do nothing but move token rows: plain 16-byte vector loads into a register queue of RING_QD tiles per wave
// (that queue is what is in flight), then ds_write_b128 into a two-slot ring of TN-token tiles in the LDS.  A load
// instruction that stalls on a full memory queue then never holds up the arithmetic; the loader waves take part in the
// same barriers.  One workgroup per CU; the query operands live in registers for the whole kernel.  Per tile t:
//   A:  barrier (slot of tile t-1 is free); loaders wait for tile t+1 only, write it into that slot, refill the queue entry
//   QK: wave (tb, kh) multiplies token block tb by its k-range kh of q on v_mfma_f32_16x16x32 -> partial scores in LDS
//   B:  barrier; softmax threads add the k-range partials, update the running max / sum, publish P and alpha
//   C:  barrier; PV: each wave owns a quarter of the value features, token-major operand via ds_read_b64_tr_b16.
// Scores-only mode (qAB without PE) stops after B and writes the summed scores.
// The start of the kernel is latency, not bandwidth: the loader branch comes first in the code and addresses its rows
// with scalar arithmetic so that the first loads leave as early as possible.
//
// LDS tile layout: C (and V) rows are row-major with a 16-byte pad (conflict-free ds_read_b128 over 16 rows and
// conflict-free transposed reads); the 128-byte RoPE-key rows are stored chunk-major ([8 chunks][TN rows][16 B]):
// lane l of loader wave w fetches chunk 2w + l/32 of row l%32 and writes it at l * 16 of that wave's 1 KiB piece.
#include "xkv_common.h"
#include "latent_ring.h"

namespace xkv {

typedef short s16x4r __attribute__((ext_vector_type(4)));
typedef short s16x8r __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4r __attribute__((ext_vector_type(4)));

// Streaming 16-byte load the compiler does not track: the register queue of the loader waves is drained with explicit
// vmcnt waits (the compiler's own counting gives up at the loop back edge and would drain the whole queue per tile).
// The value must pass through ring_landed() after the wait and before its first use.  A wave that uses these must not
// issue any other vector-memory load.
__device__ __forceinline__ u32x4 ring_ldg(const void* p) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(v) : "v"(p));
  return v;
}
// the same with a wave-uniform base in SGPRs and a 32-bit per-lane offset: the row addresses then cost SALU work only
template <int OFF> __device__ __forceinline__ u32x4 ring_ldg_s(const void* sbase, unsigned voff) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3 nt" : "=v"(v) : "v"(voff), "s"(sbase), "n"(OFF));
  return v;
}
__device__ __forceinline__ void ring_landed(u32x4& v) { asm volatile("" : "+v"(v)); }
template <int N> __device__ __forceinline__ void ring_wait() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

__device__ __forceinline__ s16x4r ring_tr4(const unsigned char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4r*)p);
}

// 16-token contraction (tiles of 16 tokens): A = 4 tokens of one feature per lane, B = 4 tokens of one head per lane
__device__ __forceinline__ f32x4 mfma16k16(__bf16, s16x4r a, s16x4r b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma16k16(_Float16, s16x4r a, s16x4r b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4r, a), __builtin_bit_cast(f16x4r, b), c, 0, 0, 0);
}

constexpr int RING_QD = 2;      // tiles per loader wave in flight in registers (deeper queues only lengthen the start); >= 2
enum { RING_SCORES = 0, RING_VSHARED = 1, RING_VDISTINCT = 2, RING_VHEADS = 3, RING_VGIVEN = 4 };
constexpr int RING_DVH = 128;   // head width of the per-head value rows (RING_VHEADS)

template <int TN, int DN, bool HAS_R, int VMODE, int NHB, int DVW>
struct RingShape {
  static constexpr int HB = 16 * NHB;
  static constexpr int CROW = DN * 2 + 16;                 // padded C row (bytes)
  static constexpr int CBYTES = TN * CROW;
  static constexpr int RBYTES = (HAS_R || VMODE == RING_VGIVEN) ? TN * 128 : 0;   // RoPE-key chunks, or a tile of given scores
  static constexpr int VROW = DVW * 2 + 16;                // padded V row (distinct-V mode)
  static constexpr int VBYTES = (VMODE == RING_VDISTINCT || VMODE == RING_VHEADS) ? TN * VROW : 0;
  static constexpr int SLOT = CBYTES + RBYTES + VBYTES;
  static constexpr int KSPLIT = 4 / (TN / 16);             // k-ranges (waves per 16-token block)
  static constexpr int SP = TN + 4;                        // partial-score row stride (floats)
  static constexpr int LDP = TN + 8;                       // P row stride (elements)
  static constexpr int TAIL = KSPLIT * HB * SP * 4 + HB * LDP * 2 + HB * 4 + HB * 8;
  static constexpr int RSLOT = 2;                          // the tile being read and the tile being written
  static constexpr int SHM = RSLOT * SLOT + TAIL;
  // staging area of the query rows (no-PE features | RoPE features | pad; a second set for the low-order part); used when
  // it fits beside the ring
  static constexpr int QSTRIDE = (DN + (HAS_R ? 64 : 0)) * 2 + 16;
  static constexpr int qst_bytes(bool lo) { return HB * QSTRIDE * (lo ? 2 : 1); }
  // (not for the 1024-wide form: its query arrives as compact 128-wide rows and is expanded in registers)
  static constexpr bool qst(bool lo) { return DN != 1024 && VMODE != RING_VGIVEN && SHM + qst_bytes(lo) <= 160 * 1024; }
  static constexpr int shm(bool lo) { return SHM + (qst(lo) ? qst_bytes(lo) : 0); }
  static_assert(SHM <= 160 * 1024, "ring does not fit the LDS");
};

// T: operand type; TN: tokens per tile (32, or 16 when two row streams share the LDS); NHB: 16-row head blocks; LO: q has
// a low-order part; DN: latent width; HAS_R: 64 RoPE features follow (TN 32 only); VMODE: scores only / V is the first
// DN features of the C row / V is a second, DVW-wide row stream / V is a second stream of DVW / 128 per-kv-head value
// rows of 128 features (plain values under absorbed factorised keys): the workgroup serves every query head, wave w
// accumulates kv heads 2w, 2w+1, and query head h multiplies the values of kv head h / (heads per kv head).
// RING_VGIVEN: no query at all - the scaled scores [b, hq, kv_len] (fp32) are an input, the C rows are the values: softmax
// and P.V over a value basis of its own, behind a kernel that produced the scores (two-pass fused decode).
// DN 1024 means eight plain kv heads of 128 side by side in a token row, against compact query rows [b, hq, 128].
template <typename T, int TN, int NHB, bool LO, int DN, bool HAS_R, int VMODE, int DVW>
__global__ __launch_bounds__(512) void latent_ring_kernel(const RingParams p) {
  static_assert(DN != 1024 || (!LO && !HAS_R), "the 1024-wide form is plain per-head keys");
  typedef typename Elem<T>::vec8 vec8;
  typedef RingShape<TN, DN, HAS_R, VMODE, NHB, DVW> S;
  constexpr bool SCORES = VMODE == RING_SCORES, V2 = VMODE == RING_VDISTINCT || VMODE == RING_VHEADS, VHEADS = VMODE == RING_VHEADS;
  constexpr bool GIVEN = VMODE == RING_VGIVEN;
  static_assert(!GIVEN || (!LO && !HAS_R && TN == 32), "given scores: plain 32-token tiles of value rows");
  constexpr int VIPR = DVW > 512 ? DVW / 512 : 1;   // load instructions per V row
  constexpr int KVH = DVW / RING_DVH, KVW = VHEADS ? KVH / 4 : 1;   // kv heads of a value row, per wave
  constexpr int HB = S::HB, CROW = S::CROW, CBYTES = S::CBYTES, VROW = S::VROW, SLOT = S::SLOT, RSLOT = S::RSLOT;
  constexpr int NTB = TN / 16, KSPLIT = S::KSPLIT, SP = S::SP, LDP = S::LDP;
  constexpr int NKS_N = DN / 32, NKS = NKS_N + (HAS_R ? 2 : 0);
  constexpr int KS_W = NKS / KSPLIT;              // k-steps per wave
  static_assert(NKS % KSPLIT == 0, "the k-ranges are equal");
  static_assert(!HAS_R || TN == 32, "RoPE-key rows need 32-token tiles");
  static_assert(DN <= 1024 && DVW <= 1024, "a row takes at most two load instructions");
  constexpr int IPR = DN > 512 ? DN / 512 : 1;    // load instructions per C row (1 KiB each; rows under 1 KiB use DN/8 lanes)
  constexpr bool CPART = DN < 512;               // a C row fills only part of a load instruction
  // waves 4..7 move the tile rows; each brings TN/4 rows of C (and V) and two 16-byte chunks of every RoPE-key row
  constexpr int QD = RING_QD;
  constexpr int RPW = TN / 4;                     // rows per loader wave per tile
  constexpr int LPT = RPW * IPR + ((HAS_R || GIVEN) ? 1 : 0) + (V2 ? RPW * VIPR : 0);   // loads per loader wave per tile
  static_assert((QD - 1) * LPT <= 63, "vmcnt holds 6 bits");
  constexpr int DV = (VMODE == RING_VSHARED || GIVEN) ? DN : VHEADS ? RING_DVH : DVW;   // value features of an output row
  constexpr int NVB = VHEADS ? RING_DVH / 16 : DV / 64;   // 16-feature blocks per wave (per kv head under VHEADS)
  constexpr int NA2 = VHEADS ? KVW : NHB;
  static_assert(!VHEADS || (TN == 16 && KVH % 4 == 0), "per-head values: 16-token tiles, kv heads split over 4 waves");
  constexpr int TPH = 256 / HB, TPT = TN / TPH;   // softmax threads per head row, tokens per thread
  static_assert(TPT >= 1, "tile too short for the softmax thread map");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n16 = lane & 15, g4 = lane >> 4;
  const int tb = wave % NTB, kh = wave / NTB;
  const int iw = wave - 4;                        // index among the loader waves (negative: a compute wave)

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
  const int hg = p.hq / p.groups, h0 = group * hg;
  const int ntiles = (end - start + TN - 1) / TN;
  const int last = end - 1;

  // ---- LDS carve-up -------------------------------------------------------------------------------------------
  unsigned char* ring = smem;
  float* s_part = reinterpret_cast<float*>(smem + RSLOT * SLOT);   // [KSPLIT][HB][SP]
  T* p_lds = reinterpret_cast<T*>(s_part + KSPLIT * HB * SP);      // [HB][LDP]
  float* alpha_lds = reinterpret_cast<float*>(p_lds + HB * LDP);   // [HB]
  float* ml_lds = alpha_lds + HB;                                  // [HB][2]

  // ---- tile loads: wave w brings rows RPW w .. +RPW of C (and V) and RoPE-key chunks 2w, 2w+1 of every row ---------
  const unsigned char* Cb = reinterpret_cast<const unsigned char*>(p.C) + (b * p.sCb + group * p.sCh) * 2;
  const unsigned char* Rb = HAS_R ? reinterpret_cast<const unsigned char*>(p.R) + (b * p.sRb + group * p.sRh) * 2 : nullptr;
  const unsigned char* Vb =
      V2 ? reinterpret_cast<const unsigned char*>(p.V) + (b * p.sVb + (VHEADS ? 0 : group * p.sVh)) * 2 : nullptr;
  const int64_t crow_bytes = p.sCl * 2, rrow_bytes = p.sRl * 2, vrow_bytes = p.sVl * 2;
  const unsigned lane_off = lane * 16;
  const int r_row = lane & 31;
  if (__builtin_expect(wave >= 4, 1)) {   // laid out first: the sooner the first loads are issued, the shorter the start
    u32x4 rq[QD][LPT];
    auto fetch = [&](int t, u32x4 (&q)[LPT]) {
      const int base = start + t * TN;
      int n = 0;
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
        int tok = base + iw * RPW + r;
        tok = tok < last ? tok : last;   // rows past the split end are masked in the softmax; keep the read in bounds
        const unsigned char* row = Cb + (int64_t)tok * crow_bytes;   // wave-uniform
        if (!CPART || lane < DN / 8) {
          q[n] = ring_ldg_s<0>(row, lane_off);
          if (IPR > 1) q[n + 1] = ring_ldg_s<1024>(row, lane_off);
        }
        n += IPR;
        if (V2) {
          const unsigned char* vrow = Vb + (int64_t)tok * vrow_bytes;
          if (DVW >= 512 || lane < DVW / 8) {
            q[n] = ring_ldg_s<0>(vrow, lane_off);
            if (VIPR > 1) q[n + 1] = ring_ldg_s<1024>(vrow, lane_off);
          }
          n += VIPR;
        }
      }
      if (HAS_R) {                       // this wave brings chunks 2 iw, 2 iw + 1 of every row
        int tok = base + r_row;
        tok = tok < last ? tok : last;
        q[n] = ring_ldg(Rb + (int64_t)tok * rrow_bytes + (2 * iw + (lane >> 5)) * 16);
      }
      if (GIVEN) {                       // given scores: head rows 8 iw .. +8 of the tile, 128 bytes (32 tokens) each
        int row = 8 * iw + (lane >> 3);
        row = row < hg ? row : hg - 1;
        int tok = base + 4 * (lane & 7);
        tok = tok + 4 <= p.kv_len ? tok : p.kv_len - 4;   // pieces past the buffer's row end: any in-bounds piece (masked later)
        q[n] = ring_ldg(reinterpret_cast<const float*>(p.scores) + ((int64_t)b * p.hq + h0 + row) * p.kv_len + tok);
      }
    };
    auto hand_on = [&](int t, u32x4 (&q)[LPT]) {   // the oldest tile of the queue: QD-1 younger ones stay in flight
      unsigned char* slot = ring + (t % RSLOT) * SLOT + lane_off;
      ring_wait<(QD - 1) * LPT>();
#pragma unroll
      for (int i = 0; i < LPT; ++i) ring_landed(q[i]);
      int n = 0;
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
#pragma unroll
        for (int c = 0; c < IPR; ++c, ++n)
          if (!CPART || lane < DN / 8) st16(slot + (iw * RPW + r) * CROW + c * 1024, q[n]);
        if (V2) {
#pragma unroll
          for (int c = 0; c < VIPR; ++c, ++n)
            if (DVW >= 512 || lane < DVW / 8) st16(slot + CBYTES + S::RBYTES + (iw * RPW + r) * VROW + c * 1024, q[n]);
        }
      }
      if (HAS_R || GIVEN) st16(slot + CBYTES + iw * 1024, q[n]);   // scores: [32 head rows][32 tokens] fp32, row-major
    };
    // Iteration j: tile j - QD leaves the queue for the ring (its slot was released by barrier A of the tile before it) and
    // tile j enters the queue in its place, so the look-ahead lives in the queue and a tile is waited for only when the
    // next iteration needs it.  Every queue entry is loaded at one place in the code and stored at one place: the loads
    // are invisible to the compiler, and a register copy between two such places would read a value that has not landed.
    // Tiles past the end are fetched too (clamped rows, never used): the vmcnt arithmetic counts on QD - 1 younger tiles.
    for (int j0 = 0; j0 <= ntiles + QD; j0 += QD) {   // j0 stays a multiple of QD, so the queue index below is static
#pragma unroll
      for (int u = 0; u < QD; ++u) {
        const int j = j0 + u, k = j - QD;
        if (j <= ntiles + QD) {
          if (k >= 1) __syncthreads();                 // A of tile k-1: the slot of tile k-2 is free
          if (k >= 0) hand_on(k, rq[u]);
          fetch(j, rq[u]);
          if (j == 0) {
            __syncthreads();                           // start: the compute waves hold their query loads back until here
          }
          if (j == 1 && S::qst(LO)) __syncthreads();   // the compute waves' barrier between staging the query rows and reading them
          if (k >= 1) {
            if (!GIVEN) __syncthreads();               // B of tile k-1 (given scores: there is no QK phase to wait for)
            if (!SCORES) __syncthreads();              // C of tile k-1
          }
        }
      }
    }
    return;
  }

  // The query loads of a workgroup are a burst several tiles long, and the CU serves its memory instructions in order: let
  // the loaders put the first tiles ahead of it (they arrive at this barrier once those loads are issued).
  __syncthreads();
  // ---- query operands in registers: lane (n16 = head row, g4) holds q[head][32 ks + 8 g4 .. +8] for its k-range ----
  vec8 qreg[KS_W][NHB], qlo[LO ? KS_W : 1][NHB];
  const int ks0 = kh * KS_W;
  if constexpr (GIVEN) {
    // no query operands
  } else if constexpr (S::qst(LO)) {
    // Whole rows, coalesced, each read once per workgroup, into the LDS; every lane then picks its operand pieces from there.
    // (Read straight into the operand layout, a load instruction touches 16 half-used cache lines and two waves fetch
    // the same rows: several microseconds at the start of a kernel that lasts tens.)
    constexpr int QSTRIDE = S::QSTRIDE, RQ = HB / 4;   // wave w stages head rows RQ w .. +RQ
    unsigned char* qst = smem + S::SHM;
    u32x4 tmp[RQ * IPR * (LO ? 2 : 1) + (HAS_R ? 1 : 0)];
    int n = 0;
#pragma unroll
    for (int r = 0; r < RQ; ++r) {
      int row = wave * RQ + r;
      row = row < hg ? row : hg - 1;   // head rows past the group repeat its last row: finite values that are never written out
      const int64_t qoff = ((int64_t)b * p.hq + h0 + row) * (DN * 2) + lane_off;
#pragma unroll
      for (int c = 0; c < IPR; ++c) {
        if (!CPART || lane < DN / 8) {
          tmp[n] = ld16<u32x4>(reinterpret_cast<const unsigned char*>(p.qn) + qoff + c * 1024);
          if (LO) tmp[n + 1] = ld16<u32x4>(reinterpret_cast<const unsigned char*>(p.qn_lo) + qoff + c * 1024);
        }
        n += LO ? 2 : 1;
      }
    }
    if (HAS_R && (lane >> 3) < RQ) {   // 128-byte RoPE rows: eight lanes each
      int row = wave * RQ + (lane >> 3);
      row = row < hg ? row : hg - 1;
      tmp[n] = ld16<u32x4>(reinterpret_cast<const unsigned char*>(p.qr) + ((int64_t)b * p.hq + h0 + row) * 128 + (lane & 7) * 16);
    }
    n = 0;
#pragma unroll
    for (int r = 0; r < RQ; ++r) {
      unsigned char* dst = qst + (wave * RQ + r) * QSTRIDE + lane_off;
#pragma unroll
      for (int c = 0; c < IPR; ++c) {
        if (!CPART || lane < DN / 8) {
          st16(dst + c * 1024, tmp[n]);
          if (LO) st16(dst + HB * QSTRIDE + c * 1024, tmp[n + 1]);
        }
        n += LO ? 2 : 1;
      }
    }
    if (HAS_R && (lane >> 3) < RQ) st16(qst + (wave * RQ + (lane >> 3)) * QSTRIDE + DN * 2 + (lane & 7) * 16, tmp[n]);
    __syncthreads();
#pragma unroll
    for (int hb = 0; hb < NHB; ++hb) {
      const unsigned char* src = qst + (hb * 16 + n16) * QSTRIDE + ks0 * 64 + g4 * 16;
#pragma unroll
      for (int k = 0; k < KS_W; ++k) {
        qreg[k][hb] = ld16<vec8>(src + k * 64);
        if (LO) qlo[k][hb] = ld16<vec8>(src + HB * QSTRIDE + k * 64);
      }
    }
  } else if constexpr (DN == 1024) {
    // Eight kv heads of 128 side by side in a token row: the query is block-diagonal and comes as its compact rows
    // [b, hq, 128]; head row r multiplies only k-steps 4 kvh .. 4 kvh + 3 of its kv head kvh = r / (heads per kv head).
    const int hpq = hg / 8;
#pragma unroll
    for (int hb = 0; hb < NHB; ++hb) {
      int row = hb * 16 + n16;
      row = row < hg ? row : hg - 1;
      const int kvh = row / hpq;
      const T* ql = reinterpret_cast<const T*>(p.qn) + ((int64_t)b * p.hq + h0 + row) * 128 + 8 * g4;
#pragma unroll
      for (int k = 0; k < KS_W; ++k) {
        const int ks = ks0 + k;
        vec8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if ((ks >> 2) == kvh) v = ld16<vec8>(ql + (ks & 3) * 32);
        qreg[k][hb] = v;
      }
    }
  } else {
#pragma unroll
    for (int hb = 0; hb < NHB; ++hb) {
      int row = hb * 16 + n16;
      row = row < hg ? row : hg - 1;
      const int64_t qh = (int64_t)b * p.hq + h0 + row;
      const T* qn_l = reinterpret_cast<const T*>(p.qn) + qh * DN + ks0 * 32 + 8 * g4;
      const T* ql_l = LO ? reinterpret_cast<const T*>(p.qn_lo) + qh * DN + ks0 * 32 + 8 * g4 : nullptr;
      const T* qr_l = HAS_R ? reinterpret_cast<const T*>(p.qr) + qh * 64 + (ks0 - NKS_N) * 32 + 8 * g4 : nullptr;
#pragma unroll
      for (int k = 0; k < KS_W; ++k) {
        if (!HAS_R || ks0 + k < NKS_N) {
          qreg[k][hb] = ld16<vec8>(qn_l + k * 32);
          if (LO) qlo[k][hb] = ld16<vec8>(ql_l + k * 32);
        } else {
          qreg[k][hb] = ld16<vec8>(qr_l + k * 32);
        }
      }
    }
  }
  // Wait for the query loads here, once, rather than at their first uses inside the loop.
  if constexpr (!GIVEN) {
#pragma unroll
    for (int k = 0; k < KS_W; ++k)
#pragma unroll
      for (int hb = 0; hb < NHB; ++hb) {
        asm volatile("" : "+v"(qreg[k][hb]));
        if (LO) asm volatile("" : "+v"(qlo[k][hb]));
      }
  }

  // ---- running state ---------------------------------------------------------------------------------------------
  const int srow = tid / TPH, ssub = tid % TPH;
  float m_run = NEG_INF, l_run = 0.f;
  f32x4 acc[SCORES ? 1 : NVB][NA2];
#pragma unroll
  for (int mb = 0; mb < (SCORES ? 1 : NVB); ++mb)
#pragma unroll
    for (int hb = 0; hb < NA2; ++hb) acc[mb][hb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int hpk = VHEADS ? hg / KVH : 0;   // query heads per kv head
  const int vcol0 = wave * (DV / 4);

  for (int t = 0; t < ntiles; ++t) {
    __syncthreads();                  // A: tile t is in its slot; every wave is past PV / score write of tile t-1
    const unsigned char* slot = ring + (t % RSLOT) * SLOT;
    const int base = start + t * TN;

    // ---- QK: partial scores of token block tb over this wave's k-range -------------------------------------------
    if constexpr (GIVEN) {               // the scores are an input: the loader waves put the tile's beside its value rows
    } else {
      f32x4 sacc[NHB];
#pragma unroll
      for (int hb = 0; hb < NHB; ++hb) sacc[hb] = f32x4{0.f, 0.f, 0.f, 0.f};
      const unsigned char* arow = slot + (tb * 16 + n16) * CROW + g4 * 16;
      const unsigned char* rrow = slot + CBYTES + (g4 * TN + tb * 16 + n16) * 16;
#pragma unroll
      for (int k = 0; k < KS_W; ++k) {
        const int ks = ks0 + k;
        const unsigned char* ap = (!HAS_R || ks < NKS_N) ? arow + ks * 64 : rrow + (ks - NKS_N) * (4 * TN * 16);
        const vec8 a = ld16<vec8>(ap);
#pragma unroll
        for (int hb = 0; hb < NHB; ++hb) {
          sacc[hb] = Elem<T>::mfma16(a, qreg[k][hb], sacc[hb]);
          if (LO) sacc[hb] = Elem<T>::mfma16(a, qlo[k][hb], sacc[hb]);
        }
      }
      // lane (n16 = head row, g4): tokens tb*16 + 4 g4 + r
#pragma unroll
      for (int hb = 0; hb < NHB; ++hb)
        *reinterpret_cast<f32x4*>(s_part + (kh * HB + hb * 16 + n16) * SP + tb * 16 + 4 * g4) = sacc[hb];
    }
    if (!GIVEN) __syncthreads();      // B: the k-range partials of every head row are visible

    if (SCORES) {
      // thread -> 4 tokens (16 bytes) of a head row, TN/4 consecutive lanes per row: every store instruction writes whole
      // 128-byte (TN 32) pieces of score rows; rows beyond the first 256 / (TN/4) come in a second pass
      constexpr int LPR = TN / 4, RPP = 256 / LPR;
      const int c0 = (tid % LPR) * 4;
#pragma unroll
      for (int row = tid / LPR; row < HB; row += RPP) {
        if (row < hg) {
          const int64_t o = ((int64_t)b * p.hq + h0 + row) * p.kv_len + base + c0;
          f32x4 a = *reinterpret_cast<const f32x4*>(s_part + row * SP + c0);
#pragma unroll
          for (int kr = 1; kr < KSPLIT; ++kr) a += *reinterpret_cast<const f32x4*>(s_part + (kr * HB + row) * SP + c0);
          a *= p.sm_scale;
          if (p.logit_cap > 0.f) {
#pragma unroll
            for (int j = 0; j < 4; ++j) a[j] = p.logit_cap * tanhf(a[j] / p.logit_cap);
          }
          if (p.scores_dtype == XKV_F32 && (p.kv_len & 3) == 0 && base + c0 + 4 <= end) {
            *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p.scores) + o) = a;
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if (base + c0 + j < end) {
                if (p.scores_dtype == XKV_F32) reinterpret_cast<float*>(p.scores)[o + j] = a[j];
                else reinterpret_cast<T*>(p.scores)[o + j] = from_f32<T>(a[j]);
              }
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
        float s = 0.f;
        if constexpr (GIVEN) {
          s = reinterpret_cast<const float*>(slot + CBYTES)[srow * TN + c];
        } else {
#pragma unroll
          for (int kr = 0; kr < KSPLIT; ++kr) s += s_part[(kr * HB + srow) * SP + c];
        }
        s *= p.sm_scale;
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
        p_lds[srow * LDP + ssub * TPT + i] = from_f32<T>(e);
      }
      sum = row_reduce<false, TPH>(sum);
      l_run = l_run * alpha + sum;
      m_run = m_new;
      if (ssub == 0) alpha_lds[srow] = alpha;
    }
    __syncthreads();                  // C: P and alpha of tile t are visible

    // ---- PV: acc^T[feature, head] += V^T P^T, this wave's quarter of the value features -----------------------------
    if (VHEADS) {
      // per kv head j of this wave: acc^T[feature, query head of j] += V_j^T P^T; column n16 of the P operand is query
      // head hpk * j + n16 (columns past the heads of j repeat the last row and are never written out)
      const unsigned char* vbase = slot + CBYTES + S::RBYTES;
#pragma unroll
      for (int j = 0; j < KVW; ++j) {
        const int kvh = wave * KVW + j;
        int prow = hpk * kvh + n16;
        prow = prow < HB - 1 ? prow : HB - 1;
        const float al = alpha_lds[prow];
        const s16x4r pb = *reinterpret_cast<const s16x4r*>(p_lds + prow * LDP + 4 * g4);
        const unsigned char* vrow = vbase + (4 * g4 + (n16 >> 2)) * VROW + (kvh * RING_DVH + 4 * (n16 & 3)) * 2;
#pragma unroll
        for (int mb = 0; mb < NVB; ++mb) acc[mb][j] = mfma16k16(T(), ring_tr4(vrow + mb * 32), pb, acc[mb][j] * al);
      }
    } else {
      constexpr int VR = VMODE == RING_VDISTINCT ? VROW : CROW;
      const unsigned char* vbase = slot + (VMODE == RING_VDISTINCT ? CBYTES + S::RBYTES : 0);
      float al[NHB];
#pragma unroll
      for (int hb = 0; hb < NHB; ++hb) al[hb] = alpha_lds[hb * 16 + n16];
      if (TN == 32) {
        vec8 pb[NHB];
#pragma unroll
        for (int hb = 0; hb < NHB; ++hb) pb[hb] = ld16<vec8>(p_lds + (hb * 16 + n16) * LDP + 8 * g4);
        const unsigned char* vrow = vbase + (8 * g4 + (n16 >> 2)) * VR + (vcol0 + 4 * (n16 & 3)) * 2;
#pragma unroll
        for (int mb = 0; mb < NVB; ++mb) {
          const s16x8r a8 = __builtin_shufflevector(ring_tr4(vrow + mb * 32), ring_tr4(vrow + mb * 32 + 4 * VR), 0, 1, 2, 3, 4, 5, 6, 7);
          const vec8 a = __builtin_bit_cast(vec8, a8);
#pragma unroll
          for (int hb = 0; hb < NHB; ++hb) acc[mb][hb] = Elem<T>::mfma16(a, pb[hb], acc[mb][hb] * al[hb]);
        }
      } else {
        s16x4r pb[NHB];
#pragma unroll
        for (int hb = 0; hb < NHB; ++hb) pb[hb] = *reinterpret_cast<const s16x4r*>(p_lds + (hb * 16 + n16) * LDP + 4 * g4);
        const unsigned char* vrow = vbase + (4 * g4 + (n16 >> 2)) * VR + (vcol0 + 4 * (n16 & 3)) * 2;
#pragma unroll
        for (int mb = 0; mb < NVB; ++mb) {
          const s16x4r a = ring_tr4(vrow + mb * 32);
#pragma unroll
          for (int hb = 0; hb < NHB; ++hb) acc[mb][hb] = mfma16k16(T(), a, pb[hb], acc[mb][hb] * al[hb]);
        }
      }
    }
  }
  if (SCORES) return;

  // ---- epilogue: normalise, write partial + lse --------------------------------------------------------------------
  if (ssub == 0) { ml_lds[2 * srow] = m_run; ml_lds[2 * srow + 1] = l_run; }
  __syncthreads();
  if (VHEADS) {
#pragma unroll
    for (int j = 0; j < KVW; ++j) {
      const int hrow = hpk * (wave * KVW + j) + n16;
      if (n16 < hpk) {
        const float m = ml_lds[2 * hrow], l = ml_lds[2 * hrow + 1];
        const float inv = 1.f / l;
        const int64_t ph = ((int64_t)b * p.hq + hrow) * p.max_splits + split;
        float* dst = p.partial + ph * RING_DVH + 4 * g4;
#pragma unroll
        for (int mb = 0; mb < NVB; ++mb) *reinterpret_cast<f32x4*>(dst + mb * 16) = acc[mb][j] * inv;
        if (g4 == 0) p.lse[ph] = m + __logf(l);
      }
    }
    return;
  }
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

template <typename T, int TN, int NHB, bool LO, int DN, bool HAS_R, int VMODE, int DVW = 512>
static int launch_ring_t(const RingParams& p, int batch, hipStream_t st) {
  constexpr int SHM = RingShape<TN, DN, HAS_R, VMODE, NHB, DVW>::shm(LO);
  auto kern = latent_ring_kernel<T, TN, NHB, LO, DN, HAS_R, VMODE, DVW>;
  static DynLds lds;
  const int e = ensure_dynamic_lds(lds, reinterpret_cast<const void*>(kern), SHM, true);
  if (e != XKV_OK) return e;
  const int total = batch * p.groups * p.max_splits;
  kern<<<dim3(xcd_grid(total, p.groups)), dim3(512), SHM, st>>>(p);
  return launch_status();
}

// which instantiation serves a call; -1: none (the register-staged kernel runs instead)
// plain per-kv-head values [token][8 heads][128] under one shared, absorbed key basis: the call's kv groups all scan the
// same C rows, so one workgroup per (sequence, split) serves every head
// - or plain per-head keys too, viewed as one 1024-wide row against a block-diagonal query (no low-order part)
static bool ring_vheads(const RingParams& p, bool vshared) {
  const bool absorbed = p.qn_lo && (p.dn == 512 || p.dn == 384 || p.dn == 256);
  const bool plain_keys = !p.qn_lo && p.dn == 1024 && p.heads_in_row == 8;
  return !p.scores && !vshared && p.groups * RING_DVH == 1024 && p.dv == RING_DVH && p.sVh == RING_DVH && p.sCh == 0 &&
         (absorbed || plain_keys) && !p.R && p.hq <= 32 && p.hq % p.groups == 0 && p.sCl >= p.dn && p.sVl >= 1024;
}

static int ring_vmode(const RingParams& p, bool vshared) {
  if (p.scores) return RING_SCORES;
  if (ring_vheads(p, vshared)) return RING_VHEADS;
  if (vshared && p.dv == p.dn && (p.dn == 512 || p.dn == 384 || p.dn == 256)) return RING_VSHARED;
  if (!vshared && (p.dv == 512 || p.dv == 384 || p.dv == 256)) return RING_VDISTINCT;
  return -1;
}

// softmax + P.V over given scores: the value rows are the C stream
template <typename T>
static int launch_ring_given_dt(const RingParams& p, int batch, hipStream_t st) {
  const int nhb = p.hq <= 16 ? 1 : 2;
#define XKV_RING_GIVEN(NHB, DN) \
  if (nhb == NHB && p.dn == DN) return launch_ring_t<T, 32, NHB, false, DN, false, RING_VGIVEN>(p, batch, st);
  XKV_RING_GIVEN(1, 512) XKV_RING_GIVEN(2, 512) XKV_RING_GIVEN(1, 384) XKV_RING_GIVEN(2, 384) XKV_RING_GIVEN(1, 256) XKV_RING_GIVEN(2, 256)
#undef XKV_RING_GIVEN
  return XKV_EUNSUPPORTED;
}

template <typename T>
static int launch_ring_dt(const RingParams& p, int batch, bool vshared, hipStream_t st) {
  const int hg = p.hq / p.groups, vm = ring_vmode(p, vshared);
  const bool lo = p.qn_lo != nullptr, r = p.R != nullptr;
  if (vm == RING_VHEADS) {
    RingParams a = p;
    a.groups = 1;
    a.total_wg = batch * p.max_splits;
#define XKV_RING_VH(NHB, DN) \
  if (lo && (p.hq <= 16 ? 1 : 2) == NHB && p.dn == DN) return launch_ring_t<T, 16, NHB, true, DN, false, RING_VHEADS, 1024>(a, batch, st);
    XKV_RING_VH(1, 512) XKV_RING_VH(2, 512) XKV_RING_VH(1, 384) XKV_RING_VH(2, 384) XKV_RING_VH(1, 256) XKV_RING_VH(2, 256)
#undef XKV_RING_VH
    if (p.dn == 1024 && !lo)
      return p.hq <= 16 ? launch_ring_t<T, 16, 1, false, 1024, false, RING_VHEADS, 1024>(a, batch, st)
                        : launch_ring_t<T, 16, 2, false, 1024, false, RING_VHEADS, 1024>(a, batch, st);
    return XKV_EUNSUPPORTED;
  }
  const int nhb = hg <= 16 ? 1 : 2;
#define XKV_RING_CASE(TN, NHB, LO, DN, HAS_R, VM) \
  if (nhb == NHB && lo == LO && p.dn == DN && r == HAS_R && vm == VM) return launch_ring_t<T, TN, NHB, LO, DN, HAS_R, VM>(p, batch, st);
  // 512-wide rows, one stream: scores (absorbed q carries a low part or not), shared-tile decode (+ RoPE keys)
  XKV_RING_CASE(32, 1, true, 512, false, RING_SCORES)    XKV_RING_CASE(32, 2, true, 512, false, RING_SCORES)
  XKV_RING_CASE(32, 1, false, 512, false, RING_SCORES)   XKV_RING_CASE(32, 2, false, 512, false, RING_SCORES)
  XKV_RING_CASE(32, 1, false, 512, false, RING_VSHARED)  XKV_RING_CASE(32, 2, false, 512, false, RING_VSHARED)
  XKV_RING_CASE(32, 1, true, 512, false, RING_VSHARED)   XKV_RING_CASE(32, 2, true, 512, false, RING_VSHARED)
  XKV_RING_CASE(32, 1, false, 512, true, RING_VSHARED)   XKV_RING_CASE(32, 2, false, 512, true, RING_VSHARED)
  // two row streams (keys 256 .. 1024 wide, values 256 .. 512 wide): 16-token tiles
#define XKV_RING_V2(NHB, LO, DN, DVW) \
  if (nhb == NHB && lo == LO && p.dn == DN && !r && vm == RING_VDISTINCT && p.dv == DVW) \
    return launch_ring_t<T, 16, NHB, LO, DN, false, RING_VDISTINCT, DVW>(p, batch, st);
#define XKV_RING_V2_ALL(LO, DN) \
  XKV_RING_V2(1, LO, DN, 512) XKV_RING_V2(2, LO, DN, 512) XKV_RING_V2(1, LO, DN, 384) XKV_RING_V2(2, LO, DN, 384) \
  XKV_RING_V2(1, LO, DN, 256) XKV_RING_V2(2, LO, DN, 256)
  XKV_RING_V2_ALL(true, 512) XKV_RING_V2_ALL(true, 384) XKV_RING_V2_ALL(true, 256)   // absorbed query, both factorised
  XKV_RING_V2_ALL(false, 1024)                                                       // per-head keys as one row, V factorised
  XKV_RING_V2(1, false, 512, 512) XKV_RING_V2(2, false, 512, 512)                    // plain 512-wide keys and values
#undef XKV_RING_V2_ALL
#undef XKV_RING_V2
  // ranks 384 and 256, one stream (absorbed queries always carry a low part)
  XKV_RING_CASE(32, 1, true, 384, false, RING_SCORES)    XKV_RING_CASE(32, 2, true, 384, false, RING_SCORES)
  XKV_RING_CASE(32, 1, true, 384, false, RING_VSHARED)   XKV_RING_CASE(32, 2, true, 384, false, RING_VSHARED)
  XKV_RING_CASE(32, 1, true, 256, false, RING_SCORES)    XKV_RING_CASE(32, 2, true, 256, false, RING_SCORES)
  XKV_RING_CASE(32, 1, true, 256, false, RING_VSHARED)   XKV_RING_CASE(32, 2, true, 256, false, RING_VSHARED)
#undef XKV_RING_CASE
  return XKV_EUNSUPPORTED;
}

bool ring_eligible(const RingParams& p, bool vshared) {
  const int hg = p.hq / p.groups, vm = ring_vmode(p, vshared);
  const bool lo = p.qn_lo != nullptr, r = p.R != nullptr;
  if (vm == RING_VHEADS) return true;
  if (hg > 32 || vm < 0) return false;
  if ((p.dn == 1024) != (p.heads_in_row == 8)) return false;   // the 1024-wide form is only the eight-heads-in-a-row one
  if (p.dn != 512 && !(p.dn == 1024 && vm == RING_VDISTINCT && !lo) && !((p.dn == 384 || p.dn == 256) && lo && !r)) return false;
  if (r && (p.dr != 64 || lo || vm != RING_VSHARED)) return false;
  if (p.sCl < p.dn || (r && p.sRl < 64) || (vm == RING_VDISTINCT && p.sVl < p.dv)) return false;
  if (vm == RING_VDISTINCT && p.dn == 512 && !lo && p.dv != 512) return false;
  return true;
}

int launch_ring_given(const RingParams& p, int batch, int dtype, hipStream_t st) {
  return dtype == XKV_BF16 ? launch_ring_given_dt<__bf16>(p, batch, st) : launch_ring_given_dt<_Float16>(p, batch, st);
}

int launch_ring(const RingParams& p, int batch, bool vshared, int dtype, hipStream_t st) {
  return dtype == XKV_BF16 ? launch_ring_dt<__bf16>(p, batch, vshared, st) : launch_ring_dt<_Float16>(p, batch, vshared, st);
}

}  // namespace xkv
