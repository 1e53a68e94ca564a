// Parameters of the split-K stage 1 over dot-product scores, and the entry of its wide-row (LDS ring) variant.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace xkv {

struct LatentParams {
  const void* qn; const void* qn_lo; const void* qr;
  const void* C; const void* R; const void* V;
  int64_t sCb, sCl, sCh, sRb, sRl, sRh, sVb, sVl, sVh;   // element strides
  int dn, dr, dv;
  float* partial; float* lse; void* scores; int scores_dtype;
  const int32_t* num_splits; const int32_t* kv_lens;
  int hq, groups, kv_len, max_splits, total_wg;
  int split_cap;   // > 0: no split longer than this many tokens (effective_splits)
  const int32_t* split_plan;   // not null: [0] cap (the cap in force is max(split_cap, it)), [1] jobs, then (sequence, split) pairs
  int heads_in_row;   // 8: C rows are 8 plain kv heads of 128 side by side and qn holds compact rows [b, hq, 128]; else 0
  float sm_scale, logit_cap;
};
typedef LatentParams RingParams;

// True when the shape is one the ring kernel is built for: 512-wide latent rows (optionally + 64 RoPE features), or
// 384 / 256 wide ones scanned with an absorbed query (hi + lo parts); V the latent itself, scores only, a second row
// stream 256 / 384 / 512 wide (keys then 256 .. 1024 wide), or plain per-kv-head values [token][8][128] under one shared
// absorbed key basis or under plain per-head keys taken as one 1024-wide row.  Everything else runs the register-staged kernel.
bool ring_eligible(const RingParams& p, bool vshared);
int launch_ring(const RingParams& p, int batch, bool vshared, int dtype, hipStream_t st);
// Softmax + P.V over scores that are an input (p.scores: fp32 [batch, hq, kv_len], already scaled); p.C = the value rows
// (256 / 384 / 512 wide, one row per token for every head), p.groups == 1, hq <= 32, kv_len % 4 == 0.
int launch_ring_given(const RingParams& p, int batch, int dtype, hipStream_t st);

}  // namespace xkv
