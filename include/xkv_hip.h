/* xkv_hip.h - C ABI of libxkv_hip.so: MI355X (gfx950) kernels of the xKV compressed-KV decode path.
 *
 * The reference project is pure Python + Triton; the "FFI" each entry point replaces is
 * therefore a Triton kernel launch (`kernel[grid](...)`) inside one of its Python wrappers.
 * Each prototype cites that launch (paths relative to the reference repository).
 *
 * Conventions
 *   - plain pointers, 32/64-bit integers and floats only; no torch / pybind types.
 *   - every pointer is DEVICE memory unless named host_*; the library never allocates,
 *     frees or keeps state between calls (workspaces are caller-owned).
 *   - all launches go to `stream` (a hipStream_t passed as void*) and return without
 *     synchronising.  Return value: XKV_OK, a negative XKV_E* argument error detected on the
 *     host before any launch, or a positive hipError_t from the launch.
 *   - strides are in ELEMENTS.  The innermost (feature) axis of every 16-bit operand is
 *     unit-stride and every row start is 16-byte aligned (strides multiple of 8 elements).
 *   - `dtype` is the 16-bit operand type of q / A / B / K / V (XKV_F16 or XKV_BF16);
 *     accumulation is always fp32.
 *   - split arithmetic (which tokens split i of a sequence covers, which splits are live) is
 *     the reference's, flash_decoding/gqa.py:95-99 and :273-281, bit for bit, with the
 *     sequence length taken from kv_lens[b] when kv_lens != NULL (ragged batch) else kv_len.
 *   - `split_cap_tokens` (xkv_latent_stage1, xkv_merge_stage2; 0 = off): no split longer than this many tokens.  Sequence b is
 *     then scanned with max(num_kv_splits[b], ceil(len_b / split_cap_tokens)) splits in that same arithmetic, evaluated on
 *     the device by stage 1 and by the merge alike, so a ragged batch whose caller asks for long splits is still spread over
 *     the whole chip.  max_splits - the split dimension of the workspaces - must then be at least ceil(kv_len /
 *     split_cap_tokens) (XKV_EINVAL otherwise).  Split-K is exact under the merge: the result does not depend on it.
 *   - `split_plan` (same two entry points; NULL = off): the int32 array xkv_plan_splits wrote in device memory.  Its
 *     first word is a cap; the cap in force is then max(split_cap_tokens, plan[0]) - the host value bounds the workspaces,
 *     the device value, chosen from the lengths of the batch, which the host never reads, makes the splits as long as the
 *     batch allows while every CU still gets one.  Stage 1 also takes its (sequence, split) pairs from the plan's job
 *     list, so the workgroups that have work are the first ones of the grid and spread evenly over the XCDs.
 */
#ifndef XKV_HIP_H
#define XKV_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XKV_ABI_VERSION 6

enum { XKV_F16 = 0, XKV_BF16 = 1, XKV_F32 = 2 };

enum {
  XKV_OK = 0,
  XKV_EINVAL = -1,      /* null pointer / non-positive size */
  XKV_EUNSUPPORTED = -2,/* shape outside the built envelope (see each function) */
  XKV_EALIGN = -3,      /* stride or pointer not 16-byte aligned */
  XKV_EDTYPE = -4,
  XKV_ESCRATCH = -5,    /* xkv_recon_stage1_static: needs more than XKV_STATIC_SCRATCH_BYTES */
  XKV_ETOOLCHAIN = -6   /* this build of a kernel that tracks its own loads spills registers: rebuild with the validated compiler */
};

int xkv_abi_version(void);
const char* xkv_error_string(int code);

/* RoPE tables: sin[l, j] / cos[l, j] of angle float(start + l) * inv_freq[j], l < seqlen, j < half_dim,
 * written as out_dtype (XKV_F32 / XKV_F16 / XKV_BF16), row stride = half_dim.
 * Replaces _rotary_sin_cos_kernel_multi[grid] at flash_recontruction/rope/sin_cos.py:92-97
 * (angles follow the eager closed form of rope/rope_ref.py:3-9: fp32 pos * fp32 inv_freq). */
int xkv_rope_table(void* sin_out, void* cos_out, const float* inv_freq, int64_t seqlen, int64_t start,
                   int half_dim, int out_dtype, void* stream);

/* Rotate-half RoPE applied on the device, out of place or in place (out == x):
 *   pos            = (positions ? positions[b] : pos0) + r            (positions: device int64 [batch], may be NULL)
 *   out[b,r,h,j]        = x[b,r,h,j] * cos(a) - x[b,r,h,j+dim/2] * sin(a),   a = float(pos) * inv_freq[j]  (fp32)
 *   out[b,r,h,j+dim/2]  = x[b,r,h,j+dim/2] * cos(a) + x[b,r,h,j] * sin(a)
 * for x, out [batch, rows, heads, dim] with element strides (b, r, h) and a unit feature stride; dtype XKV_F32 / F16 /
 * BF16 (arithmetic in fp32).  A decode step's query is rows == 1 at positions[b] = that sequence's length; a tail of
 * freshly decoded keys is rows == its length at positions[b] = its first position.
 * Replaces the eager x * cos + rotate_half(x) * sin of flash_recontruction/rope/rope_ref.py:17-20 on tables from
 * rope_ref.py:3-9 (what the reference's callers run on the host side of every kernel that takes `q_pe`). */
int xkv_rope_apply(const void* x, void* out, const float* inv_freq, const int64_t* positions, int64_t pos0,
                   int batch, int rows, int heads, int dim,
                   int64_t stride_x_b, int64_t stride_x_r, int64_t stride_x_h,
                   int64_t stride_o_b, int64_t stride_o_r, int64_t stride_o_h,
                   int dtype, void* stream);

/* Absorb the query into the per-kv-head factor: qt[b, h, rho] = sum_d q[b, h, d] * B[b, h / G, rho, d]
 * as a 16-bit high part `qt_hi` and (optional, may be NULL) residual `qt_lo` so that hi + lo carries
 * ~16 mantissa bits.  q is [batch, hq, d] contiguous.  qt_* are [batch, hq, rank] contiguous.
 * Replaces the host-side torch.matmul(q_nope, kv_B_nope.transpose(1, 2)) at
 * flash_decoding/mla2/mla_flash_decoding.py:81-82 and is what makes the no-PE score scan a GEMV
 * over A (the eager form attention.py:312-318) instead of the per-tile reconstruction of
 * flash_recontruction/qAB_no_pe/v1.py:53-74.   d <= 512, d % 8 == 0. */
int xkv_absorb_q(const void* q, const void* B, void* qt_hi, void* qt_lo,
                 int batch, int hq, int hkv, int d, int rank,
                 int64_t stride_B_b, int64_t stride_B_h, int64_t stride_B_r,
                 int dtype, void* stream);

/* Block-diagonal query: out[b, h, kh * d + c] = q[b, h, c] when kh == h / (hq / hkv), else 0; q is [batch, hq, d],
 * out [batch, hq, hkv * d], both contiguous.  Against it the per-head keys of a token, stored side by side
 * ([batch, kv_len, hkv, d] with unit head stride d), behave as one hkv*d-wide row shared by every head, so
 * xkv_latent_stage1 can serve all heads of a sequence from one workgroup (n_kv_groups = 1) and read a value basis
 * that the heads share once per token instead of once per kv head.  No reference counterpart: the reference has the
 * V-only factorised decode only in eager form (attention.py:202-274).   d % 8 == 0. */
int xkv_blockdiag_q(const void* q, void* out, int batch, int hq, int hkv, int d, int dtype, void* stream);

/* Operand descriptors of the generic split-K stage 1. */
typedef struct {
  const void* ptr;     /* [batch, kv_len, heads?, dim]; NULL = absent                      */
  int64_t stride_b;    /* batch stride                                                     */
  int64_t stride_l;    /* token stride                                                     */
  int64_t stride_h;    /* kv-head stride (0 when one latent serves every head)             */
  int dim;             /* feature width                                                    */
} xkv_kv_operand;

typedef struct {
  const void* ptr;     /* [batch, hq, dim] contiguous; NULL = absent                       */
  int dim;
} xkv_q_operand;

/* Split-K flash-decoding stage 1 over "latent-like" operands (plain dot-product scores):
 *
 *   s[b, h, l]   = sm_scale * ( qn[b,h,:] . C[b,l,kvh(h),:]  (+ qn_lo . C)  (+ qr[b,h,:] . R[b,l,kvh(h),:]) )
 *   per live split i of sequence b (tokens [start,end)):
 *     m = max_l s ; den = sum_l exp(s - m) ; partial[b,h,i,:] = sum_l exp(s-m) V[b,l,kvh(h),:] / den ;
 *     lse[b,h,i] = m + log(den)
 *
 * kvh(h) = h / (hq / n_kv_groups).  With n_kv_groups == 1 every head shares one latent row
 * (xKV no-PE after xkv_absorb_q: C = k_A, V = v_A; MLA: C = V = c_kv, R = k_pe).  With
 * n_kv_groups == hkv it is plain GQA (C = K, V = V) or a mix (C = K, V = v_A with stride_h 0).
 * If V.ptr == C.ptr with equal strides and dim the tile is loaded once.
 * If scores_out != NULL the kernel ONLY writes scores (scaled) as [batch, hq, kv_len] in
 * scores_dtype and skips softmax/PV (qAB no-PE form).
 * Dead splits write nothing.  partial is [batch, hq, max_splits, V.dim] fp32, lse [batch, hq, max_splits] fp32.
 * Envelope: heads per kv group <= 32; C.dim % 32 == 0, <= 1024; R.dim % 32 == 0, <= 128;
 *           V.dim % 64 == 0, <= 512.
 * Plain keys of 8 kv heads x 128 stored side by side in a token row (n_kv_groups == 8, C.dim == 128, C.stride_h == 128,
 * hq <= 32), with values laid out the same way or as one shared 256 / 384 / 512-wide row (V.stride_h == 0), are served
 * by one workgroup per (sequence, split) for ALL heads: the token's keys are then one 1024-wide row against a block-
 * diagonal query that the kernel builds from qn.  Same call, same result; only the work distribution differs (one job
 * per split instead of eight), which is what xkv_plan_splits' target_jobs should count.
 * Replaces _fwd_grouped_kernel_stage1[grid] at flash_decoding/gqa.py:205-237,
 * flash_decoding/mla.py (same launcher, :243-283), flash_decoding/mla2/stage1.py:213-249,
 * flash_recontruction/fused_attention/no_pe/v1.py:227-262 (and v2.py / v1_k_only.py twins) and,
 * in scores_out mode, _qAB_fwd[grid] at flash_recontruction/qAB_no_pe/v1.py:123-132 (v2.py:117-126). */
int xkv_latent_stage1(xkv_q_operand qn, const void* qn_lo, xkv_q_operand qr,
                      xkv_kv_operand C, xkv_kv_operand R, xkv_kv_operand V,
                      float* partial, float* lse,
                      void* scores_out, int scores_dtype,
                      const int32_t* num_kv_splits, const int32_t* kv_lens,
                      int batch, int hq, int n_kv_groups, int kv_len, int max_splits, int split_cap_tokens,
                      const int32_t* split_plan, float sm_scale, float logit_cap, int dtype, void* stream);

/* Split-K stage 1 over scores that already exist: per live split, the online softmax of scores[b, h, start:end] and
 *   partial[b,h,i,:] = sum_l exp(s - m) V[b,l,:] / den ;  lse[b,h,i] = m + log(den)
 * with scores fp32 [batch, hq, kv_len] as written (scaled) by the scores_out mode of xkv_recon_stage1 or
 * xkv_latent_stage1, and V one row per token shared by every head (V.stride_h == 0; V.dim 256 / 384 / 512).  It is the
 * second pass of a fused decode whose value basis differs from its key basis: the first pass rebuilds and rotates the keys
 * at the rate of the scores-only kernel, this one streams v_A once for all heads.  Splits, kv_lens, split_cap_tokens and
 * split_plan as in xkv_latent_stage1; the softmax weights are rounded to `dtype` before P.V as everywhere else.
 * hq <= 32; kv_len % 4 == 0.  No single reference launch: the reference fuses this into its stage-1 kernels
 * (fused_attention/no_pe/v1.py:40-190) and has no RoPE-aware fused decode at all. */
int xkv_softmax_pv_stage1(const float* scores, xkv_kv_operand V, float* partial, float* lse,
                          const int32_t* num_kv_splits, const int32_t* kv_lens,
                          int batch, int hq, int kv_len, int max_splits, int split_cap_tokens, const int32_t* split_plan,
                          int dtype, void* stream);

/* Split-K stage 1 with fused key reconstruction and RoPE:
 *
 *   K[b,kh,l,:]  = kA[b,l,:] @ kB[b,kh,:,:]                      (rank x 128, fp32 accumulate)
 *   K'           = rotate-half RoPE of K at position pos_offset + l, angle float(pos) * inv_freq[j]
 *                  (or, if sin_cos != NULL, sin = sin_cos[l, j], cos = sin_cos[l, 64 + j], a
 *                  [kv_len, 128] table of the operand dtype, row stride sc_stride_l)
 *   s[b,h,l]     = sm_scale * q_pe[b,h,:] . K'[b,h/G,l,:]        (K' rounded to the operand dtype)
 *
 * then either scores_out (as above) or the split softmax with V = vA (rank-space partials
 * [batch, hq, max_splits, vA.dim]).  rope == 0 skips the rotation (pure reconstruction).
 * Envelope: head_dim == 128, G = hq/hkv <= 16, rank % 32 == 0, rank <= 512, vA.dim % 64 == 0 <= 512.
 * With computed angles (sin_cos == NULL), G <= 8 and a workspace of xkv_recon_workspace_bytes() the call runs a
 * specialised kernel (kB packed once into the workspace, stationary in registers; v_mfma_f32_32x32x16; direct-to-LDS tile
 * rings): at ranks 256 / 384 / 512 with scores_out or vA the same tensor as kA the wave-specialised kernel (four
 * reconstruction waves in a 2 x 2 rank/feature split hand fp16 key tiles to four waves that rotate, score, soften and
 * accumulate P.A; scores only at rank 256: the 4-wave form, two workgroups per CU); at those ranks with a separate vA of
 * rank 256 / 384 / 512 the 8-wave kernel (2 x 4 split, second row stream for vA).  Otherwise the generic one.
 * Replaces _qAB_fwd[grid] at flash_recontruction/qAB/v1.py:135-145 (v3.py / v4.py / ref.py twins) and
 * _qAB_fwd_precomp[grid] at qAB/v2.py:170-186 in scores_out mode; the fused form has no single
 * reference launch - it composes that reconstruction with the stage 1 of
 * fused_attention/no_pe/v1.py:227-262. */
int xkv_recon_stage1(const void* q_pe, xkv_kv_operand kA, const void* kB,
                     int64_t stride_kB_b, int64_t stride_kB_h, int64_t stride_kB_r,
                     xkv_kv_operand vA,
                     float* partial, float* lse,
                     void* scores_out, int scores_dtype,
                     const int32_t* num_kv_splits, const int32_t* kv_lens,
                     int batch, int hq, int hkv, int kv_len, int max_splits,
                     float sm_scale, int rope, const float* inv_freq, int64_t pos_offset,
                     const void* sin_cos, int64_t sc_stride_l,
                     void* workspace, int64_t workspace_bytes,
                     int dtype, void* stream);

/* Bytes of caller-owned scratch that lets xkv_recon_stage1 take its MFMA-bound fast path (kB re-packed into MFMA
 * operand order: one copy per batch entry, a single copy when stride_kB_b == 0).  0: no fast path for this rank.
 * Passing workspace == NULL (or too few bytes) is valid and selects the generic kernel.  No reference counterpart. */
int64_t xkv_recon_workspace_bytes(int batch, int hkv, int rank, int64_t stride_kB_b);

/* xkv_recon_stage1 for callers that cannot allocate device memory (code under HIP graph capture, serving loops or
 * harnesses that forbid hipMalloc): the same arguments without the workspace, the same kernels and results.  The scratch
 * that the fast paths need (xkv_recon_workspace_bytes(): kB re-packed into MFMA operand order) is a static device array of
 * XKV_STATIC_SCRATCH_BYTES inside the library, one copy per GPU, held until the process ends; the call allocates and
 * frees nothing.  A shape that needs more (hkv * rank * 128 * 2 bytes per copy of kB, one copy per batch entry unless
 * stride_kB_b == 0) returns XKV_ESCRATCH and launches nothing.  Every call on a GPU uses that GPU's one array and
 * overwrites what the previous call left there: calls on the same GPU must not overlap (two streams, two threads) - they
 * would race on it; calls in stream order on one stream are safe.  The device current at the call must be the stream's.
 * The FIRST call on a device for a given kernel shape does host-side set-up (the array's address is looked up with
 * hipGetSymbolAddress, the kernel's dynamic LDS size is raised with hipFuncSetAttribute): make one warm-up call per device
 * and shape outside stream capture before capturing.  XKV_ESCRATCH is returned only for shapes that would take a path that
 * packs kB (generated RoPE angles, at most 8 query heads per kv head); other shapes run the generic kernel without scratch.
 * No counterpart in the reference, whose wrappers allocate with torch.empty on every call
 * (flash_recontruction/fused_attention/no_pe/v1.py:434-446). */
#define XKV_STATIC_SCRATCH_BYTES (4 << 20)
int xkv_recon_stage1_static(const void* q_pe, xkv_kv_operand kA, const void* kB,
                            int64_t stride_kB_b, int64_t stride_kB_h, int64_t stride_kB_r,
                            xkv_kv_operand vA,
                            float* partial, float* lse,
                            void* scores_out, int scores_dtype,
                            const int32_t* num_kv_splits, const int32_t* kv_lens,
                            int batch, int hq, int hkv, int kv_len, int max_splits,
                            float sm_scale, int rope, const float* inv_freq, int64_t pos_offset,
                            const void* sin_cos, int64_t sc_stride_l,
                            int dtype, void* stream);

/* Stage 2: LSE-weighted merge of the live splits in increasing split id,
 *   out[b,h,:] = sum_i w_i partial[b,h,i,:] / sum_i w_i ,  w_i = exp(lse_i - max lse),
 * optionally followed by the value up-projection out[b,h,:] = merged[b,h,:] @ vB[b, h/G, :, :]
 * (vB == NULL: none; then out width = dv).  out is [batch, hq, out_dim] with strides
 * (stride_o_b, stride_o_h), written as out_dtype.
 * Replaces _fwd_kernel_stage2[grid] at flash_decoding/gqa.py:322-337 (mla.py, mla2/stage2.py:117-135,
 * fused_attention/no_pe/v1.py:345-362 twins) and the torch.matmul with v_B_buffer at
 * fused_attention/no_pe/v2.py:468-471 / v1.py:458-460.   dv <= 512; d_out <= 512.
 * lse_out (may be NULL): the log-sum-exp of the merged range, lse_out[b * stride_lse_b + h * stride_lse_h] =
 * log sum_i exp(lse_i), which lets the merged row take part in a further merge as one split (prefix + tail decode,
 * flash_decoding/deepseek_mla/flash_decoding.py:137-155 concatenates the workspaces instead). */
int xkv_merge_stage2(const float* partial, const float* lse, void* out,
                     const void* vB, int64_t stride_vB_b, int64_t stride_vB_h, int64_t stride_vB_r,
                     int d_out, int vB_dtype,
                     const int32_t* num_kv_splits, const int32_t* kv_lens,
                     int batch, int hq, int hkv, int kv_len, int max_splits, int split_cap_tokens,
                     const int32_t* split_plan, int dv,
                     int64_t stride_o_b, int64_t stride_o_h, int out_dtype,
                     float* lse_out, int64_t stride_lse_b, int64_t stride_lse_h, void* stream);

/* Split plan for a ragged batch: plan[0] = cap, the smallest multiple of 32, not below floor_tokens, such that
 * sum_b ceil(kv_lens[b] / cap) <= target_jobs; plan[1] = the number of jobs, i.e. live (sequence, split) pairs when
 * sequence b is cut into max(num_kv_splits[b], ceil(kv_lens[b] / cap)) splits; plan[2 + 2 j], plan[3 + 2 j] = sequence and
 * split of job j (whole splits first, each sequence's last - shorter - split after them).  With target_jobs = the number
 * of CUs, a stage 1 that runs one workgroup per CU gives every CU exactly one job and the jobs are as equal as the lengths
 * allow; a batch scanned in fixed-length splits ends on whatever the last workgroups happen to hold.  plan holds
 * 2 + 2 * batch * max_splits int32 (max_splits as passed to stage 1, >= ceil(kv_len / floor_tokens)).  Pass plan as
 * split_plan, and floor_tokens as split_cap_tokens, to xkv_latent_stage1 and xkv_merge_stage2 on the same stream.  One
 * small workgroup; no host synchronisation.  No counterpart in the reference, whose batches have one length
 * (flash_decoding/gqa.py:60,194). */
int xkv_plan_splits(const int32_t* kv_lens, const int32_t* num_kv_splits, int batch, int max_splits, int floor_tokens,
                    int target_jobs, int32_t* plan, void* stream);

/* Measurement aids (no counterpart in the reference; bench.py --config ceilings): what this GPU sustains with nothing but
 * the instruction a kernel is bound by.
 * xkv_ceiling_mfma: every wave of `workgroups` x 256 threads issues iters x 32 v_mfma_f32_32x32x16 (dtype XKV_BF16 / XKV_F16) on
 *   register operands, four independent accumulator chains; FLOP = workgroups * 4 * iters * 32 * 32768.  out: workgroups * 256 floats.
 * xkv_ceiling_stream: reads the first workgroups * 4 * 8192 * floor(bytes / (workgroups * 4 * 8192)) bytes of src once, each wave
 *   its own contiguous share in 8 KiB steps, into registers (to_lds == 0), straight into a per-wave LDS ring of `depth` steps
 *   (to_lds == 1; depth 2, 3 or 4; depth - 1 steps in flight) that nothing reads, or into a register queue `depth` steps deep (to_lds
 *   == 2; depth 2, 4 or 6) whose steps are written on to LDS with ds_write_b128 as they land.  out: 256 floats
 *   (to_lds == 2: workgroups * 256 floats, the number of 16-byte packets each thread handed on). */
int xkv_ceiling_mfma(float* out, int workgroups, int iters, int dtype, void* stream);
int xkv_ceiling_stream(const void* src, int64_t bytes, int workgroups, int to_lds, int depth, float* out, void* stream);

/* Test aid (no counterpart in the reference; tests/test_gpu_lds_poison.py).  The LDS is not cleared between kernels.  With
 * seen == NULL: fills all 160 KiB of LDS of every CU with `pattern` (0x7FFF7FFF is a NaN as fp16, bf16 and fp32), so that a
 * kernel launched next on the stream which reads LDS that it has not written yet, or whose asynchronous tile loads have not
 * landed, computes NaNs instead of plausible stale rows.  With seen != NULL (2 int32, zeroed by the caller): one workgroup
 * per CU adds the number of LDS words that still hold `pattern` to seen[0] and the number it looked at to seen[1], which tells
 * a test whether the poison of the previous call was still there. */
int xkv_poison_lds(uint32_t pattern, int32_t* seen, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* XKV_HIP_H */
