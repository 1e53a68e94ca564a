/* Brute-force double-precision restatement of the xKV decode path.
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/libxkv_oracle.so and loaded by
 * tests/ (and by nothing under kernel_collections_amd/).  Every routine is a
 * direct loop nest over the defining sums, written independently of the eager
 * PyTorch restatement in xkv_oracle.py so that a transposed operand, a wrong
 * rotate-half sign or a dropped scale in either one shows up as a mismatch.
 * Sizes are meant to be tiny (seconds of scalar work).
 *
 * Reference lines followed (paths relative to the reference repository):
 *   split arithmetic      flash_decoding/gqa.py:95-99, :273-281
 *   RoPE closed form      flash_recontruction/rope/rope_ref.py:3-20
 *   reconstruct + rotate  test_qAB_rope.py:19-43
 *   factorised decode     attention.py:276-357
 *   plain decode          flash_decoding/mla.py:442-471 (scale multiplied)
 *   MLA latent decode     flash_decoding/mla2/ref.py:3-33 (scale multiplied)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

#define MIN_BLOCK_KV 32

static int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

/* gqa.py:95-99 */
void xo_split_bounds(int64_t kv_len, int64_t splits, int64_t id, int64_t *start, int64_t *end)
{
    int64_t per = cdiv(cdiv(kv_len, splits), MIN_BLOCK_KV) * MIN_BLOCK_KV;
    int64_t s = per * id, e = s + per;
    if (e > kv_len) e = kv_len;
    *start = s;
    *end = e;
}

/* exact-angle cos/sin of position pos for pair index j (j < dim/2) */
void xo_rope_cs(int64_t pos, int64_t j, int64_t dim, double theta, double *c, double *s)
{
    double ang = (double)pos * pow(theta, -2.0 * (double)j / (double)dim);
    *c = cos(ang);
    *s = sin(ang);
}

/* K[l, :] = sum_rho A[l,rho] * B[rho,:]; optional rotate-half RoPE at position pos0+l.
 * x' = x*cos + rotate_half(x)*sin, rotate_half(x) = (-x[h:], x[:h])   (rope_ref.py:11-20) */
static void key_row(const double *A_l, const double *Bh, int64_t r, int64_t d,
                    int rope, double theta, int64_t pos, double *k)
{
    for (int64_t c = 0; c < d; ++c) {
        double a = 0.0;
        for (int64_t rho = 0; rho < r; ++rho) a += A_l[rho] * Bh[rho * d + c];
        k[c] = a;
    }
    if (rope) {
        int64_t h = d / 2;
        for (int64_t j = 0; j < h; ++j) {
            double cs, sn, x0 = k[j], x1 = k[j + h];
            xo_rope_cs(pos, j, d, theta, &cs, &sn);
            k[j] = x0 * cs - x1 * sn;
            k[j + h] = x1 * cs + x0 * sn;
        }
    }
}

/* scores[b,hq,l] = q[b,hq,:] . K[b,hq/g,l,:]   (no scale), K = (RoPE of) A@B.
 * q [b,hq,d], A [b,L,r], B [b,hkv,r,d], out [b,hq,L] */
void xo_qab(const double *q, const double *A, const double *B, double *out,
            int64_t b, int64_t hq, int64_t hkv, int64_t d, int64_t L, int64_t r,
            int rope, double theta, int64_t pos0)
{
    int64_t g = hq / hkv;
    double *k = (double *)malloc(sizeof(double) * d);
    for (int64_t ib = 0; ib < b; ++ib)
        for (int64_t h = 0; h < hkv; ++h)
            for (int64_t l = 0; l < L; ++l) {
                key_row(A + (ib * L + l) * r, B + (ib * hkv + h) * r * d, r, d, rope, theta, pos0 + l, k);
                for (int64_t gi = 0; gi < g; ++gi) {
                    const double *qq = q + (ib * hq + h * g + gi) * d;
                    double s = 0.0;
                    for (int64_t c = 0; c < d; ++c) s += qq[c] * k[c];
                    out[(ib * hq + h * g + gi) * L + l] = s;
                }
            }
    free(k);
}

/* softmax over l of sm_scale*scores, then out[b,hq,:] = sum_l p_l * V[b,hkv,l,:]
 * with V = vA @ vB (vA [b,L,rv], vB [b,hkv,rv,d]).  Full factorised decode. */
void xo_decode_factorized(const double *q, const double *kA, const double *kB,
                          const double *vA, const double *vB, double *out,
                          int64_t b, int64_t hq, int64_t hkv, int64_t d, int64_t L,
                          int64_t rk, int64_t rv, double sm_scale,
                          int rope, double theta, int64_t pos0)
{
    int64_t g = hq / hkv;
    double *sc = (double *)malloc(sizeof(double) * b * hq * L);
    double *v = (double *)malloc(sizeof(double) * d);
    xo_qab(q, kA, kB, sc, b, hq, hkv, d, L, rk, rope, theta, pos0);
    for (int64_t ib = 0; ib < b; ++ib)
        for (int64_t h = 0; h < hq; ++h) {
            double *s = sc + (ib * hq + h) * L, m = -INFINITY, den = 0.0;
            double *o = out + (ib * hq + h) * d;
            for (int64_t l = 0; l < L; ++l) { s[l] *= sm_scale; if (s[l] > m) m = s[l]; }
            for (int64_t l = 0; l < L; ++l) { s[l] = exp(s[l] - m); den += s[l]; }
            for (int64_t c = 0; c < d; ++c) o[c] = 0.0;
            for (int64_t l = 0; l < L; ++l) {
                key_row(vA + (ib * L + l) * rv, vB + (ib * hkv + h / g) * rv * d, rv, d, 0, 0.0, 0, v);
                for (int64_t c = 0; c < d; ++c) o[c] += s[l] / den * v[c];
            }
        }
    free(sc);
    free(v);
}

/* plain GQA decode: q [b,hq,dk], K [b,L,hkv,dk], V [b,L,hkv,dv] -> out [b,hq,dv] */
void xo_decode_plain(const double *q, const double *K, const double *V, double *out,
                     int64_t b, int64_t hq, int64_t hkv, int64_t dk, int64_t dv, int64_t L,
                     double sm_scale)
{
    int64_t g = hq / hkv;
    double *s = (double *)malloc(sizeof(double) * L);
    for (int64_t ib = 0; ib < b; ++ib)
        for (int64_t h = 0; h < hq; ++h) {
            int64_t kh = h / g;
            const double *qq = q + (ib * hq + h) * dk;
            double m = -INFINITY, den = 0.0, *o = out + (ib * hq + h) * dv;
            for (int64_t l = 0; l < L; ++l) {
                const double *kk = K + ((ib * L + l) * hkv + kh) * dk;
                double a = 0.0;
                for (int64_t c = 0; c < dk; ++c) a += qq[c] * kk[c];
                s[l] = a * sm_scale;
                if (s[l] > m) m = s[l];
            }
            for (int64_t l = 0; l < L; ++l) { s[l] = exp(s[l] - m); den += s[l]; }
            for (int64_t c = 0; c < dv; ++c) o[c] = 0.0;
            for (int64_t l = 0; l < L; ++l) {
                const double *vv = V + ((ib * L + l) * hkv + kh) * dv;
                for (int64_t c = 0; c < dv; ++c) o[c] += s[l] / den * vv[c];
            }
        }
    free(s);
}

/* MLA latent decode: q_nope [b,H,c], q_rope [b,H,e], ckv [b,L,c], kpe [b,L,e] -> out [b,H,c] */
void xo_mla(const double *qn, const double *qr, const double *ckv, const double *kpe, double *out,
            int64_t b, int64_t H, int64_t c, int64_t e, int64_t L, double sm_scale)
{
    double *s = (double *)malloc(sizeof(double) * L);
    for (int64_t ib = 0; ib < b; ++ib)
        for (int64_t h = 0; h < H; ++h) {
            double m = -INFINITY, den = 0.0, *o = out + (ib * H + h) * c;
            for (int64_t l = 0; l < L; ++l) {
                double a = 0.0;
                for (int64_t i = 0; i < c; ++i) a += qn[(ib * H + h) * c + i] * ckv[(ib * L + l) * c + i];
                for (int64_t i = 0; i < e; ++i) a += qr[(ib * H + h) * e + i] * kpe[(ib * L + l) * e + i];
                s[l] = a * sm_scale;
                if (s[l] > m) m = s[l];
            }
            for (int64_t l = 0; l < L; ++l) { s[l] = exp(s[l] - m); den += s[l]; }
            for (int64_t i = 0; i < c; ++i) o[i] = 0.0;
            for (int64_t l = 0; l < L; ++l)
                for (int64_t i = 0; i < c; ++i) o[i] += s[l] / den * ckv[(ib * L + l) * c + i];
        }
    free(s);
}
