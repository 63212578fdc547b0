/* CPU restatement, in plain C, of the fused GatedDeltaNet decode step and the sequential recurrence of
 * wang90063/Qwen-tailor.
 *
 * TEST INFRASTRUCTURE ONLY: this file is the checker (and the timed CPU baseline) for the HIP kernels.
 * The product library never links or calls it.
 *
 * Follows qwen35/batch.py:36-125 (deltanet_b), qwen35/kernels.py:476-541 (deltanet), qwen35/mslib.py:7-27
 * (bf16 rounding structure of sigmoid / silu / softplus) and qwen35/gated_delta.py:75-126 (the recurrence).
 * The arithmetic contract is the one of gdn_oracle.py: exp/log are the double-precision libm results rounded
 * to float, sums of squares are exact (double) and rounded once, rsqrt = (float)(1/sqrt) in double, and the dot products of the
 * recurrence are accumulated in double (acc64 != 0) or in float, sequentially (acc64 == 0).
 *
 * Build: gcc -O2 -fopenmp -ffp-contract=off -shared -fPIC gdn_oracle.c -o libgdn_oracle.so -lm
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

enum { HV = 16, DK = 128, DV = 128, KD = 2048, CD = 6144, PW = 8224 };

static inline float bf2f(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint16_t f2bf(float f) { /* round to nearest even */
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static inline float BF(float f) { return bf2f(f2bf(f)); }
static inline float exp32(float x) { return (float)exp((double)x); }
static inline float log32(float x) { return (float)log((double)x); }

static inline float log1p_mx(float x) { /* mslib.py:11-15 */
    float xp1 = 1.0f + x;
    if (xp1 == 1.0f) return x;
    return x * (log32(xp1) / (xp1 - 1.0f));
}
static inline float sigmoid_bf16(float x) { /* mslib.py:16-20 */
    float y = BF(1.0f / BF(1.0f + BF(exp32(fabsf(x)))));
    return x < 0.0f ? y : BF(1.0f - y);
}
static inline float silu_bf16(float x) { return BF(x * sigmoid_bf16(x)); } /* mslib.py:21-22 */
static inline float softplus_bf16(float x) {                               /* mslib.py:23-26 */
    return BF(fmaxf(x, 0.0f) + BF(log1p_mx(BF(exp32(-fabsf(x))))));
}

/* conv4 + silu of channel ch: win = 3 previous rows (oldest first, row stride CD), x = current row (kernels.py:480-484) */
static inline float conv_silu(const uint16_t* win, const uint16_t* x, const uint16_t* cw, int ch) {
    float s = bf2f(win[ch]) * bf2f(cw[ch * 4]);
    s = s + bf2f(win[CD + ch]) * bf2f(cw[ch * 4 + 1]);
    s = s + bf2f(win[2 * CD + ch]) * bf2f(cw[ch * 4 + 2]);
    s = s + bf2f(x[ch]) * bf2f(cw[ch * 4 + 3]);
    return silu_bf16(BF(s));
}

static void norm_scale(float* u, float sc) { /* kernels.py:504-510 */
    const float inv_scale = 0.08838834764831845f;
    const float e2 = (1e-6f * inv_scale) * inv_scale;
    double ss = 0.0;
    for (int i = 0; i < DK; i++) ss += (double)u[i] * (double)u[i];
    float r = (float)(1.0 / sqrt((double)((float)ss / (float)DK + e2)));
    for (int i = 0; i < DK; i++) u[i] = BF(BF(u[i] * r) * sc);
}

/* one head, one token: s = S*g; kv = s.k; d = (v-kv)*beta; s += k*d; y = s.q   (kernels.py:518-530) */
static void head_step(float* S, const float* q, const float* k, const float* v, float g, float beta, uint16_t* y,
                      int acc64) {
    for (int r = 0; r < DV; r++) {
        float* s = S + r * DK;
        if (acc64) {
            double kv = 0.0, yy = 0.0, sd[DK];
            for (int c = 0; c < DK; c++) {
                sd[c] = (double)s[c] * (double)g;
                kv += sd[c] * (double)k[c];
            }
            double d = ((double)v[r] - kv) * (double)beta;
            for (int c = 0; c < DK; c++) {
                sd[c] += (double)k[c] * d;
                yy += sd[c] * (double)q[c];
                s[c] = (float)sd[c];
            }
            y[r] = f2bf((float)yy);
        } else {
            float kv = 0.f, yy = 0.f;
            for (int c = 0; c < DK; c++) {
                s[c] = s[c] * g;
                kv += s[c] * k[c];
            }
            float d = (v[r] - kv) * beta;
            for (int c = 0; c < DK; c++) {
                s[c] = s[c] + k[c] * d;
                yy += s[c] * q[c];
            }
            y[r] = f2bf(yy);
        }
    }
}

/* batch.deltanet_b (batch.py:128-135): one token for each of B rows; ssm_pool[slot] and conv buffer (pos&1)^1 are
 * updated in place.  proj [B,8224] bf16, conv_pool [(S+1)*2,3,6144] bf16, cw [6144*4] bf16, ssm_pool [S+1,16,128,128]
 * f32, y [B,2048] bf16. */
void gdn_oracle_decode_step(const uint16_t* proj, uint16_t* conv_pool, const uint16_t* cw, const float* A_log,
                            const float* dt_bias, float* ssm_pool, const int32_t* slots, const int32_t* pos,
                            uint16_t* y, int B, int acc64, int nthreads) {
    const float inv_scale = 0.08838834764831845f;
    const float sc_q = BF(inv_scale * inv_scale), sc_k = BF(inv_scale);
#pragma omp parallel for collapse(2) num_threads(nthreads) schedule(static)
    for (int b = 0; b < B; b++) {
        for (int h = 0; h < HV; h++) {
            const size_t slot = (size_t)slots[b];
            const int par = pos[b] & 1;
            const uint16_t* win = conv_pool + (slot * 2 + par) * 3 * CD;
            uint16_t* wout = conv_pool + (slot * 2 + (par ^ 1)) * 3 * CD;
            const uint16_t* x = proj + (size_t)b * PW;
            float q[DK], k[DK], v[DV];
            for (int i = 0; i < DK; i++) {
                q[i] = conv_silu(win, x, cw, h * DK + i);
                k[i] = conv_silu(win, x, cw, KD + h * DK + i);
                v[i] = conv_silu(win, x, cw, 2 * KD + h * DV + i);
            }
            norm_scale(q, sc_q);
            norm_scale(k, sc_k);
            float av = BF(bf2f(x[CD + KD + HV + h]) + dt_bias[h]);
            float g = exp32(-exp32(A_log[h]) * softplus_bf16(av));
            float beta = sigmoid_bf16(bf2f(x[CD + KD + h]));
            head_step(ssm_pool + (slot * HV + h) * DV * DK, q, k, v, g, beta, y + (size_t)b * KD + h * DV, acc64);
            const int base[3] = {h * DK, KD + h * DK, 2 * KD + h * DV};
            for (int u = 0; u < 3; u++)
                for (int i = 0; i < DK; i++) {
                    int ch = base[u] + i;
                    wout[ch] = win[CD + ch];
                    wout[CD + ch] = win[2 * CD + ch];
                    wout[2 * CD + ch] = x[ch];
                }
        }
    }
}

/* gated_delta_update's kernel (gated_delta.py:75-126) with g (f32) and beta (bf16) given: q, k [B,T,16,128] bf16,
 * v [B,T,16,128] bf16, g [B,T,16] f32, beta [B,T,16] bf16, state [B,16,128,128] f32 in place, y [B,T,16,128] bf16. */
void gdn_oracle_recurrent(const uint16_t* q, const uint16_t* k, const uint16_t* v, const float* g,
                          const uint16_t* beta, float* state, uint16_t* y, int B, int T, int acc64, int nthreads) {
#pragma omp parallel for collapse(2) num_threads(nthreads) schedule(static)
    for (int b = 0; b < B; b++) {
        for (int h = 0; h < HV; h++) {
            float qf[DK], kf[DK], vf[DV];
            for (int t = 0; t < T; t++) {
                size_t o = (((size_t)b * T + t) * HV + h);
                for (int i = 0; i < DK; i++) {
                    qf[i] = bf2f(q[o * DK + i]);
                    kf[i] = bf2f(k[o * DK + i]);
                    vf[i] = bf2f(v[o * DV + i]);
                }
                head_step(state + ((size_t)b * HV + h) * DV * DK, qf, kf, vf, g[o], bf2f(beta[o]), y + o * DV, acc64);
            }
        }
    }
}
