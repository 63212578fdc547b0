// Stand-alone pieces of the GatedDeltaNet layer core for gfx950: gates, q/k norm, conv4+SiLU+norm over S tokens, gated
// RMSNorm and the sequential recurrence.  Arithmetic contract: see qt_common.h.
#include "qt_common.h"

using namespace qt;

namespace {

// compute_g + beta (qwen35/gated_delta.py:16-18,158; rounding points of qwen35/kernels.py:511-515).
// a, b are read with a row stride so they can be taken straight out of the 8224-wide projection row.
__global__ __launch_bounds__(256) void gates_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ b, long a_stride,
                                                    long b_stride, const float* __restrict__ A_log,
                                                    const float* __restrict__ dt_bias, float* __restrict__ g,
                                                    float* __restrict__ lg, bf16_t* __restrict__ beta, long rows, int hv) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * hv) return;
    const long r = i / hv;
    const int h = (int)(i % hv);
    const float av = BF(bf2f(a[r * a_stride + h]) + dt_bias[h]);
    const float l = log_decay(A_log[h], av);
    if (g) g[i] = expf(l);
    if (lg) lg[i] = l;
    if (beta) beta[i] = f2bf(sigmoid_bf16(bf2f(b[r * b_stride + h])));
}

// normalize_qk (qwen35/gated_delta.py:21-30) on rows of 128: one wavefront per row, two elements per lane
__global__ __launch_bounds__(256) void normalize_qk_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                                                           bf16_t* __restrict__ qo, bf16_t* __restrict__ ko, long rows) {
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= rows) return;
    const float scq = BF(INV_SCALE * INV_SCALE), sck = BF(INV_SCALE);
    const uint32_t wq = reinterpret_cast<const uint32_t*>(q + row * DK)[lane];
    const uint32_t wk = reinterpret_cast<const uint32_t*>(k + row * DK)[lane];
    const float q0 = lo_bf(wq), q1 = hi_bf(wq), k0 = lo_bf(wk), k1 = hi_bf(wk);
    const float qs = (float)wave_sum_d((double)q0 * q0 + (double)q1 * q1);
    const float ks = (float)wave_sum_d((double)k0 * k0 + (double)k1 * k1);
    const float qr = rsqrt_rn(qs / (float)DK + qk_eps()), kr = rsqrt_rn(ks / (float)DK + qk_eps());
    reinterpret_cast<uint32_t*>(qo + row * DK)[lane] = pack_bf(BF(BF(q0 * qr) * scq), BF(BF(q1 * qr) * scq));
    reinterpret_cast<uint32_t*>(ko + row * DK)[lane] = pack_bf(BF(BF(k0 * kr) * sck), BF(BF(k1 * kr) * sck));
}

// conv_prep (qwen35/prefill.py:96-134, 228-238): proj [S,8224], cs [3,6144] -> q, k, v [S,16,128].
// A workgroup of 256 threads handles 64 consecutive tokens of one head: a 16-lane group owns 4 consecutive tokens (their 7
// input rows are loaded once and shared by the 4 sliding windows), a lane 8 consecutive channels of q, of k and of v; all row
// loads are issued before the first conv, SiLU comes from the LDS table, the sums of squares are reduced over the 16 lanes of
// the group and the 8 reciprocal square roots are evaluated one per lane.
constexpr int CP_TOK = 64;
__global__ __launch_bounds__(256, 2) void conv_prep_kernel(const bf16_t* __restrict__ proj, const bf16_t* __restrict__ cs,
                                                           const bf16_t* __restrict__ cw, const bf16_t* __restrict__ silu_tab,
                                                           bf16_t* __restrict__ q, bf16_t* __restrict__ k, bf16_t* __restrict__ v,
                                                           int S) {
    __shared__ __align__(16) bf16_t tab[SILU_TAB_SIZE];
    const int tb = blockIdx.x / HV, h = blockIdx.x % HV, tid = threadIdx.x, gi = tid >> 4, cc = tid & 15;
    const int t0 = tb * CP_TOK + 4 * gi;
    uint4 rw[3][7], wt[3][4];
#pragma unroll
    for (int part = 0; part < 3; part++) {
        const int ch0 = part * KD + h * DK + cc * 8;
#pragma unroll
        for (int e = 0; e < 4; e++) wt[part][e] = *reinterpret_cast<const uint4*>(cw + (size_t)(ch0 + 2 * e) * 4);
#pragma unroll
        for (int d = 0; d < 7; d++) {
            const int tt = min(t0 - 3 + d, S - 1);                             // rows past the end are computed and dropped
            rw[part][d] = *reinterpret_cast<const uint4*>(tt < 0 ? cs + (tt + 3) * CD + ch0 : proj + (size_t)tt * PW + ch0);
        }
    }
    silu_table_fill(tab, silu_tab, tid, 256);
    __syncthreads();
    const float scq = BF(INV_SCALE * INV_SCALE), sck = BF(INV_SCALE);
    uint4 pk[4][3];
    float ss[8], rr[8];
#pragma unroll
    for (int part = 0; part < 3; part++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const double sq = conv8_silu_packed(tab, rw[part][j], rw[part][j + 1], rw[part][j + 2], rw[part][j + 3], wt[part], pk[j][part]);
            if (part < 2) ss[2 * j + part] = (float)row16_sum_d(sq);
        }
    rsqrt_rows<8>(ss, qk_eps(), rr, cc);
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int t = t0 + j;
        if (t < S) {
            const size_t o = ((size_t)t * HV + h) * DK + cc * 8;
            *reinterpret_cast<uint4*>(q + o) = scale8_packed(pk[j][0], rr[2 * j], scq);
            *reinterpret_cast<uint4*>(k + o) = scale8_packed(pk[j][1], rr[2 * j + 1], sck);
            *reinterpret_cast<uint4*>(v + o) = pk[j][2];
        }
    }
}

__global__ __launch_bounds__(256) void silu_table_kernel(bf16_t* __restrict__ tab) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < SILU_TAB_SIZE) tab[i] = silu_table_entry(i);
}

// gated RMSNorm (qwen35/batch.py:304-343, qwen35/prefill.py:137-157): 16 lanes per (row, head), 8 elements per lane; a
// workgroup takes GN_ROWS rows (all loads first), and the GN_ROWS double-precision reciprocal square roots of a 16-lane group
// are evaluated one per lane instead of all by every lane.  GN_ROWS = 4 for many rows (the kernel is then bound by those
// evaluations), 1 for few (bound by the latency of one workgroup).
template <int GN_ROWS>
__global__ __launch_bounds__(256) void gated_norm_kernel(const bf16_t* __restrict__ y, const bf16_t* __restrict__ proj,
                                                         const float* __restrict__ gw, bf16_t* __restrict__ out, long rows,
                                                         float eps) {
    const int h = threadIdx.x >> 4, c = threadIdx.x & 15;
    const long row0 = (long)blockIdx.x * GN_ROWS;
    uint4 yv[GN_ROWS], zv[GN_ROWS];
#pragma unroll
    for (int it = 0; it < GN_ROWS; it++) {
        const long row = row0 + it < rows ? row0 + it : rows - 1;              // rows past the end are computed and dropped
        yv[it] = reinterpret_cast<const uint4*>(y + row * KD + h * DV)[c];
        zv[it] = reinterpret_cast<const uint4*>(proj + row * PW + CD + h * DV)[c];
    }
    float gwv[8];
#pragma unroll
    for (int j = 0; j < 8; j++) gwv[j] = gw[c * 8 + j];
    float ss[GN_ROWS], inv[GN_ROWS];
#pragma unroll
    for (int it = 0; it < GN_ROWS; it++) {
        float yy[8];
        unpack8(yv[it], yy);
        double s2 = 0.0;
#pragma unroll
        for (int j = 0; j < 4; j++) s2 += (double)yy[2 * j] * yy[2 * j] + (double)yy[2 * j + 1] * yy[2 * j + 1];
        ss[it] = (float)row16_sum_d(s2);
    }
    rsqrt_rows<GN_ROWS>(ss, eps, inv, c);
#pragma unroll
    for (int it = 0; it < GN_ROWS; it++) {
        if (row0 + it >= rows) break;
        float yy[8], zz[8];
        unpack8(yv[it], yy);
        unpack8(zv[it], zz);
        uint32_t o[8];
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] = gated_out(zz[j], gwv[j] * (yy[j] * inv[it]));
        reinterpret_cast<uint4*>(out + (row0 + it) * KD + h * DV)[c] =
            make_uint4(o[0] | (o[1] << 16), o[2] | (o[3] << 16), o[4] | (o[5] << 16), o[6] | (o[7] << 16));
    }
}

// gated_delta_update's kernel (qwen35/gated_delta.py:33-137): T sequential tokens with q, k, v, g, beta given.
// One workgroup of 256 threads per (batch, value head, 16-row block); a 16-lane group owns one value row, a lane 8 of its
// 128 columns; no LDS, no barriers.  q, k [B,T,Hk,128], v, y [B,T,Hv,Dv], g f32 / beta bf16 [B,T,Hv], state [B,Hv,Dv,128].
// Dv is a multiple of 8 (gated_delta.py:164-166): the last block of a Dv that is no multiple of 16 has eight idle row groups,
// which work on a copy of the last row and store nothing.
__global__ __launch_bounds__(256) void recurrent_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                                                        const bf16_t* __restrict__ v, const float* __restrict__ g,
                                                        const bf16_t* __restrict__ beta, const float* st_in,
                                                        float* st_out, bf16_t* __restrict__ y, int T, int Hk, int Hv,
                                                        int Dv) {
    const int nblk = (Dv + 15) / 16;
    const int blk = blockIdx.x % nblk, n = blockIdx.x / nblk;             // n = b*Hv + hv
    const int b = n / Hv, hv = n % Hv, hk = hv / (Hv / Hk);              // gated_delta.py:43-46
    const int tid = threadIdx.x, c = tid & 15;
    const bool live = blk * 16 + (tid >> 4) < Dv;                         // whole 16-lane groups are live or idle together
    const int row = min(blk * 16 + (tid >> 4), Dv - 1);
    const size_t so = ((size_t)n * Dv + row) * DK;
    float sv[8];
    {
        const float4 a = reinterpret_cast<const float4*>(st_in + so)[c], d = reinterpret_cast<const float4*>(st_in + so)[16 + c];
        sv[0] = a.x; sv[1] = a.y; sv[2] = a.z; sv[3] = a.w; sv[4] = d.x; sv[5] = d.y; sv[6] = d.z; sv[7] = d.w;
    }
    const bf16_t* qp = q + ((size_t)b * T * Hk + hk) * DK;
    const bf16_t* kp = k + ((size_t)b * T * Hk + hk) * DK;
    const bf16_t* vp = v + ((size_t)b * T * Hv + hv) * Dv + row;
    bf16_t* yp = y + ((size_t)b * T * Hv + hv) * Dv + row;
    const float* gp = g + (size_t)b * T * Hv + hv;
    const bf16_t* bp = beta + (size_t)b * T * Hv + hv;
    for (int t = 0; t < T; t++) {
        const uint2 qa = reinterpret_cast<const uint2*>(qp)[c], qb = reinterpret_cast<const uint2*>(qp)[16 + c];
        const uint2 ka = reinterpret_cast<const uint2*>(kp)[c], kb = reinterpret_cast<const uint2*>(kp)[16 + c];
        const float q8[8] = {lo_bf(qa.x), hi_bf(qa.x), lo_bf(qa.y), hi_bf(qa.y), lo_bf(qb.x), hi_bf(qb.x), lo_bf(qb.y), hi_bf(qb.y)};
        const float k8[8] = {lo_bf(ka.x), hi_bf(ka.x), lo_bf(ka.y), hi_bf(ka.y), lo_bf(kb.x), hi_bf(kb.x), lo_bf(kb.y), hi_bf(kb.y)};
        const float kq = dot8_row16(k8, q8);
        const float yv = gdn_row_step(sv, k8, q8, bf2f(*vp), *gp, bf2f(*bp), kq);
        if (c == 0 && live) *yp = f2bf(yv);
        qp += (size_t)Hk * DK;
        kp += (size_t)Hk * DK;
        vp += (size_t)Hv * Dv;
        yp += (size_t)Hv * Dv;
        gp += Hv;
        bp += Hv;
    }
    if (!live) return;
    reinterpret_cast<float4*>(st_out + so)[c] = make_float4(sv[0], sv[1], sv[2], sv[3]);
    reinterpret_cast<float4*>(st_out + so)[16 + c] = make_float4(sv[4], sv[5], sv[6], sv[7]);
}

inline bool al(const void* p, unsigned a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

}  // namespace

extern "C" {

int qt_gdn_gates(const void* a, const void* b, long a_stride, long b_stride, const float* A_log, const float* dt_bias,
                 float* g, float* log_g, void* beta, long rows, int hv, hipStream_t stream) {
    if (!a || !A_log || !dt_bias || (beta && !b)) return QT_ERR_NULL;
    if (rows < 0 || hv <= 0) return QT_ERR_DIM;
    if (rows == 0) return QT_OK;
    const long n = rows * hv;
    hipLaunchKernelGGL(gates_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, (const bf16_t*)a, (const bf16_t*)b,
                       a_stride, b_stride, A_log, dt_bias, g, log_g, (bf16_t*)beta, rows, hv);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

int qt_normalize_qk(const void* q, const void* k, void* q_out, void* k_out, long rows, int dk, hipStream_t stream) {
    if (!q || !k || !q_out || !k_out) return QT_ERR_NULL;
    if (dk != DK) return QT_ERR_UNSUPPORTED;
    if (rows < 0) return QT_ERR_DIM;
    if (rows == 0) return QT_OK;
    if (!al(q, 4) || !al(k, 4) || !al(q_out, 4) || !al(k_out, 4)) return QT_ERR_ALIGN;
    hipLaunchKernelGGL(normalize_qk_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, (const bf16_t*)q,
                       (const bf16_t*)k, (bf16_t*)q_out, (bf16_t*)k_out, rows);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

int qt_silu_table_bytes(void) { return SILU_TAB_SIZE * 2; }

int qt_silu_table_build(void* table, hipStream_t stream) {
    if (!table) return QT_ERR_NULL;
    if (!al(table, 16)) return QT_ERR_ALIGN;
    hipLaunchKernelGGL(silu_table_kernel, dim3((SILU_TAB_SIZE + 255) / 256), dim3(256), 0, stream, (bf16_t*)table);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

int qt_gdn_conv_prep(const void* proj, const void* conv_state, const void* conv_w, const void* silu_table, void* q, void* k,
                     void* v, int S, hipStream_t stream) {
    if (!proj || !conv_state || !conv_w || !q || !k || !v) return QT_ERR_NULL;
    if (S < 0) return QT_ERR_DIM;
    if (S == 0) return QT_OK;
    for (const void* p : {proj, conv_state, conv_w, silu_table, (const void*)q, (const void*)k, (const void*)v})
        if (!al(p, 16)) return QT_ERR_ALIGN;
    hipLaunchKernelGGL(conv_prep_kernel, dim3((unsigned)((S + CP_TOK - 1) / CP_TOK) * HV), dim3(256), 0, stream, (const bf16_t*)proj,
                       (const bf16_t*)conv_state, (const bf16_t*)conv_w, (const bf16_t*)silu_table, (bf16_t*)q, (bf16_t*)k,
                       (bf16_t*)v, S);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

int qt_gated_rmsnorm(const void* y, const void* proj, const float* gw, void* out, long rows, float eps, hipStream_t stream) {
    if (!y || !proj || !gw || !out) return QT_ERR_NULL;
    if (rows < 0) return QT_ERR_DIM;
    if (rows == 0) return QT_OK;
    if (!al(y, 16) || !al(proj, 16) || !al(out, 16)) return QT_ERR_ALIGN;
    if (rows >= 4096)
        hipLaunchKernelGGL(gated_norm_kernel<4>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, (const bf16_t*)y,
                           (const bf16_t*)proj, gw, (bf16_t*)out, rows, eps);
    else
        hipLaunchKernelGGL(gated_norm_kernel<1>, dim3((unsigned)rows), dim3(256), 0, stream, (const bf16_t*)y, (const bf16_t*)proj, gw,
                           (bf16_t*)out, rows, eps);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

int qt_gdn_recurrent(const void* q, const void* k, const void* v, const float* g, const void* beta, const float* state_in,
                     float* state_out, void* y, int B, int T, int Hk, int Hv, int Dk, int Dv, hipStream_t stream) {
    if (!q || !k || !v || !g || !beta || !state_in || !state_out || !y) return QT_ERR_NULL;
    if (Dk != DK || Dv <= 0 || Dv % 8 || Hk <= 0 || Hv <= 0 || Hv % Hk) return QT_ERR_UNSUPPORTED;   // gated_delta.py:164-166
    if (B < 0 || T < 0) return QT_ERR_DIM;
    if (B == 0) return QT_OK;
    if (!al(q, 8) || !al(k, 8) || !al(state_in, 16) || !al(state_out, 16)) return QT_ERR_ALIGN;
    hipLaunchKernelGGL(recurrent_kernel, dim3((unsigned)(B * Hv * ((Dv + 15) / 16))), dim3(256), 0, stream, (const bf16_t*)q,
                       (const bf16_t*)k, (const bf16_t*)v, g, (const bf16_t*)beta, state_in, state_out, (bf16_t*)y, T, Hk, Hv, Dv);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

}  // extern "C"
