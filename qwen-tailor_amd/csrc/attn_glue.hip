// The elementwise steps either side of the attention kernels of a full-attention layer, for gfx950: q / k RMSNorm, partial
// rotary embedding (the first 64 of 256 features, half-split pairing, theta = 1e7) and the output gate o * sigmoid(gate).
// Replaces the MLX graph ops of the reference's layer (qwen35/batch.py:505-513, qwen35/model.py:154-169):
//     qkv row = [ (q_h[256] | gate_h[256]) for h = 0..7 | k[2][256] | v[2][256] ]                         (5120 bf16)
//     q = rope(rms_norm(q_h, q_norm), pos),  k = rope(rms_norm(k, k_norm), pos),  v = v
//     out = o * sigmoid(gate)
// Arithmetic contract (fixed here so that a CPU restatement reproduces every bf16 value): sum of squares exact, rounded to
// float once; inv = correctly rounded 1/sqrt(ss/256 + eps); t = BF(x * inv); y = BF(w * t) (weight bf16); rotary angle
// theta = float(pos) * freq_i with freq_i = float(1e7^(-2 i / 64)); cos / sin = the double-precision libm values rounded to
// float; y1' = BF(y1 * c - y2 * s), y2' = BF(y1 * s + y2 * c), each product and the sum rounded to float separately;
// gate: BF(o * sigmoid_bf16(g)) with the bf16 sigmoid of the GatedDeltaNet path (qwen35/mslib.py:16-20).
#include "qt_common.h"

using namespace qt;

namespace {

constexpr int QKV_W = AH * 2 * AD + 2 * AKV * AD;      // 5120
constexpr int ROPE_DIM = 64;

__constant__ float rope_freq[ROPE_DIM / 2] = {
    1.0f, 0.604296386f, 0.365174115f, 0.220673412f, 0.133352146f, 0.0805842206f, 0.0486967526f, 0.0294272713f,
    0.0177827943f, 0.0107460786f, 0.00649381615f, 0.0039241896f, 0.00237137382f, 0.00143301254f, 0.000865964335f,
    0.000523299095f, 0.000316227757f, 0.0001910953f, 0.0001154782f, 6.97830619e-05f, 4.21696495e-05f,
    2.54829683e-05f, 1.5399266e-05f, 9.3057206e-06f, 5.62341347e-06f, 3.39820826e-06f, 2.05352512e-06f,
    1.24093776e-06f, 7.49894184e-07f, 4.5315835e-07f, 2.73841977e-07f, 1.65481708e-07f};

// One workgroup per row r = b * M + j (position pos[b] + j): threads 0..31 bring the row's 32 (cos, sin) pairs into LDS, from
// the table of rope_table_kernel where it covers the position, else evaluated here (double-precision libm, the expensive part:
// the same expression, so the same bits); then a wavefront takes one 256-wide vector at a time (lane l holds elements
// 4l .. 4l+3) out of the row's 12: 0..7 = q heads, 8..9 = k heads, 10..11 = v heads.
__global__ __launch_bounds__(256) void attn_qkv_prep_kernel(const bf16_t* __restrict__ qkv, const bf16_t* __restrict__ q_norm,
                                                            const bf16_t* __restrict__ k_norm, const int* __restrict__ pos,
                                                            bf16_t* __restrict__ q, bf16_t* __restrict__ k, bf16_t* __restrict__ v,
                                                            long R, int M, float eps, const float2* __restrict__ table,
                                                            int table_positions) {
    __shared__ float cs_s[2][ROPE_DIM / 2];
    const long r = blockIdx.x;
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const bf16_t* row = qkv + r * QKV_W;
    // all loads of this wavefront's three vectors first
    uint2 xw[3];
#pragma unroll
    for (int t = 0; t < 3; t++) {
        const int part = w + 4 * t;
        xw[t] = reinterpret_cast<const uint2*>(part < 8 ? row + part * 2 * AD : row + AH * 2 * AD + (part - 8) * AD)[lane];
    }
    const uint2 wq = reinterpret_cast<const uint2*>(q_norm)[lane], wk = reinterpret_cast<const uint2*>(k_norm)[lane];
    if (threadIdx.x < ROPE_DIM / 2) {
        const int ip = pos[r / M] + (int)(r % M);
        if (ip >= 0 && ip < table_positions) {                   // (table_positions = 0 without a table)
            const float2 cs = table[(size_t)ip * (ROPE_DIM / 2) + threadIdx.x];
            cs_s[0][threadIdx.x] = cs.x;
            cs_s[1][threadIdx.x] = cs.y;
        } else {
            const float th = __fmul_rn((float)ip, rope_freq[threadIdx.x]);
            cs_s[0][threadIdx.x] = (float)cos((double)th);
            cs_s[1][threadIdx.x] = (float)sin((double)th);
        }
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < 3; t++) {
        const int part = w + 4 * t;                              // wavefront-uniform
        if (part >= 10) {                                        // v: a plain copy into the contiguous [R,2,256] layout
            reinterpret_cast<uint2*>(v + (r * AKV + (part - 10)) * AD)[lane] = xw[t];
            continue;
        }
        const bool is_q = part < 8;
        const uint2 ww = is_q ? wq : wk;
        float x[4] = {lo_bf(xw[t].x), hi_bf(xw[t].x), lo_bf(xw[t].y), hi_bf(xw[t].y)};
        const float wt[4] = {lo_bf(ww.x), hi_bf(ww.x), lo_bf(ww.y), hi_bf(ww.y)};
        double ss = 0.0;
#pragma unroll
        for (int e = 0; e < 4; e++) ss += (double)x[e] * x[e];
        const float inv = rsqrt_rn((float)wave_sum_d(ss) / (float)AD + eps);
        float y[4];
#pragma unroll
        for (int e = 0; e < 4; e++) y[e] = BF(wt[e] * BF(x[e] * inv));
        // rotary embedding of features 0..63: lanes 0..7 hold x1 = features 0..31, lanes 8..15 their partners 32..63
        float o4[4];
#pragma unroll
        for (int e = 0; e < 4; e++) o4[e] = __shfl_xor(y[e], 8, 64);
        if (lane < 16) {
            // The two products and their sum are rounded one by one.  Plain operators inside a contract(off) block: the
            // __fmul_rn / __fadd_rn helpers are ordinary operators compiled elsewhere, which the compiler contracts into one
            // fused multiply-add after inlining (a bf16 value in ~10^5 then rounds the other way).
#pragma clang fp contract(off)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int i = (lane & 7) * 4 + e;
                const float c = cs_s[0][i], sn = cs_s[1][i];
                const float own = y[e] * c, other = o4[e] * sn;
                y[e] = BF(lane < 8 ? own - other                 // y1 c - y2 s
                                   : other + own);               // y1 s + y2 c
            }
        }
        bf16_t* dst = is_q ? q + (r * AH + part) * AD : k + (r * AKV + (part - 8)) * AD;
        reinterpret_cast<uint2*>(dst)[lane] = make_uint2(pack_bf(y[0], y[1]), pack_bf(y[2], y[3]));
    }
}

// (cos, sin) of every rotary angle of positions 0 .. n_pos - 1, exactly the values the kernel above evaluates per row:
// table[p][i] = ((float)cos((double)th), (float)sin((double)th)), th = float(p) * rope_freq[i] rounded to float
__global__ __launch_bounds__(256) void rope_table_kernel(float2* __restrict__ table, int n_pos) {
    const long t = (long)blockIdx.x * 256 + threadIdx.x;
    if (t >= (long)n_pos * (ROPE_DIM / 2)) return;
    const int p = (int)(t / (ROPE_DIM / 2)), i = (int)(t % (ROPE_DIM / 2));
    const float th = __fmul_rn((float)p, rope_freq[i]);
    table[t] = make_float2((float)cos((double)th), (float)sin((double)th));
}

// out[r][h*256 + d] = BF(o[r][h][d] * sigmoid_bf16(gate_h[d])), gate_h = qkv[r][h*512 + 256 ..]; 8 elements per thread
__global__ __launch_bounds__(256) void attn_out_gate_kernel(const bf16_t* __restrict__ o, const bf16_t* __restrict__ qkv,
                                                            bf16_t* __restrict__ out, long R) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;       // one 8-element group: AH * AD / 8 = 256 groups per row
    const long r = i >> 8;
    if (r >= R) return;
    const int c = (int)(i & 255), h = c >> 5, d = (c & 31) * 8;
    const uint4 ov = *reinterpret_cast<const uint4*>(o + (r * AH + h) * AD + d);
    const uint4 gv = *reinterpret_cast<const uint4*>(qkv + r * QKV_W + h * 2 * AD + AD + d);
    float of[8], gf[8];
    unpack8(ov, of);
    unpack8(gv, gf);
    uint32_t p[4];
#pragma unroll
    for (int e = 0; e < 4; e++) p[e] = pack_bf(of[2 * e] * sigmoid_bf16(gf[2 * e]), of[2 * e + 1] * sigmoid_bf16(gf[2 * e + 1]));
    *reinterpret_cast<uint4*>(out + (r * AH + h) * AD + d) = make_uint4(p[0], p[1], p[2], p[3]);
}

}  // namespace

extern "C" {

// rope_table: null, or the (cos, sin) pairs of positions 0 .. table_positions - 1 as qt_rope_table_build writes them; rows at
// positions beyond the table evaluate their pairs themselves, with the same bits
int qt_attn_qkv_prep_table(const void* qkv, const void* q_norm, const void* k_norm, const int32_t* pos, const void* rope_table,
                           int table_positions, void* q, void* k, void* v, long R, int M, float eps, hipStream_t stream) {
    if (!qkv || !q_norm || !k_norm || !pos || !q || !k || !v) return QT_ERR_NULL;
    if (R < 0 || M < 1 || R % M || table_positions < 0) return QT_ERR_DIM;
    if (R == 0) return QT_OK;
    for (const void* p : {qkv, q_norm, k_norm, rope_table, (const void*)q, (const void*)k, (const void*)v})
        if (reinterpret_cast<uintptr_t>(p) & 7u) return QT_ERR_ALIGN;
    hipLaunchKernelGGL(attn_qkv_prep_kernel, dim3((unsigned)R), dim3(256), 0, stream, (const bf16_t*)qkv, (const bf16_t*)q_norm,
                       (const bf16_t*)k_norm, pos, (bf16_t*)q, (bf16_t*)k, (bf16_t*)v, R, M, eps, (const float2*)rope_table,
                       rope_table ? table_positions : 0);
    QT_CHECK_LAUNCH();
    return QT_OK;
}
int qt_attn_qkv_prep(const void* qkv, const void* q_norm, const void* k_norm, const int32_t* pos, void* q, void* k, void* v, long R,
                     int M, float eps, hipStream_t stream) {
    return qt_attn_qkv_prep_table(qkv, q_norm, k_norm, pos, nullptr, 0, q, k, v, R, M, eps, stream);
}

int qt_rope_table_build(void* table, int n_pos, hipStream_t stream) {
    if (!table) return QT_ERR_NULL;
    if (n_pos < 0) return QT_ERR_DIM;
    if (reinterpret_cast<uintptr_t>(table) & 15u) return QT_ERR_ALIGN;
    if (n_pos == 0) return QT_OK;
    const long n = (long)n_pos * (ROPE_DIM / 2);
    hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, (float2*)table, n_pos);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

int qt_attn_out_gate(const void* o, const void* qkv, void* out, long R, hipStream_t stream) {
    if (!o || !qkv || !out) return QT_ERR_NULL;
    if (R < 0) return QT_ERR_DIM;
    if (R == 0) return QT_OK;
    for (const void* p : {o, qkv, (const void*)out})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    hipLaunchKernelGGL(attn_out_gate_kernel, dim3((unsigned)R), dim3(256), 0, stream, (const bf16_t*)o, (const bf16_t*)qkv,
                       (bf16_t*)out, R);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

}  // extern "C"
