// Causal prefill attention, 8 query heads on 2 KV heads, head dim 256, for gfx950 (flash-attention forward on bf16 MFMA).
// Replaces the call mx.fast.scaled_dot_product_attention(q, K[:, :, :kv_len], V[:, :, :kv_len], scale=256**-0.5,
// mask="causal") of the reference's full-attention layers (qwen35/model.py:160-167, qwen35/prefill.py:468).
//
// One wavefront owns 16 query rows and keeps everything transposed so that no value ever changes lanes:
//     S^T[keys x rows] = K_tile . Q^T          (A = K rows straight from HBM / L2, B = Q^T resident in registers)
//     O^T[d x rows]   += V^T_tile . P^T        (A = rows of V^T, B = P^T)
// In the accumulator layout lane (n, g) holds rows 4g..4g+3 of column n.  With columns = query rows, the running max, the
// rescale and the final 1/l of a query row are lane-local, and two S^T accumulators, exponentiated and packed to bf16,
// ARE the B operand of the P.V MFMA when the key index of a 32-key block is enumerated as 16 (j >> 2) + 4 g + (j & 3).
// V^T rows are read from a transposed copy of V (qt_gqa_transpose_v, one small pass) so the A operand is contiguous.
#include "qt_common.h"

using namespace qt;

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr float SCALE = 0.0625f;       // 256^-0.5
constexpr float NEG = -3.0e38f;

// V [KV][L][256] -> VT [KV][256][Lp] (keys past L are zero), 64 x 64 tiles through LDS
__global__ __launch_bounds__(256) void transpose_v_kernel(const bf16_t* __restrict__ V, bf16_t* __restrict__ VT, int L, int Lp,
                                                          long v_head_stride) {
    __shared__ bf16_t tile[64][66];
    const int kvh = blockIdx.z, k0 = blockIdx.x * 64, d0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4) {
        const int key = k0 + i;
        tile[i][tx] = key < L ? V[(size_t)kvh * v_head_stride + (size_t)key * AD + d0 + tx] : (bf16_t)0;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const int key = k0 + tx;
        if (key < Lp) VT[((size_t)kvh * AD + d0 + i) * Lp + key] = tile[tx][i];
    }
}

__global__ __launch_bounds__(256) void attn_prefill_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ K,
                                                           const bf16_t* __restrict__ VT, bf16_t* __restrict__ out, int S, int L,
                                                           int Lp, int q_pos0, long q_head_stride, long k_head_stride) {
    const int qt = gridDim.x - 1 - blockIdx.x;                   // long rows first
    const int h = blockIdx.y, kvh = h / (AH / AKV);
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
    const int r0 = qt * 64 + w * 16;
    if (r0 >= S) return;
    const int row = r0 + n;
    const bool row_ok = row < S;
    const int my_last = q_pos0 + row;                            // last key this query row may see
    const int kend = min(L, q_pos0 + min(r0 + 15, S - 1) + 1);  // keys any row of this wavefront sees

    bf16x8 bq[8];
    {
        const uint4* qr = reinterpret_cast<const uint4*>(q + (size_t)h * q_head_stride + (size_t)(row_ok ? row : r0) * AD);
#pragma unroll
        for (int kb = 0; kb < 8; kb++) {
            uint4 v = qr[kb * 4 + g];
            if (!row_ok) v = make_uint4(0, 0, 0, 0);
            bq[kb] = __builtin_bit_cast(bf16x8, v);
        }
    }
    f32x4 O[16];
#pragma unroll
    for (int mt = 0; mt < 16; mt++) O[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = NEG, l_run = 0.f;

    const bf16_t* Kh = K + (size_t)kvh * k_head_stride;
    const bf16_t* Vh = VT + (size_t)kvh * AD * Lp;
    for (int k0 = 0; k0 < kend; k0 += 32) {
        f32x4 acc[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const int key = min(k0 + 16 * t + n, L - 1);
            const uint4* kr = reinterpret_cast<const uint4*>(Kh + (size_t)key * AD);
            uint4 a[8];
#pragma unroll
            for (int kb = 0; kb < 8; kb++) a[kb] = kr[kb * 4 + g];
            acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kb = 0; kb < 8; kb++)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[kb]), bq[kb], acc[t], 0, 0, 0);
        }
        float s[8], mx = NEG;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int key = k0 + 16 * t + 4 * g + r;
                s[t * 4 + r] = (key <= my_last && key < L) ? acc[t][r] * SCALE : NEG;
                mx = fmaxf(mx, s[t * 4 + r]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        const float corr = __expf(m_run - m_new);
        float p[8], ps = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            p[i] = s[i] > 0.5f * NEG ? __expf(s[i] - m_new) : 0.f;
            ps += p[i];
        }
        l_run = l_run * corr + ps;
        m_run = m_new;
        bf16x8 pb;
#pragma unroll
        for (int i = 0; i < 8; i++) pb[i] = (__bf16)p[i];
#pragma unroll
        for (int mt = 0; mt < 16; mt++) {
            const bf16_t* vr = Vh + (size_t)(16 * mt + n) * Lp + k0 + 4 * g;
            const uint2 v0 = *reinterpret_cast<const uint2*>(vr), v1 = *reinterpret_cast<const uint2*>(vr + 16);
            const bf16x8 a = __builtin_bit_cast(bf16x8, make_uint4(v0.x, v0.y, v1.x, v1.y));
            O[mt] *= corr;
            O[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb, O[mt], 0, 0, 0);
        }
    }
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (row_ok) {
        const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
        bf16_t* orow = out + (size_t)h * q_head_stride + (size_t)row * AD;
#pragma unroll
        for (int mt = 0; mt < 16; mt++) {
            const uint2 pk = make_uint2(pack_bf(O[mt][0] * inv, O[mt][1] * inv), pack_bf(O[mt][2] * inv, O[mt][3] * inv));
            *reinterpret_cast<uint2*>(orow + 16 * mt + 4 * g) = pk;
        }
    }
}

}  // namespace

extern "C" {

// bytes of the transposed-V workspace for L keys
long qt_gqa_prefill_workspace_bytes(int L) { return L < 0 ? -1 : (long)AKV * AD * (((long)L + 63) / 64 * 64) * 2; }

// q, out [8][S][256] bf16 (head stride q_head_stride elements), K, V [2][>=L][256] bf16 (head stride kv_head_stride):
// query i sits at absolute position q_pos0 + i and sees keys 0 .. q_pos0 + i (< L).
int qt_gqa_prefill_causal(const void* q, const void* K, const void* V, void* out, void* workspace, long workspace_bytes, int S,
                          int L, int q_pos0, long q_head_stride, long kv_head_stride, hipStream_t stream) {
    if (!q || !K || !V || !out || !workspace) return QT_ERR_NULL;
    if (S < 0 || L < 1 || q_pos0 < 0 || q_head_stride < (long)S * AD || kv_head_stride < (long)L * AD) return QT_ERR_DIM;
    if (S == 0) return QT_OK;
    for (const void* p : {q, K, V, (const void*)out, (const void*)workspace})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    if ((q_head_stride | kv_head_stride) & 7) return QT_ERR_ALIGN;
    if (workspace_bytes < qt_gqa_prefill_workspace_bytes(L)) return -6;
    const int Lp = (L + 63) / 64 * 64;
    hipLaunchKernelGGL(transpose_v_kernel, dim3(Lp / 64, AD / 64, AKV), dim3(256), 0, stream, (const bf16_t*)V, (bf16_t*)workspace, L,
                       Lp, kv_head_stride);
    hipLaunchKernelGGL(attn_prefill_kernel, dim3((S + 63) / 64, AH), dim3(256), 0, stream, (const bf16_t*)q, (const bf16_t*)K,
                       (const bf16_t*)workspace, (bf16_t*)out, S, L, Lp, q_pos0, q_head_stride, kv_head_stride);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

}  // extern "C"
