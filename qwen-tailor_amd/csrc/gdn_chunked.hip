// Chunked (WY / UT transform) GatedDeltaNet prefill for gfx950, chunk size C = 64.
// Replaces the Metal kernels gdn_nax_a / gdn_nax_prep_a / gdn_nax_b (qwen35/gdn_nax.py:71-358), whose chunk is 16.
//
// Per head and chunk, with S0 [dv,dk] the state entering the chunk (gdn_nax.py:3-10):
//     Lc = cumsum(log g), gamma = exp(Lc), dec = exp(Lc_C - Lc), G_ij = exp(Lc_i - Lc_j)
//     L  = strict_lower(beta_i G_ij K K^T),  Tb = (I + L)^-1 diag(beta),  A = lower_incl(G * Q K^T)
//     D  = Tb (V - gamma * (K S0^T)),   Y = gamma * (Q S0^T) + A D,   S1 = gamma_C S0 + (dec * D)^T K
// Phase A (parallel over (chunk, head)) folds everything that does not depend on the state into MFMA operands
//     Wn = -Tb (gamma * K),  U = Tb V,  Qg = gamma * Q,  Kd = (dec * K)^T,  Am = A
// so that the serial phase B is four register-resident GEMMs per chunk:
//     D = U + Wn S0^T;   Y = Qg S0^T + Am D;   S1^T = gamma_C S0^T + Kd D.
//
// Phase B runs one wavefront per (head, 16-wide dv slice).  The state slice S^T [128 dk x 16 dv] lives in the MFMA
// accumulator layout (lane (n, g): rows 4g..4g+3 of column n); an accumulator pair, converted to half precision, IS the
// B operand of the next 16x16x32 MFMA if the contraction index is enumerated as
//     kperm(kb, g, j) = 32 kb + 16 (j >> 2) + 4 g + (j & 3),
// so phase A stores every A operand with its k index permuted the same way and the state never leaves the registers.
// Intermediate operands are fp16 (11-bit significand); accumulation and the carried state are fp32.
#include "qt_common.h"

using namespace qt;

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int C = 64;                           // chunk size
constexpr int NCT = C / 16;                     // 16-row tiles along the chunk
constexpr int OP_W = 0;                         // offsets (in halves) of the operands inside one (chunk, head) record
constexpr int OP_Q = OP_W + NCT * 4 * 512;      // Wn: [ct 4][kb 4][lane 64][8]
constexpr int OP_K = OP_Q + NCT * 4 * 512;      // Qg: same;  Kd: [mt 8][kb2 2][64][8]
constexpr int OP_A = OP_K + 8 * 2 * 512;        // Am: [ct 4][kb2 2][64][8]
constexpr int OP_HALVES = OP_A + NCT * 2 * 512; // 28672 halves = 56 KiB per (chunk, head)
constexpr int U_FLOATS = 8 * NCT * 64 * 4;      // U: [slice 8][ct 4][lane 64][4] f32 = 32 KiB per (chunk, head)

__device__ __forceinline__ half8 pack_half8(const f32x4& a, const f32x4& b) {
    half8 h;
    h[0] = (_Float16)a[0]; h[1] = (_Float16)a[1]; h[2] = (_Float16)a[2]; h[3] = (_Float16)a[3];
    h[4] = (_Float16)b[0]; h[5] = (_Float16)b[1]; h[6] = (_Float16)b[2]; h[7] = (_Float16)b[3];
    return h;
}

// Phase B: serial over the chunks.  grid = 128 wavefronts (head, dv slice); ops / U / gC are phase A's records.
__global__ __launch_bounds__(64) void gdn_phase_b_kernel(const _Float16* __restrict__ ops, const float* __restrict__ U,
                                                         const float* __restrict__ gC, const float* __restrict__ st_in,
                                                         float* __restrict__ st_out, bf16_t* __restrict__ y, int S, int NC) {
    // heads that share an XCD's L2 keep their 8 slices there: workgroup id = xcd + 8 k, head = xcd + 8 (k / 8), slice = k % 8
    const int xcd = blockIdx.x & 7, kq = blockIdx.x >> 3;
    const int h = xcd + 8 * (kq >> 3), sl = kq & 7;
    const int lane = threadIdx.x, n = lane & 15, g = lane >> 4;

    f32x4 ST[8];
    {
        const float* sp = st_in + ((size_t)h * DV + sl * 16 + n) * DK;          // S[h][dv][dk], dk contiguous
#pragma unroll
        for (int mt = 0; mt < 8; mt++) ST[mt] = *reinterpret_cast<const f32x4*>(sp + mt * 16 + 4 * g);
    }
    for (int c = 0; c < NC; c++) {
        const size_t rec = (size_t)c * HV + h;
        const half8* op = reinterpret_cast<const half8*>(ops + rec * OP_HALVES) + lane;
        const f32x4* up = reinterpret_cast<const f32x4*>(U + rec * U_FLOATS + (size_t)sl * NCT * 256) + lane;
        const float gc = gC[rec];

        half8 Sb[4];
#pragma unroll
        for (int kb = 0; kb < 4; kb++) Sb[kb] = pack_half8(ST[2 * kb], ST[2 * kb + 1]);

        f32x4 D[NCT], Y[NCT];
#pragma unroll
        for (int ct = 0; ct < NCT; ct++) {
            D[ct] = up[ct * 64];
            Y[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kb = 0; kb < 4; kb++) {
                D[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(op[(OP_W / 8) + (ct * 4 + kb) * 64], Sb[kb], D[ct], 0, 0, 0);
                Y[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(op[(OP_Q / 8) + (ct * 4 + kb) * 64], Sb[kb], Y[ct], 0, 0, 0);
            }
        }
        half8 Db[2];
        Db[0] = pack_half8(D[0], D[1]);
        Db[1] = pack_half8(D[2], D[3]);
#pragma unroll
        for (int mt = 0; mt < 8; mt++) {
            ST[mt] *= gc;
#pragma unroll
            for (int kb2 = 0; kb2 < 2; kb2++)
                ST[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(op[(OP_K / 8) + (mt * 2 + kb2) * 64], Db[kb2], ST[mt], 0, 0, 0);
        }
#pragma unroll
        for (int ct = 0; ct < NCT; ct++) {
#pragma unroll
            for (int kb2 = 0; kb2 < 2; kb2++)
                Y[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(op[(OP_A / 8) + (ct * 2 + kb2) * 64], Db[kb2], Y[ct], 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int t = c * C + ct * 16 + 4 * g + r;
                if (t < S) y[((size_t)t * HV + h) * DV + sl * 16 + n] = f2bf(Y[ct][r]);
            }
        }
    }
    {
        float* sp = st_out + ((size_t)h * DV + sl * 16 + n) * DK;
#pragma unroll
        for (int mt = 0; mt < 8; mt++) *reinterpret_cast<f32x4*>(sp + mt * 16 + 4 * g) = ST[mt];
    }
}

}  // namespace

extern "C" {

// sizes (bytes) of the phase A -> phase B buffers for S tokens: ops, U, gC
long qt_gdn_chunk_ops_bytes(int S) { return S < 0 ? -1 : (long)((S + C - 1) / C) * HV * OP_HALVES * 2; }
long qt_gdn_chunk_u_bytes(int S) { return S < 0 ? -1 : (long)((S + C - 1) / C) * HV * U_FLOATS * 4; }
long qt_gdn_chunk_gc_bytes(int S) { return S < 0 ? -1 : (long)((S + C - 1) / C) * HV * 4; }

int qt_gdn_phase_b(const void* ops, const float* U, const float* gC, const float* state_in, float* state_out, void* y, int S,
                   hipStream_t stream) {
    if (!ops || !U || !gC || !state_in || !state_out || !y) return QT_ERR_NULL;
    if (S < 0) return QT_ERR_DIM;
    for (const void* p : {ops, (const void*)U, (const void*)state_in, (const void*)state_out})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    const int NC = (S + C - 1) / C;
    hipLaunchKernelGGL(gdn_phase_b_kernel, dim3(HV * 8), dim3(64), 0, stream, (const _Float16*)ops, U, gC, state_in, state_out,
                       (bf16_t*)y, S, NC);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

}  // extern "C"
