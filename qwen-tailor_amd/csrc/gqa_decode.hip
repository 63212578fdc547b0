// Ragged GQA decode / verify attention, head dim 256, 8 query heads on 2 KV heads, for gfx950.
// Replaces the Metal kernel attn_b_{Lmax}_m{M} (qwen35/batch.py:141-237): row r = b*M + j of the batch sits at position
// pos[b] + j of slot slots[b]; it attends the pool keys below pos[b] and the new keys of rows b*M .. b*M + j, which are
// read from the inputs (never from the pool) and appended to the pool at pos[b] + j.
//
// Split-K: workgroup (b, kv head, split s) streams the pool keys [s*CH, min((s+1)*CH, pos[b])) ONCE for all 4*M query
// rows that share the KV head, so K and V are read from HBM exactly once per step.
//   scores : S^T[16 keys x 16 rows] = K_tile[16 x 256] . Q^T[256 x 16] on bf16 MFMA (16x16x32), K straight from HBM
//   P . V  : on the vector ALU, lane l owns output columns 4l .. 4l+3 of every row; probabilities are broadcast through LDS
// Each wavefront keeps its own online-softmax state (m, l, O); the 4 wavefronts of a workgroup are merged through LDS and
// the workgroup writes one unnormalised partial (m, l, O) per row; a second kernel merges the splits (batch.py:203-221).
#include "qt_common.h"

using namespace qt;

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int GQA = AH / AKV;          // 4 query heads per KV head
constexpr float SCALE = 0.0625f;       // 256^-0.5, batch.py:177
constexpr float NEG = -3.0e38f;

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// One tile of up to 16 keys for one wavefront.  kt / vt point at the first key's row (256 bf16, row stride `stride`
// elements); keys [0, nvalid) exist; `causal0` >= 0 marks new keys: key i is visible to query token j only if i <= j.
template <int M>
__device__ __forceinline__ void tile_step(const bf16_t* __restrict__ kt, const bf16_t* __restrict__ vt, size_t stride, int nvalid,
                                          bool causal, const bf16x8 (&bq)[8], float& m_run, float& l_run, float (&o)[4 * M][4],
                                          float* p_lds, float* c_lds, int lane) {
    const int n = lane & 15, g = lane >> 4;
    // ---- scores, transposed: lane (row n, group g) gets keys 4g .. 4g+3
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    {
        const int key = n < nvalid ? n : 0;                      // rows past the end re-read key 0 and are masked below
        const uint4* kr = reinterpret_cast<const uint4*>(kt + (size_t)key * stride);
        uint4 a[8];
#pragma unroll
        for (int kb = 0; kb < 8; kb++) a[kb] = kr[kb * 4 + g];
#pragma unroll
        for (int kb = 0; kb < 8; kb++) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[kb]), bq[kb], acc, 0, 0, 0);
    }
    const int jq = n / GQA;                                      // query token of this row (rows >= 4*M are padding)
    float s[4], mx = NEG;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int key = 4 * g + i;
        const bool vis = key < nvalid && (!causal || key <= jq);
        s[i] = vis ? acc[i] * SCALE : NEG;
        mx = fmaxf(mx, s[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);
    const float corr = __expf(m_run - m_new);                    // m_run = NEG initially: exp(-huge) = 0
    float ps = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float p = s[i] > 0.5f * NEG ? __expf(s[i] - m_new) : 0.f;
        ps += p;
        p_lds[(4 * g + i) * 16 + n] = p;
    }
    l_run = l_run * corr + ps;                                   // this lane's share; summed over g at the end
    m_run = m_new;
    if (g == 0) c_lds[n] = corr;
    wave_lds_sync();
    // ---- O += P V, lane owns columns 4*lane .. 4*lane+3
#pragma unroll
    for (int r = 0; r < 4 * M; r += 4) {
        const f32x4 c4 = *reinterpret_cast<const f32x4*>(c_lds + r);
#pragma unroll
        for (int rr = 0; rr < 4; rr++)
#pragma unroll
            for (int e = 0; e < 4; e++) o[r + rr][e] *= c4[rr];
    }
#pragma unroll 4
    for (int key = 0; key < 16; key++) {
        if (key < nvalid) {
            const uint2 vv = reinterpret_cast<const uint2*>(vt + (size_t)key * stride)[lane];
            const float v4[4] = {lo_bf(vv.x), hi_bf(vv.x), lo_bf(vv.y), hi_bf(vv.y)};
#pragma unroll
            for (int r = 0; r < 4 * M; r += 4) {
                const f32x4 p4 = *reinterpret_cast<const f32x4*>(p_lds + key * 16 + r);
#pragma unroll
                for (int rr = 0; rr < 4; rr++)
#pragma unroll
                    for (int e = 0; e < 4; e++) o[r + rr][e] = fmaf(p4[rr], v4[e], o[r + rr][e]);
            }
        }
    }
    wave_lds_sync();
}

// partial results of one workgroup: part_o [(b*KV + kvh)*nsplit + s][4*M rows][256] f32 (unnormalised),
// part_ml [...][4*M][2] = (running max, running sum)
template <int M>
__global__ __launch_bounds__(256) void attn_partial_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_new,
                                                           const bf16_t* __restrict__ v_new, bf16_t* Kp, bf16_t* Vp,
                                                           const int* __restrict__ slots, const int* __restrict__ pos,
                                                           float* __restrict__ part_o, float* __restrict__ part_ml, int Lmax,
                                                           int CH, int nsplit, int n_slots) {
    constexpr int R = 4 * M;
    __shared__ __align__(16) float p_s[4][16 * 16];
    __shared__ __align__(16) float c_s[4][16];
    __shared__ float m_s[4][16], l_s[4][16];
    __shared__ __align__(16) float o_s[R][AD];

    const int s = blockIdx.x % nsplit, bk = blockIdx.x / nsplit, kvh = bk % AKV, b = bk / AKV;
    const int slot = slots[b], p0 = pos[b];
    if ((unsigned)slot >= (unsigned)n_slots || p0 < 0 || p0 + M > Lmax) return;
    const int lo = s * CH, hi = min(lo + CH, p0);
    if (s > 0 && lo >= p0) return;                               // nothing to do for this split (split 0 always runs)
    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;

    // Q^T as the MFMA B operand: lane (row n, group g) holds q[row n][32 kb + 8 g .. + 8]; row n = token (n / 4), head n % 4
    bf16x8 bq[8];
    {
        const bool real = n < R;
        const bf16_t* qr = q + ((size_t)(b * M + (real ? n / GQA : 0)) * AH + kvh * GQA + (n % GQA)) * AD;
#pragma unroll
        for (int kb = 0; kb < 8; kb++) {
            uint4 v = reinterpret_cast<const uint4*>(qr)[kb * 4 + g];
            if (!real) v = make_uint4(0, 0, 0, 0);
            bq[kb] = as_bf16x8(v);
        }
    }
    float m_run = NEG, l_run = 0.f, o[R][4];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int e = 0; e < 4; e++) o[r][e] = 0.f;

    const size_t pbase = ((size_t)slot * AKV + kvh) * Lmax * AD;
    const int ntiles = hi > lo ? (hi - lo + 15) / 16 : 0;
    for (int t = w; t < ntiles; t += 4) {
        const int key0 = lo + t * 16;
        tile_step<M>(Kp + pbase + (size_t)key0 * AD, Vp + pbase + (size_t)key0 * AD, AD, min(16, hi - key0), false, bq, m_run,
                     l_run, o, p_s[w], c_s[w], lane);
    }
    if (s == 0 && w == 3) {
        // the M new keys of this sequence, straight from the inputs (batch.py:143-145), with the causal tail among them
        const bf16_t* kn = k_new + ((size_t)b * M * AKV + kvh) * AD;
        const bf16_t* vn = v_new + ((size_t)b * M * AKV + kvh) * AD;
        tile_step<M>(kn, vn, (size_t)AKV * AD, M, true, bq, m_run, l_run, o, p_s[w], c_s[w], lane);
    }
    if (s == 0 && w == 0) {
        // append (batch.py:196-201): row j of this sequence goes to pool position p0 + j
        for (int j = 0; j < M; j++) {
            const uint2 kk = reinterpret_cast<const uint2*>(k_new + ((size_t)(b * M + j) * AKV + kvh) * AD)[lane];
            const uint2 vv = reinterpret_cast<const uint2*>(v_new + ((size_t)(b * M + j) * AKV + kvh) * AD)[lane];
            reinterpret_cast<uint2*>(Kp + pbase + (size_t)(p0 + j) * AD)[lane] = kk;
            reinterpret_cast<uint2*>(Vp + pbase + (size_t)(p0 + j) * AD)[lane] = vv;
        }
    }

    // ---- merge the 4 wavefronts (deterministic order)
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (g == 0) {
        m_s[w][n] = m_run;
        l_s[w][n] = l_run;
    }
    __syncthreads();
    float f[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const float mm = fmaxf(fmaxf(m_s[0][r], m_s[1][r]), fmaxf(m_s[2][r], m_s[3][r]));
        f[r] = __expf(m_s[w][r] - mm);
    }
    for (int ww = 0; ww < 4; ww++) {
        if (w == ww) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                f32x4* dst = reinterpret_cast<f32x4*>(&o_s[r][lane * 4]);
                f32x4 cur = ww == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : *dst;
                cur[0] += o[r][0] * f[r]; cur[1] += o[r][1] * f[r]; cur[2] += o[r][2] * f[r]; cur[3] += o[r][3] * f[r];
                *dst = cur;
            }
        }
        __syncthreads();
    }
    float* po = part_o + (size_t)blockIdx.x * R * AD;
    for (int i = tid; i < R * AD / 4; i += 256)
        reinterpret_cast<f32x4*>(po)[i] = reinterpret_cast<const f32x4*>(&o_s[0][0])[i];
    if (tid < R) {
        const float mm = fmaxf(fmaxf(m_s[0][tid], m_s[1][tid]), fmaxf(m_s[2][tid], m_s[3][tid]));
        float ll = 0.f;
        for (int ww = 0; ww < 4; ww++) ll += l_s[ww][tid] * __expf(m_s[ww][tid] - mm);
        part_ml[((size_t)blockIdx.x * R + tid) * 2] = mm;
        part_ml[((size_t)blockIdx.x * R + tid) * 2 + 1] = ll;
    }
}

// merge of the splits: one workgroup of 256 threads per (sequence, kv head); thread d owns output column d of every row
template <int M>
__global__ __launch_bounds__(256) void attn_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                         const int* __restrict__ slots, const int* __restrict__ pos,
                                                         bf16_t* __restrict__ out, int Lmax, int CH, int nsplit, int n_slots) {
    constexpr int R = 4 * M;
    const int kvh = blockIdx.x % AKV, b = blockIdx.x / AKV, d = threadIdx.x;
    const int slot = slots[b], p0 = pos[b];
    if ((unsigned)slot >= (unsigned)n_slots || p0 < 0 || p0 + M > Lmax) return;
    const int ns = max(1, min(nsplit, (p0 + CH - 1) / CH));
    const size_t base = (size_t)blockIdx.x * nsplit;
    for (int r = 0; r < R; r++) {
        float mm = NEG;
        for (int s = 0; s < ns; s++) mm = fmaxf(mm, part_ml[((base + s) * R + r) * 2]);
        float l = 0.f, acc = 0.f;
        for (int s = 0; s < ns; s++) {
            const float fs = __expf(part_ml[((base + s) * R + r) * 2] - mm);
            l += part_ml[((base + s) * R + r) * 2 + 1] * fs;
            acc += part_o[((base + s) * R + r) * AD + d] * fs;
        }
        const float ov = l == 0.f ? acc : acc / l;                                   // batch.py:216
        out[((size_t)(b * M + r / GQA) * AH + kvh * GQA + (r % GQA)) * AD + d] = f2bf(ov);
    }
}

}  // namespace

extern "C" {

// bytes of workspace qt_gqa_attn_decode needs for (B sequences, M rows each, pool length Lmax, split size CH)
long qt_gqa_attn_workspace_bytes(int B, int M, int Lmax, int CH) {
    if (B < 0 || M < 1 || Lmax < 1 || CH < 16) return -1;
    const long nsplit = (Lmax + CH - 1) / CH;
    return (long)B * AKV * nsplit * (4 * M) * (AD + 2) * 4;
}

int qt_gqa_attn_decode(const void* q, const void* k_new, const void* v_new, void* Kp, void* Vp, const int32_t* slots,
                       const int32_t* pos, void* out, void* workspace, long workspace_bytes, int B, int M, int Lmax,
                       int n_slots, int CH, hipStream_t stream) {
    if (!q || !k_new || !v_new || !Kp || !Vp || !slots || !pos || !out || !workspace) return QT_ERR_NULL;
    if (B < 0 || Lmax < 1 || n_slots < 1 || CH < 16 || CH % 16) return QT_ERR_DIM;
    if (M < 1 || M > 4) return QT_ERR_UNSUPPORTED;
    if (B == 0) return QT_OK;
    for (const void* p : {q, k_new, v_new, (const void*)Kp, (const void*)Vp, (const void*)workspace})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    if (workspace_bytes < qt_gqa_attn_workspace_bytes(B, M, Lmax, CH)) return -6;
    const int nsplit = (Lmax + CH - 1) / CH;
    float* part_o = (float*)workspace;
    float* part_ml = part_o + (size_t)B * AKV * nsplit * (4 * M) * AD;
    const dim3 g1((unsigned)(B * AKV * nsplit)), g2((unsigned)(B * AKV));
#define QT_ATTN_LAUNCH(MM)                                                                                                \
    hipLaunchKernelGGL(attn_partial_kernel<MM>, g1, dim3(256), 0, stream, (const bf16_t*)q, (const bf16_t*)k_new,         \
                       (const bf16_t*)v_new, (bf16_t*)Kp, (bf16_t*)Vp, slots, pos, part_o, part_ml, Lmax, CH, nsplit, n_slots); \
    hipLaunchKernelGGL(attn_merge_kernel<MM>, g2, dim3(256), 0, stream, part_o, part_ml, slots, pos, (bf16_t*)out, Lmax, CH, \
                       nsplit, n_slots);
    switch (M) {
        case 1: QT_ATTN_LAUNCH(1) break;
        case 2: QT_ATTN_LAUNCH(2) break;
        case 3: QT_ATTN_LAUNCH(3) break;
        default: QT_ATTN_LAUNCH(4) break;
    }
    QT_CHECK_LAUNCH();
    return QT_OK;
}

}  // extern "C"
