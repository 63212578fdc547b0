// The projections either side of the GatedDeltaNet / attention core at decode and verify time, for gfx950: y = W . f(x) for a
// handful of rows (M <= a few hundred), W [N, K] bf16 row-major.  Replaces the reference's fused_gemv (qwen35/kernels.py:80-319)
// and its stand-alone prologue rms_rows (qwen35/batch.py:249-301); the gated-norm prologue is the existing gated RMSNorm kernel.
//     prologue  rms:    x' = BF(nw * (x * inv)),  inv = rsqrt(mean(x^2) + eps)                       (kernels.py:106-131)
//     product           s[m][n] = sum_k W[n][k] x'[m][k]                      fp32 accumulation       (kernels.py:249-262)
//     epilogue  none:   y = bf16(s)                                                                     (kernels.py:153-160)
//               add:    y = bf16(BF(s) + res)                                                           (kernels.py:161-169)
//               swiglu: y[m][p] = bf16(silu_bf16(BF(s[m][2p])) * BF(s[m][2p+1]))   interleaved rows     (kernels.py:170-182)
// The batch is small, so the product is bound by streaming W once from HBM.  General form: one workgroup owns 16 output
// features and all rows (64 per pass); its wavefronts split K, each feeding 16x16x32 bf16 MFMAs straight from global memory (a
// W fragment is 16 features x 32 k, an x fragment 16 rows x 32 k: both are 16-byte row-contiguous loads per lane), and the
// partial sums meet in LDS.  The wide projections of a decode batch (K = 1024, 4 to 64 rows) keep the rows in LDS instead and
// give every wavefront a feature block with all of its K (xlds_gemm_kernel): what bounds such a launch is the bytes one CU
// has to pull in, its share of W plus ALL of x.  Arithmetic contract of rms_rows: sum of squares exact, rounded to float once; inv = correctly
// rounded 1/sqrt(ss / K + eps); t = x * inv and w * t rounded to float separately, then to bf16.
#include "qt_common.h"

using namespace qt;

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// one wavefront per row, four rows per workgroup: lane l owns elements 8 (l + 64 c) .. + 8 of chunk c
__global__ __launch_bounds__(256) void rms_rows_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ nw,
                                                       bf16_t* __restrict__ y, int M, int K, float eps) {
    const int m = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (m >= M) return;
    const u32x4* xr = reinterpret_cast<const u32x4*>(x + (size_t)m * K);
    const u32x4* wr = reinterpret_cast<const u32x4*>(nw);
    u32x4* yr = reinterpret_cast<u32x4*>(y + (size_t)m * K);
    const int nvec = K / 8;
    double ss = 0.0;
    for (int i = lane; i < nvec; i += 64) {
        const u32x4 v = xr[i];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const double lo = (double)__uint_as_float(v[j] << 16), hi = (double)__uint_as_float(v[j] & 0xffff0000u);
            ss += lo * lo + hi * hi;
        }
    }
    ss = wave_sum_d(ss);
    const float inv = rsqrt_rn((float)ss / (float)K + eps);
    for (int i = lane; i < nvec; i += 64) {
        const u32x4 v = xr[i], wv = wr[i];
        u32x4 o;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float lo = __fmul_rn(__uint_as_float(wv[j] << 16), __fmul_rn(__uint_as_float(v[j] << 16), inv));
            const float hi = __fmul_rn(__uint_as_float(wv[j] & 0xffff0000u), __fmul_rn(__uint_as_float(v[j] & 0xffff0000u), inv));
            o[j] = pack_bf(lo, hi);
        }
        yr[i] = o;
    }
}

constexpr int EPI_NONE = 0, EPI_ADD = 1, EPI_SWIGLU = 2;
constexpr int MT = 64;                 // most rows a workgroup takes
constexpr int G = 2;                   // k chunks (of 32) per register batch

// One workgroup = 16 output features x 16 MS rows; its NWV wavefronts split K.  grid = (ceil(N / 16), ceil(M / 16 MS)).
// K / 32 is a multiple of G NWV: every wavefront gets a whole number of batches of G chunks.  At most 128 registers, so that
// four workgroups of four wavefronts (or one of sixteen) share a CU: 514 workgroups of the widest projection (N = 8224) are
// resident at once, and the narrow ones (N = 1024: 64 workgroups) get short K chains from sixteen wavefronts each.
// MS = 16-row blocks per workgroup (1, 2 or 4; rows past M repeat the last row and are dropped): a compile-time count keeps
// the MFMA sequence free of branches, and a small one spreads a narrow output over more workgroups.
template <int NWV, int MS, int EPI>
__global__ __launch_bounds__(64 * NWV, 16 / NWV) void skinny_gemm_kernel(const bf16_t* __restrict__ W, const bf16_t* __restrict__ x,
                                                                         const bf16_t* __restrict__ res, bf16_t* __restrict__ y, int M, int N,
                                                                         int K) {
    __shared__ float red[NWV][16][16 * MS + 1];
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16, m0 = blockIdx.y * (16 * MS);
    const int kc_w = K / 32 / NWV;                                // chunks of this wavefront
    const int k_base = w * kc_w * 32 + 8 * g;
    // lane (n, g) loads feature n0 + n and row m0 + 16 ms + n, elements k + 8 g .. + 8; rows past the end repeat the last
    const bf16_t* wp = W + (size_t)min(n0 + n, N - 1) * K + k_base;
    const bf16_t* xp[MS];
#pragma unroll
    for (int ms = 0; ms < MS; ms++) xp[ms] = x + (size_t)min(m0 + 16 * ms + n, M - 1) * K + k_base;

    f32x4 acc[MS];
#pragma unroll
    for (int ms = 0; ms < MS; ms++) acc[ms] = f32x4{0.f, 0.f, 0.f, 0.f};
    u32x4 a[2][G], b[2][G][MS];
    auto load = [&](int buf, int c0) {
#pragma unroll
        for (int c = 0; c < G; c++) {
            a[buf][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp + (c0 + c) * 32));   // W is read once
#pragma unroll
            for (int ms = 0; ms < MS; ms++) b[buf][c][ms] = *reinterpret_cast<const u32x4*>(xp[ms] + (c0 + c) * 32);
        }
    };
    auto mma = [&](int buf) {
#pragma unroll
        for (int c = 0; c < G; c++)
#pragma unroll
            for (int ms = 0; ms < MS; ms++)
                acc[ms] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[buf][c]),
                                                                 __builtin_bit_cast(bf16x8, b[buf][c][ms]), acc[ms], 0, 0, 0);
    };
    load(0, 0);
    for (int c0 = 0; c0 < kc_w; c0 += 2 * G) {                    // two batches per trip: the next one loads while this one multiplies
        if (c0 + G < kc_w) load(1, c0 + G);
        mma(0);
        if (c0 + G < kc_w) {
            if (c0 + 2 * G < kc_w) load(0, c0 + 2 * G);
            mma(1);
        }
    }
    // accumulator element i of lane (n, g) is feature 4 g + i, row 16 ms + n
#pragma unroll
    for (int ms = 0; ms < MS; ms++)
#pragma unroll
        for (int i = 0; i < 4; i++) red[w][4 * g + i][16 * ms + n] = acc[ms][i];
    __syncthreads();
    auto total = [&](int f, int m) {                              // fixed order: pairs, then pairs of pairs, ...
        float t[NWV];
#pragma unroll
        for (int i = 0; i < NWV; i++) t[i] = red[i][f][m];
#pragma unroll
        for (int st = 1; st < NWV; st *= 2)
#pragma unroll
            for (int i = 0; i < NWV; i += 2 * st) t[i] += t[i + st];
        return t[0];
    };
    if (EPI == EPI_SWIGLU) {
        for (int idx = threadIdx.x; idx < 8 * 16 * MS; idx += 64 * NWV) {
            const int p = idx % 8, m = idx / 8;
            if (m0 + m < M && n0 + 2 * p + 1 < N) {
                const float gt = BF(total(2 * p, m)), up = BF(total(2 * p + 1, m));
                y[(size_t)(m0 + m) * (N / 2) + n0 / 2 + p] = f2bf(silu_bf16(gt) * up);
            }
        }
    } else {
        for (int idx = threadIdx.x; idx < 16 * 16 * MS; idx += 64 * NWV) {
            const int f = idx % 16, m = idx / 16;
            if (m0 + m < M && n0 + f < N) {
                const size_t o = (size_t)(m0 + m) * N + n0 + f;
                const float s = total(f, m);
                y[o] = EPI == EPI_ADD ? f2bf(BF(s) + bf2f(res[o])) : f2bf(s);
            }
        }
    }
}

// Wide outputs (N in the thousands): the rows are the expensive operand, because every workgroup reads all of x from L2.  Here
// a wavefront keeps its K range of x in registers (KCW chunks x four 16-row blocks) and walks NT feature blocks with it, so
// x is fetched once per 16 NT features and only W streams.  grid = (ceil(N / 16 NT), ceil(M / 64)), K = 32 KCW NWV.
template <int NWV, int KCW, int NT, int MS, int EPI>
__global__ __launch_bounds__(64 * NWV) void wide_gemm_kernel(const bf16_t* __restrict__ W, const bf16_t* __restrict__ x,
                                                             const bf16_t* __restrict__ res, bf16_t* __restrict__ y, int M, int N, int K) {
    __shared__ float red[NWV][16][MT + 1];
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * (16 * NT), m0 = blockIdx.y * (16 * MS);
    const int k_base = w * KCW * 32 + 8 * g;
    u32x4 a[NT][KCW], b[KCW][MS];
#pragma unroll
    for (int c = 0; c < KCW; c++)                                 // the first feature block's W rides ahead of x
        a[0][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(W + (size_t)min(n0 + n, N - 1) * K + k_base + c * 32));
#pragma unroll
    for (int ms = 0; ms < MS; ms++) {
        const bf16_t* xp = x + (size_t)min(m0 + 16 * ms + n, M - 1) * K + k_base;
#pragma unroll
        for (int c = 0; c < KCW; c++) b[c][ms] = *reinterpret_cast<const u32x4*>(xp + c * 32);
    }
#pragma unroll
    for (int nt = 1; nt < NT; nt++)
#pragma unroll
        for (int c = 0; c < KCW; c++)
            a[nt][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(W + (size_t)min(n0 + 16 * nt + n, N - 1) * K + k_base + c * 32));
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
        f32x4 acc[MS];
#pragma unroll
        for (int ms = 0; ms < MS; ms++) acc[ms] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KCW; c++)
#pragma unroll
            for (int ms = 0; ms < MS; ms++)
                acc[ms] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[nt][c]),
                                                                 __builtin_bit_cast(bf16x8, b[c][ms]), acc[ms], 0, 0, 0);
        if (nt) __syncthreads();                                  // the previous block's sums have been read
#pragma unroll
        for (int ms = 0; ms < MS; ms++)
#pragma unroll
            for (int i = 0; i < 4; i++) red[w][4 * g + i][16 * ms + n] = acc[ms][i];
        __syncthreads();
        auto total = [&](int f, int m) {                          // fixed order: pairs, then pairs of pairs, ...
            float t[NWV];
#pragma unroll
            for (int i = 0; i < NWV; i++) t[i] = red[i][f][m];
#pragma unroll
            for (int st = 1; st < NWV; st *= 2)
#pragma unroll
                for (int i = 0; i < NWV; i += 2 * st) t[i] += t[i + st];
            return t[0];
        };
        const int nb = n0 + 16 * nt;
        if (EPI == EPI_SWIGLU) {
            for (int idx = threadIdx.x; idx < 8 * 16 * MS; idx += 64 * NWV) {
                const int p = idx % 8, m = idx / 8;
                if (m0 + m < M && nb + 2 * p + 1 < N) {
                    const float gt = BF(total(2 * p, m)), up = BF(total(2 * p + 1, m));
                    y[(size_t)(m0 + m) * (N / 2) + nb / 2 + p] = f2bf(silu_bf16(gt) * up);
                }
            }
        } else {
            for (int idx = threadIdx.x; idx < 16 * 16 * MS; idx += 64 * NWV) {
                const int f = idx % 16, m = idx / 16;
                if (m0 + m < M && nb + f < N) {
                    const size_t o = (size_t)(m0 + m) * N + nb + f;
                    const float s = total(f, m);
                    y[o] = EPI == EPI_ADD ? f2bf(BF(s) + bf2f(res[o])) : f2bf(s);
                }
            }
        }
    }
}

// K = 1024, wide outputs: the rows live in LDS, shared by the whole workgroup, and a wavefront owns a feature block with all
// of its K, so nothing is summed across wavefronts.  x [16 MS rows][1024] goes HBM / L2 -> LDS directly (global_load_lds: one
// instruction lands half a row, 1 KiB, contiguously), its 16-byte chunks XOR-swizzled by the row number (the loading lane
// fetches the chunk that belongs at its position) so that the fragment reads of 16 rows fall on distinct banks.  The
// wavefront's W block [16 features][1024] is 32 loads, all issued up front (128 registers); every W fragment then meets MS
// x fragments read from LDS.  Accumulator element i of lane (n, g) is feature 4 g + i of row 16 ms + n: four adjacent
// features, stored as 8 bytes.  grid = ceil(N / (16 WPB)), block = 64 WPB.
// With `full` > 0 the launch is one workgroup for every CU whatever N: wavefronts 0 .. WPB - 2 of workgroup i take feature
// blocks (WPB - 1) i + w, and the last wavefront takes block `full` + i, which exists in the first few workgroups only (the
// 514 blocks of N = 8224 are 2 x 256 + 2: with three blocks per workgroup 84 of 256 CUs would have none, and what bounds the
// launch is the bytes one CU has to pull in).  A wavefront without a block still helps to bring in the rows.
constexpr int XK = 1024;
template <int MS, int WPB, int EPI>
__global__ __launch_bounds__(64 * WPB) void xlds_gemm_kernel(const bf16_t* __restrict__ W, const bf16_t* __restrict__ x,
                                                        const bf16_t* __restrict__ res, bf16_t* __restrict__ y, int M, int N, int full) {
    __shared__ __align__(1024) bf16_t x_s[16 * MS * XK];
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
    // this wavefront's feature block (may lie past N: then it multiplies a copy of the last row block and stores nothing)
    const int n0 = 16 * (full <= 0 ? blockIdx.x * WPB + w : w < WPB - 1 ? blockIdx.x * (WPB - 1) + w : full + blockIdx.x);
    // W first (it comes from HBM): the wavefront's block is 32 loads, all in flight at once
    u32x4 a[XK / 32];
    const bool has_block = n0 < N;                                // (the same for the whole wavefront)
    if (has_block) {
        const bf16_t* wp = W + (size_t)min(n0 + n, N - 1) * XK + 8 * g;
#pragma unroll
        for (int c = 0; c < XK / 32; c++) a[c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp + 32 * c));
    }
    // x -> LDS: half-row h (of 2 * 16 MS) by wavefront h % WPB; lane l lands at chunk position 64 (h & 1) + l of row h >> 1
    // (every workgroup reads the same rows at the same time; starting each at another half-row changed nothing)
    for (int h = w; h < 32 * MS; h += WPB) {
        const int r = h >> 1, cp = 64 * (h & 1) + lane;
        const bf16_t* src = x + (size_t)min(r, M - 1) * XK + 8 * (cp ^ (r & 15));
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)(x_s + h * 512), 16, 0, 0);
    }
    // (a direct-to-LDS load in flight makes the compiler wait for every outstanding load before the first use of any, so the
    // products cannot start under the tail of the W stream; both streams are drained here)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (!has_block) return;                                       // it has done its share of the rows
    f32x4 acc[MS];
#pragma unroll
    for (int ms = 0; ms < MS; ms++) acc[ms] = f32x4{0.f, 0.f, 0.f, 0.f};
    // x fragments are read two chunks ahead of their MFMAs (a ring of three), the scheduler pinned
    auto x_frag = [&](int c, int ms) {
        return *reinterpret_cast<const u32x4*>(x_s + (16 * ms + n) * XK + 8 * ((4 * c + g) ^ n));
    };
    u32x4 b[3][MS];
#pragma unroll
    for (int ms = 0; ms < MS; ms++) b[0][ms] = x_frag(0, ms), b[1][ms] = x_frag(1, ms);
#pragma unroll
    for (int c = 0; c < XK / 32; c++) {
        __builtin_amdgcn_sched_barrier(0);
        if (c + 2 < XK / 32) {
#pragma unroll
            for (int ms = 0; ms < MS; ms++) b[(c + 2) % 3][ms] = x_frag(c + 2, ms);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ms = 0; ms < MS; ms++)
            acc[ms] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[c]), __builtin_bit_cast(bf16x8, b[c % 3][ms]),
                                                             acc[ms], 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    const int f0 = n0 + 4 * g;                                    // first of this lane's four features (N is a multiple of 4)
    if (f0 >= N) return;                                          // (also a wavefront whose whole block lies past N)
#pragma unroll
    for (int ms = 0; ms < MS; ms++) {
        const int m = 16 * ms + n;
        if (m >= M) continue;
        if (EPI == EPI_SWIGLU) {
            const float g0 = BF(acc[ms][0]), u0 = BF(acc[ms][1]), g1 = BF(acc[ms][2]), u1 = BF(acc[ms][3]);
            *reinterpret_cast<uint32_t*>(y + (size_t)m * (N / 2) + f0 / 2) = pack_bf(silu_bf16(g0) * u0, silu_bf16(g1) * u1);
        } else {
            const size_t o = (size_t)m * N + f0;
            float v[4] = {acc[ms][0], acc[ms][1], acc[ms][2], acc[ms][3]};
            if (EPI == EPI_ADD) {
                const uint2 rr = *reinterpret_cast<const uint2*>(res + o);
                v[0] = BF(v[0]) + lo_bf(rr.x), v[1] = BF(v[1]) + hi_bf(rr.x), v[2] = BF(v[2]) + lo_bf(rr.y), v[3] = BF(v[3]) + hi_bf(rr.y);
            }
            *reinterpret_cast<uint2*>(y + o) = make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3]));
        }
    }
}

template <int MS, int WPB>
void launch_xlds_wpb(int epi, const bf16_t* W, const bf16_t* x, const bf16_t* res, bf16_t* y, int M, int N, hipStream_t stream, int grid_x,
                     int full) {
    const dim3 grid(grid_x), block(64 * WPB);
    if (epi == EPI_NONE)
        hipLaunchKernelGGL((xlds_gemm_kernel<MS, WPB, EPI_NONE>), grid, block, 0, stream, W, x, res, y, M, N, full);
    else if (epi == EPI_ADD)
        hipLaunchKernelGGL((xlds_gemm_kernel<MS, WPB, EPI_ADD>), grid, block, 0, stream, W, x, res, y, M, N, full);
    else
        hipLaunchKernelGGL((xlds_gemm_kernel<MS, WPB, EPI_SWIGLU>), grid, block, 0, stream, W, x, res, y, M, N, full);
}
template <int MS>
void launch_xlds_ms(int epi, const bf16_t* W, const bf16_t* x, const bf16_t* res, bf16_t* y, int M, int N, hipStream_t stream, int cus) {
    // as few wavefronts per workgroup as keep the launch within one workgroup per CU (the rows take most of a CU's LDS)
    const int blocks = (N + 15) / 16, wpb = (blocks + cus - 1) / cus;
    // a few blocks more than a whole number per CU: every CU gets that number, the first few workgroups one more
    const int base = blocks / cus, rest = blocks - base * cus;
    if (base >= 1 && base <= 3 && rest > 0 && rest <= cus / 16) {
        const int full = base * cus;
        if (base == 1)
            launch_xlds_wpb<MS, 2>(epi, W, x, res, y, M, N, stream, cus, full);
        else if (base == 2)
            launch_xlds_wpb<MS, 3>(epi, W, x, res, y, M, N, stream, cus, full);
        else
            launch_xlds_wpb<MS, 4>(epi, W, x, res, y, M, N, stream, cus, full);
        return;
    }
    if (wpb <= 2)
        launch_xlds_wpb<MS, 2>(epi, W, x, res, y, M, N, stream, (blocks + 1) / 2, 0);
    else if (wpb == 3)
        launch_xlds_wpb<MS, 3>(epi, W, x, res, y, M, N, stream, (blocks + 2) / 3, 0);
    else
        launch_xlds_wpb<MS, 4>(epi, W, x, res, y, M, N, stream, (blocks + 3) / 4, 0);
}

// row blocks per pass: 1, 2 or 4 (3 rounds up)
inline int row_blocks(int M) { return M <= 16 ? 1 : M <= 32 ? 2 : 4; }

template <int NWV, int KCW, int NT, int MS>
void launch_wide_ms(int epi, const bf16_t* W, const bf16_t* x, const bf16_t* res, bf16_t* y, int M, int N, int K, hipStream_t stream) {
    const dim3 grid((N + 16 * NT - 1) / (16 * NT), (M + 16 * MS - 1) / (16 * MS)), block(64 * NWV);
    if (epi == EPI_NONE)
        hipLaunchKernelGGL((wide_gemm_kernel<NWV, KCW, NT, MS, EPI_NONE>), grid, block, 0, stream, W, x, res, y, M, N, K);
    else if (epi == EPI_ADD)
        hipLaunchKernelGGL((wide_gemm_kernel<NWV, KCW, NT, MS, EPI_ADD>), grid, block, 0, stream, W, x, res, y, M, N, K);
    else
        hipLaunchKernelGGL((wide_gemm_kernel<NWV, KCW, NT, MS, EPI_SWIGLU>), grid, block, 0, stream, W, x, res, y, M, N, K);
}
template <int NWV, int KCW, int NT>
void launch_wide(int epi, const bf16_t* W, const bf16_t* x, const bf16_t* res, bf16_t* y, int M, int N, int K, hipStream_t stream) {
    if (row_blocks(M) == 2)
        launch_wide_ms<NWV, KCW, NT, 2>(epi, W, x, res, y, M, N, K, stream);
    else
        launch_wide_ms<NWV, KCW, NT, 4>(epi, W, x, res, y, M, N, K, stream);
}

template <int NWV, int MS>
void launch_gemm_ms(int epi, const bf16_t* W, const bf16_t* x, const bf16_t* res, bf16_t* y, int M, int N, int K, hipStream_t stream) {
    const dim3 grid((N + 15) / 16, (M + 16 * MS - 1) / (16 * MS)), block(64 * NWV);
    if (epi == EPI_NONE)
        hipLaunchKernelGGL((skinny_gemm_kernel<NWV, MS, EPI_NONE>), grid, block, 0, stream, W, x, res, y, M, N, K);
    else if (epi == EPI_ADD)
        hipLaunchKernelGGL((skinny_gemm_kernel<NWV, MS, EPI_ADD>), grid, block, 0, stream, W, x, res, y, M, N, K);
    else
        hipLaunchKernelGGL((skinny_gemm_kernel<NWV, MS, EPI_SWIGLU>), grid, block, 0, stream, W, x, res, y, M, N, K);
}
// narrow: the output has few feature blocks, so fewer rows per workgroup (more workgroups) pay for re-reading W from L2
template <int NWV>
void launch_gemm(int epi, const bf16_t* W, const bf16_t* x, const bf16_t* res, bf16_t* y, int M, int N, int K, hipStream_t stream,
                 bool narrow) {
    int ms = row_blocks(M);
    while (narrow && ms > 1 && (long)((N + 15) / 16) * ((M + 16 * ms - 1) / (16 * ms)) < 256) ms /= 2;
    switch (ms) {
        case 1: launch_gemm_ms<NWV, 1>(epi, W, x, res, y, M, N, K, stream); break;
        case 2: launch_gemm_ms<NWV, 2>(epi, W, x, res, y, M, N, K, stream); break;
        default: launch_gemm_ms<NWV, 4>(epi, W, x, res, y, M, N, K, stream);
    }
}


}  // namespace

extern "C" {

// y [M, K] bf16 = rms prologue of x [M, K] bf16 with weight nw [K] bf16.  K a multiple of 8.
int qt_rms_rows(const void* x, const void* nw, void* y, int M, int K, float eps, hipStream_t stream) {
    if (M < 0 || K < 8 || (K & 7)) return QT_ERR_DIM;
    if (M == 0) return QT_OK;                                     // nothing to do: empty buffers may be null
    if (!x || !nw || !y) return QT_ERR_NULL;
    for (const void* p : {x, nw, (const void*)y})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    hipLaunchKernelGGL(rms_rows_kernel, dim3((M + 3) / 4), dim3(256), 0, stream, (const bf16_t*)x, (const bf16_t*)nw, (bf16_t*)y, M, K, eps);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

// y = epilogue(W [N, K] . x [M, K]^T): epilogue 0 none (y [M, N]), 1 add (res [M, N], y [M, N]), 2 swiglu (y [M, N / 2], N even).
// K a multiple of 256.
int qt_fused_gemv(const void* W, const void* x, const void* res, void* y, int M, int N, int K, int epilogue, hipStream_t stream) {
    if (epilogue < 0 || epilogue > 2) return QT_ERR_UNSUPPORTED;
    if (M < 0 || N < 1 || K < 256 || (K % 256) || (epilogue == EPI_SWIGLU && (N & 1))) return QT_ERR_DIM;
    if (M == 0) return QT_OK;                                     // nothing to do: empty buffers may be null
    if (!W || !x || !y || (epilogue == EPI_ADD && !res)) return QT_ERR_NULL;
    for (const void* p : {W, x})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    // wavefronts per workgroup: 4 when the output is wide enough to fill the chip with workgroups; 16 or 8 (as K divides) for
    // the narrow outputs, whose few workgroups would otherwise walk long K chains
    const int kc = K / 32;
    // the wide projections of a decode batch: rows in LDS.  From four rows on (in_proj, one row 6.6 us either way; 4 / 16 /
    // 64 rows: 6.9 / 7.0 / 9.7 us against 7.0 / 8.4 / 11.9 us for the kernels below)
    // (its 8-byte stores and residual loads want y and res aligned to 8 bytes; anything else takes the general kernels)
    if (K == XK && N >= 4096 && (N & 3) == 0 && M >= 4 && M <= 64 &&
        ((reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(res)) & 7u) == 0) {
        const int cus = cu_count();
        if (M <= 16)
            launch_xlds_ms<1>(epilogue, (const bf16_t*)W, (const bf16_t*)x, (const bf16_t*)res, (bf16_t*)y, M, N, stream, cus);
        else if (M <= 32)
            launch_xlds_ms<2>(epilogue, (const bf16_t*)W, (const bf16_t*)x, (const bf16_t*)res, (bf16_t*)y, M, N, stream, cus);
        else
            launch_xlds_ms<4>(epilogue, (const bf16_t*)W, (const bf16_t*)x, (const bf16_t*)res, (bf16_t*)y, M, N, stream, cus);
        QT_CHECK_LAUNCH();
        return QT_OK;
    }
    if (K == 1024 && N >= 4096 && M > 16) {                       // ... of more than 64 rows: x stays in registers
        // three feature blocks per workgroup (172 workgroups for 8224 features): four leave half the CUs without one, two
        // double what the workgroups pull of x from L2; measured 13.2 / 11.7 / 16.3 us for 4 / 3 / 2 at 64 rows
        launch_wide<8, 4, 3>(epilogue, (const bf16_t*)W, (const bf16_t*)x, (const bf16_t*)res, (bf16_t*)y, M, N, K, stream);
        QT_CHECK_LAUNCH();
        return QT_OK;
    }
    const bool wide = (long)((N + 15) / 16) * ((M + MT - 1) / MT) >= 512;
    if (!wide && kc % (2 * 16) == 0)
        launch_gemm<16>(epilogue, (const bf16_t*)W, (const bf16_t*)x, (const bf16_t*)res, (bf16_t*)y, M, N, K, stream, true);
    else if (!wide && kc % (2 * 8) == 0)
        launch_gemm<8>(epilogue, (const bf16_t*)W, (const bf16_t*)x, (const bf16_t*)res, (bf16_t*)y, M, N, K, stream, true);
    else
        launch_gemm<4>(epilogue, (const bf16_t*)W, (const bf16_t*)x, (const bf16_t*)res, (bf16_t*)y, M, N, K, stream, !wide);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

}  // extern "C"
