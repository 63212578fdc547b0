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

// Phase B runs in two kernels.
//
// The chain kernel is the serial part: S_{c+1}^T = gamma_c S_c^T + Kd_c D_c with D_c = U_c + Wn_c S_c^T.  It does not
// compute outputs; it leaves, per (chunk, head, slice), the two half-precision B operands that the outputs need
// (S_c^T and D_c, 6 KiB) in `snap`.  The output kernel then computes Y_c = Qg_c S_c^T + Am_c D_c for all chunks in parallel.
// Splitting the outputs off halves the bytes the serial kernel has to pull per step (W and Kd: 32 of the 56 KiB).
//
// Chain kernel: one workgroup of 5 wavefronts per (head, 16-wide dv slice).  MFMA wavefront w owns rows 16w..16w+15 of D
// (the chunk's tokens) and rows 32w..32w+31 of S^T (dk): per chunk it pulls only its 8 operand tiles (8 KiB) and keeps
// PB_DEP chunks of them in flight in registers, so the latency of a load is covered by PB_DEP chain steps.  Two exchanges
// through LDS per step make up for the split: every wavefront publishes its block of S^T as the fp16 B operand and reads
// all four (barrier E1), and publishes its rows of D and reads both k-blocks (barrier E2).  The fifth wavefront copies
// exactly these two LDS areas to `snap`: the MFMA wavefronts issue loads only, which keeps their vmcnt waits partial
// (a store in flight next to loads forces every wait to zero on this target).
constexpr int PB_DEP = 4;                        // chunks of operands in flight per MFMA wavefront
constexpr int SNAP_S = 4 * 512;                  // halves: S^T as B operand, [kb 4][lane 64][8]
constexpr int SNAP_D = 2 * 512;                  // halves: D as B operand, [kb2 2][lane 64][8]
constexpr int SNAP_HALVES = SNAP_S + SNAP_D;     // 6 KiB per (chunk, head, slice)
constexpr int KORD[4] = {0, 2, 1, 3};            // order in which a step consumes its Kd tiles (two independent accumulators)

__global__ __launch_bounds__(320) void gdn_chain_kernel(const _Float16* ops, const float* U, const float* gC, const float* st_in,
                                                        float* st_out, _Float16* snap, int NC) {
    // heads that share an XCD's L2 keep their 8 slices there: workgroup id = xcd + 8 k, head = xcd + 8 (k / 8), slice = k % 8
    const int xcd = blockIdx.x & 7, kq = blockIdx.x >> 3;
    const int h = xcd + 8 * (kq >> 3), sl = kq & 7;
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
    __shared__ __align__(16) _Float16 sb_x[SNAP_S];
    __shared__ __align__(16) _Float16 db_x[SNAP_D];
    const half8* sbx = reinterpret_cast<const half8*>(sb_x) + lane;
    const half8* dbx = reinterpret_cast<const half8*>(db_x) + lane;

    if (w == 4) {
        half8* dst = reinterpret_cast<half8*>(snap + ((size_t)h * 8 + sl) * SNAP_HALVES) + lane;
        const size_t cst = (size_t)HV * 8 * SNAP_HALVES / 8;                    // half8 per chunk
        for (int c = 0; c < NC; c++) {
            __builtin_amdgcn_s_barrier();                                       // E1: sb_x holds S_c^T
            asm volatile("" ::: "memory");
            const half8 a0 = sbx[0], a1 = sbx[64], a2 = sbx[128], a3 = sbx[192];
            dst[0] = a0;
            dst[64] = a1;
            dst[128] = a2;
            dst[192] = a3;
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();                                       // E2: db_x holds D_c
            asm volatile("" ::: "memory");
            const half8 d0 = dbx[0], d1 = dbx[64];
            dst[256] = d0;
            dst[320] = d1;
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            dst += cst;
        }
        return;
    }

    f32x4 ST[2];
    {
        const float* sp = st_in + ((size_t)h * DV + sl * 16 + n) * DK + w * 32 + 4 * g;   // S[h][dv][dk], dk contiguous
        ST[0] = *reinterpret_cast<const f32x4*>(sp);
        ST[1] = *reinterpret_cast<const f32x4*>(sp + 16);
    }
    const half8* opb = reinterpret_cast<const half8*>(ops + (size_t)h * OP_HALVES) + lane;
    const f32x4* upb = reinterpret_cast<const f32x4*>(U + (size_t)h * U_FLOATS + (size_t)(sl * NCT + w) * 256) + lane;
    const size_t ost = (size_t)HV * OP_HALVES / 8, ust = (size_t)HV * U_FLOATS / 4;
    const int wq = (OP_W / 8) + w * 4 * 64, kq0 = (OP_K / 8) + w * 4 * 64;       // W[ct = w][kb], Kd[mt = 2w + i][kb2]

    half8 Wt[PB_DEP][4], Kt[PB_DEP][4];
    f32x4 Ut[PB_DEP];
    float gct[PB_DEP];                       // the chunk's decay rides in the FIFO as one more (lane-uniform) vector load
#pragma unroll
    for (int j = 0; j < PB_DEP; j++) {                                          // same issue order as inside the steps
        const int cc = min(j, NC - 1);
#pragma unroll
        for (int i = 0; i < 4; i++) Wt[j][i] = opb[cc * ost + wq + i * 64];
        Ut[j] = upb[cc * ust];
#pragma unroll
        for (int i = 0; i < 4; i++) Kt[j][KORD[i]] = opb[cc * ost + kq0 + KORD[i] * 64];
        gct[j] = gC[(size_t)cc * HV + h];
    }
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");

    // One chain step on FIFO entry j (a compile-time index: the steps are unrolled PB_DEP at a time).  Every MFMA is
    // followed by the load that refills its operand for chunk c + PB_DEP and the scheduler is pinned to this order, so
    // loads complete in the order of their use and the waits name exact counts.
    auto step = [&](auto J, int c) {
        constexpr int j = decltype(J)::value;
        const int cn = min(c + PB_DEP, NC - 1);
        const half8* on = opb + cn * ost;
        reinterpret_cast<half8*>(sb_x)[w * 64 + lane] = pack_half8(ST[0], ST[1]);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();                                           // E1
        asm volatile("" ::: "memory");
        half8 Sb[4];
#pragma unroll
        for (int kb = 0; kb < 4; kb++) Sb[kb] = sbx[kb * 64];
        // U joins after the MFMAs: as an accumulator input it would tie its FIFO register to the MFMA's destination
        f32x4 D0 = f32x4{0.f, 0.f, 0.f, 0.f}, D1 = f32x4{0.f, 0.f, 0.f, 0.f};
        __builtin_amdgcn_sched_barrier(0);
        D0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(Wt[j][0], Sb[0], D0, 0, 0, 0);
        Wt[j][0] = on[wq];
        __builtin_amdgcn_sched_barrier(0);
        D1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(Wt[j][1], Sb[1], D1, 0, 0, 0);
        Wt[j][1] = on[wq + 64];
        __builtin_amdgcn_sched_barrier(0);
        D0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(Wt[j][2], Sb[2], D0, 0, 0, 0);
        Wt[j][2] = on[wq + 128];
        __builtin_amdgcn_sched_barrier(0);
        D1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(Wt[j][3], Sb[3], D1, 0, 0, 0);
        Wt[j][3] = on[wq + 192];
        __builtin_amdgcn_sched_barrier(0);
        const f32x4 D = (D0 + D1) + Ut[j];
        Ut[j] = upb[cn * ust];
        __builtin_amdgcn_sched_barrier(0);
        half4 dh;
        dh[0] = (_Float16)D[0]; dh[1] = (_Float16)D[1]; dh[2] = (_Float16)D[2]; dh[3] = (_Float16)D[3];
        // B-operand layout of D: k-block w / 2, halves 4 (w & 1) .. + 3 of the lane's eight
        reinterpret_cast<half4*>(db_x)[((w >> 1) * 64 + lane) * 2 + (w & 1)] = dh;
        ST[0] *= gct[j];
        ST[1] *= gct[j];
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();                                           // E2
        asm volatile("" ::: "memory");
        const half8 Db0 = dbx[0], Db1 = dbx[64];
        __builtin_amdgcn_sched_barrier(0);
        ST[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Kt[j][0], Db0, ST[0], 0, 0, 0);
        Kt[j][0] = on[kq0];
        __builtin_amdgcn_sched_barrier(0);
        ST[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Kt[j][2], Db0, ST[1], 0, 0, 0);
        Kt[j][2] = on[kq0 + 128];
        __builtin_amdgcn_sched_barrier(0);
        ST[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Kt[j][1], Db1, ST[0], 0, 0, 0);
        Kt[j][1] = on[kq0 + 64];
        __builtin_amdgcn_sched_barrier(0);
        ST[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Kt[j][3], Db1, ST[1], 0, 0, 0);
        Kt[j][3] = on[kq0 + 192];
        gct[j] = gC[(size_t)cn * HV + h];
        __builtin_amdgcn_sched_barrier(0);
    };
    int c = 0;
    for (; c + PB_DEP <= NC; c += PB_DEP) {
        step(std::integral_constant<int, 0>{}, c);
        step(std::integral_constant<int, 1>{}, c + 1);
        step(std::integral_constant<int, 2>{}, c + 2);
        step(std::integral_constant<int, 3>{}, c + 3);
    }
    if (c < NC) step(std::integral_constant<int, 0>{}, c);
    if (c + 1 < NC) step(std::integral_constant<int, 1>{}, c + 1);
    if (c + 2 < NC) step(std::integral_constant<int, 2>{}, c + 2);
    {
        float* sp = st_out + ((size_t)h * DV + sl * 16 + n) * DK + w * 32 + 4 * g;
        *reinterpret_cast<f32x4*>(sp) = ST[0];
        *reinterpret_cast<f32x4*>(sp + 16) = ST[1];
    }
}
static_assert(PB_DEP == 4, "the chain loop is unrolled by hand for four FIFO entries");

// Output kernel: Y_c = Qg_c S_c^T + Am_c D_c for one (chunk, head) per workgroup of 4 wavefronts; wavefront w covers the dv
// slices 2w and 2w+1.  The 64 x 128 tile goes through LDS as bf16 and leaves either as y [S,16,128] or, with NORM, straight
// through the gated RMSNorm (same arithmetic as the stand-alone kernel: 16 lanes per row, 8 columns each; batch.py:338-343).
constexpr int YS_LD = DV + 8;
template <bool NORM>
__global__ __launch_bounds__(256) void gdn_output_kernel(const _Float16* __restrict__ ops, const _Float16* __restrict__ snap,
                                                         bf16_t* __restrict__ y, const bf16_t* __restrict__ proj,
                                                         const float* __restrict__ gw, float eps, int S) {
    const int rec = blockIdx.x, c = rec / HV, h = rec % HV;
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
    __shared__ __align__(16) bf16_t ys[C * YS_LD];
    const half8* op = reinterpret_cast<const half8*>(ops + (size_t)rec * OP_HALVES) + lane;
    const half8* sp = reinterpret_cast<const half8*>(snap + ((size_t)rec * 8 + 2 * w) * SNAP_HALVES) + lane;
    half8 Sb[2][4], Db[2][2], Qt[16], At[8];
#pragma unroll
    for (int s = 0; s < 2; s++) {
#pragma unroll
        for (int kb = 0; kb < 4; kb++) Sb[s][kb] = sp[s * (SNAP_HALVES / 8) + kb * 64];
#pragma unroll
        for (int kb2 = 0; kb2 < 2; kb2++) Db[s][kb2] = sp[s * (SNAP_HALVES / 8) + (SNAP_S / 8) + kb2 * 64];
    }
#pragma unroll
    for (int i = 0; i < 16; i++) Qt[i] = op[(OP_Q / 8) + i * 64];
#pragma unroll
    for (int i = 0; i < 8; i++) At[i] = op[(OP_A / 8) + i * 64];
#pragma unroll
    for (int s = 0; s < 2; s++) {
        f32x4 Y[NCT];
#pragma unroll
        for (int ct = 0; ct < NCT; ct++) Y[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < 4; kb++)
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) Y[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Qt[ct * 4 + kb], Sb[s][kb], Y[ct], 0, 0, 0);
#pragma unroll
        for (int kb2 = 0; kb2 < 2; kb2++)
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) Y[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(At[ct * 2 + kb2], Db[s][kb2], Y[ct], 0, 0, 0);
#pragma unroll
        for (int ct = 0; ct < NCT; ct++)
#pragma unroll
            for (int r = 0; r < 4; r++) ys[(ct * 16 + 4 * g + r) * YS_LD + (2 * w + s) * 16 + n] = f2bf(Y[ct][r]);
    }
    __syncthreads();
    if (!NORM) {
        const int row = threadIdx.x >> 2, q4 = threadIdx.x & 3;
        const int t = c * C + row;
        if (t < S) {
            const uint4* src = reinterpret_cast<const uint4*>(&ys[row * YS_LD + q4 * 32]);
            uint4* dst = reinterpret_cast<uint4*>(y + ((size_t)t * HV + h) * DV + q4 * 32);
#pragma unroll
            for (int i = 0; i < 4; i++) dst[i] = src[i];
        }
    } else {
        const int cc = threadIdx.x & 15;
        float gwv[8];
#pragma unroll
        for (int j = 0; j < 8; j++) gwv[j] = gw[cc * 8 + j];
        // the four rows of this 16-lane group: all sums of squares first, then one reciprocal square root per lane
        uint4 yv4[4];
        float ss4[4], inv4[4];
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int row = it * 16 + (threadIdx.x >> 4);
            yv4[it] = *reinterpret_cast<const uint4*>(&ys[row * YS_LD + cc * 8]);
            float yy[8];
            unpack8(yv4[it], yy);
            double ss = 0.0;
#pragma unroll
            for (int j = 0; j < 4; j++) ss += (double)yy[2 * j] * yy[2 * j] + (double)yy[2 * j + 1] * yy[2 * j + 1];
            ss4[it] = (float)row16_sum_d(ss);
        }
        rsqrt_rows<4>(ss4, eps, inv4, cc);
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int row = it * 16 + (threadIdx.x >> 4);
            const int t = c * C + row;
            if (t >= S) continue;                                               // whole 16-lane groups leave together
            const uint4 zv = reinterpret_cast<const uint4*>(proj + (size_t)t * PW + CD + h * DV)[cc];
            float yy[8], zz[8];
            unpack8(yv4[it], yy);
            unpack8(zv, zz);
            uint32_t o[8];
#pragma unroll
            for (int j = 0; j < 8; j++) o[j] = gated_out(zz[j], gwv[j] * (yy[j] * inv4[it]));
            reinterpret_cast<uint4*>(y + ((size_t)t * HV + h) * DV)[cc] =
                make_uint4(o[0] | (o[1] << 16), o[2] | (o[3] << 16), o[4] | (o[5] << 16), o[6] | (o[7] << 16));
        }
    }
}

// ------------------------------------------------------------------------------------------------------------------
// Phase A: one workgroup of 256 threads per (chunk, head).
// ------------------------------------------------------------------------------------------------------------------
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));


constexpr int QS_LD = DK + 8;        // row strides (elements) of the LDS tiles: keep 16-byte alignment, spread the banks
constexpr int KT_LD = C;             // K^T / V^T rows are unpadded; their 16-byte chunks are XOR-swizzled by (row >> 3) & 7
constexpr int LS_LD = C + 4;

// element (row d, token t) of the transposed tiles: chunk (t >> 3) ^ ((d >> 3) & 7), so that the 2-byte transposing writes of
// a wavefront (16 lanes = 16 values of d >> 3, same t) spread over the banks while a 16-byte read stays one chunk
__device__ __forceinline__ int kt_at(int d, int t) { return d * KT_LD + ((((t >> 3) ^ (d >> 3)) & 7) << 3) + (t & 7); }

struct PhaseALds {                       // 68 KiB: two workgroups per CU
    union {
        struct {                         // first half of the kernel: the chunk's q, k rows
            __align__(16) bf16_t Qs[C * QS_LD];
            __align__(16) bf16_t Ks[C * QS_LD];
        };
        struct {                         // second half: L = strict_lower(beta G K K^T) and T = (I + L)^-1
            __align__(16) float Ls[C * LS_LD];
            __align__(16) float Ts[C * LS_LD];
        };
    };
    __align__(16) bf16_t KT[DK * KT_LD];
    __align__(16) bf16_t VT[DV * KT_LD];
    float Lc[C], beta[C], gam[C], dec[C];
};
struct PhaseALdsConv : PhaseALds {       // + the silu_bf16 table of the fused conv: 75 KiB, still two workgroups per CU
    __align__(16) bf16_t tab[SILU_TAB_SIZE];
};

__device__ __forceinline__ half8 to_half8(const float (&v)[8]) {
    half8 h;
#pragma unroll
    for (int j = 0; j < 8; j++) h[j] = (_Float16)v[j];
    return h;
}
__device__ __forceinline__ void unpack4(uint2 w, float* f) {
    f[0] = lo_bf(w.x); f[1] = hi_bf(w.x); f[2] = lo_bf(w.y); f[3] = hi_bf(w.y);
}

// Stores one token's normalized q, k and v (8 channels of each, bf16 pairs) into the row-major and transposed LDS tiles.
__device__ __forceinline__ void stage_token(PhaseALds& L, int tl, int cc, const uint4& rq, const uint4& rk, const uint4& rv) {
    *reinterpret_cast<uint4*>(&L.Qs[tl * QS_LD + cc * 8]) = rq;
    *reinterpret_cast<uint4*>(&L.Ks[tl * QS_LD + cc * 8]) = rk;
    const uint32_t kw[4] = {rk.x, rk.y, rk.z, rk.w};
    const uint32_t vw[4] = {rv.x, rv.y, rv.z, rv.w};
#pragma unroll
    for (int e = 0; e < 4; e++) {
        L.KT[kt_at(cc * 8 + 2 * e, tl)] = (bf16_t)(kw[e] & 0xffffu);
        L.KT[kt_at(cc * 8 + 2 * e + 1, tl)] = (bf16_t)(kw[e] >> 16);
        L.VT[kt_at(cc * 8 + 2 * e, tl)] = (bf16_t)(vw[e] & 0xffffu);
        L.VT[kt_at(cc * 8 + 2 * e + 1, tl)] = (bf16_t)(vw[e] >> 16);
    }
}

// Phase A of one (chunk, head).  FROM_PROJ = false: q, k, v [S,16,128] bf16 are inputs (convolved, normalized: conv_prep's
// outputs).  FROM_PROJ = true: they are computed here from the projection rows (conv4 + SiLU + q/k norm with the arithmetic of
// conv_prep_kernel, bit for bit; qwen35/prefill.py:96-134) and, with WRITE_QKV, also stored; the workgroups of the last chunk
// write the new conv window (the last three input rows, prefill.py:262-263) to conv_out if it is given.
// proj [S,8224] supplies the gate inputs a, b in both forms.
template <bool FROM_PROJ, bool WRITE_QKV>
__global__ __launch_bounds__(256, 2) void gdn_phase_a_kernel(const bf16_t* __restrict__ proj, bf16_t* qi, bf16_t* ki, bf16_t* vi,
                                                          const bf16_t* __restrict__ cs, const bf16_t* __restrict__ cw,
                                                          const bf16_t* __restrict__ silu_tab, bf16_t* __restrict__ conv_out,
                                                          const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                                                          _Float16* __restrict__ ops, float* __restrict__ U,
                                                          float* __restrict__ gC, int S) {
    __shared__ typename std::conditional<FROM_PROJ, PhaseALdsConv, PhaseALds>::type L;
    const int c = blockIdx.x / HV, h = blockIdx.x % HV, t0 = c * C;
    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    const size_t rec = (size_t)c * HV + h;
    _Float16* op = ops + rec * OP_HALVES;
    const int gi = tid >> 4, cc = tid & 15;

    // ---- the chunk's rows: every load is issued before anything else; rows past the end are zero (gdn_nax.py:172-174)
    uint4 raw[4][3];                               // !FROM_PROJ: token rr * 16 + gi, a lane 8 consecutive columns
    uint4 rw[3][7], wt[3][4];                      // FROM_PROJ: input rows 4 gi - 3 .. 4 gi + 3 of 8 channels of q, k, v; their taps
    if constexpr (!FROM_PROJ) {
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            const int t = t0 + rr * 16 + gi;
            const size_t o = ((size_t)min(t, S - 1) * HV + h) * DK + cc * 8;
            raw[rr][0] = *reinterpret_cast<const uint4*>(qi + o);
            raw[rr][1] = *reinterpret_cast<const uint4*>(ki + o);
            raw[rr][2] = *reinterpret_cast<const uint4*>(vi + o);
            if (t >= S) raw[rr][0] = raw[rr][1] = raw[rr][2] = make_uint4(0, 0, 0, 0);
        }
    } else {
#pragma unroll
        for (int part = 0; part < 3; part++) {
            const int ch0 = part * KD + h * DK + cc * 8;
#pragma unroll
            for (int e = 0; e < 4; e++) wt[part][e] = *reinterpret_cast<const uint4*>(cw + (size_t)(ch0 + 2 * e) * 4);
#pragma unroll
            for (int d = 0; d < 7; d++) {
                const int tt = min(t0 + 4 * gi - 3 + d, S - 1);
                rw[part][d] = *reinterpret_cast<const uint4*>(tt < 0 ? cs + (tt + 3) * CD + ch0 : proj + (size_t)tt * PW + ch0);
            }
        }
        if (conv_out && c == (S - 1) / C && tid < 3 * 48) {            // new conv window: input rows S-3 .. S-1 of this head's channels
            const int r = tid / 48, part = (tid % 48) >> 4, ch0 = part * KD + h * DK + (tid & 15) * 8, tt = S - 3 + r;
            *reinterpret_cast<uint4*>(conv_out + r * CD + ch0) =
                *reinterpret_cast<const uint4*>(tt < 0 ? cs + (tt + 3) * CD + ch0 : proj + (size_t)tt * PW + ch0);
        }
    }

    // ---- gates of the chunk's tokens (gdn_nax.py:80-104): wave 0, one token per lane
    if (w == 0) {
        const int t = t0 + lane;
        float lg = 0.f, be = 0.f;
        if (t < S) {
            lg = log_decay(A_log[h], BF(bf2f(proj[(size_t)t * PW + CD + KD + HV + h]) + dt_bias[h]));
            be = sigmoid_bf16(bf2f(proj[(size_t)t * PW + CD + KD + h]));
        }
        float lc = lg;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const float o = __shfl_up(lc, d, 64);
            if (lane >= d) lc += o;
        }
        const float tot = __shfl(lc, 63, 64);
        L.Lc[lane] = lc;
        L.beta[lane] = be;
        L.gam[lane] = expf(lc);
        L.dec[lane] = expf(tot - lc);
        if (lane == 63) gC[rec] = expf(lc);
    }
    if constexpr (!FROM_PROJ) {
#pragma unroll
        for (int rr = 0; rr < 4; rr++) stage_token(L, rr * 16 + gi, cc, raw[rr][0], raw[rr][1], raw[rr][2]);
    } else {
        silu_table_fill(L.tab, silu_tab, tid, 256);
        __syncthreads();
        const float scq = BF(INV_SCALE * INV_SCALE), sck = BF(INV_SCALE);
        uint4 pk[4][3];
        float ss[8], rr[8];
#pragma unroll
        for (int part = 0; part < 3; part++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const double sq = conv8_silu_packed(L.tab, rw[part][j], rw[part][j + 1], rw[part][j + 2], rw[part][j + 3], wt[part],
                                                    pk[j][part]);
                if (part < 2) ss[2 * j + part] = (float)row16_sum_d(sq);
            }
        rsqrt_rows<8>(ss, qk_eps(), rr, cc);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int tl = 4 * gi + j, t = t0 + tl;
            uint4 pq = scale8_packed(pk[j][0], rr[2 * j], scq), pkk = scale8_packed(pk[j][1], rr[2 * j + 1], sck), pv = pk[j][2];
            if (t >= S) pq = pkk = pv = make_uint4(0, 0, 0, 0);
            if (WRITE_QKV && t < S) {
                const size_t o = ((size_t)t * HV + h) * DK + cc * 8;
                *reinterpret_cast<uint4*>(qi + o) = pq;
                *reinterpret_cast<uint4*>(ki + o) = pkk;
                *reinterpret_cast<uint4*>(vi + o) = pv;
            }
            stage_token(L, tl, cc, pq, pkk, pv);
        }
    }
    __syncthreads();

    // ---- K K^T (lower tiles) -> L, and (Q K^T)^T -> Am, on bf16 MFMA.  Wave w: row of tiles ti = 3 - w of K K^T and the
    // Am / Qg tiles of ct = w.  L stays in registers until every wave is done with Qs / Ks, whose LDS it then takes over.
    f32x4 Lreg[4];
    {
        const int ti = 3 - w;
#pragma unroll
        for (int tj = 0; tj < 4; tj++) {
            Lreg[tj] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (tj <= ti) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kb = 0; kb < 4; kb++) {
                    const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&L.Ks[(16 * ti + n) * QS_LD + 32 * kb + 8 * g]));
                    const bf16x8 b = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&L.Ks[(16 * tj + n) * QS_LD + 32 * kb + 8 * g]));
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
                }
                const int j = 16 * tj + n;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int i = 16 * ti + 4 * g + r;
                    Lreg[tj][r] = i > j ? L.beta[i] * expf(L.Lc[i] - L.Lc[j]) * acc[r] : 0.f;
                }
            }
        }
        const int ct = w, co = 16 * ct + n;                         // Am: rows c_out = 16 ct + n, k = c_in (permuted)
        for (int kb2 = 0; kb2 < 2; kb2++) {
            f32x4 part[2];
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {
                const int tj = 2 * kb2 + hf;
                part[hf] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (tj <= ct) {
#pragma unroll
                    for (int kb = 0; kb < 4; kb++) {
                        const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&L.Ks[(16 * tj + n) * QS_LD + 32 * kb + 8 * g]));
                        const bf16x8 b = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&L.Qs[(16 * ct + n) * QS_LD + 32 * kb + 8 * g]));
                        part[hf] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, part[hf], 0, 0, 0);
                    }
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int ci = 16 * tj + 4 * g + r;
                        part[hf][r] = ci <= co ? expf(L.Lc[co] - L.Lc[ci]) * part[hf][r] : 0.f;
                    }
                }
            }
            *reinterpret_cast<half8*>(op + OP_A + (ct * 2 + kb2) * 512 + lane * 8) = pack_half8(part[0], part[1]);
        }
        // Qg = gamma * Q (rows of tile ct), k index permuted
        const float gm = L.gam[16 * ct + n];
        for (int kb = 0; kb < 4; kb++) {
            float qf[8];
            unpack4(*reinterpret_cast<const uint2*>(&L.Qs[(16 * ct + n) * QS_LD + 32 * kb + 4 * g]), qf);
            unpack4(*reinterpret_cast<const uint2*>(&L.Qs[(16 * ct + n) * QS_LD + 32 * kb + 16 + 4 * g]), qf + 4);
#pragma unroll
            for (int j = 0; j < 8; j++) qf[j] *= gm;
            *reinterpret_cast<half8*>(op + OP_Q + (ct * 4 + kb) * 512 + lane * 8) = to_half8(qf);
        }
    }
    __syncthreads();
    for (int i = tid; i < C * LS_LD; i += 256) L.Ts[i] = 0.f;                   // blocks of T above the diagonal stay zero
    {
        const int ti = 3 - w;
#pragma unroll
        for (int tj = 0; tj < 4; tj++)
            if (tj <= ti) {
#pragma unroll
                for (int r = 0; r < 4; r++) L.Ls[(16 * ti + 4 * g + r) * LS_LD + 16 * tj + n] = Lreg[tj][r];
            }
    }
    __syncthreads();

    // ---- T = (I + L)^-1 by blocks of 16 (exact fp32: forward substitution on the diagonal blocks, fp32 MFMA below them)
    f32x4 TR[4];                                   // TR[d] = block (w + d, w) of T, accumulator layout
    {
        float x[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float a = (i == n) ? 1.f : 0.f;
            const float* lr = &L.Ls[(16 * w + i) * LS_LD + 16 * w];
#pragma unroll
            for (int m = 0; m < i; m++) a -= lr[m] * x[m];
            x[i] = a;
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            float v = 0.f;
#pragma unroll
            for (int i = 0; i < 16; i++) v = (i == 4 * g + r) ? x[i] : v;
            TR[0][r] = v;
            L.Ts[(16 * w + 4 * g + r) * LS_LD + 16 * w + n] = v;
        }
    }
    __syncthreads();
#pragma unroll
    for (int d = 1; d < 4; d++) {
        if (w + d < 4) {
            const int I = w + d;
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int e = 0; e < d; e++) {
                const f32x4 a4 = *reinterpret_cast<const f32x4*>(&L.Ls[(16 * I + n) * LS_LD + 16 * (w + e) + 4 * g]);
#pragma unroll
                for (int kk = 0; kk < 4; kk++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[kk], TR[e][kk], acc, 0, 0, 0);
            }
            f32x4 res = {0.f, 0.f, 0.f, 0.f};
            const f32x4 d4 = *reinterpret_cast<const f32x4*>(&L.Ts[(16 * I + n) * LS_LD + 16 * I + 4 * g]);
#pragma unroll
            for (int kk = 0; kk < 4; kk++) res = __builtin_amdgcn_mfma_f32_16x16x4f32(d4[kk], acc[kk], res, 0, 0, 0);
            TR[d] = -res;
#pragma unroll
            for (int r = 0; r < 4; r++) L.Ts[(16 * I + 4 * g + r) * LS_LD + 16 * w + n] = TR[d][r];
        }
    }
    __syncthreads();

    // ---- Wn^T = -(gamma K)^T Tb^T and U = Tb V on fp16 MFMA; wave w owns the chunk rows of tile ct = w
    {
        const int ct = w, nkb = ct < 2 ? 1 : 2;                     // Tb is lower triangular: columns past the row tile are zero
        half8 tb[2];
#pragma unroll
        for (int kb2 = 0; kb2 < 2; kb2++) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int cp = 32 * kb2 + 8 * g + j;
                v[j] = L.Ts[(16 * ct + n) * LS_LD + cp] * L.beta[cp];
            }
            tb[kb2] = to_half8(v);
        }
        for (int kb = 0; kb < 4; kb++) {
            f32x4 acc[2];
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {
                const int mt = 2 * kb + hf;
                acc[hf] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kb2 = 0; kb2 < 2; kb2++) {
                    if (kb2 >= nkb) continue;
                    float kf[8];
                    unpack8(*reinterpret_cast<const uint4*>(&L.KT[kt_at(16 * mt + n, 32 * kb2 + 8 * g)]), kf);
#pragma unroll
                    for (int j = 0; j < 8; j++) kf[j] *= -L.gam[32 * kb2 + 8 * g + j];
                    acc[hf] = __builtin_amdgcn_mfma_f32_16x16x32_f16(to_half8(kf), tb[kb2], acc[hf], 0, 0, 0);
                }
            }
            *reinterpret_cast<half8*>(op + OP_W + (ct * 4 + kb) * 512 + lane * 8) = pack_half8(acc[0], acc[1]);
        }
        float* up = U + rec * U_FLOATS;
        for (int sl = 0; sl < 8; sl++) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kb2 = 0; kb2 < 2; kb2++) {
                if (kb2 >= nkb) continue;
                float vf[8];
                unpack8(*reinterpret_cast<const uint4*>(&L.VT[kt_at(16 * sl + n, 32 * kb2 + 8 * g)]), vf);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(tb[kb2], to_half8(vf), acc, 0, 0, 0);
            }
            *reinterpret_cast<f32x4*>(up + ((sl * NCT + ct) * 64 + lane) * 4) = acc;
        }
        // Kd = (dec * K)^T (rows dk of tiles 2w, 2w+1), k index permuted
        for (int mm = 0; mm < 2; mm++) {
            const int mt = 2 * w + mm;
            for (int kb2 = 0; kb2 < 2; kb2++) {
                float kf[8];
                unpack4(*reinterpret_cast<const uint2*>(&L.KT[kt_at(16 * mt + n, 32 * kb2 + 4 * g)]), kf);
                unpack4(*reinterpret_cast<const uint2*>(&L.KT[kt_at(16 * mt + n, 32 * kb2 + 16 + 4 * g)]), kf + 4);
#pragma unroll
                for (int j = 0; j < 8; j++) kf[j] *= L.dec[32 * kb2 + 16 * (j >> 2) + 4 * g + (j & 3)];
                *reinterpret_cast<half8*>(op + OP_K + (mt * 2 + kb2) * 512 + lane * 8) = to_half8(kf);
            }
        }
    }
}

}  // namespace

extern "C" {

// sizes (bytes) of the phase A -> phase B buffers for S tokens: ops, U, gC
long qt_gdn_chunk_ops_bytes(int S) { return S < 0 ? -1 : (long)((S + C - 1) / C) * HV * OP_HALVES * 2; }
long qt_gdn_chunk_u_bytes(int S) { return S < 0 ? -1 : (long)((S + C - 1) / C) * HV * U_FLOATS * 4; }
long qt_gdn_chunk_gc_bytes(int S) { return S < 0 ? -1 : (long)((S + C - 1) / C) * HV * 4; }

static int phase_b_launch(const void* ops, const float* U, const float* gC, void* snap, const float* state_in, float* state_out,
                          void* y, const void* proj, const float* gw, float eps, bool norm, int S, hipStream_t stream) {
    if (!ops || !U || !gC || !snap || !state_in || !state_out || !y) return QT_ERR_NULL;
    if (norm && (!proj || !gw)) return QT_ERR_NULL;
    if (S < 0) return QT_ERR_DIM;
    for (const void* p : {ops, (const void*)U, (const void*)snap, (const void*)state_in, (const void*)state_out, (const void*)y, proj})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    const int NC = (S + C - 1) / C;
    if (NC == 0) {
        if (state_out != state_in &&
            hipMemcpyAsync(state_out, state_in, sizeof(float) * HV * DV * DK, hipMemcpyDeviceToDevice, stream) != hipSuccess)
            return QT_ERR_LAUNCH;
        return QT_OK;
    }
    hipLaunchKernelGGL(gdn_chain_kernel, dim3(HV * 8), dim3(320), 0, stream, (const _Float16*)ops, U, gC, state_in, state_out,
                       (_Float16*)snap, NC);
    QT_CHECK_LAUNCH();
    if (norm)
        hipLaunchKernelGGL(gdn_output_kernel<true>, dim3(NC * HV), dim3(256), 0, stream, (const _Float16*)ops,
                           (const _Float16*)snap, (bf16_t*)y, (const bf16_t*)proj, gw, eps, S);
    else
        hipLaunchKernelGGL(gdn_output_kernel<false>, dim3(NC * HV), dim3(256), 0, stream, (const _Float16*)ops,
                           (const _Float16*)snap, (bf16_t*)y, (const bf16_t*)nullptr, (const float*)nullptr, 0.f, S);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

long qt_gdn_chunk_snap_bytes(int S) { return S < 0 ? -1 : (long)((S + C - 1) / C) * HV * 8 * SNAP_HALVES * 2; }

int qt_gdn_phase_b(const void* ops, const float* U, const float* gC, void* snap, const float* state_in, float* state_out, void* y,
                   int S, hipStream_t stream) {
    return phase_b_launch(ops, U, gC, snap, state_in, state_out, y, nullptr, nullptr, 0.f, false, S, stream);
}

int qt_gdn_phase_b_norm(const void* ops, const float* U, const float* gC, void* snap, const float* state_in, float* state_out,
                        const void* proj, const float* gw, float eps, void* out, int S, hipStream_t stream) {
    return phase_b_launch(ops, U, gC, snap, state_in, state_out, out, proj, gw, eps, true, S, stream);
}

int qt_gdn_phase_a(const void* proj, const void* q, const void* k, const void* v, const float* A_log, const float* dt_bias,
                   void* ops, float* U, float* gC, int S, hipStream_t stream) {
    if (!proj || !q || !k || !v || !A_log || !dt_bias || !ops || !U || !gC) return QT_ERR_NULL;
    if (S < 0) return QT_ERR_DIM;
    if (S == 0) return QT_OK;
    for (const void* p : {proj, q, k, v, (const void*)ops, (const void*)U})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    const int NC = (S + C - 1) / C;
    hipLaunchKernelGGL((gdn_phase_a_kernel<false, false>), dim3(NC * HV), dim3(256), 0, stream, (const bf16_t*)proj, (bf16_t*)q,
                       (bf16_t*)k, (bf16_t*)v, (const bf16_t*)nullptr, (const bf16_t*)nullptr, (const bf16_t*)nullptr,
                       (bf16_t*)nullptr, A_log, dt_bias, (_Float16*)ops, U, gC, S);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

int qt_gdn_phase_a_conv(const void* proj, const void* conv_state, const void* conv_w, const void* silu_table, const float* A_log,
                        const float* dt_bias, void* q, void* k, void* v, void* conv_out, void* ops, float* U, float* gC, int S,
                        hipStream_t stream) {
    if (!proj || !conv_state || !conv_w || !A_log || !dt_bias || !ops || !U || !gC) return QT_ERR_NULL;
    if ((q || k || v) && !(q && k && v)) return QT_ERR_NULL;
    if (S < 0) return QT_ERR_DIM;
    if (S == 0) return QT_OK;
    for (const void* p : {proj, conv_state, conv_w, silu_table, (const void*)q, (const void*)k, (const void*)v, (const void*)conv_out,
                          (const void*)ops, (const void*)U})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    if (conv_out == conv_state) return QT_ERR_UNSUPPORTED;          // the old window is still being read when the new one is written
    const int NC = (S + C - 1) / C;
    if (q)
        hipLaunchKernelGGL((gdn_phase_a_kernel<true, true>), dim3(NC * HV), dim3(256), 0, stream, (const bf16_t*)proj, (bf16_t*)q,
                           (bf16_t*)k, (bf16_t*)v, (const bf16_t*)conv_state, (const bf16_t*)conv_w, (const bf16_t*)silu_table,
                           (bf16_t*)conv_out, A_log, dt_bias, (_Float16*)ops, U, gC, S);
    else
        hipLaunchKernelGGL((gdn_phase_a_kernel<true, false>), dim3(NC * HV), dim3(256), 0, stream, (const bf16_t*)proj,
                           (bf16_t*)nullptr, (bf16_t*)nullptr, (bf16_t*)nullptr, (const bf16_t*)conv_state, (const bf16_t*)conv_w,
                           (const bf16_t*)silu_table, (bf16_t*)conv_out, A_log, dt_bias, (_Float16*)ops, U, gC, S);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

}  // extern "C"
