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
constexpr int PF_AHEAD = 8;                     // chunks the L2 prefetch wavefront runs ahead of the MFMA wavefront

__global__ __launch_bounds__(128) void gdn_phase_b_kernel(const _Float16* __restrict__ ops, const float* __restrict__ U,
                                                         const float* __restrict__ gC, const float* __restrict__ st_in,
                                                         float* __restrict__ st_out, bf16_t* __restrict__ y, int S, int NC) {
    // heads that share an XCD's L2 keep their 8 slices there: workgroup id = xcd + 8 k, head = xcd + 8 (k / 8), slice = k % 8
    const int xcd = blockIdx.x & 7, kq = blockIdx.x >> 3;
    const int h = xcd + 8 * (kq >> 3), sl = kq & 7;
    const int lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;

    // Wavefront 0 runs the serial MFMA chain and touches global memory with loads only: on gfx9-family targets loads and
    // stores share one in-order counter only as long as a single kind is in flight, so a store in the loop would force
    // every wait down to zero outstanding loads and expose the full memory latency at every chunk.
    // Wavefront 1 is its helper: it writes the finished output rows, which wavefront 0 hands over through two buffers in
    // LDS, and it pulls the records of the coming chunks into this XCD's L2 (one dword per 128-byte line), PF_AHEAD chunks
    // in front.  The hand-over is one bare s_barrier per chunk (no fence: only LDS is exchanged, and s_waitcnt lgkmcnt(0)
    // orders it): after barrier c the helper reads buffer c & 1, and wavefront 0 next writes that buffer after barrier c+1.
    __shared__ __align__(16) bf16_t y_s[2][C * 16];                           // one chunk of this slice's outputs, row major
    if (threadIdx.x >= 64) {
        unsigned sink = 0;
        for (int c = 0; c < NC; c++) {
            // touch the record of chunk c + PF_AHEAD; the values are only folded into `sink` after the hand-over below,
            // so these loads never delay the barrier
            unsigned pfv[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            const int pf = c + PF_AHEAD;
            if (PF_AHEAD > 0 && pf < NC) {
                const size_t rec = (size_t)pf * HV + h;
                const unsigned* o32 = reinterpret_cast<const unsigned*>(ops + rec * OP_HALVES) + lane * 32;
#pragma unroll
                for (int i = 0; i < OP_HALVES * 2 / 8192; i++) pfv[i] = o32[i * 2048];
                const unsigned* u32 = reinterpret_cast<const unsigned*>(U + rec * U_FLOATS + (size_t)sl * NCT * 256);
                pfv[7] = u32[(lane & 31) * 32];
            }
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            const uint4* src = reinterpret_cast<const uint4*>(&y_s[c & 1][lane * 16]);
            const uint4 lo = src[0], hi = src[1];
            const int t = c * C + lane;
            if (t < S) {
                uint4* dst = reinterpret_cast<uint4*>(y + ((size_t)t * HV + h) * DV + sl * 16);
                dst[0] = lo;
                dst[1] = hi;
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                  // the LDS reads are done before the next barrier
#pragma unroll
            for (int i = 0; i < 8; i++) sink ^= pfv[i];
        }
        if (sink == 0x9e3779b9u && S < 0) st_out[0] = 0.f;                      // keeps the prefetch loads alive; never true
        return;
    }

    f32x4 ST[8];
    {
        const float* sp = st_in + ((size_t)h * DV + sl * 16 + n) * DK;          // S[h][dv][dk], dk contiguous
#pragma unroll
        for (int mt = 0; mt < 8; mt++) ST[mt] = *reinterpret_cast<const f32x4*>(sp + mt * 16 + 4 * g);
    }
    // Operand FIFO, one chunk deep: tile i of chunk c+1 is loaded into the registers of tile i of chunk c right after the
    // MFMA that consumed it, so a whole chunk step of MFMA work covers the latency of every load.
    half8 Wt[16], Qt[16], Kt[16], At[8];
    f32x4 Ut[NCT];
    float gc;
    {
        const half8* op = reinterpret_cast<const half8*>(ops + (size_t)h * OP_HALVES) + lane;
        const f32x4* up = reinterpret_cast<const f32x4*>(U + (size_t)h * U_FLOATS + (size_t)sl * NCT * 256) + lane;
        // same issue order as inside the loop
#pragma unroll
        for (int ct = 0; ct < NCT; ct++) Ut[ct] = up[ct * 64];
#pragma unroll
        for (int kb = 0; kb < 4; kb++)
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) Wt[ct * 4 + kb] = op[(OP_W / 8) + (ct * 4 + kb) * 64];
        gc = gC[h];
#pragma unroll
        for (int kb2 = 0; kb2 < 2; kb2++)
#pragma unroll
            for (int mt = 0; mt < 8; mt++) Kt[mt * 2 + kb2] = op[(OP_K / 8) + (mt * 2 + kb2) * 64];
#pragma unroll
        for (int kb = 0; kb < 4; kb++)
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) Qt[ct * 4 + kb] = op[(OP_Q / 8) + (ct * 4 + kb) * 64];
#pragma unroll
        for (int kb2 = 0; kb2 < 2; kb2++)
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) At[ct * 2 + kb2] = op[(OP_A / 8) + (ct * 2 + kb2) * 64];
    }
    __builtin_amdgcn_sched_barrier(0);
    for (int c = 0; c < NC; c++) {
        const int cn = c + 1 < NC ? c + 1 : c;                                  // the last step re-reads its own record
        const size_t recn = (size_t)cn * HV + h;
        const half8* op = reinterpret_cast<const half8*>(ops + recn * OP_HALVES) + lane;
        const f32x4* up = reinterpret_cast<const f32x4*>(U + recn * U_FLOATS + (size_t)sl * NCT * 256) + lane;

        half8 Sb[4];
#pragma unroll
        for (int kb = 0; kb < 4; kb++) Sb[kb] = pack_half8(ST[2 * kb], ST[2 * kb + 1]);

        // Every MFMA is followed by the load that refills its operand registers for the next chunk, and the scheduler is
        // pinned to this order: loads then complete in the order in which the next chunk consumes them, so the waits stay
        // partial (a reordered load would force a wait for all 60).  Independent accumulators alternate (ct / mt inner).
        f32x4 D[NCT], Y[NCT];
#pragma unroll
        for (int ct = 0; ct < NCT; ct++) {
            D[ct] = Ut[ct];
            Ut[ct] = up[ct * 64];
            Y[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kb = 0; kb < 4; kb++)
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) {
                D[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Wt[ct * 4 + kb], Sb[kb], D[ct], 0, 0, 0);
                Wt[ct * 4 + kb] = op[(OP_W / 8) + (ct * 4 + kb) * 64];
            }
        half8 Db[2];
        Db[0] = pack_half8(D[0], D[1]);
        Db[1] = pack_half8(D[2], D[3]);
#pragma unroll
        for (int mt = 0; mt < 8; mt++) ST[mt] *= gc;
        gc = gC[recn];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kb2 = 0; kb2 < 2; kb2++)
#pragma unroll
            for (int mt = 0; mt < 8; mt++) {
                ST[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Kt[mt * 2 + kb2], Db[kb2], ST[mt], 0, 0, 0);
                Kt[mt * 2 + kb2] = op[(OP_K / 8) + (mt * 2 + kb2) * 64];
            }
#pragma unroll
        for (int kb = 0; kb < 4; kb++)
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) {
                Y[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Qt[ct * 4 + kb], Sb[kb], Y[ct], 0, 0, 0);
                Qt[ct * 4 + kb] = op[(OP_Q / 8) + (ct * 4 + kb) * 64];
            }
#pragma unroll
        for (int kb2 = 0; kb2 < 2; kb2++)
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) {
                Y[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(At[ct * 2 + kb2], Db[kb2], Y[ct], 0, 0, 0);
                At[ct * 2 + kb2] = op[(OP_A / 8) + (ct * 2 + kb2) * 64];
            }
        // hand the chunk's outputs to the helper wavefront
        {
            bf16_t* ys = y_s[c & 1];
#pragma unroll
            for (int ct = 0; ct < NCT; ct++)
#pragma unroll
                for (int r = 0; r < 4; r++) ys[(ct * 16 + 4 * g + r) * 16 + n] = f2bf(Y[ct][r]);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                      // the LDS writes have landed
        __builtin_amdgcn_s_barrier();
    }
    {
        float* sp = st_out + ((size_t)h * DV + sl * 16 + n) * DK;
#pragma unroll
        for (int mt = 0; mt < 8; mt++) *reinterpret_cast<f32x4*>(sp + mt * 16 + 4 * g) = ST[mt];
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

__device__ __forceinline__ half8 to_half8(const float (&v)[8]) {
    half8 h;
#pragma unroll
    for (int j = 0; j < 8; j++) h[j] = (_Float16)v[j];
    return h;
}
__device__ __forceinline__ void unpack4(uint2 w, float* f) {
    f[0] = lo_bf(w.x); f[1] = hi_bf(w.x); f[2] = lo_bf(w.y); f[3] = hi_bf(w.y);
}

// q, k, v [S,16,128] bf16 (convolved, normalized: conv_prep's outputs), proj [S,8224] (gate inputs a, b) -> phase B records
__global__ __launch_bounds__(256) void gdn_phase_a_kernel(const bf16_t* __restrict__ proj, const bf16_t* __restrict__ qi,
                                                          const bf16_t* __restrict__ ki, const bf16_t* __restrict__ vi,
                                                          const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                                                          _Float16* __restrict__ ops, float* __restrict__ U,
                                                          float* __restrict__ gC, int S) {
    __shared__ PhaseALds L;
    const int c = blockIdx.x / HV, h = blockIdx.x % HV, t0 = c * C;
    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    const size_t rec = (size_t)c * HV + h;
    _Float16* op = ops + rec * OP_HALVES;

    // ---- the chunk's q, k, v rows: every load is issued before anything else (a 16-lane group owns a token per round,
    // a lane 8 consecutive columns); rows past the end are zero (gdn_nax.py:172-174)
    uint4 raw[4][3];
    {
        const int gi = tid >> 4, cc = tid & 15;
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            const int t = t0 + rr * 16 + gi;
            const size_t o = ((size_t)min(t, S - 1) * HV + h) * DK + cc * 8;
            raw[rr][0] = *reinterpret_cast<const uint4*>(qi + o);
            raw[rr][1] = *reinterpret_cast<const uint4*>(ki + o);
            raw[rr][2] = *reinterpret_cast<const uint4*>(vi + o);
            if (t >= S) raw[rr][0] = raw[rr][1] = raw[rr][2] = make_uint4(0, 0, 0, 0);
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
    {
        const int gi = tid >> 4, cc = tid & 15;
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            const int tl = rr * 16 + gi;
            *reinterpret_cast<uint4*>(&L.Qs[tl * QS_LD + cc * 8]) = raw[rr][0];
            *reinterpret_cast<uint4*>(&L.Ks[tl * QS_LD + cc * 8]) = raw[rr][1];
            const uint32_t kw[4] = {raw[rr][1].x, raw[rr][1].y, raw[rr][1].z, raw[rr][1].w};
            const uint32_t vw[4] = {raw[rr][2].x, raw[rr][2].y, raw[rr][2].z, raw[rr][2].w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                L.KT[kt_at(cc * 8 + 2 * e, tl)] = (bf16_t)(kw[e] & 0xffffu);
                L.KT[kt_at(cc * 8 + 2 * e + 1, tl)] = (bf16_t)(kw[e] >> 16);
                L.VT[kt_at(cc * 8 + 2 * e, tl)] = (bf16_t)(vw[e] & 0xffffu);
                L.VT[kt_at(cc * 8 + 2 * e + 1, tl)] = (bf16_t)(vw[e] >> 16);
            }
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

int qt_gdn_phase_b(const void* ops, const float* U, const float* gC, const float* state_in, float* state_out, void* y, int S,
                   hipStream_t stream) {
    if (!ops || !U || !gC || !state_in || !state_out || !y) return QT_ERR_NULL;
    if (S < 0) return QT_ERR_DIM;
    for (const void* p : {ops, (const void*)U, (const void*)state_in, (const void*)state_out})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    const int NC = (S + C - 1) / C;
    hipLaunchKernelGGL(gdn_phase_b_kernel, dim3(HV * 8), dim3(128), 0, stream, (const _Float16*)ops, U, gC, state_in, state_out,
                       (bf16_t*)y, S, NC);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

int qt_gdn_phase_a(const void* proj, const void* q, const void* k, const void* v, const float* A_log, const float* dt_bias,
                   void* ops, float* U, float* gC, int S, hipStream_t stream) {
    if (!proj || !q || !k || !v || !A_log || !dt_bias || !ops || !U || !gC) return QT_ERR_NULL;
    if (S < 0) return QT_ERR_DIM;
    if (S == 0) return QT_OK;
    for (const void* p : {proj, q, k, v, (const void*)ops, (const void*)U})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    const int NC = (S + C - 1) / C;
    hipLaunchKernelGGL(gdn_phase_a_kernel, dim3(NC * HV), dim3(256), 0, stream, (const bf16_t*)proj, (const bf16_t*)q,
                       (const bf16_t*)k, (const bf16_t*)v, A_log, dt_bias, (_Float16*)ops, U, gC, S);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

}  // extern "C"
