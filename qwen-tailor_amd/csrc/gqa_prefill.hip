// Causal prefill attention, 8 query heads on 2 KV heads, head dim 256, for gfx950 (flash-attention forward on bf16 MFMA).
// Replaces the call mx.fast.scaled_dot_product_attention(q, K[:, :, :kv_len], V[:, :, :kv_len], scale=256**-0.5,
// mask="causal") of the reference's full-attention layers (qwen35/model.py:160-167, qwen35/prefill.py:468).
//
// One workgroup = 32 query rows x the 4 query heads that share a KV head: wavefront w owns the 16 rows of block w >> 1 for
// the two heads 2 (w & 1), 2 (w & 1) + 1, so a K / V tile of 64 keys is fetched from HBM once and staged in LDS for all of
// them, and every K or V fragment a wavefront reads from LDS feeds two MFMAs (one per head).  Per tile and wavefront:
//     S^T[keys x rows] = K_tile . Q^T     A = K rows from LDS, B = Q^T resident in registers (16x16x32 bf16 MFMA)
//     online softmax in the accumulator layout: lane (row n, group g) holds keys 4g..4g+3 of each 16-key sub-tile
//     O[rows x 256]   += P . V            A = two exponentiated S^T accumulators packed to bf16 (they ARE the A operand
//                                         when a 32-key block is enumerated as 16 (j >> 2) + 4 g + (j & 3)),
//                                         B = V through the transposing LDS load (4 consecutive keys of one column);
//                                         the row sums are one more column block, P . 1
// K / V tiles travel HBM -> LDS directly (global_load_lds_dwordx4: 64 lanes x 16 bytes land as one contiguous KiB, no
// registers in between) into double-buffered tiles.  The LDS rows are unpadded (a direct load cannot pad); instead the
// 16-byte chunks of row r are stored XOR-swizzled by r & 15 (the loading lane picks the matching global chunk), which keeps
// the fragment reads of 16 rows on distinct banks.  The tile loop is software-pipelined around one workgroup barrier per tile:
// the score MFMAs of tile t + 1 are interleaved step by step with the softmax of tile t (see `tile` below).
#include "qt_common.h"

#include <type_traits>

using namespace qt;

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr float SCALE_LOG2E = 0.0625f * 1.4426950408889634f;   // 256^-0.5 log2 e: scores are exponentiated in base 2
constexpr float NEG = -3.0e38f;
constexpr float LAZY = 8.0f;            // log2 of the growth of a row maximum that is tolerated before the row is rescaled
constexpr int KT = 64;                 // keys per tile
constexpr int TILE = KT * AD;          // elements of one K or V tile in LDS (32 KiB), rows unpadded, chunks swizzled

// AP_MARK(i): phase time stamps for profiling builds (QT_ATTN_PREFILL_PROF defines ap_prof_buf[workgroup][wave][8]: shader-clock
// ticks per phase, summed over the tiles in scalar registers and stored once at the end); otherwise only a scheduling fence
#ifdef QT_ATTN_PREFILL_PROF
__device__ long long* ap_prof_buf;
#define AP_MARK(i)                                  \
    do {                                            \
        const long long now_ = clock64();           \
        ap_acc_[i] += now_ - ap_last_;              \
        ap_last_ = now_;                            \
    } while (0)
#define AP_INIT()                                   \
    long long ap_acc_[8] = {0, 0, 0, 0, 0, 0, 0, 0}; \
    long long ap_last_ = clock64()
#define AP_STORE()                                                                                              \
    do {                                                                                                        \
        if ((threadIdx.x & 63) == 0)                                                                            \
            for (int i_ = 0; i_ < 8; i_++)                                                                      \
                ap_prof_buf[((size_t)(blockIdx.y * gridDim.x + blockIdx.x) * 4 + (threadIdx.x >> 6)) * 8 + i_] = ap_acc_[i_]; \
    } while (0)
#else
#define AP_MARK(i) __builtin_amdgcn_sched_barrier(0)     /* the phases of a tile are scheduled separately */
#define AP_INIT()
#define AP_STORE()
#endif

__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// max over the four lanes n, n + 16, n + 32, n + 48 with the VALU lane swaps of gfx950 (v_permlane32_swap exchanges the upper half
// of one register with the lower half of the other, v_permlane16_swap the odd 16-lane rows of one with the even rows of the
// other), which keeps the softmax free of LDS traffic
__device__ __forceinline__ float max_over_groups(float x) {
    const unsigned xi = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    const unsigned mi = __float_as_uint(fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1])));
    const auto b = __builtin_amdgcn_permlane16_swap(mi, mi, false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// The output accumulators live in the accumulation half of the register file, which MFMA reads and writes in place; only the
// rare rescale moves them through VALU registers.  The empty asm ties that move to the inside of the rescale branch (otherwise
// it is hoisted to the top of every tile and holds 128 VALU registers through the score phase).
#define PIN_ACC(x) asm volatile("" : "+a"(x))

// NH = heads per wavefront: 2 (32 query rows per workgroup, as described above) for long sequences; 1 (16 rows per workgroup,
// one head per wavefront: twice the workgroups, LDS-bound) when the launch would otherwise leave CUs idle.
template <int NH>
__global__ __launch_bounds__(256, 1) void attn_prefill_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ K,
                                                           const bf16_t* __restrict__ V, bf16_t* __restrict__ out, int S, int L,
                                                           int q_pos0, long q_head_stride, long kv_head_stride) {
    // four separate arrays, not [2][TILE]: the compiler tracks outstanding direct-to-LDS loads per LDS variable, so a read of
    // one buffer does not wait for the loads in flight to the others
    __shared__ __align__(1024) bf16_t k_s0[TILE];
    __shared__ __align__(1024) bf16_t k_s1[TILE];
    __shared__ __align__(1024) bf16_t v_s0[TILE];
    __shared__ __align__(1024) bf16_t v_s1[TILE];
    __shared__ __align__(16) float c_s[4][2][16];
    constexpr int RB = 16 * NH;
    const int rb = gridDim.x - 1 - blockIdx.x;                   // long rows first
    const int kvh = blockIdx.y;
    const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int h0 = kvh * (AH / AKV) + (NH == 2 ? 2 * (w & 1) : w);       // this wavefront's heads: h0 (, h0 + 1)
    const int r0 = rb * RB + (NH == 2 ? 16 * (w >> 1) : 0), row = r0 + n;   // this wavefront's 16 rows
    const bool row_ok = row < S;
    const int my_last = q_pos0 + row;                            // last key this query row may see
    const int kend = min(L, q_pos0 + min(rb * RB + RB - 1, S - 1) + 1);        // keys any row of the workgroup sees
    const int ntiles = (kend + KT - 1) / KT;
    const int kend_w = r0 < S ? min(L, q_pos0 + min(r0 + 15, S - 1) + 1) : 0;  // keys any row of this wavefront sees
    const int ntiles_w = (kend_w + KT - 1) / KT;

    // Q^T as the B operand of the score MFMA: lane (row n, group g) holds q[row][32 kb + 8 g .. + 8], for both heads
    bf16x8 bq[NH][8];
#pragma unroll
    for (int hh = 0; hh < NH; hh++) {
        const u32x4* qr = reinterpret_cast<const u32x4*>(q + (size_t)(h0 + hh) * q_head_stride + (size_t)(row_ok ? row : 0) * AD);
#pragma unroll
        for (int kb = 0; kb < 8; kb++) {
            u32x4 v = qr[kb * 4 + g];
            if (!row_ok) v = u32x4{0, 0, 0, 0};
            bq[hh][kb] = __builtin_bit_cast(bf16x8, v);
        }
    }
    // tile loader: wavefront w issues direct-to-LDS loads i = 0..7 of K and of V; load 8 w + i fills rows 2 (8 w + i) and
    // + 1 (one KiB): lane l lands at chunk position l & 31 of row 2 (8 w + i) + (l >> 5) and fetches chunk (l & 31) ^ (row & 15).
    // The per-lane byte offsets within a tile do not change from tile to tile.  A tile that would run past the end of the
    // sequence is shifted back to end at L (tile_row0): its first rows repeat keys of the tile before and are masked.  Only a
    // sequence shorter than one tile repeats its last key instead (slow path, first tile only).
    const char* kg = reinterpret_cast<const char*>(K + (size_t)kvh * kv_head_stride);
    const char* vg = reinterpret_cast<const char*>(V + (size_t)kvh * kv_head_stride);
    // byte offset of load 0 within a tile; load i differs by XOR with 1056 i (row bits 10..12, chunk bits 5..7)
    const unsigned ld_off0 = (unsigned)(16 * w + (lane >> 5)) * (AD * 2) + ((unsigned)((lane & 31) ^ (lane >> 5)) << 4);
    auto tile_row0 = [&](int t) { return max(0, min(t * KT, L - KT)); };
    // a copy of ld_off0 the compiler cannot see through: the offsets of the eight loads are then recomputed where they are
    // used (one XOR each) instead of living in registers the accumulators need
    auto opaque_off0 = [&]() {
        unsigned off0 = ld_off0;
        asm volatile("" : "+v"(off0));
        return off0;
    };
    auto load_one = [&](const char* src, bf16_t* dst, int t, int i, unsigned off0) {   // load i of tile t (L >= KT)
        // the row part of load i (2 i rows = 1024 i bytes) goes into the instruction's immediate offset, which moves the global
        // address and the LDS destination alike (at most 4095: the upper four loads start 4 KiB further in both)
        const auto gp = (const __attribute__((address_space(1))) void*)(src + (size_t)tile_row0(t) * (AD * 2) + 4096 * (i >> 2) +
                                                                        (off0 ^ (32u * i)));
        const auto lp = (__attribute__((address_space(3))) void*)(dst + (8 * w + 4 * (i >> 2)) * 512);
        switch (i & 3) {                                         // the immediate has to be a literal
            case 0: __builtin_amdgcn_global_load_lds(gp, lp, 16, 0, 0); break;
            case 1: __builtin_amdgcn_global_load_lds(gp, lp, 16, 1024, 0); break;
            case 2: __builtin_amdgcn_global_load_lds(gp, lp, 16, 2048, 0); break;
            default: __builtin_amdgcn_global_load_lds(gp, lp, 16, 3072, 0);
        }
    };
    auto load_rows = [&](const char* src, bf16_t* dst, int t) {  // one K or V tile: this wavefront's eight direct loads
        if (L >= KT) {
#pragma unroll
            for (int i = 0; i < 8; i++) load_one(src, dst, t, i, ld_off0);
        } else {                                                 // t = 0: rows past the end repeat the last key; they are masked
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const unsigned o = ld_off0 ^ (1056u * i);
                const unsigned off = (unsigned)min((int)(o >> 9), L - 1) * (AD * 2) + (o & 511u);
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + off),
                                                 (__attribute__((address_space(3))) void*)(dst + (8 * w + i) * 512), 16, 0, 0);
            }
        }
    };

    float m_run[NH];
    f32x4 Lsum[NH];                                              // row sums of P, accumulated by MFMA against a block of ones
    f32x4 O[NH][16];
#pragma unroll
    for (int hh = 0; hh < NH; hh++)
#pragma unroll
        for (int j = 0; j < 16; j++) O[hh][j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int hh = 0; hh < NH; hh++) m_run[hh] = NEG, Lsum[hh] = f32x4{0.f, 0.f, 0.f, 0.f};
    // A operand of the scores: row 16 kt + n of the tile, chunk (4 kb + g) ^ n
    const int ka_row = n * AD;
    // transposing load: within 16 lanes, lane 4q + i receives element i of the 8-byte chunks addressed by lanes q, q+4,
    // q+8, q+12; lane n of group g points at key 4g + n/4, columns 4 (n%4).. of the block and receives keys 4g..4g+3 of column n
    const int vrow = 4 * g + (n >> 2);                           // row within a 16-key block = its swizzle
    const int va_row = vrow * AD + 4 * (n & 1), vc0 = (n & 3) >> 1;

    // K fragment kb of sub-tile kt
    auto k_frag = [&](const bf16_t* ka, int kt, int kb) {
        // chunk (4 kb + g) ^ n; n < 16 leaves bit 4 alone, so fragments kb and kb + 4 share an address register
        return *reinterpret_cast<const bf16x8*>(ka + 16 * kt * AD + (((4 * (kb & 3) + g) ^ n) << 3) + 128 * (kb >> 2));
    };
    // scores of tile 0, S^T = K_tile . Q^T: each K fragment multiplies the Q^T of both heads; the fragments of the next
    // 16-key sub-tile are read while the MFMAs of the current one run
    auto scores_first = [&](const bf16_t* ka, f32x4 (&acc)[NH][4]) {
        bf16x8 Af[2][8];
#pragma unroll
        for (int kb = 0; kb < 8; kb++) Af[0][kb] = k_frag(ka, 0, kb);
#pragma unroll
        for (int kt = 0; kt < 4; kt++) {
            __builtin_amdgcn_sched_barrier(0);
            if (kt < 3) {
#pragma unroll
                for (int kb = 0; kb < 8; kb++) Af[(kt + 1) & 1][kb] = k_frag(ka, kt + 1, kb);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int hh = 0; hh < NH; hh++) acc[hh][kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kb = 0; kb < 8; kb++)
#pragma unroll
                for (int hh = 0; hh < NH; hh++)
                    acc[hh][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Af[kt & 1][kb], bq[hh][kb], acc[hh][kt], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    f32x4 accs[2][NH][4];                                        // scores of tile t live in accs[t & 1]
    AP_INIT();
    // One tile, software-pipelined around ONE workgroup barrier X(t):
    //     before X(t): the scores of tile t are in registers (computed during tile t - 1), P.V of tile t - 1 is done
    //     at X(t):     K(t + 1) and V(t) have landed; K(t)'s buffer takes K(t + 2), V(t - 1)'s buffer takes V(t + 1)
    //     after X(t):  the score MFMAs of tile t + 1 are interleaved, step by step, with the softmax VALU work of tile t
    //                  (online softmax in base 2 on the raw products: p = 2^(c s - m), c = 256^-0.5 log2 e; every row sees
    //                  key 0, so its maximum is finite from the first tile on and masked entries come out as 2^-huge = 0);
    //                  then P.V(t)
    // PAR = t & 1 picks the buffers at compile time.
    auto tile = [&](const int t, auto par) {
        constexpr int PAR = decltype(par)::value;
        f32x4 (&acc)[NH][4] = accs[PAR];
        f32x4 (&acc_next)[NH][4] = accs[PAR ^ 1];
        bf16_t* const k_cur = PAR ? k_s1 : k_s0;                 // K(t): consumed already, refilled with K(t + 2)
        const bf16_t* const k_nxt = PAR ? k_s0 : k_s1;           // K(t + 1)
        const bf16_t* const v_cur = PAR ? v_s1 : v_s0;           // V(t)
        bf16_t* const v_nxt = PAR ? v_s0 : v_s1;                 // V(t - 1): consumed, refilled with V(t + 1)
        AP_MARK(0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // this wavefront's loads of K(t + 1), V(t) have landed in LDS
        AP_MARK(1);
        __syncthreads();                                         // X(t)
        // While scores of a further tile are due (then L > KT), this wavefront's 16 loads of K(t + 2) and V(t + 1) are spread
        // over the steps below: a burst would stall on the memory pipeline's queue.  There a tile index past the end loads the
        // last tile again, harmlessly: nothing reads that buffer any more.
        const bool more = t + 1 < ntiles_w;                      // wavefront-uniform
        const int tk = min(t + 2, ntiles - 1), tv = min(t + 1, ntiles - 1);
        if (!more) {
            if (t + 2 < ntiles) load_rows(kg, k_cur, t + 2);
            if (t + 1 < ntiles) load_rows(vg, v_nxt, t + 1);
        }
        AP_MARK(2);
        if (t >= ntiles_w) return;                               // wavefront-uniform: the upper row block may see one tile more
        // only tiles that touch the diagonal or the end of the sequence need the mask (wavefront-uniform)
        if (t * KT + KT - 1 > q_pos0 + r0 || t * KT + KT > L) {
#pragma unroll
            for (int hh = 0; hh < NH; hh++)
#pragma unroll
                for (int kt = 0; kt < 4; kt++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int key = tile_row0(t) + 16 * kt + 4 * g + i;     // a shifted tile repeats keys below t * KT
                        if (!(key >= t * KT && key <= my_last && key < L)) acc[hh][kt][i] = NEG;
                    }
        }
        const bf16_t* ka = k_nxt + ka_row;
        const bf16_t* va = v_cur + va_row;
        auto v_frag = [&](int j, int q4) {
            return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) s16x4*)(const_cast<bf16_t*>(va + (16 * q4) * AD + (((2 * (j & 7) + vc0) ^ vrow) << 3) +
                                                                             128 * (j >> 3))));   // the swizzle (< 16) leaves bit 4 alone
        };
        s16x8 P[NH][2];
        s16x4 Bf[3][4];
        bool rescale = false;
        auto body = [&](auto with_scores) {
            constexpr bool SC = decltype(with_scores)::value;
            bf16x8 Af[2][8];
            if (SC) {
#pragma unroll
                for (int kb = 0; kb < 8; kb++) Af[0][kb] = k_frag(ka, 0, kb);
            }
            float m_new[NH];
#pragma unroll
            for (int hh = 0; hh < NH; hh++) {
                float mx = NEG;
#pragma unroll
                for (int kt = 0; kt < 4; kt++)
#pragma unroll
                    for (int i = 0; i < 4; i++) mx = fmaxf(mx, acc[hh][kt][i]);
                mx = max_over_groups(mx);
                // the reference point of a row only moves when its maximum has grown by more than 2^LAZY: until then p stays
                // below 2^LAZY, which bf16 and the f32 sums hold as well as values below 1, and the accumulators are left alone
                mx *= SCALE_LOG2E;
                m_new[hh] = mx > m_run[hh] + LAZY ? mx : m_run[hh];
                const float corr = __builtin_amdgcn_exp2f(m_run[hh] - m_new[hh]);   // m_run = NEG initially: 2^-huge = 0
                m_run[hh] = m_new[hh];
                c_s[w][hh][n] = corr;                            // all four groups store the same value: no divergent branch
                rescale |= corr != 1.0f;
            }
            AP_MARK(3);
            const unsigned step_off0 = SC ? opaque_off0() : 0u;
            // 32 steps: two score MFMAs of tile t + 1 (one K fragment x both heads) and one softmax element of tile t
            float pv_prev = 0.f;
#pragma unroll
            for (int st = 0; st < 32; st++) {
                const int kt = st >> 3, kb = st & 7;
                __builtin_amdgcn_sched_barrier(0);
                if (SC && (st & 1) == 0) {
                    if (st < 16)
                        load_one(kg, k_cur, tk, st >> 1, step_off0);
                    else
                        load_one(vg, v_nxt, tv, (st >> 1) - 8, step_off0);
                }
                if (SC) {
                    if (kt < 3) Af[(kt + 1) & 1][kb] = k_frag(ka, kt + 1, kb);
                    if (st >= 30) {                              // the first V fragments of P.V ride along with the last steps
#pragma unroll
                        for (int q4 = 0; q4 < 4; q4++) Bf[st - 30][q4] = v_frag(st - 30, q4);
                    }
#pragma unroll
                    for (int hh = 0; hh < NH; hh++)
                        acc_next[hh][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            Af[kt & 1][kb], bq[hh][kb], kb == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : acc_next[hh][kt], 0, 0, 0);
                }
                // softmax elements: NH * 16 of them over the 32 steps
#pragma unroll
                for (int e = (NH * 16 * st) / 32; e < (NH * 16 * (st + 1)) / 32; e++) {
                    const int hh = e >> 4, kt2 = (e >> 2) & 3, i = e & 3;
                    const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(acc[hh][kt2][i], SCALE_LOG2E, -m_new[hh]));
                    if (i & 1) {
                        const uint32_t pk = pack_bf(pv_prev, pv);
                        P[hh][kt2 >> 1][(kt2 & 1) * 4 + i - 1] = (short)(pk & 0xffff);
                        P[hh][kt2 >> 1][(kt2 & 1) * 4 + i] = (short)(pk >> 16);
                    }
                    pv_prev = pv;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (!SC) {
#pragma unroll
                for (int q4 = 0; q4 < 4; q4++) {
                    Bf[0][q4] = v_frag(0, q4);
                    Bf[1][q4] = v_frag(1, q4);
                }
            }
        };
        if (more)
            body(std::true_type{});
        else
            body(std::false_type{});
        wave_lds_sync();
        AP_MARK(4);
        if (__any(rescale)) {                                    // wavefront-uniform: most tiles leave every row's max alone
#pragma unroll
            for (int hh = 0; hh < NH; hh++) {
                const f32x4 c4 = *reinterpret_cast<const f32x4*>(&c_s[w][hh][4 * g]);
#pragma unroll
                for (int j = 0; j < 16; j++) {
                    PIN_ACC(O[hh][j]);
                    O[hh][j] *= c4;
                }
                PIN_ACC(Lsum[hh]);
                Lsum[hh] *= c4;
            }
        }
        AP_MARK(5);
        // P . V: the four transposed V fragments of a 16-column block are read two blocks ahead of their MFMAs and serve
        // both heads; the row sums are one more column block, P . 1 (the sum of exactly the rounded values that multiply V)
        {
            s16x8 ones;
#pragma unroll
            for (int e = 0; e < 8; e++) ones[e] = (short)0x3f80;
#pragma unroll
            for (int pp = 0; pp < 2; pp++)
#pragma unroll
                for (int hh = 0; hh < NH; hh++)
                    Lsum[hh] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, P[hh][pp]),
                                                                      __builtin_bit_cast(bf16x8, ones), Lsum[hh], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 16; j++) {
            __builtin_amdgcn_sched_barrier(0);
            if (j + 2 < 16) {
#pragma unroll
                for (int q4 = 0; q4 < 4; q4++) Bf[(j + 2) % 3][q4] = v_frag(j + 2, q4);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int pp = 0; pp < 2; pp++) {
                const s16x8 B = __builtin_shufflevector(Bf[j % 3][2 * pp], Bf[j % 3][2 * pp + 1], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int hh = 0; hh < NH; hh++)
                    O[hh][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, P[hh][pp]),
                                                                      __builtin_bit_cast(bf16x8, B), O[hh][j], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        AP_MARK(6);
        wave_lds_sync();                                         // c_s is rewritten by the next tile
    };

    load_rows(kg, k_s0, 0);
    load_rows(vg, v_s0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (ntiles > 1) load_rows(kg, k_s1, 1);
    if (ntiles_w > 0) scores_first(k_s0 + ka_row, accs[0]);
    for (int t = 0; t < ntiles; t += 2) {
        tile(t, std::integral_constant<int, 0>{});
        if (t + 1 < ntiles) tile(t + 1, std::integral_constant<int, 1>{});
    }
    AP_STORE();
    // ---- normalise and store: lane (n, g) holds rows 4g .. 4g+3 of column 16 j + n, and of the row sums (any column)
#pragma unroll
    for (int hh = 0; hh < NH; hh++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int orow = r0 + 4 * g + r;
            if (orow < S) {
                const float inv = 1.0f / Lsum[hh][r];
                bf16_t* dst = out + (size_t)(h0 + hh) * q_head_stride + (size_t)orow * AD + n;
#pragma unroll
                for (int j = 0; j < 16; j++) dst[16 * j] = f2bf(O[hh][j][r] * inv);
            }
        }
    }
}

}  // namespace

extern "C" {

// no workspace is needed any more; the entry point keeps its argument (may be null) so that callers do not change
long qt_gqa_prefill_workspace_bytes(int L) { return L < 0 ? -1 : 0; }

// q, out [8][S][256] bf16 (head stride q_head_stride elements), K, V [2][>=L][256] bf16 (head stride kv_head_stride):
// query i sits at absolute position q_pos0 + i and sees keys 0 .. q_pos0 + i (< L).
int qt_gqa_prefill_causal(const void* q, const void* K, const void* V, void* out, void* workspace, long workspace_bytes, int S,
                          int L, int q_pos0, long q_head_stride, long kv_head_stride, hipStream_t stream) {
    (void)workspace;
    (void)workspace_bytes;
    if (!q || !K || !V || !out) return QT_ERR_NULL;
    if (S < 0 || L < 1 || q_pos0 < 0 || q_head_stride < (long)S * AD || kv_head_stride < (long)L * AD) return QT_ERR_DIM;
    if (S == 0) return QT_OK;
    for (const void* p : {q, K, V, (const void*)out})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    if ((q_head_stride | kv_head_stride) & 7) return QT_ERR_ALIGN;
    // two heads per wavefront from about 4800 query rows on (measured: one head per wavefront 140 us at S = 4096 and 296 us at
    // S = 6144, two heads 156 us and 237 us); below that, 16-row blocks give twice the workgroups
    if ((S + 31) / 32 * AKV >= 304)
        hipLaunchKernelGGL(attn_prefill_kernel<2>, dim3((S + 31) / 32, AKV), dim3(256), 0, stream, (const bf16_t*)q, (const bf16_t*)K,
                           (const bf16_t*)V, (bf16_t*)out, S, L, q_pos0, q_head_stride, kv_head_stride);
    else
        hipLaunchKernelGGL(attn_prefill_kernel<1>, dim3((S + 15) / 16, AKV), dim3(256), 0, stream, (const bf16_t*)q, (const bf16_t*)K,
                           (const bf16_t*)V, (bf16_t*)out, S, L, q_pos0, q_head_stride, kv_head_stride);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

}  // extern "C"
