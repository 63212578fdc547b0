// Causal prefill attention, 8 query heads on 2 KV heads, head dim 256, for gfx950 (flash-attention forward on bf16 MFMA).
// Replaces the call mx.fast.scaled_dot_product_attention(q, K[:, :, :kv_len], V[:, :, :kv_len], scale=256**-0.5,
// mask="causal") of the reference's full-attention layers (qwen35/model.py:160-167, qwen35/prefill.py:468).
//
// attn_prefill_kernel<NH>: one workgroup = 16 NH query rows x the 4 query heads that share a KV head, on eight wavefronts in
// two roles; NH = heads per pair of wavefronts:
//   NH = 2   32 rows; every K or V fragment read from LDS feeds two MFMAs (one per head): launches of about 1500 rows and more
//   NH = 1   16 rows: twice the workgroups (and twice the LDS traffic per MFMA), for launches that would leave CUs idle
// The arithmetic, per 64-key tile and 16 rows of a head:
//     S^T[keys x rows] = K_tile . Q^T     A = K rows from LDS, B = Q^T resident in registers (16x16x32 bf16 MFMA)
//     online softmax in the accumulator layout: lane (row n, group g) holds keys 4g..4g+3 of each 16-key sub-tile
//     O[rows x 256]   += P . V            A = two exponentiated S^T accumulators packed to bf16 (they ARE the A operand
//                                         when a 32-key block is enumerated as 16 (j >> 2) + 4 g + (j & 3)),
//                                         B = V through the transposing LDS load (4 consecutive keys of one column);
//                                         the row sums are one more column block, P . 1
// K / V tiles travel HBM -> LDS directly (global_load_lds_dwordx4: 64 lanes x 16 bytes land as one contiguous KiB, no
// registers in between) into double-buffered tiles.  The LDS rows are unpadded (a direct load cannot pad); instead the
// 16-byte chunks of row r are stored XOR-swizzled by r & 15 (the loading lane picks the matching global chunk), which keeps
// the fragment reads of 16 rows on distinct banks.  The tile loop runs around one workgroup barrier per tile: the score MFMAs
// of tile t + 1 follow the exponentials of tile t, which are taken against the running reference points before the tile's
// row maxima are known; the bet is checked afterwards (see `publish` below).
#include "qt_common.h"

#include <algorithm>
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
constexpr int FRAG_AHEAD = 5;          // steps between the LDS read of a K fragment and its MFMAs in the tile loop
constexpr int V_FRAG_AHEAD = 2;        // 16-column blocks between the LDS reads of V fragments and their MFMAs
constexpr int TILE = KT * AD;          // elements of one K or V tile in LDS (32 KiB), rows unpadded, chunks swizzled

// PHASE_FENCE(): the phases of an iteration are scheduled separately
#define PHASE_FENCE() __builtin_amdgcn_sched_barrier(0)

// One direct-to-LDS load of 16 bytes per lane (global_load_lds_dwordx4): lane l fetches base + voff + IMM and the 64 pieces land
// at lds + IMM + 16 l.  Issued as inline assembly, not through the builtin: while a direct-to-LDS load that the compiler knows
// of is outstanding, it closes every wait for an LDS read with lgkmcnt(0) (the load counts as an access of both memories), and
// the tile loop below always has such loads in flight, so each of its fragment reads would be waited for in full.  These loads
// are waited for by hand (vmcnt(0) before the workgroup barrier of a tile).  base and lds are wavefront-uniform.
// LDS byte address of a __shared__ array, taken of the array itself: a constant.  (Taken of a pointer that has been moved, the
// cast from a generic pointer costs a null test and two scalar registers per use.)
__device__ __forceinline__ unsigned lds_address(const bf16_t* shared_array) {
    return (unsigned)(size_t)(__attribute__((address_space(3))) const void*)shared_array;
}
template <int IMM>
__device__ __forceinline__ void lds_dma16(const char* base, unsigned voff, unsigned lds) {
    const unsigned la = __builtin_amdgcn_readfirstlane(lds);
    unsigned keep;                                                // M0 belongs to the compiler: put back what it held
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%4\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "v"(voff), "s"(base), "s"(la), "n"(IMM)
                 : "memory");
}
// four such loads, KiB 0 .. 3 behind lds, under one setting of M0 (a wavefront issues one instruction every four clocks, and
// the tile loop is bound by exactly that, so the five scalar instructions around a single load count)
__device__ __forceinline__ void lds_dma16x4(const char* base, unsigned v0, unsigned v1, unsigned v2, unsigned v3, unsigned lds) {
    const unsigned la = __builtin_amdgcn_readfirstlane(lds);
    unsigned keep;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %6\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, %5\n\tglobal_load_lds_dwordx4 %2, %5 offset:1024\n\t"
                 "global_load_lds_dwordx4 %3, %5 offset:2048\n\tglobal_load_lds_dwordx4 %4, %5 offset:3072\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "v"(v0), "v"(v1), "v"(v2), "v"(v3), "s"(base), "s"(la)
                 : "memory");
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

// Key split.  A causal launch with few workgroups is as slow as its longest row block, twice the average.  With tmax > 0 the
// tiles of a row block (RB = 16 or 32 rows) are cut into parts of tmax tiles, one workgroup per part; a block with more than
// one part leaves unnormalised partial results (O, reference point m, row sums l) in the workspace and
// attn_prefill_merge_kernel combines them.  Block i counts ceil((p + i + 1) / c) parts, p = ceil(q_pos0 / RB),
// c = (64 / RB) tmax (RB rows advance the visible keys by RB / 64 of a tile), which is never fewer than its tiles need (a part
// may be empty); the parts of blocks 0 .. r-1 are then parts_upto(p + r, c) - parts_upto(p, c), and a workgroup inverts that
// sum to find its part.
__host__ __device__ inline long parts_upto(long n, long c) {      // sum over j = 1 .. n of ceil(j / c)
    const long k = n / c;
    return c * (k * (k + 1) / 2) + (n - k * c) * (k + 1);
}
// elements of one part's O, [4 heads][RB rows][256] in half precision (each row divided by its row sum, so that the values are
// weighted means of V), and floats of its m, l, [4 heads][m | l][RB rows] (RB = rows of a block: 16 or 32)
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
constexpr int part_o_floats(int RB) { return 4 * RB * AD; }
constexpr long part_bytes(int RB) { return (long)part_o_floats(RB) * 2 + (long)(4 * 2 * RB) * 4; }
constexpr int part_ml_floats(int RB) { return 4 * 2 * RB; }

// a word of LDS as a volatile object in the LDS address space (through a generic pointer, a volatile access is a flat
// instruction, which is also counted, and waited for, as an access of global memory)
__device__ __forceinline__ volatile __attribute__((address_space(3))) int* lds_word(int* shared_word) {
    return (volatile __attribute__((address_space(3))) int*)shared_word;
}

// The tile loop, with the two halves of a tile's work on different wavefronts.  The eight wavefronts of a workgroup, two per
// SIMD, form four pairs: wavefront pr (0 .. 3, the "score" wavefront of pair pr) computes the scores and the softmax of the
// pair's 16 rows x NH heads (NH = 2: rows 16 (pr >> 1) .. + 16 of the block, heads 2 (pr & 1), + 1; NH = 1: the block's 16 rows,
// head pr), and wavefront 4 + pr (the pair's "output" wavefront) multiplies the resulting P by V, one tile behind.  A
// wavefront's instructions issue one after the other (an MFMA holds its wavefront for about as long as it holds the matrix
// unit, and every LDS read, exponential or wait comes on top), while two wavefronts of a SIMD do overlap: one feeds the unit
// Q K^T while the other reads V fragments, and the softmax arithmetic of the one runs beside the P V MFMAs of the other.
// (The whole loop on one wavefront per SIMD, four per workgroup, measured 5 - 12 % slower on the same rows and heads; the
// compiler's order within the score wavefront, the softmax arithmetic as one block and then the MFMA steps back to back,
// measures better than the same arithmetic tied into the steps.)  With eight wavefronts the 512 registers of a SIMD lane are
// split in two, 256 per wavefront and no separate accumulation half: for NH = 2 the score side holds Q^T (64 registers) and
// two tiles of scores (64), the output side O (128).
//     iteration t (after barrier X(t): K(t + 1) and V(t - 1) are in LDS):
//         score wavefront:  softmax of tile t (its scores are in registers since iteration t - 1) and the score MFMAs of
//                           tile t + 1; then P(t), as packed A operands, and the rows' rescale factors go to LDS
//         output wavefront: takes P(t - 1) and the factors from LDS, rescales O and the row sums if any row's reference
//                           moved, O += P(t - 1) V(t - 1)
//         all eight:        direct-to-LDS loads of K(t + 2) into K(t)'s buffer and of V(t) into V(t - 2)'s
// P has one buffer per pair: the output wavefront reads it into registers first thing in an iteration and says so
// (taken_s[pr] = t), and the score wavefront, which writes the next P a few thousand clocks later, looks at that word first.
// grid = (row blocks, or parts when tmax > 0) x KV heads in one dimension, the KV head varying fastest: workgroups are
// dispatched in the order of their index, so both heads' long row blocks come first.
template <int NH>
__global__ __launch_bounds__(512) void attn_prefill_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ K,
                                                              const bf16_t* __restrict__ V, bf16_t* __restrict__ out, int S, int L,
                                                              int q_pos0, long q_head_stride, long kv_head_stride, int tmax,
                                                              _Float16* __restrict__ part_o, float* __restrict__ part_ml) {
    __shared__ __align__(1024) bf16_t kv_s[4 * TILE];            // K tiles of even / odd iterations, then the V tiles
    __shared__ __align__(16) u32x4 p_s[4][NH][2][64];             // [pair][head][32-key half][lane]: P as the lanes hold it
    __shared__ __align__(16) float c_s[4][NH][16];               // [pair][head][row]: factor of a row whose reference moved
    __shared__ float m_s[4][NH][16];                             // final reference points (only the parts' epilogue needs them)
    __shared__ int moved_s[4];                                   // pair: did any reference move in the tile whose P lies in p_s
    __shared__ int taken_s[4];                                   // pair: the iteration in which p_s / c_s / moved_s were last read
    constexpr int RB = 16 * NH;
    const int nitems = gridDim.x / AKV, item = blockIdx.x / AKV;
    int rb = nitems - 1 - item;                                  // long rows first
    int part = 0, nparts = 1;
    if (tmax > 0) {                                              // items are parts, again from the long end
        const int c = (KT / RB) * tmax, p = (q_pos0 + RB - 1) / RB;
        const long y = (long)rb + parts_upto(p, c);              // parts_upto(nn) <= y < parts_upto(nn + 1), nn = p + row block
        int k = 0;
        while ((long)c * ((k + 1) * (k + 2) / 2) <= y) k++;
        const int nn = k * c + (int)((y - (long)c * (k * (k + 1) / 2)) / (k + 1));
        part = (int)(y - parts_upto(nn, c));
        nparts = k + 1;
        rb = nn - p;
    }
    const int kvh = blockIdx.x % AKV;
    const size_t slot = (size_t)kvh * nitems + (nitems - 1 - item);     // parts of a block: consecutive slots
    const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int pr = w & 3;                                        // pair; w >> 2: 0 = score, 1 = output wavefront
    const int hq0 = NH == 2 ? 2 * (pr & 1) : pr;                  // this pair's first head within the KV group
    const int h0 = kvh * (AH / AKV) + hq0;
    const int r0 = rb * RB + (NH == 2 ? 16 * (pr >> 1) : 0), row = r0 + n;
    const bool row_ok = row < S;
    const int my_last = q_pos0 + row;                            // last key this query row may see
    const int kend = min(L, q_pos0 + min(rb * RB + RB - 1, S - 1) + 1);        // keys any row of the workgroup sees
    const int ntiles = (kend + KT - 1) / KT;
    const int kend_w = r0 < S ? min(L, q_pos0 + min(r0 + 15, S - 1) + 1) : 0;  // keys any row of this pair sees
    const int ntiles_w = (kend_w + KT - 1) / KT;
    // this workgroup's tiles [ta, tb); tw: where this pair's rows end (the upper rows of a block may see one tile more)
    const int ta = part * tmax, tb = tmax > 0 ? min(ntiles, ta + tmax) : ntiles;
    const int tw = min(ntiles_w, tb);

    // tile loader: wavefront w issues four direct-to-LDS loads of K and four of V per tile; load i fills rows 8 w + 2 i, + 1
    // (one KiB): lane l lands at chunk position l & 31 of row 8 w + 2 i + (l >> 5) and fetches chunk (l & 31) ^ (row & 15).  The
    // per-lane byte offsets within a tile do not change from tile to tile: load i differs from load 0 by 2 i rows, which go into
    // the instruction's immediate offset (it moves the global address and the LDS destination alike), and by an XOR of the
    // chunk with 2 i.  A tile that would run past the end of the sequence is shifted back to end at L (tile_row0): its first
    // rows repeat keys of the tile before and are masked.  Only a sequence shorter than one tile repeats its last key instead.
    const char* kg = reinterpret_cast<const char*>(K + (size_t)kvh * kv_head_stride);
    const char* vg = reinterpret_cast<const char*>(V + (size_t)kvh * kv_head_stride);
    const unsigned ld_row0 = 8u * w + (lane >> 5);
    const unsigned ld_off0 = ld_row0 * (AD * 2) + ((unsigned)((lane & 31) ^ (ld_row0 & 15u)) << 4);
    auto tile_row0 = [&](int t) { return max(0, min(t * KT, L - KT)); };
    // a copy of ld_off0 the compiler cannot see through: the offsets of the four loads are then recomputed where they are
    // used (one XOR each) instead of living in registers through the loop
    auto opaque_off0 = [&]() {
        unsigned off0 = ld_off0;
        asm volatile("" : "+v"(off0));
        return off0;
    };
    const unsigned w_lds = 4096u * w;                            // this wavefront's 4 KiB of a tile buffer
    auto load_four = [&](const char* src, unsigned dst, int t, unsigned off0) {
        if (L >= KT) {
            const char* base = src + (size_t)tile_row0(t) * (AD * 2);
            lds_dma16x4(base, off0, off0 ^ 32u, off0 ^ 64u, off0 ^ 96u, dst + w_lds);
        } else {                                                 // t = 0: rows past the end repeat the last key; they are masked
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const unsigned o = (ld_off0 ^ (32u * i)) + 1024u * i;
                lds_dma16<0>(src, (unsigned)min((int)(o >> 9), L - 1) * (AD * 2) + (o & 511u), dst + w_lds + 1024u * i);
            }
        }
    };
    // A operand of the scores: row 16 kt + n of the tile, chunk (4 kb + g) ^ n
    const int ka_row = n * AD;
    // transposing load: within 16 lanes, lane 4q + i receives element i of the 8-byte chunks addressed by lanes q, q+4,
    // q+8, q+12; lane n of group g points at key 4g + n/4, columns 4 (n%4).. of the block and receives keys 4g..4g+3 of column n
    const int vrow = 4 * g + (n >> 2);                           // row within a 16-key block = its swizzle
    const int va_row = vrow * AD + 4 * (n & 1), vc0 = (n & 3) >> 1;
    // K fragment kb of sub-tile kt: chunk (4 kb + g) ^ n; n < 16 leaves bit 4 alone, so fragments kb and kb + 4 share an
    // address register
    auto k_frag = [&](const bf16_t* ka, int kt, int kb) {
        return *reinterpret_cast<const bf16x8*>(ka + 16 * kt * AD + (((4 * (kb & 3) + g) ^ n) << 3) + 128 * (kb >> 2));
    };

    if (tid < 4) taken_s[tid] = -1, moved_s[tid] = 0;
    if (tid < 4 * NH * 16) (&m_s[0][0][0])[tid] = NEG;
    if (ta < tb) {                                               // (a part past the block's last tile is empty)
        load_four(kg, lds_address(kv_s), ta, ld_off0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tb - ta > 1) load_four(kg, lds_address(kv_s) + 2 * TILE, ta + 1, ld_off0);
    }

    if (w < 4) {
        // ------------------------------------------------------------------------------------------ score wavefront
        if (ta >= tb) return;
        // Q^T as the B operand of the score MFMA: lane (row n, group g) holds q[row][32 kb + 8 g .. + 8] of each head
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
        float m_run[NH];
#pragma unroll
        for (int hh = 0; hh < NH; hh++) m_run[hh] = NEG;
        // scores of the first tile, S^T = K_tile . Q^T: each K fragment multiplies the Q^T of every head of the pair; the fragments
        // of the next 16-key sub-tile are read while the MFMAs of the current one run
        auto first_scores = [&](f32x4 (&acc0)[NH][4]) {
            const bf16_t* ka = kv_s + ka_row;
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
                for (int hh = 0; hh < NH; hh++) acc0[hh][kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kb = 0; kb < 8; kb++)
#pragma unroll
                    for (int hh = 0; hh < NH; hh++)
                        acc0[hh][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Af[kt & 1][kb], bq[hh][kb], acc0[hh][kt], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        // the scores of tile t live in accs[(t - ta) & 1]: two iterations in the source, so that both sets are registers
        f32x4 accs[2][NH][4] = {};
        if (tw > ta) first_scores(accs[0]);
        auto s_iter = [&](const int t, f32x4 (&acc)[NH][4], f32x4 (&acc_next)[NH][4]) {
            const unsigned par = (unsigned)(t - ta) & 1u;
            const unsigned k_cur = lds_address(kv_s) + par * (2 * TILE);           // K(t): consumed, refilled with K(t + 2)
            const bf16_t* const k_nxt = kv_s + (par ^ 1u) * TILE;                  // K(t + 1)
            const unsigned v_new = lds_address(kv_s) + 4 * TILE + par * (2 * TILE);   // takes V(t)
            PHASE_FENCE();
            // this wavefront's loads of K(t + 1), V(t - 1) have landed, and its writes of P(t - 1) (the wait for those is
            // spelled out: at a loop header the compiler does not always see the LDS stores that arrive over the back edge)
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            PHASE_FENCE();
            __syncthreads();                                         // X(t)
            // While scores of a further tile are due (then L > KT), this wavefront's loads of K(t + 2) and V(t) ride on the steps
            // below: a burst would stall on the memory pipeline's queue.  There a tile index past the end loads the last tile
            // again, harmlessly: nothing reads that buffer any more.
            const bool more = t + 1 < tw;                            // wavefront-uniform
            const int tk = min(t + 2, tb - 1);
            if (!more) {
                if (t + 2 < tb) load_four(kg, k_cur, t + 2, opaque_off0());
                if (t < tb) load_four(vg, v_new, t, opaque_off0());
            }
            PHASE_FENCE();
            if (t >= tw) return;
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
            // Online softmax in base 2 on the raw products: p = 2^(c s - m), c = 256^-0.5 log2 e; every row sees key 0, so its
            // maximum is finite from the first tile on and masked entries come out as 2^-huge = 0.  The exponentials are taken
            // against the running reference point of each row at once, on the bet that no row's maximum grows by more than
            // 2^LAZY in this tile (true for all but the first few tiles of a row block); the maxima are folded in beside them
            // and the bet is checked here.  A reference point only moves when the row's maximum has grown by more than 2^LAZY:
            // until then p stays below 2^LAZY, which bf16 and the f32 sums hold as well as values below 1.
            auto publish = [&](s16x8 (&P)[NH][2], float (&mx)[NH], int taken_early) {
                bool grow = false;
#pragma unroll
                for (int hh = 0; hh < NH; hh++) {
                    mx[hh] = max_over_groups(mx[hh]) * SCALE_LOG2E;
                    grow |= mx[hh] > m_run[hh] + LAZY;
                }
                const bool any_grow = __any(grow);
                float corr[NH];
#pragma unroll
                for (int hh = 0; hh < NH; hh++) corr[hh] = 1.f;
                if (any_grow) {                                      // wavefront-uniform and rare
#pragma unroll
                    for (int hh = 0; hh < NH; hh++) {
                        const float m_new = mx[hh] > m_run[hh] + LAZY ? mx[hh] : m_run[hh];
                        corr[hh] = __builtin_amdgcn_exp2f(m_run[hh] - m_new);    // m_run = NEG initially: 2^-huge = 0
                        m_run[hh] = m_new;
                        // this tile's p again, against the new reference points (rows that did not move get the same bits)
#pragma unroll
                        for (int kt2 = 0; kt2 < 4; kt2++)
#pragma unroll
                            for (int i = 0; i < 4; i += 2) {
                                const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(acc[hh][kt2][i], SCALE_LOG2E, -m_new));
                                const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(acc[hh][kt2][i + 1], SCALE_LOG2E, -m_new));
                                const uint32_t pk = pack_bf(p0, p1);
                                P[hh][kt2 >> 1][(kt2 & 1) * 4 + i] = (short)(pk & 0xffff);
                                P[hh][kt2 >> 1][(kt2 & 1) * 4 + i + 1] = (short)(pk >> 16);
                            }
                    }
                }
                // the pair's buffers are free once the output wavefront has read tile t - 1 out of them (it does so first
                // thing in this iteration; the word was read some steps ago, so that its LDS latency is not waited for here).
                // The wait is bounded (the word is always written, and a bound costs nothing); a wait that does run out must not
                // pass in silence: the pair's rows are then rescaled by NaN, which every later stage carries to the output.
                bool gave_up = false;
                if (t > ta && __builtin_amdgcn_readfirstlane(taken_early) != t) {
                    gave_up = true;
                    for (int spin = 0; spin < (1 << 20); spin++) {
                        if (__builtin_amdgcn_readfirstlane(*lds_word(&taken_s[pr])) == t) {
                            gave_up = false;
                            break;
                        }
                        __builtin_amdgcn_s_sleep(1);
                    }
                }
                asm volatile("" ::: "memory");
                if (any_grow || gave_up) {
#pragma unroll
                    for (int hh = 0; hh < NH; hh++)              // all four groups store the same value
                        c_s[pr][hh][n] = gave_up ? __builtin_nanf("") : corr[hh];
                }
                moved_s[pr] = any_grow || gave_up ? 1 : 0;
#pragma unroll
                for (int hh = 0; hh < NH; hh++)
#pragma unroll
                    for (int pp = 0; pp < 2; pp++) p_s[pr][hh][pp][lane] = __builtin_bit_cast(u32x4, P[hh][pp]);
                if (t == tw - 1) {
#pragma unroll
                    for (int hh = 0; hh < NH; hh++) m_s[pr][hh][n] = m_run[hh];
                }
            };
            auto body = [&](auto with_scores) {
                constexpr bool SC = decltype(with_scores)::value;
                s16x8 P[NH][2];
                float mx[NH];
#pragma unroll
                for (int hh = 0; hh < NH; hh++) mx[hh] = NEG;
                bf16x8 Af[FRAG_AHEAD + 1];
                if (SC) {
#pragma unroll
                    for (int f = 0; f < FRAG_AHEAD; f++) Af[f] = k_frag(ka, f >> 3, f & 7);
                }
                // softmax elements 2 e, 2 e + 1 of tile t
                auto softmax_pair = [&](int e) {
                    const int hh = e >> 3, kt2 = (e >> 1) & 3, i = 2 * (e & 1);
                    const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(acc[hh][kt2][i], SCALE_LOG2E, -m_run[hh]));
                    const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(acc[hh][kt2][i + 1], SCALE_LOG2E, -m_run[hh]));
                    mx[hh] = fmaxf(mx[hh], fmaxf(acc[hh][kt2][i], acc[hh][kt2][i + 1]));
                    const uint32_t pk = pack_bf(p0, p1);
                    P[hh][kt2 >> 1][(kt2 & 1) * 4 + i] = (short)(pk & 0xffff);
                    P[hh][kt2 >> 1][(kt2 & 1) * 4 + i + 1] = (short)(pk >> 16);
                };
                PHASE_FENCE();
                const unsigned step_off0 = SC ? opaque_off0() : 0u;
                int taken_early = -1;
                // 32 steps: one K fragment read (FRAG_AHEAD steps ahead, a ring) and its MFMAs, one per head.  The softmax
                // pairs are written beside them, but nothing ties them to their step: the compiler gathers the arithmetic
                // into one block beside the steps, which measures better than the same arithmetic held between the MFMAs.
#pragma unroll
                for (int st = 0; st < 32; st++) {
                    const int kt = st >> 3, kb = st & 7;
                    __builtin_amdgcn_sched_barrier(0);
                    if (SC && st == 0) load_four(kg, k_cur, tk, step_off0);
                    if (SC && st == 20) load_four(vg, v_new, t, step_off0);
                    if (SC) {
                        if (st + FRAG_AHEAD < 32)
                            Af[(st + FRAG_AHEAD) % (FRAG_AHEAD + 1)] = k_frag(ka, (st + FRAG_AHEAD) >> 3, (st + FRAG_AHEAD) & 7);
#pragma unroll
                        for (int hh = 0; hh < NH; hh++)
                            acc_next[hh][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                                Af[st % (FRAG_AHEAD + 1)], bq[hh][kb], kb == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : acc_next[hh][kt], 0, 0, 0);
                    }
                    if (st % (4 / NH) == 0) softmax_pair(st / (4 / NH));       // 8 NH pairs over the 32 steps
                    if (st == 20) taken_early = *lds_word(&taken_s[pr]);   // (read early: its LDS latency passes under the steps)
                }
                __builtin_amdgcn_sched_barrier(0);
                publish(P, mx, taken_early);
            };
            if (more)
                body(std::true_type{});
            else
                body(std::false_type{});
            PHASE_FENCE();
        };
        for (int t = ta; t <= tb; t += 2) {
            s_iter(t, accs[0], accs[1]);
            if (t + 1 <= tb) s_iter(t + 1, accs[1], accs[0]);
        }
        return;
    }
    // ---------------------------------------------------------------------------------------------- output wavefront
    f32x4 O[NH][16];
    f32x4 Lsum[NH];                                                  // row sums of P, accumulated by MFMA against a block of ones
#pragma unroll
    for (int hh = 0; hh < NH; hh++) {
        Lsum[hh] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 16; j++) O[hh][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // iterations in which this wavefront only loads: the first one (no P yet), and those after its rows' last tile
    auto idle_iter = [&](int t) {
        const unsigned par = (unsigned)(t - ta) & 1u;
        PHASE_FENCE();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        PHASE_FENCE();
        __syncthreads();                                             // X(t)
        if (t + 2 < tb) load_four(kg, lds_address(kv_s) + par * (2 * TILE), t + 2, opaque_off0());
        if (t < tb) load_four(vg, lds_address(kv_s) + 4 * TILE + par * (2 * TILE), t, opaque_off0());
    };
    if (ta < tb) idle_iter(ta);
    for (int t = ta + 1; t <= tw; t++) {                             // (tw <= tb; nothing if tw <= ta)
        const unsigned par = (unsigned)(t - ta) & 1u;
        const unsigned k_cur = lds_address(kv_s) + par * (2 * TILE);               // takes K(t + 2)
        const unsigned v_new = lds_address(kv_s) + 4 * TILE + par * (2 * TILE);    // takes V(t)
        const bf16_t* const v_cur = kv_s + 2 * TILE + (par ^ 1u) * TILE;           // V(t - 1)
        PHASE_FENCE();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        PHASE_FENCE();
        __syncthreads();                                             // X(t)
        const int mv = __builtin_amdgcn_readfirstlane(moved_s[pr]);
        s16x8 P[NH][2];
#pragma unroll
        for (int hh = 0; hh < NH; hh++)
#pragma unroll
            for (int pp = 0; pp < 2; pp++) P[hh][pp] = __builtin_bit_cast(s16x8, p_s[pr][hh][pp][lane]);
        f32x4 c4[NH];
#pragma unroll
        for (int hh = 0; hh < NH; hh++) c4[hh] = mv ? *reinterpret_cast<const f32x4*>(&c_s[pr][hh][4 * g]) : f32x4{1.f, 1.f, 1.f, 1.f};
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        *lds_word(&taken_s[pr]) = t;
        asm volatile("" ::: "memory");
        const bf16_t* va = v_cur + va_row;
        auto v_frag = [&](int j, int q4) {
            return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) s16x4*)(const_cast<bf16_t*>(va + (16 * q4) * AD + (((2 * (j & 7) + vc0) ^ vrow) << 3) +
                                                                             128 * (j >> 3))));
        };
        s16x4 Bf[V_FRAG_AHEAD + 1][4];
#pragma unroll
        for (int j = 0; j < V_FRAG_AHEAD; j++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) Bf[j][q4] = v_frag(j, q4);
        if (mv) {                                                    // a reference moved: rescale what is accumulated
#pragma unroll
            for (int hh = 0; hh < NH; hh++) {
#pragma unroll
                for (int j = 0; j < 16; j++) O[hh][j] *= c4[hh];
                Lsum[hh] *= c4[hh];
            }
        }
        PHASE_FENCE();
        {                                                            // the row sums: P . 1, the sum of exactly the rounded values
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
        const unsigned step_off0 = opaque_off0();
#pragma unroll
        for (int j = 0; j < 16; j++) {
            __builtin_amdgcn_sched_barrier(0);
            if (j == 0 && t + 2 < tb) load_four(kg, k_cur, t + 2, step_off0);
            if (j == 8 && t < tb) load_four(vg, v_new, t, step_off0);
            if (j + V_FRAG_AHEAD < 16) {
#pragma unroll
                for (int q4 = 0; q4 < 4; q4++) Bf[(j + V_FRAG_AHEAD) % (V_FRAG_AHEAD + 1)][q4] = v_frag(j + V_FRAG_AHEAD, q4);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int pp = 0; pp < 2; pp++) {
                const s16x8 B = __builtin_shufflevector(Bf[j % (V_FRAG_AHEAD + 1)][2 * pp], Bf[j % (V_FRAG_AHEAD + 1)][2 * pp + 1], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int hh = 0; hh < NH; hh++)
                    O[hh][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, P[hh][pp]),
                                                                      __builtin_bit_cast(bf16x8, B), O[hh][j], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        PHASE_FENCE();
    }
    if (ta < tb)
        for (int t = max(tw, ta) + 1; t <= tb; t++) idle_iter(t);
    // ---- normalise and store: lane (n, g) holds rows 4g .. 4g+3 of column 16 j + n, and of the row sums (any column)
    if (nparts > 1) {
        // One part of several: leave O / l, m, l of this pair's heads as they are.  A row that sees no key of this part (its
        // last key lies before the part's first) has exponentiated masked scores against a masked maximum: it is written as
        // the neutral element (m = NEG, l = 0, O = 0).
        const int first_key = ta * KT, lr0 = r0 - rb * RB;
#pragma unroll
        for (int hh = 0; hh < NH; hh++) {
            const int hq = hq0 + hh;
            _Float16* po = part_o + (slot * 4 + hq) * (RB * AD);
            float* pml = part_ml + (slot * 4 + hq) * (2 * RB);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int lr = lr0 + 4 * g + r;
                const bool seen = q_pos0 + rb * RB + lr >= first_key;
                const float inv = seen ? 1.0f / Lsum[hh][r] : 0.f;
#pragma unroll
                for (int j = 0; j < 16; j++) po[lr * AD + 16 * j + n] = (_Float16)(seen ? O[hh][j][r] * inv : 0.f);
                if (n == 0) pml[RB + lr] = seen ? Lsum[hh][r] : 0.f;
            }
            if (g == 0) pml[lr0 + n] = my_last >= first_key ? m_s[pr][hh][n] : NEG;
        }
        return;
    }
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

// Combines the parts of the row blocks that were split: grid = (split blocks, KV heads, 4 heads of the group x 16-row halves of
// a block); thread (row, 16-column group) of 16 x 256 outputs.  out = sum_p w_p O_p / sum_p w_p, w_p = 2^(m_p - m) l_p, parts in order; a
// thread's loads of O do not depend on the factors, so all parts are in flight together.
template <int RB>
__global__ __launch_bounds__(256) void attn_prefill_merge_kernel(const _Float16* __restrict__ part_o, const float* __restrict__ part_ml,
                                                                 bf16_t* __restrict__ out, int S, int q_pos0, int tmax, long slots_per_kv,
                                                                 long q_head_stride) {
    constexpr int PO = part_o_floats(RB), PML = part_ml_floats(RB);
    const int c = (KT / RB) * tmax, p = (q_pos0 + RB - 1) / RB;
    const int rb = max(0, c - p) + blockIdx.x;                   // the first block with two parts is c - p
    const int np = (p + rb) / c + 1;
    const size_t slot0 = (size_t)blockIdx.y * slots_per_kv + (size_t)(parts_upto(p + rb, c) - parts_upto(p, c));
    const int hq = blockIdx.z / (RB / 16), cg = threadIdx.x & 15;
    {
        const int lr = 16 * (blockIdx.z % (RB / 16)) + (threadIdx.x >> 4);
        if (rb * RB + lr >= S) return;
        const _Float16* po = part_o + (slot0 * 4 + hq) * (RB * AD) + lr * AD + cg * 16;
        const float* pml = part_ml + (slot0 * 4 + hq) * (2 * RB) + lr;
        float m = NEG;
        for (int pp = 0; pp < np; pp++) m = fmaxf(m, pml[(size_t)pp * PML]);
        float l = 0.f;
        f32x4 acc[4];
#pragma unroll
        for (int i = 0; i < 4; i++) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
        for (int pp = 0; pp < np; pp++) {
            half8 oh[2];
#pragma unroll
            for (int i = 0; i < 2; i++) oh[i] = reinterpret_cast<const half8*>(po + (size_t)pp * PO)[i];
            const float f = __builtin_amdgcn_exp2f(pml[(size_t)pp * PML] - m) * pml[(size_t)pp * PML + RB];
            l += f;
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[i][e] += f * (float)oh[i >> 1][4 * (i & 1) + e];
        }
        const float inv = 1.0f / l;
        uint32_t pk[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            pk[2 * i] = pack_bf(acc[i][0] * inv, acc[i][1] * inv);
            pk[2 * i + 1] = pack_bf(acc[i][2] * inv, acc[i][3] * inv);
        }
        u32x4* dst = reinterpret_cast<u32x4*>(out + (size_t)(blockIdx.y * (AH / AKV) + hq) * q_head_stride + (size_t)(rb * RB + lr) * AD + cg * 16);
        dst[0] = u32x4{pk[0], pk[1], pk[2], pk[3]};
        dst[1] = u32x4{pk[4], pk[5], pk[6], pk[7]};
    }
}

}  // namespace

namespace {

inline bool two_heads_per_wave(int S) { return (S + 31) / 32 * AKV >= 288; }   // from 4577 rows on: 32-row blocks unsplit

// The key split of a launch: tmax = 0 (none) or the tiles per part, parts = grid width, split_blocks = blocks with several parts.
// Only launches that leave CUs without a workgroup are split (fewer than 2048 query rows: a short continuation of a long
// prefix, a short prompt), and only as far as the idle CUs go: a part holds the smallest number of tiles (from the launch's
// average per CU, at least 6) with which all parts are resident at once, and the split must shorten the longest workgroup
// by six tiles or more to pay for the merge launch.  A workgroup costs
// about 6 us beyond its tiles (dispatch, Q and first-tile latency, the output stores): measured at S = 2048 (256 workgroups,
// 57 us unsplit) every part size from 4 to 32 tiles came out between 53 and 61 us before the parts were even merged.
struct KeySplit {
    int nh = 1;            // heads per wavefront: row blocks of 16 nh rows
    int tmax = 0;
    long parts = 0;
    int split_blocks = 0;
    long bytes() const { return parts * AKV * part_bytes(16 * nh); }
};
KeySplit plan_split_nh(int S, int L, int q_pos0, int nh, int min_gain) {
    KeySplit ks;
    ks.nh = nh;
    const int RB = 16 * nh, nb = (S + RB - 1) / RB, cus = cu_count();
    if (S < 1 || nb * AKV >= cus) return ks;
    long total = 0;
    int longest = 0;
    for (int i = 0; i < nb; i++) {
        const int kend = std::min(L, q_pos0 + std::min(RB * i + RB - 1, S - 1) + 1), nt = (kend + KT - 1) / KT;
        total += nt;
        longest = std::max(longest, nt);
    }
    // the smallest part size (from the average per CU, at least 6 tiles) whose parts are all resident at once: a CU that has
    // to run a second part pays the per-workgroup cost twice.  (A floor of 6 against 8, us: 768 rows 18.1 / 20.7, 1536 rows
    // 28.9 / 29.9, one row after 4095 keys 19.6 / 21.1, 64 rows after 8000 keys 29.4 / 27.6; 5 and 7 are worse on more shapes.)
    const long p = (q_pos0 + RB - 1) / RB, cpt = KT / RB;
    int tmax = (int)std::max(6L, (total * AKV + cus - 1) / cus);
    while (tmax < longest && (parts_upto(p + nb, cpt * tmax) - parts_upto(p, cpt * tmax)) * AKV > cus) tmax++;
    if (longest - tmax < min_gain) return ks;                    // the merge launch has to be earned
    const long c = cpt * tmax;
    ks.tmax = tmax;
    ks.parts = parts_upto(p + nb, c) - parts_upto(p, c);
    ks.split_blocks = nb - (int)std::max(0L, c - p);
    return ks;
}
// The form of a launch, by measurement (us at q_pos0 = 0, 16-row blocks (NH = 1) in their best form / 32-row blocks (NH = 2) with
// the split: S = 1280 25.3 / 27.3, 1408 27.7 / 27.7, 1536 32.3 / 30.0, 2048 47.0 / 37.2, 2560 59.9 / 51.4, 2944 68.5 / 63.3,
// 3072 71.0 / 69.8, 3200 76.3 / 75.5, 3328 79.3 / 82.5; unsplit 4096 108 / 114, 4608 138 / 131, 5120 167 / 149):
//   from about 4600 rows on     NH = 2, unsplit (enough 32-row blocks to balance themselves);
//   from about 1500 rows on     NH = 2 with the key split, where the launch leaves room for it and, for a whole prompt, up to
//                               3200 rows (a tile of a 32-row block costs less than two tiles of 16-row blocks, but its parts
//                               are twice the size); after a prefix NH = 2 wins by more;
//   everything else             NH = 1, split if CUs would idle.
KeySplit plan_split(int S, int L, int q_pos0) {
    if (two_heads_per_wave(S)) {                                 // (two heads: S >= 1472 in every case, so L >= one tile)
        KeySplit ks;
        ks.nh = 2;
        return ks;
    }
    if (S >= 1472 && (q_pos0 > 0 || S <= 3200)) {
        const KeySplit ks = plan_split_nh(S, L, q_pos0, 2, 4);
        if (ks.tmax) return ks;
    }
    return plan_split_nh(S, L, q_pos0, 1, 6);
}

}  // namespace

extern "C" {

// Bytes of workspace the key split of this launch uses (0: the launch is not split).  Without that much workspace
// qt_gqa_prefill_causal runs the same launch unsplit, with the same results up to rounding.
long qt_gqa_prefill_workspace_bytes_for(int S, int L, int q_pos0) {
    if (S < 0 || L < 1 || q_pos0 < 0) return -1;
    const KeySplit ks = plan_split(S, L, q_pos0);
    return ks.tmax ? ks.bytes() : 0;
}
// An upper bound of the above over every launch with at most L keys (S <= L, q_pos0 = L - S or smaller): a part holds at least
// total / CUs tiles, so there are at most CUs / 2 + 2 * blocks parts per KV head, a split launch has fewer than CUs / 2 blocks,
// and a part of a 16-row block is half the size of one of a 32-row block.
long qt_gqa_prefill_workspace_bytes(int L) {
    if (L < 0) return -1;
    const long cus = cu_count(), nb16 = std::min((long)(L + 15) / 16, cus / AKV), nb32 = std::min((long)(L + 31) / 32, cus / AKV);
    const long b16 = (cus + AKV * (2 * nb16 + 2)) * part_bytes(16);
    const long b32 = (cus + AKV * (2 * nb32 + 2)) * part_bytes(32);
    return std::max(b16, b32);
}

// q, out [8][S][256] bf16 (head stride q_head_stride elements), K, V [2][>=L][256] bf16 (head stride kv_head_stride):
// query i sits at absolute position q_pos0 + i and sees keys 0 .. q_pos0 + i (< L).  workspace: see above; may be null.
int qt_gqa_prefill_causal(const void* q, const void* K, const void* V, void* out, void* workspace, long workspace_bytes, int S,
                          int L, int q_pos0, long q_head_stride, long kv_head_stride, hipStream_t stream) {
    if (!q || !K || !V || !out) return QT_ERR_NULL;
    if (S < 0 || L < 1 || q_pos0 < 0 || (long)q_pos0 + S > L || q_head_stride < (long)S * AD || kv_head_stride < (long)L * AD)
        return QT_ERR_DIM;
    if (S == 0) return QT_OK;
    for (const void* p : {q, K, V, (const void*)out, (const void*)workspace})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    if ((q_head_stride | kv_head_stride) & 7) return QT_ERR_ALIGN;
    KeySplit ks = plan_split(S, L, q_pos0);
    if (ks.tmax && (!workspace || workspace_bytes < ks.bytes())) {          // no room for the parts: the unsplit form
        ks = KeySplit();
        ks.nh = two_heads_per_wave(S) ? 2 : 1;
    }
    const int RB = 16 * ks.nh;
    const dim3 grid((ks.tmax ? (unsigned)ks.parts : (unsigned)((S + RB - 1) / RB)) * AKV);
    _Float16* part_o = ks.tmax ? (_Float16*)workspace : nullptr;
    float* part_ml = ks.tmax ? reinterpret_cast<float*>(part_o + (size_t)ks.parts * AKV * part_o_floats(RB)) : nullptr;
    if (ks.nh == 2)
        hipLaunchKernelGGL(attn_prefill_kernel<2>, grid, dim3(512), 0, stream, (const bf16_t*)q, (const bf16_t*)K, (const bf16_t*)V,
                           (bf16_t*)out, S, L, q_pos0, q_head_stride, kv_head_stride, ks.tmax, part_o, part_ml);
    else
        hipLaunchKernelGGL(attn_prefill_kernel<1>, grid, dim3(512), 0, stream, (const bf16_t*)q, (const bf16_t*)K, (const bf16_t*)V,
                           (bf16_t*)out, S, L, q_pos0, q_head_stride, kv_head_stride, ks.tmax, part_o, part_ml);
    if (ks.tmax) {
        const dim3 mgrid((unsigned)ks.split_blocks, AKV, (AH / AKV) * ks.nh);
        if (ks.nh == 2)
            hipLaunchKernelGGL(attn_prefill_merge_kernel<32>, mgrid, dim3(256), 0, stream, part_o, part_ml, (bf16_t*)out, S, q_pos0,
                               ks.tmax, ks.parts, q_head_stride);
        else
            hipLaunchKernelGGL(attn_prefill_merge_kernel<16>, mgrid, dim3(256), 0, stream, part_o, part_ml, (bf16_t*)out, S, q_pos0,
                               ks.tmax, ks.parts, q_head_stride);
    }
    QT_CHECK_LAUNCH();
    return QT_OK;
}

}  // extern "C"
