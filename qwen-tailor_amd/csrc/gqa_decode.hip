// Ragged GQA decode / verify attention, head dim 256, 8 query heads on 2 KV heads, for gfx950.
// Replaces the Metal kernel attn_b_{Lmax}_m{M} (qwen35/batch.py:141-237): row r = b*M + j of the batch sits at position
// pos[b] + j of slot slots[b]; it attends the pool keys below pos[b] and the new keys of rows b*M .. b*M + j, which are
// read from the inputs (never from the pool) and appended to the pool at pos[b] + j.
//
// Split-K over one flat tile space: segment sg = (sequence b, kv head) owns max(1, ceil(pos[b] / 16)) tiles of 16 pool keys,
// the segments are laid end to end, and each of the launch's workgroups takes the same number of consecutive tiles (it may
// cross segment borders: it then emits one partial result per segment it touches).  Every workgroup therefore streams the
// same number of bytes whatever the mix of sequence lengths, K and V are read from HBM exactly once per step for all 4*M
// query rows that share the KV head, and the launch is one round of resident workgroups (one per CU).
//   loads  : a K or V tile (16 keys x 512 bytes) is fetched as whole rows, two rows per wavefront-wide load (nontemporal),
//            and parked row-major in LDS
//   scores : S^T[16 keys x 16 rows] = K_tile[16 x 256] . Q^T[256 x 16] on bf16 MFMA (16x16x32), K fragments from LDS
//   P . V  : O[16 rows x 256] += P[16 x 16 keys] . V[16 keys x 256] on bf16 MFMA (16x16x16): the transposed scores in
//            their accumulator layout ARE the A operand; the V tile is read back through the transposing LDS load
//            (ds_read_b64_tr_b16), which delivers the B operand (4 consecutive keys of one column).
//            P is split into two bf16 terms (p = hi + lo, error 2^-17), so the product keeps fp32-like accuracy.
// Each wavefront walks its tiles with a one-tile-deep register FIFO: a register is refilled with the next tile's row right
// after the LDS store that consumed it, so a tile's loads fly during the previous tile's arithmetic.  The loop issues
// loads only, in the order of their use, which keeps every vmcnt wait partial.
// Each wavefront keeps its own online-softmax state (m, l, O); the 4 wavefronts of a workgroup are merged through LDS and
// the workgroup writes one unnormalised partial (m, l, O) per row and segment; a second kernel merges the partials
// (batch.py:203-221).
// A kernel instance holds at most four query tokens per sequence (16 rows = one MFMA tile).  More tokens per sequence (M up
// to 16) run as passes of up to four: pass j0 = 0, 4, 8, 12 takes rows j0 .. j0+3 of every sequence at position pos[b] + j0 and
// finds the rows that the earlier passes appended among its pool keys (the passes are launches on one stream, in order).
#include "qt_common.h"

using namespace qt;

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr int GQA = AH / AKV;          // 4 query heads per KV head
constexpr float SCALE = 0.0625f;       // 256^-0.5, batch.py:177
constexpr float NEG = -3.0e38f;
constexpr int VL_LD = AD + 16;         // row stride (elements) of the V tile in LDS: 544 bytes spread the 16 rows over the banks
constexpr int KL_LD = AD + 8;          // row stride of the K tile: 528 bytes, the 16 rows of a fragment read start 4 banks apart

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---- the layer form: q / k RMSNorm and rotary embedding inside the attention kernel (qwen35/batch.py:505-512) ----------------
constexpr int QKV_W = AH * 2 * AD + 2 * AKV * AD;      // 5120: [(q_h | gate_h) x 8 | k x 2 | v x 2]
constexpr int ROPE_PAIRS = 32;                         // rotary pairs (i, i + 32), i < 32, of the first 64 features

// Online-softmax update of one tile of 16 keys from its transposed scores: lane (row n, group g) holds keys 4g .. 4g+3.
// Leaves the probabilities of those keys in p (fp32) and writes the row's rescale factor to c_lds[row].
__device__ __forceinline__ void softmax_tile(const f32x4& acc, int nvalid, bool causal, float& m_run, float& l_run, float (&p)[4],
                                             float* c_lds, int lane) {
    const int n = lane & 15, g = lane >> 4;
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
        p[i] = s[i] > 0.5f * NEG ? __expf(s[i] - m_new) : 0.f;
        ps += p[i];
    }
    l_run = l_run * corr + ps;                                   // this lane's share; summed over g at the end
    m_run = m_new;
    if (g == 0) c_lds[n] = corr;
}

// O (16 rows x 256, accumulator layout: block j, lane (column 16 j + n, group g), rows 4g .. 4g+3) = c * O + P . V for the
// V tile in v_lds ([16 keys][VL_LD]).  p: this lane's probabilities (row n, keys 4g .. 4g+3).
__device__ __forceinline__ void pv_tile(f32x4 (&O)[16], const float (&p)[4], const bf16_t* v_lds, const float* c_lds, int lane) {
    const int n = lane & 15, g = lane >> 4;
    s16x4 ph, pl;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const bf16_t h = f2bf(p[i]);
        ph[i] = (short)h;
        pl[i] = (short)f2bf(p[i] - bf2f(h));
    }
    const f32x4 c4 = *reinterpret_cast<const f32x4*>(c_lds + 4 * g);
    // transposing load: within a group of 16 lanes, lane 4q + i receives element i of the 8-byte chunks addressed by lanes
    // q, q+4, q+8, q+12.  Lane j' = n of group g points at key 4g + n/4, columns 4 (n%4) .. + 3 of the block: lane n then
    // receives keys 4g .. 4g+3 of column n, the B operand.
    const bf16_t* vrow = v_lds + (4 * g + (n >> 2)) * VL_LD + 4 * (n & 3);
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const s16x4 B = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4*)(const_cast<bf16_t*>(vrow + 16 * j)));
        O[j] *= c4;
        O[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ph, B, O[j], 0, 0, 0);
        O[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(pl, B, O[j], 0, 0, 0);
    }
}

constexpr int MAX_SEG = 2048;          // segments (2 per sequence) a launch can hold
// A workgroup pays about 3 us for every segment it visits (the query rows, the first tiles' latency, the merge of its four
// wavefronts, the partial result): as much as streaming ~5 tiles.  Every segment therefore starts with that many empty
// positions in the flat tile space, so that a workgroup whose range crosses a segment border gets fewer tiles to stream.
constexpr int VISIT_TILES = 5;


// Exclusive prefix of the segments' tile counts -> seg_start[0 .. nseg] (LDS); returns the total.  Rows whose slot or position
// is out of range own no tiles (they are skipped by both kernels).  Every thread of the workgroup must call it.
template <int M, int VISIT>
__device__ __forceinline__ int build_segments(int* seg_start, const int* __restrict__ slots, const int* __restrict__ pos, int nseg,
                                              int Lmax, int n_slots, int Mtot, int j0) {
    const int tid = threadIdx.x, lane = tid & 63;
    for (int sg = tid; sg < nseg; sg += 256) {
        const int b = sg / AKV, slot = slots[b], p0 = pos[b];
        const bool ok = (unsigned)slot < (unsigned)n_slots && p0 >= 0 && p0 + Mtot <= Lmax;    // all of the sequence's rows fit, or none is taken
        seg_start[sg + 1] = ok ? max(1, (p0 + j0 + 15) >> 4) + VISIT : 0;
    }
    if (tid == 0) seg_start[0] = 0;
    __syncthreads();
    if (tid < 64) {
        int carry = 0;
        for (int base = 1; base <= nseg; base += 64) {
            const int i = base + lane;
            int v = i <= nseg ? seg_start[i] : 0;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int o = __shfl_up(v, d, 64);
                if (lane >= d) v += o;
            }
            if (i <= nseg) seg_start[i] = v + carry;
            carry += __shfl(v, 63, 64);
        }
    }
    __syncthreads();
    return seg_start[nseg];
}
// tiles per workgroup for `total` tiles spread over nwg workgroups, at least min_tiles
__device__ __forceinline__ int tiles_per_wg(int total, int nwg, int min_tiles) { return max(min_tiles, (total + nwg - 1) / nwg); }

// partial results: slot id = workgroup + segment (unique, and consecutive for the workgroups that share a segment);
// part_o [slot][4*M rows][256] f32 (unnormalised), part_ml [slot][4*M][2] = (running max, running sum)
// LAYER: q is the layer's qkv rows [B*Mtot, 5120]; the query rows and the new keys are normed and roped here, the
// new values are read from the rows' v part, and k_new / v_new are not used.
template <int M, bool LAYER>
__global__ __launch_bounds__(256, 2) void attn_partial_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_new,
                                                           const bf16_t* __restrict__ v_new, bf16_t* Kp, bf16_t* Vp,
                                                           const int* __restrict__ slots, const int* __restrict__ pos,
                                                           float* __restrict__ part_o, float* __restrict__ part_ml,
                                                           int* __restrict__ seg_tab, int B, int Lmax, int min_tiles, int n_slots,
                                                           int Mtot, int j0, const bf16_t* __restrict__ q_norm,
                                                           const bf16_t* __restrict__ k_norm, const float2* __restrict__ rope_tab,
                                                           float eps) {
    // M = tokens of this pass (rows j0 .. j0 + M - 1 of each sequence's Mtot rows)
    constexpr int R = 4 * M;
    __shared__ int seg_start[MAX_SEG + 1];
    // one V tile and one K tile per wavefront, in one array: at the end the same memory holds the four wavefronts' scaled O
    // ([4][R rows][256] f32) for the merge
    __shared__ __align__(16) bf16_t tile_s[4 * 16 * (VL_LD + KL_LD)];
    __shared__ __align__(16) float c_s[4][16];
    __shared__ float m_s[4][16], l_s[4][16];
    static_assert(sizeof(bf16_t) * 4 * 16 * (VL_LD + KL_LD) >= sizeof(float) * 4 * 16 * AD, "the four O tiles must fit into the K / V tiles");
    float* const mo = reinterpret_cast<float*>(tile_s);

    const int nseg = B * AKV;
    // (both forms cut the tile space alike, so that the layer form sums its partial results in the order of the plain one: same bits)
    constexpr int VISIT = VISIT_TILES;
    const int total = build_segments<M, VISIT>(seg_start, slots, pos, nseg, Lmax, n_slots, Mtot, j0);
    if (blockIdx.x == 0)                                         // the merge kernel reads the table instead of building it again
        for (int i = threadIdx.x; i <= nseg; i += 256) seg_tab[i] = seg_start[i];
    const int per = tiles_per_wg(total, gridDim.x, min_tiles);
    const int wt0 = blockIdx.x * per, wt1 = min(wt0 + per, total);
    if (wt0 >= wt1) return;
    int sg0 = 0;                                                 // the segment that holds tile wt0 (uniform binary search)
    for (int lo_ = 0, hi_ = nseg; lo_ < hi_;) {
        const int mid = (lo_ + hi_) >> 1;
        if (seg_start[mid + 1] <= wt0) lo_ = mid + 1; else hi_ = mid;
        sg0 = lo_;
    }
    const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int hw = lane >> 5, cl = lane & 31;

  for (int sg = sg0; sg < nseg && seg_start[sg] < wt1; sg++) {
    const int ss = seg_start[sg], se = seg_start[sg + 1];
    if (se == ss) continue;                                      // a skipped row
    const int kvh = sg % AKV, b = sg / AKV;
    const int slot = slots[b], p0 = pos[b] + j0;                 // the pass's rows start at p0; the keys below it are in the pool
    const bool first = wt0 <= ss;                                // this workgroup holds the segment's first tile
    const int lo = max(0, max(wt0, ss) - ss - VISIT) * 16, hi = min(max(0, min(wt1, se) - ss - VISIT) * 16, p0);
    const size_t pslot = (size_t)blockIdx.x + sg;

    const size_t pbase = ((size_t)slot * AKV + kvh) * Lmax * AD;
    const bf16_t* kbase = Kp + pbase;
    const bf16_t* vbase = Vp + pbase;
    bf16_t* vl = tile_s + w * (16 * VL_LD);
    bf16_t* kl = tile_s + 4 * (16 * VL_LD) + w * (16 * KL_LD);
    const int ntiles = hi > lo ? (hi - lo + 15) / 16 : 0;
    // Row addresses of a tile: key 2i (lower half wavefront) / 2i + 1 (upper half), 8 columns per lane, so one load covers
    // two whole 512-byte rows (a wavefront-wide load of 16 rows x 64 bytes streams about 15 % slower from HBM).  Keys past
    // `hi` re-read the tile's first key (they are masked / weighted by 0).
    auto row_ptr = [&](const bf16_t* base, int t, int i) {
        const int key0 = lo + t * 16, key = key0 + 2 * i + hw;
        return reinterpret_cast<const u32x4*>(base + (size_t)(key < hi ? key : key0) * AD) + cl;
    };
    u32x4 a[8], vv[8];

    // Q^T as the MFMA B operand: lane (row n, group g) holds q[row n][32 kb + 8 g .. + 8]; row n = token (n / 4), head n % 4
    bf16x8 bq[8];
    // layer form: the staged query rows lie in wavefront 0's V tile (the tiles are not in use yet), the staged new keys in an
    // array of their own (they are read after the tile loop).  With the query rows in an array of their own the workgroup's LDS
    // would pass half of a CU's: the compiler then plans for one workgroup per CU and all 512 registers, puts O into the
    // accumulation registers, and the rescale of O in the tile loop costs a register copy each way (+4 us per launch).
    __shared__ __align__(16) bf16_t k_s[LAYER ? 4 * KL_LD : 8];
    bf16_t* const q_s = tile_s;
    static_assert(16 * KL_LD <= 16 * VL_LD, "the staged query rows must fit into one V tile");
    if constexpr (LAYER) {
        // The wavefront's first tile is requested before anything else: the norm and the rotary embedding below run while it
        // is on its way from HBM.
        if (w < ntiles) {
#pragma unroll
            for (int i = 0; i < 8; i++) a[i] = __builtin_nontemporal_load(row_ptr(kbase, w, i));
#pragma unroll
            for (int i = 0; i < 8; i++) vv[i] = __builtin_nontemporal_load(row_ptr(vbase, w, i));
        }
        __builtin_amdgcn_sched_barrier(0);
        // The 4 M query rows are normed and roped once per workgroup: wavefront w takes token w (its four heads, a row per
        // 16-lane group, 16 consecutive elements per lane) and leaves the rows in LDS, where every wavefront picks up its
        // B operand.  The workgroup that holds the segment's first tile does the same for the M new keys (wavefront 0, a key
        // per 16-lane group), which it also appends to the pool (batch.py:196-201).  Same arithmetic, value for value, as
        // attn_qkv_prep_kernel: sum of squares exact in double and rounded once, correctly rounded 1 / sqrt,
        // BF(w * BF(x * inv)), rotary products and sums rounded one by one; (cos, sin) from the table qt_rope_table_build wrote.
        const int rr = lane >> 4, c = lane & 15;
        auto glue16 = [&](const bf16_t* x, const bf16_t* wgt, const float2* cs, u32x4& o0, u32x4& o1) {
            const u32x4 x0 = reinterpret_cast<const u32x4*>(x)[0], x1 = reinterpret_cast<const u32x4*>(x)[1];
            const u32x4 w0 = reinterpret_cast<const u32x4*>(wgt)[0], w1 = reinterpret_cast<const u32x4*>(wgt)[1];
            f32x4 cv[8];                                          // rotary pairs 16 (c & 1) .. + 15 (used by lanes c < 4 only)
#pragma unroll
            for (int e = 0; e < 8; e++) cv[e] = reinterpret_cast<const f32x4*>(cs)[e];
            float y[16], wt[16];
            unpack8(make_uint4(x0[0], x0[1], x0[2], x0[3]), reinterpret_cast<float(&)[8]>(y[0]));
            unpack8(make_uint4(x1[0], x1[1], x1[2], x1[3]), reinterpret_cast<float(&)[8]>(y[8]));
            unpack8(make_uint4(w0[0], w0[1], w0[2], w0[3]), reinterpret_cast<float(&)[8]>(wt[0]));
            unpack8(make_uint4(w1[0], w1[1], w1[2], w1[3]), reinterpret_cast<float(&)[8]>(wt[8]));
            double ss = 0.0;
#pragma unroll
            for (int e = 0; e < 16; e++) ss += (double)y[e] * y[e];
            const float inv = rsqrt_rn((float)row16_sum_d(ss) / (float)AD + eps);
#pragma unroll
            for (int e = 0; e < 16; e++) y[e] = BF(wt[e] * BF(y[e] * inv));
            // rotary pairs (i, i + 32), i < 32: lanes 0, 1 of a row hold the first halves, lanes 2, 3 their partners
            float other[16];
#pragma unroll
            for (int e = 0; e < 16; e++) other[e] = __shfl_xor(y[e], 2, 64);
            if (c < 4) {
#pragma clang fp contract(off)
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const float cs_c = cv[e >> 1][2 * (e & 1)], cs_s = cv[e >> 1][2 * (e & 1) + 1];
                    const float own = y[e] * cs_c, oth = other[e] * cs_s;
                    y[e] = BF(c < 2 ? own - oth                   // y1 c - y2 s
                                    : oth + own);                 // y1 s + y2 c
                }
            }
            o0 = u32x4{pack2_bf(y[0], y[1]), pack2_bf(y[2], y[3]), pack2_bf(y[4], y[5]), pack2_bf(y[6], y[7])};
            o1 = u32x4{pack2_bf(y[8], y[9]), pack2_bf(y[10], y[11]), pack2_bf(y[12], y[13]), pack2_bf(y[14], y[15])};
        };
        {
            u32x4 o0 = {0, 0, 0, 0}, o1 = {0, 0, 0, 0};           // (rows past 4 M: zeros)
            if (w < M)
                glue16(q + (size_t)(b * Mtot + j0 + w) * QKV_W + (kvh * GQA + rr) * 2 * AD + 16 * c, q_norm + 16 * c,
                       rope_tab + (size_t)(p0 + w) * ROPE_PAIRS + 16 * (c & 1), o0, o1);
            *reinterpret_cast<u32x4*>(q_s + (4 * w + rr) * KL_LD + 16 * c) = o0;
            *reinterpret_cast<u32x4*>(q_s + (4 * w + rr) * KL_LD + 16 * c + 8) = o1;
        }
        if (first && w == 0) {
            const int key = rr < M ? rr : 0;                      // (idle groups work on a copy of key 0 and store nothing)
            u32x4 o0, o1;
            glue16(q + (size_t)(b * Mtot + j0 + key) * QKV_W + AH * 2 * AD + kvh * AD + 16 * c, k_norm + 16 * c,
                   rope_tab + (size_t)(p0 + key) * ROPE_PAIRS + 16 * (c & 1), o0, o1);
            if (rr < M) {
                *reinterpret_cast<u32x4*>(k_s + rr * KL_LD + 16 * c) = o0;
                *reinterpret_cast<u32x4*>(k_s + rr * KL_LD + 16 * c + 8) = o1;
                *reinterpret_cast<u32x4*>(Kp + pbase + (size_t)(p0 + rr) * AD + 16 * c) = o0;
                *reinterpret_cast<u32x4*>(Kp + pbase + (size_t)(p0 + rr) * AD + 16 * c + 8) = o1;
            }
        }
        __syncthreads();
#pragma unroll
        for (int kb = 0; kb < 8; kb++) bq[kb] = as_bf16x8(*reinterpret_cast<const u32x4*>(q_s + n * KL_LD + 32 * kb + 8 * g));
        __syncthreads();                                          // every wavefront has its rows: wavefront 0 may park its first tile there
    } else {
        const bool real = n < R;
        const bf16_t* qr = q + ((size_t)(b * Mtot + j0 + (real ? n / GQA : 0)) * AH + kvh * GQA + (n % GQA)) * AD;
#pragma unroll
        for (int kb = 0; kb < 8; kb++) {
            u32x4 v = reinterpret_cast<const u32x4*>(qr)[kb * 4 + g];
            if (!real) v = u32x4{0, 0, 0, 0};
            bq[kb] = as_bf16x8(v);
        }
    }
    float m_run = NEG, l_run = 0.f;
    f32x4 O[16];
#pragma unroll
    for (int j = 0; j < 16; j++) O[j] = f32x4{0.f, 0.f, 0.f, 0.f};

    if (w < ntiles) {
        if constexpr (!LAYER) {
#pragma unroll
            for (int i = 0; i < 8; i++) a[i] = __builtin_nontemporal_load(row_ptr(kbase, w, i));
#pragma unroll
            for (int i = 0; i < 8; i++) vv[i] = __builtin_nontemporal_load(row_ptr(vbase, w, i));
        }
        __builtin_amdgcn_sched_barrier(0);
        for (int t = w; t < ntiles; t += 4) {
            const int tn = t + 4 < ntiles ? t + 4 : t;           // the last step re-reads its own tile
            const int nvalid = min(16, hi - (lo + t * 16));
            // park both tiles row-major in LDS; every register is refilled with the next tile's row right after its store
#pragma unroll
            for (int i = 0; i < 8; i++) {
                *reinterpret_cast<u32x4*>(kl + (2 * i + hw) * KL_LD + 8 * cl) = a[i];
                a[i] = __builtin_nontemporal_load(row_ptr(kbase, tn, i));
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                *reinterpret_cast<u32x4*>(vl + (2 * i + hw) * VL_LD + 8 * cl) = vv[i];
                vv[i] = __builtin_nontemporal_load(row_ptr(vbase, tn, i));
                __builtin_amdgcn_sched_barrier(0);
            }
            wave_lds_sync();
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kb = 0; kb < 8; kb++) {                     // A operand: lane (key n, group g) holds k[key n][32 kb + 8 g .. + 8]
                const u32x4 ka = *reinterpret_cast<const u32x4*>(kl + n * KL_LD + 32 * kb + 8 * g);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(ka), bq[kb], acc, 0, 0, 0);
            }
            float p[4];
            softmax_tile(acc, nvalid, false, m_run, l_run, p, c_s[w], lane);
            wave_lds_sync();
            pv_tile(O, p, vl, c_s[w], lane);
            wave_lds_sync();
        }
    }
    if (first && w == 3) {
        // The M new keys of this sequence, straight from the inputs (batch.py:143-145), with the causal rule among them:
        // key i is visible to query token j only if i <= j.  Not pipelined: it runs once per sequence.
        const bf16_t* kn = LAYER ? q + (size_t)(b * Mtot + j0) * QKV_W + AH * 2 * AD + kvh * AD
                                 : k_new + ((size_t)(b * Mtot + j0) * AKV + kvh) * AD;
        const bf16_t* vn = LAYER ? q + (size_t)(b * Mtot + j0) * QKV_W + AH * 2 * AD + AKV * AD + kvh * AD
                                 : v_new + ((size_t)(b * Mtot + j0) * AKV + kvh) * AD;
        const size_t stride = LAYER ? (size_t)QKV_W : (size_t)AKV * AD;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        if constexpr (LAYER) {                                    // the new keys as wavefront 0 left them in LDS
#pragma unroll
            for (int kb = 0; kb < 8; kb++) {
                u32x4 v = *reinterpret_cast<const u32x4*>(k_s + (n & 3) * KL_LD + 32 * kb + 8 * g);
                if (n >= M) v = u32x4{0, 0, 0, 0};
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(v), bq[kb], acc, 0, 0, 0);
            }
        } else {
            const u32x4* kr = reinterpret_cast<const u32x4*>(kn + (size_t)(n < M ? n : 0) * stride);
            u32x4 a[8];
#pragma unroll
            for (int kb = 0; kb < 8; kb++) a[kb] = kr[kb * 4 + g];
#pragma unroll
            for (int kb = 0; kb < 8; kb++) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[kb]), bq[kb], acc, 0, 0, 0);
        }
        float p[4];
        softmax_tile(acc, M, true, m_run, l_run, p, c_s[w], lane);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int key = 2 * i + hw;                          // rows past the M new keys are zero: their weight is 0
            u32x4 v = u32x4{0, 0, 0, 0};
            if (key < M) v = reinterpret_cast<const u32x4*>(vn + (size_t)key * stride)[cl];
            *reinterpret_cast<u32x4*>(vl + key * VL_LD + 8 * cl) = v;
        }
        wave_lds_sync();
        pv_tile(O, p, vl, c_s[w], lane);
        wave_lds_sync();
    }
    if (first && w == 0) {
        // append (batch.py:196-201): row j of this sequence goes to pool position p0 + j
        for (int j = 0; j < M; j++) {
            if constexpr (LAYER) {                               // (the keys are appended by the wavefront that norms them)
                const uint2 vv2 = reinterpret_cast<const uint2*>(q + (size_t)(b * Mtot + j0 + j) * QKV_W + AH * 2 * AD + AKV * AD + kvh * AD)[lane];
                reinterpret_cast<uint2*>(Vp + pbase + (size_t)(p0 + j) * AD)[lane] = vv2;
            } else {
                const uint2 kk = reinterpret_cast<const uint2*>(k_new + ((size_t)(b * Mtot + j0 + j) * AKV + kvh) * AD)[lane];
                const uint2 vv2 = reinterpret_cast<const uint2*>(v_new + ((size_t)(b * Mtot + j0 + j) * AKV + kvh) * AD)[lane];
                reinterpret_cast<uint2*>(Kp + pbase + (size_t)(p0 + j) * AD)[lane] = kk;
                reinterpret_cast<uint2*>(Vp + pbase + (size_t)(p0 + j) * AD)[lane] = vv2;
            }
        }
    }

    // ---- merge the 4 wavefronts (deterministic order); lane (n, g) holds rows 4g .. 4g+3 of column 16 j + n
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (g == 0) {
        m_s[w][n] = m_run;
        l_s[w][n] = l_run;
    }
    __syncthreads();                                             // also: every wavefront is done with its V tile
    float f[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int row = 4 * g + r;
        const float mm = fmaxf(fmaxf(m_s[0][row], m_s[1][row]), fmaxf(m_s[2][row], m_s[3][row]));
        f[r] = __expf(m_s[w][row] - mm);
    }
    // every wavefront leaves its scaled O in its own part of LDS; then each thread adds the four for R / 4 groups of four
    // columns, in a fixed order, and writes the partial result
    if (4 * g < R) {
#pragma unroll
        for (int j = 0; j < 16; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) mo[(w * R + 4 * g + r) * AD + 16 * j + n] = O[j][r] * f[r];
    }
    __syncthreads();
    float* po = part_o + pslot * R * AD;
#pragma unroll
    for (int i = tid; i < R * AD / 4; i += 256) {
        const f32x4* src = reinterpret_cast<const f32x4*>(mo) + i;
        reinterpret_cast<f32x4*>(po)[i] = (src[0] + src[R * AD / 4]) + (src[2 * (R * AD / 4)] + src[3 * (R * AD / 4)]);
    }
    if (tid < R) {
        const float mm = fmaxf(fmaxf(m_s[0][tid], m_s[1][tid]), fmaxf(m_s[2][tid], m_s[3][tid]));
        float ll = 0.f;
        for (int ww = 0; ww < 4; ww++) ll += l_s[ww][tid] * __expf(m_s[ww][tid] - mm);
        part_ml[(pslot * R + tid) * 2] = mm;
        part_ml[(pslot * R + tid) * 2 + 1] = ll;
    }
    __syncthreads();                                             // the LDS tiles are reused by the next segment
  }
}

// merge of the partial results: one workgroup of 256 threads per (segment, row).  The per-partial factors exp(m_s - m) are
// computed by one thread each; then wavefront w sums the partials s = w, w+4, ... (a lane owns 4 output columns, four
// partials' loads in flight) and the four wavefronts are added in order.
constexpr int MAX_SPLITS = 4096;
// GATE: out [R,2048] = BF(o * sigmoid_bf16(gate)) with the row's gate from its qkv row (qwen35/batch.py:513), value for value what
// attn_out_gate_kernel makes of the bf16 o that this kernel would store otherwise.
template <int M, bool GATE>
__global__ __launch_bounds__(256) void attn_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                         const int* __restrict__ seg_tab, bf16_t* __restrict__ out, int B, int nwg,
                                                         int min_tiles, int Mtot, int j0, const bf16_t* __restrict__ qkv) {
    constexpr int R = 4 * M;
    __shared__ float fs_s[MAX_SPLITS];
    __shared__ float red_m[4], red_l[4];
    __shared__ __align__(16) float acc_s[4][AD];
    const int r = blockIdx.x % R, sg = blockIdx.x / R, kvh = sg % AKV, b = sg / AKV;
    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63;
    const size_t row = (size_t)(b * Mtot + j0 + r / GQA);
    const int head = kvh * GQA + (r % GQA);
    bf16_t gate_raw = 0;
    if constexpr (GATE) gate_raw = qkv[row * QKV_W + head * 2 * AD + AD + tid];   // requested first, needed last
    const int total = seg_tab[B * AKV], ss = seg_tab[sg], se = seg_tab[sg + 1];   // written by the partial kernel
    if (se == ss) return;                                        // a skipped row
    const int per = tiles_per_wg(total, nwg, min_tiles);
    const int wg0 = ss / per, ns = (se - 1) / per - wg0 + 1;     // the workgroups that hold tiles of this segment
    const size_t base = (size_t)wg0 + sg;                        // their partials sit in consecutive slots
    const float* ml = part_ml + (base * R + r) * 2;              // slot stride 2 R floats
    const float* po = part_o + (base * R + r) * AD + lane * 4;   // slot stride R * AD floats
    float mx = NEG;
    for (int s = tid; s < ns; s += 256) mx = fmaxf(mx, ml[(size_t)s * 2 * R]);
    mx = wave_max(mx);
    if (lane == 0) red_m[w] = mx;
    __syncthreads();
    const float mm = fmaxf(fmaxf(red_m[0], red_m[1]), fmaxf(red_m[2], red_m[3]));
    float lp = 0.f;
    for (int s = tid; s < ns; s += 256) {
        const float f = __expf(ml[(size_t)s * 2 * R] - mm);
        fs_s[s] = f;
        lp += ml[(size_t)s * 2 * R + 1] * f;
    }
    lp = wave_sum(lp);
    if (lane == 0) red_l[w] = lp;
    __syncthreads();
    const float l = (red_l[0] + red_l[1]) + (red_l[2] + red_l[3]);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    int s = w;
    for (; s + 12 < ns; s += 16) {
        f32x4 ov[4];
#pragma unroll
        for (int i = 0; i < 4; i++) ov[i] = *reinterpret_cast<const f32x4*>(po + (size_t)(s + 4 * i) * R * AD);
#pragma unroll
        for (int i = 0; i < 4; i++) acc += ov[i] * fs_s[s + 4 * i];
    }
    for (; s < ns; s += 4) acc += *reinterpret_cast<const f32x4*>(po + (size_t)s * R * AD) * fs_s[s];
    *reinterpret_cast<f32x4*>(&acc_s[w][lane * 4]) = acc;
    __syncthreads();
    const int d = tid;
    const float a = (acc_s[0][d] + acc_s[1][d]) + (acc_s[2][d] + acc_s[3][d]);
    const float ov = l == 0.f ? a : a / l;                                           // batch.py:216
    if constexpr (GATE) {
        out[(row * AH + head) * AD + d] = f2bf(BF(ov) * sigmoid_bf16(bf2f(gate_raw)));
    } else {
        out[(row * AH + head) * AD + d] = f2bf(ov);
    }
}

}  // namespace

extern "C" {

constexpr int MAX_WG = 1024;           // upper bound of the partial kernel's grid (one workgroup per CU)
constexpr int MAX_PASS_M = 4;          // query tokens per sequence in one pass (16 rows: one MFMA tile)
constexpr int MAX_M = 16;              // query tokens per sequence in one call (as many as the verify step of the recurrent layers takes)

static int partial_grid() {            // one workgroup per CU of the current device: measured faster than two (the stream is
                                       // bandwidth-bound with 64 KiB in flight per CU; a second workgroup only adds queueing)
    const int cus = qt::cu_count();
    return cus < MAX_WG ? cus : MAX_WG;
}

constexpr long SEG_TAB_BYTES = ((MAX_SEG + 1) * 4 + 15) / 16 * 16;   // the segment table, after the partial results

// bytes of workspace qt_gqa_attn_decode needs for (B sequences, M rows each, pool length Lmax); CH is accepted for callers
// written against the fixed-split form and does not change the size
long qt_gqa_attn_workspace_bytes(int B, int M, int Lmax, int CH) {
    if (B < 0 || M < 1 || Lmax < 1 || CH < 16) return -1;
    const int mp = M < MAX_PASS_M ? M : MAX_PASS_M;                // the passes of a call with more tokens reuse one pass's space
    return ((long)MAX_WG + (long)B * AKV) * (4 * mp) * (AD + 2) * 4 + SEG_TAB_BYTES;
}

// Both entry points: checks, grid size and the two launches.  The partial results of at most `slot_cap` slots
// (slot = workgroup + segment < grid + 2 B) start at part_o / part_ml; seg_tab holds 2 B + 1 ints.
struct LayerArgs {                      // the layer form's extra operands (null q_norm: the plain form)
    const bf16_t* q_norm;
    const bf16_t* k_norm;
    const float2* rope_tab;
    float eps;
};

static int attn_launch(const void* q, const void* k_new, const void* v_new, void* Kp, void* Vp, const int32_t* slots,
                       const int32_t* pos, void* out, float* part_o, float* part_ml, int* seg_tab, int max_grid, int B, int M,
                       int Lmax, int n_slots, int CH, hipStream_t stream, LayerArgs la = LayerArgs{nullptr, nullptr, nullptr, 0.f}) {
    const int min_tiles = CH / 16;                               // a workgroup takes at least CH keys
    const long max_tiles = (long)B * AKV * ((Lmax + 15) / 16);
    const long want = (max_tiles + min_tiles - 1) / min_tiles;
    const int nwg = (int)(want < max_grid ? want : max_grid);
    const dim3 g1((unsigned)nwg);
    const bool layer = la.q_norm != nullptr;
#define QT_ATTN_LAUNCH2(MM, LY)                                                                                           \
    hipLaunchKernelGGL((attn_partial_kernel<MM, LY>), g1, dim3(256), 0, stream, (const bf16_t*)q, (const bf16_t*)k_new,   \
                       (const bf16_t*)v_new, (bf16_t*)Kp, (bf16_t*)Vp, slots, pos, part_o, part_ml, seg_tab, B, Lmax, min_tiles,    \
                       n_slots, M, j0, la.q_norm, la.k_norm, la.rope_tab, la.eps);                                        \
    hipLaunchKernelGGL((attn_merge_kernel<MM, LY>), dim3((unsigned)(B * AKV * 4 * MM)), dim3(256), 0, stream, part_o, part_ml,      \
                       seg_tab, (bf16_t*)out, B, nwg, min_tiles, M, j0, (const bf16_t*)q);
#define QT_ATTN_LAUNCH(MM)                                                                                                \
    if (layer) { QT_ATTN_LAUNCH2(MM, true) } else { QT_ATTN_LAUNCH2(MM, false) }
    for (int j0 = 0; j0 < M; j0 += MAX_PASS_M) {                 // passes of up to four tokens per sequence
        switch (M - j0 < MAX_PASS_M ? M - j0 : MAX_PASS_M) {
            case 1: QT_ATTN_LAUNCH(1) break;
            case 2: QT_ATTN_LAUNCH(2) break;
            case 3: QT_ATTN_LAUNCH(3) break;
            default: QT_ATTN_LAUNCH(4) break;
        }
        QT_CHECK_LAUNCH();
    }
#undef QT_ATTN_LAUNCH
#undef QT_ATTN_LAUNCH2
    return QT_OK;
}

static int attn_check(const void* q, const void* k_new, const void* v_new, const void* Kp, const void* Vp, const int32_t* slots,
                      const int32_t* pos, const void* out, int B, int M, int Lmax, int n_slots, int CH) {
    if (!q || !k_new || !v_new || !Kp || !Vp || !slots || !pos || !out) return QT_ERR_NULL;
    if (B < 0 || Lmax < 1 || n_slots < 1 || CH < 16 || CH % 16) return QT_ERR_DIM;
    if (M < 1 || M > MAX_M || B * AKV > MAX_SEG) return QT_ERR_UNSUPPORTED;
    for (const void* p : {q, k_new, v_new, Kp, Vp})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    return QT_OK;
}

int qt_gqa_attn_decode(const void* q, const void* k_new, const void* v_new, void* Kp, void* Vp, const int32_t* slots,
                       const int32_t* pos, void* out, void* workspace, long workspace_bytes, int B, int M, int Lmax,
                       int n_slots, int CH, hipStream_t stream) {
    if (!workspace) return QT_ERR_NULL;
    if (const int rc = attn_check(q, k_new, v_new, Kp, Vp, slots, pos, out, B, M, Lmax, n_slots, CH)) return rc;
    if (B == 0) return QT_OK;
    if (reinterpret_cast<uintptr_t>(workspace) & 15u) return QT_ERR_ALIGN;
    if (workspace_bytes < qt_gqa_attn_workspace_bytes(B, M, Lmax, CH)) return -6;
    const size_t cap = (size_t)MAX_WG + (size_t)B * AKV;
    const int mp = M < MAX_PASS_M ? M : MAX_PASS_M;
    float* part_o = (float*)workspace;
    float* part_ml = part_o + cap * (4 * mp) * AD;
    int* seg_tab = reinterpret_cast<int*>(part_ml + cap * (4 * mp) * 2);
    return attn_launch(q, k_new, v_new, Kp, Vp, slots, pos, out, part_o, part_ml, seg_tab, partial_grid(), B, M, Lmax, n_slots, CH,
                       stream);
}

// The attention half of a full-attention layer at a decode / verify step in two launches per pass: q / k RMSNorm, rotary
// embedding, the split of the qkv rows, attn_b and the output gate (qwen35/batch.py:505-513).
long qt_rope_table_bytes(int n_pos) { return n_pos < 0 ? -1 : (long)n_pos * ROPE_PAIRS * (long)sizeof(float2); }

int qt_gqa_attn_layer_decode(const void* qkv, const void* q_norm, const void* k_norm, const void* rope_table, int table_positions,
                             void* Kp, void* Vp, const int32_t* slots, const int32_t* pos, void* out, void* workspace,
                             long workspace_bytes, int B, int M, int Lmax, int n_slots, int CH, float eps, hipStream_t stream) {
    if (!workspace || !q_norm || !k_norm || !rope_table) return QT_ERR_NULL;
    if (const int rc = attn_check(qkv, qkv, qkv, Kp, Vp, slots, pos, out, B, M, Lmax, n_slots, CH)) return rc;
    if (table_positions < Lmax) return QT_ERR_DIM;               // every position a row can sit at has its (cos, sin) pairs
    if (B == 0) return QT_OK;
    for (const void* p : {(const void*)workspace, q_norm, k_norm, rope_table, (const void*)out})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    if (workspace_bytes < qt_gqa_attn_workspace_bytes(B, M, Lmax, CH)) return -6;
    const size_t cap = (size_t)MAX_WG + (size_t)B * AKV;
    const int mp = M < MAX_PASS_M ? M : MAX_PASS_M;
    float* part_o = (float*)workspace;
    float* part_ml = part_o + cap * (4 * mp) * AD;
    int* seg_tab = reinterpret_cast<int*>(part_ml + cap * (4 * mp) * 2);
    return attn_launch(qkv, nullptr, nullptr, Kp, Vp, slots, pos, out, part_o, part_ml, seg_tab, partial_grid(), B, M, Lmax, n_slots,
                       CH, stream, LayerArgs{(const bf16_t*)q_norm, (const bf16_t*)k_norm, (const float2*)rope_table, eps});
}

// ---- the same operator for callers that cannot allocate: the partial results live in a static device array -------------------
constexpr int ST_MAX_B = 128;          // sequences per call of the allocation-free entry point
constexpr int ST_MAX_WG = 256;         // its partial kernel's grid is capped here (one workgroup per CU on MI355X)
constexpr size_t ST_CAP = (size_t)ST_MAX_WG + (size_t)ST_MAX_B * AKV;
constexpr size_t ST_BYTES = ST_CAP * 16 * (AD + 2) * 4 + SEG_TAB_BYTES;        // 8.1 MiB
static __device__ __align__(256) unsigned char scratch[ST_BYTES];

// Device address of `scratch` on the current device, looked up once per device (every GPU holds its own copy of the array
// at its own address).  In host code the array's name is only a handle for this lookup, never a pointer to pass on.
static int scratch_address(unsigned char** out) {
    constexpr int MAX_DEV = 64;
    static std::atomic<unsigned char*> cache[MAX_DEV];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV) return QT_ERR_LAUNCH;
    unsigned char* p = cache[dev].load(std::memory_order_acquire);
    if (!p) {
        if (hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return QT_ERR_LAUNCH;
        cache[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return QT_OK;
}

int qt_gqa_attn_decode_static(const void* q, const void* k_new, const void* v_new, void* Kp, void* Vp, const int32_t* slots,
                              const int32_t* pos, void* out, int B, int M, int Lmax, int n_slots, int CH, hipStream_t stream) {
    if (const int rc = attn_check(q, k_new, v_new, Kp, Vp, slots, pos, out, B, M, Lmax, n_slots, CH)) return rc;
    if (B > ST_MAX_B) return QT_ERR_STATIC_MAX;
    if (B == 0) return QT_OK;
    unsigned char* base = nullptr;
    if (const int rc = scratch_address(&base)) return rc;
    // Nothing in the array has to start at zero: every partial slot and table entry a launch reads was written by that launch.
    const int mp = M < MAX_PASS_M ? M : MAX_PASS_M;
    float* part_o = reinterpret_cast<float*>(base);
    float* part_ml = part_o + ST_CAP * (4 * mp) * AD;
    int* seg_tab = reinterpret_cast<int*>(part_ml + ST_CAP * (4 * mp) * 2);
    const int grid = partial_grid() < ST_MAX_WG ? partial_grid() : ST_MAX_WG;
    return attn_launch(q, k_new, v_new, Kp, Vp, slots, pos, out, part_o, part_ml, seg_tab, grid, B, M, Lmax, n_slots, CH, stream);
}

}  // extern "C"
