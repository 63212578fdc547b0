// Device helpers shared by every kernel of the GatedDeltaNet / GQA-hd256 hot path (gfx950 only).
//
// Arithmetic contract of the elementwise prologue (conv + SiLU, q/k norm, gates, gated RMSNorm).  It keeps the
// reference's bf16 rounding points (qwen35/mslib.py:7-27, qwen35/kernels.py:476-515) and fixes the last-place
// behaviour so that a CPU restatement reproduces every bf16 value bit for bit:
//   exp32 / log32 : double-precision libm result rounded to float
//   sum of squares: exact (double), rounded to float once
//   rsqrt         : 1 / sqrt evaluated in double precision and rounded to float once
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qt {

constexpr int HV = 16, DK = 128, DV = 128, KD = 2048, CD = 6144, PW = 8224;   // qwen35/batch.py:29
constexpr int AH = 8, AKV = 2, AD = 256;                                        // qwen35/model.py:43-45

typedef uint16_t bf16_t;   // raw bf16 bits

__device__ __forceinline__ float bf2f(bf16_t b) { return __uint_as_float((uint32_t)b << 16); }

__device__ __forceinline__ bf16_t f2bf(float f) {   // round to nearest even (v_cvt_pk_bf16_f32 on gfx950)
    return __builtin_bit_cast(bf16_t, static_cast<__bf16>(f));
}

__device__ __forceinline__ float BF(float f) { return bf2f(f2bf(f)); }          // `#define BF(v)`, mslib.py:8-10

__device__ __forceinline__ float lo_bf(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float hi_bf(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ uint32_t pack_bf(float a, float b) { return (uint32_t)f2bf(a) | ((uint32_t)f2bf(b) << 16); }

__device__ __forceinline__ float exp32(float x) { return (float)exp((double)x); }
__device__ __forceinline__ float log32(float x) { return (float)log((double)x); }
__device__ __forceinline__ float rsqrt_rn(float x) { return (float)(1.0 / sqrt((double)x)); }   // correctly rounded 1/sqrt

// The bf16 -> bf16 helpers below must return the bits the contract defines (exp32 / log32 = correctly rounded), but the
// double-precision libm calls are ~10x the work of the float ones.  A float result that is off by a few ulp rounds to the
// same bf16 value unless it lies within those few ulp of a bf16 rounding boundary; only then is the slow path taken
// (about one evaluation in 10^4).  The GPU tests compare all 65536 inputs of each helper with a CPU restatement.
__device__ __forceinline__ bool near_bf16_tie(float v, uint32_t slack) {
    const uint32_t lo = __float_as_uint(v) & 0xffffu;
    return (lo - (0x8000u - slack)) <= 2u * slack;
}
__device__ __forceinline__ float bf_exp(float x) {                               // BF(exp32(x))
    float e = expf(x);                                                           // <= 1 ulp
    if (__builtin_expect(near_bf16_tie(e, 4) || fabsf(x) > 80.0f, 0)) e = exp32(x);
    return BF(e);
}
__device__ __forceinline__ float bf_rcp(float d) {                               // BF(1 / d), IEEE divide
    float r = __builtin_amdgcn_rcpf(d);                                          // <= 1 ulp
    if (__builtin_expect(near_bf16_tie(r, 3) || !(fabsf(d) > 1e-30f && fabsf(d) < 1e30f), 0)) r = __fdiv_rn(1.0f, d);
    return BF(r);
}

__device__ __forceinline__ float log1p_mx(float x) {                             // mslib.py:11-15
    float xp1 = 1.0f + x;
    if (xp1 == 1.0f) return x;
    return x * __fdiv_rn(log32(xp1), xp1 - 1.0f);
}
__device__ __forceinline__ float bf_log1p_mx(float x) {                          // BF(log1p_mx(x)) for x in [0, 1]
    const float xp1 = 1.0f + x;
    if (xp1 == 1.0f) return BF(x);
    float r = x * __fdiv_rn(logf(xp1), xp1 - 1.0f);
    if (__builtin_expect(near_bf16_tie(r, 6), 0)) r = log1p_mx(x);
    return BF(r);
}
__device__ __forceinline__ float sigmoid_bf16(float x) {                         // mslib.py:16-20
    const float y = bf_rcp(BF(1.0f + bf_exp(fabsf(x))));
    return x < 0.0f ? y : BF(1.0f - y);
}
__device__ __forceinline__ float silu_bf16(float x) { return BF(x * sigmoid_bf16(x)); }   // mslib.py:21-22
__device__ __forceinline__ float softplus_bf16(float x) {                        // mslib.py:23-26
    return BF(fmaxf(x, 0.0f) + bf_log1p_mx(bf_exp(-fabsf(x))));
}
// decay gate of one head: g = exp(-exp(A_log) * softplus_bf16(av)) (kernels.py:511-513).  The reference evaluates it with
// float exp and does not round it; here both exps are float with <= 1 ulp error.
__device__ __forceinline__ float log_decay(float A_log, float av) { return -expf(A_log) * softplus_bf16(av); }
__device__ __forceinline__ float decay_gate(float A_log, float av) { return expf(log_decay(A_log, av)); }
// exp(-z) for a bf16 value z, |z| <= 16, in four instructions.  -log2(e) = c1 + c2 with c1 of 16 significant bits, so the
// product z c1 is exact in float; exp(-z) = 2^(z c1) (1 + z c2 ln 2 + ...), the second-order term below 1e-8.  v_exp_f32 is
// good to 1 ulp, the multiply-add adds half of one.
__device__ __forceinline__ float exp_neg_bf16(float z) {
    const float e0 = __builtin_amdgcn_exp2f(z * -1.44268798828125f);
    return __builtin_fmaf(e0, z * -4.888495152129525e-06f, e0);
}
// z * sigmoid(z) * n rounded to bf16 once (kernels.py:134-137): z/(1+exp32(-z)) * n, z a bf16 value.  The fast path uses the
// hardware reciprocal and the exponential above (a few ulp off in total); a result within 16 float ulp of a bf16 rounding
// boundary, or |z| > 16, takes the exact path (IEEE divide, double-precision exp).
__device__ __forceinline__ bool gated_out_fast(float z, float n, float& o) {
    o = z * __builtin_amdgcn_rcpf(1.0f + exp_neg_bf16(z)) * n;
    return !(near_bf16_tie(o, 16) || !(fabsf(z) <= 16.0f));
}
__device__ __forceinline__ bf16_t gated_out(float z, float n) {
    float o;
    if (__builtin_expect(!gated_out_fast(z, n, o), 0)) o = __fdiv_rn(z, 1.0f + exp32(-z)) * n;
    return f2bf(o);
}

// 4-tap depthwise conv + SiLU of one channel (kernels.py:480-484): w0..w2 = the three previous input rows (oldest
// first), x = the current row, c = the channel's four taps (tap 3 multiplies the current token).
__device__ __forceinline__ float conv_silu(float w0, float w1, float w2, float x, uint2 c) {
    float s = w0 * lo_bf(c.x);
    s = s + w1 * hi_bf(c.x);
    s = s + w2 * lo_bf(c.y);
    s = s + x * hi_bf(c.y);
    return silu_bf16(BF(s));
}

// silu_bf16 is a bf16 -> bf16 map, so kernels that evaluate it many times per thread read it from a table in LDS:
// 24 exponents (bf16 exponent fields 110..133, 2^-17 <= |x| < 2^7) x 128 mantissas x 2 signs = 6144 entries (12 KiB), the two
// signs of a magnitude side by side: entry index = rotl16(x, 1) - 2 * (110 << 7).  Outside that range the map needs no
// exponential (silu_out_of_table).  The table array has 8 more entries: index SILU_TAB_N2 is where out-of-range lookups land.
constexpr int SILU_TAB_LO = 110, SILU_TAB_N2 = 2 * 24 * 128, SILU_TAB_SIZE = SILU_TAB_N2 + 8;
__device__ __forceinline__ bf16_t silu_table_entry(int i) {
    if (i >= SILU_TAB_N2) return 0;
    const bf16_t xb = (bf16_t)(((i & 1) << 15) | (SILU_TAB_LO * 128 + (i >> 1)));
    return f2bf(silu_bf16(bf2f(xb)));
}
// fills `tab` (LDS) from a prebuilt copy in global memory, or computes it when there is none
__device__ __forceinline__ void silu_table_fill(bf16_t* tab, const bf16_t* __restrict__ prebuilt, int tid, int nthreads) {
    if (prebuilt) {
        for (int i = tid; i < SILU_TAB_SIZE / 8; i += nthreads)
            reinterpret_cast<uint4*>(tab)[i] = reinterpret_cast<const uint4*>(prebuilt)[i];
    } else {
        for (int i = tid; i < SILU_TAB_SIZE; i += nthreads) tab[i] = silu_table_entry(i);
    }
}
// silu_bf16 outside the table's range.  Below 2^-17, exp(|x|) rounds to 1 in bf16 and the sigmoid is exactly 1/2.  From 2^7 on,
// exp(|x|) overflows float: the sigmoid is 1 for x > 0 (the result is x) and +0 for x < 0 (the result is x * 0: -0, and NaN for
// -inf).  NaN stays NaN.
__device__ __forceinline__ float silu_out_of_table(float x) {
    if (fabsf(x) < 1.0f) return BF(x * 0.5f);
    return x > 0.0f ? x : x * 0.0f;
}
__device__ __forceinline__ void unpack8(uint4 w, float (&f)[8]) {
    f[0] = lo_bf(w.x); f[1] = hi_bf(w.x); f[2] = lo_bf(w.y); f[3] = hi_bf(w.y);
    f[4] = lo_bf(w.z); f[5] = hi_bf(w.z); f[6] = lo_bf(w.w); f[7] = hi_bf(w.w);
}
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
// two floats rounded to bf16 (nearest even) by one v_cvt_pk_bf16_f32: a in the low half
__device__ __forceinline__ uint32_t pack2_bf(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}
// table index of both halves of a bf16 pair (packed 16-bit arithmetic): rotl16(x, 1) - 2 * (LO << 7), wrapping for small |x|
__device__ __forceinline__ u16x2 silu_index2(uint32_t w) {
    const u16x2 x = __builtin_bit_cast(u16x2, w);
    return x * (unsigned short)2 + (x >> 15) - (unsigned short)(SILU_TAB_LO * 256);
}
// conv4 + silu of 8 consecutive channels of one token: rows x0..x3 (oldest first, 8 bf16 each), taps wt (4 bf16 per channel);
// the results as four bf16 pairs (their values are what silu_bf16 returns).  An input outside the table reads the spare entry
// and is re-evaluated in one unlikely block per 8 channels.
__device__ __forceinline__ void conv8_silu_pairs(const bf16_t* tab, const uint4& x0, const uint4& x1, const uint4& x2,
                                                 const uint4& x3, const uint4 (&wt)[4], uint32_t (&r)[4]) {
    float a[8], b[8], c[8], d[8];
    unpack8(x0, a);
    unpack8(x1, b);
    unpack8(x2, c);
    unpack8(x3, d);
    float s[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const uint4 ww = wt[e >> 1];
        const uint32_t c0 = (e & 1) ? ww.z : ww.x, c1 = (e & 1) ? ww.w : ww.y;
        s[e] = a[e] * lo_bf(c0);
        s[e] = s[e] + b[e] * hi_bf(c0);
        s[e] = s[e] + c[e] * lo_bf(c1);
        s[e] = s[e] + d[e] * hi_bf(c1);
    }
    uint32_t xb[4];
    u16x2 worst = {0, 0};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        xb[i] = pack2_bf(s[2 * i], s[2 * i + 1]);
        const u16x2 idx = silu_index2(xb[i]);
        worst = __builtin_elementwise_max(worst, idx);
        const u16x2 off = __builtin_elementwise_min(idx, (u16x2){SILU_TAB_N2, SILU_TAB_N2}) << 1;     // byte offsets into the table
        const char* tb = reinterpret_cast<const char*>(tab);
        u16x2 v;
        v.x = *reinterpret_cast<const bf16_t*>(tb + off.x);
        v.y = *reinterpret_cast<const bf16_t*>(tb + off.y);
        r[i] = __builtin_bit_cast(uint32_t, v);
    }
    if (__builtin_expect(max(worst.x, worst.y) >= SILU_TAB_N2, 0)) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const u16x2 idx = silu_index2(xb[i]);
            if (idx.x >= SILU_TAB_N2) r[i] = (r[i] & 0xffff0000u) | f2bf(silu_out_of_table(lo_bf(xb[i])));
            if (idx.y >= SILU_TAB_N2) r[i] = (r[i] & 0x0000ffffu) | ((uint32_t)f2bf(silu_out_of_table(hi_bf(xb[i]))) << 16);
        }
    }
}

// conv4 + silu of 8 channels of one token, packed as bf16 pairs, and their exact sum of squares
__device__ __forceinline__ double conv8_silu_packed(const bf16_t* tab, const uint4& x0, const uint4& x1, const uint4& x2,
                                                    const uint4& x3, const uint4 (&wt)[4], uint4& packed) {
    uint32_t r[4];
    conv8_silu_pairs(tab, x0, x1, x2, x3, wt, r);
    packed = make_uint4(r[0], r[1], r[2], r[3]);
    float u[8];
    unpack8(packed, u);
    double sq = 0.0;
#pragma unroll
    for (int e = 0; e < 8; e++) sq += (double)u[e] * u[e];
    return sq;
}
// q/k normalization of 8 packed channels: BF(BF(u * r) * sc) (kernels.py:507-510)
__device__ __forceinline__ uint4 scale8_packed(const uint4& u, float r, float sc) {
    float f[8];
    unpack8(u, f);
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t t = pack2_bf(f[2 * i] * r, f[2 * i + 1] * r);
        o[i] = pack2_bf(lo_bf(t) * sc, hi_bf(t) * sc);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

constexpr float INV_SCALE = 0.08838834764831845f;                                // 128^-0.5, kernels.py:490
__device__ __forceinline__ float qk_eps() { return __fmul_rn(__fmul_rn(1e-6f, INV_SCALE), INV_SCALE); }   // kernels.py:491

// ---- cross-lane sums over an aligned group of 16 lanes (one DPP row); every lane of the group gets the total ----
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_mov<0xB1>(v);     // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E>(v);     // quad_perm [2,3,0,1]
    v += dpp_mov<0x141>(v);    // row_half_mirror
    v += dpp_mov<0x140>(v);    // row_mirror
    return v;
}
template <int CTRL>
__device__ __forceinline__ double dpp_mov_d(double v) {
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __builtin_amdgcn_update_dpp(0, lo, CTRL, 0xF, 0xF, true);
    hi = __builtin_amdgcn_update_dpp(0, hi, CTRL, 0xF, 0xF, true);
    return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double row16_sum_d(double v) {
    v += dpp_mov_d<0xB1>(v);
    v += dpp_mov_d<0x4E>(v);
    v += dpp_mov_d<0x141>(v);
    v += dpp_mov_d<0x140>(v);
    return v;
}
// value of lane I of each 16-lane row, to every lane of that row
template <int I>
__device__ __forceinline__ float row16_bcast(float v) { return dpp_mov<0x150 + I>(v); }
template <int N, int I = 0>
__device__ __forceinline__ void row16_bcast_all(float v, float (&r)[N]) {
    if constexpr (I < N) {
        r[I] = row16_bcast<I>(v);
        row16_bcast_all<N, I + 1>(v, r);
    }
}
// N <= 16 sums of squares of 128-wide rows (every lane of a 16-lane row holds all N) -> r[i] = rsqrt_rn(ss[i] / 128 + eps).
// Lane c of the row evaluates entry c % N only and the results are broadcast, so the double-precision rsqrt runs once per lane.
template <int N>
__device__ __forceinline__ void rsqrt_rows(const float (&ss)[N], float eps, float (&r)[N], int c) {
    // (each candidate passes through an empty asm: a bare chain of selects is turned into an indexed read of a stack array,
    // and a kernel that uses scratch memory at all starts its wavefronts more slowly)
    float mine = ss[0];
#pragma unroll
    for (int i = 1; i < N; i++) {
        float cand = ss[i];
        asm volatile("" : "+v"(cand));
        mine = (c % N == i) ? cand : mine;
    }
    const float rv = rsqrt_rn(mine / 128.0f + eps);
    row16_bcast_all<N>(rv, r);
}
// total over the whole 64-lane wavefront (every lane gets it)
__device__ __forceinline__ double wave_sum_d(double v) {
    v = row16_sum_d(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_mov<0xB1>(v));
    v = fmaxf(v, dpp_mov<0x4E>(v));
    v = fmaxf(v, dpp_mov<0x141>(v));
    v = fmaxf(v, dpp_mov<0x140>(v));
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}

// One value row of the gated delta rule, this lane's 8 of the 128 columns (kernels.py:518-530):
//   kv = g (S_r . k);  delta = (v - kv) beta;  y = g (S_r . q) + delta (k . q);  S_r <- g S_r + delta k
// pk / pq are reduced over the 16 lanes that share the row; kq = k . q (already reduced).  Returns y.
__device__ __forceinline__ float gdn_row_step(float (&sv)[8], const float (&k8)[8], const float (&q8)[8], float v, float g,
                                              float beta, float kq) {
    float pk = 0.f, pq = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        pk = fmaf(sv[e], k8[e], pk);
        pq = fmaf(sv[e], q8[e], pq);
    }
    pk = row16_sum(pk);
    pq = row16_sum(pq);
    const float delta = (v - g * pk) * beta;
    const float yv = fmaf(g, pq, delta * kq);
#pragma unroll
    for (int e = 0; e < 8; e++) sv[e] = fmaf(delta, k8[e], g * sv[e]);
    return yv;
}
__device__ __forceinline__ float dot8_row16(const float (&a)[8], const float (&b)[8]) {
    float t = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) t = fmaf(a[e], b[e], t);
    return row16_sum(t);
}

// workgroup id remapped so that consecutive logical ids share an XCD (8 XCDs, hardware deals workgroups round-robin)
__device__ __forceinline__ unsigned xcd_remap(unsigned id, unsigned n) {
    return (n % 8u == 0u) ? (id % 8u) * (n / 8u) + id / 8u : id;
}

}  // namespace qt

// CUs of the current device (256 if the query fails).  Cached per device id in atomics: any thread may ask, for any device,
// and the launch paths pay for the runtime query once per device.
#include <atomic>
namespace qt {
inline int cu_count() {
    constexpr int MAX_DEV = 64;
    static std::atomic<int> cache[MAX_DEV];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (dev >= 0 && dev < MAX_DEV) {
        const int c = cache[dev].load(std::memory_order_relaxed);
        if (c > 0) return c;
    }
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    if (dev >= 0 && dev < MAX_DEV) cache[dev].store(n, std::memory_order_relaxed);
    return n;
}
}  // namespace qt

// error codes of the C ABI
#define QT_OK 0
#define QT_ERR_DIM (-1)
#define QT_ERR_ALIGN (-2)
#define QT_ERR_NULL (-3)
#define QT_ERR_UNSUPPORTED (-4)
#define QT_ERR_LAUNCH (-5)
#define QT_ERR_WORKSPACE (-6)
#define QT_ERR_STATIC_MAX (-7)

#define QT_CHECK_LAUNCH()                                   \
    do {                                                    \
        hipError_t e_ = hipGetLastError();                  \
        if (e_ != hipSuccess) return QT_ERR_LAUNCH;         \
    } while (0)
