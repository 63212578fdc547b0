// Fused GatedDeltaNet decode / speculative-verify step for gfx950.
//
// One workgroup (256 threads = 4 wavefronts of 64) owns ROWS = RS*16 value rows of one (sequence, head) and streams them
// HBM -> registers -> HBM exactly once: conv4 + SiLU, q/k L2 norm, gates, then for every value row r
//     s = S[r,:] * g;  kv = s.k;  delta = (v_r - kv) * beta;  s += k * delta;  y_r = s.q
// (qwen35/kernels.py:518-530).  Replaces the Metal kernels deltanet_b (qwen35/batch.py:36-135), deltanet_bm
// (qwen35/batch_spec.py:45-150) and deltanet_m{M} (qwen35/kernels.py:461-567).
//
// Memory layout (slot-major, as qwen35/batch.py:1-12): ssm pool [S+1][16][128][128] f32, one head = 64 KiB contiguous;
// a 16-lane group reads 256 contiguous bytes of a row per load, a wavefront 4 rows, the workgroup 16 rows = 8 KiB per
// load slot.  Both dot products of a row are taken from the state as loaded,
//     kv = g * (S_r . k),   y_r = g * (S_r . q) + delta * (k . q),
// so the two 16-lane DPP reductions of a row are independent and the row is touched once.
#include "qt_common.h"

using namespace qt;

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));   // native vector: nontemporal loads / stores take it

struct RawIn {          // the un-convolved inputs one prologue thread needs for one token
    float w0, w1, w2, x;
    uint2 c;
};

// input row t of channel ch for the chained tokens of one sequence: t < 0 reads the stored window (kernels.py:477-479)
__device__ __forceinline__ float inp(const bf16_t* __restrict__ cs_in, const bf16_t* __restrict__ proj, int t, int ch) {
    return t < 0 ? bf2f(cs_in[(t + 3) * CD + ch]) : bf2f(proj[(size_t)t * PW + ch]);
}
__device__ __forceinline__ RawIn load_raw(const bf16_t* __restrict__ cs_in, const bf16_t* __restrict__ proj,
                                          const bf16_t* __restrict__ cw, int j, int ch) {
    RawIn r;
    r.w0 = inp(cs_in, proj, j - 3, ch);
    r.w1 = inp(cs_in, proj, j - 2, ch);
    r.w2 = inp(cs_in, proj, j - 1, ch);
    r.x = inp(cs_in, proj, j, ch);
    r.c = *reinterpret_cast<const uint2*>(cw + (size_t)ch * 4);
    return r;
}
__device__ __forceinline__ void store_window(bf16_t* __restrict__ cs_out, const RawIn& r, int ch) {
    cs_out[ch] = f2bf(r.w1);            // kernels.py:531: the new window is the last three input rows
    cs_out[CD + ch] = f2bf(r.w2);
    cs_out[2 * CD + ch] = f2bf(r.x);
}

// M chained tokens of one (sequence, head, row split).  Snapshot j of the state goes to st_out + j*st_stride and of the
// conv window to cs_out + j*cs_stride (strides 0 = update in place).
// NORM (whole heads only, RS = 8): y receives the gated RMSNorm of the head's 128 outputs, BF(z sigmoid(z) gw (y inv)) with
// z = proj[6144 + h*128 + row] (qwen35/batch.py:321-331), instead of the outputs themselves: same bits as the stand-alone
// norm kernel applied to the stored outputs.
template <int RS, int HPW = 1, bool NORM = false>
__device__ __forceinline__ void gdn_tokens(const bf16_t* __restrict__ proj, const bf16_t* __restrict__ cs_in,
                                           bf16_t* __restrict__ cs_out, size_t cs_stride,
                                           const bf16_t* __restrict__ cw, const float* __restrict__ A_log,
                                           const float* __restrict__ dt_bias, const float* st_in,
                                           float* st_out, size_t st_stride, bf16_t* __restrict__ y, int M, int h,
                                           int split, const float* __restrict__ gw = nullptr, float eps = 0.f) {
    static_assert(!NORM || RS == 8, "the fused norm needs the whole head in one group of 256 threads");
    constexpr int ROWS = RS * 16;
    __shared__ double red_a[HPW][4];
    __shared__ __align__(16) float qk_a[HPW][2][DK];
    __shared__ float v_a[HPW][ROWS];
    __shared__ float gb_a[HPW][2];
    // HPW heads per workgroup: each group of 256 threads runs one head, only the barriers are shared
    const int sub = HPW > 1 ? (int)(threadIdx.x >> 8) : 0;
    double* red = red_a[sub];
    float (*qk_s)[DK] = qk_a[sub];
    float* v_s = v_a[sub];
    float* gb_s = gb_a[sub];

    const int tid = threadIdx.x & 255, w = tid >> 6, lane = tid & 63, grp = lane >> 4, c = lane & 15;
    const int row0 = split * ROWS;
    const int which = tid >> 7;                                  // 0: a q channel, 1: a k channel
    const int ch_qk = which * KD + h * DK + (tid & 127);
    const bool has_v = tid < ROWS;
    const int ch_v = 2 * KD + h * DV + row0 + tid;

    // ---- token 0's prologue inputs first, then the state: the prologue runs while the state is in flight.  Every load
    // below is unconditional (threads without a v channel re-read their q/k channel) so that nothing has to be waited
    // for before the state loads are issued.
    const int ch_v_ld = has_v ? ch_v : ch_qk;
    RawIn rq = load_raw(cs_in, proj, cw, 0, ch_qk);
    RawIn rv = load_raw(cs_in, proj, cw, 0, ch_v_ld);
    // gates are evaluated by wave 3: lane 1 the decay gate (reads a), lane 2 beta (reads b)
    const int gl = lane < 3 ? lane : 0;
    float gx = bf2f(proj[CD + KD + HV * (gl == 1 ? 1 : 0) + h]);       // lane 1: a;  lanes 0, 2: b
    const float gA = A_log[h], gdt = dt_bias[h];
    // fused norm: lane c < 8 of a 16-lane group finishes the group's row i = c (row c*16 + w*4 + grp of the head)
    const int nrow = (c & 7) * 16 + w * 4 + grp;
    float nz = 0.f, ngw = 0.f;
    if (NORM) {
        nz = bf2f(proj[CD + h * DV + nrow]);
        ngw = gw[nrow];
    }
    __builtin_amdgcn_sched_barrier(0);           // keep the small loads ahead of the state loads in issue order

    f4 s[RS][2];
    {
        const f4* sin4 = reinterpret_cast<const f4*>(st_in + ((size_t)h * DV + row0) * DK);
#pragma unroll
        for (int i = 0; i < RS; i++) {
            const int row = i * 16 + w * 4 + grp;
            s[i][0] = __builtin_nontemporal_load(sin4 + row * (DK / 4) + c);
            s[i][1] = __builtin_nontemporal_load(sin4 + row * (DK / 4) + 16 + c);
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    const float sc = which == 0 ? BF(INV_SCALE * INV_SCALE) : BF(INV_SCALE);       // kernels.py:492
    for (int j = 0; j < M; j++) {
        if (j > 0) {
            rq = load_raw(cs_in, proj, cw, j, ch_qk);
            rv = load_raw(cs_in, proj, cw, j, ch_v_ld);
            gx = bf2f(proj[(size_t)j * PW + CD + KD + HV * (gl == 1 ? 1 : 0) + h]);
        }
        bf16_t* cso = cs_out + (size_t)j * cs_stride;
        // conv + silu, exact sum of squares over the head's 128 q (waves 0,1) / k (waves 2,3) channels
        const float u = conv_silu(rq.w0, rq.w1, rq.w2, rq.x, rq.c);
        const double tot = wave_sum_d((double)u * (double)u);
        if (lane == 0) red[w] = tot;
        if (split == 0) store_window(cso, rq, ch_qk);
        float vv = 0.f;
        if (has_v) {
            vv = conv_silu(rv.w0, rv.w1, rv.w2, rv.x, rv.c);
            store_window(cso, rv, ch_v);
        }
        float g = 0.f, beta = 0.f;
        if (w == 3) {                                                            // kernels.py:511-515
            // lane 1: decay gate from a; lane 2: beta from b
            g = __shfl(decay_gate(gA, BF(gx + gdt)), 1, 64);
            beta = __shfl(sigmoid_bf16(gx), 2, 64);
        }
        __syncthreads();
        {
            const float ss = (float)(red[which * 2] + red[which * 2 + 1]);
            const float r = rsqrt_rn(ss / (float)DK + qk_eps());
            qk_s[which][tid & 127] = BF(BF(u * r) * sc);                         // kernels.py:507-510
            if (has_v) v_s[tid] = vv;
            if (tid == 192) {
                gb_s[0] = g;
                gb_s[1] = beta;
            }
        }
        __syncthreads();

        // ---- the recurrence over this thread's 8 columns of RS rows
        float q8[8], k8[8];
        {
            const float4 a = reinterpret_cast<const float4*>(qk_s[0])[c], b = reinterpret_cast<const float4*>(qk_s[0])[16 + c];
            const float4 d = reinterpret_cast<const float4*>(qk_s[1])[c], e = reinterpret_cast<const float4*>(qk_s[1])[16 + c];
            q8[0] = a.x; q8[1] = a.y; q8[2] = a.z; q8[3] = a.w; q8[4] = b.x; q8[5] = b.y; q8[6] = b.z; q8[7] = b.w;
            k8[0] = d.x; k8[1] = d.y; k8[2] = d.z; k8[3] = d.w; k8[4] = e.x; k8[5] = e.y; k8[6] = e.z; k8[7] = e.w;
        }
        const float gg = gb_s[0], bb = gb_s[1];
        const float kq = dot8_row16(k8, q8);

        f4* so4 = reinterpret_cast<f4*>(st_out + (size_t)j * st_stride + ((size_t)h * DV + row0) * DK);
        bf16_t* yo = y + (size_t)j * KD + h * DV + row0;
        float yb[RS];
#pragma unroll
        for (int i = 0; i < RS; i++) {
            const int row = i * 16 + w * 4 + grp;
            float sv[8] = {s[i][0].x, s[i][0].y, s[i][0].z, s[i][0].w, s[i][1].x, s[i][1].y, s[i][1].z, s[i][1].w};
            const float yv = gdn_row_step(sv, k8, q8, v_s[row], gg, bb, kq);
            s[i][0] = f4{sv[0], sv[1], sv[2], sv[3]};
            s[i][1] = f4{sv[4], sv[5], sv[6], sv[7]};
            __builtin_nontemporal_store(s[i][0], so4 + row * (DK / 4) + c);
            __builtin_nontemporal_store(s[i][1], so4 + row * (DK / 4) + 16 + c);
            if (!NORM) {
                if (c == 0) yo[row] = f2bf(yv);
            } else {
                yb[i] = BF(yv);
            }
        }
        if (NORM) {
            // sum of squares of the head's 128 stored outputs: this lane's 8 rows, the wavefront's 4 groups, the 4 wavefronts
            double ss = 0.0;
#pragma unroll
            for (int i = 0; i < RS; i++) ss += (double)yb[i] * yb[i];
            ss += __shfl_xor(ss, 16, 64);
            ss += __shfl_xor(ss, 32, 64);
            __syncthreads();                                     // `red` was last read in the prologue
            if (lane == 0) red[w] = ss;
            __syncthreads();
            const float inv = rsqrt_rn((float)((red[0] + red[1]) + (red[2] + red[3])) / 128.f + eps);
            float mine = yb[0];
#pragma unroll
            for (int i = 1; i < RS; i++) mine = ((c & 7) == i) ? yb[i] : mine;
            if (c < 8) yo[nrow] = gated_out(nz, ngw * (mine * inv));
        }
    }
}

template <int RS>
__device__ __forceinline__ void split_id(int& b, int& h, int& split) {
    constexpr int NSPLIT = 8 / RS;
    const unsigned id = xcd_remap(blockIdx.x, gridDim.x);
    b = id / (HV * NSPLIT);
    const unsigned rem = id % (HV * NSPLIT);
    h = rem / NSPLIT;
    split = rem % NSPLIT;
}

// batch.deltanet_b (qwen35/batch.py:128-135): one token per row, pools updated in place
template <int RS>
__global__ __launch_bounds__(256) void gdn_decode_kernel(const bf16_t* __restrict__ proj, bf16_t* conv_pool,
                                                         const bf16_t* __restrict__ cw, const float* __restrict__ A_log,
                                                         const float* __restrict__ dt_bias, float* ssm_pool,
                                                         const int* __restrict__ slots, const int* __restrict__ pos,
                                                         bf16_t* __restrict__ y, int n_slots) {
    int b, h, split;
    split_id<RS>(b, h, split);
    const int slot = slots[b];
    if ((unsigned)slot >= (unsigned)n_slots) return;             // never touch memory outside the pools
    const int par = pos[b] & 1;                                  // batch.py:49-52: read buffer pos&1, write the other
    float* st = ssm_pool + (size_t)slot * HV * DV * DK;
    gdn_tokens<RS>(proj + (size_t)b * PW, conv_pool + (size_t)(slot * 2 + par) * 3 * CD,
                   conv_pool + (size_t)(slot * 2 + (par ^ 1)) * 3 * CD, 0, cw, A_log, dt_bias, st, st, 0,
                   y + (size_t)b * KD, 1, h, split);
}

// the same step with HPW heads of one row per workgroup (256 threads per head, whole heads only): the workgroup streams
// HPW * 64 KiB of contiguous state
template <int HPW, bool NORM = false>
__global__ __launch_bounds__(256 * HPW) void gdn_decode_wide_kernel(const bf16_t* __restrict__ proj, bf16_t* conv_pool,
                                                                    const bf16_t* __restrict__ cw,
                                                                    const float* __restrict__ A_log,
                                                                    const float* __restrict__ dt_bias, float* ssm_pool,
                                                                    const int* __restrict__ slots,
                                                                    const int* __restrict__ pos, bf16_t* __restrict__ y,
                                                                    int n_slots, const float* __restrict__ gw = nullptr,
                                                                    float eps = 0.f) {
    const unsigned id = xcd_remap(blockIdx.x, gridDim.x);
    const int b = id / (HV / HPW), h = (id % (HV / HPW)) * HPW + (threadIdx.x >> 8);
    const int slot = slots[b];
    if ((unsigned)slot >= (unsigned)n_slots) return;
    const int par = pos[b] & 1;
    float* st = ssm_pool + (size_t)slot * HV * DV * DK;
    gdn_tokens<8, HPW, NORM>(proj + (size_t)b * PW, conv_pool + (size_t)(slot * 2 + par) * 3 * CD,
                             conv_pool + (size_t)(slot * 2 + (par ^ 1)) * 3 * CD, 0, cw, A_log, dt_bias, st, st, 0,
                             y + (size_t)b * KD, 1, h, 0, gw, eps);
}

// batch_spec.deltanet_bm (qwen35/batch_spec.py:142-150): M chained tokens per sequence, snapshot pools in place
template <int RS>
__global__ __launch_bounds__(256) void gdn_verify_kernel(const bf16_t* __restrict__ proj, bf16_t* conv_pool,
                                                         const bf16_t* __restrict__ cw, const float* __restrict__ A_log,
                                                         const float* __restrict__ dt_bias, float* ssm_pool,
                                                         const int* __restrict__ sslots, const int* __restrict__ sels,
                                                         const int* __restrict__ pars, bf16_t* __restrict__ y, int M,
                                                         int n_entries) {
    int b, h, split;
    split_id<RS>(b, h, split);
    const int ss = sslots[b], sl = sels[b];
    if ((unsigned)ss >= (unsigned)n_entries || (unsigned)sl >= (unsigned)M) return;
    const int par = pars[b] & 1;
    const size_t hs = (size_t)HV * DV * DK;
    gdn_tokens<RS>(proj + (size_t)b * M * PW, conv_pool + ((size_t)(ss * 2 + par) * M + sl) * 3 * CD,
                   conv_pool + (size_t)(ss * 2 + (par ^ 1)) * M * 3 * CD, (size_t)3 * CD, cw, A_log, dt_bias,
                   ssm_pool + ((size_t)ss * M + sl) * hs, ssm_pool + (size_t)ss * M * hs, hs, y + (size_t)b * M * KD, M,
                   h, split);
}

// kernels.deltanet (qwen35/kernels.py:555-567): one sequence, starts from snapshot sel[0], writes M fresh snapshots
template <int RS>
__global__ __launch_bounds__(256) void gdn_solo_kernel(const bf16_t* __restrict__ proj, const bf16_t* __restrict__ cs_snap,
                                                       const bf16_t* __restrict__ cw, const float* __restrict__ A_log,
                                                       const float* __restrict__ dt_bias, const float* __restrict__ st_snap,
                                                       const int* __restrict__ sel, bf16_t* __restrict__ y,
                                                       bf16_t* __restrict__ cs_out, float* __restrict__ st_out, int M,
                                                       int n_snap) {
    int b, h, split;
    split_id<RS>(b, h, split);
    const int sl = sel[0];
    if ((unsigned)sl >= (unsigned)n_snap) return;
    const size_t hs = (size_t)HV * DV * DK;
    gdn_tokens<RS>(proj, cs_snap + (size_t)sl * 3 * CD, cs_out, (size_t)3 * CD, cw, A_log, dt_bias, st_snap + sl * hs,
                   st_out, hs, y, M, h, split);
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// rows per workgroup: few sequences -> split a head over more workgroups so the chip still fills
inline int pick_rs(int nseq, int rows_split) {
    if (rows_split == 128 || rows_split == 64 || rows_split == 32 || rows_split == 16) return rows_split / 16;
    if (nseq >= 32) return 8;
    if (nseq >= 8) return 4;
    if (nseq >= 4) return 2;
    return 1;
}

// The decode step's shape: whole heads per workgroup (1, 2 or 4) while B x 16 heads give every CU a workgroup (measured, us at
// 1 / 2 / 4 heads: B = 16 6.7 / 7.7 / 11.4, 24 11.9 / 9.8 / 12.1, 32 12.4 / 12.3 / 13.5, 48 19.2 / 21.2 / 18.5, 64 25.6 / 24.8 /
// 23.7), below that a head split over 2, 4 or 8 workgroups (B = 8: 5.5 us at 2 or 4 parts, B = 4: 4.5 us at 4).
// Beyond one round of four-head workgroups (B > 64) small workgroups balance the rounds better: half a head each (B = 96
// 38.1 against 39.5 us, B = 128 50.7 against 52.1), a whole head where the fused norm needs one.
inline int decode_heads_per_wg(int B) {
    const long heads = (long)B * HV, cus = cu_count();
    return heads > 4 * cus ? 1 : heads > 2 * cus ? 4 : heads > cus ? 2 : 1;
}
inline int decode_rs(int B) {                                    // 16-row groups per workgroup when a head is split
    const long heads = (long)B * HV, cus = cu_count();
    if (heads > 4 * cus) return 4;
    int rs = 8;
    while (rs > 1 && heads * (8 / rs) * 2 <= cus) rs >>= 1;
    return rs;
}

}  // namespace

#define QT_DISPATCH_RS(rs, KERNEL, nseq, stream, ...)                                                  \
    switch (rs) {                                                                                       \
        case 8: hipLaunchKernelGGL(KERNEL<8>, dim3((nseq) * HV * 1), dim3(256), 0, stream, __VA_ARGS__); break; \
        case 4: hipLaunchKernelGGL(KERNEL<4>, dim3((nseq) * HV * 2), dim3(256), 0, stream, __VA_ARGS__); break; \
        case 2: hipLaunchKernelGGL(KERNEL<2>, dim3((nseq) * HV * 4), dim3(256), 0, stream, __VA_ARGS__); break; \
        default: hipLaunchKernelGGL(KERNEL<1>, dim3((nseq) * HV * 8), dim3(256), 0, stream, __VA_ARGS__); break; \
    }

extern "C" {

int qt_gdn_decode_step(const void* proj, void* conv_pool, const void* conv_w, const float* A_log, const float* dt_bias,
                       float* ssm_pool, const int32_t* slots, const int32_t* pos, void* y, int B, int n_slots,
                       int rows_per_wg, hipStream_t stream) {
    if (!proj || !conv_pool || !conv_w || !A_log || !dt_bias || !ssm_pool || !slots || !pos || !y) return QT_ERR_NULL;
    if (B < 0 || n_slots <= 0) return QT_ERR_DIM;
    if (B == 0) return QT_OK;
    if (!aligned16(ssm_pool) || (reinterpret_cast<uintptr_t>(conv_w) & 7u)) return QT_ERR_ALIGN;
    // Many rows: 2 or 4 whole heads of a row per workgroup (128 / 256 KiB of contiguous state per workgroup); measured at
    // B = 64: 23.3 us against 26.0 us with one head per workgroup.  Few rows: split heads so the chip still fills.  The shape
    // that wins at every batch size measured (4 .. 64 rows) is the largest one that still gives every CU a workgroup.
    const int hpw = rows_per_wg == 512 ? 4 : rows_per_wg == 256 ? 2 : rows_per_wg != 0 ? 1 : decode_heads_per_wg(B);
    if (hpw == 4) {
        hipLaunchKernelGGL(gdn_decode_wide_kernel<4>, dim3(B * (HV / 4)), dim3(1024), 0, stream, (const bf16_t*)proj,
                           (bf16_t*)conv_pool, (const bf16_t*)conv_w, A_log, dt_bias, ssm_pool, slots, pos, (bf16_t*)y, n_slots);
    } else if (hpw == 2) {
        hipLaunchKernelGGL(gdn_decode_wide_kernel<2>, dim3(B * (HV / 2)), dim3(512), 0, stream, (const bf16_t*)proj,
                           (bf16_t*)conv_pool, (const bf16_t*)conv_w, A_log, dt_bias, ssm_pool, slots, pos, (bf16_t*)y, n_slots);
    } else {
        const int rs = rows_per_wg ? pick_rs(B, rows_per_wg) : decode_rs(B);
        QT_DISPATCH_RS(rs, gdn_decode_kernel, B, stream, (const bf16_t*)proj, (bf16_t*)conv_pool, (const bf16_t*)conv_w, A_log,
                       dt_bias, ssm_pool, slots, pos, (bf16_t*)y, n_slots);
    }
    QT_CHECK_LAUNCH();
    return QT_OK;
}

// batch.deltanet_b followed by batch.gnorm_rows (qwen35/batch.py:128-135, 338-343) in one launch: `out` receives the gated
// RMSNorm of the step's outputs (same bits as the two launches), the outputs themselves are not stored.
int qt_gdn_decode_step_gnorm(const void* proj, void* conv_pool, const void* conv_w, const float* A_log, const float* dt_bias,
                             float* ssm_pool, const int32_t* slots, const int32_t* pos, const float* gw, float eps, void* out, int B,
                             int n_slots, hipStream_t stream) {
    if (!proj || !conv_pool || !conv_w || !A_log || !dt_bias || !ssm_pool || !slots || !pos || !gw || !out) return QT_ERR_NULL;
    if (B < 0 || n_slots <= 0) return QT_ERR_DIM;
    if (B == 0) return QT_OK;
    if (!aligned16(ssm_pool) || (reinterpret_cast<uintptr_t>(conv_w) & 7u)) return QT_ERR_ALIGN;
#define QT_GNORM_LAUNCH(HPW_)                                                                                                  \
    hipLaunchKernelGGL((gdn_decode_wide_kernel<HPW_, true>), dim3(B * (HV / HPW_)), dim3(256 * HPW_), 0, stream, (const bf16_t*)proj, \
                       (bf16_t*)conv_pool, (const bf16_t*)conv_w, A_log, dt_bias, ssm_pool, slots, pos, (bf16_t*)out, n_slots, gw, eps)
    const int hpw = decode_heads_per_wg(B);
    if (hpw == 4) QT_GNORM_LAUNCH(4);
    else if (hpw == 2) QT_GNORM_LAUNCH(2);
    else QT_GNORM_LAUNCH(1);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

int qt_gdn_verify_step(const void* proj, void* conv_pool, const void* conv_w, const float* A_log, const float* dt_bias,
                       float* ssm_pool, const int32_t* sslots, const int32_t* sels, const int32_t* pars, void* y, int B,
                       int M, int n_entries, int rows_per_wg, hipStream_t stream) {
    if (!proj || !conv_pool || !conv_w || !A_log || !dt_bias || !ssm_pool || !sslots || !sels || !pars || !y) return QT_ERR_NULL;
    if (B < 0 || n_entries <= 0) return QT_ERR_DIM;
    if (M < 1 || M > 16) return QT_ERR_UNSUPPORTED;
    if (B == 0) return QT_OK;
    if (!aligned16(ssm_pool) || (reinterpret_cast<uintptr_t>(conv_w) & 7u)) return QT_ERR_ALIGN;
    const int rs = pick_rs(B, rows_per_wg);
    QT_DISPATCH_RS(rs, gdn_verify_kernel, B, stream, (const bf16_t*)proj, (bf16_t*)conv_pool, (const bf16_t*)conv_w, A_log,
                   dt_bias, ssm_pool, sslots, sels, pars, (bf16_t*)y, M, n_entries);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

int qt_gdn_deltanet(const void* proj, const void* conv_snap, const void* conv_w, const float* A_log, const float* dt_bias,
                    const float* ssm_snap, const int32_t* sel, void* y, void* cs_out, float* st_out, int M, int n_snap,
                    int rows_per_wg, hipStream_t stream) {
    if (!proj || !conv_snap || !conv_w || !A_log || !dt_bias || !ssm_snap || !sel || !y || !cs_out || !st_out) return QT_ERR_NULL;
    if (n_snap <= 0) return QT_ERR_DIM;
    if (M < 1 || M > 16) return QT_ERR_UNSUPPORTED;
    if (!aligned16(ssm_snap) || !aligned16(st_out) || (reinterpret_cast<uintptr_t>(conv_w) & 7u)) return QT_ERR_ALIGN;
    const int rs = pick_rs(1, rows_per_wg);
    QT_DISPATCH_RS(rs, gdn_solo_kernel, 1, stream, (const bf16_t*)proj, (const bf16_t*)conv_snap, (const bf16_t*)conv_w, A_log,
                   dt_bias, ssm_snap, sel, (bf16_t*)y, (bf16_t*)cs_out, st_out, M, n_snap);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

}  // extern "C"
