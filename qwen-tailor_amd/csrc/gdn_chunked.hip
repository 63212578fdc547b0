// Chunked (WY / UT transform) GatedDeltaNet prefill for gfx950, chunk size C = 64.
// Replaces the Metal kernels gdn_nax_a / gdn_nax_prep_a / gdn_nax_b (qwen35/gdn_nax.py:71-358), whose chunk is 16.
//
// Per head and chunk, with S0 [dv,dk] the state entering the chunk (gdn_nax.py:3-10):
//     Lc = cumsum(log g), gamma = exp(Lc), dec = exp(Lc_C - Lc), G_ij = exp(Lc_i - Lc_j)
//     L  = strict_lower(beta_i G_ij K K^T),  Tb = (I + L)^-1 diag(beta),  A = lower_incl(G * Q K^T)
//     D  = Tb (V - gamma * (K S0^T)),   Y = gamma * (Q S0^T) + A D,   S1 = gamma_C S0 + (dec * D)^T K
// Phase A (parallel over (chunk, head)) folds everything that does not depend on the state into MFMA operands
//     Wn = -Tb (gamma * K),  U = Tb V,  Qh = Q,  Kh = K^T,  Am = A      (half precision; gamma, dec, gamma_C as floats)
// so that the serial phase B is four register-resident GEMMs per chunk:
//     D = U + Wn S0^T;   Y = gamma * (Qh S0^T) + Am D;   S1^T = gamma_C S0^T + Kh (dec * D).
// The per-token factors gamma and dec are applied by the consumers to accumulator rows (four multiplications per tile)
// instead of by phase A to every operand element.
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
constexpr int OP_K = OP_Q + NCT * 4 * 512;      // Qh: same;  Kh: [mt 8][kb2 2][64][8]
constexpr int OP_A = OP_K + 8 * 2 * 512;        // Am: [ct 4][kb2 2][64][8]
constexpr int OP_HALVES = OP_A + NCT * 2 * 512; // 28672 halves = 56 KiB per (chunk, head)
constexpr int U_HALVES = 8 * NCT * 64 * 4;      // U: [slice 8][ct 4][lane 64][4] halves = 16 KiB per (chunk, head)
constexpr int G_GAM = 0, G_DEC = C, G_GC = 2 * C;   // gate record of a (chunk, head): gamma[64] | dec[64] | gamma_C, 0, 0, 0
constexpr int GATE_FLOATS = 2 * C + 4;

__device__ __forceinline__ half8 pack_half8(const f32x4& a, const f32x4& b) {
    half8 h;
    h[0] = (_Float16)a[0]; h[1] = (_Float16)a[1]; h[2] = (_Float16)a[2]; h[3] = (_Float16)a[3];
    h[4] = (_Float16)b[0]; h[5] = (_Float16)b[1]; h[6] = (_Float16)b[2]; h[7] = (_Float16)b[3];
    return h;
}

// Phase B has two roles.
//
// Chain workgroups (128) run the serial part: S_{c+1}^T = gamma_c S_c^T + Kh_c (dec_c * D_c) with D_c = U_c + Wn_c S_c^T.
// They compute no outputs; they leave, per (chunk, head, slice), the two half-precision B operands that the outputs need
// (S_c^T and D_c, 6 KiB) in `snap`.  Output units compute Y_c = gamma_c * (Qh_c S_c^T) + Am_c D_c from them.  Splitting the
// outputs off the chain halves the bytes the serial workgroups have to pull per step (W and Kh: 32 of the 56 KiB).
//
// Short sequences run the roles as two launches (chain, then one output workgroup per (chunk, head)).  Long ones run them as
// ONE launch: the chain publishes how many chunks are complete in a progress word per (head, slice) and the output units
// take the chunks as their snapshots appear, so only the last chunks' outputs remain when the chain ends.  In that form
// snapshots and progress words cross CUs (and XCDs, whose L2s are not coherent with each other) inside one launch, so they
// are written and read with device-scope accesses that go to memory; everything else uses plain accesses.  The writer never
// waits for its newest stores: it publishes chunk c - PUB_LAG once at most the stores of the PUB_LAG newest chunks are still
// in flight (stores of one wavefront complete in order).  The chain workgroups have the lowest indices, so all of them are
// running before the first output workgroup starts, and they wait for nothing: a consumer's producer is always running,
// whether or not every output workgroup is resident.  A consumer that does not see its snapshot within SPIN_LIMIT polls
// gives up: it sets bit 0 of the status word and leaves the item's output rows unwritten, so that every wavefront ends.
// Every workgroup of either role counts itself done when it has made its last store to the flag area (a chain workgroup
// after its final progress store has been acknowledged), and the last one to do so clears the progress words, the done
// count and the queue head: they are zero before and after every launch (the caller zeroes them once).  The status word
// is never cleared by a launch: it is the caller's to read and reset.  Bit 1 of it is set by a chain workgroup whose final
// state slice holds a value that is not finite: a half-precision operand (the state, D, U or a conv output) has overflowed.
//
// Chain role: 5 wavefronts per (head, 16-wide dv slice).  MFMA wavefront w owns rows 16w..16w+15 of D (the chunk's tokens) and
// rows 32w..32w+31 of S^T (dk): per chunk it pulls only its 8 operand tiles (8 KiB) and keeps PB_DEP chunks of them in flight
// in registers, so the latency of a load is covered by PB_DEP chain steps.  Two exchanges through LDS per step make up for
// the split: every wavefront publishes its block of S^T as the fp16 B operand and reads all four (barrier E1), and publishes
// its rows of D (scaled by dec for the update, and plain for the outputs) and reads both k-blocks (barrier E2).  The fifth
// wavefront copies S^T and the plain D from LDS to `snap`: the MFMA wavefronts issue loads only, which keeps their vmcnt
// waits partial (a store in flight next to loads forces every wait to zero on this target).
constexpr int SNAP_S = 4 * 512;                  // halves: S^T as B operand, [kb 4][lane 64][8]
constexpr int SNAP_D = 2 * 512;                  // halves: D as B operand, [kb2 2][lane 64][8]
constexpr int SNAP_HALVES = SNAP_S + SNAP_D;     // 6 KiB per (chunk, head, slice)
constexpr int KORD[4] = {0, 2, 1, 3};            // order in which a step consumes its Kh tiles (two independent accumulators)
constexpr int N_CHAIN = HV * 8;                  // chain workgroups
constexpr int PF_AHEAD = 16;                     // chunks between the L2 prefetch and the chain
constexpr int PF_SLOTS = 8;                      // prefetch loads in flight
constexpr int PUB_LAG = 8;                       // a chunk is published when at most this many newer chunks' stores are in flight
constexpr int FLAG_STRIDE = 64;                  // ints between progress words: every word has a 256-byte stretch of its own
constexpr int FLAG_WORDS = (N_CHAIN + 1) * FLAG_STRIDE;   // flag area at the head of `snap` (33 KiB): progress [128] | done count, error
constexpr int FLAG_DONE = N_CHAIN * FLAG_STRIDE, FLAG_ERR = FLAG_DONE + 1, FLAG_NEXT = FLAG_DONE + 2;   // FLAG_ERR: the status word; FLAG_NEXT: head of the item queue
constexpr int ERR_GAVE_UP = 1, ERR_NOT_FINITE = 2;
constexpr int FLAG_HALVES = FLAG_WORDS * 2;
constexpr int SPIN_LIMIT = 1 << 21;              // polls (about a second) before a consumer gives up
constexpr int MAX_OUT_WGS = 512;                 // output workgroups of the one-launch form: two for every CU (measured: 384 +2 us, 640 +4 us at 8192 tokens)
constexpr int FUSED_MIN_CHUNKS = 64;              // from 4096 tokens on the one-launch form wins (measured: 2048 tokens 37 / 35 us, 8192 134 / 155 us)
typedef unsigned long long u64;

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
// 16 bytes per lane as ONE device-scope store (a wavefront then writes eight whole 128-byte lines; the compiler's own
// device-scope stores are at most 8 bytes wide).  Counted by vmcnt like any other store.
__device__ __forceinline__ void store_coherent(_Float16* p, const half8& v) {
    const u32x4 q = __builtin_bit_cast(u32x4, v);
    // (the s_nop is the wait state this target wants between a store of more than 8 bytes and a write to its data registers;
    // the compiler inserts it for its own stores and cannot see into this one)
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(q) : "memory");
}
template <bool COHERENT>
__device__ __forceinline__ void store_snap(_Float16* p, const half8& v) {
    if (COHERENT) store_coherent(p, v);
    else *reinterpret_cast<half8*>(p) = v;
}
__device__ __forceinline__ half8 load_coherent(const _Float16* p) {
    ulonglong2 q;
    q.x = __hip_atomic_load(reinterpret_cast<const u64*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    q.y = __hip_atomic_load(reinterpret_cast<const u64*>(p) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return __builtin_bit_cast(half8, q);
}

template <bool COHERENT>
__device__ __forceinline__ half8 load_snap(const _Float16* p) {
    return COHERENT ? load_coherent(p) : *reinterpret_cast<const half8*>(p);
}

// the last workgroup of a one-launch phase B leaves the progress words, the done count and the queue head zero (not the status word)
__device__ __forceinline__ void clear_flags(int* flags, int tid, int nthreads) {
    for (int i = tid; i < N_CHAIN; i += nthreads) __hip_atomic_store(flags + i * FLAG_STRIDE, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0) {
        __hip_atomic_store(flags + FLAG_DONE, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(flags + FLAG_NEXT, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

struct ChainLds {
    __align__(16) _Float16 sb_x[SNAP_S];
    __align__(16) _Float16 db_x[SNAP_D];          // dec * D: the B operand of the state update
    __align__(16) _Float16 dn_x[SNAP_D];          // D itself: what the output workgroups need
};

// blk = (head, slice) index of this workgroup; wavefronts 0..3 compute, wavefront 4 writes snapshots and publishes progress
// PB_DEP = chunks of operands in flight per MFMA wavefront (4 in the two-launch form; 3 in the one-launch form, whose
// wavefronts share their SIMDs with output wavefronts and have 168 registers each)
template <bool PUBLISH, int PB_DEP>
__device__ __forceinline__ void chain_role(ChainLds& L, int blk, const _Float16* ops, const _Float16* U, const float* gates,
                                           const float* st_in, float* st_out, _Float16* snaps, int* flags, int NC) {
    // heads that share an XCD's L2 keep their 8 slices there: workgroup id = xcd + 8 k, head = xcd + 8 (k / 8), slice = k % 8
    const int xcd = blk & 7, kq = blk >> 3;
    const int h = xcd + 8 * (kq >> 3), sl = kq & 7;
    // (the wavefront number as a scalar: the roles are then separated by real branches, which the barriers inside them need)
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
    const half8* sbx = reinterpret_cast<const half8*>(L.sb_x) + lane;
    const half8* dbx = reinterpret_cast<const half8*>(L.db_x) + lane;
    const half8* dnx = reinterpret_cast<const half8*>(L.dn_x) + lane;

    if (w == 4) {
        _Float16* dst = snaps + ((size_t)h * 8 + sl) * SNAP_HALVES + lane * 8;
        const size_t cst = (size_t)HV * 8 * SNAP_HALVES;                        // halves per chunk
        int* flag = flags + (h * 8 + sl) * FLAG_STRIDE;
        for (int c = 0; c < NC; c++) {
            __builtin_amdgcn_s_barrier();                                       // E1: sb_x holds S_c^T
            asm volatile("" ::: "memory");
            const half8 a0 = sbx[0], a1 = sbx[64], a2 = sbx[128], a3 = sbx[192];
            store_snap<PUBLISH>(dst, a0);
            store_snap<PUBLISH>(dst + 512, a1);
            store_snap<PUBLISH>(dst + 1024, a2);
            store_snap<PUBLISH>(dst + 1536, a3);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();                                       // E2: dn_x holds D_c
            asm volatile("" ::: "memory");
            const half8 d0 = dnx[0], d1 = dnx[64];
            store_snap<PUBLISH>(dst + 2048, d0);
            store_snap<PUBLISH>(dst + 2560, d1);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            dst += cst;
            if (PUBLISH && c >= PUB_LAG) {                                      // 6 stores per chunk (+ one progress store per step)
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(7 * PUB_LAG) : "memory");
                if (lane == 0) __hip_atomic_store(flag, c - PUB_LAG + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (PUBLISH) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (lane == 0) __hip_atomic_store(flag, NC, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                    // the progress store is acknowledged before this workgroup counts as done
            int last = 0;
            if (lane == 0) last = atomicAdd(flags + FLAG_DONE, 1) == (int)gridDim.x - 1;
            if (__builtin_amdgcn_readfirstlane(last)) clear_flags(flags, lane, 64);
        }
        return;
    }
    if (w == 5) {
        // sixth wavefront: brings the operands of chunk c + PF_AHEAD into this XCD's L2 (this slice's eighth of the head's Wn
        // and Kh tiles, and its own U tiles: 48 lines of 128 bytes, one load per step, never waited for).  The operand FIFO
        // of the MFMA wavefronts covers a few steps; a load that goes to HBM while other workgroups stream takes longer.
        const char* wk = reinterpret_cast<const char*>(ops + (size_t)h * OP_HALVES);
        const char* up = reinterpret_cast<const char*>(U + (size_t)h * U_HALVES + (size_t)sl * NCT * 256);
        const size_t ostb = (size_t)HV * OP_HALVES * 2, ustb = (size_t)HV * U_HALVES * 2;
        // lanes 0..15: lines sl * 16 .. + 15 of the 128 lines of Wn; 16..31: the same of Kh; 32..47: the 16 lines of the U slice
        const int part = lane >> 4, li = lane & 15;
        const size_t off = part == 0 ? (size_t)OP_W * 2 + (sl * 16 + li) * 128 : (size_t)OP_K * 2 + (sl * 16 + li) * 128;
        // PF_SLOTS loads in flight, each into a register of its own that is read (an empty asm) before it is loaded again, one
        // round later: the compiler counts the loads, and the wait it puts before that read names a load of many steps ago
        unsigned pf[PF_SLOTS];
#pragma unroll
        for (int j = 0; j < PF_SLOTS; j++) pf[j] = 0;
        for (int c0 = 0; c0 < NC; c0 += PF_SLOTS) {
#pragma unroll
            for (int j = 0; j < PF_SLOTS; j++) {
                const int c = c0 + j;
                if (c < NC) {                                                   // uniform: every wavefront meets 2 NC barriers
                    __builtin_amdgcn_s_barrier();
                    const int cp = c + PF_AHEAD;
                    asm volatile("" ::"v"(pf[j]));
                    if (cp < NC && lane < 48) {
                        const char* a = part < 2 ? wk + cp * ostb + off : up + cp * ustb + li * 128;
                        pf[j] = *reinterpret_cast<const unsigned*>(a);
                    }
                    __builtin_amdgcn_s_barrier();
                }
            }
        }
#pragma unroll
        for (int j = 0; j < PF_SLOTS; j++) asm volatile("" ::"v"(pf[j]));
        return;
    }
    if (w > 5) return;

    f32x4 ST[2];
    {
        const float* sp = st_in + ((size_t)h * DV + sl * 16 + n) * DK + w * 32 + 4 * g;   // S[h][dv][dk], dk contiguous
        ST[0] = *reinterpret_cast<const f32x4*>(sp);
        ST[1] = *reinterpret_cast<const f32x4*>(sp + 16);
    }
    const half8* opb = reinterpret_cast<const half8*>(ops + (size_t)h * OP_HALVES) + lane;
    const half4* upb = reinterpret_cast<const half4*>(U + (size_t)h * U_HALVES + (size_t)(sl * NCT + w) * 256) + lane;
    const float* gpb = gates + (size_t)h * GATE_FLOATS;
    const size_t ost = (size_t)HV * OP_HALVES / 8, ust = (size_t)HV * U_HALVES / 4, gst = (size_t)HV * GATE_FLOATS;
    const int wq = (OP_W / 8) + w * 4 * 64, kq0 = (OP_K / 8) + w * 4 * 64;       // W[ct = w][kb], Kh[mt = 2w + i][kb2]
    const int dq = G_DEC + 16 * w + 4 * g;                                       // dec of this lane's four rows of D

    half8 Wt[PB_DEP][4], Kt[PB_DEP][4];
    half4 Ut[PB_DEP];
    f32x4 dect[PB_DEP];
    float gct[PB_DEP];                       // the chunk's decay rides in the FIFO as one more (lane-uniform) vector load
#pragma unroll
    for (int j = 0; j < PB_DEP; j++) {                                          // same issue order as inside the steps
        const int cc = min(j, NC - 1);
#pragma unroll
        for (int i = 0; i < 4; i++) Wt[j][i] = opb[cc * ost + wq + i * 64];
        Ut[j] = upb[cc * ust];
        dect[j] = *reinterpret_cast<const f32x4*>(gpb + cc * gst + dq);
#pragma unroll
        for (int i = 0; i < 4; i++) Kt[j][KORD[i]] = opb[cc * ost + kq0 + KORD[i] * 64];
        gct[j] = gpb[cc * gst + G_GC];
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
        reinterpret_cast<half8*>(L.sb_x)[w * 64 + lane] = pack_half8(ST[0], ST[1]);
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
        const f32x4 Uf = {(float)Ut[j][0], (float)Ut[j][1], (float)Ut[j][2], (float)Ut[j][3]};
        const f32x4 D = (D0 + D1) + Uf;
        Ut[j] = upb[cn * ust];
        __builtin_amdgcn_sched_barrier(0);
        const f32x4 Dd = D * dect[j];
        dect[j] = *reinterpret_cast<const f32x4*>(gpb + cn * gst + dq);
        __builtin_amdgcn_sched_barrier(0);
        half4 dh, ddh;
        dh[0] = (_Float16)D[0]; dh[1] = (_Float16)D[1]; dh[2] = (_Float16)D[2]; dh[3] = (_Float16)D[3];
        ddh[0] = (_Float16)Dd[0]; ddh[1] = (_Float16)Dd[1]; ddh[2] = (_Float16)Dd[2]; ddh[3] = (_Float16)Dd[3];
        // B-operand layout of D: k-block w / 2, halves 4 (w & 1) .. + 3 of the lane's eight
        reinterpret_cast<half4*>(L.db_x)[((w >> 1) * 64 + lane) * 2 + (w & 1)] = ddh;
        reinterpret_cast<half4*>(L.dn_x)[((w >> 1) * 64 + lane) * 2 + (w & 1)] = dh;
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
        gct[j] = gpb[cn * gst + G_GC];
        __builtin_amdgcn_sched_barrier(0);
    };
    int c = 0;
    if constexpr (PB_DEP == 4) {
        for (; c + 4 <= NC; c += 4) {
            step(std::integral_constant<int, 0>{}, c);
            step(std::integral_constant<int, 1>{}, c + 1);
            step(std::integral_constant<int, 2>{}, c + 2);
            step(std::integral_constant<int, 3>{}, c + 3);
        }
        if (c < NC) step(std::integral_constant<int, 0>{}, c);
        if (c + 1 < NC) step(std::integral_constant<int, 1>{}, c + 1);
        if (c + 2 < NC) step(std::integral_constant<int, 2>{}, c + 2);
    } else {
        static_assert(PB_DEP == 3 || PB_DEP == 4, "the chain loop is unrolled by hand");
        for (; c + 3 <= NC; c += 3) {
            step(std::integral_constant<int, 0>{}, c);
            step(std::integral_constant<int, 1>{}, c + 1);
            step(std::integral_constant<int, 2>{}, c + 2);
        }
        if (c < NC) step(std::integral_constant<int, 0>{}, c);
        if (c + 1 < NC) step(std::integral_constant<int, 1>{}, c + 1);
    }
    {
        float* sp = st_out + ((size_t)h * DV + sl * 16 + n) * DK + w * 32 + 4 * g;
        *reinterpret_cast<f32x4*>(sp) = ST[0];
        *reinterpret_cast<f32x4*>(sp + 16) = ST[1];
        // an overflow of a half-precision operand anywhere in the chain (state, D, U, conv outputs) ends here as inf or NaN
        bool bad = false;
#pragma unroll
        for (int i = 0; i < 4; i++) bad |= !(fabsf(ST[0][i]) <= 3.0e38f) | !(fabsf(ST[1][i]) <= 3.0e38f);
        if (__any(bad) && lane == 0) atomicOr(flags + FLAG_ERR, ERR_NOT_FINITE);
    }
}

// gated_out (qt_common.h) with its exact path as a called function: inlined 32 times, that path (an IEEE division and a
// double-precision exponential) is most of the norm's code, and every wavefront runs it a few times per tile.  The
// instruction cache is shared by two CUs: a chain workgroup's three-step loop has to stay in it while its neighbour's
// output workgroups run this code.
__device__ __attribute__((noinline)) float gated_out_exact(float z, float n) { return __fdiv_rn(z, 1.0f + exp32(-z)) * n; }
__device__ __forceinline__ bf16_t gated_out_small(float z, float n) {
    float o;
    if (__builtin_expect(!gated_out_fast(z, n, o), 0)) o = gated_out_exact(z, n);
    return f2bf(o);
}

// The gated RMSNorm of one 64 x 128 output tile in LDS.
constexpr int YS_LD = DV + 8;
typedef const __attribute__((address_space(3))) bf16_t* lds_bf16_ptr;
// a load of data that nothing reads again.  In the one-launch form (STREAM) it is marked nontemporal: there the output
// workgroups stream beside the chain, whose operands wait in the L2 for their step, and must not push them out.  In the
// two-launch form the same mark costs time (the records are still in the L2 from the kernel that wrote them).
template <bool STREAM, typename T>
__device__ __forceinline__ T load_once(const T* p) {
    return STREAM ? __builtin_nontemporal_load(p) : *p;
}
template <bool STREAM>
__device__ __forceinline__ void gated_norm_tile(lds_bf16_ptr ys, int tid, int c, int h, bf16_t* __restrict__ y,
                                                           const bf16_t* __restrict__ proj, const float* __restrict__ gw, float eps, int S) {
    const int cc = tid & 15;
    float gwv[8];
#pragma unroll
    for (int j = 0; j < 8; j++) gwv[j] = gw[cc * 8 + j];
    // the four rows of this 16-lane group: all sums of squares first, then one reciprocal square root per lane
    uint4 yv4[4];
    float ss4[4], inv4[4];
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int row = it * 16 + (tid >> 4);
        const u32x4 yw = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(&ys[row * YS_LD + cc * 8]);
        yv4[it] = make_uint4(yw[0], yw[1], yw[2], yw[3]);
        float yy[8];
        unpack8(yv4[it], yy);
        double ss = 0.0;
#pragma unroll
        for (int j = 0; j < 4; j++) ss += (double)yy[2 * j] * yy[2 * j] + (double)yy[2 * j + 1] * yy[2 * j + 1];
        ss4[it] = (float)row16_sum_d(ss);
    }
    // every z row is requested before the first result is stored: a wavefront's loads and stores share one counter, so a load
    // issued behind a store is waited for together with it, and a store takes microseconds to complete
    uint4 zv4[4];
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int t = min(c * C + it * 16 + (tid >> 4), S - 1);
        const u32x4 zw = load_once<STREAM>(reinterpret_cast<const u32x4*>(proj + (size_t)t * PW + CD + h * DV) + cc);
        zv4[it] = make_uint4(zw[0], zw[1], zw[2], zw[3]);
    }
    rsqrt_rows<4>(ss4, eps, inv4, cc);
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int row = it * 16 + (tid >> 4);
        const int t = c * C + row;
        if (t >= S) continue;                                       // whole 16-lane groups leave together
        float yy[8], zz[8];
        unpack8(yv4[it], yy);
        unpack8(zv4[it], zz);
        uint32_t o[8];
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] = gated_out_small(zz[j], gwv[j] * (yy[j] * inv4[it]));
        const u32x4 ov = {o[0] | (o[1] << 16), o[2] | (o[3] << 16), o[4] | (o[5] << 16), o[6] | (o[7] << 16)};
        __builtin_nontemporal_store(ov, reinterpret_cast<u32x4*>(y + ((size_t)t * HV + h) * DV) + cc);   // written once, read by a later kernel
    }
}

// Output role: Y_c = gamma_c * (Qh_c S_c^T) + Am_c D_c for one (chunk, head) by 4 wavefronts; wavefront w covers the dv slices 2w
// and 2w+1.  The 64 x 128 tile goes through LDS as bf16 and leaves either as y [S,16,128] or, with NORM, straight through the
// gated RMSNorm (same arithmetic as the stand-alone kernel: 16 lanes per row, 8 columns each; batch.py:338-343).
// With WAIT the item's snapshots come from a chain that runs in the same launch: `seq` counts the items of this workgroup.
template <bool NORM, bool WAIT>
__device__ __forceinline__ void output_item(bf16_t* ys, volatile int* ready, int seq, int spin_limit, int c, int h, const _Float16* __restrict__ ops,
                                            const _Float16* snaps, int* flags, const float* __restrict__ gates,
                                            bf16_t* __restrict__ y, const bf16_t* __restrict__ proj, const float* __restrict__ gw,
                                            float eps, int S) {
    const int tid = threadIdx.x & 255, w = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    {
        constexpr bool active = true;
        {
            const size_t rec = (size_t)c * HV + h;
            const half8* op = reinterpret_cast<const half8*>(ops + rec * OP_HALVES) + lane;
            half8 Sb[2][4], Db[2][2], Qt[16], At[8];
            // what does not depend on the chain is requested before the wait
#pragma unroll
            for (int i = 0; i < 16; i++) Qt[i] = load_once<WAIT>(&op[(OP_Q / 8) + i * 64]);
#pragma unroll
            for (int i = 0; i < 8; i++) At[i] = load_once<WAIT>(&op[(OP_A / 8) + i * 64]);
            float gam[NCT];                                                     // gamma of this lane's token of every row tile
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) gam[ct] = gates[rec * GATE_FLOATS + G_GAM + 16 * ct + n];
            // wait until the chain has published chunk c for all eight slices of the head: the unit's first wavefront polls (lanes
            // 0..7, one progress word each, about once a microsecond: thousands of pollers on one memory line would hold up the
            // chain's own progress stores) and passes the news on through LDS, where the other three wavefronts wait
            // `ready` = 2 * (items this workgroup has been let into) + (1 if the last one was given up)
            if (!WAIT) {
            } else if (w == 0) {
                const int* fp = flags + (h * 8 + (lane & 7)) * FLAG_STRIDE;
                int spins = 0;
                bool gave_up = false;
                while (true) {
                    int v = c + 1;
                    if (lane < 8) v = __hip_atomic_load(fp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    asm volatile("" ::: "memory");                              // the snapshot loads stay behind the poll
                    if (__all(v > c)) break;
                    if (++spins > spin_limit) {
                        gave_up = true;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(32);
                }
                if (lane == 0) {
                    if (gave_up) atomicOr(flags + FLAG_ERR, ERR_GAVE_UP);
                    *ready = 2 * (seq + 1) + (gave_up ? 1 : 0);
                }
                if (gave_up) return;                                            // (all four wavefronts leave here: no barrier is skipped by some only)
            } else {
                int rv;
                while (((rv = *ready) >> 1) <= seq) __builtin_amdgcn_s_sleep(2);
                asm volatile("" ::: "memory");
                if (rv & 1) return;                                             // given up: the item's rows stay unwritten
            }
            const _Float16* sp = snaps + (rec * 8 + 2 * w) * SNAP_HALVES + lane * 8;
#pragma unroll
            for (int s = 0; s < 2; s++) {
#pragma unroll
                for (int kb = 0; kb < 4; kb++) Sb[s][kb] = load_snap<WAIT>(sp + s * SNAP_HALVES + kb * 512);
#pragma unroll
                for (int kb2 = 0; kb2 < 2; kb2++) Db[s][kb2] = load_snap<WAIT>(sp + s * SNAP_HALVES + SNAP_S + kb2 * 512);
            }
#pragma unroll
            for (int s = 0; s < 2; s++) {
                // the products are taken transposed (the snapshot as the A operand, the Qh / Am tile as the B operand: the same
                // registers either way), so that a lane holds four consecutive columns of one token: Y[ct][r] = y[token 16 ct + n][dv
                // 16 (2 w + s) + 4 g + r], eight bytes of a row of the LDS tile
                f32x4 Y[NCT];
#pragma unroll
                for (int ct = 0; ct < NCT; ct++) Y[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kb = 0; kb < 4; kb++)
#pragma unroll
                    for (int ct = 0; ct < NCT; ct++) Y[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Sb[s][kb], Qt[ct * 4 + kb], Y[ct], 0, 0, 0);
#pragma unroll
                for (int ct = 0; ct < NCT; ct++) Y[ct] *= gam[ct];
#pragma unroll
                for (int kb2 = 0; kb2 < 2; kb2++)
#pragma unroll
                    for (int ct = 0; ct < NCT; ct++) Y[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Db[s][kb2], At[ct * 2 + kb2], Y[ct], 0, 0, 0);
#pragma unroll
                for (int ct = 0; ct < NCT; ct++)
                    *reinterpret_cast<uint2*>(&ys[(ct * 16 + n) * YS_LD + (2 * w + s) * 16 + 4 * g]) =
                        make_uint2(pack2_bf(Y[ct][0], Y[ct][1]), pack2_bf(Y[ct][2], Y[ct][3]));
            }
        }
        __syncthreads();
        if (active) {
            if (!NORM) {
                const int row = tid >> 2, q4 = tid & 3;
                const int t = c * C + row;
                if (t < S) {
                    const uint4* src = reinterpret_cast<const uint4*>(&ys[row * YS_LD + q4 * 32]);
                    uint4* dst = reinterpret_cast<uint4*>(y + ((size_t)t * HV + h) * DV + q4 * 32);
#pragma unroll
                    for (int i = 0; i < 4; i++) dst[i] = src[i];
                }
            } else {
                gated_norm_tile<WAIT>((lds_bf16_ptr)ys, tid, c, h, y, proj, gw, eps, S);
            }
        }
        __syncthreads();                                                        // ys is reused by the next round
    }
}

// the two-launch form: 128 chain workgroups of 320 threads, then one output workgroup of 256 threads per (chunk, head)
__global__ __launch_bounds__(384) void gdn_chain_kernel(const _Float16* ops, const _Float16* U, const float* gates, const float* st_in,
                                                        float* st_out, _Float16* snap, int NC) {
    __shared__ ChainLds chain_lds;
    chain_role<false, 4>(chain_lds, blockIdx.x, ops, U, gates, st_in, st_out, snap + FLAG_HALVES, reinterpret_cast<int*>(snap), NC);
}
template <bool NORM>
__global__ __launch_bounds__(256) void gdn_output_kernel(const _Float16* __restrict__ ops, const _Float16* __restrict__ snap,
                                                         const float* __restrict__ gates, bf16_t* __restrict__ y,
                                                         const bf16_t* __restrict__ proj, const float* __restrict__ gw, float eps,
                                                         int S, int NC) {
    __shared__ __align__(16) bf16_t ys[C * YS_LD];
    output_item<NORM, false>(ys, nullptr, 0, 0, blockIdx.x / HV, blockIdx.x % HV, ops, snap + FLAG_HALVES, nullptr, gates, y, proj, gw, eps, S);
}

// the one-launch form: N_CHAIN chain workgroups, then output workgroups (4 wavefronts at work) that take (chunk, head) items
// from a queue in chunk order.  384 threads and at most 168 registers, i.e. three wavefronts per SIMD.  Measured placement
// (hardware ids recorded by every workgroup): a CU with a chain workgroup (two wavefronts on two of its SIMDs) takes no output
// workgroup, whose six wavefronts would need the same SIMDs when it starts; every other CU holds two.  So 256 output
// workgroups run beside the chain and the rest start as chain workgroups end, on the items still in the queue.  The chain
// workgroups have the lowest indices, so they are resident before any output workgroup starts, and they wait for nothing:
// an output workgroup's wait for its item always ends.
template <bool NORM>
__global__ __launch_bounds__(384, 3) void gdn_phase_b_kernel(const _Float16* ops, const _Float16* U, const float* gates, const float* st_in,
                                                             float* st_out, _Float16* snap, bf16_t* y, const bf16_t* proj,
                                                             const float* gw, float eps, int S, int NC, int spin_limit) {
    __shared__ ChainLds chain_lds;
    __shared__ __align__(16) bf16_t ys[C * YS_LD];
    __shared__ int ready, item_s, last;
    int* flags = reinterpret_cast<int*>(snap);
    _Float16* snaps = snap + FLAG_HALVES;
    if (blockIdx.x < N_CHAIN) {
        chain_role<true, 3>(chain_lds, blockIdx.x, ops, U, gates, st_in, st_out, snaps, flags, NC);
        return;
    }
    if (threadIdx.x >= 256) return;                                             // (a wavefront that has ended is no party to the barriers)
    if (threadIdx.x == 0) ready = 0;
    const int total = NC * HV;
    for (int seq = 0;; seq++) {
        if (threadIdx.x == 0) item_s = atomicAdd(flags + FLAG_NEXT, 1);
        __syncthreads();
        const int item = item_s;
        if (item >= total) break;
        output_item<NORM, true>(ys, &ready, seq, spin_limit, item / HV, item % HV, ops, snaps, flags, gates, y, proj, gw, eps, S);
    }
    // a workgroup counts itself done when it has taken its last item; the last workgroup of the launch (of either role)
    // leaves the flag area zero for the next launch
    if (threadIdx.x == 0) last = atomicAdd(flags + FLAG_DONE, 1) == (int)gridDim.x - 1;
    __syncthreads();
    if (last) clear_flags(flags, threadIdx.x, 256);
}

// ------------------------------------------------------------------------------------------------------------------
// Phase A: one workgroup of 512 threads per (chunk, head), two workgroups per CU.
//
// A (chunk, head) costs about 10^5 vector-ALU instructions of conv + SiLU + normalisation and a chain of dependent matrix
// steps (K K^T, the 64 x 64 triangular inverse, the products with it) that keeps no unit busy.  The two run side by side:
// wavefronts 0..3 (group M) convolve k, then walk the matrix chain while wavefronts 4..7 (group V) convolve q and v and
// form A = lower(G * Q K^T).  One workgroup barrier (table, taps and gates ready); after it a consumer of k, q or v waits for
// that part's four producers through a counter in LDS.
//
// q, k and v are converted to half precision ONCE, when they are staged into LDS, and every MFMA operand is then a plain
// LDS read: row-major 16-byte reads for K K^T and Q K^T, the transposing load ds_read_b64_tr_b16 where the contraction runs
// over the tokens (K^T for Wn and Kh, V for U).  The per-token factors gamma and dec never touch an operand element:
// gamma goes into Tb's columns for Wn, and the chain / output kernels apply dec and gamma to accumulator rows.
//
// The inverse T = (I + L)^-1, L = strict_lower(beta_i G_ij k_i . k_j), is exact fp32 work by blocks of 16 and stays inside
// one wavefront per block ROW I: with LT = L^T and TT = T^T, column I of TT follows from (I + LT) TT = I as
//     TT[I][I] = T_II^T,     TT[w][I] = -T_ww^T  sum_{J = w+1..I} LT[w][J] TT[J][I]        (w = I-1 .. 0).
// In the accumulator layout (lane (n, g) holds rows 4g..4g+3 of column n) a block of TT is at once the B operand of the next
// step and, read as a block of T, the A-operand layout (row n, columns 4g..4g+3) the products with T need; LT[w][J] as an
// A operand is the accumulator layout of K_J K_w^T.  So no block of L or T goes through LDS except the four diagonal ones:
// every wavefront of group M forms all four (lane group g inverts block g by forward substitution, column n per lane), and
// writes them to the same LDS words (identical values; a wavefront reads back only after its own writes).
// ------------------------------------------------------------------------------------------------------------------
typedef short s16x4 __attribute__((ext_vector_type(4)));

constexpr int QS_LD = DK + 8;        // row stride (halves) of Qs / Ks: 16-byte row reads of 16 rows hit distinct banks
constexpr int VS_LD = DV + 16;       // row stride of Vs: the transposing loads (4 rows x 32 bytes per 16 lanes) hit distinct banks
constexpr int ND_LD = 20;            // row stride (floats) of a diagonal block
constexpr int ND_BLK = 16 * ND_LD + 4;   // floats between diagonal blocks: the four lane groups read distinct banks
constexpr float LOG2E = 1.4426950408889634f;

struct PhaseALds {                       // 73 KiB: two workgroups per CU
    __align__(16) _Float16 Ks[C * QS_LD];
    __align__(16) _Float16 Qs[C * QS_LD];
    __align__(16) _Float16 Vs[C * VS_LD];
    __align__(16) bf16_t tab[SILU_TAB_SIZE];     // fused conv only: the silu_bf16 table and this head's conv taps
    __align__(16) bf16_t taps[3 * DK * 4];
    __align__(16) float Td[4 * ND_BLK];          // their inverses: [block][column][row]
    float Lc2[C], beta[C], gam[C], dec[C];       // Lc2 = log2(e) * cumsum(log g)
    int staged[4];                               // wavefronts that have staged their part of k, q, v (PA_K, PA_Q, PA_V)
};
constexpr int PA_K = 0, PA_Q = 1, PA_V = 2;

// A wavefront announces that its LDS stores of a part are done; a consumer waits until all four producers have.  (The parts
// are produced and consumed by different wavefronts at different times: a workgroup barrier would hold up seven wavefronts
// for the slowest one three times per chunk.)
__device__ __forceinline__ void part_staged(PhaseALds& L, int part, int lane) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    if (lane == 0) __hip_atomic_fetch_add(&L.staged[part], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void await_part(PhaseALds& L, int part) {
    while (__hip_atomic_load(&L.staged[part], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < 4) __builtin_amdgcn_s_sleep(1);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

__device__ __forceinline__ half8 to_half8(const float (&v)[8]) {
    half8 h;
#pragma unroll
    for (int j = 0; j < 8; j++) h[j] = (_Float16)v[j];
    return h;
}
__device__ __forceinline__ half8 bf8_to_half8(const uint4& w) {      // exact for |x| >= 2^-14 (bf16 carries 8 significant bits)
    float f[8];
    unpack8(w, f);
    return to_half8(f);
}
// transposing LDS load: within a group of 16 lanes, lane 4 q + i receives element i of the 8-byte chunks addressed by lanes
// q, q + 4, q + 8, q + 12.  With lane n of group g pointing at (row r0 + n / 4, columns c0 + 4 (n % 4) .. + 3), lane n receives
// rows r0 .. r0 + 3 of column c0 + n.
__device__ __forceinline__ half4 lds_tr4(const _Float16* p) {
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(const_cast<_Float16*>(p)));
    return __builtin_bit_cast(half4, v);
}
// MFMA operand whose contraction index runs over the chunk's tokens, from a row-major [token][ld] tile: lane (n, g) gets
// column c0 + n of tokens kperm(kb2, g, 0..7) = 32 kb2 + 4 g + {0..3}, 32 kb2 + 16 + 4 g + {0..3}.
__device__ __forceinline__ half8 tokens_operand(const _Float16* base, int ld, int kb2, int c0, int n, int g) {
    const _Float16* p = base + (32 * kb2 + 4 * g + (n >> 2)) * ld + c0 + 4 * (n & 3);
    const half4 lo = lds_tr4(p), hi = lds_tr4(p + 16 * ld);
    half8 r;
    r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
    r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
    return r;
}
// K_I K_J^T for two 16-row blocks of Ks, accumulator layout: lane (n, g) gets k_{16 I + 4 g + r} . k_{16 J + n}
__device__ __forceinline__ f32x4 kk_block(const _Float16* Ks, int I, int J, int n, int g) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kb = 0; kb < 4; kb++) {
        const half8 a = *reinterpret_cast<const half8*>(&Ks[(16 * I + n) * QS_LD + 32 * kb + 8 * g]);
        const half8 b = *reinterpret_cast<const half8*>(&Ks[(16 * J + n) * QS_LD + 32 * kb + 8 * g]);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc, 0, 0, 0);
    }
    return acc;
}

// v_permlane32_swap: lanes 32..63 of x change places with lanes 0..31 of y; v_permlane16_swap: the odd 16-lane rows of x with
// the even rows of y
__device__ __forceinline__ void lanes32_swap(float& x, float& y) {
    const auto t = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(y), false, false);
    x = __uint_as_float(t[0]);
    y = __uint_as_float(t[1]);
}
__device__ __forceinline__ void lanes16_swap(float& x, float& y) {
    const auto t = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(y), false, false);
    x = __uint_as_float(t[0]);
    y = __uint_as_float(t[1]);
}
// steps M.. of the forward substitution: a[i] += (lane M's R value of row i) * a[M] for every row i > M
template <int M>
__device__ __forceinline__ void substitute_columns(const float (&R)[4][4], float (&a)[16]) {
    if constexpr (M < 15) {
#pragma unroll
        for (int i = M + 1; i < 16; i++) a[i] = __builtin_fmaf(row16_bcast<M>(R[i >> 2][i & 3]), a[M], a[i]);
        substitute_columns<M + 1>(R, a);
    }
}

// The matrix chain of block row I (one wavefront of group M; I is the same for the whole wavefront, so every test of it is a
// scalar branch): returns Tb = T diag(beta) for rows 16 I + n as the two operand forms of the products,
// tbU[kb2] = Tb[16 I + n][kperm(kb2, g, 0..7)] and tbW = the same with columns scaled by -gamma.
__device__ __forceinline__ void inverse_row(PhaseALds& L, const int I, int n, int g, half8 (&tbU)[2], half8 (&tbW)[2]) {
    // diagonal blocks of L, negated (all four, in every wavefront): R[b][r] = -L[16 b + 4 g + r][16 b + n]
    float R[4][4];
#pragma unroll
    for (int b = 0; b < 4; b++) {
        const f32x4 acc = kk_block(L.Ks, b, b, n, g);
        const f32x4 lci = *reinterpret_cast<const f32x4*>(&L.Lc2[16 * b + 4 * g]);
        const f32x4 bei = *reinterpret_cast<const f32x4*>(&L.beta[16 * b + 4 * g]);
        const float lcj = L.Lc2[16 * b + n];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float v = bei[r] * __builtin_amdgcn_exp2f(lci[r] - lcj) * acc[r];
            R[b][r] = (4 * g + r > n) ? -v : 0.f;
        }
    }
    // 4 x 4 transpose over (register b, lane group g) with the VALU lane swaps: afterwards lane (n, g) holds column n of its own
    // block g, R[j][r] = -L[16 g + 4 j + r][16 g + n]
#pragma unroll
    for (int r = 0; r < 4; r++) {
        lanes32_swap(R[0][r], R[2][r]);
        lanes32_swap(R[1][r], R[3][r]);
        lanes16_swap(R[0][r], R[1][r]);
        lanes16_swap(R[2][r], R[3][r]);
    }
    // lane (n, g): column n of the inverse of diagonal block g, by forward substitution in registers.  Column by column: once
    // x[m] is known every later row takes its term -L[i][m] x[m] (the factor is lane m's value, broadcast over the 16 lanes),
    // so one multiply-add per step is on the dependent path; the terms of a row are still added in ascending m.  The
    // multiply-adds are written as fused ones: both input forms of the kernel then round alike.
    {
        float a[16];
#pragma unroll
        for (int i = 0; i < 16; i++) a[i] = (i == n) ? 1.f : 0.f;
        substitute_columns<0>(R, a);
        float* tb = &L.Td[g * ND_BLK + n * ND_LD];
#pragma unroll
        for (int i = 0; i < 16; i += 4) *reinterpret_cast<f32x4*>(tb + i) = f32x4{a[i], a[i + 1], a[i + 2], a[i + 3]};
    }
    __builtin_amdgcn_sched_barrier(0);
    // blocks of L below the diagonal that this row's recursion multiplies with: LB[J (J - 1) / 2 + w] = block (J, w), w < J <= I
    f32x4 LB[6];
#pragma unroll
    for (int J = 1; J < 4; J++) {
        if (J <= I) {
            const f32x4 lci = *reinterpret_cast<const f32x4*>(&L.Lc2[16 * J + 4 * g]);
            const f32x4 bei = *reinterpret_cast<const f32x4*>(&L.beta[16 * J + 4 * g]);
#pragma unroll
            for (int w = 0; w < J; w++) {
                const f32x4 acc = kk_block(L.Ks, J, w, n, g);
                const float lcj = L.Lc2[16 * w + n];
#pragma unroll
                for (int r = 0; r < 4; r++) LB[J * (J - 1) / 2 + w][r] = bei[r] * __builtin_amdgcn_exp2f(lci[r] - lcj) * acc[r];
            }
        }
    }
    // column I of TT, upwards
    f32x4 TT[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        TT[k] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (k == I) {
#pragma unroll
            for (int r = 0; r < 4; r++) TT[k][r] = L.Td[k * ND_BLK + (4 * g + r) * ND_LD + n];     // T_II[n][4 g + r]
        }
    }
#pragma unroll
    for (int w = 2; w >= 0; w--) {
        if (w < I) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int J = 3; J > w; J--) {                                // the block found last, TT[w + 1], enters last
                if (J <= I) {
#pragma unroll
                    for (int kk = 0; kk < 4; kk++)
                        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(LB[J * (J - 1) / 2 + w][kk], TT[J][kk], acc, 0, 0, 0);
                }
            }
            const f32x4 d4 = *reinterpret_cast<const f32x4*>(&L.Td[w * ND_BLK + n * ND_LD + 4 * g]);   // T_ww[4 g + kk][n]
            f32x4 res = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < 4; kk++) res = __builtin_amdgcn_mfma_f32_16x16x4f32(d4[kk], acc[kk], res, 0, 0, 0);
            TT[w] = -res;
        }
    }
    // TT[w][r] = T[16 I + n][16 w + 4 g + r] (zero for w > I)
#pragma unroll
    for (int kb2 = 0; kb2 < 2; kb2++) {
        float u[8], v[8];
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            const int blk = 2 * kb2 + hf, cp = 16 * blk + 4 * g;
            const f32x4 b4 = *reinterpret_cast<const f32x4*>(&L.beta[cp]);
            const f32x4 g4 = *reinterpret_cast<const f32x4*>(&L.gam[cp]);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                u[4 * hf + r] = TT[blk][r] * b4[r];
                v[4 * hf + r] = -u[4 * hf + r] * g4[r];
            }
        }
        tbU[kb2] = to_half8(u);
        tbW[kb2] = to_half8(v);
    }
}

// Phase A of one (chunk, head).  from_proj = false: q, k, v [S,16,128] bf16 are inputs (convolved, normalized: conv_prep's
// outputs).  from_proj = true: they are computed here from the projection rows (conv4 + SiLU + q/k norm with the arithmetic of
// conv_prep_kernel, bit for bit; qwen35/prefill.py:96-134) and, with write_qkv, also stored; the workgroups of the last chunk
// write the new conv window (the last three input rows, prefill.py:262-263) to conv_out if it is given.
// proj [S,8224] supplies the gate inputs a, b in both forms.  The two forms give the same bits: after the staging of q, k, v
// every floating-point step is a single instruction chosen in the source (MFMA, multiplication, fused multiply-add), so the
// compiler has nothing to contract differently in the two instances.
template <bool from_proj>
__global__ __launch_bounds__(512, 4) void gdn_phase_a_kernel(const bool write_qkv,
                                                          const bf16_t* __restrict__ proj, bf16_t* qi, bf16_t* ki, bf16_t* vi,
                                                          const bf16_t* __restrict__ cs, const bf16_t* __restrict__ cw,
                                                          const bf16_t* __restrict__ silu_tab, bf16_t* __restrict__ conv_out,
                                                          const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                                                          _Float16* __restrict__ ops, _Float16* __restrict__ U,
                                                          float* __restrict__ gates, int S) {
    __shared__ PhaseALds L;
    const int c = blockIdx.x / HV, h = blockIdx.x % HV, t0 = c * C;
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 15, g = lane >> 4;
    // (the wavefront number as a scalar: the branches on it are then real branches, which the barriers inside them need)
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool grpV = wv >= 4;                          // wavefronts 4..7
    const int w = wv & 3;                               // wavefront within its group
    const int gi = (tid & 255) >> 4, cc = tid & 15;     // conv: tokens 4 gi .. 4 gi + 3, channels 8 cc .. 8 cc + 7 of a part
    const size_t rec = (size_t)c * HV + h;
    _Float16* op = ops + rec * OP_HALVES;
    bf16_t* const outA = grpV ? qi : ki;                // group M convolves k, group V q and then v
    const int partA = grpV ? 0 : 1;

    // ---- the chunk's rows: every load is issued before anything else; rows past the end are zero (gdn_nax.py:172-174)
    // one register array per part for both forms.  !from_proj: rw[rr] = token rr * 16 + gi, a lane 8 consecutive columns;
    // from_proj: rw[d] = input row 4 gi - 3 + d of 8 channels of the part
    uint4 rwA[7], rwB[7];
    // (wavefront 0 asks for its gate inputs first: loads return in order, so the gates are computed while the rows are in flight)
    bf16_t ga_raw = 0, gb_raw = 0;
    if (wv == 0 && t0 + lane < S) {
        ga_raw = proj[(size_t)(t0 + lane) * PW + CD + KD + HV + h];
        gb_raw = proj[(size_t)(t0 + lane) * PW + CD + KD + h];
    }
    if (!from_proj) {
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            const int t = t0 + rr * 16 + gi;
            const size_t o = ((size_t)min(t, S - 1) * HV + h) * DK + cc * 8;
            rwA[rr] = *reinterpret_cast<const uint4*>(outA + o);
            if (t >= S) rwA[rr] = make_uint4(0, 0, 0, 0);
        }
    } else {
        const int chA = partA * KD + h * DK + cc * 8;
#pragma unroll
        for (int d = 0; d < 7; d++) {
            const int tt = min(t0 + 4 * gi - 3 + d, S - 1);
            rwA[d] = *reinterpret_cast<const uint4*>(tt < 0 ? cs + (tt + 3) * CD + chA : proj + (size_t)tt * PW + chA);
        }
        // the head's conv taps (3 x 128 channels x 4 taps) go through LDS: every token group needs the same 3 KiB
        if (wv >= 5) {
            const int i3 = tid - 320, part = i3 >> 6, i = i3 & 63;
            reinterpret_cast<uint4*>(L.taps)[i3] = reinterpret_cast<const uint4*>(cw + (size_t)(part * KD + h * DK) * 4)[i];
        }
        if (conv_out && c == (S - 1) / C && tid >= 64 && tid < 64 + 3 * 48) {   // new conv window: input rows S-3 .. S-1 of this head's channels
            const int i3 = tid - 64;
            const int r = i3 / 48, part = (i3 % 48) >> 4, ch0 = part * KD + h * DK + (i3 & 15) * 8, tt = S - 3 + r;
            *reinterpret_cast<uint4*>(conv_out + r * CD + ch0) =
                *reinterpret_cast<const uint4*>(tt < 0 ? cs + (tt + 3) * CD + ch0 : proj + (size_t)tt * PW + ch0);
        }
    }

    // ---- gates of the chunk's tokens (gdn_nax.py:80-104): wavefront 0, one token per lane
    if (wv == 0) {
        const int t = t0 + lane;
        float lg = 0.f, be = 0.f;
        if (t < S) {
            lg = log_decay(A_log[h], BF(bf2f(ga_raw) + dt_bias[h]));
            be = sigmoid_bf16(bf2f(gb_raw));
        }
        float lc = lg;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const float o = __shfl_up(lc, d, 64);
            if (lane >= d) lc += o;
        }
        const float tot = __shfl(lc, 63, 64);
        float rs = lg;                                          // decay from token t to the chunk's end: a suffix sum of its own,
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {                      // not tot - lc (two large prefix sums that nearly cancel)
            const float o = __shfl_down(rs, d, 64);
            if (lane + d < 64) rs += o;
        }
        const float suf = __shfl_down(rs, 1, 64);
        const float gm = expf(lc), dc = lane == 63 ? 1.f : expf(suf);
        L.Lc2[lane] = lc * LOG2E;
        L.beta[lane] = be;
        L.gam[lane] = gm;
        L.dec[lane] = dc;
        float* gp = gates + rec * GATE_FLOATS;
        gp[G_GAM + lane] = gm;
        gp[G_DEC + lane] = dc;
        if (lane >= 60) gp[G_GC + lane - 60] = lane == 60 ? expf(tot) : 0.f;
    }
    if (from_proj) silu_table_fill(L.tab, silu_tab, tid, 512);
    if (tid >= 508) L.staged[tid - 508] = 0;
    __syncthreads();

    // ---- k (group M) and q (group V): conv + SiLU + L2 norm, staged as half precision
    {
        _Float16* dst = grpV ? L.Qs : L.Ks;
        if (!from_proj) {
#pragma unroll
            for (int rr = 0; rr < 4; rr++) *reinterpret_cast<half8*>(&dst[(rr * 16 + gi) * QS_LD + cc * 8]) = bf8_to_half8(rwA[rr]);
            if (grpV) {
#pragma unroll
                for (int rr = 0; rr < 4; rr++) {
                    const int t = t0 + rr * 16 + gi;
                    rwB[rr] = *reinterpret_cast<const uint4*>(vi + ((size_t)min(t, S - 1) * HV + h) * DK + cc * 8);
                    if (t >= S) rwB[rr] = make_uint4(0, 0, 0, 0);
                }
            }
        } else {
            const float sc = grpV ? BF(INV_SCALE * INV_SCALE) : BF(INV_SCALE);
            uint4 wt[4], pk[4];
            float ss[4], rr[4];
#pragma unroll
            for (int e = 0; e < 4; e++) wt[e] = *reinterpret_cast<const uint4*>(&L.taps[(partA * DK + cc * 8 + 2 * e) * 4]);
#pragma unroll
            for (int j = 0; j < 4; j++) ss[j] = (float)row16_sum_d(conv8_silu_packed(L.tab, rwA[j], rwA[j + 1], rwA[j + 2], rwA[j + 3], wt, pk[j]));
            __builtin_amdgcn_sched_barrier(0);           // (the loads below must not be moved up: there is no room for them before)
            if (grpV) {                                  // v's rows: requested once q's are consumed (the register file holds one set)
                const int chB = 2 * KD + h * DK + cc * 8;
#pragma unroll
                for (int d = 0; d < 7; d++) {
                    const int tt = min(t0 + 4 * gi - 3 + d, S - 1);
                    rwB[d] = *reinterpret_cast<const uint4*>(tt < 0 ? cs + (tt + 3) * CD + chB : proj + (size_t)tt * PW + chB);
                }
            }
            rsqrt_rows<4>(ss, qk_eps(), rr, cc);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int tl = 4 * gi + j, t = t0 + tl;
                uint4 p = scale8_packed(pk[j], rr[j], sc);
                if (t >= S) p = make_uint4(0, 0, 0, 0);
                if (write_qkv && t < S) *reinterpret_cast<uint4*>(outA + ((size_t)t * HV + h) * DK + cc * 8) = p;
                *reinterpret_cast<half8*>(&dst[tl * QS_LD + cc * 8]) = bf8_to_half8(p);
            }
        }
    }
    part_staged(L, grpV ? PA_Q : PA_K, lane);

    if (grpV) {
        // ---- v: conv + SiLU, staged
        if (!from_proj) {
#pragma unroll
            for (int rr = 0; rr < 4; rr++) *reinterpret_cast<half8*>(&L.Vs[(rr * 16 + gi) * VS_LD + cc * 8]) = bf8_to_half8(rwB[rr]);
        } else {
            uint4 wt[4];
#pragma unroll
            for (int e = 0; e < 4; e++) wt[e] = *reinterpret_cast<const uint4*>(&L.taps[(2 * DK + cc * 8 + 2 * e) * 4]);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int tl = 4 * gi + j, t = t0 + tl;
                uint4 p;
                (void)conv8_silu_packed(L.tab, rwB[j], rwB[j + 1], rwB[j + 2], rwB[j + 3], wt, p);
                if (t >= S) p = make_uint4(0, 0, 0, 0);
                if (write_qkv && t < S) *reinterpret_cast<uint4*>(vi + ((size_t)t * HV + h) * DK + cc * 8) = p;
                *reinterpret_cast<half8*>(&L.Vs[tl * VS_LD + cc * 8]) = bf8_to_half8(p);
            }
        }
        part_staged(L, PA_V, lane);
        await_part(L, PA_Q);
        await_part(L, PA_K);
        // Kh = K^T (rows dk of tiles 2w, 2w+1), k index permuted: group V has the time for it (group M ends last)
        for (int mm = 0; mm < 2; mm++) {
            const int mt = 2 * w + mm;
            for (int kb2 = 0; kb2 < 2; kb2++)
                *reinterpret_cast<half8*>(op + OP_K + (mt * 2 + kb2) * 512 + lane * 8) = tokens_operand(L.Ks, QS_LD, kb2, 16 * mt, n, g);
        }
        // ---- Am = lower_incl(G * Q K^T) transposed, rows c_out = 16 ct + n, k = c_in (permuted); G_ij = exp2(Lc2_i - Lc2_j)
        const int ct = w, co = 16 * ct + n;
        const float lco = L.Lc2[co];
        for (int kb2 = 0; kb2 < 2; kb2++) {
            f32x4 part[2];
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {
                const int tj = 2 * kb2 + hf;
                part[hf] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (tj <= ct) {
#pragma unroll
                    for (int kb = 0; kb < 4; kb++) {
                        const half8 a = *reinterpret_cast<const half8*>(&L.Ks[(16 * tj + n) * QS_LD + 32 * kb + 8 * g]);
                        const half8 b = *reinterpret_cast<const half8*>(&L.Qs[(16 * ct + n) * QS_LD + 32 * kb + 8 * g]);
                        part[hf] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, part[hf], 0, 0, 0);
                    }
                    const f32x4 lcj = *reinterpret_cast<const f32x4*>(&L.Lc2[16 * tj + 4 * g]);
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const float v = __builtin_amdgcn_exp2f(lco - lcj[r]) * part[hf][r];
                        part[hf][r] = (tj < ct || 4 * g + r <= n) ? v : 0.f;
                    }
                }
            }
            __builtin_nontemporal_store(pack_half8(part[0], part[1]), reinterpret_cast<half8*>(op + OP_A + (ct * 2 + kb2) * 512 + lane * 8));
        }
        // Qh = Q (rows of tile ct), k index permuted: two 8-byte pieces of the row
        for (int kb = 0; kb < 4; kb++) {
            const _Float16* qr = &L.Qs[(16 * ct + n) * QS_LD + 32 * kb + 4 * g];
            const half4 lo = *reinterpret_cast<const half4*>(qr), hi = *reinterpret_cast<const half4*>(qr + 16);
            half8 qh;
            qh[0] = lo[0]; qh[1] = lo[1]; qh[2] = lo[2]; qh[3] = lo[3];
            qh[4] = hi[0]; qh[5] = hi[1]; qh[6] = hi[2]; qh[7] = hi[3];
            __builtin_nontemporal_store(qh, reinterpret_cast<half8*>(op + OP_Q + (ct * 4 + kb) * 512 + lane * 8));
        }
        return;
    }

    // ---- group M: T = (I + L)^-1 by block rows, then Wn^T = K^T (-Tb gamma)^T and U = Tb V on fp16 MFMA; wavefront w owns the
    // chunk rows of tile ct = w.  Both Tb operands hold Tb[16 ct + n][kperm(kb2, g, 0..7)]: as the A operand of U, and (columns
    // scaled by -gamma) as the B operand of Wn^T.
    await_part(L, PA_K);
    __builtin_amdgcn_s_setprio(2);                       // few instructions, all of them on the critical path
    half8 tbU[2], tbW[2];
    inverse_row(L, w, n, g, tbU, tbW);
    const int ct = w, nkb = ct < 2 ? 1 : 2;              // Tb is lower triangular: columns past the row tile are zero
    for (int kb = 0; kb < 4; kb++) {
        f32x4 acc[2];
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            const int mt = 2 * kb + hf;
            acc[hf] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kb2 = 0; kb2 < 2; kb2++) {
                if (kb2 >= nkb) continue;
                acc[hf] = __builtin_amdgcn_mfma_f32_16x16x32_f16(tokens_operand(L.Ks, QS_LD, kb2, 16 * mt, n, g), tbW[kb2], acc[hf], 0, 0, 0);
            }
        }
        *reinterpret_cast<half8*>(op + OP_W + (ct * 4 + kb) * 512 + lane * 8) = pack_half8(acc[0], acc[1]);
    }
    __builtin_amdgcn_s_setprio(0);
    await_part(L, PA_V);
    _Float16* up = U + rec * U_HALVES;
    for (int sl = 0; sl < 8; sl++) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb2 = 0; kb2 < 2; kb2++) {
            if (kb2 >= nkb) continue;
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(tbU[kb2], tokens_operand(L.Vs, VS_LD, kb2, 16 * sl, n, g), acc, 0, 0, 0);
        }
        half4 uh;
        uh[0] = (_Float16)acc[0]; uh[1] = (_Float16)acc[1]; uh[2] = (_Float16)acc[2]; uh[3] = (_Float16)acc[3];
        *reinterpret_cast<half4*>(up + ((sl * NCT + ct) * 64 + lane) * 4) = uh;
    }
}

}  // namespace

extern "C" {

// sizes (bytes) of the phase A -> phase B buffers for S tokens: ops, U (half precision), gC (the gate records)
long qt_gdn_chunk_ops_bytes(int S) { return S < 0 ? -1 : (long)((S + C - 1) / C) * HV * OP_HALVES * 2; }
long qt_gdn_chunk_u_bytes(int S) { return S < 0 ? -1 : (long)((S + C - 1) / C) * HV * U_HALVES * 2; }
long qt_gdn_chunk_gc_bytes(int S) { return S < 0 ? -1 : (long)((S + C - 1) / C) * HV * GATE_FLOATS * 4; }

// polls before an output workgroup of the one-launch form gives up on its chunk (0 = the default, about a second)
static std::atomic<int> poll_limit{0};

static int phase_b_launch(const void* ops, const void* U, const float* gC, void* snap, const float* state_in, float* state_out,
                          void* y, const void* proj, const float* gw, float eps, bool norm, int S, hipStream_t stream) {
    if (!ops || !U || !gC || !snap || !state_in || !state_out || !y) return QT_ERR_NULL;
    if (norm && (!proj || !gw)) return QT_ERR_NULL;
    if (S < 0) return QT_ERR_DIM;
    for (const void* p : {ops, U, (const void*)gC, (const void*)snap, (const void*)state_in, (const void*)state_out, (const void*)y, proj})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    const int NC = (S + C - 1) / C;
    if (NC == 0) {
        if (state_out != state_in &&
            hipMemcpyAsync(state_out, state_in, sizeof(float) * HV * DV * DK, hipMemcpyDeviceToDevice, stream) != hipSuccess)
            return QT_ERR_LAUNCH;
        return QT_OK;
    }
    if (NC >= FUSED_MIN_CHUNKS) {
        const dim3 grid(N_CHAIN + min(MAX_OUT_WGS, NC * HV)), block(384);
        const int pl = poll_limit.load(std::memory_order_relaxed), spin = pl > 0 ? pl : SPIN_LIMIT;
        if (norm)
            hipLaunchKernelGGL(gdn_phase_b_kernel<true>, grid, block, 0, stream, (const _Float16*)ops, (const _Float16*)U, gC, state_in,
                               state_out, (_Float16*)snap, (bf16_t*)y, (const bf16_t*)proj, gw, eps, S, NC, spin);
        else
            hipLaunchKernelGGL(gdn_phase_b_kernel<false>, grid, block, 0, stream, (const _Float16*)ops, (const _Float16*)U, gC, state_in,
                               state_out, (_Float16*)snap, (bf16_t*)y, (const bf16_t*)nullptr, (const float*)nullptr, 0.f, S, NC, spin);
    } else {
        hipLaunchKernelGGL(gdn_chain_kernel, dim3(N_CHAIN), dim3(384), 0, stream, (const _Float16*)ops, (const _Float16*)U, gC, state_in,
                           state_out, (_Float16*)snap, NC);
        QT_CHECK_LAUNCH();
        if (norm)
            hipLaunchKernelGGL(gdn_output_kernel<true>, dim3(NC * HV), dim3(256), 0, stream, (const _Float16*)ops, (const _Float16*)snap,
                               gC, (bf16_t*)y, (const bf16_t*)proj, gw, eps, S, NC);
        else
            hipLaunchKernelGGL(gdn_output_kernel<false>, dim3(NC * HV), dim3(256), 0, stream, (const _Float16*)ops,
                               (const _Float16*)snap, gC, (bf16_t*)y, (const bf16_t*)nullptr, (const float*)nullptr, 0.f, S, NC);
    }
    QT_CHECK_LAUNCH();
    return QT_OK;
}

int qt_gdn_phase_b_poll_limit(int polls) {
    if (polls < 0) return QT_ERR_DIM;
    poll_limit.store(polls, std::memory_order_relaxed);
    return QT_OK;
}
long qt_gdn_chunk_status_offset(void) { return (long)FLAG_ERR * 4; }

long qt_gdn_chunk_snap_bytes(int S) { return S < 0 ? -1 : (long)FLAG_WORDS * 4 + (long)((S + C - 1) / C) * HV * 8 * SNAP_HALVES * 2; }

int qt_gdn_phase_b(const void* ops, const void* U, const float* gC, void* snap, const float* state_in, float* state_out, void* y,
                   int S, hipStream_t stream) {
    return phase_b_launch(ops, U, gC, snap, state_in, state_out, y, nullptr, nullptr, 0.f, false, S, stream);
}

int qt_gdn_phase_b_norm(const void* ops, const void* U, const float* gC, void* snap, const float* state_in, float* state_out,
                        const void* proj, const float* gw, float eps, void* out, int S, hipStream_t stream) {
    return phase_b_launch(ops, U, gC, snap, state_in, state_out, out, proj, gw, eps, true, S, stream);
}

int qt_gdn_phase_a(const void* proj, const void* q, const void* k, const void* v, const float* A_log, const float* dt_bias,
                   void* ops, void* U, float* gC, int S, hipStream_t stream) {
    if (!proj || !q || !k || !v || !A_log || !dt_bias || !ops || !U || !gC) return QT_ERR_NULL;
    if (S < 0) return QT_ERR_DIM;
    if (S == 0) return QT_OK;
    for (const void* p : {proj, q, k, v, (const void*)ops, (const void*)U, (const void*)gC})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    const int NC = (S + C - 1) / C;
    hipLaunchKernelGGL(gdn_phase_a_kernel<false>, dim3(NC * HV), dim3(512), 0, stream, false, (const bf16_t*)proj, (bf16_t*)q,
                       (bf16_t*)k, (bf16_t*)v, (const bf16_t*)nullptr, (const bf16_t*)nullptr, (const bf16_t*)nullptr,
                       (bf16_t*)nullptr, A_log, dt_bias, (_Float16*)ops, (_Float16*)U, gC, S);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

int qt_gdn_phase_a_conv(const void* proj, const void* conv_state, const void* conv_w, const void* silu_table, const float* A_log,
                        const float* dt_bias, void* q, void* k, void* v, void* conv_out, void* ops, void* U, float* gC, int S,
                        hipStream_t stream) {
    if (!proj || !conv_state || !conv_w || !A_log || !dt_bias || !ops || !U || !gC) return QT_ERR_NULL;
    if ((q || k || v) && !(q && k && v)) return QT_ERR_NULL;
    if (S < 0) return QT_ERR_DIM;
    if (S == 0) return QT_OK;
    for (const void* p : {proj, conv_state, conv_w, silu_table, (const void*)q, (const void*)k, (const void*)v, (const void*)conv_out,
                          (const void*)ops, (const void*)U, (const void*)gC})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return QT_ERR_ALIGN;
    if (conv_out == conv_state) return QT_ERR_UNSUPPORTED;          // the old window is still being read when the new one is written
    const int NC = (S + C - 1) / C;
    hipLaunchKernelGGL(gdn_phase_a_kernel<true>, dim3(NC * HV), dim3(512), 0, stream, q != nullptr, (const bf16_t*)proj, (bf16_t*)q,
                       (bf16_t*)k, (bf16_t*)v, (const bf16_t*)conv_state, (const bf16_t*)conv_w, (const bf16_t*)silu_table,
                       (bf16_t*)conv_out, A_log, dt_bias, (_Float16*)ops, (_Float16*)U, gC, S);
    QT_CHECK_LAUNCH();
    return QT_OK;
}

}  // extern "C"
