/* C ABI of libqwen_tailor_hip.so: the GatedDeltaNet + GQA head-dim-256 attention hot path of wang90063/Qwen-tailor
 * on MI355X (gfx950).
 *
 * The reference has no FFI: its boundary is a set of Python functions over MLX arrays that launch Metal kernels
 * (qwen35/gated_delta.py, kernels.py, batch.py, batch_spec.py, prefill.py, gdn_nax.py).  Each entry point below is what
 * one of those functions binds to; the citation names the reference function it replaces.
 *
 * Conventions: every pointer is a device pointer unless said otherwise; bf16 tensors are passed as raw 16-bit words
 * (const void*), state is float; tensors are contiguous in the layouts of the reference; index arrays are int32 on the
 * device; `stream` is a hipStream_t (passed as void* so that this header needs no HIP include).  No entry point
 * allocates or synchronises; all work is enqueued on `stream`.  What the library keeps per process: the CU count of each
 * device (asked once, cached), the static scratch array of qt_gqa_attn_decode_static with its per-device address, and the
 * poll limit set by qt_gdn_phase_b_poll_limit.  Return value: 0 on success, or
 *   -1 bad dimension, -2 misaligned pointer, -3 null pointer, -4 unsupported shape, -5 launch failure,
 *   -6 workspace too small, -7 size beyond the maximum of the allocation-free entry point.
 * Rows whose slot index lies outside the pool (or whose position would overflow it) are skipped by the kernels: nothing
 * outside the caller's buffers is ever read or written.
 */
#ifndef QWEN_TAILOR_HIP_H
#define QWEN_TAILOR_HIP_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* qt_stream_t; /* hipStream_t */

/* batch.deltanet_b (qwen35/batch.py:128-135): one decode token for each of B rows.
 * proj [B,8224] bf16; conv_pool [n_slots*2,3,6144] bf16 (reads buffer slot*2+(pos&1), writes the other one);
 * conv_w [6144*4] bf16; A_log, dt_bias [16] f32; ssm_pool [n_slots,16,128,128] f32 (updated in place);
 * slots, pos [B] int32; y [B,2048] bf16.  rows_per_wg: 0 = choose, else 16/32/64/128 value rows per workgroup
 * (qt_gdn_decode_step also takes 256 / 512 = two / four whole heads per workgroup). */
int qt_gdn_decode_step(const void* proj, void* conv_pool, const void* conv_w, const float* A_log, const float* dt_bias,
                       float* ssm_pool, const int32_t* slots, const int32_t* pos, void* y, int B, int n_slots,
                       int rows_per_wg, qt_stream_t stream);

/* qt_gdn_decode_step followed by qt_gated_rmsnorm (batch.deltanet_b + batch.gnorm_rows, qwen35/batch.py:128-135, 338-343) in one
 * launch: out [B,2048] bf16 = gated RMSNorm of the step's outputs with z = proj[:,6144:8192] and weight gw [128] f32 (same bits
 * as the two launches); the un-normalised outputs are not stored. */
int qt_gdn_decode_step_gnorm(const void* proj, void* conv_pool, const void* conv_w, const float* A_log, const float* dt_bias,
                             float* ssm_pool, const int32_t* slots, const int32_t* pos, const float* gw, float eps, void* out, int B,
                             int n_slots, qt_stream_t stream);

/* batch_spec.deltanet_bm (qwen35/batch_spec.py:142-150): M chained tokens for each of B sequences, a state snapshot
 * after every token.  proj [B*M,8224]; conv_pool [n_entries*2,M,3,6144]; ssm_pool [n_entries,M,16,128,128];
 * sslots, sels, pars [B] int32 (pool entry, snapshot to start from, conv buffer to read); y [B*M,2048].  1 <= M <= 16. */
int qt_gdn_verify_step(const void* proj, void* conv_pool, const void* conv_w, const float* A_log, const float* dt_bias,
                       float* ssm_pool, const int32_t* sslots, const int32_t* sels, const int32_t* pars, void* y, int B,
                       int M, int n_entries, int rows_per_wg, qt_stream_t stream);

/* kernels.deltanet (qwen35/kernels.py:555-567): one sequence, M tokens from snapshot sel[0] of conv_snap [n_snap,3,6144]
 * / ssm_snap [n_snap,16,128,128]; writes y [M,2048], cs_out [M,3,6144], st_out [M,16,128,128]. */
int qt_gdn_deltanet(const void* proj, const void* conv_snap, const void* conv_w, const float* A_log, const float* dt_bias,
                    const float* ssm_snap, const int32_t* sel, void* y, void* cs_out, float* st_out, int M, int n_snap,
                    int rows_per_wg, qt_stream_t stream);

/* compute_g and beta = sigmoid(b) (qwen35/gated_delta.py:16-18,158).  a, b: bf16, `rows` rows of hv values with row strides
 * a_stride / b_stride (elements), so they can point into the projection rows.  Outputs (each may be null): g f32
 * [rows,hv], log_g f32 [rows,hv] (= log of g before the final exp), beta bf16 [rows,hv]. */
int qt_gdn_gates(const void* a, const void* b, long a_stride, long b_stride, const float* A_log, const float* dt_bias,
                 float* g, float* log_g, void* beta, long rows, int hv, qt_stream_t stream);

/* normalize_qk (qwen35/gated_delta.py:21-30) on `rows` rows of dk = 128 bf16 values. */
int qt_normalize_qk(const void* q, const void* k, void* q_out, void* k_out, long rows, int dk, qt_stream_t stream);

/* prefill.conv_prep (qwen35/prefill.py:228-238): proj [S,8224], conv_state [3,6144] -> q, k, v [S,16,128] bf16.
 * silu_table: the qt_silu_table_bytes() byte table written once by qt_silu_table_build (the bf16 -> bf16 map of
 * mslib.py:21-22 on 2^-9 <= |x| < 2^5), owned by the caller; null = every workgroup computes its own copy. */
int qt_silu_table_bytes(void);
int qt_silu_table_build(void* table, qt_stream_t stream);
int qt_gdn_conv_prep(const void* proj, const void* conv_state, const void* conv_w, const void* silu_table, void* q, void* k,
                     void* v, int S, qt_stream_t stream);

/* batch.gnorm_rows / prefill.gated_norm (qwen35/batch.py:338-343, qwen35/prefill.py:241-244): y [rows,2048] bf16,
 * z = proj[:,6144:8192] of proj [rows,8224], gw [128] f32 -> out [rows,2048] bf16. */
int qt_gated_rmsnorm(const void* y, const void* proj, const float* gw, void* out, long rows, float eps, qt_stream_t stream);

/* gated_delta_update's recurrence kernel (qwen35/gated_delta.py:143-174) with g (f32) and beta (bf16) [B,T,Hv] given:
 * q, k [B,T,Hk,128], v, y [B,T,Hv,Dv] bf16, state [B,Hv,Dv,128] f32.  Dk must be 128 and Dv a multiple of 8, otherwise -4
 * (where the reference raises ValueError, gated_delta.py:164-166). */
int qt_gdn_recurrent(const void* q, const void* k, const void* v, const float* g, const void* beta, const float* state_in,
                     float* state_out, void* y, int B, int T, int Hk, int Hv, int Dk, int Dv, qt_stream_t stream);

/* batch.attn_b (qwen35/batch.py:230-237): ragged decode / verify attention, 8 query heads on 2 KV heads, head dim 256.
 * q [B*M,8,256], k_new / v_new [B*M,2,256], pools Kp / Vp [n_slots,2,Lmax,256] bf16 (rows pos[b]..pos[b]+M-1 are appended),
 * out [B*M,8,256].  1 <= M <= 16 (the limit of qt_gdn_verify_step; the reference kernel is generic in M), B <= 1024.  Up to
 * four tokens per sequence share one pass over the pool; more run as passes of four (rows 4p .. 4p+3 at pos[b] + 4p), each a
 * pair of launches.  The batch's 16-key tiles are spread evenly over one workgroup per CU (split-K
 * over a flat tile space, so ragged lengths balance); CH = smallest number of pool keys one workgroup takes (multiple of 16).
 * Workspace of at least qt_gqa_attn_workspace_bytes(B, M, Lmax, CH) bytes, 16-byte aligned, owned by the caller. */
long qt_gqa_attn_workspace_bytes(int B, int M, int Lmax, int CH);
int qt_gqa_attn_decode(const void* q, const void* k_new, const void* v_new, void* Kp, void* Vp, const int32_t* slots,
                       const int32_t* pos, void* out, void* workspace, long workspace_bytes, int B, int M, int Lmax,
                       int n_slots, int CH, qt_stream_t stream);

/* qt_gqa_attn_decode without the workspace argument.  No counterpart in the reference: it is for callers that cannot
 * allocate device memory or pass a workspace along (code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation).  The split-K partial results live in an 8.1 MiB static device array inside the library (one copy per GPU, held
 * until the process ends), so B <= 128 (otherwise -7) and the partial kernel's grid is capped at 256 workgroups; same kernels,
 * same results as qt_gqa_attn_decode.  The entry point allocates nothing; its first call on a device looks the array's address up
 * (make that call outside graph capture).  All calls on one GPU share the array: calls that overlap there (two streams, two
 * threads) race, so serialise them. */
int qt_gqa_attn_decode_static(const void* q, const void* k_new, const void* v_new, void* Kp, void* Vp, const int32_t* slots,
                              const int32_t* pos, void* out, int B, int M, int Lmax, int n_slots, int CH, qt_stream_t stream);

/* The attention half of a full-attention layer at a decode / verify step, between its qkv and o projections, in two launches per
 * pass of four tokens: qt_attn_qkv_prep, qt_gqa_attn_decode and qt_attn_out_gate in one (qwen35/batch.py:505-513: mx.fast.rms_norm
 * and mx.fast.rope on q / k, attn_b, o * sigmoid(gate)).  qkv [B*M,5120] bf16 as for qt_attn_qkv_prep; q_norm, k_norm [256] bf16;
 * out [B*M,2048] bf16, the same values as the three calls give.  The query rows and the new keys are normed and roped inside
 * the attention kernel by every workgroup that needs them, the gate is applied where the split-K parts are merged; q, k, v
 * and the un-gated o are never stored.  rope_table: the (cos, sin) pairs of positions 0 .. table_positions - 1
 * (qt_rope_table_bytes(n) bytes, written once by qt_rope_table_build, owned by the caller, 16-byte aligned); table_positions >=
 * Lmax.  Workspace, limits and the treatment of out-of-range rows as for qt_gqa_attn_decode. */
long qt_rope_table_bytes(int n_pos);
int qt_rope_table_build(void* table, int n_pos, qt_stream_t stream);
int qt_gqa_attn_layer_decode(const void* qkv, const void* q_norm, const void* k_norm, const void* rope_table, int table_positions,
                             void* Kp, void* Vp, const int32_t* slots, const int32_t* pos, void* out, void* workspace,
                             long workspace_bytes, int B, int M, int Lmax, int n_slots, int CH, float eps, qt_stream_t stream);

/* Chunked (chunk = 64) GatedDeltaNet prefill, two phases (qwen35/gdn_nax.py:394-426: prep_a / gdn_chunked's phase A, phase_b).
 * Phase A is parallel over (chunk, head): it takes q, k, v [S,16,128] bf16 (qt_gdn_conv_prep's outputs) and the gate inputs in
 * proj [S,8224], and computes the gates, K K^T / Q K^T on fp16 MFMA, the 64 x 64 unit-lower-triangular inverse in fp32 and the
 * state-independent MFMA operands of phase B.  It fills three caller-owned buffers of qt_gdn_chunk_{ops,u,gc}_bytes(S) bytes, all
 * 16-byte aligned: `ops` and `U` (half-precision operand tiles) and `gC` (f32: per (chunk, head) the 64 per-token decay
 * factors gamma and dec and the chunk's total decay, which phase B applies to accumulator rows).
 * Intermediate operands are half precision (fp16: 11 significant bits, largest finite value 65504): conv outputs |v| and
 * states |S| beyond that are not representable and are not supported; values below 6e-5 lose precision gracefully.
 * Phase B: state_in / state_out [16,128,128] f32, y [S,16,128] bf16.  128 workgroups run the serial state chain over the chunks
 * and leave the per-chunk B operands in `snap`; others compute the outputs of a chunk from them: as a second launch up to 63
 * chunks (4032 tokens), from 64 chunks on in the same launch, as soon as the chain has published the chunk.  `snap`: qt_gdn_chunk_snap_bytes(S) bytes, caller-owned, 16-byte aligned; its
 * first 33 KiB (qt_gdn_chunk_snap_bytes(0) bytes) are the flag area of the launch and MUST BE ZERO when a launch starts (memory that
 * was merely allocated will not do: the one-launch form reads its queue head and progress words from it).  A launch leaves
 * them zero, so the caller zeroes them once; launches that use the same `snap` must not overlap.  The one word a launch may
 * leave set is the STATUS WORD, the int32 at byte qt_gdn_chunk_status_offset() (32772) of `snap`; no launch clears it, the
 * caller reads it after (or asynchronously behind) the launch and resets it:
 *   bit 0: an output workgroup of the one-launch form polled for its chunk longer than the poll limit (about a second) and
 *          gave up; its rows of y were NOT written.  It cannot happen while the chain workgroups run undisturbed.
 *   bit 1: the final state holds a value that is not finite: an operand left the half-precision range (above) and y is not
 *          to be trusted either.
 * qt_gdn_phase_b_poll_limit(polls) sets the poll limit of later launches (0 = the default); it exists so that the give-up
 * path can be exercised from the host with a tiny limit.
 * qt_gdn_phase_b_norm is the same with prefill.gated_norm (qwen35/prefill.py:241-244) fused into the output kernel: it
 * writes out [S,2048] bf16 = gated RMSNorm of y with z = proj[:,6144:8192] and weight gw [128] f32 instead of y. */
long qt_gdn_chunk_ops_bytes(int S);
long qt_gdn_chunk_u_bytes(int S);
long qt_gdn_chunk_gc_bytes(int S);
long qt_gdn_chunk_snap_bytes(int S);
long qt_gdn_chunk_status_offset(void);
int qt_gdn_phase_b_poll_limit(int polls);
int qt_gdn_phase_a(const void* proj, const void* q, const void* k, const void* v, const float* A_log, const float* dt_bias,
                   void* ops, void* U, float* gC, int S, qt_stream_t stream);
/* qt_gdn_phase_a with qt_gdn_conv_prep fused in (the reference's fused prep kernel, qwen35/gdn_nax.py:394-401 prep_a, with the
 * conv-state roll of qwen35/prefill.py:262-263): q, k, v are computed from proj [S,8224], conv_state [3,6144] and conv_w
 * [6144*4] inside the kernel (same bits as qt_gdn_conv_prep).  q, k, v: all three null, or all three [S,16,128] bf16 outputs.
 * conv_out: null or [3,6144] bf16, receives the new conv window (must not alias conv_state).  silu_table as qt_gdn_conv_prep. */
int qt_gdn_phase_a_conv(const void* proj, const void* conv_state, const void* conv_w, const void* silu_table, const float* A_log,
                        const float* dt_bias, void* q, void* k, void* v, void* conv_out, void* ops, void* U, float* gC, int S,
                        qt_stream_t stream);
int qt_gdn_phase_b(const void* ops, const void* U, const float* gC, void* snap, const float* state_in, float* state_out,
                   void* y, int S, qt_stream_t stream);
int qt_gdn_phase_b_norm(const void* ops, const void* U, const float* gC, void* snap, const float* state_in, float* state_out,
                        const void* proj, const float* gw, float eps, void* out, int S, qt_stream_t stream);

/* Causal prefill attention: the mx.fast.scaled_dot_product_attention(..., mask="causal") call of the full-attention layers
 * (qwen35/model.py:160-167, qwen35/prefill.py:468).  q, out [8][S][256] bf16 with head stride q_head_stride (elements);
 * K, V [2][>=L][256] bf16 with head stride kv_head_stride; query i sits at position q_pos0 + i and sees keys 0..q_pos0+i.
 * Launches that would leave CUs idle (a prompt of up to about 2800 rows, or rows continuing a long prefix) are split along
 * the keys; the parts meet in `workspace` and a second kernel combines them.  qt_gqa_prefill_workspace_bytes_for gives the bytes this launch uses (0: not split),
 * qt_gqa_prefill_workspace_bytes an upper bound for every launch with at most L keys.  With a null or smaller workspace the
 * launch runs unsplit: same results up to rounding, slower.  Requires q_pos0 + S <= L. */
long qt_gqa_prefill_workspace_bytes(int L);
long qt_gqa_prefill_workspace_bytes_for(int S, int L, int q_pos0);
int qt_gqa_prefill_causal(const void* q, const void* K, const void* V, void* out, void* workspace, long workspace_bytes, int S,
                          int L, int q_pos0, long q_head_stride, long kv_head_stride, qt_stream_t stream);

/* The elementwise steps either side of the attention kernels in a full-attention layer (qwen35/batch.py:505-513,
 * qwen35/model.py:154-169).  qkv [R,5120] bf16 = [(q_h[256] | gate_h[256]) for 8 heads | k[2][256] | v[2][256]].
 * qt_attn_qkv_prep: q [R,8,256], k [R,2,256] = rope(rms_norm(., q_norm / k_norm [256] bf16, eps), position), v [R,2,256] = v;
 * rotary embedding of the first 64 features, half-split pairing, theta 1e7; row r = b*M + j sits at position pos[b] + j.
 * qt_attn_qkv_prep_table: the same (the same call of the reference, the same bits) with the (cos, sin) pairs of positions
 * 0 .. table_positions - 1 read from rope_table (as for qt_gqa_attn_layer_decode above; may be null) instead of evaluated
 * per row; rows at positions beyond the table evaluate their own.
 * qt_attn_out_gate: out [R,2048] = o [R,8,256] * sigmoid(gate). */
int qt_attn_qkv_prep(const void* qkv, const void* q_norm, const void* k_norm, const int32_t* pos, void* q, void* k, void* v, long R,
                     int M, float eps, qt_stream_t stream);
int qt_attn_qkv_prep_table(const void* qkv, const void* q_norm, const void* k_norm, const int32_t* pos, const void* rope_table,
                           int table_positions, void* q, void* k, void* v, long R, int M, float eps, qt_stream_t stream);
int qt_attn_out_gate(const void* o, const void* qkv, void* out, long R, qt_stream_t stream);

/* The projections either side of the core at decode / verify time: the reference's fused_gemv (qwen35/kernels.py:80-319) on
 * plain bf16 weights and its stand-alone prologue rms_rows (qwen35/batch.py:249-301).
 * qt_rms_rows: y [M,K] bf16 = BF(nw * (x * rsqrt(mean(x^2) + eps))), x [M,K] bf16, nw [K] bf16; K a multiple of 8.
 * qt_fused_gemv: s = x [M,K] . W [N,K]^T accumulated in fp32 (bf16 MFMA), then epilogue
 *     0: y [M,N] = bf16(s)        1: y [M,N] = bf16(BF(s) + res [M,N])
 *     2: y [M,N/2], y[m][p] = bf16(silu_bf16(BF(s[m][2p])) * BF(s[m][2p+1]))   (interleaved gate / up rows, N even)
 * K a multiple of 256.  The gated-norm prologue of the reference is qt_gated_rmsnorm applied to x first; the rms prologue is
 * qt_rms_rows: both round to bf16 before the product, exactly as the fused forms do. */
int qt_rms_rows(const void* x, const void* nw, void* y, int M, int K, float eps, qt_stream_t stream);
int qt_fused_gemv(const void* W, const void* x, const void* res, void* y, int M, int N, int K, int epilogue, qt_stream_t stream);

/* batch.blit (qwen35/batch.py:365-372), the in-place strided copy behind Pools.load / read (batch.py:431-462) and the
 * scheduler's plain <-> speculative state moves (qwen35/serve.py:310-348):
 *     dst.flat[d0 + y*dstride + i] = src.flat[s0 + y*sstride + i]   for i < n, y < ny   (offsets and strides in elements)
 * elem_size = 2 (bf16) or 4 (f32); ny <= 65535; the ranges written must not overlap the ranges read. */
int qt_blit(void* dst, const void* src, int elem_size, long n, long d0, long s0, long ny, long dstride, long sstride,
            qt_stream_t stream);

/* `count` qt_blit copies in one launch (a sequence's admission is 48 of them: Pools.load, qwen35/batch.py:431-447).
 * dst[k], src[k]: device base pointers (the arrays themselves are host memory); meta[7k .. 7k+6] (host memory) =
 * { elem_size, n, d0, s0, ny, dstride, sstride } as for qt_blit.  Every copy must be 16-byte granular (base pointers, and
 * n, d0, s0, dstride, sstride in bytes), otherwise -2 and nothing is launched. */
int qt_blit_batch(void* const* dst, const void* const* src, const long* meta, int count, qt_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
