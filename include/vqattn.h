/*
 * libvqattn_gfx950 -- C ABI of the MI355X (gfx950) fused VQ-attention kernels.
 *
 * This is the boundary a host binds instead of the reference's Triton launches.  Every entry point
 *   - takes plain device pointers, sizes and element strides (no torch types),
 *   - enqueues its kernels on the given HIP stream and returns without synchronising,
 *   - allocates nothing and keeps no state between calls (scratch comes in through `workspace`; the one exception,
 *     vqa_decode_static_bf16, works in a fixed device array of the library and says so below).  What the library does
 *     remember, behind a mutex, is per-device set-up done on first use: the raised dynamic-LDS limit of the kernels
 *     that need more than 64 KB (the count kernel at head dim 128, the pipelined prefill / window kernels) and the
 *     device address of that array.  Both belong to the device that owns the call's operands, which must be the
 *     calling thread's current device (VQA_ERR_BAD_ARGUMENT otherwise: the kernels would be launched elsewhere),
 *   - returns VQA_OK (0) or a negative vqa_status; it never throws or aborts.
 * Tensors are addressed as base + sum(index_i * stride_i) in ELEMENTS of their own type; the innermost
 * (head_dim / codebook index M) stride must be 1.  Head dims of the attention entry points: 64 and 128; vqa_local_attn_*,
 * vqa_rerope_full_* and vqa_vqcount_* also take 32 (the reference's kernels of these kinds accept 16, 32, 64 and 128,
 * ops/triton_fused_attn_rerope.py:192, ops/triton_fused_vq_attn.py:198-199; a caller with head dim 16 zero-pads its
 * operands to 32, which leaves the scores unchanged, and drops the padded output columns -- the Python layer does).
 * The encoder, preprocessing and rotary entry points state their own limits.
 *
 * Log-sum-exp values are base 2 of the scaled scores, lse2 = log2(sum_j exp(s_ij * sm_scale)), the convention of
 * the reference kernels (ops/triton_fused_vq_attn.py:179, ops/triton_fused_local_attn_rerope.py:214-216).
 */
#ifndef VQATTN_H
#define VQATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef VQA_NO_HIP_STREAM_TYPEDEF
typedef struct ihipStream_t* vqa_stream_t; /* == hipStream_t */
#endif

typedef enum vqa_status {
    VQA_OK = 0,
    VQA_ERR_NULL_POINTER = -1,
    VQA_ERR_BAD_SHAPE = -2,
    VQA_ERR_UNSUPPORTED_HEAD_DIM = -3,
    VQA_ERR_UNSUPPORTED_CODEBOOK = -4,
    VQA_ERR_MISALIGNED = -5,
    VQA_ERR_WORKSPACE_TOO_SMALL = -6,
    VQA_ERR_BAD_ARGUMENT = -7,
    VQA_ERR_LAUNCH_FAILED = -8,
    VQA_ERR_SCRATCH_LIMIT = -9
} vqa_status;

/* Library version (major * 10000 + minor * 100 + patch). */
int vqa_version(void);

/* Static, NUL-terminated description of a vqa_status value. */
const char* vqa_strerror(int status);

/* ------------------------------------------------------------------------------------------------------------------
 * Decode: seqlen_q = 1 attention over additive-quantiser key codes.
 *
 *   out[b,h,:] = softmax_j( sm_scale * sum_m <q[b,h], codebooks[h,m,codes[b,h,j,m]]> ) . v[b,h,j,:]     j in [0, N)
 *
 * Replaces the seqlen_q == 1 route the reference sends through `naive_attn`
 * (ops/attn_vq.py:247-248, 445-479; "handled by a separate kernel", ops/README.md:3).
 *
 *   q         [B,H,1,D]  bf16 / f16          strides[0..1]  = (b, h)
 *   codes     [B,H,N,M]  uint8               strides[2..3]  = (b, h); rows are packed: stride(n) = M, stride(m) = 1
 *   codebooks [H,M,K,D]  same type as q      strides[4..6]  = (h, m, k)
 *   v         [B,H,N,D]  same type as q      strides[7..9]  = (b, h, n); each row 16-byte aligned
 *   out       [B,H,1,D]  same type as q      strides[10..11] = (b, h)
 *   lse       [B,H] float, base 2, nullable
 *   M in {1,2,4,8}, K <= 256, D in {64,128}.  Codes must lie in [0, K); a code >= K is scored as codeword K - 1 (the
 *   same clamp applies to vqa_prefill_*), it never reads outside the codebook.
 *   num_splits: KV splits per (b,h); <= 0 lets the library choose (vqa_decode_default_splits).
 *   workspace: >= vqa_decode_workspace_bytes(...) bytes of device memory, 256-byte aligned, owned by the caller.
 * ------------------------------------------------------------------------------------------------------------------ */
#define VQA_DECODE_NUM_STRIDES 12

int vqa_decode_default_splits(int B, int H, int N);

size_t vqa_decode_workspace_bytes(int B, int H, int N, int D, int M, int K, int num_splits);

int vqa_decode_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, void* out, float* lse,
                    void* workspace, size_t workspace_bytes, int B, int H, int N, int D, int M, int K,
                    const int64_t* strides, float sm_scale, int num_splits, vqa_stream_t stream);

int vqa_decode_f16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, void* out, float* lse,
                   void* workspace, size_t workspace_bytes, int B, int H, int N, int D, int M, int K,
                   const int64_t* strides, float sm_scale, int num_splits, vqa_stream_t stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Sliding-window exact attention, seqlen_q == seqlen_k == N, causal.  One kernel, three masks:
 *
 *   mode 0 (VQA_LOCAL_STRICT)  key j visible iff j <= i and i - j <= window
 *                              replaces ops/triton_fused_local_attn.py:254-262 (flash_attn_func)
 *   mode 1 (VQA_LOCAL_LOOSE)   key j visible iff j <= i and j >= floor(i/128)*128 - window  (whole 128-blocks)
 *                              replaces ops/triton_fused_local_attn2.py:249-256
 *   mode 2 (VQA_LOCAL_REROPE)  visible as mode 1; score = q1.k1 when i - j <= window, else q2.k2
 *                              replaces ops/triton_fused_local_attn_rerope.py:287-294
 *
 *   q1,q2,k1,k2,v,out: [B,H,N,D]-addressable bf16/f16 tensors; strides[0..17] = (b,h,n) element strides of
 *   q1, q2, k1, k2, v, out in this order (a [B,N,H,D] tensor is passed with its h and n strides swapped).
 *   q2/k2 are read only in mode 2 (may be NULL otherwise).  Inputs 16-byte aligned rows, out 8-byte aligned rows.
 *   lse: [B,H,N] contiguous float, base 2, nullable.
 *
 *   The library runs one of two kernels behind these entry points: the general one (any window and length), or --
 *   for head dims 64 / 128, windows of 512 keys or more that are multiples of 128, lengths that are multiples of 64 and
 *   at least 1024 query tiles of 128 rows -- a software-pipelined one (0.73 - 0.97 of the general kernel's time); a
 *   window that covers the sequence (plain causal attention) goes to the pipelined prefill kernel from 2048 tokens
 *   on.  The pipelined kernels multiply the query by sm_scale * log2(e) and round it to 16 bits before the products
 *   (the general kernel scales the fp32 scores): results agree within the 16-bit output tolerance, the base-2 lse
 *   within 1e-2 in bf16 (3e-3 on N(0,1) data).
 * ------------------------------------------------------------------------------------------------------------------ */
#define VQA_LOCAL_STRICT 0
#define VQA_LOCAL_LOOSE 1
#define VQA_LOCAL_REROPE 2
#define VQA_LOCAL_NUM_STRIDES 18

int vqa_local_attn_bf16(const void* q1, const void* q2, const void* k1, const void* k2, const void* v, void* out,
                        float* lse, int B, int H, int N, int D, const int64_t* strides, int window, int mode,
                        float sm_scale, vqa_stream_t stream);

int vqa_local_attn_f16(const void* q1, const void* q2, const void* k1, const void* k2, const void* v, void* out,
                       float* lse, int B, int H, int N, int D, const int64_t* strides, int window, int mode,
                       float sm_scale, vqa_stream_t stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Full-context ReRoPE attention: score(i,j) = q1_i.k1_j if |i - j| < window (strict) else q2_i.k2_j; keys j <= i
 * when `causal`, all keys otherwise.  Replaces ops/triton_fused_attn_rerope.py:185-233 (attention).
 * Arguments as vqa_local_attn_* (same 18 strides).  Causal calls of 2048 tokens or more with a window that is a
 * multiple of 64 (head dims 64 / 128) run on the pipelined kernel (0.83 of the general kernel's time at 16k tokens),
 * with the same note on the rounded query as above.
 * ------------------------------------------------------------------------------------------------------------------ */
int vqa_rerope_full_bf16(const void* q1, const void* q2, const void* k1, const void* k2, const void* v, void* out,
                         float* lse, int B, int H, int N, int D, const int64_t* strides, int window, int causal,
                         float sm_scale, vqa_stream_t stream);

int vqa_rerope_full_f16(const void* q1, const void* q2, const void* k1, const void* k2, const void* v, void* out,
                        float* lse, int B, int H, int N, int D, const int64_t* strides, int window, int causal,
                        float sm_scale, vqa_stream_t stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Prefill attention over additive-quantiser key codes with an optional exact sliding window (seqlen_q == seqlen_k).
 * Generalises what vq_attn_forward computes (ops/triton_fused_vq_attn.py:190-251, naive form ops/attn_vq.py:308-333)
 * from one codebook to M, in one fused pass (no separate merge):
 *
 *   keys j <  boundary(i)          quantised:  score = qf_i . sum_m codebooks[h,m,codes[b,h,j,m]],  qf = q2 if given else q
 *   keys boundary(i) <= j < i - W  exact strip: score = q2_i . k2_j when q2 and k2 are given, else q_i . k_exact_j
 *   keys i - W <= j <= i           exact window: score = q_i . k_exact_j
 *   boundary(i) = max(0, floor((i - W)/128)*128)  (boundary_mode 0, the reference's block rule)
 *               = max(0, i - W)                   (boundary_mode 1)
 *   k_exact == NULL: every visible key is quantised (window ignored); causal == 0 requires k_exact == NULL.
 *
 *   strides[0..22]: q(b,h,n) codes(b,h) codebooks(h,m,k) v(b,h,n) k_exact(b,h,n) q2(b,h,n) k2(b,h,n) out(b,h,n);
 *   code rows are packed (stride(n) = M).  M in [1,16], K <= 256, D in {64,128}.
 *   workspace: >= vqa_prefill_workspace_bytes(B,H,N,D) bytes, 256-byte aligned.  On return it holds the reconstructed
 *   keys [B,H,N,D] of every key some query scores as a quantised key: all of them when k_exact == NULL, else the keys
 *   below boundary(N - 1), rounded up to a block of 128 (the rest of the buffer is not written).
 * ------------------------------------------------------------------------------------------------------------------ */
#define VQA_BOUNDARY_BLOCK 0
#define VQA_BOUNDARY_EXACT 1
#define VQA_PREFILL_NUM_STRIDES 23

size_t vqa_prefill_workspace_bytes(int B, int H, int N, int D);

int vqa_prefill_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, const void* k_exact,
                     const void* q2, const void* k2, void* out, float* lse, void* workspace, size_t workspace_bytes,
                     int B, int H, int N, int D, int M, int K, const int64_t* strides, int window, int boundary_mode,
                     int causal, float sm_scale, vqa_stream_t stream);

int vqa_prefill_f16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, const void* k_exact,
                    const void* q2, const void* k2, void* out, float* lse, void* workspace, size_t workspace_bytes,
                    int B, int H, int N, int D, int M, int K, const int64_t* strides, int window, int boundary_mode,
                    int causal, float sm_scale, vqa_stream_t stream);

/* vqa_prefill_* picks between two schedules of the fused kernel:
 *   tiled     -- 128-row query tiles, two workgroups per CU, every combination of arguments;
 *   pipelined -- 256-row query tiles, one wave per SIMD with 64 query rows, the exponentials of a key tile evaluated
 *                under the score MFMAs of the next one; only for the reference's long-prefill configuration: no
 *                second query / key pair, the block boundary rule, `window` a multiple of 128 (or k_exact == NULL:
 *                every key quantised).
 * It takes the pipelined one where it applies and N >= 2048 (measured on MI355X over batch x heads 1 - 256, head dims 64
 * and 128, 1k - 32k tokens: 0.69 - 0.96 of the tiled kernel's time from 2048 tokens on).  The two entry points below force
 * a schedule: vqa_prefill_tiled_* has vqa_prefill_*'s signature; vqa_prefill_pipelined_* returns VQA_ERR_BAD_ARGUMENT
 * where the pipelined schedule does not apply (same strides array, the q2 / k2 slots are ignored).  Same workspace,
 * same results within the 16-bit tolerance.  Counterpart in the reference: the two launches of
 * ops/triton_fused_vq_attn.py:202-245. */
int vqa_prefill_tiled_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v,
                           const void* k_exact, const void* q2, const void* k2, void* out, float* lse, void* workspace,
                           size_t workspace_bytes, int B, int H, int N, int D, int M, int K, const int64_t* strides,
                           int window, int boundary_mode, int causal, float sm_scale, vqa_stream_t stream);

int vqa_prefill_tiled_f16(const void* q, const uint8_t* codes, const void* codebooks, const void* v,
                          const void* k_exact, const void* q2, const void* k2, void* out, float* lse, void* workspace,
                          size_t workspace_bytes, int B, int H, int N, int D, int M, int K, const int64_t* strides,
                          int window, int boundary_mode, int causal, float sm_scale, vqa_stream_t stream);

int vqa_prefill_pipelined_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v,
                               const void* k_exact, void* out, float* lse, void* workspace, size_t workspace_bytes,
                               int B, int H, int N, int D, int M, int K, const int64_t* strides, int window, int causal,
                               float sm_scale, vqa_stream_t stream);

int vqa_prefill_pipelined_f16(const void* q, const uint8_t* codes, const void* codebooks, const void* v,
                              const void* k_exact, void* out, float* lse, void* workspace, size_t workspace_bytes,
                              int B, int H, int N, int D, int M, int K, const int64_t* strides, int window, int causal,
                              float sm_scale, vqa_stream_t stream);

/* fp32 validation instantiation of the prefill: every visible key quantised (no exact window), plain fp32 FMA
 * arithmetic with the lookup-table formulation (LUT[i,m,c] = <q_i, codebooks[h,m,c]>, score = sum_m LUT[i,m,code_jm]);
 * checks the additive-code attention against a dense fp32 softmax to 1e-4.  q, v, out float [B,H,N,D]-addressable,
 * codebooks float [H,M,K,D]; strides[0..13]: q(b,h,n) codes(b,h) codebooks(h,m,k) v(b,h,n) out(b,h,n).  M <= 8.
 * Counterpart of the fp32 branch of the naive reference (softmax in fp32, ops/attn_vq.py:331). */
#define VQA_PREFILL_F32_NUM_STRIDES 14

int vqa_prefill_f32(const float* q, const uint8_t* codes, const float* codebooks, const float* v, float* out,
                    float* lse, int B, int H, int N, int D, int M, int K, const int64_t* strides, int causal,
                    float sm_scale, vqa_stream_t stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Count-weighted far-context kernel of the single-codebook formulation.  Replaces _vq_fwd_kernel
 * (ops/triton_fused_vq_attn.py:88-187) including the host-side zero / -inf initialisation (:214-215):
 * rows i < window + 128 get out = 0, lse = -inf; query tile t (rows window+128+128t ..) attends over the C codewords
 * with cnt[b,h,t,:] and the per-code V prefix sums v_vq[b,h,vi[b,h,t,c],:].
 *
 *   strides[0..16]: q2(b,h,n) k_vq(h,c) k_vq_cnt(b,h,t) v_vq(b,h,n) vi(b,h,t) out(b,h,n); k_vq_cnt has q2's element
 *   type, vi is int64; both have unit stride along c.  lse: [B,H,N] contiguous float, base 2, nullable.
 * ------------------------------------------------------------------------------------------------------------------ */
#define VQA_VQCOUNT_NUM_STRIDES 17

int vqa_vqcount_fwd_bf16(const void* q2, const void* k_vq, const void* k_vq_cnt, const void* v_vq, const int64_t* vi,
                         void* out, float* lse, int B, int H, int N, int D, int C, const int64_t* strides, int window,
                         float sm_scale, vqa_stream_t stream);

int vqa_vqcount_fwd_f16(const void* q2, const void* k_vq, const void* k_vq_cnt, const void* v_vq, const int64_t* vi,
                        void* out, float* lse, int B, int H, int N, int D, int C, const int64_t* strides, int window,
                        float sm_scale, vqa_stream_t stream);

/* Same kernel with the merge fused into its epilogue: out [B,H,N,D] / lse [B,H,N] (contiguous) already hold an
 * attention state (the window kernel's o1, l1) and receive merge((o1, l1), (o2, l2)) in place; rows below window + 128
 * are left untouched.  Replaces the count kernel launch plus the flashinfer merge and its four layout copies
 * (ops/triton_fused_vq_attn.py:222-250) by one launch. */
int vqa_vqcount_merge_bf16(const void* q2, const void* k_vq, const void* k_vq_cnt, const void* v_vq, const int64_t* vi,
                           void* out, float* lse, int B, int H, int N, int D, int C, const int64_t* strides,
                           int window, float sm_scale, vqa_stream_t stream);

int vqa_vqcount_merge_f16(const void* q2, const void* k_vq, const void* k_vq_cnt, const void* v_vq, const int64_t* vi,
                          void* out, float* lse, int B, int H, int N, int D, int C, const int64_t* strides, int window,
                          float sm_scale, vqa_stream_t stream);

/* vqa_vqcount_fwd / vqa_vqcount_merge with the per-block key counts as exact integers (int64 [B,H,NT,C], the dtype in
 * which the reference builds them, ops/attn_vq.py:352-353, before it casts them to the model dtype at :431 -- a cast
 * that rounds bf16 counts above 256).  Same strides array; the k_vq_cnt strides count int64 elements. */
int vqa_vqcount_fwd_icnt_bf16(const void* q2, const void* k_vq, const int64_t* k_vq_cnt, const void* v_vq,
                              const int64_t* vi, void* out, float* lse, int B, int H, int N, int D, int C,
                              const int64_t* strides, int window, float sm_scale, vqa_stream_t stream);

int vqa_vqcount_fwd_icnt_f16(const void* q2, const void* k_vq, const int64_t* k_vq_cnt, const void* v_vq,
                             const int64_t* vi, void* out, float* lse, int B, int H, int N, int D, int C,
                             const int64_t* strides, int window, float sm_scale, vqa_stream_t stream);

int vqa_vqcount_merge_icnt_bf16(const void* q2, const void* k_vq, const int64_t* k_vq_cnt, const void* v_vq,
                                const int64_t* vi, void* out, float* lse, int B, int H, int N, int D, int C,
                                const int64_t* strides, int window, float sm_scale, vqa_stream_t stream);

int vqa_vqcount_merge_icnt_f16(const void* q2, const void* k_vq, const int64_t* k_vq_cnt, const void* v_vq,
                               const int64_t* vi, void* out, float* lse, int B, int H, int N, int D, int C,
                               const int64_t* strides, int window, float sm_scale, vqa_stream_t stream);

/* ------------------------------------------------------------------------------------------------------------------
 * In-place merge of two attention states with base-2 log-sum-exp: m = max(s, s'), o <- (o 2^(s-m) + o' 2^(s'-m)) /
 * (2^(s-m) + 2^(s'-m)), s <- m + log2(2^(s-m) + 2^(s'-m)); a side with s = -inf is ignored.
 * Replaces flashinfer.merge_state_in_place as called at ops/triton_fused_vq_attn.py:246-250.
 *
 *   o, o_other: [B,H,N,D]-addressable; s, s_other: [B,H,N]-addressable float; strides[0..11] = (b,h,n) of
 *   o, s, o_other, s_other.  (flashinfer's [N, B*H, D] / [N, B*H] layout is B = 1, H = B*H with n outermost.)
 * ------------------------------------------------------------------------------------------------------------------ */
#define VQA_MERGE_NUM_STRIDES 12

int vqa_merge_state_inplace_bf16(void* o, float* s, const void* o_other, const float* s_other, int B, int H, int N,
                                 int D, const int64_t* strides, vqa_stream_t stream);

int vqa_merge_state_inplace_f16(void* o, float* s, const void* o_other, const float* s_other, int B, int H, int N,
                                int D, const int64_t* strides, vqa_stream_t stream);

/* vqa_decode with the number of keys read from device memory when the kernels run: *n_keys_dev (clamped to
 * [0, N_max]) keys are attended, N_max is the bound the buffers, the workspace and the split count are sized for.  One
 * recorded launch sequence (a HIP graph of a decode step) can then be replayed while the cache grows.  No counterpart
 * in the reference (its decode route is not functional, ops/attn_vq.py:445-479). */
int vqa_decode_devlen_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, void* out,
                           float* lse, void* workspace, size_t workspace_bytes, int B, int H, int N_max, int D, int M,
                           int K, const int64_t* strides, float sm_scale, int num_splits, const int32_t* n_keys_dev,
                           vqa_stream_t stream);

int vqa_decode_devlen_f16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, void* out,
                          float* lse, void* workspace, size_t workspace_bytes, int B, int H, int N_max, int D, int M,
                          int K, const int64_t* strides, float sm_scale, int num_splits, const int32_t* n_keys_dev,
                          vqa_stream_t stream);

/* vqa_decode for a query that has not been rotated yet: rope_cos / rope_sin are ONE row [D] each of the rotary tables
 * (the row of the position every coded key sees the query at: the clamped ReRoPE position window + 1), 16-byte
 * aligned, and the lookup-table kernel rotates the query as it reads it,
 *     q' = q * cos + rotate_half(q) * sin,  every product and the sum rounded to the element type,
 * bit for bit what vqa_rope_* writes, so a generation step needs no rotary launch for its query.  n_keys_dev as in
 * vqa_decode_devlen_* or NULL (then N_max keys are attended).  Counterpart in the reference: the rotation of the
 * query to `window_length + 1` in front of its (non-functional) seqlen_q == 1 branch, ops/attn_vq.py:445-479. */
int vqa_decode_roped_bf16(const void* q, const void* rope_cos, const void* rope_sin, const uint8_t* codes,
                          const void* codebooks, const void* v, void* out, float* lse, void* workspace,
                          size_t workspace_bytes, int B, int H, int N_max, int D, int M, int K, const int64_t* strides,
                          float sm_scale, int num_splits, const int32_t* n_keys_dev, vqa_stream_t stream);

int vqa_decode_roped_f16(const void* q, const void* rope_cos, const void* rope_sin, const uint8_t* codes,
                         const void* codebooks, const void* v, void* out, float* lse, void* workspace,
                         size_t workspace_bytes, int B, int H, int N_max, int D, int M, int K, const int64_t* strides,
                         float sm_scale, int num_splits, const int32_t* n_keys_dev, vqa_stream_t stream);

/* vqa_decode_bf16 for callers that cannot allocate or hand over device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): no workspace argument, the lookup table and the split states live
 * in a fixed VQA_DECODE_STATIC_SCRATCH_BYTES array inside the library, one copy per GPU, held until the process ends.
 * It has no counterpart in the reference.  Same arguments, kernels and results as vqa_decode_bf16 otherwise.
 *   - a problem whose vqa_decode_workspace_bytes(...) exceeds VQA_DECODE_STATIC_SCRATCH_BYTES is refused with
 *     VQA_ERR_SCRATCH_LIMIT before anything is enqueued;
 *   - the first call on a device looks up the array's device address (hipGetSymbolAddress); make that call outside a
 *     stream capture;
 *   - every call on one GPU uses the same array: calls that may overlap on that GPU (different streams) race, calls
 *     ordered on one stream do not.  Every byte a call reads from the array it has written itself before. */
#define VQA_DECODE_STATIC_SCRATCH_BYTES (8u << 20)

int vqa_decode_static_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, void* out,
                           float* lse, int B, int H, int N, int D, int M, int K, const int64_t* strides, float sm_scale,
                           int num_splits, vqa_stream_t stream);

/* ------------------------------------------------------------------------------------------------------------------
 * seqlen_q = 1 attention over exact keys: out[b,h] = softmax_j(sm_scale * <q[b,h], k[b,h,j]>) . v[b,h,j], no mask.
 * The generation step of the ReRoPE module and the short-context fallback of the VQ module make this call through a
 * third-party flash-attention package in the reference (ops/attn_rerope.py:279-286, ops/attn_vq.py:463-477); with
 * lse it also yields the exact-window state that vqa_merge_state_inplace combines with vqa_decode's far-context state.
 *
 *   q, out [B,H,1,D]; k, v [B,H,N,D]; lse [B,H] (nullable); D in {64,128}.
 *   strides[0..9] = q(b,h) k(b,h,n) v(b,h,n) out(b,h).  Workspace: vqa_decode_exact_workspace_bytes, 256-byte aligned.
 * ------------------------------------------------------------------------------------------------------------------ */
#define VQA_DECODE_EXACT_NUM_STRIDES 10

size_t vqa_decode_exact_workspace_bytes(int B, int H, int N, int D, int num_splits);

int vqa_decode_exact_bf16(const void* q, const void* k, const void* v, void* out, float* lse, void* workspace,
                          size_t workspace_bytes, int B, int H, int N, int D, const int64_t* strides, float sm_scale,
                          int num_splits, vqa_stream_t stream);

int vqa_decode_exact_f16(const void* q, const void* k, const void* v, void* out, float* lse, void* workspace,
                         size_t workspace_bytes, int B, int H, int N, int D, const int64_t* strides, float sm_scale,
                         int num_splits, vqa_stream_t stream);

/* ------------------------------------------------------------------------------------------------------------------
 * seqlen_q = 1 attention with an exact recent window: keys [0, N - W) are scored through their codes with q_far (the
 * position-clamped query of the ReRoPE VQ module), the last W keys exactly with q_win against k_win [B,H,W,D]; v
 * [B,H,N,D] covers both ranges.  The coded and the exact streaming kernels write their split states into one
 * workspace and one merge produces out / lse.  This is the decode-time counterpart of the cache the reference
 * describes (codes for the far context, a window of exact keys: ops/attn_vq.py:31-52, 290-333), which it never got
 * to run at seqlen_q == 1.
 *   strides[0..16] = q_far(b,h) q_win(b,h) codes(b,h) codebooks(h,m,k) v(b,h,n) k_win(b,h,n) out(b,h).
 *   codes may be null when W == N.  Workspace: vqa_decode_windowed_workspace_bytes, 256-byte aligned.
 * ------------------------------------------------------------------------------------------------------------------ */
#define VQA_DECODE_WINDOWED_NUM_STRIDES 17

size_t vqa_decode_windowed_workspace_bytes(int B, int H, int N, int W, int D, int M);

int vqa_decode_windowed_bf16(const void* q_far, const void* q_win, const uint8_t* codes, const void* codebooks,
                             const void* v, const void* k_win, void* out, float* lse, void* workspace,
                             size_t workspace_bytes, int B, int H, int N, int W, int D, int M, int K,
                             const int64_t* strides, float sm_scale, vqa_stream_t stream);

int vqa_decode_windowed_f16(const void* q_far, const void* q_win, const uint8_t* codes, const void* codebooks,
                            const void* v, const void* k_win, void* out, float* lse, void* workspace,
                            size_t workspace_bytes, int B, int H, int N, int W, int D, int M, int K,
                            const int64_t* strides, float sm_scale, vqa_stream_t stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Key encoder: nearest-codeword search of every key against its head's codebooks.
 *   mode 0: id_m = argmax_c <x, codebooks[h,m,c]> for every codebook m independently (inner product, first maximum
 *           on ties) -- replaces multi_head_single_quantize, ops/mini_vq.py:4-18 (M = 1); with round_scores != 0 the
 *           scores are rounded to the element type before the comparison, like the reference's einsum in the model
 *           dtype (ops/mini_vq.py:10-11).
 *   mode 1: greedy residual (additive) encoding in the L2 sense: r = x; id_m = argmax_c (<r, cb[h,m,c]> - |cb|^2/2);
 *           r -= cb[h,m,id_m].  Produces the [B,H,N,M] codes of vqa_decode / vqa_prefill; the reference trains such
 *           codebooks offline (build_quantizer/120_build_additive_quantizer.py:23-32) and has no runtime encoder.
 *
 *   x [B,H,N,D]; codebooks [H,M,K,D], K % 32 == 0; codes [B,H,N,M] uint8 (nullable, needs K <= 256);
 *   ids [B,H,N,M] int64 (nullable); at least one output.  D in {64,128}.
 *   strides[0..11] = x(b,h,n) codebooks(h,m,k) codes(b,h,n) ids(b,h,n); m is innermost in codes and ids.
 * ------------------------------------------------------------------------------------------------------------------ */
#define VQA_ENCODE_NUM_STRIDES 12

int vqa_encode_keys_bf16(const void* x, const void* codebooks, uint8_t* codes, int64_t* ids, int B, int H, int N, int D,
                         int M, int K, const int64_t* strides, int mode, int round_scores, vqa_stream_t stream);

int vqa_encode_keys_f16(const void* x, const void* codebooks, uint8_t* codes, int64_t* ids, int B, int H, int N, int D,
                        int M, int K, const int64_t* strides, int mode, int round_scores, vqa_stream_t stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Inputs of vqa_vqcount_fwd from per-key code ids -- replaces the one-hot cumulative sum, argsort and global prefix
 * sum of ops/attn_vq.py:352-384 and the block sampling at :410-413:
 *   cnt[t,c] = #{j < (t+1)*128 : id_j == c}, t < N/128;   vi[t,c] = cnt[t,c] + #{j < N : id_j < c};
 *   v_vq[0] = 0, v_vq[1+r] = running sum of V over the keys of r's code in (code, position) order up to row r
 *   (fp32 running sum per code, rounded to the element type).
 *
 *   ids [B,H,N] int64 (values outside [0, C) are clamped); v [B,H,N,D]; cnt [B,H,N/128,C] int64 (nullable);
 *   cnt_elem: the same counts in the element type, as vqa_vqcount_fwd reads them (nullable); v_vq [B,H,N+1,D];
 *   vi [B,H,N/128,C] int64 (may be null when N < 128).  C <= 8192, D even and <= 128.
 *   strides[0..17] = ids(b,h,n) v(b,h,n) cnt(b,h,t) cnt_elem(b,h,t) v_vq(b,h,n) vi(b,h,t).
 * ------------------------------------------------------------------------------------------------------------------ */
#define VQA_PREPROCESS_NUM_STRIDES 18

size_t vqa_preprocess_workspace_bytes(int B, int H, int N, int C);

int vqa_preprocess_bf16(const int64_t* ids, const void* v, int64_t* cnt, void* cnt_elem, void* v_vq, int64_t* vi,
                        void* workspace, size_t workspace_bytes, int B, int H, int N, int D, int C,
                        const int64_t* strides, vqa_stream_t stream);

int vqa_preprocess_f16(const int64_t* ids, const void* v, int64_t* cnt, void* cnt_elem, void* v_vq, int64_t* vi,
                       void* workspace, size_t workspace_bytes, int B, int H, int N, int D, int C,
                       const int64_t* strides, vqa_stream_t stream);

/* The same preprocessing that also leaves the count state of the whole sequence -- what vqa_count_state_add_* (below)
 * builds from the same ids and values, bit for bit: state_cnt[b,h,c] = #{j : id_j == c} (int32, [B,H,C] contiguous),
 * state_vsum[b,h,c,:] = sum of v over those keys in position order (fp32, [B,H,C,D] contiguous, 8-byte aligned).  Both
 * are overwritten, not accumulated.  The walk over each code's keys ends with these totals anyway, so a prefill that
 * needs both the count-kernel inputs and the generation-step state gets the state for nothing (a separate fold of
 * 8192 keys costs ~190 us).  Counterpart in the reference: `update_prefill`, ops/attn_vq.py:89-127. */
int vqa_preprocess_state_bf16(const int64_t* ids, const void* v, int64_t* cnt, void* cnt_elem, void* v_vq, int64_t* vi,
                              int32_t* state_cnt, float* state_vsum, void* workspace, size_t workspace_bytes, int B,
                              int H, int N, int D, int C, const int64_t* strides, vqa_stream_t stream);

int vqa_preprocess_state_f16(const int64_t* ids, const void* v, int64_t* cnt, void* cnt_elem, void* v_vq, int64_t* vi,
                             int32_t* state_cnt, float* state_vsum, void* workspace, size_t workspace_bytes, int B,
                             int H, int N, int D, int C, const int64_t* strides, vqa_stream_t stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Rotary position embedding in the model's 16-bit type: out = x * cos[pos] + rotate_half(x) * sin[pos] with
 * rotate_half(x) = cat(-x[D/2:], x[:D/2]); each product and the sum are rounded to the element type, so the result
 * equals the operator-by-operator evaluation on 16-bit tensors that the reference's callers perform
 * (apply_rotary_pos_emb and the clamped query at ops/attn_vq.py:402-407; ops/attn_rerope.py:160-180).
 *
 *   x, out [B,H,N,D]; position_ids [B,N] int64, or null to rotate every row to `fixed_pos`; cos, sin [n_pos, D] with
 *   row stride table_stride.  out_fixed (nullable, only with position_ids; addressed with out's strides) receives the
 *   same rows rotated to `fixed_pos` from the same pass over x -- the clamped ReRoPE query next to the true-position
 *   one.  D % 16 == 0.  strides[0..7] = x(b,h,n) position_ids(b,n) out(b,h,n).
 * ------------------------------------------------------------------------------------------------------------------ */
#define VQA_ROPE_NUM_STRIDES 8

int vqa_rope_bf16(const void* x, const int64_t* position_ids, const void* cos, const void* sin, void* out,
                  void* out_fixed, int B, int H, int N, int D, int n_pos, int64_t table_stride, const int64_t* strides,
                  int fixed_pos, vqa_stream_t stream);

int vqa_rope_f16(const void* x, const int64_t* position_ids, const void* cos, const void* sin, void* out,
                 void* out_fixed, int B, int H, int N, int D, int n_pos, int64_t table_stride, const int64_t* strides,
                 int fixed_pos, vqa_stream_t stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Count state of a single-codebook key cache and the generation step over it.  With one codebook a quantised key IS a
 * codeword, so attention over N quantised keys equals attention over the C codewords with weights:
 *     sum_j exp(q.cb[id_j]) v_j = sum_c exp(q.cb[c]) Vsum[c],      Z = sum_c cnt[c] exp(q.cb[c]).
 * (cnt, Vsum) is the state the reference's cache stores after a prefill -- key counts and cumulated values,
 * ops/attn_vq.py:89-127 -- for the seqlen_q == 1 route it leaves unimplemented (ops/attn_vq.py:176-223, 445-479).
 * A step costs O(C D) whatever the context length.
 *
 *   vqa_count_state_add: fold T keys into the state, cnt[b,h,ids[b,h,t]] += 1 and Vsum[b,h,ids[b,h,t],:] += v[b,h,t,:]
 *     (fp32 sums in position order, no atomics: results are reproducible).  ids [B,H,T] int64 (entries outside [0, C)
 *     are clamped into it, as everywhere in this library), v [B,H,T,D]; cnt [B,H,C] int32 and vsum [B,H,C,D] fp32 contiguous, zeroed by the caller before the
 *     first call.  strides[0..5] = ids(b,h,t) v(b,h,t).  D in {64, 128}.
 *   vqa_count_decode: out[b,h,:] = sum_c e_c Vsum[b,h,c,:] / Z with e_c = exp(q[b,h].cb[h,c] * sm_scale) for the
 *     codewords with cnt > 0; lse (nullable, [B,H] fp32) = log2 Z, -inf for an empty state (out = 0) -- the pair is an
 *     attention state that vqa_merge_state_inplace combines with the state of an exact window.
 *     q, out [B,H,D]; codebook [H,C,D]; strides[0..5] = q(b,h) codebook(h,c) out(b,h).  C <= VQA_COUNT_STATE_MAX_CODES.
 * ------------------------------------------------------------------------------------------------------------------ */
#define VQA_COUNT_STATE_MAX_CODES 8192
#define VQA_COUNT_STATE_NUM_STRIDES 6

int vqa_count_state_add_bf16(const int64_t* ids, const void* v, int32_t* cnt, float* vsum, int B, int H, int T, int D,
                             int C, const int64_t* strides, vqa_stream_t stream);

int vqa_count_state_add_f16(const int64_t* ids, const void* v, int32_t* cnt, float* vsum, int B, int H, int T, int D,
                            int C, const int64_t* strides, vqa_stream_t stream);

int vqa_count_decode_bf16(const void* q, const void* codebook, const int32_t* cnt, const float* vsum, void* out,
                          float* lse, int B, int H, int C, int D, const int64_t* strides, float sm_scale,
                          vqa_stream_t stream);

int vqa_count_decode_f16(const void* q, const void* codebook, const int32_t* cnt, const float* vsum, void* out,
                         float* lse, int B, int H, int C, int D, const int64_t* strides, float sm_scale,
                         vqa_stream_t stream);

/*   vqa_count_step: one launch for a whole generation step on the state -- what vqa_count_state_add_* (T = 1),
 *     vqa_rope_* and vqa_count_decode_* do in three, bit for bit: the new key (codeword id [B,H] int64, clamped; value v
 *     [B,H,D]) is folded into cnt / vsum, the RAW query is rotated to the position of rope_cos / rope_sin (one [D] row
 *     each, 4-byte aligned; both NULL: the query comes rotated) and attends over the updated state.
 *     strides[0..9] = q(b,h) codebook(h,c) out(b,h) id(b,h) v(b,h).  A generation step of the reference's VQ module is
 *     then two launches (the codeword search for the new key, this), where five separate ones are host-bound. */
int vqa_count_step_bf16(const void* q, const void* rope_cos, const void* rope_sin, const int64_t* id, const void* v,
                        const void* codebook, int32_t* cnt, float* vsum, void* out, float* lse, int B, int H, int C,
                        int D, const int64_t* strides, float sm_scale, vqa_stream_t stream);

int vqa_count_step_f16(const void* q, const void* rope_cos, const void* rope_sin, const int64_t* id, const void* v,
                       const void* codebook, int32_t* cnt, float* vsum, void* out, float* lse, int B, int H, int C,
                       int D, const int64_t* strides, float sm_scale, vqa_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* VQATTN_H */
