/*
 * libvqattn_gfx950 -- C ABI of the MI355X (gfx950) fused VQ-attention kernels.
 *
 * This is the boundary a host binds instead of the reference's Triton launches.  Every entry point
 *   - takes plain device pointers, sizes and element strides (no torch types),
 *   - enqueues its kernels on the given HIP stream and returns without synchronising,
 *   - allocates nothing and keeps no mutable global state (scratch comes in through `workspace`),
 *   - returns VQA_OK (0) or a negative vqa_status; it never throws or aborts.
 * Tensors are addressed as base + sum(index_i * stride_i) in ELEMENTS of their own type; the innermost
 * (head_dim / codebook index M) stride must be 1.  Head dims: 64 and 128.
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
    VQA_ERR_LAUNCH_FAILED = -8
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
 *   M in {1,2,4,8}, K <= 256, D in {64,128}.
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

#ifdef __cplusplus
}
#endif
#endif /* VQATTN_H */
