// Key encoder: nearest-codeword search of every key against its head's codebooks on the matrix cores.
//
//   mode 0 (inner product):   id_m = argmax_c <x, cb[h,m,c]>                       for every codebook m independently
//   mode 1 (greedy residual): r = x;  id_m = argmax_c (<r, cb[h,m,c]> - |cb[h,m,c]|^2 / 2);  r -= cb[h,m,id_m]
//
// One workgroup = 4 waves x 32 keys of one (batch, head).  Scores are computed transposed, S^T = CB . R^T, with the
// codebook chunk (128 codewords, staged in LDS) as the A operand and the keys as the B operand, so a lane owns one key
// and sees 16 codeword scores per 32x32 block: the running argmax lives in registers.  The residual is kept in fp32 and
// fed to the 16-bit MFMA as a (high, low) pair of 16-bit values, which reproduces fp32 inner products to ~2^-16.
#include "vqa_common.h"

namespace vqa {
namespace encode {

constexpr int kThreads = 256;
constexpr int kKeysPerBlock = 128;
constexpr int kChunk = 128;  // codewords staged per pass

struct Params {
    const uint16_t* x;
    int64_t x_sb, x_sh, x_sn;
    const uint16_t* cb;
    int64_t cb_sh, cb_sm, cb_sk;
    uint8_t* codes;
    int64_t c_sb, c_sh, c_sn;
    int64_t* ids;
    int64_t i_sb, i_sh, i_sn;
    int H, N, M, K;
    int mode, round_scores;
};

template <typename Tag, int D>
__global__ __launch_bounds__(kThreads) void encode_kernel(Params p) {
    typedef typename Elem<Tag>::vec8 vec8;
    constexpr int kSteps = D / 16;      // MFMA k-steps
    constexpr int kRowElems = D + 8;    // padded LDS row: 16-byte reads of 16 consecutive rows hit distinct banks
    constexpr int kChunksPerRow = D / 8;
    __shared__ __attribute__((aligned(16))) uint16_t s_cb[kChunk * kRowElems];
    __shared__ float s_norm[kChunk];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int half = lane >> 5;
    const int bh = blockIdx.y;
    const int b = bh / p.H, h = bh % p.H;
    const int key = blockIdx.x * kKeysPerBlock + wave * 32 + (lane & 31);
    const int key_c = min(key, p.N - 1);

    // this lane's slice of its key: elements ks*16 + half*8 + [0, 8)
    float r[kSteps * 8];
    {
        const uint16_t* xp = p.x + b * p.x_sb + h * p.x_sh + (int64_t)key_c * p.x_sn + half * 8;
#pragma unroll
        for (int ks = 0; ks < kSteps; ++ks) {
            const uint4 w = *reinterpret_cast<const uint4*>(xp + ks * 16);
            const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                r[ks * 8 + 2 * e] = Elem<Tag>::from_bits((uint16_t)(ww[e] & 0xffffu));
                r[ks * 8 + 2 * e + 1] = Elem<Tag>::from_bits((uint16_t)(ww[e] >> 16));
            }
        }
    }

    for (int m = 0; m < p.M; ++m) {
        const uint16_t* cbm = p.cb + h * p.cb_sh + m * p.cb_sm;
        const bool with_low = p.mode == 1 && m > 0;  // the residual is no longer a 16-bit value after one subtraction

        // split the fp32 residual into the two 16-bit MFMA operands
        vec8 hi[kSteps], lo[kSteps];
#pragma unroll
        for (int ks = 0; ks < kSteps; ++ks) {
            uint32_t wh[4], wl[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float a0 = r[ks * 8 + 2 * e], a1 = r[ks * 8 + 2 * e + 1];
                const float h0 = Elem<Tag>::round_keep_f32(a0), h1 = Elem<Tag>::round_keep_f32(a1);
                wh[e] = Elem<Tag>::pack2(h0, h1);
                wl[e] = Elem<Tag>::pack2(a0 - h0, a1 - h1);
            }
            const uint4 vh = make_uint4(wh[0], wh[1], wh[2], wh[3]);
            const uint4 vl = make_uint4(wl[0], wl[1], wl[2], wl[3]);
            hi[ks] = __builtin_bit_cast(vec8, vh);
            lo[ks] = __builtin_bit_cast(vec8, vl);
        }

        float best = -INFINITY;
        int best_i = 0;
        for (int c0 = 0; c0 < p.K; c0 += kChunk) {
            const int rows = min(kChunk, p.K - c0);
            __syncthreads();  // the previous chunk is no longer read
            for (int i = tid; i < rows * kChunksPerRow; i += kThreads) {
                const int row = i / kChunksPerRow, col = i % kChunksPerRow;
                *reinterpret_cast<uint4*>(&s_cb[row * kRowElems + col * 8]) =
                    *reinterpret_cast<const uint4*>(cbm + (int64_t)(c0 + row) * p.cb_sk + col * 8);
            }
            __syncthreads();
            if (p.mode == 1) {
                if (tid < rows) {
                    float acc = 0.f;
                    for (int d = 0; d < D; ++d) {
                        const float cv = Elem<Tag>::from_bits(s_cb[tid * kRowElems + d]);
                        acc += cv * cv;
                    }
                    s_norm[tid] = 0.5f * acc;
                }
                __syncthreads();
            }
            for (int blk = 0; blk * 32 < rows; ++blk) {
                f32x16_t acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                const uint16_t* ap = &s_cb[(blk * 32 + (lane & 31)) * kRowElems + half * 8];
#pragma unroll
                for (int ks = 0; ks < kSteps; ++ks) {
                    const vec8 a = *reinterpret_cast<const vec8*>(ap + ks * 16);
                    acc = Elem<Tag>::mfma32(a, hi[ks], acc);
                    if (with_low) acc = Elem<Tag>::mfma32(a, lo[ks], acc);
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int cl = blk * 32 + 8 * (e / 4) + 4 * half + (e % 4);  // codeword within the chunk
                    float s = acc[e];
                    if (p.mode == 1) s -= s_norm[cl];
                    if (p.round_scores) s = Elem<Tag>::round_keep_f32(s);
                    if (s > best) {  // a lane visits its codewords in increasing order: the first maximum stays
                        best = s;
                        best_i = c0 + cl;
                    }
                }
            }
        }
        // the two half-waves hold disjoint codewords of the same key
        const float o_s = __shfl_xor(best, 32, 64);
        const int o_i = __shfl_xor(best_i, 32, 64);
        if (o_s > best || (o_s == best && o_i < best_i)) {
            best = o_s;
            best_i = o_i;
        }
        if (half == 0 && key < p.N) {
            if (p.codes) p.codes[b * p.c_sb + h * p.c_sh + (int64_t)key * p.c_sn + m] = (uint8_t)best_i;
            if (p.ids) p.ids[b * p.i_sb + h * p.i_sh + (int64_t)key * p.i_sn + m] = best_i;
        }
        if (p.mode == 1 && m + 1 < p.M) {
            const uint16_t* cp = cbm + (int64_t)best_i * p.cb_sk + half * 8;
#pragma unroll
            for (int ks = 0; ks < kSteps; ++ks) {
                const uint4 w = *reinterpret_cast<const uint4*>(cp + ks * 16);
                const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    r[ks * 8 + 2 * e] -= Elem<Tag>::from_bits((uint16_t)(ww[e] & 0xffffu));
                    r[ks * 8 + 2 * e + 1] -= Elem<Tag>::from_bits((uint16_t)(ww[e] >> 16));
                }
            }
        }
    }
}

// strides: x(b,h,n) codebooks(h,m,k) codes(b,h,n) ids(b,h,n); last dims contiguous (codes / ids: m innermost)
template <typename Tag>
int encode(const void* x, const void* codebooks, uint8_t* codes, int64_t* ids, int B, int H, int N, int D, int M, int K,
           const int64_t* strides, int mode, int round_scores, hipStream_t stream) {
    if (!x || !codebooks || !strides || (!codes && !ids)) return VQA_ERR_NULL_POINTER;
    if (B <= 0 || H <= 0 || N <= 0 || M <= 0 || K <= 0 || (K % 32) != 0) return VQA_ERR_BAD_SHAPE;
    if (mode != 0 && mode != 1) return VQA_ERR_BAD_ARGUMENT;
    if (codes && K > 256) return VQA_ERR_BAD_ARGUMENT;  // a uint8 code cannot name more than 256 codewords
    if ((int64_t)B * H > 65535) return VQA_ERR_BAD_ARGUMENT;
    Params p;
    p.x = static_cast<const uint16_t*>(x);
    p.x_sb = strides[0], p.x_sh = strides[1], p.x_sn = strides[2];
    p.cb = static_cast<const uint16_t*>(codebooks);
    p.cb_sh = strides[3], p.cb_sm = strides[4], p.cb_sk = strides[5];
    p.codes = codes;
    p.c_sb = strides[6], p.c_sh = strides[7], p.c_sn = strides[8];
    p.ids = ids;
    p.i_sb = strides[9], p.i_sh = strides[10], p.i_sn = strides[11];
    p.H = H, p.N = N, p.M = M, p.K = K;
    p.mode = mode, p.round_scores = round_scores;
    if (!aligned16(x) || !aligned16(codebooks) || ((p.x_sb | p.x_sh | p.x_sn | p.cb_sh | p.cb_sm | p.cb_sk) & 7))
        return VQA_ERR_MISALIGNED;
    const dim3 grid((N + kKeysPerBlock - 1) / kKeysPerBlock, B * H);
    switch (D) {
        case 16: hipLaunchKernelGGL((encode_kernel<Tag, 16>), grid, dim3(kThreads), 0, stream, p); break;
        case 32: hipLaunchKernelGGL((encode_kernel<Tag, 32>), grid, dim3(kThreads), 0, stream, p); break;
        case 64: hipLaunchKernelGGL((encode_kernel<Tag, 64>), grid, dim3(kThreads), 0, stream, p); break;
        case 128: hipLaunchKernelGGL((encode_kernel<Tag, 128>), grid, dim3(kThreads), 0, stream, p); break;
        default: return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    }
    return launch_status();
}

}  // namespace encode
}  // namespace vqa

extern "C" {

int vqa_encode_keys_bf16(const void* x, const void* codebooks, uint8_t* codes, int64_t* ids, int B, int H, int N, int D,
                         int M, int K, const int64_t* strides, int mode, int round_scores, vqa_stream_t stream) {
    return vqa::encode::encode<vqa::bf16_tag>(x, codebooks, codes, ids, B, H, N, D, M, K, strides, mode, round_scores,
                                              stream);
}

int vqa_encode_keys_f16(const void* x, const void* codebooks, uint8_t* codes, int64_t* ids, int B, int H, int N, int D,
                        int M, int K, const int64_t* strides, int mode, int round_scores, vqa_stream_t stream) {
    return vqa::encode::encode<vqa::f16_tag>(x, codebooks, codes, ids, B, H, N, D, M, K, strides, mode, round_scores,
                                             stream);
}

}  // extern "C"
