// Key encoder: nearest-codeword search of every key against its head's codebooks on the matrix cores.
//
//   mode 0 (inner product):   id_m = argmax_c <x, cb[h,m,c]>                       for every codebook m independently
//   mode 1 (greedy residual): r = x;  id_m = argmax_c (<r, cb[h,m,c]> - |cb[h,m,c]|^2 / 2);  r -= cb[h,m,id_m]
//
// One workgroup = 4 waves x 32 keys of one (batch, head).  The codebooks stream through LDS in 64-codeword tiles with
// the attention kernels' machinery (direct-to-LDS copies, XOR-swizzled rows, double buffering across tiles and
// stages), and the scores are the same transposed product S^T = CB_tile . R^T: a lane owns one key and sees 2 x 16
// codeword scores per tile, in increasing codeword order, so the running arg-max is two registers and the first
// maximum wins ties.  The residual is kept in fp32 and fed to the 16-bit MFMA as a (high, low) pair of 16-bit
// values, which reproduces fp32 inner products to ~2^-16.
#include "vqa_flash.h"

namespace vqa {
namespace encode {

using flash::kBN;
constexpr int kThreads = 256;
constexpr int kKeysPerBlock = 128;

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
__global__ __launch_bounds__(kThreads, 2) void encode_kernel(Params p) {
    typedef flash::Geom<D> G;
    typedef typename Elem<Tag>::vec8 vec8;
    constexpr int kSteps = D / 16;
    __shared__ __attribute__((aligned(1024))) char s_cb[2][G::kTileBytes];
    __shared__ __attribute__((aligned(16))) float s_norm[kBN];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;
    const int bh = blockIdx.y;
    const int b = bh / p.H, h = bh % p.H;
    const int key = blockIdx.x * kKeysPerBlock + wave * 32 + (lane & 31);
    const int key_c = min(key, p.N - 1);
    const uint16_t* cb_h = p.cb + h * p.cb_sh;

    flash::TileCopy<D, false> copy;
    copy.init(wave, lane);
    const int tiles_per_stage = (p.K + kBN - 1) / kBN;
    const int n_tiles = p.M * tiles_per_stage;
    auto request = [&](int idx, int buf) {  // tile idx = (codebook m, 64-codeword tile t); rows past K repeat row K-1
        const int m = idx / tiles_per_stage, t = idx % tiles_per_stage;
        copy.load(s_cb[buf], cb_h + m * p.cb_sm, p.cb_sk, t * kBN, p.K);
    };
    request(0, 0);

    // this lane's slice of its key: elements ks*16 + half*8 + [0, 8), the B-operand layout of the score product
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

    int idx = 0;
    for (int m = 0; m < p.M; ++m) {
        const uint16_t* cbm = cb_h + m * p.cb_sm;
        const bool with_low = p.mode == 1 && m > 0;  // the residual is no longer a 16-bit value after one subtraction

        // split the fp32 residual into the two 16-bit MFMA operands
        flash::QFrag<Tag, D> hi, lo;
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
            const flash::u32x4_t vh = {wh[0], wh[1], wh[2], wh[3]};
            const flash::u32x4_t vl = {wl[0], wl[1], wl[2], wl[3]};
            hi.f[ks] = __builtin_bit_cast(vec8, vh);
            lo.f[ks] = __builtin_bit_cast(vec8, vl);
        }

        float best = -INFINITY;
        int best_i = 0;
        for (int t = 0; t < tiles_per_stage; ++t, ++idx) {
            const int buf = idx & 1;
            flash::wait_tile_loads();
            __syncthreads();  // tile idx is complete in `buf`; every wave is done with the other buffer and s_norm
            if (idx + 1 < n_tiles) request(idx + 1, buf ^ 1);
            if (p.mode == 1) {
                // |c|^2 / 2 of the tile's 64 codewords: 4 threads per row, 16-byte chunks through the row swizzle
                constexpr int kCPT = G::kChunksPerRow / 4;  // chunks per thread
                const int row = tid >> 2, part = tid & 3;
                float acc = 0.f;
#pragma unroll
                for (int j = 0; j < kCPT; ++j) {
                    const int chunk = (part * kCPT + j) ^ G::swz_k(row);
                    const flash::u32x4_t w = *reinterpret_cast<const flash::u32x4_t*>(
                        &s_cb[buf][row * G::kRowBytes + chunk * 16]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float lo16 = Elem<Tag>::from_bits((uint16_t)(w[e] & 0xffffu));
                        const float hi16 = Elem<Tag>::from_bits((uint16_t)(w[e] >> 16));
                        acc += lo16 * lo16 + hi16 * hi16;
                    }
                }
                acc += __shfl_xor(acc, 1, 64);
                acc += __shfl_xor(acc, 2, 64);
                if (part == 0) s_norm[row] = 0.5f * acc;
                __syncthreads();
            }
            f32x16_t s[2];
            flash::qk_mma<Tag, D>(s, hi, s_cb[buf], lane);
            if (with_low) {
                f32x16_t s2[2];
                flash::qk_mma<Tag, D>(s2, lo, s_cb[buf], lane);
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int e = 0; e < 16; ++e) s[kb][e] += s2[kb][e];
            }
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    // registers 4g .. 4g+3 of block kb are codewords kb*32 + 8g + 4*half + 0..3 of the tile
                    const int cl0 = kb * 32 + 8 * g + 4 * half;
                    f32x4_t nrm = {0.f, 0.f, 0.f, 0.f};
                    if (p.mode == 1) nrm = *reinterpret_cast<const f32x4_t*>(&s_norm[cl0]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float sc = s[kb][4 * g + e] - nrm[e];
                        if (p.round_scores) sc = Elem<Tag>::round_keep_f32(sc);
                        const int c = t * kBN + cl0 + e;
                        if (c < p.K && sc > best) {  // a lane meets its codewords in increasing order: first maximum
                            best = sc;
                            best_i = c;
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
    if (!row_stride_ok(p.cb_sk)) return VQA_ERR_BAD_ARGUMENT;
    if (!aligned16(x) || !aligned16(codebooks) || ((p.x_sb | p.x_sh | p.x_sn | p.cb_sh | p.cb_sm | p.cb_sk) & 7))
        return VQA_ERR_MISALIGNED;
    const dim3 grid((N + kKeysPerBlock - 1) / kKeysPerBlock, B * H);
    switch (D) {
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
