// fp32 validation instantiation of the additive-code prefill (every visible key quantised, causal optional).
//
// Plain FMA arithmetic, no matrix cores: this entry point exists to check the lookup-table formulation to 1e-4
// against a dense softmax, not to be fast.  A workgroup owns RB consecutive queries: it first builds their lookup
// table LUT[row][m][c] = <q_row, codebooks[h,m,c]> in LDS, then each wave walks the keys of one row at a time in
// chunks of 1024: scores (lane = key, M table lookups), online base-2 softmax across chunks, and P.V with lane = d.
#include "vqa_common.h"

namespace vqa {
namespace prefill_f32 {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kChunk = 1024;  // keys scored per pass of a wave

struct Params {
    const float* q;
    const uint8_t* codes;
    const float* cb;
    const float* v;
    float* out;
    float* lse;
    int64_t q_sb, q_sh, q_sn;
    int64_t c_sb, c_sh;
    int64_t cb_sh, cb_sm, cb_sk;
    int64_t v_sb, v_sh, v_sn;
    int64_t o_sb, o_sh, o_sn;
    int H, N, M, K, RB, causal;
    float scale_log2e;
};

template <int D>
__global__ __launch_bounds__(kThreads) void kernel(Params p) {
    extern __shared__ float smem[];
    float* s_lut = smem;                                   // [RB][M][256]
    float* s_q = s_lut + p.RB * p.M * 256;                 // [RB][D]
    float* s_p = s_q + p.RB * D;                           // [kWaves][kChunk]
    constexpr int DPL = D / 64;                            // output elements per lane

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bh = blockIdx.y;
    const int b = bh / p.H, h = bh % p.H;
    const int row0 = blockIdx.x * p.RB;
    const int n_rows = min(p.RB, p.N - row0);

    const float* q = p.q + b * p.q_sb + h * p.q_sh;
    const float* cb = p.cb + h * p.cb_sh;
    const float* v = p.v + b * p.v_sb + h * p.v_sh;
    const uint8_t* codes = p.codes + b * p.c_sb + h * p.c_sh;

    for (int i = tid; i < n_rows * D; i += kThreads) s_q[i] = q[(int64_t)(row0 + i / D) * p.q_sn + i % D];
    __syncthreads();
    // lookup table: thread t owns codewords t, t+256, ... of the M*K list, for every row of the block
    for (int e = tid; e < p.M * p.K; e += kThreads) {
        const int m = e / p.K, c = e % p.K;
        const float* w = cb + m * p.cb_sm + (int64_t)c * p.cb_sk;
        for (int r = 0; r < n_rows; ++r) {
            float acc = 0.f;
#pragma unroll 8
            for (int d = 0; d < D; ++d) acc = __builtin_fmaf(s_q[r * D + d], w[d], acc);
            s_lut[(r * p.M + m) * 256 + c] = acc * p.scale_log2e;
        }
    }
    __syncthreads();

    float* my_p = s_p + wave * kChunk;
    for (int r = wave; r < n_rows; r += kWaves) {
        const int i = row0 + r;
        const int n_keys = p.causal ? i + 1 : p.N;
        const float* lut = s_lut + r * p.M * 256;
        float m_run = -INFINITY, l_run = 0.f;
        float acc[DPL];
#pragma unroll
        for (int e = 0; e < DPL; ++e) acc[e] = 0.f;
        for (int j0 = 0; j0 < n_keys; j0 += kChunk) {
            const int cn = min(kChunk, n_keys - j0);
            float mx = -INFINITY;
            for (int j = lane; j < cn; j += 64) {
                const uint8_t* code = codes + (int64_t)(j0 + j) * p.M;
                float s = 0.f;
                for (int m = 0; m < p.M; ++m) s += lut[m * 256 + code[m]];
                my_p[j] = s;
                mx = fmaxf(mx, s);
            }
            mx = wave_max(mx);
            const float m_new = fmaxf(m_run, mx);
            const float alpha = exp2f(m_run - m_new);  // 0 on the first chunk
            float sum = 0.f;
            for (int j = lane; j < cn; j += 64) {
                const float pj = exp2f(my_p[j] - m_new);
                my_p[j] = pj;
                sum += pj;
            }
            sum = wave_sum(sum);
            l_run = l_run * alpha + sum;
            m_run = m_new;
            wave_lds_sync();
#pragma unroll
            for (int e = 0; e < DPL; ++e) acc[e] *= alpha;
            const float* vrow = v + (int64_t)j0 * p.v_sn + lane;
            for (int j = 0; j < cn; ++j) {
                const float pj = my_p[j];
#pragma unroll
                for (int e = 0; e < DPL; ++e) acc[e] = __builtin_fmaf(pj, vrow[e * 64], acc[e]);
                vrow += p.v_sn;
            }
            wave_lds_sync();
        }
        float* o = p.out + b * p.o_sb + h * p.o_sh + (int64_t)i * p.o_sn + lane;
        const float inv = 1.f / l_run;
#pragma unroll
        for (int e = 0; e < DPL; ++e) o[e * 64] = acc[e] * inv;
        if (p.lse && lane == 0) p.lse[(int64_t)bh * p.N + i] = m_run + log2f(l_run);
    }
}

}  // namespace prefill_f32
}  // namespace vqa

extern "C" int vqa_prefill_f32(const float* q, const uint8_t* codes, const float* codebooks, const float* v, float* out,
                               float* lse, int B, int H, int N, int D, int M, int K, const int64_t* strides, int causal,
                               float sm_scale, vqa_stream_t stream) {
    using namespace vqa::prefill_f32;
    if (!q || !codes || !codebooks || !v || !out || !strides) return VQA_ERR_NULL_POINTER;
    if (B <= 0 || H <= 0 || N <= 0) return VQA_ERR_BAD_SHAPE;
    if (D != 64 && D != 128) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    if (M < 1 || M > 8 || K < 1 || K > 256) return VQA_ERR_UNSUPPORTED_CODEBOOK;
    if ((int64_t)B * H > 65535 || !(sm_scale > 0.f)) return VQA_ERR_BAD_ARGUMENT;
    Params p;
    p.q = q, p.codes = codes, p.cb = codebooks, p.v = v, p.out = out, p.lse = lse;
    p.q_sb = strides[0], p.q_sh = strides[1], p.q_sn = strides[2];
    p.c_sb = strides[3], p.c_sh = strides[4];
    p.cb_sh = strides[5], p.cb_sm = strides[6], p.cb_sk = strides[7];
    p.v_sb = strides[8], p.v_sh = strides[9], p.v_sn = strides[10];
    p.o_sb = strides[11], p.o_sh = strides[12], p.o_sn = strides[13];
    p.H = H, p.N = N, p.M = M, p.K = K, p.causal = causal;
    p.RB = 32 / M < 16 ? 32 / M : 16;  // lookup table of the block stays within 32 KB of LDS
    p.scale_log2e = sm_scale * vqa::kLog2e;
    const size_t smem = ((size_t)p.RB * M * 256 + (size_t)p.RB * D + kWaves * kChunk) * sizeof(float);
    const dim3 grid((N + p.RB - 1) / p.RB, B * H);
    if (D == 64)
        hipLaunchKernelGGL((kernel<64>), grid, dim3(kThreads), smem, stream, p);
    else
        hipLaunchKernelGGL((kernel<128>), grid, dim3(kThreads), smem, stream, p);
    return vqa::launch_status();
}
