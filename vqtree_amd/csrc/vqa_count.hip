// Count-weighted softmax over codewords (single-codebook far context) and the base-2 log-sum-exp state merge.
//
// count kernel: query tile t covers rows [W + T + t*T, W + T + (t+1)*T) and attends over the C codewords of its
// head: score_c = q2 . codebook[c]; codewords that no key up to block t uses (cnt == 0) are masked; the numerator
// sums P . v_vq[vi[t, c]] (per-code running sums of V), the denominator weights exp by cnt[t, c].
#include <mutex>

#include "vqa_flash.h"

namespace vqa {
namespace flash {

struct CountParams {
    View q;                 // q2 [B,H,N,D]
    const uint16_t* cb;     // [H,C,D]
    int64_t cb_sh, cb_sc;
    const uint16_t* cnt;    // [B,H,NT,C] in the element type, or
    const int64_t* cnt_i64;  // the same as exact integers (then cnt is null); same strides
    int64_t cnt_sb, cnt_sh, cnt_st;
    View vvq;               // [B,H,N+1,D]
    const int64_t* vi;      // [B,H,NT,C]
    int64_t vi_sb, vi_sh, vi_st;
    uint16_t* out;
    int64_t o_sb, o_sh, o_sn;
    float* lse;             // [B,H,N]
    int H, N, C, window, n_far_tiles;
    int merge_into;  // out / lse already hold an attention state: merge this kernel's state into it
    float scale_log2e;
};

template <typename Tag, int D>
__global__ __launch_bounds__(kThreads, 2) void count_kernel(CountParams p) {
    typedef Geom<D> G;
    typedef typename Elem<Tag>::vec8 vec8;
    // dynamic LDS (4 tiles + 2 x 64 counts is 512 bytes past the 64 KB static limit at D = 128):
    // K tiles | V tiles | counts, each double-buffered
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    char(*s_k)[G::kTileBytes] = reinterpret_cast<char(*)[G::kTileBytes]>(smem);
    char(*s_v)[G::kTileBytes] = reinterpret_cast<char(*)[G::kTileBytes]>(smem + 2 * G::kTileBytes);
    float(*s_cnt)[kBN] = reinterpret_cast<float(*)[kBN]>(smem + 4 * G::kTileBytes);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;
    const int bh = blockIdx.y;
    const int b = bh / p.H, h = bh % p.H;
    uint16_t* out_base = p.out + b * p.o_sb + h * p.o_sh;
    float* lse_base = p.lse ? p.lse + (int64_t)bh * p.N : nullptr;
    const int first = p.window + kTile;  // first row with a far context

    if ((int)blockIdx.x >= p.n_far_tiles) {
        // rows [0, W+T): no far context -> out = 0, lse = -inf
        const int m0 = ((int)blockIdx.x - p.n_far_tiles) * kBM;
        const int rows = min(min(first, p.N) - m0, kBM);
        for (int i = tid; i < rows * (D / 4); i += kThreads) {
            const int r = i / (D / 4), c = i % (D / 4);
            *reinterpret_cast<uint2*>(out_base + (int64_t)(m0 + r) * p.o_sn + c * 4) = make_uint2(0u, 0u);
        }
        if (lse_base)
            for (int r = tid; r < rows; r += kThreads) lse_base[m0 + r] = -INFINITY;
        return;
    }

    const int t = blockIdx.x;
    const int row0 = first + t * kTile + wave * 32;
    const uint16_t* cb = p.cb + h * p.cb_sh;
    const int64_t cnt_off = b * p.cnt_sb + h * p.cnt_sh + t * p.cnt_st;
    const uint16_t* cnt = p.cnt + cnt_off;
    const int64_t* cnt_i64 = p.cnt_i64 ? p.cnt_i64 + cnt_off : nullptr;
    const int64_t* vi = p.vi + b * p.vi_sb + h * p.vi_sh + t * p.vi_st;
    const uint16_t* vvq = p.vvq.p + b * p.vvq.sb + h * p.vvq.sh;

    QFrag<Tag, D> q;
    load_q<Tag, D>(q, p.q.p + b * p.q.sb + h * p.q.sh, p.q.sn, row0, p.N, lane);
    SoftmaxState<D> st;
    st.init();

    TileCopy<D, false> k_copy;
    TileCopy<D, true> v_copy;
    k_copy.init(wave, lane);
    v_copy.init(wave, lane);

    // Codeword tiles are double-buffered: tile c+1 (codebook rows, gathered V sums, counts) is requested before tile
    // c is computed.  The row indices and counts of a tile are fetched into registers one tile earlier still, so the
    // request never waits on them.
    int64_t rows[TileCopy<D, true>::kInstr];
    float cnt_f = 0.f;
    auto fetch_meta = [&](int c0) {
        v_copy.fetch_rows(rows, vi, c0, p.C, p.N);  // v_vq has N + 1 rows
        cnt_f = 0.f;  // 0: masked
        if (tid < kBN && c0 + tid < p.C)
            cnt_f = cnt_i64 ? (float)cnt_i64[c0 + tid] : Elem<Tag>::from_bits(cnt[c0 + tid]);
    };
    auto request = [&](int c0, int buf) {  // uses the metadata fetched for c0
        k_copy.load(s_k[buf], cb, p.cb_sc, c0, p.C);
        v_copy.load_rows(s_v[buf], vvq, p.vvq.sn, rows);
        if (tid < kBN) s_cnt[buf][tid] = cnt_f;
    };
    fetch_meta(0);
    request(0, 0);
    if (kBN < p.C) fetch_meta(kBN);
    int buf = 0;
    for (int c0 = 0; c0 < p.C; c0 += kBN, buf ^= 1) {
        wait_tile_loads();
        __syncthreads();  // tile c0 is complete in `buf`; every wave is done with the other buffer
        if (c0 + kBN < p.C) {
            request(c0 + kBN, buf ^ 1);
            if (c0 + 2 * kBN < p.C) fetch_meta(c0 + 2 * kBN);
        }

        f32x16_t s[2];
        qk_mma<Tag, D>(s, q, s_k[buf], lane);
        float w[2][16];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                // registers 4g .. 4g+3 hold codewords kb*32 + 8g + 4*half + 0..3: one 16-byte LDS read
                const f32x4_t c4 = *reinterpret_cast<const f32x4_t*>(&s_cnt[buf][kb * 32 + 8 * g + 4 * half]);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    w[kb][4 * g + e] = c4[e];
                    s[kb][4 * g + e] = (c4[e] != 0.f) ? s[kb][4 * g + e] : -INFINITY;
                }
            }
        vec8 pf[2][2];
        softmax_update<Tag, D, true>(st, s, p.scale_log2e, pf, w);
        pv_mma<Tag, D>(st.o, pf, s_v[buf], lane);
    }
    if (!p.merge_into) {
        store_output<Tag, D>(st, out_base, p.o_sn, lse_base, row0, p.N, lane);
        return;
    }
    // merge with the state already in out / lse (base-2 log-sum-exp), in place
    {
        const int n = lane & 31;
        const int row = row0 + n;
        if (row >= p.N) return;
        const float l_tot = st.l + __shfl_xor(st.l, 32, 64);
        const float s2 = l_tot > 0.f ? st.m + fast_log2(l_tot) : -INFINITY;
        const float s1 = lse_base[row];
        const float mx = fmaxf(s1, s2);
        const float m_safe = (mx == -INFINITY) ? 0.f : mx;
        const float w1 = fast_exp2(s1 - m_safe), w2 = fast_exp2(s2 - m_safe);
        const float den = w1 + w2;
        const float inv = den > 0.f ? 1.f / den : 0.f;
        const float f1 = w1 * inv;                                  // weight of the stored (normalised) output
        const float f2 = l_tot > 0.f ? w2 * inv / l_tot : 0.f;      // weight of this kernel's unnormalised sums
        uint16_t* dst = out_base + (int64_t)row * p.o_sn;
#pragma unroll
        for (int db = 0; db < Geom<D>::kDBlocks; ++db) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                uint2* at = reinterpret_cast<uint2*>(dst + db * 32 + 8 * g + 4 * half);
                const uint2 old = *at;
                const uint32_t ow[2] = {old.x, old.y};
                uint32_t nw[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float lo = Elem<Tag>::from_bits((uint16_t)(ow[e] & 0xffffu)) * f1 + st.o[db][4 * g + 2 * e] * f2;
                    const float hi = Elem<Tag>::from_bits((uint16_t)(ow[e] >> 16)) * f1 + st.o[db][4 * g + 2 * e + 1] * f2;
                    nw[e] = (uint32_t)Elem<Tag>::to_bits(lo) | ((uint32_t)Elem<Tag>::to_bits(hi) << 16);
                }
                *at = make_uint2(nw[0], nw[1]);
            }
        }
        if (half == 0) lse_base[row] = den > 0.f ? mx + fast_log2(den) : -INFINITY;
    }
}

template <typename Tag, int D>
int launch_count(const CountParams& p, dim3 grid, hipStream_t stream) {
    constexpr size_t kLds = 4 * Geom<D>::kTileBytes + 2 * kBN * sizeof(float);
    if (kLds > 65536) {
        // more than the 64 KB of LDS a launch gets by default: raised once per device (the one that owns the
        // operands, which must be the current one) and instantiation
        static std::mutex mu;
        static bool raised[kMaxDevices] = {};
        int dev = 0;
        const int rc = device_of_pointer(p.q.p, &dev);
        if (rc != VQA_OK) return rc;
        std::lock_guard<std::mutex> lock(mu);
        if (!raised[dev]) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(&count_kernel<Tag, D>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLds) != hipSuccess) {
                (void)hipGetLastError();
                return VQA_ERR_LAUNCH_FAILED;
            }
            raised[dev] = true;
        }
    }
    hipLaunchKernelGGL((count_kernel<Tag, D>), grid, dim3(kThreads), kLds, stream, p);
    return launch_status();
}

// strides: q2(b,h,n) k_vq(h,c) k_vq_cnt(b,h,t) v_vq(b,h,n) vi(b,h,t) out(b,h,n)
template <typename Tag>
int vqcount(const void* q2, const void* k_vq, const void* k_vq_cnt, const void* v_vq, const int64_t* vi, void* out,
            float* lse, int B, int H, int N, int D, int C, const int64_t* strides, int window, float sm_scale,
            bool merge_into, bool integer_counts, hipStream_t stream) {
    if (!q2 || !k_vq || !k_vq_cnt || !v_vq || !vi || !out || !strides) return VQA_ERR_NULL_POINTER;
    if (merge_into && !lse) return VQA_ERR_NULL_POINTER;
    if (B <= 0 || H <= 0 || N <= 0 || C <= 0) return VQA_ERR_BAD_SHAPE;
    if (window < 0 || !(sm_scale > 0.f) || (int64_t)B * H > 65535) return VQA_ERR_BAD_ARGUMENT;
    if (!row_stride_ok(strides[2]) || !row_stride_ok(strides[4]) || !row_stride_ok(strides[10])) return VQA_ERR_BAD_ARGUMENT;
    CountParams p;
    p.q = View{static_cast<const uint16_t*>(q2), strides[0], strides[1], strides[2]};
    p.cb = static_cast<const uint16_t*>(k_vq);
    p.cb_sh = strides[3], p.cb_sc = strides[4];
    p.cnt = integer_counts ? nullptr : static_cast<const uint16_t*>(k_vq_cnt);
    p.cnt_i64 = integer_counts ? static_cast<const int64_t*>(k_vq_cnt) : nullptr;
    p.cnt_sb = strides[5], p.cnt_sh = strides[6], p.cnt_st = strides[7];
    p.vvq = View{static_cast<const uint16_t*>(v_vq), strides[8], strides[9], strides[10]};
    p.vi = vi;
    p.vi_sb = strides[11], p.vi_sh = strides[12], p.vi_st = strides[13];
    p.out = static_cast<uint16_t*>(out);
    p.o_sb = strides[14], p.o_sh = strides[15], p.o_sn = strides[16];
    p.lse = lse;
    p.H = H, p.N = N, p.C = C, p.window = window;
    p.scale_log2e = sm_scale * kLog2e;
    if (!aligned16(p.q.p) || !aligned16(p.cb) || !aligned16(p.vvq.p) || ((uintptr_t)p.out & 7))
        return VQA_ERR_MISALIGNED;
    if (((p.q.sb | p.q.sh | p.q.sn | p.cb_sh | p.cb_sc | p.vvq.sb | p.vvq.sh | p.vvq.sn) & 7) ||
        ((p.o_sb | p.o_sh | p.o_sn) & 3))
        return VQA_ERR_MISALIGNED;
    const int first = window + kTile;
    p.n_far_tiles = N > first ? (N - first + kTile - 1) / kTile : 0;
    p.merge_into = merge_into ? 1 : 0;
    // rows below window + 128 have no far context: zero / -inf when this kernel writes a state of its own, left
    // untouched when it merges into an existing one
    const int zero_tiles = merge_into ? 0 : ((first < N ? first : N) + kBM - 1) / kBM;
    if (p.n_far_tiles + zero_tiles == 0) return VQA_OK;
    const dim3 grid(p.n_far_tiles + zero_tiles, B * H);
    if (D == 32) return launch_count<Tag, 32>(p, grid, stream);
    if (D == 64) return launch_count<Tag, 64>(p, grid, stream);
    if (D == 128) return launch_count<Tag, 128>(p, grid, stream);
    return VQA_ERR_UNSUPPORTED_HEAD_DIM;
}

// ---------------------------------------------------------------------------------------------------------------
// merge: (o, s) <- merge((o, s), (o', s')) with base-2 log-sum-exp s; one thread per 4 output elements.
// ---------------------------------------------------------------------------------------------------------------
struct MergeParams {
    uint16_t* o;
    int64_t o_sb, o_sh, o_sn;
    float* s;
    int64_t s_sb, s_sh, s_sn;
    const uint16_t* o2;
    int64_t o2_sb, o2_sh, o2_sn;
    const float* s2;
    int64_t s2_sb, s2_sh, s2_sn;
    int H, N, D;
};

template <typename Tag>
__global__ __launch_bounds__(256) void merge_kernel(MergeParams p) {
    const int cpr = p.D / 4;  // 4-element chunks per row
    const int rows_per_block = 256 / cpr;
    const int n = blockIdx.x * rows_per_block + threadIdx.x / cpr;
    const int c = threadIdx.x % cpr;
    const int bh = blockIdx.y;
    const int b = bh / p.H, h = bh % p.H;
    const bool active = n < p.N && (int)threadIdx.x < rows_per_block * cpr;
    const int nn = active ? n : blockIdx.x * rows_per_block;  // inactive threads shadow the block's first row
    float* sp = p.s + b * p.s_sb + h * p.s_sh + nn * p.s_sn;
    const float s1 = *sp;
    const float s2 = p.s2[b * p.s2_sb + h * p.s2_sh + nn * p.s2_sn];
    const float m = fmaxf(s1, s2);
    const float m_safe = (m == -INFINITY) ? 0.f : m;
    const float w1 = fast_exp2(s1 - m_safe), w2 = fast_exp2(s2 - m_safe);
    const float den = w1 + w2;
    const float inv = den > 0.f ? 1.f / den : 0.f;
    uint16_t* op = p.o + b * p.o_sb + h * p.o_sh + nn * p.o_sn + c * 4;
    const uint16_t* op2 = p.o2 + b * p.o2_sb + h * p.o2_sh + nn * p.o2_sn + c * 4;
    const uint2 a = *reinterpret_cast<const uint2*>(op);
    const uint2 bb = *reinterpret_cast<const uint2*>(op2);
    const uint32_t aw[2] = {a.x, a.y}, bw[2] = {bb.x, bb.y};
    uint32_t rw[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const float lo = (Elem<Tag>::from_bits((uint16_t)(aw[e] & 0xffffu)) * w1 +
                          Elem<Tag>::from_bits((uint16_t)(bw[e] & 0xffffu)) * w2) * inv;
        const float hi = (Elem<Tag>::from_bits((uint16_t)(aw[e] >> 16)) * w1 +
                          Elem<Tag>::from_bits((uint16_t)(bw[e] >> 16)) * w2) * inv;
        rw[e] = (uint32_t)Elem<Tag>::to_bits(lo) | ((uint32_t)Elem<Tag>::to_bits(hi) << 16);
    }
    if (active) *reinterpret_cast<uint2*>(op) = make_uint2(rw[0], rw[1]);
    __syncthreads();  // every thread of the row has read s before it is rewritten
    if (active && c == 0) *sp = den > 0.f ? m + fast_log2(den) : -INFINITY;
}

// strides: o(b,h,n) s(b,h,n) o_other(b,h,n) s_other(b,h,n)
template <typename Tag>
int merge(void* o, float* s, const void* o_other, const float* s_other, int B, int H, int N, int D,
          const int64_t* strides, hipStream_t stream) {
    if (!o || !s || !o_other || !s_other || !strides) return VQA_ERR_NULL_POINTER;
    if (B <= 0 || H <= 0 || N <= 0) return VQA_ERR_BAD_SHAPE;
    if (D < 4 || D > 1024 || (D & 3)) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    if ((int64_t)B * H > 65535) return VQA_ERR_BAD_ARGUMENT;
    MergeParams p;
    p.o = static_cast<uint16_t*>(o);
    p.o_sb = strides[0], p.o_sh = strides[1], p.o_sn = strides[2];
    p.s = s;
    p.s_sb = strides[3], p.s_sh = strides[4], p.s_sn = strides[5];
    p.o2 = static_cast<const uint16_t*>(o_other);
    p.o2_sb = strides[6], p.o2_sh = strides[7], p.o2_sn = strides[8];
    p.s2 = s_other;
    p.s2_sb = strides[9], p.s2_sh = strides[10], p.s2_sn = strides[11];
    p.H = H, p.N = N, p.D = D;
    if (((uintptr_t)o & 7) || ((uintptr_t)o_other & 7) ||
        ((p.o_sb | p.o_sh | p.o_sn | p.o2_sb | p.o2_sh | p.o2_sn) & 3))
        return VQA_ERR_MISALIGNED;
    const int cpr = D / 4;
    if (cpr > 256) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    const int rows_per_block = 256 / cpr;
    const dim3 grid((N + rows_per_block - 1) / rows_per_block, B * H);
    hipLaunchKernelGGL((merge_kernel<Tag>), grid, dim3(256), 0, stream, p);
    return launch_status();
}

}  // namespace flash
}  // namespace vqa

extern "C" {

int vqa_vqcount_fwd_bf16(const void* q2, const void* k_vq, const void* k_vq_cnt, const void* v_vq, const int64_t* vi,
                         void* out, float* lse, int B, int H, int N, int D, int C, const int64_t* strides, int window,
                         float sm_scale, vqa_stream_t stream) {
    return vqa::flash::vqcount<vqa::bf16_tag>(q2, k_vq, k_vq_cnt, v_vq, vi, out, lse, B, H, N, D, C, strides, window,
                                              sm_scale, false, false, stream);
}

int vqa_vqcount_fwd_f16(const void* q2, const void* k_vq, const void* k_vq_cnt, const void* v_vq, const int64_t* vi,
                        void* out, float* lse, int B, int H, int N, int D, int C, const int64_t* strides, int window,
                        float sm_scale, vqa_stream_t stream) {
    return vqa::flash::vqcount<vqa::f16_tag>(q2, k_vq, k_vq_cnt, v_vq, vi, out, lse, B, H, N, D, C, strides, window,
                                             sm_scale, false, false, stream);
}

int vqa_vqcount_merge_bf16(const void* q2, const void* k_vq, const void* k_vq_cnt, const void* v_vq, const int64_t* vi,
                           void* out, float* lse, int B, int H, int N, int D, int C, const int64_t* strides,
                           int window, float sm_scale, vqa_stream_t stream) {
    return vqa::flash::vqcount<vqa::bf16_tag>(q2, k_vq, k_vq_cnt, v_vq, vi, out, lse, B, H, N, D, C, strides, window,
                                              sm_scale, true, false, stream);
}

int vqa_vqcount_merge_f16(const void* q2, const void* k_vq, const void* k_vq_cnt, const void* v_vq, const int64_t* vi,
                          void* out, float* lse, int B, int H, int N, int D, int C, const int64_t* strides, int window,
                          float sm_scale, vqa_stream_t stream) {
    return vqa::flash::vqcount<vqa::f16_tag>(q2, k_vq, k_vq_cnt, v_vq, vi, out, lse, B, H, N, D, C, strides, window,
                                             sm_scale, true, false, stream);
}

int vqa_vqcount_fwd_icnt_bf16(const void* q2, const void* k_vq, const int64_t* k_vq_cnt, const void* v_vq,
                              const int64_t* vi, void* out, float* lse, int B, int H, int N, int D, int C,
                              const int64_t* strides, int window, float sm_scale, vqa_stream_t stream) {
    return vqa::flash::vqcount<vqa::bf16_tag>(q2, k_vq, k_vq_cnt, v_vq, vi, out, lse, B, H, N, D, C, strides, window,
                                              sm_scale, false, true, stream);
}

int vqa_vqcount_fwd_icnt_f16(const void* q2, const void* k_vq, const int64_t* k_vq_cnt, const void* v_vq,
                             const int64_t* vi, void* out, float* lse, int B, int H, int N, int D, int C,
                             const int64_t* strides, int window, float sm_scale, vqa_stream_t stream) {
    return vqa::flash::vqcount<vqa::f16_tag>(q2, k_vq, k_vq_cnt, v_vq, vi, out, lse, B, H, N, D, C, strides, window,
                                             sm_scale, false, true, stream);
}

int vqa_vqcount_merge_icnt_bf16(const void* q2, const void* k_vq, const int64_t* k_vq_cnt, const void* v_vq,
                                const int64_t* vi, void* out, float* lse, int B, int H, int N, int D, int C,
                                const int64_t* strides, int window, float sm_scale, vqa_stream_t stream) {
    return vqa::flash::vqcount<vqa::bf16_tag>(q2, k_vq, k_vq_cnt, v_vq, vi, out, lse, B, H, N, D, C, strides, window,
                                              sm_scale, true, true, stream);
}

int vqa_vqcount_merge_icnt_f16(const void* q2, const void* k_vq, const int64_t* k_vq_cnt, const void* v_vq,
                               const int64_t* vi, void* out, float* lse, int B, int H, int N, int D, int C,
                               const int64_t* strides, int window, float sm_scale, vqa_stream_t stream) {
    return vqa::flash::vqcount<vqa::f16_tag>(q2, k_vq, k_vq_cnt, v_vq, vi, out, lse, B, H, N, D, C, strides, window,
                                             sm_scale, true, true, stream);
}

int vqa_merge_state_inplace_bf16(void* o, float* s, const void* o_other, const float* s_other, int B, int H, int N,
                                 int D, const int64_t* strides, vqa_stream_t stream) {
    return vqa::flash::merge<vqa::bf16_tag>(o, s, o_other, s_other, B, H, N, D, strides, stream);
}

int vqa_merge_state_inplace_f16(void* o, float* s, const void* o_other, const float* s_other, int B, int H, int N,
                                int D, const int64_t* strides, vqa_stream_t stream) {
    return vqa::flash::merge<vqa::f16_tag>(o, s, o_other, s_other, B, H, N, D, strides, stream);
}

}  // extern "C"
