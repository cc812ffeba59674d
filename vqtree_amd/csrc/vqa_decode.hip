// seqlen_q = 1 attention over additive-quantiser key codes (gfx950).
//
// Three launches per call, all on the caller's stream:
//   1. lut_kernel    LUT[b,h,m,c] = sm_scale*log2(e) * <q[b,h], codebooks[h,m,c]>        (MFMA 16x16x32, tiny)
//   2. main_kernel   one workgroup per (KV split, b*H+h): streams packed uint8 codes and V rows from HBM,
//                    score_j = sum_m LUT[m][code_jm] from LDS, online base-2 softmax, fp32 accumulation of p*V;
//                    writes one unnormalised partial state (o[D], m, l) per split
//   3. merge_kernel  log-sum-exp merge of the split states, normalise, cast, optional lse
// The main kernel is HBM-bound: per key it reads M code bytes and one D-element V row and nothing else.
#include <mutex>

#include "vqa_common.h"

namespace vqa {
namespace decode {

constexpr int kLutStride = 256;   // LUT entries reserved per codebook (uint8 codes)
constexpr int kThreads = 256;     // main kernel workgroup: 4 waves
constexpr int kWaves = kThreads / kWave;
constexpr int kBatch = 64;        // keys scored per wave per step (one per lane)

struct Strides {
    int64_t q_b, q_h;
    int64_t c_b, c_h;
    int64_t cb_h, cb_m, cb_k;
    int64_t v_b, v_h, v_n;
    int64_t o_b, o_h;
};

// ---------------------------------------------------------------------------------------------------------------
// 1. lookup table.  One wave owns 16 codewords of one (h, m) and sweeps the batch 16 rows at a time:
//    C[code, b] = sum_d cb[code, d] * q[b, d] as D/32 MFMA 16x16x32 steps; A and B fragments come straight from
//    global memory (each lane: 8 contiguous elements of its row).
// ---------------------------------------------------------------------------------------------------------------
//    With rope_cos / rope_sin (one [D] row each: the tables at the query's position) the query is rotated on the way in,
//    q' = q * cos + rotate_half(q) * sin with every product and the sum rounded to the element type -- bit for bit what
//    the rotary kernel (vqa_rope.hip) writes -- so a caller with an unrotated query needs no launch for it.
template <typename Tag>
__device__ __forceinline__ float rnd16(float x) { return Elem<Tag>::round_keep_f32(x); }

// one 8-element slice of the rotated query: x = the slice itself, xp = its rotate_half partner (D/2 elements away),
// c / s = the cos / sin slices at x's place; upper = x lies in the upper half of the row
template <typename Tag>
__device__ __forceinline__ typename Elem<Tag>::vec8 rotate_slice(typename Elem<Tag>::vec8 x, typename Elem<Tag>::vec8 xp,
                                                                 typename Elem<Tag>::vec8 c, typename Elem<Tag>::vec8 s,
                                                                 bool upper) {
// every product and the sum round on their own: no fused multiply-add (for f16 the compiler turns the conversions below
// into 16-bit arithmetic, which it would then contract)
#pragma clang fp contract(off)
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 xw = __builtin_bit_cast(u32x4, x), pw = __builtin_bit_cast(u32x4, xp);
    const u32x4 cw = __builtin_bit_cast(u32x4, c), sw = __builtin_bit_cast(u32x4, s);
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        uint32_t pair = 0;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int sh = 16 * t;
            const float xv = Elem<Tag>::from_bits((uint16_t)(xw[e] >> sh)), pv = Elem<Tag>::from_bits((uint16_t)(pw[e] >> sh));
            const float cv = Elem<Tag>::from_bits((uint16_t)(cw[e] >> sh)), sv = Elem<Tag>::from_bits((uint16_t)(sw[e] >> sh));
            // lower half: x*cos + (-partner)*sin; upper half: x*cos + partner*sin (products of two 16-bit values are
            // exact in fp32, so each rounding below is the only one of its operator)
            // (rounding is symmetric: subtracting the rounded product is adding the rounded negated one)
            const float t0 = rnd16<Tag>(xv * cv), t1 = rnd16<Tag>(pv * sv);
            const float r = rnd16<Tag>(upper ? t0 + t1 : t0 - t1);
            pair |= (uint32_t)Elem<Tag>::to_bits(r) << sh;
        }
        o[e] = pair;
    }
    return __builtin_bit_cast(typename Elem<Tag>::vec8, o);
}

template <typename Tag, int D>
__global__ __launch_bounds__(kThreads) void lut_kernel(const uint16_t* __restrict__ q,
                                                       const uint16_t* __restrict__ cb, float* __restrict__ lut,
                                                       int B, int H, int M, int K, Strides st, float scale_log2e,
                                                       const uint16_t* __restrict__ rope_cos,
                                                       const uint16_t* __restrict__ rope_sin) {
    typedef typename Elem<Tag>::vec8 vec8;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    // 16-codeword tile inside this codebook; all kLutStride entries are written, those past K repeat codeword K - 1,
    // so a code >= K scores (deterministically) as K - 1
    const int tile = blockIdx.x * kWaves + wave;
    if (tile * 16 >= kLutStride) return;
    const int hm = blockIdx.y;
    const int h = hm / M, m = hm % M;
    const int r = lane & 15;   // A row (codeword) / B column (batch row)
    const int kq = lane >> 4;  // which 8-element slice of each 32-wide k step
    const int code = min(tile * 16 + r, K - 1);
    const uint16_t* a_row = cb + h * st.cb_h + m * st.cb_m + (int64_t)code * st.cb_k + kq * 8;
    vec8 a[D / 32];
#pragma unroll
    for (int kk = 0; kk < D / 32; ++kk) a[kk] = *reinterpret_cast<const vec8*>(a_row + kk * 32);

    for (int b0 = 0; b0 < B; b0 += 16) {
        const int bb = b0 + r;
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
        const uint16_t* b_row = q + (int64_t)min(bb, B - 1) * st.q_b + h * st.q_h + kq * 8;
        vec8 bv[D / 32];
#pragma unroll
        for (int kk = 0; kk < D / 32; ++kk) bv[kk] = *reinterpret_cast<const vec8*>(b_row + kk * 32);
        if (rope_cos != nullptr) {  // (uniform)
            vec8 rv[D / 32];
#pragma unroll
            for (int kk = 0; kk < D / 32; ++kk) {
                constexpr int kHalf = D / 64;  // slices per half row: the partner of slice kk is kk ^ kHalf
                const vec8 c = *reinterpret_cast<const vec8*>(rope_cos + kk * 32 + kq * 8);
                const vec8 sn = *reinterpret_cast<const vec8*>(rope_sin + kk * 32 + kq * 8);
                rv[kk] = rotate_slice<Tag>(bv[kk], bv[kk ^ kHalf], c, sn, kk >= kHalf);
            }
#pragma unroll
            for (int kk = 0; kk < D / 32; ++kk) bv[kk] = rv[kk];
        }
#pragma unroll
        for (int kk = 0; kk < D / 32; ++kk) acc = Elem<Tag>::mfma16(a[kk], bv[kk], acc);
        // acc[i]: codeword row 4*kq + i, batch column r
        if (bb < B) {
            float* dst = lut + ((int64_t)(bb * H + h) * M + m) * kLutStride + tile * 16 + kq * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[i] = acc[i] * scale_log2e;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// 2. main streaming kernel
// ---------------------------------------------------------------------------------------------------------------
template <int M>
struct CodeWord;
template <>
struct CodeWord<1> {
    typedef uint8_t type;
};
template <>
struct CodeWord<2> {
    typedef uint16_t type;
};
template <>
struct CodeWord<4> {
    typedef uint32_t type;
};
template <>
struct CodeWord<8> {
    typedef uint2 type;
};

template <int M>
__device__ __forceinline__ float score_from_lut(const float* s_lut, typename CodeWord<M>::type cw) {
    if constexpr (M == 8) {
        float s = 0.f;
#pragma unroll
        for (int m = 0; m < 4; ++m) s += s_lut[m * kLutStride + ((cw.x >> (8 * m)) & 0xffu)];
#pragma unroll
        for (int m = 0; m < 4; ++m) s += s_lut[(4 + m) * kLutStride + ((cw.y >> (8 * m)) & 0xffu)];
        return s;
    } else {
        const uint32_t w = cw;
        float s = 0.f;
#pragma unroll
        for (int m = 0; m < M; ++m) s += s_lut[m * kLutStride + ((w >> (8 * m)) & 0xffu)];
        return s;
    }
}

// Lane layout inside a wave: LPR = D/8 lanes cover one V row with 16-byte loads, so one load instruction covers
// G = 64/LPR consecutive rows; a 64-key batch takes R = 64/G loads per lane.  Lane (g, c) accumulates rows
// {i*G + g} into its 8 output elements c*8..c*8+7; the G row groups are summed once at the end.
//
// Each wave walks batches k0, k0 + 256, ... of its split.  The R row buffers roll: as soon as row i of the current
// batch has been accumulated its registers receive row i of the next batch, so every wave keeps R 16-byte loads per
// lane in flight at all times with only R*4 buffer registers.  A ragged last batch is moved back to end exactly at
// the split end (keys already consumed get weight zero), so no load in the loop needs clamping.
template <typename Tag, int D, int M>
__global__ __launch_bounds__(kThreads, 3) void main_kernel(const uint8_t* __restrict__ codes,
                                                           const uint16_t* __restrict__ v,
                                                           const float* __restrict__ lut,
                                                           float* __restrict__ part_o, float* __restrict__ part_ml,
                                                           int H, int N, int S, int keys_per_split, Strides st,
                                                           const int* __restrict__ n_keys_dev, int slot_stride,
                                                           int slot_off, uint16_t* __restrict__ out_direct,
                                                           float* __restrict__ lse_direct) {
    constexpr int LPR = D / 8;
    constexpr int G = kWave / LPR;
    constexpr int R = kBatch / G;
    constexpr int kStep = kWaves * kBatch;
    typedef typename CodeWord<M>::type code_t;

    __shared__ float s_lut[M * kLutStride];
    __shared__ __attribute__((aligned(16))) float s_p[kWaves][kBatch];
    __shared__ float s_red[kWaves][G][D];
    __shared__ float s_m[kWaves];
    __shared__ float s_l[kWaves];

    const int split = blockIdx.x;
    const int bh = blockIdx.y;
    const int b = bh / H, h = bh % H;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane / LPR, c = lane % LPR;
    if (n_keys_dev != nullptr) {
        // the number of keys lives in device memory (a launch recorded once and replayed as the cache grows):
        // N is only the bound the buffers were sized for
        N = max(0, min(N, *n_keys_dev));
        keys_per_split = ((N + S - 1) / S + kThreads - 1) / kThreads * kThreads;
    }

    for (int i = tid; i < M * kLutStride; i += kThreads) s_lut[i] = lut[(int64_t)bh * M * kLutStride + i];
    __syncthreads();

    const int k_begin = split * keys_per_split;
    const int k_end = min(N, k_begin + keys_per_split);
    const code_t* code_base = reinterpret_cast<const code_t*>(codes + b * st.c_b + h * st.c_h);
    const char* v_bh = reinterpret_cast<const char*>(v + b * st.v_b + h * st.v_h);
    const int64_t row_bytes = st.v_n * 2;
    const uint32_t lane_off = (uint32_t)(g * row_bytes) + c * 16;  // this lane's slice of row g of a batch
    const uint32_t grp_bytes = (uint32_t)(G * row_bytes);          // distance between consecutive loads

    float m_run = -INFINITY;
    float l_run = 0.f;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;

    uint4 buf[R];
    code_t cw_cur, cw_nxt;

    const int k0 = k_begin + wave * kBatch;
    const int n_batches = k0 < k_end ? (k_end - k0 + kStep - 1) / kStep : 0;
    // batch j scores keys [valid_from, k_end) of the 64 loaded from load_from
    auto batch_bounds = [&](int j, int& load_from, int& valid_from) {
        valid_from = k0 + j * kStep;
        load_from = (valid_from + kBatch <= k_end) ? valid_from : max(k_end - kBatch, 0);
    };
    auto load_code = [&](int load_from) { return code_base[min(load_from + lane, N - 1)]; };

    auto process = [&](auto prefetch, int load_from, int valid_from, int next_load_from) {
        constexpr bool kPrefetch = decltype(prefetch)::value;
        float s = score_from_lut<M>(s_lut, cw_cur);
        const int key = load_from + lane;
        s = (key >= valid_from && key < k_end) ? s : -INFINITY;
        if constexpr (kPrefetch) cw_nxt = load_code(next_load_from);
        const float m_new = fmaxf(m_run, wave_max(s));
        if (m_new > m_run) {  // same outcome in every lane of the wave
            const float alpha = fast_exp2(m_run - m_new);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] *= alpha;
            l_run *= alpha;
            m_run = m_new;
        }
        float p = (s == -INFINITY) ? 0.f : fast_exp2(s - m_run);
        p = Elem<Tag>::round_keep_f32(p);  // P is rounded to the V type before P.V; l sums the same values
        l_run += p;
        // key lane -> slot (key % G) * R + key / G, so row group g finds its R weights contiguous
        s_p[wave][(lane % G) * R + lane / G] = p;
        wave_lds_sync();
        float pr[R];
#pragma unroll
        for (int i = 0; i < R; i += 4) {
            const f32x4_t t = *reinterpret_cast<const f32x4_t*>(&s_p[wave][g * R + i]);
            pr[i] = t[0];
            pr[i + 1] = t[1];
            pr[i + 2] = t[2];
            pr[i + 3] = t[3];
        }
        wave_lds_sync();
        const char* next_base = v_bh + (int64_t)next_load_from * row_bytes;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            // packed weight pairs (p, 0) and (0, p) in the V element type
            const uint32_t pbits = Elem<Tag>::rounded_to_bits(pr[i]);
            const uint32_t p_lo = pbits, p_hi = pbits << 16;
            const uint32_t w[4] = {buf[i].x, buf[i].y, buf[i].z, buf[i].w};
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                acc[2 * d] = Elem<Tag>::dot2(w[d], p_lo, acc[2 * d]);
                acc[2 * d + 1] = Elem<Tag>::dot2(w[d], p_hi, acc[2 * d + 1]);
            }
            if constexpr (kPrefetch) {
                buf[i] = load_stream16(next_base + (lane_off + i * grp_bytes));
                __builtin_amdgcn_sched_barrier(0);  // keep the reload right behind the row it replaces
            }
        }
        if constexpr (kPrefetch) cw_cur = cw_nxt;
    };

    if (n_batches > 0) {
        int load_from, valid_from;
        batch_bounds(0, load_from, valid_from);
        cw_cur = load_code(load_from);
        const char* base = v_bh + (int64_t)load_from * row_bytes;
        if (N >= kBatch) {
#pragma unroll
            for (int i = 0; i < R; ++i)
                buf[i] = load_stream16(base + (lane_off + i * grp_bytes));
        } else {  // fewer keys than one batch in the whole sequence: clamp rows (their weight is zero)
#pragma unroll
            for (int i = 0; i < R; ++i)
                buf[i] = load_stream16(v_bh + (int64_t)min(i * G + g, N - 1) * row_bytes + c * 16);
        }
        for (int j = 0; j + 1 < n_batches; ++j) {
            int next_load_from, next_valid_from;
            batch_bounds(j + 1, next_load_from, next_valid_from);
            process(std::true_type{}, load_from, valid_from, next_load_from);
            load_from = next_load_from;
            valid_from = next_valid_from;
        }
        process(std::false_type{}, load_from, valid_from, load_from);
    }

    // combine the G row groups of each wave and the waves of the workgroup
    const float l_wave = wave_sum(l_run);
#pragma unroll
    for (int e = 0; e < 8; ++e) s_red[wave][g][c * 8 + e] = acc[e];
    if (lane == 0) {
        s_m[wave] = m_run;
        s_l[wave] = l_wave;
    }
    __syncthreads();
    if (tid < D) {
        float m_all = s_m[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) m_all = fmaxf(m_all, s_m[w]);
        float o = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float wgt = (s_m[w] == -INFINITY) ? 0.f : fast_exp2(s_m[w] - m_all);
            float t = 0.f;
#pragma unroll
            for (int gg = 0; gg < G; ++gg) t += s_red[w][gg][tid];
            o += wgt * t;
            l += wgt * s_l[w];
        }
        if (out_direct != nullptr) {
            // a single split whose state is the result: normalise and store, no merge launch behind this kernel
            const int b = bh / H, h = bh % H;
            out_direct[b * st.o_b + h * st.o_h + tid] = Elem<Tag>::to_bits(l > 0.f ? o / l : 0.f);
            if (tid == 0 && lse_direct != nullptr) lse_direct[bh] = l > 0.f ? m_all + fast_log2(l) : -INFINITY;
            return;
        }
        // partial states of one (batch, head) are contiguous: slot_stride of them, this launch's from slot_off on
        const int64_t slot = (int64_t)bh * slot_stride + slot_off + split;
        part_o[slot * D + tid] = o;
        if (tid == 0) {
            part_ml[slot * 2] = m_all;
            part_ml[slot * 2 + 1] = l;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// 3. merge of the split states
// ---------------------------------------------------------------------------------------------------------------
template <typename Tag, int D>
__global__ __launch_bounds__(D) void merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                  uint16_t* __restrict__ out, float* __restrict__ lse, int H, int S,
                                                  Strides st) {
    const int bh = blockIdx.x;
    const int b = bh / H, h = bh % H;
    const int d = threadIdx.x;
    float m_all = -INFINITY;
    for (int s = 0; s < S; ++s) m_all = fmaxf(m_all, part_ml[((int64_t)bh * S + s) * 2]);
    float o = 0.f, l = 0.f;
    for (int s = 0; s < S; ++s) {
        const int64_t slot = (int64_t)bh * S + s;
        const float ms = part_ml[slot * 2];
        const float wgt = (ms == -INFINITY) ? 0.f : fast_exp2(ms - m_all);
        o += wgt * part_o[slot * D + d];
        l += wgt * part_ml[slot * 2 + 1];
    }
    const float res = l > 0.f ? o / l : 0.f;
    out[b * st.o_b + h * st.o_h + d] = Elem<Tag>::to_bits(res);
    if (lse != nullptr && d == 0) lse[bh] = l > 0.f ? m_all + fast_log2(l) : -INFINITY;
}

// ---------------------------------------------------------------------------------------------------------------
// Exact-key variant of the streaming kernel: score_j = sm_scale * <q, K_j> from the key rows themselves (no codes, no
// lookup table).  Same lane layout for K as for V (LPR lanes per row, G rows per load, R loads per 64-key batch): a
// lane multiplies its 8-element slice of the row with its slice of q, the LPR lanes of the row add up, and every lane
// of row group g ends up holding the R scores of its own rows -- exactly the weights it needs for its V rows, so no
// exchange through LDS is needed.  Both row-buffer sets roll as in the coded kernel.  HBM bound: 2 rows per key.
// ---------------------------------------------------------------------------------------------------------------
struct ExactStrides {
    int64_t q_b, q_h;
    int64_t k_b, k_h, k_n;
    int64_t v_b, v_h, v_n;
};

template <typename Tag, int D>
__global__ __launch_bounds__(kThreads, 2) void exact_kernel(const uint16_t* __restrict__ q,
                                                            const uint16_t* __restrict__ k,
                                                            const uint16_t* __restrict__ v,
                                                            float* __restrict__ part_o, float* __restrict__ part_ml,
                                                            int H, int N, int S, int keys_per_split, ExactStrides st,
                                                            float scale_log2e, int slot_stride, int slot_off) {
    constexpr int LPR = D / 8;
    constexpr int G = kWave / LPR;
    constexpr int R = kBatch / G;
    constexpr int kStep = kWaves * kBatch;

    __shared__ float s_red[kWaves][G][D];
    __shared__ float s_m[kWaves];
    __shared__ float s_l[kWaves];

    const int split = blockIdx.x;
    const int bh = blockIdx.y;
    const int b = bh / H, h = bh % H;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane / LPR, c = lane % LPR;

    const uint4 qv = *reinterpret_cast<const uint4*>(q + b * st.q_b + h * st.q_h + c * 8);
    const uint32_t qw[4] = {qv.x, qv.y, qv.z, qv.w};

    const int k_begin = split * keys_per_split;
    const int k_end = min(N, k_begin + keys_per_split);
    const char* k_bh = reinterpret_cast<const char*>(k + b * st.k_b + h * st.k_h);
    const char* v_bh = reinterpret_cast<const char*>(v + b * st.v_b + h * st.v_h);
    const int64_t k_row_bytes = st.k_n * 2, v_row_bytes = st.v_n * 2;
    const uint32_t k_lane_off = (uint32_t)(g * k_row_bytes) + c * 16, k_grp = (uint32_t)(G * k_row_bytes);
    const uint32_t v_lane_off = (uint32_t)(g * v_row_bytes) + c * 16, v_grp = (uint32_t)(G * v_row_bytes);

    float m_run = -INFINITY;
    float l_run = 0.f;  // sum over this lane's row group only; the groups are added at the end
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    uint4 kbuf[R], vbuf[R];

    const int k0 = k_begin + wave * kBatch;
    const int n_batches = k0 < k_end ? (k_end - k0 + kStep - 1) / kStep : 0;
    auto batch_bounds = [&](int j, int& load_from, int& valid_from) {
        valid_from = k0 + j * kStep;
        load_from = (valid_from + kBatch <= k_end) ? valid_from : max(k_end - kBatch, 0);
    };

    auto process = [&](auto prefetch, int load_from, int valid_from, int next_load_from) {
        constexpr bool kPrefetch = decltype(prefetch)::value;
        const char* next_k = k_bh + (int64_t)next_load_from * k_row_bytes;
        const char* next_v = v_bh + (int64_t)next_load_from * v_row_bytes;
        float sc[R];
        float m_loc = -INFINITY;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const uint32_t w[4] = {kbuf[i].x, kbuf[i].y, kbuf[i].z, kbuf[i].w};
            float part = 0.f;
#pragma unroll
            for (int d = 0; d < 4; ++d) part = Elem<Tag>::dot2(w[d], qw[d], part);
#pragma unroll
            for (int off = LPR / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, 64);
            const int key = load_from + i * G + g;
            sc[i] = (key >= valid_from && key < k_end) ? part * scale_log2e : -INFINITY;
            m_loc = fmaxf(m_loc, sc[i]);
            if constexpr (kPrefetch) {
                kbuf[i] = load_stream16(next_k + (k_lane_off + i * k_grp));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int off = LPR; off < kWave; off <<= 1) m_loc = fmaxf(m_loc, __shfl_xor(m_loc, off, 64));
        const float m_new = fmaxf(m_run, m_loc);
        if (m_new > m_run) {  // same outcome in every lane of the wave
            const float alpha = fast_exp2(m_run - m_new);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] *= alpha;
            l_run *= alpha;
            m_run = m_new;
        }
#pragma unroll
        for (int i = 0; i < R; ++i) {
            float p = (sc[i] == -INFINITY) ? 0.f : fast_exp2(sc[i] - m_run);
            p = Elem<Tag>::round_keep_f32(p);  // P is rounded to the V type before P.V; l sums the same values
            l_run += p;
            const uint32_t pbits = Elem<Tag>::rounded_to_bits(p);
            const uint32_t p_lo = pbits, p_hi = pbits << 16;
            const uint32_t w[4] = {vbuf[i].x, vbuf[i].y, vbuf[i].z, vbuf[i].w};
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                acc[2 * d] = Elem<Tag>::dot2(w[d], p_lo, acc[2 * d]);
                acc[2 * d + 1] = Elem<Tag>::dot2(w[d], p_hi, acc[2 * d + 1]);
            }
            if constexpr (kPrefetch) {
                vbuf[i] = load_stream16(next_v + (v_lane_off + i * v_grp));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    if (n_batches > 0) {
        int load_from, valid_from;
        batch_bounds(0, load_from, valid_from);
        if (N >= kBatch) {
            const char* kb = k_bh + (int64_t)load_from * k_row_bytes;
            const char* vb = v_bh + (int64_t)load_from * v_row_bytes;
#pragma unroll
            for (int i = 0; i < R; ++i) kbuf[i] = load_stream16(kb + (k_lane_off + i * k_grp));
#pragma unroll
            for (int i = 0; i < R; ++i) vbuf[i] = load_stream16(vb + (v_lane_off + i * v_grp));
        } else {  // fewer keys than one batch in the whole sequence: clamp rows (their weight is zero)
#pragma unroll
            for (int i = 0; i < R; ++i) {
                const int64_t row = min(i * G + g, N - 1);
                kbuf[i] = load_stream16(k_bh + row * k_row_bytes + c * 16);
                vbuf[i] = load_stream16(v_bh + row * v_row_bytes + c * 16);
            }
        }
        for (int j = 0; j + 1 < n_batches; ++j) {
            int next_load_from, next_valid_from;
            batch_bounds(j + 1, next_load_from, next_valid_from);
            process(std::true_type{}, load_from, valid_from, next_load_from);
            load_from = next_load_from;
            valid_from = next_valid_from;
        }
        process(std::false_type{}, load_from, valid_from, load_from);
    }

    // combine the G row groups of each wave and the waves of the workgroup
    float l_wave = l_run;
#pragma unroll
    for (int off = LPR; off < kWave; off <<= 1) l_wave += __shfl_xor(l_wave, off, 64);
#pragma unroll
    for (int e = 0; e < 8; ++e) s_red[wave][g][c * 8 + e] = acc[e];
    if (lane == 0) {
        s_m[wave] = m_run;
        s_l[wave] = l_wave;
    }
    __syncthreads();
    if (tid < D) {
        float m_all = s_m[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) m_all = fmaxf(m_all, s_m[w]);
        float o = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float wgt = (s_m[w] == -INFINITY) ? 0.f : fast_exp2(s_m[w] - m_all);
            float t = 0.f;
#pragma unroll
            for (int gg = 0; gg < G; ++gg) t += s_red[w][gg][tid];
            o += wgt * t;
            l += wgt * s_l[w];
        }
        // partial states of one (batch, head) are contiguous: slot_stride of them, this launch's from slot_off on
        const int64_t slot = (int64_t)bh * slot_stride + slot_off + split;
        part_o[slot * D + tid] = o;
        if (tid == 0) {
            part_ml[slot * 2] = m_all;
            part_ml[slot * 2 + 1] = l;
        }
    }
}

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

struct Workspace {
    size_t lut_off, po_off, pml_off, total;
};

inline Workspace plan(int B, int H, int D, int M, int S) {
    Workspace w;
    const size_t bh = (size_t)B * H;
    w.lut_off = 0;
    w.po_off = align_up(bh * M * kLutStride * sizeof(float), 256);
    w.pml_off = w.po_off + align_up(bh * S * D * sizeof(float), 256);
    w.total = w.pml_off + align_up(bh * S * 2 * sizeof(float), 256);
    return w;
}

inline int default_splits(int B, int H, int N) {
    // Measured on the streaming kernel (batch x heads from 8 to 512, 32k - 64k keys): a call is fastest with about a
    // thousand workgroups, each streaming at least 4096 keys -- more, shorter splits pay the per-workgroup prologue
    // (table copy, first loads) and a longer merge, fewer leave compute units idle.  With very few (batch, head) units
    // shorter splits are accepted to get workgroups onto every CU at all.  From 512 units on a single split per unit
    // already keeps two workgroups on every CU, runs as fast as two splits, and needs no merge launch.
    const int64_t bh = (int64_t)B * H;
    if (bh <= 0 || N <= 0) return 1;
    int64_t s = bh >= 512 ? 1 : (1024 + bh - 1) / bh;  // 512 units: one split each fills the chip, and needs no merge
    const int64_t min_keys = bh >= 16 ? 4096 : 1024;
    const int64_t max_s = (N + min_keys - 1) / min_keys;
    if (s > max_s) s = max_s;
    if (s < 1) s = 1;
    if (s > 256) s = 256;
    return (int)s;
}

template <typename Tag, int D, int M>
int launch_main(const uint8_t* codes, const uint16_t* v, const float* lut, float* po, float* pml, int B, int H, int N,
                int S, int kps, const Strides& st, const int* n_keys_dev, int slot_stride, int slot_off,
                hipStream_t stream, uint16_t* out_direct = nullptr, float* lse_direct = nullptr) {
    hipLaunchKernelGGL((main_kernel<Tag, D, M>), dim3(S, B * H), dim3(kThreads), 0, stream, codes, v, lut, po, pml, H,
                       N, S, kps, st, n_keys_dev, slot_stride, slot_off, out_direct, lse_direct);
    return launch_status();
}

template <typename Tag, int D>
int run_d(const void* q, const uint8_t* codes, const void* codebooks, const void* v, void* out, float* lse,
          void* workspace, int B, int H, int N, int M, int K, const Strides& st, float sm_scale, int S,
          const int* n_keys_dev, hipStream_t stream, const uint16_t* rope_cos = nullptr,
          const uint16_t* rope_sin = nullptr) {
    const Workspace ws = plan(B, H, D, M, S);
    char* base = static_cast<char*>(workspace);
    float* lut = reinterpret_cast<float*>(base + ws.lut_off);
    float* po = reinterpret_cast<float*>(base + ws.po_off);
    float* pml = reinterpret_cast<float*>(base + ws.pml_off);
    const uint16_t* q16 = static_cast<const uint16_t*>(q);
    const uint16_t* cb16 = static_cast<const uint16_t*>(codebooks);
    const uint16_t* v16 = static_cast<const uint16_t*>(v);

    const int tiles = kLutStride / 16;
    hipLaunchKernelGGL((lut_kernel<Tag, D>), dim3((tiles + kWaves - 1) / kWaves, H * M), dim3(kThreads), 0, stream,
                       q16, cb16, lut, B, H, M, K, st, sm_scale * kLog2e, rope_cos, rope_sin);
    int rc = launch_status();
    if (rc != VQA_OK) return rc;

    // keys per split: a multiple of the workgroup's 256-key stride so only the last split is ragged
    int kps = (N + S - 1) / S;
    kps = (kps + kThreads - 1) / kThreads * kThreads;
    // with a single split the streaming kernel's state is the result: it stores the output itself, no merge launch
    uint16_t* direct = S == 1 ? static_cast<uint16_t*>(out) : nullptr;
    float* direct_lse = S == 1 ? lse : nullptr;
    switch (M) {
        case 1: rc = launch_main<Tag, D, 1>(codes, v16, lut, po, pml, B, H, N, S, kps, st, n_keys_dev, S, 0, stream, direct, direct_lse); break;
        case 2: rc = launch_main<Tag, D, 2>(codes, v16, lut, po, pml, B, H, N, S, kps, st, n_keys_dev, S, 0, stream, direct, direct_lse); break;
        case 4: rc = launch_main<Tag, D, 4>(codes, v16, lut, po, pml, B, H, N, S, kps, st, n_keys_dev, S, 0, stream, direct, direct_lse); break;
        case 8: rc = launch_main<Tag, D, 8>(codes, v16, lut, po, pml, B, H, N, S, kps, st, n_keys_dev, S, 0, stream, direct, direct_lse); break;
        default: return VQA_ERR_UNSUPPORTED_CODEBOOK;
    }
    if (rc != VQA_OK || S == 1) return rc;
    hipLaunchKernelGGL((merge_kernel<Tag, D>), dim3(B * H), dim3(D), 0, stream, po, pml,
                       static_cast<uint16_t*>(out), lse, H, S, st);
    return launch_status();
}

// ---------------------------------------------------------------------------------------------------------------
// Scratch of the allocation-free entry point (lookup table + split states): one copy per GPU, held until the process
// ends.  Host code never passes `scratch` itself to a kernel -- the name is only a host-side handle -- but the device
// address that hipGetSymbolAddress returns for the current device, looked up once per device.
// ---------------------------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[VQA_DECODE_STATIC_SCRATCH_BYTES];

// `operand`: a device pointer of the call; the scratch copy used is the one of the device that owns it, which must be
// the calling thread's current device (the launches that follow run there)
inline int static_scratch(const void* operand, void** out) {
    static std::mutex mu;
    static void* ptrs[kMaxDevices] = {};
    int dev = -1;
    const int rc = device_of_pointer(operand, &dev);
    if (rc != VQA_OK) return rc;
    std::lock_guard<std::mutex> lock(mu);
    if (ptrs[dev] == nullptr) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
            (void)hipGetLastError();
            return VQA_ERR_LAUNCH_FAILED;
        }
        ptrs[dev] = ptr;
    }
    *out = ptrs[dev];
    return VQA_OK;
}

template <typename Tag>
int run(const void* q, const uint8_t* codes, const void* codebooks, const void* v, void* out, float* lse,
        void* workspace, size_t workspace_bytes, int B, int H, int N, int D, int M, int K, const int64_t* strides,
        float sm_scale, int num_splits, const int* n_keys_dev, hipStream_t stream, const void* rope_cos = nullptr,
        const void* rope_sin = nullptr) {
    if (!q || !codes || !codebooks || !v || !out || !workspace || !strides) return VQA_ERR_NULL_POINTER;
    if ((rope_cos == nullptr) != (rope_sin == nullptr)) return VQA_ERR_NULL_POINTER;
    if (!aligned16(rope_cos) || !aligned16(rope_sin)) return VQA_ERR_MISALIGNED;
    if (B <= 0 || H <= 0 || N <= 0) return VQA_ERR_BAD_SHAPE;
    if (D != 64 && D != 128) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    if ((M != 1 && M != 2 && M != 4 && M != 8) || K < 1 || K > 256) return VQA_ERR_UNSUPPORTED_CODEBOOK;
    Strides st;
    st.q_b = strides[0], st.q_h = strides[1];
    st.c_b = strides[2], st.c_h = strides[3];
    st.cb_h = strides[4], st.cb_m = strides[5], st.cb_k = strides[6];
    st.v_b = strides[7], st.v_h = strides[8], st.v_n = strides[9];
    st.o_b = strides[10], st.o_h = strides[11];
    // 16-byte vector loads of q / codebook / V rows; M-byte loads of packed code rows
    if (!aligned16(q) || !aligned16(codebooks) || !aligned16(v) || ((uintptr_t)workspace & 255u))
        return VQA_ERR_MISALIGNED;
    if ((st.q_b | st.q_h | st.cb_h | st.cb_m | st.cb_k | st.v_b | st.v_h | st.v_n) & 7) return VQA_ERR_MISALIGNED;
    if (((uintptr_t)codes | (uintptr_t)st.c_b | (uintptr_t)st.c_h) & (uintptr_t)(M - 1)) return VQA_ERR_MISALIGNED;
    if (!row_stride_ok(st.v_n)) return VQA_ERR_BAD_ARGUMENT;
    int S = num_splits > 0 ? num_splits : default_splits(B, H, N);
    if (S > 65535 || (int64_t)B * H > 65535) return VQA_ERR_BAD_ARGUMENT;
    if (workspace_bytes < plan(B, H, D, M, S).total) return VQA_ERR_WORKSPACE_TOO_SMALL;
    const uint16_t* rc16 = static_cast<const uint16_t*>(rope_cos);
    const uint16_t* rs16 = static_cast<const uint16_t*>(rope_sin);
    if (D == 64)
        return run_d<Tag, 64>(q, codes, codebooks, v, out, lse, workspace, B, H, N, M, K, st, sm_scale, S, n_keys_dev,
                              stream, rc16, rs16);
    return run_d<Tag, 128>(q, codes, codebooks, v, out, lse, workspace, B, H, N, M, K, st, sm_scale, S, n_keys_dev,
                           stream, rc16, rs16);
}

// strides: q(b,h) k(b,h,n) v(b,h,n) out(b,h)
template <typename Tag>
int run_exact(const void* q, const void* k, const void* v, void* out, float* lse, void* workspace,
              size_t workspace_bytes, int B, int H, int N, int D, const int64_t* strides, float sm_scale,
              int num_splits, hipStream_t stream) {
    if (!q || !k || !v || !out || !workspace || !strides) return VQA_ERR_NULL_POINTER;
    if (B <= 0 || H <= 0 || N <= 0) return VQA_ERR_BAD_SHAPE;
    if (D != 64 && D != 128) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    ExactStrides es;
    es.q_b = strides[0], es.q_h = strides[1];
    es.k_b = strides[2], es.k_h = strides[3], es.k_n = strides[4];
    es.v_b = strides[5], es.v_h = strides[6], es.v_n = strides[7];
    Strides st = {};
    st.o_b = strides[8], st.o_h = strides[9];
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || ((uintptr_t)workspace & 255u)) return VQA_ERR_MISALIGNED;
    if ((es.q_b | es.q_h | es.k_b | es.k_h | es.k_n | es.v_b | es.v_h | es.v_n) & 7) return VQA_ERR_MISALIGNED;
    if (!row_stride_ok(es.k_n) || !row_stride_ok(es.v_n)) return VQA_ERR_BAD_ARGUMENT;
    const int S = num_splits > 0 ? num_splits : default_splits(B, H, N);
    if (S > 65535 || (int64_t)B * H > 65535) return VQA_ERR_BAD_ARGUMENT;
    const Workspace ws = plan(B, H, D, 0, S);
    if (workspace_bytes < ws.total) return VQA_ERR_WORKSPACE_TOO_SMALL;
    char* base = static_cast<char*>(workspace);
    float* po = reinterpret_cast<float*>(base + ws.po_off);
    float* pml = reinterpret_cast<float*>(base + ws.pml_off);
    int kps = (N + S - 1) / S;
    kps = (kps + kThreads - 1) / kThreads * kThreads;
    const uint16_t* q16 = static_cast<const uint16_t*>(q);
    const uint16_t* k16 = static_cast<const uint16_t*>(k);
    const uint16_t* v16 = static_cast<const uint16_t*>(v);
    if (D == 64) {
        hipLaunchKernelGGL((exact_kernel<Tag, 64>), dim3(S, B * H), dim3(kThreads), 0, stream, q16, k16, v16, po, pml,
                           H, N, S, kps, es, sm_scale * kLog2e, S, 0);
    } else {
        hipLaunchKernelGGL((exact_kernel<Tag, 128>), dim3(S, B * H), dim3(kThreads), 0, stream, q16, k16, v16, po, pml,
                           H, N, S, kps, es, sm_scale * kLog2e, S, 0);
    }
    int rc = launch_status();
    if (rc != VQA_OK) return rc;
    if (D == 64)
        hipLaunchKernelGGL((merge_kernel<Tag, 64>), dim3(B * H), dim3(64), 0, stream, po, pml,
                           static_cast<uint16_t*>(out), lse, H, S, st);
    else
        hipLaunchKernelGGL((merge_kernel<Tag, 128>), dim3(B * H), dim3(128), 0, stream, po, pml,
                           static_cast<uint16_t*>(out), lse, H, S, st);
    return launch_status();
}

// Coded far keys + exact recent window in one call: keys [0, N - W) are scored through their codes with q_far, the
// last W keys exactly (k_win [B,H,W,D]) with q_win; both streaming kernels write their split states into one
// workspace and a single merge produces the output.
// strides: q_far(b,h) q_win(b,h) codes(b,h) codebooks(h,m,k) v(b,h,n) k_win(b,h,n) out(b,h)
inline void windowed_splits(int B, int H, int N, int W, int& s_far, int& s_win) {
    s_far = N > W ? default_splits(B, H, N - W) : 0;
    // the window is short: one workgroup step (256 keys) per split is enough to spread it over the chip
    const int64_t bh = (int64_t)B * H;
    int64_t s = (2048 + bh - 1) / bh;
    const int64_t max_s = (W + kThreads - 1) / kThreads;
    if (s > max_s) s = max_s;
    s_win = (int)(s < 1 ? 1 : (s > 256 ? 256 : s));
}

template <typename Tag, int D>
int run_windowed_d(const uint16_t* q_far, const uint16_t* q_win, const uint8_t* codes, const uint16_t* cb,
                   const uint16_t* v, const uint16_t* k_win, void* out, float* lse, char* base, int B, int H, int N,
                   int W, int M, int K, const Strides& st, const ExactStrides& es, float sm_scale, hipStream_t stream) {
    int s_far, s_win;
    windowed_splits(B, H, N, W, s_far, s_win);
    const int s_tot = s_far + s_win;
    const Workspace ws = plan(B, H, D, M, s_tot);
    float* lut = reinterpret_cast<float*>(base + ws.lut_off);
    float* po = reinterpret_cast<float*>(base + ws.po_off);
    float* pml = reinterpret_cast<float*>(base + ws.pml_off);
    int rc = VQA_OK;
    const int far = N - W;
    if (far > 0) {
        const int tiles = kLutStride / 16;
        hipLaunchKernelGGL((lut_kernel<Tag, D>), dim3((tiles + kWaves - 1) / kWaves, H * M), dim3(kThreads), 0, stream,
                           q_far, cb, lut, B, H, M, K, st, sm_scale * kLog2e, nullptr, nullptr);
        if ((rc = launch_status()) != VQA_OK) return rc;
        int kps = ((far + s_far - 1) / s_far + kThreads - 1) / kThreads * kThreads;
        switch (M) {
            case 1: rc = launch_main<Tag, D, 1>(codes, v, lut, po, pml, B, H, far, s_far, kps, st, nullptr, s_tot, 0, stream); break;
            case 2: rc = launch_main<Tag, D, 2>(codes, v, lut, po, pml, B, H, far, s_far, kps, st, nullptr, s_tot, 0, stream); break;
            case 4: rc = launch_main<Tag, D, 4>(codes, v, lut, po, pml, B, H, far, s_far, kps, st, nullptr, s_tot, 0, stream); break;
            case 8: rc = launch_main<Tag, D, 8>(codes, v, lut, po, pml, B, H, far, s_far, kps, st, nullptr, s_tot, 0, stream); break;
            default: return VQA_ERR_UNSUPPORTED_CODEBOOK;
        }
        if (rc != VQA_OK) return rc;
    }
    const int kps_w = ((W + s_win - 1) / s_win + kThreads - 1) / kThreads * kThreads;
    hipLaunchKernelGGL((exact_kernel<Tag, D>), dim3(s_win, B * H), dim3(kThreads), 0, stream, q_win, k_win,
                       v + (int64_t)far * st.v_n, po, pml, H, W, s_win, kps_w, es, sm_scale * kLog2e, s_tot, s_far);
    if ((rc = launch_status()) != VQA_OK) return rc;
    hipLaunchKernelGGL((merge_kernel<Tag, D>), dim3(B * H), dim3(D), 0, stream, po, pml, static_cast<uint16_t*>(out),
                       lse, H, s_tot, st);
    return launch_status();
}

template <typename Tag>
int run_windowed(const void* q_far, const void* q_win, const uint8_t* codes, const void* codebooks, const void* v,
                 const void* k_win, void* out, float* lse, void* workspace, size_t workspace_bytes, int B, int H, int N,
                 int W, int D, int M, int K, const int64_t* strides, float sm_scale, hipStream_t stream) {
    if (!q_far || !q_win || !codebooks || !v || !k_win || !out || !workspace || !strides) return VQA_ERR_NULL_POINTER;
    if (B <= 0 || H <= 0 || N <= 0 || W <= 0 || W > N) return VQA_ERR_BAD_SHAPE;
    if (N > W && !codes) return VQA_ERR_NULL_POINTER;
    if (D != 64 && D != 128) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    if ((M != 1 && M != 2 && M != 4 && M != 8) || K < 1 || K > 256) return VQA_ERR_UNSUPPORTED_CODEBOOK;
    Strides st = {};
    st.q_b = strides[0], st.q_h = strides[1];
    st.c_b = strides[4], st.c_h = strides[5];
    st.cb_h = strides[6], st.cb_m = strides[7], st.cb_k = strides[8];
    st.v_b = strides[9], st.v_h = strides[10], st.v_n = strides[11];
    st.o_b = strides[15], st.o_h = strides[16];
    ExactStrides es;
    es.q_b = strides[2], es.q_h = strides[3];
    es.k_b = strides[12], es.k_h = strides[13], es.k_n = strides[14];
    es.v_b = st.v_b, es.v_h = st.v_h, es.v_n = st.v_n;
    if (!aligned16(q_far) || !aligned16(q_win) || !aligned16(codebooks) || !aligned16(v) || !aligned16(k_win) ||
        ((uintptr_t)workspace & 255u))
        return VQA_ERR_MISALIGNED;
    if ((st.q_b | st.q_h | es.q_b | es.q_h | st.cb_h | st.cb_m | st.cb_k | st.v_b | st.v_h | st.v_n | es.k_b | es.k_h |
         es.k_n) & 7)
        return VQA_ERR_MISALIGNED;
    if (codes && (((uintptr_t)codes | (uintptr_t)st.c_b | (uintptr_t)st.c_h) & (uintptr_t)(M - 1)))
        return VQA_ERR_MISALIGNED;
    if ((int64_t)B * H > 65535 || !row_stride_ok(st.v_n) || !row_stride_ok(es.k_n)) return VQA_ERR_BAD_ARGUMENT;
    int s_far, s_win;
    windowed_splits(B, H, N, W, s_far, s_win);
    if (workspace_bytes < plan(B, H, D, M, s_far + s_win).total) return VQA_ERR_WORKSPACE_TOO_SMALL;
    const uint16_t* qf = static_cast<const uint16_t*>(q_far);
    const uint16_t* qw = static_cast<const uint16_t*>(q_win);
    const uint16_t* cb = static_cast<const uint16_t*>(codebooks);
    const uint16_t* v16 = static_cast<const uint16_t*>(v);
    const uint16_t* kw = static_cast<const uint16_t*>(k_win);
    char* base = static_cast<char*>(workspace);
    if (D == 64)
        return run_windowed_d<Tag, 64>(qf, qw, codes, cb, v16, kw, out, lse, base, B, H, N, W, M, K, st, es, sm_scale,
                                       stream);
    return run_windowed_d<Tag, 128>(qf, qw, codes, cb, v16, kw, out, lse, base, B, H, N, W, M, K, st, es, sm_scale,
                                    stream);
}

}  // namespace decode
}  // namespace vqa

extern "C" {

size_t vqa_decode_windowed_workspace_bytes(int B, int H, int N, int W, int D, int M) {
    if (B <= 0 || H <= 0 || N <= 0 || W <= 0 || W > N || D <= 0 || M <= 0) return 0;
    int s_far, s_win;
    vqa::decode::windowed_splits(B, H, N, W, s_far, s_win);
    return vqa::decode::plan(B, H, D, M, s_far + s_win).total;
}

int vqa_decode_windowed_bf16(const void* q_far, const void* q_win, const uint8_t* codes, const void* codebooks,
                             const void* v, const void* k_win, void* out, float* lse, void* workspace,
                             size_t workspace_bytes, int B, int H, int N, int W, int D, int M, int K,
                             const int64_t* strides, float sm_scale, vqa_stream_t stream) {
    return vqa::decode::run_windowed<vqa::bf16_tag>(q_far, q_win, codes, codebooks, v, k_win, out, lse, workspace,
                                                    workspace_bytes, B, H, N, W, D, M, K, strides, sm_scale, stream);
}

int vqa_decode_windowed_f16(const void* q_far, const void* q_win, const uint8_t* codes, const void* codebooks,
                            const void* v, const void* k_win, void* out, float* lse, void* workspace,
                            size_t workspace_bytes, int B, int H, int N, int W, int D, int M, int K,
                            const int64_t* strides, float sm_scale, vqa_stream_t stream) {
    return vqa::decode::run_windowed<vqa::f16_tag>(q_far, q_win, codes, codebooks, v, k_win, out, lse, workspace,
                                                   workspace_bytes, B, H, N, W, D, M, K, strides, sm_scale, stream);
}

size_t vqa_decode_exact_workspace_bytes(int B, int H, int N, int D, int num_splits) {
    if (B <= 0 || H <= 0 || N <= 0 || D <= 0) return 0;
    const int S = num_splits > 0 ? num_splits : vqa::decode::default_splits(B, H, N);
    return vqa::decode::plan(B, H, D, 0, S).total;
}

int vqa_decode_exact_bf16(const void* q, const void* k, const void* v, void* out, float* lse, void* workspace,
                          size_t workspace_bytes, int B, int H, int N, int D, const int64_t* strides, float sm_scale,
                          int num_splits, vqa_stream_t stream) {
    return vqa::decode::run_exact<vqa::bf16_tag>(q, k, v, out, lse, workspace, workspace_bytes, B, H, N, D, strides,
                                                 sm_scale, num_splits, stream);
}

int vqa_decode_exact_f16(const void* q, const void* k, const void* v, void* out, float* lse, void* workspace,
                         size_t workspace_bytes, int B, int H, int N, int D, const int64_t* strides, float sm_scale,
                         int num_splits, vqa_stream_t stream) {
    return vqa::decode::run_exact<vqa::f16_tag>(q, k, v, out, lse, workspace, workspace_bytes, B, H, N, D, strides,
                                                sm_scale, num_splits, stream);
}

int vqa_decode_default_splits(int B, int H, int N) { return vqa::decode::default_splits(B, H, N); }

size_t vqa_decode_workspace_bytes(int B, int H, int N, int D, int M, int K, int num_splits) {
    (void)K;
    if (B <= 0 || H <= 0 || N <= 0 || D <= 0 || M <= 0) return 0;
    const int S = num_splits > 0 ? num_splits : vqa::decode::default_splits(B, H, N);
    return vqa::decode::plan(B, H, D, M, S).total;
}

int vqa_decode_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, void* out, float* lse,
                    void* workspace, size_t workspace_bytes, int B, int H, int N, int D, int M, int K,
                    const int64_t* strides, float sm_scale, int num_splits, vqa_stream_t stream) {
    return vqa::decode::run<vqa::bf16_tag>(q, codes, codebooks, v, out, lse, workspace, workspace_bytes, B, H, N, D, M,
                                           K, strides, sm_scale, num_splits, nullptr, stream);
}

int vqa_decode_f16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, void* out, float* lse,
                   void* workspace, size_t workspace_bytes, int B, int H, int N, int D, int M, int K,
                   const int64_t* strides, float sm_scale, int num_splits, vqa_stream_t stream) {
    return vqa::decode::run<vqa::f16_tag>(q, codes, codebooks, v, out, lse, workspace, workspace_bytes, B, H, N, D, M,
                                          K, strides, sm_scale, num_splits, nullptr, stream);
}

int vqa_decode_static_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, void* out,
                           float* lse, int B, int H, int N, int D, int M, int K, const int64_t* strides, float sm_scale,
                           int num_splits, vqa_stream_t stream) {
    // the size check comes first and needs no device: a problem beyond the static scratch is refused outright
    if (B <= 0 || H <= 0 || N <= 0 || D <= 0 || M <= 0) return VQA_ERR_BAD_SHAPE;
    const int S = num_splits > 0 ? num_splits : vqa::decode::default_splits(B, H, N);
    if (vqa::decode::plan(B, H, D, M, S).total > (size_t)VQA_DECODE_STATIC_SCRATCH_BYTES) return VQA_ERR_SCRATCH_LIMIT;
    void* ws = nullptr;
    const int rc = vqa::decode::static_scratch(q, &ws);
    if (rc != VQA_OK) return rc;
    return vqa::decode::run<vqa::bf16_tag>(q, codes, codebooks, v, out, lse, ws, VQA_DECODE_STATIC_SCRATCH_BYTES, B, H,
                                           N, D, M, K, strides, sm_scale, S, nullptr, stream);
}

int vqa_decode_devlen_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, void* out,
                           float* lse, void* workspace, size_t workspace_bytes, int B, int H, int N_max, int D, int M,
                           int K, const int64_t* strides, float sm_scale, int num_splits, const int32_t* n_keys_dev,
                           vqa_stream_t stream) {
    if (!n_keys_dev) return VQA_ERR_NULL_POINTER;
    return vqa::decode::run<vqa::bf16_tag>(q, codes, codebooks, v, out, lse, workspace, workspace_bytes, B, H, N_max, D,
                                           M, K, strides, sm_scale, num_splits, n_keys_dev, stream);
}

int vqa_decode_devlen_f16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, void* out,
                          float* lse, void* workspace, size_t workspace_bytes, int B, int H, int N_max, int D, int M,
                          int K, const int64_t* strides, float sm_scale, int num_splits, const int32_t* n_keys_dev,
                          vqa_stream_t stream) {
    if (!n_keys_dev) return VQA_ERR_NULL_POINTER;
    return vqa::decode::run<vqa::f16_tag>(q, codes, codebooks, v, out, lse, workspace, workspace_bytes, B, H, N_max, D,
                                          M, K, strides, sm_scale, num_splits, n_keys_dev, stream);
}

int vqa_decode_roped_bf16(const void* q, const void* rope_cos, const void* rope_sin, const uint8_t* codes,
                          const void* codebooks, const void* v, void* out, float* lse, void* workspace,
                          size_t workspace_bytes, int B, int H, int N_max, int D, int M, int K, const int64_t* strides,
                          float sm_scale, int num_splits, const int32_t* n_keys_dev, vqa_stream_t stream) {
    if (!rope_cos || !rope_sin) return VQA_ERR_NULL_POINTER;
    return vqa::decode::run<vqa::bf16_tag>(q, codes, codebooks, v, out, lse, workspace, workspace_bytes, B, H, N_max, D,
                                           M, K, strides, sm_scale, num_splits, n_keys_dev, stream, rope_cos, rope_sin);
}

int vqa_decode_roped_f16(const void* q, const void* rope_cos, const void* rope_sin, const uint8_t* codes,
                         const void* codebooks, const void* v, void* out, float* lse, void* workspace,
                         size_t workspace_bytes, int B, int H, int N_max, int D, int M, int K, const int64_t* strides,
                         float sm_scale, int num_splits, const int32_t* n_keys_dev, vqa_stream_t stream) {
    if (!rope_cos || !rope_sin) return VQA_ERR_NULL_POINTER;
    return vqa::decode::run<vqa::f16_tag>(q, codes, codebooks, v, out, lse, workspace, workspace_bytes, B, H, N_max, D,
                                          M, K, strides, sm_scale, num_splits, n_keys_dev, stream, rope_cos, rope_sin);
}

}  // extern "C"
