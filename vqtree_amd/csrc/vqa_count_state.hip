// Count state of a single-codebook VQ key cache, and the generation step over it.
//
// With one codebook every quantised key IS a codeword, so attention over N quantised keys collapses to attention over
// the C codewords with weights:  sum_j exp(q.cb[id_j]) v_j = sum_c exp(q.cb[c]) Vsum[c],  Z = sum_c cnt[c] exp(q.cb[c])
// where cnt[c] = #{j : id_j = c} and Vsum[c] = sum of the values of those keys.  The state (cnt [B,H,C] int32,
// Vsum [B,H,C,D] fp32) is what the reference's cache stores after a prefill (key counts and cumulated values,
// ops/attn_vq.py:89-127); a generation step costs O(C D) whatever the context length.
//
//   count_state_add : fold T more keys (codeword ids and values) into the state, in position order (deterministic:
//                     every (b, h, codeword) is owned by one workgroup, no atomics)
//   count_decode    : one query per (b, h) against the state -> normalised output and base-2 log-sum-exp, ready to be
//                     merged with the state of an exact window
#include "vqa_common.h"

namespace vqa {
namespace count_state {

// Codewords owned by one workgroup of count_state_add.  A workgroup scans all T ids whatever it owns, so many keys
// want many small groups (more workgroups in flight to hide the latency of the scan and of the row loads: 8192 keys,
// 512 codewords, 32 heads take 251 us with 16 codewords per group and 195 us with 4), while the single key of a
// generation step wants few, large groups (the launch is all fixed cost).
constexpr int kCodesManyKeys = 4;
constexpr int kCodesFewKeys = 32;
constexpr int kManyKeys = 1024;
constexpr int kBatch = 8;           // value rows whose loads are in flight together

// grid (C / kCodesPerGroup groups, B*H), D threads: thread d owns element d of the group's accumulators.
template <typename Tag, int D, int kCodesPerGroup>
__global__ __launch_bounds__(D) void add_kernel(const int64_t* __restrict__ ids, const uint16_t* __restrict__ v,
                                                int32_t* __restrict__ cnt, float* __restrict__ vsum, int H, int T, int C,
                                                int64_t i_sb, int64_t i_sh, int64_t i_st, int64_t v_sb, int64_t v_sh,
                                                int64_t v_st) {
    constexpr int kWaves = D / kWave;
    __shared__ int s_list[D];        // positions of the chunk's keys that belong to this group, in order
    __shared__ int s_code[D];        // their codeword (0..15 within the group)
    __shared__ int s_wave_n[kWaves];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bh = blockIdx.y, b = bh / H, h = bh % H;
    const int c0 = blockIdx.x * kCodesPerGroup;
    const int64_t* my_ids = ids + b * i_sb + h * i_sh;
    const uint16_t* my_v = v + b * v_sb + h * v_sh;

    float acc[kCodesPerGroup];
    int n[kCodesPerGroup];
#pragma unroll
    for (int c = 0; c < kCodesPerGroup; ++c) {
        acc[c] = 0.f;
        n[c] = 0;
    }
    for (int t0 = 0; t0 < T; t0 += D) {
        // order-preserving compaction of the chunk's keys that belong to this group
        const int t = t0 + tid;
        // an id outside [0, C) counts as the nearest valid codeword, the rule of every kernel that reads ids or codes
        // (preprocessing, key reconstruction, lookup table): the state then matches the prefill of the same cache
        const int64_t raw = t < T ? my_ids[t * i_st] : 0;
        const int64_t id = raw < 0 ? 0 : (raw >= C ? C - 1 : raw);
        const int64_t rel = id - c0;
        const bool mine = t < T && rel >= 0 && rel < kCodesPerGroup;
        const uint64_t mask = __builtin_amdgcn_ballot_w64(mine);
        if (lane == 0) s_wave_n[wave] = __builtin_popcountll(mask);
        __syncthreads();
        int base = 0, total = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const int nw = s_wave_n[w];
            if (w < wave) base += nw;
            total += nw;
        }
        if (mine) {
            const int slot = base + __builtin_popcountll(mask & ((uint64_t(1) << lane) - 1));
            s_list[slot] = t;
            s_code[slot] = (int)rel;
        }
        __syncthreads();
        // thread d adds element d of every listed row, kBatch rows' loads in flight together
        for (int i0 = 0; i0 < total; i0 += kBatch) {
            float x[kBatch];
            int code[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                const int i = min(i0 + j, total - 1);
                code[j] = (i0 + j < total) ? s_code[i] : -1;
                x[j] = Elem<Tag>::from_bits(my_v[(int64_t)s_list[i] * v_st + tid]);
            }
#pragma unroll
            for (int j = 0; j < kBatch; ++j)
#pragma unroll
                for (int c = 0; c < kCodesPerGroup; ++c) {  // compile-time register index: no scratch
                    if (code[j] == c) {
                        acc[c] += x[j];
                        n[c] += 1;
                    }
                }
        }
        __syncthreads();  // the lists are rewritten by the next chunk
    }
    const int n_codes = min(kCodesPerGroup, C - c0);
#pragma unroll
    for (int c = 0; c < kCodesPerGroup; ++c) {
        if (c < n_codes && n[c] > 0) {
            const int64_t row = (int64_t)bh * C + c0 + c;
            vsum[row * D + tid] += acc[c];
            if (tid == 0) cnt[row] += n[c];
        }
    }
}

// grid B*H, 256 threads.
constexpr int kDecodeThreads = 256;

// What a generation step adds to the plain decode (all null / unused for vqa_count_decode_*): the new key, folded into
// the state before the query attends to it, and the rotary of the raw query.
struct StepArgs {
    const int64_t* id;      // [B,H] codeword of the new key (clamped into [0, C)); null: plain decode
    int64_t id_sb, id_sh;
    const uint16_t* v;      // [B,H,D] value of the new key
    int64_t v_sb, v_sh;
    const uint16_t* cos;    // [D] rotary rows of the query's position; null: the query comes rotated
    const uint16_t* sin;
};

template <typename Tag>
__device__ __forceinline__ float rnd_elem(float x) { return Elem<Tag>::round_keep_f32(x); }

template <typename Tag, int D>
__global__ __launch_bounds__(kDecodeThreads) void decode_kernel(const uint16_t* __restrict__ q,
                                                                const uint16_t* __restrict__ codebook,
                                                                int32_t* __restrict__ cnt, float* __restrict__ vsum,
                                                                uint16_t* __restrict__ out, float* __restrict__ lse,
                                                                int H, int C, int64_t q_sb, int64_t q_sh, int64_t cb_sh,
                                                                int64_t cb_sc, int64_t o_sb, int64_t o_sh,
                                                                float scale_log2e, StepArgs step) {
    extern __shared__ float s_e[];  // C scores, then weights exp2(score - max) (0 for codewords with no key)
    __shared__ uint32_t s_q[D / 2];
    __shared__ uint32_t s_raw[D / 2];
    __shared__ float s_red[kDecodeThreads / kWave];
    __shared__ float s_part[kDecodeThreads / (D / 4)][D];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bh = blockIdx.x, b = bh / H, h = bh % H;
    const uint16_t* my_q = q + b * q_sb + h * q_sh;
    const uint16_t* my_cb = codebook + h * cb_sh;
    int32_t* my_cnt = cnt + (int64_t)bh * C;
    float* my_vsum = vsum + (int64_t)bh * C * D;

    // A generation step folds the new key in first: cnt[id] += 1, Vsum[id] += v (the fp32 additions of
    // vqa_count_state_add_*).  One workgroup owns the (batch, head): the barrier below orders these writes before its
    // own reads of the state.
    if (step.id != nullptr) {
        const int64_t raw = step.id[b * step.id_sb + h * step.id_sh];
        const int id = (int)(raw < 0 ? 0 : (raw >= C ? C - 1 : raw));
        if (tid < D) my_vsum[(int64_t)id * D + tid] += Elem<Tag>::from_bits(step.v[b * step.v_sb + h * step.v_sh + tid]);
        if (tid == 0) my_cnt[id] += 1;
    }
    if (step.cos == nullptr) {
        if (tid < D / 2) s_q[tid] = reinterpret_cast<const uint32_t*>(my_q)[tid];
    } else {
        // q' = q * cos + rotate_half(q) * sin, every product and the sum rounded to the element type (the bits
        // vqa_rope_* writes): element pair t of the lower half has its partner pair at t + D/4, and vice versa
        if (tid < D / 2) s_raw[tid] = reinterpret_cast<const uint32_t*>(my_q)[tid];
        __syncthreads();
        if (tid < D / 2) {
#pragma clang fp contract(off)
            const bool upper = tid >= D / 4;
            const uint32_t x = s_raw[tid], xp = s_raw[tid ^ (D / 4)];
            const uint32_t cw = reinterpret_cast<const uint32_t*>(step.cos)[tid];
            const uint32_t sw = reinterpret_cast<const uint32_t*>(step.sin)[tid];
            uint32_t pair = 0;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int sh = 16 * t;
                const float xv = Elem<Tag>::from_bits((uint16_t)(x >> sh)), pv = Elem<Tag>::from_bits((uint16_t)(xp >> sh));
                const float cv = Elem<Tag>::from_bits((uint16_t)(cw >> sh)), sv = Elem<Tag>::from_bits((uint16_t)(sw >> sh));
                const float t0 = rnd_elem<Tag>(xv * cv), t1 = rnd_elem<Tag>(pv * sv);
                pair |= (uint32_t)Elem<Tag>::to_bits(rnd_elem<Tag>(upper ? t0 + t1 : t0 - t1)) << sh;
            }
            s_q[tid] = pair;
        }
    }
    __threadfence_block();
    __syncthreads();

    // scores: one codeword per thread; the query is read from LDS at a wave-uniform address (broadcast)
    float m = -INFINITY;
    for (int c = tid; c < C; c += kDecodeThreads) {
        const uint4* row = reinterpret_cast<const uint4*>(my_cb + (int64_t)c * cb_sc);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < D / 8; ++i) {
            const uint4 kx = row[i];
            s = Elem<Tag>::dot2(kx.x, s_q[4 * i + 0], s);
            s = Elem<Tag>::dot2(kx.y, s_q[4 * i + 1], s);
            s = Elem<Tag>::dot2(kx.z, s_q[4 * i + 2], s);
            s = Elem<Tag>::dot2(kx.w, s_q[4 * i + 3], s);
        }
        s *= scale_log2e;
        s_e[c] = s;
        if (my_cnt[c] > 0) m = fmaxf(m, s);
    }
    m = wave_max(m);
    if (lane == 0) s_red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
    __syncthreads();
    float z = 0.f;
    for (int c = tid; c < C; c += kDecodeThreads) {
        const int n = my_cnt[c];
        const float e = n > 0 ? fast_exp2(s_e[c] - m) : 0.f;
        s_e[c] = e;
        z += e * (float)n;
    }
    z = wave_sum(z);
    if (lane == 0) s_red[wave] = z;
    __syncthreads();
    z = (s_red[0] + s_red[1]) + (s_red[2] + s_red[3]);

    // out[d] = sum_c e_c Vsum[c][d]: D/4 lanes cover a row (16 bytes each), the groups of lanes take rows in turn
    constexpr int kLanesPerRow = D / 4, kGroups = kDecodeThreads / kLanesPerRow;
    const int g = tid / kLanesPerRow, dl = tid % kLanesPerRow;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int c = g; c < C; c += kGroups) {
        const float e = s_e[c];
        if (e != 0.f) acc += e * *reinterpret_cast<const f32x4_t*>(my_vsum + (int64_t)c * D + dl * 4);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) s_part[g][dl * 4 + i] = acc[i];
    __syncthreads();
    if (tid < D) {
        float o = 0.f;
#pragma unroll
        for (int gg = 0; gg < kGroups; ++gg) o += s_part[gg][tid];
        const float inv = z > 0.f ? 1.f / z : 0.f;
        out[b * o_sb + h * o_sh + tid] = Elem<Tag>::to_bits(o * inv);
    }
    if (tid == 0 && lse) lse[bh] = z > 0.f ? m + fast_log2(z) : -INFINITY;
}

template <typename Tag>
int add(const int64_t* ids, const void* v, int32_t* cnt, float* vsum, int B, int H, int T, int D, int C,
        const int64_t* st, hipStream_t stream) {
    if (B <= 0 || H <= 0 || T < 0 || C <= 0) return VQA_ERR_BAD_SHAPE;
    if (D != 64 && D != 128) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    if (!ids || !v || !cnt || !vsum || !st) return VQA_ERR_NULL_POINTER;
    if (T == 0) return VQA_OK;
    if ((int64_t)B * H > 65535) return VQA_ERR_BAD_SHAPE;
    const uint16_t* vp = static_cast<const uint16_t*>(v);
    auto launch = [&](auto kernel, int codes_per_group, int threads) {
        const dim3 grid((C + codes_per_group - 1) / codes_per_group, B * H);
        hipLaunchKernelGGL(kernel, grid, dim3(threads), 0, stream, ids, vp, cnt, vsum, H, T, C, st[0], st[1], st[2],
                           st[3], st[4], st[5]);
    };
    const bool many = T >= kManyKeys;
    if (D == 64 && many) launch(add_kernel<Tag, 64, kCodesManyKeys>, kCodesManyKeys, 64);
    if (D == 64 && !many) launch(add_kernel<Tag, 64, kCodesFewKeys>, kCodesFewKeys, 64);
    if (D == 128 && many) launch(add_kernel<Tag, 128, kCodesManyKeys>, kCodesManyKeys, 128);
    if (D == 128 && !many) launch(add_kernel<Tag, 128, kCodesFewKeys>, kCodesFewKeys, 128);
    return launch_status();
}

template <typename Tag>
int decode(const void* q, const void* codebook, int32_t* cnt, float* vsum, void* out, float* lse, int B, int H, int C,
           int D, const int64_t* st, float sm_scale, hipStream_t stream, const StepArgs& step) {
    if (B <= 0 || H <= 0 || C <= 0 || C > VQA_COUNT_STATE_MAX_CODES) return VQA_ERR_BAD_SHAPE;
    if (D != 64 && D != 128) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    if (!q || !codebook || !cnt || !vsum || !out || !st) return VQA_ERR_NULL_POINTER;
    if (!aligned16(codebook) || (st[2] % 8) || (st[3] % 8) || (reinterpret_cast<uintptr_t>(q) & 3u) || (st[0] % 2) ||
        (st[1] % 2) || !aligned16(vsum))
        return VQA_ERR_MISALIGNED;
    if ((reinterpret_cast<uintptr_t>(step.cos) | reinterpret_cast<uintptr_t>(step.sin)) & 3u) return VQA_ERR_MISALIGNED;
    if ((int64_t)B * H > 0x7fffffff) return VQA_ERR_BAD_SHAPE;
    const uint16_t* qp = static_cast<const uint16_t*>(q);
    const uint16_t* cb = static_cast<const uint16_t*>(codebook);
    uint16_t* op = static_cast<uint16_t*>(out);
    const size_t lds = (size_t)C * sizeof(float);
    const float scale_log2e = sm_scale * kLog2e;
    if (D == 64)
        hipLaunchKernelGGL((decode_kernel<Tag, 64>), dim3(B * H), dim3(kDecodeThreads), lds, stream, qp, cb, cnt, vsum,
                           op, lse, H, C, st[0], st[1], st[2], st[3], st[4], st[5], scale_log2e, step);
    else
        hipLaunchKernelGGL((decode_kernel<Tag, 128>), dim3(B * H), dim3(kDecodeThreads), lds, stream, qp, cb, cnt, vsum,
                           op, lse, H, C, st[0], st[1], st[2], st[3], st[4], st[5], scale_log2e, step);
    return launch_status();
}

// strides: q(b,h) codebook(h,c) out(b,h) id(b,h) v(b,h)
template <typename Tag>
int step(const void* q, const void* rope_cos, const void* rope_sin, const int64_t* id, const void* v,
         const void* codebook, int32_t* cnt, float* vsum, void* out, float* lse, int B, int H, int C, int D,
         const int64_t* st, float sm_scale, hipStream_t stream) {
    if (!id || !v || !st) return VQA_ERR_NULL_POINTER;
    if ((rope_cos == nullptr) != (rope_sin == nullptr)) return VQA_ERR_NULL_POINTER;
    StepArgs a;
    a.id = id, a.id_sb = st[6], a.id_sh = st[7];
    a.v = static_cast<const uint16_t*>(v), a.v_sb = st[8], a.v_sh = st[9];
    a.cos = static_cast<const uint16_t*>(rope_cos), a.sin = static_cast<const uint16_t*>(rope_sin);
    return decode<Tag>(q, codebook, cnt, vsum, out, lse, B, H, C, D, st, sm_scale, stream, a);
}

}  // namespace count_state
}  // namespace vqa

extern "C" {

int vqa_count_state_add_bf16(const int64_t* ids, const void* v, int32_t* cnt, float* vsum, int B, int H, int T, int D,
                             int C, const int64_t* strides, vqa_stream_t stream) {
    return vqa::count_state::add<vqa::bf16_tag>(ids, v, cnt, vsum, B, H, T, D, C, strides, stream);
}
int vqa_count_state_add_f16(const int64_t* ids, const void* v, int32_t* cnt, float* vsum, int B, int H, int T, int D,
                            int C, const int64_t* strides, vqa_stream_t stream) {
    return vqa::count_state::add<vqa::f16_tag>(ids, v, cnt, vsum, B, H, T, D, C, strides, stream);
}
int vqa_count_decode_bf16(const void* q, const void* codebook, const int32_t* cnt, const float* vsum, void* out,
                          float* lse, int B, int H, int C, int D, const int64_t* strides, float sm_scale,
                          vqa_stream_t stream) {
    return vqa::count_state::decode<vqa::bf16_tag>(q, codebook, const_cast<int32_t*>(cnt), const_cast<float*>(vsum), out,
                                                   lse, B, H, C, D, strides, sm_scale, stream,
                                                   vqa::count_state::StepArgs{});
}
int vqa_count_decode_f16(const void* q, const void* codebook, const int32_t* cnt, const float* vsum, void* out,
                         float* lse, int B, int H, int C, int D, const int64_t* strides, float sm_scale,
                         vqa_stream_t stream) {
    return vqa::count_state::decode<vqa::f16_tag>(q, codebook, const_cast<int32_t*>(cnt), const_cast<float*>(vsum), out,
                                                  lse, B, H, C, D, strides, sm_scale, stream,
                                                  vqa::count_state::StepArgs{});
}

int vqa_count_step_bf16(const void* q, const void* rope_cos, const void* rope_sin, const int64_t* id, const void* v,
                        const void* codebook, int32_t* cnt, float* vsum, void* out, float* lse, int B, int H, int C,
                        int D, const int64_t* strides, float sm_scale, vqa_stream_t stream) {
    return vqa::count_state::step<vqa::bf16_tag>(q, rope_cos, rope_sin, id, v, codebook, cnt, vsum, out, lse, B, H, C, D,
                                                 strides, sm_scale, stream);
}
int vqa_count_step_f16(const void* q, const void* rope_cos, const void* rope_sin, const int64_t* id, const void* v,
                       const void* codebook, int32_t* cnt, float* vsum, void* out, float* lse, int B, int H, int C,
                       int D, const int64_t* strides, float sm_scale, vqa_stream_t stream) {
    return vqa::count_state::step<vqa::f16_tag>(q, rope_cos, rope_sin, id, v, codebook, cnt, vsum, out, lse, B, H, C, D,
                                                strides, sm_scale, stream);
}

}  // extern "C"
