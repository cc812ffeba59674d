// Inputs of the count kernel from per-key code ids, without a one-hot cumulative sum or a sort:
//
//   cnt[t, c]  = #{ j < (t+1)*128 : id_j == c }                            (t < N / 128)
//   start[c]   = #{ j < N : id_j < c }                                      (first sorted row of code c)
//   vi[t, c]   = cnt[t, c] + start[c]
//   v_vq[0]    = 0;   v_vq[1 + r] = sum of V over the keys of r's code up to and including sorted row r,
//                where keys are ordered by (code, position)
//
// Passes per (batch, head): per-128-key histograms; a running sum over blocks, an exclusive scan over codes and the
// block-sampled outputs;
// a scatter of key positions into sorted order (rank = start + keys of the code in earlier blocks + earlier keys of
// the code in the same block); one wave per code walking its segment with an fp32 running sum.
#include "vqa_common.h"

namespace vqa {
namespace prep {

constexpr int kBlock = 128;
constexpr int kMaxCodes = 8192;

struct Params {
    const int64_t* ids;
    int64_t id_sb, id_sh, id_sn;
    const uint16_t* v;
    int64_t v_sb, v_sh, v_sn;
    int64_t* cnt;       // nullable
    int64_t cn_sb, cn_sh, cn_st;
    uint16_t* cnt_elem; // nullable
    int64_t ce_sb, ce_sh, ce_st;
    uint16_t* vvq;
    int64_t vq_sb, vq_sh, vq_sn;
    int64_t* vi;
    int64_t vi_sb, vi_sh, vi_st;
    int32_t* hist;      // [B*H, NB, C]   per-block histograms, then inclusive running counts
    int32_t* start;     // [B*H, C]
    int32_t* order;     // [B*H, N]       key position of every sorted row
    int32_t* state_cnt; // nullable: [B*H, C]    keys per code over the whole sequence
    float* state_vsum;  // nullable: [B*H, C, D] fp32 value sum per code over the whole sequence
    int H, N, D, C, NB; // NB = ceil(N / 128)
};

__device__ __forceinline__ int load_id(const Params& p, int b, int h, int j) {
    const int64_t id = p.ids[b * p.id_sb + h * p.id_sh + (int64_t)j * p.id_sn];
    return (int)min(max(id, (int64_t)0), (int64_t)(p.C - 1));  // an id outside [0, C) is clamped, never dereferenced
}

__global__ __launch_bounds__(kBlock) void hist_kernel(Params p) {
    extern __shared__ int s_hist[];
    const int t = blockIdx.x, bh = blockIdx.y;
    const int b = bh / p.H, h = bh % p.H;
    for (int c = threadIdx.x; c < p.C; c += kBlock) s_hist[c] = 0;
    __syncthreads();
    const int j = t * kBlock + threadIdx.x;
    if (j < p.N) atomicAdd(&s_hist[load_id(p, b, h, j)], 1);
    __syncthreads();
    int32_t* out = p.hist + ((int64_t)bh * p.NB + t) * p.C;
    for (int c = threadIdx.x; c < p.C; c += kBlock) out[c] = s_hist[c];
}

// running count over blocks, in place; one thread per code.  total[c] lands in `start` until start_kernel replaces it.
__global__ __launch_bounds__(256) void cumulate_kernel(Params p) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    const int bh = blockIdx.y;
    if (c >= p.C) return;
    int32_t* hist = p.hist + (int64_t)bh * p.NB * p.C + c;
    int run = 0;
    for (int t = 0; t < p.NB; ++t) {
        run += hist[(int64_t)t * p.C];
        hist[(int64_t)t * p.C] = run;
    }
    p.start[(int64_t)bh * p.C + c] = run;
}

// start[c] = exclusive prefix sum of the totals over codes; one workgroup per (batch, head)
__global__ __launch_bounds__(256) void start_kernel(Params p) {
    __shared__ int s_part[256];
    const int bh = blockIdx.x;
    const int tid = threadIdx.x;
    int32_t* start = p.start + (int64_t)bh * p.C;
    const int strip = (p.C + 255) / 256;  // every thread owns a contiguous strip of codes
    const int c_lo = min(tid * strip, p.C), c_hi = min(c_lo + strip, p.C);
    int sum = 0;
    for (int c = c_lo; c < c_hi; ++c) sum += start[c];
    s_part[tid] = sum;
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int i = 0; i < 256; ++i) {
            const int x = s_part[i];
            s_part[i] = run;
            run += x;
        }
    }
    __syncthreads();
    int run = s_part[tid];
    for (int c = c_lo; c < c_hi; ++c) {
        const int x = start[c];
        start[c] = run;
        run += x;
    }
}

// block-sampled outputs: cnt[t, c], its element-type copy, vi[t, c] = cnt + start[c]
template <typename Tag>
__global__ __launch_bounds__(256) void emit_kernel(Params p) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    const int t = blockIdx.y, bh = blockIdx.z;
    const int b = bh / p.H, h = bh % p.H;
    if (c >= p.C) return;
    const int n = p.hist[((int64_t)bh * p.NB + t) * p.C + c];
    if (p.cnt) p.cnt[b * p.cn_sb + h * p.cn_sh + (int64_t)t * p.cn_st + c] = n;
    if (p.cnt_elem) p.cnt_elem[b * p.ce_sb + h * p.ce_sh + (int64_t)t * p.ce_st + c] = Elem<Tag>::to_bits((float)n);
    p.vi[b * p.vi_sb + h * p.vi_sh + (int64_t)t * p.vi_st + c] = (int64_t)n + p.start[(int64_t)bh * p.C + c];
}

__global__ __launch_bounds__(kBlock) void scatter_kernel(Params p) {
    __shared__ int s_id[kBlock];
    const int t = blockIdx.x, bh = blockIdx.y;
    const int b = bh / p.H, h = bh % p.H;
    const int j = t * kBlock + threadIdx.x;
    const int id = j < p.N ? load_id(p, b, h, j) : -1;
    s_id[threadIdx.x] = id;
    __syncthreads();
    if (j >= p.N) return;
    int earlier = 0;  // keys of the same code earlier in this block
    for (int i = 0; i < (int)threadIdx.x; ++i) earlier += s_id[i] == id;
    const int before = t > 0 ? p.hist[((int64_t)bh * p.NB + t - 1) * p.C + id] : 0;
    const int rank = p.start[(int64_t)bh * p.C + id] + before + earlier;
    p.order[(int64_t)bh * p.N + rank] = j;
}

// One wave per code: running fp32 sum of V over the code's keys in position order.  The sorted positions are
// fetched 64 at a time (one per lane) and the V rows eight at a time, so only the additions form a dependent chain.
// The totals the wave ends with are the count state of the sequence (per-code key count and fp32 value sum, what
// vqa_count_state_add_* would build from the same keys, same order of additions): written out when asked for.
template <typename Tag>
__global__ __launch_bounds__(256) void segment_sum_kernel(Params p) {
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int bh = blockIdx.y;
    const int b = bh / p.H, h = bh % p.H;
    if (c >= p.C) return;
    const int d = lane * 2;
    const bool live = d < p.D;
    const int dd = live ? d : 0;  // idle lanes shadow column 0 and never store
    uint16_t* out = p.vvq + b * p.vq_sb + h * p.vq_sh + dd;
    if (c == 0 && live) *reinterpret_cast<uint32_t*>(out) = 0u;  // row 0
    const int s = p.start[(int64_t)bh * p.C + c];
    const int e = s + p.hist[((int64_t)bh * p.NB + p.NB - 1) * p.C + c];
    const int32_t* order = p.order + (int64_t)bh * p.N;
    const uint16_t* v = p.v + b * p.v_sb + h * p.v_sh + dd;
    float a0 = 0.f, a1 = 0.f;
    for (int r0 = s; r0 < e; r0 += 64) {
        const int n = min(64, e - r0);
        const int mine = order[r0 + min(lane, n - 1)];
        for (int k0 = 0; k0 < n; k0 += 8) {
            uint32_t w[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int j = __shfl(mine, min(k0 + u, n - 1), 64);
                w[u] = *reinterpret_cast<const uint32_t*>(v + (int64_t)j * p.v_sn);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (k0 + u < n) {
                    a0 += Elem<Tag>::from_bits((uint16_t)(w[u] & 0xffffu));
                    a1 += Elem<Tag>::from_bits((uint16_t)(w[u] >> 16));
                    if (live)
                        *reinterpret_cast<uint32_t*>(out + (int64_t)(1 + r0 + k0 + u) * p.vq_sn) =
                            (uint32_t)Elem<Tag>::to_bits(a0) | ((uint32_t)Elem<Tag>::to_bits(a1) << 16);
                }
            }
        }
    }
    if (p.state_vsum != nullptr && live)
        *reinterpret_cast<float2*>(p.state_vsum + ((int64_t)bh * p.C + c) * p.D + d) = make_float2(a0, a1);
    if (p.state_cnt != nullptr && lane == 0) p.state_cnt[(int64_t)bh * p.C + c] = e - s;
}

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

inline size_t workspace_bytes(int B, int H, int N, int C) {
    if (B <= 0 || H <= 0 || N <= 0 || C <= 0) return 0;
    const size_t bh = (size_t)B * H, nb = (size_t)(N + kBlock - 1) / kBlock;
    return align256(bh * nb * C * 4) + align256(bh * C * 4) + align256(bh * (size_t)N * 4);
}

// strides: ids(b,h,n) v(b,h,n) cnt(b,h,t) cnt_elem(b,h,t) v_vq(b,h,n) vi(b,h,t); last dims contiguous
template <typename Tag>
int preprocess(const int64_t* ids, const void* v, int64_t* cnt, void* cnt_elem, void* v_vq, int64_t* vi,
               void* workspace, size_t ws_bytes, int B, int H, int N, int D, int C, const int64_t* strides,
               hipStream_t stream, int32_t* state_cnt = nullptr, float* state_vsum = nullptr) {
    if (!ids || !v || !v_vq || !workspace || !strides) return VQA_ERR_NULL_POINTER;
    if (!vi && N >= kBlock) return VQA_ERR_NULL_POINTER;  // no block-sampled row exists below 128 keys
    if (B <= 0 || H <= 0 || N <= 0 || C <= 0 || C > kMaxCodes || N / kBlock > 65535) return VQA_ERR_BAD_SHAPE;
    if (D < 2 || D > 128 || (D & 1)) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    if ((int64_t)B * H > 65535) return VQA_ERR_BAD_ARGUMENT;
    if (ws_bytes < workspace_bytes(B, H, N, C)) return VQA_ERR_WORKSPACE_TOO_SMALL;
    if ((state_cnt == nullptr) != (state_vsum == nullptr)) return VQA_ERR_NULL_POINTER;
    if ((uintptr_t)state_vsum & 7) return VQA_ERR_MISALIGNED;
    Params p;
    p.state_cnt = state_cnt;
    p.state_vsum = state_vsum;
    p.ids = ids;
    p.id_sb = strides[0], p.id_sh = strides[1], p.id_sn = strides[2];
    p.v = static_cast<const uint16_t*>(v);
    p.v_sb = strides[3], p.v_sh = strides[4], p.v_sn = strides[5];
    p.cnt = cnt;
    p.cn_sb = strides[6], p.cn_sh = strides[7], p.cn_st = strides[8];
    p.cnt_elem = static_cast<uint16_t*>(cnt_elem);
    p.ce_sb = strides[9], p.ce_sh = strides[10], p.ce_st = strides[11];
    p.vvq = static_cast<uint16_t*>(v_vq);
    p.vq_sb = strides[12], p.vq_sh = strides[13], p.vq_sn = strides[14];
    p.vi = vi;
    p.vi_sb = strides[15], p.vi_sh = strides[16], p.vi_st = strides[17];
    if (((uintptr_t)v & 3) || ((uintptr_t)v_vq & 3) || ((uintptr_t)workspace & 255) ||
        ((p.v_sb | p.v_sh | p.v_sn | p.vq_sb | p.vq_sh | p.vq_sn) & 1))
        return VQA_ERR_MISALIGNED;
    p.H = H, p.N = N, p.D = D, p.C = C;
    p.NB = (N + kBlock - 1) / kBlock;
    const size_t bh = (size_t)B * H;
    char* ws = static_cast<char*>(workspace);
    p.hist = reinterpret_cast<int32_t*>(ws);
    ws += align256(bh * p.NB * C * 4);
    p.start = reinterpret_cast<int32_t*>(ws);
    ws += align256(bh * C * 4);
    p.order = reinterpret_cast<int32_t*>(ws);
    int rc;
    hipLaunchKernelGGL(hist_kernel, dim3(p.NB, B * H), dim3(kBlock), C * sizeof(int), stream, p);
    if ((rc = launch_status()) != VQA_OK) return rc;
    hipLaunchKernelGGL(cumulate_kernel, dim3((C + 255) / 256, B * H), dim3(256), 0, stream, p);
    if ((rc = launch_status()) != VQA_OK) return rc;
    hipLaunchKernelGGL(start_kernel, dim3(B * H), dim3(256), 0, stream, p);
    if ((rc = launch_status()) != VQA_OK) return rc;
    if (N / kBlock > 0) {
        hipLaunchKernelGGL((emit_kernel<Tag>), dim3((C + 255) / 256, N / kBlock, B * H), dim3(256), 0, stream, p);
        if ((rc = launch_status()) != VQA_OK) return rc;
    }
    hipLaunchKernelGGL(scatter_kernel, dim3(p.NB, B * H), dim3(kBlock), 0, stream, p);
    if ((rc = launch_status()) != VQA_OK) return rc;
    hipLaunchKernelGGL((segment_sum_kernel<Tag>), dim3((C + 3) / 4, B * H), dim3(256), 0, stream, p);
    return launch_status();
}

}  // namespace prep
}  // namespace vqa

extern "C" {

size_t vqa_preprocess_workspace_bytes(int B, int H, int N, int C) { return vqa::prep::workspace_bytes(B, H, N, C); }

int vqa_preprocess_bf16(const int64_t* ids, const void* v, int64_t* cnt, void* cnt_elem, void* v_vq, int64_t* vi,
                        void* workspace, size_t workspace_bytes, int B, int H, int N, int D, int C,
                        const int64_t* strides, vqa_stream_t stream) {
    return vqa::prep::preprocess<vqa::bf16_tag>(ids, v, cnt, cnt_elem, v_vq, vi, workspace, workspace_bytes, B, H, N,
                                                D, C, strides, stream);
}

int vqa_preprocess_f16(const int64_t* ids, const void* v, int64_t* cnt, void* cnt_elem, void* v_vq, int64_t* vi,
                       void* workspace, size_t workspace_bytes, int B, int H, int N, int D, int C,
                       const int64_t* strides, vqa_stream_t stream) {
    return vqa::prep::preprocess<vqa::f16_tag>(ids, v, cnt, cnt_elem, v_vq, vi, workspace, workspace_bytes, B, H, N, D,
                                               C, strides, stream);
}

int vqa_preprocess_state_bf16(const int64_t* ids, const void* v, int64_t* cnt, void* cnt_elem, void* v_vq, int64_t* vi,
                              int32_t* state_cnt, float* state_vsum, void* workspace, size_t workspace_bytes, int B,
                              int H, int N, int D, int C, const int64_t* strides, vqa_stream_t stream) {
    if (!state_cnt || !state_vsum) return VQA_ERR_NULL_POINTER;
    return vqa::prep::preprocess<vqa::bf16_tag>(ids, v, cnt, cnt_elem, v_vq, vi, workspace, workspace_bytes, B, H, N,
                                                D, C, strides, stream, state_cnt, state_vsum);
}

int vqa_preprocess_state_f16(const int64_t* ids, const void* v, int64_t* cnt, void* cnt_elem, void* v_vq, int64_t* vi,
                             int32_t* state_cnt, float* state_vsum, void* workspace, size_t workspace_bytes, int B,
                             int H, int N, int D, int C, const int64_t* strides, vqa_stream_t stream) {
    if (!state_cnt || !state_vsum) return VQA_ERR_NULL_POINTER;
    return vqa::prep::preprocess<vqa::f16_tag>(ids, v, cnt, cnt_elem, v_vq, vi, workspace, workspace_bytes, B, H, N, D,
                                               C, strides, stream, state_cnt, state_vsum);
}

}  // extern "C"
