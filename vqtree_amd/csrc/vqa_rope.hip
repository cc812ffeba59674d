// Rotary position embedding of a [B,H,N,D] tensor in the model's 16-bit type:
//     out = x * cos[pos] + rotate_half(x) * sin[pos],   rotate_half(x) = cat(-x[D/2:], x[:D/2])
// with every product and the sum rounded to the element type, which is what the same expression gives when it is
// evaluated operator by operator on 16-bit tensors.  pos comes from position_ids[b, n] or is one fixed position for
// every row (the clamped ReRoPE query).
#include "vqa_common.h"

// every product and sum below must round on its own: no fused multiply-add
#pragma clang fp contract(off)

namespace vqa {
namespace rope {

struct Params {
    const uint16_t* x;
    int64_t x_sb, x_sh, x_sn;
    const int64_t* pos;  // [B,N] or null
    int64_t p_sb, p_sn;
    const uint16_t* cos;
    const uint16_t* sin;
    int64_t t_sp;  // row stride of the tables
    uint16_t* out;
    int64_t o_sb, o_sh, o_sn;
    uint16_t* out_fixed;  // nullable: the same rows rotated to fixed_pos as well (same strides as out)
    int H, N, D, n_pos, fixed_pos;
    int64_t rows;  // B*H*N
};

template <typename Tag>
__device__ __forceinline__ float rnd(float v) { return Elem<Tag>::round_keep_f32(v); }

template <typename Tag>
__global__ __launch_bounds__(256) void rope_kernel(Params p) {
    const int tpr = p.D / 16;  // threads per row: each handles 8 elements of the low half and their partners
    const int64_t row = (int64_t)blockIdx.x * (256 / tpr) + threadIdx.x / tpr;
    if ((int)threadIdx.x >= (256 / tpr) * tpr || row >= p.rows) return;
    const int c = (threadIdx.x % tpr) * 8;
    const int n = (int)(row % p.N);
    const int h = (int)((row / p.N) % p.H);
    const int b = (int)(row / ((int64_t)p.N * p.H));
    const int half_d = p.D / 2;
    const uint16_t* xr = p.x + b * p.x_sb + h * p.x_sh + (int64_t)n * p.x_sn;
    const uint4 xl = load_stream16(xr + c), xh = load_stream16(xr + half_d + c);
    const uint32_t xlw[4] = {xl.x, xl.y, xl.z, xl.w}, xhw[4] = {xh.x, xh.y, xh.z, xh.w};
    const int64_t row_off = b * p.o_sb + h * p.o_sh + (int64_t)n * p.o_sn;

    auto rotate_to = [&](int64_t pos, uint16_t* orow) {
        pos = min(max(pos, (int64_t)0), (int64_t)p.n_pos - 1);  // a position outside the tables is clamped
        const uint16_t* cr = p.cos + pos * p.t_sp;
        const uint16_t* sr = p.sin + pos * p.t_sp;
        const uint4 cl = *reinterpret_cast<const uint4*>(cr + c), ch = *reinterpret_cast<const uint4*>(cr + half_d + c);
        const uint4 sl = *reinterpret_cast<const uint4*>(sr + c), sh = *reinterpret_cast<const uint4*>(sr + half_d + c);
        const uint32_t clw[4] = {cl.x, cl.y, cl.z, cl.w}, chw[4] = {ch.x, ch.y, ch.z, ch.w};
        const uint32_t slw[4] = {sl.x, sl.y, sl.z, sl.w}, shw[4] = {sh.x, sh.y, sh.z, sh.w};
        uint32_t olw[4], ohw[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            uint32_t lo_pair = 0, hi_pair = 0;
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const int sh16 = 16 * s;
                const float a = Elem<Tag>::from_bits((uint16_t)(xlw[e] >> sh16));   // x[d], d < D/2
                const float bq = Elem<Tag>::from_bits((uint16_t)(xhw[e] >> sh16));  // x[d + D/2]
                const float c0 = Elem<Tag>::from_bits((uint16_t)(clw[e] >> sh16));
                const float c1 = Elem<Tag>::from_bits((uint16_t)(chw[e] >> sh16));
                const float s0 = Elem<Tag>::from_bits((uint16_t)(slw[e] >> sh16));
                const float s1 = Elem<Tag>::from_bits((uint16_t)(shw[e] >> sh16));
                const float lo = rnd<Tag>(rnd<Tag>(a * c0) + rnd<Tag>(-bq * s0));
                const float hi = rnd<Tag>(rnd<Tag>(bq * c1) + rnd<Tag>(a * s1));
                lo_pair |= (uint32_t)Elem<Tag>::to_bits(lo) << sh16;
                hi_pair |= (uint32_t)Elem<Tag>::to_bits(hi) << sh16;
            }
            olw[e] = lo_pair;
            ohw[e] = hi_pair;
        }
        store_stream16(orow + c, make_uint4(olw[0], olw[1], olw[2], olw[3]));
        store_stream16(orow + half_d + c, make_uint4(ohw[0], ohw[1], ohw[2], ohw[3]));
    };
    rotate_to(p.pos ? p.pos[b * p.p_sb + n * p.p_sn] : (int64_t)p.fixed_pos, p.out + row_off);
    if (p.out_fixed) rotate_to(p.fixed_pos, p.out_fixed + row_off);
}

// strides: x(b,h,n) position_ids(b,n) out(b,h,n); the tables are [n_pos, D] with row stride table_stride
template <typename Tag>
int rope(const void* x, const int64_t* position_ids, const void* cos, const void* sin, void* out, void* out_fixed, int B,
         int H, int N, int D, int n_pos, int64_t table_stride, const int64_t* strides, int fixed_pos,
         hipStream_t stream) {
    if (!x || !cos || !sin || !out || !strides) return VQA_ERR_NULL_POINTER;
    if (out_fixed && !position_ids) return VQA_ERR_BAD_ARGUMENT;  // the second output is for the position_ids form
    if (B <= 0 || H <= 0 || N <= 0 || n_pos <= 0) return VQA_ERR_BAD_SHAPE;
    if (D < 16 || D > 512 || (D % 16) != 0) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    if ((!position_ids || out_fixed) && (fixed_pos < 0 || fixed_pos >= n_pos)) return VQA_ERR_BAD_ARGUMENT;
    Params p;
    p.x = static_cast<const uint16_t*>(x);
    p.x_sb = strides[0], p.x_sh = strides[1], p.x_sn = strides[2];
    p.pos = position_ids;
    p.p_sb = strides[3], p.p_sn = strides[4];
    p.cos = static_cast<const uint16_t*>(cos);
    p.sin = static_cast<const uint16_t*>(sin);
    p.t_sp = table_stride;
    p.out = static_cast<uint16_t*>(out);
    p.out_fixed = static_cast<uint16_t*>(out_fixed);
    p.o_sb = strides[5], p.o_sh = strides[6], p.o_sn = strides[7];
    p.H = H, p.N = N, p.D = D, p.n_pos = n_pos, p.fixed_pos = fixed_pos;
    p.rows = (int64_t)B * H * N;
    if (!aligned16(x) || !aligned16(cos) || !aligned16(sin) || !aligned16(out) || !aligned16(out_fixed) ||
        ((p.x_sb | p.x_sh | p.x_sn | p.o_sb | p.o_sh | p.o_sn | p.t_sp) & 7))
        return VQA_ERR_MISALIGNED;
    const int rows_per_block = 256 / (D / 16);
    const int64_t blocks = (p.rows + rows_per_block - 1) / rows_per_block;
    if (blocks > 0x7fffffff) return VQA_ERR_BAD_SHAPE;
    hipLaunchKernelGGL((rope_kernel<Tag>), dim3((unsigned)blocks), dim3(256), 0, stream, p);
    return launch_status();
}

}  // namespace rope
}  // namespace vqa

extern "C" {

int vqa_rope_bf16(const void* x, const int64_t* position_ids, const void* cos, const void* sin, void* out,
                  void* out_fixed, int B, int H, int N, int D, int n_pos, int64_t table_stride, const int64_t* strides,
                  int fixed_pos, vqa_stream_t stream) {
    return vqa::rope::rope<vqa::bf16_tag>(x, position_ids, cos, sin, out, out_fixed, B, H, N, D, n_pos, table_stride,
                                          strides, fixed_pos, stream);
}

int vqa_rope_f16(const void* x, const int64_t* position_ids, const void* cos, const void* sin, void* out,
                 void* out_fixed, int B, int H, int N, int D, int n_pos, int64_t table_stride, const int64_t* strides,
                 int fixed_pos, vqa_stream_t stream) {
    return vqa::rope::rope<vqa::f16_tag>(x, position_ids, cos, sin, out, out_fixed, B, H, N, D, n_pos, table_stride,
                                         strides, fixed_pos, stream);
}

}  // extern "C"
