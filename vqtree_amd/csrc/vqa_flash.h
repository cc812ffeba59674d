// Building blocks of the MFMA flash-attention kernels (gfx950), shared by the window / ReRoPE / VQ-prefill kernel
// and the count-weighted codeword kernel.
//
// Work split: one workgroup = 4 waves = 128 query rows; each wave owns 32 query rows and sweeps 64-key tiles.
// Scores are computed TRANSPOSED, S^T[key, query] = K . Q^T with v_mfma_f32_32x32x16: the key tile comes from LDS
// as the A operand, the wave's 32 queries stay in registers as the B operand.  In the 32x32 accumulator layout a
// lane then holds ONE query column (lane % 32) and 16 of the 32 keys, so the row statistics of the online softmax
// are per-lane scalars (plus one exchange with lane ^ 32), and the probabilities are already laid out as the B
// operand of O^T[d, query] = V^T . P^T.  V^T fragments (8 keys for one d per lane) are read from the row-major V
// tile in LDS with ds_read_b64_tr_b16.
#pragma once

#include "vqa_common.h"

namespace vqa {
namespace flash {

constexpr int kBM = 128;      // query rows per workgroup
constexpr int kBN = 64;       // keys per tile
constexpr int kThreads = 256; // 4 waves
constexpr int kTile = 128;    // T: block granularity of the window / far-context boundary rules

typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));  // native vector: stays in registers

struct View {  // [B,H,N,D] tensor with unit innermost stride, element strides
    const uint16_t* p;
    int64_t sb, sh, sn;
};

template <int D>
struct Geom {
    static constexpr int kPitch = D * 2 + 32;              // LDS row pitch in bytes (row shift of 8 banks)
    static constexpr int kTileBytes = kBN * kPitch;
    static constexpr int kChunksPerRow = D / 8;            // 16-byte chunks
    static constexpr int kChunks = kBN * kChunksPerRow / kThreads;  // per thread
    static constexpr int kKSteps = D / 16;                 // 32x32x16 steps along head_dim
    static constexpr int kDBlocks = D / 32;                // 32-row blocks of O^T
};

// Q fragment of one wave: B operand of S^T = K.Q^T.  Lane (n = lane%32, half = lane/32) holds
// q[row0 + n][kk*16 + half*8 .. +8] for each k-step kk.
template <typename Tag, int D>
struct QFrag {
    typename Elem<Tag>::vec8 f[Geom<D>::kKSteps];
};

template <typename Tag, int D>
__device__ __forceinline__ void load_q(QFrag<Tag, D>& q, const uint16_t* base, int64_t sn, int row0, int n_rows,
                                       int lane) {
    typedef typename Elem<Tag>::vec8 vec8;
    const int n = lane & 31, half = lane >> 5;
    const int row = min(row0 + n, n_rows - 1);  // rows past the end are computed but never stored
    const uint16_t* r = base + (int64_t)row * sn + half * 8;
#pragma unroll
    for (int kk = 0; kk < Geom<D>::kKSteps; ++kk) q.f[kk] = *reinterpret_cast<const vec8*>(r + kk * 16);
}

// Tile staging: global -> registers (16-byte chunks, row clamped to the last valid row) -> LDS.
template <int D>
struct TileRegs {
    u32x4_t c[Geom<D>::kChunks];
};

template <int D>
__device__ __forceinline__ void tile_g2r(TileRegs<D>& r, const uint16_t* base, int64_t sn, int n0, int n_rows,
                                         int tid) {
#pragma unroll
    for (int i = 0; i < Geom<D>::kChunks; ++i) {
        const int ch = tid + i * kThreads;
        const int row = ch / Geom<D>::kChunksPerRow, col = ch % Geom<D>::kChunksPerRow;
        const int g = min(n0 + row, n_rows - 1);
        r.c[i] = *reinterpret_cast<const u32x4_t*>(base + (int64_t)g * sn + col * 8);
    }
}

// Same, with the global row taken from an index list (rows of a gathered tensor).
template <int D>
__device__ __forceinline__ void tile_g2r_gather(TileRegs<D>& r, const uint16_t* base, int64_t sn,
                                                const int64_t* row_index, int n0, int n_rows, int tid) {
#pragma unroll
    for (int i = 0; i < Geom<D>::kChunks; ++i) {
        const int ch = tid + i * kThreads;
        const int row = ch / Geom<D>::kChunksPerRow, col = ch % Geom<D>::kChunksPerRow;
        const int64_t g = row_index[min(n0 + row, n_rows - 1)];
        r.c[i] = *reinterpret_cast<const u32x4_t*>(base + g * sn + col * 8);
    }
}

template <int D>
__device__ __forceinline__ void tile_r2s(const TileRegs<D>& r, char* lds, int tid) {
#pragma unroll
    for (int i = 0; i < Geom<D>::kChunks; ++i) {
        const int ch = tid + i * kThreads;
        const int row = ch / Geom<D>::kChunksPerRow, col = ch % Geom<D>::kChunksPerRow;
        *reinterpret_cast<u32x4_t*>(lds + row * Geom<D>::kPitch + col * 16) = r.c[i];
    }
}

// S^T (64 keys x 32 queries) = Ktile . Q^T.  s[kb] is the accumulator of key block kb (32 keys); in it lane
// (n, half) holds, at register r, key  kb*32 + 8*(r/4) + 4*half + r%4  of query n.
template <typename Tag, int D>
__device__ __forceinline__ void qk_mma(f32x16_t (&s)[2], const QFrag<Tag, D>& q, const char* lds_k, int lane) {
    typedef typename Elem<Tag>::vec8 vec8;
    const int r = lane & 31, half = lane >> 5;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
        f32x16_t acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
        const char* row = lds_k + (kb * 32 + r) * Geom<D>::kPitch + half * 16;
#pragma unroll
        for (int kk = 0; kk < Geom<D>::kKSteps; ++kk) {
            const vec8 a = *reinterpret_cast<const vec8*>(row + kk * 32);
            acc = Elem<Tag>::mfma32(a, q.f[kk], acc);
        }
        s[kb] = acc;
    }
}

// key offset inside a 32-key block held at accumulator register r by a lane of the given half
__device__ __forceinline__ int key_of_reg(int r, int half) { return 8 * (r >> 2) + 4 * half + (r & 3); }

// O^T (D x 32 queries) += Vtile^T . P^T.  p[kb][j2] packs the probabilities of keys kb*32 + j2*16 + {4*half..+3,
// 8+4*half..+3} (registers j2*8 .. j2*8+7 of s[kb]) as the B operand; the matching V^T A operand is gathered by two
// transposing LDS reads: inside every 16-lane group, source lane s points at V[key0 + s/4][d0 + 4*(s%4)] and lane L
// receives V[key0 .. key0+3][d0 + L].
template <typename Tag, int D>
__device__ __forceinline__ void pv_mma(f32x16_t (&o)[Geom<D>::kDBlocks], const typename Elem<Tag>::vec8 (&p)[2][2],
                                       const char* lds_v, int lane) {
    typedef typename Elem<Tag>::vec8 vec8;
    typedef __attribute__((address_space(3))) s16x4_t* lds_ptr_t;
    const int half = lane >> 5;
    const int dsub = (lane >> 4) & 1;  // which 16 of the 32 d rows this 16-lane group produces
    const int s = lane & 15;
    // address of this lane's 4-element source chunk for key0 = 0, d block 0
    const char* src = lds_v + (4 * half + (s >> 2)) * Geom<D>::kPitch + (dsub * 16 + 4 * (s & 3)) * 2;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int j2 = 0; j2 < 2; ++j2) {
            const char* kbase = src + (kb * 32 + j2 * 16) * Geom<D>::kPitch;
#pragma unroll
            for (int db = 0; db < Geom<D>::kDBlocks; ++db) {
                const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(kbase + db * 64));
                const s16x4_t hi =
                    __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(kbase + 8 * Geom<D>::kPitch + db * 64));
                const short __attribute__((ext_vector_type(8))) av = {lo[0], lo[1], lo[2], lo[3],
                                                                      hi[0], hi[1], hi[2], hi[3]};
                o[db] = Elem<Tag>::mfma32(__builtin_bit_cast(vec8, av), p[kb][j2], o[db]);
            }
        }
    }
}

// Online-softmax state of one wave: every lane carries the running max of ITS query (identical in lane ^ 32) and
// the partial row sum of the keys it has seen; o[] is O^T in accumulator layout (lane = query column).
template <int D>
struct SoftmaxState {
    float m, l;
    f32x16_t o[Geom<D>::kDBlocks];
    __device__ __forceinline__ void init() {
        m = -INFINITY;
        l = 0.f;
#pragma unroll
        for (int db = 0; db < Geom<D>::kDBlocks; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
    }
};

// s holds scaled (base-2) scores with masked entries at -inf; w (nullable per-register weights) multiplies the
// probabilities in the row sum only (count-weighted softmax).  Produces the packed P^T fragments.
template <typename Tag, int D, bool kWeighted>
__device__ __forceinline__ void softmax_update(SoftmaxState<D>& st, f32x16_t (&s)[2],
                                               typename Elem<Tag>::vec8 (&p)[2][2], const float (*w)[16]) {
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kb][i]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(st.m, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;  // a row with nothing visible yet keeps p = 0
    const float alpha = fast_exp2(st.m - m_safe);
    float sum = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int j2 = 0; j2 < 2; ++j2) {
            short __attribute__((ext_vector_type(8))) pk;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int r = j2 * 8 + e;
                const float pe = fast_exp2(s[kb][r] - m_safe);
                if constexpr (kWeighted)
                    sum += pe * w[kb][r];
                else
                    sum += pe;
                pk[e] = (short)Elem<Tag>::to_bits(pe);
            }
            p[kb][j2] = __builtin_bit_cast(typename Elem<Tag>::vec8, pk);
        }
    }
    st.l = st.l * alpha + sum;
    st.m = m_new;
#pragma unroll
    for (int db = 0; db < Geom<D>::kDBlocks; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) st.o[db][i] *= alpha;
}

// Normalise and store the wave's 32 output rows; lse2 = m + log2(l).  A row that saw no key stores 0 / -inf.
template <typename Tag, int D>
__device__ __forceinline__ void store_output(const SoftmaxState<D>& st, uint16_t* out_base, int64_t sn, float* lse,
                                             int row0, int n_rows, int lane) {
    const int n = lane & 31, half = lane >> 5;
    const float l_tot = st.l + __shfl_xor(st.l, 32, 64);
    const int row = row0 + n;
    if (row >= n_rows) return;
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    uint16_t* dst = out_base + (int64_t)row * sn;
#pragma unroll
    for (int db = 0; db < Geom<D>::kDBlocks; ++db) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            // registers 4g..4g+3 are d = db*32 + 8g + 4*half + 0..3
            uint2 pk;
            pk.x = (uint32_t)Elem<Tag>::to_bits(st.o[db][4 * g] * inv) |
                   ((uint32_t)Elem<Tag>::to_bits(st.o[db][4 * g + 1] * inv) << 16);
            pk.y = (uint32_t)Elem<Tag>::to_bits(st.o[db][4 * g + 2] * inv) |
                   ((uint32_t)Elem<Tag>::to_bits(st.o[db][4 * g + 3] * inv) << 16);
            *reinterpret_cast<uint2*>(dst + db * 32 + 8 * g + 4 * half) = pk;
        }
    }
    if (lse != nullptr && half == 0) lse[row] = l_tot > 0.f ? st.m + fast_log2(l_tot) : -INFINITY;
}

}  // namespace flash
}  // namespace vqa
