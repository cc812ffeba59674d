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
//
// K / V tiles travel HBM/L2 -> LDS without touching registers (global_load_lds_dwordx4: lane l of a wave writes
// 16 bytes at LDS base + 16*l).  The tiles are unpadded; bank conflicts are avoided by an XOR swizzle of the 16-byte
// chunk index with a function of the row, applied on the global-address side of the copy and undone when the MFMA
// operands are read.
#pragma once

#include "vqa_common.h"

namespace vqa {
namespace flash {

constexpr int kBM = 128;      // query rows per workgroup
constexpr int kBN = 64;       // keys per tile
constexpr int kThreads = 256; // 4 waves
constexpr int kWaves = 4;
constexpr int kTile = 128;    // T: block granularity of the window / far-context boundary rules

typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef const __attribute__((address_space(1))) void* global_void_ptr;

struct View {  // [B,H,N,D] tensor with unit innermost stride, element strides
    const uint16_t* p;
    int64_t sb, sh, sn;
};

template <int D>
struct Geom {
    static constexpr int kRowBytes = D * 2;
    static constexpr int kTileBytes = kBN * kRowBytes;
    static constexpr int kChunksPerRow = D / 8;                 // 16-byte chunks per row
    static constexpr int kRowsPerInstr = 64 / kChunksPerRow;    // rows one wave-wide 16-byte load covers
    static constexpr int kRowsPerBankCycle = 256 / kRowBytes;   // rows that share one sweep over the 64 banks
    static constexpr int kKSteps = D / 16;                      // 32x32x16 steps along head_dim
    static constexpr int kDBlocks = D / 32;                     // 32-row blocks of O^T

    // chunk-index XOR of a K tile row: 16 consecutive rows read the same logical chunk (ds_read_b128)
    static __device__ __forceinline__ int swz_k(int row) {
        return (int)(((unsigned)row / (unsigned)kRowsPerBankCycle) % (unsigned)kChunksPerRow);
    }
    // chunk-index XOR of a V tile row.  One ds_read_b64_tr_b16 reads 8 consecutive rows x 4 consecutive chunks (64
    // bytes per row), its two 32-lane halves 4 rows each; the rows of a half must land in different 64-byte bank
    // groups or they are served one after the other (measured: XOR 2*(row % 8), which maps rows 2k and 2k+1 to the
    // same group, costs 4 LDS cycles and 2 conflict cycles per instruction; this one 2 and 0).  Multiples of 4 only:
    // the 4 chunks of a read stay together.
    static __device__ __forceinline__ int swz_v(int row) {
        constexpr unsigned kGroups = kChunksPerRow / 4 > 0 ? kChunksPerRow / 4 : 1;  // 64-byte groups per row
        return (int)(4u * (((unsigned)row / (unsigned)kRowsPerBankCycle) % kGroups));
    }
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

// ---------------------------------------------------------------------------------------------------------------
// Tile copy global -> LDS.  Wave w brings rows [16w, 16w+16) of the 64-row tile; one instruction covers
// kRowsPerInstr rows: lane l lands at LDS chunk (row, l % kChunksPerRow) and therefore fetches the global chunk
// (l % kChunksPerRow) ^ swizzle(row).
// ---------------------------------------------------------------------------------------------------------------
// 16 bytes per lane from global memory straight into LDS: lane l of the wave lands at lds_addr + 16*l.
// Issued as inline assembly on purpose: the compiler makes every later LDS read wait for all direct-to-LDS loads
// it knows of (it cannot tell the buffer being filled from the one being read), which would serialise the
// prefetch with the compute.  The kernels wait for these loads themselves (wait_tile_loads + barrier).
__device__ __forceinline__ void dma16(const void* gptr, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_addr)
                 : "memory");  // m0 is written too; no other instruction of these kernels uses it
}

// same with the global address split into a wave-uniform base (scalar registers) and a 32-bit per-lane byte offset
__device__ __forceinline__ void dma16_uniform(const void* uniform_base, uint32_t lane_offset, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(lane_offset), "s"(uniform_base), "s"(lds_addr)
                 : "memory");
}

__device__ __forceinline__ uint32_t lds_addr_of(const char* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)p;
}

template <int D, bool kIsV, int NW = kWaves>
struct TileCopy {
    static constexpr int kRowsPerWave = kBN / NW;                         // rows of the tile one wave brings
    static constexpr int kInstr = kRowsPerWave / Geom<D>::kRowsPerInstr;  // direct-to-LDS loads per wave and tile
    static_assert(kInstr >= 1, "too many waves for this tile");
    int wave;
    int lane_row;                  // row (within the kRowsPerInstr rows of one instruction) of this lane
    int chunk;                     // LDS chunk column of this lane
    uint32_t chunk_bytes[kInstr];  // byte offset inside the global row that lands in that column

    __device__ __forceinline__ void init(int wave_, int lane) {
        wave = wave_;
        lane_row = (int)((unsigned)lane / (unsigned)Geom<D>::kChunksPerRow);
        chunk = (int)((unsigned)lane % (unsigned)Geom<D>::kChunksPerRow);
#pragma unroll
        for (int i = 0; i < kInstr; ++i) chunk_bytes[i] = (uint32_t)src_chunk(row(i)) * 16u;
    }
    __device__ __forceinline__ int row(int i) const {
        return wave * kRowsPerWave + i * Geom<D>::kRowsPerInstr + lane_row;
    }
    __device__ __forceinline__ int src_chunk(int r) const {
        return chunk ^ (kIsV ? Geom<D>::swz_v(r) : Geom<D>::swz_k(r));
    }
    __device__ __forceinline__ uint32_t dst(const char* lds_tile, int i) const {
        return lds_addr_of(lds_tile) + (wave * kRowsPerWave + i * Geom<D>::kRowsPerInstr) * Geom<D>::kRowBytes;
    }
    // rows [n0, n0+64), all inside the matrix: uniform (scalar) row-group base + one 32-bit per-lane offset
    __device__ __forceinline__ void load_full(const char* lds_tile, const uint16_t* base, int64_t sn, int n0) const {
        const uint32_t lane_off = (uint32_t)lane_row * (uint32_t)(sn * 2);
        const char* grp = reinterpret_cast<const char*>(base + (int64_t)(n0 + wave * kRowsPerWave) * sn);
        const int64_t step = (int64_t)Geom<D>::kRowsPerInstr * sn * 2;  // bytes between the row groups of two loads
#pragma unroll
        for (int i = 0; i < kInstr; ++i) dma16_uniform(grp + i * step, lane_off + chunk_bytes[i], dst(lds_tile, i));
    }
    // rows [n0, n0+64) of a [n_rows, D] matrix with row stride sn (elements); rows past the end repeat the last row
    __device__ __forceinline__ void load(const char* lds_tile, const uint16_t* base, int64_t sn, int n0,
                                         int n_rows) const {
        if (n0 + kBN <= n_rows) {
            load_full(lds_tile, base, sn, n0);
        } else {
#pragma unroll
            for (int i = 0; i < kInstr; ++i) {
                const int g = min(n0 + row(i), n_rows - 1);
                const char* src = reinterpret_cast<const char*>(base + (int64_t)g * sn) + chunk_bytes[i];
                dma16(src, dst(lds_tile, i));
            }
        }
    }
    // same with the global rows taken from an index list, in two steps so that the indices can be fetched a tile
    // ahead of the copy that uses them: rows[i] = row_index[n0 + row(i)] (clamped), then one copy per index
    // (index values are clamped to [0, max_index], so a corrupt list cannot send the copy outside the matrix)
    __device__ __forceinline__ void fetch_rows(int64_t (&rows)[kInstr], const int64_t* row_index, int n0, int n_rows,
                                               int64_t max_index) const {
#pragma unroll
        for (int i = 0; i < kInstr; ++i) {
            const int64_t r = row_index[min(n0 + row(i), n_rows - 1)];
            rows[i] = r < 0 ? 0 : (r > max_index ? max_index : r);
        }
    }
    __device__ __forceinline__ void load_rows(const char* lds_tile, const uint16_t* base, int64_t sn,
                                              const int64_t (&rows)[kInstr]) const {
#pragma unroll
        for (int i = 0; i < kInstr; ++i) {
            const char* src = reinterpret_cast<const char*>(base + rows[i] * sn) + chunk_bytes[i];
            dma16(src, dst(lds_tile, i));
        }
    }
};

// all of this wave's direct-to-LDS loads have landed
// (s_waitcnt vmcnt(0) with expcnt / lgkmcnt left at their maxima)
__device__ __forceinline__ void wait_tile_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// S^T (64 keys x 32 queries) = Ktile . Q^T.  s[kb] is the accumulator of key block kb (32 keys); in it lane
// (n, half) holds, at register r, key  kb*32 + 8*(r/4) + 4*half + r%4  of query n.
// The A fragments are software-pipelined kAhead steps in front of their MFMA; the scheduling barriers pin that order
// so only kAhead + 1 fragments are ever live (left alone, the scheduler hoists every LDS read to the top).
template <typename Tag, int D>
__device__ __forceinline__ void qk_mma(f32x16_t (&s)[2], const QFrag<Tag, D>& q, const char* lds_k, int lane) {
    typedef typename Elem<Tag>::vec8 vec8;
    typedef Geom<D> G;
    constexpr int KS = G::kKSteps;
    constexpr int kSteps = 2 * KS;
    constexpr int kAhead = 3;
    const int r = lane & 31, half = lane >> 5;
    // logical chunk of step kk is 2*kk + half = (2*kk) ^ half; it is stored at chunk ^ swz_k(row), and
    // swz_k(r) == swz_k(r + 32), so one per-lane base serves both key blocks
    // (the tile is 1 KiB-aligned in LDS, so the XOR may be applied to the full 32-bit LDS address)
    typedef const __attribute__((address_space(3))) vec8* lds_vec8_ptr;
    const uint32_t base = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)lds_k +
                          ((uint32_t)(r * G::kRowBytes) | (uint32_t)((half ^ G::swz_k(r)) << 4));
    // step n works on key block n % 2 and k-step n / 2: the two accumulation chains alternate, so an MFMA never
    // has to wait for the one issued just before it
    auto frag = [&](int n) {
        const uint32_t addr = (base ^ (uint32_t)((2 * (n / 2)) << 4)) + (n % 2) * 32 * G::kRowBytes;
        return *(lds_vec8_ptr)(uintptr_t)addr;
    };
    vec8 a[kAhead + 1];
#pragma unroll
    for (int i = 0; i < kAhead; ++i) a[i] = frag(i);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) s[kb][e] = 0.f;
#pragma unroll
    for (int i = 0; i < kSteps; ++i) {
        if (i + kAhead < kSteps) a[(i + kAhead) % (kAhead + 1)] = frag(i + kAhead);
        s[i % 2] = Elem<Tag>::mfma32(a[i % (kAhead + 1)], q.f[i / 2], s[i % 2]);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// One 32-key block of S^T (key block kb of the tile), for the rarely taken multi-pair tiles where register
// pressure matters more than pipelining.
template <typename Tag, int D>
__device__ __forceinline__ f32x16_t qk_block(const QFrag<Tag, D>& q, const char* lds_k, int kb, int lane) {
    typedef typename Elem<Tag>::vec8 vec8;
    typedef Geom<D> G;
    typedef const __attribute__((address_space(3))) vec8* lds_vec8_ptr;
    const int r = lane & 31, half = lane >> 5;
    const uint32_t base = lds_addr_of(lds_k) + kb * 32 * G::kRowBytes +
                          ((uint32_t)(r * G::kRowBytes) | (uint32_t)((half ^ G::swz_k(r)) << 4));
    f32x16_t acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
#pragma unroll
    for (int kk = 0; kk < G::kKSteps; ++kk) {
        const vec8 a = *(lds_vec8_ptr)(uintptr_t)(base ^ (uint32_t)((2 * kk) << 4));
        acc = Elem<Tag>::mfma32(a, q.f[kk], acc);
        __builtin_amdgcn_sched_barrier(0);
    }
    return acc;
}

// key offset inside a 32-key block held at accumulator register r by a lane of the given half
__device__ __forceinline__ int key_of_reg(int r, int half) { return 8 * (r >> 2) + 4 * half + (r & 3); }

// O^T (D x 32 queries) += Vtile^T . P^T.  p[kb][j2] packs the probabilities of keys kb*32 + j2*16 + {4*half..+3,
// 8+4*half..+3} (registers j2*8 .. j2*8+7 of s[kb]) as the B operand; the matching V^T A operand is gathered by two
// transposing LDS reads: inside every 16-lane group, source lane s points at V[key0 + s/4][d0 + 4*(s%4)] and lane L
// receives V[key0 .. key0+3][d0 + L].  Pipelined like qk_mma.
template <typename Tag, int D>
__device__ __forceinline__ void pv_mma(f32x16_t (&o)[Geom<D>::kDBlocks], const typename Elem<Tag>::vec8 (&p)[2][2],
                                       const char* lds_v, int lane) {
    typedef typename Elem<Tag>::vec8 vec8;
    typedef __attribute__((address_space(3))) s16x4_t* lds_ptr_t;
    typedef Geom<D> G;
    constexpr int DB = G::kDBlocks;
    constexpr int kSteps = 4 * DB;  // (kb, j2, db)
    constexpr int kAhead = 3;
    const int half = lane >> 5;
    const int dsub = (lane >> 4) & 1;  // which 16 of the 32 d rows this 16-lane group produces
    const int sl = lane & 15;
    // source of this lane for key0 = 0, d block 0: row 4*half + sl/4, elements d = dsub*16 + 4*(sl%4) .. +3, i.e.
    // logical chunk 2*dsub + (sl%4)/2, 8-byte piece (sl%4)%2.  Rows advance by multiples of 8, which leaves swz_v
    // unchanged; d block db adds 4*db to the chunk, an XOR because the lane part only uses bits 0-1.
    const int row = 4 * half + (sl >> 2);
    const uint32_t base = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)lds_v +
                          ((uint32_t)(row * G::kRowBytes) |
                           (uint32_t)(((2 * dsub + ((sl & 3) >> 1)) ^ G::swz_v(row)) << 4) | (uint32_t)((sl & 1) << 3));
    s16x4_t lo[kAhead + 1], hi[kAhead + 1];
    auto fetch = [&](int n) {
        const uint32_t addr = (base ^ (uint32_t)((4 * (n % DB)) << 4)) + (n / DB) * 16 * G::kRowBytes;
        lo[n % (kAhead + 1)] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(uintptr_t)addr);
        hi[n % (kAhead + 1)] =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(uintptr_t)(addr + 8 * G::kRowBytes));
    };
#pragma unroll
    for (int i = 0; i < kAhead; ++i) fetch(i);
#pragma unroll
    for (int i = 0; i < kSteps; ++i) {
        if (i + kAhead < kSteps) fetch(i + kAhead);
        const s16x4_t l4 = lo[i % (kAhead + 1)], h4 = hi[i % (kAhead + 1)];
        const short __attribute__((ext_vector_type(8))) av = {l4[0], l4[1], l4[2], l4[3], h4[0], h4[1], h4[2], h4[3]};
        const int kbj = i / DB;  // kb*2 + j2
        o[i % DB] = Elem<Tag>::mfma32(__builtin_bit_cast(vec8, av), p[kbj >> 1][kbj & 1], o[i % DB]);
        __builtin_amdgcn_sched_barrier(0);
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

// s holds RAW scores (masked entries at -inf); scale = sm_scale*log2(e) > 0 is folded into the exponent:
// p = 2^(s*scale - m).  w (nullable per-register weights) multiplies the probabilities in the row sum only
// (count-weighted softmax).  O is rescaled only when some row of the wave raised its maximum.  Produces the packed
// P^T fragments.
template <typename Tag, int D, bool kWeighted>
__device__ __forceinline__ void softmax_update(SoftmaxState<D>& st, f32x16_t (&s)[2], float scale,
                                               typename Elem<Tag>::vec8 (&p)[2][2], const float (*w)[16]) {
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kb][i]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(st.m, mx * scale);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;  // a row with nothing visible yet keeps p = 0
    if (__builtin_amdgcn_ballot_w64(m_new != st.m) != 0) {
        const float alpha = fast_exp2(st.m - m_safe);
        st.l *= alpha;
#pragma unroll
        for (int db = 0; db < Geom<D>::kDBlocks; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) st.o[db][i] *= alpha;
        st.m = m_new;
    }
    float sum = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int j2 = 0; j2 < 2; ++j2) {
            u32x4_t pk;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int r = j2 * 8 + 2 * e;
                const float p0 = fast_exp2(__builtin_fmaf(s[kb][r], scale, -m_safe));
                const float p1 = fast_exp2(__builtin_fmaf(s[kb][r + 1], scale, -m_safe));
                pk[e] = Elem<Tag>::pack2(p0, p1);
                if constexpr (kWeighted)
                    sum += p0 * w[kb][r] + p1 * w[kb][r + 1];
                else
                    sum += p0 + p1;  // (fp32 additions, not v_dot2 on the packed pair: the dot instructions run on
                                     // the matrix pipe and cost its time while another wave's MFMAs wait)
            }
            p[kb][j2] = __builtin_bit_cast(typename Elem<Tag>::vec8, pk);
        }
    }
    st.l += sum;
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
