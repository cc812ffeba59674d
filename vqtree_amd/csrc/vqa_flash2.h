// Software-pipelined MFMA flash-attention core of the window / ReRoPE / VQ-prefill kernel (gfx950).
//
// Work split: one workgroup = 4 waves = 256 query rows, ONE wave per SIMD with the whole 512-register budget.  A wave
// owns 64 query rows as two 32-row blocks, so every K / V^T fragment it reads from LDS feeds two MFMAs (half the LDS
// operand traffic per FLOP of a 32-row wave), and the K / V tiles a workgroup copies serve 256 rows.
//
// With a single wave per SIMD nothing else hides the softmax behind the matrix pipe, so the wave does it itself: the
// scores of key tile u+1 are accumulated (S^T = K.Q^T, v_mfma_f32_32x32x16) while the exponentials of tile u are
// evaluated, and the row maxima of tile u+1 are taken while P(u).V(u) runs.  The code is written as MFMA "slots":
// slot i issues one MFMA followed by its share of everything else (VALU work, LDS fragment reads a few slots ahead,
// tile copies); scheduling barriers between slots keep that interleaving.
//
// What bounds a lone wave is instruction ISSUE: it issues one instruction every 5 - 6 clocks whatever its kind (an
// exponential every 9), an MFMA occupies the matrix pipe for 32, so about four other instructions fit in the shadow
// of an MFMA and every further one idles the pipe.  The loop is therefore written for instruction COUNT:
//   * the query is pre-multiplied by scale * log2(e) and the first score MFMA of a tile adds -m (a register tuple per
//     query block as its C operand), so a score leaves the pipe ready for exp2: no per-score multiply-add;
//   * row sums are fp32 additions, not v_dot2 (the dot instructions execute on the matrix pipe);
//   * fragments are read from LDS in pairs with one s_waitcnt per pair, tile copies take two instructions per load
//     and ride on the MFMA slots, per-lane addresses are computed once, the usual case of the maximum update is two
//     compares and a branch.
//
// Layouts (as in vqa_flash.h): scores are transposed, a lane (n = lane % 32, half = lane / 32) holds ONE query column
// per 32-row block, so row statistics are per-lane scalars (one v_permlane32_swap joins the halves) and the
// probabilities are already the B operand of O^T = V^T.P^T.
//
// Row maxima are lazy: the reference maximum of a row only moves when a tile exceeds it by more than 2^kLazy, so the
// O rescale (which has to wait for the matrix pipe) is rare; probabilities then reach at most 2^kLazy, exactly
// representable headroom in bf16 / f16 and harmless in the fp32 sums.
#pragma once

#include <utility>

#include "vqa_flash.h"

namespace vqa {
namespace flash2 {

using flash::Geom;
using flash::QFrag;
using flash::u32x4_t;
using flash::s16x4_t;

constexpr int kBM = 256;      // query rows per workgroup
constexpr int kBN = 64;       // keys per tile
constexpr int kThreads = 256;
constexpr int kWaveRows = 64; // query rows per wave (two 32-row blocks)
constexpr float kLazy = 8.f;  // log2 of the headroom a row maximum may fall behind

template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// The lane id as a value the optimiser cannot see through.  Per-lane LDS / global address variants (swizzle XORs,
// row offsets) derived from it are recomputed where they are used -- a handful of VALU operations -- and not
// hoisted out of the tile loop, where they would pin dozens of registers across every phase and end up spilled.
__device__ __forceinline__ int opaque_lane(int lane) {
    asm volatile("" : "+v"(lane));
    return lane;
}

// max over the two half-waves: lane l and lane l ^ 32 end up with the same value
__device__ __forceinline__ float join_halves_max(float x) {
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
__device__ __forceinline__ float join_halves_sum(float x) {
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

// Keeps a value where the program computes it: the optimiser may neither sink its computation below this point nor
// hoist its uses above (volatile statements keep their order, and the MFMA statements below are volatile too).
// Without it the exponentials written between the score MFMAs are sunk next to their first use, behind the P.V MFMAs.
template <typename T>
__device__ __forceinline__ void pin(T& x) {
    asm volatile("" : "+v"(x));
}

// MFMA forms with the register file chosen by hand.  The compiler's allocator does not find the split this kernel
// needs by itself (O^T, the query fragments and the K / V^T fragments in AccVGPRs, everything the VALU touches in
// VGPRs) and spills; inline assembly pins it.  The compiler inserts no hazard wait states around inline assembly: an
// MFMA result is read by another MFMA only several MFMAs later (independent accumulation chains), `mfma_settle()`
// stands wherever the VALU may read a result that the last few instructions produced, and no MFMA operand is
// written by a VALU instruction in the slot before it (the query fragments are DEFINED in AccVGPRs, see prescale_q,
// so the compiler has no copy to place there; the probabilities are packed at least a slot ahead).
template <typename Tag>
struct Mai;
template <>
struct Mai<bf16_tag> {
    // s += a . b   (a, b: AccVGPRs, s: VGPRs)
    static __device__ __forceinline__ void score(f32x16_t& s, u32x4_t a, u32x4_t b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(s) : "a"(a), "a"(b));
    }
    // s = c + a . b   (c: a second VGPR tuple, left untouched)
    static __device__ __forceinline__ void score_first(f32x16_t& s, u32x4_t a, u32x4_t b, const f32x16_t& c) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(s) : "a"(a), "a"(b), "v"(c));
    }
    // o += a . b   (a: AccVGPRs, b: VGPRs, o: AccVGPRs)
    static __device__ __forceinline__ void accumulate(f32x16_t& o, u32x4_t a, u32x4_t b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(o) : "a"(a), "v"(b));
    }
};
template <>
struct Mai<f16_tag> {
    static __device__ __forceinline__ void score(f32x16_t& s, u32x4_t a, u32x4_t b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(s) : "a"(a), "a"(b));
    }
    static __device__ __forceinline__ void score_first(f32x16_t& s, u32x4_t a, u32x4_t b, const f32x16_t& c) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(s) : "a"(a), "a"(b), "v"(c));
    }
    static __device__ __forceinline__ void accumulate(f32x16_t& o, u32x4_t a, u32x4_t b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(o) : "a"(a), "v"(b));
    }
};
// o *= alpha for an accumulator block that lives in AccVGPRs.  The empty volatile statement makes the block a fresh
// value INSIDE the (rare) branch that rescales; without it the compiler hoists the AccVGPR reads in front of the
// branch, 128 moves per tile whether a row maximum moved or not.
__device__ __forceinline__ void rescale_acc(f32x16_t& o, float alpha) {
    asm volatile("" : "+a"(o));
#pragma unroll
    for (int i = 0; i < 16; ++i) o[i] *= alpha;
    asm volatile("" : "+a"(o));
}

// 16 wait states: more than an 8-pass MFMA needs before the VALU may read its result.  The values that must not be
// read earlier are operands of the statement: a compiler-generated read may be moved across a volatile statement it
// does not depend on (only volatile statements keep their order among themselves), so the wait is tied to the data.
__device__ __forceinline__ void mfma_settle() { asm volatile("s_nop 15" ::: "memory"); }
__device__ __forceinline__ void mfma_settle(f32x16_t& x) { asm volatile("s_nop 15" : "+v"(x)::"memory"); }

// Scores of one key tile for the wave's two query blocks: s[qb][kb], accumulator layout of vqa_flash.h
// (lane (n, half), register r  <->  key kb*32 + 8*(r/4) + 4*half + r%4 of query n of block qb).
struct Scores {
    f32x16_t s[2][2];
};
__device__ __forceinline__ void mfma_settle(Scores& sc) {
    asm volatile("s_nop 15" : "+v"(sc.s[0][0]), "+v"(sc.s[0][1]), "+v"(sc.s[1][0]), "+v"(sc.s[1][1])::"memory");
}

template <typename Tag, int D>
struct Wave {
    typedef Geom<D> G;
    QFrag<Tag, D> q[2];            // query blocks (B operands of S^T = K.Q^T), pre-multiplied by scale * log2(e)
    f32x16_t o[2][G::kDBlocks];    // O^T accumulators
    f32x16_t negm[2];              // -m in every element: the addend of the first score MFMA of a tile
    float m[2];                    // reference maximum (base 2, scaled; -inf while nothing was seen), per block
    float l[2][2];                 // two partial row sums per block (even / odd keys of the lane)
    u32x4_t p[2][4];               // packed probabilities of the current tile: [block][16-key step]
    float ex[2][2];                // exp stream: exponentials of the current unit and of the one before

    __device__ __forceinline__ void init() {
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            m[qb] = -INFINITY;
            l[qb][0] = l[qb][1] = 0.f;
#pragma unroll
            for (int i = 0; i < 16; ++i) negm[qb][i] = 0.f;
#pragma unroll
            for (int db = 0; db < G::kDBlocks; ++db)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[qb][db][i] = 0.f;
        }
    }
};

// q *= c (fp32 product, one rounding to the element type).  The kernels fold softmax_scale * log2(e) into the query
// once, so that a score leaves the matrix pipe ready for exp2.
template <typename Tag, int D>
__device__ __forceinline__ void prescale_q(QFrag<Tag, D>& q, float c) {
    typedef typename Elem<Tag>::vec8 vec8;
#pragma unroll
    for (int kk = 0; kk < Geom<D>::kKSteps; ++kk) {
        u32x4_t x = __builtin_bit_cast(u32x4_t, q.f[kk]);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            x[e] = Elem<Tag>::pack2(Elem<Tag>::from_bits((uint16_t)(x[e] & 0xffffu)) * c,
                                    Elem<Tag>::from_bits((uint16_t)(x[e] >> 16)) * c);
        // the fragments live in AccVGPRs from here on (they are only ever an MFMA operand): defined there, the
        // register allocator keeps them there instead of copying them in front of every product
        asm volatile("" : "+a"(x));
        q.f[kk] = __builtin_bit_cast(vec8, x);
    }
}

// Copy of a whole 64-row tile, global -> LDS, with the per-lane part of the addresses computed once per kernel: load i
// of a wave (rows 16 * wave + kRowsPerInstr * i ...) takes a wave-uniform row address (scalar registers), the lane's
// 32-bit byte offset off[i] (row inside the group, swizzled 16-byte chunk) and an LDS address in M0.  The two halves
// of a load -- M0 write, direct-to-LDS load -- are issued separately so that the caller can put an MFMA between them
// (a load may not follow the M0 write directly).
template <int D, bool kIsV, int NW = 4>
struct TileDma {
    typedef Geom<D> G;
    static constexpr int kRowsPerWave = kBN / NW;  // NW waves share a tile copy
    static constexpr int kInstr = kRowsPerWave / G::kRowsPerInstr;
    uint32_t off[kInstr];
    __device__ __forceinline__ void init(int wave, int lane, int64_t sn) {
        const int lane_row = (int)((unsigned)lane / (unsigned)G::kChunksPerRow);
        const int chunk = (int)((unsigned)lane % (unsigned)G::kChunksPerRow);
#pragma unroll
        for (int i = 0; i < kInstr; ++i) {
            const int row_in_wave = i * G::kRowsPerInstr + lane_row;
            const int row = wave * kRowsPerWave + row_in_wave;
            const int src_chunk = chunk ^ (kIsV ? G::swz_v(row) : G::swz_k(row));
            off[i] = (uint32_t)row_in_wave * (uint32_t)(sn * 2) + (uint32_t)src_chunk * 16u;
        }
    }
    // LDS byte address of this wave's rows inside the tile at lds_tile
    static __device__ __forceinline__ uint32_t lds_of_wave(uint32_t lds_tile, int wave) {
        return lds_tile + (uint32_t)(wave * kRowsPerWave * G::kRowBytes);
    }
    template <int I>
    static __device__ __forceinline__ void aim(uint32_t lds_wave) {
        asm volatile("s_add_u32 m0, %0, %1" : : "s"(lds_wave), "n"(I * G::kRowsPerInstr * G::kRowBytes) : "scc");
    }
    template <int I>
    __device__ __forceinline__ void fire(const char* wave_rows) const {
        asm volatile("global_load_lds_dwordx4 %0, %1" : : "v"(off[I]), "s"(wave_rows) : "memory");
    }
};

template <typename Tag, int D, int NW = 4>
struct Pipe {
    typedef Geom<D> G;
    typedef typename Elem<Tag>::vec8 vec8;
    typedef const __attribute__((address_space(3))) vec8* lds_vec8_ptr;
    typedef __attribute__((address_space(3))) s16x4_t* lds_tr_ptr;
    static constexpr int KS = G::kKSteps, DB = G::kDBlocks;
    static constexpr int kScoreSlots = 4 * KS;  // MFMAs of S^T for both query blocks
    static constexpr int kPvSlots = 8 * DB;     // MFMAs of O^T += V^T.P^T for both query blocks
    static constexpr int kUnits = 32;           // exp units per tile: one packed pair of probabilities each

    // The VALU work of a tile is cut into single instructions ("micro-ops") and dealt out evenly over the MFMA slots:
    // a lone wave gets four to five VALU instructions into the shadow of one MFMA, every further one idles the matrix
    // pipe, and an empty slot is a wasted shadow.
    //   exp stream of the CURRENT tile: 5 micro-ops per stream step, kUnits + 1 steps (see exp_micro_op); the first
    //   kMicroScore of them run under the score MFMAs of the NEXT tile, the rest under the first kPvStream P.V MFMAs;
    //   row maxima of the NEXT tile: kUnits v_max3 over the P.V slots from kMaxFirst on.
    static constexpr int kMicroOps = 5 * (kUnits + 1);
#ifdef VQA_TUNE_MICRO_SCORE
    static constexpr int kMicroScore = VQA_TUNE_MICRO_SCORE;
    static constexpr int kPvStream = VQA_TUNE_PV_STREAM;
#else
    static constexpr int kMicroScore = D == 128 ? 100 : 80;
    static constexpr int kPvStream = D == 128 ? 22 : 11;
#endif
#ifdef VQA_TUNE_MAX_FIRST
    static constexpr int kMaxFirst = VQA_TUNE_MAX_FIRST;
#else
    static constexpr int kMaxFirst = D == 128 ? 16 : 2;  // (>= 2: the last score MFMA must be two MFMAs old)
#endif
    // micro-ops finished once slot g is through (score slots first, then the P.V slots)
    static constexpr int micro_done(int g) {
        if (g < 0) return 0;
        if (g < kScoreSlots) return kMicroScore * (g + 1) / kScoreSlots;
        const int i = g - kScoreSlots;
        if (i >= kPvStream) return kMicroOps;
        return kMicroScore + (kMicroOps - kMicroScore) * (i + 1) / kPvStream;
    }
    static constexpr int max_done(int i) {  // v_max3 units finished once P.V slot i is through
        if (i < kMaxFirst) return 0;
        return kUnits * (i - kMaxFirst + 1) / (kPvSlots - kMaxFirst);
    }
    // the probabilities of 16-key step j (units 8j .. 8j+7, packed by micro-op 5 * (unit + 1) + 2) are complete, with
    // a slot to spare, before the first P.V MFMA that reads them
    static constexpr bool deadlines_met() {
        for (int j = 0; j < 4; ++j)
            if (micro_done(kScoreSlots + 2 * DB * j - 2) < 5 * (8 * j + 8) + 3) return false;
        return true;
    }
    static_assert(deadlines_met(), "the exp stream is too late for the P.V products");
    static_assert(kPvStream <= kPvSlots && kMicroScore <= kMicroOps, "schedule out of range");

    // per-lane LDS address of the A fragment (row block rb, k-step 0) of a swizzled 64-row tile
    // (tiles are named by their 32-bit LDS byte address)
    static __device__ __forceinline__ uint32_t frag_base(uint32_t lds_tile, int lane) {
        const int r = lane & 31, half = lane >> 5;
        return lds_tile + ((uint32_t)(r * G::kRowBytes) | (uint32_t)((half ^ G::swz_k(r)) << 4));
    }
    static __device__ __forceinline__ vec8 frag(uint32_t base, int rb, int kk) {
        const uint32_t addr = (base ^ (uint32_t)((2 * kk) << 4)) + rb * 32 * G::kRowBytes;
        return *(lds_vec8_ptr)(uintptr_t)addr;
    }
    static __device__ __forceinline__ uint32_t vfrag_base(uint32_t lds_v, int lane) {
        const int half = lane >> 5, dsub = (lane >> 4) & 1, sl = lane & 15;
        const int row = 4 * half + (sl >> 2);
        return lds_v +
               ((uint32_t)(row * G::kRowBytes) | (uint32_t)(((2 * dsub + ((sl & 3) >> 1)) ^ G::swz_v(row)) << 4) |
                (uint32_t)((sl & 1) << 3));
    }
    // V^T fragment of 16-key step j, d block db (two transposing reads)
    static __device__ __forceinline__ vec8 vfrag(uint32_t base, int j, int db) {
        const uint32_t addr = (base ^ (uint32_t)((4 * db) << 4)) + j * 16 * G::kRowBytes;
        const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(uintptr_t)addr);
        const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(uintptr_t)(addr + 8 * G::kRowBytes));
        const short __attribute__((ext_vector_type(8))) av = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(vec8, av);
    }

    // The exponentials of a tile are a stream of 32 units (one packed pair of probabilities each: unit = step*8 +
    // block*4 + e;  16-key step = kb*2 + j2;  registers j2*8 + 2e, +1 of s[block][kb]), evaluated in two stages one unit
    // apart -- stream step K does   the two exp2 of unit K,   then pack and the two row-sum additions of unit K-1   --
    // so that no instruction consumes the result of the one right before it (a transcendental feeding the next
    // instruction costs wait states).  Micro-op X is instruction X % 5 of stream step X / 5.  The scores arrive as
    // scale * s - m (query pre-scaled, -m added by the first score MFMA): the exponent needs no arithmetic.
    // The row sums are plain fp32 additions of the unrounded exponentials: v_dot2 on the packed pair would be one
    // instruction instead of two, but the dot instructions share the matrix pipe -- next to MFMAs each costs ~8 clocks
    // of that pipe (measured: MFMA + 4 v_dot2c 69 clocks, MFMA + 4 of any other VALU instruction 39).
    template <int X>
    static __device__ __forceinline__ void exp_micro_op(Wave<Tag, D>& w, const Scores& sc) {
        constexpr int K = X / 5, part = X % 5;
        if constexpr (part < 2) {
            if constexpr (K < kUnits) {
                constexpr int step = K / 8, qb = (K / 4) % 2, e = K % 4;
                constexpr int kb = step / 2, j2 = step % 2, r = j2 * 8 + 2 * e;
                w.ex[K % 2][part] = fast_exp2(sc.s[qb][kb][r + part]);
                pin(w.ex[K % 2][part]);
            }
        } else if constexpr (K >= 1) {
            constexpr int U = K - 1, step = U / 8, qb = (U / 4) % 2, e = U % 4;
            if constexpr (part == 2) {
                uint32_t pk = Elem<Tag>::pack2(w.ex[U % 2][0], w.ex[U % 2][1]);
                pin(pk);
                w.p[qb][step][e] = pk;
            } else {
                w.l[qb][part - 3] += w.ex[U % 2][part - 3];
                pin(w.l[qb][part - 3]);
            }
        }
    }
    // max unit IDX: mx[block] = max(mx[block], two more scores of the tile in `sn`)
    template <int IDX>
    static __device__ __forceinline__ void max_unit(float (&mx)[2], const Scores& sn) {
        // the two blocks alternate, so that a v_max3 never waits for the one right before it
        constexpr int qb = IDX % 2, t = IDX / 2, kb = t / 8, r = 2 * (t % 8);
        mx[qb] = fmaxf(fmaxf(mx[qb], sn.s[qb][kb][r]), sn.s[qb][kb][r + 1]);
        pin(mx[qb]);
    }

    // Operand fragments travel LDS -> AccVGPRs in PAIRS (two consecutive fragments of the consumption order), the
    // second of a pair requested first: LDS returns data in order, so the wait in front of the first use of the pair
    // covers both, one s_waitcnt per pair instead of one per fragment (every instruction of a lone wave costs issue
    // time, also the ones that do nothing).  kPairsAhead pairs are in flight; the first ones of a phase ("head") are
    // requested before the phase starts, under the tail of the previous one.
#ifdef VQA_TUNE_PAIRS_AHEAD
    static constexpr int kPairsAhead = VQA_TUNE_PAIRS_AHEAD;
#else
    static constexpr int kPairsAhead = 2;
#endif
    static constexpr int kRingPairs = kPairsAhead + 1;
    struct Frags {
        vec8 f[2 * kRingPairs];
        uint32_t base;  // per-lane LDS address of fragment 0 of the tile being read
    };
    // K fragment f = 2 * kk + kb (k-step kk, key block kb); pair P = k-step P
    template <int P>
    static __device__ __forceinline__ void load_k_pair(Frags& r) {
        constexpr int s = (P % kRingPairs) * 2;
        r.f[s + 1] = frag(r.base, 1, P);
        __builtin_amdgcn_sched_barrier(0);
        r.f[s] = frag(r.base, 0, P);
        __builtin_amdgcn_sched_barrier(0);
    }
    static __device__ __forceinline__ void k_head(Frags& r, uint32_t lds_k, int lane) {
        r.base = frag_base(lds_k, lane);
        static_for<kPairsAhead>([&](auto P) { load_k_pair<decltype(P)::value>(r); });
    }
    // V^T fragment f = j * DB + db (16-key step j, d block db); pair P = fragments 2P, 2P + 1
    template <int P>
    static __device__ __forceinline__ void load_v_pair(Frags& r) {
        constexpr int s = (P % kRingPairs) * 2;
        r.f[s + 1] = vfrag(r.base, (2 * P + 1) / DB, (2 * P + 1) % DB);
        __builtin_amdgcn_sched_barrier(0);
        r.f[s] = vfrag(r.base, (2 * P) / DB, (2 * P) % DB);
        __builtin_amdgcn_sched_barrier(0);
    }
    static __device__ __forceinline__ void v_head(Frags& r, uint32_t lds_v, int lane) {
        r.base = vfrag_base(lds_v, lane);
        static_for<kPairsAhead>([&](auto P) { load_v_pair<decltype(P)::value>(r); });
    }

    // Score phase.  kMma: sn = -m + K tile . Q^T for both blocks (kf: the tile's fragment ring, head requested).  kExp: the
    // first kMicroScore micro-ops of the exp stream of `sc`.  kVHead: ends by requesting the head of the V tile lds_v.
    // kDma: the wave's share of two tile copies (K tile: kd / kr, V tile: vd / vr) rides along, one load per slot with
    // the MFMA between the M0 write and the load.
    struct TileRequest {
        const char* rows;  // wave-uniform global address of the wave's first row of the tile
        uint32_t lds;      // LDS byte address of that row in the destination tile
    };
    typedef TileDma<D, false, NW> KDma;
    typedef TileDma<D, true, NW> VDma;
    static_assert(KDma::kInstr == VDma::kInstr && 2 * KDma::kInstr <= kScoreSlots, "tile copy does not fit the slots");
    template <bool kMma, bool kExp, bool kVHead, bool kDma>
    static __device__ __forceinline__ void score_phase(Wave<Tag, D>& w, Scores& sn, Frags& kf, const Scores& sc,
                                                       Frags& vf, uint32_t lds_v, int lane, const KDma& kd,
                                                       const TileRequest& kr, const VDma& vd, const TileRequest& vr) {
        constexpr int NI = KDma::kInstr;
        static_assert(kMma || !kDma, "the loads ride on the MFMA slots");
        static_for<kScoreSlots>([&](auto I) {
            constexpr int i = decltype(I)::value;
            constexpr int f = i / 2, qb = i % 2, kk = f / 2, kb = f % 2;
            if constexpr (kDma && i < NI) KDma::template aim<i>(kr.lds);
            if constexpr (kDma && i >= NI && i < 2 * NI) VDma::template aim<i - NI>(vr.lds);
            if constexpr (kMma) {
                if constexpr (i % 4 == 0 && kk + kPairsAhead < KS) load_k_pair<kk + kPairsAhead>(kf);
                const u32x4_t a = __builtin_bit_cast(u32x4_t, kf.f[(kk % kRingPairs) * 2 + kb]);
                const u32x4_t bq = __builtin_bit_cast(u32x4_t, w.q[qb].f[kk]);
                if constexpr (kk == 0)
                    Mai<Tag>::score_first(sn.s[qb][kb], a, bq, w.negm[qb]);
                else
                    Mai<Tag>::score(sn.s[qb][kb], a, bq);
            }
            if constexpr (kExp) {
                constexpr int x0 = micro_done(i - 1), x1 = micro_done(i);
                static_for<x1 - x0>([&](auto X) { exp_micro_op<x0 + decltype(X)::value>(w, sc); });
            }
            if constexpr (kDma && i < NI) kd.template fire<i>(kr.rows);
            if constexpr (kDma && i >= NI && i < 2 * NI) vd.template fire<i - NI>(vr.rows);
            if constexpr (kVHead && i == kScoreSlots - 3) v_head(vf, lds_v, lane);
            __builtin_amdgcn_sched_barrier(0);
        });
    }

    // P.V phase.  kPv: O^T += V^T.P^T (vf: the V tile's fragment ring, head requested) with the rest of the exp stream of
    // `sc` under its first MFMAs, kMax: the row maxima of `sn`.
    template <bool kPv, bool kMax>
    static __device__ __forceinline__ void pv_phase(Wave<Tag, D>& w, Frags& vf, const Scores& sc, Scores& sn,
                                                    float (&mx)[2]) {
        constexpr int NP = 2 * DB;  // pairs of V^T fragments
        if constexpr (!kPv && kMax) mfma_settle(sn);  // the maxima follow the score MFMAs directly
        static_for<kPvSlots>([&](auto I) {
            constexpr int i = decltype(I)::value;
            constexpr int f = i / 2, qb = i % 2, j = f / DB, db = f % DB, pr = f / 2;
            if constexpr (kPv) {
                if constexpr (i % 4 == 0 && pr + kPairsAhead < NP) load_v_pair<pr + kPairsAhead>(vf);
                Mai<Tag>::accumulate(w.o[qb][db], __builtin_bit_cast(u32x4_t, vf.f[(pr % kRingPairs) * 2 + f % 2]),
                                     w.p[qb][j]);
                constexpr int x0 = micro_done(kScoreSlots + i - 1), x1 = micro_done(kScoreSlots + i);
                static_for<x1 - x0>([&](auto X) { exp_micro_op<x0 + decltype(X)::value>(w, sc); });
            }
            if constexpr (kMax) {
                constexpr int u0 = i == 0 ? 0 : max_done(i - 1), u1 = max_done(i);
                static_for<u1 - u0>([&](auto U) { max_unit<u0 + decltype(U)::value>(mx, sn); });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    }

    // Waits out the last P.V MFMAs with the O tuples as operands: whatever reads O afterwards -- the stores below, but
    // also a copy the register allocator decides to make -- depends on this statement and cannot precede it.  (A
    // compiler-made v_accvgpr_read right behind the last MFMA returned a stale last element of each tuple.)
    static __device__ __forceinline__ void settle_o(Wave<Tag, D>& w) {
        static_assert(DB == 4 || DB == 2, "head dims 128 and 64");
        if constexpr (DB == 4)
            asm volatile("s_nop 15"
                         : "+a"(w.o[0][0]), "+a"(w.o[0][1]), "+a"(w.o[0][2]), "+a"(w.o[0][3]), "+a"(w.o[1][0]),
                           "+a"(w.o[1][1]), "+a"(w.o[1][2]), "+a"(w.o[1][3])::"memory");
        else
            asm volatile("s_nop 15" : "+a"(w.o[0][0]), "+a"(w.o[0][1]), "+a"(w.o[1][0]), "+a"(w.o[1][1])::"memory");
    }

    // Moves the reference maxima of the wave's rows for the tile whose scores are in `sc` (relative to the present
    // maxima, as the matrix pipe delivered them) and whose per-lane maxima are in mx.  Lazy rule: a row moves only when
    // the tile exceeds its maximum by more than 2^kLazy (or is the first one it sees).  Where a row moved, l and O are
    // rescaled, the tile's scores are shifted to the new maximum and the addend of the coming score MFMAs is renewed.
    // Must run after the previous tile's P.V and before this tile's exp units and the next tile's score MFMAs.
    // The usual case -- no row of the wave moves -- is two compares and a branch: a row's maximum is the larger of the
    // values its two lanes hold, so "some row exceeds its threshold" can be read off the lanes before they are joined.
    static __device__ __forceinline__ void update_max(Wave<Tag, D>& w, const float (&mx)[2], Scores& sc) {
        const bool any0 = mx[0] > ((w.m[0] == -INFINITY) ? -INFINITY : kLazy);
        const bool any1 = mx[1] > ((w.m[1] == -INFINITY) ? -INFINITY : kLazy);
        if (__builtin_amdgcn_ballot_w64(any0 || any1) == 0) return;
        // rows that see their first key have l = O = 0: nothing to rescale.  That is every row at the start of a query
        // tile, so the first tile of a key loop does not pay for reading and writing all of O.
        const bool resc0 = any0 && w.m[0] != -INFINITY, resc1 = any1 && w.m[1] != -INFINITY;
        const bool rescale = __builtin_amdgcn_ballot_w64(resc0 || resc1) != 0;
        if (rescale) settle_o(w);  // O was last written by the previous tile's final MFMAs
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            const float rel = join_halves_max(mx[qb]);
            const bool first = w.m[qb] == -INFINITY;
            const bool need = rel > (first ? -INFINITY : kLazy);
            const float delta = need ? rel : 0.f;
            if (rescale) {
                // (a first key among rows that do move: any finite factor keeps l = O = 0; 2^-rel may overflow)
                const float alpha = (need && !first) ? fast_exp2(-delta) : (need ? 0.f : 1.f);
                w.l[qb][0] *= alpha;
                w.l[qb][1] *= alpha;
#pragma unroll
                for (int db = 0; db < DB; ++db) rescale_acc(w.o[qb][db], alpha);
            }
            const float m_old = first ? 0.f : w.m[qb];
            if (need) w.m[qb] = m_old + delta;
            // (-m as old value minus delta, element by element: written like this the register allocator updates the
            // tuple in place; a freshly built tuple ends up in other registers and is copied on the hot path)
#pragma unroll
            for (int i = 0; i < 16; ++i) w.negm[qb][i] -= delta;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int i = 0; i < 16; ++i) sc.s[qb][kb][i] -= delta;
        }
    }

    // Second operand pair of a tile (ReRoPE window edge): where take(qb, kb, r) holds, the score of `sn` is replaced by
    // -m + K tile (lds_k) . q^T with the wave's CURRENT query fragments.  One accumulation chain at a time with a
    // 16-register temporary; the chain's K fragments go through the (idle) fragment ring kf, six ahead, so that the
    // chain waits for LDS once and not eight times.  Nothing else is overlapped with it (it runs once per query tile
    // and wave).
    template <typename Take>
    static __device__ __forceinline__ void second_pair(Wave<Tag, D>& w, Scores& sn, uint32_t lds_k, int lane, Frags& kf,
                                                       Take take) {
        const uint32_t base = frag_base(lds_k, opaque_lane(lane));
        constexpr int kBuf = 2 * kRingPairs;
        constexpr int kPre = KS < kBuf ? KS : kBuf;
        static_for<4>([&](auto C) {
            constexpr int qb = decltype(C)::value / 2, kb = decltype(C)::value % 2;
            f32x16_t t;
            static_for<kPre>([&](auto I) { kf.f[decltype(I)::value] = frag(base, kb, decltype(I)::value); });
            static_for<KS>([&](auto KK) {
                constexpr int kk = decltype(KK)::value;
                const u32x4_t a = __builtin_bit_cast(u32x4_t, kf.f[kk % kBuf]);
                const u32x4_t bq = __builtin_bit_cast(u32x4_t, w.q[qb].f[kk]);
                if constexpr (kk == 0)
                    Mai<Tag>::score_first(t, a, bq, w.negm[qb]);
                else
                    Mai<Tag>::score(t, a, bq);
                // the buffer of the fragment used one step ago takes the fragment kBuf - 1 steps ahead
                if constexpr (kk >= 1 && kk - 1 + kBuf < KS) kf.f[(kk - 1) % kBuf] = frag(base, kb, kk - 1 + kBuf);
                __builtin_amdgcn_sched_barrier(0);
            });
            mfma_settle(t);
#pragma unroll
            for (int r = 0; r < 16; ++r) sn.s[qb][kb][r] = take(qb, kb, r) ? t[r] : sn.s[qb][kb][r];
        });
    }

    // The same without a staging area: every lane stores the 8-byte pieces of its own row (64 rows per instruction).
    // For callers whose LDS is in use when the rows are ready (tiles of the next query tile already on their way).
    static __device__ __forceinline__ void store_direct(Wave<Tag, D>& w, uint16_t* out_base, int64_t sn,
                                                        float* lse, int row0, int n_rows, int lane) {
        const int n = lane & 31, half = lane >> 5;
        settle_o(w);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            const float l_tot = join_halves_sum(w.l[qb][0] + w.l[qb][1]);
            const int row = row0 + qb * 32 + n;
            if (row >= n_rows) continue;
            const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
            uint16_t* dst = out_base + (int64_t)row * sn;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    uint2 pk;
                    pk.x = (uint32_t)Elem<Tag>::to_bits(w.o[qb][db][4 * g] * inv) |
                           ((uint32_t)Elem<Tag>::to_bits(w.o[qb][db][4 * g + 1] * inv) << 16);
                    pk.y = (uint32_t)Elem<Tag>::to_bits(w.o[qb][db][4 * g + 2] * inv) |
                           ((uint32_t)Elem<Tag>::to_bits(w.o[qb][db][4 * g + 3] * inv) << 16);
                    *reinterpret_cast<uint2*>(dst + db * 32 + 8 * g + 4 * half) = pk;
                }
            }
            if (lse != nullptr && half == 0) lse[row] = l_tot > 0.f ? w.m[qb] + fast_log2(l_tot) : -INFINITY;
        }
    }

    // Normalise and store the wave's 64 output rows; lse2 = m + log2(l).  A row that saw no key stores 0 / -inf.
    // In the accumulator layout a lane holds 4-element pieces of ONE row: stored directly, every instruction would
    // touch 64 rows.  The rows go through the wave's own LDS staging area instead (kStoreBytes at lds_stage, rows
    // padded by 8 bytes so that the 8-byte pieces of 32 rows fall into different banks) and leave as whole 256-byte
    // rows, 16 bytes per lane.  The caller makes sure no wave still reads what lies in that LDS area.
    static constexpr int kStoreRowBytes = G::kRowBytes + 8;
    static constexpr int kStoreBytes = kWaveRows * kStoreRowBytes;
    static __device__ __forceinline__ void store(Wave<Tag, D>& w, uint16_t* out_base, int64_t sn, float* lse,
                                                 int row0, int n_rows, int lane, char* lds_stage) {
        const int n = lane & 31, half = lane >> 5;
        settle_o(w);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            const float l_tot = join_halves_sum(w.l[qb][0] + w.l[qb][1]);
            const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
            char* dst = lds_stage + (qb * 32 + n) * kStoreRowBytes;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    // registers 4g..4g+3 are d = db*32 + 8g + 4*half + 0..3
                    uint2 pk;
                    pk.x = (uint32_t)Elem<Tag>::to_bits(w.o[qb][db][4 * g] * inv) |
                           ((uint32_t)Elem<Tag>::to_bits(w.o[qb][db][4 * g + 1] * inv) << 16);
                    pk.y = (uint32_t)Elem<Tag>::to_bits(w.o[qb][db][4 * g + 2] * inv) |
                           ((uint32_t)Elem<Tag>::to_bits(w.o[qb][db][4 * g + 3] * inv) << 16);
                    *reinterpret_cast<uint2*>(dst + (db * 32 + 8 * g + 4 * half) * 2) = pk;
                }
            }
            const int row = row0 + qb * 32 + n;
            if (lse != nullptr && half == 0 && row < n_rows)
                lse[row] = l_tot > 0.f ? w.m[qb] + fast_log2(l_tot) : -INFINITY;
        }
        wave_lds_sync();
        constexpr int kLanesPerRow = G::kRowBytes / 16, kRowsPerInstr = 64 / kLanesPerRow;
        const int r_in = lane / kLanesPerRow, c = lane % kLanesPerRow;
#pragma unroll
        for (int i = 0; i < kWaveRows / kRowsPerInstr; ++i) {
            const int r = i * kRowsPerInstr + r_in;
            // (8-byte reads: the padded rows are only 8-byte aligned)
            const uint2 lo = *reinterpret_cast<const uint2*>(lds_stage + r * kStoreRowBytes + c * 16);
            const uint2 hi = *reinterpret_cast<const uint2*>(lds_stage + r * kStoreRowBytes + c * 16 + 8);
            if (row0 + r < n_rows)
                *reinterpret_cast<uint4*>(out_base + (int64_t)(row0 + r) * sn + c * 8) = make_uint4(lo.x, lo.y, hi.x, hi.y);
        }
    }
};

}  // namespace flash2
}  // namespace vqa
