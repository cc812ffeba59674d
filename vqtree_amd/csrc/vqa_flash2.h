// Software-pipelined MFMA flash-attention core of the window / ReRoPE / VQ-prefill kernel (gfx950).
//
// Work split: one workgroup = 4 waves = 256 query rows, ONE wave per SIMD with the whole 512-register budget.  A wave
// owns 64 query rows as two 32-row blocks, so every K / V^T fragment it reads from LDS feeds two MFMAs (half the LDS
// operand traffic per FLOP of a 32-row wave), and the K / V tiles a workgroup copies serve 256 rows.
//
// With a single wave per SIMD nothing else hides the softmax behind the matrix pipe, so the wave does it itself: the
// scores of key tile u+1 are accumulated (S^T = K.Q^T, v_mfma_f32_32x32x16) while the exponentials of tile u are
// evaluated, and the row maxima of tile u+1 are taken while P(u).V(u) runs.  The code is written as MFMA "slots":
// slot i issues one MFMA (and the LDS read of a fragment a few slots ahead) followed by its share of the VALU work;
// scheduling barriers between slots keep that interleaving.
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
// needs by itself (O^T and the query fragments in AccVGPRs, everything the VALU touches in VGPRs) and spills; inline
// assembly pins it.  The compiler inserts no hazard wait states around inline assembly: an MFMA result is read by
// another MFMA only several MFMAs later (independent accumulation chains), and `mfma_settle()` stands wherever the
// VALU may read a result that the last few instructions produced.  The forms that take an AccVGPR operand start with
// two wait states of their own: when the compiler parks a query fragment in VGPRs it copies it (v_accvgpr_write)
// right in front of the statement, and an MFMA may not read a register a VALU instruction wrote in the two cycles
// before.
template <typename Tag>
struct Mai;
template <>
struct Mai<bf16_tag> {
    // s += a . b   (a: VGPRs, b: AccVGPRs, s: VGPRs)
    static __device__ __forceinline__ void score(f32x16_t& s, u32x4_t a, u32x4_t b) {
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(s) : "v"(a), "a"(b));
    }
    static __device__ __forceinline__ void score_first(f32x16_t& s, u32x4_t a, u32x4_t b) {
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(s) : "v"(a), "a"(b));
    }
    // the same with b in VGPRs (query fragments that come from LDS)
    static __device__ __forceinline__ void score_vb(f32x16_t& s, u32x4_t a, u32x4_t b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(s) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void score_first_vb(f32x16_t& s, u32x4_t a, u32x4_t b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(s) : "v"(a), "v"(b));
    }
    // o += a . b   (a, b: VGPRs, o: AccVGPRs)
    static __device__ __forceinline__ void accumulate(f32x16_t& o, u32x4_t a, u32x4_t b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(o) : "v"(a), "v"(b));
    }
};
template <>
struct Mai<f16_tag> {
    static __device__ __forceinline__ void score(f32x16_t& s, u32x4_t a, u32x4_t b) {
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(s) : "v"(a), "a"(b));
    }
    static __device__ __forceinline__ void score_first(f32x16_t& s, u32x4_t a, u32x4_t b) {
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(s) : "v"(a), "a"(b));
    }
    static __device__ __forceinline__ void score_vb(f32x16_t& s, u32x4_t a, u32x4_t b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(s) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void score_first_vb(f32x16_t& s, u32x4_t a, u32x4_t b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(s) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void accumulate(f32x16_t& o, u32x4_t a, u32x4_t b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(o) : "v"(a), "v"(b));
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

// 16 wait states: more than an 8-pass MFMA needs before the VALU may read its result
__device__ __forceinline__ void mfma_settle() { asm volatile("s_nop 15" ::: "memory"); }

// Scores of one key tile for the wave's two query blocks: s[qb][kb], accumulator layout of vqa_flash.h
// (lane (n, half), register r  <->  key kb*32 + 8*(r/4) + 4*half + r%4 of query n of block qb).
struct Scores {
    f32x16_t s[2][2];
};

template <typename Tag, int D>
struct Wave {
    typedef Geom<D> G;
    QFrag<Tag, D> q[2];            // query blocks (B operands of S^T = K.Q^T)
    f32x16_t o[2][G::kDBlocks];    // O^T accumulators
    float m[2], l[2];              // reference maximum (base 2, scaled) and partial row sum, per block
    float m_use[2];                // m, or 0 while the row has seen nothing
    u32x4_t p[2][4];               // packed probabilities of the current tile: [block][16-key step]
    float ex[2][2];                // exp stream: exponentials of the unit before the current one, not packed yet
    uint32_t pk[2];                // exp stream: packed pair of the unit two back, not summed yet

    __device__ __forceinline__ void init() {
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            m[qb] = -INFINITY;
            l[qb] = 0.f;
            m_use[qb] = 0.f;
#pragma unroll
            for (int db = 0; db < G::kDBlocks; ++db)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[qb][db][i] = 0.f;
        }
    }
};

template <typename Tag, int D>
struct Pipe {
    typedef Geom<D> G;
    typedef typename Elem<Tag>::vec8 vec8;
    typedef const __attribute__((address_space(3))) vec8* lds_vec8_ptr;
    typedef __attribute__((address_space(3))) s16x4_t* lds_tr_ptr;
    static constexpr int KS = G::kKSteps, DB = G::kDBlocks;
    static constexpr int kScoreSlots = 4 * KS;  // MFMAs of S^T for both query blocks
    static constexpr int kPvSlots = 8 * DB;     // MFMAs of O^T += V^T.P^T for both query blocks
    static constexpr int kUnits = 32;           // exp units per tile: one packed pair of probabilities each
    static constexpr int kStreamSteps = kUnits + 2;
    static constexpr int kStepsEarly = 20;      // stream steps evaluated under the score MFMAs
    static constexpr int kMaxUnits = 32;        // v_max3 steps of the next tile's row maxima
    static constexpr int kAhead = 3;            // fragments read ahead of their MFMA

    // per-lane LDS address of the A fragment (row block rb, k-step 0) of a swizzled 64-row tile
    static __device__ __forceinline__ uint32_t frag_base(const char* lds_tile, int lane) {
        const int r = lane & 31, half = lane >> 5;
        return flash::lds_addr_of(lds_tile) + ((uint32_t)(r * G::kRowBytes) | (uint32_t)((half ^ G::swz_k(r)) << 4));
    }
    static __device__ __forceinline__ vec8 frag(uint32_t base, int rb, int kk) {
        const uint32_t addr = (base ^ (uint32_t)((2 * kk) << 4)) + rb * 32 * G::kRowBytes;
        return *(lds_vec8_ptr)(uintptr_t)addr;
    }
    static __device__ __forceinline__ uint32_t vfrag_base(const char* lds_v, int lane) {
        const int half = lane >> 5, dsub = (lane >> 4) & 1, sl = lane & 15;
        const int row = 4 * half + (sl >> 2);
        return flash::lds_addr_of(lds_v) +
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
    // block*4 + e;  16-key step = kb*2 + j2;  registers j2*8 + 2e, +1 of s[block][kb]), evaluated in three stages that
    // are one unit apart -- stream step K does   scale/subtract + exp of unit K,   pack of unit K-1,   row sum of unit
    // K-2   -- so that no instruction consumes the result of the one right before it (a transcendental or a pack
    // feeding the next instruction costs wait states).  kUnits + 2 stream steps finish a tile.
    template <int K>
    static __device__ __forceinline__ void exp_stream_step(Wave<Tag, D>& w, const Scores& sc, float scale) {
        if constexpr (K < kUnits) {
            constexpr int step = K / 8, qb = (K / 4) % 2, e = K % 4;
            constexpr int kb = step / 2, j2 = step % 2, r = j2 * 8 + 2 * e;
            w.ex[K % 2][0] = fast_exp2(__builtin_fmaf(sc.s[qb][kb][r], scale, -w.m_use[qb]));
            w.ex[K % 2][1] = fast_exp2(__builtin_fmaf(sc.s[qb][kb][r + 1], scale, -w.m_use[qb]));
        }
        if constexpr (K >= 1 && K <= kUnits) {
            constexpr int U = K - 1, step = U / 8, qb = (U / 4) % 2, e = U % 4;
            uint32_t pk = Elem<Tag>::pack2(w.ex[U % 2][0], w.ex[U % 2][1]);
            pin(pk);
            w.p[qb][step][e] = pk;
            w.pk[U % 2] = pk;
        }
        if constexpr (K >= 2 && K <= kUnits + 1) {
            constexpr int U = K - 2, qb = (U / 4) % 2;
            // sum of the ROUNDED pair, as P.V uses it
            w.l[qb] = Elem<Tag>::dot2(w.pk[U % 2], Elem<Tag>::pack2(1.f, 1.f), w.l[qb]);
            if constexpr (U % 4 == 3) pin(w.l[qb]);
        }
    }
    // max unit IDX: mx[block] = max(mx[block], two more scores of the tile in `sn`)
    template <int IDX>
    static __device__ __forceinline__ void max_unit(float (&mx)[2], const Scores& sn) {
        constexpr int qb = IDX / 16, t = IDX % 16, kb = t / 8, r = 2 * (t % 8);
        mx[qb] = fmaxf(fmaxf(mx[qb], sn.s[qb][kb][r]), sn.s[qb][kb][r + 1]);
        if constexpr (t % 4 == 3) pin(mx[qb]);
    }

    // Score phase.  kMma: sn = K tile (lds_k) . Q^T for both blocks.  kExp: the first kStepsEarly steps of the exp stream of `sc`.
    template <bool kMma, bool kExp>
    static __device__ __forceinline__ void score_phase(Wave<Tag, D>& w, Scores& sn, const char* lds_k,
                                                       const Scores& sc, float scale, int lane) {
        constexpr int NF = 2 * KS;  // K fragments: (k-step, key block)
        uint32_t base = 0;
        vec8 kf[kAhead + 1];
        if constexpr (kMma) {
            base = frag_base(lds_k, opaque_lane(lane));
#pragma unroll
            for (int f = 0; f < kAhead; ++f) kf[f] = frag(base, f % 2, f / 2);
        }
        static_for<kScoreSlots>([&](auto I) {
            constexpr int i = decltype(I)::value;
            constexpr int f = i / 2, qb = i % 2, kk = f / 2, kb = f % 2;
            if constexpr (kMma) {
                if constexpr (qb == 0 && f + kAhead < NF)
                    kf[(f + kAhead) % (kAhead + 1)] = frag(base, (f + kAhead) % 2, (f + kAhead) / 2);
                const u32x4_t a = __builtin_bit_cast(u32x4_t, kf[f % (kAhead + 1)]);
                const u32x4_t bq = __builtin_bit_cast(u32x4_t, w.q[qb].f[kk]);
                if constexpr (kk == 0)
                    Mai<Tag>::score_first(sn.s[qb][kb], a, bq);
                else
                    Mai<Tag>::score(sn.s[qb][kb], a, bq);
            }
            if constexpr (kExp) {
                constexpr int u0 = i * kStepsEarly / kScoreSlots, u1 = (i + 1) * kStepsEarly / kScoreSlots;
                static_for<u1 - u0>([&](auto U) { exp_stream_step<u0 + decltype(U)::value>(w, sc, scale); });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    }

    // P.V phase.  kPv: the rest of the exp stream of `sc` under the first half of O^T += V^T.P^T, kMax: the row maxima of
    // `sn` under the second half.
    template <bool kPv, bool kMax>
    static __device__ __forceinline__ void pv_phase(Wave<Tag, D>& w, const char* lds_v, const Scores& sc,
                                                    const Scores& sn, float (&mx)[2], float scale, int lane) {
        constexpr int NF = 4 * DB;  // V^T fragments: (16-key step, d block)
        constexpr int kHalf = kPvSlots / 2;
        uint32_t base = 0;
        vec8 vf[kAhead + 1];
        if constexpr (kPv) {
            base = vfrag_base(lds_v, opaque_lane(lane));
#pragma unroll
            for (int f = 0; f < kAhead; ++f) vf[f] = vfrag(base, f / DB, f % DB);
        } else if constexpr (kMax) {
            mfma_settle();  // the maxima follow the score MFMAs directly
        }
        static_for<kPvSlots>([&](auto I) {
            constexpr int i = decltype(I)::value;
            constexpr int f = i / 2, qb = i % 2, j = f / DB, db = f % DB;
            if constexpr (kPv) {
                if constexpr (qb == 0 && f + kAhead < NF)
                    vf[(f + kAhead) % (kAhead + 1)] = vfrag(base, (f + kAhead) / DB, (f + kAhead) % DB);
                Mai<Tag>::accumulate(w.o[qb][db], __builtin_bit_cast(u32x4_t, vf[f % (kAhead + 1)]), w.p[qb][j]);
                if constexpr (i < kHalf) {
                    constexpr int rest = kStreamSteps - kStepsEarly;
                    constexpr int u0 = kStepsEarly + i * rest / kHalf, u1 = kStepsEarly + (i + 1) * rest / kHalf;
                    static_for<u1 - u0>([&](auto U) { exp_stream_step<u0 + decltype(U)::value>(w, sc, scale); });
                }
            }
            if constexpr (kMax && i >= kHalf) {
                constexpr int u0 = (i - kHalf) * kMaxUnits / kHalf, u1 = (i - kHalf + 1) * kMaxUnits / kHalf;
                static_for<u1 - u0>([&](auto U) { max_unit<u0 + decltype(U)::value>(mx, sn); });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    }

    // Moves the reference maxima of the wave's rows for the tile whose raw row maxima are in mx (lazy rule) and
    // rescales l / O where a row moved.  Must run after the previous tile's P.V and before this tile's exp units.
    static __device__ __forceinline__ void update_max(Wave<Tag, D>& w, const float (&mx)[2], float scale) {
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            const float mxs = join_halves_max(mx[qb]) * scale;  // scale > 0
            const bool need = mxs > w.m[qb] + kLazy;             // also true for the first visible key (m = -inf)
            if (__builtin_amdgcn_ballot_w64(need) != 0) {
                mfma_settle();  // O was last written by the previous tile's final MFMAs
                const float m_new = need ? mxs : w.m[qb];
                const float alpha = need ? fast_exp2(w.m[qb] - m_new) : 1.f;  // m = -inf: alpha = 0, l = O = 0 anyway
                w.l[qb] *= alpha;
#pragma unroll
                for (int db = 0; db < DB; ++db) rescale_acc(w.o[qb][db], alpha);
                w.m[qb] = m_new;
            }
            w.m_use[qb] = (w.m[qb] == -INFINITY) ? 0.f : w.m[qb];
        }
    }

    // Extra operand pair of a tile: s2[kb] = K tile (lds_k) . Qx^T for query block qb, with the query fragments taken
    // from registers (kFromRegs) or from this wave's swizzled copy of the other query tensor in LDS (lds_q).
    template <bool kFromRegs>
    static __device__ __forceinline__ void extra_scores(f32x16_t (&s2)[2], const char* lds_k, const QFrag<Tag, D>& qreg,
                                                        const char* lds_q, int qb, int lane) {
        lane = opaque_lane(lane);
        const uint32_t kbase = frag_base(lds_k, lane);
        const uint32_t qbase = frag_base(lds_q, lane);
        static_for<KS>([&](auto KK) {
            constexpr int kk = decltype(KK)::value;
            // the register-held fragments are used exactly as in the score phase (AccVGPR operand), so that they keep
            // ONE home: a second kind of use makes the compiler park them in VGPRs and copy before every MFMA
            u32x4_t qf;
            if constexpr (!kFromRegs) qf = __builtin_bit_cast(u32x4_t, frag(qbase, qb, kk));
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const u32x4_t a = __builtin_bit_cast(u32x4_t, frag(kbase, kb, kk));
                if constexpr (kFromRegs) {
                    const u32x4_t bq = __builtin_bit_cast(u32x4_t, qreg.f[kk]);
                    if constexpr (kk == 0)
                        Mai<Tag>::score_first(s2[kb], a, bq);
                    else
                        Mai<Tag>::score(s2[kb], a, bq);
                } else {
                    if constexpr (kk == 0)
                        Mai<Tag>::score_first_vb(s2[kb], a, qf);
                    else
                        Mai<Tag>::score_vb(s2[kb], a, qf);
                }
            }
        });
        mfma_settle();
    }

    // Normalise and store the wave's 64 output rows; lse2 = m + log2(l).  A row that saw no key stores 0 / -inf.
    static __device__ __forceinline__ void store(const Wave<Tag, D>& w, uint16_t* out_base, int64_t sn, float* lse,
                                                 int row0, int n_rows, int lane) {
        const int n = lane & 31, half = lane >> 5;
        mfma_settle();
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            const float l_tot = join_halves_sum(w.l[qb]);
            const int row = row0 + qb * 32 + n;
            if (row >= n_rows) continue;
            const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
            uint16_t* dst = out_base + (int64_t)row * sn;
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
                    *reinterpret_cast<uint2*>(dst + db * 32 + 8 * g + 4 * half) = pk;
                }
            }
            if (lse != nullptr && half == 0) lse[row] = l_tot > 0.f ? w.m[qb] + fast_log2(l_tot) : -INFINITY;
        }
    }
};

}  // namespace flash2
}  // namespace vqa
