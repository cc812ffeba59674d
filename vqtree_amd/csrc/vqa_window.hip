// Exact sliding-window / ReRoPE / VQ-far-context prefill attention (seqlen_q == seqlen_k), one kernel template.
//
// Every variant is "causal flash attention whose score for (query i, key j) comes from one of up to three operand
// pairs, chosen by integer predicates on (i, j)":
//     pair A = (qa, ka)   in-window keys, rotary at true positions
//     pair B = (qb, kb)   keys beyond the window scored with the position-clamped query (ReRoPE)
//     pair C = (qb, kc)   far keys replaced by their additive-quantiser reconstruction kc = sum_m codebook[m][code]
// Tiles whose 128 x 64 (query x key) block uses a single pair and needs no mask take a fast path (one K tile,
// prefetched a tile ahead); tiles on the diagonal, on the window edge or on the far-context boundary are one step per
// pair they touch (each wave scoring only the pairs its own 32 rows select, merged and masked per element), every
// step's K tile requested one step ahead and the query operand of the next step requested behind the current product.
#include "vqa_flash.h"

namespace vqa {
namespace flash {

enum Mode : int {
    kLocalStrict = 0,  // j <= i, i - j <= W                                      (one pair)
    kLocalLoose = 1,   // j <= i, j >= floor(i/T)*T - W                           (one pair)
    kLocalRerope = 2,  // visible as loose; pair A iff i - j <= W, else pair B
    kFullRerope = 3,   // all keys (causal optional); pair A iff |i - j| < W, else pair B
    kVqPrefill = 4,    // causal optional; j < far_bnd(i) -> pair C; else A iff i - j <= W, else B
    kVqPrefill2 = 5    // same without a distinct pair B (no q2/k2 strip): two pairs, lower register pressure
};

enum Boundary : int { kBoundaryBlock = 0, kBoundaryExact = 1, kBoundaryAllFar = 2 };

struct Params {
    View qa, qb, ka, kb, kc, v;
    uint16_t* out;
    int64_t o_sb, o_sh, o_sn;
    float* lse;  // [B,H,N] contiguous, nullable
    int H, N;
    int window;
    int causal;
    int boundary;  // Boundary, kVqPrefill only
    int has_b;     // kVqPrefill: pair B is distinct from pair A (q2 and k2 both given)
    int pair_tiles;  // a workgroup handles query tiles (n-1-k, k) instead of one tile
    float scale_log2e;
};

// the value unchanged, but opaque to the optimiser: what is derived from it is not hoisted out of loops
__device__ __forceinline__ int opaque(int x) {
    asm volatile("" : "+v"(x));
    return x;
}

__device__ __forceinline__ int floor_div(int a, int b) { return (a >= 0) ? a / b : -((-a + b - 1) / b); }

template <int MODE>
struct Rules {
    int N, W, causal, boundary, has_b;

    // first key that is NOT quantised for query i (kVqPrefill)
    __device__ __forceinline__ int far_bnd(int i) const {
        if (boundary == kBoundaryAllFar) return 0x7fffffff;
        if (boundary == kBoundaryExact) return max(0, i - W);
        return max(0, floor_div(i - W, kTile) * kTile);
    }
    // lowest visible key for query i
    __device__ __forceinline__ int vis_lo(int i) const {
        if (MODE == kLocalStrict) return i - W;
        if (MODE == kLocalLoose || MODE == kLocalRerope) return (i / kTile) * kTile - W;
        return 0;
    }
    static constexpr bool kIsVq = (MODE == kVqPrefill || MODE == kVqPrefill2);
    __device__ __forceinline__ bool pair_b() const { return MODE == kVqPrefill2 ? false : has_b != 0; }
    __device__ __forceinline__ bool is_causal() const { return (MODE == kFullRerope || kIsVq) ? causal != 0 : true; }
    // Per-element predicates take the row's bounds precomputed (they depend on the query only):
    // lo = vis_lo(i), fb = far_bnd(i).
    __device__ __forceinline__ bool visible(int i, int j, int lo) const {
        return j < N && (!is_causal() || j <= i) && j >= lo;
    }
    // 0 = A, 1 = B, 2 = C
    __device__ __forceinline__ int source(int i, int j, int fb) const {
        if (MODE == kLocalStrict || MODE == kLocalLoose) return 0;
        if (MODE == kLocalRerope) return (i - j <= W) ? 0 : 1;
        if (MODE == kFullRerope) return (abs(i - j) < W) ? 0 : 1;
        if (j < fb) return 2;
        return (i - j <= W || !pair_b()) ? 0 : 1;
    }
};

struct TileClass {
    int need;   // bit s set: pair s is selected somewhere in the tile (may be a superset)
    bool fast;  // one pair, no mask
    int main;   // pair whose K tile is prefetched with V
};

// Classification of the key tile [n0, n0+64) against query rows [m0, m1] (workgroup-uniform).
template <int MODE>
__device__ __forceinline__ TileClass classify(const Rules<MODE>& r, int m0, int m1, int n0) {
    TileClass t;
    const int n1 = n0 + kBN - 1;
    const int dmin = m0 - n1, dmax = m1 - n0;  // range of i - j over the block
    const bool all_visible = (n1 < r.N) && (!r.is_causal() || n1 <= m0) && (n0 >= r.vis_lo(m1));
    bool needA = true, needB = false, needC = false;
    bool allA = true, allB = false, allC = false;
    if (MODE == kLocalRerope) {
        needA = dmin <= r.W;
        needB = dmax > r.W;
        allA = !needB;
        allB = !needA;
    } else if (MODE == kFullRerope) {
        needA = dmin < r.W && dmax > -r.W;
        allA = dmax < r.W && dmin > -r.W;
        needB = !allA;
        allB = !needA;
    } else if (Rules<MODE>::kIsVq) {
        needC = n0 < r.far_bnd(m1);
        allC = n1 < r.far_bnd(m0);
        needB = !allC && r.pair_b() && dmax > r.W;
        needA = !allC && (dmin <= r.W || !r.pair_b());
        allA = !needC && !needB;
        allB = !needC && !needA;
    }
    t.need = (needA ? 1 : 0) | (needB ? 2 : 0) | (needC ? 4 : 0);
    t.fast = all_visible && (allA || allB || allC);
    t.main = allC ? 2 : (needA ? 0 : (needB ? 1 : 2));
    return t;
}

template <typename Tag, int D, int MODE>
__global__ __launch_bounds__(kThreads, 2) void window_kernel(Params p) {
    typedef Geom<D> G;
    typedef typename Elem<Tag>::vec8 vec8;
    constexpr bool kDual = (MODE == kLocalRerope || MODE == kFullRerope || MODE == kVqPrefill || MODE == kVqPrefill2);

    // double-buffered K and V tiles, filled by direct global -> LDS loads one tile ahead of the compute
    __shared__ __attribute__((aligned(1024))) char s_k[2][G::kTileBytes];
    __shared__ __attribute__((aligned(1024))) char s_v[2][G::kTileBytes];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5, nq = lane & 31;
    // Workgroups are dispatched round-robin over the 8 XCDs (each with its own L2) in linear-id order.  Give every
    // XCD whole (batch, head) problems: the query tiles of one head then share its K/V through one L2.
    // With `pair_tiles` a workgroup takes query tile k from the end AND tile k from the start, so that under a
    // causal mask every workgroup does the same amount of work.
    const int n_tiles = (p.N + kBM - 1) / kBM;
    int bh, slot;
    {
        const int n_slots = gridDim.x, n_bh = gridDim.y;
        const int id = blockIdx.x + n_slots * blockIdx.y;
        if (n_bh % 8 == 0) {
            const int xcd = id & 7, k = id >> 3;
            bh = xcd + 8 * (k / n_slots);
            slot = k % n_slots;
        } else {
            bh = blockIdx.y;
            slot = blockIdx.x;
        }
    }
    const int b = bh / p.H, h = bh % p.H;
    const int t_first = n_tiles - 1 - slot;  // long (late) query tiles are scheduled first
    const int n_pass = (p.pair_tiles && slot != t_first) ? 2 : 1;

    Rules<MODE> rules{p.N, p.window, p.causal, p.boundary, p.has_b};

    const uint16_t* ka = p.ka.p + b * p.ka.sb + h * p.ka.sh;
    const uint16_t* kb_ = p.kb.p + b * p.kb.sb + h * p.kb.sh;
    const uint16_t* kc = p.kc.p + b * p.kc.sb + h * p.kc.sh;
    const uint16_t* v_src = p.v.p + b * p.v.sb + h * p.v.sh;
    auto k_ptr = [&](int src) { return src == 0 ? ka : (src == 1 ? kb_ : kc); };
    auto k_stride = [&](int src) { return src == 0 ? p.ka.sn : (src == 1 ? p.kb.sn : p.kc.sn); };

    TileCopy<D, false> k_copy;
    TileCopy<D, true> v_copy;
    k_copy.init(wave, lane);
    v_copy.init(wave, lane);

    const uint16_t* qa_src = p.qa.p + b * p.qa.sb + h * p.qa.sh;
    const uint16_t* qb_src = p.qb.p + b * p.qb.sb + h * p.qb.sh;
    uint16_t* out_base = p.out + b * p.o_sb + h * p.o_sh;
    float* lse_base = p.lse ? p.lse + (int64_t)bh * p.N : nullptr;

    // The workgroup walks a flat list of STEPS: step = one (key tile, operand pair) score product.  A key tile that
    // needs a single pair is one step; a tile on the window edge or the far-context boundary is one step per pair it
    // touches, the products being merged per element.  The list runs over the key tiles of the first query tile, in
    // the order given below, then over those of the second query tile (paired launch), so the loads of every step --
    // the first of a query tile included -- are requested one step ahead, and the K buffers alternate per step, the
    // V buffers per key tile.  Within a tile the pair scored last in the previous tile goes first, which keeps the
    // number of changes of the query operand per query tile at its minimum.
    //
    // Order of the key tiles of one query tile.  Modes that see the whole prefix walk up from key 0: the workgroups
    // of one head start together and so read the same K / V tiles at about the same time, sharing them through
    // the L2.  Sliding-window modes walk their window in a rotated order, key tile index modulo the number of
    // tiles in a window -- [u0, u_hi) then [u_lo, u0) -- for the same reason: at any step the workgroups of
    // neighbouring query tiles, which share most of their key tiles, are on tiles of the same residue.
    constexpr bool kRotate = (MODE == kLocalStrict || MODE == kLocalLoose || MODE == kLocalRerope);
    struct Cursor {
        int pass, m0, m1, u, seg_hi, u_lo, u0, wrapped, valid;  // plain ints: the struct stays in scalar registers
    };
    auto open_pass = [&](int pass) __attribute__((always_inline)) {
        Cursor c;
        c.valid = pass < n_pass ? 1 : 0;
        c.pass = pass;
        const int t = pass == 0 ? t_first : slot;
        c.m0 = t * kBM;
        c.m1 = min(c.m0 + kBM - 1, p.N - 1);
        const int hi_key = rules.is_causal() ? min(p.N, c.m1 + 1) : p.N;
        c.seg_hi = (hi_key + kBN - 1) / kBN;
        c.u_lo = max(0, rules.vis_lo(c.m0)) / kBN;
        c.u0 = c.u_lo;
        if (kRotate) {
            const int period = (rules.W + kBM + kBN - 1) / kBN;
            c.u0 = (c.u_lo + period - 1) / period * period;
            if (c.u0 >= c.seg_hi) c.u0 = c.u_lo;
        }
        c.u = c.u0;
        c.wrapped = (c.u0 == c.u_lo) ? 1 : 0;
        return c;
    };
    auto last_of_pass = [&](const Cursor& c) __attribute__((always_inline)) {
        return c.u + 1 >= c.seg_hi && c.wrapped;
    };
    auto next_tile = [&](const Cursor& c) __attribute__((always_inline)) {
        if (c.u + 1 < c.seg_hi) {
            Cursor n = c;
            ++n.u;
            return n;
        }
        if (!c.wrapped) {
            Cursor n = c;
            n.u = c.u_lo;
            n.seg_hi = c.u0;
            n.wrapped = 1;
            return n;
        }
        return open_pass(c.pass + 1);
    };
    // What one wave (32 query rows) has to do with a key tile, packed into one scalar: bits 0-2 the pairs that some
    // element of the wave's 32 x 64 block selects, bit 3 "a single pair and nothing masked", bit 4 "some element
    // is visible at all".
    auto wave_tile = [&](const Cursor& c) __attribute__((always_inline)) {
        const int r0 = min(c.m0 + wave * 32, p.N - 1), r1 = min(c.m0 + wave * 32 + 31, p.N - 1);
        const int n0 = c.u * kBN;
        const TileClass t = classify<MODE>(rules, r0, r1, n0);
        const bool visible = (!rules.is_causal() || n0 <= r1) && (n0 + kBN - 1 >= rules.vis_lo(r0));
        return t.need | (t.fast ? 8 : 0) | (visible ? 16 : 0);
    };
    auto wave_works = [](int tw, int src) __attribute__((always_inline)) { return (tw & 16) && ((tw >> src) & 1); };
    // the workgroup-wide classification packed the same way: bits 0-2 pairs needed, bit 3 fast, bits 4-5 main pair
    auto wg_tile = [&](const Cursor& c) __attribute__((always_inline)) {
        const TileClass t = classify<MODE>(rules, c.m0, c.m1, c.u * kBN);
        return t.need | (t.fast ? 8 : 0) | (t.main << 4);
    };
    auto first_src = [](int need, int prefer) __attribute__((always_inline)) {
        return ((need >> prefer) & 1) ? prefer : __builtin_ctz(need);
    };
    auto next_src = [](int need, int done) __attribute__((always_inline)) {
        const int rest = need & ~done;
        return rest ? __builtin_ctz(rest) : -1;
    };

    // One query fragment set lives in registers: pair A's or pair B's (pairs B and C share the query).
    QFrag<Tag, D> q;
    int q_held = -1;
    auto q_id = [&](const Cursor& c, int src) __attribute__((always_inline)) {
        return 2 * c.pass + ((kDual && src != 0) ? 1 : 0);
    };
    auto fetch_q = [&](const Cursor& c, int src) __attribute__((always_inline)) {
        const bool second = kDual && src != 0;
        load_q<Tag, D>(q, second ? qb_src : qa_src, second ? p.qb.sn : p.qa.sn, c.m0 + wave * 32, p.N, lane);
        q_held = q_id(c, src);
    };

    SoftmaxState<D> st;
    st.init();

    Cursor c = open_pass(0);
    int tc = wg_tile(c);
    int tw = wave_tile(c);
    int src = first_src(tc & 7, tc >> 4);
    int kbuf = 0, vbuf = 0;
    k_copy.load(s_k[0], k_ptr(src), k_stride(src), c.u * kBN, p.N);
    v_copy.load(s_v[0], v_src, p.v.sn, c.u * kBN, p.N);
    if (wave_works(tw, src)) fetch_q(c, src);

    while (c.valid) {
        // A run of tiles that every wave scores with one pair and no mask goes through a loop of its own: nothing
        // to classify per wave, whole-tile loads, one barrier per tile.  The last tile of a run is left to the
        // general code below, which knows how to request whatever follows.
        if (tc & 8) {
            const int run_src = tc >> 4;
            int run = 0;  // tiles after this one, contiguous in this segment, of the same kind
            while (c.u + run + 1 < c.seg_hi) {
                const TileClass t2 = classify<MODE>(rules, c.m0, c.m1, (c.u + run + 1) * kBN);
                if (!t2.fast || t2.main != run_src) break;
                ++run;
            }
            if (run > 0) {
                if (q_held != q_id(c, run_src)) {
                    wait_tile_loads();
                    fetch_q(c, run_src);
                    wait_tile_loads();
                }
                const uint16_t* run_k = k_ptr(run_src);
                const int64_t run_sn = k_stride(run_src);
                for (; run > 0; --run) {
                    wait_tile_loads();
                    __syncthreads();
                    k_copy.load_full(s_k[kbuf ^ 1], run_k, run_sn, (c.u + 1) * kBN);
                    v_copy.load_full(s_v[vbuf ^ 1], v_src, p.v.sn, (c.u + 1) * kBN);
                    f32x16_t s[2];
                    qk_mma<Tag, D>(s, q, s_k[kbuf], lane);
                    vec8 pf[2][2];
                    softmax_update<Tag, D, false>(st, s, p.scale_log2e, pf, nullptr);
                    pv_mma<Tag, D>(st.o, pf, s_v[vbuf], lane);
                    kbuf ^= 1;
                    vbuf ^= 1;
                    ++c.u;
                }
                tw = wave_tile(c);  // tc is unchanged: same kind of tile
            }
        }
        const Cursor nc = next_tile(c);
        int ntc = tc, ntw = tw;
        if (nc.valid) {
            ntc = wg_tile(nc);
            ntw = wave_tile(nc);
        }
        const int n0 = c.u * kBN;
        f32x16_t s[2];
        bool have_s = false, first_step = true;
        int done = 0, last_src = src;
        while (src >= 0) {
            done |= 1 << src;
            last_src = src;
            const int same = next_src(tc & 7, done);  // next pair of this tile, if any
            const bool work = wave_works(tw, src);
            wait_tile_loads();
            __syncthreads();  // this step's K (and the tile's V) are complete; every wave is done with the last step
            if (work && q_held != q_id(c, src)) {  // not requested ahead: this wave sat out the previous step
                fetch_q(c, src);
                wait_tile_loads();
            }
            // request what the next step reads
            int f_src = same;
            if (same >= 0) {
                k_copy.load(s_k[kbuf ^ 1], k_ptr(same), k_stride(same), n0, p.N);
            } else if (nc.valid) {
                f_src = first_src(ntc & 7, src);
                k_copy.load(s_k[kbuf ^ 1], k_ptr(f_src), k_stride(f_src), nc.u * kBN, p.N);
            }
            if (first_step && nc.valid) v_copy.load(s_v[vbuf ^ 1], v_src, p.v.sn, nc.u * kBN, p.N);
            first_step = false;

            if (work) {
                if (!have_s) {
                    qk_mma<Tag, D>(s, q, s_k[kbuf], lane);
                    have_s = true;
                } else {
                    // per-lane row data is recomputed here (a few VALU operations) instead of living in registers
                    // across the whole loop nest
                    const int ln = opaque(lane);
                    const int qi = c.m0 + wave * 32 + (ln & 31);
                    const int qi_far_bnd = Rules<MODE>::kIsVq ? rules.far_bnd(qi) : 0;
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb) {
                        const f32x16_t s2 = qk_block<Tag, D>(q, s_k[kbuf], kb, lane);
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const int j = n0 + kb * 32 + key_of_reg(r, ln >> 5);
                            if (rules.source(qi, j, qi_far_bnd) == src) s[kb][r] = s2[r];
                        }
                    }
                }
            }
            // the query operand of the step after this one, if this wave takes part in it and holds the other one:
            // requested now, behind the products that read the registers, so that the softmax and P.V hide it
            if (f_src >= 0) {
                __builtin_amdgcn_sched_barrier(0);  // keep the reload behind the products: one operand set in registers
                const bool f_same = same >= 0;
                const int fw = f_same ? tw : ntw;
                if (wave_works(fw, f_src)) {
                    if (f_same) {
                        if (q_held != q_id(c, f_src)) fetch_q(c, f_src);
                    } else {
                        if (q_held != q_id(nc, f_src)) fetch_q(nc, f_src);
                    }
                }
            }
            kbuf ^= 1;
            src = same;
        }
        if (have_s) {
            if (!(tw & 8)) {
                const int ln = opaque(lane);
                const int qi = c.m0 + wave * 32 + (ln & 31);
                const int qi_vis_lo = rules.vis_lo(qi);
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int j = n0 + kb * 32 + key_of_reg(r, ln >> 5);
                        s[kb][r] = rules.visible(qi, j, qi_vis_lo) ? s[kb][r] : -INFINITY;
                    }
            }
            vec8 pf[2][2];
            softmax_update<Tag, D, false>(st, s, p.scale_log2e, pf, nullptr);
            pv_mma<Tag, D>(st.o, pf, s_v[vbuf], lane);
        }
        if (last_of_pass(c)) {  // last key tile of this query tile
            store_output<Tag, D>(st, out_base, p.o_sn, lse_base, c.m0 + wave * 32, p.N, lane);
            st.init();
        }
        vbuf ^= 1;
        c = nc;
        tc = ntc;
        tw = ntw;
        src = c.valid ? first_src(tc & 7, last_src) : -1;
    }
}

template <typename Tag, int D, int MODE>
int launch(Params p, int B, hipStream_t stream) {
    const int n_tiles = (p.N + kBM - 1) / kBM;
    // Pair late (long) and early (short) query tiles whenever enough workgroups remain to fill the 256 CUs twice
    // over: under a causal mask every workgroup then does the same amount of work.
    p.pair_tiles = ((int64_t)(n_tiles / 2) * B * p.H >= 1024) ? 1 : 0;
    const dim3 grid(p.pair_tiles ? (n_tiles + 1) / 2 : n_tiles, B * p.H);
    hipLaunchKernelGGL((window_kernel<Tag, D, MODE>), grid, dim3(kThreads), 0, stream, p);
    return launch_status();
}

template <typename Tag, int D>
int dispatch_mode(const Params& p, int B, int mode, hipStream_t stream) {
    switch (mode) {
        case kLocalStrict: return launch<Tag, D, kLocalStrict>(p, B, stream);
        case kLocalLoose: return launch<Tag, D, kLocalLoose>(p, B, stream);
        case kLocalRerope: return launch<Tag, D, kLocalRerope>(p, B, stream);
        case kFullRerope: return launch<Tag, D, kFullRerope>(p, B, stream);
        case kVqPrefill:
            return p.has_b ? launch<Tag, D, kVqPrefill>(p, B, stream) : launch<Tag, D, kVqPrefill2>(p, B, stream);
        default: return VQA_ERR_BAD_ARGUMENT;
    }
}

inline bool view_ok(const View& v) {
    return v.p != nullptr && aligned16(v.p) && ((v.sb | v.sh | v.sn) & 7) == 0;
}

// every host-side check of a launch; nothing is enqueued before it passes
inline int validate(const Params& p, int B, int D) {
    if (B <= 0 || p.H <= 0 || p.N <= 0) return VQA_ERR_BAD_SHAPE;
    if ((int64_t)B * p.H > 65535) return VQA_ERR_BAD_ARGUMENT;
    if (p.window < 0 || !(p.scale_log2e > 0.f)) return VQA_ERR_BAD_ARGUMENT;
    if (D != 32 && D != 64 && D != 128) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    if (!view_ok(p.qa) || !view_ok(p.qb) || !view_ok(p.ka) || !view_ok(p.kb) || !view_ok(p.kc) || !view_ok(p.v))
        return (p.qa.p && p.qb.p && p.ka.p && p.kb.p && p.kc.p && p.v.p) ? VQA_ERR_MISALIGNED : VQA_ERR_NULL_POINTER;
    if (!row_stride_ok(p.qa.sn) || !row_stride_ok(p.qb.sn) || !row_stride_ok(p.ka.sn) || !row_stride_ok(p.kb.sn) ||
        !row_stride_ok(p.kc.sn) || !row_stride_ok(p.v.sn))
        return VQA_ERR_BAD_ARGUMENT;
    if (!p.out) return VQA_ERR_NULL_POINTER;
    if (((uintptr_t)p.out & 7) || ((p.o_sb | p.o_sh | p.o_sn) & 3)) return VQA_ERR_MISALIGNED;
    return VQA_OK;
}

// head dim 32: the window modes and the full ReRoPE mode (the reference's kernels of these kinds accept it,
// ops/triton_fused_attn_rerope.py:192, ops/triton_fused_vq_attn.py:198-199); the additive-code prefill does not
template <typename Tag>
int dispatch_mode_d32(const Params& p, int B, int mode, hipStream_t stream) {
    switch (mode) {
        case kLocalStrict: return launch<Tag, 32, kLocalStrict>(p, B, stream);
        case kLocalLoose: return launch<Tag, 32, kLocalLoose>(p, B, stream);
        case kLocalRerope: return launch<Tag, 32, kLocalRerope>(p, B, stream);
        case kFullRerope: return launch<Tag, 32, kFullRerope>(p, B, stream);
        default: return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    }
}

template <typename Tag>
int run(Params p, int B, int D, int mode, hipStream_t stream) {
    const int rc = validate(p, B, D);
    if (rc != VQA_OK) return rc;
    if (D == 32) return dispatch_mode_d32<Tag>(p, B, mode, stream);
    if (D == 64) return dispatch_mode<Tag, 64>(p, B, mode, stream);
    if (D == 128) return dispatch_mode<Tag, 128>(p, B, mode, stream);
    return VQA_ERR_UNSUPPORTED_HEAD_DIM;
}

inline View make_view(const void* ptr, const int64_t* s) {
    return View{static_cast<const uint16_t*>(ptr), s[0], s[1], s[2]};
}

// strides: 6 tensors x (b, h, n): q1, q2, k1, k2, v, out
// the software-pipelined kernel for the long-prefill configuration (vqa_prefill_pipe.hip)
constexpr int kPipeMinTokens = 2048;  // shorter sequences stay on the tiled schedule
bool prefill_pipe_applies(int window, int boundary_is_block, bool has_exact, bool has_second_pair);
template <typename Tag>
int prefill_pipe_run(const View& q, const View& ka, const View& kc, const View& v, uint16_t* out, int64_t o_sb,
                     int64_t o_sh, int64_t o_sn, float* lse, int B, int H, int N, int D, int window, int causal,
                     bool all_far, float scale_log2e, hipStream_t stream);
// causal full-context ReRoPE on the same 256-row kernel (window a multiple of 64)
bool rerope_full_pipe_applies(int window, int N, int causal);
template <typename Tag>
int rerope_full_pipe_run(const View& q1, const View& q2, const View& k1, const View& k2, const View& v, uint16_t* out,
                         int64_t o_sb, int64_t o_sh, int64_t o_sn, float* lse, int B, int H, int N, int D, int window,
                         float scale_log2e, hipStream_t stream);
// the same core for the sliding-window modes (window_rule = Mode 0 / 1 / 2) with a window that is a multiple of 128
bool window_pipe_applies(int window, int N);
template <typename Tag>
int window_pipe_run(const View& q1, const View& q2, const View& k1, const View& k2, const View& v, uint16_t* out,
                    int64_t o_sb, int64_t o_sh, int64_t o_sn, float* lse, int B, int H, int N, int D, int window,
                    int window_rule, float scale_log2e, hipStream_t stream);

template <typename Tag>
int local_attn(const void* q1, const void* q2, const void* k1, const void* k2, const void* v, void* out, float* lse,
               int B, int H, int N, int D, const int64_t* strides, int window, int mode, int causal, float sm_scale,
               hipStream_t stream) {
    if (!strides || !q1 || !k1 || !v || !out) return VQA_ERR_NULL_POINTER;
    if (mode < kLocalStrict || mode > kFullRerope) return VQA_ERR_BAD_ARGUMENT;
    const bool dual = (mode == kLocalRerope || mode == kFullRerope);
    if (dual && (!q2 || !k2)) return VQA_ERR_NULL_POINTER;
    Params p;
    p.qa = make_view(q1, strides);
    p.qb = dual ? make_view(q2, strides + 3) : p.qa;
    p.ka = make_view(k1, strides + 6);
    p.kb = dual ? make_view(k2, strides + 9) : p.ka;
    p.kc = p.ka;
    p.v = make_view(v, strides + 12);
    p.out = static_cast<uint16_t*>(out);
    p.o_sb = strides[15], p.o_sh = strides[16], p.o_sn = strides[17];
    p.lse = lse;
    p.H = H, p.N = N, p.window = window;
    p.causal = causal;
    p.boundary = kBoundaryBlock;
    p.has_b = 1;
    p.scale_log2e = sm_scale * kLog2e;
    // A window that covers the whole sequence is plain causal attention: where the pipelined schedule is the faster
    // one (same rule as in prefill() below) it runs that, every key tile an exact one.
    if ((mode == kLocalStrict || mode == kLocalLoose) && window >= N && (D == 64 || D == 128) && N >= kPipeMinTokens) {
        const int rc = validate(p, B, D);
        if (rc != VQA_OK) return rc;
        const int cover = (N + kTile - 1) / kTile * kTile;  // a multiple of 128 that is >= N
        return prefill_pipe_run<Tag>(p.qa, p.ka, p.ka, p.v, p.out, p.o_sb, p.o_sh, p.o_sn, p.lse, B, H, N, D, cover, 1,
                                     false, p.scale_log2e, stream);
    }
    // Sliding windows: the pipelined core (vqa_prefill_pipe.hip: 128-row query tiles, two workgroups per CU, every
    // workgroup walking several query tiles) where it is the faster one.  Measured against the tiled kernel over
    // batch x heads 4 - 128, 2k - 32k tokens, head dims 64 and 128, the three window modes: 0.73 - 0.97 of its time
    // from W = 512 on (0.84 - 0.88 at W = 512, 16k tokens, 64 heads; 0.78 - 0.81 at W = 2048), level at W = 128 and on
    // grids of under a thousand query tiles.  The window must be a multiple of 128 and the length one of 64.
    if (mode <= kLocalRerope && window_pipe_applies(window, N) && (D == 64 || D == 128) && window >= 512 &&
        (int64_t)((N + 127) / 128) * B * H >= 1024) {
        const int rc = validate(p, B, D);
        if (rc != VQA_OK) return rc;
        return window_pipe_run<Tag>(p.qa, p.qb, p.ka, p.kb, p.v, p.out, p.o_sb, p.o_sh, p.o_sn, p.lse, B, H, N, D,
                                    window, mode, p.scale_log2e, stream);
    }
    // Causal full-context ReRoPE on long sequences: the 256-row pipelined kernel (same rule as the VQ prefill).
    if (mode == kFullRerope && rerope_full_pipe_applies(window, N, causal) && (D == 64 || D == 128) &&
        N >= kPipeMinTokens) {
        const int rc = validate(p, B, D);
        if (rc != VQA_OK) return rc;
        return rerope_full_pipe_run<Tag>(p.qa, p.qb, p.ka, p.kb, p.v, p.out, p.o_sb, p.o_sh, p.o_sn, p.lse, B, H, N, D,
                                         window, p.scale_log2e, stream);
    }
    return run<Tag>(p, B, D, mode, stream);
}

// ---------------------------------------------------------------------------------------------------------------
// Far-context keys: kc[b,h,j,:] = sum_m codebooks[h, m, codes[b,h,j,m], :], summed in fp32, rounded once, for the keys
// j < n_keys (the keys some query scores as far keys; the attention kernels read no others from kc).
// One thread per (key, 8-element chunk) and kKeysPerThread keys 16 rows apart; the codebooks of a head (M*K*D elements)
// stay L2-resident.  The kernel is bound by the latency of the chain code -> codeword row, so a thread first fetches
// the code words of all its keys (one 4- or 8-byte load per key when M is 4 or 8 and the rows are so aligned: `wide`)
// and then has kKeysPerThread
// independent gathers per codebook in flight.
// ---------------------------------------------------------------------------------------------------------------
template <typename Tag, int D>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ codes,
                                                      const uint16_t* __restrict__ cb, uint16_t* __restrict__ kc,
                                                      int H, int N, int n_keys, int M, int K, int wide,
                                                      int64_t c_sb, int64_t c_sh, int64_t cb_sh, int64_t cb_sm,
                                                      int64_t cb_sk) {
    constexpr int CPR = D / 8;
    constexpr int KPT = 4;                 // keys per thread
    constexpr int kRows = 256 / CPR;       // keys one pass of the workgroup covers
    const int bh = blockIdx.y;
    const int b = bh / H, h = bh % H;
    const int col = threadIdx.x % CPR;
    const int j0 = blockIdx.x * (kRows * KPT) + threadIdx.x / CPR;
    if (j0 >= n_keys) return;
    const uint8_t* code = codes + b * c_sb + h * c_sh;
    const uint16_t* cbh = cb + h * cb_sh + col * 8;
    float acc[KPT][8];
#pragma unroll
    for (int k = 0; k < KPT; ++k)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[k][e] = 0.f;
    auto add_rows = [&](int m0, int m_count, const uint32_t (&cw)[KPT][2]) __attribute__((always_inline)) {
#pragma unroll
        for (int mm = 0; mm < 8; ++mm) {
            if (mm >= m_count) break;
            u32x4_t w[KPT];
#pragma unroll
            for (int k = 0; k < KPT; ++k) {
                const int c = min((int)((cw[k][mm / 4] >> (8 * (mm % 4))) & 0xffu), K - 1);  // a code >= K reads codeword K - 1
                w[k] = *reinterpret_cast<const u32x4_t*>(cbh + (m0 + mm) * cb_sm + (int64_t)c * cb_sk);
            }
#pragma unroll
            for (int k = 0; k < KPT; ++k)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc[k][2 * e] += Elem<Tag>::from_bits((uint16_t)(w[k][e] & 0xffffu));
                    acc[k][2 * e + 1] += Elem<Tag>::from_bits((uint16_t)(w[k][e] >> 16));
                }
        }
    };
    // code words of the thread's keys, 8 codebooks at a time
    for (int m0 = 0; m0 < M; m0 += 8) {
        const int m_count = min(8, M - m0);
        uint32_t cw[KPT][2];
#pragma unroll
        for (int k = 0; k < KPT; ++k) {
            const int j = min(j0 + k * kRows, n_keys - 1);
            const uint8_t* cj = code + (int64_t)j * M + m0;
            if (wide && M == 4) {
                cw[k][0] = *reinterpret_cast<const uint32_t*>(cj);
                cw[k][1] = 0;
            } else if (wide && M == 8) {
                const uint2 t = *reinterpret_cast<const uint2*>(cj);
                cw[k][0] = t.x, cw[k][1] = t.y;
            } else {
                cw[k][0] = cw[k][1] = 0;
                for (int mm = 0; mm < m_count; ++mm) cw[k][mm / 4] |= (uint32_t)cj[mm] << (8 * (mm % 4));
            }
        }
        add_rows(m0, m_count, cw);
    }
#pragma unroll
    for (int k = 0; k < KPT; ++k) {
        const int j = j0 + k * kRows;
        if (j >= n_keys) break;
        u32x4_t o;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            o[e] = (uint32_t)Elem<Tag>::to_bits(acc[k][2 * e]) | ((uint32_t)Elem<Tag>::to_bits(acc[k][2 * e + 1]) << 16);
        // whole 256-byte rows leave the wave at once: the streaming store spares the read-for-ownership of the lines
        store_stream16(kc + ((int64_t)bh * N + j) * D + col * 8, make_uint4(o[0], o[1], o[2], o[3]));
    }
}

// Keys that some query scores as far keys: j < boundary(N - 1), rounded up to the 128-key block the attention kernels'
// tiles are aligned to.
inline int far_key_count(int N, int window, int boundary_mode, bool has_exact) {
    if (!has_exact) return N;
    const int last = N - 1 - window;
    if (last <= 0) return 0;
    const int nf = boundary_mode == kBoundaryBlock ? last / kTile * kTile : last;
    return min(N, (nf + kTile - 1) / kTile * kTile);
}

inline size_t prefill_workspace_bytes(int B, int H, int N, int D) {
    return ((size_t)B * H * N * D * 2 + 255) / 256 * 256;
}

enum Schedule : int { kScheduleAuto = 0, kScheduleTiled = 1, kSchedulePipelined = 2 };

// strides: q(b,h,n) codes(b,h) codebooks(h,m,k) v(b,h,n) k_exact(b,h,n) q2(b,h,n) k2(b,h,n) out(b,h,n)
template <typename Tag>
int prefill(const void* q, const uint8_t* codes, const void* codebooks, const void* v, const void* k_exact,
            const void* q2, const void* k2, void* out, float* lse, void* workspace, size_t workspace_bytes, int B,
            int H, int N, int D, int M, int K, const int64_t* strides, int window, int boundary_mode, int causal,
            float sm_scale, int schedule, hipStream_t stream) {
    if (!q || !codes || !codebooks || !v || !out || !workspace || !strides) return VQA_ERR_NULL_POINTER;
    const bool pipe_ok = prefill_pipe_applies(window, boundary_mode == kBoundaryBlock, k_exact != nullptr,
                                              k_exact && q2 && k2);
    if (schedule == kSchedulePipelined && !pipe_ok) return VQA_ERR_BAD_ARGUMENT;
    // Measured over batch x heads from 1 to 256, 1k - 32k tokens, head dims 64 and 128: the pipelined schedule
    // (256-row query tiles, one workgroup per CU) is the faster one from 2048 tokens on (0.69 - 0.96 of the tiled
    // kernel's time, the more the longer the sequence); at 1024 tokens its longer prologue makes it level or slower.
    const bool pipelined = schedule == kSchedulePipelined || (schedule == kScheduleAuto && pipe_ok && N >= kPipeMinTokens);
    if (B <= 0 || H <= 0 || N <= 0) return VQA_ERR_BAD_SHAPE;
    if (D != 64 && D != 128) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    if (M < 1 || M > 16 || K < 1 || K > 256) return VQA_ERR_UNSUPPORTED_CODEBOOK;
    if (boundary_mode != kBoundaryBlock && boundary_mode != kBoundaryExact) return VQA_ERR_BAD_ARGUMENT;
    if (!causal && k_exact) return VQA_ERR_BAD_ARGUMENT;
    if ((int64_t)B * H > 65535) return VQA_ERR_BAD_ARGUMENT;
    if (workspace_bytes < prefill_workspace_bytes(B, H, N, D)) return VQA_ERR_WORKSPACE_TOO_SMALL;
    const int64_t* s_q = strides;
    const int64_t* s_c = strides + 3;
    const int64_t* s_cb = strides + 5;
    const int64_t* s_v = strides + 8;
    const int64_t* s_ke = strides + 11;
    const int64_t* s_q2 = strides + 14;
    const int64_t* s_k2 = strides + 17;
    const int64_t* s_o = strides + 20;
    if (!aligned16(codebooks) || ((uintptr_t)workspace & 255u) || ((s_cb[0] | s_cb[1] | s_cb[2]) & 7))
        return VQA_ERR_MISALIGNED;

    uint16_t* kc = static_cast<uint16_t*>(workspace);
    Params p;
    p.qa = make_view(q, s_q);
    p.qb = q2 ? make_view(q2, s_q2) : p.qa;
    p.kc = View{kc, (int64_t)H * N * D, (int64_t)N * D, (int64_t)D};
    p.ka = k_exact ? make_view(k_exact, s_ke) : p.kc;
    p.has_b = (k_exact && q2 && k2) ? 1 : 0;
    p.kb = p.has_b ? make_view(k2, s_k2) : p.ka;
    p.v = make_view(v, s_v);
    p.out = static_cast<uint16_t*>(out);
    p.o_sb = s_o[0], p.o_sh = s_o[1], p.o_sn = s_o[2];
    p.lse = lse;
    p.H = H, p.N = N, p.window = window;
    p.causal = causal;
    p.boundary = k_exact ? boundary_mode : kBoundaryAllFar;
    p.scale_log2e = sm_scale * kLog2e;
    int rc = validate(p, B, D);
    if (rc != VQA_OK) return rc;

    // 4- and 8-byte code loads where every row of codes starts on such a boundary
    const int wide = ((M == 4 || M == 8) &&
                      !(((uintptr_t)codes | (uintptr_t)s_c[0] | (uintptr_t)s_c[1]) & (uintptr_t)(M - 1))) ? 1 : 0;
    const int n_far = far_key_count(N, window, boundary_mode, k_exact != nullptr);
    if (n_far > 0) {
        const int keys_per_wg = (256 / (D / 8)) * 4;  // kRows * KPT of dequant_kernel
        const dim3 dq_grid((n_far + keys_per_wg - 1) / keys_per_wg, B * H);
        if (D == 64)
            hipLaunchKernelGGL((dequant_kernel<Tag, 64>), dq_grid, dim3(256), 0, stream, codes,
                               static_cast<const uint16_t*>(codebooks), kc, H, N, n_far, M, K, wide, s_c[0], s_c[1],
                               s_cb[0], s_cb[1], s_cb[2]);
        else
            hipLaunchKernelGGL((dequant_kernel<Tag, 128>), dq_grid, dim3(256), 0, stream, codes,
                               static_cast<const uint16_t*>(codebooks), kc, H, N, n_far, M, K, wide, s_c[0], s_c[1],
                               s_cb[0], s_cb[1], s_cb[2]);
    }
    rc = launch_status();
    if (rc != VQA_OK) return rc;
    if (pipelined)
        return prefill_pipe_run<Tag>(p.qa, p.ka, p.kc, p.v, p.out, p.o_sb, p.o_sh, p.o_sn, p.lse, B, H, N, D, window,
                                     causal, k_exact == nullptr, p.scale_log2e, stream);
    return run<Tag>(p, B, D, kVqPrefill, stream);
}

}  // namespace flash
}  // namespace vqa

extern "C" {

int vqa_local_attn_bf16(const void* q1, const void* q2, const void* k1, const void* k2, const void* v, void* out,
                        float* lse, int B, int H, int N, int D, const int64_t* strides, int window, int mode,
                        float sm_scale, vqa_stream_t stream) {
    if (mode < 0 || mode > 2) return VQA_ERR_BAD_ARGUMENT;
    return vqa::flash::local_attn<vqa::bf16_tag>(q1, q2, k1, k2, v, out, lse, B, H, N, D, strides, window, mode, 1,
                                                 sm_scale, stream);
}

int vqa_local_attn_f16(const void* q1, const void* q2, const void* k1, const void* k2, const void* v, void* out,
                       float* lse, int B, int H, int N, int D, const int64_t* strides, int window, int mode,
                       float sm_scale, vqa_stream_t stream) {
    if (mode < 0 || mode > 2) return VQA_ERR_BAD_ARGUMENT;
    return vqa::flash::local_attn<vqa::f16_tag>(q1, q2, k1, k2, v, out, lse, B, H, N, D, strides, window, mode, 1,
                                                sm_scale, stream);
}

int vqa_rerope_full_bf16(const void* q1, const void* q2, const void* k1, const void* k2, const void* v, void* out,
                         float* lse, int B, int H, int N, int D, const int64_t* strides, int window, int causal,
                         float sm_scale, vqa_stream_t stream) {
    return vqa::flash::local_attn<vqa::bf16_tag>(q1, q2, k1, k2, v, out, lse, B, H, N, D, strides, window,
                                                 vqa::flash::kFullRerope, causal, sm_scale, stream);
}

int vqa_rerope_full_f16(const void* q1, const void* q2, const void* k1, const void* k2, const void* v, void* out,
                        float* lse, int B, int H, int N, int D, const int64_t* strides, int window, int causal,
                        float sm_scale, vqa_stream_t stream) {
    return vqa::flash::local_attn<vqa::f16_tag>(q1, q2, k1, k2, v, out, lse, B, H, N, D, strides, window,
                                                vqa::flash::kFullRerope, causal, sm_scale, stream);
}

size_t vqa_prefill_workspace_bytes(int B, int H, int N, int D) {
    if (B <= 0 || H <= 0 || N <= 0 || D <= 0) return 0;
    return vqa::flash::prefill_workspace_bytes(B, H, N, D);
}

int vqa_prefill_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, const void* k_exact,
                     const void* q2, const void* k2, void* out, float* lse, void* workspace, size_t workspace_bytes,
                     int B, int H, int N, int D, int M, int K, const int64_t* strides, int window, int boundary_mode,
                     int causal, float sm_scale, vqa_stream_t stream) {
    return vqa::flash::prefill<vqa::bf16_tag>(q, codes, codebooks, v, k_exact, q2, k2, out, lse, workspace,
                                              workspace_bytes, B, H, N, D, M, K, strides, window, boundary_mode,
                                              causal, sm_scale, vqa::flash::kScheduleAuto, stream);
}

int vqa_prefill_f16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, const void* k_exact,
                    const void* q2, const void* k2, void* out, float* lse, void* workspace, size_t workspace_bytes,
                    int B, int H, int N, int D, int M, int K, const int64_t* strides, int window, int boundary_mode,
                    int causal, float sm_scale, vqa_stream_t stream) {
    return vqa::flash::prefill<vqa::f16_tag>(q, codes, codebooks, v, k_exact, q2, k2, out, lse, workspace,
                                             workspace_bytes, B, H, N, D, M, K, strides, window, boundary_mode, causal,
                                             sm_scale, vqa::flash::kScheduleAuto, stream);
}

int vqa_prefill_tiled_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v,
                           const void* k_exact, const void* q2, const void* k2, void* out, float* lse, void* workspace,
                           size_t workspace_bytes, int B, int H, int N, int D, int M, int K, const int64_t* strides,
                           int window, int boundary_mode, int causal, float sm_scale, vqa_stream_t stream) {
    return vqa::flash::prefill<vqa::bf16_tag>(q, codes, codebooks, v, k_exact, q2, k2, out, lse, workspace,
                                              workspace_bytes, B, H, N, D, M, K, strides, window, boundary_mode,
                                              causal, sm_scale, vqa::flash::kScheduleTiled, stream);
}

int vqa_prefill_tiled_f16(const void* q, const uint8_t* codes, const void* codebooks, const void* v,
                          const void* k_exact, const void* q2, const void* k2, void* out, float* lse, void* workspace,
                          size_t workspace_bytes, int B, int H, int N, int D, int M, int K, const int64_t* strides,
                          int window, int boundary_mode, int causal, float sm_scale, vqa_stream_t stream) {
    return vqa::flash::prefill<vqa::f16_tag>(q, codes, codebooks, v, k_exact, q2, k2, out, lse, workspace,
                                             workspace_bytes, B, H, N, D, M, K, strides, window, boundary_mode, causal,
                                             sm_scale, vqa::flash::kScheduleTiled, stream);
}

int vqa_prefill_pipelined_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v,
                               const void* k_exact, void* out, float* lse, void* workspace, size_t workspace_bytes,
                               int B, int H, int N, int D, int M, int K, const int64_t* strides, int window, int causal,
                               float sm_scale, vqa_stream_t stream) {
    return vqa::flash::prefill<vqa::bf16_tag>(q, codes, codebooks, v, k_exact, nullptr, nullptr, out, lse, workspace,
                                              workspace_bytes, B, H, N, D, M, K, strides, window,
                                              vqa::flash::kBoundaryBlock, causal, sm_scale, vqa::flash::kSchedulePipelined, stream);
}

int vqa_prefill_pipelined_f16(const void* q, const uint8_t* codes, const void* codebooks, const void* v,
                              const void* k_exact, void* out, float* lse, void* workspace, size_t workspace_bytes,
                              int B, int H, int N, int D, int M, int K, const int64_t* strides, int window, int causal,
                              float sm_scale, vqa_stream_t stream) {
    return vqa::flash::prefill<vqa::f16_tag>(q, codes, codebooks, v, k_exact, nullptr, nullptr, out, lse, workspace,
                                             workspace_bytes, B, H, N, D, M, K, strides, window,
                                             vqa::flash::kBoundaryBlock, causal, sm_scale, vqa::flash::kSchedulePipelined, stream);
}

}  // extern "C"
