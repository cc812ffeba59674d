// Exact sliding-window / ReRoPE / VQ-far-context prefill attention (seqlen_q == seqlen_k), one kernel template.
//
// Every variant is "causal flash attention whose score for (query i, key j) comes from one of up to three operand
// pairs, chosen by integer predicates on (i, j)":
//     pair A = (qa, ka)   in-window keys, rotary at true positions
//     pair B = (qb, kb)   keys beyond the window scored with the position-clamped query (ReRoPE)
//     pair C = (qb, kc)   far keys replaced by their additive-quantiser reconstruction kc = sum_m codebook[m][code]
// Tiles whose 128 x 64 (query x key) block uses a single pair and needs no mask take a fast path (one K tile,
// prefetched a tile ahead); tiles on the diagonal, on the window edge or on the far-context boundary compute every
// pair they touch and select / mask per element.
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

    for (int pass = 0; pass < n_pass; ++pass) {
    const int t = pass == 0 ? t_first : slot;
    const int m0 = t * kBM;
    const int m1 = min(m0 + kBM - 1, p.N - 1);
    const int row0 = m0 + wave * 32;
    const int qi = row0 + nq;  // this lane's query and its row bounds
    const int qi_vis_lo = rules.vis_lo(qi);
    const int qi_far_bnd = Rules<MODE>::kIsVq ? rules.far_bnd(qi) : 0;
    if (pass) __syncthreads();  // the previous tile's last reads of the LDS buffers are done

    // One query fragment set lives in registers: pair A's or pair B's.  Tiles are visited far -> near, so the
    // operand in use changes O(1) times per workgroup; a change re-reads the wave's 32 rows (L2 hits).
    const uint16_t* qa_src = p.qa.p + b * p.qa.sb + h * p.qa.sh;
    const uint16_t* qb_src = p.qb.p + b * p.qb.sb + h * p.qb.sh;
    QFrag<Tag, D> q;
    int q_held = -1;
    auto hold_q = [&](int which) {  // which: 0 = qa, 1 = qb (workgroup-uniform)
        if (q_held != which) {
            load_q<Tag, D>(q, which == 0 ? qa_src : qb_src, which == 0 ? p.qa.sn : p.qb.sn, row0, p.N, lane);
            wait_tile_loads();  // settle the reload here so that later waits never have to cover it
            q_held = which;
        }
    };

    // key tiles this workgroup visits
    const int hi_key = rules.is_causal() ? min(p.N, m1 + 1) : p.N;
    const int u_hi = (hi_key + kBN - 1) / kBN;
    const int u_lo = max(0, rules.vis_lo(m0)) / kBN;
    // Sliding-window modes: neighbouring query tiles share most of their key tiles, and the workgroups of an XCD that
    // run at the same time are neighbours.  If each started at its own first key tile, a key tile would be read by
    // its (window / 128 + 1) users several steps apart, with megabytes of other tiles in between -- more than the L2
    // holds, so it would come from memory again for each of them.  Instead every workgroup walks its window in the
    // same rotated order, key tile index modulo the number of tiles in a window: at any step all of them are on
    // tiles of the same residue, so the users of one tile read it at about the same time.  (The online softmax does
    // not care about the order.)  The walk is [u0, u_hi) followed by [u_lo, u0).
    constexpr bool kRotate = (MODE == kLocalStrict || MODE == kLocalLoose || MODE == kLocalRerope);
    int u0 = u_lo;
    if (kRotate) {
        const int period = (rules.W + kBM + kBN - 1) / kBN;
        u0 = (u_lo + period - 1) / period * period;
        if (u0 >= u_hi) u0 = u_lo;
    }

    SoftmaxState<D> st;
    st.init();

    int buf = 0;  // buffer holding the tile about to be computed: K of its main pair, and V
    {
        const int src = classify<MODE>(rules, m0, m1, u0 * kBN).main;
        k_copy.load(s_k[0], k_ptr(src), k_stride(src), u0 * kBN, p.N);
        v_copy.load(s_v[0], v_src, p.v.sn, u0 * kBN, p.N);
    }

    // scores -> probabilities -> O update for the tile whose K / V sit in cur_k / cur_v
    auto attend_tile = [&](f32x16_t(&s)[2], const char* cur_v) {
        vec8 pf[2][2];
        softmax_update<Tag, D, false>(st, s, p.scale_log2e, pf, nullptr);
        pv_mma<Tag, D>(st.o, pf, cur_v, lane);
    };

    int u = u0;
    int seg_hi = u_hi;           // end of the ascending segment being walked
    bool wrapped = (u0 == u_lo);  // the second segment [u_lo, u0) is under way (or empty)
    while (true) {
        const TileClass tc = classify<MODE>(rules, m0, m1, u * kBN);
        // length of the run of tiles that use this same single pair with no mask (whole tiles, in range)
        int u_end = u;
        if (tc.fast) {
            u_end = u + 1;
            while (u_end < seg_hi) {
                const TileClass t2 = classify<MODE>(rules, m0, m1, u_end * kBN);
                if (!t2.fast || t2.main != tc.main) break;
                ++u_end;
            }
        }
        if (u_end - u >= 2) {
            // hot loop: tiles u .. u_end-2 (the run's last tile goes through the general path below, which also
            // knows how to fetch whatever follows the run)
            hold_q(kDual && tc.main != 0 ? 1 : 0);
            const uint16_t* run_k = k_ptr(tc.main);
            const int64_t run_sn = k_stride(tc.main);
            for (; u < u_end - 1; ++u) {
                wait_tile_loads();
                __syncthreads();  // tile u is complete in `buf`; every wave is done with the other buffer
                k_copy.load_full(s_k[buf ^ 1], run_k, run_sn, (u + 1) * kBN);
                v_copy.load_full(s_v[buf ^ 1], v_src, p.v.sn, (u + 1) * kBN);
                f32x16_t s[2];
                qk_mma<Tag, D>(s, q, s_k[buf], lane);
                attend_tile(s, s_v[buf]);
                buf ^= 1;
            }
        }

        // general tile: every pair it touches, per-element selection and masking
        const int n0 = u * kBN;
        const TileClass tg = classify<MODE>(rules, m0, m1, n0);
        const char* cur_k = s_k[buf];
        const char* nxt_k = s_k[buf ^ 1];
        wait_tile_loads();
        __syncthreads();
        f32x16_t s[2];
        auto extra_pair = [&](int src) {  // pair `src` is scored in this tile besides the main one
            if (MODE == kVqPrefill2 && src == 1) return false;
            if (MODE != kVqPrefill && MODE != kVqPrefill2 && src == 2) return false;
            return src != tg.main && ((tg.need >> src) & 1) != 0;
        };
        // the first extra pair's K tile is requested before the main product so that the product hides its latency
        int early = -1;
        if constexpr (kDual) {
            early = extra_pair(0) ? 0 : (extra_pair(1) ? 1 : (extra_pair(2) ? 2 : -1));
            if (early >= 0) k_copy.load(nxt_k, k_ptr(early), k_stride(early), n0, p.N);
        }
        hold_q(kDual && tg.main != 0 ? 1 : 0);
        qk_mma<Tag, D>(s, q, cur_k, lane);
        if constexpr (kDual) {
            // the other pairs, one K tile at a time through the (still free) K buffer of the next tile
            for (int src = 0; src < 3; ++src) {
                if (!extra_pair(src)) continue;
                if (src != early) k_copy.load(nxt_k, k_ptr(src), k_stride(src), n0, p.N);
                hold_q(src == 0 ? 0 : 1);
                wait_tile_loads();
                __syncthreads();
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    const f32x16_t s2 = qk_block<Tag, D>(q, nxt_k, kb, lane);
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int j = n0 + kb * 32 + key_of_reg(r, half);
                        if (rules.source(qi, j, qi_far_bnd) == src) s[kb][r] = s2[r];
                    }
                }
                __syncthreads();  // all waves have read this pair's K tile before the buffer is reused
            }
        }
        if (!tg.fast) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int j = n0 + kb * 32 + key_of_reg(r, half);
                    s[kb][r] = rules.visible(qi, j, qi_vis_lo) ? s[kb][r] : -INFINITY;
                }
        }
        const int u_next = (u + 1 < seg_hi) ? u + 1 : (wrapped ? -1 : u_lo);
        if (u_next >= 0) {
            const int src = classify<MODE>(rules, m0, m1, u_next * kBN).main;
            k_copy.load(nxt_k, k_ptr(src), k_stride(src), u_next * kBN, p.N);
            v_copy.load(s_v[buf ^ 1], v_src, p.v.sn, u_next * kBN, p.N);
        }
        attend_tile(s, s_v[buf]);
        buf ^= 1;
        if (u_next < 0) break;
        if (u_next != u + 1) {
            wrapped = true;
            seg_hi = u0;
        }
        u = u_next;
    }

    store_output<Tag, D>(st, p.out + b * p.o_sb + h * p.o_sh, p.o_sn,
                         p.lse ? p.lse + (int64_t)bh * p.N : nullptr, row0, p.N, lane);
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
    if (D != 64 && D != 128) return VQA_ERR_UNSUPPORTED_HEAD_DIM;
    if (!view_ok(p.qa) || !view_ok(p.qb) || !view_ok(p.ka) || !view_ok(p.kb) || !view_ok(p.kc) || !view_ok(p.v))
        return (p.qa.p && p.qb.p && p.ka.p && p.kb.p && p.kc.p && p.v.p) ? VQA_ERR_MISALIGNED : VQA_ERR_NULL_POINTER;
    if (!row_stride_ok(p.qa.sn) || !row_stride_ok(p.qb.sn) || !row_stride_ok(p.ka.sn) || !row_stride_ok(p.kb.sn) ||
        !row_stride_ok(p.kc.sn) || !row_stride_ok(p.v.sn))
        return VQA_ERR_BAD_ARGUMENT;
    if (!p.out) return VQA_ERR_NULL_POINTER;
    if (((uintptr_t)p.out & 7) || ((p.o_sb | p.o_sh | p.o_sn) & 3)) return VQA_ERR_MISALIGNED;
    return VQA_OK;
}

template <typename Tag>
int run(Params p, int B, int D, int mode, hipStream_t stream) {
    const int rc = validate(p, B, D);
    if (rc != VQA_OK) return rc;
    if (D == 64) return dispatch_mode<Tag, 64>(p, B, mode, stream);
    if (D == 128) return dispatch_mode<Tag, 128>(p, B, mode, stream);
    return VQA_ERR_UNSUPPORTED_HEAD_DIM;
}

inline View make_view(const void* ptr, const int64_t* s) {
    return View{static_cast<const uint16_t*>(ptr), s[0], s[1], s[2]};
}

// strides: 6 tensors x (b, h, n): q1, q2, k1, k2, v, out
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
    return run<Tag>(p, B, D, mode, stream);
}

// ---------------------------------------------------------------------------------------------------------------
// Far-context keys: kc[b,h,j,:] = sum_m codebooks[h, m, codes[b,h,j,m], :], summed in fp32, rounded once.
// One thread per (key, 8-element chunk); the codebooks of a head (M*K*D elements) stay L2-resident.
// ---------------------------------------------------------------------------------------------------------------
template <typename Tag, int D>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ codes,
                                                      const uint16_t* __restrict__ cb, uint16_t* __restrict__ kc,
                                                      int H, int N, int M, int K, int64_t c_sb, int64_t c_sh,
                                                      int64_t cb_sh, int64_t cb_sm, int64_t cb_sk) {
    constexpr int CPR = D / 8;
    constexpr int KPT = 4;  // keys per thread: their gathers are independent and overlap
    const int bh = blockIdx.y;
    const int b = bh / H, h = bh % H;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    const int j0 = (idx / CPR) * KPT, col = idx % CPR;
    if (j0 >= N) return;
    const uint8_t* code = codes + b * c_sb + h * c_sh;
    const uint16_t* cbh = cb + h * cb_sh + col * 8;
    float acc[KPT][8];
#pragma unroll
    for (int k = 0; k < KPT; ++k)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[k][e] = 0.f;
    for (int m = 0; m < M; ++m) {
        u32x4_t w[KPT];
#pragma unroll
        for (int k = 0; k < KPT; ++k) {
            const int j = min(j0 + k, N - 1);
            const int c = min((int)code[(int64_t)j * M + m], K - 1);  // a code >= K reads codeword K - 1
            w[k] = *reinterpret_cast<const u32x4_t*>(cbh + m * cb_sm + (int64_t)c * cb_sk);
        }
#pragma unroll
        for (int k = 0; k < KPT; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc[k][2 * e] += Elem<Tag>::from_bits((uint16_t)(w[k][e] & 0xffffu));
                acc[k][2 * e + 1] += Elem<Tag>::from_bits((uint16_t)(w[k][e] >> 16));
            }
    }
#pragma unroll
    for (int k = 0; k < KPT; ++k) {
        if (j0 + k >= N) break;
        u32x4_t o;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            o[e] = (uint32_t)Elem<Tag>::to_bits(acc[k][2 * e]) | ((uint32_t)Elem<Tag>::to_bits(acc[k][2 * e + 1]) << 16);
        *reinterpret_cast<u32x4_t*>(kc + ((int64_t)bh * N + j0 + k) * D + col * 8) = o;
    }
}

// the software-pipelined kernel for the long-prefill configuration (vqa_prefill_pipe.hip)
bool prefill_pipe_applies(int window, int boundary_is_block, bool has_exact, bool has_second_pair);
template <typename Tag>
int prefill_pipe_run(const View& q, const View& ka, const View& kc, const View& v, uint16_t* out, int64_t o_sb,
                     int64_t o_sh, int64_t o_sn, float* lse, int B, int H, int N, int D, int window, int causal,
                     bool all_far, float scale_log2e, hipStream_t stream);

inline size_t prefill_workspace_bytes(int B, int H, int N, int D) {
    return ((size_t)B * H * N * D * 2 + 255) / 256 * 256;
}

// strides: q(b,h,n) codes(b,h) codebooks(h,m,k) v(b,h,n) k_exact(b,h,n) q2(b,h,n) k2(b,h,n) out(b,h,n)
template <typename Tag>
int prefill(const void* q, const uint8_t* codes, const void* codebooks, const void* v, const void* k_exact,
            const void* q2, const void* k2, void* out, float* lse, void* workspace, size_t workspace_bytes, int B,
            int H, int N, int D, int M, int K, const int64_t* strides, int window, int boundary_mode, int causal,
            float sm_scale, bool pipelined, hipStream_t stream) {
    if (!q || !codes || !codebooks || !v || !out || !workspace || !strides) return VQA_ERR_NULL_POINTER;
    if (pipelined && !prefill_pipe_applies(window, boundary_mode == kBoundaryBlock, k_exact != nullptr,
                                           k_exact && q2 && k2))
        return VQA_ERR_BAD_ARGUMENT;
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

    const int chunks = ((N + 3) / 4) * (D / 8);  // one thread per 16-byte column of 4 consecutive keys
    const dim3 dq_grid((chunks + 255) / 256, B * H);
    if (D == 64)
        hipLaunchKernelGGL((dequant_kernel<Tag, 64>), dq_grid, dim3(256), 0, stream, codes,
                           static_cast<const uint16_t*>(codebooks), kc, H, N, M, K, s_c[0], s_c[1], s_cb[0], s_cb[1],
                           s_cb[2]);
    else
        hipLaunchKernelGGL((dequant_kernel<Tag, 128>), dq_grid, dim3(256), 0, stream, codes,
                           static_cast<const uint16_t*>(codebooks), kc, H, N, M, K, s_c[0], s_c[1], s_cb[0], s_cb[1],
                           s_cb[2]);
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
                                              causal, sm_scale, false, stream);
}

int vqa_prefill_f16(const void* q, const uint8_t* codes, const void* codebooks, const void* v, const void* k_exact,
                    const void* q2, const void* k2, void* out, float* lse, void* workspace, size_t workspace_bytes,
                    int B, int H, int N, int D, int M, int K, const int64_t* strides, int window, int boundary_mode,
                    int causal, float sm_scale, vqa_stream_t stream) {
    return vqa::flash::prefill<vqa::f16_tag>(q, codes, codebooks, v, k_exact, q2, k2, out, lse, workspace,
                                             workspace_bytes, B, H, N, D, M, K, strides, window, boundary_mode, causal,
                                             sm_scale, false, stream);
}

int vqa_prefill_pipelined_bf16(const void* q, const uint8_t* codes, const void* codebooks, const void* v,
                               const void* k_exact, void* out, float* lse, void* workspace, size_t workspace_bytes,
                               int B, int H, int N, int D, int M, int K, const int64_t* strides, int window, int causal,
                               float sm_scale, vqa_stream_t stream) {
    return vqa::flash::prefill<vqa::bf16_tag>(q, codes, codebooks, v, k_exact, nullptr, nullptr, out, lse, workspace,
                                              workspace_bytes, B, H, N, D, M, K, strides, window,
                                              vqa::flash::kBoundaryBlock, causal, sm_scale, true, stream);
}

int vqa_prefill_pipelined_f16(const void* q, const uint8_t* codes, const void* codebooks, const void* v,
                              const void* k_exact, void* out, float* lse, void* workspace, size_t workspace_bytes,
                              int B, int H, int N, int D, int M, int K, const int64_t* strides, int window, int causal,
                              float sm_scale, vqa_stream_t stream) {
    return vqa::flash::prefill<vqa::f16_tag>(q, codes, codebooks, v, k_exact, nullptr, nullptr, out, lse, workspace,
                                             workspace_bytes, B, H, N, D, M, K, strides, window,
                                             vqa::flash::kBoundaryBlock, causal, sm_scale, true, stream);
}

}  // extern "C"
