// Long sequences on the software-pipelined core (vqa_flash2.h), three kinds of causal attention (Kind):
//
//   kVq      VQ prefill: far keys (j < boundary(i)) are scored against the reconstructed keys K_hat, recent keys against
//            the exact keys, both with the same query tensor, boundary(i) = max(0, floor((i - W) / 128) * 128) with W a
//            multiple of 128 -- the configuration of the reference's long prefill (ops/attn_vq.py:311, window lengths
//            are multiples of its 128 block) -- or every key far (no exact keys).  prefill_pipe_kernel.
//   kWindow  sliding window with one operand pair: keys j <= i with j >= i - W (strict) or j >= floor(i/128)*128 - W
//            (the reference's block rule, ops/triton_fused_local_attn2.py), W a multiple of 128.  window_pipe_kernel.
//   kRerope  the block-rule window with the ReRoPE pair rule (ops/triton_fused_local_attn_rerope.py:38-78): score
//            q1.k1 where i - j <= W, else q2.k2.  window_pipe_kernel.
//
// Everything else (a second query / key pair next to quantised keys, the exact boundary rule, other window lengths)
// stays with the general kernel in vqa_window.hip.
//
// What makes these cases simple: a wave's 64 query rows lie inside one 128-row block, so they share one boundary and,
// with 64-key tiles, every (wave, tile) block uses ONE key source -- but for the one tile per wave that the ReRoPE
// window edge crosses, which gets a second product.  A workgroup's waves differ by a few 64-key steps, so for a few
// tiles per query tile the workgroup brings both K sources and each wave reads the one it needs; no per-element
// selection exists elsewhere, masks only on the causal diagonal, at the lower window edge and at the end of the
// sequence.  The tile schedule is plain arithmetic on (m0, W, N).
#include <algorithm>
#include <mutex>

#include "vqa_flash2.h"

namespace vqa {
namespace pipe {

using flash::Geom;
using flash::View;
using flash2::Scores;

constexpr int kBN = flash2::kBN;
constexpr int kBlock = 128;  // granularity of the far-context boundary and of the block-rule window

enum Kind : int { kVq = 0, kWindow = 1, kRerope = 2 };

struct Params {
    View q, q2, ka, kc, v;  // ka: exact keys / first pair (unused when all_far), kc: reconstructed keys / second pair
    uint16_t* out;
    int64_t o_sb, o_sh, o_sn;
    float* lse;  // [B,H,N] contiguous, nullable
    int H, N, window;
    int causal, all_far;  // kVq
    int strict;           // kWindow: j >= i - W instead of the block rule
    int pair_tiles;
    int tiles_per_wg;  // sliding-window kinds: query tiles one workgroup walks
    float scale_log2e;
};

// kVq: 4 waves = 256 query rows, one workgroup per CU (long key loops; the tile copies serve 256 rows).
// LDS: exact-K tiles [2] | reconstructed-K tiles [2] | V tiles [2]
constexpr int kBM = flash2::kBM;
template <int D>
constexpr size_t lds_bytes() {
    return (size_t)Geom<D>::kTileBytes * 6;
}

// KIND: kVq, or kRerope = causal full-context ReRoPE (ops/triton_fused_attn_rerope.py:114-167): every key j <= i is
// visible, scored q1.k1 where i - j < W and q2.k2 elsewhere.  To this kernel that is the VQ prefill with the second
// keys in the place of the reconstructed ones -- a long run of second-source tiles, then first-source tiles up to
// the diagonal -- plus what the sliding-window kernel does at a wave's window-edge tile: the wave scores its
// second-source tiles with the second query, and at the tile the edge crosses it loads the first query, gives the tile
// a second product and keeps the first query from there on.
template <typename Tag, int D, int KIND>
__global__ __launch_bounds__(flash2::kThreads, 1) void prefill_pipe_kernel(Params p) {
    static_assert(KIND == kVq || KIND == kRerope, "kinds of the 256-row kernel");
    typedef Geom<D> G;
    typedef flash2::Pipe<Tag, D> Pipe;
    typedef typename Pipe::KDma KDma;
    typedef typename Pipe::VDma VDma;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // tiles are named by their LDS byte address
    const uint32_t lds0 = flash::lds_addr_of(smem);
    auto s_ka = [&](int par) { return lds0 + (uint32_t)((par & 1) * G::kTileBytes); };
    auto s_kc = [&](int par) { return lds0 + (uint32_t)((2 + (par & 1)) * G::kTileBytes); };
    auto s_v = [&](int par) { return lds0 + (uint32_t)((4 + (par & 1)) * G::kTileBytes); };
    auto lds_ptr = [&](uint32_t addr) { return smem + (addr - lds0); };

    // every XCD (own L2) gets whole (batch, head) problems; late and early query tiles are paired per workgroup so
    // that causal work is balanced
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
    const int t_first = n_tiles - 1 - slot;
    const int n_pass = (p.pair_tiles && slot != t_first) ? 2 : 1;

    const uint16_t* ka = p.ka.p + b * p.ka.sb + h * p.ka.sh;
    const uint16_t* kc = p.kc.p + b * p.kc.sb + h * p.kc.sh;
    const uint16_t* v_src = p.v.p + b * p.v.sb + h * p.v.sh;
    const uint16_t* q_src = p.q.p + b * p.q.sb + h * p.q.sh;
    const uint16_t* q2_src = p.q2.p + b * p.q2.sb + h * p.q2.sh;

    // whole-tile copies that ride on the score MFMAs: per-lane offsets once per kernel (one set per row stride)
    KDma kd_a, kd_c;
    VDma vd;
    kd_a.init(wave, lane, p.ka.sn);
    kd_c.init(wave, lane, p.kc.sn);
    vd.init(wave, lane, p.v.sn);
    // any other tile copy (first tiles of a pass, tiles that run over the end of the sequence, the second K source of
    // a boundary tile): issued as a block
    auto copy_k = [&](uint32_t lds_tile, const uint16_t* base, int64_t sn, int n0) __attribute__((always_inline)) {
        flash::TileCopy<D, false> c;
        c.init(wave, flash2::opaque_lane(lane));
        c.load(lds_ptr(lds_tile), base, sn, n0, p.N);
    };
    auto copy_v = [&](uint32_t lds_tile, int n0) __attribute__((always_inline)) {
        flash::TileCopy<D, true> c;
        c.init(wave, flash2::opaque_lane(lane));
        c.load(lds_ptr(lds_tile), v_src, p.v.sn, n0, p.N);
    };

    for (int pass = 0; pass < n_pass; ++pass) {
    const int t = pass == 0 ? t_first : slot;
    const int m0 = t * kBM;
    const int m1 = min(m0 + kBM - 1, p.N - 1);
    const int row0 = m0 + wave * flash2::kWaveRows;  // this wave's 64 rows (inside one 128-row block)
    if (pass) __syncthreads();  // the previous query tile's last reads of the LDS buffers are done

    // kVq: first exact key of the two 128-row blocks of the workgroup, and of this wave's block.
    // kRerope: the second pair scores the keys j <= i - W, i.e. whole tiles below the wave's edge tile (the one at
    // row0 - W) and part of that tile: in the same three variables, the first tile that needs the first source at
    // all (the first wave's edge tile), the end of the last wave's edge tile, the end of this wave's edge tile.
    const int kNever = 0x7fffffff;
    const int edge_w = KIND == kRerope ? row0 - p.window : -1;
    const int fb_lo = p.all_far ? kNever : max(0, m0 - p.window);
    const int fb_hi = p.all_far ? kNever : max(0, m0 + (KIND == kRerope ? kBM : kBlock) - p.window);
    const int fb_w = KIND == kRerope ? max(0, edge_w + kBN) : ((wave < 2) ? fb_lo : fb_hi);
    // tiles [0, n_iter): keys up to the last row of the query tile (causal) or all of them
    const int hi_key = p.causal ? min(p.N, m1 + 1) : p.N;
    const int n_iter = (hi_key + kBN - 1) / kBN;
    const int n_whole = min(n_iter, p.N / kBN);  // tiles that lie inside the sequence with all 64 rows
    // K tiles a key tile needs (workgroup-uniform) and the buffer this wave scores from
    auto needs_far = [&](int u) { return u * kBN < fb_hi; };
    auto needs_exact = [&](int u) { return u * kBN >= fb_lo; };
    auto request_k = [&](int u, int par) __attribute__((always_inline)) {
        if (needs_far(u)) copy_k(s_kc(par), kc, p.kc.sn, u * kBN);
        if (needs_exact(u)) copy_k(s_ka(par), ka, p.ka.sn, u * kBN);
    };

    // the first tiles are requested before anything else of the pass: their latency covers the query loads
    request_k(0, 0);
    copy_v(s_v(0), 0);
    if (n_iter > 1) request_k(1, 1);

    flash2::Wave<Tag, D> w;
    w.init();
    {
        // kRerope: a wave that meets second-pair keys starts with the second query
        const bool second = KIND == kRerope && edge_w >= 0;
        const uint16_t* src = second ? q2_src : q_src;
        const int64_t sn_q = second ? p.q2.sn : p.q.sn;
        flash::load_q<Tag, D>(w.q[0], src, sn_q, row0, p.N, lane);
        flash::load_q<Tag, D>(w.q[1], src, sn_q, row0 + 32, p.N, lane);
        flash2::prescale_q<Tag, D>(w.q[0], p.scale_log2e);
        flash2::prescale_q<Tag, D>(w.q[1], p.scale_log2e);
    }

    Scores s_even, s_odd;
    typename Pipe::Frags kf, vf;
    float mx[2] = {-INFINITY, -INFINITY};

    // masks of tile u for this wave: causal diagonal and end of the sequence; a tile past the wave's last row (or
    // past the last tile) ends up fully masked
    auto mask_tile = [&](Scores& sn, int u) __attribute__((always_inline)) {
        const int n0 = u * kBN;
        const bool whole = (n0 + kBN <= p.N) && (!p.causal || n0 + kBN - 1 <= row0) && u < n_iter;
        if (whole) return;  // (wave-uniform)
        flash2::mfma_settle(sn);  // the scores below were produced by the last MFMAs
        const int lane_o = flash2::opaque_lane(lane);  // keeps the predicates inside this branch
        const int half = lane_o >> 5;
        const int j_hi = u < n_iter ? p.N : 0;  // no such tile: nothing visible
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            const int i = row0 + qb * 32 + (lane_o & 31);
            const int lim = p.causal ? min(j_hi, i + 1) : j_hi;  // keys j < lim are visible
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int j = n0 + kb * 32 + flash::key_of_reg(r, half);
                    sn.s[qb][kb][r] = j < lim ? sn.s[qb][kb][r] : -INFINITY;
                }
        }
    };
    auto k_tile_of_wave = [&](int u, int par) { return (u * kBN < fb_w) ? s_kc(par) : s_ka(par); };
    // after the scores of tile u: masks, and (kRerope) at the wave's edge tile the change-over to the first pair: the
    // scores so far are q2.k2, the keys with i - j < W take q1.k1, and q1 serves every later tile
    auto finish_scores = [&](Scores& sn, int u, int par) __attribute__((always_inline)) {
        mask_tile(sn, u);
        if constexpr (KIND == kRerope) {
            if (u * kBN == edge_w) {  // (wave-uniform; the tile lies below the diagonal: no mask touched it)
                flash::load_q<Tag, D>(w.q[0], q_src, p.q.sn, row0, p.N, lane);
                flash::load_q<Tag, D>(w.q[1], q_src, p.q.sn, row0 + 32, p.N, lane);
                flash2::prescale_q<Tag, D>(w.q[0], p.scale_log2e);
                flash2::prescale_q<Tag, D>(w.q[1], p.scale_log2e);
                const int lane_o = flash2::opaque_lane(lane);
                const int half = lane_o >> 5, n = lane_o & 31;
                Pipe::second_pair(w, sn, s_ka(par), lane, kf, [&](int qb, int kb, int r) {
                    // i - j < W  with  i = row0 + qb*32 + n,  j = edge_w + kb*32 + key:  qb*32 + n < kb*32 + key
                    return qb * 32 + n < kb * 32 + flash::key_of_reg(r, half);
                });
            }
        }
    };
    const typename Pipe::TileRequest no_req{nullptr, 0};

    // first tile: scores, masks, row maxima (nothing to overlap with yet)
    flash::wait_tile_loads();
    __syncthreads();
    Pipe::k_head(kf, k_tile_of_wave(0, 0), lane);
    Pipe::template score_phase<true, false, false, false>(w, s_even, kf, s_odd, vf, 0u, lane, kd_c, no_req, vd, no_req);
    finish_scores(s_even, 0, 0);
    Pipe::template pv_phase<false, true>(w, vf, s_odd, s_even, mx);

    // Row addresses of this wave's share of the tiles the main loop requests next: K tile u + 2, V tile u + 1.
    const int64_t kc_step = (int64_t)kBN * p.kc.sn * 2, ka_step = (int64_t)kBN * p.ka.sn * 2, v_step = (int64_t)kBN * p.v.sn * 2;
    const char* kc_rows = reinterpret_cast<const char*>(kc + (int64_t)(2 * kBN + wave * KDma::kRowsPerWave) * p.kc.sn);
    const char* ka_rows = reinterpret_cast<const char*>(ka + (int64_t)(2 * kBN + wave * KDma::kRowsPerWave) * p.ka.sn);
    const char* v_rows = reinterpret_cast<const char*>(v_src + (int64_t)(kBN + wave * VDma::kRowsPerWave) * p.v.sn);
    // Iteration u finishes tile u (exponentials, P.V) and prepares tile u + 1 (scores, masks, row maxima); K(u+1) and
    // V(u) were requested one iteration earlier and sit in the buffers of parity u + 1 and u.  It requests K(u+2) and
    // V(u+1): whole tiles ride on the score MFMAs (kRide), anything else goes out as a block in front of them.
    auto iteration = [&](auto u_is_odd, auto ride, int u) __attribute__((always_inline)) {
        constexpr int par = decltype(u_is_odd)::value ? 1 : 0;
        constexpr bool kRide = decltype(ride)::value;
        Scores& sc = par ? s_odd : s_even;
        Scores& sn = par ? s_even : s_odd;
        flash::wait_tile_loads();
        __syncthreads();  // K(u+1) and V(u) are complete; every wave is done with K(u) and V(u-1)
        Pipe::k_head(kf, k_tile_of_wave(u + 1, par + 1), lane);
        typename Pipe::TileRequest kr = no_req, vr = no_req;
        KDma kd = kd_c;
        if constexpr (kRide) {
            const int n2 = (u + 2) * kBN;
            const bool far = needs_far(u + 2);
            kr.rows = far ? kc_rows : ka_rows;
            kr.lds = KDma::lds_of_wave(far ? s_kc(par) : s_ka(par), wave);
#pragma unroll
            for (int i = 0; i < KDma::kInstr; ++i) kd.off[i] = far ? kd_c.off[i] : kd_a.off[i];
            vr.rows = v_rows;
            vr.lds = VDma::lds_of_wave(s_v(par + 1), wave);
            if (far && needs_exact(u + 2)) copy_k(s_ka(par), ka, p.ka.sn, n2);  // boundary tile: both sources
            kc_rows += kc_step, ka_rows += ka_step, v_rows += v_step;
        } else {
            if (u + 2 < n_iter) request_k(u + 2, par);
            if (u + 1 < n_iter) copy_v(s_v(par + 1), (u + 1) * kBN);
        }
        Pipe::update_max(w, mx, sc);
        Pipe::template score_phase<true, true, true, kRide>(w, sn, kf, sc, vf, s_v(par), lane, kd, kr, vd, vr);
        finish_scores(sn, u + 1, par + 1);
        mx[0] = mx[1] = -INFINITY;
        Pipe::template pv_phase<true, true>(w, vf, sc, sn, mx);
    };
    // main loop: pairs of iterations whose requests are whole tiles; then the last few, which may run over the end
    int u = 0;
    for (; u + 3 < n_whole; u += 2) {
        iteration(std::false_type{}, std::true_type{}, u);
        iteration(std::true_type{}, std::true_type{}, u + 1);
    }
    for (; u < n_iter; u += 2) {
        iteration(std::false_type{}, std::false_type{}, u);
        if (u + 1 < n_iter) iteration(std::true_type{}, std::false_type{}, u + 1);
    }

    // the output rows leave through LDS (every wave its own part of the tile buffers) once no wave reads tiles any more
    Pipe::settle_o(w);
    __syncthreads();
    static_assert((size_t)4 * Pipe::kStoreBytes <= lds_bytes<D>(), "staging area exceeds the tile buffers");
    Pipe::store(w, p.out + b * p.o_sb + h * p.o_sh, p.o_sn, p.lse ? p.lse + (int64_t)bh * p.N : nullptr, row0, p.N,
                lane, smem + wave * Pipe::kStoreBytes);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Sliding-window kinds (kWindow, kRerope): 128-row query tiles (2 waves), two workgroups per CU, and every workgroup
// walks several query tiles of one (batch, head).  A query tile meets only (W + 128) / 64 key tiles, so
// what surrounds its key loop weighs as much as the loop: a cold start (first tiles and queries from HBM), the
// drained software pipeline, the output rows, the launch of the next workgroup.  Walking a run removes the launches
// and lets the LAST iteration of a query tile -- which has no next key tile to score -- bring the first tiles and the
// queries of the next query tile instead, under its exponentials and its P.V product.
//
// Tile buffers: first-source K [2] | V [2] | (kRerope) second-source K [1].  Their parity is logical: a query tile may
// end on either one, the next starts on the free V buffer (`flip`).  The sequence length is a multiple of 64 (the
// host sends other lengths to the general kernel), so every tile copy is a whole tile.
// ---------------------------------------------------------------------------------------------------------------
template <int KIND>
constexpr size_t window_lds_bytes(int tile_bytes) {
    return (size_t)tile_bytes * (KIND == kRerope ? 5 : 4);
}

template <typename Tag, int D, int KIND>
__global__ __launch_bounds__(128, 1) void window_pipe_kernel(Params p) {
    static_assert(KIND == kWindow || KIND == kRerope, "sliding-window kinds only");
    typedef Geom<D> G;
    constexpr int NW = 2;
    constexpr int kBM = NW * flash2::kWaveRows;
    typedef flash2::Pipe<Tag, D, NW> Pipe;
    typedef typename Pipe::KDma KDma;
    typedef typename Pipe::VDma VDma;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lds0 = flash::lds_addr_of(smem);
    auto lds_ptr = [&](uint32_t addr) { return smem + (addr - lds0); };

    // every XCD (own L2) gets whole (batch, head) problems
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
    const int n_tiles = (p.N + kBM - 1) / kBM;
    // The workgroups of a (batch, head) take its query tiles in turn (workgroup s: tiles s, s + S, s + 2S, ...), so
    // the workgroups running at one time work on neighbouring query tiles and share their K / V tiles in the L2.
    // (Runs of ADJACENT tiles per workgroup were measured 1.2 x slower: every workgroup then streams a region of
    // its own and nothing is shared.)
    const int t_step = gridDim.x;
    const int t_begin = slot, t_end = n_tiles;
    if (t_begin >= t_end) return;  // (workgroup-uniform)

    const uint16_t* ka = p.ka.p + b * p.ka.sb + h * p.ka.sh;
    const uint16_t* kc = p.kc.p + b * p.kc.sb + h * p.kc.sh;
    const uint16_t* v_src = p.v.p + b * p.v.sb + h * p.v.sh;
    const uint16_t* q_src = p.q.p + b * p.q.sb + h * p.q.sh;
    const uint16_t* q2_src = p.q2.p + b * p.q2.sb + h * p.q2.sh;
    uint16_t* out = p.out + b * p.o_sb + h * p.o_sh;
    float* lse = p.lse ? p.lse + (int64_t)bh * p.N : nullptr;

    KDma kd_a;
    VDma vd;
    kd_a.init(wave, lane, p.ka.sn);
    vd.init(wave, lane, p.v.sn);
    const int64_t ka_step = (int64_t)kBN * p.ka.sn * 2, v_step = (int64_t)kBN * p.v.sn * 2;
    const int n_key_tiles = p.N / kBN;  // all whole
    auto copy_tile = [&](uint32_t lds_tile, const uint16_t* base, int64_t sn, int n0, auto is_v)
        __attribute__((always_inline)) {
        flash::TileCopy<D, decltype(is_v)::value, NW> c;
        c.init(wave, flash2::opaque_lane(lane));
        c.load_full(lds_ptr(lds_tile), base, sn, n0);
    };

    // geometry of one query tile for this wave
    struct Tile {
        int m0, row0, edge_w, lo_w, u0, n_iter;
    };
    auto tile_of = [&](int t) {
        Tile g;
        g.m0 = t * kBM;
        g.row0 = g.m0 + wave * flash2::kWaveRows;
        // kRerope: the second pair scores the keys j < i - W: whole tiles below edge_w, half of the tile at edge_w
        g.edge_w = KIND == kRerope ? g.row0 - p.window : -1;
        // lowest visible key of the wave's rows (of its first row for the strict rule)
        g.lo_w = p.strict ? g.row0 - p.window : (g.row0 / kBlock) * kBlock - p.window;
        g.u0 = max(0, g.m0 - p.window) / kBN;
        g.n_iter = (min(p.N, g.m0 + kBM) + kBN - 1) / kBN;
        return g;
    };
    Tile g = tile_of(t_begin);
    int flip = 0;  // physical buffer of logical parity 0
    auto s_ka = [&](int par) { return lds0 + (uint32_t)(((par ^ flip) & 1) * G::kTileBytes); };
    auto s_v = [&](int par) { return lds0 + (uint32_t)((2 + ((par ^ flip) & 1)) * G::kTileBytes); };
    const uint32_t s_kc = lds0 + 4u * G::kTileBytes;
    // second-source tiles: up to the last wave's edge tile
    auto needs_c = [&](const Tile& x, int u) { return KIND == kRerope && u * kBN <= x.m0 + (NW - 1) * flash2::kWaveRows - p.window; };
    auto wave_reads_c = [&](int u) { return KIND == kRerope && u * kBN <= g.edge_w; };
    auto k_tile_of_wave = [&](int u, int par) { return wave_reads_c(u) ? s_kc : s_ka(par); };
    // first tiles of a query tile (as a block): K(u0), V(u0), K(u0 + 1), and the second source of K(u0)
    auto request_first = [&](const Tile& x) __attribute__((always_inline)) {
        copy_tile(s_ka(0), ka, p.ka.sn, x.u0 * kBN, std::false_type{});
        copy_tile(s_v(0), v_src, p.v.sn, x.u0 * kBN, std::true_type{});
        if (x.u0 + 1 < x.n_iter) copy_tile(s_ka(1), ka, p.ka.sn, (x.u0 + 1) * kBN, std::false_type{});
        if (needs_c(x, x.u0)) copy_tile(s_kc, kc, p.kc.sn, x.u0 * kBN, std::false_type{});
    };
    // a wave that meets second-pair keys starts with the second query and changes over at its edge tile
    auto first_query_of = [&](const Tile& x, const uint16_t*& src, int64_t& sn_q) {
        const bool second = KIND == kRerope && x.edge_w >= 0;
        src = second ? q2_src : q_src;
        sn_q = second ? p.q2.sn : p.q.sn;
    };

    flash2::Wave<Tag, D> w;
    Scores s_even, s_odd;
    typename Pipe::Frags kf, vf;
    float mx[2];
    const typename Pipe::TileRequest no_req{nullptr, 0};

    request_first(g);
    {
        const uint16_t* src;
        int64_t sn_q;
        first_query_of(g, src, sn_q);
        flash::load_q<Tag, D>(w.q[0], src, sn_q, g.row0, p.N, lane);
        flash::load_q<Tag, D>(w.q[1], src, sn_q, g.row0 + 32, p.N, lane);
        flash2::prescale_q<Tag, D>(w.q[0], p.scale_log2e);
        flash2::prescale_q<Tag, D>(w.q[1], p.scale_log2e);
    }

    for (int t = t_begin; t < t_end; t += t_step) {
    w.init();
    mx[0] = mx[1] = -INFINITY;
    const int row0 = g.row0;

    // masks of tile u for this wave: causal diagonal, lower window edge, tiles past the wave's last row.  A tile that
    // lies wholly above the wave's rows, below its window (block rule: the edge is tile-aligned) or past the last
    // tile is cleared without a compare; on the diagonal one compare per element (the sequence length is a multiple
    // of the tile, so no key of a tile below n_iter lies past it); the strict rule adds its per-row lower edge.
    auto mask_tile = [&](Scores& sn, int u) __attribute__((always_inline)) {
        const int n0 = u * kBN;
        const int lo_last = g.lo_w + (p.strict ? flash2::kWaveRows - 1 : 0);  // of the wave's last row
        const bool whole = n0 + kBN - 1 <= row0 && u < g.n_iter && n0 >= lo_last;
        if (whole) return;  // (wave-uniform)
        flash2::mfma_settle(sn);  // the scores below were produced by the last MFMAs
        const bool none = u >= g.n_iter || n0 > row0 + flash2::kWaveRows - 1 || n0 + kBN - 1 < g.lo_w;
        if (none) {  // (wave-uniform)
#pragma unroll
            for (int qb = 0; qb < 2; ++qb)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) sn.s[qb][kb][r] = -INFINITY;
            return;
        }
        const int lane_o = flash2::opaque_lane(lane);  // keeps the predicates inside this branch
        const int half = lane_o >> 5;
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            const int i_rel = row0 - n0 + qb * 32 + (lane_o & 31);  // query row relative to the tile's first key
            const int lo_rel = p.strict ? i_rel - p.window : -1;    // keys lo_rel <= j - n0 <= i_rel are visible
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int j_rel = kb * 32 + flash::key_of_reg(r, half);
                    const bool vis = p.strict ? (j_rel <= i_rel && j_rel >= lo_rel) : j_rel <= i_rel;
                    sn.s[qb][kb][r] = vis ? sn.s[qb][kb][r] : -INFINITY;
                }
        }
    };
    // after the scores of tile u: masks, and at the wave's ReRoPE edge tile the change-over to the first pair (the
    // scores so far are q2.k2; keys with i - j <= W take q1.k1, and q1 serves every later tile)
    auto finish_scores = [&](Scores& sn, int u, int par) __attribute__((always_inline)) {
        mask_tile(sn, u);
        if constexpr (KIND == kRerope) {
            if (u * kBN == g.edge_w) {  // (wave-uniform; every key of this tile is visible to every row of the wave)
                flash::load_q<Tag, D>(w.q[0], q_src, p.q.sn, row0, p.N, lane);
                flash::load_q<Tag, D>(w.q[1], q_src, p.q.sn, row0 + 32, p.N, lane);
                flash2::prescale_q<Tag, D>(w.q[0], p.scale_log2e);
                flash2::prescale_q<Tag, D>(w.q[1], p.scale_log2e);
                const int lane_o = flash2::opaque_lane(lane);
                const int half = lane_o >> 5, n = lane_o & 31;
                Pipe::second_pair(w, sn, s_ka(par), lane, kf, [&](int qb, int kb, int r) {
                    // i - j <= W  with  i = row0 + qb*32 + n,  j = edge_w + kb*32 + key:  qb*32 + n <= kb*32 + key
                    return qb * 32 + n <= kb * 32 + flash::key_of_reg(r, half);
                });
            }
        }
    };

    // first tile: scores, masks, row maxima (nothing to overlap with yet)
    flash::wait_tile_loads();
    __syncthreads();
    Pipe::k_head(kf, k_tile_of_wave(g.u0, 0), lane);
    Pipe::template score_phase<true, false, false, false>(w, s_even, kf, s_odd, vf, 0u, lane, kd_a, no_req, vd, no_req);
    finish_scores(s_even, g.u0, 0);
    Pipe::template pv_phase<false, true>(w, vf, s_odd, s_even, mx);

    // rows of this wave's share of K tile u + 2 and V tile u + 1
    const int r2 = (g.u0 + 2) * kBN + wave * KDma::kRowsPerWave;
    const char* ka_rows = reinterpret_cast<const char*>(ka + (int64_t)r2 * p.ka.sn);
    const char* v_rows = reinterpret_cast<const char*>(v_src + (int64_t)(r2 - kBN) * p.v.sn);
    // Iteration u finishes tile u (exponentials, P.V) and prepares tile u + 1 (scores, masks, row maxima); K(u+1) and
    // V(u) were requested one iteration earlier and sit in the buffers of parity u + 1 and u.  It requests K(u+2) and
    // V(u+1), which ride on the score MFMAs.
    auto iteration = [&](auto u_is_odd, int u) __attribute__((always_inline)) {
        constexpr int par = decltype(u_is_odd)::value ? 1 : 0;
        Scores& sc = par ? s_odd : s_even;
        Scores& sn = par ? s_even : s_odd;
        flash::wait_tile_loads();
        __syncthreads();  // K(u+1) and V(u) are complete; every wave is done with K(u) and V(u-1)
        if constexpr (KIND == kRerope) {
            // the one second-source buffer is free now: the tile about to be scored is brought and waited for (once per
            // query tile; the other workgroup of the CU computes meanwhile)
            if (needs_c(g, u + 1)) {  // (workgroup-uniform)
                copy_tile(s_kc, kc, p.kc.sn, (u + 1) * kBN, std::false_type{});
                flash::wait_tile_loads();
                __syncthreads();
            }
        }
        Pipe::k_head(kf, k_tile_of_wave(u + 1, par + 1), lane);
        typename Pipe::TileRequest kr, vr;
        // K(u+2) may lie past the sequence for the last query tile: the copy then repeats the last tile into a buffer
        // nobody reads any more
        kr.rows = (u + 2 < n_key_tiles) ? ka_rows : ka_rows - ka_step;
        kr.lds = KDma::lds_of_wave(s_ka(par), wave);
        vr.rows = v_rows;
        vr.lds = VDma::lds_of_wave(s_v(par + 1), wave);
        ka_rows += ka_step, v_rows += v_step;
        Pipe::update_max(w, mx, sc);
        Pipe::template score_phase<true, true, true, true>(w, sn, kf, sc, vf, s_v(par), lane, kd_a, kr, vd, vr);
        finish_scores(sn, u + 1, par + 1);
        mx[0] = mx[1] = -INFINITY;
        Pipe::template pv_phase<true, true>(w, vf, sc, sn, mx);
    };
    // The last iteration finishes the last tile.  There is no next key tile; in its place the first tiles of the next
    // query tile are requested (both K buffers and the other V buffer are free) and its queries are loaded, and both
    // are on their way while the exponentials and the P.V product run and the output rows leave.
    const bool has_next = t + t_step < t_end;
    const Tile gn = tile_of(has_next ? t + t_step : t);
    // (one body: a query tile that ends on the odd buffer moves its last scores over first, 64 moves per query tile)
    auto last_iteration = [&](int par) __attribute__((always_inline)) {
        Scores& sc = s_even;
        Scores& sn = s_odd;  // (unused: no scores are produced)
        flash::wait_tile_loads();
        __syncthreads();  // V(u) is complete; every wave is done with K(u) and V(u-1)
        const uint32_t lds_v_now = s_v(par);
        if (has_next) {  // (the query fragments are free: this iteration scores nothing)
            flip ^= par ^ 1;  // logical parity 0 of the next query tile = the V buffer that is free now
            request_first(gn);
            const uint16_t* src;
            int64_t sn_q;
            first_query_of(gn, src, sn_q);
            flash::load_q<Tag, D>(w.q[0], src, sn_q, gn.row0, p.N, lane);
            flash::load_q<Tag, D>(w.q[1], src, sn_q, gn.row0 + 32, p.N, lane);
        }
        Pipe::update_max(w, mx, sc);
        Pipe::template score_phase<false, true, true, false>(w, sn, kf, sc, vf, lds_v_now, lane, kd_a, no_req, vd, no_req);
        Pipe::template pv_phase<true, false>(w, vf, sc, sn, mx);
        Pipe::settle_o(w);  // (here, not only in the store: nothing may touch O between the last MFMA and the wait)
    };
    int u = g.u0;
    for (; u + 2 < g.n_iter; u += 2) {
        iteration(std::false_type{}, u);
        iteration(std::true_type{}, u + 1);
    }
    int last_par = 0;
    if (u + 1 < g.n_iter) {
        iteration(std::false_type{}, u);
        s_even = s_odd;
        last_par = 1;
    }
    last_iteration(last_par);
    Pipe::store_direct(w, out, p.o_sn, lse, row0, p.N, lane);
    if (has_next) {
        flash2::prescale_q<Tag, D>(w.q[0], p.scale_log2e);
        flash2::prescale_q<Tag, D>(w.q[1], p.scale_log2e);
    }
    g = gn;
    }
}

template <typename Tag, int D, int KIND>
int launch(Params p, int B, hipStream_t stream) {
    // more than the 64 KB of LDS a launch gets by default: raised once per device and instantiation
    static std::mutex mu;
    static bool raised[kMaxDevices] = {};
    int dev = 0;
    const int rc = device_of_pointer(p.q.p, &dev);
    if (rc != VQA_OK) return rc;
    {
        std::lock_guard<std::mutex> lock(mu);
        if (!raised[dev]) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_pipe_kernel<Tag, D, KIND>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes<D>()) != hipSuccess) {
                (void)hipGetLastError();
                return VQA_ERR_LAUNCH_FAILED;
            }
            raised[dev] = true;
        }
    }
    const int n_tiles = (p.N + kBM - 1) / kBM;
    // causal work grows with the query tile: late and early tiles are paired once there are enough workgroups
    p.pair_tiles = (p.causal && (int64_t)(n_tiles / 2) * B * p.H >= 512) ? 1 : 0;
    const dim3 grid(p.pair_tiles ? (n_tiles + 1) / 2 : n_tiles, B * p.H);
    hipLaunchKernelGGL((prefill_pipe_kernel<Tag, D, KIND>), grid, dim3(flash2::kThreads), lds_bytes<D>(), stream, p);
    return launch_status();
}

template <typename Tag, int D, int KIND>
int launch_window(Params p, int B, hipStream_t stream) {
    constexpr size_t kLds = window_lds_bytes<KIND>(Geom<D>::kTileBytes);
    static std::mutex mu;
    static bool raised[kMaxDevices] = {};
    int dev = 0;
    const int rc = device_of_pointer(p.q.p, &dev);
    if (rc != VQA_OK) return rc;
    {
        std::lock_guard<std::mutex> lock(mu);
        if (!raised[dev]) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(&window_pipe_kernel<Tag, D, KIND>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLds) != hipSuccess) {
                (void)hipGetLastError();
                return VQA_ERR_LAUNCH_FAILED;
            }
            raised[dev] = true;
        }
    }
    // Query tiles per workgroup.  Short windows: one workgroup per place of the chip (256 CUs x 2), which walks all
    // its tiles -- no second launch round, every start but the first overlapped (W = 512 at 16k tokens: 524 us against
    // 538 with two rounds and 555 with four).  Long windows: two rounds, which balance better (W = 4096: 1 645 us
    // against 1 752).
    const int n_tiles = (p.N + 127) / 128;
    const int64_t total = (int64_t)n_tiles * B * p.H;
    const int64_t places = (p.window + 128) / kBN <= 20 ? 512 : 1024;
    p.tiles_per_wg = (int)std::max<int64_t>(1, std::min<int64_t>(32, total / places));
    const dim3 grid((n_tiles + p.tiles_per_wg - 1) / p.tiles_per_wg, B * p.H);
    hipLaunchKernelGGL((window_pipe_kernel<Tag, D, KIND>), grid, dim3(128), kLds, stream, p);
    return launch_status();
}

template <typename Tag, int KIND>
int launch_d(const Params& p, int B, int D, hipStream_t stream) {
    if constexpr (KIND == kVq) {
        if (D == 64) return launch<Tag, 64, kVq>(p, B, stream);
        if (D == 128) return launch<Tag, 128, kVq>(p, B, stream);
    } else {
        if (D == 64) return launch_window<Tag, 64, KIND>(p, B, stream);
        if (D == 128) return launch_window<Tag, 128, KIND>(p, B, stream);
    }
    return VQA_ERR_UNSUPPORTED_HEAD_DIM;
}

}  // namespace pipe

// entries used by vqa_prefill_* and vqa_local_attn_* (vqa_window.hip) once their arguments are validated (and K_hat
// is written)
namespace flash {

bool prefill_pipe_applies(int window, int boundary_is_block, bool has_exact, bool has_second_pair) {
    if (has_second_pair) return false;
    if (!has_exact) return true;
    return boundary_is_block && window % pipe::kBlock == 0;
}

// sliding-window kinds: window_rule 0 = strict (j >= i - W), 1 = block rule, 2 = block rule with the ReRoPE pair
bool window_pipe_applies(int window, int N) {
    return window > 0 && window % pipe::kBlock == 0 && window < N && N % pipe::kBN == 0;
}

template <typename Tag>
int prefill_pipe_run(const View& q, const View& ka, const View& kc, const View& v, uint16_t* out, int64_t o_sb,
                     int64_t o_sh, int64_t o_sn, float* lse, int B, int H, int N, int D, int window, int causal,
                     bool all_far, float scale_log2e, hipStream_t stream) {
    pipe::Params p;
    p.q = q, p.q2 = q, p.ka = ka, p.kc = kc, p.v = v;
    p.out = out;
    p.o_sb = o_sb, p.o_sh = o_sh, p.o_sn = o_sn;
    p.lse = lse;
    p.H = H, p.N = N, p.window = window;
    p.causal = causal;
    p.all_far = all_far ? 1 : 0;
    p.strict = 0;
    p.pair_tiles = 0;
    p.tiles_per_wg = 1;
    p.scale_log2e = scale_log2e;
    return pipe::launch_d<Tag, pipe::kVq>(p, B, D, stream);
}

template <typename Tag>
int window_pipe_run(const View& q1, const View& q2, const View& k1, const View& k2, const View& v, uint16_t* out,
                    int64_t o_sb, int64_t o_sh, int64_t o_sn, float* lse, int B, int H, int N, int D, int window,
                    int window_rule, float scale_log2e, hipStream_t stream) {
    pipe::Params p;
    p.q = q1, p.q2 = q2, p.ka = k1, p.kc = k2, p.v = v;
    p.out = out;
    p.o_sb = o_sb, p.o_sh = o_sh, p.o_sn = o_sn;
    p.lse = lse;
    p.H = H, p.N = N, p.window = window;
    p.causal = 1;
    p.all_far = 0;
    p.strict = window_rule == 0 ? 1 : 0;
    p.pair_tiles = 0;
    p.tiles_per_wg = 1;
    p.scale_log2e = scale_log2e;
    if (window_rule == 2) return pipe::launch_d<Tag, pipe::kRerope>(p, B, D, stream);
    return pipe::launch_d<Tag, pipe::kWindow>(p, B, D, stream);
}

// causal full-context ReRoPE on the 256-row kernel
bool rerope_full_pipe_applies(int window, int N, int causal) {
    return causal && window > 0 && window % pipe::kBN == 0 && window < N;
}

template <typename Tag>
int rerope_full_pipe_run(const View& q1, const View& q2, const View& k1, const View& k2, const View& v, uint16_t* out,
                         int64_t o_sb, int64_t o_sh, int64_t o_sn, float* lse, int B, int H, int N, int D, int window,
                         float scale_log2e, hipStream_t stream) {
    pipe::Params p;
    p.q = q1, p.q2 = q2, p.ka = k1, p.kc = k2, p.v = v;
    p.out = out;
    p.o_sb = o_sb, p.o_sh = o_sh, p.o_sn = o_sn;
    p.lse = lse;
    p.H = H, p.N = N, p.window = window;
    p.causal = 1;
    p.all_far = 0;
    p.strict = 0;
    p.pair_tiles = 0;
    p.tiles_per_wg = 1;
    p.scale_log2e = scale_log2e;
    if (D == 64) return pipe::launch<Tag, 64, pipe::kRerope>(p, B, stream);
    if (D == 128) return pipe::launch<Tag, 128, pipe::kRerope>(p, B, stream);
    return VQA_ERR_UNSUPPORTED_HEAD_DIM;
}

template int rerope_full_pipe_run<bf16_tag>(const View&, const View&, const View&, const View&, const View&, uint16_t*,
                                            int64_t, int64_t, int64_t, float*, int, int, int, int, int, float,
                                            hipStream_t);
template int rerope_full_pipe_run<f16_tag>(const View&, const View&, const View&, const View&, const View&, uint16_t*,
                                           int64_t, int64_t, int64_t, float*, int, int, int, int, int, float,
                                           hipStream_t);
template int prefill_pipe_run<bf16_tag>(const View&, const View&, const View&, const View&, uint16_t*, int64_t, int64_t,
                                        int64_t, float*, int, int, int, int, int, int, bool, float, hipStream_t);
template int prefill_pipe_run<f16_tag>(const View&, const View&, const View&, const View&, uint16_t*, int64_t, int64_t,
                                       int64_t, float*, int, int, int, int, int, int, bool, float, hipStream_t);
template int window_pipe_run<bf16_tag>(const View&, const View&, const View&, const View&, const View&, uint16_t*,
                                       int64_t, int64_t, int64_t, float*, int, int, int, int, int, int, float,
                                       hipStream_t);
template int window_pipe_run<f16_tag>(const View&, const View&, const View&, const View&, const View&, uint16_t*,
                                      int64_t, int64_t, int64_t, float*, int, int, int, int, int, int, float,
                                      hipStream_t);

}  // namespace flash
}  // namespace vqa
