// Long-context VQ prefill on the software-pipelined core (vqa_flash2.h): causal attention whose far keys
// (j < boundary(i)) are scored against the reconstructed keys K_hat and whose recent keys against the exact keys, both
// with the same query tensor, boundary(i) = max(0, floor((i - W) / 128) * 128) with W a multiple of 128 -- the
// configuration of the reference's long prefill (ops/attn_vq.py:311, window lengths are multiples of its 128 block) --
// or every key far (no exact keys).  Everything else (a second query / key pair for the strip between boundary and
// window, the exact boundary rule, other window lengths) stays with the general kernel in vqa_window.hip.
//
// What makes this case simple: a wave's 64 query rows lie inside one 128-row block, so they share one boundary and,
// with 64-key tiles, every (wave, tile) block uses ONE key source.  A workgroup's two 128-row blocks differ by one
// 128-key step, so for two tiles per query tile the workgroup brings both the exact and the reconstructed K tile and
// each wave reads the one it needs; no per-element selection exists, masks only on the causal diagonal and at the
// end of the sequence.  The tile schedule is plain arithmetic on (m0, W, N).
#include "vqa_flash2.h"

namespace vqa {
namespace pipe {

using flash::Geom;
using flash::View;
using flash2::Scores;

constexpr int kBM = flash2::kBM;
constexpr int kBN = flash2::kBN;
constexpr int kBlock = 128;  // granularity of the far-context boundary

struct Params {
    View q, ka, kc, v;  // ka: exact keys (unused when all_far), kc: reconstructed keys
    uint16_t* out;
    int64_t o_sb, o_sh, o_sn;
    float* lse;  // [B,H,N] contiguous, nullable
    int H, N, window;
    int causal, all_far;
    int pair_tiles;
    float scale_log2e;
};

// LDS: exact-K tiles [2] | reconstructed-K tiles [2] | V tiles [2]
template <int D>
constexpr size_t lds_bytes() {
    return (size_t)Geom<D>::kTileBytes * 6;
}

template <typename Tag, int D>
__global__ __launch_bounds__(flash2::kThreads, 1) void prefill_pipe_kernel(Params p) {
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

    // first exact key of the two 128-row blocks of the workgroup, and of this wave's block
    const int kNever = 0x7fffffff;
    const int fb_lo = p.all_far ? kNever : max(0, m0 - p.window);
    const int fb_hi = p.all_far ? kNever : max(0, m0 + kBlock - p.window);
    const int fb_w = (wave < 2) ? fb_lo : fb_hi;
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

    flash2::Wave<Tag, D> w;
    w.init();
    flash::load_q<Tag, D>(w.q[0], q_src, p.q.sn, row0, p.N, lane);
    flash::load_q<Tag, D>(w.q[1], q_src, p.q.sn, row0 + 32, p.N, lane);
    flash2::prescale_q<Tag, D>(w.q[0], p.scale_log2e);
    flash2::prescale_q<Tag, D>(w.q[1], p.scale_log2e);

    Scores s_even, s_odd;
    typename Pipe::Frags kf, vf;
    float mx[2] = {-INFINITY, -INFINITY};

    // masks of tile u for this wave: causal diagonal and end of the sequence; a tile past the wave's last row (or
    // past the last tile) ends up fully masked
    auto mask_tile = [&](Scores& sn, int u) __attribute__((always_inline)) {
        const int n0 = u * kBN;
        const bool whole = (n0 + kBN <= p.N) && (!p.causal || n0 + kBN - 1 <= row0) && u < n_iter;
        if (whole) return;  // (wave-uniform)
        flash2::mfma_settle();  // the scores below were produced by the last MFMAs
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
    const typename Pipe::TileRequest no_req{nullptr, 0};

    // first tile: scores, masks, row maxima (nothing to overlap with yet)
    request_k(0, 0);
    flash::wait_tile_loads();
    __syncthreads();
    if (n_iter > 1) request_k(1, 1);
    copy_v(s_v(0), 0);
    Pipe::k_head(kf, k_tile_of_wave(0, 0), lane);
    Pipe::template score_phase<true, false, false, false>(w, s_even, kf, s_odd, vf, 0u, lane, kd_c, no_req, vd, no_req);
    mask_tile(s_even, 0);
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
        mask_tile(sn, u + 1);
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

    Pipe::store(w, p.out + b * p.o_sb + h * p.o_sh, p.o_sn, p.lse ? p.lse + (int64_t)bh * p.N : nullptr, row0, p.N,
                lane);
    }
}

template <typename Tag, int D>
int launch(Params p, int B, hipStream_t stream) {
    // more than the 64 KB of LDS a launch gets by default: raised once per device and instantiation
    static bool raised[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return VQA_ERR_LAUNCH_FAILED;
    if (!raised[dev]) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_pipe_kernel<Tag, D>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes<D>()) != hipSuccess) {
            (void)hipGetLastError();
            return VQA_ERR_LAUNCH_FAILED;
        }
        raised[dev] = true;
    }
    const int n_tiles = (p.N + kBM - 1) / kBM;
    p.pair_tiles = (p.causal && (int64_t)(n_tiles / 2) * B * p.H >= 512) ? 1 : 0;
    const dim3 grid(p.pair_tiles ? (n_tiles + 1) / 2 : n_tiles, B * p.H);
    hipLaunchKernelGGL((prefill_pipe_kernel<Tag, D>), grid, dim3(flash2::kThreads), lds_bytes<D>(), stream, p);
    return launch_status();
}

}  // namespace pipe

// entry used by vqa_prefill_* (vqa_window.hip) once its arguments are validated and K_hat is written
namespace flash {

bool prefill_pipe_applies(int window, int boundary_is_block, bool has_exact, bool has_second_pair) {
    if (has_second_pair) return false;
    if (!has_exact) return true;
    return boundary_is_block && window % pipe::kBlock == 0;
}

template <typename Tag>
int prefill_pipe_run(const View& q, const View& ka, const View& kc, const View& v, uint16_t* out, int64_t o_sb,
                     int64_t o_sh, int64_t o_sn, float* lse, int B, int H, int N, int D, int window, int causal,
                     bool all_far, float scale_log2e, hipStream_t stream) {
    pipe::Params p;
    p.q = q, p.ka = ka, p.kc = kc, p.v = v;
    p.out = out;
    p.o_sb = o_sb, p.o_sh = o_sh, p.o_sn = o_sn;
    p.lse = lse;
    p.H = H, p.N = N, p.window = window;
    p.causal = causal;
    p.all_far = all_far ? 1 : 0;
    p.pair_tiles = 0;
    p.scale_log2e = scale_log2e;
    if (D == 64) return pipe::launch<Tag, 64>(p, B, stream);
    if (D == 128) return pipe::launch<Tag, 128>(p, B, stream);
    return VQA_ERR_UNSUPPORTED_HEAD_DIM;
}

template int prefill_pipe_run<bf16_tag>(const View&, const View&, const View&, const View&, uint16_t*, int64_t, int64_t,
                                        int64_t, float*, int, int, int, int, int, int, bool, float, hipStream_t);
template int prefill_pipe_run<f16_tag>(const View&, const View&, const View&, const View&, uint16_t*, int64_t, int64_t,
                                       int64_t, float*, int, int, int, int, int, int, bool, float, hipStream_t);

}  // namespace flash
}  // namespace vqa
