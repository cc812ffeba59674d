// LDS read rates of the two ways to score far (quantised) keys in the prefill kernel, per compute unit:
//   "table"  : score(i, j) = sum_m LUT_m[i][code_jm] -- one 4-byte LDS gather per (query, key, codebook).  In the
//              transposed score layout a lane is a query and a register a key, so the 32 lanes of a half-wave read the
//              SAME table column in 32 different rows: rows are padded by one word, which makes that conflict-free.
//   "matrix" : score = q . K_hat[j] on the matrix pipes -- the reconstructed key tile is an MFMA operand read with
//              ds_read_b128 (swizzled rows), as the exact keys are.
// Also the transposing 8-byte reads of the V operand.  Every pattern runs on all CUs with 4 waves per workgroup and
// 1, 2 or 4 workgroups per CU (one wave alone cannot keep the LDS pipe busy); the figures are bytes per clock per CU
// at the clock measured inside the kernel.  The tables of the gather patterns are cut to 64 entries per row (padded
// to 65 words) so that four workgroups fit a CU; the bank pattern is that of the full 256-entry tables (odd stride).
//
//   hipcc -O3 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops lds_far_path.hip -o lds_far_path
#include <hip/hip_runtime.h>

#include <cstdio>

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4* lds_tr_ptr;

enum Pattern { kGatherRows = 0, kGatherRandom = 1, kOperandB128 = 2, kOperandTr = 3 };

extern __shared__ __attribute__((aligned(1024))) char lds[];

template <int PATTERN>
__global__ __launch_bounds__(256) void k(unsigned* out, int iters, long long* clk, int lds_words) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < lds_words; i += 256) ((unsigned*)lds)[i] = i * 2654435761u;
    __syncthreads();
    const unsigned base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)lds;
    unsigned addr[32];
    if (PATTERN == kGatherRows || PATTERN == kGatherRandom) {
        // one table per query row, rows padded by one word; a wave owns 32 rows
        const int row = lane & 31, half = lane >> 5;
        for (int r = 0; r < 32; ++r) {
            unsigned code = ((unsigned)(r * 2 + half) * 2654435761u >> 13) & 63u;          // one key per (register, half)
            if (PATTERN == kGatherRandom) code = ((unsigned)(r * 64 + lane) * 2246822519u >> 11) & 63u;  // per lane
            addr[r] = base + ((wave * 32 + row) * 65 + code) * 4;
        }
    } else if (PATTERN == kOperandB128) {
        const int r = lane & 31, half = lane >> 5;  // K tile 64 x 128 bf16, 16-byte chunks XOR-swizzled by row % 16
        for (int i = 0; i < 16; ++i) {
            const int kk = i / 2, kb = i % 2;
            addr[i] = base + (kb * 32 + r) * 256 + ((((2 * kk) + half) ^ (r % 16)) << 4);
            addr[16 + i] = addr[i] + 16384;
        }
    } else {
        const int half = lane >> 5, dsub = (lane >> 4) & 1, sl = lane & 15;  // V tile, transposing reads
        const int row = 4 * half + (sl >> 2);
        for (int i = 0; i < 32; ++i) {
            const int f = i / 2, db = f % 4, j = f / 4, hi = i % 2;
            const int chunk = (4 * db + 2 * dsub + ((sl & 3) >> 1)) ^ (4 * (row % 4));
            addr[i] = base + (j * 16 + row + 8 * hi) * 256 + chunk * 16 + ((sl & 1) << 3);
        }
    }
    unsigned acc = 0;
    const long long t0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            if (PATTERN == kGatherRows || PATTERN == kGatherRandom) {
                acc += *(const __attribute__((address_space(3))) unsigned*)(size_t)addr[i];
            } else if (PATTERN == kOperandB128) {
                const u32x4 v = *(const __attribute__((address_space(3))) u32x4*)(size_t)addr[i];
                acc += v[0] ^ v[1] ^ v[2] ^ v[3];
            } else {
                const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(size_t)addr[i]);
                acc += a[0] ^ a[3];
            }
        }
        asm volatile("" ::: "memory");
    }
    const long long t1 = clock64(), w1 = wall_clock64();
    if (blockIdx.x == 3 && tid == 0) { clk[0] = t1 - t0; clk[1] = w1 - w0; }
    out[blockIdx.x * 256 + tid] = acc;
}

template <int PATTERN>
void run(const char* name, int bytes_per_lane, int wgs_per_cu) {
    unsigned* o; long long* clk; long long hc[2];
    (void)hipMalloc(&o, 1024 * 256 * 4); (void)hipMalloc(&clk, 16);
    const int lds_bytes = 36 * 1024, iters = 4000, blocks = 256 * wgs_per_cu;
    (void)hipFuncSetAttribute((const void*)k<PATTERN>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    k<PATTERN><<<blocks, 256, lds_bytes>>>(o, 10, clk, lds_bytes / 4);
    (void)hipDeviceSynchronize();
    hipEvent_t a, b; (void)hipEventCreate(&a); (void)hipEventCreate(&b);
    (void)hipEventRecord(a);
    k<PATTERN><<<blocks, 256, lds_bytes>>>(o, iters, clk, lds_bytes / 4);
    (void)hipEventRecord(b); (void)hipEventSynchronize(b);
    float ms; (void)hipEventElapsedTime(&ms, a, b);
    (void)hipMemcpy(hc, clk, 16, hipMemcpyDeviceToHost);
    const double mhz = hc[0] / (hc[1] / 100.0);
    const double instr_per_cu = (double)wgs_per_cu * 4 * iters * 32;  // wave instructions per CU
    const double clocks = ms * 1e-3 * mhz * 1e6;
    printf("%-34s %d WG/CU  %7.3f ms  %5.0f MHz  %6.2f clk/wave-instr/CU  %6.1f B/clk/CU  (%s)\n", name, wgs_per_cu, ms, mhz,
           clocks / instr_per_cu, instr_per_cu * 64 * bytes_per_lane / clocks, hipGetErrorString(hipGetLastError()));
    (void)hipFree(o); (void)hipFree(clk);
}

int main() {
    for (int w = 1; w <= 4; w *= 2) {
        run<kGatherRows>("table gather, padded rows (b32)", 4, w);
        run<kGatherRandom>("table gather, random lanes (b32)", 4, w);
        run<kOperandB128>("K operand, swizzled (b128)", 16, w);
        run<kOperandTr>("V operand, transposing (b64_tr_b16)", 8, w);
    }
    return 0;
}
