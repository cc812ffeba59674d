"""Per-wave instruction issue micro-benchmarks for gfx950: loops whose bodies are fixed instruction sequences (inline
assembly, so the compiler cannot reorder or drop them) -- v_mfma_f32_32x32x16_bf16 alone, MFMAs with n independent
VALU / transcendental / LDS instructions between them, and the VALU instructions alone -- timed per iteration with the
shader clock, one wave per SIMD (256 threads per workgroup, one workgroup per CU) and two.

    python3 issue_rate.py /tmp/issue_rate.hip
    hipcc -O3 --offload-arch=gfx950 /tmp/issue_rate.hip -o /tmp/issue_rate && /tmp/issue_rate

An iteration holds 4 MFMAs (or 32 VALU instructions / 8 LDS reads in the "_only" variants)."""
import sys

variants = {}
def mfma(i): return f"v_mfma_f32_32x32x16_bf16 %{i}, %4, %5, %{i}\n"
def fma(j): return f"v_fma_f32 %{6+j}, %{6+j}, %{6+j}, %{6+j}\n"
def exp(j): return f"v_exp_f32 %{6+j}, %{6+j}\n"
def mx3(j): return f"v_max3_f32 %{6+j}, %{6+j}, %{6+(j+1)%8}, %{6+(j+2)%8}\n"
def cvt(j): return f"v_cvt_pk_bf16_f32 %{6+j}, %{6+j}, %{6+(j+1)%8}\n"
def dsr(j): return f"ds_read_b128 %{14+j%2}, %16 offset:{(j*1024)%32768}\n"
def body(per, kind, n_mfma=4):
    s = ""
    k = 0
    for i in range(n_mfma):
        s += mfma(i % 4)
        for e in range(per):
            s += kind(k % 8); k += 1
    return s
variants["mfma4"] = body(0, fma)
for n in (1, 2, 4, 6, 8, 12):
    variants[f"mfma_fma{n}"] = body(n, fma)
for n in (1, 2, 4, 6):
    variants[f"mfma_exp{n}"] = body(n, exp)
variants["fma32_only"] = "".join(fma(j % 8) for j in range(32))
variants["exp32_only"] = "".join(exp(j % 8) for j in range(32))
variants["max3_32_only"] = "".join(mx3(j % 8) for j in range(32))
variants["cvt32_only"] = "".join(cvt(j % 8) for j in range(32))
for n in (1, 2, 3):
    variants[f"mfma_ds{n}"] = body(n, dsr) + "s_waitcnt lgkmcnt(0)\n"
variants["ds8_only"] = "".join(dsr(j) for j in range(8)) + "s_waitcnt lgkmcnt(0)\n"
# mixed: like a softmax slice: per MFMA 1 exp + 1 fma + 1 max3(0.5) ...
def mix(j): return fma(j) + exp((j+3)%8)
variants["mfma_fmaexp1"] = body(1, mix)
variants["mfma_fmaexp2"] = body(2, mix)
variants["mfma_fmaexp3"] = body(3, mix)

src = r'''
#include <hip/hip_runtime.h>
#include <cstdio>
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
#define KERNEL(NAME, BODY) \
__global__ __launch_bounds__(512) void NAME(float* out, int iters, long long* clk) { \
  __shared__ char lds[65536]; \
  bf16x8 a, b; \
  for (int e = 0; e < 8; ++e) { a[e] = (__bf16)(float)(threadIdx.x + e); b[e] = (__bf16)(float)(e); } \
  f32x16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0}; \
  float x0 = threadIdx.x * 1e-3f, x1 = x0 + 1, x2 = x0 + 2, x3 = x0 + 3, x4 = x0 + 4, x5 = x0 + 5, x6 = x0 + 6, x7 = x0 + 7; \
  f32x4 d0 = {0}, d1 = {0}; \
  unsigned la = (unsigned)(size_t)(__attribute__((address_space(3))) char*)lds + (threadIdx.x & 63) * 16; \
  if (threadIdx.x == 9999) lds[0] = 1; \
  __syncthreads(); \
  const long long t0 = clock64(), w0 = wall_clock64(); \
  for (int it = 0; it < iters; ++it) { \
    asm volatile(BODY : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(a), "v"(b), "v"(x0), "v"(x1), "v"(x2), "v"(x3), "v"(x4), "v"(x5), "v"(x6), "v"(x7), "v"(d0), "v"(d1), "v"(la) : "memory"); \
  } \
  const long long t1 = clock64(), w1 = wall_clock64(); \
  if (blockIdx.x == 17 && threadIdx.x == 0) { clk[0] = t1 - t0; clk[1] = w1 - w0; } \
  out[blockIdx.x * blockDim.x + threadIdx.x] = c0[0] + c1[1] + c2[2] + c3[3] + x0 + x1 + x2 + x3 + x4 + x5 + x6 + x7 + d0[0] + d1[1]; \
}
'''
for name, b in variants.items():
    lit = "".join('"' + l + '\\n"\n' for l in b.strip().split("\n"))
    src += f"KERNEL(k_{name}, {lit})\n"
src += r'''
typedef void (*kern_t)(float*, int, long long*);
void run(const char* name, kern_t k, int threads) {
  float* o; hipMalloc(&o, 256 * 512 * 4);
  long long* clk; hipMalloc(&clk, 16); long long hc[2];
  const int iters = 20000;
  hipLaunchKernelGGL(k, dim3(256), dim3(threads), 0, 0, o, 10, clk);
  hipDeviceSynchronize();
  hipLaunchKernelGGL(k, dim3(256), dim3(threads), 0, 0, o, iters, clk);
  hipDeviceSynchronize();
  hipMemcpy(hc, clk, 16, hipMemcpyDeviceToHost);
  printf("%-16s waves/SIMD %d: %8.1f clk/iter  (%.0f MHz)\n", name, threads / 256, (double)hc[0] / iters, hc[0] / (hc[1] / 100.0));
  hipFree(o); hipFree(clk);
}
int main() {
'''
for name in variants:
    src += f'  run("{name}", k_{name}, 256);\n'
for name in ("mfma4", "mfma_fma4", "mfma_fma8", "mfma_exp2", "mfma_exp4", "mfma_fmaexp2", "mfma_fmaexp3", "mfma_ds2"):
    src += f'  run("{name}", k_{name}, 512);\n'
src += '  printf("err %s\\n", hipGetErrorString(hipGetLastError()));\n}\n'
open(sys.argv[1] if len(sys.argv) > 1 else "issue_rate.hip", "w").write(src)
