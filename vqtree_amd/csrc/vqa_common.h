// Internal helpers shared by the gfx950 kernels of libvqattn (not part of the C ABI).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#define VQA_NO_HIP_STREAM_TYPEDEF
typedef hipStream_t vqa_stream_t;
#include "../../include/vqattn.h"

namespace vqa {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kWave = 64;

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

struct bf16_tag {};
struct f16_tag {};

// Element-type traits: 16-bit storage, fp32 arithmetic.
template <typename Tag>
struct Elem;

template <>
struct Elem<bf16_tag> {
    typedef bf16x8_t vec8;
    // round-to-nearest-even fp32 -> bf16, returned as an fp32 whose low 16 bits are zero
    static __device__ __forceinline__ float round_keep_f32(float x) {
        uint32_t u = __builtin_bit_cast(uint32_t, x);
        u += 0x7fffu + ((u >> 16) & 1u);
        return __builtin_bit_cast(float, u & 0xffff0000u);
    }
    static __device__ __forceinline__ uint16_t to_bits(float x) {
        return (uint16_t)(__builtin_bit_cast(uint32_t, round_keep_f32(x)) >> 16);
    }
    // bits of a value round_keep_f32 already produced
    static __device__ __forceinline__ uint32_t rounded_to_bits(float x) {
        return __builtin_bit_cast(uint32_t, x) >> 16;
    }
    static __device__ __forceinline__ float from_bits(uint16_t b) {
        return __builtin_bit_cast(float, (uint32_t)b << 16);
    }
    // acc + a.lo*b.lo + a.hi*b.hi with a, b packed pairs
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc,
                                               false);
    }
    // two fp32 -> packed pair (lo = a, hi = b), round to nearest even (v_cvt_pk_bf16_f32)
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        const f32x2_t v = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
    }
    static __device__ __forceinline__ f32x4_t mfma16(vec8 a, vec8 b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x16_t mfma32(vec8 a, vec8 b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};

template <>
struct Elem<f16_tag> {
    typedef f16x8_t vec8;
    static __device__ __forceinline__ float round_keep_f32(float x) { return (float)(_Float16)x; }
    static __device__ __forceinline__ uint16_t to_bits(float x) {
        return __builtin_bit_cast(uint16_t, (_Float16)x);
    }
    static __device__ __forceinline__ uint32_t rounded_to_bits(float x) { return to_bits(x); }
    static __device__ __forceinline__ float from_bits(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b), acc, false);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        const f32x2_t v = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
    }
    static __device__ __forceinline__ f32x4_t mfma16(vec8 a, vec8 b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x16_t mfma32(vec8 a, vec8 b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
    return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
    return x;
}

// Orders this wave's LDS writes before its later LDS reads by other lanes (no cross-wave effect).
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
}

// 16-byte accesses to data that is touched exactly once (streams): the non-temporal hint keeps the stream from
// displacing lines that are re-read.  Measured on a 4 GiB read-only sweep it lifts the rate from ~6.3 to ~7.1 TB/s.
typedef uint32_t stream_u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_stream16(const void* p) {
    const stream_u32x4_t t = __builtin_nontemporal_load(static_cast<const stream_u32x4_t*>(p));
    return make_uint4(t[0], t[1], t[2], t[3]);
}
__device__ __forceinline__ void store_stream16(void* p, uint4 v) {
    const stream_u32x4_t t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, static_cast<stream_u32x4_t*>(p));
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Row strides (in elements of a 16-bit type) for which 64 consecutive rows still fit the 32-bit per-lane byte offsets
// of the streaming and tile-copy loops; anything else is rejected on the host before a launch.
inline bool row_stride_ok(int64_t sn) { return sn >= 0 && sn < (int64_t(1) << 24); }

inline int launch_status() { return hipGetLastError() == hipSuccess ? VQA_OK : VQA_ERR_LAUNCH_FAILED; }

// Per-device set-up (a kernel attribute raised once, the address of a file-scope device array) belongs to the device
// that OWNS the memory a call works on, which need not be the calling thread's current device.  Returns that device
// for a device pointer, VQA_ERR_BAD_ARGUMENT if it is not the current device (the launch that follows would run on
// the current one), VQA_ERR_LAUNCH_FAILED if the runtime cannot tell.
constexpr int kMaxDevices = 64;
inline int device_of_pointer(const void* ptr, int* device) {
    int cur = 0;
    if (hipGetDevice(&cur) != hipSuccess || cur < 0 || cur >= kMaxDevices) return VQA_ERR_LAUNCH_FAILED;
    hipPointerAttribute_t attr;
    if (ptr != nullptr && hipPointerGetAttributes(&attr, ptr) == hipSuccess) {
        if (attr.type == hipMemoryTypeDevice && attr.device != cur) return VQA_ERR_BAD_ARGUMENT;
    } else {
        (void)hipGetLastError();  // not a pointer the runtime knows (host code tests pass such): current device
    }
    *device = cur;
    return VQA_OK;
}

}  // namespace vqa
