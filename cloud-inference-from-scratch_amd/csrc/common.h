// Shared device helpers for the gfx950 kernels: storage types, bf16 conversion,
// wave64 and workgroup reductions, launch-error reporting.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define CIE_API extern "C" __attribute__((visibility("default")))

// Return codes of every entry point.  0 is success; the Python side turns the
// others into exceptions that name the entry point.
enum {
    CIE_OK = 0,
    CIE_BAD_ARGUMENT = 1,   // a size or option the kernel does not take
    CIE_LAUNCH_FAILED = 2,  // hipGetLastError() after the launch
    CIE_TOO_LARGE = 3,      // more than the fixed scratch memory of an entry point that allocates nothing holds
    CIE_SETUP_FAILED = 4,   // the library's own device memory could not be found on this device
};

constexpr int kWave = 64;

// Activation / weight storage.  dtype codes used across the C ABI.
enum { CIE_F32 = 0, CIE_BF16 = 1 };

struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) {
    return __uint_as_float(static_cast<uint32_t>(x.bits) << 16);
}

// Round to nearest even; NaN stays NaN.
__device__ __forceinline__ uint16_t bf16_bits_from_float(float x) {
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

// Two floats to two bfloat16 in one word (low half first), round to nearest even: on gfx950 this is
// the v_cvt_pk_bf16_f32 instruction.
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float floatx2_t __attribute__((ext_vector_type(2)));
    const floatx2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

template <typename T>
__device__ __forceinline__ T from_float(float x);
template <>
__device__ __forceinline__ float from_float<float>(float x) {
    return x;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float x) {
    bf16_t r;
    r.bits = static_cast<uint16_t>(pack_bf16(x, 0.f) & 0xffffu);
    return r;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, kWave);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, kWave));
    return v;
}

// Reductions over the four 16-lane rows of a wave (lanes r, r+16, r+32, r+48; every lane gets the
// result) with gfx950's row-swap instructions, which stay in the vector ALU: no round trip through LDS.
// v_permlane16_swap(a, b) exchanges the odd rows of a with the even rows of b; v_permlane32_swap(a, b)
// the upper half of a with the lower half of b.  Fed the same value twice, the two results hold, in
// every lane, the lane's own value and its partner's.
typedef unsigned swap_pair_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float rows_max(float v) {
    swap_pair_t a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    swap_pair_t b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

__device__ __forceinline__ float rows_sum(float v) {
    swap_pair_t a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    swap_pair_t b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Sum over a workgroup of up to 16 waves; every thread gets the result.
// `scratch` is at least 16 floats of LDS; the call contains barriers.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int waves = (blockDim.x + kWave - 1) / kWave;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < waves; ++w) total += scratch[w];
    return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int waves = (blockDim.x + kWave - 1) / kWave;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = scratch[0];
    for (int w = 1; w < waves; ++w) total = fmaxf(total, scratch[w]);
    return total;
}

static inline int cie_after_launch() {
    return hipGetLastError() == hipSuccess ? CIE_OK : CIE_LAUNCH_FAILED;
}
