// Shared helpers of the gfx950 kernels: element types, wave and block
// reductions, the error channel of the C entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;

// Element type codes of the C entry points.
enum { TFF_F32 = 0, TFF_BF16 = 1 };

#define TFF_WAVE 64

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Sum over a block of up to 1024 threads; `red` holds at least 17 floats.
// Every thread gets the result.  The order of the additions is fixed.
__device__ __forceinline__ float block_sum(float v, float* red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nwave = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        float s = 0.f;
        for (int i = 0; i < nwave; ++i) s += red[i];
        red[16] = s;
    }
    __syncthreads();
    return red[16];
}
__device__ __forceinline__ float block_max(float v, float* red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nwave = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        float s = red[0];
        for (int i = 1; i < nwave; ++i) s = fmaxf(s, red[i]);
        red[16] = s;
    }
    __syncthreads();
    return red[16];
}

// Host side: the entry points return 0 or a negative code and leave a message
// that tff_last_error() hands out.
int tff_fail(const char* fmt, ...);
int tff_check_launch(const char* what);

#define TFF_REQUIRE(cond, ...)                     \
    do {                                           \
        if (!(cond)) return tff_fail(__VA_ARGS__); \
    } while (0)

// Maximum / sum over the four lanes i, i ^ 16, i ^ 32, i ^ 48 (the four 16-lane rows of a wave),
// the result in all four.  v_permlane16_swap exchanges the odd rows of one register with the
// even rows of another and v_permlane32_swap the upper half of one with the lower half of the
// other: applied to two copies of a value, the two results hold, lane by lane, the two values
// to combine.  No trip through LDS, unlike a shuffle across rows.  The sum adds in the order
// (row 0 + row 1) + (row 2 + row 3), as two shuffle steps would.
typedef unsigned tff_uint2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float rows_max(float v) {
    tff_uint2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    const float m = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(m), __float_as_uint(m), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float rows_sum(float v) {
    tff_uint2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    const float m = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(m), __float_as_uint(m), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Copies 16 bytes a lane from global memory straight into LDS: lane i's bytes land at
// lds_wave_base + 16 i (global_load_lds_dwordx4; the LDS base travels in M0 and is the same for
// the whole wave).  It is written as inline assembly on purpose: the compiler's own builtin
// makes every later LDS read wait for *all* copies in flight (it cannot tell which stage a
// read touches), which turns a pipeline of several stages into one of a single stage.  Here
// the compiler knows nothing of the copy; the kernels wait for their copies themselves
// (s_waitcnt vmcnt(n), copies complete in the order they were issued) before the barrier that
// lets other waves read them.
// The same with the LDS address (bytes from the start of LDS) worked out by the caller.
__device__ __forceinline__ void copy16_to_lds_at(const void* gptr, unsigned lds_wave_addr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_wave_addr)), "v"(gptr)
                 : "memory", "m0");
}
__device__ __forceinline__ void copy16_to_lds(const void* gptr, void* lds_wave_base) {
    const unsigned base = (unsigned)(size_t)(__attribute__((address_space(3))) void*)lds_wave_base;
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(base)), "v"(gptr)
                 : "memory", "m0");
}
