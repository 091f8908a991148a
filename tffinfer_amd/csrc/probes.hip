// Two measuring kernels for the ceilings the other kernels are judged by on the
// machine at hand: how fast memory can be streamed into registers, and how
// fast the matrix cores run 16x16x32 bfloat16 MFMAs back to back (with operands
// that never change, and with operands that change as those of a real product do).  They compute
// nothing of use; the callers time them.
#include "common.h"
#include "tffinfer_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

// every wave reads runs of 1 KB (16 bytes a lane), eight loads in flight, a grid-stride apart
__global__ __launch_bounds__(256) void probe_stream_kernel(const uint4* __restrict__ src, size_t n16,
                                                           uint32_t* __restrict__ sink) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint4 acc = make_uint4(0, 0, 0, 0);
    for (; i + 7 * stride < n16; i += 8 * stride) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = src[i + u * stride];
#pragma unroll
        for (int u = 0; u < 8; ++u) { acc.x ^= v[u].x; acc.y ^= v[u].y; acc.z ^= v[u].z; acc.w ^= v[u].w; }
    }
    for (; i < n16; i += stride) { const uint4 v = src[i]; acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w; }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = acc.x;   // keeps the loads alive
}

// VARIED = false: every MFMA multiplies the same two registers of small integers (few bits change
// from one instruction to the next, the lowest power the matrix cores can draw); true: eight
// registers of pseudo-random values on either side, taken in turn, as the operands of a real
// product change.  The difference between the two rates is what the power limit costs.
__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}
template <bool VARIED>
__global__ __launch_bounds__(256) void probe_mfma_kernel(float* __restrict__ sink, int iters) {
    floatx4 acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
    constexpr int R = VARIED ? 8 : 1;
    bf16x8 a[R], b[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if constexpr (VARIED) {
                const uint32_t h1 = probe_hash(threadIdx.x * 977u + r * 131u + e * 7u + 1u), h2 = probe_hash(h1 + 12345u);
                a[r][e] = (bf16_t)(((int)(h1 & 0xffff) - 32768) * (0.05f / 32768.f));
                b[r][e] = (bf16_t)(((int)(h2 & 0xffff) - 32768) * (1.0f / 32768.f));
            } else {
                a[r][e] = (bf16_t)(float)((threadIdx.x + e) & 7);
                b[r][e] = (bf16_t)(float)(e + 1);
            }
        }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i)
            acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i % R], b[(i * 3 + 1) % R], acc[i], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    if (s == 12345.678f) sink[0] = s;
}

// Reads `bytes` (a multiple of 16) from src once.
TFF_API int tff_probe_stream_read(const void* src, size_t bytes, void* sink, int blocks, tff_stream_t stream) {
    TFF_REQUIRE(src && sink && bytes % 16 == 0 && ((uintptr_t)src % 16) == 0 && blocks > 0,
                "probe_stream_read: needs a 16-byte aligned buffer of a multiple of 16 bytes");
    probe_stream_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((const uint4*)src, bytes / 16, (uint32_t*)sink);
    return tff_check_launch("probe_stream_read");
}

// blocks x 4 waves, each issuing iters x 16 independent MFMAs: blocks * 4 * iters * 16 * 16384 flops.
TFF_API int tff_probe_mfma(void* sink, int blocks, int iters, int varied_operands, tff_stream_t stream) {
    TFF_REQUIRE(sink && blocks > 0 && iters > 0, "probe_mfma: bad arguments");
    if (varied_operands) probe_mfma_kernel<true><<<blocks, 256, 0, (hipStream_t)stream>>>((float*)sink, iters);
    else probe_mfma_kernel<false><<<blocks, 256, 0, (hipStream_t)stream>>>((float*)sink, iters);
    return tff_check_launch("probe_mfma");
}
