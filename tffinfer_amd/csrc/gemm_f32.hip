// float32 matrix product C = A . W^T on plain FMA (no matrix cores, so no
// reduced-precision mode can slip in).  The sum over k runs in ascending order
// for every element whatever M is, so a row's result does not depend on how
// many other rows the step holds.
//
// The reference's own float32 product is a 128x128x16 SIMT kernel
// (src/kernel/cuda/mat_mul.cu:149-518); this one is tiled for 64-wide waves:
// 64x64x16 tiles, 256 threads, 4x4 outputs each, operands staged through LDS.
#include "common.h"
#include "tffinfer_kernels.h"

#define F32_BM 64
#define F32_BN 64
#define F32_BK 16

template <typename TC>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A,
                                                        const float* __restrict__ W,
                                                        TC* __restrict__ C, int M, int N, int K,
                                                        int lda) {
    __shared__ float As[F32_BK][F32_BM + 4];
    __shared__ float Ws[F32_BK][F32_BN + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * F32_BM;
    const int n0 = blockIdx.x * F32_BN;
    const int tx = tid & 15;   // 16 column groups of 4
    const int ty = tid >> 4;   // 16 row groups of 4
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    // each thread stages 4 elements of each operand: row = tid / 4 (+0), k = (tid % 4) * 4 .. +3
    const int lr = tid >> 2;        // 0..63
    const int lk = (tid & 3) * 4;   // 0,4,8,12
    for (int k0 = 0; k0 < K; k0 += F32_BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int am = m0 + lr;
            const int wn = n0 + lr;
            As[lk + i][lr] = (am < M && k < K) ? A[(size_t)am * lda + k] : 0.f;
            Ws[lk + i][lr] = (wn < N && k < K) ? W[(size_t)wn * K + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < F32_BK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) C[(size_t)m * N + n] = from_f32<TC>(acc[i][j]);
        }
    }
}

int tff_gemm_f32(const float* A, const float* W, void* C, int M, int N, int K, int lda,
                 int c_dtype, hipStream_t s) {
    dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM);
    TFF_REQUIRE(grid.y <= 65535, "gemm: too many rows M=%d", M);
    if (c_dtype == TFF_F32)
        gemm_f32_kernel<float><<<grid, 256, 0, s>>>(A, W, (float*)C, M, N, K, lda);
    else
        return tff_fail("gemm: a float32 product writes float32, not type %d", c_dtype);
    return tff_check_launch("gemm_f32");
}
