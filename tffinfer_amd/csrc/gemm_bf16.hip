// bfloat16 matrix product C = A . W^T on the gfx950 matrix cores
// (v_mfma_f32_16x16x32_bf16), float32 accumulation.  Replaces the reference's
// SIMT products (src/kernel/cuda/quant/quant_q_8_0_mat_mul.cu:338-447,
// src/kernel/cuda/mat_mul.cu:149-518) with a design for 64-wide waves.
//
// Both operands are stored with k contiguous ([M, K] and [N, K]), which is the
// layout an MFMA lane wants: lane l feeds 8 consecutive k of row (l % 16) at
// k-chunk (l / 16).  The W tile is the MFMA's first operand, so a lane ends up
// with 4 consecutive output columns of one row and stores them as one vector.
#include "common.h"
#include "tffinfer_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define G_BM 128
#define G_BN 128
#define G_BK 64
#define G_LD (G_BK + 8)  // LDS row stride in elements; 144 bytes keeps 16-byte reads aligned and spreads banks

__device__ __forceinline__ uint4 ld16(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }

template <typename TC>
__global__ __launch_bounds__(256) void gemm_bf16_tiled_kernel(const bf16_t* __restrict__ A,
                                                               const bf16_t* __restrict__ W,
                                                               TC* __restrict__ C, int M, int N,
                                                               int K, int lda) {
    __shared__ __attribute__((aligned(16))) bf16_t As[2][G_BM * G_LD];
    __shared__ __attribute__((aligned(16))) bf16_t Ws[2][G_BN * G_LD];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * G_BM, n0 = blockIdx.x * G_BN;
    const int fr = lane & 15, fg = lane >> 4;

    floatx4 acc[4][4];  // [n subtile][m subtile]
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    uint4 ra[4], rw[4];
    const uint4 zero = make_uint4(0, 0, 0, 0);
    auto load_global = [&](int k0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = tid + 256 * j;       // 1024 chunks of 8 elements per operand tile
            const int row = c >> 3, kc = (c & 7) * 8;
            const int k = k0 + kc;
            const int am = m0 + row, wr = n0 + row;
            ra[j] = (am < M && k < K) ? ld16(A + (size_t)am * lda + k) : zero;
            rw[j] = (wr < N && k < K) ? ld16(W + (size_t)wr * K + k) : zero;
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = tid + 256 * j;
            const int row = c >> 3, kc = (c & 7) * 8;
            *reinterpret_cast<uint4*>(&As[buf][row * G_LD + kc]) = ra[j];
            *reinterpret_cast<uint4*>(&Ws[buf][row * G_LD + kc]) = rw[j];
        }
    };

    const int nk = (K + G_BK - 1) / G_BK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) load_global((kt + 1) * G_BK);
#pragma unroll
        for (int ks = 0; ks < G_BK; ks += 32) {
            bf16x8 fw[4], fa[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                fw[i] = *reinterpret_cast<const bf16x8*>(&Ws[buf][(wn * 64 + i * 16 + fr) * G_LD + ks + fg * 8]);
                fa[i] = *reinterpret_cast<const bf16x8*>(&As[buf][(wm * 64 + i * 16 + fr) * G_LD + ks + fg * 8]);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[i], fa[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) store_lds(buf ^ 1);
        __syncthreads();
    }

    // lane holds C[m][n .. n+3], n = n0 + wn*64 + i*16 + fg*4, m = m0 + wm*64 + j*16 + fr
    const bool vec = (N % 4) == 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int n = n0 + wn * 64 + i * 16 + fg * 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m0 + wm * 64 + j * 16 + fr;
            if (m >= M || n >= N) continue;
            TC* dst = C + (size_t)m * N + n;
            if (vec) {  // n % 4 == 0 and N % 4 == 0: the four columns exist
                if constexpr (sizeof(TC) == 4) {
                    *reinterpret_cast<float4*>(dst) =
                        make_float4(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
                } else {
                    union { bf16_t h[4]; uint2 u; } pk;
#pragma unroll
                    for (int e = 0; e < 4; ++e) pk.h[e] = (bf16_t)acc[i][j][e];
                    *reinterpret_cast<uint2*>(dst) = pk.u;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < N) dst[e] = from_f32<TC>(acc[i][j][e]);
            }
        }
    }
}

// ------------------------------------------------------------- skinny M ---
// For a few rows of A (decoding: M = number of live requests) the product is
// a stream of W from HBM; what counts is bytes in flight, not LDS tiling.
// A block owns a slab of 16*R rows of W for the whole of K; its waves split K
// among them in contiguous runs, each wave reading W straight from global
// memory into MFMA operands (16 rows x 64 contiguous bytes per load) and the
// few rows of A from cache; partial sums meet in LDS and are added in a fixed
// order, so no partial result goes through global memory and the result does
// not depend on the launch.
#define SK_WAVES 8

// UNROLL k-steps of loads are issued before the first is used: a wave keeps
// UNROLL * (R + MT) KB in flight, which is what hides the latency of HBM.
template <int MT, int R, int UNROLL, typename TC>
__global__ __launch_bounds__(64 * SK_WAVES) void gemm_bf16_skinny_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, TC* __restrict__ C, int M, int N,
    int K, int lda) {
    __shared__ floatx4 part[SK_WAVES - 1][R * MT][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fr = lane & 15, fg = lane >> 4;
    const int n0 = blockIdx.x * (16 * R);

    floatx4 acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[r][t] = floatx4{0.f, 0.f, 0.f, 0.f};

    // k-steps of 32 are dealt out to the waves in contiguous runs
    const int nsteps = (K + 31) / 32;
    const int per = (nsteps + SK_WAVES - 1) / SK_WAVES;
    const int s_begin = wave * per;
    const int s_end = min(nsteps, s_begin + per);

    const bf16_t* wrow[R];
    bool wok[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int n = n0 + r * 16 + fr;
        wok[r] = n < N;
        wrow[r] = W + (size_t)(wok[r] ? n : 0) * K;
    }
    const bf16_t* arow[MT];
    bool aok[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + fr;
        aok[t] = m < M;
        arow[t] = A + (size_t)(aok[t] ? m : 0) * lda;
    }
    const uint4 zero = make_uint4(0, 0, 0, 0);
    for (int s0 = s_begin; s0 < s_end; s0 += UNROLL) {
        uint4 rw[UNROLL][R], ra[UNROLL][MT];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int k = (s0 + u) * 32 + fg * 8;
            const bool kok = (s0 + u) < s_end && k < K;
#pragma unroll
            for (int r = 0; r < R; ++r) rw[u][r] = (kok && wok[r]) ? ld16(wrow[r] + k) : zero;
#pragma unroll
            for (int t = 0; t < MT; ++t) ra[u][t] = (kok && aok[t]) ? ld16(arow[t] + k) : zero;
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        *reinterpret_cast<bf16x8*>(&rw[u][r]), *reinterpret_cast<bf16x8*>(&ra[u][t]),
                        acc[r][t], 0, 0, 0);
    }
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < MT; ++t) part[wave - 1][r * MT + t][lane] = acc[r][t];
    }
    __syncthreads();
    if (wave == 0) {
        const bool vec = (N % 4) == 0;
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                floatx4 v = acc[r][t];
#pragma unroll
                for (int w = 0; w < SK_WAVES - 1; ++w) {
                    const floatx4 p = part[w][r * MT + t][lane];
                    v[0] += p[0]; v[1] += p[1]; v[2] += p[2]; v[3] += p[3];
                }
                const int n = n0 + r * 16 + fg * 4;
                const int m = t * 16 + fr;
                if (m >= M || n >= N) continue;
                TC* dst = C + (size_t)m * N + n;
                if (vec) {
                    if constexpr (sizeof(TC) == 4) {
                        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
                    } else {
                        union { bf16_t h[4]; uint2 u; } pk;
#pragma unroll
                        for (int e = 0; e < 4; ++e) pk.h[e] = (bf16_t)v[e];
                        *reinterpret_cast<uint2*>(dst) = pk.u;
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < N) dst[e] = from_f32<TC>(v[e]);
                }
            }
    }
}

template <int MT, int R, int UNROLL>
static int launch_skinny(const bf16_t* A, const bf16_t* W, void* C, int M, int N, int K, int lda,
                         int c_dtype, hipStream_t s) {
    const dim3 grid((N + 16 * R - 1) / (16 * R));
    if (c_dtype == TFF_F32)
        gemm_bf16_skinny_kernel<MT, R, UNROLL, float><<<grid, 64 * SK_WAVES, 0, s>>>(A, W, (float*)C, M, N, K, lda);
    else
        gemm_bf16_skinny_kernel<MT, R, UNROLL, bf16_t><<<grid, 64 * SK_WAVES, 0, s>>>(A, W, (bf16_t*)C, M, N, K, lda);
    return tff_check_launch("gemm_bf16_skinny");
}

int tff_gemm_bf16(const bf16_t* A, const bf16_t* W, void* C, int M, int N, int K, int lda,
                  int c_dtype, hipStream_t s) {
    TFF_REQUIRE(K % 8 == 0 && lda % 8 == 0,
                "gemm: the bfloat16 product needs the inner size (K=%d, row stride %d) to be a multiple of 8",
                K, lda);
    TFF_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)C % 16) == 0,
                "gemm: operands must be 16-byte aligned");
    TFF_REQUIRE(c_dtype == TFF_F32 || c_dtype == TFF_BF16, "gemm: unknown output type %d", c_dtype);
    if (M <= 64) {
        // slabs of 32 rows when that still gives every CU several blocks, else of 16
        const bool wide = N >= 32 * 1024;
        const int mt = (M + 15) / 16;
        switch (mt * 2 + (wide ? 1 : 0)) {
            case 2: return launch_skinny<1, 1, 16>(A, W, C, M, N, K, lda, c_dtype, s);
            case 3: return launch_skinny<1, 2, 8>(A, W, C, M, N, K, lda, c_dtype, s);
            case 4: return launch_skinny<2, 1, 8>(A, W, C, M, N, K, lda, c_dtype, s);
            case 5: return launch_skinny<2, 2, 6>(A, W, C, M, N, K, lda, c_dtype, s);
            case 6: return launch_skinny<3, 1, 6>(A, W, C, M, N, K, lda, c_dtype, s);
            case 7: return launch_skinny<3, 2, 4>(A, W, C, M, N, K, lda, c_dtype, s);
            case 8: return launch_skinny<4, 1, 6>(A, W, C, M, N, K, lda, c_dtype, s);
            default: return launch_skinny<4, 2, 4>(A, W, C, M, N, K, lda, c_dtype, s);
        }
    }
    dim3 grid((N + G_BN - 1) / G_BN, (M + G_BM - 1) / G_BM);
    TFF_REQUIRE(grid.y <= 65535, "gemm: too many rows M=%d", M);
    if (c_dtype == TFF_F32)
        gemm_bf16_tiled_kernel<float><<<grid, 256, 0, s>>>(A, W, (float*)C, M, N, K, lda);
    else if (c_dtype == TFF_BF16)
        gemm_bf16_tiled_kernel<bf16_t><<<grid, 256, 0, s>>>(A, W, (bf16_t*)C, M, N, K, lda);
    else
        return tff_fail("gemm: unknown output type %d", c_dtype);
    return tff_check_launch("gemm_bf16");
}

int tff_gemm_f32(const float* A, const float* W, void* C, int M, int N, int K, int lda,
                 int c_dtype, hipStream_t s);

TFF_API int tff_gemm(const void* A, const void* W, void* C, int M, int N, int K, int lda,
                     int ab_dtype, int c_dtype, tff_stream_t stream) {
    TFF_REQUIRE(A && W && C, "gemm: null pointer");
    TFF_REQUIRE(M >= 0 && N > 0 && K > 0 && lda >= K, "gemm: bad sizes M=%d N=%d K=%d lda=%d", M, N, K, lda);
    if (M == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (ab_dtype == TFF_F32) return tff_gemm_f32((const float*)A, (const float*)W, C, M, N, K, lda, c_dtype, s);
    if (ab_dtype == TFF_BF16) return tff_gemm_bf16((const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, c_dtype, s);
    return tff_fail("gemm: unknown operand type %d", ab_dtype);
}
