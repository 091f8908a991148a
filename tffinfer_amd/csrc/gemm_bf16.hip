// bfloat16 matrix product C = A . W^T on the gfx950 matrix cores
// (v_mfma_f32_16x16x32_bf16), float32 accumulation.  Replaces the reference's
// SIMT products (src/kernel/cuda/quant/quant_q_8_0_mat_mul.cu:338-447,
// src/kernel/cuda/mat_mul.cu:149-518) with a design for 64-wide waves.
//
// Weights are kept in *fragment order*: W [N, K] is cut into tiles of 16 rows
// by 32 k, and each tile is stored as the 1 KB an MFMA operand is, lane after
// lane: element (n, k) lies at
//     ((n / 16) * (Kp / 32) + k / 32) * 512 + (((k % 32) / 8) * 16 + n % 16) * 8 + k % 8
// with N and K padded to multiples of 16 and 32 by zeros.  A wave fetches an
// operand with one fully contiguous 1 KB load (measured: a quarter more of
// the HBM bandwidth than 16 rows x 64 bytes of a row-major matrix), and a tile
// staged in LDS in the same order is read back without bank conflicts.
// Activations A [M, K] stay row-major.  The W tile is the MFMA's first operand,
// so a lane ends up with 4 consecutive output columns of one row.
#include "common.h"
#include "tffinfer_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

__device__ __forceinline__ uint4 ld16(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ bf16x8 as_frag(const uint4& v) { return *reinterpret_cast<const bf16x8*>(&v); }

template <typename TC>
__device__ __forceinline__ void store4(TC* dst, const floatx4& v, int n, int N, bool vec) {
    if (vec) {  // n % 4 == 0 and N % 4 == 0: the four columns exist
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

// GLU: the 16-row groups of W alternate between a gate and an up projection
// (group 2p gate, group 2p+1 up); the epilogue writes silu(gate) * up, N / 2 columns.
__device__ __forceinline__ floatx4 silu_mul(const floatx4& g, const floatx4& u) {
    floatx4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = g[e] / (1.0f + __expf(-g[e])) * u[e];
    return o;
}

// ------------------------------------------------------- tiled, async copy ---
// Block tile (WGM*WTM*16) x (WGN*WTN*16) x (32 KPS) on WGM x WGN waves, each wave
// WTM x WTN MFMA tiles.  Both operands are staged in LDS in fragment order; the
// padding of W to 32 k holds zeros, so k past the end of A only has to be
// readable: what it multiplies is zero.  The copies global -> LDS are done by
// the load unit itself (global_load_lds_dwordx4: every lane's 16 bytes land at
// LDS base + lane * 16, which is exactly fragment order), so no register and no
// LDS store instruction is spent on staging, and STAGES - 1 tiles are in flight
// while one is worked on.
// A wave waits for its own copies of the tile it is about to read
// (s_waitcnt vmcnt), the barrier that follows makes the other waves' visible.
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* glb_ptr_t;

constexpr int vmcnt_imm(int v) { return (v & 15) | (7 << 4) | (15 << 8) | ((v >> 4) << 14); }

template <int WGM, int WGN, int WTM, int WTN, int STAGES, bool GLU, typename TC, int KPS = 2, bool EARLY = false>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_bf16_async_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Wp, TC* __restrict__ C, int M, int N,
    int K, int lda, int KB, int n_out, float* __restrict__ part) {
    // WGM x WGN waves, each WTM x WTN MFMA tiles of 16 x 16
    constexpr int NW = WGM * WGN;
    constexpr int BM = WGM * WTM * 16, BN = WGN * WTN * 16;
    constexpr int AF = BM / 16 * KPS, WF = BN / 16 * KPS;   // fragments per operand tile (KPS k-steps of 32)
    constexpr int FR = AF + WF;                          // fragments per stage, 1 KB each
    // copies a wave issues per tile: fragment wave + NW j is copy j of a wave; where the fragments
    // do not go round evenly the last waves copy the last fragment once more (same bytes to the
    // same place), so that every wave has the same number of copies in flight
    constexpr int LPW = (FR + NW - 1) / NW;
    static_assert((STAGES - 2) * LPW < 64, "vmcnt has 6 bits");
    __shared__ __attribute__((aligned(1024))) bf16_t smem[STAGES * FR * 512];
    const int tid = threadIdx.x;
    // (the wave's index as a scalar: what follows from it, the fragments it copies and where they
    // land in LDS, is then worked out by the scalar unit)
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int fr = lane & 15, fg = lane >> 4;
    // Blocks are handed to the eight XCDs in turn, and each XCD has an L2 of its own: block b
    // of the launch runs on XCD b % 8.  Row tiles are taken in groups of eight; within a group
    // the tiles are numbered column tile by column tile, and XCD x works through the x-th
    // eighth of that sequence one after the other: with 32 blocks of an XCD in flight these are
    // four column tiles by eight row tiles, a tile of W is fetched into one L2 only (two at the
    // seam of two eighths) and the (smaller) A is what every L2 holds.  A full group gives
    // every XCD exactly TN tiles whatever TN is; only the last, smaller group pads the launch.
    const int TM = (M + BM - 1) / BM, TN = (N + BN - 1) / BN;
    const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
    const int full = (TM >> 3) * TN;           // blocks an XCD runs for the full groups
    int grp, grp_rows, j;
    if (seq < full) {
        grp = seq / TN;
        grp_rows = 8;
        j = xcd * TN + (seq - grp * TN);
    } else {
        grp = TM >> 3;
        grp_rows = TM & 7;
        const int per = (grp_rows * TN + 7) >> 3;
        j = xcd * per + (seq - full);
        if (seq - full >= per || j >= grp_rows * TN) return;   // the launch is padded to eight equal shares
    }
    const int tn = j / grp_rows, tm = grp * 8 + j % grp_rows;
    const int m0 = tm * BM, n0 = tn * BN;
    const int NB = (N + 15) / 16;
    const int nk = (K + 32 * KPS - 1) / (32 * KPS);
    // With gridDim.z > 1 the blocks of one tile split K among them and leave partial sums in
    // part[z][M][N], which a second kernel adds up in a fixed order.
    const int kt_per = (nk + (int)gridDim.z - 1) / (int)gridDim.z;
    const int kt0 = (int)blockIdx.z * kt_per;
    const int kt1 = min(nk, kt0 + kt_per);

    floatx4 acc[WTN][WTM];
#pragma unroll
    for (int i = 0; i < WTN; ++i)
#pragma unroll
        for (int j = 0; j < WTM; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    // this wave's copies: fragments f = wave + NW j of a stage; f < AF is of A, else of W
    const bf16_t* src[LPW];
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
        const int f = min(wave + NW * j, FR - 1);
        if (f < AF) {
            const int row = min(m0 + (f / KPS) * 16 + fr, M - 1);   // rows past the end repeat the last
            src[j] = A + (size_t)row * lda;
        } else {
            const int nb = min(n0 / 16 + (f - AF) / KPS, NB - 1);
            src[j] = Wp + (size_t)nb * KB * 512 + lane * 8;
        }
    }
    // Tiles past the end are copied too (as the last tile, into stages nobody reads any more):
    // then the number of copies in flight is the same in every iteration and one constant wait
    // covers them all.
#define TFF_ISSUE_TILE(tile)                                                                       \
    {                                                                                              \
        const int kt_ = min((tile), nk - 1);                                                       \
        const int st_ = ((tile) - kt0) % STAGES;                                                   \
        _Pragma("unroll") for (int j = 0; j < LPW; ++j) {                                          \
            const int f = min(wave + NW * j, FR - 1);                                               \
            const bf16_t* g_;                                                                      \
            if (f < AF) g_ = src[j] + min((kt_ * KPS + f % KPS) * 32 + fg * 8, K - 8);                 \
            else g_ = src[j] + (size_t)min(KPS * kt_ + (f - AF) % KPS, KB - 1) * 512;                  \
            copy16_to_lds(g_, smem + (st_ * FR + f) * 512);                                        \
        }                                                                                          \
    }

#pragma unroll
    for (int t = 0; t < STAGES - 1; ++t) TFF_ISSUE_TILE(kt0 + t)
    if constexpr (EARLY) {
        // The barrier stands between a tile's LDS reads and its MFMAs: a wave arrives with its
        // operands on the way, and when the barrier opens every wave can start its MFMAs at once
        // (with the barrier before the reads, all waves read at the same time and the matrix
        // cores wait for the first operands after every barrier).  The barrier of tile kt makes
        // tile kt + 1 visible, so the copies have to be one tile further ahead.
        static_assert(KPS == 1 && STAGES >= 3, "one k-step a tile, three stages or more");
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * LPW));
        __syncthreads();
        for (int kt = kt0; kt < kt1; ++kt) {
            const bf16_t* st = smem + ((kt - kt0) % STAGES) * FR * 512;
            bf16x8 fw[WTN], fa[WTM];
#pragma unroll
            for (int i = 0; i < WTN; ++i)
                fw[i] = *reinterpret_cast<const bf16x8*>(st + (AF + wn * WTN + i) * 512 + lane * 8);
#pragma unroll
            for (int j = 0; j < WTM; ++j)
                fa[j] = *reinterpret_cast<const bf16x8*>(st + (wm * WTM + j) * 512 + lane * 8);
            __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 3) * LPW));   // this wave's part of tile kt + 1 is in
            asm volatile("s_barrier" ::: "memory");
            TFF_ISSUE_TILE(kt + STAGES - 1)                              // into the stage of tile kt - 1
            if (kt < KB) {
#pragma unroll
                for (int i = 0; i < WTN; ++i)
#pragma unroll
                    for (int j = 0; j < WTM; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[i], fa[j], acc[i][j], 0, 0, 0);
            }
        }
    } else
    for (int kt = kt0; kt < kt1; ++kt) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * LPW));   // this wave's part of tile kt is in
        __syncthreads();                                             // ... and everybody else's
        TFF_ISSUE_TILE(kt + STAGES - 1)                              // into the stage read last iteration
        const bf16_t* st = smem + ((kt - kt0) % STAGES) * FR * 512;
#pragma unroll
        for (int ks = 0; ks < KPS; ++ks) {
            if (KPS * kt + ks < KB) {   // k-steps past the end of K are not in W
                bf16x8 fw[WTN], fa[WTM];
#pragma unroll
                for (int i = 0; i < WTN; ++i)
                    fw[i] = *reinterpret_cast<const bf16x8*>(st + (AF + (wn * WTN + i) * KPS + ks) * 512 + lane * 8);
#pragma unroll
                for (int j = 0; j < WTM; ++j)
                    fa[j] = *reinterpret_cast<const bf16x8*>(st + ((wm * WTM + j) * KPS + ks) * 512 + lane * 8);
#pragma unroll
                for (int i = 0; i < WTN; ++i)
#pragma unroll
                    for (int j = 0; j < WTM; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[i], fa[j], acc[i][j], 0, 0, 0);
            }
        }
    }
#undef TFF_ISSUE_TILE
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));   // the copies past the end must not outlive the block

    if (part) {   // partial sums over this block's share of K, columns as W has them
        float* P = part + (size_t)blockIdx.z * M * N;
        const bool vec = (N % 4) == 0;
#pragma unroll
        for (int i = 0; i < WTN; ++i) {
            const int n = n0 + (wn * WTN + i) * 16 + fg * 4;
#pragma unroll
            for (int j = 0; j < WTM; ++j) {
                const int m = m0 + (wm * WTM + j) * 16 + fr;
                if (m < M && n < N) store4<float>(P + (size_t)m * N + n, acc[i][j], n, N, vec);
            }
        }
        return;
    }
    if constexpr (GLU) {
        static_assert(WTN % 2 == 0, "gate and up groups come in pairs");
        const bool vec = (n_out % 4) == 0;
#pragma unroll
        for (int i = 0; i < WTN; i += 2) {
            const int n = (n0 + (wn * WTN + i) * 16) / 2 + fg * 4;
#pragma unroll
            for (int j = 0; j < WTM; ++j) {
                const int m = m0 + (wm * WTM + j) * 16 + fr;
                if (m < M && n < n_out)
                    store4<TC>(C + (size_t)m * n_out + n, silu_mul(acc[i][j], acc[i + 1][j]), n, n_out, vec);
            }
        }
    } else {
        const bool vec = (N % 4) == 0;
#pragma unroll
        for (int i = 0; i < WTN; ++i) {
            const int n = n0 + (wn * WTN + i) * 16 + fg * 4;
#pragma unroll
            for (int j = 0; j < WTM; ++j) {
                const int m = m0 + (wm * WTM + j) * 16 + fr;
                if (m < M && n < N) store4<TC>(C + (size_t)m * N + n, acc[i][j], n, N, vec);
            }
        }
    }
}

// Adds up the partial sums part[s][M][N] of a product whose blocks split K, s = 0, 1, ... in
// turn, and writes C; with GLU, columns come as gate and up groups of 16 in turn and
// C[m][j] = silu(gate) * up.  One thread makes four neighbouring outputs.
template <bool GLU, typename TC>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* __restrict__ part, int S,
                                                                  int M, int N, TC* __restrict__ C,
                                                                  int n_out) {
    const int per_row = (n_out + 3) / 4;
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)M * per_row) return;
    const int m = (int)(idx / per_row), j = (int)(idx % per_row) * 4;
    const size_t plane = (size_t)M * N;
    floatx4 a = floatx4{0.f, 0.f, 0.f, 0.f}, b = a;
    if constexpr (GLU) {
        const int c = (j >> 4) * 32 + (j & 15);   // N is a multiple of 32 here: whole float4s
        const float* p = part + (size_t)m * N + c;
        for (int s = 0; s < S; ++s, p += plane) {
            const float4 g = *reinterpret_cast<const float4*>(p);
            const float4 u = *reinterpret_cast<const float4*>(p + 16);
            a[0] += g.x; a[1] += g.y; a[2] += g.z; a[3] += g.w;
            b[0] += u.x; b[1] += u.y; b[2] += u.z; b[3] += u.w;
        }
        a = silu_mul(a, b);
    } else {
        const float* p = part + (size_t)m * N + j;
        const bool vec = (N % 4) == 0;
        for (int s = 0; s < S; ++s, p += plane) {
            if (vec) {
                const float4 v = *reinterpret_cast<const float4*>(p);
                a[0] += v.x; a[1] += v.y; a[2] += v.z; a[3] += v.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (j + e < N) a[e] += p[e];
            }
        }
    }
    store4<TC>(C + (size_t)m * n_out + j, a, j, n_out, (n_out % 4) == 0);
}

// splits > 1: the blocks of a tile split K among them; part holds splits * M * N floats
template <int WGM, int WGN, int WTM, int WTN, int STAGES, bool GLU = false, int KPS = 2, bool EARLY = false>
static int launch_async_g(const bf16_t* A, const bf16_t* Wp, void* C, int M, int N, int K, int lda,
                          int c_dtype, int n_out, hipStream_t s, int splits = 1, float* part = nullptr,
                          bool reduce = true) {
    const int KB = (K + 31) / 32;
    constexpr int BM = WGM * WTM * 16, BN = WGN * WTN * 16;
    if (splits <= 1 || !part) { splits = 1; part = nullptr; }
    const long TM = (M + BM - 1) / BM, TN = (N + BN - 1) / BN;
    const long tiles = 8 * ((TM / 8) * TN + ((TM % 8) * TN + 7) / 8);   // eight equal shares, see the kernel
    TFF_REQUIRE(tiles < (1L << 31), "gemm: too many tiles for M=%d N=%d", M, N);
    const dim3 grid((unsigned)tiles, 1, splits);
    if (c_dtype == TFF_F32)
        gemm_bf16_async_kernel<WGM, WGN, WTM, WTN, STAGES, GLU, float, KPS, EARLY>
            <<<grid, 64 * WGM * WGN, 0, s>>>(A, Wp, (float*)C, M, N, K, lda, KB, n_out, part);
    else
        gemm_bf16_async_kernel<WGM, WGN, WTM, WTN, STAGES, GLU, bf16_t, KPS, EARLY>
            <<<grid, 64 * WGM * WGN, 0, s>>>(A, Wp, (bf16_t*)C, M, N, K, lda, KB, n_out, part);
    if (int rc = tff_check_launch("gemm_bf16_async")) return rc;
    if (splits > 1 && reduce) {
        const int No = GLU ? n_out : N;
        const long threads = (long)M * ((No + 3) / 4);
        const int blocks = (int)((threads + 255) / 256);
        if (c_dtype == TFF_F32)
            gemm_splitk_reduce_kernel<GLU, float><<<blocks, 256, 0, s>>>(part, splits, M, N, (float*)C, No);
        else
            gemm_splitk_reduce_kernel<GLU, bf16_t><<<blocks, 256, 0, s>>>(part, splits, M, N, (bf16_t*)C, No);
        return tff_check_launch("gemm_splitk_reduce");
    }
    return 0;
}

// ------------------------------------------- four waves, whole cache lines ---
// Block tile 256 x (32 WTN) on 2 x 2 waves (or 128 x (64 WTN) on 1 x 4, for products of few rows,
// whose time is the weight's stream: all four waves then read the same rows of A), one wave to a
// SIMD, each wave 8 x WTN MFMA tiles: half the LDS reads per MFMA of sixteen waves of 64 x 64.  With one wave to a SIMD nothing overlaps unless
// the wave interleaves it itself: the fragments of k-tile t + 1 are read from LDS into a second set
// of registers, and the copies of later tiles are issued, between the MFMAs of k-tile t.
//
// What bounds this product is the number of requests to L2, not their bytes: a row-major A read 32 k
// at a time is 64 bytes a row, half a cache line a request.  So A is copied 64 k at a time, eight
// rows x 128 bytes a copy (a unit of two k-tiles, NA = 3 of them in LDS), W 32 k at a time as it is
// packed (NWS k-tiles in LDS).  Within a copy's 1 KB lane i lands at byte 16 i; it fetches row
// i / 8, 16-byte chunk (i % 8) ^ (i / 8), so that the sixteen rows an MFMA operand is made of are
// read back from different banks.
// In k-tile t (32 k) a wave issues, if t is even, its copies of A unit t / 2 + 2, and its copies of W
// tile t + NWS - 1; at the start of t it needs W tile t + 1 and the A unit of t + 1, issued in tile
// t - NWS + 2 at the latest.  Copies complete in the order issued, so the wait is by count.
// K a multiple of 64; a split of K takes whole units.
__device__ __forceinline__ void mfma_acc(floatx4& c, const bf16x8& a, const bf16x8& b) {
    // accumulate in place, in the accumulation registers, as the instruction itself says it: through
    // the builtin the register allocator moves accumulators between the two files around every MFMA
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void copy16_to_lds_sbase(unsigned long long base, unsigned lane_off, unsigned lds_wave_addr) {
    // the address is a uniform base and a 32-bit offset per lane: walking k is scalar work
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_wave_addr), "v"(lane_off), "s"(base)
                 : "memory", "m0");
}

// The lane's index, taken where it is asked for: what the epilogue works out from it is then worked out
// after the main loop, where there are registers for it, instead of before it and kept (or spilled) across.
__device__ __forceinline__ int w4_lane() {
    int lane;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
    return lane;
}

// A wave's 128 rows x OW column groups of results go out through LDS, so that a store instruction
// writes whole rows instead of 16 rows x 8 or 16 bytes: a lane leaves its four columns of a row in
// the wave's own region of LDS (rows padded by 16 bytes against bank conflicts) and takes 16 bytes
// of a row back.  Only this wave touches the region, LDS works through a wave's accesses in order,
// so no barrier is needed within; RC of the 8 row groups go through at a time, as many as the
// region holds.  A store instruction takes 64 / LPR rows, LPR lanes to a row (the power of two that
// holds a row's 16-byte pieces; the lanes beyond them idle), so that the address of a lane's store
// is that of its last one plus a constant.  vec: the rows of the result are a multiple of 16 bytes
// long, the 16 bytes are one store; otherwise they go out element by element (slow, and rare: a
// width that is no multiple of 8).  This is the kernel's only way out for its results on purpose:
// with a second one beside it the compiler converts accumulators for both before the branch, runs
// out of registers and spills, and a kernel that uses scratch memory pays some 15 us at its launch.
template <int OW, int REGION, typename TO, int WTM = 8, typename F>
__device__ __forceinline__ void w4_store_rows(char* region, F val, TO* out, size_t ld, int m_base, int n_base,
                                              int M, int ncols, int lane, bool vec) {
    constexpr int E = 16 / (int)sizeof(TO);           // columns in 16 bytes
    constexpr int RB = OW * 16 * (int)sizeof(TO), RBP = RB + 16, CPR = RB / 16;
    constexpr int LPR = CPR <= 4 ? 4 : CPR <= 8 ? 8 : CPR <= 16 ? 16 : 32;   // lanes a row
    static_assert(CPR <= LPR, "a row's pieces fit its lanes");
    constexpr int RPI = 64 / LPR;                     // rows a store instruction
    constexpr int RC = WTM * 16 * RBP <= REGION ? WTM : WTM / 2;   // row groups that go through the region at a time
    static_assert(RC >= 1 && RC * 16 * RBP <= REGION, "the wave's region of LDS holds half its row groups at least");
    const int fr = lane & 15, fg = lane >> 4;
    const int srow = lane / LPR, sch = lane % LPR;    // this lane's row of an instruction's, and its piece
    const int n = n_base + sch * E;
    const bool mine = sch < CPR && n < ncols;
    const char* src = region + srow * RBP + sch * 16;
#pragma unroll
    for (int p = 0; p < WTM / RC; ++p) {
#pragma unroll
        for (int jj = 0; jj < RC; ++jj) {
            __builtin_amdgcn_sched_barrier(0);   // a row group at a time: all accumulators converted at once do not fit the registers
#pragma unroll
            for (int i = 0; i < OW; ++i) {
                const floatx4 v = val(i, p * RC + jj);
                char* dst = region + (jj * 16 + fr) * RBP + (i * 16 + fg * 4) * (int)sizeof(TO);
                if constexpr (sizeof(TO) == 4) {
                    *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
                } else {
                    union { bf16_t h[4]; uint2 u; } pk;
#pragma unroll
                    for (int e = 0; e < 4; ++e) pk.h[e] = (bf16_t)v[e];
                    *reinterpret_cast<uint2*>(dst) = pk.u;
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        int m = m_base + p * RC * 16 + srow;
        TO* dst = out + (size_t)m * ld + n;
        if (vec) {   // (the branch outside the loop: its reads of LDS are then issued together, not one per store)
#pragma unroll
            for (int t = 0; t < RC * 16 / RPI; ++t) {
                const uint4 v = *reinterpret_cast<const uint4*>(src + t * RPI * RBP);
                if (mine && m < M) *reinterpret_cast<uint4*>(dst) = v;
                m += RPI;
                dst += (size_t)RPI * ld;
            }
        } else {
            for (int t = 0; t < RC * 16 / RPI; ++t) {
                union { uint4 u; TO e[E]; } v;
                v.u = *reinterpret_cast<const uint4*>(src + t * RPI * RBP);
                if (mine && m < M) {
#pragma unroll
                    for (int e = 0; e < E; ++e)
                        if (n + e < ncols) dst[e] = v.e[e];
                }
                m += RPI;
                dst += (size_t)RPI * ld;
            }
        }
    }
}

// SCALE: A's rows (up to 16 of them) still lack the factor of the RMS norm they went through; the
// factor, rsqrt(sum of the row's sums of squares / dim + eps), is applied to the accumulators.
struct W4Scale {
    const float* ss;        // [16][stride] sums of squares, count of them a row
    int stride, count;
    float inv_dim, eps;
};
template <int WTN, int NWS, bool GLU, typename TC, int WGM = 2, bool SCALE = false, int WTM = 8>
__global__ __launch_bounds__(256) void gemm_bf16_w4_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Wp, TC* __restrict__ C, int M, int N,
    int K, int lda, int KB, int n_out, W4Scale sc) {
    static_assert(!SCALE || WGM == 1, "rows that lack their norm's factor: up to 16, one row tile");
    // WGM: waves along the rows, 2 (a block tile of 256 rows, two waves side by side) or 1 (128 rows, four side by side)
    // WTM: row groups of 16 a wave, 8, or with the waves side by side 4 or 2 (a block tile of 64 or 32 rows)
    constexpr int NW = 4, NA = 3, WGN = NW / WGM;
    static_assert(WGM == 1 || WGM == 2, "four waves as 2 x 2 or 1 x 4");
    static_assert(WTM == 8 || (WGM == 1 && (WTM == 4 || WTM == 2)), "fewer rows a wave only with the waves side by side");
    constexpr int BM = WGM * WTM * 16, BN = WGN * WTN * 16;
    constexpr int WF = BN / 16;                       // W fragments a k-tile, 1 KB each
    constexpr int ACP = BM / 8;                       // A copies a unit, 1 KB each
    constexpr int LPA = ACP / NW, LPW = (WF + NW - 1) / NW;
    constexpr int NMF = WTM * WTN;                    // MFMAs a k-tile
    constexpr int RPM = NMF / (WTM + WTN);            // a read after every RPM MFMAs
    constexpr int CPM = NMF / (LPA + LPW);            // a copy after every CPM MFMAs
    constexpr int D = NWS - 1;                        // W is copied D tiles ahead
    static_assert(D == 3 || D == 4, "the waits below are written for three or four tiles ahead");
    static_assert(RPM >= 1 && CPM >= 1, "not enough MFMAs to hide the reads and copies");
    constexpr unsigned A_UNIT = ACP * 1024u, W_TILE = WF * 1024u, W_BASE = NA * A_UNIT;
    static_assert(W_BASE + NWS * W_TILE <= 160 * 1024, "LDS");
    __shared__ __attribute__((aligned(1024))) char smem[W_BASE + NWS * W_TILE];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = WGM == 2 ? wave >> 1 : 0, wn = WGM == 2 ? wave & 1 : wave;
    const int fr = lane & 15, fg = lane >> 4;
    const int TM = (M + BM - 1) / BM, TN = (N + BN - 1) / BN;
    const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
    const int full = (TM >> 3) * TN;
    int grp, grp_rows, j;
    if (seq < full) {
        grp = seq / TN;
        grp_rows = 8;
        j = xcd * TN + (seq - grp * TN);
    } else {
        grp = TM >> 3;
        grp_rows = TM & 7;
        const int per = (grp_rows * TN + 7) >> 3;
        j = xcd * per + (seq - full);
        if (seq - full >= per || j >= grp_rows * TN) return;
    }
    const int tn = j / grp_rows, tm = grp * 8 + j % grp_rows;
    const int m0 = tm * BM, n0 = tn * BN;
    const int NB = (N + 15) / 16;
    const int nu = KB / 2;                            // units of 64 k
    const int u_per = (nu + (int)gridDim.z - 1) / (int)gridDim.z;
    const int u0 = (int)blockIdx.z * u_per;
    const int u1 = min(nu, u0 + u_per);
    const int kt0 = 2 * u0, kt1 = 2 * u1;

    floatx4 acc[WTN][WTM];
#pragma unroll
    for (int i = 0; i < WTN; ++i)
#pragma unroll
        for (int jj = 0; jj < WTM; ++jj) acc[i][jj] = floatx4{0.f, 0.f, 0.f, 0.f};
    // (a lane's results are four columns of row fr of each row group: of row fr itself in the first,
    // the only one that counts with up to 16 rows; the four lanes of a row share out its sums)
    float row_ss = 0.f;
    if constexpr (SCALE) {
        // (16 bytes a load, eight loads asked for before the first is added: one trip to memory for rows of up to 8,192 elements)
        const float* sp = sc.ss + (size_t)fr * sc.stride;
        const int vec_end = sc.count & ~3;
        for (int j0 = fg * 4; j0 < vec_end; j0 += 16 * 8) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                v[u] = j0 + 16 * u < vec_end ? *reinterpret_cast<const float4*>(sp + j0 + 16 * u) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int u = 0; u < 8; ++u) row_ss += (v[u].x + v[u].y) + (v[u].z + v[u].w);
        }
        if (fg == 0)
            for (int j = vec_end; j < sc.count; ++j) row_ss += sp[j];
    }

    // this wave's copies: of an A unit the copies wave + 4 c, of a W tile the fragments wave + 4 c
    unsigned long long abase[LPA], wbase[LPW];
    unsigned aoff[LPA];
    unsigned wlds[LPW];
    const unsigned woff = lane * 16;
#pragma unroll
    for (int c = 0; c < LPA; ++c) {
        const int cp = wave + NW * c;
        const int row0 = min(m0 + cp * 8, M - 1);
        const int row = min(m0 + cp * 8 + (lane >> 3), M - 1);
        abase[c] = (unsigned long long)(A + (size_t)row0 * lda + (size_t)kt0 * 32);
        aoff[c] = (unsigned)(row - row0) * (unsigned)lda * 2u + (unsigned)(((lane & 7) ^ (lane >> 3)) * 16);
    }
#pragma unroll
    for (int c = 0; c < LPW; ++c) {
        const int f = min(wave + NW * c, WF - 1);     // the last waves copy the last fragment once more
        const int nb = min(n0 / 16 + f, NB - 1);
        wbase[c] = (unsigned long long)(Wp + ((size_t)nb * KB + kt0) * 512);
        wlds[c] = W_BASE + (unsigned)f * 1024u;
    }
    const unsigned smem_addr = (unsigned)(size_t)(lds_ptr_t)smem;
    // copies past the end repeat the last unit or tile, so that the counts in flight stay the same
    int a_next = u0, w_next = kt0;                    // the next unit and tile to copy
    unsigned a_ws = 0, w_ws = 0;                      // where they go: byte offsets of the slots
#define W4_COPY_A(c)                                                                                \
    {                                                                                               \
        copy16_to_lds_sbase(abase[c], aoff[c], smem_addr + a_ws + (unsigned)(wave + NW * (c)) * 1024u); \
        abase[c] += a_next + 1 < u1 ? 128ull : 0ull;                                                \
    }
#define W4_A_ISSUED()                                                                               \
    {                                                                                               \
        a_next += a_next + 1 < u1 ? 1 : 0;                                                          \
        a_ws = a_ws + A_UNIT == NA * A_UNIT ? 0u : a_ws + A_UNIT;                                   \
    }
#define W4_COPY_W(c)                                                                                \
    {                                                                                               \
        copy16_to_lds_sbase(wbase[c], woff, smem_addr + w_ws + wlds[c]);                            \
        wbase[c] += w_next + 1 < kt1 ? 1024ull : 0ull;                                              \
    }
#define W4_W_ISSUED()                                                                               \
    {                                                                                               \
        w_next += w_next + 1 < kt1 ? 1 : 0;                                                         \
        w_ws = w_ws + W_TILE == NWS * W_TILE ? 0u : w_ws + W_TILE;                                  \
    }
    if (u0 < u1) {   // (a part of a split K that holds no unit only stores its zeros)
        // the tiles before the first, in the order of the loop: t = -4 .. -1
#pragma unroll
        for (int t = -4; t < 0; ++t) {
            if ((t & 1) == 0) {
#pragma unroll
                for (int c = 0; c < LPA; ++c) W4_COPY_A(c)
                W4_A_ISSUED()
            }
            if (t + D >= 0) {
#pragma unroll
                for (int c = 0; c < LPW; ++c) W4_COPY_W(c)
                W4_W_ISSUED()
            }
        }
        // what may still be in flight at the start of tile t: the copies of tiles t - D + 2 .. t - 1
        constexpr int EVEN = LPA + LPW, ODD = LPW;
        constexpr int FLY_E = D == 4 ? EVEN + ODD : ODD;  // t even: t - 1 is odd
        constexpr int FLY_O = D == 4 ? EVEN + ODD : EVEN;
        // a lane's 16 bytes of an A operand: row fr of 16, chunk h * 4 + fg of the row's 8
        unsigned a_rd[2];
#pragma unroll
        for (int h = 0; h < 2; ++h)
            a_rd[h] = (unsigned)(wm * WTM * 2 + (fr >> 3)) * 1024u + (unsigned)(((fr & 7) * 8 + ((h * 4 + fg) ^ (fr & 7))) * 16);
        const unsigned w_rd = W_BASE + (unsigned)(wn * WTN) * 1024u + lane * 16;
        unsigned a_rs = 0, w_rs = W_TILE;                 // slots of the tile whose fragments are read next (kt0 + 1)
        // before the first tile: A unit u0 and W tile kt0, issued in tile -4 and tile -D
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(D == 4 ? LPA + 3 * LPW : LPA + 2 * LPW));
        __syncthreads();
        bf16x8 fw[2][WTN], fa[2][WTM];
#pragma unroll
        for (int i = 0; i < WTN; ++i) fw[0][i] = *reinterpret_cast<const bf16x8*>(smem + w_rd + i * 1024);
#pragma unroll
        for (int jj = 0; jj < WTM; ++jj) fa[0][jj] = *reinterpret_cast<const bf16x8*>(smem + a_rd[0] + jj * 2048);

        // a k-tile's MFMAs with the LDS reads of the next tile and the copies of later ones between them
#define W4_TILE(h)                                                                                  \
        {                                                                                           \
            __builtin_amdgcn_s_waitcnt(vmcnt_imm((h) ? FLY_O : FLY_E));                             \
            asm volatile("s_barrier" ::: "memory");                                                 \
            const char* na = smem + a_rs + a_rd[(h) ^ 1];                                           \
            const char* nw = smem + w_rs + w_rd;                                                    \
            _Pragma("unroll") for (int i = 0; i < WTN; ++i)                                         \
                _Pragma("unroll") for (int jj = 0; jj < WTM; ++jj) {                                \
                    const int q = i * WTM + jj;                                                     \
                    mfma_acc(acc[i][jj], fw[h][i], fa[h][jj]);                                      \
                    if (q % RPM == RPM - 1 && q / RPM < WTN + WTM) {                                \
                        const int rd = q / RPM;                                                     \
                        if (rd < WTM) fa[(h) ^ 1][rd < WTM ? rd : 0] = *reinterpret_cast<const bf16x8*>(na + rd * 2048); \
                        else fw[(h) ^ 1][rd >= WTM ? rd - WTM : 0] = *reinterpret_cast<const bf16x8*>(nw + (rd - WTM) * 1024); \
                    }                                                                               \
                    if (q % CPM == CPM - 1) {                                                       \
                        const int cp = q / CPM;                                                     \
                        if ((h) == 0) {                                                             \
                            if (cp < LPA) W4_COPY_A(cp < LPA ? cp : 0)                              \
                            else if (cp < LPA + LPW) W4_COPY_W(cp >= LPA && cp < LPA + LPW ? cp - LPA : 0) \
                        } else if (cp < LPW) W4_COPY_W(cp < LPW ? cp : 0)                           \
                    }                                                                               \
                }                                                                                   \
            if ((h) == 0) W4_A_ISSUED()                                                             \
            W4_W_ISSUED()                                                                           \
            if ((h) == 0) a_rs = a_rs + A_UNIT == NA * A_UNIT ? 0u : a_rs + A_UNIT;                 \
            w_rs = w_rs + W_TILE == NWS * W_TILE ? 0u : w_rs + W_TILE;                              \
        }
        // tile 2 u reads its successor from its own unit, tile 2 u + 1 from the next: a_rs moves on after an even tile
        for (int kt = kt0; kt < kt1; kt += 2) {
            W4_TILE(0)
            W4_TILE(1)
        }
    }
#undef W4_TILE
#undef W4_COPY_A
#undef W4_COPY_W
#undef W4_A_ISSUED
#undef W4_W_ISSUED
    // every copy has landed and every read of LDS has come back, in every wave: LDS is free for the results
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");   // (and the last MFMAs have written their accumulators)
    __syncthreads();
    constexpr int REGION = (int)((W_BASE + NWS * W_TILE) / 4) & ~1023;
    char* region = smem + wave * REGION;
    const int mw = m0 + wm * WTM * 16;                // the wave's first row
    constexpr int E = 16 / (int)sizeof(TC);
    const int lane_out = w4_lane();
    float rs = 1.f;
    if constexpr (SCALE) {
        row_ss += __shfl_xor(row_ss, 16, 64);
        row_ss += __shfl_xor(row_ss, 32, 64);
        rs = rsqrtf(row_ss * sc.inv_dim + sc.eps);
    }
    auto scaled = [&](const floatx4& v) {
        if constexpr (SCALE) return floatx4{v[0] * rs, v[1] * rs, v[2] * rs, v[3] * rs};
        else return v;
    };
    if constexpr (GLU) {
        static_assert(WTN % 2 == 0, "gate and up groups come in pairs");
        w4_store_rows<WTN / 2, REGION, TC, WTM>(region, [&](int i, int jj) { return silu_mul(scaled(acc[2 * i][jj]), scaled(acc[2 * i + 1][jj])); },
                                           C, (size_t)n_out, mw, (n0 + wn * WTN * 16) / 2, M, n_out, lane_out,
                                           n_out % E == 0);
    } else {
        // (partial sums of a split K: plane blockIdx.z of the launcher's float32 workspace, which it passes as C)
        TC* out = C + (size_t)blockIdx.z * M * N;
        w4_store_rows<WTN, REGION, TC, WTM>(region, [&](int i, int jj) { return scaled(acc[i][jj]); }, out, (size_t)N, mw,
                                       n0 + wn * WTN * 16, M, N, lane_out, N % E == 0);
    }
}

// splits > 1: the blocks of a tile split K among them in units of 64; part holds splits * M * N floats
template <int WTN, int NWS, bool GLU = false, int WGM = 2, bool SCALE = false, int WTM = 8>
static int launch_w4(const bf16_t* A, const bf16_t* Wp, void* C, int M, int N, int K, int lda, int c_dtype,
                     int n_out, hipStream_t s, int splits = 1, float* part = nullptr, bool reduce = true,
                     W4Scale sc = W4Scale{nullptr, 0, 0, 0.f, 0.f}) {
    TFF_REQUIRE(!SCALE || (M <= 16 && sc.ss && (splits <= 1 || !part)),
                "gemm: rows that lack their norm's factor: up to 16 of them and K in one part");
    TFF_REQUIRE(K % 64 == 0, "gemm: the four-wave tiles take K in units of 64, not K=%d", K);
    const int KB = K / 32;
    constexpr int BM = 16 * WTM * WGM, BN = (4 / WGM) * WTN * 16;
    if (splits <= 1 || !part) { splits = 1; part = nullptr; }
    TFF_REQUIRE(splits <= KB / 2, "gemm: %d parts of %d units of K", splits, KB / 2);
    const long TM = (M + BM - 1) / BM, TN = (N + BN - 1) / BN;
    const long tiles = 8 * ((TM / 8) * TN + ((TM % 8) * TN + 7) / 8);   // eight equal shares, see the kernel
    TFF_REQUIRE(tiles < (1L << 31), "gemm: too many tiles for M=%d N=%d", M, N);
    TFF_REQUIRE((size_t)15 * lda * 2 + 128 < (1ull << 32), "gemm: row stride %d too large", lda);
    const dim3 grid((unsigned)tiles, 1, splits);
    // the blocks of a split K leave plain float32 sums, plane by plane; a gate is applied when they are added up
    if (splits > 1)
        gemm_bf16_w4_kernel<WTN, NWS, false, float, WGM, false, WTM><<<grid, 256, 0, s>>>(A, Wp, part, M, N, K, lda, KB, 0, sc);
    else if (c_dtype == TFF_F32)
        gemm_bf16_w4_kernel<WTN, NWS, GLU, float, WGM, SCALE, WTM><<<grid, 256, 0, s>>>(A, Wp, (float*)C, M, N, K, lda, KB, n_out, sc);
    else
        gemm_bf16_w4_kernel<WTN, NWS, GLU, bf16_t, WGM, SCALE, WTM><<<grid, 256, 0, s>>>(A, Wp, (bf16_t*)C, M, N, K, lda, KB, n_out, sc);
    if (int rc = tff_check_launch("gemm_bf16_w4")) return rc;
    if (splits > 1 && reduce) {
        const int No = GLU ? n_out : N;
        const long threads = (long)M * ((No + 3) / 4);
        const int blocks = (int)((threads + 255) / 256);
        if (c_dtype == TFF_F32)
            gemm_splitk_reduce_kernel<GLU, float><<<blocks, 256, 0, s>>>(part, splits, M, N, (float*)C, No);
        else
            gemm_splitk_reduce_kernel<GLU, bf16_t><<<blocks, 256, 0, s>>>(part, splits, M, N, (bf16_t*)C, No);
        return tff_check_launch("gemm_splitk_reduce");
    }
    return 0;
}

// ------------------------------------------------------------- skinny M ---
// For a few rows of A (decoding: M = number of live requests) the product is
// a stream of W from HBM; what counts is bytes in flight, not LDS tiling.
// A block owns a slab of 16*R rows of W for the whole of K; its waves split K
// among them in contiguous runs, each wave reading its W fragments straight
// from global memory into MFMA operands and the few rows of A from cache;
// partial sums meet in LDS and are added in a fixed order, so no partial
// result goes through global memory and the result does not depend on the
// launch.  UNROLL k-steps of loads are issued before the first is used: a wave
// keeps UNROLL * (R + MT) KB in flight, which is what hides the latency of HBM.
// The block's waves form NSETS sets of KSPLIT waves: a set works on R row groups
// of W, its waves split K.  Sets walk K at the same pace, so the rows of A one
// set has fetched are in cache for the others: with many rows of A (MT > 1)
// that, not W, is most of a wave's traffic.  With GLU, sets 2p and 2p+1 hold a
// gate group and the up group that follows it in W; the epilogue writes
// silu(gate) * up.
//
// An RMS norm between two such products costs a kernel of a few microseconds for a few rows.
// Its per-row factor commutes with the product that follows it, so the two products take the
// norm between them (EPI):
//   2, the product before the norm (float32 result): its epilogue adds its result to the
//      residual stream in place, writes the sum times the norm's weight as the bfloat16 input
//      of the next product, *without* the factor rsqrt(mean of squares + eps), and leaves the
//      sum of squares of its 16 columns of every row in ss_out[row][row group];
//   1, the product after the norm: adds up the sums of squares of a row, in a fixed order, and
//      multiplies its float32 accumulators by the row's factor before anything else is done
//      to them.
// The sum of squares is over the float32 residual stream, as in the norm's own kernel.
struct SkinnyFuse {
    const float* ss_in;     // EPI 1: [16][ss_stride] sums of squares, ss_count of them a row
    int ss_stride, ss_count;
    float inv_dim, eps;     // 1 / row length of the normalised tensor
    float* resid;           // EPI 2: [M, N] float32, updated in place
    const float* norm_w;    // [N]
    bf16_t* x_out;          // [M, N]
    float* ss_out;          // [16][ss_out_stride]
    int ss_out_stride;
};

template <int MT, int R, int UNROLL, int KSPLIT, int NSETS, bool GLU, typename TC, bool RING = false, int EPI = 0>
__global__ __launch_bounds__(64 * KSPLIT * NSETS) void gemm_bf16_skinny_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Wp, TC* __restrict__ C, int M, int N,
    int K, int lda, int KB, int n_out, SkinnyFuse fz) {
    static_assert(EPI == 0 || MT == 1, "the fused norm is for up to 16 rows");
    static_assert(EPI != 2 || !GLU, "the product before a norm has a plain float32 result");
    constexpr int SK_WAVES = KSPLIT * NSETS;
    static_assert(!GLU || (R == 1 && NSETS % 2 == 0), "a gate and its up group are one row group each");
    __shared__ floatx4 part[SK_WAVES][R * MT][64];
    const int lane = threadIdx.x & 63, wave_id = threadIdx.x >> 6;
    const int set = wave_id / KSPLIT, wave = wave_id % KSPLIT;
    const int fr = lane & 15, fg = lane >> 4;
    const int NB = (N + 15) / 16;
    const int nb0 = (blockIdx.x * NSETS + set) * R;

    floatx4 acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[r][t] = floatx4{0.f, 0.f, 0.f, 0.f};

    // k-steps of 32 are dealt out to the waves in contiguous runs
    const int per = (KB + KSPLIT - 1) / KSPLIT;
    const int s_begin = wave * per;
    const int s_end = min(KB, s_begin + per);

    // Row groups past the end of W and rows past the end of A repeat the last: their results
    // are never stored, and no load of the main loop carries a predicate.
    const bf16_t* wfrag[R];
#pragma unroll
    for (int r = 0; r < R; ++r) wfrag[r] = Wp + (size_t)min(nb0 + r, NB - 1) * KB * 512 + lane * 8;
    const bf16_t* arow[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) arow[t] = A + (size_t)min(t * 16 + fr, M - 1) * lda;

    // What the epilogue needs from memory is asked for first, so that it has arrived long
    // before the stream of W ends.
    float row_scale = 1.f;
    float4 resid_in[R], normw_in[R];
#pragma unroll
    for (int r = 0; r < R; ++r) resid_in[r] = normw_in[r] = make_float4(0.f, 0.f, 0.f, 0.f);
    // EPI 1: lane (fr, fg) of a set's first wave adds every fourth group of four sums of row fr,
    // then the four lanes of a row meet: the same order in every block.  The loads are issued
    // here, ahead of the stream of W, and added up (TFF_ROW_SCALE) when that stream has ended.
    constexpr int SSV = 16;   // 16-byte loads a lane keeps: rows of up to 64 * SSV sums
    float4 ssv[EPI == 1 ? SSV : 1];
    // (the waves that write results: the first of a set, of the gate's set with GLU; rows that exist)
    const bool scales = EPI == 1 && wave == 0 && (!GLU || (set & 1) == 0) && fr < M;
    if constexpr (EPI == 1) {
        if (scales) {
            const float* sp = fz.ss_in + (size_t)fr * fz.ss_stride;
            const int vec_end = fz.ss_count & ~3;
#pragma unroll
            for (int u = 0; u < SSV; ++u) {
                const int j = fg * 4 + 16 * u;
                ssv[u] = j < vec_end ? *reinterpret_cast<const float4*>(sp + j) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    }
#define TFF_ROW_SCALE()                                                                            \
    if constexpr (EPI == 1) {                                                                      \
        if (scales) {                                                                              \
            const float* sp = fz.ss_in + (size_t)fr * fz.ss_stride;                                \
            const int vec_end = fz.ss_count & ~3;                                                  \
            float ssum = 0.f;                                                                      \
            _Pragma("unroll") for (int u = 0; u < SSV; ++u)                                        \
                if (fg * 4 + 16 * u < vec_end) ssum += (ssv[u].x + ssv[u].y) + (ssv[u].z + ssv[u].w); \
            for (int j = fg * 4 + 16 * SSV; j < vec_end; j += 16) {   /* very long rows */           \
                const float4 v = *reinterpret_cast<const float4*>(sp + j);                         \
                ssum += (v.x + v.y) + (v.z + v.w);                                                 \
            }                                                                                      \
            if (fg == 0)                                                                           \
                for (int j = vec_end; j < fz.ss_count; ++j) ssum += sp[j];                         \
            ssum += __shfl_xor(ssum, 16, 64);                                                      \
            ssum += __shfl_xor(ssum, 32, 64);                                                      \
            row_scale = rsqrtf(ssum * fz.inv_dim + fz.eps);                                        \
        }                                                                                          \
    }
    if constexpr (EPI == 2) {
        if (wave == 0) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int n = (nb0 + r) * 16 + fg * 4;
                if (fr < M && n < N) {
                    resid_in[r] = *reinterpret_cast<const float4*>(fz.resid + (size_t)fr * N + n);
                    normw_in[r] = *reinterpret_cast<const float4*>(fz.norm_w + n);
                }
            }
        }
    }

    const int full_end = min(s_end, K / 32);   // steps below K / 32 have all their 32 k in A
    int s0 = s_begin;
    if constexpr (RING) {
        // A ring of UNROLL k-steps in registers: a slot is loaded again as soon as it has been
        // used, so the wave has UNROLL * (R + MT) KB in flight from its first step to its last.
        // Loads come back in order, so the wait before a slot's use leaves the younger ones in
        // flight.  Steps past the end load the last step again and are not used.
        if (s0 < full_end) {
            uint4 rw[UNROLL][R], ra[UNROLL][MT];
            const int last = full_end - 1;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int st = min(s0 + u, last);
#pragma unroll
                for (int r = 0; r < R; ++r) rw[u][r] = ld16(wfrag[r] + (size_t)st * 512);
#pragma unroll
                for (int t = 0; t < MT; ++t) ra[u][t] = ld16(arow[t] + st * 32 + fg * 8);
            }
            for (; s0 < full_end; s0 += UNROLL) {
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    if (s0 + u < full_end) {
#pragma unroll
                        for (int r = 0; r < R; ++r)
#pragma unroll
                            for (int t = 0; t < MT; ++t)
                                acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                                    as_frag(rw[u][r]), as_frag(ra[u][t]), acc[r][t], 0, 0, 0);
                    }
                    const int st = min(s0 + UNROLL + u, last);
#pragma unroll
                    for (int r = 0; r < R; ++r) rw[u][r] = ld16(wfrag[r] + (size_t)st * 512);
#pragma unroll
                    for (int t = 0; t < MT; ++t) ra[u][t] = ld16(arow[t] + st * 32 + fg * 8);
                }
            }
            s0 = full_end;
        }
    }
    for (; !RING && s0 + UNROLL <= full_end; s0 += UNROLL) {
        uint4 rw[UNROLL][R], ra[UNROLL][MT];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
#pragma unroll
            for (int r = 0; r < R; ++r) rw[u][r] = ld16(wfrag[r] + (size_t)(s0 + u) * 512);
#pragma unroll
            for (int t = 0; t < MT; ++t) ra[u][t] = ld16(arow[t] + (s0 + u) * 32 + fg * 8);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(rw[u][r]), as_frag(ra[u][t]),
                                                                        acc[r][t], 0, 0, 0);
    }
    // what is left, a step at a time; in the last step of K some k may not exist in A
    for (; s0 < s_end; ++s0) {
        const int k = s0 * 32 + fg * 8;
        const bool kok = k < K;
        uint4 rw[R], ra[MT];
#pragma unroll
        for (int r = 0; r < R; ++r) rw[r] = ld16(wfrag[r] + (size_t)s0 * 512);
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const uint4 v = ld16(arow[t] + (kok ? k : 0));
            ra[t] = kok ? v : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < MT; ++t)
                acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(rw[r]), as_frag(ra[t]), acc[r][t], 0, 0, 0);
    }
    TFF_ROW_SCALE()
#undef TFF_ROW_SCALE
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t) part[wave_id][r * MT + t][lane] = acc[r][t];
    __syncthreads();
    if (wave == 0) {   // the first wave of every set adds up the set's partial sums, in a fixed order
        if constexpr (GLU) {
            if ((set & 1) == 0) {
                const bool vec = (n_out % 4) == 0;
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    floatx4 g = part[set * KSPLIT][t][lane], u = part[(set + 1) * KSPLIT][t][lane];
#pragma unroll
                    for (int w = 1; w < KSPLIT; ++w) {
                        const floatx4 pg = part[set * KSPLIT + w][t][lane], pu = part[(set + 1) * KSPLIT + w][t][lane];
#pragma unroll
                        for (int e = 0; e < 4; ++e) { g[e] += pg[e]; u[e] += pu[e]; }
                    }
                    if constexpr (EPI == 1) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) { g[e] *= row_scale; u[e] *= row_scale; }
                    }
                    const int n = (nb0 >> 1) * 16 + fg * 4;
                    const int m = t * 16 + fr;
                    if (m < M && n < n_out) store4<TC>(C + (size_t)m * n_out + n, silu_mul(g, u), n, n_out, vec);
                }
            }
        } else {
            const bool vec = (N % 4) == 0;
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    floatx4 v = part[set * KSPLIT][r * MT + t][lane];
#pragma unroll
                    for (int w = 1; w < KSPLIT; ++w) {
                        const floatx4 p = part[set * KSPLIT + w][r * MT + t][lane];
                        v[0] += p[0]; v[1] += p[1]; v[2] += p[2]; v[3] += p[3];
                    }
                    const int n = (nb0 + r) * 16 + fg * 4;
                    const int m = t * 16 + fr;
                    if constexpr (EPI == 1) {
                        v[0] *= row_scale; v[1] *= row_scale; v[2] *= row_scale; v[3] *= row_scale;
                    }
                    if constexpr (EPI == 2) {
                        // N is a multiple of 4 here: four columns are in or out together
                        float ss = 0.f;
                        if (m < M && n < N) {
                            const float4 sum = make_float4(resid_in[r].x + v[0], resid_in[r].y + v[1],
                                                           resid_in[r].z + v[2], resid_in[r].w + v[3]);
                            *reinterpret_cast<float4*>(fz.resid + (size_t)m * N + n) = sum;
                            union { bf16_t h[4]; uint2 u; } pk;
                            pk.h[0] = (bf16_t)(sum.x * normw_in[r].x);
                            pk.h[1] = (bf16_t)(sum.y * normw_in[r].y);
                            pk.h[2] = (bf16_t)(sum.z * normw_in[r].z);
                            pk.h[3] = (bf16_t)(sum.w * normw_in[r].w);
                            *reinterpret_cast<uint2*>(fz.x_out + (size_t)m * N + n) = pk.u;
                            ss = fmaf(sum.x, sum.x, fmaf(sum.y, sum.y, fmaf(sum.z, sum.z, sum.w * sum.w)));
                        }
                        ss += __shfl_xor(ss, 16, 64);
                        ss += __shfl_xor(ss, 32, 64);
                        if (fg == 0 && nb0 + r < NB) fz.ss_out[(size_t)fr * fz.ss_out_stride + nb0 + r] = ss;
                    } else if (m < M && n < N) {
                        store4<TC>(C + (size_t)m * N + n, v, n, N, vec);
                    }
                }
        }
    }
}

template <int MT, int R, int UNROLL, int KSPLIT, int NSETS = 1, bool GLU = false, bool RING = false, int EPI = 0>
static int launch_skinny(const bf16_t* A, const bf16_t* Wp, void* C, int M, int N, int K, int lda,
                         int c_dtype, int n_out, hipStream_t s, const SkinnyFuse* fuse = nullptr) {
    const int NB = (N + 15) / 16, KB = (K + 31) / 32;
    const int per_block = NSETS * R;
    const dim3 grid((NB + per_block - 1) / per_block);
    const SkinnyFuse fz = fuse ? *fuse : SkinnyFuse{nullptr, 0, 0, 0.f, 0.f, nullptr, nullptr, nullptr, nullptr, 0};
    if (c_dtype == TFF_F32)
        gemm_bf16_skinny_kernel<MT, R, UNROLL, KSPLIT, NSETS, GLU, float, RING, EPI>
            <<<grid, 64 * KSPLIT * NSETS, 0, s>>>(A, Wp, (float*)C, M, N, K, lda, KB, n_out, fz);
    else if constexpr (EPI != 2)
        gemm_bf16_skinny_kernel<MT, R, UNROLL, KSPLIT, NSETS, GLU, bf16_t, RING, EPI>
            <<<grid, 64 * KSPLIT * NSETS, 0, s>>>(A, Wp, (bf16_t*)C, M, N, K, lda, KB, n_out, fz);
    else
        return tff_fail("gemm: the product before a norm has a float32 result");
    return tff_check_launch("gemm_bf16_skinny");
}

// The tiled product's plan for M > 16: which tile, and into how many parts the blocks of a
// tile split K, by a small cost model (see plan_for).  With K in units of 64: the four-wave
// kernel's tiles of 256 rows (256, 192 or 128 columns), of 128 rows (384, 256 or 128 columns) and,
// up to 64 and 32 rows, of 64 and 32 rows (256 or 128 columns), and from 65 to 512 rows also
// 64 x 128 with several row tiles; otherwise the sixteen-wave kernel's tiles.
struct GemmPlan { int tile; int bn; int splits; };   // tile = rows of a block tile
// Compute units of the current device (256 on an MI355X, which the rates below were fitted on; a
// device with another count gets plans for its own number of blocks a round).  256 if it cannot
// be asked.
static int device_cus() {
    static int cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}
// Up to 16 rows, not gated: more row groups of 16 columns than CUs, but at most 1.6 times as many
// (a second round of blocks that would be less than 0.6 full): the streaming kernel then gives a block
// two row groups (skinny_for).
static bool two_row_groups(int N) {
    const int nb = (N + 15) / 16, cus = device_cus();
    return nb > cus && nb * 10 <= cus * 16;
}
// Up to 16 rows, gated: the streaming kernel's blocks each fetch all of A's rows, so its time grows
// with the rows, and with a very large weight (the 32B shape's gate+up, 262M elements, 3,200 blocks)
// that traffic shows even with one row.  The four-wave kernel's tiles of 32 rows, K in one part, take
// the same time whatever the rows, so each weight crosses over at its number of rows (us at 1 / 4 /
// 8 / 12 / 16 rows, streaming against tiles): the 32B shape 94 / 96 / 100 / 107 / 120 against 91 to
// 92; the 14B shape (1.8e8 elements) 67 / 69 / 71 / 77 / 89 against 68 to 70; the 8B shape (1.0e8)
// 36 / 37 / 37 / 40 / 44 against 39; the 4B shape (5e7) 21 / 21 / 22 / 24 / 28 against 25.
static bool few_rows_gated_on_tiles(int M, int N, int K) {
    const double w = (double)N * K;
    return K % 64 == 0 && (w >= 2.4e8 || (w >= 1.6e8 && M >= 5) || (w >= 0.9e8 && M >= 12) || (w >= 0.45e8 && M >= 14));
}
// One row tile of 32 rows, K in one part: the width (128 or 256 columns) that plan_for's model prices lowest.
static int plan_rows32(int N, int K) {
    const double CUS = (double)device_cus();
    const int widths[2] = {128, 256};
    const double rates[2] = {1.3e6, 1.4e6};
    int best = 256;
    double best_t = 1e30;
    for (int i = 0; i < 2; ++i) {
        const double blocks = (double)((N + widths[i] - 1) / widths[i]);
        const double bw = fmin(6.0e4, 7.72e6 / fmin(blocks, CUS));
        const double unit = fmax(2.0 * 32 * widths[i] * 64.0 / rates[i], widths[i] * 128.0 / bw);
        const double t = ceil(blocks / CUS) * (K / 64.0 * unit + 3.0);
        if (t < best_t) { best_t = t; best = widths[i]; }
    }
    return best;
}

static GemmPlan plan_for(int M, int N, int K, bool glu, bool keep) {
    const double CUS = (double)device_cus();
    // Up to 16 rows: the streaming kernel, a block per 16 columns, unless those blocks go badly
    // round the 256 CUs (320 of them take as long as 512 would: N = 5120), the caller takes
    // partial sums anyway and the weight is large enough for the gain (three eighths of its
    // stream) to pay for the norm's own kernel, which the streaming kernel would have taken into
    // its epilogue: then the tiles below, whose blocks split K as finely as it takes.
    if (M <= 16 && glu && few_rows_gated_on_tiles(M, N, K)) return {32, plan_rows32(N, K), 1};
    if (M <= 16) {
        const int nb = (N + 15) / 16;
        const double fill = (double)nb / (ceil(nb / CUS) * CUS);
        if (glu || !keep || fill >= 0.8 || (double)N * K < 40e6) return {0, 0, 1};
        // (two row groups a block: ahead of the tiles up to 8 rows, and up to 16 where K is short)
        if (two_row_groups(N) && (M <= 8 || (double)N * K < 45e6)) return {0, 0, 1};
    }
    const int nk = (K + 63) / 64;
    if (K % 64 == 0) {
        // The four-wave kernel's tiles (256 rows on 2 x 2 waves, 128 rows on 1 x 4) and, up to 512 rows,
        // its 64 x 128, two blocks to a CU (the last candidate; its rate is that of the sixteen-wave
        // kernel's 64 x 128, which it replaced and is 8 to 17 % faster than at 128 to 512 rows, so
        // the model picks it rather too seldom).  A block goes through its part of K in
        // units of 64; a unit takes what its MFMAs take at the tile's rate or what its columns of W take
        // to arrive, whichever is longer: a block's share of the HBM stream, at most what one CU pulls.
        // Blocks go round the CUs; each round ends with the pipeline filled and the tile stored.  The
        // constants were fitted to measurements of the four products of the 8B, 14B and 32B shapes at
        // 17 .. 4,096 rows on an MI355X (weights in turn, so that none comes from a cache; every tile
        // with 1 .. 8 parts, 204 cases): the pick is 0.3 % from the best candidate on average, 6 % at worst.
        // Up to 64 rows the four waves side by side take 64 or 32 rows: a product of so few rows is its
        // weight's stream, and a block that does not work through 128 rows for 32 asks for its next
        // columns sooner (3 to 10 % less time than the tiles of 128 rows and the sixteen-wave kernel's
        // 64 x 128 on the four products of the three shapes at 17 to 64 rows; their rates fitted to
        // those 88 cases stand for that, the pick 0.5 % from the best on average, 5 % at worst).
        struct Cand { int bm, bn, slots; double rate; };
        static const Cand cands[11] = {{256, 256, 1, 6.01e6}, {256, 192, 1, 5.45e6}, {256, 128, 1, 5.04e6},
                                       {128, 384, 1, 3.24e6}, {128, 256, 1, 4.61e6}, {128, 128, 1, 3.45e6},
                                       {64, 256, 1, 2.4e6}, {64, 128, 1, 2.0e6}, {32, 256, 1, 1.4e6}, {32, 128, 1, 1.3e6},
                                       {64, 128, 2, 2.18e6}};
        const double HBM = 7.72e6, CU_MAX = 6.0e4;       // bytes a microsecond: all CUs together, one alone
        GemmPlan best = {128, 128, 1};
        double best_t = 1e30;
        for (const Cand& c : cands) {
            if (c.bm == 256 && M <= 64) continue;
            if (c.slots == 1 && c.bm <= 64 && M > c.bm) continue;         // (four waves side by side: one row tile)
            if (c.slots == 2 && (M <= 64 || M > 512)) continue;            // (64 x 128 with several row tiles)
            for (int S = 1; S <= ((glu && M > 64) ? 2 : 8); S *= 2) {
                if (S > 1 && nk / S < 4) break;
                const double blocks = (double)((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn) * S;
                const double rounds = ceil(blocks / (CUS * c.slots));
                const double share = fmin((double)c.slots, ceil(blocks / CUS));   // blocks that share a CU's MFMAs
                const double bw = fmin(CU_MAX, HBM / fmin(blocks, CUS * c.slots));
                const double unit = fmax(2.0 * c.bm * c.bn * 64.0 * share / c.rate, c.bn * 128.0 / bw);
                double t = rounds * ((double)nk / S * unit + 3.0) + 3.0;
                // the partial sums: written, read and added by a second kernel, or (kept) read by the
                // consumer in place of one plane
                if (S > 1) t += keep ? (S - 1.0) * M * N * 4.0 / 4e6 : (double)S * M * N * 4.0 / 2.54e6 + 2.7;
                if (t < best_t) { best_t = t; best = {c.bm, c.bn, S}; }
            }
        }
        return best;
    }
    if (M <= 64) {
        // A stream of W: a CU pulls a block's k-tile of 64 (16 KB) in some 0.63 us whatever else
        // runs, blocks go round the 256 CUs, and the most loaded CU sets the time.  Splitting K
        // evens the load out (272 blocks are two rounds for 16 CUs and one for the rest; 1,088
        // quarters are five rounds against 4.25) at the price of the partial sums' traffic and
        // of some 4 us that a block spends before its first and after its last k-tile (two
        // blocks of a CU overlap theirs).
        const long blocks = (N + 127) / 128;
        int best_s = 1;
        double best_t = 1e30;
        for (int S = 1; S <= 8; S *= 2) {
            if (S > 1 && nk / S < 4) break;
            double t = ceil(blocks * S / CUS) * ceil((double)nk / S) * 0.63 + ceil(blocks * S / (2.0 * CUS)) * 4.0 + 1.0;
            if (S > 1) t += keep ? (S - 1.0) * M * N * 4.0 / 4e6 : (double)S * M * N * 8.0 / 4e6 + 3.0;
            if (t < best_t) { best_t = t; best_s = S; }
        }
        return {64, 128, best_s};
    }
    // K in no units of 64, more than 64 rows: the sixteen-wave kernel's tiles.  rate: flops a microsecond
    // that a CU sustains on blocks of this tile; slots: blocks a CU holds.
    struct Cand { int bm, bn, slots; double rate; };
    static const Cand cands_w16[5] = {{256, 256, 1, 5.2e6}, {256, 192, 1, 4.4e6}, {128, 256, 1, 3.6e6},
                                      {128, 128, 1, 2.6e6}, {64, 128, 2, 2.2e6}};
    GemmPlan best = {256, 256, 1};
    double best_t = 1e30;
    for (const Cand& c : cands_w16) {
        for (int S = 1; S <= (glu ? 2 : 8); S *= 2) {
            // gate and up groups come in pairs, an even number a wave: three a wave of the sixteen do not do
            if (glu && c.bn == 192) break;
            if (S > 1 && nk / S < 8) break;
            const double blocks = (double)((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn) * S;
            const double rounds = ceil(blocks / (CUS * c.slots));
            // a round: the blocks' work at the tile's rate plus some 3 us to fill the pipeline and
            // store the tile; a last round that fills part of the machine takes as long as a full one
            const double round_us = 2.0 * c.bm * c.bn * ((double)K / S) * c.slots / c.rate + 3.0;
            double t = round_us * rounds + 3.0;
            // the partial sums: written, read and added by a second kernel, or (kept) read by the
            // consumer in place of one plane
            if (S > 1) t += keep ? (S - 1.0) * M * N * 4.0 / 4e6 : (double)S * M * N * 4.0 / 3e6 + 3.0;
            if (t < best_t) { best_t = t; best = {c.bm, c.bn, S}; }
        }
    }
    return best;
}

TFF_API size_t tff_gemm_workspace_bytes(int M, int N, int K, int ab_dtype, int glu, int keep_partials) {
    if (ab_dtype != TFF_BF16 || M <= 0 || N <= 0 || K <= 0) return 0;
    const GemmPlan p = plan_for(M, N, K, glu != 0, keep_partials != 0);
    return p.splits > 1 ? (size_t)p.splits * M * N * sizeof(float) : 0;
}

// For tests and tuning: the plan's tile (rows x columns) and number of parts.
TFF_API int tff_gemm_plan(int M, int N, int K, int glu, int keep_partials, int* tile_rows, int* tile_cols,
                          int* splits) {
    const GemmPlan p = plan_for(M, N, K, glu != 0, keep_partials != 0);
    if (tile_rows) *tile_rows = p.tile;
    if (tile_cols) *tile_cols = p.bn;
    if (splits) *splits = p.splits;
    return 0;
}

// Up to 16 rows: which streaming kernel.  Gated: with 512 row groups and more a wave takes
// a group's whole K through a ring (384 such waves, at N = 6,144, are too few: 3 % slower).  Plain: more waves per block where there are few blocks
// (small N) or long rows (large K), fewer and deeper ones in between.
template <int EPI>
static int skinny_for(const bf16_t* A, const bf16_t* Wp, void* C, int M, int N, int K, int lda, int c_dtype,
                      int glu_out, hipStream_t s, const SkinnyFuse* fuse) {
    if (glu_out > 0) {
        if constexpr (EPI != 2) {
            if (N >= 8 * 1024)
                return launch_skinny<1, 1, 8, 1, 2, true, true, EPI>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, fuse);
            // A wave takes a quarter of K in groups of k-steps whose loads are issued together, and
            // the steps that are left when a group is not full go one at a time: groups of eight
            // where a quarter of K is fewer than 32 steps, of 32 (with the norm's factor taken in,
            // which needs registers of its own, 24) otherwise.
            if (K < 4096)
                return launch_skinny<1, 1, 8, 4, 2, true, false, EPI>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, fuse);
            return launch_skinny<1, 1, (EPI == 1 ? 24 : 32), 4, 2, true, false, EPI>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, fuse);
        } else {
            return tff_fail("gemm: a gated product does not come before a norm");
        }
    }
    // A block per 16 columns goes badly round the CUs when there are a little more row groups than
    // CUs (320 of them, N = 5120, take as long as 512 would).  Then a block takes two row groups:
    // half as many blocks, all at once, and between them they still pull what HBM gives (some 130
    // CUs do).  Measured at N = 5120 against tiles that split K with a norm kernel to add their
    // parts: O of the 14B shape 11.9 / 14.1 / 16.7 us at 1 / 8 / 16 rows against 13.7 / 15.1 / 19.0,
    // of the 32B shape 20.4 / 21.6 / 24.0 against 27.2 / 27.4 / 27.5; down of the 14B shape 33.4 /
    // 39.8 against 42.9 / 42.8 at 1 / 8 rows (at 16 rows the tiles are ahead, see plan_for).  Not for
    // the product after a norm: the row factors' registers do not fit beside two row groups.
    if constexpr (EPI != 1) {
        if (two_row_groups(N)) return launch_skinny<1, 2, 4, 16, 1, false, false, EPI>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, fuse);
    }
    // A very wide product (an output head) has thousands of blocks, each of which fetches all of A's
    // rows: with many rows and a long K that traffic shows (152k columns, K = 4,096: 196 / 217 / 281 us
    // at 1 / 8 / 16 rows).  Two groups of 16 columns a block halve it: 243 us at 16 rows, K = 5,120 at
    // 8 / 16 rows 264 / 303 us against 278 / 366; with fewer rows one group a block stays ahead.
    if constexpr (EPI == 0) {
        if (N >= 32 * 1024 && (long)M * K >= 40000)
            return launch_skinny<1, 2, 4, 8, 1, false, false, 0>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, fuse);
    }
    // (K up to 1,024: sixteen waves would have two k-steps each, less than a group of four)
    if (N >= 32 * 1024 || K <= 1024)
        return launch_skinny<1, 1, 4, 8, 1, false, false, EPI>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, fuse);
    if (K >= 8192 || N <= 4096)
        return launch_skinny<1, 1, 4, 16, 1, false, false, EPI>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, fuse);
    return launch_skinny<1, 1, 8, 4, 1, false, false, EPI>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, fuse);
}

// glu_out > 0: W holds gate and up groups in turn (N = 2 * ceil16(glu_out) rows) and C is
// [M, glu_out] = silu(gate) * up.  workspace: room for partial sums (tff_gemm_workspace_bytes);
// with less the blocks do not split K.
// keep_partials: where the plan splits K, the partial sums stay in the workspace
// ([splits, M, N] float32) for the caller to add up, and C is not written.
int tff_gemm_bf16(const bf16_t* A, const bf16_t* Wp, void* C, int M, int N, int K, int lda,
                  int c_dtype, int glu_out, float* workspace, size_t workspace_bytes,
                  int keep_partials, hipStream_t s) {
    TFF_REQUIRE(K % 8 == 0 && lda % 8 == 0,
                "gemm: the bfloat16 product needs the inner size (K=%d, row stride %d) to be a multiple of 8",
                K, lda);
    TFF_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)Wp % 16) == 0 && ((uintptr_t)C % 16) == 0,
                "gemm: operands must be 16-byte aligned");
    TFF_REQUIRE(c_dtype == TFF_F32 || c_dtype == TFF_BF16, "gemm: unknown output type %d", c_dtype);
    GemmPlan plan = plan_for(M, N, K, glu_out > 0, keep_partials != 0);
    const int planned_splits = plan.splits;
    if (!workspace || workspace_bytes < (size_t)plan.splits * M * N * sizeof(float)) plan.splits = 1;
    const int S = plan.splits;
    const bool red = !keep_partials;
    TFF_REQUIRE(!keep_partials || (glu_out == 0 && c_dtype == TFF_F32),
                "gemm: partial sums are kept for a plain float32 result only");
    if (glu_out > 0) {
        TFF_REQUIRE(N % 32 == 0 && glu_out <= N / 2 && glu_out > N / 2 - 16,
                    "gemm: a gated weight of %d rows does not fit %d output columns", N, glu_out);
        if (plan.tile == 0) return skinny_for<0>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, nullptr);
        if (plan.tile <= 64 && K % 64 == 0) {                // the four waves side by side on 64 or 32 rows
            if (plan.tile == 32 && plan.bn == 128) return launch_w4<2, 5, true, 1, false, 2>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
            if (plan.tile == 32) return launch_w4<4, 5, true, 1, false, 2>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
            if (plan.bn == 128) return launch_w4<2, 5, true, 1, false, 4>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
            return launch_w4<4, 5, true, 1, false, 4>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
        }
        if (plan.tile == 64)
            return launch_async_g<2, 2, 2, 4, 3, true>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
        if (K % 64 == 0) {
            if (plan.tile == 128) {
                if (plan.bn == 128) return launch_w4<2, 5, true, 1>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
                if (plan.bn == 256) return launch_w4<4, 5, true, 1>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
                return launch_w4<6, 4, true, 1>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
            }
            if (plan.bn == 128) return launch_w4<4, 5, true>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
            if (plan.bn == 192) return launch_w4<6, 5, true>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
            return launch_w4<8, 4, true>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
        }
        if (plan.tile == 128 && plan.bn == 128)
            return launch_async_g<2, 2, 4, 4, 3, true>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
        if (plan.tile == 128)
            return launch_async_g<2, 4, 4, 4, 3, true>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
        return launch_async_g<4, 4, 4, 4, 5, true, 1, true>(A, Wp, C, M, N, K, lda, c_dtype, glu_out, s, S, workspace);
    }
    if (plan.tile == 0) return skinny_for<0>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, nullptr);
    if (plan.tile == 64 || plan.tile == 32) {
        // few columns and no room for partial sums: the streaming kernel, whose blocks split K
        // among their waves
        if (S == 1 && planned_splits > 1 && M <= 64) {
            if (M <= 32) return launch_skinny<2, 2, 4, 8>(A, Wp, C, M, N, K, lda, c_dtype, 0, s);
            return launch_skinny<4, 2, 4, 8>(A, Wp, C, M, N, K, lda, c_dtype, 0, s);
        }
        if (K % 64 == 0) {                                   // the four waves side by side on 64 or 32 rows
            if (plan.tile == 32 && plan.bn == 128) return launch_w4<2, 5, false, 1, false, 2>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
            if (plan.tile == 32) return launch_w4<4, 5, false, 1, false, 2>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
            if (plan.bn == 128) return launch_w4<2, 5, false, 1, false, 4>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
            return launch_w4<4, 5, false, 1, false, 4>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
        }
        return launch_async_g<2, 2, 2, 4, 3>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
    }
    if (K % 64 == 0) {
        if (plan.tile == 128) {
            if (plan.bn == 128) return launch_w4<2, 5, false, 1>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
            if (plan.bn == 256) return launch_w4<4, 5, false, 1>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
            return launch_w4<6, 4, false, 1>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
        }
        if (plan.bn == 128) return launch_w4<4, 5>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
        if (plan.bn == 192) return launch_w4<6, 5>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
        return launch_w4<8, 4>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
    }
    if (plan.tile == 128 && plan.bn == 128)
        return launch_async_g<2, 2, 4, 4, 3>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
    if (plan.tile == 128)
        return launch_async_g<2, 4, 4, 4, 3>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
    if (plan.bn == 192)
        return launch_async_g<4, 4, 4, 3, 5, false, 1, true>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
    return launch_async_g<4, 4, 4, 4, 5, false, 1, true>(A, Wp, C, M, N, K, lda, c_dtype, 0, s, S, workspace, red);
}

// ---- the norm between two products of up to 16 rows, taken into them ----
static int check_fused_operands(const char* what, const void* A, const void* Wp, int M, int N, int K, int lda) {
    TFF_REQUIRE(A && Wp, "%s: null pointer", what);
    TFF_REQUIRE(M >= 1 && M <= 16 && N > 0 && K > 0 && lda >= K, "%s: bad sizes M=%d N=%d K=%d lda=%d (1 to 16 rows)",
                what, M, N, K, lda);
    TFF_REQUIRE(K % 8 == 0 && lda % 8 == 0, "%s: the inner size (K=%d, row stride %d) must be a multiple of 8", what,
                K, lda);
    TFF_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)Wp % 16) == 0, "%s: operands must be 16-byte aligned", what);
    return 0;
}

// resid[M, N] += A . W^T (bfloat16 A and packed W, float32 sums); x_out[M, N] = bfloat16 of the new
// resid times norm_w[N]; ss_out[m][g] (16 rows of ss_stride floats, ss_stride >= ceil(N / 16)) =
// sum of squares of the new resid over columns 16 g .. 16 g + 15 of row m.  N a multiple of 8.
TFF_API int tff_gemm_residual_prenorm(const void* A, const void* Wp, int M, int N, int K, int lda, float* resid,
                                      const float* norm_w, void* x_out, float* ss_out, int ss_stride,
                                      tff_stream_t stream) {
    if (int rc = check_fused_operands("gemm_residual_prenorm", A, Wp, M, N, K, lda)) return rc;
    TFF_REQUIRE(resid && norm_w && x_out && ss_out, "gemm_residual_prenorm: null pointer");
    TFF_REQUIRE(N % 8 == 0 && ss_stride >= (N + 15) / 16, "gemm_residual_prenorm: N=%d must be a multiple of 8 and "
                "ss_out needs %d floats a row, has %d", N, (N + 15) / 16, ss_stride);
    TFF_REQUIRE(((uintptr_t)resid % 16) == 0 && ((uintptr_t)norm_w % 16) == 0 && ((uintptr_t)x_out % 8) == 0,
                "gemm_residual_prenorm: operands must be 16-byte aligned");
    SkinnyFuse fz{nullptr, 0, 0, 0.f, 0.f, resid, norm_w, (bf16_t*)x_out, ss_out, ss_stride};
    return skinny_for<2>((const bf16_t*)A, (const bf16_t*)Wp, resid, M, N, K, lda, TFF_F32, 0, (hipStream_t)stream, &fz);
}

// C = rstd[m] * (A . W^T) with rstd[m] = rsqrt(sum_g ss[m][g] / dim + eps), g < ss_count: the product
// after tff_gemm_residual_prenorm (A = its x_out, ss = its ss_out, dim = its N).  glu_out as in tff_gemm.
TFF_API int tff_gemm_row_scaled(const void* A, const void* Wp, void* C, int M, int N, int K, int lda, int c_dtype,
                                int glu_out, const float* ss, int ss_stride, int ss_count, int dim, float eps,
                                tff_stream_t stream) {
    if (int rc = check_fused_operands("gemm_row_scaled", A, Wp, M, N, K, lda)) return rc;
    TFF_REQUIRE(C && ss && ((uintptr_t)C % 16) == 0 && ((uintptr_t)ss % 16) == 0, "gemm_row_scaled: null or unaligned pointer");
    TFF_REQUIRE(c_dtype == TFF_F32 || c_dtype == TFF_BF16, "gemm_row_scaled: unknown output type %d", c_dtype);
    TFF_REQUIRE(ss_count > 0 && ss_stride >= ss_count && ss_stride % 4 == 0 && dim > 0,
                "gemm_row_scaled: %d sums of squares a row, %d apart (a multiple of 4), over %d elements", ss_count,
                ss_stride, dim);
    if (glu_out > 0)
        TFF_REQUIRE(N % 32 == 0 && glu_out <= N / 2 && glu_out > N / 2 - 16,
                    "gemm_row_scaled: a gated weight of %d rows does not fit %d output columns", N, glu_out);
    // (the four-wave kernel's tiles of 32 rows take the rows' factors into their epilogue too)
    if (glu_out > 0 && few_rows_gated_on_tiles(M, N, K)) {
        const W4Scale sc{ss, ss_stride, ss_count, 1.0f / (float)dim, eps};
        const bf16_t* a = (const bf16_t*)A;
        const bf16_t* w = (const bf16_t*)Wp;
        hipStream_t s = (hipStream_t)stream;
        if (plan_rows32(N, K) == 128)
            return launch_w4<2, 5, true, 1, true, 2>(a, w, C, M, N, K, lda, c_dtype, glu_out, s, 1, nullptr, true, sc);
        return launch_w4<4, 5, true, 1, true, 2>(a, w, C, M, N, K, lda, c_dtype, glu_out, s, 1, nullptr, true, sc);
    }
    SkinnyFuse fz{ss, ss_stride, ss_count, 1.0f / (float)dim, eps, nullptr, nullptr, nullptr, nullptr, 0};
    return skinny_for<1>((const bf16_t*)A, (const bf16_t*)Wp, C, M, N, K, lda, c_dtype, glu_out, (hipStream_t)stream, &fz);
}

int tff_gemm_f32(const float* A, const float* W, void* C, int M, int N, int K, int lda,
                 int c_dtype, hipStream_t s);

TFF_API int tff_gemm(const void* A, const void* W, void* C, int M, int N, int K, int lda,
                     int ab_dtype, int c_dtype, int w_packed, int glu_out, void* workspace,
                     size_t workspace_bytes, int keep_partials, tff_stream_t stream) {
    TFF_REQUIRE(A && W && C, "gemm: null pointer");
    TFF_REQUIRE(M >= 0 && N > 0 && K > 0 && lda >= K, "gemm: bad sizes M=%d N=%d K=%d lda=%d", M, N, K, lda);
    if (M == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (ab_dtype == TFF_F32) {
        TFF_REQUIRE(!w_packed && glu_out == 0 && !keep_partials,
                    "gemm: the float32 product takes a plain row-major weight and keeps no partial sums");
        return tff_gemm_f32((const float*)A, (const float*)W, C, M, N, K, lda, c_dtype, s);
    }
    if (ab_dtype == TFF_BF16) {
        TFF_REQUIRE(w_packed, "gemm: the bfloat16 product takes a weight in fragment order");
        TFF_REQUIRE(((uintptr_t)workspace % 16) == 0, "gemm: the workspace must be 16-byte aligned");
        return tff_gemm_bf16((const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, c_dtype, glu_out,
                             (float*)workspace, workspace ? workspace_bytes : 0, keep_partials, s);
    }
    return tff_fail("gemm: unknown operand type %d", ab_dtype);
}

// ------------------------------------------------------------- packing ---
// Row-major [N, K] -> fragment order, with zero padding to 16 rows and 32 k.
__global__ void pack_weight_kernel(const bf16_t* __restrict__ src, bf16_t* __restrict__ dst, int N,
                                   int K, int KB, size_t total_chunks) {
    // one thread per 16-byte chunk of the packed matrix
    const size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= total_chunks) return;
    const int l = (int)(c & 63);
    const size_t frag = c >> 6;
    const int kb = (int)(frag % KB);
    const int nb = (int)(frag / KB);
    const int n = nb * 16 + (l & 15);
    const int k = kb * 32 + (l >> 4) * 8;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (n < N && k < K) v = *reinterpret_cast<const uint4*>(src + (size_t)n * K + k);   // K % 8 == 0
    *reinterpret_cast<uint4*>(dst + c * 8) = v;
}

TFF_API int tff_pack_weight(const void* src, void* dst, int N, int K, tff_stream_t stream) {
    TFF_REQUIRE(src && dst, "pack_weight: null pointer");
    TFF_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "pack_weight: inner size %d must be a multiple of 8", K);
    const int NB = (N + 15) / 16, KB = (K + 31) / 32;
    const size_t chunks = (size_t)NB * KB * 64;
    const size_t blocks = (chunks + 255) / 256;
    TFF_REQUIRE(blocks < 2147483647ULL, "pack_weight: matrix too large");
    pack_weight_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((const bf16_t*)src, (bf16_t*)dst, N, K,
                                                                           KB, chunks);
    return tff_check_launch("pack_weight");
}

// Gather of rows out of a matrix in fragment order (the embedding of a model whose
// output head shares the table): out[t, :] = float(E[ids[t], :]).
__global__ void embed_packed_kernel(const bf16_t* __restrict__ table, const int32_t* __restrict__ ids,
                                    float* __restrict__ out, int H, int V, int KB) {
    const int t = blockIdx.x;
    int id = ids[t];
    const bool bad = id < 0 || id >= V;
    if (bad) id = 0;
    const bf16_t* base = table + (size_t)(id / 16) * KB * 512 + (id % 16) * 8;
    float* o = out + (size_t)t * H;
    for (int c = threadIdx.x; c < H / 8; c += blockDim.x) {   // chunk c holds k = 8c .. 8c+7
        const bf16_t* p = base + (size_t)(c / 4) * 512 + (c % 4) * 128;
        union { uint4 u; bf16_t h[8]; } v;
        v.u = *reinterpret_cast<const uint4*>(p);
#pragma unroll
        for (int e = 0; e < 8; ++e) o[c * 8 + e] = bad ? __builtin_nanf("") : (float)v.h[e];
    }
}

TFF_API int tff_embed_packed(const void* table, const int32_t* ids, float* out, int T, int H, int V,
                             tff_stream_t stream) {
    TFF_REQUIRE(table && ids && out, "embed: null pointer");
    TFF_REQUIRE(T >= 0 && H > 0 && V > 0 && H % 8 == 0, "embed: bad sizes T=%d H=%d V=%d", T, H, V);
    if (T == 0) return 0;
    embed_packed_kernel<<<T, 256, 0, (hipStream_t)stream>>>((const bf16_t*)table, ids, out, H, V, (H + 31) / 32);
    return tff_check_launch("embed_packed");
}
