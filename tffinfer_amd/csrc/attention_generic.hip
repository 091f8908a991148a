// Attention over the paged cache for any head size, group size, page size and
// window, in float32 arithmetic: the path of the 32-bit model, and the yardstick
// the matrix-core kernels are checked against.
//
// One wave per (token, q head).  Keys are taken 64 at a time, one per lane:
//   s_j = (q . k_j) * scale                   (scale after the product,
//                                              reference paged_flash_attention.cu:723)
//   visible iff  lo <= j <= pos               (causal: mask_op.cu:37-43; lo from the window)
//   running max m and sum l over chunks       (paged_flash_attention.cu:746-790)
//   o = sum_j exp(s_j - m) v_j / l
// q head h reads kv head h / (nq / nkv)       (paged_flash_attention.cu:891-892).
// Keys lie [page, kv head, slot, element], values [page, kv head, element, slot].
// Keys are found by block id arithmetic, not by a table of addresses as in the
// reference (src/kernel/cuda/get_row.cu:73-109).
#include "common.h"
#include "tffinfer_kernels.h"

#define AG_MAX_D 512

template <typename T, typename TC>
__global__ __launch_bounds__(64) void attention_generic_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, const TC* __restrict__ k_cache,
    const TC* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int bt_stride,
    const int32_t* __restrict__ token_req, const int32_t* __restrict__ positions, int nq, int nkv,
    int d, int page_size, int window, float scale) {
    __shared__ float qs[AG_MAX_D];
    __shared__ long long voff[64];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int G = nq / nkv;
    const int g = h / G;
    const int r = token_req[t];
    const int pos = positions[t];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int32_t* bt = block_tables + (size_t)r * bt_stride;

    const T* qp = q + (size_t)t * q_stride + (size_t)h * d;
    for (int e = lane; e < d; e += 64) qs[e] = to_f32(qp[e]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[AG_MAX_D / 64];
#pragma unroll
    for (int i = 0; i < AG_MAX_D / 64; ++i) acc[i] = 0.f;

    for (int base = lo; base <= pos; base += 64) {
        const int j = base + lane;
        const bool valid = j <= pos;
        float s = -INFINITY;
        long long off = 0;
        if (valid) {
            const int page = bt[j / page_size];
            const long long head_base = ((long long)page * nkv + g) * page_size * d;
            off = head_base + (j % page_size);   // values: [element][slot]
            const TC* kp = k_cache + head_base + (long long)(j % page_size) * d;
            float dot = 0.f;
            for (int e = 0; e < d; ++e) dot = fmaf(qs[e], to_f32(kp[e]), dot);
            s = dot * scale;
        }
        __syncthreads();  // earlier readers of voff are done
        voff[lane] = off;
        const float cmax = wave_max(s);
        const float m_new = fmaxf(m, cmax);
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);  // 0 on the first chunk (m = -inf)
        l = l * corr + wave_sum(p);
        m = m_new;
        __syncthreads();
        const int nvalid = min(64, pos - base + 1);
#pragma unroll
        for (int i = 0; i < AG_MAX_D / 64; ++i) acc[i] *= corr;
        for (int jj = 0; jj < nvalid; ++jj) {
            const float pj = __shfl(p, jj, 64);
            const TC* vp = v_cache + voff[jj];
#pragma unroll
            for (int i = 0; i < AG_MAX_D / 64; ++i) {
                const int e = lane + 64 * i;
                if (e < d) acc[i] = fmaf(pj, to_f32(vp[(long long)e * page_size]), acc[i]);
            }
        }
    }
    T* op = out + (size_t)t * nq * d + (size_t)h * d;
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < AG_MAX_D / 64; ++i) {
        const int e = lane + 64 * i;
        if (e < d) op[e] = from_f32<T>(acc[i] * inv);
    }
}

TFF_API int tff_attention_generic(const void* q, int q_stride, void* out, const void* k_cache,
                                  const void* v_cache, const int32_t* block_tables, int bt_stride,
                                  const int32_t* token_req, const int32_t* positions, int T, int nq,
                                  int nkv, int d, int page_size, int num_pages, int window,
                                  float scale, int dtype, int cache_dtype, tff_stream_t stream) {
    TFF_REQUIRE(q && out && k_cache && v_cache && block_tables && token_req && positions,
                "attention: null pointer");
    TFF_REQUIRE(T >= 0 && nq > 0 && nkv > 0 && nq % nkv == 0,
                "attention: %d query heads are not a multiple of %d key heads", nq, nkv);
    TFF_REQUIRE(d > 0 && d <= AG_MAX_D, "attention: head size %d not supported (1..%d)", d, AG_MAX_D);
    TFF_REQUIRE(page_size > 0 && num_pages > 0 && bt_stride > 0 && window >= 0,
                "attention: bad cache geometry page_size=%d pages=%d table stride=%d window=%d",
                page_size, num_pages, bt_stride, window);
    TFF_REQUIRE(q_stride >= nq * d, "attention: query row stride %d below %d", q_stride, nq * d);
    TFF_REQUIRE(dtype == cache_dtype, "attention: cache type %d differs from activation type %d",
                cache_dtype, dtype);
    TFF_REQUIRE(nq <= 65535, "attention: too many heads");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(T, nq);
    if (dtype == TFF_F32)
        attention_generic_kernel<float, float><<<grid, 64, 0, s>>>(
            (const float*)q, q_stride, (float*)out, (const float*)k_cache, (const float*)v_cache,
            block_tables, bt_stride, token_req, positions, nq, nkv, d, page_size, window, scale);
    else if (dtype == TFF_BF16)
        attention_generic_kernel<bf16_t, bf16_t><<<grid, 64, 0, s>>>(
            (const bf16_t*)q, q_stride, (bf16_t*)out, (const bf16_t*)k_cache,
            (const bf16_t*)v_cache, block_tables, bt_stride, token_req, positions, nq, nkv, d,
            page_size, window, scale);
    else
        return tff_fail("attention: unknown dtype %d", dtype);
    return tff_check_launch("attention_generic");
}
