// Token choice on the device: argmax, repetition penalty, and a draw from the
// temperature softmax under top-k / top-p / min-p.
//
// The reference chooses on the CPU: std::max_element for greedy
// (src/core/sampler/LLMSampler.cpp:43-45), logits * 1/temp (:36-41), the
// penalty of seen tokens (:21-34), a discrete draw (:47-54); top_k, top_p and
// min_p are fields of its SamplingConfig (LLMSampler.h:55-63).  Here one block
// works on one row of float32 logits.  Thresholds are found by bisection over
// the bit patterns of the unnormalised probabilities e_i = exp((l_i - max)/temp)
// instead of a sort; sums that decide a threshold or the drawn index are kept
// in float64 and run in a fixed order, so the same row and the same uniform
// number give the same token in any batch.
#include "common.h"
#include "tffinfer_kernels.h"

#define SAMPLE_THREADS 1024

__device__ __forceinline__ double block_sum_f64(double v, double* red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nwave = (blockDim.x + 63) >> 6;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        double s = 0.0;
        for (int i = 0; i < nwave; ++i) s += red[i];
        red[16] = s;
    }
    __syncthreads();
    return red[16];
}

// lowest index among the maxima; every thread gets it
__device__ __forceinline__ int block_argmax(const float* __restrict__ x, int V, float* redv,
                                            int* redi, float* max_out) {
    float best = -INFINITY;
    int arg = 0x7fffffff;
    // One block reads the whole row, so what counts is loads in flight: eight 16-byte loads
    // per thread are issued before the first is compared.
    const int head = min(V, (int)(((16 - ((uintptr_t)x & 15)) & 15) / 4));   // up to a 16-byte boundary
    const int nvec = (V - head) / 4;
    const float4* x4 = reinterpret_cast<const float4*>(x + head);
    constexpr int UN = 8;
    for (int i0 = threadIdx.x; i0 < nvec; i0 += UN * blockDim.x) {
        float4 v[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int j = i0 + u * blockDim.x;
            v[u] = x4[min(j, nvec - 1)];
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int j = i0 + u * blockDim.x;
            if (j < nvec) {
                const int i = head + 4 * j;
                if (v[u].x > best || (v[u].x == best && i < arg)) { best = v[u].x; arg = i; }
                if (v[u].y > best || (v[u].y == best && i + 1 < arg)) { best = v[u].y; arg = i + 1; }
                if (v[u].z > best || (v[u].z == best && i + 2 < arg)) { best = v[u].z; arg = i + 2; }
                if (v[u].w > best || (v[u].w == best && i + 3 < arg)) { best = v[u].w; arg = i + 3; }
            }
        }
    }
    for (int t = threadIdx.x; t < V - 4 * nvec; t += blockDim.x) {   // before and after the 16-byte part
        const int i = t < head ? t : t + 4 * nvec;
        const float v = x[i];
        if (v > best || (v == best && i < arg)) { best = v; arg = i; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(arg, o, 64);
        if (ov > best || (ov == best && oi < arg)) { best = ov; arg = oi; }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nwave = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) { redv[wave] = best; redi[wave] = arg; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float b = redv[0];
        int a = redi[0];
        for (int i = 1; i < nwave; ++i)
            if (redv[i] > b || (redv[i] == b && redi[i] < a)) { b = redv[i]; a = redi[i]; }
        redv[16] = b;
        redi[16] = a;
    }
    __syncthreads();
    *max_out = redv[16];
    return redi[16];
}

__global__ __launch_bounds__(SAMPLE_THREADS) void argmax_kernel(const float* __restrict__ logits,
                                                                 int32_t* __restrict__ out, int V) {
    __shared__ float redv[17];
    __shared__ int redi[17];
    float mx;
    const int a = block_argmax(logits + (size_t)blockIdx.x * V, V, redv, redi, &mx);
    if (threadIdx.x == 0) out[blockIdx.x] = a == 0x7fffffff ? 0 : a;  // all NaN: index 0
}

TFF_API int tff_argmax(const float* logits, int32_t* out, int rows, int V, tff_stream_t stream) {
    TFF_REQUIRE(logits && out, "argmax: null pointer");
    TFF_REQUIRE(rows >= 0 && V > 0, "argmax: bad sizes rows=%d V=%d", rows, V);
    if (rows == 0) return 0;
    argmax_kernel<<<rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(logits, out, V);
    return tff_check_launch("argmax");
}

__global__ void repetition_penalty_kernel(float* __restrict__ logits, int V,
                                          const int32_t* __restrict__ seen,
                                          const int32_t* __restrict__ cu_seen,
                                          const float* __restrict__ penalty) {
    const int r = blockIdx.x;
    const float pen = penalty[r];
    if (pen == 1.0f) return;
    float* row = logits + (size_t)r * V;
    for (int i = cu_seen[r] + threadIdx.x; i < cu_seen[r + 1]; i += blockDim.x) {
        const int tok = seen[i];
        if (tok >= 0 && tok < V) {
            const float v = row[tok];
            row[tok] = v > 0.f ? v / pen : v * pen;
        }
    }
}

TFF_API int tff_repetition_penalty(float* logits, int rows, int V, const int32_t* seen,
                                   const int32_t* cu_seen, const float* penalty,
                                   tff_stream_t stream) {
    TFF_REQUIRE(logits && seen && cu_seen && penalty, "repetition_penalty: null pointer");
    TFF_REQUIRE(rows >= 0 && V > 0, "repetition_penalty: bad sizes rows=%d V=%d", rows, V);
    if (rows == 0) return 0;
    repetition_penalty_kernel<<<rows, 256, 0, (hipStream_t)stream>>>(logits, V, seen, cu_seen, penalty);
    return tff_check_launch("repetition_penalty");
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int32_t* __restrict__ out, int V,
    const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ top_p, const float* __restrict__ min_p,
    const float* __restrict__ uniform, float* __restrict__ probs_out) {
    __shared__ float redv[17];
    __shared__ int redi[17];
    __shared__ double redd[17];
    __shared__ double seg[SAMPLE_THREADS];
    __shared__ int chosen;
    const int r = blockIdx.x;
    const float* x = logits + (size_t)r * V;
    const float temp = temperature[r];
    float mx;
    const int amax = block_argmax(x, V, redv, redi, &mx);
    if (temp <= 0.f || amax == 0x7fffffff) {
        if (threadIdx.x == 0) out[r] = amax == 0x7fffffff ? 0 : amax;
        if (probs_out)
            for (int i = threadIdx.x; i < V; i += blockDim.x) probs_out[(size_t)r * V + i] = i == amax ? 1.f : 0.f;
        return;
    }
    const float inv_t = 1.0f / temp;
#define E_OF(i) expf((x[i] - mx) * inv_t)
    uint32_t thr = 0;  // bit pattern; keep e_i with bits >= thr
    const int k = top_k ? top_k[r] : 0;
    if (k > 0 && k < V) {
        uint32_t lo = 0, hi = 0x3F800001u;  // count(>= lo) >= k holds, count(>= hi) = 0
        while (hi - lo > 1) {
            const uint32_t mid = lo + (hi - lo) / 2;
            double c = 0.0;
            for (int i = threadIdx.x; i < V; i += blockDim.x) c += __float_as_uint(E_OF(i)) >= mid ? 1.0 : 0.0;
            c = block_sum_f64(c, redd);
            if (c >= (double)k) lo = mid; else hi = mid;
        }
        thr = lo;
    }
    const float pp = top_p ? top_p[r] : 1.0f;
    if (pp < 1.0f) {
        double z = 0.0;
        for (int i = threadIdx.x; i < V; i += blockDim.x) {
            const float e = E_OF(i);
            if (__float_as_uint(e) >= thr) z += (double)e;
        }
        z = block_sum_f64(z, redd);
        const double need = (double)pp * z;
        uint32_t lo = thr, hi = 0x3F800001u;  // mass(>= lo) = z >= need; mass(>= hi) = 0
        while (hi - lo > 1) {
            const uint32_t mid = lo + (hi - lo) / 2;
            double c = 0.0;
            for (int i = threadIdx.x; i < V; i += blockDim.x) {
                const float e = E_OF(i);
                if (__float_as_uint(e) >= mid) c += (double)e;
            }
            c = block_sum_f64(c, redd);
            if (c >= need) lo = mid; else hi = mid;
        }
        thr = lo;
    }
    const float mp = min_p ? min_p[r] : 0.0f;
    if (mp > 0.f) {
        const uint32_t b = __float_as_uint(mp);  // e_max = 1
        if (b > thr) thr = b;
    }
    // contiguous segment per thread, so the cumulative sum runs in index order
    const int per = (V + blockDim.x - 1) / blockDim.x;
    const int beg = min(V, (int)threadIdx.x * per), end = min(V, beg + per);
    double mine = 0.0;
    for (int i = beg; i < end; ++i) {
        const float e = E_OF(i);
        if (__float_as_uint(e) >= thr) mine += (double)e;
    }
    seg[threadIdx.x] = mine;
    if (threadIdx.x == 0) chosen = -1;
    __syncthreads();
    if (threadIdx.x == 0) {
        double run = 0.0;
        for (int i = 0; i < (int)blockDim.x; ++i) { const double s = seg[i]; seg[i] = run; run += s; }
        redd[16] = run;
    }
    __syncthreads();
    const double total = redd[16];
    const double target = (double)uniform[r] * total;
    const double before = seg[threadIdx.x];
    if (mine > 0.0 && before <= target && target < before + mine) {
        double c = before;
        int pick = -1, last = -1;
        for (int i = beg; i < end; ++i) {
            const float e = E_OF(i);
            if (__float_as_uint(e) >= thr && e > 0.f) {
                last = i;
                c += (double)e;
                if (target < c) { pick = i; break; }
            }
        }
        chosen = pick >= 0 ? pick : last;
    }
    __syncthreads();
    if (threadIdx.x == 0) out[r] = chosen >= 0 ? chosen : amax;  // target == total: rounding at the very end
    if (probs_out) {
        for (int i = threadIdx.x; i < V; i += blockDim.x) {
            const float e = E_OF(i);
            probs_out[(size_t)r * V + i] = __float_as_uint(e) >= thr ? (float)((double)e / total) : 0.f;
        }
    }
#undef E_OF
}

TFF_API int tff_sample(const float* logits, int32_t* out, int rows, int V, const float* temperature,
                       const int32_t* top_k, const float* top_p, const float* min_p,
                       const float* uniform, float* probs_out, tff_stream_t stream) {
    TFF_REQUIRE(logits && out && temperature && uniform, "sample: null pointer");
    TFF_REQUIRE(rows >= 0 && V > 0, "sample: bad sizes rows=%d V=%d", rows, V);
    if (rows == 0) return 0;
    sample_kernel<<<rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(
        logits, out, V, temperature, top_k, top_p, min_p, uniform, probs_out);
    return tff_check_launch("sample");
}
