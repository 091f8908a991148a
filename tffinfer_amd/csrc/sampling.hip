// Token choice on the device: argmax, repetition penalty, and a draw from the
// temperature softmax under top-k / top-p / min-p.
//
// The reference chooses on the CPU: std::max_element for greedy
// (src/core/sampler/LLMSampler.cpp:43-45), logits * 1/temp (:36-41), the
// penalty of seen tokens (:21-34), a discrete draw (:47-54); top_k, top_p and
// min_p are fields of its SamplingConfig (LLMSampler.h:55-63).  Here one block
// works on one row of float32 logits.  Thresholds are found by a radix search
// over the bit patterns of the unnormalised probabilities e_i = exp((l_i - max)/temp)
// instead of a sort (histograms of 11, 11 and 8 bits: two passes over the row as a rule);
// sums that decide a threshold or the drawn index are sums of integers, so the same
// row and the same uniform number give the same token in any batch.
#include "common.h"
#include "tffinfer_kernels.h"

#define SAMPLE_THREADS 1024

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
    // A thread meets its elements in the order of their indices (those before the aligned part, the
    // aligned part, those after it), so "greater" alone keeps the first of equal maxima.
    if ((int)threadIdx.x < head && x[threadIdx.x] > best) { best = x[threadIdx.x]; arg = threadIdx.x; }
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
                if (v[u].x > best) { best = v[u].x; arg = i; }
                if (v[u].y > best) { best = v[u].y; arg = i + 1; }
                if (v[u].z > best) { best = v[u].z; arg = i + 2; }
                if (v[u].w > best) { best = v[u].w; arg = i + 3; }
            }
        }
    }
    {
        const int i = head + 4 * nvec + (int)threadIdx.x;   // (at most three elements after the aligned part)
        if (i < V && x[i] > best) { best = x[i]; arg = i; }
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

// A few rows of a large vocabulary: one block a row reads at what one CU pulls (some 50 GB/s: 12 us
// for 152k logits).  The row is then cut into ARGMAX_CHUNKS runs, a block each, and a second kernel
// takes the first of the runs' maxima.
#define ARGMAX_CHUNKS 32
__global__ __launch_bounds__(256) void argmax_chunk_kernel(const float* __restrict__ logits, float* __restrict__ part_v,
                                                           int32_t* __restrict__ part_i, int V) {
    __shared__ float redv[17];
    __shared__ int redi[17];
    const int r = blockIdx.y, c = blockIdx.x;
    const int per = (V + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
    const int i0 = min(V, c * per), n = min(V, i0 + per) - i0;
    float mx = -INFINITY;
    int a = 0x7fffffff;
    if (n > 0) {
        a = block_argmax(logits + (size_t)r * V + i0, n, redv, redi, &mx);
        if (a != 0x7fffffff) a += i0;
    }
    if (threadIdx.x == 0) {
        part_v[r * ARGMAX_CHUNKS + c] = a == 0x7fffffff ? -INFINITY : mx;
        part_i[r * ARGMAX_CHUNKS + c] = a;
    }
}
__global__ __launch_bounds__(64) void argmax_merge_kernel(const float* __restrict__ part_v, const int32_t* __restrict__ part_i,
                                                          int32_t* __restrict__ out) {
    static_assert(ARGMAX_CHUNKS <= 64, "a lane a run");
    const int r = blockIdx.x, lane = threadIdx.x;
    float best = lane < ARGMAX_CHUNKS ? part_v[r * ARGMAX_CHUNKS + lane] : -INFINITY;
    int arg = lane < ARGMAX_CHUNKS ? part_i[r * ARGMAX_CHUNKS + lane] : 0x7fffffff;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(arg, o, 64);
        if (ov > best || (ov == best && oi < arg)) { best = ov; arg = oi; }
    }
    if (lane == 0) out[r] = arg == 0x7fffffff ? 0 : arg;
}

TFF_API size_t tff_argmax_workspace_bytes(int rows, int V) {
    // few rows, many columns: the two-kernel form (with more rows than CUs to spare a block a row keeps them all busy)
    return (rows > 0 && rows <= 64 && V >= 32768) ? (size_t)rows * ARGMAX_CHUNKS * 8 : 0;
}

// workspace: tff_argmax_workspace_bytes(rows, V) bytes (16-byte aligned), or null for the one-kernel form.
TFF_API int tff_argmax(const float* logits, int32_t* out, int rows, int V, void* workspace, tff_stream_t stream) {
    TFF_REQUIRE(logits && out, "argmax: null pointer");
    TFF_REQUIRE(rows >= 0 && V > 0, "argmax: bad sizes rows=%d V=%d", rows, V);
    if (rows == 0) return 0;
    if (workspace && tff_argmax_workspace_bytes(rows, V) > 0) {
        float* pv = (float*)workspace;
        int32_t* pi = (int32_t*)(pv + (size_t)rows * ARGMAX_CHUNKS);
        argmax_chunk_kernel<<<dim3(ARGMAX_CHUNKS, rows), 256, 0, (hipStream_t)stream>>>(logits, pv, pi, V);
        if (int rc = tff_check_launch("argmax")) return rc;
        argmax_merge_kernel<<<rows, 64, 0, (hipStream_t)stream>>>(pv, pi, out);
        return tff_check_launch("argmax");
    }
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

// ---- the draw ----
// The unnormalised probabilities e_i = exp((l_i - max) / temp) lie in [0, 1]; their bit patterns
// (30 bits) order them.  Every sum of probabilities is a sum of the integers floor(e_i 2^40): it does
// not depend on the order of its terms, so counts and sums may come from LDS atomics and any tree
// of partial sums, and the same row and the same uniform number give the same token in any batch.
// (152k tokens of weight 2^40 stay far below 2^64; what is lost, 2^-41 a token, is 7e-8 of the
// largest probability over the whole vocabulary.)
// inv_t2 = log2(e) / temp: the exponential is the hardware's 2^x, one instruction (a pass over the
// row is bound by its arithmetic, not by memory).  x = max gives exactly 1.
__device__ __forceinline__ uint32_t sample_key(float x, float mx, float inv_t2) {
    const float e = __builtin_amdgcn_exp2f((x - mx) * inv_t2);
    return __float_as_uint(fmaxf(e, 0.f));          // (a NaN logit weighs nothing)
}
__device__ __forceinline__ unsigned long long sample_mass(uint32_t key) {
    return (unsigned long long)(__uint_as_float(key) * 0x1p40f);
}

// f4(j, v) for every aligned group of four elements of the row (x[head + 4 j ..]) and f1(i, x[i]) for
// the elements before and after the aligned part, each once, in no particular order: 16-byte loads,
// eight in flight per thread (a block has the row to itself: what counts is loads in flight).
template <typename F4, typename F1>
__device__ __forceinline__ void row_for_each4(const float* __restrict__ x, int V, F4 f4, F1 f1) {
    const int head = min(V, (int)(((16 - ((uintptr_t)x & 15)) & 15) / 4));
    const int nvec = (V - head) / 4;
    const float4* x4 = reinterpret_cast<const float4*>(x + head);
    constexpr int UN = 8;
    for (int i0 = threadIdx.x; i0 < nvec; i0 += UN * blockDim.x) {
        float4 v[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) v[u] = x4[min(i0 + u * (int)blockDim.x, nvec - 1)];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int j = i0 + u * blockDim.x;
            if (j < nvec) f4(j, v[u]);
        }
    }
    for (int t = threadIdx.x; t < V - 4 * nvec; t += blockDim.x) {
        const int i = t < head ? t : t + 4 * nvec;
        f1(i, x[i]);
    }
}
template <typename F>
__device__ __forceinline__ void row_for_each(const float* __restrict__ x, int V, F f) {
    row_for_each4(
        x, V,
        [&](int, const float4& v) {
            f(v.x);
            f(v.y);
            f(v.z);
            f(v.w);
        },
        [&](int, float v) { f(v); });
}

__device__ __forceinline__ unsigned long long wave_scan_incl(unsigned long long v, int lane) {
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const unsigned long long up = __shfl_up(v, o, 64);
        if (lane >= o) v += up;
    }
    return v;
}

struct SampleCross {
    int bin;                                   // the highest bin whose suffix sum reaches what was asked for
    unsigned long long cnt_above, mass_above;  // counts and masses of the bins above it
    unsigned long long cnt_bin, mass_bin;      // and its own
};

// Bins of a histogram (counts and masses, nb of them, in LDS) from the top down: the first bin at
// which the running count (BY_COUNT) or mass reaches `need`.  need >= 1 and at most the total.
template <bool BY_COUNT>
__device__ SampleCross sample_find_crossing(const uint32_t* cnt, const unsigned long long* mass, int nb,
                                            unsigned long long need, unsigned long long* red,
                                            SampleCross* shared) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nwave = (blockDim.x + 63) >> 6;
    const int per = (nb + (int)blockDim.x - 1) / (int)blockDim.x;
    // thread t takes the bins nb - 1 - (t per + u): threads in order walk the bins downwards
    unsigned long long c = 0, m = 0;
    for (int u = 0; u < per; ++u) {
        const int j = tid * per + u;
        if (j < nb) { c += cnt[nb - 1 - j]; m += mass[nb - 1 - j]; }
    }
    const unsigned long long ci = wave_scan_incl(c, lane), mi = wave_scan_incl(m, lane);
    if (tid == 0) *shared = SampleCross{0, 0, 0, 0, 0};
    __syncthreads();
    if (lane == 63) { red[wave] = ci; red[16 + wave] = mi; }
    __syncthreads();
    unsigned long long c0 = ci - c, m0 = mi - m;   // what lies above this thread's bins
    for (int w = 0; w < wave && w < nwave; ++w) { c0 += red[w]; m0 += red[16 + w]; }
    for (int u = 0; u < per; ++u) {
        const int j = tid * per + u;
        if (j >= nb) break;
        const unsigned long long cb = cnt[nb - 1 - j], mb = mass[nb - 1 - j];
        const unsigned long long have = BY_COUNT ? c0 : m0, with = BY_COUNT ? c0 + cb : m0 + mb;
        if (have < need && with >= need) *shared = SampleCross{nb - 1 - j, c0, m0, cb, mb};
        c0 += cb;
        m0 += mb;
    }
    __syncthreads();
    const SampleCross r = *shared;
    __syncthreads();
    return r;
}

#define SAMPLE_LIST 4096  // keys of one bin of the first histogram that LDS holds

// The largest bit pattern thr with  count(e >= thr) >= need  (BY_COUNT)  or  mass(e >= thr) >=
// frac x (the mass of all of them), over the elements with e >= floor_key.  A radix search over the
// 30 bits: a histogram of the top 11 bits (one pass over the row), then the keys of the bin that
// holds the threshold are gathered into LDS (a second pass) and the histograms of the next 11 and
// the last 8 bits are taken from there; a bin with more keys than LDS holds (a row of equal
// logits) is worked through by passes over the row instead.
template <bool BY_COUNT>
__device__ uint32_t sample_threshold(const float* __restrict__ x, int V, float mx, float inv_t, uint32_t floor_key,
                                     unsigned long long need, float frac, uint32_t* cnt, unsigned long long* mass,
                                     uint32_t* list, int* list_n, unsigned long long* red, SampleCross* shared) {
    uint32_t prefix = 0, known = 0;            // the bits found so far, and a mask of them
    const int shifts[3] = {19, 8, 0}, widths[3] = {11, 11, 8};
    int n_list = -1;                           // keys in LDS (-1: none, the row is read)
#pragma unroll
    for (int level = 0; level < 3; ++level) {
        const int shift = shifts[level], nb = 1 << widths[level];
        for (int b = threadIdx.x; b < nb; b += blockDim.x) { cnt[b] = 0; mass[b] = 0; }
        __syncthreads();
        auto count_key = [&](uint32_t key) {
            if ((key & known) == prefix && key >= floor_key) {
                const int b = (key >> shift) & (nb - 1);
                atomicAdd(&cnt[b], 1u);
                if (!BY_COUNT) atomicAdd(&mass[b], sample_mass(key));
            }
        };
        if (n_list >= 0) {
            for (int i = threadIdx.x; i < n_list; i += blockDim.x) count_key(list[i]);
        } else {
            row_for_each(x, V, [&](float v) { count_key(sample_key(v, mx, inv_t)); });
        }
        __syncthreads();
        if (level == 0 && !BY_COUNT) {
            // what is asked for is a share of everything there is
            unsigned long long m = 0;
            for (int b = threadIdx.x; b < nb; b += blockDim.x) m += mass[b];
            m = wave_scan_incl(m, threadIdx.x & 63);
            if ((threadIdx.x & 63) == 63) red[threadIdx.x >> 6] = m;
            __syncthreads();
            unsigned long long z = 0;
            for (int w = 0; w < (int)(blockDim.x >> 6); ++w) z += red[w];
            __syncthreads();
            need = (unsigned long long)((double)fmaxf(frac, 0.f) * (double)z);
        }
        if (need < 1) need = 1;
        const SampleCross c = sample_find_crossing<BY_COUNT>(cnt, mass, nb, need, red, shared);
        need -= BY_COUNT ? c.cnt_above : c.mass_above;
        prefix |= (uint32_t)c.bin << shift;
        known |= (uint32_t)(nb - 1) << shift;
        if (level == 0 && c.cnt_bin <= SAMPLE_LIST) {
            if (threadIdx.x == 0) *list_n = 0;
            __syncthreads();
            row_for_each(x, V, [&](float v) {
                const uint32_t key = sample_key(v, mx, inv_t);
                if ((key & known) == prefix && key >= floor_key) list[atomicAdd(list_n, 1)] = key;
            });
            __syncthreads();
            n_list = *list_n;                  // (= c.cnt_bin; their order does not matter)
        }
    }
    return prefix;
}

#define SAMPLE_TILES 256  // tiles of 256 elements in a wave's run of the row, at most
#define SAMPLE_MAX_V (SAMPLE_TILES * 256 * (SAMPLE_THREADS / 64))

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int32_t* __restrict__ out, int V,
    const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ top_p, const float* __restrict__ min_p,
    const float* __restrict__ uniform, float* __restrict__ probs_out) {
    constexpr int NWAVE = SAMPLE_THREADS / 64;
    static_assert(SAMPLE_TILES % 64 == 0, "the tiles of a run go round the lanes of a wave");
    __shared__ float redv[17];
    __shared__ int redi[17];
    __shared__ uint32_t cnt[2048];
    __shared__ unsigned long long mass[2048];
    __shared__ uint32_t list[SAMPLE_LIST];
    __shared__ unsigned long long red[32];
    __shared__ SampleCross cross;
    __shared__ unsigned long long run_mass[NWAVE + 2];   // and the elements before and after the aligned part
    __shared__ unsigned long long tile_mass[SAMPLE_TILES];
    __shared__ int chosen, list_n;
    const int r = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float* x = logits + (size_t)r * V;
    const float temp = temperature[r];
    float mx;
    const int amax = block_argmax(x, V, redv, redi, &mx);
    if (temp <= 0.f || amax == 0x7fffffff) {
        if (tid == 0) out[r] = amax == 0x7fffffff ? 0 : amax;
        if (probs_out)
            for (int i = tid; i < V; i += blockDim.x) probs_out[(size_t)r * V + i] = i == amax ? 1.f : 0.f;
        return;
    }
    const float inv_t = 1.4426950408889634f / temp;   // log2(e) / temp, see sample_key
    uint32_t thr = 0;  // keep e_i with bits >= thr
    const int k = top_k ? top_k[r] : 0;
    if (k > 0 && k < V)
        thr = sample_threshold<true>(x, V, mx, inv_t, 0u, (unsigned long long)k, 0.f, cnt, mass, list, &list_n, red, &cross);
    const float pp = top_p ? top_p[r] : 1.0f;
    if (pp < 1.0f)   // the smallest set of the most likely of what is kept so far that holds pp of its mass
        thr = sample_threshold<false>(x, V, mx, inv_t, thr, 0ull, pp, cnt, mass, list, &list_n, red, &cross);
    const float mp = min_p ? min_p[r] : 0.0f;
    if (mp > 0.f) {
        const uint32_t b = __float_as_uint(mp);  // e_max = 1
        if (b > thr) thr = b;
    }
    // The draw, by inverse CDF in index order.  The aligned part of the row is cut into a run for each
    // wave, which adds up what its run weighs (integers: in any order); the run that holds the target is
    // cut into tiles of 256 elements, whose sums the waves take between them, and the tile that holds it
    // is walked through by one wave.
    const int head = min(V, (int)(((16 - ((uintptr_t)x & 15)) & 15) / 4));
    const int nvec = (V - head) / 4;
    const float4* x4 = reinterpret_cast<const float4*>(x + head);
    auto run_begin = [&](int w) { return (int)(((long long)nvec * w) / NWAVE); };
    auto kept = [&](float v) {
        const uint32_t key = sample_key(v, mx, inv_t);
        return key >= thr ? sample_mass(key) : 0ull;
    };
    auto kept4 = [&](const float4& v) { return kept(v.x) + kept(v.y) + kept(v.z) + kept(v.w); };
    {
        const int j0 = run_begin(wave), j1 = run_begin(wave + 1);
        unsigned long long m = 0;
        constexpr int UN = 8;
        for (int jb = j0 + lane; jb < j1; jb += 64 * UN) {
            float4 v[UN];
#pragma unroll
            for (int u = 0; u < UN; ++u) v[u] = x4[min(jb + 64 * u, j1 - 1)];
#pragma unroll
            for (int u = 0; u < UN; ++u)
                if (jb + 64 * u < j1) m += kept4(v[u]);
        }
        m = wave_scan_incl(m, lane);
        if (lane == 63) run_mass[wave] = m;
    }
    if (tid == 0) {
        unsigned long long mh = 0, mt = 0;
        for (int i = 0; i < head; ++i) mh += kept(x[i]);
        for (int i = head + 4 * nvec; i < V; ++i) mt += kept(x[i]);
        run_mass[NWAVE] = mh;
        run_mass[NWAVE + 1] = mt;
        chosen = -1;
    }
    __syncthreads();
    // in order: the elements before the aligned part, the runs, the elements after it (every thread works this out)
    const unsigned long long mh = run_mass[NWAVE], mt = run_mass[NWAVE + 1];
    unsigned long long total = mh + mt;
    for (int w = 0; w < NWAVE; ++w) total += run_mass[w];
    unsigned long long target = (unsigned long long)((double)uniform[r] * (double)total);
    if (total > 0 && target >= total) target = total - 1;
    int part = -3;                                          // -3: nothing weighs anything
    unsigned long long before = 0;
    if (total > 0) {
        if (target < mh) {
            part = -1;
        } else if (target >= total - mt) {
            part = -2;
            before = total - mt;
        } else {
            unsigned long long acc = mh;
            for (int w = 0; w < NWAVE; ++w) {
                const unsigned long long m = run_mass[w];
                if (part == -3 && m > 0 && target < acc + m) { part = w; before = acc; }
                acc += m;
            }
        }
    }
    if (part >= 0) {
        const int j0 = run_begin(part), j1 = run_begin(part + 1);
        const int T = (j1 - j0 + 63) / 64;                  // at most SAMPLE_TILES: the entry point checks V
        for (int t = wave; t < T; t += NWAVE) {
            const int j = j0 + 64 * t + lane;
            unsigned long long m = j < j1 ? kept4(x4[j]) : 0ull;
            m = wave_scan_incl(m, lane);
            if (lane == 63) tile_mass[t] = m;
        }
        __syncthreads();
        if (wave == 0) {
            constexpr int TPL = SAMPLE_TILES / 64;          // tiles a lane
            unsigned long long s[TPL], mine = 0;
#pragma unroll
            for (int q = 0; q < TPL; ++q) {
                s[q] = TPL * lane + q < T ? tile_mass[TPL * lane + q] : 0ull;
                mine += s[q];
            }
            const unsigned long long incl = wave_scan_incl(mine, lane);
            unsigned long long b0 = before + incl - mine;
            const bool hit = mine > 0 && b0 <= target && target < b0 + mine;
            int tq = 0;
            if (hit) {
                bool found = false;
#pragma unroll
                for (int q = 0; q < TPL; ++q) {
                    if (!found && s[q] > 0 && target < b0 + s[q]) { tq = TPL * lane + q; found = true; }
                    if (!found) b0 += s[q];
                }
            }
            const unsigned long long bal = __ballot(hit);
            if (bal) {
                const int src = __ffsll((long long)bal) - 1;
                tq = __shfl(tq, src, 64);
                b0 = __shfl(b0, src, 64);
                const int j = j0 + 64 * tq + lane;
                const bool in = j < j1;
                const float4 v = x4[min(j, j1 - 1)];
                const unsigned long long m0 = in ? kept(v.x) : 0ull, m1 = in ? kept(v.y) : 0ull,
                                         m2 = in ? kept(v.z) : 0ull, m3 = in ? kept(v.w) : 0ull;
                const unsigned long long mine4 = m0 + m1 + m2 + m3;
                const unsigned long long bl = b0 + wave_scan_incl(mine4, lane) - mine4;
                if (mine4 > 0 && bl <= target && target < bl + mine4) {
                    const int i = head + 4 * j;
                    int pick = i + 3;
                    if (target < bl + m0) pick = i;
                    else if (target < bl + m0 + m1) pick = i + 1;
                    else if (target < bl + m0 + m1 + m2) pick = i + 2;
                    chosen = pick;
                }
            }
        }
    } else if (part > -3 && tid == 0) {
        unsigned long long run = before;
        const int i0 = part == -1 ? 0 : head + 4 * nvec, i1 = part == -1 ? head : V;
        for (int i = i0; i < i1; ++i) {
            const unsigned long long m = kept(x[i]);
            if (m > 0 && target < run + m) { chosen = i; break; }
            run += m;
        }
    }
    __syncthreads();
    if (tid == 0) out[r] = chosen >= 0 ? chosen : amax;
    if (probs_out) {
        // (as floats: a token too unlikely to weigh anything in the draw still shows its probability)
        const double tot = total > 0 ? (double)total * 0x1p-40 : 1.0;
        for (int i = tid; i < V; i += blockDim.x) {
            const uint32_t key = sample_key(x[i], mx, inv_t);
            probs_out[(size_t)r * V + i] = key >= thr ? (float)((double)__uint_as_float(key) / tot) : 0.f;
        }
    }
}

TFF_API int tff_sample(const float* logits, int32_t* out, int rows, int V, const float* temperature,
                       const int32_t* top_k, const float* top_p, const float* min_p,
                       const float* uniform, float* probs_out, tff_stream_t stream) {
    TFF_REQUIRE(logits && out && temperature && uniform, "sample: null pointer");
    TFF_REQUIRE(rows >= 0 && V > 0, "sample: bad sizes rows=%d V=%d", rows, V);
    TFF_REQUIRE(V <= SAMPLE_MAX_V, "sample: a vocabulary of %d is more than the %d the draw is laid out for", V,
                SAMPLE_MAX_V);
    if (rows == 0) return 0;
    sample_kernel<<<rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(
        logits, out, V, temperature, top_k, top_p, min_p, uniform, probs_out);
    return tff_check_launch("sample");
}
