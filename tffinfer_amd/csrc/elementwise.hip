// Row-wise and element-wise kernels: embedding gather, fused residual sum and
// RMS norm, per-head q/k norm with rotation and the cache write, SwiGLU, casts.
// All arithmetic is float32; only loads and stores see bfloat16.
#include "common.h"
#include "tffinfer_kernels.h"

#include <stdarg.h>
#include <stdio.h>

// ---------------------------------------------------------------- errors ---
static thread_local char g_error[1024] = "";

int tff_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return -1;
}
int tff_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return tff_fail("%s: launch failed: %s", what, hipGetErrorString(e));
    return 0;
}
TFF_API const char* tff_last_error() { return g_error; }
TFF_API int tff_abi_version() { return 21; }

// ----------------------------------------------------------------- embed ---
// x[t, :] = E[token[t], :]   (reference: src/kernel/cpu/embedding.cpp:34-49,
// done there on the CPU; here a gather on the device into the float32
// residual stream).
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int32_t* __restrict__ ids,
                             float* __restrict__ out, int H, int V) {
    const int t = blockIdx.x;
    int id = ids[t];
    const bool bad = id < 0 || id >= V;
    if (bad) id = 0;
    const T* row = table + (size_t)id * H;
    float* o = out + (size_t)t * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) o[j] = bad ? __builtin_nanf("") : to_f32(row[j]);
}

TFF_API int tff_embed(const void* table, const int32_t* ids, float* out, int T, int H, int V,
                      int dtype, tff_stream_t stream) {
    TFF_REQUIRE(table && ids && out, "embed: null pointer");
    TFF_REQUIRE(T >= 0 && H > 0 && V > 0, "embed: bad sizes T=%d H=%d V=%d", T, H, V);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TFF_F32)
        embed_kernel<float><<<T, 256, 0, s>>>((const float*)table, ids, out, H, V);
    else if (dtype == TFF_BF16)
        embed_kernel<bf16_t><<<T, 256, 0, s>>>((const bf16_t*)table, ids, out, H, V);
    else
        return tff_fail("embed: unknown dtype %d", dtype);
    return tff_check_launch("embed");
}

// ----------------------------------------------------------- add+rmsnorm ---
// y_j = v_j * rsqrt(mean(v^2) + eps) * w_j, v = resid (+ delta)
// (reference: src/kernel/cuda/norm.cu:31-48; the residual sum of
// src/kernel/cuda/binary.cu:16-29 is folded in).
// delta may come as `planes` partial sums, `plane` elements apart, which are added up first,
// plane 0, 1, ... in turn.
template <typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const float* __restrict__ delta,
                                   int planes, size_t plane, const float* __restrict__ w, float eps,
                                   TO* __restrict__ out, const int32_t* __restrict__ rows, int H) {
    __shared__ float red[17];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    float* x = resid + (size_t)r * H;
    const float* dl = delta ? delta + (size_t)r * H : nullptr;
    const bool store = rows == nullptr && dl != nullptr;
    float ss = 0.f;
    for (int j = threadIdx.x; j < H; j += blockDim.x) {
        float v = x[j];
        if (dl) {
            float d = dl[j];
            for (int p = 1; p < planes; ++p) d += dl[p * plane + j];
            v += d;
        }
        if (store) x[j] = v;
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, red);
    const float rr = rsqrtf(ss / (float)H + eps);
    TO* o = out + (size_t)i * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) {
        float v = x[j];
        if (dl && !store) {
            float d = dl[j];
            for (int p = 1; p < planes; ++p) d += dl[p * plane + j];
            v += d;
        }
        o[j] = from_f32<TO>(v * rr * w[j]);
    }
}

// The same for rows whose width is a multiple of 4: 16-byte accesses, and rows of up to 4096
// elements pass through memory once (the sum is kept in registers for the second sweep).
template <typename TO>
__device__ __forceinline__ void store_out4(TO* o, float4 v);
template <>
__device__ __forceinline__ void store_out4<float>(float* o, float4 v) { *reinterpret_cast<float4*>(o) = v; }
template <>
__device__ __forceinline__ void store_out4<bf16_t>(bf16_t* o, float4 v) {
    union { bf16_t h[4]; uint2 u; } pk;
    pk.h[0] = (bf16_t)v.x; pk.h[1] = (bf16_t)v.y; pk.h[2] = (bf16_t)v.z; pk.h[3] = (bf16_t)v.w;
    *reinterpret_cast<uint2*>(o) = pk.u;
}

// planes are added in their order; four loads are in flight at a time
__device__ __forceinline__ float4 delta_sum4(const float4* d4, int j, int planes, size_t plane4) {
    float4 d = d4[j];
    for (int p = 1; p < planes; p += 4) {
        float4 e[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
            e[u] = p + u < planes ? d4[(size_t)(p + u) * plane4 + j] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (p + u < planes) { d.x += e[u].x; d.y += e[u].y; d.z += e[u].z; d.w += e[u].w; }
    }
    return d;
}

// NT threads a row: 256, or 1024 where there are few rows (more loads in flight for each)
template <typename TO, int NT>
__global__ __launch_bounds__(NT) void add_rmsnorm_vec_kernel(float* __restrict__ resid,
                                                               const float* __restrict__ delta,
                                                               int planes, size_t plane,
                                                               const float* __restrict__ w, float eps,
                                                               TO* __restrict__ out,
                                                               const int32_t* __restrict__ rows, int H) {
    const size_t plane4 = plane >> 2;
    __shared__ float red[17];
    const int i = blockIdx.x, tid = threadIdx.x;
    const int r = rows ? rows[i] : i;
    const int H4 = H >> 2;
    float4* x4 = reinterpret_cast<float4*>(resid + (size_t)r * H);
    const float4* d4 = delta ? reinterpret_cast<const float4*>(delta + (size_t)r * H) : nullptr;
    const float4* w4 = reinterpret_cast<const float4*>(w);
    const bool store = rows == nullptr && d4 != nullptr;
    constexpr int ITS = 1024 / NT;
    float4 cache[ITS];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < ITS; ++it) {
        const int j = tid + it * NT;
        if (j < H4) {
            float4 v = x4[j];
            if (d4) { const float4 dv = delta_sum4(d4, j, planes, plane4); v.x += dv.x; v.y += dv.y; v.z += dv.z; v.w += dv.w; }
            if (store) x4[j] = v;
            cache[it] = v;
            ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
        }
    }
    for (int j = tid + 1024; j < H4; j += NT) {
        float4 v = x4[j];
        if (d4) { const float4 dv = delta_sum4(d4, j, planes, plane4); v.x += dv.x; v.y += dv.y; v.z += dv.z; v.w += dv.w; }
        if (store) x4[j] = v;
        ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
    }
    ss = block_sum(ss, red);
    const float rr = rsqrtf(ss / (float)H + eps);
    TO* o = out + (size_t)i * H;
#pragma unroll
    for (int it = 0; it < ITS; ++it) {
        const int j = tid + it * NT;
        if (j < H4) {
            const float4 v = cache[it], wv = w4[j];
            store_out4<TO>(o + 4 * j, make_float4(v.x * rr * wv.x, v.y * rr * wv.y, v.z * rr * wv.z, v.w * rr * wv.w));
        }
    }
    for (int j = tid + 1024; j < H4; j += NT) {
        float4 v = x4[j];
        if (d4 && !store) { const float4 dv = delta_sum4(d4, j, planes, plane4); v.x += dv.x; v.y += dv.y; v.z += dv.z; v.w += dv.w; }
        const float4 wv = w4[j];
        store_out4<TO>(o + 4 * j, make_float4(v.x * rr * wv.x, v.y * rr * wv.y, v.z * rr * wv.z, v.w * rr * wv.w));
    }
}

TFF_API int tff_add_rmsnorm(float* resid, const float* delta, int delta_planes, size_t delta_plane,
                            const float* weight, float eps, void* out, const int32_t* rows, int n,
                            int H, int out_dtype, tff_stream_t stream) {
    TFF_REQUIRE(resid && weight && out, "add_rmsnorm: null pointer");
    TFF_REQUIRE(n >= 0 && H > 0, "add_rmsnorm: bad sizes n=%d H=%d", n, H);
    TFF_REQUIRE(!delta || (delta_planes >= 1 && (delta_planes == 1 || delta_plane % 4 == 0)),
                "add_rmsnorm: %d planes of partial sums, %zu elements apart", delta_planes, delta_plane);
    const int planes = delta ? delta_planes : 0;
    const size_t plane = delta_plane;
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    TFF_REQUIRE(out_dtype == TFF_F32 || out_dtype == TFF_BF16, "add_rmsnorm: unknown dtype %d", out_dtype);
    const bool vec = H % 4 == 0 && ((uintptr_t)resid % 16) == 0 && ((uintptr_t)weight % 16) == 0 &&
                     ((uintptr_t)out % 16) == 0 && (!delta || ((uintptr_t)delta % 16) == 0);
    if (vec) {
        const bool wide = n <= 128 && H >= 2048;
        if (out_dtype == TFF_F32) {
            if (wide) add_rmsnorm_vec_kernel<float, 1024><<<n, 1024, 0, s>>>(resid, delta, planes, plane, weight, eps, (float*)out, rows, H);
            else add_rmsnorm_vec_kernel<float, 256><<<n, 256, 0, s>>>(resid, delta, planes, plane, weight, eps, (float*)out, rows, H);
        } else {
            if (wide) add_rmsnorm_vec_kernel<bf16_t, 1024><<<n, 1024, 0, s>>>(resid, delta, planes, plane, weight, eps, (bf16_t*)out, rows, H);
            else add_rmsnorm_vec_kernel<bf16_t, 256><<<n, 256, 0, s>>>(resid, delta, planes, plane, weight, eps, (bf16_t*)out, rows, H);
        }
        return tff_check_launch("add_rmsnorm");
    }
    const int threads = H >= 2048 ? 1024 : 256;
    if (out_dtype == TFF_F32)
        add_rmsnorm_kernel<float><<<n, threads, 0, s>>>(resid, delta, planes, plane, weight, eps, (float*)out, rows, H);
    else
        add_rmsnorm_kernel<bf16_t><<<n, threads, 0, s>>>(resid, delta, planes, plane, weight, eps, (bf16_t*)out, rows, H);
    return tff_check_launch("add_rmsnorm");
}

template <typename T>
__global__ void rmsnorm_kernel(const T* __restrict__ x, const float* __restrict__ w, float eps,
                               T* __restrict__ out, int H) {
    __shared__ float red[17];
    const T* xr = x + (size_t)blockIdx.x * H;
    float ss = 0.f;
    for (int j = threadIdx.x; j < H; j += blockDim.x) {
        const float v = to_f32(xr[j]);
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, red);
    const float rr = rsqrtf(ss / (float)H + eps);
    T* o = out + (size_t)blockIdx.x * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) o[j] = from_f32<T>(to_f32(xr[j]) * rr * w[j]);
}

TFF_API int tff_rmsnorm(const void* x, const float* weight, float eps, void* out, int n, int H,
                        int dtype, tff_stream_t stream) {
    TFF_REQUIRE(x && weight && out, "rmsnorm: null pointer");
    TFF_REQUIRE(n >= 0 && H > 0, "rmsnorm: bad sizes n=%d H=%d", n, H);
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TFF_F32)
        rmsnorm_kernel<float><<<n, 256, 0, s>>>((const float*)x, weight, eps, (float*)out, H);
    else if (dtype == TFF_BF16)
        rmsnorm_kernel<bf16_t><<<n, 256, 0, s>>>((const bf16_t*)x, weight, eps, (bf16_t*)out, H);
    else
        return tff_fail("rmsnorm: unknown dtype %d", dtype);
    return tff_check_launch("rmsnorm");
}

// ------------------------------------------------- q/k norm, rotation, kv ---
// One wave per (token, head).  q and k heads: RMS norm over d with a [d]
// weight shared by all heads (reference: src/core/model/qwen3/QWen3Creator.cpp:93-101),
// then the rotation x'_a = x_a cos - x_b sin, x'_b = x_a sin + x_b cos
// (src/kernel/cuda/paged_flash_attention.cu:343-355) with (cos, sin) from a
// table indexed by the token's position (src/kernel/cuda/rope_table.cu:32-36).
// The reference stores k before the rotation and rotates at every read
// (QWen3Creator.cpp:104-120); storing it rotated once is the same product.
#define QK_MAX_D 512
template <typename T, typename TC>
__global__ void qk_norm_rope_kv_kernel(T* __restrict__ qkv, int nq, int nkv, int d,
                                       const float* __restrict__ qw, const float* __restrict__ kw,
                                       float eps, const float* __restrict__ cos_sin, int rot,
                                       int pairing, const int32_t* __restrict__ positions,
                                       const int32_t* __restrict__ slot_mapping,
                                       TC* __restrict__ k_cache, TC* __restrict__ v_cache,
                                       int page_size) {
    __shared__ float xs[QK_MAX_D];
    const int t = blockIdx.x;
    const int hh = blockIdx.y;
    const int lane = threadIdx.x;
    const int width = (nq + 2 * nkv) * d;
    T* x = qkv + (size_t)t * width + (size_t)hh * d;
    const int kind = hh < nq ? 0 : (hh < nq + nkv ? 1 : 2);  // q, k, v
    const int slot = slot_mapping[t];
    if (kind != 0 && slot < 0) return;

    TC* dst = nullptr;
    if (kind != 0) {
        const int head = kind == 1 ? hh - nq : hh - nq - nkv;
        const int page = slot / page_size, off = slot % page_size;
        TC* base = kind == 1 ? k_cache : v_cache;
        dst = base + (((size_t)page * nkv + head) * page_size + off) * d;
    }
    if (kind == 2) {
        // values are kept transposed, [page, kv head, element, slot]: the slots of one element
        // lie side by side, which is the order a matrix-core operand of P.V wants
        const int head = hh - nq - nkv;
        const int page = slot / page_size, off = slot % page_size;
        TC* vt = v_cache + ((size_t)page * nkv + head) * d * page_size + off;
        for (int e = lane; e < d; e += 64) vt[(size_t)e * page_size] = from_f32<TC>(to_f32(x[e]));
        return;
    }
    const float* w = kind == 0 ? qw : kw;
    float ss = 0.f;
    for (int e = lane; e < d; e += 64) {
        const float v = to_f32(x[e]);
        xs[e] = v;
        ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    __syncthreads();
    if (w) {
        const float rr = rsqrtf(ss / (float)d + eps);
        for (int e = lane; e < d; e += 64) xs[e] = xs[e] * rr * w[e];
        __syncthreads();
    }
    if (cos_sin) {
        const int pos = positions[t];
        const int half = rot >> 1;
        const float* cs = cos_sin + (size_t)pos * rot;  // [pos][pair][cos, sin]
        for (int p = lane; p < half; p += 64) {
            const int a = pairing == 0 ? p : 2 * p;
            const int b = pairing == 0 ? p + half : 2 * p + 1;
            const float c = cs[2 * p], s = cs[2 * p + 1];
            const float xa = xs[a], xb = xs[b];
            xs[a] = xa * c - xb * s;
            xs[b] = xa * s + xb * c;
        }
        __syncthreads();
    }
    if (kind == 0) {
        for (int e = lane; e < d; e += 64) x[e] = from_f32<T>(xs[e]);
    } else {
        for (int e = lane; e < d; e += 64) dst[e] = from_f32<TC>(xs[e]);
    }
}

// The same when the whole head is rotated (or nothing is): a lane holds both elements of its
// pairs, so norm and rotation stay in registers; four heads share a block.
template <typename T, typename TC>
__global__ __launch_bounds__(256) void qk_norm_rope_kv_reg_kernel(
    T* __restrict__ qkv, int nq, int nkv, int d, const float* __restrict__ qw,
    const float* __restrict__ kw, float eps, const float* __restrict__ cos_sin, int pairing,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slot_mapping,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache, int page_size) {
    const int t = blockIdx.x;
    const int hh = blockIdx.y * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (hh >= nq + 2 * nkv) return;
    const int width = (nq + 2 * nkv) * d;
    T* x = qkv + (size_t)t * width + (size_t)hh * d;
    const int kind = hh < nq ? 0 : (hh < nq + nkv ? 1 : 2);  // q, k, v
    const int slot = slot_mapping[t];
    if (kind != 0 && slot < 0) return;
    const int page = slot / page_size, off = slot % page_size;
    if (kind == 2) {
        const int head = hh - nq - nkv;
        TC* vt = v_cache + ((size_t)page * nkv + head) * d * page_size + off;
        for (int e = lane; e < d; e += 64) vt[(size_t)e * page_size] = from_f32<TC>(to_f32(x[e]));
        return;
    }
    const int half = d >> 1;
    float xa[4], xb[4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int p = lane + 64 * i;
        if (p < half) {
            const int a = pairing == 0 ? p : 2 * p, b = pairing == 0 ? p + half : 2 * p + 1;
            xa[i] = to_f32(x[a]);
            xb[i] = to_f32(x[b]);
            ss = fmaf(xa[i], xa[i], fmaf(xb[i], xb[i], ss));
        }
    }
    ss = wave_sum(ss);
    const float* w = kind == 0 ? qw : kw;
    const float rr = w ? rsqrtf(ss / (float)d + eps) : 1.f;
    const float* cs = cos_sin ? cos_sin + (size_t)positions[t] * d : nullptr;   // [pos][pair][cos, sin]
    TC* kdst = kind == 1 ? k_cache + (((size_t)page * nkv + (hh - nq)) * page_size + off) * d : nullptr;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int p = lane + 64 * i;
        if (p < half) {
            const int a = pairing == 0 ? p : 2 * p, b = pairing == 0 ? p + half : 2 * p + 1;
            float va = xa[i], vb = xb[i];
            if (w) { va = va * rr * w[a]; vb = vb * rr * w[b]; }
            if (cs) {
                const float c = cs[2 * p], sn = cs[2 * p + 1];
                const float ra = va * c - vb * sn, rb = va * sn + vb * c;
                va = ra; vb = rb;
            }
            if (kind == 0) { x[a] = from_f32<T>(va); x[b] = from_f32<T>(vb); }
            else { kdst[a] = from_f32<TC>(va); kdst[b] = from_f32<TC>(vb); }
        }
    }
}

// The values of 8 consecutive tokens and one kv head go to their (transposed) pages: where the 8
// slots are consecutive and start at a multiple of 8 in a page, a thread writes one element's 8
// tokens as one 16-byte run; else token by token.  (Blocks of qk_norm_rope_vec_kernel's grid.)
__device__ __forceinline__ void v_page_write_block(
    const bf16_t* __restrict__ qkv, int T, int nq, int nkv, int d, const int32_t* __restrict__ slot_mapping,
    bf16_t* __restrict__ v_cache, int page_size, int t0, int head) {
    __shared__ __attribute__((aligned(16))) bf16_t tile[8][QK_MAX_D];
    __shared__ int32_t slots[8];
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int width = (nq + 2 * nkv) * d;
    const int cpr = d / 8;   // 16-byte chunks per row
    if (tid < 8) slots[tid] = t0 + tid < T ? slot_mapping[t0 + tid] : -1;
    for (int i = tid; i < 8 * cpr; i += nthr) {
        const int tk = i / cpr, c = i % cpr;
        uint4 val = make_uint4(0, 0, 0, 0);
        if (t0 + tk < T)
            val = *reinterpret_cast<const uint4*>(qkv + (size_t)(t0 + tk) * width + (size_t)(nq + nkv + head) * d + c * 8);
        *reinterpret_cast<uint4*>(&tile[tk][c * 8]) = val;
    }
    __syncthreads();
    const int s0 = slots[0];
    bool run = s0 >= 0 && (s0 & 7) == 0 && (s0 % page_size) + 8 <= page_size;
#pragma unroll
    for (int i = 1; i < 8; ++i) run = run && slots[i] == s0 + i;
    if (run) {
        bf16_t* vt = v_cache + ((size_t)(s0 / page_size) * nkv + head) * d * page_size + (s0 % page_size);
        for (int e = tid; e < d; e += nthr) {
            union { uint4 u; bf16_t h[8]; } pk;
#pragma unroll
            for (int i = 0; i < 8; ++i) pk.h[i] = tile[i][e];
            *reinterpret_cast<uint4*>(vt + (size_t)e * page_size) = pk.u;
        }
    } else {
        for (int i = 0; i < 8; ++i) {
            const int slot = slots[i];
            if (slot < 0) continue;
            bf16_t* vt = v_cache + ((size_t)(slot / page_size) * nkv + head) * d * page_size + (slot % page_size);
            for (int e = tid; e < d; e += nthr) vt[(size_t)e * page_size] = tile[i][e];
        }
    }
}

// bfloat16, head sizes 16 .. 256 that are powers of two, the whole head rotated (or none of it):
// a lane has 8 consecutive elements of a head (one 16-byte access), LPH = d / 8 lanes a head,
// 64 / LPH heads a wave.  The sum of squares goes over the head's lanes by shuffles; with pairs
// (i, i + d/2) a lane's partner is LPH / 2 lanes away, with pairs (2i, 2i+1) it is the lane itself.
template <int LPH>
__global__ __launch_bounds__(256) void qk_norm_rope_vec_kernel(
    bf16_t* __restrict__ qkv, int nq, int nkv, const float* __restrict__ qw,
    const float* __restrict__ kw, float eps, const float* __restrict__ cos_sin, int pairing,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slot_mapping,
    bf16_t* __restrict__ k_cache, int page_size, int qk_rows, int T, bf16_t* __restrict__ v_cache) {
    constexpr int D = LPH * 8, HPW = 64 / LPH;
    // The grid's rows beyond the q and k heads' are the values' way to their pages, 8 tokens and one kv
    // head a block: one launch for both, and they run side by side.
    if ((int)blockIdx.y >= qk_rows) {
        const long item = (long)((int)blockIdx.y - qk_rows) * T + blockIdx.x;     // (8 tokens, kv head), heads fastest
        if (item < (long)((T + 7) / 8) * nkv)
            v_page_write_block(qkv, T, nq, nkv, D, slot_mapping, v_cache, page_size, (int)(item / nkv) * 8, (int)(item % nkv));
        return;
    }
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l = lane % LPH;
    const int hh = (blockIdx.y * 4 + wave) * HPW + lane / LPH;
    const bool valid = hh < nq + nkv;
    const int h = valid ? hh : 0;
    const bool is_k = h >= nq;
    bf16_t* x = qkv + (size_t)t * (nq + 2 * nkv) * D + (size_t)h * D + l * 8;
    // everything that does not depend on something loaded is asked for at once, the position
    // (which the angles' address waits for) first
    const int pos = cos_sin ? positions[t] : 0;
    const int slot = is_k ? slot_mapping[t] : 0;
    const float* w = is_k ? kw : qw;
    float4 w0 = make_float4(1.f, 1.f, 1.f, 1.f), w1 = w0;
    if (w) {
        w0 = *reinterpret_cast<const float4*>(w + l * 8);
        w1 = *reinterpret_cast<const float4*>(w + l * 8 + 4);
    }
    union { uint4 u; bf16_t e[8]; } in, outv;
    in.u = *reinterpret_cast<const uint4*>(x);
    float4 q0 = make_float4(0.f, 0.f, 0.f, 0.f), q1 = q0, q2 = q0, q3 = q0;
    if (cos_sin) {
        const float* cs = cos_sin + (size_t)pos * D;   // [pos][pair][cos, sin]
        if (pairing == 0) {
            const float4* c4 = reinterpret_cast<const float4*>(cs + (l % (LPH / 2)) * 16);
            q0 = c4[0]; q1 = c4[1]; q2 = c4[2]; q3 = c4[3];
        } else {
            const float4* c4 = reinterpret_cast<const float4*>(cs + l * 8);
            q0 = c4[0]; q1 = c4[1];
        }
    }
    float v[8];
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        v[e] = (float)in.e[e];
        ss = fmaf(v[e], v[e], ss);
    }
#pragma unroll
    for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    if (w) {
        const float rr = rsqrtf(ss / (float)D + eps);
        v[0] = v[0] * rr * w0.x; v[1] = v[1] * rr * w0.y; v[2] = v[2] * rr * w0.z; v[3] = v[3] * rr * w0.w;
        v[4] = v[4] * rr * w1.x; v[5] = v[5] * rr * w1.y; v[6] = v[6] * rr * w1.z; v[7] = v[7] * rr * w1.w;
    }
    if (cos_sin) {
        if (pairing == 0) {
            constexpr int HL = LPH / 2;
            const float c[8] = {q0.x, q0.z, q1.x, q1.z, q2.x, q2.z, q3.x, q3.z};
            const float sn[8] = {q0.y, q0.w, q1.y, q1.w, q2.y, q2.w, q3.y, q3.w};
            const bool first = l < HL;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float pv = __shfl_xor(v[e], HL, 64);
                // first half: a = v, b = pv -> a c - b s;  second half: a = pv, b = v -> a s + b c
                v[e] = first ? v[e] * c[e] - pv * sn[e] : pv * sn[e] + v[e] * c[e];
            }
        } else {
            const float c[4] = {q0.x, q0.z, q1.x, q1.z};
            const float sn[4] = {q0.y, q0.w, q1.y, q1.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float a = v[2 * i], b = v[2 * i + 1];
                v[2 * i] = a * c[i] - b * sn[i];
                v[2 * i + 1] = a * sn[i] + b * c[i];
            }
        }
    }
    if (!valid) return;
#pragma unroll
    for (int e = 0; e < 8; ++e) outv.e[e] = (bf16_t)v[e];
    if (!is_k) {
        *reinterpret_cast<uint4*>(x) = outv.u;
    } else {
        if (slot < 0) return;
        const int page = slot / page_size, off = slot % page_size;
        bf16_t* kdst = k_cache + (((size_t)page * nkv + (h - nq)) * page_size + off) * D + l * 8;
        *reinterpret_cast<uint4*>(kdst) = outv.u;
    }
}

template <int LPH>
static void launch_qk_vec(bf16_t* qkv, int T, int nq, int nkv, const float* qw, const float* kw, float eps,
                          const float* cos_sin, int pairing, const int32_t* positions,
                          const int32_t* slot_mapping, bf16_t* k_cache, bf16_t* v_cache, int page_size, hipStream_t s) {
    constexpr int HPB = 4 * (64 / LPH);
    const int qk_rows = (nq + nkv + HPB - 1) / HPB;
    const int v_rows = (int)(((long)((T + 7) / 8) * nkv + T - 1) / T);   // the values' blocks fill whole rows of the grid
    qk_norm_rope_vec_kernel<LPH><<<dim3(T, qk_rows + v_rows), 256, 0, s>>>(
        qkv, nq, nkv, qw, kw, eps, cos_sin, pairing, positions, slot_mapping, k_cache, page_size, qk_rows, T, v_cache);
}

TFF_API int tff_qk_norm_rope_kv(void* qkv, int T, int nq, int nkv, int d, const float* q_weight,
                                const float* k_weight, float eps, const float* cos_sin,
                                int rot_dim, int pairing, int max_pos, const int32_t* positions,
                                const int32_t* slot_mapping, void* k_cache, void* v_cache,
                                int page_size, int num_pages, int dtype, int cache_dtype,
                                tff_stream_t stream) {
    TFF_REQUIRE(qkv && positions && slot_mapping && k_cache && v_cache,
                "qk_norm_rope_kv: null pointer");
    TFF_REQUIRE(T >= 0 && nq > 0 && nkv > 0 && page_size > 0 && num_pages > 0,
                "qk_norm_rope_kv: bad sizes T=%d nq=%d nkv=%d page_size=%d pages=%d", T, nq, nkv,
                page_size, num_pages);
    TFF_REQUIRE(d > 0 && d <= QK_MAX_D && d % 2 == 0,
                "qk_norm_rope_kv: head size %d not supported (even, at most %d)", d, QK_MAX_D);
    TFF_REQUIRE((q_weight == nullptr) == (k_weight == nullptr),
                "qk_norm_rope_kv: q and k norm weights must both be given or both be absent");
    if (cos_sin) {
        TFF_REQUIRE(rot_dim > 0 && rot_dim <= d && rot_dim % 2 == 0,
                    "qk_norm_rope_kv: rotary size %d must be even and at most the head size %d",
                    rot_dim, d);
        TFF_REQUIRE(pairing == 0 || pairing == 1, "qk_norm_rope_kv: unknown pairing %d", pairing);
        TFF_REQUIRE(max_pos > 0, "qk_norm_rope_kv: empty rotation table");
    }
    TFF_REQUIRE(dtype == cache_dtype, "qk_norm_rope_kv: cache type %d differs from activation type %d",
                cache_dtype, dtype);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    TFF_REQUIRE(dtype == TFF_F32 || dtype == TFF_BF16, "qk_norm_rope_kv: unknown dtype %d", dtype);
    const bool pow2 = d >= 16 && d <= 256 && (d & (d - 1)) == 0;
    // for prompt portions: 16-byte accesses, the q and k heads and the values in blocks of their own of one launch
    if (T >= 128 && dtype == TFF_BF16 && pow2 && (!cos_sin || rot_dim == d) && ((uintptr_t)qkv % 16) == 0 &&
        ((uintptr_t)k_cache % 16) == 0 && ((uintptr_t)v_cache % 16) == 0 &&
        (!q_weight || (((uintptr_t)q_weight % 16) == 0 && ((uintptr_t)k_weight % 16) == 0)) &&
        (!cos_sin || ((uintptr_t)cos_sin % 16) == 0)) {
#define TFF_QK_VEC(L)                                                                               \
    launch_qk_vec<L>((bf16_t*)qkv, T, nq, nkv, q_weight, k_weight, eps, cos_sin, pairing, positions, \
                     slot_mapping, (bf16_t*)k_cache, (bf16_t*)v_cache, page_size, s)
        switch (d) {
            case 16: TFF_QK_VEC(2); break;
            case 32: TFF_QK_VEC(4); break;
            case 64: TFF_QK_VEC(8); break;
            case 128: TFF_QK_VEC(16); break;
            default: TFF_QK_VEC(32); break;
        }
#undef TFF_QK_VEC
        return tff_check_launch("qk_norm_rope");
    }
    if (!cos_sin || rot_dim == d) {
        dim3 grid4(T, (nq + 2 * nkv + 3) / 4);
        if (dtype == TFF_F32)
            qk_norm_rope_kv_reg_kernel<float, float><<<grid4, 256, 0, s>>>(
                (float*)qkv, nq, nkv, d, q_weight, k_weight, eps, cos_sin, pairing, positions, slot_mapping,
                (float*)k_cache, (float*)v_cache, page_size);
        else
            qk_norm_rope_kv_reg_kernel<bf16_t, bf16_t><<<grid4, 256, 0, s>>>(
                (bf16_t*)qkv, nq, nkv, d, q_weight, k_weight, eps, cos_sin, pairing, positions, slot_mapping,
                (bf16_t*)k_cache, (bf16_t*)v_cache, page_size);
        return tff_check_launch("qk_norm_rope_kv");
    }
    dim3 grid(T, nq + 2 * nkv);
    if (dtype == TFF_F32)
        qk_norm_rope_kv_kernel<float, float><<<grid, 64, 0, s>>>(
            (float*)qkv, nq, nkv, d, q_weight, k_weight, eps, cos_sin, rot_dim, pairing, positions,
            slot_mapping, (float*)k_cache, (float*)v_cache, page_size);
    else if (dtype == TFF_BF16)
        qk_norm_rope_kv_kernel<bf16_t, bf16_t><<<grid, 64, 0, s>>>(
            (bf16_t*)qkv, nq, nkv, d, q_weight, k_weight, eps, cos_sin, rot_dim, pairing, positions,
            slot_mapping, (bf16_t*)k_cache, (bf16_t*)v_cache, page_size);
    else
        return tff_fail("qk_norm_rope_kv: unknown dtype %d", dtype);
    return tff_check_launch("qk_norm_rope_kv");
}

// ---------------------------------------------------------------- swiglu ---
// m = silu(g) * u, silu(x) = x / (1 + exp(-x))  (reference:
// src/kernel/cuda/unary.cu:10-27, x1 = gate, x2 = up).
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int64_t total, int I) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int64_t t = idx / I;
    const int i = (int)(idx - t * I);
    const float g = to_f32(gu[t * 2 * I + i]);
    const float u = to_f32(gu[t * 2 * I + I + i]);
    out[idx] = from_f32<T>(g / (1.0f + expf(-g)) * u);
}

TFF_API int tff_swiglu(const void* gu, void* out, int T, int I, int dtype, tff_stream_t stream) {
    TFF_REQUIRE(gu && out, "swiglu: null pointer");
    TFF_REQUIRE(T >= 0 && I > 0, "swiglu: bad sizes T=%d I=%d", T, I);
    if (T == 0) return 0;
    const int64_t total = (int64_t)T * I;
    const int64_t blocks = (total + 255) / 256;
    TFF_REQUIRE(blocks < 2147483647LL, "swiglu: too many elements");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TFF_F32)
        swiglu_kernel<float><<<(unsigned)blocks, 256, 0, s>>>((const float*)gu, (float*)out, total, I);
    else if (dtype == TFF_BF16)
        swiglu_kernel<bf16_t><<<(unsigned)blocks, 256, 0, s>>>((const bf16_t*)gu, (bf16_t*)out, total, I);
    else
        return tff_fail("swiglu: unknown dtype %d", dtype);
    return tff_check_launch("swiglu");
}

// ------------------------------------------------------------------ cast ---
template <typename TS, typename TD>
__global__ void cast_kernel(const TS* __restrict__ src, TD* __restrict__ dst, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        dst[i] = from_f32<TD>(to_f32(src[i]));
}

TFF_API int tff_cast(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t n,
                     tff_stream_t stream) {
    TFF_REQUIRE(src && dst, "cast: null pointer");
    TFF_REQUIRE(n >= 0, "cast: negative count");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    int64_t blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (src_dtype == TFF_F32 && dst_dtype == TFF_BF16)
        cast_kernel<float, bf16_t><<<(unsigned)blocks, 256, 0, s>>>((const float*)src, (bf16_t*)dst, n);
    else if (src_dtype == TFF_BF16 && dst_dtype == TFF_F32)
        cast_kernel<bf16_t, float><<<(unsigned)blocks, 256, 0, s>>>((const bf16_t*)src, (float*)dst, n);
    else if (src_dtype == TFF_F32 && dst_dtype == TFF_F32)
        cast_kernel<float, float><<<(unsigned)blocks, 256, 0, s>>>((const float*)src, (float*)dst, n);
    else if (src_dtype == TFF_BF16 && dst_dtype == TFF_BF16)
        cast_kernel<bf16_t, bf16_t><<<(unsigned)blocks, 256, 0, s>>>((const bf16_t*)src, (bf16_t*)dst, n);
    else
        return tff_fail("cast: unknown dtypes %d -> %d", src_dtype, dst_dtype);
    return tff_check_launch("cast");
}
