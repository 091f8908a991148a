// bfloat16 attention over the paged cache on the gfx950 matrix cores, for
// prompt portions and for decoding (with the keys split over several waves and
// merged by a second kernel).  It replaces the reference's fused kernel
// (src/kernel/cuda/paged_flash_attention.cu:855-1055: 8 queries x 32 keys per
// block on SIMT FMA, one shape only) and computes the same thing:
//   s = (q . k) * scale after the product (:723), causal (mask_op.cu:37-43),
//   running max / sum over key tiles (:746-790), o = softmax(s) . v,
//   q head h reads kv head h / G (:891-892).
//
// One wave works on up to NQT*16 *columns* of one request and one kv head; a
// column is a (token, q head of the group) pair, columns are numbered
// token * G + head, so neighbouring columns share their keys.  Per 32 keys:
//
//   S^T[key][col] = K[key][:] . Q[col][:]      MFMA 16x16x32, first operand K:
//       lane (row = key, g) reads 8 consecutive elements of its key's row, which
//       is how keys lie in a page ([slot][element]);
//   the result leaves lane (col, g) with keys g*4..g*4+3 of each 16-key tile:
//       8 scores of its own column, so max, exp and sum need two shuffles only;
//   O^T[elem][col] += V^T[elem][key] . P^T[key][col]   MFMA 16x16x32 whose 8
//       contraction slots per lane group g are defined as keys {g*4..g*4+3} of
//       the first and of the second tile: exactly what the lane already holds
//       of P, and two 8-byte runs of a value page, which is kept transposed
//       ([element][slot]) for this purpose.  No operand goes through LDS.
#include <mutex>

#include "common.h"
#include "tffinfer_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* glb_ptr_t;
// s_waitcnt immediate: vmcnt = 0, the other counters untouched
constexpr int vmcnt_imm0() { return (7 << 4) | (15 << 8); }

// Page and slot of a key: a shift and a mask.  These kernels take pages of a power of two of
// tokens only (the GPU has no integer divider); other page sizes run on the general kernel.
__device__ __forceinline__ int page_index(int j, int page_size, int page_shift) {
    (void)page_size;
    return j >> page_shift;
}
__device__ __forceinline__ int page_slot(int j, int page_size, int page_shift) {
    (void)page_shift;
    return j & (page_size - 1);
}

// ------------------------------------------------ one column tile per wave ---
// Decoding (and portions of a few tokens): one wave, 16 columns.  What counts
// here is bytes in flight.  The wave's part of the block table goes to LDS
// first, so that no page number is waited for among the loads of keys and
// values (loads come back in order: a wait for a page number would be a wait
// for every load issued before it).  Keys and values of RING steps of 32 keys
// are in flight at any time: a step's registers are loaded again as soon as
// its arithmetic is done.  Within a step the 16 rows of key tile t are the keys
// (r / 4) * 8 + t * 4 + r % 4, so lane (col, g) holds the scores of the eight
// consecutive keys g*8 .. g*8+7 and reads its values as one 16-byte run.
#define ATTN_WAVE_BT 1024

// What the decoding kernel needs to take q, k and v as the fused projection left them (one row
// of (nq + 2 nkv) d elements per token) instead of a finished q and a cache that already holds
// the token: the weights of the per-head RMS norms of q and k (null: no norm), the table of
// rotation angles [position][pair][cos, sin] (null: no rotation; else the whole head is
// rotated), the pairing (0: (i, i + d/2), 1: (2i, 2i+1)) and the caches to write the token's
// key and value into (null: the cache holds them already and is only read; so it is for a
// token whose slot_mapping entry is negative: a padding row of a captured step, say).
struct AttnFuse {
    const float* q_weight;
    const float* k_weight;
    const float* cos_sin;
    bf16_t* k_write;
    bf16_t* v_write;
    const int32_t* slot_mapping;   // per token; a negative entry: this token's key and value are not written
    float eps;
    int pairing;
    // Runs of keys dealt by the host (null: the launch splits every entry's keys alike): run i is
    // (entry, first key, end of keys, the entry's position), 16 bytes, and gets a wave per kv head.
    // An entry of negative number: the run is not in use.
    const int32_t* key_runs;
};

// RMS norm over the head and rotation of one head held as MFMA operand fragments: lane group kg
// has the elements ks * 32 + kg * 8 .. + 7 of every 32-element step ks, so with pairs (i, i + d/2)
// (d a multiple of 64) both elements of a pair are in the same lane, KS / 2 steps apart, and with
// pairs (2i, 2i+1) they are neighbours.  The four lane groups of a column add up the squares.
// w and cs point into LDS (the kernel put the weights and the position's angles there).
template <int DT>
__device__ __forceinline__ void norm_rope_fragments(bf16x8 (&f)[(DT * 16 + 31) / 32], bool has_norm,
                                                    const float* w, float eps, bool has_rope,
                                                    const float* cs, int pairing, int kg) {
    constexpr int D = DT * 16;
    constexpr int KS = (D + 31) / 32;
    float x[KS][8];
    float ss = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            x[ks][j] = (float)f[ks][j];
            ss = fmaf(x[ks][j], x[ks][j], ss);
        }
    ss = rows_sum(ss);
    if (has_norm) {
        const float rr = rsqrtf(ss / (float)D + eps);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int e = ks * 32 + kg * 8;
            if (e < D) {
#pragma unroll
                for (int j = 0; j < 8; ++j) x[ks][j] = x[ks][j] * rr * w[e + j];
            }
        }
    }
    if (has_rope) {
        if (pairing == 0) {
            if constexpr (KS % 2 == 0) {
#pragma unroll
                for (int ks = 0; ks < KS / 2; ++ks)
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int p = ks * 32 + kg * 8 + j;
                        const float c = cs[2 * p], sn = cs[2 * p + 1];
                        const float a = x[ks][j], b = x[ks + KS / 2][j];
                        x[ks][j] = a * c - b * sn;
                        x[ks + KS / 2][j] = a * sn + b * c;
                    }
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int e = ks * 32 + kg * 8;
                if (e < D) {
#pragma unroll
                    for (int j = 0; j < 8; j += 2) {
                        const int p = (e + j) >> 1;
                        const float c = cs[2 * p], sn = cs[2 * p + 1];
                        const float a = x[ks][j], b = x[ks][j + 1];
                        x[ks][j] = a * c - b * sn;
                        x[ks][j + 1] = a * sn + b * c;
                    }
                }
            }
        }
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int j = 0; j < 8; ++j) f[ks][j] = (bf16_t)x[ks][j];
}
// BW > 1 (entries of one token, FUSED): a block of BW waves per entry and kv head.  The waves
// split the entry's keys among them (what blockIdx.z does for SPLIT), and their partial results
// meet in LDS instead of global memory: no second kernel, no partial results written and read.
// A wave alone streams some 16 GB/s, eight of them on a CU together as much as the CU takes
// (≈ 100 GB/s), so this pays once there are entries x kv heads enough for the blocks to saturate
// HBM between them (64 and more); with fewer, the keys are split over blocks as before.
template <int DT, bool SPLIT, int RING, bool FUSED = false, int BW = 1>
__global__ __launch_bounds__(64 * BW, 1) void attn_wave_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int bt_stride,
    const int32_t* __restrict__ cu_tokens, const int32_t* __restrict__ start_pos,
    const int32_t* __restrict__ work, int tiles_per_entry, int nq, int nkv, int page_size,
    int page_shift, int window, float scale, int T_total, AttnFuse fz) {
    constexpr int D = DT * 16;
    constexpr int KS = (D + 31) / 32;
    static_assert(BW == 1 || (FUSED && !SPLIT), "blocks of several waves are for fused decode steps, and merge in LDS");
    constexpr int BT_LEN = BW == 1 ? ATTN_WAVE_BT : ATTN_WAVE_BT / 4;     // page numbers a wave keeps at a time
    __shared__ int32_t bt_all[BW * BT_LEN];
    __shared__ __attribute__((aligned(16))) float fz_all[BW * (FUSED ? 3 * D : 4)];   // q weight, k weight, (cos, sin) pairs
    const int lane = threadIdx.x & 63, qc = lane & 15, kg = lane >> 4;
    const int wv = BW == 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int32_t* bt_lds = bt_all + wv * BT_LEN;
    float* fz_lds = fz_all + wv * (FUSED ? 3 * D : 4);
    // what a wave writes to its part of LDS only itself reads: with one wave a block the barrier is the
    // fence; with several, a fence of the wave's own (LDS works through a wave's accesses in order)
    auto wave_sync = [&]() {
        if constexpr (BW == 1) {
            __syncthreads();
        } else {
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
            __builtin_amdgcn_wave_barrier();
        }
    };
    // Runs dealt by the host: a grid of one dimension over (run, kv head), a multiple of eight
    // runs, in this order: eight runs by eight, within them the kv heads, within a kv head the
    // eight runs.  Blocks go to the XCDs in turn by their number, so run i is on XCD i % 8 with
    // all its kv heads: the runs of a long entry, which follow each other, land on all XCDs
    // (splitting every entry alike puts all waves of an entry on the one XCD that the entry's
    // number selects), and a page of keys is read through one XCD's L2 and address translation,
    // not through all eight.  The runs that are not in use come last, after every wave with work
    // has its place: strewn among the others they took places on half of the CUs and left the
    // waves with work crowded on the other half (a fifth slower at 64 entries of one run each).
    bool by_runs = false;
    if constexpr (SPLIT || (FUSED && BW > 1)) by_runs = fz.key_runs != nullptr;
    int r, col0, g = blockIdx.y, run_index = 0;
    int4 run = make_int4(0, 0, 0, 0);
    if (by_runs) {
        const int eight = blockIdx.x / (8 * nkv), within = blockIdx.x - eight * (8 * nkv);
        run_index = eight * 8 + (within & 7);
        g = within >> 3;
        run = reinterpret_cast<const int4*>(fz.key_runs)[run_index];
        r = run.x;
        if (r < 0) return;
        col0 = blockIdx.z * 16;
    } else if (work) {
        r = work[2 * blockIdx.x];
        col0 = work[2 * blockIdx.x + 1];
    } else {
        r = blockIdx.x / tiles_per_entry;
        col0 = (blockIdx.x % tiles_per_entry) * 16;
    }
    const int G = nq / nkv;
    // (a run brings its entry's position with it, and its entry has one token, which in a step of
    // one token per entry, as the fused form takes it, is the entry's number: nothing to wait for
    // between the run and the page numbers)
    const int tok0 = (FUSED && by_runs) ? r : cu_tokens[r];
    const int n = by_runs ? 1 : cu_tokens[r + 1] - tok0;
    const int P = by_runs ? run.w : start_pos[r];
    const int ncols = n * G;
    const int32_t* bt = block_tables + (size_t)r * bt_stride;

    const int c = col0 + qc;
    const bool c_ok = c < ncols;
    const int cc = c_ok ? c : ncols - 1;
    const int tl = cc / G;
    const int c_tok = tok0 + tl;
    const int c_head = g * G + (cc - tl * G);
    const int c_pos = c_ok ? P + tl : -1;   // a missing column sees no key
    const int c_lo = window > 0 ? max(0, P + tl - window + 1) : 0;
    // keys any column of this wave can see
    const int tl_first = col0 / G;
    const int tl_last = (min(col0 + 16, ncols) - 1) / G;
    const int kmin = window > 0 ? max(0, P + tl_first - window + 1) : 0;
    const int kmax = P + tl_last;
    const int kb0 = (kmin / 32) * 32;
    const int nsteps = (kmax - kb0) / 32 + 1;
    int s_begin = 0, s_end = nsteps;
    if (by_runs) {
        s_begin = min(nsteps, max(0, (run.y - kb0) >> 5));
        s_end = min(nsteps, max(s_begin, (run.z - kb0 + 31) >> 5));
    }
    // (an entry whose keys are one run has its result from that run's wave or block, no partial one;
    // runs neither overlap nor leave a gap)
    const bool run_is_partial = by_runs && (s_begin > 0 || s_end < nsteps);
    if constexpr (BW > 1) {
        // the block's keys (all of the entry's, or its run) among its waves, never under 96 keys a
        // wave, as below
        const int lo = s_begin, hi = s_end;
        const int per = max((hi - lo + BW - 1) / BW, min(3, hi - lo));
        s_begin = min(hi, lo + wv * per);
        s_end = min(hi, s_begin + per);
    }
    if (SPLIT && !by_runs) {
        // The launch is sized for the longest context the engine allows; with shorter ones a run
        // of keys is not made shorter than 256 keys as long as some 256 waves are left with
        // work (the other waves of the launch end at once; their partial results are empty), and
        // never shorter than 128: runs of 128 keys were 7 % slower at 8 requests of 2,048 tokens
        // and 2 % at 4, and one request's 22 runs of 96 keys 2 % of the step slower than 16 of 128
        // (up to 16 partial results the merge fetches in one go).
        const int busy = (256 + (int)(gridDim.x * gridDim.y) - 1) / (int)(gridDim.x * gridDim.y);
        const int per = max(max((nsteps + (int)gridDim.z - 1) / (int)gridDim.z, min(8, (nsteps + busy - 1) / busy)),
                            min(4, nsteps));
        s_begin = min(nsteps, (int)blockIdx.z * per);
        s_end = min(nsteps, s_begin + per);
    }

    // FUSED (entries of one token): q comes as the projection left it and is normalised and
    // rotated here; the wave whose keys end with the token's own position does the same for
    // the token's key, puts key and value into their page and works on them from registers.
    // The norm weights and the position's angles go to LDS beside the page numbers; the raw q, k
    // and v are loaded after the barrier and worked on once the first keys and values are on
    // their way, so that they delay nothing.
    const bool owns_new = FUSED && fz.k_write != nullptr && s_begin < s_end && s_end == nsteps && fz.slot_mapping[tok0] >= 0;
    const bool has_norm = FUSED && fz.q_weight != nullptr, has_rope = FUSED && fz.cos_sin != nullptr;

    // The page numbers of this wave's keys come from LDS, always: a lookup in the table itself
    // is a memory load, and to wait for it is to wait for every key and value load issued
    // before it, one round trip to HBM after the other.  Keys beyond what ATTN_WAVE_BT pages
    // hold are worked through in segments, each with its own page numbers in LDS.
    const int seg_steps = max(1, ((BT_LEN - 1) * page_size) >> 5);
    int pi0 = 0;
    auto fill_pages = [&](int seg0, int seg1, int from) {
        pi0 = page_index(kb0 + seg0 * 32, page_size, page_shift);
        const int pi1 = page_index(min(kmax, kb0 + seg1 * 32 - 1), page_size, page_shift);
        for (int i = from + lane; i <= pi1 - pi0; i += 64) bt_lds[i] = bt[pi0 + i];
    };
    // Everything the wave needs before its first keys is asked for at once, the page numbers
    // first (loads come back in the order they were issued, so the wait for the page numbers
    // is a wait for nothing else): one round trip instead of one per table.  What is not needed
    // for the addresses of the keys (norm weights, angles, the raw q, k and v) is put to use
    // after the first keys and values are on their way.
    int new_page = 0, first_page = 0, first_count = 0;
    if (s_begin < s_end) {
        pi0 = page_index(kb0 + s_begin * 32, page_size, page_shift);
        first_count = page_index(min(kmax, kb0 + min(s_end, s_begin + seg_steps) * 32 - 1), page_size, page_shift) - pi0 + 1;
        if (lane < first_count) first_page = bt[pi0 + lane];
    }
    if constexpr (FUSED) {
        if (owns_new) new_page = bt[page_index(P, page_size, page_shift)];
    }
    constexpr int FZN = FUSED ? (D + 63) / 64 : 1;
    float fz_q[FZN], fz_k[FZN], fz_cs[FZN];
    if constexpr (FUSED) {
#pragma unroll
        for (int u = 0; u < FZN; ++u) {
            const int i = lane + 64 * u;
            fz_q[u] = fz_k[u] = fz_cs[u] = 0.f;
            if (i < D) {
                if (has_norm) {
                    fz_q[u] = fz.q_weight[i];
                    fz_k[u] = fz.k_weight[i];
                }
                if (has_rope) fz_cs[u] = fz.cos_sin[(size_t)P * D + i];
            }
        }
    }

    bf16x8 qf[KS];
    {
        const bf16_t* qp = q + (size_t)c_tok * q_stride + (size_t)c_head * D;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int e = ks * 32 + kg * 8;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (c_ok && e < D) v = *reinterpret_cast<const uint4*>(qp + e);
            qf[ks] = *reinterpret_cast<bf16x8*>(&v);
        }
    }
    bf16x8 knew[KS];
    bf16_t vnew[DT];
    if constexpr (FUSED) {
        if (owns_new) {
            const bf16_t* kraw = q + (size_t)tok0 * q_stride + (size_t)(nq + g) * D;
            const bf16_t* vraw = kraw + (size_t)nkv * D;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int e = ks * 32 + kg * 8;
                uint4 v = make_uint4(0, 0, 0, 0);
                if (e < D) v = *reinterpret_cast<const uint4*>(kraw + e);
                knew[ks] = *reinterpret_cast<bf16x8*>(&v);
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) vnew[dt] = vraw[dt * 16 + qc];
        }
    }

    // the page numbers of the first segment: the first 64 came with the loads above
    if (lane < first_count) bt_lds[lane] = first_page;
    if (first_count > 64) fill_pages(s_begin, min(s_end, s_begin + seg_steps), 64);
    wave_sync();

    floatx4 oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    bf16x8 kf[RING][2][KS];   // [ring slot][key tile][k-step]
    bf16x8 vf[RING][DT];

#define TFF_WAVE_PAGE(j) bt_lds[page_index((j), page_size, page_shift) - pi0]
#define TFF_WAVE_LOAD(buf, step)                                                                    \
    {                                                                                               \
        const int kb_ = kb0 + (step) * 32;                                                          \
        _Pragma("unroll") for (int kt = 0; kt < 2; ++kt) {                                          \
            /* rows past the last key repeat it; they are masked */                                 \
            const int j_ = min(kb_ + (qc >> 2) * 8 + kt * 4 + (qc & 3), kmax);                      \
            const int page_ = TFF_WAVE_PAGE(j_);                                                    \
            const bf16_t* kp_ = k_cache + (((size_t)page_ * nkv + g) * page_size + page_slot(j_, page_size, page_shift)) * D; \
            _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) {                                     \
                const int e_ = ks * 32 + kg * 8;                                                    \
                uint4 v_ = make_uint4(0, 0, 0, 0);                                                  \
                if (e_ < D) v_ = *reinterpret_cast<const uint4*>(kp_ + e_);                         \
                kf[buf][kt][ks] = *reinterpret_cast<bf16x8*>(&v_);                                  \
            }                                                                                       \
        }                                                                                           \
        /* the values of keys kb + g*8 .. +7: a run of 16 bytes in a page (pages hold a multiple */ \
        /* of 8 keys); a run past the last key is read from the last key's run and masked */       \
        const int j0_ = min(kb_ + kg * 8, (kmax >> 3) << 3);                                        \
        const int vpage_ = TFF_WAVE_PAGE(j0_);                                                      \
        const bf16_t* vrun_ = v_cache + ((size_t)vpage_ * nkv + g) * D * page_size + page_slot(j0_, page_size, page_shift); \
        _Pragma("unroll") for (int dt = 0; dt < DT; ++dt) {                                         \
            const uint4 v_ = *reinterpret_cast<const uint4*>(vrun_ + (size_t)(dt * 16 + qc) * page_size); \
            vf[buf][dt] = *reinterpret_cast<const bf16x8*>(&v_);                                    \
        }                                                                                           \
    }
    /* the token's own key and value (the last key of the last step): from registers, not from */
    /* the page */
#define TFF_WAVE_PATCH(buf, step)                                                                   \
    {                                                                                               \
        const int kb_ = kb0 + (step) * 32;                                                          \
        _Pragma("unroll") for (int kt = 0; kt < 2; ++kt)                                            \
            if (kb_ + (qc >> 2) * 8 + kt * 4 + (qc & 3) >= kmax) {                                  \
                _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) kf[buf][kt][ks] = knew[ks];       \
            }                                                                                       \
        const int at_ = kmax - min(kb_ + kg * 8, (kmax >> 3) << 3);                                 \
        _Pragma("unroll") for (int dt = 0; dt < DT; ++dt)                                           \
            _Pragma("unroll") for (int e = 0; e < 8; ++e)                                           \
                if (e == at_) vf[buf][dt][e] = vnew[dt];                                            \
    }
    // The softmax works on raw scores with the scale folded into the exponent,
    //   p = 2^((s - m) * scale * log2 e),
    // masks only the steps that touch a column's causal or window edge, and moves the reference m
    // (and rescales the accumulators) only when some score exceeds it by more than 8 in the
    // exponent's units: until then p stays below 2^8 and the quotient o / l does not depend on the
    // reference.  A wave alone on its SIMD is bound by the instructions of a step, not by memory;
    // rescaling 4 DT accumulator registers in every step was a quarter of them.
    const float sl2 = scale * 1.44269504088896f;
    const float slack = 8.0f / sl2;
    int w_min_pos = c_ok ? c_pos : 0x7fffffff, w_max_lo = c_ok ? c_lo : 0;   // over the wave's columns
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        w_min_pos = min(w_min_pos, __shfl_xor(w_min_pos, o, 64));
        w_max_lo = max(w_max_lo, __shfl_xor(w_max_lo, o, 64));
    }
#define TFF_WAVE_COMPUTE(buf, step)                                                                 \
    {                                                                                               \
        const int kb_ = kb0 + (step) * 32;                                                          \
        floatx4 sacc_[2];                                                                           \
        sacc_[0] = sacc_[1] = floatx4{0.f, 0.f, 0.f, 0.f};                                          \
        _Pragma("unroll") for (int kt = 0; kt < 2; ++kt)                                            \
            _Pragma("unroll") for (int ks = 0; ks < KS; ++ks)                                       \
                sacc_[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[buf][kt][ks], qf[ks], sacc_[kt], 0, 0, 0); \
        float sv_[8];                                                                               \
        _Pragma("unroll") for (int e = 0; e < 8; ++e) sv_[e] = sacc_[e >> 2][e & 3];                \
        if (kb_ + 31 > w_min_pos || kb_ < w_max_lo) {   /* the step touches an edge of some column (a column */ \
            /* that does not exist has a query of zeros and is masked with the others) */          \
            _Pragma("unroll") for (int e = 0; e < 8; ++e) {                                         \
                const int j = kb_ + kg * 8 + e;                                                     \
                if (!(j >= c_lo && j <= c_pos)) sv_[e] = -INFINITY;                                 \
            }                                                                                       \
        }                                                                                           \
        float mt_ = fmaxf(fmaxf(fmaxf(sv_[0], sv_[1]), fmaxf(sv_[2], sv_[3])),                      \
                          fmaxf(fmaxf(sv_[4], sv_[5]), fmaxf(sv_[6], sv_[7])));                     \
        float m_new_ = m_run, alpha_ = 1.f;                                                         \
        if (__any(mt_ > m_run + slack)) {                                                           \
            mt_ = rows_max(mt_);                                                                    \
            m_new_ = fmaxf(m_run, mt_);                                                             \
            alpha_ = m_new_ == -INFINITY ? 1.f : __builtin_amdgcn_exp2f((m_run - m_new_) * sl2);    \
        }                                                                                           \
        const float mb_ = m_new_ == -INFINITY ? 0.f : m_new_ * sl2;                                 \
        float ps_ = 0.f;                                                                            \
        bf16x8 pv_;                                                                                 \
        _Pragma("unroll") for (int e = 0; e < 8; ++e) {                                             \
            const float p = __builtin_amdgcn_exp2f(fmaf(sv_[e], sl2, -mb_));   /* 2^-inf = 0 for masked scores */ \
            ps_ += p;                                                                               \
            pv_[e] = (bf16_t)p;                                                                     \
        }                                                                                           \
        l_run = l_run * alpha_ + ps_;                                                               \
        m_run = m_new_;                                                                             \
        if (__any(alpha_ != 1.f)) {                                                                 \
            _Pragma("unroll") for (int dt = 0; dt < DT; ++dt) {                                     \
                oacc[dt][0] *= alpha_; oacc[dt][1] *= alpha_;                                       \
                oacc[dt][2] *= alpha_; oacc[dt][3] *= alpha_;                                       \
            }                                                                                       \
        }                                                                                           \
        _Pragma("unroll") for (int dt = 0; dt < DT; ++dt)                                           \
            oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[buf][dt], pv_, oacc[dt], 0, 0, 0); \
    }

    for (int seg0 = s_begin; seg0 < s_end; seg0 += seg_steps) {
        const int seg1 = min(s_end, seg0 + seg_steps);
        if (seg0 > s_begin) {
            wave_sync();            // the segment before is read
            fill_pages(seg0, seg1, 0);
            wave_sync();
        }
        // steps past the end load the last step again and are not used
#pragma unroll
        for (int u = 0; u < RING; ++u) TFF_WAVE_LOAD(u, min(seg0 + u, seg1 - 1))
        if constexpr (FUSED) {   // while the first keys and values travel
            if (seg0 == s_begin) {
#pragma unroll
                for (int u = 0; u < FZN; ++u) {
                    const int i = lane + 64 * u;
                    if (i < D) {
                        fz_lds[i] = fz_q[u];
                        fz_lds[D + i] = fz_k[u];
                        fz_lds[2 * D + i] = fz_cs[u];
                    }
                }
                wave_sync();
                if (has_norm || has_rope) norm_rope_fragments<DT>(qf, has_norm, fz_lds, fz.eps, has_rope, fz_lds + 2 * D, fz.pairing, kg);
                if (owns_new) {
                    norm_rope_fragments<DT>(knew, has_norm, fz_lds + D, fz.eps, has_rope, fz_lds + 2 * D, fz.pairing, kg);
                    if (col0 == 0) {
                        const int page = new_page;
                        const int slot = page_slot(P, page_size, page_shift);
                        if (qc == 0) {
                            bf16_t* kd = fz.k_write + (((size_t)page * nkv + g) * page_size + slot) * D;
#pragma unroll
                            for (int ks = 0; ks < KS; ++ks) {
                                const int e = ks * 32 + kg * 8;
                                if (e < D) *reinterpret_cast<uint4*>(kd + e) = *reinterpret_cast<const uint4*>(&knew[ks]);
                            }
                        }
                        if (kg == 0) {
                            bf16_t* vd = fz.v_write + ((size_t)page * nkv + g) * D * page_size + slot;
#pragma unroll
                            for (int dt = 0; dt < DT; ++dt) vd[(size_t)(dt * 16 + qc) * page_size] = vnew[dt];
                        }
                    }
                }
            }
        }
        int s = seg0;
        for (; seg1 - s > RING; s += RING) {
#pragma unroll
            for (int u = 0; u < RING; ++u) {
                TFF_WAVE_COMPUTE(u, s + u)
                TFF_WAVE_LOAD(u, min(s + u + RING, seg1 - 1))
            }
        }
#pragma unroll
        for (int u = 0; u < RING; ++u)
            if (s + u < seg1) {
                if constexpr (FUSED) {
                    if (owns_new && s + u == s_end - 1) TFF_WAVE_PATCH(u, s + u)
                }
                TFF_WAVE_COMPUTE(u, s + u)
            }
    }
#undef TFF_WAVE_PAGE
#undef TFF_WAVE_PATCH
#undef TFF_WAVE_LOAD
#undef TFF_WAVE_COMPUTE

    float l = l_run;
    l = rows_sum(l);
    if constexpr (BW > 1) {
        // The waves' partial results meet in LDS: [wave][value tile][lane] four floats, and a
        // maximum and a sum per wave and column.  Wave w then merges value tiles w, w + BW, ...:
        //   m = max m_s, l = sum l_s e^(m_s - m), o = sum o_s e^(m_s - m) / l
        // in the order of the waves, whatever their number of keys.
        __shared__ __attribute__((aligned(16))) float mo[BW * DT * 256];
        __shared__ float mml[BW * 32];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            *reinterpret_cast<float4*>(mo + ((wv * DT + dt) * 64 + lane) * 4) =
                make_float4(oacc[dt][0], oacc[dt][1], oacc[dt][2], oacc[dt][3]);
        if (kg == 0) {
            mml[wv * 32 + qc * 2] = m_run * scale;   // (in the exponent's natural units)
            mml[wv * 32 + qc * 2 + 1] = l;
        }
        __syncthreads();
        if (!c_ok) return;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < BW; ++w) m = fmaxf(m, mml[w * 32 + qc * 2]);
        float wgt[BW], lsum = 0.f;
#pragma unroll
        for (int w = 0; w < BW; ++w) {
            const float ms = mml[w * 32 + qc * 2];
            wgt[w] = ms == -INFINITY ? 0.f : __expf(ms - m);
            lsum = fmaf(mml[w * 32 + qc * 2 + 1], wgt[w], lsum);
        }
        const float inv = 1.0f / lsum;
        bf16_t* op = out + ((size_t)c_tok * nq + c_head) * D;
        // (a run of an entry that has several: the block's result is a partial one, kept by run)
        const size_t prow = (size_t)run_index * nq + c_head;
        if (run_is_partial && wv == 0 && kg == 0) {
            part_ml[prow * 2] = m;
            part_ml[prow * 2 + 1] = lsum;
        }
        for (int dt = wv; dt < DT; dt += BW) {
            float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int w = 0; w < BW; ++w) {
                const float4 o = *reinterpret_cast<const float4*>(mo + ((w * DT + dt) * 64 + lane) * 4);
                acc.x = fmaf(o.x, wgt[w], acc.x);
                acc.y = fmaf(o.y, wgt[w], acc.y);
                acc.z = fmaf(o.z, wgt[w], acc.z);
                acc.w = fmaf(o.w, wgt[w], acc.w);
            }
            if (run_is_partial) {
                *reinterpret_cast<float4*>(part_o + prow * D + dt * 16 + kg * 4) = acc;
                continue;
            }
            union { bf16_t h[4]; uint2 u; } pk;
            pk.h[0] = (bf16_t)(acc.x * inv);
            pk.h[1] = (bf16_t)(acc.y * inv);
            pk.h[2] = (bf16_t)(acc.z * inv);
            pk.h[3] = (bf16_t)(acc.w * inv);
            *reinterpret_cast<uint2*>(op + dt * 16 + kg * 4) = pk.u;
        }
        return;
    }
    if (!c_ok) return;
    const bool partial = by_runs ? run_is_partial : SPLIT;
    if (partial) {
        // keys are split for entries of one token only: partial results are kept by entry, or by run
        const size_t row = by_runs ? (size_t)run_index * nq + c_head : ((size_t)blockIdx.z * T_total + r) * nq + c_head;
        float* po = part_o + row * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            *reinterpret_cast<float4*>(po + dt * 16 + kg * 4) =
                make_float4(oacc[dt][0], oacc[dt][1], oacc[dt][2], oacc[dt][3]);
        if (kg == 0) {
            part_ml[row * 2] = m_run * scale;   // (the merge works with e^(m_s - m): the reference in the exponent's natural units)
            part_ml[row * 2 + 1] = l;
        }
    } else {
        const float inv = 1.0f / l;
        bf16_t* op = out + ((size_t)c_tok * nq + c_head) * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            union { bf16_t h[4]; uint2 u; } pk;
#pragma unroll
            for (int i = 0; i < 4; ++i) pk.h[i] = (bf16_t)(oacc[dt][i] * inv);
            *reinterpret_cast<uint2*>(op + dt * 16 + kg * 4) = pk.u;
        }
    }
}

// merges the partial results of the key splits:
//   m = max m_s, l = sum l_s e^(m_s - m), o = sum o_s e^(m_s - m) / l
__global__ __launch_bounds__(256) void attn_split_reduce_kernel(const float* __restrict__ part_o,
                                                                 const float* __restrict__ part_ml,
                                                                 bf16_t* __restrict__ out, int splits,
                                                                 int R_total, int nq, int d,
                                                                 const int32_t* __restrict__ rows) {
    __shared__ float w[256];
    __shared__ float red[17];
    // rows: (entry, token) pairs; without them entry i is token i
    const int r = rows ? rows[2 * blockIdx.x] : (int)blockIdx.x;
    const int t = rows ? rows[2 * blockIdx.x + 1] : (int)blockIdx.x;
    const int h = blockIdx.y, tid = threadIdx.x;
    float ms = -INFINITY, ls = 0.f;
    if (tid < splits) {
        const float* ml = part_ml + (((size_t)tid * R_total + r) * nq + h) * 2;
        ms = ml[0];
        ls = ml[1];
    }
    // the first splits' elements are asked for together with the maxima and sums, not after the
    // reductions that need those: one trip to memory instead of two
    constexpr int AHEAD = 16;
    float po[AHEAD];
#pragma unroll
    for (int s = 0; s < AHEAD; ++s)
        po[s] = (tid < d && s < splits) ? part_o[(((size_t)s * R_total + r) * nq + h) * d + tid] : 0.f;
    const float m = block_max(ms, red);
    const float ws = ms == -INFINITY ? 0.f : __expf(ms - m);
    w[tid] = ws;
    // A launch is sized for the longest context; the runs of keys past an entry's own are empty and
    // come last: the splits up to the last one that weighs something are fetched, the rest not.
    __shared__ int used_w[4];
    {
        const unsigned long long nz = __ballot(ws != 0.f);
        if ((tid & 63) == 0) used_w[tid >> 6] = nz ? (tid & ~63) + 64 - __clzll((long long)nz) : 0;
    }
    const float l = block_sum(ls * ws, red);   // its barriers also publish w and used_w
    const int used = max(max(used_w[0], used_w[1]), max(used_w[2], used_w[3]));
    const float inv = 1.0f / l;
    for (int e = tid; e < d; e += blockDim.x) {
        float acc = 0.f;
        int s0 = 0;
        if (e == tid) {   // (the thread's first element) splits in their order, as below
#pragma unroll
            for (int s = 0; s < AHEAD; ++s)
                if (s < splits) acc = fmaf(po[s], w[s], acc);
            s0 = AHEAD;
        }
#pragma unroll 8
        for (int s = s0; s < used; ++s)
            acc = fmaf(part_o[(((size_t)s * R_total + r) * nq + h) * d + e], w[s], acc);
        out[((size_t)t * nq + h) * d + e] = (bf16_t)(acc * inv);
    }
}

// The same for a few splits (many requests): one wave per (row, head), four to a block, and no
// exchange between lanes: every lane goes
// through the splits' maxima and sums itself (the loads are the same for the whole wave) and
// adds up its own elements of the head, in the order of the splits.
__global__ __launch_bounds__(256) void attn_split_reduce_few_kernel(const float* __restrict__ part_o,
                                                                 const float* __restrict__ part_ml,
                                                                 bf16_t* __restrict__ out, int splits,
                                                                 int R_total, int nq, int d,
                                                                 const int32_t* __restrict__ rows, int n) {
    const int lane = threadIdx.x & 63;
    const int pair = blockIdx.x * 4 + (threadIdx.x >> 6);     // (row, head), heads fastest
    if (pair >= n * nq) return;
    const int i = pair / nq, h = pair - i * nq;
    // rows: (entry, token) pairs; without them entry i is token i
    const int r = rows ? rows[2 * i] : i;
    const int t = rows ? rows[2 * i + 1] : i;
    const size_t stride_ml = (size_t)R_total * nq * 2, stride_o = (size_t)R_total * nq * d;
    const float* ml = part_ml + ((size_t)r * nq + h) * 2;
    const float* po = part_o + ((size_t)r * nq + h) * d;
    float m = -INFINITY;
    for (int s = 0; s < splits; ++s) m = fmaxf(m, ml[s * stride_ml]);
    float l = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};              // d <= 256: up to four elements a lane
    for (int s0 = 0; s0 < splits; s0 += 4) {
        float w[4], v[4][4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {                            // four splits' loads in flight
            const int s = min(s0 + u, splits - 1);
            const float ms = ml[s * stride_ml];
            w[u] = (s0 + u < splits && ms != -INFINITY) ? __expf(ms - m) : 0.f;
            l = fmaf(ml[s * stride_ml + 1], w[u], l);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[u][e] = lane + 64 * e < d ? po[s * stride_o + lane + 64 * e] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = fmaf(v[u][e], w[u], acc[e]);
    }
    const float inv = 1.0f / l;
    bf16_t* o = out + ((size_t)t * nq + h) * d;
#pragma unroll
    for (int e = 0; e < 4; ++e)
        if (lane + 64 * e < d) o[lane + 64 * e] = (bf16_t)(acc[e] * inv);
}

// The same for runs of keys dealt by the host: entry r has the runs run_start[r] ..
// run_start[r + 1] - 1, any number of them, their partial results one after the other.  One block
// of four waves per (entry, head); an entry of one run has its result already.  The runs go to the
// waves sixteen at a time, in turn: up to sixteen runs are the first wave's alone (the others end
// at once), a hundred are two rounds a wave instead of seven one after the other, each a round
// trip to memory.  The first wave asks for its first sixteen runs' elements together with the
// maxima and sums (lane s takes those of run s, s + 64, ...), the weights of those runs then come
// from the lanes that hold them; in the other rounds every lane reads the runs' maxima and sums
// itself (one address for the whole wave).  Every lane adds up its own elements of the head in the
// order of its wave's runs, and the first wave adds the other waves' sums to its own in their order.
__global__ __launch_bounds__(256) void attn_run_merge_kernel(const float* __restrict__ part_o,
                                                              const float* __restrict__ part_ml,
                                                              bf16_t* __restrict__ out,
                                                              const int32_t* __restrict__ run_start,
                                                              const int32_t* __restrict__ tokens,
                                                              int R, int nq, int d) {
    constexpr int AHEAD = 16;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int pair = blockIdx.x;                              // (entry, head), heads fastest
    const int r = pair / nq, h = pair - r * nq;
    const int first = run_start[r], count = run_start[r + 1] - first;
    if (count <= 1 || (count <= AHEAD && wv > 0)) return;     // (with up to sixteen runs no wave waits for another below)
    const size_t stride_ml = (size_t)nq * 2, stride_o = (size_t)nq * d;
    const float* ml = part_ml + ((size_t)first * nq + h) * 2;
    const float* po = part_o + ((size_t)first * nq + h) * d;
    const int e0 = 2 * lane, e1 = 128 + 2 * lane;             // d <= 256 and even: up to two pairs of elements a lane
    float ms0 = -INFINITY, ls0 = 0.f, m = -INFINITY;
    if (lane < count) {
        ms0 = ml[lane * stride_ml];
        ls0 = ml[lane * stride_ml + 1];
        m = ms0;
    }
    float2 v[AHEAD][2];
    if (wv == 0) {
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            const size_t o = (size_t)min(u, count - 1) * stride_o;
            v[u][0] = e0 < d ? *reinterpret_cast<const float2*>(po + o + e0) : make_float2(0.f, 0.f);
            v[u][1] = e1 < d ? *reinterpret_cast<const float2*>(po + o + e1) : make_float2(0.f, 0.f);
        }
    }
    for (int s = lane + 64; s < count; s += 64) m = fmaxf(m, ml[s * stride_ml]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    float l = 0.f;
    float2 acc[2] = {make_float2(0.f, 0.f), make_float2(0.f, 0.f)};
    if (wv == 0) {
        const float w0 = ms0 == -INFINITY ? 0.f : __expf(ms0 - m);   // (a lane past the last run: 0)
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            const float w = __shfl(w0, u, 64);
            l = fmaf(__shfl(ls0, u, 64), w, l);
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                acc[k].x = fmaf(v[u][k].x, w, acc[k].x);
                acc[k].y = fmaf(v[u][k].y, w, acc[k].y);
            }
        }
    }
    for (int s0 = AHEAD * (wv == 0 ? 4 : wv); s0 < count; s0 += 4 * AHEAD) {
        float w[AHEAD];
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            const int s = min(s0 + u, count - 1);
            const float ms = ml[s * stride_ml];
            w[u] = (s0 + u < count && ms != -INFINITY) ? __expf(ms - m) : 0.f;
            l = fmaf(ml[s * stride_ml + 1], w[u], l);
            v[u][0] = e0 < d ? *reinterpret_cast<const float2*>(po + s * stride_o + e0) : make_float2(0.f, 0.f);
            v[u][1] = e1 < d ? *reinterpret_cast<const float2*>(po + s * stride_o + e1) : make_float2(0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < AHEAD; ++u)
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                acc[k].x = fmaf(v[u][k].x, w[u], acc[k].x);
                acc[k].y = fmaf(v[u][k].y, w[u], acc[k].y);
            }
    }
    if (count > AHEAD) {
        // (all four waves are still here, one without runs with sums of zero)
        __shared__ float4 sum_o[3][64];
        __shared__ float sum_l[3];
        if (wv > 0) {
            sum_o[wv - 1][lane] = make_float4(acc[0].x, acc[0].y, acc[1].x, acc[1].y);
            if (lane == 0) sum_l[wv - 1] = l;
        }
        __syncthreads();
        if (wv > 0) return;
        for (int o = 0; o < 3; ++o) {
            const float4 t = sum_o[o][lane];
            acc[0].x += t.x; acc[0].y += t.y; acc[1].x += t.z; acc[1].y += t.w;
            l += sum_l[o];
        }
    }
    const float inv = 1.0f / l;
    bf16_t* o = out + ((size_t)(tokens ? tokens[r] : r) * nq + h) * d;   // (tokens: the row of out that entry r's token has)
    if (e0 < d) {
        o[e0] = (bf16_t)(acc[0].x * inv);
        o[e0 + 1] = (bf16_t)(acc[0].y * inv);
    }
    if (e1 < d) {
        o[e1] = (bf16_t)(acc[1].x * inv);
        o[e1 + 1] = (bf16_t)(acc[1].y * inv);
    }
}

__device__ __forceinline__ float max3_raw(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// ------------------------------------------------- prompt portions, by block ---
// For portions of many tokens a block of NW waves shares its keys and values:
// every 32-key slice is copied once from the pages into LDS (by the load unit,
// global_load_lds_dwordx4, in MFMA operand order, three slices in flight) and
// read from there by all waves, each of which works on NQT column tiles.  Under
// a causal mask the last columns of a prompt see many times the keys of the
// first; so that no CU idles while another works through a long run, a block
// is given several work items with about the same total of slices as every
// other block's.
//
// Within a slice the 16 rows of key tile t are the keys (r / 4) * 8 + t * 4 + r % 4:
// lane (col, g) then holds the scores of the 8 consecutive keys g*8 .. g*8+7,
// which makes the P.V operand of values one 16-byte run of a value page.
#define ATTN_BT_LDS 2048
#define ATTN_STAGES 4
constexpr int attn_vmcnt_imm(int v) { return (v & 15) | (7 << 4) | (15 << 8) | ((v >> 4) << 14); }

template <int DT, int NQT, int NW, int KGRP>
__global__ __launch_bounds__(64 * NW * KGRP, (NW * KGRP <= 4 ? 2 : 1)) void attn_mfma_block_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int bt_stride, const int32_t* __restrict__ cu_tokens,
    const int32_t* __restrict__ start_pos, const int32_t* __restrict__ work,
    const int32_t* __restrict__ block_items, int nq, int nkv, int page_size, int page_shift,
    int window, float scale) {
    constexpr int D = DT * 16;
    constexpr int KS = (D + 31) / 32;
    constexpr int KFR = 2 * KS, VFR = DT, FR = KFR + VFR;   // 1 KB fragments per slice
    // KGRP groups of NW waves: group k works on the slices k, k + KGRP, ... of the same columns
    // and the groups' results are merged at the end; a stage holds KGRP slices, one per group
    constexpr int NWT = NW * KGRP, FRT = FR * KGRP;
    constexpr int LPW = (FRT + NWT - 1) / NWT;               // copies a wave issues per stage
    constexpr int BCOLS = NW * NQT * 16;                     // columns of a block
    constexpr int STAGES = ATTN_STAGES;                      // stages in LDS: one in use, the rest in flight
    __shared__ __attribute__((aligned(1024))) bf16_t smem[STAGES * FRT * 512];
    __shared__ int32_t pages[ATTN_BT_LDS];
    static_assert(ATTN_STAGES >= 3, "the barrier between reads and MFMAs needs the copies one slice further ahead");
    static_assert(KGRP == 1 || (size_t)STAGES * FRT * 1024 >= (size_t)NW * NQT * (DT * 1024 + 512),
                  "the merge of the key groups borrows the stages");
    const int tid = threadIdx.x, lane = tid & 63, wave_all = tid >> 6;
    const int wave = wave_all % NW, kgi = wave_all / NW;     // column tile(s) and key group of this wave
    const int qc = lane & 15, kg = lane >> 4;
    const int g = blockIdx.y;
    const int G = nq / nkv;
    // A block works through the items block_items[b] .. block_items[b + 1] of the work table one
    // after the other (the host deals items to blocks so that all blocks have about the same
    // number of slices to go through); without that table block b has item b, the last ones,
    // which see the most keys, first.
    const int it_begin = block_items ? block_items[blockIdx.x] : (int)(gridDim.x - 1 - blockIdx.x);
    const int it_end = block_items ? block_items[blockIdx.x + 1] : it_begin + 1;
    for (int item = it_begin; item < it_end; ++item) {
    if (item > it_begin) __syncthreads();   // the last item's slices and page numbers are read
    const int r = work[2 * item];
    const int bcol0 = work[2 * item + 1];
    const int tok0 = cu_tokens[r];
    const int n = cu_tokens[r + 1] - tok0;
    const int P = start_pos[r];
    const int ncols = n * G;
    const int32_t* bt = block_tables + (size_t)r * bt_stride;
    const int col0 = bcol0 + wave * (NQT * 16);   // this wave's first column

    int c_tok[NQT], c_head[NQT], c_pos[NQT], c_lo[NQT];
    bool c_ok[NQT];
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
        const int c = col0 + t * 16 + qc;
        c_ok[t] = c < ncols;
        const int cc = c_ok[t] ? c : ncols - 1;
        const int tl = cc / G;
        c_tok[t] = tok0 + tl;
        c_head[t] = g * G + (cc - tl * G);
        c_pos[t] = c_ok[t] ? P + tl : -1;
        c_lo[t] = window > 0 ? max(0, P + tl - window + 1) : 0;
    }
    // keys any column of the block can see (the same for all four waves)
    const int tl_first = bcol0 / G;
    const int tl_last = (min(bcol0 + BCOLS, ncols) - 1) / G;
    const int kmin = window > 0 ? max(0, P + tl_first - window + 1) : 0;
    const int kmax = P + tl_last;
    const int kb0 = (kmin / 32) * 32;
    const int nsteps = (kmax - kb0) / 32 + 1;
    // The page numbers of the block's keys come from LDS, always (a lookup in the table itself
    // is a memory load, and to wait for it is to wait for every copy in flight).  Keys beyond
    // what ATTN_BT_LDS pages hold are worked through in segments, each with its own page numbers
    // in LDS and a pipeline of copies of its own.
    const int seg_steps = max(KGRP, ((((ATTN_BT_LDS - 1) * page_size) >> 5) / KGRP) * KGRP);
    int pg0 = 0;

    bf16x8 qf[NQT][KS];
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
        const bf16_t* qp = q + (size_t)c_tok[t] * q_stride + (size_t)c_head[t] * D;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int e = ks * 32 + kg * 8;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (c_ok[t] && e < D) v = *reinterpret_cast<const uint4*>(qp + e);   // zero past D: K may hold anything there
            qf[t][ks] = *reinterpret_cast<bf16x8*>(&v);
        }
    }
    floatx4 oacc[NQT][DT];
    float m_run[NQT], l_run[NQT];
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
        m_run[t] = -INFINITY;
        l_run[t] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) oacc[t][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    // q is waited for here, once: the compiler does not see the copies below (they are inline
    // assembly), so a wait for q that it placed inside the loop would be a wait for all copies
    // in flight, in every iteration.
    __builtin_amdgcn_s_waitcnt(vmcnt_imm0());

    // (what LDS holds is a page's start in units of 16 bytes: page number x page_stride / 8)
#define ATTN_PAGE(j) pages[page_index((j), page_size, page_shift) - pg0]
    // fragment f of a slice: f < KFR is key tile f / KS, k-step f % KS; else value tile f - KFR
    // Every wave issues LPW copies per slice, also past the last slice (clamped to it) and past
    // the last fragment (a second copy of it): the count in flight is then the same for every
    // wave and iteration, and one constant wait covers the slice about to be read.
    // What does not change from slice to slice is worked out once per copy: which fragment
    // (the wave's index is made a scalar, so that the choice between a key and a value
    // fragment is a branch of the whole wave and not two masked halves), the lane's key within
    // the slice and its offset within a page; a slice then costs a page lookup and one
    // multiply-add per copy.
    const int wave_u = __builtin_amdgcn_readfirstlane(wave_all);
    const unsigned smem_addr = (unsigned)(size_t)(lds_ptr_t)smem;    // where the stages begin in LDS
    const uint32_t page_stride = (uint32_t)nkv * page_size * D;      // elements of a page, K or V (the host checks that it fits)
    const bf16_t* kbase = k_cache + (size_t)g * page_size * D;
    const bf16_t* vbase = v_cache + (size_t)g * D * page_size;
    const int vkmax = (kmax >> 3) << 3;
    int cp_F[LPW], cp_sub[LPW], cp_key[LPW], cp_off[LPW];
    bool cp_is_k[LPW];
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
        const int F = min(wave_u + NWT * j, FRT - 1);
        const int f = F % FR;
        cp_F[j] = F;
        cp_sub[j] = F / FR;
        cp_is_k[j] = f < KFR;
        if (f < KFR) {
            const int kt = f / KS, ks = f - kt * KS;
            cp_key[j] = (qc >> 2) * 8 + kt * 4 + (qc & 3);
            cp_off[j] = min(ks * 32 + kg * 8, D - 8) >> 3;          // in units of 8 elements, as the page starts are
        } else {
            cp_key[j] = kg * 8;
            cp_off[j] = (((f - KFR) * 16 + qc) * page_size) >> 3;   // (pages hold a multiple of 8 tokens)
        }
    }
#define ATTN_ISSUE(step)                                                                            \
    {                                                                                               \
        const int st_ = (step) % STAGES;                                                            \
        _Pragma("unroll") for (int j = 0; j < LPW; ++j) {                                           \
            const int kb_ = kb0 + min(seg0 + (step) * KGRP + cp_sub[j], seg1 - 1) * 32;             \
            const bf16_t* g_;                                                                       \
            if (cp_is_k[j]) {                                                                       \
                const int key = min(kb_ + cp_key[j], kmax);                                         \
                g_ = kbase + ((uint64_t)((uint32_t)ATTN_PAGE(key) +                                 \
                              (uint32_t)(page_slot(key, page_size, page_shift) * (D / 8) + cp_off[j])) << 3); \
            } else {                                                                                \
                const int j0 = min(kb_ + cp_key[j], vkmax);                                         \
                g_ = vbase + ((uint64_t)((uint32_t)ATTN_PAGE(j0) +                                  \
                              (uint32_t)(cp_off[j] + (page_slot(j0, page_size, page_shift) >> 3))) << 3); \
            }                                                                                       \
            copy16_to_lds_at(g_, smem_addr + (unsigned)(st_ * FRT + cp_F[j]) * 1024u);              \
        }                                                                                           \
    }

    // The softmax works on raw scores with the scale folded into the exponent:
    //   p = 2^((s - m) * scale * log2 e),
    // masks only the slices that touch a column's causal or window edge, and rescales the
    // accumulators only when some column's maximum moved: away from the diagonal the vector
    // unit then has a fused multiply-add, an exponential and an addition per score to do.
    const float sl2 = scale * 1.44269504088896f;
    const float slack = 8.0f / sl2;   // 8 in the exponent's units, as a raw score
    int t_min_pos[NQT], t_max_lo[NQT];
#pragma unroll
    for (int t = 0; t < NQT; ++t) {
        int mn = c_pos[t], mx = c_lo[t];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            mn = min(mn, __shfl_xor(mn, o, 64));
            mx = max(mx, __shfl_xor(mx, o, 64));
        }
        t_min_pos[t] = mn;
        t_max_lo[t] = mx;
    }

    for (int seg0 = 0; seg0 < nsteps; seg0 += seg_steps) {
    const int seg1 = min(nsteps, seg0 + seg_steps);
    if (seg0 > 0) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm0());   // the segment before: its copies past the end have landed,
        __syncthreads();                            // its slices and page numbers are read
    }
    pg0 = page_index(kb0 + seg0 * 32, page_size, page_shift);
    {
        const int npg = page_index(min(kmax, kb0 + seg1 * 32 - 1), page_size, page_shift) - pg0 + 1;
        for (int i = tid; i < npg; i += 64 * NWT) pages[i] = (int32_t)((uint32_t)bt[pg0 + i] * (page_stride >> 3));
    }
    __syncthreads();   // pages[] is written
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) ATTN_ISSUE(s)
    const int nsup = (seg1 - seg0 + KGRP - 1) / KGRP;
    // The barrier of a slice stands between the reads of its key fragments and their MFMAs: a
    // wave arrives with its keys on the way and starts its MFMAs when the barrier opens.  The
    // barrier of slice s makes slice s + 1 visible, so the copies are one slice further ahead.
    __builtin_amdgcn_s_waitcnt(attn_vmcnt_imm((STAGES - 2) * LPW));   // this wave's copies of the first stage are in
    __syncthreads();
    for (int s = 0; s < nsup; ++s) {
        const bool mine = !(KGRP > 1 && seg0 + s * KGRP + kgi >= seg1);   // past the last slice: nothing for this group
        const bf16_t* st = smem + ((s % STAGES) * FRT + kgi * FR) * 512;
        bf16x8 kfr[2][KS];   // (read also where there is no slice for this group: the stage is there)
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                kfr[kt][ks] = *reinterpret_cast<const bf16x8*>(st + (kt * KS + ks) * 512 + lane * 8);
        __builtin_amdgcn_s_waitcnt(attn_vmcnt_imm((STAGES - 3) * LPW));   // this wave's copies of stage s + 1 are in
        asm volatile("s_barrier" ::: "memory");     // ... and the other waves'; stage s - 1 is read
        ATTN_ISSUE(s + STAGES - 1)                  // into the stage of step s - 1
        if (!mine) continue;
        const int kb = kb0 + (seg0 + s * KGRP + kgi) * 32;
        floatx4 sacc[NQT][2];
#pragma unroll
        for (int t = 0; t < NQT; ++t) sacc[t][0] = sacc[t][1] = floatx4{0.f, 0.f, 0.f, 0.f};
        __builtin_amdgcn_s_setprio(1);   // a wave with its keys in registers goes before the softmax of the others
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                for (int t = 0; t < NQT; ++t)
                    sacc[t][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kfr[kt][ks], qf[t][ks], sacc[t][kt], 0, 0, 0);
            }
        __builtin_amdgcn_s_setprio(0);
        bf16x8 pf[NQT];
#pragma unroll
        for (int t = 0; t < NQT; ++t) {
            float sv[8];
            // lane (col, g): key kb + g*8 + e is row g*4 + e%4 of tile e/4
#pragma unroll
            for (int e = 0; e < 8; ++e) sv[e] = sacc[t][e >> 2][e & 3];
            if (kb + 31 > t_min_pos[t] || kb < t_max_lo[t]) {   // the slice touches an edge of some column
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int j = kb + kg * 8 + e;
                    if (!(j >= c_lo[t] && j <= c_pos[t])) sv[e] = -INFINITY;
                }
            }
            // (three-operand maxima as the instruction is: fmaxf has every operand quieted first, eight more instructions a slice)
            float mt = max3_raw(max3_raw(sv[0], sv[1], sv[2]), max3_raw(sv[3], sv[4], sv[5]), fmaxf(sv[6], sv[7]));
            // m_run is the reference the exponentials are taken against: the largest score seen
            // when it was last moved, in raw score units.  It is moved (the maximum over a
            // column's four lanes, the accumulators rescaled) only when some score exceeds it by
            // more than 8 in the exponent's units: until then p stays below 2^8, far from any
            // overflow, and the quotient o / l does not depend on the reference.  Scores that
            // creep up slice after slice, as they do towards the diagonal under a rotation,
            // would otherwise rescale the accumulators in every slice.
            float m_new = m_run[t], alpha = 1.f;
            if (__any(mt > m_run[t] + slack)) {
                mt = rows_max(mt);
                m_new = fmaxf(m_run[t], mt);
                alpha = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f((m_run[t] - m_new) * sl2);
            }
            const float mb = m_new == -INFINITY ? 0.f : m_new * sl2;
            float ps = 0.f;
            bf16x8 pv;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float p = __builtin_amdgcn_exp2f(fmaf(sv[e], sl2, -mb));   // 2^-inf = 0 for masked scores
                ps += p;
                pv[e] = (bf16_t)p;
            }
            pf[t] = pv;
            l_run[t] = l_run[t] * alpha + ps;
            m_run[t] = m_new;
            if (__any(alpha != 1.f)) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    oacc[t][dt][0] *= alpha; oacc[t][dt][1] *= alpha;
                    oacc[t][dt][2] *= alpha; oacc[t][dt][3] *= alpha;
                }
            }
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const bf16x8 vfr = *reinterpret_cast<const bf16x8*>(st + (KFR + dt) * 512 + lane * 8);
#pragma unroll
            for (int t = 0; t < NQT; ++t)
                oacc[t][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vfr, pf[t], oacc[t][dt], 0, 0, 0);
        }
    }
    }   // segments
#undef ATTN_ISSUE
#undef ATTN_PAGE
    __builtin_amdgcn_s_waitcnt(vmcnt_imm0());   // the copies past the end must not outlive the block

    if constexpr (KGRP > 1) {
        // The second key group hands its maxima, sums and accumulators to the first through the
        // stages (all copies have landed and all slices are read after the barrier).
        static_assert(KGRP == 2, "the merge is written for two groups");
        float* mo = reinterpret_cast<float*>(smem) + wave * NQT * (DT * 256 + 128);
        __syncthreads();
        if (kgi == 1) {
#pragma unroll
            for (int t = 0; t < NQT; ++t) {
                float* mt = mo + t * (DT * 256 + 128);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    *reinterpret_cast<float4*>(mt + dt * 256 + lane * 4) =
                        make_float4(oacc[t][dt][0], oacc[t][dt][1], oacc[t][dt][2], oacc[t][dt][3]);
                mt[DT * 256 + lane * 2] = m_run[t];
                mt[DT * 256 + lane * 2 + 1] = l_run[t];
            }
        }
        __syncthreads();
        if (kgi == 1) continue;   // the next item, if any
#pragma unroll
        for (int t = 0; t < NQT; ++t) {
            const float* mt = mo + t * (DT * 256 + 128);
            const float m2 = mt[DT * 256 + lane * 2], l2 = mt[DT * 256 + lane * 2 + 1];
            const float m = fmaxf(m_run[t], m2);
            const float a1 = m_run[t] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m_run[t] - m) * sl2);
            const float a2 = m2 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m2 - m) * sl2);
            l_run[t] = l_run[t] * a1 + l2 * a2;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const float4 o2 = *reinterpret_cast<const float4*>(mt + dt * 256 + lane * 4);
                oacc[t][dt][0] = oacc[t][dt][0] * a1 + o2.x * a2;
                oacc[t][dt][1] = oacc[t][dt][1] * a1 + o2.y * a2;
                oacc[t][dt][2] = oacc[t][dt][2] * a1 + o2.z * a2;
                oacc[t][dt][3] = oacc[t][dt][3] * a1 + o2.w * a2;
            }
        }
    }

#pragma unroll
    for (int t = 0; t < NQT; ++t) {
        float l = l_run[t];
        l = rows_sum(l);
        if (!c_ok[t]) continue;
        const float inv = 1.0f / l;
        bf16_t* op = out + ((size_t)c_tok[t] * nq + c_head[t]) * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            union { bf16_t h[4]; uint2 u; } pk;
#pragma unroll
            for (int i = 0; i < 4; ++i) pk.h[i] = (bf16_t)(oacc[t][dt][i] * inv);
            *reinterpret_cast<uint2*>(op + dt * 16 + kg * 4) = pk.u;
        }
    }
    }   // items
}

template <int DT>
static int launch_attn(const bf16_t* q, int q_stride, bf16_t* out, float* part_o, float* part_ml,
                       const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* block_tables,
                       int bt_stride, const int32_t* cu_tokens, const int32_t* start_pos,
                       const int32_t* work, int num_work, const int32_t* block_items, int num_blocks,
                       int tiles_per_entry, int cols_per_wave,
                       int splits, int nq, int nkv, int page_size, int window, float scale,
                       int T_total, hipStream_t s, const AttnFuse* fuse = nullptr, int key_groups = 2,
                       const AttnFuse* runs_only = nullptr) {
    int page_shift = 0;   // the page size is a power of two (tff_attention_mfma_supported)
    while ((1 << page_shift) < page_size) ++page_shift;
    if (cols_per_wave == 256) {
        // Eight waves of two column tiles each, one block a CU (a wave has 256 registers): every
        // key and value fragment read from LDS feeds two MFMAs, half the LDS traffic per flop of
        // the blocks below.  For prompts long enough to give every block several items.
        if constexpr (DT <= 8) {
            attn_mfma_block_kernel<DT, 2, 8, 1><<<dim3(num_blocks, nkv), 512, 0, s>>>(
                q, q_stride, out, k_cache, v_cache, block_tables, bt_stride, cu_tokens, start_pos, work,
                block_items, nq, nkv, page_size, page_shift, window, scale);
            return tff_check_launch("attention_mfma_block256");
        } else {
            return tff_fail("attention_mfma: blocks of 256 columns take head sizes up to 128");
        }
    }
    if (cols_per_wave == 128) {   // blocks of eight waves that share their keys through LDS
        // Two groups of eight waves that take every other slice, where LDS holds their stages:
        // half as many slices one after the other for a block, which is what counts when there
        // is little work for the machine; with plenty of it, blocks of one group, two to a CU,
        // spend less on merging and waiting for each other.
        if constexpr (DT <= 8) {
            if (key_groups == 2)
                attn_mfma_block_kernel<DT, 1, 8, 2><<<dim3(num_blocks, nkv), 1024, 0, s>>>(
                    q, q_stride, out, k_cache, v_cache, block_tables, bt_stride, cu_tokens, start_pos, work,
                    block_items, nq, nkv, page_size, page_shift, window, scale);
            else
                attn_mfma_block_kernel<DT, 1, 8, 1><<<dim3(num_blocks, nkv), 512, 0, s>>>(
                    q, q_stride, out, k_cache, v_cache, block_tables, bt_stride, cu_tokens, start_pos, work,
                    block_items, nq, nkv, page_size, page_shift, window, scale);
        } else
            attn_mfma_block_kernel<DT, 1, 8, 1><<<dim3(num_blocks, nkv), 512, 0, s>>>(
                q, q_stride, out, k_cache, v_cache, block_tables, bt_stride, cu_tokens, start_pos, work,
                block_items, nq, nkv, page_size, page_shift, window, scale);
        return tff_check_launch("attention_mfma_block");
    }
    const dim3 grid(num_work, nkv, max(splits, 1));
    // (runs_only: nothing to fuse, q is finished and the pages hold the tokens; only the runs of keys are set)
    const AttnFuse fz = fuse ? *fuse : runs_only ? *runs_only
                                                 : AttnFuse{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0.f, 0, nullptr};
#define TFF_ATTN_ARGS                                                                              \
    q, q_stride, out, part_o, part_ml, k_cache, v_cache, block_tables, bt_stride, cu_tokens,       \
        start_pos, work, tiles_per_entry, nq, nkv, page_size, page_shift, window, scale, T_total
    if (fuse && splits == 0) {
        // a block of eight waves per entry (or run of keys dealt by the host) and kv head: the keys split
        // among its waves, merged in LDS
        if constexpr (DT <= 8) {
            // (two waves to a SIMD have 256 registers each: four steps of keys and values in flight a wave up to
            // a head size of 64, two up to 96, one beyond; eight waves keep a CU's 100 GB/s busy either way)
            const dim3 bgrid = fuse->key_runs ? dim3(num_work * nkv, 1, 1) : dim3(num_work, nkv, 1);
            attn_wave_kernel<DT, false, (DT <= 4 ? 4 : DT <= 6 ? 2 : 1), true, 8><<<bgrid, 512, 0, s>>>(TFF_ATTN_ARGS, fz);
        } else {
            return tff_fail("attention_decode_fused: blocks of eight waves take head sizes up to 128");
        }
    } else if (fuse && fuse->key_runs) {
        // runs of keys dealt by the host: num_work runs, a wave per run, kv head and column tile
        attn_wave_kernel<DT, true, (DT <= 8 ? 4 : 1), true><<<dim3(num_work * nkv, 1, tiles_per_entry), 64, 0, s>>>(TFF_ATTN_ARGS, fz);
    } else if (fuse) {
        if (splits > 1)
            attn_wave_kernel<DT, true, (DT <= 8 ? 4 : 1), true><<<grid, 64, 0, s>>>(TFF_ATTN_ARGS, fz);
        else
            attn_wave_kernel<DT, false, (DT <= 8 ? 4 : 1), true><<<grid, 64, 0, s>>>(TFF_ATTN_ARGS, fz);
    } else if (fz.key_runs) {
        // (the same for q, k and v that are finished and in their pages)
        attn_wave_kernel<DT, true, (DT <= 8 ? 4 : 2)><<<dim3(num_work * nkv, 1, tiles_per_entry), 64, 0, s>>>(TFF_ATTN_ARGS, fz);
    } else if (splits > 1) {
        attn_wave_kernel<DT, true, (DT <= 8 ? 4 : 2)><<<grid, 64, 0, s>>>(TFF_ATTN_ARGS, fz);
    } else {
        attn_wave_kernel<DT, false, (DT <= 8 ? 4 : 2)><<<grid, 64, 0, s>>>(TFF_ATTN_ARGS, fz);
    }
#undef TFF_ATTN_ARGS
    return tff_check_launch("attention_mfma");
}

TFF_API int tff_attention_mfma_supported(int d, int page_size) {
    if (page_size < 8 || (page_size & (page_size - 1))) return 0;   // a power of two, at least 8
    switch (d) {
        case 16: case 32: case 48: case 64: case 80: case 96: case 112: case 128: case 192: case 256:
            return 1;
        default:
            return 0;
    }
}

TFF_API int tff_attention_mfma(const void* q, int q_stride, void* out, float* part_o, float* part_ml,
                               const void* k_cache, const void* v_cache,
                               const int32_t* block_tables, int bt_stride, const int32_t* cu_tokens,
                               const int32_t* start_pos, const int32_t* work, int num_work,
                               const int32_t* block_items, int num_blocks,
                               int tiles_per_entry, int cols_per_wave, int key_groups, int splits, int T_total,
                               int nq, int nkv, int d, int page_size, int num_pages, int window,
                               float scale, tff_stream_t stream) {
    TFF_REQUIRE(q && out && k_cache && v_cache && block_tables && cu_tokens && start_pos,
                "attention_mfma: null pointer");
    TFF_REQUIRE(key_groups == 1 || key_groups == 2, "attention_mfma: %d key groups (1 or 2)", key_groups);
    TFF_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0,
                "attention_mfma: %d query heads are not a multiple of %d key heads", nq, nkv);
    TFF_REQUIRE(tff_attention_mfma_supported(d, page_size),
                "attention_mfma: head size %d with pages of %d is not supported by the matrix-core "
                "kernel (head sizes 16..128 in steps of 16, 192, 256; pages of a power of two, at least 8)", d, page_size);
    TFF_REQUIRE((long)nkv * page_size * d < (1L << 31), "attention_mfma: a page of %d x %d x %d elements is too large", nkv, page_size, d);
    // (the blocks of long portions keep a page's start as a 32-bit count of 16-byte units)
    TFF_REQUIRE(cols_per_wave < 128 || (long)num_pages * nkv * page_size * d / 8 < (1L << 32),
                "attention_mfma: a cache of %d pages of %d x %d x %d elements is too large for the kernel of long portions",
                num_pages, nkv, page_size, d);
    TFF_REQUIRE(q_stride >= nq * d && q_stride % 8 == 0 && ((uintptr_t)q % 16) == 0,
                "attention_mfma: query rows must be 16-byte aligned (stride %d)", q_stride);
    TFF_REQUIRE(cols_per_wave == 16 || cols_per_wave == 128 || cols_per_wave == 256,
                "attention_mfma: bad tile width %d", cols_per_wave);
    TFF_REQUIRE(cols_per_wave < 128 || (work && splits == 1),
                "attention_mfma: blocks of 128 or 256 columns take a work table and no key split");
    TFF_REQUIRE(cols_per_wave != 256 || d <= 128, "attention_mfma: blocks of 256 columns take head sizes up to 128, not %d", d);
    if (cols_per_wave >= 128) {
        if (!block_items) num_blocks = num_work;
        TFF_REQUIRE(num_blocks >= 0 && num_blocks <= num_work,
                    "attention_mfma: %d blocks for %d work items", num_blocks, num_work);
        if (num_blocks == 0) return 0;
    }
    TFF_REQUIRE(splits >= 1 && splits <= 65535 && nkv <= 65535, "attention_mfma: bad split count %d", splits);
    TFF_REQUIRE(splits == 1 || (part_o && part_ml), "attention_mfma: split keys need a workspace");
    TFF_REQUIRE(splits == 1 || cols_per_wave == 16,
                "attention_mfma: keys are split for entries of one token (16 columns a wave) only");
    TFF_REQUIRE(work || tiles_per_entry >= 1, "attention_mfma: neither a work table nor a tile count");
    TFF_REQUIRE(bt_stride > 0 && num_pages > 0 && window >= 0 && T_total >= 0, "attention_mfma: bad geometry");
    if (num_work <= 0) return 0;
    hipStream_t s = (hipStream_t)stream;
#define TFF_ATTN_CASE(DTV)                                                                          \
    case DTV * 16:                                                                                  \
        return launch_attn<DTV>((const bf16_t*)q, q_stride, (bf16_t*)out, part_o, part_ml,          \
                                (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables,       \
                                bt_stride, cu_tokens, start_pos, work, num_work, block_items,       \
                                num_blocks, tiles_per_entry,                                        \
                                cols_per_wave, splits, nq, nkv, page_size, window, scale, T_total, s, \
                                nullptr, key_groups);
    switch (d) {
        TFF_ATTN_CASE(1) TFF_ATTN_CASE(2) TFF_ATTN_CASE(3) TFF_ATTN_CASE(4) TFF_ATTN_CASE(5)
        TFF_ATTN_CASE(6) TFF_ATTN_CASE(7) TFF_ATTN_CASE(8) TFF_ATTN_CASE(12) TFF_ATTN_CASE(16)
        default: break;
    }
#undef TFF_ATTN_CASE
    return tff_fail("attention_mfma: head size %d", d);
}

// Decoding steps (every entry brings one token) from the fused projection's output: q, k and v
// of token r are row r of qkv ([R, (nq + 2 nkv) d]).  Per head, q and k get their RMS norm
// (weights [d]; both null: none) and the rotation by the angles of the token's position
// start_pos[r] (cos_sin [max_pos, d/2, 2]; null: none; the whole head is rotated; pairing 0:
// (i, i + d/2), which needs d to be a multiple of 64, 1: (2i, 2i+1)).  Where slot_mapping[r] >= 0
// the token's key and value go to position start_pos[r] of the entry's pages (the slot that
// the entry's block table gives for it); where it is negative, and everywhere if slot_mapping
// is null, the pages hold them already and are only read.  Then attention as
// tff_attention_mfma does it for such a step.
TFF_API int tff_attention_decode_fused(const void* qkv, int qkv_stride, void* out, float* part_o,
                                       float* part_ml, void* k_cache, void* v_cache,
                                       const int32_t* block_tables, int bt_stride,
                                       const int32_t* cu_tokens, const int32_t* start_pos,
                                       const int32_t* slot_mapping,
                                       const float* q_weight, const float* k_weight, float eps,
                                       const float* cos_sin, int max_pos, int pairing,
                                       int splits, int R, int nq, int nkv, int d, int page_size,
                                       int num_pages, int window, float scale, tff_stream_t stream) {
    TFF_REQUIRE(qkv && out && k_cache && v_cache && block_tables && cu_tokens && start_pos,
                "attention_decode_fused: null pointer");
    TFF_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0,
                "attention_decode_fused: %d query heads are not a multiple of %d key heads", nq, nkv);
    TFF_REQUIRE(tff_attention_mfma_supported(d, page_size),
                "attention_decode_fused: head size %d with pages of %d is not supported by the "
                "matrix-core kernel", d, page_size);
    TFF_REQUIRE(qkv_stride >= (nq + 2 * nkv) * d && qkv_stride % 8 == 0 && ((uintptr_t)qkv % 16) == 0,
                "attention_decode_fused: rows of %d elements do not hold (nq + 2 nkv) d = %d, 16-byte aligned",
                qkv_stride, (nq + 2 * nkv) * d);
    TFF_REQUIRE((q_weight == nullptr) == (k_weight == nullptr),
                "attention_decode_fused: q and k norm weights must both be given or both be absent");
    TFF_REQUIRE(!cos_sin || ((pairing == 1 || (pairing == 0 && d % 64 == 0)) && max_pos > 0),
                "attention_decode_fused: pairing %d with head size %d is not supported here", pairing, d);
    // splits 0: a block of eight waves per entry and kv head splits the keys among its waves and
    // merges in LDS (head sizes up to 128; no workspace, no tff_attention_split_reduce afterwards)
    TFF_REQUIRE(splits >= 0 && splits <= 256 && nkv <= 65535, "attention_decode_fused: bad split count %d", splits);
    TFF_REQUIRE(splits != 0 || d <= 128, "attention_decode_fused: blocks of eight waves take head sizes up to 128, not %d", d);
    TFF_REQUIRE(splits <= 1 || (part_o && part_ml), "attention_decode_fused: split keys need a workspace");
    TFF_REQUIRE(bt_stride > 0 && num_pages > 0 && window >= 0 && R >= 0, "attention_decode_fused: bad geometry");
    if (R == 0) return 0;
    const int tiles = (nq / nkv + 15) / 16;
    AttnFuse fz{q_weight, k_weight, cos_sin, slot_mapping ? (bf16_t*)k_cache : nullptr,
                slot_mapping ? (bf16_t*)v_cache : nullptr, slot_mapping, eps, pairing, nullptr};
    hipStream_t s = (hipStream_t)stream;
#define TFF_ATTN_CASE(DTV)                                                                          \
    case DTV * 16:                                                                                  \
        return launch_attn<DTV>((const bf16_t*)qkv, qkv_stride, (bf16_t*)out, part_o, part_ml,      \
                                (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables,       \
                                bt_stride, cu_tokens, start_pos, nullptr, R * tiles, nullptr, 0,    \
                                tiles, 16, splits, nq, nkv, page_size, window, scale, R, s, &fz);
    switch (d) {
        TFF_ATTN_CASE(1) TFF_ATTN_CASE(2) TFF_ATTN_CASE(3) TFF_ATTN_CASE(4) TFF_ATTN_CASE(5)
        TFF_ATTN_CASE(6) TFF_ATTN_CASE(7) TFF_ATTN_CASE(8) TFF_ATTN_CASE(12) TFF_ATTN_CASE(16)
        default: break;
    }
#undef TFF_ATTN_CASE
    return tff_fail("attention_decode_fused: head size %d", d);
}

TFF_API int tff_attention_split_reduce(const float* part_o, const float* part_ml, void* out,
                                       int splits, int R_total, int nq, int d, const int32_t* rows,
                                       int num_rows, tff_stream_t stream) {
    TFF_REQUIRE(part_o && part_ml && out, "attention_split_reduce: null pointer");
    TFF_REQUIRE(splits >= 1 && R_total >= 0 && nq > 0 && nq <= 65535 && d > 0,
                "attention_split_reduce: bad sizes");
    const int n = rows ? num_rows : R_total;
    TFF_REQUIRE(n >= 0 && n <= R_total, "attention_split_reduce: %d rows of %d entries", n, R_total);
    if (n == 0) return 0;
    TFF_REQUIRE(splits <= 256, "attention_split_reduce: at most 256 splits, got %d", splits);
    if (splits <= 4 && d <= 256)
        attn_split_reduce_few_kernel<<<(n * nq + 3) / 4, 256, 0, (hipStream_t)stream>>>(
            part_o, part_ml, (bf16_t*)out, splits, R_total, nq, d, rows, n);
    else
        attn_split_reduce_kernel<<<dim3(n, nq), 256, 0, (hipStream_t)stream>>>(
            part_o, part_ml, (bf16_t*)out, splits, R_total, nq, d, rows);
    return tff_check_launch("attention_split_reduce");
}

// The same step with every entry's keys dealt into runs by the caller, who knows the entries'
// lengths: key_runs [num_runs][4] = (entry, first key, end of keys, the entry's position), 16-byte
// aligned, the runs of entry r being run_start[r] .. run_start[r + 1] - 1 (run_start [R + 1]), in
// the order of the keys, without gap or overlap; a run's first key is the entry's first visible
// key rounded down to a multiple of 32, plus a multiple of 32; an entry number < 0 marks a run that
// is not in use.  A wave per run, kv head and column tile; runs
// of similar length keep all waves busy alike however uneven the entries' lengths are, where
// equal splits of every entry leave the longest entry's waves at work long after the others.
// block_waves 8: a block of eight waves per run and kv head instead, which split the run among them
// and merge in LDS (head sizes up to 128, one column tile).  merge 0: the caller knows that every
// entry is one run (run_start[r] = r), so nothing is partial and the second kernel is left out.
// Partial results (part_o [num_runs][nq][d], part_ml [num_runs][nq][2]) of the entries with more
// than one run are merged by a second kernel.
TFF_API int tff_attention_decode_runs(const void* qkv, int qkv_stride, void* out, float* part_o,
                                      float* part_ml, void* k_cache, void* v_cache,
                                      const int32_t* block_tables, int bt_stride,
                                      const int32_t* cu_tokens, const int32_t* start_pos,
                                      const int32_t* slot_mapping,
                                      const float* q_weight, const float* k_weight, float eps,
                                      const float* cos_sin, int max_pos, int pairing,
                                      const int32_t* key_runs, const int32_t* run_start, int num_runs,
                                      int block_waves, int merge, int R, int nq, int nkv, int d, int page_size,
                                      int num_pages, int window, float scale, tff_stream_t stream) {
    TFF_REQUIRE(qkv && out && k_cache && v_cache && block_tables && cu_tokens && start_pos,
                "attention_decode_runs: null pointer");
    TFF_REQUIRE(block_waves == 1 || (block_waves == 8 && d <= 128 && nq / nkv <= 16),
                "attention_decode_runs: a run gets one wave, or a block of eight (head sizes up to 128, up to 16 "
                "query heads a kv head), not %d with head size %d and %d query heads a kv head", block_waves, d, nq / nkv);
    TFF_REQUIRE(key_runs && run_start && part_o && part_ml, "attention_decode_runs: the runs and the workspace are needed");
    TFF_REQUIRE(((uintptr_t)key_runs % 16) == 0, "attention_decode_runs: key_runs must be 16-byte aligned");
    TFF_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0,
                "attention_decode_runs: %d query heads are not a multiple of %d key heads", nq, nkv);
    TFF_REQUIRE(tff_attention_mfma_supported(d, page_size),
                "attention_decode_runs: head size %d with pages of %d is not supported by the "
                "matrix-core kernel", d, page_size);
    TFF_REQUIRE(qkv_stride >= (nq + 2 * nkv) * d && qkv_stride % 8 == 0 && ((uintptr_t)qkv % 16) == 0,
                "attention_decode_runs: rows of %d elements do not hold (nq + 2 nkv) d = %d, 16-byte aligned",
                qkv_stride, (nq + 2 * nkv) * d);
    TFF_REQUIRE((q_weight == nullptr) == (k_weight == nullptr),
                "attention_decode_runs: q and k norm weights must both be given or both be absent");
    TFF_REQUIRE(!cos_sin || ((pairing == 1 || (pairing == 0 && d % 64 == 0)) && max_pos > 0),
                "attention_decode_runs: pairing %d with head size %d is not supported here", pairing, d);
    const int tiles = (nq / nkv + 15) / 16;
    TFF_REQUIRE(num_runs >= 0 && num_runs % 8 == 0 && (long)num_runs * nkv < (1L << 31) && tiles <= 65535 && d <= 256,
                "attention_decode_runs: %d runs (a multiple of eight is needed), %d kv heads, %d column tiles (at most "
                "65,535), head size %d (at most 256)", num_runs, nkv, tiles, d);
    TFF_REQUIRE(bt_stride > 0 && num_pages > 0 && window >= 0 && R >= 0, "attention_decode_runs: bad geometry");
    if (R == 0 || num_runs == 0) return 0;
    AttnFuse fz{q_weight, k_weight, cos_sin, slot_mapping ? (bf16_t*)k_cache : nullptr,
                slot_mapping ? (bf16_t*)v_cache : nullptr, slot_mapping, eps, pairing, key_runs};
    hipStream_t s = (hipStream_t)stream;
    int rc = -1;
#define TFF_ATTN_CASE(DTV)                                                                          \
    case DTV * 16:                                                                                  \
        rc = launch_attn<DTV>((const bf16_t*)qkv, qkv_stride, (bf16_t*)out, part_o, part_ml,        \
                              (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables,         \
                              bt_stride, cu_tokens, start_pos, nullptr, num_runs, nullptr, 0,       \
                              tiles, 16, block_waves == 8 ? 0 : 2, nq, nkv, page_size, window,      \
                              scale, R, s, &fz);                                                    \
        break;
    switch (d) {
        TFF_ATTN_CASE(1) TFF_ATTN_CASE(2) TFF_ATTN_CASE(3) TFF_ATTN_CASE(4) TFF_ATTN_CASE(5)
        TFF_ATTN_CASE(6) TFF_ATTN_CASE(7) TFF_ATTN_CASE(8) TFF_ATTN_CASE(12) TFF_ATTN_CASE(16)
        default: return tff_fail("attention_decode_runs: head size %d", d);
    }
#undef TFF_ATTN_CASE
    if (rc || !merge) return rc;
    attn_run_merge_kernel<<<R * nq, 256, 0, s>>>(part_o, part_ml, (bf16_t*)out, run_start, nullptr, R, nq, d);
    return tff_check_launch("attention_run_merge");
}

// Entries of one token among a step's entries (requests that decode beside prompt portions), q
// finished and the tokens' keys and values in their pages (tff_qk_norm_rope_kv), their keys
// dealt into runs by the caller as for tff_attention_decode_runs: key_runs [num_runs][4] = (the
// entry's row in the step's tables, first key, end of keys, the entry's position); the runs of
// the i-th such entry are run_start[i] .. run_start[i + 1] - 1 (run_start [num_entries + 1]) and
// tokens[i] is its token's row in q and out.  Rows of out that belong to other entries are not
// touched.  merge 0: the caller knows that every such entry is one run.
TFF_API int tff_attention_mfma_runs(const void* q, int q_stride, void* out, float* part_o, float* part_ml,
                                    const void* k_cache, const void* v_cache,
                                    const int32_t* block_tables, int bt_stride,
                                    const int32_t* cu_tokens, const int32_t* start_pos,
                                    const int32_t* key_runs, const int32_t* run_start,
                                    const int32_t* tokens, int num_runs, int num_entries, int merge,
                                    int T, int nq, int nkv, int d, int page_size, int num_pages,
                                    int window, float scale, tff_stream_t stream) {
    TFF_REQUIRE(q && out && k_cache && v_cache && block_tables && cu_tokens && start_pos,
                "attention_mfma_runs: null pointer");
    TFF_REQUIRE(key_runs && run_start && tokens && part_o && part_ml,
                "attention_mfma_runs: the runs, the tokens' rows and the workspace are needed");
    TFF_REQUIRE(((uintptr_t)key_runs % 16) == 0, "attention_mfma_runs: key_runs must be 16-byte aligned");
    TFF_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0,
                "attention_mfma_runs: %d query heads are not a multiple of %d key heads", nq, nkv);
    TFF_REQUIRE(tff_attention_mfma_supported(d, page_size),
                "attention_mfma_runs: head size %d with pages of %d is not supported by the matrix-core kernel",
                d, page_size);
    TFF_REQUIRE(q_stride >= nq * d && q_stride % 8 == 0 && ((uintptr_t)q % 16) == 0,
                "attention_mfma_runs: q rows of %d elements must hold nq*d = %d and be 16-byte aligned", q_stride, nq * d);
    const int tiles = (nq / nkv + 15) / 16;
    TFF_REQUIRE(num_runs >= 0 && num_runs % 8 == 0 && (long)num_runs * nkv < (1L << 31) && tiles <= 65535 && d <= 256,
                "attention_mfma_runs: %d runs (a multiple of eight is needed), %d kv heads, %d column tiles (at most "
                "65,535), head size %d (at most 256)", num_runs, nkv, tiles, d);
    TFF_REQUIRE(bt_stride > 0 && num_pages > 0 && window >= 0 && num_entries >= 0 && T >= 0, "attention_mfma_runs: bad geometry");
    if (num_entries == 0 || num_runs == 0) return 0;
    AttnFuse fz{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0.f, 0, key_runs};
    hipStream_t s = (hipStream_t)stream;
    int rc = -1;
#define TFF_ATTN_CASE(DTV)                                                                          \
    case DTV * 16:                                                                                  \
        rc = launch_attn<DTV>((const bf16_t*)q, q_stride, (bf16_t*)out, part_o, part_ml,            \
                              (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables,         \
                              bt_stride, cu_tokens, start_pos, nullptr, num_runs, nullptr, 0,       \
                              tiles, 16, 2, nq, nkv, page_size, window, scale, T, s, nullptr, 2, &fz); \
        break;
    switch (d) {
        TFF_ATTN_CASE(1) TFF_ATTN_CASE(2) TFF_ATTN_CASE(3) TFF_ATTN_CASE(4) TFF_ATTN_CASE(5)
        TFF_ATTN_CASE(6) TFF_ATTN_CASE(7) TFF_ATTN_CASE(8) TFF_ATTN_CASE(12) TFF_ATTN_CASE(16)
        default: return tff_fail("attention_mfma_runs: head size %d", d);
    }
#undef TFF_ATTN_CASE
    if (rc || !merge) return rc;
    attn_run_merge_kernel<<<num_entries * nq, 256, 0, s>>>(part_o, part_ml, (bf16_t*)out, run_start, tokens,
                                                                    num_entries, nq, d);
    return tff_check_launch("attention_run_merge");
}

// ------------------------------------------ decoding without any allocation ---
// The partial results of split keys need device memory besides the inputs and outputs.  The
// entry points above take it from the caller; this one keeps it in the library: one array per
// GPU, part of the code object, there from the moment the library is loaded on a device until
// the process ends.  Nothing in it has to start at zero (every wave of a split launch writes its
// rows, the empty ones too: maximum -inf, sum 0), so a call leaves nothing that the next one
// has to clear.
#define TFF_ATTN_STATIC_FLOATS (TFF_ATTENTION_STATIC_SCRATCH_BYTES / sizeof(float))   // 16 MiB a GPU
static __device__ __align__(256) float attn_static_scratch[TFF_ATTN_STATIC_FLOATS];

#define TFF_MAX_DEVICES 64
static float* attn_static_ptr[TFF_MAX_DEVICES];   // the array's address on each device, once asked for
static std::mutex attn_static_mutex;

// The device address of the current device's copy of the array.  The array's name is a host-side
// handle, not an address a kernel could use; every GPU has its own copy at its own address.
static int attn_static_address(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return tff_fail("attention_decode_fused_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= TFF_MAX_DEVICES)
        return tff_fail("attention_decode_fused_static: device %d is beyond the %d this library keeps scratch for",
                        dev, TFF_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(attn_static_mutex);
    if (!attn_static_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(attn_static_scratch));
        if (e != hipSuccess || !p)
            return tff_fail("attention_decode_fused_static: hipGetSymbolAddress on device %d: %s", dev,
                            hipGetErrorString(e));
        attn_static_ptr[dev] = (float*)p;
    }
    *out = attn_static_ptr[dev];
    return 0;
}

TFF_API int tff_attention_decode_fused_static(const void* qkv, int qkv_stride, void* out, void* k_cache,
                                              void* v_cache, const int32_t* block_tables, int bt_stride,
                                              const int32_t* cu_tokens, const int32_t* start_pos,
                                              const int32_t* slot_mapping, const float* q_weight,
                                              const float* k_weight, float eps, const float* cos_sin,
                                              int max_pos, int pairing, int splits, int R, int nq, int nkv,
                                              int d, int page_size, int num_pages, int window, float scale,
                                              tff_stream_t stream) {
    TFF_REQUIRE(splits >= 1 && splits <= 256 && R >= 0 && nq > 0 && d > 0,
                "attention_decode_fused_static: bad sizes (splits %d, entries %d, heads %d, head size %d)",
                splits, R, nq, d);
    float *part_o = nullptr, *part_ml = nullptr;
    if (splits > 1 && R > 0) {
        const size_t rows = (size_t)splits * R * nq;
        const size_t need = rows * ((size_t)d + 2);
        TFF_REQUIRE(need <= TFF_ATTN_STATIC_FLOATS,
                    "attention_decode_fused_static: %d splits x %d entries x %d heads of %d need %zu bytes of "
                    "partial results, the library keeps %zu a GPU (use fewer splits, or tff_attention_decode_fused "
                    "with a workspace of your own)",
                    splits, R, nq, d, need * sizeof(float), (size_t)TFF_ATTN_STATIC_FLOATS * sizeof(float));
        float* base = nullptr;
        if (int rc = attn_static_address(&base)) return rc;
        part_o = base;
        part_ml = base + rows * d;      // rows * d is a multiple of 16 floats: d is
    }
    if (int rc = tff_attention_decode_fused(qkv, qkv_stride, out, part_o, part_ml, k_cache, v_cache, block_tables,
                                            bt_stride, cu_tokens, start_pos, slot_mapping, q_weight, k_weight, eps,
                                            cos_sin, max_pos, pairing, splits, R, nq, nkv, d, page_size, num_pages,
                                            window, scale, stream))
        return rc;
    if (splits > 1 && R > 0)
        return tff_attention_split_reduce(part_o, part_ml, out, splits, R, nq, d, nullptr, 0, stream);
    return 0;
}
