// C entry points of the gfx950 kernel library.  Every function takes device
// pointers, checks its arguments on the host, launches on `stream` and returns
// 0, or a negative code after leaving a message for tff_last_error().
// Element type codes: 0 = float32, 1 = bfloat16.
//
// The export macro plays the part of the reference's DEEP_TFF_API
// (include/ExportInc.h:6-16).
#pragma once
#include <stdint.h>

#define TFF_API extern "C" __attribute__((visibility("default")))

typedef void* tff_stream_t;

TFF_API const char* tff_last_error();
TFF_API int tff_abi_version();

// out[t, :] = float(table[ids[t], :]).  table [V, H] of `dtype`, out float32.
TFF_API int tff_embed(const void* table, const int32_t* ids, float* out,
                      int T, int H, int V, int dtype, tff_stream_t stream);

// Fused residual sum and RMS norm over rows of width H:
//   v = resid[r] + (delta ? delta[r] : 0);  out[i] = v * rsqrt(mean(v^2)+eps) * w
// rows == null: r = i for i < n, and resid[r] = v is stored back.
// rows != null: r = rows[i]; resid is left as it is (norm of gathered rows).
// delta may come as delta_planes partial sums, delta_plane elements apart (what
// tff_gemm leaves with keep_partials); they are added up first, plane 0, 1, ...
TFF_API int tff_add_rmsnorm(float* resid, const float* delta, int delta_planes, size_t delta_plane,
                            const float* weight, float eps, void* out, const int32_t* rows, int n,
                            int H, int out_dtype, tff_stream_t stream);

// RMS norm of a plain [n, H] tensor of `dtype` with a float32 weight.
TFF_API int tff_rmsnorm(const void* x, const float* weight, float eps, void* out,
                        int n, int H, int dtype, tff_stream_t stream);

// C[M, N] = A[M, K] . W[N, K]^T.  A has row stride lda (elements), C is dense.
// A and W are of ab_dtype; C is of c_dtype.  float32 runs on plain FMA in a
// fixed summation order with a row-major W (w_packed = 0); bfloat16 runs on
// MFMA with float32 accumulation and takes W in fragment order (w_packed = 1,
// see tff_pack_weight).  glu_out > 0 (bfloat16 only): the 16-row groups of W
// alternate between a gate and an up projection, N = 2 * ceil16(glu_out), and
// C is [M, glu_out] = silu(gate) * up.
// workspace (may be null): device memory of tff_gemm_workspace_bytes() bytes the
// product may keep partial sums in; with less it takes a path that needs none.
// keep_partials (float32 result, no GLU): if the workspace is used, that is, if
// tff_gemm_workspace_bytes() > 0 (asked with the same keep_partials: the plan counts the
// cheaper hand-over) and the workspace has that size, the partial
// sums [bytes / (M * N * 4), M, N] are left there for the caller to add up
// (tff_add_rmsnorm takes them as they are) and C is not written.
TFF_API int tff_gemm(const void* A, const void* W, void* C, int M, int N, int K, int lda,
                     int ab_dtype, int c_dtype, int w_packed, int glu_out, void* workspace,
                     size_t workspace_bytes, int keep_partials, tff_stream_t stream);
TFF_API size_t tff_gemm_workspace_bytes(int M, int N, int K, int ab_dtype, int glu, int keep_partials);
// The bfloat16 product's plan for these sizes: rows and columns of a block tile (0: the
// streaming kernel for up to 16 rows) and the number of parts K is split into.
TFF_API int tff_gemm_plan(int M, int N, int K, int glu, int keep_partials, int* tile_rows, int* tile_cols,
                          int* splits);

// An RMS norm between two bfloat16 products of up to 16 rows, taken into them (its per-row
// factor commutes with the product after it):
//   tff_gemm_residual_prenorm: resid[M, N] += A . W^T in place (float32); x_out[M, N] = bfloat16
//     of the new resid times norm_w[N]; ss_out[m][g] = sum of squares of the new resid over
//     columns 16 g .. 16 g + 15 of row m (16 rows of ss_stride floats).  N a multiple of 8.
//   tff_gemm_row_scaled: C = rstd[m] * (A . W^T), rstd[m] = rsqrt(sum_{g < ss_count} ss[m][g] / dim
//     + eps), the sums added in a fixed order; glu_out as in tff_gemm.
TFF_API int tff_gemm_residual_prenorm(const void* A, const void* Wp, int M, int N, int K, int lda, float* resid,
                                      const float* norm_w, void* x_out, float* ss_out, int ss_stride,
                                      tff_stream_t stream);
TFF_API int tff_gemm_row_scaled(const void* A, const void* Wp, void* C, int M, int N, int K, int lda, int c_dtype,
                                int glu_out, const float* ss, int ss_stride, int ss_count, int dim, float eps,
                                tff_stream_t stream);

// bfloat16 row-major [N, K] (K a multiple of 8) -> fragment order: tiles of
// 16 rows x 32 k, each stored as the 1 KB operand of a 16x16x32 MFMA, element
// (n, k) at ((n/16) * ceil(K/32) + k/32) * 512 + (((k%32)/8) * 16 + n%16) * 8 + k%8,
// zero padded.  dst holds ceil(N/16) * ceil(K/32) * 512 elements.
TFF_API int tff_pack_weight(const void* src, void* dst, int N, int K, tff_stream_t stream);

// tff_embed for a table in fragment order.
TFF_API int tff_embed_packed(const void* table, const int32_t* ids, float* out, int T, int H,
                             int V, tff_stream_t stream);

// Per (token, head) of a fused projection output qkv [T, (nq + 2 nkv) d]:
// q and k heads get an RMS norm over d (q_weight / k_weight, skipped if null),
// then the rotation of pairs by cos_sin[pos, pair] (skipped if null); q is
// written back in place, k and v go to their page slot slot_mapping[t]
// (skipped if negative).  pairing 0: pairs (i, i + rot/2); 1: pairs (2i, 2i+1).
// Cache layout: keys [pages, nkv, page_size, d], values transposed [pages, nkv, d, page_size].
TFF_API int tff_qk_norm_rope_kv(void* qkv, int T, int nq, int nkv, int d,
                                const float* q_weight, const float* k_weight, float eps,
                                const float* cos_sin, int rot_dim, int pairing, int max_pos,
                                const int32_t* positions, const int32_t* slot_mapping,
                                void* k_cache, void* v_cache, int page_size, int num_pages,
                                int dtype, int cache_dtype, tff_stream_t stream);

// Attention of every token of a step over its request's cached keys.
// q: [T, q_stride] with nq heads of d at the start of each row; out [T, nq*d].
// token_req[t] names the row of block_tables; token t sees keys at positions
// max(0, pos-window+1) .. pos of that request (window 0: from 0).
// Works for every head size that is a multiple of 8 up to 512.
TFF_API int tff_attention_generic(const void* q, int q_stride, void* out,
                                  const void* k_cache, const void* v_cache,
                                  const int32_t* block_tables, int bt_stride,
                                  const int32_t* token_req, const int32_t* positions,
                                  int T, int nq, int nkv, int d, int page_size, int num_pages,
                                  int window, float scale, int dtype, int cache_dtype,
                                  tff_stream_t stream);

// bfloat16 attention on the matrix cores.  A wave works on `cols_per_wave` (16)
// columns of one request and kv head; a column is a (token, q head of
// the group) pair numbered token * G + head.  work != null: pairs (request,
// first column) per wave; work == null: every request brings one token and
// gets tiles_per_entry waves.  splits > 1 (entries of one token, 16 columns a
// wave) cuts each request's keys into runs whose partial results (part_o
// [splits, R, nq, d], part_ml [splits, R, nq, 2], float32, R = T_total the
// number of entries) tff_attention_split_reduce merges.  cols_per_wave 128: work items
// are runs of 128 columns for a block of eight waves that stages keys and
// values in LDS; block b works through items block_items[b] ..
// block_items[b + 1] of the work table (block_items null: item b); key_groups 2 (head sizes
// up to 128): a block is two groups of eight waves that take every other slice, 1: one group.
// cols_per_wave 256 (head sizes up to 128): the same with work items of 256 columns for blocks of eight waves of two
// column tiles each, one block a CU, half the LDS reads per flop: for long prompts.  Head sizes 16..128 in steps of
// 16, 192 and 256; pages of a power of two of tokens, at least 8; values transposed in their pages.
TFF_API int tff_attention_mfma_supported(int d, int page_size);
TFF_API int tff_attention_mfma(const void* q, int q_stride, void* out, float* part_o, float* part_ml,
                               const void* k_cache, const void* v_cache,
                               const int32_t* block_tables, int bt_stride, const int32_t* cu_tokens,
                               const int32_t* start_pos, const int32_t* work, int num_work,
                               const int32_t* block_items, int num_blocks,
                               int tiles_per_entry, int cols_per_wave, int key_groups, int splits, int T_total,
                               int nq, int nkv, int d, int page_size, int num_pages, int window,
                               float scale, tff_stream_t stream);
// Decoding steps (every entry brings one token), bfloat16, from the fused projection's output:
// row r of qkv ([R, (nq + 2 nkv) d], q heads first, then k, then v) is token r.  The kernel
// does what tff_qk_norm_rope_kv and tff_attention_mfma do one after the other, in one pass:
// per-head RMS norm of q and k (weights [d]; both null: none), rotation by the angles of the
// token's position start_pos[r] (cos_sin [max_pos, d/2, 2]; null: none; the whole head is
// rotated; pairing 0 needs d to be a multiple of 64), the token's key and value written to
// position start_pos[r] of the entry's pages where slot_mapping[r] >= 0 (negative, or
// slot_mapping null: the pages hold them already), attention over the pages.  With
// splits > 1 the partial results need tff_attention_split_reduce as there.  splits 0 (head sizes up to
// 128): a block of eight waves per entry and kv head splits the keys among its waves and merges in LDS;
// no workspace, no second call.  Worth it from some 256 pairs of entry and kv head on.
TFF_API int tff_attention_decode_fused(const void* qkv, int qkv_stride, void* out, float* part_o,
                                       float* part_ml, void* k_cache, void* v_cache,
                                       const int32_t* block_tables, int bt_stride,
                                       const int32_t* cu_tokens, const int32_t* start_pos,
                                       const int32_t* slot_mapping,
                                       const float* q_weight, const float* k_weight, float eps,
                                       const float* cos_sin, int max_pos, int pairing,
                                       int splits, int R, int nq, int nkv, int d, int page_size,
                                       int num_pages, int window, float scale, tff_stream_t stream);
// Merges partial results kept by entry (part_o [splits, R_total, nq, d]) into out rows:
// rows (may be null: entry i is token i for all R_total) holds (entry, token) pairs.
TFF_API int tff_attention_split_reduce(const float* part_o, const float* part_ml, void* out,
                                       int splits, int R_total, int nq, int d, const int32_t* rows,
                                       int num_rows, tff_stream_t stream);

// tff_attention_decode_fused with every entry's keys dealt into runs by the caller, who knows
// the entries' lengths, and the merge of the partial results, in one call.  key_runs
// [num_runs][4] = (entry, first key, end of keys, the entry's position = start_pos[entry]), 16-byte
// aligned: a wave per run, kv head and column tile; the runs of entry r are run_start[r] ..
// run_start[r + 1] - 1 (run_start [R + 1]) and follow each other in the order of the keys, without
// gap or overlap; a run's first key is the entry's first visible key rounded down to a multiple
// of 32, plus a multiple of 32; an entry number < 0: the run is not in use.
// Workspace: part_o [num_runs, nq, d], part_ml [num_runs, nq, 2] (float32).  Runs of similar
// length keep the waves busy alike however uneven the entries' lengths are.  block_waves 1: a wave
// per run and kv head; 8: a block of eight waves that split the run among them and merge in LDS
// (head sizes up to 128, up to 16 query heads a kv head), for runs dealt with that in mind.
// num_runs is a multiple of eight.  merge 0: the caller knows that every entry is one run, so no
// result is partial and the merging kernel is not launched (a wrong 0 leaves the entries of
// several runs without a result).
TFF_API int tff_attention_decode_runs(const void* qkv, int qkv_stride, void* out, float* part_o,
                                      float* part_ml, void* k_cache, void* v_cache,
                                      const int32_t* block_tables, int bt_stride,
                                      const int32_t* cu_tokens, const int32_t* start_pos,
                                      const int32_t* slot_mapping,
                                      const float* q_weight, const float* k_weight, float eps,
                                      const float* cos_sin, int max_pos, int pairing,
                                      const int32_t* key_runs, const int32_t* run_start, int num_runs,
                                      int block_waves, int merge, int R, int nq, int nkv, int d, int page_size,
                                      int num_pages, int window, float scale, tff_stream_t stream);

// The entries of one token among a step's entries (requests that decode beside prompt portions),
// with q finished and the tokens' keys and values in their pages (tff_qk_norm_rope_kv), and
// their keys dealt into runs as for tff_attention_decode_runs: key_runs [num_runs][4] = (the
// entry's row in the step's tables, first key, end of keys, the entry's position); the runs of
// the i-th such entry are run_start[i] .. run_start[i + 1] - 1 (run_start [num_entries + 1]) and
// tokens[i] is its token's row in q and out; other rows of out are not touched.  Workspace:
// part_o [num_runs, nq, d], part_ml [num_runs, nq, 2].  num_runs is a multiple of eight; merge 0:
// the caller knows that every such entry is one run.  T: rows of q.
TFF_API int tff_attention_mfma_runs(const void* q, int q_stride, void* out, float* part_o, float* part_ml,
                                    const void* k_cache, const void* v_cache,
                                    const int32_t* block_tables, int bt_stride,
                                    const int32_t* cu_tokens, const int32_t* start_pos,
                                    const int32_t* key_runs, const int32_t* run_start,
                                    const int32_t* tokens, int num_runs, int num_entries, int merge,
                                    int T, int nq, int nkv, int d, int page_size, int num_pages,
                                    int window, float scale, tff_stream_t stream);

// tff_attention_decode_fused followed by tff_attention_split_reduce, for callers that cannot
// allocate device memory: code under HIP graph capture, tight serving loops, harnesses that
// forbid hipMalloc.  It has no counterpart in the reference.  The partial results of split keys
// live in an array that is part of the library, TFF_ATTENTION_STATIC_SCRATCH_BYTES (16 MiB)
// on every GPU the library runs on, held until the process ends; the call allocates and frees
// nothing, on the device or through any library.  It refuses, with a message, sizes whose
// partial results (splits * R * nq * (d + 2) floats) do not fit.  All calls on one GPU share
// that GPU's array: calls that overlap there (two streams, two threads) race; calls on one
// stream, or otherwise ordered, do not.  The array keeps the last call's contents and nothing
// in it has to be cleared between calls.  The array's address on a device is looked up at the
// first call on that device (make it outside a graph capture).  Arguments as for
// tff_attention_decode_fused, without the workspace; out [R, nq * d] is final.
#define TFF_ATTENTION_STATIC_SCRATCH_BYTES (16u << 20)
TFF_API int tff_attention_decode_fused_static(const void* qkv, int qkv_stride, void* out, void* k_cache,
                                              void* v_cache, const int32_t* block_tables, int bt_stride,
                                              const int32_t* cu_tokens, const int32_t* start_pos,
                                              const int32_t* slot_mapping, const float* q_weight,
                                              const float* k_weight, float eps, const float* cos_sin,
                                              int max_pos, int pairing, int splits, int R, int nq, int nkv,
                                              int d, int page_size, int num_pages, int window, float scale,
                                              tff_stream_t stream);

// out[t, i] = silu(gu[t, i]) * gu[t, I + i]
TFF_API int tff_swiglu(const void* gu, void* out, int T, int I, int dtype, tff_stream_t stream);

// Element type conversion of n elements.
TFF_API int tff_cast(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t n,
                     tff_stream_t stream);

// out[r] = lowest index among the maxima of logits[r, :].
// workspace: tff_argmax_workspace_bytes(rows, V) bytes, 16-byte aligned (0: none needed), for the
// form that cuts a row into runs over several blocks; null selects one block a row.
TFF_API size_t tff_argmax_workspace_bytes(int rows, int V);
TFF_API int tff_argmax(const float* logits, int32_t* out, int rows, int V, void* workspace, tff_stream_t stream);

// logits[r, seen] is divided by penalty[r] if positive, multiplied otherwise,
// for the distinct token ids seen[cu_seen[r] .. cu_seen[r+1]).
TFF_API int tff_repetition_penalty(float* logits, int rows, int V, const int32_t* seen,
                                   const int32_t* cu_seen, const float* penalty,
                                   tff_stream_t stream);

// Draw from softmax(logits / temperature) restricted by top_k (0: off), top_p
// (1: off) and min_p (0: off), by inverse CDF in index order with the given
// uniform number per row.  temperature[r] <= 0 selects the argmax.  Probabilities
// are weighed in units of 2^-40 of the largest one (a token below that is never
// drawn); V up to 1,048,576.
TFF_API int tff_sample(const float* logits, int32_t* out, int rows, int V,
                       const float* temperature, const int32_t* top_k, const float* top_p,
                       const float* min_p, const float* uniform, float* probs_out,
                       tff_stream_t stream);

// Measuring kernels (csrc/probes.hip): stream `bytes` from src once; run blocks x 4 waves of
// iters x 16 back-to-back 16x16x32 bfloat16 MFMAs, on operands that never change or
// (varied_operands) that change from one instruction to the next.  The caller times them.
TFF_API int tff_probe_stream_read(const void* src, size_t bytes, void* sink, int blocks, tff_stream_t stream);
TFF_API int tff_probe_mfma(void* sink, int blocks, int iters, int varied_operands, tff_stream_t stream);
