// C entry points of the kernel library.  Every function takes the HIP stream
// to launch on, returns 0 on success and nonzero after leaving a message for
// pa_last_error().  `dtype` codes: 0 = float32, 1 = bfloat16.  All pointers
// are device pointers unless said otherwise; nothing here allocates.
#pragma once
#ifdef __cplusplus
extern "C" {
#endif

const char* pa_last_error();
int pa_device_arch(char* out, int cap);
int pa_num_compute_units();

// A kernel that only reads: `bytes` (a multiple of 16) from src by `blocks` workgroups; out holds a word per
// workgroup.  For measuring the rate at which this device streams memory.
int pa_stream_read(void* stream, const void* src, long bytes, void* out, int blocks);
// out[t, :] = table[ids[t], :]
int pa_embed_gather(void* stream, int dtype, const int* ids, const void* table, void* out, int tokens, int hidden,
                    int vocab);
// ids[dst[i]] = sampled[src[i]] for i < n with src[i] >= 0 (token ids handed from one step to the next on the device).
int pa_carry_tokens(void* stream, const int* sampled, const int* src, const int* dst, int* ids, int n, int sampled_rows,
                    int tokens);
// Clears row slots[i] of data [num_rows, row_bytes] for every sequence i < nseq with fresh[i] != 0 and slots[i] >= 0:
// per-request state of fixed size starts from zero, decided on the device (so a captured step can do it).
int pa_zero_fresh_rows(void* stream, void* data, long row_bytes, const int* slots, const int* fresh, int nseq,
                       int num_rows);
// RMSNorm of x (+ residual, which then receives the sum) with a 32-bit weight;
// with `rows`, output row r comes from input row rows[r] and the residual is left alone.
int pa_rmsnorm(void* stream, int dtype, const void* x, void* residual, const float* w, void* out, const int* rows,
               int nrows, int hidden, float eps);
// The same with x given as `slices` 32-bit partial sums [slices, rows, hidden], slice_stride elements apart (what
// pa_gemm_mid leaves of a product cut along its inner size): they are added in order as they are loaded.
int pa_rmsnorm_slices(void* stream, int dtype, const float* parts, int slices, long slice_stride, void* residual,
                      const float* w, void* out, const int* rows, int nrows, int hidden, float eps);
// out[t, c] = act(gate_up[t, 2c]) * gate_up[t, 2c + 1]   (columns alternate gate_j, up_j); act: 0 SiLU, 1 GELU in its
// tanh form.  The products' gated epilogues take the same choice as epilogue code 1 + act.
int pa_silu_mul(void* stream, int dtype, const void* gate_up, void* out, int tokens, int inter, int act);
int pa_gather_rows(void* stream, int dtype, const void* x, const int* rows, void* out, int nrows, int width);
int pa_add_bias(void* stream, int dtype, void* y, const float* b, int tokens, int width);
int pa_to_f32(void* stream, int dtype, const void* x, float* out, long total);

// qkv [tokens, (nh + 2 nkv) * hd] -> q_out [tokens, nh, hd] (normed, rotated) and, where slots[t] >= 0,
// K (normed, rotated) into a cache laid out [page, nkv, page_size, hd] and V into one laid out
// [page, nkv, hd, page_size]; slot = page * page_size + offset.
int pa_qknorm_rope_kv(void* stream, int dtype, const void* qkv, const float* q_weight, const float* k_weight,
                      const float* cos_table, const float* sin_table, const int* positions, const int* slots,
                      void* q_out, void* k_cache, void* v_cache, int tokens, int nh, int nkv, int hd, int rot,
                      int page_size, float eps);

// C[m, n] = X[m, k] W[n, k]^T, bfloat16 with 32-bit accumulation, by hipBLASLt called directly; `workspace` is
// device memory its kernels may use.  The first call with a shape makes and keeps that shape's plan in host memory.
int pa_gemm_library(void* stream, const void* x, const void* w, void* c, int m, int n, int k, long ldx, long ldc,
                    void* workspace, long workspace_bytes);
// C[m, n] = A[m, k] W[n, k]^T (+ bias[n]), true 32-bit arithmetic.
int pa_gemm_plain(void* stream, int in_dtype, int out_dtype, const void* a, const void* w, const float* bias, void* c,
                  int m, int n, int k, long lda, long ldw, long ldc);

// C[m, n] = X[m, k] W[n, k]^T for m <= 64 in bfloat16 (32-bit accumulation); out_dtype 0 = float32, 1 = bfloat16.
// epilogue 0: (+ bias[n]); 1: C[m, n/2] = silu(gate) * up for a weight whose rows alternate gate_j, up_j.
// tiled 1: w is the weight as pa_pack_tiles lays it out.
int pa_gemm_skinny_slices(int k, int slices);
int pa_gemm_skinny_sliced(void* stream, const void* x, const void* w, const float* bias, float* parts, int m, int n, int k,
                          long ldx, int slices, int waves);
int pa_gemm_skinny(void* stream, int out_dtype, int epilogue, const void* x, const void* w, const float* bias, void* c,
                   int m, int n, int k, long ldx, long ldc, int tiled);
// C[m, n] = X[m, k] W[n, k]^T for m <= 128 from the weight in tiles, X staged through LDS and W streamed by
// `waves` wavefronts a workgroup, 16 rows of W each (3, 4, 5, 6 or 8; 0: chosen from the weight's shape; the same
// bits at every number).  slices 1: as pa_gemm_skinny (epilogue 0 (+ bias) / 1 SiLU * up).
// slices > 1 (epilogue 0): the inner size is cut into that many slices, each left as 32-bit sums in
// parts [slices, m, n] (pa_gemm_mid_parts floats; the bias in the first) for the reader to add in order, and c is
// not written.  pa_gemm_mid_slices: the number of slices that suits an [n, k] weight.
int pa_gemm_mid_slices(int n, int k);
long pa_gemm_mid_parts(int m, int n, int slices);
int pa_gemm_mid(void* stream, int out_dtype, int epilogue, const void* x, const void* w, const float* bias, void* c,
                float* parts, int m, int n, int k, long ldx, long ldc, int slices, int waves);
// pa_gemm_mid's gated product of up to 16 rows with the residual add and RMSNorm in front of it, done as X is staged:
// res_out = x + res (another buffer than res), c = act(gate) * up of rmsnorm(x + res; gain, eps) W^T.
int pa_gemm_mid_normed(void* stream, int epilogue, const void* x, const void* res, const float* gain, float eps,
                       void* res_out, const void* w, void* c, int m, int n, int k, long ldx, long ldc, int waves);
// C = X W^T for any number of rows from the weight in tiles, the output tiled both ways (gemm_tall.hip): 16 mt rows
// of X by 64 nt rows of W a workgroup (mt, nt = 0, 0: the launcher's choice, what pa_gemm_tall_shape puts into
// out[0], out[1]).  epilogue 0: C (+ bias) in bfloat16; 1: C[m, n/2] = silu(gate) * up.  slices > 1 (epilogue 0): parts
// [slices, m, n] as pa_gemm_mid leaves them, c not written.
void pa_gemm_tall_shape(int m, int n, int k, int slices, int* out);
int pa_gemm_tall(void* stream, int epilogue, const void* x, const void* w, const float* bias, void* c, float* parts,
                 int m, int n, int k, long ldx, long ldc, int slices, int mt, int nt);
// out[i] = parts[0, i] + parts[1, i] + ..; out_dtype 0 = float32, 1 = bfloat16; total = rows * columns.
int pa_sum_slices(void* stream, int out_dtype, const float* parts, void* out, int slices, long total);
// out[tile][step][half][g][r][8] = w[16 tile + r][64 step + 16 g + 8 half ..], zero-padded: ceil(n/16) * ceil(k/64) * 1024 elements.
int pa_pack_tiles(void* stream, const void* w, void* out, int n, int k);

// Paged causal attention, one query token per (seq_of_token[t], positions[t]); window 0 = all keys.
// softcap (here and in the matrix-core entry points): 0 = none; > 0 bends every scaled score to
// softcap * tanh(score / softcap) before the softmax.
int pa_attn_generic(void* stream, int dtype, const void* q, const void* k_cache, const void* v_cache,
                    const int* block_table, int table_stride, const int* seq_of_token, const int* positions, void* out,
                    int tokens, int nh, int nkv, int hd, int page_size, int window, float scale, float softcap);

// Matrix-core attention in bfloat16 (K cache [page, nkv, page_size, hd], V cache [page, nkv, hd, page_size]).
// seq_ids lists the sequences of the step a call handles; cu_q[s] is the first packed token row of sequence s,
// context_lens[s] its tokens in the cache after the step.  Decode takes sequences that feed one token and cuts
// each one's keys into splits of split_keys; workspace must hold pa_attn_decode_workspace(...) floats.
// The two decode entry points take seq_ids = null for the sequences 0 .. nseq - 1 (a step of single tokens only).
int pa_attn_mfma_supports(int hd, int page_size);
long pa_attn_decode_workspace(int nseq, int nh, int hd, int max_splits);
int pa_attn_decode(void* stream, const void* q, const void* kc, const void* vc, const int* block_table,
                   int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out,
                   float* workspace, int nseq, int nh, int nkv, int hd, int page_size, int window, float scale,
                   float softcap, int split_keys, int max_splits);
// pa_qknorm_rope_kv + pa_attn_decode in one kernel for steps of single tokens: takes the merged projection,
// norms and rotates the queries in place of loading them, and writes each token's key and value first.
int pa_attn_decode_fused(void* stream, const void* qkv, const float* q_weight, const float* k_weight,
                         const float* cos_table, const float* sin_table, const int* slots, float eps,
                         void* kc, void* vc, const int* block_table, int table_stride, const int* seq_ids, const int* cu_q,
                         const int* context_lens, void* out, float* workspace, int nseq, int nh, int nkv, int hd,
                         int page_size, int window, float scale, float softcap, int split_keys, int max_splits);
int pa_attn_decode_fused_supports(int nh, int nkv, int hd, int rot, int page_size);
int pa_attn_prefill(void* stream, const void* q, const void* kc, const void* vc, const int* block_table,
                    int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out,
                    int nseq, int max_q_len, int min_prefix, int nh, int nkv, int hd, int page_size, int window,
                    float scale, float softcap);
// min_prefix: the fewest keys any sequence has before its portion (0 if unknown), a hint for the cut of the work.
// The same with the cut of the work given (for tests and measurements): tiles in pairs, heads a wavefront (1, 2, 4),
// head groups a workgroup (1, 2), keys staged in LDS; -1 leaves one to the launcher.
int pa_attn_prefill_cut(void* stream, const void* q, const void* kc, const void* vc, const int* block_table,
                        int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out,
                        int nseq, int max_q_len, int min_prefix, int nh, int nkv, int hd, int page_size, int window,
                        float scale, float softcap, int paired, int heads, int groups, int staged);

// out[r] = index of the largest of logits[r, :], the lowest index among equals.
// scratch: pa_argmax_scratch(rows, vocab) floats (none for narrow rows).
int pa_argmax_scratch(int rows, int vocab);
int pa_argmax(void* stream, const float* logits, int* out, float* scratch, int rows, int vocab);
// pa_argmax without a scratch argument and without any allocation, for callers that cannot allocate (code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
// reference.  The candidates of wide rows go to an array inside the library, pa_argmax_static_capacity() floats
// (65,536 = 256 KB) on every GPU the library runs on, held until the process ends; rows * ceil(vocab / 2048) * 2
// must fit it (64 rows of 151,936 entries take 9,600), else the call is refused.  The first call on a GPU looks
// up where that GPU's copy lies (make it before a capture begins).  Nothing in the array has to be cleared between
// calls: what the second launch reads the first has written.  All calls on a GPU share the one array: calls
// that overlap there (two streams, two threads) race, calls in order on one stream do not.
int pa_argmax_static_capacity();
int pa_argmax_static(void* stream, const float* logits, int* out, int rows, int vocab);

// Per row: temperature < 1e-7 -> argmax; else a draw from softmax(logits / T) kept to the top_k largest
// (0 = all) and to the shortest descending prefix of mass top_p (>= 1 = all), at the uniform number uniform[r] in [0, 1).
int pa_sample(void* stream, const float* logits, const float* temperature, const int* top_k, const float* top_p,
              const float* uniform, int* out, int rows, int vocab);
// The same choice for long rows with every pass spread over the chip; modes: bit 0 some row may have a top-k,
// bit 1 some row may have a top-p.  workspace: pa_sample_wide_workspace(rows, vocab) bytes, 16-byte aligned.
long pa_sample_wide_workspace(int rows, int vocab);
// lp[r] = logits[r, ids[r]] - logsumexp(logits[r]) (0 where ids[r] < 0); for k > 0 also the entries among the row's
// k largest with their log-probabilities, ties at the k-th value included, unsorted, at most cap a row:
// top_v / top_i [rows, cap], count [rows].
int pa_logprobs(void* stream, const float* logits, const int* ids, float* lp, float* top_v, int* top_i, int* count,
                int rows, int vocab, int k, int cap);
int pa_sample_wide(void* stream, const float* logits, const float* temperature, const int* top_k, const float* top_p,
                   const float* uniform, int* out, void* workspace, int rows, int vocab, int modes);

#ifdef __cplusplus
}
#endif
