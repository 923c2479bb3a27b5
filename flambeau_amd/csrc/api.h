// C interface of the kernel library.  Every function returns 0 on success, a negative
// value when it refuses its arguments or a launch fails; fl_last_error() then gives
// the reason.  Pointers are device pointers unless a name says otherwise; `stream` is a
// hipStream_t.  dtype codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* fl_last_error(void);
int fl_abi_version(void);
int fl_compute_units(void);        // compute units of the current device: what the kernels' plans count blocks against

// ---- plain kernels (plain.hip) ----
int fl_embed(const void* table, int dtype, const int* tokens, float* out, int n, int H, int V,
             hipStream_t stream);
int fl_rmsnorm(const float* x, const float* delta, float* resid_out, const int* rows,
               const float* w, void* out, int out_dtype, int n_rows, int H, float eps,
               hipStream_t stream);
int fl_add_inplace(float* x, const float* delta, long n, hipStream_t stream);
int fl_gemm_plain(const void* x, const void* w, void* out, int in_dtype, int out_dtype, int M,
                  int N, int K, hipStream_t stream);
int fl_rope_kv_write(const void* qkv, int in_dtype, int ld, const int* positions,
                     const int* tok_seq, const int* block_table, int max_blocks, void* q_out,
                     void* cache_base, int dtype, int n, int nh, int nkv, int hd, int page_size,
                     int n_pages, int rot, float theta, int write_cache, const float* cs, int paired,
                     int n_parts, long part_stride, hipStream_t stream);
// cs[n][rot / 2][2]: cosine and sine of every (token, rotation pair) of a step
int fl_rope_table(const int* positions, int n, int rot, float theta, float* cs, hipStream_t stream);
// the same from frequencies of the caller's own: cs = magnitude * (cos, sin)(position * inv_freq[i]), inv_freq[rot / 2] double
int fl_rope_table_ladder(const int* positions, int n, int rot, const double* inv_freq, float magnitude,
                         float* cs, hipStream_t stream);
int fl_attn_plain(const void* q, void* out, const void* cache_base, int dtype,
                  const int* positions, const int* tok_seq, const int* block_table,
                  int max_blocks, int n, int nh, int nkv, int hd, int page_size, int n_pages,
                  float scale, int window, hipStream_t stream);
int fl_attn_max_head_dim(void);             // the largest head size the attention kernels take
int fl_silu_mul(const void* gu, int in_dtype, void* out, int out_dtype, int n, int I,
                hipStream_t stream);
int fl_feed_tokens(int* tokens, const int* ids, const int* src, int n, hipStream_t stream);
int fl_argmax(const float* logits, int* out, int rows, int V, hipStream_t stream);
int fl_sample(const float* logits, const float* inv_temp, const float* uniform, int* out,
              int rows, int V, hipStream_t stream);
// The same draw through top-k, top-p and min-p for the rows that ask for them (top_k[r] >= 1 as a float,
// 0 < top_p[r] < 1, min_p[r] > 0); other rows are left to fl_sample.  At most fl_sample_filtered_max_k()
// candidates are kept.  stash: rows * V values of scratch for vocabularies beyond 32,768, or null.
int fl_sample_filtered(const float* logits, const float* inv_temp, const float* uniform, const float* top_k,
                       const float* top_p, const float* min_p, int* out, int rows, int V, unsigned* stash,
                       hipStream_t stream);
int fl_sample_filtered_max_k(void);
int fl_sample_filtered_max_vocab(void);      // the largest vocabulary fl_sample_filtered takes
// Penalties over the tokens a request has generated (counts[slot][V], 16-bit, one row per state slot) and
// logit bias, in place on the step's logits before the draw; slot[r] < 0 (as a float): the row has none.
int fl_sample_penalise(float* logits, int rows, int V, const unsigned short* counts, const float* slot,
                       const float* repetition, const float* presence, const float* frequency, hipStream_t stream);
int fl_sample_bias(float* logits, int V, int n, const float* row, const float* token, const float* value,
                   hipStream_t stream);
int fl_sample_count(unsigned short* counts, int V, int rows, const float* slot, const int* ids, hipStream_t stream);
int fl_sample_history(unsigned short* counts, int V, int slot, const int* tokens, int n, hipStream_t stream);

// ---- tuned bf16 kernels ----
// nw_hint: waves per block that split K (0: chosen from the sizes)
// epilogue: 0 = plain product; 1 = SwiGLU over interleaved gate/up rows, out_cols <= N / 2
int fl_gemm_skinny(const void* x, const void* w_packed, void* out, int out_dtype, int M, int N, int K,
                   int nw_hint, int epilogue, int out_cols, hipStream_t stream);

// The same product fused with the norms around it (at most 16 rows).  in_ssq (or null): [M, in_parts]
// partial sums of squares; every row of the result is multiplied by rsqrt(sum / K + eps).
// epilogue 2: resid[M, N] += the product, xg[M, N] = bf16(resid * g), out_ssq[M, ceil(N / 16)] = the
// blocks' sums of resid^2; nothing is stored in out.
int fl_gemm_skinny_fused(const void* x, const void* w_packed, void* out, int out_dtype, int M, int N, int K,
                         int epilogue, int out_cols, const float* in_ssq, int in_parts, float eps,
                         float* resid, const float* g, void* xg, float* out_ssq, hipStream_t stream);
int fl_gemm_skinny_scale_parts(int N, int K, int in_parts);

// 17 to 64 rows, K a multiple of 32; a shape with fl_gemm_mid_splits > 1 needs a float workspace
// of splits * M * N values
int fl_gemm_mid(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                int M, int N, int K, int epilogue, int out_cols, hipStream_t stream);
int fl_gemm_mid_splits(int M, int N, int K);
// for tests and measurements: waves per block (0, 4, 8) and K-splits (0 = chosen) from the caller
int fl_gemm_mid_ex(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                   int M, int N, int K, int epilogue, int out_cols, const float* in_ssq, int in_parts,
                   float eps, int waves, int forced_splits, hipStream_t stream);
int fl_gemm_mid_splits_ex(int M, int N, int K, int waves, int forced);
// The same fused with the norms around it, as fl_gemm_skinny_fused: a row scale from partial sums of
// squares, and the product added to the residual stream with the next norm left in factors
// (out_ssq[M, fl_gemm_mid_parts(N)]; the workspace holds splits * M * N floats, also for one split).
int fl_gemm_mid_scaled(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                       int M, int N, int K, int epilogue, int out_cols, const float* in_ssq, int in_parts,
                       float eps, hipStream_t stream);
int fl_gemm_mid_residual(const void* x, const void* w_packed, float* workspace, int M, int N, int K,
                         float* resid, const float* g, void* xg, float* out_ssq, hipStream_t stream);
int fl_gemm_mid_partials(const void* x, const void* w_packed, float* workspace, int M, int N, int K,
                         const float* in_ssq, int in_parts, float eps, hipStream_t stream);
int fl_gemm_mid_parts(int N);
// The adding half of fl_gemm_mid_residual for any number of rows: part[splits][M][N] -> resid, xg, out_ssq.
int fl_reduce_residual(const float* part, float* resid, const float* g, void* xg, float* out_ssq, int M, int N,
                       int splits, hipStream_t stream);

int fl_gemm_tiled(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                  int M, int N, int K, int epilogue, int out_cols, hipStream_t stream);
int fl_gemm_tiled_splits(int M, int N, int K);
// for tests and measurements: block shape (0 = chosen, 3 = 256 features x 128 tokens, 7 = 192 x 128,
// 8 = 128 x 128; with eight waves 10 = 256 x 256, 6 = 128 x 256) and K-splits (0 = chosen) from the caller
int fl_gemm_tiled_ex(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                     int M, int N, int K, int epilogue, int out_cols, const float* in_ssq, int in_parts,
                     float eps, int variant, int forced_splits, hipStream_t stream);
int fl_gemm_tiled_splits_ex(int M, int N, int K, int forced);
int fl_gemm_tiled_shape(int M, int N, int K, int may_split);
int fl_gemm_tiled_residual_ex(const void* x, const void* w_packed, float* workspace, int M, int N, int K, float* resid,
                              const float* g, void* xg, float* out_ssq, int variant, hipStream_t stream);
int fl_gemm_tiled_parts_ex(int M, int N, int K, int variant);
int fl_gemm_tiled_rope_ex(const void* x, const void* w_packed, int M, int N, int K, const float* in_ssq,
                          int in_parts, float eps, const int* positions, const int* tok_seq,
                          const int* block_table, int max_blocks, const float* cs, void* q_out, void* cache_base,
                          int nh, int nkv, int hd, int page_size, int n_pages, int rot, int write_cache, int variant,
                          hipStream_t stream);
// The joined q/k/v projection (rows of w in paired order) with rotation and the stores of q and the
// cache rows in the product's kernel: at most 16 rows, and many rows (shapes whose K is not split).
int fl_gemm_skinny_rope(const void* x, const void* w_packed, int M, int N, int K, const float* in_ssq,
                        int in_parts, float eps, const int* positions, const int* tok_seq,
                        const int* block_table, int max_blocks, const float* cs, void* q_out,
                        void* cache_base, int nh, int nkv, int hd, int page_size, int n_pages, int rot,
                        int write_cache, hipStream_t stream);
int fl_gemm_tiled_rope(const void* x, const void* w_packed, int M, int N, int K, const float* in_ssq,
                       int in_parts, float eps, const int* positions, const int* tok_seq,
                       const int* block_table, int max_blocks, const float* cs, void* q_out, void* cache_base,
                       int nh, int nkv, int hd, int page_size, int n_pages, int rot, int write_cache,
                       hipStream_t stream);
// The tiled product fused with the norms around it, as fl_gemm_skinny_fused.  The residual form leaves
// out_ssq[M, fl_gemm_tiled_residual_parts(M, N, K)] and needs a workspace of splits * M * N floats where K is split.
int fl_gemm_tiled_scaled(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                         int M, int N, int K, int epilogue, int out_cols, const float* in_ssq, int in_parts,
                         float eps, hipStream_t stream);
int fl_gemm_tiled_residual(const void* x, const void* w_packed, float* workspace, int M, int N, int K, float* resid,
                           const float* g, void* xg, float* out_ssq, hipStream_t stream);
int fl_gemm_tiled_parts(int M, int N, int K);
// The K-splits left apart in workspace[fl_gemm_tiled_splits(M, N, K)][M][N], each scaled by in_ssq's row scale.
int fl_gemm_tiled_partials(const void* x, const void* w_packed, float* workspace, int M, int N, int K,
                           const float* in_ssq, int in_parts, float eps, hipStream_t stream);
int fl_gemm_tiled_residual_parts(int M, int N, int K);
int fl_attn_decode(const void* q, void* out, float* part_o, float* part_ml, const void* cache_base,
                   const int* items, int n_items, const int* block_table, int max_blocks, int nh, int nkv, int hd, int page_size,
                   int n_pages, float scale, int window, int n_split, hipStream_t stream);
// fl_attn_decode with splits per row: items[i] = (row, position, request, split + 256 * splits), a row's
// splits one after the other from split 0 on (up to 255 of them; 1: no split), row < 0: unused place.
// part_o: n_items * nh * (hd rounded up to 32) floats, part_ml: n_items * nh * 2.  firsts[r] = (row,
// index of the row's first item, its splits, 0), n_rows of them; null: every row has one split,
// nothing is merged (and no workspace needed).
int fl_attn_decode_items(const void* q, void* out, float* part_o, float* part_ml, const void* cache_base,
                         const int* items, int n_items, const int* block_table, int max_blocks, int nh, int nkv,
                         int hd, int page_size, int n_pages, float scale, int window, const int* firsts, int n_rows,
                         hipStream_t stream);
// fl_attn_decode for callers that cannot allocate device memory (code under graph capture, tight
// serving loops, harnesses that forbid it).  It has no counterpart in the reference.  The splits'
// partial results, which fl_attn_decode takes as part_o / part_ml, go to an array of
// FL_ATTN_DECODE_STATIC_FLOATS floats (8 MiB) that is part of the library's image on every GPU it
// runs on; the call allocates and frees nothing.  It refuses n_items * nh * n_split * (hd rounded
// up to 32, + 2) floats beyond that size.  Every call on a GPU uses that GPU's one array: calls
// that overlap on one GPU (two streams, two threads) race; calls on one stream do not.  Nothing in
// the array has to start at zero: every slot a call reads was written by the same call before.
#define FL_ATTN_DECODE_STATIC_FLOATS (2u << 20)
int fl_attn_decode_static(const void* q, void* out, const void* cache_base, const int* items, int n_items,
                          const int* block_table, int max_blocks, int nh, int nkv, int hd, int page_size,
                          int n_pages, float scale, int window, int n_split, hipStream_t stream);
long fl_attn_decode_static_capacity(void);
int fl_attn_prefill(const void* q, void* out, const void* cache_base, const int* tiles, int n_tiles,
                    const int* positions, const int* block_table, int max_blocks, int nh, int nkv, int hd,
                    int page_size, int n_pages, float scale, int window, int qt_hint, float* part_o, float* part_ml,
                    int n_split, hipStream_t stream);
// Block-table entries of a request that a block of fl_attn_prefill can keep at a head size, and whether
// it takes a cache shape with tables max_blocks wide (with a window only the window's pages count).
int fl_attn_prefill_max_pages(int hd);
int fl_attn_prefill_takes(int hd, int page_size, int max_blocks, int window);
int fl_attn_prefill_splits(int n_tiles, int nh, int nkv, int hd, int max_keys);
int fl_attn_prefill_heads(int n_tiles, int nh, int nkv, int hd, int max_keys);      // query heads per wave: the qt_hint to pass
int fl_attn_prefill_workspace(int n_rows, int nh, int hd, int n_split, long* o_floats, long* ml_floats);
int fl_attn_decode_workspace(int n_items, int nh, int hd, int n_split, long* o_floats, long* ml_floats);

// ---- step programs (program.hip): launches recorded once, replayed with one call ----
typedef union FlArg { void* p; long l; int i; float f; } FlArg;
void* fl_program_new(void);
void fl_program_free(void* program);
int fl_program_size(const void* program);
// name: a launch function the recorder knows (every function above that takes a stream); args: its
// arguments in order, the stream's value is ignored
int fl_program_append(void* program, const char* name, const FlArg* args, int n_args);
int fl_program_run(const void* program, hipStream_t stream, int* failed_at);
// What the recorder knows: launch functions register themselves (FL_RECORDABLE in recordable.h puts a
// registrar beside a definition); a launch function of another library is added with
// fl_program_register, `call` being a function that unpacks the recorded arguments and calls it with
// the stream given.  fl_program_knows: the number of arguments (stream included) or -1.
typedef int (*FlTrampoline)(const FlArg* args, hipStream_t stream);
int fl_program_register(const char* name, FlTrampoline call, int n_args);
int fl_program_knows(const char* name);

#ifdef __cplusplus
}
#endif
