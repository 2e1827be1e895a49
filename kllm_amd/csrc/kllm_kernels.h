/* C ABI of the gfx950 kernel library.
 *
 * Every function takes device pointers and the HIP stream to launch on, checks
 * on the host that the sizes fit what its kernel and grid assume, and returns
 * 0, a positive HIP error code, or a negative KLLM_ERR_* value; the text of the
 * calling thread's last error is read with kllm_last_error.  The role is the
 * one backend/shim.h plays in the reference (error codes :19-27), but the
 * boundary lies lower: the host keeps the model, the cache tables and the
 * batch, and calls one kernel at a time.
 *
 * dtype arguments: 0 = float32, 1 = bfloat16.
 */
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KLLM_ERR_STATE (-1)
#define KLLM_ERR_ARG (-2)

#define KLLM_GEMM_PLAIN 0
#define KLLM_GEMM_TILED_F32 1
#define KLLM_GEMM_MFMA_BF16 2
#define KLLM_GEMM_SKINNY_BF16 3
#define KLLM_GEMM_GEMV 4
#define KLLM_GEMM_GEMV_LDS 5 /* kllm_gemv_plain, reached through the Python wrapper */
#define KLLM_GEMM_MFMA_F32 6 /* MFMA 32x32x2 with 32-bit operands: no reduced precision */

/* Copies the calling thread's last error text; returns its length. */
int kllm_last_error(char* buf, int len);
/* One line about the device: name, architecture, compute units, memory. */
int kllm_device_info(int device, char* buf, int len);
/* ABI version, bumped when a signature changes. */
int kllm_abi_version(void);
/* Compute units and XCDs of the current device (the launch heuristics scale with them). */
int kllm_device_cus(void);
int kllm_device_xcds(void);

/* What the box reaches with nothing in the way, for quoting measured figures against: a
 * plain copy of `bytes` (a multiple of 16) and a loop of `iters` rounds of four independent
 * MFMAs per wave on every CU (bfloat16 32x32x16 or float32 32x32x2); *flops receives the
 * floating-point operations of the launch.  The caller times them. */
int kllm_calibrate_copy(void* dst, const void* src, long bytes, hipStream_t stream);
/* A read-only stream over `bytes`: sink receives one float per workgroup
 * (kllm_calibrate_read_workgroups() of them). */
int kllm_calibrate_read(const void* src, long bytes, float* sink, hipStream_t stream);
int kllm_calibrate_read_workgroups(void);
int kllm_calibrate_mfma(int dtype, int iters, float* sink, double* flops, hipStream_t stream);

/* out[t] = scale * table[ids[t]]; with `from` (and `sampled`), token t whose from[t] >= 0 takes its id
 * from sampled[from[t]], a token id that an earlier launch left on the device.  `copy` (or null):
 * the same rows in the table's own type. */
int kllm_embed(float* out, const void* table, const int* ids, const int* from, const int* sampled,
               int n, int d, int vocab, int dtype, float scale, void* copy, hipStream_t stream);

/* v = x[src] + sum of the nsplit partial deltas (delta may be null);
 * x[src] = v when write_x; out[r] = rmsnorm(v) * w when out is not null.
 * src = rows[r] when rows is given (then write_x must be 0), else r. */
int kllm_add_rmsnorm(float* x, const void* delta, int delta_dtype, int nsplit, long split_stride,
                     const float* w, void* out, int out_dtype, const int* rows, int n, int d,
                     float eps, int write_x, hipStream_t stream);

/* cos and sin [n][head_dim/2] of positions[t] * theta^(-2j/head_dim), angle in double. */
int kllm_rope_tables(float* cos_t, float* sin_t, const int* positions, int n, int head_dim,
                     double theta, hipStream_t stream);

/* qkv: [nsplit][n][H*hd + 2*KV*hd] (only [n][H*hd] when cache is null).
 * Rotates q and k when cos/sin ([n][rot/2]) are given, writes q_out [n][H*hd]
 * and puts k, v into the pages of `cache` ([pages][2][KV][page_size*hd]; keys
 * [slot][hd], values [hd][slot]).  The first `rot` elements of a head are
 * rotated (rot even, at most hd; the rest pass through), in pairs (j, j + rot/2)
 * or, `interleaved`, (2j, 2j + 1). */
int kllm_rope_append(const void* qkv, int in_dtype, int nsplit, long split_stride, void* q_out,
                     const float* cos_t, const float* sin_t, void* cache, const int* positions,
                     const int* span_of_token, const int* block_table, int max_pages,
                     int page_size, int n, int H, int KV, int hd, int rot, int interleaved, int dtype,
                     hipStream_t stream);

/* The gate's activation of a gated feed-forward (`act` below). */
#define KLLM_ACT_SILU 0
#define KLLM_ACT_GELU_TANH 1

/* out[n][f] = act(gu[:, :f]) * gu[:, f:], gu = [nsplit][n][2f]. */
int kllm_silu_mul(const void* gu, int in_dtype, int nsplit, long split_stride, void* out,
                  int out_dtype, int n, int f, int act, hipStream_t stream);

/* out[count] = sum over s of in[s][count], rounded to out_dtype. */
int kllm_sum_splits(const float* in, int nsplit, long count, void* out, int out_dtype,
                    hipStream_t stream);

/* Columns of the tiles that a decode batch of n rows (at most 64) gets against w[m][k] on the
 * MFMA kernel: a caller that cuts K into slices counts its workgroups with it. */
int kllm_gemm_decode_tile_cols(int n, int m, int k);
/* y[nsplit][n][m] = x[n][k] . w[m][k]^T, 32-bit accumulation. */
int kllm_gemm(const void* x, const void* w, void* y, int n, int m, int k, int dtype, int out_dtype,
              int algo, int nsplit, hipStream_t stream);

/* h[n][f] = act(x . w[0:f]^T) * (x . w[f:2f]^T) on the MFMA tiles, h in dtype. */
int kllm_gemm_swiglu(const void* x, const void* w_gate_up, void* h, int n, int f, int k, int dtype,
                     int act, hipStream_t stream);

/* h[n][m] = act(x . w^T) on the MFMA tiles, h in dtype; act is one of the activations without
 * a gate (see kllm_unary_act), act_params its learned constants where it has them. */
int kllm_gemm_act(const void* x, const void* w, void* h, int n, int m, int k, int dtype, int act,
                  const float* act_params, hipStream_t stream);

/* Products for up to 8 rows of x with the whole of K in one wave (no partial
 * sums) and the next elementwise step in the epilogue.  m even, K a multiple
 * of 8 (bfloat16) or 4 (float32).
 *   plain:       y[n][m] float32 = x . w^T
 *   swiglu:      h[n][f] = act(x . w[0:f]^T) * (x . w[f:2f]^T), h in dtype
 *   rope_append: w = [q; k; v] rows (only q when cache is null); rotates q and k
 *                with cos/sin [n][hd/2] (if given), writes q_out [n][H*hd] and
 *                puts k, v into the pages of `cache`
 * With `normed` (may be null) x is not read (it may be null): the kernel stages
 * normed->x * rsqrt(sum of normed->ss[row][:] / k + eps) * normed->weight, rounded to dtype,
 * the RMS norm of the residual stream that a resid product (kllm_gemv_resid) has just
 * updated, without a launch of its own; built for up to 4 rows. */
typedef struct {
  const float* x;      /* the residual stream [n][k], float32 */
  const float* weight; /* the norm's weight [k] */
  const float* ss;     /* [n][parts rounded up to 4] partial sums of squares of x's rows */
  int parts;           /* at most 512 */
  float eps;
} KllmNormedInput;     /* all three 16-byte aligned */
int kllm_gemv_plain(const void* x, const void* w, float* y, int n, int m, int k, int dtype,
                    const KllmNormedInput* normed, hipStream_t stream);
int kllm_gemv_swiglu(const void* x, const void* w_gate_up, void* h, int n, int f, int k, int dtype,
                     int act, const KllmNormedInput* normed, hipStream_t stream);
/* resid [n][m] float32 += x . w^T in place; ss_out [n][P rounded up to 4] = the
 * workgroups' partial sums of squares of resid's new rows, P = kllm_gemv_resid_parts(m). */
int kllm_gemv_resid(const void* x, const void* w, float* resid, float* ss_out, int n, int m, int k,
                    int dtype, hipStream_t stream);
int kllm_gemv_resid_parts(int m);
/* Limits of the kernels above: rows of x, rows when `normed` is given, normed->parts. */
int kllm_gemv_max_rows(void);
int kllm_gemv_normed_max_rows(void);
int kllm_gemv_normed_max_parts(void);
int kllm_gemv_rope_append(const void* x, const void* w_qkv, void* q_out, const float* cos_t,
                          const float* sin_t, void* cache, const int* positions,
                          const int* span_of_token, const int* block_table, int max_pages,
                          int page_size, int n, int H, int KV, int hd, int k, int dtype,
                          const KllmNormedInput* normed, hipStream_t stream);

/* Products of a decode batch (bfloat16, up to KLLM_FUSED_LINEAR_MAX_ROWS rows)
 * on the matrix cores, fused with the step after them.  x is [n][k] with a row
 * stride of x_stride elements (0 = k), w is [m][k].  Output:
 *   PARTS   y float32 [nsplit][n][m]; only this one may split K
 *   RESID   resid float32 [n][m] += x . w^T in place; y bfloat16 [n][m] = the new rows times
 *           norm_w [m] (the weight of the RMS norm behind the addition); ss_out
 *           [n][P rounded up to 4] = the workgroups' sums of squares of the new rows,
 *           P = kllm_fused_linear_resid_parts(m, tiles_per_wg), at most
 *           kllm_fused_linear_max_parts()
 *   SWIGLU  y bfloat16 [n][m/2] = act(x . w[0:m/2]^T) * (x . w[m/2:m]^T)
 *   ROPE    w = [q; k; v] rows (only q when cache is null): q and k rotated with
 *           cos/sin [n][hd/2] (if given); y = q_out [n][H*hd], k and v go to the
 *           tokens' pages of `cache`
 * With ss_in (SWIGLU and ROPE only) x is such a y and the sums are multiplied by the row's
 * rsqrt(sum of ss_in[row][0:ss_parts] / k + eps) before the epilogue: the RMS norm of the
 * stream, rounded to bfloat16 before the row scale instead of after it.
 * All of a workgroup's slice of K for all rows is staged in LDS:
 * kllm_fused_linear_lds_bytes says how much that needs; beyond 160 KiB see
 * kllm_fused_linear_passes. */
#define KLLM_FUSED_LINEAR_MAX_ROWS 32
#define KLLM_LINEAR_OUT_PARTS 0
#define KLLM_LINEAR_OUT_RESID 1
#define KLLM_LINEAR_OUT_SWIGLU 2
#define KLLM_LINEAR_OUT_ROPE 3
typedef struct {
  void* y;
  const float* cos_t;
  const float* sin_t;
  void* cache;
  const int* positions;
  const int* span_of_token;
  const int* block_table;
  int kind;
  int nsplit;
  int max_pages, page_size, H, KV, hd;
  int act;
  float* resid;         /* RESID */
  const float* norm_w;  /* RESID */
  float* ss_out;        /* RESID */
  const float* ss_in;   /* row scale of the sums, or null; 16-byte aligned */
  int ss_parts;
  float eps;
  int tiled;            /* w is the copy that kllm_fused_linear_tile made of the weights for this kind */
} KllmLinearOut;
long kllm_fused_linear_lds_bytes(int n, int k, int nsplit);
/* Where that is more than LDS holds, the rows are staged and multiplied in passes over K, with
 * one tile to a workgroup (tiles_per_wg = 1): how many passes a call needs (1: all at once; 0:
 * the kernel does not take the sizes). */
int kllm_fused_linear_passes(int n, int k, int nsplit);
/* A copy of w[m][k] in the order the kernel's lanes read it (a load instruction then reads one
 * contiguous kilobyte instead of 64 bytes of each of 16 rows: weights stream 20-30 % faster),
 * for one output kind (PARTS and RESID share theirs; ROPE with the heads it will be called
 * with, with_kv: whether k and v rows follow q's): wt holds
 * kllm_fused_linear_tiled_elements(kind, m, k) elements.  Pass it as w with out->tiled = 1. */
long kllm_fused_linear_tiled_elements(int kind, int m, int k);
int kllm_fused_linear_tile(const void* w, void* wt, int kind, int m, int k, int H, int KV, int hd, int with_kv,
                           hipStream_t stream);
int kllm_fused_linear_resid_parts(int m, int tiles_per_wg);
int kllm_fused_linear_max_parts(void);
int kllm_fused_linear(const void* x, int x_stride, const KllmLinearOut* out, const void* w, int n, int m,
                      int k, int tiles_per_wg, hipStream_t stream);

/* Causal attention of n tokens over the paged cache; any head size up to 256.
 * `slopes` (here and in the other attention entry points; null: none) holds one number per
 * head: slopes[h] * (query position - key position) is taken off the scaled score, a bias
 * that grows with the distance to the key.
 * `vd`: width of a value (a page holds keys [KV][slot][hd], then values [KV][vd][slot]);
 * `chunk` > 0: the query at position p reads no key before p - p % chunk; `sink` != 0: the
 * softmax's denominator has one more term, exp(0); `keep_first` > 0: the first keep_first
 * positions of a request stay readable behind the window (their pages are kept). */
int kllm_attn_generic(const void* q, void* out, const void* cache, const int* positions,
                      const int* span_of_token, const int* block_table, int max_pages,
                      int page_size, int n, int H, int KV, int hd, int vd, int window, int chunk,
                      int sink, float scale, const float* slopes, int dtype, int keep_first, hipStream_t stream);

/* Decode attention on the matrix cores: every token's keys are cut into
 * `nslices` slices (1..256) that run side by side (bfloat16: a workgroup of 4
 * or 8 waves to a slice; head sizes 16..128 in steps of 16, 192,
 * 256, pages a multiple of 16; float32: one wave to a slice, 32-bit MFMA, head
 * sizes in steps of 8, pages a multiple of 4); `part` is float32 scratch of
 * n*H*nslices*(hd+2) elements (bfloat16 with one slice writes the output at once
 * and leaves it untouched).  kllm_attn_decode_slices proposes nslices for a batch
 * whose longest request has at most max_keys keys (0: unknown, as for contexts
 * of 2,048).  With token_list only the n_listed tokens it names are computed (q,
 * out and part stay indexed by token row). */
int kllm_attn_decode_slices(int n, int KV, int H, int hd, int dtype, int max_keys);
/* Whether the float32 attention on the matrix cores takes this head size and page size. */
int kllm_attn_f32_fits(int hd, int page_size);
/* `chunk`, `sink` and `keep_first` in kllm_attn_decode and kllm_attn_prefill: as in kllm_attn_generic
 * (kept first positions: bfloat16 only). */
int kllm_attn_decode(const void* q, void* out, float* part, long part_floats, const void* cache,
                     const int* positions, const int* span_of_token, const int* block_table,
                     int max_pages, int page_size, int n, int H, int KV, int hd, int window,
                     int chunk, int sink, int keep_first, float scale, const float* slopes, int nslices, int dtype,
                     const int* token_list, int n_listed, hipStream_t stream);

/* kllm_attn_decode without a workspace argument and without any allocation: for callers
 * that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The partial
 * results go to an array that the library holds on every GPU it runs on
 * (KLLM_ATTN_DECODE_STATIC_FLOATS floats = 4 MiB, kept until the process ends); a call whose
 * n * H * nslices * (hd + 2) exceeds that is refused.  The array's address is looked up at
 * the first call on a device, which must be the current device (and the stream's), or by
 * kllm_attn_decode_static_init(); a first call while the stream is being captured is refused
 * (the lookup is not graph work): call the init function on the device before recording.
 * All calls on one GPU share the array and it keeps the last call's contents: the caller
 * must serialise them on one stream per GPU (calls that overlap on one GPU, from two streams
 * or two threads, a replayed graph beside eager calls, race on it); nothing in it needs
 * clearing between calls.  Same kernels, same results as kllm_attn_decode. */
#define KLLM_ATTN_DECODE_STATIC_FLOATS (1 << 20)
int kllm_attn_decode_static_init(void);
int kllm_attn_decode_static(const void* q, void* out, const void* cache, const int* positions,
                            const int* span_of_token, const int* block_table, int max_pages,
                            int page_size, int n, int H, int KV, int hd, int window, float scale,
                            int nslices, int dtype, const int* token_list, int n_listed,
                            hipStream_t stream);

/* Prompt attention on the matrix cores (bfloat16, or float32 with 32-bit MFMA).
 * query_tiles holds (first token row, span) pairs: up to 128 consecutive tokens
 * of one span.  bfloat16: head sizes 32, 64, 96, 128, 192, 256, pages a multiple
 * of 16 and of at most 2,048 tokens, max_pages * page_size at most 2^24.
 * keys_total / keys_longest: the keys that the blocks read, all together and the
 * longest block alone, for the choice of the kernel (0: not known). */
int kllm_attn_prefill(const void* q, void* out, const void* cache, const int* query_tiles,
                      int n_tiles, const int* span_start, const int* span_pos,
                      const int* block_table, int max_pages, int page_size, int H, int KV, int hd,
                      int window, int chunk, int sink, int keep_first, float scale, const float* slopes, long keys_total,
                      int keys_longest, float* part, long part_floats, int nslices, int n_rows, int dtype,
                      hipStream_t stream);
/* nslices of kllm_attn_prefill: how many workgroups share out the keys of a block and head
 * (1: none; more where few blocks of a large head would leave CUs idle; taken only when
 * keys_longest says that the longest block reads 1,280 keys or more).  With more than one,
 * `part` is room for n_rows (the rows of q) x H x nslices x (hd + 2) floats, and the results
 * are merged by a second kernel of the same call. */
int kllm_attn_prefill_slices(int n_tiles, int H, int hd);

/* x[t][c] += sin(a) for even c, cos(a) for odd c, a = positions[t] * base^(-2 (c/2) / d), angle in double. */
int kllm_add_sinusoid(float* x, const int* positions, int n, int d, double base, hipStream_t stream);

/* Activations without a gate (`act` below): the gates' two, and xIELU with the two learned
 * numbers params[0], params[1] (p, q): for z > 0, softplus(p) z^2 + z/2; otherwise
 * (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2. */
#define KLLM_ACT_XIELU 2
#define KLLM_ACT_TANH 3
#define KLLM_ACT_RELU_SQ 4      /* max(z, 0)^2 */
/* out[n][f] = act(sum over s of in[s][n][f]), rounded to out_dtype; a row of `in` begins every
 * in_row_stride elements (f if the rows follow each other). */
int kllm_unary_act(const float* in, int nsplit, long split_stride, int in_row_stride, void* out, int out_dtype,
                   int n, int f, int act, const float* params, hipStream_t stream);

/* The norm of a layer whose sub-layers run side by side.  v = x[src] + mult * (sum of d1's ns1
 * slices + sum of d2's ns2 slices + bias) (each of d1, d2, bias may be null); x[src] = v when
 * write_x; when out is not null, out[r] = v / sqrt(mean over the channel's group of v^2 + eps)
 * * w, the d channels being cut into `groups` equal consecutive groups (1: an RMS norm).
 * src = rows[r] when rows is given (then write_x must be 0), else r. */
int kllm_group_norm_add(float* x, const float* d1, int ns1, long st1, const float* d2, int ns2, long st2,
                        const float* bias, float mult, const float* w, void* out, int out_dtype,
                        const int* rows, int n, int d, int groups, float eps, int write_x,
                        hipStream_t stream);

/* Between the query/key product and attention where queries and keys are normalised over the
 * whole projection.  qk holds the sums [nsplit][n][(H + KV) * hd + KV * dv] (queries, keys,
 * values).  Biases are added (null: none); the whole query row and the whole key row are each
 * divided by their root mean square (eps inside the root) and multiplied by q_w, k_w (null: no
 * norm); the first `rot` elements of every query and key head then turn (cos/sin [n][rot/2] or
 * null; pairs (2j, 2j+1) if `interleaved`, else (j, j + rot/2)); the query is multiplied by
 * 1 + temp_coef * ln(floor((position + 1) / temp_every) + 1) (temp_every 0: not); q_out
 * [n][H*hd] is written, and into the pages of `cache` (null: no append; keys [KV][slot][hd], then
 * values [KV][dv][slot]) go the key and the value; with dv == 0 the values are the keys: the key
 * before its norm (bias added) is cached as the value. */
int kllm_qk_norm_append(const float* qk, int nsplit, long split_stride, const float* q_bias,
                        const float* k_bias, const float* q_w, const float* k_w, float eps, float temp_coef,
                        int temp_every, void* q_out, void* cache, const int* positions,
                        const int* span_of_token, const int* block_table, int max_pages, int page_size,
                        int n, int H, int KV, int hd, int dtype, int dv, const float* cos_t, const float* sin_t,
                        int rot, int interleaved, hipStream_t stream);

/* A recurrent mixer with a matrix state per head, S_t = diag(w) S - (a u)(u^T S) + k v^T,
 * o = S^T r, u = k / sqrt(sum k^2 + key_eps).
 * prep: proj [nsplit][n][5*H*hd + L] holds the sums of the products r | k | v | g | a | w1;
 *   w = exp(-decay_scale * sigmoid(w2 tanh(w1) + w0)), a = sigmoid(a + a_bias); writes scan_in
 *   [H][n][6][hd] (r, k, v, w, u, a*u; a head's tokens follow each other) and gate [n][H*hd] = sigmoid(g).  w2 is [H*hd][L] in w_dtype;
 *   with `low` (sums [low_nsplit][n][H*hd] of w2 tanh(w1), made by a matrix kernel) it is not read.
 * scan: the n tokens of n_spans requests, each request through its state [slots][H][hd][hd] (float32; zero at
 *   position 0), o_out [n][H*hd]; hd up to kllm_delta_scan_max_dim().
 * out: out[n][H*hd] = o / sqrt(mean over the head of o^2 + eps) * weight * gate. */
int kllm_delta_prep(const float* proj, int nsplit, long split_stride, const float* a_bias, const void* w2,
                    const float* w0, const float* low, int low_nsplit, long low_stride, float decay_scale,
                    float key_eps, float* scan_in, float* gate, int n, int H, int hd, int L, int w_dtype,
                    hipStream_t stream);
int kllm_delta_scan_max_dim(void);
int kllm_delta_scan(const float* scan_in, float* o_out, float* state, const int* slots,
                    const int* span_start, const int* span_pos, int n_spans, int n, int H, int hd,
                    hipStream_t stream);
int kllm_delta_out(const float* o, const float* gate, const float* weight, float eps, void* out, int n, int H,
                   int hd, int dtype, hipStream_t stream);

/* Layers whose norm stands behind the sub-layer.  x [n, d] float32.  With sums (`delta`, float32
 * [nsplit][n][d], plus `bias` [d] or null): x += mult * weight * N(delta + bias); without: x =
 * weight * N(x); N(v) = v / sqrt(mean(v^2) + eps).  `out` (or null) receives the new rows of x in
 * `out_dtype`, for the next product; with `next_weight` [d] it receives next_weight * N(x) of the
 * new rows instead: the norm in front of the next sub-layer.  `delta_scale` [n] (or null) is a
 * factor per row on delta's slices.  With `pair_b` ([pair_nb][n][d]) the sums are those of two
 * sub-layers side by side, each normed before they are added: pair_sa * pair_wa * N(delta) +
 * pair_sb * pair_wb * N(pair_b) stands where delta's slices stood.
 * The sums may also be those of a routed feed-forward's chosen experts, not yet added up
 * (`chosen_y` [n * top][d], null: none): then the row is the sum over the token's choices of
 * chosen_wgt * (chosen_idx < E ? chosen_y : chosen_x, the feed-forward's input [n][d]) + delta's
 * slices (a shared expert's; may be null) + bias. */
int kllm_norm_residual(float* x, const float* delta, int nsplit, long split_stride, const float* bias,
                       const float* weight, void* out, int out_dtype, int n, int d, float eps,
                       const float* chosen_y, const void* chosen_x, int chosen_x_dtype, const int* chosen_idx,
                       const float* chosen_wgt, int top, int E, float mult, const float* next_weight,
                       const float* delta_scale, const float* pair_b, int pair_nb, long pair_stride,
                       const float* pair_wa, const float* pair_wb, float pair_sa, float pair_sb, hipStream_t stream);
/* cos/sin [n][half] = factor * cos/sin(positions[t] * freq[i]), the angle in double. */
int kllm_rope_tables_freq(float* cos_t, float* sin_t, const int* positions, const double* freq, int n,
                          int half, double factor, hipStream_t stream);
/* qkv: float32 sums [nsplit][n][(H + KV) dk + KV dv] of the query, key and value products.  Adds
 * `bias` (or null), turns the first `rot` elements of every query and key head (pairs (2j, 2j+1)
 * if `interleaved`, else (j, j + rot/2); cos/sin [n][rot/2] or null), divides every query and
 * key head by its root mean square (`unit_norm`, eps inside the root), writes the queries and
 * appends keys and values to the pages (keys [KV][slot][dk], then values [KV][dv][slot]).
 * With `q_weight` and `k_weight` ([dk] each, shared by the heads) the norm comes first and has
 * weights: every query and key head is divided by its root mean square and multiplied by the
 * weight, then rotated (`unit_norm` is then not looked at). */
int kllm_qkv_norm_append(const float* qkv, int nsplit, long split_stride, const float* bias,
                         const float* cos_t, const float* sin_t, int rot, int interleaved, int unit_norm,
                         float eps, void* q_out, void* cache, const int* positions,
                         const int* span_of_token, const int* block_table, int max_pages, int page_size,
                         int n, int H, int KV, int dk, int dv, int dtype, const float* q_weight,
                         const float* k_weight, hipStream_t stream);
/* out [n][f] = gated(g, u) of the float32 sums gu [nsplit][n][2 f] (gates, then ups) plus `bias`
 * [2 f] or null.  act: a gate's activation (act(g) u), or 4: with g' = min(g, limit) and u' =
 * clamp(u, -limit, limit), g' sigmoid(alpha g') (u' + 1). */
int kllm_gate_bias(const float* gu, int nsplit, long split_stride, const float* bias, void* out,
                   int out_dtype, int n, int f, int act, float limit, float alpha, hipStream_t stream);

/* A routed feed-forward.  route: z float32 sums [nsplit][n][cols] of the router, the first R of a
 * row over all R experts; idx/wgt [n][top] receive the `top` experts with the largest score +
 * correction (null: none) and their scores divided by their sum (`renorm`), times `scale`; the
 * score is softmax(z) (`scoring` 0) or the logistic function of z (1).  With `groups` > 1 (up to
 * 64) the experts form that many equal groups of neighbours, a group's score is the sum of its two
 * largest, and only experts of the `keep` best groups can be chosen.  With `sgate` [n] the sum
 * behind the experts' (column R) is a gate's: sgate = its logistic function.  plan: the entries (token * top + choice) whose
 * expert is below E, grouped by expert into `sorted`, and `tiles` [max_tiles][3] = (expert, first
 * place in sorted, entries <= tile_rows); tile_rows is kllm_moe_tile_rows() or twice that (the
 * same in plan and expert); max_tiles >= ceil(entries / tile_rows) + E.
 * expert, mode 0: out [entries][m] (dtype) = gated(gate, up) of x [tokens][k] against w [E][2 m][k];
 * mode 1: out [entries][m] float32 = x [entries][k] against w [E][m][k].  combine: out [n][d] =
 * sum over a token's choices of wgt * (expert < E ? y [entries][d] : xin [n][d]) + the slices of
 * `shared` [ns][n][d] (null: none), each token's times shared_scale [n] (null: one). */
int kllm_moe_tile_rows(void);
int kllm_moe_route(const float* z, int nsplit, long split_stride, const float* correction, int n, int R,
                   int top, int* idx, float* wgt, int scoring, int groups, int keep, float scale, int renorm,
                   int cols, float* sgate, hipStream_t stream);
int kllm_moe_plan(const int* idx, int entries, int E, int max_tiles, int tile_rows, int* sorted, int* tiles,
                  hipStream_t stream);
int kllm_moe_expert(const void* x, const void* w, void* out, const int* sorted, const int* tiles,
                    int max_tiles, int tile_rows, int top, int m, int k, int mode, int act, float limit,
                    float alpha, int dtype, hipStream_t stream);
/* kllm_moe_expert without tiles, entry by entry (idx [entries] names each entry's expert; those
 * from E on are skipped): for decode batches. */
int kllm_moe_expert_rows(const void* x, const void* w, void* out, const int* idx, int entries, int E,
                         int top, int m, int k, int mode, int act, float limit, float alpha, int dtype,
                         hipStream_t stream);
int kllm_moe_combine(const float* y, const void* xin, const int* idx, const float* wgt, const float* shared,
                     int ns, long shared_stride, float* out, int n, int d, int top, int E, int dtype,
                     const float* shared_scale, hipStream_t stream);

/* out[r] = sampled index of logits[r][:]; temperature/uniform null: greedy. */
int kllm_sample(int* out, const float* logits, const float* temperature, const float* uniform,
                int rows, int vocab, hipStream_t stream);

/* A step's launches in one call.  `words` is a buffer of n_words 64-bit words holding commands
 * (executor.hpp describes the layout: entry point, argument words, structs that arguments
 * point to); they run in order on `stream`, whatever stream argument was recorded.
 * kllm_command_op gives the number that names an entry point of this header in a command
 * (-1: it cannot be recorded), kllm_command_nargs its number of arguments.  Returns 0, or the
 * code of the first command that failed with *failed = its index (-3: the buffer itself is
 * malformed); commands before it have run, none after it.  The role of the reference's
 * te_forward_batch (backend/shim.h:106-117): one call across the language boundary for the
 * whole forward pass. */
int kllm_command_op(const char* name);
int kllm_command_nargs(int op);
int kllm_run_commands(const uint64_t* words, long n_words, int* failed, hipStream_t stream);

/* ---- recurrent mixers with a short convolution (recurrent.hip) ----
 * `proj` are float32 sums [nsplit][n][cols] of a step's projections.  A request's state is a run of
 * `slot_stride` floats per slot; the pointers given here point at the field in slot 0. */

/* The convolution's part of the state, [C][taps - 1] per slot: the inputs (columns col0 .. col0 + C of
 * proj, plus in_bias [C] or null) of each span's last taps - 1 positions. */
int kllm_conv_state_update(const float* proj, int nsplit, long split_stride, int cols, int col0, int C,
                           const float* in_bias, float* state, long slot_stride, int taps, const int* slots,
                           const int* span_start, const int* span_pos, int n_spans, hipStream_t stream);
/* Gated delta rule, what the recurrence reads.  proj columns (`cols` of them): q (G dk) | k (G dk) |
 * v (H dv) | b (H) | a (H) | gate (H dv) | anything else.  conv_w [2 G dk + H dv][taps]; state: the
 * convolution's field.  Writes qn, kn [n][G dk] (unit vectors per head, qn times dk^-1/2), vv [n][H dv],
 * gb [n][2][H] (decay, beta) and gate [n][H dv] = silu of the gate's sums (`gate_sigmoid`: their
 * logistic function).  With `a_sums` ([a_ns][n][a_row], a_stride between slices, the first H dk of
 * a row) the decay has one number per head and key channel, exp(-exp(a_log[h]) softplus(a +
 * dt_bias[h][c])), written to `dec` [n][H dk]; proj then has no a columns.  With `gate_sums`
 * ([g_ns][n][g_row], the first H dv of a row) the gate's sums are these and proj has no gate
 * columns. */
int kllm_gated_delta_prep(const float* proj, int nsplit, long split_stride, const float* conv_w, int taps,
                          const float* state, long slot_stride, const float* a_log, const float* dt_bias,
                          const int* span_of_token, const int* slots, const int* span_start, const int* span_pos,
                          float* qn, float* kn, float* vv, float* gb, float* gate, int n, int H, int G, int dk,
                          int dv, float unit_eps, int cols, const float* a_sums, int a_ns, long a_stride, int a_row,
                          const float* gate_sums, int g_ns, long g_stride, int g_row, int gate_sigmoid, float* dec,
                          hipStream_t stream);
int kllm_gated_delta_max_dim(void);
/* The recurrence: state [H][dk][dv] per slot, o_out [n][H dv].  `dec` (or null): decays per head and
 * key channel [n][H dk], which then take the place of gb's decay. */
int kllm_gated_delta_scan(const float* qn, const float* kn, const float* vv, const float* gb, float* o_out,
                          float* state, long slot_stride, const int* slots, const int* span_start,
                          const int* span_pos, int n_spans, int H, int G, int dk, int dv, const float* dec,
                          hipStream_t stream);
/* Gated linear recurrence.  proj columns: y (W) | x (W).  wr_t, wi_t: the gates' block-diagonal matrices
 * [blocks][in][out]; rate [W] = 8 softplus(lambda).  Writes a and the added term, [n][W] each. */
int kllm_linear_recurrence_prep(const float* proj, int nsplit, long split_stride, const float* x_bias,
                                const float* conv_w, const float* conv_b, int taps, const float* state,
                                long slot_stride, const float* wr_t, const float* wi_t, const float* br,
                                const float* bi, const float* rate, const int* span_of_token, const int* slots,
                                const int* span_start, const int* span_pos, float* a_out, float* b_out, int n, int W,
                                int blocks, hipStream_t stream);
/* S <- a S + b per span and channel (state [W] per slot); out [n][W] = S * gelu_tanh(y + y_bias). */
int kllm_linear_recurrence_scan(const float* a_in, const float* b_in, const float* proj, int nsplit,
                                long split_stride, const float* y_bias, float* state, long slot_stride,
                                const int* slots, const int* span_start, const int* span_pos, void* out, int n_spans,
                                int W, int dtype, hipStream_t stream);

/* out[i] = sa * sum over a's slices + sb * sum over b's slices (float32, `count` elements a slice). */
int kllm_scaled_sum(float* out, const float* a, int na, long stride_a, float sa, const float* b, int nb,
                    long stride_b, float sb, long count, hipStream_t stream);
/* out [n][d] = sa * wa * N(a) + sb * wb * N(b), row by row, of the float32 sums a [na][n][d] and b
 * [nb][n][d]; N(v) = v / sqrt(mean(v^2) + eps); wa, wb [d]. */
int kllm_normed_sum(float* out, const float* a, int na, long stride_a, float sa, const float* wa, const float* b,
                    int nb, long stride_b, float sb, const float* wb, int n, int d, float eps, hipStream_t stream);

/* ---- attention through low-rank latents (latent.hip): one cached row of rank + dr per token ---- */
int kllm_latent_max_row(void);
int kllm_latent_kv_append(const float* dkv, int nsplit, long split_stride, const float* weight, float eps,
                          const float* cos_t, const float* sin_t, void* cache, const int* positions,
                          const int* span_of_token, const int* block_table, int max_pages, int page_size, int n,
                          int rank, int dr, int dtype, long in_stride, hipStream_t stream);
/* out [n][r] = RMS norm with `weight` of r columns of float32 sums whose rows are in_stride apart. */
int kllm_latent_norm(const float* in, int nsplit, long split_stride, long in_stride, const float* weight, float eps,
                     void* out, int n, int r, int dtype, hipStream_t stream);
int kllm_latent_query(const float* q, int nsplit, long split_stride, const void* w_uk, const float* cos_t,
                      const float* sin_t, void* out, int n, int H, int d, int dr, int rank, int dtype,
                      int transposed, hipStream_t stream);
int kllm_attn_latent(const void* q, void* out, const void* cache, const int* positions, const int* span_of_token,
                     const int* block_table, int max_pages, int page_size, int n, int H, int row, int rank,
                     float scale, int dtype, int mode, float* part, long part_floats, int nslices, hipStream_t stream);
int kllm_latent_out(const void* attended, const void* w_uv, const float* gate, int nsplit, long split_stride,
                    long gate_stride, void* out, int n, int H, int dv, int rank, int dtype, hipStream_t stream);

#ifdef __cplusplus
}
#endif
