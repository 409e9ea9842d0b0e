// Flat C ABI of the gfx950 kernel library. Every pointer is a device pointer unless a
// comment says otherwise; `stream` is a hipStream_t. Every function returns 0 on success
// and -1 on failure, after which fw_last_error() describes what was refused. Shapes are
// checked on the host before anything is launched; a kernel never runs on operands it
// was not written for.
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* fw_last_error(void);
int fw_abi_version(void);

// out[r][:] = table[ids[r]][:] * scale  (float32 out: the residual stream); with a second table (places
// null: none) + places_table[places[r]][:], not scaled (a learned vector per position)
int fw_embed_rows(const void* table, int table_dtype, const int32_t* ids, float* out,
                  int rows, int hidden, int vocab, float scale, const void* places_table, int places_dtype,
                  const int32_t* places, int places_entries, void* stream);

// x <- x * scale, then with cap > 0: x <- cap * tanh(x / cap); float32, in place
int fw_scale_softcap(float* x, long long count, float scale, float cap, void* stream);

// RMS norm of float32 rows: out[r] = x[src] * rsqrt(mean(x[src]^2) + eps) * w, where
// src = row_index ? row_index[r] : r.  one_centered: multiply by (1 + w) instead of w.
int fw_rmsnorm_rows(const float* x, const float* weight, void* out, int out_dtype,
                    const int32_t* row_index, int rows, int hidden, float eps,
                    int one_centered, void* stream);

// out = a[M][K] . w[N][K]^T (+ bias[N]); out_mode 0: store in out_dtype,
// 1: out (float32) += result (the residual sum).
int fw_gemm_generic(const void* a, int a_dtype, const void* w, int w_dtype, const float* bias,
                    void* out, int out_dtype, int out_mode, int M, int N, int K, void* stream);

// bfloat16 matrix products on the matrix cores, float32 accumulation. a [M][K], w [N][K], K a
// multiple of 8. mode 0: out = a . w^T (+ bias) stored as out_dtype; mode 1: out (float32) +=
// a . w^T (+ bias); mode 2 (SwiGLU): w is [2N][K], gate rows then up rows, out [M][N] bfloat16 =
// silu(a . gate^T) * (a . up^T). fw_gemm_skinny streams w once for M <= 64 (decode);
// fw_gemm_mfma tiles both operands through LDS (prompts).
int fw_gemm_skinny(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                   int M, int N, int K, void* stream);
int fw_gemm_mfma(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                 int M, int N, int K, void* stream);
// The prompt product with large tiles (256 x 256 or 256 x 192; storing products also 128 rows by as many columns,
// where that fills the chip better), for shapes that give enough of them to fill the chip
// (fw_gemm_mfma_big_tiles says how many, fw_gemm_mfma_big_plan also which).
int fw_gemm_mfma_big(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                     int M, int N, int K, void* stream);
int fw_gemm_mfma_big_tiles(int mode, int M, int N, int K);     // 0: the kernel does not take the shape
int fw_gemm_mfma_big_plan(int mode, int M, int N, int K, int* rows, int* columns);     // the same, and the tile's edges
// The prompt product with tiles of 128 rows and `columns` (128 or 64) columns whose four waves split
// K (half the LDS traffic per flop of fw_gemm_mfma's tiles), for outputs too narrow for the
// 256 x 256 tiles to fill the chip. Modes 0 and 1; K a multiple of 64 (fw_gemm_mfma_deep_tiles says
// 0 for shapes it does not take, else the number of tiles).
int fw_gemm_mfma_deep(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                      int M, int N, int K, int columns, void* stream);
int fw_gemm_mfma_deep_tiles(int mode, int M, int N, int K, int columns);
// fw_gemm_mfma with K cut into slices for products with fewer tiles than compute units (a few
// hundred rows, a narrow output). fw_gemm_mfma_split_plan says what a shape needs: bytes of
// workspace and int32 counters that are zero before the first call and are left zero (both 0: the
// shape is not cut, use fw_gemm_mfma). Calls that overlap on one device need their own of both.
int fw_gemm_mfma_split_plan(int mode, int M, int N, int K, size_t* workspace_bytes, int* counters);
int fw_gemm_mfma_split(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                       int M, int N, int K, void* workspace, size_t workspace_bytes, int* counters,
                       int counters_len, void* stream);
// The same product for 1..64 rows with K split over workgroups, so that a is not re-read by every
// few features (decode steps of 17..64 requests). fw_gemm_medium_plan says what a shape needs:
// bytes of workspace (0: none) and int32 counters (0: none) that are zero before the first call;
// the kernel leaves them zero. Calls that overlap on one device need their own of both.
// The accumulating product can leave what the norm after it needs, as fw_gemm_decode does
// (next_activations [M][N] bfloat16, next_squares [squares_rows][16 for M <= 16, else 64]), and
// any mode takes such prepared activations as a, with squares / squares_rows / eps.
int fw_gemm_medium_plan(int M, int N, int K, int mode, size_t* workspace_bytes, int* counters, int* squares_rows);
int fw_gemm_medium(const void* a, const void* w, int w_tiled, const float* bias, void* out, int out_dtype, int mode,
                   int M, int N, int K, void* workspace, size_t workspace_bytes, int* counters,
                   int counters_len, const float* next_norm_weight, int next_one_centered,
                   void* next_activations, float* next_squares, const float* squares, int squares_rows,
                   float eps, float glu_limit, float glu_alpha, float glu_shift, void* stream);

// Fused product for decode steps of up to 16 rows. prologue 0: a is bfloat16 [M][K]; 1: a is
// float32 rows, RMS-normed with norm_weight/eps (rows gathered through row_index if given) inside
// the kernel. epilogue 0: store out_dtype [M][N]; 1: float32 out += ; 2: SwiGLU, w = [gate rows;
// up rows], out bfloat16 [M][N]; 3: gated short convolution of single-token segments, w = [B rows;
// C rows; x rows] of N channels each, state [slots][N][kernel_size - 1] read and shifted.
// fw_gemm_decode_fits says whether a shape is taken (1) or must go to separate kernels (0).
// The accumulating epilogue can also leave what the NEXT norm needs: next_activations bfloat16
// [M][N] = x_new * w_next and next_squares [fw_gemm_decode_accumulate_tiles(N)][16], per-tile sums
// of x_new^2 of every row. A later call takes them with prologue 2 (a = those activations,
// squares/squares_tiles = those sums, eps) and applies the row's scale in its epilogue.
// glu_limit / glu_alpha / glu_shift (here and in fw_gemm_medium, epilogue 2 only): with a limit <= 0 the
// gated unit is SwiGLU, silu(gate) * up; with a positive one its halves are clamped, g = min(gate,
// limit), u = clamp(up, -limit, limit), and out = g * sigmoid(alpha * g) * (u + shift).
// w_tiled (here and in fw_gemm_medium): w is not row-major [rows][K] but lies in operand tiles,
// [rows / 16][K / 32][4][16][8]: tile (i, j) holds rows 16 i .. 16 i + 15, columns 32 j .. 32 j + 31 as
// 1 KB in the order in which a wave loads a matrix-core operand (lane = 16 * (column / 8) + row), so
// that a wave reads whole contiguous kilobytes (rows padded with zeros to a multiple of 16; K a
// multiple of 32). The same sums in the same order: the results are bit for bit those of row-major w.
int fw_gemm_decode(int prologue, const void* a, const float* norm_weight, const int32_t* row_index, float eps,
                   int one_centered, const void* w, int w_tiled, const float* bias, void* out, int out_dtype, int epilogue,
                   int M, int N, int K, const float* taps, const float* conv_bias, float* state,
                   const int32_t* seg_slot, int kernel_size, const float* next_norm_weight,
                   int next_one_centered, void* next_activations, float* next_squares, const float* squares,
                   int squares_tiles, float glu_limit, float glu_alpha, float glu_shift, void* stream);
int fw_gemm_decode_fits(int M, int N, int K, int epilogue);
int fw_gemm_decode_accumulate_tiles(int N);

// out[r][i] = silu(gu[r][i]) * gu[r][I + i]; the input may be float32 beside a bfloat16 output
int fw_swiglu(const void* gate_up, int in_dtype, void* out, int out_dtype, int rows, int intermediate,
              void* stream);

// cos/sin of position * inv_freq for every row: tables [rows][half]
int fw_rope_table(const int32_t* positions, const double* inv_freq, float* cos_out, float* sin_out,
                  int rows, int half, void* stream);

// out[r] = 1 + coef * ln(floor((positions[r] + 1) / every) + 1): a factor on a row's queries that grows with its position
int fw_query_temperature(const int32_t* positions, float* out, int rows, float coef, int every, void* stream);

// Gated short convolution over a mixed batch. bcx [rows][3H] = (B | C | x); taps [H][L]
// oldest first; conv_bias [H] or null; state [slots][H][L-1] float32, oldest first.
// Row r belongs to segment row_seg[r]; segment s covers rows seg_row0[s]..seg_row0[s+1]
// and continues the sequence whose state lives in slot seg_slot[s].
int fw_shortconv(const void* bcx, int in_dtype, void* out, int out_dtype, const float* taps,
                 const float* conv_bias, float* state, const int32_t* row_seg, const int32_t* seg_row0,
                 const int32_t* seg_slot, int rows, int segments, int hidden, int kernel_size,
                 int slots, void* stream);

// Per-head RMS norm of q and k (weights may be null: no norm), rotation of the
// first rotary_dim channels by the row's angle (interleaved 0: channel i turns with channel i + rotary_dim / 2;
// 1: channel 2i with channel 2i + 1; the tables are the same), q out, k and v appended to the pages of
// the row's segment. qkv [rows][(nh + nkv) hd + nkv vd]: values may have a size vd of their own.
// k_pages [pages][nkv][P][hd]; v_pages [pages][nkv][vd][P]. block_table [segments][table_stride].
int fw_qk_norm_rope_kv_write(const void* qkv, int in_dtype, void* q_out, int dtype, const float* q_norm_weight,
                             const float* k_norm_weight, float eps, const float* cos_table,
                             const float* sin_table, int rotary_dim, void* k_pages, void* v_pages,
                             const int32_t* block_table, int table_stride, const int32_t* row_seg,
                             const int32_t* row_pos, int rows, int num_heads, int num_kv_heads,
                             int head_dim, int v_dim, int page_size, int num_pages, int write_kv, int interleaved, int q_only,
                             const float* q_row_scale, void* stream);

// Causal attention of every row over the cached keys 0..row_pos[r] of its segment, or the last `window`
// of them, or with `chunk` > 0 those of its own chunk of that many positions (counted from position 0
// of the sequence); softcap c > 0: score <- c * tanh(score / c) after the scale. out [rows][nh*vd].
// keep_first n > 0 (beside a window): the first n keys of the sequence are seen as well, wherever the window
// stands. sinks (float32 [heads], or null): one more term exp(sinks[head]) in the softmax's denominator, with
// no key and no value, not scaled. (q_only of fw_qk_norm_rope_kv_write / fw_attention_decode_fused: the rows
// of qkv hold the queries alone, [heads * head_dim]: the keys and values are another layer's.)
// slopes (float32 [heads], or null): a bias by distance, slopes[head] * (row's position - key's position) is taken off
// the score behind the cap. q_row_scale (float32 [rows], or null; fw_qk_norm_rope_kv_write and
// fw_attention_decode_fused): a factor on the row's normed and rotated queries (one that depends on the position, say).
int fw_attention_generic(const void* q, void* out, int dtype, const void* k_pages,
                         const void* v_pages, const int32_t* block_table, int table_stride,
                         const int32_t* row_seg, const int32_t* row_pos, int rows, int num_heads,
                         int num_kv_heads, int head_dim, int v_dim, float scale, int window, int chunk, float softcap,
                         int keep_first, const float* sinks, const float* slopes, int page_size, int num_pages, void* stream);

// The same attention on the matrix cores, bfloat16 only, head_dim and v_dim (the size of a value and of a
// head's output: out [rows][nh * v_dim]) multiples of 16 up to 256.
// Prompt portions: rows are cut into tiles of up to 64 that never span two segments (tile_seg,
// tile_row0), in any order: workgroups start in the order of the tiles, so the caller lists those
// that see the most keys first. heads_together: how many query heads of a kv group one workgroup takes, reading
// the keys and values once for all of them (1, or 4 up to head_dim 64: 4 pays behind a long
// context, 1 evens out a short causal prompt); 0: chosen from the shape alone.
int fw_attention_prefill(const void* q, void* out, const void* k_pages, const void* v_pages,
                         const int32_t* block_table, int table_stride, const int32_t* tile_seg,
                         const int32_t* tile_row0, int tiles, const int32_t* seg_row0, const int32_t* row_pos,
                         int rows, int num_heads, int num_kv_heads, int head_dim, int v_dim, float scale, int window,
                         int chunk, float softcap, int keep_first, const float* sinks, const float* slopes, int page_size, int num_pages,
                         int heads_together, void* stream);
// Decode (one row per request): the keys are split between workgroups in runs of 4 pages and
// merged in order by the workgroup that finishes last. partial: float32 workspace
// [rows][heads][max_splits][v_dim + 4]; max_context: an upper bound on position + 1 of every
// row, known to the caller; tickets: rows * kv_heads * ceil(heads / kv_heads / 16) int32 counters,
// zero before the first call and left zero. decode_work: null, or one int32 on the device, the runs
// of 4 pages that all the rows of the step see together; with it a workgroup takes as many runs as
// bring the step down to about 512 workgroups.
int fw_attention_decode(const void* q, void* out, float* partial, int max_splits, int max_context,
                        const int32_t* decode_work, int* tickets, int tickets_len, const void* k_pages, const void* v_pages, const int32_t* block_table, int table_stride,
                        const int32_t* row_seg, const int32_t* row_pos, int rows, int num_heads, int num_kv_heads,
                        int head_dim, int v_dim, float scale, int window, int chunk, float softcap, int keep_first,
                        const float* sinks, const float* slopes, int page_size, int num_pages, void* stream);

// The same with the work of fw_qk_norm_rope_kv_write in front of it, in one kernel: qkv float32
// [rows][(heads + kv_heads) * head_dim + kv_heads * v_dim] are the step's raw projections; every workgroup norms and
// rotates the query heads it works on, and the one whose pages hold the row's own position stores
// the new key (normed, rotated) and value (write_kv 0: they are in the cache already).
int fw_attention_decode_fused(const float* qkv, const float* q_norm_weight, const float* k_norm_weight, float eps,
                              const float* cos_table, const float* sin_table, int rotary_dim, int write_kv, void* out,
                              float* partial, int max_splits, int max_context, const int32_t* decode_work, int* tickets,
                              int tickets_len, void* k_pages,
                              void* v_pages, const int32_t* block_table, int table_stride, const int32_t* row_seg,
                              const int32_t* row_pos, int rows, int num_heads, int num_kv_heads, int head_dim, int v_dim,
                              float scale, int window, int chunk, float softcap, int interleaved, int q_only, int keep_first,
                              const float* sinks, const float* slopes, const float* q_row_scale, int page_size, int num_pages, void* stream);

// ids[r] = argmax(logits[r]) with ties to the lowest id, also written to also[r] if that is not null;
// advance[r] += 1 if that is not null; workspace: rows * 64 64-bit words
int fw_argmax_rows(const float* logits, int32_t* ids, int32_t* also, int32_t* advance, void* workspace, int rows, int vocab,
                   void* stream);

// fw_argmax_rows for callers that cannot allocate device memory (code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc) and so have no workspace to bring. It has no
// counterpart in the reference. The keys of the parts go to an array built into the library, one
// copy per GPU (512 KB, held until the process ends); at most fw_argmax_rows_static_max_rows() rows
// (1,024), more is refused with an error. The call allocates and frees nothing. Every call on a GPU
// uses that GPU's one array: calls that overlap there (several streams or threads) race; calls that
// follow each other in one stream do not. Same results as fw_argmax_rows.
int fw_argmax_rows_static(const float* logits, int32_t* ids, int32_t* also, int32_t* advance, int rows, int vocab,
                          void* stream);
int fw_argmax_rows_static_max_rows(void);

// The next token of every row, drawn on the device: settings float32 [rows][4] = temperature (0:
// greedy, the best candidate, ties to the lowest id), top_k (0: all candidates), top_p, min_p;
// states [rows]: the rows' xorshift64* generators, moved on by the rows that draw. also / advance
// as in fw_argmax_rows. Candidates are taken in (value descending, id ascending) order; the sums of
// a list of up to 1,024 candidates are float64, in that order, those of a longer one whole numbers
// (parts in 2^-46 fixed point at 65,536 logits).
int fw_sample_rows(const float* logits, const float* settings, unsigned long long* states, int32_t* ids, int32_t* also,
                   int32_t* advance, int rows, int vocab, void* stream);

// Layer norm with a weight and no bias: out[r] = (x[src] - mean) / sqrt(mean((x[src] - mean)^2) + eps) * w,
// src = row_index ? row_index[r] : r.
int fw_layernorm_rows(const float* x, const float* weight, void* out, int out_dtype, const int32_t* row_index,
                      int rows, int hidden, float eps, void* stream);

// out[r][j] = gelu_tanh(z[r][j]) * table[ids[r]][col0 + j] for j < width; z float32 [rows][z_stride],
// table [table_rows][table_width] (a second token table of which a layer reads its own columns).
int fw_gelu_gate_rows(const float* z, int z_stride, const void* table, int table_dtype, int table_rows, int table_width,
                      int col0, const int32_t* ids, void* out, int out_dtype, int rows, int width, void* stream);

int fw_fill_zero(void* ptr, long long bytes, void* stream);
// `pieces` runs of `bytes` each, `stride_bytes` apart, cleared in one launch
int fw_fill_zero_pieces(void* ptr, int pieces, long long bytes, long long stride_bytes, void* stream);

// ---- the gated delta rule (a linear recurrence over a matrix state per head) -----------------------
// What the recurrence reads, from one step's projections, as one record per (row, head):
// [q (d4) | k (d4) | g (d4) | beta, 3 unused | v (v4)] float32, d4 and v4 the head sizes rounded up to a
// multiple of 4 (fw_delta_record_floats floats in all; what lies past dim or vdim is zero).
// proj [rows][proj_stride]: columns 0 .. 2 G d + H vd - 1 hold q | k | v before their short causal
// convolutions (G = kv_heads heads of d = dim channels for q and for k, H = heads of vd = vdim channels
// for v; head h reads q/k head h / (H / G)), columns beta_col .. + H - 1 the write strengths before
// their sigmoid. a [rows][a_stride]: the decays' arguments in its first H d columns. taps
// [channels][L], the last column the current token's; conv_state [slots][channels][L - 1], oldest
// first, read and then moved on by the segment's rows. q, k, v are the silu of the convolutions, q and
// k of unit length per head (sum of squares + 1e-6 under the root), q also times d^-1/2;
// g = exp(-exp(A_log[h]) * softplus(a + dt_bias)). decay_per_head: a holds one argument per head
// (its first H columns) and dt_bias [H]; every key channel of the head then decays alike.
int fw_delta_record_floats(int dim, int vdim);
int fw_delta_prepare(const void* proj, int dtype, int proj_stride, int beta_col, const void* a, int a_stride, const float* taps,
                     float* conv_state, const float* A_log, const float* dt_bias, const int32_t* row_seg,
                     const int32_t* seg_row0, const int32_t* seg_slot, float* records, int rows, int segments,
                     int heads, int kv_heads, int dim, int vdim, int taps_count, int slots, int decay_per_head, void* stream);
// Per segment and head, token by token: S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T;
// o = S^T q. records [rows][H][fw_delta_record_floats]. state [slots][H][vd][d] (S transposed), read
// at the segment's start and written at its end. out [rows][H vd].
int fw_gated_delta_rule(const float* records, float* state, float* out, const int32_t* seg_row0,
                        const int32_t* seg_slot, int rows, int segments, int heads, int dim, int vdim,
                        int slots, void* stream);
// out[r][h][j] = o[r][h][j] * rsqrt(mean_j o[r][h]^2 + eps) * weight[j] * act(gate[r][h vd + j]);
// act is the sigmoid, or with gate_silu z * sigmoid(z)
int fw_gated_head_norm(const float* o, const void* gate, int gate_dtype, int gate_stride, const float* weight, int weight_per_head,
                       void* out, int out_dtype, int rows, int heads, int vdim, float eps, int gate_silu, void* stream);

// ---- sublayers whose output is normed ------------------------------------------------------------
// x[r] += mult * rmsnorm(scale_a a[r] + scale_b b[r]) * w (b may be null; one_centered: 1 + w);
// rounded (may be null): the new x once more in rounded_dtype, for the products that read it next.
int fw_norm_scale_add(float* x, const float* a, const float* b, float scale_a, float scale_b, const float* weight,
                      int one_centered, float eps, float mult, void* rounded, int rounded_dtype, int rows,
                      int hidden, void* stream);
// A sublayer between two norms: x[r] += norm(a[r]) * weight (RMS: a / sqrt(mean(a^2) + eps); centered: the
// row's mean taken off first), and what reads x next, formed from the new row in the same pass:
// next_kind 0 nothing, 1 x rounded to next_dtype, 2 the RMS norm of x times next_weight, 3 the same with
// the mean taken off (next_eps under its root); next_out [rows][hidden] of next_dtype.
int fw_norm_add_norm(float* x, const float* a, const float* weight, int centered, float eps, int next_kind,
                     const float* next_weight, float next_eps, void* next_out, int next_dtype, int rows, int hidden,
                     void* stream);
// out (bfloat16) = x (float32), count elements
int fw_round_rows(const float* x, void* out, long long count, void* stream);
// gate_up [rows][2 I]: out[r][i] = g sigmoid(alpha g) (u + shift), g = min(gate, limit),
// u = clamp(up, -limit, limit)
int fw_clamped_glu(const void* gate_up, int in_dtype, void* out, int out_dtype, int rows, int intermediate,
                   float limit, float alpha, float shift, void* stream);

// ---- attention over a cached latent ---------------------------------------------------------------
// The latent of a step's rows: columns col0 .. col0 + rank - 1 of raw [rows][raw_stride] (float32), RMS-normed
// (eps under the root) times weight [rank], stored at each row's position in both layouts of a cache
// with one key/value head of `rank` channels: k_pages [pages][1][P][rank + rot], v_pages [pages][1][rank][P].
// rot > 0: the next rot columns of raw are a key part that all heads share: not normed, neighbouring channels
// (2i, 2i + 1) of its first `turn` turned by the row's angles (tables [rows][turn / 2]), stored behind the latent in the key layout only.
int fw_latent_norm_write(const float* raw, int raw_stride, int col0, const float* weight, float eps, void* k_pages,
                         void* v_pages, int dtype, const int32_t* block_table, int table_stride, const int32_t* row_seg,
                         const int32_t* row_pos, int rows, int rank, int rot, int turn, const float* cos_table, const float* sin_table,
                         int page_size, int num_pages, void* stream);
// A map per head: out[r][h N + n] = sum_k in[r][h K + k] * w[h][n][k], with a gate (may be null) times
// sigmoid(gate[r][h N + n]). in [rows][in_stride], w [heads][N][K], gate float32 [rows][gate_stride],
// out [rows][heads N]. in_head / out_head / out_stride (0: K, N, heads * out_head): a head's inputs lie in_head apart
// and its outputs out_head apart in rows out_stride wide, where a head's vector holds more than the map reads or writes.
int fw_head_linear(const void* in, int in_dtype, int in_stride, const void* w, int w_dtype, const float* gate, int gate_stride,
                   void* out, int out_dtype, int rows, int heads, int N, int K, int in_head, int out_head, int out_stride,
                   void* stream);
// Channels col0 .. col0 + rot - 1 of every head's vector (heads in_head apart in rows in_stride wide) turned, neighbouring
// channels (2i, 2i + 1) of the first `turn` by the row's angles (tables [rows][turn / 2]), and stored from channel out_col0 of the head's
// vector in out (heads out_head apart in rows out_stride wide).
int fw_rotate_place(const void* in, int in_dtype, int in_stride, int in_head, int col0, const float* cos_table,
                    const float* sin_table, void* out, int out_dtype, int out_stride, int out_head, int out_col0, int rows,
                    int heads, int rot, int turn, void* stream);

// ---- a recurrence with a decay per key channel formed by the token ("wkv") --------------------------------
// Token shift: h = rmsnorm(x) * (w or 1 + w) (norm_weight null: h = x); out[s][r] = h[r] + (h[r - 1] - h[r]) * mu[s],
// s < mixes, out [mixes][rows][hidden] of out_dtype; the row before a segment's first is last[slot] (float32
// [slots][hidden]), which is moved on to the h of the segment's last row.
int fw_token_shift_mix(const float* x, const float* norm_weight, float eps, int one_centered, const float* mu, int mixes,
                       float* last, int slots, const int32_t* row_seg, const int32_t* seg_row0, const int32_t* seg_slot,
                       void* out, int out_dtype, int rows, int segments, int hidden, void* stream);
// out = tanh(x): float32 in, out_dtype out
int fw_tanh_rows(const float* x, void* out, int out_dtype, long long count, void* stream);
// Per head: o_t = S^T r_t + (r_t . (u k_t)) v_t; S <- diag(exp(-exp(a_t + w0))) S + k_t v_t^T. r, k, v float32 rows of
// rkv_stride floats (heads * dim used), a rows of a_stride; w0 [heads * dim], u [heads * dim]; state float32
// [slots][heads][dim (key)][dim (value)]; out float32 [rows][heads * dim].
int fw_wkv_recurrence(const float* r, const float* k, const float* v, int rkv_stride, const float* a, int a_stride,
                      const float* w0, const float* u, float* state, int slots, float* out, const int32_t* seg_row0,
                      const int32_t* seg_slot, int rows, int segments, int heads, int dim, void* stream);

// ---- a mixture of feed-forward units chosen per token ------------------------------------------------------
// chosen / weight [rows][top]: the `top` largest of logits[r] + bias (float32 [rows][experts]; ties: the lowest
// id; bias may be null), largest first, and the softmax over those alone. groups > 1: the experts form that many equal
// groups of neighbours, a group's score is its best expert's, and only experts of the `keep` best groups (ties: the
// lowest group) can be chosen. score_all: the weights are the softmax over ALL experts at the chosen ones, divided by
// their sum + 1e-20.
int fw_moe_route(const float* logits, const float* bias, int32_t* chosen, float* weight, int rows, int experts, int top,
                 int groups, int keep, int score_all, void* stream);
// The pairs (row, choice) sorted by expert, in the order of the pairs within an expert: expert_begin
// [experts + 1], place_row [rows * top] (the row of each place), pair_place [rows * top] (the place of each pair).
int fw_moe_arrange(const int32_t* chosen, int32_t* expert_begin, int32_t* place_row, int32_t* pair_place, int rows, int experts,
                   int top, void* stream);
// out[place] = a[place_row ? place_row[place] : place] . w[expert of place]^T; w [experts][N][K], or with
// gated [experts][2 N][K] (gate rows, then up rows) and out = silu(gate) * up, or with a glu_limit > 0 the clamped
// unit g sigmoid(glu_alpha g) (u + glu_shift), g = min(gate, limit), u = clamp(up, -limit, limit). out [places][N].
int fw_grouped_gemm(const void* a, int a_dtype, const int32_t* place_row, const void* w, int w_dtype,
                    const int32_t* expert_begin, void* out, int out_dtype, int gated, int places, int experts, int N, int K,
                    float glu_limit, float glu_alpha, float glu_shift, void* stream);
// x[r] += sum_j weight[r][j] * y[pair_place[r][j]], j in order; float32
int fw_moe_combine(float* x, const float* y, const float* weight, const int32_t* pair_place, int rows, int top, int hidden,
                   void* stream);

// ---- a short causal convolution per channel, and a gated linear recurrence per channel -----------------------------
// y[t][c] = sum_j taps[c][j] * x[t - L + 1 + j][c] (+ bias[c]; null: none) over mixed segments, float32. in [rows][in_stride]
// (the first `channels` columns), taps [channels][L] with the last column the current token's, state [slots][channels][L - 1]
// oldest first: the inputs before a segment's first row, read and then moved on by the segment's rows. out [rows][out_stride];
// channels echo_col0 .. + echo_cols - 1 are written once more from column echo_to on (echo_cols 0: none). single_rows: every
// segment is one row (row r is segment r): outputs and the slots' move in one launch.
int fw_causal_conv(const float* in, int in_stride, const float* taps, const float* bias, float* state, const int32_t* row_seg,
                   const int32_t* seg_row0, const int32_t* seg_slot, float* out, int out_stride, int echo_col0, int echo_cols,
                   int echo_to, int rows, int segments, int channels, int taps_count, int slots, int single_rows, void* stream);
// Per segment and channel c, row by row: r = sigmoid(gates[r_col] + r_bias[c]), i = sigmoid(gates[i_col] + i_bias[c]),
// a = exp(-rate * r * softplus(lam[c])), S <- a S + sqrt(1 - a^2) * i * u[c], out[c] = S * gelu_tanh(y[c]). The gates of a
// block of block_width channels lie side by side, [r of the block | i of the block], block after block (gates rows of
// gates_stride >= 2 * channels floats). state float32 [slots][channels], read at a segment's start, written at its end.
// All float32; out [rows][channels] of out_dtype. workspace: null, or 2 * rows * channels floats: segments of more than 256
// rows are then walked in chunks of 64 rows side by side (their sums differ from the walk in order by rounding alone).
int fw_rglru_scan(const float* u, int u_stride, const float* gates, int gates_stride, const float* y, int y_stride,
                  const float* r_bias, const float* i_bias, const float* lam, float rate, float* state, const int32_t* seg_row0,
                  const int32_t* seg_slot, void* out, int out_dtype, int rows, int segments, int channels, int block_width,
                  int slots, float* workspace, void* stream);

#ifdef __cplusplus
}
#endif
