// C entry points of the kernel library (loaded through ctypes).
//
// Every function returns 0 on success; otherwise bc4g_last_error() holds the
// reason (sizes a kernel refuses, a failed launch).  Pointers are device
// pointers; `stream` is a hipStream_t.  dtype codes: 0 = float32, 1 = bfloat16.
// Shapes are checked here, on the host, before anything is launched.
#pragma once

#include <stdint.h>

extern "C" {

const char* bc4g_last_error();
int bc4g_version();
const char* bc4g_sources_digest();   // digest of the sources and flags the library was built from

// x[t, :] = float(table[ids[t], :])            (reference: embedding_lookup.cu:16-31)
int bc4g_embed_gather(const void* table, int table_dtype, const int32_t* ids, float* out,
                      int n_tokens, int hidden, int vocab, void* stream);

// x[t, :] (+)= float(table[ids[t], :]) * factor  (add 0: stored, 1: added to what x holds)
int bc4g_embed_rows(const void* table, int table_dtype, const int32_t* ids, float* out, int n_tokens, int hidden, int vocab,
                    float factor, int add, void* stream);

// out[r, :] = x[rows ? rows[r] : r, :] * rsqrt(mean(x^2) + eps) * w      (rmsnorm.cu:16-41)
// x is the float residual stream; out has out_dtype; w has w_dtype.
int bc4g_rmsnorm(const float* x, const int32_t* rows, const void* w, int w_dtype, void* out,
                 int out_dtype, int n_rows, int hidden, float eps, void* stream);
// The same with every row in `groups` equal runs of neighbouring channels, each run brought to unit mean square by itself (w spans the row).
int bc4g_rmsnorm_groups(const float* x, const int32_t* rows, const void* w, int w_dtype, void* out, int out_dtype, int n_rows,
                        int hidden, int groups, float eps, void* stream);
// x = (keep ? x : 0) + scale * y + bias on the float32 stream x [n_rows, hidden] (y float32 of that shape; scale, bias float32
// [hidden], each may be null: 1, 0), written back; with w (and out, in out_dtype) also out = the norm of the new x in
// `groups` parts as bc4g_rmsnorm_groups computes it (stream_update.hip).
int bc4g_stream_update(float* x, const float* y, const float* scale, const float* bias, int keep, const void* w, int w_dtype,
                       void* out, int out_dtype, int n_rows, int hidden, int groups, float eps, void* stream);
// out[t] = [x[t, :] | table[ids[t], :] * factor] in out_dtype, [n_tokens, 2 hidden]: the stream beside the embedding.
int bc4g_embed_beside(const float* x, const void* table, int table_dtype, const int32_t* ids, float factor, void* out,
                      int out_dtype, int n_tokens, int hidden, int vocab, void* stream);
// The same for a stream whose last addition is still in parts [n_parts, n_rows, hidden] (float32, as
// bc4g_gemm_mfma_parts leaves them): x += parts[0] + parts[1] + ... in that order, written back, then out = its norm
// (bfloat16).  hidden a multiple of 8, at most 8192.
int bc4g_rmsnorm_sum(float* x, const float* parts, int n_parts, const void* w, int w_dtype, void* out, int out_dtype,
                     int n_rows, int hidden, float eps, void* stream);

// out[m, n] (+)= sum_k a[m, k] * w[n, k]        (gemm_tiled.cuh:36-96, plain float FMA)
// accumulate != 0 adds into a float `out` (the residual stream).
int bc4g_gemm_generic(const void* a, int a_dtype, const void* w, int w_dtype, void* out,
                      int out_dtype, int accumulate, int m, int n, int k, void* stream);

// out[t, i] = silu(gate_i) * up_i                                        (swiglu.cu:17-25)
// interleaved 0: gu[t] = all gates, then all ups.  1: blocks of 16 = eight gates, then the eight
// ups of the same outputs.
int bc4g_swiglu(const void* gu, void* out, int dtype, int n_tokens, int inter, int interleaved, void* stream);

// Rotates q (in place) and k by each row's position, and writes k and v into
// their cache pages (rope.cu:18-55, kv_cache_write.cu:10-20).
// qkv: [n_tokens, (n_heads + 2 n_kv_heads) * head_dim]; slot_map[t] = page * page_tokens +
// offset of the row's token; k_cache: [pages, n_kv_heads, page_tokens, head_dim]; v_cache is kept
// transposed, [pages, n_kv_heads, head_dim, page_tokens].  That is the plain layout, of float caches
// and of sizes the matrix-core attention kernel does not take.  A bfloat16 cache with head_dim
// (16 .. 256) and page_tokens multiples of 16 is in *fragment order*: the same tensors, but inside
// every [page_tokens, head_dim] region the elements lie as that kernel's lanes read them,
//   keys    [token / 16][dim / 8][token % 16][dim % 8]
//   values  [token / 16][dim / 16][(token % 16) / 4][dim % 16][token % 4]
// (cache_fragment_order and the two offset functions in common.h).  Every writer below and the
// matrix-core kernel apply this rule by themselves; bc4g_attention_generic reads the plain layout only.
// rotary_dim 0 switches the rotation off; write_kv 0 leaves the cache alone.  block_pairs 1: every
// head's dimensions come reordered in blocks of 16 (dimensions 8b..8b+7, then their rotation
// partners head_dim/2 + 8b..), the order the fused weight-streaming kernel works in; queries, keys and
// values then all live in that order (scores and outputs do not care, as long as all agree).
int bc4g_rope_kv_write(void* qkv, int dtype, const int32_t* positions, const int32_t* slot_map,
                       void* k_cache, void* v_cache, int n_tokens, int n_heads, int n_kv_heads,
                       int head_dim, int rotary_dim, float theta, int page_tokens, int num_pages,
                       int write_kv, int block_pairs, void* stream);

// The angles of a step, for every layer to share: table [n_tokens, rotary_dim / 2, 2] = (cos, sin)
// of position * theta^(-2i / rotary_dim).
int bc4g_rope_table(const int32_t* positions, float* table, int n_tokens, int rotary_dim, float theta, void* stream);

// bc4g_rope_kv_write for the block layout (block_pairs), rotating by a table from bc4g_rope_table
// (rotate != 0: the whole head, rotary_dim == head_dim), in 16-byte pieces.
int bc4g_rope_kv_write_blocks(void* qkv, int dtype, const float* table, const int32_t* slot_map, void* k_cache,
                              void* v_cache, int n_tokens, int n_heads, int n_kv_heads, int head_dim, int rotate,
                              int page_tokens, int write_kv, void* stream);

// Causal softmax attention of every row over its request's cached keys
// (attention_qk.cu:17-70, softmax.cu:22-43, attention_av.cu:18-46, fused).
// Row t of request s = row_seq[t] at position p = positions[t] sees keys
// max(0, p - window + 1) .. p (window 0 = all); key j lies in page
// block_table[s, j / page_tokens].  The query of row t, head h is read at qkv + t * q_stride + h * head_dim
// (the rows of the fused q|k|v product, or of a buffer of queries alone); out: [n_tokens, n_heads*head_dim].
int bc4g_attention_generic(const void* qkv, int q_stride, void* out, int dtype, const void* k_cache,
                           const void* v_cache, const int32_t* block_table, int table_stride,
                           const int32_t* row_seq, const int32_t* positions, int n_tokens,
                           int n_heads, int n_kv_heads, int head_dim, int page_tokens,
                           int num_pages, int window, float scale, void* stream);

// out[r] = lowest index of the row's maximum                      (logits_argmax.cu:22-65)
// part_v, part_i: scratch [n_rows, 64] each (the best of every slice of a row).
int bc4g_argmax(const float* logits, int32_t* out, float* part_v, int32_t* part_i, int n_rows, int vocab,
                void* stream);

// out[r] = first i with cumsum(exp((l - max) / temperature[r]))[i] > u[r] * total, walking the
// vocabulary in order (engine/src/sampler.cpp:39-61); temperature <= 0 gives the argmax.
int bc4g_sample(const float* logits, const float* temperature, const double* u, int32_t* out,
                int n_rows, int vocab, void* stream);

// out[rows[i]] = the token drawn for logits row rows[i] with top_k[i] and top_p[i]: the tokens by falling weight
// exp((l - max) / temperature[i]), lower id first among equals; the top_k likeliest (0 or >= vocab: all); of those
// the fewest whose sum reaches top_p of their total (>= 1: all); the first at which u[i] of the kept mass is passed
// (engine/src/sampler.cpp:63-104).  Not for a row with neither limit: bc4g_sample walks those in the order of the ids.
int bc4g_sample_filtered(const float* logits, const int32_t* rows, const float* temperature, const double* u,
                         const int32_t* top_k, const double* top_p, int32_t* out, int n, int vocab, void* stream);
}

extern "C" {
// bfloat16 x [m, k] (m <= 64) times bfloat16 w [n, k] transposed, weights streamed once through
// the matrix cores.  w comes packed in fragment order: [ceil(n/16)][ceil(k/32)][64][8], where lane l
// of a k-step holds row l % 16 of the block and k 8 * (l / 16) .. + 7 of the step, zeros past n and k.
// epilogue: 0 store bfloat16 [m, n]; 1 store float32; 2 add into float32;
// 3 SwiGLU: every 16 rows of w are eight gate rows and the eight up rows of the same outputs
// (n = 2 * inter), out bfloat16 [m, inter] = silu(gate) * up.
int bc4g_gemm_skinny(const void* x, const void* w, void* out, int epilogue, int m, int n, int k, void* stream);
}

extern "C" {
// Attention on the matrix cores (bfloat16, the cache in fragment order): see attention_mfma.hip.
// A wave takes q_tiles tiles of 16 rows, each tokens_per_tile tokens times the query heads of one
// key/value head.  q_tiles is 1, or 4 for head sizes up to 64 and 2 up to 128.  `form` says what a
// workgroup is, and with it what tile_start counts (tile_start[s]: the first piece of request s when
// every request's rows are cut into pieces; n_tiles their total):
//   0  four independent waves; pieces of q_tiles * tokens_per_tile tokens (a wave's)
//   1  one tile (q_tiles 1) whose waves cut the tile's keys between them and combine in LDS, for
//      few rows over long contexts; pieces of tokens_per_tile tokens
//   2  four waves with consecutive tiles of one request that walk their keys together, every key
//      tile staged in LDS once for all of them; pieces of 4 * q_tiles * tokens_per_tile tokens
// With n_splits > 1 the keys are, moreover, cut into that many parts over workgroups, whose float
// partials (part_o [n_splits, T, heads, d], part_ml [n_splits, T, heads, 2]) a second kernel
// merges into out.  A request without pieces (tile_start[s + 1] == tile_start[s]) is left out: its
// rows of out are not written, provided row_seq ([T]: each row's request) is given for the merge
// to see which rows those are -- so two launches of different forms can share one out.
// items (form 2): a work list instead of the grid's own order -- n_items entries, piece | part << 20 | parts << 24, in
// the order in which the workgroups are to start (the host puts the longest walks first and cuts a piece's keys
// into as many parts as balances the walks); row_parts [T] then says for every row into how many parts its keys
// were cut (rows with one part are written at once and left alone by the merge).
// single_rows (form 1): every request brings exactly one row, so request s is tile s and row s and the
// kernel looks nothing up before it asks for the block table and the query (a decode step).
int bc4g_attention_mfma(const void* qkv, int q_stride, void* out, float* part_o, float* part_ml, const void* k_cache,
                        const void* v_cache, const int32_t* block_table, int table_stride,
                        const int32_t* seq_start, const int32_t* seq_ctx, const int32_t* tile_start,
                        int n_seqs, int n_tiles, int n_tokens, int n_heads, int n_kv_heads, int head_dim,
                        int page_tokens, int window, float scale, int tokens_per_tile, int q_tiles,
                        int form, int n_splits, const int32_t* items, int n_items, const int32_t* row_parts,
                        int single_rows, const int32_t* row_seq, void* stream);
}

extern "C" {
// bfloat16 a [m, k] times bfloat16 w [n, k] transposed on the matrix cores, any m.
// epilogue: 0 store bfloat16; 1 store float32; 2 add into float32; 3 SwiGLU as in bc4g_gemm_skinny.
// w_packed 1: w lies in the order of the weight-streaming kernel (bc4g_gemm_skinny: [ceil(n / 16)][k / 32][64 lanes][8]),
// so that one copy of a weight serves both kernels: the kernel with operands straight into LDS reads it (k a multiple
// of 64, operands on 16-byte boundaries).  0: w lies by rows, [n, k], for the kernel that stages its tiles through
// registers (any k that is a multiple of 8).  The sums are the same bits either way.  The three entry points below
// are forms of the first kernel and take the packed weight only.
int bc4g_gemm_mfma(const void* a, const void* w, int w_packed, void* out, int epilogue, int m, int n, int k, void* stream);
// The same product with k cut into k_parts equal parts (each a multiple of 64), part p's sums stored as float32 in
// parts [k_parts, m, n]: for few rows and a long k, where one workgroup per 64 x 64 tile would walk all of k alone.
// Whoever reads the parts adds them up in order (bc4g_rmsnorm_sum).
int bc4g_gemm_mfma_parts(const void* a, const void* w, int w_packed, float* parts, int m, int n, int k, int k_parts,
                         void* stream);
// The SwiGLU product (epilogue 3) of rows that lack their RMSNorm's common factor: a = bfloat16(residual * g) [m, k] and
// the parts of the rows' sums of squares as bc4g_gemm_skinny_emit leaves them (ssq_parts [ssq_blocks][ssq_stride]); every
// row's sums are multiplied by 1 / sqrt(sum of squares / k + eps) before the activation, the parts added in the order
// of bc4g_gemm_skinny_prenormed.  k a multiple of 64, n of 16, operands on 16-byte boundaries; any m.
int bc4g_gemm_mfma_swiglu_scaled(const void* a, const float* ssq_parts, int ssq_blocks, int ssq_stride, float eps,
                                 const void* w, int w_packed, void* out, int m, int n, int k, void* stream);
// The output tile (rows, columns) bc4g_gemm_mfma (qkv 0) or bc4g_gemm_mfma_qkv (qkv 1) takes for these operands: for
// the accounting of bytes and for tests that want to meet every tile.  Launches nothing.
int bc4g_gemm_mfma_tile(const void* a, const void* w, int m, int n, int k, int qkv, int* rows, int* cols);
// The q|k|v product of many rows with rotation and cache write in its epilogue, as bc4g_gemm_skinny_qkv for few (k a
// multiple of 64, operands on 16-byte boundaries): w [n, k] holds n_heads query, n_kv_heads key and as many value heads of
// head_dim (a multiple of 16), every head's rows in blocks of eight dimensions followed by their rotation partners.  out
// [m, n_heads * head_dim] bfloat16 receives the rotated queries; keys go rotated, values as they are into the pages that
// slot_map [m] names, in the cache's layout (write_kv 0: nowhere).  table [m, head_dim / 2, 2]: cosine and sine
// of every row's position and pair (bc4g_rope_table; null: nothing is rotated).
int bc4g_gemm_mfma_qkv(const void* a, const void* w, int w_packed, void* out, const float* table, const int32_t* slot_map, void* k_cache,
                       void* v_cache, int m, int n, int k, int n_heads, int n_kv_heads, int head_dim, int page_tokens,
                       int write_kv, void* stream);
}

extern "C" {
// RMSNorm fused into the skinny product (m <= 16): x is the float residual stream (row m reads
// x[rows[m]] if rows is given), g the norm's scale (g_dtype 0 float32, 1 bfloat16); the result is
// rsqrt(mean(x^2) + eps) * sum_k bf16(x[k] g[k]) w[n, k], with the epilogues of bc4g_gemm_skinny
// except adding into a float output.
int bc4g_gemm_skinny_normed(const float* x, const int32_t* rows, const void* g, int g_dtype, float eps,
                            const void* w, void* out, int epilogue, int m, int n, int k, void* stream);
}

extern "C" {
// The query/key/value product of a decode step with rotary positions and the cache write in its
// epilogue (see gemm_skinny.hip).  x: bfloat16 [m, k] with g null (m <= 64), or the float32 residual
// stream with RMSNorm fused (g given, m <= 16).  w: [(heads + 2 kv heads) * head_dim, k] with every
// head's rows reordered in blocks of 16.  q_out: bfloat16 [m, heads * head_dim].
// With ssq_parts (g null) x is bfloat16(residual * g) and the rows' scales come from the parts, as
// in bc4g_gemm_skinny_prenormed.
int bc4g_gemm_skinny_qkv(const void* x, const void* g, int g_dtype, float eps, const float* ssq_parts, int ssq_blocks,
                         int ssq_stride, const void* w, void* q_out,
                         const int32_t* positions, const int32_t* slot_map, void* k_cache, void* v_cache,
                         int m, int k, int n_heads, int n_kv_heads, int head_dim, int rotary_dim, float theta,
                         int page_tokens, int write_kv, void* stream);
}

extern "C" {
// The adding product that prepares the RMSNorm after it: out (the float32 residual stream, [m, n])
// += x w^T; emit_x [m, n] = bfloat16(new residual * g) (g: that norm's scale, g_dtype 0 float32, 1
// bfloat16); emit_ssq [ceil(n / 16)][emit_stride]: block b's part (16 columns) of every row's sum of
// squares.  bc4g_gemm_skinny_prenormed takes such an x (k = this n) and the parts instead of a norm:
// out = rmsnorm(residual) w^T, the row's rsqrt(sum of the parts / k + eps) applied to the finished
// sums; epilogues of bc4g_gemm_skinny except the adding one.
int bc4g_gemm_skinny_emit(const void* x, const void* w, float* out, const void* g, int g_dtype, void* emit_x,
                          float* emit_ssq, int emit_stride, int m, int n, int k, void* stream);
int bc4g_gemm_skinny_prenormed(const void* x, const float* ssq_parts, int ssq_blocks, int ssq_stride, float eps,
                               const void* w, void* out, int epilogue, int m, int n, int k, void* stream);
}

extern "C" {
// What the device delivers to a kernel that does nothing else (probes.hip): bc4g_probe_read reads
// `bytes` of device memory once (sixteen 16-byte loads of a thread in flight); bc4g_probe_mfma runs
// iters x 16 back-to-back 32x32x16 bfloat16 MFMAs in every one of its workgroups' four waves
// (workgroups * 4 * iters * 16 * 32768 operations) on the caller's operands, 12 * 256 * 16 bytes of bfloat16:
// the rate depends on them (the clock follows the power that toggling operands draw).  The caller times them.
int bc4g_probe_read(const void* p, long bytes, float* sink, int workgroups, void* stream);
int bc4g_probe_mfma(const void* operands, int iters, float* sink, int workgroups, void* stream);
}

extern "C" {
// x[r, :] += y[r, :] * rsqrt(mean(y[r]^2) + eps) * w: the norm after a sublayer, added to the float residual stream
// (w float32, as it multiplies; y float32 or bfloat16).
int bc4g_rmsnorm_add(float* x, const void* y, int y_dtype, const float* w, int n_rows, int hidden, float eps, void* stream);
// out = act(in) elementwise with act(z) = softplus(p) z^2 + z / 2 for z > 0 and (1/2 + softplus(q)) (e^z - 1 - z) + z / 2
// otherwise; pq = (p, q) float32 on the device.
int bc4g_xielu(const void* in, void* out, int dtype, const float* pq, long total, void* stream);

// out[t] = h[t] + (h[t - 1] - h[t]) * mix, h = x * rsqrt(mean(x^2) + eps) * w rounded to ``dtype`` (out's and state's): an RMS
// norm of the float32 stream and the token shift behind it.  h[-1] of a request's first row of the step is its state
// [slots, hidden] (zero when the request was admitted), which then receives the h of the request's last row.  The step's
// rows are grouped by request: row_seq [T], seq_start [S + 1], seq_slots [S].  w, mix: float32 [hidden].
int bc4g_rmsnorm_shift(const float* x, const float* w, const float* mix, void* out, void* state, int dtype,
                       const int32_t* row_seq, const int32_t* seq_start, const int32_t* seq_slots, int n_rows, int hidden,
                       float eps, void* stream);

// A causal convolution over time on each channel, across steps: out[t, c] = (add_input ? in[t, c] : 0) + out_bias[c] +
// sum_j w[j, c] * input(t - taps + 1 + j)[c] (w comes by taps, [taps][channels], so that neighbouring channels lie side
// by side; its last row is the current token's), where a row's input is in[row] + in_bias (rounded to the storage type) and
// the inputs before a step's first row come from the request's state [slots, taps - 1, channels] (zero when the request
// was admitted: zeros before the sequence).  Afterwards the state holds the request's last taps - 1 inputs.  The
// step's rows are grouped by request: row_seq [T], seq_start [S + 1], seq_slots [S].  w, biases: float32.  in_row: elements
// from one row of in to the next (in may be a part of wider rows).
int bc4g_causal_conv(const void* in, int dtype, const float* in_bias, const float* w, const float* out_bias, int add_input,
                     void* out, void* state, const int32_t* row_seq, const int32_t* seq_start, const int32_t* seq_slots,
                     int n_rows, int n_seqs, int channels, int taps, long in_row, void* stream);
// The real-gated linear recurrent unit over a step's rows.  pre [T, blocks, 2 bs] (float32): the gates' sums of
// every block, Ra u_b then Ri u_b (a product per block: bc4g_heads_gemm); u, y [T, width]; decay a = exp(-8
// sigmoid(Ra u + ra_b) softplus(lam)), S_t = a S_(t-1) + sqrt(1 - a^2) sigmoid(Ri u + ri_b) u along every request's
// rows, from state [slots, width] (float32) and back into it; out[t] = S_t * gelu_tanh(y[t] + y_bias).  A request's
// rows are walked in chunks of 64 by threads of their own: chunk_a, chunk_b [S, ceil(most_rows / 64), width] and
// before [S, width] are scratch (float32); most_rows: the most rows one request brings; y_row: elements from one row of y
// to the next.
int bc4g_rglru_scan(const float* pre, const void* u, const void* y, int dtype, const float* ra_b, const float* ri_b,
                    const float* lam, const float* y_bias, void* out, float* state, float* chunk_a, float* chunk_b,
                    float* before, const int32_t* seq_start, const int32_t* seq_slots, int n_rows, int n_seqs, int most_rows,
                    int width, int blocks, long y_row, void* stream);

// Latent attention (attention_latent.hip).  q [T, heads, plain + rot] and dkv [T, rank + rot] as projected; the row's
// cache slot (slot_map[t] = page * page_tokens + offset; cache [pages, page_tokens, rank + rot]; null: nothing is
// written) receives [rmsnorm(dkv[:rank]) * g | rotate(dkv[rank:])], and q_lat [T, heads, rank + rot] (float32) the
// rotated part of every head's query in its last rot numbers.  Elements 2i and 2i + 1 of the first `dims` numbers of
// a rotated part turn by position * base^(-2i / dims): angles [T, dims / 2, 2] holds every row's cosines and sines
// (bc4g_latent_angles makes it, the angles worked out in double: once a step for all layers of one rotation).  q_row,
// dkv_row: elements from one row to the next (q and dkv may be parts of one product's rows).
int bc4g_latent_angles(const int32_t* positions, float* table, int n_rows, int dims, float base, void* stream);
int bc4g_latent_prepare(const void* q, const void* dkv, int dtype, const float* g, float eps, const float* angles,
                        const int32_t* slot_map, void* cache, float* q_lat, int n_rows, int heads, int plain, int rot,
                        int rank, int dims, long q_row, long dkv_row, void* stream);
// out[t, h, :n] = w[h] a[t, h, :k] for every head: a at a + t * a_row + h * a_head, out likewise, w [heads, n, k].
int bc4g_heads_gemm(const void* a, int a_dtype, long a_row, long a_head, const void* w, int w_dtype, void* out, int out_dtype,
                    long o_row, long o_head, int m, int n, int k, int heads, void* stream);
// out[t, h, :rank] = sum_j p_j cache[j, :rank] with p = exp(scale * q_lat[t, h] . cache[j]) over the keys the row sees
// (max(0, p - window + 1) .. p), divided by their sum plus exp(sink[h]) (sink null: no such term).  float32 in and out.
int bc4g_attention_latent(const float* q_lat, float* out, const void* cache, int dtype, const float* sink,
                          const int32_t* block_table, int table_stride, const int32_t* row_seq, const int32_t* positions,
                          int n_rows, int heads, int rank, int rot, int page_tokens, int window, float scale, void* stream);
// The same on the matrix cores for a bfloat16 cache (attention_latent_mfma.hip): rank + rot a multiple of 32 up to 576,
// rank a multiple of 16 up to 512 (bc4g_attention_latent_mfma_takes).  The step's rows are grouped by request (seq_start
// [S + 1], seq_ctx [S]: tokens cached before the step); most_tokens: the most rows one request brings.  n_splits > 1 cuts
// every walk over the keys into that many parts over workgroups, merged from part_o [n_splits, T, heads, rank] and
// part_ml [n_splits, T, heads, 2] (float32).
int bc4g_attention_latent_mfma_takes(int rank, int rot);
int bc4g_attention_latent_mfma(const float* q_lat, float* out, float* part_o, float* part_ml, const void* cache,
                               const float* sink, const int32_t* block_table, int table_stride, const int32_t* seq_start,
                               const int32_t* seq_ctx, int n_seqs, int n_tokens, int most_tokens, int heads, int rank, int rot,
                               int page_tokens, int window, float scale, int n_splits, void* stream);
}

extern "C" {
// out[t, i] = g sigmoid(slope g) (u + 1), g = min(gate, limit), u = clamp(up, -limit, limit); gu [T, 2 I] holds a row's gates,
// then its ups.
int bc4g_clamped_glu(const void* gu, void* out, int dtype, float limit, float slope, int n_rows, int inter, void* stream);

// A residual stream in n copies, x [T, n, H] float32 (streams.hip).  read: out[r] = N(sum_s read[s] x[rows ? rows[r] : r, s])
// with N(u) = (tanh(alpha u) g + b) out_scale (alpha null: out = the sum; read null: every copy counts once).  write:
// x'[t] = sum_s mix[s, t] x[s] + write[t] y for all copies at once, and with next_out also the next reader's input
// N(sum_t next_read[t] x'[t]).  fill: every copy = in.  At most 16 copies.
int bc4g_streams_read(const float* x, const int32_t* rows, const float* read, const float* alpha, const float* g, const float* b,
                      float out_scale, void* out, int out_dtype, int n_rows, int n_streams, int hidden, void* stream);
int bc4g_streams_write(float* x, const float* y, const float* mix, const float* write, const float* next_read,
                       const float* alpha, const float* g, const float* b, void* next_out, int out_dtype, int n_rows,
                       int n_streams, int hidden, void* stream);
int bc4g_streams_fill(const float* in, float* out, int n_rows, int n_streams, int hidden, void* stream);

// table [T, half, 2]: cos and sin of positions[t] * freqs[i], times amp; the angle in double (decay_scan.hip).
int bc4g_rotary_table(const int32_t* positions, const double* freqs, double amp, float* table, int n_rows, int half, void* stream);
// Per (row, head) of in [T, heads, dim] (rows in_row apart): + bias [heads, dim], RMS norm over dim with weight norm_w [dim]
// (null: none), rotation of the first 2 * half elements by the table (element i with element i + half), times factor;
// into out [T, heads, dim] (rows out_row apart) or, with slot_map (slot = page * page_tokens + offset), into a cache
// at out + page * page_stride + head * head_stride + offset * token_stride.  dim at most 256.
// The same for up to four sections of the same rows in one launch: every field as the argument of that name below.
struct bc4g_prepare_section {
  const void* in; const float* bias; const float* norm_w; const float* table; void* out; const int32_t* slot_map;
  long in_row, out_row, page_stride, head_stride, token_stride;
  int in_dtype, out_dtype, half, page_tokens, heads, dim;
  float eps, factor;
  // pairing 0: element i turns with element i + half, 1: element 2i with element 2i + 1.  unit_after 1: after the
  // rotation the head is divided by sqrt(mean(head^2) + eps), without a weight.
  // norm_rows 1: the norm before the rotation is taken over the whole row -- all heads at once, mean over heads * dim --
  // and norm_w is [heads * dim]; 0: over each head, norm_w [dim].
  int pairing, unit_after, norm_rows;
};
int bc4g_heads_prepare_many(const bc4g_prepare_section* sections, int n_sections, int n_rows, void* stream);
int bc4g_heads_prepare(const void* in, int in_dtype, long in_row, const float* bias, const float* norm_w, float eps,
                       const float* table, int half, float factor, void* out, int out_dtype, long out_row,
                       const int32_t* slot_map, int page_tokens, long page_stride, long head_stride, long token_stride,
                       int n_rows, int heads, int dim, void* stream);
// out[t, h] = o[t, h] / sqrt(mean(o[t, h]^2) + eps) (* w [vdim]) * factor * act(gate[t, h]); act 0: none, 1: silu,
// 2: sigmoid; o float32 [T, heads, vdim]; vdim at most 256.
int bc4g_heads_finish(const float* o, const float* w, float eps, float factor, const void* gate, int gate_dtype, long gate_row,
                      int act, void* out, int out_dtype, int n_rows, int heads, int vdim, void* stream);
// S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T (q_t q_scale) along every request's rows, from state
// [slots, heads, dim, vdim] (float32) and back into it; out float32 [T, heads, vdim].  a_t = head_decay[head], or with
// gate logits z [T, heads, dim]: sigmoid(z + z_bias)^inv_tau.  Requests that bring more than 32 rows are walked in
// chunks: chunk_state [chunks, heads, dim, vdim], chunk_decay [chunks, heads, dim] (float32 scratch) and chunk_base [S],
// the first chunk of every request among all chunks of requests that have two or more.  dim at most 256.
int bc4g_decay_scan(const void* q, int q_dtype, long q_row, float q_scale, const void* k, int k_dtype, long k_row,
                    const void* v, int v_dtype, long v_row, const float* head_decay, const void* z, int z_dtype, long z_row,
                    const float* z_bias, float inv_tau, float* out, float* state, float* chunk_state, float* chunk_decay,
                    const int32_t* seq_start, const int32_t* seq_slots, const int32_t* chunk_base, int n_rows, int n_seqs,
                    int most_rows, int heads, int dim, int vdim, void* stream);

// Attention with one or two score maps per query head over the same values (attention_maps.hip): q float32
// [T, heads, maps, dim]; keys [page, kv_head * maps + map, token, dim], values [page, kv_head, token, vdim]; a row at p
// sees j <= p with p - j < window or j < keep_first (window 0: all).  o = a1 - lambda a2 (one map: a1), with normalize
// divided by sqrt(mean(o^2) + eps), times factor, times act(gate) (1: silu, 2: sigmoid; gate null: none).  waves (1 to 8):
// how many waves cut one row's keys among them.  sink [heads] (or null): exp(sink) joins every map's denominator.
// far1, far2 [heads] (both or neither): far1 ln(1 + far2 (p - j)) is taken off the scaled score.
// block > 0 (then window and keep_first 0): a row sees the keys of its own block of `block` positions counted from 0,
// j <= p with j / block == p / block.  cap > 0: the scaled score becomes cap tanh(score / cap).  point [heads] (or null; then
// no sink): no softmax -- the weight of a visible key is sigmoid(score + point[head]), nothing is normalised over keys.
int bc4g_attention_maps(const float* q, long q_row, const void* k_cache, const void* v_cache, int cache_dtype,
                        const int32_t* block_table, int table_stride, const int32_t* row_seq, const int32_t* positions,
                        float lambda, int normalize, float eps, float factor, const void* gate, int gate_dtype, long gate_row,
                        int gate_act, void* out, int out_dtype, int n_rows, int n_heads, int n_kv_heads, int maps, int dim,
                        int vdim, int page_tokens, int window, int keep_first, float scale, int waves, const float* sink,
                        const float* far1, const float* far2, int block, float cap, const float* point, void* stream);

// Windowed softmax attention whose heads' weights are mixed before they meet the values (attention_talk.hip): q float32
// [T, heads, dim]; keys [page, kv_head, token, dim], values [page, kv_head, token, vdim]; a row at p sees j <= p with
// p - j < window (0: all).  score = q . k * scale - far1 ln(1 + far2 (p - j)); w_g = exp(score_g) / (sum_j exp(score_g)
// + exp(sink_g)); head h weighs the values of its own key/value head by sum_g talk[h, g] w_g; times sigmoid(gate[t, h])
// if a gate [T, heads] is given (rows gate_row apart).  sink, far1/far2 and talk ([heads, heads]) may each be null.
// heads * dim at most 8192, heads at most 64.  n_parts > 1: every row's keys are cut into that many parts, a workgroup each;
// stats (float [T, n_parts, heads, 2]) and partial (float [T, n_parts, heads, vdim]) are the room they need.
// kept (float [T, heads, kept_stride], kept_stride whole tiles of 64 that hold a row's visible keys; may be null): room for
// the first walk's scores, which the second walk then reads instead of computing them again.
int bc4g_attention_talk(const float* q, long q_row, const void* k_cache, const void* v_cache, int cache_dtype,
                        const int32_t* block_table, int table_stride, const int32_t* row_seq, const int32_t* positions,
                        const float* sink, const float* far1, const float* far2, const float* talk, const void* gate,
                        int gate_dtype, long gate_row, void* out, int out_dtype, int n_rows, int n_heads, int n_kv_heads,
                        int dim, int vdim, int page_tokens, int window, float scale, int n_parts, float* stats, float* partial,
                        float* kept, long kept_stride, void* stream);

// out[t, :] += float(table[ids[t], :]): the embedding once more, added to the stream.
int bc4g_embed_add(const void* table, int table_dtype, const int32_t* ids, float* out, int n_tokens, int hidden, int vocab,
                   void* stream);

// z -> z Phi(z) (the exact gelu, by erf), element by element; out may be the input.
int bc4g_gelu(const void* in, void* out, int dtype, long total, void* stream);

// The choice of experts for every row (moe.hip).  logits float32 [T, >= experts] (rows logits_row apart): s =
// softmax over the experts; choice = s + correction (null: s); the experts lie in `groups` equal groups of neighbours, a
// group counts by its largest choice, and only experts of the `keep` best groups can be chosen; the `top` largest
// choices win (the lower index among equals).  weights float32 [T, experts]: s of the chosen, 0 elsewhere.
// chosen int32 [T, top] (may be null).  experts at most 1024.  squash 1: s = sigmoid(logit), every expert by itself,
// instead of the softmax.  normalize 1: the chosen experts' weights are their s divided by the sum of the chosen s
// (+ 1e-20).  The weights are multiplied by `factor` last.
int bc4g_moe_route(const float* logits, long logits_row, const float* correction, float* weights, int32_t* chosen,
                   int n_rows, int experts, int groups, int keep, int top, int squash, int normalize, float factor,
                   void* stream);
// Plain units of all experts side by side, weighted: z [T, experts * ff + shared_ff] holds every expert's ff units and
// last the shared unit's; out (may be z) = weights[t, e] * gelu(z) with the exact gelu, the shared unit's as they are.
int bc4g_routed_gelu(const void* z, void* out, int dtype, const float* weights, int n_rows, int experts, int ff, int shared_ff,
                     void* stream);
// Clamped gated units of all experts side by side, weighted: gu [T, experts * 2 ff + 2 shared_ff] holds per expert its
// ff gates, then its ff ups, and last the shared unit's gates and ups; out [T, experts * ff + shared_ff] =
// weights[t, e] * g sigmoid(slope g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit), the shared unit
// (its own limit) weighted by sigmoid(shared_logit[t]) (float32, rows shared_row apart; null with shared_ff 0).
int bc4g_routed_glu(const void* gu, void* out, int dtype, const float* weights, const float* shared_logit, long shared_row,
                    float limit, float shared_limit, float slope, int n_rows, int experts, int ff, int shared_ff, void* stream);
}
