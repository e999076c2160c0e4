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

// out[r, :] = x[rows ? rows[r] : r, :] * rsqrt(mean(x^2) + eps) * w      (rmsnorm.cu:16-41)
// x is the float residual stream; out has out_dtype; w has w_dtype.
int bc4g_rmsnorm(const float* x, const int32_t* rows, const void* w, int w_dtype, void* out,
                 int out_dtype, int n_rows, int hidden, float eps, void* stream);
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
