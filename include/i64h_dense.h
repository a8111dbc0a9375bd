/* libi64hip_dense.so - C ABI of the gfx950 (MI355X) kernels for decoder models with bf16 weights and a 32-bit residual:
 * tiled Linear on the bf16 / f32 matrix cores with fused epilogues, scaled embedding, gated post-norm residual with
 * grouped RMS norm and depth mixing, latent (low-rank, shared-key) attention over a paged cache with a sliding window,
 * row sampling.  A library of its own so that a process that serves such a model builds and loads nothing else.
 *
 * Conventions are those of libi64hip.so (include/i64h.h): raw device pointers, caller-allocated outputs, no allocation
 * and no synchronisation inside, 0 on success, the reason of a failure in i64h_last_error() of THIS library.
 * Descriptor structs are passed by host pointer and read before the call returns.
 */
#ifndef I64H_DENSE_H
#define I64H_DENSE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

const char* i64h_last_error(void);
int i64h_version(void);
int i64h_device_check(void);

/* ---- Linear ------------------------------------------------------------------------------------------------------------
 * C[b][m, n] = epilogue( sum_k A[b][row(m), k] * W[b][n, k] ),  b < batch (one launch; blockIdx.z is the batch index).
 *   A fp32, row stride lda, batch b starts a_batch * b elements further (a column block of a wider matrix);
 *   row(m) = a_rows ? a_rows[m] : m;  W bf16 [N, K] row-major, batch stride w_batch elements;  C fp32, row stride ldc,
 *   batch stride c_batch.
 * exact = 0: A is rounded to bf16 (nearest even) while it is staged, products on v_mfma_f32_16x16x32_bf16, fp32 sums.
 * exact = 1: W is widened to fp32 while it is staged, products on v_mfma_f32_16x16x4_f32: true 32-bit arithmetic.
 * epilogue: I64H_EPI_STORE; I64H_EPI_GELU_MUL: gelu_tanh(A W^T) * (A W2^T) with W2 = W + N * K (gate rows, then up rows);
 *   I64H_EPI_MUL_SIGMOID: * sigmoid(E[b][m, n]) (E fp32, row stride lde, batch stride e_batch);
 *   I64H_EPI_SOFTCAP: cap * tanh(. / cap).
 * Any M, N, K >= 1; 16-byte loads are used where strides and addresses allow, element loads otherwise.
 * Launches with M <= I64H_SKINNY_ROWS take a weight-streaming form (one wave per output column group). */
#define I64H_EPI_STORE 0
#define I64H_EPI_GELU_MUL 1
#define I64H_EPI_MUL_SIGMOID 2
#define I64H_EPI_SOFTCAP 3
#define I64H_SKINNY_ROWS 8
typedef struct {
    const float* A;
    int64_t lda;
    const int32_t* a_rows;
    const void* W;
    float* C;
    int64_t ldc;
    int64_t M;
    int32_t N, K;
    int32_t batch;
    int64_t a_batch, w_batch, c_batch;
    int32_t exact;
    int32_t epilogue;
    const float* E;
    int64_t lde, e_batch;
    float softcap;
} i64h_linear;
int i64h_linear_run(const i64h_linear* d, void* stream);

/* out[t, :] = float(table[ids[t], :]) * scale; table bf16 [V, W]; ids outside [0, V) are clamped. */
int i64h_embed_scaled(const int64_t* ids, const void* table_bf16, float scale, float* out, int64_t n, int32_t W, int64_t V, void* stream);

/* ---- gated post-norm residual + grouped RMS norm + depth mix, one launch per sublayer --------------------------------------
 * v = alpha * x[row(m)] + g * y[m],  g = gate_pre ? sigmoid(gate_pre[m] + gate_bias) : 1,  y == NULL: v = alpha * x;
 * out[m] = v / sqrt(mean over the group of v^2 + eps) * norm_w, the W columns cut into `groups` equal consecutive parts;
 * with mix_w != NULL the row is also stored at hist[hist_index][m] and
 *   mix_out[m] = sum_{j < hist_index} mix_w[j] * hist[j][m] + mix_w[hist_index] * out[m]        (hist fp32 [*, n, W]).
 * x_rows (may be NULL) gathers input rows (the final norm of the rows whose logits are wanted).  All math fp32. */
typedef struct {
    const float* x;
    const int32_t* x_rows;
    const float* y;
    int64_t ldy;
    const float* gate_pre;
    int64_t ldg;
    const float* gate_bias;
    float alpha;
    const float* norm_w;
    int32_t groups;
    float eps;
    float* out;
    float* hist;
    int32_t hist_index;
    const float* mix_w;
    float* mix_out;
    int64_t n;
    int32_t W;
} i64h_postnorm;
int i64h_gated_postnorm(const i64h_postnorm* d, void* stream);

/* ---- latent attention ----------------------------------------------------------------------------------------------------
 * One cached row per token and layer: [kv_rank latent values | rot_dim rotated key values], shared by all heads, in a paged
 * cache (num_blocks, block_size, kv_rank + rot_dim) of fp32 (cache_dtype 0) or bf16 (2); the row of (slot, position) is
 * block_table[slot * max_blocks_per_seq + position / block_size] * block_size + position % block_size.
 *
 * i64h_latent_prep, per token t of the projection rows P (fp32, row stride ldp):
 *   latent = P[t, dkv_off : +kv_rank] / sqrt(mean^2 + eps) * c_norm_w           -> cache row, columns [0, kv_rank)
 *   key    = rotate(P[t, dkv_off + kv_rank : +rot_dim], position)               -> cache row, columns [kv_rank, +rot_dim)
 *   Q[t, h, kv_rank : +rot_dim] = rotate(P[t, q_off + h * (dim + rot_dim) + dim : +rot_dim], position)   for every head h
 * rotate: the first rot_dims values in interleaved pairs (2i, 2i+1) by the angle position * inv_freq[i] (fp32 product,
 * full-range sine / cosine), the rest unchanged.  Q fp32 [n, heads, kv_rank + rot_dim]; its first kv_rank columns per head
 * (the query carried into latent space) are written by the caller's Linear. */
typedef struct {
    const float* P;
    int64_t ldp;
    int32_t q_off, dkv_off;
    int32_t heads, dim, rot_dim, kv_rank, rot_dims;
    const float* c_norm_w;
    float eps;
    const float* inv_freq;
    const int32_t* positions;
    const int32_t* slot_ids;
    const int32_t* block_table;
    int32_t max_blocks_per_seq, block_size;
    void* cache;
    int32_t cache_dtype;
    float* Q;
    int64_t n;
} i64h_latent_prep_args;
int i64h_latent_prep(const i64h_latent_prep_args* d, void* stream);

/* i64h_latent_attn: row t (sequence slot_ids[t], position p = positions[t]) sees the cached rows j of its sequence with
 * 0 <= p - j < window (window <= 0: every j <= p);  s_j = scale * Q[t, h, :] . row_j;  ordinary softmax over the visible j;
 * out[t, h, :kv_rank] = sum_j w_j * row_j[:kv_rank].  Scores, weights and sums in fp32.  out fp32 [n, heads, kv_rank].
 * mode 1: one wave per (row, head), fp32 products, any sizes and cache type.  Modes 0 / 2 / 3 take the matrix-core form when the cache
 * is bf16, kv_rank % 16 == 0 and <= 256, (kv_rank + rot_dim) % 8 == 0 and <= 320 (the row form otherwise): 2 (and 0) one wave per token
 * and group of 16 heads (rows that are one per sequence), 3 one wave per 16 consecutive rows and head (portions of prompts; rows of
 * different sequences in one tile are handled run by run). */
typedef struct {
    const float* Q;
    const void* cache;
    int32_t cache_dtype;
    const int32_t* block_table;
    int32_t max_blocks_per_seq, block_size;
    const int32_t* slot_ids;
    const int32_t* positions;
    int32_t window;
    float scale;
    float* out;
    int64_t n;
    int32_t heads, kv_rank, rot_dim;
    int32_t mode;
    int32_t splits;      /* mode 2: every token's keys are dealt to this many waves (tiles of 32 keys in turn) and merged by a second launch */
    float* workspace;    /* i64h_latent_attn_workspace_floats(n, heads, kv_rank, splits) floats when splits > 1 (NULL: no split) */
} i64h_latent_attn_args;
int i64h_set_latent_attn_decode_form(int32_t on); /* tuning / test knob: 1 (default) = mode 2 launches run the kernel that requests a tile's fragments a tile ahead; 0 = the general matrix-core kernel; same results up to summation order */
int64_t i64h_latent_attn_workspace_floats(int64_t n, int32_t heads, int32_t kv_rank, int32_t splits);
int i64h_latent_attn(const i64h_latent_attn_args* d, void* stream);

/* ---- sampling --------------------------------------------------------------------------------------------------------------
 * out[r] = a token drawn from row r of logits fp32 [rows, V]: temperature[r] <= 0 -> the first index of the maximum (greedy);
 * otherwise from softmax(logits / temperature) restricted to the top_k[r] largest (top_k <= 0: all) and then to the smallest
 * set of largest probabilities whose sum reaches top_p[r] (top_p >= 1: all), using the uniform number u[r] in [0, 1). */
int i64h_sample_rows(const float* logits, int64_t* out, int64_t rows, int32_t V, const float* temperature, const int32_t* top_k,
                     const float* top_p, const float* u, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* I64H_DENSE_H */
