/* C-ABI of libpromptcache_blocks.so: building-block kernels (gfx950) for decoder designs that keep plain row-major bf16 or fp32
 * tensors and an fp32 residual stream.  Built from prompt-cache_amd/csrc/pb_*.hip; bound by promptcache_amd/_blocks.py.
 *
 * Conventions: every entry point returns PCB_OK or a negative code (pcb_last_error_string() says why), validates its arguments
 * on the host before it launches anything, launches on `stream` (a hipStream_t) without synchronising, and takes device
 * pointers unless a parameter says otherwise.  `dtype` selects the element type E of weights, activations and cached keys:
 * PCB_BF16 (products on the bf16 matrix cores, fp32 accumulation) or PCB_F32 (fp32 matrix cores: true 32-bit products).
 * Residual streams, norms, scores, softmax weights, router logits and reductions are fp32 in both.
 */
#ifndef PROMPTCACHE_BLOCKS_H
#define PROMPTCACHE_BLOCKS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PCB_ABI_VERSION 1
#define PCB_OK 0
#define PCB_ERR_ARG (-2001)
#define PCB_ERR_HIP_BASE (-3000)

#define PCB_BF16 0
#define PCB_F32 1

int pcb_version(void);
const char* pcb_last_error_string(void);

/* out[r][:] = fp32(table[ids[r]][:]) : the embedding rows as the first residual stream. */
int pcb_embed_rows(const void* table, int32_t dtype, const int32_t* ids, float* out, int32_t n_rows, int32_t width, int32_t vocab,
                   void* stream);

/* Weighted sum of residual streams + up to two RMS norms of the result, one workgroup per row:
 *   x[r]    = n_terms > 0 ? sum_j coef[j] * hist[j][src(r)] : hist[0][src(r)]       src(r) = rows ? rows[r] : r
 *   out1[r] = x[r] / sqrt(mean(x[r]^2) + eps) * gain1                               (E; likewise out2 with gain2 when given)
 * x_out (fp32 [n_rows][width]) receives x when given. */
typedef struct pcb_mix_norm_args {
    uint32_t struct_bytes;
    int32_t dtype;
    const float* hist;
    int64_t hist_stride; /* elements between stream j and stream j + 1 */
    const float* coef;
    int32_t n_terms;
    float* x_out;
    const int32_t* rows;
    const float* gain1;
    void* out1;
    const float* gain2;
    void* out2;
    float eps;
    int32_t n_rows;
    int32_t width;
} pcb_mix_norm_args;
int pcb_mix_norm(const pcb_mix_norm_args* a, void* stream);

/* Y = A W^T (+ bias), A = gathered / scaled rows of X.  W is [N][K] row-major (nn.Linear layout).
 *
 * rows      A row r = row_scale[r] * X[row_src ? row_src[r] : r]   (the scaled row is rounded to E)
 * groups    n_groups > 0: rows [group_off[g], group_off[g+1]) use W + g * w_group_stride (and W2 likewise); M is then an upper
 *           bound of group_off[n_groups] (the launch covers it; the kernel reads the offsets)
 * epilogue  PCB_EPI_STORE      v = acc + bias[n]
 *           PCB_EPI_SILU_MUL   v = silu(acc) * acc2, acc2 = A W2^T   (gated unit; no bias)
 *           PCB_EPI_SCALE_ADD  v = (base ? base[m][n] : y32[m][n]) + col_scale[n] * (acc + bias[n]), stored fp32 (ldy)
 * output    STORE / SILU_MUL: element type E, or fp32 when out_f32; row m goes to y + (row_dst ? row_dst[m] : m) * ldy.
 *           split_n > 0 (STORE only): columns n >= split_n go to y2 instead: row m at y2 + row_off2[m], column c = n - split_n at
 *           (c / head_dim2) * head_stride2 + c % head_dim2  (a projection that appends its second part to a key cache). */
#define PCB_EPI_STORE 0
#define PCB_EPI_SILU_MUL 1
#define PCB_EPI_SCALE_ADD 2
typedef struct pcb_linear_args {
    uint32_t struct_bytes;
    int32_t dtype;
    int32_t epilogue;
    const void* x;
    int64_t ldx;
    const int32_t* row_src;
    const float* row_scale;
    const void* w;
    const void* w2;
    int64_t ldw;
    const void* bias; /* [N] E, may be null */
    int32_t M, N, K;
    const int32_t* group_off;
    int32_t n_groups;
    int64_t w_group_stride;
    void* y;
    int64_t ldy;
    int32_t out_f32;
    const int32_t* row_dst;
    const float* base;
    int64_t ldbase;
    const float* col_scale; /* [N] fp32 */
    int32_t split_n;
    void* y2;
    const int64_t* row_off2;
    int32_t head_dim2;
    int64_t head_stride2;
} pcb_linear_args;
int pcb_linear(const pcb_linear_args* a, void* stream);

/* out[r][f] = c0 * z/rms(z) + c1 * z^2/rms(z^2) + c2 * z^3/rms(z^3) + c3 over row r of z (fp32 [n_rows][ff]), rms with eps inside the
 * root; coef = {c0, c1, c2, c3} fp32 on the device; out is E. */
int pcb_polynorm(const float* z, const float* coef, void* out, int32_t dtype, float eps, int32_t n_rows, int32_t ff, void* stream);

/* Top-k choice of a sigmoid router: logits fp32 [n_rows][n_experts] (the router projection, e.g. pcb_linear with an fp32
 * destination), score = sigmoid(logit), the `top` largest scores win (ties: the lower index).  pair p = r * top + k: expert[p],
 * weight[p] = the score itself (not renormalised). */
int pcb_router_topk(const float* logits, int32_t n_rows, int32_t n_experts, int32_t top, int32_t* expert, float* weight, void* stream);

/* Bucket the pairs by expert: group_off[n_experts + 1], and per bucketed row its token (row_src), its pair (row_dst) and its
 * weight (row_scale).  One workgroup; n_pairs <= 1 << 20. */
int pcb_moe_plan(const int32_t* expert, const float* weight, int32_t n_pairs, int32_t top, int32_t n_experts, int32_t* group_off,
                 int32_t* row_src, int32_t* row_dst, float* row_scale, void* stream);

/* y[r][n] += col_scale[n] * sum_k pair_out[r * top + k][n]  (fixed order over k). */
int pcb_moe_combine(const float* pair_out, const float* col_scale, float* y, int32_t n_rows, int32_t width, int32_t top, void* stream);

/* Causal attention over a slot-addressed key cache whose values ARE the keys (one plane), with optional
 *   - linear distance bias: score_h -= slopes[h] * (i - j)
 *   - cross-head mixing of the biased scores before the softmax: score_h <- sum_g talk[h][g] * score_g
 *   - sliding window: key j is seen by query i iff 0 <= i - j < window (window <= 0: all earlier keys)
 *   - sink: one more term exp(0) in the softmax denominator that carries no value
 * Queries are flat rows; tile t = {slot, first query position, query rows (<= 16), first flat row} (int32 x 4, device).  The
 * cache holds key j of kv head g of slot s at cache + s * slot_stride + g * head_stride + j * head_dim and must already contain
 * the queries' own keys.  Query head h reads kv head h / (H / Hkv).  scratch: fp32 [n_tiles * 16][H][band] with
 * band = pcb_attn_talk_band(window, max_kv_len) (the distances a row can see, padded); out is E [rows][ldo], head h at column
 * h * head_dim. */
typedef struct pcb_attn_talk_args {
    uint32_t struct_bytes;
    int32_t dtype;
    const void* q;
    int64_t ldq;
    const int32_t* tiles;
    int32_t n_tiles;
    const void* cache;
    int64_t slot_stride;
    int64_t head_stride;
    int32_t H, Hkv, head_dim;
    float scale;
    int32_t window;
    int32_t max_kv_len; /* no tile reaches a key position >= this */
    const float* slopes; /* [H] or null */
    const float* talk;   /* [H][H] or null */
    int32_t sink;
    float* scratch;
    int64_t scratch_floats;
    void* out;
    int64_t ldo;
    const int32_t* tiles64; /* optional: the same rows cut into tiles of up to 64 queries (same record) for the value pass */
    int32_t n_tiles64;
    int32_t max_tile_rows; /* an upper bound of the tiles' query rows when the host knows one (0: unknown); <= 4 selects the
                              value pass written for decoding */
} pcb_attn_talk_args;
int32_t pcb_attn_talk_band(int32_t window, int32_t max_kv_len);
int pcb_attn_talk(const pcb_attn_talk_args* a, void* stream);

#ifdef __cplusplus
}
#endif
#endif
