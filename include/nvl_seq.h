/* C ABI of libnvl_seq.so: gfx950 kernels for models whose layers carry per-sequence state beside (or instead of) a
 * full-attention KV cache: scalar-weight RMS norms on a 32-bit residual stream, sinusoidal embeddings, stateful causal
 * convolutions, the real-gated linear recurrence, the state-space-duality recurrence, sliding-window paged attention
 * with any head size, and the activations that go with them.
 *
 * Conventions (as include/nvl.h): raw device pointers, sizes, a hipStream_t as void*; enqueue-only (no allocation, no
 * synchronisation => hipGraph-capturable); 0 on success, negative code + nvs_last_error() otherwise; arguments are
 * validated on the host. `dtype` names the element type of ACTIVATION and WEIGHT tensors (NVS_BF16 / NVS_F32); what is
 * typed float* is 32-bit whatever `dtype` says: the residual stream, recurrent and convolution state, gate inputs.
 *
 * Batch layout ("portions"): a step holds `nseq` portions of sequences, packed token-major. cu_q[s] .. cu_q[s+1] are the
 * token rows of portion s; ctx0[s] is the number of tokens of that sequence processed by EARLIER steps (the position of
 * the portion's first token); slot[s] is the sequence's state slot; tseq[t] is the portion a token row belongs to.
 * A portion with ctx0 == 0 starts from zero state whatever its slot holds (slots are reused without clearing). */
#ifndef NVL_SEQ_H
#define NVL_SEQ_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define NVS_BF16 0
#define NVS_F32 1
#define NVS_OK 0
#define NVS_EINVAL -1
#define NVS_ELAUNCH -2

int nvs_abi_version(void);
const char* nvs_last_error(void);

/* x[t, :] = table[ids[t], :] * scale + sinusoid(pos[t]); entry 2i = sin(pos * base^(-2i/width)), 2i+1 = cos of the same
 * angle (angles in 32-bit from an exact integer position); base == 0: no sinusoid. xh (nullable): copy of x in `dtype`. */
int nvs_embed_sinusoid(const void* table, int dtype, const int64_t* ids, const int64_t* pos, int64_t n, int width,
                       float scale, float base, float* x, void* xh, void* stream);

/* Residual update with the norm on the sublayer OUTPUT: x += g * rms(m), g one number (device, `dtype`).
 * With m2 != NULL the sublayer output is the mean of two branches, each RMS-normed with a per-channel weight first:
 * m' = (rms(m) * w1 + rms(m2) * w2) / 2, x += g * rms(m'). rms(v) = v / sqrt(mean(v^2) + eps). xh (nullable): x in `dtype`. */
int nvs_norm_residual(const void* m, const void* m2, const void* w1, const void* w2, const void* g, int dtype, int64_t n,
                      int width, float eps, float* x, void* xh, void* stream);

/* Input-side norm on the residual stream, with the adds that precede it: x[t, :] += a_mult * a[t, :] + b[t, :] (a in `dtype`,
 * b 32-bit, either may be NULL), then out[t, :] = group_rms(x[t, :]) * w: every one of `groups` equal consecutive parts of the
 * row is divided by its own sqrt(mean(part^2) + eps); with center != 0 the part's mean is taken off first and it is divided by
 * sqrt(mean of squared deviations + eps) (a layer norm without bias). out == NULL: the adds only. With rows != NULL nothing is
 * added and out[r, :] is the norm of x[rows[r], :]. out and w in `dtype`. */
int nvs_add_group_norm(float* x, const void* a, float a_mult, const float* b, const int32_t* rows, int64_t nrows, const void* w,
                       int dtype, int width, int groups, float eps, int center, void* out, void* stream);

/* Norms on both sides of a sublayer, on the 32-bit residual. The sublayer's output y[t, :] = a_mult * a[t, :] + a2_mult * a2[t, :]
 * (a2 may be NULL) is divided by its root mean square and multiplied by (w_off + wa), and added: x[t, :] += rms(y) * (w_off + wa);
 * then out[t, :] = rms(x[t, :]) * (w_off + w), the next sublayer's input. a == NULL: nothing is added; out == NULL: the add only.
 * w_off = 1 serves weights that are stored as their distance from one. With rows != NULL nothing is added and out[r, :] is the
 * norm of x[rows[r], :]. a, a2, wa, w, out in `dtype`; every sum in 32-bit. */
int nvs_sandwich_norm(float* x, const void* a, float a_mult, const void* a2, float a2_mult, const void* wa, const int32_t* rows,
                      int64_t nrows, const void* w, float w_off, int dtype, int width, float eps, void* out, void* stream);

/* out[i] = cap * tanh(in[i] * scale / cap), or in[i] * scale with cap <= 0; in `dtype`, out 32-bit. */
int nvs_scale_softcap(const void* in, int dtype, float scale, float cap, int64_t numel, float* out, void* stream);

/* out[r, :] = g * rms(x[rows[r], :]) in `dtype` (rows == NULL: row r). */
int nvs_scalar_norm_rows(const float* x, const int32_t* rows, int64_t nrows, int width, const void* g, int dtype, float eps,
                         void* out, void* stream);

/* xIELU, elementwise: z > 0: softplus(p) z^2 + beta z; z <= 0: (beta + softplus(q)) (exp(z) - 1 - z) + beta z. pq = {p, q}
 * (device, `dtype`). In place allowed. */
int nvs_xielu(const void* in, const void* pq, float beta, int dtype, int64_t numel, void* out, void* stream);

/* Per-channel causal convolution over the packed portions, continuing each sequence from its state.
 * in: [n, channels] with row stride in_stride (elements, `dtype`); w [channels, taps] (last tap = current token), b [channels]
 * (nullable); act: 0 none, 1 SiLU. state [nslots, taps-1, channels] (32-bit) holds each sequence's last taps-1 inputs and
 * is advanced by the call (a second launch, after the outputs have been computed). out [n, channels] in out_dtype: NVS_F32, or
 * `dtype` itself (sums are 32-bit either way). */
int nvs_causal_conv(const void* in, int64_t in_stride, int dtype, const void* w, const void* b, int channels, int taps, int act,
                    const int32_t* cu_q, const int32_t* ctx0, const int32_t* slot, const int32_t* tseq, int nseq, int64_t n,
                    float* state, void* out, int out_dtype, void* stream);

/* Real-gated linear recurrence. gates [blocks, n, 2*bw] (32-bit): per block the pre-activations of the recurrence gate
 * (first bw) and of the input gate (last bw), biases included; u [n, C] 32-bit; ypre [n, C] (row stride y_stride) the
 * pre-activation of the output branch (GELU-tanh is applied here); lam [C]. For every channel, token by token:
 *   a = exp(-c * sigmoid(gr) * softplus(lam)),  S = a S + sqrt(1 - a^2) * sigmoid(gi) * u,  out = S * gelu_tanh(ypre).
 * S [nslots, C] 32-bit, advanced. out [n, C] `dtype`. Long portions of a step with few (portion, channel) threads are scanned
 * in segments, twice, in `ws` (nvs_rglru_scan_workspace floats; NULL: never), as nvs_ssd_scan below explains; max_q = the
 * longest portion of the step. */
int64_t nvs_rglru_scan_workspace(int channels, int nseq, int64_t max_q);
int nvs_rglru_scan(const float* gates, const float* u, const void* ypre, int64_t y_stride, int dtype, const void* lam, float c,
                   int channels, int blocks, const int32_t* cu_q, const int32_t* ctx0, const int32_t* slot, int nseq, int64_t n,
                   int64_t max_q, float* S, void* out, float* ws, int64_t ws_floats, void* stream);

/* State-space-duality recurrence, recurrent form. xbc [n, inner + 2*G*N] 32-bit (x | B | C after convolution + SiLU),
 * dt: column dt_col .. dt_col + heads of proj [n, proj_stride] (`dtype`); dt_bias, A_log, D [heads] (`dtype`). Per head h
 * (group h / (heads / G)), token by token: dt = softplus(dt + dt_bias), S = exp(-exp(A_log) dt) S + dt B x^T,
 * y = S^T C + D x. State memory is [nslots, heads, P, N] (n fastest), 32-bit, advanced. y [n, heads * P] 32-bit.
 * A workgroup walks a (portion, head)'s tokens one after the other; when such pairs are few and portions long (max_q = the
 * longest portion of the step), portions are cut into segments that are scanned twice — local states from zero, then from
 * the combined states of the segments before — in `ws` (nvs_ssd_scan_workspace floats; NULL or 0: never segmented). */
int64_t nvs_ssd_scan_workspace(int heads, int P, int N, int nseq, int64_t max_q);
int nvs_ssd_scan(const float* xbc, const void* proj, int64_t proj_stride, int64_t dt_col, int dtype, const void* dt_bias,
                 const void* A_log, const void* D, int heads, int P, int N, int G, const int32_t* cu_q, const int32_t* ctx0,
                 const int32_t* slot, int nseq, int64_t n, int64_t max_q, float* S, float* y, float* ws, int64_t ws_floats,
                 void* stream);

/* The decaying outer-product recurrence of linear ("lightning") attention, in 32-bit: per head h, token by token,
 *   S = decay[h] S + k v^T,  o = S^T q,  with q, k (dk per head) and v (dv per head) = SiLU of columns q_col / k_col / v_col
 * (+ head * size) of proj [n, proj_stride] (`dtype`); SiLU is applied here. decay [heads] 32-bit. State memory is
 * [nslots, heads, dv, dk] (dk fastest), advanced. y [n, heads * dv] 32-bit. The walk, the segments for long portions and the
 * workspace (nvs_ssd_scan_workspace(heads, dv, dk, nseq, max_q)) are those of nvs_ssd_scan. */
int nvs_decay_scan(const void* proj, int64_t proj_stride, int64_t v_col, int64_t k_col, int64_t q_col, int dtype, const float* decay,
                   int heads, int dk, int dv, const int32_t* cu_q, const int32_t* ctx0, const int32_t* slot, int nseq, int64_t n,
                   int64_t max_q, float* S, float* y, float* ws, int64_t ws_floats, void* stream);

/* The matrix memory with exponential gates, in 32-bit. Per head h and token, from the gate pre-activations zi, zf (columns i_col + h,
 * f_col + h of proj [n, proj_stride], `dtype`, plus i_bias[h] / f_bias[h]): i = cap tanh(zi / cap), f = logsigmoid(cap tanh(zf / cap));
 * with the running maximum m (0 at a sequence's start): m' = max(f + m, i),
 *   S <- exp(f + m - m') S + exp(i - m') k v^T,   n <- exp(f + m - m') n + exp(i - m') k,
 * q (times q_scale), k (dk per head) and v (dv per head) being columns q_col / k_col / v_col (+ head * size) of proj, read as they
 * are. y [n, heads * dv] receives the numerators S^T q, den [n, heads] the divisors max(|n . q|, exp(-m')) + 1e-6 (both 32-bit; the
 * norm that follows divides: nvs_gated_group_norm's `den`). State: S [nslots, heads, dv + 1, dk] (row dv is n; dk fastest) and
 * M [nslots, heads], advanced. The walk is nvs_ssd_scan's, one workgroup per (portion, head), and so are the segments for long
 * portions (`ws`: nvs_gated_memory_scan_workspace floats; NULL: never; a segment's local state is combined with what came before
 * it through its own maximum and the sum of its log forget gates). dv <= 256. */
int64_t nvs_gated_memory_scan_workspace(int heads, int dk, int dv, int nseq, int64_t max_q);
int nvs_gated_memory_scan(const void* proj, int64_t proj_stride, int64_t v_col, int64_t k_col, int64_t q_col, int64_t i_col, int64_t f_col,
                          int dtype, const void* i_bias, const void* f_bias, float cap, float q_scale, int heads, int dk, int dv,
                          const int32_t* cu_q, const int32_t* ctx0, const int32_t* slot, int nseq, int64_t n, int64_t max_q, float* S,
                          float* M, float* y, float* den, float* ws, int64_t ws_floats, void* stream);

/* order 0: out = group_rms(y * silu(z)) * w: the gate first, then each of `groups` equal parts of a row by its own root mean
 * square. order 1: out = group_rms(y) * w * sigmoid(z): the norm first. y [n, inner] 32-bit; z [n, inner] with row stride z_stride
 * (`dtype`); w [inner]; out [n, inner] `dtype`. den (nullable, order 1 only) [n, groups] 32-bit: every entry of group g of row t is
 * divided by den[t, g] first. */
int nvs_gated_group_norm(const float* y, const void* z, int64_t z_stride, int dtype, const void* w, int inner, int groups,
                         float eps, int order, int64_t n, const float* den, void* out, void* stream);

/* Key norm / rotation + paged K/V store. Rotation (rot_dims > 0, after the norm): entries (2i, 2i+1), i < rot_dims / 2, of every key head turn by
 * the angle pos[t] * rot_freq[i] (32-bit): (u, v) -> (u cos - v sin, v cos + u sin); the other entries pass. k [n, G, d] / v [n, G, dv] are column ranges of one projection output (row stride `stride`,
 * `dtype`). k is RMS-normed over d with weight knorm [d] (NULL: stored as is). Token t goes to cache slot slots[t] (< 0:
 * skipped); slot = page * block_size + offset. Caches, `dtype`: k_cache [slot][G][d]; v_cache [page][G][dv][block_size] — values
 * are kept TRANSPOSED inside a page, so that a column's consecutive tokens are contiguous (the matrix-core attention reads 8 at a
 * time). */
int nvs_knorm_kvstore(const void* k, const void* v, int64_t stride, int dtype, const void* knorm, float eps, int G, int d, int dv,
                      int block_size, const int32_t* slots, const int64_t* pos, const float* rot_freq, int rot_dims, int64_t n,
                      void* k_cache, void* v_cache, void* stream);

/* Locally masked softmax attention over the paged cache, one query per token row, any d, dv <= 1024.
 * q [n, H, d] (row stride q_stride), RMS-normed per head with qnorm [d] here (NULL: none), then rotated like the keys
 * (rot_dims, rot_freq; 0: not). Token t of portion s sits at position p = ctx0[s] + (t - cu_q[s]) and sees keys j with
 * 0 <= p - j < window (window > 0), or the keys j <= p of its own block, floor(j / chunk) == floor(p / chunk) (chunk > 0; blocks
 * are counted from position 0 of the sequence), or every j <= p (both 0), read through block_tables [nseq, bt_stride]. score = q.k * scale
 * * (1 + qt_coef * ln(floor((p + 1) / qt_every) + 1)) (qt_every == 0: no such factor), softmax in 32-bit; with sink != NULL ([H],
 * 32-bit) the denominator of head h also holds exp(sink[h]), a score that is not scaled and has no value. gate (nullable) [n, H*dv] with row stride
 * gate_stride: out *= sigmoid(gate); with gate_per_head != 0 the gate is [n, H], one entry for all columns of a head. out [n, H*dv] `dtype`.
 * bf16 with d % 8 == 0, d and dv <= 256 and block_size % 8 == 0 runs on the matrix cores (16 queries per wavefront — 16 positions of
 * one head, or in steps of single tokens with 8 or more query heads per kv head 16 heads at one position; the weights enter the
 * second product as bf16); everything else, and every float32 call, takes the scalar kernel (one wavefront per query). */
int nvs_window_attn(const void* q, int64_t q_stride, const void* qnorm, float eps, const void* gate, int64_t gate_stride, int gate_per_head, int dtype,
                    const void* k_cache, const void* v_cache, const int32_t* block_tables, int64_t bt_stride, int block_size,
                    const int32_t* cu_q, const int32_t* ctx0, const int32_t* tseq, int nseq, int64_t n, int H, int G, int d, int dv,
                    float scale, int window, int chunk, const float* rot_freq, int rot_dims, const float* sink, float qt_coef, int qt_every,
                    void* out, void* stream);

/* Gated feed-forward activation on a fused [gate | up] projection: gu [n, 2 ff] with row stride `stride` -> out [n, ff] (`dtype`).
 * kind 0: silu(g) u. kind 1: g' = min(g, limit), u' = clamp(u, -limit, limit), out = g' sigmoid(alpha g') (u' + 1).
 * kind 2: no gate at all, gu [n, ff]: out = 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))). */
int nvs_glu_act(const void* gu, int64_t stride, int dtype, int ff, int kind, float limit, float alpha, int64_t n, void* out, void* stream);

/* Routing of a mixture of experts, 32-bit. z [n, total] (row stride z_stride): router logits of all `total` entries.
 * s = softmax(z) (score 0) or sigmoid(z) (score 1); choice score c = s + correction (NULL: none). Entries form `count` equal groups of neighbours; a group's score
 * is its largest c, and only entries of the `keep` best groups can be chosen. The `top` entries with the largest c are chosen:
 * ids [n, top]; wts [n, top] = s[chosen] / (sum of them + 1e-20) * scale, or s[chosen] * scale with renorm == 0. Ties go to
 * the lower index. */
int nvs_moe_route(const float* z, int64_t z_stride, const float* correction, int64_t n, int total, int top, int count, int keep, float scale,
                  int score, int renorm, int32_t* ids, float* wts, void* stream);

/* Routing without a router: ids[t, k] = table[tokens[t], k] (table [vocab, top], int32; a row's entries differ), wts[t, k] = weight. */
int nvs_moe_table_route(const int64_t* tokens, const int32_t* table, int64_t n, int top, float weight, int32_t* ids, float* wts, void* stream);

/* Sort the pairs (token, choice) by expert. Pairs whose id >= experts have no rows (pass-through entries). Every expert's rows are
 * padded to whole tiles of tm (16, 64 or 128) rows; cap = nvs_moe_rows(n * top, experts, tm) rows are laid out.
 * tile_expert [cap / tm]: the tile's expert or -1; row_token [cap]: the row's token or -1; pair_row [n * top]: the pair's row or -1. */
int64_t nvs_moe_rows(int64_t pairs, int experts, int tm);
int nvs_moe_plan(const int32_t* ids, int64_t n, int top, int experts, int tm, int32_t* tile_expert, int32_t* row_token, int32_t* pair_row,
                 void* stream);

/* Grouped product over the planned rows: out[r, :] = W[expert of r] x(r). mode 1: W [experts, 2 nout, K] (gate rows, then up rows),
 * x(r) = X[row_token[r], :], out = silu(gate) * up; mode 0: W [experts, nout, K], x(r) = X[r, :]; mode 2: W [experts, nout, K],
 * x(r) = X[row_token[r], :], out = max(W x, 0)^2 (an ungated expert's first product). X, W, out in `dtype`; bf16 with
 * K % 8 == 0 and ldx % 8 == 0 runs on the matrix cores (tm 128: LDS-tiled, for steps with many rows per expert). Padding rows are
 * not written. */
int nvs_moe_gemm(const void* X, int64_t ldx, const void* W, int dtype, int mode, int nout, int K, const int32_t* tile_expert,
                 const int32_t* row_token, int64_t cap, int tm, void* out, int64_t ldo, void* stream);
/* tests: 1 routes bf16 calls through the plain kernel as well */
void nvs_moe_force_plain(int on);

/* out[t, :] = sum_k wts[t, k] * (pair_row[t, k] >= 0 ? rows[pair_row[t, k], :] : h[t, :]) + sigmoid(shared_gate[t]) * shared[t, :]
 * (shared NULL: no shared expert; shared_gate 32-bit pre-activations with row stride gate_stride, NULL: the shared expert is added
 * as it is). */
int nvs_moe_combine(const void* rows, int64_t ldr, const int32_t* pair_row, const float* wts, int top, const void* h, int64_t ldh,
                    const void* shared, const float* shared_gate, int64_t gate_stride, int dtype, int64_t n, int width, void* out,
                    void* stream);

/* Latent attention, around the attention call (nvs_window_attn with one kv head of size kv_rank + rot_dim, values = the latent).
 * proj [n, stride] (`dtype`) is a fused projection output. Columns q_col .. + q_rank are RMS-normed with q_norm into cq [n, q_rank].
 * With kv_col >= 0, columns kv_col .. + kv_rank are RMS-normed with kv_norm (the latent c) and the next rot_dim columns are the
 * shared key part: its leading rot_dims entries turn by pos[t] * rot_freq[i], i < rot_dims / 2, pair (2i, 2i+1) or, with
 * rot_halves, (i, i + rot_dims / 2); cos and sin are multiplied by rot_mag. Token t goes to cache slot slots[t] (< 0: skipped):
 * k_cache [slot][kv_rank + rot_dim] = [c | rotated part]; v_cache [page][kv_rank][block_size] = c, transposed inside the page. */
int nvs_latent_prep(const void* proj, int64_t stride, int dtype, int q_col, int q_rank, const void* q_norm, void* cq, int kv_col,
                    int kv_rank, int rot_dim, const void* kv_norm, const int64_t* pos, const float* rot_freq, int rot_dims, int rot_halves,
                    float rot_mag, float eps, int block_size, const int32_t* slots, void* k_cache, void* v_cache, int64_t n, void* stream);

/* out[t, h, 0 .. width) = in[t, h, 0 .. width) with the leading rot_dims entries rotated as above; rows t have strides in_stride /
 * out_stride, heads in_head / out_head (elements, `dtype`). */
int nvs_rotate_heads(const void* in, int64_t in_stride, int in_head, void* out, int64_t out_stride, int out_head, int dtype, int H,
                     int width, const int64_t* pos, const float* rot_freq, int rot_dims, int rot_halves, float rot_mag, int64_t n,
                     void* stream);

/* Tests and A/B runs: 1 routes bf16 calls through the scalar kernel too; 2 keeps the matrix-core kernel but without sharing
 * K / V tiles through LDS; 3 keeps the LDS kernel but never packs heads into the query tiles of single-token steps; 0 restores
 * the defaults. */
void nvs_window_attn_force_scalar(int on);

#ifdef __cplusplus
}
#endif
#endif
