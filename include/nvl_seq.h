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
 * angle (angles in 32-bit from an exact integer position). xh (nullable): copy of x in `dtype`. */
int nvs_embed_sinusoid(const void* table, int dtype, const int64_t* ids, const int64_t* pos, int64_t n, int width,
                       float scale, float base, float* x, void* xh, void* stream);

/* Residual update with the norm on the sublayer OUTPUT: x += g * rms(m), g one number (device, `dtype`).
 * With m2 != NULL the sublayer output is the mean of two branches, each RMS-normed with a per-channel weight first:
 * m' = (rms(m) * w1 + rms(m2) * w2) / 2, x += g * rms(m'). rms(v) = v / sqrt(mean(v^2) + eps). xh (nullable): x in `dtype`. */
int nvs_norm_residual(const void* m, const void* m2, const void* w1, const void* w2, const void* g, int dtype, int64_t n,
                      int width, float eps, float* x, void* xh, void* stream);

/* out[r, :] = g * rms(x[rows[r], :]) in `dtype` (rows == NULL: row r). */
int nvs_scalar_norm_rows(const float* x, const int32_t* rows, int64_t nrows, int width, const void* g, int dtype, float eps,
                         void* out, void* stream);

/* xIELU, elementwise: z > 0: softplus(p) z^2 + beta z; z <= 0: (beta + softplus(q)) (exp(z) - 1 - z) + beta z. pq = {p, q}
 * (device, `dtype`). In place allowed. */
int nvs_xielu(const void* in, const void* pq, float beta, int dtype, int64_t numel, void* out, void* stream);

/* Per-channel causal convolution over the packed portions, continuing each sequence from its state.
 * in: [n, channels] with row stride in_stride (elements, `dtype`); w [channels, taps] (last tap = current token), b [channels]
 * (nullable); act: 0 none, 1 SiLU. state [nslots, taps-1, channels] (32-bit) holds each sequence's last taps-1 inputs and
 * is advanced by the call (a second launch, after the outputs have been computed). out [n, channels], 32-bit. */
int nvs_causal_conv(const void* in, int64_t in_stride, int dtype, const void* w, const void* b, int channels, int taps, int act,
                    const int32_t* cu_q, const int32_t* ctx0, const int32_t* slot, const int32_t* tseq, int nseq, int64_t n,
                    float* state, float* out, void* stream);

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

/* out = group_rms(y * silu(z)) * w: the gate first, then each of `groups` equal parts of a row by its own root mean square.
 * y [n, inner] 32-bit; z [n, inner] with row stride z_stride (`dtype`); w [inner]; out [n, inner] `dtype`. */
int nvs_gated_group_norm(const float* y, const void* z, int64_t z_stride, int dtype, const void* w, int inner, int groups,
                         float eps, int64_t n, void* out, void* stream);

/* Key norm + paged K/V store. k [n, G, d] / v [n, G, dv] are column ranges of one projection output (row stride `stride`,
 * `dtype`). k is RMS-normed over d with weight knorm [d] (NULL: stored as is). Token t goes to cache slot slots[t] (< 0:
 * skipped); slot = page * block_size + offset. Caches, `dtype`: k_cache [slot][G][d]; v_cache [page][G][dv][block_size] — values
 * are kept TRANSPOSED inside a page, so that a column's consecutive tokens are contiguous (the matrix-core attention reads 8 at a
 * time). */
int nvs_knorm_kvstore(const void* k, const void* v, int64_t stride, int dtype, const void* knorm, float eps, int G, int d, int dv,
                      int block_size, const int32_t* slots, int64_t n, void* k_cache, void* v_cache, void* stream);

/* Sliding-window softmax attention over the paged cache, one query per token row, any d, dv <= 256.
 * q [n, H, d] (row stride q_stride), RMS-normed per head with qnorm [d] here (NULL: none). Token t of portion s sits at position
 * p = ctx0[s] + (t - cu_q[s]) and sees keys j with 0 <= p - j < window (window <= 0: every j <= p), read through
 * block_tables [nseq, bt_stride]. score = q.k * scale, ordinary softmax in 32-bit. gate (nullable) [n, H*dv] with row stride
 * gate_stride: out *= sigmoid(gate). out [n, H*dv] `dtype`.
 * bf16 with d % 8 == 0 and block_size % 8 == 0 runs on the matrix cores (16 queries per wavefront; the weights enter the
 * second product as bf16); everything else, and every float32 call, takes the scalar kernel (one wavefront per query). */
int nvs_window_attn(const void* q, int64_t q_stride, const void* qnorm, float eps, const void* gate, int64_t gate_stride, int dtype,
                    const void* k_cache, const void* v_cache, const int32_t* block_tables, int64_t bt_stride, int block_size,
                    const int32_t* cu_q, const int32_t* ctx0, const int32_t* tseq, int nseq, int64_t n, int H, int G, int d, int dv,
                    float scale, int window, void* out, void* stream);

/* Tests and A/B runs: 1 routes bf16 calls through the scalar kernel too; 2 keeps the matrix-core kernel but without sharing
 * K / V tiles through LDS; 0 restores the defaults. */
void nvs_window_attn_force_scalar(int on);

#ifdef __cplusplus
}
#endif
#endif
