// C interface of the gfx950 kernel library.  Every function launches on the given
// stream and returns at once; 0 means the launch was accepted, a negative value
// means the arguments were refused (kvc_last_error() holds the reason) and nothing
// was launched.  Pointers are device pointers unless named host_*.
//
// dtype codes: 0 = float32, 1 = bfloat16.  "dt" in a comment means that type.
#pragma once

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* kvc_stream;

const char* kvc_last_error(void);
int kvc_version(void);
// Compute units of the current device: what the launch plans of the attention kernels count
// blocks against.
int kvc_compute_units(void);
// The variant that this thread's last launch of a kernel family took, as a short text such as
// "prefill_attention_kernel<128,1,8,8> x1" (head size, column tiles, key blocks a tile, waves,
// then the number of splits) or "rope_kv_write_tile_kernel"; "" if the family has not been
// launched.  Families: 0 attention over portions of prompts, 1 rotation with the cache write.
const char* kvc_last_variant(int family);

// Measurement only (peaks.hip).  kvc_peak_read: `blocks` blocks of 256 threads read `bytes` bytes
// of `buffer` once with 16-byte loads and store nothing (`sink`: four bytes that are practically
// never written); timed by the caller over buffers too large for the caches, it gives the read
// bandwidth that a kernel can reach at all.  kvc_peak_mfma_bf16: every wave of `blocks` blocks
// of four issues `rounds` x 4 independent 32x32x16 bfloat16 matrix instructions on operands in
// registers (2 x 32 x 32 x 16 flops each) and stores one float a thread into `out`.
int kvc_peak_read(const void* buffer, int64_t bytes, int blocks, void* sink, kvc_stream stream);
int kvc_peak_mfma_bf16(float* out, int blocks, int rounds, kvc_stream stream);

// residual[t, :] = float(table[ids[t], :]) * scale; an id outside [0, V) gives a NaN row.
int kvc_embed(float* residual, const void* table, const int32_t* ids, int T, int H, int V,
              int dtype, float scale, kvc_stream stream);

// What a head may do to its logits [S, V] (float32, rows row_stride apart) after the product,
// in place: x += bias[v] (bias of bias_dtype, or null); x = soft_cap * tanh(x / soft_cap) when
// soft_cap > 0; x *= scale.
int kvc_logits_finish(float* logits, int S, int V, int64_t row_stride, const void* bias,
                      int bias_dtype, float soft_cap, float scale, kvc_stream stream);

// Every element of the pages pages[i * page_stride], i < n, in all `outer` planes of a cache
// group's storage [outer, num_pages, page_elems] (elements of elem_bytes = 2 or 4) becomes the
// bit pattern `bits` (its low 16 bits for 2-byte elements): zeros, or a NaN that makes a read
// of a slot nobody wrote show in the logits.  The null page (0) and ids outside the pool are
// skipped.  Reference: kvcore/model/model_runner.py:646-657 zeroes new blocks with index_fill_.
int kvc_fill_pages(void* storage, const int32_t* pages, int page_stride, int n, int outer,
                   int num_pages, int64_t page_elems, int elem_bytes, uint32_t bits, kvc_stream stream);

// out[i] = mean + std * z_i for i < n, out of dtype: z_i is a standard normal variate that is a
// function of (seed_lo, seed_hi, i) alone, worked out in single float32 operations that a host
// program can repeat bit for bit (see random_fill.hip).
int kvc_fill_normal(void* out, int64_t n, int dtype, uint32_t seed_lo, uint32_t seed_hi, float mean,
                    float std, kvc_stream stream);

// residual += delta (skipped when delta is null); out = weight * residual *
// rsqrt(mean(residual^2) + eps), rounded to dt.  residual stays float32.
int kvc_add_rmsnorm(void* out, float* residual, const void* delta, const float* weight,
                    float eps, int T, int H, int dtype, kvc_stream stream);
// The same with the pending output given as float32 partial sums [slices, T, H] of a product
// cut along K (see kvc_gemm_mid_bf16, mode 2) and an optional bfloat16 bias [H]: the slices
// are added up in their order, then into the residual.  H a multiple of 8, at most 16384.
int kvc_add_slices_rmsnorm(void* out, float* residual, const float* partial, int slices,
                           const void* bias, const float* weight, float eps, int T, int H, int dtype,
                           kvc_stream stream);

// out = weight * x * rsqrt(mean(x^2) + eps) on rows of dt (no residual), row strides given.
int kvc_rmsnorm(void* out, const void* x, const float* weight, float eps, int T, int H,
                int64_t x_stride, int64_t out_stride, int dtype, kvc_stream stream);

// residual += delta, nothing else.
int kvc_residual_add(float* residual, const void* delta, int T, int H, int dtype,
                     kvc_stream stream);
// residual[t] += a[t] + b[t] (the two added first), a and b of their own dtypes.
int kvc_residual_add2(float* residual, const void* a, int a_dtype, const void* b, int b_dtype, int T,
                      int H, kvc_stream stream);

// out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i].
int kvc_silu_mul(void* out, const void* gate_up, int T, int I, int dtype, kvc_stream stream);
// out[t, i] = act(gate_up[t, i]) * gate_up[t, I + i]; act 0: silu, 1: gelu in its tanh form,
// 0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3))).
int kvc_gate_mul(void* out, const void* gate_up, int T, int I, int act, int dtype, kvc_stream stream);

// out = act(x) elementwise over n values (in place is fine); act 0: the square of relu.
int kvc_activation(void* out, const void* x, int64_t n, int act, int dtype, kvc_stream stream);

// out[s, :] = in[rows[s], :]; `in` may be float32 (in_dtype 0) while out is dt.
int kvc_gather_rows(void* out, const void* in, const int32_t* rows, int S, int H, int in_dtype,
                    int out_dtype, kvc_stream stream);

// out = float(in) elementwise (n values).
int kvc_to_float(float* out, const void* in, int64_t n, int dtype, kvc_stream stream);

// cos/sin[t, j] of the angle float(positions[t]) * inv_freq[j], j < half.
int kvc_rope_table(float* cos_out, float* sin_out, const int32_t* positions,
                   const float* inv_freq, int T, int half, kvc_stream stream);

// kv_slot[t] = page * page_size + position % page_size, where page = table[slots[
// token_req[t]], position / page_size]; -1 when the table holds no page there, -2 for a
// padding token (token_req < 0).
int kvc_kv_slots(int32_t* kv_slot, const int32_t* positions, const int32_t* token_req,
                 const int32_t* slots, const int32_t* table, int table_stride, int T,
                 int page_size, int num_pages, kvc_stream stream);

// Rotates the first rot_dim elements of every q and k head of qkv [T, (nh+2nkv)*d] in
// place (pairs (j, j+rot_dim/2), or (2j, 2j+1) when interleaved), then, when write_kv is
// set and kv_slot[t] >= 0, stores the rotated k and the v of token t at that slot:
//   k_cache[page, kv_head, offset, :] and v_cache[page, kv_head, :, offset]
//   (V pages keep the keys contiguous: the layout the matrix cores read).
// Tokens with kv_slot == -2 are left alone.  Without rotate_q the q heads stay as they are
// (for a consumer that rotates them itself, as kvc_prefill_attention can).
int kvc_rope_kv_write(void* qkv, void* k_cache, void* v_cache, const float* cos_tab,
                      const float* sin_tab, int rot_dim, int interleaved, const int32_t* kv_slot,
                      int T, int nh, int nkv, int d, int page_size, int write_kv, int rotate_q,
                      int dtype, kvc_stream stream);

// Attention of every token over its request's cache: token t at position p sees keys
// max(0, p - window + 1) .. p (window <= 0: all), read through the block table.
// q is [T, nh, d] with q_stride elements between tokens; keys have d elements, values dv (K
// pages [kv head, page_size, d], V pages [kv head, dv, page_size]); out is [T, nh*dv].
// slopes (float32 [nh], or null): slopes[h] * (p - key position) is taken off every score of head
// h.  chunk > 0: a token sees only the keys j with j / chunk == p / chunk.  sinks (float32 [nh],
// or null): exp(sinks[h]) is added to the softmax's denominator of head h: a logit of its own,
// taken as it is (scale does not apply), that brings no value into the weighted sum.
// out_f32: out is float32 whatever dtype says of the operands (the weighted sums as they are, for a
// consumer that joins results before anything is rounded); the two kernels below take it too.
int kvc_paged_attention(void* out, const void* q, int64_t q_stride, const void* k_cache,
                        const void* v_cache, const int32_t* table, int table_stride,
                        const int32_t* positions, const int32_t* token_req,
                        const int32_t* slots, int T, int nh, int nkv, int d, int dv, int page_size,
                        int num_pages, float scale, int window, const float* slopes, int chunk,
                        const float* sinks, int out_f32, int dtype, kvc_stream stream);

// What kvc_rope_kv_write does, for heads whose keys (d) and values (dv) may differ in size,
// with a norm of every q and k head before the rotation: rows of qkv are [nh q heads of d |
// nkv k heads of d | nkv v heads of dv], row_stride elements apart.  With q_gain and k_gain
// ([d] each, shared by all heads; both null: no norm) a head becomes gain * x / sqrt(mean(x^2)
// + eps); then its first rot_dim elements are rotated by cos/sin [T, rot_dim / 2].  q and k are
// rewritten in place; with write_kv, k goes to K[page, kv head, offset, :] and v to V[page, kv
// head, :, offset] at kv_slot[t] (as kvc_kv_slots gives it).  The values may be kept in
// num_v_planes (1 to 4) planes of dv / num_v_planes elements a head each (host_v_planes: a host
// array of their device pointers): element i of a value head then lies in plane i / (dv /
// num_v_planes), so that kernels whose keys and values are of one size can serve a plane each.
int kvc_qk_norm_rope_kv_write(void* qkv, int64_t row_stride, void* k_cache,
                              void* const* host_v_planes, int num_v_planes, const float* q_gain, const float* k_gain, float eps,
                              const float* cos_tab, const float* sin_tab, int rot_dim,
                              int interleaved, const int32_t* kv_slot, int T, int nh, int nkv, int d,
                              int dv, int page_size, int write_kv, int dtype, kvc_stream stream);

// residual += delta (skipped when delta is null); out = (residual - mean) / sqrt(var + eps) *
// weight + bias (bias may be null), var the mean of the squared deviations; rounded to dt.
int kvc_add_layernorm(void* out, float* residual, const void* delta, const float* weight,
                      const float* bias, float eps, int T, int H, int dtype, kvc_stream stream);

// out[t] = (1 / n) * sum_b gain_b * x_b[t] / sqrt(mean(x_b[t]^2) + eps) over n <= 4 branches of
// float32 rows [T, H]; host_x and host_gain are host arrays of n device pointers.
int kvc_rms_branches_mean(void* out, const float* const* host_x, const float* const* host_gain,
                          int n, float eps, int T, int H, int dtype, kvc_stream stream);

// out[t] = [a[t] | b[t]] ([T, 2H] of dt from two float32 [T, H]);  x[t, :] += v[:] (float32).
int kvc_concat2(void* out, const float* a, const float* b, int T, int H, int dtype, kvc_stream stream);
int kvc_add_row(float* x, const float* v, int T, int H, kvc_stream stream);

// ---- mixers with a state of fixed size per request (recurrent.hip).  q_start [R+1], positions
// [T], token_req [T] (-1: padding), slots [R] describe the flattened batch; a request whose
// first token of the step is at position 0 starts from a zero state, any other from its slot's.
//
// Causal convolution per channel: out[t, c] = act(bias[c] + sum_j weight[c, K-1-j] * in(p - j)),
// act 0 none or 1 silu, in() being zero before the sequence's start; state [slots, K-1, C]
// float32 holds the K-1 inputs before the step and, with update_state, afterwards those before
// the next.  x and out are rows of their dtypes with strides (x may be columns of a wider row).
// single_tokens: the caller vouches that every request brings exactly one token (T = R); the
// state then moves on in the convolution's own kernel instead of a second one.
int kvc_causal_conv(void* out, int64_t out_stride, int out_dtype, const void* x, int64_t x_stride,
                    int x_dtype, const float* weight, const float* bias, float* state,
                    const int32_t* positions, const int32_t* token_req, const int32_t* q_start,
                    const int32_t* slots, int T, int R, int C, int K, int act, int update_state,
                    int single_tokens, kvc_stream stream);
// Gates of the real-gated linear recurrent unit on u [T, W] float32, W in nb blocks: r =
// sigmoid(wa[b] u_b + ba), i = sigmoid(wi[b] u_b + bi) (wa, wi [nb, W/nb, W/nb] float32, [out,
// in]); a_out = exp(-c_decay * r * softplus(lam)); drive = sqrt(1 - a^2) * i * u.
int kvc_rglru_gates(float* a_out, float* drive, const float* u, const float* wa, const float* wi,
                    const float* ba, const float* bi, const float* lam, float c_decay, int T, int W,
                    int nb, kvc_stream stream);
// S_t = a_t S_(t-1) + drive_t per channel along each request (state [slots, W] float32);
// out[t] = S_t * gelu_tanh(y[t]).  max_query_len bounds the tokens of a request in this step;
// with a workspace of R * (ceil(max_query_len / kvc_rglru_scan_segment()) + 1) * 2 * W floats,
// requests longer than a segment are scanned segment by segment side by side (two kernels: the
// segments' sums, then the results); without one, or for short portions, one thread walks a
// request's tokens for each channel.
int kvc_rglru_scan_segment(void);
int kvc_rglru_scan(void* out, int out_dtype, const float* a, const float* drive, const void* y,
                   int64_t y_stride, int y_dtype, float* state, const int32_t* positions,
                   const int32_t* token_req, const int32_t* q_start, const int32_t* slots, int R,
                   int W, int max_query_len, float* workspace, int64_t workspace_floats,
                   kvc_stream stream);
// State-space recurrence with a scalar decay per head: xbc [T, >= nh*P + 2*G*N] float32 rows
// hold x (nh heads of P), then B and C (G groups of N); per head h of group h / (nh / G):
// dt = softplus(dt_raw[t, h] + dt_bias[h]); S = exp(-exp(a_log[h]) dt) S + dt B x^T (S [N, P],
// state [slots, nh, N, P] float32); y[t, h] = S^T C + d_skip[h] x, y [T, nh*P] float32.
// N at most kvc_ssm_scan_max_state().
int kvc_ssm_scan_max_state(void);
int kvc_ssm_scan(float* y, const float* xbc, int64_t xbc_stride, const void* dt_raw,
                 int64_t dt_stride, int dt_dtype, const float* dt_bias, const float* a_log,
                 const float* d_skip, float* state, const int32_t* positions,
                 const int32_t* token_req, const int32_t* q_start, const int32_t* slots, int R,
                 int nh, int P, int N, int G, kvc_stream stream);
// out[t, c] = gain[c] * v / sqrt(mean of v^2 over c's part + eps), v = y[t, c] * silu(z[t, c]),
// the width cut into `groups` equal parts.
int kvc_gated_group_rmsnorm(void* out, int out_dtype, const float* y, const void* z,
                            int64_t z_stride, int z_dtype, const float* gain, float eps, int T,
                            int width, int groups, kvc_stream stream);

// ---- mixers whose state is a float32 matrix S [d, dv] per head (linear_attention.hip).  The batch
// is described as for the recurrent mixers above; state is [slots, nh, dpad, dv] float32, dpad = d
// rounded up to a multiple of 4, a head's element (n, c) at ((n / 4) * dv + c) * 4 + n % 4.
// Per head h (its q and k come from head h / (nh / nqk) of nqk heads of d), token by token:
//   delta_rule 0:  S = diag(decay[t, h, :]) S + k v^T            (decay rows of nh * d values)
//   delta_rule 1:  S = decay[t, h] S;  u = beta[t, h] (v - S^T k);  S = S + k u^T
//   delta_rule 2:  S = decay[t, h] S + beta[t, h] k v^T          (scalar gates per head)
// and out[t, h] = S^T (q_scale q) after the token's write; out is [T, nh * dv] float32.  q, k, v, decay and
// beta are float32 rows with strides.  d at most 256.  With ones_column the rows of v hold dv - 1
// values a head and column dv - 1 of every head takes a one for each token: a normaliser that is
// gated and read like the matrix, out[t, h, dv - 1] being its product with the query.
int kvc_linear_state_scan(float* out, const float* q, int64_t q_stride, const float* k,
                          int64_t k_stride, const float* v, int64_t v_stride, const float* decay,
                          int64_t decay_stride, const float* beta, int64_t beta_stride, float* state,
                          const int32_t* positions, const int32_t* token_req, const int32_t* q_start,
                          const int32_t* slots, int R, int nh, int nqk, int d, int dv, int delta_rule,
                          float q_scale, int ones_column, kvc_stream stream);
// The gates of a matrix memory with log gates and a running maximum m (mLSTM), per request in
// token order: i = cap tanh((i_raw + i_bias) / cap), f = logsigmoid(cap tanh((f_raw + f_bias) / cap)),
// m_t = max(f + m_(t-1), i), keep[t, h] = exp(f + m_(t-1) - m_t), take[t, h] = exp(i - m_t),
// m_out[t, h] = m_t; m is 0 before position 0, else m_state[slot, h], which receives the last m.
// keep, take, m_out are [T, nh] float32; i_raw and f_raw float32 rows with strides.
int kvc_max_gates(float* keep, float* take, float* m_out, const float* i_raw, int64_t i_stride,
                  const float* f_raw, int64_t f_stride, const float* i_bias, const float* f_bias,
                  float cap, float* m_state, const int32_t* positions, const int32_t* token_req,
                  const int32_t* q_start, const int32_t* slots, int T, int R, int nh,
                  kvc_stream stream);
// out[t, h, c] = y / sqrt(mean_c y^2 + eps) * gain[h * dv + c] * sigmoid(gate[t, h, c]) with
// y = o[t, h, c] / (max(|o[t, h, dv]|, exp(-m[t, h])) + den_eps); o is [T, heads, dv + 1] float32.
int kvc_max_gated_finish(void* out, int out_dtype, const float* o, const float* m, const void* gate,
                         int64_t gate_stride, int gate_dtype, const float* gain, float eps,
                         float den_eps, int T, int heads, int dv, kvc_stream stream);
// a[t, i] = sigmoid(z[t, i] + bias[i]) ^ inv_tau, computed as exp(inv_tau * log sigmoid); bias may be null.
int kvc_sigmoid_power(float* a, const float* z, int64_t z_stride, const float* bias, float inv_tau,
                      int T, int W, kvc_stream stream);
// g[t, h] = exp(-exp(a_log[h]) * softplus(a_raw[t, h] + dt_bias[h])); beta[t, h] = sigmoid(b_raw[t, h]).
int kvc_decay_and_write_gates(float* g, float* beta, const float* a_raw, int64_t a_stride,
                              const float* b_raw, int64_t b_stride, const float* a_log,
                              const float* dt_bias, int T, int nh, kvc_stream stream);
// x[t, h, :] *= scale / sqrt(sum x[t, h, :]^2 + eps), in place, heads of d float32 values; the first
// first_heads heads take first_scale instead of scale.
int kvc_unit_heads(float* x, int64_t stride, int T, int heads, int d, float eps, float scale,
                   int first_heads, float first_scale, kvc_stream stream);
// out[t, h, c] = o[t, h, c] / sqrt(mean_c o[t, h, :]^2 + eps) * gain[c] * silu(gate[t, h, c]).
int kvc_head_rmsnorm_gate(void* out, int out_dtype, const float* o, const void* gate,
                          int64_t gate_stride, int gate_dtype, const float* gain, float eps, int T,
                          int heads, int dv, kvc_stream stream);

// ---- routed experts (moe.hip); see the head of that file.  choice and weight are [T, top];
// sorted [pairs]; tiles [max_tiles, 3] (expert, first sorted row, rows); num_tiles [1].
// kvc_moe_gemm multiplies every tile's rows by its expert's matrix: w is [E, N, K], or with
// `gated` [E, 2N, K] (gate rows, then up rows) and the activation applied; a sorted row i reads
// x row sorted[i] / in_div (in_div 0: row i itself) and writes out row i (out_sorted) or
// sorted[i].  dtype is that of x and w.  packed: w is the copy kvc_pack_weight makes of the whole
// stacked matrix (bfloat16, N a multiple of 16, K of 64).
// score_fn 0: softmax over the experts, 1: sigmoid of each logit.  correction [E] (or null) is added
// to the scores for the choice alone.  group_best 1 or 2: a group is worth its best choice score, or
// the sum of its best two.  The weights are multiplied by weight_scale.
int kvc_moe_route(int32_t* choice, float* weight, const float* logits, int T, int E, int top,
                  int groups, int keep, int score_fn, const float* correction, int group_best,
                  float weight_scale, kvc_stream stream);
// Tiles hold up to tile_rows rows, 16 or 64 (kvc_moe_tile_rows says which a step's size asks
// for; 64 is for bfloat16 with K a multiple of 32).
int kvc_moe_tile_rows(int pairs, int E);
// The router's logits (x [T, H] of x_dtype times router [E, H] float32, float32 sums in one fixed order)
// and the choice of kvc_moe_route in one kernel.
int kvc_moe_router(int32_t* choice, float* weight, const void* x, int64_t x_stride, int x_dtype,
                   const float* router, int T, int H, int E, int top, int groups, int keep, int score_fn,
                   const float* correction, int group_best, float weight_scale, kvc_stream stream);
int kvc_moe_max_tiles(int pairs, int E, int tile_rows);
int kvc_moe_align(int32_t* sorted, int32_t* tiles, int32_t* num_tiles, const int32_t* choice,
                  int pairs, int E, int max_tiles, int tile_rows, kvc_stream stream);
int kvc_moe_gemm(void* out, int64_t out_stride, int out_dtype, const void* x, int64_t x_stride,
                 const void* w, int dtype, const int32_t* sorted, const int32_t* tiles,
                 const int32_t* num_tiles, int max_tiles, int tile_rows, int N, int K, int in_div, int out_sorted,
                 int gated, float limit, float alpha, float up_shift, int packed, kvc_stream stream);
// out[t] = sum_c weight[t, c] * y[t * top + c] + add0[t] + add1[t] (either may be null; add0 of
// dtype add0_dtype, add1 float32), float32.
// accumulate: the sum is added into out instead of stored.
int kvc_moe_combine(float* out, const float* y, const float* weight, int top, const void* add0,
                    int add0_dtype, const float* add1, int T, int H, int accumulate, kvc_stream stream);
// out[t, i] = g * sigmoid(alpha * g) * (u + 1), g = min(gate_up[t, i], limit),
// u = clamp(gate_up[t, I + i], -limit, limit).
int kvc_clamped_glu(void* out, const void* gate_up, int T, int I, float limit, float alpha, int dtype,
                    kvc_stream stream);

// The same attention for bfloat16 steps of single tokens on the matrix cores, a block of
// several waves per (token, kv head, split), which also does what kvc_rope_kv_write does for
// its token: qkv rows are [nh q heads | nkv k heads | nkv v heads]; the first rot_dim elements
// of every q head (and of the k head) are rotated by cos/sin [T, rot_dim / 2] on the way in
// (rot_dim 0: taken as they are) and qkv itself is left unchanged; with write_kv the
// token's key and value are stored in their cache slot and attended to (without write_kv
// the cache must already hold them).  nsplit > 1 needs part_o [T, nh, nsplit, d] and part_ml
// [T, nh, nsplit, 2] float32; a second kernel combines the splits (a "last block combines"
// scheme needs device-scope fences, which on this chip write back and invalidate a whole L2
// slice per block and cost more than the launch they save).
// token_rows [T], if not null, holds slots[token_req[t]] (-1 for padding) and saves the
// kernel one dependent load.
// kvc_decode_attention_supported tells whether a shape is served (else use
// kvc_paged_attention); kvc_decode_attention_waves how many waves share a block's key range.
// kvc_decode_attention_max_table: the widest block table (entries per request) whose page ids
// for one split still fit in a block's LDS; a wider one is refused, so engines check it when
// they are built.
// slopes, sinks (float32 [nh] or null) and chunk as for kvc_paged_attention; the kernel for portions
// (kvc_prefill_attention) takes them too.
int kvc_decode_attention_supported(int nh, int nkv, int d, int page_size, int dtype);
int kvc_decode_attention_waves(int nh, int nkv, int d);
int kvc_decode_attention_max_table(int nh, int nkv, int d);
int kvc_decode_attention(void* out, void* part_o, void* part_ml, const void* qkv,
                         int64_t qkv_stride, void* k_cache, void* v_cache, const int32_t* table,
                         int table_stride, const int32_t* positions, const int32_t* token_req,
                         const int32_t* slots, const int32_t* token_rows, const float* cos_tab,
                         const float* sin_tab, int rot_dim, int interleaved, int write_kv, int T,
                         int nh, int nkv, int d, int page_size, int num_pages, float scale,
                         int window, const float* slopes, int chunk, const float* sinks, int nsplit,
                         int out_f32, kvc_stream stream);

// The same attention for bfloat16 portions of prompts on the matrix cores: a block per
// (tile of a request's tokens, kv head), keys staged through LDS.  q_start [R+1] bounds
// each request's tokens in the flattened batch; slots [R] names its block-table row;
// positions must rise by one along a request's tokens.  With nsplit > 1 the keys of every
// tile are dealt to that many blocks (for few query rows against many keys) and a second
// kernel joins their results; part_o [T*nh*nsplit, d] and part_ml [T*nh*nsplit, 2] float32
// are its workspace.  With cos_tab and sin_tab [T, rot_dim / 2] the queries come unrotated
// and are rotated on their way in, as kvc_rope_kv_write would have (rot_dim a multiple of 64,
// or of 32 when interleaved); without, they are taken as they are.
int kvc_prefill_attention_supported(int nh, int nkv, int d, int page_size, int dtype);
int kvc_prefill_attention(void* out, const void* q, int64_t q_stride, const void* k_cache,
                          const void* v_cache, const int32_t* table, int table_stride,
                          const int32_t* positions, const int32_t* q_start, const int32_t* slots,
                          int T, int R, int nh, int nkv, int d, int page_size, int num_pages,
                          float scale, int window, const float* slopes, int chunk, const float* sinks, void* part_o,
                          void* part_ml, int nsplit,
                          const float* cos_tab, const float* sin_tab, int rot_dim, int interleaved,
                          int out_f32, kvc_stream stream);

// ---- norms after a sublayer, norms over a whole projection, gates per head (norm_ops.hip)
// residual[t, :] += post_gain * delta[t, :] / sqrt(mean(delta[t, :]^2) + eps), and then, if out is
// not null, out[t, :] = next_gain * residual[t, :] / sqrt(mean(residual[t, :]^2) + next_eps): the norm
// behind a sublayer, the sum into the float32 stream and the norm before the next sublayer in one
// pass.  delta is float32 (delta_dtype 0) or bfloat16 (1); out likewise (out_dtype).  slices > 1:
// delta holds [slices, T, H] float32 partial sums of a product cut along K (kvc_gemm_mid_bf16 mode
// 2) and a row of the result is their sum in slice order.
int kvc_norm_add_norm(void* out, int out_dtype, float* residual, const void* delta, int delta_dtype,
                      const float* post_gain, float eps, const float* next_gain, float next_eps,
                      int T, int H, int slices, kvc_stream stream);
// Rows of attn are [heads][2][dv]: out[t, h] = (a1 - lambda * a2) / sqrt(mean((a1 - lambda * a2)^2) + eps)
// * post over the head's dv values, out [T, heads * dv] of dtype; attn of attn_dtype (dtype, or float32);
// float32 arithmetic.
int kvc_diff_heads_norm(void* out, const void* attn, int64_t attn_stride, int attn_dtype, float lambda, float eps,
                        float post, int T, int heads, int dv, int dtype, kvc_stream stream);
// Rows of qkv are [nq | nk | ...]: the first nq values (all query heads at once) are divided by
// their root mean square (eps inside the root) and multiplied by q_gain [nq], the next nk values
// likewise with k_gain [nk], in place; with copy_k the nk values as they were before the norm
// are copied behind them first (values that are the keys as projected).
int kvc_wide_qk_norm(void* qkv, int64_t stride, const float* q_gain, const float* k_gain, float eps,
                     int T, int nq, int nk, int copy_k, int dtype, kvc_stream stream);
// Rows of down are [q_rank | rank | rot | ...]: cq[t] = q_gain * rms-normed first run; key[t] and
// value[t] (rows kv_stride apart) both receive [the rot values as they are | kv_gain * rms-normed
// second run]: what a latent attention caches a token, laid out with the rotated part first.
int kvc_latent_rows(void* cq, int64_t cq_stride, void* key, void* value, int64_t kv_stride, const void* down,
                    int64_t down_stride, const float* q_gain, const float* kv_gain, float eps, int T,
                    int q_rank, int rank, int rot, int dtype, kvc_stream stream);
// out[t, h * n + e] = x[t * x_stride + h * head_stride + skip + e] * sigmoid(gate[t * gate_stride + h]),
// e < n: a gate per head, and a run of each head's columns kept.  gate has the dtype of x and out.
int kvc_head_gate(void* out, const void* x, int64_t x_stride, const void* gate, int64_t gate_stride,
                  int T, int heads, int head_stride, int skip, int n, int dtype, kvc_stream stream);

// A residual stream of `copies` (1 to 8) rows a token, streams [T, copies, H] float32.  With y ([T, H]
// of y_dtype; or, y_slices > 1, that many float32 partial sums [y_slices, T, H] whose sum it is; plus
// y_bias [H] of y_bias_dtype, if not null): x_t <- sum_s mix[s * copies + t] x_s + mult * out_w[t] * y for all copies at once (mix
// null: the identity, out_w null: ones).  Then, with out ([T, H] of out_dtype): u = sum_t in_w[t] x_t
// (in_w null: ones), out = gain * u / sqrt(mean(u^2) + eps).
int kvc_hyper_step(void* out, int out_dtype, float* streams, const void* y, int y_dtype, int y_slices,
                   const void* y_bias, int y_bias_dtype, const float* mix, const float* out_w, float mult, const float* in_w, const float* gain, float eps,
                   int T, int H, int copies, kvc_stream stream);
// streams[t, c, :] = rows[t, :] for every copy c.
int kvc_spread_streams(float* streams, const float* rows, int T, int H, int copies, kvc_stream stream);

// C[M, N] = A[M, K] * W[N, K]^T (+ bias[N]) in float32 with float32 products and sums;
// each element is one running sum over k = 0..K-1, whatever M is.
int kvc_gemm_f32(float* C, const float* A, const float* W, const float* bias, int M, int N,
                 int K, int64_t lda, int64_t ldc, kvc_stream stream);

// The same product for 17 to 192 rows, where the waves of a block share the rows of A through
// LDS (K a multiple of 512).  mode 0: C = A W^T (+ bias), float32 (out_dtype 0) or bfloat16
// (1).  mode 1: C[M, N] = silu(A Wg^T + bg) * (A Wu^T + bu) in bfloat16, W [2N, K] holding Wg
// then Wu (mode 4: the same with the tanh form of gelu for silu).  mode 2: narrow outputs are cut along K into kvc_gemm_mid_slices(N, K) slices and
// only their float32 partial sums are stored, partial [slices, M, N] (no bias); the kernel
// that consumes them adds them up in slice order.  mode 3: as mode 0, but cut along K like
// mode 2 when `partial` is given, with a second kernel that sums the slices.  With `packed` W
// is what kvc_pack_weight made of the matrix (the same sums, read in contiguous kilobytes).
int kvc_gemm_mid_slices(int N, int K);
int kvc_gemm_mid_bf16(void* C, void* partial, const void* A, const void* W, const void* bias, int M,
                      int N, int K, int64_t lda, int64_t ldc, int out_dtype, int mode, int packed,
                      kvc_stream stream);

// C[M, N] = A[M, K] * W[N, K]^T (+ bias[N]) for M <= 64 rows of bfloat16 on the matrix
// cores, float32 sums, weights streamed once; C is float32 (out_dtype 0) or bfloat16 (1).
// K and lda must be multiples of 8, A and W 16-byte aligned.  With `packed` W is what
// kvc_pack_weight made of the matrix (N a multiple of 16, K of 64): the same sums in the same
// order, read in contiguous kilobytes.
int kvc_gemm_skinny_bf16(void* C, const void* A, const void* W, const void* bias, int M, int N,
                         int K, int64_t lda, int64_t ldc, int out_dtype, int packed,
                         kvc_stream stream);
// The same product with an activation on the way out, C bfloat16: act 0, the square of relu, of
// the product (+ bias) rounded to bfloat16 first, so that it equals the product stored and
// kvc_activation applied to it, bit for bit.
int kvc_gemm_skinny_act_bf16(void* C, const void* A, const void* W, const void* bias, int M, int N,
                             int K, int64_t lda, int64_t ldc, int act, int packed, kvc_stream stream);

// dst = src [N, K] bfloat16 in tiles of 16 rows x 32 columns of 1 KB each, the tiles of 16
// rows one after the other along K (N a multiple of 16, K of 64): element (n, k) goes to
// ((n / 16) * (K / 32) + k / 32) * 512 + (n % 16) * 32 + k % 32.  That is the order in which
// the products for few rows read the weights, whose loads then are one contiguous kilobyte
// instead of 64 bytes from each of 16 rows.
int kvc_pack_weight(void* dst, const void* src, int N, int K, kvc_stream stream);

// C[M, N] = silu(A Wg^T + bg) * (A Wu^T + bu) for M <= 64 rows of bfloat16, where Wg is rows
// 0..N-1 of W[2N, K] and Wu rows N..2N-1 (bias[2N] likewise): the gated feed-forward's first
// product with its activation, both factors rounded to bfloat16 before the activation as the
// two-kernel form stores them.  C is bfloat16.
int kvc_gemm_skinny_silu_mul_bf16(void* C, const void* A, const void* W, const void* bias, int M,
                                  int N, int K, int64_t lda, int64_t ldc, int packed,
                                  kvc_stream stream);

// The same products with the RMS norm of the rows folded in, for steps of at most 16 tokens,
// so that no separate norm kernel runs between them:
//  - in_ss [M, in_parts] (or null): A holds rows with the norm's gain applied but not yet
//    normalised; row m's sums are multiplied by rsqrt(sum_p in_ss[m, p] / in_width + in_eps)
//    before bias (and activation);
//  - residual [M, ldr] float32 (or null; not with gated): residual += product (+ bias); C
//    receives bfloat16(residual * gain[n]) and out_ss [M, blocks] the new residual's sums of
//    squares per block of columns, blocks = kvc_gemm_skinny_blocks(N, K, 0, packed): the in_ss of the
//    product that consumes C.
// gated = 1 is kvc_gemm_skinny_silu_mul_bf16's product (N = the gate's rows).
int kvc_gemm_skinny_blocks(int N, int K, int gated, int packed);
int kvc_gemm_skinny_fused_bf16(void* C, const void* A, const void* W, const void* bias, int M, int N,
                               int K, int64_t lda, int64_t ldc, int gated, const float* in_ss,
                               int in_parts, int in_width, float in_eps, float* residual,
                               int64_t ldr, const float* gain, float* out_ss, int packed,
                               kvc_stream stream);

// table[triples[3i], triples[3i+1]] = triples[3i+2] for i < n.
int kvc_table_update(int32_t* table, int table_stride, int table_rows, const int32_t* triples,
                     int n, kvc_stream stream);

// out[s] = index of the largest logit of row s (the lowest index among equals).  With a
// workspace (part_val, part_idx: part_capacity >= S * ceil(V / 8192) entries each) long rows
// are searched by several blocks; the pointers may be null.
int kvc_argmax(int32_t* out, const float* logits, int S, int V, int64_t row_stride,
               float* part_val, int32_t* part_idx, int part_capacity, kvc_stream stream);

// kvc_argmax for callers that cannot allocate device memory and bring no workspace (code
// under HIP graph capture, tight serving loops, harnesses that forbid allocation).  It has no
// counterpart in the reference.  The partial results of long rows live in a static device
// array of kvc_argmax_static_capacity() = 16384 entries (128 KB that every GPU the library
// runs on holds until the process ends); S * ceil(V / 8192) beyond that is refused with an
// error, rows of at most 8192 values need no partial results and are never refused.  The call
// allocates and frees nothing, on the device or through any library.  The array keeps the last
// call's contents; nothing in it has to start at zero, since every entry that is read was
// written earlier in the same call.  All calls on one GPU share that GPU's array: calls that
// overlap there (different streams or threads) race, calls on one stream do not.  The results
// equal kvc_argmax's.
int kvc_argmax_static_capacity(void);
int kvc_argmax_static(int32_t* out, const float* logits, int S, int V, int64_t row_stride,
                      kvc_stream stream);

// Per row s: temperature[s] < 1e-5 gives the argmax; otherwise
// argmax_v(logits[v] / temperature - log(e_v)), e_v exponential noise keyed by
// (seed_lo[s], seed_hi[s], index[s], v), over the entries that top_k[s] (<= 0: all) and
// top_p[s] (>= 1: all) keep.  With a workspace of kvc_sample_workspace_words(S, V) 64-bit
// words (0: rows too short to gain) every row is dealt to several blocks, which gives the
// same draws; it need not be cleared.  filters: bit 0, some row has a top_k; bit 1, some row
// has a top_p < 1 (passes that no row needs are left out; 3 is always right).
int kvc_sample_workspace_words(int S, int V);
int kvc_sample(int32_t* out, const float* logits, int S, int V, int64_t row_stride,
               const float* temperature, const int32_t* top_k, const float* top_p,
               const uint32_t* seed_lo, const uint32_t* seed_hi, const uint32_t* index,
               void* workspace, int64_t workspace_words, int filters, kvc_stream stream);

#ifdef __cplusplus
}
#endif
