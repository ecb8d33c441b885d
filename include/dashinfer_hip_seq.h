/* dashinfer_hip_seq.h -- C-ABI of libdashinfer_hip_seq.so: the operators of the ragged-batch sequence engine
 * (dash-infer_amd/engine.py): row-major linear layers, strided norms, the depth-weighted residual stream, windowed
 * attention over a paged latent cache with a softmax sink, causal short convolutions and gated linear recurrences with
 * per-sequence state slots.  Conventions are those of dashinfer_hip.h: plain pointers and sizes, `stream` = hipStream_t,
 * status 0 = success, dihip_seq_last_error() holds the text of the last failure of the calling thread; dtype codes
 * DIHIP_F32 / DIHIP_BF16.
 *
 * A step's tokens are ONE flat list of T rows (portions of prompts beside single decoded tokens).  Per row:
 *   tok_slot[t]  the state slot of the row's sequence,   tok_pos[t]  its position in the sequence (from 0),
 *   tok_off[t]   its index inside the portion this step brings (0 = the portion's first row).
 * Paged caches are tables of span pointers, one row of `span_stride` pointers per slot (as dihip_kv_append takes them);
 * a span holds `span_len` consecutive positions.  Nothing here depends on what else is in the batch: every output row
 * is computed by the same instructions in the same order whatever T is. */
#ifndef DASHINFER_HIP_SEQ_H_
#define DASHINFER_HIP_SEQ_H_
#include <stddef.h>
#include <stdint.h>

#include "dashinfer_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

const char* dihip_seq_version(void);
const char* dihip_seq_last_error(void);

/* math of dihip_linear: EXACT = every product and sum in f32, k ascending; BF16 = operands rounded to bf16, f32
 * accumulation on the matrix cores (T > DIHIP_LINEAR_SKINNY_ROWS) or in a weight-streaming dot-product kernel */
enum { DIHIP_MATH_F32 = 0, DIHIP_MATH_BF16 = 1, DIHIP_MATH_F32_STREAM = 2 };
/* F32_STREAM = F32 products of the unrounded operands, but few rows (decoding) stream the weight through the dot-product
 * kernel, whose sums run in the lanes' order: for the f32 parts of a bf16 engine (gates of a recurrence) */

/* y[g][t, n] = epilogue( sum_k x[g % x_groups][t, k] * w[g][n, k] + bias[g][n] ),  g < groups, t < T, n < N
 *   x: [T, .] rows of stride ldx, group g starts at column (g % x_groups) * x_gstride;  w: [groups][N][K] row-major,
 *   bias: [groups][N] or NULL (w_dtype);  y: rows of stride ldy, group g at column g * y_gstride;
 *   epilogue: activation `act` on the columns act_lo <= g * N + n < act_hi, then * mul[t, g * y_gstride + n] (rows of
 *   stride ldm, f32; NULL: none). */
int dihip_linear(void* stream, const void* x, int x_dtype, long ldx, long x_gstride, int x_groups,
                 const void* w, int w_dtype, const void* bias, void* y, int y_dtype, long ldy, long y_gstride,
                 const float* mul, long ldm, int T, int N, int K, int groups, int act, int act_lo, int act_hi, int math);

/* The same product for rows that are grouped by owner (mixture of experts): group g owns the output rows seg[g] .. seg[g + 1]
 * (seg: [groups + 1] on the device, ascending, seg[groups] <= R), output row r reads the x row row_map[r] (NULL: r itself) and
 * the weight w[g] ([groups][N][K]); bias [groups][N] or NULL; `act` on every column.  seg_max_rows: a host-known bound on the
 * rows of one group (it sizes the grid and chooses the kernel). */
int dihip_linear_segmented(void* stream, const void* x, int x_dtype, long ldx, const void* w, int w_dtype, const void* bias,
                           void* y, int y_dtype, long ldy, int R, int N, int K, int groups, const int32_t* seg,
                           const int32_t* row_map, int seg_max_rows, int act, int math);

/* The norm without statistics, fused with the residual step of a layer whose sublayers run side by side:
 *   x_out[r] = x_in[r] + (a[r] + b[r])   (a NULL: x_in itself; b NULL: a alone),   h[i] = tanh(alpha * x_out[r]) * w + bias
 * r = row_idx ? row_idx[i] : i (with row_idx x_out must be NULL).  x_in / x_out: contiguous [., K] f32 (may alias); h f32
 * and / or h16 bf16 [M, K] (either may be NULL; w NULL: no norm). */
int dihip_add_dyt(void* stream, float* x_out, const float* x_in, const float* a, long lda, const float* b, long ldb,
                  const int32_t* row_idx, float alpha, const void* w, const void* bias, int w_dtype, float* h, void* h16,
                  int M, int K);

/* Layers that run their sublayers side by side on a layer-normed stream: the residual step and the NEXT input norm in one launch,
 *   x_out[r] = x_in[r] + mult * (a[r] + b[r])   (a NULL: x_in itself; b NULL: a alone),
 *   h[i] = (x_out[r] - mean) / sqrt(var + eps) * w (+ bias)   (mean and variance over the row; bias NULL: none; w NULL: no norm)
 * r = row_idx ? row_idx[i] : i (with row_idx x_out must be NULL).  x_in / x_out: contiguous [., K] f32 (may alias); h: rows of
 * stride ldh, f32 or bf16. */
int dihip_residual_layernorm(void* stream, float* x_out, const float* x_in, const float* a, long lda, const float* b, long ldb,
                             float mult, const int32_t* row_idx, const void* w, const void* bias, int w_dtype, float eps, void* h,
                             int h_dtype, long ldh, int M, int K);
/* y[t] = c0 z / rms(z) + c1 z^2 / rms(z^2) + c2 z^3 / rms(z^3) + c3,  powers per element, rms(v) = sqrt(mean(v^2) + eps) over the
 * F elements of the row; coef = (c0, c1, c2, c3) of w_dtype */
int dihip_polynorm(void* stream, void* y, int y_dtype, long ldy, const float* z, long ldz, const void* coef, int w_dtype, float eps,
                   int T, int F);
/* y[t] = coef * (xa[t] / rms(xa[t]) * wa + xb[t] / rms(xb[t]) * wb)   (wa, wb [K] of w_dtype) */
int dihip_rmsnorm_pair(void* stream, float* y, long ldy, const float* xa, long lda, const void* wa, const float* xb, long ldb,
                       const void* wb, int w_dtype, float coef, float eps, int T, int K);
/* v = (o + skip[c / P] * x) * silu(z)  (skip [heads] or NULL);  y = v / rms(v over its part) * w,  the row of heads * P elements
 * in `groups` equal parts, w [heads * P] */
int dihip_gate_group_rmsnorm(void* stream, void* y, int y_dtype, long ldy, const float* o, long ldo, const float* x, long ldx,
                             const void* skip, const float* z, long ldz, const void* w, int w_dtype, float eps, int T, int heads, int P,
                             int groups);
/* Attention through a latent with ONE rotated key part shared by the heads.  ckv[t] = [R latent | rot key part] (f32): the page
 * row of the token (Rp elements) becomes [latent / rms * gamma | rotated key part | zeros]  (spans NULL: nothing is appended --
 * a layer that reads another layer's pages).  q_rot[t] = [H][rot]: every head's rotated query part goes to ql[t][h * Rp + R ..]
 * (behind the head's absorbed query).  Rotation: dimension i with i + rot / 2 by the angle float(pos) * freq[i]. */
int dihip_latent_rope_append(void* stream, void* const* spans, int span_stride, int span_len, int cache_dtype, const float* ckv,
                             long ldc, const void* gamma, int w_dtype, float eps, int R, int rot, int Rp, const float* freq,
                             const float* q_rot, long ldqr, float* ql, long ldql, int H, const int32_t* tok_slot,
                             const int32_t* tok_pos, int T);

/* State-space mixer with a scalar decay per head and a matrix state [D, DV] per head and slot (the state kernels of dihip_gla):
 *   step = softplus(dt[t, h] + dt_bias[h]);  S <- exp(-exp(a_log[h]) * step) S + step * B[t, g] x[t, h]^T;  out[t, h] = S^T C[t, g]
 * g = h / (H / G).  x [T, H * DV], B / C [T, G * D], dt [T, H] f32 rows; workspace: dihip_gla_workspace_bytes. */
int dihip_ssd(void* stream, float* out, long ldo, const float* x, long ldx, const float* B, long ldb, const float* Cq, long ldc,
              const float* dt, long lddt, const void* dt_bias, const void* a_log, int w_dtype, float* state, const int32_t* ent_slot,
              const int32_t* ent_row0, const int32_t* ent_count, int T, int E, int max_count, int H, int G, int D, int DV, int chunked,
              void* ws, size_t ws_bytes);

/* Grouped-query attention whose softmax maps are mixed between the heads after the softmax:
 *   w_g(i, j) = softmax over the row's window of q_g(i) . k(j) * scale * temp[g];  out_h(i) = sum_j (sum_g talk[h, g] w_g(i, j)) v(j)
 * q: f32 rows [H, D] (already rotated), keys [G, D] and values [G, DV] in their pages, head h reads key/value head h / (H / G);
 * window <= 0: every key up to the row's own; temp [H] or NULL, talk [H, H] (w_dtype); gate: f32 [T, H * DV] multiplier or NULL;
 * out: rows [H * DV] of out_dtype.  nsplit: parts of the key walk (a host choice); workspace: the statistics and the parts. */
size_t dihip_talk_attn_workspace_bytes(int T, int H, int DV, int nsplit);
int dihip_talk_attn(void* stream, void* out, int out_dtype, long ldo, const float* q, long ldq, void* const* kspans, void* const* vspans,
                    int span_stride, int span_len, int cache_dtype, const void* temp, const void* talk, int w_dtype, const float* gate,
                    long ldg, const int32_t* tok_slot, const int32_t* tok_pos, int T, int H, int G, int D, int DV, float scale,
                    int window, int nsplit, void* ws, size_t ws_bytes);

/* The same attention for few rows (decoding): the work spread over (row, head, 64-key chunk) workgroups.  max_keys: a host bound on
 * the keys a row reads (min(window, last position + 1)).  Workspace: the raw scores, the chunks' statistics and the parts. */
size_t dihip_talk_attn_few_workspace_bytes(int T, int H, int DV, int max_keys);
int dihip_talk_attn_few(void* stream, void* out, int out_dtype, long ldo, const float* q, long ldq, void* const* kspans,
                        void* const* vspans, int span_stride, int span_len, int cache_dtype, const void* temp, const void* talk,
                        int w_dtype, const float* gate, long ldg, const int32_t* tok_slot, const int32_t* tok_pos, int T, int H, int G,
                        int D, int DV, float scale, int window, int max_keys, void* ws, size_t ws_bytes);
/* The same attention on the matrix cores (bf16 pages; H <= 32, D % 32 == 0 <= 128, DV % 16 == 0 <= 128, span_len % 16 == 0): rows as
 * portions (ent_slot / ent_row0 / ent_count [E], max_count = the largest portion: a host number that sizes the grid), the whole key
 * walk of a 16-row tile in one workgroup.  talk32: the mixing matrix as f32 [H, H].  The weights are mixed in f32 and handed to the
 * value product in bf16.  Workspace: the (maximum, denominator) of every (row, head). */
int dihip_talk_attn_mc_supported(int H, int G, int D, int DV, int span_len, int cache_dtype);
size_t dihip_talk_attn_mc_workspace_bytes(int T, int H);
int dihip_talk_attn_mc(void* stream, void* out, int out_dtype, long ldo, const float* q, long ldq, void* const* kspans,
                       void* const* vspans, int span_stride, int span_len, const void* temp, int w_dtype, const float* talk32,
                       const float* gate, long ldg, const int32_t* tok_pos, const int32_t* ent_slot, const int32_t* ent_row0,
                       const int32_t* ent_count, int E, int max_count, int T, int H, int G, int D, int DV, float scale, int window,
                       void* ws, size_t ws_bytes);

/* Grouped-query attention, step 1: per token the rows qkv[t] hold q [H, maps, D] at column q_off, k [G, maps, D] at k_off,
 * v [G, DV] at v_off (f32; maps = the softmax maps per head, 1 for ordinary attention).  Every query and key head is divided by its root mean square and scaled by qnorm / knorm [D] (NULL: no norm),
 * then rotated on its first rot_dims dimensions by the angles tok_pos[t] * freq[i] (f32 product; layout 0: dimension 2i
 * with 2i + 1, layout 1: i with i + rot_dims / 2; cos and sin times `mag`).  Queries are written back in place, keys go to
 * the key pages (rows of G * maps * D elements of cache_dtype), values to the value pages (rows of G * DV) after
 *   v <- (1 - lam) v + lam vfirst_in[t]   (vfirst_in NULL: v as it is);   vfirst_out[t] <- v   (NULL: not kept). */
int dihip_qkv_prep_append(void* stream, float* qkv, long ld, int q_off, int k_off, int v_off, int H, int G, int D, int DV, int maps,
                          const void* qnorm, const void* knorm, int w_dtype, float eps, const float* freq, int rot_dims,
                          int layout, float mag, float lam, const float* vfirst_in, float* vfirst_out, long ldvf,
                          void* const* kspans, void* const* vspans, int span_stride, int span_len, int cache_dtype,
                          const int32_t* tok_slot, const int32_t* tok_pos, int T);

/* step 2: causal attention of every row over its sequence's pages; query head h reads key/value head h / (H / G):
 *   s_j = scale * q[t, h, m] . k_j[m],  softcap > 0: s_j <- softcap * tanh(s_j / softcap),
 *   over the keys j <= p = tok_pos[t] with  p - j < window  or  j < keep_first  (window <= 0: every j <= p)
 *   p = softmax over {s_j} and, with sink_mode 1 / 2, one more logit sink[h] / 0 that has no value
 *   out[t, h, m] = gate[t, h] * sum_j p_j v_j   (gate NULL: 1)
 * for every map m < maps of the head (each a softmax of its own over the same values).
 * q [T, H, maps, D], out [T, H, maps, DV] f32.  Every product and sum in f32. */
int dihip_gqa_attn(void* stream, float* out, long ldo, const float* q, long ldq, void* const* kspans, void* const* vspans,
                   int span_stride, int span_len, int cache_dtype, const void* sink, int w_dtype, int sink_mode, float softcap,
                   const float* gate, long ldg, const int32_t* tok_slot, const int32_t* tok_pos, int T, int H, int G, int D,
                   int DV, float scale, int maps, int window, int keep_first);
/* the same on the matrix cores for bf16 pages (D, DV multiples of 8 up to 256 / 128, span_len a multiple of 32): rows given
 * as portions, the key walk split over nsplit workgroups (see dihip_latent_window_attn_mc).  diff_out != NULL (maps == 2):
 * dihip_maps_diff_norm of the result goes to diff_out [T, H, DV] (rows of ldd elements of diff_dtype) -- inside the merge of a
 * split walk, else as a launch of its own; `out` is then scratch. */
int dihip_gqa_attn_mc_supported(int D, int DV, int span_len, int cache_dtype);
size_t dihip_gqa_attn_mc_workspace_bytes(int T, int H_times_maps, int DV, int nsplit);
int dihip_gqa_attn_mc(void* stream, float* out, long ldo, const float* q, long ldq, void* const* kspans, void* const* vspans,
                      int span_stride, int span_len, const void* sink, int w_dtype, int sink_mode, float softcap,
                      const float* gate, long ldg, const int32_t* tok_pos, const int32_t* ent_slot, const int32_t* ent_row0,
                      const int32_t* ent_count, int E, int max_count, int T, int H, int G, int D, int DV, float scale,
                      int maps, int window, int keep_first, int nsplit, void* ws, size_t ws_bytes, void* diff_out, int diff_dtype,
                      long ldd, float lam, float out_scale, float eps);
/* two maps per head -> one (differential attention):  d = x[t, h, 0] - lam * x[t, h, 1];
 *   y[t, h, :] = d / sqrt(mean(d^2) + eps) * out_scale        x f32 [T, H, 2, DV], y [T, H, DV] of y_dtype */
int dihip_maps_diff_norm(void* stream, void* y, int y_dtype, long ldy, const float* x, long ldx, float lam, float out_scale,
                         float eps, int T, int H, int DV);

/* Gated linear attention, per head and portion, rows in order, f32:
 *   alpha = sigmoid(z[t, h, :])^(1 / tau);   S <- diag(alpha) S + k[t, h] v[t, h]^T;   out[t, h] = S^T (q[t, h] * q_scale)
 * S: state [slots][H][D][DV] f32, read at the portion's start and written back at its end.  chunked != 0: portions cut into
 * chunks of 64 rows that run side by side (f32 rounding differs).  ws: .._workspace_bytes, always needed (the rows' decays,
 * keys and scaled queries are staged there). */
size_t dihip_gla_workspace_bytes(int T, int E, int max_count, int H, int D, int DV, int chunked);
int dihip_gla(void* stream, float* out, long ldo, const float* q, long ldq, const float* k, long ldk, const float* v, long ldv,
              const float* z, long ldz, float q_scale, float tau, float* state, const int32_t* ent_slot,
              const int32_t* ent_row0, const int32_t* ent_count, int T, int E, int max_count, int H, int D, int DV,
              int chunked, void* ws, size_t ws_bytes);
/* y[t, h, :] = x[t, h, :] / sqrt(mean(x[t, h, :]^2) + eps) * gamma * mul[t, h, :]   (gamma [DV] shared by the heads; mul NULL: 1) */
int dihip_head_rmsnorm_mul(void* stream, void* y, int y_dtype, long ldy, const float* x, long ldx, const void* gamma,
                           int w_dtype, float eps, const float* mul, long ldm, int T, int H, int DV);

/* Mixture of experts: per token the `top` experts of largest logit (ties: the lower index) and the softmax over the chosen
 * logits (scoring 0), or scores = softmax over all E logits, the `top` experts of largest score + correction[e] (correction
 * [E] of w_dtype, NULL: none) and weights = their scores / (the sum of their scores + 1e-20) (scoring 1) -> ids / wts [T, top]; the T * top (token, choice) pairs grouped by expert -> seg [E + 1], src_row [T * top] (the
 * token a sorted row reads), dst [T * top] (the sorted row of pair t * top + k); counts: [E] scratch.
 * ngroups > 1: the experts form ngroups equal groups of neighbours; a group counts by its largest score (scoring 1) or logit, and
 * only experts of the `keep` best groups can be chosen (ngroups = keep = 1: no limit). */
int dihip_seq_moe_route(void* stream, const float* logits, long ldl, int32_t* ids, float* wts, int32_t* counts, int32_t* seg,
                    int32_t* src_row, int32_t* dst, int T, int E, int top, int scoring, const void* correction, int w_dtype,
                    int ngroups, int keep);
/* unit 0: y[r, c] = g * sigmoid(slope * g) * (u + 1),  g = min(gu[r, c], limit),  u = clamp(gu[r, F + c], -limit, limit)
 * unit 1: y[r, c] = silu(gu[r, c]) * gu[r, F + c] */
int dihip_seq_moe_glu(void* stream, void* y, int y_dtype, long ldy, const float* gu, long ldgu, int R, int F, float limit,
                  float slope, int unit);
/* out[t] = sum_k wts[t, k] * rows[dst[t * top + k]] (+ add[t]),  k ascending.  ids != NULL: a choice ids[t * top + k] >= n_real
 * is an identity expert, its row is the token's own row own[t] (of own_dtype).  add NULL: nothing added. */
int dihip_seq_moe_combine(void* stream, float* out, long ldo, const float* rows, long ldr, const int32_t* dst, const float* wts,
                      int T, int top, int K, const int32_t* ids, int n_real, const void* own, int own_dtype, long ldown,
                      const float* add, long ldadd);

/* h[t, :] = float(table[ids[t], :]) + float(table2[rows2[t], :])   (table2 NULL: the first term alone) */
int dihip_embed_sum(void* stream, float* h, const int32_t* ids, const void* table, const int32_t* rows2,
                    const void* table2, int w_dtype, int T, int K);

/* y[t, :] = float(table[ids[t], col0 .. col0 + K)) * scale;  table rows of ldt elements of w_dtype, y rows of ldy of y_dtype */
int dihip_embed_rows(void* stream, void* y, int y_dtype, long ldy, const int32_t* ids, const void* table, int w_dtype,
                     long ldt, long col0, float scale, int T, int K);

/* y[i, :] = x[r, :] / sqrt(mean(x[r, :]^2) + eps) * (gamma_add + gamma) * out_scale,  r = row_idx ? row_idx[i] : i;  x f32 rows
 * of stride ldx  (gamma_add 1: a weight stored as its deviation from one) */
int dihip_rmsnorm_strided(void* stream, void* y, int y_dtype, long ldy, const float* x, long ldx,
                          const int32_t* row_idx, const void* gamma, int w_dtype, float gamma_add, float out_scale, float eps,
                          int M, int K);

/* The residual step of a layer with a norm before and after every sublayer, fused with the next sublayer's input norm:
 *   xo = x_in + m / rms(m) * (add_m + gamma_m)      (m NULL: xo = x_in, x_out unused)
 *   x_out = xo;   xc = xo  (a copy of xc_dtype in rows of stride ldc; NULL: none);
 *   h = xo / rms(xo) * (add_h + gamma_h)            (of h_dtype, rows of stride ldh; NULL: none)
 * rms(v) = sqrt(mean(v^2) + eps).  x_in / x_out: contiguous [T, K] f32 (may alias). */
int dihip_residual_norm_step(void* stream, float* x_out, const float* x_in, const float* m, long ldm, const void* gamma_m,
                             float add_m, const void* gamma_h, float add_h, int w_dtype, float eps, void* xc, int xc_dtype,
                             long ldc, void* h, int h_dtype, long ldh, int T, int K);
/* the same norm, written into the paged cache at (tok_slot[t], tok_pos[t]): span row of K elements of cache_dtype */
int dihip_norm_span_append(void* stream, void* const* spans, int span_stride, int span_len, int cache_dtype,
                           const float* x, long ldx, const void* gamma, int w_dtype, float eps,
                           const int32_t* tok_slot, const int32_t* tok_pos, int T, int K);

/* The residual step with the norm on the sublayer's OUTPUT and the depth-weighted stream:
 *   x_out[t] = x_in[t] + rmsnorm(m[t]; gamma, eps)
 *   n_mix > 0:  stack[n_mix - 1][t] = x_out[t];  x_mix[t] = sum_{j < n_mix} mix_w[j] * stack[j][t]
 * stack: [.][stack_stride] f32 (stack_stride >= T * K elements per level); x_out may alias x_in.
 * next16 (may be NULL): [T, K] bf16 copy of what the next product reads (x_mix where n_mix > 0, else x_out): the product
 * rounds its operand to bf16 anyway, so reading the copy changes no bit and halves its operand traffic. */
int dihip_norm_residual_mix(void* stream, float* x_out, const float* x_in, const float* m, long ldm,
                            const void* gamma, int w_dtype, float eps, float* stack, size_t stack_stride,
                            const void* mix_w, int n_mix, float* x_mix, void* next16, int T, int K);

/* Windowed attention of every row over its sequence's cached latent rows, all heads sharing the cache:
 *   s_j = scale * q[t, h, :] . c_j   for  0 <= tok_pos[t] - j < window  (window <= 0: every j <= tok_pos[t]),
 *   p = softmax over {s_j} and one extra logit sink[h] that has no value (sink NULL: none),
 *   out[t, h, :] = sum_j p_j c_j.
 * q, out: f32 [T, H, R] (rows of stride ldq / ldo); the cache holds rows of R elements of cache_dtype. */
int dihip_latent_window_attn(void* stream, float* out, long ldo, const float* q, long ldq, void* const* spans,
                             int span_stride, int span_len, int cache_dtype, const void* sink, int w_dtype,
                             const int32_t* tok_slot, const int32_t* tok_pos, int T, int H, int R, int window,
                             float scale, int math);

/* The same attention on the matrix cores for a bf16 cache (R a multiple of 32 up to 512, span_len a multiple of 32; see
 * .._supported): the rows are given as portions (ent_*: [E], rows ent_row0 .. + ent_count of one slot at consecutive
 * positions from tok_pos[ent_row0]; max_count = the largest ent_count).  nsplit > 1 splits every row's key walk over
 * that many workgroups (few rows: decoding) and merges the partial softmax records in a second launch through `ws`
 * (.._workspace_bytes).  Operands are rounded to bf16, sums are f32; a row's result depends on the tiling only by rounding. */
int dihip_latent_window_attn_mc_supported(int R, int span_len, int cache_dtype);
size_t dihip_latent_window_attn_mc_workspace_bytes(int T, int H, int R, int nsplit);
int dihip_latent_window_attn_mc(void* stream, float* out, long ldo, const float* q, long ldq, void* const* spans,
                                int span_stride, int span_len, const void* sink, int w_dtype, const int32_t* tok_pos,
                                const int32_t* ent_slot, const int32_t* ent_row0, const int32_t* ent_count, int E,
                                int max_count, int T, int H, int R, int window, float scale, int nsplit, void* ws,
                                size_t ws_bytes);

/* u[t, c] = bias[c] + sum_{k < taps} w[c, k] * src(t, k),  src = x[t - (taps - 1 - k), c] inside the portion, else the
 * slot's tail state [slots][taps - 1][C] f32 (the last taps - 1 inputs of the sequence; zeros at its start); act: 0, or 5 for
 * silu on the result */
int dihip_causal_conv_state(void* stream, float* u, long ldu, const float* x, long ldx, const void* w,
                            const void* bias, int w_dtype, const float* tail, const int32_t* tok_slot,
                            const int32_t* tok_off, int T, int C, int taps, int act);
/* after it: tail <- the last taps - 1 inputs of every portion (ent_slot / ent_row0 / ent_count: [E]) */
int dihip_conv_tail_update(void* stream, float* tail, const float* x, long ldx, const int32_t* ent_slot,
                           const int32_t* ent_row0, const int32_t* ent_count, int E, int C, int taps);

/* Real-gated linear recurrence, per channel c and portion, rows in order:
 *   a = exp(-decay * r[t, c] * softplus(lam[c]));  S = a * S + sqrt(1 - a^2) * i[t, c] * u[t, c];  out[t, c] = S * y[t, c]
 * S: state [slots][C] f32, read at the portion's start and written back at its end.  r, i, u, y, out: f32 rows. */
int dihip_gated_recurrence(void* stream, float* out, long ldo, const float* r, const float* i, long ldg,
                           const float* u, long ldu, const float* y, long ldy, const void* lam, int w_dtype,
                           float decay, float* state, const int32_t* ent_slot, const int32_t* ent_row0,
                           const int32_t* ent_count, int E, int C);
/* the same recurrence with every portion cut into chunks of 64 rows that run side by side (three launches: compose each
 * chunk from zero, carry the states over the chunks, run the chunks from their true start states): for long portions.
 * The result differs from the row-by-row form by f32 rounding only.  max_count = the largest ent_count. */
size_t dihip_gated_recurrence_chunked_workspace_bytes(int E, int max_count, int C);
int dihip_gated_recurrence_chunked(void* stream, float* out, long ldo, const float* r, const float* i, long ldg,
                                   const float* u, long ldu, const float* y, long ldy, const void* lam, int w_dtype,
                                   float decay, float* state, const int32_t* ent_slot, const int32_t* ent_row0,
                                   const int32_t* ent_count, int E, int max_count, int C, void* ws, size_t ws_bytes);

#ifdef __cplusplus
}
#endif
#endif
