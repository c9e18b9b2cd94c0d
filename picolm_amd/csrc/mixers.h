// Called operations of the library's own (csrc/engine.h, PICOLM_OP_CALL): mixers with state, an
// attention with a bias by distance and a sink, and the row-wise steps around them.  Each is a
// function `int f(void* user, const picolm_step_view*)` whose `user` is one of the structures
// below; a part of a model names it in ProgramBuilder.call.  Sizes, offsets and constants are
// fields: no function knows which model it runs in.
//
// Rows are dense: a row of a buffer has the width its structure names, whatever the buffer's own
// row size (buffers are shared between operations and sized for the widest).
#pragma once
#include <stdint.h>

#include "engine.h"

#ifdef __cplusplus
extern "C" {
#endif

// x <- step, joined <- [x ; first] (engine dtype): what a pass over a looped stretch of layers does
// before its product  x += W_in joined.
//   in: `first` float rows [width] (the embedding's output); out: x float rows [width];
//   extra[0]: joined rows [2 width] in the engine's dtype
typedef struct {
    const float* step;       // [width], this pass's vector
    int32_t width;
} picolm_loop_input_args;
int picolm_call_loop_input(void* user, const picolm_step_view* v);

// Softmax attention over the cache entry with biases of the projections, a rotation by position, a
// norm of queries and keys, a bias by distance, a sink and an output gate, each optional.  A token's
// q and k are prepared in this order: the projection's bias is added, the first rot_dims entries are
// turned by the position, the norm is taken; values only get their bias.
//   in: float rows [in_stride] holding q [H d], k [G d], v [G dv] and the gate's pre-activations
//   [H dv] at the offsets named (v_off may name the keys' place: the values are then the keys as
//   projected); out: rows [H dv] in the engine's dtype (float with out_float); extra[0]: scratch rows
//   [H d] in the engine's dtype.  Flags: PICOLM_CALL_KV | PICOLM_CALL_ATTENDS, partial_floats =
//   H (dv + 2), tile_rows = picolm_attn_plain_mfma_tile_rows() where the engine runs in bfloat16 and
//   picolm_attn_plain_mfma_takes(d, dv) (the matrix-core kernel then runs), else
//   picolm_attn_prefill_tile_rows().  The operation writes its own pages: as plain arrays, or for the
//   matrix-core kernel in the order of its operands.
// maps > 1: a head's d entries are `maps` queries (and a KV head's `maps` keys) of d / maps entries
//   side by side, each an attention of its own over the same values: query m of a head meets part m of
//   the cached key.  The attention then runs over H maps heads: out rows [H maps][dv], scratch rows
//   [H maps][d], partial_floats = H maps (dv + 2); norm and rotation cover each part by itself; no
//   gate and no bias by distance; a sink has H maps entries.
typedef struct {
    int32_t n_heads, n_kv_heads, head_dim, v_head_dim;
    int32_t in_stride, q_off, k_off, v_off, gate_off;     // gate_off < 0: no gate
    float scale, eps;
    const float* q_norm;     // [head_dim / maps] RMS norm of each query head (null: none), and of each key head
    const float* k_norm;
    const float* bias;       // [H][bias_rows] by distance, the last entry for every distance beyond; null: none
    int32_t bias_rows;
    const float* sink;       // [H] or null
    int32_t window;          // > 0: a query sees its last `window` keys, no more than the cache entry's own window (which
                             // bounds the pages a step visits); 0: what the cache entry's window says
    int32_t chunk;           // > 0: a query sees the keys of its own stretch of `chunk` positions (counted from the
                             // sequence's first position) up to itself
    int32_t maps;            // 0 or 1: one query a head
    int32_t out_float;       // 1: the output rows are float
    int32_t unit_qk;         // 1: queries and keys are divided by their root mean square (eps inside the root) where
                             // q_norm / k_norm give no weight
    const float* in_bias;    // [in_stride]: added to the input row where it is read (null: none)
    const float* cos_table;  // [table_positions][rot_dims / 2]; null: no rotation
    const float* sin_table;
    int32_t table_positions, rot_dims, rot_half;      // rot_half = 1: entry i pairs with i + rot_dims / 2; 0: entry 2i with 2i + 1
} picolm_sink_attention_args;
int picolm_call_sink_attention(void* user, const picolm_step_view* v);

// A short causal convolution over time per channel, with the last taps - 1 inputs of a sequence kept
// in its state: y[t][c] = act(bias[c] + sum_j weight[c][taps-1-j] x[t-j][c]).
//   in: float rows [in_stride], channels at in_off; out: float rows [out_stride], channels at out_off;
//   state: floats [taps-1][channels] at state_off of the slot's state (oldest first).
typedef struct {
    const float* weight;     // [channels][taps]
    const float* bias;       // [channels] or null
    int32_t channels, taps;
    int32_t in_stride, in_off, out_stride, out_off;
    int64_t state_off;       // in floats
    int32_t act;             // 0 none, 1 silu
} picolm_short_conv_args;
int picolm_call_short_conv(void* user, const picolm_step_view* v);

// A matrix state S [key_dim][value_dim] per head and sequence, walked over the step's tokens in
// order, kept in float in the slot's state.  With per-token decay a and strength w (both per head):
//   rule 0 (outer product):  S <- a S + w k v^T;                      o = S^T q + skip v
//   rule 1 (delta rule):     S <- a S;  S <- S + k (w (v - S^T k))^T;  o = S^T q
//   a = exp(-exp(A_log) softplus(raw_a + dt_bias));  w = softplus(raw_w + dt_bias) (rule 0) or
//   sigmoid(raw_w) (rule 1).  unit_qk: q and k are first made unit vectors per head
//   (x / sqrt(sum x^2 + unit_eps)); q is multiplied by q_scale.
//   in: float rows [in_stride] with raw_a and raw_w per head at a_off, w_off; extra[0]: float rows
//   [qkv_stride] with q, k [key_heads][key_dim] and v [heads][value_dim] at q_off, k_off, v_off
//   (changed in place by unit_qk); extra[1]: scratch float rows [2 heads]; out: float rows
//   [heads value_dim].  Head h uses q/k head h / (heads / key_heads).
typedef struct {
    int32_t rule;
    int32_t n_heads, n_key_heads, key_dim, value_dim;
    int32_t in_stride, a_off, w_off;
    int32_t qkv_stride, q_off, k_off, v_off;
    const float* A_log;      // [heads]
    const float* dt_bias;    // [heads]
    const float* skip;       // [heads] or null
    int32_t unit_qk;
    float unit_eps, q_scale;
    int64_t state_off;       // in floats: [heads][key_dim][value_dim]
} picolm_state_scan_args;
int picolm_call_state_scan(void* user, const picolm_step_view* v);
#define PICOLM_STATE_SCAN_MAX_KEY_DIM 256

// RMS norm in equal parts of a row with a gate of silu(g):
//   gate_first = 0:  y = x / rms(x) * weight * silu(g);   gate_first = 1:  y = (x silu(g)) / rms(x silu(g)) * weight
//   the mean is over each part of `group` columns; weight[c % weight_len].
//   in: float rows [width]; extra[0]: float rows [gate_stride], g at gate_off; out: rows [width] in
//   the engine's dtype.
typedef struct {
    const float* weight;
    int32_t weight_len, width, group;
    float eps;
    int32_t gate_first, gate_stride, gate_off;
} picolm_gated_norm_args;
int picolm_call_gated_norm(void* user, const picolm_step_view* v);

// out += mult (a / rms(a) * w_a + b / rms(b) * w_b): two branches that read the same input meet
// the residual rows.  in: a, float rows [width]; extra[0]: b, float rows [width] (null w_b: one
// branch); out: float rows [width].
typedef struct {
    const float* w_a;
    const float* w_b;
    int32_t width;
    float eps, mult;
} picolm_normed_sum_args;
int picolm_call_normed_sum(void* user, const picolm_step_view* v);

// out <- f(in) element by element over rows [width] (`in` absent: in place, one dtype):
//   kind 1: max(x, 0)^2;  kind 2: param tanh(x / param);  kind 3: param x
typedef struct {
    int32_t kind, width;
    int32_t in_dtype, out_dtype;     // PICOLM_F32 / PICOLM_BF16
    float param;
} picolm_map_rows_args;
int picolm_call_map_rows(void* user, const picolm_step_view* v);


// ---- row-wise steps of layers that norm after the sum, shift tokens and gate their branches ------

// x[t][c] += sin(p f_i) for c = 2 i, cos(p f_i) for c = 2 i + 1, p the token's position.
//   out: x float rows [width]
typedef struct {
    const double* freq;      // [ceil(width / 2)], f_i = base^(-2 i / width)
    int32_t width;
} picolm_add_positions_args;
int picolm_call_add_positions(void* user, const picolm_step_view* v);

// What a mixer reads where every token is blended with the one before it:
//   y[t] = x[t] + (x[t-1] - x[t]) * mu, x[-1] of a sequence being what its state holds (zeros at the
//   start); the state then takes the sequence's last x.
//   in: x float rows [width]; out: y rows [width] in the engine's dtype; extra[0] (optional): x
//   itself in the engine's dtype; state: floats [width] at state_off of the slot's state.
typedef struct {
    const float* mu;         // [width]
    int32_t width;
    int64_t state_off;       // in floats
} picolm_token_shift_args;
int picolm_call_token_shift(void* user, const picolm_step_view* v);

// out[c] = x[c] * act(g[c] + bias[c]) over `width` columns; act 0: no gate (a copy into another
// dtype or stride), 1: silu, 2: sigmoid.  g_per_row = 1: one gate a row, the float at g_off, for
// every column (no bias then).
//   in: x rows [x_stride] of x_dtype, columns at x_off; extra[0]: g float rows [g_stride], columns at
//   g_off (act > 0); out: rows [width] of out_dtype.
typedef struct {
    int32_t width, act;
    int32_t x_stride, x_off, x_dtype;
    int32_t g_stride, g_off;
    int32_t out_dtype;
    const float* bias;       // [width] or null
    int32_t g_per_row;
} picolm_gate_rows_args;
int picolm_call_gate_rows(void* user, const picolm_step_view* v);

// RMS norm of a stretch of columns: out[out_off + c] = x[in_off + c] / sqrt(mean_c(x^2) + eps) * weight[c].
//   in: float rows [in_stride]; out: rows [out_stride] of out_dtype.
typedef struct {
    const float* weight;     // [width]
    int32_t width;
    int32_t in_stride, in_off, out_stride, out_off, out_dtype;
    float eps;
} picolm_slice_norm_args;
int picolm_call_slice_norm(void* user, const picolm_step_view* v);

// A product per head: out[h] = W_h in[h] (transposed = 0: W [heads out_dim][in_dim]) or
// out[h] = W_h^T in[h] (transposed = 1: W [heads in_dim][out_dim]), float accumulation, and then
// out *= act(g) with g at the output's columns (gate_act 0: none, 1 silu, 2 sigmoid), or with
// gate_per_head = 1 one g a head, head h's at gate_off + h.
//   in: rows [in_stride] of in_dtype, head h at in_off + h in_head_stride; out: rows [out_stride] of
//   out_dtype, head h at out_off + h out_head_stride (a head stride of 0: the heads lie side by
//   side, in_dim or out_dim apart); extra[0]: g float rows [gate_stride], at gate_off.
typedef struct {
    const void* weight;
    int32_t weight_dt;       // PICOLM_F32 / PICOLM_BF16
    int32_t heads, in_dim, out_dim, transposed;
    int32_t in_stride, in_off, in_dtype;
    int32_t out_stride, out_off, out_dtype;
    int32_t gate_act, gate_stride, gate_off;
    int32_t in_head_stride, out_head_stride, gate_per_head;
} picolm_head_linear_args;
int picolm_call_head_linear(void* user, const picolm_step_view* v);

// The sum and the norm of a layer that norms after adding:
//   x <- (alpha x + u act(g + bias)) / rms(.) * weight          act = sigmoid where g is given, 1 else
//   out: x float rows [width]; in: u float rows [width]; extra[0] (optional): g float rows [width];
//   extra[1] (optional): the new x once more, in the engine's dtype, for the products that read it next.
typedef struct {
    const float* weight;     // [width]
    const float* gate_bias;  // [width] or null
    int32_t width;
    float alpha, eps;
} picolm_gated_postnorm_args;
int picolm_call_gated_postnorm(void* user, const picolm_step_view* v);

// What a matrix state with a forget gate per key channel needs of a token, from pre-activations:
//   q = silu(q_raw);  a = lower + (1 - lower) sigmoid(f_raw + bias);  k = 1 - a
//   in: float rows [in_stride], q_raw and f_raw [channels] at q_off, f_off; out: float rows
//   [3 channels]: q | k | a.
typedef struct {
    const float* lower;      // [channels]
    const float* bias;       // [channels] or null
    int32_t channels, in_stride, q_off, f_off;
} picolm_forget_gates_args;
int picolm_call_forget_gates(void* user, const picolm_step_view* v);

// A matrix state S [key_dim][value_dim] per head and sequence whose every element decays by a
// factor of its own, walked over the step's tokens in order, kept in float in the slot's state:
//   S[i][j] <- a[i][j] S[i][j] + k[i] w[j];   o[j] = sum_i S[i][j] q[i] + skip[j] x[j]
//   kind 1: a[i][j] = a[i], a row's decay, given per token and key head; w = x
//   kind 2: a[i][j] = exp(dt[j] A[j][i]), dt = softplus(dt_raw + dt_bias) per value channel; w = dt x
//   extra[0]: float rows [qk_stride] with q, k (and kind 1: a) [key_heads][key_dim] at q_off, k_off,
//   a_off; in: float rows [x_stride] with x [heads value_dim] at x_off; extra[1] (kind 2): float
//   rows [dt_stride] with dt_raw [heads value_dim] at dt_off; out: float rows [heads value_dim].
//   Head h uses q/k head h / (heads / key_heads).
typedef struct {
    int32_t kind;
    int32_t n_heads, n_key_heads, key_dim, value_dim;
    int32_t qk_stride, q_off, k_off, a_off;
    int32_t x_stride, x_off;
    int32_t dt_stride, dt_off;
    const float* dt_bias;    // [heads value_dim] or null
    const float* A;          // kind 2: [heads value_dim][key_dim], negative
    const float* skip;       // [heads value_dim] or null
    int64_t state_off;       // in floats: [heads][key_dim][value_dim]
} picolm_decay_scan_args;
int picolm_call_decay_scan(void* user, const picolm_step_view* v);

// Layer norm with a weight and an optional bias: out = (x - mean) / sqrt(var + eps) * weight + bias,
// var the mean of the squared deviations, all in float.
//   in: x float rows [width]; out: rows [width] of out_dtype.  gathers = 1: the operation covers the
//   wanted rows, and row i reads the row of x that the step's want_rows[i] names.
typedef struct {
    const float* weight;     // [width]
    const float* bias;       // [width] or null
    int32_t width, out_dtype;
    float eps;
    int32_t gathers;
} picolm_layer_norm_args;
int picolm_call_layer_norm(void* user, const picolm_step_view* v);

// Rotation by position of `heads` stretches of a row: of each stretch's first `dims` entries, entry
// i < dims / 2 is paired with entry i + dims / 2 (half = 1) or entry 2i with 2i + 1 (half = 0); the
// pair (u, v) of a token at position p becomes (u cos - v sin, v cos + u sin) with
// cos = cos_table[p][i], sin = sin_table[p][i]; the stretch's other entries are copied.
//   in: float rows [in_stride], stretch h at in_off + h in_head_stride; out: float rows
//   [out_stride], stretch h at out_off + h out_head_stride (in place: out names the same buffer,
//   and the offsets and strides are equal).
// In the same pass, where in and out are two buffers: `more_heads` further stretches of the same
// shape at offsets and strides of their own (a key part beside the queries' heads, say), and a
// stretch of `norm_width` columns at norm_in_off that is divided by its root mean square (eps inside
// the root), multiplied by norm_weight and written at norm_out_off (more_heads = 0, norm_weight
// null: none).
typedef struct {
    const float* cos_table;  // [table_positions][dims / 2]
    const float* sin_table;
    int32_t table_positions, dims, half, heads, width;      // width: entries of a stretch, >= dims
    int32_t in_stride, in_off, in_head_stride;
    int32_t out_stride, out_off, out_head_stride;
    int32_t more_heads, more_in_off, more_in_head_stride, more_out_off, more_out_head_stride;
    const float* norm_weight;  // [norm_width] or null
    int32_t norm_width, norm_in_off, norm_out_off;
    float norm_eps;
} picolm_rotate_heads_args;
int picolm_call_rotate_heads(void* user, const picolm_step_view* v);

// out[c] += in[c] + vec[c] over `width` columns of float rows: what a pass over a looped stretch of
// layers adds before its first layer (the embedding's rows again, and the pass's vector), or any
// other sum of rows.  in: float rows [width] or absent; vec: [width] or null.
typedef struct {
    const float* vec;
    int32_t width;
} picolm_add_rows_args;
int picolm_call_add_rows(void* user, const picolm_step_view* v);

// Two RMS norms of the same float rows, which share the root: a = x / sqrt(mean(x^2) + eps) * w_a and
// b = the same times w_b: what a layer needs whose two branches read the same rows, each behind a norm
// of its own.  in: x float rows [width]; out: a, rows [width] of out_dtype; extra[0]: b, likewise.
typedef struct {
    const float* w_a;        // [width]
    const float* w_b;
    int32_t width, out_dtype;
    float eps;
} picolm_rms_pair_args;
int picolm_call_rms_pair(void* user, const picolm_step_view* v);

// Two attention maps a head become one: o = a1 - lambda a2, divided by its root mean square over the
// head's `vdim` values (eps inside the root, no weight), times `mult`.
//   in: float rows [heads][2][vdim], map m of head h at (2 h + m) vdim; out: rows [heads vdim] of out_dtype.
typedef struct {
    int32_t heads, vdim, out_dtype;
    float lambda, eps, mult;
} picolm_map_difference_args;
int picolm_call_map_difference(void* user, const picolm_step_view* v);

// ---- a routed feed-forward ---------------------------------------------------------------------
// Each row picks `top` of its `experts` router outputs (ties: the lower index).
//   scoring 0: the largest logits + bias are picked, weighted by the softmax over the picked
//              (biased) logits alone;
//   scoring 1: s = softmax over all the logits; the largest s + bias are picked; the weights are
//              the picked s over their sum (+ 1e-20), times `scale`.
//   scoring 2: s = sigmoid(logit); the largest s + bias are picked; the weights are the picked s
//              themselves, times `scale`.
//   in: float rows [in_stride] (0: experts) whose first `experts` entries are the router logits
//   without bias; out: rows of 2 top words: the picked outputs (int32) and then their weights (float).
typedef struct {
    const float* bias;       // [experts] or null
    int32_t experts, top;
    int32_t scoring, in_stride;
    float scale;             // scoring 1
} picolm_route_top_args;
int picolm_call_route_top(void* user, const picolm_step_view* v);

// The picked experts of every row: y[t][k] = W_down[e] (silu(W_gate[e] h) * (W_up[e] h)), e the k-th
// pick of row t, and their weighted sum  out[t] = sum_k w[t][k] y[t][k] (+ out[t] if `adds`).  A pick
// e with experts <= e < experts + identity stands for an expert that gives its input back:
// y[t][k] = h[t]; such picks read no weights.
//   in: h rows [width] in the engine's dtype; extra[0]: the picks as route_top leaves them; extra[1]:
//   scratch float rows [top ff]; out: float rows [width].  With extra[2], scratch float rows
//   [top width], and extra[3], scratch rows of top + experts + 1 words, a step of many rows in
//   bfloat16 sorts its (row, pick) pairs by expert and runs them through the matrix cores.
typedef struct {
    const void* gate;        // [experts][ff][width]
    const void* up;          // [experts][ff][width]
    const void* down;        // [experts][width][ff]
    int32_t weight_dt;
    int32_t experts, top, width, ff;
    int32_t adds;            // 1: out += the sum; 0: out = the sum
    int32_t identity;        // picks from `experts` up to experts + identity give the row itself
    int32_t act;             // 0: silu(g) * u.  1: g' = min(g, limit), u' = clamp(u, -limit, limit), g' sigmoid(alpha g') (u' + 1)
    float limit, alpha;
    int32_t weight_on_input; // 1: a pick's weight multiplies what its expert reads (g and u before the activation), and the
                             // sum over a row's picks is plain
} picolm_routed_experts_args;
int picolm_call_routed_experts(void* user, const picolm_step_view* v);

#ifdef __cplusplus
}
#endif
