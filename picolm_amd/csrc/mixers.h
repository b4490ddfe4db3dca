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

// Softmax attention over the cache entry with a norm of queries and keys, a bias by distance, a
// sink and an output gate, each optional.
//   in: float rows [in_stride] holding q [H d], k [G d], v [G dv] and the gate's pre-activations
//   [H dv] at the offsets named; out: rows [H dv] in the engine's dtype; extra[0]: scratch rows
//   [H d] in the engine's dtype.  Flags: PICOLM_CALL_KV | PICOLM_CALL_ATTENDS, partial_floats =
//   H (dv + 2), tile_rows = picolm_attn_plain_mfma_tile_rows() where the engine runs in bfloat16 and
//   picolm_attn_plain_mfma_takes(d, dv) (the matrix-core kernel then runs), else
//   picolm_attn_prefill_tile_rows().  The operation writes its own pages: as plain arrays, or for the
//   matrix-core kernel in the order of its operands.
typedef struct {
    int32_t n_heads, n_kv_heads, head_dim, v_head_dim;
    int32_t in_stride, q_off, k_off, v_off, gate_off;     // gate_off < 0: no gate
    float scale, eps;
    const float* q_norm;     // [head_dim] RMS norm of each query head (null: none), and of each key head
    const float* k_norm;
    const float* bias;       // [H][bias_rows] by distance, the last entry for every distance beyond; null: none
    int32_t bias_rows;
    const float* sink;       // [H] or null
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
//   kind 1: max(x, 0)^2;  kind 2: param tanh(x / param)
typedef struct {
    int32_t kind, width;
    int32_t in_dtype, out_dtype;     // PICOLM_F32 / PICOLM_BF16
    float param;
} picolm_map_rows_args;
int picolm_call_map_rows(void* user, const picolm_step_view* v);

#ifdef __cplusplus
}
#endif
