/*
 * tllm_stack_api.h - ragged-batch step executor for decoder stacks that are described at run time.
 *
 * Where tllm_runtime_api.h runs one fixed network (the LLaMA decoder) on a rectangular batch, this engine runs a stack whose
 * layers are listed in its configuration - each a token mixer of a registered kind plus an optional gated feed-forward - on a
 * PACKED batch: a step carries, side by side, portions of prompts and single decoded tokens of several sequences.  What a
 * sequence leaves behind lives in two stores that the caller's cache manager hands out (tensorrt_llm.runtime.KVCacheManager /
 * StateSlotManager): pages of a block pool shared by all attention layers (one block id is valid in every layer's pool) and
 * state slots for the recurrent layers.  The engine owns the memory, the caller owns the bookkeeping: a step names, per entry,
 * the position of its first token, its slot and its block table.
 *
 * Mixer kinds: "attention" (grouped-query, `maps` attention maps per head over shared values - 2 = differential attention -,
 * interleaved rotary positions on the first rot_dims dimensions with YaRN-style frequency scaling, tanh soft cap, per-head RMS
 * norm of the output; optionally projection biases, unit-RMS queries and keys, a per-head temperature, a linear or logarithmic
 * distance penalty, a sliding-window or chunked mask, sigmoid weights instead of a softmax, a softmax sink, a per-head output
 * gate; a window that also keeps the sequence's first keys, values that are the keys as projected, weights mixed across heads by a
 * learned matrix after the softmax, a gate per output channel, weighted q / k norms, three-band frequency scaling, an output bias),
 * "latent_attention" (keys and values expanded from one low-rank latent per token plus one rotated key part shared by the
 * heads; the cache holds the latent and that part, attention runs in the absorbed form; optionally queries expanded from a normed
 * latent of their own, half-split rotation pairs with YaRN-style frequency scaling, a window or chunk mask, a softmax sink), "hgrn2"
 * (gated linear recurrence with a lower-bounded forget gate, fp32 state) and "mamba2" (selective state-space layer: a short causal
 * convolution whose last inputs are part of the state, S <- exp(-exp(A_log) dt) S + dt B x^T per head over grouped B / C, skip, gate,
 * RMS norm in parts of the row) and "delta_rule" (gated delta rule with a decay per key channel: q | k | v through a short causal
 * convolution and silu, unit q and k, S <- diag(g) S, u = beta (v - S^T k), S <- S + k u^T, o = S^T q; RMS norm per head and a low-rank
 * sigmoid gate).  The embedding may add a hashed row per (previous token, token) pair, and every mixer's normed input may be blended
 * with the previous token's (token shift); both carry one item per sequence in its state slot.  Feed-forwards: gated dense, relu^2, or a routed mixture of gated experts (softmax router with a
 * choice correction, groups of experts of which only the best can be chosen, identity experts).  A layer may run on an earlier
 * layer's weights (layer.<i>.weights_of), with a cache / state of its own.  Two block forms: parallel sublayers on one residual whose updates are gated by
 * sigmoid(W h + b), RMS norms in groups, a range of layers optionally run several times in a row (every pass with a cache / state
 * of its own); or sequential pre-norm sublayers on `streams` hyper-connected residual copies (u = sum_s in[s] x_s feeds the
 * sublayer, x_t <- sum_s mix[s, t] x_s + out[t] y lands its result; the output norm reads sum_s x_s).
 *
 * Element type bfloat16: weights, activations and caches in bfloat16, fp32 accumulation, and fp32 for the residual stream, norms,
 * scores and softmax, rotation angles, gates of a recurrence and its state.  float32: everything in fp32 with plain FMAs.
 *
 * Errors: NULL / non-zero + tllm_last_error().  Nothing synchronises except tllm_stack_step (it returns host results).
 */
#ifndef TLLM_STACK_API_H
#define TLLM_STACK_API_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tllm_stack* tllm_stack_t;

/* Configuration text, one key=value per line:
 *   dtype (bfloat16 | float32), width, vocab, num_layers, norm_groups (1), norm_eps (1e-5), embedding_scale (1),
 *   loop_start, loop_stop, loop_times (0, 0, 1: no loop), page_size (64), num_blocks, num_slots, debug_taps (0),
 *   block (parallel | sequential), residual (gated | hyper; parallel goes with gated, sequential with hyper), streams (1 .. 8),
 *   norm_offset (0: a norm weight is applied as norm_offset + stored value),
 *   pair_buckets (0: none; the tensor `bigram` [pair_buckets + 1, width] adds row (prev * pair_mul_prev + token * pair_mul_cur) mod
 *     pair_buckets to a token's embedding, its last row to a sequence's first token), pair_mul_prev, pair_mul_cur,
 *   token_shift (0 | 1: the mixer reads h + (h_prev - h) * l<i>.shift, h the normed row; sequential blocks only),
 *   per layer i: layer.<i>.type (attention | latent_attention | hgrn2 | mamba2 | delta_rule), .heads, .dim, .vdim, .ff (0: no feed-forward),
 *     .weights_of (an earlier layer with weights of its own; sequential blocks only),
 *     .mlp (gelu_gate: W_down (gelu_tanh(W_gate h) * W_up h) | relu2: W_down relu(W_up h)^2 | moe: .experts experts
 *       W_down (silu(W_gate h) * W_up h) of size .ff plus .identity identity outputs, .top chosen per token among the .route_keep best
 *       of .route_groups equal groups, weights = softmax score * .route_scale; .route_score softmax | sigmoid (every output's
 *       score by itself), .route_weight output | input (an expert runs on weight x row and the outputs are summed as they
 *       are); relu2 and moe in sequential blocks only),
 *     attention: .kv_heads, .maps (1 | 2), .diff (the constant of the second map's weight and of the output scale 1 - diff),
 *       .scale, .softcap (0: none), .head_norm (0 | 1), .rot_dims, .rot_base, .rot_factor (0: no frequency scaling),
 *       .rot_original, .rot_fast, .rot_slow, .qkv_bias (0 | 1), .qk_norm (0 | 1: q and k / their RMS over dim), .head_temp (0 | 1),
 *       .pos_bias (none | linear: slope_h = 2^(-slope_base (h + 1) / heads) | log: r1_h ln(1 + r2_h (i - j))), .slope_base (8),
 *       .mask (causal | window | chunk), .mask_size, .mask_keep (windows: the first keys every row keeps seeing), .weights (softmax |
 *       sigmoid), .sink (0 | 1: learned per head | 2: a constant logit of 0), .out_gate (0 | 1), .gate_wide (0 | 1: a gate per output
 *       channel), .talk (0 | 1: weights mixed across heads by mix.talk [heads, heads]), .values_are_keys (0 | 1: no value projection),
 *       .qk_norm_weight (0 | 1: mix.q.norm / mix.k.norm [dim]), .o_bias (0 | 1), .rot_scaling (yarn | banded: .rot_low, .rot_high);
 *     latent_attention: .kv_rank, .rot_dim (size of the shared rotated part), .rot_dims (how many of them turn), .rot_base, .scale,
 *       .q_rank (0: queries straight from the input), .rot_pairing (neighbours | halves), .rot_factor / .rot_original / .rot_fast /
 *       .rot_slow, .mask, .mask_size, .sink;
 *     mamba2: .state (rows of a head's state; takes the place of .dim), .groups, .conv (taps), .ssm_norm_groups;
 *     delta_rule: .kv_heads (q / k heads), .conv (taps), .decay_rank, .gate_rank (of the two low-rank pairs).
 * Weights are named l<i>.norm1, l<i>.norm2, l<i>.mix.{q,k,v,o,lq1,lk1,lq2,lk2} (attention; with the options also q.b, k.b, v.b,
 * temp, r1, r2, sink, pb, g, talk, q.norm, k.norm, o.b), l<i>.mix.{q,dkv,dkv.norm,uk,uv,o} (latent_attention; with a query latent dq, dq.norm, uq instead of q;
 * sink), l<i>.mix.{q,f,f.b,lower,v,norm,o} (hgrn2), l<i>.mix.{in,conv,conv.b,dt_bias,A_log,D,norm,o} (mamba2),
 * l<i>.mix.{q,k,v,q.conv,k.conv,v.conv,b,a1,a2,dt_bias,A_log,g1,g2,norm,o} (delta_rule), l<i>.shift (token shift), bigram,
 * l<i>.mlp.{gate,up,down} (moe: l<i>.mlp.e<k>.{gate,up,down}, l<i>.mlp.router, l<i>.mlp.correction), l<i>.rg1, l<i>.rg1.b, l<i>.rg2, l<i>.rg2.b (gated residual), l<i>.hc{1,2}.{in,out,mix} (hyper
 * residual; absent with one stream: the plain sum), embed, loop.step, final.norm, head; linear weights [out, in]. */
tllm_stack_t tllm_stack_create(const char* config_text);

/* One weight tensor from HOST memory; dtype 0 = fp32, 7 = bfloat16 (nvinfer1::DataType codes).  Converted to the engine's element
 * type on the way in. */
int32_t tllm_stack_set_tensor(tllm_stack_t s, const char* name, int32_t dtype, const int64_t* dims, int32_t nbDims, const void* data);

/* Resolves the weights against the configuration (names the first missing / mis-shaped one), fuses the projections that share an
 * input, allocates block pools and state slots. */
int32_t tllm_stack_finalize(tllm_stack_t s);

typedef struct
{
    int32_t n_tokens, n_entries, n_want, max_blocks;
    const int32_t* tokens;      /* [n_tokens] ids, entries back to back */
    const int32_t* ent_count;   /* [n_entries] tokens of each entry (>= 1) */
    const int32_t* ent_pos0;    /* [n_entries] position of the entry's first token in its sequence (0: a new sequence) */
    const int32_t* ent_slot;    /* [n_entries] state slot of the sequence */
    const int32_t* block_table; /* [n_entries, max_blocks] block ids of the sequence, in order */
    const int32_t* want_rows;   /* [n_want] rows of the packed batch whose logits are asked for */
} tllm_stack_batch_t;

/* Runs one step.  logits_out: host fp32 [n_want, vocab] or NULL; next_ids_out: host int32 [n_want] (arg-max of each wanted row, the
 * greedy sampler) or NULL.  Every index is checked on the host before anything is launched. */
int32_t tllm_stack_step(tllm_stack_t s, const tllm_stack_batch_t* batch, float* logits_out, int32_t* next_ids_out, void* stream);

/* Geometry the cache manager needs. */
int32_t tllm_stack_page_size(tllm_stack_t s);
int32_t tllm_stack_num_blocks(tllm_stack_t s);
int32_t tllm_stack_num_slots(tllm_stack_t s);
int32_t tllm_stack_vocab(tllm_stack_t s);
int32_t tllm_stack_layer_runs(tllm_stack_t s); /* layers as executed, a looped layer counted once per pass */
int64_t tllm_stack_weight_bytes(tllm_stack_t s);
/* bytes one step moves at least: weights once, plus the cache / state the given contexts touch (roofline denominators); of a
 * routed feed-forward the experts that the step's tokens reach when every choice falls on another expert */
int64_t tllm_stack_step_bytes(tllm_stack_t s, int32_t n_tokens, int64_t context_tokens, int32_t n_entries);

/* debug_taps=1: the residual stream behind layer run `run` of the last step (the sum of the streams, if there are several), fp32
 * [n_tokens, width], to host memory. */
int32_t tllm_stack_get_tap(tllm_stack_t s, int32_t run, float* out, size_t n_floats);

void tllm_stack_destroy(tllm_stack_t s);

#ifdef __cplusplus
}
#endif
#endif
