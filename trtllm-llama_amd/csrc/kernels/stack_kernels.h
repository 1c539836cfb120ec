// Host-side launch interface of the kernels behind the ragged-batch stack engine (runtime/stack_engine.cpp): decoder
// stacks whose layers are described at run time (grouped RMS norms, gated residuals or hyper-connected residual streams, looped
// layer ranges, attention over a paged cache in its variants - differential maps, masks, distance penalties, sigmoid weights, sinks,
// a shared latent -, HGRN2 and selective state-space recurrences over per-sequence state slots, routed mixtures of experts).
//
// A step is one packed batch of `tokens` rows: portions of prompts and single decoded tokens of several sequences side
// by side.  Row t belongs to batch entry tok_entry[t] and sits at position tok_pos[t] of its sequence.  Every kernel is
// built for two element types: DT_BF16 (activations, weights and caches in bfloat16; what a recurrence, a norm, a
// softmax or the residual touches in fp32) and DT_FLOAT (everything in fp32, plain FMA, no reduced-precision matrix
// mode).  Same conventions as kernels.h: enqueue on `stream`, never synchronise, 0 on success, negative + set_error on a
// shape that cannot run.
#pragma once
#include "kernels.h"

namespace tllm
{
namespace kernels
{

constexpr int32_t DT_BF16 = 7; // nvinfer1::DataType::kBF16

// ---------------------------------------------------------------------------------------------
// Dense product C[m,n] = sum_k A[m,k] * W[n,k] for the stack engine, with the layer's seam in the epilogue.
//   dtype DT_BF16: MFMA tiles (gemm_mfma.hip, v_mfma_f32_32x32x16_bf16) for M > 8, the streaming skinny kernel below it;
//   dtype DT_FLOAT: fp32 FMA tiles (stack_gemm.hip).
// Epilogue, when `resid` is set: resid[m, n] += sigmoid(gate[m, n] + gate_bias[n]) * C[m, n]  (fp32 residual stream, the
// sublayer's gate taken from another projection's columns); nothing is written to `c` then.  Otherwise `bias` (fp32 [N]) is added
// to the accumulator and `act` is applied to the value rounded to the element type: ACT_RELU2 = max(v, 0)^2.
// `batch` > 1: that many independent products of the same shape, operand b at a + b * stride_a (elements) and so on - the
// per-head products of latent attention (one weight block per head over one slice of a shared row).
// ---------------------------------------------------------------------------------------------
constexpr int32_t ACT_NONE = 0, ACT_RELU2 = 1;

struct StackGemmParams
{
    int32_t dtype = DT_BF16;     // element type of a, w (and of c unless out_f32)
    int32_t out_f32 = 0;         // c is fp32 (logits)
    int32_t M = 0, N = 0, K = 0;
    const void* a = nullptr;
    int64_t lda = 0;             // elements
    const void* w = nullptr;     // [N, K] row-major, K contiguous
    void* c = nullptr;
    int64_t ldc = 0;
    float* resid = nullptr;      // fp32 [M, ldr]
    int64_t ldr = 0;
    const void* gate = nullptr;  // element type `dtype`, [M, ldg]: pre-activation of the gate (null: plain accumulate into resid)
    int64_t ldg = 0;
    const float* gate_bias = nullptr; // fp32 [N] or null
    const float* bias = nullptr;      // fp32 [N] or null (no resid)
    int32_t act = ACT_NONE;           // (no resid)
    int32_t batch = 1;
    int64_t stride_a = 0, stride_w = 0, stride_c = 0; // elements, between the operands of consecutive products
    // Grouped form of a batch (a mixture of experts): device int32 [batch + 1]; product b takes rows [group_off[b], group_off[b + 1]) of
    // a and c (stride_a = stride_c = 0) and weight block b; M is the host's bound on the rows of one group.
    const int32_t* group_off = nullptr;
    int32_t group_rows = 0; // the rows a group is expected to have (tile shapes are chosen for it), 0: M
};
int launch_stack_gemm(const StackGemmParams& p, hipStream_t stream);

// ---------------------------------------------------------------------------------------------
// Pointwise pieces.
// ---------------------------------------------------------------------------------------------
// x[t, :] = table[ids[t], :] * scale (fp32 residual stream); keep (optional) receives the same rows; copies > 1: the row is also
// written to x + c * copy_stride, c < copies (residual streams that all start from the embedding output)
int launch_stack_embed(float* x, float* keep, const int32_t* ids, const void* table, int32_t dtype, int32_t tokens, int32_t width,
    int32_t vocab, float scale, hipStream_t stream, int32_t copies = 1, int64_t copy_stride = 0);
// A hashed pair embedding on top of the rows above: x[t, :] += pair_table[row(t), :], row = (prev[t] * mul_prev + ids[t] * mul_cur) mod
// buckets (64-bit arithmetic), or the extra row `buckets` where prev[t] < 0 (a sequence's first token).  pair_table [buckets + 1, width].
int launch_stack_pair_embed(float* x, const int32_t* ids, const int32_t* prev, const void* pair_table, int32_t dtype, int32_t tokens,
    int32_t width, int32_t buckets, int32_t mul_prev, int32_t mul_cur, hipStream_t stream, int32_t copies = 1, int64_t copy_stride = 0);
// Token shift: h[t, :] = n[t, :] + (n[t - 1, :] - n[t, :]) * mu[:] over fp32 rows n (a norm's output), t - 1 the previous token of the
// same sequence: the row above inside an entry, for an entry's first row the sequence's carried row carry[slot, :] (zeros when the
// entry starts its sequence).  The carry then takes the entry's last row of n.  h in the element type; n is not changed.
struct StackShiftParams
{
    int32_t dtype = DT_BF16;
    int32_t tokens = 0, entries = 0, width = 0;
    const float* n = nullptr;  // [tokens, width]
    const float* mu = nullptr; // [width]
    float* carry = nullptr;    // [slots, width]
    void* h = nullptr;         // [tokens, width]
    const int32_t* tok_entry = nullptr;
    const int32_t* tok_pos = nullptr;
    const int32_t* ent_slot = nullptr;
    const int32_t* ent_first = nullptr;
    const int32_t* ent_count = nullptr;
    const int32_t* ent_pos0 = nullptr;
};
int launch_stack_token_shift(const StackShiftParams& p, hipStream_t stream);
// x[t, :] += (add ? add[t, :] : 0) + (row ? row[:] : 0): the entry of a pass over a looped layer range
int launch_stack_pass_entry(float* x, const float* add, const float* row, int32_t tokens, int32_t width, hipStream_t stream);
// RMS norm in `groups` equal consecutive parts of the row, every part divided by its own sqrt(mean(part^2) + eps); the two
// outputs share the normalised row and differ in their weights (the parallel layer's two norms of the same x).  rows: optional
// gather (row r reads x[rows[r]]).  y2 / w2 may be null.
int launch_stack_group_rmsnorm(void* y1, void* y2, const float* x, const int32_t* rows, const float* w1, const float* w2, int32_t dtype,
    int32_t n_rows, int32_t width, int32_t groups, float eps, hipStream_t stream);
// Hyper-connected residual streams xs[s] = x + s * stream_stride (fp32 [tokens, width] each, `streams` >= 1 of them; one stream with
// mix = out = in = 1 is the plain residual sum).  In one pass over a row:
//   1. y != null: a sublayer's result lands, all streams at once from the old ones: xs[t] <- sum_s mix[s * streams + t] xs[s] + out[t] y
//   2. u = sum_s in[s] xs[s]  (in == null: the plain sum)
//   3. h != null: h = u / sqrt(mean(u^2) + eps) * w   (element type `dtype`: the next sublayer's input)
//      sum_out != null: sum_out = u (fp32)
// rows (optional gather): launch row r works on packed row rows[r] and writes h row r - the last reader of the streams (the output
// norm) only touches the rows whose logits are wanted, and writes nothing back into the streams.  Everything is fp32 but h.  mix / out / in are device arrays.
struct StackHyperParams
{
    int32_t dtype = DT_BF16;
    int32_t tokens = 0, width = 0, streams = 1;
    float* x = nullptr;
    int64_t stream_stride = 0;
    const float* y = nullptr;   // [tokens, width] or null
    const float* mix = nullptr; // [streams, streams], indexed [from, to]
    const float* out = nullptr; // [streams]
    const float* in = nullptr;  // [streams] or null
    void* h = nullptr;
    const float* w = nullptr;   // [width] norm weight as applied (any offset already added)
    float eps = 1e-5f;
    float* sum_out = nullptr;
    float* h32 = nullptr;          // [tokens, width] or null: the normed row in fp32 as well (a token shift reads it)
    const int32_t* rows = nullptr; // [tokens] or null
};
int launch_stack_hyper_norm(const StackHyperParams& p, hipStream_t stream);
// y[t, c] = act(gu[t, c]) * gu[t, ff + c] over a [tokens, ld] projection that holds gate then up columns; act: GATE_GELU_TANH | GATE_SILU
constexpr int32_t GATE_GELU_TANH = 0, GATE_SILU = 1;
int launch_stack_gelu_gate(void* y, const void* gu, int32_t dtype, int32_t tokens, int32_t ff, int64_t ld, hipStream_t stream,
    int32_t act = GATE_GELU_TANH);
// y[r, :n] = x[r, :n] / sqrt(mean(x[r, :n]^2) + eps) * w over rows of the element type with their own strides (a low-rank latent
// inside a wider projection); one wave per row
int launch_stack_row_rmsnorm(void* y, int64_t ldy, const void* x, int64_t ldx, const float* w, int32_t dtype, int32_t rows, int32_t n, float eps,
    hipStream_t stream);

// ---------------------------------------------------------------------------------------------
// Rotary positions: pair (2i, 2i + 1) of the first `dims` dimensions of every map of every head, angle = pos * freq[i]
// (fp32), cos / sin scaled by `mscale`; freq carries whatever frequency scaling the model uses (host: stack_rope_freqs).
// Paged cache of one attention layer: K pool [blocks, kv_heads * maps, page, dim], V pool [blocks, kv_heads, vdim, page] (values
// channel-major inside a page: the MFMA kernel reads V^T rows).
// ---------------------------------------------------------------------------------------------
struct StackAttnParams
{
    int32_t dtype = DT_BF16;
    int32_t tokens = 0, entries = 0;
    int32_t heads = 0, kv_heads = 0, maps = 1, dim = 0, vdim = 0;
    int32_t rot_dims = 0;
    int32_t rot_halves = 0;      // latent_prep: 0 pairs (2i, 2i + 1), 1 pairs (i, i + rot_dims / 2)
    const float* freq = nullptr; // fp32 [rot_dims / 2], device
    float mscale = 1.f;
    float scale = 1.f, softcap = 0.f; // score = softcap * tanh(q.k * scale / softcap) when softcap > 0
    // maps == 2: o = a1 - lambda * a2; head_norm: o /= sqrt(mean(o^2) + eps) over vdim, then * out_scale
    float lambda = 0.f, out_scale = 1.f, eps = 1e-5f;
    int32_t head_norm = 0;
    // Per-head numbers, fp32 [heads] on the device, null = absent.  With i the row's position and j the key's:
    //   score = q.k * scale (soft cap) * temp[h] - slope[h] * (i - j) - log_r1[h] * ln(1 + log_r2[h] * (i - j))
    const float* temp = nullptr;
    const float* slope = nullptr;
    const float* log_r1 = nullptr;
    const float* log_r2 = nullptr;
    // mask: which keys j <= i a row sees.  MASK_WINDOW: i - j < mask_size; MASK_CHUNK: floor(i / mask_size) == floor(j / mask_size);
    // mask_keep > 0 (windows): the sequence's first mask_keep keys stay visible to every later row (each at its own position: nothing about them is shifted)
    int32_t mask = 0, mask_size = 0, mask_keep = 0;
    // weights: WEIGHTS_SOFTMAX, its denominator also holding exp(sink[h]) when sink is set (a logit without key or value);
    // WEIGHTS_SIGMOID: weight = sigmoid(score + wbias[h]) per key, not normalised over keys
    int32_t weights = 0;
    const float* sink = nullptr;
    const float* wbias = nullptr;
    // the head's output times sigmoid(out_gate[t * ld_gate + h]) (pre-activations in the element type), null = none;
    // gate_wide: one gate per output channel, out_gate[t * ld_gate + h * vdim + c]
    const void* out_gate = nullptr;
    int64_t ld_gate = 0;
    int32_t gate_wide = 0;
    // talking heads: talk [heads, heads] fp32 on the device, null = none.  After the softmax (sink included in the denominators) head
    // h's weight on key j becomes sum_g talk[h * heads + g] w_g(i, j); head h applies it to the values of its own key/value head.
    const float* talk = nullptr;
    // cross_values (launch_stack_attention only): `heads` counts (query head, value head) pairs, query heads x kv_heads of them in
    // this order; pair (g, c) applies query head g's weights (over the keys of g's own key head) to the rows of value head c; q holds
    // heads / kv_heads query heads, out [tokens, heads * vdim].  The terms of head-mixed weights: launch_stack_talk_combine sums them.
    int32_t cross_values = 0;
    // room for those terms, [tokens, heads * kv_heads * vdim] of the element type: with it (and a shape of the tile kernels) a layer
    // with `talk` runs as a cross_values launch plus launch_stack_talk_combine; without it, on the general kernel
    void* pair_ws = nullptr;
    // values_are_keys: the layer has no value projection; a token's value row is its key as projected (unrotated, unnormed); vdim == dim
    int32_t values_are_keys = 0;
    // weights of the q / k norm (qk_unit_norm), fp32 [dim] each, null = plain unit RMS
    const float* q_norm_w = nullptr;
    const float* k_norm_w = nullptr;
    // the projection's rows before anything else: + bias (fp32 [q | k | v columns]), then q and k of every head and map divided by
    // their root mean square over dim (qk_unit_norm, eps)
    const float* bias = nullptr;
    int32_t qk_unit_norm = 0;
    const void* proj = nullptr; // [tokens, ldp]: q rows (heads * maps * dim), k rows (kv_heads * maps * dim), v rows (kv_heads * vdim)
    int64_t ldp = 0;
    void* q = nullptr;          // scratch [tokens, heads * maps * dim]: rotated queries
    void* k_pool = nullptr;
    void* v_pool = nullptr;
    int32_t page = 64, max_blocks = 0;
    const int32_t* block_table = nullptr; // [entries, max_blocks]
    const int32_t* tok_entry = nullptr;   // [tokens]
    const int32_t* tok_pos = nullptr;     // [tokens]
    const int32_t* ent_first = nullptr;   // [entries] first row of the entry in the packed batch
    const int32_t* ent_count = nullptr;   // [entries] rows of the entry
    const int32_t* ent_pos0 = nullptr;    // [entries] position of its first row
    int32_t max_count = 0;                // host: the largest ent_count of the step
    int32_t max_context = 0;              // host: the largest pos0 + count of the step
    void* out = nullptr;                  // [tokens, heads * vdim]
    float* split_ws = nullptr;            // decoding steps: partials of the cross-workgroup key split (stack_attn_workspace_floats); null: no split
};
constexpr int32_t MASK_CAUSAL = 0, MASK_WINDOW = 1, MASK_CHUNK = 2;
constexpr int32_t WEIGHTS_SOFTMAX = 0, WEIGHTS_SIGMOID = 1;
// rotates q and k, appends k and v of the step's rows to the paged cache
int launch_stack_rope_kv(const StackAttnParams& p, hipStream_t stream);
// causal attention of the step's rows over their sequences' cache (which already holds the step's own keys)
int launch_stack_attention(const StackAttnParams& p, hipStream_t stream);
size_t stack_attn_workspace_floats(int32_t heads, int32_t maps, int32_t vdim);
// Talking heads from their terms: pairs [tokens, heads * kv_heads * vdim] holds, for query head g and value head c, a_gc = sum_j w_g(i, j)
// v_c(j) (launch_stack_attention with cross_values).  out[t, h, :] = sigmoid gate * sum_g talk[h * heads + g] a_{g, kv(h)}, kv(h) = h /
// (heads / kv_heads); gate: out_gate / ld_gate / gate_wide of `a` (null: none).  a.heads counts query heads here.
int launch_stack_talk_combine(const StackAttnParams& a, const void* pairs, hipStream_t stream); // floats of split_ws a layer of this shape needs
// frequencies of the rotation with YaRN-style scaling (factor <= 0: none): fills freq[dims / 2], returns the cos / sin multiplier
float stack_rope_freqs(float* freq, int32_t dims, double base, double factor, double original, double fast, double slow);
// frequencies with the three-band scaling by wavelength l = 2 pi / f: f stays where l < original / high, becomes f / factor where
// l > original / low, and is blended by s = (original / l - low) / (high - low) between (factor <= 0: none)
void stack_rope_freqs_banded(float* freq, int32_t dims, double base, double factor, double original, double low, double high);

// ---------------------------------------------------------------------------------------------
// Latent attention: a token leaves one latent c [rank] (RMS-normed with a plain weight) and one rotated key part [rot] that all
// heads share; a head's unrotated key is W_uk c and its value W_uv c.  The cache holds c and the rotated part only, and attention
// runs in the absorbed form: with a = W_uk^T q_plain (per head, [rank]) the score is a.c + q_rot.k_rot, and the head's output is
// W_uv (sum_j p_j c_j).  That is launch_stack_attention with one key/value head of dim = rank + rot and vdim = rank:
//   K pool rows [c | k_rot], V pool rows c, queries [a | q_rot].
// This kernel does the pointwise part for the step's rows; the two per-head products around the attention are batched
// launch_stack_gemm calls.  proj [tokens, ldp]: q (heads * (dim + rot): per head plain then rotated part), then rank + rot columns.
// It writes the rotated q part into q_abs[t, h, rank : rank + rot] and appends the token to the cache; a.dim = rank + rot,
// a.vdim = rank, a.kv_heads = 1, a.rot_dims = how many of the rot dimensions turn (pairs (2i, 2i + 1), the rest pass), a.freq,
// a.q = q_abs and the pools are read from `a`; a.rot_halves chooses the pairing, a.mscale multiplies cos and sin.  Where the
// queries come from a projection of their own (a query latent), q_src [tokens, ldq] holds them and dkv_col is the column of proj at
// which the rank + rot columns start.
// ---------------------------------------------------------------------------------------------
int launch_stack_latent_prep(const StackAttnParams& a, int32_t qk_dim, const float* latent_norm_w, hipStream_t stream,
    const void* q_src = nullptr, int64_t ldq = 0, int32_t dkv_col = -1);

// ---------------------------------------------------------------------------------------------
// HGRN2: per head a state S [dim, vdim] (fp32, one per sequence slot), S <- diag(f) S + (1 - f) v^T, o = S^T q with
// q = silu(q_raw), f = lower + (1 - lower) * sigmoid(f_raw + f_bias); then o / sqrt(mean(o^2) + eps) * norm_w per head.
// proj [tokens, ldp]: q_raw (heads * dim), f_raw (heads * dim), v (heads * vdim).  An entry whose pos0 is 0 starts from zero.
// ---------------------------------------------------------------------------------------------
struct StackHgrnParams
{
    int32_t dtype = DT_BF16;
    int32_t tokens = 0, entries = 0;
    int32_t heads = 0, dim = 0, vdim = 0;
    const void* proj = nullptr;
    int64_t ldp = 0;
    const float* f_bias = nullptr; // [heads * dim]
    const float* lower = nullptr;  // [heads * dim]
    const float* norm_w = nullptr; // [vdim]
    float eps = 1e-5f;
    float* state = nullptr;        // [slots, heads, dim, vdim]
    const int32_t* ent_slot = nullptr;
    const int32_t* ent_first = nullptr;
    const int32_t* ent_count = nullptr;
    const int32_t* ent_pos0 = nullptr;
    int32_t max_count = 0;         // host: the largest ent_count of the step
    float* o32 = nullptr;          // scratch [tokens, heads * vdim]
    void* out = nullptr;           // [tokens, heads * vdim]
};
int launch_stack_hgrn2(const StackHgrnParams& p, hipStream_t stream);
bool stack_hgrn2_serves(int32_t dim, int32_t vdim); // shapes one of its two forms takes

// ---------------------------------------------------------------------------------------------
// Selective state-space layer (Mamba-2): proj [tokens, ldp] = [z: inner | x: inner | B: groups * state | C: groups * state |
// dt: heads], inner = heads * vdim.  x, B, C pass a causal convolution over `taps` tokens per channel (conv_w [channels, taps], the
// last column meets the current token; bias) and silu: launch_stack_ssm_conv writes them to xbc [tokens, channels] and moves the
// sequence's last taps - 1 raw inputs into conv_state [slots, taps - 1, channels].  launch_stack_ssm_scan: per head h (reading group
// h / (heads / groups)), with dt = softplus(dt + dt_bias[h]):
//   S <- exp(-exp(a_log[h]) dt) S + dt B x^T   (S [state, vdim], fp32, one per slot),   y = S^T C + d_skip[h] x,
// and y32 [tokens, inner] = y * silu(z) in fp32 (the grouped norm behind it is launch_stack_group_rmsnorm).  An entry whose pos0 is 0
// starts from zero state and zero convolution inputs.
// ---------------------------------------------------------------------------------------------
struct StackSsmParams
{
    int32_t dtype = DT_BF16;
    int32_t tokens = 0, entries = 0;
    int32_t heads = 0, vdim = 0, state = 0, groups = 1, taps = 0;
    const void* proj = nullptr;
    int64_t ldp = 0;
    const float* conv_w = nullptr; // [channels, taps]
    const float* conv_b = nullptr; // [channels]
    const float* dt_bias = nullptr; // [heads]
    const float* a_log = nullptr;   // [heads]
    const float* d_skip = nullptr;  // [heads]
    float* conv_state = nullptr;    // [slots, taps - 1, channels]
    float* ssm_state = nullptr;     // [slots, heads, state, vdim]
    void* xbc = nullptr;            // scratch [tokens, channels], element type
    float* y32 = nullptr;           // [tokens, inner]
    // launch_stack_ssm_conv alone, for another layer kind: conv_channels > 0 channels that start at column conv_col of proj
    // (instead of the x | B | C columns behind z); conv_b may be null
    int32_t conv_channels = 0;
    int64_t conv_col = 0;
    const int32_t* tok_entry = nullptr;
    const int32_t* tok_pos = nullptr;
    const int32_t* ent_slot = nullptr;
    const int32_t* ent_first = nullptr;
    const int32_t* ent_count = nullptr;
    const int32_t* ent_pos0 = nullptr;
};
int launch_stack_ssm_conv(const StackSsmParams& p, hipStream_t stream);
int launch_stack_ssm_scan(const StackSsmParams& p, hipStream_t stream);
bool stack_ssm_serves(int32_t vdim, int32_t state, int32_t taps);

// ---------------------------------------------------------------------------------------------
// Routed mixture of experts.  Router: z = router_w h in fp32 over experts + identity outputs, s = softmax(z); the choice is made on
// s + correction among the experts of the group_keep groups (of group_count equal groups of neighbours) whose largest such value is
// largest, `top` of them; a chosen expert's weight is s * scale (without the correction, not renormalised).  The last `identity`
// outputs are experts without weights that return h.
//   launch_stack_moe_route   -> topk_idx / topk_w [tokens, top]
//   launch_stack_moe_sort    -> group_off [experts + 1], slot_of_pair [tokens * top] (-1: identity), a_sorted: the rows of h in
//                               expert order, one per (token, chosen expert); the grouped products (launch_stack_gemm, group_off) run on them
//   launch_stack_moe_combine -> y[t, :] = sum_k w_k * (expert: y_sorted[slot_k, :] | identity: h[t, :]), fp32
// ---------------------------------------------------------------------------------------------
struct StackMoeParams
{
    int32_t dtype = DT_BF16;
    int32_t tokens = 0, width = 0;
    int32_t experts = 0, identity = 0, top = 0, group_count = 1, group_keep = 1;
    float scale = 1.f;
    int32_t score = 0;        // ROUTE_SOFTMAX: s = softmax(z) over all outputs; ROUTE_SIGMOID: s = sigmoid(z), every output by itself
    int32_t weight_input = 0; // 1: an expert runs on w h (a_sorted = w h), the outputs are summed unweighted
    const void* h = nullptr;          // [tokens, width]
    const float* router_w = nullptr;  // [experts + identity, width]
    const float* correction = nullptr; // [experts + identity] or null
    float* logits = nullptr;          // scratch [tokens, experts + identity]
    int32_t* topk_idx = nullptr;
    float* topk_w = nullptr;
    int32_t* group_off = nullptr;
    int32_t* slot_of_pair = nullptr;
    int32_t* pair_of_slot = nullptr;  // [tokens * top], -1 behind the last used slot
    void* a_sorted = nullptr;         // [tokens * top, width]
};
constexpr int32_t ROUTE_SOFTMAX = 0, ROUTE_SIGMOID = 1;
int launch_stack_moe_route(const StackMoeParams& p, hipStream_t stream);
int launch_stack_moe_sort(const StackMoeParams& p, hipStream_t stream);
int launch_stack_moe_combine(const StackMoeParams& p, const float* y_sorted, float* y, hipStream_t stream);

// ---------------------------------------------------------------------------------------------
// Gated delta rule with one decay per key channel.  Per head h a state S [dim, vdim] (fp32, one per slot); head h reads the q / k
// head h / (heads / qk_heads).  x [tokens, channels] holds q (qk_heads * dim) | k (qk_heads * dim) | v (heads * vdim) behind their
// convolution and silu.  Per token, in fp32:
//   q <- q / sqrt(sum q^2 + 1e-6) / sqrt(dim),  k <- k / sqrt(sum k^2 + 1e-6),  beta = sigmoid(beta_raw[t, h]),
//   g[d] = exp(-exp(a_log[h]) * softplus(decay_raw[t, h * dim + d] + dt_bias[h * dim + d])),
//   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q   (read after the token's own write)
// launch_stack_delta_scan leaves o in o32 [tokens, heads * vdim]; launch_stack_delta_out turns it into
//   out[t, h, c] = o / sqrt(mean_c o^2 + eps) * norm_w[c] * sigmoid(gate_raw[t, h * vdim + c]).
// An entry whose pos0 is 0 starts from a zero state.
// ---------------------------------------------------------------------------------------------
struct StackDeltaParams
{
    int32_t dtype = DT_BF16;
    int32_t tokens = 0, entries = 0;
    int32_t heads = 0, qk_heads = 0, dim = 0, vdim = 0;
    const void* x = nullptr;          // [tokens, 2 * qk_heads * dim + heads * vdim], element type
    const void* beta_raw = nullptr;   // element type, beta_raw[t * ld_beta + h]
    int64_t ld_beta = 0;
    const float* decay_raw = nullptr; // fp32 [tokens, heads * dim]
    const float* dt_bias = nullptr;   // [heads * dim]
    const float* a_log = nullptr;     // [heads]
    const float* gate_raw = nullptr;  // fp32 [tokens, heads * vdim]
    const float* norm_w = nullptr;    // [vdim]
    float eps = 1e-5f;
    float* state = nullptr;           // [slots, heads, dim, vdim]
    float* o32 = nullptr;             // [tokens, heads * vdim]
    void* out = nullptr;              // [tokens, heads * vdim], element type
    const int32_t* ent_slot = nullptr;
    const int32_t* ent_first = nullptr;
    const int32_t* ent_count = nullptr;
    const int32_t* ent_pos0 = nullptr;
    int32_t max_count = 0;            // host: the largest ent_count of the step
};
int launch_stack_delta_scan(const StackDeltaParams& p, hipStream_t stream);
int launch_stack_delta_out(const StackDeltaParams& p, hipStream_t stream);
bool stack_delta_serves(int32_t dim, int32_t vdim);

} // namespace kernels
} // namespace tllm
