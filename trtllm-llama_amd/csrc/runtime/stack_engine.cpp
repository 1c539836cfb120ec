// extern "C" surface of include/tllm_stack_api.h: the ragged-batch step executor for run-time described decoder stacks.
//
// One step = embedding -> the layer runs in order -> final norm + head on the wanted rows -> arg-max.  A layer run is
//   h1, h2 = norm1(x), norm2(x)                                  one launch (the two norms share the normalised row)
//   P1 = h1 [Wq; Wk; Wv; Wrg1]^T   (hgrn2: [Wq; Wf; Wv; Wrg1])    one product: everything that reads h1
//   ctx = mixer(P1)                                              rotary + cache append + attention | recurrence + head norm
//   x += sigmoid(P1[rg1] + b1) * (ctx Wo^T)                      product with the gated-residual seam in its epilogue
//   P2 = h2 [Wgate; Wup; Wrg2]^T ; a = gelu(P2[gate]) * P2[up]
//   x += sigmoid(P2[rg2] + b2) * (a Wdown^T)
// on the packed rows of the step (block=parallel, residual=gated).  With block=sequential, residual=hyper a layer run is pre-norm
// with `streams` hyper-connected copies of the residual:
//   h1 = norm1(sum_s in1[s] x_s)                                  one launch, which also lands the sublayer before it (below)
//   P1 = h1 [Wq; Wk; Wv; Wg]^T  (latent attention: [Wq; Wdkv])    mixer as above, per-head output gate inside the attention launch
//   y = ctx Wo^T (fp32);  x_t <- sum_s mix1[s, t] x_s + out1[t] y   folded into the next launch that reads the streams
//   h2 = norm2(sum_s in2[s] x_s);  a = relu(h2 Wup^T)^2 (product epilogue);  y = a Wdown^T;  x_t <- sum_s mix2[s, t] x_s + out2[t] y
// A mamba2 mixer is  P1 = h1 W_in^T = [z | x | B | C | dt]  ->  convolution + silu of x | B | C (and the sequence's new tail)  ->  the
// recurrence with skip and gate  ->  RMS norm in parts of the row;  a latent layer with a query latent projects [W_dq; W_dkv], norms
// the query latent and expands it before the latent's pointwise part.  A routed feed-forward is  router (fp32 logits, softmax, kept
// groups, top-k)  ->  (token, expert) pairs ordered by expert  ->  [gate_e; up_e] grouped product  ->  silu(gate) * up  ->  down_e
// grouped product in fp32  ->  weighted sum per token (identity experts add w h).  A layer with weights_of runs on another layer's
// device tensors; caches and states belong to runs.
// The residual streams are fp32 in both element types.
#include "../../../include/tllm_stack_api.h"
#include "../kernels/stack_kernels.h"
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

using namespace tllm;
using namespace tllm::kernels;

namespace
{

struct HostTensor
{
    std::vector<int64_t> dims;
    std::vector<float> v; // every weight passes through fp32 on the host (bfloat16 -> fp32 is exact)
    int64_t numel() const
    {
        int64_t n = 1;
        for (auto d : dims)
            n *= d;
        return n;
    }
};

enum MixerKind
{
    MIX_ATTENTION = 0,
    MIX_HGRN2 = 1,
    MIX_LATENT = 2,
    MIX_MAMBA2 = 3,
    MIX_DELTA = 4
};
enum MlpKind
{
    MLP_GELU_GATE = 0, // W_down (gelu_tanh(W_gate h) * W_up h)
    MLP_RELU2 = 1,     // W_down relu(W_up h)^2
    MLP_MOE = 2        // routed experts W_down (silu(W_gate h) * W_up h) of size ff, the last `identity` router outputs return h
};
struct HyperW
{
    float *mix = nullptr, *out = nullptr, *in = nullptr;
};

struct Layer
{
    int kind = MIX_ATTENTION;
    int heads = 0, kv_heads = 0, dim = 0, vdim = 0, maps = 1, ff = 0, head_norm = 0;
    double diff = 0, scale = 1, softcap = 0;
    int rot_dims = 0;
    double rot_base = 10000, rot_factor = 0, rot_original = 0, rot_fast = 0, rot_slow = 0, rot_low = 1, rot_high = 4;
    // derived
    int n_q = 0, n_k = 0, n_v = 0, n_mix = 0, n_ctx = 0; // columns of P1: q | k (or f) | v | rg1
    float lambda = 0.f, mscale = 1.f;
    int mlp = MLP_GELU_GATE;
    int qkv_bias = 0, qk_norm = 0, head_temp = 0, pos_bias = 0 /* 0 none, 1 linear, 2 log */, mask = MASK_CAUSAL, mask_size = 0,
        weights = WEIGHTS_SOFTMAX, sink = 0, out_gate = 0;
    double slope_base = 8;
    int kv_rank = 0, rot_part = 0;  // latent attention: rank of the latent, size of the shared rotated key part (rot_dims of it turn)
    int n_gate = 0, n_rg = 0;       // further columns of P1: per-head output gates, the gated residual's projection
    int n_lat = 0;                  // latent attention: heads * kv_rank
    int q_rank = 0, rot_halves = 0; // latent attention: rank of a query latent (0: queries straight from the input), half-split pairs
    int weights_of = -1;            // the layer whose weights this one runs on (its cache / state is its own)
    int groups = 1, taps = 0, ssm_norm_groups = 1, n_conv = 0; // mamba2 (dim = state rows): B / C groups, convolution taps, parts of the output norm
    int experts = 0, identity = 0, top = 0, route_groups = 1, route_keep = 1; // moe
    double route_scale = 1;
    int route_sigmoid = 0, route_weight_input = 0; // moe: sigmoid scores instead of a softmax; the weight scales the expert's input
    int mask_keep = 0, talk = 0, values_are_keys = 0, gate_wide = 0, qk_norm_weight = 0, o_bias = 0, rot_banded = 0; // attention
    int decay_rank = 0, gate_rank = 0, n_beta = 0; // delta_rule: ranks of the two low-rank projections, padded beta columns
    // device
    void *w_mix = nullptr, *w_o = nullptr, *w_gu = nullptr, *w_down = nullptr, *w_ukT = nullptr, *w_uv = nullptr;
    float *norm1 = nullptr, *norm2 = nullptr, *rg1_b = nullptr, *rg2_b = nullptr, *f_bias = nullptr, *lower = nullptr, *hnorm = nullptr,
          *freq = nullptr, *bias = nullptr, *temp = nullptr, *slope = nullptr, *r1 = nullptr, *r2 = nullptr, *sinkv = nullptr, *wbias = nullptr,
          *lat_norm = nullptr, *cq_norm = nullptr, *conv_w = nullptr, *conv_b = nullptr, *dt_bias = nullptr, *a_log = nullptr,
          *d_skip = nullptr, *router_w = nullptr, *correction = nullptr, *talkw = nullptr, *q_norm = nullptr, *k_norm = nullptr, *o_biasv = nullptr,
          *shift = nullptr;
    void *w_a2 = nullptr, *w_g2 = nullptr; // delta_rule: the second halves of the decay's and the gate's low-rank projections
    void* w_uq = nullptr;
    HyperW hc[2];
};

struct Run
{
    int layer = 0, pass = 0;
    bool enters_pass = false;
    void *k_pool = nullptr, *v_pool = nullptr; // attention
    float* state = nullptr;                    // hgrn2, mamba2
    float* conv_state = nullptr;               // mamba2, delta_rule: the last taps - 1 inputs of the convolution
    float* shift_carry = nullptr;              // token shift: the sequence's last normed row, [slots, width]
};

} // namespace

struct tllm_stack
{
    std::map<std::string, std::string> cfg;
    std::map<std::string, HostTensor> host;
    int dtype = DT_BF16, es = 2;
    int width = 0, vocab = 0, groups = 1, page = 64, blocks = 0, slots = 0, taps = 0;
    int loop_start = 0, loop_stop = 0, loop_times = 1;
    bool sequential = false, hyper = false;
    int streams = 1;
    float norm_offset = 0.f, *ones = nullptr;
    float eps = 1e-5f, emb_scale = 1.f;
    std::vector<Layer> layers;
    std::vector<Run> runs;
    void *embed = nullptr, *head = nullptr;
    float *final_norm = nullptr, *loop_step = nullptr, *attn_ws = nullptr;
    bool finalized = false;
    int64_t weight_bytes = 0;
    std::vector<void*> owned;
    // scratch, grown to the largest step seen
    int cap_tokens = 0, cap_want = 0, cap_ints = 0;
    float *x = nullptr, *x0 = nullptr, *o32 = nullptr, *logits = nullptr, *tap = nullptr, *y32 = nullptr;
    void *h1 = nullptr, *h2 = nullptr, *proj = nullptr, *q = nullptr, *ctx = nullptr, *act = nullptr, *hw = nullptr, *lat = nullptr;
    int32_t *ints = nullptr, *ids_out = nullptr, *pinned = nullptr;
    void *xbc = nullptr, *cq = nullptr, *qfull = nullptr, *moe_a = nullptr;
    float *moe_y = nullptr, *moe_w = nullptr;
    int32_t* moe_i = nullptr;
    // pair embedding (a hashed row per (previous token, token)) and token shift; the previous token of every slot's sequence
    int pair_buckets = 0, pair_mul_prev = 0, pair_mul_cur = 0, token_shift = 0;
    void* pair_table = nullptr;
    std::vector<int32_t> last_tok;
    float *h32 = nullptr, *dl_a = nullptr, *dl_g = nullptr;
    void* pairs = nullptr; // talking heads: every query head's weights over every value head's rows, [tokens, heads * kv_heads * vdim]
    int max_hd = 0, max_pairs = 0;
    int max_proj = 0, max_q = 0, max_ctx = 0, max_ff = 0, max_lat = 0, max_conv = 0, max_qrank = 0, max_qfull = 0, max_top = 0, max_experts = 0, max_outputs = 0;
    int tap_tokens = 0;

    ~tllm_stack()
    {
        for (void* p : owned)
            (void) hipFree(p);
        free_scratch();
        if (pinned)
            (void) hipHostFree(pinned);
    }
    void free_scratch()
    {
        void* all[] = {x, x0, o32, logits, tap, y32, h1, h2, proj, q, ctx, act, hw, lat, ints, ids_out, xbc, cq, qfull, moe_a, moe_y, moe_w, moe_i,
            h32, dl_a, dl_g, pairs};
        for (void* p : all)
            if (p)
                (void) hipFree(p);
        x = x0 = o32 = logits = tap = y32 = nullptr;
        h1 = h2 = proj = q = ctx = act = hw = lat = nullptr;
        ints = ids_out = nullptr;
        xbc = cq = qfull = moe_a = nullptr;
        moe_y = moe_w = nullptr;
        moe_i = nullptr;
        h32 = dl_a = dl_g = nullptr;
        pairs = nullptr;
    }
};

namespace
{

#define HIP_OK(call)                                                                                                              \
    do                                                                                                                              \
    {                                                                                                                               \
        const hipError_t e_ = (call);                                                                                               \
        if (e_ != hipSuccess)                                                                                                       \
        {                                                                                                                           \
            set_error("stack engine: %s failed: %s", #call, hipGetErrorString(e_));                                               \
            return -1;                                                                                                              \
        }                                                                                                                           \
    } while (0)

inline uint16_t host_f2bf(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u)
        return (uint16_t) ((u >> 16) | 0x40u);
    return (uint16_t) ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

double getd(const tllm_stack* s, const std::string& k, double dflt)
{
    auto it = s->cfg.find(k);
    return it == s->cfg.end() ? dflt : std::atof(it->second.c_str());
}
int geti(const tllm_stack* s, const std::string& k, int dflt)
{
    auto it = s->cfg.find(k);
    return it == s->cfg.end() ? dflt : std::atoi(it->second.c_str());
}
std::string gets(const tllm_stack* s, const std::string& k, const std::string& dflt)
{
    auto it = s->cfg.find(k);
    return it == s->cfg.end() ? dflt : it->second;
}

// rows of several [n_i, K] host matrices stacked into one device matrix of the engine's element type
int upload_rows(tllm_stack* s, const std::vector<const HostTensor*>& parts, void** out)
{
    int64_t n = 0;
    for (auto* t : parts)
        n += t->numel();
    void* d = nullptr;
    HIP_OK(hipMalloc(&d, (size_t) (n ? n : 1) * s->es));
    s->owned.push_back(d);
    s->weight_bytes += n * s->es;
    int64_t off = 0;
    std::vector<uint16_t> tmp;
    for (auto* t : parts)
    {
        if (s->dtype == DT_FLOAT)
            HIP_OK(hipMemcpy((char*) d + off * 4, t->v.data(), t->v.size() * 4, hipMemcpyHostToDevice));
        else
        {
            tmp.resize(t->v.size());
            for (size_t i = 0; i < tmp.size(); ++i)
                tmp[i] = host_f2bf(t->v[i]);
            HIP_OK(hipMemcpy((char*) d + off * 2, tmp.data(), tmp.size() * 2, hipMemcpyHostToDevice));
        }
        off += t->numel();
    }
    *out = d;
    return 0;
}

int upload_f32(tllm_stack* s, const float* v, size_t n, float** out)
{
    void* d = nullptr;
    HIP_OK(hipMalloc(&d, (n ? n : 1) * 4));
    s->owned.push_back(d);
    s->weight_bytes += (int64_t) n * 4;
    HIP_OK(hipMemcpy(d, v, n * 4, hipMemcpyHostToDevice));
    *out = (float*) d;
    return 0;
}

const HostTensor* need(tllm_stack* s, const std::string& name, std::initializer_list<int64_t> dims)
{
    auto it = s->host.find(name);
    if (it == s->host.end())
    {
        set_error("tllm_stack_finalize: tensor %s is missing", name.c_str());
        return nullptr;
    }
    const std::vector<int64_t> want(dims);
    if (it->second.dims != want)
    {
        std::string have, w;
        for (auto d : it->second.dims)
            have += std::to_string(d) + " ";
        for (auto d : want)
            w += std::to_string(d) + " ";
        set_error("tllm_stack_finalize: tensor %s has shape [ %s], the configuration asks for [ %s]", name.c_str(), have.c_str(), w.c_str());
        return nullptr;
    }
    return &it->second;
}

int alloc_zero(tllm_stack* s, size_t bytes, void** out)
{
    void* d = nullptr;
    HIP_OK(hipMalloc(&d, bytes ? bytes : 16));
    s->owned.push_back(d);
    HIP_OK(hipMemset(d, 0, bytes ? bytes : 16));
    *out = d;
    return 0;
}

int ensure_scratch(tllm_stack* s, int tokens, int want, int n_ints)
{
    if (tokens > s->cap_tokens || want > s->cap_want || n_ints > s->cap_ints)
    {
        HIP_OK(hipDeviceSynchronize());
        s->free_scratch();
        if (s->pinned)
        {
            (void) hipHostFree(s->pinned);
            s->pinned = nullptr;
        }
        const size_t T = (size_t) std::max(tokens, s->cap_tokens), W = (size_t) std::max(want, s->cap_want);
        const size_t NI = (size_t) std::max(n_ints, s->cap_ints);
        const size_t es = s->es, wd = s->width;
        HIP_OK(hipMalloc((void**) &s->x, T * wd * 4 * (size_t) s->streams));
        HIP_OK(hipMalloc((void**) &s->y32, T * wd * 4));
        HIP_OK(hipMalloc(&s->lat, T * std::max(s->max_lat, 1) * es));
        HIP_OK(hipMalloc((void**) &s->x0, T * wd * 4));
        HIP_OK(hipMalloc((void**) &s->o32, T * std::max(s->max_ctx, 1) * 4));
        HIP_OK(hipMalloc((void**) &s->logits, W * s->vocab * 4));
        HIP_OK(hipMalloc(&s->h1, T * wd * es));
        HIP_OK(hipMalloc(&s->h2, T * wd * es));
        HIP_OK(hipMalloc(&s->proj, T * std::max(s->max_proj, 1) * es));
        HIP_OK(hipMalloc(&s->q, T * std::max(s->max_q, 1) * es));
        HIP_OK(hipMalloc(&s->ctx, T * std::max(s->max_ctx, 1) * es));
        HIP_OK(hipMalloc(&s->act, T * std::max(s->max_ff, 1) * es));
        HIP_OK(hipMalloc(&s->hw, W * wd * es));
        HIP_OK(hipMalloc((void**) &s->ints, NI * 4));
        HIP_OK(hipMalloc((void**) &s->ids_out, W * 4));
        HIP_OK(hipMalloc(&s->xbc, T * std::max(s->max_conv, 1) * es));
        HIP_OK(hipMalloc(&s->cq, T * std::max(s->max_qrank, 1) * es));
        HIP_OK(hipMalloc(&s->qfull, T * std::max(s->max_qfull, 1) * es));
        HIP_OK(hipMalloc((void**) &s->h32, (s->token_shift ? T * wd : 1) * 4));
        HIP_OK(hipMalloc(&s->pairs, T * std::max(s->max_pairs, 1) * es));
        HIP_OK(hipMalloc((void**) &s->dl_a, T * std::max(s->max_hd, 1) * 4));
        HIP_OK(hipMalloc((void**) &s->dl_g, (s->max_hd ? T * std::max(s->max_ctx, 1) : 1) * 4));
        {
            // a mixture of experts works on one row per (token, chosen expert)
            const size_t pairs = T * (size_t) std::max(s->max_top, 1);
            HIP_OK(hipMalloc(&s->moe_a, (s->max_top ? pairs * wd : 1) * es));
            HIP_OK(hipMalloc((void**) &s->moe_y, (s->max_top ? pairs * wd : 1) * 4));
            HIP_OK(hipMalloc((void**) &s->moe_w, (pairs + T * (size_t) (s->max_outputs + 1)) * 4));
            HIP_OK(hipMalloc((void**) &s->moe_i, (3 * pairs + (size_t) s->max_experts + 1) * 4));
        }
        HIP_OK(hipHostMalloc((void**) &s->pinned, NI * 4, hipHostMallocDefault));
        if (s->taps)
            HIP_OK(hipMalloc((void**) &s->tap, s->runs.size() * T * wd * 4));
        s->cap_tokens = (int) T;
        s->cap_want = (int) W;
        s->cap_ints = (int) NI;
    }
    return 0;
}

} // namespace

extern "C" {

tllm_stack_t tllm_stack_create(const char* config_text)
{
    if (!config_text)
    {
        set_error("tllm_stack_create: no configuration");
        return nullptr;
    }
    auto* s = new tllm_stack();
    std::string text(config_text);
    size_t at = 0;
    while (at < text.size())
    {
        size_t nl = text.find('\n', at);
        if (nl == std::string::npos)
            nl = text.size();
        const std::string line = text.substr(at, nl - at);
        at = nl + 1;
        const size_t eq = line.find('=');
        if (eq == std::string::npos)
            continue;
        s->cfg[line.substr(0, eq)] = line.substr(eq + 1);
    }
    const std::string dt = gets(s, "dtype", "bfloat16");
    if (dt == "bfloat16")
        s->dtype = DT_BF16, s->es = 2;
    else if (dt == "float32")
        s->dtype = DT_FLOAT, s->es = 4;
    else
    {
        set_error("tllm_stack_create: dtype %s (bfloat16 or float32)", dt.c_str());
        delete s;
        return nullptr;
    }
    s->width = geti(s, "width", 0);
    s->vocab = geti(s, "vocab", 0);
    s->groups = geti(s, "norm_groups", 1);
    s->eps = (float) getd(s, "norm_eps", 1e-5);
    s->emb_scale = (float) getd(s, "embedding_scale", 1.0);
    s->page = geti(s, "page_size", 64);
    s->blocks = geti(s, "num_blocks", 0);
    s->slots = geti(s, "num_slots", 0);
    s->taps = geti(s, "debug_taps", 0);
    s->loop_start = geti(s, "loop_start", 0);
    s->loop_stop = geti(s, "loop_stop", 0);
    s->loop_times = geti(s, "loop_times", 1);
    s->norm_offset = (float) getd(s, "norm_offset", 0.0);
    s->streams = geti(s, "streams", 1);
    s->pair_buckets = geti(s, "pair_buckets", 0);
    if (s->pair_buckets > 0)
    {
        // the multipliers only matter modulo the bucket count: (a m) mod B = (a (m mod B)) mod B, and the kernel's 64-bit products then
        // have room for any vocabulary
        auto mod_b = [&](const char* key) {
            const long long m = std::atoll(gets(s, key, "0").c_str()) % s->pair_buckets;
            return (int) (m < 0 ? m + s->pair_buckets : m);
        };
        s->pair_mul_prev = mod_b("pair_mul_prev");
        s->pair_mul_cur = mod_b("pair_mul_cur");
    }
    s->token_shift = geti(s, "token_shift", 0);
    const std::string block = gets(s, "block", "parallel"), residual = gets(s, "residual", "gated");
    s->sequential = block == "sequential";
    s->hyper = residual == "hyper";
    const int L = geti(s, "num_layers", 0);
    auto fail = [&](const char* why) {
        set_error("tllm_stack_create: %s", why);
        delete s;
        return (tllm_stack_t) nullptr;
    };
    if (s->width < 1 || s->vocab < 1 || L < 1)
        return fail("width, vocab and num_layers must be positive");
    if (s->groups < 1 || s->width % s->groups)
        return fail("width must split into norm_groups equal parts");
    if (s->page < 1 || s->blocks < 1 || s->slots < 1)
        return fail("page_size, num_blocks and num_slots must be positive");
    if ((block != "parallel" && block != "sequential") || (residual != "gated" && residual != "hyper") || s->sequential != s->hyper)
        return fail("block=parallel goes with residual=gated, block=sequential with residual=hyper");
    if (s->streams < 1 || s->streams > 8 || (!s->hyper && s->streams != 1))
        return fail("streams: 1 to 8, more than one only with residual=hyper");
    if (s->hyper && s->loop_stop > s->loop_start)
        return fail("looped layers are built for the gated residual only");
    if (s->pair_buckets < 0 || (s->token_shift && !s->hyper))
        return fail("pair_buckets >= 0; the token shift is built for block=sequential");
    s->last_tok.assign((size_t) s->slots, -1);
    if (s->loop_times < 1 || s->loop_start < 0 || s->loop_stop < s->loop_start || s->loop_stop > L)
        return fail("the loop must satisfy 0 <= loop_start <= loop_stop <= num_layers, loop_times >= 1");
    s->layers.resize(L);
    for (int i = 0; i < L; ++i)
    {
        Layer& l = s->layers[i];
        const std::string p = "layer." + std::to_string(i) + ".";
        const std::string kind = gets(s, p + "type", "");
        if (kind == "attention")
            l.kind = MIX_ATTENTION;
        else if (kind == "hgrn2")
            l.kind = MIX_HGRN2;
        else if (kind == "latent_attention")
            l.kind = MIX_LATENT;
        else if (kind == "mamba2")
            l.kind = MIX_MAMBA2;
        else if (kind == "delta_rule")
            l.kind = MIX_DELTA;
        else
        {
            set_error("tllm_stack_create: layer %d has mixer type '%s' (attention | latent_attention | hgrn2 | mamba2 | delta_rule)", i, kind.c_str());
            delete s;
            return nullptr;
        }
        l.heads = geti(s, p + "heads", 0);
        l.dim = geti(s, p + (l.kind == MIX_MAMBA2 ? "state" : "dim"), 0);
        l.vdim = geti(s, p + "vdim", l.dim);
        l.weights_of = geti(s, p + "weights_of", -1);
        if (l.weights_of >= i || (l.weights_of >= 0 && s->layers[l.weights_of].weights_of >= 0))
            return fail("weights_of names an earlier layer that has weights of its own");
        l.ff = geti(s, p + "ff", 0);
        if (l.heads < 1 || l.dim < 1 || l.vdim < 1 || l.ff < 0)
            return fail("a layer needs heads, dim and vdim");
        l.n_ctx = l.heads * l.vdim;
        const std::string mlp = gets(s, p + "mlp", "gelu_gate");
        if (mlp != "gelu_gate" && mlp != "relu2" && mlp != "moe")
            return fail("a layer's mlp is gelu_gate, relu2 or moe");
        l.mlp = mlp == "relu2" ? MLP_RELU2 : (mlp == "moe" ? MLP_MOE : MLP_GELU_GATE);
        if (l.mlp != MLP_GELU_GATE && !s->sequential)
            return fail("the relu2 and moe feed-forwards are built for block=sequential");
        if ((l.kind == MIX_MAMBA2 || l.kind == MIX_DELTA || l.weights_of >= 0) && !s->sequential)
            return fail("mamba2 and delta_rule layers and shared weights are built for block=sequential");
        if (l.mlp == MLP_MOE && l.ff > 0)
        {
            l.experts = geti(s, p + "experts", 0);
            l.identity = geti(s, p + "identity", 0);
            l.top = geti(s, p + "top", 1);
            l.route_groups = geti(s, p + "route_groups", 1);
            l.route_keep = geti(s, p + "route_keep", l.route_groups);
            l.route_scale = getd(s, p + "route_scale", 1.0);
            const std::string rs = gets(s, p + "route_score", "softmax"), rw = gets(s, p + "route_weight", "output");
            if ((rs != "softmax" && rs != "sigmoid") || (rw != "output" && rw != "input"))
                return fail("moe: route_score softmax | sigmoid, route_weight output | input");
            l.route_sigmoid = rs == "sigmoid";
            l.route_weight_input = rw == "input";
            const int ne = l.experts + l.identity;
            if (l.experts < 1 || l.identity < 0 || ne > 1024 || l.top < 1 || l.top > 16 || l.top > ne || l.route_groups < 1 || ne % l.route_groups
                || l.route_keep < 1 || l.route_keep > l.route_groups)
                return fail("moe: experts >= 1, experts + identity <= 1024 in equal route_groups, 1 <= route_keep <= route_groups, top <= 16");
            s->max_top = std::max(s->max_top, l.top);
            s->max_experts = std::max(s->max_experts, l.experts);
            s->max_outputs = std::max(s->max_outputs, ne);
        }
        l.n_rg = s->hyper ? 0 : s->width;
        if (l.kind == MIX_LATENT)
        {
            l.kv_rank = geti(s, p + "kv_rank", 0);
            l.rot_part = geti(s, p + "rot_dim", 0);
            l.rot_dims = geti(s, p + "rot_dims", l.rot_part);
            l.rot_base = getd(s, p + "rot_base", 10000);
            l.rot_factor = getd(s, p + "rot_factor", 0);
            l.rot_original = getd(s, p + "rot_original", 0);
            l.rot_fast = getd(s, p + "rot_fast", 0);
            l.rot_slow = getd(s, p + "rot_slow", 0);
            l.scale = getd(s, p + "scale", 1.0 / std::sqrt((double) (l.dim + l.rot_part)));
            l.q_rank = geti(s, p + "q_rank", 0);
            const std::string pairing = gets(s, p + "rot_pairing", "neighbours"), mk = gets(s, p + "mask", "causal");
            if ((pairing != "neighbours" && pairing != "halves") || (mk != "causal" && mk != "window" && mk != "chunk"))
                return fail("latent_attention: rot_pairing neighbours | halves, mask causal | window | chunk");
            l.rot_halves = pairing == "halves";
            l.mask = mk == "window" ? MASK_WINDOW : (mk == "chunk" ? MASK_CHUNK : MASK_CAUSAL);
            l.mask_size = geti(s, p + "mask_size", 0);
            l.sink = geti(s, p + "sink", 0);
            if (l.kv_rank < 1 || l.rot_part < 0 || l.rot_dims < 0 || (l.rot_dims & 1) || l.rot_dims > l.rot_part || l.q_rank < 0)
                return fail("latent_attention: kv_rank positive, rot_dims even and <= rot_dim");
            if (l.mask != MASK_CAUSAL && l.mask_size < 1)
                return fail("latent_attention: a window or chunk mask needs mask_size >= 1");
            l.kv_heads = 1;
            // columns of the mixer's projection: the queries of every head, or the query latent they are expanded from
            l.n_q = l.q_rank > 0 ? l.q_rank : l.heads * (l.dim + l.rot_part);
            l.n_k = l.kv_rank + l.rot_part; // the down projection: latent | rotated key part
            l.n_v = 0;
            s->max_qrank = std::max(s->max_qrank, l.q_rank);
            if (l.q_rank > 0)
                s->max_qfull = std::max(s->max_qfull, l.heads * (l.dim + l.rot_part));
            l.n_lat = l.heads * l.kv_rank;
            s->max_lat = std::max(s->max_lat, l.n_lat);
            s->max_q = std::max(s->max_q, l.heads * (l.kv_rank + l.rot_part));
        }
        else if (l.kind == MIX_ATTENTION)
        {
            l.qkv_bias = geti(s, p + "qkv_bias", 0);
            l.qk_norm = geti(s, p + "qk_norm", 0);
            l.head_temp = geti(s, p + "head_temp", 0);
            const std::string pb = gets(s, p + "pos_bias", "none"), mk = gets(s, p + "mask", "causal"), wt = gets(s, p + "weights", "softmax");
            if ((pb != "none" && pb != "linear" && pb != "log") || (mk != "causal" && mk != "window" && mk != "chunk")
                || (wt != "softmax" && wt != "sigmoid"))
                return fail("attention: pos_bias none | linear | log, mask causal | window | chunk, weights softmax | sigmoid");
            l.pos_bias = pb == "linear" ? 1 : (pb == "log" ? 2 : 0);
            l.slope_base = getd(s, p + "slope_base", 8.0);
            l.mask = mk == "window" ? MASK_WINDOW : (mk == "chunk" ? MASK_CHUNK : MASK_CAUSAL);
            l.mask_size = geti(s, p + "mask_size", 0);
            l.weights = wt == "sigmoid" ? WEIGHTS_SIGMOID : WEIGHTS_SOFTMAX;
            l.sink = geti(s, p + "sink", 0);
            l.out_gate = geti(s, p + "out_gate", 0);
            l.mask_keep = geti(s, p + "mask_keep", 0);
            l.talk = geti(s, p + "talk", 0);
            l.values_are_keys = geti(s, p + "values_are_keys", 0);
            l.gate_wide = geti(s, p + "gate_wide", 0);
            l.qk_norm_weight = geti(s, p + "qk_norm_weight", 0);
            l.o_bias = geti(s, p + "o_bias", 0);
            const std::string rsc = gets(s, p + "rot_scaling", "yarn");
            if (rsc != "yarn" && rsc != "banded")
                return fail("attention: rot_scaling yarn | banded");
            l.rot_banded = rsc == "banded";
            l.rot_low = getd(s, p + "rot_low", 1.0);
            l.rot_high = getd(s, p + "rot_high", 4.0);
            if (l.rot_banded && !(l.rot_high > l.rot_low && l.rot_low > 0))
                return fail("attention: banded frequency scaling needs 0 < rot_low < rot_high");
            if (l.mask != MASK_CAUSAL && l.mask_size < 1)
                return fail("attention: a window or chunk mask needs mask_size >= 1");
            if (l.mask_keep < 0 || (l.mask_keep > 0 && l.mask != MASK_WINDOW) || (l.values_are_keys && l.vdim != l.dim)
                || (l.gate_wide && !l.out_gate) || (l.qk_norm_weight && !l.qk_norm) || (l.o_bias && !s->hyper))
                return fail("attention: mask_keep goes with a window, values_are_keys with vdim = dim, gate_wide with out_gate, qk_norm_weight "
                            "with qk_norm, o_bias with block=sequential");
            if (l.sink && l.weights == WEIGHTS_SIGMOID)
                return fail("attention: a sink belongs to softmax weights");
            l.n_gate = l.out_gate ? (l.gate_wide ? l.heads * l.vdim : l.heads) : 0;
            l.kv_heads = geti(s, p + "kv_heads", l.heads);
            l.maps = geti(s, p + "maps", 1);
            l.diff = getd(s, p + "diff", 0);
            l.scale = getd(s, p + "scale", 1.0 / std::sqrt((double) l.dim));
            l.softcap = getd(s, p + "softcap", 0);
            l.head_norm = geti(s, p + "head_norm", 0);
            l.rot_dims = geti(s, p + "rot_dims", 0);
            l.rot_base = getd(s, p + "rot_base", 10000);
            l.rot_factor = getd(s, p + "rot_factor", 0);
            l.rot_original = getd(s, p + "rot_original", 0);
            l.rot_fast = getd(s, p + "rot_fast", 0);
            l.rot_slow = getd(s, p + "rot_slow", 0);
            if (l.kv_heads < 1 || l.heads % l.kv_heads || l.maps < 1 || l.maps > 2 || (l.rot_dims > 0 && (l.dim & 1)) || (l.rot_dims & 1)
                || l.rot_dims > l.dim)
                return fail("attention: heads must be a multiple of kv_heads, maps 1 or 2, rot_dims even and <= dim, dim even where anything turns");
            if (l.talk && (l.maps != 1 || l.weights != WEIGHTS_SOFTMAX || l.softcap > 0 || l.head_norm || l.head_temp || l.pos_bias))
                return fail("attention: talking heads go with one plain softmax map");
            if (l.talk)
                s->max_pairs = std::max(s->max_pairs, l.heads * l.kv_heads * l.vdim);
            l.n_q = l.heads * l.maps * l.dim;
            l.n_k = l.kv_heads * l.maps * l.dim;
            l.n_v = l.values_are_keys ? 0 : l.kv_heads * l.vdim; // columns of the projection; the cache holds value rows either way
        }
        else if (l.kind == MIX_MAMBA2)
        {
            l.groups = geti(s, p + "groups", 1);
            l.taps = geti(s, p + "conv", 4);
            l.ssm_norm_groups = geti(s, p + "ssm_norm_groups", 1);
            if (l.groups < 1 || l.heads % l.groups || l.ssm_norm_groups < 1 || (l.heads * l.vdim) % l.ssm_norm_groups
                || !stack_ssm_serves(l.vdim, l.dim, l.taps))
                return fail("mamba2: heads a multiple of groups, heads * vdim a multiple of ssm_norm_groups, conv 1 .. 16, state x vdim up to 32 x 1024");
            // columns of the projection: z | x | B | C | dt; the convolution runs over x | B | C
            l.n_conv = l.heads * l.vdim + 2 * l.groups * l.dim;
            l.n_q = l.heads * l.vdim;
            l.n_k = l.n_conv;
            l.n_v = l.heads;
            s->max_conv = std::max(s->max_conv, l.n_conv);
        }
        else if (l.kind == MIX_DELTA)
        {
            l.kv_heads = geti(s, p + "kv_heads", l.heads);
            l.taps = geti(s, p + "conv", 4);
            l.decay_rank = geti(s, p + "decay_rank", 0);
            l.gate_rank = geti(s, p + "gate_rank", 0);
            if (l.kv_heads < 1 || l.heads % l.kv_heads || l.taps < 1 || l.taps > 16 || l.decay_rank < 1 || l.gate_rank < 1
                || !stack_delta_serves(l.dim, l.vdim))
                return fail("delta_rule: heads a multiple of kv_heads, conv 1 .. 16, decay_rank and gate_rank positive, dim up to 512");
            // columns of the projection: q | k | v (the convolution's channels) | beta, padded to 8 | decay latent | gate latent
            l.n_q = l.kv_heads * l.dim;
            l.n_k = l.kv_heads * l.dim;
            l.n_v = l.heads * l.vdim;
            l.n_conv = l.n_q + l.n_k + l.n_v;
            l.n_beta = (l.heads + 7) / 8 * 8;
            l.n_gate = l.n_beta + l.decay_rank + l.gate_rank;
            l.n_gate = (l.n_conv + l.n_gate + 7) / 8 * 8 - l.n_conv; // rows of the element type stay 16-byte aligned
            s->max_conv = std::max(s->max_conv, l.n_conv);
            s->max_hd = std::max(s->max_hd, l.heads * l.dim);
        }
        else
        {
            if (!stack_hgrn2_serves(l.dim, l.vdim))
                return fail("hgrn2: dim up to 512");
            l.n_q = l.heads * l.dim;
            l.n_k = l.heads * l.dim; // forget gate
            l.n_v = l.heads * l.vdim;
        }
        l.n_mix = l.n_q + l.n_k + l.n_v + l.n_rg + l.n_gate;
        const int ff_rows = l.mlp == MLP_MOE ? l.top : 1; // a mixture's products run on one row per (token, chosen expert)
        s->max_proj = std::max(s->max_proj, std::max(l.n_mix, ff_rows * (l.mlp == MLP_RELU2 ? l.ff : 2 * l.ff) + l.n_rg));
        s->max_q = std::max(s->max_q, l.n_q);
        s->max_ctx = std::max(s->max_ctx, l.n_ctx);
        s->max_ff = std::max(s->max_ff, ff_rows * l.ff);
    }
    // execution order
    auto add = [&](int layer, int pass, bool enters) {
        Run r;
        r.layer = layer;
        r.pass = pass;
        r.enters_pass = enters;
        s->runs.push_back(r);
    };
    const bool looped = s->loop_stop > s->loop_start;
    for (int i = 0; i < (looped ? s->loop_start : L); ++i)
        add(i, 0, false);
    if (looped)
    {
        for (int t = 0; t < s->loop_times; ++t)
            for (int i = s->loop_start; i < s->loop_stop; ++i)
                add(i, t, i == s->loop_start);
        for (int i = s->loop_stop; i < L; ++i)
            add(i, 0, false);
    }
    return s;
}

int32_t tllm_stack_set_tensor(tllm_stack_t s, const char* name, int32_t dtype, const int64_t* dims, int32_t nbDims, const void* data)
{
    if (!s || !name || !data || nbDims < 0 || nbDims > 4 || s->finalized)
    {
        set_error("tllm_stack_set_tensor: bad arguments (or the engine is already finalized)");
        return -1;
    }
    HostTensor t;
    for (int i = 0; i < nbDims; ++i)
        t.dims.push_back(dims[i]);
    const int64_t n = t.numel();
    t.v.resize((size_t) n);
    if (dtype == DT_FLOAT)
        std::memcpy(t.v.data(), data, (size_t) n * 4);
    else if (dtype == DT_BF16)
    {
        const uint16_t* b = static_cast<const uint16_t*>(data);
        for (int64_t i = 0; i < n; ++i)
        {
            const uint32_t u = (uint32_t) b[i] << 16;
            std::memcpy(&t.v[(size_t) i], &u, 4);
        }
    }
    else
    {
        set_error("tllm_stack_set_tensor(%s): dtype %d (0 = fp32, 7 = bfloat16)", name, dtype);
        return -1;
    }
    s->host[name] = std::move(t);
    return 0;
}

int32_t tllm_stack_finalize(tllm_stack_t s)
{
    if (!s || s->finalized)
    {
        set_error("tllm_stack_finalize: no engine, or finalized twice");
        return -1;
    }
    const int64_t Wd = s->width;
    const HostTensor* t = need(s, "embed", {s->vocab, Wd});
    if (!t || upload_rows(s, {t}, &s->embed))
        return -1;
    t = need(s, "head", {s->vocab, Wd});
    if (!t || upload_rows(s, {t}, &s->head))
        return -1;
    // a norm weight as the kernels apply it: the stored value plus the design's offset (0, or 1 for weights stored around zero)
    auto norm_vec = [&](const std::string& name, int64_t len, float** out) {
        const HostTensor* v = need(s, name, {len});
        if (!v)
            return -1;
        std::vector<float> w(v->v);
        for (float& f : w)
            f += s->norm_offset;
        return upload_f32(s, w.data(), w.size(), out);
    };
    auto norm_plain = [&](const std::string& name, int64_t len, float** out) {
        const HostTensor* v = need(s, name, {len});
        return (!v || upload_f32(s, v->v.data(), v->v.size(), out)) ? -1 : 0;
    };
    if (norm_vec("final.norm", Wd, &s->final_norm))
        return -1;
    {
        const std::vector<float> one(64, 1.f);
        if (upload_f32(s, one.data(), one.size(), &s->ones))
            return -1;
    }
    if (s->pair_buckets > 0)
    {
        t = need(s, "bigram", {s->pair_buckets + 1, Wd});
        if (!t || upload_rows(s, {t}, &s->pair_table))
            return -1;
    }
    if (s->loop_stop > s->loop_start)
    {
        t = need(s, "loop.step", {s->loop_times, Wd});
        if (!t || upload_f32(s, t->v.data(), t->v.size(), &s->loop_step))
            return -1;
    }
    for (size_t i = 0; i < s->layers.size(); ++i)
    {
        Layer& l = s->layers[i];
        const std::string p = "l" + std::to_string(i) + ".";
        auto vec = [&](const std::string& n, int64_t len, float** out) {
            const HostTensor* v = need(s, p + n, {len});
            return (!v || upload_f32(s, v->v.data(), v->v.size(), out)) ? -1 : 0;
        };
        if (l.weights_of >= 0)
        {
            // the layer runs on another layer's weights: same description, same device tensors; caches and states go by run
            const Layer& src = s->layers[(size_t) l.weights_of];
            if (src.kind != l.kind || src.n_mix != l.n_mix || src.n_ctx != l.n_ctx || src.ff != l.ff || src.mlp != l.mlp || src.dim != l.dim
                || src.heads != l.heads || src.experts != l.experts || src.identity != l.identity || src.kv_rank != l.kv_rank
                || src.rot_part != l.rot_part || src.taps != l.taps)
            {
                set_error("tllm_stack_finalize: layer %d uses the weights of layer %d, but their shapes differ", (int) i, l.weights_of);
                return -1;
            }
            const int from = l.weights_of;
            l = src;
            l.weights_of = from;
            continue;
        }
        if (norm_vec(p + "norm1", Wd, &l.norm1))
            return -1;
        if (s->token_shift && vec("shift", Wd, &l.shift))
            return -1;
        const HostTensor* rg1 = nullptr;
        if (!s->hyper)
        {
            rg1 = need(s, p + "rg1", {Wd, Wd});
            if (!rg1 || vec("rg1.b", Wd, &l.rg1_b))
                return -1;
        }
        else
        {
            // hyper-connections of the two sublayers; a model with one plain stream has no such tensors: mix = out = in = 1
            for (int q = 0; q < 2; ++q)
            {
                HyperW& hw = l.hc[q];
                const std::string hp = "hc" + std::to_string(q + 1) + ".";
                if (s->host.count(p + hp + "mix") == 0 && s->streams == 1)
                {
                    hw.mix = hw.out = hw.in = s->ones;
                    continue;
                }
                if (q == 1 && l.ff == 0)
                    continue;
                const HostTensor* m = need(s, p + hp + "mix", {s->streams, s->streams});
                if (!m || upload_f32(s, m->v.data(), m->v.size(), &hw.mix) || vec(hp + "out", s->streams, &hw.out)
                    || vec(hp + "in", s->streams, &hw.in))
                    return -1;
            }
        }
        if (l.kind == MIX_MAMBA2)
        {
            const HostTensor* win = need(s, p + "mix.in", {l.n_mix, Wd});
            const HostTensor* wo = need(s, p + "mix.o", {Wd, l.n_ctx});
            const HostTensor* cw = need(s, p + "mix.conv", {l.n_conv, l.taps});
            if (!win || !wo || !cw || upload_rows(s, {win}, &l.w_mix) || upload_rows(s, {wo}, &l.w_o)
                || upload_f32(s, cw->v.data(), cw->v.size(), &l.conv_w) || vec("mix.conv.b", l.n_conv, &l.conv_b)
                || vec("mix.dt_bias", l.heads, &l.dt_bias) || vec("mix.A_log", l.heads, &l.a_log) || vec("mix.D", l.heads, &l.d_skip)
                || vec("mix.norm", l.n_ctx, &l.hnorm))
                return -1;
        }
        if (l.kind == MIX_DELTA)
        {
            const int64_t QK = l.n_q, HV = l.n_v, HD = (int64_t) l.heads * l.dim;
            const HostTensor *wq = need(s, p + "mix.q", {QK, Wd}), *wk = need(s, p + "mix.k", {QK, Wd}), *wv = need(s, p + "mix.v", {HV, Wd}),
                             *wb = need(s, p + "mix.b", {l.heads, Wd}), *a1 = need(s, p + "mix.a1", {l.decay_rank, Wd}),
                             *a2 = need(s, p + "mix.a2", {HD, l.decay_rank}), *g1 = need(s, p + "mix.g1", {l.gate_rank, Wd}),
                             *g2 = need(s, p + "mix.g2", {HV, l.gate_rank}), *wo = need(s, p + "mix.o", {Wd, HV}),
                             *cq = need(s, p + "mix.q.conv", {QK, l.taps}), *ck = need(s, p + "mix.k.conv", {QK, l.taps}),
                             *cv = need(s, p + "mix.v.conv", {HV, l.taps});
            if (!wq || !wk || !wv || !wb || !a1 || !a2 || !g1 || !g2 || !wo || !cq || !ck || !cv)
                return -1;
            HostTensor pad_b, pad_end; // zero rows: beta's columns up to a multiple of 8, the projection's up to a multiple of 8
            pad_b.dims = {l.n_beta - l.heads, Wd};
            pad_b.v.assign((size_t) pad_b.numel(), 0.f);
            pad_end.dims = {l.n_gate - l.n_beta - l.decay_rank - l.gate_rank, Wd};
            pad_end.v.assign((size_t) pad_end.numel(), 0.f);
            std::vector<float> taps(cq->v);
            taps.insert(taps.end(), ck->v.begin(), ck->v.end());
            taps.insert(taps.end(), cv->v.begin(), cv->v.end());
            if (upload_rows(s, {wq, wk, wv, wb, &pad_b, a1, g1, &pad_end}, &l.w_mix) || upload_rows(s, {wo}, &l.w_o) || upload_rows(s, {a2}, &l.w_a2)
                || upload_rows(s, {g2}, &l.w_g2) || upload_f32(s, taps.data(), taps.size(), &l.conv_w) || vec("mix.dt_bias", HD, &l.dt_bias)
                || vec("mix.A_log", l.heads, &l.a_log) || vec("mix.norm", l.vdim, &l.hnorm))
                return -1;
        }
        const bool own_mix = l.kind == MIX_MAMBA2 || l.kind == MIX_DELTA; // kinds whose projection is put together above
        const bool q_latent = l.kind == MIX_LATENT && l.q_rank > 0;
        const HostTensor* wq = own_mix ? nullptr : need(s, p + (q_latent ? "mix.dq" : "mix.q"), {l.n_q, Wd});
        const HostTensor* wk = own_mix
            ? nullptr
            : need(s, p + (l.kind == MIX_ATTENTION ? "mix.k" : (l.kind == MIX_LATENT ? "mix.dkv" : "mix.f")), {l.n_k, Wd});
        const HostTensor* wv = (l.kind == MIX_LATENT || own_mix || l.values_are_keys) ? nullptr : need(s, p + "mix.v", {l.n_v, Wd});
        const HostTensor* wo = own_mix ? nullptr : need(s, p + "mix.o", {Wd, l.n_ctx});
        const HostTensor* wg = l.n_gate ? need(s, p + "mix.g", {l.n_gate, Wd}) : nullptr;
        if (!own_mix && (!wq || !wk || (!wv && l.kind != MIX_LATENT && !l.values_are_keys) || !wo || (l.n_gate && !wg)))
            return -1;
        if (!own_mix)
        {
            std::vector<const HostTensor*> rows = {wq, wk};
            if (wv)
                rows.push_back(wv);
            if (rg1)
                rows.push_back(rg1);
            if (wg)
                rows.push_back(wg);
            if (upload_rows(s, rows, &l.w_mix) || upload_rows(s, {wo}, &l.w_o))
                return -1;
        }
        if (l.kind == MIX_ATTENTION || l.kind == MIX_LATENT)
        {
            std::vector<float> fr((size_t) std::max(l.rot_dims / 2, 1));
            if (l.rot_banded)
                stack_rope_freqs_banded(fr.data(), l.rot_dims, l.rot_base, l.rot_factor, l.rot_original, l.rot_low, l.rot_high), l.mscale = 1.f;
            else
                l.mscale = stack_rope_freqs(fr.data(), l.rot_dims, l.rot_base, l.rot_factor, l.rot_original, l.rot_fast, l.rot_slow);
            if (upload_f32(s, fr.data(), fr.size(), &l.freq))
                return -1;
        }
        if (l.kind == MIX_LATENT)
        {
            const int64_t C = l.kv_rank, D = l.dim, E = l.vdim, H = l.heads;
            const HostTensor* uk = need(s, p + "mix.uk", {H * D, C});
            const HostTensor* uv = need(s, p + "mix.uv", {H * E, C});
            if (!uk || !uv || norm_plain(p + "mix.dkv.norm", C, &l.lat_norm))
                return -1;
            if (q_latent)
            {
                const HostTensor* uq = need(s, p + "mix.uq", {H * (D + l.rot_part), l.q_rank});
                if (!uq || upload_rows(s, {uq}, &l.w_uq) || norm_plain(p + "mix.dq.norm", l.q_rank, &l.cq_norm))
                    return -1;
            }
            if (l.sink && vec("mix.sink", l.heads, &l.sinkv))
                return -1;
            // W_uk^T per head, [kv_rank, dim]: the query side of the absorbed score is a product with these rows
            HostTensor tr;
            tr.dims = {H * C, D};
            tr.v.resize((size_t) (H * C * D));
            for (int64_t h = 0; h < H; ++h)
                for (int64_t d = 0; d < D; ++d)
                    for (int64_t c = 0; c < C; ++c)
                        tr.v[(size_t) ((h * C + c) * D + d)] = uk->v[(size_t) ((h * D + d) * C + c)];
            if (upload_rows(s, {&tr}, &l.w_ukT) || upload_rows(s, {uv}, &l.w_uv))
                return -1;
        }
        else if (l.kind == MIX_ATTENTION)
        {
            l.lambda = 0.f;
            if (l.maps == 2)
            {
                const HostTensor *a1 = need(s, p + "mix.lq1", {l.dim}), *b1 = need(s, p + "mix.lk1", {l.dim}),
                                 *a2 = need(s, p + "mix.lq2", {l.dim}), *b2 = need(s, p + "mix.lk2", {l.dim});
                if (!a1 || !b1 || !a2 || !b2)
                    return -1;
                float d1 = 0.f, d2 = 0.f;
                for (int d = 0; d < l.dim; ++d)
                {
                    d1 += a1->v[d] * b1->v[d];
                    d2 += a2->v[d] * b2->v[d];
                }
                l.lambda = std::exp(d1) - std::exp(d2) + (float) l.diff;
            }
            if (l.qkv_bias)
            {
                const HostTensor *bq = need(s, p + "mix.q.b", {l.n_q}), *bk = need(s, p + "mix.k.b", {l.n_k}),
                                 *bv = l.values_are_keys ? nullptr : need(s, p + "mix.v.b", {l.n_v});
                if (!bq || !bk || (!bv && !l.values_are_keys))
                    return -1;
                std::vector<float> b(bq->v);
                b.insert(b.end(), bk->v.begin(), bk->v.end());
                if (bv)
                    b.insert(b.end(), bv->v.begin(), bv->v.end());
                if (upload_f32(s, b.data(), b.size(), &l.bias))
                    return -1;
            }
            if (l.head_temp && vec("mix.temp", l.heads, &l.temp))
                return -1;
            if (l.pos_bias == 1)
            {
                std::vector<float> sl((size_t) l.heads);
                for (int h = 0; h < l.heads; ++h)
                    sl[(size_t) h] = (float) std::exp2(-l.slope_base * (h + 1) / l.heads);
                if (upload_f32(s, sl.data(), sl.size(), &l.slope))
                    return -1;
            }
            if (l.pos_bias == 2 && (vec("mix.r1", l.heads, &l.r1) || vec("mix.r2", l.heads, &l.r2)))
                return -1;
            if (l.sink == 1 && vec("mix.sink", l.heads, &l.sinkv))
                return -1;
            if (l.sink == 2)
            {
                // a constant sink of logit 0: the softmax denominator holds one more 1
                const std::vector<float> zero((size_t) l.heads, 0.f);
                if (upload_f32(s, zero.data(), zero.size(), &l.sinkv))
                    return -1;
            }
            if (l.weights == WEIGHTS_SIGMOID && vec("mix.pb", l.heads, &l.wbias))
                return -1;
            if (l.talk)
            {
                const HostTensor* tk = need(s, p + "mix.talk", {l.heads, l.heads});
                if (!tk || upload_f32(s, tk->v.data(), tk->v.size(), &l.talkw))
                    return -1;
            }
            if (l.qk_norm_weight && (vec("mix.q.norm", l.dim, &l.q_norm) || vec("mix.k.norm", l.dim, &l.k_norm)))
                return -1;
            if (l.o_bias && vec("mix.o.b", Wd, &l.o_biasv))
                return -1;
        }
        else if (l.kind == MIX_HGRN2)
        {
            if (vec("mix.f.b", l.n_k, &l.f_bias) || vec("mix.lower", l.n_k, &l.lower) || vec("mix.norm", l.vdim, &l.hnorm))
                return -1;
        }
        if (l.ff > 0 && l.mlp == MLP_MOE)
        {
            // experts stacked: [gate_e; up_e] rows per expert, then the down matrices; router and correction stay fp32
            const int ne = l.experts + l.identity;
            const HostTensor* rw = need(s, p + "mlp.router", {ne, Wd});
            if (norm_vec(p + "norm2", Wd, &l.norm2) || !rw || upload_f32(s, rw->v.data(), rw->v.size(), &l.router_w))
                return -1;
            if (s->host.count(p + "mlp.correction") && vec("mlp.correction", ne, &l.correction))
                return -1;
            std::vector<const HostTensor*> gu, dn;
            for (int e = 0; e < l.experts; ++e)
            {
                const std::string ep = p + "mlp.e" + std::to_string(e) + ".";
                const HostTensor *g = need(s, ep + "gate", {l.ff, Wd}), *u = need(s, ep + "up", {l.ff, Wd}), *d = need(s, ep + "down", {Wd, l.ff});
                if (!g || !u || !d)
                    return -1;
                gu.push_back(g);
                gu.push_back(u);
                dn.push_back(d);
            }
            if (upload_rows(s, gu, &l.w_gu) || upload_rows(s, dn, &l.w_down))
                return -1;
        }
        else if (l.ff > 0)
        {
            if (norm_vec(p + "norm2", Wd, &l.norm2))
                return -1;
            const HostTensor* rg2 = nullptr;
            if (!s->hyper)
            {
                rg2 = need(s, p + "rg2", {Wd, Wd});
                if (!rg2 || vec("rg2.b", Wd, &l.rg2_b))
                    return -1;
            }
            const HostTensor* wgt = l.mlp == MLP_GELU_GATE ? need(s, p + "mlp.gate", {l.ff, Wd}) : nullptr;
            const HostTensor* wu = need(s, p + "mlp.up", {l.ff, Wd});
            const HostTensor* wd = need(s, p + "mlp.down", {Wd, l.ff});
            if ((l.mlp == MLP_GELU_GATE && !wgt) || !wu || !wd)
                return -1;
            std::vector<const HostTensor*> rows;
            if (wgt)
                rows.push_back(wgt);
            rows.push_back(wu);
            if (rg2)
                rows.push_back(rg2);
            if (upload_rows(s, rows, &l.w_gu) || upload_rows(s, {wd}, &l.w_down))
                return -1;
        }
    }
    size_t ws_floats = 0;
    for (const Layer& l : s->layers)
        if (l.kind == MIX_ATTENTION)
            ws_floats = std::max(ws_floats, stack_attn_workspace_floats(l.talk ? l.heads * l.kv_heads : l.heads, l.maps, l.vdim));
        else if (l.kind == MIX_LATENT)
            ws_floats = std::max(ws_floats, stack_attn_workspace_floats(l.heads, 1, l.kv_rank));
    if (ws_floats)
    {
        void* ws = nullptr;
        if (alloc_zero(s, ws_floats * 4, &ws))
            return -1;
        s->attn_ws = (float*) ws;
    }
    for (Run& r : s->runs)
    {
        const Layer& l = s->layers[r.layer];
        if (l.kind == MIX_LATENT)
        {
            // one key row [latent | rotated part] and one value row (the latent, channel-major) per token, shared by all heads
            if (alloc_zero(s, (size_t) s->blocks * s->page * (l.kv_rank + l.rot_part) * s->es, &r.k_pool)
                || alloc_zero(s, (size_t) s->blocks * s->page * l.kv_rank * s->es, &r.v_pool))
                return -1;
        }
        else if (l.kind == MIX_ATTENTION)
        {
            if (alloc_zero(s, (size_t) s->blocks * l.kv_heads * l.maps * s->page * l.dim * s->es, &r.k_pool)
                || alloc_zero(s, (size_t) s->blocks * l.kv_heads * s->page * l.vdim * s->es, &r.v_pool))
                return -1;
        }
        else if (l.kind == MIX_MAMBA2 || l.kind == MIX_DELTA)
        {
            void *st = nullptr, *cv = nullptr;
            if (alloc_zero(s, (size_t) s->slots * l.heads * l.dim * l.vdim * 4, &st)
                || alloc_zero(s, (size_t) s->slots * (l.taps - 1) * l.n_conv * 4, &cv))
                return -1;
            r.state = (float*) st;
            r.conv_state = (float*) cv;
        }
        else
        {
            void* st = nullptr;
            if (alloc_zero(s, (size_t) s->slots * l.heads * l.dim * l.vdim * 4, &st))
                return -1;
            r.state = (float*) st;
        }
        if (s->token_shift)
        {
            void* cr = nullptr;
            if (alloc_zero(s, (size_t) s->slots * s->width * 4, &cr))
                return -1;
            r.shift_carry = (float*) cr;
        }
    }
    s->host.clear();
    s->finalized = true;
    return 0;
}

int32_t tllm_stack_step(tllm_stack_t s, const tllm_stack_batch_t* b, float* logits_out, int32_t* next_ids_out, void* stream_v)
{
    if (!s || !s->finalized || !b)
    {
        set_error("tllm_stack_step: the engine is not finalized");
        return -1;
    }
    hipStream_t stream = (hipStream_t) stream_v;
    const int T = b->n_tokens, E = b->n_entries, NW = b->n_want, MB = b->max_blocks;
    if (T < 1 || E < 1 || NW < 0 || MB < 1 || !b->tokens || !b->ent_count || !b->ent_pos0 || !b->ent_slot || !b->block_table
        || (NW > 0 && !b->want_rows))
    {
        set_error("tllm_stack_step: empty batch or missing array");
        return -1;
    }
    // ---- every index the kernels will follow is checked here
    int64_t sum = 0;
    int max_count = 0, max_ctx = 0;
    for (int e = 0; e < E; ++e)
    {
        const int c = b->ent_count[e], p0 = b->ent_pos0[e], sl = b->ent_slot[e];
        if (c < 1 || p0 < 0 || sl < 0 || sl >= s->slots)
        {
            set_error("tllm_stack_step: entry %d has count %d, pos0 %d, slot %d (slots: %d)", e, c, p0, sl, s->slots);
            return -1;
        }
        for (int e2 = 0; e2 < e; ++e2)
            if (b->ent_slot[e2] == sl)
            {
                set_error("tllm_stack_step: entries %d and %d share slot %d", e2, e, sl);
                return -1;
            }
        const int nb = (p0 + c + s->page - 1) / s->page;
        if (nb > MB)
        {
            set_error("tllm_stack_step: entry %d needs %d blocks, its table has %d", e, nb, MB);
            return -1;
        }
        for (int j = 0; j < nb; ++j)
        {
            const int id = b->block_table[(size_t) e * MB + j];
            if (id < 0 || id >= s->blocks)
            {
                set_error("tllm_stack_step: entry %d, block %d of its table is %d (pool: %d blocks)", e, j, id, s->blocks);
                return -1;
            }
        }
        sum += c;
        max_count = std::max(max_count, c);
        max_ctx = std::max(max_ctx, p0 + c);
    }
    if (sum != T)
    {
        set_error("tllm_stack_step: the entries hold %lld tokens, the batch %d", (long long) sum, T);
        return -1;
    }
    for (int t = 0; t < T; ++t)
        if (b->tokens[t] < 0 || b->tokens[t] >= s->vocab)
        {
            set_error("tllm_stack_step: token %d at row %d is outside the vocabulary of %d", b->tokens[t], t, s->vocab);
            return -1;
        }
    for (int i = 0; i < NW; ++i)
        if (b->want_rows[i] < 0 || b->want_rows[i] >= T)
        {
            set_error("tllm_stack_step: wanted row %d is outside the batch of %d", b->want_rows[i], T);
            return -1;
        }
    // ---- metadata: one packed int32 image, one copy
    const size_t n_ints = (size_t) 4 * T + (size_t) 4 * E + (size_t) E * MB + NW;
    if (ensure_scratch(s, T, std::max(NW, 1), (int) n_ints))
        return -1;
    int32_t* h = s->pinned;
    int32_t *h_tok = h, *h_tent = h + T, *h_tpos = h + 2 * T, *h_first = h + 3 * T, *h_count = h_first + E, *h_pos0 = h_count + E,
            *h_slot = h_pos0 + E, *h_table = h_slot + E, *h_want = h_table + (size_t) E * MB, *h_prev = h_want + NW;
    std::memcpy(h_tok, b->tokens, (size_t) T * 4);
    int row = 0;
    for (int e = 0; e < E; ++e)
    {
        h_first[e] = row;
        h_count[e] = b->ent_count[e];
        h_pos0[e] = b->ent_pos0[e];
        h_slot[e] = b->ent_slot[e];
        for (int i = 0; i < b->ent_count[e]; ++i, ++row)
        {
            h_tent[row] = e;
            h_tpos[row] = b->ent_pos0[e] + i;
            // the token before this one in its sequence (-1: none): the row above, or what the slot's sequence ended its last step with
            h_prev[row] = i > 0 ? b->tokens[row - 1] : (b->ent_pos0[e] > 0 ? s->last_tok[(size_t) b->ent_slot[e]] : -1);
        }
        s->last_tok[(size_t) b->ent_slot[e]] = b->tokens[row - 1];
        const int nb = (b->ent_pos0[e] + b->ent_count[e] + s->page - 1) / s->page;
        for (int j = 0; j < MB; ++j)
            h_table[(size_t) e * MB + j] = j < nb ? b->block_table[(size_t) e * MB + j] : 0;
    }
    for (int i = 0; i < NW; ++i)
        h_want[i] = b->want_rows[i];
    HIP_OK(hipMemcpyAsync(s->ints, h, n_ints * 4, hipMemcpyHostToDevice, stream));
    const int32_t* d = s->ints;
    const int32_t *d_tok = d, *d_tent = d + T, *d_tpos = d + 2 * T, *d_first = d + 3 * T, *d_count = d_first + E, *d_pos0 = d_count + E,
                  *d_slot = d_pos0 + E, *d_table = d_slot + E, *d_want = d_table + (size_t) E * MB, *d_prev = d_want + NW;

    const int Wd = s->width;
    const bool looped = s->loop_stop > s->loop_start;
    const int64_t stream_stride = (int64_t) T * Wd;
    if (launch_stack_embed(s->x, looped && s->loop_times > 1 ? s->x0 : nullptr, d_tok, s->embed, s->dtype, T, Wd, s->vocab, s->emb_scale, stream,
            s->streams, stream_stride))
        return -1;
    if (s->pair_buckets > 0
        && launch_stack_pair_embed(s->x, d_tok, d_prev, s->pair_table, s->dtype, T, Wd, s->pair_buckets, s->pair_mul_prev, s->pair_mul_cur, stream,
            s->streams, stream_stride))
        return -1;
    s->tap_tokens = T;

    // P1 = h1 W_mix^T, then the mixer: its context rows land in s->ctx
    auto run_mixer = [&](const Layer& l, const Run& r) -> int {
        StackGemmParams g;
        g.dtype = s->dtype;
        g.M = T;
        g.N = l.n_mix;
        g.K = Wd;
        g.a = s->h1;
        g.lda = Wd;
        g.w = l.w_mix;
        g.c = s->proj;
        g.ldc = l.n_mix;
        if (launch_stack_gemm(g, stream))
            return -1;
        if (l.kind == MIX_DELTA)
        {
            // convolution + silu of q | k | v (and the sequence's new tail)
            StackSsmParams sp;
            sp.dtype = s->dtype;
            sp.tokens = T;
            sp.entries = E;
            sp.taps = l.taps;
            sp.proj = s->proj;
            sp.ldp = l.n_mix;
            sp.conv_w = l.conv_w;
            sp.conv_channels = l.n_conv;
            sp.conv_col = 0;
            sp.conv_state = r.conv_state;
            sp.xbc = s->xbc;
            sp.tok_entry = d_tent;
            sp.tok_pos = d_tpos;
            sp.ent_slot = d_slot;
            sp.ent_first = d_first;
            sp.ent_count = d_count;
            sp.ent_pos0 = d_pos0;
            if (launch_stack_ssm_conv(sp, stream))
                return -1;
            // the two low-rank projections' second halves, in fp32: the decay's pre-activation and the output gate's
            const int col_b = l.n_conv, col_a = col_b + l.n_beta, col_g = col_a + l.decay_rank;
            StackGemmParams lr;
            lr.dtype = s->dtype;
            lr.out_f32 = 1;
            lr.M = T;
            lr.N = l.heads * l.dim;
            lr.K = l.decay_rank;
            lr.a = (const char*) s->proj + (size_t) col_a * s->es;
            lr.lda = l.n_mix;
            lr.w = l.w_a2;
            lr.c = s->dl_a;
            lr.ldc = lr.N;
            if (launch_stack_gemm(lr, stream))
                return -1;
            lr.N = l.n_ctx;
            lr.K = l.gate_rank;
            lr.a = (const char*) s->proj + (size_t) col_g * s->es;
            lr.w = l.w_g2;
            lr.c = s->dl_g;
            lr.ldc = lr.N;
            if (launch_stack_gemm(lr, stream))
                return -1;
            StackDeltaParams dp;
            dp.dtype = s->dtype;
            dp.tokens = T;
            dp.entries = E;
            dp.heads = l.heads;
            dp.qk_heads = l.kv_heads;
            dp.dim = l.dim;
            dp.vdim = l.vdim;
            dp.x = s->xbc;
            dp.beta_raw = (const char*) s->proj + (size_t) col_b * s->es;
            dp.ld_beta = l.n_mix;
            dp.decay_raw = s->dl_a;
            dp.dt_bias = l.dt_bias;
            dp.a_log = l.a_log;
            dp.gate_raw = s->dl_g;
            dp.norm_w = l.hnorm;
            dp.eps = s->eps;
            dp.state = r.state;
            dp.o32 = s->o32;
            dp.out = s->ctx;
            dp.ent_slot = d_slot;
            dp.ent_first = d_first;
            dp.ent_count = d_count;
            dp.ent_pos0 = d_pos0;
            dp.max_count = max_count;
            return (launch_stack_delta_scan(dp, stream) || launch_stack_delta_out(dp, stream)) ? -1 : 0;
        }
        if (l.kind == MIX_MAMBA2)
        {
            StackSsmParams sp;
            sp.dtype = s->dtype;
            sp.tokens = T;
            sp.entries = E;
            sp.heads = l.heads;
            sp.vdim = l.vdim;
            sp.state = l.dim;
            sp.groups = l.groups;
            sp.taps = l.taps;
            sp.proj = s->proj;
            sp.ldp = l.n_mix;
            sp.conv_w = l.conv_w;
            sp.conv_b = l.conv_b;
            sp.dt_bias = l.dt_bias;
            sp.a_log = l.a_log;
            sp.d_skip = l.d_skip;
            sp.conv_state = r.conv_state;
            sp.ssm_state = r.state;
            sp.xbc = s->xbc;
            sp.y32 = s->o32;
            sp.tok_entry = d_tent;
            sp.tok_pos = d_tpos;
            sp.ent_slot = d_slot;
            sp.ent_first = d_first;
            sp.ent_count = d_count;
            sp.ent_pos0 = d_pos0;
            // convolution + silu (and the sequence's new tail), the recurrence with skip and gate, the norm in parts of the row
            if (launch_stack_ssm_conv(sp, stream) || launch_stack_ssm_scan(sp, stream))
                return -1;
            return launch_stack_group_rmsnorm(s->ctx, nullptr, s->o32, nullptr, l.hnorm, nullptr, s->dtype, T, l.n_ctx, l.ssm_norm_groups, s->eps,
                stream);
        }
        if (l.kind == MIX_HGRN2)
        {
            StackHgrnParams hp;
            hp.dtype = s->dtype;
            hp.tokens = T;
            hp.entries = E;
            hp.heads = l.heads;
            hp.dim = l.dim;
            hp.vdim = l.vdim;
            hp.proj = s->proj;
            hp.ldp = l.n_mix;
            hp.f_bias = l.f_bias;
            hp.lower = l.lower;
            hp.norm_w = l.hnorm;
            hp.eps = s->eps;
            hp.state = r.state;
            hp.ent_slot = d_slot;
            hp.ent_first = d_first;
            hp.ent_count = d_count;
            hp.ent_pos0 = d_pos0;
            hp.max_count = max_count;
            hp.o32 = s->o32;
            hp.out = s->ctx;
            return launch_stack_hgrn2(hp, stream);
        }
        StackAttnParams a;
        a.dtype = s->dtype;
        a.tokens = T;
        a.entries = E;
        a.heads = l.heads;
        a.freq = l.freq;
        a.scale = (float) l.scale;
        a.eps = s->eps;
        a.proj = s->proj;
        a.ldp = l.n_mix;
        a.q = s->q;
        a.k_pool = r.k_pool;
        a.v_pool = r.v_pool;
        a.page = s->page;
        a.max_blocks = MB;
        a.block_table = d_table;
        a.tok_entry = d_tent;
        a.tok_pos = d_tpos;
        a.ent_first = d_first;
        a.ent_count = d_count;
        a.ent_pos0 = d_pos0;
        a.max_count = max_count;
        a.max_context = max_ctx;
        a.split_ws = s->attn_ws;
        if (l.kind == MIX_LATENT)
        {
            // absorbed form: one shared key/value head over [latent | rotated part]; queries [W_uk^T q_plain | rotated q part]
            const int C = l.kv_rank, R = l.rot_part, D = l.dim, H = l.heads;
            a.kv_heads = 1;
            a.maps = 1;
            a.dim = C + R;
            a.vdim = C;
            a.rot_dims = l.rot_dims;
            a.rot_halves = l.rot_halves;
            a.mscale = l.mscale;
            a.mask = l.mask;
            a.mask_size = l.mask_size;
            a.sink = l.sinkv;
            a.out = s->lat;
            const void* q_src = s->proj;
            int64_t ldq = l.n_mix;
            if (l.q_rank > 0)
            {
                // queries through their own latent: norm of the first q_rank columns, then the expansion to every head's [plain | rotated]
                if (launch_stack_row_rmsnorm(s->cq, l.q_rank, s->proj, l.n_mix, l.cq_norm, s->dtype, T, l.q_rank, s->eps, stream))
                    return -1;
                StackGemmParams uq;
                uq.dtype = s->dtype;
                uq.M = T;
                uq.N = H * (D + R);
                uq.K = l.q_rank;
                uq.a = s->cq;
                uq.lda = l.q_rank;
                uq.w = l.w_uq;
                uq.c = s->qfull;
                uq.ldc = uq.N;
                if (launch_stack_gemm(uq, stream))
                    return -1;
                q_src = s->qfull;
                ldq = uq.N;
            }
            if (launch_stack_latent_prep(a, D, l.lat_norm, stream, q_src, ldq, l.n_q))
                return -1;
            StackGemmParams qa;
            qa.dtype = s->dtype;
            qa.M = T;
            qa.N = C;
            qa.K = D;
            qa.a = q_src;
            qa.lda = ldq;
            qa.w = l.w_ukT;
            qa.c = s->q;
            qa.ldc = (int64_t) H * (C + R);
            qa.batch = H;
            qa.stride_a = D + R;
            qa.stride_w = (int64_t) C * D;
            qa.stride_c = C + R;
            if (launch_stack_gemm(qa, stream) || launch_stack_attention(a, stream))
                return -1;
            StackGemmParams ve; // head h: ctx[:, h] = lat[:, h] W_uv,h^T
            ve.dtype = s->dtype;
            ve.M = T;
            ve.N = l.vdim;
            ve.K = C;
            ve.a = s->lat;
            ve.lda = (int64_t) H * C;
            ve.w = l.w_uv;
            ve.c = s->ctx;
            ve.ldc = l.n_ctx;
            ve.batch = H;
            ve.stride_a = C;
            ve.stride_w = (int64_t) l.vdim * C;
            ve.stride_c = l.vdim;
            return launch_stack_gemm(ve, stream);
        }
        a.kv_heads = l.kv_heads;
        a.maps = l.maps;
        a.dim = l.dim;
        a.vdim = l.vdim;
        a.rot_dims = l.rot_dims;
        a.mscale = l.mscale;
        a.softcap = (float) l.softcap;
        a.lambda = l.lambda;
        a.out_scale = (float) (1.0 - l.diff);
        a.head_norm = l.head_norm;
        a.temp = l.temp;
        a.slope = l.slope;
        a.log_r1 = l.r1;
        a.log_r2 = l.r2;
        a.mask = l.mask;
        a.mask_size = l.mask_size;
        a.mask_keep = l.mask_keep;
        a.talk = l.talkw;
        a.pair_ws = l.talk ? s->pairs : nullptr;
        a.values_are_keys = l.values_are_keys;
        a.gate_wide = l.gate_wide;
        a.q_norm_w = l.q_norm;
        a.k_norm_w = l.k_norm;
        a.weights = l.weights;
        a.sink = l.sinkv;
        a.wbias = l.wbias;
        a.bias = l.bias;
        a.qk_unit_norm = l.qk_norm;
        if (l.n_gate)
        {
            a.out_gate = (const char*) s->proj + (size_t) (l.n_q + l.n_k + l.n_v + l.n_rg) * s->es;
            a.ld_gate = l.n_mix;
        }
        a.out = s->ctx;
        return (launch_stack_rope_kv(a, stream) || launch_stack_attention(a, stream)) ? -1 : 0;
    };

    // residual=hyper: the sublayer result in y32 that has not yet been folded into the streams, and the launch that folds it,
    // combines the streams for the next reader and norms the combination
    const HyperW* pending = nullptr;
    auto hyper = [&](const float* in, void* h, const float* w, float* sum_out, float* h32 = nullptr) -> int {
        StackHyperParams hp;
        hp.dtype = s->dtype;
        hp.tokens = T;
        hp.width = Wd;
        hp.streams = s->streams;
        hp.x = s->x;
        hp.stream_stride = stream_stride;
        if (pending)
        {
            hp.y = s->y32;
            hp.mix = pending->mix;
            hp.out = pending->out;
        }
        hp.in = in;
        hp.h = h;
        hp.w = w;
        hp.eps = s->eps;
        hp.sum_out = sum_out;
        hp.h32 = h32;
        pending = nullptr;
        return launch_stack_hyper_norm(hp, stream);
    };

    for (size_t ri = 0; ri < s->runs.size(); ++ri)
    {
        const Run& r = s->runs[ri];
        const Layer& l = s->layers[r.layer];
        if (s->hyper)
        {
            if (s->token_shift)
            {
                // the norm leaves its row in fp32; the mixer reads it blended with the previous token's
                StackShiftParams sh;
                sh.dtype = s->dtype;
                sh.tokens = T;
                sh.entries = E;
                sh.width = Wd;
                sh.n = s->h32;
                sh.mu = l.shift;
                sh.carry = r.shift_carry;
                sh.h = s->h1;
                sh.tok_entry = d_tent;
                sh.tok_pos = d_tpos;
                sh.ent_slot = d_slot;
                sh.ent_first = d_first;
                sh.ent_count = d_count;
                sh.ent_pos0 = d_pos0;
                if (hyper(l.hc[0].in, nullptr, l.norm1, nullptr, s->h32) || launch_stack_token_shift(sh, stream))
                    return -1;
            }
            else if (hyper(l.hc[0].in, s->h1, l.norm1, nullptr))
                return -1;
            if (run_mixer(l, r))
                return -1;
            StackGemmParams o; // y = ctx Wo^T in fp32: the residual sum is 32-bit
            o.dtype = s->dtype;
            o.out_f32 = 1;
            o.M = T;
            o.N = Wd;
            o.K = l.n_ctx;
            o.a = s->ctx;
            o.lda = l.n_ctx;
            o.w = l.w_o;
            o.c = s->y32;
            o.ldc = Wd;
            o.bias = l.o_biasv;
            if (launch_stack_gemm(o, stream))
                return -1;
            pending = &l.hc[0];
            if (l.ff > 0)
            {
                if (hyper(l.hc[1].in, s->h1, l.norm2, nullptr))
                    return -1;
                StackGemmParams u;
                u.dtype = s->dtype;
                u.M = T;
                u.K = Wd;
                u.a = s->h1;
                u.lda = Wd;
                u.w = l.w_gu;
                const void* act = s->act;
                if (l.mlp == MLP_MOE)
                {
                    const size_t pairs = (size_t) T * l.top;
                    StackMoeParams mp;
                    mp.dtype = s->dtype;
                    mp.tokens = T;
                    mp.width = Wd;
                    mp.experts = l.experts;
                    mp.identity = l.identity;
                    mp.top = l.top;
                    mp.group_count = l.route_groups;
                    mp.group_keep = l.route_keep;
                    mp.scale = (float) l.route_scale;
                    mp.score = l.route_sigmoid ? ROUTE_SIGMOID : ROUTE_SOFTMAX;
                    mp.weight_input = l.route_weight_input;
                    mp.h = s->h1;
                    mp.router_w = l.router_w;
                    mp.correction = l.correction;
                    mp.topk_idx = s->moe_i;
                    mp.slot_of_pair = s->moe_i + pairs;
                    mp.pair_of_slot = s->moe_i + 2 * pairs;
                    mp.group_off = s->moe_i + 3 * pairs;
                    mp.topk_w = s->moe_w;
                    mp.logits = s->moe_w + pairs;
                    mp.a_sorted = s->moe_a;
                    if (launch_stack_moe_route(mp, stream) || launch_stack_moe_sort(mp, stream))
                        return -1;
                    // per expert: [gate; up] on its rows, silu(gate) * up, down in fp32; an expert's rows are at most one per token
                    u.M = T;
                    u.N = 2 * l.ff;
                    u.a = s->moe_a;
                    u.c = s->proj;
                    u.ldc = u.N;
                    u.batch = l.experts;
                    u.stride_w = (int64_t) 2 * l.ff * Wd;
                    u.group_off = mp.group_off;
                    u.group_rows = (int) std::min<int64_t>(T, (pairs + l.experts - 1) / l.experts);
                    if (launch_stack_gemm(u, stream)
                        || launch_stack_gelu_gate(s->act, s->proj, s->dtype, (int) pairs, l.ff, u.N, stream, GATE_SILU))
                        return -1;
                    StackGemmParams dn;
                    dn.dtype = s->dtype;
                    dn.out_f32 = 1;
                    dn.M = T;
                    dn.N = Wd;
                    dn.K = l.ff;
                    dn.a = s->act;
                    dn.lda = l.ff;
                    dn.w = l.w_down;
                    dn.c = s->moe_y;
                    dn.ldc = Wd;
                    dn.batch = l.experts;
                    dn.stride_w = (int64_t) Wd * l.ff;
                    dn.group_off = mp.group_off;
                    dn.group_rows = u.group_rows;
                    if (launch_stack_gemm(dn, stream) || launch_stack_moe_combine(mp, s->moe_y, s->y32, stream))
                        return -1;
                    pending = &l.hc[1];
                    if (s->taps && hyper(nullptr, nullptr, nullptr, s->tap + ri * (size_t) T * Wd))
                        return -1;
                    continue;
                }
                if (l.mlp == MLP_RELU2)
                {
                    u.N = l.ff;
                    u.c = s->act;
                    u.ldc = l.ff;
                    u.act = ACT_RELU2;
                    if (launch_stack_gemm(u, stream))
                        return -1;
                }
                else
                {
                    u.N = 2 * l.ff;
                    u.c = s->proj;
                    u.ldc = u.N;
                    if (launch_stack_gemm(u, stream) || launch_stack_gelu_gate(s->act, s->proj, s->dtype, T, l.ff, u.N, stream))
                        return -1;
                }
                StackGemmParams dn;
                dn.dtype = s->dtype;
                dn.out_f32 = 1;
                dn.M = T;
                dn.N = Wd;
                dn.K = l.ff;
                dn.a = act;
                dn.lda = l.ff;
                dn.w = l.w_down;
                dn.c = s->y32;
                dn.ldc = Wd;
                if (launch_stack_gemm(dn, stream))
                    return -1;
                pending = &l.hc[1];
            }
            if (s->taps && hyper(nullptr, nullptr, nullptr, s->tap + ri * (size_t) T * Wd))
                return -1;
            continue;
        }
        if (r.enters_pass
            && launch_stack_pass_entry(s->x, r.pass > 0 ? s->x0 : nullptr, s->loop_step + (size_t) r.pass * Wd, T, Wd, stream))
            return -1;
        if (launch_stack_group_rmsnorm(s->h1, l.ff > 0 ? s->h2 : nullptr, s->x, nullptr, l.norm1, l.norm2, s->dtype, T, Wd, s->groups, s->eps,
                stream))
            return -1;
        if (run_mixer(l, r))
            return -1;
        // x += sigmoid(P1[rg1] + b1) * (ctx Wo^T)
        StackGemmParams o;
        o.dtype = s->dtype;
        o.M = T;
        o.N = Wd;
        o.K = l.n_ctx;
        o.a = s->ctx;
        o.lda = l.n_ctx;
        o.w = l.w_o;
        o.resid = s->x;
        o.ldr = Wd;
        o.gate = (const char*) s->proj + (size_t) (l.n_q + l.n_k + l.n_v) * s->es;
        o.ldg = l.n_mix;
        o.gate_bias = l.rg1_b;
        if (launch_stack_gemm(o, stream))
            return -1;
        if (l.ff > 0)
        {
            // the feed-forward reads the same x as the mixer (h2 was normed before the mixer's update landed); P1's columns are
            // consumed once the mixer and the O product have run, so P2 may take their place
            StackGemmParams u;
            u.dtype = s->dtype;
            u.M = T;
            u.K = Wd;
            u.a = s->h2;
            u.lda = Wd;
            u.w = l.w_gu;
            u.c = s->proj;
            const int n_act = l.mlp == MLP_RELU2 ? l.ff : 2 * l.ff; // columns ahead of the residual gate's
            u.N = n_act + Wd;
            u.ldc = u.N;
            if (launch_stack_gemm(u, stream))
                return -1;
            if (launch_stack_gelu_gate(s->act, s->proj, s->dtype, T, l.ff, u.N, stream))
                return -1;
            StackGemmParams dn;
            dn.dtype = s->dtype;
            dn.M = T;
            dn.N = Wd;
            dn.K = l.ff;
            dn.a = s->act;
            dn.lda = l.ff;
            dn.w = l.w_down;
            dn.resid = s->x;
            dn.ldr = Wd;
            dn.gate = (const char*) s->proj + (size_t) n_act * s->es;
            dn.ldg = u.N;
            dn.gate_bias = l.rg2_b;
            if (launch_stack_gemm(dn, stream))
                return -1;
        }
        if (s->taps)
            HIP_OK(hipMemcpyAsync(s->tap + ri * (size_t) T * Wd, s->x, (size_t) T * Wd * 4, hipMemcpyDeviceToDevice, stream));
    }
    if (NW > 0)
    {
        if (s->hyper)
        {
            // the output norm reads the sum of the streams; the last sublayer lands in the same launch, on the wanted rows only
            StackHyperParams hp;
            hp.dtype = s->dtype;
            hp.tokens = NW;
            hp.width = Wd;
            hp.streams = s->streams;
            hp.x = s->x;
            hp.stream_stride = stream_stride;
            if (pending)
            {
                hp.y = s->y32;
                hp.mix = pending->mix;
                hp.out = pending->out;
            }
            hp.h = s->hw;
            hp.w = s->final_norm;
            hp.eps = s->eps;
            hp.rows = d_want;
            if (launch_stack_hyper_norm(hp, stream))
                return -1;
        }
        else if (launch_stack_group_rmsnorm(s->hw, nullptr, s->x, d_want, s->final_norm, nullptr, s->dtype, NW, Wd, s->groups, s->eps, stream))
            return -1;
        StackGemmParams hd;
        hd.dtype = s->dtype;
        hd.out_f32 = 1;
        hd.M = NW;
        hd.N = s->vocab;
        hd.K = Wd;
        hd.a = s->hw;
        hd.lda = Wd;
        hd.w = s->head;
        hd.c = s->logits;
        hd.ldc = s->vocab;
        if (launch_stack_gemm(hd, stream))
            return -1;
        if (next_ids_out && launch_argmax(s->ids_out, s->logits, NW, s->vocab, stream))
            return -1;
        if (logits_out)
            HIP_OK(hipMemcpyAsync(logits_out, s->logits, (size_t) NW * s->vocab * 4, hipMemcpyDeviceToHost, stream));
        if (next_ids_out)
            HIP_OK(hipMemcpyAsync(next_ids_out, s->ids_out, (size_t) NW * 4, hipMemcpyDeviceToHost, stream));
    }
    HIP_OK(hipStreamSynchronize(stream));
    return 0;
}

int32_t tllm_stack_page_size(tllm_stack_t s)
{
    return s ? s->page : 0;
}
int32_t tllm_stack_num_blocks(tllm_stack_t s)
{
    return s ? s->blocks : 0;
}
int32_t tllm_stack_num_slots(tllm_stack_t s)
{
    return s ? s->slots : 0;
}
int32_t tllm_stack_vocab(tllm_stack_t s)
{
    return s ? s->vocab : 0;
}
int32_t tllm_stack_layer_runs(tllm_stack_t s)
{
    return s ? (int32_t) s->runs.size() : 0;
}
int64_t tllm_stack_weight_bytes(tllm_stack_t s)
{
    return s ? s->weight_bytes : 0;
}

int64_t tllm_stack_step_bytes(tllm_stack_t s, int32_t n_tokens, int64_t context_tokens, int32_t n_entries)
{
    if (!s)
        return 0;
    // weights once (a looped layer's weights once per pass), keys and values of the contexts once per attention run, states read and
    // written once per recurrent run, the embedding rows instead of the whole table
    int64_t bytes = (int64_t) s->vocab * s->width * s->es + (int64_t) n_tokens * s->width * s->es;
    for (const Run& r : s->runs)
    {
        const Layer& l = s->layers[r.layer];
        int64_t ff_rows = l.ff > 0 ? (l.mlp == MLP_RELU2 ? 2 : 3) * (int64_t) l.ff + l.n_rg : 0;
        if (l.ff > 0 && l.mlp == MLP_MOE)
        {
            // the experts that the step's tokens can reach at most, and the fp32 router
            ff_rows *= std::min<int64_t>(l.experts, (int64_t) n_tokens * l.top);
            bytes += (int64_t) (l.experts + l.identity) * s->width * 4;
        }
        bytes += ((int64_t) l.n_mix + l.n_ctx + ff_rows) * s->width * s->es;
        if (l.kind == MIX_LATENT && l.q_rank > 0)
            bytes += (int64_t) l.heads * (l.dim + l.rot_part) * l.q_rank * s->es;
        if (l.kind == MIX_LATENT)
        {
            // the two per-head expansions, and per context token the key row [latent | rotated part] and the latent again as value
            bytes += (int64_t) l.heads * l.kv_rank * (l.dim + l.vdim) * s->es;
            const int64_t ctx = l.mask == MASK_CAUSAL ? context_tokens : std::min<int64_t>(context_tokens, (int64_t) n_entries * l.mask_size);
            bytes += ctx * (2 * (int64_t) l.kv_rank + l.rot_part) * s->es;
        }
        else if (l.kind == MIX_ATTENTION)
        {
            // a window or a chunk bounds what a row reads of its context
            const int64_t ctx = l.mask == MASK_CAUSAL ? context_tokens : std::min<int64_t>(context_tokens, (int64_t) n_entries * l.mask_size);
            bytes += ctx * ((int64_t) l.n_k + l.n_v) * s->es;
        }
        else if (l.kind == MIX_DELTA)
            bytes += ((int64_t) l.heads * l.dim * l.decay_rank + (int64_t) l.n_ctx * l.gate_rank) * s->es
                + 2 * (int64_t) n_entries * ((int64_t) l.heads * l.dim * l.vdim + (int64_t) (l.taps - 1) * l.n_conv) * 4;
        else if (l.kind == MIX_MAMBA2)
            bytes += 2 * (int64_t) n_entries * ((int64_t) l.heads * l.dim * l.vdim + (int64_t) (l.taps - 1) * l.n_conv) * 4;
        else
            bytes += 2 * (int64_t) n_entries * l.heads * l.dim * l.vdim * 4;
    }
    return bytes;
}

int32_t tllm_stack_get_tap(tllm_stack_t s, int32_t run, float* out, size_t n_floats)
{
    if (!s || !s->taps || !s->tap || run < 0 || run >= (int) s->runs.size() || n_floats != (size_t) s->tap_tokens * s->width)
    {
        set_error("tllm_stack_get_tap: taps are off (debug_taps=1), or run / size do not fit the last step");
        return -1;
    }
    HIP_OK(hipMemcpy(out, s->tap + (size_t) run * s->tap_tokens * s->width, n_floats * 4, hipMemcpyDeviceToHost));
    return 0;
}

void tllm_stack_destroy(tllm_stack_t s)
{
    delete s;
}

} // extern "C"
