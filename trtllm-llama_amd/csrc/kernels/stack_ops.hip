// Pointwise, rotary / cache-append, general attention and HGRN2 kernels of the ragged-batch stack engine (stack_kernels.h).
// Everything that a norm, a softmax, a recurrence or the residual stream touches is fp32; `DT` is the storage type of
// activations, weights and caches (bfloat16 or fp32).
#include "dev_utils.h"
#include "stack_kernels.h"
#include <algorithm>
#include <cmath>
#include <vector>

namespace tllm
{
namespace kernels
{
using namespace dev;

namespace
{

template <int DT>
struct El;
template <>
struct El<DT_FLOAT>
{
    typedef float type;
    static __device__ __forceinline__ float ld(const void* p, int64_t i)
    {
        return reinterpret_cast<const float*>(p)[i];
    }
    static __device__ __forceinline__ void st(void* p, int64_t i, float v)
    {
        reinterpret_cast<float*>(p)[i] = v;
    }
};
template <>
struct El<DT_BF16>
{
    typedef uint16_t type;
    static __device__ __forceinline__ float ld(const void* p, int64_t i)
    {
        return bf2f(reinterpret_cast<const uint16_t*>(p)[i]);
    }
    static __device__ __forceinline__ void st(void* p, int64_t i, float v)
    {
        reinterpret_cast<uint16_t*>(p)[i] = f2bf(v);
    }
};

inline int launched(const char* what)
{
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess)
    {
        set_error("%s launch failed: %s", what, hipGetErrorString(e));
        return -1;
    }
    return 0;
}

inline bool known_dtype(int32_t dt, const char* what)
{
    if (dt == DT_BF16 || dt == DT_FLOAT)
        return true;
    set_error("%s: element type %d is not served (bfloat16 or float32)", what, dt);
    return false;
}

// ------------------------------------------------------------------------------------------------------------ pointwise
template <int DT>
__global__ __launch_bounds__(256) void embed_kernel(float* x, float* keep, const int32_t* ids, const void* table, int width, int vocab,
    float scale, int copies, int64_t copy_stride)
{
    const int t = blockIdx.x;
    int id = ids[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    for (int c = threadIdx.x; c < width; c += blockDim.x)
    {
        const float v = El<DT>::ld(table, (int64_t) id * width + c) * scale;
        for (int k = 0; k < copies; ++k)
            x[k * copy_stride + (int64_t) t * width + c] = v;
        if (keep)
            keep[(int64_t) t * width + c] = v;
    }
}

// x[t, :] += pair_table[row, :]: the row is a hash of (previous token, token), or the table's extra last row for a first token
template <int DT>
__global__ __launch_bounds__(256) void pair_embed_kernel(float* x, const int32_t* ids, const int32_t* prev, const void* table, int width,
    int buckets, int mul_prev, int mul_cur, int copies, int64_t copy_stride)
{
    const int t = blockIdx.x;
    const int pv = prev[t];
    int64_t row = buckets;
    if (pv >= 0)
        row = ((int64_t) pv * mul_prev + (int64_t) ids[t] * mul_cur) % buckets;
    for (int c = threadIdx.x; c < width; c += blockDim.x)
    {
        const float v = El<DT>::ld(table, row * width + c);
        for (int k = 0; k < copies; ++k)
            x[k * copy_stride + (int64_t) t * width + c] += v;
    }
}

// Token shift.  Workgroups [0, tokens): rows behind their entry's first read the step's own rows.  Workgroups [tokens, tokens +
// entries): an entry's first row, which reads the sequence's carried row, and the new carry - one thread per (entry, channel) reads
// the old carry before it writes, so the launch has no ordering between workgroups to keep.
template <int DT>
__global__ __launch_bounds__(256) void token_shift_kernel(const StackShiftParams p)
{
    const int W = p.width;
    if ((int) blockIdx.x < p.tokens)
    {
        const int t = blockIdx.x, e = p.tok_entry[t];
        if (p.tok_pos[t] == p.ent_pos0[e])
            return;
        for (int c = blockIdx.y * 256 + threadIdx.x; c < W; c += gridDim.y * 256)
        {
            const float a = p.n[(int64_t) t * W + c], b = p.n[(int64_t) (t - 1) * W + c];
            El<DT>::st(p.h, (int64_t) t * W + c, a + (b - a) * p.mu[c]);
        }
        return;
    }
    const int e = blockIdx.x - p.tokens;
    const int first = p.ent_first[e], last = first + p.ent_count[e] - 1;
    float* carry = p.carry + (int64_t) p.ent_slot[e] * W;
    const bool fresh = p.ent_pos0[e] == 0;
    for (int c = blockIdx.y * 256 + threadIdx.x; c < W; c += gridDim.y * 256)
    {
        const float b = fresh ? 0.f : carry[c];
        const float a = p.n[(int64_t) first * W + c];
        El<DT>::st(p.h, (int64_t) first * W + c, a + (b - a) * p.mu[c]);
        carry[c] = p.n[(int64_t) last * W + c];
    }
}

// Hyper-connected residual streams: one workgroup per row; the combined row u stays in LDS between the sum of squares and the
// scaling, the streams are read and written once.
constexpr int HY_T = 256, HY_MAXS = 8;

template <int DT>
__global__ __launch_bounds__(HY_T) void hyper_norm_kernel(const StackHyperParams p)
{
    extern __shared__ float u_s[]; // [width]
    __shared__ float red[32];
    __shared__ float cm[HY_MAXS * HY_MAXS], co[HY_MAXS], ci[HY_MAXS];
    const int t = p.rows ? p.rows[blockIdx.x] : blockIdx.x, tid = threadIdx.x, S = p.streams;
    if (tid < S * S)
        cm[tid] = p.y ? p.mix[tid] : 0.f;
    if (tid < S)
    {
        co[tid] = p.y ? p.out[tid] : 0.f;
        ci[tid] = p.in ? p.in[tid] : 1.f;
    }
    __syncthreads();
    float ss = 0.f;
    for (int c = tid; c < p.width; c += HY_T)
    {
        const int64_t o = (int64_t) t * p.width + c;
        float xs[HY_MAXS], u = 0.f;
#pragma unroll
        for (int s = 0; s < HY_MAXS; ++s)
            xs[s] = s < S ? p.x[s * p.stream_stride + o] : 0.f;
        if (p.y)
        {
            const float y = p.y[o];
#pragma unroll
            for (int to = 0; to < HY_MAXS; ++to)
            {
                if (to < S)
                {
                    float a = 0.f;
#pragma unroll
                    for (int s = 0; s < HY_MAXS; ++s)
                        if (s < S)
                            a = fmaf(cm[s * S + to], xs[s], a);
                    a = fmaf(co[to], y, a);
                    if (!p.rows) // a gathered launch is the streams' last reader (and a row may be asked for twice): nothing is written back
                        p.x[to * p.stream_stride + o] = a;
                    u = fmaf(ci[to], a, u);
                }
            }
        }
        else
        {
#pragma unroll
            for (int s = 0; s < HY_MAXS; ++s)
                if (s < S)
                    u = fmaf(ci[s], xs[s], u);
        }
        if (p.sum_out)
            p.sum_out[o] = u;
        u_s[c] = u;
        ss += u * u;
    }
    if (!p.h && !p.h32)
        return;
    ss = block_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float) p.width + p.eps);
    for (int c = tid; c < p.width; c += HY_T)
    {
        const float v = u_s[c] * inv * p.w[c];
        if (p.h)
            El<DT>::st(p.h, (int64_t) blockIdx.x * p.width + c, v);
        if (p.h32)
            p.h32[(int64_t) blockIdx.x * p.width + c] = v;
    }
}

__global__ __launch_bounds__(256) void pass_entry_kernel(float* x, const float* add, const float* row, int64_t n, int width)
{
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n)
        return;
    float v = x[i];
    if (add)
        v += add[i];
    if (row)
        v += row[i % width];
    x[i] = v;
}

// one workgroup per (row, group): the group's elements stay in registers between the sum of squares and the scaling
constexpr int GN_T = 256, GN_EPT = 8;

template <int DT>
__global__ __launch_bounds__(GN_T) void group_rmsnorm_kernel(void* y1, void* y2, const float* x, const int32_t* rows, const float* w1,
    const float* w2, int width, int groups, float eps)
{
    __shared__ float red[32];
    const int r = blockIdx.x, g = blockIdx.y, tid = threadIdx.x;
    const int gs = width / groups;
    const float* xg = x + (int64_t) (rows ? rows[r] : r) * width + g * gs;
    float v[GN_EPT], ss = 0.f;
#pragma unroll
    for (int k = 0; k < GN_EPT; ++k)
    {
        const int i = tid + k * GN_T;
        v[k] = i < gs ? xg[i] : 0.f;
        ss += v[k] * v[k];
    }
    for (int i = tid + GN_EPT * GN_T; i < gs; i += GN_T) // groups beyond GN_T * GN_EPT elements: the tail is read twice
        ss += xg[i] * xg[i];
    ss = block_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float) gs + eps);
#pragma unroll
    for (int k = 0; k < GN_EPT; ++k)
    {
        const int i = tid + k * GN_T;
        if (i < gs)
        {
            const int c = g * gs + i;
            const float n = v[k] * inv;
            El<DT>::st(y1, (int64_t) r * width + c, n * w1[c]);
            if (y2)
                El<DT>::st(y2, (int64_t) r * width + c, n * w2[c]);
        }
    }
    for (int i = tid + GN_EPT * GN_T; i < gs; i += GN_T)
    {
        const int c = g * gs + i;
        const float n = xg[i] * inv;
        El<DT>::st(y1, (int64_t) r * width + c, n * w1[c]);
        if (y2)
            El<DT>::st(y2, (int64_t) r * width + c, n * w2[c]);
    }
}

__device__ __forceinline__ float gelu_tanh(float z)
{
    return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <int DT>
__global__ __launch_bounds__(256) void gelu_gate_kernel(void* y, const void* gu, int tokens, int ff, int64_t ld, int act)
{
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t) tokens * ff)
        return;
    const int t = (int) (i / ff), c = (int) (i % ff);
    const float g = El<DT>::ld(gu, (int64_t) t * ld + c), u = El<DT>::ld(gu, (int64_t) t * ld + ff + c);
    float a = act == GATE_SILU ? g / (1.f + expf(-g)) : gelu_tanh(g);
    if (DT == DT_BF16)
        a = bf2f(f2bf(a)); // the activation is a bfloat16 value before it meets the other branch
    El<DT>::st(y, i, a * u);
}

// one wave per row: y = x / sqrt(mean(x^2) + eps) * w over n elements of the element type, rows with their own strides
template <int DT>
__global__ __launch_bounds__(256) void row_rmsnorm_kernel(void* y, int64_t ldy, const void* x, int64_t ldx, const float* w, int rows, int n,
    float eps)
{
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (r >= rows)
        return;
    float ss = 0.f;
    for (int c = lane; c < n; c += 64)
    {
        const float v = El<DT>::ld(x, (int64_t) r * ldx + c);
        ss += v * v;
    }
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float) n + eps);
    for (int c = lane; c < n; c += 64)
        El<DT>::st(y, (int64_t) r * ldy + c, El<DT>::ld(x, (int64_t) r * ldx + c) * inv * w[c]);
}

// --------------------------------------------------------------------------------------------------- rotary + cache append
template <int DT>
__global__ __launch_bounds__(256) void rope_kv_kernel(const StackAttnParams p)
{
    const int t = blockIdx.x;
    const int e = p.tok_entry[t], pos = p.tok_pos[t];
    const int blk = p.block_table[(int64_t) e * p.max_blocks + pos / p.page], off = pos % p.page;
    const int D = p.dim, nq = p.heads * p.maps * D, nk = p.kv_heads * p.maps * D, nv = p.kv_heads * p.vdim;
    const int64_t row = (int64_t) t * p.ldp;
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < nq + nk; i += gridDim.y * blockDim.x)
    {
        const int d = i % D;
        float v = El<DT>::ld(p.proj, row + i);
        if (d < p.rot_dims)
        {
            const float other = El<DT>::ld(p.proj, row + (i ^ 1)); // pairs (2i, 2i + 1): D is even, so is every map's start
            const float a = (float) pos * p.freq[d >> 1];
            float sn, cs;
            sincosf(a, &sn, &cs);
            sn *= p.mscale;
            cs *= p.mscale;
            v = (d & 1) ? v * cs + other * sn : v * cs - other * sn;
        }
        if (i < nq)
            El<DT>::st(p.q, (int64_t) t * nq + i, v);
        else
        {
            const int j = i - nq, gm = j / D; // gm = kv head * maps + map
            El<DT>::st(p.k_pool, (((int64_t) blk * (p.kv_heads * p.maps) + gm) * p.page + off) * D + d, v);
        }
    }
    const int v_col = p.values_are_keys ? nq : nq + nk; // a layer without a value projection keeps its keys as projected
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < nv; i += gridDim.y * blockDim.x)
    {
        const int g = i / p.vdim, c = i % p.vdim;
        El<DT>::st(p.v_pool, (((int64_t) blk * p.kv_heads + g) * p.vdim + c) * p.page + off, El<DT>::ld(p.proj, row + v_col + i));
    }
}

// The general form of the step before attention: one wave per (row, vector), a vector being one map of one query head, one map of
// one key head, or one value head.  Projection bias, unit RMS of q and k over dim (fp32), rotation of neighbouring pairs (the
// partner sits in the neighbouring lane), then the store into the query scratch or the page.  dim, vdim <= 64 * PREP_EPL.
constexpr int PREP_EPL = 8;

template <int DT>
__global__ __launch_bounds__(256) void attn_prep_kernel(const StackAttnParams p)
{
    const int t = blockIdx.x, lane = threadIdx.x & 63;
    const int vec = blockIdx.y * 4 + (threadIdx.x >> 6);
    const int D = p.dim, nqv = p.heads * p.maps, nkv = p.kv_heads * p.maps;
    if (vec >= nqv + nkv + p.kv_heads)
        return;
    const int e = p.tok_entry[t], pos = p.tok_pos[t];
    const int blk = p.block_table[(int64_t) e * p.max_blocks + pos / p.page], off = pos % p.page;
    const int64_t row = (int64_t) t * p.ldp;
    if (vec >= nqv + nkv)
    {
        const int g = vec - nqv - nkv, col0 = (p.values_are_keys ? nqv : nqv + nkv) * D + g * p.vdim;
        for (int c = lane; c < p.vdim; c += 64)
        {
            float v = El<DT>::ld(p.proj, row + col0 + c);
            if (p.bias)
                v += p.bias[col0 + c];
            El<DT>::st(p.v_pool, (((int64_t) blk * p.kv_heads + g) * p.vdim + c) * p.page + off, v);
        }
        return;
    }
    const int col0 = vec * D;
    float v[PREP_EPL], ss = 0.f;
#pragma unroll
    for (int k = 0; k < PREP_EPL; ++k)
    {
        const int d = lane + 64 * k;
        v[k] = 0.f;
        if (d < D)
        {
            v[k] = El<DT>::ld(p.proj, row + col0 + d);
            if (p.bias)
                v[k] += p.bias[col0 + d];
            if (DT == DT_BF16 && p.bias)
                v[k] = bf2f(f2bf(v[k])); // the biased projection is a value of the element type
        }
        ss += v[k] * v[k];
    }
    float inv = 1.f;
    if (p.qk_unit_norm)
        inv = 1.f / sqrtf(wave_sum(ss) / (float) D + p.eps);
    const float* nw = p.qk_unit_norm ? (vec < nqv ? p.q_norm_w : p.k_norm_w) : nullptr;
#pragma unroll
    for (int k = 0; k < PREP_EPL; ++k)
    {
        const int d = lane + 64 * k;
        float x = v[k] * inv;
        if (nw && d < D)
            x *= nw[d];
        const float other = __shfl_xor(x, 1, 64); // pairs (2i, 2i + 1): lane parity = dimension parity
        if (d < p.rot_dims)
        {
            float sn, cs;
            sincosf((float) pos * p.freq[d >> 1], &sn, &cs);
            sn *= p.mscale;
            cs *= p.mscale;
            x = (d & 1) ? x * cs + other * sn : x * cs - other * sn;
        }
        if (d < D)
        {
            if (vec < nqv)
                El<DT>::st(p.q, (int64_t) t * nqv * D + col0 + d, x);
            else
                El<DT>::st(p.k_pool, (((int64_t) blk * nkv + (vec - nqv)) * p.page + off) * D + d, x);
        }
    }
}

// Latent attention, the pointwise part: per row the latent's RMS norm (plain weight) and the rotation of the shared key part into
// the page ([c | k_rot] as the key row, c channel-major as the value row), and the rotation of every head's rotated query part into
// the absorbed query [a | q_rot] (the `a` part is a product of its own).  One wave per (row, head) plus one per row for the latent.
template <int DT>
__global__ __launch_bounds__(256) void latent_prep_kernel(const StackAttnParams p, int qk_dim, const float* norm_w, const void* q_src,
    int64_t ldq, int dkv_col)
{
    const int t = blockIdx.x, lane = threadIdx.x & 63;
    const int vec = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (vec > p.heads)
        return;
    const int C = p.vdim, R = p.dim - C, pos = p.tok_pos[t]; // of the R dimensions of the rotated part the first rot_dims turn
    const int64_t row = (int64_t) t * p.ldp;
    const int half = p.rot_dims >> 1;
    // dimension d < rot_dims of a rotated part: its partner, its frequency, and whether it is the second of its pair
    auto turn = [&](const void* base, int64_t src, int d) -> float {
        float x = El<DT>::ld(base, src + d);
        if (d < p.rot_dims)
        {
            const int partner = p.rot_halves ? (d < half ? d + half : d - half) : (d ^ 1);
            const int fi = p.rot_halves ? (d < half ? d : d - half) : (d >> 1);
            const bool second = p.rot_halves ? d >= half : (d & 1);
            const float other = El<DT>::ld(base, src + partner);
            float sn, cs;
            sincosf((float) pos * p.freq[fi], &sn, &cs);
            sn *= p.mscale;
            cs *= p.mscale;
            x = second ? x * cs + other * sn : x * cs - other * sn;
        }
        return x;
    };
    if (vec < p.heads)
    {
        const int64_t src = (int64_t) t * ldq + (int64_t) vec * (qk_dim + R) + qk_dim;
        for (int d = lane; d < R; d += 64)
            El<DT>::st(p.q, ((int64_t) t * p.heads + vec) * p.dim + C + d, turn(q_src, src, d));
        return;
    }
    const int e = p.tok_entry[t];
    const int blk = p.block_table[(int64_t) e * p.max_blocks + pos / p.page], off = pos % p.page;
    const int64_t src = row + dkv_col;
    float ss = 0.f;
    for (int c = lane; c < C; c += 64)
    {
        const float x = El<DT>::ld(p.proj, src + c);
        ss += x * x;
    }
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float) C + p.eps);
    const int64_t krow = ((int64_t) blk * p.page + off) * p.dim;
    for (int c = lane; c < C; c += 64)
    {
        const float x = El<DT>::ld(p.proj, src + c) * inv * norm_w[c];
        El<DT>::st(p.k_pool, krow + c, x);
        El<DT>::st(p.v_pool, ((int64_t) blk * C + c) * p.page + off, x);
    }
    for (int d = lane; d < R; d += 64)
        El<DT>::st(p.k_pool, krow + C + d, turn(p.proj, src + C, d));
}

// ------------------------------------------------------------------------------------------------ attention, general form
// One workgroup per (row, head): scores of 128 keys at a time by one thread per key, online softmax per map, P V by one thread
// per value channel.  Any dim / vdim <= 512, both element types; the tiled kernels of stack_attn.hip take the shapes they serve.
constexpr int AT = 128, A_CPT = 4;

template <int DT, int MAPS>
__global__ __launch_bounds__(AT) void attn_general_kernel(const StackAttnParams p)
{
    extern __shared__ float sm[];
    float* qs = sm;                      // [MAPS][dim]
    float* ps = qs + MAPS * p.dim;       // [MAPS][AT]
    float* red = ps + MAPS * AT;         // [32]
    __shared__ int blk_of[AT];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int e = p.tok_entry[t], pos = p.tok_pos[t];
    const int g = h / (p.heads / p.kv_heads), D = p.dim, V = p.vdim;
    const int32_t* table = p.block_table + (int64_t) e * p.max_blocks;
    for (int i = tid; i < MAPS * D; i += AT)
        qs[i] = El<DT>::ld(p.q, ((int64_t) t * p.heads + h) * MAPS * D + i);
    float m_run[MAPS], l_run[MAPS], acc[MAPS][A_CPT];
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
    {
        m_run[m] = -INFINITY;
        l_run[m] = 0.f;
#pragma unroll
        for (int c = 0; c < A_CPT; ++c)
            acc[m][c] = 0.f;
    }
    __syncthreads();
    const int nkeys = pos + 1;
    // the first key the mask lets this row see: a window's lower edge, the start of the row's chunk
    int k_lo = 0;
    if (p.mask == MASK_WINDOW)
        k_lo = pos - p.mask_size + 1 > 0 ? pos - p.mask_size + 1 : 0;
    else if (p.mask == MASK_CHUNK)
        k_lo = pos / p.mask_size * p.mask_size;
    const float temp = p.temp ? p.temp[h] : 1.f, slope = p.slope ? p.slope[h] : 0.f;
    const float r1 = p.log_r1 ? p.log_r1[h] : 0.f, r2 = p.log_r1 ? p.log_r2[h] : 0.f;
    const bool sigm = p.weights == WEIGHTS_SIGMOID;
    const float wb = sigm && p.wbias ? p.wbias[h] : 0.f;
    // kept first keys that lie before the window: a segment of their own ahead of the window's
    const int keep_hi = (p.mask == MASK_WINDOW && p.mask_keep > 0) ? (p.mask_keep < k_lo ? p.mask_keep : k_lo) : 0;
    for (int seg = keep_hi > 0 ? 0 : 1; seg < 2; ++seg)
    for (int k0 = seg ? k_lo : 0, nkeys = seg ? pos + 1 : keep_hi; k0 < nkeys; k0 += AT)
    {
        const int kj = k0 + tid;
        float s[MAPS];
        int blk = 0;
        if (kj < nkeys)
        {
            blk = table[kj / p.page];
            const int off = kj % p.page;
#pragma unroll
            for (int m = 0; m < MAPS; ++m)
            {
                const int64_t kb = (((int64_t) blk * (p.kv_heads * MAPS) + g * MAPS + m) * p.page + off) * D;
                float a = 0.f;
                for (int d = 0; d < D; ++d)
                    a += qs[m * D + d] * El<DT>::ld(p.k_pool, kb + d);
                a *= p.scale;
                if (p.softcap > 0.f)
                    a = p.softcap * tanhf(a / p.softcap);
                a *= temp;
                const float dist = (float) (pos - kj);
                a -= slope * dist;
                if (p.log_r1)
                    a -= r1 * logf(1.f + r2 * dist);
                s[m] = a;
            }
        }
        else
        {
#pragma unroll
            for (int m = 0; m < MAPS; ++m)
                s[m] = -INFINITY;
        }
        blk_of[tid] = blk;
        float corr[MAPS];
#pragma unroll
        for (int m = 0; m < MAPS; ++m)
        {
            if (sigm)
            {
                // every key's weight stands alone: no running maximum, no denominator
                corr[m] = 1.f;
                ps[m * AT + tid] = kj < nkeys ? 1.f / (1.f + expf(-(s[m] + wb))) : 0.f;
                continue;
            }
            const float bm = block_max(s[m], red);
            const float mn = fmaxf(m_run[m], bm);
            corr[m] = expf(m_run[m] - mn); // 0 at the first block
            const float pj = kj < nkeys ? expf(s[m] - mn) : 0.f;
            ps[m * AT + tid] = pj;
            const float bs = block_sum(pj, red);
            l_run[m] = l_run[m] * corr[m] + bs;
            m_run[m] = mn;
        }
        __syncthreads();
        const int nb = nkeys - k0 < AT ? nkeys - k0 : AT;
#pragma unroll
        for (int c = 0; c < A_CPT; ++c)
        {
            const int ch = tid + c * AT;
            if (ch >= V)
                break;
            float a[MAPS];
#pragma unroll
            for (int m = 0; m < MAPS; ++m)
                a[m] = acc[m][c] * corr[m];
            for (int j = 0; j < nb; ++j)
            {
                const float v = El<DT>::ld(p.v_pool, (((int64_t) blk_of[j] * p.kv_heads + g) * V + ch) * p.page + (k0 + j) % p.page);
#pragma unroll
                for (int m = 0; m < MAPS; ++m)
                    a[m] += ps[m * AT + j] * v;
            }
#pragma unroll
            for (int m = 0; m < MAPS; ++m)
                acc[m][c] = a[m];
        }
        __syncthreads();
    }
    float fin[MAPS]; // what turns a map's accumulator into its output
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
    {
        if (sigm)
            fin[m] = 1.f;
        else if (p.sink)
        {
            // the sink joins the denominator like one more key with this logit, and brings no value
            const float sk = p.sink[h], mf = fmaxf(m_run[m], sk);
            const float w_keys = expf(m_run[m] - mf);
            fin[m] = w_keys / (l_run[m] * w_keys + expf(sk - mf));
        }
        else
            fin[m] = 1.f / l_run[m];
    }
    float og = 1.f;
    if (p.out_gate && !p.gate_wide)
        og = 1.f / (1.f + expf(-El<DT>::ld(p.out_gate, (int64_t) t * p.ld_gate + h)));
    float o[A_CPT], ss = 0.f;
#pragma unroll
    for (int c = 0; c < A_CPT; ++c)
    {
        o[c] = 0.f;
        if (tid + c * AT < V)
        {
            o[c] = acc[0][c] * fin[0];
            if (MAPS == 2)
                o[c] -= p.lambda * (acc[MAPS - 1][c] * fin[MAPS - 1]);
            ss += o[c] * o[c];
        }
    }
    float mul = 1.f;
    if (p.head_norm)
    {
        ss = block_sum(ss, red);
        mul = p.out_scale / sqrtf(ss / (float) V + p.eps);
    }
#pragma unroll
    for (int c = 0; c < A_CPT; ++c)
        if (tid + c * AT < V)
        {
            if (p.out_gate && p.gate_wide)
                og = 1.f / (1.f + expf(-El<DT>::ld(p.out_gate, (int64_t) t * p.ld_gate + (int64_t) h * V + tid + c * AT)));
            El<DT>::st(p.out, ((int64_t) t * p.heads + h) * V + tid + c * AT, o[c] * mul * og);
        }
}

// Talking heads from their terms (see launch_stack_talk_combine): one workgroup per row, the mixing matrix in LDS, one thread per
// output channel of the row.
template <int DT>
__global__ __launch_bounds__(256) void talk_combine_kernel(const StackAttnParams p, const void* pairs)
{
    extern __shared__ float tk_s[]; // [H][H]
    const int H = p.heads, G = p.kv_heads, V = p.vdim, per = H / G;
    const int64_t t = blockIdx.x;
    for (int i = threadIdx.x; i < H * H; i += 256)
        tk_s[i] = p.talk[i];
    __syncthreads();
    for (int oc = blockIdx.y * 256 + threadIdx.x; oc < H * V; oc += gridDim.y * 256)
    {
        const int h = oc / V, ch = oc % V, c = h / per;
        float a = 0.f;
        for (int g = 0; g < H; ++g)
            a = fmaf(tk_s[h * H + g], El<DT>::ld(pairs, (t * H * G + g * G + c) * V + ch), a);
        if (p.out_gate)
            a *= 1.f / (1.f + expf(-El<DT>::ld(p.out_gate, t * p.ld_gate + (p.gate_wide ? oc : h))));
        El<DT>::st(p.out, t * H * V + oc, a);
    }
}

// Talking heads, general form: one workgroup per row holds ALL heads, because a head's final weight on a key mixes every head's
// normalised weight on it.  Two passes over the visible keys, 128 at a time by one thread per key: the first leaves every head's
// running maximum and denominator (sink included); the second recomputes the scores, normalises, mixes w'_h = sum_g talk[h, g] w_g per
// key in the thread that owns it, and multiplies with the values of head h's own key/value head, one thread per output channel of
// the whole row (heads * vdim / TK_T of them per thread).  One map, softmax weights; any dim, heads * vdim <= TK_T * TK_CPT.
constexpr int TK_T = 256, TK_CPT = 32, TK_MAXH = 64;

template <int DT>
__global__ __launch_bounds__(TK_T) void attn_talk_kernel(const StackAttnParams p)
{
    extern __shared__ float sm[];
    const int H = p.heads, G = p.kv_heads, D = p.dim, V = p.vdim, per = H / G;
    float* qs = sm;                 // [H][D]
    float* ws = qs + H * D;         // [H][TK_T] normalised weights of the block's keys
    float* wm = ws + H * TK_T;      // [H][TK_T] the same, mixed across heads
    float* tk = wm + H * TK_T;      // [H][H]
    float* mh = tk + H * H;         // [H] running maxima
    float* lh = mh + H;             // [H] denominators
    float* red = lh + H;            // [32]
    __shared__ int blk_of[TK_T];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int e = p.tok_entry[t], pos = p.tok_pos[t];
    const int32_t* table = p.block_table + (int64_t) e * p.max_blocks;
    for (int i = tid; i < H * D; i += TK_T)
        qs[i] = El<DT>::ld(p.q, (int64_t) t * H * D + i);
    for (int i = tid; i < H * H; i += TK_T)
        tk[i] = p.talk ? p.talk[i] : ((i / H == i % H) ? 1.f : 0.f);
    for (int i = tid; i < H; i += TK_T)
    {
        mh[i] = -INFINITY;
        lh[i] = 0.f;
    }
    __syncthreads();
    int k_lo = 0;
    if (p.mask == MASK_WINDOW)
        k_lo = pos - p.mask_size + 1 > 0 ? pos - p.mask_size + 1 : 0;
    else if (p.mask == MASK_CHUNK)
        k_lo = pos / p.mask_size * p.mask_size;
    const int keep_hi = (p.mask == MASK_WINDOW && p.mask_keep > 0) ? (p.mask_keep < k_lo ? p.mask_keep : k_lo) : 0;
    float acc[TK_CPT];
#pragma unroll
    for (int c = 0; c < TK_CPT; ++c)
        acc[c] = 0.f;
    for (int pass = 0; pass < 2; ++pass)
    {
        if (pass == 1)
        {
            // every head's denominator takes its sink; from here lh holds 1 / denominator relative to mh
            __syncthreads();
            for (int h = tid; h < H; h += TK_T)
            {
                float m = mh[h], l = lh[h];
                if (p.sink)
                {
                    const float sk = p.sink[h], mf = fmaxf(m, sk);
                    l = l * expf(m - mf) + expf(sk - mf);
                    m = mf;
                }
                mh[h] = m;
                lh[h] = 1.f / l;
            }
            __syncthreads();
        }
        for (int seg = keep_hi > 0 ? 0 : 1; seg < 2; ++seg)
            for (int k0 = seg ? k_lo : 0, nkeys = seg ? pos + 1 : keep_hi; k0 < nkeys; k0 += TK_T)
            {
                const int kj = k0 + tid;
                const bool live = kj < nkeys;
                int blk = 0;
                if (live)
                    blk = table[kj / p.page];
                const int off = kj % p.page;
                blk_of[tid] = blk;
                for (int g = 0; g < G; ++g)
                {
                    // a key row is read once per key/value head and serves the query heads of its group
                    const int64_t kb = (((int64_t) blk * G + g) * p.page + off) * D;
                    for (int hh = 0; hh < per; ++hh)
                    {
                        const int h = g * per + hh;
                        float a = -INFINITY;
                        if (live)
                        {
                            a = 0.f;
                            for (int d = 0; d < D; ++d)
                                a += qs[h * D + d] * El<DT>::ld(p.k_pool, kb + d);
                            a *= p.scale;
                        }
                        if (pass == 0)
                        {
                            const float bm = block_max(a, red);
                            const float mo = mh[h], mn = fmaxf(mo, bm);
                            const float bs = block_sum(live ? expf(a - mn) : 0.f, red);
                            __syncthreads();
                            if (tid == 0)
                            {
                                lh[h] = lh[h] * expf(mo - mn) + bs;
                                mh[h] = mn;
                            }
                            __syncthreads();
                        }
                        else
                            ws[h * TK_T + tid] = live ? expf(a - mh[h]) * lh[h] : 0.f;
                    }
                }
                if (pass == 0)
                    continue;
                // mix across heads for this thread's key: its own column of ws, which it wrote itself, into wm
                for (int h = 0; h < H; ++h)
                {
                    float m = 0.f;
                    for (int g = 0; g < H; ++g)
                        m = fmaf(tk[h * H + g], ws[g * TK_T + tid], m);
                    wm[h * TK_T + tid] = m;
                }
                __syncthreads();
                const int nb = nkeys - k0 < TK_T ? nkeys - k0 : TK_T;
#pragma unroll
                for (int c = 0; c < TK_CPT; ++c)
                {
                    const int oc = tid + c * TK_T;
                    if (oc >= H * V)
                        break;
                    const int h = oc / V, ch = oc % V, g = h / per;
                    float a = acc[c];
                    for (int j = 0; j < nb; ++j)
                        a += wm[h * TK_T + j]
                            * El<DT>::ld(p.v_pool, (((int64_t) blk_of[j] * G + g) * V + ch) * p.page + (k0 + j) % p.page);
                    acc[c] = a;
                }
                __syncthreads();
            }
    }
#pragma unroll
    for (int c = 0; c < TK_CPT; ++c)
    {
        const int oc = tid + c * TK_T;
        if (oc >= H * V)
            break;
        float og = 1.f;
        if (p.out_gate)
            og = 1.f / (1.f + expf(-El<DT>::ld(p.out_gate, (int64_t) t * p.ld_gate + (p.gate_wide ? oc : oc / V))));
        El<DT>::st(p.out, (int64_t) t * H * V + oc, acc[c] * og);
    }
}

// ------------------------------------------------------------------------------------------------------------------ HGRN2
// One wave per (entry, head, 64 value channels): lane v keeps column S[:, v] in registers and walks the entry's rows in
// order; the row's q and forget gate are computed once per (row, channel of dim) by the lanes and shared through LDS, HC rows
// at a time.  No cross-lane traffic in the recurrence itself.
constexpr int HC = 8;

template <int DT, int DMAX>
__global__ __launch_bounds__(64) void hgrn2_scan_kernel(const StackHgrnParams p)
{
    __shared__ float qf[HC][2][DMAX];
    const int e = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int v = blockIdx.z * 64 + lane;
    const int D = p.dim, V = p.vdim, HD = p.heads * D;
    const int first = p.ent_first[e], count = p.ent_count[e];
    const bool live = v < V;
    float* sp = p.state + (((int64_t) p.ent_slot[e] * p.heads + h) * D) * V + v;
    float S[DMAX];
#pragma unroll
    for (int d = 0; d < DMAX; ++d)
        S[d] = (live && d < D && p.ent_pos0[e] > 0) ? sp[(int64_t) d * V] : 0.f;
    for (int t0 = 0; t0 < count; t0 += HC)
    {
        const int nt = count - t0 < HC ? count - t0 : HC;
        __syncthreads();
        for (int i = lane; i < nt * D; i += 64)
        {
            const int tt = i / D, d = i % D;
            const int64_t row = (int64_t) (first + t0 + tt) * p.ldp;
            float qr = El<DT>::ld(p.proj, row + h * D + d);
            qr = qr / (1.f + expf(-qr));
            if (DT == DT_BF16)
                qr = bf2f(f2bf(qr)); // the projection's activation is a bfloat16 value; everything behind it is fp32
            const float fr = El<DT>::ld(p.proj, row + HD + h * D + d) + p.f_bias[h * D + d];
            const float lo = p.lower[h * D + d];
            qf[tt][0][d] = qr;
            qf[tt][1][d] = lo + (1.f - lo) * (1.f / (1.f + expf(-fr)));
        }
        __syncthreads();
        if (live)
        {
            for (int tt = 0; tt < nt; ++tt)
            {
                const int64_t r = first + t0 + tt;
                const float vv = El<DT>::ld(p.proj, r * p.ldp + 2 * HD + h * V + v);
                float o = 0.f;
#pragma unroll
                for (int d = 0; d < DMAX; ++d)
                {
                    if (d < D)
                    {
                        const float f = qf[tt][1][d];
                        S[d] = f * S[d] + (1.f - f) * vv;
                        o += S[d] * qf[tt][0][d];
                    }
                }
                p.o32[r * (p.heads * V) + h * V + v] = o;
            }
        }
    }
    if (live)
    {
#pragma unroll
        for (int d = 0; d < DMAX; ++d)
            if (d < D)
                sp[(int64_t) d * V] = S[d];
    }
}

// The head-wide form: one workgroup per (entry, head) when the head's vdim channels fit (<= 256).  The state is spread over
// vpad x DS threads: thread (s, v) keeps the DSZ rows [s DSZ, (s + 1) DSZ) of column S[:, v] in registers (every wave has one s, so
// the row's gates and queries come out of LDS as broadcasts).  Rows go through in chunks of HTC: the chunk's gates and queries are
// computed once per (row, channel of dim), its raw projections having been requested while the chunk before it was in the
// recurrence; the recurrence itself has no cross-lane traffic, the DS partial outputs of a row meet in LDS once per chunk, and the
// per-head RMS norm of the outputs is taken in the same launch (no fp32 round trip of o, no second kernel).
// HTC rows per chunk (8; 16 measured the same: the time goes with the rows, not with the chunks), H_PPT (row, channel) pairs of gate /
// query work per thread and chunk: 4 where one workgroup of up to 1024 threads holds a head, DSZ / 2 in the 16-column groups of up to 256.

template <int DT, int DSZ, int HTC, int H_PPT, int MAXT>
__global__ __launch_bounds__(MAXT) void hgrn2_head_kernel(const StackHgrnParams p, int vpad, int DS, int fuse_norm)
{
    extern __shared__ float hsm[];
    const int D = p.dim, V = p.vdim, HD = p.heads * D, NT = blockDim.x;
    float2* fq = reinterpret_cast<float2*>(hsm);        // [HTC][D] {forget gate, query}
    float* vs = hsm + 2 * HTC * D;                      // [HTC][vpad]
    float* os = vs + HTC * vpad;                        // [HTC][DS][vpad]
    float* red = os + HTC * DS * vpad;                  // [HTC][vpad / 64]
    const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    // the workgroup's columns: [blockIdx.z * vpad, + vpad).  fuse_norm: one workgroup holds the whole head (vpad a multiple of 64, a
    // wave one slice) and norms it; otherwise a head is spread over several workgroups, o goes out in fp32 and a pass norms it
    const int s = tid / vpad, vl = tid % vpad, v = blockIdx.z * vpad + vl, lane = tid & 63, vw = vl >> 6, nvw = (vpad + 63) >> 6;
    const int first = p.ent_first[e], count = p.ent_count[e];
    const bool live = v < V;
    const int d0 = s * DSZ;
    float* sp = p.state + (((int64_t) p.ent_slot[e] * p.heads + h) * D) * V + v;
    const bool carry = p.ent_pos0[e] > 0;
    float S[DSZ];
#pragma unroll
    for (int j = 0; j < DSZ; ++j)
        S[j] = (live && d0 + j < D && carry) ? sp[(int64_t) (d0 + j) * V] : 0.f;
    const float nw = live ? p.norm_w[v] : 0.f;

    // raw projections of the next chunk (rq / rf / rv) and of the one behind it (nq / nf / nv): a chunk's loads are issued two
    // chunks before it is computed, so a chunk waits for memory only at the very start of an entry
    float rq[H_PPT], rf[H_PPT], rv[HTC], nq[H_PPT], nf[H_PPT], nv[HTC];
    auto request = [&](int t0, float (&q_)[H_PPT], float (&f_)[H_PPT], float (&v_)[HTC]) {
        const int nt = count - t0 < HTC ? count - t0 : HTC;
#pragma unroll
        for (int k = 0; k < H_PPT; ++k)
        {
            const int i = tid + k * NT;
            q_[k] = f_[k] = 0.f;
            if (i < nt * D)
            {
                const int64_t row = (int64_t) (first + t0 + i / D) * p.ldp;
                q_[k] = El<DT>::ld(p.proj, row + h * D + i % D);
                f_[k] = El<DT>::ld(p.proj, row + HD + h * D + i % D);
            }
        }
#pragma unroll
        for (int tt = 0; tt < HTC; ++tt)
            v_[tt] = (s == 0 && live && tt < nt) ? El<DT>::ld(p.proj, (int64_t) (first + t0 + tt) * p.ldp + 2 * HD + h * V + v) : 0.f;
    };
    request(0, rq, rf, rv);
    if (HTC < count)
        request(HTC, nq, nf, nv);
    for (int t0 = 0; t0 < count; t0 += HTC)
    {
        const int nt = count - t0 < HTC ? count - t0 : HTC;
#pragma unroll
        for (int k = 0; k < H_PPT; ++k)
        {
            const int i = tid + k * NT;
            if (i < nt * D)
            {
                const int d = i % D;
                float qr = rq[k] / (1.f + expf(-rq[k]));
                if (DT == DT_BF16)
                    qr = bf2f(f2bf(qr)); // the projection's activation is a bfloat16 value; everything behind it is fp32
                const float lo = p.lower[h * D + d];
                fq[i] = make_float2(lo + (1.f - lo) * (1.f / (1.f + expf(-(rf[k] + p.f_bias[h * D + d])))), qr);
            }
        }
        if (s == 0)
        {
#pragma unroll
            for (int tt = 0; tt < HTC; ++tt)
                vs[tt * vpad + vl] = rv[tt];
        }
        __syncthreads();
        if (t0 + HTC < count)
        {
#pragma unroll
            for (int k = 0; k < H_PPT; ++k)
            {
                rq[k] = nq[k];
                rf[k] = nf[k];
            }
#pragma unroll
            for (int tt = 0; tt < HTC; ++tt)
                rv[tt] = nv[tt];
            if (t0 + 2 * HTC < count)
                request(t0 + 2 * HTC, nq, nf, nv); // in flight under this chunk's and the next chunk's recurrence
        }
        for (int tt = 0; tt < nt; ++tt)
        {
            const float x = vs[tt * vpad + vl];
            float o = 0.f;
#pragma unroll
            for (int j = 0; j < DSZ; ++j)
            {
                if (d0 + j < D)
                {
                    const float2 c = fq[tt * D + d0 + j];
                    S[j] = c.x * S[j] + (1.f - c.x) * x;
                    o += S[j] * c.y;
                }
            }
            os[(tt * DS + s) * vpad + vl] = live ? o : 0.f;
        }
        __syncthreads();
        // rows of the chunk are shared out over the slices: thread (s, v) finishes rows s, s + DS, ...
        if (!fuse_norm)
        {
            for (int tt = s; tt < nt; tt += DS)
            {
                if (live)
                {
                    float o = 0.f;
                    for (int s2 = 0; s2 < DS; ++s2)
                        o += os[(tt * DS + s2) * vpad + vl];
                    p.o32[(int64_t) (first + t0 + tt) * (p.heads * V) + h * V + v] = o;
                }
            }
            __syncthreads();
            continue;
        }
        for (int tt = s; tt < nt; tt += DS) // wave-uniform
        {
            float o = 0.f;
            for (int s2 = 0; s2 < DS; ++s2)
                o += os[(tt * DS + s2) * vpad + vl];
            const float ss = wave_sum(o * o);
            if (lane == 0)
                red[tt * nvw + vw] = ss;
        }
        __syncthreads();
        for (int tt = s; tt < nt; tt += DS)
        {
            if (live)
            {
                float o = 0.f, ss = 0.f;
                for (int s2 = 0; s2 < DS; ++s2)
                    o += os[(tt * DS + s2) * vpad + vl];
                for (int w = 0; w < nvw; ++w)
                    ss += red[tt * nvw + w];
                El<DT>::st(p.out, (int64_t) (first + t0 + tt) * (p.heads * V) + h * V + v, o * (1.f / sqrtf(ss / (float) V + p.eps)) * nw);
            }
        }
        // (the next chunk's first write to fq / vs is behind this chunk's last read of them: the barrier above; os and red are
        // rewritten only behind the next chunk's first barrier)
    }
    if (live)
    {
#pragma unroll
        for (int j = 0; j < DSZ; ++j)
            if (d0 + j < D)
                sp[(int64_t) (d0 + j) * V] = S[j];
    }
}

// per (row, head): o / sqrt(mean(o^2) + eps) * w over the head's vdim channels; one wave each
template <int DT>
__global__ __launch_bounds__(256) void head_rmsnorm_kernel(void* y, const float* o, const float* w, int64_t n_heads_total, int vdim, float eps)
{
    const int64_t i = (int64_t) blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (i >= n_heads_total)
        return;
    const float* oi = o + i * vdim;
    float ss = 0.f;
    for (int c = lane; c < vdim; c += 64)
        ss += oi[c] * oi[c];
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float) vdim + eps);
    for (int c = lane; c < vdim; c += 64)
        El<DT>::st(y, i * vdim + c, oi[c] * inv * w[c]);
}

} // namespace

// ---------------------------------------------------------------------------------------------------------------- launchers
int launch_stack_embed(float* x, float* keep, const int32_t* ids, const void* table, int32_t dtype, int32_t tokens, int32_t width,
    int32_t vocab, float scale, hipStream_t stream, int32_t copies, int64_t copy_stride)
{
    if (tokens <= 0)
        return 0;
    if (!known_dtype(dtype, "stack_embed"))
        return -1;
    if (dtype == DT_BF16)
        hipLaunchKernelGGL((embed_kernel<DT_BF16>), dim3(tokens), dim3(256), 0, stream, x, keep, ids, table, width, vocab, scale, copies,
            copy_stride);
    else
        hipLaunchKernelGGL((embed_kernel<DT_FLOAT>), dim3(tokens), dim3(256), 0, stream, x, keep, ids, table, width, vocab, scale, copies,
            copy_stride);
    return launched("stack_embed");
}

int launch_stack_pair_embed(float* x, const int32_t* ids, const int32_t* prev, const void* pair_table, int32_t dtype, int32_t tokens,
    int32_t width, int32_t buckets, int32_t mul_prev, int32_t mul_cur, hipStream_t stream, int32_t copies, int64_t copy_stride)
{
    if (tokens <= 0)
        return 0;
    if (!known_dtype(dtype, "stack_pair_embed"))
        return -1;
    if (buckets < 1 || !ids || !prev || !pair_table || !x)
    {
        set_error("stack_pair_embed: %d buckets, or a missing operand", buckets);
        return -1;
    }
    if (dtype == DT_BF16)
        hipLaunchKernelGGL((pair_embed_kernel<DT_BF16>), dim3(tokens), dim3(256), 0, stream, x, ids, prev, pair_table, width, buckets, mul_prev,
            mul_cur, copies, copy_stride);
    else
        hipLaunchKernelGGL((pair_embed_kernel<DT_FLOAT>), dim3(tokens), dim3(256), 0, stream, x, ids, prev, pair_table, width, buckets, mul_prev,
            mul_cur, copies, copy_stride);
    return launched("stack_pair_embed");
}

int launch_stack_token_shift(const StackShiftParams& p, hipStream_t stream)
{
    if (p.tokens <= 0 || p.entries <= 0)
        return 0;
    if (!known_dtype(p.dtype, "stack_token_shift"))
        return -1;
    if (p.width < 1 || !p.n || !p.mu || !p.carry || !p.h || !p.tok_entry || !p.tok_pos || !p.ent_slot || !p.ent_first || !p.ent_count || !p.ent_pos0)
    {
        set_error("stack_token_shift: width %d, or a missing operand", p.width);
        return -1;
    }
    // few rows (decoding): a row's channels are spread over workgroups
    const dim3 grid(p.tokens + p.entries, p.tokens >= 128 ? 1 : std::min((p.width + 255) / 256, 16));
    if (p.dtype == DT_BF16)
        hipLaunchKernelGGL((token_shift_kernel<DT_BF16>), grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((token_shift_kernel<DT_FLOAT>), grid, dim3(256), 0, stream, p);
    return launched("stack_token_shift");
}

namespace
{
// The form for rows of a multiple of 4 up to HV_K * 4096 elements: up to 1024 threads, a thread owns HV_K float4 columns of every
// stream and has ALL of them in flight before its first store (the streams are read and written through the same pointer, so in
// a loop every store would fence the loads behind it); the combined row stays in registers.
constexpr int HV_K = 2;

template <int DT, int SM>
__global__ __launch_bounds__(1024) void hyper_norm_vec_kernel(const StackHyperParams p)
{
    __shared__ float red[32];
    const int t = p.rows ? p.rows[blockIdx.x] : blockIdx.x, tid = threadIdx.x, S = p.streams, W4 = p.width >> 2, NT = blockDim.x;
    float4 xs[HV_K][SM], yv[HV_K], u[HV_K];
#pragma unroll
    for (int k = 0; k < HV_K; ++k)
    {
        const int c4 = tid + k * NT;
        yv[k] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int s = 0; s < SM; ++s)
            xs[k][s] = (s < S && c4 < W4) ? reinterpret_cast<const float4*>(p.x + s * p.stream_stride + (int64_t) t * p.width)[c4]
                                          : make_float4(0.f, 0.f, 0.f, 0.f);
        if (p.y && c4 < W4)
            yv[k] = reinterpret_cast<const float4*>(p.y + (int64_t) t * p.width)[c4];
    }
    float cm[SM][SM], co[SM], ci[SM];
#pragma unroll
    for (int a = 0; a < SM; ++a)
    {
        co[a] = (p.y && a < S) ? p.out[a] : 0.f;
        ci[a] = a < S ? (p.in ? p.in[a] : 1.f) : 0.f;
#pragma unroll
        for (int b = 0; b < SM; ++b)
            cm[a][b] = (p.y && a < S && b < S) ? p.mix[a * S + b] : 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < HV_K; ++k)
    {
        const int c4 = tid + k * NT;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int to = 0; to < SM; ++to)
        {
            float4 n = xs[k][to];
            if (p.y)
            {
                n = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int s = 0; s < SM; ++s)
                {
                    n.x = fmaf(cm[s][to], xs[k][s].x, n.x);
                    n.y = fmaf(cm[s][to], xs[k][s].y, n.y);
                    n.z = fmaf(cm[s][to], xs[k][s].z, n.z);
                    n.w = fmaf(cm[s][to], xs[k][s].w, n.w);
                }
                n.x = fmaf(co[to], yv[k].x, n.x);
                n.y = fmaf(co[to], yv[k].y, n.y);
                n.z = fmaf(co[to], yv[k].z, n.z);
                n.w = fmaf(co[to], yv[k].w, n.w);
                if (to < S && c4 < W4 && !p.rows) // a gathered launch is the streams' last reader: nothing is written back
                    reinterpret_cast<float4*>(p.x + to * p.stream_stride + (int64_t) t * p.width)[c4] = n;
            }
            acc.x = fmaf(ci[to], n.x, acc.x);
            acc.y = fmaf(ci[to], n.y, acc.y);
            acc.z = fmaf(ci[to], n.z, acc.z);
            acc.w = fmaf(ci[to], n.w, acc.w);
        }
        u[k] = acc;
        if (p.sum_out && c4 < W4)
            reinterpret_cast<float4*>(p.sum_out + (int64_t) t * p.width)[c4] = acc;
        ss += acc.x * acc.x + acc.y * acc.y + acc.z * acc.z + acc.w * acc.w;
    }
    if (!p.h && !p.h32)
        return;
    ss = block_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float) p.width + p.eps);
#pragma unroll
    for (int k = 0; k < HV_K; ++k)
    {
        const int c4 = tid + k * NT;
        if (c4 < W4)
        {
            const float4 w = reinterpret_cast<const float4*>(p.w)[c4];
            const int64_t o = (int64_t) blockIdx.x * p.width + 4 * c4;
            if (p.h32)
                *reinterpret_cast<float4*>(p.h32 + o) = make_float4(u[k].x * inv * w.x, u[k].y * inv * w.y, u[k].z * inv * w.z, u[k].w * inv * w.w);
            if (!p.h)
                continue;
            if (DT == DT_BF16)
                *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(p.h) + o)
                    = make_uint2((uint32_t) f2bf(u[k].x * inv * w.x) | ((uint32_t) f2bf(u[k].y * inv * w.y) << 16),
                        (uint32_t) f2bf(u[k].z * inv * w.z) | ((uint32_t) f2bf(u[k].w * inv * w.w) << 16));
            else
                *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.h) + o)
                    = make_float4(u[k].x * inv * w.x, u[k].y * inv * w.y, u[k].z * inv * w.z, u[k].w * inv * w.w);
        }
    }
}

template <int DT>
void launch_hyper_vec(const StackHyperParams& p, int nt, hipStream_t stream)
{
    if (p.streams <= 1)
        hipLaunchKernelGGL((hyper_norm_vec_kernel<DT, 1>), dim3(p.tokens), dim3(nt), 0, stream, p);
    else if (p.streams <= 2)
        hipLaunchKernelGGL((hyper_norm_vec_kernel<DT, 2>), dim3(p.tokens), dim3(nt), 0, stream, p);
    else if (p.streams <= 4)
        hipLaunchKernelGGL((hyper_norm_vec_kernel<DT, 4>), dim3(p.tokens), dim3(nt), 0, stream, p);
    else
        hipLaunchKernelGGL((hyper_norm_vec_kernel<DT, 8>), dim3(p.tokens), dim3(nt), 0, stream, p);
}

} // namespace

int launch_stack_hyper_norm(const StackHyperParams& p, hipStream_t stream)
{
    if (p.tokens <= 0)
        return 0;
    if (!known_dtype(p.dtype, "stack_hyper_norm"))
        return -1;
    if (p.streams < 1 || p.streams > HY_MAXS || p.width < 1 || !p.x || (p.y && (!p.mix || !p.out)) || ((p.h || p.h32) && !p.w))
    {
        set_error("stack_hyper_norm: %d streams (1 .. %d) of width %d, or a missing operand", p.streams, HY_MAXS, p.width);
        return -1;
    }
    const bool al16 = !(reinterpret_cast<uintptr_t>(p.x) & 15) && !(reinterpret_cast<uintptr_t>(p.y) & 15) && !(reinterpret_cast<uintptr_t>(p.h) & 15)
        && !(reinterpret_cast<uintptr_t>(p.w) & 15) && !(reinterpret_cast<uintptr_t>(p.sum_out) & 15) && !(reinterpret_cast<uintptr_t>(p.h32) & 15)
        && p.stream_stride % 4 == 0;
    if (p.width % 4 == 0 && p.width <= HV_K * 4096 && al16)
    {
        const int nt = std::min(1024, (p.width / 4 + 63) / 64 * 64);
        if (p.dtype == DT_BF16)
            launch_hyper_vec<DT_BF16>(p, nt, stream);
        else
            launch_hyper_vec<DT_FLOAT>(p, nt, stream);
        return launched("stack_hyper_norm");
    }
    const size_t lds = sizeof(float) * (size_t) p.width;
    if (lds > 64 * 1024)
    {
        set_error("stack_hyper_norm: width %d is beyond the row it keeps in LDS", p.width);
        return -1;
    }
    if (p.dtype == DT_BF16)
        hipLaunchKernelGGL((hyper_norm_kernel<DT_BF16>), dim3(p.tokens), dim3(HY_T), lds, stream, p);
    else
        hipLaunchKernelGGL((hyper_norm_kernel<DT_FLOAT>), dim3(p.tokens), dim3(HY_T), lds, stream, p);
    return launched("stack_hyper_norm");
}

int launch_stack_pass_entry(float* x, const float* add, const float* row, int32_t tokens, int32_t width, hipStream_t stream)
{
    const int64_t n = (int64_t) tokens * width;
    if (n <= 0 || (!add && !row))
        return 0;
    hipLaunchKernelGGL(pass_entry_kernel, dim3((unsigned) ((n + 255) / 256)), dim3(256), 0, stream, x, add, row, n, width);
    return launched("stack_pass_entry");
}

int launch_stack_group_rmsnorm(void* y1, void* y2, const float* x, const int32_t* rows, const float* w1, const float* w2, int32_t dtype,
    int32_t n_rows, int32_t width, int32_t groups, float eps, hipStream_t stream)
{
    if (n_rows <= 0)
        return 0;
    if (!known_dtype(dtype, "stack_group_rmsnorm"))
        return -1;
    if (groups < 1 || width % groups)
    {
        set_error("stack_group_rmsnorm: width %d does not split into %d equal groups", width, groups);
        return -1;
    }
    if (dtype == DT_BF16)
        hipLaunchKernelGGL((group_rmsnorm_kernel<DT_BF16>), dim3(n_rows, groups), dim3(GN_T), 0, stream, y1, y2, x, rows, w1, w2, width, groups, eps);
    else
        hipLaunchKernelGGL((group_rmsnorm_kernel<DT_FLOAT>), dim3(n_rows, groups), dim3(GN_T), 0, stream, y1, y2, x, rows, w1, w2, width, groups, eps);
    return launched("stack_group_rmsnorm");
}

int launch_stack_gelu_gate(void* y, const void* gu, int32_t dtype, int32_t tokens, int32_t ff, int64_t ld, hipStream_t stream, int32_t act)
{
    const int64_t n = (int64_t) tokens * ff;
    if (n <= 0)
        return 0;
    if (!known_dtype(dtype, "stack_gelu_gate"))
        return -1;
    const dim3 grid((unsigned) ((n + 255) / 256));
    if (dtype == DT_BF16)
        hipLaunchKernelGGL((gelu_gate_kernel<DT_BF16>), grid, dim3(256), 0, stream, y, gu, tokens, ff, ld, act);
    else
        hipLaunchKernelGGL((gelu_gate_kernel<DT_FLOAT>), grid, dim3(256), 0, stream, y, gu, tokens, ff, ld, act);
    return launched("stack_gelu_gate");
}

int launch_stack_row_rmsnorm(void* y, int64_t ldy, const void* x, int64_t ldx, const float* w, int32_t dtype, int32_t rows, int32_t n, float eps,
    hipStream_t stream)
{
    if (rows <= 0 || n <= 0)
        return 0;
    if (!known_dtype(dtype, "stack_row_rmsnorm"))
        return -1;
    const dim3 grid((rows + 3) / 4);
    if (dtype == DT_BF16)
        hipLaunchKernelGGL((row_rmsnorm_kernel<DT_BF16>), grid, dim3(256), 0, stream, y, ldy, x, ldx, w, rows, n, eps);
    else
        hipLaunchKernelGGL((row_rmsnorm_kernel<DT_FLOAT>), grid, dim3(256), 0, stream, y, ldy, x, ldx, w, rows, n, eps);
    return launched("stack_row_rmsnorm");
}

static bool attn_shape_ok(const StackAttnParams& p, const char* what)
{
    if (!known_dtype(p.dtype, what))
        return false;
    if (p.heads < 1 || p.kv_heads < 1 || p.heads % p.kv_heads || p.maps < 1 || p.maps > 2 || p.dim < 1 || p.vdim < 1 || p.page < 1
        || p.max_blocks < 1)
    {
        set_error("%s: heads %d, kv_heads %d, maps %d, dim %d, vdim %d, page %d, max_blocks %d is not a shape it serves", what, p.heads,
            p.kv_heads, p.maps, p.dim, p.vdim, p.page, p.max_blocks);
        return false;
    }
    if ((p.rot_dims & 1) || p.rot_dims > p.dim || p.rot_dims < 0)
    {
        set_error("%s: the rotation pairs neighbours: rot_dims %d must be even and <= dim %d", what, p.rot_dims, p.dim);
        return false;
    }
    if (p.mask < MASK_CAUSAL || p.mask > MASK_CHUNK || (p.mask != MASK_CAUSAL && p.mask_size < 1) || p.mask_keep < 0
        || (p.mask_keep > 0 && p.mask != MASK_WINDOW) || (p.values_are_keys && p.vdim != p.dim) || p.weights < WEIGHTS_SOFTMAX
        || p.weights > WEIGHTS_SIGMOID || (p.log_r1 && !p.log_r2))
    {
        set_error("%s: mask %d of size %d, weights %d is not a form it serves", what, p.mask, p.mask_size, p.weights);
        return false;
    }
    return true;
}

int launch_stack_rope_kv(const StackAttnParams& p, hipStream_t stream)
{
    if (p.tokens <= 0)
        return 0;
    if (!attn_shape_ok(p, "stack_rope_kv"))
        return -1;
    if (p.rot_dims > 0 && (p.dim & 1))
    {
        set_error("stack_rope_kv: the rotation pairs (2i, 2i + 1) inside every head: dim %d must be even", p.dim);
        return -1;
    }
    if (p.bias || p.qk_unit_norm)
    {
        if (p.dim > 64 * PREP_EPL)
        {
            set_error("stack_rope_kv: dim %d is beyond the %d a wave keeps", p.dim, 64 * PREP_EPL);
            return -1;
        }
        const int vecs = (p.heads + p.kv_heads) * p.maps + p.kv_heads;
        const dim3 pg(p.tokens, (vecs + 3) / 4);
        if (p.dtype == DT_BF16)
            hipLaunchKernelGGL((attn_prep_kernel<DT_BF16>), pg, dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL((attn_prep_kernel<DT_FLOAT>), pg, dim3(256), 0, stream, p);
        return launched("stack_rope_kv (general)");
    }
    // few rows (decoding): one element per thread; many rows: a workgroup per row walks it
    const int per_row = (p.heads + p.kv_heads) * p.maps * p.dim;
    const dim3 grid(p.tokens, p.tokens >= 64 ? 1 : (per_row + 255) / 256);
    if (p.dtype == DT_BF16)
        hipLaunchKernelGGL((rope_kv_kernel<DT_BF16>), grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((rope_kv_kernel<DT_FLOAT>), grid, dim3(256), 0, stream, p);
    return launched("stack_rope_kv");
}

int launch_stack_latent_prep(const StackAttnParams& p, int32_t qk_dim, const float* latent_norm_w, hipStream_t stream, const void* q_src,
    int64_t ldq, int32_t dkv_col)
{
    if (!q_src)
    {
        q_src = p.proj;
        ldq = p.ldp;
    }
    if (dkv_col < 0)
        dkv_col = p.heads * (qk_dim + (p.dim - p.vdim));
    if (p.tokens <= 0)
        return 0;
    if (!attn_shape_ok(p, "stack_latent_prep"))
        return -1;
    if (p.kv_heads != 1 || p.maps != 1 || p.rot_dims > p.dim - p.vdim || p.vdim < 1 || qk_dim < 1 || !latent_norm_w || !p.freq)
    {
        set_error("stack_latent_prep: one key/value head of dim = rank + rotated part and vdim = rank (dim %d, vdim %d, rot %d, kv_heads %d, maps %d)",
            p.dim, p.vdim, p.rot_dims, p.kv_heads, p.maps);
        return -1;
    }
    const dim3 grid(p.tokens, (p.heads + 1 + 3) / 4);
    if (p.dtype == DT_BF16)
        hipLaunchKernelGGL((latent_prep_kernel<DT_BF16>), grid, dim3(256), 0, stream, p, qk_dim, latent_norm_w, q_src, ldq, dkv_col);
    else
        hipLaunchKernelGGL((latent_prep_kernel<DT_FLOAT>), grid, dim3(256), 0, stream, p, qk_dim, latent_norm_w, q_src, ldq, dkv_col);
    return launched("stack_latent_prep");
}

int launch_stack_talk_combine(const StackAttnParams& p, const void* pairs, hipStream_t stream)
{
    if (p.tokens <= 0)
        return 0;
    if (!known_dtype(p.dtype, "stack_talk_combine"))
        return -1;
    const size_t lds = sizeof(float) * (size_t) p.heads * p.heads;
    if (!p.talk || !pairs || !p.out || p.heads < 1 || p.kv_heads < 1 || p.heads % p.kv_heads || p.vdim < 1 || lds > 64 * 1024)
    {
        set_error("stack_talk_combine: %d heads over %d key/value heads, vdim %d, or a missing operand", p.heads, p.kv_heads, p.vdim);
        return -1;
    }
    // few rows (decoding): a row's output channels are spread over workgroups
    const dim3 grid(p.tokens, p.tokens >= 256 ? 1 : std::min((p.heads * p.vdim + 255) / 256, 16));
    if (p.dtype == DT_BF16)
        hipLaunchKernelGGL((talk_combine_kernel<DT_BF16>), grid, dim3(256), lds, stream, p, pairs);
    else
        hipLaunchKernelGGL((talk_combine_kernel<DT_FLOAT>), grid, dim3(256), lds, stream, p, pairs);
    return launched("stack_talk_combine");
}

int launch_stack_attention_general(const StackAttnParams& p, hipStream_t stream)
{
    // (the dispatcher launch_stack_attention lives in stack_attn.hip)
    if (p.tokens <= 0)
        return 0;
    if (!attn_shape_ok(p, "stack_attention"))
        return -1;
    if (p.talk)
    {
        const size_t lds = sizeof(float) * ((size_t) p.heads * p.dim + 2 * (size_t) p.heads * TK_T + (size_t) p.heads * p.heads + 2 * (size_t) p.heads + 32);
        if (p.maps != 1 || p.weights != WEIGHTS_SOFTMAX || p.softcap > 0.f || p.temp || p.slope || p.log_r1 || p.head_norm || p.heads > TK_MAXH
            || p.heads * p.vdim > TK_T * TK_CPT || lds > 150 * 1024)
        {
            set_error("stack_attention: talking heads go with one softmax map without penalties, up to %d heads and %d output channels "
                      "(heads %d, vdim %d, dim %d)",
                TK_MAXH, TK_T * TK_CPT, p.heads, p.vdim, p.dim);
            return -1;
        }
        if (p.dtype == DT_BF16)
        {
            if (lds > 64 * 1024)
                (void) hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_talk_kernel<DT_BF16>), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds);
            hipLaunchKernelGGL((attn_talk_kernel<DT_BF16>), dim3(p.tokens), dim3(TK_T), lds, stream, p);
        }
        else
        {
            if (lds > 64 * 1024)
                (void) hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_talk_kernel<DT_FLOAT>), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds);
            hipLaunchKernelGGL((attn_talk_kernel<DT_FLOAT>), dim3(p.tokens), dim3(TK_T), lds, stream, p);
        }
        return launched("stack_attention (talking heads)");
    }
    if (p.vdim > AT * A_CPT)
    {
        set_error("stack_attention: vdim %d is beyond the %d channels the general kernel keeps", p.vdim, AT * A_CPT);
        return -1;
    }
    const size_t lds = sizeof(float) * ((size_t) p.maps * p.dim + (size_t) p.maps * AT + 32);
    const dim3 grid(p.tokens, p.heads);
#define TLLM_ATTN_GEN(DT, MAPS) hipLaunchKernelGGL((attn_general_kernel<DT, MAPS>), grid, dim3(AT), lds, stream, p)
    if (p.dtype == DT_BF16)
    {
        if (p.maps == 2)
            TLLM_ATTN_GEN(DT_BF16, 2);
        else
            TLLM_ATTN_GEN(DT_BF16, 1);
    }
    else
    {
        if (p.maps == 2)
            TLLM_ATTN_GEN(DT_FLOAT, 2);
        else
            TLLM_ATTN_GEN(DT_FLOAT, 1);
    }
#undef TLLM_ATTN_GEN
    return launched("stack_attention");
}

float stack_rope_freqs(float* freq, int32_t dims, double base, double factor, double original, double fast, double slow)
{
    const int n = dims / 2;
    const double two_pi = 6.283185307179586476925286766559;
    double lo = 0, hi = 0;
    if (factor > 0)
    {
        auto dim_of = [&](double turns) { return dims * std::log(original / (two_pi * turns)) / (2.0 * std::log(base)); };
        lo = std::max(std::floor(dim_of(fast)), 0.0);
        hi = std::min(std::ceil(dim_of(slow)), (double) (dims - 1));
    }
    for (int i = 0; i < n; ++i)
    {
        double f = std::pow(base, -2.0 * i / dims);
        if (factor > 0)
        {
            double ramp = (i - lo) / std::max(hi - lo, 0.001);
            ramp = ramp < 0 ? 0 : (ramp > 1 ? 1 : ramp);
            f = f / factor * ramp + f * (1 - ramp);
        }
        freq[i] = (float) f;
    }
    return factor > 0 ? (float) (0.1 * std::log(factor) + 1.0) : 1.f;
}

void stack_rope_freqs_banded(float* freq, int32_t dims, double base, double factor, double original, double low, double high)
{
    const double two_pi = 6.283185307179586476925286766559;
    for (int i = 0; i < dims / 2; ++i)
    {
        double f = std::pow(base, -2.0 * i / dims);
        if (factor > 0)
        {
            const double wave = two_pi / f;
            if (wave > original / low)
                f = f / factor;
            else if (!(wave < original / high))
            {
                const double s = (original / wave - low) / (high - low);
                f = (1.0 - s) * f / factor + s * f;
            }
        }
        freq[i] = (float) f;
    }
}

bool stack_hgrn2_serves(int32_t dim, int32_t vdim)
{
    if (dim < 1 || vdim < 1)
        return false;
    return dim <= 512; // 16-column groups x 16 slices of 32 rows; up to 128 the column-per-thread form serves too
}

int launch_stack_hgrn2(const StackHgrnParams& p, hipStream_t stream)
{
    if (p.tokens <= 0 || p.entries <= 0)
        return 0;
    if (!known_dtype(p.dtype, "stack_hgrn2"))
        return -1;
    if (p.heads < 1 || !stack_hgrn2_serves(p.dim, p.vdim))
    {
        set_error("stack_hgrn2: heads %d, dim %d, vdim %d is not a shape it serves (dim up to 512)", p.heads, p.dim, p.vdim);
        return -1;
    }
    {
        // Long portions (a prompt): a head is cut into groups of 16 columns, one workgroup each, so that the sequential walk over
        // the rows runs on many CUs at once; the head norm is then a pass of its own.  Short portions and decoded tokens: one
        // workgroup holds the whole head (vdim <= 256) and norms it in the same launch.
        bool spread = p.max_count >= 32 || p.vdim > 256;
        int vpad = 0, DS = 0, dsz = 0, NT = 0, htc = 0, ppt = 0;
        auto shape = [&]() {
            vpad = spread ? 16 : (p.vdim + 63) / 64 * 64;
            htc = 8;
            const int max_threads = spread ? 256 : 1024;
            DS = std::min(max_threads / vpad, (p.dim + 7) / 8);
            dsz = (p.dim + DS - 1) / DS;
            dsz = dsz <= 8 ? 8 : (dsz <= 16 ? 16 : 32);
            DS = (p.dim + dsz - 1) / dsz;
            NT = vpad * DS;
            ppt = spread ? dsz / 2 : 4; // (row, channel) pairs per thread and chunk: 8 * dim / NT <= dsz / 2 resp. 8 * dsz / vpad <= 4
            return dsz * DS >= p.dim && NT <= max_threads && htc * p.dim <= ppt * NT;
        };
        bool fits = shape();
        if (!fits && !spread)
        {
            spread = true; // a head too tall for one workgroup: the column groups take it
            fits = shape();
        }
        if (fits)
        {
            const size_t lds = sizeof(float) * ((size_t) 2 * htc * p.dim + (size_t) htc * vpad + (size_t) htc * DS * vpad + (size_t) htc * ((vpad + 63) / 64));
            const dim3 hg(p.entries, p.heads, spread ? (p.vdim + vpad - 1) / vpad : 1);
            const int fuse = spread ? 0 : 1;
#define TLLM_HGRN_K(DT, DSZ)                                                                                                    \
    do                                                                                                                              \
    {                                                                                                                               \
        if (spread)                                                                                                                 \
            hipLaunchKernelGGL((hgrn2_head_kernel<DT, DSZ, 8, DSZ / 2, 256>), hg, dim3(NT), lds, stream, p, vpad, DS, fuse);                  \
        else                                                                                                                        \
            hipLaunchKernelGGL((hgrn2_head_kernel<DT, DSZ, 8, 4, 1024>), hg, dim3(NT), lds, stream, p, vpad, DS, fuse);                   \
    } while (0)
#define TLLM_HGRN_H(DT)                                                                                                         \
    do                                                                                                                              \
    {                                                                                                                               \
        if (dsz == 8)                                                                                                               \
            TLLM_HGRN_K(DT, 8);                                                                                                     \
        else if (dsz == 16)                                                                                                         \
            TLLM_HGRN_K(DT, 16);                                                                                                    \
        else                                                                                                                        \
            TLLM_HGRN_K(DT, 32);                                                                                                    \
    } while (0)
            if (p.dtype == DT_BF16)
                TLLM_HGRN_H(DT_BF16);
            else
                TLLM_HGRN_H(DT_FLOAT);
#undef TLLM_HGRN_H
#undef TLLM_HGRN_K
            if (launched("stack_hgrn2 (sliced)"))
                return -1;
            if (fuse)
                return 0;
            const int64_t nh = (int64_t) p.tokens * p.heads;
            if (p.dtype == DT_BF16)
                hipLaunchKernelGGL((head_rmsnorm_kernel<DT_BF16>), dim3((unsigned) ((nh + 3) / 4)), dim3(256), 0, stream, p.out, p.o32, p.norm_w,
                    nh, p.vdim, p.eps);
            else
                hipLaunchKernelGGL((head_rmsnorm_kernel<DT_FLOAT>), dim3((unsigned) ((nh + 3) / 4)), dim3(256), 0, stream, p.out, p.o32, p.norm_w,
                    nh, p.vdim, p.eps);
            return launched("stack_hgrn2 norm");
        }
    }
    if (p.dim > 128)
    {
        set_error("stack_hgrn2: dim %d with vdim %d fits neither form", p.dim, p.vdim);
        return -1;
    }
    const dim3 grid(p.entries, p.heads, (p.vdim + 63) / 64);
#define TLLM_HGRN(DT, DMAX) hipLaunchKernelGGL((hgrn2_scan_kernel<DT, DMAX>), grid, dim3(64), 0, stream, p)
#define TLLM_HGRN_D(DT)                                                                                                         \
    do                                                                                                                              \
    {                                                                                                                               \
        if (p.dim <= 16)                                                                                                            \
            TLLM_HGRN(DT, 16);                                                                                                      \
        else if (p.dim <= 32)                                                                                                       \
            TLLM_HGRN(DT, 32);                                                                                                      \
        else if (p.dim <= 64)                                                                                                       \
            TLLM_HGRN(DT, 64);                                                                                                      \
        else                                                                                                                        \
            TLLM_HGRN(DT, 128);                                                                                                     \
    } while (0)
    if (p.dtype == DT_BF16)
        TLLM_HGRN_D(DT_BF16);
    else
        TLLM_HGRN_D(DT_FLOAT);
#undef TLLM_HGRN_D
#undef TLLM_HGRN
    if (launched("stack_hgrn2 scan"))
        return -1;
    const int64_t nh = (int64_t) p.tokens * p.heads;
    if (p.dtype == DT_BF16)
        hipLaunchKernelGGL((head_rmsnorm_kernel<DT_BF16>), dim3((unsigned) ((nh + 3) / 4)), dim3(256), 0, stream, p.out, p.o32, p.norm_w, nh,
            p.vdim, p.eps);
    else
        hipLaunchKernelGGL((head_rmsnorm_kernel<DT_FLOAT>), dim3((unsigned) ((nh + 3) / 4)), dim3(256), 0, stream, p.out, p.o32, p.norm_w, nh,
            p.vdim, p.eps);
    return launched("stack_hgrn2 norm");
}

} // namespace kernels
} // namespace tllm
