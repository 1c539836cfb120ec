// Routed mixture of experts of the ragged-batch stack engine (stack_kernels.h): the fp32 router with its grouped top-k choice,
// the ordering of (token, chosen expert) pairs by expert for the grouped products, and the weighted sum of the experts' outputs.
#include "dev_utils.h"
#include "stack_kernels.h"
#include <algorithm>

namespace tllm
{
namespace kernels
{
using namespace dev;

namespace
{

template <int DT>
__device__ __forceinline__ float ld_el(const void* p, int64_t i)
{
    if constexpr (DT == DT_BF16)
        return bf2f(reinterpret_cast<const uint16_t*>(p)[i]);
    else
        return reinterpret_cast<const float*>(p)[i];
}

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

// the lane that holds the largest value of the wave, the lowest index among equals; every lane gets (value, index)
__device__ __forceinline__ void wave_argmax(float& v, int& idx)
{
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1)
    {
        const float ov = __shfl_xor(v, d, 64);
        const int oi = __shfl_xor(idx, d, 64);
        if (ov > v || (ov == v && oi < idx))
        {
            v = ov;
            idx = oi;
        }
    }
}

constexpr int RT = 8;         // tokens per logits workgroup: a router row is read once for all of them
constexpr int MAX_OUT = 1024; // router outputs (experts + identities)
constexpr int MAX_TOP = 16;
constexpr int FEW_TOKENS = 8; // steps of this many tokens or fewer route in one launch and gather inside the sort

// Router logits, fp32: workgroup (x, y) = 4 router rows (one per wave) x RT tokens; lanes split the width in float4 pieces where
// rows are 16-byte aligned.  z [tokens, outputs].
template <int DT>
__global__ __launch_bounds__(256) void moe_logits_kernel(const StackMoeParams p, float* z)
{
    const int NE = p.experts + p.identity, W = p.width;
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63, t0 = blockIdx.y * RT;
    if (e >= NE)
        return;
    float acc[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r)
        acc[r] = 0.f;
    const float* wr = p.router_w + (int64_t) e * W;
    const int nt = p.tokens - t0 < RT ? p.tokens - t0 : RT;
    if ((W & 7) == 0)
    {
        for (int k = lane * 8; k < W; k += 64 * 8)
        {
            const float4 w0 = *reinterpret_cast<const float4*>(wr + k), w1 = *reinterpret_cast<const float4*>(wr + k + 4);
            const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
            for (int r = 0; r < RT; ++r)
            {
                if (r < nt)
                {
                    float hv[8];
                    if constexpr (DT == DT_BF16)
                    {
                        const uint4 u = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.h) + (int64_t) (t0 + r) * W + k);
                        const uint32_t us[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                        {
                            hv[2 * i] = __builtin_bit_cast(float, us[i] << 16);
                            hv[2 * i + 1] = __builtin_bit_cast(float, us[i] & 0xffff0000u);
                        }
                    }
                    else
                    {
                        const float* hp = reinterpret_cast<const float*>(p.h) + (int64_t) (t0 + r) * W + k;
                        const float4 h0 = *reinterpret_cast<const float4*>(hp), h1 = *reinterpret_cast<const float4*>(hp + 4);
                        hv[0] = h0.x, hv[1] = h0.y, hv[2] = h0.z, hv[3] = h0.w, hv[4] = h1.x, hv[5] = h1.y, hv[6] = h1.z, hv[7] = h1.w;
                    }
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        acc[r] = fmaf(wv[i], hv[i], acc[r]);
                }
            }
        }
    }
    else
    {
        for (int k = lane; k < W; k += 64)
        {
            const float wv = wr[k];
#pragma unroll
            for (int r = 0; r < RT; ++r)
                if (r < nt)
                    acc[r] = fmaf(wv, ld_el<DT>(p.h, (int64_t) (t0 + r) * W + k), acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < RT; ++r)
    {
        const float sum = wave_sum(acc[r]);
        if (lane == 0 && r < nt)
            z[(int64_t) (t0 + r) * NE + e] = sum;
    }
}

// One wave finishes one token: zr [outputs] holds its logits (LDS) and leaves as scores, cr [outputs] is room for the choice values.
__device__ __forceinline__ void select_token(const StackMoeParams& p, float* zr, float* cr, int lane, int t)
{
    const int NE = p.experts + p.identity;
    if (p.score == ROUTE_SIGMOID)
    {
        // every output's score by itself
        for (int e = lane; e < NE; e += 64)
        {
            const float s = 1.f / (1.f + expf(-zr[e]));
            zr[e] = s;
            cr[e] = s + (p.correction ? p.correction[e] : 0.f);
        }
    }
    else
    {
        float mx = -INFINITY;
        for (int e = lane; e < NE; e += 64)
            mx = fmaxf(mx, zr[e]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int e = lane; e < NE; e += 64)
        {
            const float x = expf(zr[e] - mx);
            zr[e] = x;
            sum += x;
        }
        sum = wave_sum(sum);
        const float inv = 1.f / sum;
        for (int e = lane; e < NE; e += 64)
        {
            const float s = zr[e] * inv;
            zr[e] = s;
            cr[e] = s + (p.correction ? p.correction[e] : 0.f);
        }
    }
    __builtin_amdgcn_wave_barrier();
    const int GC = p.group_count, GS = NE / GC;
    if (GC > 1 && p.group_keep < GC)
    {
        // a group's value: its largest choice value; the group_keep best groups stay, the others' experts cannot be chosen
        float gv[(MAX_OUT + 63) / 64];
        const int per_lane = (GC + 63) / 64;
        for (int i = 0; i < per_lane; ++i)
        {
            const int g = lane + i * 64;
            float m = -INFINITY;
            if (g < GC)
                for (int j = 0; j < GS; ++j)
                    m = fmaxf(m, cr[g * GS + j]);
            gv[i] = m;
        }
        bool kept[(MAX_OUT + 63) / 64];
        for (int i = 0; i < per_lane; ++i)
            kept[i] = false;
        for (int k = 0; k < p.group_keep; ++k)
        {
            float bv = -INFINITY;
            int bi = 0x7fffffff;
            for (int i = 0; i < per_lane; ++i)
            {
                const int g = lane + i * 64;
                if (g < GC && !kept[i] && (gv[i] > bv || (gv[i] == bv && g < bi)))
                {
                    bv = gv[i];
                    bi = g;
                }
            }
            wave_argmax(bv, bi);
            for (int i = 0; i < per_lane; ++i)
                if (lane + i * 64 == bi)
                    kept[i] = true;
        }
        for (int i = 0; i < per_lane; ++i)
        {
            const int g = lane + i * 64;
            if (g < GC && !kept[i])
                for (int j = 0; j < GS; ++j)
                    cr[g * GS + j] = -INFINITY;
        }
        __builtin_amdgcn_wave_barrier();
    }
    for (int k = 0; k < p.top; ++k)
    {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int e = lane; e < NE; e += 64)
        {
            const float c = cr[e];
            if (c > bv || (c == bv && e < bi && c > -INFINITY))
            {
                bv = c;
                bi = e;
            }
        }
        wave_argmax(bv, bi);
        if (bi >= NE) // fewer choosable experts than `top`: the place stays empty (weight 0 on an identity)
            bi = NE - 1, bv = -INFINITY;
        if (lane == 0)
        {
            p.topk_idx[(int64_t) t * p.top + k] = bi;
            p.topk_w[(int64_t) t * p.top + k] = bv == -INFINITY ? 0.f : zr[bi] * p.scale;
            cr[bi] = -INFINITY;
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// One wave per token (4 per workgroup): softmax over the logits, choice values, the kept groups, the top-k among them.
__global__ __launch_bounds__(256) void moe_select_kernel(const StackMoeParams p, const float* zg)
{
    extern __shared__ float sm[];
    const int NE = p.experts + p.identity;
    float* z = sm;              // [4][NE] scores
    float* ch = z + 4 * NE;     // [4][NE] choice values
    const int t0 = blockIdx.x * 4, lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    if (t0 + wid < p.tokens)
        for (int e = lane; e < NE; e += 64)
            z[wid * NE + e] = zg[(int64_t) (t0 + wid) * NE + e];
    __syncthreads();
    const int t = t0 + wid;
    if (t >= p.tokens)
        return;
    select_token(p, z + wid * NE, ch + wid * NE, lane, t);
}

// Few tokens (a step of decoded tokens): one workgroup of 16 waves per token computes its logits (a wave per router row, 16-byte
// pieces) and wave 0 finishes the token, in one launch.
template <int DT>
__global__ __launch_bounds__(1024) void moe_route_few_kernel(const StackMoeParams p)
{
    extern __shared__ float sm[];
    const int NE = p.experts + p.identity, W = p.width, t = blockIdx.x;
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    for (int e = wid; e < NE; e += 16)
    {
        const float* wr = p.router_w + (int64_t) e * W;
        float acc = 0.f;
        if ((W & 7) == 0)
        {
            for (int k = lane * 8; k < W; k += 64 * 8)
            {
                const float4 w0 = *reinterpret_cast<const float4*>(wr + k), w1 = *reinterpret_cast<const float4*>(wr + k + 4);
                const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
                float hv[8];
                if constexpr (DT == DT_BF16)
                {
                    const uint4 u = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.h) + (int64_t) t * W + k);
                    const uint32_t us[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        hv[2 * i] = __builtin_bit_cast(float, us[i] << 16);
                        hv[2 * i + 1] = __builtin_bit_cast(float, us[i] & 0xffff0000u);
                    }
                }
                else
                {
                    const float* hp = reinterpret_cast<const float*>(p.h) + (int64_t) t * W + k;
                    const float4 h0 = *reinterpret_cast<const float4*>(hp), h1 = *reinterpret_cast<const float4*>(hp + 4);
                    hv[0] = h0.x, hv[1] = h0.y, hv[2] = h0.z, hv[3] = h0.w, hv[4] = h1.x, hv[5] = h1.y, hv[6] = h1.z, hv[7] = h1.w;
                }
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    acc = fmaf(wv[i], hv[i], acc);
            }
        }
        else
        {
            for (int k = lane; k < W; k += 64)
                acc = fmaf(wr[k], ld_el<DT>(p.h, (int64_t) t * W + k), acc);
        }
        acc = wave_sum(acc);
        if (lane == 0)
            sm[e] = acc;
    }
    __syncthreads();
    if (wid == 0)
        select_token(p, sm, sm + NE, lane, t);
}

// dst[:] = w * src[:] over one row of the element type (the weight of a pair applied to the expert's input), thread `i` of `n`
__device__ __forceinline__ void scaled_row(const StackMoeParams& p, char* dst, const char* src, float w, int i, int n)
{
    if (p.dtype == DT_BF16)
        for (int c = i; c < p.width; c += n)
            reinterpret_cast<uint16_t*>(dst)[c] = f2bf(w * bf2f(reinterpret_cast<const uint16_t*>(src)[c]));
    else
        for (int c = i; c < p.width; c += n)
            reinterpret_cast<float*>(dst)[c] = w * reinterpret_cast<const float*>(src)[c];
}

// One workgroup: counts per expert, offsets, a slot per pair.  Which of an expert's slots a pair gets depends on the order of the
// atomics; a row's product does not depend on its neighbours in a tile, so the results do not.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const StackMoeParams p, int gather_row_bytes)
{
    extern __shared__ int si[];
    int* cnt = si;                  // [experts]
    int* off = cnt + p.experts;     // [experts + 1]
    const int pairs = p.tokens * p.top, tid = threadIdx.x, NT = blockDim.x;
    for (int e = tid; e < p.experts; e += NT)
        cnt[e] = 0;
    __syncthreads();
    for (int i = tid; i < pairs; i += NT)
    {
        const int e = p.topk_idx[i];
        if (e < p.experts)
            atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (tid == 0)
    {
        int run = 0;
        for (int e = 0; e < p.experts; ++e)
        {
            off[e] = run;
            run += cnt[e];
        }
        off[p.experts] = run;
    }
    __syncthreads();
    for (int e = tid; e <= p.experts; e += NT)
    {
        p.group_off[e] = off[e];
        if (e < p.experts)
            cnt[e] = 0;
    }
    const int used = off[p.experts];
    for (int i = used + tid; i < pairs; i += NT)
        p.pair_of_slot[i] = -1;
    __syncthreads();
    for (int i = tid; i < pairs; i += NT)
    {
        const int e = p.topk_idx[i];
        int slot = -1;
        if (e < p.experts)
        {
            slot = off[e] + atomicAdd(&cnt[e], 1);
            p.pair_of_slot[slot] = i;
        }
        p.slot_of_pair[i] = slot;
    }
    if (gather_row_bytes <= 0)
        return;
    // few pairs: the rows are copied here (a wave per pair) instead of by a launch of their own
    __syncthreads();
    const int lane = tid & 63;
    for (int i = tid >> 6; i < pairs; i += NT >> 6)
    {
        const int slot = p.slot_of_pair[i];
        if (slot < 0)
            continue;
        const char* src = reinterpret_cast<const char*>(p.h) + (int64_t) (i / p.top) * gather_row_bytes;
        char* dst = reinterpret_cast<char*>(p.a_sorted) + (int64_t) slot * gather_row_bytes;
        if (p.weight_input)
            scaled_row(p, dst, src, p.topk_w[i], lane, 64);
        else if ((gather_row_bytes & 15) == 0)
            for (int b = lane * 16; b < gather_row_bytes; b += 64 * 16)
                *reinterpret_cast<uint4*>(dst + b) = *reinterpret_cast<const uint4*>(src + b);
        else
            for (int b = lane * 2; b < gather_row_bytes; b += 64 * 2)
                *reinterpret_cast<uint16_t*>(dst + b) = *reinterpret_cast<const uint16_t*>(src + b);
    }
}

// a_sorted[slot, :] = h[token of the slot's pair, :]; 16 bytes per thread where the rows allow it
__global__ __launch_bounds__(256) void moe_gather_kernel(const StackMoeParams p, int row_bytes)
{
    const int slot = blockIdx.x;
    const int pair = p.pair_of_slot[slot];
    if (pair < 0)
        return;
    const char* src = reinterpret_cast<const char*>(p.h) + (int64_t) (pair / p.top) * row_bytes;
    char* dst = reinterpret_cast<char*>(p.a_sorted) + (int64_t) slot * row_bytes;
    if (p.weight_input)
        scaled_row(p, dst, src, p.topk_w[pair], threadIdx.x, 256);
    else if ((row_bytes & 15) == 0)
    {
        for (int i = threadIdx.x * 16; i < row_bytes; i += 256 * 16)
            *reinterpret_cast<uint4*>(dst + i) = *reinterpret_cast<const uint4*>(src + i);
    }
    else
    {
        for (int i = threadIdx.x * 2; i < row_bytes; i += 256 * 2)
            *reinterpret_cast<uint16_t*>(dst + i) = *reinterpret_cast<const uint16_t*>(src + i);
    }
}

template <int DT>
__global__ __launch_bounds__(256) void moe_combine_kernel(const StackMoeParams p, const float* ys, float* y)
{
    __shared__ int slot_s[MAX_TOP];
    __shared__ float w_s[MAX_TOP];
    const int t = blockIdx.x;
    if ((int) threadIdx.x < p.top)
    {
        slot_s[threadIdx.x] = p.slot_of_pair[(int64_t) t * p.top + threadIdx.x];
        w_s[threadIdx.x] = p.topk_w[(int64_t) t * p.top + threadIdx.x];
    }
    __syncthreads();
    for (int c = threadIdx.x; c < p.width; c += 256)
    {
        float acc = 0.f;
        for (int k = 0; k < p.top; ++k)
        {
            const int slot = slot_s[k];
            const float v = slot >= 0 ? ys[(int64_t) slot * p.width + c] : ld_el<DT>(p.h, (int64_t) t * p.width + c);
            acc = fmaf((p.weight_input && slot >= 0) ? 1.f : w_s[k], v, acc); // an input-weighted expert's output is summed as it is

        }
        y[(int64_t) t * p.width + c] = acc;
    }
}

bool moe_ok(const StackMoeParams& p, const char* what)
{
    if (p.dtype != DT_BF16 && p.dtype != DT_FLOAT)
    {
        set_error("%s: element type %d is not served (bfloat16 or float32)", what, p.dtype);
        return false;
    }
    const int NE = p.experts + p.identity;
    if (p.experts < 1 || p.identity < 0 || NE > MAX_OUT || p.top < 1 || p.top > MAX_TOP || p.top > NE || p.group_count < 1 || NE % p.group_count
        || p.group_keep < 1 || p.group_keep > p.group_count || p.width < 1)
    {
        set_error("%s: %d experts + %d identities in %d groups of which %d are kept, top %d is not a router it serves (at most %d outputs, "
                  "top <= %d, equal groups)",
            what, p.experts, p.identity, p.group_count, p.group_keep, p.top, MAX_OUT, MAX_TOP);
        return false;
    }
    return true;
}

} // namespace

int launch_stack_moe_route(const StackMoeParams& p, hipStream_t stream)
{
    if (p.tokens <= 0)
        return 0;
    if (!moe_ok(p, "stack_moe_route"))
        return -1;
    if (!p.logits)
    {
        set_error("stack_moe_route: no room for the logits");
        return -1;
    }
    const int NE = p.experts + p.identity;
    if (p.tokens <= FEW_TOKENS)
    {
        if (p.dtype == DT_BF16)
            hipLaunchKernelGGL((moe_route_few_kernel<DT_BF16>), dim3(p.tokens), dim3(1024), sizeof(float) * 2 * NE, stream, p);
        else
            hipLaunchKernelGGL((moe_route_few_kernel<DT_FLOAT>), dim3(p.tokens), dim3(1024), sizeof(float) * 2 * NE, stream, p);
        return launched("stack_moe_route (few tokens)");
    }
    const dim3 lg((NE + 3) / 4, (p.tokens + RT - 1) / RT);
    if (p.dtype == DT_BF16)
        hipLaunchKernelGGL((moe_logits_kernel<DT_BF16>), lg, dim3(256), 0, stream, p, p.logits);
    else
        hipLaunchKernelGGL((moe_logits_kernel<DT_FLOAT>), lg, dim3(256), 0, stream, p, p.logits);
    if (launched("stack_moe_logits"))
        return -1;
    hipLaunchKernelGGL(moe_select_kernel, dim3((p.tokens + 3) / 4), dim3(256), sizeof(float) * 2 * 4 * NE, stream, p, p.logits);
    return launched("stack_moe_select");
}

int launch_stack_moe_sort(const StackMoeParams& p, hipStream_t stream)
{
    if (p.tokens <= 0)
        return 0;
    if (!moe_ok(p, "stack_moe_sort"))
        return -1;
    const size_t lds = sizeof(int) * (2 * (size_t) p.experts + 1);
    const int row_bytes = p.width * (p.dtype == DT_BF16 ? 2 : 4);
    const bool few = p.tokens <= FEW_TOKENS;
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), lds, stream, p, few ? row_bytes : 0);
    const int rc = launched("stack_moe_sort");
    if (rc || few)
        return rc;
    hipLaunchKernelGGL(moe_gather_kernel, dim3(p.tokens * p.top), dim3(256), 0, stream, p, row_bytes);
    return launched("stack_moe_gather");
}

int launch_stack_moe_combine(const StackMoeParams& p, const float* y_sorted, float* y, hipStream_t stream)
{
    if (p.tokens <= 0)
        return 0;
    if (!moe_ok(p, "stack_moe_combine"))
        return -1;
    if (p.dtype == DT_BF16)
        hipLaunchKernelGGL((moe_combine_kernel<DT_BF16>), dim3(p.tokens), dim3(256), 0, stream, p, y_sorted, y);
    else
        hipLaunchKernelGGL((moe_combine_kernel<DT_FLOAT>), dim3(p.tokens), dim3(256), 0, stream, p, y_sorted, y);
    return launched("stack_moe_combine");
}

} // namespace kernels
} // namespace tllm
