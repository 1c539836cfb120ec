// Gated delta rule with a decay per key channel, for the ragged-batch stack engine (stack_kernels.h): the recurrence over
// per-sequence state slots and the head norm with its gate behind it.  Unit norms, step sizes, decays, beta, the state and the
// read-out are fp32 in both element types; `DT` is the storage type of the convolution's output and of the layer's output.
#include "dev_utils.h"
#include "launch_util.h"
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
template <int DT>
__device__ __forceinline__ void st_el(void* p, int64_t i, float v)
{
    if constexpr (DT == DT_BF16)
        reinterpret_cast<uint16_t*>(p)[i] = f2bf(v);
    else
        reinterpret_cast<float*>(p)[i] = v;
}

__device__ __forceinline__ float softplus_f(float z)
{
    return z > 20.f ? z : log1pf(expf(z));
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

// rows of a chunk: their q, k and decay vectors are prepared together, then every thread walks them in order
constexpr int DL_RC = 8;

// sum over the DS consecutive lanes (a power of two, <= 64) that hold the slices of one state column
__device__ __forceinline__ float slice_sum(float v, int DS)
{
    for (int o = 1; o < DS; o <<= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}

// One workgroup per (entry, head, group of `cols` value channels).  Thread (vl, s) = tid / DS, tid % DS keeps rows
// [s NSZ, (s + 1) NSZ) of state column S[:, v] in registers.  Per chunk of DL_RC rows: the waves prepare unit q and k, the decay and
// beta of every row into LDS (a wave per row, lanes over the key channels); then the recurrence runs row by row without leaving
// the registers but for two slice sums (the column's S^T k and S^T q).  A head's columns are independent, so a launch with few
// (entry, head) pairs cuts them over workgroups; the head norm is a pass of its own (delta_out_kernel).
template <int DT, int NSZ>
__global__ __launch_bounds__(1024) void delta_scan_kernel(const StackDeltaParams p, int DS, int cols)
{
    extern __shared__ float sm[];
    const int D = p.dim, V = p.vdim;
    float* qs = sm;                  // [DL_RC][D]
    float* ks = qs + DL_RC * D;      // [DL_RC][D]
    float* gs = ks + DL_RC * D;      // [DL_RC][D]
    float* bs = gs + DL_RC * D;      // [DL_RC]
    const int e = blockIdx.x, h = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6, nwaves = blockDim.x >> 6;
    const int s = tid % DS, vl = tid / DS, v = blockIdx.z * cols + vl;
    const bool live = vl < cols && v < V;
    const int first = p.ent_first[e], count = p.ent_count[e];
    const int hk = h / (p.heads / p.qk_heads);
    const int QK = p.qk_heads * D, CH = 2 * QK + p.heads * V, HD = p.heads * D, HV = p.heads * V;
    float* st = p.state + ((int64_t) p.ent_slot[e] * p.heads + h) * D * V;
    float S[NSZ];
#pragma unroll
    for (int i = 0; i < NSZ; ++i)
    {
        const int d = s * NSZ + i;
        S[i] = (live && d < D && p.ent_pos0[e] > 0) ? st[(int64_t) d * V + v] : 0.f;
    }
    const float rate = expf(p.a_log[h]);
    const float q_mul = 1.f / sqrtf((float) D);
    for (int r0 = 0; r0 < count; r0 += DL_RC)
    {
        const int nr = count - r0 < DL_RC ? count - r0 : DL_RC;
        __syncthreads(); // the chunk before this one has been read
        for (int r = wid; r < nr; r += nwaves)
        {
            const int64_t t = first + r0 + r;
            float sq = 0.f, sk = 0.f;
            for (int d = lane; d < D; d += 64)
            {
                const float qv = ld_el<DT>(p.x, t * CH + hk * D + d), kv = ld_el<DT>(p.x, t * CH + QK + hk * D + d);
                sq += qv * qv;
                sk += kv * kv;
            }
            const float iq = q_mul / sqrtf(wave_sum(sq) + 1e-6f), ik = 1.f / sqrtf(wave_sum(sk) + 1e-6f);
            for (int d = lane; d < D; d += 64)
            {
                qs[r * D + d] = ld_el<DT>(p.x, t * CH + hk * D + d) * iq;
                ks[r * D + d] = ld_el<DT>(p.x, t * CH + QK + hk * D + d) * ik;
                gs[r * D + d] = expf(-rate * softplus_f(p.decay_raw[t * HD + h * D + d] + p.dt_bias[h * D + d]));
            }
            if (lane == 0)
                bs[r] = 1.f / (1.f + expf(-ld_el<DT>(p.beta_raw, t * p.ld_beta + h)));
        }
        __syncthreads();
        for (int r = 0; r < nr; ++r)
        {
            const int64_t t = first + r0 + r;
            const float vv = live ? ld_el<DT>(p.x, t * CH + 2 * QK + h * V + v) : 0.f;
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < NSZ; ++i)
            {
                const int d = s * NSZ + i;
                if (d < D)
                {
                    S[i] *= gs[r * D + d];
                    dot = fmaf(S[i], ks[r * D + d], dot);
                }
            }
            dot = slice_sum(dot, DS);
            const float u = bs[r] * (vv - dot);
            float o = 0.f;
#pragma unroll
            for (int i = 0; i < NSZ; ++i)
            {
                const int d = s * NSZ + i;
                if (d < D)
                {
                    S[i] = fmaf(ks[r * D + d], u, S[i]);
                    o = fmaf(S[i], qs[r * D + d], o);
                }
            }
            o = slice_sum(o, DS);
            if (live && s == 0)
                p.o32[t * HV + h * V + v] = o;
        }
    }
    if (live)
    {
#pragma unroll
        for (int i = 0; i < NSZ; ++i)
        {
            const int d = s * NSZ + i;
            if (d < D)
                st[(int64_t) d * V + v] = S[i];
        }
    }
}

// out[t, h, :] = o / sqrt(mean(o^2) + eps) * norm_w * sigmoid(gate_raw[t, h, :]); one wave per (row, head)
template <int DT>
__global__ __launch_bounds__(256) void delta_out_kernel(const StackDeltaParams p)
{
    const int64_t i = (int64_t) blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, V = p.vdim;
    if (i >= (int64_t) p.tokens * p.heads)
        return;
    const float* o = p.o32 + i * V;
    float ss = 0.f;
    for (int c = lane; c < V; c += 64)
        ss += o[c] * o[c];
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float) V + p.eps);
    for (int c = lane; c < V; c += 64)
    {
        const float g = 1.f / (1.f + expf(-p.gate_raw[i * V + c]));
        st_el<DT>(p.out, i * V + c, o[c] * inv * p.norm_w[c] * g);
    }
}

// slices per state column and rows per slice for a shape: the fewest rows per thread that still fit a workgroup
struct DeltaShape
{
    int nsz = 0, ds = 0;
};
DeltaShape delta_shape(int dim, int vdim)
{
    (void) vdim;
    DeltaShape r;
    for (int limit : {16, 64}) // up to 16 slices where 32 rows per thread allow it (four shuffle steps per sum), else up to a wave
        for (int nsz : {8, 16, 32})
        {
            int ds = 1;
            while (ds * nsz < dim)
                ds <<= 1;
            if (ds <= limit && r.nsz == 0)
                r.nsz = nsz, r.ds = ds;
        }
    return r;
}

template <int DT>
int launch_scan(const StackDeltaParams& p, hipStream_t stream)
{
    const DeltaShape sh = delta_shape(p.dim, p.vdim);
    // columns per workgroup: the whole head, or fewer while the launch would leave most of the chip idle
    int cols = std::min(p.vdim, 1024 / sh.ds);
    const int cus = launch_util::device_cus();
    while (cols > 16 && (int64_t) p.entries * p.heads * ((p.vdim + cols - 1) / cols) < cus && (cols / 2) * sh.ds >= 64)
        cols = (cols + 1) / 2;
    const int threads = std::min(1024, (cols * sh.ds + 63) / 64 * 64);
    const dim3 grid(p.entries, p.heads, (p.vdim + cols - 1) / cols);
    const size_t lds = sizeof(float) * ((size_t) 3 * DL_RC * p.dim + DL_RC);
    switch (sh.nsz)
    {
    case 8: hipLaunchKernelGGL((delta_scan_kernel<DT, 8>), grid, dim3(threads), lds, stream, p, sh.ds, cols); break;
    case 16: hipLaunchKernelGGL((delta_scan_kernel<DT, 16>), grid, dim3(threads), lds, stream, p, sh.ds, cols); break;
    default: hipLaunchKernelGGL((delta_scan_kernel<DT, 32>), grid, dim3(threads), lds, stream, p, sh.ds, cols); break;
    }
    return launched("stack_delta_scan");
}

bool delta_ok(const StackDeltaParams& p, const char* what)
{
    if (p.dtype != DT_BF16 && p.dtype != DT_FLOAT)
    {
        set_error("%s: element type %d is not served (bfloat16 or float32)", what, p.dtype);
        return false;
    }
    if (p.heads < 1 || p.qk_heads < 1 || p.heads % p.qk_heads || !stack_delta_serves(p.dim, p.vdim))
    {
        set_error("%s: heads %d over %d q/k heads, dim %d, vdim %d is not a shape it serves (heads a multiple of the q/k heads, dim <= 2048)",
            what, p.heads, p.qk_heads, p.dim, p.vdim);
        return false;
    }
    return true;
}

} // namespace

bool stack_delta_serves(int32_t dim, int32_t vdim)
{
    return dim >= 1 && vdim >= 1 && dim <= 2048 && delta_shape(dim, vdim).nsz > 0;
}

int launch_stack_delta_scan(const StackDeltaParams& p, hipStream_t stream)
{
    if (p.tokens <= 0 || p.entries <= 0)
        return 0;
    if (!delta_ok(p, "stack_delta_scan"))
        return -1;
    if (!p.x || !p.beta_raw || !p.decay_raw || !p.dt_bias || !p.a_log || !p.state || !p.o32 || !p.ent_slot || !p.ent_first || !p.ent_count
        || !p.ent_pos0)
    {
        set_error("stack_delta_scan: a missing operand");
        return -1;
    }
    return p.dtype == DT_BF16 ? launch_scan<DT_BF16>(p, stream) : launch_scan<DT_FLOAT>(p, stream);
}

int launch_stack_delta_out(const StackDeltaParams& p, hipStream_t stream)
{
    if (p.tokens <= 0)
        return 0;
    if (!delta_ok(p, "stack_delta_out"))
        return -1;
    if (!p.o32 || !p.gate_raw || !p.norm_w || !p.out)
    {
        set_error("stack_delta_out: a missing operand");
        return -1;
    }
    const int64_t vecs = (int64_t) p.tokens * p.heads;
    const dim3 grid((unsigned) ((vecs + 3) / 4));
    if (p.dtype == DT_BF16)
        hipLaunchKernelGGL((delta_out_kernel<DT_BF16>), grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((delta_out_kernel<DT_FLOAT>), grid, dim3(256), 0, stream, p);
    return launched("stack_delta_out");
}

} // namespace kernels
} // namespace tllm
