// Gated delta rule with a decay per key channel, for the ragged-batch stack engine (stack_kernels.h): the recurrence over
// per-sequence state slots and the head norm with its gate behind it.  Unit norms, step sizes, decays, beta, the state and the
// read-out are fp32 in both element types; `DT` is the storage type of the convolution's output and of the layer's output.
#include "dev_utils.h"
#include "launch_util.h"
#include "stack_kernels.h"
#include <algorithm>
#include <cstdlib>

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

// exp(-rate * softplus(z)).  The bfloat16 engine takes the hardware's base-2 exponential and logarithm: their error, relative to
// 1 + e^z, is a few 1e-7 - far below what rounding the activations leaves; the fp32 engine keeps the library's functions.
template <int DT>
__device__ __forceinline__ float decay_of(float rate, float z)
{
    if constexpr (DT == DT_BF16)
    {
        constexpr float LOG2E = 1.4426950408889634f;
        const float sp2 = z > 20.f ? z * LOG2E : __builtin_amdgcn_logf(1.f + __builtin_amdgcn_exp2f(z * LOG2E)); // softplus / ln 2
        return __builtin_amdgcn_exp2f(-rate * sp2);
    }
    else
        return expf(-rate * softplus_f(z));
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
constexpr int DL_RC = 16;

// sum over the DS consecutive lanes (a power of two, <= 64) that hold the slices of one state column; constant distances, so the
// first steps are cross-lane moves inside a row of 16 lanes rather than trips through LDS
__device__ __forceinline__ float slice_sum(float v, int DS)
{
    if (DS > 1)
        v += __shfl_xor(v, 1, 64);
    if (DS > 2)
        v += __shfl_xor(v, 2, 64);
    if (DS > 4)
        v += __shfl_xor(v, 4, 64);
    if (DS > 8)
        v += __shfl_xor(v, 8, 64);
    if (DS > 16)
        v += __shfl_xor(v, 16, 64);
    if (DS > 32)
        v += __shfl_xor(v, 32, 64);
    return v;
}

// One workgroup per (entry, head, group of `cols` value channels).  Thread (vl, s) = tid / DS, tid % DS keeps rows
// [s NSZ, (s + 1) NSZ) of state column S[:, v] in registers.  Per chunk of DL_RC rows: the waves prepare unit q and k, the decay and
// beta of every row into LDS (a wave per row, lanes over the key channels) and every thread requests its column's values of the
// whole chunk; then the recurrence runs row by row without leaving the registers: per row only the slice sum of S^T k sits on the
// chain from one row to the next (four independent partial sums, then log2 DS cross-lane steps); the read-outs S^T q are left as
// per-thread partials in the thread's own LDS slot and summed over the slices once per chunk, off that chain, so nothing goes to
// memory inside the row loop.  A
// head's columns are independent, so a launch with few (entry, head) pairs cuts them over workgroups; the head norm is a pass of
// its own (delta_out_kernel).
template <int DT, int NSZ>
__global__ __launch_bounds__(256) void delta_scan_kernel(const StackDeltaParams p, int DS, int cols, int probe)
{
    extern __shared__ float sm[];
    const int D = p.dim, V = p.vdim;
    const int DP = DS * NSZ;         // a row of the stage holds every slice whole: zeros past dim
    float* qs = sm;                  // [DL_RC][DP]
    float* ks = qs + DL_RC * DP;     // [DL_RC][DP]
    float* gs = ks + DL_RC * DP;     // [DL_RC][DP]
    float* bs = gs + DL_RC * DP;     // [DL_RC]
    float* iqs = bs + DL_RC;         // [DL_RC] 1 / (|q| sqrt(dim)) and 1 / |k| of the chunk's rows
    float* iks = iqs + DL_RC;
    float* vs = iks + DL_RC;         // [DL_RC][threads] every thread's own value / read-out partial of a row: no other thread reads it
    const int NT = blockDim.x;
    const int e = blockIdx.x, h = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6, nwaves = blockDim.x >> 6;
    const int s = tid % DS, vl = tid / DS, v = blockIdx.z * cols + vl;
    const bool live = vl < cols && v < V;
    const int first = p.ent_first[e], count = p.ent_count[e];
    const int hk = h / (p.heads / p.qk_heads);
    const int QK = p.qk_heads * D, CH = 2 * QK + p.heads * V, HD = p.heads * D, HV = p.heads * V;
    float* st = p.state + ((int64_t) p.ent_slot[e] * p.heads + h) * D * V;
    const int d0 = s * NSZ;
    float S[NSZ];
#pragma unroll
    for (int i = 0; i < NSZ; ++i)
        S[i] = (live && d0 + i < D && p.ent_pos0[e] > 0) ? st[(int64_t) (d0 + i) * V + v] : 0.f;
    constexpr int PF = NSZ < 16 ? NSZ : 16; // elements of the stage a thread fetches per pass
    const int dp_shift = __ffs(DP) - 1;     // DP is a power of two
    const float rate = expf(p.a_log[h]);
    const float q_mul = 1.f / sqrtf((float) D);
    // A chunk's inputs - per (row, key channel) q, k and the decay's pre-activation, per row the thread's own value and beta - are
    // fetched into registers with every load in flight at once, and land in the stage behind a barrier.  Every load is unconditional,
    // at an index clamped into the chunk: a load under a condition would sit in a block of its own with its wait, and the chunk
    // would pay one memory latency per element instead of one per pass.  Where one pass holds a whole chunk (the usual case), the
    // next chunk is fetched while this one is scanned.
    float rq[PF], rk[PF], ra[PF], rv[DL_RC], rb = 0.f;
    const int vc = v < V ? v : V - 1;
    auto fetch = [&](int r0f, int nrf, int base) {
#pragma unroll
        for (int j = 0; j < PF; ++j)
        {
            const int el = base + j * NT + tid, r = min(el >> dp_shift, nrf - 1), d = min(el & (DP - 1), D - 1);
            const int64_t t = first + r0f + r;
            rq[j] = ld_el<DT>(p.x, t * CH + hk * D + d);
            rk[j] = ld_el<DT>(p.x, t * CH + QK + hk * D + d);
            ra[j] = p.decay_raw[t * HD + h * D + d] + p.dt_bias[h * D + d];
        }
        if (base == 0)
        {
#pragma unroll
            for (int r = 0; r < DL_RC; ++r)
                rv[r] = ld_el<DT>(p.x, (int64_t) (first + r0f + min(r, nrf - 1)) * CH + 2 * QK + h * V + vc);
            rb = ld_el<DT>(p.beta_raw, (int64_t) (first + r0f + min(tid, nrf - 1)) * p.ld_beta + h);
        }
    };
    auto land = [&](int nrf, int base) {
#pragma unroll
        for (int j = 0; j < PF; ++j)
        {
            const int el = base + j * NT + tid;
            if (el < nrf * DP)
            {
                const bool in = (el & (DP - 1)) < D;
                qs[el] = in ? rq[j] : 0.f;
                ks[el] = in ? rk[j] : 0.f;
                gs[el] = in ? ((probe & 2) ? ra[j] : decay_of<DT>(rate, ra[j])) : 0.f;
            }
        }
        if (base == 0)
        {
#pragma unroll
            for (int r = 0; r < DL_RC; ++r)
                vs[r * NT + tid] = live ? rv[r] : 0.f;
            if (tid < nrf)
                bs[tid] = 1.f / (1.f + expf(-rb));
        }
    };
    const bool one_pass = DL_RC * DP <= NT * PF && NT >= DL_RC; // uniform
    if (one_pass && count > 0)
        fetch(0, count < DL_RC ? count : DL_RC, 0);
    for (int r0 = 0; r0 < count; r0 += DL_RC)
    {
        const int nr = count - r0 < DL_RC ? count - r0 : DL_RC;
        __syncthreads(); // the chunk before this one has been read
        if (one_pass)
            land(nr, 0);
        else
            for (int base = 0; base < nr * DP; base += NT * PF)
            {
                fetch(r0, nr, base);
                land(nr, base);
            }
        __syncthreads();
        if (one_pass && r0 + DL_RC < count)
            fetch(r0 + DL_RC, count - r0 - DL_RC < DL_RC ? count - r0 - DL_RC : DL_RC, 0);
        // q and k stay as projected in the stage; their unit-norm factors are applied to the sums they enter
        for (int r = wid; r < ((probe & 4) ? 0 : nr); r += nwaves)
        {
            float sq = 0.f, sk = 0.f;
            for (int d = lane; d < D; d += 64)
            {
                sq = fmaf(qs[r * DP + d], qs[r * DP + d], sq);
                sk = fmaf(ks[r * DP + d], ks[r * DP + d], sk);
            }
            sq = wave_sum(sq);
            sk = wave_sum(sk);
            if (lane == 0)
            {
                iqs[r] = q_mul / sqrtf(sq + 1e-6f);
                iks[r] = 1.f / sqrtf(sk + 1e-6f);
            }
        }
        __syncthreads();
        for (int r = 0; r < ((probe & 1) ? 0 : nr); ++r)
        {
            {
                // rows of the stage past dim hold zeros and the state rows there stay zero: no guard inside the slices
                const float* gr = gs + r * DP + d0;
                const float* kr = ks + r * DP + d0;
                const float* qr = qs + r * DP + d0;
                float part[4] = {0.f, 0.f, 0.f, 0.f};
                {
#pragma unroll
                    for (int i = 0; i < NSZ; i += 4)
                    {
                        const float4 g4 = *reinterpret_cast<const float4*>(gr + i), k4 = *reinterpret_cast<const float4*>(kr + i);
                        S[i] *= g4.x;
                        S[i + 1] *= g4.y;
                        S[i + 2] *= g4.z;
                        S[i + 3] *= g4.w;
                        part[0] = fmaf(S[i], k4.x, part[0]);
                        part[1] = fmaf(S[i + 1], k4.y, part[1]);
                        part[2] = fmaf(S[i + 2], k4.z, part[2]);
                        part[3] = fmaf(S[i + 3], k4.w, part[3]);
                    }
                }
                const float dot = slice_sum((part[0] + part[1]) + (part[2] + part[3]), DS) * iks[r];
                const float u = bs[r] * (vs[r * NT + tid] - dot) * iks[r]; // times the key's norm factor: S += k_hat u = k (u / |k|)
                float op[4] = {0.f, 0.f, 0.f, 0.f};
                {
#pragma unroll
                    for (int i = 0; i < NSZ; i += 4)
                    {
                        const float4 k4 = *reinterpret_cast<const float4*>(kr + i), q4 = *reinterpret_cast<const float4*>(qr + i);
                        S[i] = fmaf(k4.x, u, S[i]);
                        S[i + 1] = fmaf(k4.y, u, S[i + 1]);
                        S[i + 2] = fmaf(k4.z, u, S[i + 2]);
                        S[i + 3] = fmaf(k4.w, u, S[i + 3]);
                        op[0] = fmaf(S[i], q4.x, op[0]);
                        op[1] = fmaf(S[i + 1], q4.y, op[1]);
                        op[2] = fmaf(S[i + 2], q4.z, op[2]);
                        op[3] = fmaf(S[i + 3], q4.w, op[3]);
                    }
                }
                vs[r * NT + tid] = ((op[0] + op[1]) + (op[2] + op[3])) * iqs[r];
            }
        }
        for (int r = 0; r < nr; ++r)
        {
            const float o = slice_sum(vs[r * NT + tid], DS);
            if (live && s == 0)
                p.o32[(int64_t) (first + r0 + r) * HV + h * V + v] = o;
        }
    }
    if (live)
    {
#pragma unroll
        for (int i = 0; i < NSZ; ++i)
            if (d0 + i < D)
                st[(int64_t) (d0 + i) * V + v] = S[i];
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
    // up to 16 slices with the fewest rows per thread that allow it (measured at dim 128: 8 rows x 16 slices beat 32 x 4 - the time
    // of a row is the thread's own instructions, not the four cross-lane steps), else 32 rows per thread and up to a wave of slices
    for (int limit : {16, 64})
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
    // columns per workgroup: four waves' worth (a wave per SIMD, and the chunk's rows are prepared once for all of them), fewer
    // while the launch would leave most of the chip idle
    int cols = std::min(p.vdim, std::max(256 / sh.ds, 1));
    const int cus = launch_util::device_cus();
    while (cols * sh.ds > 128 && (int64_t) p.entries * p.heads * ((p.vdim + cols - 1) / cols) * 2 <= cus)
        cols = (cols + 1) / 2;
    const int threads = (cols * sh.ds + 63) / 64 * 64; // at most 256: cols * slices <= 256, or one column of up to 64 slices
    const dim3 grid(p.entries, p.heads, (p.vdim + cols - 1) / cols);
    // measurement knob, bits: 1 = no recurrence, 2 = decays without their exponentials, 4 = no unit norms (what is left is the
    // chunk's traffic and barriers); results are wrong with any of them
    const char* pv = std::getenv("TLLM_STACK_DELTA_PROBE");
    const int probe = pv ? std::atoi(pv) : 0;
    const size_t lds = sizeof(float) * ((size_t) 3 * DL_RC * sh.ds * sh.nsz + 3 * DL_RC + (size_t) DL_RC * threads);
    switch (sh.nsz)
    {
    case 8: hipLaunchKernelGGL((delta_scan_kernel<DT, 8>), grid, dim3(threads), lds, stream, p, sh.ds, cols, probe); break;
    case 16: hipLaunchKernelGGL((delta_scan_kernel<DT, 16>), grid, dim3(threads), lds, stream, p, sh.ds, cols, probe); break;
    default:
        launch_util::ensure_dynamic_lds(reinterpret_cast<const void*>(&delta_scan_kernel<DT, 32>), 120 * 1024); // raised once, for the largest dim
        hipLaunchKernelGGL((delta_scan_kernel<DT, 32>), grid, dim3(threads), lds, stream, p, sh.ds, cols, probe);
        break;
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
        set_error("%s: heads %d over %d q/k heads, dim %d, vdim %d is not a shape it serves (heads a multiple of the q/k heads, dim <= 512)",
            what, p.heads, p.qk_heads, p.dim, p.vdim);
        return false;
    }
    return true;
}

} // namespace

bool stack_delta_serves(int32_t dim, int32_t vdim)
{
    return dim >= 1 && vdim >= 1 && dim <= 512 && delta_shape(dim, vdim).nsz > 0; // 16 staged rows of q, k and the decay within 128 KiB of LDS
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
