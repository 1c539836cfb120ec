// Selective state-space layer (Mamba-2) of the ragged-batch stack engine (stack_kernels.h): the short causal convolution with
// its per-sequence tail, and the recurrence over per-sequence state slots.  Step sizes, decays, the state and everything that
// enters the recurrence are fp32 in both element types; `DT` is the storage type of the projection and of the convolution's output.
#include "dev_utils.h"
#include "launch_util.h"
#include "stack_kernels.h"
#include <algorithm>
#include <cstdlib>
#include <type_traits>

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

__device__ __forceinline__ float silu_f(float z)
{
    return z / (1.f + expf(-z));
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

constexpr int MAX_TAPS = 16;

// Workgroups [0, tokens): row t, 256 channels each (blockIdx.y): rows that lie at least taps - 1 tokens into their entry read
// nothing but the step's own projection rows.  Workgroups [tokens, tokens + entries): the first taps - 1 rows of an entry, which
// reach into the sequence's tail of raw inputs, and the new tail - one thread per (entry, channel) reads the old tail before it
// writes, so the launch has no ordering between workgroups to keep.
template <int DT>
__global__ __launch_bounds__(256) void ssm_conv_kernel(const StackSsmParams p)
{
    const int inner = p.heads * p.vdim, CH = p.conv_channels > 0 ? p.conv_channels : inner + 2 * p.groups * p.state, K = p.taps;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= CH)
        return;
    const float* w = p.conv_w + (int64_t) c * K;
    const float bias = p.conv_b ? p.conv_b[c] : 0.f;
    const int64_t col = (p.conv_channels > 0 ? p.conv_col : inner) + c; // mamba2: the convolution's inputs sit behind the z columns
    if ((int) blockIdx.x < p.tokens)
    {
        const int t = blockIdx.x, e = p.tok_entry[t];
        const int i = p.tok_pos[t] - p.ent_pos0[e];
        if (i < K - 1)
            return;
        float acc = bias;
        for (int k = 0; k < K; ++k)
            acc = fmaf(w[k], ld_el<DT>(p.proj, (int64_t) (t - (K - 1) + k) * p.ldp + col), acc);
        st_el<DT>(p.xbc, (int64_t) t * CH + c, silu_f(acc));
        return;
    }
    const int e = blockIdx.x - p.tokens;
    const int first = p.ent_first[e], count = p.ent_count[e];
    float* tail = p.conv_state + (int64_t) p.ent_slot[e] * (K - 1) * CH + c;
    float old[MAX_TAPS - 1];
#pragma unroll
    for (int j = 0; j < MAX_TAPS - 1; ++j)
        old[j] = (j < K - 1 && p.ent_pos0[e] > 0) ? tail[(int64_t) j * CH] : 0.f;
    // input at index i of the entry (negative: the tail; old[K - 1 + i])
    auto input = [&](int i) -> float {
        if (i >= 0)
            return ld_el<DT>(p.proj, (int64_t) (first + i) * p.ldp + col);
        float v = 0.f;
#pragma unroll
        for (int j = 0; j < MAX_TAPS - 1; ++j)
            v = (j == K - 1 + i) ? old[j] : v;
        return v;
    };
    const int head = count < K - 1 ? count : K - 1;
    for (int i = 0; i < head; ++i)
    {
        float acc = bias;
        for (int k = 0; k < K; ++k)
            acc = fmaf(w[k], input(i - (K - 1) + k), acc);
        st_el<DT>(p.xbc, (int64_t) (first + i) * CH + c, silu_f(acc));
    }
    for (int j = 0; j < K - 1; ++j)
        tail[(int64_t) j * CH] = input(count - (K - 1) + j);
}

// One workgroup per (entry, head): thread (s, v) keeps rows [s NSZ, (s + 1) NSZ) of state column S[:, v] in registers.  Rows go
// through in chunks of RC: the chunk's decays, dt B, C and x are staged in LDS once, the recurrence runs without cross-lane
// traffic, the NS partial outputs of a row meet in LDS once per chunk, where the skip term and the gate are applied.
constexpr int RC = 8;

template <int DT, int NSZ>
__global__ __launch_bounds__(1024) void ssm_scan_kernel(const StackSsmParams p, int NS)
{
    extern __shared__ float sm[];
    const int P = p.vdim, N = p.state, H = p.heads, G = p.groups;
    const int inner = H * P, GN = G * N, CH = inner + 2 * GN;
    float* dec = sm;                 // [RC] decay of the row
    float* kb = dec + RC;            // [RC][N] dt * B
    float* cc = kb + RC * N;         // [RC][N] C
    float* xs = cc + RC * N;         // [RC][P]
    float* os = xs + RC * P;         // [RC][NS][P]
    const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, NT = blockDim.x;
    const int g = h / (H / G);
    const int s = tid / P, v = tid % P;
    const bool live = s < NS;
    const int n0 = s * NSZ;
    const int first = p.ent_first[e], count = p.ent_count[e];
    float* sp = p.ssm_state + (((int64_t) p.ent_slot[e] * H + h) * N) * P + v;
    const bool carry = p.ent_pos0[e] > 0;
    float S[NSZ];
#pragma unroll
    for (int j = 0; j < NSZ; ++j)
        S[j] = (live && n0 + j < N && carry) ? sp[(int64_t) (n0 + j) * P] : 0.f;
    const float rate = -expf(p.a_log[h]), dtb = p.dt_bias[h], dsk = p.d_skip[h];
    for (int t0 = 0; t0 < count; t0 += RC)
    {
        const int nt = count - t0 < RC ? count - t0 : RC;
        for (int i = tid; i < nt * N; i += NT)
        {
            const int tt = i / N, n = i % N;
            const int64_t r = first + t0 + tt;
            const float z = ld_el<DT>(p.proj, r * p.ldp + 2 * inner + 2 * GN + h) + dtb;
            const float dt = z > 20.f ? z : log1pf(expf(z));
            kb[tt * N + n] = dt * ld_el<DT>(p.xbc, r * CH + inner + g * N + n);
            cc[tt * N + n] = ld_el<DT>(p.xbc, r * CH + inner + GN + g * N + n);
            if (n == 0)
                dec[tt] = expf(rate * dt);
        }
        for (int i = tid; i < nt * P; i += NT)
            xs[i] = ld_el<DT>(p.xbc, (int64_t) (first + t0 + i / P) * CH + h * P + i % P);
        __syncthreads();
        if (live)
        {
            for (int tt = 0; tt < nt; ++tt)
            {
                const float x = xs[tt * P + v], a = dec[tt];
                float o = 0.f;
#pragma unroll
                for (int j = 0; j < NSZ; ++j)
                {
                    if (n0 + j < N)
                    {
                        S[j] = fmaf(a, S[j], kb[tt * N + n0 + j] * x);
                        o = fmaf(S[j], cc[tt * N + n0 + j], o);
                    }
                }
                os[(tt * NS + s) * P + v] = o;
            }
        }
        __syncthreads();
        for (int i = tid; i < nt * P; i += NT)
        {
            const int tt = i / P, c = i % P;
            const int64_t r = first + t0 + tt;
            float y = 0.f;
            for (int s2 = 0; s2 < NS; ++s2)
                y += os[(tt * NS + s2) * P + c];
            y = fmaf(dsk, xs[i], y);
            p.y32[r * inner + h * P + c] = y * silu_f(ld_el<DT>(p.proj, r * p.ldp + h * P + c));
        }
        __syncthreads();
    }
    if (live)
    {
#pragma unroll
        for (int j = 0; j < NSZ; ++j)
            if (n0 + j < N)
                sp[(int64_t) (n0 + j) * P] = S[j];
    }
}

// The pipelined form of the same walk, for shapes whose chunk fits KMAX values per thread: the raw B, C, x, z and dt of chunk c + 1
// are requested into registers before the recurrence of chunk c starts and land in the other half of a double-buffered LDS stage,
// so a chunk waits for memory only at the start of an entry and has two barriers; step size and decay are computed once per row,
// and the step size meets x (one product per thread and row) instead of every element of B.
constexpr int KMAX = 8;
constexpr size_t kMaxLds = 128 * 1024; // of a CU's 160 KiB

template <int DT, int NSZ>
__global__ __launch_bounds__(1024) void ssm_scan_pipe_kernel(const StackSsmParams p, int NS, int rc, int P)
{
    extern __shared__ float sm[];
    // P: the columns of the head this workgroup keeps, [blockIdx.z P, + P) of its PH
    const int PH = p.vdim, N = p.state, H = p.heads, G = p.groups, c0 = blockIdx.z * P;
    const int inner = H * PH, GN = G * N, CH = inner + 2 * GN;
    const int stage = rc * (2 + 2 * N + 2 * P);
    float* os = sm + 2 * stage;      // [rc][NS][P]
    const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, NT = blockDim.x;
    const int g = h / (H / G);
    const int s = tid / P, v = tid % P;
    const bool live = s < NS && c0 + v < PH;
    const int n0 = s * NSZ;
    const int first = p.ent_first[e], count = p.ent_count[e];
    float* sp = p.ssm_state + (((int64_t) p.ent_slot[e] * H + h) * N) * PH + c0 + v;
    const bool carry = p.ent_pos0[e] > 0;
    float S[NSZ];
#pragma unroll
    for (int j = 0; j < NSZ; ++j)
        S[j] = (live && n0 + j < N && carry) ? sp[(int64_t) (n0 + j) * PH] : 0.f;
    const float rate = -expf(p.a_log[h]), dtb = p.dt_bias[h], dsk = p.d_skip[h];
    const bool vec4 = (N % NSZ) == 0 && (N & 3) == 0 && (P & 1) == 0; // (every LDS region then starts on 16 bytes)
    // requested values stay raw bits until they are staged: a conversion next to its load would make the wave wait for it there
    typedef typename std::conditional<DT == DT_BF16, uint16_t, float>::type Raw;
    auto cvt = [](Raw r) -> float {
        if constexpr (DT == DT_BF16)
            return bf2f(r);
        else
            return r;
    };
    const Raw* xbc = reinterpret_cast<const Raw*>(p.xbc);
    const Raw* prj = reinterpret_cast<const Raw*>(p.proj);
    Raw rb[KMAX], rcv[KMAX], rx[KMAX], rz[KMAX], rdt = 0;
    // element i = tid + k NT of a [rows, N] (or [rows, P]) chunk is (row, column) = (i / N, i % N): stepped, not divided, per k
    const int qN = NT / N, mN = NT % N, qP = NT / P, mP = NT % P, rowN0 = tid / N, colN0 = tid % N;
    const int kN = (rc * N + NT - 1) / NT, kP = (rc * P + NT - 1) / NT; // values per thread and chunk (<= KMAX)
    auto request = [&](int t0) {
        const int nt = count - t0 < rc ? count - t0 : rc;
        int rowN = rowN0, colN = colN0, rowP = s, colP = v;
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
        {
            // every lane loads from a row of the chunk (clamped), so that nothing branches around a load
            if (k < kN)
            {
                const int64_t r = first + t0 + (rowN < nt ? rowN : nt - 1);
                rb[k] = xbc[r * CH + inner + g * N + colN];
                rcv[k] = xbc[r * CH + inner + GN + g * N + colN];
            }
            if (k < kP)
            {
                const int64_t r = first + t0 + (rowP < nt ? rowP : nt - 1);
                const int col = c0 + colP < PH ? c0 + colP : PH - 1;
                rx[k] = xbc[r * CH + h * PH + col];
                rz[k] = prj[r * p.ldp + h * PH + col];
            }
            rowN += qN, colN += mN;
            if (colN >= N)
                colN -= N, ++rowN;
            rowP += qP, colP += mP;
            if (colP >= P)
                colP -= P, ++rowP;
        }
        rdt = prj[(int64_t) (first + t0 + (tid < nt ? tid : nt - 1)) * p.ldp + 2 * inner + 2 * GN + h];
    };
    request(0);
    int buf = 0;
    for (int t0 = 0; t0 < count; t0 += rc, buf ^= 1)
    {
        const int nt = count - t0 < rc ? count - t0 : rc;
        float* dd = sm + buf * stage;    // [rc][2] decay, step size
        float* bs = dd + 2 * rc;         // [rc][N]
        float* cs = bs + rc * N;         // [rc][N]
        float* xs = cs + rc * N;         // [rc][P]
        float* zs = xs + rc * P;         // [rc][P]
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
        {
            const int i = tid + k * NT;
            if (i < nt * N)
            {
                bs[i] = cvt(rb[k]);
                cs[i] = cvt(rcv[k]);
            }
            if (i < nt * P)
            {
                xs[i] = cvt(rx[k]);
                zs[i] = cvt(rz[k]);
            }
            if (i >= rc * N && i >= rc * P)
                break;
        }
        if (tid < nt)
        {
            const float z = cvt(rdt) + dtb;
            const float dt = z > 20.f ? z : log1pf(expf(z));
            dd[2 * tid] = expf(rate * dt);
            dd[2 * tid + 1] = dt;
        }
        __syncthreads();
        if (t0 + rc < count)
            request(t0 + rc); // in flight under this chunk's recurrence
        if (live)
        {
            for (int tt = 0; tt < nt; ++tt)
            {
                const float a = dd[2 * tt], xd = xs[tt * P + v] * dd[2 * tt + 1];
                const float* bt = bs + tt * N + n0;
                const float* ct = cs + tt * N + n0;
                float o = 0.f;
                if (vec4)
                {
                    // rows of B and C are 16-byte aligned and the slice is whole: four values per LDS read
#pragma unroll
                    for (int j = 0; j < NSZ; j += 4)
                    {
                        const float4 b4 = *reinterpret_cast<const float4*>(bt + j), c4 = *reinterpret_cast<const float4*>(ct + j);
                        S[j] = fmaf(a, S[j], b4.x * xd);
                        S[j + 1] = fmaf(a, S[j + 1], b4.y * xd);
                        S[j + 2] = fmaf(a, S[j + 2], b4.z * xd);
                        S[j + 3] = fmaf(a, S[j + 3], b4.w * xd);
                        o = fmaf(S[j], c4.x, o);
                        o = fmaf(S[j + 1], c4.y, o);
                        o = fmaf(S[j + 2], c4.z, o);
                        o = fmaf(S[j + 3], c4.w, o);
                    }
                }
                else
                {
#pragma unroll
                    for (int j = 0; j < NSZ; ++j)
                    {
                        if (n0 + j < N)
                        {
                            S[j] = fmaf(a, S[j], bt[j] * xd);
                            o = fmaf(S[j], ct[j], o);
                        }
                    }
                }
                os[(tt * NS + s) * P + v] = o;
            }
        }
        __syncthreads();
        for (int i = tid, tt = s, c = v; i < nt * P; i += NT)
        {
            float y = 0.f;
            for (int s2 = 0; s2 < NS; ++s2)
                y += os[(tt * NS + s2) * P + c];
            y = fmaf(dsk, xs[i], y);
            if (c0 + c < PH)
                p.y32[(int64_t) (first + t0 + tt) * inner + h * PH + c0 + c] = y * silu_f(zs[i]);
            tt += qP, c += mP;
            if (c >= P)
                c -= P, ++tt;
        }
        // (the next chunk stages into the other buffer; os is written again only behind the next chunk's first barrier, which no
        // thread passes before it has finished these sums)
    }
    if (live)
    {
#pragma unroll
        for (int j = 0; j < NSZ; ++j)
            if (n0 + j < N)
                sp[(int64_t) (n0 + j) * PH] = S[j];
    }
}

// rows of state a thread keeps, for a head of P columns and N rows: the fewest that fit the workgroup, at least 4
inline int slice_rows(int P, int N)
{
    for (int limit : {512, 1024})
        for (int nsz : {4, 8, 16, 32})
            if ((int64_t) ((N + nsz - 1) / nsz) * P <= limit)
                return nsz;
    return 0;
}

} // namespace

bool stack_ssm_serves(int32_t vdim, int32_t state, int32_t taps)
{
    return vdim >= 1 && state >= 1 && taps >= 1 && taps <= MAX_TAPS && slice_rows(vdim, state) > 0;
}

static bool ssm_ok(const StackSsmParams& p, const char* what)
{
    if (p.dtype != DT_BF16 && p.dtype != DT_FLOAT)
    {
        set_error("%s: element type %d is not served (bfloat16 or float32)", what, p.dtype);
        return false;
    }
    if (p.heads < 1 || p.groups < 1 || p.heads % p.groups || !stack_ssm_serves(p.vdim, p.state, p.taps))
    {
        set_error("%s: heads %d in %d groups, vdim %d, state %d, %d taps is not a shape it serves (heads a multiple of groups, taps <= %d, "
                  "state x vdim <= 1024 x 32)",
            what, p.heads, p.groups, p.vdim, p.state, p.taps, MAX_TAPS);
        return false;
    }
    return true;
}

int launch_stack_ssm_conv(const StackSsmParams& p, hipStream_t stream)
{
    if (p.tokens <= 0 || p.entries <= 0)
        return 0;
    if (p.conv_channels > 0)
    {
        // the convolution alone, over a range of columns of another layer kind's projection
        if ((p.dtype != DT_BF16 && p.dtype != DT_FLOAT) || p.taps < 1 || p.taps > MAX_TAPS || p.conv_col < 0 || !p.conv_w || !p.conv_state || !p.xbc)
        {
            set_error("stack_ssm_conv: %d channels, %d taps (1 .. %d), or a missing operand", p.conv_channels, p.taps, MAX_TAPS);
            return -1;
        }
    }
    else if (!ssm_ok(p, "stack_ssm_conv"))
        return -1;
    const int CH = p.conv_channels > 0 ? p.conv_channels : p.heads * p.vdim + 2 * p.groups * p.state;
    const dim3 grid(p.tokens + p.entries, (CH + 255) / 256);
    if (p.dtype == DT_BF16)
        hipLaunchKernelGGL((ssm_conv_kernel<DT_BF16>), grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((ssm_conv_kernel<DT_FLOAT>), grid, dim3(256), 0, stream, p);
    return launched("stack_ssm_conv");
}

int launch_stack_ssm_scan(const StackSsmParams& p, hipStream_t stream)
{
    if (p.tokens <= 0 || p.entries <= 0)
        return 0;
    if (!ssm_ok(p, "stack_ssm_scan"))
        return -1;
    static const bool plain_only = [] {
        const char* v = std::getenv("TLLM_STACK_SSM_PLAIN"); // measurement knob: 1 = every shape on the form without prefetch
        return v && v[0] == '1';
    }();
    {
        // The pipelined form.  A head's columns are cut over workgroups (halves, quarters, down to 16 columns) while the launch has
        // fewer workgroups than the chip has CUs: a sequence's rows are walked in order, so the columns are what a long prompt of
        // few sequences can spread.  Rows per chunk: as many as KMAX values per thread and 128 KiB of LDS hold.
        const int cus = launch_util::device_cus();
        int pc = p.vdim;
        while (pc % 2 == 0 && pc / 2 >= 16 && (int64_t) p.entries * p.heads * (p.vdim / pc) < cus)
            pc /= 2;
        const int nsz = slice_rows(pc, p.state);
        const int NS = nsz ? (p.state + nsz - 1) / nsz : 0;
        const int threads = std::max(64, (NS * pc + 63) / 64 * 64);
        int rc = 0;
        for (int c : {16, 8, 4, 2})
            if (nsz && c * p.state <= KMAX * threads && c * pc <= KMAX * threads && c <= threads
                && sizeof(float) * (size_t) c * (2 * (2 + 2 * p.state + 2 * pc) + (size_t) NS * pc) <= kMaxLds)
            {
                rc = c;
                break;
            }
        if (rc > 0 && !plain_only)
        {
            const dim3 grid(p.entries, p.heads, p.vdim / pc);
            const size_t plds = sizeof(float) * (size_t) rc * (2 * (2 + 2 * p.state + 2 * pc) + (size_t) NS * pc);
#define TLLM_SSMP(DT, NSZ)                                                                                                               \
    do                                                                                                                                    \
    {                                                                                                                                     \
        launch_util::ensure_dynamic_lds(reinterpret_cast<const void*>(&ssm_scan_pipe_kernel<DT, NSZ>), plds > 64 * 1024 ? kMaxLds : 0);   \
        hipLaunchKernelGGL((ssm_scan_pipe_kernel<DT, NSZ>), grid, dim3(threads), plds, stream, p, NS, rc, pc);                            \
    } while (0)
#define TLLM_SSMP_DT(DT)                                                                                                                 \
    switch (nsz)                                                                                                                          \
    {                                                                                                                                     \
    case 4: TLLM_SSMP(DT, 4); break;                                                                                                    \
    case 8: TLLM_SSMP(DT, 8); break;                                                                                                    \
    case 16: TLLM_SSMP(DT, 16); break;                                                                                                  \
    default: TLLM_SSMP(DT, 32); break;                                                                                                  \
    }
            if (p.dtype == DT_BF16)
            {
                TLLM_SSMP_DT(DT_BF16)
            }
            else
            {
                TLLM_SSMP_DT(DT_FLOAT)
            }
#undef TLLM_SSMP_DT
#undef TLLM_SSMP
            return launched("stack_ssm_scan (pipelined)");
        }
    }
    const int nsz = slice_rows(p.vdim, p.state), NS = (p.state + nsz - 1) / nsz;
    const int threads = std::max(64, (NS * p.vdim + 63) / 64 * 64);
    const dim3 grid(p.entries, p.heads);
    const size_t lds = sizeof(float) * ((size_t) RC * (1 + 2 * p.state + p.vdim + (size_t) NS * p.vdim));
#define TLLM_SSM(DT, NSZ) hipLaunchKernelGGL((ssm_scan_kernel<DT, NSZ>), grid, dim3(threads), lds, stream, p, NS)
#define TLLM_SSM_DT(DT)                                                                                                                  \
    switch (nsz)                                                                                                                          \
    {                                                                                                                                     \
    case 4: TLLM_SSM(DT, 4); break;                                                                                                     \
    case 8: TLLM_SSM(DT, 8); break;                                                                                                     \
    case 16: TLLM_SSM(DT, 16); break;                                                                                                   \
    default: TLLM_SSM(DT, 32); break;                                                                                                   \
    }
    if (p.dtype == DT_BF16)
    {
        TLLM_SSM_DT(DT_BF16)
    }
    else
    {
        TLLM_SSM_DT(DT_FLOAT)
    }
#undef TLLM_SSM_DT
#undef TLLM_SSM
    return launched("stack_ssm_scan");
}

} // namespace kernels
} // namespace tllm
