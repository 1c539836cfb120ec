// Products of the stack engine (stack_kernels.h): C[m,n] = sum_k A[m,k] * W[n,k] with the layer seam in the epilogue.
//
//   bfloat16, M >= 32, K % 64 == 0: the LDS-DMA staged MFMA tiles of gemm_glds_impl.h instantiated for bfloat16 operands
//                     (v_mfma_f32_32x32x16_bf16), tile shape by the same rounds x area rule as the fp16 form;
//   bfloat16, other M > 8: the register-staged MFMA tiles of gemm_mfma.hip;
//   bfloat16, M <= 8: skinny_kernel below - HBM-bound, a wave streams R weight rows with 16-byte non-temporal loads and keeps the
//                     M activation rows' chunks in registers; fp32 accumulation, DPP reduction;
//   float32         : fma_tile_kernel - 64 x 64 tiles of plain fp32 FMAs through LDS (no reduced-precision matrix mode), any shape;
//                     also the fallback for bfloat16 operands whose rows are not 16-byte aligned.
#include "dev_utils.h"
#include "gemm_glds_impl.h"
#include "stack_kernels.h"
#include <cstdlib>

namespace tllm
{
namespace kernels
{
int launch_gemm_mfma(const GemmParams& p, hipStream_t stream); // gemm_mfma.hip; 1: shape not served

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
__device__ __forceinline__ void seam(const StackGemmParams& p, int row, int col, float v)
{
    if (p.resid)
    {
        float g = 1.f;
        if (p.gate)
        {
            const float z = ld_el<DT>(p.gate, (int64_t) row * p.ldg + col) + (p.gate_bias ? p.gate_bias[col] : 0.f);
            g = 1.f / (1.f + expf(-z));
        }
        p.resid[(int64_t) row * p.ldr + col] += g * v;
    }
    else
    {
        const bool narrow = !(p.out_f32 || DT == DT_FLOAT);
        if (p.bias)
            v += p.bias[col];
        if (p.act == ACT_RELU2)
        {
            v = narrow ? bf2f(f2bf(v)) : v; // the projection's value in its element type, then its activation
            v = fmaxf(v, 0.f);
            v *= v;
        }
        if (narrow)
            reinterpret_cast<uint16_t*>(p.c)[(int64_t) row * p.ldc + col] = f2bf(v);
        else
            reinterpret_cast<float*>(p.c)[(int64_t) row * p.ldc + col] = v;
    }
}

// operands of product blockIdx.z of a batched launch
template <int DT>
__device__ __forceinline__ StackGemmParams batch_slice(StackGemmParams p)
{
    const int64_t b = blockIdx.z;
    constexpr int ES = DT == DT_BF16 ? 2 : 4;
    p.a = reinterpret_cast<const char*>(p.a) + b * p.stride_a * ES;
    p.w = reinterpret_cast<const char*>(p.w) + b * p.stride_w * ES;
    if (p.c)
        p.c = reinterpret_cast<char*>(p.c) + b * p.stride_c * ((p.out_f32 || DT == DT_FLOAT) ? 4 : 2);
    if (p.group_off)
    {
        // grouped form: this product's rows are a range of a and c that the device knows
        const int64_t o = p.group_off[b];
        p.M = p.group_off[b + 1] - (int) o;
        p.a = reinterpret_cast<const char*>(p.a) + o * p.lda * ES;
        if (p.c)
            p.c = reinterpret_cast<char*>(p.c) + o * p.ldc * ((p.out_f32 || DT == DT_FLOAT) ? 4 : 2);
    }
    return p;
}

constexpr int TM = 64, TN = 64, TK = 16;

template <int DT>
__global__ __launch_bounds__(256) void fma_tile_kernel(const StackGemmParams p_in)
{
    const StackGemmParams p = batch_slice<DT>(p_in);
    __shared__ float As[TK][TM + 4];
    __shared__ float Ws[TK][TN + 4];
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
    if (m0 >= p.M)
        return; // (a group with fewer rows than the launch's bound)
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            acc[i][j] = 0.f;
    for (int k0 = 0; k0 < p.K; k0 += TK)
    {
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            const int idx = tid + i * 256, r = idx / TK, k = idx % TK;
            As[k][r] = (m0 + r < p.M && k0 + k < p.K) ? ld_el<DT>(p.a, (int64_t) (m0 + r) * p.lda + k0 + k) : 0.f;
            Ws[k][r] = (n0 + r < p.N && k0 + k < p.K) ? ld_el<DT>(p.w, (int64_t) (n0 + r) * p.K + k0 + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < TK; ++k)
        {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                a[i] = As[k][ty * 4 + i];
                w[i] = Ws[k][tx * 4 + i];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const int row = m0 + ty * 4 + i, col = n0 + tx * 4 + j;
            if (row < p.M && col < p.N)
                seam<DT>(p, row, col, acc[i][j]);
        }
}

// bfloat16, M <= MR rows: 4 waves per workgroup, R weight rows per wave
constexpr int SK_R = 2;

template <int MR>
__global__ __launch_bounds__(256) void skinny_kernel(const StackGemmParams p_in)
{
    const StackGemmParams p = batch_slice<DT_BF16>(p_in);
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int n0 = (blockIdx.x * 4 + wid) * SK_R;
    if (n0 >= p.N || p.M <= 0)
        return;
    float acc[SK_R][MR];
#pragma unroll
    for (int r = 0; r < SK_R; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m)
            acc[r][m] = 0.f;
    const uint16_t* a = reinterpret_cast<const uint16_t*>(p.a);
    const uint16_t* w = reinterpret_cast<const uint16_t*>(p.w);
    for (int k = lane * 8; k < p.K; k += 64 * 8)
    {
        uint4 wv[SK_R];
#pragma unroll
        for (int r = 0; r < SK_R; ++r)
            wv[r] = n0 + r < p.N ? ld_nt16(w + (int64_t) (n0 + r) * p.K + k) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int m = 0; m < MR; ++m)
        {
            if (m >= p.M)
                break;
            const uint4 xv = *reinterpret_cast<const uint4*>(a + (int64_t) m * p.lda + k);
            const uint32_t xs[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
            for (int r = 0; r < SK_R; ++r)
            {
                const uint32_t ws[4] = {wv[r].x, wv[r].y, wv[r].z, wv[r].w};
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    acc[r][m] = fmaf(__builtin_bit_cast(float, xs[i] << 16), __builtin_bit_cast(float, ws[i] << 16), acc[r][m]);
                    acc[r][m] = fmaf(__builtin_bit_cast(float, xs[i] & 0xffff0000u), __builtin_bit_cast(float, ws[i] & 0xffff0000u), acc[r][m]);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < SK_R; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m)
        {
            const float s = wave_sum(acc[r][m]);
            if (lane == 0 && m < p.M && n0 + r < p.N)
                seam<DT_BF16>(p, m, n0 + r, s);
        }
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

// the lock-step tile shapes of the LDS-DMA kernel and what a tile of each kind costs per area (measured on fp16 operands; the
// bfloat16 MFMA has the same rate and byte geometry): fewest workgroup rounds x area x cost
int launch_glds_bf16(const GemmParams& g, hipStream_t stream, int m_expected = 0)
{
    // m_expected: the rows a product of a grouped launch has on average (g.M is their bound, which sizes the grid): the tile shape is
    // chosen for what is expected, or tall tiles would run half empty on every group
    struct Shape
    {
        int id, bm, bn;
        double f;
    };
    static const Shape shapes[] = {{0, 128, 128, 1.40}, {1, 256, 192, 1.0}, {2, 256, 256, 1.04}, {3, 128, 256, 1.39}};
    const int cus = launch_util::device_cus();
    double best = 1e30;
    int pick = 0;
    for (const Shape& sh : shapes)
    {
        const int m = m_expected > 0 ? m_expected : g.M;
        const int64_t tiles = (int64_t) ((m + sh.bm - 1) / sh.bm) * ((g.N + sh.bn - 1) / sh.bn) * (g.batch > 1 ? g.batch : 1);
        const double cost = (double) ((tiles + cus - 1) / cus) * sh.bm * sh.bn * sh.f;
        if (cost < best)
        {
            best = cost;
            pick = sh.id;
        }
    }
    if (m_expected > 0)
    {
        // groups of up to two 128-row tiles: the small square tile (more, shorter workgroups behind the ones that leave at once)
        // measured 9 % ahead of the three larger shapes on a 1024-token prompt over 32 experts
        if (m_expected <= 256)
            pick = 0;
        static const int forced = [] {
            const char* v = std::getenv("TLLM_STACK_GROUP_TILE"); // measurement knob: tile shape 0 .. 3 for grouped products
            return v && v[0] >= '0' && v[0] <= '3' ? v[0] - '0' : -1;
        }();
        if (forced >= 0)
            pick = forced;
    }
    switch (pick)
    {
    case 1: return launch_cfg<W_BF16, 4, 2, 2, 3, 1, 64, 5>(g, stream);
    case 2: return launch_cfg<W_BF16, 2, 4, 4, 2, 1, 64, 4>(g, stream);
    case 3: return launch_cfg<W_BF16, 2, 2, 2, 4, 1, 64, 4>(g, stream);
    default: return launch_cfg<W_BF16, 2, 2, 2, 2, 1, 128, 4>(g, stream);
    }
}

} // namespace

int launch_stack_gemm(const StackGemmParams& p, hipStream_t stream)
{
    if (p.M <= 0 || p.N <= 0)
        return 0;
    if (p.K <= 0 || !p.a || !p.w || (!p.c && !p.resid))
    {
        set_error("stack_gemm: M %d N %d K %d with a missing operand", p.M, p.N, p.K);
        return -1;
    }
    if (p.dtype != DT_BF16 && p.dtype != DT_FLOAT)
    {
        set_error("stack_gemm: element type %d is not served (bfloat16 or float32)", p.dtype);
        return -1;
    }
    if (p.batch < 1 || (p.batch > 1 && p.resid) || (p.group_off && (p.resid || p.stride_a || p.stride_c)))
    {
        set_error("stack_gemm: batch %d (a batched product has no residual seam; a grouped one takes its rows from one a and one c)", p.batch);
        return -1;
    }
    const dim3 tiles((p.N + TN - 1) / TN, (p.M + TM - 1) / TM, p.batch);
    if (p.dtype == DT_FLOAT)
    {
        hipLaunchKernelGGL((fma_tile_kernel<DT_FLOAT>), tiles, dim3(256), 0, stream, p);
        return launched("stack_gemm fp32");
    }
    const bool aligned = !(reinterpret_cast<uintptr_t>(p.a) & 15) && !(reinterpret_cast<uintptr_t>(p.w) & 15) && p.K % 8 == 0 && p.lda % 8 == 0
        && (p.batch == 1 || (p.stride_a % 8 == 0 && p.stride_w % 8 == 0));
    if (aligned && p.M <= 8)
    {
        const dim3 grid((p.N + 4 * SK_R - 1) / (4 * SK_R), 1, p.batch);
        if (p.M <= 1)
            hipLaunchKernelGGL((skinny_kernel<1>), grid, dim3(256), 0, stream, p);
        else if (p.M <= 4)
            hipLaunchKernelGGL((skinny_kernel<4>), grid, dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL((skinny_kernel<8>), grid, dim3(256), 0, stream, p);
        return launched("stack_gemm skinny");
    }
    if (aligned && (!p.group_off || p.K % 64 == 0))
    {
        // the LDS-DMA tiles take a batch in one launch (blockIdx.y); the register-staged tiles one product per launch (and no
        // groups: their row count is the device's)
        const bool glds = (p.M >= 32 || p.group_off) && p.K % 64 == 0;
        const int launches = glds ? 1 : p.batch;
        int rc = 0;
        for (int b = 0; b < launches && rc == 0; ++b)
        {
            GemmParams g;
            g.wtype = W_BF16;
            g.out_dtype = p.out_f32 ? DT_FLOAT : DT_BFLOAT16;
            g.M = p.M;
            g.N = p.N;
            g.K = p.K;
            g.a = reinterpret_cast<const char*>(p.a) + (int64_t) b * p.stride_a * 2;
            g.lda = p.lda;
            g.w = reinterpret_cast<const char*>(p.w) + (int64_t) b * p.stride_w * 2;
            g.ldw = (int64_t) p.K * 2;
            g.c = p.c ? reinterpret_cast<char*>(p.c) + (int64_t) b * p.stride_c * (p.out_f32 ? 4 : 2) : nullptr;
            g.ldc = p.ldc;
            g.resid = p.resid;
            g.ldr = p.ldr;
            g.gate = p.gate;
            g.ldg = p.ldg;
            g.gate_bias = p.gate_bias;
            g.bias = p.bias;
            g.act = p.act;
            if (glds)
            {
                g.batch = p.batch;
                g.batch_a = p.stride_a * 2;
                g.batch_w = p.stride_w * 2;
                g.batch_c = p.stride_c * (p.out_f32 ? 4 : 2);
                g.group_off = p.group_off;
                rc = launch_glds_bf16(g, stream, p.group_off ? p.group_rows : 0);
            }
            else
                rc = launch_gemm_mfma(g, stream);
        }
        if (rc <= 0)
            return rc;
    }
    hipLaunchKernelGGL((fma_tile_kernel<DT_BF16>), tiles, dim3(256), 0, stream, p);
    return launched("stack_gemm bf16 fma tiles");
}

} // namespace kernels
} // namespace tllm
