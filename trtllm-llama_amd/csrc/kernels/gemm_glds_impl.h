// The LDS-DMA staged MFMA GEMM kernel template of gemm_glds.hip and its per-shape launcher, in a header so that the translation
// units that instantiate it for their operand types (gemm_glds.hip: SmoothQuant int8 and fp16; stack_gemm.hip: bfloat16) share
// one source.  Everything has internal linkage.
#pragma once
#include "dev_utils.h"
#include "kernels.h"
#include "launch_util.h"

namespace tllm
{
namespace kernels
{
namespace
{
using namespace dev;

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 glds_bf16x8 __attribute__((ext_vector_type(8)));


typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void gbl_void_t;

// One LDS-DMA instruction: 64 lanes x 16 bytes from per-lane global addresses to LDS [m0 + lane * 16].
// Issued from inline asm ON PURPOSE: for the builtin hipcc places `s_waitcnt vmcnt(0)` in front of the next ds_read (it
// cannot prove the DMA targets the other buffer), which serialises the DMA of tile t+1 with the MFMAs of tile t.  With
// the asm form the compiler sees no outstanding VMEM operation; the kernel waits by hand (vmcnt(0) before the barrier
// that publishes the tile).
__device__ __forceinline__ void glds16(const void* gptr, uint32_t lds_byte)
{
    uint32_t m0_keep;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0" : "=&s"(m0_keep) : "v"(gptr), "s"(lds_byte) : "memory");
}

// the same from a wave-uniform base + a per-lane 32-bit offset
__device__ __forceinline__ void glds16s(const char* base, uint32_t off, uint32_t lds_byte)
{
    uint32_t m0_keep;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0" : "=&s"(m0_keep) : "v"(off), "s"(base), "s"(lds_byte) : "memory");
}

// byte offset of 16-byte piece c16 of tile row `row`: XOR swizzle so that the 16 lanes of a ds_read_b128 phase
// (16 consecutive rows, same k-piece) hit 16 different 16-byte bank groups
template <int BKB>
__device__ __forceinline__ int swz(int row, int c16)
{
    if constexpr (BKB == 128)
        return row * 128 + ((c16 ^ ((row >> 1) & 7)) << 4);
    else
        return row * 64 + ((c16 ^ ((row >> 2) & 3)) << 4);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// LW > 0: LW extra waves that do nothing but issue the LDS-DMA.  One wave sustains about one LDS-DMA instruction per ~150
// cycles whatever else it does (the instruction holds its issuer for 100 - 185 cycles), which in the 8-wave 256 x 192 shape is a
// third of every compute wave's issue time; loaders (the shape's 160 VGPRs leave room for a third wave per SIMD) take that
// over and run the ring's look-ahead.
template <int WT, int WM, int WN, int MT, int NT, int KG, int BKB, int S, int LW = 0>
__global__ __launch_bounds__(64 * (WM * WN * KG + LW)) void gemm_glds_kernel(const GemmParams p_in)
{
    GemmParams p = p_in;
    if constexpr (WT == W_BF16)
    {
        // a batch of independent products of one shape (the stack engine's per-head products): blockIdx.y picks the operands
        p.a = reinterpret_cast<const char*>(p.a) + (int64_t) blockIdx.y * p.batch_a;
        p.w = reinterpret_cast<const char*>(p.w) + (int64_t) blockIdx.y * p.batch_w;
        p.c = reinterpret_cast<char*>(p.c) + (int64_t) blockIdx.y * p.batch_c;
        if (p.group_off)
        {
            const int64_t o = p.group_off[blockIdx.y];
            p.M = p.group_off[blockIdx.y + 1] - (int) o;
            if (p.M <= 0)
                return;
            p.a = reinterpret_cast<const char*>(p.a) + o * p.lda * 2;
            p.c = reinterpret_cast<char*>(p.c) + o * p.ldc * (p.out_dtype == DT_FLOAT ? 4 : 2);
        }
    }
    constexpr bool SQ = WT == W_INT8_SQ;
    constexpr int ES = SQ ? 1 : 2; // bytes per A / W element
    constexpr int NWC = WM * WN * KG;             // compute waves: KG groups of WM x WN waves split the k-steps of every stage
    constexpr int NW = LW > 0 ? LW : NWC;         // waves that issue the DMA
    static_assert(LW == 0 || KG == 1, "loader waves: one K-group");
    constexpr int KSTEPS = BKB / 32 / KG;         // k-steps per stage per group
    static_assert(KG == 1 || (KG == 2 && BKB == 128 && MT % 2 == 0), "K-groups: 2, on 128-byte stages");
    constexpr int BM = WM * MT * 32, BN = WN * NT * 32;
    constexpr int ROWS = BM + BN;                 // tile rows of [A; W]
    constexpr int RPC = 1024 / BKB;               // tile rows per 1 KiB DMA instruction (8 | 16)
    constexpr int PPR = BKB / 16;                 // 16-byte pieces per row (8 | 4)
    constexpr int CHUNKS = ROWS / RPC;            // DMA instructions per stage
    constexpr int CPW = (CHUNKS + NW - 1) / NW;   // ... per wave (the last one may be missing on the high waves)
    constexpr bool RAGGED = CHUNKS % NW != 0;
    constexpr int STAGE = ROWS * BKB;             // bytes per LDS stage
    constexpr int D = S - 1;                      // stages in flight ahead of the one being computed
    extern __shared__ __attribute__((aligned(16))) char lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6); // wave-uniform, and the compiler knows it (LDS-DMA base)
    // clock evidence for the microbench (tllm_gemm_set_clock_probe; GemmParams::clock_probe, set by the launcher only)
    void* const clk_probe = SQ ? p.clock_probe : nullptr;
    const uint64_t clk0 = clk_probe ? __builtin_readcyclecounter() : 0, rt0 = clk_probe ? __builtin_amdgcn_s_memrealtime() : 0;
    const bool loader = LW > 0 && wid >= NWC;     // wave-uniform
    const int iw = LW > 0 ? (wid >= NWC ? wid - NWC : 0) : wid; // index among the issuing waves
    const int kg = wid / (WM * WN), wq = wid % (WM * WN);
    const int wm = wq / WN, wn = wq % WN;
    // XCD-aware tile order: consecutive workgroup ids go to different XCDs (round-robin dispatch); give each XCD a
    // contiguous range of tiles so that the tiles sharing an A row-panel / W column-panel share an L2
    const int nwg = gridDim.x;
    int wg = blockIdx.x;
    // (a grouped product has fewer tiles than the grid, the first ids: in launch order they already go round the XCDs, while
    // contiguous ranges per XCD would leave every group's tiles on the first XCDs)
    if (!(WT == W_BF16 && p.group_off))
    {
        const int q = nwg >> 3, r = nwg & 7, xcd = wg & 7, idx = wg >> 3;
        wg = (xcd < r ? xcd * (q + 1) : r * (q + 1) + (xcd - r) * q) + idx;
    }
    const int tiles_m = (p.M + BM - 1) / BM;
    const int tm = wg % tiles_m, tn = wg / tiles_m; // M fastest: the (few) row panels of one W panel run together
    const int m0 = tm * BM, n0 = tn * BN;
    const int M = p.M, N = p.N;
    if constexpr (WT == W_BF16)
    {
        if (n0 >= N)
            return; // a group with fewer rows than the launch's bound has fewer tiles than the grid
    }
    const int ntile = (p.K * ES) / BKB;

    // ---- DMA source addresses: chunk c (RPC tile rows) -> lane l: row c * RPC + l / PPR, LDS piece l % PPR
    const char* a_base = reinterpret_cast<const char*>(p.a);
    const char* w_base = reinterpret_cast<const char*>(p.w);
    const char* src[LW > 0 ? 1 : CPW];
    // loader waves carry twice the chunks of a compute wave: 32-bit offsets from the two (wave-uniform) operand bases instead
    // of 64-bit addresses, or the 168-register budget of three waves per SIMD spills
    uint32_t soff[LW > 0 ? CPW : 1];
    constexpr int ACH = BM / RPC; // chunks of the A part of a stage
    static_assert(LW == 0 || ACH % LW == 0, "loader waves: A / W chunk boundary must not split a loader's turn");
    const bool short_wave = RAGGED && (CPW - 1) * NW + iw >= CHUNKS; // this wave has CPW - 1 DMA instructions
#pragma unroll
    for (int i = 0; i < CPW; ++i)
    {
        int c = i * NW + iw;
        c = c < CHUNKS ? c : CHUNKS - 1;
        const int row = c * RPC + lane / PPR;
        const int col = BKB == 128 ? (lane & 7) ^ ((row >> 1) & 7) : (lane & 3) ^ ((row >> 2) & 3);
        if (row < BM)
        {
            const int gr = m0 + row < M ? m0 + row : M - 1;
            if constexpr (LW > 0)
                soff[i] = (uint32_t) ((int64_t) gr * p.lda * ES + col * 16);
            else
                src[i] = a_base + (int64_t) gr * p.lda * ES + col * 16;
        }
        else
        {
            const int gr = n0 + row - BM < N ? n0 + row - BM : N - 1;
            if constexpr (LW > 0)
                soff[i] = (uint32_t) ((int64_t) gr * p.ldw + col * 16);
            else
                src[i] = w_base + (int64_t) gr * p.ldw + col * 16;
        }
    }
    const uint32_t lds_base = (uint32_t) (uintptr_t) (lds_void_t*) lds;
    auto issue = [&](int t) {
        const int stg = t % S;
#pragma unroll
        for (int i = 0; i < CPW; ++i)
        {
            const int c = i * NW + iw;
            if constexpr (LW > 0)
            {
                if (!RAGGED || i < CPW - 1 || !short_wave) // wave-uniform
                    glds16s((i < ACH / LW ? a_base : w_base) + (int64_t) t * BKB, soff[i], lds_base + stg * STAGE + c * 1024);
            }
            else if (!RAGGED || i < CPW - 1 || !short_wave) // wave-uniform
                glds16(src[i] + (int64_t) t * BKB, lds_base + stg * STAGE + c * 1024);
        }
    };
    // the same, spread over the k-steps of the tile being computed: this wave's DMA instructions number i with
    // i mod PARTS == part.  Issued in one burst right after the barrier they held every wave of the SIMD out of the matrix
    // pipe for the whole burst (an LDS-DMA instruction costs its issuer 60-185 cycles); between the MFMA groups their issue
    // time hides under the MFMAs already queued.
    auto issue_part = [&](int t, int part, int parts) {
        const int stg = t % S;
#pragma unroll
        for (int i = 0; i < CPW; ++i)
        {
            const int c = i * NW + iw;
            if constexpr (LW == 0)
                if (i % parts == part && (!RAGGED || i < CPW - 1 || !short_wave)) // wave-uniform
                    glds16(src[i] + (int64_t) t * BKB, lds_base + stg * STAGE + c * 1024);
        }
    };

    using acc_t = typename std::conditional<SQ, i32x16, f32x16>::type;
    acc_t acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0;

    const int fr = lane & 31, fk = lane >> 5;
    const bool vec_out = p.out_dtype == (WT == W_BF16 ? DT_BFLOAT16 : DT_HALF) && !p.resid && !p.bias && !p.act && !(p.ldc & 7) && !(N & 7) && !(reinterpret_cast<uintptr_t>(p.c) & 15)
        && !(reinterpret_cast<uintptr_t>(p.residual) & 15);
    if constexpr (LW > 0)
    {
        // the loaders' whole life: request, wait, barrier, request ... - a loop of its own, so that none of the compute waves'
        // registers (accumulators, fragments) is live in it and vice versa
        if (loader)
        {
#pragma unroll
            for (int t = 0; t < D; ++t)
                if (t < ntile)
                    issue(t);
            for (int t = 0; t < ntile; ++t)
            {
                if (t + D - 1 < ntile)
                {
                    if (short_wave)
                        wait_vmcnt<(D - 1) * (CPW - 1)>();
                    else
                        wait_vmcnt<(D - 1) * CPW>();
                }
                else
                    wait_vmcnt<0>();
                __syncthreads();
                if (t + D < ntile)
                    issue(t + D);
            }
            if (vec_out)
                __syncthreads(); // the epilogue's barrier
            return;
        }
    }
    const bool issuer = LW == 0;
    if (issuer)
    {
#pragma unroll
        for (int t = 0; t < D; ++t)
            if (t < ntile)
                issue(t);
    }
    for (int t = 0; t < ntile; ++t)
    {
        // stage t has landed: own DMA by the counted wait (the D - 1 younger stages stay in flight), everyone's by the
        // barrier; the same barrier says nobody still reads stage t - 1, whose buffer the next DMA overwrites
        if (issuer)
        {
            if (t + D - 1 < ntile)
            {
                if (short_wave)
                    wait_vmcnt<(D - 1) * (CPW - 1)>();
                else
                    wait_vmcnt<(D - 1) * CPW>();
            }
            else
                wait_vmcnt<0>();
        }
        __syncthreads();

        // the DMA of tile t + D is spread over the k-steps of tile t (see issue_part): every k-step with stages to spare, the
        // first two k-steps when only one stage is ahead (it must land before the next barrier).  128 x 128 / 3 ahead (O, down)
        // 49 -> 44 us in the real prefill, 256 x 192 / 1 ahead (QKV, gate, up) 53 -> 51 us stand-alone
        constexpr int SPREAD_PARTS = S >= 3 ? KSTEPS : (KSTEPS >= 2 ? 2 : 1);
        const char* As = lds + (t % S) * STAGE;
        const char* Bs = As + BM * BKB;
#pragma unroll
        for (int k2 = 0; k2 < KSTEPS; ++k2)
        {
            const int ks = kg * KSTEPS + k2;
            uint4 af[MT], bf[NT];
#pragma unroll
            for (int i = 0; i < MT; ++i)
                af[i] = *reinterpret_cast<const uint4*>(As + swz<BKB>((wm * MT + i) * 32 + fr, ks * 2 + fk));
#pragma unroll
            for (int j = 0; j < NT; ++j)
                bf[j] = *reinterpret_cast<const uint4*>(Bs + swz<BKB>((wn * NT + j) * 32 + fr, ks * 2 + fk));
            if (LW == 0 && k2 < SPREAD_PARTS && t + D < ntile)
            {
                __builtin_amdgcn_sched_barrier(0);
                issue_part(t + D, k2, SPREAD_PARTS);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NT; ++j)
                {
                    if constexpr (SQ)
                    {
                        const i32x4 a4 = {(int) af[i].x, (int) af[i].y, (int) af[i].z, (int) af[i].w};
                        const i32x4 b4 = {(int) bf[j].x, (int) bf[j].y, (int) bf[j].z, (int) bf[j].w};
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a4, b4, acc[i][j], 0, 0, 0);
                    }
                    else if constexpr (WT == W_BF16)
                    {
                        glds_bf16x8 a8, b8;
                        __builtin_memcpy(&a8, &af[i], 16);
                        __builtin_memcpy(&b8, &bf[j], 16);
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a8, b8, acc[i][j], 0, 0, 0);
                    }
                    else
                    {
                        f16x8 a8, b8;
                        __builtin_memcpy(&a8, &af[i], 16);
                        __builtin_memcpy(&b8, &bf[j], 16);
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a8, b8, acc[i][j], 0, 0, 0);
                    }
                }
        }
    }

    // ---- K-groups: exchange halves through LDS (int32 sums are exact in any order), then group g finalises the
    // MFMA rows i in [g * MT / 2, (g + 1) * MT / 2)
    int i_lo = 0, i_hi = MT;
    if constexpr (KG == 2)
    {
        constexpr int HALF = MT / 2;
        static_assert((size_t) HALF * NT * 16 * 4 * 64 * WM * WN <= (size_t) S * STAGE, "exchange buffer must fit the stages");
        using elem_t = typename std::conditional<SQ, int, float>::type;
        elem_t* xch = reinterpret_cast<elem_t*>(lds) + wq * 64 + lane; // [reg][wave-in-group][lane]
        constexpr int RS = WM * WN * 64;                                // elements per register slot
#pragma unroll
        for (int g = 0; g < 2; ++g)
        {
            // group 1 - g hands its partial sums of the rows that group g finalises
            __syncthreads();
            if (kg == 1 - g)
            {
#pragma unroll
                for (int i = 0; i < HALF; ++i)
#pragma unroll
                    for (int j = 0; j < NT; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            xch[((i * NT + j) * 16 + r) * RS] = acc[g * HALF + i][j][r];
            }
            __syncthreads();
            if (kg == g)
            {
#pragma unroll
                for (int i = 0; i < HALF; ++i)
#pragma unroll
                    for (int j = 0; j < NT; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            acc[g * HALF + i][j][r] += xch[((i * NT + j) * 16 + r) * RS];
            }
        }
        i_lo = kg * HALF;
        i_hi = i_lo + HALF;
    }

    if (clk_probe && tid == 0)
    {
        uint64_t* dbg = reinterpret_cast<uint64_t*>(clk_probe) + 2 * blockIdx.x;
        dbg[0] = __builtin_readcyclecounter() - clk0;
        dbg[1] = __builtin_amdgcn_s_memrealtime() - rt0;
    }
    // ---- epilogue.  acc[i][j][r]: col = lane & 31, row = (r & 3) + 8 * (r >> 2) + 4 * (lane >> 5)
    const float* s_row = p.scale_row;
    const int wave_n0 = n0 + wn * NT * 32;
    float sc[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j)
    {
        const int col = wave_n0 + j * 32 + (lane & 31);
        sc[j] = 1.f;
        if constexpr (!SQ)
        {
            if (p.scale_col) // weight-only: integers expanded to fp16, fp16 scale per output channel
                sc[j] = h2f(reinterpret_cast<const uint16_t*>(p.scale_col)[col < N ? col : N - 1]);
        }
        if constexpr (SQ)
            sc[j] = p.per_channel ? reinterpret_cast<const float*>(p.scale_col)[col < N ? col : N - 1]
                                  : reinterpret_cast<const float*>(p.scale_col)[0];
    }
    if (vec_out)
    {
        // fp16 rows through a wave-private LDS scratch: [32 rows][NT * 32 halfs], pitch chosen so that the two lane
        // halves (rows + 4) land 16 banks apart
        constexpr int PITCH = NT * 64 + 16;
        __syncthreads(); // every wave has finished reading the operand buffers
        char* scr = lds + wid * (32 * PITCH);
#pragma unroll
        for (int i = 0; i < MT; ++i)
        {
            if (i < i_lo || i >= i_hi) // wave-uniform (K-groups)
                continue;
            const int row_base = m0 + (wm * MT + i) * 32;
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                {
                    const int rr = (r & 3) + 8 * (r >> 2) + 4 * (lane >> 5);
                    float v;
                    if constexpr (SQ)
                    {
                        const int grow = row_base + rr;
                        const float sr = p.per_token ? s_row[grow < M ? grow : M - 1] : s_row[0];
                        v = (float) acc[i][j][r] * (sc[j] * sr);
                    }
                    else
                        v = acc[i][j][r] * sc[j];
                    *reinterpret_cast<uint16_t*>(scr + rr * PITCH + (j * 32 + (lane & 31)) * 2) = WT == W_BF16 ? f2bf(v) : f2h(v);
                }
            // 32 rows x (NT * 4) 16-byte pieces
            constexpr int PIECES = NT * 4;
#pragma unroll
            for (int s = lane; s < 32 * PIECES; s += 64)
            {
                const int rr = s / PIECES, pc = s % PIECES;
                uint4 v = *reinterpret_cast<const uint4*>(scr + rr * PITCH + pc * 16);
                const int grow = row_base + rr, gcol = wave_n0 + pc * 8;
                if (grow < M && gcol < N)
                {
                    const int64_t o = (int64_t) grow * p.ldc + gcol;
                    if (p.residual)
                    {
                        const uint4 rv = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.residual) + o);
                        const uint32_t a4[4] = {v.x, v.y, v.z, v.w}, b4[4] = {rv.x, rv.y, rv.z, rv.w};
                        uint32_t o4[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            o4[e] = (uint32_t) f2h(h2f((uint16_t) (a4[e] & 0xffffu)) + h2f((uint16_t) (b4[e] & 0xffffu)))
                                | ((uint32_t) f2h(h2f((uint16_t) (a4[e] >> 16)) + h2f((uint16_t) (b4[e] >> 16))) << 16);
                        v = make_uint4(o4[0], o4[1], o4[2], o4[3]);
                    }
                    else if (p.silu_gate)
                        v = epi_silu_gate8(v, *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.silu_gate) + o));
                    *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.c) + o) = v;
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
        {
            const int col = wave_n0 + j * 32 + (lane & 31);
            if (col >= N || i < i_lo || i >= i_hi)
                continue;
#pragma unroll
            for (int r = 0; r < 16; ++r)
            {
                const int row = m0 + (wm * MT + i) * 32 + (r & 3) + 8 * (r >> 2) + 4 * (lane >> 5);
                if (row >= M)
                    continue;
                const int64_t o = (int64_t) row * p.ldc + col;
                if constexpr (SQ)
                {
                    const int a = acc[i][j][r];
                    {
                        const float sr = p.per_token ? s_row[row] : s_row[0];
                        const float v = (float) a * (sc[j] * sr);
                        if (p.out_dtype == DT_INT32)
                            reinterpret_cast<int32_t*>(p.c)[o] = f2i32_rni_sat(v);
                        else if (p.out_dtype == DT_HALF)
                            reinterpret_cast<uint16_t*>(p.c)[o] = f2h(v);
                        else
                            reinterpret_cast<float*>(p.c)[o] = v;
                    }
                }
                else if constexpr (WT == W_BF16)
                {
                    // the stack engine's seam: resid += sigmoid(gate + bias) * product, or a bfloat16 / fp32 store
                    const float v = acc[i][j][r];
                    if (p.resid)
                    {
                        float g = 1.f;
                        if (p.gate)
                        {
                            const float z = bf2f(reinterpret_cast<const uint16_t*>(p.gate)[(int64_t) row * p.ldg + col])
                                + (p.gate_bias ? p.gate_bias[col] : 0.f);
                            g = 1.f / (1.f + __expf(-z));
                        }
                        p.resid[(int64_t) row * p.ldr + col] += g * v;
                    }
                    else
                    {
                        float u = p.bias ? v + p.bias[col] : v;
                        if (p.act == 1)
                        {
                            u = p.out_dtype == DT_BFLOAT16 ? bf2f(f2bf(u)) : u;
                            u = fmaxf(u, 0.f);
                            u *= u;
                        }
                        if (p.out_dtype == DT_BFLOAT16)
                            reinterpret_cast<uint16_t*>(p.c)[o] = f2bf(u);
                        else
                            reinterpret_cast<float*>(p.c)[o] = u;
                    }
                }
                else
                {
                    const float v = acc[i][j][r] * sc[j];
                    if (p.out_dtype == DT_HALF)
                        reinterpret_cast<uint16_t*>(p.c)[o] = f2h(v);
                    else
                        reinterpret_cast<float*>(p.c)[o] = v;
                }
            }
        }
}

template <int WT, int WM, int WN, int MT, int NT, int KG, int BKB, int S, int LW = 0>
int launch_cfg(const GemmParams& p, hipStream_t stream)
{
    constexpr int BM = WM * MT * 32, BN = WN * NT * 32;
    constexpr size_t smem = (size_t) S * (BM + BN) * BKB;
    static_assert(smem <= 160 * 1024, "LDS budget");
    static_assert(smem >= (size_t) WM * WN * KG * 32 * (NT * 64 + 16), "epilogue scratch must fit the operand stages");
    auto kfn = gemm_glds_kernel<WT, WM, WN, MT, NT, KG, BKB, S, LW>;
    launch_util::ensure_dynamic_lds(reinterpret_cast<const void*>(kfn), smem);
    const int tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
    hipLaunchKernelGGL(kfn, dim3(tiles, WT == W_BF16 && p.batch > 1 ? p.batch : 1), dim3(64 * (WM * WN * KG + LW)), smem, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
    {
        set_error("gemm_glds launch failed: %s", hipGetErrorString(e));
        return -1;
    }
    return 0;
}

} // namespace
} // namespace kernels
} // namespace tllm
