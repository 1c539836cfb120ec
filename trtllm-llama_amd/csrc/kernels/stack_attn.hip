// Attention of the stack engine over the paged cache: the MFMA tile kernel for bfloat16 (prefill portions and decoded tokens
// alike), and the dispatch between it and the general kernel of stack_ops.hip (any shape, both element types).
//
// attn_tile_kernel: one workgroup per (16 rows of one entry, head); its NW waves split the key blocks (32 keys each) round-robin -
// key-split waves, so a decoded token with a long context still has NW waves in flight - and merge their partial (max, sum, O)
// through LDS.  Everything is computed TRANSPOSED so that no operand ever changes layout between the two products:
//   S^T = K Q^T      A = K rows straight from the page (key-major, 16 bytes of dim per lane), B = Q^T fragments kept in registers;
//                    the result has one query row per lane column, 4 keys per lane and tile;
//   O^T += V^T P^T   B = P^T, which is exactly what the lane already holds (its 8 scores of the block, as bfloat16);
//                    A = V^T rows, which is why the cache stores values channel-major inside a page ([vdim][page]).
// Both maps of a differential head run side by side and share the V^T fragments.  fp32: scores, soft cap, softmax state, O.
#include "dev_utils.h"
#include "launch_util.h"
#include "stack_kernels.h"
#include <algorithm>
#include <cstdlib>

namespace tllm
{
namespace kernels
{
int launch_stack_attention_general(const StackAttnParams& p, hipStream_t stream); // stack_ops.hip

using namespace dev;

namespace
{
constexpr int kSplitRows = 64, kMaxSplits = 16;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 as_bf16x8(const uint4& u)
{
    bf16x8 r;
    __builtin_memcpy(&r, &u, 16);
    return r;
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// max / sum over the four lanes that hold the same query row (lane ^ 16, lane ^ 32)
__device__ __forceinline__ float rows_max(float v)
{
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    return fmaxf(v, __shfl_xor(v, 32, 64));
}
__device__ __forceinline__ float rows_sum(float v)
{
    v += __shfl_xor(v, 16, 64);
    return v + __shfl_xor(v, 32, 64);
}

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi)
{
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}

// What a head does to its raw scores, in the base-2 domain (an exponential is one v_exp_f32, a logarithm one v_log_f32):
//   score2 = cap(q.k * scale) * temp * log2 e - slope2 * (i - j) - r1 * log2(1 + r2 * (i - j))
// and how scores become weights: softmax (running maximum and sum), or a sigmoid per key (no state across keys).
struct HeadMods
{
    float scale2, cap2, cap_arg, temp, slope2, r1, r2, wb2;
    int pen, sigm; // pen: any of temp / slope / r1 is set
    int keep;      // the first `keep` keys of the sequence stay visible behind a window
};

// Which query, key and value head a launch's head index h stands for.  Ordinarily h is the query head and reads the key / value head
// of its group.  cross_values: p.heads = query heads x kv_heads, and h = query head * kv_heads + value head - every query head's
// weights applied to every value head's rows (the terms a mixing of weights across heads is made of).
struct HeadMap
{
    int qh, kh, vh, q_heads;
};
__device__ __forceinline__ HeadMap head_map(const StackAttnParams& p, int h)
{
    HeadMap m;
    m.q_heads = p.cross_values ? p.heads / p.kv_heads : p.heads;
    m.qh = p.cross_values ? h / p.kv_heads : h;
    m.kh = m.qh / (m.q_heads / p.kv_heads);
    m.vh = p.cross_values ? h % p.kv_heads : m.kh;
    return m;
}

__device__ __forceinline__ HeadMods head_mods(const StackAttnParams& p, int h)
{
    constexpr float LOG2E = 1.4426950408889634f;
    h = p.cross_values ? h / p.kv_heads : h; // per-head numbers belong to query heads
    HeadMods m;
    m.temp = p.temp ? p.temp[h] : 1.f;
    m.scale2 = p.scale * LOG2E * (p.softcap > 0.f ? 1.f : m.temp);
    m.cap2 = p.softcap > 0.f ? p.softcap * LOG2E * m.temp : 0.f;
    m.cap_arg = p.softcap > 0.f ? p.scale / p.softcap * 2.f * LOG2E : 0.f;
    m.slope2 = p.slope ? p.slope[h] * LOG2E : 0.f;
    m.r1 = p.log_r1 ? p.log_r1[h] : 0.f;
    m.r2 = p.log_r1 ? p.log_r2[h] : 0.f;
    m.pen = (p.slope || p.log_r1) ? 1 : 0;
    m.sigm = p.weights == WEIGHTS_SIGMOID;
    m.wb2 = m.sigm && p.wbias ? p.wbias[h] * LOG2E : 0.f;
    m.keep = p.mask == MASK_WINDOW ? p.mask_keep : 0;
    return m;
}

// the first key position a row at `pos` sees
__device__ __forceinline__ int first_visible(const StackAttnParams& p, int pos)
{
    if (p.mask == MASK_WINDOW)
        return pos - p.mask_size + 1 > 0 ? pos - p.mask_size + 1 : 0;
    if (p.mask == MASK_CHUNK)
        return pos / p.mask_size * p.mask_size;
    return 0;
}

// The 32-key blocks a tile walks: from the block that holds its first row's first visible key up to the block of its last row;
// with kept first keys, the blocks that hold them and lie before that range come first.  Step v of n visits block walk_block(w, v).
struct BlockWalk
{
    int nkeep, lo, n;
};
__device__ __forceinline__ BlockWalk block_walk(const StackAttnParams& p, int first_row_pos, int nblk)
{
    BlockWalk w;
    w.lo = first_visible(p, first_row_pos) / 32;
    const int kept = (p.mask == MASK_WINDOW && p.mask_keep > 0) ? (p.mask_keep + 31) / 32 : 0;
    w.nkeep = kept < w.lo ? kept : w.lo;
    w.n = w.nkeep + (nblk - w.lo);
    return w;
}
__device__ __forceinline__ int walk_block(const BlockWalk& w, int v)
{
    return v < w.nkeep ? v : v - w.nkeep + w.lo;
}

// Scores of one 32-key block of one map -> its P^T fragment, with the online-softmax state of the lane's query row brought up to
// date.  `masked` is wave-uniform: only blocks that reach past the first row's position, or start before the last row's first
// visible key, compare keys with positions.
template <int VT>
__device__ __forceinline__ uint4 softmax_block(f32x4 (&s)[2], float& m_run, float& l_run, f32x4 (&acc)[VT], const HeadMods& hm, bool masked,
    int key_lane0, int qpos, int klo)
{
    float bm = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            float v;
            if (hm.cap2 > 0.f)
            {
                // cap * tanh(x / cap) with tanh(y) = (e^{2y} - 1) / (e^{2y} + 1); cap_arg = scale / cap * 2 log2 e
                const float t2 = __builtin_amdgcn_exp2f(fminf(fmaxf(s[t][i] * hm.cap_arg, -43.f), 43.f));
                v = hm.cap2 * (t2 - 1.f) * __builtin_amdgcn_rcpf(t2 + 1.f);
            }
            else
                v = s[t][i] * hm.scale2;
            const int kidx = key_lane0 + t * 16 + i;
            if (hm.pen)
            {
                const float dist = (float) (qpos - kidx);
                v -= hm.slope2 * dist;
                if (hm.r1 != 0.f)
                    v -= hm.r1 * __builtin_amdgcn_logf(fmaxf(1.f + hm.r2 * dist, 1e-30f));
            }
            if (masked && (kidx > qpos || (kidx < klo && kidx >= hm.keep)))
                v = -INFINITY;
            s[t][i] = v;
            bm = fmaxf(bm, v);
        }
    if (hm.sigm)
    {
        // every key's weight stands alone: 1 / (1 + 2^-(score2 + offset2)); a hidden key's is 2^-inf = 0
        float pv[8];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                pv[t * 4 + i] = s[t][i] == -INFINITY ? 0.f : __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-(s[t][i] + hm.wb2)));
        return make_uint4(pack_bf16(pv[0], pv[1]), pack_bf16(pv[2], pv[3]), pack_bf16(pv[4], pv[5]), pack_bf16(pv[6], pv[7]));
    }
    bm = rows_max(bm);
    const float mn = fmaxf(m_run, bm);
    const bool none = mn == -INFINITY; // this row sees no key of this block (nor of any before)
    const float corr = none ? 1.f : __builtin_amdgcn_exp2f(m_run - mn);
    float rs = 0.f, pv[8];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            pv[t * 4 + i] = none ? 0.f : __builtin_amdgcn_exp2f(s[t][i] - mn);
            rs += pv[t * 4 + i];
        }
    rs = rows_sum(rs);
    l_run = l_run * corr + rs;
    m_run = mn;
    // the accumulators are rescaled only when some row's maximum moved (wave-uniform test): behind the first blocks of a long
    // context it rarely does, and the accumulators sit in the matrix pipe's registers, a round trip per element away
    if (__builtin_amdgcn_ballot_w64(corr != 1.f) != 0)
    {
#pragma unroll
        for (int ct = 0; ct < VT; ++ct)
            acc[ct] *= corr;
    }
    return make_uint4(pack_bf16(pv[0], pv[1]), pack_bf16(pv[2], pv[3]), pack_bf16(pv[4], pv[5]), pack_bf16(pv[6], pv[7]));
}

// How a finished row leaves: the softmax denominator also takes the head's sink (a logit without key or value), given the row's
// running maximum M (base 2) and sum L relative to it -> the factor on the accumulator; sigmoid weights are not normalised.
__device__ __forceinline__ float finish_factor(const StackAttnParams& p, int h, float M, float L)
{
    if (p.weights == WEIGHTS_SIGMOID)
        return 1.f;
    if (!p.sink)
        return 1.f / L;
    const float sk = p.sink[p.cross_values ? h / p.kv_heads : h] * 1.4426950408889634f, mf = fmaxf(M, sk);
    const float wk = __builtin_amdgcn_exp2f(M - mf);
    return wk / (L * wk + __builtin_amdgcn_exp2f(sk - mf));
}

__device__ __forceinline__ float out_gate_of(const StackAttnParams& p, int64_t t, int h)
{
    if (!p.out_gate)
        return 1.f;
    const float z = bf2f(reinterpret_cast<const uint16_t*>(p.out_gate)[t * p.ld_gate + h]);
    return 1.f / (1.f + __expf(-z));
}

template <int MAPS, int DK, int VT, int NW>
__global__ __launch_bounds__(NW * 64) void attn_tile_kernel(const StackAttnParams p, int below_count, int ks, int head_rows)
{
    constexpr int D = DK * 32, V = VT * 16;
    extern __shared__ float lds[];
    float* o_part = lds;                          // [NW][MAPS][16][V]
    float* ml_part = lds + NW * MAPS * 16 * V;    // [NW][MAPS][16][2]
    // ks == 1: blockIdx.x is the entry's 16-row tile.  ks > 1 (decoding steps: every entry one tile): blockIdx.x is the key split -
    // workgroup `split` of an (entry, head) takes the key blocks split * NW + w, + ks * NW, ... and leaves an unnormalised partial
    // (max, sum, O per map and row) in split_ws; attn_split_merge_kernel finishes the rows.
    // head_rows (a step of single decoded tokens whose heads all share ONE key/value head and have no numbers of their own): the
    // tile's 16 rows are 16 HEADS of the entry's one token, blockIdx.z the group of heads - the keys are walked once per 16 heads
    const int e = blockIdx.y, hbase = head_rows ? blockIdx.z * 16 : 0, h = head_rows ? hbase : blockIdx.z;
    const int r0 = (ks > 1 || head_rows) ? 0 : blockIdx.x * 16;
    const int split = ks > 1 ? blockIdx.x : 0;
    const int count = p.ent_count[e];
    if (r0 >= count || count >= below_count) // entries of below_count rows and more are the prefill form's
        return;
    const int first = p.ent_first[e], pos0 = p.ent_pos0[e];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int col = lane & 15, g4 = lane >> 4;
    const HeadMap hd = head_map(p, h);
    const int g = hd.kh, gv = hd.vh;
    const int page = p.page;
    const int32_t* table = p.block_table + (int64_t) e * p.max_blocks;
    const HeadMods hm = head_mods(p, h);
    const uint16_t* kp = reinterpret_cast<const uint16_t*>(p.k_pool);
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(p.v_pool);

    const int qrow = head_rows ? 0 : (r0 + col < count ? r0 + col : count - 1);
    const int qhead = head_rows ? (hbase + col < p.heads ? hbase + col : p.heads - 1) : hd.qh;
    const int qpos = pos0 + qrow;
    const int klo = first_visible(p, qpos);
    bf16x8 qf[MAPS][DK];
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
#pragma unroll
        for (int ks = 0; ks < DK; ++ks)
            qf[m][ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
                reinterpret_cast<const uint16_t*>(p.q) + (((int64_t) (first + qrow) * hd.q_heads + qhead) * MAPS + m) * D + ks * 32 + 8 * g4));
    const int last_row = head_rows ? 0 : (r0 + 15 < count ? r0 + 15 : count - 1);
    const int nblk = (pos0 + last_row) / 32 + 1;
    // the tile's key blocks: from the one that holds the first row's first visible key; klo_last: the last row's (the largest)
    const int blk_lo = first_visible(p, pos0 + r0) / 32, klo_last = first_visible(p, pos0 + last_row);

    float m_run[MAPS], l_run[MAPS];
    f32x4 acc[MAPS][VT];
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
    {
        m_run[m] = -INFINITY;
        l_run[m] = 0.f;
#pragma unroll
        for (int ct = 0; ct < VT; ++ct)
            acc[m][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // Software pipeline: the K fragments of a block are requested one iteration ahead, its V^T fragments at the top of its own
    // iteration, so that the score / softmax arithmetic of a block (the long part: it is all VALU) runs with both in flight.
    uint4 kf[MAPS][2][DK];
    auto request_k = [&](int kb, int blk) {
        const int off = (kb * 32) % page;
#pragma unroll
        for (int m = 0; m < MAPS; ++m)
#pragma unroll
            for (int t = 0; t < 2; ++t)
            {
                const uint16_t* krow = kp + (((int64_t) blk * (p.kv_heads * MAPS) + g * MAPS + m) * page + off + t * 16 + col) * D + 8 * g4;
#pragma unroll
                for (int ks = 0; ks < DK; ++ks)
                    kf[m][t][ks] = *reinterpret_cast<const uint4*>(krow + ks * 32);
            }
    };
    const BlockWalk bw = block_walk(p, pos0 + r0, nblk);
    const int vb0 = split * NW + w, kstep = ks * NW;
    int kb_next = vb0 < bw.n ? walk_block(bw, vb0) : 0;
    int blk = vb0 < bw.n ? table[kb_next * 32 / page] : 0;
    if (vb0 < bw.n)
        request_k(kb_next, blk);
    for (int vb = vb0; vb < bw.n; vb += kstep)
    {
        const int kb = kb_next;
        const int key0 = kb * 32, off = key0 % page;
        uint2 vlo[VT], vhi[VT];
        {
            const uint16_t* vrow = vp + (((int64_t) blk * p.kv_heads + gv) * V + col) * page + off + 4 * g4;
#pragma unroll
            for (int ct = 0; ct < VT; ++ct)
            {
                vlo[ct] = *reinterpret_cast<const uint2*>(vrow + (int64_t) ct * 16 * page);
                vhi[ct] = *reinterpret_cast<const uint2*>(vrow + (int64_t) ct * 16 * page + 16);
            }
        }
        f32x4 s[MAPS][2];
#pragma unroll
        for (int m = 0; m < MAPS; ++m)
#pragma unroll
            for (int t = 0; t < 2; ++t)
            {
                s[m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < DK; ++ks)
                    s[m][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf[m][t][ks]), qf[m][ks], s[m][t], 0, 0, 0);
            }
        if (vb + kstep < bw.n)
        {
            kb_next = walk_block(bw, vb + kstep);
            blk = table[kb_next * 32 / page];
            request_k(kb_next, blk);
        }
        uint4 pf[MAPS]; // P^T fragment of the block, 8 bfloat16 per map
        const bool masked = key0 + 31 > pos0 + r0 || key0 < klo_last; // wave-uniform
#pragma unroll
        for (int m = 0; m < MAPS; ++m)
            pf[m] = softmax_block<VT>(s[m], m_run[m], l_run[m], acc[m], hm, masked, key0 + 4 * g4, qpos, klo);
        // O^T += V^T P^T: slot j of the lane's k group is key 4 g4 + j (j < 4) or 16 + 4 g4 + (j - 4) of the block, in both operands
#pragma unroll
        for (int ct = 0; ct < VT; ++ct)
        {
            const bf16x8 vf = as_bf16x8(make_uint4(vlo[ct].x, vlo[ct].y, vhi[ct].x, vhi[ct].y));
#pragma unroll
            for (int m = 0; m < MAPS; ++m)
                acc[m][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, as_bf16x8(pf[m]), acc[m][ct], 0, 0, 0);
        }
    }

    // ---- merge of the waves' partials
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
    {
        if (g4 == 0)
        {
            ml_part[((w * MAPS + m) * 16 + col) * 2] = m_run[m];
            ml_part[((w * MAPS + m) * 16 + col) * 2 + 1] = l_run[m];
        }
#pragma unroll
        for (int ct = 0; ct < VT; ++ct)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                o_part[((w * MAPS + m) * 16 + col) * V + ct * 16 + 4 * g4 + i] = acc[m][ct][i];
    }
    __syncthreads();
    // 16 threads per row at NW = 4 (NW * 4 in general), each a strided set of channels
    constexpr int TPR = NW * 4;
    const int row = threadIdx.x / TPR, sub = threadIdx.x % TPR;
    // where tile row `row` leaves: (packed row, head)
    const int64_t out_t = first + (head_rows ? 0 : r0 + row);
    const int out_h = head_rows ? hbase + row : h;
    const bool out_ok = head_rows ? hbase + row < p.heads : r0 + row < count;
    float wgt[MAPS][NW];
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
    {
        float M = -INFINITY;
#pragma unroll
        for (int ww = 0; ww < NW; ++ww)
            M = fmaxf(M, ml_part[((ww * MAPS + m) * 16 + row) * 2]);
        float L = 0.f;
#pragma unroll
        for (int ww = 0; ww < NW; ++ww)
        {
            const float mw = ml_part[((ww * MAPS + m) * 16 + row) * 2];
            wgt[m][ww] = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - M); // the running maxima are base-2 exponents
            if (hm.sigm)
                wgt[m][ww] = 1.f; // sigmoid weights: the waves' sums simply add
            L += wgt[m][ww] * ml_part[((ww * MAPS + m) * 16 + row) * 2 + 1];
        }
        if (ks > 1)
        {
            // partial of this split: weights stay relative to the split's own maximum, nothing is divided yet
            if (sub == 0 && out_ok)
            {
                float* ws = p.split_ws + (((out_t * p.heads + out_h) * ks + split) * MAPS + m) * (V + 2);
                ws[V] = M;
                ws[V + 1] = L;
            }
        }
        else
        {
            const float fin = finish_factor(p, h, M, L);
#pragma unroll
            for (int ww = 0; ww < NW; ++ww)
                wgt[m][ww] *= fin;
        }
    }
    constexpr int CPT = (V + TPR - 1) / TPR;
    if (ks > 1)
    {
        if (out_ok)
        {
#pragma unroll
            for (int m = 0; m < MAPS; ++m)
            {
                float* ws = p.split_ws + (((out_t * p.heads + out_h) * ks + split) * MAPS + m) * (V + 2);
#pragma unroll
                for (int c = 0; c < CPT; ++c)
                {
                    const int ch = sub + c * TPR;
                    if (ch < V)
                    {
                        float a = 0.f;
#pragma unroll
                        for (int ww = 0; ww < NW; ++ww)
                            a += wgt[m][ww] * o_part[((ww * MAPS + m) * 16 + row) * V + ch];
                        ws[ch] = a;
                    }
                }
            }
        }
        return;
    }
    float o[CPT], ss = 0.f;
#pragma unroll
    for (int c = 0; c < CPT; ++c)
    {
        const int ch = sub + c * TPR;
        o[c] = 0.f;
        if (ch < V)
        {
            float a[MAPS];
#pragma unroll
            for (int m = 0; m < MAPS; ++m)
            {
                a[m] = 0.f;
#pragma unroll
                for (int ww = 0; ww < NW; ++ww)
                    a[m] += wgt[m][ww] * o_part[((ww * MAPS + m) * 16 + row) * V + ch];
            }
            o[c] = MAPS == 2 ? a[0] - p.lambda * a[MAPS - 1] : a[0];
            ss += o[c] * o[c];
        }
    }
    float mul = 1.f;
    if (p.head_norm)
    {
#pragma unroll
        for (int d = 1; d < TPR; d <<= 1)
            ss += __shfl_xor(ss, d, 64);
        mul = p.out_scale / sqrtf(ss / (float) V + p.eps);
    }
    if (out_ok)
    {
        mul *= out_gate_of(p, out_t, out_h);
        uint16_t* out = reinterpret_cast<uint16_t*>(p.out) + (out_t * p.heads + out_h) * V;
#pragma unroll
        for (int c = 0; c < CPT; ++c)
            if (sub + c * TPR < V)
                out[sub + c * TPR] = f2bf(o[c] * mul);
    }
}

// attn_prefill_kernel: the form for entries that bring many rows.  One workgroup per (64 rows of an entry, head), wave w owns rows
// 16 w .. 16 w + 15; all four waves walk the same 32-key blocks, which the workgroup stages once through LDS (K rows padded to an odd
// number of 16-byte pieces, V^T rows to 80 bytes: the fragment reads spread over the banks) - the next block's global loads are in
// flight while this block is computed.  Same transposed products and operand slots as attn_tile_kernel; no merge: a wave finishes
// its own rows (lambda combination, head norm, bfloat16 store).  Tiles are handed out heaviest first (the last rows see most keys).
template <int MAPS, int DK, int VT>
__global__ __launch_bounds__(256) void attn_prefill_kernel(const StackAttnParams p, int min_count)
{
    constexpr int D = DK * 32, V = VT * 16;
    constexpr int KP = D * 2 + 16, VP = 80;                 // LDS row pitches in bytes
    constexpr int K16 = MAPS * 32 * (D / 8), V16 = V * 4;   // 16-byte pieces per block
    constexpr int KPT = (K16 + 255) / 256, VPT = (V16 + 255) / 256;
    __shared__ __attribute__((aligned(16))) char k_s[MAPS * 32 * KP];
    __shared__ __attribute__((aligned(16))) char v_s[V * VP];
    const int e = blockIdx.y, h = blockIdx.z;
    const int count = p.ent_count[e];
    if (count < min_count)
        return;
    const int tile = (count + 63) / 64 - 1 - (int) blockIdx.x;
    if (tile < 0)
        return;
    const int first = p.ent_first[e], pos0 = p.ent_pos0[e];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int col = lane & 15, g4 = lane >> 4;
    const HeadMap hd = head_map(p, h);
    const int g = hd.kh, gv = hd.vh;
    const int page = p.page;
    const int32_t* table = p.block_table + (int64_t) e * p.max_blocks;
    const HeadMods hm = head_mods(p, h);
    const uint16_t* kp = reinterpret_cast<const uint16_t*>(p.k_pool);
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(p.v_pool);

    const int r0 = tile * 64 + w * 16;
    const bool wave_rows = r0 < count; // wave-uniform
    const int qrow = r0 + col < count ? r0 + col : count - 1;
    const int qpos = pos0 + qrow;
    const int klo = first_visible(p, qpos);
    bf16x8 qf[MAPS][DK];
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
#pragma unroll
        for (int ks = 0; ks < DK; ++ks)
            qf[m][ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
                reinterpret_cast<const uint16_t*>(p.q) + (((int64_t) (first + qrow) * hd.q_heads + hd.qh) * MAPS + m) * D + ks * 32 + 8 * g4));
    const int wg_last = tile * 64 + 63 < count ? tile * 64 + 63 : count - 1;
    const int nblk = (pos0 + wg_last) / 32 + 1;
    const int my_last = r0 + 15 < count ? r0 + 15 : count - 1;
    const int my_blk = wave_rows ? (pos0 + my_last) / 32 : -1; // the wave's last block that holds a visible key
    // ... and its first, and the workgroup's first (a window or a chunk hides everything before it)
    const int my_lo = wave_rows ? first_visible(p, pos0 + r0) / 32 : 0, klo_last = wave_rows ? first_visible(p, pos0 + my_last) : 0;
    const int wg_lo = first_visible(p, pos0 + tile * 64) / 32;

    float m_run[MAPS], l_run[MAPS];
    f32x4 acc[MAPS][VT];
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
    {
        m_run[m] = -INFINITY;
        l_run[m] = 0.f;
#pragma unroll
        for (int ct = 0; ct < VT; ++ct)
            acc[m][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    uint4 kr[KPT], vr[VPT];
    // the page id of a block is fetched one block before its rows are requested: one memory latency per block, not two in a row
    const BlockWalk bw = block_walk(p, pos0 + tile * 64, nblk);
    // blocks below this index hold kept first keys, which every row sees whatever its own window (a wave whose rows start further
    // down than the workgroup's first takes part in them too)
    const int keep_blk = (p.mask == MASK_WINDOW && p.mask_keep > 0) ? (p.mask_keep + 31) / 32 : 0;
    int blk_next = table[walk_block(bw, 0) * 32 / page];
    auto request = [&](int vb) {
        const int key0 = walk_block(bw, vb) * 32;
        const int blk = blk_next, off = key0 % page;
        blk_next = table[vb + 1 < bw.n ? walk_block(bw, vb + 1) * 32 / page : key0 / page];
#pragma unroll
        for (int i = 0; i < KPT; ++i)
        {
            const int idx = tid + i * 256;
            if (K16 % 256 == 0 || idx < K16)
            {
                const int row = idx / (D / 8), piece = idx % (D / 8); // row = map * 32 + key
                kr[i] = *reinterpret_cast<const uint4*>(
                    kp + (((int64_t) blk * (p.kv_heads * MAPS) + g * MAPS + row / 32) * page + off + row % 32) * D + piece * 8);
            }
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i)
        {
            const int idx = tid + i * 256;
            if (V16 % 256 == 0 || idx < V16)
                vr[i] = *reinterpret_cast<const uint4*>(vp + (((int64_t) blk * p.kv_heads + gv) * V + idx / 4) * page + off + (idx % 4) * 8);
        }
    };
    request(0);
    for (int vb = 0; vb < bw.n; ++vb)
    {
        const int kb = walk_block(bw, vb);
#pragma unroll
        for (int i = 0; i < KPT; ++i)
        {
            const int idx = tid + i * 256;
            if (K16 % 256 == 0 || idx < K16)
                *reinterpret_cast<uint4*>(k_s + (idx / (D / 8)) * KP + (idx % (D / 8)) * 16) = kr[i];
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i)
        {
            const int idx = tid + i * 256;
            if (V16 % 256 == 0 || idx < V16)
                *reinterpret_cast<uint4*>(v_s + (idx / 4) * VP + (idx % 4) * 16) = vr[i];
        }
        __syncthreads();
        if (vb + 1 < bw.n)
            request(vb + 1);
        if (kb <= my_blk && (kb >= my_lo || kb < keep_blk))
        {
            const int key0 = kb * 32;
            uint4 pf[MAPS];
            const bool masked = key0 + 31 > pos0 + r0 || key0 < klo_last; // wave-uniform
#pragma unroll
            for (int m = 0; m < MAPS; ++m)
            {
                f32x4 s[2];
#pragma unroll
                for (int t = 0; t < 2; ++t)
                {
                    s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < DK; ++ks)
                        s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            as_bf16x8(*reinterpret_cast<const uint4*>(k_s + (m * 32 + t * 16 + col) * KP + (ks * 32 + 8 * g4) * 2)), qf[m][ks], s[t],
                            0, 0, 0);
                }
                pf[m] = softmax_block<VT>(s, m_run[m], l_run[m], acc[m], hm, masked, key0 + 4 * g4, qpos, klo);
            }
#pragma unroll
            for (int ct = 0; ct < VT; ++ct)
            {
                const char* vrow = v_s + (ct * 16 + col) * VP + 8 * g4;
                const uint2 lo = *reinterpret_cast<const uint2*>(vrow);
                const uint2 hi = *reinterpret_cast<const uint2*>(vrow + 32);
                const bf16x8 vf = as_bf16x8(make_uint4(lo.x, lo.y, hi.x, hi.y));
#pragma unroll
                for (int m = 0; m < MAPS; ++m)
                    acc[m][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, as_bf16x8(pf[m]), acc[m][ct], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    if (!wave_rows)
        return;
    // lane (col, g4) holds, for row col, channels ct * 16 + 4 g4 + i
    float inv[MAPS];
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
        inv[m] = finish_factor(p, h, m_run[m], l_run[m]);
    float ss = 0.f;
#pragma unroll
    for (int ct = 0; ct < VT; ++ct)
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            float o = acc[0][ct][i] * inv[0];
            if (MAPS == 2)
                o -= p.lambda * (acc[MAPS - 1][ct][i] * inv[MAPS - 1]);
            acc[0][ct][i] = o;
            ss += o * o;
        }
    float mul = 1.f;
    if (p.head_norm)
    {
        ss += __shfl_xor(ss, 16, 64);
        ss += __shfl_xor(ss, 32, 64);
        mul = p.out_scale / sqrtf(ss / (float) V + p.eps);
    }
    if (r0 + col < count)
    {
        mul *= out_gate_of(p, first + r0 + col, h);
        uint16_t* out = reinterpret_cast<uint16_t*>(p.out) + ((int64_t) (first + r0 + col) * p.heads + h) * V + 4 * g4;
#pragma unroll
        for (int ct = 0; ct < VT; ++ct)
            *reinterpret_cast<uint2*>(out + ct * 16) = make_uint2((uint32_t) f2bf(acc[0][ct][0] * mul) | ((uint32_t) f2bf(acc[0][ct][1] * mul) << 16),
                (uint32_t) f2bf(acc[0][ct][2] * mul) | ((uint32_t) f2bf(acc[0][ct][3] * mul) << 16));
    }
}

// attn_prefill_wide_kernel: the staged form for one map and long rows (dim of 160 and more), where the fragment reads out of LDS, not
// the matrix pipe, bound attn_prefill_kernel: a wave owns TWO 16-row tiles (a workgroup 128 rows) and every K and V^T fragment it reads
// from LDS feeds both, which halves the LDS traffic per score.  Same staging, same products, same finish.
template <int DK, int VT>
__global__ __launch_bounds__(256) void attn_prefill_wide_kernel(const StackAttnParams p, int min_count)
{
    constexpr int RT = 2, ROWS = 64 * RT;
    constexpr int D = DK * 32, V = VT * 16;
    constexpr int KP = D * 2 + 16, VP = 80;
    constexpr int K16 = 32 * (D / 8), V16 = V * 4;
    constexpr int KPT = (K16 + 255) / 256, VPT = (V16 + 255) / 256;
    __shared__ __attribute__((aligned(16))) char k_s[32 * KP];
    __shared__ __attribute__((aligned(16))) char v_s[V * VP];
    const int e = blockIdx.y, h = blockIdx.z;
    const int count = p.ent_count[e];
    if (count < min_count)
        return;
    const int tile = (count + ROWS - 1) / ROWS - 1 - (int) blockIdx.x;
    if (tile < 0)
        return;
    const int first = p.ent_first[e], pos0 = p.ent_pos0[e];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int col = lane & 15, g4 = lane >> 4;
    const HeadMap hd = head_map(p, h);
    const int g = hd.kh, gv = hd.vh;
    const int page = p.page;
    const int32_t* table = p.block_table + (int64_t) e * p.max_blocks;
    const HeadMods hm = head_mods(p, h);
    const uint16_t* kp = reinterpret_cast<const uint16_t*>(p.k_pool);
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(p.v_pool);

    int r0[RT], qpos[RT], klo[RT], my_blk[RT], my_lo[RT], klo_last[RT];
    bool rows_ok[RT];
    bf16x8 qf[RT][DK];
    float m_run[RT], l_run[RT];
    f32x4 acc[RT][VT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
    {
        r0[rt] = tile * ROWS + (w * RT + rt) * 16;
        rows_ok[rt] = r0[rt] < count; // wave-uniform
        const int qrow = r0[rt] + col < count ? r0[rt] + col : count - 1;
        qpos[rt] = pos0 + qrow;
        klo[rt] = first_visible(p, qpos[rt]);
#pragma unroll
        for (int ks = 0; ks < DK; ++ks)
            qf[rt][ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
                reinterpret_cast<const uint16_t*>(p.q) + ((int64_t) (first + qrow) * hd.q_heads + hd.qh) * D + ks * 32 + 8 * g4));
        const int my_last = r0[rt] + 15 < count ? r0[rt] + 15 : count - 1;
        my_blk[rt] = rows_ok[rt] ? (pos0 + my_last) / 32 : -1;
        my_lo[rt] = rows_ok[rt] ? first_visible(p, pos0 + r0[rt]) / 32 : 0;
        klo_last[rt] = rows_ok[rt] ? first_visible(p, pos0 + my_last) : 0;
        m_run[rt] = -INFINITY;
        l_run[rt] = 0.f;
#pragma unroll
        for (int ct = 0; ct < VT; ++ct)
            acc[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const int wg_last = tile * ROWS + ROWS - 1 < count ? tile * ROWS + ROWS - 1 : count - 1;
    const int nblk = (pos0 + wg_last) / 32 + 1;
    const int wg_lo = first_visible(p, pos0 + tile * ROWS) / 32;

    uint4 kr[KPT], vr[VPT];
    const BlockWalk bw = block_walk(p, pos0 + tile * ROWS, nblk);
    // blocks below this index hold kept first keys, which every row sees whatever its own window (a wave whose rows start further
    // down than the workgroup's first takes part in them too)
    const int keep_blk = (p.mask == MASK_WINDOW && p.mask_keep > 0) ? (p.mask_keep + 31) / 32 : 0;
    int blk_next = table[walk_block(bw, 0) * 32 / page];
    auto request = [&](int vb) {
        const int key0 = walk_block(bw, vb) * 32;
        const int blk = blk_next, off = key0 % page;
        blk_next = table[vb + 1 < bw.n ? walk_block(bw, vb + 1) * 32 / page : key0 / page];
#pragma unroll
        for (int i = 0; i < KPT; ++i)
        {
            const int idx = tid + i * 256;
            if (K16 % 256 == 0 || idx < K16)
            {
                const int row = idx / (D / 8), piece = idx % (D / 8);
                kr[i] = *reinterpret_cast<const uint4*>(kp + (((int64_t) blk * p.kv_heads + g) * page + off + row) * D + piece * 8);
            }
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i)
        {
            const int idx = tid + i * 256;
            if (V16 % 256 == 0 || idx < V16)
                vr[i] = *reinterpret_cast<const uint4*>(vp + (((int64_t) blk * p.kv_heads + gv) * V + idx / 4) * page + off + (idx % 4) * 8);
        }
    };
    request(0);
    for (int vb = 0; vb < bw.n; ++vb)
    {
        const int kb = walk_block(bw, vb);
#pragma unroll
        for (int i = 0; i < KPT; ++i)
        {
            const int idx = tid + i * 256;
            if (K16 % 256 == 0 || idx < K16)
                *reinterpret_cast<uint4*>(k_s + (idx / (D / 8)) * KP + (idx % (D / 8)) * 16) = kr[i];
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i)
        {
            const int idx = tid + i * 256;
            if (V16 % 256 == 0 || idx < V16)
                *reinterpret_cast<uint4*>(v_s + (idx / 4) * VP + (idx % 4) * 16) = vr[i];
        }
        __syncthreads();
        if (vb + 1 < bw.n)
            request(vb + 1);
        bool on[RT]; // wave-uniform
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
            on[rt] = kb <= my_blk[rt] && (kb >= my_lo[rt] || kb < keep_blk);
        if (on[0] || on[RT - 1])
        {
            const int key0 = kb * 32;
            f32x4 s[RT][2];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
                s[rt][0] = s[rt][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int ks = 0; ks < DK; ++ks)
                {
                    const bf16x8 kfr = as_bf16x8(*reinterpret_cast<const uint4*>(k_s + (t * 16 + col) * KP + (ks * 32 + 8 * g4) * 2));
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                        if (on[rt])
                            s[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kfr, qf[rt][ks], s[rt][t], 0, 0, 0);
                }
            uint4 pf[RT];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
            {
                pf[rt] = make_uint4(0, 0, 0, 0);
                if (on[rt])
                {
                    const bool masked = key0 + 31 > pos0 + r0[rt] || key0 < klo_last[rt];
                    pf[rt] = softmax_block<VT>(s[rt], m_run[rt], l_run[rt], acc[rt], hm, masked, key0 + 4 * g4, qpos[rt], klo[rt]);
                }
            }
#pragma unroll
            for (int ct = 0; ct < VT; ++ct)
            {
                const char* vrow = v_s + (ct * 16 + col) * VP + 8 * g4;
                const uint2 lo = *reinterpret_cast<const uint2*>(vrow);
                const uint2 hi = *reinterpret_cast<const uint2*>(vrow + 32);
                const bf16x8 vf = as_bf16x8(make_uint4(lo.x, lo.y, hi.x, hi.y));
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    if (on[rt])
                        acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, as_bf16x8(pf[rt]), acc[rt][ct], 0, 0, 0);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
    {
        if (!rows_ok[rt] || r0[rt] + col >= count)
            continue;
        const float mul = finish_factor(p, h, m_run[rt], l_run[rt]) * out_gate_of(p, first + r0[rt] + col, h);
        uint16_t* out = reinterpret_cast<uint16_t*>(p.out) + ((int64_t) (first + r0[rt] + col) * p.heads + h) * V + 4 * g4;
#pragma unroll
        for (int ct = 0; ct < VT; ++ct)
            *reinterpret_cast<uint2*>(out + ct * 16)
                = make_uint2((uint32_t) f2bf(acc[rt][ct][0] * mul) | ((uint32_t) f2bf(acc[rt][ct][1] * mul) << 16),
                    (uint32_t) f2bf(acc[rt][ct][2] * mul) | ((uint32_t) f2bf(acc[rt][ct][3] * mul) << 16));
    }
}

// Second pass of the key split: one wave per (row, head) combines the ks partials of each map, then the differential combination,
// the head norm and the bfloat16 store.
template <int MAPS>
__global__ __launch_bounds__(64) void attn_split_merge_kernel(const StackAttnParams p, int ks, int below_count)
{
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    if (p.ent_count[p.tok_entry[t]] >= below_count)
        return;
    const int V = p.vdim;
    const float* base = p.split_ws + (((int64_t) t * p.heads + h) * ks) * MAPS * (V + 2);
    // lane l < ks * MAPS owns partial (split l / MAPS, map l % MAPS): all maxima and sums are fetched at once, the weights are
    // formed with wave reductions and handed to the channel lanes by shuffles
    const bool owner = lane < ks * MAPS;
    const float pm = owner ? base[lane * (V + 2) + V] : -INFINITY;
    const float pl = owner ? base[lane * (V + 2) + V + 1] : 0.f;
    float wl = 0.f;
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
    {
        const bool mine = owner && lane % MAPS == m;
        const float M = wave_max(mine ? pm : -INFINITY);
        const float e_ = p.weights == WEIGHTS_SIGMOID ? 1.f : (mine && pm != -INFINITY ? __builtin_amdgcn_exp2f(pm - M) : 0.f);
        const float L = wave_sum(mine ? e_ * pl : 0.f);
        if (mine)
            wl = e_ * finish_factor(p, h, M, L);
    }
    constexpr int MC = 4; // vdim <= 256: four channels per lane
    float o[MC], ss = 0.f;
    float a[MC][MAPS];
#pragma unroll
    for (int c = 0; c < MC; ++c)
#pragma unroll
        for (int m = 0; m < MAPS; ++m)
            a[c][m] = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxSplits * MAPS; ++i)
    {
        const float wgt = __shfl(wl, i, 64);
        if (i < ks * MAPS) // wave-uniform
        {
#pragma unroll
            for (int c = 0; c < MC; ++c)
                if (lane + c * 64 < V)
                    a[c][i % MAPS] += wgt * base[i * (V + 2) + lane + c * 64];
        }
    }
#pragma unroll
    for (int c = 0; c < MC; ++c)
    {
        o[c] = 0.f;
        if (lane + c * 64 < V)
        {
            o[c] = MAPS == 2 ? a[c][0] - p.lambda * a[c][MAPS - 1] : a[c][0];
            ss += o[c] * o[c];
        }
    }
    float mul = 1.f;
    if (p.head_norm)
        mul = p.out_scale / sqrtf(wave_sum(ss) / (float) V + p.eps);
    mul *= out_gate_of(p, t, h);
    uint16_t* out = reinterpret_cast<uint16_t*>(p.out) + ((int64_t) t * p.heads + h) * V;
#pragma unroll
    for (int c = 0; c < MC; ++c)
        if (lane + c * 64 < V)
            out[lane + c * 64] = f2bf(o[c] * mul);
}

template <int MAPS, int DK, int VT>
int launch_tile(const StackAttnParams& p, hipStream_t stream)
{
    constexpr int NW = 4;
    const size_t lds = sizeof(float) * ((size_t) NW * MAPS * 16 * VT * 16 + (size_t) NW * MAPS * 16 * 2);
    const void* fn = reinterpret_cast<const void*>(&attn_tile_kernel<MAPS, DK, VT, NW>);
    launch_util::ensure_dynamic_lds(fn, lds);
    // entries of PREFILL_ROWS rows and more go to the staged form, the rest (decoded tokens, short portions) to the key-split form;
    // a mixed step launches both, each skipping the other's entries
    static const int PREFILL_ROWS = [] {
        const char* v = std::getenv("TLLM_STACK_PREFILL_ROWS"); // measurement knob: rows from which an entry takes the staged form
        return v && std::atoi(v) > 0 ? std::atoi(v) : 32;
    }();
    const int small_rows = p.max_count < PREFILL_ROWS ? p.max_count : (p.tokens > p.max_count ? PREFILL_ROWS - 1 : 0);
    if (p.max_count >= PREFILL_ROWS)
    {
        // the wide form (128 rows per workgroup) where it still fills the chip; otherwise twice as many workgroups of 64 rows
        bool wide = false;
        if constexpr (MAPS == 1 && DK >= 5)
        {
            const char* force = std::getenv("TLLM_STACK_WIDE_PREFILL"); // test / measurement knob: 1 = always, 0 = never
            wide = !p.head_norm
                && (force ? force[0] == '1' : (int64_t) ((p.max_count + 127) / 128) * p.entries * p.heads >= launch_util::device_cus());
        }
        if constexpr (MAPS == 1 && DK >= 5)
        {
            if (wide)
            {
                const dim3 pg((p.max_count + 127) / 128, p.entries, p.heads);
                hipLaunchKernelGGL((attn_prefill_wide_kernel<DK, VT>), pg, dim3(256), 0, stream, p, PREFILL_ROWS);
            }
        }
        if (!wide)
        {
            const dim3 pg((p.max_count + 63) / 64, p.entries, p.heads);
            hipLaunchKernelGGL((attn_prefill_kernel<MAPS, DK, VT>), pg, dim3(256), 0, stream, p, PREFILL_ROWS);
        }
    }
    if (small_rows > 0)
    {
        // a step of decoded tokens only (every entry within one tile, few rows in all): the keys of an (entry, head) are split over
        // ks workgroups so that a long context is walked by ks * NW waves, two key blocks or so each
        int ks = 1;
        if (p.split_ws && p.max_count <= 16 && p.tokens <= kSplitRows)
        {
            // a window or a chunk bounds the keys a row walks
            const int span = p.mask == MASK_CAUSAL ? p.max_context
                                                   : std::min(p.max_context, p.mask_size + 31 + (p.mask_keep > 0 ? p.mask_keep + 31 : 0));
            const int nblk = (span + 31) / 32;
            ks = std::min(kMaxSplits, (nblk + 2 * NW - 1) / (2 * NW));
        }
        // single decoded tokens whose heads share one key/value head and carry no per-head numbers: 16 heads are the tile's rows
        const int head_rows = (p.max_count == 1 && p.kv_heads == 1 && !p.cross_values && MAPS == 1 && p.heads >= 8 && !p.temp && !p.slope && !p.log_r1 && !p.sink
                                  && !p.wbias && !p.head_norm)
            ? 1
            : 0;
        const dim3 grid(ks > 1 ? ks : (small_rows + 15) / 16, p.entries, head_rows ? (p.heads + 15) / 16 : p.heads);
        hipLaunchKernelGGL((attn_tile_kernel<MAPS, DK, VT, NW>), grid, dim3(NW * 64), lds, stream, p, PREFILL_ROWS, ks, head_rows);
        if (ks > 1)
            hipLaunchKernelGGL((attn_split_merge_kernel<MAPS>), dim3(p.tokens, p.heads), dim3(64), 0, stream, p, ks, PREFILL_ROWS);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess)
    {
        set_error("stack_attention (tile kernels) launch failed: %s", hipGetErrorString(e));
        return -1;
    }
    return 0;
}

template <int MAPS, int DK>
int launch_tile_v(const StackAttnParams& p, hipStream_t stream)
{
    switch (p.vdim)
    {
    case 32: return launch_tile<MAPS, DK, 2>(p, stream);
    case 64: return launch_tile<MAPS, DK, 4>(p, stream);
    case 128: return launch_tile<MAPS, DK, 8>(p, stream);
    default: return 1;
    }
}

// one shared key/value head of dim = latent + rotated part, vdim = latent (latent attention in absorbed form)
int launch_tile_latent(const StackAttnParams& p, hipStream_t stream)
{
    if (p.dim == 160 && p.vdim == 128)
        return launch_tile<1, 5, 8>(p, stream);
    if (p.dim == 320 && p.vdim == 256)
        return launch_tile<1, 10, 16>(p, stream);
    return 1;
}

template <int MAPS>
int launch_tile_d(const StackAttnParams& p, hipStream_t stream)
{
    switch (p.dim)
    {
    case 32: return launch_tile_v<MAPS, 1>(p, stream);
    case 64: return launch_tile_v<MAPS, 2>(p, stream);
    case 128: return launch_tile_v<MAPS, 4>(p, stream);
    default: return 1;
    }
}

} // namespace

// partials of the cross-workgroup key split: steps of up to kSplitRows rows, up to kMaxSplits splits per (row, head)
size_t stack_attn_workspace_floats(int32_t heads, int32_t maps, int32_t vdim)
{
    return (size_t) kSplitRows * heads * kMaxSplits * maps * (vdim + 2);
}

// the tile kernel's shapes: bfloat16, dim 32 / 64 / 128, vdim 32 / 64 / 128, pages of a multiple of 32 keys
bool stack_attention_tiled(const StackAttnParams& p)
{
    const bool std_shape = (p.dim == 32 || p.dim == 64 || p.dim == 128) && (p.vdim == 32 || p.vdim == 64 || p.vdim == 128);
    const bool latent_shape = p.maps == 1 && p.kv_heads == 1 && ((p.dim == 160 && p.vdim == 128) || (p.dim == 320 && p.vdim == 256));
    // what only the general kernels do: head-mixed weights, a gate per channel, kept first keys under a window
    if (p.talk || (p.out_gate && p.gate_wide))
        return false;
    return p.dtype == DT_BF16 && (std_shape || latent_shape) && p.page % 32 == 0 && p.max_count > 0 && p.entries > 0 && !(reinterpret_cast<uintptr_t>(p.q) & 15)
        && !(reinterpret_cast<uintptr_t>(p.k_pool) & 15) && !(reinterpret_cast<uintptr_t>(p.v_pool) & 7);
}

int launch_stack_attention(const StackAttnParams& p, hipStream_t stream)
{
    if (p.tokens <= 0)
        return 0;
    static const bool general_only = [] {
        const char* v = std::getenv("TLLM_STACK_ATTN_GENERAL"); // measurement knob: 1 = every shape on the general kernel
        return v && v[0] == '1';
    }();
    if (!general_only && p.talk && p.pair_ws && p.maps == 1 && p.heads >= 1 && p.kv_heads >= 1 && p.heads % p.kv_heads == 0)
    {
        // head-mixed weights on the tile kernels: every query head's weights over every value head's rows (kv_heads x the pairs of a
        // plain launch), then the mixing as a sum over those terms - the mixing is linear in the weights, so it commutes with P V
        StackAttnParams c = p;
        c.talk = nullptr;
        c.out_gate = nullptr;
        c.heads = p.heads * p.kv_heads;
        c.cross_values = 1;
        c.out = p.pair_ws;
        if (stack_attention_tiled(c))
        {
            const int rc = launch_tile_d<1>(c, stream);
            if (rc < 0)
                return rc;
            if (rc == 0)
                return launch_stack_talk_combine(p, p.pair_ws, stream);
        }
    }
    if (!general_only && p.heads >= 1 && p.kv_heads >= 1 && p.heads % p.kv_heads == 0 && stack_attention_tiled(p))
    {
        int rc = p.maps == 2 ? launch_tile_d<2>(p, stream) : (p.maps == 1 ? launch_tile_d<1>(p, stream) : 1);
        if (rc == 1 && p.maps == 1)
            rc = launch_tile_latent(p, stream);
        if (rc <= 0)
            return rc;
    }
    return launch_stack_attention_general(p, stream);
}

} // namespace kernels
} // namespace tllm
