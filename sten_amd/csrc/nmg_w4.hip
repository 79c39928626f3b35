// Decode-shape linear layer on a 2:4-pruned, int4-quantised weight (the benchmark's "sparse-marlin"
// configuration: Llama-like MLP weight, 2:4 along K, symmetric int4 with one fp16 scale per 128
// dense positions of a row, few tokens).  Memory-bound: 0.39 bytes per dense weight element are
// streamed once, dequantised in registers and multiplied on the sparse matrix cores
// (V_SMFMAC_F32_32X32X32_F16), tokens padded to the 32 columns of the instruction.
//
// What the reference has for this configuration is a call into an external library with random
// operands and no assertion (tests/test_sparse_marlin.py:42-57,113), so the format below is this
// library's own and results are pinned against the dequantised dense product only.
//
// Quantisation (per row, per group of 128 dense positions):
//   keep, in every aligned group of 4, the 2 entries of largest magnitude (ties: lower position);
//   s = fp16(max |kept| / 7), or 1 if that is 0;  q = clamp(rint(w / s) + 8, 0, 15);
//   the dequantised weight is fp16((q - 8) * s).
// Layout, for a block of 32 rows (mb) and a group of 128 positions (kq) -- one record of
//   B     [MB][KQ][64 lanes][16 bytes]  the 4 x 8 nibbles lane l feeds to the 4 instructions of the
//                                       group (row l%32, same lane/pair order as the fragpack
//                                       operand); element e of instruction i sits in 32-bit word i
//                                       at bit 4*(e/2) + 16*(e%2), so that a shift and a mask
//                                       yield two fp16 lanes at once
//   meta  [MB][KQ][64 lanes][2] u32     2-bit positions, 16 bits per instruction
//   s     [MB][KQ][32 rows] fp16
// Rows are padded to a multiple of 32 with q = 8 (zero).
#include "nmg_common.h"
#include "nmg_tile.h"

namespace nmg {

typedef _Float16 w4_f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 w4_f16x16 __attribute__((ext_vector_type(16)));
typedef _Float16 w4_f16x2 __attribute__((ext_vector_type(2)));

struct W4Params {
    const void *w;       // dense input of pack / output of unpack
    void *B;
    uint32_t *meta;
    void *s;
    const void *x;
    void *y;
    const void *bias;
    int64_t M, K, T, ldw, ldx, ldy;
    int MB, KQ;
};

// lane / pair of the aligned 4-group kg (0..7) of a 32-wide instruction step (see nmg_smfmac.hip)
__device__ __forceinline__ void w4_slot(int kg, int &ga, int &q)
{
    ga = (kg >> 1) & 1;
    q = ((kg >> 2) << 1) | (kg & 1);
}

// One thread per (row, group of 128): prune, scale, quantise, scatter into the record.
__global__ __launch_bounds__(256) void w4_pack_kernel(W4Params P)
{
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = (int64_t)P.MB * 32 * P.KQ;
    if (gid >= total) return;
    const int kq = (int)(gid % P.KQ);
    const int64_t row = gid / P.KQ;
    const int mb = (int)(row >> 5), r = (int)(row & 31);
    const bool live = row < P.M;
    const __half *w = (const __half *)P.w + (live ? row : 0) * P.ldw + (int64_t)kq * 128;

    float kept[64];
    uint8_t pos[64];
    float amax = 0.f;
    for (int gq = 0; gq < 32; gq++) {
        float a[4];
        for (int i = 0; i < 4; i++) a[i] = live ? __half2float(w[gq * 4 + i]) : 0.f;
        // the two largest magnitudes, lower position first on ties, positions kept increasing
        int i0 = 0;
        for (int i = 1; i < 4; i++)
            if (fabsf(a[i]) > fabsf(a[i0])) i0 = i;
        int i1 = -1;
        for (int i = 0; i < 4; i++) {
            if (i == i0) continue;
            if (i1 < 0 || fabsf(a[i]) > fabsf(a[i1])) i1 = i;
        }
        const int lo = i0 < i1 ? i0 : i1, hi = i0 < i1 ? i1 : i0;
        kept[2 * gq] = a[lo];
        kept[2 * gq + 1] = a[hi];
        pos[2 * gq] = (uint8_t)lo;
        pos[2 * gq + 1] = (uint8_t)hi;
        amax = fmaxf(amax, fmaxf(fabsf(a[lo]), fabsf(a[hi])));
    }
    __half sh = __float2half(amax / 7.0f);
    if (__half2float(sh) == 0.f) sh = __float2half(1.0f);
    const float s = __half2float(sh);
    ((__half *)P.s)[((int64_t)mb * P.KQ + kq) * 32 + r] = sh;

    uint32_t words[2][4] = {{0, 0, 0, 0}, {0, 0, 0, 0}};   // [ga][instruction]
    uint32_t meta[2][2] = {{0, 0}, {0, 0}};                // [ga][pair of instructions]
    for (int gq = 0; gq < 32; gq++) {
        const int ins = gq >> 3, kg = gq & 7;
        int ga, q;
        w4_slot(kg, ga, q);
        for (int i = 0; i < 2; i++) {
            float qf = rintf(kept[2 * gq + i] / s) + 8.0f;
            qf = fminf(fmaxf(qf, 0.f), 15.f);
            const uint32_t nib = live ? (uint32_t)qf : 8u;
            const int e = 2 * q + i;
            words[ga][ins] |= nib << (4 * (e >> 1) + 16 * (e & 1));
        }
        const uint32_t pp = live ? (uint32_t)(pos[2 * gq] | (pos[2 * gq + 1] << 2)) : 4u;
        meta[ga][ins >> 1] |= pp << (4 * q + 16 * (ins & 1));
    }
    for (int ga = 0; ga < 2; ga++) {
        const int64_t rec = ((int64_t)mb * P.KQ + kq) * 64 + r + 32 * ga;
        u32x4 v = {words[ga][0], words[ga][1], words[ga][2], words[ga][3]};
        ((u32x4 *)P.B)[rec] = v;
        P.meta[rec * 2] = meta[ga][0];
        P.meta[rec * 2 + 1] = meta[ga][1];
    }
}

// 8 nibbles of one instruction -> 8 fp16 weights: (1024 + q) - 1032 = q - 8 exactly, then one
// rounding in the product with the scale.  A nibble at bits 4..7 of a half is read in place
// under the exponent of 64, where the last mantissa place is 1/16: (64 + q) - 72.
__device__ __forceinline__ u32x4 w4_dequant(uint32_t word, w4_f16x2 s2)
{
    u32x4 out;
    const w4_f16x2 off_lo = {(_Float16)1032.0f, (_Float16)1032.0f};
    const w4_f16x2 off_hi = {(_Float16)72.0f, (_Float16)72.0f};
    uint32_t o[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        union {
            uint32_t u;
            w4_f16x2 h;
        } c;
        const uint32_t w = t < 2 ? word : word >> 8;
        // (w & mask) | exponent in one instruction (two literals do not fit one: the mask comes
        // in a register)
        if (t & 1) {
            asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(c.u) : "v"(w), "v"(0x00F000F0u), "s"(0x54005400u));
            c.h = (c.h - off_hi) * s2;
        } else {
            asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(c.u) : "v"(w), "v"(0x000F000Fu), "s"(0x64006400u));
            c.h = (c.h - off_lo) * s2;
        }
        o[t] = c.u;
    }
    out.x = o[0];
    out.y = o[1];
    out.z = o[2];
    out.w = o[3];
    return out;
}

// One thread per (row, group of 128): the dequantised dense weight, zeros at dropped positions.
__global__ __launch_bounds__(256) void w4_unpack_kernel(W4Params P)
{
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= P.M * P.KQ) return;
    const int kq = (int)(gid % P.KQ);
    const int64_t row = gid / P.KQ;
    const int mb = (int)(row >> 5), r = (int)(row & 31);
    const _Float16 sv = ((const _Float16 *)P.s)[((int64_t)mb * P.KQ + kq) * 32 + r];
    const w4_f16x2 s2 = {sv, sv};
    uint16_t *out = (uint16_t *)P.w + row * P.ldw + (int64_t)kq * 128;
    for (int i = 0; i < 128; i++) out[i] = 0;
    for (int ga = 0; ga < 2; ga++) {
        const int64_t rec = ((int64_t)mb * P.KQ + kq) * 64 + r + 32 * ga;
        const u32x4 v = ((const u32x4 *)P.B)[rec];
        const uint32_t words[4] = {v.x, v.y, v.z, v.w};
        for (int ins = 0; ins < 4; ins++) {
            const u32x4 d = w4_dequant(words[ins], s2);
            const uint32_t dw[4] = {d.x, d.y, d.z, d.w};
            const uint32_t mt = (P.meta[rec * 2 + (ins >> 1)] >> (16 * (ins & 1))) & 0xFFFFu;
            for (int q = 0; q < 4; q++) {
                const int kg = 4 * (q >> 1) + 2 * ga + (q & 1);
                for (int i = 0; i < 2; i++) {
                    const int p = (mt >> (4 * q + 2 * i)) & 3;
                    out[ins * 32 + kg * 4 + p] = (uint16_t)(dw[q] >> (16 * i));
                }
            }
        }
    }
}

// Streaming product for T <= 16 tokens: one workgroup per 32 rows, its NW wavefronts split K,
// partial sums reduced through LDS.
template <int NW, int W4_NB, int RB>
__global__ __launch_bounds__(64 * NW) void w4_linear_kernel(W4Params P)
{
    // RB blocks of 32 rows per workgroup share each wavefront's activation fragments: every
    // workgroup reads all T x K activations through L2, which at 16 tokens outweighs its share
    // of the weight.
    __shared__ float red[NW][RB * 32][17];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int mb0 = blockIdx.x * RB;
    const int KQ = P.KQ;
    const int j = lane & 31, h = lane >> 5;
    const u32x4 zero4 = {0, 0, 0, 0};
    const int per = (KQ + NW - 1) / NW;
    const int kq_lo = wave * per, kq_hi = min(KQ, kq_lo + per);

    f32x16 acc[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[rb][r] = 0.f;

    const u32x4 *bv = (const u32x4 *)P.B + lane;
    const uint2 *mv = (const uint2 *)P.meta + lane;
    const _Float16 *sv = (const _Float16 *)P.s + j;
    const bool tok_ok = j < P.T;
    const unsigned char *xrow = (const unsigned char *)P.x + ((int64_t)(tok_ok ? j : 0) * P.ldx + 16 * h) * 2;

    struct Batch {
        u32x4 a[RB];
        uint2 ix[RB];
        _Float16 s[RB];
        u32x4 b[4][2];
    };
    auto fetch = [&](Batch &B, int kq) {
        const bool live = kq < kq_hi;
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            const bool ok = live && mb0 + rb < P.MB;
            const int64_t rec = (int64_t)(mb0 + rb) * KQ + kq;
            B.a[rb] = ok ? bv[rec * 64] : zero4;
            B.ix[rb] = ok ? mv[rec * 64] : make_uint2(0x44444444u, 0x44444444u);
            B.s[rb] = ok ? sv[rec * 32] : (_Float16)0.f;
        }
#pragma unroll
        for (int ins = 0; ins < 4; ins++)
#pragma unroll
            for (int c = 0; c < 2; c++)
                B.b[ins][c] = (live && tok_ok) ? *(const u32x4 *)(xrow + ((int64_t)kq * 128 + ins * 32 + 8 * c) * 2)
                                               : zero4;
    };
    auto consume = [&](const Batch &B) {
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            const w4_f16x2 s2 = {B.s[rb], B.s[rb]};
            const uint32_t words[4] = {B.a[rb].x, B.a[rb].y, B.a[rb].z, B.a[rb].w};
#pragma unroll
            for (int ins = 0; ins < 4; ins++) {
                union {
                    u32x4 u4;
                    w4_f16x8 v;
                } ca;
                ca.u4 = w4_dequant(words[ins], s2);
                union {
                    u32x4 u4[2];
                    w4_f16x16 v;
                } cb;
                cb.u4[0] = B.b[ins][0];
                cb.u4[1] = B.b[ins][1];
                const int ix = (int)(ins < 2 ? B.ix[rb].x : B.ix[rb].y);
                if (ins & 1)
                    acc[rb] = __builtin_amdgcn_smfmac_f32_32x32x32_f16(ca.v, cb.v, acc[rb], ix, 0, 1);
                else
                    acc[rb] = __builtin_amdgcn_smfmac_f32_32x32x32_f16(ca.v, cb.v, acc[rb], ix, 0, 0);
            }
        }
    };

    // W4_NB groups of 128 in flight per wavefront
    Batch bt[W4_NB];
#pragma unroll
    for (int u = 0; u < W4_NB; u++) fetch(bt[u], kq_lo + u);
    for (int kq = kq_lo; kq < kq_hi; kq += W4_NB) {
#pragma unroll
        for (int u = 0; u < W4_NB; u++) {
            consume(bt[u]);
            fetch(bt[u], kq + W4_NB + u);
        }
    }
    // D[row][col = token]: lane holds token j, rows 8*(r/4) + 4*h + r%4
    if (j < 16) {
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int r = 0; r < 16; r++) red[wave][rb * 32 + (r >> 2) * 8 + h * 4 + (r & 3)][j] = acc[rb][r];
    }
    __syncthreads();
    for (int e = tid; e < RB * 32 * 16; e += 64 * NW) {
        const int line = e % (RB * 32), tok = e / (RB * 32);
        const int64_t f = (int64_t)mb0 * 32 + line;
        if (tok >= P.T || f >= P.M) continue;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NW; w++) s += red[w][line][tok];
        if (P.bias) s += __half2float(((const __half *)P.bias)[f]);
        ((__half *)P.y)[tok * P.ldy + f] = __float2half(s);
    }
}

// The same product with the activations staged through LDS: a wavefront's direct activation loads
// touch 32 bytes of a token row per instruction; here a group's 4 ND token rows x 256 bytes arrive
// by row-contiguous DMA loads into a staging area private to the wavefront (no barrier), issued
// before the group's weight loads so that one counted wait covers both; 16-byte pieces of a row
// are XOR-swizzled with the row number so that a fragment read hits distinct banks.  A wavefront
// keeps NS groups in flight (four up to 8 tokens: all of its range of a 4096-wide reduction is
// requested before anything else happens; two beyond, where a group's activations take 3-4 KiB of
// LDS).  Groups are refilled while a whole round of real ones is left; the last round waits for
// exactly the groups behind each one and requests nothing, so no load is in flight at the end
// that nobody reads.  A stand-in (fewer groups than sets, or the refills of the round before the
// last) reads one cache line at the start of the operands.
template <int NW, int ND, int NS>
__global__ __launch_bounds__(64 * NW) void w4_linear_staged_kernel(W4Params P)
{
    constexpr int OPS = ND + 3;
    constexpr int BUF = ND * 1024;
    static_assert((NS - 1) * OPS < 64, "vmcnt is a 6-bit counter");
    extern __shared__ __align__(16) unsigned char w4_smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int mb = blockIdx.x;
    const int KQ = P.KQ;
    const int j = lane & 31, h = lane >> 5;
    const int per = (KQ + NW - 1) / NW;
    const int kq_lo = wave * per, kq_hi = min(KQ, kq_lo + per);
    unsigned char *stage = w4_smem + wave * (NS * BUF);

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;

    const unsigned char *bv = (const unsigned char *)P.B + ((int64_t)mb * KQ) * 1024;
    const unsigned char *mv = (const unsigned char *)P.meta + ((int64_t)mb * KQ) * 512;
    const unsigned char *sv = (const unsigned char *)P.s + ((int64_t)mb * KQ) * 64;
    const uint32_t lane16 = lane * 16, lane8 = lane * 8, row2 = j * 2;
    uint32_t x_off[ND];
#pragma unroll
    for (int i = 0; i < ND; i++) {
        const int row = 4 * i + (lane >> 4);
        const int q = (lane & 15) ^ (row & 15);
        const int64_t tok = row < P.T ? row : P.T - 1;   // surplus rows repeat the last token, never stored
        x_off[i] = (uint32_t)((tok * P.ldx + q * 8) * 2);
    }
    int b_off[4][2];
#pragma unroll
    for (int ins = 0; ins < 4; ins++)
#pragma unroll
        for (int c = 0; c < 2; c++) b_off[ins][c] = (j & 15) * 256 + (((ins * 4 + 2 * h + c) ^ (j & 15)) << 4);

    struct WSet {
        u32x4 a;
        uint2 ix;
        uint32_t s;
    };
    WSet ws[NS];
    // (`s_nop 4`: a scalar base that the compiler reads back from a vector register lane needs five
    // wait states before a memory instruction may use it, and the compiler does not look into
    // instruction statements)
    auto issue = [&](int kq, unsigned char *buf, WSet &W) __attribute__((always_inline)) {
        const bool real = kq < kq_hi;
        const int kc = real ? kq : 0;         // a stand-in: same count of operations, one cache line each
        const unsigned char *xb = (const unsigned char *)P.x + (int64_t)kc * 256;
#pragma unroll
        for (int i = 0; i < ND; i++)
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(xb + x_off[i]), (lds_ptr_t)(buf + i * 1024), 16, 0, 0);
        const unsigned char *pb = bv + (int64_t)kc * 1024, *pm = mv + (int64_t)kc * 512, *ps = sv + (int64_t)kc * 64;
        const uint32_t o16 = real ? lane16 : 0u, o8 = real ? lane8 : 0u, o2 = real ? row2 : 0u;
        asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2" : "=v"(W.a) : "v"(o16), "s"(pb) : "memory");
        asm volatile("s_nop 4\n\tglobal_load_dwordx2 %0, %1, %2" : "=v"(W.ix) : "v"(o8), "s"(pm) : "memory");
        asm volatile("s_nop 4\n\tglobal_load_ushort %0, %1, %2" : "=v"(W.s) : "v"(o2), "s"(ps) : "memory");
    };
    // set k has landed: `left` groups requested behind it may still be on their way
    auto landed = [&](WSet &W, auto left_tag) __attribute__((always_inline)) {
        constexpr int LEFT = decltype(left_tag)::value;
        asm volatile("s_waitcnt vmcnt(%3)" : "+v"(W.a), "+v"(W.ix), "+v"(W.s) : "n"(LEFT * OPS) : "memory");
    };
    auto consume = [&](const unsigned char *buf, const WSet &W) __attribute__((always_inline)) {
        u32x4 b[4][2];
#pragma unroll
        for (int ins = 0; ins < 4; ins++)
#pragma unroll
            for (int c = 0; c < 2; c++) b[ins][c] = *(const u32x4 *)(buf + b_off[ins][c]);
        union {
            uint16_t u;
            _Float16 f;
        } sc;
        sc.u = (uint16_t)W.s;
        const w4_f16x2 s2 = {sc.f, sc.f};
        const uint32_t words[4] = {W.a.x, W.a.y, W.a.z, W.a.w};
#pragma unroll
        for (int ins = 0; ins < 4; ins++) {
            union {
                u32x4 u4;
                w4_f16x8 v;
            } ca;
            ca.u4 = w4_dequant(words[ins], s2);
            union {
                u32x4 u4[2];
                w4_f16x16 v;
            } cb;
            cb.u4[0] = b[ins][0];
            cb.u4[1] = b[ins][1];
            const int ix = (int)(ins < 2 ? W.ix.x : W.ix.y);
            if (ins & 1)
                acc = __builtin_amdgcn_smfmac_f32_32x32x32_f16(ca.v, cb.v, acc, ix, 0, 1);
            else
                acc = __builtin_amdgcn_smfmac_f32_32x32x32_f16(ca.v, cb.v, acc, ix, 0, 0);
        }
    };

#pragma unroll
    for (int k = 0; k < NS; k++) issue(kq_lo + k, stage + k * BUF, ws[k]);
    int kq0 = kq_lo;
    for (; kq0 + NS < kq_hi; kq0 += NS) {
#pragma unroll
        for (int k = 0; k < NS; k++) {
            landed(ws[k], std::integral_constant<int, NS - 1>{});
            __builtin_amdgcn_sched_barrier(0);
            consume(stage + k * BUF, ws[k]);
            __builtin_amdgcn_sched_barrier(0);
            issue(kq0 + NS + k, stage + k * BUF, ws[k]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    auto last = [&](WSet &W, auto k_tag) __attribute__((always_inline)) {
        constexpr int K = decltype(k_tag)::value;
        landed(W, std::integral_constant<int, NS - 1 - K>{});
        __builtin_amdgcn_sched_barrier(0);
        if (kq0 + K < kq_hi) consume(stage + K * BUF, W);
        __builtin_amdgcn_sched_barrier(0);
    };
    last(ws[0], std::integral_constant<int, 0>{});
    last(ws[1], std::integral_constant<int, 1>{});
    if constexpr (NS == 4) {
        last(ws[2], std::integral_constant<int, 2>{});
        last(ws[3], std::integral_constant<int, 3>{});
    }
    __syncthreads();
    float(*red)[32][17] = (float(*)[32][17])w4_smem;
    if (j < 16) {
#pragma unroll
        for (int r = 0; r < 16; r++) red[wave][(r >> 2) * 8 + h * 4 + (r & 3)][j] = acc[r];
    }
    __syncthreads();
    for (int e = tid; e < 32 * 16; e += 64 * NW) {
        const int line = e & 31, tok = e >> 5;
        const int64_t f = (int64_t)mb * 32 + line;
        if (tok >= P.T || f >= P.M) continue;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NW; w++) s += red[w][line][tok];
        if (P.bias) s += __half2float(((const __half *)P.bias)[f]);
        ((__half *)P.y)[tok * P.ldy + f] = __float2half(s);
    }
}

template <int NW, int ND> static void w4_launch_staged(const W4Params &P, hipStream_t s)
{
    constexpr int NS = ND <= 2 ? 4 : 2;
    // (the sums of the wavefronts reuse the staging area: 32 x 17 floats per wavefront)
    constexpr size_t lds = (size_t)NW * (NS * ND * 1024 > 32 * 17 * 4 ? NS * ND * 1024 : 32 * 17 * 4);
    hipLaunchKernelGGL((w4_linear_staged_kernel<NW, ND, NS>), dim3((unsigned)P.MB), dim3(64 * NW), lds, s, P);
}
template <int NW> static void w4_launch_staged_nd(const W4Params &P, hipStream_t s)
{
    switch ((int)(P.T + 3) / 4) {
    case 1: w4_launch_staged<NW, 1>(P, s); break;
    case 2: w4_launch_staged<NW, 2>(P, s); break;
    case 3: w4_launch_staged<NW, 3>(P, s); break;
    default: w4_launch_staged<NW, 4>(P, s); break;
    }
}

template <int NW, int NB, int RB> static void w4_launch(const W4Params &P, hipStream_t s)
{
    hipLaunchKernelGGL((w4_linear_kernel<NW, NB, RB>), dim3((unsigned)((P.MB + RB - 1) / RB)), dim3(64 * NW), 0, s, P);
}

static int w4_check(int64_t M, int64_t K)
{
    NMG_REQUIRE(M >= 0 && K >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(K % 128 == 0, NMG_ERR_UNSUPPORTED, "K (%lld) must be a multiple of the scale group, 128",
                (long long)K);
    NMG_REQUIRE(M < ((int64_t)1 << 31) && K < ((int64_t)1 << 31), NMG_ERR_UNSUPPORTED, "extent too large");
    return NMG_OK;
}

}  // namespace nmg

using namespace nmg;

extern "C" int nmg_w4_sizes(int64_t M, int64_t K, int64_t *b_bytes, int64_t *meta_words, int64_t *scales)
{
    if (int rc = w4_check(M, K)) return rc;
    NMG_REQUIRE(b_bytes && meta_words && scales, NMG_ERR_ARG, "null output pointer");
    const int64_t rec = ((M + 31) / 32) * (K / 128);
    *b_bytes = rec * 64 * 16;
    *meta_words = rec * 64 * 2;
    *scales = rec * 32;
    return NMG_OK;
}

extern "C" int nmg_w4_pack(const void *d_w, int64_t ldw, int64_t M, int64_t K, void *d_B, void *d_meta,
                           void *d_s, void *stream)
{
    if (int rc = w4_check(M, K)) return rc;
    NMG_REQUIRE(ldw >= K, NMG_ERR_ARG, "leading dimension smaller than row length");
    if (M == 0 || K == 0) return NMG_OK;
    NMG_REQUIRE(d_w && d_B && d_meta && d_s, NMG_ERR_ARG, "null device pointer");
    W4Params P{};
    P.w = d_w;
    P.B = d_B;
    P.meta = (uint32_t *)d_meta;
    P.s = d_s;
    P.M = M;
    P.K = K;
    P.ldw = ldw;
    P.MB = (int)((M + 31) / 32);
    P.KQ = (int)(K / 128);
    const int64_t total = (int64_t)P.MB * 32 * P.KQ;
    hipLaunchKernelGGL(w4_pack_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, P);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

extern "C" int nmg_w4_to_dense(const void *d_B, const void *d_meta, const void *d_s, int64_t M, int64_t K,
                               void *d_out, int64_t ldo, void *stream)
{
    if (int rc = w4_check(M, K)) return rc;
    NMG_REQUIRE(ldo >= K, NMG_ERR_ARG, "leading dimension smaller than row length");
    if (M == 0 || K == 0) return NMG_OK;
    NMG_REQUIRE(d_B && d_meta && d_s && d_out, NMG_ERR_ARG, "null device pointer");
    W4Params P{};
    P.w = d_out;
    P.B = const_cast<void *>(d_B);
    P.meta = (uint32_t *)const_cast<void *>(d_meta);
    P.s = const_cast<void *>(d_s);
    P.M = M;
    P.K = K;
    P.ldw = ldo;
    P.MB = (int)((M + 31) / 32);
    P.KQ = (int)(K / 128);
    const int64_t total = M * P.KQ;
    hipLaunchKernelGGL(w4_unpack_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, P);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

extern "C" int nmg_w4_linear(const void *d_B, const void *d_meta, const void *d_s, int64_t M, int64_t K,
                             const void *d_x, int64_t ldx, void *d_y, int64_t ldy, const void *d_bias,
                             int64_t T, void *stream)
{
    if (int rc = w4_check(M, K)) return rc;
    NMG_REQUIRE(T >= 0 && T <= 16, NMG_ERR_UNSUPPORTED, "the int4 kernel serves at most 16 tokens, got %lld",
                (long long)T);
    NMG_REQUIRE(ldx >= K && ldy >= M, NMG_ERR_ARG, "leading dimension smaller than row length");
    NMG_REQUIRE(ldx % 8 == 0 && ((uintptr_t)d_x % 16) == 0, NMG_ERR_UNSUPPORTED,
                "activations must be 16-byte aligned with ldx a multiple of 8");
    if (M == 0 || T == 0) return NMG_OK;
    NMG_REQUIRE(d_B && d_meta && d_s && d_x && d_y, NMG_ERR_ARG, "null device pointer");
    W4Params P{};
    P.B = const_cast<void *>(d_B);
    P.meta = (uint32_t *)const_cast<void *>(d_meta);
    P.s = const_cast<void *>(d_s);
    P.x = d_x;
    P.y = d_y;
    P.bias = d_bias;
    P.M = M;
    P.K = K;
    P.T = T;
    P.ldx = ldx;
    P.ldy = ldy;
    P.MB = (int)((M + 31) / 32);
    P.KQ = (int)(K / 128);
    hipStream_t s = (hipStream_t)stream;
    // One block of 32 rows per workgroup measured best on the 11008 x 4096 weight (two row blocks
    // per workgroup sharing the activation fragments: 19 us against 8.9 -- the kernel lives on the
    // number of workgroups pulling data at once).  Staged activations and counted waits: 6.6 us at
    // one token, 7.8 us at 16 (direct loads: 8.8 / 13.2); the direct kernel remains for K = 0 and
    // activations beyond 2 GiB.
    if (P.KQ >= 1 && P.T * P.ldx * 2 < ((int64_t)1 << 31)) {
        if (P.KQ >= 16)
            w4_launch_staged_nd<8>(P, s);
        else
            w4_launch_staged_nd<4>(P, s);
    } else if (P.KQ >= 16)
        w4_launch<8, 1, 1>(P, s);
    else
        w4_launch<4, 1, 1>(P, s);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}
