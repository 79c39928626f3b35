// Few tokens with the reduction along the *group* dim: Y[T, S] = X[T, G] * W, W given as the
// rowpack operand (per line of the group dim and block of m outputs: the n kept values and the
// pattern number).  This is what F.linear does with a weight in the reference's default
// orientation (n:m blocks along the outputs, sten_impls.py:24-31; the reference kernel gathers
// rows of B per pattern, dace_gnm_mult.py:200-213).  The zeros are not along the reduction, so
// the sparse matrix cores cannot use them; what the compressed form saves here is memory traffic,
// and with at most 16 tokens the product is bound by the stream of the weight from HBM.  The
// kernel therefore streams the compressed lines once (n/m of the dense bytes plus one byte per
// block), expands them in registers and multiplies on the dense matrix cores:
//
//  * V_MFMA_F32_16X16X32: A = 16 outputs x 32 lines, lane (i, kq) = (l % 16, l / 16) holds lines
//    8 kq .. 8 kq + 7 of output row i.  A lane loads, for each of its 8 lines, the values and
//    patterns of BL = 16 / m consecutive blocks (16 outputs): a quarter wavefront reads 16 * BL
//    blocks of one line as one contiguous run (256 bytes of values and 64 of patterns at 2:4).
//    Output q of the lane (q = 0 .. 15) across its 8 lines is one A fragment, so a 32-line tile is
//    16 MFMAs, and row i of MFMA q is output 16 i + q of the workgroup's span of 256.
//  * Expansion: for a block with pattern p, position r holds value j(p, r) or nothing.  A table in
//    LDS gives, per (pattern of line u, pattern of line u + 1, position r), the selector word with
//    which one V_PERM_B32 builds the pair (weight of line u, weight of line u + 1) at position r
//    from the two lines' value words (0x0c: a zero byte): one vector instruction per pair of dense
//    weights, one 16-byte table read per four positions of a pair of lines.
//  * A workgroup is 8 wavefronts on one span of 256 outputs and one slice of the reduction; a
//    wavefront walks its lines in tiles of 32, one tile in flight (the other wavefronts keep the
//    memory busy).  The wavefronts add their sums in LDS in a fixed order (results do not depend
//    on timing) and write single-precision partial sums part[slice][token][output];
//    splitk_sum_kernel adds the slices in order, adds the bias and rounds once.
#include "nmg_common.h"
#include "nmg_tile.h"

#include <algorithm>
#include <type_traits>

namespace nmg {

typedef _Float16 gs_f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 gs_bf16x8 __attribute__((ext_vector_type(8)));

template <typename T> struct GsMfma;
template <> struct GsMfma<__half> {
    using F = gs_f16x8;
    __device__ static f32x4 run(F a, F b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};
template <> struct GsMfma<__hip_bfloat16> {
    using F = gs_bf16x8;
    __device__ static f32x4 run(F a, F b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};

struct GStream {
    const unsigned char *gp;       // the operand in tile order ("gpack", see gpack_kernel)
    uint32_t order[14];            // [c][n] kept positions per pattern, one byte each (c * n <= 56 for m <= 8, n <= 2)
    const unsigned char *x;        // [T][ldx] 16-bit activations
    float *part;                   // [slices][T][part_ld]
    int64_t G, ldx, T, part_ld;
    int64_t ltiles;                // tiles of 32 lines: ceil(G / 32)
    int wave_tiles;                // tiles per wavefront (a slice is GS_WAVES * wave_tiles tiles)
    int c, spans;
};

constexpr int GS_QS = 24;          // floats between the rows of two outputs q of a token in the LDS sums
constexpr int GS_RPAD = 4;         // floats of padding behind a token row there

// bytes of the selector tables in LDS (pair table, code table), rounded to 16
__host__ __device__ constexpr int gs_table_bytes(int npar, int c, int m)
{
    return (npar * c * c * m * 4 + npar * c * m * 2 + 15) & ~15;
}

// OPL outputs per lane (a workgroup spans 16 * OPL outputs), NW wavefronts per workgroup.
template <typename T, int N, int M, int OPL, int NW>
__global__ __launch_bounds__(NW * 64) void gstream_kernel(GStream P)
{
    constexpr int TB = 1, GS_WAVES = NW, GS_OPL = OPL, GS_SPAN = 16 * OPL;
    static_assert((NW & (NW - 1)) == 0 && NW >= 2, "a power of two of wavefronts");
    static_assert(M == 4 || M == 8, "blocks of 4 or 8 outputs");
    static_assert(N == 1 || N == 2, "one or two kept values per block");
    static_assert(GS_OPL == 16, "a lane holds 16 outputs: 16, 8 or 4 bytes of values per line");
    constexpr int BL = GS_OPL / M;          // blocks per lane
    constexpr int VB = BL * N * 2;          // bytes of values per lane and line: 16, 8, 4 or 2
    constexpr int NPAR = N == 1 ? 2 : 1;    // n = 1: two blocks share a value word, the selector depends on the parity
    constexpr int MAXC = M == 4 ? 6 : 28;
    // floats per token row of the LDS sums; + 4: the 16 token rows that the lanes of a quarter
    // wavefront write at once start 16 bytes apart in the banks (a multiple of 64 floats would put
    // them all into the same ones: 16 tokens then cost 3 us more than one)
    constexpr int RS = GS_OPL * GS_QS + GS_RPAD;
    using F = typename GsMfma<T>::F;

    // LDS: [pair table][code table][sums of the wavefronts, two wavefronts per slab]
    extern __shared__ __align__(16) unsigned char gs_smem[];
    uint32_t *pair = (uint32_t *)gs_smem;                                  // [NPAR][c][c][M]
    uint16_t *code = (uint16_t *)(gs_smem + NPAR * P.c * P.c * M * 4);     // [NPAR][c][M]
    float *red = (float *)(gs_smem + gs_table_bytes(NPAR, P.c, M));        // [GS_WAVES / 2][T][RS]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);    // wavefront-uniform: bases stay in scalar registers
    const int i = lane & 15, kq = lane >> 4;
    // Workgroup ids go to the 8 XCDs in turn; consecutive spans of a slice read neighbouring parts
    // of the same 128-byte lines (a quarter wavefront takes 256 bytes of values and 64 of patterns
    // per line at 2:4), so every XCD gets a contiguous run of (slice, span) pairs, span fastest.
    int id = blockIdx.x;
    if ((gridDim.x & 7) == 0) id = (id & 7) * (gridDim.x >> 3) + (id >> 3);
    const int span = id % P.spans, slice = id / P.spans;

    // The wavefront's tiles of 32 lines: consecutive in the operand (10 KiB each at 2:4), so its
    // loads walk one contiguous run.  Lines beyond G and blocks beyond the last hold zeros there;
    // only the activations need masking (G is a multiple of 8: a group of 8 lines is whole or absent).
    constexpr int PBITS = (M == 4 || N == 1) ? 4 : 8;      // bits of a pattern number (c <= 16: 4)
    constexpr int PL = 8 * BL * PBITS / 8;                 // bytes of patterns per lane and tile: 16 or 8
    constexpr uint32_t TBYTES = 512 * VB + 64 * PL;        // bytes of a tile: values [u][lane], patterns [lane]
    const int64_t tile0 = ((int64_t)slice * GS_WAVES + wave) * P.wave_tiles;
    const int64_t left = P.ltiles - tile0;
    const uint32_t ntiles = left <= 0 ? 0u : (left < P.wave_tiles ? (uint32_t)left : (uint32_t)P.wave_tiles);
    const int64_t tb0 = ntiles ? tile0 : 0;      // (a wavefront without tiles stands on the first, which exists)
    const int64_t lines_left = P.G - tb0 * 32;
    const uint32_t nlines = ntiles == 0 ? 0u : (lines_left < (int64_t)ntiles * 32 ? (uint32_t)lines_left : ntiles * 32);
    const unsigned char *twave = P.gp + ((int64_t)span * P.ltiles + tb0) * TBYTES;
    const unsigned char *xwave = P.x + tb0 * 32 * 2;
    uint32_t x_tok[TB], x_live[TB];
#pragma unroll
    for (int tb = 0; tb < TB; tb++) {
        const bool live = tb * 16 + i < P.T;
        x_tok[tb] = live ? (uint32_t)((tb * 16 + i) * P.ldx * 2) : 0u;
        x_live[tb] = live ? 0xffffffffu : 0u;
    }

    f32x4 acc[GS_OPL][TB];
#pragma unroll
    for (int q = 0; q < GS_OPL; q++)
#pragma unroll
        for (int tb = 0; tb < TB; tb++) acc[q][tb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // One register set: a tile of 32 lines in flight per wavefront.  The loads are instruction
    // statements with a wait of their own -- left to the compiler, the 17 loads of a tile are
    // waited for one by one as they are used; every register of the set passes through the wait,
    // so the compiler orders its uses behind it (that nothing touches them earlier is checked on
    // the compiled code, `python -m sten_amd.isa_check`).
    typedef uint32_t gs_u32x2 __attribute__((ext_vector_type(2)));
    using VT = std::conditional_t<VB == 16, u32x4, std::conditional_t<VB == 8, gs_u32x2, uint32_t>>;
    using PT = std::conditional_t<PL == 16, u32x4, gs_u32x2>;
    struct Regs {
        VT vals[8];             // line u of the lane's octet
        PT pats;                // pattern (u, block bl) at bit (u BL + bl) PBITS
        u32x4 xf[TB];
        uint32_t xmask[TB];     // all ones where the lane's token and lines exist, else zero
    } rs[1];
    static_assert(TB == 1, "the wait lists one activation fragment");

    // (`s_nop 4` in front of every load: the bases are scalar registers, and where the compiler
    // parks one in a lane of a vector register it reads it back with a vector instruction right
    // before the use -- a scalar register written by the vector unit needs five wait states before
    // a memory instruction may read it, and the compiler does not look into instruction statements)
    auto issue_tile = [&](Regs &R, uint32_t t) __attribute__((always_inline)) {
        // (beyond the range every lane reads the first bytes of the base: one cache line)
        const bool none = t >= ntiles;
        const bool in_range = !none && t * 32 + 8 * kq < nlines;
        const uint32_t v_off = none ? 0u : t * TBYTES + (uint32_t)lane * VB;
        const uint32_t p_off = none ? 0u : t * TBYTES + 512u * VB + (uint32_t)lane * PL;
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const unsigned char *vp = twave + u * (64 * VB);
            if constexpr (VB == 16)
                asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2" : "=v"(R.vals[u]) : "v"(v_off), "s"(vp) : "memory");
            else if constexpr (VB == 8)
                asm volatile("s_nop 4\n\tglobal_load_dwordx2 %0, %1, %2" : "=v"(R.vals[u]) : "v"(v_off), "s"(vp) : "memory");
            else
                asm volatile("s_nop 4\n\tglobal_load_dword %0, %1, %2" : "=v"(R.vals[u]) : "v"(v_off), "s"(vp) : "memory");
        }
        if constexpr (PL == 16)
            asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2" : "=v"(R.pats) : "v"(p_off), "s"(twave) : "memory");
        else
            asm volatile("s_nop 4\n\tglobal_load_dwordx2 %0, %1, %2" : "=v"(R.pats) : "v"(p_off), "s"(twave) : "memory");
#pragma unroll
        for (int tb = 0; tb < TB; tb++) {
            const uint32_t xo = in_range ? x_tok[tb] + (t * 32 + 8 * kq) * 2 : 0u;
            asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2" : "=v"(R.xf[tb]) : "v"(xo), "s"(xwave) : "memory");
            R.xmask[tb] = in_range ? x_live[tb] : 0u;
        }
    };
    // the tile has landed (every register of the set passes through the wait, so the compiler
    // orders its uses behind it)
    auto landed = [&](Regs &R) __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(0)"
                     : "+v"(R.vals[0]), "+v"(R.vals[1]), "+v"(R.vals[2]), "+v"(R.vals[3]), "+v"(R.vals[4]), "+v"(R.vals[5]),
                       "+v"(R.vals[6]), "+v"(R.vals[7]), "+v"(R.pats), "+v"(R.xf[0])
                     :
                     : "memory");
    };
    // pattern of line u, block bl
    auto pat_of = [](const PT &v, int u, int bl) __attribute__((always_inline)) -> uint32_t {
        const int bit = (u * BL + bl) * PBITS;
        return (v[bit / 32] >> (bit % 32)) & ((1u << PBITS) - 1);
    };
    auto word = [](const VT &v, int w) __attribute__((always_inline)) -> uint32_t {
        if constexpr (VB >= 8) return v[w];
        else return v;
    };

    // The first tile is requested before anything else happens; the selector table is built
    // while they are on their way, from the order table in the kernel arguments (scalar loads: no
    // vector-memory operation of the compiler's own sits between the counted ones).  Entry
    // (par, p, r) = byte selectors that fetch the value kept at position r into the low half of a
    // word (from a value word that is the *low* source of V_PERM_B32).
    issue_tile(rs[0], 0u);      // (a stand-in where the wavefront has no tile)
    // code(par, p, r): where the value kept at position r of pattern p lies in its value word
    for (int e = tid; e < NPAR * P.c * M; e += GS_WAVES * 64) {
        const int my_p = (e / M) % P.c, my_r = e % M, my_par = e / (P.c * M);
        uint16_t sel = 0x0c0c;
#pragma unroll
        for (int p = 0; p < MAXC; p++)
#pragma unroll
            for (int j = 0; j < N; j++) {
                const int k = p * N + j;
                const int pos = (int)((P.order[k >> 2] >> (8 * (k & 3))) & 0xffu);
                if (p < P.c && p == my_p && pos == my_r) sel = (N == 1 ? my_par : j) ? 0x0302 : 0x0100;
            }
        code[e] = sel;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    // pair(par, p0, p1, r): the selector word that builds (weight of line u, weight of line u + 1)
    // at position r from the value words of the two lines, u the *low* source of V_PERM_B32 and
    // u + 1 the high one (bytes 4 .. 7: 0x0c | 0x04 stays 0x0c, zero)
    for (int e = tid; e < NPAR * P.c * P.c * M; e += GS_WAVES * 64) {
        const int r = e % M, p1 = (e / M) % P.c, p0 = (e / (M * P.c)) % P.c, par = e / (M * P.c * P.c);
        pair[e] = (uint32_t)code[(par * P.c + p0) * M + r] | (((uint32_t)code[(par * P.c + p1) * M + r] | 0x0404u) << 16);
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    const uint32_t cM4 = (uint32_t)P.c * M * 4;      // bytes of the pair table per p0
    auto multiply_tile = [&](const Regs &R) __attribute__((always_inline)) {
        u32x4 xm[TB];
#pragma unroll
        for (int tb = 0; tb < TB; tb++) xm[tb] = R.xf[tb] & R.xmask[tb];
#pragma unroll
        for (int bl = 0; bl < BL; bl++) {
            uint32_t sel[4][M];
#pragma unroll
            for (int up = 0; up < 4; up++) {
                const uint32_t p0 = pat_of(R.pats, 2 * up, bl), p1 = pat_of(R.pats, 2 * up + 1, bl);
                const unsigned char *e = (const unsigned char *)pair + (N == 1 ? (bl & 1) * P.c * cM4 : 0u) +
                                         __umul24(p0, cM4) + p1 * (M * 4);
#pragma unroll
                for (int w = 0; w < M / 4; w++) {
                    const u32x4 v = *(const u32x4 *)(e + 16 * w);
                    sel[up][4 * w + 0] = v.x; sel[up][4 * w + 1] = v.y; sel[up][4 * w + 2] = v.z; sel[up][4 * w + 3] = v.w;
                }
            }
            constexpr int dwn = N == 2 ? 1 : 2;     // blocks per value word
            const int dw = bl / dwn;
#pragma unroll
            for (int r = 0; r < M; r++) {
                uint32_t a[4];
#pragma unroll
                for (int up = 0; up < 4; up++)
                    a[up] = __builtin_amdgcn_perm(word(R.vals[2 * up + 1], dw), word(R.vals[2 * up], dw), sel[up][r]);
                const u32x4 aw = {a[0], a[1], a[2], a[3]};
                const int q = bl * M + r;
#pragma unroll
                for (int tb = 0; tb < TB; tb++)
                    acc[q][tb] = GsMfma<T>::run(__builtin_bit_cast(F, aw), __builtin_bit_cast(F, xm[tb]), acc[q][tb]);
            }
        }
    };

    // One tile in flight per wavefront: request, wait for it, multiply; the other wavefronts keep
    // the memory busy.  (A wavefront's whole range requested at once was no faster at one token and
    // slower at 16: the chip's requests are then served in no particular order while a wavefront's
    // loads complete in issue order, so every tile lands near the end of the stream.)  Nothing is
    // in flight across the loop's back edge, and no stand-in is requested behind the last tile.
    landed(rs[0]);      // (the first tile, or the stand-in of an empty range)
    __builtin_amdgcn_sched_barrier(0);
    if (ntiles > 0) multiply_tile(rs[0]);
    __builtin_amdgcn_sched_barrier(0);
    for (uint32_t t1 = 1; t1 < ntiles; t1++) {
        issue_tile(rs[0], t1);
        __builtin_amdgcn_sched_barrier(0);
        landed(rs[0]);
        __builtin_amdgcn_sched_barrier(0);
        multiply_tile(rs[0]);
        __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();

    // Sums of the wavefronts: the upper half writes a slab each, the lower half adds theirs to the
    // same slabs, then every output adds its slabs in order (fixed order: results do not depend on
    // timing).  A lane holds token l % 16 and outputs OPL (4 (l / 16) + r) + q of MFMA q.
    const int tcol = lane & 15, rq = lane >> 4;
    float *slab = red + (size_t)(wave & (GS_WAVES / 2 - 1)) * P.T * RS;
#pragma unroll
    for (int half = 1; half >= 0; half--) {
        if ((wave >= GS_WAVES / 2 ? 1 : 0) == half) {
#pragma unroll
            for (int tb = 0; tb < TB; tb++) {
                if (tb * 16 + tcol < P.T) {
#pragma unroll
                    for (int q = 0; q < GS_OPL; q++) {
                        f32x4 *dst = (f32x4 *)&slab[(tb * 16 + tcol) * RS + q * GS_QS + 4 * rq];
                        if (half == 1) *dst = acc[q][tb];
                        else *dst += acc[q][tb];
                    }
                }
            }
        }
        __syncthreads();
    }
    // partial sums of the slice: coalesced along the outputs
    for (int e = tid; e < (int)P.T * GS_SPAN; e += GS_WAVES * 64) {
        const int tok = e / GS_SPAN, o = e % GS_SPAN;
        const float *src = red + tok * RS + (o % GS_OPL) * GS_QS + o / GS_OPL;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < GS_WAVES / 2; w++) sum += src[(size_t)w * P.T * RS];
        P.part[((int64_t)slice * P.T + tok) * P.part_ld + (int64_t)span * GS_SPAN + o] = sum;
    }
}

// The shape of the launch: outputs per lane and wavefronts per workgroup.  With 16 outputs per lane
// a tile of 32 lines x 256 outputs is 10 loads of up to 9 KiB in all.
constexpr int GS_OPL = 16, GS_WAVES = 8, GS_SPAN = 16 * GS_OPL;

// bytes of a tile of the operand and bits of a pattern number (as the kernel has them)
static void gpack_shape(int n, int m, int *vb, int *pbits, int *pl, int64_t *tbytes)
{
    const int bl = GS_OPL / m;
    *vb = bl * n * 2;
    *pbits = (m == 4 || n == 1) ? 4 : 8;
    *pl = 8 * bl * *pbits / 8;
    *tbytes = 512 * (int64_t)*vb + 64 * (int64_t)*pl;
}

// ---- the operand: rowpack in tile order.  Tile (span sp, line tile lt) = 32 lines x 256 outputs:
//   values   [u 0..7][lane 0..63][VB bytes]   lane (i, kq) = (l % 16, l / 16): line 32 lt + 8 kq + u,
//                                             blocks 16 BL sp + BL i .. + BL - 1 (BL = 16 / m)
//   patterns [lane][PL bytes]                 pattern of (u, block bl) at bit (u BL + bl) PBITS
// tiles ordered [sp][lt], so the tiles a wavefront walks are one contiguous run.  Lines beyond G and
// blocks beyond the last are zeros with pattern 0.
struct GPack {
    const unsigned char *pk_val;   // [G][nb][n] 16-bit values
    const unsigned char *pk_pat;   // [G][nb] pattern numbers, one byte each
    unsigned char *gp;
    int64_t G, nb, ltiles, spans;
    int n, m;
};

__global__ __launch_bounds__(256) void gpack_kernel(GPack P)
{
    const int bl_n = GS_OPL / P.m, vb = bl_n * P.n * 2;
    const int pbits = (P.m == 4 || P.n == 1) ? 4 : 8, pl = 8 * bl_n * pbits / 8;
    const int64_t tbytes = 512 * (int64_t)vb + 64 * (int64_t)pl;
    const int64_t tile = blockIdx.x;
    const int64_t sp = tile / P.ltiles, lt = tile - sp * P.ltiles;
    unsigned char *out = P.gp + tile * tbytes;
    // values: 512 (u, lane) shares of vb bytes, as 16-bit elements
    for (int e = threadIdx.x; e < 512 * (vb / 2); e += 256) {
        const int h = e % (vb / 2), share = e / (vb / 2);
        const int lane = share & 63, u = share >> 6, i = lane & 15, kq = lane >> 4;
        const int64_t line = lt * 32 + 8 * kq + u;
        const int64_t blk0 = sp * (16 * bl_n) + (int64_t)i * bl_n;      // the lane's first block
        const int64_t blk = blk0 + h / P.n;
        uint16_t v = 0;
        if (line < P.G && blk < P.nb) v = ((const uint16_t *)P.pk_val)[(line * P.nb + blk) * P.n + h % P.n];
        ((uint16_t *)out)[share * (vb / 2) + h] = v;
    }
    // patterns: one 32-bit word per thread
    for (int e = threadIdx.x; e < 64 * (pl / 4); e += 256) {
        const int w = e % (pl / 4), lane = e / (pl / 4), i = lane & 15, kq = lane >> 4;
        uint32_t word = 0;
        for (int f = 0; f < 32 / pbits; f++) {
            const int idx = (w * 32) / pbits + f;          // = u * bl_n + bl
            const int u = idx / bl_n, bl = idx - u * bl_n;
            const int64_t line = lt * 32 + 8 * kq + u;
            const int64_t blk = sp * (16 * bl_n) + (int64_t)i * bl_n + bl;
            uint32_t p = 0;
            if (line < P.G && blk < P.nb) p = P.pk_pat[line * P.nb + blk];
            word |= p << (f * pbits);
        }
        ((uint32_t *)(out + 512 * (int64_t)vb))[lane * (pl / 4) + w] = word;
    }
}

// slices of the reduction: one workgroup per CU when the weight allows it; a wavefront walks
// whole tiles of 32 lines
static void gstream_plan(int64_t G, int64_t S, int *spans, int *slices, int *wave_tiles)
{
    const int64_t sp = (S + GS_SPAN - 1) / GS_SPAN;
    const int64_t ltiles = (G + 31) / 32;
    const int64_t want = std::max<int64_t>(1, 256 / sp);                     // slices wanted
    const int64_t per = (ltiles + want * GS_WAVES - 1) / (want * GS_WAVES);  // tiles per wavefront
    *wave_tiles = (int)std::max<int64_t>(per, 1);
    *spans = (int)sp;
    *slices = (int)((ltiles + (int64_t)*wave_tiles * GS_WAVES - 1) / ((int64_t)*wave_tiles * GS_WAVES));
}

}  // namespace nmg

using namespace nmg;

extern "C" int nmg_spmm_gstream_supported(int n, int m)
{
    return (m == 4 || m == 8) && (n == 1 || n == 2) ? 1 : 0;
}

extern "C" int nmg_gpack_bytes(int64_t G, int64_t S, int n, int m, int64_t *bytes)
{
    NMG_REQUIRE(bytes, NMG_ERR_ARG, "null output pointer");
    NMG_REQUIRE(nmg_spmm_gstream_supported(n, m), NMG_ERR_UNSUPPORTED, "the streaming product takes m = 4, 8 and n = 1, 2");
    NMG_REQUIRE(G >= 0 && S >= 0, NMG_ERR_ARG, "negative extent");
    int vb, pbits, pl;
    int64_t tbytes;
    gpack_shape(n, m, &vb, &pbits, &pl, &tbytes);
    *bytes = ((S + GS_SPAN - 1) / GS_SPAN) * ((G + 31) / 32) * tbytes;
    return NMG_OK;
}

extern "C" int nmg_gpack(const void *d_pk_val, const void *d_pk_pat, int64_t G, int64_t S, int n, int m, void *d_gp,
                         int dtype, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "the operand holds f16/bf16");
    NMG_REQUIRE(nmg_spmm_gstream_supported(n, m), NMG_ERR_UNSUPPORTED, "the streaming product takes m = 4, 8 and n = 1, 2");
    NMG_REQUIRE(G >= 0 && S >= 0, NMG_ERR_ARG, "negative extent");
    if (G == 0 || S == 0) return NMG_OK;
    NMG_REQUIRE(d_pk_val && d_pk_pat && d_gp, NMG_ERR_ARG, "null device pointer");
    NMG_REQUIRE(((uintptr_t)d_gp % 16) == 0 && ((uintptr_t)d_pk_val % 2) == 0, NMG_ERR_ARG, "the operand must be 16-byte aligned");
    NMG_REQUIRE(binom(m, n) <= ((m == 4 || n == 1) ? 16 : 256), NMG_ERR_UNSUPPORTED, "pattern numbers beyond their field");
    GPack P;
    P.pk_val = (const unsigned char *)d_pk_val;
    P.pk_pat = (const unsigned char *)d_pk_pat;
    P.gp = (unsigned char *)d_gp;
    P.G = G;
    P.nb = (S + m - 1) / m;
    P.ltiles = (G + 31) / 32;
    P.spans = (S + GS_SPAN - 1) / GS_SPAN;
    P.n = n;
    P.m = m;
    const int64_t tiles = P.ltiles * P.spans;
    NMG_REQUIRE(tiles <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "weight too large for one launch");
    hipLaunchKernelGGL(gpack_kernel, dim3((unsigned)tiles), dim3(256), 0, (hipStream_t)stream, P);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

extern "C" int nmg_spmm_gstream_plan(int64_t G, int64_t S, int64_t T, int n, int m, int *slices, int64_t *ws_bytes)
{
    NMG_REQUIRE(slices && ws_bytes, NMG_ERR_ARG, "null output pointer");
    NMG_REQUIRE(nmg_spmm_gstream_supported(n, m), NMG_ERR_UNSUPPORTED, "the streaming product takes m = 4, 8 and n = 1, 2");
    NMG_REQUIRE(G >= 0 && S >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    int spans = 1, wave_tiles = 1;
    gstream_plan(std::max<int64_t>(G, 1), std::max<int64_t>(S, 1), &spans, slices, &wave_tiles);
    *ws_bytes = (int64_t)*slices * T * spans * GS_SPAN * 4;
    return NMG_OK;
}

extern "C" int nmg_spmm_gstream(const void *d_gp, int64_t G, int64_t S, const void *d_x, int64_t ldx, void *d_y,
                                int64_t ldy, const void *d_bias, int64_t T, int n, int m, int dtype, void *d_ws,
                                int64_t ws_bytes, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "the streaming product takes f16/bf16");
    NMG_REQUIRE(nmg_spmm_gstream_supported(n, m), NMG_ERR_UNSUPPORTED, "the streaming product takes m = 4, 8 and n = 1, 2");
    NMG_REQUIRE(G >= 0 && S >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(T <= 16, NMG_ERR_UNSUPPORTED, "the streaming product serves at most 16 tokens");
    NMG_REQUIRE(ldx >= G && ldy >= S, NMG_ERR_ARG, "leading dimension smaller than row length");
    if (T == 0 || S == 0) return NMG_OK;
    NMG_REQUIRE(G > 0, NMG_ERR_UNSUPPORTED, "empty reduction: clear the output instead");
    NMG_REQUIRE(G % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)d_x % 16) == 0, NMG_ERR_UNSUPPORTED,
                "the streaming product needs a reduction extent and a row pitch of the activations that are multiples "
                "of 8, and 16-byte aligned activations");
    NMG_REQUIRE(d_gp && d_x && d_y && d_ws, NMG_ERR_ARG, "null device pointer");
    NMG_REQUIRE(((uintptr_t)d_gp % 16) == 0, NMG_ERR_UNSUPPORTED, "the operand must be 16-byte aligned");
    NMG_REQUIRE(T * ldx * 2 < ((int64_t)1 << 31), NMG_ERR_UNSUPPORTED, "activations beyond 2 GiB");

    GStream P;
    int slices = 1;
    gstream_plan(G, S, &P.spans, &slices, &P.wave_tiles);
    P.part_ld = (int64_t)P.spans * GS_SPAN;
    NMG_REQUIRE(ws_bytes >= (int64_t)slices * T * P.part_ld * 4, NMG_ERR_ARG,
                "workspace too small: %lld bytes given, %lld needed (nmg_spmm_gstream_plan)", (long long)ws_bytes,
                (long long)((int64_t)slices * T * P.part_ld * 4));
    NMG_REQUIRE((int64_t)P.spans * slices <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "weight too large for one launch");
    int vb, pbits, pl;
    int64_t tbytes;
    gpack_shape(n, m, &vb, &pbits, &pl, &tbytes);
    NMG_REQUIRE(((int64_t)P.wave_tiles + 1) * tbytes < ((int64_t)1 << 31), NMG_ERR_UNSUPPORTED,
                "the tiles of one wavefront span more than 2 GiB");
    P.gp = (const unsigned char *)d_gp;
    const int8_t *ord = host_order(n, m);
    NMG_REQUIRE(ord != nullptr && binom(m, n) * n <= (int64_t)sizeof(P.order), NMG_ERR_ARG, "invalid n:m = %d:%d", n, m);
    for (int e = 0; e < 14; e++) P.order[e] = 0;
    for (int64_t e = 0; e < binom(m, n) * n; e++) P.order[e >> 2] |= (uint32_t)(uint8_t)ord[e] << (8 * (e & 3));
    P.x = (const unsigned char *)d_x;
    P.part = (float *)d_ws;
    P.G = G;
    P.ltiles = (G + 31) / 32;
    P.ldx = ldx;
    P.T = T;
    P.c = (int)binom(m, n);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)(P.spans * slices)), block(GS_WAVES * 64);
    const size_t lds = (size_t)gs_table_bytes(n == 1 ? 2 : 1, P.c, m) + (size_t)(GS_WAVES / 2) * T * (GS_OPL * GS_QS + GS_RPAD) * 4;
    NMG_REQUIRE(lds <= 160 * 1024, NMG_ERR_UNSUPPORTED, "LDS");
#define NMG_GS_TB(TT, NN, MM)                                                                              \
    {                                                                                                        \
        auto k = gstream_kernel<TT, NN, MM, GS_OPL, GS_WAVES>;                                              \
        if (lds > 64 * 1024)                                                                                 \
            NMG_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        hipLaunchKernelGGL(k, grid, block, lds, s, P);                                                       \
    }
#define NMG_GS_NM(TT)                                                  \
    if (n == 2 && m == 4) { NMG_GS_TB(TT, 2, 4) }                      \
    else if (n == 1 && m == 4) { NMG_GS_TB(TT, 1, 4) }                 \
    else if (n == 2 && m == 8) { NMG_GS_TB(TT, 2, 8) }                 \
    else { NMG_GS_TB(TT, 1, 8) }
    if (dtype == NMG_F16) { NMG_GS_NM(__half) } else { NMG_GS_NM(__hip_bfloat16) }
#undef NMG_GS_NM
#undef NMG_GS_TB
    NMG_HIP_TRY(hipGetLastError());
    SplitSum Q;
    Q.part = P.part;
    Q.y = d_y;
    Q.bias = d_bias;
    Q.M = S;
    Q.T = T;
    Q.ldy = ldy;
    Q.part_ld = P.part_ld;
    Q.slices = slices;
    if (dtype == NMG_F16) return launch_splitk_sum<__half>(Q, s);
    return launch_splitk_sum<__hip_bfloat16>(Q, s);
}
