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
    const unsigned char *pk_val;   // [G][nb][n] 16-bit values
    const unsigned char *pk_pat;   // [G][nb] pattern numbers, one byte each
    uint32_t order[14];            // [c][n] kept positions per pattern, one byte each (c * n <= 56 for m <= 8, n <= 2)
    const unsigned char *x;        // [T][ldx] 16-bit activations
    float *part;                   // [slices][T][part_ld]
    int64_t G, nb, ldx, T, part_ld;
    int64_t slice_lines;           // lines per slice, a multiple of 8 * GS_WAVES
    int c, spans;
};

constexpr uint32_t GS_NONE = 0xffffff00u;   // "no tile": a line offset beyond any range
constexpr int GS_QS = 24;          // floats between the rows of two outputs q of a token in the LDS sums

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
    constexpr int BL = GS_OPL / M;          // blocks per lane
    constexpr int VB = BL * N * 2;          // bytes of values per lane and line: 16, 8, 4 or 2
    constexpr int NPAR = N == 1 ? 2 : 1;    // n = 1: two blocks share a value word, the selector depends on the parity
    constexpr int MAXC = M == 4 ? 6 : 28;
    constexpr int RS = GS_OPL * GS_QS;      // floats per token row of the LDS sums
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

    const int64_t b_lane = (int64_t)span * (16 * BL) + i * BL;      // first block of the lane
    const bool lane_ok = b_lane < P.nb;
    const int64_t val_pitch = P.nb * N * 2, pat_pitch = P.nb;

    const int64_t wave_lines = P.slice_lines / GS_WAVES;            // a multiple of 8
    const int64_t l0 = (int64_t)slice * P.slice_lines + (int64_t)wave * wave_lines;
    const int64_t l1 = l0 + wave_lines < P.G ? l0 + wave_lines : P.G;

    // Addresses: a base per wavefront and line u (scalar registers) plus one 32-bit offset per
    // lane and tile.  Nothing in the loads is conditional: a lane beyond the last block reads block 0
    // and its sums are never stored, a group of 8 lines beyond the wavefront's range reads the
    // range's first group and meets activations masked to zero, a tile beyond it reads the first
    // bytes of the bases and is not multiplied.
    const uint32_t nlines = l1 > l0 ? (uint32_t)(l1 - l0) : 0u;
    // (a wavefront whose range is empty stands on the first lines of the slice, which exist)
    const int64_t lb = nlines ? l0 : (int64_t)slice * P.slice_lines;
    const unsigned char *vwave = P.pk_val + lb * val_pitch;
    const unsigned char *pwave = P.pk_pat + lb * pat_pitch;
    const unsigned char *xwave = P.x + lb * 2;
    const uint32_t ntiles = (nlines + 31) / 32;
    const uint32_t bl_lane = lane_ok ? (uint32_t)b_lane : 0u;
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
    struct Regs {
        VT vals[8];
        uint32_t pats[8];
        u32x4 xf[TB];
        uint32_t xmask[TB];     // all ones where the lane's token and lines exist, else zero
    } rs[1];
    static_assert(TB == 1, "the wait lists one activation fragment");

    // (`s_nop 4` in front of every load: the bases are scalar registers, and where the compiler
    // parks one in a lane of a vector register it reads it back with a vector instruction right
    // before the use -- a scalar register written by the vector unit needs five wait states before
    // a memory instruction may read it, and the compiler does not look into instruction statements)
    auto issue_tile = [&](Regs &R, uint32_t rel) __attribute__((always_inline)) {
        // ranges are multiples of 8 lines: a group of 8 is whole or absent
        const bool in_range = rel < nlines && rel + 8 * kq < nlines;
        const uint32_t lrel = in_range ? rel + 8 * kq : 0u;      // lines from the range's first
        // (24-bit factors, checked by the host: one multiply-add each)
        // (beyond the whole range every lane reads the first bytes of the base: one cache line)
        const bool none = rel >= nlines;
        const uint32_t v_off = none ? 0u : __umul24(lrel, (uint32_t)val_pitch) + bl_lane * (N * 2);
        const uint32_t p_off = none ? 0u : __umul24(lrel, (uint32_t)pat_pitch) + bl_lane;
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const unsigned char *vp = vwave + u * val_pitch;
            const unsigned char *pp = pwave + u * pat_pitch;
            if constexpr (VB == 16)
                asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2" : "=v"(R.vals[u]) : "v"(v_off), "s"(vp) : "memory");
            else if constexpr (VB == 8)
                asm volatile("s_nop 4\n\tglobal_load_dwordx2 %0, %1, %2" : "=v"(R.vals[u]) : "v"(v_off), "s"(vp) : "memory");
            else if constexpr (VB == 4)
                asm volatile("s_nop 4\n\tglobal_load_dword %0, %1, %2" : "=v"(R.vals[u]) : "v"(v_off), "s"(vp) : "memory");
            else
                asm volatile("s_nop 4\n\tglobal_load_ushort %0, %1, %2" : "=v"(R.vals[u]) : "v"(v_off), "s"(vp) : "memory");
            if constexpr (BL == 4)
                asm volatile("s_nop 4\n\tglobal_load_dword %0, %1, %2" : "=v"(R.pats[u]) : "v"(p_off), "s"(pp) : "memory");
            else if constexpr (BL == 2)
                asm volatile("s_nop 4\n\tglobal_load_ushort %0, %1, %2" : "=v"(R.pats[u]) : "v"(p_off), "s"(pp) : "memory");
            else
                asm volatile("s_nop 4\n\tglobal_load_ubyte %0, %1, %2" : "=v"(R.pats[u]) : "v"(p_off), "s"(pp) : "memory");
        }
#pragma unroll
        for (int tb = 0; tb < TB; tb++) {
            const uint32_t xo = none ? 0u : x_tok[tb] + lrel * 2;
            asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2" : "=v"(R.xf[tb]) : "v"(xo), "s"(xwave) : "memory");
            R.xmask[tb] = in_range ? x_live[tb] : 0u;
        }
    };
    // the tile has landed (every register of the set passes through the wait, so the compiler
    // orders its uses behind it)
    auto landed = [&](Regs &R) __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(0)"
                     : "+v"(R.vals[0]), "+v"(R.vals[1]), "+v"(R.vals[2]), "+v"(R.vals[3]), "+v"(R.vals[4]), "+v"(R.vals[5]),
                       "+v"(R.vals[6]), "+v"(R.vals[7]), "+v"(R.pats[0]), "+v"(R.pats[1]), "+v"(R.pats[2]), "+v"(R.pats[3]),
                       "+v"(R.pats[4]), "+v"(R.pats[5]), "+v"(R.pats[6]), "+v"(R.pats[7]), "+v"(R.xf[0])
                     :
                     : "memory");
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
    issue_tile(rs[0], ntiles ? 0u : GS_NONE);
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
                const uint32_t p0 = (R.pats[2 * up] >> (8 * bl)) & 0xffu, p1 = (R.pats[2 * up + 1] >> (8 * bl)) & 0xffu;
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
        issue_tile(rs[0], 32 * t1);
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
// a tile is 17 loads of up to 10.6 KiB, in runs of 256 bytes per line.
constexpr int GS_OPL = 16, GS_WAVES = 8, GS_SPAN = 16 * GS_OPL;

static int gstream_plan(int64_t G, int64_t S, int m, int *spans, int *slices, int64_t *slice_lines)
{
    const int64_t nb = (S + m - 1) / m;
    const int64_t sp = (nb * m + GS_SPAN - 1) / GS_SPAN;
    // one workgroup per CU when the weight allows it; a wavefront gets at least 32 lines
    int64_t sl = std::max<int64_t>(1, 256 / sp);
    const int64_t quantum = 8 * GS_WAVES;
    int64_t lines = (G + sl - 1) / sl;
    lines = std::max<int64_t>((lines + quantum - 1) / quantum * quantum, 32 * GS_WAVES);
    sl = (G + lines - 1) / lines;
    *spans = (int)sp;
    *slices = (int)std::max<int64_t>(sl, 1);
    *slice_lines = lines;
    return NMG_OK;
}

}  // namespace nmg

using namespace nmg;

extern "C" int nmg_spmm_gstream_supported(int n, int m)
{
    return (m == 4 || m == 8) && (n == 1 || n == 2) ? 1 : 0;
}

extern "C" int nmg_spmm_gstream_plan(int64_t G, int64_t S, int64_t T, int n, int m, int *slices, int64_t *ws_bytes)
{
    NMG_REQUIRE(slices && ws_bytes, NMG_ERR_ARG, "null output pointer");
    NMG_REQUIRE(nmg_spmm_gstream_supported(n, m), NMG_ERR_UNSUPPORTED, "the streaming product takes m = 4, 8 and n = 1, 2");
    NMG_REQUIRE(G >= 0 && S >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    int spans = 1;
    int64_t lines = 0;
    gstream_plan(std::max<int64_t>(G, 1), std::max<int64_t>(S, 1), m, &spans, slices, &lines);
    *ws_bytes = (int64_t)*slices * T * spans * GS_SPAN * 4;
    return NMG_OK;
}

extern "C" int nmg_spmm_gstream(const void *d_pk_val, const void *d_pk_pat, int64_t G, int64_t S, const void *d_x,
                                int64_t ldx, void *d_y, int64_t ldy, const void *d_bias, int64_t T, int n, int m,
                                int dtype, void *d_ws, int64_t ws_bytes, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "the streaming product takes f16/bf16");
    NMG_REQUIRE(nmg_spmm_gstream_supported(n, m), NMG_ERR_UNSUPPORTED, "the streaming product takes m = 4, 8 and n = 1, 2");
    NMG_REQUIRE(G >= 0 && S >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(T <= 16, NMG_ERR_UNSUPPORTED, "the streaming product serves at most 16 tokens");
    NMG_REQUIRE(ldx >= G && ldy >= S, NMG_ERR_ARG, "leading dimension smaller than row length");
    if (T == 0 || S == 0) return NMG_OK;
    NMG_REQUIRE(G > 0, NMG_ERR_UNSUPPORTED, "empty reduction: clear the output instead");
    const int64_t nb = (S + m - 1) / m;
    const int BL = GS_OPL / m;
    NMG_REQUIRE(G % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)d_x % 16) == 0, NMG_ERR_UNSUPPORTED,
                "the streaming product needs a reduction extent and a row pitch of the activations that are multiples "
                "of 8, and 16-byte aligned activations");
    NMG_REQUIRE(nb % BL == 0 && ((uintptr_t)d_pk_val % 16) == 0 && ((uintptr_t)d_pk_pat % 4) == 0, NMG_ERR_UNSUPPORTED,
                "the streaming product needs whole groups of %d blocks per line and aligned operands", BL);
    NMG_REQUIRE(d_pk_val && d_pk_pat && d_x && d_y && d_ws, NMG_ERR_ARG, "null device pointer");
    NMG_REQUIRE(T * ldx * 2 < ((int64_t)1 << 31), NMG_ERR_UNSUPPORTED, "activations beyond 2 GiB");

    GStream P;
    int slices = 1;
    gstream_plan(G, S, m, &P.spans, &slices, &P.slice_lines);
    P.part_ld = (int64_t)P.spans * GS_SPAN;
    NMG_REQUIRE(ws_bytes >= (int64_t)slices * T * P.part_ld * 4, NMG_ERR_ARG,
                "workspace too small: %lld bytes given, %lld needed (nmg_spmm_gstream_plan)", (long long)ws_bytes,
                (long long)((int64_t)slices * T * P.part_ld * 4));
    NMG_REQUIRE((int64_t)P.spans * slices <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "weight too large for one launch");
    NMG_REQUIRE((P.slice_lines / GS_WAVES + 8) * nb * n * 2 < ((int64_t)1 << 31) && nb * n * 2 < (1 << 24) &&
                    P.slice_lines / GS_WAVES < (1 << 23),
                NMG_ERR_UNSUPPORTED, "lines of more than 16 MiB, or the lines of one wavefront span more than 2 GiB");
    P.pk_val = (const unsigned char *)d_pk_val;
    P.pk_pat = (const unsigned char *)d_pk_pat;
    const int8_t *ord = host_order(n, m);
    NMG_REQUIRE(ord != nullptr && binom(m, n) * n <= (int64_t)sizeof(P.order), NMG_ERR_ARG, "invalid n:m = %d:%d", n, m);
    for (int e = 0; e < 14; e++) P.order[e] = 0;
    for (int64_t e = 0; e < binom(m, n) * n; e++) P.order[e >> 2] |= (uint32_t)(uint8_t)ord[e] << (8 * (e & 3));
    P.x = (const unsigned char *)d_x;
    P.part = (float *)d_ws;
    P.G = G;
    P.nb = nb;
    P.ldx = ldx;
    P.T = T;
    P.c = (int)binom(m, n);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)(P.spans * slices)), block(GS_WAVES * 64);
    const size_t lds = (size_t)gs_table_bytes(n == 1 ? 2 : 1, P.c, m) + (size_t)(GS_WAVES / 2) * T * (GS_OPL * GS_QS) * 4;
    NMG_REQUIRE(lds <= 160 * 1024, NMG_ERR_UNSUPPORTED, "LDS");
#define NMG_GS_TB(TT, NN, MM)                                                                              \
    {                                                                                                        \
        auto k = gstream_kernel<TT, NN, MM, GS_OPL, GS_WAVES>;                                                            \
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
