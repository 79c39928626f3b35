// Very few tokens with the reduction along the *group* dim at 2:4: Y[T, S] = X[T, G] * W (+ bias)
// with every workgroup owning 16 outputs over the whole reduction, so that the sums never leave the
// workgroup (nmg_gstream.hip cuts the reduction into slices over workgroups and adds the slices'
// sums with a second kernel, which at these sizes is a quarter of the time).  This is F.linear on
// a weight in the reference's default orientation (n:m blocks along the outputs,
// sten_impls.py:24-31; the reference kernel gathers rows of B per pattern, dace_gnm_mult.py:200-213).
//
//  * No matrix instruction: with at most 4 tokens the product is 2 x 16 x G x T multiply-adds per
//    workgroup and what counts is the vector instructions per byte of the stream.  Lane
//    l = (line group lg = l / 4, block b = l % 4) of a wavefront holds, per set of 256 lines, the 16
//    lines 16 lg .. 16 lg + 15 of block b (4 of the workgroup's 16 outputs) as 8 pairs of lines: per
//    pair two value words and two pattern nibbles.  A table in LDS gives, per pair of pattern
//    numbers, the four selector words with which V_PERM_B32 builds (weight of the lower line,
//    weight of the upper line) at each of the block's four positions; one V_DOT2_F32 with the pair's
//    two activations (one word of the token row) adds both lines to the output's sum: per pair
//    one LDS read, four permutes and 4 T dot products -- and no exchange between lanes until the
//    sums of the 16 line groups are added at the very end.
//  * Operand ("opack", nmg_opack from the rowpack operand, once per weight version): per span of
//    16 outputs and set of 256 lines, what the lanes fetch, in lane order: values
//    [4][64 lanes][16 bytes] (load j holds pairs 2 j, 2 j + 1: two value words each), patterns
//    [64 lanes][8 bytes] (byte p: the nibbles of the two lines of pair p).  Sets ordered
//    [span][set]: a wavefront's sets are one contiguous run.  1.125 bytes per dense weight.
//  * A workgroup is 16 wavefronts that split the sets; one set (4.5 KiB) in flight per wavefront;
//    their sums meet in LDS, fixed order, bias and the 16-bit store in the same kernel.
//  * Every workgroup reads the token rows over the whole reduction (the sliced kernel reads a
//    slice of them): the right choice for a handful of tokens, not for 16.
#include "nmg_common.h"
#include "nmg_tile.h"

#include <algorithm>

namespace nmg {

typedef _Float16 os_f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 os_bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t os_u32x2 __attribute__((ext_vector_type(2)));

// a.lo * b.lo + a.hi * b.hi + c in single precision (V_DOT2C_F32_F16 / _BF16)
template <typename T> __device__ __forceinline__ float os_dot2(uint32_t a, uint32_t b, float c);
template <> __device__ __forceinline__ float os_dot2<__half>(uint32_t a, uint32_t b, float c)
{
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(os_f16x2, a), __builtin_bit_cast(os_f16x2, b), c, false);
}
template <> __device__ __forceinline__ float os_dot2<__hip_bfloat16>(uint32_t a, uint32_t b, float c)
{
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(os_bf16x2, a), __builtin_bit_cast(os_bf16x2, b), c, false);
}

constexpr int OS_WAVES = 16;
constexpr int OS_SET_LINES = 256;                 // 8 tiles of 32 lines
constexpr uint32_t OS_SETB = 4 * 1024 + 512;      // bytes of a set: values, then patterns

struct OStream {
    const unsigned char *op;       // opack
    const unsigned char *x;        // [T][ldx]
    void *y;                       // [T][ldy]
    const void *bias;              // [S] or null
    int64_t G, S, ldx, ldy, T;
    int64_t nsets;                 // ceil(G / 256)
    int sets_per_wave;
    uint32_t order[3];             // [6][2] kept positions per pattern of 2:4, one byte each
};

// TT = token rows the lanes hold (T <= TT)
template <typename T, int TT> __global__ __launch_bounds__(OS_WAVES * 64) void ostream_kernel(OStream P)
{
    // selector words: entry (p1 << 4 | p0, r) builds (weight of the lower line, weight of the upper
    // line) at position r from the two lines' value words (the lower line is the low source of
    // V_PERM_B32, bytes 0 .. 3; the upper one bytes 4 .. 7; 0x0c: a zero byte)
    __shared__ __align__(16) uint32_t tab[256 * 4];
    __shared__ __align__(16) float red[OS_WAVES][TT][17];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lg = lane >> 2, b = lane & 3;
    const int64_t span = blockIdx.x;

    const int64_t w_lo = (int64_t)wave * P.sets_per_wave;
    const uint32_t s_lo = (uint32_t)(w_lo < P.nsets ? w_lo : P.nsets);
    const int64_t w_hi = (int64_t)s_lo + P.sets_per_wave;
    const uint32_t cnt = (uint32_t)(w_hi < P.nsets ? w_hi : P.nsets) - s_lo;
    const int64_t s0 = cnt ? s_lo : 0;      // (a wavefront without sets stands on the first, which exists)
    const unsigned char *owave = P.op + (span * P.nsets + s0) * OS_SETB;
    const unsigned char *xwave = P.x + s0 * OS_SET_LINES * 2;
    const int64_t lines_left = P.G - s0 * OS_SET_LINES;      // lines from the wavefront's first set on
    uint32_t x_tok[TT];
#pragma unroll
    for (int k = 0; k < TT; k++) x_tok[k] = (k < P.T ? (uint32_t)(k * P.ldx * 2) : 0u) + (uint32_t)lg * 32;

    float acc[TT][4];
#pragma unroll
    for (int k = 0; k < TT; k++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[k][r] = 0.f;

    struct Regs {
        u32x4 vals[4];          // load j: pairs 2 j, 2 j + 1, two value words each (lower, upper line)
        os_u32x2 pats;          // byte p: the nibbles of the two lines of pair p
        u32x4 xf[TT][2];        // token k: the activations of the lane's 16 lines, a word per pair
        uint32_t live[2];       // all ones where the lane's lines 0 .. 7 / 8 .. 15 exist
    } R;

    // (`s_nop 4` in front of every load: a base that the compiler has parked in a lane of a vector
    // register comes back through a vector instruction right before its use, and a scalar register
    // written by the vector unit needs five wait states before a memory instruction may read it;
    // the compiler does not look into instruction statements)
    auto issue_set = [&](uint32_t rel) __attribute__((always_inline)) {
        const bool none = rel >= cnt;      // (a stand-in: every lane reads the first bytes of the bases)
        const uint32_t vo = none ? 0u : rel * OS_SETB + (uint32_t)lane * 16;
        const uint32_t po = none ? 0u : rel * OS_SETB + 4096u + (uint32_t)lane * 8;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const unsigned char *vp = owave + j * 1024;
            asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2" : "=v"(R.vals[j]) : "v"(vo), "s"(vp) : "memory");
        }
        asm volatile("s_nop 4\n\tglobal_load_dwordx2 %0, %1, %2" : "=v"(R.pats) : "v"(po), "s"(owave) : "memory");
#pragma unroll
        for (int h = 0; h < 2; h++) {
            // G is a multiple of 8: an octet of lines is whole or absent (absent: the operand holds
            // zeros there, and the activations are masked so that no NaN of a stand-in meets them)
            const bool in = !none && (int64_t)rel * OS_SET_LINES + 16 * lg + 8 * h < lines_left;
            R.live[h] = in ? 0xffffffffu : 0u;
#pragma unroll
            for (int k = 0; k < TT; k++) {
                const uint32_t xo = in ? x_tok[k] + (rel * OS_SET_LINES) * 2 + 16 * h : 0u;
                asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2" : "=v"(R.xf[k][h]) : "v"(xo), "s"(xwave) : "memory");
            }
        }
    };
    // the set has landed: every register of it passes through the wait, so the compiler orders its
    // uses behind it (checked on the compiled code, `python -m sten_amd.isa_check`)
    auto landed = [&]() __attribute__((always_inline)) {
        if constexpr (TT == 1)
            asm volatile("s_waitcnt vmcnt(0)"
                         : "+v"(R.vals[0]), "+v"(R.vals[1]), "+v"(R.vals[2]), "+v"(R.vals[3]), "+v"(R.pats), "+v"(R.xf[0][0]), "+v"(R.xf[0][1])
                         :
                         : "memory");
        else if constexpr (TT == 2)
            asm volatile("s_waitcnt vmcnt(0)"
                         : "+v"(R.vals[0]), "+v"(R.vals[1]), "+v"(R.vals[2]), "+v"(R.vals[3]), "+v"(R.pats), "+v"(R.xf[0][0]), "+v"(R.xf[0][1]),
                           "+v"(R.xf[TT > 1 ? 1 : 0][0]), "+v"(R.xf[TT > 1 ? 1 : 0][1])
                         :
                         : "memory");
        else
            asm volatile("s_waitcnt vmcnt(0)"
                         : "+v"(R.vals[0]), "+v"(R.vals[1]), "+v"(R.vals[2]), "+v"(R.vals[3]), "+v"(R.pats), "+v"(R.xf[0][0]), "+v"(R.xf[0][1]),
                           "+v"(R.xf[TT > 1 ? 1 : 0][0]), "+v"(R.xf[TT > 1 ? 1 : 0][1]), "+v"(R.xf[TT > 2 ? 2 : 0][0]), "+v"(R.xf[TT > 2 ? 2 : 0][1]),
                           "+v"(R.xf[TT > 3 ? 3 : 0][0]), "+v"(R.xf[TT > 3 ? 3 : 0][1])
                         :
                         : "memory");
    };
    static_assert(TT == 1 || TT == 2 || TT == 4, "one, two or four token rows");

    // The first set is requested before anything else happens; the selector table is built while it
    // is on its way, from the order table in the kernel arguments (scalar loads only).
    issue_set(0u);
    {
        const int e = tid;                       // 1024 entries, one per thread
        const int r = e & 3, p0 = (e >> 2) & 15, p1 = e >> 6;
        uint32_t c0 = 0x0c0c, c1 = 0x0c0c;       // where position r lies in the value word of pattern p0, p1
#pragma unroll
        for (int p = 0; p < 6; p++)
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int k = 2 * p + j;
                const int pos = (int)((P.order[k >> 2] >> (8 * (k & 3))) & 0xffu);
                if (pos == r) {
                    if (p == p0) c0 = j ? 0x0302 : 0x0100;
                    if (p == p1) c1 = j ? 0x0302 : 0x0100;
                }
            }
        tab[e] = (p0 < 6 && p1 < 6) ? (c0 | ((c1 | 0x0404u) << 16)) : 0x0c0c0c0cu;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    auto multiply_set = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < 8; p++) {
            const uint32_t v0 = R.vals[p / 2][2 * (p % 2)], v1 = R.vals[p / 2][2 * (p % 2) + 1];
            const uint32_t pb = (R.pats[p / 4] >> (8 * (p % 4))) & 0xffu;
            const u32x4 sel = *(const u32x4 *)((const unsigned char *)tab + pb * 16);
            uint32_t w[4];
            w[0] = __builtin_amdgcn_perm(v1, v0, sel.x);
            w[1] = __builtin_amdgcn_perm(v1, v0, sel.y);
            w[2] = __builtin_amdgcn_perm(v1, v0, sel.z);
            w[3] = __builtin_amdgcn_perm(v1, v0, sel.w);
#pragma unroll
            for (int k = 0; k < TT; k++) {
                const uint32_t xw = R.xf[k][p / 4][p % 4] & R.live[p / 4];
#pragma unroll
                for (int r = 0; r < 4; r++) acc[k][r] = os_dot2<T>(w[r], xw, acc[k][r]);
            }
        }
    };

    // One set in flight per wavefront: request, wait, multiply; the other wavefronts keep the memory
    // busy.  Nothing is in flight across the loop's back edge, no stand-in behind the last set.
    landed();      // (the first set, or the stand-in of a wavefront without sets)
    __builtin_amdgcn_sched_barrier(0);
    if (cnt > 0) multiply_set();
    __builtin_amdgcn_sched_barrier(0);
    for (uint32_t s1 = 1; s1 < cnt; s1++) {
        issue_set(s1);
        __builtin_amdgcn_sched_barrier(0);
        landed();
        __builtin_amdgcn_sched_barrier(0);
        multiply_set();
        __builtin_amdgcn_sched_barrier(0);
    }

    // sums over the 16 line groups of the wavefront (lanes 4 apart and more), then over the wavefronts
#pragma unroll
    for (int k = 0; k < TT; k++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            float v = acc[k][r];
            v += __shfl_xor(v, 4);
            v += __shfl_xor(v, 8);
            v += __shfl_xor(v, 16);
            v += __shfl_xor(v, 32);
            if (lg == 0) red[wave][k][4 * b + r] = v;
        }
    __syncthreads();
    for (int e = tid; e < (int)P.T * 16; e += OS_WAVES * 64) {
        const int tok = e >> 4, o = e & 15;
        const int64_t out = span * 16 + o;
        if (out >= P.S) continue;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < OS_WAVES; w++) sum += red[w][tok][o];
        if (P.bias) sum += to_f32(((const T *)P.bias)[out]);
        ((uint16_t *)P.y)[tok * P.ldy + out] = f32_to_bits16(sum, (T *)nullptr);
    }
}

// ---- the operand: one thread per (span, set, lane)
struct OPack {
    const uint32_t *pk_val;        // [G][nb] value words (two 16-bit values per block)
    const uint8_t *pk_pat;         // [G][nb]
    unsigned char *op;
    int64_t G, nb, nsets, shares;  // shares = spans * nsets * 64
};

__global__ __launch_bounds__(256) void opack_kernel(OPack P)
{
    const int64_t sh = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (sh >= P.shares) return;
    const int lane = (int)(sh & 63), lg = lane >> 2, b = lane & 3;
    const int64_t ss = sh >> 6, span = ss / P.nsets, set = ss - span * P.nsets;
    unsigned char *out = P.op + ss * OS_SETB;
    const int64_t blk = span * 4 + b;
    uint32_t pats[2] = {0u, 0u};
    for (int p = 0; p < 8; p++) {
        uint32_t w[2], q[2];
        for (int h = 0; h < 2; h++) {
            const int64_t line = set * OS_SET_LINES + 16 * lg + 2 * p + h;
            const bool ok = line < P.G && blk < P.nb;
            w[h] = ok ? P.pk_val[line * P.nb + blk] : 0u;
            q[h] = ok ? P.pk_pat[line * P.nb + blk] : 0u;
        }
        uint32_t *dst = (uint32_t *)(out + (p / 2) * 1024 + lane * 16) + 2 * (p % 2);
        dst[0] = w[0];
        dst[1] = w[1];
        pats[p / 4] |= (q[0] | (q[1] << 4)) << (8 * (p % 4));
    }
    uint32_t *pd = (uint32_t *)(out + 4096 + lane * 8);
    pd[0] = pats[0];
    pd[1] = pats[1];
}

}  // namespace nmg

using namespace nmg;

extern "C" int nmg_spmm_ostream_supported(int n, int m) { return n == 2 && m == 4 ? 1 : 0; }

extern "C" int nmg_opack_bytes(int64_t G, int64_t S, int n, int m, int64_t *bytes)
{
    NMG_REQUIRE(bytes, NMG_ERR_ARG, "null output pointer");
    NMG_REQUIRE(nmg_spmm_ostream_supported(n, m), NMG_ERR_UNSUPPORTED, "this product takes 2:4");
    NMG_REQUIRE(G >= 0 && S >= 0, NMG_ERR_ARG, "negative extent");
    *bytes = ((S + 15) / 16) * ((G + OS_SET_LINES - 1) / OS_SET_LINES) * (int64_t)OS_SETB;
    return NMG_OK;
}

extern "C" int nmg_opack(const void *d_pk_val, const void *d_pk_pat, int64_t G, int64_t S, int n, int m, void *d_op,
                         int dtype, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "the operand holds f16/bf16");
    NMG_REQUIRE(nmg_spmm_ostream_supported(n, m), NMG_ERR_UNSUPPORTED, "this product takes 2:4");
    NMG_REQUIRE(G >= 0 && S >= 0, NMG_ERR_ARG, "negative extent");
    if (G == 0 || S == 0) return NMG_OK;
    NMG_REQUIRE(d_pk_val && d_pk_pat && d_op, NMG_ERR_ARG, "null device pointer");
    NMG_REQUIRE(((uintptr_t)d_op % 16) == 0 && ((uintptr_t)d_pk_val % 4) == 0, NMG_ERR_ARG,
                "the operand must be 16-byte aligned, the values 4-byte aligned");
    OPack P;
    P.pk_val = (const uint32_t *)d_pk_val;
    P.pk_pat = (const uint8_t *)d_pk_pat;
    P.op = (unsigned char *)d_op;
    P.G = G;
    P.nb = (S + m - 1) / m;
    P.nsets = (G + OS_SET_LINES - 1) / OS_SET_LINES;
    P.shares = ((S + 15) / 16) * P.nsets * 64;
    const int64_t blocks = (P.shares + 255) / 256;
    NMG_REQUIRE(blocks <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "weight too large for one launch");
    hipLaunchKernelGGL(opack_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, P);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

extern "C" int nmg_spmm_ostream(const void *d_op, int64_t G, int64_t S, const void *d_x, int64_t ldx, void *d_y,
                                int64_t ldy, const void *d_bias, int64_t T, int n, int m, int dtype, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "this product takes f16/bf16");
    NMG_REQUIRE(nmg_spmm_ostream_supported(n, m), NMG_ERR_UNSUPPORTED, "this product takes 2:4");
    NMG_REQUIRE(G >= 0 && S >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(T <= 4, NMG_ERR_UNSUPPORTED, "this product serves at most 4 tokens");
    NMG_REQUIRE(ldx >= G && ldy >= S, NMG_ERR_ARG, "leading dimension smaller than row length");
    if (T == 0 || S == 0) return NMG_OK;
    NMG_REQUIRE(G > 0, NMG_ERR_UNSUPPORTED, "empty reduction: clear the output instead");
    NMG_REQUIRE(G % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)d_x % 16) == 0 && ((uintptr_t)d_op % 16) == 0, NMG_ERR_UNSUPPORTED,
                "this product needs a reduction extent and a row pitch of the activations that are multiples of 8, "
                "and 16-byte aligned activations and operand");
    NMG_REQUIRE(d_op && d_x && d_y, NMG_ERR_ARG, "null device pointer");
    NMG_REQUIRE(T * ldx * 2 < ((int64_t)1 << 31), NMG_ERR_UNSUPPORTED, "activations beyond 2 GiB");
    OStream P;
    P.op = (const unsigned char *)d_op;
    P.x = (const unsigned char *)d_x;
    P.y = d_y;
    P.bias = d_bias;
    P.G = G;
    P.S = S;
    P.ldx = ldx;
    P.ldy = ldy;
    P.T = T;
    P.nsets = (G + OS_SET_LINES - 1) / OS_SET_LINES;
    P.sets_per_wave = (int)((P.nsets + OS_WAVES - 1) / OS_WAVES);
    NMG_REQUIRE(((int64_t)P.sets_per_wave + 1) * OS_SETB < ((int64_t)1 << 31), NMG_ERR_UNSUPPORTED, "reduction too long");
    const int8_t *ord = host_order(n, m);
    NMG_REQUIRE(ord != nullptr, NMG_ERR_ARG, "invalid n:m = %d:%d", n, m);
    for (int e = 0; e < 3; e++) P.order[e] = 0;
    for (int e = 0; e < 12; e++) P.order[e >> 2] |= (uint32_t)(uint8_t)ord[e] << (8 * (e & 3));
    const int64_t spans = (S + 15) / 16;
    NMG_REQUIRE(spans <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "weight too large for one launch");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)spans), block(OS_WAVES * 64);
#define NMG_OS_TT(TT_)                                                              \
    if (dtype == NMG_F16)                                                            \
        hipLaunchKernelGGL((ostream_kernel<__half, TT_>), grid, block, 0, s, P);     \
    else                                                                             \
        hipLaunchKernelGGL((ostream_kernel<__hip_bfloat16, TT_>), grid, block, 0, s, P);
    if (T == 1) { NMG_OS_TT(1) } else if (T == 2) { NMG_OS_TT(2) } else { NMG_OS_TT(4) }
#undef NMG_OS_TT
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}
