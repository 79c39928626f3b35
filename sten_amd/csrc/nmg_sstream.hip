// Few tokens on a compressed weight with blocks of 8 along the reduction (1:8, 2:8, 4:8):
// Y[T, G] = X[T, S] * W^T (+ bias), W given as the rowpack operand (per output line and block of 8
// reduction positions: the n kept values and the pattern number).  The operand of the sparse
// matrix cores stores two values and two positions for every 4 reduction positions whatever the
// pattern keeps, 1.125 bytes per dense weight; at 2:8 the rowpack operand holds 0.625 (1:8: 0.375),
// and with at most 16 tokens the product is bound by the stream of the weight from HBM -- so these
// patterns stream the rowpack operand, expand it in registers and multiply on the dense matrix
// cores (the reference's kernel walks val / idx the same way, one gathered FMA per kept value:
// dace_gnm_mult.py:185-253).
//
//  * V_MFMA_F32_16X16X32: lane (i, kq) = (l % 16, l / 16) of the A operand holds 8 consecutive
//    reduction positions of output row i -- exactly one block.  Which block of a step a lane takes
//    is free as long as the activation fragment follows: in a set of 32 blocks lane (i, kq) owns
//    the blocks 16 a + 4 e + kq (a = 0, 1; e = 0 .. 3; MFMA step 4 a + e), so the four lanes of a
//    token read 64 contiguous bytes of its activations per step.
//  * Operand ("lanepack8", written once per weight version by nmg_lanepack8 from the rowpack
//    operand): for a group of 32 lines and a set of 32 blocks, per row block rb and half a the 64
//    lanes' shares in lane order -- lp_val [group][set][rb][a][lane][4 blocks][n] values,
//    lp_pat [group][set][rb][a][lane][4] pattern bytes (4:8) or [group][set][lane] three words of
//    sixteen 5-bit pattern numbers, (rb, a, e) at bit 5 (f % 6) of word f / 6 with f = 8 rb + 4 a + e
//    (1:8, 2:8: at most 28 patterns) -- so every load of the kernel is one
//    contiguous run of 256 bytes to 2 KiB.  Lines beyond the last hold zeros.
//  * Expansion: a table in LDS gives per pattern the four byte selectors (V_PERM_B32) that spread
//    the block's value words over the four words of the fragment: one LDS read and four vector
//    instructions per block.
//  * A workgroup is 32 output lines (two row blocks that share the activation fragments) -- 16 where
//    the weight has too few lines to give every CU a workgroup -- and 16 wavefronts that split
//    the reduction; their sums meet in LDS, fixed order, one kernel.
//  * Loads are instruction statements with a wait of their own (left to the compiler, the loads
//    of a set would be waited for one by one as they are used).  A wavefront has one set in flight;
//    the 16 wavefronts of a workgroup keep the memory busy.  A wavefront without sets requests a
//    stand-in (every lane reads the first bytes of the operand) so that all run the same code up
//    to the first wait.
#include "nmg_common.h"
#include "nmg_tile.h"

#include <algorithm>
#include <type_traits>

namespace nmg {

typedef _Float16 ss_f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 ss_bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t ss_u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t ss_u32x3 __attribute__((ext_vector_type(3)));

template <typename T> struct SsMfma;
template <> struct SsMfma<__half> {
    using F = ss_f16x8;
    __device__ static f32x4 run(F a, F b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};
template <> struct SsMfma<__hip_bfloat16> {
    using F = ss_bf16x8;
    __device__ static f32x4 run(F a, F b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};

struct SStream {
    const unsigned char *lp_val;   // lanepack8 values
    const unsigned char *lp_pat;   // lanepack8 pattern bytes
    const unsigned char *x;        // [T][ldx]
    void *y;                       // [T][ldy]
    const void *bias;              // [G] or null
    int64_t G, nb, ldx, ldy, T;
    int sets_per_wave;             // sets of 32 blocks per wavefront
    int c;
    uint32_t order[70];            // [c][n] kept positions per pattern, one byte each (c * n <= 280)
};

constexpr int SS_WAVES = 16;
constexpr int SS_LINES = 32;            // output lines per workgroup
constexpr uint32_t SS_NONE = 0xffffff00u;

// RBN = 2: a workgroup takes the 32 lines of a group; RBN = 1: two workgroups share a group, 16 lines
// each (weights of few lines: twice the workgroups pull the operand; both read the token rows).
template <typename T, int N, int RBN>
__global__ __launch_bounds__(SS_WAVES * 64) void sstream_kernel(SStream P)
{
    static_assert(RBN == 1 || RBN == 2, "one or two row blocks of 16 lines");
    static_assert(N == 1 || N == 2 || N == 4, "1:8, 2:8, 4:8");
    constexpr int PB = 4 * N * 2;            // bytes of values a lane reads per half set: 8, 16, 32
    constexpr int VL = PB / 16 > 0 ? PB / 16 : 1;   // loads they take
    constexpr int NPAR = N == 1 ? 2 : 1;
    constexpr int MAXC = N == 1 ? 8 : (N == 2 ? 28 : 70);
    using F = typename SsMfma<T>::F;
    using VT = std::conditional_t<PB == 8, ss_u32x2, u32x4>;

    __shared__ __align__(16) uint32_t tab[NPAR * MAXC * 4];
    __shared__ uint32_t ord[(MAXC * N + 3) / 4];
    __shared__ __align__(16) float red[SS_WAVES][16][16 * RBN + 1];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i = lane & 15, kq = lane >> 4;
    const int64_t group = RBN == 2 ? (int64_t)blockIdx.x : (int64_t)(blockIdx.x >> 1);
    const int rb0 = RBN == 2 ? 0 : (int)(blockIdx.x & 1);      // first row block of the workgroup
    const int64_t l0 = group * SS_LINES + rb0 * 16;

    // the wavefront's sets of 32 blocks
    const uint32_t total_sets = (uint32_t)(P.nb / 32);
    const uint32_t s_lo = min((uint32_t)wave * P.sets_per_wave, total_sets);
    const uint32_t nsets = min(s_lo + P.sets_per_wave, total_sets) - s_lo;
    // a set of the operand: [rb][a][lane] shares of PB / 4 bytes
    constexpr bool PK5 = N <= 2;             // pattern numbers in 5 bits, sixteen per lane and set in three words
    constexpr uint32_t VSET = 4 * 64 * PB, PSET = PK5 ? 64 * 12 : 4 * 64 * 4;
    const unsigned char *vwave = P.lp_val + (group * total_sets + (nsets ? s_lo : 0)) * VSET + rb0 * (2 * 64 * PB);
    const unsigned char *pwave = P.lp_pat + (group * total_sets + (nsets ? s_lo : 0)) * PSET + (PK5 ? 0 : rb0 * (2 * 64 * 4));
    const unsigned char *xwave = P.x + (int64_t)(nsets ? s_lo : 0) * 32 * 16;
    const bool tok_live = i < P.T;
    const uint32_t x_lane = (tok_live ? (uint32_t)(i * P.ldx * 2) : 0u) + (uint32_t)kq * 16;

    f32x4 acc[RBN];
#pragma unroll
    for (int rb = 0; rb < RBN; rb++) acc[rb] = f32x4{0.f, 0.f, 0.f, 0.f};

    struct Regs {
        VT vals[RBN][2][VL];    // [row block][half set][load]
        uint32_t pats[RBN][2];  // (4:8) a word of four pattern bytes per (row block, half set)
        ss_u32x3 pk;            // (1:8, 2:8) the lane's sixteen 5-bit pattern numbers of the set
        u32x4 xf[2][4];         // [half set][block of the lane]
        uint32_t xmask;
    } rs[1];

    // loads of set `rel` of the wavefront's range (SS_NONE: a stand-in beyond the range -- every
    // lane reads the first bytes of the wavefront's base, one cache line)
    // (`s_nop 4` in front of every load: a base that the compiler has parked in a lane of a vector
    // register comes back through a vector instruction right before its use, and a scalar register
    // written by the vector unit needs five wait states before a memory instruction may read it;
    // the compiler does not look into instruction statements)
    auto issue_set = [&](Regs &R, uint32_t rel) __attribute__((always_inline)) {
        const bool in_range = rel < nsets;      // (SS_NONE lies beyond any range)
#pragma unroll
        for (int rb = 0; rb < RBN; rb++)
#pragma unroll
            for (int a = 0; a < 2; a++) {
                const uint32_t vo = in_range ? rel * VSET + (uint32_t)((rb * 2 + a) * 64 + lane) * PB : 0u;
                const uint32_t po = in_range ? rel * PSET + (uint32_t)((rb * 2 + a) * 64 + lane) * 4 : 0u;
                if constexpr (PB == 8) {
                    asm volatile("s_nop 4\n\tglobal_load_dwordx2 %0, %1, %2" : "=v"(R.vals[rb][a][0]) : "v"(vo), "s"(vwave) : "memory");
                } else {
#pragma unroll
                    for (int v = 0; v < VL; v++)
                        asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2" : "=v"(R.vals[rb][a][v]) : "v"(vo + 16 * v), "s"(vwave) : "memory");
                }
                if constexpr (!PK5)
                    asm volatile("s_nop 4\n\tglobal_load_dword %0, %1, %2" : "=v"(R.pats[rb][a]) : "v"(po), "s"(pwave) : "memory");
            }
        if constexpr (PK5) {
            const uint32_t po = in_range ? rel * PSET + (uint32_t)lane * 12 : 0u;
            asm volatile("s_nop 4\n\tglobal_load_dwordx3 %0, %1, %2" : "=v"(R.pk) : "v"(po), "s"(pwave) : "memory");
        }
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t xo = in_range ? x_lane + (rel * 32 + 16 * a + 4 * e) * 16 : 0u;
                asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2" : "=v"(R.xf[a][e]) : "v"(xo), "s"(xwave) : "memory");
            }
        R.xmask = (in_range && tok_live) ? 0xffffffffu : 0u;
    };
    // Every register of a set passes through the counted wait, so the compiler orders its uses
    // behind it; that nothing touches them earlier is checked on the compiled code.
#define NMG_SS_X(R)                                                                                          \
    "+v"(R.xf[0][0]), "+v"(R.xf[0][1]), "+v"(R.xf[0][2]), "+v"(R.xf[0][3]), "+v"(R.xf[1][0]), "+v"(R.xf[1][1]), \
        "+v"(R.xf[1][2]), "+v"(R.xf[1][3])
#define NMG_SS_P(R, rb) "+v"(R.pats[rb][0]), "+v"(R.pats[rb][1])
#define NMG_SS_K(R) "+v"(R.pk)
#define NMG_SS_V0(R, rb) "+v"(R.vals[rb][0][0]), "+v"(R.vals[rb][1][0])
#define NMG_SS_V1(R, rb) "+v"(R.vals[rb][0][VL - 1]), "+v"(R.vals[rb][1][VL - 1])
    // the set has landed (every register of the set is named exactly once: a register named twice
    // would be copied)
    auto landed = [&](Regs &R) __attribute__((always_inline)) {
        if constexpr (PK5 && RBN == 2)
            asm volatile("s_waitcnt vmcnt(0)" : NMG_SS_V0(R, 0), NMG_SS_V0(R, 1), NMG_SS_K(R), NMG_SS_X(R) : : "memory");
        else if constexpr (PK5)
            asm volatile("s_waitcnt vmcnt(0)" : NMG_SS_V0(R, 0), NMG_SS_K(R), NMG_SS_X(R) : : "memory");
        else if constexpr (RBN == 2)
            asm volatile("s_waitcnt vmcnt(0)" : NMG_SS_V0(R, 0), NMG_SS_V0(R, 1), NMG_SS_V1(R, 0), NMG_SS_V1(R, 1), NMG_SS_P(R, 0), NMG_SS_P(R, 1), NMG_SS_X(R) : : "memory");
        else
            asm volatile("s_waitcnt vmcnt(0)" : NMG_SS_V0(R, 0), NMG_SS_V1(R, 0), NMG_SS_P(R, 0), NMG_SS_X(R) : : "memory");
    };
    static_assert(PK5 == (VL == 1), "the lists above: one load of values per share with 5-bit patterns, two at 4:8");

    // The first set is requested before anything else happens (a wavefront without sets requests a
    // stand-in, so that the code up to the first wait is the same for all).
    issue_set(rs[0], nsets ? 0u : SS_NONE);

    // selector table: entry (par, p) = four selector words; word w builds positions 2 w, 2 w + 1 of
    // the block from its value words (bytes 0 .. 7 of the pair {high, low}; 0x0c: zero).  The order
    // table comes with the kernel arguments (scalar loads: no vector-memory operation of the
    // compiler's own sits between the counted ones).
    // (the order table goes to LDS first, one word per thread picked with compile-time indices: a
    // lane-dependent index into the kernel arguments would put the table into scratch memory)
    if (tid < (MAXC * N + 3) / 4) {
        uint32_t word = 0;
#pragma unroll
        for (int q = 0; q < (MAXC * N + 3) / 4; q++)
            if (tid == q) word = P.order[q];
        ord[tid] = word;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    for (int e = tid; e < NPAR * P.c * 4; e += SS_WAVES * 64) {
        const int w = e & 3, p = (e >> 2) % P.c, par = (e >> 2) / P.c;
        uint32_t sel = 0x0c0c0c0cu;
#pragma unroll
        for (int j = 0; j < N; j++) {
            const uint32_t pos = ((const unsigned char *)ord)[p * N + j];
            // value j of the block sits at half-word hw of the value words the perm sees
            const uint32_t hw = N == 1 ? (uint32_t)par : (uint32_t)j;
            const uint32_t two = (2 * hw) | ((2 * hw + 1) << 8);
            if ((pos >> 1) == (uint32_t)w) sel = (sel & ~(0xffffu << (16 * (pos & 1)))) | (two << (16 * (pos & 1)));
        }
        tab[e] = sel;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    auto word_of = [](const VT (&v)[VL], int w) __attribute__((always_inline)) -> uint32_t {
        if constexpr (PB == 8) return v[0][w];
        else return v[w / 4][w % 4];
    };
    auto multiply_set = [&](const Regs &R) __attribute__((always_inline)) {
        // the workgroup's pattern numbers from bit 0 on, six per word (a workgroup of 16 lines takes
        // the upper eight of the lane's sixteen: fields 8 .. 15 lie from bit 10 of word 1 on)
        uint32_t q[3] = {0u, 0u, 0u};
        if constexpr (PK5) {
            if (RBN == 2 || rb0 == 0) {
                q[0] = R.pk[0];
                q[1] = R.pk[1];
                q[2] = R.pk[2];
            } else {
                q[0] = (R.pk[1] >> 10) | ((R.pk[2] & 0x3ffu) << 20);
                q[1] = (R.pk[2] >> 10) & 0x3ffu;
            }
        }
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const u32x4 xm = R.xf[a][e] & R.xmask;
#pragma unroll
                for (int rb = 0; rb < RBN; rb++) {
                    uint32_t p;
                    if constexpr (PK5) {
                        const int f = 8 * rb + 4 * a + e;
                        p = (q[f / 6] >> (5 * (f % 6))) & 31u;
                    } else {
                        p = (R.pats[rb][a] >> (8 * e)) & 0xffu;
                    }
                    const u32x4 sel = *(const u32x4 *)&tab[((N == 1 ? (e & 1) * P.c : 0) + p) * 4];
                    // the block's value words: n = 2: word e; n = 4: words 2 e, 2 e + 1; n = 1: word e / 2
                    uint32_t lo, hi;
                    if constexpr (N == 4) {
                        lo = word_of(R.vals[rb][a], 2 * e);
                        hi = word_of(R.vals[rb][a], 2 * e + 1);
                    } else if constexpr (N == 2) {
                        lo = hi = word_of(R.vals[rb][a], e);
                    } else {
                        lo = hi = word_of(R.vals[rb][a], e / 2);
                    }
                    const u32x4 aw = {__builtin_amdgcn_perm(hi, lo, sel.x), __builtin_amdgcn_perm(hi, lo, sel.y),
                                      __builtin_amdgcn_perm(hi, lo, sel.z), __builtin_amdgcn_perm(hi, lo, sel.w)};
                    acc[rb] = SsMfma<T>::run(__builtin_bit_cast(F, aw), __builtin_bit_cast(F, xm), acc[rb]);
                }
            }
    };

    // One set in flight per wavefront: request, wait for it, multiply.  Few bytes in flight on
    // purpose.  With a wavefront's whole range requested at once (four sets) the memory system
    // serves the chip's requests in no particular order while a wavefront's loads complete in issue
    // order, so every set lands near the end of the stream and every multiplication is exposed
    // (measured on 8192 x 8192 at 2:8, one token: each of the four sets cost 0.6 us on top of a
    // 9.8 us stream, 12.2 us; two sets in flight 11.2; one 10.6, with 16 wavefronts 10.4).  What
    // keeps the memory busy is the other wavefronts: four per SIMD.  Nothing is in flight across
    // the loop's back edge and no stand-in is requested behind the last set.
    landed(rs[0]);      // (the first set, requested above -- or the stand-in of a wavefront without sets)
    __builtin_amdgcn_sched_barrier(0);
    if (nsets > 0) multiply_set(rs[0]);
    __builtin_amdgcn_sched_barrier(0);
    for (uint32_t s1 = 1; s1 < nsets; s1++) {
        issue_set(rs[0], s1);
        __builtin_amdgcn_sched_barrier(0);
        landed(rs[0]);
        __builtin_amdgcn_sched_barrier(0);
        multiply_set(rs[0]);
        __builtin_amdgcn_sched_barrier(0);
    }
#undef NMG_SS_X
#undef NMG_SS_P
#undef NMG_SS_K
#undef NMG_SS_V0
#undef NMG_SS_V1

    // sums of the wavefronts: lane (t = l % 16, rq = l / 16) holds token t, lines 16 rb + 4 rq + r
    const int rq = lane >> 4;
    constexpr int WL = 16 * RBN;        // lines of the workgroup
    if (tok_live) {
#pragma unroll
        for (int rb = 0; rb < RBN; rb++)
#pragma unroll
            for (int r = 0; r < 4; r++) red[wave][i][rb * 16 + 4 * rq + r] = acc[rb][r];
    }
    __syncthreads();
    for (int e = tid; e < (int)P.T * WL; e += SS_WAVES * 64) {
        const int tok = e / WL, ln = e % WL;
        const int64_t line = l0 + ln;
        if (line >= P.G) continue;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < SS_WAVES; w++) sum += red[w][tok][ln];
        if (P.bias) sum += to_f32(((const T *)P.bias)[line]);
        ((uint16_t *)P.y)[tok * P.ldy + line] = f32_to_bits16(sum, (T *)nullptr);
    }
}

// ---- the operand: one thread per (group, set, rb, a, lane) gathers the lane's four blocks
struct LanePack {
    const uint16_t *pk_val;    // [G][nb][n]
    const uint8_t *pk_pat;     // [G][nb]
    uint16_t *lp_val;
    uint8_t *lp_pat;
    int64_t G, nb, sets, shares;   // shares = groups * sets * 4 * 64
    int n;
};

__global__ __launch_bounds__(256) void lanepack8_kernel(LanePack P)
{
    const int64_t sh = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (sh >= P.shares) return;
    const int lane = (int)(sh & 63), ra = (int)((sh >> 6) & 3);
    const int64_t gs = sh >> 8, group = gs / P.sets, set = gs - group * P.sets;
    const int rb = ra >> 1, a = ra & 1, i = lane & 15, kq = lane >> 4;
    const int64_t line = group * SS_LINES + rb * 16 + i;
    const bool live = line < P.G;
    uint32_t pats = 0;
    for (int e = 0; e < 4; e++) {
        const int64_t blk = set * 32 + 16 * a + 4 * e + kq;
        const int64_t src = (live ? line : 0) * P.nb + blk;
        for (int j = 0; j < P.n; j++) P.lp_val[(sh * 4 + e) * P.n + j] = live ? P.pk_val[src * P.n + j] : (uint16_t)0;
        pats |= (live ? (uint32_t)P.pk_pat[src] : 0u) << (8 * e);
    }
    if (P.n == 4) ((uint32_t *)P.lp_pat)[sh] = pats;
}

// 1:8, 2:8: the sixteen pattern numbers of a lane and set in 5 bits each, six per word --
// one thread per (group, set, lane)
__global__ __launch_bounds__(256) void lanepack8_pat5_kernel(LanePack P)
{
    const int64_t rec = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (rec >= P.shares / 4) return;
    const int lane = (int)(rec & 63), i = lane & 15, kq = lane >> 4;
    const int64_t gs = rec >> 6, group = gs / P.sets, set = gs - group * P.sets;
    uint32_t w[3] = {0u, 0u, 0u};
    for (int f = 0; f < 16; f++) {
        const int rb = f >> 3, a = (f >> 2) & 1, e = f & 3;
        const int64_t line = group * SS_LINES + rb * 16 + i;
        const int64_t blk = set * 32 + 16 * a + 4 * e + kq;
        const uint32_t p = line < P.G ? (uint32_t)P.pk_pat[line * P.nb + blk] : 0u;
        w[f / 6] |= p << (5 * (f % 6));
    }
    uint32_t *dst = (uint32_t *)P.lp_pat + rec * 3;
    dst[0] = w[0];
    dst[1] = w[1];
    dst[2] = w[2];
}

}  // namespace nmg

using namespace nmg;

extern "C" int nmg_spmm_sstream_supported(int n, int m) { return m == 8 && (n == 1 || n == 2 || n == 4) ? 1 : 0; }

extern "C" int nmg_lanepack8_sizes(int64_t G, int64_t S, int n, int64_t *val_elems, int64_t *pat_bytes)
{
    NMG_REQUIRE(val_elems && pat_bytes, NMG_ERR_ARG, "null output pointer");
    NMG_REQUIRE(G >= 0 && S >= 0 && (n == 1 || n == 2 || n == 4), NMG_ERR_ARG, "invalid extents or n");
    NMG_REQUIRE(S % 256 == 0, NMG_ERR_UNSUPPORTED, "the operand holds whole sets of 32 blocks: S must be a multiple of 256");
    const int64_t shares = ((G + SS_LINES - 1) / SS_LINES) * (S / 256) * 4 * 64;
    *val_elems = shares * 4 * n;
    *pat_bytes = n == 4 ? shares * 4 : shares * 3;      // a word per share, or three words per lane and set
    return NMG_OK;
}

extern "C" int nmg_lanepack8(const void *d_pk_val, const void *d_pk_pat, int64_t G, int64_t S, int n, void *d_lp_val,
                             void *d_lp_pat, int dtype, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "the operand holds f16/bf16");
    NMG_REQUIRE(G >= 0 && S >= 0 && (n == 1 || n == 2 || n == 4), NMG_ERR_ARG, "invalid extents or n");
    NMG_REQUIRE(S % 256 == 0, NMG_ERR_UNSUPPORTED, "the operand holds whole sets of 32 blocks: S must be a multiple of 256");
    if (G == 0 || S == 0) return NMG_OK;
    NMG_REQUIRE(d_pk_val && d_pk_pat && d_lp_val && d_lp_pat, NMG_ERR_ARG, "null device pointer");
    NMG_REQUIRE(((uintptr_t)d_lp_pat % 4) == 0, NMG_ERR_ARG, "the pattern bytes must be 4-byte aligned");
    LanePack P;
    P.pk_val = (const uint16_t *)d_pk_val;
    P.pk_pat = (const uint8_t *)d_pk_pat;
    P.lp_val = (uint16_t *)d_lp_val;
    P.lp_pat = (uint8_t *)d_lp_pat;
    P.G = G;
    P.nb = S / 8;
    P.sets = S / 256;
    P.shares = ((G + SS_LINES - 1) / SS_LINES) * P.sets * 4 * 64;
    P.n = n;
    const int64_t blocks = (P.shares + 255) / 256;
    NMG_REQUIRE(blocks <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "weight too large for one launch");
    hipLaunchKernelGGL(lanepack8_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, P);
    if (n != 4)
        hipLaunchKernelGGL(lanepack8_pat5_kernel, dim3((unsigned)((P.shares / 4 + 255) / 256)), dim3(256), 0,
                           (hipStream_t)stream, P);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

extern "C" int nmg_spmm_sstream(const void *d_lp_val, const void *d_lp_pat, int64_t G, int64_t S, const void *d_x,
                                int64_t ldx, void *d_y, int64_t ldy, const void *d_bias, int64_t T, int n, int m,
                                int dtype, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "the streaming product takes f16/bf16");
    NMG_REQUIRE(nmg_spmm_sstream_supported(n, m), NMG_ERR_UNSUPPORTED, "the streaming product takes 1:8, 2:8 and 4:8");
    NMG_REQUIRE(G >= 0 && S >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(T <= 16, NMG_ERR_UNSUPPORTED, "the streaming product serves at most 16 tokens");
    NMG_REQUIRE(ldx >= S && ldy >= G, NMG_ERR_ARG, "leading dimension smaller than row length");
    if (T == 0 || G == 0) return NMG_OK;
    NMG_REQUIRE(S > 0 && S % 256 == 0, NMG_ERR_UNSUPPORTED,
                "the streaming product needs a reduction extent that is a multiple of 256 (whole sets of 32 blocks)");
    NMG_REQUIRE(ldx % 8 == 0 && ((uintptr_t)d_x % 16) == 0 && ((uintptr_t)d_lp_val % 16) == 0 && ((uintptr_t)d_lp_pat % 4) == 0,
                NMG_ERR_UNSUPPORTED, "the streaming product needs 16-byte aligned operands and ldx a multiple of 8");
    NMG_REQUIRE(d_lp_val && d_lp_pat && d_x && d_y, NMG_ERR_ARG, "null device pointer");
    const int64_t nb = S / 8;
    NMG_REQUIRE(T * ldx * 2 < ((int64_t)1 << 31) && (S / 256) * 4 * 64 * 8 * n < ((int64_t)1 << 31), NMG_ERR_UNSUPPORTED,
                "activations beyond 2 GiB, or 32 lines of the weight beyond 2 GiB");
    SStream P;
    P.lp_val = (const unsigned char *)d_lp_val;
    P.lp_pat = (const unsigned char *)d_lp_pat;
    P.x = (const unsigned char *)d_x;
    P.y = d_y;
    P.bias = d_bias;
    P.G = G;
    P.nb = nb;
    P.ldx = ldx;
    P.ldy = ldy;
    P.T = T;
    P.c = (int)binom(m, n);
    const int64_t sets = nb / 32;
    P.sets_per_wave = (int)((sets + SS_WAVES - 1) / SS_WAVES);
    NMG_REQUIRE((int64_t)P.sets_per_wave * 4 * 64 * 8 * n < ((int64_t)1 << 31), NMG_ERR_UNSUPPORTED, "reduction too long");
    const int8_t *ord = host_order(n, m);
    NMG_REQUIRE(ord != nullptr && binom(m, n) * n <= (int64_t)sizeof(P.order), NMG_ERR_ARG, "invalid n:m = %d:%d", n, m);
    for (size_t e = 0; e < sizeof(P.order) / 4; e++) P.order[e] = 0;
    for (int64_t e = 0; e < binom(m, n) * n; e++) P.order[e >> 2] |= (uint32_t)(uint8_t)ord[e] << (8 * (e & 3));
    const int64_t groups = (G + SS_LINES - 1) / SS_LINES;
    NMG_REQUIRE(groups <= 0x3fffffffLL, NMG_ERR_UNSUPPORTED, "weight too large for one launch");
    hipStream_t s = (hipStream_t)stream;
    // 32 lines per workgroup where that gives the chip enough workgroups, else 16 (the token rows are
    // then read by twice the workgroups)
    const bool halves = groups < 192;
    const dim3 grid((unsigned)(halves ? 2 * groups : groups)), block(SS_WAVES * 64);
#define NMG_SS_N(TT, RB)                                                                     \
    switch (n) {                                                                               \
    case 1: hipLaunchKernelGGL((sstream_kernel<TT, 1, RB>), grid, block, 0, s, P); break;     \
    case 2: hipLaunchKernelGGL((sstream_kernel<TT, 2, RB>), grid, block, 0, s, P); break;     \
    default: hipLaunchKernelGGL((sstream_kernel<TT, 4, RB>), grid, block, 0, s, P); break;    \
    }
    if (dtype == NMG_F16) {
        if (halves) { NMG_SS_N(__half, 1) } else { NMG_SS_N(__half, 2) }
    } else {
        if (halves) { NMG_SS_N(__hip_bfloat16, 1) } else { NMG_SS_N(__hip_bfloat16, 2) }
    }
#undef NMG_SS_N
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}
