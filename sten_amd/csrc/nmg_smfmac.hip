// nmg x dense matmul on the sparse matrix cores (V_SMFMAC_F32_32X32X32_{F16,BF16}).
//
// Applies when the reduction runs along the sparse dim and every aligned group of 4 positions
// keeps at most 2 values (2:4, 1:4, 1:8, 2:8, 1:2, ...): the weight is the sparse A operand of
// the instruction, the activations the dense B operand.
//
//   Y[tok, f] = sum_k X[tok, k] * W[f, k] (+ bias[f])
//
// Operand ("fragpack", built once per weight by nmg_fragpack):
//   fp_val [MB][KS][64 lanes][8]  -- for feature block mb (32 rows) and k-step ks (32 dense k),
//                                    lane l holds the 4 pairs of kept values of row mb*32 + l%32
//   fp_idx [MB][KP][64 lanes] u32 -- 2-bit positions of those 8 values; low half-word = even
//                                    k-step of the pair, high half-word = odd k-step (ABID 0/1)
// Instruction layout (measured on gfx950): with B lane (col = l%32, h = l/32) holding dense
// k = 16h + e (e = 0..15), A lane (row = l%32, ga = l/32) pair q = 0..3 covers the 4-wide
// k-group kg = 4*(q/2) + 2*ga + (q%2); element 2q+i is selected by idx bits [4q+2i+1 : 4q+2i].
//
// Workgroup: WM x WN wavefronts, each 128 features x 64 tokens (4 x 2 accumulator blocks).
// A fragments go global -> registers (already in lane order, fully coalesced); the activation
// tile goes global -> registers -> LDS (double buffered), one barrier per 64-wide K step.
#include "nmg_common.h"

#include <map>
#include <mutex>
#include "nmg_tile.h"

#include <algorithm>
#include <type_traits>

namespace nmg {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x16 __attribute__((ext_vector_type(16)));

template <typename T> struct Smf;
template <> struct Smf<__half> {
    using A = f16x8;
    using B = f16x16;
    template <int ABID> __device__ static f32x16 run(A a, B b, f32x16 c, int idx)
    {
        return __builtin_amdgcn_smfmac_f32_32x32x32_f16(a, b, c, idx, 0, ABID);
    }
};
template <> struct Smf<__hip_bfloat16> {
    using A = bf16x8;
    using B = bf16x16;
    template <int ABID> __device__ static f32x16 run(A a, B b, f32x16 c, int idx)
    {
        return __builtin_amdgcn_smfmac_f32_32x32x32_bf16(a, b, c, idx, 0, ABID);
    }
};

struct SmfParams {
    const void *fp_val;
    const uint32_t *fp_idx;
    const void *x;
    void *y;
    const void *bias;
    int64_t M, K, T, ldx, ldy;
    int MB, KP;          // feature blocks of 32, k pairs of 64
    int tiles_m, tiles_n;
    int band;            // direct kernel: line tiles per band of the tile walk (4 or 8)
    // direct kernel with the reduction cut into slices (0 / 1: whole): slice s of a tile writes
    // its sums in single precision to part[s][token][feature], part_ld features per token
    int ksplit;
    float *part;
    int64_t part_ld;
};

constexpr int SMF_ROW = 144;  // bytes per token row in LDS: 64 k * 2 B + 16 B pad (conflict-free b128 reads)

// WM x WN wavefronts per workgroup, FB x TB accumulator blocks (32 features x 32 tokens) per
// wavefront, MINW = wavefronts per SIMD the register budget is sized for.  GUARD = false assumes
// K % 64 == 0 (no bounds checks in the K loop; token rows are clamped, feature blocks are padded
// in the operand).
template <typename T, int WM, int WN, int FB, int TB, int MINW, bool GUARD>
__global__ __launch_bounds__(64 * WM * WN, MINW) void spmm_smfmac_kernel(SmfParams P)
{
    using S = Smf<T>;
    constexpr int BMf = WM * FB * 32, BNt = WN * TB * 32;   // workgroup tile
    constexpr int NTHR = 64 * WM * WN;
    constexpr int NLOAD = BNt * 8 / NTHR;          // 16-byte chunks of the X tile per thread
    static_assert(NLOAD * NTHR == BNt * 8, "X tile must split evenly over the threads");
    extern __shared__ __align__(16) unsigned char smf_lds[];
    unsigned char (*Xs)[BNt * SMF_ROW] = (unsigned char (*)[BNt * SMF_ROW])smf_lds;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    // Workgroup -> tile: consecutive ids are dealt round-robin to the 8 XCDs, so give each XCD a
    // contiguous run of tiles (token tile fastest) and let it reuse its weight rows from its L2.
    int id = blockIdx.x;
    const int ntiles = P.tiles_m * P.tiles_n;
    if ((ntiles & 7) == 0) id = (id & 7) * (ntiles >> 3) + (id >> 3);
    const int tile_m = id / P.tiles_n, tile_n = id - tile_m * P.tiles_n;
    const int64_t f0 = (int64_t)tile_m * BMf, t0 = (int64_t)tile_n * BNt;

    const int KS = P.KP * 2;
    const int mb0 = (int)(f0 / 32) + wm * FB;
    const u32x4 zero4 = {0, 0, 0, 0};

    f32x16 acc[FB][TB];
#pragma unroll
    for (int i = 0; i < FB; i++)
#pragma unroll
        for (int j = 0; j < TB; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // ---- per-thread source pointers (advanced by one K step per iteration) ----
    const u32x4 *a_ptr[FB];
    const uint32_t *i_ptr[FB];
#pragma unroll
    for (int fb = 0; fb < FB; fb++) {
        // the operand is padded to whole workgroup tiles of feature blocks, so mb is always valid
        const int mb = mb0 + fb;
        a_ptr[fb] = (const u32x4 *)P.fp_val + (int64_t)mb * KS * 64 + lane;
        i_ptr[fb] = P.fp_idx + (int64_t)mb * P.KP * 64 + lane;
    }
    const unsigned char *x_ptr[NLOAD];
    bool x_ok[NLOAD];
    int x_lds[NLOAD];
#pragma unroll
    for (int i = 0; i < NLOAD; i++) {
        const int c = tid + i * NTHR;
        const int row = c >> 3, kc = c & 7;
        int64_t tok = t0 + row;
        x_ok[i] = tok < P.T;
        if (tok >= P.T) tok = P.T - 1;  // clamped rows are computed and never stored
        x_ptr[i] = (const unsigned char *)P.x + (tok * P.ldx + kc * 8) * 2;
        x_lds[i] = row * SMF_ROW + kc * 16;
    }

    u32x4 a_cur[FB][2], a_nxt[FB][2];
    uint32_t i_cur[FB], i_nxt[FB];
    u32x4 x_reg[NLOAD];

    auto load_a = [&](u32x4 (&a)[FB][2], uint32_t (&ix)[FB]) {
#pragma unroll
        for (int fb = 0; fb < FB; fb++) {
            a[fb][0] = a_ptr[fb][0];
            a[fb][1] = a_ptr[fb][64];
            ix[fb] = *i_ptr[fb];
            a_ptr[fb] += 128;
            i_ptr[fb] += 64;
        }
    };
    auto load_x = [&](int kp) {
#pragma unroll
        for (int i = 0; i < NLOAD; i++) {
            if (GUARD) {
                const int kc = (tid + i * NTHR) & 7;
                u32x4 v = zero4;
                if (x_ok[i] && (int64_t)kp * 64 + kc * 8 < P.K) v = *(const u32x4 *)x_ptr[i];
                x_reg[i] = v;
            } else {
                x_reg[i] = *(const u32x4 *)x_ptr[i];
            }
            x_ptr[i] += 128;
        }
    };
    auto store_x = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NLOAD; i++) *(u32x4 *)(&Xs[buf][x_lds[i]]) = x_reg[i];
    };

    load_a(a_cur, i_cur);
    load_x(0);
    store_x(0);
    __syncthreads();

    const int b_off = (lane & 31) * SMF_ROW + (lane >> 5) * 32 + wn * (TB * 32) * SMF_ROW;
    for (int kp = 0; kp < P.KP; kp++) {
        const int cur = kp & 1;
        const bool more = kp + 1 < P.KP;
        if (more) {
            load_a(a_nxt, i_nxt);
            load_x(kp + 1);
        }
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            typename S::B b[TB];
#pragma unroll
            for (int tb = 0; tb < TB; tb++) {
                const unsigned char *p = &Xs[cur][b_off + tb * 32 * SMF_ROW + ks * 64];
                union {
                    u32x4 u[2];
                    typename S::B v;
                } cv;
                cv.u[0] = *(const u32x4 *)p;
                cv.u[1] = *(const u32x4 *)(p + 16);
                b[tb] = cv.v;
            }
#pragma unroll
            for (int fb = 0; fb < FB; fb++) {
                union {
                    u32x4 u;
                    typename S::A v;
                } ca;
                ca.u = a_cur[fb][ks];
#pragma unroll
                for (int tb = 0; tb < TB; tb++) {
                    if (ks == 0)
                        acc[fb][tb] = S::template run<0>(ca.v, b[tb], acc[fb][tb], (int)i_cur[fb]);
                    else
                        acc[fb][tb] = S::template run<1>(ca.v, b[tb], acc[fb][tb], (int)i_cur[fb]);
                }
            }
        }
        if (more) {
            store_x(cur ^ 1);
#pragma unroll
            for (int fb = 0; fb < FB; fb++) {
                a_cur[fb][0] = a_nxt[fb][0];
                a_cur[fb][1] = a_nxt[fb][1];
                i_cur[fb] = i_nxt[fb];
            }
        }
        __syncthreads();
    }

    // ---- epilogue: D[row = feature][col = token]; lane holds token l%32, features
    //      8*(r/4) + 4*(l/32) + r%4 -> four consecutive features per register quad ----
    uint16_t *Y = (uint16_t *)P.y;
    const T *bias = (const T *)P.bias;
    const bool vec_ok = (P.ldy & 3) == 0 && ((uintptr_t)P.y & 7) == 0;
#pragma unroll
    for (int tb = 0; tb < TB; tb++) {
        const int64_t tok = t0 + (wn * TB + tb) * 32 + (lane & 31);
        if (tok >= P.T) continue;
#pragma unroll
        for (int fb = 0; fb < FB; fb++) {
#pragma unroll
            for (int rq = 0; rq < 4; rq++) {
                const int64_t f = f0 + (wm * FB + fb) * 32 + rq * 8 + (lane >> 5) * 4;
                if (f >= P.M) continue;
                uint16_t h[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    float v = acc[fb][tb][rq * 4 + i];
                    if (bias && f + i < P.M) v += to_f32(bias[f + i]);
                    h[i] = f32_to_bits16(v, (T *)nullptr);
                }
                uint16_t *dst = Y + tok * P.ldy + f;
                if (vec_ok && f + 3 < P.M) {
                    uint2 pk;
                    pk.x = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
                    pk.y = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
                    *(uint2 *)dst = pk;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (f + i < P.M) dst[i] = h[i];
                }
            }
        }
    }
}


// ------------------------------------------------------------- pipelined kernel, direct weights
// The fragpack operand is already in the register order of the instruction, so the weight
// fragments do not have to pass through LDS at all: each wavefront fetches its own fragments and
// index words from global memory into a ring of DR_D+1 register sets, DR_D K steps ahead of their
// use, and LDS carries the activation tile only.
//
// What bounds these kernels is the path from L2 through the CU's vector cache (64 B per clock):
// with the MFMAs alone a K step takes 0.29 us, with the LDS reads 0.33 us, and every KiB that a
// K step pulls through the vector cache adds to that.  So the wavefronts are stacked on the
// feature dim (WM = 4, each 64 features x all tokens of the tile): no two wavefronts fetch the
// same weight fragment, and a workgroup moves 18 KiB of weights + 16 KiB of activations per
// K step, the minimum for its tile.
//
// A workgroup is 4 wavefronts, one per SIMD, with the whole register file of the SIMD to
// itself; each also issues its quarter of the activation tile's DMA loads.  Every K step a
// wavefront issues XL DMA loads and 3*FB register loads for step kp+DR_D, so "step kp+1 has
// landed" is vmcnt <= OPS*(DR_D-1); the barrier that follows publishes the activation rows of
// all four wavefronts.  A DMA load writes 64 lanes x 16 B contiguously, so the activation rows
// cannot be padded; instead the 16-byte chunks of a row are XOR-swizzled with (row/2)%8, chosen on
// the global side, which makes the fragment reads (32 rows x 16 B at one logical chunk)
// conflict-free.  Requires K % 64 == 0 and activations smaller than 2 GiB (32-bit lane offsets).
//
// A K step is cut into 2 * NH phases (k-step of 32 x a part of the wavefront's token blocks): the
// MFMAs of a phase run while the activation fragments of the next one are read from LDS into a
// second register set.  Short phases pay: with four MFMAs per phase the 256 x 128 tile is 3-12 %
// faster than with eight (fewer fragments wait in registers, the LDS reads are spread thinner).
constexpr int DR_D = 3;                 // K steps in flight
constexpr int DR_NS = 4;                // activation stages in LDS (>= DR_D + 1)

//
// XT = true is the product with both dense operands transposed, C[M, T] = W * B for B [K, T]
// (what torch.mm(W, B) asks for): the activation tile of a K step is then 64 reduction rows x TT
// tokens, fetched as it lies in memory, and an activation fragment -- a lane wants 16 consecutive
// reduction positions of its token -- is four LDS transpose reads (DS_READ_B64_TR_B16: in every
// group of 16 lanes, lane i receives as element j the 16-bit element i%4 of the 8 bytes addressed
// by lane 4j + i/4); the epilogue stages [feature][token] and stores token-contiguous rows.
template <typename T, int FB, int TB, int WM, int WN, int NH, bool XT = false>
__global__ __launch_bounds__(256, 1) void spmm_smfmac_direct_kernel(SmfParams P)
{
    using S = Smf<T>;
    static_assert(WM * WN == 4, "four wavefronts");
    static_assert(TB % NH == 0, "token blocks split evenly into phases");
    constexpr int TF = WM * FB * 32, TT = WN * TB * 32;   // workgroup tile: features x tokens
    constexpr int STAGE = TT * 128;                       // activation bytes per K step
    constexpr int XL = TT / 32;                           // DMA loads per wavefront per K step
    constexpr int OPS = XL + 3 * FB;                      // memory operations per wavefront per K step
    constexpr int BT = TB / NH;                           // token blocks per phase
    constexpr int NP = 2 * NH;                            // phases per K step: (k-step, token part)
    constexpr int NM = FB * BT;                           // MFMAs per phase
    static_assert(OPS * DR_D < 64, "vmcnt is a 6-bit counter");
    static_assert(NM >= 4, "phase too short to hide the loads behind");
    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    int id = blockIdx.x;
    const int ntiles = P.tiles_m * P.tiles_n;
    // slices of the reduction: the slices of a tile are workgroups ntiles apart
    const int slice = P.ksplit > 1 ? id / ntiles : 0;
    id -= slice * ntiles;
    if ((ntiles & 7) == 0) id = (id & 7) * (ntiles >> 3) + (id >> 3);
    const int GH = P.band;
    const int band = id / (GH * P.tiles_n);
    const int band_h = min(P.tiles_m - band * GH, GH);
    const int in_band = id - band * GH * P.tiles_n;
    const int tile_m = band * GH + in_band % band_h, tile_n = in_band / band_h;
    const int64_t f0 = (int64_t)tile_m * TF, t0 = (int64_t)tile_n * TT;
    // k pairs kp_lo .. kp_lo + KP - 1 of the operand's KPT (the host leaves no slice empty)
    const int KPT = P.KP;
    const int kp_per = P.ksplit > 1 ? (KPT + P.ksplit - 1) / P.ksplit : KPT;
    const int kp_lo = slice * kp_per;
    const int KP = min(KPT, kp_lo + kp_per) - kp_lo;
    const int wm = wave / WN, wn = wave % WN;
    const int mb0 = (int)(f0 / 32) + wm * FB;

    // ---- global sources (wavefront-uniform bases in scalar registers, the lane's share as a
    //      32-bit offset) ----
    const unsigned char *av_base[FB];
    const unsigned char *ai_base[FB];
#pragma unroll
    for (int fb = 0; fb < FB; fb++) {
        av_base[fb] = (const unsigned char *)P.fp_val + (((int64_t)(mb0 + fb) * KPT + kp_lo) * 2) * 1024;
        ai_base[fb] = (const unsigned char *)P.fp_idx + ((int64_t)(mb0 + fb) * KPT + kp_lo) * 256;
    }
    const uint32_t lane16 = lane * 16, lane4 = lane * 4;
    // K step kp of the activations starts kp * XSTEP bytes into the operand
    const int64_t XSTEP = XT ? 64 * P.ldx * 2 : 128;
    const unsigned char *x_base = (const unsigned char *)P.x + (int64_t)kp_lo * XSTEP;
    uint32_t x_off[XL];
#pragma unroll
    for (int i = 0; i < XL; i++) {
        if constexpr (XT) {
            // a DMA load fills 1 KiB = 1024 / (TT * 2) reduction rows of the tile; piece p (8 tokens)
            // of row k holds the logical chunk p ^ 4*(k%4), which spreads the transpose reads
            // of four consecutive rows over all banks
            constexpr int PPR = TT / 8;                       // 16-byte pieces per row
            const int row = (wave * XL + i) * (64 / PPR) + lane / PPR;
            const int chunk = (lane % PPR) ^ ((row & 3) << 2);
            int64_t tok = t0 + chunk * 8;
            if (tok > P.T - 8) tok = (P.T - 1) / 8 * 8;       // clamped columns are computed, never stored
            x_off[i] = (uint32_t)((row * P.ldx + tok) * 2);
        } else {
            const int row = (wave * XL + i) * 8 + (lane >> 3);
            const int piece = lane & 7;
            const int q = piece ^ ((row >> 1) & 7);
            int64_t tok = t0 + row;
            if (tok >= P.T) tok = P.T - 1;
            x_off[i] = (uint32_t)((tok * P.ldx + q * 8) * 2);
        }
    }

    struct WSet {
        u32x4 a[FB][2];
        uint32_t ix[FB];
    };
    WSet ws[DR_D + 1];
    // Load number i (0 .. OPS-1) of K step kp: first the XL activation DMA loads, then per
    // feature block two weight fragments and the index word.  Steps beyond the last repeat it:
    // the operation count stays uniform, the data is unused.
    auto issue_one = [&](int kp, WSet &w, int i) {
        if (kp >= KP) kp = KP - 1;
        if (i < XL) {
            unsigned char *base = smem + (kp & (DR_NS - 1)) * STAGE;
            const unsigned char *xb = x_base + (int64_t)kp * XSTEP;
#pragma unroll
            for (int q = 0; q < XL; q++)
                if (q == i)
                    __builtin_amdgcn_global_load_lds((glb_ptr_t)(xb + x_off[q]),
                                                     (lds_ptr_t)(base + (wave * XL + q) * 1024), 16, 0, 0);
        } else {
            // Written as instructions so that their completion is tracked by the explicit vmcnt
            // waits below and by nothing else (left to itself the compiler waits for vmcnt(0) at
            // the loop head, which empties the pipeline every K step), and with accumulation
            // registers as targets: the ring does not fit beside the accumulators in the 256
            // architectural registers, and a compiler-made copy of a register whose load is
            // still in flight would copy stale data.
#pragma unroll
            for (int fb = 0; fb < FB; fb++) {
                const unsigned char *av = av_base[fb] + (int64_t)kp * 2048;
                const unsigned char *ai = ai_base[fb] + (int64_t)kp * 256;
                if (XL + fb * 3 == i)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=a"(w.a[fb][0]) : "v"(lane16), "s"(av) : "memory");
                if (XL + fb * 3 + 1 == i)
                    asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024" : "=a"(w.a[fb][1]) : "v"(lane16), "s"(av) : "memory");
                if (XL + fb * 3 + 2 == i)
                    asm volatile("global_load_dword %0, %1, %2" : "=v"(w.ix[fb]) : "v"(lane4), "s"(ai) : "memory");
            }
        }
    };
    auto issue_step = [&](int kp, WSet &w) {
#pragma unroll
        for (int i = 0; i < OPS; i++) issue_one(kp, w, i);
    };

    f32x16 acc[FB][TB];
#pragma unroll
    for (int i = 0; i < FB; i++)
#pragma unroll
        for (int j = 0; j < TB; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // 256 accumulators fill the architectural registers exactly; left alone the allocator
    // puts them all there and spills everything else.  Pin half of them to the accumulation
    // registers (the MFMA takes its C/D operand from either file).
    auto pin_acc = [&]() {
        if constexpr (FB * TB * 16 > 128) {
#pragma unroll
            for (int tb = 0; tb < TB; tb++) asm volatile("" : "+a"(acc[FB - 1][tb]));
        }
    };
    pin_acc();

    const int j = lane & 31, h = lane >> 5, sw = (j >> 1) & 7;
    int b_off[2][2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int c = 0; c < 2; c++)
            b_off[ks][c] = (wn * TB * 32 + j) * 128 + (((ks * 4 + h * 2 + c) ^ sw) << 4);

    // Activation fragments of one phase (k-step ks, token part hh); two sets alternate.
    struct BFrags {
        u32x4 b[BT][2];
    };
    BFrags fr[2];
    // XT: lane (g = l/16, i = l%16) of a transpose read supplies the 8 bytes at reduction row
    // 16*(g/2) + i/4 (+ 32*ks + 4*r), tokens 16*(g%2) + 4*(i%4) .. +3 of the 32-token block, and
    // receives token l%32 at rows 16*(l/32) + 4r + 0..3: reads r = 0..3 are the lane's 16 positions.
    int t_off[TB];
    if constexpr (XT) {
        const int g = lane >> 4, i16 = lane & 15, a = i16 >> 2;
#pragma unroll
        for (int tb = 0; tb < TB; tb++) {
            const int chunk = (wn * TB + tb) * 4 + 2 * (g & 1) + ((i16 & 3) >> 1);   // 8-token chunk of the row
            t_off[tb] = (16 * (g >> 1) + a) * (TT * 2) + ((chunk ^ (a << 2)) << 4) + (i16 & 1) * 8;
        }
    }
    // part 0 / 1: the first / second half of the phase's reads (part < 0: all of them)
    auto read_b = [&](BFrags &f, const unsigned char *base, int ph, int part = -1) {
        const int ks = ph / NH, hh = ph % NH;
#pragma unroll
        for (int t = 0; t < BT; t++) {
            if (BT >= 2 && part >= 0 && t / (BT / 2) != part) continue;
            if constexpr (XT) {
                typedef short i16x4 __attribute__((ext_vector_type(4)));
                typedef __attribute__((address_space(3))) i16x4 *lds_i16x4;
                union {
                    i16x4 h[4];
                    u32x4 u[2];
                } c;
#pragma unroll
                for (int r = 0; r < 4; r++)
                    c.h[r] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (lds_i16x4)(base + t_off[hh * BT + t] + (32 * ks + 4 * r) * (TT * 2)));
                f.b[t][0] = c.u[0];
                f.b[t][1] = c.u[1];
            } else {
                if (BT >= 2 || part != 1) f.b[t][0] = *(const u32x4 *)(base + b_off[ks][0] + (hh * BT + t) * 32 * 128);
                if (BT >= 2 || part != 0) f.b[t][1] = *(const u32x4 *)(base + b_off[ks][1] + (hh * BT + t) * 32 * 128);
            }
        }
    };
    // MFMAs lo..hi-1 of phase PH, numbered fb * BT + t
    auto mma = [&](const WSet &w, const BFrags &f, auto ph_tag, int lo, int hi) {
        constexpr int PH = decltype(ph_tag)::value, KSI = PH / NH, HH = PH % NH;
#pragma unroll
        for (int fb = 0; fb < FB; fb++) {
            union {
                u32x4 u;
                typename S::A v;
            } ca;
            ca.u = w.a[fb][KSI];
#pragma unroll
            for (int t = 0; t < BT; t++) {
                if (fb * BT + t < lo || fb * BT + t >= hi) continue;
                union {
                    u32x4 u[2];
                    typename S::B v;
                } cb;
                cb.u[0] = f.b[t][0];
                cb.u[1] = f.b[t][1];
                acc[fb][HH * BT + t] = S::template run<KSI>(ca.v, cb.v, acc[fb][HH * BT + t], (int)w.ix[fb]);
            }
        }
    };

    // The counted wait.  (1) A wavefront's vector memory operations complete in issue order and
    // it issues exactly OPS of them per K step, all of step kp+DR_D before the wait at the end of
    // step kp: when the counter is down to (DR_D-1) * OPS, step kp+1 has landed; the barrier after
    // it extends that to the DMA loads of the other wavefronts.  (2) The weight set of step kp+1
    // passes through the wait as in/out operands, so its later uses are ordered after the wait by
    // the compiler as well; that nothing touches a register with a load in flight *before* the
    // wait is checked on the compiled code (`python -m sten_amd.isa_check`).  (3) LDS stage
    // (kp+DR_D) % DR_NS is refilled during step kp; its last readers, the fragment reads of step
    // kp+DR_D-DR_NS < kp, completed (lgkmcnt(0), same wait) before the barrier of their step.
    static_assert(DR_NS > DR_D, "a stage must not be refilled while the step that reads it is in flight");
    static_assert(NP % 2 == 0, "fragment sets alternate by phase across K steps");
    static_assert(FB == 2, "the wait lists the registers of two fragment rows");
    auto landed = [&](WSet &w) {
        asm volatile("s_waitcnt vmcnt(%6) lgkmcnt(0)"
                     : "+a"(w.a[0][0]), "+a"(w.a[0][1]), "+v"(w.ix[0]), "+a"(w.a[1][0]), "+a"(w.a[1][1]), "+v"(w.ix[1])
                     : "n"((DR_D - 1) * OPS)
                     : "memory");
    };

    // prologue: steps 0 .. DR_D-1 in flight, then wait for step 0
#pragma unroll
    for (int st = 0; st < DR_D; st++) {
        issue_step(st, ws[st]);
    }
    landed(ws[0]);
    asm volatile("s_barrier" ::: "memory");
    read_b(fr[0], smem, 0);

    for (int kp0 = 0; kp0 < KP; kp0 += DR_D + 1) {
#pragma unroll
        for (int u = 0; u <= DR_D; u++) {
            const int kp = kp0 + u;
            if (kp >= KP) break;
            const unsigned char *base = smem + (kp & (DR_NS - 1)) * STAGE;
            const unsigned char *next = smem + ((kp + 1) & (DR_NS - 1)) * STAGE;
            // One phase: two MFMAs; the LDS reads of the next phase into the other fragment set;
            // its share of the loads of step kp+DR_D between the rest of the MFMAs.  Before the
            // reads of the last phase, which fetch from the next stage, the barrier.  The
            // instruction statements fence the scheduler, so this is also the issue order.
            auto phase = [&](auto ph_tag) {
                constexpr int PH = decltype(ph_tag)::value;
                constexpr int L0 = PH * OPS / NP, L1 = (PH + 1) * OPS / NP;
                // One memory instruction (or two LDS reads) goes into the shadow of one MFMA: a load
                // holds the wavefront's issue for about 20 clocks, an LDS read for 7, an MFMA runs 32.
                // (XT: the transposing reads of a block stay together.)
                constexpr bool SPLIT = !XT && BT >= 2 && NM >= 4;   // measured in steady state: -3..6 % on the 256 x 256 tile, -1 % on 256 x 128
                if (PH == NP - 1) {
                    mma(ws[u], fr[PH % 2], ph_tag, 0, 2);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int i = L0; i < OPS; i++) issue_one(kp + DR_D, ws[(u + DR_D) % (DR_D + 1)], i);
                    __builtin_amdgcn_sched_barrier(0);
                    // fragments of step kp are in registers, my share of step kp+1 has landed ...
                    landed(ws[(u + 1) % (DR_D + 1)]);
                    asm volatile("s_barrier" ::: "memory");              // ... and everybody else's
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (SPLIT) {
                        mma(ws[u], fr[PH % 2], ph_tag, 2, 3);
                        __builtin_amdgcn_sched_barrier(0);
                        read_b(fr[(PH + 1) % 2], next, 0, 0);
                        __builtin_amdgcn_sched_barrier(0);
                        mma(ws[u], fr[PH % 2], ph_tag, 3, 4);
                        __builtin_amdgcn_sched_barrier(0);
                        read_b(fr[(PH + 1) % 2], next, 0, 1);
                        __builtin_amdgcn_sched_barrier(0);
                        mma(ws[u], fr[PH % 2], ph_tag, 4, NM);
                    } else {
                        read_b(fr[(PH + 1) % 2], next, 0);
                        mma(ws[u], fr[PH % 2], ph_tag, 2, NM);
#pragma unroll
                        for (int i = 0; i < BT; i++) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                        }
                    }
                } else {
                    if constexpr (SPLIT) {
                        mma(ws[u], fr[PH % 2], ph_tag, 0, 1);
                        __builtin_amdgcn_sched_barrier(0);
                        read_b(fr[(PH + 1) % 2], base, PH + 1, 0);
                        __builtin_amdgcn_sched_barrier(0);
                        mma(ws[u], fr[PH % 2], ph_tag, 1, 2);
                        __builtin_amdgcn_sched_barrier(0);
                        read_b(fr[(PH + 1) % 2], base, PH + 1, 1);
                    } else {
                        mma(ws[u], fr[PH % 2], ph_tag, 0, 2);
                        __builtin_amdgcn_sched_barrier(0);
                        read_b(fr[(PH + 1) % 2], base, PH + 1);
                    }
                    // the step's OPS loads are dealt out over its phases, one at a time between MFMAs
#pragma unroll
                    for (int i = L0; i < L1; i++) {
                        __builtin_amdgcn_sched_barrier(0);
                        if (2 + i - L0 < NM) mma(ws[u], fr[PH % 2], ph_tag, 2 + i - L0, 3 + i - L0);
                        __builtin_amdgcn_sched_barrier(0);
                        issue_one(kp + DR_D, ws[(u + DR_D) % (DR_D + 1)], i);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if (2 + L1 - L0 < NM) mma(ws[u], fr[PH % 2], ph_tag, 2 + L1 - L0, NM);
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            phase(std::integral_constant<int, 0>{});
            phase(std::integral_constant<int, 1>{});
            if constexpr (NP >= 4) {
                phase(std::integral_constant<int, 2>{});
                phase(std::integral_constant<int, 3>{});
            }
            if constexpr (NP == 8) {
                phase(std::integral_constant<int, 4>{});
                phase(std::integral_constant<int, 5>{});
                phase(std::integral_constant<int, 6>{});
                phase(std::integral_constant<int, 7>{});
            }
            static_assert(NP == 2 || NP == 4 || NP == 8, "one, two or four token parts");
        }
    }
    pin_acc();
    // The loads of the steps beyond the last are still in flight and nothing reads what they bring:
    // every register of the ring passes through the final wait, so that none of them is given to
    // the epilogue while a load may still land in it.
    static_assert(DR_D == 3 && FB == 2, "the final wait lists four weight sets of two fragment rows");
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+a"(ws[0].a[0][0]), "+a"(ws[0].a[0][1]), "+a"(ws[0].a[1][0]), "+a"(ws[0].a[1][1]), "+v"(ws[0].ix[0]), "+v"(ws[0].ix[1]),
                   "+a"(ws[1].a[0][0]), "+a"(ws[1].a[0][1]), "+a"(ws[1].a[1][0]), "+a"(ws[1].a[1][1]), "+v"(ws[1].ix[0]), "+v"(ws[1].ix[1]),
                   "+a"(ws[2].a[0][0]), "+a"(ws[2].a[0][1]), "+a"(ws[2].a[1][0]), "+a"(ws[2].a[1][1]), "+v"(ws[2].ix[0]), "+v"(ws[2].ix[1]),
                   "+a"(ws[3].a[0][0]), "+a"(ws[3].a[0][1]), "+a"(ws[3].a[1][0]), "+a"(ws[3].a[1][1]), "+v"(ws[3].ix[0]), "+v"(ws[3].ix[1])
                 :
                 : "memory");
    asm volatile("s_barrier" ::: "memory");
    if (P.ksplit > 1) {
        store_partial_tile<FB, TB>(acc, P.part + (int64_t)slice * P.T * P.part_ld, P.part_ld, lane,
                                   f0 + wm * FB * 32, t0 + wn * TB * 32, P.T);
        return;
    }
    const TileOut out{P.y, P.bias, P.M, P.T, P.ldy};
    if constexpr (XT)
        smf_store_tile_t<T, FB, TB>(acc, smem + wave * (FB * 32 * (TB * 64 + 16)), lane, f0 + wm * FB * 32,
                                    t0 + wn * TB * 32, out);
    else
        smf_store_tile<T, FB, TB>(acc, smem + wave * (TB * 32 * (FB * 64 + 16)), lane, f0 + wm * FB * 32,
                                  t0 + wn * TB * 32, out);
}

template <typename T, int FB, int TB, int WM, int WN, int NH, bool XT = false>
static int launch_smfmac_direct(SmfParams &P, hipStream_t s)
{
    constexpr int TF = WM * FB * 32, TT = WN * TB * 32;
    static_assert(TF == 256, "the operand is padded to 256 lines");
    P.tiles_m = (int)((P.M + TF - 1) / TF);
    P.tiles_n = (int)((P.T + TT - 1) / TT);
    // An XCD works on 32 consecutive tiles of the walk at a time, a block of `band` line tiles x
    // 32 / band token tiles, and fetches that block's weights and activations into its L2: the
    // block is taller where a token tile's activations outweigh a line tile's weights.
    P.band = (int64_t)TT * 2 * 8 > (int64_t)TF * 9 ? 8 : 4;   // bytes per reduction position: TT * 2 against TF * 9 / 8
    const int slices = P.ksplit > 1 ? P.ksplit : 1;
    dim3 grid((unsigned)(P.tiles_m * P.tiles_n * slices));
    constexpr size_t ring = (size_t)DR_NS * TT * 128;
    constexpr size_t stg = XT ? (size_t)4 * FB * 32 * (TB * 64 + 16) : (size_t)4 * TB * 32 * (FB * 64 + 16);
    constexpr size_t lds = ring > stg ? ring : stg;
    static_assert(lds <= 160 * 1024, "LDS");
    static_assert(!XT || (TT == 128 && WN == 1), "the transposed tile is 64 rows of 128 tokens");
    auto k = spmm_smfmac_direct_kernel<T, FB, TB, WM, WN, NH, XT>;
    NMG_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(k, grid, dim3(256), lds, s, P);
    NMG_HIP_TRY(hipGetLastError());
    if (slices > 1) {
        const SplitSum Q{P.part, P.y, P.bias, P.M, P.T, P.ldy, P.part_ld, slices};
        return launch_splitk_sum<T>(Q, s);
    }
    return NMG_OK;
}

// --------------------------------------------------------------------------- decode kernel
// Few tokens (T <= 16): the weight is streamed once from HBM and everything else is noise, so
// the kernel is built around keeping many coalesced 1 KiB fragment loads in flight.  The sparse
// matrix core still does the arithmetic -- tokens are padded to the 32 columns of one MFMA,
// which costs nothing when the kernel is bandwidth-bound and spares any cross-lane reduction.
// One workgroup owns a block of 32 lines; its SK_NW wavefronts split K, keep two batches of
// loads in flight (fetch batch i+1, multiply batch i), accumulate in registers, and are summed
// through LDS at the end.  (Splitting K over several workgroups as well was tried and dropped:
// the device-scope fences it needs write back and invalidate the XCD's L2 and cost 10x.)
// SK_NW wavefronts per workgroup, SK_UNROLL k pairs (64 dense k each) fetched per batch.
template <typename T, int SK_NW, int SK_UNROLL>
__global__ __launch_bounds__(64 * SK_NW) void spmm_smfmac_skinny_kernel(SmfParams P)
{
    using S = Smf<T>;
    __shared__ float red[SK_NW][32][17];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int mb = blockIdx.x;
    const int KP = P.KP;
    const int j = lane & 31, h = lane >> 5;
    const u32x4 zero4 = {0, 0, 0, 0};
    // this wavefront's k pairs: a contiguous slice
    const int per = (KP + SK_NW - 1) / SK_NW;
    const int kp_lo = wave * per, kp_hi = min(KP, kp_lo + per);

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;

    const u32x4 *aval = (const u32x4 *)P.fp_val + ((int64_t)mb * KP * 2) * 64 + lane;
    const uint32_t *aidx = P.fp_idx + ((int64_t)mb * KP) * 64 + lane;
    const bool tok_ok = j < P.T;
    const unsigned char *xrow = (const unsigned char *)P.x + ((int64_t)(tok_ok ? j : 0) * P.ldx + 16 * h) * 2;

    struct Batch {
        u32x4 a[SK_UNROLL][2], b[SK_UNROLL][2][2];
        uint32_t ix[SK_UNROLL];
    };
    auto fetch = [&](Batch &B, int kp0) {
#pragma unroll
        for (int u = 0; u < SK_UNROLL; u++) {
            const int kp = kp0 + u;
            const bool live = kp < kp_hi;
            B.a[u][0] = live ? aval[(int64_t)kp * 128] : zero4;
            B.a[u][1] = live ? aval[(int64_t)kp * 128 + 64] : zero4;
            B.ix[u] = live ? aidx[(int64_t)kp * 64] : 0x44444444u;
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    const int64_t k = (int64_t)kp * 64 + ks * 32 + 16 * h + 8 * c;
                    B.b[u][ks][c] = (live && tok_ok && k < P.K)
                                        ? *(const u32x4 *)(xrow + ((int64_t)kp * 64 + ks * 32 + 8 * c) * 2)
                                        : zero4;
                }
        }
    };
    auto consume = [&](const Batch &B) {
#pragma unroll
        for (int u = 0; u < SK_UNROLL; u++) {
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                union {
                    u32x4 u4;
                    typename S::A v;
                } ca;
                ca.u4 = B.a[u][ks];
                union {
                    u32x4 u4[2];
                    typename S::B v;
                } cb;
                cb.u4[0] = B.b[u][ks][0];
                cb.u4[1] = B.b[u][ks][1];
                if (ks == 0)
                    acc = S::template run<0>(ca.v, cb.v, acc, (int)B.ix[u]);
                else
                    acc = S::template run<1>(ca.v, cb.v, acc, (int)B.ix[u]);
            }
        }
    };

    Batch b0, b1;
    fetch(b0, kp_lo);
    for (int kp0 = kp_lo; kp0 < kp_hi; kp0 += 2 * SK_UNROLL) {
        fetch(b1, kp0 + SK_UNROLL);
        consume(b0);
        fetch(b0, kp0 + 2 * SK_UNROLL);
        consume(b1);
    }
    // D[row = line][col = token]: lane holds token j, lines 8*(r/4) + 4*h + r%4
    if (j < 16) {
#pragma unroll
        for (int r = 0; r < 16; r++) red[wave][(r >> 2) * 8 + h * 4 + (r & 3)][j] = acc[r];
    }
    __syncthreads();
    // 32 lines x 16 tokens = 512 sums over SK_NW partials
    for (int e = tid; e < 32 * 16; e += 64 * SK_NW) {
        const int line = e & 31, tok = e >> 5;
        const int64_t f = (int64_t)mb * 32 + line;
        if (tok >= P.T || f >= P.M) continue;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < SK_NW; w++) s += red[w][line][tok];
        if (P.bias) s += to_f32(((const T *)P.bias)[f]);
        ((uint16_t *)P.y)[tok * P.ldy + f] = f32_to_bits16(s, (T *)nullptr);
    }
}

template <typename T, int NW, int UN> static int launch_smfmac_skinny(SmfParams &P, hipStream_t s)
{
    dim3 grid((unsigned)((P.M + 31) / 32));
    hipLaunchKernelGGL((spmm_smfmac_skinny_kernel<T, NW, UN>), grid, dim3(64 * NW), 0, s, P);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

// Decode kernel with staged activations (the default when K % 128 == 0).  In the kernel above a
// wavefront's activation loads touch 32 bytes of each token row per instruction (two lanes per
// token); from 8 tokens on the activations weigh as much as the weight in the vector memory
// path (18.7 us against 12.7 us here at 16 tokens on a 4096 x 11008 weight; 12.0 against 9.9 at
// one token).  Here a wavefront stages the
// activations of its next 128 reduction positions in LDS with row-contiguous DMA loads (256 bytes
// per token and instruction) and reads its fragments from there.  The staging area is private to
// the wavefront, so no barrier is involved: a chunk's DMA loads are issued before its weight
// loads, and the counted wait for the chunk covers both.
// Chunk = 2 k pairs (128 dense positions): ND DMA loads (4 token rows each) + 6 weight loads.
// One chunk is in flight while the previous one is multiplied.  16-byte pieces of a row are
// XOR-swizzled with the row number so that the 16 rows of a fragment read hit distinct banks.
// A weight of few blocks (4096 lines: 128) would leave half of the CUs without a workgroup:
// SPLIT workgroups share a block, each fetches the runs of its 32 / SPLIT lines of every
// fragment and multiplies zeros in the other lanes -- no sum across workgroups is needed.
template <typename T, int SK_NW, int ND, int SPLIT, int TK = 16>
__global__ __launch_bounds__(64 * SK_NW) void spmm_smfmac_decode_staged_kernel(SmfParams P)
{
    using S = Smf<T>;
    constexpr int OPS = ND + 6;
    constexpr int LPB = 32 / SPLIT;                     // lines of the block that this workgroup owns
    constexpr int BUF = TK * 256;                       // one chunk: TK (16 or 32) token rows x 256 bytes
    static_assert((TK == 16 || TK == 32) && ND * 4 <= TK, "four token rows per DMA load");
    extern __shared__ __align__(16) unsigned char smem[];
    static_assert(SK_NW * 2 * BUF >= SK_NW * 32 * (TK + 1) * 4, "the reduction buffer reuses the staging area");
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int mb = blockIdx.x / SPLIT, part = blockIdx.x % SPLIT;
    const int KP = P.KP;
    const int j = lane & 31, h = lane >> 5;
    // The lanes of this workgroup's lines fetch their share of a fragment (a run of 16 * LPB
    // bytes in each half of it); the other lanes repeat those addresses and multiply zeros.
    const bool mine = (j / LPB) == part;
    const int src_lane = (lane & 32) | (part * LPB + (j & (LPB - 1)));
    // an even number of k pairs per wavefront: chunks never straddle two ranges (KP is even)
    const int per = (((KP + SK_NW - 1) / SK_NW) + 1) & ~1;
    const int kp_lo = wave * per, kp_hi = min(KP, kp_lo + per);
    unsigned char *stage = smem + wave * (2 * BUF);

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;

    const unsigned char *aval = (const unsigned char *)P.fp_val + ((int64_t)mb * KP * 2) * 1024;
    const unsigned char *aidx = (const unsigned char *)P.fp_idx + ((int64_t)mb * KP) * 256;
    const uint32_t lane16 = src_lane * 16, lane4 = src_lane * 4;
    // DMA source of lane l in load i: token row 4i + l/16 (clamped: surplus rows repeat the last
    // token and are never stored), logical 16-byte piece (l%16) ^ row
    uint32_t x_off[ND];
#pragma unroll
    for (int i = 0; i < ND; i++) {
        const int row = 4 * i + (lane >> 4);
        const int q = (lane & 15) ^ (row & 15);
        const int64_t tok = row < P.T ? row : P.T - 1;
        x_off[i] = (uint32_t)((tok * P.ldx + q * 8) * 2);
    }
    // fragment read offsets: lane (token j, half h), k pair kl, k-step ks, piece c
    int b_off[2][2][2];
#pragma unroll
    for (int kl = 0; kl < 2; kl++)
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
#pragma unroll
            for (int c = 0; c < 2; c++)
                b_off[kl][ks][c] = (j & (TK - 1)) * 256 + (((kl * 8 + ks * 4 + 2 * h + c) ^ (j & 15)) << 4);

    struct ASet {
        u32x4 a[2][2];
        uint32_t ix[2];
    };
    ASet as[2];
    // Loads of the chunk that starts at k pair kp0.  Beyond the wavefront's range they repeat its
    // last chunk (just fetched: no traffic to HBM), so the count of operations stays uniform;
    // the data is zeroed later.
    const int kp_last = max(kp_hi - 2, 0);
    auto issue_x = [&](int kp0, unsigned char *buf) {
        const unsigned char *xb = (const unsigned char *)P.x + (int64_t)min(kp0, kp_last) * 128;
#pragma unroll
        for (int i = 0; i < ND; i++)
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(xb + x_off[i]), (lds_ptr_t)(buf + i * 1024), 16, 0, 0);
    };
    auto issue_w = [&](int kp0, ASet &A) {
#pragma unroll
        for (int kl = 0; kl < 2; kl++) {
            const int kp = min(kp0, kp_last) + kl;
            const unsigned char *av = aval + (int64_t)kp * 2048;
            const unsigned char *ai = aidx + (int64_t)kp * 256;
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(A.a[kl][0]) : "v"(lane16), "s"(av) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024" : "=v"(A.a[kl][1]) : "v"(lane16), "s"(av) : "memory");
            asm volatile("global_load_dword %0, %1, %2" : "=v"(A.ix[kl]) : "v"(lane4), "s"(ai) : "memory");
        }
    };
    auto consume = [&](int kp0, const unsigned char *buf, ASet &A) {
        u32x4 b[2][2][2];
#pragma unroll
        for (int kl = 0; kl < 2; kl++)
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
#pragma unroll
                for (int c = 0; c < 2; c++) b[kl][ks][c] = *(const u32x4 *)(buf + b_off[kl][ks][c]);
#pragma unroll
        for (int kl = 0; kl < 2; kl++) {
            // k pairs beyond the wavefront's range (or, when K is not a multiple of 128, beyond the
            // chunk's real extent) contribute nothing: their weights are replaced by zeros
            const bool live = kp0 + kl < kp_hi && (SPLIT == 1 || mine);
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                union {
                    u32x4 u4;
                    typename S::A v;
                } ca;
                const u32x4 zero4 = {0, 0, 0, 0};
                ca.u4 = live ? A.a[kl][ks] : zero4;
                union {
                    u32x4 u4[2];
                    typename S::B v;
                } cb;
                cb.u4[0] = b[kl][ks][0];
                cb.u4[1] = b[kl][ks][1];
                if (ks == 0)
                    acc = S::template run<0>(ca.v, cb.v, acc, (int)A.ix[kl]);
                else
                    acc = S::template run<1>(ca.v, cb.v, acc, (int)A.ix[kl]);
            }
        }
    };

    issue_x(kp_lo, stage);
    issue_w(kp_lo, as[0]);
    for (int kp0 = kp_lo; kp0 < kp_hi; kp0 += 4) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int kc = kp0 + 2 * u;
            if (kc >= kp_hi) break;
            // (the other buffer was read out before the MFMAs of the previous chunk)
            issue_x(kc + 2, stage + ((u + 1) & 1) * BUF);
            issue_w(kc + 2, as[(u + 1) & 1]);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(OPS) : "memory");   // chunk kc has landed
            __builtin_amdgcn_sched_barrier(0);
            consume(kc, stage + (u & 1) * BUF, as[u]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // the last loads (beyond the wavefront's range) are in flight and unused: their registers pass
    // through the final wait, so that none is reused while a load may still land in it
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(as[0].a[0][0]), "+v"(as[0].a[0][1]), "+v"(as[0].a[1][0]), "+v"(as[0].a[1][1]), "+v"(as[0].ix[0]), "+v"(as[0].ix[1]),
                   "+v"(as[1].a[0][0]), "+v"(as[1].a[0][1]), "+v"(as[1].a[1][0]), "+v"(as[1].a[1][1]), "+v"(as[1].ix[0]), "+v"(as[1].ix[1])
                 :
                 : "memory");
    __syncthreads();   // every wavefront is done with its staging area: reuse it for the reduction
    float(*red)[32][TK + 1] = (float(*)[32][TK + 1])smem;
    // D[row = line][col = token]: lane holds token j, lines 8*(r/4) + 4*h + r%4
    if (j < TK) {
#pragma unroll
        for (int r = 0; r < 16; r++) red[wave][(r >> 2) * 8 + h * 4 + (r & 3)][j] = acc[r];
    }
    __syncthreads();
    for (int e = tid; e < LPB * TK; e += 64 * SK_NW) {
        const int line = part * LPB + (e & (LPB - 1)), tok = e / LPB;
        const int64_t f = (int64_t)mb * 32 + line;
        if (tok >= P.T || f >= P.M) continue;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < SK_NW; w++) s += red[w][line][tok];
        if (P.bias) s += to_f32(((const T *)P.bias)[f]);
        ((uint16_t *)P.y)[tok * P.ldy + f] = f32_to_bits16(s, (T *)nullptr);
    }
}

template <typename T, int NW, int ND, int SPLIT, int TK = 16>
static int launch_smfmac_decode_staged(SmfParams &P, hipStream_t s)
{
    dim3 grid((unsigned)((P.M + 31) / 32 * SPLIT));
    constexpr size_t lds = (size_t)NW * 2 * TK * 256;
    if (lds > 160 * 1024) return NMG_ERR_UNSUPPORTED;   // (16 wavefronts x 32 token rows: not dispatched)
    auto k = spmm_smfmac_decode_staged_kernel<T, NW, ND, SPLIT, TK>;
    if (lds > 64 * 1024)
        NMG_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(k, grid, dim3(64 * NW), lds, s, P);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

template <typename T, int NW, int SPLIT = 1>
static int launch_smfmac_decode_staged_nd(SmfParams &P, hipStream_t s)
{
    switch ((int)(P.T + 3) / 4) {
    case 1: return launch_smfmac_decode_staged<T, NW, 1, SPLIT>(P, s);
    case 2: return launch_smfmac_decode_staged<T, NW, 2, SPLIT>(P, s);
    case 3: return launch_smfmac_decode_staged<T, NW, 3, SPLIT>(P, s);
    case 4: return launch_smfmac_decode_staged<T, NW, 4, SPLIT>(P, s);
    // 17 .. 32 tokens: the second half of the instruction's 32 token columns is used too
    case 5: return launch_smfmac_decode_staged<T, NW, 5, SPLIT, 32>(P, s);
    case 6: return launch_smfmac_decode_staged<T, NW, 6, SPLIT, 32>(P, s);
    case 7: return launch_smfmac_decode_staged<T, NW, 7, SPLIT, 32>(P, s);
    default: return launch_smfmac_decode_staged<T, NW, 8, SPLIT, 32>(P, s);
    }
}

// ------------------------------------------------------------------------------ fragpack
struct FragpackParams {
    const void *pk_val;   // rowpack values [G, nb, n]
    const void *pk_pat;   // rowpack patterns [G, nb]
    const int8_t *order;
    void *fp_val;
    uint32_t *fp_idx;
    int64_t G, S, nb;
    int n, m, pat_bytes, MB, KP;
};

// One thread per (feature block, k pair, lane): emits its 2 x 8 values and one index word.
template <typename T> __global__ void fragpack_kernel(FragpackParams P)
{
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = (int64_t)P.MB * P.KP * 64;
    if (gid >= total) return;
    const int lane = (int)(gid & 63);
    const int64_t rest = gid >> 6;
    const int kp = (int)(rest % P.KP);
    const int mb = (int)(rest / P.KP);
    const int64_t row = (int64_t)mb * 32 + (lane & 31);
    const int ga = lane >> 5;
    const T *pkv = (const T *)P.pk_val;
    uint32_t idxword = 0;
    for (int ks = 0; ks < 2; ks++) {
        uint16_t vals[8];
        uint32_t half = 0;
        for (int q = 0; q < 4; q++) {
            const int kg = 4 * (q >> 1) + 2 * ga + (q & 1);
            const int64_t k4 = ((int64_t)kp * 2 + ks) * 32 + kg * 4;
            int pos[2] = {0, 1};
            uint16_t v[2] = {0, 0};
            int cnt = 0;
            if (row < P.G) {
                for (int i = 0; i < 4 && cnt < 2; i++) {
                    const int64_t k = k4 + i;
                    if (k >= P.S) break;
                    const int64_t b = k / P.m;
                    const int r = (int)(k - b * P.m);
                    const int p = (P.pat_bytes == 1) ? (int)((const uint8_t *)P.pk_pat)[row * P.nb + b]
                                                     : (int)((const uint16_t *)P.pk_pat)[row * P.nb + b];
                    for (int j = 0; j < P.n; j++)
                        if (P.order[p * P.n + j] == r) {
                            T x = pkv[(row * P.nb + b) * P.n + j];
                            pos[cnt] = i;
                            v[cnt] = *reinterpret_cast<uint16_t *>(&x);
                            cnt++;
                            break;
                        }
                }
            }
            if (cnt == 0) {
                pos[0] = 0;
                pos[1] = 1;
            } else if (cnt == 1) {
                // add a zero at an unused position, keeping positions increasing
                if (pos[0] == 3) {
                    pos[1] = 3;
                    v[1] = v[0];
                    pos[0] = 0;
                    v[0] = 0;
                } else {
                    pos[1] = 3;
                    v[1] = 0;
                }
            }
            vals[2 * q] = v[0];
            vals[2 * q + 1] = v[1];
            half |= (uint32_t)(pos[0] | (pos[1] << 2)) << (4 * q);
        }
        idxword |= half << (16 * ks);
        uint16_t *dst = (uint16_t *)P.fp_val + (((int64_t)mb * (P.KP * 2) + kp * 2 + ks) * 64 + lane) * 8;
        for (int e = 0; e < 8; e++) dst[e] = vals[e];
    }
    P.fp_idx[((int64_t)mb * P.KP + kp) * 64 + lane] = idxword;
}

// Every aligned group of 4 positions inside an m-block must keep <= 2 values.
static bool pattern_fits_2of4(int n, int m)
{
    if (!(m % 4 == 0 || 4 % m == 0)) return false;
    const int8_t *ord = host_order(n, m);
    if (!ord) return false;
    const int64_t c = binom(m, n);
    if (m < 4) return n * (4 / m) <= 2;
    for (int64_t p = 0; p < c; p++) {
        int cnt[16] = {0};
        for (int j = 0; j < n; j++) {
            int grp = ord[p * n + j] / 4;
            if (++cnt[grp] > 2) return false;
        }
    }
    return true;
}

}  // namespace nmg

using namespace nmg;

extern "C" int nmg_fragpack_supported(int n, int m) { return pattern_fits_2of4(n, m) ? 1 : 0; }

extern "C" int nmg_fragpack_sizes(int64_t G, int64_t S, int64_t *val_elems, int64_t *idx_words)
{
    NMG_REQUIRE(G >= 0 && S >= 0 && val_elems && idx_words, NMG_ERR_ARG, "bad fragpack size query");
    const int64_t MB = (G + 255) / 256 * 8, KP = (S + 63) / 64;  // whole 256-line workgroup tiles
    *val_elems = MB * KP * 2 * 64 * 8;
    *idx_words = MB * KP * 64;
    return NMG_OK;
}

extern "C" int nmg_fragpack(const void *d_pk_val, const void *d_pk_pat, int64_t G, int64_t S,
                            void *d_fp_val, void *d_fp_idx, int n, int m, int dtype, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED,
                "the sparse matrix cores take f16/bf16 only");
    NMG_REQUIRE(m >= 1 && m <= 64 && n >= 0 && n <= m, NMG_ERR_ARG, "invalid n:m = %d:%d", n, m);
    NMG_REQUIRE(pattern_fits_2of4(n, m), NMG_ERR_UNSUPPORTED,
                "%d:%d patterns do not fit 2-of-4 groups", n, m);
    if (G == 0 || S == 0) return NMG_OK;
    NMG_REQUIRE(d_pk_val && d_pk_pat && d_fp_val && d_fp_idx, NMG_ERR_ARG, "null device pointer");
    FragpackParams P{};
    P.pk_val = d_pk_val;
    P.pk_pat = d_pk_pat;
    if (int rc = device_order(n, m, &P.order)) return rc;
    P.fp_val = d_fp_val;
    P.fp_idx = (uint32_t *)d_fp_idx;
    P.G = G;
    P.S = S;
    P.nb = (S + m - 1) / m;
    P.n = n;
    P.m = m;
    P.pat_bytes = (int)nmg_rowpack_pat_bytes(n, m);
    P.MB = (int)((G + 255) / 256 * 8);
    P.KP = (int)((S + 63) / 64);
    const int64_t total = (int64_t)P.MB * P.KP * 64;
    const int bs = 256;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NMG_F16)
        hipLaunchKernelGGL(fragpack_kernel<__half>, dim3((unsigned)((total + bs - 1) / bs)), dim3(bs), 0, s, P);
    else
        hipLaunchKernelGGL(fragpack_kernel<__hip_bfloat16>, dim3((unsigned)((total + bs - 1) / bs)), dim3(bs), 0, s, P);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

template <typename T, int WM, int WN, int FB, int TB, int MINW>
static int launch_smfmac_cfg(SmfParams &P, hipStream_t s)
{
    constexpr int BMf = WM * FB * 32, BNt = WN * TB * 32;
    P.tiles_m = (int)((P.M + BMf - 1) / BMf);
    P.tiles_n = (int)((P.T + BNt - 1) / BNt);
    dim3 grid((unsigned)(P.tiles_m * P.tiles_n));
    const size_t lds = (size_t)2 * BNt * SMF_ROW;
    const bool guard = (P.K % 64) != 0;
    auto k = guard ? spmm_smfmac_kernel<T, WM, WN, FB, TB, MINW, true>
                   : spmm_smfmac_kernel<T, WM, WN, FB, TB, MINW, false>;
    if (lds > 64 * 1024)
        NMG_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(k, grid, dim3(64 * WM * WN), lds, s, P);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

template <typename T> static int launch_smfmac(SmfParams &P, int variant, hipStream_t s)
{
    if (variant < 0) {
        // Large-batch default.  The 256 x 256 tile moves a quarter fewer bytes per flop through the
        // vector caches and is 2-4 % faster per flop in steady state (16384 x 4096 x 4096 tokens:
        // 267 against 273 us; 8192^2 x 4096, 2:8: 250 against 260); what decides is how the tiles
        // fill the chip: rounds of 256 tiles, a 256 x 256 tile taking twice the time of a 256 x 128
        // one (both are one workgroup per CU: 260 and 448 registers per lane).
        const int64_t tm = (P.M + 255) / 256, t256 = tm * ((P.T + 255) / 256), t128 = tm * ((P.T + 127) / 128);
        const double cost128 = (double)((t128 + 255) / 256), cost256 = (double)((t256 + 255) / 256) * 2.0 / 1.025;
        variant = (P.ksplit <= 1 && cost256 < cost128) ? 8 : 6;
    }
    switch (variant) {
    case 0: return launch_smfmac_cfg<T, 2, 2, 4, 2, 1>(P, s);  // register-prefetch kernel, 256 lines x 128 tokens: any K
    case 5:                                                     // decode shapes, T <= 16 (staged form: <= 32)
        if (P.T > 32 || (P.T > 16 && !(P.K % 128 == 0 && P.T * P.ldx * 2 < ((int64_t)1 << 31))))
            return launch_smfmac_cfg<T, 2, 2, 4, 2, 1>(P, s);
        // few line blocks: many wavefronts per workgroup keep enough loads in flight per CU;
        // many line blocks: small workgroups pack several per CU and balance better
        // reduction extents that are a multiple of 128: activations staged through LDS
        if (P.K % 128 == 0 && P.T * P.ldx * 2 < ((int64_t)1 << 31)) {
            // Weights that are not in a cache, 4096 x 11008 (128 blocks), 1 / 16 tokens: one
            // workgroup of 16 wavefronts per block 13.2 / 18.4 us, two of 8 wavefronts 12.1 / 15.5,
            // two of 16 12.2 / 16.7, four of 4 16.2 / 22.9 (runs of 128 bytes).  11008 x 4096
            // (344 blocks): one of 4 wavefronts 11.6 / 14.0, two of 4 12.1 / 16.2.
            const int64_t blocks = (P.M + 31) / 32;
            if (blocks >= 256) return launch_smfmac_decode_staged_nd<T, 4, 1>(P, s);
            if (blocks >= 64 || P.T > 16) return launch_smfmac_decode_staged_nd<T, 8, 2>(P, s);   // (32 token rows: 16 wavefronts would not fit LDS)
            return launch_smfmac_decode_staged_nd<T, 16, 2>(P, s);
        }
        if ((P.M + 31) / 32 >= 256) return launch_smfmac_skinny<T, 4, 4>(P, s);
        return launch_smfmac_skinny<T, 16, 1>(P, s);
    case 6:                                                     // 256 x 128, weights straight to registers
    case 8:                                                     // 256 x 256
        if (P.K % 64 != 0 || P.T * P.ldx * 2 >= (int64_t)1 << 31)
            return launch_smfmac_cfg<T, 2, 2, 4, 2, 1>(P, s);
        if (variant == 8) return launch_smfmac_direct<T, 2, 8, 4, 1, 4>(P, s);
        return launch_smfmac_direct<T, 2, 4, 4, 1, 2>(P, s);
    }
    return NMG_ERR_ARG;
}

extern "C" int nmg_spmm_smfmac(const void *d_fp_val, const void *d_fp_idx, int64_t M, int64_t K,
                               const void *d_x, int64_t ldx, void *d_y, int64_t ldy,
                               const void *d_bias, int64_t T, int dtype, int variant, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED,
                "the sparse matrix cores take f16/bf16 only");
    NMG_REQUIRE(M >= 0 && K >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(variant == -1 || variant == 0 || variant == 5 || variant == 6 || variant == 8, NMG_ERR_ARG,
                "unknown tile variant %d", variant);
    NMG_REQUIRE(ldx >= K && ldy >= M, NMG_ERR_ARG, "leading dimension smaller than row length");
    NMG_REQUIRE((K % 8) == 0 && (ldx % 8) == 0 && ((uintptr_t)d_x % 16) == 0, NMG_ERR_UNSUPPORTED,
                "activations must be 16-byte aligned with K and ldx multiples of 8");
    if (M == 0 || K == 0 || T == 0) return NMG_OK;
    NMG_REQUIRE(d_fp_val && d_fp_idx && d_x && d_y, NMG_ERR_ARG, "null device pointer");
    SmfParams P{};
    P.fp_val = d_fp_val;
    P.fp_idx = (const uint32_t *)d_fp_idx;
    P.x = d_x;
    P.y = d_y;
    P.bias = d_bias;
    P.M = M;
    P.K = K;
    P.T = T;
    P.ldx = ldx;
    P.ldy = ldy;
    P.MB = (int)((M + 255) / 256 * 8);
    P.KP = (int)((K + 63) / 64);
    hipStream_t s = (hipStream_t)stream;
    return dtype == NMG_F16 ? launch_smfmac<__half>(P, variant, s)
                            : launch_smfmac<__hip_bfloat16>(P, variant, s);
}


extern "C" int nmg_splitk_plan(int64_t M, int64_t K, int64_t T, int *slices,
                                           int64_t *workspace_bytes)
{
    NMG_REQUIRE(M >= 0 && K >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(slices && workspace_bytes, NMG_ERR_ARG, "null output pointer");
    const int64_t tiles_m = (M + 255) / 256, tiles = tiles_m * ((T + 127) / 128), KP = (K + 63) / 64;
    int S = 1;
    // Between the decode shapes and a batch that fills the chip a product has fewer tiles of
    // 256 x 128 than the GPU has CUs, and every workgroup walks the whole reduction: the slices
    // bring the workgroups towards one per CU, at eight K steps or more each and at most eight
    // slices (sixteen for a handful of tiles): every slice writes and the sum reads a tile in
    // single precision.  4096 x 11008 2:4 on 17 / 64 / 128 / 256 / 512 / 1024 tokens: 58 / 58 / 64 /
    // 65 / 72 / 94 us whole, 20 / 20 / 25 / 33 / 42 / 67 us in 8 / 8 / 8 / 8 / 4 / 2 slices (16 slices
    // at 64 tokens: 22 us).
    if (T > 16 && K % 64 == 0 && tiles > 0 && tiles <= 128)
        S = splitk_fit(KP, std::min<int64_t>(std::min<int64_t>(256 / tiles, tiles <= 8 ? 16 : 8), KP / 8));
    *slices = S;
    *workspace_bytes = S > 1 ? (int64_t)S * T * tiles_m * 256 * 4 : 0;
    return NMG_OK;
}

extern "C" int nmg_spmm_smfmac_splitk(const void *d_fp_val, const void *d_fp_idx, int64_t M, int64_t K,
                                      const void *d_x, int64_t ldx, void *d_y, int64_t ldy,
                                      const void *d_bias, int64_t T, int dtype, int slices,
                                      void *d_workspace, int64_t workspace_bytes, void *stream)
{
    if (slices <= 1)
        return nmg_spmm_smfmac(d_fp_val, d_fp_idx, M, K, d_x, ldx, d_y, ldy, d_bias, T, dtype, -1, stream);
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED,
                "the sparse matrix cores take f16/bf16 only");
    NMG_REQUIRE(M >= 0 && K >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(ldx >= K && ldy >= M, NMG_ERR_ARG, "leading dimension smaller than row length");
    NMG_REQUIRE((K % 64) == 0 && (ldx % 8) == 0 && ((uintptr_t)d_x % 16) == 0, NMG_ERR_UNSUPPORTED,
                "a split reduction needs K % 64 == 0 and 16-byte aligned activations");
    NMG_REQUIRE(T > 16 && T * ldx * 2 < ((int64_t)1 << 31), NMG_ERR_UNSUPPORTED,
                "a split reduction takes more than 16 tokens and activations below 2 GiB");
    if (M == 0 || K == 0) return NMG_OK;
    const int64_t KP = K / 64, tiles_m = (M + 255) / 256;
    NMG_REQUIRE(slices <= 256 && splitk_fit(KP, slices) == slices, NMG_ERR_ARG,
                "%d slices leave one empty (%lld K steps)", slices, (long long)KP);
    const int64_t need = (int64_t)slices * T * tiles_m * 256 * 4;
    NMG_REQUIRE(d_workspace && workspace_bytes >= need && ((uintptr_t)d_workspace % 16) == 0, NMG_ERR_ARG,
                "workspace of %lld bytes (16-byte aligned) needed, %lld given", (long long)need,
                (long long)workspace_bytes);
    NMG_REQUIRE(d_fp_val && d_fp_idx && d_x && d_y, NMG_ERR_ARG, "null device pointer");
    SmfParams P{};
    P.fp_val = d_fp_val;
    P.fp_idx = (const uint32_t *)d_fp_idx;
    P.x = d_x;
    P.y = d_y;
    P.bias = d_bias;
    P.M = M;
    P.K = K;
    P.T = T;
    P.ldx = ldx;
    P.ldy = ldy;
    P.MB = (int)(tiles_m * 8);
    P.KP = (int)KP;
    P.ksplit = slices;
    P.part = (float *)d_workspace;
    P.part_ld = tiles_m * 256;
    hipStream_t s = (hipStream_t)stream;
    return dtype == NMG_F16 ? launch_smfmac_direct<__half, 2, 4, 4, 1, 2>(P, s)
                            : launch_smfmac_direct<__hip_bfloat16, 2, 4, 4, 1, 2>(P, s);
}

// ---- both dense operands transposed: C[M, T] = W * B (+ bias per row), B [K, T] ------------------
extern "C" int nmg_spmm_smfmac_tt(const void *d_fp_val, const void *d_fp_idx, int64_t M, int64_t K,
                                  const void *d_b, int64_t ldb, void *d_c, int64_t ldc, const void *d_bias,
                                  int64_t T, int dtype, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED,
                "the sparse matrix cores take f16/bf16 only");
    NMG_REQUIRE(M >= 0 && K >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(ldb >= T && ldc >= T, NMG_ERR_ARG, "leading dimension smaller than row length");
    NMG_REQUIRE((K % 64) == 0 && K > 0 && (ldb % 8) == 0 && ((uintptr_t)d_b % 16) == 0, NMG_ERR_UNSUPPORTED,
                "the transposed product needs K %% 64 == 0, ldb %% 8 == 0 and a 16-byte aligned B");
    NMG_REQUIRE(ldb < ((int64_t)1 << 24), NMG_ERR_UNSUPPORTED, "leading dimension too large");
    if (M == 0 || T == 0) return NMG_OK;
    NMG_REQUIRE(d_fp_val && d_fp_idx && d_b && d_c, NMG_ERR_ARG, "null device pointer");
    SmfParams P{};
    P.fp_val = d_fp_val;
    P.fp_idx = (const uint32_t *)d_fp_idx;
    P.x = d_b;
    P.y = d_c;
    P.bias = d_bias;
    P.M = M;
    P.K = K;
    P.T = T;
    P.ldx = ldb;
    P.ldy = ldc;
    P.MB = (int)((M + 255) / 256 * 8);
    P.KP = (int)(K / 64);
    hipStream_t s = (hipStream_t)stream;
    return dtype == NMG_F16 ? launch_smfmac_direct<__half, 2, 4, 4, 1, 2, true>(P, s)
                            : launch_smfmac_direct<__hip_bfloat16, 2, 4, 4, 1, 2, true>(P, s);
}

// ---- the split reduction for callers that cannot allocate -----------------------------------
// Same kernels as nmg_spmm_smfmac_splitk; the single-precision partial sums of the slices go to a
// file-scope array of this library instead of a workspace the caller brings.  Each GPU holds its
// own copy of the array (until the process ends) at its own address, looked up once per device.
// Every call on a GPU uses that GPU's array: calls that overlap on one GPU (two streams) race.
// Nothing in it has to start at zero -- a call reads only what its own slices wrote -- so it is
// never cleared, and a call may follow a larger one.
namespace nmg {
constexpr int64_t kSplitkScratchBytes = (int64_t)32 << 20;
static __device__ __align__(256) unsigned char g_splitk_scratch[kSplitkScratchBytes];
static std::mutex g_scratch_mu;
static std::map<int, void *> g_scratch_ptr;   // device -> address of its copy

static int splitk_scratch(void **ptr)
{
    int dev = 0;
    NMG_HIP_TRY(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    auto it = g_scratch_ptr.find(dev);
    if (it == g_scratch_ptr.end()) {
        void *p = nullptr;
        NMG_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(g_splitk_scratch)));
        it = g_scratch_ptr.emplace(dev, p).first;
    }
    *ptr = it->second;
    return NMG_OK;
}
}  // namespace nmg

extern "C" int64_t nmg_noalloc_scratch_bytes(void) { return kSplitkScratchBytes; }

extern "C" int nmg_noalloc_prepare(void)
{
    void *p = nullptr;
    return splitk_scratch(&p);
}

extern "C" int nmg_spmm_smfmac_splitk_noalloc(const void *d_fp_val, const void *d_fp_idx, int64_t M, int64_t K,
                                              const void *d_x, int64_t ldx, void *d_y, int64_t ldy,
                                              const void *d_bias, int64_t T, int dtype, int slices, void *stream)
{
    NMG_REQUIRE(M >= 0 && K >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    if (slices > 1) {
        const int64_t tiles_m = (M + 255) / 256;
        const int64_t need = (int64_t)slices * T * tiles_m * 256 * 4;
        NMG_REQUIRE(need <= kSplitkScratchBytes, NMG_ERR_UNSUPPORTED,
                    "%d slices of %lld tokens x %lld features need %lld bytes of partial sums; the built-in "
                    "scratch holds %lld (use nmg_spmm_smfmac_splitk with a workspace of your own)",
                    slices, (long long)T, (long long)(tiles_m * 256), (long long)need,
                    (long long)kSplitkScratchBytes);
    }
    void *ws = nullptr;
    if (int rc = splitk_scratch(&ws)) return rc;
    return nmg_spmm_smfmac_splitk(d_fp_val, d_fp_idx, M, K, d_x, ldx, d_y, ldy, d_bias, T, dtype, slices, ws,
                                  kSplitkScratchBytes, stream);
}

