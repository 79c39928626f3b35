// nmg x dense matmul on the dense matrix cores (V_MFMA_F32_16X16X32_{F16,BF16}) with the weight
// expanded beforehand into the register order of the matrix instructions ("densefrag" operand).
//
// Serves what the sparse matrix cores cannot: patterns that do not fit 2-of-4 groups (4:8,
// 3:4, ...) and the reduction along the *group* dim, i.e. the gradient with respect to the
// activations of a weight that is n:m along its own reduction dim:
//
//   transpose = 0:  Y[tok, q] = sum_s X[tok, s] * W2[q, s]      (q = line, s = sparse position)
//   transpose = 1:  Y[tok, s] = sum_q X[tok, q] * W2[q, s]
//
// Two kernels:
//   densefrag_kernel       rowpack -> densefrag, through an LDS tile (reads and writes contiguous);
//   dense16_direct_kernel  the multiplication, same skeleton as the direct-weights kernel of the
//                          sparse matrix cores: 4 wavefronts stacked on the output dim, weight
//                          fragments global -> registers DD_D K steps ahead, activation tile
//                          global -> LDS by DMA, one barrier per K step of 64.
//
// densefrag [OB][K16][64 lanes][8]: for output block ob (32 outputs) and k-step k16 (16 reduction
// positions), lane l holds the 8 weights of output ob*32 + l%32 at reduction positions
// k16*16 + 8*(l/32) + 0..7 -- the A operand of V_MFMA_F32_32X32X16, which the first form of the
// multiplication used; the 16 x 16 x 32 instruction finds its fragments in it with another lane
// offset (below).  OB is padded to a multiple of 8 (256 outputs), the reduction extent must be a
// multiple of 64; padding is zero.
#include "nmg_common.h"
#include "nmg_tile.h"

#include <type_traits>

namespace nmg {

typedef _Float16 df_f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 df_bf16x8 __attribute__((ext_vector_type(8)));

// ------------------------------------------------------------------ rowpack -> densefrag
constexpr int DFX_L = 64, DFX_P = 128;   // LDS tile: lines x positions (at most; a tile holds whole blocks)

struct DfExpandParams {
    const void *pk_val;
    const void *pk_pat;
    void *df;
    const int8_t *order;
    int64_t G, S, nb;
    int64_t OB, K16;                      // blocks of the operand
    int n, m, pat_bytes, bpt, transpose;  // bpt = blocks of m positions per tile
    int pt;                               // positions per tile: bpt * m, a multiple of 32, at most 128
    int order_bytes;                      // size of the order table (specialised kernels: it fits 2 KiB)
};

// NV = n where the kernel is specialised for it (1, 2, 4: the n values of a block are one load, the
// order table sits in LDS, and a thread has the loads of four blocks in flight before it scatters
// the first -- pattern -> order entry -> value is otherwise a chain of round trips per block),
// 0 = any n.
template <typename T, int NV> __global__ __launch_bounds__(256) void densefrag_kernel(DfExpandParams P)
{
    // transpose = 0: tile[line][position], outputs = lines;  transpose = 1: tile[position][line],
    // outputs = positions.  Rows are outputs, columns the reduction; +8 elements of padding keep
    // rows 16-byte aligned and spread the banks.
    constexpr int PAD = 8;
    __shared__ __align__(16) uint16_t tile[DFX_L * (DFX_P + PAD) > DFX_P * (DFX_L + PAD) ? DFX_L * (DFX_P + PAD)
                                                                                        : DFX_P * (DFX_L + PAD)];
    static_assert(sizeof(T) == 2, "16-bit data");
    const int tid = threadIdx.x;
    const int64_t q0 = (int64_t)blockIdx.y * DFX_L, b0 = (int64_t)blockIdx.x * P.bpt;
    const int rows = P.transpose ? P.pt : DFX_L, cols = P.transpose ? DFX_L : P.pt;
    const int pitch = cols + PAD;
    {
        uint4 z = {0, 0, 0, 0};
        for (int i = tid; i < rows * pitch / 8; i += 256) ((uint4 *)tile)[i] = z;
    }
    __syncthreads();
    const uint16_t *pv = (const uint16_t *)P.pk_val;
    if constexpr (NV > 0) {
        __shared__ int8_t s_ord[2048];
        for (int i = tid; i < P.order_bytes; i += 256) s_ord[i] = P.order[i];
        __syncthreads();
        const int items = DFX_L * P.bpt;
        for (int base = tid; base < items; base += 4 * 256) {
            int pat[4];
            uint16_t v[4][NV];
            bool live[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int i = base + u * 256;
                const int ql = i / P.bpt, bl = i - ql * P.bpt;
                const int64_t q = q0 + ql, b = b0 + bl;
                live[u] = i < items && q < P.G && b < P.nb;
                const int64_t blk = live[u] ? q * P.nb + b : 0;
                pat[u] = P.pat_bytes == 1 ? (int)((const uint8_t *)P.pk_pat)[blk]
                                          : (int)((const uint16_t *)P.pk_pat)[blk];
                if constexpr (NV == 1) {
                    v[u][0] = pv[blk];
                } else if constexpr (NV == 2) {
                    const uint32_t w = ((const uint32_t *)pv)[blk];
                    v[u][0] = (uint16_t)w;
                    v[u][1] = (uint16_t)(w >> 16);
                } else {
                    const uint2 w = ((const uint2 *)pv)[blk];
                    v[u][0] = (uint16_t)w.x;
                    v[u][1] = (uint16_t)(w.x >> 16);
                    v[u][2] = (uint16_t)w.y;
                    v[u][3] = (uint16_t)(w.y >> 16);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (!live[u]) continue;
                const int i = base + u * 256;
                const int ql = i / P.bpt, bl = i - ql * P.bpt;
                const int8_t *ord = s_ord + pat[u] * NV;
#pragma unroll
                for (int j = 0; j < NV; j++) {
                    const int pos = bl * P.m + ord[j];
                    if (P.transpose)
                        tile[pos * pitch + ql] = v[u][j];
                    else
                        tile[ql * pitch + pos] = v[u][j];
                }
            }
        }
    } else {
        for (int i = tid; i < DFX_L * P.bpt; i += 256) {
            const int ql = i / P.bpt, bl = i - ql * P.bpt;
            const int64_t q = q0 + ql, b = b0 + bl;
            if (q >= P.G || b >= P.nb) continue;
            const int64_t blk = q * P.nb + b;
            const int pat = P.pat_bytes == 1 ? (int)((const uint8_t *)P.pk_pat)[blk]
                                             : (int)((const uint16_t *)P.pk_pat)[blk];
            const int8_t *ord = P.order + pat * P.n;
            for (int j = 0; j < P.n; j++) {
                const int pos = bl * P.m + ord[j];
                const uint16_t v = pv[blk * P.n + j];
                if (P.transpose)
                    tile[pos * pitch + ql] = v;
                else
                    tile[ql * pitch + pos] = v;
            }
        }
    }
    __syncthreads();
    // tile -> fragments: (rows/32) x (cols/16) fragments of 64 lanes x 16 B
    const int64_t ob0 = (P.transpose ? b0 * P.m : q0) / 32, k0 = (P.transpose ? q0 : b0 * P.m) / 16;
    const int nfk = cols / 16, nfrag = (rows / 32) * nfk;
    uint4 *df = (uint4 *)P.df;
    for (int i = tid; i < nfrag * 64; i += 256) {
        const int f = i >> 6, l = i & 63;
        const int fo = f / nfk, fk = f - fo * nfk;
        const int64_t ob = ob0 + fo, k16 = k0 + fk;
        if (ob >= P.OB || k16 >= P.K16) continue;
        const uint4 v = *(const uint4 *)(tile + (fo * 32 + (l & 31)) * pitch + fk * 16 + 8 * (l >> 5));
        df[(ob * P.K16 + k16) * 64 + l] = v;
    }
}

// ----------------------------------------------------------------------------- the matmul
struct DfParams {
    const void *df;
    const void *x;
    void *y;
    const void *bias;
    int64_t O, K, T, ldx, ldy;
    int KP;              // K steps of 64
    int tiles_m, tiles_n;
    // reduction cut into slices (0 / 1: whole): slice s of a tile stores its sums in single
    // precision at part[s][token][output], part_ld outputs per token
    int ksplit;
    float *part;
    int64_t part_ld;
};

constexpr int DD_D = 2;    // K steps in flight (a dense K step takes twice the MFMA time of a sparse one)
constexpr int DD_NS = 4;   // activation stages in LDS (>= DD_D + 1)

// V_MFMA_F32_16X16X32: of the two dense forms of the instruction the one that draws less power
// per flop (from registers, random operands: 1.76-1.97 against 1.61-1.71 PFLOP/s for 32 x 32 x 16),
// and with this skeleton around it the difference stays: the first form of this kernel, on
// 32 x 32 x 16, reached matrix-pipe utilisation 0.90 and was 9-15 % slower.
//   A fragment (16 outputs x 32 k): lane (r = l%16, kq = l/16) wants the 8 weights of output
//     16*ab + r at k = 32*k32 + 8*kq + 0..7, which the densefrag operand stores in fragment
//     (ob = ab/2, k16 = 2*k32 + kq/2) at lane 32*(kq%2) + 16*(ab%2) + r: a load still covers four
//     runs of 256 contiguous bytes.
//   B fragment (16 tokens x 32 k): lane (j = l%16, kq) reads the 16-byte chunk 4*k32 + kq of token
//     row 16*tb + j; with the chunks XOR-swizzled by (row/2)%8 sixteen consecutive rows cover all
//     banks.
//   D: lane holds token l%16, outputs 4*(l/16) + 0..3 of the 16 x 16 block.
// A wavefront owns 64 outputs x TB*16 tokens: 4 x TB accumulator blocks of 4 registers, all of
// them in the accumulation registers.  A K step of 64 is two k-steps of 32; a phase is one
// (k-step, token part) pair of 4 * TB / NH MFMAs: they run while the activation fragments of the
// next phase are read from LDS, and the loads of K step kp+DD_D are dealt out over the phases.
// XT = true is the product with both dense operands transposed, C[O, T] = A * B for B [K, T] (the
// gradient with respect to B of torch.mm(W, B): W^T * grad_out as they lie in memory): the
// activation tile of a K step is then 64 reduction rows x TT tokens, fetched as it lies, an
// activation fragment is two LDS transpose reads (DS_READ_B64_TR_B16), and the epilogue stages
// [output][token] and stores token-contiguous rows.
template <typename T> struct DfMma16;
template <> struct DfMma16<__half> {
    using F = df_f16x8;
    __device__ static f32x4 run(F a, F b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};
template <> struct DfMma16<__hip_bfloat16> {
    using F = df_bf16x8;
    __device__ static f32x4 run(F a, F b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};

template <typename T, int TB, int NH, bool XT = false>
__global__ __launch_bounds__(256, 1) void dense16_direct_kernel(DfParams P)
{
    using Mm = DfMma16<T>;
    constexpr int AB = 4;                                 // blocks of 16 outputs per wavefront
    constexpr int TF = 256, TT = TB * 16;                 // workgroup tile: outputs x tokens
    constexpr int STAGE = TT * 128;                       // activation bytes per K step
    constexpr int XL = TT / 32;                           // DMA loads per wavefront per K step
    constexpr int OPS = XL + 2 * AB;                      // memory operations per wavefront per K step
    constexpr int BT = TB / NH;                           // token blocks per phase
    constexpr int NP = 2 * NH;                            // phases per K step
    constexpr int NM = AB * BT;                           // MFMAs per phase
    static_assert(TB % NH == 0, "token blocks split evenly into phases");
    static_assert(OPS * DD_D < 64, "vmcnt is a 6-bit counter");
    static_assert(NP >= 2 && NP % 2 == 0, "fragment sets alternate by phase across K steps");
    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // Workgroup -> tile: consecutive ids are dealt round-robin to the 8 XCDs; give each XCD a
    // contiguous run of ids and walk the grid in bands of 4 output tiles, so that a run covers
    // a compact block of tiles whose weights and activations stay in that XCD's L2.
    int id = blockIdx.x;
    const int ntiles = P.tiles_m * P.tiles_n;
    // slices of the reduction: the slices of a tile are workgroups ntiles apart
    const int slice = P.ksplit > 1 ? id / ntiles : 0;
    id -= slice * ntiles;
    if ((ntiles & 7) == 0) id = (id & 7) * (ntiles >> 3) + (id >> 3);
    constexpr int GH = 4;
    const int band = id / (GH * P.tiles_n);
    const int band_h = min(P.tiles_m - band * GH, GH);
    const int in_band = id - band * GH * P.tiles_n;
    const int tile_m = band * GH + in_band % band_h, tile_n = in_band / band_h;
    const int64_t f0 = (int64_t)tile_m * TF, t0 = (int64_t)tile_n * TT;
    // K steps kp_lo .. kp_lo + KP - 1 of the operand's KPT (the host leaves no slice empty)
    const int KPT = P.KP;
    const int kp_per = P.ksplit > 1 ? (KPT + P.ksplit - 1) / P.ksplit : KPT;
    const int kp_lo = slice * kp_per;
    const int KP = min(KPT, kp_lo + kp_per) - kp_lo;
    const int ob0 = (int)(f0 / 32) + wave * 2;

    const unsigned char *av_base[2];
#pragma unroll
    for (int o = 0; o < 2; o++)
        av_base[o] = (const unsigned char *)P.df + (((int64_t)(ob0 + o) * KPT + kp_lo) * 4) * 1024;
    const int r16 = lane & 15, kq = lane >> 4;
    const uint32_t lane_a = (uint32_t)((kq >> 1) * 1024 + ((kq & 1) * 32 + r16) * 16);
    // K step kp of the activations starts kp * XSTEP bytes into the operand
    const int64_t XSTEP = XT ? 64 * P.ldx * 2 : 128;
    const unsigned char *x_base = (const unsigned char *)P.x + (int64_t)kp_lo * XSTEP;
    uint32_t x_off[XL];
#pragma unroll
    for (int i = 0; i < XL; i++) {
        if constexpr (XT) {
            // a DMA load fills 1 KiB = 1024 / (TT * 2) reduction rows of the tile; piece p (8 tokens)
            // of row k holds the logical chunk p ^ (4*(k%4) + 2*((k/8)%2)): the 32 lanes of a
            // transpose read that are served together take rows k .. k+3 and k+8 .. k+11 of one
            // 16-token block, which then fall into 16 different pieces = every bank once
            constexpr int PPR = TT / 8;                       // 16-byte pieces per row
            const int row = (wave * XL + i) * (64 / PPR) + lane / PPR;
            const int chunk = (lane % PPR) ^ (((row & 3) << 2) | (((row >> 3) & 1) << 1));
            int64_t tok = t0 + chunk * 8;
            if (tok > P.T - 8) tok = (P.T - 1) / 8 * 8;       // clamped columns are computed, never stored
            x_off[i] = (uint32_t)((row * P.ldx + tok) * 2);
        } else {
            const int row = (wave * XL + i) * 8 + (lane >> 3);
            const int piece = lane & 7;
            const int q = piece ^ ((row >> 1) & 7);   // logical 16-byte chunk stored at this piece
            int64_t tok = t0 + row;
            if (tok >= P.T) tok = P.T - 1;            // clamped rows are computed, never stored
            x_off[i] = (uint32_t)((tok * P.ldx + q * 8) * 2);
        }
    }

    struct WSet {
        u32x4 a[AB][2];   // [block of 16 outputs][k-step of 32]
    };
    WSet ws[DD_D + 1];
    // load number i (0 .. OPS-1) of K step kp: first the XL activation DMA loads, then the 2 * AB
    // weight fragments.  Steps beyond the last repeat it: the operation count stays uniform, the
    // data is unused.
    auto issue_one = [&](int kp, WSet &w, int i) {
        if (kp >= KP) kp = KP - 1;
        if (i < XL) {
            unsigned char *base = smem + (kp & (DD_NS - 1)) * STAGE;
            const unsigned char *xb = x_base + (int64_t)kp * XSTEP;
#pragma unroll
            for (int q = 0; q < XL; q++)
                if (q == i)
                    __builtin_amdgcn_global_load_lds((glb_ptr_t)(xb + x_off[q]),
                                                     (lds_ptr_t)(base + (wave * XL + q) * 1024), 16, 0, 0);
        } else {
            // Written as instructions so that their completion is tracked by the explicit vmcnt
            // waits below and by nothing else.
#pragma unroll
            for (int ab = 0; ab < AB; ab++)
#pragma unroll
                for (int k32 = 0; k32 < 2; k32++)
                    if (XL + ab * 2 + k32 == i) {
                        const unsigned char *av = av_base[ab >> 1] + (int64_t)kp * 4096;
                        asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3"
                                     : "=v"(w.a[ab][k32])
                                     : "v"(lane_a), "s"(av), "n"(k32 * 2048 + (ab & 1) * 256)
                                     : "memory");
                    }
        }
    };

    f32x4 acc[AB][TB];
#pragma unroll
    for (int i = 0; i < AB; i++)
#pragma unroll
        for (int t = 0; t < TB; t++) acc[i][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    auto pin_acc = [&]() {
#pragma unroll
        for (int i = 0; i < AB; i++)
#pragma unroll
            for (int t = 0; t < TB; t++) asm volatile("" : "+a"(acc[i][t]));
    };
    pin_acc();

    const int sw = (r16 >> 1) & 7;
    int b_off[2];
#pragma unroll
    for (int k32 = 0; k32 < 2; k32++) b_off[k32] = r16 * 128 + (((k32 * 4 + kq) ^ sw) << 4);

    struct BFrags {
        u32x4 b[BT];
    };
    BFrags fr[2];
    // XT: lane (kq, i) of a transpose read supplies the 8 bytes at reduction row 8 kq + i/4 (+ 32 k32
    // + 4 r), tokens 4 (i%4) .. +3 of the 16-token block, and receives token i at rows
    // 8 kq + 4 r + 0..3: reads r = 0, 1 are the lane's 8 reduction positions.
    int t_off[XT ? TB : 1];
    if constexpr (XT) {
        const int a = r16 >> 2;
#pragma unroll
        for (int tb = 0; tb < TB; tb++) {
            const int chunk = tb * 2 + ((r16 & 3) >> 1);   // 8-token chunk of the row
            t_off[tb] = (8 * kq + a) * (TT * 2) + ((chunk ^ ((a << 2) | ((kq & 1) << 1))) << 4) + (r16 & 1) * 8;
        }
    }
    auto read_one = [&](BFrags &f, const unsigned char *base, int ph, int t) {
        const int k32 = ph / NH, hh = ph % NH;
        if constexpr (XT) {
            typedef short i16x4 __attribute__((ext_vector_type(4)));
            typedef __attribute__((address_space(3))) i16x4 *lds_i16x4;
            union {
                i16x4 h[2];
                u32x4 u;
            } c;
#pragma unroll
            for (int r = 0; r < 2; r++)
                c.h[r] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_i16x4)(base + t_off[hh * BT + t] + (32 * k32 + 4 * r) * (TT * 2)));
            f.b[t] = c.u;
        } else {
            f.b[t] = *(const u32x4 *)(base + b_off[k32] + (hh * BT + t) * 16 * 128);
        }
    };
    // MFMA number i of phase PH (i = ab * BT + t)
    auto mma = [&](const WSet &w, const BFrags &f, auto ph_tag, int i) {
        constexpr int PH = decltype(ph_tag)::value, K32 = PH / NH, HH = PH % NH;
        const int ab = i / BT, t = i % BT;
        union {
            u32x4 u;
            typename Mm::F v;
        } ca, cb;
        ca.u = w.a[ab][K32];
        cb.u = f.b[t];
        acc[ab][HH * BT + t] = Mm::run(ca.v, cb.v, acc[ab][HH * BT + t]);
    };

    // The counted wait.  Invariants it rests on:
    //  (1) a wavefront's vector memory operations complete in issue order, and it issues exactly
    //      OPS of them per K step (XL DMA loads, then 2 * AB weight fragments), all of step
    //      kp+DD_D before the wait in the last phase of step kp; so at that wait the newest
    //      (DD_D-1) * OPS operations are the steps kp+2 .. kp+DD_D and everything older -- step
    //      kp+1 -- has landed once the counter is down to (DD_D-1) * OPS.  The barrier after it
    //      makes that true for the DMA loads of the other wavefronts too.
    //  (2) the weight set of step kp+1 is passed through the wait as in/out operands: whatever
    //      uses those registers afterwards is ordered after the wait by the compiler as well.
    //      (What it does with them *before* the wait is checked on the compiled code: no
    //      instruction may touch a register with a load in flight, `python -m sten_amd.isa_check`.)
    //  (3) LDS stage (kp+DD_D) % DD_NS is refilled during step kp; its last readers were the
    //      fragment reads of step kp+DD_D-DD_NS <= kp-2, complete (lgkmcnt(0), same wait) before
    //      the barrier that ended that step.  The two fragment sets alternate by phase; NP is
    //      even, so the set read after the barrier (for phase 0 of the next step) is set 0.
    static_assert(DD_NS > DD_D, "a stage must not be refilled while the step that reads it is in flight");
    auto landed = [&](WSet &w) {
        asm volatile("s_waitcnt vmcnt(%8) lgkmcnt(0)"
                     : "+v"(w.a[0][0]), "+v"(w.a[0][1]), "+v"(w.a[1][0]), "+v"(w.a[1][1]),
                       "+v"(w.a[2][0]), "+v"(w.a[2][1]), "+v"(w.a[3][0]), "+v"(w.a[3][1])
                     : "n"((DD_D - 1) * OPS)
                     : "memory");
    };

    // prologue: steps 0 .. DD_D-1 in flight, then wait for step 0
#pragma unroll
    for (int st = 0; st < DD_D; st++)
#pragma unroll
        for (int i = 0; i < OPS; i++) issue_one(st, ws[st], i);
    landed(ws[0]);
    asm volatile("s_barrier" ::: "memory");
#pragma unroll
    for (int t = 0; t < BT; t++) read_one(fr[0], smem, 0, t);

    for (int kp0 = 0; kp0 < KP; kp0 += DD_D + 1) {
#pragma unroll
        for (int u = 0; u <= DD_D; u++) {
            const int kp = kp0 + u;
            if (kp >= KP) break;
            const unsigned char *base = smem + (kp & (DD_NS - 1)) * STAGE;
            const unsigned char *next = smem + ((kp + 1) & (DD_NS - 1)) * STAGE;
            // A phase: its MFMAs, and behind one MFMA each the fragment reads of the next phase and
            // this phase's share of the loads of step kp+DD_D (dealt out over all phases but the
            // last).  The last phase waits for step kp+1 after two MFMAs, meets the other
            // wavefronts and reads the first fragments of the next stage behind the rest.
            auto phase = [&](auto ph_tag) {
                constexpr int PH = decltype(ph_tag)::value;
                if constexpr (PH == NP - 1) {
                    mma(ws[u], fr[PH % 2], ph_tag, 0);
                    mma(ws[u], fr[PH % 2], ph_tag, 1);
                    __builtin_amdgcn_sched_barrier(0);
                    landed(ws[(u + 1) % (DD_D + 1)]);
                    asm volatile("s_barrier" ::: "memory");
                    __builtin_amdgcn_sched_barrier(0);
                    constexpr int SP = (NM - 2) / BT;
#pragma unroll
                    for (int i = 2; i < NM; i++) {
                        mma(ws[u], fr[PH % 2], ph_tag, i);
                        __builtin_amdgcn_sched_barrier(0);
                        if ((i - 2) % SP == 0 && (i - 2) / SP < BT) read_one(fr[(PH + 1) % 2], next, 0, (i - 2) / SP);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
                    constexpr int L0 = PH * OPS / (NP - 1), L1 = (PH + 1) * OPS / (NP - 1);
                    constexpr int NOPS = BT + L1 - L0;
                    constexpr int SP = NM / NOPS > 0 ? NM / NOPS : 1;
                    static_assert(NOPS <= NM, "one memory instruction behind one MFMA");
#pragma unroll
                    for (int i = 0; i < NM; i++) {
                        mma(ws[u], fr[PH % 2], ph_tag, i);
                        __builtin_amdgcn_sched_barrier(0);
                        if (i % SP == 0 && i / SP < NOPS) {
                            const int op = i / SP;
                            if (op < BT)
                                read_one(fr[(PH + 1) % 2], base, PH + 1, op);
                            else
                                issue_one(kp + DD_D, ws[(u + DD_D) % (DD_D + 1)], L0 + op - BT);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            };
            phase(std::integral_constant<int, 0>{});
            phase(std::integral_constant<int, 1>{});
            if constexpr (NP >= 4) {
                phase(std::integral_constant<int, 2>{});
                phase(std::integral_constant<int, 3>{});
            }
            if constexpr (NP >= 8) {
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
    // every register of the ring passes through the final wait.
    static_assert(DD_D == 2, "the final wait lists three weight sets");
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(ws[0].a[0][0]), "+v"(ws[0].a[0][1]), "+v"(ws[0].a[1][0]), "+v"(ws[0].a[1][1]),
                   "+v"(ws[0].a[2][0]), "+v"(ws[0].a[2][1]), "+v"(ws[0].a[3][0]), "+v"(ws[0].a[3][1]),
                   "+v"(ws[1].a[0][0]), "+v"(ws[1].a[0][1]), "+v"(ws[1].a[1][0]), "+v"(ws[1].a[1][1]),
                   "+v"(ws[1].a[2][0]), "+v"(ws[1].a[2][1]), "+v"(ws[1].a[3][0]), "+v"(ws[1].a[3][1]),
                   "+v"(ws[2].a[0][0]), "+v"(ws[2].a[0][1]), "+v"(ws[2].a[1][0]), "+v"(ws[2].a[1][1]),
                   "+v"(ws[2].a[2][0]), "+v"(ws[2].a[2][1]), "+v"(ws[2].a[3][0]), "+v"(ws[2].a[3][1])
                 :
                 : "memory");
    asm volatile("s_barrier" ::: "memory");
    if (P.ksplit > 1) {
        store_partial_tile16<AB, TB>(acc, P.part + (int64_t)slice * P.T * P.part_ld, P.part_ld, lane,
                                     f0 + wave * 64, t0, P.T);
        return;
    }
    const TileOut out{P.y, P.bias, P.O, P.T, P.ldy};
    if constexpr (XT)
        store_tile16_t<T, AB, TB>(acc, smem + wave * (AB * 16 * (TT * 2 + 16)), lane, f0 + wave * 64, t0, out);
    else
        store_tile16<T, AB, TB>(acc, smem + wave * (TT * (AB * 32 + 16)), lane, f0 + wave * 64, t0, out);
}

template <typename T, int TB, int NH, bool XT = false> static int launch_dense16(DfParams &P, hipStream_t s)
{
    constexpr int TT = TB * 16;
    P.tiles_m = (int)((P.O + 255) / 256);
    P.tiles_n = (int)((P.T + TT - 1) / TT);
    const int slices = P.ksplit > 1 ? P.ksplit : 1;
    dim3 grid((unsigned)(P.tiles_m * P.tiles_n * slices));
    constexpr size_t ring = (size_t)DD_NS * TT * 128;
    constexpr size_t stg = XT ? (size_t)4 * 64 * (TT * 2 + 16) : (size_t)4 * TT * (4 * 32 + 16);
    constexpr size_t lds = ring > stg ? ring : stg;
    static_assert(lds <= 160 * 1024, "LDS");
    auto k = dense16_direct_kernel<T, TB, NH, XT>;
    NMG_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(k, grid, dim3(256), lds, s, P);
    NMG_HIP_TRY(hipGetLastError());
    if (slices > 1) {
        const SplitSum Q{P.part, P.y, P.bias, P.O, P.T, P.ldy, P.part_ld, slices};
        return launch_splitk_sum<T>(Q, s);
    }
    return NMG_OK;
}

template <typename T> static int launch_dense(DfParams &P, int variant, hipStream_t s)
{
    // Variant 0: 256 outputs x 128 tokens per workgroup, 1: 256 x 256.  The larger tile moves fewer
    // bytes per flop through the vector caches and is 5-6 % faster per flop in steady state; one
    // workgroup per CU either way, so what decides is how full the last round of tiles is.
    // (A sixteen-phase form of the 256 x 256 tile on the 32 x 32 x 16 instruction once gave wrong
    // values now and then; the forms here pass the static check of their hand-tracked loads and
    // the repeated full-chip test.)
    if (variant < 0) {
        const int64_t tm = (P.O + 255) / 256, t256 = tm * ((P.T + 255) / 256), t128 = tm * ((P.T + 127) / 128);
        const double fill256 = (double)t256 / (double)((t256 + 255) / 256 * 256);
        const double fill128 = (double)t128 / (double)((t128 + 255) / 256 * 256);
        variant = (P.ksplit <= 1 && t256 >= 256 && fill256 * 1.055 >= fill128) ? 1 : 0;
    }
    if (variant == 1) return launch_dense16<T, 16, 4>(P, s);
    return launch_dense16<T, 8, 2>(P, s);
}

}  // namespace nmg

using namespace nmg;

// positions per expansion tile: the largest multiple of lcm(m, 32) that fits 128 (0: none)
static int densefrag_tile_positions(int m)
{
    if (m < 1 || m > 64) return 0;
    int l = m;
    while (l % 32 != 0) l += m;   // lcm(m, 32)
    return l <= DFX_P ? DFX_P / l * l : 0;
}

extern "C" int nmg_densefrag_supported(int n, int m)
{
    // m a power of two, or three times one (3, 6, 12, 24, 48): a tile of whole blocks that is also
    // a whole number of 32-output blocks and 16-position k-steps
    return (n >= 0 && n <= m && densefrag_tile_positions(m) > 0) ? 1 : 0;
}

extern "C" int nmg_densefrag_elems(int64_t O, int64_t K, int64_t *elems)
{
    NMG_REQUIRE(O >= 0 && K >= 0 && elems, NMG_ERR_ARG, "invalid extents");
    NMG_REQUIRE(K % 64 == 0, NMG_ERR_UNSUPPORTED, "the reduction extent must be a multiple of 64");
    *elems = ((O + 255) / 256) * 256 * K;
    return NMG_OK;
}

extern "C" int nmg_densefrag(const void *d_pk_val, const void *d_pk_pat, int64_t G, int64_t S, int transpose,
                             void *d_df, int n, int m, int dtype, void *stream)
{
    NMG_REQUIRE(nmg_densefrag_supported(n, m), NMG_ERR_UNSUPPORTED,
                "densefrag needs m to be a power of two or three times one (at most 64), got %d:%d", n, m);
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "densefrag takes f16/bf16");
    NMG_REQUIRE(G >= 0 && S >= 0, NMG_ERR_ARG, "negative extent");
    const int64_t O = transpose ? S : G, K = transpose ? G : S;
    NMG_REQUIRE(K % 64 == 0, NMG_ERR_UNSUPPORTED, "the reduction extent (%lld) must be a multiple of 64",
                (long long)K);
    if (O == 0 || K == 0) return NMG_OK;
    NMG_REQUIRE(d_pk_val && d_pk_pat && d_df, NMG_ERR_ARG, "null device pointer");
    DfExpandParams P{};
    if (int rc = device_order(n, m, &P.order)) return rc;
    P.pk_val = d_pk_val;
    P.pk_pat = d_pk_pat;
    P.df = d_df;
    P.G = G;
    P.S = S;
    P.nb = (S + m - 1) / m;
    P.OB = (O + 255) / 256 * 8;
    P.K16 = K / 16;
    P.n = n;
    P.m = m;
    P.pat_bytes = binom(m, n) <= 256 ? 1 : 2;
    P.pt = densefrag_tile_positions(m);
    P.bpt = P.pt / m;
    P.transpose = transpose ? 1 : 0;
    // the grid covers the padded operand: outputs up to a multiple of 256
    const int64_t Gp = transpose ? G : P.OB * 32, Sp = transpose ? P.OB * 32 : S;
    const int64_t gx = (Sp + P.pt - 1) / P.pt, gy = (Gp + DFX_L - 1) / DFX_L;
    NMG_REQUIRE(gx <= 0x7fffffffLL && gy <= 65535, NMG_ERR_UNSUPPORTED, "weight too large for one launch");
    dim3 grid((unsigned)gx, (unsigned)gy);
    hipStream_t s = (hipStream_t)stream;
    // the specialised forms load the n values of a block as one word: n * 2 bytes, aligned
    const int64_t table = binom(m, n) * n;
    P.order_bytes = (int)(table <= 2048 ? table : 0);
    const int nv = (n == 1 || n == 2 || n == 4) && table <= 2048 && (uintptr_t)d_pk_val % (2 * n) == 0 ? n : 0;
    auto launch = [&](auto tag) {
        using T = decltype(tag);
        switch (nv) {
        case 1: hipLaunchKernelGGL((densefrag_kernel<T, 1>), grid, dim3(256), 0, s, P); break;
        case 2: hipLaunchKernelGGL((densefrag_kernel<T, 2>), grid, dim3(256), 0, s, P); break;
        case 4: hipLaunchKernelGGL((densefrag_kernel<T, 4>), grid, dim3(256), 0, s, P); break;
        default: hipLaunchKernelGGL((densefrag_kernel<T, 0>), grid, dim3(256), 0, s, P); break;
        }
    };
    if (dtype == NMG_F16)
        launch(__half{});
    else
        launch(__hip_bfloat16{});
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

extern "C" int nmg_spmm_densefrag(const void *d_df, int64_t O, int64_t K, const void *d_x, int64_t ldx,
                                  void *d_y, int64_t ldy, const void *d_bias, int64_t T, int dtype,
                                  int variant, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "densefrag takes f16/bf16");
    NMG_REQUIRE(O >= 0 && K >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(variant >= -1 && variant <= 1, NMG_ERR_ARG, "unknown tile variant %d", variant);
    NMG_REQUIRE(ldx >= K && ldy >= O, NMG_ERR_ARG, "leading dimension smaller than row length");
    NMG_REQUIRE(K % 64 == 0 && K > 0 && ldx % 8 == 0 && ((uintptr_t)d_x % 16) == 0, NMG_ERR_UNSUPPORTED,
                "needs K %% 64 == 0 and 16-byte aligned activation rows");
    NMG_REQUIRE(T * ldx * 2 < ((int64_t)1 << 31), NMG_ERR_UNSUPPORTED, "activations must be smaller than 2 GiB");
    if (O == 0 || T == 0) return NMG_OK;
    NMG_REQUIRE(d_df && d_x && d_y, NMG_ERR_ARG, "null device pointer");
    DfParams P{};
    P.df = d_df;
    P.x = d_x;
    P.y = d_y;
    P.bias = d_bias;
    P.O = O;
    P.K = K;
    P.T = T;
    P.ldx = ldx;
    P.ldy = ldy;
    P.KP = (int)(K / 64);
    hipStream_t s = (hipStream_t)stream;
    return dtype == NMG_F16 ? launch_dense<__half>(P, variant, s) : launch_dense<__hip_bfloat16>(P, variant, s);
}

extern "C" int nmg_spmm_densefrag_tt(const void *d_df, int64_t O, int64_t K, const void *d_b, int64_t ldb, void *d_c,
                                     int64_t ldc, const void *d_bias, int64_t T, int dtype, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "densefrag takes f16/bf16");
    NMG_REQUIRE(O >= 0 && K >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(ldb >= T && ldc >= T, NMG_ERR_ARG, "leading dimension smaller than row length");
    NMG_REQUIRE(K % 64 == 0 && K > 0 && ldb % 8 == 0 && ((uintptr_t)d_b % 16) == 0, NMG_ERR_UNSUPPORTED,
                "the transposed product needs K %% 64 == 0, ldb %% 8 == 0 and a 16-byte aligned B");
    NMG_REQUIRE(ldb < ((int64_t)1 << 24), NMG_ERR_UNSUPPORTED, "leading dimension too large");
    if (O == 0 || T == 0) return NMG_OK;
    NMG_REQUIRE(d_df && d_b && d_c, NMG_ERR_ARG, "null device pointer");
    DfParams P{};
    P.df = d_df;
    P.x = d_b;
    P.y = d_c;
    P.bias = d_bias;
    P.O = O;
    P.K = K;
    P.T = T;
    P.ldx = ldb;
    P.ldy = ldc;
    P.KP = (int)(K / 64);
    hipStream_t s = (hipStream_t)stream;
    // 256 x 128 tiles only: the fragments of this form are LDS transpose reads, 8 bytes per lane, and
    // the 256 x 256 tile, which doubles them per wavefront, measured slower (16384x4096 x 4096
    // columns: 724 against 582 us; the plain product on a transposed copy: 360 + 60 for the copy).
    return dtype == NMG_F16 ? launch_dense16<__half, 8, 2, true>(P, s) : launch_dense16<__hip_bfloat16, 8, 2, true>(P, s);
}

extern "C" int nmg_spmm_densefrag_splitk(const void *d_df, int64_t O, int64_t K, const void *d_x, int64_t ldx,
                                         void *d_y, int64_t ldy, const void *d_bias, int64_t T, int dtype,
                                         int slices, void *d_workspace, int64_t workspace_bytes, void *stream)
{
    if (slices <= 1) return nmg_spmm_densefrag(d_df, O, K, d_x, ldx, d_y, ldy, d_bias, T, dtype, -1, stream);
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "densefrag takes f16/bf16");
    NMG_REQUIRE(O >= 0 && K >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(ldx >= K && ldy >= O, NMG_ERR_ARG, "leading dimension smaller than row length");
    NMG_REQUIRE(K % 64 == 0 && K > 0 && ldx % 8 == 0 && ((uintptr_t)d_x % 16) == 0, NMG_ERR_UNSUPPORTED,
                "needs K %% 64 == 0 and 16-byte aligned activation rows");
    NMG_REQUIRE(T * ldx * 2 < ((int64_t)1 << 31), NMG_ERR_UNSUPPORTED, "activations must be smaller than 2 GiB");
    if (O == 0 || T == 0) return NMG_OK;
    const int64_t KP = K / 64, tiles_m = (O + 255) / 256;
    NMG_REQUIRE(slices <= 256 && splitk_fit(KP, slices) == slices, NMG_ERR_ARG,
                "%d slices leave one empty (%lld K steps)", slices, (long long)KP);
    const int64_t need = (int64_t)slices * T * tiles_m * 256 * 4;
    NMG_REQUIRE(d_workspace && workspace_bytes >= need && ((uintptr_t)d_workspace % 16) == 0, NMG_ERR_ARG,
                "workspace of %lld bytes (16-byte aligned) needed, %lld given", (long long)need,
                (long long)workspace_bytes);
    NMG_REQUIRE(d_df && d_x && d_y, NMG_ERR_ARG, "null device pointer");
    DfParams P{};
    P.df = d_df;
    P.x = d_x;
    P.y = d_y;
    P.bias = d_bias;
    P.O = O;
    P.K = K;
    P.T = T;
    P.ldx = ldx;
    P.ldy = ldy;
    P.KP = (int)KP;
    P.ksplit = slices;
    P.part = (float *)d_workspace;
    P.part_ld = tiles_m * 256;
    hipStream_t s = (hipStream_t)stream;
    return dtype == NMG_F16 ? launch_dense16<__half, 8, 2>(P, s) : launch_dense16<__hip_bfloat16, 8, 2>(P, s);
}
