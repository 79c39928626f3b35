// Masked weight gradient of a grouped n:m weight, written straight into the `val` layout:
//
//   val[t, s, j] = sum_tok L[tok, line(t, s)] * P[tok, pos(t, s, j)]
//
// L [T, G] holds, per token, the operand that runs along the group dim of the weight (its
// "lines"), P [T, S] the operand along the sparse dim ("positions"); for a weight W [out, in]
// that is n:m along `in`, L is the upstream gradient dY [T, out] and P the activations X [T, in].
// Only the kept positions are stored; no dense [G, S] product is ever written.
//
// Both operands have the reduction (tokens) as their slow dim, the opposite of what the matrix
// cores want (a lane holds 8 consecutive reduction positions of one row).  The transposition is
// done by the LDS transpose read of gfx950, DS_READ_B64_TR_B16: token-major tiles go global ->
// LDS by DMA (global_load_lds, 16 bytes per lane), and a fragment of V_MFMA_F32_16X16X32 is two
// such reads.  Measured lane layout of the instruction: in every group of 16 lanes, lane i
// receives as element j the 16-bit element (i % 4) of the 8 bytes addressed by lane 4j + i/4.
//
// Workgroup: 4 wavefronts, tile 256 positions x 256 lines, each wavefront 128 x 128 (8 x 8
// accumulator blocks of 16 x 16, 256 accumulator registers).  A K step is 32 tokens -- one
// reduction step of the instruction; its two operand tiles (2 x 16 KiB) are one stage of a
// 4-stage LDS ring filled 3 steps ahead.
//
// Epilogue: the four registers a lane holds of an accumulator block are four consecutive
// positions of one line -- one block of m = 4, half a block of m = 8 -- so for those patterns
// the kept values are picked in registers and stored by the lane itself.  Every other pattern
// stages the tile in LDS as [line][position] in the output type; thread = line walks the blocks
// of m positions, looks up the slot of (line, block) in the slot map (the inverse of `idx`,
// built once per pattern by nmg_slotmap), derives the pattern from the slot and writes the n
// kept values of the block to their place in `val`.
#include "nmg_common.h"
#include "nmg_tile.h"

#include <type_traits>

namespace nmg {

typedef _Float16 sd_f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 sd_bf16x8 __attribute__((ext_vector_type(8)));
typedef short sd_i16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) sd_i16x4 *sd_lds_i16x4;

// fp32 -> stored 16 bits, round to nearest even (bf16 by the conversion instruction of gfx950)
template <typename T> __device__ __forceinline__ uint16_t sd_bits16(float x);
template <> __device__ __forceinline__ uint16_t sd_bits16<__half>(float x) { return __half_as_ushort(__float2half(x)); }
template <> __device__ __forceinline__ uint16_t sd_bits16<__hip_bfloat16>(float x)
{
    const __bf16 b = (__bf16)x;
    return __builtin_bit_cast(uint16_t, b);
}

// An accumulator, read where it is used: without this the compiler copies all 256 accumulation
// registers to architectural ones at the end of the product loop, and spills to make room.
__device__ __forceinline__ float sd_from_acc(float a)
{
    float v;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
    return v;
}

// ------------------------------------------------------------------------------- slot map
// slot[b][q] (b = block of the sparse dim, q = line of the padded group dim, Gpad = chunks * c*g):
// the slot s with idx[(q / cg) * nb + b][s] == q % cg.  Every line has exactly one slot per block
// (idx of a tile is a permutation of 0 .. cg-1).
struct SlotParams {
    const int16_t *idx;
    int16_t *slot;
    int64_t entries;   // chunks * nb * cg
    int64_t nb, Gpad;
    int cg;
};

__global__ __launch_bounds__(256) void slotmap_kernel(SlotParams P)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= P.entries) return;
    const int64_t t = e / P.cg;
    const int s = (int)(e - t * P.cg);
    const int64_t kc = t / P.nb, b = t - kc * P.nb;
    const int col = P.idx[e];
    if (col < 0 || col >= P.cg) return;   // not a column of the tile (the product kernel clamps what it reads here)
    P.slot[b * P.Gpad + kc * P.cg + col] = (int16_t)s;
}

// ------------------------------------------------------------------------------ the product
struct SddmmParams {
    const void *lop;   // L [T, G]
    const void *pop;   // P [T, S]
    void *val;
    const int16_t *slot;
    const int8_t *order;
    const void *zero;  // 16 zero bytes: source of the tokens beyond T
    const void *bias;  // dense product: bias per position, or null
    int64_t ldl, ldp, G, S, T, Gpad, nb;
    int64_t ldv;       // dense product: elements between two lines of the result
    int n, m, g, cg;
    uint32_t inv_g;    // ceil(2^32 / g) for g > 1
    uint64_t ord4;     // m == 4: byte p = the kept positions of pattern p, 2 bits each
    int order_bytes;
    int KP;            // K steps of 32 tokens
    int tiles_p, tiles_l;
};

constexpr int SD_KS = 32;            // tokens per K step
constexpr int SD_NS = 4;             // stages of the ring
constexpr int SD_D = 3;              // K steps in flight
constexpr int SD_OP = SD_KS * 512;   // bytes of one operand tile: 32 tokens x 256 features
constexpr int SD_STAGE = 2 * SD_OP;
constexpr int SD_LPW = 8;            // DMA loads per wavefront per K step (32 KiB / 4 / 1 KiB)
constexpr int SD_PITCH = 520;        // staged output row: 256 positions x 2 bytes + 8
constexpr int SD_LDS = 256 * SD_PITCH + kOrderSlotBytes;
static_assert(SD_NS * SD_STAGE <= 256 * SD_PITCH, "the ring lies inside the staging area");
static_assert(SD_LDS <= 160 * 1024, "LDS of a CU");
static_assert(SD_D < SD_NS, "a stage is refilled only after the barrier that ends its last read");
static_assert(SD_D * SD_LPW < 64, "vmcnt is a 6-bit counter");

// Second half of the staged epilogue: the tile lies in LDS as [line][position] in the output type
// (SD_PITCH bytes per line), the order table behind it; thread = line walks the blocks of m
// positions that meet the tile, looks up the slot of (line, block) in the slot map, derives the
// pattern from the slot and writes the n kept values of the block to their place in val.
__device__ __forceinline__ void sd_staged_walk(const SddmmParams &P, const unsigned char *smem, int tid, int64_t l0,
                                               int64_t p0)
{
    const int8_t *s_ord = (const int8_t *)(smem + 256 * SD_PITCH);
    uint16_t *val = (uint16_t *)P.val;
    const int n = P.n, m = P.m;
    const int64_t line = l0 + tid;
    if (line >= P.Gpad) return;
    const bool line_ok = line < P.G;
    const int64_t chunk = line / P.cg;
    const unsigned char *row = smem + tid * SD_PITCH;
    const int64_t b_lo = p0 / m, b_hi = min(P.nb, (p0 + 256 + m - 1) / m);
    const int64_t pend = min(p0 + 256, P.S);
    const bool whole = (256 % m) == 0;   // blocks do not straddle tiles
    constexpr int UB = 32;               // blocks in flight: their slots are loaded together
    for (int64_t bb = b_lo; bb < b_hi; bb += UB) {
        int slot[UB];
#pragma unroll
        for (int u = 0; u < UB; u++) slot[u] = bb + u < b_hi ? (int)P.slot[(bb + u) * P.Gpad + line] : 0;
#pragma unroll 4
        for (int u = 0; u < UB; u++) {
            const int64_t b = bb + u;
            if (b >= b_hi) break;
            const int s = min(max(slot[u], 0), P.cg - 1);
            const int p = P.g > 1 ? (int)__umulhi((uint32_t)s, P.inv_g) : s;
            const int8_t *ord = s_ord + p * n;
            uint16_t *dst = val + (((chunk * P.nb + b) * P.cg + s) * (int64_t)n);
            const int64_t pb = b * m;
            if (whole && n == 2) {
                const int64_t q0 = pb + ord[0], q1 = pb + ord[1];
                const uint16_t v0 = (line_ok && q0 < pend) ? *(const uint16_t *)(row + (q0 - p0) * 2) : 0;
                const uint16_t v1 = (line_ok && q1 < pend) ? *(const uint16_t *)(row + (q1 - p0) * 2) : 0;
                *(uint32_t *)dst = (uint32_t)v0 | ((uint32_t)v1 << 16);
            } else {
                for (int j = 0; j < n; j++) {
                    const int64_t qq = pb + ord[j];
                    if (qq < p0 || qq >= p0 + 256) continue;   // that position belongs to a neighbouring tile
                    dst[j] = (line_ok && qq < pend) ? *(const uint16_t *)(row + (qq - p0) * 2) : (uint16_t)0;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------ the product
// V_MFMA_F32_16X16X32: of the two dense forms of the instruction the one that sustains more flops
// under the power limit (10-17 % more than 32 x 32 x 16), and its reduction step is the K step.
//   fragments: lane (kq = l/16, i = l%16) holds feature i of a 16-feature block at tokens
//     8 kq .. 8 kq + 7 -- two transposing reads (token-major operands) or one 16-byte read
//     (reduction-contiguous operands).  For the transposing reads the 64-byte granules of a token
//     row are XOR-swizzled with (t % 4) + 4 * ((t / 8) % 2).  (The 32 lanes served together cover
//     tokens t .. t+3 and t+8 .. t+11 of one 32-byte feature block; with this placement the two
//     token groups still meet in the same banks -- the counters show two-way conflicts -- but the
//     placement that separates them, 16-byte pieces XOR 4 * (t % 4) + 2 * ((t / 8) % 2), measured
//     conflict-free and 2.4 % slower: the LDS reads are not what the loop waits for.)
//   accumulators: 8 x 8 blocks of 16 positions x 16 lines, 4 registers each; lane (j = l%16,
//     q = l/16) holds line j and the positions 4q .. 4q+3 of the block.
//   a K step is two phases (position blocks 0..3, 4..7) of 32 MFMAs, column by column; the line
//     fragments live in one register set: column y of the second phase frees fragment y, which is
//     then read for the next step.
// MODE 1 .. 4: m == 4, n == MODE; the epilogue stays in registers: the kept values of a block are
// picked with one byte permute (per-pattern selector) and stored by the lane itself; the slots of
// the lane's 64 (line, block) pairs are fetched when the kernel starts and wait in registers.
// MODE 8 + n (n = 1, 2, 4): m == 8; the two lanes that hold the halves of a block exchange them
// first (V_PERMLANE16_SWAP), then two byte permutes per output word.
// MODE 0: any n:m, through the staged tile.
// MODE 5: no pattern at all -- the dense product L^T P [G, S] (the weight gradient of a linear layer
// in a dense format), staged like MODE 0 and stored as rows of `val` with a pitch of `ldv` elements
// (+ bias per position).
// NT = true: the operands are given with the reduction (tokens) as their fast dim, L^T [G, T] and
// P^T [S, T] (the weight gradient of torch.mm(W, B): grad_out [R, N] and B [C, N] as they lie in
// memory).  An operand tile of a K step is then 256 feature rows of 64 bytes; a fragment -- the
// lane's 8 consecutive tokens of its feature -- is one 16-byte LDS read, and the 16-byte pieces of
// a row are XOR-swizzled with (row/4)%4 on the global side.
template <typename T> struct SdMma16;
template <> struct SdMma16<__half> {
    using F = sd_f16x8;
    __device__ static f32x4 run(F a, F b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};
template <> struct SdMma16<__hip_bfloat16> {
    using F = sd_bf16x8;
    __device__ static f32x4 run(F a, F b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};

template <typename T, int MODE, bool NT = false>
__global__ __launch_bounds__(256, 1) void sddmm16_kernel(SddmmParams P)
{
    using Mm = SdMma16<T>;
    static_assert((MODE >= 0 && MODE <= 5) || MODE == 9 || MODE == 10 || MODE == 12,
                  "the staged tile; m == 4, n == MODE; the dense product; m == 8, n == MODE - 8");
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // Workgroup -> tile.  Consecutive ids are dealt round-robin to the 8 XCDs: give each XCD a
    // contiguous run of ids, and walk the grid in bands of 4 position tiles, so that a run covers
    // a compact block of tiles whose operands stay in that XCD's L2.
    int id = blockIdx.x;
    const int ntiles = P.tiles_p * P.tiles_l;
    if ((ntiles & 7) == 0) id = (id & 7) * (ntiles >> 3) + (id >> 3);
    constexpr int GH = 4;
    const int band = id / (GH * P.tiles_l);
    const int band_h = min(P.tiles_p - band * GH, GH);
    const int in_band = id - band * GH * P.tiles_l;
    const int tile_p = band * GH + in_band % band_h, tile_l = in_band / band_h;
    const int64_t p0 = (int64_t)tile_p * 256, l0 = (int64_t)tile_l * 256;
    const int wm = wave >> 1, wn = wave & 1;   // position half / line half of the wavefront
    const int KP = P.KP;
    const int j16 = lane & 15, kq = lane >> 4;

    // ---- the lane's slots, two per register.  MODE 1..4: accumulator block (x, y) is line
    // l0 + wn*128 + 16 y + l%16, block p0/4 + wm*32 + 4 x + l/16 (x even in the low half).
    // MODE 8 + n: a block of 8 positions lies in the lanes q = l/16 even (positions 0..3) and odd
    // (4..7) of one accumulator block; after the exchange in the epilogue a lane owns, per pair of
    // position blocks xp, block p0/8 + wm*16 + 4 xp + 2 (q%2) + q/2 of its line (xp even in the low half).
    uint32_t my_slot[(MODE == 0 || MODE == 5) ? 1 : (MODE <= 4 ? 32 : 16)];
    if constexpr (MODE >= 1 && MODE <= 4) {
        uint32_t *s_sel = (uint32_t *)(smem + 256 * SD_PITCH);
        if (tid < 16) {
            const uint32_t o = (uint32_t)(P.ord4 >> (8 * (tid & 7)));
            const int jj = (tid >> 3) * 2;
            const uint32_t a = (o >> (2 * jj)) & 3, b = (o >> (2 * jj + 2)) & 3;
            s_sel[tid] = (2 * a) | ((2 * a + 1) << 8) | ((2 * b) << 16) | ((2 * b + 1) << 24);
        }
#pragma unroll
        for (int y = 0; y < 8; y++) {
            const int64_t line = min(l0 + wn * 128 + y * 16 + j16, P.Gpad - 1);
#pragma unroll
            for (int xp = 0; xp < 4; xp++) {
                const int blk0 = min((int)(p0 / 4) + wm * 32 + (2 * xp) * 4 + kq, (int)P.nb - 1);
                const int blk1 = min((int)(p0 / 4) + wm * 32 + (2 * xp + 1) * 4 + kq, (int)P.nb - 1);
                my_slot[y * 4 + xp] = (uint32_t)(uint16_t)P.slot[blk0 * P.Gpad + line] |
                                      ((uint32_t)(uint16_t)P.slot[blk1 * P.Gpad + line] << 16);
            }
        }
    } else if constexpr (MODE > 8) {
        // selector table: per pattern and output word two V_PERM_B32 selectors, one for the
        // positions 0..3, one for 4..7 (bytes that come from the other half select zero)
        constexpr int N = MODE - 8, ND = (N + 1) / 2;
        uint32_t *s_sel = (uint32_t *)(smem + 256 * SD_PITCH);
        for (int e = tid; e < P.order_bytes / N * ND; e += 256) {
            const int pat = e / ND, w = e - pat * ND;
            uint32_t sa = 0x0c0c0c0cu, sb = 0x0c0c0c0cu;
#pragma unroll
            for (int jj = 0; jj < 2; jj++) {
                const int j = 2 * w + jj;
                if (j >= N) break;
                const uint32_t q = (uint32_t)P.order[pat * N + j] & 7u;
                const uint32_t two = (2 * (q & 3)) | ((2 * (q & 3) + 1) << 8);
                if (q < 4) sa = (sa & ~(0xffffu << (16 * jj))) | (two << (16 * jj));
                else sb = (sb & ~(0xffffu << (16 * jj))) | (two << (16 * jj));
            }
            s_sel[2 * e] = sa;
            s_sel[2 * e + 1] = sb;
        }
        const int own = 2 * (kq & 1) + (kq >> 1);
#pragma unroll
        for (int y = 0; y < 8; y++) {
            const int64_t line = min(l0 + wn * 128 + y * 16 + j16, P.Gpad - 1);
#pragma unroll
            for (int xq = 0; xq < 2; xq++) {
                const int blk0 = min((int)(p0 / 8) + wm * 16 + 4 * (2 * xq) + own, (int)P.nb - 1);
                const int blk1 = min((int)(p0 / 8) + wm * 16 + 4 * (2 * xq + 1) + own, (int)P.nb - 1);
                my_slot[y * 2 + xq] = (uint32_t)(uint16_t)P.slot[blk0 * P.Gpad + line] |
                                      ((uint32_t)(uint16_t)P.slot[blk1 * P.Gpad + line] << 16);
            }
        }
    }

    // ---- DMA sources.  Wavefronts 0, 1 fetch the position tile, 2, 3 the line tile; load i of a
    // wavefront fills token rows 2r, 2r+1 (r = (wave & 1) * 8 + i) of its operand tile: 1 KiB of
    // LDS, lane l -> row 2r + l/32, 16-byte piece l%32, which holds the logical chunk (8 features)
    // (l%32) ^ 4 * ((t % 4) + 4 * ((t / 8) % 2)) of token row t.  NT: load i fills feature rows
    // (wave & 1) * 128 + 16 i + l/4, slot l%4 <- logical piece (l%4) ^ (row/4)%4 (8 tokens); rows
    // beyond the extent repeat the last one (never stored).
    const bool is_l = wave >= 2;
    const unsigned char *gsrc = (const unsigned char *)(is_l ? P.lop : P.pop);
    const int64_t ld = is_l ? P.ldl : P.ldp, ext = is_l ? P.G : P.S, f0 = is_l ? l0 : p0;
    uint32_t g_off[SD_LPW];
#pragma unroll
    for (int i = 0; i < SD_LPW; i++) {
        if constexpr (NT) {
            const int row = (wave & 1) * 128 + 16 * i + (lane >> 2);
            const int piece = (lane & 3) ^ ((row >> 2) & 3);
            int64_t feat = f0 + row;
            if (feat > ext - 1) feat = ext - 1;
            g_off[i] = (uint32_t)(((feat - min(f0, ext - 1)) * ld + piece * 8) * 2);
        } else {
            const int tok = (((wave & 1) * 8 + i) << 1) + (lane >> 5);
            const int chunk = (lane & 31) ^ (((tok & 3) | ((tok >> 1) & 4)) << 2);
            int64_t feat = f0 + chunk * 8;
            if (feat > ext - 8) feat = ext - 8;   // columns beyond the extent feed outputs that are never stored
            g_off[i] = (uint32_t)((tok * ld + feat) * 2);
        }
    }
    const int tok_hi = lane >> 5;
    const int nt_tok = ((lane & 3) ^ ((lane >> 4) & 3)) * 8;
    const unsigned char *zero = (const unsigned char *)P.zero;
    // The DMA loads are written as instructions: they have no destination registers, so nothing
    // the compiler does with registers can race with them, and the compiler -- which would make
    // every LDS read wait for all DMA loads in flight -- does not see them.  Their completion is
    // tracked by the counted waits below.  (Every load that writes registers is the compiler's.)
    // K step kp goes to stage kp % SD_NS.  Steps beyond the last are fetched like the last one
    // (the count of outstanding operations stays uniform; the data is never used).
    struct Step {
        const unsigned char *b;   // first token row of the step in the wavefront's operand
        uint32_t dst;             // LDS address of the wavefront's first load
        int rem;                  // valid token rows of the step (>= SD_KS except at the end)
    };
    auto step_of = [&](int kp) {
        const int kc = kp < KP ? kp : KP - 1;
        Step st;
        st.b = NT ? gsrc + (min(f0, ext - 1) * ld + (int64_t)kc * SD_KS) * 2 : gsrc + (int64_t)kc * SD_KS * ld * 2;
        st.dst = (uint32_t)(uintptr_t)(lds_ptr_t)(smem + (kp & (SD_NS - 1)) * SD_STAGE + (is_l ? SD_OP : 0) +
                                                  (wave & 1) * 8 * 1024);
        st.rem = (int)min((int64_t)SD_KS, P.T - (int64_t)kc * SD_KS);
        return st;
    };
    // tail_tag: the step may hold the end of the operands -- token rows beyond it come from a page
    // of zeros, at the price of a 64-bit address per lane; the steps before the last take the
    // scalar base + 32-bit lane offset form.
    auto issue_one = [&](const Step &st, int i, auto tail_tag) {
        if constexpr (decltype(tail_tag)::value) {
            const int tok = NT ? nt_tok : (((wave & 1) * 8 + i) << 1) + tok_hi;
            const unsigned char *src = tok < st.rem ? st.b + g_off[i] : zero;
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                         :: "v"(src), "s"(st.dst + i * 1024) : "memory");
        } else {
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         :: "v"(g_off[i]), "s"(st.b), "s"(st.dst + i * 1024) : "memory");
        }
    };

    // ---- fragment addresses.  Token-major: lane (kq, i) of a transposing read supplies the 8 bytes
    // at token 8 kq + 4 r + i/4, features 4 (i%4) .. +3 of the block, and receives feature i at
    // tokens 8 kq + 4 r + 0..3.  Feature block f of an operand tile lies in granule f/2 (^ the
    // swizzle of the token), half f%2.
    const int tsw = (j16 >> 2) | ((kq & 1) << 2);
    const int tn_base = (8 * kq + (j16 >> 2)) * 512 + (j16 & 3) * 8;
    int fa_off[4], fb_off[4];   // per pair of feature blocks of the wavefront
#pragma unroll
    for (int f = 0; f < 4; f++) {
        if constexpr (NT) {
            // lane (kq, i) reads the 16 bytes of feature row 16 f' + i, piece kq ^ (row/4)%4
            fa_off[f] = (wm * 128 + f * 32 + j16) * 64 + ((kq ^ ((j16 >> 2) & 3)) << 4);
            fb_off[f] = (wn * 128 + f * 32 + j16) * 64 + ((kq ^ ((j16 >> 2) & 3)) << 4) + SD_OP;
        } else {
            fa_off[f] = tn_base + (((wm * 4 + f) ^ tsw) << 6);
            fb_off[f] = tn_base + (((wn * 4 + f) ^ tsw) << 6) + SD_OP;
        }
    }
    struct Frag {
        sd_i16x4 h[2];
    };
    Frag fa[2][4], fb[8];
    // half 0 / 1 of fragment f (0..7) of the position side (is_a) or the line side
    auto read_half = [&](Frag &d, const unsigned char *stage, bool is_a, int f, int r) {
        const int off = (is_a ? fa_off[f >> 1] : fb_off[f >> 1]);
        if constexpr (NT) {
            if (r == 0) {
                union {
                    u32x4 u;
                    sd_i16x4 h[2];
                } c;
                c.u = *(const u32x4 *)(stage + off + (f & 1) * 16 * 64);
                d.h[0] = c.h[0];
                d.h[1] = c.h[1];
            }
        } else {
            d.h[r] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((sd_lds_i16x4)(stage + off + (f & 1) * 32 + r * 4 * 512));
        }
    };
    constexpr int RPF = NT ? 1 : 2;   // LDS reads per fragment

    f32x4 acc[8][8];   // [position block][line block]
#pragma unroll
    for (int x = 0; x < 8; x++)
#pragma unroll
        for (int y = 0; y < 8; y++) acc[x][y] = f32x4{0.f, 0.f, 0.f, 0.f};
    auto pin_acc = [&]() {
#pragma unroll
        for (int x = 0; x < 8; x++)
#pragma unroll
            for (int y = 0; y < 8; y++) asm volatile("" : "+a"(acc[x][y]));
    };
    pin_acc();
    auto mma = [&](const Frag &a, const Frag &b, int x, int y) {
        union {
            sd_i16x4 h[2];
            typename Mm::F v;
        } ca, cb;
        ca.h[0] = a.h[0];
        ca.h[1] = a.h[1];
        cb.h[0] = b.h[0];
        cb.h[1] = b.h[1];
        acc[x][y] = Mm::run(ca.v, cb.v, acc[x][y]);
    };

    // Invariants of the ring.  (1) Outstanding memory operations of a wavefront complete in issue
    // order, SD_LPW per K step; at the counted wait of step kp the steps kp+1 .. kp+SD_D are
    // outstanding, so vmcnt((SD_D-1) * SD_LPW) means "my share of step kp+1 has landed", and the
    // barrier after it "everybody's".  (2) Stage (kp+SD_D) % SD_NS = (kp-1) % SD_NS is refilled
    // during the first phase of step kp; its last readers were the first-phase reads of step kp-1
    // (from their own stage) and the second-phase reads of step kp-2 (which fetch ahead); both
    // completed (lgkmcnt(0)) before the barrier of step kp-1, which every wavefront has passed
    // before it issues the loads of step kp.
#pragma unroll
    for (int s0 = 0; s0 < SD_D; s0++) {
        const Step st = step_of(s0);
#pragma unroll
        for (int i = 0; i < SD_LPW; i++) issue_one(st, i, std::true_type{});
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((SD_D - 1) * SD_LPW) : "memory");
    asm volatile("s_barrier" ::: "memory");
#pragma unroll
    for (int f = 0; f < 4; f++)
#pragma unroll
        for (int r = 0; r < RPF; r++) read_half(fa[0][f], smem, true, f, r);
#pragma unroll
    for (int f = 0; f < 8; f++)
#pragma unroll
        for (int r = 0; r < RPF; r++) read_half(fb[f], smem, false, f, r);

    auto k_step = [&](int kp, auto tail_tag) {
        const unsigned char *cur = smem + (kp & (SD_NS - 1)) * SD_STAGE;
        const unsigned char *nxt = smem + ((kp + 1) & (SD_NS - 1)) * SD_STAGE;
        const Step st = step_of(kp + SD_D);
        // phase 0: position blocks 0..3, column by column; behind the MFMAs the position
        // fragments 4..7 of this step and the DMA loads of step kp + SD_D, alternating
        constexpr int NA = 4 * RPF;   // reads of four position fragments
#pragma unroll
        for (int i = 0; i < 32; i++) {
            mma(fa[0][i & 3], fb[i >> 2], i & 3, i >> 2);
            __builtin_amdgcn_sched_barrier(0);
            if (i % 2 == 0) {
                const int k = i / 2;   // 0..15: read, load, read, load ...
                if (k % 2 == 0 && k / 2 < NA)
                    read_half(fa[1][(k / 2) / RPF], cur, true, 4 + (k / 2) / RPF, (k / 2) % RPF);
                else if (k % 2 == 1 && k / 2 < SD_LPW)
                    issue_one(st, k / 2, tail_tag);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // wait for step kp+1 and meet the other wavefronts (the reads of stage kp are complete)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((SD_D - 1) * SD_LPW) : "memory");
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        // phase 1: position blocks 4..7; behind the MFMAs first the position fragments 0..3 of the
        // next step, then its line fragments, fragment y once column y is done
#pragma unroll
        for (int i = 0; i < 32; i++) {
            mma(fa[1][i & 3], fb[i >> 2], 4 + (i & 3), i >> 2);
            __builtin_amdgcn_sched_barrier(0);
            if (i < NA) {
                read_half(fa[0][i / RPF], nxt, true, i / RPF, i % RPF);
            } else {
                // line fragment read number k = i - NA, not before column k / RPF is done
#pragma unroll
                for (int k = 0; k < 8 * RPF; k++) {
                    const int at = NA + k > 4 * (k / RPF) + 3 ? NA + k : 4 * (k / RPF) + 3;
                    if (at == i) read_half(fb[k / RPF], nxt, false, k / RPF, k % RPF);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // reads whose slot lies beyond the last MFMA
#pragma unroll
        for (int k = 0; k < 8 * RPF; k++) {
            const int at = NA + k > 4 * (k / RPF) + 3 ? NA + k : 4 * (k / RPF) + 3;
            if (at >= 32) read_half(fb[k / RPF], nxt, false, k / RPF, k % RPF);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    // steps whose prefetch (step kp + SD_D) lies before the last step take the short address form
    const int kp_tail = max(0, KP - 1 - SD_D);
    for (int kp = 0; kp < kp_tail; kp++) k_step(kp, std::false_type{});
    for (int kp = kp_tail; kp < KP; kp++) k_step(kp, std::true_type{});
    pin_acc();
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");

    if constexpr (MODE == 0) {
        // ---- epilogue through LDS: stage [line][position] in the output type, then thread = line
        asm volatile("s_barrier" ::: "memory");   // every wavefront is done with the ring
        int8_t *s_ord = (int8_t *)(smem + 256 * SD_PITCH);
        for (int i = tid; i < P.order_bytes; i += 256) s_ord[i] = P.order[i];
#pragma unroll
        for (int y = 0; y < 8; y++)
#pragma unroll
            for (int x = 0; x < 8; x++) {
                uint16_t hh[4];
#pragma unroll
                for (int r = 0; r < 4; r++) hh[r] = sd_bits16<T>(sd_from_acc(acc[x][y][r]));
                uint2 pk;
                pk.x = (uint32_t)hh[0] | ((uint32_t)hh[1] << 16);
                pk.y = (uint32_t)hh[2] | ((uint32_t)hh[3] << 16);
                const int line = wn * 128 + y * 16 + j16, pos = wm * 128 + x * 16 + kq * 4;
                *(uint2 *)(smem + line * SD_PITCH + pos * 2) = pk;
            }
        __syncthreads();
        sd_staged_walk(P, smem, tid, l0, p0);
    } else if constexpr (MODE == 5) {
        // ---- dense product: stage [line][position] in the output type, then whole rows: a
        // wavefront stores two lines per instruction, 16 bytes per lane
        asm volatile("s_barrier" ::: "memory");   // every wavefront is done with the ring
#pragma unroll
        for (int y = 0; y < 8; y++)
#pragma unroll
            for (int x = 0; x < 8; x++) {
                uint16_t hh[4];
#pragma unroll
                for (int r = 0; r < 4; r++) hh[r] = sd_bits16<T>(sd_from_acc(acc[x][y][r]));
                uint2 pk;
                pk.x = (uint32_t)hh[0] | ((uint32_t)hh[1] << 16);
                pk.y = (uint32_t)hh[2] | ((uint32_t)hh[3] << 16);
                const int line = wn * 128 + y * 16 + j16, pos = wm * 128 + x * 16 + kq * 4;
                *(uint2 *)(smem + line * SD_PITCH + pos * 2) = pk;
            }
        __syncthreads();
        const int64_t pos = p0 + (lane & 31) * 8;
        float bv[8];
#pragma unroll
        for (int e = 0; e < 8; e++) bv[e] = (P.bias && pos + e < P.S) ? to_f32(((const T *)P.bias)[pos + e]) : 0.f;
        for (int it = wave; it < 128; it += 4) {
            const int row = 2 * it + (lane >> 5);
            const int64_t line = l0 + row;
            const unsigned char *src = smem + row * SD_PITCH + (lane & 31) * 16;
            uint2 lo = *(const uint2 *)src, hi = *(const uint2 *)(src + 8);   // (rows are 8-byte aligned)
            if (line >= P.G || pos >= P.S) continue;                          // S % 8 == 0: a piece is whole or absent
            uint32_t w[4] = {lo.x, lo.y, hi.x, hi.y};
            if (P.bias) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    uint16_t a = (uint16_t)w[e], b = (uint16_t)(w[e] >> 16);
                    a = sd_bits16<T>(to_f32(__builtin_bit_cast(T, a)) + bv[2 * e]);
                    b = sd_bits16<T>(to_f32(__builtin_bit_cast(T, b)) + bv[2 * e + 1]);
                    w[e] = (uint32_t)a | ((uint32_t)b << 16);
                }
            }
            *(u32x4 *)((uint16_t *)P.val + line * P.ldv + pos) = u32x4{w[0], w[1], w[2], w[3]};
        }
    } else if constexpr (MODE > 8) {
        // ---- epilogue in registers, m == 8.  The lanes q even / odd round and pack their halves of
        // the blocks in the accumulator blocks 2 xp and 2 xp + 1 and exchange them
        // (V_PERMLANE16_SWAP: odd rows of 16 lanes of the first operand <-> even rows of the second),
        // after which each owns one whole block as four words; the kept values are picked with two
        // byte permutes per output word.
        constexpr int N = MODE - 8, ND = (N + 1) / 2;
        const uint32_t *s_sel = (const uint32_t *)(smem + 256 * SD_PITCH);
        asm volatile("s_barrier" ::: "memory");   // the selector table was written by other wavefronts
        int blk_base = (int)(p0 / 8) + wm * 16 + 2 * (kq & 1) + (kq >> 1);
        asm volatile("" : "+v"(blk_base));
        const uint32_t cg = (uint32_t)P.cg, nb = (uint32_t)P.nb;
        const uint32_t g1_mask = P.g > 1 ? 0u : ~0u;
        unsigned char *vbase = (unsigned char *)P.val;
        auto epilogue = [&](auto interior_tag) {
            constexpr bool INTERIOR = decltype(interior_tag)::value;
#pragma unroll
            for (int y = 0; y < 8; y++) {
                const uint32_t line = (uint32_t)l0 + wn * 128 + y * 16 + j16;
                const bool line_in = INTERIOR || line < (uint32_t)P.Gpad, line_ok = INTERIOR || line < (uint32_t)P.G;
                const uint32_t rowbase = ((line / cg) * nb + (uint32_t)blk_base) * cg;
#pragma unroll
                for (int xp = 0; xp < 4; xp++) {
                    const uint32_t sl = min((my_slot[y * 2 + (xp >> 1)] >> (16 * (xp & 1))) & 0x7fffu, cg - 1);
                    const uint32_t pat = __umulhi(sl, P.inv_g) + (sl & g1_mask);
                    uint32_t sel[ND][2];
#pragma unroll
                    for (int w = 0; w < ND; w++) {
                        sel[w][0] = s_sel[(pat * ND + w) * 2];
                        sel[w][1] = s_sel[(pat * ND + w) * 2 + 1];
                    }
                    uint32_t d[4];   // before the exchange: block 2 xp words 0, 1, block 2 xp + 1 words 0, 1
#pragma unroll
                    for (int qd = 0; qd < 2; qd++)
#pragma unroll
                        for (int w = 0; w < 2; w++) {
                            const uint16_t lo16 = sd_bits16<T>(sd_from_acc(acc[2 * xp + qd][y][2 * w]));
                            const uint16_t hi16 = sd_bits16<T>(sd_from_acc(acc[2 * xp + qd][y][2 * w + 1]));
                            d[qd * 2 + w] = (uint32_t)lo16 | ((uint32_t)hi16 << 16);
                        }
                    uint32_t blkw[4];   // positions 0,1 | 2,3 | 4,5 | 6,7 of the lane's block
#pragma unroll
                    for (int w = 0; w < 2; w++) {
                        const auto sw = __builtin_amdgcn_permlane16_swap(d[w], d[2 + w], false, false);
                        blkw[w] = sw[0];
                        blkw[2 + w] = sw[1];
                    }
                    if (!INTERIOR && !line_ok) blkw[0] = blkw[1] = blkw[2] = blkw[3] = 0;
                    if (!INTERIOR && (!line_in || blk_base + xp * 4 >= (int)nb)) continue;
                    unsigned char *dst =
                        vbase + (size_t)((rowbase + (uint32_t)(xp * 4) * cg + sl) * (uint32_t)(2 * N));
                    uint32_t out[ND];
#pragma unroll
                    for (int w = 0; w < ND; w++)
                        out[w] = __builtin_amdgcn_perm(blkw[1], blkw[0], sel[w][0]) |
                                 __builtin_amdgcn_perm(blkw[3], blkw[2], sel[w][1]);
                    if constexpr (N == 1) {
                        *(uint16_t *)dst = (uint16_t)out[0];
                    } else if constexpr (N == 2) {
                        *(uint32_t *)dst = out[0];
                    } else {
                        static_assert(N == 4, "m == 8 is built for n = 1, 2, 4");
                        *(uint2 *)dst = uint2{out[0], out[1]};
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        if (l0 + 256 <= P.G && p0 + 256 <= P.nb * 8)
            epilogue(std::true_type{});
        else
            epilogue(std::false_type{});
    } else {
        // ---- epilogue in registers: the 4 registers of an accumulator block are one block of the
        // lane's line.  Offsets into val are 32-bit (the host checks that val is smaller than 4 GiB).
        constexpr int N = MODE;
        const uint32_t *s_sel = (const uint32_t *)(smem + 256 * SD_PITCH);
        int blk_base = (int)(p0 / 4) + wm * 32 + kq;
        asm volatile("" : "+v"(blk_base));
        const uint32_t cg = (uint32_t)P.cg, nb = (uint32_t)P.nb;
        const uint32_t g1_mask = P.g > 1 ? 0u : ~0u;   // inv_g is 0 for g == 1
        unsigned char *vbase = (unsigned char *)P.val;
        asm volatile("s_barrier" ::: "memory");   // the selector table was written by other wavefronts
        auto epilogue = [&](auto interior_tag) {
            constexpr bool INTERIOR = decltype(interior_tag)::value;
#pragma unroll
            for (int y = 0; y < 8; y++) {
                const uint32_t line = (uint32_t)l0 + wn * 128 + y * 16 + j16;
                const bool line_in = INTERIOR || line < (uint32_t)P.Gpad, line_ok = INTERIOR || line < (uint32_t)P.G;
                const uint32_t rowbase = ((line / cg) * nb + (uint32_t)blk_base) * cg;
#pragma unroll
                for (int xq = 0; xq < 2; xq++) {
                    uint32_t sl[4], sel[4], sel2[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int x = xq * 4 + e;
                        sl[e] = min((my_slot[y * 4 + (x >> 1)] >> (16 * (x & 1))) & 0x7fffu, cg - 1);
                        const uint32_t pat = __umulhi(sl[e], P.inv_g) + (sl[e] & g1_mask);   // slot / g without a branch
                        if constexpr (N < 4) sel[e] = s_sel[pat & 7];
                        if constexpr (N == 3) sel2[e] = s_sel[8 + (pat & 7)];
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int x = xq * 4 + e;
                        uint16_t hh[4];
#pragma unroll
                        for (int r = 0; r < 4; r++) hh[r] = sd_bits16<T>(sd_from_acc(acc[x][y][r]));
                        uint32_t lo = (uint32_t)hh[0] | ((uint32_t)hh[1] << 16);
                        uint32_t hi = (uint32_t)hh[2] | ((uint32_t)hh[3] << 16);
                        if (!INTERIOR && !line_ok) lo = hi = 0;
                        if (!INTERIOR && (!line_in || blk_base + x * 4 >= (int)nb)) continue;
                        unsigned char *dst =
                            vbase + (size_t)((rowbase + (uint32_t)(x * 4) * cg + sl[e]) * (uint32_t)(2 * N));
                        if constexpr (N == 4) {
                            *(uint2 *)dst = uint2{lo, hi};
                        } else {
                            const uint32_t out = __builtin_amdgcn_perm(hi, lo, sel[e]);
                            if constexpr (N == 1) {
                                *(uint16_t *)dst = (uint16_t)out;
                            } else if constexpr (N == 2) {
                                *(uint32_t *)dst = out;
                            } else {   // 6-byte entries are 2-byte aligned only
                                const uint32_t out2 = __builtin_amdgcn_perm(hi, lo, sel2[e]);
                                ((uint16_t *)dst)[0] = (uint16_t)out;
                                ((uint16_t *)dst)[1] = (uint16_t)(out >> 16);
                                ((uint16_t *)dst)[2] = (uint16_t)out2;
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        if (l0 + 256 <= P.G && p0 + 256 <= P.nb * 4)
            epilogue(std::true_type{});
        else
            epilogue(std::false_type{});
    }
}

}  // namespace nmg

using namespace nmg;

extern "C" int nmg_slotmap(const int16_t *d_idx, int64_t G, int64_t S, int16_t *d_slot, int n, int m, int g,
                           void *stream)
{
    NMG_REQUIRE(host_order(n, m) != nullptr && g >= 1, NMG_ERR_ARG, "invalid n:m:g = %d:%d:%d", n, m, g);
    NMG_REQUIRE(G >= 0 && S >= 0, NMG_ERR_ARG, "negative extent");
    const int64_t cg = binom(m, n) * g;
    NMG_REQUIRE(cg < 32768, NMG_ERR_ARG, "c*g must be below 2^15");
    if (G == 0 || S == 0) return NMG_OK;
    NMG_REQUIRE(d_idx && d_slot, NMG_ERR_ARG, "null device pointer");
    SlotParams P{};
    P.idx = d_idx;
    P.slot = d_slot;
    P.nb = (S + m - 1) / m;
    const int64_t chunks = (G + cg - 1) / cg;
    P.Gpad = chunks * cg;
    P.cg = (int)cg;
    P.entries = chunks * P.nb * cg;
    const int64_t blocks = (P.entries + 255) / 256;
    NMG_REQUIRE(blocks <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "weight too large for one launch");
    hipLaunchKernelGGL(slotmap_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, P);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

static int sddmm_impl(bool nt, const void *d_lines, int64_t ld_lines, const void *d_pos, int64_t ld_pos, int64_t T,
                      const int16_t *d_slot, int64_t G, int64_t S, void *d_val, int n, int m, int g, int dtype,
                      void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "the masked product takes f16/bf16");
    NMG_REQUIRE(host_order(n, m) != nullptr && g >= 1, NMG_ERR_ARG, "invalid n:m:g = %d:%d:%d", n, m, g);
    NMG_REQUIRE(G >= 0 && S >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    const int64_t cg = binom(m, n) * g;
    NMG_REQUIRE(cg < 32768, NMG_ERR_ARG, "c*g must be below 2^15");
    NMG_REQUIRE(nt ? (ld_lines >= T && ld_pos >= T) : (ld_lines >= G && ld_pos >= S), NMG_ERR_ARG,
                "leading dimension smaller than row length");
    if (G == 0 || S == 0 || n == 0) return NMG_OK;
    NMG_REQUIRE(T > 0, NMG_ERR_UNSUPPORTED, "no tokens: clear val instead");
    NMG_REQUIRE((nt || (G % 8 == 0 && S % 8 == 0)) && ld_lines % 8 == 0 && ld_pos % 8 == 0 &&
                    ((uintptr_t)d_lines % 16) == 0 && ((uintptr_t)d_pos % 16) == 0,
                NMG_ERR_UNSUPPORTED, "needs extents and leading dimensions that are multiples of 8 and 16-byte aligned operands");
    NMG_REQUIRE(ld_lines < ((int64_t)1 << (nt ? 22 : 25)) && ld_pos < ((int64_t)1 << (nt ? 22 : 25)), NMG_ERR_UNSUPPORTED,
                "leading dimension too large");
    NMG_REQUIRE(!nt || T % 8 == 0, NMG_ERR_UNSUPPORTED, "reduction-contiguous operands need a token count that is a multiple of 8");
    NMG_REQUIRE(d_lines && d_pos && d_slot && d_val, NMG_ERR_ARG, "null device pointer");
    SddmmParams P{};
    if (int rc = device_order(n, m, &P.order)) return rc;
    if (int rc = device_zero_page(&P.zero)) return rc;
    P.lop = d_lines;
    P.pop = d_pos;
    P.val = d_val;
    P.slot = d_slot;
    P.ldl = ld_lines;
    P.ldp = ld_pos;
    P.G = G;
    P.S = S;
    P.T = T;
    P.nb = (S + m - 1) / m;
    P.Gpad = (G + cg - 1) / cg * cg;
    P.n = n;
    P.m = m;
    P.g = g;
    P.cg = (int)cg;
    P.inv_g = g > 1 ? (uint32_t)((((uint64_t)1 << 32) + g - 1) / (uint64_t)g) : 0u;
    P.order_bytes = (int)(binom(m, n) * n);
    P.KP = (int)((T + SD_KS - 1) / SD_KS);
    P.tiles_p = (int)((P.nb * m + 255) / 256);
    P.tiles_l = (int)((P.Gpad + 255) / 256);
    NMG_REQUIRE((int64_t)P.tiles_p * P.tiles_l <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "weight too large for one launch");
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)(P.tiles_p * P.tiles_l));
    // m == 4, val 8-byte aligned and smaller than 4 GiB: the epilogue that stays in registers
    const int64_t val_bytes = ((G + cg - 1) / cg) * P.nb * cg * n * 2;
    const bool small = ((uintptr_t)d_val % 8) == 0 && val_bytes < ((int64_t)1 << 32) && P.Gpad < ((int64_t)1 << 31);
    const bool in_regs = m == 4 && n >= 1 && small;
    const bool in_regs8 = m == 8 && (n == 1 || n == 2 || n == 4) && small;
    if (in_regs) {
        const int8_t *ho = host_order(n, m);
        for (int64_t p = 0; p < binom(m, n); p++)
            for (int j = 0; j < n; j++) P.ord4 |= (uint64_t)(ho[p * n + j] & 3) << (8 * p + 2 * j);
    }
    auto launch = [&](auto k) -> int {
        NMG_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, SD_LDS));
        hipLaunchKernelGGL(k, grid, dim3(256), SD_LDS, s, P);
        return NMG_OK;
    };
    auto launch_t = [&](auto tag) -> int {
        using T = decltype(tag);
        if (nt) {   // reduction-contiguous operands; the epilogues in registers need every block of m positions whole
            if (in_regs && S % 4 == 0) {
                switch (n) {
                case 1: return launch(sddmm16_kernel<T, 1, true>);
                case 2: return launch(sddmm16_kernel<T, 2, true>);
                case 3: return launch(sddmm16_kernel<T, 3, true>);
                default: return launch(sddmm16_kernel<T, 4, true>);
                }
            }
            if (in_regs8 && S % 8 == 0) {
                if (n == 1) return launch(sddmm16_kernel<T, 9, true>);
                if (n == 2) return launch(sddmm16_kernel<T, 10, true>);
                return launch(sddmm16_kernel<T, 12, true>);
            }
            return launch(sddmm16_kernel<T, 0, true>);
        }
        if (in_regs8) {
            if (n == 1) return launch(sddmm16_kernel<T, 9>);
            if (n == 2) return launch(sddmm16_kernel<T, 10>);
            return launch(sddmm16_kernel<T, 12>);
        }
        if (!in_regs) return launch(sddmm16_kernel<T, 0>);
        switch (n) {
        case 1: return launch(sddmm16_kernel<T, 1>);
        case 2: return launch(sddmm16_kernel<T, 2>);
        case 3: return launch(sddmm16_kernel<T, 3>);
        default: return launch(sddmm16_kernel<T, 4>);
        }
    };
    const int rc = dtype == NMG_F16 ? launch_t(__half{}) : launch_t(__hip_bfloat16{});
    if (rc) return rc;
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

namespace nmg {
// Dense product on the same kernel: Y[G, S] = L[T, G]^T P[T, S] (+ bias[s]) in a 16-bit type, fp32
// accumulation, rounded once.  Both operands token-major with extents and pitches that are
// multiples of 8 and 16-byte aligned bases (NMG_ERR_UNSUPPORTED otherwise).
int dense_tn16(const void *d_lines, int64_t ld_lines, const void *d_pos, int64_t ld_pos, int64_t T, int64_t G, int64_t S,
               void *d_y, int64_t ldy, const void *d_bias, int dtype, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "the 16-bit product takes f16/bf16");
    if (G == 0 || S == 0) return NMG_OK;
    NMG_REQUIRE(T > 0, NMG_ERR_UNSUPPORTED, "no tokens: clear the result instead");
    NMG_REQUIRE(G % 8 == 0 && S % 8 == 0 && ld_lines % 8 == 0 && ld_pos % 8 == 0 && ldy % 8 == 0 &&
                    ((uintptr_t)d_lines % 16) == 0 && ((uintptr_t)d_pos % 16) == 0 && ((uintptr_t)d_y % 16) == 0,
                NMG_ERR_UNSUPPORTED, "needs extents and leading dimensions that are multiples of 8 and 16-byte aligned operands");
    NMG_REQUIRE(ld_lines < ((int64_t)1 << 25) && ld_pos < ((int64_t)1 << 25), NMG_ERR_UNSUPPORTED, "leading dimension too large");
    NMG_REQUIRE(d_lines && d_pos && d_y, NMG_ERR_ARG, "null device pointer");
    SddmmParams P{};
    if (int rc = device_zero_page(&P.zero)) return rc;
    P.lop = d_lines;
    P.pop = d_pos;
    P.val = d_y;
    P.bias = d_bias;
    P.ldl = ld_lines;
    P.ldp = ld_pos;
    P.ldv = ldy;
    P.G = G;
    P.S = S;
    P.T = T;
    P.nb = S;
    P.Gpad = G;
    P.n = P.m = P.g = 1;
    P.cg = 1;
    P.KP = (int)((T + SD_KS - 1) / SD_KS);
    P.tiles_p = (int)((S + 255) / 256);
    P.tiles_l = (int)((G + 255) / 256);
    NMG_REQUIRE((int64_t)P.tiles_p * P.tiles_l <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "product too large for one launch");
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)(P.tiles_p * P.tiles_l));
    if (dtype == NMG_F16) {
        auto k = sddmm16_kernel<__half, 5>;
        NMG_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, SD_LDS));
        hipLaunchKernelGGL(k, grid, dim3(256), SD_LDS, s, P);
    } else {
        auto k = sddmm16_kernel<__hip_bfloat16, 5>;
        NMG_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, SD_LDS));
        hipLaunchKernelGGL(k, grid, dim3(256), SD_LDS, s, P);
    }
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}
}  // namespace nmg

extern "C" int nmg_sddmm(const void *d_lines, int64_t ld_lines, const void *d_pos, int64_t ld_pos, int64_t T,
                         const int16_t *d_slot, int64_t G, int64_t S, void *d_val, int n, int m, int g,
                         int dtype, void *stream)
{
    return sddmm_impl(false, d_lines, ld_lines, d_pos, ld_pos, T, d_slot, G, S, d_val, n, m, g, dtype, stream);
}

extern "C" int nmg_sddmm_nt(const void *d_lines_t, int64_t ld_lines, const void *d_pos_t, int64_t ld_pos, int64_t T,
                            const int16_t *d_slot, int64_t G, int64_t S, void *d_val, int n, int m, int g,
                            int dtype, void *stream)
{
    return sddmm_impl(true, d_lines_t, ld_lines, d_pos_t, ld_pos, T, d_slot, G, S, d_val, n, m, g, dtype, stream);
}
