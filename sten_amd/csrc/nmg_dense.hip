// nmg x dense matmul on the dense matrix cores (V_MFMA_F32_32X32X16_{F16,BF16}), pipelined.
//
// Serves what the sparse matrix cores cannot: patterns that do not fit 2-of-4 groups (4:8, 3:4,
// ...) and, above all, the reduction along the *group* dim, i.e. the gradient with respect to
// the activations of a weight that is n:m along its own reduction dim:
//
//   reduce_sparse = 1:  Y[tok, q] = sum_s X[tok, s] * W2[q, s]      (q = line, s = sparse position)
//   reduce_sparse = 0:  Y[tok, s] = sum_q X[tok, q] * W2[q, s]
//
// Structure (same skeleton as the sparse-matrix-core pipeline): a workgroup of 8 wavefronts
// computes 256 outputs x 128 tokens; 4 matrix wavefronts (128 x 64 each) only read fragments
// from LDS and issue MFMAs, 4 loader wavefronts build the operands in a ring of 3 LDS stages
// (64 reduction steps each):
//   - activations: LDS-DMA loads, 16-byte chunks XOR-swizzled per row;
//   - weights: the rowpack operand (n values + pattern number per block) is fetched into
//     registers one stage ahead, expanded to dense rows -- transposed on the way for
//     reduce_sparse = 0, where 8 consecutive lines become one 16-byte chunk -- and written with
//     ds_write_b128 into the same swizzled layout.
// One s_barrier per stage.  n and m are template parameters so that the expansion is
// straight-line code on registers.  Requirements: 16-bit data, K % 64 == 0, m in {4, 8}.
//
// The file also holds the two halves of "expand, then multiply": the expansion of the rowpack
// operand into a dense matrix, and the plain NT GEMMs that multiply it (the 16-bit one on the
// pipeline above, the single-precision one -- gemm_nt_f32_kernel, V_MFMA_F32_32X32X2_F32 -- with
// its own three-stage loop; single-precision products with more than 16 tokens run on it).
#include "nmg_common.h"

#include <type_traits>

namespace nmg {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void *lds_ptr_t;
typedef const __attribute__((address_space(1))) void *glb_ptr_t;

template <typename T> struct Dmma;
template <> struct Dmma<__half> {
    using F = f16x8;
    __device__ static f32x16 run(F a, F b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct Dmma<__hip_bfloat16> {
    using F = bf16x8;
    __device__ static f32x16 run(F a, F b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};

__device__ __forceinline__ uint16_t dn_bits16(float x, __half *) { return __half_as_ushort(__float2half(x)); }
__device__ __forceinline__ uint16_t dn_bits16(float x, __hip_bfloat16 *)
{
    __hip_bfloat16 b = __float2bfloat16(x);
    return *reinterpret_cast<uint16_t *>(&b);
}

struct DenseParams {
    const void *pk_val;
    const void *pk_pat;
    const int8_t *order;
    const void *x;
    void *y;
    const void *bias;
    int64_t G, S, nb, T, ldx, ldy;
    int64_t K, O;  // reduction extent, output features
    int c, tiles_m, tiles_n;
};

constexpr int DN_NS = 3;                  // ring stages
constexpr int DN_P = 256 * 128;           // weight tile: 256 output rows x 64 k (bytes)
constexpr int DN_Q = 128 * 128;           // activation tile: 128 tokens x 64 k
constexpr int DN_STAGE = DN_P + DN_Q;
constexpr int DN_LUT = 2048;              // per pattern, M/2 byte-permute selectors
constexpr int DN_OUT_ROW = 128 * 2 + 16;

// swizzled byte offset of 16-byte chunk `chunk` of row `row` in a [rows][128 B] tile
__device__ __forceinline__ int dn_sw(int row, int chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); }

template <typename T, int N, int M, bool REDUCE_SPARSE>
__global__ __launch_bounds__(512, 2) void spmm_dense_pipe_kernel(DenseParams P)
{
    using D = Dmma<T>;
    // N == 0: the weight operand is already dense, row-major [O, K] with leading dimension P.nb
    // (pk_val points at it); both operands then travel by DMA and the loaders do nothing else.
    constexpr bool PDENSE = (N == 0);
    static_assert(M == 4 || M == 8 || M == 16, "block size");
    static_assert(N >= 0 && N <= 4 && N <= M, "kept values per block (one 64-bit permute source)");
    constexpr int FA = 4, FB = 2;
    extern __shared__ __align__(16) unsigned char smem_all[];
    uint32_t *lut = (uint32_t *)smem_all;
    unsigned char *smem = smem_all + DN_LUT;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    int id = blockIdx.x;
    const int ntiles = P.tiles_m * P.tiles_n;
    if ((ntiles & 7) == 0) id = (id & 7) * (ntiles >> 3) + (id >> 3);
    constexpr int GH = 4;
    const int band = id / (GH * P.tiles_n);
    const int band_h = min(P.tiles_m - band * GH, GH);
    const int in_band = id - band * GH * P.tiles_n;
    const int tile_m = band * GH + in_band % band_h, tile_n = in_band / band_h;
    const int64_t o0 = (int64_t)tile_m * 256, t0 = (int64_t)tile_n * 128;
    const int KP = (int)(P.K / 64);

    // lut[p][k], k < M/2: v_perm_b32 selector that builds dense positions 2k, 2k+1 of a block
    // with pattern p from its packed kept values (bytes 0..2N-1 of a 64-bit source); 0x0C = zero.
    for (int e = tid; !PDENSE && e < P.c * (M / 2); e += 512) {
        const int p = e / (M / 2), k = e % (M / 2);
        uint32_t sel = 0;
        for (int hh = 0; hh < 2; hh++) {
            const int r = 2 * k + hh;
            uint32_t sb = 0x0C0Cu;
            for (int jj = 0; jj < N; jj++)
                if (P.order[p * N + jj] == r) sb = (uint32_t)(2 * jj) | ((uint32_t)(2 * jj + 1) << 8);
            sel |= sb << (16 * hh);
        }
        lut[e] = sel;
    }
    __syncthreads();

    if (wave >= 4) {
        // ================================ loader wavefronts ================================
        // Two groups of two wavefronts; group g builds the stages s with s % 2 == g.  A group
        // issues everything for stage s (DMA loads, and the register loads of its next stage
        // s+2) right after barrier s-3 and only waits for it (vmcnt(0)) just before barrier
        // s-1, two K steps later, so fabric latency is covered without counting loads.
        const int grp = (wave - 4) >> 1;
        const int gw = (wave - 4) & 1;            // wavefront inside the group
        const int gt = gw * 64 + lane;            // thread inside the group, 0..127
        const uint16_t *pkv = (const uint16_t *)P.pk_val;
        const uint8_t *pkp = (const uint8_t *)P.pk_pat;
        // activations (DMA): wavefront gw moves row groups 8gw..8gw+7 (8 rows each)
        const unsigned char *x_base = (const unsigned char *)P.x;
        uint32_t x_off[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int row = (gw * 8 + i) * 8 + (lane >> 3);
            const int q = (lane & 7) ^ ((row >> 1) & 7);
            int64_t tok = t0 + row;
            if (tok >= P.T) tok = P.T - 1;
            x_off[i] = (uint32_t)((tok * P.ldx + q * 8) * 2);
        }

        // ---- register image of one stage of compressed weights (vector loads) ----
        // reduce_sparse: this thread owns output lines o0 + gt and o0 + gt + 128; per line and
        //   stage 64/M blocks: RS_VW words of packed values, RS_PW words of pattern bytes.
        // otherwise: one item per thread = 16 consecutive sparse positions (16/M blocks) of 8
        //   consecutive lines; per line RG_VW words of values and 16/M pattern bytes.
        constexpr int NBLK = 64 / M;
        constexpr int RS_VW = NBLK * N / 2;
        constexpr int RS_PW = NBLK / 4;
        constexpr int RG_NB = 16 / M;                 // blocks per item and line
        constexpr int RG_VW = RG_NB * N / 2;          // words of values per item and line
        static_assert((NBLK * N) % 8 == 0, "a stage row of values must be whole 16-byte chunks");
        static_assert((RG_NB * N) % 2 == 0, "an item row of values must be whole words");
        constexpr int NVW = PDENSE ? 1 : (REDUCE_SPARSE ? 2 * RS_VW : 8 * RG_VW);
        constexpr int NPW = PDENSE ? 1 : (REDUCE_SPARSE ? 2 * RS_PW : 8);
        // dense weight operand (DMA): wavefront gw moves row groups 16gw..16gw+15 (8 rows each)
        uint32_t p_off[16];
        if (PDENSE) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int row = (gw * 16 + i) * 8 + (lane >> 3);
                const int q = (lane & 7) ^ ((row >> 1) & 7);
                int64_t o = o0 + row;
                if (o >= P.O) o = P.O - 1;                 // clamped rows are computed, never stored
                p_off[i] = (uint32_t)((o * P.nb + q * 8) * 2);
            }
        }
        uint32_t rv[NVW];   // packed 16-bit values
        uint32_t rp[NPW];   // pattern bytes

        auto load_regs = [&](int kp) {
            if constexpr (PDENSE) {
            } else if constexpr (REDUCE_SPARSE) {
#pragma unroll
                for (int rr = 0; rr < 2; rr++) {
                    const int64_t q = o0 + gt + rr * 128;
                    const bool live = q < P.G;
                    const int64_t blk0 = (live ? q : 0) * P.nb + (int64_t)kp * NBLK;
                    const u32x4 *pv = (const u32x4 *)(pkv + blk0 * N);
#pragma unroll
                    for (int e = 0; e < RS_VW / 4; e++) {
                        u32x4 v = live ? pv[e] : u32x4{0, 0, 0, 0};
                        rv[rr * RS_VW + e * 4 + 0] = v.x;
                        rv[rr * RS_VW + e * 4 + 1] = v.y;
                        rv[rr * RS_VW + e * 4 + 2] = v.z;
                        rv[rr * RS_VW + e * 4 + 3] = v.w;
                    }
                    const uint32_t *pp = (const uint32_t *)(pkp + blk0);
#pragma unroll
                    for (int e = 0; e < RS_PW; e++) rp[rr * RS_PW + e] = live ? pp[e] : 0u;
                }
            } else {
                const int lg = gt & 7, pg = gt >> 3;
                const int64_t b0 = o0 / M + pg * RG_NB;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const int64_t q = (int64_t)kp * 64 + lg * 8 + i;
                    const bool live = q < P.G && b0 < P.nb;
                    const int64_t blk = (live ? q : 0) * P.nb + (live ? b0 : 0);
                    const uint32_t *pv = (const uint32_t *)(pkv + blk * N);
#pragma unroll
                    for (int e = 0; e < RG_VW; e++) rv[i * RG_VW + e] = live ? pv[e] : 0u;
                    uint32_t pw = 0;
                    if (live) {
                        if (RG_NB == 8) {
                            // 8 pattern bytes: only the low 4 are kept in one word, the rest in the next load
                            pw = *(const uint32_t *)(pkp + blk);
                        } else if (RG_NB == 4) {
                            pw = *(const uint32_t *)(pkp + blk);
                        } else if (RG_NB == 2) {
                            pw = *(const uint16_t *)(pkp + blk);
                        } else {
                            pw = pkp[blk];
                        }
                    }
                    rp[i] = pw;
                }
            }
        };
        // 64-bit window of a packed 16-bit array starting at element e0 (static)
        auto window = [&](const uint32_t *w, int e0, int nwords, uint32_t &lo, uint32_t &hi) {
            const int w0 = e0 >> 1;
            const uint32_t a0 = w[w0];
            const uint32_t a1 = (w0 + 1 < nwords) ? w[w0 + 1] : 0u;
            const uint32_t a2 = (w0 + 2 < nwords) ? w[w0 + 2] : 0u;
            if (e0 & 1) {
                lo = __builtin_amdgcn_alignbyte(a1, a0, 2);
                hi = __builtin_amdgcn_alignbyte(a2, a1, 2);
            } else {
                lo = a0;
                hi = a1;
            }
        };
        auto expand = [&](unsigned char *tile, int s) {
            if constexpr (PDENSE) {
                const unsigned char *pb = (const unsigned char *)P.pk_val + (int64_t)s * 128;
#pragma unroll
                for (int i = 0; i < 16; i++)
                    __builtin_amdgcn_global_load_lds((glb_ptr_t)(pb + p_off[i]),
                                                     (lds_ptr_t)(tile + (gw * 16 + i) * 1024), 16, 0, 0);
            } else if constexpr (REDUCE_SPARSE) {
                // all selector reads first (one LDS round trip), then the permutes
                uint32_t sel[2][NBLK][M / 2];
#pragma unroll
                for (int rr = 0; rr < 2; rr++)
#pragma unroll
                    for (int b = 0; b < NBLK; b++) {
                        const uint32_t pat = (rp[rr * RS_PW + (b >> 2)] >> ((b & 3) * 8)) & 0xFFu;
#pragma unroll
                        for (int k = 0; k < M / 2; k++) sel[rr][b][k] = lut[pat * (M / 2) + k];
                    }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int rr = 0; rr < 2; rr++) {
                    uint32_t w[32];   // one dense row of 64 k
#pragma unroll
                    for (int b = 0; b < NBLK; b++) {
                        uint32_t lo, hi;
                        window(&rv[rr * RS_VW], b * N, RS_VW, lo, hi);
#pragma unroll
                        for (int k = 0; k < M / 2; k++)
                            w[b * (M / 2) + k] = __builtin_amdgcn_perm(hi, lo, sel[rr][b][k]);
                    }
#pragma unroll
                    for (int ch = 0; ch < 8; ch++) {
                        u32x4 v = {w[ch * 4], w[ch * 4 + 1], w[ch * 4 + 2], w[ch * 4 + 3]};
                        *(u32x4 *)(tile + dn_sw(gt + rr * 128, ch)) = v;
                    }
                }
            } else {
                const int lg = gt & 7, pg = gt >> 3;
                uint32_t sel[RG_NB][8][M / 2];
#pragma unroll
                for (int b = 0; b < RG_NB; b++)
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const uint32_t pat = (rp[i] >> ((b & 3) * 8)) & 0xFFu;
#pragma unroll
                        for (int k = 0; k < M / 2; k++) sel[b][i][k] = lut[pat * (M / 2) + k];
                    }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int b = 0; b < RG_NB; b++) {
                    uint32_t dense[8][M / 2];   // the block of each of the 8 lines, expanded
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        uint32_t lo, hi;
                        window(&rv[i * RG_VW], b * N, RG_VW, lo, hi);
#pragma unroll
                        for (int k = 0; k < M / 2; k++) dense[i][k] = __builtin_amdgcn_perm(hi, lo, sel[b][i][k]);
                    }
#pragma unroll
                    for (int r = 0; r < M; r++) {
                        // position r of lines i, i+1 -> one word: halves (r&1) of dense[i][r/2], dense[i+1][r/2]
                        const uint32_t ps = (r & 1) ? 0x07060302u : 0x05040100u;
                        u32x4 v;
                        v.x = __builtin_amdgcn_perm(dense[1][r >> 1], dense[0][r >> 1], ps);
                        v.y = __builtin_amdgcn_perm(dense[3][r >> 1], dense[2][r >> 1], ps);
                        v.z = __builtin_amdgcn_perm(dense[5][r >> 1], dense[4][r >> 1], ps);
                        v.w = __builtin_amdgcn_perm(dense[7][r >> 1], dense[6][r >> 1], ps);
                        *(u32x4 *)(tile + dn_sw(pg * 16 + b * M + r, lg)) = v;
                    }
                }
            }
        };
        auto produce = [&](int s) {
            unsigned char *base = smem + (s % DN_NS) * DN_STAGE;
            expand(base, s);
            const unsigned char *xb = x_base + (int64_t)s * 128;
#pragma unroll
            for (int i = 0; i < 8; i++)
                __builtin_amdgcn_global_load_lds((glb_ptr_t)(xb + x_off[i]),
                                                 (lds_ptr_t)(base + DN_P + (gw * 8 + i) * 1024), 16, 0, 0);
            if (s + 2 < KP) load_regs(s + 2);
        };

        // prologue: group 0 builds stages 0 and 2, group 1 stage 1
        if (grp < KP) {
            load_regs(grp);
            produce(grp);
            if (grp == 0 && 2 < KP) produce(2);
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        asm volatile("s_barrier" ::: "memory");
#pragma unroll 1
        for (int kp = 0; kp < KP; kp++) {
            const bool duty = ((kp + 1) & 1) == grp;   // this group built stage kp+1 and builds kp+3
            if (duty) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            asm volatile("s_barrier" ::: "memory");
            if (duty && kp + DN_NS < KP) produce(kp + DN_NS);
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        return;
    }

    // ================================== matrix wavefronts ==================================
    const int wm = wave >> 1, wn = wave & 1;
    f32x16 acc[FA][FB];
#pragma unroll
    for (int i = 0; i < FA; i++)
#pragma unroll
        for (int j = 0; j < FB; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    const int j = lane & 31, h = lane >> 5;
    struct Frags {
        u32x4 a[FA], b[FB];
    };
    Frags f0, f1;
    auto read_frags = [&](Frags &f, const unsigned char *base, int kk) {
#pragma unroll
        for (int i = 0; i < FA; i++) f.a[i] = *(const u32x4 *)(base + dn_sw(wm * 128 + i * 32 + j, kk * 2 + h));
#pragma unroll
        for (int i = 0; i < FB; i++) f.b[i] = *(const u32x4 *)(base + DN_P + dn_sw(wn * 64 + i * 32 + j, kk * 2 + h));
    };
    auto mma = [&](const Frags &f, auto lo_tag, auto hi_tag) {
#pragma unroll
        for (int i = decltype(lo_tag)::value; i < decltype(hi_tag)::value; i++) {
            union {
                u32x4 u;
                typename D::F v;
            } ca;
            ca.u = f.a[i];
#pragma unroll
            for (int t = 0; t < FB; t++) {
                union {
                    u32x4 u;
                    typename D::F v;
                } cb;
                cb.u = f.b[t];
                acc[i][t] = D::run(ca.v, cb.v, acc[i][t]);
            }
        }
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using IFA = std::integral_constant<int, FA>;

    asm volatile("s_barrier" ::: "memory");  // stage 0 is ready
    read_frags(f0, smem, 0);
    for (int kp = 0; kp < KP; kp++) {
        const unsigned char *base = smem + (kp % DN_NS) * DN_STAGE;
        // k sub-steps 0..2: multiply one register set while the other is being fetched
        read_frags(f1, base, 1);
        mma(f0, I0{}, IFA{});
#pragma unroll
        for (int i = 0; i < FA * FB; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < 6) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        read_frags(f0, base, 2);
        mma(f1, I0{}, IFA{});
#pragma unroll
        for (int i = 0; i < FA * FB; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < 6) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        read_frags(f1, base, 3);
        mma(f0, I0{}, IFA{});
#pragma unroll
        for (int i = 0; i < FA * FB; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < 6) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        // last sub-step: two MFMAs, hand the stage back, then fetch the next stage's first set
        mma(f1, I0{}, I1{});
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        read_frags(f0, smem + ((kp + 1) % DN_NS) * DN_STAGE, 0);
        mma(f1, I1{}, IFA{});
#pragma unroll
        for (int i = 0; i < (FA - 1) * FB; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- epilogue: D[row = output][col = token] -> LDS [token][output] -> 16-byte stores ----
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    unsigned char *stg = smem + wave * (64 * DN_OUT_ROW);
#pragma unroll
    for (int tb = 0; tb < FB; tb++)
#pragma unroll
        for (int fb = 0; fb < FA; fb++)
#pragma unroll
            for (int rq = 0; rq < 4; rq++) {
                uint16_t hh[4];
#pragma unroll
                for (int i = 0; i < 4; i++) hh[i] = dn_bits16(acc[fb][tb][rq * 4 + i], (T *)nullptr);
                uint2 pk;
                pk.x = (uint32_t)hh[0] | ((uint32_t)hh[1] << 16);
                pk.y = (uint32_t)hh[2] | ((uint32_t)hh[3] << 16);
                *(uint2 *)(stg + (tb * 32 + j) * DN_OUT_ROW + (fb * 32 + rq * 8 + h * 4) * 2) = pk;
            }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    uint16_t *Y = (uint16_t *)P.y;
    const T *bias = (const T *)P.bias;
    const bool vec_ok = (P.ldy & 7) == 0 && ((uintptr_t)P.y & 15) == 0;
    const int fc = lane & 15;
    const int64_t f = o0 + wm * 128 + fc * 8;
    float bv[8];
#pragma unroll
    for (int i = 0; i < 8; i++) bv[i] = (bias && f + i < P.O) ? to_f32(bias[f + i]) : 0.f;
#pragma unroll 4
    for (int it = 0; it < 16; it++) {
        const int tl = it * 4 + (lane >> 4);
        const int64_t tok = t0 + wn * 64 + tl;
        u32x4 v = *(const u32x4 *)(stg + tl * DN_OUT_ROW + fc * 16);
        if (tok >= P.T || f >= P.O) continue;
        if (bias) {
            uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                uint16_t lo = (uint16_t)(w[i] & 0xFFFF), hi = (uint16_t)(w[i] >> 16);
                T tlo = *reinterpret_cast<T *>(&lo), thi = *reinterpret_cast<T *>(&hi);
                lo = dn_bits16(to_f32(tlo) + bv[2 * i], (T *)nullptr);
                hi = dn_bits16(to_f32(thi) + bv[2 * i + 1], (T *)nullptr);
                w[i] = (uint32_t)lo | ((uint32_t)hi << 16);
            }
            v.x = w[0]; v.y = w[1]; v.z = w[2]; v.w = w[3];
        }
        uint16_t *dst = Y + tok * P.ldy + f;
        if (vec_ok && f + 7 < P.O) {
            *(u32x4 *)dst = v;
        } else {
            uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (f + i < P.O) dst[i] = (uint16_t)(w[i >> 1] >> ((i & 1) * 16));
        }
    }
}

template <typename T, int N, int M> static int launch_dense_nm(DenseParams &P, int reduce_sparse, hipStream_t s)
{
    const size_t lds = (size_t)DN_LUT + (size_t)DN_NS * DN_STAGE;
    static_assert(DN_NS * DN_STAGE >= 4 * 64 * DN_OUT_ROW, "epilogue staging must fit in the ring");
    dim3 grid((unsigned)(P.tiles_m * P.tiles_n));
    if (reduce_sparse) {
        auto k = spmm_dense_pipe_kernel<T, N, M, true>;
        NMG_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL(k, grid, dim3(512), lds, s, P);
    } else {
        auto k = spmm_dense_pipe_kernel<T, N, M, false>;
        NMG_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL(k, grid, dim3(512), lds, s, P);
    }
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

template <typename T> static int launch_dense(DenseParams &P, int reduce_sparse, int n, int m, hipStream_t s)
{
#define NMG_DENSE_CASE(NN, MM) \
    if (n == NN && m == MM) return launch_dense_nm<T, NN, MM>(P, reduce_sparse, s)
    NMG_DENSE_CASE(1, 4);
    NMG_DENSE_CASE(2, 4);
    NMG_DENSE_CASE(3, 4);
    NMG_DENSE_CASE(1, 8);
    NMG_DENSE_CASE(2, 8);
    NMG_DENSE_CASE(4, 8);
#undef NMG_DENSE_CASE
    return NMG_ERR_UNSUPPORTED;
}

// 1 if the pipelined dense kernel has an instantiation for this n:m
bool dense_pipe_supports(int n, int m)
{
    static const int ok[][2] = {{1, 4}, {2, 4}, {3, 4}, {1, 8}, {2, 8}, {4, 8}};
    for (auto &p : ok)
        if (p[0] == n && p[1] == m) return true;
    return false;
}

// Called from nmg_spmm (nmg_spmm.hip) for NMG_KERNEL_MFMA / AUTO when the shape qualifies.
int spmm_dense_pipe(const void *pk_val, const void *pk_pat, const int8_t *d_order, int64_t G, int64_t S,
                    const void *x, int64_t ldx, void *y, int64_t ldy, const void *bias, int64_t T,
                    int reduce_sparse, int n, int m, int dtype, hipStream_t s)
{
    DenseParams P{};
    P.pk_val = pk_val;
    P.pk_pat = pk_pat;
    P.order = d_order;
    P.x = x;
    P.y = y;
    P.bias = bias;
    P.G = G;
    P.S = S;
    P.nb = (S + m - 1) / m;
    P.T = T;
    P.ldx = ldx;
    P.ldy = ldy;
    P.K = reduce_sparse ? S : G;
    P.O = reduce_sparse ? G : S;
    P.c = (int)binom(m, n);
    P.tiles_m = (int)((P.O + 255) / 256);
    P.tiles_n = (int)((T + 127) / 128);
    return dtype == NMG_F16 ? launch_dense<__half>(P, reduce_sparse, n, m, s)
                            : launch_dense<__hip_bfloat16>(P, reduce_sparse, n, m, s);
}

// ------------------------------------------------------------------ rowpack -> dense weight
// Expands the rowpack operand into a plain dense matrix, either as [lines, positions] or
// transposed, through an LDS tile of 64 lines x (up to) 128 positions so that both the reads
// (values in rowpack order) and the writes (whole rows of the tile) are contiguous.
constexpr int EX_L = 64, EX_P = 128;

struct ExpandParams {
    const void *pk_val;
    const void *pk_pat;
    void *out;
    const int8_t *order;
    int64_t G, S, nb, ld;
    int n, m, c, pat_bytes, bpt, transpose;   // c = patterns, bpt = blocks per tile
};

template <typename T> __global__ __launch_bounds__(256) void expand_kernel(ExpandParams P)
{
    // [64][128 + pad] or, transposed, [128][64 + pad]; pad keeps 16-byte rows and spreads banks
    constexpr int PAD = 16 / sizeof(T);
    __shared__ __align__(16) T tile[EX_L * (EX_P + PAD) > EX_P * (EX_L + PAD) ? EX_L * (EX_P + PAD)
                                                                             : EX_P * (EX_L + PAD)];
    const int tid = threadIdx.x;
    const int tp = P.bpt * P.m;                              // positions per tile
    const int64_t q0 = (int64_t)blockIdx.y * EX_L, b0 = (int64_t)blockIdx.x * P.bpt;
    const int rows = P.transpose ? tp : EX_L, cols = P.transpose ? EX_L : tp;
    const int pitch = (P.transpose ? EX_L : EX_P) + PAD;
    {
        const uint4 z = {0, 0, 0, 0};
        for (int i = tid; i < rows * pitch * (int)sizeof(T) / 16; i += 256) ((uint4 *)tile)[i] = z;   // pitch * sizeof(T) % 16 == 0
    }
    // the order table in LDS where it fits: pattern -> order entry -> LDS store is otherwise a round
    // trip to L2 per block
    __shared__ int8_t s_ord[1024];
    const int ord_n = P.c * P.n;
    const bool ord_lds = ord_n <= 1024;
    if (ord_lds)
        for (int i = tid; i < ord_n; i += 256) s_ord[i] = P.order[i];
    const int8_t *order = ord_lds ? s_ord : P.order;
    __syncthreads();
    // One item = one (line, block): its pattern number and its n values, the values as one word where
    // n * sizeof(T) is 4 or 8.  The loads of four items are issued before the first item is placed.
    const T *pv = (const T *)P.pk_val;
    const int bpt = P.bpt, n = P.n, m = P.m;
    const int items = EX_L * bpt;
    // NV > 0: n is the constant NV and the values of a block are one aligned word of 4 or 8 bytes
    auto place = [&](auto nv_tag) {
        constexpr int NV = decltype(nv_tag)::value;
        constexpr int WB = NV * (int)sizeof(T);
        using Word = typename std::conditional<WB == 8, uint2, uint32_t>::type;
        for (int base = tid; base < items; base += 4 * 256) {
            int pat[4];
            Word vw[4];
            int64_t blk[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int it = base + u * 256;
                const int ql = it / bpt, bl = it - ql * bpt;
                const int64_t q = q0 + ql, b = b0 + bl;
                const bool in = it < items && q < P.G && b < P.nb;
                blk[u] = in ? q * P.nb + b : -1;
                const int64_t at = in ? blk[u] : 0;
                pat[u] = P.pat_bytes == 1 ? (int)((const uint8_t *)P.pk_pat)[at] : (int)((const uint16_t *)P.pk_pat)[at];
                if (NV > 0) vw[u] = ((const Word *)pv)[at];
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (blk[u] < 0) continue;
                const int it = base + u * 256;
                const int ql = it / bpt, bl = it - ql * bpt;
                if constexpr (NV > 0) {
                    T w[NV];
                    __builtin_memcpy(w, &vw[u], WB);
#pragma unroll
                    for (int j = 0; j < NV; j++) {
                        const int pos = bl * m + order[pat[u] * NV + j];
                        tile[P.transpose ? pos * pitch + ql : ql * pitch + pos] = w[j];
                    }
                } else {
                    for (int j = 0; j < n; j++) {
                        const int pos = bl * m + order[pat[u] * n + j];
                        tile[P.transpose ? pos * pitch + ql : ql * pitch + pos] = pv[blk[u] * n + j];
                    }
                }
            }
        }
    };
    const int vb = n * (int)sizeof(T);
    const bool aligned = ((uintptr_t)pv % 8) == 0;
    if (aligned && vb == 4 && n == 1) place(std::integral_constant<int, (sizeof(T) == 4 ? 1 : 0)>{});
    else if (aligned && vb == 4 && n == 2) place(std::integral_constant<int, (sizeof(T) == 2 ? 2 : 0)>{});
    else if (aligned && vb == 8 && n == 2) place(std::integral_constant<int, (sizeof(T) == 4 ? 2 : 0)>{});
    else if (aligned && vb == 8 && n == 4) place(std::integral_constant<int, (sizeof(T) == 2 ? 4 : 0)>{});
    else place(std::integral_constant<int, 0>{});
    __syncthreads();
    // rows of the tile -> global, 16 bytes per lane where the row is aligned
    T *out = (T *)P.out;
    const int64_t r0 = P.transpose ? b0 * P.m : q0, c0 = P.transpose ? q0 : b0 * P.m;
    const int64_t R = P.transpose ? P.S : P.G, C = P.transpose ? P.G : P.S;
    constexpr int V = 16 / sizeof(T);
    const bool vec = (P.ld % V) == 0 && (c0 % V) == 0 && ((uintptr_t)P.out % 16) == 0;
    const int cv = (cols + V - 1) / V;
    for (int i = tid; i < rows * cv; i += 256) {
        const int r = i / cv, cc = (i - r * cv) * V;
        if (r0 + r >= R || c0 + cc >= C) continue;
        T *dst = out + (r0 + r) * P.ld + c0 + cc;
        const T *src = tile + r * pitch + cc;
        if (vec && cc + V <= cols && c0 + cc + V <= C) {
            *(uint4 *)dst = *(const uint4 *)src;
        } else {
            for (int e = 0; e < V && cc + e < cols && c0 + cc + e < C; e++) dst[e] = src[e];
        }
    }
}

// -------------------------------------------------------------- single precision, plain NT GEMM
//   Y[T, O] = X[T, K] * A[O, K]^T (+ bias[o]),  all float, V_MFMA_F32_32X32X2_F32
// The single-precision matrix instruction is 16 times slower than the 16-bit ones (64 clocks for a
// 32 x 32 x 2 step), so operand traffic is no problem: 16 reduction positions of a 128 x 128 tile
// keep a wavefront's matrix pipe busy for 2048 clocks and need 16 KiB.  What the kernel has to do
// is keep the instructions back to back, with one wavefront per SIMD:
//   * three stages: while the MFMAs of step s run from registers, the fragments of step s+1 are
//     read from LDS and the tile of step s+2 is on its way from memory; one barrier per step, in
//     the middle of the MFMAs, where all waves arrive together;
//   * LDS holds a tile as [row][k] with a pitch of BKT + 4 floats; lane (j, h) of the instruction
//     reads row j, reduction positions 8h .. 8h+7 with two 128-bit reads (16 lanes x 4 banks, the
//     pitch spreads them over all 64), and MFMA number kk pairs position kk with 8 + kk -- any
//     pairing is right as long as both operands use the same one.
// The 4 wavefronts are WM x WN x WK: WM x WN sub-tiles of (32 MI) x (32 NJ), and WK ways over the
// reduction inside the workgroup (BKT = 16 WK positions per step, partial sums added through LDS
// at the end) for products too small to fill the chip with whole tiles.
struct GemmF32Params {
    const float *a, *x, *bias;
    float *y;
    int64_t lda, ldx, ldy, O, K, T;
    int vec;   // rows are 16-byte aligned: load four reduction positions at a time
};

// FAST: rows 16-byte aligned and K a multiple of BKT -- the loads of a step are one 128-bit load
// per element through pointers computed once (rows past the end are clamped to the last one; their
// results are never stored), nothing else stands between the MFMAs.
// AKM: the weight-side operand is given as A[K, O] (reduction-major: Y = X * A, the dense operand of
// torch.mm as it lies in memory).  Its loads then run along the outputs and the tile is transposed
// on the way into LDS: element e = (k = e % BKT, group of 4 outputs e / BKT), four 32-bit stores;
// 16 reduction positions x 4 groups per wavefront fall on 64 different banks.
// XKM: the same for the activation-side operand, X[K, T] (Y = X^T * A: the weight gradient of a
// linear layer from the upstream gradient and the activations as they lie).
template <int WM, int WN, int WK, int MI, int NJ, bool FAST, bool AKM, bool XKM>
__global__ __launch_bounds__(256) void gemm_nt_f32_kernel(GemmF32Params P)
{
    static_assert(WM * WN * WK == 4, "four wavefronts");
    constexpr int BM = WM * MI * 32, BN = WN * NJ * 32, BKT = 16 * WK, PITCH = BKT + 4;
    constexpr int KV = BKT / 4;                                      // float4 per tile row
    constexpr int XE = BM * KV, AE = BN * KV;                        // float4 per tile
    constexpr int XV = (XE + 255) / 256, AV = (AE + 255) / 256;      // ... per thread
    constexpr int TILE_FLOATS = 2 * (BM + BN) * PITCH;
    constexpr int RED_FLOATS = (WK - 1) * WM * WN * MI * NJ * 16 * 64;
    __shared__ __align__(16) float lds[TILE_FLOATS > RED_FLOATS ? TILE_FLOATS : RED_FLOATS];
    float *const Xs = lds;                                           // [2][BM][PITCH]
    float *const As = lds + 2 * BM * PITCH;                          // [2][BN][PITCH]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wk = wave % WK, wn = (wave / WK) % WN, wm = wave / (WK * WN);
    const int64_t tok0 = (int64_t)blockIdx.y * BM, o0 = (int64_t)blockIdx.x * BN;

    f32x16 acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int q = 0; q < NJ; q++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][q][r] = 0.f;

    // Element e of a tile's load.  Row-major operand: row e / KV, reduction positions 4 (e % KV) .. +3.
    // Reduction-major operand: position e % BKT, rows 4 (e / BKT) .. +3.
    auto fetch_rm = [&](const float *base, int64_t ld, int64_t row, int64_t nrows, int64_t k) {
        f32x4 r = {0.f, 0.f, 0.f, 0.f};
        if (row < nrows) {
            const float *src = base + row * ld + k;
            if (P.vec && k + 3 < P.K) {
                r = *(const f32x4 *)src;
            } else {
                if (k < P.K) r[0] = src[0];
                if (k + 1 < P.K) r[1] = src[1];
                if (k + 2 < P.K) r[2] = src[2];
                if (k + 3 < P.K) r[3] = src[3];
            }
        }
        return r;
    };
    auto fetch_km = [&](const float *base, int64_t ld, int64_t row, int64_t nrows, int64_t k) {
        f32x4 r = {0.f, 0.f, 0.f, 0.f};
        if (k < P.K) {
            const float *src = base + k * ld + row;
            if (row < nrows) r[0] = src[0];
            if (row + 1 < nrows) r[1] = src[1];
            if (row + 2 < nrows) r[2] = src[2];
            if (row + 3 < nrows) r[3] = src[3];
        }
        return r;
    };
    // pointer of the thread's element in the first step (FAST: rows past the end are clamped)
    auto first_ptr = [&](const float *base, int64_t ld, int64_t r0, int64_t nrows, int e, bool km) {
        if (km) {
            const int64_t row = r0 + (e / BKT) * 4 + 3 < nrows ? r0 + (e / BKT) * 4 : (nrows >= 4 ? nrows - 4 : 0);
            return base + (int64_t)(e % BKT) * ld + row;
        }
        const int64_t row = r0 + e / KV < nrows ? r0 + e / KV : nrows - 1;
        return base + row * ld + (e % KV) * 4;
    };
    struct Stage { f32x4 x[XV], a[AV]; };
    const float *xp[XV], *ap[AV];
#pragma unroll
    for (int v = 0; v < XV; v++)
        xp[v] = first_ptr(P.x, P.ldx, tok0, P.T, (XE % 256 == 0 || tid + v * 256 < XE) ? tid + v * 256 : 0, XKM);
#pragma unroll
    for (int v = 0; v < AV; v++)
        ap[v] = first_ptr(P.a, P.lda, o0, P.O, (AE % 256 == 0 || tid + v * 256 < AE) ? tid + v * 256 : 0, AKM);
    // one load / LDS store of a tile: first the activations, then the weight
    constexpr int NG = XV + AV, CSX = XKM ? 4 : 1, CSA = AKM ? 4 : 1, NS = CSX * XV + CSA * AV;
    auto load_op = [&](Stage &G, int64_t k0, int o) {
        if (o < XV) {
            const int e = tid + o * 256;
            if constexpr (FAST) G.x[o] = *(const f32x4 *)(xp[o] + (XKM ? k0 * P.ldx : k0));
            else if (XE % 256 == 0 || e < XE)
                G.x[o] = XKM ? fetch_km(P.x, P.ldx, tok0 + (e / BKT) * 4, P.T, k0 + e % BKT)
                             : fetch_rm(P.x, P.ldx, tok0 + e / KV, P.T, k0 + (e % KV) * 4);
        } else {
            const int v = o - XV, e = tid + v * 256;
            if constexpr (FAST) G.a[v] = *(const f32x4 *)(ap[v] + (AKM ? k0 * P.lda : k0));
            else if (AE % 256 == 0 || e < AE)
                G.a[v] = AKM ? fetch_km(P.a, P.lda, o0 + (e / BKT) * 4, P.O, k0 + e % BKT)
                             : fetch_rm(P.a, P.lda, o0 + e / KV, P.O, k0 + (e % KV) * 4);
        }
    };
    auto store_op = [&](const Stage &G, int buf, int o) {
        if (o < CSX * XV) {
            const int v = o / CSX, c = o % CSX, e = tid + v * 256;
            if (XE % 256 == 0 || e < XE) {
                if constexpr (XKM) Xs[(buf * BM + (e / BKT) * 4 + c) * PITCH + e % BKT] = G.x[v][c];
                else *(f32x4 *)(Xs + (buf * BM + e / KV) * PITCH + (e % KV) * 4) = G.x[v];
            }
        } else {
            const int v = (o - CSX * XV) / CSA, c = (o - CSX * XV) % CSA, e = tid + v * 256;
            if (AE % 256 == 0 || e < AE) {
                if constexpr (AKM) As[(buf * BN + (e / BKT) * 4 + c) * PITCH + e % BKT] = G.a[v][c];
                else *(f32x4 *)(As + (buf * BN + e / KV) * PITCH + (e % KV) * 4) = G.a[v];
            }
        }
    };
    auto load_tile = [&](Stage &G, int64_t k0) {
#pragma unroll
        for (int o = 0; o < NG; o++) load_op(G, k0, o);
    };
    auto store_tile = [&](const Stage &G, int buf) {
#pragma unroll
        for (int o = 0; o < NS; o++) store_op(G, buf, o);
    };

    struct Frags { f32x4 a[MI][2], b[NJ][2]; };
    const int j = lane & 31, h = lane >> 5;
    const int x_off = (wm * MI * 32 + j) * PITCH + wk * 16 + h * 8;
    const int a_off = (wn * NJ * 32 + j) * PITCH + wk * 16 + h * 8;
    // fragment read number o: first the halves that the MFMAs 0 .. 4 MI NJ - 1 of a step use
    constexpr int NR = 2 * (MI + NJ);
    auto read_op = [&](Frags &F, int buf, int o) {
        const int half = o / (MI + NJ), f = o % (MI + NJ);
        if (f < MI) F.a[f][half] = *(const f32x4 *)(Xs + buf * BM * PITCH + x_off + f * 32 * PITCH + half * 4);
        else F.b[f - MI][half] = *(const f32x4 *)(As + buf * BN * PITCH + a_off + (f - MI) * 32 * PITCH + half * 4);
    };
    auto read_frags = [&](Frags &F, int buf) {
#pragma unroll
        for (int o = 0; o < NR; o++) read_op(F, buf, o);
    };
    // X is the A operand of the instruction (rows = tokens), the weight tile the B operand (columns
    // = outputs); MFMA number m of a half step
    constexpr int NH = 4 * MI * NJ;
    auto mma_one = [&](const Frags &F, int half, int m) {
        const int kk = m / (MI * NJ), i = (m / NJ) % MI, q = m % NJ;
        acc[i][q] = __builtin_amdgcn_mfma_f32_32x32x2f32(F.a[i][half][kk], F.b[q][half][kk], acc[i][q], 0, 0, 0);
    };

    const int steps = (int)((P.K + BKT - 1) / BKT);
    Frags F0, F1;
    Stage G0, G1;            // tile t waits in G(t & 1) from step t-3 (its loads) to step t-1 (its LDS stores)
    load_tile(G0, 0);
    store_tile(G0, 0);
    // unconditional (a short reduction loads its last tile again): a branch here would make the
    // compiler's wait counts in the loop assume the worst, a wait for every load in flight
    load_tile(G1, (int64_t)(steps > 1 ? 1 : steps - 1) * BKT);
    load_tile(G0, (int64_t)(steps > 2 ? 2 : steps - 1) * BKT);
    __syncthreads();
    read_frags(F0, 0);
    // step st: `cur` holds the fragments of tile st, `G` tile st+1, the other stage tile st+2.  The
    // accumulators are pinned to the accumulation registers at every step (left alone, the compiler
    // moves all of them to vector registers and back around the loop's branches), and the steps
    // that have a third-next tile run in a loop without branches.
    auto pin = [&]() {
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int q = 0; q < NJ; q++) asm volatile("" : "+a"(acc[i][q]));
    };
    // The memory instructions go out one at a time between the MFMAs (64 clocks each): first half
    // step the LDS stores of tile st+1 and the loads of tile st+3 (two steps, 4096 matrix clocks,
    // ahead of their use), then the barrier, second half step the fragment reads of tile st+1.
    // The fences keep that order; without them the scheduler moves the barrier up to the first
    // MFMA and the next step's LDS stores up to the loads they wait for.
    auto step = [&](int st, const Frags &cur, Frags &nxt, Stage &G, bool more, bool more3) {
        pin();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < NH; m++) {
            mma_one(cur, 0, m);
#pragma unroll
            for (int o = 0; o < NS + NG; o++)
                if (o * NH / (NS + NG) == m) {
                    if (o < NS) { if (more) store_op(G, (st + 1) & 1, o); }   // last read before the barrier of step st-1
                    else if (more3) load_op(G, (int64_t)(st + 3) * BKT, o - NS);
                }
            __builtin_amdgcn_sched_barrier(0);
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < NH; m++) {
            mma_one(cur, 1, m);
#pragma unroll
            for (int o = 0; o < NR; o++)
                if (o * NH / (2 * NR) == m && more) read_op(nxt, (st + 1) & 1, o);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    int st = 0;
    for (; st + 4 < steps; st += 2) {
        step(st, F0, F1, G1, true, true);
        step(st + 1, F1, F0, G0, true, true);
    }
    for (; st < steps; st += 2) {
        step(st, F0, F1, G1, st + 1 < steps, st + 3 < steps);
        if (st + 1 < steps) step(st + 1, F1, F0, G0, st + 2 < steps, st + 4 < steps);
    }
    pin();

    if constexpr (WK > 1) {
        // add the partial sums of the WK wavefronts that share a sub-tile; the tiles in LDS are dead
        // (no wavefront reads them after the barrier of the last step)
        __syncthreads();
        float *red = lds;
        if (wk > 0) {
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int q = 0; q < NJ; q++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        red[((((wk - 1) * WM * WN + wm * WN + wn) * MI * NJ + i * NJ + q) * 16 + r) * 64 + lane] = acc[i][q][r];
        }
        __syncthreads();
        if (wk > 0) return;
#pragma unroll
        for (int w = 0; w < WK - 1; w++)
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int q = 0; q < NJ; q++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        acc[i][q][r] += red[(((w * WM * WN + wm * WN + wn) * MI * NJ + i * NJ + q) * 16 + r) * 64 + lane];
    }

    // D[row = token][col = output]: lane holds output j, tokens 8*(r/4) + 4*h + r%4
#pragma unroll
    for (int q = 0; q < NJ; q++) {
        const int64_t o = o0 + (wn * NJ + q) * 32 + j;
        if (o >= P.O) continue;
        const float bv = P.bias ? P.bias[o] : 0.f;
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t tok = tok0 + (wm * MI + i) * 32 + (r >> 2) * 8 + h * 4 + (r & 3);
                if (tok < P.T) P.y[tok * P.ldy + o] = acc[i][q][r] + bv;
            }
    }
}

template <int WM, int WN, int WK, int MI, int NJ>
static void launch_gemm_f32(const GemmF32Params &Q, int form, hipStream_t st)
{
    // form 0: X[T, K], A[O, K];  1: X[T, K], A[K, O];  2: X[K, T], A[K, O]
    constexpr int BM = WM * MI * 32, BN = WN * NJ * 32, BKT = 16 * WK;
    dim3 grid((unsigned)((Q.O + BN - 1) / BN), (unsigned)((Q.T + BM - 1) / BM));
    const bool fast = Q.vec && Q.K % BKT == 0 && (form < 1 || (Q.O % 4 == 0 && Q.O >= 4)) &&
                      (form < 2 || (Q.T % 4 == 0 && Q.T >= 4));
#define NMG_F32_LAUNCH(FAST_, AKM_, XKM_) \
    hipLaunchKernelGGL((gemm_nt_f32_kernel<WM, WN, WK, MI, NJ, FAST_, AKM_, XKM_>), grid, dim3(256), 0, st, Q)
    if (form == 0) {
        if (fast) NMG_F32_LAUNCH(true, false, false);
        else NMG_F32_LAUNCH(false, false, false);
    } else if (form == 1) {
        if (fast) NMG_F32_LAUNCH(true, true, false);
        else NMG_F32_LAUNCH(false, true, false);
    } else {
        if (fast) NMG_F32_LAUNCH(true, true, true);
        else NMG_F32_LAUNCH(false, true, true);
    }
#undef NMG_F32_LAUNCH
}

// Tile shapes of the single-precision kernel: {tokens, outputs, relative efficiency of a tile}.
// A CU works its tiles off one after the other as far as the matrix pipe is concerned, so a launch
// costs ceil(tiles / 256) x the cost of one tile; the shape with the smallest product wins (768
// outputs x 4096 tokens: 192 tiles of 128 x 128 leave a quarter of the CUs idle, 256 of 128 x 96 none).
struct GemmF32Shape { int bm, bn; double eff; };
static const GemmF32Shape kGemmF32Shapes[] = {
    {128, 128, 1.00}, {128, 96, 0.97}, {128, 64, 0.92}, {64, 64, 0.80}, {32, 32, 0.55},
};

}  // namespace nmg

using namespace nmg;

// single precision: any K and any row pitch; `form` as in launch_gemm_f32
static int gemm_f32_host(const void *d_a, int64_t lda, const void *d_x, int64_t ldx, void *d_y, int64_t ldy,
                         const void *d_bias, int64_t O, int64_t K, int64_t T, int form, void *stream)
{
    if (O == 0 || T == 0) return NMG_OK;
    NMG_REQUIRE(K > 0, NMG_ERR_UNSUPPORTED, "the fp32 GEMM needs K > 0");
    NMG_REQUIRE(d_a && d_x && d_y, NMG_ERR_ARG, "null device pointer");
    GemmF32Params Q{};
    Q.a = (const float *)d_a;
    Q.x = (const float *)d_x;
    Q.bias = (const float *)d_bias;
    Q.y = (float *)d_y;
    Q.lda = lda;
    Q.ldx = ldx;
    Q.ldy = ldy;
    Q.O = O;
    Q.K = K;
    Q.T = T;
    Q.vec = (lda % 4 == 0 && ldx % 4 == 0 && ((uintptr_t)d_a % 16) == 0 && ((uintptr_t)d_x % 16) == 0) ? 1 : 0;
    hipStream_t st = (hipStream_t)stream;
    NMG_REQUIRE((T + 31) / 32 <= 65535, NMG_ERR_UNSUPPORTED, "too many tokens for one launch");
    int best = 0;
    double best_cost = 0;
    for (int c = 0; c < (int)(sizeof(kGemmF32Shapes) / sizeof(kGemmF32Shapes[0])); c++) {
        const GemmF32Shape &S = kGemmF32Shapes[c];
        const int64_t tiles = ((T + S.bm - 1) / S.bm) * ((O + S.bn - 1) / S.bn);
        const double cost = (double)((tiles + 255) / 256) * S.bm * S.bn / S.eff;
        if (c == 0 || cost < best_cost) { best = c; best_cost = cost; }
    }
    switch (best) {
    case 0: launch_gemm_f32<2, 2, 1, 2, 2>(Q, form, st); break;
    case 1: launch_gemm_f32<4, 1, 1, 1, 3>(Q, form, st); break;
    case 2: launch_gemm_f32<2, 2, 1, 2, 1>(Q, form, st); break;
    case 3: launch_gemm_f32<2, 2, 1, 1, 1>(Q, form, st); break;
    default: launch_gemm_f32<1, 1, 4, 1, 1>(Q, form, st); break;
    }
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

extern "C" int nmg_gemm_nn(const void *d_a, int64_t lda, const void *d_x, int64_t ldx, void *d_y, int64_t ldy,
                           const void *d_bias, int64_t O, int64_t K, int64_t T, int dtype, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F32, NMG_ERR_UNSUPPORTED, "gemm_nn takes f32");
    NMG_REQUIRE(O >= 0 && K >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(lda >= O && ldx >= K && ldy >= O, NMG_ERR_ARG, "leading dimension smaller than row length");
    return gemm_f32_host(d_a, lda, d_x, ldx, d_y, ldy, d_bias, O, K, T, 1, stream);
}

extern "C" int nmg_gemm_tn(const void *d_a, int64_t lda, const void *d_x, int64_t ldx, void *d_y, int64_t ldy,
                           const void *d_bias, int64_t O, int64_t K, int64_t T, int dtype, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F32 || dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED, "gemm_tn takes f32/f16/bf16");
    NMG_REQUIRE(O >= 0 && K >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(lda >= O && ldx >= T && ldy >= O, NMG_ERR_ARG, "leading dimension smaller than row length");
    // 16-bit: the kernel of the masked weight gradient without its mask (rows of Y = the operand X)
    if (dtype != NMG_F32) return dense_tn16(d_x, ldx, d_a, lda, K, T, O, d_y, ldy, d_bias, dtype, stream);
    return gemm_f32_host(d_a, lda, d_x, ldx, d_y, ldy, d_bias, O, K, T, 2, stream);
}

extern "C" int nmg_gemm_nt(const void *d_a, int64_t lda, const void *d_x, int64_t ldx, void *d_y,
                           int64_t ldy, const void *d_bias, int64_t O, int64_t K, int64_t T,
                           int dtype, void *stream)
{
    NMG_REQUIRE(dtype == NMG_F32 || dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED,
                "gemm_nt takes f32/f16/bf16");
    NMG_REQUIRE(O >= 0 && K >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(lda >= K && ldx >= K && ldy >= O, NMG_ERR_ARG, "leading dimension smaller than row length");
    if (dtype == NMG_F32)
        return gemm_f32_host(d_a, lda, d_x, ldx, d_y, ldy, d_bias, O, K, T, 0, stream);
    NMG_REQUIRE(K % 64 == 0 && lda % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)d_a % 16) == 0 &&
                    ((uintptr_t)d_x % 16) == 0,
                NMG_ERR_UNSUPPORTED, "gemm_nt needs K % 64 == 0 and 16-byte aligned rows");
    NMG_REQUIRE(O * lda * 2 < ((int64_t)1 << 31) && T * ldx * 2 < ((int64_t)1 << 31), NMG_ERR_UNSUPPORTED,
                "gemm_nt operands must be smaller than 2 GiB");
    if (O == 0 || T == 0) return NMG_OK;
    NMG_REQUIRE(K > 0, NMG_ERR_UNSUPPORTED, "gemm_nt needs K > 0");
    NMG_REQUIRE(d_a && d_x && d_y, NMG_ERR_ARG, "null device pointer");
    DenseParams P{};
    P.pk_val = d_a;
    P.x = d_x;
    P.y = d_y;
    P.bias = d_bias;
    P.nb = lda;
    P.T = T;
    P.ldx = ldx;
    P.ldy = ldy;
    P.K = K;
    P.O = O;
    P.tiles_m = (int)((O + 255) / 256);
    P.tiles_n = (int)((T + 127) / 128);
    hipStream_t s = (hipStream_t)stream;
    return dtype == NMG_F16 ? launch_dense_nm<__half, 0, 4>(P, 1, s)
                            : launch_dense_nm<__hip_bfloat16, 0, 4>(P, 1, s);
}

extern "C" int nmg_rowpack_expand(const void *d_pk_val, const void *d_pk_pat, int64_t G, int64_t S,
                                  void *d_out, int64_t ld_out, int transpose, int n, int m, int dtype,
                                  void *stream)
{
    NMG_REQUIRE(m >= 1 && m <= 64 && n >= 0 && n <= m, NMG_ERR_ARG, "invalid n:m = %d:%d", n, m);
    NMG_REQUIRE(dtype == NMG_F32 || dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED,
                "rowpack supports f32/f16/bf16");
    NMG_REQUIRE(G >= 0 && S >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(ld_out >= (transpose ? G : S), NMG_ERR_ARG, "leading dimension smaller than row length");
    if (G == 0 || S == 0) return NMG_OK;
    NMG_REQUIRE(d_pk_val && d_pk_pat && d_out, NMG_ERR_ARG, "null device pointer");
    ExpandParams P{};
    if (int rc = device_order(n, m, &P.order)) return rc;
    P.pk_val = d_pk_val;
    P.pk_pat = d_pk_pat;
    P.out = d_out;
    P.G = G;
    P.S = S;
    P.nb = (S + m - 1) / m;
    P.ld = ld_out;
    P.n = n;
    P.m = m;
    P.c = (int)binom(m, n);
    P.pat_bytes = binom(m, n) <= 256 ? 1 : 2;
    P.bpt = EX_P / m;
    P.transpose = transpose ? 1 : 0;
    const int64_t gx = (P.nb + P.bpt - 1) / P.bpt, gy = (G + EX_L - 1) / EX_L;
    NMG_REQUIRE(gx <= 0x7fffffffLL && gy <= 65535, NMG_ERR_UNSUPPORTED, "weight too large for one launch");
    dim3 grid((unsigned)gx, (unsigned)gy);
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
    case NMG_F32: hipLaunchKernelGGL(expand_kernel<float>, grid, dim3(256), 0, s, P); break;
    case NMG_F16: hipLaunchKernelGGL(expand_kernel<__half>, grid, dim3(256), 0, s, P); break;
    case NMG_BF16: hipLaunchKernelGGL(expand_kernel<__hip_bfloat16>, grid, dim3(256), 0, s, P); break;
    }
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}
