// The matmul operands of a 2-D weight from its canonical val/idx in one pass: the rowpack operand
// (per line of the group dim and block of the sparse dim: the kept values and the pattern number)
// and, for 16-bit types and 2-of-4 compatible patterns, the fragpack operand of the sparse matrix
// cores.  Same results as nmg_rowpack followed by nmg_fragpack, bit for bit.
//
// val/idx are tile-major (a tile = c*g lines of one chunk of the group dim x one block of the
// sparse dim; its slots are ordered by pattern, and idx names each slot's line), the operands are
// line-major.  A workgroup takes R lines (a multiple of the chunk and of the 32 lines of a
// fragment) x NBW blocks: the tiles it reads are contiguous in val/idx along the blocks, the slots
// are scattered to their lines in LDS, and both operands are written from there in whole
// contiguous runs.  The scatter kernels this replaces wrote n values per thread at a stride of a
// whole line, and gathered every fragment value by value from global memory.
#include "nmg_common.h"

namespace nmg {

struct PackParams {
    const void *val;
    const int16_t *idx;
    void *pk_val;
    void *pk_pat;
    void *fp_val;        // null: rowpack only
    uint32_t *fp_idx;
    int64_t G, S, nb, num_chunks;
    int n, m, g, cols, pat_bytes;
    int R, NBW, PW;      // lines and blocks per workgroup; pitch of a line in LDS, in blocks (odd)
    int KP, MBtot;       // fragpack extents: pairs of 32 positions, blocks of 32 lines
    int m_log2;
    int whole_groups;    // m is 4 or 8 and S % 4 == 0: every group of 4 positions lies in one block
    uint64_t magic_cols, magic_g;   // ceil(2^32 / d): x / d == (x * magic) >> 32 for x < 2^16
    uint32_t masks[32];  // position mask of every pattern, four per word (fragpack: m <= 8)
};

template <typename T, typename PT>
__global__ __launch_bounds__(256) void pack_kernel(PackParams P)
{
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr PT ABSENT = (PT)~(PT)0;
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int n = P.n, cols = P.cols, R = P.R, NBW = P.NBW, PW = P.PW;
    T *s_val = (T *)smem;                                        // [R][PW][n]: an odd pitch spreads the 32 lines of a fragment over the banks
    PT *s_pat = (PT *)(smem + (((size_t)R * PW * n * sizeof(T) + 15) & ~(size_t)15));   // [R][NBW] (rows stay 16-byte aligned where NBW is a multiple of 16)
    uint8_t *s_mask = (uint8_t *)(s_pat + (size_t)R * PW);      // [c] (fragpack only)

    const int64_t r0 = (int64_t)blockIdx.y * R;       // first line
    const int64_t b0 = (int64_t)blockIdx.x * NBW;     // first block
    const int nbw = (int)(P.nb - b0 < NBW ? P.nb - b0 : NBW);   // blocks that exist

    for (int e = tid; e < R * PW; e += nthr) s_pat[e] = ABSENT;
    if (P.fp_val != nullptr) {
        for (int w = 0; w < 32; w++) {
            const uint32_t four = P.masks[w];
            if (tid == 0) ((uint32_t *)(((uintptr_t)s_mask + 3) & ~(uintptr_t)3))[w] = four;
        }
    }
    __syncthreads();

    // ---- tiles -> lines in LDS: consecutive threads read consecutive slots of consecutive tiles
    const T *val = (const T *)P.val;
    for (int kcl = 0; kcl * cols < R; kcl++) {
        const int64_t kc = r0 / cols + kcl;
        if (kc >= P.num_chunks) break;
        const int64_t slot0 = (kc * P.nb + b0) * cols;   // first slot of the chunk's tiles here
        const int cnt = nbw * cols;
        if (n == 2 && sizeof(T) == 2) {
            // the two values of a slot travel as one 32-bit word, four slots per thread in flight
            // (-11 % on the whole kernel against two 16-bit loads and stores per slot; pairs of
            // slots per thread, one 64-bit and one 32-bit load, gained another 2 % at 2:4 and lost
            // as much at 2:8)
            const uint32_t *val2 = (const uint32_t *)P.val;
            uint32_t *s_val2 = (uint32_t *)smem;
            for (int base = tid; base < cnt; base += 4 * nthr) {
                int o[4];
                uint32_t vw[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int e = base + u * nthr;
                    const bool in = e < cnt;
                    o[u] = in ? (int)P.idx[slot0 + e] : -1;
                    vw[u] = val2[slot0 + (in ? e : 0)];
                }
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int e = base + u * nthr;
                    if (o[u] < 0 || kc * cols + o[u] >= P.G) continue;
                    const int bl = (int)(((uint64_t)e * P.magic_cols) >> 32), slot = e - bl * cols;
                    const int at = (kcl * cols + o[u]) * PW + bl;
                    s_pat[(kcl * cols + o[u]) * NBW + bl] = (PT)(((uint64_t)slot * P.magic_g) >> 32);
                    s_val2[at] = vw[u];
                }
            }
        } else if (n <= 4) {
            // four slots per thread are loaded (index and values) before the first is placed:
            // one round trip to HBM per batch instead of one per slot
            for (int base = tid; base < cnt; base += 4 * nthr) {
                int o[4];
                T vv[4][4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int e = base + u * nthr;
                    const bool in = e < cnt;
                    o[u] = in ? (int)P.idx[slot0 + e] : -1;
                    const T *v = val + (slot0 + (in ? e : 0)) * n;
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        if (j < n) vv[u][j] = v[j];
                }
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int e = base + u * nthr;
                    if (o[u] < 0 || kc * cols + o[u] >= P.G) continue;
                    const int bl = (int)(((uint64_t)e * P.magic_cols) >> 32), slot = e - bl * cols;
                    const int at = (kcl * cols + o[u]) * PW + bl;
                    s_pat[(kcl * cols + o[u]) * NBW + bl] = (PT)(((uint64_t)slot * P.magic_g) >> 32);
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        if (j < n) s_val[at * n + j] = vv[u][j];
                }
            }
        } else {
            for (int e = tid; e < cnt; e += nthr) {
                const int bl = (int)(((uint64_t)e * P.magic_cols) >> 32), slot = e - bl * cols;
                const int o = P.idx[slot0 + e];
                if (o < 0 || kc * cols + o >= P.G) continue;
                const int at = (kcl * cols + o) * PW + bl;
                s_pat[(kcl * cols + o) * NBW + bl] = (PT)(((uint64_t)slot * P.magic_g) >> 32);
                const T *v = val + (slot0 + e) * n;
                for (int j = 0; j < n; j++) s_val[at * n + j] = v[j];
            }
        }
    }
    __syncthreads();

    // ---- rowpack: the runs of the lines go out as one flat list of pieces -- 16 bytes where the
    //      ends of a run are aligned (four 32-bit LDS reads each: the odd pitch keeps the rows
    //      word-aligned only), else 4 bytes, else single elements -- so that every lane has a piece
    //      (a wavefront per line wrote 2 bytes per lane, and 12 lanes of 64 where a run is 24 bytes)
    auto write_runs = [&](unsigned char *dst, int64_t row_b, const unsigned char *src, int pitch_b, int run_b,
                          int unit_b, bool rows16) {
        // largest piece that divides the run, the rows' distance and both starts
        const uintptr_t mis = (uintptr_t)dst | (uintptr_t)row_b | (uintptr_t)run_b;
        const int piece = (mis % 16 == 0 && pitch_b % 4 == 0 && rows16) ? 16 : (mis % 4 == 0 && pitch_b % 4 == 0) ? 4 : unit_b;
        const int ppl = run_b / piece;   // pieces per line
        const uint64_t magic = (((uint64_t)1 << 32) + ppl - 1) / (ppl > 0 ? ppl : 1);
        const int total = R * ppl;       // < 2^22 (the tile fits LDS): the magic division is exact
        if (piece == 16) {
            for (int i = tid; i < total; i += nthr) {
                const int r = (int)(((uint64_t)i * magic) >> 32), ch = i - r * ppl;
                if (r0 + r >= P.G) continue;
                const uint32_t *w = (const uint32_t *)(src + (size_t)r * pitch_b + (size_t)ch * 16);
                *(uint4 *)(dst + (r0 + r) * row_b + (size_t)ch * 16) = make_uint4(w[0], w[1], w[2], w[3]);
            }
        } else if (piece == 4) {
            for (int i = tid; i < total; i += nthr) {
                const int r = (int)(((uint64_t)i * magic) >> 32), ch = i - r * ppl;
                if (r0 + r >= P.G) continue;
                *(uint32_t *)(dst + (r0 + r) * row_b + (size_t)ch * 4) = *(const uint32_t *)(src + (size_t)r * pitch_b + (size_t)ch * 4);
            }
        } else {
            for (int i = tid; i < total; i += nthr) {
                const int r = (int)(((uint64_t)i * magic) >> 32), ch = i - r * ppl;
                if (r0 + r >= P.G) continue;
                unsigned char *d = dst + (r0 + r) * row_b + (size_t)ch * piece;
                const unsigned char *sp = src + (size_t)r * pitch_b + (size_t)ch * piece;
                if (piece == 2) *(uint16_t *)d = *(const uint16_t *)sp;
                else if (piece == 1) *d = *sp;
                else for (int e = 0; e < piece; e++) d[e] = sp[e];
            }
        }
    };
    write_runs((unsigned char *)P.pk_val + b0 * n * sizeof(T), (int64_t)P.nb * n * (int64_t)sizeof(T),
               (const unsigned char *)s_val, PW * n * (int)sizeof(T), nbw * n * (int)sizeof(T), (int)sizeof(T), true);
    write_runs((unsigned char *)P.pk_pat + b0 * sizeof(PT), (int64_t)P.nb * (int64_t)sizeof(PT),
               (const unsigned char *)s_pat, NBW * (int)sizeof(PT), nbw * (int)sizeof(PT), (int)sizeof(PT),
               (NBW * sizeof(PT)) % 16 == 0);
    if (P.fp_val == nullptr) return;

    // ---- fragpack: one wavefront per (32 lines, 64 positions); a lane emits its 2 x 8 values and
    //      one index word in the register order of V_SMFMAC_F32_32X32X32
    const uint8_t *mask = (const uint8_t *)(((uintptr_t)s_mask + 3) & ~(uintptr_t)3);
    const int lane = tid & 63, wave = tid >> 6, waves = nthr >> 6;
    const int RM = R / 32, KPW = (NBW << P.m_log2) / 64;
    const int row_in = lane & 31, ga = lane >> 5;
    const int m = P.m;
    for (int job = wave; job < RM * KPW; job += waves) {
        const int mbl = job / KPW, kpl = job - mbl * KPW;
        const int64_t mbg = r0 / 32 + mbl, kpg = ((b0 << P.m_log2) >> 6) + kpl;
        if (mbg >= P.MBtot || kpg >= P.KP) continue;
        const int r = mbl * 32 + row_in;
        // The lane probes 2 x 4 groups of 4 positions.  Per half, all patterns are read first,
        // then all masks, then all candidate values, so the LDS round trips are three and not one
        // chain per position.
        uint32_t idxword = 0;
        if (P.whole_groups) {
            // m = 4 or 8 and no partial group of 4 at the end of the sparse dim: a group of 4
            // positions lies in one block, so it takes one pattern, one mask and its (at most two)
            // kept values, which sit side by side in the block's value list
            for (int ks = 0; ks < 2; ks++) {
                PT pt[4];
                int mkb[4], blk[4], base[4];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int k0 = (kpl * 2 + ks) * 32 + (4 * (q >> 1) + 2 * ga + (q & 1)) * 4;
                    const bool in = (b0 << P.m_log2) + k0 < P.S;
                    blk[q] = in ? k0 >> P.m_log2 : 0;
                    base[q] = k0 & (m - 1);
                    pt[q] = in ? s_pat[r * NBW + blk[q]] : ABSENT;
                }
#pragma unroll
                for (int q = 0; q < 4; q++) mkb[q] = pt[q] == ABSENT ? 0 : (int)mask[pt[q]];
                uint16_t c0[4], c1[4];
                if (m == 4 && n == 2) {
                    // a block is a group: its two values are one word
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const uint32_t w = ((const uint32_t *)s_val)[r * PW + blk[q]];
                        c0[q] = (uint16_t)(w & 0xFFFFu);
                        c1[q] = (uint16_t)(w >> 16);
                    }
                } else
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int j0 = __popc(mkb[q] & ((1 << base[q]) - 1));
                    const T *bv = s_val + ((size_t)r * PW + blk[q]) * n;
                    const T x0 = bv[j0 < n ? j0 : 0], x1 = bv[j0 + 1 < n ? j0 + 1 : 0];
                    c0[q] = *reinterpret_cast<const uint16_t *>(&x0);
                    c1[q] = *reinterpret_cast<const uint16_t *>(&x1);
                }
                uint16_t vals[8];
                uint32_t half = 0;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int gm = (mkb[q] >> base[q]) & 0xF;
                    const int cnt = __popc(gm);
                    int p0 = 0, p1 = 1;
                    uint16_t v0 = 0, v1 = 0;
                    if (cnt >= 2) {
                        p0 = __ffs(gm) - 1;
                        p1 = __ffs(gm & (gm - 1)) - 1;
                        v0 = c0[q];
                        v1 = c1[q];
                    } else if (cnt == 1) {
                        // add a zero at an unused position, keeping positions increasing
                        const int pp = __ffs(gm) - 1;
                        if (pp == 3) {
                            p0 = 0;
                            p1 = 3;
                            v1 = c0[q];
                        } else {
                            p0 = pp;
                            p1 = 3;
                            v0 = c0[q];
                        }
                    }
                    vals[2 * q] = v0;
                    vals[2 * q + 1] = v1;
                    half |= (uint32_t)(p0 | (p1 << 2)) << (4 * q);
                }
                idxword |= half << (16 * ks);
                uint4 out;
                out.x = vals[0] | ((uint32_t)vals[1] << 16);
                out.y = vals[2] | ((uint32_t)vals[3] << 16);
                out.z = vals[4] | ((uint32_t)vals[5] << 16);
                out.w = vals[6] | ((uint32_t)vals[7] << 16);
                *(uint4 *)((uint16_t *)P.fp_val + ((mbg * (P.KP * 2) + kpg * 2 + ks) * 64 + lane) * 8) = out;
            }
            P.fp_idx[(mbg * P.KP + kpg) * 64 + lane] = idxword;
            continue;
        }
        for (int ks = 0; ks < 2; ks++) {
            PT pat[16];
            int mk[16];
            uint16_t cand[16];
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int q = e >> 2, i = e & 3;
                const int k = (kpl * 2 + ks) * 32 + (4 * (q >> 1) + 2 * ga + (q & 1)) * 4 + i;   // from the first block
                // beyond S the probe reads its line's first block; it is ignored below
                pat[e] = s_pat[r * NBW + ((b0 << P.m_log2) + k < P.S ? k >> P.m_log2 : 0)];
            }
#pragma unroll
            for (int e = 0; e < 16; e++) mk[e] = pat[e] == ABSENT ? 0 : (int)mask[pat[e]];
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int q = e >> 2, i = e & 3;
                const int k = (kpl * 2 + ks) * 32 + (4 * (q >> 1) + 2 * ga + (q & 1)) * 4 + i;
                const int j = __popc(mk[e] & ((1 << (k & (m - 1))) - 1));
                const T x = s_val[((size_t)r * PW + ((b0 << P.m_log2) + k < P.S ? k >> P.m_log2 : 0)) * n + (j < n ? j : 0)];
                cand[e] = *reinterpret_cast<const uint16_t *>(&x);
            }
            uint16_t vals[8];
            uint32_t half = 0;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                int pos[2] = {0, 1};
                uint16_t v[2] = {0, 0};
                int cnt = 0;
                bool alive = true;   // a position beyond S, or a line beyond G, ends the group
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int e = q * 4 + i;
                    const int k = (kpl * 2 + ks) * 32 + (4 * (q >> 1) + 2 * ga + (q & 1)) * 4 + i;
                    alive = alive && (b0 << P.m_log2) + k < P.S && pat[e] != ABSENT;
                    if (alive && cnt < 2 && ((mk[e] >> (k & (m - 1))) & 1)) {
                        pos[cnt] = i;
                        v[cnt] = cand[e];
                        cnt++;
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
            uint4 out;
            out.x = vals[0] | ((uint32_t)vals[1] << 16);
            out.y = vals[2] | ((uint32_t)vals[3] << 16);
            out.z = vals[4] | ((uint32_t)vals[5] << 16);
            out.w = vals[6] | ((uint32_t)vals[7] << 16);
            *(uint4 *)((uint16_t *)P.fp_val + ((mbg * (P.KP * 2) + kpg * 2 + ks) * 64 + lane) * 8) = out;
        }
        P.fp_idx[(mbg * P.KP + kpg) * 64 + lane] = idxword;
    }
}

static int64_t gcd64(int64_t a, int64_t b)
{
    while (b) {
        const int64_t t = a % b;
        a = b;
        b = t;
    }
    return a;
}

}  // namespace nmg

using namespace nmg;

extern "C" int nmg_pack_operands(const void *d_val, const int16_t *d_idx, int64_t G, int64_t S,
                                 void *d_pk_val, void *d_pk_pat, void *d_fp_val, void *d_fp_idx,
                                 int n, int m, int g, int dtype, void *stream)
{
    NMG_REQUIRE(m >= 1 && m <= 64 && n >= 0 && n <= m && g >= 1, NMG_ERR_ARG, "invalid n:m:g = %d:%d:%d", n, m, g);
    NMG_REQUIRE(dtype == NMG_F32 || dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_UNSUPPORTED,
                "the matmul operands support f32/f16/bf16");
    NMG_REQUIRE(G >= 0 && S >= 0, NMG_ERR_ARG, "negative extent");
    const bool frag = d_fp_val != nullptr;
    NMG_REQUIRE(!frag || d_fp_idx != nullptr, NMG_ERR_ARG, "fragpack values without index words");
    NMG_REQUIRE(!frag || (dtype != NMG_F32 && nmg_fragpack_supported(n, m)), NMG_ERR_UNSUPPORTED,
                "no sparse-matrix-core operand for %d:%d of this type", n, m);
    if (G == 0 || S == 0) return NMG_OK;
    NMG_REQUIRE(d_val && d_idx && d_pk_val && d_pk_pat, NMG_ERR_ARG, "null device pointer");
    nmg_view v{1, G, S, 0, S, 1};
    const TileGeom tg = tile_geom(v, n, m, g);
    NMG_REQUIRE((int64_t)tg.c * g < 32768, NMG_ERR_ARG, "chunk_size * group_size = %lld must be < 2^15",
                (long long)((int64_t)tg.c * g));
    hipStream_t s = (hipStream_t)stream;

    // The one-pass kernel needs the tile to fit LDS (and, for the fragments, m in 1, 2, 4, 8 and at
    // most 128 patterns); what it does not take goes through the two scatter kernels.
    const int elem = (int)dtype_size(dtype);
    const int pat_bytes = (int)nmg_rowpack_pat_bytes(n, m);
    const bool pow2 = (m & (m - 1)) == 0;
    const int64_t R64 = (int64_t)tg.cols / gcd64(tg.cols, 32) * 32;   // lcm(cols, 32)
    const int nbw_unit = frag ? (64 / m > 0 ? 64 / m : 1) : 1;   // blocks per 64 positions
    const int64_t per_block = R64 * ((int64_t)n * elem + pat_bytes);
    // about 24 KiB of LDS per workgroup (many small workgroups hide each other's latencies: 55 us
    // against 83 us with 48 KiB on a 4096 x 4096 2:4:16 weight), but at least three blocks per line
    // where a line's run would otherwise be a few bytes
    int64_t NBW = per_block > 0 ? (24 * 1024) / per_block : 0;
    if (NBW < 3 && per_block > 0) NBW = (64 * 1024) / per_block < 3 ? (64 * 1024) / per_block : 3;
    NBW = NBW / nbw_unit * nbw_unit;
    if (NBW < nbw_unit) NBW = nbw_unit;
    if (NBW > 256) NBW = 256 / nbw_unit * nbw_unit;
    // Pitch of a line in LDS: odd, so that the 32 lines a fragment reads side by side fall on
    // different banks (-10 % on 2:4:16: 6 workgroups of 23.7 KB per CU instead of 7 of 23.2), but
    // only where six padded workgroups still fit a CU: at 2:8:32 the padding takes the CU from
    // four workgroups of 36 KB to three (+3 %).
    auto lds_for = [&](int64_t pw) {
        return (((size_t)R64 * pw * n * elem + 15) & ~(size_t)15) + (size_t)R64 * pw * pat_bytes + 160;
    };
    const int64_t PW = lds_for(NBW | 1) * 6 <= 156 * 1024 ? (NBW | 1) : NBW;
    const size_t lds = lds_for(PW);
    const bool one_pass = n >= 1 && lds <= 96 * 1024 && (int64_t)NBW * tg.cols < 65536 && R64 * NBW * (int64_t)(n > 1 ? n : 1) < ((int64_t)1 << 30) &&
                          (!frag || (pow2 && m <= 8 && tg.c <= 128));
    if (!one_pass) {
        if (int rc = nmg_rowpack(d_val, d_idx, G, S, d_pk_val, d_pk_pat, n, m, g, dtype, stream)) return rc;
        if (frag) return nmg_fragpack(d_pk_val, d_pk_pat, G, S, d_fp_val, d_fp_idx, n, m, dtype, stream);
        return NMG_OK;
    }

    PackParams P{};
    P.val = d_val;
    P.idx = d_idx;
    P.pk_val = d_pk_val;
    P.pk_pat = d_pk_pat;
    P.fp_val = d_fp_val;
    P.fp_idx = (uint32_t *)d_fp_idx;
    P.G = G;
    P.S = S;
    P.nb = tg.num_blocks;
    P.num_chunks = tg.num_chunks;
    P.n = n;
    P.m = m;
    P.g = g;
    P.cols = tg.cols;
    P.pat_bytes = pat_bytes;
    P.R = (int)R64;
    P.NBW = (int)NBW;
    P.PW = (int)PW;
    P.KP = (int)((S + 63) / 64);
    P.MBtot = (int)((G + 255) / 256 * 8);
    P.m_log2 = 0;
    while ((1 << P.m_log2) < m) P.m_log2++;
    P.whole_groups = (m == 4 || m == 8) && S % 4 == 0 ? 1 : 0;
    P.magic_cols = (((uint64_t)1 << 32) + tg.cols - 1) / tg.cols;
    P.magic_g = (((uint64_t)1 << 32) + g - 1) / g;
    if (frag) {
        const int8_t *order = host_order(n, m);
        NMG_REQUIRE(order != nullptr, NMG_ERR_ARG, "invalid n:m = %d:%d", n, m);
        for (int p = 0; p < tg.c; p++)
            for (int j = 0; j < n; j++) P.masks[p / 4] |= 1u << (8 * (p % 4) + order[p * n + j]);
    }
    // lines: the chunks' padded extent, and for the fragments the 256-line padding of the operand
    int64_t lines = tg.num_chunks * tg.cols;
    if (frag && (int64_t)P.MBtot * 32 > lines) lines = (int64_t)P.MBtot * 32;
    const int64_t gy = (lines + R64 - 1) / R64, gx = (tg.num_blocks + NBW - 1) / NBW;
    NMG_REQUIRE(gy <= 65535 && gx <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "weight too large for the pack kernel");
    dim3 grid((unsigned)gx, (unsigned)gy);
#define NMG_PACK_LAUNCH(T, PT)                                                                        \
    do {                                                                                              \
        auto kern = pack_kernel<T, PT>;                                                               \
        if (lds > 64 * 1024)                                                                          \
            NMG_HIP_TRY(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, P);                                         \
    } while (0)
    if (dtype == NMG_F32) {
        if (pat_bytes == 1) NMG_PACK_LAUNCH(float, uint8_t); else NMG_PACK_LAUNCH(float, uint16_t);
    } else if (dtype == NMG_F16) {
        if (pat_bytes == 1) NMG_PACK_LAUNCH(__half, uint8_t); else NMG_PACK_LAUNCH(__half, uint16_t);
    } else {
        if (pat_bytes == 1) NMG_PACK_LAUNCH(__hip_bfloat16, uint8_t); else NMG_PACK_LAUNCH(__hip_bfloat16, uint16_t);
    }
#undef NMG_PACK_LAUNCH
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}
