// Dense -> grouped n:m compressor (bit-exact with the reference CPU sparsifier), plus the
// element-wise companions: to_dense scatter, same-pattern gather and the rowpack re-ordering.
//
// Reference algorithm (grouped_nm_tensor.py:255-297), per tile of c*g columns x m values:
//   score[o][p] = sum_j |d[o][order[p][j]]|  (left to right, in the input precision)
//   sort all (score, o, p) descending (ties: larger o, then larger p)
//   walk the sorted list; accept (o, p) if column o is free and pattern p has < g members;
//   the k-th column accepted by pattern p lands in slot p*g + k.
//
// GPU formulation (same result, no global sort): the sorted walk always accepts next the
// largest key among {(o, p): o free, p not full}.  Every free column keeps its "head" = its best
// key over the patterns that still have room; one step = arg-max of the heads over the free
// columns, accept it, and if that filled the pattern, recompute the heads that pointed to it.
// A step is a wavefront (or workgroup) max-reduction; a tile needs c*g steps.  The kernels
// further down batch these steps: the lane teams run many small tiles per wavefront, and the
// rounds accept in one pass everything the walk accepts before the next pattern fills.
//
// Work split: a "team" of TW wavefronts owns one tile; a workgroup holds NT teams that work on
// NT consecutive tiles, which are adjacent in memory along the sparse dim when that dim is the
// contiguous one, so the cooperative tile load is coalesced across them.
#include "nmg_common.h"

#include <algorithm>

namespace nmg {

template <typename T> struct ScoreOf { using type = float; using bits = uint32_t; };
template <> struct ScoreOf<double> { using type = double; using bits = uint64_t; };

__device__ __forceinline__ uint32_t score_bits(float s) { return __float_as_uint(s); }
__device__ __forceinline__ uint64_t score_bits(double s) { return (uint64_t)__double_as_longlong(s); }

__device__ __forceinline__ float score_of(float x) { return fabsf(x); }
__device__ __forceinline__ double score_of(double x) { return fabs(x); }
__device__ __forceinline__ float score_of(__half x) { return fabsf(__half2float(x)); }
__device__ __forceinline__ float score_of(__hip_bfloat16 x) { return fabsf(__bfloat162float(x)); }

// Key = (score bits, (o << 16 | p) + 1); the all-zero key means "nothing".
template <typename SB> struct Key {
    SB s;
    uint32_t op;
};
template <typename SB> __device__ __forceinline__ bool key_gt(const Key<SB> &a, const Key<SB> &b)
{
    return a.s > b.s || (a.s == b.s && a.op > b.op);
}

__device__ __forceinline__ uint32_t shfl_xor_bits(uint32_t v, int mask)
{
    return (uint32_t)__shfl_xor((int)v, mask, 64);
}
__device__ __forceinline__ uint64_t shfl_xor_bits(uint64_t v, int mask)
{
    uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)v, mask, 64);
    uint32_t hi = (uint32_t)__shfl_xor((int)(uint32_t)(v >> 32), mask, 64);
    return ((uint64_t)hi << 32) | lo;
}

template <typename SB> __device__ __forceinline__ Key<SB> wave_max(Key<SB> k)
{
#pragma unroll
    for (int mask = 32; mask >= 1; mask >>= 1) {
        Key<SB> o;
        o.s = shfl_xor_bits(k.s, mask);
        o.op = shfl_xor_bits(k.op, mask);
        if (key_gt(o, k)) k = o;
    }
    return k;
}

struct SparsifyParams {
    const void *dense;
    void *val;
    int16_t *idx;
    const int8_t *order;  // device table [c][n]
    ViewDev view;
    int64_t outer;
    int n, m, g, c, cols;
    int team_bytes;  // LDS bytes of one team's region
    int off_hs, off_hp, off_cnt, off_oval, off_oidx, off_wbest;  // offsets inside a team region
};

template <int TW> __device__ __forceinline__ void team_sync()
{
    if (TW == 1) {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    } else {
        __syncthreads();
    }
}

template <typename T, int TW, int NT>
__global__ __launch_bounds__(64 * TW * NT) void sparsify_kernel(SparsifyParams P)
{
    using CT = typename ScoreOf<T>::type;
    using SB = typename ScoreOf<T>::bits;
    constexpr int TS = 64 * TW;  // threads per team
    extern __shared__ __align__(16) unsigned char smem[];

    const int n = P.n, m = P.m, g = P.g, c = P.c, cols = P.cols;
    const int tid = threadIdx.x;
    const int team = tid / TS, tt = tid % TS;
    const int wave_in_team = tt / 64;

    // LDS: [order table][team 0 region][team 1 region]...
    int8_t *s_order = (int8_t *)smem;
    const int order_bytes = (c * n + 15) & ~15;
    unsigned char *region = smem + order_bytes + (size_t)team * P.team_bytes;
    T *s_d = (T *)region;
    SB *s_hs = (SB *)(region + P.off_hs);
    uint16_t *s_hp = (uint16_t *)(region + P.off_hp);
    int16_t *s_cnt = (int16_t *)(region + P.off_cnt);
    T *s_oval = (T *)(region + P.off_oval);
    int16_t *s_oidx = (int16_t *)(region + P.off_oidx);
    Key<SB> *s_wbest = (Key<SB> *)(region + P.off_wbest);

    for (int i = tid; i < c * n; i += 64 * TW * NT) s_order[i] = P.order[i];

    // ---- cooperative load of the NT tiles of this workgroup (zero beyond G / S) ----
    const int64_t tile0 = (int64_t)blockIdx.x * NT;
    const T *dense = (const T *)P.dense;
    const int per_tile = cols * m;
    for (int e = tid; e < NT * per_tile; e += 64 * TW * NT) {
        int r = e % m;
        int rest = e / m;
        int tm = rest % NT;
        int o = rest / NT;
        int64_t t = tile0 + tm;
        T v = Zero<T>::v();
        if (t < P.outer) {
            int64_t tiles_per_b = P.view.num_chunks * P.view.num_blocks;
            int64_t b = t / tiles_per_b;
            int64_t rem = t - b * tiles_per_b;
            int64_t kc = rem / P.view.num_blocks;
            int64_t mb = rem - kc * P.view.num_blocks;
            int64_t gi = kc * cols + o, si = mb * m + r;
            if (gi < P.view.G && si < P.view.S)
                v = dense[b * P.view.stride_b + gi * P.view.stride_g + si * P.view.stride_s];
        }
        T *dst = (T *)(smem + order_bytes + (size_t)tm * P.team_bytes);
        dst[o * m + r] = v;
    }
    for (int p = tt; p < c; p += TS) s_cnt[p] = 0;
    __syncthreads();

    // Best key of column o over the patterns that still have room (skip_p = pattern that just
    // filled up and whose counter may not be visible yet).
    auto head_of = [&](int o, int skip_p, SB &best_s, int &best_p) {
        best_p = -1;
        best_s = 0;
        const T *col = s_d + o * m;
        for (int p = 0; p < c; p++) {
            if (p == skip_p || s_cnt[p] >= g) continue;
            CT acc = 0;
            for (int j = 0; j < n; j++) acc += score_of(col[s_order[p * n + j]]);
            SB sb = score_bits(acc);
            if (best_p < 0 || sb >= best_s) {  // ties: larger p wins
                best_s = sb;
                best_p = p;
            }
        }
    };
    auto local_best = [&]() {
        Key<SB> lb;
        lb.s = 0;
        lb.op = 0;
        for (int o = tt; o < cols; o += TS) {
            uint16_t hp = s_hp[o];
            if (hp == 0xFFFF) continue;
            Key<SB> k;
            k.s = s_hs[o];
            k.op = (((uint32_t)o << 16) | hp) + 1u;
            if (key_gt(k, lb)) lb = k;
        }
        return lb;
    };

    for (int o = tt; o < cols; o += TS) {
        SB bs;
        int bp;
        head_of(o, -1, bs, bp);
        s_hs[o] = bs;
        s_hp[o] = (uint16_t)bp;
    }
    Key<SB> lb = local_best();

    for (int step = 0; step < cols; step++) {
        Key<SB> b = wave_max(lb);
        if (TW > 1) {
            if ((tt & 63) == 0) s_wbest[wave_in_team] = b;
            __syncthreads();
            b = s_wbest[0];
#pragma unroll
            for (int w = 1; w < TW; w++) {
                Key<SB> o = s_wbest[w];
                if (key_gt(o, b)) b = o;
            }
        }
        const uint32_t op = b.op - 1u;
        const int o_star = (int)(op >> 16), p_star = (int)(op & 0xFFFFu);
        const int oldcnt = s_cnt[p_star];
        team_sync<TW>();
        bool dirty = false;
        if (o_star % TS == tt) {
            const int slot = p_star * g + oldcnt;
            s_cnt[p_star] = (int16_t)(oldcnt + 1);
            s_hp[o_star] = 0xFFFF;
            s_oidx[slot] = (int16_t)o_star;
            for (int j = 0; j < n; j++) s_oval[slot * n + j] = s_d[o_star * m + s_order[p_star * n + j]];
            dirty = true;
        }
        if (oldcnt + 1 == g) {
            for (int o = tt; o < cols; o += TS) {
                if (s_hp[o] != (uint16_t)p_star) continue;
                SB bs;
                int bp;
                head_of(o, p_star, bs, bp);
                s_hs[o] = bs;
                s_hp[o] = (uint16_t)bp;
                dirty = true;
            }
        }
        if (dirty) lb = local_best();
        team_sync<TW>();
    }

    // ---- coalesced store of the team's tile ----
    __syncthreads();
    const int64_t t = tile0 + team;
    if (t < P.outer) {
        T *val = (T *)P.val + t * (int64_t)cols * n;
        int16_t *idx = P.idx + t * (int64_t)cols;
        for (int i = tt; i < cols * n; i += TS) val[i] = s_oval[i];
        for (int i = tt; i < cols; i += TS) idx[i] = s_oidx[i];
    }
}

static inline int align_up(int x, int a) { return (x + a - 1) / a * a; }

template <typename T, int TW, int NT>
static int launch_sparsify(SparsifyParams &P, hipStream_t stream)
{
    using SB = typename ScoreOf<T>::bits;
    const int cols = P.cols, n = P.n, m = P.m, c = P.c;
    int off = align_up(cols * m * (int)sizeof(T), 16);
    P.off_hs = off;
    off = align_up(off + cols * (int)sizeof(SB), 16);
    P.off_hp = off;
    off = align_up(off + cols * 2, 16);
    P.off_cnt = off;
    off = align_up(off + c * 2, 16);
    P.off_oval = off;
    off = align_up(off + cols * (n > 0 ? n : 1) * (int)sizeof(T), 16);
    P.off_oidx = off;
    off = align_up(off + cols * 2, 16);
    P.off_wbest = off;
    off = align_up(off + TW * (int)sizeof(Key<SB>), 16);
    P.team_bytes = off;
    const size_t lds = (size_t)align_up(c * n, 16) + (size_t)NT * P.team_bytes;
    NMG_REQUIRE(lds <= 160 * 1024, NMG_ERR_UNSUPPORTED,
                "sparsify tile (c*g=%d columns, m=%d) needs %zu bytes of LDS, limit 163840", cols,
                m, lds);
    auto kern = sparsify_kernel<T, TW, NT>;
    if (lds > 64 * 1024)
        NMG_HIP_TRY(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)lds));
    const int64_t grid = (P.outer + NT - 1) / NT;
    NMG_REQUIRE(grid <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "too many tiles (%lld)", (long long)grid);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(64 * TW * NT), lds, stream, P);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

// ------------------------------------------------------------- small tiles: lane teams
// For tiles of a few hundred columns a wavefront-wide arg-max per step wastes most of the
// machine on communication.  Here a tile belongs to a *team* of L consecutive lanes (16 tiles
// per wavefront for L = 4); lane j of the team owns the columns o = j (mod L) and keeps the best
// of them in registers, so a step is a short scan of the owner's own columns plus log2(L)
// exchanges inside the team.
//
// Heads are maintained lazily: when a pattern fills up, the heads that point to it are left
// stale.  A stale head is an upper bound of the column's true key (the true head is the best over
// a subset of the patterns), so the largest head over the free columns is either valid -- then it
// is the true maximum and is accepted -- or stale, and then only that one column is recomputed
// over the patterns that still have room and the step is repeated.  Every iteration of a team
// is therefore one "pop": accept or repair, followed by the owner's rescan.
//
// LDS per team: the tile's data, head score (+1, 0 = column taken), head pattern, pattern
// counters and the idx output; a team region is padded to L (mod 64) words so that the teams of
// a wavefront, which all touch the same offsets of their regions, hit distinct banks.
// Exchange inside a team of L consecutive lanes without going through LDS: DPP lane
// permutations.  After the stages for L the value has been combined over the whole team:
// quad_perm [1,0,3,2] and [2,3,0,1] reduce a quad, row_half_mirror (i <-> 7-i) joins the two
// quads of 8 lanes, row_mirror (i <-> 15-i) the two halves of 16.
template <int CTRL> __device__ __forceinline__ uint32_t dpp_u32(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
template <int CTRL> __device__ __forceinline__ uint64_t dpp_u64(uint64_t v)
{
    return ((uint64_t)dpp_u32<CTRL>((uint32_t)(v >> 32)) << 32) | dpp_u32<CTRL>((uint32_t)v);
}
template <int CTRL> __device__ __forceinline__ uint32_t dpp_bits(uint32_t v) { return dpp_u32<CTRL>(v); }
template <int CTRL> __device__ __forceinline__ uint64_t dpp_bits(uint64_t v) { return dpp_u64<CTRL>(v); }

template <int CTRL, typename SB> __device__ __forceinline__ void team_stage(Key<SB> &b)
{
    Key<SB> o;
    o.s = dpp_bits<CTRL>(b.s);
    o.op = dpp_u32<CTRL>(b.op);
    if (key_gt(o, b)) b = o;
}
template <int L, typename SB> __device__ __forceinline__ Key<SB> team_max(Key<SB> b)
{
    if (L >= 2) team_stage<0xB1>(b);    // quad_perm [1,0,3,2]
    if (L >= 4) team_stage<0x4E>(b);    // quad_perm [2,3,0,1]
    if (L >= 8) team_stage<0x141>(b);   // row_half_mirror
    if (L >= 16) team_stage<0x140>(b);  // row_mirror
    static_assert(L <= 16, "a team lives inside one DPP row of 16 lanes");
    return b;
}

struct TeamParams {
    SparsifyParams sp;
    int region_bytes;                  // LDS bytes of one team
    int t_hs, t_hp, t_cnt, t_oidx;     // offsets inside a team region
    int teams;                         // teams (= tiles) per workgroup
    uint64_t magic_cols, magic_g;      // ceil(2^32 / cols), ceil(2^32 / g): x / d == (x * magic) >> 32 for x < 2^16
};

template <typename T, int L, bool SMALLC>
__global__ __launch_bounds__(128) void sparsify_teams_kernel(TeamParams Q)
{
    using CT = typename ScoreOf<T>::type;
    using SB = typename ScoreOf<T>::bits;
    const SparsifyParams &P = Q.sp;
    extern __shared__ __align__(16) unsigned char smem[];

    const int n = P.n, m = P.m, g = P.g, c = P.c, cols = P.cols;
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int team = tid / L, tl = tid % L;
    const int teams = Q.teams;

    // LDS: [order table][pattern masks (m <= 8)][team regions]
    int8_t *s_order = (int8_t *)smem;
    uint8_t *s_mask = (uint8_t *)(smem + ((c * n + 15) & ~15));
    const int order_bytes = ((c * n + 15) & ~15) + ((c + 15) & ~15);
    unsigned char *region = smem + order_bytes + (size_t)team * Q.region_bytes;
    T *s_d = (T *)region;
    SB *s_hs = (SB *)(region + Q.t_hs);
    uint16_t *s_hp = (uint16_t *)(region + Q.t_hp);
    int16_t *s_cnt = (int16_t *)(region + Q.t_cnt);
    int16_t *s_oidx = (int16_t *)(region + Q.t_oidx);

    for (int i = tid; i < c * n; i += nthr) s_order[i] = P.order[i];
    if (m <= 8)
        for (int p = tid; p < c; p += nthr) {
            int mk = 0;
            for (int j = 0; j < n; j++) mk |= 1 << P.order[p * n + j];
            s_mask[p] = (uint8_t)mk;
        }

    // ---- cooperative load of the workgroup's tiles (zero beyond G / S); consecutive threads
    //      take the same column of consecutive tiles, which are adjacent along the sparse dim ----
    const int64_t tile0 = (int64_t)blockIdx.x * teams;
    const T *dense = (const T *)P.dense;
    const int64_t tiles_per_b = P.view.num_chunks * P.view.num_blocks;
    // A thread keeps one (tile, position r) pair and walks the tile's columns, so the 64-bit
    // index arithmetic is done once per pair and the loads of the walk are independent.
    for (int pair = tid; pair < teams * m; pair += nthr) {
        const int tm = pair / m, r = pair - tm * m;
        const int64_t t = tile0 + tm;
        T *dst = (T *)(smem + order_bytes + (size_t)tm * Q.region_bytes) + r;
        const T *src = nullptr;
        int valid_cols = 0;
        if (t < P.outer) {
            const int64_t b = t / tiles_per_b;
            const int64_t rem = t - b * tiles_per_b;
            const int64_t kc = rem / P.view.num_blocks;
            const int64_t mb = rem - kc * P.view.num_blocks;
            const int64_t si = mb * m + r;
            if (si < P.view.S) {
                src = dense + b * P.view.stride_b + kc * cols * P.view.stride_g + si * P.view.stride_s;
                const int64_t left = P.view.G - kc * cols;
                valid_cols = left < cols ? (int)left : cols;
            }
        }
        const int64_t sg = P.view.stride_g;
#pragma unroll 8
        for (int o = 0; o < cols; o++) dst[o * m] = o < valid_cols ? src[o * sg] : Zero<T>::v();
    }
    if (team < teams)
        for (int p = tl; p < c; p += L) s_cnt[p] = 0;
    __syncthreads();

    const bool live = team < teams && tile0 + team < P.outer;

    // SMALLC (at most 8 patterns, m <= 8, g <= 255): the pattern masks and the pattern counters
    // (8 bits each, packed) stay in registers of every lane of the team -- all lanes see every
    // accepted (column, pattern) -- so neither the staleness test nor a repair waits for LDS
    // beyond the read of the column itself.
    int mk_r[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    uint64_t cnt64 = 0;
    if (SMALLC) {
#pragma unroll
        for (int p = 0; p < 8; p++) mk_r[p] = p < c ? (int)s_mask[p] : 0;
    }
    auto cnt_of = [&](int p) { return (int)((cnt64 >> (8 * p)) & 0xFF); };

    // Best key of column o over the patterns that still have room: score bits + 1 and pattern.
    // LDS reads are issued in batches of independent loads (the column first, then 8 patterns'
    // masks and counters at a time): the loop is latency-bound, not throughput-bound.
    auto head_of = [&](int o, SB &best_s, int &best_p) {
        best_p = 0;
        best_s = 0;
        const T *col = s_d + o * m;
        if (SMALLC) {
            CT a[8];
#pragma unroll
            for (int r = 0; r < 8; r++) a[r] = score_of(col[r < m ? r : 0]);
#pragma unroll
            for (int p = 0; p < 8; p++) {
                if (p >= c || cnt_of(p) >= g) continue;
                CT acc = 0;
#pragma unroll
                for (int r = 0; r < 8; r++) {
                    if (r >= m) break;
                    if ((mk_r[p] >> r) & 1) acc += a[r];
                }
                const SB sb = score_bits(acc) + 1;
                if (sb >= best_s) {
                    best_s = sb;
                    best_p = p;
                }
            }
            return;
        }
        if (m <= 8) {
            CT a[8];
#pragma unroll
            for (int r = 0; r < 8; r++) a[r] = score_of(col[r < m ? r : 0]);
            for (int p0 = 0; p0 < c; p0 += 8) {
                int mk[8], cn[8];
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const int p = p0 + i < c ? p0 + i : c - 1;
                    mk[i] = s_mask[p];
                    cn[i] = s_cnt[p];
                }
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    if (p0 + i >= c || cn[i] >= g) continue;
                    // left-to-right sum over the pattern's positions (ascending), as the reference
                    CT acc = 0;
#pragma unroll
                    for (int r = 0; r < 8; r++) {
                        if (r >= m) break;
                        if ((mk[i] >> r) & 1) acc += a[r];
                    }
                    const SB sb = score_bits(acc) + 1;
                    if (sb >= best_s) {  // ties: larger p wins
                        best_s = sb;
                        best_p = p0 + i;
                    }
                }
            }
            return;
        }
        for (int p = 0; p < c; p++) {
            if (s_cnt[p] >= g) continue;
            CT acc = 0;
            for (int j = 0; j < n; j++) acc += score_of(col[s_order[p * n + j]]);
            const SB sb = score_bits(acc) + 1;
            if (sb >= best_s) {
                best_s = sb;
                best_p = p;
            }
        }
    };
    // Largest head among this lane's free columns (ties: larger o wins); s == 0 when none is left.
    // A lane owns at most 32 columns (the launcher picks L accordingly), kept as 4 groups of 8
    // whose maxima live in registers: a change rescans one group only.
    SB gs[4] = {0, 0, 0, 0};
    int go[4] = {0, 0, 0, 0};   // column << 16 | pattern of the group's best head
    auto scan_group = [&](int k) {
        SB v[8];
        int hp[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int o = tl + L * (k * 8 + i);
            v[i] = s_hs[o < cols ? o : tl];
            hp[i] = s_hp[o < cols ? o : tl];
        }
        // pairwise (tree) reduction; on equal scores the larger column, i.e. the later entry, wins
        SB bs[8];
        int bo[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int o = tl + L * (k * 8 + i);
            bs[i] = o < cols ? v[i] : 0;
            bo[i] = (o << 16) | hp[i];
        }
#pragma unroll
        for (int w = 1; w < 8; w <<= 1)
#pragma unroll
            for (int i = 0; i < 8; i += 2 * w)
                if (bs[i + w] >= bs[i] && bs[i + w] != 0) {
                    bs[i] = bs[i + w];
                    bo[i] = bo[i + w];
                }
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (q == k) {
                gs[q] = bs[0];
                go[q] = bo[0];
            }
    };
    auto local_best = [&]() {
        Key<SB> lb;
        lb.s = 0;
        lb.op = 0;
        SB best_s = 0;
        int best_op = 0;
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (gs[q] != 0 && gs[q] >= best_s) {
                best_s = gs[q];
                best_op = go[q];
            }
        lb.s = best_s;
        lb.op = best_s != 0 ? (uint32_t)best_op : 0u;
        return lb;
    };

    Key<SB> lb;
    lb.s = 0;
    lb.op = 0;
    if (live) {
        for (int o = tl; o < cols; o += L) {
            SB bs;
            int bp;
            head_of(o, bs, bp);
            s_hs[o] = bs;
            s_hp[o] = (uint16_t)bp;
        }
#pragma unroll
        for (int k = 0; k < 4; k++) scan_group(k);
        lb = local_best();
    }

    // Every column is accepted once and repaired at most once per pattern that fills up, which
    // bounds the loop whatever the data.
    int accepted = live ? 0 : cols;
    const int max_iter = cols * (c + 1);
    for (int iter = 0; iter < max_iter && __any(accepted < cols); iter++) {
        if (accepted < cols) {
            // ---- team arg-max ----
            const Key<SB> b = team_max<L>(lb);
            const int o_star = (int)(b.op >> 16), p_star = (int)(b.op & 0xFFFFu);
            const int cntp = SMALLC ? cnt_of(p_star) : (int)s_cnt[p_star];
            const bool stale = cntp >= g;
            if (SMALLC && !stale) cnt64 += (uint64_t)1 << (8 * p_star);
            if (o_star % L == tl) {
                if (stale) {
                    SB bs;
                    int bp;
                    head_of(o_star, bs, bp);
                    s_hs[o_star] = bs;
                    s_hp[o_star] = (uint16_t)bp;
                } else {
                    if (!SMALLC) s_cnt[p_star] = (int16_t)(cntp + 1);
                    s_hs[o_star] = 0;
                    s_oidx[p_star * g + cntp] = (int16_t)o_star;
                }
                scan_group((o_star / L) >> 3);
                lb = local_best();
            }
            if (!stale) accepted++;
        }
        // the team's LDS writes must be visible to its other lanes in the next iteration
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }

    // ---- coalesced store of the workgroup's tiles: one thread per slot writes its index and
    //      gathers its n values from the tile data (divisions by multiplication: e < 2^16) ----
    __syncthreads();
    T *val = (T *)P.val;
    for (int e = tid; e < teams * cols; e += nthr) {
        const int tm = (int)(((uint64_t)e * Q.magic_cols) >> 32), slot = e - tm * cols;
        const int64_t t = tile0 + tm;
        if (t >= P.outer) break;
        const unsigned char *reg = smem + order_bytes + (size_t)tm * Q.region_bytes;
        const int o = ((const int16_t *)(reg + Q.t_oidx))[slot];
        const int p = (int)(((uint64_t)slot * Q.magic_g) >> 32);
        const T *col = (const T *)reg + o * m;
        const int64_t at = t * (int64_t)cols + slot;
        P.idx[at] = (int16_t)o;
        for (int j = 0; j < n; j++) val[at * n + j] = col[s_order[p * n + j]];
    }
}

template <typename T, int L> static int launch_sparsify_teams(SparsifyParams &P, hipStream_t stream, bool *done)
{
    using SB = typename ScoreOf<T>::bits;
    *done = false;
    TeamParams Q{};
    Q.sp = P;
    const int cols = P.cols, m = P.m, c = P.c, n = P.n;
    int off = align_up(cols * m * (int)sizeof(T), 8);
    Q.t_hs = off;
    off = align_up(off + cols * (int)sizeof(SB), 4);
    Q.t_hp = off;
    off = align_up(off + cols * 2, 4);
    Q.t_cnt = off;
    off = align_up(off + c * 2, 4);
    Q.t_oidx = off;
    off = align_up(off + cols * 2, 4);
    // region size = L (mod 64) words spreads the teams of a wavefront over the banks; regions of
    // 8-byte data stay 8-byte aligned (an even number of words)
    int words = off / 4, target = L % 64;
    if ((sizeof(T) == 8 || sizeof(SB) == 8) && (target & 1)) target++;
    while (words % 64 != target) words++;
    Q.region_bytes = words * 4;
    const size_t order_bytes = (size_t)align_up(c * n, 16) + (size_t)align_up(c, 16);
    // workgroups of 128 threads when two of them fit in a CU's LDS, else 64 threads
    int threads = 128;
    size_t lds = order_bytes + (size_t)(threads / L) * Q.region_bytes;
    if (lds > 80 * 1024) {
        threads = 64;
        lds = order_bytes + (size_t)(threads / L) * Q.region_bytes;
    }
    if (lds > 160 * 1024) return NMG_OK;   // too large for this kernel: the caller falls back
    Q.teams = threads / L;
    Q.magic_cols = (((uint64_t)1 << 32) + cols - 1) / cols;
    Q.magic_g = (((uint64_t)1 << 32) + P.g - 1) / P.g;
    const bool smallc = c <= 8 && m <= 8 && P.g <= 255;
    auto kern = smallc ? sparsify_teams_kernel<T, L, true> : sparsify_teams_kernel<T, L, false>;
    if (lds > 64 * 1024)
        NMG_HIP_TRY(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)lds));
    const int64_t grid = (P.outer + Q.teams - 1) / Q.teams;
    NMG_REQUIRE(grid <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "too many tiles (%lld)", (long long)grid);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(threads), lds, stream, Q);
    NMG_HIP_TRY(hipGetLastError());
    *done = true;
    return NMG_OK;
}

// ------------------------------------------------------------- rounds: batched acceptance
// The sorted walk accepts, between two moments at which a pattern fills up, exactly the heads of
// the free columns whose key is at least the key at which the next pattern fills: until then no
// pattern is full, so every column met in the walk is accepted by the first pattern it asks for
// (its head).  One *round* therefore does in parallel what the step-by-step formulation does in
// up to c*g steps:
//   1. every free column proposes to its head pattern (best key over the patterns with room);
//   2. the proposals are grouped by pattern (counting sort) and every proposal gets its rank
//      inside its pattern's group in descending key order;
//   3. a pattern with more proposals than room fills at the key of its proposal of rank room-1;
//      t = the largest such key over the patterns (0 when no pattern overflows);
//   4. every proposal with key >= t is accepted into slot p*g + used[p] + rank: inside a pattern
//      the walk hands out slots in descending key order, and the keys accepted later are smaller;
//   5. the columns whose head pattern is now full compute a new head.
// Every round fills at least one pattern or ends the tile, so a tile takes at most c rounds.
//
// A tile belongs to NT threads: 16, 32 or 64 lanes of a wavefront (256 threads per workgroup,
// wavefront-level synchronisation only; the teams of a wavefront run the same instruction stream
// on their own tiles and simply diverge where their rounds differ) or a whole workgroup.  The free columns live in a compact list that
// every round rewrites, so a round costs as many wavefront passes as the columns that are still
// free need, not as the tile has.  For scores of 32 bits (every type but double) and m <= 8; a
// key is one 64-bit word: (score bits + 1) << 32 | column << 16 | pattern.
constexpr long binom_c(int m, int n)
{
    long r = 1;
    for (int i = 1; i <= n; i++) r = r * (m - n + i) / i;
    return r;
}

struct RoundParams {
    SparsifyParams sp;
    int region_bytes;                          // LDS bytes of one tile
    int r_gk, r_fk, r_oidx, r_int;             // offsets inside a tile region
    int tiles;                                 // tiles per workgroup
    int cpad_log2;                             // log2 of the power of two >= c
    int vec_bytes;                             // m values of a column are one aligned load of 4, 8 or 16 bytes (else 0)
    int val_pairs;                             // val is aligned to 4 bytes
    uint32_t masks[32];                        // position mask of every pattern, four per word
    uint64_t magic_cols, magic_g;
};

template <int NT> __device__ __forceinline__ void tile_sync()
{
    if (NT <= 64) {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    } else {
        __syncthreads();
    }
}

// Inclusive prefix sum over the 64 lanes of a wavefront (or over each half of it) with DPP moves: shifts by 1, 2, 4, 8
// inside the rows of 16 lanes, then lane 15 of rows 0 and 2 is added to rows 1 and 3, then lane
// 31 to rows 2 and 3.
template <int CTRL, int ROWS> __device__ __forceinline__ int dpp_move0(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROWS, 0xF, CTRL < 0x140);
}
template <int LANES> __device__ __forceinline__ int wave_prefix_sum(int v)
{
    v += dpp_move0<0x111, 0xF>(v);   // row_shr:1
    v += dpp_move0<0x112, 0xF>(v);   // row_shr:2
    v += dpp_move0<0x114, 0xF>(v);   // row_shr:4
    v += dpp_move0<0x118, 0xF>(v);   // row_shr:8
    if (LANES >= 32) v += dpp_move0<0x142, 0xA>(v);   // row_bcast:15 into rows 1 and 3
    if (LANES == 64) v += dpp_move0<0x143, 0xC>(v);   // row_bcast:31 into rows 2 and 3
    return v;   // LANES == 32, 16: one sum per half, per row of the wavefront
}

// SN, SM, SG != 0: the kernel is compiled for that n:m:g (the loops over patterns and positions
// unroll, the divisions by c*g and g fold); 0: taken from the arguments.
template <typename T, int NT, int CPT, int SN = 0, int SM = 0, int SG = 0>
__global__ __launch_bounds__(NT <= 64 ? 256 : NT) void sparsify_rounds_kernel(RoundParams Q)
{
    const SparsifyParams &P = Q.sp;
    extern __shared__ __align__(16) unsigned char smem[];

    constexpr int SC = SM ? (int)binom_c(SM, SN) : 0;   // patterns of the compiled-in n:m
    const int n = SN ? SN : P.n, m = SM ? SM : P.m, g = SG ? SG : P.g, c = SC ? SC : P.c,
              cols = (SC && SG) ? SC * SG : P.cols;
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int tile = tid / NT, tt = tid % NT;
    constexpr int tiles = NT <= 64 ? 256 / NT : 1;   // tiles per workgroup (what the launch puts in Q.tiles)

    // LDS: [pattern masks][tile regions]
    uint8_t *s_mask = (uint8_t *)smem;
    const int order_bytes = (c + 15) & ~15;
    unsigned char *region = smem + order_bytes + (size_t)tile * Q.region_bytes;
    T *s_d = (T *)region;
    // proposals grouped by pattern: key >> 16; between two rounds its first entries are the
    // columns waiting for a new head: best (score bits + 1) << 32 | column << 16 | pattern
    uint64_t *s_gk = (uint64_t *)(region + Q.r_gk);
    uint64_t *s_fk = (uint64_t *)(region + Q.r_fk);     // free columns: key of the head
    int16_t *s_oidx = (int16_t *)(region + Q.r_oidx);
    int *s_dem = (int *)(region + Q.r_int);             // proposals per pattern in this round
    int *s_start = s_dem + c;                           // first entry of the pattern's group
    int *s_used = s_start + c;                          // slots taken
    int *s_new = s_used + c;                            // slots taken in this round
    int *s_cnt = s_new + c;                             // free columns: list of this round, of the next
    int *s_nwork = s_cnt + 2;
    int *s_props = s_nwork + 1;                         // proposals of this round
    uint64_t *s_fill = (uint64_t *)(s_dem + 4 * c + 4);   // largest fill key of the round

    // The position masks of the patterns (bit r = position r is kept; a pattern's positions in
    // ascending order are its entry of the order table) come with the kernel arguments and go
    // to LDS through the scalar unit: a workgroup lives for some ten microseconds and would
    // spend one or two of them waiting for a table in global memory.
    for (int w = 0; w < (c + 3) / 4; w++) {
        const uint32_t four = Q.masks[w];
        if (tid == 0) ((uint32_t *)s_mask)[w] = four;
    }

    // ---- cooperative load of the workgroup's tiles (zero beyond G / S) ----
    // Workgroups go to the 8 XCDs in turn, each with an L2 of its own, and up to 8 workgroups on
    // consecutive tiles (adjacent along the sparse dim) read from the same 128-byte lines: among
    // every 64 workgroups, XCD x gets the tile groups 8x .. 8x+7, so a line is fetched from HBM
    // once, not once per XCD.  Last tiles first: the tiles of the last chunk of the group dim
    // are padded with zero columns and should not be the tail.
    int64_t grp = blockIdx.x;
    if (grp < (int64_t)(gridDim.x & ~63u)) grp = (grp & ~63LL) | ((grp & 7) << 3) | ((grp >> 3) & 7);
    const int64_t tile0 = ((int64_t)gridDim.x - 1 - grp) * tiles;
    const T *dense = (const T *)P.dense;
    const int64_t tiles_per_b = P.view.num_chunks * P.view.num_blocks;
    // (batch, chunk of the group dim, block of the sparse dim) of the workgroup's first tile, once and
    // on the scalar unit; a tile tm further on is reached by walking the blocks with wrap-around
    // (a 64-bit division per thread costs more than a hundred instructions)
    const int64_t b_first = tile0 / tiles_per_b;
    const int64_t rem_first = tile0 - b_first * tiles_per_b;
    const int64_t kc_first = rem_first / P.view.num_blocks, mb_first = rem_first - kc_first * P.view.num_blocks;
    auto locate = [&](int tm, int64_t &b, int64_t &kc, int64_t &mb) {
        b = b_first;
        kc = kc_first;
        mb = mb_first + tm;
        while (mb >= P.view.num_blocks) {
            mb -= P.view.num_blocks;
            if (++kc == P.view.num_chunks) {
                kc = 0;
                b++;
            }
        }
    };
    if (Q.vec_bytes != 0) {
        // the m values of a column are contiguous and aligned: one load and one LDS write each.
        // Consecutive threads take the same column of consecutive tiles (adjacent along the
        // sparse dim, so adjacent in memory), then the next columns.
        const int walkers = nthr / tiles;
        if (tid < walkers * tiles) {
            const int o0 = tid / tiles, tm = tid - o0 * tiles;
            const int64_t t = tile0 + tm;
            unsigned char *dst = smem + order_bytes + (size_t)tm * Q.region_bytes;
            const T *src = nullptr;
            int valid_cols = 0;
            if (t < P.outer) {
                int64_t b, kc, mb;
                locate(tm, b, kc, mb);
                src = dense + b * P.view.stride_b + kc * cols * P.view.stride_g + mb * m;
                const int64_t left = P.view.G - kc * cols;
                valid_cols = left < cols ? (int)left : cols;
            }
            const int64_t sg = P.view.stride_g;
            if (Q.vec_bytes == 16) {
#pragma unroll 4
                for (int o = o0; o < cols; o += walkers)
                    ((uint4 *)dst)[o] = o < valid_cols ? *(const uint4 *)(src + o * sg) : make_uint4(0, 0, 0, 0);
            } else if (Q.vec_bytes == 8) {
#pragma unroll 4
                for (int o = o0; o < cols; o += walkers)
                    ((uint2 *)dst)[o] = o < valid_cols ? *(const uint2 *)(src + o * sg) : make_uint2(0, 0);
            } else {
#pragma unroll 4
                for (int o = o0; o < cols; o += walkers)
                    ((uint32_t *)dst)[o] = o < valid_cols ? *(const uint32_t *)(src + o * sg) : 0u;
            }
        }
    } else if (P.view.stride_g == 1) {
        // The columns are contiguous: a wavefront takes 64 consecutive columns of one line of
        // the region (tile, position), four such runs in flight before the first is stored.
        // The tiles' base offsets come from a small table, computed once.
        __shared__ int64_t s_tbase[16];
        __shared__ int s_tcols[16], s_trows[16];
        if (tid < tiles) {
            const int64_t t = tile0 + tid;
            int64_t base = 0;
            int vc = 0, vr = 0;
            if (t < P.outer) {
                int64_t b, kc, mb;
                locate(tid, b, kc, mb);
                base = b * P.view.stride_b + kc * cols + mb * m * P.view.stride_s;
                const int64_t left = P.view.G - kc * cols, below = P.view.S - mb * m;
                vc = left < cols ? (int)left : cols;
                vr = below < m ? (int)below : m;
            }
            s_tbase[tid] = base;
            s_tcols[tid] = vc;
            s_trows[tid] = vr;
        }
        __syncthreads();
        const int cpl = (cols + 63) >> 6;                 // runs of 64 columns per line
        const int nruns = tiles * m * cpl;
        const int wv = __builtin_amdgcn_readfirstlane(tid >> 6), ln = tid & 63, nw = nthr >> 6;
        for (int c0 = wv; c0 < nruns; c0 += 4 * nw) {
            T v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int ce = c0 + u * nw;
                v[u] = Zero<T>::v();
                if (ce < nruns) {
                    const int line = ce / cpl, oc = ce - line * cpl;
                    const int tm = line / m, r = line - tm * m;
                    const int o = oc * 64 + ln;
                    if (o < s_tcols[tm] && r < s_trows[tm])
                        v[u] = dense[s_tbase[tm] + (int64_t)r * P.view.stride_s + o];
                }
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int ce = c0 + u * nw;
                if (ce >= nruns) continue;
                const int line = ce / cpl, oc = ce - line * cpl;
                const int tm = line / m, r = line - tm * m;
                const int o = oc * 64 + ln;
                if (o < cols) ((T *)(smem + order_bytes + (size_t)tm * Q.region_bytes))[o * m + r] = v[u];
            }
        }
    } else {
        // consecutive threads take the m values of a column, then the same column of the next
        // tile (adjacent along the sparse dim); a thread keeps its (tile, position) pair and walks
        // the columns, so the 64-bit index arithmetic is done once
        const int per = tiles * m, walkers = nthr / per;
        if (tid < walkers * per) {
            const int o0 = tid / per, rest = tid - o0 * per;
            const int tm = rest / m, r = rest - tm * m;
            const int64_t t = tile0 + tm;
            T *dst = (T *)(smem + order_bytes + (size_t)tm * Q.region_bytes) + r;
            const T *src = nullptr;
            int valid_cols = 0;
            if (t < P.outer) {
                int64_t b, kc, mb;
                locate(tm, b, kc, mb);
                const int64_t si = mb * m + r;
                if (si < P.view.S) {
                    src = dense + b * P.view.stride_b + kc * cols * P.view.stride_g + si * P.view.stride_s;
                    const int64_t left = P.view.G - kc * cols;
                    valid_cols = left < cols ? (int)left : cols;
                }
            }
            const int64_t sg = P.view.stride_g;
#pragma unroll 4
            for (int o = o0; o < cols; o += walkers) dst[o * m] = o < valid_cols ? src[o * sg] : Zero<T>::v();
        }
    }
    if (tile < tiles)
        for (int p = tt; p < 4 * c + 6; p += NT) s_dem[p] = 0;   // counters and the fill key
    __syncthreads();

    const bool live = tile < tiles && tile0 + tile < P.outer;
    // Real columns of this tile; the rest (beyond the end of the group dim) is zero padding.
    int real_cols = cols;
    if (live) {
        int64_t b_mine, kc_mine, mb_mine;
        locate(tile, b_mine, kc_mine, mb_mine);
        const int64_t left = P.view.G - kc_mine * cols;
        if (left < cols) real_cols = (int)left;
    }

    // Score of column o for the pattern with position mask mk: the sum runs over the pattern's
    // positions in ascending order, in single precision, as the reference's.
    auto load_col = [&](int o, float (&a)[8]) {
        const T *col = s_d + o * m;
        if (sizeof(T) == 2 && m == 8) {
            // the tile starts on a 16-byte boundary of LDS: one read for the column
            const uint4 raw = *(const uint4 *)col;
            T v[8];
            __builtin_memcpy(v, &raw, 16);
#pragma unroll
            for (int r = 0; r < 8; r++) a[r] = score_of(v[r]);
        } else if (sizeof(T) == 2 && m == 4) {
            const uint2 raw = *(const uint2 *)col;
            T v[4];
            __builtin_memcpy(v, &raw, 8);
#pragma unroll
            for (int r = 0; r < 8; r++) a[r] = score_of(v[r & 3]);
        } else {
#pragma unroll
            for (int r = 0; r < 8; r++) a[r] = score_of(col[r < m ? r : 0]);
        }
    };
    auto score = [&](const float (&a)[8], int mk) {
        float acc = 0;
#pragma unroll
        for (int r = 0; r < 8; r++) {
            if (r >= m) break;
            if ((mk >> r) & 1) acc += a[r];
        }
        return acc;
    };

    if (live) {
        // heads of all columns: every pattern has room; on equal scores the larger pattern wins.
        // The patterns are the outer loop: a pattern's mask is fetched once for the thread's
        // columns and made a scalar, so its positions are picked without lane selects.
        {
            float a[CPT][8];
            uint32_t bs[CPT];
            int bp[CPT];
            const int ns0 = (real_cols + NT - 1) / NT;
#pragma unroll
            for (int i = 0; i < CPT; i++) {
                bs[i] = 0;
                bp[i] = 0;
                load_col(i < ns0 && tt + NT * i < real_cols ? tt + NT * i : 0, a[i]);
            }
            // Four masks per LDS word; a position of the pattern is a branch of the whole
            // wavefront around one addition per column (0 + x is x: the first one is exact too).
            for (int w = 0; w < (c + 3) / 4; w++) {
                const uint32_t four = __builtin_amdgcn_readfirstlane(((const uint32_t *)s_mask)[w]);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int p = 4 * w + j;
                    if (p >= c) break;
                    const uint32_t mk = (four >> (8 * j)) & 0xFFu;
                    float acc[CPT];
#pragma unroll
                    for (int i = 0; i < CPT; i++) acc[i] = 0;
#pragma unroll
                    for (int r = 0; r < 8; r++)
                        if ((mk >> r) & 1) {
                            asm volatile("");   // keeps the branch: a select per column costs more
#pragma unroll
                            for (int i = 0; i < CPT; i++) acc[i] += a[i][r];
                        }
#pragma unroll
                    for (int i = 0; i < CPT; i++) {
                        const uint32_t sb = score_bits(acc[i]) + 1;
                        if (sb >= bs[i]) {
                            bs[i] = sb;
                            bp[i] = p;
                        }
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < CPT; i++) {
                const int o = tt + NT * i;
                if (i < ns0 && o < real_cols)
                    s_fk[o] = ((uint64_t)bs[i] << 32) | ((uint32_t)o << 16) | (uint32_t)bp[i];
            }
        }
        if (tt == 0) s_cnt[0] = real_cols;
        tile_sync<NT>();

        // Zero padding: the padded columns have score 0 for every pattern and the largest column
        // numbers of the tile, so the walk meets them after every key with a positive score and
        // before every other key with score 0, in descending column order, and each takes the
        // largest pattern with room.  They never enter the list: the rounds first run on the
        // positive keys alone (hold = true: a column whose head has score 0 waits), then the
        // padded columns are placed in closed form, then the rounds go on with what is left.
        bool hold = real_cols < cols;
        for (int round = 0; round <= 2 * c + 2; round++) {
            // The free columns of this round: the list of the columns whose head stayed valid,
            // then the columns that were given a new head at the end of the last round.
            const int q = round & 1;
            const int nlist = s_cnt[q], nredo = *s_nwork;
            const int nfree = nlist + nredo;
            if (nfree == 0 && !hold) break;
            // entries per thread in this round; a wavefront beyond the end of the list has none
            // and only keeps the barriers
            const int ns = (tt & ~63) < nfree ? (nfree + NT - 1) / NT : 0;
            uint64_t key[CPT];   // key of the head; 0 = no entry, or placed
            int pos[CPT];        // place inside the pattern's group, then rank
            uint32_t waiting = 0;   // entries held back in this round
            // 1. proposals per pattern; the returned count is the place inside the group
#pragma unroll
            for (int i = 0; i < CPT; i++) {
                key[i] = 0;
                pos[i] = 0;
                const int e = tt + NT * i;
                if (i < ns && e < nfree) {
                    key[i] = e < nlist ? s_fk[e] : s_gk[e - nlist];
                    if (hold && (key[i] >> 32) == 1) waiting |= 1u << i;
                    else pos[i] = atomicAdd(&s_dem[(int)(key[i] & 0xFFFFu)], 1);
                }
            }
            tile_sync<NT>();
            // 2. the slots taken in the last round are booked; group offsets: exclusive prefix sum
            //    of the demands (first wavefront of the tile; c <= 128, two patterns per lane)
            if (tt < 64) {
                const int p0 = 2 * tt, p1 = 2 * tt + 1;
                const int d0 = p0 < c ? s_dem[p0] : 0, d1 = p1 < c ? s_dem[p1] : 0;
                const int excl = wave_prefix_sum<(NT < 64 ? NT : 64)>(d0 + d1) - (d0 + d1);
                if (p0 < c) {
                    s_start[p0] = excl;
                    s_used[p0] += s_new[p0];
                    s_new[p0] = 0;
                }
                if (p1 < c) {
                    s_start[p1] = excl + d0;
                    s_used[p1] += s_new[p1];
                    s_new[p1] = 0;
                }
                if (tt == 0) {
                    s_cnt[q ^ 1] = 0;   // the list of the next round starts empty
                    *s_nwork = 0;
                    *s_fill = 0;
                }
                if (tt == (NT < 64 ? NT : 64) - 1) *s_props = excl + d0 + d1;   // proposals of this round
            }
            tile_sync<NT>();
            if (hold && *s_props == 0) {
                // No positive key is left.  Padded column number k from the top (column
                // cols-1-k) goes to the pattern p with top(p) <= k < top(p) + room(p), where
                // top(p) = room of the patterns above p.  Lane l of the first wavefront takes the
                // patterns c-1-2l and c-2-2l.
                if (tt < 64) {
                    const int p0 = c - 1 - 2 * tt, p1 = c - 2 - 2 * tt;
                    const int r0 = p0 >= 0 ? g - s_used[p0] : 0, r1 = p1 >= 0 ? g - s_used[p1] : 0;
                    const int excl = wave_prefix_sum<(NT < 64 ? NT : 64)>(r0 + r1) - (r0 + r1);
                    if (p0 >= 0) s_start[p0] = excl;
                    if (p1 >= 0) s_start[p1] = excl + r0;
                }
                tile_sync<NT>();
                const int npad = cols - real_cols;
                for (int k = tt; k < npad; k += NT) {
                    // top() grows as p falls: the pattern is the smallest p with top(p) <= k
                    // (then k < top(p-1) = top(p) + room(p), and the total room covers k at p = 0)
                    int lo = 0, hi = c - 1;
                    while (lo < hi) {
                        const int mid = (lo + hi) >> 1;
                        if (s_start[mid] <= k) hi = mid;
                        else lo = mid + 1;
                    }
                    s_oidx[lo * g + s_used[lo] + (k - s_start[lo])] = (int16_t)(cols - 1 - k);
                }
                tile_sync<NT>();
                for (int p = tt; p < c; p += NT) {
                    // pattern p has taken the padded columns [top, top + room) that exist
                    const int top = s_start[p], room = g - s_used[p];
                    s_used[p] += npad - top < room ? (npad - top > 0 ? npad - top : 0) : room;
                }
                // the held entries may now point to a full pattern: all of them take a new head
#pragma unroll
                for (int i = 0; i < CPT; i++)
                    if ((waiting >> i) & 1) {
                        const int w = atomicAdd(s_nwork, 1);
                        s_gk[w] = key[i] & 0xFFFF0000ull;
                    }
                hold = false;
                tile_sync<NT>();
            } else {
                // 3. grouped list: (score bits + 1) << 16 | column
#pragma unroll
                for (int i = 0; i < CPT; i++)
                    if (i < ns && key[i] != 0 && !((waiting >> i) & 1))
                        s_gk[s_start[(int)(key[i] & 0xFFFFu)] + pos[i]] = key[i] >> 16;
                tile_sync<NT>();
                // 4. rank inside the group (keys differ in the column at least); the proposal at
                //    which an overflowing pattern fills publishes its key
#pragma unroll
                for (int i = 0; i < CPT; i++)
                    if (i < ns && key[i] != 0 && !((waiting >> i) & 1)) {
                        const int p = (int)(key[i] & 0xFFFFu);
                        const uint64_t mine = key[i] >> 16;
                        const int seg = s_start[p], d = s_dem[p];
                        const int room = g - s_used[p];
                        // Eight entries are in flight at a time (the loop is bound by the LDS round
                        // trip).  A proposal that has seen `room` larger keys cannot be accepted in
                        // this round -- its pattern fills above it -- and stops counting.
                        // Whole batches are counted unmasked; the last, partial one reads past
                        // the group (into the next group or the array behind the list, both inside
                        // the tile's LDS) and masks what it read there.
                        const uint64_t *grp = s_gk + seg;
                        int r = 0, j0 = 0;
                        for (; j0 + 8 <= d && r < room; j0 += 8) {
                            uint64_t e[8];
#pragma unroll
                            for (int u = 0; u < 8; u++) e[u] = grp[j0 + u];
#pragma unroll
                            for (int u = 0; u < 8; u++) r += e[u] > mine ? 1 : 0;
                        }
                        if (j0 < d && r < room) {
                            uint64_t e[8];
#pragma unroll
                            for (int u = 0; u < 8; u++) e[u] = grp[j0 + u];
#pragma unroll
                            for (int u = 0; u < 8; u++) r += (j0 + u < d && e[u] > mine) ? 1 : 0;
                        }
                        pos[i] = r;
                        if (d > room && r == room - 1) atomicMax((unsigned long long *)s_fill, (unsigned long long)key[i]);
                    }
                tile_sync<NT>();
                // 5. What lies at or above the largest fill key (0: no pattern overflows) is
                //    accepted.  The pattern of that key is the one pattern that this round leaves
                //    without room while proposals to it remain: of the columns that stay free,
                //    those need a new head, the others go to the next round's list as they are.
                const uint64_t fill = *s_fill;
                const int filled = fill != 0 ? (int)(fill & 0xFFFFu) : -1;
#pragma unroll
                for (int i = 0; i < CPT; i++)
                    if (i < ns && key[i] != 0) {
                        const int p = (int)(key[i] & 0xFFFFu);
                        if (!((waiting >> i) & 1) && key[i] >= fill) {
                            s_oidx[p * g + s_used[p] + pos[i]] = (int16_t)((key[i] >> 16) & 0xFFFFu);
                            atomicAdd(&s_new[p], 1);
                        } else if (p == filled) {
                            const int w = atomicAdd(s_nwork, 1);
                            s_gk[w] = key[i] & 0xFFFF0000ull;
                        } else {
                            s_fk[atomicAdd(&s_cnt[q ^ 1], 1)] = key[i];
                        }
                    }
                for (int p = tt; p < c; p += NT) s_dem[p] = 0;
                tile_sync<NT>();
            }
            // 6. new heads, one thread per (column, pattern): these columns are few and a loop
            //    over the patterns is a chain of LDS round trips; the best key of a column is
            //    gathered with an LDS maximum (the grouped list, free between two rounds, holds
            //    it, and the next round reads it from there)
            const int nwork = *s_nwork;
            if (nwork > 0) {
                const int cl = Q.cpad_log2;
                for (int e = tt; e < (nwork << cl); e += NT) {
                    const int w = e >> cl, p = e & ((1 << cl) - 1);
                    if (p < c && s_used[p] + s_new[p] < g) {
                        float a[8];
                        // the column sits in bits 16..31 of the entry, which the maxima leave alone
                        const uint32_t o = ((const uint16_t *)&s_gk[w])[1];
                        load_col((int)o, a);
                        const uint32_t sb = score_bits(score(a, s_mask[p])) + 1;
                        atomicMax((unsigned long long *)&s_gk[w], ((unsigned long long)sb << 32) | (o << 16) | (unsigned)p);
                    }
                }
                tile_sync<NT>();
            }
        }
    }

    // ---- coalesced store of the workgroup's tiles: one thread per slot writes its index and
    //      gathers its n values from the tile data ----
    __syncthreads();
    T *val = (T *)P.val;
    for (int e = tid; e < tiles * cols; e += nthr) {
        const int tm = (int)(((uint64_t)e * Q.magic_cols) >> 32), slot = e - tm * cols;
        const int64_t t = tile0 + tm;
        if (t >= P.outer) continue;
        const unsigned char *reg = smem + order_bytes + (size_t)tm * Q.region_bytes;
        const int o = ((const int16_t *)(reg + Q.r_oidx))[slot];
        const int p = (int)(((uint64_t)slot * Q.magic_g) >> 32);
        const T *col = (const T *)reg + o * m;
        const int64_t at = t * (int64_t)cols + slot;
        P.idx[at] = (int16_t)o;
        int mk = s_mask[p];
        if (sizeof(T) == 2 && n == 2 && Q.val_pairs) {
            // both values in one store
            T v[2];
            v[0] = col[__ffs(mk) - 1];
            mk &= mk - 1;
            v[1] = col[__ffs(mk) - 1];
            uint32_t raw;
            __builtin_memcpy(&raw, v, 4);
            ((uint32_t *)val)[at] = raw;
        } else {
            for (int j = 0; j < n; j++) {
                val[at * n + j] = col[__ffs(mk) - 1];   // the j-th kept position
                mk &= mk - 1;
            }
        }
    }
}

template <typename T, int NT, int CPT, int SN = 0, int SM = 0, int SG = 0>
static int launch_sparsify_rounds(SparsifyParams &P, hipStream_t stream, bool *done)
{
    *done = false;
    if (sizeof(typename ScoreOf<T>::bits) != 4) return NMG_OK;
    RoundParams Q{};
    Q.sp = P;
    const int cols = P.cols, m = P.m, c = P.c, n = P.n;
    if (m > 8 || c > 128 || n < 1 || cols > NT * CPT) return NMG_OK;
    Q.tiles = NT <= 64 ? 256 / NT : 1;
    if (NT < 64 && c > 2 * NT) return NMG_OK;   // the prefix sums take two patterns per lane
    if ((int64_t)Q.tiles * cols >= 65536) return NMG_OK;   // the magic divisions hold below 2^16
    int off = align_up(cols * m * (int)sizeof(T), 8);
    Q.r_gk = off;
    off += cols * 8;
    Q.r_fk = off;
    off += cols * 8;
    Q.r_oidx = off;
    off = align_up(off + cols * 2, 8);
    Q.r_int = off;
    off = align_up(off + (4 * c + 6) * 4, 8);
    Q.region_bytes = align_up(off, 16);
    const int threads = NT <= 64 ? 256 : NT;
    // one aligned load per column where its m values are contiguous: sparse dim with stride 1
    // and no partial last block, every column start a multiple of the vector size
    const int vb = m * (int)sizeof(T);
    if ((vb == 4 || vb == 8 || vb == 16) && P.view.stride_s == 1 && P.view.S % m == 0 &&
        (uintptr_t)P.dense % vb == 0 && P.view.stride_g % m == 0 && P.view.stride_b % m == 0)
        Q.vec_bytes = vb;
    Q.val_pairs = (uintptr_t)P.val % 4 == 0;
    const size_t order_bytes = (size_t)align_up(c, 16);
    const size_t lds = order_bytes + (size_t)Q.tiles * Q.region_bytes;
    if (lds > 159 * 1024) return NMG_OK;   // too large for this kernel (which has a small static table too): the caller falls back
    Q.cpad_log2 = 0;
    while ((1 << Q.cpad_log2) < c) Q.cpad_log2++;
    const int8_t *order = host_order(n, m);
    NMG_REQUIRE(order != nullptr, NMG_ERR_ARG, "invalid n:m = %d:%d", n, m);
    for (int p = 0; p < c; p++)
        for (int j = 0; j < n; j++) Q.masks[p / 4] |= 1u << (8 * (p % 4) + order[p * n + j]);
    Q.magic_cols = (((uint64_t)1 << 32) + cols - 1) / cols;
    Q.magic_g = (((uint64_t)1 << 32) + P.g - 1) / P.g;
    auto kern = sparsify_rounds_kernel<T, NT, CPT, SN, SM, SG>;
    if (lds > 64 * 1024)
        NMG_HIP_TRY(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)lds));
    const int64_t grid = (P.outer + Q.tiles - 1) / Q.tiles;
    NMG_REQUIRE(grid <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "too many tiles (%lld)", (long long)grid);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(threads), lds, stream, Q);
    NMG_HIP_TRY(hipGetLastError());
    *done = true;
    return NMG_OK;
}

template <typename T, int NT, int CPT, int SN, int SM, int SG>
static int launch_rounds_for(SparsifyParams &P, hipStream_t stream, bool *done)
{
    if constexpr (sizeof(T) == 2)
        return launch_sparsify_rounds<T, NT, CPT, SN, SM, SG>(P, stream, done);
    else
        return launch_sparsify_rounds<T, NT, CPT>(P, stream, done);
}

template <typename T> static int dispatch_sparsify(SparsifyParams &P, hipStream_t stream)
{
    // Tiles of at least 16 columns: batched rounds, with as many lanes per tile as its later
    // rounds keep busy -- a quarter, a half or a whole wavefront (several tiles share the
    // wavefront's instruction stream), else a workgroup.  Measured on 4096 x 4096 fp16, 2:4 with
    // g = 4 / 8 / 16 / 32 / 64: 182 / 125 / 125 / 130 / 141 us against 320 / 407 / 402 / 742 / 1204 us
    // for the lane teams below; 8192 x 8192, 1:8:32 / 2:8:32 / 4:8:32: 0.39 / 0.92 / 2.1 ms against
    // 2.6 / 10.9 / 56 ms for the step-by-step kernels.  Half a wavefront loses to a whole one from
    // about 20 patterns on (2:8:4, 112 columns: 430 against 324 us); tiles of fewer than 16 columns
    // stay with the lane teams (2:4:2: 200 against 315 us).  A tile's rounds are a chain of
    // barriers and LDS round trips, so what counts is how many tiles a CU holds at once (34 bytes
    // of LDS per column): 2240-column tiles (4:8:32) take 2.1 ms with 512 threads, two tiles per
    // CU, against 3.4 ms with 1024 threads, whose registers allow one.
    if (P.cols >= 16 && P.n > 0) {
        bool done = false;
        int rc;
        if (P.cols <= 64 && P.c <= 32) rc = launch_sparsify_rounds<T, 16, 4>(P, stream, &done);
        // the benchmark's patterns on 16-bit weights: kernels compiled for their n:m:g (10-15 % fewer
        // instructions: 4096^2 2:4:16 113 -> 100 us)
        else if (sizeof(T) == 2 && P.n == 2 && P.m == 4 && P.g == 16) rc = launch_rounds_for<T, 32, 4, 2, 4, 16>(P, stream, &done);
        else if (sizeof(T) == 2 && P.n == 1 && P.m == 8 && P.g == 32) rc = launch_rounds_for<T, 64, 4, 1, 8, 32>(P, stream, &done);
        else if (sizeof(T) == 2 && P.n == 2 && P.m == 8 && P.g == 32) rc = launch_rounds_for<T, 256, 4, 2, 8, 32>(P, stream, &done);
        else if (sizeof(T) == 2 && P.n == 4 && P.m == 8 && P.g == 32) rc = launch_rounds_for<T, 512, 5, 4, 8, 32>(P, stream, &done);
        else if (P.cols <= 128 && P.c <= 20) rc = launch_sparsify_rounds<T, 32, 4>(P, stream, &done);
        else if (P.cols <= 128) rc = launch_sparsify_rounds<T, 64, 2>(P, stream, &done);
        else if (P.cols <= 256) rc = launch_sparsify_rounds<T, 64, 4>(P, stream, &done);
        else if (P.cols <= 512) rc = launch_sparsify_rounds<T, 128, 4>(P, stream, &done);
        else if (P.cols <= 1024) rc = launch_sparsify_rounds<T, 256, 4>(P, stream, &done);
        else if (P.cols <= 2560) rc = launch_sparsify_rounds<T, 512, 5>(P, stream, &done);
        else rc = launch_sparsify_rounds<T, 1024, 4>(P, stream, &done);
        if (rc != NMG_OK || done) return rc;
    }
    // What the rounds do not take (tiles of fewer than 16 columns, double, m > 8, more than 128
    // patterns) goes step by step: lane teams for tiles of up to 512 columns, else one
    // wavefront per tile (four tiles per workgroup) or four wavefronts per tile -- more of them
    // lose to the two workgroup barriers of every step (measured on 896-column tiles: 1 / 2 / 4 /
    // 8 / 16 wavefronts -> 17.6 / 12.6 / 10.9 / 21.1 / 69 ms for an 8192 x 8192 weight).
    if (P.cols <= 512 && P.n > 0) {
        // lane teams: about 16 to 32 columns per lane
        bool done = false;
        int rc;
        if (P.cols <= 32) rc = launch_sparsify_teams<T, 1>(P, stream, &done);
        else if (P.cols <= 64) rc = launch_sparsify_teams<T, 2>(P, stream, &done);
        else if (P.cols <= 128) rc = launch_sparsify_teams<T, 4>(P, stream, &done);
        else if (P.cols <= 256) rc = launch_sparsify_teams<T, 8>(P, stream, &done);
        else rc = launch_sparsify_teams<T, 16>(P, stream, &done);
        if (rc != NMG_OK || done) return rc;
    }
    if (P.cols <= 128) return launch_sparsify<T, 1, 4>(P, stream);
    return launch_sparsify<T, 4, 1>(P, stream);
}

static int check_common(const nmg_view *view, int n, int m, int g, int dtype, TileGeom *tg)
{
    NMG_REQUIRE(view != nullptr, NMG_ERR_ARG, "null view");
    NMG_REQUIRE(m >= 1 && m <= 64 && n >= 0 && n <= m && g >= 1, NMG_ERR_ARG,
                "invalid n:m:g = %d:%d:%d", n, m, g);
    NMG_REQUIRE(dtype_size(dtype) != 0, NMG_ERR_ARG, "invalid dtype code %d", dtype);
    NMG_REQUIRE(view->batch >= 0 && view->G >= 0 && view->S >= 0, NMG_ERR_ARG, "negative extent");
    int64_t c = binom(m, n);
    NMG_REQUIRE(c * g < 32768, NMG_ERR_ARG,
                "chunk_size * group_size = %lld must be < 2^15 (int16 indices)", (long long)(c * g));
    *tg = tile_geom(*view, n, m, g);
    return NMG_OK;
}

static ViewDev view_dev(const nmg_view &v, const TileGeom &tg)
{
    ViewDev d;
    d.G = v.G;
    d.S = v.S;
    d.stride_b = v.stride_b;
    d.stride_g = v.stride_g;
    d.stride_s = v.stride_s;
    d.num_chunks = tg.num_chunks;
    d.num_blocks = tg.num_blocks;
    return d;
}

// ------------------------------------------------------------------ element-wise companions

struct ScatterParams {
    const void *val;
    const int16_t *idx;
    void *dense;
    const int8_t *order;
    ViewDev view;
    int64_t outer;
    int n, m, g, c, cols;
};

// One thread per slot: writes the m values of its column (kept ones + zeros), so every element
// of the view is written exactly once (idx is a permutation of the tile's columns).
template <typename T> __global__ void to_dense_kernel(ScatterParams P)
{
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= P.outer * P.cols) return;
    const int64_t t = gid / P.cols;
    const int slot = (int)(gid - t * P.cols);
    const int p = slot / P.g;
    const int o = P.idx[gid];
    if (o < 0 || o >= P.cols) return;
    const int64_t tiles_per_b = P.view.num_chunks * P.view.num_blocks;
    const int64_t b = t / tiles_per_b;
    const int64_t rem = t - b * tiles_per_b;
    const int64_t kc = rem / P.view.num_blocks, mb = rem - kc * P.view.num_blocks;
    const int64_t gi = kc * P.cols + o;
    if (gi >= P.view.G) return;
    const T *v = (const T *)P.val + gid * P.n;
    T *base = (T *)P.dense + b * P.view.stride_b + gi * P.view.stride_g;
    int j = 0;
    for (int r = 0; r < P.m; r++) {
        T x = Zero<T>::v();
        if (j < P.n && P.order[p * P.n + j] == r) x = v[j++];
        const int64_t si = mb * P.m + r;
        if (si < P.view.S) base[si * P.view.stride_s] = x;
    }
}

template <typename T> __global__ void gather_kernel(ScatterParams P)
{
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= P.outer * P.cols) return;
    const int64_t t = gid / P.cols;
    const int slot = (int)(gid - t * P.cols);
    const int p = slot / P.g;
    const int o = P.idx[gid];
    const int64_t tiles_per_b = P.view.num_chunks * P.view.num_blocks;
    const int64_t b = t / tiles_per_b;
    const int64_t rem = t - b * tiles_per_b;
    const int64_t kc = rem / P.view.num_blocks, mb = rem - kc * P.view.num_blocks;
    const int64_t gi = kc * P.cols + o;
    T *v = (T *)P.val + gid * P.n;  // here val is the output
    const T *base = (const T *)P.dense + b * P.view.stride_b + gi * P.view.stride_g;
    for (int j = 0; j < P.n; j++) {
        const int64_t si = mb * P.m + P.order[p * P.n + j];
        T x = Zero<T>::v();
        if (o >= 0 && gi < P.view.G && si < P.view.S) x = base[si * P.view.stride_s];
        v[j] = x;
    }
}

struct RowpackParams {
    const void *val;
    const int16_t *idx;
    void *pk_val;
    void *pk_pat;
    int64_t G, nb, num_chunks, outer;
    int n, g, c, cols, pat_bytes;
};

template <typename T> __global__ void rowpack_kernel(RowpackParams P)
{
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= P.outer * P.cols) return;
    const int64_t t = gid / P.cols;
    const int slot = (int)(gid - t * P.cols);
    const int p = slot / P.g;
    const int o = P.idx[gid];
    const int64_t kc = t / P.nb, mb = t - kc * P.nb;
    const int64_t q = kc * P.cols + o;
    if (o < 0 || q >= P.G) return;
    const T *v = (const T *)P.val + gid * P.n;
    T *dst = (T *)P.pk_val + (q * P.nb + mb) * P.n;
    for (int j = 0; j < P.n; j++) dst[j] = v[j];
    if (P.pat_bytes == 1)
        ((uint8_t *)P.pk_pat)[q * P.nb + mb] = (uint8_t)p;
    else
        ((uint16_t *)P.pk_pat)[q * P.nb + mb] = (uint16_t)p;
}

}  // namespace nmg

using namespace nmg;

extern "C" int nmg_sparsify(const void *d_dense, const nmg_view *view, void *d_val, int16_t *d_idx,
                            int n, int m, int g, int dtype, void *stream)
{
    TileGeom tg;
    if (int rc = check_common(view, n, m, g, dtype, &tg)) return rc;
    if (tg.outer == 0) return NMG_OK;
    NMG_REQUIRE(d_dense && d_val && d_idx, NMG_ERR_ARG, "null device pointer");
    SparsifyParams P{};
    P.dense = d_dense;
    P.val = d_val;
    P.idx = d_idx;
    if (int rc = device_order(n, m, &P.order)) return rc;
    P.view = view_dev(*view, tg);
    P.outer = tg.outer;
    P.n = n;
    P.m = m;
    P.g = g;
    P.c = tg.c;
    P.cols = tg.cols;
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
    case NMG_F32: return dispatch_sparsify<float>(P, s);
    case NMG_F16: return dispatch_sparsify<__half>(P, s);
    case NMG_BF16: return dispatch_sparsify<__hip_bfloat16>(P, s);
    case NMG_F64: return dispatch_sparsify<double>(P, s);
    }
    return NMG_ERR_ARG;
}

template <template <typename> class K> struct Launch;

// Tiled forms of the two kernels above for views whose sparse dim is contiguous (the layout of
// a weight with n:m blocks along its rows' direction).  There a tile is c*g lines x m positions:
// one slot's m values are a few bytes of a line, so the slot-per-thread kernels touch every cache
// line of the dense tensor many times.  Here a workgroup takes NT tiles that are neighbours along
// the sparse dim -- a region of c*g lines x NT*m contiguous positions -- and moves it through
// LDS: rows of the region go to / come from global memory as contiguous segments, val / idx are
// contiguous for the NT tiles anyway.
struct TiledParams {
    ScatterParams sp;
    int nt;                      // tiles per workgroup
    int pitch;                   // elements per region row in LDS
    int groups_per_chunk;        // workgroups along the sparse dim
    uint64_t magic_cols, magic_g;
};

// GC: the group dim is the contiguous one instead (the reference's default orientation of a Linear
// weight).  The region of NT tiles that are neighbours along the sparse dim is then NT*m rows (one
// per position) of c*g contiguous columns; LDS holds it as [position][column].
template <typename T, bool GATHER, bool GC>
__global__ __launch_bounds__(256) void scatter_tiled_kernel(TiledParams Q)
{
    const ScatterParams &P = Q.sp;
    extern __shared__ __align__(16) unsigned char smem[];
    T *tile = (T *)smem;
    const int tid = threadIdx.x;
    const int n = P.n, m = P.m, cols = P.cols, nt = Q.nt, pitch = Q.pitch;
    // workgroup -> (batch, group-dim chunk, first block)
    const int64_t wg = blockIdx.x;
    const int64_t chunk_id = wg / Q.groups_per_chunk;
    const int64_t mb0 = (wg - chunk_id * Q.groups_per_chunk) * nt;
    const int64_t b = chunk_id / P.view.num_chunks, kc = chunk_id - b * P.view.num_chunks;
    const int64_t t0 = (b * P.view.num_chunks + kc) * P.view.num_blocks + mb0;
    const int tiles = (int)min((int64_t)nt, P.view.num_blocks - mb0);
    const int64_t g0 = kc * cols, s0 = mb0 * m;
    // region: `all_rows` rows of `width` contiguous elements; rows / valid_w of them exist
    const int width = GC ? cols : tiles * m;
    const int all_rows = GC ? tiles * m : cols;
    const int rows = GC ? (int)max((int64_t)0, min((int64_t)all_rows, P.view.S - s0))
                        : (int)min((int64_t)cols, P.view.G - g0);
    const int valid_w = GC ? (int)min((int64_t)cols, P.view.G - g0)
                           : (int)max((int64_t)0, min((int64_t)width, P.view.S - s0));
    const int64_t row_stride = GC ? P.view.stride_s : P.view.stride_g;
    T *dense = (T *)P.dense + b * P.view.stride_b + g0 * P.view.stride_g + s0 * P.view.stride_s;
    constexpr int V = 16 / sizeof(T);
    const bool vec = (row_stride % V) == 0 && ((GC ? g0 : s0) % V) == 0 && (P.view.stride_b % V) == 0 &&
                     ((uintptr_t)P.dense % 16) == 0 && (pitch % V) == 0;
    const int wv = (width + V - 1) / V;

    if (GATHER) {
        // region -> LDS (zeros beyond G / S)
        for (int i = tid; i < all_rows * wv; i += 256) {
            const int r = i / wv, cc = (i - r * wv) * V;
            T *dst = tile + r * pitch + cc;
            const T *src = dense + (int64_t)r * row_stride + cc;
            if (vec && r < rows && cc + V <= valid_w) {
                *(uint4 *)dst = *(const uint4 *)src;
            } else {
                for (int e = 0; e < V && cc + e < pitch; e++)
                    dst[e] = (r < rows && cc + e < valid_w) ? src[e] : Zero<T>::v();
            }
        }
    } else {
        const uint4 z = {0, 0, 0, 0};
        for (int i = tid; i < all_rows * pitch * (int)sizeof(T) / 16; i += 256) ((uint4 *)tile)[i] = z;
    }
    // the order table in LDS where it fits: a slot's positions are then one LDS read away instead
    // of a round trip to L2 behind the load of its index
    __shared__ int8_t s_ord[1024];
    const bool ord_lds = P.c * n <= 1024;
    if (ord_lds)
        for (int i = tid; i < P.c * n; i += 256) s_ord[i] = P.order[i];
    const int8_t *order = ord_lds ? s_ord : P.order;
    __syncthreads();
    // slots of the NT tiles: contiguous in val / idx (slot e of the workgroup is element
    // t0 * cols + e).  Four slots per thread are loaded before the first is used: index -> LDS ->
    // store is otherwise one round trip to HBM per slot and thread.
    const int total = tiles * cols;
    const int64_t at0 = t0 * (int64_t)cols;
    // NV > 0: n is the constant NV and a slot's NV values are one aligned word of 4 or 8 bytes -- one
    // load (issued with the index loads) or store per slot instead of NV of 2 or 4 bytes; NV = 0:
    // any n, value by value.
    auto run_slots = [&](auto nv_tag) {
        constexpr int NV = decltype(nv_tag)::value;
        constexpr int WB = NV * (int)sizeof(T);            // bytes of a slot's word
        using Word = typename std::conditional<WB == 8, uint2, uint32_t>::type;
        for (int base = tid; base < total; base += 4 * 256) {
            int o[4];
            Word vw[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int e = base + u * 256;
                o[u] = e < total ? (int)P.idx[at0 + e] : -1;
                if (!GATHER && NV > 0) vw[u] = ((const Word *)P.val)[at0 + (e < total ? e : 0)];
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int e = base + u * 256;
                if (e >= total) continue;
                const int tm = (int)(((uint64_t)e * Q.magic_cols) >> 32), slot = e - tm * cols;
                const int p = (int)(((uint64_t)slot * Q.magic_g) >> 32);
                const bool ok = o[u] >= 0 && o[u] < cols;
                T *v = (T *)P.val + (at0 + e) * n;
                // element (column oc, position ps of tile tm) of the region
                const int oc = ok ? o[u] : 0;
                auto at = [&](int ps) { return GC ? (tm * m + ps) * pitch + oc : oc * pitch + tm * m + ps; };
                if constexpr (NV > 0) {
                    T w[NV];
                    if (GATHER) {
#pragma unroll
                        for (int j = 0; j < NV; j++) w[j] = ok ? tile[at(order[p * NV + j])] : Zero<T>::v();
                        Word raw;
                        __builtin_memcpy(&raw, w, WB);
                        ((Word *)P.val)[at0 + e] = raw;
                    } else if (ok) {
                        __builtin_memcpy(w, &vw[u], WB);
#pragma unroll
                        for (int j = 0; j < NV; j++) tile[at(order[p * NV + j])] = w[j];
                    }
                } else {
                    if (GATHER) {
                        for (int j = 0; j < n; j++) v[j] = ok ? tile[at(order[p * n + j])] : Zero<T>::v();
                    } else if (ok) {
                        for (int j = 0; j < n; j++) tile[at(order[p * n + j])] = v[j];
                    }
                }
            }
        }
    };
    const int vbytes = n * (int)sizeof(T);
    const bool aligned = ((uintptr_t)P.val % 8) == 0;
    if (aligned && vbytes == 4 && n == 1) run_slots(std::integral_constant<int, (sizeof(T) == 4 ? 1 : 0)>{});
    else if (aligned && vbytes == 4 && n == 2) run_slots(std::integral_constant<int, (sizeof(T) == 2 ? 2 : 0)>{});
    else if (aligned && vbytes == 8 && n == 2) run_slots(std::integral_constant<int, (sizeof(T) == 4 ? 2 : 0)>{});
    else if (aligned && vbytes == 8 && n == 4) run_slots(std::integral_constant<int, (sizeof(T) == 2 ? 4 : 0)>{});
    else run_slots(std::integral_constant<int, 0>{});
    if (GATHER) return;
    __syncthreads();
    // LDS -> region
    for (int i = tid; i < rows * wv; i += 256) {
        const int r = i / wv, cc = (i - r * wv) * V;
        if (cc >= valid_w) continue;
        const T *src = tile + r * pitch + cc;
        T *dst = dense + (int64_t)r * row_stride + cc;
        if (vec && cc + V <= valid_w) {
            *(uint4 *)dst = *(const uint4 *)src;
        } else {
            for (int e = 0; e < V && cc + e < valid_w; e++) dst[e] = src[e];
        }
    }
}

// Launches the tiled kernel when it applies; *done tells whether it did.
template <typename T>
static int launch_scatter_tiled(bool gather, ScatterParams &P, hipStream_t s, bool *done)
{
    *done = false;
    const bool gc = P.view.stride_s != 1 && P.view.stride_g == 1;   // group dim contiguous
    if ((P.view.stride_s != 1 && !gc) || P.view.num_blocks < 4) return NMG_OK;
    // Tiles per workgroup: about 8 KiB of LDS (many small workgroups overlap each other's
    // latencies: a 16384 x 4096 2:4:16 gather takes 81 us with 10 tiles, 112 us with 64), but at
    // least 8 tiles so that a row of the region is a decent run of bytes, or 4 where 8 do not fit
    // (2:8:32 with 8 tiles of 896 lines: 139 us against 760 us for the slot-per-thread kernel).
    const int V = 16 / (int)sizeof(T);
    const int64_t per_tile = (int64_t)P.cols * P.m * (int64_t)sizeof(T);
    int nt = (int)std::min<int64_t>(64, (8 * 1024) / per_tile);
    if (nt < 8) nt = 8;
    nt = (int)std::min<int64_t>(nt, P.view.num_blocks);
    auto pitch_of = [&](int tiles, bool pad) { return (((gc ? P.cols : tiles * P.m) + V - 1) / V) * V + (pad ? V : 0); };
    bool pad = true;
    auto lds_of = [&](int tiles, bool pd) {
        return (size_t)(gc ? tiles * P.m : P.cols) * pitch_of(tiles, pd) * sizeof(T);
    };
    // group dim contiguous, gather: with one large workgroup per CU the slot-per-thread kernel is
    // ahead (8192^2 2:8:32, 115 KB: 110 us against 70), so the region must stay under 64 KB
    if (gc && gather && lds_of(nt, pad) > 64 * 1024) nt = (int)std::min<int64_t>(4, P.view.num_blocks);
    if (gc && gather && lds_of(nt, pad) > 64 * 1024) return NMG_OK;
    if (lds_of(nt, pad) > 150 * 1024) nt = (int)std::min<int64_t>(4, P.view.num_blocks);
    if (lds_of(nt, pad) > 150 * 1024) pad = false;    // rows without the vector of padding
    if (lds_of(nt, pad) > 150 * 1024 || nt < 4) return NMG_OK;
    TiledParams Q{};
    Q.sp = P;
    Q.nt = nt;
    Q.pitch = pitch_of(nt, pad);
    Q.groups_per_chunk = (int)((P.view.num_blocks + nt - 1) / nt);
    Q.magic_cols = (((uint64_t)1 << 32) + P.cols - 1) / P.cols;
    Q.magic_g = (((uint64_t)1 << 32) + P.g - 1) / P.g;
    const size_t lds = lds_of(nt, pad);
    if ((int64_t)nt * P.cols >= 65536) return NMG_OK;
    const int64_t chunks = P.outer / P.view.num_blocks;   // batches x group-dim chunks
    const int64_t grid = chunks * Q.groups_per_chunk;
    if (grid > 0x7fffffffLL) return NMG_OK;
    auto kern = gc ? (gather ? scatter_tiled_kernel<T, true, true> : scatter_tiled_kernel<T, false, true>)
                   : (gather ? scatter_tiled_kernel<T, true, false> : scatter_tiled_kernel<T, false, false>);
    if (lds > 64 * 1024)
        NMG_HIP_TRY(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, s, Q);
    NMG_HIP_TRY(hipGetLastError());
    *done = true;
    return NMG_OK;
}

static int launch_scatter(bool gather, const void *dense, const nmg_view *view, const void *val,
                          const int16_t *idx, int n, int m, int g, int dtype, void *stream)
{
    TileGeom tg;
    if (int rc = check_common(view, n, m, g, dtype, &tg)) return rc;
    if (tg.outer == 0) return NMG_OK;
    NMG_REQUIRE(dense && val && idx, NMG_ERR_ARG, "null device pointer");
    ScatterParams P{};
    P.val = val;
    P.idx = idx;
    P.dense = (void *)dense;
    if (int rc = device_order(n, m, &P.order)) return rc;
    P.view = view_dev(*view, tg);
    P.outer = tg.outer;
    P.n = n;
    P.m = m;
    P.g = g;
    P.c = tg.c;
    P.cols = tg.cols;
    const int64_t total = tg.outer * tg.cols;
    const int bs = 256;
    const int64_t grid = (total + bs - 1) / bs;
    NMG_REQUIRE(grid <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "too many slots");
    hipStream_t s = (hipStream_t)stream;
    {
        bool done = false;
        int rc = NMG_OK;
        switch (dtype) {
        case NMG_F32: rc = launch_scatter_tiled<float>(gather, P, s, &done); break;
        case NMG_F16: rc = launch_scatter_tiled<__half>(gather, P, s, &done); break;
        case NMG_BF16: rc = launch_scatter_tiled<__hip_bfloat16>(gather, P, s, &done); break;
        case NMG_F64: rc = launch_scatter_tiled<double>(gather, P, s, &done); break;
        }
        if (rc != NMG_OK || done) return rc;
    }
#define NMG_LAUNCH(T)                                                                         \
    do {                                                                                      \
        if (gather)                                                                           \
            hipLaunchKernelGGL(gather_kernel<T>, dim3((unsigned)grid), dim3(bs), 0, s, P);    \
        else                                                                                  \
            hipLaunchKernelGGL(to_dense_kernel<T>, dim3((unsigned)grid), dim3(bs), 0, s, P);  \
    } while (0)
    switch (dtype) {
    case NMG_F32: NMG_LAUNCH(float); break;
    case NMG_F16: NMG_LAUNCH(__half); break;
    case NMG_BF16: NMG_LAUNCH(__hip_bfloat16); break;
    case NMG_F64: NMG_LAUNCH(double); break;
    }
#undef NMG_LAUNCH
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

extern "C" int nmg_to_dense(const void *d_val, const int16_t *d_idx, void *d_dense,
                            const nmg_view *view, int n, int m, int g, int dtype, void *stream)
{
    return launch_scatter(false, d_dense, view, d_val, d_idx, n, m, g, dtype, stream);
}

extern "C" int nmg_gather(const void *d_dense, const nmg_view *view, const int16_t *d_idx,
                          void *d_val, int n, int m, int g, int dtype, void *stream)
{
    return launch_scatter(true, d_dense, view, d_val, d_idx, n, m, g, dtype, stream);
}

extern "C" int64_t nmg_rowpack_pat_bytes(int n, int m) { return binom(m, n) <= 256 ? 1 : 2; }

extern "C" int nmg_rowpack(const void *d_val, const int16_t *d_idx, int64_t G, int64_t S,
                           void *d_pk_val, void *d_pk_pat, int n, int m, int g, int dtype,
                           void *stream)
{
    nmg_view v{1, G, S, 0, S, 1};
    TileGeom tg;
    if (int rc = check_common(&v, n, m, g, dtype, &tg)) return rc;
    NMG_REQUIRE(dtype != NMG_F64, NMG_ERR_UNSUPPORTED, "rowpack supports f32/f16/bf16");
    if (tg.outer == 0) return NMG_OK;
    NMG_REQUIRE(d_val && d_idx && d_pk_val && d_pk_pat, NMG_ERR_ARG, "null device pointer");
    RowpackParams P{};
    P.val = d_val;
    P.idx = d_idx;
    P.pk_val = d_pk_val;
    P.pk_pat = d_pk_pat;
    P.G = G;
    P.nb = tg.num_blocks;
    P.num_chunks = tg.num_chunks;
    P.outer = tg.outer;
    P.n = n;
    P.g = g;
    P.c = tg.c;
    P.cols = tg.cols;
    P.pat_bytes = (int)nmg_rowpack_pat_bytes(n, m);
    const int64_t total = tg.outer * tg.cols;
    const int bs = 256;
    const int64_t grid = (total + bs - 1) / bs;
    NMG_REQUIRE(grid <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "too many slots");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
    case NMG_F32: hipLaunchKernelGGL(rowpack_kernel<float>, dim3((unsigned)grid), dim3(bs), 0, s, P); break;
    case NMG_F16: hipLaunchKernelGGL(rowpack_kernel<__half>, dim3((unsigned)grid), dim3(bs), 0, s, P); break;
    case NMG_BF16: hipLaunchKernelGGL(rowpack_kernel<__hip_bfloat16>, dim3((unsigned)grid), dim3(bs), 0, s, P); break;
    }
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}
