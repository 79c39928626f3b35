/*
 * nmg_oracle.c -- CPU restatement of the reference's grouped n:m ("nmg") algorithms.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker that the HIP path is
 * compared against; it is never linked into, imported by, or called from the
 * product (sten_amd/).  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load the library built from it.
 *
 * Every function names the reference lines it restates (paths are relative to
 * the reference repository root):
 *
 *   nmg_ref_order        src/sten/grouped_nm/grouped_nm_tensor.py:37-50   (make_n_m)
 *   nmg_ref_sparsify_*   src/sten/grouped_nm/grouped_nm_tensor.py:255-297 (CPU sparsifier)
 *   nmg_ref_to_dense_*   src/sten/grouped_nm/grouped_nm_tensor.py:742-757 (CPU to_dense)
 *   nmg_ref_gather_*     src/sten/grouped_nm/grouped_nm_tensor.py:908-951 (clone_layout, disabled)
 *   nmg_ref_spmm_f32     src/sten/grouped_nm/dace_gnm_mult.py:141-256 (microkernel),
 *                        :724-805 (loop nest), :599-613 (tile constants)
 *
 * Parity status of each function (what pins it besides its own text):
 *   nmg_ref_order      -- pinned by tables traced by hand through the recursion
 *                         (tests/golden/hand_traced.json: 1:2, 1:3, 2:3, 1:4, 2:4,
 *                         3:4, 2:5, 3:5, 2:6, 3:6, 1:8, 2:8, 3:8, 4:8, 7:8), by the
 *                         1:m closed form, and for every (n,m) by the validity
 *                         invariants (increasing tuples, neighbours differ in one
 *                         slot, count C(m,n)).  For the other (n,m) with more than
 *                         8 patterns (5:8, 6:8, m > 8) the exact order is fixed only
 *                         by the recursion itself: "parity unpinned" beyond the
 *                         invariants for those.
 *   nmg_ref_sparsify_* -- pinned by hand-worked tiles, the n==m closed form, the
 *                         all-zero closed form and a brute-force matcher on tiny
 *                         tiles (tests/test_oracle.py).
 *   nmg_ref_to_dense_* -- pinned by the scatter closed form and round trips.
 *   nmg_ref_spmm_f32   -- pinned by the equation the reference asserts,
 *                         C[:M,:N] == to_dense(A) @ B (dace_gnm_mult.py:1123,1189-1199).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ order */

static int64_t binom(int m, int n)
{
    if (n < 0 || n > m) return 0;
    int64_t r = 1;
    for (int i = 1; i <= n; i++) r = r * (m - n + i) / i;
    return r;
}

int64_t nmg_ref_chunk(int n, int m) { return binom(m, n); }

/* make_n_m(n, m, special): returns number of tuples written to out[count][n].
 * grouped_nm_tensor.py:37-50:
 *   n==m or n==0            -> [range(n)]
 *   first  = make(n, m-1, True), reversed iff special
 *   second = [t + (m-1,) for t in make(n-1, m-1, not special)]
 *   result = first + second                                              */
static int64_t order_rec(int n, int m, int special, int8_t *out)
{
    if (n == m || n == 0) {
        for (int j = 0; j < n; j++) out[j] = (int8_t)j;
        return 1;
    }
    int64_t c1 = order_rec(n, m - 1, 1, out);
    if (special) {
        for (int64_t a = 0, b = c1 - 1; a < b; a++, b--)
            for (int j = 0; j < n; j++) {
                int8_t t = out[a * n + j];
                out[a * n + j] = out[b * n + j];
                out[b * n + j] = t;
            }
    }
    int64_t c2max = binom(m - 1, n - 1);
    int8_t *tmp = (int8_t *)malloc((size_t)(c2max * (n > 1 ? n - 1 : 1)));
    int64_t c2 = order_rec(n - 1, m - 1, !special, tmp);
    for (int64_t i = 0; i < c2; i++) {
        for (int j = 0; j < n - 1; j++) out[(c1 + i) * n + j] = tmp[i * (n - 1) + j];
        out[(c1 + i) * n + (n - 1)] = (int8_t)(m - 1);
    }
    free(tmp);
    return c1 + c2;
}

/* out must hold C(m,n)*n int8.  Returns C(m,n), or -1 on bad arguments. */
int64_t nmg_ref_order(int n, int m, int8_t *out)
{
    if (n < 0 || n > m || m > 127) return -1;
    return order_rec(n, m, 0, out);
}

/* --------------------------------------------------------------- sparsify */

#define DEFINE_SPARSIFY(NAME, T, ABS)                                                      \
    typedef struct {                                                                       \
        T acc;                                                                             \
        int16_t o;                                                                         \
        int16_t p;                                                                         \
    } cand_##NAME;                                                                         \
    /* std::greater<> on tuple(acc, orig_idx, nnz_idx): descending lexicographic */       \
    static int cmp_##NAME(const void *a_, const void *b_)                                  \
    {                                                                                      \
        const cand_##NAME *a = (const cand_##NAME *)a_, *b = (const cand_##NAME *)b_;      \
        if (a->acc > b->acc) return -1;                                                    \
        if (a->acc < b->acc) return 1;                                                     \
        if (a->o != b->o) return a->o > b->o ? -1 : 1;                                     \
        if (a->p != b->p) return a->p > b->p ? -1 : 1;                                     \
        return 0;                                                                          \
    }                                                                                      \
    /* dense: [outer, c, g, m]; val: [outer, c, g, n]; idx: [outer, c, g] (int16).         \
     * val/idx must be pre-filled by the caller with 0 / -1 as the reference               \
     * driver does (grouped_nm_tensor.py:652-655); every slot is overwritten.  */          \
    int NAME(const T *dense, T *val, int16_t *idx, int64_t outer, int n, int m, int g)     \
    {                                                                                      \
        int64_t c = binom(m, n);                                                           \
        if (c * g >= 32768) return 1; /* grouped_nm_tensor.py:229 */                       \
        int8_t *order = (int8_t *)malloc((size_t)(c * (n ? n : 1)));                       \
        nmg_ref_order(n, m, order);                                                        \
        int64_t cols = c * g, nacc = c * cols;                                             \
        cand_##NAME *accs = (cand_##NAME *)malloc(sizeof(cand_##NAME) * (size_t)nacc);     \
        int16_t *cnt = (int16_t *)malloc(sizeof(int16_t) * (size_t)c);                     \
        char *taken = (char *)malloc((size_t)cols);                                        \
        for (int64_t t = 0; t < outer; t++) {                                              \
            const T *d = dense + t * cols * m;                                             \
            T *v = val + t * cols * n;                                                     \
            int16_t *ix = idx + t * cols;                                                  \
            for (int64_t o = 0; o < cols; o++)                                             \
                for (int64_t p = 0; p < c; p++) {                                          \
                    T acc = 0;                                                             \
                    for (int j = 0; j < n; j++) acc += ABS(d[order[p * n + j] + o * m]);   \
                    cand_##NAME *e = &accs[p + o * c];                                     \
                    e->acc = acc;                                                          \
                    e->o = (int16_t)o;                                                     \
                    e->p = (int16_t)p;                                                     \
                }                                                                          \
            qsort(accs, (size_t)nacc, sizeof(cand_##NAME), cmp_##NAME);                    \
            memset(cnt, 0, sizeof(int16_t) * (size_t)c);                                   \
            memset(taken, 0, (size_t)cols);                                                \
            for (int64_t a = 0; a < nacc; a++) {                                           \
                int o = accs[a].o, p = accs[a].p;                                          \
                if (!taken[o] && cnt[p] < g) {                                             \
                    taken[o] = 1;                                                          \
                    int slot = cnt[p]++ + p * g;                                           \
                    ix[slot] = (int16_t)o;                                                 \
                    for (int j = 0; j < n; j++) v[j + slot * n] = d[order[p * n + j] + o * m]; \
                }                                                                          \
            }                                                                              \
        }                                                                                  \
        free(order);                                                                       \
        free(accs);                                                                        \
        free(cnt);                                                                         \
        free(taken);                                                                       \
        return 0;                                                                          \
    }

DEFINE_SPARSIFY(nmg_ref_sparsify_f32, float, fabsf)
DEFINE_SPARSIFY(nmg_ref_sparsify_f64, double, fabs)

/* --------------------------------------------------------------- to_dense */

#define DEFINE_TO_DENSE(NAME, T)                                                           \
    /* dense[t, idx[t,s]*m + order[s/g][j]] = val[t,s,j]; dense pre-zeroed by caller */    \
    int NAME(const T *val, const int16_t *idx, T *dense, int64_t outer, int n, int m, int g) \
    {                                                                                      \
        int64_t c = binom(m, n), cols = c * g;                                             \
        int8_t *order = (int8_t *)malloc((size_t)(c * (n ? n : 1)));                       \
        nmg_ref_order(n, m, order);                                                        \
        for (int64_t t = 0; t < outer; t++)                                                \
            for (int64_t p = 0; p < c; p++)                                                \
                for (int64_t s = 0; s < g; s++) {                                          \
                    int64_t slot = s + p * g;                                              \
                    int16_t o = idx[t * cols + slot];                                      \
                    for (int j = 0; j < n; j++)                                            \
                        dense[t * cols * m + order[p * n + j] + o * m] =                   \
                            val[t * cols * n + j + slot * n];                              \
                }                                                                          \
        free(order);                                                                       \
        return 0;                                                                          \
    }

DEFINE_TO_DENSE(nmg_ref_to_dense_f32, float)
DEFINE_TO_DENSE(nmg_ref_to_dense_f64, double)

/* ----------------------------------------------- same-pattern re-compress */

/* The intended semantics of clone_layout (grouped_nm_tensor.py:908-951, disabled
 * upstream): keep idx, re-gather values of a new dense tensor at the kept
 * positions: val[t,s,j] = dense[t, idx[t,s]*m + order[s/g][j]].            */
int nmg_ref_gather_f32(const float *dense, const int16_t *idx, float *val, int64_t outer, int n,
                       int m, int g)
{
    int64_t c = binom(m, n), cols = c * g;
    int8_t *order = (int8_t *)malloc((size_t)(c * (n ? n : 1)));
    nmg_ref_order(n, m, order);
    for (int64_t t = 0; t < outer; t++)
        for (int64_t slot = 0; slot < cols; slot++) {
            int64_t p = slot / g;
            int16_t o = idx[t * cols + slot];
            for (int j = 0; j < n; j++)
                val[t * cols * n + slot * n + j] = dense[t * cols * m + o * m + order[p * n + j]];
        }
    free(order);
    return 0;
}

/* ------------------------------------------------------------------- spmm */

/* C[Mpad, N] (row-major, fully overwritten) = to_dense(A) @ B, A given as
 *   A_val [DKI, DMI, c, g, n] f32, A_idx [DKI, DMI, c, g] i16
 * (dace_gnm_mult.py:615-616) i.e. n:m blocks along M, groups of g columns along
 * K share a pattern; B is [K, N] row-major with leading dimension ldb.
 *
 * Scalar restatement of the AVX microkernel: for one (K-tile, M-block) keep n
 * accumulator rows; walk the patterns in order; after pattern p flush
 * accumulator j to row order[p][j] iff that row differs in pattern p+1 (or p is
 * the last one) (dace_gnm_mult.py:228-246).  In the K-remainder tile a slot
 * whose index lies outside [0, Krem) ends the pattern's slot loop
 * (dace_gnm_mult.py:205-208).  K-tiles are visited sequentially, the remainder
 * tile last (dace_gnm_mult.py:750-779).                                    */
int nmg_ref_spmm_f32(const float *A_val, const int16_t *A_idx, const float *B, int64_t ldb,
                     float *C, int64_t ldc, int64_t M, int64_t K, int64_t N, int n, int m, int g)
{
    int64_t c = binom(m, n), tileK = c * g;
    int64_t DMI = (M + m - 1) / m, DKI = (K + tileK - 1) / tileK;
    int64_t Krem = K % tileK;
    int8_t *order = (int8_t *)malloc((size_t)(c * (n ? n : 1)));
    nmg_ref_order(n, m, order);
    float *acc = (float *)malloc(sizeof(float) * (size_t)(n ? n : 1) * (size_t)N);
    for (int64_t r = 0; r < DMI * m; r++) memset(C + r * ldc, 0, sizeof(float) * (size_t)N);
    for (int64_t bk = 0; bk < DKI; bk++) {
        int in_rem = (Krem != 0) && (bk == DKI - 1);
        const float *Bt = B + bk * tileK * ldb;
        for (int64_t bm = 0; bm < DMI; bm++) {
            const float *av = A_val + (bk * DMI + bm) * tileK * n;
            const int16_t *ai = A_idx + (bk * DMI + bm) * tileK;
            float *Ct = C + bm * m * ldc;
            memset(acc, 0, sizeof(float) * (size_t)n * (size_t)N);
            for (int64_t p = 0; p < c; p++) {
                for (int64_t s = 0; s < g; s++) {
                    int64_t slot = p * g + s;
                    int16_t r = ai[slot];
                    if (in_rem && (r < 0 || r >= Krem)) break;
                    const float *brow = Bt + (int64_t)r * ldb;
                    for (int j = 0; j < n; j++) {
                        float a = av[slot * n + j];
                        float *accj = acc + (int64_t)j * N;
                        for (int64_t q = 0; q < N; q++) accj[q] = fmaf(a, brow[q], accj[q]);
                    }
                }
                for (int j = 0; j < n; j++) {
                    int last = (p == c - 1);
                    if (last || order[p * n + j] != order[(p + 1) * n + j]) {
                        float *crow = Ct + (int64_t)order[p * n + j] * ldc;
                        float *accj = acc + (int64_t)j * N;
                        for (int64_t q = 0; q < N; q++) crow[q] += accj[q];
                        if (!last) memset(accj, 0, sizeof(float) * (size_t)N);
                    }
                }
            }
        }
    }
    free(order);
    free(acc);
    return 0;
}
