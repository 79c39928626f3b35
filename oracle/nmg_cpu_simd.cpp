// nmg_cpu_simd.cpp -- SIMD + OpenMP CPU restatement of the reference's nmg spmm.
//
// TEST / BASELINE INFRASTRUCTURE ONLY: used as the "cpu_baseline" leg of the
// benchmark and as a second checker in tests; never loaded by the product.
//
// Follows src/sten/grouped_nm/dace_gnm_mult.py:
//   :141-256  AVX-512 microkernel (n x 4 vector accumulators, flush-on-row-change)
//   :23-138   AVX2 twin (8-wide)
//   :724-805  loop nest: parallel over N-slabs of 4*v columns; per slab a local
//             copy of B[:, slab] and a local C; sequential K-tiles; M-blocks;
//             K-remainder tile last; C[:, slab] = Clocal
//   :599-613  tile constants (v = 16|8, 4 vectors per slab, N % (4*v) == 0)
// The reference bakes every shape into generated code; here n is a template
// parameter and the remaining sizes are run-time arguments.
#include <immintrin.h>
#include <omp.h>

#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <vector>

extern "C" int64_t nmg_ref_order(int n, int m, int8_t *out);
extern "C" int64_t nmg_ref_chunk(int n, int m);

#if defined(__AVX512F__)
typedef __m512 vec_t;
static constexpr int VW = 16;
static inline vec_t vzero() { return _mm512_setzero_ps(); }
static inline vec_t vload(const float *p) { return _mm512_loadu_ps(p); }
static inline void vstore(float *p, vec_t v) { _mm512_storeu_ps(p, v); }
static inline vec_t vbcast(float a) { return _mm512_set1_ps(a); }
static inline vec_t vfma(vec_t a, vec_t b, vec_t c) { return _mm512_fmadd_ps(a, b, c); }
static inline vec_t vadd(vec_t a, vec_t b) { return _mm512_add_ps(a, b); }
static const char *kKernelName = "avx512";
#else
typedef __m256 vec_t;
static constexpr int VW = 8;
static inline vec_t vzero() { return _mm256_setzero_ps(); }
static inline vec_t vload(const float *p) { return _mm256_loadu_ps(p); }
static inline void vstore(float *p, vec_t v) { _mm256_storeu_ps(p, v); }
static inline vec_t vbcast(float a) { return _mm256_set1_ps(a); }
static inline vec_t vfma(vec_t a, vec_t b, vec_t c) { return _mm256_fmadd_ps(a, b, c); }
static inline vec_t vadd(vec_t a, vec_t b) { return _mm256_add_ps(a, b); }
static const char *kKernelName = "avx2";
#endif

static constexpr int NV = 4;           // vectors per slab (num_vectors_b)
static constexpr int SLAB = NV * VW;   // columns per N-slab

// One (K-tile, M-block, N-slab) microkernel.  Bt: local B rows of this K-tile
// [tileK, SLAB]; Ct: local C rows of this M-block [m, SLAB].
template <int NN>
static inline void microkernel(const float *av, const int16_t *ai, const float *Bt, float *Ct,
                               const int8_t *order, int64_t c, int g, int64_t Krem, bool in_rem)
{
    vec_t acc[NN][NV];
    for (int j = 0; j < NN; j++)
        for (int q = 0; q < NV; q++) acc[j][q] = vzero();
    for (int64_t p = 0; p < c; p++) {
        for (int s = 0; s < g; s++) {
            int64_t slot = p * g + s;
            int16_t r = ai[slot];
            if (in_rem && (r < 0 || r >= Krem)) break;
            const float *brow = Bt + (int64_t)r * SLAB;
            vec_t va[NN];
            for (int j = 0; j < NN; j++) va[j] = vbcast(av[slot * NN + j]);
            for (int q = 0; q < NV; q++) {
                vec_t vb = vload(brow + q * VW);
                for (int j = 0; j < NN; j++) acc[j][q] = vfma(va[j], vb, acc[j][q]);
            }
        }
        bool last = (p == c - 1);
        for (int j = 0; j < NN; j++) {
            if (last || order[p * NN + j] != order[(p + 1) * NN + j]) {
                float *crow = Ct + (int64_t)order[p * NN + j] * SLAB;
                for (int q = 0; q < NV; q++) {
                    vstore(crow + q * VW, vadd(vload(crow + q * VW), acc[j][q]));
                    acc[j][q] = vzero();
                }
            }
        }
    }
}

template <int NN>
static int spmm_impl(const float *A_val, const int16_t *A_idx, const float *B, int64_t ldb,
                     float *C, int64_t ldc, int64_t M, int64_t K, int64_t N, int m, int g)
{
    const int64_t c = nmg_ref_chunk(NN, m), tileK = c * g;
    const int64_t DMI = (M + m - 1) / m, DKI = (K + tileK - 1) / tileK, Krem = K % tileK;
    const int64_t Mpad = DMI * m, nslabs = N / SLAB;
    std::vector<int8_t> order((size_t)(c * NN));
    nmg_ref_order(NN, m, order.data());
#pragma omp parallel
    {
        std::vector<float> Bl((size_t)(DKI * tileK * SLAB), 0.f), Cl((size_t)(Mpad * SLAB));
#pragma omp for schedule(static)
        for (int64_t bn = 0; bn < nslabs; bn++) {
            for (int64_t k = 0; k < K; k++)
                std::memcpy(&Bl[(size_t)(k * SLAB)], B + k * ldb + bn * SLAB, sizeof(float) * SLAB);
            std::fill(Cl.begin(), Cl.end(), 0.f);
            for (int64_t bk = 0; bk < DKI; bk++) {
                bool in_rem = (Krem != 0) && (bk == DKI - 1);
                for (int64_t bm = 0; bm < DMI; bm++)
                    microkernel<NN>(A_val + (bk * DMI + bm) * tileK * NN,
                                    A_idx + (bk * DMI + bm) * tileK, &Bl[(size_t)(bk * tileK * SLAB)],
                                    &Cl[(size_t)(bm * m * SLAB)], order.data(), c, g, Krem, in_rem);
            }
            for (int64_t r = 0; r < Mpad; r++)
                std::memcpy(C + r * ldc + bn * SLAB, &Cl[(size_t)(r * SLAB)], sizeof(float) * SLAB);
        }
    }
    return 0;
}

extern "C" const char *nmg_simd_kernel_name() { return kKernelName; }
extern "C" int nmg_simd_slab() { return SLAB; }
extern "C" int nmg_simd_threads() { return omp_get_max_threads(); }

// C[Mpad, N] = to_dense(A) @ B; layouts as nmg_ref_spmm_f32.  N must be a
// multiple of 4*v (dace_gnm_mult.py:605-606); returns 2 otherwise.
extern "C" int nmg_simd_spmm_f32(const float *A_val, const int16_t *A_idx, const float *B,
                                 int64_t ldb, float *C, int64_t ldc, int64_t M, int64_t K,
                                 int64_t N, int n, int m, int g)
{
    if (N % SLAB != 0) return 2;
    switch (n) {
    case 1: return spmm_impl<1>(A_val, A_idx, B, ldb, C, ldc, M, K, N, m, g);
    case 2: return spmm_impl<2>(A_val, A_idx, B, ldb, C, ldc, M, K, N, m, g);
    case 3: return spmm_impl<3>(A_val, A_idx, B, ldb, C, ldc, M, K, N, m, g);
    case 4: return spmm_impl<4>(A_val, A_idx, B, ldb, C, ldc, M, K, N, m, g);
    case 5: return spmm_impl<5>(A_val, A_idx, B, ldb, C, ldc, M, K, N, m, g);
    case 6: return spmm_impl<6>(A_val, A_idx, B, ldb, C, ldc, M, K, N, m, g);
    default: return 3;
    }
}
