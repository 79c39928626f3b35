// Ungrouped ("perfect") n:m: every block of m consecutive indices of the sparse dim keeps its n
// largest magnitudes, independently of its neighbours -- the upper bound of what a grouped n:m
// tensor can preserve, and a second sparsifier of the format family.
//
// The dense tensor is seen as [outer, S, inner] (dims before / at / after the sparse dim of a
// contiguous tensor).  Outputs have the reference's shapes: val [outer, nb, n, inner] and idx
// [outer, nb, n, inner] int64 (position inside the block), kept values in descending magnitude;
// equal magnitudes keep the lower position first (the reference sorts with an unstable argsort,
// so it does not define that order).  HBM-bound: one read of the tensor, n/m of it written.
#include "nmg_common.h"

namespace nmg {

struct PerfectParams {
    const void *dense;
    void *val;
    int64_t *idx;
    int64_t outer, S, inner, nb;
    int n, m;
};

template <typename T> struct Mag {
    __device__ static float of(T x) { return fabsf(to_f32(x)); }
};
template <> struct Mag<double> {
    __device__ static double of(double x) { return fabs(x); }
};

constexpr int PF_MAX_M = 64;

template <typename T> __global__ __launch_bounds__(256) void perfect_nm_kernel(PerfectParams P)
{
    // one thread per (outer, block, inner); inner fastest, so reads and writes of a wavefront are
    // contiguous whenever the sparse dim is not the last one
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t total = P.outer * P.nb * P.inner;
    if (gid >= total) return;
    const int64_t i = gid % P.inner, ob = gid / P.inner;
    const int64_t b = ob % P.nb, o = ob / P.nb;
    const T *src = (const T *)P.dense + (o * P.S + b * P.m) * P.inner + i;
    T *val = (T *)P.val + (ob * P.n) * P.inner + i;
    int64_t *idx = P.idx + (ob * P.n) * P.inner + i;
    const int live = (int)min((int64_t)P.m, P.S - b * P.m);   // positions beyond S are zero padding
    uint64_t taken = 0;
    for (int j = 0; j < P.n; j++) {
        int best = -1;
        decltype(Mag<T>::of(src[0])) best_mag = -1;
        T best_val = Zero<T>::v();
        for (int r = 0; r < P.m; r++) {
            if ((taken >> r) & 1) continue;
            const T v = r < live ? src[(int64_t)r * P.inner] : Zero<T>::v();
            auto a = Mag<T>::of(v);
            if (!(a == a)) a = INFINITY;   // NaN counts as the largest magnitude, as in a descending sort
            if (a > best_mag) {   // strict: the lower position wins a tie
                best_mag = a;
                best = r;
                best_val = v;
            }
        }
        taken |= (uint64_t)1 << best;
        val[(int64_t)j * P.inner] = best_val;
        idx[(int64_t)j * P.inner] = best;
    }
}

template <typename T> __global__ __launch_bounds__(256) void perfect_nm_to_dense_kernel(PerfectParams P)
{
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t total = P.outer * P.nb * P.inner;
    if (gid >= total) return;
    const int64_t i = gid % P.inner, ob = gid / P.inner;
    const int64_t b = ob % P.nb, o = ob / P.nb;
    T *dst = (T *)P.dense + (o * P.S + b * P.m) * P.inner + i;
    const T *val = (const T *)P.val + (ob * P.n) * P.inner + i;
    const int64_t *idx = P.idx + (ob * P.n) * P.inner + i;
    const int live = (int)min((int64_t)P.m, P.S - b * P.m);
    for (int r = 0; r < live; r++) dst[(int64_t)r * P.inner] = Zero<T>::v();
    for (int j = 0; j < P.n; j++) {
        const int64_t r = idx[(int64_t)j * P.inner];
        if (r >= 0 && r < live) dst[r * P.inner] = val[(int64_t)j * P.inner];
    }
}

static int fill_params(PerfectParams &P, const void *dense, void *val, int64_t *idx, int64_t outer, int64_t S,
                       int64_t inner, int n, int m)
{
    NMG_REQUIRE(m >= 1 && m <= PF_MAX_M && n >= 0 && n <= m, NMG_ERR_ARG, "invalid n:m = %d:%d (m <= %d)", n, m,
                PF_MAX_M);
    NMG_REQUIRE(outer >= 0 && S >= 0 && inner >= 0, NMG_ERR_ARG, "negative extent");
    P.dense = dense;
    P.val = val;
    P.idx = idx;
    P.outer = outer;
    P.S = S;
    P.inner = inner;
    P.nb = (S + m - 1) / m;
    P.n = n;
    P.m = m;
    return NMG_OK;
}

}  // namespace nmg

using namespace nmg;

extern "C" int nmg_perfect_nm(const void *d_dense, int64_t outer, int64_t S, int64_t inner, void *d_val,
                              int64_t *d_idx, int n, int m, int dtype, void *stream)
{
    PerfectParams P{};
    if (int rc = fill_params(P, d_dense, d_val, d_idx, outer, S, inner, n, m)) return rc;
    NMG_REQUIRE(dtype_size(dtype) != 0, NMG_ERR_ARG, "unknown dtype %d", dtype);
    const int64_t total = P.outer * P.nb * P.inner;
    if (total == 0 || n == 0) return NMG_OK;
    NMG_REQUIRE(d_dense && d_val && d_idx, NMG_ERR_ARG, "null device pointer");
    const int64_t blocks = (total + 255) / 256;
    NMG_REQUIRE(blocks <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "tensor too large for one launch");
    const dim3 grid((unsigned)blocks), block(256);
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
    case NMG_F32: hipLaunchKernelGGL(perfect_nm_kernel<float>, grid, block, 0, s, P); break;
    case NMG_F16: hipLaunchKernelGGL(perfect_nm_kernel<__half>, grid, block, 0, s, P); break;
    case NMG_BF16: hipLaunchKernelGGL(perfect_nm_kernel<__hip_bfloat16>, grid, block, 0, s, P); break;
    default: hipLaunchKernelGGL(perfect_nm_kernel<double>, grid, block, 0, s, P); break;
    }
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

extern "C" int nmg_perfect_nm_to_dense(const void *d_val, const int64_t *d_idx, int64_t outer, int64_t S,
                                       int64_t inner, void *d_dense, int n, int m, int dtype, void *stream)
{
    PerfectParams P{};
    if (int rc = fill_params(P, d_dense, (void *)d_val, (int64_t *)d_idx, outer, S, inner, n, m)) return rc;
    NMG_REQUIRE(dtype_size(dtype) != 0, NMG_ERR_ARG, "unknown dtype %d", dtype);
    const int64_t total = P.outer * P.nb * P.inner;
    if (total == 0) return NMG_OK;
    NMG_REQUIRE(d_dense && (n == 0 || (d_val && d_idx)), NMG_ERR_ARG, "null device pointer");
    const int64_t blocks = (total + 255) / 256;
    NMG_REQUIRE(blocks <= 0x7fffffffLL, NMG_ERR_UNSUPPORTED, "tensor too large for one launch");
    const dim3 grid((unsigned)blocks), block(256);
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
    case NMG_F32: hipLaunchKernelGGL(perfect_nm_to_dense_kernel<float>, grid, block, 0, s, P); break;
    case NMG_F16: hipLaunchKernelGGL(perfect_nm_to_dense_kernel<__half>, grid, block, 0, s, P); break;
    case NMG_BF16: hipLaunchKernelGGL(perfect_nm_to_dense_kernel<__hip_bfloat16>, grid, block, 0, s, P); break;
    default: hipLaunchKernelGGL(perfect_nm_to_dense_kernel<double>, grid, block, 0, s, P); break;
    }
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}
