// nmg x dense matmul, generic path: the weight tile is decompressed from the rowpack operand
// into LDS as a dense tile and multiplied with dense MFMA (32x32 blocks, fp32 accumulate).
// Serves every n:m, both reduction directions and f32/f16/bf16.
//
//   Y[tok, o] = sum_k X[tok, k] * Wd[o, k] (+ bias[o])
//   reduce_sparse = 1:  o = line q of the group dim, k runs along the sparse dim
//   reduce_sparse = 0:  o runs along the sparse dim, k = line q of the group dim
//
// Workgroup tile: 128 tokens x 128 outputs, K step 64 (16-bit) / 32 (f32); 4 wavefronts in a
// 2x2 grid, each owning 64x64 = 2x2 MFMA blocks.  X is the MFMA A operand (rows = tokens), the
// weight tile the B operand (columns = outputs), so a wavefront's lanes hold consecutive
// outputs of one token row and the stores to row-major Y are contiguous.
#include "nmg_common.h"

#include <cstdlib>

namespace nmg {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

template <typename T> struct Mma;
template <> struct Mma<__half> {
    static constexpr int KPI = 16, EPL = 8, BK = 64, PAD = 8;
    using Frag = f16x8;
    __device__ static f32x16 run(Frag a, Frag b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mma<__hip_bfloat16> {
    static constexpr int KPI = 16, EPL = 8, BK = 64, PAD = 8;
    using Frag = bf16x8;
    __device__ static f32x16 run(Frag a, Frag b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mma<float> {
    static constexpr int KPI = 2, EPL = 1, BK = 32, PAD = 1;
    using Frag = float;
    __device__ static f32x16 run(Frag a, Frag b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
};

__device__ __forceinline__ void from_f32(float x, float &o) { o = x; }
__device__ __forceinline__ void from_f32(float x, __half &o) { o = __float2half(x); }
__device__ __forceinline__ void from_f32(float x, __hip_bfloat16 &o) { o = __float2bfloat16(x); }

struct SpmmParams {
    const void *pk_val;
    const void *pk_pat;
    const int8_t *order;
    const void *x;
    void *y;
    const void *bias;
    int64_t G, S, nb, T, ldx, ldy;
    int64_t K, O;  // reduction extent, output features
    int n, m, c, pat_bytes;
};

// Tile BM tokens x BN outputs per workgroup of 2 x 2 wavefronts: 128 x 128, or 64 x 64 for products
// whose 128 x 128 tiles would leave most of the CUs without work.
template <typename T, bool REDUCE_SPARSE, int BM, int BN>
__global__ __launch_bounds__(256) void spmm_mfma_kernel(SpmmParams P)
{
    using M = Mma<T>;
    constexpr int WMT = BM / 2, WNT = BN / 2;   // tokens x outputs per wavefront
    constexpr int MI = WMT / 32, NJ = WNT / 32; // 32 x 32 accumulator blocks per wavefront
    constexpr int BK = M::BK, LDSW = BK + M::PAD;
    __shared__ __align__(16) T As[BM * LDSW];
    __shared__ __align__(16) T Bs[BN * LDSW];
    __shared__ int8_t s_order[kOrderSlotBytes / 4];  // c*n <= 2048 served from LDS, else global

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t tok0 = (int64_t)blockIdx.y * BM, o0 = (int64_t)blockIdx.x * BN;
    const int n = P.n, m = P.m;
    const bool order_in_lds = P.c * n <= (int)sizeof(s_order);
    if (order_in_lds)
        for (int i = tid; i < P.c * n; i += 256) s_order[i] = P.order[i];
    const int8_t *order = order_in_lds ? s_order : P.order;

    const T *X = (const T *)P.x;
    const T *pkv = (const T *)P.pk_val;

    f32x16 acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // extents of the weight tile in (line, sparse position) coordinates
    for (int64_t k0 = 0; k0 < P.K; k0 += BK) {
        __syncthreads();
        // ---- X tile -> As[token][k] ----
        for (int e = tid; e < BM * BK; e += 256) {
            int row = e / BK, kk = e % BK;
            int64_t tok = tok0 + row, k = k0 + kk;
            T v = Zero<T>::v();
            if (tok < P.T && k < P.K) v = X[tok * P.ldx + k];
            As[row * LDSW + kk] = v;
        }
        // ---- weight tile -> Bs[output][k], decompressed ----
        {
            // line range [q0, q0+QN), sparse-position range [s0, s0+SN)
            const int64_t q0 = REDUCE_SPARSE ? o0 : k0;
            const int QN = REDUCE_SPARSE ? BN : BK;
            const int64_t s0 = REDUCE_SPARSE ? k0 : o0;
            const int SN = REDUCE_SPARSE ? BK : BN;
            const int64_t b_lo = s0 / m;
            const int NBL = (int)((s0 + SN + m - 1) / m - b_lo);
            for (int e = tid; e < QN * NBL; e += 256) {
                int ql = e / NBL, bl = e % NBL;
                int64_t q = q0 + ql, b = b_lo + bl;
                bool live = (q < P.G) && (b < P.nb);
                int p = 0;
                if (live)
                    p = (P.pat_bytes == 1) ? (int)((const uint8_t *)P.pk_pat)[q * P.nb + b]
                                           : (int)((const uint16_t *)P.pk_pat)[q * P.nb + b];
                const T *v = pkv + (q * P.nb + b) * n;
                int j = 0;
                for (int r = 0; r < m; r++) {
                    T w = Zero<T>::v();
                    if (live && j < n && order[p * n + j] == r) w = v[j++];
                    int64_t s = b * m + r;
                    int sl = (int)(s - s0);
                    if (sl < 0 || sl >= SN) continue;
                    if (REDUCE_SPARSE)
                        Bs[ql * LDSW + sl] = w;
                    else
                        Bs[sl * LDSW + ql] = w;
                }
            }
        }
        __syncthreads();
        // ---- MFMA ----
#pragma unroll
        for (int kk = 0; kk < BK; kk += M::KPI) {
            typename M::Frag a[MI], b[NJ];
            const int koff = kk + (lane >> 5) * M::EPL;
#pragma unroll
            for (int i = 0; i < MI; i++)
                a[i] = *(const typename M::Frag *)&As[(wm * WMT + i * 32 + (lane & 31)) * LDSW + koff];
#pragma unroll
            for (int j = 0; j < NJ; j++)
                b[j] = *(const typename M::Frag *)&Bs[(wn * WNT + j * 32 + (lane & 31)) * LDSW + koff];
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < NJ; j++) acc[i][j] = M::run(a[i], b[j], acc[i][j]);
        }
    }

    // ---- epilogue: D[row = token][col = output]; lane holds col = lane%32,
    //      rows 8*(r/4) + 4*(lane/32) + r%4 ----
    T *Y = (T *)P.y;
    const T *bias = (const T *)P.bias;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int64_t o = o0 + wn * WNT + j * 32 + (lane & 31);
        if (o >= P.O) continue;
        const float bv = bias ? to_f32(bias[o]) : 0.f;
#pragma unroll
        for (int i = 0; i < MI; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t tok = tok0 + wm * WMT + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                if (tok < P.T) {
                    T out;
                    from_f32(acc[i][j][r] + bv, out);
                    Y[tok * P.ldy + o] = out;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------ skinny path
// Few tokens (<= 16), reduction along the sparse dim: bandwidth-bound.  One wavefront per output
// line; lanes stride over the line's blocks, gather the activations the kept positions point
// at, and a butterfly reduction sums the lanes.
template <typename T, int TT>
__global__ __launch_bounds__(256) void spmm_skinny_kernel(SpmmParams P)
{
    __shared__ int8_t s_order[kOrderSlotBytes / 4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = P.n, m = P.m;
    const bool order_in_lds = P.c * n <= (int)sizeof(s_order);
    if (order_in_lds)
        for (int i = tid; i < P.c * n; i += 256) s_order[i] = P.order[i];
    __syncthreads();
    const int8_t *order = order_in_lds ? s_order : P.order;
    const int64_t q = (int64_t)blockIdx.x * 4 + wave;
    if (q >= P.G) return;
    const T *X = (const T *)P.x;
    const T *pkv = (const T *)P.pk_val + q * P.nb * n;
    float acc[TT];
#pragma unroll
    for (int t = 0; t < TT; t++) acc[t] = 0.f;
    for (int64_t b = lane; b < P.nb; b += 64) {
        const int p = (P.pat_bytes == 1) ? (int)((const uint8_t *)P.pk_pat)[q * P.nb + b]
                                         : (int)((const uint16_t *)P.pk_pat)[q * P.nb + b];
        for (int j = 0; j < n; j++) {
            const float w = to_f32(pkv[b * n + j]);
            const int64_t k = b * m + order[p * n + j];
            if (k < P.S) {
#pragma unroll
                for (int t = 0; t < TT; t++)
                    if (t < P.T) acc[t] += w * to_f32(X[t * P.ldx + k]);
            }
        }
    }
#pragma unroll
    for (int t = 0; t < TT; t++) {
        float v = acc[t];
#pragma unroll
        for (int mask = 32; mask >= 1; mask >>= 1) v += __shfl_xor(v, mask, 64);
        acc[t] = v;
    }
    if (lane == 0) {
        const T *bias = (const T *)P.bias;
        const float bv = bias ? to_f32(bias[q]) : 0.f;
        T *Y = (T *)P.y;
#pragma unroll
        for (int t = 0; t < TT; t++)
            if (t < P.T) {
                T out;
                from_f32(acc[t] + bv, out);
                Y[t * P.ldy + q] = out;
            }
    }
}

bool dense_pipe_supports(int n, int m);
int spmm_dense_pipe(const void *pk_val, const void *pk_pat, const int8_t *d_order, int64_t G, int64_t S,
                    const void *x, int64_t ldx, void *y, int64_t ldy, const void *bias, int64_t T,
                    int reduce_sparse, int n, int m, int dtype, hipStream_t s);

template <typename T> static int launch_spmm(SpmmParams &P, int reduce_sparse, int kernel, hipStream_t s)
{
    if (kernel == NMG_KERNEL_SKINNY) {
        dim3 grid((unsigned)((P.G + 3) / 4));
        if (P.T <= 1)
            hipLaunchKernelGGL((spmm_skinny_kernel<T, 1>), grid, dim3(256), 0, s, P);
        else if (P.T <= 4)
            hipLaunchKernelGGL((spmm_skinny_kernel<T, 4>), grid, dim3(256), 0, s, P);
        else
            hipLaunchKernelGGL((spmm_skinny_kernel<T, 16>), grid, dim3(256), 0, s, P);
    } else {
        const int64_t big = ((P.O + 127) / 128) * ((P.T + 127) / 128);
        if (big >= 128) {
            dim3 grid((unsigned)((P.O + 127) / 128), (unsigned)((P.T + 127) / 128));
            if (reduce_sparse)
                hipLaunchKernelGGL((spmm_mfma_kernel<T, true, 128, 128>), grid, dim3(256), 0, s, P);
            else
                hipLaunchKernelGGL((spmm_mfma_kernel<T, false, 128, 128>), grid, dim3(256), 0, s, P);
        } else {
            dim3 grid((unsigned)((P.O + 63) / 64), (unsigned)((P.T + 63) / 64));
            if (reduce_sparse)
                hipLaunchKernelGGL((spmm_mfma_kernel<T, true, 64, 64>), grid, dim3(256), 0, s, P);
            else
                hipLaunchKernelGGL((spmm_mfma_kernel<T, false, 64, 64>), grid, dim3(256), 0, s, P);
        }
    }
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

}  // namespace nmg

using namespace nmg;

extern "C" int nmg_spmm(const void *d_pk_val, const void *d_pk_pat, int64_t G, int64_t S,
                        const void *d_x, int64_t ldx, void *d_y, int64_t ldy, const void *d_bias,
                        int64_t T, int reduce_sparse, int n, int m, int dtype, int kernel,
                        void *stream)
{
    NMG_REQUIRE(m >= 1 && m <= 64 && n >= 0 && n <= m, NMG_ERR_ARG, "invalid n:m = %d:%d", n, m);
    NMG_REQUIRE(dtype == NMG_F32 || dtype == NMG_F16 || dtype == NMG_BF16, NMG_ERR_ARG,
                "spmm supports f32/f16/bf16, got dtype code %d", dtype);
    NMG_REQUIRE(G >= 0 && S >= 0 && T >= 0, NMG_ERR_ARG, "negative extent");
    NMG_REQUIRE(kernel >= NMG_KERNEL_AUTO && kernel <= NMG_KERNEL_SKINNY, NMG_ERR_ARG,
                "unknown kernel selector %d", kernel);
    if (G == 0 || S == 0 || T == 0) return NMG_OK;
    NMG_REQUIRE(d_pk_val && d_pk_pat && d_x && d_y, NMG_ERR_ARG, "null device pointer");
    NMG_REQUIRE(ldx >= (reduce_sparse ? S : G) && ldy >= (reduce_sparse ? G : S), NMG_ERR_ARG,
                "leading dimension smaller than row length");
    if (kernel == NMG_KERNEL_AUTO) kernel = (reduce_sparse && T <= 16) ? NMG_KERNEL_SKINNY : NMG_KERNEL_MFMA;
    if (kernel == NMG_KERNEL_SKINNY)
        NMG_REQUIRE(reduce_sparse && T <= 16, NMG_ERR_UNSUPPORTED,
                    "skinny kernel needs reduce_sparse=1 and T <= 16");
    NMG_REQUIRE(kernel != NMG_KERNEL_SMFMAC, NMG_ERR_UNSUPPORTED, "SMFMAC kernel not available");
    SpmmParams P{};
    P.pk_val = d_pk_val;
    P.pk_pat = d_pk_pat;
    if (int rc = device_order(n, m, &P.order)) return rc;
    P.x = d_x;
    P.y = d_y;
    P.bias = d_bias;
    P.G = G;
    P.S = S;
    P.nb = (S + m - 1) / m;
    P.T = T;
    P.ldx = ldx;
    P.ldy = ldy;
    P.K = reduce_sparse ? S : G;
    P.O = reduce_sparse ? G : S;
    P.n = n;
    P.m = m;
    P.c = (int)binom(m, n);
    P.pat_bytes = (int)nmg_rowpack_pat_bytes(n, m);
    hipStream_t s = (hipStream_t)stream;
    // Large 16-bit problems go to the pipelined dense-MFMA kernel (nmg_dense.hip); the simple
    // tiled kernel below keeps serving f32, ragged K, unusual n:m and explicit requests.
    if (kernel == NMG_KERNEL_MFMA && (dtype == NMG_F16 || dtype == NMG_BF16) && T > 16 &&
        dense_pipe_supports(n, m) && P.K % 64 == 0 && P.K >= 64 && (ldx % 8) == 0 && ((uintptr_t)d_x % 16) == 0 &&
        T * ldx * 2 < ((int64_t)1 << 31) && binom(m, n) <= 256)
        return spmm_dense_pipe(d_pk_val, d_pk_pat, P.order, G, S, d_x, ldx, d_y, ldy, d_bias, T,
                               reduce_sparse, n, m, dtype, s);
    switch (dtype) {
    case NMG_F32: return launch_spmm<float>(P, reduce_sparse, kernel, s);
    case NMG_F16: return launch_spmm<__half>(P, reduce_sparse, kernel, s);
    case NMG_BF16: return launch_spmm<__hip_bfloat16>(P, reduce_sparse, kernel, s);
    }
    return NMG_ERR_ARG;
}
