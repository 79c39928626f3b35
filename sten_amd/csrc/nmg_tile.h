// Pieces shared by the pipelined matrix-core kernels: vector types, LDS-DMA pointer types and the
// output-tile epilogue.
#pragma once
#include "nmg_common.h"

namespace nmg {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void *lds_ptr_t;
typedef const __attribute__((address_space(1))) void *glb_ptr_t;

__device__ __forceinline__ uint16_t f32_to_bits16(float x, __half *) { return __half_as_ushort(__float2half(x)); }
__device__ __forceinline__ uint16_t f32_to_bits16(float x, __hip_bfloat16 *)
{
    __hip_bfloat16 b = __float2bfloat16(x);
    return *reinterpret_cast<uint16_t *>(&b);
}

// Where an output tile goes: Y[T, M] row-major with leading dimension ldy, optional bias[M].
struct TileOut {
    void *y;
    const void *bias;
    int64_t M, T, ldy;
};

// Epilogue of the pipelined kernels.  D[row = feature][col = token]; a lane holds token
// l%32 and features 8*(r/4) + 4*(l/32) + r%4.  The wavefront's TB*32 tokens x FB*32 features are
// staged through its own LDS region `stg` as [token][feature] so the global stores are 16 B per
// lane and FB*64 B contiguous per token row.  fw / tw = first feature / token of the wavefront.
// The caller guarantees that no load into LDS is pending.
// Second half of the staged epilogues: NROWS token rows of FB*64 B (+16 B pad) lie in `stg`; every
// lane moves 16 B per pass, FB*64 B contiguous per token row, adding the bias on the way.
template <typename T, int FB, int NROWS>
__device__ __forceinline__ void store_staged_rows(const unsigned char *stg, int lane, int64_t fw, int64_t tw,
                                                  const TileOut &P)
{
    constexpr int ROW = FB * 64 + 16;       // bytes per staged token row (16 B pad: conflict-free)
    constexpr int CPR = FB * 4;             // 16-byte chunks per row
    constexpr int RPP = 64 / CPR;           // token rows per pass of the wavefront
    uint16_t *Y = (uint16_t *)P.y;
    const T *bias = (const T *)P.bias;
    const bool vec_ok = (P.ldy & 7) == 0 && ((uintptr_t)P.y & 15) == 0;
    const int fc = lane % CPR;                      // 8-feature chunk of the row
    const int64_t f = fw + fc * 8;
    float bv[8];
#pragma unroll
    for (int i = 0; i < 8; i++) bv[i] = (bias && f + i < P.M) ? to_f32(bias[f + i]) : 0.f;
#pragma unroll 4
    for (int it = 0; it < NROWS / RPP; it++) {
        const int tl = it * RPP + lane / CPR;
        const int64_t tok = tw + tl;
        u32x4 v = *(const u32x4 *)(stg + tl * ROW + fc * 16);
        if (tok >= P.T || f >= P.M) continue;
        if (bias) {
            uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                uint16_t lo = (uint16_t)(w[i] & 0xFFFF), hi = (uint16_t)(w[i] >> 16);
                T tlo = *reinterpret_cast<T *>(&lo), thi = *reinterpret_cast<T *>(&hi);
                lo = f32_to_bits16(to_f32(tlo) + bv[2 * i], (T *)nullptr);
                hi = f32_to_bits16(to_f32(thi) + bv[2 * i + 1], (T *)nullptr);
                w[i] = (uint32_t)lo | ((uint32_t)hi << 16);
            }
            v.x = w[0]; v.y = w[1]; v.z = w[2]; v.w = w[3];
        }
        uint16_t *dst = Y + tok * P.ldy + f;
        if (vec_ok && f + 7 < P.M) {
            *(u32x4 *)dst = v;
        } else {
            uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (f + i < P.M) dst[i] = (uint16_t)(w[i >> 1] >> ((i & 1) * 16));
        }
    }
}

template <typename T, int FB, int TB>
__device__ __forceinline__ void smf_store_tile(const f32x16 (&acc)[FB][TB], unsigned char *stg, int lane,
                                               int64_t fw, int64_t tw, const TileOut &P)
{
    constexpr int ROW = FB * 64 + 16;
    const int j = lane & 31, h = lane >> 5;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int tb = 0; tb < TB; tb++)
#pragma unroll
        for (int fb = 0; fb < FB; fb++)
#pragma unroll
            for (int rq = 0; rq < 4; rq++) {
                uint16_t hh[4];
#pragma unroll
                for (int i = 0; i < 4; i++) hh[i] = f32_to_bits16(acc[fb][tb][rq * 4 + i], (T *)nullptr);
                uint2 pk;
                pk.x = (uint32_t)hh[0] | ((uint32_t)hh[1] << 16);
                pk.y = (uint32_t)hh[2] | ((uint32_t)hh[3] << 16);
                *(uint2 *)(stg + (tb * 32 + j) * ROW + (fb * 32 + rq * 8 + h * 4) * 2) = pk;
            }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    store_staged_rows<T, FB, TB * 32>(stg, lane, fw, tw, P);
}

// The 16 x 16 form of the instruction: a lane holds token l%16 and outputs 4*(l/16) + 0..3 of every
// 16 x 16 block.  AB blocks of 16 outputs (a multiple of 2) x TB blocks of 16 tokens per wavefront.
template <typename T, int AB, int TB>
__device__ __forceinline__ void store_tile16(const f32x4 (&acc)[AB][TB], unsigned char *stg, int lane,
                                             int64_t fw, int64_t tw, const TileOut &P)
{
    static_assert(AB % 2 == 0, "whole 32-output rows of the staging area");
    constexpr int ROW = AB * 32 + 16;
    const int j = lane & 15, q = lane >> 4;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int tb = 0; tb < TB; tb++)
#pragma unroll
        for (int ab = 0; ab < AB; ab++) {
            uint16_t hh[4];
#pragma unroll
            for (int i = 0; i < 4; i++) hh[i] = f32_to_bits16(acc[ab][tb][i], (T *)nullptr);
            uint2 pk;
            pk.x = (uint32_t)hh[0] | ((uint32_t)hh[1] << 16);
            pk.y = (uint32_t)hh[2] | ((uint32_t)hh[3] << 16);
            *(uint2 *)(stg + (tb * 16 + j) * ROW + (ab * 16 + q * 4) * 2) = pk;
        }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    store_staged_rows<T, AB / 2, TB * 16>(stg, lane, fw, tw, P);
}

// The same epilogue for a transposed output, Y[M, T] row-major (tokens contiguous): the
// wavefront's FB*32 features x TB*32 tokens are staged as [feature][token], so that a lane stores
// 16 bytes = 8 tokens of one feature row and TB*64 bytes per row are contiguous.  The bias of a
// feature is added to its whole row.
// Second half of the transposed epilogues: NROWS output rows of TB*64 B (+16 B pad) lie in `stg`
// as [output][token]; a lane moves 16 bytes = 8 tokens of one output row per pass.  The bias of an
// output is added to its whole row.
template <typename T, int TB, int NROWS>
__device__ __forceinline__ void store_staged_rows_t(const unsigned char *stg, int lane, int64_t fw, int64_t tw,
                                                    const TileOut &P)
{
    constexpr int ROW = TB * 64 + 16;       // bytes per staged feature row
    constexpr int CPR = TB * 4;             // 16-byte chunks per row
    constexpr int RPP = 64 / CPR;           // feature rows per pass of the wavefront
    uint16_t *Y = (uint16_t *)P.y;
    const T *bias = (const T *)P.bias;
    const bool vec_ok = (P.ldy & 7) == 0 && ((uintptr_t)P.y & 15) == 0;
    const int tc = lane % CPR;                      // 8-token chunk of the row
    const int64_t tok = tw + tc * 8;
#pragma unroll 4
    for (int it = 0; it < NROWS / RPP; it++) {
        const int fl = it * RPP + lane / CPR;
        const int64_t f = fw + fl;
        u32x4 v = *(const u32x4 *)(stg + fl * ROW + tc * 16);
        if (f >= P.M || tok >= P.T) continue;
        if (bias) {
            const float bv = to_f32(bias[f]);
            uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                uint16_t lo = (uint16_t)(w[i] & 0xFFFF), hi = (uint16_t)(w[i] >> 16);
                T tlo = *reinterpret_cast<T *>(&lo), thi = *reinterpret_cast<T *>(&hi);
                lo = f32_to_bits16(to_f32(tlo) + bv, (T *)nullptr);
                hi = f32_to_bits16(to_f32(thi) + bv, (T *)nullptr);
                w[i] = (uint32_t)lo | ((uint32_t)hi << 16);
            }
            v.x = w[0]; v.y = w[1]; v.z = w[2]; v.w = w[3];
        }
        uint16_t *dst = Y + f * P.ldy + tok;
        if (vec_ok && tok + 7 < P.T) {
            *(u32x4 *)dst = v;
        } else {
            uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (tok + i < P.T) dst[i] = (uint16_t)(w[i >> 1] >> ((i & 1) * 16));
        }
    }
}

template <typename T, int FB, int TB>
__device__ __forceinline__ void smf_store_tile_t(const f32x16 (&acc)[FB][TB], unsigned char *stg, int lane,
                                                 int64_t fw, int64_t tw, const TileOut &P)
{
    constexpr int ROW = TB * 64 + 16;       // bytes per staged feature row
    const int j = lane & 31, h = lane >> 5;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int tb = 0; tb < TB; tb++)
#pragma unroll
        for (int fb = 0; fb < FB; fb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int f = fb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                *(uint16_t *)(stg + f * ROW + (tb * 32 + j) * 2) = f32_to_bits16(acc[fb][tb][r], (T *)nullptr);
            }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    store_staged_rows_t<T, TB, FB * 32>(stg, lane, fw, tw, P);
}

// The 16 x 16 form, transposed output: AB blocks of 16 outputs x TB16 blocks of 16 tokens (an even
// number) per wavefront, staged as [output][token].
template <typename T, int AB, int TB16>
__device__ __forceinline__ void store_tile16_t(const f32x4 (&acc)[AB][TB16], unsigned char *stg, int lane,
                                               int64_t fw, int64_t tw, const TileOut &P)
{
    static_assert(TB16 % 2 == 0, "whole 32-token pieces of a staged row");
    constexpr int ROW = TB16 * 32 + 16;
    const int j = lane & 15, q = lane >> 4;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int tb = 0; tb < TB16; tb++)
#pragma unroll
        for (int ab = 0; ab < AB; ab++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                *(uint16_t *)(stg + (ab * 16 + q * 4 + r) * ROW + (tb * 16 + j) * 2) =
                    f32_to_bits16(acc[ab][tb][r], (T *)nullptr);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    store_staged_rows_t<T, TB16 / 2, AB * 16>(stg, lane, fw, tw, P);
}

// ---- reductions cut into slices (products with fewer tiles than the GPU has CUs) ----
// Slice s of a tile stores its sums in single precision at part[s][token][feature] (part_ld
// features per token, a multiple of 256: the padded features of the last tile are stored too);
// splitk_sum_kernel adds the slices in order (+ bias) and rounds once.
struct SplitSum {
    const float *part;
    void *y;
    const void *bias;
    int64_t M, T, ldy, part_ld;
    int slices;
};

// A lane holds token l%32 and features 8*(r/4) + 4*(l/32) + r%4 of every 32 x 32 block: four
// consecutive features are one 16-byte store.  fw / tw = first feature / token of the wavefront.
template <int FB, int TB>
__device__ __forceinline__ void store_partial_tile(const f32x16 (&acc)[FB][TB], float *part, int64_t part_ld,
                                                   int lane, int64_t fw, int64_t tw, int64_t T)
{
    const int j = lane & 31, h = lane >> 5;
#pragma unroll
    for (int tb = 0; tb < TB; tb++) {
        const int64_t tok = tw + tb * 32 + j;
        if (tok >= T) continue;
#pragma unroll
        for (int fb = 0; fb < FB; fb++)
#pragma unroll
            for (int rq = 0; rq < 4; rq++) {
                float4 v;
                v.x = acc[fb][tb][rq * 4 + 0];
                v.y = acc[fb][tb][rq * 4 + 1];
                v.z = acc[fb][tb][rq * 4 + 2];
                v.w = acc[fb][tb][rq * 4 + 3];
                *(float4 *)(part + tok * part_ld + fw + fb * 32 + rq * 8 + h * 4) = v;
            }
    }
}

// The same for the 16 x 16 form: a lane holds token l%16 and outputs 4*(l/16) + 0..3 of every block.
template <int AB, int TB>
__device__ __forceinline__ void store_partial_tile16(const f32x4 (&acc)[AB][TB], float *part, int64_t part_ld,
                                                     int lane, int64_t fw, int64_t tw, int64_t T)
{
    const int j = lane & 15, q = lane >> 4;
#pragma unroll
    for (int tb = 0; tb < TB; tb++) {
        const int64_t tok = tw + tb * 16 + j;
        if (tok >= T) continue;
#pragma unroll
        for (int ab = 0; ab < AB; ab++) {
            float4 v;
            v.x = acc[ab][tb][0];
            v.y = acc[ab][tb][1];
            v.z = acc[ab][tb][2];
            v.w = acc[ab][tb][3];
            *(float4 *)(part + tok * part_ld + fw + ab * 16 + q * 4) = v;
        }
    }
}

template <typename T> __global__ __launch_bounds__(256) void splitk_sum_kernel(SplitSum P)
{
    const int64_t quads = (P.M + 3) / 4;
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= P.T * quads) return;
    const int64_t tok = gid / quads, f = (gid - tok * quads) * 4;
    const float *src = P.part + tok * P.part_ld + f;
    // sixteen slices are fetched at a time (the kernel is a chain of round trips to memory otherwise:
    // the sums were written through other L2s) and added in slice order
    const int64_t step = P.T * P.part_ld;
    float4 sum = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < P.slices; s0 += 16) {
        float4 v[16];
#pragma unroll
        for (int u = 0; u < 16; u++)
            v[u] = s0 + u < P.slices ? *(const float4 *)(src + (int64_t)(s0 + u) * step) : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < 16; u++) {
            sum.x += v[u].x;
            sum.y += v[u].y;
            sum.z += v[u].z;
            sum.w += v[u].w;
        }
    }
    const float o[4] = {sum.x, sum.y, sum.z, sum.w};
    uint16_t *dst = (uint16_t *)P.y + tok * P.ldy + f;
    const T *bias = (const T *)P.bias;
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (f + i < P.M) dst[i] = f32_to_bits16(o[i] + (bias ? to_f32(bias[f + i]) : 0.f), (T *)nullptr);
}

template <typename T> static inline int launch_splitk_sum(const SplitSum &P, hipStream_t s)
{
    const int64_t threads = P.T * ((P.M + 3) / 4);
    hipLaunchKernelGGL(splitk_sum_kernel<T>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, P);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

// Largest number of slices <= S that leaves none empty: slices of ceil(KP / S) K steps.
static inline int splitk_fit(int64_t KP, int64_t S)
{
    while (S > 1 && (S - 1) * ((KP + S - 1) / S) >= KP) S--;
    return (int)(S < 1 ? 1 : S);
}

}  // namespace nmg
