// Measurement aid: what the matrix cores sustain when nothing else happens.  A wavefront keeps a
// 128 x 128 tile of accumulators and eight operand fragments per side in registers and issues the
// matrix instructions of a K = 64 slab back to back, `iters` times, with no memory traffic inside
// the loop; 1024 workgroups of four wavefronts fill the chip four times over.  With all-zero
// operands the instruction's own issue rate shows; with random operands the power limit decides.
// The measured rates are what a product kernel's fraction of the nominal peak has to be read
// against (gfx950, MI355X, measured: dense f16 32x32x16 1.71 PFLOP/s on random operands and 2.45 on
// zeros, 16x16x32 1.94 / 2.43; sparse 32x32x32 2.6 / 3.6 dense-equivalent, 16x16x64 3.45 / 4.9).
// Built into its own library (libnmg_probe.so, declared in include/nmg_probe.h): it serves bench.py
// only and is not part of the product's C ABI.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/nmg_probe.h"

namespace nmg {

typedef _Float16 pb_f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 pb_f16x16 __attribute__((ext_vector_type(16)));
typedef float pb_f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// KIND 0: V_MFMA_F32_32X32X16_F16, 1: V_MFMA_F32_16X16X32_F16,
//      2: V_SMFMAC_F32_32X32X32_F16, 3: V_SMFMAC_F32_16X16X64_F16
template <int KIND> __global__ __launch_bounds__(256, 1) void probe_kernel(const pb_f16x8 *src, float *out, int iters)
{
    const int tid = threadIdx.x + blockIdx.x * 256;
    pb_f16x8 a[8], bd[8];   // dense kinds: eight fragments per side
    pb_f16x16 b[8];         // sparse kinds: the dense side holds twice the reduction per fragment
    int ix[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = src[(tid * 32 + i) & 0xffff];
        const pb_f16x8 lo = src[(tid * 32 + 8 + 2 * i) & 0xffff], hi = src[(tid * 32 + 9 + 2 * i) & 0xffff];
        bd[i] = lo;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            b[i][e] = lo[e];
            b[i][8 + e] = hi[e];
        }
        // every stored pair takes positions (0 or 1, 2 or 3): valid selectors whatever the bits are
        ix[i] = (((const int *)src)[(tid * 8 + i) & 0xffff] & 0x44444444) | 0x88888888;
    }
    float sum = 0;
    if constexpr (KIND == 0 || KIND == 2) {
        f32x16 acc[4][4];
#pragma unroll
        for (int x = 0; x < 4; x++)
#pragma unroll
            for (int y = 0; y < 4; y++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[x][y][r] = 0;
        // the accumulators fill the accumulation registers, the operands stay in the architectural
        // ones: left alone the allocator shuffles registers between the two files inside the loop
#pragma unroll
        for (int x = 0; x < 4; x++)
#pragma unroll
            for (int y = 0; y < 4; y++) asm volatile("" : "+a"(acc[x][y]));
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int kk = 0; kk < (KIND == 0 ? 4 : 2); kk++)
#pragma unroll
                for (int x = 0; x < 4; x++)
#pragma unroll
                    for (int y = 0; y < 4; y++) {
                        if constexpr (KIND == 0) {
                            acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[(kk & 1) * 4 + x], bd[(kk & 1) * 4 + y],
                                                                               acc[x][y], 0, 0, 0);
                        } else {
                            acc[x][y] = __builtin_amdgcn_smfmac_f32_32x32x32_f16(a[kk * 4 + x], b[kk * 4 + y], acc[x][y],
                                                                                 ix[kk * 4 + x], 0, 0);
                        }
                    }
        }
#pragma unroll
        for (int x = 0; x < 4; x++)
#pragma unroll
            for (int y = 0; y < 4; y++)
#pragma unroll
                for (int r = 0; r < 16; r++) sum += acc[x][y][r];
    } else {
        pb_f32x4 acc[8][8];
#pragma unroll
        for (int x = 0; x < 8; x++)
#pragma unroll
            for (int y = 0; y < 8; y++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[x][y][r] = 0;
        if constexpr (KIND == 1) {   // (the allocator places the 16x16x64 form well by itself, and badly when told)
#pragma unroll
            for (int x = 0; x < 8; x++)
#pragma unroll
                for (int y = 0; y < 8; y++) asm volatile("" : "+a"(acc[x][y]));
        }
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int kk = 0; kk < (KIND == 1 ? 2 : 1); kk++)
#pragma unroll
                for (int x = 0; x < 8; x++)
#pragma unroll
                    for (int y = 0; y < 8; y++) {
                        if constexpr (KIND == 1) {
                            acc[x][y] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[x], bd[y], acc[x][y], 0, 0, 0);
                        } else {
                            acc[x][y] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a[x], b[y], acc[x][y], ix[x], 0, 0);
                        }
                    }
        }
#pragma unroll
        for (int x = 0; x < 8; x++)
#pragma unroll
            for (int y = 0; y < 8; y++)
#pragma unroll
                for (int r = 0; r < 4; r++) sum += acc[x][y][r];
    }
    out[tid] = sum;
}

constexpr int PB_GROUPS = 1024;

}  // namespace nmg

using namespace nmg;

extern "C" int64_t nmg_probe_matrix_rate_flops(int kind, int iters)
{
    if (kind < 0 || kind > 3 || iters < 0) return -1;
    // 128 x 128 x 64 per wavefront and iteration, dense-equivalent for the sparse instructions
    return (int64_t)2 * 128 * 128 * 64 * iters * 4 * PB_GROUPS;
}

extern "C" int nmg_probe_matrix_rate(int kind, const void *d_operands, float *d_out, int iters, void *stream)
{
    // 1: bad argument, 2: the launch failed
    if (kind < 0 || kind > 3 || iters < 1 || iters > (1 << 24) || !d_operands || !d_out ||
        ((uintptr_t)d_operands % 16) != 0)
        return 1;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(PB_GROUPS), block(256);
    const pb_f16x8 *src = (const pb_f16x8 *)d_operands;
    switch (kind) {
    case 0: hipLaunchKernelGGL(probe_kernel<0>, grid, block, 0, s, src, d_out, iters); break;
    case 1: hipLaunchKernelGGL(probe_kernel<1>, grid, block, 0, s, src, d_out, iters); break;
    case 2: hipLaunchKernelGGL(probe_kernel<2>, grid, block, 0, s, src, d_out, iters); break;
    default: hipLaunchKernelGGL(probe_kernel<3>, grid, block, 0, s, src, d_out, iters); break;
    }
    return hipGetLastError() == hipSuccess ? 0 : 2;
}
