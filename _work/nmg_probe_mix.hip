// Measurement aid: what a K step of the large-batch kernels costs beyond its matrix instructions.
// A workgroup per CU replays the instruction mix of one K step of 64 -- the matrix instructions,
// the LDS fragment reads, the weight loads into registers and the DMA loads of the activation
// tile into a 4-stage LDS ring -- on random data that stays in L2, with nothing else around it:
// no prologue, no epilogue, no HBM traffic.  Parts of the mix can be left out, and the instruction
// and the layout of the wavefronts exchanged, which shows what each part costs and which form of
// the instruction keeps its advantage with the memory instructions around it.  The values that the
// loads bring are used as operands one step later (a load targets the register set that the
// matrix instructions do not read in this step), so the data the matrix cores see is the loaded,
// random data; the sums are written out only to keep the loop alive.
//   dense tile 256 outputs x 256 tokens (the dense-matrix-core kernel): per wavefront and step
//     64 x V_MFMA_F32_32X32X16 or 128 x V_MFMA_F32_16X16X32, 32 LDS reads of 16 bytes per lane,
//     8 weight loads, 8 DMA loads (four wavefronts; eight: half of the MFMAs, reads and DMA loads each);
//   sparse tile 256 lines x 128 tokens (the sparse-matrix-core kernel): 16 x V_SMFMAC_F32_32X32X32
//     or 32 x V_SMFMAC_F32_16X16X64, 16 LDS reads, 4 weight loads + 2 index loads, 4 DMA loads;
//     x 256 tokens: twice the MFMAs, reads and DMA loads.
#include "nmg_common.h"
#include "nmg_tile.h"

#include <type_traits>

namespace nmg {

typedef _Float16 mx_f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t mx_u32x8 __attribute__((ext_vector_type(8)));

// MEM bit 0: LDS reads, bit 1: weight loads, bit 2: DMA loads (sparse: bit 3: no index loads)
template <bool MI16, int WAVES, int MEM>   // MEM bit 0: LDS reads, bit 1: weight loads, bit 2: DMA
__global__ __launch_bounds__(WAVES * 64, 1) void mix_dense_kernel(const unsigned char *src, float *out, int steps)
{
#if defined(__HIP_DEVICE_COMPILE__)   // instruction statements: nothing for the host pass to see
    extern __shared__ __align__(16) unsigned char smem[];   // 128 KiB
    constexpr int TOK = WAVES == 4 ? 256 : 128;
    constexpr int NB = TOK / 32;            // B fragments (1 KiB each) per phase
    constexpr int DMA = 32 / WAVES;         // DMA loads per wavefront per step
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = WAVES == 4 ? 0 : wave & 1;
    const unsigned char *wsrc = src + (size_t)(blockIdx.x & 63) * 65536;
    const unsigned char *xsrc = src + 4 * 1024 * 1024 + (size_t)(blockIdx.x & 31) * 131072 + wave * DMA * 1024;
    const unsigned lane16 = lane * 16;
    u32x4 a[2][8], b[2][NB];
    f32x16 acc32[2][NB];
    f32x4 acc16[4][2 * NB];
    if constexpr (MI16) {
#pragma unroll
        for (int x = 0; x < 4; x++)
#pragma unroll
            for (int y = 0; y < 2 * NB; y++) { acc16[x][y] = f32x4{0, 0, 0, 0}; asm volatile("" : "+a"(acc16[x][y])); }
    } else {
#pragma unroll
        for (int x = 0; x < 2; x++)
#pragma unroll
            for (int y = 0; y < NB; y++) {
#pragma unroll
                for (int r = 0; r < 16; r++) acc32[x][y][r] = 0;
                asm volatile("" : "+a"(acc32[x][y]));
            }
    }
    // fill the LDS ring and the first register sets
    for (int i = threadIdx.x; i < 8192; i += WAVES * 64) ((u32x4 *)smem)[i] = ((const u32x4 *)(src + 4 * 1024 * 1024))[i];
#pragma unroll
    for (int i = 0; i < 8; i++) a[0][i] = a[1][i] = *(const u32x4 *)(wsrc + i * 1024 + lane16);
#pragma unroll
    for (int i = 0; i < NB; i++) b[0][i] = b[1][i] = *(const u32x4 *)(smem + (wn * NB + i) * 1024 + lane16);
    __syncthreads();

    auto mma = [&](const u32x4 *af, const u32x4 *bf, int ph, int i) {
        // MFMA number i of phase ph
        union { u32x4 u; mx_f16x8 h; } ca, cb;
        if constexpr (MI16) {
            // phase = (k32 step ph/2, token half ph%2): 4 A fragments x NB B fragments
            const int x = i / NB, y = i % NB;
            ca.u = af[(ph >> 1) * 4 + x];
            cb.u = bf[y];
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc16[x][(ph & 1) * NB + y]) : "v"(ca.h), "v"(cb.h));
        } else {
            // phase = k16 step ph: 2 A fragments x NB B fragments
            const int x = i / NB, y = i % NB;
            ca.u = af[ph * 2 + x];
            cb.u = bf[y];
            asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc32[x][y]) : "v"(ca.h), "v"(cb.h));
        }
    };
    constexpr int NM = MI16 ? 4 * NB : 2 * NB;   // MFMAs per phase
    constexpr int PER = NM / NB;                 // MFMAs per LDS read

    auto step = [&](int s, auto par_tag) {
        constexpr int PAR = decltype(par_tag)::value;
        const unsigned lds_base = (unsigned)(uintptr_t)(lds_ptr_t)(smem + (s & 3) * 32768 + wn * NB * 4096) + lane16;
        const unsigned dma_dst = (unsigned)(uintptr_t)(lds_ptr_t)(smem + ((s + 2) & 3) * 32768 + wave * DMA * 1024);
        const unsigned char *xs = xsrc + (size_t)(s & 3) * 32768;
        const unsigned char *ws = wsrc + (size_t)((s + (wave >> (WAVES == 8))) & 7) * 8192;
#pragma unroll
        for (int ph = 0; ph < 4; ph++) {
#pragma unroll
            for (int i = 0; i < NM; i++) {
                mma(a[PAR], b[ph & 1], ph, i);
                __builtin_amdgcn_sched_barrier(0);
                if ((MEM & 1) && i % PER == 0) {
                    // fragment i/PER of the next phase
                    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(b[(ph + 1) & 1][i / PER]) : "v"(lds_base), "n"(((i / PER) * 4 + ((ph + 1) & 3)) * 1024));
                }
                if ((MEM & 2) && ph < 2 && i % (NM / 4) == 1) {
                    const int li = ph * 4 + i / (NM / 4);
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(a[PAR ^ 1][li]) : "v"(lane16), "s"(ws + li * 1024));
                }
                if ((MEM & 4) && ph < 2 && i % (NM / (DMA / 2)) == 2) {
                    const int di = ph * (DMA / 2) + i / (NM / (DMA / 2));
                    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                                 :: "v"(lane16), "s"(xs + di * 1024), "s"(dma_dst + di * 1024) : "memory");
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (ph == 3) {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                asm volatile("s_barrier" ::: "memory");
            }
        }
    };
    for (int s = 0; s < steps; s += 2) {
        step(s, std::integral_constant<int, 0>{});
        step(s + 1, std::integral_constant<int, 1>{});
    }
    float sum = 0;
    if constexpr (MI16) {
#pragma unroll
        for (int x = 0; x < 4; x++)
#pragma unroll
            for (int y = 0; y < 2 * NB; y++) sum += acc16[x][y][0] + acc16[x][y][3];
    } else {
#pragma unroll
        for (int x = 0; x < 2; x++)
#pragma unroll
            for (int y = 0; y < NB; y++) sum += acc32[x][y][0] + acc32[x][y][15];
    }
    out[blockIdx.x * WAVES * 64 + threadIdx.x] = sum;
#endif
}


template <bool MI16, bool TOK256, int MEM, bool L22 = false>   // MEM bit 0: LDS reads, bit 1: weight loads, bit 2: DMA
__global__ __launch_bounds__(256, 1) void mix_sparse_kernel(const unsigned char *src, float *out, int steps)
{
#if defined(__HIP_DEVICE_COMPILE__)   // instruction statements: nothing for the host pass to see
    extern __shared__ __align__(16) unsigned char smem[];   // 4 stages
    constexpr int TOK = TOK256 ? 256 : 128;
    constexpr int STAGE = TOK * 128;
    constexpr int DMA = TOK / 32;           // DMA loads per wavefront per step
    constexpr int NPH = 4;                  // phases per step
    constexpr int NBF = L22 ? 1 : TOK / 32 / 2;       // B fragments (2 KiB each = two b128 reads) per phase: 2 or 4
    constexpr int NA = L22 ? 8 : 4, NI = L22 ? 4 : 2, LB = L22 ? 4 : 2;   // weight fragments, index words, line blocks
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned char *wsrc = src + (size_t)(blockIdx.x & 63) * 65536;
    const unsigned char *xsrc = src + 4 * 1024 * 1024 + (size_t)(blockIdx.x & 31) * 131072 + wave * DMA * 1024;
    const unsigned lane16 = lane * 16, lane4 = lane * 4;
    u32x4 a[2][NA];
    unsigned ix[2][NI];
    mx_u32x8 b[2][NBF];
    f32x16 acc32[LB][L22 ? 2 : TOK / 32];
    f32x4 acc16[4][TOK / 16];
    if constexpr (MI16) {
#pragma unroll
        for (int x = 0; x < 4; x++)
#pragma unroll
            for (int y = 0; y < TOK / 16; y++) { acc16[x][y] = f32x4{0, 0, 0, 0}; asm volatile("" : "+a"(acc16[x][y])); }
    } else {
#pragma unroll
        for (int x = 0; x < LB; x++)
#pragma unroll
            for (int y = 0; y < (L22 ? 2 : TOK / 32); y++) {
#pragma unroll
                for (int r = 0; r < 16; r++) acc32[x][y][r] = 0;
                asm volatile("" : "+a"(acc32[x][y]));
            }
    }
    for (int i = threadIdx.x; i < 4 * STAGE / 16; i += 256) ((u32x4 *)smem)[i] = ((const u32x4 *)(src + 4 * 1024 * 1024))[i];
#pragma unroll
    for (int i = 0; i < NA; i++) a[0][i] = a[1][i] = *(const u32x4 *)(wsrc + i * 1024 + lane16);
#pragma unroll
    for (int i = 0; i < NI; i++) ix[0][i] = ix[1][i] = *(const unsigned *)(wsrc + 8192 + i * 256 + lane4) & 0x44444444u;
#pragma unroll
    for (int i = 0; i < NBF; i++) b[0][i] = b[1][i] = *(const mx_u32x8 *)(smem + i * 2048 + lane * 32);
    __syncthreads();

    // MFMAs per phase: 32x32x32: phase = (k32 = ph/2, token half ph%2): 2 line blocks x NBF token blocks;
    // 16x16x64: phase = token quarter: 4 line blocks x NBF*... token blocks of 16 (a B fragment of 2 KiB
    // is 16 tokens x 64 k).
    constexpr int NM = MI16 ? 4 * NBF : LB * NBF;
    auto mma = [&](int par, int ph, int i) {
        if constexpr (MI16) {
            const int x = i / NBF, y = i % NBF;
            asm volatile("v_smfmac_f32_16x16x64_f16 %0, %1, %2, %3"
                         : "+a"(acc16[x][ph * NBF + y]) : "v"(a[par][x]), "v"(b[ph & 1][y]), "v"(ix[par][x >> 1]));
        } else {
            const int x = i / NBF, y = i % NBF;
            asm volatile("v_smfmac_f32_32x32x32_f16 %0, %1, %2, %3"
                         : "+a"(acc32[x][(ph & 1) * NBF + y]) : "v"(a[par][(ph >> 1) * LB + x]), "v"(b[ph & 1][y]), "v"(ix[par][x]));
        }
    };
    constexpr int NREAD = 2 * NBF;                       // b128 reads per phase
    constexpr int NLOAD = NA + NI, NOPS_STEP = NLOAD + DMA;    // loads dealt over phases 0..2

    auto step = [&](int s, auto par_tag) {
        constexpr int PAR = decltype(par_tag)::value;
        const unsigned lds_base = (unsigned)(uintptr_t)(lds_ptr_t)(smem + (s & 3) * STAGE + (L22 ? (wave & 1) * 8192 : 0)) + lane16;
        const unsigned dma_dst = (unsigned)(uintptr_t)(lds_ptr_t)(smem + ((s + 2) & 3) * STAGE + wave * DMA * 1024);
        const unsigned char *xs = xsrc + (size_t)(s & 3) * STAGE;
        const unsigned char *ws = wsrc + (size_t)((s + (L22 ? (wave >> 1) * 2 : wave)) & 3) * 16384;
#pragma unroll
        for (int ph = 0; ph < NPH; ph++) {
            const int l0 = ph * NOPS_STEP / 3, l1 = ph < 3 ? (ph + 1) * NOPS_STEP / 3 : l0;
            const int nops = ((MEM & 1) ? NREAD : 0) + (l1 - l0);
#pragma unroll
            for (int i = 0; i < NM; i++) {
                mma(PAR, ph, i);
                __builtin_amdgcn_sched_barrier(0);
                // ops due after MFMA i: spread evenly, ceil((i+1) * nops / NM) in total
                const int lo = (i * nops + NM - 1) / NM, hi = ((i + 1) * nops + NM - 1) / NM;
#pragma unroll
                for (int k0 = 0; k0 < 16; k0++) {
                    if (k0 < lo || k0 >= hi) continue;
                    int k = k0;
                    if (MEM & 1) {
                        if (k < NREAD) {
                            u32x4 *dst = (u32x4 *)&b[(ph + 1) & 1][k / 2];
                            if (k % 2 == 0)
                                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst[0]) : "v"(lds_base), "n"(((ph + 1) & 3) * NREAD * 1024 + k * 1024));
                            else
                                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst[1]) : "v"(lds_base), "n"(((ph + 1) & 3) * NREAD * 1024 + k * 1024));
                            continue;
                        }
                        k -= NREAD;
                    }
                    const int li = l0 + k;
                    if (li < NLOAD) {
                        if (!(MEM & 2)) continue;
                        if (li < NA)
                            asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(a[PAR ^ 1][li]) : "v"(lane16), "s"(ws + li * 1024));
                        else if (!(MEM & 8))
                            asm volatile("global_load_dword %0, %1, %2" : "=v"(ix[PAR ^ 1][li - NA]) : "v"(lane4), "s"(ws + 8192 + (li - NA) * 256));
                    } else {
                        if (!(MEM & 4)) continue;
                        const int di = li - NLOAD;
                        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                                     :: "v"(lane16), "s"(xs + di * 1024), "s"(dma_dst + di * 1024) : "memory");
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (ph == 3) {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                asm volatile("s_barrier" ::: "memory");
            }
        }
    };
    for (int s = 0; s < steps; s += 2) {
        step(s, std::integral_constant<int, 0>{});
        step(s + 1, std::integral_constant<int, 1>{});
    }
    float sum = 0;
    if constexpr (MI16) {
#pragma unroll
        for (int x = 0; x < 4; x++)
#pragma unroll
            for (int y = 0; y < TOK / 16; y++) sum += acc16[x][y][0] + acc16[x][y][3];
    } else {
#pragma unroll
        for (int x = 0; x < 2; x++)
#pragma unroll
            for (int y = 0; y < TOK / 32; y++) sum += acc32[x][y][0] + acc32[x][y][15];
    }
    out[blockIdx.x * 256 + threadIdx.x] = sum;
#endif
}


template <bool MI16, int WAVES, int MEM> static int launch_mix_dense(const unsigned char *src, float *out, int steps, hipStream_t s)
{
    auto k = mix_dense_kernel<MI16, WAVES, MEM>;
    NMG_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
    hipLaunchKernelGGL(k, dim3(256), dim3(WAVES * 64), 128 * 1024, s, src, out, steps);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

template <bool MI16, bool TOK256, int MEM, bool L22 = false>
static int launch_mix_sparse(const unsigned char *src, float *out, int steps, hipStream_t s)
{
    auto k = mix_sparse_kernel<MI16, TOK256, MEM, L22>;
    constexpr int lds = 4 * (TOK256 ? 256 : 128) * 128;
    NMG_HIP_TRY(hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    hipLaunchKernelGGL(k, dim3(256), dim3(256), lds, s, src, out, steps);
    NMG_HIP_TRY(hipGetLastError());
    return NMG_OK;
}

constexpr int MIX_KINDS = 21;

}  // namespace nmg

using namespace nmg;

extern "C" int64_t nmg_probe_instruction_mix_flops(int kind, int steps)
{
    if (kind < 0 || kind >= MIX_KINDS || steps < 0) return -1;
    // dense-equivalent flops of one launch: 256 workgroups, tile 256 x (128 or 256), K step 64
    const bool tok128 = kind >= 10 && kind <= 18;
    return (int64_t)2 * 256 * (tok128 ? 128 : 256) * 64 * steps * 256;
}

extern "C" int nmg_probe_instruction_mix(int kind, const void *d_data, int64_t data_bytes, float *d_out,
                                         int64_t out_elems, int steps, void *stream)
{
    NMG_REQUIRE(kind >= 0 && kind < MIX_KINDS, NMG_ERR_ARG, "unknown instruction mix %d", kind);
    NMG_REQUIRE(steps >= 2 && steps % 2 == 0 && steps <= (1 << 24), NMG_ERR_ARG, "steps must be even and at least 2");
    NMG_REQUIRE(d_data && d_out, NMG_ERR_ARG, "null device pointer");
    NMG_REQUIRE(data_bytes >= (int64_t)16 << 20 && ((uintptr_t)d_data % 16) == 0, NMG_ERR_ARG,
                "needs 16 MiB of operand data, 16-byte aligned");
    NMG_REQUIRE(out_elems >= 256 * 512, NMG_ERR_ARG, "needs 131072 floats of output");
    const unsigned char *src = (const unsigned char *)d_data;
    hipStream_t s = (hipStream_t)stream;
    switch (kind) {
    // dense tile 256 x 256, four wavefronts: 32x32x16 alone / + LDS reads / everything; 16x16x32 the same
    case 0: return launch_mix_dense<false, 4, 0>(src, d_out, steps, s);
    case 1: return launch_mix_dense<false, 4, 1>(src, d_out, steps, s);
    case 2: return launch_mix_dense<false, 4, 7>(src, d_out, steps, s);
    case 3: return launch_mix_dense<true, 4, 0>(src, d_out, steps, s);
    case 4: return launch_mix_dense<true, 4, 1>(src, d_out, steps, s);
    case 5: return launch_mix_dense<true, 4, 7>(src, d_out, steps, s);
    // eight wavefronts (two per SIMD), everything
    case 6: return launch_mix_dense<false, 8, 7>(src, d_out, steps, s);
    case 7: return launch_mix_dense<true, 8, 7>(src, d_out, steps, s);
    // sparse tile 256 x 256, everything: 32x32x32, 16x16x64
    case 8: return launch_mix_sparse<false, true, 7>(src, d_out, steps, s);
    case 9: return launch_mix_sparse<true, true, 7>(src, d_out, steps, s);
    // sparse tile 256 x 128, 32x32x32: alone / + LDS reads / everything / without the DMA loads /
    // without the weight loads / without the index loads / wavefronts 2 x 2
    case 10: return launch_mix_sparse<false, false, 0>(src, d_out, steps, s);
    case 11: return launch_mix_sparse<false, false, 1>(src, d_out, steps, s);
    case 12: return launch_mix_sparse<false, false, 7>(src, d_out, steps, s);
    case 13: return launch_mix_sparse<false, false, 3>(src, d_out, steps, s);
    case 14: return launch_mix_sparse<false, false, 5>(src, d_out, steps, s);
    case 15: return launch_mix_sparse<false, false, 15>(src, d_out, steps, s);
    case 16: return launch_mix_sparse<false, false, 7, true>(src, d_out, steps, s);
    // 16x16x64 on the 256 x 128 tile: alone / everything
    case 17: return launch_mix_sparse<true, false, 0>(src, d_out, steps, s);
    case 18: return launch_mix_sparse<true, false, 7>(src, d_out, steps, s);
    // sparse tile 256 x 256 alone: 32x32x32, 16x16x64
    case 19: return launch_mix_sparse<false, true, 0>(src, d_out, steps, s);
    default: return launch_mix_sparse<true, true, 0>(src, d_out, steps, s);
    }
}
