// Shared host/device helpers for the nmg HIP library (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#include "../../include/nmg_hip.h"

namespace nmg {

// ---- error reporting (thread-local message, integer status) -------------------------------
void set_error(const char *fmt, ...);
int hip_fail(hipError_t e, const char *what, const char *file, int line);

#define NMG_HIP_TRY(expr)                                                         \
    do {                                                                          \
        hipError_t _e = (expr);                                                   \
        if (_e != hipSuccess) return ::nmg::hip_fail(_e, #expr, __FILE__, __LINE__); \
    } while (0)

#define NMG_REQUIRE(cond, code, ...)     \
    do {                                 \
        if (!(cond)) {                   \
            ::nmg::set_error(__VA_ARGS__); \
            return (code);               \
        }                                \
    } while (0)

// ---- pattern order tables -----------------------------------------------------------------
constexpr int kOrderSlotBytes = 8192;      // largest table: c*n int8 entries of one (n, m) pair
constexpr int kOrderPoolBytes = 64 * 1024;  // all tables of one device, packed 16-byte aligned

int64_t binom(int m, int n);
// Host copy of the table (cached per (n, m)); nullptr when (n, m) is invalid.
const int8_t *host_order(int n, int m);
// Device copy living in this library's file-scope table on the current device; copied there
// with a blocking hipMemcpy the first time an (n, m) pair is used on that device.
int device_order(int n, int m, const int8_t **d_order);
// 256 bytes of zeros on the current device (file-scope array, never written).
int device_zero_page(const void **d_zero);


// Y[G, S] = L[T, G]^T P[T, S] (+ bias[s]) in a 16-bit type on the matrix cores (nmg_sddmm.hip).
int dense_tn16(const void *d_lines, int64_t ld_lines, const void *d_pos, int64_t ld_pos, int64_t T, int64_t G, int64_t S,
               void *d_y, int64_t ldy, const void *d_bias, int dtype, void *stream);

inline size_t dtype_size(int dtype)
{
    switch (dtype) {
    case NMG_F32: return 4;
    case NMG_F16: return 2;
    case NMG_BF16: return 2;
    case NMG_F64: return 8;
    default: return 0;
    }
}

struct TileGeom {
    int64_t outer;       // number of tiles
    int64_t num_chunks;  // ceil(G / (c*g))
    int64_t num_blocks;  // ceil(S / m)
    int c, cols;         // patterns per tile; columns per tile = c*g
};

inline TileGeom tile_geom(const nmg_view &v, int n, int m, int g)
{
    TileGeom t;
    t.c = (int)binom(m, n);
    t.cols = t.c * g;
    t.num_chunks = (v.G + t.cols - 1) / t.cols;
    t.num_blocks = (v.S + m - 1) / m;
    t.outer = v.batch * t.num_chunks * t.num_blocks;
    return t;
}

// ---- device helpers -------------------------------------------------------------------------
#if defined(__HIPCC__)

// Element <-> fp32 conversions that keep the stored bits exact on the way back.
__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(__half x) { return __half2float(x); }
__device__ __forceinline__ float to_f32(__hip_bfloat16 x) { return __bfloat162float(x); }

template <typename T> struct Zero;
template <> struct Zero<float> { __device__ static float v() { return 0.f; } };
template <> struct Zero<double> { __device__ static double v() { return 0.0; } };
template <> struct Zero<__half> { __device__ static __half v() { return __ushort_as_half((unsigned short)0); } };
template <> struct Zero<__hip_bfloat16> {
    __device__ static __hip_bfloat16 v() { return __float2bfloat16(0.f); }
};

// Address of element (group index gi, sparse index si) of batch b in a strided view.
struct ViewDev {
    int64_t G, S, stride_b, stride_g, stride_s;
    int64_t num_chunks, num_blocks;
};

#endif

}  // namespace nmg
