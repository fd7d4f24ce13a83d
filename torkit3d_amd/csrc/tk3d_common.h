// Shared host/device helpers for the gfx950 point-cloud kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <stdint.h>

#include "tk3d.h"

// All kernels are written for 64-lane wavefronts.
#define TK_WAVE 64

// Every source file is compiled with -ffp-contract=off; the fused steps of the
// canonical distance are written out here and nowhere else.
template <typename T> __device__ __forceinline__ T tk_fma(T a, T b, T c);
template <> __device__ __forceinline__ float tk_fma<float>(float a, float b, float c)
{
    return __builtin_fmaf(a, b, c);
}
template <> __device__ __forceinline__ double tk_fma<double>(double a, double b, double c)
{
    return __builtin_fma(a, b, c);
}

template <typename T> __device__ __forceinline__ T tk_min(T a, T b);
template <> __device__ __forceinline__ float tk_min<float>(float a, float b)
{
    return __builtin_fminf(a, b);
}
template <> __device__ __forceinline__ double tk_min<double>(double a, double b)
{
    return __builtin_fmin(a, b);
}
template <typename T> __device__ __forceinline__ T tk_max(T a, T b);
template <> __device__ __forceinline__ float tk_max<float>(float a, float b)
{
    return __builtin_fmaxf(a, b);
}
template <> __device__ __forceinline__ double tk_max<double>(double a, double b)
{
    return __builtin_fmax(a, b);
}

template <typename T> __device__ __forceinline__ T tk_inf()
{
    return (T)__builtin_huge_valf();
}

// Squared distance between key (kx,ky,kz) and query (qx,qy,qz):
// fma(dz,dz, fma(dy,dy, dx*dx)) with dx = kx - qx, the value the reference
// kernels produce (e.g. chamfer_distance_kernel.cu:65-71 under nvcc's default
// contraction).
template <typename T>
__device__ __forceinline__ T tk_dist2(T kx, T ky, T kz, T qx, T qy, T qz)
{
    const T dx = kx - qx;
    const T dy = ky - qy;
    const T dz = kz - qz;
    T d = dx * dx;
    d = tk_fma<T>(dy, dy, d);
    d = tk_fma<T>(dz, dz, d);
    return d;
}

// The three coordinates p[0..2] of one point as a single 12-byte (fp64: 24-byte) load;
// p needs only the alignment of T, which is all a row of an [N,3] array has.
template <typename T> struct __attribute__((packed, aligned(sizeof(T)))) TkPoint3 {
    T x, y, z;
};
template <typename T> __device__ __forceinline__ TkPoint3<T> tk_load3(const T *p)
{
    return *reinterpret_cast<const TkPoint3<T> *>(p);
}

// ---- fp16 pieces for scores computed on the matrix cores ------------------------------

typedef _Float16 tk_f16x8 __attribute__((ext_vector_type(8)));
typedef float tk_f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ unsigned tk_f16_bits(float x)  // nearest fp16
{
    return (unsigned)__builtin_bit_cast(unsigned short, (_Float16)x);
}
__device__ __forceinline__ float tk_f16_value(unsigned b)
{
    return (float)__builtin_bit_cast(_Float16, (unsigned short)b);
}
// x = hi + lo + e with |e| <= 2^-23 |x| + 2^-25 (fp16 has 11 significant bits: the first
// piece is within 2^-11 |x| of x, the second within 2^-12 of the rest or within half the
// subnormal spacing 2^-24); returns hi | lo << 16. x beyond +-65504 gives an infinite hi
// and a NaN lo.
__device__ __forceinline__ unsigned tk_f16_split2(float x)
{
    const unsigned hi = tk_f16_bits(x);
    const unsigned lo = tk_f16_bits(x - tk_f16_value(hi));  // the difference is exact
    return hi | (lo << 16);
}

// ---- host side --------------------------------------------------------------

static inline int tk_launch_status()
{
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? TK3D_OK : (int)e;
}

// Raises the dynamic LDS limit of `Kernel` to `bytes` on the current device; done once
// per device and kernel (the attribute belongs to the device's copy of the code).
// Returns TK3D_OK or the hipError_t.
template <auto Kernel> static inline int tk_allow_dynamic_lds(int bytes)
{
    static std::atomic<unsigned long long> done{0};  // one bit per device ordinal
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return (int)e;
    if (dev >= 0 && dev < 64 && ((done.load(std::memory_order_acquire) >> dev) & 1ull))
        return TK3D_OK;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(Kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess)
        return (int)e;
    if (dev >= 0 && dev < 64)
        done.fetch_or(1ull << dev, std::memory_order_release);
    return TK3D_OK;
}

// Compute units of the current device (256 when the query fails), looked up once per device.
static inline int tk_cu_count()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return 256;
    int n = cached[dev].load(std::memory_order_acquire);
    if (n > 0)
        return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
        n = 256;
    cached[dev].store(n, std::memory_order_release);
    return n;
}

// True when a*b*c... of non-negative sizes fits in int64 and is below `limit`.
static inline bool tk_fits(int64_t limit, int64_t a, int64_t b = 1, int64_t c = 1,
                           int64_t d = 1)
{
    const int64_t v[4] = {a, b, c, d};
    __int128 p = 1;
    for (int i = 0; i < 4; ++i) {
        if (v[i] < 0)
            return false;
        p *= v[i];
        if (p > (__int128)limit)
            return false;
    }
    return true;
}

// Largest element count a kernel addresses with a signed 64-bit offset in bytes.
#define TK_MAX_ELEMS ((int64_t)1 << 58)
// Largest value carried in a 32-bit in-kernel index.
#define TK_MAX_I32 ((int64_t)0x7fffffff)
