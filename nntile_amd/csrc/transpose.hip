// dst = alpha * src^T for an m x n matrix in Fortran order (element (i, j) of
// src at i + j*m, element (j, i) of dst at j + i*n), the step that moves the
// projections into the attention layout and the attention output back
// (src/kernel/transpose/cpu.cc:21-43 is the arithmetic: one product in fp32,
// one rounding to the tile type).  A workgroup moves a 64 x 64 block through
// LDS: reads run along i, writes along j, both over whole 64-element rows.
#include "sdpa_common.hpp"

namespace nntile_hip
{

struct TrF32
{
    typedef float storage;
    static __device__ __forceinline__ float to_float(float v) { return v; }
    static __device__ __forceinline__ float from_float(float v) { return v; }
};
struct TrBf16
{
    typedef uint16_t storage;
    static __device__ __forceinline__ float to_float(uint16_t v) { return Bf16::to_float(v); }
    static __device__ __forceinline__ uint16_t from_float(float v) { return Bf16::from_float(v); }
};
struct TrFp16
{
    typedef uint16_t storage;
    static __device__ __forceinline__ float to_float(uint16_t v) { return Fp16::to_float(v); }
    static __device__ __forceinline__ uint16_t from_float(float v) { return Fp16::from_float(v); }
};

constexpr int kTrTile = 64;

template<typename S>
__global__ __launch_bounds__(256)
void transpose_kernel(int64_t m, int64_t n, int64_t tiles_m, float alpha,
        const typename S::storage *src, typename S::storage *dst)
{
    typedef typename S::storage E;
    // one column of padding: the transposed reads of a wave fall on 64 banks
    __shared__ E tile[kTrTile][kTrTile + (sizeof(E) == 2 ? 2 : 1)];
    const int64_t i0 = (int64_t)(blockIdx.x % tiles_m) * kTrTile;
    const int64_t j0 = (int64_t)(blockIdx.x / tiles_m) * kTrTile;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    // tile[j][i] = src(i0 + i, j0 + j): 64 consecutive i per wave load
#pragma unroll
    for(int r = 0; r < 16; ++r)
    {
        const int j = ty * 16 + r;
        if(i0 + tx < m && j0 + j < n)
        {
            tile[j][tx] = src[(i0 + tx) + (j0 + j) * m];
        }
    }
    __syncthreads();
    // dst(j0 + j, i0 + i) = alpha * tile[j][i]: 64 consecutive j per wave store
#pragma unroll
    for(int r = 0; r < 16; ++r)
    {
        const int i = ty * 16 + r;
        if(i0 + i < m && j0 + tx < n)
        {
            dst[(j0 + tx) + (i0 + i) * n] = S::from_float(alpha * S::to_float(tile[tx][i]));
        }
    }
}

// 16-bit tiles with m and n multiples of 8 and 16-byte aligned buffers: a
// block of 128 (i) x 32 (j) per workgroup, 16 bytes per global access.  A
// thread reads 8 consecutive i of two neighbouring columns, pairs them into
// 32-bit words (i, j..j+1) and writes those to LDS row i; then it reads 8
// consecutive j of one row and stores them as one 16-byte chunk, a wave 64
// neighbouring chunks.  With n == 32 the block is one contiguous piece of dst.
#ifndef NNTILE_TR16_ITERS
#define NNTILE_TR16_ITERS 1
#endif
constexpr int kTr16Iters = NNTILE_TR16_ITERS;       // 128 rows i per iteration
constexpr int kTr16I = 128 * kTr16Iters, kTr16J = 32, kTr16Pitch = kTr16J / 2 + 1;   // pitch in words

template<typename S>
__global__ __launch_bounds__(256)
void transpose16_kernel(int64_t m, int64_t n, int64_t tiles_m, float alpha,
        const uint16_t *src, uint16_t *dst)
{
    __shared__ uint32_t tile[kTr16I * kTr16Pitch];
    const int64_t i0 = (int64_t)(blockIdx.x % tiles_m) * kTr16I;
    const int64_t j0 = (int64_t)(blockIdx.x / tiles_m) * kTr16J;
    const int tid = threadIdx.x;
    {
        const int c = tid % 16, jp = tid / 16;          // 8 rows i, column pair
        const int64_t j = j0 + 2 * jp;
        u32x4 a[kTr16Iters], b[kTr16Iters];
#pragma unroll
        for(int it = 0; it < kTr16Iters; ++it)
        {
            const int64_t i = i0 + 128 * it + 8 * c;
            a[it] = u32x4{0, 0, 0, 0};
            b[it] = u32x4{0, 0, 0, 0};
            if(i < m && j < n)
            {
                a[it] = __builtin_nontemporal_load(
                        reinterpret_cast<const u32x4 *>(src + i + j * m));
                b[it] = __builtin_nontemporal_load(
                        reinterpret_cast<const u32x4 *>(src + i + (j + 1) * m));
            }
        }
#pragma unroll
        for(int it = 0; it < kTr16Iters; ++it)
        {
#pragma unroll
            for(int e = 0; e < 4; ++e)
            {
                // a[e] holds rows 2e, 2e+1 of column j; b[e] those of column j+1
                const int r = 128 * it + 8 * c + 2 * e;
                tile[r * kTr16Pitch + jp] = (a[it][e] & 0xffffu) | (b[it][e] << 16);
                tile[(r + 1) * kTr16Pitch + jp] = (a[it][e] >> 16) | (b[it][e] & 0xffff0000u);
            }
        }
    }
    __syncthreads();
    // a wave stores 64 neighbouring 16-byte chunks: 4 chunks (32 columns) a row
#pragma unroll
    for(int q = 0; q < 2 * kTr16Iters; ++q)
    {
        const int k = tid + 256 * q;
        const int r = k / 4, part = k % 4;
        const int64_t i = i0 + r, j = j0 + 8 * part;
        uint32_t w[4];
#pragma unroll
        for(int x = 0; x < 4; ++x)
        {
            w[x] = tile[r * kTr16Pitch + 4 * part + x];
        }
        if(alpha != 1.0f)
        {
#pragma unroll
            for(int x = 0; x < 4; ++x)
            {
                const float lo = alpha * S::to_float((uint16_t)(w[x] & 0xffffu));
                const float hi = alpha * S::to_float((uint16_t)(w[x] >> 16));
                w[x] = (uint32_t)S::from_float(lo) | ((uint32_t)S::from_float(hi) << 16);
            }
        }
        if(i < m && j < n)
        {
            __builtin_nontemporal_store(u32x4{w[0], w[1], w[2], w[3]},
                    reinterpret_cast<u32x4 *>(dst + j + i * n));
        }
    }
}

template<typename S>
static int launch_transpose_typed(hipStream_t stream, int64_t m, int64_t n, float alpha,
        const void *src, void *dst)
{
    typedef typename S::storage E;
    if constexpr(sizeof(E) == 2)
    {
        if(m % 8 == 0 && n % 8 == 0 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0
                && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0)
        {
            const int64_t tm = (m + kTr16I - 1) / kTr16I, tn = (n + kTr16J - 1) / kTr16J;
            if(tm > 0x7fffffff / tn)
            {
                return NNTILE_HIP_EINVAL;
            }
            hipLaunchKernelGGL((transpose16_kernel<S>), dim3((unsigned)(tm * tn)), dim3(256), 0,
                    stream, m, n, tm, alpha, static_cast<const uint16_t *>(src),
                    static_cast<uint16_t *>(dst));
            return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
        }
    }
    const int64_t tiles_m = (m + kTrTile - 1) / kTrTile, tiles_n = (n + kTrTile - 1) / kTrTile;
    if(tiles_m > 0x7fffffff / tiles_n)
    {
        return NNTILE_HIP_EINVAL;
    }
    hipLaunchKernelGGL((transpose_kernel<S>), dim3((unsigned)(tiles_m * tiles_n)), dim3(256), 0,
            stream, m, n, tiles_m, alpha, static_cast<const E *>(src), static_cast<E *>(dst));
    return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
}

// dtype: 0 bf16, 1 fp16, 2 fp32
int launch_transpose(hipStream_t stream, int dtype, int64_t m, int64_t n, float alpha,
        const void *src, void *dst)
{
    switch(dtype)
    {
        case 0: return launch_transpose_typed<TrBf16>(stream, m, n, alpha, src, dst);
        case 1: return launch_transpose_typed<TrFp16>(stream, m, n, alpha, src, dst);
        case 2: return launch_transpose_typed<TrF32>(stream, m, n, alpha, src, dst);
        default: return NNTILE_HIP_EINVAL;
    }
}

} // namespace nntile_hip
