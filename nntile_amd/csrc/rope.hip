// Rotary position embedding and its backward on a (2, m, n) tensor with
// sines and cosines of shape (m) (src/kernel/rope/cpu.cc:22-52,
// src/kernel/rope_backward/cpu.cc:22-53 are the arithmetic this follows):
//
//   forward:   dst[2i,j]   = cos[i] src[2i,j] - sin[i] src[2i+1,j]
//              dst[2i+1,j] = sin[i] src[2i,j] + cos[i] src[2i+1,j]
//   backward:  dx[2i,j]    = cos[i] dy[2i,j] + sin[i] dy[2i+1,j]
//              dx[2i+1,j]  = cos[i] dy[2i+1,j] - sin[i] dy[2i,j]
//
// (the backward writes dx, it does not add to it).  Products and sums in fp32,
// one rounding to the tile type.  Pure streaming: a thread takes four
// neighbouring pairs - 16 bytes of a 16-bit tensor, 32 of an fp32 one - and
// the four sines and cosines that go with them; m not a multiple of 4, or
// addresses that are not aligned for that, take one pair per thread.
#include "sdpa_common.hpp"

namespace nntile_hip
{

struct RopeF32
{
    typedef float storage;
    static __device__ __forceinline__ float to_float(float v) { return v; }
    static __device__ __forceinline__ float from_float(float v) { return v; }
};
struct RopeBf16
{
    typedef uint16_t storage;
    static __device__ __forceinline__ float to_float(uint16_t v) { return Bf16::to_float(v); }
    static __device__ __forceinline__ uint16_t from_float(float v) { return Bf16::from_float(v); }
};
struct RopeFp16
{
    typedef uint16_t storage;
    static __device__ __forceinline__ float to_float(uint16_t v) { return Fp16::to_float(v); }
    static __device__ __forceinline__ uint16_t from_float(float v) { return Fp16::from_float(v); }
};

template<bool BACKWARD>
__device__ __forceinline__ void rotate(float c, float s, float a, float b, float &x, float &y)
{
    if(BACKWARD)
    {
        x = fmaf(c, a, s * b);
        y = fmaf(c, b, -(s * a));
    }
    else
    {
        x = fmaf(c, a, -(s * b));
        y = fmaf(s, a, c * b);
    }
}

template<typename S, bool BACKWARD>
__global__ __launch_bounds__(256)
void rope_vec_kernel(int64_t m, int64_t quads, const typename S::storage *sin,
        const typename S::storage *cos, const typename S::storage *src,
        typename S::storage *dst)
{
    typedef typename S::storage E;
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if(t >= quads)
    {
        return;
    }
    const int64_t i = (4 * t) % m;              // m % 4 == 0: the four share a column j
    __attribute__((aligned(16))) E in[8];
    __attribute__((aligned(16))) E out[8];
    __attribute__((aligned(16))) E sv[4];
    __attribute__((aligned(16))) E cv[4];
    // src and dst pass through once (non-temporal); sin and cos are re-read
    // by every column j and stay cached
    if constexpr(sizeof(E) == 2)
    {
        *reinterpret_cast<u32x4 *>(in) = __builtin_nontemporal_load(
                reinterpret_cast<const u32x4 *>(src + 8 * t));
        *reinterpret_cast<u32x2 *>(sv) = *reinterpret_cast<const u32x2 *>(sin + i);
        *reinterpret_cast<u32x2 *>(cv) = *reinterpret_cast<const u32x2 *>(cos + i);
    }
    else
    {
        reinterpret_cast<u32x4 *>(in)[0] = __builtin_nontemporal_load(
                reinterpret_cast<const u32x4 *>(src + 8 * t));
        reinterpret_cast<u32x4 *>(in)[1] = __builtin_nontemporal_load(
                reinterpret_cast<const u32x4 *>(src + 8 * t) + 1);
        *reinterpret_cast<u32x4 *>(sv) = *reinterpret_cast<const u32x4 *>(sin + i);
        *reinterpret_cast<u32x4 *>(cv) = *reinterpret_cast<const u32x4 *>(cos + i);
    }
#pragma unroll
    for(int k = 0; k < 4; ++k)
    {
        float x, y;
        rotate<BACKWARD>(S::to_float(cv[k]), S::to_float(sv[k]), S::to_float(in[2 * k]),
                S::to_float(in[2 * k + 1]), x, y);
        out[2 * k] = S::from_float(x);
        out[2 * k + 1] = S::from_float(y);
    }
    if constexpr(sizeof(E) == 2)
    {
        __builtin_nontemporal_store(*reinterpret_cast<const u32x4 *>(out),
                reinterpret_cast<u32x4 *>(dst + 8 * t));
    }
    else
    {
        __builtin_nontemporal_store(reinterpret_cast<const u32x4 *>(out)[0],
                reinterpret_cast<u32x4 *>(dst + 8 * t));
        __builtin_nontemporal_store(reinterpret_cast<const u32x4 *>(out)[1],
                reinterpret_cast<u32x4 *>(dst + 8 * t) + 1);
    }
}

template<typename S, bool BACKWARD>
__global__ __launch_bounds__(256)
void rope_pair_kernel(int64_t m, int64_t pairs, const typename S::storage *sin,
        const typename S::storage *cos, const typename S::storage *src,
        typename S::storage *dst)
{
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if(t >= pairs)
    {
        return;
    }
    const int64_t i = t % m;
    float x, y;
    rotate<BACKWARD>(S::to_float(cos[i]), S::to_float(sin[i]), S::to_float(src[2 * t]),
            S::to_float(src[2 * t + 1]), x, y);
    dst[2 * t] = S::from_float(x);
    dst[2 * t + 1] = S::from_float(y);
}

template<typename S, bool BACKWARD>
static int launch_rope_typed(hipStream_t stream, int64_t m, int64_t n, const void *sin_,
        const void *cos_, const void *src_, void *dst_)
{
    typedef typename S::storage E;
    const E *sin = static_cast<const E *>(sin_), *cos = static_cast<const E *>(cos_);
    const E *src = static_cast<const E *>(src_);
    E *dst = static_cast<E *>(dst_);
    const int64_t pairs = m * n;
    auto aligned = [](const void *p, uintptr_t a)
    {
        return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
    };
    const bool vec = m % 4 == 0 && aligned(src, 16) && aligned(dst, 16)
        && aligned(sin, 4 * sizeof(E)) && aligned(cos, 4 * sizeof(E));
    const int64_t threads = vec ? pairs / 4 : pairs;
    const int64_t blocks = (threads + 255) / 256;
    if(blocks > 0x7fffffff)
    {
        return NNTILE_HIP_EINVAL;
    }
    if(vec)
    {
        hipLaunchKernelGGL((rope_vec_kernel<S, BACKWARD>), dim3((unsigned)blocks), dim3(256), 0,
                stream, m, threads, sin, cos, src, dst);
    }
    else
    {
        hipLaunchKernelGGL((rope_pair_kernel<S, BACKWARD>), dim3((unsigned)blocks), dim3(256), 0,
                stream, m, threads, sin, cos, src, dst);
    }
    return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
}

// dtype: 0 bf16, 1 fp16, 2 fp32
int launch_rope(hipStream_t stream, int dtype, bool backward, int64_t m, int64_t n,
        const void *sin, const void *cos, const void *src, void *dst)
{
    switch(dtype * 2 + (backward ? 1 : 0))
    {
        case 0: return launch_rope_typed<RopeBf16, false>(stream, m, n, sin, cos, src, dst);
        case 1: return launch_rope_typed<RopeBf16, true>(stream, m, n, sin, cos, src, dst);
        case 2: return launch_rope_typed<RopeFp16, false>(stream, m, n, sin, cos, src, dst);
        case 3: return launch_rope_typed<RopeFp16, true>(stream, m, n, sin, cos, src, dst);
        case 4: return launch_rope_typed<RopeF32, false>(stream, m, n, sin, cos, src, dst);
        case 5: return launch_rope_typed<RopeF32, true>(stream, m, n, sin, cos, src, dst);
        default: return NNTILE_HIP_EINVAL;
    }
}

} // namespace nntile_hip
