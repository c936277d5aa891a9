// Class of one tile of a materialised attention mask, so that the layer above
// the kernel can decide per (query tile, key tile) pair whether a task is
// needed at all and whether it needs the mask
// (src/tensor/flash_sdpa_fwd_cudnn.cc:246-274 submits every pair with its
// mask tile).  The tile is [k_rows, q_cols] in Fortran order - query q, key k
// at mask[k + q*k_rows] - additive in the tile type (0 visible, -inf hidden)
// or bool (true visible).
//
// One pass over the tile sets four flags in a device word:
//   VISIBLE  some element is visible (0 / true)
//   HIDDEN   some element is hidden (-inf / false)
//   OTHER    some additive element is neither 0 nor -inf (a bias: the mask
//            must then be read by the attention kernel)
//   OFF_RULE some element differs from the rule  visible <=> k <= q + offset
// HBM-bound: reads the tile once, writes nothing but the word.
#include "sdpa_common.hpp"

namespace nntile_hip
{

enum : uint32_t { kSeenVisible = 1, kSeenHidden = 2, kSeenOther = 4, kSeenOffRule = 8 };

struct MaskF32
{
    typedef float storage;
    static __device__ __forceinline__ uint32_t kind(float v)
    {
        return v == 0.0f ? kSeenVisible : (v == -__builtin_inff() ? kSeenHidden : kSeenOther);
    }
};
struct MaskBf16
{
    typedef uint16_t storage;
    static __device__ __forceinline__ uint32_t kind(uint16_t v)
    {
        return (v & 0x7fffu) == 0 ? kSeenVisible : (v == 0xff80u ? kSeenHidden : kSeenOther);
    }
};
struct MaskFp16
{
    typedef uint16_t storage;
    static __device__ __forceinline__ uint32_t kind(uint16_t v)
    {
        return (v & 0x7fffu) == 0 ? kSeenVisible : (v == 0xfc00u ? kSeenHidden : kSeenOther);
    }
};
struct MaskBool
{
    typedef uint8_t storage;
    static __device__ __forceinline__ uint32_t kind(uint8_t v)
    {
        return v ? kSeenVisible : kSeenHidden;
    }
};

// One workgroup per CHUNK elements of the flattened tile; a thread walks its
// elements with stride 256 so that a wave reads neighbouring addresses.
constexpr int kClassifyChunk = 4096;

template<typename M>
__global__ __launch_bounds__(256)
void mask_classify_kernel(int64_t k_rows, int64_t total, int64_t offset,
        const typename M::storage *mask, uint32_t *flags)
{
    const int64_t base = (int64_t)blockIdx.x * kClassifyChunk;
    const int64_t end = min(base + kClassifyChunk, total);
    uint32_t seen = 0;
    // position of the first element of this thread, then advanced by 256
    int64_t e = base + threadIdx.x;
    int64_t q = e / k_rows;
    int64_t k = e - q * k_rows;
    const int64_t dq = 256 / k_rows, dk = 256 - dq * k_rows;
    for(; e < end; e += 256)
    {
        const uint32_t kind = M::kind(mask[e]);
        const bool rule_visible = k <= q + offset;
        seen |= kind;
        if((kind == kSeenVisible) != rule_visible)
        {
            seen |= kSeenOffRule;
        }
        q += dq;
        k += dk;
        if(k >= k_rows)
        {
            k -= k_rows;
            q += 1;
        }
    }
    // OR over the wave, then one atomic per wave that has anything new to say
#pragma unroll
    for(int bit = 1; bit <= 8; bit <<= 1)
    {
        if(__builtin_amdgcn_ballot_w64((seen & bit) != 0) != 0)
        {
            seen |= bit;
        }
    }
    // Bits are only ever set, so a wave whose bits are all in the word already
    // has nothing to add: after the first few waves the atomics stop.
    if((threadIdx.x & 63) == 0
            && (seen & ~__atomic_load_n(flags, __ATOMIC_RELAXED)) != 0)
    {
        atomicOr(flags, seen);
    }
}

__global__ void mask_classify_clear_kernel(uint32_t *flags)
{
    *flags = 0;
}

// dtype: 0 bf16, 1 fp16, 2 fp32, 3 bool.  flags: one device word.
int launch_mask_classify(hipStream_t stream, int dtype, int64_t k_rows, int64_t q_cols,
        int64_t offset, const void *mask, uint32_t *flags)
{
    const int64_t total = k_rows * q_cols;
    const int64_t blocks = (total + kClassifyChunk - 1) / kClassifyChunk;
    if(blocks > 0x7fffffff)
    {
        return NNTILE_HIP_EINVAL;
    }
    hipLaunchKernelGGL(mask_classify_clear_kernel, dim3(1), dim3(1), 0, stream, flags);
    const dim3 grid((unsigned)blocks), block(256);
    switch(dtype)
    {
        case 0:
            hipLaunchKernelGGL(mask_classify_kernel<MaskBf16>, grid, block, 0, stream, k_rows,
                    total, offset, static_cast<const uint16_t *>(mask), flags);
            break;
        case 1:
            hipLaunchKernelGGL(mask_classify_kernel<MaskFp16>, grid, block, 0, stream, k_rows,
                    total, offset, static_cast<const uint16_t *>(mask), flags);
            break;
        case 2:
            hipLaunchKernelGGL(mask_classify_kernel<MaskF32>, grid, block, 0, stream, k_rows,
                    total, offset, static_cast<const float *>(mask), flags);
            break;
        case 3:
            hipLaunchKernelGGL(mask_classify_kernel<MaskBool>, grid, block, 0, stream, k_rows,
                    total, offset, static_cast<const uint8_t *>(mask), flags);
            break;
        default:
            return NNTILE_HIP_EINVAL;
    }
    return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
}

} // namespace nntile_hip
