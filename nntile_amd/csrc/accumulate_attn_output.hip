// Merge of a partial (lse, attn) pair into the running pair, row by row:
//   L = logaddexp(dst_lse, src_lse)
//   dst_attn <- exp(dst_lse - L) * dst_attn + exp(src_lse - L) * src_attn
//   dst_lse  <- L
// A side at -inf has weight 0 (its values are not read); rows whose source is
// at -inf are left untouched.  Pure streaming: 16-byte accesses, one row's
// chunks on neighbouring lanes.
#include "sdpa_common.hpp"

namespace nntile_hip
{

struct F32Store
{
    typedef float storage;
    static constexpr int VEC = 4;
    static __device__ __forceinline__ float to_float(float v) { return v; }
    static __device__ __forceinline__ float from_float(float v) { return v; }
};
struct Bf16Store
{
    typedef uint16_t storage;
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float to_float(uint16_t v) { return Bf16::to_float(v); }
    static __device__ __forceinline__ uint16_t from_float(float v) { return Bf16::from_float(v); }
};
struct Fp16Store
{
    typedef uint16_t storage;
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float to_float(uint16_t v) { return Fp16::to_float(v); }
    static __device__ __forceinline__ uint16_t from_float(float v) { return Fp16::from_float(v); }
};

__device__ __forceinline__ bool row_weights(float have, float inc, float &w_have,
        float &w_inc, float &merged)
{
    // A source row whose logsumexp is not finite (-inf: no key seen; NaN or
    // +inf: a broken partial) leaves the destination as it is, the rule of the
    // reference's GPU kernel (src/kernel/accumulate_attn_output/cuda.cu:43-50).
    if(!__builtin_isfinite(inc))
    {
        return false;
    }
    merge_weights(have, inc, w_have, w_inc, merged);
    return true;
}

// Vector path: head % VEC == 0 and head / VEC <= 256.
template<typename S>
__global__ __launch_bounds__(256)
void accumulate_attn_output_vec_kernel(int64_t head, int64_t nrows,
        int chunks_per_row, int rows_per_block, const float *src_lse,
        const typename S::storage *src_attn, float *dst_lse,
        typename S::storage *dst_attn)
{
    typedef typename S::storage E;
    const int r_in_block = threadIdx.x / chunks_per_row;
    const int chunk = threadIdx.x % chunks_per_row;
    const int64_t row = (int64_t)blockIdx.x * rows_per_block + r_in_block;
    const bool active = r_in_block < rows_per_block && row < nrows;
    float w_have = 1.0f, w_inc = 0.0f, merged = 0.0f;
    bool touch = false;
    if(active)
    {
        touch = row_weights(dst_lse[row], src_lse[row], w_have, w_inc, merged);
    }
    __syncthreads();        // all lse reads of the block precede the lse writes
    if(!touch)
    {
        return;
    }
    if(chunk == 0)
    {
        dst_lse[row] = merged;
    }
    const int64_t off = row * head + (int64_t)chunk * S::VEC;
    __attribute__((aligned(16))) E in[S::VEC];
    __attribute__((aligned(16))) E out[S::VEC];
    *reinterpret_cast<u32x4 *>(in) = *reinterpret_cast<const u32x4 *>(src_attn + off);
    if(w_have != 0.0f)
    {
        *reinterpret_cast<u32x4 *>(out) = *reinterpret_cast<const u32x4 *>(dst_attn + off);
#pragma unroll
        for(int e = 0; e < S::VEC; ++e)
        {
            out[e] = S::from_float(w_have * S::to_float(out[e])
                    + w_inc * S::to_float(in[e]));
        }
    }
    else
    {
#pragma unroll
        for(int e = 0; e < S::VEC; ++e)
        {
            out[e] = S::from_float(w_inc * S::to_float(in[e]));
        }
    }
    *reinterpret_cast<u32x4 *>(dst_attn + off) = *reinterpret_cast<u32x4 *>(out);
}

// Any head size: one thread per row.
template<typename S>
__global__ __launch_bounds__(256)
void accumulate_attn_output_row_kernel(int64_t head, int64_t nrows,
        const float *src_lse, const typename S::storage *src_attn,
        float *dst_lse, typename S::storage *dst_attn)
{
    const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(row >= nrows)
    {
        return;
    }
    float w_have, w_inc, merged;
    if(!row_weights(dst_lse[row], src_lse[row], w_have, w_inc, merged))
    {
        return;
    }
    dst_lse[row] = merged;
    for(int64_t h = 0; h < head; ++h)
    {
        const int64_t e = row * head + h;
        const float old = (w_have != 0.0f) ? w_have * S::to_float(dst_attn[e]) : 0.0f;
        dst_attn[e] = S::from_float(old + w_inc * S::to_float(src_attn[e]));
    }
}

template<typename S>
int launch_accumulate(hipStream_t stream, int64_t head, int64_t seq,
        int64_t batch, const float *src_lse, const void *src_attn,
        float *dst_lse, void *dst_attn)
{
    typedef typename S::storage E;
    const int64_t nrows = seq * batch;
    const E *src = static_cast<const E *>(src_attn);
    E *dst = static_cast<E *>(dst_attn);
    const bool aligned = (reinterpret_cast<uintptr_t>(src) % 16 == 0)
        && (reinterpret_cast<uintptr_t>(dst) % 16 == 0);
    if(head % S::VEC == 0 && head / S::VEC <= 256 && aligned)
    {
        const int cpr = (int)(head / S::VEC);
        const int rpb = 256 / cpr;
        const int64_t blocks = (nrows + rpb - 1) / rpb;
        if(blocks > 0x7fffffff)
        {
            return NNTILE_HIP_EINVAL;
        }
        hipLaunchKernelGGL((accumulate_attn_output_vec_kernel<S>),
                dim3((unsigned)blocks), dim3(256), 0, stream, head, nrows, cpr,
                rpb, src_lse, src, dst_lse, dst);
    }
    else
    {
        const int64_t blocks = (nrows + 255) / 256;
        if(blocks > 0x7fffffff)
        {
            return NNTILE_HIP_EINVAL;
        }
        hipLaunchKernelGGL((accumulate_attn_output_row_kernel<S>),
                dim3((unsigned)blocks), dim3(256), 0, stream, head, nrows,
                src_lse, src, dst_lse, dst);
    }
    return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
}

template int launch_accumulate<F32Store>(hipStream_t, int64_t, int64_t, int64_t,
        const float *, const void *, float *, void *);
template int launch_accumulate<Bf16Store>(hipStream_t, int64_t, int64_t, int64_t,
        const float *, const void *, float *, void *);
template int launch_accumulate<Fp16Store>(hipStream_t, int64_t, int64_t, int64_t,
        const float *, const void *, float *, void *);

} // namespace nntile_hip
