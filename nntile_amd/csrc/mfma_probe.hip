// Measurement aid, not part of the product library: the rate at which the
// matrix units execute v_mfma_f32_32x32x16_bf16 on operands that stay in
// registers, two wavefronts per SIMD and nothing else going on.  bench.py runs
// it for a second or two on zero and on N(0,1) operands: what the board's
// power management leaves of the published peak on such data bounds every
// kernel that feeds its matrix units with it.
#include <hip/hip_runtime.h>
#include <cstdint>

namespace
{

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

// operands: 4 x 256 lanes x 8 bf16 values (16 KiB); four independent
// accumulator chains per wavefront
__global__ __launch_bounds__(256, 2)
void mfma_probe_kernel(const bf16x8 *operands, float *sink, int iters)
{
    const int lane = threadIdx.x;
    const bf16x8 a0 = operands[lane], a1 = operands[256 + lane];
    const bf16x8 b0 = operands[512 + lane], b1 = operands[768 + lane];
    f32x16 c0, c1, c2, c3;
    for(int r = 0; r < 16; ++r)
    {
        c0[r] = 0.0f;
        c1[r] = 0.0f;
        c2[r] = 0.0f;
        c3[r] = 0.0f;
    }
    for(int it = 0; it < iters; ++it)
    {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b0, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b0, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b1, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b1, c3, 0, 0, 0);
    }
    float s = 0.0f;
    for(int r = 0; r < 16; ++r)
    {
        s += c0[r] + c1[r] + c2[r] + c3[r];
    }
    if(s == 12345.678f)     // (keeps the products alive)
    {
        sink[0] = s;
    }
}

} // namespace

// FLOPs one launch executes: workgroups x 4 wavefronts x iters x 4 MFMAs x 32768.
extern "C" int nntile_hip_probe_mfma(void *stream, const void *operands, float *sink,
        int32_t iters, int32_t workgroups)
{
    if(operands == nullptr || sink == nullptr || iters <= 0 || workgroups <= 0)
    {
        return 1;
    }
    hipLaunchKernelGGL(mfma_probe_kernel, dim3((unsigned)workgroups), dim3(256), 0,
            static_cast<hipStream_t>(stream), static_cast<const bf16x8 *>(operands), sink, iters);
    return hipGetLastError() == hipSuccess ? 0 : 5;
}
