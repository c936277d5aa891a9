// Registration of the HIP codelet bodies with a StarPU built with its HIP
// driver.  The reference registers CUDA bodies only
// (src/starpu/codelet.cc:71-83: cuda_funcs[i], STARPU_CUDA_ASYNC, where |=
// STARPU_CUDA) and declares the attention bodies in
// include/nntile/starpu/flash_sdpa_fwd_cudnn.hh:77-87 and
// include/nntile/starpu/flash_sdpa_bwd_cudnn.hh; this unit is the HIP twin
// of those lines.  It compiles to two stubs where <starpu.h> is not installed
// (as in this repository's image): everything that needs StarPU sits behind
// __has_include, and the layout assumptions the C-ABI bodies make about
// StarPU's structures are static_asserts that a StarPU build checks.
#include <cstddef>
#include <cstdint>

#include "../../include/nntile_hip_sdpa.h"
#include "../../include/nntile_hip_starpu.h"

#if defined(__has_include)
#if __has_include(<starpu.h>) && __has_include(<starpu_hip.h>)
#define NNTILE_HIP_HAVE_STARPU 1
#endif
#endif

#ifdef NNTILE_HIP_HAVE_STARPU

#include <starpu.h>
#include <starpu_hip.h>

// The bodies read buffers[i] as nntile_hip_variable_interface: it must be
// StarPU's struct starpu_variable_interface, member for member
// (include/nntile/starpu/handle.hh:146-161 reads .ptr the same way).
static_assert(sizeof(nntile_hip_variable_interface) == sizeof(struct starpu_variable_interface),
        "nntile_hip_variable_interface differs from starpu_variable_interface");
static_assert(offsetof(nntile_hip_variable_interface, id)
        == offsetof(struct starpu_variable_interface, id), "id");
static_assert(offsetof(nntile_hip_variable_interface, ptr)
        == offsetof(struct starpu_variable_interface, ptr), "ptr");
static_assert(offsetof(nntile_hip_variable_interface, dev_handle)
        == offsetof(struct starpu_variable_interface, dev_handle), "dev_handle");
static_assert(offsetof(nntile_hip_variable_interface, offset)
        == offsetof(struct starpu_variable_interface, offset), "offset");
static_assert(offsetof(nntile_hip_variable_interface, elemsize)
        == offsetof(struct starpu_variable_interface, elemsize), "elemsize");
static_assert(sizeof(hipStream_t) == sizeof(void *), "streams travel as void *");

namespace
{

void *local_stream()
{
    // one stream per HIP worker; the bodies only enqueue on it
    return static_cast<void *>(starpu_hip_get_local_stream());
}

void add_hip(struct starpu_codelet *cl, void (*body)(void **, void *))
{
    cl->hip_funcs[0] = body;
    cl->hip_flags[0] = STARPU_HIP_ASYNC;    // StarPU waits on the stream, the body returns at once
    cl->where |= STARPU_HIP;
}

} // namespace

extern "C" int nntile_hip_starpu_available(void)
{
    return 1;
}

// cl_fwd, cl_bwd: the starpu_codelet objects behind
// starpu::FlashSdpaFwdCudnn<std::tuple<T>>::codelet and its backward twin
// (they derive from starpu_codelet, include/nntile/starpu/codelet.hh);
// dtype: NNTILE_HIP_DTYPE_BF16 / NNTILE_HIP_DTYPE_FP16 / 2 for fp32 (forward
// only).  Either pointer may be null.  Returns 0, or -1 for a dtype without
// a body.
extern "C" int nntile_hip_starpu_register(void *cl_fwd, void *cl_bwd, int dtype)
{
    nntile_hip_set_stream_provider(&local_stream);
    void (*fwd)(void **, void *) = nullptr;
    void (*bwd)(void **, void *) = nullptr;
    switch(dtype)
    {
        case NNTILE_HIP_DTYPE_BF16:
            fwd = nntile_hip_flash_sdpa_fwd_codelet_bf16;
            bwd = nntile_hip_flash_sdpa_bwd_codelet_bf16;
            break;
        case NNTILE_HIP_DTYPE_FP16:
            fwd = nntile_hip_flash_sdpa_fwd_codelet_fp16;
            bwd = nntile_hip_flash_sdpa_bwd_codelet_fp16;
            break;
        case 2:
            fwd = nntile_hip_flash_sdpa_fwd_codelet_fp32;
            break;
        default:
            return -1;
    }
    if(cl_fwd != nullptr)
    {
        add_hip(static_cast<struct starpu_codelet *>(cl_fwd), fwd);
    }
    if(cl_bwd != nullptr)
    {
        if(bwd == nullptr)
        {
            return -1;
        }
        add_hip(static_cast<struct starpu_codelet *>(cl_bwd), bwd);
    }
    return 0;
}

// The codelets of the whole-grid calls take any number of handles
extern "C" int nntile_hip_starpu_register_grid(void *cl_fwd_grid, void *cl_bwd_grid, int dtype)
{
    nntile_hip_set_stream_provider(&local_stream);
    void (*fwd)(void **, void *) = nullptr;
    void (*bwd)(void **, void *) = nullptr;
    switch(dtype)
    {
        case NNTILE_HIP_DTYPE_BF16:
            fwd = nntile_hip_sdpa_fwd_grid_codelet_bf16;
            bwd = nntile_hip_sdpa_bwd_grid_codelet_bf16;
            break;
        case NNTILE_HIP_DTYPE_FP16:
            fwd = nntile_hip_sdpa_fwd_grid_codelet_fp16;
            bwd = nntile_hip_sdpa_bwd_grid_codelet_fp16;
            break;
        case 2:
            fwd = nntile_hip_sdpa_fwd_grid_codelet_fp32;
            break;
        default:
            return -1;
    }
    if(cl_fwd_grid != nullptr)
    {
        auto *cl = static_cast<struct starpu_codelet *>(cl_fwd_grid);
        cl->nbuffers = STARPU_VARIABLE_NBUFFERS;
        add_hip(cl, fwd);
    }
    if(cl_bwd_grid != nullptr)
    {
        if(bwd == nullptr)
        {
            return -1;
        }
        auto *cl = static_cast<struct starpu_codelet *>(cl_bwd_grid);
        cl->nbuffers = STARPU_VARIABLE_NBUFFERS;
        add_hip(cl, bwd);
    }
    return 0;
}

#else // no StarPU in this build

extern "C" int nntile_hip_starpu_available(void)
{
    return 0;
}

extern "C" int nntile_hip_starpu_register(void *, void *, int)
{
    return -1;      // built without StarPU
}

extern "C" int nntile_hip_starpu_register_grid(void *, void *, int)
{
    return -1;
}

#endif
