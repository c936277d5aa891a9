/* Registration of the HIP codelet bodies of nntile_hip_sdpa.h with a StarPU
 * that was built with its HIP driver.  Exported by libnntile_host.so
 * (nntile_amd/host/starpu_hip_registration.cc).
 *
 * The reference registers CUDA bodies only (src/starpu/codelet.cc:71-83:
 * cuda_funcs[i], cuda_flags[i] = STARPU_CUDA_ASYNC, where |= STARPU_CUDA); these
 * functions do the same for hip_funcs[0] / STARPU_HIP_ASYNC / STARPU_HIP on the
 * starpu_codelet objects the reference's codelet wrappers derive from
 * (include/nntile/starpu/codelet.hh), and install starpu_hip_get_local_stream
 * as the stream the bodies enqueue on.  Where the library was built without
 * StarPU's headers they are stubs: available() returns 0, the others -1. */
#ifndef NNTILE_HIP_STARPU_H
#define NNTILE_HIP_STARPU_H

#ifdef __cplusplus
extern "C" {
#endif

/* 1 when the library was built against <starpu.h> and <starpu_hip.h> */
int nntile_hip_starpu_available(void);

/* cl_fwd, cl_bwd: struct starpu_codelet * of
 * starpu::FlashSdpaFwdCudnn<std::tuple<T>> and starpu::FlashSdpaBwdCudnn<...>
 * (include/nntile/starpu/flash_sdpa_fwd_cudnn.hh:44-145,
 * include/nntile/starpu/flash_sdpa_bwd_cudnn.hh); either may be null.
 * dtype: NNTILE_HIP_DTYPE_BF16, NNTILE_HIP_DTYPE_FP16, or 2 for fp32 (forward
 * only).  Returns 0, or -1 for a dtype without a body. */
int nntile_hip_starpu_register(void *cl_fwd, void *cl_bwd, int dtype);

/* The same for the codelets of the whole-grid calls
 * (nntile_hip_sdpa_fwd_grid_codelet_*, nntile_hip_sdpa_bwd_grid_codelet_*):
 * two further starpu_codelet objects with nbuffers = STARPU_VARIABLE_NBUFFERS,
 * as src/starpu/codelet.cc:58 sets it for every NNTile codelet. */
int nntile_hip_starpu_register_grid(void *cl_fwd_grid, void *cl_bwd_grid, int dtype);

#ifdef __cplusplus
}
#endif

#endif /* NNTILE_HIP_STARPU_H */
