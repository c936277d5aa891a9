/* C ABI of the MI355X (gfx950) tile-level scaled-dot-product-attention forward.
 *
 * One shared library, libnntile_hip_sdpa.so, plain pointers and sizes only.
 * Every entry point only ENQUEUES work on the HIP stream it is given: it never
 * allocates, never frees and - with one exception, the mask classification
 * nntile_hip_mask_tile_class_* of section 10, which hands a value back to the
 * host and therefore waits for the stream - never synchronises.  Return
 * value: 0 on success, a negative NNTILE_HIP_E* code otherwise (nothing is
 * enqueued on error).
 *
 * Data layout (NNTile tiles are Fortran-ordered):
 *   K, V       [head, k_seq, kv_batch]   element (h, s, b) at h + head*(s + k_seq*b)
 *   Q, A       [head, q_seq, batch]      element (h, s, b) at h + head*(s + q_seq*b)
 *   lse        [q_seq, batch]            fp32, natural-log units
 *   mask       [k_seq, q_seq]            element (k, q) at k + q*k_seq
 * 16-bit types are passed as their uint16 storage (bf16 / IEEE fp16).
 * Scores are scaled by 1/sqrt(head) BEFORE the mask is applied.
 *
 * Semantics shared by all forward entry points: the call attends the given
 * queries to the given keys and MERGES the result into the running pair
 * (lse, A): lse <- logaddexp(lse, lse_new), A <- w_old*A + w_new*A_new.  A
 * caller starts with lse = -inf (A may hold anything then, it is not read for
 * such rows) and calls once per key tile, in any order.  A query that sees no
 * key in this call leaves its lse and A row untouched.
 */
#ifndef NNTILE_HIP_SDPA_H
#define NNTILE_HIP_SDPA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NNTILE_HIP_OK            0
#define NNTILE_HIP_EINVAL       (-1)  /* null pointer / non-positive size / bad enum */
#define NNTILE_HIP_EUNSUPPORTED (-2)  /* head size or combination without a kernel */
#define NNTILE_HIP_ELAUNCH      (-3)  /* the HIP runtime refused the launch */
#define NNTILE_HIP_EWORKSPACE   (-4)  /* workspace missing or too small */

/* flags (tile, grid and decode entry points) */
/* The running pair is taken to be empty: lse and A are not read, every query
 * row of the call is written, rows without a visible key get lse = -inf and
 * A = 0.  Saves the fill of lse (wrappers/python/nntile/layer/sdpa.py:538-539)
 * and one read of A when the caller knows this is the first key tile. */
#define NNTILE_HIP_SDPA_OVERWRITE 1
/* Tile and grid calls, for tests and tuning: fix the workgroup shape instead
 * of letting the size of the launch pick it.  fp32: 128 queries sharing every
 * key step (SHARED), or 32 queries whose four wavefronts split the key steps
 * (SPLIT).  16-bit: 128 queries and four wavefronts (SHARED), or the same 128
 * queries held by two groups of four wavefronts that take every second key
 * step each and merge through LDS (SPLIT; head 64 and 128; what a launch of
 * at most one workgroup per CU takes by itself).  Both set: ignored. */
#define NNTILE_HIP_SDPA_FORM_SHARED 0x100
#define NNTILE_HIP_SDPA_FORM_SPLIT  0x200
/* 16-bit tile and grid calls with an analytic mask, head 64 or 128, for tests
 * and tuning: workgroups of 256 queries (eight wavefronts, one workgroup per
 * CU) instead of 128 (four, two per CU).  Without it a launch picks the form
 * from its size (256 queries at head 128 when every CU gets two workgroups);
 * NNTILE_HIP_SDPA_FORM_SHARED keeps such a call at 128 queries. */
#define NNTILE_HIP_SDPA_FORM_WIDE   0x4000
/* decode calls, for tests and tuning: merge the key splits in a second launch
 * instead of inside the main one (SEPARATE_MERGE); exchange the partials of
 * the in-launch merge through device-scope fences whatever XCD the
 * workgroups run on (FENCED). */
#define NNTILE_HIP_SDPA_DECODE_SEPARATE_MERGE 0x400
#define NNTILE_HIP_SDPA_DECODE_FENCED         0x800

/* How visibility of key k to query q is given. */
enum nntile_hip_mask_mode
{
    /* mask points at T values [k_seq, q_seq] that are ADDED to the scaled
     * score: 0 = visible, -inf = hidden.  This is what the reference's flash
     * codelet receives (src/kernel/flash_sdpa_fwd_cudnn/cuda.cc:103-109). */
    NNTILE_HIP_MASK_ADDITIVE = 0,
    /* no mask: every key is visible */
    NNTILE_HIP_MASK_NONE = 1,
    /* analytic: key at position k_pos0+k is visible to the query at position
     * q_pos0+q iff k_pos0+k <= q_pos0+q+causal_offset.  No mask memory is
     * read and key blocks that are hidden from a whole query block are
     * skipped. */
    NNTILE_HIP_MASK_CAUSAL = 2,
    /* mask points at bytes [k_seq, q_seq]: non-zero = visible.  This is the
     * reference's vanilla-path mask (src/kernel/mask_scalar/cpu.cc:21-49). */
    NNTILE_HIP_MASK_BOOL = 3
};

/* ---- 1. drop-in for the reference kernel call -----------------------------
 * Replaces kernel::flash_sdpa_fwd_cudnn::execute_graph<T>
 * (include/nntile/kernel/flash_sdpa_fwd_cudnn/cuda.hh:61-76,
 *  src/kernel/flash_sdpa_fwd_cudnn/cuda.cc:145-202): same argument order and
 * meaning, the cuDNN handle/graph pair replaced by the stream.  One square
 * tile: seq queries against seq keys, additive mask [seq, seq] in T.
 * The merge is fused into the kernel, so neither scratch tile is needed for
 * it and both may be null.  scratch_A is never touched.  scratch_lse (seq *
 * batch floats, as the reference registers it) may be overwritten: when the
 * mask is 1 MiB or larger the 16-bit variants scan it once per call - by the
 * first workgroups of the attention launch, or, on a stream that is being
 * captured, by a small launch of their own - and keep what they found (24
 * bytes per 128 queries and key range) there, instead of letting the
 * workgroups of every batch entry scan the same rows.  Same result, bit for
 * bit.
 *
 * SIZE OF scratch_lse: the call has no argument for it and takes it to be
 * what the reference registers, seq * batch floats.  Pass NULL or a buffer of
 * at least seq * batch * 4 bytes - never a smaller dummy: the device would
 * write past its end.  (The codelet bodies of section 6 know the size of
 * their scratch buffer from its interface and leave a smaller one alone; a
 * pointer that is not 8-byte aligned is left alone as well.  The fp32
 * variant never touches it.) */
int nntile_hip_flash_sdpa_fwd_bf16(void *stream, int64_t seq, int64_t head,
        int64_t batch, const uint16_t *K, const uint16_t *Q,
        const uint16_t *mask, float *scratch_lse, const uint16_t *V,
        uint16_t *scratch_A, float *lse, uint16_t *A);
int nntile_hip_flash_sdpa_fwd_fp16(void *stream, int64_t seq, int64_t head,
        int64_t batch, const uint16_t *K, const uint16_t *Q,
        const uint16_t *mask, float *scratch_lse, const uint16_t *V,
        uint16_t *scratch_A, float *lse, uint16_t *A);
/* fp32 has no counterpart in the reference's flash pack
 * (include/nntile/starpu/flash_sdpa_fwd_cudnn.hh:149-153 lists bf16, fp16);
 * it is added so that fp32 models take the same path. */
int nntile_hip_flash_sdpa_fwd_fp32(void *stream, int64_t seq, int64_t head,
        int64_t batch, const float *K, const float *Q, const float *mask,
        float *scratch_lse, const float *V, float *scratch_A, float *lse,
        float *A);

/* ---- 2. one (query tile, key tile) pair, general form ----------------------
 * What tile::flash_sdpa_fwd_cudnn_async (src/tile/flash_sdpa_fwd_cudnn.cc:
 * 161-196) would submit if tiles need not be square and the mask need not be
 * materialised.  Query batch entry b reads key/value entry
 *   (b % n_batch) + n_batch * (b / (n_batch*kv_group)),
 * i.e. Q is [head, q_seq, n_batch, kv_group, n_head_kv] and K/V are
 * [head, k_seq, n_batch, n_head_kv] without the per-group repeat of
 * wrappers/python/nntile/model/llama_attention.py:579-580; kv_group = 1 and
 * n_batch = batch give the plain one-to-one case. */
typedef struct nntile_hip_sdpa_tile_args
{
    int64_t q_seq, k_seq, head;
    int64_t batch;        /* flattened query batch */
    int64_t n_batch;      /* size of the innermost batch axis shared by Q and K/V */
    int64_t kv_group;     /* query heads per key/value head */
    int32_t mask_mode;    /* enum nntile_hip_mask_mode */
    int32_t flags;        /* 0 or NNTILE_HIP_SDPA_OVERWRITE */
    int64_t q_pos0, k_pos0, causal_offset;   /* NNTILE_HIP_MASK_CAUSAL only */
    const void *K, *Q, *mask, *V;
    float *lse;
    void *A;
} nntile_hip_sdpa_tile_args;

int nntile_hip_sdpa_fwd_tile_bf16(void *stream, const nntile_hip_sdpa_tile_args *args);
int nntile_hip_sdpa_fwd_tile_fp16(void *stream, const nntile_hip_sdpa_tile_args *args);
int nntile_hip_sdpa_fwd_tile_fp32(void *stream, const nntile_hip_sdpa_tile_args *args);

/* ---- 2b. backward of one (query tile, key tile) pair ------------------------
 * Replaces kernel::flash_sdpa_bwd_cudnn::execute_graph<T>
 * (include/nntile/kernel/flash_sdpa_bwd_cudnn/cuda.hh:44-68,
 *  src/kernel/flash_sdpa_bwd_cudnn/cuda.cc:171-218): the reference's argument
 * order and meaning MINUS ITS LAST ARGUMENT - the cuDNN handle/graph pair is
 * replaced by the stream, and the trailing `void *workspace` (cuDNN's own
 * scratch, cuda.hh:58) has no counterpart and is dropped: seq, head, batch
 * and the 13 tile pointers are the reference's, in its order.  The forward output A and the logsumexp are inputs; the
 * gradients of this tile pair are ADDED to dK, dQ, dV (the reference computes
 * them into the scratch tiles and adds those, cuda.cc:213-217).  scratch_dK
 * and scratch_dV are accepted for signature compatibility and never touched;
 * scratch_dQ is the call's workspace (it must not be null): its first
 * seq*batch floats hold the row dots dA.A, the bytes behind them one class
 * per 64 x 64 block of the mask.  The reference's pack is
 * {bf16, fp16} (include/nntile/starpu/flash_sdpa_bwd_cudnn.hh). */
int nntile_hip_flash_sdpa_bwd_bf16(void *stream, int64_t seq, int64_t head,
        int64_t batch, const uint16_t *K, const uint16_t *Q, const uint16_t *V,
        const uint16_t *A, const uint16_t *dA, const uint16_t *mask,
        const float *lse, uint16_t *scratch_dK, uint16_t *scratch_dQ,
        uint16_t *scratch_dV, uint16_t *dK, uint16_t *dQ, uint16_t *dV);
int nntile_hip_flash_sdpa_bwd_fp16(void *stream, int64_t seq, int64_t head,
        int64_t batch, const uint16_t *K, const uint16_t *Q, const uint16_t *V,
        const uint16_t *A, const uint16_t *dA, const uint16_t *mask,
        const float *lse, uint16_t *scratch_dK, uint16_t *scratch_dQ,
        uint16_t *scratch_dV, uint16_t *dK, uint16_t *dQ, uint16_t *dV);

/* General form, what tile::flash_sdpa_bwd_cudnn_async
 * (src/tile/flash_sdpa_bwd_cudnn.cc) would submit if tiles need not be square
 * and the mask need not be materialised: shapes, batch mapping, mask modes
 * and positions as in nntile_hip_sdpa_tile_args; with kv_group > 1 the
 * gradients of a key/value head sum over its query heads.  flags:
 * NNTILE_HIP_SDPA_OVERWRITE writes the gradients instead of adding to them.
 * workspace: device memory of nntile_hip_sdpa_bwd_workspace_bytes(args)
 * bytes, 4-byte aligned, private to the call until it has completed:
 * q_seq*batch floats (the row dots dA.A), then, for the two modes that pass
 * the mask as values, one byte per 64 x 64 block of the mask (whether the
 * block hides everything, nothing, or some).  A workspace that only holds the
 * floats is accepted: the kernels then read every value of the mask instead
 * of skipping by block.  A mask passed as values may have at most 2^24 keys
 * per row (NNTILE_HIP_EUNSUPPORTED beyond). */
typedef struct nntile_hip_sdpa_bwd_args
{
    int64_t q_seq, k_seq, head;
    int64_t batch, n_batch, kv_group;
    int32_t mask_mode;
    int32_t flags;
    int64_t q_pos0, k_pos0, causal_offset;
    const void *K, *Q, *V, *A, *dA, *mask;
    const float *lse;
    void *dK, *dQ, *dV;
    void *workspace;
    size_t workspace_bytes;
} nntile_hip_sdpa_bwd_args;

size_t nntile_hip_sdpa_bwd_workspace_bytes(const nntile_hip_sdpa_bwd_args *args);
int nntile_hip_sdpa_bwd_tile_bf16(void *stream, const nntile_hip_sdpa_bwd_args *args);
int nntile_hip_sdpa_bwd_tile_fp16(void *stream, const nntile_hip_sdpa_bwd_args *args);

/* ---- 3. a whole grid of tiles in one launch ---------------------------------
 * What tensor::flash_sdpa_fwd_cudnn_async (src/tensor/flash_sdpa_fwd_cudnn.cc:
 * 210-279) computes when every tile of one (batch, head) slab is resident on
 * this GPU: for each query tile, all key tiles are merged in one pass with the
 * output kept in registers, instead of one task (and one round trip of A
 * through T) per tile pair.  Tiles are separate allocations, as in NNTile;
 * all query tiles hold q_tile rows and all key tiles k_tile rows, except the
 * last of each, which holds the remainder of q_seq / k_seq.  Only the
 * analytic masks (NONE, CAUSAL) are accepted; positions count from row 0 of
 * tile 0 plus q_pos0 / k_pos0.
 *
 * n_slabs > 1 puts several such slabs into the one launch - the tiles the
 * tensor-level loop walks along the batch axes, each slab a set of separate
 * allocations with the same extents and `batch` entries: the tables then hold
 * slab s's tiles at [s*n_q_tiles + t] (Q, lse, A) and [s*n_kv_tiles + t] (K,
 * V), and n_slabs*n_q_tiles and n_slabs*n_kv_tiles must not exceed
 * NNTILE_HIP_SDPA_MAX_TILES.  batch, n_batch and kv_group describe one slab.
 * 0 stands for 1.  (A launch picks its workgroup shape from its total size,
 * so the fp32 results of a many-slab launch may differ from per-slab launches
 * in the last bits: the key steps of a row are summed in another order.) */
#define NNTILE_HIP_SDPA_MAX_TILES 64

typedef struct nntile_hip_sdpa_grid_args
{
    int64_t q_seq, k_seq, q_tile, k_tile, head;
    int64_t batch, n_batch, kv_group;
    int32_t mask_mode, n_q_tiles, n_kv_tiles, flags;
    int32_t n_slabs, reserved;
    int64_t q_pos0, k_pos0, causal_offset;
    const void *K[NNTILE_HIP_SDPA_MAX_TILES];
    const void *V[NNTILE_HIP_SDPA_MAX_TILES];
    const void *Q[NNTILE_HIP_SDPA_MAX_TILES];
    float *lse[NNTILE_HIP_SDPA_MAX_TILES];
    void *A[NNTILE_HIP_SDPA_MAX_TILES];
} nntile_hip_sdpa_grid_args;

int nntile_hip_sdpa_fwd_grid_bf16(void *stream, const nntile_hip_sdpa_grid_args *args);
int nntile_hip_sdpa_fwd_grid_fp16(void *stream, const nntile_hip_sdpa_grid_args *args);
int nntile_hip_sdpa_fwd_grid_fp32(void *stream, const nntile_hip_sdpa_grid_args *args);

/* The backward over the same grid of tiles in one call: what
 * tensor::flash_sdpa_bwd_cudnn_async (src/tensor/flash_sdpa_bwd_cudnn.cc:
 * 172-247) computes by submitting one task per (dQ tile, key tile) pair, for
 * one (batch, head) slab whose tiles are all resident on this GPU.  dQ of a
 * query tile sums over every key tile, dK and dV of a key tile over every
 * query tile (and, with kv_group > 1, over the query heads of the group); the
 * sums are carried in fp32 and rounded once, where the pair-by-pair form
 * rounds after every pair.  Tiles are separate allocations laid out as in
 * nntile_hip_sdpa_grid_args; A, dA, dQ and lse follow the query tiles, dK and
 * dV the key tiles.  q_tile and k_tile must be multiples of 128 (the rows a
 * workgroup owns) unless the axis has a single tile; other sizes get
 * NNTILE_HIP_EUNSUPPORTED and are served pair by pair through
 * nntile_hip_sdpa_bwd_tile_*.  Only the analytic masks (NONE, CAUSAL).
 * flags: NNTILE_HIP_SDPA_OVERWRITE writes the gradients instead of adding to
 * them.  n_slabs > 1 (0 stands for 1) puts several slabs of the batch grid,
 * each `batch` entries in tiles of its own with the same extents, into the
 * one call, slab s's tiles at [s*n_q_tiles + t] / [s*n_kv_tiles + t] of the
 * tables as in nntile_hip_sdpa_grid_args; n_slabs*n_q_tiles and
 * n_slabs*n_kv_tiles must not exceed NNTILE_HIP_SDPA_BWD_MAX_TILES.
 * workspace: n_slabs*q_seq*batch floats of device memory
 * (nntile_hip_sdpa_bwd_grid_workspace_bytes), 4-byte aligned, private to the
 * call until it has completed. */
#define NNTILE_HIP_SDPA_BWD_MAX_TILES 32

typedef struct nntile_hip_sdpa_bwd_grid_args
{
    int64_t q_seq, k_seq, q_tile, k_tile, head;
    int64_t batch, n_batch, kv_group;
    int32_t mask_mode, n_q_tiles, n_kv_tiles, flags;
    int32_t n_slabs, reserved;
    int64_t q_pos0, k_pos0, causal_offset;
    const void *K[NNTILE_HIP_SDPA_BWD_MAX_TILES];
    const void *V[NNTILE_HIP_SDPA_BWD_MAX_TILES];
    const void *Q[NNTILE_HIP_SDPA_BWD_MAX_TILES];
    const void *A[NNTILE_HIP_SDPA_BWD_MAX_TILES];
    const void *dA[NNTILE_HIP_SDPA_BWD_MAX_TILES];
    const float *lse[NNTILE_HIP_SDPA_BWD_MAX_TILES];
    void *dK[NNTILE_HIP_SDPA_BWD_MAX_TILES];
    void *dQ[NNTILE_HIP_SDPA_BWD_MAX_TILES];
    void *dV[NNTILE_HIP_SDPA_BWD_MAX_TILES];
    void *workspace;
    size_t workspace_bytes;
} nntile_hip_sdpa_bwd_grid_args;

size_t nntile_hip_sdpa_bwd_grid_workspace_bytes(const nntile_hip_sdpa_bwd_grid_args *args);
int nntile_hip_sdpa_bwd_grid_bf16(void *stream, const nntile_hip_sdpa_bwd_grid_args *args);
int nntile_hip_sdpa_bwd_grid_fp16(void *stream, const nntile_hip_sdpa_bwd_grid_args *args);

/* ---- 4. short-query / long-key decode ----------------------------------------
 * The shape of LlamaAttention.forward_dynamic
 * (wrappers/python/nntile/model/llama_attention.py:627-760), which in the
 * reference repeats K/V per group and runs the vanilla composition.  Here the
 * kv_group query heads of one key/value head share one pass over the cache,
 * and the key axis is split over workgroups; partial results are merged with
 * the accumulate_attn_output rule.  args->q_seq*kv_group must be <= 64.
 * workspace: device memory of at least
 * nntile_hip_sdpa_fwd_decode_workspace_bytes(args) bytes, private to the call
 * until the stream has passed it (a STARPU_SCRATCH buffer in NNTile terms). */
size_t nntile_hip_sdpa_fwd_decode_workspace_bytes(const nntile_hip_sdpa_tile_args *args);
int nntile_hip_sdpa_fwd_decode_bf16(void *stream, const nntile_hip_sdpa_tile_args *args,
        void *workspace, size_t workspace_bytes);
int nntile_hip_sdpa_fwd_decode_fp16(void *stream, const nntile_hip_sdpa_tile_args *args,
        void *workspace, size_t workspace_bytes);
/* fp32 tiles (the reference runs forward_dynamic in fp32 as well,
 * wrappers/python/tests/model/test_llama_attention.py:296-345): the same
 * sharing of K/V among the query heads of a group and the same split of the
 * keys, with v_mfma_f32_16x16x4_f32; the partials are fp32, so the workspace
 * has a size function of its own, and the merge is always a second launch. */
size_t nntile_hip_sdpa_fwd_decode_workspace_bytes_fp32(const nntile_hip_sdpa_tile_args *args);
int nntile_hip_sdpa_fwd_decode_fp32(void *stream, const nntile_hip_sdpa_tile_args *args,
        void *workspace, size_t workspace_bytes);

/* ---- 4b. decode for callers that cannot allocate -------------------------------
 * No counterpart in the reference.  For callers that cannot call hipMalloc
 * and have no scratch buffer to pass: work under HIP graph capture, tight
 * serving loops, harnesses that forbid allocation.  Same computation and
 * result as nntile_hip_sdpa_fwd_decode_{bf16,fp16} (dtype picks the tile
 * type), with the split partials in a device array that is part of the
 * library's code object: NNTILE_HIP_DECODE_STATIC_SCRATCH_BYTES per GPU,
 * held from the library's load until the process ends.  The call allocates
 * and frees nothing.  A shape whose partials need more
 * (nntile_hip_sdpa_fwd_decode_workspace_bytes(args) tells) is refused with
 * NNTILE_HIP_EWORKSPACE and a line on stderr.  The array's address on the
 * current device is looked up on the first call made with that device current
 * (make that call outside a capture); the stream must belong to the current
 * device - a stream of another GPU is refused with NNTILE_HIP_EINVAL.  All calls on one GPU share the array: two of them in flight at the
 * same time (different streams) race, calls on one stream do not. */
#define NNTILE_HIP_DECODE_STATIC_SCRATCH_BYTES (16u << 20)
#define NNTILE_HIP_DTYPE_BF16 0
#define NNTILE_HIP_DTYPE_FP16 1
int nntile_hip_sdpa_fwd_decode_static(void *stream, int32_t dtype,
        const nntile_hip_sdpa_tile_args *args);

/* ---- 4c. diagnostics of the decode entry points ------------------------------
 * No counterpart in the reference.  When a (batch entry, kv head) unit has
 * several key splits and the units come in multiples of 8, the merge of the
 * splits runs inside the main launch: merge workgroups behind the main ones
 * wait for flags in the workspace.  That wait is bounded (2 s of the 100 MHz
 * device clock unless set otherwise here; returns the previous bound); a merge
 * workgroup that gives up leaves its rows untouched and is counted.  The
 * count since the library was loaded (blocking; -1 on error): */
unsigned long long nntile_hip_debug_decode_spin_limit(unsigned long long ticks);
long long nntile_hip_debug_decode_sync_timeouts(void);
/* The partials reach the merge workgroups through the L2 of the XCD that the
 * unit's main workgroups ran on: a launch's workgroups go round the XCDs in
 * index order, and a unit's main and merge workgroups have equal indices
 * modulo 8.  Every flag carries the number of the XCD that raised it; a merge
 * workgroup that finds a split of its unit raised elsewhere than on its own
 * XCD leaves its rows untouched and is counted here (never observed, also not
 * with several queues dispatching at once; blocking; -1 on error): */
long long nntile_hip_debug_decode_sync_misplaced(void);

/* ---- 5. the running-statistics hand-off on its own ---------------------------
 * Replaces kernel::accumulate_attn_output::cuda<T>
 * (src/kernel/accumulate_attn_output/cuda.cu:115-135; CPU statement
 * src/kernel/accumulate_attn_output/cpu.cc:38-115): merges (src_lse, src_attn)
 * into (dst_lse, dst_attn) for seq*batch rows of head values. */
int nntile_hip_accumulate_attn_output_bf16(void *stream, int64_t head, int64_t seq,
        int64_t batch, const float *src_lse, const uint16_t *src_attn,
        float *dst_lse, uint16_t *dst_attn);
int nntile_hip_accumulate_attn_output_fp16(void *stream, int64_t head, int64_t seq,
        int64_t batch, const float *src_lse, const uint16_t *src_attn,
        float *dst_lse, uint16_t *dst_attn);
int nntile_hip_accumulate_attn_output_fp32(void *stream, int64_t head, int64_t seq,
        int64_t batch, const float *src_lse, const float *src_attn,
        float *dst_lse, float *dst_attn);

/* ---- 6. StarPU codelet bodies ---------------------------------------------------
 * Same shape as FlashSdpaFwdCudnn<T>::cuda(void *buffers[], void *cl_args)
 * (src/starpu/flash_sdpa_fwd_cudnn.cc:60-155), to be placed in the codelet's
 * hip_funcs[0] with STARPU_HIP_ASYNC.  buffers[i] point at StarPU variable
 * interfaces in the reference's order: K(R) Q(R) mask(R) lse(RW) V(R) A(RW)
 * scratch_lse(SCRATCH) scratch_A(SCRATCH); cl_args points at
 * nntile_hip_flash_sdpa_cl_args, whose first four members are the
 * reference's args_t (include/nntile/starpu/flash_sdpa_fwd_cudnn.hh:58-64).
 * Errors are reported on stderr and the task becomes a no-op, as in the
 * reference.  The stream comes from the function registered with
 * nntile_hip_set_stream_provider (starpu_hip_get_local_stream in a StarPU
 * build); without a provider the null stream is used. */
typedef struct nntile_hip_variable_interface
{
    int id;              /* enum starpu_data_interface_id */
    uintptr_t ptr;       /* device pointer of the tile */
    uintptr_t dev_handle;
    size_t offset;
    size_t elemsize;
} nntile_hip_variable_interface;

typedef struct nntile_hip_flash_sdpa_cl_args
{
    void *owner;
    int64_t seq, head, batch;
} nntile_hip_flash_sdpa_cl_args;

typedef void *(*nntile_hip_stream_provider)(void);
void nntile_hip_set_stream_provider(nntile_hip_stream_provider fn);

void nntile_hip_flash_sdpa_fwd_codelet_bf16(void *buffers[], void *cl_args);
void nntile_hip_flash_sdpa_fwd_codelet_fp16(void *buffers[], void *cl_args);
void nntile_hip_flash_sdpa_fwd_codelet_fp32(void *buffers[], void *cl_args);
/* Backward twin: the body of starpu::FlashSdpaBwdCudnn<T>::cuda
 * (src/starpu/flash_sdpa_bwd_cudnn.cc:51-157), 13 buffers in the reference's
 * order K Q V A dA mask logsumexp dK dQ dV scratch_dK scratch_dQ scratch_dV
 * (:103-115) and the same args_t prefix {owner, seq, head, batch}
 * (include/nntile/starpu/flash_sdpa_bwd_cudnn.hh:48-57). */
void nntile_hip_flash_sdpa_bwd_codelet_bf16(void *buffers[], void *cl_args);
void nntile_hip_flash_sdpa_bwd_codelet_fp16(void *buffers[], void *cl_args);

/* ---- 6b. StarPU codelet bodies of the whole-grid calls ---------------------------
 * The fused launches as tasks: what tensor::flash_sdpa_fwd_cudnn_async
 * (src/tensor/flash_sdpa_fwd_cudnn.cc:246-274) submits as one task per (output
 * tile, key tile) pair becomes ONE task per group of slabs, submitted like the
 * reference's (src/starpu/flash_sdpa_fwd_cudnn.cc:181-210: starpu_task_insert
 * on a codelet with nbuffers = STARPU_VARIABLE_NBUFFERS, src/starpu/codelet.cc:
 * 58, so the number of handles is free).  buffers[] point at StarPU variable
 * interfaces, tile after tile, in this order and with these access modes
 * (nK = n_slabs*n_kv_tiles, nQ = n_slabs*n_q_tiles, slab s's tiles at
 * [s*n_kv_tiles + t] / [s*n_q_tiles + t] as in nntile_hip_sdpa_grid_args):
 *   forward : K[nK](R) V[nK](R) Q[nQ](R) lse[nQ](RW) A[nQ](RW)
 *             (with NNTILE_HIP_SDPA_OVERWRITE in flags lse and A may be W)
 *   backward: K[nK](R) V[nK](R) Q[nQ](R) A[nQ](R) dA[nQ](R) lse[nQ](R)
 *             dK[nK](RW) dQ[nQ](RW) dV[nK](RW) workspace(SCRATCH, at least
 *             nntile_hip_sdpa_bwd_grid_workspace_bytes)
 * cl_args points at nntile_hip_sdpa_grid_cl_args: the reference's args_t
 * members first (seq = rows of a full query tile, head, batch = entries of one
 * slab), then the geometry of nntile_hip_sdpa_grid_args.  Same error
 * behaviour as the per-pair bodies: a line on stderr, the task does nothing. */
typedef struct nntile_hip_sdpa_grid_cl_args
{
    void *owner;
    int64_t seq, head, batch;           /* args_t of the reference */
    int64_t q_seq, k_seq, q_tile, k_tile;
    int64_t n_batch, kv_group;
    int64_t q_pos0, k_pos0, causal_offset;
    int32_t mask_mode, flags;
    int32_t n_q_tiles, n_kv_tiles, n_slabs, reserved;
} nntile_hip_sdpa_grid_cl_args;

void nntile_hip_sdpa_fwd_grid_codelet_bf16(void *buffers[], void *cl_args);
void nntile_hip_sdpa_fwd_grid_codelet_fp16(void *buffers[], void *cl_args);
void nntile_hip_sdpa_fwd_grid_codelet_fp32(void *buffers[], void *cl_args);
void nntile_hip_sdpa_bwd_grid_codelet_bf16(void *buffers[], void *cl_args);
void nntile_hip_sdpa_bwd_grid_codelet_fp16(void *buffers[], void *cl_args);

/* ---- 7. The step before the attention kernel: rotary position embedding ----
 * Replace kernel::rope::cuda<T> (include/nntile/kernel/rope/cuda.hh:24-27,
 * src/kernel/rope/cuda.cu:22-55) and kernel::rope_backward::cuda<T>
 * (include/nntile/kernel/rope_backward/cuda.hh:24-27,
 * src/kernel/rope_backward/cuda.cu): same argument order and meaning.  src
 * and dst are (2, m, n) in memory order, sin and cos hold m values each:
 *   dst[2i,j]   = cos[i] src[2i,j] - sin[i] src[2i+1,j]
 *   dst[2i+1,j] = sin[i] src[2i,j] + cos[i] src[2i+1,j]
 * and the backward is the transposed rotation, written (not added) to dx.
 * Arithmetic in fp32, one rounding to the tile type.  m == 0 or n == 0 is a
 * no-op; src and dst may be the same buffer. */
int nntile_hip_rope_bf16(void *stream, int64_t m, int64_t n, const uint16_t *sin,
        const uint16_t *cos, const uint16_t *src, uint16_t *dst);
int nntile_hip_rope_fp16(void *stream, int64_t m, int64_t n, const uint16_t *sin,
        const uint16_t *cos, const uint16_t *src, uint16_t *dst);
int nntile_hip_rope_fp32(void *stream, int64_t m, int64_t n, const float *sin,
        const float *cos, const float *src, float *dst);
int nntile_hip_rope_backward_bf16(void *stream, int64_t m, int64_t n, const uint16_t *sin,
        const uint16_t *cos, const uint16_t *dy, uint16_t *dx);
int nntile_hip_rope_backward_fp16(void *stream, int64_t m, int64_t n, const uint16_t *sin,
        const uint16_t *cos, const uint16_t *dy, uint16_t *dx);
int nntile_hip_rope_backward_fp32(void *stream, int64_t m, int64_t n, const float *sin,
        const float *cos, const float *dy, float *dx);

/* ---- 8. The transposes either side of the attention block -------------------
 * Replace kernel::transpose::cuda<T> (include/nntile/kernel/transpose/cuda.hh:25,
 * arithmetic src/kernel/transpose/cpu.cc:21-43): dst = alpha * src^T for an
 * m x n matrix in Fortran order (src(i,j) at i + j*m, dst(j,i) at j + i*n).
 * The reference's Scalar alpha is a float.  src and dst must not overlap. */
int nntile_hip_transpose_bf16(void *stream, int64_t m, int64_t n, float alpha,
        const uint16_t *src, uint16_t *dst);
int nntile_hip_transpose_fp16(void *stream, int64_t m, int64_t n, float alpha,
        const uint16_t *src, uint16_t *dst);
int nntile_hip_transpose_fp32(void *stream, int64_t m, int64_t n, float alpha,
        const float *src, float *dst);

/* ---- 9. key/value cache of the decode path -----------------------------------
 * Replaces KVCache.append (wrappers/python/nntile/layer/cache_utils.py:
 * 146-175: two copy_intersection_async calls into tensors preallocated with
 * max_cache_size rows on the sequence axis) for caches of shape
 * [head, capacity, n_batch, n_head_kv]: the rows of k_new and v_new
 * ([head, rows, n_batch, n_head_kv], entries = n_batch*n_head_kv) are written
 * behind the `filled` rows that each entry of k_cache / v_cache already
 * holds, both tensors in one launch.  rows > capacity - filled is
 * NNTILE_HIP_EINVAL, the condition on which LlamaAttention._append_to_kv_cache
 * raises (wrappers/python/nntile/model/llama_attention.py:524-529); nothing
 * is written then.  rows == 0 is a no-op. */
int nntile_hip_kv_cache_append_bf16(void *stream, int64_t head, int64_t rows, int64_t entries,
        int64_t capacity, int64_t filled, const uint16_t *k_new, const uint16_t *v_new,
        uint16_t *k_cache, uint16_t *v_cache);
int nntile_hip_kv_cache_append_fp16(void *stream, int64_t head, int64_t rows, int64_t entries,
        int64_t capacity, int64_t filled, const uint16_t *k_new, const uint16_t *v_new,
        uint16_t *k_cache, uint16_t *v_cache);
int nntile_hip_kv_cache_append_fp32(void *stream, int64_t head, int64_t rows, int64_t entries,
        int64_t capacity, int64_t filled, const float *k_new, const float *v_new,
        float *k_cache, float *v_cache);

/* nntile_hip_sdpa_fwd_decode_* reading such a cache where it lies: args->K and
 * args->V point at the caches, args->k_seq is the number of filled rows and
 * `capacity` (>= k_seq) the rows between two entries.  This stands for the
 * k_partial / v_partial copies of the filled part that the reference makes
 * before every attention call (cache_utils.py:177-215) and, with
 * NNTILE_HIP_MASK_CAUSAL and causal_offset = k_seq - q_seq, for the bool mask
 * that Sdpa._prepare_mask_for_kv_cache materialises
 * (wrappers/python/nntile/layer/sdpa.py:489-531).  Workspace as for
 * nntile_hip_sdpa_fwd_decode_* (its size does not depend on capacity). */
int nntile_hip_sdpa_fwd_decode_cache_bf16(void *stream, const nntile_hip_sdpa_tile_args *args,
        int64_t capacity, void *workspace, size_t workspace_bytes);
int nntile_hip_sdpa_fwd_decode_cache_fp16(void *stream, const nntile_hip_sdpa_tile_args *args,
        int64_t capacity, void *workspace, size_t workspace_bytes);
int nntile_hip_sdpa_fwd_decode_cache_fp32(void *stream, const nntile_hip_sdpa_tile_args *args,
        int64_t capacity, void *workspace, size_t workspace_bytes);
/* The append and the attention of a decode step in ONE launch (no counterpart
 * in the reference, where they are the copy_intersection calls of
 * cache_utils.py:146-175 followed by the attention): k_new, v_new
 * [head, rows_new, n_batch, n_head_kv] are the keys and values of the newest
 * rows_new tokens, args->k_seq counts the rows of the caches INCLUDING them,
 * i.e. they belong at rows [k_seq - rows_new, k_seq) of every entry.  The
 * attention reads those rows from k_new / v_new and the rest from the caches;
 * workgroups at the end of the launch copy the new rows into the caches, so
 * after the call the caches are what nntile_hip_kv_cache_append_* would have
 * made them, and (lse, A) what nntile_hip_sdpa_fwd_decode_cache_* would then
 * have computed, bit for bit.  NNTILE_HIP_EINVAL when rows_new exceeds k_seq
 * or the capacity is smaller than k_seq.  The fp32 form is the fp32 decode
 * kernel with the same two additions. */
int nntile_hip_sdpa_fwd_decode_append_cache_bf16(void *stream,
        const nntile_hip_sdpa_tile_args *args, int64_t capacity, const uint16_t *k_new,
        const uint16_t *v_new, int64_t rows_new, void *workspace, size_t workspace_bytes);
int nntile_hip_sdpa_fwd_decode_append_cache_fp16(void *stream,
        const nntile_hip_sdpa_tile_args *args, int64_t capacity, const uint16_t *k_new,
        const uint16_t *v_new, int64_t rows_new, void *workspace, size_t workspace_bytes);
int nntile_hip_sdpa_fwd_decode_append_cache_fp32(void *stream,
        const nntile_hip_sdpa_tile_args *args, int64_t capacity, const float *k_new,
        const float *v_new, int64_t rows_new, void *workspace, size_t workspace_bytes);

/* nntile_hip_sdpa_fwd_tile_* reading the cache the same way, for what the
 * decode form does not take: fp32 caches (the reference runs forward_dynamic
 * in fp32 too, wrappers/python/tests/model/test_llama_attention.py:296-345),
 * head 32, and chunks of more than 64 / kv_group new tokens.  No workspace. */
int nntile_hip_sdpa_fwd_tile_cache_bf16(void *stream, const nntile_hip_sdpa_tile_args *args,
        int64_t capacity);
int nntile_hip_sdpa_fwd_tile_cache_fp16(void *stream, const nntile_hip_sdpa_tile_args *args,
        int64_t capacity);
int nntile_hip_sdpa_fwd_tile_cache_fp32(void *stream, const nntile_hip_sdpa_tile_args *args,
        int64_t capacity);

/* ---- 10. class of a mask tile -------------------------------------------------
 * For the layer that submits one task per (query tile, key tile) pair with
 * the pair's mask tile (src/tensor/flash_sdpa_fwd_cudnn.cc:246-274, which
 * submits every pair): reads one tile of a materialised mask - [k_rows,
 * q_cols] in Fortran order, additive in the tile type (0 visible, -inf
 * hidden) or bool (nonzero visible) - and tells whether the pair needs a task
 * and whether that task needs the mask:
 *   HIDDEN  every element hidden: the pair leaves (lse, A) as they are
 *   OPEN    every element visible: NNTILE_HIP_MASK_NONE gives the same result
 *   CAUSAL  visible exactly where k <= q + offset (k, q counted inside the
 *           tile): NNTILE_HIP_MASK_CAUSAL with causal_offset = offset does
 *   MIXED   anything else, additive values other than 0 and -inf included:
 *           the mask must be passed
 * Blocking: synchronises the stream and writes *class_out on the host.  A
 * mask is classified once and the classes kept with it; workspace is one
 * 4-byte aligned device word, private to the call. */
#define NNTILE_HIP_MASK_TILE_MIXED 0
#define NNTILE_HIP_MASK_TILE_OPEN 1
#define NNTILE_HIP_MASK_TILE_HIDDEN 2
#define NNTILE_HIP_MASK_TILE_CAUSAL 3
int nntile_hip_mask_tile_class_bf16(void *stream, int64_t k_rows, int64_t q_cols,
        const uint16_t *mask, int64_t offset, int32_t *workspace, int32_t *class_out);
int nntile_hip_mask_tile_class_fp16(void *stream, int64_t k_rows, int64_t q_cols,
        const uint16_t *mask, int64_t offset, int32_t *workspace, int32_t *class_out);
int nntile_hip_mask_tile_class_fp32(void *stream, int64_t k_rows, int64_t q_cols,
        const float *mask, int64_t offset, int32_t *workspace, int32_t *class_out);
int nntile_hip_mask_tile_class_bool(void *stream, int64_t k_rows, int64_t q_cols,
        const uint8_t *mask, int64_t offset, int32_t *workspace, int32_t *class_out);

/* Library version and the ISA it was built for ("gfx950"). */
const char *nntile_hip_sdpa_version(void);

#ifdef __cplusplus
}
#endif

#endif /* NNTILE_HIP_SDPA_H */
