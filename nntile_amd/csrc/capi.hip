// C ABI of libnntile_hip_sdpa.so: argument checks and dispatch to the kernels.
#include <atomic>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "sdpa_common.hpp"

namespace nntile_hip
{

template<typename T>
int launch_prefill_16bit(hipStream_t stream, PrefillParams &p, int head, int mode,
        void *scan_scratch, size_t scan_scratch_bytes);
int launch_prefill_fp32(hipStream_t stream, PrefillParams &p, int head, int mode);

template<typename T>
int launch_decode_16bit(hipStream_t stream, DecodeParams &p, int head, int mode);
int decode_choose_splits(int units, int n_steps);
template<typename T>
int launch_bwd_16bit(hipStream_t stream, const BwdParams &p, int head, int mode);
template<typename T>
int launch_bwd_grid_16bit(hipStream_t stream, const BwdGridParams &p,
        const void *const *A_tiles, int n_q_tiles, int head, int mode);
size_t decode_workspace_bytes(int units, int n_splits, int rows, int head);
size_t decode_partial_o_bytes(int units, int n_splits, int rows, int head);
size_t decode_partial_ml_bytes(int units, int n_splits, int rows);
int launch_decode_fp32(hipStream_t stream, const DecodeParams &p, int head, int mode);
int decode_fp32_steps(int64_t k_seq);
int decode_fp32_choose_splits(int units, int n_steps);
size_t decode_fp32_workspace_bytes(int units, int n_splits, int rows, int head);

struct F32Store;
struct Bf16Store;
struct Fp16Store;
template<typename S>
int launch_accumulate(hipStream_t stream, int64_t head, int64_t seq,
        int64_t batch, const float *src_lse, const void *src_attn,
        float *dst_lse, void *dst_attn);

int launch_rope(hipStream_t stream, int dtype, bool backward, int64_t m, int64_t n,
        const void *sin, const void *cos, const void *src, void *dst);

int launch_transpose(hipStream_t stream, int dtype, int64_t m, int64_t n, float alpha,
        const void *src, void *dst);

int launch_kv_cache_append(hipStream_t stream, int elem, int64_t head, int64_t rows,
        int64_t entries, int64_t capacity, int64_t filled, const void *k_new,
        const void *v_new, void *k_cache, void *v_cache);

int launch_mask_classify(hipStream_t stream, int dtype, int64_t k_rows, int64_t q_cols,
        int64_t offset, const void *mask, uint32_t *flags);

enum class DType { bf16, fp16, fp32 };

static bool aligned16(const void *p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

static bool mode_ok(int mode)
{
    return mode >= NNTILE_HIP_MASK_ADDITIVE && mode <= NNTILE_HIP_MASK_BOOL;
}

// the workgroup shape a caller asked for: 0 none, 1 shared, 2 split, 8 wide (16-bit kernels)
static int prefill_form(int32_t flags)
{
    const bool shared = (flags & NNTILE_HIP_SDPA_FORM_SHARED) != 0;
    const bool split = (flags & NNTILE_HIP_SDPA_FORM_SPLIT) != 0;
    if(flags & NNTILE_HIP_SDPA_FORM_WIDE)
    {
        return 8;       // 16-bit kernels: 256-query workgroups
    }
    return shared == split ? 0 : (shared ? 1 : 2);
}

static int dispatch_prefill(DType dt, hipStream_t stream, PrefillParams &p,
        int64_t head, int mode, void *scan_scratch = nullptr,
        size_t scan_scratch_bytes = 0)
{
    if(head != 32 && head != 64 && head != 128)
    {
        return NNTILE_HIP_EUNSUPPORTED;
    }
    p.scale = 1.0f / sqrtf(static_cast<float>(head));
    switch(dt)
    {
        case DType::bf16:
            return launch_prefill_16bit<Bf16>(stream, p, (int)head, mode, scan_scratch,
                    scan_scratch_bytes);
        case DType::fp16:
            return launch_prefill_16bit<Fp16>(stream, p, (int)head, mode, scan_scratch,
                    scan_scratch_bytes);
        default:
            return launch_prefill_fp32(stream, p, (int)head, mode);
    }
}

// scan_scratch: device memory the call may overwrite (the reference's
// scratch_logsumexp tile, scan_scratch_bytes of it), or null
static int tile_call(DType dt, void *stream, const nntile_hip_sdpa_tile_args *a,
        int64_t kv_rows = 0, void *scan_scratch = nullptr, size_t scan_scratch_bytes = 0)
{
    if(a == nullptr || a->q_seq <= 0 || a->k_seq <= 0 || a->head <= 0
            || a->batch <= 0 || a->n_batch <= 0 || a->kv_group <= 0
            || !mode_ok(a->mask_mode) || a->K == nullptr || a->Q == nullptr
            || a->V == nullptr || a->lse == nullptr || a->A == nullptr
            || a->batch % (a->n_batch * a->kv_group) != 0
            || a->batch > 0x7fffffff || a->q_seq > 0x7fffffff
            || a->k_seq > 0x7fffffff)
    {
        return NNTILE_HIP_EINVAL;
    }
    const bool explicit_mask = a->mask_mode == NNTILE_HIP_MASK_ADDITIVE
        || a->mask_mode == NNTILE_HIP_MASK_BOOL;
    if(explicit_mask && a->mask == nullptr)
    {
        return NNTILE_HIP_EINVAL;
    }
    if(!aligned16(a->K) || !aligned16(a->Q) || !aligned16(a->V)
            || !aligned16(a->A))
    {
        return NNTILE_HIP_EINVAL;
    }
    PrefillParams p;
    std::memset(&p, 0, sizeof(p));
    p.q_seq = p.q_tile = a->q_seq;
    p.k_seq = p.k_tile = a->k_seq;
    p.q_pos0 = a->q_pos0;
    p.k_pos0 = a->k_pos0;
    p.causal_offset = a->causal_offset;
    p.mask = a->mask;
    p.mask_ld = a->k_seq;
    p.kv_rows = kv_rows;
    p.n_q_tiles = p.n_kv_tiles = 1;
    p.n_slabs = 1;
    p.batch = (int32_t)a->batch;
    p.n_batch = (int32_t)a->n_batch;
    p.kv_group = (int32_t)a->kv_group;
    p.overwrite = (a->flags & NNTILE_HIP_SDPA_OVERWRITE) ? 1 : 0;
    p.form = prefill_form(a->flags);
    p.K[0] = a->K;
    p.V[0] = a->V;
    p.Q[0] = a->Q;
    p.lse[0] = a->lse;
    p.A[0] = a->A;
    return dispatch_prefill(dt, static_cast<hipStream_t>(stream), p, a->head,
            a->mask_mode, scan_scratch, scan_scratch_bytes);
}

static int bwd_call(DType dt, void *stream, const nntile_hip_sdpa_bwd_args *a)
{
    if(a == nullptr || a->q_seq <= 0 || a->k_seq <= 0 || a->head <= 0
            || a->batch <= 0 || a->n_batch <= 0 || a->kv_group <= 0
            || !mode_ok(a->mask_mode) || a->K == nullptr || a->Q == nullptr
            || a->V == nullptr || a->A == nullptr || a->dA == nullptr
            || a->lse == nullptr || a->dK == nullptr || a->dQ == nullptr
            || a->dV == nullptr
            || a->batch % (a->n_batch * a->kv_group) != 0
            || a->batch > 0x7fffffff || a->q_seq > 0x7fffffff
            || a->k_seq > 0x7fffffff)
    {
        return NNTILE_HIP_EINVAL;
    }
    const bool explicit_mask = a->mask_mode == NNTILE_HIP_MASK_ADDITIVE
        || a->mask_mode == NNTILE_HIP_MASK_BOOL;
    if(explicit_mask && a->mask == nullptr)
    {
        return NNTILE_HIP_EINVAL;
    }
    if(!aligned16(a->K) || !aligned16(a->Q) || !aligned16(a->V) || !aligned16(a->A)
            || !aligned16(a->dA) || !aligned16(a->dK) || !aligned16(a->dQ)
            || !aligned16(a->dV))
    {
        return NNTILE_HIP_EINVAL;
    }
    if(a->head != 32 && a->head != 64 && a->head != 128)
    {
        return NNTILE_HIP_EUNSUPPORTED;
    }
    // the kernels address 128 rows of a mask given as values with 32 bits
    if(explicit_mask && a->k_seq > (1 << 24))
    {
        return NNTILE_HIP_EUNSUPPORTED;
    }
    // workspace: q_seq*batch floats (the row dots), then, if there is room
    // and the mask is given as values, one byte per 64 x 64 block of the mask
    const size_t d_bytes = (size_t)a->q_seq * (size_t)a->batch * sizeof(float);
    if(a->workspace == nullptr || a->workspace_bytes < d_bytes
            || (reinterpret_cast<uintptr_t>(a->workspace) & 3u) != 0)
    {
        return NNTILE_HIP_EWORKSPACE;
    }
    const int64_t q_blocks64 = (a->q_seq + 63) / 64, k_blocks64 = (a->k_seq + 63) / 64;
    const size_t cls_bytes = (size_t)q_blocks64 * (size_t)k_blocks64;
    BwdParams p;
    std::memset(&p, 0, sizeof(p));
    p.q_seq = a->q_seq;
    p.k_seq = a->k_seq;
    p.q_pos0 = a->q_pos0;
    p.k_pos0 = a->k_pos0;
    p.causal_offset = a->causal_offset;
    p.mask = a->mask;
    p.mask_ld = a->k_seq;
    p.K = a->K;
    p.Q = a->Q;
    p.V = a->V;
    p.A = a->A;
    p.dA = a->dA;
    p.lse = a->lse;
    p.D = static_cast<float *>(a->workspace);
    if(explicit_mask && a->workspace_bytes >= d_bytes + cls_bytes && k_blocks64 <= 0x7fffffff)
    {
        p.mask_class = static_cast<const uint8_t *>(a->workspace) + d_bytes;
        p.class_ld = (int32_t)k_blocks64;
    }
    p.dK = a->dK;
    p.dQ = a->dQ;
    p.dV = a->dV;
    p.batch = (int32_t)a->batch;
    p.n_batch = (int32_t)a->n_batch;
    p.kv_group = (int32_t)a->kv_group;
    p.overwrite = (a->flags & NNTILE_HIP_SDPA_OVERWRITE) ? 1 : 0;
    p.scale = 1.0f / sqrtf(static_cast<float>(a->head));
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dt == DType::bf16 ? launch_bwd_16bit<Bf16>(s, p, (int)a->head, a->mask_mode)
        : launch_bwd_16bit<Fp16>(s, p, (int)a->head, a->mask_mode);
}

static int bwd_grid_call(DType dt, void *stream, const nntile_hip_sdpa_bwd_grid_args *a)
{
    if(a == nullptr || a->q_seq <= 0 || a->k_seq <= 0 || a->q_tile <= 0
            || a->k_tile <= 0 || a->head <= 0 || a->batch <= 0
            || a->n_batch <= 0 || a->kv_group <= 0
            || a->batch % (a->n_batch * a->kv_group) != 0
            || a->batch > 0x7fffffff || a->q_seq > 0x7fffffff
            || a->k_seq > 0x7fffffff
            || a->n_q_tiles <= 0 || a->n_q_tiles > NNTILE_HIP_SDPA_BWD_MAX_TILES
            || a->n_kv_tiles <= 0 || a->n_kv_tiles > NNTILE_HIP_SDPA_BWD_MAX_TILES
            || a->n_slabs < 0 || a->n_slabs > NNTILE_HIP_SDPA_BWD_MAX_TILES)
    {
        return NNTILE_HIP_EINVAL;
    }
    const int n_slabs = a->n_slabs == 0 ? 1 : a->n_slabs;
    const int n_q_all = n_slabs * a->n_q_tiles, n_kv_all = n_slabs * a->n_kv_tiles;
    if(n_q_all > NNTILE_HIP_SDPA_BWD_MAX_TILES || n_kv_all > NNTILE_HIP_SDPA_BWD_MAX_TILES
            || a->batch * n_slabs > 0x7fffffff)
    {
        return NNTILE_HIP_EINVAL;
    }
    if(a->mask_mode != NNTILE_HIP_MASK_NONE && a->mask_mode != NNTILE_HIP_MASK_CAUSAL)
    {
        return mode_ok(a->mask_mode) ? NNTILE_HIP_EUNSUPPORTED : NNTILE_HIP_EINVAL;
    }
    // the tile counts must match the extents
    if((a->q_seq + a->q_tile - 1) / a->q_tile != a->n_q_tiles
            || (a->k_seq + a->k_tile - 1) / a->k_tile != a->n_kv_tiles)
    {
        return NNTILE_HIP_EINVAL;
    }
    if(a->head != 32 && a->head != 64 && a->head != 128)
    {
        return NNTILE_HIP_EUNSUPPORTED;
    }
    // a workgroup's 128 rows must not straddle two allocations
    if((a->n_q_tiles > 1 && a->q_tile % 128 != 0) || (a->n_kv_tiles > 1 && a->k_tile % 128 != 0))
    {
        return NNTILE_HIP_EUNSUPPORTED;
    }
    const size_t d_bytes = (size_t)n_slabs * (size_t)a->q_seq * (size_t)a->batch * sizeof(float);
    if(a->workspace == nullptr || a->workspace_bytes < d_bytes
            || (reinterpret_cast<uintptr_t>(a->workspace) & 3u) != 0)
    {
        return NNTILE_HIP_EWORKSPACE;
    }
    BwdGridParams p;
    std::memset(static_cast<void *>(&p), 0, sizeof(p));
    p.n_slabs = n_slabs;
    p.n_q_tiles = a->n_q_tiles;
    p.n_kv_tiles = a->n_kv_tiles;
    p.q_seq = a->q_seq;
    p.k_seq = a->k_seq;
    p.q_tile = a->q_tile;
    p.k_tile = a->k_tile;
    p.q_pos0 = a->q_pos0;
    p.k_pos0 = a->k_pos0;
    p.causal_offset = a->causal_offset;
    p.D = static_cast<float *>(a->workspace);
    p.batch = (int32_t)a->batch;
    p.n_batch = (int32_t)a->n_batch;
    p.kv_group = (int32_t)a->kv_group;
    p.overwrite = (a->flags & NNTILE_HIP_SDPA_OVERWRITE) ? 1 : 0;
    p.scale = 1.0f / sqrtf(static_cast<float>(a->head));
    for(int t = 0; t < n_kv_all; ++t)
    {
        if(a->K[t] == nullptr || a->V[t] == nullptr || a->dK[t] == nullptr
                || a->dV[t] == nullptr || !aligned16(a->K[t]) || !aligned16(a->V[t])
                || !aligned16(a->dK[t]) || !aligned16(a->dV[t]))
        {
            return NNTILE_HIP_EINVAL;
        }
        p.Kt[t] = a->K[t];
        p.Vt[t] = a->V[t];
        p.dKt[t] = a->dK[t];
        p.dVt[t] = a->dV[t];
    }
    for(int t = 0; t < n_q_all; ++t)
    {
        if(a->Q[t] == nullptr || a->A[t] == nullptr || a->dA[t] == nullptr
                || a->lse[t] == nullptr || a->dQ[t] == nullptr || !aligned16(a->Q[t])
                || !aligned16(a->A[t]) || !aligned16(a->dA[t]) || !aligned16(a->dQ[t]))
        {
            return NNTILE_HIP_EINVAL;
        }
        p.Qt[t] = a->Q[t];
        p.dAt[t] = a->dA[t];
        p.lset[t] = a->lse[t];
        p.dQt[t] = a->dQ[t];
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dt == DType::bf16
        ? launch_bwd_grid_16bit<Bf16>(s, p, a->A, a->n_q_tiles, (int)a->head, a->mask_mode)
        : launch_bwd_grid_16bit<Fp16>(s, p, a->A, a->n_q_tiles, (int)a->head, a->mask_mode);
}

static int flash_bwd_call(DType dt, void *stream, int64_t seq, int64_t head,
        int64_t batch, const void *K, const void *Q, const void *V, const void *A,
        const void *dA, const void *mask, const float *lse, void *scratch_dQ,
        void *dK, void *dQ, void *dV)
{
    nntile_hip_sdpa_bwd_args a;
    std::memset(&a, 0, sizeof(a));
    a.q_seq = a.k_seq = seq;
    a.head = head;
    a.batch = a.n_batch = batch;
    a.kv_group = 1;
    a.mask_mode = NNTILE_HIP_MASK_ADDITIVE;
    a.K = K;
    a.Q = Q;
    a.V = V;
    a.A = A;
    a.dA = dA;
    a.mask = mask;
    a.lse = lse;
    a.dK = dK;
    a.dQ = dQ;
    a.dV = dV;
    // the scratch tile of dQ (seq*head*batch 16-bit values) holds the row dots
    a.workspace = scratch_dQ;
    a.workspace_bytes = (size_t)seq * (size_t)head * (size_t)batch * 2;
    return bwd_call(dt, stream, &a);
}

// bytes of a [seq, batch] fp32 tile (what the reference registers as
// scratch_logsumexp); 0 for sizes that are refused anyway
static size_t tile_floats_bytes(int64_t seq, int64_t batch)
{
    return (seq > 0 && batch > 0 && seq <= 0x7fffffff && batch <= 0x7fffffff)
        ? (size_t)seq * (size_t)batch * sizeof(float) : 0;
}

// scratch_lse: the reference's scratch tile for the logsumexp of the pair
// (seq * batch floats, src/starpu/flash_sdpa_fwd_cudnn.cc:128-136); the merge
// is fused into the kernel, so the tile is free: a large mask is scanned once
// into it instead of once per batch entry.  May be null.
static int flash_call(DType dt, void *stream, int64_t seq, int64_t head,
        int64_t batch, const void *K, const void *Q, const void *mask,
        const void *V, float *lse, void *A, float *scratch_lse,
        size_t scratch_lse_bytes)
{
    nntile_hip_sdpa_tile_args a;
    std::memset(&a, 0, sizeof(a));
    a.q_seq = a.k_seq = seq;
    a.head = head;
    a.batch = batch;
    a.n_batch = batch;
    a.kv_group = 1;
    a.mask_mode = NNTILE_HIP_MASK_ADDITIVE;
    a.K = K;
    a.Q = Q;
    a.mask = mask;
    a.V = V;
    a.lse = lse;
    a.A = A;
    return tile_call(dt, stream, &a, 0, scratch_lse, scratch_lse_bytes);
}

static int grid_call(DType dt, void *stream, const nntile_hip_sdpa_grid_args *a)
{
    if(a == nullptr || a->q_seq <= 0 || a->k_seq <= 0 || a->q_tile <= 0
            || a->k_tile <= 0 || a->head <= 0 || a->batch <= 0
            || a->n_batch <= 0 || a->kv_group <= 0
            || a->batch % (a->n_batch * a->kv_group) != 0
            || a->batch > 0x7fffffff || a->q_seq > 0x7fffffff
            || a->k_seq > 0x7fffffff
            || a->n_q_tiles <= 0 || a->n_q_tiles > NNTILE_HIP_SDPA_MAX_TILES
            || a->n_kv_tiles <= 0 || a->n_kv_tiles > NNTILE_HIP_SDPA_MAX_TILES
            || a->n_slabs < 0 || a->n_slabs > NNTILE_HIP_SDPA_MAX_TILES)
    {
        return NNTILE_HIP_EINVAL;
    }
    const int n_slabs = a->n_slabs == 0 ? 1 : a->n_slabs;
    const int n_q_all = n_slabs * a->n_q_tiles, n_kv_all = n_slabs * a->n_kv_tiles;
    if(n_q_all > NNTILE_HIP_SDPA_MAX_TILES || n_kv_all > NNTILE_HIP_SDPA_MAX_TILES
            || a->batch * n_slabs > 0x7fffffff)
    {
        return NNTILE_HIP_EINVAL;
    }
    if(a->mask_mode != NNTILE_HIP_MASK_NONE
            && a->mask_mode != NNTILE_HIP_MASK_CAUSAL)
    {
        return mode_ok(a->mask_mode) ? NNTILE_HIP_EUNSUPPORTED
            : NNTILE_HIP_EINVAL;
    }
    // the tile counts must match the extents
    if((a->q_seq + a->q_tile - 1) / a->q_tile != a->n_q_tiles
            || (a->k_seq + a->k_tile - 1) / a->k_tile != a->n_kv_tiles)
    {
        return NNTILE_HIP_EINVAL;
    }
    PrefillParams p;
    std::memset(&p, 0, sizeof(p));
    p.q_seq = a->q_seq;
    p.k_seq = a->k_seq;
    p.q_tile = a->q_tile;
    p.k_tile = a->k_tile;
    p.q_pos0 = a->q_pos0;
    p.k_pos0 = a->k_pos0;
    p.causal_offset = a->causal_offset;
    p.n_q_tiles = a->n_q_tiles;
    p.n_kv_tiles = a->n_kv_tiles;
    p.n_slabs = n_slabs;
    p.batch = (int32_t)a->batch;
    p.n_batch = (int32_t)a->n_batch;
    p.kv_group = (int32_t)a->kv_group;
    p.overwrite = (a->flags & NNTILE_HIP_SDPA_OVERWRITE) ? 1 : 0;
    p.form = prefill_form(a->flags);
    for(int t = 0; t < n_kv_all; ++t)
    {
        if(a->K[t] == nullptr || a->V[t] == nullptr || !aligned16(a->K[t])
                || !aligned16(a->V[t]))
        {
            return NNTILE_HIP_EINVAL;
        }
        p.K[t] = a->K[t];
        p.V[t] = a->V[t];
    }
    for(int t = 0; t < n_q_all; ++t)
    {
        if(a->Q[t] == nullptr || a->A[t] == nullptr || a->lse[t] == nullptr
                || !aligned16(a->Q[t]) || !aligned16(a->A[t]))
        {
            return NNTILE_HIP_EINVAL;
        }
        p.Q[t] = a->Q[t];
        p.A[t] = a->A[t];
        p.lse[t] = a->lse[t];
    }
    return dispatch_prefill(dt, static_cast<hipStream_t>(stream), p, a->head,
            a->mask_mode);
}

static bool decode_args_ok(const nntile_hip_sdpa_tile_args *a)
{
    return a != nullptr && a->q_seq > 0 && a->k_seq > 0 && a->head > 0
        && a->batch > 0 && a->n_batch > 0 && a->kv_group > 0
        && a->batch % (a->n_batch * a->kv_group) == 0
        && a->batch <= 0x7fffffff && a->k_seq <= 0x7fffffff
        && a->q_seq * a->kv_group <= 64;
}

static void decode_geometry(const nntile_hip_sdpa_tile_args *a, int &units,
        int &n_steps, int &splits, int &rows)
{
    units = (int)(a->batch / a->kv_group);
    n_steps = (int)((a->k_seq + kDecKeys - 1) / kDecKeys);
    splits = decode_choose_splits(units, n_steps);
    rows = (int)(a->q_seq * a->kv_group);
}

// k_new, v_new, n_new: rows [k_seq - n_new, k_seq) of every entry are not in
// the caches yet; the launch reads them from k_new / v_new and writes them
// into the caches as well (n_new == 0: nothing of the kind)
static int decode_call(DType dt, void *stream, const nntile_hip_sdpa_tile_args *a,
        int64_t kv_rows, void *workspace, size_t workspace_bytes,
        const void *k_new = nullptr, const void *v_new = nullptr, int64_t n_new = 0)
{
    if(n_new != 0 && (a == nullptr || n_new < 0 || n_new > a->k_seq || n_new > 0x7fffffff
                || k_new == nullptr || v_new == nullptr || !aligned16(k_new)
                || !aligned16(v_new)))
    {
        return NNTILE_HIP_EINVAL;
    }
    if(!decode_args_ok(a) || kv_rows < a->k_seq || !mode_ok(a->mask_mode) || a->K == nullptr
            || a->Q == nullptr || a->V == nullptr || a->lse == nullptr
            || a->A == nullptr || !aligned16(a->K) || !aligned16(a->Q)
            || !aligned16(a->V) || !aligned16(a->A))
    {
        return NNTILE_HIP_EINVAL;
    }
    const bool explicit_mask = a->mask_mode == NNTILE_HIP_MASK_ADDITIVE
        || a->mask_mode == NNTILE_HIP_MASK_BOOL;
    if(explicit_mask && a->mask == nullptr)
    {
        return NNTILE_HIP_EINVAL;
    }
    if(a->head != 64 && a->head != 128)
    {
        return NNTILE_HIP_EUNSUPPORTED;
    }
    int units, n_steps, splits, rows;
    decode_geometry(a, units, n_steps, splits, rows);
    const size_t need = decode_workspace_bytes(units, splits, rows, (int)a->head);
    if(workspace == nullptr || workspace_bytes < need || !aligned16(workspace))
    {
        return NNTILE_HIP_EWORKSPACE;
    }
    DecodeParams p;
    std::memset(&p, 0, sizeof(p));
    p.q_seq = a->q_seq;
    p.k_seq = a->k_seq;
    p.kv_rows = kv_rows;
    p.q_pos0 = a->q_pos0;
    p.k_pos0 = a->k_pos0;
    p.causal_offset = a->causal_offset;
    p.mask = a->mask;
    p.mask_ld = a->k_seq;
    p.K = a->K;
    p.V = a->V;
    p.Q = a->Q;
    p.lse = a->lse;
    p.A = a->A;
    p.part_o = static_cast<float *>(workspace);
    p.part_ml = reinterpret_cast<float *>(static_cast<char *>(workspace)
            + decode_partial_o_bytes(units, splits, rows, (int)a->head));
    p.sync = reinterpret_cast<unsigned long long *>(reinterpret_cast<char *>(p.part_ml)
            + decode_partial_ml_bytes(units, splits, rows));
    p.fused = (a->flags & NNTILE_HIP_SDPA_DECODE_SEPARATE_MERGE) ? 0 : 1;
    p.fenced = (a->flags & NNTILE_HIP_SDPA_DECODE_FENCED) ? 1 : 0;
    p.k_new = k_new;
    p.v_new = v_new;
    p.n_new = (int32_t)n_new;
    p.n_batch = (int32_t)a->n_batch;
    p.kv_group = (int32_t)a->kv_group;
    p.n_head_kv = (int32_t)(units / a->n_batch);
    p.rows = rows;
    p.n_splits = splits;
    p.n_steps = n_steps;
    p.overwrite = (a->flags & NNTILE_HIP_SDPA_OVERWRITE) ? 1 : 0;
    p.steps_per_split = (n_steps + splits - 1) / splits;
    p.scale = 1.0f / sqrtf(static_cast<float>(a->head));
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dt == DType::bf16 ? launch_decode_16bit<Bf16>(s, p, (int)a->head, a->mask_mode)
        : launch_decode_16bit<Fp16>(s, p, (int)a->head, a->mask_mode);
}

// The fp32 twin: steps of 32 keys, partials in fp32, the merge always a second
// launch.
static void decode_fp32_geometry(const nntile_hip_sdpa_tile_args *a, int &units,
        int &n_steps, int &splits, int &rows)
{
    units = (int)(a->batch / a->kv_group);
    n_steps = decode_fp32_steps(a->k_seq);
    splits = decode_fp32_choose_splits(units, n_steps);
    rows = (int)(a->q_seq * a->kv_group);
}

static int decode_fp32_call(void *stream, const nntile_hip_sdpa_tile_args *a,
        int64_t kv_rows, void *workspace, size_t workspace_bytes,
        const void *k_new = nullptr, const void *v_new = nullptr, int64_t n_new = 0)
{
    if(n_new != 0 && (a == nullptr || n_new < 0 || n_new > a->k_seq || n_new > 0x7fffffff
                || k_new == nullptr || v_new == nullptr || !aligned16(k_new)
                || !aligned16(v_new)))
    {
        return NNTILE_HIP_EINVAL;
    }
    if(!decode_args_ok(a) || kv_rows < a->k_seq || !mode_ok(a->mask_mode) || a->K == nullptr
            || a->Q == nullptr || a->V == nullptr || a->lse == nullptr
            || a->A == nullptr || !aligned16(a->K) || !aligned16(a->Q)
            || !aligned16(a->V) || !aligned16(a->A))
    {
        return NNTILE_HIP_EINVAL;
    }
    const bool explicit_mask = a->mask_mode == NNTILE_HIP_MASK_ADDITIVE
        || a->mask_mode == NNTILE_HIP_MASK_BOOL;
    if(explicit_mask && a->mask == nullptr)
    {
        return NNTILE_HIP_EINVAL;
    }
    if(a->head != 64 && a->head != 128)
    {
        return NNTILE_HIP_EUNSUPPORTED;
    }
    int units, n_steps, splits, rows;
    decode_fp32_geometry(a, units, n_steps, splits, rows);
    const size_t need = decode_fp32_workspace_bytes(units, splits, rows, (int)a->head);
    if(workspace == nullptr || workspace_bytes < need || !aligned16(workspace))
    {
        return NNTILE_HIP_EWORKSPACE;
    }
    DecodeParams p;
    std::memset(&p, 0, sizeof(p));
    p.q_seq = a->q_seq;
    p.k_seq = a->k_seq;
    p.kv_rows = kv_rows;
    p.q_pos0 = a->q_pos0;
    p.k_pos0 = a->k_pos0;
    p.causal_offset = a->causal_offset;
    p.mask = a->mask;
    p.mask_ld = a->k_seq;
    p.K = a->K;
    p.V = a->V;
    p.Q = a->Q;
    p.lse = a->lse;
    p.A = a->A;
    p.part_o = static_cast<float *>(workspace);
    p.part_ml = p.part_o + (size_t)units * splits * rows * a->head;
    p.n_batch = (int32_t)a->n_batch;
    p.kv_group = (int32_t)a->kv_group;
    p.n_head_kv = (int32_t)(units / a->n_batch);
    p.rows = rows;
    p.n_splits = splits;
    p.n_steps = n_steps;
    p.overwrite = (a->flags & NNTILE_HIP_SDPA_OVERWRITE) ? 1 : 0;
    p.steps_per_split = (n_steps + splits - 1) / splits;
    p.scale = 1.0f / sqrtf(static_cast<float>(a->head));
    p.k_new = k_new;
    p.v_new = v_new;
    p.n_new = (int32_t)n_new;
    return launch_decode_fp32(static_cast<hipStream_t>(stream), p, (int)a->head, a->mask_mode);
}

// ---- decode with the split partials in memory the library owns ---------------
// For callers that may not allocate (a stream under graph capture, a serving
// loop that forbids it): the workspace of decode_call is this file-scope
// device array instead of a caller's buffer.  Every GPU holds its own copy at
// its own address; in host code the array's name is only a handle for
// hipGetSymbolAddress, never an address to pass on.  The decode kernels write
// every partial they later read, so nothing has to be cleared between calls;
// calls that overlap on one GPU share the array and race.
static __device__ __align__(256) unsigned char scratch[NNTILE_HIP_DECODE_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static std::atomic<void *> scratch_ptr[kMaxDevices];
static std::mutex scratch_mutex;

// Device address of `scratch` on the current device, resolved on the first
// call per device; `stream` must be a stream of that device.
static int static_scratch(hipStream_t stream, void **out)
{
    int dev = -1;
    if(hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    {
        return NNTILE_HIP_ELAUNCH;
    }
    // The array of the CURRENT device is the one handed to the kernels, so a
    // stream of another GPU would run them on an address of the wrong device:
    // refused.  (A query only: legal on a capturing stream; the null stream
    // reports the current device.)
    if(stream != nullptr)
    {
        hipDevice_t stream_dev = -1;
        if(hipStreamGetDevice(stream, &stream_dev) != hipSuccess)
        {
            (void)hipGetLastError();
            return NNTILE_HIP_EINVAL;
        }
        if((int)stream_dev != dev)
        {
            std::fprintf(stderr, "nntile_hip_sdpa_fwd_decode_static: the stream belongs to "
                    "device %d, the current device is %d\n", (int)stream_dev, dev);
            return NNTILE_HIP_EINVAL;
        }
    }
    void *ptr = scratch_ptr[dev].load(std::memory_order_acquire);
    if(ptr == nullptr)
    {
        std::lock_guard<std::mutex> guard(scratch_mutex);
        ptr = scratch_ptr[dev].load(std::memory_order_acquire);
        if(ptr == nullptr)
        {
            if(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess
                    || ptr == nullptr)
            {
                (void)hipGetLastError();
                return NNTILE_HIP_ELAUNCH;
            }
            scratch_ptr[dev].store(ptr, std::memory_order_release);
        }
    }
    *out = ptr;
    return NNTILE_HIP_OK;
}

static int decode_static_call(void *stream, int32_t dtype,
        const nntile_hip_sdpa_tile_args *a)
{
    if(dtype != NNTILE_HIP_DTYPE_BF16 && dtype != NNTILE_HIP_DTYPE_FP16)
    {
        return NNTILE_HIP_EINVAL;
    }
    if(!decode_args_ok(a))
    {
        return NNTILE_HIP_EINVAL;
    }
    if(a->head != 64 && a->head != 128)
    {
        return NNTILE_HIP_EUNSUPPORTED;
    }
    int units, n_steps, splits, rows;
    decode_geometry(a, units, n_steps, splits, rows);
    const size_t need = decode_workspace_bytes(units, splits, rows, (int)a->head);
    if(need > (size_t)NNTILE_HIP_DECODE_STATIC_SCRATCH_BYTES)
    {
        std::fprintf(stderr, "nntile_hip_sdpa_fwd_decode_static: the split partials of this "
                "shape need %zu bytes, the library's own buffer holds %zu; use "
                "nntile_hip_sdpa_fwd_decode_* with a workspace\n", need,
                (size_t)NNTILE_HIP_DECODE_STATIC_SCRATCH_BYTES);
        return NNTILE_HIP_EWORKSPACE;
    }
    void *ws = nullptr;
    const int rc = static_scratch(static_cast<hipStream_t>(stream), &ws);
    if(rc != NNTILE_HIP_OK)
    {
        return rc;
    }
    return decode_call(dtype == NNTILE_HIP_DTYPE_BF16 ? DType::bf16 : DType::fp16, stream, a,
            a->k_seq, ws, (size_t)NNTILE_HIP_DECODE_STATIC_SCRATCH_BYTES);
}

template<typename S>
static int accumulate_call(void *stream, int64_t head, int64_t seq,
        int64_t batch, const float *src_lse, const void *src_attn,
        float *dst_lse, void *dst_attn)
{
    if(head <= 0 || seq <= 0 || batch <= 0)
    {
        return NNTILE_HIP_OK;   // the reference kernel returns silently
    }
    if(src_lse == nullptr || src_attn == nullptr || dst_lse == nullptr
            || dst_attn == nullptr)
    {
        return NNTILE_HIP_EINVAL;
    }
    return launch_accumulate<S>(static_cast<hipStream_t>(stream), head, seq,
            batch, src_lse, src_attn, dst_lse, dst_attn);
}

static int rope_call(DType dt, bool backward, void *stream, int64_t m, int64_t n,
        const void *sin, const void *cos, const void *src, void *dst)
{
    if(m < 0 || n < 0)
    {
        return NNTILE_HIP_EINVAL;
    }
    if(m == 0 || n == 0)
    {
        return NNTILE_HIP_OK;   // nothing to rotate (the reference launches an empty grid)
    }
    if(sin == nullptr || cos == nullptr || src == nullptr || dst == nullptr
            || m > (int64_t)0x3fffffffffffffff / n)
    {
        return NNTILE_HIP_EINVAL;
    }
    const int code = dt == DType::bf16 ? 0 : (dt == DType::fp16 ? 1 : 2);
    return launch_rope(static_cast<hipStream_t>(stream), code, backward, m, n, sin, cos, src,
            dst);
}

static int transpose_call(DType dt, void *stream, int64_t m, int64_t n, float alpha,
        const void *src, void *dst)
{
    if(m < 0 || n < 0)
    {
        return NNTILE_HIP_EINVAL;
    }
    if(m == 0 || n == 0)
    {
        return NNTILE_HIP_OK;
    }
    if(src == nullptr || dst == nullptr || src == dst
            || m > (int64_t)0x3fffffffffffffff / n)
    {
        return NNTILE_HIP_EINVAL;
    }
    const int code = dt == DType::bf16 ? 0 : (dt == DType::fp16 ? 1 : 2);
    return launch_transpose(static_cast<hipStream_t>(stream), code, m, n, alpha, src, dst);
}

static int kv_append_call(int elem, void *stream, int64_t head, int64_t rows, int64_t entries,
        int64_t capacity, int64_t filled, const void *k_new, const void *v_new, void *k_cache,
        void *v_cache)
{
    if(head <= 0 || rows < 0 || entries < 0 || capacity <= 0 || filled < 0)
    {
        return NNTILE_HIP_EINVAL;
    }
    if(rows > capacity - filled)
    {
        // LlamaAttention._append_to_kv_cache raises here
        // (wrappers/python/nntile/model/llama_attention.py:524-529)
        return NNTILE_HIP_EINVAL;
    }
    if(rows == 0 || entries == 0)
    {
        return NNTILE_HIP_OK;
    }
    if(k_new == nullptr || v_new == nullptr || k_cache == nullptr || v_cache == nullptr
            || entries > (int64_t)0x0fffffffffffffff / (capacity * head))
    {
        return NNTILE_HIP_EINVAL;
    }
    return launch_kv_cache_append(static_cast<hipStream_t>(stream), elem, head, rows, entries,
            capacity, filled, k_new, v_new, k_cache, v_cache);
}

// Blocking: the class comes back to the host.
static int mask_class_call(int dtype, void *stream, int64_t k_rows, int64_t q_cols,
        const void *mask, int64_t offset, int32_t *workspace, int32_t *class_out)
{
    if(k_rows <= 0 || q_cols <= 0 || mask == nullptr || workspace == nullptr
            || class_out == nullptr || k_rows > (int64_t)0x3fffffffffffffff / q_cols
            || (reinterpret_cast<uintptr_t>(workspace) & 3u) != 0)
    {
        return NNTILE_HIP_EINVAL;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int rc = launch_mask_classify(s, dtype, k_rows, q_cols, offset, mask,
            reinterpret_cast<uint32_t *>(workspace));
    if(rc != NNTILE_HIP_OK)
    {
        return rc;
    }
    uint32_t seen = 0;
    if(hipMemcpyAsync(&seen, workspace, sizeof(seen), hipMemcpyDeviceToHost, s) != hipSuccess
            || hipStreamSynchronize(s) != hipSuccess)
    {
        return NNTILE_HIP_ELAUNCH;
    }
    const bool visible = seen & 1u, hidden = seen & 2u, other = seen & 4u, off_rule = seen & 8u;
    if(other)
    {
        *class_out = NNTILE_HIP_MASK_TILE_MIXED;
    }
    else if(!hidden)
    {
        *class_out = NNTILE_HIP_MASK_TILE_OPEN;
    }
    else if(!visible)
    {
        *class_out = NNTILE_HIP_MASK_TILE_HIDDEN;
    }
    else
    {
        *class_out = off_rule ? NNTILE_HIP_MASK_TILE_MIXED : NNTILE_HIP_MASK_TILE_CAUSAL;
    }
    return NNTILE_HIP_OK;
}

static nntile_hip_stream_provider g_stream_provider = nullptr;

static void codelet_call(DType dt, const char *name, void *buffers[],
        void *cl_args)
{
    // Error behaviour of the reference body: report and return, the task
    // becomes a no-op (src/starpu/flash_sdpa_fwd_cudnn.cc:69-115).
    if(buffers == nullptr || cl_args == nullptr)
    {
        std::fprintf(stderr, "HIP Worker: %s: null buffers or arguments, "
                "skipping task\n", name);
        return;
    }
    const auto *args = static_cast<const nntile_hip_flash_sdpa_cl_args *>(cl_args);
    auto **ifs = reinterpret_cast<nntile_hip_variable_interface **>(buffers);
    for(int i = 0; i < 6; ++i)
    {
        if(ifs[i] == nullptr)
        {
            std::fprintf(stderr, "HIP Worker: %s: buffer %d is null, skipping "
                    "task\n", name, i);
            return;
        }
    }
    void *stream = g_stream_provider ? g_stream_provider() : nullptr;
    const int rc = flash_call(dt, stream, args->seq, args->head, args->batch,
            reinterpret_cast<const void *>(ifs[0]->ptr),
            reinterpret_cast<const void *>(ifs[1]->ptr),
            reinterpret_cast<const void *>(ifs[2]->ptr),
            reinterpret_cast<const void *>(ifs[4]->ptr),
            reinterpret_cast<float *>(ifs[3]->ptr),
            reinterpret_cast<void *>(ifs[5]->ptr),
            // buffer 6: the scratch tile for the pair's logsumexp
            ifs[6] != nullptr ? reinterpret_cast<float *>(ifs[6]->ptr) : nullptr,
            ifs[6] != nullptr ? ifs[6]->elemsize : 0);
    if(rc != NNTILE_HIP_OK)
    {
        std::fprintf(stderr, "HIP Worker: %s: launch failed with code %d "
                "(seq=%lld head=%lld batch=%lld), skipping task\n", name, rc,
                (long long)args->seq, (long long)args->head,
                (long long)args->batch);
    }
}

static void bwd_codelet_call(DType dt, const char *name, void *buffers[],
        void *cl_args)
{
    // Buffer order of the reference body (src/starpu/flash_sdpa_bwd_cudnn.cc:
    // 103-115, modes :175-187): K Q V A dA mask logsumexp (R), dK dQ dV (RW),
    // scratch_dK scratch_dQ scratch_dV (SCRATCH); same error behaviour.
    if(buffers == nullptr || cl_args == nullptr)
    {
        std::fprintf(stderr, "HIP Worker: %s: null buffers or arguments, "
                "skipping task\n", name);
        return;
    }
    const auto *args = static_cast<const nntile_hip_flash_sdpa_cl_args *>(cl_args);
    auto **ifs = reinterpret_cast<nntile_hip_variable_interface **>(buffers);
    for(int i = 0; i < 12; ++i)
    {
        if(i != 10 && ifs[i] == nullptr)
        {
            std::fprintf(stderr, "HIP Worker: %s: buffer %d is null, skipping "
                    "task\n", name, i);
            return;
        }
    }
    void *stream = g_stream_provider ? g_stream_provider() : nullptr;
    auto ptr = [&](int i) { return reinterpret_cast<void *>(ifs[i]->ptr); };
    const int rc = flash_bwd_call(dt, stream, args->seq, args->head, args->batch,
            ptr(0), ptr(1), ptr(2), ptr(3), ptr(4), ptr(5),
            reinterpret_cast<const float *>(ifs[6]->ptr), ptr(11), ptr(7), ptr(8), ptr(9));
    if(rc != NNTILE_HIP_OK)
    {
        std::fprintf(stderr, "HIP Worker: %s: launch failed with code %d "
                "(seq=%lld head=%lld batch=%lld), skipping task\n", name, rc,
                (long long)args->seq, (long long)args->head,
                (long long)args->batch);
    }
}

// Geometry of a grid call out of the codelet arguments; false (after a line on
// stderr) when the task cannot be run.
static bool grid_codelet_geometry(const char *name, void *buffers[], void *cl_args,
        int max_tiles, const nntile_hip_sdpa_grid_cl_args *&args, int &n_k, int &n_q)
{
    if(buffers == nullptr || cl_args == nullptr)
    {
        std::fprintf(stderr, "HIP Worker: %s: null buffers or arguments, "
                "skipping task\n", name);
        return false;
    }
    args = static_cast<const nntile_hip_sdpa_grid_cl_args *>(cl_args);
    const int n_slabs = args->n_slabs > 0 ? args->n_slabs : 1;
    if(args->n_q_tiles <= 0 || args->n_kv_tiles <= 0
            || (int64_t)n_slabs * args->n_q_tiles > max_tiles
            || (int64_t)n_slabs * args->n_kv_tiles > max_tiles)
    {
        std::fprintf(stderr, "HIP Worker: %s: %d slabs of %d x %d tiles do not fit one "
                "call, skipping task\n", name, n_slabs, args->n_q_tiles, args->n_kv_tiles);
        return false;
    }
    n_k = n_slabs * args->n_kv_tiles;
    n_q = n_slabs * args->n_q_tiles;
    return true;
}

template<typename A>
static void grid_codelet_fill(A &a, const nntile_hip_sdpa_grid_cl_args *args)
{
    std::memset(&a, 0, sizeof(a));
    a.q_seq = args->q_seq;
    a.k_seq = args->k_seq;
    a.q_tile = args->q_tile;
    a.k_tile = args->k_tile;
    a.head = args->head;
    a.batch = args->batch;
    a.n_batch = args->n_batch;
    a.kv_group = args->kv_group;
    a.mask_mode = args->mask_mode;
    a.n_q_tiles = args->n_q_tiles;
    a.n_kv_tiles = args->n_kv_tiles;
    a.flags = args->flags;
    a.n_slabs = args->n_slabs;
    a.q_pos0 = args->q_pos0;
    a.k_pos0 = args->k_pos0;
    a.causal_offset = args->causal_offset;
}

static void fwd_grid_codelet_call(DType dt, const char *name, void *buffers[], void *cl_args)
{
    const nntile_hip_sdpa_grid_cl_args *args = nullptr;
    int n_k = 0, n_q = 0;
    if(!grid_codelet_geometry(name, buffers, cl_args, NNTILE_HIP_SDPA_MAX_TILES, args, n_k, n_q))
    {
        return;
    }
    auto **ifs = reinterpret_cast<nntile_hip_variable_interface **>(buffers);
    const int n_buffers = 2 * n_k + 3 * n_q;
    for(int i = 0; i < n_buffers; ++i)
    {
        if(ifs[i] == nullptr)
        {
            std::fprintf(stderr, "HIP Worker: %s: buffer %d is null, skipping task\n", name, i);
            return;
        }
    }
    nntile_hip_sdpa_grid_args a;
    grid_codelet_fill(a, args);
    for(int t = 0; t < n_k; ++t)
    {
        a.K[t] = reinterpret_cast<const void *>(ifs[t]->ptr);
        a.V[t] = reinterpret_cast<const void *>(ifs[n_k + t]->ptr);
    }
    for(int t = 0; t < n_q; ++t)
    {
        a.Q[t] = reinterpret_cast<const void *>(ifs[2 * n_k + t]->ptr);
        a.lse[t] = reinterpret_cast<float *>(ifs[2 * n_k + n_q + t]->ptr);
        a.A[t] = reinterpret_cast<void *>(ifs[2 * n_k + 2 * n_q + t]->ptr);
    }
    void *stream = g_stream_provider ? g_stream_provider() : nullptr;
    const int rc = grid_call(dt, stream, &a);
    if(rc != NNTILE_HIP_OK)
    {
        std::fprintf(stderr, "HIP Worker: %s: launch failed with code %d (q_seq=%lld k_seq=%lld "
                "head=%lld batch=%lld), skipping task\n", name, rc, (long long)args->q_seq,
                (long long)args->k_seq, (long long)args->head, (long long)args->batch);
    }
}

static void bwd_grid_codelet_call(DType dt, const char *name, void *buffers[], void *cl_args)
{
    const nntile_hip_sdpa_grid_cl_args *args = nullptr;
    int n_k = 0, n_q = 0;
    if(!grid_codelet_geometry(name, buffers, cl_args, NNTILE_HIP_SDPA_BWD_MAX_TILES, args, n_k,
                n_q))
    {
        return;
    }
    auto **ifs = reinterpret_cast<nntile_hip_variable_interface **>(buffers);
    const int n_buffers = 4 * n_k + 5 * n_q + 1;
    for(int i = 0; i < n_buffers; ++i)
    {
        if(ifs[i] == nullptr)
        {
            std::fprintf(stderr, "HIP Worker: %s: buffer %d is null, skipping task\n", name, i);
            return;
        }
    }
    nntile_hip_sdpa_bwd_grid_args a;
    grid_codelet_fill(a, args);
    int at = 0;
    auto take = [&]() { return reinterpret_cast<void *>(ifs[at++]->ptr); };
    for(int t = 0; t < n_k; ++t) { a.K[t] = take(); }
    for(int t = 0; t < n_k; ++t) { a.V[t] = take(); }
    for(int t = 0; t < n_q; ++t) { a.Q[t] = take(); }
    for(int t = 0; t < n_q; ++t) { a.A[t] = take(); }
    for(int t = 0; t < n_q; ++t) { a.dA[t] = take(); }
    for(int t = 0; t < n_q; ++t) { a.lse[t] = static_cast<const float *>(take()); }
    for(int t = 0; t < n_k; ++t) { a.dK[t] = take(); }
    for(int t = 0; t < n_q; ++t) { a.dQ[t] = take(); }
    for(int t = 0; t < n_k; ++t) { a.dV[t] = take(); }
    a.workspace_bytes = ifs[at]->elemsize;
    a.workspace = take();
    void *stream = g_stream_provider ? g_stream_provider() : nullptr;
    const int rc = bwd_grid_call(dt, stream, &a);
    if(rc != NNTILE_HIP_OK)
    {
        std::fprintf(stderr, "HIP Worker: %s: launch failed with code %d (q_seq=%lld k_seq=%lld "
                "head=%lld batch=%lld), skipping task\n", name, rc, (long long)args->q_seq,
                (long long)args->k_seq, (long long)args->head, (long long)args->batch);
    }
}

} // namespace nntile_hip

using namespace nntile_hip;

extern "C"
{

int nntile_hip_flash_sdpa_fwd_bf16(void *stream, int64_t seq, int64_t head,
        int64_t batch, const uint16_t *K, const uint16_t *Q,
        const uint16_t *mask, float *scratch_lse, const uint16_t *V, uint16_t *,
        float *lse, uint16_t *A)
{
    return flash_call(DType::bf16, stream, seq, head, batch, K, Q, mask, V, lse, A,
            scratch_lse, tile_floats_bytes(seq, batch));
}

int nntile_hip_flash_sdpa_fwd_fp16(void *stream, int64_t seq, int64_t head,
        int64_t batch, const uint16_t *K, const uint16_t *Q,
        const uint16_t *mask, float *scratch_lse, const uint16_t *V, uint16_t *,
        float *lse, uint16_t *A)
{
    return flash_call(DType::fp16, stream, seq, head, batch, K, Q, mask, V, lse, A,
            scratch_lse, tile_floats_bytes(seq, batch));
}

int nntile_hip_flash_sdpa_fwd_fp32(void *stream, int64_t seq, int64_t head,
        int64_t batch, const float *K, const float *Q, const float *mask,
        float *, const float *V, float *, float *lse, float *A)
{
    return flash_call(DType::fp32, stream, seq, head, batch, K, Q, mask, V, lse, A, nullptr, 0);
}

int nntile_hip_sdpa_fwd_tile_bf16(void *stream, const nntile_hip_sdpa_tile_args *args)
{
    return tile_call(DType::bf16, stream, args);
}

int nntile_hip_sdpa_fwd_tile_fp16(void *stream, const nntile_hip_sdpa_tile_args *args)
{
    return tile_call(DType::fp16, stream, args);
}

int nntile_hip_sdpa_fwd_tile_fp32(void *stream, const nntile_hip_sdpa_tile_args *args)
{
    return tile_call(DType::fp32, stream, args);
}

int nntile_hip_sdpa_fwd_grid_bf16(void *stream, const nntile_hip_sdpa_grid_args *args)
{
    return grid_call(DType::bf16, stream, args);
}

int nntile_hip_sdpa_fwd_grid_fp16(void *stream, const nntile_hip_sdpa_grid_args *args)
{
    return grid_call(DType::fp16, stream, args);
}

int nntile_hip_sdpa_fwd_grid_fp32(void *stream, const nntile_hip_sdpa_grid_args *args)
{
    return grid_call(DType::fp32, stream, args);
}

size_t nntile_hip_sdpa_fwd_decode_workspace_bytes(const nntile_hip_sdpa_tile_args *args)
{
    if(!decode_args_ok(args))
    {
        return 0;
    }
    int units, n_steps, splits, rows;
    decode_geometry(args, units, n_steps, splits, rows);
    return decode_workspace_bytes(units, splits, rows, (int)args->head);
}

int nntile_hip_sdpa_fwd_decode_bf16(void *stream, const nntile_hip_sdpa_tile_args *args,
        void *workspace, size_t workspace_bytes)
{
    return decode_call(DType::bf16, stream, args, args ? args->k_seq : 0, workspace,
            workspace_bytes);
}

int nntile_hip_sdpa_fwd_decode_fp16(void *stream, const nntile_hip_sdpa_tile_args *args,
        void *workspace, size_t workspace_bytes)
{
    return decode_call(DType::fp16, stream, args, args ? args->k_seq : 0, workspace,
            workspace_bytes);
}

size_t nntile_hip_sdpa_fwd_decode_workspace_bytes_fp32(const nntile_hip_sdpa_tile_args *args)
{
    if(!decode_args_ok(args))
    {
        return 0;
    }
    int units, n_steps, splits, rows;
    decode_fp32_geometry(args, units, n_steps, splits, rows);
    return decode_fp32_workspace_bytes(units, splits, rows, (int)args->head);
}

int nntile_hip_sdpa_fwd_decode_fp32(void *stream, const nntile_hip_sdpa_tile_args *args,
        void *workspace, size_t workspace_bytes)
{
    return decode_fp32_call(stream, args, args ? args->k_seq : 0, workspace, workspace_bytes);
}

int nntile_hip_sdpa_fwd_decode_static(void *stream, int32_t dtype,
        const nntile_hip_sdpa_tile_args *args)
{
    return decode_static_call(stream, dtype, args);
}

int nntile_hip_accumulate_attn_output_bf16(void *stream, int64_t head, int64_t seq,
        int64_t batch, const float *src_lse, const uint16_t *src_attn,
        float *dst_lse, uint16_t *dst_attn)
{
    return accumulate_call<Bf16Store>(stream, head, seq, batch, src_lse, src_attn,
            dst_lse, dst_attn);
}

int nntile_hip_accumulate_attn_output_fp16(void *stream, int64_t head, int64_t seq,
        int64_t batch, const float *src_lse, const uint16_t *src_attn,
        float *dst_lse, uint16_t *dst_attn)
{
    return accumulate_call<Fp16Store>(stream, head, seq, batch, src_lse, src_attn,
            dst_lse, dst_attn);
}

int nntile_hip_accumulate_attn_output_fp32(void *stream, int64_t head, int64_t seq,
        int64_t batch, const float *src_lse, const float *src_attn,
        float *dst_lse, float *dst_attn)
{
    return accumulate_call<F32Store>(stream, head, seq, batch, src_lse, src_attn,
            dst_lse, dst_attn);
}

void nntile_hip_set_stream_provider(nntile_hip_stream_provider fn)
{
    g_stream_provider = fn;
}

void nntile_hip_flash_sdpa_fwd_codelet_bf16(void *buffers[], void *cl_args)
{
    codelet_call(DType::bf16, "nntile_flash_sdpa_fwd_hip_bf16", buffers, cl_args);
}

void nntile_hip_flash_sdpa_fwd_codelet_fp16(void *buffers[], void *cl_args)
{
    codelet_call(DType::fp16, "nntile_flash_sdpa_fwd_hip_fp16", buffers, cl_args);
}

void nntile_hip_flash_sdpa_fwd_codelet_fp32(void *buffers[], void *cl_args)
{
    codelet_call(DType::fp32, "nntile_flash_sdpa_fwd_hip_fp32", buffers, cl_args);
}

size_t nntile_hip_sdpa_bwd_workspace_bytes(const nntile_hip_sdpa_bwd_args *a)
{
    if(a == nullptr || a->q_seq <= 0 || a->k_seq <= 0 || a->batch <= 0)
    {
        return 0;
    }
    // the row dots, then the classes of the 64 x 64 blocks of a mask given
    // as values
    size_t bytes = (size_t)a->q_seq * (size_t)a->batch * sizeof(float);
    if(a->mask_mode == NNTILE_HIP_MASK_ADDITIVE || a->mask_mode == NNTILE_HIP_MASK_BOOL)
    {
        bytes += (size_t)((a->q_seq + 63) / 64) * (size_t)((a->k_seq + 63) / 64);
    }
    return bytes;
}

size_t nntile_hip_sdpa_bwd_grid_workspace_bytes(const nntile_hip_sdpa_bwd_grid_args *a)
{
    if(a == nullptr || a->q_seq <= 0 || a->batch <= 0)
    {
        return 0;
    }
    const size_t n_slabs = a->n_slabs <= 0 ? 1 : (size_t)a->n_slabs;
    return n_slabs * (size_t)a->q_seq * (size_t)a->batch * sizeof(float);
}

int nntile_hip_sdpa_bwd_grid_bf16(void *stream, const nntile_hip_sdpa_bwd_grid_args *args)
{
    return bwd_grid_call(DType::bf16, stream, args);
}

int nntile_hip_sdpa_bwd_grid_fp16(void *stream, const nntile_hip_sdpa_bwd_grid_args *args)
{
    return bwd_grid_call(DType::fp16, stream, args);
}

int nntile_hip_sdpa_bwd_tile_bf16(void *stream, const nntile_hip_sdpa_bwd_args *args)
{
    return bwd_call(DType::bf16, stream, args);
}

int nntile_hip_sdpa_bwd_tile_fp16(void *stream, const nntile_hip_sdpa_bwd_args *args)
{
    return bwd_call(DType::fp16, stream, args);
}

int nntile_hip_flash_sdpa_bwd_bf16(void *stream, int64_t seq, int64_t head,
        int64_t batch, const uint16_t *K, const uint16_t *Q, const uint16_t *V,
        const uint16_t *A, const uint16_t *dA, const uint16_t *mask,
        const float *lse, uint16_t *, uint16_t *scratch_dQ, uint16_t *,
        uint16_t *dK, uint16_t *dQ, uint16_t *dV)
{
    return flash_bwd_call(DType::bf16, stream, seq, head, batch, K, Q, V, A, dA, mask,
            lse, scratch_dQ, dK, dQ, dV);
}

int nntile_hip_flash_sdpa_bwd_fp16(void *stream, int64_t seq, int64_t head,
        int64_t batch, const uint16_t *K, const uint16_t *Q, const uint16_t *V,
        const uint16_t *A, const uint16_t *dA, const uint16_t *mask,
        const float *lse, uint16_t *, uint16_t *scratch_dQ, uint16_t *,
        uint16_t *dK, uint16_t *dQ, uint16_t *dV)
{
    return flash_bwd_call(DType::fp16, stream, seq, head, batch, K, Q, V, A, dA, mask,
            lse, scratch_dQ, dK, dQ, dV);
}

void nntile_hip_sdpa_fwd_grid_codelet_bf16(void *buffers[], void *cl_args)
{
    fwd_grid_codelet_call(DType::bf16, "nntile_sdpa_fwd_grid_hip_bf16", buffers, cl_args);
}

void nntile_hip_sdpa_fwd_grid_codelet_fp16(void *buffers[], void *cl_args)
{
    fwd_grid_codelet_call(DType::fp16, "nntile_sdpa_fwd_grid_hip_fp16", buffers, cl_args);
}

void nntile_hip_sdpa_fwd_grid_codelet_fp32(void *buffers[], void *cl_args)
{
    fwd_grid_codelet_call(DType::fp32, "nntile_sdpa_fwd_grid_hip_fp32", buffers, cl_args);
}

void nntile_hip_sdpa_bwd_grid_codelet_bf16(void *buffers[], void *cl_args)
{
    bwd_grid_codelet_call(DType::bf16, "nntile_sdpa_bwd_grid_hip_bf16", buffers, cl_args);
}

void nntile_hip_sdpa_bwd_grid_codelet_fp16(void *buffers[], void *cl_args)
{
    bwd_grid_codelet_call(DType::fp16, "nntile_sdpa_bwd_grid_hip_fp16", buffers, cl_args);
}

void nntile_hip_flash_sdpa_bwd_codelet_bf16(void *buffers[], void *cl_args)
{
    bwd_codelet_call(DType::bf16, "nntile_flash_sdpa_bwd_hip_bf16", buffers, cl_args);
}

void nntile_hip_flash_sdpa_bwd_codelet_fp16(void *buffers[], void *cl_args)
{
    bwd_codelet_call(DType::fp16, "nntile_flash_sdpa_bwd_hip_fp16", buffers, cl_args);
}

#define NNTILE_HIP_ROPE_ENTRY(suffix, dt, ctype) \
    int nntile_hip_rope_##suffix(void *stream, int64_t m, int64_t n, const ctype *sin, \
            const ctype *cos, const ctype *src, ctype *dst) \
    { \
        return rope_call(dt, false, stream, m, n, sin, cos, src, dst); \
    } \
    int nntile_hip_rope_backward_##suffix(void *stream, int64_t m, int64_t n, const ctype *sin, \
            const ctype *cos, const ctype *dy, ctype *dx) \
    { \
        return rope_call(dt, true, stream, m, n, sin, cos, dy, dx); \
    }
NNTILE_HIP_ROPE_ENTRY(bf16, DType::bf16, uint16_t)
NNTILE_HIP_ROPE_ENTRY(fp16, DType::fp16, uint16_t)
NNTILE_HIP_ROPE_ENTRY(fp32, DType::fp32, float)
#undef NNTILE_HIP_ROPE_ENTRY

int nntile_hip_transpose_bf16(void *stream, int64_t m, int64_t n, float alpha,
        const uint16_t *src, uint16_t *dst)
{
    return transpose_call(DType::bf16, stream, m, n, alpha, src, dst);
}

int nntile_hip_transpose_fp16(void *stream, int64_t m, int64_t n, float alpha,
        const uint16_t *src, uint16_t *dst)
{
    return transpose_call(DType::fp16, stream, m, n, alpha, src, dst);
}

int nntile_hip_transpose_fp32(void *stream, int64_t m, int64_t n, float alpha,
        const float *src, float *dst)
{
    return transpose_call(DType::fp32, stream, m, n, alpha, src, dst);
}

int nntile_hip_kv_cache_append_bf16(void *stream, int64_t head, int64_t rows, int64_t entries,
        int64_t capacity, int64_t filled, const uint16_t *k_new, const uint16_t *v_new,
        uint16_t *k_cache, uint16_t *v_cache)
{
    return kv_append_call(2, stream, head, rows, entries, capacity, filled, k_new, v_new,
            k_cache, v_cache);
}

int nntile_hip_kv_cache_append_fp16(void *stream, int64_t head, int64_t rows, int64_t entries,
        int64_t capacity, int64_t filled, const uint16_t *k_new, const uint16_t *v_new,
        uint16_t *k_cache, uint16_t *v_cache)
{
    return kv_append_call(2, stream, head, rows, entries, capacity, filled, k_new, v_new,
            k_cache, v_cache);
}

int nntile_hip_kv_cache_append_fp32(void *stream, int64_t head, int64_t rows, int64_t entries,
        int64_t capacity, int64_t filled, const float *k_new, const float *v_new,
        float *k_cache, float *v_cache)
{
    return kv_append_call(4, stream, head, rows, entries, capacity, filled, k_new, v_new,
            k_cache, v_cache);
}

int nntile_hip_sdpa_fwd_tile_cache_bf16(void *stream, const nntile_hip_sdpa_tile_args *args,
        int64_t capacity)
{
    return args != nullptr && capacity < args->k_seq ? NNTILE_HIP_EINVAL
        : tile_call(DType::bf16, stream, args, capacity);
}

int nntile_hip_sdpa_fwd_tile_cache_fp16(void *stream, const nntile_hip_sdpa_tile_args *args,
        int64_t capacity)
{
    return args != nullptr && capacity < args->k_seq ? NNTILE_HIP_EINVAL
        : tile_call(DType::fp16, stream, args, capacity);
}

int nntile_hip_sdpa_fwd_tile_cache_fp32(void *stream, const nntile_hip_sdpa_tile_args *args,
        int64_t capacity)
{
    return args != nullptr && capacity < args->k_seq ? NNTILE_HIP_EINVAL
        : tile_call(DType::fp32, stream, args, capacity);
}

int nntile_hip_sdpa_fwd_decode_cache_bf16(void *stream, const nntile_hip_sdpa_tile_args *args,
        int64_t capacity, void *workspace, size_t workspace_bytes)
{
    return decode_call(DType::bf16, stream, args, capacity, workspace, workspace_bytes);
}

int nntile_hip_sdpa_fwd_decode_cache_fp16(void *stream, const nntile_hip_sdpa_tile_args *args,
        int64_t capacity, void *workspace, size_t workspace_bytes)
{
    return decode_call(DType::fp16, stream, args, capacity, workspace, workspace_bytes);
}

int nntile_hip_sdpa_fwd_decode_append_cache_bf16(void *stream,
        const nntile_hip_sdpa_tile_args *args, int64_t capacity, const uint16_t *k_new,
        const uint16_t *v_new, int64_t rows_new, void *workspace, size_t workspace_bytes)
{
    return decode_call(DType::bf16, stream, args, capacity, workspace, workspace_bytes, k_new,
            v_new, rows_new);
}

int nntile_hip_sdpa_fwd_decode_append_cache_fp16(void *stream,
        const nntile_hip_sdpa_tile_args *args, int64_t capacity, const uint16_t *k_new,
        const uint16_t *v_new, int64_t rows_new, void *workspace, size_t workspace_bytes)
{
    return decode_call(DType::fp16, stream, args, capacity, workspace, workspace_bytes, k_new,
            v_new, rows_new);
}

int nntile_hip_sdpa_fwd_decode_append_cache_fp32(void *stream,
        const nntile_hip_sdpa_tile_args *args, int64_t capacity, const float *k_new,
        const float *v_new, int64_t rows_new, void *workspace, size_t workspace_bytes)
{
    return decode_fp32_call(stream, args, capacity, workspace, workspace_bytes, k_new, v_new,
            rows_new);
}

int nntile_hip_sdpa_fwd_decode_cache_fp32(void *stream, const nntile_hip_sdpa_tile_args *args,
        int64_t capacity, void *workspace, size_t workspace_bytes)
{
    return decode_fp32_call(stream, args, capacity, workspace, workspace_bytes);
}

int nntile_hip_mask_tile_class_bf16(void *stream, int64_t k_rows, int64_t q_cols,
        const uint16_t *mask, int64_t offset, int32_t *workspace, int32_t *class_out)
{
    return mask_class_call(0, stream, k_rows, q_cols, mask, offset, workspace, class_out);
}

int nntile_hip_mask_tile_class_fp16(void *stream, int64_t k_rows, int64_t q_cols,
        const uint16_t *mask, int64_t offset, int32_t *workspace, int32_t *class_out)
{
    return mask_class_call(1, stream, k_rows, q_cols, mask, offset, workspace, class_out);
}

int nntile_hip_mask_tile_class_fp32(void *stream, int64_t k_rows, int64_t q_cols,
        const float *mask, int64_t offset, int32_t *workspace, int32_t *class_out)
{
    return mask_class_call(2, stream, k_rows, q_cols, mask, offset, workspace, class_out);
}

int nntile_hip_mask_tile_class_bool(void *stream, int64_t k_rows, int64_t q_cols,
        const uint8_t *mask, int64_t offset, int32_t *workspace, int32_t *class_out)
{
    return mask_class_call(3, stream, k_rows, q_cols, mask, offset, workspace, class_out);
}

const char *nntile_hip_sdpa_version(void)
{
    return "nntile_hip_sdpa 0.1 (gfx950)";
}

} // extern "C"
