// Appending the keys and values of new tokens to a preallocated cache
// (wrappers/python/nntile/layer/cache_utils.py:146-175 does this with two
// copy_intersection_async calls, then copies the filled part of both caches
// out again, :177-215, because its attention needs dense operands).
//
// The caches are [head, capacity, n_batch, n_head_kv] (Fortran order): entry
// e of the flattened batch owns capacity*head elements, of which the first
// `filled` rows hold tokens.  The new rows, [head, rows, n_batch, n_head_kv],
// go to rows filled .. filled+rows-1 of every entry, for K and V in ONE
// launch (blockIdx.y picks the tensor).  Pure copy: 16-byte pieces where row
// bytes and addresses allow it, elements otherwise.  The decode entry point
// that takes the capacity then reads the cache where it lies.
#include "sdpa_common.hpp"

namespace nntile_hip
{

struct KvAppendParams
{
    const char *src[2];
    char *dst[2];
    int64_t row_bytes;      // head * sizeof(T)
    int64_t rows;           // new tokens
    int64_t capacity;       // rows per entry of the cache
    int64_t filled;         // rows already in the cache
    int64_t pieces;         // per tensor: entries * rows * (row_bytes / PIECE)
};

template<int PIECE>
__global__ __launch_bounds__(256)
void kv_cache_append_kernel(KvAppendParams p)
{
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if(t >= p.pieces)
    {
        return;
    }
    const int which = blockIdx.y;
    const int64_t per_row = p.row_bytes / PIECE;
    const int64_t row = t / per_row;                // entry * rows + token
    const int64_t in_row = (t - row * per_row) * PIECE;
    const int64_t entry = row / p.rows;
    const int64_t token = row - entry * p.rows;
    const char *s = p.src[which] + row * p.row_bytes + in_row;
    char *d = p.dst[which] + (entry * p.capacity + p.filled + token) * p.row_bytes + in_row;
    if constexpr(PIECE == 16)
    {
        *reinterpret_cast<u32x4 *>(d) = __builtin_nontemporal_load(
                reinterpret_cast<const u32x4 *>(s));
    }
    else if constexpr(PIECE == 4)
    {
        *reinterpret_cast<uint32_t *>(d) = *reinterpret_cast<const uint32_t *>(s);
    }
    else
    {
        *reinterpret_cast<uint16_t *>(d) = *reinterpret_cast<const uint16_t *>(s);
    }
}

// elem: bytes per element (2 or 4)
int launch_kv_cache_append(hipStream_t stream, int elem, int64_t head, int64_t rows,
        int64_t entries, int64_t capacity, int64_t filled, const void *k_new,
        const void *v_new, void *k_cache, void *v_cache)
{
    KvAppendParams p;
    p.src[0] = static_cast<const char *>(k_new);
    p.src[1] = static_cast<const char *>(v_new);
    p.dst[0] = static_cast<char *>(k_cache);
    p.dst[1] = static_cast<char *>(v_cache);
    p.row_bytes = head * elem;
    p.rows = rows;
    p.capacity = capacity;
    p.filled = filled;
    auto aligned = [](const void *q, uintptr_t a)
    {
        return (reinterpret_cast<uintptr_t>(q) & (a - 1)) == 0;
    };
    int piece = elem;
    if(p.row_bytes % 16 == 0 && aligned(k_new, 16) && aligned(v_new, 16)
            && aligned(k_cache, 16) && aligned(v_cache, 16))
    {
        piece = 16;
    }
    p.pieces = entries * rows * (p.row_bytes / piece);
    const int64_t blocks = (p.pieces + 255) / 256;
    if(blocks > 0x7fffffff)
    {
        return NNTILE_HIP_EINVAL;
    }
    const dim3 grid((unsigned)blocks, 2);
    if(piece == 16)
    {
        hipLaunchKernelGGL(kv_cache_append_kernel<16>, grid, dim3(256), 0, stream, p);
    }
    else if(piece == 4)
    {
        hipLaunchKernelGGL(kv_cache_append_kernel<4>, grid, dim3(256), 0, stream, p);
    }
    else
    {
        hipLaunchKernelGGL(kv_cache_append_kernel<2>, grid, dim3(256), 0, stream, p);
    }
    return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
}

} // namespace nntile_hip
