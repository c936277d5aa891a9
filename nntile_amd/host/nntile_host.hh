// Host-side mirror of the NNTile layers the attention hot path crosses
// (tile -> starpu codelet -> kernel), on a minimal stand-in runtime.
//
// Names, argument order, shape rules and error messages follow the reference:
//   TileTraits / TensorTraits     include/nntile/tile/traits.hh:27-195,
//                                 include/nntile/tensor/traits.hh:23-116
//   starpu::FlashSdpaFwdCudnn     include/nntile/starpu/flash_sdpa_fwd_cudnn.hh:44-145,
//                                 src/starpu/flash_sdpa_fwd_cudnn.cc:37-296
//   tile::flash_sdpa_fwd_cudnn*   src/tile/flash_sdpa_fwd_cudnn.cc:25-213
//   tensor::flash_sdpa_fwd_cudnn* src/tensor/flash_sdpa_fwd_cudnn.cc:23-297
//   starpu::FlashSdpaBwdCudnn     include/nntile/starpu/flash_sdpa_bwd_cudnn.hh:44-187,
//                                 src/starpu/flash_sdpa_bwd_cudnn.cc:31-196
//   tile::flash_sdpa_bwd_cudnn*   src/tile/flash_sdpa_bwd_cudnn.cc:24-151
//   tensor::flash_sdpa_bwd_cudnn* src/tensor/flash_sdpa_bwd_cudnn.cc:22-261
// What differs, on purpose: the codelet carries a HIP body (the C-ABI entry
// point nntile_hip_flash_sdpa_fwd_codelet_<T>) next to the empty CPU list, the
// pack gains fp32, and tensor:: gains flash_sdpa_fwd_hip_async, which merges
// all key tiles of a slab in one launch when the mask is analytic.
//
// The runtime here is NOT StarPU: a Handle is a device allocation, submit()
// runs the codelet body at once on the context's stream (in-order execution
// gives the sequential consistency that StarPU derives from access modes).
#pragma once

#include <array>
#include <atomic>
#include <cstdint>
#include <cstdlib>
#include <functional>
#include <memory>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

#include "../../include/nntile_hip_sdpa.h"

namespace nntile
{

using Index = std::int64_t;     // include/nntile/base_types.hh:45
using Scalar = float;           // include/nntile/base_types.hh:48

// Tile value types: storage only (include/nntile/base_types.hh:241-737).
struct fp32_t { using storage_t = float; static constexpr const char *short_name = "fp32"; };
struct bf16_t { using storage_t = std::uint16_t; static constexpr const char *short_name = "bf16"; };
struct fp16_t { using storage_t = std::uint16_t; static constexpr const char *short_name = "fp16"; };

namespace tile
{

//! Integer properties of a contiguous Fortran-ordered tile
class TileTraits
{
public:
    Index ndim;
    std::vector<Index> shape;
    std::vector<Index> stride;      // stride[0] = 1, stride[i+1] = stride[i]*shape[i]
    Index nelems;
    std::vector<std::array<Index, 2>> matrix_shape;
    explicit TileTraits(const std::vector<Index> &shape_);
    //! Linear offset of an element
    Index index_to_linear(const std::vector<Index> &index) const;
    std::vector<Index> linear_to_index(Index linear) const;
};

} // namespace tile

namespace starpu
{

//! Device allocation standing in for a StarPU variable handle
class Handle
{
    std::shared_ptr<void> mem;
    std::size_t nbytes = 0;
    //! Shared by all copies of the handle: a process-wide unique number taken
    //! when the memory is allocated and again at every write access.  Two
    //! equal stamps of one address mean "same allocation, not written in
    //! between" - what a cache of facts about the contents is keyed on.
    std::shared_ptr<std::atomic<std::uint64_t>> stamp;
public:
    Handle() = default;
    explicit Handle(std::size_t size);      // allocates device memory
    void *get_ptr() const { return mem.get(); }
    std::size_t size() const { return nbytes; }
    //! Blocking copies (the analogue of acquire/release on the host)
    void from_host(const void *src) const;
    void to_host(void *dst) const;
    //! To be called by whoever gives a writer access to the memory (under
    //! StarPU: every acquire or task access in a W or RW mode)
    void mark_written() const;
    std::uint64_t write_stamp() const { return stamp ? stamp->load() : 0; }
    //! The reference's scratch handles are unregistered right after the
    //! submission (src/tile/flash_sdpa_fwd_cudnn.cc:194-195)
    void unregister_submit() { mem.reset(); nbytes = 0; }
};

using VariableHandle = Handle;

//! Scratch memory of the one worker this stand-in has: at least `size` bytes,
//! valid until the next call asks for more.  Under StarPU a STARPU_SCRATCH
//! handle costs a task no allocation (the runtime keeps such buffers per
//! worker); a Handle(size) here would call hipMalloc per task.  All bodies run
//! in order on one stream, so consecutive tasks can share the buffer.
Handle worker_scratch(std::size_t size);

//! Stream every codelet body of this process enqueues on
void *get_local_stream();
void task_wait_for_all();
//! Launches that tensor-level functions made through the C ABI directly
//! (not as codelet tasks) since the start of the process: single tile pairs
//! whose mask tile is open or on the causal rule (the whole-grid calls are
//! tasks of the SdpaFwdGrid / SdpaBwdGrid codelets)
std::int64_t direct_launches();
void count_direct_launch();
//! Milliseconds the stream needs for what `enqueue` puts on it (HIP events
//! around it; blocks until done)
double time_on_stream_ms(const std::function<void()> &enqueue);

//! Wrapper of the attention codelet for one value type
template<typename T> class FlashSdpaFwdCudnn;

template<typename T>
class FlashSdpaFwdCudnn<std::tuple<T>>
{
public:
    std::string name;       // "nntile_flash_sdpa_fwd_cudnn_<type>"
    //! Arguments handed to the body (reference args_t, same leading members)
    struct args_t
    {
        FlashSdpaFwdCudnn<std::tuple<T>> *owner;
        Index seq;
        Index head;
        Index batch;
    };
    FlashSdpaFwdCudnn();
    static std::uint32_t hash_parameters(Index seq, Index head, Index batch);
    //! No CPU implementation, as in the reference
    static constexpr std::array<void (*)(void **, void *), 1> cpu_funcs = {nullptr};
    //! The HIP body, same shape as the reference's cuda(buffers, cl_args)
    static void hip(void *buffers[], void *cl_args) noexcept;
    void submit(Index seq, Index head, Index batch, Handle K, Handle Q,
            Handle mask, Handle logsumexp, Handle V, Handle A,
            Handle scratch_logsumexp, Handle scratch_A);
    //! Number of tasks submitted so far (for tests)
    Index submitted = 0;
};

//! One codelet object per value type, looked up by type
template<typename T> FlashSdpaFwdCudnn<std::tuple<T>> &flash_sdpa_fwd_cudnn();

//! Wrapper of the backward codelet for one value type (bf16, fp16)
template<typename T> class FlashSdpaBwdCudnn;

template<typename T>
class FlashSdpaBwdCudnn<std::tuple<T>>
{
public:
    std::string name;       // "nntile_flash_sdpa_bwd_cudnn_<type>"
    struct args_t
    {
        FlashSdpaBwdCudnn<std::tuple<T>> *owner;
        Index seq;
        Index head;
        Index batch;
    };
    FlashSdpaBwdCudnn();
    static std::uint32_t hash_parameters(Index seq, Index head, Index batch);
    static constexpr std::array<void (*)(void **, void *), 1> cpu_funcs = {nullptr};
    static void hip(void *buffers[], void *cl_args) noexcept;
    //! Handles in the reference's order; dK, dQ, dV are read-write (the
    //! gradients of the tile pair are added), the last three are scratch
    void submit(Index seq, Index head, Index batch, Handle K, Handle Q,
            Handle V, Handle A, Handle dA, Handle mask, Handle logsumexp,
            Handle dK, Handle dQ, Handle dV, Handle scratch_dK,
            Handle scratch_dQ, Handle scratch_dV);
    Index submitted = 0;
};

template<typename T> FlashSdpaBwdCudnn<std::tuple<T>> &flash_sdpa_bwd_cudnn();

//! Codelets of the whole-grid calls: ONE task for all (query tile, key tile)
//! pairs of a group of slabs of the batch grid.  No counterpart object in the
//! reference, which submits a FlashSdpaFwdCudnn / FlashSdpaBwdCudnn task per
//! pair (src/tensor/flash_sdpa_fwd_cudnn.cc:246-274,
//! src/tensor/flash_sdpa_bwd_cudnn.cc:172-247); built like those: a body with
//! the codelet signature, arguments malloc'ed per task and owned by it, the
//! number of handles free (nbuffers = STARPU_VARIABLE_NBUFFERS,
//! src/starpu/codelet.cc:58).  Handles travel tile after tile:
//!   forward : K tiles (R), V tiles (R), Q tiles (R), logsumexp tiles (RW),
//!             A tiles (RW)
//!   backward: K, V, Q, A, dA, logsumexp tiles (R), dK, dQ, dV tiles (RW),
//!             one scratch buffer
template<typename T> class SdpaFwdGrid;

template<typename T>
class SdpaFwdGrid<std::tuple<T>>
{
public:
    std::string name;       // "nntile_sdpa_fwd_grid_hip_<type>"
    //! the reference's args_t members first, then the geometry of the grid
    using args_t = nntile_hip_sdpa_grid_cl_args;
    SdpaFwdGrid();
    static constexpr std::array<void (*)(void **, void *), 1> cpu_funcs = {nullptr};
    static void hip(void *buffers[], void *cl_args) noexcept;
    void submit(const args_t &geometry, const std::vector<Handle> &K,
            const std::vector<Handle> &V, const std::vector<Handle> &Q,
            const std::vector<Handle> &logsumexp, const std::vector<Handle> &A);
    Index submitted = 0;
};

template<typename T> SdpaFwdGrid<std::tuple<T>> &sdpa_fwd_grid();

template<typename T> class SdpaBwdGrid;

template<typename T>
class SdpaBwdGrid<std::tuple<T>>
{
public:
    std::string name;       // "nntile_sdpa_bwd_grid_hip_<type>"
    using args_t = nntile_hip_sdpa_grid_cl_args;
    SdpaBwdGrid();
    static constexpr std::array<void (*)(void **, void *), 1> cpu_funcs = {nullptr};
    static void hip(void *buffers[], void *cl_args) noexcept;
    void submit(const args_t &geometry, const std::vector<Handle> &K,
            const std::vector<Handle> &V, const std::vector<Handle> &Q,
            const std::vector<Handle> &A, const std::vector<Handle> &dA,
            const std::vector<Handle> &logsumexp, const std::vector<Handle> &dK,
            const std::vector<Handle> &dQ, const std::vector<Handle> &dV, Handle scratch);
    Index submitted = 0;
};

template<typename T> SdpaBwdGrid<std::tuple<T>> &sdpa_bwd_grid();

} // namespace starpu

namespace tile
{

template<typename T>
class Tile: public TileTraits, public starpu::Handle
{
public:
    explicit Tile(const std::vector<Index> &shape_):
        TileTraits(shape_),
        starpu::Handle(sizeof(typename T::storage_t) * nelems)
    {
    }
    explicit Tile(const TileTraits &traits):
        TileTraits(traits),
        starpu::Handle(sizeof(typename T::storage_t) * nelems)
    {
    }
};

//! Shape rules of one tile task; throws std::runtime_error
void flash_sdpa_fwd_cudnn_check(const TileTraits &K, const TileTraits &Q,
        const TileTraits &mask, const TileTraits &logsumexp,
        const TileTraits &V, const TileTraits &A);

template<typename T>
void flash_sdpa_fwd_cudnn_async(const Tile<T> &K, const Tile<T> &Q,
        const Tile<T> &mask, const Tile<fp32_t> &logsumexp, const Tile<T> &V,
        const Tile<T> &A);

template<typename T>
void flash_sdpa_fwd_cudnn(const Tile<T> &K, const Tile<T> &Q,
        const Tile<T> &mask, const Tile<fp32_t> &logsumexp, const Tile<T> &V,
        const Tile<T> &A);

//! Shape rules of one backward tile task; throws std::runtime_error
void flash_sdpa_bwd_cudnn_check(const TileTraits &K, const TileTraits &Q,
        const TileTraits &V, const TileTraits &A, const TileTraits &dA,
        const TileTraits &mask, const TileTraits &logsumexp,
        const TileTraits &dK, const TileTraits &dQ, const TileTraits &dV);

//! dK, dQ, dV += gradients of one (query tile, key tile) pair
template<typename T>
void flash_sdpa_bwd_cudnn_async(const Tile<T> &K, const Tile<T> &Q,
        const Tile<T> &V, const Tile<T> &A, const Tile<T> &dA,
        const Tile<T> &mask, const Tile<fp32_t> &logsumexp, const Tile<T> &dK,
        const Tile<T> &dQ, const Tile<T> &dV);

template<typename T>
void flash_sdpa_bwd_cudnn(const Tile<T> &K, const Tile<T> &Q,
        const Tile<T> &V, const Tile<T> &A, const Tile<T> &dA,
        const Tile<T> &mask, const Tile<fp32_t> &logsumexp, const Tile<T> &dK,
        const Tile<T> &dQ, const Tile<T> &dV);

} // namespace tile

namespace tensor
{

class TensorTraits: public tile::TileTraits
{
public:
    std::vector<Index> basetile_shape;
    tile::TileTraits grid;
    std::vector<Index> leftover_shape;
    TensorTraits(const std::vector<Index> &shape_,
            const std::vector<Index> &basetile_shape_);
    std::vector<Index> get_tile_shape(const std::vector<Index> &tile_index) const;
};

template<typename T>
class Tensor: public TensorTraits
{
    std::vector<tile::Tile<T>> tiles;
public:
    Tensor(const std::vector<Index> &shape_, const std::vector<Index> &basetile_shape_);
    const tile::Tile<T> &get_tile(Index linear) const { return tiles.at(linear); }
    const tile::Tile<T> &get_tile(const std::vector<Index> &tile_index) const
    {
        return tiles.at(grid.index_to_linear(tile_index));
    }
    //! Whole-tensor Fortran-ordered host array <-> tiles (blocking)
    void from_array(const typename T::storage_t *src) const;
    void to_array(typename T::storage_t *dst) const;
};

//! Every element of every tile set to val (fill_async of the reference,
//! src/tensor/fill.cc; what the layer does to logsumexp before the forward)
void fill_async(float val, const Tensor<fp32_t> &dst);

//! Shape and tiling rules of the tensor-level operation; throws
void flash_sdpa_fwd_cudnn_check(const TensorTraits &K, const TensorTraits &Q,
        const TensorTraits &mask, const TensorTraits &logsumexp,
        const TensorTraits &V, const TensorTraits &A);

//! The reference's operation with the reference's arguments
//! (src/tensor/flash_sdpa_fwd_cudnn.cc:210-279).  What it computes is the
//! reference's result; how it is submitted depends on what is known about the
//! mask.  Nothing known (the default): one task per (output tile, key tile)
//! pair with the pair's mask tile, exactly as flash_sdpa_fwd_cudnn_pairs_async
//! - the mask is read by the kernels when they run, so a mask that any task,
//! kernel or copy has rewritten in the meantime is honoured.  Declared constant
//! (flash_sdpa_mask_declare_constant): as the overload that takes the classes -
//! a mask that is the causal rule or hides nothing becomes one task of the
//! whole-grid codelet per group of slabs, otherwise hidden pairs are not
//! submitted, open and causal pairs run without mask memory, the rest (a mask
//! with bias values: every pair) as the reference does.  Never blocks: only
//! the declaration does.
template<typename T>
void flash_sdpa_fwd_cudnn_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &mask, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &V, const Tensor<T> &A);

//! One tile task per (output tile, key tile) pair with the pair's mask tile,
//! in the reference's order, none skipped: the reference's submission
//! literally (src/tensor/flash_sdpa_fwd_cudnn.cc:221-274)
template<typename T>
void flash_sdpa_fwd_cudnn_pairs_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &mask, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &V, const Tensor<T> &A);

//! The caller's statement that the contents of `mask` stay as they are from
//! now on - what a layer says once after it has built its mask (the reference
//! builds it at construction and never writes it again:
//! wrappers/python/nntile/model/gpt2_attention.py:72-87).  BLOCKING: the
//! mask's tiles are classified against the rule key <= query + causal_offset
//! (one pass over the mask, one word per tile read back) and the classes are
//! kept with the tiles' handles until flash_sdpa_mask_forget, until this
//! runtime hands a tile to a writer (Handle::mark_written), or until the
//! memory is freed.  The contract is the caller's: whoever rewrites a declared
//! mask by means this runtime does not see (a kernel or copy of its own on
//! get_ptr()) must call flash_sdpa_mask_forget first, exactly as it would have
//! to tell StarPU about such a write.  Under StarPU the entry is keyed on the
//! tiles' starpu_data_handle_t and dropped where the tensor unregisters or
//! invalidates them (include/nntile/starpu/handle.hh: unregister,
//! invalidate_submit).
template<typename T>
void flash_sdpa_mask_declare_constant(const Tensor<T> &mask, Index causal_offset = 0);

//! Drops what flash_sdpa_mask_declare_constant stored for this mask
template<typename T>
void flash_sdpa_mask_forget(const Tensor<T> &mask);

//! The classes stored for this mask and offset, if any; never blocks
template<typename T>
bool flash_sdpa_mask_known_classes(const Tensor<T> &mask, Index causal_offset,
        std::vector<int> &classes);

//! Opt-in for callers that cannot add the declaration: with the environment
//! variable NNTILE_HIP_SDPA_CLASSIFY_ON_FIRST_SIGHT set (not "0"), a call with
//! the reference's signature declares an unknown mask constant itself - it
//! BLOCKS on that first call, and foreign writes to the mask go unnoticed.
bool flash_sdpa_classify_on_first_sight();

//! Counters of the store since the start of the process (look-ups that found
//! an entry, look-ups that did not, blocking classifications), and a reset of
//! the store (not of the counters)
struct MaskCacheStats { std::uint64_t hits, misses, classifications; };
MaskCacheStats flash_sdpa_mask_cache_stats();
void flash_sdpa_mask_cache_clear();

template<typename T>
void flash_sdpa_fwd_cudnn(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &mask, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &V, const Tensor<T> &A);

//! Same result with an analytic mask (mask_mode NNTILE_HIP_MASK_NONE or
//! NNTILE_HIP_MASK_CAUSAL with `causal_offset`): for every (batch, group,
//! head) slab all key tiles are merged into all query tiles in ONE launch,
//! and slabs with the same number of entries share a launch as far as its
//! tile tables reach (NNTILE_HIP_SDPA_MAX_TILES tiles per axis).
//! `overwrite` = the running pair need not be initialised by the caller.
//! Returns the number of launches.
template<typename T>
Index flash_sdpa_fwd_hip_async(const Tensor<T> &K, const Tensor<T> &Q,
        int mask_mode, Index causal_offset, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &V, const Tensor<T> &A, bool overwrite);

//! Class (NNTILE_HIP_MASK_TILE_*) of every tile of a materialised mask, in
//! the linear order of mask.grid, against the rule key <= query +
//! causal_offset on global positions.  Blocking; a layer does this once per
//! mask and keeps the result with it.
template<typename T>
std::vector<int> flash_sdpa_mask_classes(const Tensor<T> &mask, Index causal_offset);

//! NNTILE_HIP_MASK_NONE if the classes say the mask hides nothing,
//! NNTILE_HIP_MASK_CAUSAL if they say it is exactly the rule key <= query +
//! causal_offset, -1 otherwise
int flash_sdpa_mask_rule(const TensorTraits &mask, const std::vector<int> &mask_classes,
        Index causal_offset);

//! flash_sdpa_fwd_cudnn_async that uses those classes.  A mask that is the
//! causal rule itself (or hides nothing) runs as flash_sdpa_fwd_hip_async.
//! Otherwise, per pair: a mask tile
//! that hides everything - nothing submitted; one that hides nothing - no
//! mask; one on the causal rule - the analytic mask; the rest as in the
//! reference.  Returns the number of launches.
template<typename T>
Index flash_sdpa_fwd_cudnn_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &mask, const std::vector<int> &mask_classes,
        Index causal_offset, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &V, const Tensor<T> &A);

//! Shape and tiling rules of the tensor-level backward; throws
void flash_sdpa_bwd_cudnn_check(const TensorTraits &K, const TensorTraits &Q,
        const TensorTraits &V, const TensorTraits &A, const TensorTraits &dA,
        const TensorTraits &mask, const TensorTraits &logsumexp,
        const TensorTraits &dK, const TensorTraits &dQ, const TensorTraits &dV);

//! The reference's operation with the reference's arguments
//! (src/tensor/flash_sdpa_bwd_cudnn.cc:172-247); a mask declared constant is
//! submitted through the classes of its tiles like the forward (hidden pairs
//! not submitted, open and causal pairs without mask memory, the rest as the
//! reference does), any other mask pair by pair as the reference does
template<typename T>
void flash_sdpa_bwd_cudnn_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &V, const Tensor<T> &A, const Tensor<T> &dA,
        const Tensor<T> &mask, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &dK, const Tensor<T> &dQ, const Tensor<T> &dV);

//! One tile task per (dQ tile, key tile) pair, in the reference's order, none
//! skipped: the reference's submission literally
template<typename T>
void flash_sdpa_bwd_cudnn_pairs_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &V, const Tensor<T> &A, const Tensor<T> &dA,
        const Tensor<T> &mask, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &dK, const Tensor<T> &dQ, const Tensor<T> &dV);

template<typename T>
void flash_sdpa_bwd_cudnn(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &V, const Tensor<T> &A, const Tensor<T> &dA,
        const Tensor<T> &mask, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &dK, const Tensor<T> &dQ, const Tensor<T> &dV);

//! Same gradients with an analytic mask (NNTILE_HIP_MASK_NONE, or
//! NNTILE_HIP_MASK_CAUSAL with `causal_offset`): no mask tensor.  Where the
//! sequence tiles are multiples of 128 rows (or an axis is one tile) and at
//! most NNTILE_HIP_SDPA_BWD_MAX_TILES an axis, one call per slab of the batch
//! grid takes all its tile pairs; otherwise one call per (dQ tile, key tile)
//! pair with the pair's positions, and pairs that a causal mask hides
//! completely are not submitted.  Gradients are added.  Returns the number
//! of calls made (slabs, or tile pairs).
template<typename T>
Index flash_sdpa_bwd_hip_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &V, const Tensor<T> &A, const Tensor<T> &dA,
        int mask_mode, Index causal_offset, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &dK, const Tensor<T> &dQ, const Tensor<T> &dV);

//! flash_sdpa_bwd_cudnn_async that uses the classes of the mask's tiles
//! (flash_sdpa_mask_classes): no call for a pair whose mask tile hides
//! everything, analytic masks for open and causal ones, the reference's tile
//! operation for the rest; a mask whose classes say it is the causal rule
//! itself (or hides nothing) goes the way of flash_sdpa_bwd_hip_async.
//! Gradients are added.  Returns the calls made (tile pairs, or slabs).
template<typename T>
Index flash_sdpa_bwd_cudnn_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &V, const Tensor<T> &A, const Tensor<T> &dA,
        const Tensor<T> &mask, const std::vector<int> &mask_classes,
        Index causal_offset, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &dK, const Tensor<T> &dQ, const Tensor<T> &dV);

} // namespace tensor

} // namespace nntile
