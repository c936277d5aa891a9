// Implementation of the host-side mirror (see nntile_host.hh).
#include "nntile_host.hh"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>
#include <iostream>
#include <mutex>

namespace nntile
{

// ---------------------------------------------------------------------------
// TileTraits: include/nntile/tile/traits.hh:27-195
// ---------------------------------------------------------------------------
namespace tile
{

static std::vector<Index> checked_shape(const std::vector<Index> &shape)
{
    for(Index s : shape)
    {
        if(s <= 0)
        {
            throw std::runtime_error("shape[i] <= 0");
        }
    }
    return shape;
}

TileTraits::TileTraits(const std::vector<Index> &shape_):
    ndim(static_cast<Index>(shape_.size())),
    shape(checked_shape(shape_)),
    stride(ndim),
    matrix_shape(ndim + 1)
{
    Index rows = 1;
    matrix_shape[0][0] = 1;
    for(Index i = 1; i <= ndim; ++i)
    {
        rows *= shape[i-1];
        matrix_shape[i][0] = rows;
    }
    nelems = rows;
    Index cols = 1;
    matrix_shape[ndim][1] = 1;
    for(Index i = ndim; i >= 1; --i)
    {
        cols *= shape[i-1];
        matrix_shape[i-1][1] = cols;
    }
    for(Index i = 0; i < ndim; ++i)
    {
        stride[i] = matrix_shape[i][0];
    }
}

Index TileTraits::index_to_linear(const std::vector<Index> &index) const
{
    if(static_cast<Index>(index.size()) != ndim)
    {
        throw std::runtime_error("Wrong dimensionality");
    }
    Index linear = 0;
    for(Index i = 0; i < ndim; ++i)
    {
        if(index[i] < 0 || index[i] >= shape[i])
        {
            throw std::runtime_error("Index out of bounds");
        }
        linear += index[i] * stride[i];
    }
    return linear;
}

std::vector<Index> TileTraits::linear_to_index(Index linear) const
{
    if(linear < 0 || linear >= nelems)
    {
        throw std::runtime_error("Index out of bounds");
    }
    std::vector<Index> index(ndim);
    for(Index i = 0; i < ndim; ++i)
    {
        index[i] = linear % shape[i];
        linear /= shape[i];
    }
    return index;
}

} // namespace tile

// ---------------------------------------------------------------------------
// Stand-in runtime
// ---------------------------------------------------------------------------
namespace starpu
{

static void hip_check(hipError_t err, const char *what)
{
    if(err != hipSuccess)
    {
        throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(err));
    }
}

void *get_local_stream()
{
    static hipStream_t stream = nullptr;
    static std::once_flag once;
    std::call_once(once, []()
    {
        hip_check(hipStreamCreate(&stream), "hipStreamCreate");
        // the C-ABI codelet bodies ask this function for their stream, as they
        // would ask starpu_hip_get_local_stream() under StarPU
        nntile_hip_set_stream_provider(&get_local_stream);
    });
    return stream;
}

void task_wait_for_all()
{
    hip_check(hipStreamSynchronize(static_cast<hipStream_t>(get_local_stream())),
            "hipStreamSynchronize");
}

static std::uint64_t next_stamp()
{
    static std::atomic<std::uint64_t> counter{0};
    return ++counter;
}

static std::atomic<std::int64_t> direct_launch_counter{0};

std::int64_t direct_launches()
{
    return direct_launch_counter.load();
}

void count_direct_launch()
{
    ++direct_launch_counter;
}

double time_on_stream_ms(const std::function<void()> &enqueue)
{
    hipStream_t stream = static_cast<hipStream_t>(get_local_stream());
    hipEvent_t e0, e1;
    hip_check(hipEventCreate(&e0), "hipEventCreate");
    hip_check(hipEventCreate(&e1), "hipEventCreate");
    hip_check(hipEventRecord(e0, stream), "hipEventRecord");
    enqueue();
    hip_check(hipEventRecord(e1, stream), "hipEventRecord");
    hip_check(hipEventSynchronize(e1), "hipEventSynchronize");
    float ms = 0.0f;
    hip_check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return ms;
}

Handle::Handle(std::size_t size): nbytes(size)
{
    void *ptr = nullptr;
    hip_check(hipMalloc(&ptr, size > 0 ? size : 1), "hipMalloc");
    mem = std::shared_ptr<void>(ptr, [](void *p) { (void)hipFree(p); });
    stamp = std::make_shared<std::atomic<std::uint64_t>>(next_stamp());
}

Handle worker_scratch(std::size_t size)
{
    static std::mutex guard;
    static Handle buffer;
    std::lock_guard<std::mutex> lock(guard);
    if(buffer.size() < size)
    {
        // tasks already enqueued may still use the old buffer
        task_wait_for_all();
        buffer = Handle(size < (std::size_t(1) << 20) ? (std::size_t(1) << 20) : size);
    }
    return buffer;
}

void Handle::mark_written() const
{
    if(stamp)
    {
        stamp->store(next_stamp());
    }
}

void Handle::from_host(const void *src) const
{
    task_wait_for_all();
    mark_written();
    hip_check(hipMemcpy(mem.get(), src, nbytes, hipMemcpyHostToDevice), "hipMemcpy");
}

void Handle::to_host(void *dst) const
{
    task_wait_for_all();
    hip_check(hipMemcpy(dst, mem.get(), nbytes, hipMemcpyDeviceToHost), "hipMemcpy");
}

// CRC32C, most significant bit first, one byte at a time: the recurrence of
// StarPU's starpu_hash_crc32c_be_n, which the reference uses to key the
// codelet's performance model (src/starpu/flash_sdpa_fwd_cudnn.cc:159-168).
// StarPU is not available to compare values with; only the property the
// reference relies on (equal sizes <=> equal footprint, with overwhelming
// probability) is tested.
static std::uint32_t crc32c_be_n(const void *input, std::size_t n, std::uint32_t crc)
{
    const auto *p = static_cast<const std::uint8_t *>(input);
    for(std::size_t i = 0; i < n; ++i)
    {
        crc ^= static_cast<std::uint32_t>(p[i]) << 24;
        for(int bit = 0; bit < 8; ++bit)
        {
            crc = (crc << 1) ^ ((crc & 0x80000000u) ? 0x1EDC6F41u : 0u);
        }
    }
    return crc;
}

template<typename T>
FlashSdpaFwdCudnn<std::tuple<T>>::FlashSdpaFwdCudnn():
    name(std::string("nntile_flash_sdpa_fwd_cudnn_") + T::short_name)
{
}

template<typename T>
std::uint32_t FlashSdpaFwdCudnn<std::tuple<T>>::hash_parameters(Index seq,
        Index head, Index batch)
{
    std::uint32_t hash = 0;
    hash = crc32c_be_n(&seq, sizeof(seq), hash);
    hash = crc32c_be_n(&head, sizeof(head), hash);
    hash = crc32c_be_n(&batch, sizeof(batch), hash);
    return hash;
}

template<> void FlashSdpaFwdCudnn<std::tuple<bf16_t>>::hip(void *buffers[], void *cl_args) noexcept
{
    nntile_hip_flash_sdpa_fwd_codelet_bf16(buffers, cl_args);
}

template<> void FlashSdpaFwdCudnn<std::tuple<fp16_t>>::hip(void *buffers[], void *cl_args) noexcept
{
    nntile_hip_flash_sdpa_fwd_codelet_fp16(buffers, cl_args);
}

template<> void FlashSdpaFwdCudnn<std::tuple<fp32_t>>::hip(void *buffers[], void *cl_args) noexcept
{
    nntile_hip_flash_sdpa_fwd_codelet_fp32(buffers, cl_args);
}

template<typename T>
void FlashSdpaFwdCudnn<std::tuple<T>>::submit(Index seq, Index head, Index batch,
        Handle K, Handle Q, Handle mask, Handle logsumexp, Handle V, Handle A,
        Handle scratch_logsumexp, Handle scratch_A)
{
    // Codelet arguments: malloc'ed and owned by the task, as in the reference
    // (src/starpu/flash_sdpa_fwd_cudnn.cc:186-204)
    auto *args = static_cast<args_t *>(std::malloc(sizeof(args_t)));
    if(args == nullptr)
    {
        throw std::runtime_error("Error in flash_sdpa_fwd_cudnn task submission");
    }
    args->owner = this;
    args->seq = seq;
    args->head = head;
    args->batch = batch;
    // Buffer order and access modes of the reference:
    //   K(R) Q(R) mask(R) logsumexp(RW) V(R) A(RW) scratch_logsumexp(SCRATCH) scratch_A(SCRATCH)
    const Handle *handles[8] = {&K, &Q, &mask, &logsumexp, &V, &A,
        &scratch_logsumexp, &scratch_A};
    nntile_hip_variable_interface ifs[8];
    void *buffers[8];
    for(int i = 0; i < 8; ++i)
    {
        ifs[i].id = 2;      // STARPU_VARIABLE_INTERFACE_ID
        ifs[i].ptr = reinterpret_cast<std::uintptr_t>(handles[i]->get_ptr());
        ifs[i].dev_handle = ifs[i].ptr;
        ifs[i].offset = 0;
        ifs[i].elemsize = handles[i]->size();
        buffers[i] = &ifs[i];
    }
    (void)get_local_stream();       // makes sure the provider is registered
    logsumexp.mark_written();       // the RW buffers
    A.mark_written();
    // "Task execution": the body only enqueues on the stream; the stream's
    // order is the order of submission.
    hip(buffers, args);
    std::free(args);
    ++submitted;
}

template<typename T> FlashSdpaFwdCudnn<std::tuple<T>> &flash_sdpa_fwd_cudnn()
{
    static FlashSdpaFwdCudnn<std::tuple<T>> codelet;
    return codelet;
}

template class FlashSdpaFwdCudnn<std::tuple<bf16_t>>;
template class FlashSdpaFwdCudnn<std::tuple<fp16_t>>;
template class FlashSdpaFwdCudnn<std::tuple<fp32_t>>;
template FlashSdpaFwdCudnn<std::tuple<bf16_t>> &flash_sdpa_fwd_cudnn<bf16_t>();
template FlashSdpaFwdCudnn<std::tuple<fp16_t>> &flash_sdpa_fwd_cudnn<fp16_t>();
template FlashSdpaFwdCudnn<std::tuple<fp32_t>> &flash_sdpa_fwd_cudnn<fp32_t>();

// ---- backward codelet: src/starpu/flash_sdpa_bwd_cudnn.cc:31-196 ----------

template<typename T>
FlashSdpaBwdCudnn<std::tuple<T>>::FlashSdpaBwdCudnn():
    name(std::string("nntile_flash_sdpa_bwd_cudnn_") + T::short_name)
{
}

template<typename T>
std::uint32_t FlashSdpaBwdCudnn<std::tuple<T>>::hash_parameters(Index seq,
        Index head, Index batch)
{
    std::uint32_t hash = 0;
    hash = crc32c_be_n(&seq, sizeof(seq), hash);
    hash = crc32c_be_n(&head, sizeof(head), hash);
    hash = crc32c_be_n(&batch, sizeof(batch), hash);
    return hash;
}

template<> void FlashSdpaBwdCudnn<std::tuple<bf16_t>>::hip(void *buffers[], void *cl_args) noexcept
{
    nntile_hip_flash_sdpa_bwd_codelet_bf16(buffers, cl_args);
}

template<> void FlashSdpaBwdCudnn<std::tuple<fp16_t>>::hip(void *buffers[], void *cl_args) noexcept
{
    nntile_hip_flash_sdpa_bwd_codelet_fp16(buffers, cl_args);
}

template<typename T>
void FlashSdpaBwdCudnn<std::tuple<T>>::submit(Index seq, Index head, Index batch,
        Handle K, Handle Q, Handle V, Handle A, Handle dA, Handle mask,
        Handle logsumexp, Handle dK, Handle dQ, Handle dV, Handle scratch_dK,
        Handle scratch_dQ, Handle scratch_dV)
{
    auto *args = static_cast<args_t *>(std::malloc(sizeof(args_t)));
    if(args == nullptr)
    {
        throw std::runtime_error("Error in flash_sdpa_bwd_cudnn task submission");
    }
    args->owner = this;
    args->seq = seq;
    args->head = head;
    args->batch = batch;
    // Buffer order and access modes of the reference
    // (src/starpu/flash_sdpa_bwd_cudnn.cc:175-187):
    //   K Q V A dA mask logsumexp (R), dK dQ dV (RW), three scratch buffers
    const Handle *handles[13] = {&K, &Q, &V, &A, &dA, &mask, &logsumexp, &dK,
        &dQ, &dV, &scratch_dK, &scratch_dQ, &scratch_dV};
    nntile_hip_variable_interface ifs[13];
    void *buffers[13];
    for(int i = 0; i < 13; ++i)
    {
        ifs[i].id = 2;      // STARPU_VARIABLE_INTERFACE_ID
        ifs[i].ptr = reinterpret_cast<std::uintptr_t>(handles[i]->get_ptr());
        ifs[i].dev_handle = ifs[i].ptr;
        ifs[i].offset = 0;
        ifs[i].elemsize = handles[i]->size();
        buffers[i] = &ifs[i];
    }
    (void)get_local_stream();
    dK.mark_written();              // the RW buffers
    dQ.mark_written();
    dV.mark_written();
    hip(buffers, args);
    std::free(args);
    ++submitted;
}

template<typename T> FlashSdpaBwdCudnn<std::tuple<T>> &flash_sdpa_bwd_cudnn()
{
    static FlashSdpaBwdCudnn<std::tuple<T>> codelet;
    return codelet;
}

template class FlashSdpaBwdCudnn<std::tuple<bf16_t>>;
template class FlashSdpaBwdCudnn<std::tuple<fp16_t>>;
template FlashSdpaBwdCudnn<std::tuple<bf16_t>> &flash_sdpa_bwd_cudnn<bf16_t>();
template FlashSdpaBwdCudnn<std::tuple<fp16_t>> &flash_sdpa_bwd_cudnn<fp16_t>();

// ---- codelets of the whole-grid calls ------------------------------------------

// "Task execution" of a codelet with a free number of handles: look-alike
// variable interfaces in the order given, the body called at once on the
// context's stream (it only enqueues).
static void run_body(void (*body)(void **, void *),
        const std::vector<const Handle *> &handles, void *args)
{
    std::vector<nntile_hip_variable_interface> ifs(handles.size());
    std::vector<void *> buffers(handles.size());
    for(std::size_t i = 0; i < handles.size(); ++i)
    {
        ifs[i].id = 2;      // STARPU_VARIABLE_INTERFACE_ID
        ifs[i].ptr = reinterpret_cast<std::uintptr_t>(handles[i]->get_ptr());
        ifs[i].dev_handle = ifs[i].ptr;
        ifs[i].offset = 0;
        ifs[i].elemsize = handles[i]->size();
        buffers[i] = &ifs[i];
    }
    (void)get_local_stream();       // makes sure the provider is registered
    body(buffers.data(), args);
}

static void check_tile_counts(const nntile_hip_sdpa_grid_cl_args &g, std::size_t n_k,
        std::size_t n_q, const char *what)
{
    const std::size_t n_slabs = g.n_slabs > 0 ? static_cast<std::size_t>(g.n_slabs) : 1;
    if(n_k != n_slabs * static_cast<std::size_t>(g.n_kv_tiles)
            || n_q != n_slabs * static_cast<std::size_t>(g.n_q_tiles))
    {
        throw std::runtime_error(std::string("Error in ") + what
                + " task submission: handle counts do not match the tile grid");
    }
}

template<typename T>
SdpaFwdGrid<std::tuple<T>>::SdpaFwdGrid():
    name(std::string("nntile_sdpa_fwd_grid_hip_") + T::short_name)
{
}

template<> void SdpaFwdGrid<std::tuple<bf16_t>>::hip(void *buffers[], void *cl_args) noexcept
{
    nntile_hip_sdpa_fwd_grid_codelet_bf16(buffers, cl_args);
}

template<> void SdpaFwdGrid<std::tuple<fp16_t>>::hip(void *buffers[], void *cl_args) noexcept
{
    nntile_hip_sdpa_fwd_grid_codelet_fp16(buffers, cl_args);
}

template<> void SdpaFwdGrid<std::tuple<fp32_t>>::hip(void *buffers[], void *cl_args) noexcept
{
    nntile_hip_sdpa_fwd_grid_codelet_fp32(buffers, cl_args);
}

template<typename T>
void SdpaFwdGrid<std::tuple<T>>::submit(const args_t &geometry,
        const std::vector<Handle> &K, const std::vector<Handle> &V,
        const std::vector<Handle> &Q, const std::vector<Handle> &logsumexp,
        const std::vector<Handle> &A)
{
    check_tile_counts(geometry, K.size(), Q.size(), "sdpa_fwd_grid");
    if(V.size() != K.size() || logsumexp.size() != Q.size() || A.size() != Q.size())
    {
        throw std::runtime_error("Error in sdpa_fwd_grid task submission: handle counts differ");
    }
    // arguments malloc'ed and owned by the task, as in the reference
    auto *args = static_cast<args_t *>(std::malloc(sizeof(args_t)));
    if(args == nullptr)
    {
        throw std::runtime_error("Error in sdpa_fwd_grid task submission");
    }
    *args = geometry;
    args->owner = this;
    std::vector<const Handle *> handles;
    handles.reserve(2 * K.size() + 3 * Q.size());
    for(const auto &h : K) { handles.push_back(&h); }              // R
    for(const auto &h : V) { handles.push_back(&h); }              // R
    for(const auto &h : Q) { handles.push_back(&h); }              // R
    for(const auto &h : logsumexp) { handles.push_back(&h); h.mark_written(); }    // RW
    for(const auto &h : A) { handles.push_back(&h); h.mark_written(); }            // RW
    run_body(&hip, handles, args);
    std::free(args);
    ++submitted;
}

template<typename T> SdpaFwdGrid<std::tuple<T>> &sdpa_fwd_grid()
{
    static SdpaFwdGrid<std::tuple<T>> codelet;
    return codelet;
}

template class SdpaFwdGrid<std::tuple<bf16_t>>;
template class SdpaFwdGrid<std::tuple<fp16_t>>;
template class SdpaFwdGrid<std::tuple<fp32_t>>;
template SdpaFwdGrid<std::tuple<bf16_t>> &sdpa_fwd_grid<bf16_t>();
template SdpaFwdGrid<std::tuple<fp16_t>> &sdpa_fwd_grid<fp16_t>();
template SdpaFwdGrid<std::tuple<fp32_t>> &sdpa_fwd_grid<fp32_t>();

template<typename T>
SdpaBwdGrid<std::tuple<T>>::SdpaBwdGrid():
    name(std::string("nntile_sdpa_bwd_grid_hip_") + T::short_name)
{
}

template<> void SdpaBwdGrid<std::tuple<bf16_t>>::hip(void *buffers[], void *cl_args) noexcept
{
    nntile_hip_sdpa_bwd_grid_codelet_bf16(buffers, cl_args);
}

template<> void SdpaBwdGrid<std::tuple<fp16_t>>::hip(void *buffers[], void *cl_args) noexcept
{
    nntile_hip_sdpa_bwd_grid_codelet_fp16(buffers, cl_args);
}

template<typename T>
void SdpaBwdGrid<std::tuple<T>>::submit(const args_t &geometry,
        const std::vector<Handle> &K, const std::vector<Handle> &V,
        const std::vector<Handle> &Q, const std::vector<Handle> &A,
        const std::vector<Handle> &dA, const std::vector<Handle> &logsumexp,
        const std::vector<Handle> &dK, const std::vector<Handle> &dQ,
        const std::vector<Handle> &dV, Handle scratch)
{
    check_tile_counts(geometry, K.size(), Q.size(), "sdpa_bwd_grid");
    if(V.size() != K.size() || dK.size() != K.size() || dV.size() != K.size()
            || A.size() != Q.size() || dA.size() != Q.size() || logsumexp.size() != Q.size()
            || dQ.size() != Q.size())
    {
        throw std::runtime_error("Error in sdpa_bwd_grid task submission: handle counts differ");
    }
    auto *args = static_cast<args_t *>(std::malloc(sizeof(args_t)));
    if(args == nullptr)
    {
        throw std::runtime_error("Error in sdpa_bwd_grid task submission");
    }
    *args = geometry;
    args->owner = this;
    std::vector<const Handle *> handles;
    handles.reserve(4 * K.size() + 5 * Q.size() + 1);
    for(const auto *group : {&K, &V, &Q, &A, &dA, &logsumexp})     // R
    {
        for(const auto &h : *group) { handles.push_back(&h); }
    }
    for(const auto *group : {&dK, &dQ, &dV})                        // RW
    {
        for(const auto &h : *group) { handles.push_back(&h); h.mark_written(); }
    }
    handles.push_back(&scratch);                                     // SCRATCH
    run_body(&hip, handles, args);
    std::free(args);
    ++submitted;
}

template<typename T> SdpaBwdGrid<std::tuple<T>> &sdpa_bwd_grid()
{
    static SdpaBwdGrid<std::tuple<T>> codelet;
    return codelet;
}

template class SdpaBwdGrid<std::tuple<bf16_t>>;
template class SdpaBwdGrid<std::tuple<fp16_t>>;
template SdpaBwdGrid<std::tuple<bf16_t>> &sdpa_bwd_grid<bf16_t>();
template SdpaBwdGrid<std::tuple<fp16_t>> &sdpa_bwd_grid<fp16_t>();

} // namespace starpu

// ---------------------------------------------------------------------------
// tile level: src/tile/flash_sdpa_fwd_cudnn.cc:25-213
// ---------------------------------------------------------------------------
namespace tile
{

static void require(bool ok, const char *message)
{
    if(!ok)
    {
        throw std::runtime_error(message);
    }
}

void flash_sdpa_fwd_cudnn_check(const TileTraits &K, const TileTraits &Q,
        const TileTraits &mask, const TileTraits &logsumexp,
        const TileTraits &V, const TileTraits &A)
{
    // K/Q/V/A are 5-D [head_size, n_seq, n_batch, kv_group_size, n_head_kv],
    // mask is 2-D [n_seq, n_seq], logsumexp is 4-D (the same minus head_size)
    require(K.ndim == 5, "K.ndim != 5");
    require(Q.ndim == 5, "Q.ndim != 5");
    require(V.ndim == 5, "V.ndim != 5");
    require(A.ndim == 5, "A.ndim != 5");
    require(mask.ndim == 2, "mask.ndim != 2");
    require(logsumexp.ndim == 4, "logsumexp.ndim != 4");
    require(K.shape[0] == Q.shape[0], "K.shape[0] != Q.shape[0]");
    require(K.shape[0] == V.shape[0], "K.shape[0] != V.shape[0]");
    require(K.shape[0] == A.shape[0], "K.shape[0] != A.shape[0]");
    require(K.shape[1] == Q.shape[1], "K.shape[1] != Q.shape[1]");
    require(K.shape[1] == V.shape[1], "K.shape[1] != V.shape[1]");
    require(K.shape[1] == A.shape[1], "K.shape[1] != A.shape[1]");
    require(K.shape[1] == mask.shape[0], "K.shape[1] != mask.shape[0]");
    require(K.shape[1] == mask.shape[1], "K.shape[1] != mask.shape[1]");
    require(K.shape[1] == logsumexp.shape[0], "K.shape[1] != logsumexp.shape[0]");
    static const char *const names[3][4] = {
        {"K.shape[2] != Q.shape[2]", "K.shape[2] != V.shape[2]",
            "K.shape[2] != A.shape[2]", "K.shape[2] != logsumexp.shape[1]"},
        {"K.shape[3] != Q.shape[3]", "K.shape[3] != V.shape[3]",
            "K.shape[3] != A.shape[3]", "K.shape[3] != logsumexp.shape[2]"},
        {"K.shape[4] != Q.shape[4]", "K.shape[4] != V.shape[4]",
            "K.shape[4] != A.shape[4]", "K.shape[4] != logsumexp.shape[3]"}};
    for(int d = 2; d < 5; ++d)
    {
        require(K.shape[d] == Q.shape[d], names[d-2][0]);
        require(K.shape[d] == V.shape[d], names[d-2][1]);
        require(K.shape[d] == A.shape[d], names[d-2][2]);
        require(K.shape[d] == logsumexp.shape[d-1], names[d-2][3]);
    }
}

template<typename T>
void flash_sdpa_fwd_cudnn_async(const Tile<T> &K, const Tile<T> &Q,
        const Tile<T> &mask, const Tile<fp32_t> &logsumexp, const Tile<T> &V,
        const Tile<T> &A)
{
    flash_sdpa_fwd_cudnn_check(K, Q, mask, logsumexp, V, A);
    const Index seq = K.shape[1];
    const Index head = K.shape[0];
    // n_batch * kv_group_size * n_head_kv -> one flat batch
    const Index batch = K.shape[2] * K.shape[3] * K.shape[4];
    // The reference registers two scratch handles per call
    // (src/tile/flash_sdpa_fwd_cudnn.cc:176-195).  The HIP body fuses the
    // merge and needs neither for it; it scans a large mask once into the
    // first (seq * batch floats).  The second stays empty.
    starpu::VariableHandle scratch_logsumexp = starpu::worker_scratch(
            sizeof(float) * static_cast<std::size_t>(seq) * static_cast<std::size_t>(batch));
    starpu::VariableHandle scratch_A;
    starpu::flash_sdpa_fwd_cudnn<T>().submit(seq, head, batch, K, Q, mask,
            logsumexp, V, A, scratch_logsumexp, scratch_A);
    scratch_logsumexp.unregister_submit();
    scratch_A.unregister_submit();
}

template<typename T>
void flash_sdpa_fwd_cudnn(const Tile<T> &K, const Tile<T> &Q,
        const Tile<T> &mask, const Tile<fp32_t> &logsumexp, const Tile<T> &V,
        const Tile<T> &A)
{
    flash_sdpa_fwd_cudnn_async<T>(K, Q, mask, logsumexp, V, A);
    starpu::task_wait_for_all();
}

#define NNTILE_HOST_INSTANTIATE_TILE(T) \
    template void flash_sdpa_fwd_cudnn_async<T>(const Tile<T> &, const Tile<T> &, \
            const Tile<T> &, const Tile<fp32_t> &, const Tile<T> &, const Tile<T> &); \
    template void flash_sdpa_fwd_cudnn<T>(const Tile<T> &, const Tile<T> &, \
            const Tile<T> &, const Tile<fp32_t> &, const Tile<T> &, const Tile<T> &);
NNTILE_HOST_INSTANTIATE_TILE(bf16_t)
NNTILE_HOST_INSTANTIATE_TILE(fp16_t)
NNTILE_HOST_INSTANTIATE_TILE(fp32_t)

// ---- backward: src/tile/flash_sdpa_bwd_cudnn.cc:24-151 ---------------------

// The ten traits share the rules below at both levels (tile and tensor).
template<typename Traits>
static void bwd_common_check(const Traits &K, const Traits &Q, const Traits &V,
        const Traits &A, const Traits &dA, const Traits &mask,
        const Traits &logsumexp, const Traits &dK, const Traits &dQ,
        const Traits &dV)
{
    const Traits *five[8] = {&K, &Q, &V, &A, &dA, &dK, &dQ, &dV};
    static const char *const names[8] = {"K", "Q", "V", "A", "dA", "dK", "dQ", "dV"};
    for(int i = 0; i < 8; ++i)
    {
        if(five[i]->ndim != 5)
        {
            throw std::runtime_error(std::string(names[i]) + ".ndim != 5");
        }
    }
    require(mask.ndim == 2, "mask.ndim != 2");
    require(logsumexp.ndim == 4, "logsumexp.ndim != 4");
    // every 5-D operand has the shape of K (square tile pairs only)
    for(int i = 1; i < 8; ++i)
    {
        if(K.shape != five[i]->shape)
        {
            throw std::runtime_error(std::string("K.shape != ") + names[i] + ".shape");
        }
    }
    require(K.shape[1] == mask.shape[0] && K.shape[1] == mask.shape[1],
            "Mask shape mismatch");
    require(K.shape[1] == logsumexp.shape[0], "logsumexp axis 0 must match sequence length");
    require(K.shape[2] == logsumexp.shape[1], "logsumexp axis 1 must match batch");
    require(K.shape[3] == logsumexp.shape[2], "logsumexp axis 2 must match kv_group_size");
    require(K.shape[4] == logsumexp.shape[3], "logsumexp axis 3 must match n_head_kv");
}

void flash_sdpa_bwd_cudnn_check(const TileTraits &K, const TileTraits &Q,
        const TileTraits &V, const TileTraits &A, const TileTraits &dA,
        const TileTraits &mask, const TileTraits &logsumexp,
        const TileTraits &dK, const TileTraits &dQ, const TileTraits &dV)
{
    bwd_common_check(K, Q, V, A, dA, mask, logsumexp, dK, dQ, dV);
}

template<typename T>
void flash_sdpa_bwd_cudnn_async(const Tile<T> &K, const Tile<T> &Q,
        const Tile<T> &V, const Tile<T> &A, const Tile<T> &dA,
        const Tile<T> &mask, const Tile<fp32_t> &logsumexp, const Tile<T> &dK,
        const Tile<T> &dQ, const Tile<T> &dV)
{
    flash_sdpa_bwd_cudnn_check(K, Q, V, A, dA, mask, logsumexp, dK, dQ, dV);
    const Index seq = K.shape[1];
    const Index head = K.shape[0];
    const Index batch = K.shape[2] * K.shape[3] * K.shape[4];
    // The reference registers three scratch handles of the size of the
    // gradients.  The HIP body adds into dK, dQ, dV directly and only uses
    // scratch_dQ (for the row dots dA.A and the classes of the mask blocks);
    // the other two stay empty and keep the submit signature.
    starpu::VariableHandle scratch_dK, scratch_dV;
    starpu::VariableHandle scratch_dQ(sizeof(typename T::storage_t) * dQ.nelems);
    starpu::flash_sdpa_bwd_cudnn<T>().submit(seq, head, batch, K, Q, V, A, dA,
            mask, logsumexp, dK, dQ, dV, scratch_dK, scratch_dQ, scratch_dV);
    scratch_dK.unregister_submit();
    scratch_dQ.unregister_submit();
    scratch_dV.unregister_submit();
}

template<typename T>
void flash_sdpa_bwd_cudnn(const Tile<T> &K, const Tile<T> &Q,
        const Tile<T> &V, const Tile<T> &A, const Tile<T> &dA,
        const Tile<T> &mask, const Tile<fp32_t> &logsumexp, const Tile<T> &dK,
        const Tile<T> &dQ, const Tile<T> &dV)
{
    flash_sdpa_bwd_cudnn_async<T>(K, Q, V, A, dA, mask, logsumexp, dK, dQ, dV);
    starpu::task_wait_for_all();
}

#define NNTILE_HOST_INSTANTIATE_TILE_BWD(T) \
    template void flash_sdpa_bwd_cudnn_async<T>(const Tile<T> &, const Tile<T> &, \
            const Tile<T> &, const Tile<T> &, const Tile<T> &, const Tile<T> &, \
            const Tile<fp32_t> &, const Tile<T> &, const Tile<T> &, const Tile<T> &); \
    template void flash_sdpa_bwd_cudnn<T>(const Tile<T> &, const Tile<T> &, \
            const Tile<T> &, const Tile<T> &, const Tile<T> &, const Tile<T> &, \
            const Tile<fp32_t> &, const Tile<T> &, const Tile<T> &, const Tile<T> &);
NNTILE_HOST_INSTANTIATE_TILE_BWD(bf16_t)
NNTILE_HOST_INSTANTIATE_TILE_BWD(fp16_t)

} // namespace tile

// ---------------------------------------------------------------------------
// tensor level: include/nntile/tensor/traits.hh:23-116,
//               src/tensor/flash_sdpa_fwd_cudnn.cc:23-297
// ---------------------------------------------------------------------------
namespace tensor
{

static std::vector<Index> grid_shape_of(const std::vector<Index> &shape,
        const std::vector<Index> &basetile)
{
    if(basetile.size() != shape.size())
    {
        throw std::runtime_error("basetile_shape.size() != ndim");
    }
    std::vector<Index> grid(shape.size());
    for(std::size_t i = 0; i < shape.size(); ++i)
    {
        if(basetile[i] <= 0)
        {
            throw std::runtime_error("basetile_shape[i] <= 0");
        }
        grid[i] = (shape[i] - 1) / basetile[i] + 1;
    }
    return grid;
}

TensorTraits::TensorTraits(const std::vector<Index> &shape_,
        const std::vector<Index> &basetile_shape_):
    tile::TileTraits(shape_),
    basetile_shape(basetile_shape_),
    grid(grid_shape_of(shape, basetile_shape_)),
    leftover_shape(ndim)
{
    for(Index i = 0; i < ndim; ++i)
    {
        leftover_shape[i] = shape[i] - (grid.shape[i] - 1) * basetile_shape[i];
    }
}

std::vector<Index> TensorTraits::get_tile_shape(
        const std::vector<Index> &tile_index) const
{
    if(static_cast<Index>(tile_index.size()) != ndim)
    {
        throw std::runtime_error("Wrong dimensionality");
    }
    std::vector<Index> tile_shape(basetile_shape);
    for(Index i = 0; i < ndim; ++i)
    {
        if(tile_index[i] < 0 || tile_index[i] >= grid.shape[i])
        {
            throw std::runtime_error("Index out of bounds");
        }
        if(grid.shape[i] - tile_index[i] == 1)
        {
            tile_shape[i] = leftover_shape[i];
        }
    }
    return tile_shape;
}

template<typename T>
Tensor<T>::Tensor(const std::vector<Index> &shape_,
        const std::vector<Index> &basetile_shape_):
    TensorTraits(shape_, basetile_shape_)
{
    tiles.reserve(grid.nelems);
    for(Index i = 0; i < grid.nelems; ++i)
    {
        tiles.emplace_back(get_tile_shape(grid.linear_to_index(i)));
    }
}

// Walks the elements of tile `t` in the tile's own (Fortran) order and calls
// f(offset in the tile, offset in the whole tensor).
template<typename F>
static void for_each_tile_element(const TensorTraits &tt,
        const std::vector<Index> &tile_index, const tile::TileTraits &tile, F f)
{
    std::vector<Index> idx(tt.ndim, 0);
    Index base = 0;
    for(Index d = 0; d < tt.ndim; ++d)
    {
        base += tile_index[d] * tt.basetile_shape[d] * tt.stride[d];
    }
    for(Index e = 0; e < tile.nelems; ++e)
    {
        Index global = base;
        for(Index d = 0; d < tt.ndim; ++d)
        {
            global += idx[d] * tt.stride[d];
        }
        f(e, global);
        for(Index d = 0; d < tt.ndim; ++d)
        {
            if(++idx[d] < tile.shape[d])
            {
                break;
            }
            idx[d] = 0;
        }
    }
}

template<typename T>
void Tensor<T>::from_array(const typename T::storage_t *src) const
{
    for(Index i = 0; i < grid.nelems; ++i)
    {
        const auto &t = tiles[i];
        std::vector<typename T::storage_t> buf(t.nelems);
        for_each_tile_element(*this, grid.linear_to_index(i), t,
                [&](Index e, Index g) { buf[e] = src[g]; });
        t.from_host(buf.data());
    }
}

template<typename T>
void Tensor<T>::to_array(typename T::storage_t *dst) const
{
    for(Index i = 0; i < grid.nelems; ++i)
    {
        const auto &t = tiles[i];
        std::vector<typename T::storage_t> buf(t.nelems);
        t.to_host(buf.data());
        for_each_tile_element(*this, grid.linear_to_index(i), t,
                [&](Index e, Index g) { dst[g] = buf[e]; });
    }
}

static void require(bool ok, const char *message)
{
    if(!ok)
    {
        throw std::runtime_error(message);
    }
}

void fill_async(float val, const Tensor<fp32_t> &dst)
{
    std::uint32_t bits;
    std::memcpy(&bits, &val, sizeof(bits));
    for(Index i = 0; i < dst.grid.nelems; ++i)
    {
        const auto &tile = dst.get_tile(i);
        tile.mark_written();
        if(hipMemsetD32Async(reinterpret_cast<hipDeviceptr_t>(tile.get_ptr()),
                    static_cast<int>(bits), static_cast<std::size_t>(tile.nelems),
                    static_cast<hipStream_t>(starpu::get_local_stream())) != hipSuccess)
        {
            throw std::runtime_error("Error in fill_async");
        }
    }
}

void flash_sdpa_fwd_cudnn_check(const TensorTraits &K, const TensorTraits &Q,
        const TensorTraits &mask, const TensorTraits &logsumexp,
        const TensorTraits &V, const TensorTraits &A)
{
    require(K.ndim == 5, "K.ndim != 5");
    require(Q.ndim == 5, "Q.ndim != 5");
    require(V.ndim == 5, "V.ndim != 5");
    require(A.ndim == 5, "A.ndim != 5");
    require(mask.ndim == 2, "mask.ndim != 2");
    require(logsumexp.ndim == 4, "logsumexp.ndim != 4");
    require(K.shape[0] == Q.shape[0], "K.shape[0] != Q.shape[0]");
    require(K.shape[0] == V.shape[0], "K.shape[0] != V.shape[0]");
    require(K.shape[0] == A.shape[0], "K.shape[0] != A.shape[0]");
    require(K.shape[1] == Q.shape[1], "K.shape[1] != Q.shape[1]");
    require(K.shape[1] == V.shape[1], "K.shape[1] != V.shape[1]");
    require(K.shape[1] == A.shape[1], "K.shape[1] != A.shape[1]");
    require(K.shape[1] == mask.shape[0], "K sequence dimension must match mask axis 0");
    require(Q.shape[1] == mask.shape[1], "Q sequence dimension must match mask axis 1");
    require(K.shape[1] == logsumexp.shape[0], "K.shape[1] != logsumexp.shape[0]");
    static const char *const names[3][4] = {
        {"K.shape[2] != Q.shape[2]", "K.shape[2] != V.shape[2]",
            "K.shape[2] != A.shape[2]", "K.shape[2] != logsumexp.shape[1]"},
        {"K.shape[3] != Q.shape[3]", "K.shape[3] != V.shape[3]",
            "K.shape[3] != A.shape[3]", "K.shape[3] != logsumexp.shape[2]"},
        {"K.shape[4] != Q.shape[4]", "K.shape[4] != V.shape[4]",
            "K.shape[4] != A.shape[4]", "K.shape[4] != logsumexp.shape[3]"}};
    for(int d = 2; d < 5; ++d)
    {
        require(K.shape[d] == Q.shape[d], names[d-2][0]);
        require(K.shape[d] == V.shape[d], names[d-2][1]);
        require(K.shape[d] == A.shape[d], names[d-2][2]);
        require(K.shape[d] == logsumexp.shape[d-1], names[d-2][3]);
    }
    // basetile compatibility for multi-tile execution
    const auto &Kb = K.basetile_shape, &Qb = Q.basetile_shape,
          &Vb = V.basetile_shape, &Ab = A.basetile_shape,
          &Mb = mask.basetile_shape, &Lb = logsumexp.basetile_shape;
    require(Qb == Ab, "Q and A basetile shapes must match");
    for(Index d : {Index(0), Index(2), Index(3), Index(4)})
    {
        require(Kb[d] == Qb[d], "K and Q basetile shapes mismatch");
        require(Vb[d] == Qb[d], "V and Q basetile shapes mismatch");
        require(Ab[d] == Qb[d], "A and Q basetile shapes mismatch");
    }
    require(Mb[0] == Kb[1], "mask basetile axis 0 must match K basetile sequence dimension");
    require(Mb[1] == Qb[1], "mask basetile axis 1 must match Q basetile sequence dimension");
    require(Lb[0] == Qb[1] && Lb[1] == Qb[2] && Lb[2] == Qb[3] && Lb[3] == Qb[4],
            "logsumexp basetile shape must match Q basetile shape (excluding head dimension)");
    require(Kb[0] == K.shape[0] && Qb[0] == Q.shape[0] && Vb[0] == V.shape[0]
            && Ab[0] == A.shape[0], "head dimension must not be tiled for K/Q/V/A");
}

template<typename T>
void flash_sdpa_fwd_cudnn_pairs_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &mask, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &V, const Tensor<T> &A)
{
    flash_sdpa_fwd_cudnn_check(K, Q, mask, logsumexp, V, A);
    const Index num_k_seq_tiles = K.grid.shape[1];
    // Output tiles define the Q and logsumexp tiles; every key tile along the
    // sequence axis is merged into each of them, none is skipped
    // (src/tensor/flash_sdpa_fwd_cudnn.cc:221-274)
    for(Index a_linear = 0; a_linear < A.grid.nelems; ++a_linear)
    {
        const auto a_index = A.grid.linear_to_index(a_linear);
        const auto &Q_tile = Q.get_tile(a_linear);
        const auto &A_tile = A.get_tile(a_linear);
        const auto &lse_tile = logsumexp.get_tile(
                {a_index[1], a_index[2], a_index[3], a_index[4]});
        const Index seq_q = Q_tile.shape[1];
        for(Index k_idx = 0; k_idx < num_k_seq_tiles; ++k_idx)
        {
            auto kv_index = a_index;
            kv_index[1] = k_idx;
            const auto &K_tile = K.get_tile(kv_index);
            const auto &V_tile = V.get_tile(kv_index);
            const auto &mask_tile = mask.get_tile({k_idx, a_index[1]});
            require(K_tile.shape[1] == seq_q, "K tile sequence length mismatches Q tile");
            require(mask_tile.shape[0] == K_tile.shape[1] && mask_tile.shape[1] == seq_q,
                    "Mask tile shape mismatches Q/K tiles");
            require(lse_tile.shape[0] == seq_q, "logsumexp tile shape mismatches Q tile");
            tile::flash_sdpa_fwd_cudnn_async<T>(K_tile, Q_tile, mask_tile,
                    lse_tile, V_tile, A_tile);
        }
    }
}

template<typename T>
void flash_sdpa_fwd_cudnn(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &mask, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &V, const Tensor<T> &A)
{
    flash_sdpa_fwd_cudnn_async<T>(K, Q, mask, logsumexp, V, A);
    starpu::task_wait_for_all();
}

// ---- what is known about a mask, kept with its handles ----------------------
// A layer builds its mask once and passes the same tensor to every call
// (wrappers/python/nntile/model/gpt2_attention.py:72-87).  When it says so
// (flash_sdpa_mask_declare_constant, once, after building the mask) the classes
// of the mask's tiles are computed in one blocking pass and kept here; the
// calls with the reference's signature look them up and never block.  An
// entry is dropped by flash_sdpa_mask_forget, and - in this runtime, where
// every write access goes through Handle::mark_written - when a tile is given
// to a writer or its memory is reallocated (Handle::write_stamp); the key is
// the first tile's address.  A mask that was not declared is never looked at
// ahead of time: its pairs are submitted with their mask tiles, as the
// reference does, whatever the tiles hold at that moment.
namespace
{

struct MaskCacheEntry
{
    std::vector<std::pair<const void *, std::uint64_t>> tiles;  // (address, stamp)
    Index causal_offset;
    std::vector<Index> shape, basetile;
    std::vector<int> classes;
};

std::mutex mask_cache_mutex;
std::vector<MaskCacheEntry> mask_cache;         // few masks per process: linear search
std::uint64_t mask_cache_hits = 0, mask_cache_misses = 0, mask_cache_classifications = 0;
constexpr std::size_t kMaskCacheEntries = 64;

} // namespace

MaskCacheStats flash_sdpa_mask_cache_stats()
{
    std::lock_guard<std::mutex> guard(mask_cache_mutex);
    return MaskCacheStats{mask_cache_hits, mask_cache_misses, mask_cache_classifications};
}

void flash_sdpa_mask_cache_clear()
{
    std::lock_guard<std::mutex> guard(mask_cache_mutex);
    mask_cache.clear();
}

template<typename T> struct GridCall;
template<> struct GridCall<bf16_t>
{
    static int run(void *s, const nntile_hip_sdpa_grid_args *a) { return nntile_hip_sdpa_fwd_grid_bf16(s, a); }
};
template<> struct GridCall<fp16_t>
{
    static int run(void *s, const nntile_hip_sdpa_grid_args *a) { return nntile_hip_sdpa_fwd_grid_fp16(s, a); }
};
template<> struct GridCall<fp32_t>
{
    static int run(void *s, const nntile_hip_sdpa_grid_args *a) { return nntile_hip_sdpa_fwd_grid_fp32(s, a); }
};

template<typename T>
Index flash_sdpa_fwd_hip_async(const Tensor<T> &K, const Tensor<T> &Q,
        int mask_mode, Index causal_offset, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &V, const Tensor<T> &A, bool overwrite)
{
    // Same shape rules as the reference operation, with a stand-in for the
    // mask that is no longer materialised.
    const TensorTraits mask({K.shape[1], Q.shape[1]},
            {K.basetile_shape[1], Q.basetile_shape[1]});
    flash_sdpa_fwd_cudnn_check(K, Q, mask, logsumexp, V, A);
    require(mask_mode == NNTILE_HIP_MASK_NONE || mask_mode == NNTILE_HIP_MASK_CAUSAL,
            "flash_sdpa_fwd_hip: mask_mode must be NONE or CAUSAL");
    const Index n_q = Q.grid.shape[1], n_kv = K.grid.shape[1];
    require(n_q <= NNTILE_HIP_SDPA_MAX_TILES && n_kv <= NNTILE_HIP_SDPA_MAX_TILES,
            "flash_sdpa_fwd_hip: too many sequence tiles for one launch");
    // The slabs of the batch grid (each with all its query and key tiles) go
    // into as few launches as the tile tables hold: slabs with the same
    // number of entries share a launch, up to NNTILE_HIP_SDPA_MAX_TILES
    // tiles per axis.
    struct Slab { Index g2, g3, g4, batch; };
    std::vector<Slab> slabs;
    for(Index g4 = 0; g4 < Q.grid.shape[4]; ++g4)
    {
        for(Index g3 = 0; g3 < Q.grid.shape[3]; ++g3)
        {
            for(Index g2 = 0; g2 < Q.grid.shape[2]; ++g2)
            {
                const auto &q0 = Q.get_tile({0, 0, g2, g3, g4});
                slabs.push_back({g2, g3, g4, q0.shape[2] * q0.shape[3] * q0.shape[4]});
            }
        }
    }
    const std::size_t per_launch = static_cast<std::size_t>(
            NNTILE_HIP_SDPA_MAX_TILES / std::max(n_q, n_kv));
    Index launches = 0;
    for(std::size_t first = 0; first < slabs.size();)
    {
        std::size_t count = 1;
        while(first + count < slabs.size() && count < per_launch
                && slabs[first + count].batch == slabs[first].batch)
        {
            ++count;
        }
        // one task of the whole-grid codelet for these slabs
        nntile_hip_sdpa_grid_cl_args a;
        std::memset(&a, 0, sizeof(a));
        a.seq = Q.basetile_shape[1];
        a.head = Q.shape[0];
        a.batch = slabs[first].batch;
        a.q_seq = Q.shape[1];
        a.k_seq = K.shape[1];
        a.q_tile = Q.basetile_shape[1];
        a.k_tile = K.basetile_shape[1];
        a.n_batch = a.batch;
        a.kv_group = 1;
        a.mask_mode = mask_mode;
        a.flags = overwrite ? NNTILE_HIP_SDPA_OVERWRITE : 0;
        a.n_q_tiles = static_cast<std::int32_t>(n_q);
        a.n_kv_tiles = static_cast<std::int32_t>(n_kv);
        a.n_slabs = static_cast<std::int32_t>(count);
        a.causal_offset = causal_offset;
        std::vector<starpu::Handle> Kh, Vh, Qh, Lh, Ah;
        for(std::size_t s = 0; s < count; ++s)
        {
            const Index g2 = slabs[first + s].g2, g3 = slabs[first + s].g3,
                  g4 = slabs[first + s].g4;
            for(Index t = 0; t < n_kv; ++t)
            {
                Kh.push_back(K.get_tile({0, t, g2, g3, g4}));
                Vh.push_back(V.get_tile({0, t, g2, g3, g4}));
            }
            for(Index t = 0; t < n_q; ++t)
            {
                Qh.push_back(Q.get_tile({0, t, g2, g3, g4}));
                Ah.push_back(A.get_tile({0, t, g2, g3, g4}));
                Lh.push_back(logsumexp.get_tile({t, g2, g3, g4}));
            }
        }
        starpu::sdpa_fwd_grid<T>().submit(a, Kh, Vh, Qh, Lh, Ah);
        first += count;
        ++launches;
    }
    return launches;
}

template<typename T> struct TileCall;
template<> struct TileCall<bf16_t>
{
    static int run(void *s, const nntile_hip_sdpa_tile_args *a) { return nntile_hip_sdpa_fwd_tile_bf16(s, a); }
    static int classify(void *s, Index k, Index q, const void *m, Index off, int32_t *ws, int32_t *out)
    {
        return nntile_hip_mask_tile_class_bf16(s, k, q, static_cast<const uint16_t *>(m), off, ws, out);
    }
};
template<> struct TileCall<fp16_t>
{
    static int run(void *s, const nntile_hip_sdpa_tile_args *a) { return nntile_hip_sdpa_fwd_tile_fp16(s, a); }
    static int classify(void *s, Index k, Index q, const void *m, Index off, int32_t *ws, int32_t *out)
    {
        return nntile_hip_mask_tile_class_fp16(s, k, q, static_cast<const uint16_t *>(m), off, ws, out);
    }
};
template<> struct TileCall<fp32_t>
{
    static int run(void *s, const nntile_hip_sdpa_tile_args *a) { return nntile_hip_sdpa_fwd_tile_fp32(s, a); }
    static int classify(void *s, Index k, Index q, const void *m, Index off, int32_t *ws, int32_t *out)
    {
        return nntile_hip_mask_tile_class_fp32(s, k, q, static_cast<const float *>(m), off, ws, out);
    }
};

template<typename T>
std::vector<int> flash_sdpa_mask_classes(const Tensor<T> &mask, Index causal_offset)
{
    require(mask.ndim == 2, "mask must be 2-dimensional");
    std::vector<int> classes(mask.grid.nelems, NNTILE_HIP_MASK_TILE_MIXED);
    starpu::VariableHandle word(sizeof(int32_t));
    for(Index i = 0; i < mask.grid.nelems; ++i)
    {
        const auto index = mask.grid.linear_to_index(i);
        const auto &tile = mask.get_tile(i);
        // positions inside the tile: key k0 + k, query q0 + q
        const Index k0 = index[0] * mask.basetile_shape[0];
        const Index q0 = index[1] * mask.basetile_shape[1];
        int32_t cls = NNTILE_HIP_MASK_TILE_MIXED;
        const int rc = TileCall<T>::classify(starpu::get_local_stream(), tile.shape[0],
                tile.shape[1], tile.get_ptr(), q0 - k0 + causal_offset,
                static_cast<int32_t *>(word.get_ptr()), &cls);
        if(rc != NNTILE_HIP_OK)
        {
            throw std::runtime_error("Error in mask_tile_class launch (code "
                    + std::to_string(rc) + ")");
        }
        classes[i] = cls;
    }
    word.unregister_submit();
    return classes;
}

template<typename T>
static std::vector<std::pair<const void *, std::uint64_t>> mask_identity(const Tensor<T> &mask)
{
    std::vector<std::pair<const void *, std::uint64_t>> ident(mask.grid.nelems);
    for(Index i = 0; i < mask.grid.nelems; ++i)
    {
        const auto &tile = mask.get_tile(i);
        ident[i] = {tile.get_ptr(), tile.write_stamp()};
    }
    return ident;
}

template<typename T>
bool flash_sdpa_mask_known_classes(const Tensor<T> &mask, Index causal_offset,
        std::vector<int> &classes)
{
    require(mask.ndim == 2, "mask must be 2-dimensional");
    const auto ident = mask_identity(mask);
    std::lock_guard<std::mutex> guard(mask_cache_mutex);
    for(std::size_t e = 0; e < mask_cache.size(); )
    {
        auto &entry = mask_cache[e];
        if(entry.tiles.empty() || ident.empty() || entry.tiles[0].first != ident[0].first)
        {
            ++e;
            continue;
        }
        if(entry.tiles == ident && entry.causal_offset == causal_offset
                && entry.shape == mask.shape && entry.basetile == mask.basetile_shape)
        {
            ++mask_cache_hits;
            classes = entry.classes;
            return true;
        }
        if(entry.tiles[0].second != ident[0].second)
        {
            // the memory at this address was given to a writer or reallocated
            mask_cache.erase(mask_cache.begin() + static_cast<std::ptrdiff_t>(e));
            continue;
        }
        ++e;
    }
    ++mask_cache_misses;
    return false;
}

template<typename T>
void flash_sdpa_mask_declare_constant(const Tensor<T> &mask, Index causal_offset)
{
    require(mask.ndim == 2, "mask must be 2-dimensional");
    // (outside the lock: this blocks on the device)
    MaskCacheEntry fresh;
    fresh.classes = flash_sdpa_mask_classes<T>(mask, causal_offset);
    fresh.tiles = mask_identity(mask);
    fresh.causal_offset = causal_offset;
    fresh.shape = mask.shape;
    fresh.basetile = mask.basetile_shape;
    std::lock_guard<std::mutex> guard(mask_cache_mutex);
    ++mask_cache_classifications;
    // one entry per mask and offset: an earlier declaration is replaced
    for(std::size_t e = 0; e < mask_cache.size(); )
    {
        const auto &entry = mask_cache[e];
        if(!entry.tiles.empty() && !fresh.tiles.empty()
                && entry.tiles[0].first == fresh.tiles[0].first
                && entry.causal_offset == causal_offset)
        {
            mask_cache.erase(mask_cache.begin() + static_cast<std::ptrdiff_t>(e));
            continue;
        }
        ++e;
    }
    if(mask_cache.size() >= kMaskCacheEntries)
    {
        mask_cache.erase(mask_cache.begin());
    }
    mask_cache.push_back(std::move(fresh));
}

template<typename T>
void flash_sdpa_mask_forget(const Tensor<T> &mask)
{
    if(mask.grid.nelems == 0)
    {
        return;
    }
    const void *first = mask.get_tile(0).get_ptr();
    std::lock_guard<std::mutex> guard(mask_cache_mutex);
    for(std::size_t e = 0; e < mask_cache.size(); )
    {
        if(!mask_cache[e].tiles.empty() && mask_cache[e].tiles[0].first == first)
        {
            mask_cache.erase(mask_cache.begin() + static_cast<std::ptrdiff_t>(e));
            continue;
        }
        ++e;
    }
}

bool flash_sdpa_classify_on_first_sight()
{
    static const bool on = []
    {
        const char *v = std::getenv("NNTILE_HIP_SDPA_CLASSIFY_ON_FIRST_SIGHT");
        return v != nullptr && v[0] != '\0' && v[0] != '0';
    }();
    return on;
}

// The classes of a mask for the calls with the reference's signature: known
// if the mask was declared constant (and neither written through this runtime
// nor forgotten since); with the opt-in above an unknown mask is declared on
// the spot (blocking).
template<typename T>
static bool classes_for_reference_call(const Tensor<T> &mask, std::vector<int> &classes)
{
    if(flash_sdpa_mask_known_classes<T>(mask, 0, classes))
    {
        return true;
    }
    if(!flash_sdpa_classify_on_first_sight())
    {
        return false;
    }
    flash_sdpa_mask_declare_constant<T>(mask, 0);
    return flash_sdpa_mask_known_classes<T>(mask, 0, classes);
}

// What the classes say about the mask as a whole: NNTILE_HIP_MASK_NONE when
// every tile is open, NNTILE_HIP_MASK_CAUSAL when every tile is what the rule
// key <= query + causal_offset makes of it (open below the diagonal band,
// hidden above, exactly on the rule where the band crosses), -1 otherwise.
// Classes are exact statements about every element, so the answer is too.
int flash_sdpa_mask_rule(const TensorTraits &mask, const std::vector<int> &mask_classes,
        Index causal_offset)
{
    bool all_open = true, on_rule = true;
    for(Index i = 0; i < mask.grid.nelems; ++i)
    {
        const auto index = mask.grid.linear_to_index(i);
        const Index k0 = index[0] * mask.basetile_shape[0];
        const Index q0 = index[1] * mask.basetile_shape[1];
        const Index k_len = std::min(mask.basetile_shape[0], mask.shape[0] - k0);
        const Index q_len = std::min(mask.basetile_shape[1], mask.shape[1] - q0);
        // the rule inside the tile: visible <=> k0 + k <= q0 + q + causal_offset
        const bool rule_all_visible = k0 + k_len - 1 <= q0 + causal_offset;
        const bool rule_all_hidden = k0 > q0 + q_len - 1 + causal_offset;
        const int expected = rule_all_visible ? NNTILE_HIP_MASK_TILE_OPEN
            : (rule_all_hidden ? NNTILE_HIP_MASK_TILE_HIDDEN : NNTILE_HIP_MASK_TILE_CAUSAL);
        all_open = all_open && mask_classes[i] == NNTILE_HIP_MASK_TILE_OPEN;
        on_rule = on_rule && mask_classes[i] == expected;
    }
    return all_open ? NNTILE_HIP_MASK_NONE : (on_rule ? NNTILE_HIP_MASK_CAUSAL : -1);
}

template<typename T>
Index flash_sdpa_fwd_cudnn_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &mask, const std::vector<int> &mask_classes,
        Index causal_offset, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &V, const Tensor<T> &A)
{
    flash_sdpa_fwd_cudnn_check(K, Q, mask, logsumexp, V, A);
    require(static_cast<Index>(mask_classes.size()) == mask.grid.nelems,
            "one class per mask tile is required");
    const Index num_k_seq_tiles = K.grid.shape[1];
    const Index q_tile = Q.basetile_shape[1], k_tile = K.basetile_shape[1];
    // A mask that is the causal rule itself, or hides nothing, needs no tasks
    // per pair: one launch per slab of the batch grid merges all key tiles
    // into all query tiles.
    const int whole = flash_sdpa_mask_rule(mask, mask_classes, causal_offset);
    if(whole >= 0 && Q.grid.shape[1] <= NNTILE_HIP_SDPA_MAX_TILES
            && num_k_seq_tiles <= NNTILE_HIP_SDPA_MAX_TILES)
    {
        return flash_sdpa_fwd_hip_async<T>(K, Q, whole, causal_offset, logsumexp, V, A, false);
    }
    Index submitted = 0;
    for(Index a_linear = 0; a_linear < A.grid.nelems; ++a_linear)
    {
        const auto a_index = A.grid.linear_to_index(a_linear);
        const auto &Q_tile = Q.get_tile(a_linear);
        const auto &A_tile = A.get_tile(a_linear);
        const auto &lse_tile = logsumexp.get_tile(
                {a_index[1], a_index[2], a_index[3], a_index[4]});
        for(Index k_idx = 0; k_idx < num_k_seq_tiles; ++k_idx)
        {
            const Index m_linear = mask.grid.index_to_linear({k_idx, a_index[1]});
            const int cls = mask_classes[m_linear];
            if(cls == NNTILE_HIP_MASK_TILE_HIDDEN)
            {
                continue;       // the pair would leave (lse, A) as they are
            }
            auto kv_index = a_index;
            kv_index[1] = k_idx;
            const auto &K_tile = K.get_tile(kv_index);
            const auto &V_tile = V.get_tile(kv_index);
            ++submitted;
            if(cls == NNTILE_HIP_MASK_TILE_MIXED)
            {
                tile::flash_sdpa_fwd_cudnn_async<T>(K_tile, Q_tile, mask.get_tile(m_linear),
                        lse_tile, V_tile, A_tile);
                continue;
            }
            nntile_hip_sdpa_tile_args a;
            std::memset(&a, 0, sizeof(a));
            a.q_seq = Q_tile.shape[1];
            a.k_seq = K_tile.shape[1];
            a.head = Q_tile.shape[0];
            a.batch = Q_tile.shape[2] * Q_tile.shape[3] * Q_tile.shape[4];
            a.n_batch = a.batch;
            a.kv_group = 1;
            a.mask_mode = cls == NNTILE_HIP_MASK_TILE_OPEN ? NNTILE_HIP_MASK_NONE
                : NNTILE_HIP_MASK_CAUSAL;
            a.q_pos0 = a_index[1] * q_tile;
            a.k_pos0 = k_idx * k_tile;
            a.causal_offset = causal_offset;
            a.K = K_tile.get_ptr();
            a.Q = Q_tile.get_ptr();
            a.V = V_tile.get_ptr();
            a.lse = static_cast<float *>(lse_tile.get_ptr());
            a.A = A_tile.get_ptr();
            lse_tile.mark_written();
            A_tile.mark_written();
            starpu::count_direct_launch();
            const int rc = TileCall<T>::run(starpu::get_local_stream(), &a);
            if(rc != NNTILE_HIP_OK)
            {
                throw std::runtime_error("Error in flash_sdpa_fwd tile launch (code "
                        + std::to_string(rc) + ")");
            }
        }
    }
    return submitted;
}

template<typename T>
void flash_sdpa_fwd_cudnn_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &mask, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &V, const Tensor<T> &A)
{
    flash_sdpa_fwd_cudnn_check(K, Q, mask, logsumexp, V, A);
    // The reference's signature carries no offset: its masks are square
    // (K.shape[1] == Q.shape[1] is one of its checks), the rule to look for is
    // key <= query.  A mask nothing is known about is read as the reference
    // reads it: one task per pair with the pair's mask tile.
    std::vector<int> classes;
    if(classes_for_reference_call<T>(mask, classes))
    {
        (void)flash_sdpa_fwd_cudnn_async<T>(K, Q, mask, classes, 0, logsumexp, V, A);
        return;
    }
    flash_sdpa_fwd_cudnn_pairs_async<T>(K, Q, mask, logsumexp, V, A);
}

// ---- backward: src/tensor/flash_sdpa_bwd_cudnn.cc:22-261 -------------------

void flash_sdpa_bwd_cudnn_check(const TensorTraits &K, const TensorTraits &Q,
        const TensorTraits &V, const TensorTraits &A, const TensorTraits &dA,
        const TensorTraits &mask, const TensorTraits &logsumexp,
        const TensorTraits &dK, const TensorTraits &dQ, const TensorTraits &dV)
{
    tile::bwd_common_check(K, Q, V, A, dA, mask, logsumexp, dK, dQ, dV);
    // basetile compatibility for multi-tile execution
    const auto &Kb = K.basetile_shape, &Qb = Q.basetile_shape,
          &Vb = V.basetile_shape, &Ab = A.basetile_shape,
          &dAb = dA.basetile_shape, &dKb = dK.basetile_shape,
          &dQb = dQ.basetile_shape, &dVb = dV.basetile_shape,
          &Mb = mask.basetile_shape, &Lb = logsumexp.basetile_shape;
    require(Qb == dQb && Qb == Ab && Qb == dAb, "Q, dQ, A, dA basetile shapes must match");
    for(Index d : {Index(0), Index(2), Index(3), Index(4)})
    {
        require(Kb[d] == Qb[d], "K and Q basetile shapes mismatch");
        require(Vb[d] == Qb[d], "V and Q basetile shapes mismatch");
        require(dKb[d] == Qb[d], "dK and Q basetile shapes mismatch");
        require(dVb[d] == Qb[d], "dV and Q basetile shapes mismatch");
    }
    require(Mb[0] == Kb[1], "mask basetile axis 0 must match K basetile sequence dimension");
    require(Mb[1] == Qb[1], "mask basetile axis 1 must match Q basetile sequence dimension");
    require(Lb[0] == Qb[1] && Lb[1] == Qb[2] && Lb[2] == Qb[3] && Lb[3] == Qb[4],
            "logsumexp basetile shape must match Q basetile shape (excluding head dimension)");
    require(Kb[0] == K.shape[0] && Qb[0] == Q.shape[0] && Vb[0] == V.shape[0]
            && Ab[0] == A.shape[0] && dAb[0] == dA.shape[0] && dKb[0] == dK.shape[0]
            && dQb[0] == dQ.shape[0] && dVb[0] == dV.shape[0],
            "head dimension must not be tiled");
}

template<typename T>
void flash_sdpa_bwd_cudnn_pairs_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &V, const Tensor<T> &A, const Tensor<T> &dA,
        const Tensor<T> &mask, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &dK, const Tensor<T> &dQ, const Tensor<T> &dV)
{
    flash_sdpa_bwd_cudnn_check(K, Q, V, A, dA, mask, logsumexp, dK, dQ, dV);
    const Index num_k_seq_tiles = K.grid.shape[1];
    // dQ tiles define the Q, A, dA and logsumexp tiles; each gets the
    // contribution of every key tile along the sequence axis, and each key
    // tile's dK, dV collect over the dQ tiles of their slab
    // (src/tensor/flash_sdpa_bwd_cudnn.cc:172-247)
    for(Index dq_linear = 0; dq_linear < dQ.grid.nelems; ++dq_linear)
    {
        const auto dq_index = dQ.grid.linear_to_index(dq_linear);
        const auto &Q_tile = Q.get_tile(dq_linear);
        const auto &A_tile = A.get_tile(dq_linear);
        const auto &dA_tile = dA.get_tile(dq_linear);
        const auto &dQ_tile = dQ.get_tile(dq_linear);
        const auto &lse_tile = logsumexp.get_tile(
                {dq_index[1], dq_index[2], dq_index[3], dq_index[4]});
        const Index seq = dQ_tile.shape[1];
        for(Index k_idx = 0; k_idx < num_k_seq_tiles; ++k_idx)
        {
            auto kv_index = dq_index;
            kv_index[1] = k_idx;
            const auto &K_tile = K.get_tile(kv_index);
            const auto &V_tile = V.get_tile(kv_index);
            const auto &dK_tile = dK.get_tile(kv_index);
            const auto &dV_tile = dV.get_tile(kv_index);
            const auto &mask_tile = mask.get_tile({k_idx, dq_index[1]});
            require(K_tile.shape[1] == seq, "K tile sequence length mismatches dQ tile");
            require(mask_tile.shape[0] == K_tile.shape[1] && mask_tile.shape[1] == seq,
                    "Mask tile shape mismatches dQ/K tiles");
            require(lse_tile.shape[0] == seq, "logsumexp tile shape mismatches dQ tile");
            tile::flash_sdpa_bwd_cudnn_async<T>(K_tile, Q_tile, V_tile, A_tile,
                    dA_tile, mask_tile, lse_tile, dK_tile, dQ_tile, dV_tile);
        }
    }
}

template<typename T>
void flash_sdpa_bwd_cudnn(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &V, const Tensor<T> &A, const Tensor<T> &dA,
        const Tensor<T> &mask, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &dK, const Tensor<T> &dQ, const Tensor<T> &dV)
{
    flash_sdpa_bwd_cudnn_async<T>(K, Q, V, A, dA, mask, logsumexp, dK, dQ, dV);
    starpu::task_wait_for_all();
}

template<typename T> struct BwdTileCall;
template<> struct BwdTileCall<bf16_t>
{
    static int run(void *s, const nntile_hip_sdpa_bwd_args *a) { return nntile_hip_sdpa_bwd_tile_bf16(s, a); }
};
template<> struct BwdTileCall<fp16_t>
{
    static int run(void *s, const nntile_hip_sdpa_bwd_args *a) { return nntile_hip_sdpa_bwd_tile_fp16(s, a); }
};

// Per (dQ tile, key tile) pair: analytic calls with the pair's positions.
// With `mask` and its classes, the pair's class picks the mode (hidden: no
// call; mixed: the reference's tile operation with the mask tile); without,
// every pair runs in `mask_mode` and pairs a causal mask hides are skipped.
template<typename T>
static Index bwd_pairs(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &V, const Tensor<T> &A, const Tensor<T> &dA,
        const Tensor<T> *mask, const std::vector<int> *mask_classes,
        int mask_mode, Index causal_offset, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &dK, const Tensor<T> &dQ, const Tensor<T> &dV)
{
    const Index num_k_seq_tiles = K.grid.shape[1];
    const Index q_tile = Q.basetile_shape[1], k_tile = K.basetile_shape[1];
    // One workspace for all calls: they run in order on one stream, and each
    // call writes what it reads there.
    std::size_t ws_bytes = 0;
    for(Index i = 0; i < dQ.grid.nelems; ++i)
    {
        const auto &t = dQ.get_tile(i);
        ws_bytes = std::max(ws_bytes, static_cast<std::size_t>(
                    t.shape[1] * t.shape[2] * t.shape[3] * t.shape[4]) * sizeof(float));
    }
    starpu::VariableHandle workspace(ws_bytes);
    Index submitted = 0;
    for(Index dq_linear = 0; dq_linear < dQ.grid.nelems; ++dq_linear)
    {
        const auto dq_index = dQ.grid.linear_to_index(dq_linear);
        const auto &Q_tile = Q.get_tile(dq_linear);
        const auto &lse_tile = logsumexp.get_tile(
                {dq_index[1], dq_index[2], dq_index[3], dq_index[4]});
        const Index q_pos0 = dq_index[1] * q_tile;
        const Index q_len = Q_tile.shape[1];
        for(Index k_idx = 0; k_idx < num_k_seq_tiles; ++k_idx)
        {
            const Index k_pos0 = k_idx * k_tile;
            auto kv_index = dq_index;
            kv_index[1] = k_idx;
            const auto &K_tile = K.get_tile(kv_index);
            int pair_mode = mask_mode;
            if(mask != nullptr)
            {
                const Index m_linear = mask->grid.index_to_linear({k_idx, dq_index[1]});
                const int cls = (*mask_classes)[m_linear];
                if(cls == NNTILE_HIP_MASK_TILE_HIDDEN)
                {
                    continue;       // no gradient flows through this pair
                }
                if(cls == NNTILE_HIP_MASK_TILE_MIXED)
                {
                    tile::flash_sdpa_bwd_cudnn_async<T>(K_tile, Q_tile, V.get_tile(kv_index),
                            A.get_tile(dq_linear), dA.get_tile(dq_linear),
                            mask->get_tile(m_linear), lse_tile, dK.get_tile(kv_index),
                            dQ.get_tile(dq_linear), dV.get_tile(kv_index));
                    ++submitted;
                    continue;
                }
                pair_mode = cls == NNTILE_HIP_MASK_TILE_OPEN ? NNTILE_HIP_MASK_NONE
                    : NNTILE_HIP_MASK_CAUSAL;
            }
            // the last query of the tile sees keys up to its position + offset
            else if(mask_mode == NNTILE_HIP_MASK_CAUSAL
                    && k_pos0 > q_pos0 + q_len - 1 + causal_offset)
            {
                continue;
            }
            nntile_hip_sdpa_bwd_args a;
            std::memset(&a, 0, sizeof(a));
            a.q_seq = q_len;
            a.k_seq = K_tile.shape[1];
            a.head = Q_tile.shape[0];
            a.batch = Q_tile.shape[2] * Q_tile.shape[3] * Q_tile.shape[4];
            a.n_batch = a.batch;
            a.kv_group = 1;
            a.mask_mode = pair_mode;
            a.q_pos0 = q_pos0;
            a.k_pos0 = k_pos0;
            a.causal_offset = causal_offset;
            a.K = K_tile.get_ptr();
            a.Q = Q_tile.get_ptr();
            a.V = V.get_tile(kv_index).get_ptr();
            a.A = A.get_tile(dq_linear).get_ptr();
            a.dA = dA.get_tile(dq_linear).get_ptr();
            a.lse = static_cast<const float *>(lse_tile.get_ptr());
            a.dK = dK.get_tile(kv_index).get_ptr();
            a.dQ = dQ.get_tile(dq_linear).get_ptr();
            a.dV = dV.get_tile(kv_index).get_ptr();
            a.workspace = workspace.get_ptr();
            a.workspace_bytes = ws_bytes;
            dK.get_tile(kv_index).mark_written();
            dQ.get_tile(dq_linear).mark_written();
            dV.get_tile(kv_index).mark_written();
            starpu::count_direct_launch();
            const int rc = BwdTileCall<T>::run(starpu::get_local_stream(), &a);
            if(rc != NNTILE_HIP_OK)
            {
                throw std::runtime_error("Error in flash_sdpa_bwd_hip launch (code "
                        + std::to_string(rc) + ")");
            }
            ++submitted;
        }
    }
    workspace.unregister_submit();
    return submitted;
}

template<typename T> struct BwdGridCall;
template<> struct BwdGridCall<bf16_t>
{
    static int run(void *s, const nntile_hip_sdpa_bwd_grid_args *a) { return nntile_hip_sdpa_bwd_grid_bf16(s, a); }
};
template<> struct BwdGridCall<fp16_t>
{
    static int run(void *s, const nntile_hip_sdpa_bwd_grid_args *a) { return nntile_hip_sdpa_bwd_grid_fp16(s, a); }
};

// Whether one call can take all tile pairs of a slab: the argument block has
// room for the tiles, and no workgroup's 128 rows straddle two tiles.
static bool bwd_grid_fits(const TensorTraits &K, const TensorTraits &Q)
{
    const Index n_q = Q.grid.shape[1], n_kv = K.grid.shape[1];
    return n_q <= NNTILE_HIP_SDPA_BWD_MAX_TILES && n_kv <= NNTILE_HIP_SDPA_BWD_MAX_TILES
        && (n_q == 1 || Q.basetile_shape[1] % 128 == 0)
        && (n_kv == 1 || K.basetile_shape[1] % 128 == 0);
}

// All (dQ tile, key tile) pairs of the slabs of the batch grid in as few
// calls as the tile tables allow, for a mask that is the causal rule or
// hides nothing: the sums over the pairs
// (src/tensor/flash_sdpa_bwd_cudnn.cc:172-247) are carried in fp32 inside the
// kernels instead of through the 16-bit gradient tiles.  Returns the calls.
template<typename T>
static Index bwd_grid(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &V, const Tensor<T> &A, const Tensor<T> &dA,
        int mask_mode, Index causal_offset, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &dK, const Tensor<T> &dQ, const Tensor<T> &dV)
{
    const Index n_q = Q.grid.shape[1], n_kv = K.grid.shape[1];
    // The slabs of the batch grid go into as few calls as the tile tables
    // hold: slabs with the same number of entries share a call.
    struct Slab { Index g2, g3, g4, batch; };
    std::vector<Slab> slabs;
    for(Index g4 = 0; g4 < Q.grid.shape[4]; ++g4)
    {
        for(Index g3 = 0; g3 < Q.grid.shape[3]; ++g3)
        {
            for(Index g2 = 0; g2 < Q.grid.shape[2]; ++g2)
            {
                const auto &q0 = Q.get_tile({0, 0, g2, g3, g4});
                slabs.push_back({g2, g3, g4, q0.shape[2] * q0.shape[3] * q0.shape[4]});
            }
        }
    }
    const std::size_t per_call = static_cast<std::size_t>(
            NNTILE_HIP_SDPA_BWD_MAX_TILES / std::max(n_q, n_kv));
    // One workspace for all calls: they run in order on one stream, and each
    // call writes what it reads there.
    const std::size_t ws_bytes = sizeof(float) * per_call * static_cast<std::size_t>(Q.shape[1]
            * Q.basetile_shape[2] * Q.basetile_shape[3] * Q.basetile_shape[4]);
    starpu::VariableHandle workspace = starpu::worker_scratch(ws_bytes);
    Index calls = 0;
    for(std::size_t first = 0; first < slabs.size();)
    {
        std::size_t count = 1;
        while(first + count < slabs.size() && count < per_call
                && slabs[first + count].batch == slabs[first].batch)
        {
            ++count;
        }
        // one task of the whole-grid codelet for these slabs
        nntile_hip_sdpa_grid_cl_args a;
        std::memset(&a, 0, sizeof(a));
        a.seq = Q.basetile_shape[1];
        a.head = Q.shape[0];
        a.batch = slabs[first].batch;
        a.q_seq = Q.shape[1];
        a.k_seq = K.shape[1];
        a.q_tile = Q.basetile_shape[1];
        a.k_tile = K.basetile_shape[1];
        a.n_batch = a.batch;
        a.kv_group = 1;
        a.mask_mode = mask_mode;
        a.n_q_tiles = static_cast<std::int32_t>(n_q);
        a.n_kv_tiles = static_cast<std::int32_t>(n_kv);
        a.n_slabs = static_cast<std::int32_t>(count);
        a.causal_offset = causal_offset;
        std::vector<starpu::Handle> Kh, Vh, Qh, Ah, dAh, Lh, dKh, dQh, dVh;
        for(std::size_t s = 0; s < count; ++s)
        {
            const Index g2 = slabs[first + s].g2, g3 = slabs[first + s].g3,
                  g4 = slabs[first + s].g4;
            for(Index t = 0; t < n_kv; ++t)
            {
                Kh.push_back(K.get_tile({0, t, g2, g3, g4}));
                Vh.push_back(V.get_tile({0, t, g2, g3, g4}));
                dKh.push_back(dK.get_tile({0, t, g2, g3, g4}));
                dVh.push_back(dV.get_tile({0, t, g2, g3, g4}));
            }
            for(Index t = 0; t < n_q; ++t)
            {
                Qh.push_back(Q.get_tile({0, t, g2, g3, g4}));
                Ah.push_back(A.get_tile({0, t, g2, g3, g4}));
                dAh.push_back(dA.get_tile({0, t, g2, g3, g4}));
                dQh.push_back(dQ.get_tile({0, t, g2, g3, g4}));
                Lh.push_back(logsumexp.get_tile({t, g2, g3, g4}));
            }
        }
        starpu::sdpa_bwd_grid<T>().submit(a, Kh, Vh, Qh, Ah, dAh, Lh, dKh, dQh, dVh, workspace);
        ++calls;
        first += count;
    }
    workspace.unregister_submit();
    return calls;
}

template<typename T>
Index flash_sdpa_bwd_hip_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &V, const Tensor<T> &A, const Tensor<T> &dA,
        int mask_mode, Index causal_offset, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &dK, const Tensor<T> &dQ, const Tensor<T> &dV)
{
    // Same shape rules as the reference operation, with a stand-in for the
    // mask that is no longer materialised.
    const TensorTraits mask({K.shape[1], Q.shape[1]},
            {K.basetile_shape[1], Q.basetile_shape[1]});
    flash_sdpa_bwd_cudnn_check(K, Q, V, A, dA, mask, logsumexp, dK, dQ, dV);
    require(mask_mode == NNTILE_HIP_MASK_NONE || mask_mode == NNTILE_HIP_MASK_CAUSAL,
            "flash_sdpa_bwd_hip: mask_mode must be NONE or CAUSAL");
    if(bwd_grid_fits(K, Q))
    {
        return bwd_grid<T>(K, Q, V, A, dA, mask_mode, causal_offset, logsumexp, dK, dQ, dV);
    }
    return bwd_pairs<T>(K, Q, V, A, dA, nullptr, nullptr, mask_mode, causal_offset,
            logsumexp, dK, dQ, dV);
}

template<typename T>
Index flash_sdpa_bwd_cudnn_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &V, const Tensor<T> &A, const Tensor<T> &dA,
        const Tensor<T> &mask, const std::vector<int> &mask_classes,
        Index causal_offset, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &dK, const Tensor<T> &dQ, const Tensor<T> &dV)
{
    flash_sdpa_bwd_cudnn_check(K, Q, V, A, dA, mask, logsumexp, dK, dQ, dV);
    require(static_cast<Index>(mask_classes.size()) == mask.grid.nelems,
            "one class per mask tile is required");
    // A mask that is the causal rule itself, or hides nothing, needs no call
    // per pair (as in the forward operation above).
    const int whole = flash_sdpa_mask_rule(mask, mask_classes, causal_offset);
    if(whole >= 0 && bwd_grid_fits(K, Q))
    {
        return bwd_grid<T>(K, Q, V, A, dA, whole, causal_offset, logsumexp, dK, dQ, dV);
    }
    return bwd_pairs<T>(K, Q, V, A, dA, &mask, &mask_classes, NNTILE_HIP_MASK_CAUSAL,
            causal_offset, logsumexp, dK, dQ, dV);
}

template<typename T>
void flash_sdpa_bwd_cudnn_async(const Tensor<T> &K, const Tensor<T> &Q,
        const Tensor<T> &V, const Tensor<T> &A, const Tensor<T> &dA,
        const Tensor<T> &mask, const Tensor<fp32_t> &logsumexp,
        const Tensor<T> &dK, const Tensor<T> &dQ, const Tensor<T> &dV)
{
    flash_sdpa_bwd_cudnn_check(K, Q, V, A, dA, mask, logsumexp, dK, dQ, dV);
    std::vector<int> classes;
    if(classes_for_reference_call<T>(mask, classes))
    {
        (void)flash_sdpa_bwd_cudnn_async<T>(K, Q, V, A, dA, mask, classes, 0, logsumexp,
                dK, dQ, dV);
        return;
    }
    flash_sdpa_bwd_cudnn_pairs_async<T>(K, Q, V, A, dA, mask, logsumexp, dK, dQ, dV);
}

#define NNTILE_HOST_INSTANTIATE_TENSOR_BWD(T) \
    template Index flash_sdpa_bwd_cudnn_async<T>(const Tensor<T> &, const Tensor<T> &, \
            const Tensor<T> &, const Tensor<T> &, const Tensor<T> &, const Tensor<T> &, \
            const std::vector<int> &, Index, const Tensor<fp32_t> &, const Tensor<T> &, \
            const Tensor<T> &, const Tensor<T> &); \
    template Index flash_sdpa_bwd_hip_async<T>(const Tensor<T> &, const Tensor<T> &, \
            const Tensor<T> &, const Tensor<T> &, const Tensor<T> &, int, Index, \
            const Tensor<fp32_t> &, const Tensor<T> &, const Tensor<T> &, const Tensor<T> &); \
    template void flash_sdpa_bwd_cudnn_async<T>(const Tensor<T> &, const Tensor<T> &, \
            const Tensor<T> &, const Tensor<T> &, const Tensor<T> &, const Tensor<T> &, \
            const Tensor<fp32_t> &, const Tensor<T> &, const Tensor<T> &, const Tensor<T> &); \
    template void flash_sdpa_bwd_cudnn<T>(const Tensor<T> &, const Tensor<T> &, \
            const Tensor<T> &, const Tensor<T> &, const Tensor<T> &, const Tensor<T> &, \
            const Tensor<fp32_t> &, const Tensor<T> &, const Tensor<T> &, const Tensor<T> &); \
    template void flash_sdpa_bwd_cudnn_pairs_async<T>(const Tensor<T> &, const Tensor<T> &, \
            const Tensor<T> &, const Tensor<T> &, const Tensor<T> &, const Tensor<T> &, \
            const Tensor<fp32_t> &, const Tensor<T> &, const Tensor<T> &, const Tensor<T> &);
NNTILE_HOST_INSTANTIATE_TENSOR_BWD(bf16_t)
NNTILE_HOST_INSTANTIATE_TENSOR_BWD(fp16_t)

#define NNTILE_HOST_INSTANTIATE_TENSOR(T) \
    template class Tensor<T>; \
    template void flash_sdpa_fwd_cudnn_async<T>(const Tensor<T> &, const Tensor<T> &, \
            const Tensor<T> &, const Tensor<fp32_t> &, const Tensor<T> &, const Tensor<T> &); \
    template void flash_sdpa_fwd_cudnn<T>(const Tensor<T> &, const Tensor<T> &, \
            const Tensor<T> &, const Tensor<fp32_t> &, const Tensor<T> &, const Tensor<T> &); \
    template Index flash_sdpa_fwd_hip_async<T>(const Tensor<T> &, const Tensor<T> &, int, \
            Index, const Tensor<fp32_t> &, const Tensor<T> &, const Tensor<T> &, bool); \
    template std::vector<int> flash_sdpa_mask_classes<T>(const Tensor<T> &, Index); \
    template bool flash_sdpa_mask_known_classes<T>(const Tensor<T> &, Index, std::vector<int> &); \
    template void flash_sdpa_mask_declare_constant<T>(const Tensor<T> &, Index); \
    template void flash_sdpa_mask_forget<T>(const Tensor<T> &); \
    template void flash_sdpa_fwd_cudnn_pairs_async<T>(const Tensor<T> &, const Tensor<T> &, \
            const Tensor<T> &, const Tensor<fp32_t> &, const Tensor<T> &, const Tensor<T> &); \
    template Index flash_sdpa_fwd_cudnn_async<T>(const Tensor<T> &, const Tensor<T> &, \
            const Tensor<T> &, const std::vector<int> &, Index, const Tensor<fp32_t> &, \
            const Tensor<T> &, const Tensor<T> &);
NNTILE_HOST_INSTANTIATE_TENSOR(bf16_t)
NNTILE_HOST_INSTANTIATE_TENSOR(fp16_t)
NNTILE_HOST_INSTANTIATE_TENSOR(fp32_t)

} // namespace tensor

} // namespace nntile
