// Flat C interface over the host-side mirror, for tests and scripts: tensors
// are created from shapes and Fortran-ordered host arrays, the operations are
// the mirror's tile::/tensor:: functions, exceptions come back as messages.
#include <cstring>
#include <functional>
#include <string>

#include "nntile_host.hh"

using namespace nntile;

namespace
{

enum DType { DT_BF16 = 0, DT_FP16 = 1, DT_FP32 = 2 };

struct AnyTensor
{
    int dtype;
    std::unique_ptr<tensor::Tensor<bf16_t>> bf16;
    std::unique_ptr<tensor::Tensor<fp16_t>> fp16;
    std::unique_ptr<tensor::Tensor<fp32_t>> fp32;
};

int fail(char *err, int errlen, const std::exception &e)
{
    if(err != nullptr && errlen > 0)
    {
        std::strncpy(err, e.what(), static_cast<size_t>(errlen) - 1);
        err[errlen - 1] = '\0';
    }
    return 1;
}

std::vector<Index> vec(const int64_t *p, int n)
{
    return std::vector<Index>(p, p + n);
}

template<typename T> tensor::Tensor<T> &get(AnyTensor *t);
template<> tensor::Tensor<bf16_t> &get<bf16_t>(AnyTensor *t) { return *t->bf16; }
template<> tensor::Tensor<fp16_t> &get<fp16_t>(AnyTensor *t) { return *t->fp16; }
template<> tensor::Tensor<fp32_t> &get<fp32_t>(AnyTensor *t) { return *t->fp32; }

template<typename T>
void run_op(int op, AnyTensor *K, AnyTensor *Q, AnyTensor *mask, AnyTensor *lse,
        AnyTensor *V, AnyTensor *A, int mask_mode, int64_t offset, int overwrite)
{
    switch(op)
    {
        case 0:     // tensor-level, the reference's signature, blocking
            tensor::flash_sdpa_fwd_cudnn<T>(get<T>(K), get<T>(Q), get<T>(mask),
                    get<fp32_t>(lse), get<T>(V), get<T>(A));
            break;
        case 1:     // tile-level on single-tile tensors, blocking
            tile::flash_sdpa_fwd_cudnn<T>(get<T>(K).get_tile(0), get<T>(Q).get_tile(0),
                    get<T>(mask).get_tile(0), get<fp32_t>(lse).get_tile(0),
                    get<T>(V).get_tile(0), get<T>(A).get_tile(0));
            break;
        case 2:     // tensor-level, one launch per slab, analytic mask
            tensor::flash_sdpa_fwd_hip_async<T>(get<T>(K), get<T>(Q), mask_mode,
                    offset, get<fp32_t>(lse), get<T>(V), get<T>(A), overwrite != 0);
            starpu::task_wait_for_all();
            break;
        case 3:     // tensor-level, the reference's submission literally: every pair, blocking
            tensor::flash_sdpa_fwd_cudnn_pairs_async<T>(get<T>(K), get<T>(Q), get<T>(mask),
                    get<fp32_t>(lse), get<T>(V), get<T>(A));
            starpu::task_wait_for_all();
            break;
        default:
            throw std::runtime_error("unknown operation");
    }
}

template<typename T>
void run_async(int op, AnyTensor *K, AnyTensor *Q, AnyTensor *mask, AnyTensor *lse,
        AnyTensor *V, AnyTensor *A)
{
    if(op == 0)
    {
        tensor::flash_sdpa_fwd_cudnn_async<T>(get<T>(K), get<T>(Q), get<T>(mask),
                get<fp32_t>(lse), get<T>(V), get<T>(A));
    }
    else if(op == 3)
    {
        tensor::flash_sdpa_fwd_cudnn_pairs_async<T>(get<T>(K), get<T>(Q), get<T>(mask),
                get<fp32_t>(lse), get<T>(V), get<T>(A));
    }
    else
    {
        throw std::runtime_error("unknown operation");
    }
}

template<typename T>
int64_t run_bwd(int op, AnyTensor *K, AnyTensor *Q, AnyTensor *V, AnyTensor *A,
        AnyTensor *dA, AnyTensor *mask, AnyTensor *lse, AnyTensor *dK,
        AnyTensor *dQ, AnyTensor *dV, int mask_mode, int64_t offset)
{
    switch(op)
    {
        case 2:     // tensor-level, analytic mask, hidden tile pairs skipped
        {
            const Index n = tensor::flash_sdpa_bwd_hip_async<T>(get<T>(K), get<T>(Q), get<T>(V),
                    get<T>(A), get<T>(dA), mask_mode, offset, get<fp32_t>(lse),
                    get<T>(dK), get<T>(dQ), get<T>(dV));
            starpu::task_wait_for_all();
            return n;
        }
        case 3:     // tensor-level, mask tiles classified first
        {
            const auto cls = tensor::flash_sdpa_mask_classes<T>(get<T>(mask), offset);
            const Index n = tensor::flash_sdpa_bwd_cudnn_async<T>(get<T>(K), get<T>(Q), get<T>(V),
                    get<T>(A), get<T>(dA), get<T>(mask), cls, offset, get<fp32_t>(lse),
                    get<T>(dK), get<T>(dQ), get<T>(dV));
            starpu::task_wait_for_all();
            return n;
        }
        case 0:     // tensor-level, the reference's signature, blocking
            tensor::flash_sdpa_bwd_cudnn<T>(get<T>(K), get<T>(Q), get<T>(V),
                    get<T>(A), get<T>(dA), get<T>(mask), get<fp32_t>(lse),
                    get<T>(dK), get<T>(dQ), get<T>(dV));
            break;
        case 4:     // tensor-level, the reference's submission literally: every pair
            tensor::flash_sdpa_bwd_cudnn_pairs_async<T>(get<T>(K), get<T>(Q), get<T>(V),
                    get<T>(A), get<T>(dA), get<T>(mask), get<fp32_t>(lse),
                    get<T>(dK), get<T>(dQ), get<T>(dV));
            starpu::task_wait_for_all();
            break;
        case 1:     // tile-level on single-tile tensors, blocking
            tile::flash_sdpa_bwd_cudnn<T>(get<T>(K).get_tile(0), get<T>(Q).get_tile(0),
                    get<T>(V).get_tile(0), get<T>(A).get_tile(0), get<T>(dA).get_tile(0),
                    get<T>(mask).get_tile(0), get<fp32_t>(lse).get_tile(0),
                    get<T>(dK).get_tile(0), get<T>(dQ).get_tile(0), get<T>(dV).get_tile(0));
            break;
        default:
            throw std::runtime_error("unknown operation");
    }
    return 0;
}

} // namespace

extern "C"
{

void *nntile_host_tensor_create(int dtype, int ndim, const int64_t *shape,
        const int64_t *basetile, char *err, int errlen)
{
    try
    {
        auto *t = new AnyTensor;
        t->dtype = dtype;
        if(dtype == DT_BF16) t->bf16.reset(new tensor::Tensor<bf16_t>(vec(shape, ndim), vec(basetile, ndim)));
        else if(dtype == DT_FP16) t->fp16.reset(new tensor::Tensor<fp16_t>(vec(shape, ndim), vec(basetile, ndim)));
        else t->fp32.reset(new tensor::Tensor<fp32_t>(vec(shape, ndim), vec(basetile, ndim)));
        return t;
    }
    catch(const std::exception &e)
    {
        fail(err, errlen, e);
        return nullptr;
    }
}

void nntile_host_tensor_free(void *t)
{
    delete static_cast<AnyTensor *>(t);
}

int nntile_host_tensor_from_array(void *t_, const void *src, char *err, int errlen)
{
    auto *t = static_cast<AnyTensor *>(t_);
    try
    {
        if(t->dtype == DT_BF16) t->bf16->from_array(static_cast<const uint16_t *>(src));
        else if(t->dtype == DT_FP16) t->fp16->from_array(static_cast<const uint16_t *>(src));
        else t->fp32->from_array(static_cast<const float *>(src));
        return 0;
    }
    catch(const std::exception &e) { return fail(err, errlen, e); }
}

int nntile_host_tensor_to_array(void *t_, void *dst, char *err, int errlen)
{
    auto *t = static_cast<AnyTensor *>(t_);
    try
    {
        if(t->dtype == DT_BF16) t->bf16->to_array(static_cast<uint16_t *>(dst));
        else if(t->dtype == DT_FP16) t->fp16->to_array(static_cast<uint16_t *>(dst));
        else t->fp32->to_array(static_cast<float *>(dst));
        return 0;
    }
    catch(const std::exception &e) { return fail(err, errlen, e); }
}

int64_t nntile_host_tensor_ntiles(void *t_)
{
    auto *t = static_cast<AnyTensor *>(t_);
    if(t->dtype == DT_BF16) return t->bf16->grid.nelems;
    if(t->dtype == DT_FP16) return t->fp16->grid.nelems;
    return t->fp32->grid.nelems;
}

// op: 0 tensor::flash_sdpa_fwd_cudnn, 1 tile::flash_sdpa_fwd_cudnn (single-tile
// tensors), 2 tensor::flash_sdpa_fwd_hip_async + wait (mask may be null),
// 3 tensor::flash_sdpa_fwd_cudnn_pairs_async + wait
int nntile_host_flash_sdpa_fwd(int op, int dtype, void *K, void *Q, void *mask,
        void *lse, void *V, void *A, int mask_mode, int64_t offset, int overwrite,
        char *err, int errlen)
{
    try
    {
        auto k = static_cast<AnyTensor *>(K), q = static_cast<AnyTensor *>(Q),
             m = static_cast<AnyTensor *>(mask), l = static_cast<AnyTensor *>(lse),
             v = static_cast<AnyTensor *>(V), a = static_cast<AnyTensor *>(A);
        if(dtype == DT_BF16) run_op<bf16_t>(op, k, q, m, l, v, a, mask_mode, offset, overwrite);
        else if(dtype == DT_FP16) run_op<fp16_t>(op, k, q, m, l, v, a, mask_mode, offset, overwrite);
        else run_op<fp32_t>(op, k, q, m, l, v, a, mask_mode, offset, overwrite);
        return 0;
    }
    catch(const std::exception &e) { return fail(err, errlen, e); }
}

} // extern "C"

namespace
{

template<typename T>
int64_t run_classified(AnyTensor *K, AnyTensor *Q, AnyTensor *mask, AnyTensor *lse,
        AnyTensor *V, AnyTensor *A, int64_t offset, int32_t *classes, int64_t n_classes)
{
    const auto cls = tensor::flash_sdpa_mask_classes<T>(get<T>(mask), offset);
    for(int64_t i = 0; classes != nullptr && i < n_classes
            && i < static_cast<int64_t>(cls.size()); ++i)
    {
        classes[i] = cls[i];
    }
    const Index n = tensor::flash_sdpa_fwd_cudnn_async<T>(get<T>(K), get<T>(Q), get<T>(mask),
            cls, offset, get<fp32_t>(lse), get<T>(V), get<T>(A));
    starpu::task_wait_for_all();
    return n;
}

} // namespace

extern "C"
{

// tensor::flash_sdpa_mask_rule on a [k_seq, q_seq] mask tiled [k_tile, q_tile]
// (no device memory): *rule = NNTILE_HIP_MASK_NONE, NNTILE_HIP_MASK_CAUSAL or -1
int nntile_host_mask_rule(int64_t k_seq, int64_t q_seq, int64_t k_tile, int64_t q_tile,
        const int32_t *classes, int64_t n_classes, int64_t offset, int32_t *rule,
        char *err, int errlen)
{
    try
    {
        const tensor::TensorTraits mask({k_seq, q_seq}, {k_tile, q_tile});
        if(n_classes != mask.grid.nelems)
        {
            throw std::runtime_error("one class per mask tile is required");
        }
        const std::vector<int> cls(classes, classes + n_classes);
        *rule = tensor::flash_sdpa_mask_rule(mask, cls, offset);
        return 0;
    }
    catch(const std::exception &e) { return fail(err, errlen, e); }
}

// tensor::flash_sdpa_mask_classes, then tensor::flash_sdpa_fwd_cudnn_async
// with those classes + wait.  classes (may be null): room for n_classes
// values, one per mask tile in the linear order of the mask's grid;
// *submitted = tile pairs launched.
int nntile_host_flash_sdpa_fwd_classified(int dtype, void *K, void *Q, void *mask,
        void *lse, void *V, void *A, int64_t offset, int32_t *classes, int64_t n_classes,
        int64_t *submitted, char *err, int errlen)
{
    try
    {
        auto k = static_cast<AnyTensor *>(K), q = static_cast<AnyTensor *>(Q),
             m = static_cast<AnyTensor *>(mask), l = static_cast<AnyTensor *>(lse),
             v = static_cast<AnyTensor *>(V), a = static_cast<AnyTensor *>(A);
        int64_t n;
        if(dtype == DT_BF16) n = run_classified<bf16_t>(k, q, m, l, v, a, offset, classes, n_classes);
        else if(dtype == DT_FP16) n = run_classified<fp16_t>(k, q, m, l, v, a, offset, classes, n_classes);
        else n = run_classified<fp32_t>(k, q, m, l, v, a, offset, classes, n_classes);
        if(submitted != nullptr) *submitted = n;
        return 0;
    }
    catch(const std::exception &e) { return fail(err, errlen, e); }
}

// Shape rules only (no device memory): level 0 = tile, 1 = tensor.  Shapes are
// given as 6 x (ndim, dims..., basetile dims...) blocks in the order
// K, Q, mask, logsumexp, V, A.
int nntile_host_check_shapes(int level, const int64_t *desc, char *err, int errlen)
{
    try
    {
        std::vector<tensor::TensorTraits> tt;
        const int64_t *p = desc;
        for(int i = 0; i < 6; ++i)
        {
            const int nd = static_cast<int>(*p++);
            auto shape = vec(p, nd); p += nd;
            auto base = vec(p, nd); p += nd;
            tt.emplace_back(shape, base);
        }
        if(level == 0)
        {
            tile::flash_sdpa_fwd_cudnn_check(tt[0], tt[1], tt[2], tt[3], tt[4], tt[5]);
        }
        else
        {
            tensor::flash_sdpa_fwd_cudnn_check(tt[0], tt[1], tt[2], tt[3], tt[4], tt[5]);
        }
        return 0;
    }
    catch(const std::exception &e) { return fail(err, errlen, e); }
}

// op: 0 tensor::flash_sdpa_bwd_cudnn, 1 tile::flash_sdpa_bwd_cudnn (single-tile
// tensors), 2 tensor::flash_sdpa_bwd_hip_async + wait (mask may be null), 3
// tensor::flash_sdpa_mask_classes + the overload that takes the classes + wait
// (ops 2 and 3: *submitted = tile pairs launched), 4
// tensor::flash_sdpa_bwd_cudnn_pairs_async + wait; dtype bf16 or fp16, as the
// reference's pack
int nntile_host_flash_sdpa_bwd(int op, int dtype, void *K, void *Q, void *V,
        void *A, void *dA, void *mask, void *lse, void *dK, void *dQ, void *dV,
        int mask_mode, int64_t offset, int64_t *submitted, char *err, int errlen)
{
    try
    {
        AnyTensor *t[10] = {static_cast<AnyTensor *>(K), static_cast<AnyTensor *>(Q),
            static_cast<AnyTensor *>(V), static_cast<AnyTensor *>(A),
            static_cast<AnyTensor *>(dA), static_cast<AnyTensor *>(mask),
            static_cast<AnyTensor *>(lse), static_cast<AnyTensor *>(dK),
            static_cast<AnyTensor *>(dQ), static_cast<AnyTensor *>(dV)};
        int64_t n = 0;
        if(dtype == DT_BF16) n = run_bwd<bf16_t>(op, t[0], t[1], t[2], t[3], t[4], t[5], t[6], t[7], t[8], t[9], mask_mode, offset);
        else if(dtype == DT_FP16) n = run_bwd<fp16_t>(op, t[0], t[1], t[2], t[3], t[4], t[5], t[6], t[7], t[8], t[9], mask_mode, offset);
        else throw std::runtime_error("flash_sdpa_bwd_cudnn: no fp32 instance");
        if(submitted != nullptr) *submitted = n;
        return 0;
    }
    catch(const std::exception &e) { return fail(err, errlen, e); }
}

// Shape rules of the backward only: level 0 = tile, 1 = tensor; 10 blocks
// (ndim, dims..., basetile dims...) in the order K, Q, V, A, dA, mask,
// logsumexp, dK, dQ, dV.
int nntile_host_check_shapes_bwd(int level, const int64_t *desc, char *err, int errlen)
{
    try
    {
        std::vector<tensor::TensorTraits> tt;
        const int64_t *p = desc;
        for(int i = 0; i < 10; ++i)
        {
            const int nd = static_cast<int>(*p++);
            auto shape = vec(p, nd); p += nd;
            auto base = vec(p, nd); p += nd;
            tt.emplace_back(shape, base);
        }
        if(level == 0)
        {
            tile::flash_sdpa_bwd_cudnn_check(tt[0], tt[1], tt[2], tt[3], tt[4], tt[5],
                    tt[6], tt[7], tt[8], tt[9]);
        }
        else
        {
            tensor::flash_sdpa_bwd_cudnn_check(tt[0], tt[1], tt[2], tt[3], tt[4], tt[5],
                    tt[6], tt[7], tt[8], tt[9]);
        }
        return 0;
    }
    catch(const std::exception &e) { return fail(err, errlen, e); }
}

uint32_t nntile_host_footprint_bwd(int64_t seq, int64_t head, int64_t batch)
{
    return starpu::FlashSdpaBwdCudnn<std::tuple<bf16_t>>::hash_parameters(seq, head, batch);
}

int64_t nntile_host_tasks_submitted_bwd(int dtype)
{
    if(dtype == DT_BF16) return starpu::flash_sdpa_bwd_cudnn<bf16_t>().submitted;
    if(dtype == DT_FP16) return starpu::flash_sdpa_bwd_cudnn<fp16_t>().submitted;
    return -1;
}

const char *nntile_host_codelet_name_bwd(int dtype)
{
    if(dtype == DT_BF16) return starpu::flash_sdpa_bwd_cudnn<bf16_t>().name.c_str();
    if(dtype == DT_FP16) return starpu::flash_sdpa_bwd_cudnn<fp16_t>().name.c_str();
    return "";
}

uint32_t nntile_host_footprint(int64_t seq, int64_t head, int64_t batch)
{
    return starpu::FlashSdpaFwdCudnn<std::tuple<bf16_t>>::hash_parameters(seq, head, batch);
}

int64_t nntile_host_tasks_submitted(int dtype)
{
    if(dtype == DT_BF16) return starpu::flash_sdpa_fwd_cudnn<bf16_t>().submitted;
    if(dtype == DT_FP16) return starpu::flash_sdpa_fwd_cudnn<fp16_t>().submitted;
    return starpu::flash_sdpa_fwd_cudnn<fp32_t>().submitted;
}

// Tasks of the whole-grid codelets (one per group of slabs) submitted so far
int64_t nntile_host_grid_tasks_submitted(int dtype, int backward)
{
    if(backward)
    {
        if(dtype == DT_BF16) return starpu::sdpa_bwd_grid<bf16_t>().submitted;
        if(dtype == DT_FP16) return starpu::sdpa_bwd_grid<fp16_t>().submitted;
        return -1;
    }
    if(dtype == DT_BF16) return starpu::sdpa_fwd_grid<bf16_t>().submitted;
    if(dtype == DT_FP16) return starpu::sdpa_fwd_grid<fp16_t>().submitted;
    return starpu::sdpa_fwd_grid<fp32_t>().submitted;
}

const char *nntile_host_grid_codelet_name(int dtype, int backward)
{
    if(backward)
    {
        if(dtype == DT_BF16) return starpu::sdpa_bwd_grid<bf16_t>().name.c_str();
        if(dtype == DT_FP16) return starpu::sdpa_bwd_grid<fp16_t>().name.c_str();
        return "";
    }
    if(dtype == DT_BF16) return starpu::sdpa_fwd_grid<bf16_t>().name.c_str();
    if(dtype == DT_FP16) return starpu::sdpa_fwd_grid<fp16_t>().name.c_str();
    return starpu::sdpa_fwd_grid<fp32_t>().name.c_str();
}

const char *nntile_host_codelet_name(int dtype)
{
    if(dtype == DT_BF16) return starpu::flash_sdpa_fwd_cudnn<bf16_t>().name.c_str();
    if(dtype == DT_FP16) return starpu::flash_sdpa_fwd_cudnn<fp16_t>().name.c_str();
    return starpu::flash_sdpa_fwd_cudnn<fp32_t>().name.c_str();
}

// Counters of the mask-class cache behind the reference-signature tensor
// operations, a reset of the cache, and a "some writer got this tensor" mark
// on every tile of a tensor.
void nntile_host_mask_cache_stats(uint64_t *hits, uint64_t *misses)
{
    const auto st = tensor::flash_sdpa_mask_cache_stats();
    *hits = st.hits;
    *misses = st.misses;
}

uint64_t nntile_host_mask_classifications(void)
{
    return tensor::flash_sdpa_mask_cache_stats().classifications;
}

// tensor::flash_sdpa_mask_declare_constant (forget != 0: flash_sdpa_mask_forget)
int nntile_host_mask_declare_constant(void *mask_, int forget, char *err, int errlen)
{
    try
    {
        auto *m = static_cast<AnyTensor *>(mask_);
        if(m->dtype == DT_BF16)
        {
            forget ? tensor::flash_sdpa_mask_forget<bf16_t>(*m->bf16)
                : tensor::flash_sdpa_mask_declare_constant<bf16_t>(*m->bf16);
        }
        else if(m->dtype == DT_FP16)
        {
            forget ? tensor::flash_sdpa_mask_forget<fp16_t>(*m->fp16)
                : tensor::flash_sdpa_mask_declare_constant<fp16_t>(*m->fp16);
        }
        else
        {
            forget ? tensor::flash_sdpa_mask_forget<fp32_t>(*m->fp32)
                : tensor::flash_sdpa_mask_declare_constant<fp32_t>(*m->fp32);
        }
        return 0;
    }
    catch(const std::exception &e) { return fail(err, errlen, e); }
}

// Device address of tile `i` of a tensor (for tests that write a tile by
// means the runtime does not see)
void *nntile_host_tensor_tile_ptr(void *t_, int64_t i)
{
    auto *t = static_cast<AnyTensor *>(t_);
    if(t->dtype == DT_BF16) return t->bf16->get_tile(i).get_ptr();
    if(t->dtype == DT_FP16) return t->fp16->get_tile(i).get_ptr();
    return t->fp32->get_tile(i).get_ptr();
}

int64_t nntile_host_tensor_tile_bytes(void *t_, int64_t i)
{
    auto *t = static_cast<AnyTensor *>(t_);
    if(t->dtype == DT_BF16) return static_cast<int64_t>(t->bf16->get_tile(i).size());
    if(t->dtype == DT_FP16) return static_cast<int64_t>(t->fp16->get_tile(i).size());
    return static_cast<int64_t>(t->fp32->get_tile(i).size());
}

void nntile_host_mask_cache_clear(void)
{
    tensor::flash_sdpa_mask_cache_clear();
}

void nntile_host_tensor_mark_written(void *t_)
{
    auto *t = static_cast<AnyTensor *>(t_);
    const int64_t n = nntile_host_tensor_ntiles(t_);
    for(int64_t i = 0; i < n; ++i)
    {
        if(t->dtype == DT_BF16) t->bf16->get_tile(i).mark_written();
        else if(t->dtype == DT_FP16) t->fp16->get_tile(i).mark_written();
        else t->fp32->get_tile(i).mark_written();
    }
}

// Times `steps` passes (after `warmup` untimed ones) of what a layer does per
// forward through the reference's interface (Sdpa._forward_flash,
// wrappers/python/nntile/layer/sdpa.py:533-557): logsumexp filled with -inf,
// then tensor::flash_sdpa_fwd_cudnn_async (op 0) or
// tensor::flash_sdpa_fwd_cudnn_pairs_async (op 3), with HIP events on the
// mirror's stream.  *ms = milliseconds per pass, *launches = attention
// launches per pass (tile tasks + whole-grid tasks + direct launches).
int nntile_host_time_flash_sdpa_fwd(int op, int dtype, void *K, void *Q, void *mask,
        void *lse, void *V, void *A, int steps, int warmup, double *ms, int64_t *launches,
        char *err, int errlen)
{
    try
    {
        auto k = static_cast<AnyTensor *>(K), q = static_cast<AnyTensor *>(Q),
             m = static_cast<AnyTensor *>(mask), l = static_cast<AnyTensor *>(lse),
             v = static_cast<AnyTensor *>(V), a = static_cast<AnyTensor *>(A);
        auto count = [&]()
        {
            return nntile_host_tasks_submitted(dtype) + nntile_host_grid_tasks_submitted(dtype, 0)
                + starpu::direct_launches();
        };
        const int64_t before = count();
        double total = 0.0;
        auto pass = [&]()
        {
            tensor::fill_async(-__builtin_huge_valf(), get<fp32_t>(l));
            if(dtype == DT_BF16) run_async<bf16_t>(op, k, q, m, l, v, a);
            else if(dtype == DT_FP16) run_async<fp16_t>(op, k, q, m, l, v, a);
            else run_async<fp32_t>(op, k, q, m, l, v, a);
        };
        for(int i = 0; i < warmup; ++i)
        {
            pass();
        }
        starpu::task_wait_for_all();
        const int64_t mid = count();
        total = starpu::time_on_stream_ms([&]()
        {
            for(int i = 0; i < steps; ++i)
            {
                pass();
            }
        });
        const int64_t after = count();
        (void)before;
        *ms = total / (steps > 0 ? steps : 1);
        *launches = steps > 0 ? (after - mid) / steps : 0;
        return 0;
    }
    catch(const std::exception &e) { return fail(err, errlen, e); }
}

} // extern "C"
