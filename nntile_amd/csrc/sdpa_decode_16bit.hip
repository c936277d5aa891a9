// Short-query / long-key attention forward (decode against a KV cache) for
// 16-bit tiles on gfx950.  The shape is bound by the one pass over K and V in
// HBM, so the kernel is built around that stream:
//
//  * all kv_group query heads that share one key/value head are processed
//    together (rows = kv_group * q_seq <= 64), so K and V are read once, not
//    once per query head;
//  * the key axis of each (batch entry, kv head) unit is split over
//    workgroups so that every CU streams; each workgroup writes an
//    un-normalised partial (max, sum, O) and a second small kernel merges the
//    partials and folds them into the running (lse, A) pair;
//  * global loads are 16 bytes per lane over contiguous rows, staged through
//    LDS; a wavefront owns 16 rows and uses v_mfma_f32_16x16x32 (S^T = K Q^T,
//    O^T += V^T P^T with P^T taken from the S^T accumulators; V is transposed
//    on its way into LDS, keys stored in the order the accumulators list them).
#include "sdpa_common.hpp"

namespace nntile_hip
{


constexpr int kDecKeys = 64;      // keys per step
constexpr int kDecThreads = 256;


typedef __attribute__((ext_vector_type(4))) float acc4;

template<typename T> struct Mfma16;
template<> struct Mfma16<Bf16>
{
    static __device__ __forceinline__ acc4 run(bf16x8 a, bf16x8 b, acc4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};
template<> struct Mfma16<Fp16>
{
    static __device__ __forceinline__ acc4 run(f16x8 a, f16x8 b, acc4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};

template<typename T, int HEAD, int MODE>
__global__ __launch_bounds__(kDecThreads, 3)
void sdpa_decode_16bit_kernel(const DecodeParams p)
{
    typedef typename T::vec8 vec8;
    constexpr int KSTEPS = HEAD / 32;       // MFMA steps along head for S
    constexpr int DBLOCKS = HEAD / 16;      // 16-row blocks of O^T
    constexpr int KPAD = HEAD + 8;
    constexpr int VPAD = kDecKeys + 8;
    constexpr int CHUNKS = HEAD / 8;
    constexpr bool EXPLICIT = (MODE == NNTILE_HIP_MASK_ADDITIVE
            || MODE == NNTILE_HIP_MASK_BOOL);

    __shared__ __attribute__((aligned(16))) uint16_t Ks[kDecKeys * KPAD];
    __shared__ __attribute__((aligned(16))) uint16_t Vt[HEAD * VPAD];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int col = lane & 15;       // row (query) within the wavefront
    const int quad = lane >> 4;      // 0..3

    const int split = blockIdx.x % p.n_splits;
    const int unit = blockIdx.x / p.n_splits;        // nb + n_batch*hkv
    const int nb = unit % p.n_batch;
    const int hkv = unit / p.n_batch;

    // Row of this lane: rr = g*q_seq + tok.
    const int rr = wave * 16 + col;
    const bool row_ok = rr < p.rows;
    const int g = row_ok ? rr / (int)p.q_seq : 0;
    const int tok = row_ok ? rr % (int)p.q_seq : 0;
    const int64_t qb = nb + (int64_t)p.n_batch * (g + (int64_t)p.kv_group * hkv);
    const int64_t my_qpos = p.q_pos0 + tok;

    // Q fragments: B operand, lane (row, quad) holds head values
    // 32*ks + 8*quad .. +7.
    vec8 qf[KSTEPS];
    {
        const uint16_t *src = static_cast<const uint16_t *>(p.Q)
            + (qb * p.q_seq + tok) * HEAD + quad * 8;
#pragma unroll
        for(int ks = 0; ks < KSTEPS; ++ks)
        {
            u32x4 raw = row_ok ? *reinterpret_cast<const u32x4 *>(src + ks * 32)
                : u32x4{0, 0, 0, 0};
            qf[ks] = __builtin_bit_cast(vec8, raw);
        }
    }

    const uint16_t *Kb = static_cast<const uint16_t *>(p.K)
        + (int64_t)unit * p.k_seq * HEAD;
    const uint16_t *Vb = static_cast<const uint16_t *>(p.V)
        + (int64_t)unit * p.k_seq * HEAD;

    // Cooperative loads (see the prefill kernel): K plain, V regrouped.
    constexpr int K_ROWS_PER_PASS = kDecThreads / CHUNKS;
    constexpr int K_PASSES = kDecKeys / K_ROWS_PER_PASS;
    const int k_chunk = tid % CHUNKS;
    const int k_row = tid / CHUNKS;
    constexpr int V_UNITS = 16 * CHUNKS;
    const bool v_active = tid < V_UNITS;
    const int v_kg = tid & 15;
    const int v_chunk = tid >> 4;
    // LDS position of keys 4*kg..4*kg+3: within each group of 32 keys the
    // order is [quad][a][c] for key = 16a + 4*quad + c.
    const int v_pos = 32 * (v_kg >> 3) + 8 * (v_kg & 3) + 4 * ((v_kg & 7) >> 2);

    u32x4 k_regs[K_PASSES];
    u32x4 v_regs[4];

    auto fetch = [&](int step)
    {
        const int64_t row0 = (int64_t)step * kDecKeys;
#pragma unroll
        for(int i = 0; i < K_PASSES; ++i)
        {
            const int64_t r = row0 + k_row + i * K_ROWS_PER_PASS;
            k_regs[i] = (r < p.k_seq)
                ? __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(
                            Kb + r * HEAD + k_chunk * 8))
                : u32x4{0, 0, 0, 0};
        }
        if(v_active)
        {
#pragma unroll
            for(int j = 0; j < 4; ++j)
            {
                const int64_t r = row0 + 4 * v_kg + j;
                v_regs[j] = (r < p.k_seq)
                    ? __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(
                                Vb + r * HEAD + v_chunk * 8))
                    : u32x4{0, 0, 0, 0};
            }
        }
    };

    auto stage = [&]()
    {
#pragma unroll
        for(int i = 0; i < K_PASSES; ++i)
        {
            *reinterpret_cast<u32x4 *>(&Ks[(k_row + i * K_ROWS_PER_PASS) * KPAD
                    + k_chunk * 8]) = k_regs[i];
        }
        if(v_active)
        {
#pragma unroll
            for(int w = 0; w < 4; ++w)
            {
                const uint32_t r0 = v_regs[0][w], r1 = v_regs[1][w],
                      r2 = v_regs[2][w], r3 = v_regs[3][w];
                u32x2 even, odd;
                even[0] = __builtin_amdgcn_perm(r1, r0, 0x05040100u);
                even[1] = __builtin_amdgcn_perm(r3, r2, 0x05040100u);
                odd[0] = __builtin_amdgcn_perm(r1, r0, 0x07060302u);
                odd[1] = __builtin_amdgcn_perm(r3, r2, 0x07060302u);
                const int d = v_chunk * 8 + 2 * w;
                *reinterpret_cast<u32x2 *>(&Vt[d * VPAD + v_pos]) = even;
                *reinterpret_cast<u32x2 *>(&Vt[(d + 1) * VPAD + v_pos]) = odd;
            }
        }
    };

    const int step_lo = split * p.steps_per_split;
    const int step_hi = min(step_lo + p.steps_per_split, p.n_steps);
    const float c = EXPLICIT ? kLog2e : p.scale * kLog2e;

    acc4 o[DBLOCKS];
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
        o[db] = acc4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    float m_run = neg_inf();
    float l_run = 0.0f;

    if(step_lo < step_hi)
    {
        fetch(step_lo);
    }
    for(int step = step_lo; step < step_hi; ++step)
    {
        __syncthreads();
        stage();
        __syncthreads();
        if(step + 1 < step_hi)
        {
            fetch(step + 1);
        }
        const int64_t k_row0 = (int64_t)step * kDecKeys;
        const int64_t k_pos_base = p.k_pos0 + k_row0;
        const int keys_here = (int)min((int64_t)kDecKeys, p.k_seq - k_row0);

        // ---- S^T = K Q^T: 4 blocks of 16 keys ----------------------------------
        acc4 s[4];
#pragma unroll
        for(int kb = 0; kb < 4; ++kb)
        {
            s[kb] = acc4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for(int ks = 0; ks < KSTEPS; ++ks)
            {
                const vec8 a = *reinterpret_cast<const vec8 *>(
                        &Ks[(kb * 16 + col) * KPAD + ks * 32 + quad * 8]);
                s[kb] = Mfma16<T>::run(a, qf[ks], s[kb]);
            }
        }

        // ---- mask: s[kb][r] is key 16*kb + 4*quad + r ----------------------------
        if(EXPLICIT)
        {
            // the mask is [k_seq, q_seq]: row index = token
#pragma unroll
            for(int kb = 0; kb < 4; ++kb)
            {
                const int key0 = 16 * kb + 4 * quad;
#pragma unroll
                for(int e = 0; e < 4; ++e)
                {
                    float add;
                    const int64_t mi = (int64_t)tok * p.mask_ld + k_row0 + key0 + e;
                    if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                    {
                        add = (key0 + e < keys_here)
                            ? T::to_float(static_cast<const uint16_t *>(p.mask)[mi])
                            : neg_inf();
                    }
                    else
                    {
                        add = (key0 + e < keys_here
                                && static_cast<const uint8_t *>(p.mask)[mi] != 0)
                            ? 0.0f : neg_inf();
                    }
                    const float v = s[kb][e] * p.scale + add;
                    s[kb][e] = (add == neg_inf()) ? neg_inf() : v;
                }
            }
        }
        else
        {
            const bool ragged = keys_here < kDecKeys;
            const bool diagonal = (MODE == NNTILE_HIP_MASK_CAUSAL)
                && (k_pos_base + kDecKeys - 1 > p.q_pos0 + p.causal_offset);
            if(ragged || diagonal)
            {
                const int64_t vis = (MODE == NNTILE_HIP_MASK_CAUSAL)
                    ? (my_qpos + p.causal_offset - k_pos_base)
                    : (int64_t)kDecKeys;
                const int lim = (int)max((int64_t)-1,
                        min(vis, (int64_t)keys_here - 1));
#pragma unroll
                for(int kb = 0; kb < 4; ++kb)
                {
#pragma unroll
                    for(int e = 0; e < 4; ++e)
                    {
                        if(16 * kb + 4 * quad + e > lim)
                        {
                            s[kb][e] = neg_inf();
                        }
                    }
                }
            }
        }

        // ---- online softmax ---------------------------------------------------
        float mx = neg_inf();
#pragma unroll
        for(int kb = 0; kb < 4; ++kb)
        {
#pragma unroll
            for(int e = 0; e < 4; ++e)
            {
                mx = fmaxf(mx, s[kb][e]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
        const float alpha = fast_exp2((m_run - m_use) * c);
        const float mc = m_use * c;
        m_run = m_new;
        float rs = 0.0f;
        uint32_t pk[4][2];
#pragma unroll
        for(int kb = 0; kb < 4; ++kb)
        {
            const float p0 = fast_exp2(fmaf(s[kb][0], c, -mc));
            const float p1 = fast_exp2(fmaf(s[kb][1], c, -mc));
            const float p2 = fast_exp2(fmaf(s[kb][2], c, -mc));
            const float p3 = fast_exp2(fmaf(s[kb][3], c, -mc));
            rs += (p0 + p1) + (p2 + p3);
            pk[kb][0] = T::pack2(p0, p1);
            pk[kb][1] = T::pack2(p2, p3);
        }
        l_run = l_run * alpha + rs;
#pragma unroll
        for(int db = 0; db < DBLOCKS; ++db)
        {
            o[db] *= alpha;
        }

        // ---- O^T += V^T P^T: 2 steps of 32 keys ----------------------------------
#pragma unroll
        for(int t = 0; t < 2; ++t)
        {
            const u32x4 praw = {pk[2 * t][0], pk[2 * t][1], pk[2 * t + 1][0],
                pk[2 * t + 1][1]};
            const vec8 pb = __builtin_bit_cast(vec8, praw);
#pragma unroll
            for(int db = 0; db < DBLOCKS; ++db)
            {
                const vec8 a = *reinterpret_cast<const vec8 *>(
                        &Vt[(db * 16 + col) * VPAD + 32 * t + 8 * quad]);
                o[db] = Mfma16<T>::run(a, pb, o[db]);
            }
        }
    }

    // ---- write the partial ---------------------------------------------------------
    float l_tot = l_run + __shfl_xor(l_run, 16);
    l_tot += __shfl_xor(l_tot, 32);
    if(!row_ok)
    {
        return;
    }
    const int64_t prow = ((int64_t)unit * p.n_splits + split) * p.rows + rr;
    if(quad == 0)
    {
        // max in natural-log units so that the reduce kernel needs no mode
        const float to_ln = EXPLICIT ? 1.0f : p.scale;
        p.part_ml[2 * prow] = (m_run == neg_inf()) ? neg_inf() : m_run * to_ln;
        p.part_ml[2 * prow + 1] = l_tot;
    }
    // o[db][r] is head value 16*db + 4*quad + r of row rr
    float *dst = p.part_o + prow * HEAD + 4 * quad;
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
        *reinterpret_cast<acc4 *>(dst + 16 * db) = o[db];
    }
}

// Merge the split partials of each row and fold the result into (lse, A).
// One workgroup of HEAD threads per (unit, row).
template<typename T, int HEAD>
__global__ __launch_bounds__(HEAD)
void sdpa_decode_reduce_kernel(const DecodeParams p)
{
    const int rr = blockIdx.x % p.rows;
    const int unit = blockIdx.x / p.rows;
    const int nb = unit % p.n_batch;
    const int hkv = unit / p.n_batch;
    const int g = rr / (int)p.q_seq, tok = rr % (int)p.q_seq;
    const int64_t qb = nb + (int64_t)p.n_batch * (g + (int64_t)p.kv_group * hkv);
    const int d = threadIdx.x;

    const int64_t base = (int64_t)unit * p.n_splits * p.rows + rr;
    float top = neg_inf();
    for(int s = 0; s < p.n_splits; ++s)
    {
        top = fmaxf(top, p.part_ml[2 * (base + (int64_t)s * p.rows)]);
    }
    const int64_t row = qb * p.q_seq + tok;
    uint16_t *Arow = static_cast<uint16_t *>(p.A) + row * HEAD;
    if(top == neg_inf())
    {
        // no visible key at all: leave lse and A untouched, or write the
        // empty row when the running pair is being overwritten
        if(p.overwrite)
        {
            Arow[d] = 0;
            if(d == 0)
            {
                p.lse[row] = neg_inf();
            }
        }
        return;
    }
    float l = 0.0f, acc = 0.0f;
    for(int s = 0; s < p.n_splits; ++s)
    {
        const int64_t prow = base + (int64_t)s * p.rows;
        const float m = p.part_ml[2 * prow];
        if(m == neg_inf())
        {
            continue;
        }
        const float w = __expf(m - top);
        l += w * p.part_ml[2 * prow + 1];
        acc += w * p.part_o[prow * HEAD + d];
    }
    const float lse_new = top + __logf(l);
    const float lse_old = p.overwrite ? neg_inf() : p.lse[row];
    float w_old, w_new, lse_out;
    merge_weights(lse_old, lse_new, w_old, w_new, lse_out);
    float v = acc * (w_new / l);
    if(w_old != 0.0f)
    {
        v += w_old * T::to_float(Arow[d]);
    }
    Arow[d] = T::from_float(v);
    __syncthreads();    // every thread has read lse_old before it changes
    if(d == 0)
    {
        p.lse[row] = lse_out;
    }
}

template<typename T, int HEAD>
static int launch_decode_head(hipStream_t stream, const DecodeParams &p, int mode)
{
    const int units = p.n_batch * p.n_head_kv;
    const dim3 grid((unsigned)(units * p.n_splits));
    switch(mode)
    {
        case NNTILE_HIP_MASK_ADDITIVE:
            hipLaunchKernelGGL((sdpa_decode_16bit_kernel<T, HEAD,
                        NNTILE_HIP_MASK_ADDITIVE>), grid, dim3(kDecThreads), 0,
                    stream, p);
            break;
        case NNTILE_HIP_MASK_NONE:
            hipLaunchKernelGGL((sdpa_decode_16bit_kernel<T, HEAD,
                        NNTILE_HIP_MASK_NONE>), grid, dim3(kDecThreads), 0,
                    stream, p);
            break;
        case NNTILE_HIP_MASK_CAUSAL:
            hipLaunchKernelGGL((sdpa_decode_16bit_kernel<T, HEAD,
                        NNTILE_HIP_MASK_CAUSAL>), grid, dim3(kDecThreads), 0,
                    stream, p);
            break;
        case NNTILE_HIP_MASK_BOOL:
            hipLaunchKernelGGL((sdpa_decode_16bit_kernel<T, HEAD,
                        NNTILE_HIP_MASK_BOOL>), grid, dim3(kDecThreads), 0,
                    stream, p);
            break;
        default:
            return NNTILE_HIP_EINVAL;
    }
    if(hipGetLastError() != hipSuccess)
    {
        return NNTILE_HIP_ELAUNCH;
    }
    hipLaunchKernelGGL((sdpa_decode_reduce_kernel<T, HEAD>),
            dim3((unsigned)(units * p.rows)), dim3(HEAD), 0, stream, p);
    return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
}

// Number of key splits per unit: enough workgroups to give every CU several
// resident streams, never more than one split per key step.
int decode_choose_splits(int units, int n_steps)
{
    const int target_wg = 1024;     // 256 CUs x 4 resident workgroups
    int splits = (target_wg + units - 1) / units;
    splits = splits < 1 ? 1 : splits;
    splits = splits > n_steps ? n_steps : splits;
    splits = splits > 64 ? 64 : splits;
    return splits;
}

size_t decode_workspace_bytes(int units, int n_splits, int rows, int head)
{
    return (size_t)units * n_splits * rows * (head + 2) * sizeof(float);
}

template<typename T>
int launch_decode_16bit(hipStream_t stream, DecodeParams &p, int head, int mode)
{
    switch(head)
    {
        case 64:
            return launch_decode_head<T, 64>(stream, p, mode);
        case 128:
            return launch_decode_head<T, 128>(stream, p, mode);
        default:
            return NNTILE_HIP_EUNSUPPORTED;
    }
}

template int launch_decode_16bit<Bf16>(hipStream_t, DecodeParams &, int, int);
template int launch_decode_16bit<Fp16>(hipStream_t, DecodeParams &, int, int);

} // namespace nntile_hip
