// Short-query / long-key attention for fp32 tiles: the fp32 twin of
// sdpa_decode_16bit.hip.  The reference runs LlamaAttention.forward_dynamic
// in fp32 as well (wrappers/python/tests/model/test_llama_attention.py:296-345),
// repeating K/V per group and going through the vanilla composition
// (wrappers/python/nntile/layer/sdpa.py:407-455); here the kv_group query heads
// of one key/value head share one pass over the cache and the key axis is
// split over workgroups.
//
//  - unit = one (batch entry, kv head): its kv_group*q_seq <= 64 query rows, 16
//    per wavefront, share every K/V byte;
//  - a workgroup (4 wavefronts) streams its range of 32-key steps HBM -> LDS
//    through a ring of two buffers of 2 x 16 KiB (head 128): 64 KiB, two
//    workgroups a CU;
//  - S^T = K Q^T and O^T += V^T P^T with v_mfma_f32_16x16x4_f32; the
//    accumulator layout of S^T (lane = query row, registers = 4 consecutive
//    keys) is the B operand layout of the second product, so the
//    probabilities never leave the registers;
//  - partial (max, sum) and the normalised partial output of every split go to
//    the workspace in fp32; a second small kernel merges the splits and folds
//    the result into (lse, A) by the rule of accumulate_attn_output
//    (src/kernel/accumulate_attn_output/cpu.cc:38-115).
//
// Bound: at cfg4's shape in fp32 (541 MB, 17.2 GFLOP) the fp32 matrix rate
// (157.3 TFLOP/s: 110 us) and the HBM stream (98 us at 5.5 TB/s) are about
// equally far.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "../../include/nntile_hip_sdpa.h"
#include "sdpa_common.hpp"

namespace nntile_hip
{

constexpr int kDecF32Keys = 32;         // keys per step
constexpr int kDecF32Threads = 256;
constexpr int kDecF32CUs = 256;

template<int N> __device__ __forceinline__ void f32dec_wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
    asm volatile("" ::: "memory");
}

// Row of the output tiles that row rr of a unit is: rr = g*q_seq + tok, query
// batch entry nb + n_batch*(g + kv_group*hkv).
__device__ __forceinline__ int64_t f32dec_row(const DecodeParams &p, int unit, int rr)
{
    const int nb = unit % p.n_batch, hkv = unit / p.n_batch;
    const int g = rr / (int)p.q_seq, tok = rr % (int)p.q_seq;
    const int64_t qb = nb + (int64_t)p.n_batch * (g + (int64_t)p.kv_group * hkv);
    return qb * p.q_seq + tok;
}

template<int HEAD, int MODE>
__global__ __launch_bounds__(kDecF32Threads, 2)
void sdpa_decode_fp32_kernel(const DecodeParams p)
{
    constexpr int KT = HEAD / 16;           // 16-byte operand reads along head per 16-key block of S
    constexpr int DBLOCKS = HEAD / 16;      // 16-row blocks of O^T
    constexpr int KB = kDecF32Keys / 16;    // 16-key blocks of S^T per step
    constexpr int RB = HEAD * 4;            // bytes per K/V row
    constexpr int CPR = RB / 16;            // 16-byte chunks per row
    constexpr int ROWS_PER_LOAD = 1024 / RB;
    constexpr int LOADS = kDecF32Keys / ROWS_PER_LOAD;  // per K (or V) step
    constexpr int LOADS_PER_WAVE = LOADS / 4;
    constexpr int K_BYTES = kDecF32Keys * RB;
    constexpr int STAGE_BYTES = 2 * K_BYTES;            // K then V
    constexpr bool EXPLICIT = (MODE == NNTILE_HIP_MASK_ADDITIVE
            || MODE == NNTILE_HIP_MASK_BOOL);
    static_assert(LOADS_PER_WAVE >= 1 && CPR >= 16, "head size does not fit this tiling");
    static_assert(2 * LOADS_PER_WAVE < 64, "vmcnt");

    __shared__ __attribute__((aligned(1024))) char ring0[STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring1[STAGE_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int col = lane & 15;       // row (query) within the wavefront; key within a block for operand reads
    const int quad = lane >> 4;      // 0..3

    // Behind the units x splits attention workgroups the grid holds, when rows
    // are being appended to the caches by this call, one copying workgroup per
    // unit: the new rows into the caches, 16 bytes a thread and piece.  Nobody
    // in this launch reads them there (the attention takes them from k_new /
    // v_new), so there is nothing to wait for or to signal.
    {
        const int n_main = p.n_batch * p.n_head_kv * p.n_splits;
        if((int)blockIdx.x >= n_main)
        {
            const int unit_a = (int)blockIdx.x - n_main;
            const int64_t filled = p.k_seq - p.n_new;
            const int n16 = p.n_new * (RB / 16);
            for(int t = tid; t < 2 * n16; t += kDecF32Threads)
            {
                const int which = t >= n16 ? 1 : 0;
                const int piece = t - which * n16;
                const char *src = static_cast<const char *>(which ? p.v_new : p.k_new)
                    + ((int64_t)unit_a * p.n_new * RB + (int64_t)piece * 16);
                char *dst = static_cast<char *>(const_cast<void *>(which ? p.V : p.K))
                    + (((int64_t)unit_a * p.kv_rows + filled) * RB + (int64_t)piece * 16);
                *reinterpret_cast<f32x4 *>(dst) = *reinterpret_cast<const f32x4 *>(src);
            }
            return;
        }
    }

    // Workgroups go round the 8 XCDs in index order: all key splits of a unit
    // get indices that are equal modulo 8, i.e. one XCD and one L2 for the
    // unit's K/V (the four wavefronts' query heads read them once).
    int split, unit;
    {
        const int units = p.n_batch * p.n_head_kv;
        if(units % 8 == 0)
        {
            const int x = blockIdx.x & 7, j = blockIdx.x >> 3;
            unit = (j / p.n_splits) * 8 + x;
            split = j % p.n_splits;
        }
        else
        {
            split = blockIdx.x % p.n_splits;
            unit = blockIdx.x / p.n_splits;
        }
    }

    const int rr = wave * 16 + col;
    const bool row_ok = rr < p.rows;
    // a wavefront none of whose 16 rows exists (one new token of a group of
    // four: three of the four) takes part in the loads and barriers only
    const bool wave_idle = __builtin_amdgcn_readfirstlane(wave) * 16 >= p.rows;
    const int tok = row_ok ? rr % (int)p.q_seq : 0;
    const int64_t my_qpos = p.q_pos0 + tok;

    // Q fragments, B operand: the MFMA's contraction index is free to mean any
    // head value as long as both operands agree; lane (row, quad) holds head
    // values 16*t + 4*quad + e for the four MFMAs e of group t, which is one
    // 16-byte load here and one 16-byte LDS read of K.
    f32x4 qf[KT];
    {
        const float *src = static_cast<const float *>(p.Q)
            + f32dec_row(p, unit, row_ok ? rr : 0) * HEAD + 4 * quad;
#pragma unroll
        for(int t = 0; t < KT; ++t)
        {
            qf[t] = row_ok ? *reinterpret_cast<const f32x4 *>(src + 16 * t)
                : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }

    const char *Kb = static_cast<const char *>(p.K) + (int64_t)unit * p.kv_rows * RB;
    const char *Vb = static_cast<const char *>(p.V) + (int64_t)unit * p.kv_rows * RB;

    // ---- LDS layout ------------------------------------------------------------
    // Rows of RB bytes, unpadded; 16-byte chunk c of row r sits at position
    //   K:  c ^ (r % 16)              operand read: 16 consecutive rows, one chunk -> 16 positions
    //   V:  c ^ (4 * ((r / 4) % 4))   operand read: 4 rows 4 apart x 4 neighbouring chunks -> 16 positions
    // Load instruction `ld` fills rows [ld*ROWS_PER_LOAD, +ROWS_PER_LOAD): lane L
    // lands on row ld*ROWS_PER_LOAD + L/CPR at position L % CPR and fetches the
    // chunk that belongs there.
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    uint32_t k_goff[LOADS_PER_WAVE], v_goff[LOADS_PER_WAVE];
    int ld_row[LOADS_PER_WAVE];
#pragma unroll
    for(int i = 0; i < LOADS_PER_WAVE; ++i)
    {
        const int r = (wave * LOADS_PER_WAVE + i) * ROWS_PER_LOAD + lane / CPR;
        const int pos = lane % CPR;
        ld_row[i] = r;
        k_goff[i] = (uint32_t)(r * RB + (pos ^ (r % 16)) * 16);
        v_goff[i] = (uint32_t)(r * RB + (pos ^ (4 * ((r / 4) % 4))) * 16);
    }
    // S operand: lane (col, quad) reads key row 16*kb + col, chunk 4*t + quad
    uint32_t k_raddr[KT];
#pragma unroll
    for(int t = 0; t < KT; ++t)
    {
        k_raddr[t] = (uint32_t)(col * RB + ((4 * t + quad) ^ col) * 16);
    }
    // PV operand: lane (col, quad) reads head value 16*db + col of key row
    // 16*kb + 4*quad + e; 16*kb + e goes into the immediate offset
    uint32_t v_raddr[DBLOCKS];
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
        v_raddr[db] = (uint32_t)(K_BYTES + (4 * quad) * RB
                + ((4 * db + (col >> 2)) ^ (4 * quad)) * 16 + (col & 3) * 4);
    }

    // Loads of key step `step` into a ring slot; rows past the end of the
    // keys are clamped to the last row (their probabilities are exactly 0).
    auto fetch = [&](int step, char *slot_base)
    {
        const int64_t row0 = (int64_t)step * kDecF32Keys;
        const char *Kp = Kb + row0 * RB;
        const char *Vp = Vb + row0 * RB;
        char *kdst = slot_base + wave_u * LOADS_PER_WAVE * 1024;
        char *vdst = kdst + K_BYTES;
        const int last = (int)min((int64_t)kDecF32Keys, p.k_seq - row0) - 1;
        if(p.n_new > 0 && row0 + kDecF32Keys > p.k_seq - p.n_new)
        {
            // some rows of this step are new tokens: they are not in the caches
            // yet and are read from where the caller holds them (rows past
            // the end clamped to the last row, as below)
            const int64_t filled = p.k_seq - p.n_new;
            const char *Kn = static_cast<const char *>(p.k_new) + (int64_t)unit * p.n_new * RB;
            const char *Vn = static_cast<const char *>(p.v_new) + (int64_t)unit * p.n_new * RB;
#pragma unroll
            for(int i = 0; i < LOADS_PER_WAVE; ++i)
            {
                const int64_t g = min(row0 + ld_row[i], p.k_seq - 1);
                const uint32_t kc = k_goff[i] - (uint32_t)(ld_row[i] * RB);     // the chunk within the row
                const uint32_t vc = v_goff[i] - (uint32_t)(ld_row[i] * RB);
                const bool fresh = g >= filled;
                const char *ks = fresh ? Kn + (g - filled) * RB : Kb + g * RB;
                const char *vs = fresh ? Vn + (g - filled) * RB : Vb + g * RB;
                load_to_lds16<0, true>(ks + kc, kdst + i * 1024);
                load_to_lds16<0, true>(vs + vc, vdst + i * 1024);
            }
            return;
        }
#pragma unroll
        for(int i = 0; i < LOADS_PER_WAVE; ++i)
        {
            const uint32_t back = (uint32_t)(max(ld_row[i] - last, 0) * RB);
            load_to_lds16<0, true>(Kp + (k_goff[i] - back), kdst + i * 1024);
            load_to_lds16<0, true>(Vp + (v_goff[i] - back), vdst + i * 1024);
        }
    };

    const int step_lo = split * p.steps_per_split;
    const int step_hi = min(step_lo + p.steps_per_split, p.n_steps);
    const int n_local = max(step_hi - step_lo, 0);
    const float c = EXPLICIT ? kLog2e : p.scale * kLog2e;

    f32x4 o[DBLOCKS];
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
        o[db] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    float m_run = neg_inf();
    float l_run = 0.0f;

    if(n_local > 0)
    {
        fetch(step_lo, ring0);
    }

    auto body = [&](int it, auto slot_tag)
    {
        constexpr int SLOT = decltype(slot_tag)::value;
        const int step = step_lo + it;
        // this step's data has landed, for every wavefront, and everyone is
        // done with the other slot (a bare barrier: LDS reads are ordered by
        // lgkmcnt, the loads by the explicit vmcnt)
        f32dec_wait_vmcnt<0>();
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if(it + 1 < n_local)
        {
            fetch(step + 1, SLOT ? ring0 : ring1);
        }
        const char *Ks = SLOT ? ring1 : ring0;
        if(wave_idle)
        {
            return;
        }

        const int64_t k_row0 = (int64_t)step * kDecF32Keys;
        const int64_t k_pos_base = p.k_pos0 + k_row0;
        const int keys_here = (int)min((int64_t)kDecF32Keys, p.k_seq - k_row0);

        // ---- S^T = K Q^T: blocks of 16 keys ------------------------------------
        f32x4 s[KB];
#pragma unroll
        for(int kb = 0; kb < KB; ++kb)
        {
            s[kb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for(int t = 0; t < KT; ++t)
            {
                const f32x4 a = *reinterpret_cast<const f32x4 *>(
                        Ks + k_raddr[t] + kb * 16 * RB);
#pragma unroll
                for(int e = 0; e < 4; ++e)
                {
                    s[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], qf[t][e], s[kb],
                            0, 0, 0);
                }
            }
        }

        // ---- mask: s[kb][e] is key 16*kb + 4*quad + e --------------------------
        if(EXPLICIT)
        {
            // the mask is [k_seq, q_seq]: row index = token; keys past the end
            // of a ragged step are hidden, their loads clamped to the step's
            // last key instead of being branched around
            const int64_t mrow = (int64_t)tok * p.mask_ld + k_row0;
#pragma unroll
            for(int kb = 0; kb < KB; ++kb)
            {
                const int key0 = 16 * kb + 4 * quad;
#pragma unroll
                for(int e = 0; e < 4; ++e)
                {
                    const int64_t mi = mrow + max(min(key0 + e, keys_here - 1), 0);
                    float add;
                    if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                    {
                        add = static_cast<const float *>(p.mask)[mi];
                    }
                    else
                    {
                        add = static_cast<const uint8_t *>(p.mask)[mi] != 0 ? 0.0f : neg_inf();
                    }
                    if(key0 + e >= keys_here)
                    {
                        add = neg_inf();
                    }
                    const float v = s[kb][e] * p.scale + add;
                    s[kb][e] = (add == neg_inf()) ? neg_inf() : v;
                }
            }
        }
        else
        {
            const bool ragged = keys_here < kDecF32Keys;
            const bool diagonal = (MODE == NNTILE_HIP_MASK_CAUSAL)
                && (k_pos_base + kDecF32Keys - 1 > p.q_pos0 + p.causal_offset);
            if(ragged || diagonal)
            {
                const int64_t vis = (MODE == NNTILE_HIP_MASK_CAUSAL)
                    ? (my_qpos + p.causal_offset - k_pos_base)
                    : (int64_t)kDecF32Keys;
                const int lim = (int)max((int64_t)-1, min(vis, (int64_t)keys_here - 1));
#pragma unroll
                for(int kb = 0; kb < KB; ++kb)
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
        for(int kb = 0; kb < KB; ++kb)
        {
#pragma unroll
            for(int e = 0; e < 4; ++e)
            {
                mx = fmaxf(mx, s[kb][e]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = max_across_halves(mx);
        const float m_new = fmaxf(m_run, mx);
        const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
        const float mc = m_use * c;
        if(__builtin_amdgcn_ballot_w64(m_new != m_run) != 0)
        {
            const float alpha = fast_exp2((m_run - m_use) * c);
            l_run *= alpha;
#pragma unroll
            for(int db = 0; db < DBLOCKS; ++db)
            {
                o[db] *= alpha;
            }
            m_run = m_new;
        }
        float rs = 0.0f;
#pragma unroll
        for(int kb = 0; kb < KB; ++kb)
        {
#pragma unroll
            for(int e = 0; e < 4; ++e)
            {
                s[kb][e] = fast_exp2(fmaf(s[kb][e], c, -mc));
                rs += s[kb][e];
            }
        }
        l_run += rs;

        // ---- O^T += V^T P^T ------------------------------------------------------
        // MFMA (kb, e) contracts over the keys 16*kb + 4*quad' + e, quad' = 0..3:
        // its B operand is register e of block kb as it stands.  The operand
        // reads of a key block come first, then its MFMAs.
#pragma unroll
        for(int kb = 0; kb < KB; ++kb)
        {
#pragma unroll
            for(int e = 0; e < 4; ++e)
            {
                float a[DBLOCKS];
#pragma unroll
                for(int db = 0; db < DBLOCKS; ++db)
                {
                    a[db] = *reinterpret_cast<const float *>(
                            Ks + v_raddr[db] + (16 * kb + e) * RB);
                }
#pragma unroll
                for(int db = 0; db < DBLOCKS; ++db)
                {
                    o[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[db], s[kb][e], o[db],
                            0, 0, 0);
                }
            }
        }
    };

    for(int it = 0; it < n_local; it += 2)
    {
        body(it, std::integral_constant<int, 0>{});
        if(it + 1 < n_local)
        {
            body(it + 1, std::integral_constant<int, 1>{});
        }
    }

    // ---- the partial: (max in natural-log units, sum) and the normalised output
    float l_tot = l_run + __shfl_xor(l_run, 16);
    l_tot = sum_across_halves(l_tot);
    if(!row_ok)
    {
        return;
    }
    const int64_t prow = ((int64_t)unit * p.n_splits + split) * p.rows + rr;
    if(quad == 0)
    {
        const float to_ln = EXPLICIT ? 1.0f : p.scale;
        p.part_ml[2 * prow] = (m_run == neg_inf()) ? neg_inf() : m_run * to_ln;
        p.part_ml[2 * prow + 1] = l_tot;
    }
    // o[db][r] is head value 16*db + 4*quad + r of row rr
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    float *dst = p.part_o + prow * HEAD + 4 * quad;
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
        *reinterpret_cast<f32x4 *>(dst + 16 * db) = o[db] * inv;
    }
}

// Merge the split partials of each row and fold the result into (lse, A).  A
// thread handles 4 head values of one row; a workgroup of 256 threads handles
// 1024/HEAD rows.
template<int HEAD>
__global__ __launch_bounds__(256)
void sdpa_decode_fp32_reduce_kernel(const DecodeParams p)
{
    constexpr int TPR = HEAD / 4;               // threads per row
    constexpr int ROWS_PER_WG = 256 / TPR;
    const int tid = threadIdx.x;
    const int64_t grow = (int64_t)blockIdx.x * ROWS_PER_WG + tid / TPR;
    const int64_t total = (int64_t)p.n_batch * p.n_head_kv * p.rows;
    if(grow >= total)
    {
        return;
    }
    const int unit = (int)(grow / p.rows), rr = (int)(grow % p.rows);
    const int d4 = (tid % TPR) * 4;
    const int64_t base = (int64_t)unit * p.n_splits * p.rows + rr;
    // eight splits at a time, all their loads issued before anything is used
    // (a loop of dependent trips to memory otherwise: 10.5 us for cfg4's shape)
    const int64_t row = f32dec_row(p, unit, rr);
    float *Adst = static_cast<float *>(p.A) + row * HEAD + d4;
    typedef __attribute__((ext_vector_type(2))) float f32x2;
    float top = neg_inf();
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    float wsum = 0.0f;
    for(int s0 = 0; s0 < p.n_splits; s0 += 8)
    {
        f32x2 ml[8];
        f32x4 v[8];
#pragma unroll
        for(int j = 0; j < 8; ++j)
        {
            // (splits past the last re-read the last one and get weight 0)
            const int64_t prow = base + (int64_t)min(s0 + j, p.n_splits - 1) * p.rows;
            ml[j] = *reinterpret_cast<const f32x2 *>(p.part_ml + 2 * prow);
            v[j] = *reinterpret_cast<const f32x4 *>(p.part_o + prow * HEAD + d4);
        }
        float lse_s[8];
        float top8 = top;
#pragma unroll
        for(int j = 0; j < 8; ++j)
        {
            const bool there = s0 + j < p.n_splits && ml[j][0] != neg_inf() && ml[j][1] > 0.0f;
            lse_s[j] = there ? ml[j][0] + __logf(ml[j][1]) : neg_inf();
            top8 = fmaxf(top8, lse_s[j]);
        }
        if(top8 == neg_inf())
        {
            continue;       // nothing visible so far
        }
        // what was accumulated against the old reference point
        const float rescale = (top == neg_inf()) ? 0.0f : __expf(top - top8);
        acc *= rescale;
        wsum *= rescale;
        top = top8;
#pragma unroll
        for(int j = 0; j < 8; ++j)
        {
            const float w = (lse_s[j] == neg_inf()) ? 0.0f : __expf(lse_s[j] - top);
            wsum += w;
            acc += w * v[j];
        }
    }
    if(top == neg_inf())
    {
        // no visible key at all: leave lse and A untouched, or write the
        // empty row when the running pair is being overwritten
        if(p.overwrite)
        {
            *reinterpret_cast<f32x4 *>(Adst) = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            if(d4 == 0)
            {
                p.lse[row] = neg_inf();
            }
        }
        return;
    }
    const float lse_new = top + __logf(wsum);
    const float lse_old = p.overwrite ? neg_inf() : p.lse[row];
    float w_old, w_new, lse_out;
    merge_weights(lse_old, lse_new, w_old, w_new, lse_out);
    f32x4 v = acc * (w_new / wsum);
    if(w_old != 0.0f)
    {
        v += w_old * *reinterpret_cast<const f32x4 *>(Adst);
    }
    *reinterpret_cast<f32x4 *>(Adst) = v;
    // The threads of a row sit in one wavefront (TPR <= 32 divides 64) and
    // run in lock step: all of them have read lse_old by now.
    if(d4 == 0)
    {
        p.lse[row] = lse_out;
    }
}

int decode_fp32_steps(int64_t k_seq)
{
    return (int)((k_seq + kDecF32Keys - 1) / kDecF32Keys);
}

// Key splits per unit: two workgroups per CU when the units allow it, never
// more than one split per key step.
int decode_fp32_choose_splits(int units, int n_steps)
{
    int splits = (2 * kDecF32CUs + units - 1) / units;
    splits = splits < 1 ? 1 : splits;
    splits = splits > n_steps ? n_steps : splits;
    return splits > 64 ? 64 : splits;
}

// The workspace: the partial outputs [unit][split][rows][head] and the (max,
// sum) pairs [unit][split][rows][2], both fp32
size_t decode_fp32_workspace_bytes(int units, int n_splits, int rows, int head)
{
    return (size_t)units * n_splits * rows * (head + 2) * sizeof(float);
}

template<int HEAD>
static int launch_decode_fp32_head(hipStream_t stream, const DecodeParams &p, int mode)
{
    const int units = p.n_batch * p.n_head_kv;
    // (one more workgroup per unit when the call appends rows to the caches)
    const dim3 grid((unsigned)(units * p.n_splits + (p.n_new > 0 ? units : 0))),
        block(kDecF32Threads);
    switch(mode)
    {
        case NNTILE_HIP_MASK_ADDITIVE:
            hipLaunchKernelGGL((sdpa_decode_fp32_kernel<HEAD, NNTILE_HIP_MASK_ADDITIVE>), grid,
                    block, 0, stream, p);
            break;
        case NNTILE_HIP_MASK_NONE:
            hipLaunchKernelGGL((sdpa_decode_fp32_kernel<HEAD, NNTILE_HIP_MASK_NONE>), grid,
                    block, 0, stream, p);
            break;
        case NNTILE_HIP_MASK_CAUSAL:
            hipLaunchKernelGGL((sdpa_decode_fp32_kernel<HEAD, NNTILE_HIP_MASK_CAUSAL>), grid,
                    block, 0, stream, p);
            break;
        case NNTILE_HIP_MASK_BOOL:
            hipLaunchKernelGGL((sdpa_decode_fp32_kernel<HEAD, NNTILE_HIP_MASK_BOOL>), grid,
                    block, 0, stream, p);
            break;
        default:
            return NNTILE_HIP_EINVAL;
    }
    if(hipGetLastError() != hipSuccess)
    {
        return NNTILE_HIP_ELAUNCH;
    }
    constexpr int rows_per_wg = 256 / (HEAD / 4);
    const int64_t total_rows = (int64_t)units * p.rows;
    hipLaunchKernelGGL((sdpa_decode_fp32_reduce_kernel<HEAD>),
            dim3((unsigned)((total_rows + rows_per_wg - 1) / rows_per_wg)), dim3(256), 0,
            stream, p);
    return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
}

// p: fully filled but for nothing; part_o and part_ml point into the
// workspace, n_splits / n_steps / steps_per_split from the functions above.
int launch_decode_fp32(hipStream_t stream, const DecodeParams &p, int head, int mode)
{
    switch(head)
    {
        case 64:
            return launch_decode_fp32_head<64>(stream, p, mode);
        case 128:
            return launch_decode_fp32_head<128>(stream, p, mode);
        default:
            return NNTILE_HIP_EUNSUPPORTED;
    }
}

} // namespace nntile_hip
