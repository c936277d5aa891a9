// Prefill attention forward for fp32 tiles on gfx950.
//
// Same decomposition as the 16-bit kernel (one workgroup = 4 wavefronts = 128
// queries, S^T = K Q^T and O^T += V^T P^T with a lane owning one query), but
// on v_mfma_f32_32x32x2_f32: operands and products are true fp32, which the
// 1e-4 tolerance of the fp32 configurations needs.  Keys are walked in steps
// of 32.  With a 2-deep contraction per MFMA the lane half h supplies the
// operand element k = h, so:
//   S^T: 4 consecutive MFMAs consume one 16-byte read K[key][8j+4h .. +3]
//        against the matching 4 query values held in registers;
//   O^T: the B operand is the S^T accumulator register itself (key
//        8*(r/4) + 4h + r%4), the A operand is V[that key][d] read from LDS
//        with the head axis across lanes - no transposition is needed.
//
// SPLIT variant, for launches with fewer workgroups than CUs: a workgroup is
// 32 queries, and its four wavefronts take every fourth key step each (four
// steps are staged per iteration), then merge their (max, sum, O) through LDS.
// The chain of dependent steps a wavefront walks, which bounds such a launch,
// is a quarter as long, and four times as many workgroups spread over the CUs.
#include "sdpa_common.hpp"

namespace nntile_hip
{

// 16-byte K operand reads issued ahead of the MFMAs that use them
#ifndef NNTILE_F32_AHEAD
#define NNTILE_F32_AHEAD 2
#endif
constexpr int kQRows32 = 128;
constexpr int kKeys32 = 32;
constexpr int kThreads32 = 256;          // first form: 4 wavefronts
#ifndef NNTILE_F32_SPLIT_WAVES
#define NNTILE_F32_SPLIT_WAVES 4
#endif
// second form: wavefronts sharing the keys.  Head 64 stages 8 steps (139 KiB
// of LDS); head 128 has room for 4, head 32 has 256 16-byte chunks a step.
__host__ __device__ constexpr int split_waves32(int head)
{
    return head == 64 ? NNTILE_F32_SPLIT_WAVES : 4;
}

template<int HEAD, int MODE, bool SPLIT>
__global__ __launch_bounds__(SPLIT ? split_waves32(HEAD) * 64 : kThreads32, SPLIT ? 1 : 2)
void sdpa_prefill_fp32_kernel(const PrefillParams p)
{
    constexpr int QROWS = SPLIT ? 32 : kQRows32;    // queries per workgroup
    constexpr int THREADS = SPLIT ? split_waves32(HEAD) * 64 : kThreads32;
    constexpr int NSUB = SPLIT ? split_waves32(HEAD) : 1;   // key steps staged per iteration
    constexpr int QSTEPS = HEAD / 8;        // 16-byte groups per lane half along head
    constexpr int DBLOCKS = HEAD / 32;
    constexpr int PAD = HEAD + 4;           // row stride in LDS (floats)
    constexpr int CHUNKS = HEAD / 4;        // 16-byte chunks per row
    constexpr bool EXPLICIT = (MODE == NNTILE_HIP_MASK_ADDITIVE
            || MODE == NNTILE_HIP_MASK_BOOL);

    __shared__ __attribute__((aligned(16))) float Ks[NSUB * kKeys32 * PAD];
    __shared__ __attribute__((aligned(16))) float Vs[NSUB * kKeys32 * PAD];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int col = lane & 31;
    const int half = lane >> 5;

    const int q_blocks = p.n_q_tiles * p.q_blocks_per_tile;
    int wg = blockIdx.x;
    if(p.xcd_remap)
    {
        const int per_xcd = gridDim.x >> 3;
        wg = (wg & 7) * per_xcd + (wg >> 3);
    }
    const int b = wg / q_blocks;
    const int qblk = q_blocks - 1 - (wg % q_blocks);
    const int qt = qblk / p.q_blocks_per_tile;
    const int qb = qblk % p.q_blocks_per_tile;
    const int64_t q_len = min(p.q_tile, p.q_seq - (int64_t)qt * p.q_tile);
    const int64_t q_row0 = (int64_t)qb * QROWS;
    if(q_row0 >= q_len)
    {
        return;
    }
    const int kvb = kv_entry(b, p.n_batch, p.kv_group);

    const float *Qt = static_cast<const float *>(p.Q[qt])
        + (int64_t)b * q_len * HEAD;
    const int64_t my_q = q_row0 + (SPLIT ? 0 : wave * 32) + col;
    const bool q_ok = my_q < q_len;
    const int64_t my_qpos = p.q_pos0 + (int64_t)qt * p.q_tile + my_q;

    // Q values of this lane: for group j, head values 8j + 4*half .. +3.
    f32x4 qf[QSTEPS];
    {
        const float *src = Qt + (q_ok ? my_q : 0) * HEAD + half * 4;
#pragma unroll
        for(int j = 0; j < QSTEPS; ++j)
        {
            qf[j] = q_ok ? *reinterpret_cast<const f32x4 *>(src + j * 8)
                : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }

    const int64_t last_k_len = p.k_seq - (int64_t)(p.n_kv_tiles - 1) * p.k_tile;
    int n_steps = (p.n_kv_tiles - 1) * p.k_blocks_per_tile
        + (int)((last_k_len + kKeys32 - 1) / kKeys32);
    const int64_t wg_qpos_hi = p.q_pos0 + (int64_t)qt * p.q_tile
        + min(q_row0 + QROWS, q_len) - 1;
    const int64_t wave_qpos_lo = p.q_pos0 + (int64_t)qt * p.q_tile + q_row0
        + (SPLIT ? 0 : wave * 32);
    const int64_t wave_qpos_hi = wave_qpos_lo + 31;

    // Cooperative loads: 32 rows x CHUNKS chunks for K and for V.
    constexpr int ROWS_PER_PASS = THREADS / CHUNKS;
    static_assert(THREADS <= kKeys32 * CHUNKS, "more threads than 16-byte chunks of a step");
    constexpr int PASSES = kKeys32 / ROWS_PER_PASS;
    const int ld_chunk = tid % CHUNKS;
    const int ld_row = tid / CHUNKS;
    f32x4 k_regs[NSUB][PASSES], v_regs[NSUB][PASSES];

    // Where the rows of a key step come from.  One key tile (every tile-pair
    // call): the tile's addresses are computed once, a step needs no division
    // and no look-up in the tile table.
    struct StepSource
    {
        const float *K, *V;
        int row0, last_row;
    };
    const int64_t k_len0 = min(p.k_tile, p.k_seq);
    const bool one_tile = p.n_kv_tiles == 1;
    const int64_t entry_rows0 = p.kv_rows > 0 ? p.kv_rows : k_len0;
    const float *K0 = static_cast<const float *>(p.K[0]) + ((int64_t)kvb * entry_rows0) * HEAD;
    const float *V0 = static_cast<const float *>(p.V[0]) + ((int64_t)kvb * entry_rows0) * HEAD;
    auto locate = [&](int g, int n_steps_all) -> StepSource
    {
        // steps past the last re-read the last one (nobody uses them)
        g = min(g, max(n_steps_all - 1, 0));
        StepSource src;
        if(one_tile)
        {
            src.K = K0;
            src.V = V0;
            src.row0 = g * kKeys32;
            src.last_row = (int)k_len0 - 1;
        }
        else
        {
            const int kt = g / p.k_blocks_per_tile;
            const int kb = g % p.k_blocks_per_tile;
            const int64_t k_len = min(p.k_tile, p.k_seq - (int64_t)kt * p.k_tile);
            src.K = static_cast<const float *>(p.K[kt]) + ((int64_t)kvb * k_len) * HEAD;
            src.V = static_cast<const float *>(p.V[kt]) + ((int64_t)kvb * k_len) * HEAD;
            src.row0 = kb * kKeys32;
            src.last_row = (int)k_len - 1;
        }
        return src;
    };
    // The loads of the staged steps, one 16-byte load per thread and piece:
    // piece k is step k / (2 PASSES), pass (k / 2) % PASSES, K for even k and V
    // for odd k.  Rows past the end of the tile re-read its last row: their
    // keys are masked out of the scores, so their probabilities are exactly
    // 0, and a load that is never conditional does not make the wave wait.
    // (the launcher keeps a tile's rows x HEAD within 31 bits)
    constexpr int PIECES = NSUB * PASSES * 2;
    StepSource src[NSUB];
    auto fetch_piece = [&](int k) __attribute__((always_inline))
    {
        const int sub = k / (2 * PASSES), i = (k / 2) % PASSES;
        const uint32_t off = (uint32_t)min(src[sub].row0 + ld_row + i * ROWS_PER_PASS,
                src[sub].last_row) * HEAD + ld_chunk * 4;
        if(k % 2 == 0)
        {
            k_regs[sub][i] = *reinterpret_cast<const f32x4 *>(src[sub].K + off);
        }
        else
        {
            v_regs[sub][i] = *reinterpret_cast<const f32x4 *>(src[sub].V + off);
        }
    };
    // A wave gets one load accepted every ~70 cycles and stands still until
    // then; inside the loop the pieces therefore go between the MFMAs, which
    // run meanwhile: slot t of SLOTS takes the pieces k with k*SLOTS/PIECES == t.
    constexpr int SLOTS = QSTEPS + 16;
    auto fetch_slot = [&](int t) __attribute__((always_inline))
    {
#pragma unroll
        for(int k = 0; k < PIECES; ++k)
        {
            if(k * SLOTS / PIECES == t)
            {
                fetch_piece(k);
            }
        }
    };

    auto stage = [&]()
    {
#pragma unroll
        for(int sub = 0; sub < NSUB; ++sub)
        {
#pragma unroll
            for(int i = 0; i < PASSES; ++i)
            {
                const int off = (sub * kKeys32 + ld_row + i * ROWS_PER_PASS) * PAD
                    + ld_chunk * 4;
                *reinterpret_cast<f32x4 *>(&Ks[off]) = k_regs[sub][i];
                *reinterpret_cast<f32x4 *>(&Vs[off]) = v_regs[sub][i];
            }
        }
    };

    if(MODE == NNTILE_HIP_MASK_CAUSAL)
    {
        const int64_t hi = wg_qpos_hi + p.causal_offset - p.k_pos0;
        if(hi < 0)
        {
            if(!p.overwrite)
            {
                return;
            }
            n_steps = 0;    // nothing visible: the epilogue writes empty rows
        }
        const int64_t kt_hi = hi < 0 ? (int64_t)p.n_kv_tiles : hi / p.k_tile;
        if(kt_hi < p.n_kv_tiles)
        {
            const int64_t in_tile = hi - kt_hi * p.k_tile;
            const int steps = (int)(kt_hi * p.k_blocks_per_tile
                    + in_tile / kKeys32 + 1);
            n_steps = min(n_steps, steps);
        }
    }

    const float c = EXPLICIT ? kLog2e : p.scale * kLog2e;

    f32x16 o[DBLOCKS];
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
#pragma unroll
        for(int r = 0; r < 16; ++r)
        {
            o[db][r] = 0.0f;
        }
    }
    float m_run = neg_inf();
    float l_run = 0.0f;

    const int n_iter = (n_steps + NSUB - 1) / NSUB;
    // this wavefront's part of the staged keys
    const float *Kw = Ks + (SPLIT ? wave * kKeys32 * PAD : 0);
    const float *Vw = Vs + (SPLIT ? wave * kKeys32 * PAD : 0);
    if(n_iter > 0)
    {
#pragma unroll
        for(int sub = 0; sub < NSUB; ++sub)
        {
            src[sub] = locate(sub, n_steps);
        }
#pragma unroll
        for(int k = 0; k < PIECES; ++k)
        {
            fetch_piece(k);
        }
    }
    for(int G = 0; G < n_iter; ++G)
    {
        __syncthreads();
        stage();
        __syncthreads();
        // the next iteration's steps: located now, loaded between the MFMAs
#pragma unroll
        for(int sub = 0; sub < NSUB; ++sub)
        {
            src[sub] = locate((G + 1) * NSUB + sub, n_steps);
        }
        const int g = SPLIT ? G * NSUB + wave : G;      // this wavefront's step
        if(g >= n_steps)
        {
#pragma unroll
            for(int k = 0; k < PIECES; ++k)
            {
                fetch_piece(k);
            }
            continue;
        }

        const int kt = g / p.k_blocks_per_tile;
        const int kb = g % p.k_blocks_per_tile;
        const int64_t k_len = min(p.k_tile, p.k_seq - (int64_t)kt * p.k_tile);
        const int64_t k_row0 = (int64_t)kb * kKeys32;
        const int64_t k_pos_base = p.k_pos0 + (int64_t)kt * p.k_tile + k_row0;
        const int keys_here = (int)min((int64_t)kKeys32, k_len - k_row0);

        if(MODE == NNTILE_HIP_MASK_CAUSAL
                && k_pos_base > wave_qpos_hi + p.causal_offset)
        {
            // (nothing visible for this wavefront; its share of the loads remains)
#pragma unroll
            for(int k = 0; k < PIECES; ++k)
            {
                fetch_piece(k);
            }
            continue;
        }

        // ---- S^T = K Q^T ---------------------------------------------------
        f32x16 s;
#pragma unroll
        for(int r = 0; r < 16; ++r)
        {
            s[r] = 0.0f;
        }
        // (the K operands of the step are read ahead of the chain of
        // dependent MFMAs: a read issued behind four of them would only start
        // once they have all been issued, i.e. when the last one runs)
        {
            constexpr int AHEAD = NNTILE_F32_AHEAD < QSTEPS ? NNTILE_F32_AHEAD : QSTEPS;
            f32x4 ka[QSTEPS];
#pragma unroll
            for(int j = 0; j < AHEAD; ++j)
            {
                ka[j] = *reinterpret_cast<const f32x4 *>(&Kw[col * PAD + j * 8 + half * 4]);
            }
#pragma unroll
            for(int j = 0; j < QSTEPS; ++j)
            {
                if(j + AHEAD < QSTEPS)
                {
                    ka[j + AHEAD] = *reinterpret_cast<const f32x4 *>(
                            &Kw[col * PAD + (j + AHEAD) * 8 + half * 4]);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(int e = 0; e < 4; ++e)
                {
                    s = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[j][e], qf[j][e], s,
                            0, 0, 0);
                    if(e == 0)
                    {
                        fetch_slot(j);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }

        // ---- mask: register r holds key 8*(r/4) + 4*half + r%4 ---------------
        if(EXPLICIT)
        {
            const int64_t qrow = q_ok ? my_q : 0;
#pragma unroll
            for(int rg = 0; rg < 4; ++rg)
            {
                const int key0 = 8 * rg + 4 * half;
                const int64_t krow = k_row0 + key0;
#pragma unroll
                for(int e = 0; e < 4; ++e)
                {
                    float add;
                    if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                    {
                        add = (key0 + e < keys_here)
                            ? static_cast<const float *>(p.mask)[
                                qrow * p.mask_ld + krow + e]
                            : neg_inf();
                    }
                    else
                    {
                        add = (key0 + e < keys_here
                                && static_cast<const uint8_t *>(p.mask)[
                                    qrow * p.mask_ld + krow + e] != 0)
                            ? 0.0f : neg_inf();
                    }
                    const float v = s[4 * rg + e] * p.scale + add;
                    s[4 * rg + e] = (add == neg_inf()) ? neg_inf() : v;
                }
            }
        }
        else
        {
            const bool ragged = keys_here < kKeys32;
            const bool diagonal = (MODE == NNTILE_HIP_MASK_CAUSAL)
                && (k_pos_base + kKeys32 - 1 > wave_qpos_lo + p.causal_offset);
            if(ragged || diagonal)
            {
                const int64_t vis = (MODE == NNTILE_HIP_MASK_CAUSAL)
                    ? (my_qpos + p.causal_offset - k_pos_base)
                    : (int64_t)kKeys32;
                const int lim = (int)max((int64_t)-1,
                        min(vis, (int64_t)keys_here - 1));
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    const int key = 8 * (r >> 2) + 4 * half + (r & 3);
                    if(key > lim)
                    {
                        s[r] = neg_inf();
                    }
                }
            }
        }

        // ---- online softmax ---------------------------------------------------
        float mx = neg_inf();
#pragma unroll
        for(int r = 0; r < 16; ++r)
        {
            mx = fmaxf(mx, s[r]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
        const float alpha = fast_exp2((m_run - m_use) * c);
        const float mc = m_use * c;
        m_run = m_new;
        float rs = 0.0f;
#pragma unroll
        for(int r = 0; r < 16; ++r)
        {
            s[r] = fast_exp2(fmaf(s[r], c, -mc));
            rs += s[r];
        }
        l_run = l_run * alpha + rs;
#pragma unroll
        for(int db = 0; db < DBLOCKS; ++db)
        {
#pragma unroll
            for(int r = 0; r < 16; ++r)
            {
                o[db][r] *= alpha;
            }
        }

        // ---- O^T += V^T P^T ----------------------------------------------------
        // (V operands four keys at a time, one group ahead of its MFMAs)
        {
            float va[16][DBLOCKS];
            auto read_group = [&](int g4)
            {
#pragma unroll
                for(int x = 0; x < 4; ++x)
                {
                    const int r = 4 * g4 + x;
                    const int key = 8 * (r >> 2) + 4 * half + (r & 3);
#pragma unroll
                    for(int db = 0; db < DBLOCKS; ++db)
                    {
                        va[r][db] = Vw[key * PAD + db * 32 + col];
                    }
                }
            };
            read_group(0);
#pragma unroll
            for(int g4 = 0; g4 < 4; ++g4)
            {
                if(g4 + 1 < 4)
                {
                    read_group(g4 + 1);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(int x = 0; x < 4; ++x)
                {
                    const int r = 4 * g4 + x;
#pragma unroll
                    for(int db = 0; db < DBLOCKS; ++db)
                    {
                        o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[r][db], s[r], o[db],
                                0, 0, 0);
                        if(db == 0)
                        {
                            fetch_slot(QSTEPS + r);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            }
        }
    }

    // ---- SPLIT: merge the four wavefronts' results into wavefront 0 ----------------
    if constexpr(SPLIT)
    {
        // word w of lane l of wavefront v (v = 1..3) sits at ((v-1)*NW + w)*64 + l
        constexpr int NW = 2 + 16 * DBLOCKS;
        static_assert((NSUB - 1) * NW * 64 <= NSUB * kKeys32 * PAD, "exchange area does not fit");
        float *xch = Ks;
        __syncthreads();        // everyone is done with the staged keys
        if(wave > 0)
        {
            float *dst = xch + (wave - 1) * NW * 64 + lane;
            dst[0] = m_run;
            dst[64] = l_run;
#pragma unroll
            for(int db = 0; db < DBLOCKS; ++db)
            {
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    dst[(2 + 16 * db + r) * 64] = o[db][r];
                }
            }
        }
        __syncthreads();
        if(wave > 0)
        {
            return;
        }
#pragma unroll
        for(int v = 0; v < NSUB - 1; ++v)
        {
            const float *src = xch + v * NW * 64 + lane;
            const float m_other = src[0];
            const float m_new = fmaxf(m_run, m_other);
            const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
            const float a_mine = fast_exp2((m_run - m_use) * c);
            const float a_other = fast_exp2((m_other - m_use) * c);
            l_run = l_run * a_mine + src[64] * a_other;
#pragma unroll
            for(int db = 0; db < DBLOCKS; ++db)
            {
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    o[db][r] = o[db][r] * a_mine + src[(2 + 16 * db + r) * 64] * a_other;
                }
            }
            m_run = m_new;
        }
    }

    // ---- epilogue --------------------------------------------------------------
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const bool empty = !(l_tot > 0.0f);     // no visible key for this query
    if(!q_ok || (empty && !p.overwrite))
    {
        return;     // leave lse and A as they are
    }
    const float to_ln = EXPLICIT ? 1.0f : p.scale;
    const float lse_new = empty ? neg_inf() : m_run * to_ln + __logf(l_tot);
    float *lse_ptr = p.lse[qt] + (int64_t)b * q_len + my_q;
    const float lse_old = p.overwrite ? neg_inf() : *lse_ptr;
    float w_old = 0.0f, w_new = 0.0f, lse_out = neg_inf();
    if(!empty)
    {
        merge_weights(lse_old, lse_new, w_old, w_new, lse_out);
    }
    if(half == 0)
    {
        *lse_ptr = lse_out;
    }
    const float w_o = empty ? 0.0f : w_new / l_tot;
    float *Arow = static_cast<float *>(p.A[qt])
        + ((int64_t)b * q_len + my_q) * HEAD;
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
#pragma unroll
        for(int rg = 0; rg < 4; ++rg)
        {
            float *dst = Arow + db * 32 + 8 * rg + 4 * half;
            f32x4 v;
#pragma unroll
            for(int e = 0; e < 4; ++e)
            {
                v[e] = empty ? 0.0f : o[db][4 * rg + e] * w_o;
            }
            if(w_old != 0.0f)
            {
                const f32x4 old = *reinterpret_cast<const f32x4 *>(dst);
#pragma unroll
                for(int e = 0; e < 4; ++e)
                {
                    v[e] += w_old * old[e];
                }
            }
            *reinterpret_cast<f32x4 *>(dst) = v;
        }
    }
}

template<int HEAD, bool SPLIT>
static int launch_mode32(hipStream_t stream, const PrefillParams &p, int mode,
        dim3 grid)
{
    switch(mode)
    {
        case NNTILE_HIP_MASK_ADDITIVE:
            hipLaunchKernelGGL((sdpa_prefill_fp32_kernel<HEAD,
                        NNTILE_HIP_MASK_ADDITIVE, SPLIT>), grid, dim3(SPLIT ? split_waves32(HEAD) * 64 : kThreads32), 0,
                    stream, p);
            break;
        case NNTILE_HIP_MASK_NONE:
            hipLaunchKernelGGL((sdpa_prefill_fp32_kernel<HEAD,
                        NNTILE_HIP_MASK_NONE, SPLIT>), grid, dim3(SPLIT ? split_waves32(HEAD) * 64 : kThreads32), 0,
                    stream, p);
            break;
        case NNTILE_HIP_MASK_CAUSAL:
            hipLaunchKernelGGL((sdpa_prefill_fp32_kernel<HEAD,
                        NNTILE_HIP_MASK_CAUSAL, SPLIT>), grid, dim3(SPLIT ? split_waves32(HEAD) * 64 : kThreads32), 0,
                    stream, p);
            break;
        case NNTILE_HIP_MASK_BOOL:
            hipLaunchKernelGGL((sdpa_prefill_fp32_kernel<HEAD,
                        NNTILE_HIP_MASK_BOOL, SPLIT>), grid, dim3(SPLIT ? split_waves32(HEAD) * 64 : kThreads32), 0,
                    stream, p);
            break;
        default:
            return NNTILE_HIP_EINVAL;
    }
    return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
}

int launch_prefill_fp32(hipStream_t stream, PrefillParams &p, int head, int mode)
{
    p.k_blocks_per_tile = (int)((p.k_tile + kKeys32 - 1) / kKeys32);
    // the kernel addresses the rows of a key tile with 32-bit element offsets
    if(p.k_tile * head >= ((int64_t)1 << 31))
    {
        return NNTILE_HIP_EUNSUPPORTED;
    }
    // with fewer 128-query workgroups than CUs, 32-query workgroups whose
    // wavefronts share the keys instead
    const int64_t n_wide = (int64_t)p.batch * p.n_q_tiles
        * ((p.q_tile + kQRows32 - 1) / kQRows32);
    const bool split = n_wide < 256;
    const int q_rows = split ? 32 : kQRows32;
    p.q_blocks_per_tile = (int)((p.q_tile + q_rows - 1) / q_rows);
    const int64_t n_wg = (int64_t)p.batch * p.n_q_tiles * p.q_blocks_per_tile;
    if(n_wg <= 0 || n_wg > 0x7fffffff)
    {
        return NNTILE_HIP_EINVAL;
    }
    p.xcd_remap = (n_wg % 8 == 0) ? 1 : 0;
    const dim3 grid((unsigned)n_wg);
    switch(head)
    {
        case 32:
            return split ? launch_mode32<32, true>(stream, p, mode, grid)
                : launch_mode32<32, false>(stream, p, mode, grid);
        case 64:
            return split ? launch_mode32<64, true>(stream, p, mode, grid)
                : launch_mode32<64, false>(stream, p, mode, grid);
        case 128:
            return split ? launch_mode32<128, true>(stream, p, mode, grid)
                : launch_mode32<128, false>(stream, p, mode, grid);
        default:
            return NNTILE_HIP_EUNSUPPORTED;
    }
}

} // namespace nntile_hip
