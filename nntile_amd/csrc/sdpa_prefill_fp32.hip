// Prefill attention forward for fp32 tiles on gfx950.
//
// Same decomposition as the 16-bit kernel (S^T = K Q^T and O^T += V^T P^T with
// a lane owning one query), but on v_mfma_f32_32x32x2_f32: operands and
// products are true fp32, which the 1e-4 tolerance of the fp32 configurations
// needs.  Keys are walked in steps of 32.  With a 2-deep contraction per MFMA
// the lane half h supplies the operand element k = h, so:
//   S^T: 4 consecutive MFMAs consume one 16-byte read K[key][8j+4h .. +3]
//        against the matching 4 query values held in registers;
//   O^T: the B operand is the S^T accumulator register itself (key
//        8*(r/4) + 4h + r%4), the A operand is V[that key][d] read from LDS
//        with the head axis across lanes - no transposition is needed.
// K and V steps go from global memory straight into LDS (global_load_lds, 16
// bytes per lane, 1 KB per instruction, no registers in between); rows are
// unpadded and their 16-byte chunks XOR-swizzled by row against bank
// conflicts, as in the 16-bit kernel.
//
// Two forms:
//   * 128 queries per workgroup, four wavefronts of 32 queries sharing every
//     key step: two LDS buffers per operand, the loads of step g+1 issued at
//     the top of step g, one barrier per step;
//   * SPLIT, for launches with fewer such workgroups than CUs: a workgroup is
//     32 queries and its four wavefronts take every fourth key step each, each
//     through its own LDS buffer - K of the next step is requested when the
//     scores of this one are done, V when its output products are, and there
//     is no barrier in the loop; at the end the four merge their (max, sum, O)
//     through LDS.  The chain of dependent steps a wavefront walks, which
//     bounds such a launch, is a quarter as long, and four times as many
//     workgroups spread over the CUs.
#include <type_traits>

#include "sdpa_common.hpp"

namespace nntile_hip
{

// 16-byte K operand reads issued ahead of the MFMAs that use them
#ifndef NNTILE_F32_AHEAD
#define NNTILE_F32_AHEAD 2
#endif
// Developer builds can turn F32_STAMP into time stamps of one wavefront
#ifndef F32_STAMP
#define F32_STAMP(i)
#define F32_STAMP_DECL
#define F32_STAMP_DUMP
#endif
// SPLIT form: the softmax of the previous step behind every score MFMA (1) or
// behind the first of each group of four (0)
#ifndef NNTILE_F32_FINE
#define NNTILE_F32_FINE 0
#endif
// Launches with fewer 128-query workgroups than this take the SPLIT form.
// Measured crossovers (fused launches of batch x seq x head, 100 launches
// each): under a causal mask the 32-query workgroups, dealt longest first,
// fill the triangle far better - head 64: 48 x 1024 81.7 us against 139.5,
// 32 x 4096 619 against 771, 192 x 2048 1005 against 1087, and only at 384 x
// 2048 (6144 such workgroups) 2301 against 2022; head 128: 96 x 1024 353
// against 385, 64 x 2048 809 against 820, 96 x 2048 1227 against 1118.
// Without a mask the shared key steps win earlier: head 64, 48 x 1024 122
// against 139, 96 x 1024 243 against 202.
static int split_below(int head, int mode)
{
#ifdef NNTILE_F32_SPLIT_BELOW
    return NNTILE_F32_SPLIT_BELOW;
#else
    const bool causal = mode == NNTILE_HIP_MASK_CAUSAL;
    if(head >= 128)
    {
        return causal ? 1025 : 256;
    }
    return causal ? 4096 : 512;
#endif
}
constexpr int kQRows32 = 128;
constexpr int kKeys32 = 32;
constexpr int kThreads32 = 256;          // 4 wavefronts in both forms

template<int N> __device__ __forceinline__ void f32_wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    // s_waitcnt simm16: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[15:14]
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
    asm volatile("" ::: "memory");
}

template<int HEAD, int MODE, bool SPLIT>
__global__ __launch_bounds__(kThreads32, (SPLIT && HEAD == 128) ? 1 : 2)
void sdpa_prefill_fp32_kernel(const PrefillParams p)
{
    constexpr int QROWS = SPLIT ? 32 : kQRows32;    // queries per workgroup
    constexpr int NSUB = SPLIT ? 4 : 1;     // key steps in flight side by side (one per wavefront)
    constexpr int QSTEPS = HEAD / 8;        // 16-byte groups per lane half along head
    constexpr int DBLOCKS = HEAD / 32;
    constexpr int RB = HEAD * 4;            // bytes per K/V row
    constexpr int CPR = HEAD / 4;           // 16-byte chunks per row
    constexpr int RPL = CPR >= 16 ? 1 : 16 / CPR;   // rows per 256-byte line of LDS banks
    constexpr int KSW = CPR >= 16 ? 16 : CPR;       // K: chunk c of row r at c ^ ((r / RPL) % KSW)
    constexpr int ROWS_PER_LOAD = 1024 / RB;        // rows one load instruction fills
    constexpr int LOADS = kKeys32 / ROWS_PER_LOAD;  // load instructions per K (or V) step
    constexpr int LPW = SPLIT ? LOADS : LOADS / 4;  // ... of them issued by one wavefront
    constexpr int BLOCK_BYTES = kKeys32 * RB;
    constexpr bool EXPLICIT = (MODE == NNTILE_HIP_MASK_ADDITIVE
            || MODE == NNTILE_HIP_MASK_BOOL);
    static_assert(LPW >= 1, "head size does not fit this tiling");

    // SPLIT: lds_k0 / lds_v0 hold one step per wavefront (wavefront w owns
    // bytes [w * BLOCK_BYTES, +BLOCK_BYTES)); lds_k1 / lds_v1 are not used.
    // Otherwise step g of the workgroup lives in lds_k[g % 2], lds_v[g % 2].
    // (Separate arrays: the compiler then knows that what streams into one
    // cannot alias the reads of another.)
    __shared__ __attribute__((aligned(1024))) char lds_k0[NSUB * BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char lds_v0[NSUB * BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char lds_k1[SPLIT ? 16 : BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char lds_v1[SPLIT ? 16 : BLOCK_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int col = lane & 31;
    const int half = lane >> 5;
    F32_STAMP_DECL

    const int q_blocks = p.n_q_tiles * p.q_blocks_per_tile;
    const int batch_all = p.batch * p.n_slabs;
    int wg = blockIdx.x;
    int b, qblk;
    if(SPLIT)
    {
        // A launch of this form fits the GPU at once, so where a workgroup
        // lands decides how evenly the CUs are loaded.  Workgroups are dealt
        // round-robin to the 8 XCDs; each XCD puts its first 32 on its 32 CUs
        // and the next ones beside them, i + 32 next to i.  Query blocks go out
        // longest first (all batch entries of a block before the next block),
        // and the workgroups beyond the first 32 of an XCD in reverse: the CU
        // with the longest workgroup gets the shortest as its second.
        const int per_xcd = (int)((gridDim.x + 7u - (unsigned)(wg & 7)) >> 3);
        int i = wg >> 3;
        if(i >= 32 && per_xcd <= 64)
        {
            i = 32 + (per_xcd - 1 - i);
        }
        const int k = (i << 3) | (wg & 7);
        b = k % batch_all;
        qblk = q_blocks - 1 - k / batch_all;
    }
    else
    {
        if(p.xcd_remap)
        {
            const int per_xcd = gridDim.x >> 3;
            wg = (wg & 7) * per_xcd + (wg >> 3);
        }
        b = wg / q_blocks;
        qblk = q_blocks - 1 - (wg % q_blocks);
    }
    // the slab of this entry: its tiles are allocations of their own
    int q_tile0 = 0, k_tile0 = 0;
    if(p.n_slabs > 1)
    {
        const int slab = b / p.batch;
        b -= slab * p.batch;
        q_tile0 = slab * p.n_q_tiles;
        k_tile0 = slab * p.n_kv_tiles;
    }
    const int qt = qblk / p.q_blocks_per_tile;
    const int qb = qblk % p.q_blocks_per_tile;
    const int64_t q_len = min(p.q_tile, p.q_seq - (int64_t)qt * p.q_tile);
    const int64_t q_row0 = (int64_t)qb * QROWS;
    if(q_row0 >= q_len)
    {
        return;
    }
    const int kvb = kv_entry(b, p.n_batch, p.kv_group);

    const float *Qt = static_cast<const float *>(p.Q[q_tile0 + qt])
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

    // ---- LDS layout and the lane's fixed addresses ---------------------------
    // A step's K (and V) block is 32 rows of RB bytes, unpadded.  The 16-byte
    // chunk c of row r is stored at chunk position
    //   K:  c ^ ((r / RPL) % KSW)      consecutive rows, same c -> different bank groups
    //   V:  c ^ (8 * ((r / 4) % 2))    (rows of 256 bytes and more) the two lane
    //                                  halves read rows 4 apart: different halves of the banks
    // Load instruction `ld` fills rows [ld*ROWS_PER_LOAD, +ROWS_PER_LOAD): lane L
    // lands on row ld*ROWS_PER_LOAD + L/CPR, chunk position L % CPR, and fetches
    // the chunk that belongs there.
    constexpr int VSW = CPR >= 16 ? 8 : 0;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    uint32_t k_goff[LPW], v_goff[LPW];
    int ld_row[LPW];
    const int ld_cpos = lane % CPR;
#pragma unroll
    for(int i = 0; i < LPW; ++i)
    {
        const int ld = SPLIT ? i : wave * LPW + i;
        const int r = ld * ROWS_PER_LOAD + lane / CPR;
        ld_row[i] = r;
        k_goff[i] = (uint32_t)(r * RB + (ld_cpos ^ ((r / RPL) % KSW)) * 16);
        v_goff[i] = (uint32_t)(r * RB + (ld_cpos ^ (VSW * ((r >> 2) & 1))) * 16);
    }
    // S operand: lane (col, half) reads row col, logical chunk 2*j + half.
    uint32_t k_raddr[QSTEPS];
#pragma unroll
    for(int j = 0; j < QSTEPS; ++j)
    {
        k_raddr[j] = (uint32_t)(col * RB + ((2 * j + half) ^ ((col / RPL) % KSW)) * 16);
    }
    // PV operand: register r of the scores is key 8*(r/4) + 4*half + r%4, whose
    // swizzle only depends on the lane half; lane (col, half) reads head value
    // 32*db + col of that row.  8*(r/4) + r%4 goes into the immediate offset.
    uint32_t v_raddr[DBLOCKS];
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
        v_raddr[db] = (uint32_t)(4 * half * RB
                + (((db * 8 + col / 4) ^ (VSW * half)) * 4 + col % 4) * 4);
    }

    // Where the rows of a key step come from.
    struct StepSource
    {
        const char *K, *V;      // first row of the step
        int rows_left;          // rows of the tile from this step on
    };
    const int64_t k_len0 = min(p.k_tile, p.k_seq);
    const bool one_tile = p.n_kv_tiles == 1;
    const int64_t entry_rows0 = p.kv_rows > 0 ? p.kv_rows : k_len0;
    const char *K0 = static_cast<const char *>(p.K[k_tile0]) + ((int64_t)kvb * entry_rows0) * RB;
    const char *V0 = static_cast<const char *>(p.V[k_tile0]) + ((int64_t)kvb * entry_rows0) * RB;
    auto locate = [&](int g) -> StepSource
    {
        StepSource src;
        if(one_tile)
        {
            src.K = K0 + (int64_t)g * kKeys32 * RB;
            src.V = V0 + (int64_t)g * kKeys32 * RB;
            src.rows_left = (int)k_len0 - g * kKeys32;
        }
        else
        {
            const int kt = g / p.k_blocks_per_tile;
            const int kb = g % p.k_blocks_per_tile;
            const int64_t k_len = min(p.k_tile, p.k_seq - (int64_t)kt * p.k_tile);
            const int64_t off = ((int64_t)kvb * k_len + (int64_t)kb * kKeys32) * RB;
            src.K = static_cast<const char *>(p.K[k_tile0 + kt]) + off;
            src.V = static_cast<const char *>(p.V[k_tile0 + kt]) + off;
            src.rows_left = (int)k_len - kb * kKeys32;
        }
        return src;
    };
    // Global -> LDS loads of this wavefront's share of the K (or V) rows of a
    // step.  Rows past the end of the tile are clamped to its last row: their
    // keys are masked out of the scores, so their probabilities are exactly 0.
    auto fetch = [&](const char *src, int rows_left, const uint32_t (&goff)[LPW], char *dst_base)
    {
        char *dst = dst_base + wave_u * (SPLIT ? BLOCK_BYTES : LPW * 1024);
        if(rows_left >= kKeys32)
        {
#pragma unroll
            for(int i = 0; i < LPW; ++i)
            {
                load_to_lds16<0, false>(src, goff[i], dst + i * 1024);
            }
        }
        else
        {
            const int last = rows_left - 1;
#pragma unroll
            for(int i = 0; i < LPW; ++i)
            {
                const uint32_t back = (uint32_t)(max(ld_row[i] - last, 0) * RB);
                load_to_lds16<0, false>(src, goff[i] - back, dst + i * 1024);
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

    // Scores of key step g from the K block at Kw: S^T = K Q^T, mask.
    // `between(t)` is called after MFMA t of the 4 * QSTEPS: whatever it issues
    // (a load instruction, a few VALU instructions) runs while the matrix unit
    // is busy with that MFMA - as long as it is short: work bunched up behind
    // one MFMA leaves the unit idle for the rest of it.
    auto scores = [&](int g, const char *Kw, f32x16 &s, auto between) __attribute__((always_inline))
    {
        const int kt = g / p.k_blocks_per_tile;
        const int kb = g % p.k_blocks_per_tile;
        const int64_t k_len = min(p.k_tile, p.k_seq - (int64_t)kt * p.k_tile);
        const int64_t k_row0 = (int64_t)kb * kKeys32;
        const int64_t k_pos_base = p.k_pos0 + (int64_t)kt * p.k_tile + k_row0;
        const int keys_here = (int)min((int64_t)kKeys32, k_len - k_row0);
        // Explicit mask: the step's 16 values of this lane are loaded here,
        // ahead of the chain of MFMAs.  Register r holds key
        // 8*(r/4) + 4*half + r%4: four groups of four consecutive keys.  A full
        // step of an aligned mask takes one 16-byte (additive) or 4-byte
        // (boolean) load per group; lanes are queries, a mask row apart, so
        // the cost of a load is the cache lines it touches, not its width.
        // Otherwise element by element: keys past the end of a ragged step
        // are hidden, and their loads are clamped to the step's last key
        // instead of being branched around, so that the loads are independent.
        float madd[EXPLICIT ? 16 : 1];
        if(EXPLICIT)
        {
            const int64_t mrow = (q_ok ? my_q : 0) * p.mask_ld + k_row0;
            constexpr int ES = (MODE == NNTILE_HIP_MASK_ADDITIVE) ? 4 : 1;
            const bool wide = (p.mask_ld % 4 == 0) && (k_row0 % 4 == 0)
                && (reinterpret_cast<uintptr_t>(p.mask) % (4 * ES) == 0)
                && keys_here == kKeys32;
            if(wide)
            {
#pragma unroll
                for(int rg = 0; rg < 4; ++rg)
                {
                    const int64_t at = mrow + 8 * rg + 4 * half;
                    if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                    {
                        const f32x4 v = *reinterpret_cast<const f32x4 *>(
                                static_cast<const float *>(p.mask) + at);
#pragma unroll
                        for(int e = 0; e < 4; ++e)
                        {
                            madd[4 * rg + e] = v[e];
                        }
                    }
                    else
                    {
                        const uint32_t w = *reinterpret_cast<const uint32_t *>(
                                static_cast<const uint8_t *>(p.mask) + at);
#pragma unroll
                        for(int e = 0; e < 4; ++e)
                        {
                            madd[4 * rg + e] = ((w >> (8 * e)) & 0xffu) != 0u
                                ? 0.0f : neg_inf();
                        }
                    }
                }
            }
            else
            {
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    const int key = 8 * (r >> 2) + 4 * half + (r & 3);
                    const int64_t at = mrow + max(min(key, keys_here - 1), 0);
                    if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                    {
                        madd[r] = static_cast<const float *>(p.mask)[at];
                    }
                    else
                    {
                        madd[r] = static_cast<const uint8_t *>(p.mask)[at] != 0
                            ? 0.0f : neg_inf();
                    }
                    if(key >= keys_here)
                    {
                        madd[r] = neg_inf();
                    }
                }
            }
        }
        // One accumulator chain: a dependent MFMA of this shape issues right
        // behind its predecessor (64 cycles apart, measured), and the first one
        // takes a constant zero, so nothing is cleared or added up afterwards.
        // (the K operands of the step are read ahead of the chain of MFMAs: a
        // read issued behind four of them would only start once they have all
        // been issued)
        {
            constexpr int AHEAD = NNTILE_F32_AHEAD < QSTEPS ? NNTILE_F32_AHEAD : QSTEPS;
            f32x16 zero16;
#pragma unroll
            for(int r = 0; r < 16; ++r)
            {
                zero16[r] = 0.0f;
            }
            f32x4 ka[QSTEPS];
#pragma unroll
            for(int j = 0; j < AHEAD; ++j)
            {
                ka[j] = *reinterpret_cast<const f32x4 *>(Kw + k_raddr[j]);
            }
#pragma unroll
            for(int j = 0; j < QSTEPS; ++j)
            {
                if(j + AHEAD < QSTEPS)
                {
                    ka[j + AHEAD] = *reinterpret_cast<const f32x4 *>(Kw + k_raddr[j + AHEAD]);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(int e = 0; e < 4; ++e)
                {
                    s = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[j][e], qf[j][e],
                            (j == 0 && e == 0) ? zero16 : s, 0, 0, 0);
                    between(4 * j + e);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }

        // ---- mask: register r holds key 8*(r/4) + 4*half + r%4 ---------------
        if(EXPLICIT)
        {
#pragma unroll
            for(int r = 0; r < 16; ++r)
            {
                const float v = s[r] * p.scale + madd[r];
                s[r] = (madd[r] == neg_inf()) ? neg_inf() : v;
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
    };

    // Online softmax of the scores (they become the probabilities) and the
    // rescale of what has been accumulated.
    auto softmax = [&](f32x16 &s) __attribute__((always_inline))
    {
        float mx = neg_inf();
#pragma unroll
        for(int r = 0; r < 16; ++r)
        {
            mx = fmaxf(mx, s[r]);
        }
        mx = max_across_halves(mx);
        const float m_new = fmaxf(m_run, mx);
        const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
        const float mc = m_use * c;
        // the running maximum rarely moves after the first steps
        if(__builtin_amdgcn_ballot_w64(m_new != m_run) != 0)
        {
            const float alpha = fast_exp2((m_run - m_use) * c);
            l_run *= alpha;
#pragma unroll
            for(int db = 0; db < DBLOCKS; ++db)
            {
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    o[db][r] *= alpha;
                }
            }
            m_run = m_new;
        }
        float rs = 0.0f;
#pragma unroll
        for(int r = 0; r < 16; ++r)
        {
            s[r] = fast_exp2(fmaf(s[r], c, -mc));
            rs += s[r];
        }
        l_run += rs;
    };

    // O^T += V^T P^T from the V block at Vw: MFMA n of the 16 * DBLOCKS takes
    // key n / DBLOCKS and output block n % DBLOCKS; its V operand is read from
    // LDS eight MFMAs ahead.  `between(n)` is called after MFMA n.
    auto output = [&](const char *Vw, const f32x16 &s, auto between) __attribute__((always_inline))
    {
        constexpr int NM = 16 * DBLOCKS;
        constexpr int AH = 8;
        float va[NM];
        auto read_operand = [&](int n) __attribute__((always_inline))
        {
            const int r = n / DBLOCKS, db = n % DBLOCKS;
            va[n] = *reinterpret_cast<const float *>(
                    Vw + v_raddr[db] + (8 * (r >> 2) + (r & 3)) * RB);
        };
#pragma unroll
        for(int n = 0; n < AH; ++n)
        {
            read_operand(n);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for(int n = 0; n < NM; ++n)
        {
            if(n + AH < NM)
            {
                read_operand(n + AH);
            }
            const int r = n / DBLOCKS, db = n % DBLOCKS;
            o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[n], s[r], o[db], 0, 0, 0);
            between(n);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto nothing = [](int) {};
    // one load instruction of a step's K (or V) share: piece i of LPW
    auto fetch_piece = [&](const char *src, int rows_left, const uint32_t (&goff)[LPW],
            char *dst_base, int i) __attribute__((always_inline))
    {
        char *dst = dst_base + wave_u * (SPLIT ? BLOCK_BYTES : LPW * 1024);
        const int last = rows_left - 1;
        const uint32_t back = (uint32_t)(max(ld_row[i] - last, 0) * RB);
        load_to_lds16<0, false>(src, goff[i] - back, dst + i * 1024);
    };

    // nothing of key step g is visible to this wavefront
    auto hidden = [&](int g) -> bool
    {
        if(MODE != NNTILE_HIP_MASK_CAUSAL)
        {
            return false;
        }
        const int kt = g / p.k_blocks_per_tile;
        const int kb = g % p.k_blocks_per_tile;
        const int64_t k_pos_base = p.k_pos0 + (int64_t)kt * p.k_tile + (int64_t)kb * kKeys32;
        return k_pos_base > wave_qpos_hi + p.causal_offset;
    };

    if constexpr(SPLIT)
    {
        // ---- every wavefront walks its own key steps wave, wave + 4, ... ---------
        // through two buffers of its own and shares nothing with the others
        // inside the loop, so the loop has no barrier.  The steps are software
        // pipelined: the softmax of step i runs in the shadow of the score
        // MFMAs of step i+1, then the output MFMAs of step i follow.
        //   buffer R (lds_k0): K(i+1) while those scores are computed;
        //   buffer P (lds_v0): V(i) while that output is computed - and K(0)
        //                      at the very start, so that nothing waits for it.
        // Loads complete in the order they were issued:
        //   K(0)->P K(1)->R | V(0)->P K(2)->R | V(1)->P K(3)->R | ...
        // V(i) is requested between the score MFMAs of step i+1 (P is free once
        // the output of step i-1 is done), K(i+2) between the output MFMAs of
        // step i (R is free once the scores of step i+1 are done): a load
        // instruction issued behind an MFMA costs the wavefront nothing.
        char *Rw = lds_k0 + wave_u * BLOCK_BYTES;
        char *Pw = lds_v0 + wave_u * BLOCK_BYTES;
        const int n_my = wave_u < n_steps ? (n_steps - wave_u + 3) / 4 : 0;
        // Both phases have 4 * LPW MFMAs: load instruction i of the next block
        // goes out behind MFMA 4 * i.  (Issuing them earlier in the phase - all
        // in its first half, its first quarter, or at once - changed nothing.)
        static_assert(LPW == QSTEPS && 16 * DBLOCKS == 4 * LPW, "one load instruction per four MFMAs");
        if(n_my > 0)
        {
            const StepSource src0 = locate(wave_u);
            fetch(src0.K, src0.rows_left, k_goff, lds_v0);         // K(0) into P
            StepSource src1 = {nullptr, nullptr, 0};
            if(n_my > 1)
            {
                src1 = locate(wave_u + 4);
                fetch(src1.K, src1.rows_left, k_goff, lds_k0);     // K(1) into R
                // K(0) has landed, K(1) may still be on its way.  (This also
                // says that the Q values, ordinary loads, have arrived, with an
                // instruction the compiler's own wait insertion sees: otherwise
                // it waits for them at their first use inside the loop, on every
                // pass, with vmcnt(0).)
                f32_wait_vmcnt<LPW>();
            }
            else
            {
                f32_wait_vmcnt<0>();
            }
            F32_STAMP(1)
            f32x16 s_cur;
            scores(wave_u, Pw, s_cur, nothing);
            F32_STAMP(2)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // P has been read
            StepSource cur = src0;      // step i: its V is still to be requested
            StepSource nxt = src1;      // step i+1: its K is in R or on its way there
            for(int i = 0; i < n_my; ++i)
            {
                const int g = wave_u + 4 * i;
                const bool more = i + 1 < n_my;
                const bool more2 = i + 2 < n_my;
                StepSource nxt2 = {nullptr, nullptr, 0};
                if(more2)
                {
                    nxt2 = locate(g + 8);
                }
                // ---- the softmax of step i, in pieces ----------------------------
                float mc = 0.0f, rs = 0.0f;
                auto softmax_head = [&]() __attribute__((always_inline))
                {
                    float mx = neg_inf();
#pragma unroll
                    for(int r = 0; r < 16; ++r)
                    {
                        mx = fmaxf(mx, s_cur[r]);
                    }
                    mx = max_across_halves(mx);
                    const float m_new = fmaxf(m_run, mx);
                    const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
                    mc = m_use * c;
                    // the running maximum rarely moves after the first steps
                    if(__builtin_amdgcn_ballot_w64(m_new != m_run) != 0)
                    {
                        const float alpha = fast_exp2((m_run - m_use) * c);
                        l_run *= alpha;
#pragma unroll
                        for(int db = 0; db < DBLOCKS; ++db)
                        {
#pragma unroll
                            for(int r = 0; r < 16; ++r)
                            {
                                o[db][r] *= alpha;
                            }
                        }
                        m_run = m_new;
                    }
                    asm volatile("" : "+v"(mc));
                };
                // elements [lo, hi) of the 16 scores of a lane
                auto softmax_part = [&](int lo, int hi) __attribute__((always_inline))
                {
#pragma unroll
                    for(int r = 0; r < 16; ++r)
                    {
                        if(r >= lo && r < hi)
                        {
                            float e = fast_exp2(fmaf(s_cur[r], c, -mc));
                            // (keeps the exponential where it is written: its
                            // result is first used by the output MFMAs, and the
                            // compiler would otherwise move it down to them,
                            // out of the shadow of the score MFMAs)
                            asm volatile("" : "+v"(e));
                            s_cur[r] = e;
                            rs += e;
                        }
                    }
                    asm volatile("" : "+v"(rs));
                };
                f32x16 s_nxt;
                F32_STAMP(3 + 4 * i)
                if(more)
                {
                    // K(i+1) has landed in R (everything requested so far has)
                    f32_wait_vmcnt<0>();
                    F32_STAMP(4 + 4 * i)
                    scores(g + 4, Rw, s_nxt, [&](int t)
                    {
                        // behind the first MFMA of a group: V(i) goes out, into P;
                        // behind the second MFMA of all: the head of the softmax;
                        // behind the others: an element of it or none
#if NNTILE_F32_FINE
                        constexpr int NFREE = 3 * QSTEPS - 1;
                        if(t % 4 == 0)
                        {
                            fetch_piece(cur.V, cur.rows_left, v_goff, lds_v0, t / 4);
                        }
                        else if(t == 1)
                        {
                            softmax_head();
                        }
                        else
                        {
                            const int k = t - 2 - t / 4;    // which of the NFREE other places
                            softmax_part(k * 16 / NFREE, (k + 1) * 16 / NFREE);
                        }
#else
                        if(t % 4 == 0)
                        {
                            const int j = t / 4;
                            fetch_piece(cur.V, cur.rows_left, v_goff, lds_v0, j);
                            if(j == 0)
                            {
                                softmax_head();
                            }
                            else
                            {
                                softmax_part((j - 1) * 16 / (QSTEPS - 1), j * 16 / (QSTEPS - 1));
                            }
                        }
#endif
                    });
                }
                else
                {
                    fetch(cur.V, cur.rows_left, v_goff, lds_v0);
                    softmax_head();
                    softmax_part(0, 16);
                }
                l_run += rs;
                // R has been read, V(i) has landed in P
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                F32_STAMP(5 + 4 * i)
                f32_wait_vmcnt<0>();
                F32_STAMP(6 + 4 * i)
                // (two copies of the phase rather than a branch around every
                // load instruction inside it)
                if(more2)
                {
                    output(Pw, s_cur, [&](int t)
                    {
                        // K(i+2) goes out, into R
                        if(t % 4 == 0)
                        {
                            fetch_piece(nxt2.K, nxt2.rows_left, k_goff, lds_k0, t / 4);
                        }
                    });
                }
                else
                {
                    output(Pw, s_cur, nothing);
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // P has been read
                if(more)
                {
#pragma unroll
                    for(int r = 0; r < 16; ++r)
                    {
                        s_cur[r] = s_nxt[r];
                    }
                }
                cur = nxt;
                nxt = nxt2;
            }
        }
        else
        {
            f32_wait_vmcnt<0>();
        }
    }
    else
    {
        // ---- the four wavefronts share every key step ------------------------------
        if(n_steps > 0)
        {
            const StepSource src = locate(0);
            fetch(src.K, src.rows_left, k_goff, lds_k0);
            fetch(src.V, src.rows_left, v_goff, lds_v0);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        auto step = [&](int g, auto buf_tag) __attribute__((always_inline))
        {
            constexpr int BUF = decltype(buf_tag)::value;
            // loads of the next step into the other buffers (every wavefront
            // passed the barrier that ended step g-1: nobody reads them)
            if(g + 1 < n_steps)
            {
                const StepSource nxt = locate(g + 1);
                fetch(nxt.K, nxt.rows_left, k_goff, BUF ? lds_k0 : lds_k1);
                fetch(nxt.V, nxt.rows_left, v_goff, BUF ? lds_v0 : lds_v1);
            }
            if(!hidden(g))
            {
                f32x16 s;
                scores(g, BUF ? lds_k1 : lds_k0, s, nothing);
                softmax(s);
                output(BUF ? lds_v1 : lds_v0, s, nothing);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        };
        for(int g = 0; g < n_steps; g += 2)
        {
            step(g, std::integral_constant<int, 0>{});
            if(g + 1 < n_steps)
            {
                step(g + 1, std::integral_constant<int, 1>{});
            }
        }
    }

    // ---- SPLIT: merge the four wavefronts' results into wavefront 0 ----------------
    if constexpr(SPLIT)
    {
        // word w of lane l of wavefront v (v = 1..3) sits at ((v-1)*NW + w)*64 + l
        constexpr int NW = 2 + 16 * DBLOCKS;
        static_assert((NSUB - 1) * NW * 64 * 4 <= NSUB * BLOCK_BYTES, "exchange area does not fit");
        float *xch = reinterpret_cast<float *>(lds_k0);
        F32_STAMP(43)
        f32_wait_vmcnt<0>();
        __syncthreads();        // everyone is done with the key buffers
        F32_STAMP(44)
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
    F32_STAMP(45)
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const bool empty = !(l_tot > 0.0f);     // no visible key for this query
    if(!q_ok || (empty && !p.overwrite))
    {
        return;     // leave lse and A as they are
    }
    const float to_ln = EXPLICIT ? 1.0f : p.scale;
    const float lse_new = empty ? neg_inf() : m_run * to_ln + __logf(l_tot);
    float *lse_ptr = p.lse[q_tile0 + qt] + (int64_t)b * q_len + my_q;
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
    float *Arow = static_cast<float *>(p.A[q_tile0 + qt])
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
    F32_STAMP(46)
    F32_STAMP_DUMP
}

template<int HEAD, bool SPLIT>
static int launch_mode32(hipStream_t stream, const PrefillParams &p, int mode,
        dim3 grid)
{
    switch(mode)
    {
        case NNTILE_HIP_MASK_ADDITIVE:
            hipLaunchKernelGGL((sdpa_prefill_fp32_kernel<HEAD,
                        NNTILE_HIP_MASK_ADDITIVE, SPLIT>), grid, dim3(kThreads32), 0,
                    stream, p);
            break;
        case NNTILE_HIP_MASK_NONE:
            hipLaunchKernelGGL((sdpa_prefill_fp32_kernel<HEAD,
                        NNTILE_HIP_MASK_NONE, SPLIT>), grid, dim3(kThreads32), 0,
                    stream, p);
            break;
        case NNTILE_HIP_MASK_CAUSAL:
            hipLaunchKernelGGL((sdpa_prefill_fp32_kernel<HEAD,
                        NNTILE_HIP_MASK_CAUSAL, SPLIT>), grid, dim3(kThreads32), 0,
                    stream, p);
            break;
        case NNTILE_HIP_MASK_BOOL:
            hipLaunchKernelGGL((sdpa_prefill_fp32_kernel<HEAD,
                        NNTILE_HIP_MASK_BOOL, SPLIT>), grid, dim3(kThreads32), 0,
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
    // with fewer 128-query workgroups than CUs, or query tiles so short that
    // half of such a workgroup's wavefronts would have no rows (the new tokens
    // of a decode step), 32-query workgroups whose wavefronts share the keys
    // instead
    const int64_t batch_all = (int64_t)p.batch * p.n_slabs;
    const int64_t n_wide = batch_all * p.n_q_tiles
        * ((p.q_tile + kQRows32 - 1) / kQRows32);
    const bool split = p.form != 0 ? p.form == 2
        : (n_wide < split_below(head, mode) || p.q_tile <= 64);
    const int q_rows = split ? 32 : kQRows32;
    p.q_blocks_per_tile = (int)((p.q_tile + q_rows - 1) / q_rows);
    const int64_t n_wg = batch_all * p.n_q_tiles * p.q_blocks_per_tile;
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
