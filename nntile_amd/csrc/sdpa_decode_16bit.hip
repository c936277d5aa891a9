// Short-query / long-key attention forward (decode against a KV cache) for
// 16-bit tiles on gfx950.  The shape is bound by the one pass over K and V in
// HBM, so the kernel is built around that stream:
//
//  * all kv_group query heads that share one key/value head are processed
//    together (rows = kv_group * q_seq <= 64), so K and V are read once, not
//    once per query head;
//  * the key axis of each (batch entry, kv head) unit is split over
//    workgroups so that every CU streams; each workgroup writes a partial
//    (the output normalised and rounded to the tile type, max and sum in
//    fp32), and merge workgroups at the end of the same grid - or a second
//    small kernel - merge the partials and fold them into the running
//    (lse, A) pair; a unit with a single split writes (lse, A) itself;
//  * rows that are being appended to a cache by the same call are read from
//    the caller's tensors, and one more workgroup per unit at the very end
//    of the grid copies them into the caches;
//  * K and V steps go from global memory straight into LDS (global_load_lds,
//    16 bytes per lane, 1 KB contiguous per instruction, no registers in
//    between) through a ring of STAGES buffers, so that STAGES-1 steps of 32 KB
//    are in flight per workgroup while one is consumed;
//  * a wavefront owns 16 rows and uses v_mfma_f32_16x16x32 (S^T = K Q^T,
//    O^T += V^T P^T with P^T taken from the S^T accumulators); LDS rows are
//    unpadded and XOR-swizzled by 16-byte chunks against bank conflicts, and
//    the V operand is gathered with the transposing ds_read_b64_tr_b16.
#include <atomic>
#include <random>
#include <type_traits>

#include "sdpa_common.hpp"

namespace nntile_hip
{

// Cache policy of the K/V stream: non-temporal (each byte is used once).
#ifndef NNTILE_DMA_NT
#define NNTILE_DMA_NT true
#endif

constexpr int kDecThreads = 256;  // 4 wavefronts x 16 query rows
constexpr int kDecodeCUs = 256;   // MI355X
// Ring stages and workgroups per CU the kernel is built for
#ifndef NNTILE_DEC_STAGES
#define NNTILE_DEC_STAGES 2
#endif
#ifndef NNTILE_DEC_WGS_PER_CU
#define NNTILE_DEC_WGS_PER_CU 2
#endif

// Partial outputs of the key splits: 1 = normalised and in the tile type,
// 0 = unnormalised fp32
#ifndef NNTILE_DEC_PART16
#define NNTILE_DEC_PART16 1
#endif
typedef __attribute__((ext_vector_type(4))) float acc4;

// Developer build (-DNNTILE_DEC_TRACE): wall-clock stamps (100 MHz) of every
// workgroup of the last launch, read back with nntile_hip_debug_dec_trace.
#ifdef NNTILE_DEC_TRACE
__device__ unsigned long long dec_trace[8 * 2048];
#define DEC_STAMP(i) do { if(__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) == 0 \
        && blockIdx.x < 2048) { dec_trace[8 * blockIdx.x + (i)] = wall_clock64(); } } while(0)
#else
#define DEC_STAMP(i)
#endif

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

__device__ __forceinline__ u32x2 dec_lds_read_tr16(const char *lds_ptr)
{
    typedef __attribute__((ext_vector_type(4))) short s16x4;
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(lds_ptr));
    return __builtin_bit_cast(u32x2, v);
}

// The wait of the K/V ring, counted by hand: vmcnt retires in issue order, so
// "at most N outstanding" means everything but the N youngest loads is done.
// What a wavefront issues, in order (f(i) = the VM_PER_STEP global->LDS loads
// of key step i, m(i) = the KB ordinary loads of step i's mask values; the
// compiler's own wait counting sees m, not f, which is inline asm):
//   prologue   m(0) f(0) .. f(STAGES-2)
//   step it    wait_vmcnt<(STAGES-2)*VM_PER_STEP>   -> f(it) and m(it) are done:
//                  younger than them are only f(it+1) .. f(it+STAGES-2)
//              mcur = m(it)   (the compiler adds vmcnt(0) here, as it knows of
//                  no younger load: with two stages nothing is outstanding at
//                  that point; with three or four it drains f(it+1).., one
//                  step more than needed, for explicit masks only)
//              m(it+1) f(it+STAGES-1)
// so the most a wavefront ever has outstanding is (STAGES-1)*VM_PER_STEP + KB,
// which must stay below the counter's 64 (checked where VM_PER_STEP is defined).
// In the tail (fewer than STAGES-1 steps ahead) the wait is for everything.
template<int N> __device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    // s_waitcnt simm16: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[15:14]
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
    asm volatile("" ::: "memory");
}

// Loads that are served by the L2 (never by a CU's own cache): what one
// workgroup reads of memory another workgroup of the same launch has written.
template<bool COH>
__device__ __forceinline__ unsigned long long ld64(const void *ptr)
{
    if(COH)
    {
        return __hip_atomic_load(
                const_cast<unsigned long long *>(static_cast<const unsigned long long *>(ptr)),
                __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return *static_cast<const unsigned long long *>(ptr);
}

template<bool COH>
__device__ __forceinline__ float ld32f(const float *ptr)
{
    if(COH)
    {
        return __hip_atomic_load(const_cast<float *>(ptr), __ATOMIC_RELAXED,
                __HIP_MEMORY_SCOPE_AGENT);
    }
    return *ptr;
}

// The XCD this wavefront runs on (hardware register XCC_ID, bits 3:0).
__device__ __forceinline__ int xcc_id()
{
    return (int)(__builtin_amdgcn_s_getreg((31 << 11) | 20) & 15u);
}

// Merge workgroups of the fused form that gave up waiting for a flag (they
// leave their rows untouched); read with nntile_hip_debug_decode_sync_timeouts.
__device__ unsigned int decode_sync_timeouts;
// ... and those that found a split of their unit on another XCD than their own
// (rows untouched as well); read with nntile_hip_debug_decode_sync_misplaced.
__device__ unsigned int decode_sync_misplaced;

// Merge the split partials of row rr of a unit and fold the result into
// (lse, A).  The calling thread handles head values d4 .. d4+3.  COH: the
// partials were written by other workgroups of this launch.
template<typename T, int HEAD, bool COH>
__device__ __forceinline__ void decode_merge_row(const DecodeParams &p, int unit, int rr, int d4)
{
    static_assert(!COH || NNTILE_DEC_PART16, "the fused merge reads 16-bit partials");
    const int nb = unit % p.n_batch;
    const int hkv = unit / p.n_batch;
    const int g = rr / (int)p.q_seq, tok = rr % (int)p.q_seq;
    const int64_t qb = nb + (int64_t)p.n_batch * (g + (int64_t)p.kv_group * hkv);

    const int64_t base = (int64_t)unit * p.n_splits * p.rows + rr;
    const int last_split = p.n_splits - 1;
    typedef __attribute__((ext_vector_type(2))) float f32x2;
    // The loads of up to 8 splits are issued together (indices past the last
    // split are clamped and get weight 0): the latency of the partials is
    // paid once per 8 splits, not once per split; with at most 8 splits the
    // maxima and the values travel in the same round trip.
    const int64_t row = qb * p.q_seq + tok;
    uint16_t *Adst = static_cast<uint16_t *>(p.A) + row * HEAD + d4;
    float top = neg_inf();
    float l = 0.0f;
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    auto load8 = [&](int s0, f32x2 (&ml)[8], f32x4 (&v)[8])
    {
#pragma unroll
        for(int j = 0; j < 8; ++j)
        {
            const int sidx = min(s0 + j, last_split);
            const int64_t prow = base + (int64_t)sidx * p.rows;
            ml[j] = __builtin_bit_cast(f32x2, ld64<COH>(p.part_ml + 2 * prow));
#if NNTILE_DEC_PART16
            const u32x2 raw = __builtin_bit_cast(u32x2, ld64<COH>(
                    reinterpret_cast<const uint16_t *>(p.part_o) + prow * HEAD + d4));
            v[j] = f32x4{T::to_float((uint16_t)(raw[0] & 0xffffu)), T::to_float((uint16_t)(raw[0] >> 16)),
                T::to_float((uint16_t)(raw[1] & 0xffffu)), T::to_float((uint16_t)(raw[1] >> 16))};
#else
            v[j] = *reinterpret_cast<const f32x4 *>(p.part_o + prow * HEAD + d4);
#endif
        }
    };
    auto add8 = [&](int s0, const f32x2 (&ml)[8], const f32x4 (&v)[8])
    {
#pragma unroll
        for(int j = 0; j < 8; ++j)
        {
            const bool live = (s0 + j <= last_split) && (ml[j][0] != neg_inf());
#if NNTILE_DEC_PART16
            const float w = live ? __expf(ml[j][0] - top) * ml[j][1] : 0.0f;
            l += w;
#else
            const float w = live ? __expf(ml[j][0] - top) : 0.0f;
            l += w * ml[j][1];
#endif
            acc += w * v[j];
        }
    };
    if(p.n_splits <= 8)
    {
        f32x2 ml[8];
        f32x4 v[8];
        load8(0, ml, v);
#pragma unroll
        for(int j = 0; j < 8; ++j)
        {
            top = fmaxf(top, ml[j][0]);
        }
        if(top != neg_inf())
        {
            add8(0, ml, v);
        }
    }
    else
    {
        for(int s0 = 0; s0 < p.n_splits; s0 += 8)
        {
            float m[8];
#pragma unroll
            for(int j = 0; j < 8; ++j)
            {
                const int sidx = min(s0 + j, last_split);
                m[j] = ld32f<COH>(p.part_ml + 2 * (base + (int64_t)sidx * p.rows));
            }
#pragma unroll
            for(int j = 0; j < 8; ++j)
            {
                top = fmaxf(top, m[j]);
            }
        }
        if(top != neg_inf())
        {
            for(int s0 = 0; s0 < p.n_splits; s0 += 8)
            {
                f32x2 ml[8];
                f32x4 v[8];
                load8(s0, ml, v);
                add8(s0, ml, v);
            }
        }
    }
    if(top == neg_inf())
    {
        // no visible key at all: leave lse and A untouched, or write the
        // empty row when the running pair is being overwritten
        if(p.overwrite)
        {
            *reinterpret_cast<u32x2 *>(Adst) = u32x2{0, 0};
            if(d4 == 0)
            {
                p.lse[row] = neg_inf();
            }
        }
        return;
    }
    const float lse_new = top + __logf(l);
    const float lse_old = p.overwrite ? neg_inf() : p.lse[row];
    float w_old, w_new, lse_out;
    merge_weights(lse_old, lse_new, w_old, w_new, lse_out);
    const float sc = w_new / l;
    float v[4] = {acc[0] * sc, acc[1] * sc, acc[2] * sc, acc[3] * sc};
    if(w_old != 0.0f)
    {
        const u32x2 old = *reinterpret_cast<const u32x2 *>(Adst);
        v[0] += w_old * T::to_float((uint16_t)(old[0] & 0xffffu));
        v[1] += w_old * T::to_float((uint16_t)(old[0] >> 16));
        v[2] += w_old * T::to_float((uint16_t)(old[1] & 0xffffu));
        v[3] += w_old * T::to_float((uint16_t)(old[1] >> 16));
    }
    u32x2 out;
    out[0] = T::pack2(v[0], v[1]);
    out[1] = T::pack2(v[2], v[3]);
    *reinterpret_cast<u32x2 *>(Adst) = out;
    // The threads of a row sit in one wavefront (TPR <= 32 divides 64) and
    // run in lock step: all of them have read lse_old by now.
    if(d4 == 0)
    {
        p.lse[row] = lse_out;
    }
}

// A merge workgroup of the fused form: block `idx` behind the main workgroups.
// It is dispatched when main workgroups have left (the hardware starts the
// workgroups of a launch in index order, and the main ones never wait for
// anything), waits until every split of its unit has raised its flag, merges
// its rows and lowers the flags again.
//
// Placement: the workgroups of one launch go round the 8 XCDs in index order,
// so the main workgroups of a unit and its merge workgroups, whose indices
// are equal modulo 8 by construction, share an XCD and its L2: partials
// written by plain stores are there for plain loads once the writer's stores
// are acknowledged, no cache has to be written back or invalidated.  Where
// the round starts is not the launch's to say (XCD 0 on a fresh queue, another
// one after a graph launch or on a second stream - but one start per launch,
// also with several queues dispatching at once), so nothing here assumes a
// particular XCD: every main workgroup puts the number of the XCD it ran on
// (hardware register XCC_ID) into its flag and the merge workgroup compares
// it with its own.  A difference - never seen - is counted and the rows are
// left alone rather than merged from data that may not have arrived.  With
// p.fenced both sides use device-scope fences instead and placement is not
// looked at (for comparison: the fences write back and invalidate whole L2s).
template<typename T, int HEAD>
__device__ __forceinline__ void decode_merge_workgroup(const DecodeParams &p, int idx)
{
    constexpr int TPR = HEAD / 4;               // threads per row
    constexpr int ROWS_PER_WG = 256 / TPR;
    const int tid = threadIdx.x;
    const int x = idx & 7, j = idx >> 3;
    const int unit = (j / p.merge_blocks_per_unit) * 8 + x;
    const int rb = j % p.merge_blocks_per_unit;
    unsigned long long *flags = p.sync + (int64_t)unit * p.sync_stride + 1 + rb * p.n_splits;
    int bad = 0;
    if(tid < p.n_splits)
    {
        // (the tag's low four bits are clear: the flag carries the writer's XCD there)
        const unsigned long long t0 = wall_clock64();
        unsigned long long seen;
        while(((seen = ld64<true>(flags + tid)) & ~15ull) != p.tag)
        {
            __builtin_amdgcn_s_sleep(4);
            if(wall_clock64() - t0 > p.spin_limit)
            {
                bad = 1;
                break;
            }
        }
        if(!bad && !p.fenced && (int)(seen & 15ull) != xcc_id())
        {
            bad = 2;
        }
    }
    bad = __syncthreads_or(bad);
    if(bad)
    {
        if(tid == 0)
        {
            atomicAdd((bad & 1) ? &decode_sync_timeouts : &decode_sync_misplaced, 1u);
        }
        return;
    }
    if(p.fenced)
    {
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    }
    const int rr = rb * ROWS_PER_WG + tid / TPR;
    if(rr < p.rows)
    {
        decode_merge_row<T, HEAD, true>(p, unit, rr, (tid % TPR) * 4);
    }
    // every partial of these rows has been read: the flags go down for the
    // next call on this workspace (a replay of a captured graph has this
    // call's tag again)
    __syncthreads();
    if(tid < p.n_splits)
    {
        __hip_atomic_store(flags + tid, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// DIRECT: the unit has one key split, so the partial is the result and is
// folded into (lse, A) here; no partials are written and no merge kernel runs.
template<typename T, int HEAD, int MODE, int STAGES, bool DIRECT = false>
__global__ __launch_bounds__(kDecThreads, NNTILE_DEC_WGS_PER_CU)
void sdpa_decode_16bit_kernel(const DecodeParams p)
{
    typedef typename T::vec8 vec8;
    constexpr int KSTEPS = HEAD / 32;       // MFMA steps along head for S
    constexpr int DBLOCKS = HEAD / 16;      // 16-row blocks of O^T
    constexpr int KB = kDecKeys / 16;       // 16-key blocks of S^T per step
    constexpr int RB = HEAD * 2;            // bytes per K/V row
    constexpr int CPR = HEAD / 8;           // 16-byte chunks per row
    constexpr int RPL = 16 / CPR;           // rows per 256-byte line of LDS banks
    constexpr int ROWS_PER_LOAD = 1024 / RB;
    constexpr int LOADS = kDecKeys / ROWS_PER_LOAD;     // per K (or V) step
    constexpr int LOADS_PER_WAVE = LOADS / 4;
    constexpr int K_BYTES = kDecKeys * RB;
    constexpr int STAGE_BYTES = 2 * K_BYTES;            // K then V
    constexpr int VM_PER_STEP = 2 * LOADS_PER_WAVE;     // load instructions a wave issues per step
    static_assert((STAGES - 1) * VM_PER_STEP + kDecKeys / 16 < 64,
            "the ring's loads and one step's mask loads must fit the 6-bit vmcnt");
    constexpr bool EXPLICIT = (MODE == NNTILE_HIP_MASK_ADDITIVE
            || MODE == NNTILE_HIP_MASK_BOOL);
    static_assert(LOADS_PER_WAVE >= 1, "head size too small for this tiling");

    // One array per ring slot, not one array for all: the compiler then knows
    // that loads streaming into one slot cannot alias the reads of another and
    // does not make those reads wait for the loads.  (Unused slots of a
    // shallower ring are dropped.)
    __shared__ __attribute__((aligned(1024))) char ring0[STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring1[STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring2[STAGES > 2 ? STAGE_BYTES : 16];
    __shared__ __attribute__((aligned(1024))) char ring3[STAGES > 3 ? STAGE_BYTES : 16];
    auto ring = [&](auto tag) -> char *
    {
        constexpr int I = decltype(tag)::value % STAGES;
        if constexpr(I == 0) { return ring0; }
        else if constexpr(I == 1) { return ring1; }
        else if constexpr(I == 2) { return ring2; }
        else { return ring3; }
    };

    // The grid: n_main main workgroups, then (merge in the launch) the merge
    // workgroups, then (append in the launch) one copying workgroup per unit.
    if((int)blockIdx.x >= p.n_main)
    {
        const int n_merge = p.fused ? p.n_batch * p.n_head_kv * p.merge_blocks_per_unit : 0;
        const int behind = (int)blockIdx.x - p.n_main;
        if(behind >= n_merge)
        {
            // New rows into the caches: 16 bytes a thread and piece.  Nobody in
            // this launch reads them there (the main workgroups take them from
            // k_new / v_new), so there is nothing to wait for or to signal.
            const int unit_a = behind - n_merge;
            const int64_t filled = p.k_seq - p.n_new;
            const int n16 = p.n_new * (RB / 16);
            for(int t = threadIdx.x; t < 2 * n16; t += kDecThreads)
            {
                const int which = t >= n16 ? 1 : 0;
                const int piece = t - which * n16;
                const char *src = static_cast<const char *>(which ? p.v_new : p.k_new)
                    + ((int64_t)unit_a * p.n_new * RB + (int64_t)piece * 16);
                char *dst = static_cast<char *>(const_cast<void *>(which ? p.V : p.K))
                    + (((int64_t)unit_a * p.kv_rows + filled) * RB + (int64_t)piece * 16);
                *reinterpret_cast<u32x4 *>(dst) = *reinterpret_cast<const u32x4 *>(src);
            }
            return;
        }
        if constexpr(!DIRECT)
        {
            DEC_STAMP(5);
            decode_merge_workgroup<T, HEAD>(p, behind);
#ifdef NNTILE_DEC_TRACE
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            DEC_STAMP(6);
#endif
        }
        return;
    }
    DEC_STAMP(0);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int col = lane & 15;       // row (query) within the wavefront
    const int quad = lane >> 4;      // 0..3

    // Workgroups are dealt round-robin to the 8 XCDs.  All key splits of a
    // unit go to one XCD, and so do the workgroups of the merge kernel that
    // read the unit's partials: the partials then stay within one L2
    // (cfg4: 50.6 -> 50.0 us per step).
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
            unit = blockIdx.x / p.n_splits;        // nb + n_batch*hkv
        }
    }
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

    const char *Kb = static_cast<const char *>(p.K) + (int64_t)unit * p.kv_rows * RB;
    const char *Vb = static_cast<const char *>(p.V) + (int64_t)unit * p.kv_rows * RB;

    // ---- LDS layout and the lane's fixed addresses ---------------------------
    // chunk c of row r sits at chunk position
    //   K:  c ^ ((r / RPL) % CPR)          16 consecutive rows, same c -> 16 bank groups
    //   V:  c ^ (2 * ((r / RPL) % (CPR/2)))  8 consecutive rows x 32 B -> 8 bank groups
    // Load instruction `ld` fills rows [ld*ROWS_PER_LOAD, +ROWS_PER_LOAD): lane L
    // lands on row ld*ROWS_PER_LOAD + L/CPR, chunk position L % CPR.
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    uint32_t k_goff[LOADS_PER_WAVE], v_goff[LOADS_PER_WAVE];
    int ld_row[LOADS_PER_WAVE];
    const int ld_cpos = lane % CPR;
#pragma unroll
    for(int i = 0; i < LOADS_PER_WAVE; ++i)
    {
        const int r = (wave * LOADS_PER_WAVE + i) * ROWS_PER_LOAD + lane / CPR;
        ld_row[i] = r;
        k_goff[i] = (uint32_t)(r * RB + (ld_cpos ^ ((r / RPL) % CPR)) * 16);
        v_goff[i] = (uint32_t)(r * RB
                + (ld_cpos ^ (2 * ((r / RPL) % (CPR / 2)))) * 16);
    }
    // S operand: lane (col, quad) reads row 16*kb + col, logical chunk 4*ks + quad;
    // 16*kb goes into the immediate offset.
    uint32_t k_raddr[KSTEPS];
#pragma unroll
    for(int ks = 0; ks < KSTEPS; ++ks)
    {
        k_raddr[ks] = (uint32_t)(col * RB + ((4 * ks + quad) ^ ((col / RPL) % CPR)) * 16);
    }
    // PV operand through the transposing read: a 16-lane block is one quad;
    // lane i addresses key j = i/4 and head values 4*(i%4)..+3 of the block's
    // 16 head values and receives keys 0..3 of head value i.  For the 32-key
    // step t and instruction a the row is 32t + 16a + 4*quad + j; 32t + 16a goes
    // into the immediate offset.
    uint32_t v_raddr[DBLOCKS];
    {
        const int j = col >> 2, r4 = col & 3;
        const int r = 4 * quad + j;
        const int swz = 2 * ((r / RPL) % (CPR / 2));
#pragma unroll
        for(int db = 0; db < DBLOCKS; ++db)
        {
            const int c = 2 * db + (r4 >> 1);
            v_raddr[db] = (uint32_t)(K_BYTES + r * RB + (c ^ swz) * 16 + 8 * (r4 & 1));
        }
    }


    // Loads of key step `step` into ring slot `slot`; rows past the end of the
    // cache are clamped to its last row (their probabilities are exactly 0).
    auto fetch = [&](int step, char *slot_base)
    {
        const int64_t row0 = (int64_t)step * kDecKeys;
        const char *Kp = Kb + row0 * RB;
        const char *Vp = Vb + row0 * RB;
        char *kdst = slot_base + wave_u * LOADS_PER_WAVE * 1024;
        char *vdst = kdst + K_BYTES;
        const int rows_left = (int)min((int64_t)kDecKeys, p.k_seq - row0);
        if(p.n_new > 0 && row0 + kDecKeys > p.k_seq - p.n_new)
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
                load_to_lds16<0, NNTILE_DMA_NT>(ks + kc, kdst + i * 1024);
                load_to_lds16<0, NNTILE_DMA_NT>(vs + vc, vdst + i * 1024);
            }
        }
        else if(rows_left >= kDecKeys)
        {
#pragma unroll
            for(int i = 0; i < LOADS_PER_WAVE; ++i)
            {
                load_to_lds16<0, NNTILE_DMA_NT>(Kp + k_goff[i], kdst + i * 1024);
                load_to_lds16<0, NNTILE_DMA_NT>(Vp + v_goff[i], vdst + i * 1024);
            }
        }
        else
        {
            const int last = rows_left - 1;
#pragma unroll
            for(int i = 0; i < LOADS_PER_WAVE; ++i)
            {
                const uint32_t back = (uint32_t)(max(ld_row[i] - last, 0) * RB);
                load_to_lds16<0, NNTILE_DMA_NT>(Kp + (k_goff[i] - back), kdst + i * 1024);
                load_to_lds16<0, NNTILE_DMA_NT>(Vp + (v_goff[i] - back), vdst + i * 1024);
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

    // The workgroups of a launch advance through their key ranges at the same
    // pace and the ranges start a power-of-two number of bytes apart, which
    // would keep all of them on the same few memory channels at any moment.
    // Each workgroup therefore starts at its own rotation of its range (the
    // online softmax does not care about the order of the steps).
    const int n_local = step_hi - step_lo;
    const int rot = n_local > 0 ? (int)((blockIdx.x * 7u + (blockIdx.x >> 3)) % (unsigned)n_local) : 0;
    auto actual = [&](int i) -> int
    {
        const int j = i + rot;
        return step_lo + (j >= n_local ? j - n_local : j);
    };

    // Explicit mask: the raw values of a full step of the mask - per
    // block of 16 keys the lane's four consecutive keys, one 8-byte (additive)
    // or 4-byte (boolean) load - are requested one step ahead, BEFORE that
    // step's K/V loads are issued.  Waiting for a load also waits for every
    // load issued before it, so mask values requested behind the K/V loads of
    // the next step would make each step wait for its successor's data.
    u32x2 mnext[KB];
#pragma unroll
    for(int kb = 0; kb < KB; ++kb)
    {
        mnext[kb] = u32x2{0u, 0u};
    }
    bool mnext_wide = false;
    // (masks of any row length and start: the loads carry the alignment of one
    // element, which global memory accepts)
    const bool mask_aligned = EXPLICIT;
    typedef u32x2 __attribute__((aligned(2))) u32x2_any;
    typedef uint32_t __attribute__((aligned(1))) u32_any;
    auto mask_request = [&](int it_req)
    {
        mnext_wide = false;
        if(EXPLICIT && mask_aligned && it_req < n_local)
        {
            const int64_t kr = (int64_t)actual(it_req) * kDecKeys;
            if(p.k_seq - kr >= kDecKeys)
            {
                mnext_wide = true;
                const int64_t at = (int64_t)tok * p.mask_ld + kr + 4 * quad;
#pragma unroll
                for(int kb = 0; kb < KB; ++kb)
                {
                    if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                    {
                        mnext[kb] = *reinterpret_cast<const u32x2_any *>(
                                static_cast<const uint16_t *>(p.mask) + at + 16 * kb);
                    }
                    else
                    {
                        mnext[kb][0] = *reinterpret_cast<const u32_any *>(
                                static_cast<const uint8_t *>(p.mask) + at + 16 * kb);
                    }
                }
            }
        }
    };
    mask_request(0);

    // prologue: STAGES-1 steps in flight
    if(0 < n_local) { fetch(actual(0), ring(std::integral_constant<int, 0>{})); }
    if(STAGES > 2 && 1 < n_local) { fetch(actual(1), ring(std::integral_constant<int, 1>{})); }
    if(STAGES > 3 && 2 < n_local) { fetch(actual(2), ring(std::integral_constant<int, 2>{})); }

    // One key step on ring slot SLOT (a compile-time constant).
    auto body = [&](int it, auto slot_tag)
    {
        constexpr int SLOT = decltype(slot_tag)::value;
        const int step = actual(it);
        // this step's data has landed: everything but the loads of the later
        // steps in flight is complete (in the tail fewer steps are in flight)
        if(it + STAGES - 1 <= n_local)
        {
            wait_vmcnt<(STAGES - 2) * VM_PER_STEP>();
        }
        else
        {
            wait_vmcnt<0>();
        }
        // ... for every wavefront, and everyone is done with the previous step.
        // A bare barrier: __syncthreads() would also drain the loads of the
        // later steps (its release fence waits for every outstanding store,
        // and a global->LDS load counts as one), which is exactly what the
        // ring is there to avoid.  LDS reads are ordered by lgkmcnt, the
        // loads by the explicit vmcnt above.
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#ifdef NNTILE_DEC_TRACE
        if(it == 0) { DEC_STAMP(1); }
        if(it == n_local - 1) { DEC_STAMP(2); }
#endif
        // this step's mask values (they arrived with the wait above: the use
        // below is where the compiler puts its own wait), then the request
        // for the next step's
        u32x2 mcur[KB];
        const bool cur_wide = mnext_wide;
        if(EXPLICIT)
        {
#pragma unroll
            for(int kb = 0; kb < KB; ++kb)
            {
                mcur[kb] = mnext[kb];
                asm volatile("" : "+v"(mcur[kb]));
            }
            mask_request(it + 1);
        }
        {
            const int ahead = it + STAGES - 1;
            if(ahead < n_local)
            {
                // into the slot the previous step used
                fetch(actual(ahead),
                        ring(std::integral_constant<int, SLOT + STAGES - 1>{}));
            }
        }
        const char *Ks = ring(slot_tag);

        const int64_t k_row0 = (int64_t)step * kDecKeys;
        const int64_t k_pos_base = p.k_pos0 + k_row0;
        const int keys_here = (int)min((int64_t)kDecKeys, p.k_seq - k_row0);

        // ---- S^T = K Q^T: 4 blocks of 16 keys ----------------------------------
        acc4 s[KB];
#pragma unroll
        for(int kb = 0; kb < KB; ++kb)
        {
            s[kb] = acc4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for(int ks = 0; ks < KSTEPS; ++ks)
            {
                const vec8 a = *reinterpret_cast<const vec8 *>(
                        Ks + k_raddr[ks] + kb * 16 * RB);
                s[kb] = Mfma16<T>::run(a, qf[ks], s[kb]);
            }
        }

        // ---- mask: s[kb][r] is key 16*kb + 4*quad + r ----------------------------
        if(EXPLICIT)
        {
            // the mask is [k_seq, q_seq]: row index = token.  A full step of
            // an aligned mask finds its values in mcur.  Otherwise element by
            // element: keys past the end of a ragged step are hidden, and
            // their loads are clamped to the step's last key instead of being
            // branched around, so that a lane's loads are independent.
            const int64_t mrow = (int64_t)tok * p.mask_ld + k_row0;
#pragma unroll
            for(int kb = 0; kb < KB; ++kb)
            {
                const int key0 = 16 * kb + 4 * quad;
                float add[4];
                if(cur_wide)
                {
                    const u32x2 w = mcur[kb];
#pragma unroll
                    for(int e = 0; e < 4; ++e)
                    {
                        if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                        {
                            add[e] = T::to_float((uint16_t)(
                                        (e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu)));
                        }
                        else
                        {
                            add[e] = ((w[0] >> (8 * e)) & 0xffu) != 0u ? 0.0f : neg_inf();
                        }
                    }
                }
                else
                {
#pragma unroll
                    for(int e = 0; e < 4; ++e)
                    {
                        const int64_t mi = mrow + max(min(key0 + e, keys_here - 1), 0);
                        if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                        {
                            add[e] = T::to_float(static_cast<const uint16_t *>(p.mask)[mi]);
                        }
                        else
                        {
                            add[e] = static_cast<const uint8_t *>(p.mask)[mi] != 0
                                ? 0.0f : neg_inf();
                        }
                        if(key0 + e >= keys_here)
                        {
                            add[e] = neg_inf();
                        }
                    }
                }
#pragma unroll
                for(int e = 0; e < 4; ++e)
                {
                    const float v = s[kb][e] * p.scale + add[e];
                    s[kb][e] = (add[e] == neg_inf()) ? neg_inf() : v;
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
        uint32_t pk[KB][2];
#pragma unroll
        for(int kb = 0; kb < KB; ++kb)
        {
            const float p0 = fast_exp2(fmaf(s[kb][0], c, -mc));
            const float p1 = fast_exp2(fmaf(s[kb][1], c, -mc));
            const float p2 = fast_exp2(fmaf(s[kb][2], c, -mc));
            const float p3 = fast_exp2(fmaf(s[kb][3], c, -mc));
            pk[kb][0] = T::pack2(p0, p1);
            pk[kb][1] = T::pack2(p2, p3);
            // (plain additions: the dot-product instruction that would sum a
            // packed pair waits for the matrix unit)
            rs += (p0 + p1) + (p2 + p3);
        }
        l_run += rs;

        // ---- O^T += V^T P^T: 2 steps of 32 keys ----------------------------------
#pragma unroll
        for(int t = 0; t < KB / 2; ++t)
        {
            const u32x4 praw = {pk[2 * t][0], pk[2 * t][1], pk[2 * t + 1][0],
                pk[2 * t + 1][1]};
            const vec8 pb = __builtin_bit_cast(vec8, praw);
            // all operand reads of this 32-key step first, then the MFMAs, so
            // that the LDS latency is paid once and not once per MFMA
            u32x4 araw[DBLOCKS];
#pragma unroll
            for(int db = 0; db < DBLOCKS; ++db)
            {
                const char *src = Ks + v_raddr[db] + (32 * t) * RB;
                const u32x2 lo = dec_lds_read_tr16(src);
                const u32x2 hi = dec_lds_read_tr16(src + 16 * RB);
                araw[db] = u32x4{lo[0], lo[1], hi[0], hi[1]};
            }
#pragma unroll
            for(int db = 0; db < DBLOCKS; ++db)
            {
                o[db] = Mfma16<T>::run(__builtin_bit_cast(vec8, araw[db]), pb, o[db]);
            }
        }
    };

    for(int it = 0; it < n_local; it += STAGES)
    {
        body(it, std::integral_constant<int, 0>{});
        if(it + 1 < n_local) { body(it + 1, std::integral_constant<int, 1>{}); }
        if(STAGES > 2 && it + 2 < n_local) { body(it + 2, std::integral_constant<int, 2>{}); }
        if(STAGES > 3 && it + 3 < n_local) { body(it + 3, std::integral_constant<int, 3>{}); }
    }

    // ---- write the partial ---------------------------------------------------------
    DEC_STAMP(3);
    float l_tot = l_run + __shfl_xor(l_run, 16);
    l_tot = sum_across_halves(l_tot);
    if constexpr(DIRECT)
    {
        if(!row_ok)
        {
            return;
        }
        const int g = rr / (int)p.q_seq, tok = rr % (int)p.q_seq;
        const int64_t qb = nb + (int64_t)p.n_batch * (g + (int64_t)p.kv_group * hkv);
        const int64_t row = qb * p.q_seq + tok;
        uint16_t *Adst = static_cast<uint16_t *>(p.A) + row * HEAD + 4 * quad;
        if(m_run == neg_inf() || !(l_tot > 0.0f))
        {
            // no visible key at all: leave lse and A untouched, or write the
            // empty row when the running pair is being overwritten
            if(p.overwrite)
            {
#pragma unroll
                for(int db = 0; db < DBLOCKS; ++db)
                {
                    *reinterpret_cast<u32x2 *>(Adst + 16 * db) = u32x2{0, 0};
                }
                if(quad == 0)
                {
                    p.lse[row] = neg_inf();
                }
            }
            return;
        }
        const float to_ln = EXPLICIT ? 1.0f : p.scale;
        const float lse_new = m_run * to_ln + __logf(l_tot);
        const float lse_old = p.overwrite ? neg_inf() : p.lse[row];
        float w_old, w_new, lse_out;
        merge_weights(lse_old, lse_new, w_old, w_new, lse_out);
        const float sc = w_new / l_tot;
#pragma unroll
        for(int db = 0; db < DBLOCKS; ++db)
        {
            float v[4] = {o[db][0] * sc, o[db][1] * sc, o[db][2] * sc, o[db][3] * sc};
            if(w_old != 0.0f)
            {
                const u32x2 old = *reinterpret_cast<const u32x2 *>(Adst + 16 * db);
                v[0] += w_old * T::to_float((uint16_t)(old[0] & 0xffffu));
                v[1] += w_old * T::to_float((uint16_t)(old[0] >> 16));
                v[2] += w_old * T::to_float((uint16_t)(old[1] & 0xffffu));
                v[3] += w_old * T::to_float((uint16_t)(old[1] >> 16));
            }
            u32x2 w;
            w[0] = T::pack2(v[0], v[1]);
            w[1] = T::pack2(v[2], v[3]);
            *reinterpret_cast<u32x2 *>(Adst + 16 * db) = w;
        }
        // The four lanes of a row sit in one wavefront and run in lock step:
        // all of them have read lse_old by now.
        if(quad == 0)
        {
            p.lse[row] = lse_out;
        }
        return;
    }
    if(row_ok)
    {
    const int64_t prow = ((int64_t)unit * p.n_splits + split) * p.rows + rr;
    if(quad == 0)
    {
        // max in natural-log units so that the reduce kernel needs no mode
        const float to_ln = EXPLICIT ? 1.0f : p.scale;
        p.part_ml[2 * prow] = (m_run == neg_inf()) ? neg_inf() : m_run * to_ln;
        p.part_ml[2 * prow + 1] = l_tot;
    }
    // o[db][r] is head value 16*db + 4*quad + r of row rr
#if NNTILE_DEC_PART16
    // the partial output, normalised, in the tile type: half the bytes of
    // fp32 partials (one more rounding, as the reference's scratch tile has)
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    uint16_t *dst = reinterpret_cast<uint16_t *>(p.part_o) + prow * HEAD + 4 * quad;
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
        u32x2 w;
        w[0] = T::pack2(o[db][0] * inv, o[db][1] * inv);
        w[1] = T::pack2(o[db][2] * inv, o[db][3] * inv);
        *reinterpret_cast<u32x2 *>(dst + 16 * db) = w;
    }
#else
    float *dst = p.part_o + prow * HEAD + 4 * quad;
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
        *reinterpret_cast<acc4 *>(dst + 16 * db) = o[db];
    }
#endif
    }
#ifdef NNTILE_DEC_TRACE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    DEC_STAMP(4);
#endif
    if(p.fused)
    {
        // The partial is complete in this XCD's L2 once every wavefront's
        // stores have been acknowledged (the barrier's release waits for
        // them); then one flag per merge workgroup of the unit goes up, with
        // the number of this XCD in its low bits.
        __syncthreads();
        if(p.fenced)
        {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        }
        if(tid < p.merge_blocks_per_unit)
        {
            __hip_atomic_store(p.sync + (int64_t)unit * p.sync_stride + 1 + tid * p.n_splits + split,
                    p.tag | (unsigned long long)xcc_id(), __ATOMIC_RELAXED,
                    __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// Merge the split partials of each row and fold the result into (lse, A).
// A thread handles 4 head values of one row; a workgroup of 256 threads
// handles 1024/HEAD rows.
template<typename T, int HEAD>
__global__ __launch_bounds__(256)
void sdpa_decode_reduce_kernel(const DecodeParams p)
{
    DEC_STAMP(5);
    constexpr int TPR = HEAD / 4;               // threads per row
    constexpr int ROWS_PER_WG = 256 / TPR;
    const int64_t total_rows = (int64_t)p.n_batch * p.n_head_kv * p.rows;
    // (the unit's row blocks on the XCD that computed its partials)
    int64_t grow;
    {
        const int units = p.n_batch * p.n_head_kv;
        const int blocks_per_unit = (p.rows + ROWS_PER_WG - 1) / ROWS_PER_WG;
        if(units % 8 == 0 && p.rows % ROWS_PER_WG == 0)
        {
            const int x = blockIdx.x & 7, j = blockIdx.x >> 3;
            const int u = (j / blocks_per_unit) * 8 + x;
            const int rb = j % blocks_per_unit;
            grow = (int64_t)u * p.rows + rb * ROWS_PER_WG + threadIdx.x / TPR;
        }
        else
        {
            grow = (int64_t)blockIdx.x * ROWS_PER_WG + threadIdx.x / TPR;
        }
    }
    if(grow >= total_rows)
    {
        return;
    }
    decode_merge_row<T, HEAD, false>(p, (int)(grow / p.rows), (int)(grow % p.rows),
            (threadIdx.x % TPR) * 4);
#ifdef NNTILE_DEC_TRACE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    DEC_STAMP(6);
#endif
}

#ifdef NNTILE_DEC_TRACE
extern "C" int nntile_hip_debug_dec_trace(unsigned long long *host)
{
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(dec_trace), sizeof(dec_trace));
}
#endif

// 64-bit words of the sync area per unit (fused merge): one reserved word and
// a flag per (merge workgroup of the unit, split), rounded to 64 bytes.
int decode_sync_stride(int n_splits, int rows, int head)
{
    const int rows_per_wg = 256 / (head / 4);
    const int merge_blocks = (rows + rows_per_wg - 1) / rows_per_wg;
    return (1 + merge_blocks * n_splits + 7) / 8 * 8;
}

// A value no earlier call of this process has used and that memory left
// behind by anything else is unlikely to hold: a random upper half fixed at
// load time, a counter below it; the low four bits stay clear (a flag holds
// the tag plus the number of the XCD that raised it).
static unsigned long long next_decode_tag()
{
    static const unsigned long long salt = []
    {
        std::random_device rd;
        return ((unsigned long long)rd() << 32) | 0x80000000ull;
    }();
    static std::atomic<unsigned long long> counter{0};
    unsigned long long tag = salt + ((counter.fetch_add(1, std::memory_order_relaxed) + 1ull) << 4);
    return tag == 0ull ? 16ull : tag;
}

// Longest wait of a merge workgroup for a flag, in ticks of the 100 MHz clock
// (2 s unless a test sets it).
static std::atomic<unsigned long long> decode_spin_limit{200000000ull};

extern "C" unsigned long long nntile_hip_debug_decode_spin_limit(unsigned long long ticks)
{
    return decode_spin_limit.exchange(ticks);
}

extern "C" long long nntile_hip_debug_decode_sync_misplaced(void)
{
    unsigned int n = 0;
    if(hipMemcpyFromSymbol(&n, HIP_SYMBOL(decode_sync_misplaced), sizeof(n)) != hipSuccess)
    {
        (void)hipGetLastError();
        return -1;
    }
    return (long long)n;
}

extern "C" long long nntile_hip_debug_decode_sync_timeouts(void)
{
    unsigned int n = 0;
    if(hipMemcpyFromSymbol(&n, HIP_SYMBOL(decode_sync_timeouts), sizeof(n)) != hipSuccess)
    {
        return -1;
    }
    return (long long)n;
}

template<typename T, int HEAD, int MODE, int STAGES>
static void launch_decode_main(hipStream_t stream, const DecodeParams &p, dim3 grid)
{
    if(p.n_splits == 1)
    {
        auto kernel = sdpa_decode_16bit_kernel<T, HEAD, MODE, STAGES, true>;
        hipLaunchKernelGGL(kernel, grid, dim3(kDecThreads), 0, stream, p);
        return;
    }
    auto kernel = sdpa_decode_16bit_kernel<T, HEAD, MODE, STAGES>;
    hipLaunchKernelGGL(kernel, grid, dim3(kDecThreads), 0, stream, p);
}

template<typename T, int HEAD, int STAGES>
static int launch_decode_stages(hipStream_t stream, DecodeParams &p, int mode)
{
    const int units = p.n_batch * p.n_head_kv;
    constexpr int rows_per_wg = 256 / (HEAD / 4);
    const int merge_blocks = (p.rows + rows_per_wg - 1) / rows_per_wg;
    // The merge rides in the main launch when the caller allows it, the unit
    // has several splits and the units map onto the XCDs (8 at a time).
    p.fused = (p.fused && p.n_splits > 1 && units % 8 == 0 && p.sync != nullptr
            && NNTILE_DEC_PART16) ? 1 : 0;
    p.n_main = units * p.n_splits;
    p.merge_blocks_per_unit = merge_blocks;
    p.sync_stride = decode_sync_stride(p.n_splits, p.rows, HEAD);
    if(p.fused)
    {
        p.tag = next_decode_tag();
        p.spin_limit = decode_spin_limit.load(std::memory_order_relaxed);
    }
    p.n_append = p.n_new > 0 ? units : 0;
    const dim3 grid((unsigned)(p.n_main + (p.fused ? units * merge_blocks : 0) + p.n_append));
    switch(mode)
    {
        case NNTILE_HIP_MASK_ADDITIVE:
            launch_decode_main<T, HEAD, NNTILE_HIP_MASK_ADDITIVE, STAGES>(stream, p, grid);
            break;
        case NNTILE_HIP_MASK_NONE:
            launch_decode_main<T, HEAD, NNTILE_HIP_MASK_NONE, STAGES>(stream, p, grid);
            break;
        case NNTILE_HIP_MASK_CAUSAL:
            launch_decode_main<T, HEAD, NNTILE_HIP_MASK_CAUSAL, STAGES>(stream, p, grid);
            break;
        case NNTILE_HIP_MASK_BOOL:
            launch_decode_main<T, HEAD, NNTILE_HIP_MASK_BOOL, STAGES>(stream, p, grid);
            break;
        default:
            return NNTILE_HIP_EINVAL;
    }
    if(hipGetLastError() != hipSuccess)
    {
        return NNTILE_HIP_ELAUNCH;
    }
    if(p.n_splits > 1 && !p.fused)
    {
        const int64_t total_rows = (int64_t)units * p.rows;
        hipLaunchKernelGGL((sdpa_decode_reduce_kernel<T, HEAD>),
                dim3((unsigned)((total_rows + rows_per_wg - 1) / rows_per_wg)),
                dim3(256), 0, stream, p);
    }
    return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
}

// Ring depth 2 (64 KB of LDS at head 128) lets two workgroups share a CU, which
// measured faster than one workgroup with a deeper ring.
template<typename T, int HEAD>
static int launch_decode_head(hipStream_t stream, DecodeParams &p, int mode)
{
    return launch_decode_stages<T, HEAD, NNTILE_DEC_STAGES>(stream, p, mode);
}

// Number of key splits per unit: two workgroups per CU when the units allow
// it, never more than one split per key step.  Fewer splits mean fewer
// partials to write and merge.
int decode_choose_splits(int units, int n_steps)
{
    int splits = (NNTILE_DEC_WGS_PER_CU * kDecodeCUs + units - 1) / units;
    splits = splits < 1 ? 1 : splits;
    splits = splits > n_steps ? n_steps : splits;
    splits = splits > 64 ? 64 : splits;
    return splits;
}

// The workspace: the partial outputs [unit][split][rows][head], then the
// (max, sum) pairs [unit][split][rows][2] in fp32
size_t decode_partial_o_bytes(int units, int n_splits, int rows, int head)
{
    return (size_t)units * n_splits * rows * head * (NNTILE_DEC_PART16 ? 2 : sizeof(float));
}

size_t decode_partial_ml_bytes(int units, int n_splits, int rows)
{
    return (size_t)units * n_splits * rows * 2 * sizeof(float);
}

size_t decode_workspace_bytes(int units, int n_splits, int rows, int head)
{
    return decode_partial_o_bytes(units, n_splits, rows, head)
        + decode_partial_ml_bytes(units, n_splits, rows)
        + (size_t)units * decode_sync_stride(n_splits, rows, head) * sizeof(unsigned long long);
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
