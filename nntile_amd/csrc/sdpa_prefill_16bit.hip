// Prefill attention forward for 16-bit tiles (bf16 / fp16) on gfx950.
//
// One workgroup = 4 wavefronts = 128 queries of one (batch entry, query tile);
// each wavefront owns 32 queries.  Keys are walked in steps of 64.
//
//   S^T = K Q^T    v_mfma_f32_32x32x16: A = 32 keys x 16 head values read from
//                  LDS, B = 16 head values x 32 queries held in registers for
//                  the whole kernel.  In the 32x32 accumulator layout a lane
//                  holds ONE query (lane % 32) and 16 of the 32 keys, so the
//                  row maximum and the row sum of the softmax are reductions
//                  over the lane's own registers plus one exchange with lane^32.
//   O^T += V^T P^T A = 32 head values x 16 keys read from LDS, B = P^T taken
//                  straight from the S^T accumulators (converted to 16 bit) -
//                  the accumulator layout of the first product IS the B layout
//                  of the second, up to a fixed permutation of the 16 keys,
//                  and the V operand is gathered in that permuted key order.
//
// K and V steps go from global memory straight into LDS (global_load_lds,
// 16 bytes per lane, no register round trip), double-buffered, one barrier per
// step; the loads of step g+1 are issued at the top of step g.  A load
// instruction fills 1 KB of LDS contiguously, so rows cannot be padded; bank
// conflicts are avoided by XOR-swizzling the 16-byte chunks of a row instead
// (each lane picks the global chunk that belongs at its LDS position).
// V arrives with the head axis contiguous but the second product contracts
// over keys: its MFMA operand is read with ds_read_b64_tr_b16, which hands
// each lane 4 keys of one head value from a 4 x 16 block.
//
// The running (max, sum) pair lives in registers across all key tiles of a
// query tile; the epilogue merges the result into the (lse, A) pair in memory
// (the hand-off between NNTile tasks), so one launch can stand for one task or
// for a whole row of tasks.
#include <atomic>
#include <random>
#include <type_traits>

#include "sdpa_common.hpp"

#ifndef NNTILE_PF_AHEAD
#define NNTILE_PF_AHEAD 3
#endif

namespace nntile_hip
{

constexpr int kQRows = 128;     // queries per workgroup of four wavefronts
constexpr int kKeys = 64;       // keys per step
constexpr int kThreads = 256;
constexpr unsigned kCUsPerXCD = 32;   // MI355X: 256 CUs in 8 XCDs

// Walks the key steps of all key tiles in order: tile kt, step kb within the
// tile, rows left in the tile from this step on.
struct StepCursor
{
    int kt, kb, rows_left;
    const char *Kp, *Vp;    // first row of the step in the current key tile
};

// ds_read_b64_tr_b16: within each block of 16 lanes, lane i supplies the
// address of 4 consecutive 16-bit values of row i/4 (values 4*(i%4)..+3 of
// 16) and receives value i of rows 0..3.
__device__ __forceinline__ u32x2 lds_read_tr16(const char *lds_ptr)
{
    typedef __attribute__((ext_vector_type(4))) short s16x4;
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(lds_ptr));
    return __builtin_bit_cast(u32x2, v);
}

// Developer build (-DNNTILE_PF_TRACE): wall-clock stamps (100 MHz) of every
// workgroup of the last launch - start, first step in LDS, end of the
// pipelined loop, end of the key steps, end - plus where it ran and how many
// steps it had; read back with nntile_hip_debug_pf_trace.
#ifdef NNTILE_PF_TRACE
__device__ unsigned long long pf_trace[8 * 4096];
#define PF_STAMP(i) do { if(__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) == 0 \
        && blockIdx.x < 4096) { pf_trace[8 * blockIdx.x + (i)] = wall_clock64(); } } while(0)
#define PF_NOTE(i, v) do { if(__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) == 0 \
        && blockIdx.x < 4096) { pf_trace[8 * blockIdx.x + (i)] = (unsigned long long)(v); } } while(0)
extern "C" int nntile_hip_debug_pf_trace(unsigned long long *host)
{
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(pf_trace), sizeof(pf_trace));
}
#else
#define PF_STAMP(i)
#define PF_NOTE(i, v)
#endif

// WAVES: wavefronts per workgroup, 32 queries each.  4: two workgroups share a
// CU.  8 (analytic masks, head 64 and 128): one workgroup of 256 queries per
// CU, whose eight wavefronts share every K/V step - a CU then brings each step
// into LDS once where two workgroups of four bring it twice.
// Scan of the mask rows of query block qb over key range sp of kMaskBitSplits:
// the workgroup (THREADS threads) ORs what it finds in its range of 16-byte
// chunks into bits[0] (bit s: some value of 64-key step s is not "open") and
// bits[1] (not "hidden"); steps from 63 on share bit 63.  ES: bytes per mask
// element; open / hidden: the 32-bit pattern of four (two) visible / hidden
// elements.  bits is valid for every thread on return.
template<int ES, int THREADS>
__device__ __forceinline__ void mask_scan_range(const char *mask, int ld_bytes, int q_len,
        int n_chunks, uint32_t open_word, uint32_t hidden_word, int qb, int sp,
        unsigned long long *bits)
{
    constexpr int CHUNKS_PER_STEP = kKeys * ES / 16;
    const int tid = threadIdx.x;
    if(tid == 0)
    {
        bits[0] = 0ull;
        bits[1] = 0ull;
    }
    __syncthreads();
    const int per_split = (n_chunks + kMaskBitSplits - 1) / kMaskBitSplits;
    const int c_lo = min(sp * per_split, n_chunks);
    const int n_loc = min(c_lo + per_split, n_chunks) - c_lo;
    const int q_row0 = qb * kQRows;
    const int n_rows = min(kQRows, q_len - q_row0);
    unsigned long long not_open = 0ull, not_hidden = 0ull;
    if(n_loc > 0)
    {
        const int total = n_rows * n_loc;
        const char *mbase = mask + (int64_t)q_row0 * ld_bytes + (int64_t)c_lo * 16;
        // chunk tid, tid + THREADS, ... of the rows' pieces laid end to end
        const int d_row = THREADS / n_loc, d_c = THREADS % n_loc;
        int row = tid / n_loc, c = tid % n_loc;
        for(int base = 0; base < total; base += 16 * THREADS)
        {
            // (rows past the end re-read the last row: no branches, so that
            // the 16 loads are in flight together)
            u32x4 v[16];
            int st[16];
#pragma unroll
            for(int u = 0; u < 16; ++u)
            {
                const int r = min(row, n_rows - 1);
                st[u] = min((c_lo + c) / CHUNKS_PER_STEP, 63);
                v[u] = *reinterpret_cast<const u32x4 *>(
                        mbase + (uint32_t)(r * ld_bytes + c * 16));
                row += d_row;
                c += d_c;
                if(c >= n_loc)
                {
                    c -= n_loc;
                    row += 1;
                }
            }
#pragma unroll
            for(int u = 0; u < 16; ++u)
            {
                const uint32_t any1 = v[u][0] | v[u][1] | v[u][2] | v[u][3];
                const uint32_t all1 = v[u][0] & v[u][1] & v[u][2] & v[u][3];
                const bool open = (any1 == open_word) & (all1 == open_word);
                const bool hidden = (any1 == hidden_word) & (all1 == hidden_word);
                not_open |= (unsigned long long)(!open) << st[u];
                not_hidden |= (unsigned long long)(!hidden) << st[u];
            }
        }
    }
    // One LDS atomic per wavefront and word, not one per lane: the range
    // covers few steps, and a ballot per step says whether any lane has its bit.
    {
        const int s_lo = min(c_lo / CHUNKS_PER_STEP, 63);
        const int s_hi = min((c_lo + max(n_loc, 1) - 1) / CHUNKS_PER_STEP, 63);
        unsigned long long w_open = 0ull, w_hidden = 0ull;
        for(int st = s_lo; st <= s_hi; ++st)
        {
            if(__builtin_amdgcn_ballot_w64(((not_open >> st) & 1ull) != 0ull) != 0ull)
            {
                w_open |= 1ull << st;
            }
            if(__builtin_amdgcn_ballot_w64(((not_hidden >> st) & 1ull) != 0ull) != 0ull)
            {
                w_hidden |= 1ull << st;
            }
        }
        if((tid & 63) == 0)
        {
            if(w_open != 0ull)
            {
                atomicOr(&bits[0], w_open);
            }
            if(w_hidden != 0ull)
            {
                atomicOr(&bits[1], w_hidden);
            }
        }
    }
    __syncthreads();
}

template<typename T, int HEAD, int MODE, int WAVES = 4, int GROUPS = 1>
__global__ __launch_bounds__(WAVES * 64, WAVES == 4 ? 2 : 1)
void sdpa_prefill_16bit_kernel(const PrefillParams p)
{
    PF_STAMP(0);
    // GROUPS == 2: the eight wavefronts are two groups of four; both groups
    // hold the same 128 queries, group g takes the key steps g, g + 2, ...
    // through a K/V ring of its own, and the two (maximum, sum, output)
    // triples are merged through LDS before the epilogue.  For launches that
    // have no second workgroup to put on a CU: two wavefronts per SIMD (one's
    // softmax beside the other's MFMAs) and half the chain of dependent steps.
    constexpr int QW = WAVES / GROUPS;      // wavefronts that share a key step
    constexpr int kQRows = QW * 32;
    constexpr int kThreads = WAVES * 64;
    typedef typename T::vec8 vec8;
    constexpr int KSTEPS = HEAD / 16;       // MFMA steps along head for S
    constexpr int DBLOCKS = HEAD / 32;      // 32-row blocks of O^T
    constexpr int RB = HEAD * 2;            // bytes per K/V row
    constexpr int CPR = HEAD / 8;           // 16-byte chunks per row
    constexpr int RPL = 16 / CPR;           // rows per 256-byte line of LDS banks
    constexpr int ROWS_PER_LOAD = 1024 / RB;   // rows one load instruction fills
    constexpr int LOADS = kKeys / ROWS_PER_LOAD;  // load instructions per K (or V) step
    constexpr int LOADS_PER_WAVE = LOADS / QW;
    constexpr int K_BYTES = kKeys * RB;
    constexpr bool EXPLICIT = (MODE == NNTILE_HIP_MASK_ADDITIVE
            || MODE == NNTILE_HIP_MASK_BOOL);
    static_assert(LOADS_PER_WAVE * QW == LOADS
            && (LOADS_PER_WAVE == 1 || LOADS_PER_WAVE == 2 || LOADS_PER_WAVE == 4),
            "head size does not fit this tiling");
    static_assert(GROUPS == 1 || (GROUPS == 2 && WAVES == 8), "two groups of four wavefronts");
    static_assert(WAVES == 4 || (WAVES == 8 && (GROUPS == 2 || !EXPLICIT)),
            "eight wavefronts on 256 queries: analytic masks only");

    // Separate arrays, not one: the compiler then knows that the loads
    // streaming into one of them cannot alias the reads of the others and
    // does not make those reads wait for the loads.  Key step g lives in
    // lds_k[g % 2] and lds_v[g % 2].
    // (GROUPS == 2: group g's half of every array starts at g * K_BYTES; that
    // offset is part of the lanes' read addresses and of the loads' targets)
    __shared__ __attribute__((aligned(1024))) char lds_k0[K_BYTES * GROUPS];
    __shared__ __attribute__((aligned(1024))) char lds_k1[K_BYTES * GROUPS];
    __shared__ __attribute__((aligned(1024))) char lds_v0[K_BYTES * GROUPS];
    __shared__ __attribute__((aligned(1024))) char lds_v1[K_BYTES * GROUPS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int grp = GROUPS > 1 ? (tid >> 6) / QW : 0;      // which key steps
    const int wave = (tid >> 6) - grp * QW;                 // which 32 queries
    const int lds_grp_off = GROUPS > 1 ? __builtin_amdgcn_readfirstlane(grp) * K_BYTES : 0;
    const int col = lane & 31;      // query within the wavefront / row of a block
    const int half = lane >> 5;

    // ---- which queries --------------------------------------------------
    // Workgroups are dealt round-robin to the 8 XCDs.  With xcd_remap every
    // XCD gets a contiguous range of batch entries (their query blocks share
    // K and V in that XCD's L2); in both layouts the query blocks are handed
    // out last-first, all batch entries of a block before the next block, so
    // that under a causal mask the longest workgroups start first.
    //
    // An XCD places its workgroups i = 0..31 on its 32 CUs and i = 32..63
    // beside them, i+32 next to i.  With the plain longest-first order the CU
    // that gets the longest workgroup also gets the longest of the second
    // group, and the CUs end the first round with very different amounts of
    // work done.  The second group is therefore dealt in reverse: the longest
    // workgroup shares its CU with the shortest of the first 64.
    const int q_blocks = p.n_q_tiles * p.q_blocks_per_tile;
    unsigned wg = blockIdx.x;
    if constexpr(EXPLICIT)
    {
        // The first workgroups of the grid scan the mask for everybody (one
        // query tile, one key tile): they wait for nothing, so the attention
        // workgroups behind them can wait for their flags.
        if(p.n_scan_wgs > 0)
        {
            if((int)blockIdx.x < p.n_scan_wgs)
            {
                constexpr int ES = (MODE == NNTILE_HIP_MASK_ADDITIVE) ? 2 : 1;
                __shared__ unsigned long long pub_bits[2];
                mask_scan_range<ES, kThreads>(static_cast<const char *>(p.mask),
                        (int)(p.mask_ld * ES), (int)p.q_seq, (int)(p.k_seq * ES / 16),
                        (MODE == NNTILE_HIP_MASK_ADDITIVE) ? 0u : 0x01010101u,
                        (MODE == NNTILE_HIP_MASK_ADDITIVE) ? T::kNegInfPair : 0u,
                        (int)blockIdx.x / kMaskBitSplits, (int)blockIdx.x % kMaskBitSplits,
                        pub_bits);
                if(tid == 0)
                {
                    // written through to memory (device scope), acknowledged,
                    // then the flag: readers on any XCD find the words
                    unsigned long long *e = p.mask_bits + 3 * (int64_t)blockIdx.x;
                    __hip_atomic_store(e, pub_bits[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(e + 1, pub_bits[1], __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_AGENT);
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __hip_atomic_store(e + 2, p.mask_tag, __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_AGENT);
                }
                return;
            }
            wg -= (unsigned)p.n_scan_wgs;
        }
    }
    if(WAVES == 4 && gridDim.x >= 8u * 2u * kCUsPerXCD)
    {
        const unsigned i = wg >> 3;
        if(i >= kCUsPerXCD && i < 2u * kCUsPerXCD)
        {
            wg = ((3u * kCUsPerXCD - 1u - i) << 3) | (wg & 7u);
        }
    }
    int b, qblk;
    const int batch_all = p.batch * p.n_slabs;
    if(p.xcd_remap)
    {
        const int b_per_xcd = batch_all >> 3;
        const int i = (int)(wg >> 3);
        b = (int)(wg & 7) * b_per_xcd + i % b_per_xcd;
        qblk = q_blocks - 1 - i / b_per_xcd;
    }
    else
    {
        b = (int)wg % batch_all;
        qblk = q_blocks - 1 - (int)wg / batch_all;
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
    const int q_len = (int)min(p.q_tile, p.q_seq - (int64_t)qt * p.q_tile);
    const int q_row0 = qb * kQRows;                     // within the tile
    if(q_row0 >= q_len)
    {
        return;
    }
    const int kvb = kv_entry(b, p.n_batch, p.kv_group);

    const uint16_t *Qt = static_cast<const uint16_t *>(p.Q[q_tile0 + qt])
        + (int64_t)b * q_len * HEAD;
    const int my_q = q_row0 + wave * 32 + col;          // row within tile
    const bool q_ok = my_q < q_len;

    // Q fragments, resident for the whole kernel.
    vec8 qf[KSTEPS];
    {
        const uint16_t *src = Qt + (int64_t)(q_ok ? my_q : 0) * HEAD + half * 8;
#pragma unroll
        for(int ks = 0; ks < KSTEPS; ++ks)
        {
            u32x4 raw = *reinterpret_cast<const u32x4 *>(src + ks * 16);
            if(!q_ok)
            {
                raw = u32x4{0, 0, 0, 0};
            }
            qf[ks] = __builtin_bit_cast(vec8, raw);
        }
    }

    // ---- which keys --------------------------------------------------------
    // rel0: position of the workgroup's first query minus the position of key
    // row 0, plus the causal offset; key row kg is visible to query row
    // (q_row0 + r) iff kg <= rel0 + r.  Clamped so that the 32-bit arithmetic
    // below cannot overflow.
    const int k_seq = (int)p.k_seq, k_tile = (int)p.k_tile;
    int rel0 = 0;
    const int last_k_len = k_seq - (p.n_kv_tiles - 1) * k_tile;
    int n_steps = (p.n_kv_tiles - 1) * p.k_blocks_per_tile
        + (last_k_len + kKeys - 1) / kKeys;
    if(MODE == NNTILE_HIP_MASK_CAUSAL)
    {
        int64_t rel = p.q_pos0 + (int64_t)qt * p.q_tile + q_row0
            + p.causal_offset - p.k_pos0;
        rel = max((int64_t)-(1 << 30), min(rel, (int64_t)(1 << 30)));
        rel0 = (int)rel;
        const int hi = min(rel0 + min(kQRows, q_len - q_row0) - 1, k_seq - 1);
        if(hi < 0)
        {
            if(!p.overwrite)
            {
                return;
            }
            n_steps = 0;    // nothing visible: the epilogue writes empty rows
        }
        else
        {
            const int kt_hi = hi / k_tile;
            n_steps = min(n_steps, kt_hi * p.k_blocks_per_tile
                    + (hi - kt_hi * k_tile) / kKeys + 1);
        }
    }
    const int wave_rel_lo = rel0 + wave * 32;       // first query of the wavefront
    const int my_rel = wave_rel_lo + col;

    // ---- LDS layout and the lane's fixed addresses ---------------------------
    // A step's K (and V) block is kKeys rows of RB bytes, unpadded.  The
    // 16-byte chunk c of row r is stored at chunk position
    //   K:  c ^ ((r / RPL) % CPR)        16 consecutive rows, same c -> 16 bank groups
    //   V:  c ^ (4 * ((r / RPL) % (CPR/4)))   4 consecutive rows x 64 B -> 4 quarters
    // Load instruction `ld` fills rows [ld*ROWS_PER_LOAD, +ROWS_PER_LOAD): lane
    // L lands on row ld*ROWS_PER_LOAD + L/CPR, chunk position L%CPR, and so must
    // fetch the logical chunk that belongs there.
    // (V: the swizzle repeats from one load instruction to the next, so its
    // offsets are v_goff0 + i*1024 and go into the instructions' immediates,
    // which advance the global and the LDS address alike)
    uint32_t k_goff[LOADS_PER_WAVE], v_goff0 = 0;
    int ld_row0 = 0;
    const int ld_cpos = lane % CPR;
#pragma unroll
    for(int i = 0; i < LOADS_PER_WAVE; ++i)
    {
        const int ld = wave * LOADS_PER_WAVE + i;
        const int r = ld * ROWS_PER_LOAD + lane / CPR;
        k_goff[i] = (uint32_t)(r * RB + (ld_cpos ^ ((r / RPL) % CPR)) * 16);
        if(i == 0)
        {
            ld_row0 = r;
            v_goff0 = (uint32_t)(r * RB
                    + (ld_cpos ^ (4 * ((r / RPL) % (CPR >= 4 ? CPR / 4 : 1)))) * 16);
        }
    }
    // S operand: lane (col, half) reads row mb*32+col, logical chunk 2*ks+half.
    uint32_t k_raddr[2][KSTEPS];
#pragma unroll
    for(int mb = 0; mb < 2; ++mb)
    {
        const int r = mb * 32 + col;
#pragma unroll
        for(int ks = 0; ks < KSTEPS; ++ks)
        {
            k_raddr[mb][ks] = (uint32_t)(grp * K_BYTES + r * RB
                    + ((2 * ks + half) ^ ((r / RPL) % CPR)) * 16);
        }
    }
    // PV operand through the transposing read: within a 16-lane block, lane i
    // addresses key j = i/4 and head values 4*(i%4)..+3 of the block's 16 head
    // values, and receives keys 0..3 of head value i.  Blocks: lanes 16..31
    // take the upper 16 head values of a 32-row block, lanes 32..63 the keys
    // 4..7 (lane half h).  For step t (16 keys) and instruction a (keys
    // 8a + 4h + j) the row is 16t + 8a + 4h + j; 16t + 8a goes into the
    // instruction's immediate offset.
    uint32_t v_raddr[DBLOCKS];
    {
        const int i16 = lane & 15, dblk = (lane >> 4) & 1;
        const int j = i16 >> 2, r4 = i16 & 3;
        const int r = 4 * half + j;         // row modulo 8: enough for the swizzle
        const int swz = 4 * ((r / RPL) % (CPR >= 4 ? CPR / 4 : 1));
#pragma unroll
        for(int db = 0; db < DBLOCKS; ++db)
        {
            const int c = 4 * db + 2 * dblk + (r4 >> 1);
            v_raddr[db] = (uint32_t)(grp * K_BYTES + r * RB + (c ^ swz) * 16
                    + 8 * (r4 & 1));
        }
    }

    auto tile_rows = [&](int kt) -> int
    {
        return min(k_tile, k_seq - kt * k_tile);
    };

    // Byte offset of batch entry kvb's slab inside key tile kt.
    auto slab = [&](int kt) -> int64_t
    {
        const int64_t rows = p.kv_rows > 0 ? p.kv_rows : (int64_t)tile_rows(kt);
        return (int64_t)kvb * rows * HEAD * 2;
    };

    // Global -> LDS loads of the K (or V) rows of one step.  Rows past the end
    // of the tile are clamped to its last row: their scores are masked and
    // their probabilities are exactly 0, so any finite stand-in value works.
    auto fetch_k = [&](const StepCursor &cur, char *dst_base)
    {
        // (wave index made visibly uniform: the LDS target goes into M0)
        char *dst = dst_base + lds_grp_off
            + __builtin_amdgcn_readfirstlane(wave) * LOADS_PER_WAVE * 1024;
        if(cur.rows_left >= kKeys)
        {
#pragma unroll
            for(int i = 0; i < LOADS_PER_WAVE; ++i)
            {
                load_to_lds16<0, false>(cur.Kp + k_goff[i], dst + i * 1024);
            }
        }
        else
        {
            const int last = cur.rows_left - 1;
#pragma unroll
            for(int i = 0; i < LOADS_PER_WAVE; ++i)
            {
                // same chunk, clamped row
                const uint32_t back = (uint32_t)(
                        max(ld_row0 + i * ROWS_PER_LOAD - last, 0) * RB);
                load_to_lds16<0, false>(cur.Kp + (k_goff[i] - back), dst + i * 1024);
            }
        }
    };
    auto fetch_v = [&](const StepCursor &cur, char *dst_base)
    {
        char *dst = dst_base + lds_grp_off
            + __builtin_amdgcn_readfirstlane(wave) * LOADS_PER_WAVE * 1024;
        if(cur.rows_left >= kKeys)
        {
            const char *src = cur.Vp + v_goff0;
            load_to_lds16<0, false>(src, dst);
            if(LOADS_PER_WAVE > 1)
            {
                load_to_lds16<1024, false>(src, dst);
            }
            if(LOADS_PER_WAVE > 2)
            {
                load_to_lds16<2048, false>(src, dst);
                load_to_lds16<3072, false>(src, dst);
            }
        }
        else
        {
            const int last = cur.rows_left - 1;
#pragma unroll
            for(int i = 0; i < LOADS_PER_WAVE; ++i)
            {
                const uint32_t back = (uint32_t)(
                        max(ld_row0 + i * ROWS_PER_LOAD - last, 0) * RB);
                load_to_lds16<0, false>(cur.Vp + (v_goff0 + i * 1024 - back), dst + i * 1024);
            }
        }
    };

    // Next step; the tile base pointers are re-read only when the tile changes.
    auto advance_one = [&](StepCursor &cur)
    {
        cur.kb += 1;
        cur.rows_left -= kKeys;
        cur.Kp += kKeys * RB;
        cur.Vp += kKeys * RB;
        if(cur.rows_left <= 0)
        {
            cur.kt += 1;
            cur.kb = 0;
            if(cur.kt < p.n_kv_tiles)
            {
                cur.rows_left = tile_rows(cur.kt);
                cur.Kp = static_cast<const char *>(p.K[k_tile0 + cur.kt]) + slab(cur.kt);
                cur.Vp = static_cast<const char *>(p.V[k_tile0 + cur.kt]) + slab(cur.kt);
            }
            else
            {
                cur.rows_left = 0;
            }
        }
    };
    // ... the next step of this wavefront's group
    auto advance = [&](StepCursor &cur)
    {
        advance_one(cur);
        if(GROUPS > 1)
        {
            advance_one(cur);
        }
    };

    // Score units: the raw dot product is kept and the scale is folded into
    // the exponent; an additive mask value is divided by the scale before it
    // is added, which is the same thing.
    const float c = p.scale * kLog2e;
    const float inv_scale = 1.0f / p.scale;

    // ---- explicit mask tiles ----------------------------------------------------
    // The lane's 32 mask values of a key step (query my_q, keys
    // mb*32 + 8*rg + 4*half + 0..3) are 8 groups of 4 consecutive elements:
    // one 8-byte (additive) or 4-byte (boolean) load per group, issued one
    // step ahead.  At the top of a step the wavefront classifies its 32 x 64
    // block from the raw bits: nothing hidden (the step runs as if there were
    // no mask), everything hidden (the step is skipped), or mixed (the values
    // are applied).  Ragged steps and masks that are not aligned for the wide
    // loads take the element-wise path.
    constexpr int MW = (MODE == NNTILE_HIP_MASK_ADDITIVE) ? 16 : 8;    // dwords per lane and step
    enum { MASK_ZERO = 0, MASK_HIDDEN = 1, MASK_MIXED = 2, MASK_SLOW = 3 };
    uint32_t mraw[MW];
#pragma unroll
    for(int i = 0; i < MW; ++i)
    {
        mraw[i] = 0;
    }
    const int64_t mask_row = (int64_t)(q_ok ? my_q : 0) * p.mask_ld;
    // (every full step of any mask: the wide loads below carry the alignment
    // of one element, and global memory takes unaligned accesses - a row
    // length that is not a multiple of 4 costs some loads a second cache
    // line, not a load per element)
    const bool mask_wide = EXPLICIT;
    // loads of the mask values of key step kb (a full step) into mraw
    auto mask_fetch = [&](int kb)
    {
        if(MODE == NNTILE_HIP_MASK_ADDITIVE)
        {
            typedef u32x2 __attribute__((aligned(2))) u32x2_any;
            const uint16_t *mp = static_cast<const uint16_t *>(p.mask) + mask_row
                + kb * kKeys + 4 * half;
#pragma unroll
            for(int i = 0; i < 8; ++i)
            {
                const u32x2 v = *reinterpret_cast<const u32x2_any *>(
                        mp + (i >> 2) * 32 + (i & 3) * 8);
                mraw[2 * i] = v[0];
                mraw[2 * i + 1] = v[1];
            }
        }
        else if(MODE == NNTILE_HIP_MASK_BOOL)
        {
            typedef uint32_t __attribute__((aligned(1))) u32_any;
            const uint8_t *mp = static_cast<const uint8_t *>(p.mask) + mask_row
                + kb * kKeys + 4 * half;
#pragma unroll
            for(int i = 0; i < 8; ++i)
            {
                mraw[i] = *reinterpret_cast<const u32_any *>(
                        mp + (i >> 2) * 32 + (i & 3) * 8);
            }
        }
    };
    auto mask_classify = [&]() -> int
    {
        uint32_t all_or = 0u, all_and = 0xffffffffu;
#pragma unroll
        for(int i = 0; i < MW; ++i)
        {
            all_or |= mraw[i];
            all_and &= mraw[i];
        }
        bool lane_open, lane_hidden;
        if(MODE == NNTILE_HIP_MASK_ADDITIVE)
        {
            lane_open = (all_or == 0u);                 // every value is +0
            lane_hidden = (all_or == T::kNegInfPair) && (all_and == T::kNegInfPair);
        }
        else
        {
            lane_open = (all_or == 0x01010101u) && (all_and == 0x01010101u);
            lane_hidden = (all_or == 0u);
        }
        if(__builtin_amdgcn_ballot_w64(!lane_open) == 0)
        {
            return MASK_ZERO;
        }
        if(__builtin_amdgcn_ballot_w64(!lane_hidden) == 0)
        {
            return MASK_HIDDEN;
        }
        return MASK_MIXED;
    };

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
    float l_run = 0.0f;      // this lane half's share of the row sum

    PHASE_DECL
    StepCursor cur = {0, 0, tile_rows(0),
        static_cast<const char *>(p.K[k_tile0]) + slab(0),
        static_cast<const char *>(p.V[k_tile0]) + slab(0)};     // step being computed
    if(GROUPS > 1 && grp == 1)
    {
        advance_one(cur);       // the second group starts at step 1
    }
    StepCursor nxt = cur;                        // step being fetched
    // Masks given as values: the first step's K and V are requested before the
    // mask is looked at (below: a wait for the scanning workgroups' flags, or a
    // scan of this workgroup's own rows).  What the mask then says may make
    // the step unnecessary, which costs nothing but the request.
    bool first_requested = false;
    if(EXPLICIT)
    {
        const int own = GROUPS > 1 ? max(n_steps - grp + GROUPS - 1, 0) / GROUPS : n_steps;
        if(own > 0)
        {
            fetch_k(nxt, lds_k0);
            fetch_v(nxt, lds_v0);
            first_requested = true;
        }
    }
    // Explicit masks: number of leading key steps in which the mask changes
    // nothing for any query of the workgroup (they run in the pipelined loop).
    int n_open = 0;
    if(EXPLICIT)
    {
        // The workgroup's rows of the mask are scanned once, 16 bytes per
        // thread and load, 16 loads in flight, beside the first step's loads.
        // Per key step the scan records whether every value is "open" (+0 /
        // true) and whether every value is "hidden" (-inf / false).  Hidden
        // steps at the end are dropped - a tile pair above the diagonal of a
        // causal mask given as values costs this scan instead of a pass over K
        // and V - and the open steps at the start need no mask handling.
        constexpr int ES = (MODE == NNTILE_HIP_MASK_ADDITIVE) ? 2 : 1;
        constexpr int CHUNKS_PER_STEP = kKeys * ES / 16;
        constexpr uint32_t OPEN = (MODE == NNTILE_HIP_MASK_ADDITIVE) ? 0u : 0x01010101u;
        constexpr uint32_t HIDDEN = (MODE == NNTILE_HIP_MASK_ADDITIVE) ? T::kNegInfPair : 0u;
        const int64_t row_bytes = (int64_t)k_seq * ES;
        // bit s: some value of step s (steps >= 63 share bit 63) is not open / not hidden
        unsigned long long not_open = 0ull, not_hidden = 0ull;
        bool scanned = false;
        if(n_steps > 0 && p.mask_bits != nullptr && p.n_scan_wgs == 0)
        {
            // the scan was done once for all batch entries before the launch
            const unsigned long long *w = p.mask_bits + (int64_t)qb * (3 * kMaskBitSplits);
#pragma unroll
            for(int sp = 0; sp < kMaskBitSplits; ++sp)
            {
                not_open |= w[3 * sp];
                not_hidden |= w[3 * sp + 1];
            }
            scanned = true;
        }
        else if(n_steps > 0 && p.mask_bits != nullptr)
        {
            // ... or is being done by the first workgroups of this launch: one
            // thread per key range waits for that range's flag (bounded; the
            // Q fragments are on their way meanwhile), then everybody ORs
            __shared__ unsigned long long got_bits[2];
            __shared__ int got_all;
            if(tid == 0)
            {
                got_bits[0] = 0ull;
                got_bits[1] = 0ull;
                got_all = 1;
            }
            __syncthreads();
            if(tid < kMaskBitSplits)
            {
                unsigned long long *e = p.mask_bits
                    + 3 * ((int64_t)qb * kMaskBitSplits + tid);
                const unsigned long long t0 = wall_clock64();
                bool ok = true;
                while(__hip_atomic_load(e + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                        != p.mask_tag)
                {
                    __builtin_amdgcn_s_sleep(2);
                    if(wall_clock64() - t0 > p.mask_spin_limit)
                    {
                        ok = false;
                        break;
                    }
                }
                if(ok)
                {
                    atomicOr(&got_bits[0], __hip_atomic_load(e, __ATOMIC_RELAXED,
                                __HIP_MEMORY_SCOPE_AGENT));
                    atomicOr(&got_bits[1], __hip_atomic_load(e + 1, __ATOMIC_RELAXED,
                                __HIP_MEMORY_SCOPE_AGENT));
                }
                else
                {
                    got_all = 0;
                }
            }
            __syncthreads();
            if(got_all)
            {
                not_open = got_bits[0];
                not_hidden = got_bits[1];
                scanned = true;
            }
        }
        // (rows whose length or start is not a multiple of 16 bytes are not
        // scanned: with loads at the alignment of one element the scan cost
        // what it saved - 49.6 against 48.1 us on 32 x 1001 x 128)
        if(!scanned && n_steps > 0 && row_bytes % 16 == 0 && (p.mask_ld * ES) % 16 == 0
                && reinterpret_cast<uintptr_t>(p.mask) % 16 == 0
                && p.mask_ld * ES * kQRows < (int64_t)(1 << 30))
        {
            __shared__ unsigned long long scan_bits[2];
            if(tid == 0)
            {
                scan_bits[0] = 0ull;
                scan_bits[1] = 0ull;
            }
            __syncthreads();
            const int n_chunks = (int)(row_bytes / 16);
            const int n_rows = min(kQRows, q_len - q_row0);
            const int total = n_rows * n_chunks;
            const char *mbase = static_cast<const char *>(p.mask)
                + (int64_t)q_row0 * p.mask_ld * ES;
            // chunk tid, tid + 256, ... of the rows laid end to end: (row, c)
            // advances by 256 chunks per load without a division
            const int d_row = kThreads / n_chunks, d_c = kThreads % n_chunks;
            const int ld_bytes = (int)(p.mask_ld * ES);     // fits: checked above
            int row = tid / n_chunks, c = tid % n_chunks;
            for(int base = 0; base < total; base += 16 * kThreads)
            {
                // (rows past the end re-read the last row: no branches, so
                // that the 16 loads are in flight together)
                u32x4 v[16];
                int st[16];
#pragma unroll
                for(int u = 0; u < 16; ++u)
                {
                    const int r = min(row, n_rows - 1);
                    st[u] = min(c / CHUNKS_PER_STEP, 63);
                    v[u] = *reinterpret_cast<const u32x4 *>(
                            mbase + (uint32_t)(r * ld_bytes + c * 16));
                    row += d_row;
                    c += d_c;
                    if(c >= n_chunks)
                    {
                        c -= n_chunks;
                        row += 1;
                    }
                }
#pragma unroll
                for(int u = 0; u < 16; ++u)
                {
                    const uint32_t any1 = v[u][0] | v[u][1] | v[u][2] | v[u][3];
                    const uint32_t all1 = v[u][0] & v[u][1] & v[u][2] & v[u][3];
                    const bool open = (any1 == OPEN) & (all1 == OPEN);
                    const bool hidden = (any1 == HIDDEN) & (all1 == HIDDEN);
                    not_open |= (unsigned long long)(!open) << st[u];
                    not_hidden |= (unsigned long long)(!hidden) << st[u];
                }
            }
            if(not_open != 0ull)
            {
                atomicOr(&scan_bits[0], not_open);
            }
            if(not_hidden != 0ull)
            {
                atomicOr(&scan_bits[1], not_hidden);
            }
            __syncthreads();
            not_open = scan_bits[0];
            not_hidden = scan_bits[1];
            scanned = true;
        }
        if(scanned)
        {
            if(not_hidden == 0ull)
            {
                if(!p.overwrite)
                {
                    // (the first step's loads may be on their way into LDS)
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    return;
                }
                n_steps = 0;    // the epilogue writes empty rows
            }
            else if((not_hidden >> 63) == 0ull)
            {
                n_steps = min(n_steps, 64 - __builtin_clzll(not_hidden));
            }
            n_open = not_open == 0ull ? 63 : min(__builtin_ctzll(not_open), 63);
        }
    }
    // Leading steps that are complete (64 keys) and visible to every query of
    // the workgroup need no mask at all; they run in the pipelined loop below.
    int n_fast = 0;
    int n_spread = 0;       // leading steps that exist and are complete
    {
        const int n_full = (p.n_kv_tiles == 1 || k_tile % kKeys == 0)
            ? k_seq / kKeys : k_tile / kKeys;
        n_fast = min(n_steps, n_full);
        n_spread = n_fast;
        if(MODE == NNTILE_HIP_MASK_CAUSAL)
        {
            n_fast = min(n_fast, max(rel0 + 1, 0) / kKeys);
        }
        if(EXPLICIT)
        {
            n_fast = min(n_fast, n_open);
        }
        if(GROUPS > 1)
        {
            // counted in the group's own steps (its step j is step
            // GROUPS * j + grp), and the same for both groups: the barriers of
            // the pipelined loop are the workgroup's
            n_fast /= GROUPS;
            n_spread /= GROUPS;
        }
        n_fast = n_fast >= 2 ? n_fast : 0;
    }
    // Rounds of the workgroup; from here on n_steps counts the group's own
    // steps.  A group that has one step fewer than the other goes through the
    // last round idle: every wavefront meets every barrier.
    const int n_rounds = (n_steps + GROUPS - 1) / GROUPS;
    if(GROUPS > 1)
    {
        n_steps = max(n_steps - grp + GROUPS - 1, 0) / GROUPS;
    }
    if(n_steps > 0)
    {
        if(!first_requested)
        {
            fetch_k(nxt, lds_k0);
            fetch_v(nxt, lds_v0);
        }
        advance(nxt);
        if(n_fast > 0)
        {
            fetch_k(nxt, lds_k1);       // the pipelined loop keeps K two steps ahead
        }
        if(mask_wide && n_fast == 0 && cur.rows_left >= kKeys)
        {
            mask_fetch(cur.kb);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    PF_STAMP(1);
#ifdef NNTILE_PF_TRACE
    const unsigned long long pf_cycles0 = clock64();
#endif
    PF_NOTE(5, ((unsigned long long)__builtin_amdgcn_s_getreg(63508) << 32)
            | (unsigned)__builtin_amdgcn_s_getreg(63492));
    PF_NOTE(6, ((unsigned long long)(unsigned)n_steps << 32) | (unsigned)(b * 1024 + qblk));

    // One key step on LDS buffer BUF (a compile-time constant, so that every
    // LDS address is a fixed register plus an immediate).
    auto step = [&](int g, auto buf_tag) __attribute__((always_inline))
    {
        constexpr int BUF = decltype(buf_tag)::value;
        const char *Ks = BUF ? lds_k1 : lds_k0;
        const char *Vs = BUF ? lds_v1 : lds_v0;
        const int k_row0 = cur.kb * kKeys;                   // within the tile
        const int kg0 = cur.kt * k_tile + k_row0;            // key row overall
        const int keys_here = min(kKeys, cur.rows_left);
        // explicit mask: what this wavefront's block of the mask looks like
        // (the values were loaded during the previous step)
        int mask_class = MASK_SLOW;
        if(EXPLICIT && mask_wide && keys_here == kKeys)
        {
            mask_class = mask_classify();
        }
        // nothing of this step is visible to this wavefront, or the step is
        // the other group's last one and this group has none in this round
        const bool idle = (GROUPS > 1 && g >= n_steps)
            || (EXPLICIT ? (mask_class == MASK_HIDDEN)
            : ((MODE == NNTILE_HIP_MASK_CAUSAL) && (kg0 > wave_rel_lo + 31)));

        // ---- loads of the next step into the other buffer ----------------------
        // (every wavefront passed the barrier that ended step g-1, so nobody
        // still reads that buffer)
        NNTILE_PHASE(0)
        if(g + 1 < n_steps)
        {
            fetch_k(nxt, BUF ? lds_k0 : lds_k1);
            fetch_v(nxt, BUF ? lds_v0 : lds_v1);
            advance(nxt);
        }

        uint32_t pk[2][8];
        if(!idle)
        {
            // ---- S^T = K Q^T -------------------------------------------------
            f32x16 s[2];
#pragma unroll
            for(int mb = 0; mb < 2; ++mb)
            {
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    s[mb][r] = 0.0f;
                }
#pragma unroll
                for(int ks = 0; ks < KSTEPS; ++ks)
                {
                    const vec8 a = *reinterpret_cast<const vec8 *>(
                            Ks + k_raddr[mb][ks]);
                    s[mb] = T::mfma(a, qf[ks], s[mb]);
                }
            }
            NNTILE_PHASE(1)

            // ---- mask ---------------------------------------------------------
            // register r of block mb holds key  mb*32 + 8*(r/4) + 4*half + r%4
            if(EXPLICIT)
            {
                if(mask_class == MASK_MIXED)
                {
#pragma unroll
                    for(int i = 0; i < 8; ++i)
                    {
                        // group i: block i/4, registers 4*(i%4) .. +3
                        const int mb = i >> 2, r0 = 4 * (i & 3);
                        if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                        {
#pragma unroll
                            for(int e = 0; e < 4; ++e)
                            {
                                const uint32_t w = mraw[2 * i + (e >> 1)];
                                const float add = T::to_float((uint16_t)(
                                            (e & 1) ? (w >> 16) : (w & 0xffffu)));
                                s[mb][r0 + e] = fmaf(add, inv_scale, s[mb][r0 + e]);
                            }
                        }
                        else
                        {
#pragma unroll
                            for(int e = 0; e < 4; ++e)
                            {
                                if(((mraw[i] >> (8 * e)) & 0xffu) == 0u)
                                {
                                    s[mb][r0 + e] = neg_inf();
                                }
                            }
                        }
                    }
                }
                else if(mask_class == MASK_SLOW)
                {
#pragma unroll
                    for(int mb = 0; mb < 2; ++mb)
                    {
#pragma unroll
                        for(int rg = 0; rg < 4; ++rg)
                        {
                            const int key0 = mb * 32 + 8 * rg + 4 * half;
#pragma unroll
                            for(int e = 0; e < 4; ++e)
                            {
                                // out-of-range keys of a ragged step are hidden;
                                // their loads are clamped to the step's last key
                                // instead of being branched around, so that the
                                // 32 loads of a lane are independent and overlap
                                const int64_t at = mask_row + k_row0
                                    + max(min(key0 + e, keys_here - 1), 0);
                                float add;
                                if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                                {
                                    add = T::to_float(static_cast<const uint16_t *>(
                                                p.mask)[at]);
                                }
                                else
                                {
                                    add = static_cast<const uint8_t *>(
                                            p.mask)[at] != 0
                                        ? 0.0f : neg_inf();
                                }
                                if(key0 + e >= keys_here)
                                {
                                    add = neg_inf();
                                }
                                s[mb][4 * rg + e] = fmaf(add, inv_scale,
                                        s[mb][4 * rg + e]);
                            }
                        }
                    }
                }
            }
            else
            {
                const bool ragged = keys_here < kKeys;
                const bool diagonal = (MODE == NNTILE_HIP_MASK_CAUSAL)
                    && (kg0 + kKeys - 1 > wave_rel_lo);
                if(ragged || diagonal)
                {
                    // last visible key of this step for this lane's query
                    int lim = keys_here - 1;
                    if(MODE == NNTILE_HIP_MASK_CAUSAL)
                    {
                        lim = min(lim, my_rel - kg0);
                    }
#pragma unroll
                    for(int mb = 0; mb < 2; ++mb)
                    {
#pragma unroll
                        for(int r = 0; r < 16; ++r)
                        {
                            const int key = mb * 32 + 8 * (r >> 2) + 4 * half
                                + (r & 3);
                            if(key > lim)
                            {
                                s[mb][r] = neg_inf();
                            }
                        }
                    }
                }
            }

            // ---- online softmax -------------------------------------------------
            float mx = neg_inf();
#pragma unroll
            for(int mb = 0; mb < 2; ++mb)
            {
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    mx = fmaxf(mx, s[mb][r]);
                }
            }
            mx = max_across_halves(mx);
            const float m_new = fmaxf(m_run, mx);
            const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
            const float mc = m_use * c;
            // The running maximum rarely moves after the first steps; the
            // rescale of the 16*DBLOCKS output registers is skipped unless
            // some query of the wavefront needs it.
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

            // row sums by plain additions (the dot-product instruction that
            // would sum a packed pair waits for the matrix unit)
            float rs0 = 0.0f, rs1 = 0.0f;
#pragma unroll
            for(int mb = 0; mb < 2; ++mb)
            {
#pragma unroll
                for(int r = 0; r < 16; r += 2)
                {
                    const float p0 = fast_exp2(fmaf(s[mb][r], c, -mc));
                    const float p1 = fast_exp2(fmaf(s[mb][r + 1], c, -mc));
                    pk[mb][r >> 1] = T::pack2(p0, p1);
                    rs0 += p0;
                    rs1 += p1;
                }
            }
            l_run += rs0 + rs1;
        }
        // mask values of the next step (this step's have been consumed)
        if(EXPLICIT && mask_wide && g + 1 < n_steps
                && cur.rows_left - GROUPS * kKeys >= kKeys)
        {
            mask_fetch(cur.kb + GROUPS);
        }
        NNTILE_PHASE(2)

        // ---- O^T += V^T P^T ------------------------------------------------------
        if(!idle)
        {
#pragma unroll
            for(int t = 0; t < 4; ++t)
            {
                const int mb = t >> 1, tt = t & 1;
                const u32x4 praw = {pk[mb][4 * tt], pk[mb][4 * tt + 1],
                    pk[mb][4 * tt + 2], pk[mb][4 * tt + 3]};
                const vec8 pb = __builtin_bit_cast(vec8, praw);
#pragma unroll
                for(int db = 0; db < DBLOCKS; ++db)
                {
                    const char *src = Vs + v_raddr[db] + (16 * t) * RB;
                    const u32x2 lo = lds_read_tr16(src);
                    const u32x2 hi = lds_read_tr16(src + 8 * RB);
                    const u32x4 araw = {lo[0], lo[1], hi[0], hi[1]};
                    const vec8 a = __builtin_bit_cast(vec8, araw);
                    o[db] = T::mfma(a, pb, o[db]);
                }
            }
        }
        advance(cur);
        NNTILE_PHASE(3)
        // this wavefront's loads of the next step have landed in LDS
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        NNTILE_PHASE(4)
    };

    // ---- pipelined loop over the unmasked steps ---------------------------------
    // A step is two sub-blocks of 32 keys.  While the softmax of sub-block j
    // runs on the vector ALU, the matrix unit computes the scores of sub-block
    // j+1 and adds sub-block j-1 to the output: the three are independent, and
    // a wavefront's MFMAs execute in the background of its own VALU work.  One
    // MFMA and a slice of the softmax form a slot; scheduling barriers keep the
    // compiler from regrouping the slots.  K is fetched two steps ahead and V
    // one step ahead, with one workgroup barrier in the middle of each step.
    int g_first = 0;        // first step of the general loop
    if(n_fast > 0)
    {
        constexpr int NSLOT = 2 * KSTEPS;       // KSTEPS score MFMAs + 2*DBLOCKS output MFMAs
        constexpr int NITEM = 24;               // softmax work items of a sub-block
        constexpr float kLazyLimit = 16384.0f;  // largest row sum of a sub-block taken without a new maximum
        constexpr int AHEAD = NNTILE_PF_AHEAD;  // LDS operands are read this many slots early
        f32x16 zero16;
#pragma unroll
        for(int r = 0; r < 16; ++r)
        {
            zero16[r] = 0.0f;
        }
        f32x16 sa = zero16, sb = zero16;        // scores of the current / next sub-block
        uint32_t pp[8];                         // probabilities (packed pairs) of a sub-block
#pragma unroll
        for(int i = 0; i < 8; ++i)
        {
            pp[i] = 0u;
        }
        float alpha_pending = 1.0f;             // rescale of O that the last softmax asked for
        bool rescale_pending = false;           // ... if it asked for one (the same for the whole wavefront)
        StepCursor c1 = nxt;                    // step g+1: its V is fetched during step g
        StepCursor c2 = nxt;                    // step g+2: its K is fetched during step g
        advance(c2);

        // MFMA of slot sl.  Order: first the score MFMAs (one accumulator
        // chain, which costs nothing extra), then the output MFMAs: the scores
        // are complete half a body before the next body's softmax needs them.
        //   kind 0: output MFMA number idx (16-key half idx / DBLOCKS, block idx % DBLOCKS)
        //   kind 1: score MFMA number idx (head values 16*idx .. +15)
        auto slot_kind = [](int sl) -> int
        {
            return sl < KSTEPS ? 1 : 0;
        };
        auto slot_idx = [](int sl) -> int
        {
            return sl < KSTEPS ? sl : sl - KSTEPS;
        };

        // One sub-block body.  s_cur: scores to turn into probabilities;
        // s_nxt: scores to compute from the 32 keys of block kh of buffer Kb;
        // the probabilities in pp multiply the keys 32*vh.. of buffer Vb.
        // With DO_FETCH the loads of K(c2) into kdst and V(c1) into vdst (both
        // full steps) are issued one every second slot: issued together after
        // the barrier they queue up behind each other - the loads of a step
        // take the CU's memory path about 500 cycles - and the wavefront
        // stands still until its last one is accepted.
        auto body = [&](auto do_s_tag, auto do_pv_tag, auto do_sm_tag, auto do_fetch_tag,
                const char *Kb, int kh, const char *Vb, int vh, const f32x16 &s_cur,
                f32x16 &s_nxt, char *kdst, char *vdst)
            __attribute__((always_inline))
        {
            constexpr bool DO_S = decltype(do_s_tag)::value;
            constexpr bool DO_PV = decltype(do_pv_tag)::value;
            constexpr bool DO_SM = decltype(do_sm_tag)::value;
            constexpr bool DO_FETCH = decltype(do_fetch_tag)::value;
            static_assert(2 * LOADS_PER_WAVE <= NSLOT / 2, "one load every second slot");
            auto fetch_piece = [&](int i) __attribute__((always_inline))
            {
                if(i < LOADS_PER_WAVE)
                {
                    load_to_lds16<0, false>(c2.Kp, k_goff[i], kdst + i * 1024);
                }
                else if(i < 2 * LOADS_PER_WAVE)
                {
                    switch(i - LOADS_PER_WAVE)
                    {
                        case 0: load_to_lds16<0, false>(c1.Vp, v_goff0, vdst); break;
                        case 1: load_to_lds16<1024, false>(c1.Vp, v_goff0, vdst); break;
                        case 2: load_to_lds16<2048, false>(c1.Vp, v_goff0, vdst); break;
                        default: load_to_lds16<3072, false>(c1.Vp, v_goff0, vdst); break;
                    }
                }
            };
            // the rescale that the previous softmax decided on (rare after the
            // first steps): O holds every sub-block up to j-2 at this point
            if(rescale_pending)
            {
#pragma unroll
                for(int db = 0; db < DBLOCKS; ++db)
                {
#pragma unroll
                    for(int r = 0; r < 16; ++r)
                    {
                        o[db][r] *= alpha_pending;
                    }
                }
            }
            vec8 opnd[NSLOT];       // LDS operand of each slot's MFMA
            // the probabilities of sub-block j-1, as they are on entry: pp is
            // rewritten with those of sub-block j while the output MFMAs run
            uint32_t pin[8];
#pragma unroll
            for(int i = 0; i < 8; ++i)
            {
                pin[i] = pp[i];
            }
            auto read_operand = [&](int sl) __attribute__((always_inline))
            {
                if(sl >= NSLOT)
                {
                    return;
                }
                const int i = slot_idx(sl);
                if(slot_kind(sl) == 1)
                {
                    if(DO_S)
                    {
                        opnd[sl] = *reinterpret_cast<const vec8 *>(Kb + k_raddr[0][i]
                                + kh * 32 * RB);
                    }
                }
                else if(DO_PV)
                {
                    const int t = 2 * vh + i / DBLOCKS, db = i % DBLOCKS;
                    const char *src = Vb + v_raddr[db] + (16 * t) * RB;
                    const u32x2 lo = lds_read_tr16(src);
                    const u32x2 hi = lds_read_tr16(src + 8 * RB);
                    const u32x4 raw = {lo[0], lo[1], hi[0], hi[1]};
                    opnd[sl] = __builtin_bit_cast(vec8, raw);
                }
            };
            // Lazy maximum: the probabilities are taken relative to the running
            // maximum as it stands, without looking at this sub-block's scores
            // first (softmax does not depend on the reference point, only
            // overflow does).  The row sums, which are needed anyway, tell
            // afterwards whether that was safe; if not (first sub-block, or
            // scores far above everything seen so far) the sub-block is redone
            // with a new maximum at the end of the body.
            const float mc = m_run * c;
            float rs = 0.0f;
            float pe[2] = {0.0f, 0.0f};
            auto item = [&](int it) __attribute__((always_inline))
            {
                const int k = it / 3, r = it % 3;
                if(r < 2)
                {
                    pe[r] = fast_exp2(fmaf(s_cur[2 * k + r], c, -mc));
                }
                else
                {
                    // (plain additions: the dot-product instruction that sums a
                    // packed pair waits for the matrix unit, 15 cycles each)
                    rs += pe[0];
                    rs += pe[1];
                    pp[k] = T::pack2(pe[0], pe[1]);
                    // (keeps the conversion in this slot)
                    asm volatile("" : "+v"(pp[k]));
                }
            };
#pragma unroll
            for(int sl = 0; sl < AHEAD; ++sl)
            {
                read_operand(sl);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for(int sl = 0; sl < NSLOT; ++sl)
            {
                read_operand(sl + AHEAD);
                const int i = slot_idx(sl);
                if(slot_kind(sl) == 1)
                {
                    if(DO_S)
                    {
                        s_nxt = T::mfma(opnd[sl], qf[i], i == 0 ? zero16 : s_nxt);
                    }
                }
                else if(DO_PV)
                {
                    const int t = i / DBLOCKS, db = i % DBLOCKS;
                    const u32x4 praw = {pin[4 * t], pin[4 * t + 1], pin[4 * t + 2],
                        pin[4 * t + 3]};
                    o[db] = T::mfma(opnd[sl], __builtin_bit_cast(vec8, praw), o[db]);
                }
                // the softmax items are spread over the slots 1 .. NSLOT-1
                if(DO_SM && sl >= 1)
                {
#pragma unroll
                    for(int it = (sl - 1) * NITEM / (NSLOT - 1);
                            it < sl * NITEM / (NSLOT - 1); ++it)
                    {
                        item(it);
                    }
                }
                if(DO_FETCH && (sl & 1))
                {
                    fetch_piece(sl >> 1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            rescale_pending = false;
            if(DO_SM)
            {
                if(__builtin_amdgcn_ballot_w64(!(rs <= kLazyLimit)) != 0)
                {
                    float mx = s_cur[0];
#pragma unroll
                    for(int r = 1; r < 16; ++r)
                    {
                        mx = fmaxf(mx, s_cur[r]);
                    }
                    // every key of these steps is visible: the new maximum is finite
                    const float m_new = max_with_other_half(m_run, mx);
                    const float alpha = fast_exp2((m_run - m_new) * c);
                    const float mc_new = m_new * c;
                    rs = 0.0f;
#pragma unroll
                    for(int k = 0; k < 8; ++k)
                    {
                        const float p0 = fast_exp2(fmaf(s_cur[2 * k], c, -mc_new));
                        const float p1 = fast_exp2(fmaf(s_cur[2 * k + 1], c, -mc_new));
                        pp[k] = T::pack2(p0, p1);
                        rs += p0;
                        rs += p1;
                    }
                    l_run *= alpha;
                    m_run = m_new;
                    alpha_pending = alpha;
                    rescale_pending = true;
                }
                l_run += rs;
            }
            // Everything above belongs to this body: without this the compiler
            // sinks the tail of the softmax, whose results are first used by
            // the next body, behind that body's rescale branch and out of the
            // shadow of the MFMAs.
            asm volatile("" : "+v"(pp[0]), "+v"(pp[1]), "+v"(pp[2]), "+v"(pp[3]),
                    "+v"(pp[4]), "+v"(pp[5]), "+v"(pp[6]), "+v"(pp[7]),
                    "+v"(l_run), "+v"(m_run));
            if(DO_S)
            {
                asm volatile("" : "+v"(s_nxt));
            }
        };
        typedef std::integral_constant<bool, true> Yes;
        typedef std::integral_constant<bool, false> No;

        // scores of sub-block (0, 0)
#pragma unroll
        for(int ks = 0; ks < KSTEPS; ++ks)
        {
            const vec8 a = *reinterpret_cast<const vec8 *>(lds_k0 + k_raddr[0][ks]);
            sa = T::mfma(a, qf[ks], ks == 0 ? zero16 : sa);
        }

        // The middle of step g on the buffers of parity BUF: K(g+1) and V(g)
        // have landed for everyone (they were requested a step ago) and nobody
        // reads K(g) or V(g-1) any more, so their buffers take K(g+2), V(g+1).
        auto mid_step = [&](int g, auto buf_tag) __attribute__((always_inline))
        {
            constexpr int BUF = decltype(buf_tag)::value;
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if(g + 2 < n_steps)
            {
                fetch_k(c2, BUF ? lds_k1 : lds_k0);
            }
            if(g + 1 < n_steps)
            {
                fetch_v(c1, BUF ? lds_v0 : lds_v1);
            }
            c1 = c2;
            advance(c2);
        };
        char *const no_dst = nullptr;
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        // One step on the buffers of parity BUF: sub-block (g, 0) with the
        // scores of (g, 1) and the output of (g-1, 1), then sub-block (g, 1)
        // with the scores of (g+1, 0) and the output of (g, 0).  (After the
        // last pipelined step the scores computed ahead are not used.)
        // spread_tag: steps g+1 and g+2 exist and are complete, and their
        // loads go into the slots of the second sub-block.
        auto fast_step = [&](int g, auto buf_tag, auto spread_tag) __attribute__((always_inline))
        {
            constexpr int BUF = decltype(buf_tag)::value;
            body(Yes{}, Yes{}, Yes{}, No{}, BUF ? lds_k1 : lds_k0, 1, BUF ? lds_v0 : lds_v1, 1,
                    sa, sb, no_dst, no_dst);
            if(decltype(spread_tag)::value)
            {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                char *kdst = (BUF ? lds_k1 : lds_k0) + lds_grp_off + wave_u * LOADS_PER_WAVE * 1024;
                char *vdst = (BUF ? lds_v0 : lds_v1) + lds_grp_off + wave_u * LOADS_PER_WAVE * 1024;
                body(Yes{}, Yes{}, Yes{}, Yes{}, BUF ? lds_k0 : lds_k1, 0,
                        BUF ? lds_v1 : lds_v0, 0, sb, sa, kdst, vdst);
                c1 = c2;
                advance(c2);
            }
            else
            {
                mid_step(g, buf_tag);
                body(Yes{}, Yes{}, Yes{}, No{}, BUF ? lds_k0 : lds_k1, 0,
                        BUF ? lds_v1 : lds_v0, 0, sb, sa, no_dst, no_dst);
            }
            advance(cur);
        };
        // step 0: there is no output yet in its first half
        body(Yes{}, No{}, Yes{}, No{}, lds_k0, 1, lds_v1, 1, sa, sb, no_dst, no_dst);
        mid_step(0, std::integral_constant<int, 0>{});
        body(Yes{}, Yes{}, Yes{}, No{}, lds_k1, 0, lds_v0, 0, sb, sa, no_dst, no_dst);
        advance(cur);
        int g = 1;
        for(; g + 1 < n_fast && g + 3 < n_spread; g += 2)
        {
            fast_step(g, std::integral_constant<int, 1>{}, Yes{});
            fast_step(g + 1, std::integral_constant<int, 0>{}, Yes{});
        }
        // the last steps, whose successors may be incomplete or absent
        for(; g < n_fast; g += 2)
        {
            fast_step(g, std::integral_constant<int, 1>{}, No{});
            if(g + 1 < n_fast)
            {
                fast_step(g + 1, std::integral_constant<int, 0>{}, No{});
            }
        }
        // drain: the output of the last sub-block
        if((n_fast - 1) & 1)
        {
            body(No{}, Yes{}, No{}, No{}, lds_k0, 0, lds_v1, 1, sb, sa, no_dst, no_dst);
        }
        else
        {
            body(No{}, Yes{}, No{}, No{}, lds_k0, 0, lds_v0, 1, sb, sa, no_dst, no_dst);
        }
        g_first = n_fast;
        nxt = c1;
        if(EXPLICIT && mask_wide && g_first < n_steps && cur.rows_left >= kKeys)
        {
            mask_fetch(cur.kb);     // the general step finds its mask values loaded
        }
        // the general loop expects step g_first complete in its buffers
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    PF_STAMP(2);
    {
        int g = g_first;
        if(g < n_rounds && (g & 1))
        {
            step(g, std::integral_constant<int, 1>{});
            g += 1;
        }
        for(; g < n_rounds; g += 2)
        {
            step(g, std::integral_constant<int, 0>{});
            if(g + 1 < n_rounds)
            {
                step(g + 1, std::integral_constant<int, 1>{});
            }
        }
    }
    NNTILE_PHASE_DUMP()
    PF_STAMP(3);
    PF_NOTE(7, clock64() - pf_cycles0);     // shader-clock cycles between stamps 1 and 3

    // ---- the second group hands its triple to the first -------------------------
    // Through the K/V arrays, which nobody reads any more: wavefront w of the
    // second group writes (O, maximum, sum) lane by lane into array w, its
    // counterpart in the first group - same queries, same lanes - combines
    // them with its own as two partial softmaxes are combined.
    if constexpr(GROUPS > 1)
    {
        constexpr int NO = 16 * DBLOCKS;
        static_assert(GROUPS == 1 || (NO + 2) * 256 <= K_BYTES * GROUPS - 32 * RB,
                "the triple and the epilogue's staging rows share an array");
        float *mrg = reinterpret_cast<float *>(wave == 0 ? lds_k0 : wave == 1 ? lds_k1
                : wave == 2 ? lds_v0 : lds_v1) + lane;
        __syncthreads();
        if(grp == 1)
        {
#pragma unroll
            for(int db = 0; db < DBLOCKS; ++db)
            {
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    mrg[(16 * db + r) * 64] = o[db][r];
                }
            }
            mrg[NO * 64] = m_run;
            mrg[(NO + 1) * 64] = l_run;
        }
        __syncthreads();
        if(grp == 1)
        {
            return;
        }
        const float m_other = mrg[NO * 64];
        const float l_other = mrg[(NO + 1) * 64];
        const float m_new = fmaxf(m_run, m_other);
        // (a group that saw no visible key has maximum -inf and weight 0)
        const float a_mine = (m_run == neg_inf()) ? 0.0f : fast_exp2((m_run - m_new) * c);
        const float a_other = (m_other == neg_inf()) ? 0.0f : fast_exp2((m_other - m_new) * c);
#pragma unroll
        for(int db = 0; db < DBLOCKS; ++db)
        {
#pragma unroll
            for(int r = 0; r < 16; ++r)
            {
                o[db][r] = o[db][r] * a_mine + mrg[(16 * db + r) * 64] * a_other;
            }
        }
        l_run = l_run * a_mine + l_other * a_other;
        m_run = m_new;
    }

    // ---- epilogue: normalise, merge into the running (lse, A) ----------------
    const float l_tot = sum_across_halves(l_run);
    const bool empty = !(l_tot > 0.0f);     // no visible key for this query
    // rows that are written; the others leave lse and A as they are
    const bool live = q_ok && !(empty && !p.overwrite);
    const float to_ln = p.scale;
    const float lse_new = empty ? neg_inf() : m_run * to_ln + __logf(l_tot);
    float *lse_ptr = p.lse[q_tile0 + qt] + (int64_t)b * q_len + (q_ok ? my_q : 0);
    const float lse_old = (p.overwrite || !live) ? neg_inf() : *lse_ptr;
    float w_old = 0.0f, w_new = 0.0f, lse_out = neg_inf();
    if(live && !empty)
    {
        merge_weights(lse_old, lse_new, w_old, w_new, lse_out);
    }
    if(live && half == 0)
    {
        *lse_ptr = lse_out;
    }
    const float w_o = (empty || !live) ? 0.0f : w_new / l_tot;
    // register r of block db holds head value  db*32 + 8*(r/4) + 4*half + r%4

    if(__builtin_amdgcn_ballot_w64(live && w_old != 0.0f) == 0)
    {
        // Nothing of the old A is needed by this wavefront: its 32 rows go
        // through LDS (its own quarter of the K buffers, which nobody reads
        // any more after the last barrier) so that they leave as whole rows,
        // 16 bytes per lane, instead of 8-byte pieces 2*HEAD bytes apart.
        // 16-byte chunk c of row r sits at chunk position c ^ (r % CPR).
        // (two wavefronts per buffer: K0, K1, then V0, V1 for wavefronts 4 to 7)
        // (two groups: wavefront w uses the end of array w, behind the triple
        // it has just read - a neighbour may still be reading its own)
        char *xch = GROUPS > 1
            ? (wave == 0 ? lds_k0 : wave == 1 ? lds_k1 : wave == 2 ? lds_v0 : lds_v1)
                + (K_BYTES * GROUPS - 32 * RB)
            : ((wave >> 1) == 0 ? lds_k0 : (wave >> 1) == 1 ? lds_k1
                : (wave >> 1) == 2 ? lds_v0 : lds_v1) + (wave & 1) * 32 * RB;
#pragma unroll
        for(int db = 0; db < DBLOCKS; ++db)
        {
#pragma unroll
            for(int rg = 0; rg < 4; ++rg)
            {
                u32x2 out;
                out[0] = T::pack2(o[db][4 * rg] * w_o, o[db][4 * rg + 1] * w_o);
                out[1] = T::pack2(o[db][4 * rg + 2] * w_o, o[db][4 * rg + 3] * w_o);
                const int cpos = (db * 4 + rg) ^ (col % CPR);
                *reinterpret_cast<u32x2 *>(xch + col * RB + cpos * 16 + 8 * half) = out;
            }
        }
        const uint64_t live_rows = __builtin_amdgcn_ballot_w64(live && half == 0);
        constexpr int ROWS_PER_ST = 1024 / RB;      // rows one store instruction covers
        char *Abase = static_cast<char *>(p.A[q_tile0 + qt])
            + ((int64_t)b * q_len + q_row0 + wave * 32) * RB;
#pragma unroll
        for(int i = 0; i < 32 / ROWS_PER_ST; ++i)
        {
            const int r = i * ROWS_PER_ST + lane / CPR;
            const int c = lane % CPR;
            const u32x4 v = *reinterpret_cast<const u32x4 *>(
                    xch + r * RB + (c ^ (r % CPR)) * 16);
            if((live_rows >> r) & 1)
            {
                *reinterpret_cast<u32x4 *>(Abase + (int64_t)r * RB + c * 16) = v;
            }
        }
#ifdef NNTILE_PF_TRACE
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        PF_STAMP(4);
#endif
        return;
    }
    if(!live)
    {
        return;
    }
    uint16_t *Arow = static_cast<uint16_t *>(p.A[q_tile0 + qt])
        + ((int64_t)b * q_len + my_q) * HEAD;
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
#pragma unroll
        for(int rg = 0; rg < 4; ++rg)
        {
            uint16_t *dst = Arow + db * 32 + 8 * rg + 4 * half;
            float v[4];
#pragma unroll
            for(int e = 0; e < 4; ++e)
            {
                v[e] = empty ? 0.0f : o[db][4 * rg + e] * w_o;
            }
            if(w_old != 0.0f)
            {
                const u32x2 old = *reinterpret_cast<const u32x2 *>(dst);
                v[0] += w_old * T::to_float((uint16_t)(old[0] & 0xffffu));
                v[1] += w_old * T::to_float((uint16_t)(old[0] >> 16));
                v[2] += w_old * T::to_float((uint16_t)(old[1] & 0xffffu));
                v[3] += w_old * T::to_float((uint16_t)(old[1] >> 16));
            }
            u32x2 out;
            out[0] = T::pack2(v[0], v[1]);
            out[1] = T::pack2(v[2], v[3]);
            *reinterpret_cast<u32x2 *>(dst) = out;
        }
    }
}

template<typename T, int HEAD>
static int launch_mode(hipStream_t stream, const PrefillParams &p, int mode,
        dim3 grid, bool wide, bool key_split)
{
    constexpr int kThreads = 256;
    if constexpr(HEAD >= 64)
    {
        if(key_split)
        {
            switch(mode)
            {
                case NNTILE_HIP_MASK_ADDITIVE:
                    hipLaunchKernelGGL((sdpa_prefill_16bit_kernel<T, HEAD,
                                NNTILE_HIP_MASK_ADDITIVE, 8, 2>), grid, dim3(512), 0, stream, p);
                    break;
                case NNTILE_HIP_MASK_NONE:
                    hipLaunchKernelGGL((sdpa_prefill_16bit_kernel<T, HEAD,
                                NNTILE_HIP_MASK_NONE, 8, 2>), grid, dim3(512), 0, stream, p);
                    break;
                case NNTILE_HIP_MASK_CAUSAL:
                    hipLaunchKernelGGL((sdpa_prefill_16bit_kernel<T, HEAD,
                                NNTILE_HIP_MASK_CAUSAL, 8, 2>), grid, dim3(512), 0, stream, p);
                    break;
                case NNTILE_HIP_MASK_BOOL:
                    hipLaunchKernelGGL((sdpa_prefill_16bit_kernel<T, HEAD,
                                NNTILE_HIP_MASK_BOOL, 8, 2>), grid, dim3(512), 0, stream, p);
                    break;
                default:
                    return NNTILE_HIP_EINVAL;
            }
            return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
        }
    }
    switch(mode)
    {
        case NNTILE_HIP_MASK_ADDITIVE:
            hipLaunchKernelGGL((sdpa_prefill_16bit_kernel<T, HEAD,
                        NNTILE_HIP_MASK_ADDITIVE>), grid, dim3(kThreads), 0,
                    stream, p);
            break;
        case NNTILE_HIP_MASK_NONE:
            if constexpr(HEAD >= 64)
            {
                if(wide)
                {
                    hipLaunchKernelGGL((sdpa_prefill_16bit_kernel<T, HEAD,
                                NNTILE_HIP_MASK_NONE, 8>), grid, dim3(512), 0, stream, p);
                    break;
                }
            }
            hipLaunchKernelGGL((sdpa_prefill_16bit_kernel<T, HEAD,
                        NNTILE_HIP_MASK_NONE>), grid, dim3(kThreads), 0,
                    stream, p);
            break;
        case NNTILE_HIP_MASK_CAUSAL:
            if constexpr(HEAD >= 64)
            {
                if(wide)
                {
                    hipLaunchKernelGGL((sdpa_prefill_16bit_kernel<T, HEAD,
                                NNTILE_HIP_MASK_CAUSAL, 8>), grid, dim3(512), 0, stream, p);
                    break;
                }
            }
            hipLaunchKernelGGL((sdpa_prefill_16bit_kernel<T, HEAD,
                        NNTILE_HIP_MASK_CAUSAL>), grid, dim3(kThreads), 0,
                    stream, p);
            break;
        case NNTILE_HIP_MASK_BOOL:
            hipLaunchKernelGGL((sdpa_prefill_16bit_kernel<T, HEAD,
                        NNTILE_HIP_MASK_BOOL>), grid, dim3(kThreads), 0,
                    stream, p);
            break;
        default:
            return NNTILE_HIP_EINVAL;
    }
    return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
}

// The scan of an explicit mask that every workgroup of the attention kernel
// would do for its own 128 rows, done once for all batch entries, as a launch
// of its own (calls under stream capture; otherwise the scan rides in the
// attention launch): workgroup (query block, key range) writes its two words
// to entry blockIdx.x of the table (three words an entry, the third unused
// here; see PrefillParams::mask_bits).
template<int ES>
__global__ __launch_bounds__(kThreads)
void mask_step_bits_kernel(const char *mask, int ld_bytes, int q_len, int n_chunks,
        uint32_t open_word, uint32_t hidden_word, unsigned long long *table)
{
    __shared__ unsigned long long bits[2];
    mask_scan_range<ES, kThreads>(mask, ld_bytes, q_len, n_chunks, open_word, hidden_word,
            (int)blockIdx.x / kMaskBitSplits, (int)blockIdx.x % kMaskBitSplits, bits);
    if(threadIdx.x == 0)
    {
        table[3 * (int64_t)blockIdx.x] = bits[0];
        table[3 * (int64_t)blockIdx.x + 1] = bits[1];
    }
}

// Masks below this size are scanned by the attention kernel's workgroups
// themselves: the launch of the scan would cost more than it saves.
constexpr int64_t kMaskScanLaunchBytes = 1 << 20;

// A value no earlier call of this process has used and that memory left
// behind by anything else is unlikely to hold (never 0).
static unsigned long long next_scan_tag()
{
    static const unsigned long long salt = []
    {
        std::random_device rd;
        return ((unsigned long long)rd() << 32) | 0x40000000ull;
    }();
    static std::atomic<unsigned long long> counter{0};
    const unsigned long long tag = salt + counter.fetch_add(1, std::memory_order_relaxed) + 1ull;
    return tag == 0ull ? 1ull : tag;
}

// One-tile calls with an explicit mask and a scratch buffer of the caller's
// (the reference's scratch_logsumexp tile): scan the mask once, into the
// scratch, instead of once per batch entry - by the first workgroups of the
// attention launch itself, or, on a stream that is being captured (a replay
// would carry this call's tag again and find the flags of the replay before
// it), by a launch of its own.  Leaves p.mask_bits null when the conditions of
// the kernel's own scan do not hold or the scratch is too small.
template<typename T>
static int scan_mask_once(hipStream_t stream, PrefillParams &p, int mode,
        void *scratch, size_t scratch_bytes)
{
    p.n_scan_wgs = 0;
    const bool additive = mode == NNTILE_HIP_MASK_ADDITIVE;
    if((!additive && mode != NNTILE_HIP_MASK_BOOL) || scratch == nullptr
            || p.n_q_tiles != 1 || p.n_kv_tiles != 1 || p.mask == nullptr)
    {
        return NNTILE_HIP_OK;
    }
    const int64_t es = additive ? 2 : 1;
    const int64_t row_bytes = p.k_seq * es;
    const int64_t table_bytes = (int64_t)p.q_blocks_per_tile * kMaskBitSplits * 24;
    if(row_bytes % 16 != 0 || (p.mask_ld * es) % 16 != 0
            || reinterpret_cast<uintptr_t>(p.mask) % 16 != 0
            || p.mask_ld * es * kQRows >= (int64_t)(1 << 30)
            || reinterpret_cast<uintptr_t>(scratch) % 8 != 0
            || (int64_t)scratch_bytes < table_bytes
            || p.q_seq * row_bytes < kMaskScanLaunchBytes || p.batch < 2)
    {
        return NNTILE_HIP_OK;
    }
    auto *table = static_cast<unsigned long long *>(scratch);
    const dim3 grid((unsigned)(p.q_blocks_per_tile * kMaskBitSplits));
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if(hipStreamIsCapturing(stream, &capturing) != hipSuccess)
    {
        (void)hipGetLastError();
        capturing = hipStreamCaptureStatusActive;       // the careful form
    }
    if(capturing == hipStreamCaptureStatusNone)
    {
        p.mask_bits = table;
        p.n_scan_wgs = (int32_t)grid.x;
        p.mask_tag = next_scan_tag();
        p.mask_spin_limit = 100000000ull;       // 1 s of the 100 MHz clock
        return NNTILE_HIP_OK;
    }
    if(additive)
    {
        hipLaunchKernelGGL((mask_step_bits_kernel<2>), grid, dim3(kThreads), 0, stream,
                static_cast<const char *>(p.mask), (int)(p.mask_ld * es), (int)p.q_seq,
                (int)(row_bytes / 16), 0u, T::kNegInfPair, table);
    }
    else
    {
        hipLaunchKernelGGL((mask_step_bits_kernel<1>), grid, dim3(kThreads), 0, stream,
                static_cast<const char *>(p.mask), (int)(p.mask_ld * es), (int)p.q_seq,
                (int)(row_bytes / 16), 0x01010101u, 0u, table);
    }
    if(hipGetLastError() != hipSuccess)
    {
        return NNTILE_HIP_ELAUNCH;
    }
    p.mask_bits = table;
    return NNTILE_HIP_OK;
}

// Host launcher shared by the tile and grid entry points.  p must be fully
// filled except for the block counts and the remap flag.  scan_scratch: device
// memory the call may use for a scan of an explicit mask (may be null).
template<typename T>
int launch_prefill_16bit(hipStream_t stream, PrefillParams &p, int head,
        int mode, void *scan_scratch, size_t scan_scratch_bytes)
{
    // 256-query workgroups (eight wavefronts, one workgroup a CU): when asked
    // for (p.form == 8), and by themselves where they measured faster - head
    // 128, whole 256-query blocks, and enough of them that every CU gets two
    // under a causal mask (one workgroup a CU has nobody to share the CU with
    // while it starts and ends, and a causal launch of one round is set by its
    // longest workgroup), or a whole number of rounds without a mask.
    // p.form == 1 keeps the 128-query form.
    const bool can_wide = (head == 64 || head == 128)
        && (mode == NNTILE_HIP_MASK_NONE || mode == NNTILE_HIP_MASK_CAUSAL);
    bool wide = can_wide && p.form == 8;
    if(can_wide && p.form == 0 && head == 128 && (p.q_tile % 256 == 0 || p.n_q_tiles == 1))
    {
        const int64_t n_w = (int64_t)p.batch * p.n_slabs * p.n_q_tiles * ((p.q_tile + 255) / 256);
        wide = mode == NNTILE_HIP_MASK_CAUSAL ? n_w >= 512
            : (n_w >= 256 && (n_w % 256 == 0 || n_w >= 1024));
    }
    const int q_rows = wide ? 256 : kQRows;
    p.q_blocks_per_tile = (int)((p.q_tile + q_rows - 1) / q_rows);
    p.k_blocks_per_tile = (int)((p.k_tile + kKeys - 1) / kKeys);
    const int64_t batch_all = (int64_t)p.batch * p.n_slabs;
    const int64_t n_wg = batch_all * p.n_q_tiles * p.q_blocks_per_tile;
    if(n_wg <= 0 || n_wg > 0x7fffffff)
    {
        return NNTILE_HIP_EINVAL;
    }
    // Two groups of four wavefronts per workgroup, each taking every second
    // key step (p.form == 2, or by itself): when the launch has at most one
    // 128-query workgroup per CU, so that a CU would otherwise hold one
    // wavefront per SIMD, and enough key steps to share (with a mask given as
    // values a 1024-key tile measured no gain or a small loss - the scan of
    // the mask rows and the mask loads weigh more there - 4096 keys 7-11 %;
    // analytic masks: 3-8 % at 1024 keys and 256 workgroups, 12-20 % on
    // longer rows or fewer workgroups).
    const bool can_split = (head == 64 || head == 128) && !wide;
    const bool explicit_mask = mode == NNTILE_HIP_MASK_ADDITIVE || mode == NNTILE_HIP_MASK_BOOL;
    const bool key_split = can_split && (p.form == 2
            || (p.form == 0 && n_wg <= 8 * (int64_t)kCUsPerXCD
                && p.k_seq >= (explicit_mask ? 32 : 4) * kKeys));
    p.mask_bits = nullptr;
    const int scan_rc = scan_mask_once<T>(stream, p, mode, scan_scratch, scan_scratch_bytes);
    if(scan_rc != NNTILE_HIP_OK)
    {
        return scan_rc;
    }
    p.xcd_remap = (batch_all % 8 == 0) ? 1 : 0;
    // (the scanning workgroups come first; their number is a multiple of 8, so
    // the attention workgroups keep their places in the round of the XCDs)
    const dim3 grid((unsigned)(n_wg + p.n_scan_wgs));
    switch(head)
    {
        case 32:
            return launch_mode<T, 32>(stream, p, mode, grid, false, false);
        case 64:
            return launch_mode<T, 64>(stream, p, mode, grid, wide, key_split);
        case 128:
            return launch_mode<T, 128>(stream, p, mode, grid, wide, key_split);
        default:
            return NNTILE_HIP_EUNSUPPORTED;
    }
}

template int launch_prefill_16bit<Bf16>(hipStream_t, PrefillParams &, int, int, void *, size_t);
template int launch_prefill_16bit<Fp16>(hipStream_t, PrefillParams &, int, int, void *, size_t);

} // namespace nntile_hip
