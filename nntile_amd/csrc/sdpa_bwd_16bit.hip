// Scaled dot-product attention backward for 16-bit tiles on gfx950, in the
// flash form: the forward output A and the logsumexp are inputs, the
// probabilities are recomputed from them,
//
//   P[q,k]  = exp(scale q.k + mask[q,k] - lse[q])        D[q] = dA[q,:] . A[q,:]
//   dP[q,k] = dA[q,:] . V[k,:]                           dS   = P (dP - D)
//   dV[k,:] += sum_q P[q,k] dA[q,:]      dQ[q,:] += scale sum_k dS[q,k] K[k,:]
//   dK[k,:] += scale sum_q dS[q,k] Q[q,:]
//
// (include/nntile/kernel/flash_sdpa_bwd_cudnn/cuda.hh:44-68 is the interface
// this replaces; tests/kernel/flash_sdpa_bwd_cudnn.cc:174-262 the arithmetic).
// A small kernel writes D; then ONE launch computes the three gradients, each
// by its own workgroups (no atomics, results independent of timing):
//
//  * sdpa_bwd_dq_body: a workgroup owns 128 queries (a wavefront 32, a lane
//    one query) and walks the keys in steps of 64, as the forward kernel does:
//    S^T = K Q^T and dP^T = V dA^T with Q and dA fragments in registers and K, V
//    rows from LDS; dS^T packed to 16 bits is the B operand of
//    dQ^T += K^T dS^T, whose A operand comes through the transposing LDS read.
//  * sdpa_bwd_dkv_body<PART>: a workgroup owns 128 keys (a lane one key) and
//    walks the queries of every head of its group in steps of 64: S = Q K^T
//    and dP = dA V^T with K and V fragments in registers and Q, dA rows from
//    LDS; dV^T += dA^T P or dK^T += Q^T dS (PART) through transposing reads of
//    the same two LDS tiles.
//
// K, V, Q, dA steps go from global memory straight into LDS, double buffered;
// 16-byte chunk c of row r of a step sits at chunk position c ^ swz(r)
// (BwdTile::swz), which keeps both the row reads and the transposing reads
// free of bank conflicts.
#include <type_traits>

#include "sdpa_common.hpp"

namespace nntile_hip
{

// Developer build (-DNNTILE_BWD_TRACE): shader-clock cycles that the first
// wavefront of every key-owning workgroup spends in each phase of its steps,
// summed over the steps; read back with nntile_hip_debug_bwd_trace.
#ifdef NNTILE_BWD_TRACE
__device__ unsigned long long bwd_trace[8 * 4096];
__device__ unsigned long long bwd_wall[4 * 4096];
#define BWD_WALL(i, part) do { if(threadIdx.x == 0 && blockIdx.x < 4096) { \
        bwd_wall[4 * blockIdx.x + (i)] = wall_clock64(); bwd_wall[4 * blockIdx.x + 2] = (part); } } while(0)
#define BWD_WALL_AT(i) do { if(threadIdx.x == 0 && blockIdx.x < 4096) { \
        bwd_wall[4 * blockIdx.x + (i)] = wall_clock64(); } } while(0)
#define BWD_TRACE_DECL unsigned long long bt_sum[7] = {0, 0, 0, 0, 0, 0, 0}, bt_last = 0; int bt_steps = 0;
#define BWD_TRACE_START() do { bt_last = clock64(); } while(0)
#define BWD_TRACE_MARK(i) do { const unsigned long long now_ = clock64(); bt_sum[i] += now_ - bt_last; \
        bt_last = now_; } while(0)
#define BWD_TRACE_STEP() do { bt_steps += 1; } while(0)
#define BWD_TRACE_FLUSH(part) do { if(threadIdx.x == 0 && blockIdx.x < 4096) { \
        for(int i_ = 0; i_ < 6; ++i_) { bwd_trace[8 * blockIdx.x + i_] = bt_sum[i_]; } \
        bwd_trace[8 * blockIdx.x + 6] = (unsigned long long)bt_steps; \
        bwd_trace[8 * blockIdx.x + 7] = (unsigned long long)(part); } } while(0)
}
extern "C" int nntile_hip_debug_bwd_wall(unsigned long long *host)
{
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(nntile_hip::bwd_wall), sizeof(nntile_hip::bwd_wall));
}
extern "C" int nntile_hip_debug_bwd_trace(unsigned long long *host)
{
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(nntile_hip::bwd_trace), sizeof(nntile_hip::bwd_trace));
}
namespace nntile_hip
{
#else
#define BWD_TRACE_DECL
#define BWD_TRACE_START()
#define BWD_TRACE_MARK(i)
#define BWD_TRACE_STEP()
#define BWD_TRACE_FLUSH(part)
#define BWD_WALL(i, part)
#define BWD_WALL_AT(i)
#endif


// Where the tile loads of the next step are issued: 0 = all at the start of
// the step, 1 = between the MFMAs of the step's first half, 2 = of the whole
// 1: a step's two query (key) blocks overlap - the matrix products of one
// beside the vector work of the other; 0: one block after the other
#ifndef NNTILE_BWD_PIPE
#define NNTILE_BWD_PIPE 1
#endif
#ifndef NNTILE_BWD_PIPE_DQ
#define NNTILE_BWD_PIPE_DQ 1        // the same in the dQ workgroups
#endif
#ifndef NNTILE_BWD_AHEAD
#define NNTILE_BWD_AHEAD 2          // LDS operands are read this many MFMAs early
#endif
#ifndef NNTILE_BWD_SPREAD
#define NNTILE_BWD_SPREAD 2
#endif
#ifndef NNTILE_BWD_SWIZZLE_ROTATED
#define NNTILE_BWD_SWIZZLE_ROTATED 1
#endif
constexpr int kBwdRows = 128;       // queries (dQ workgroups) / keys (dK, dV workgroups) per workgroup
constexpr int kBwdStep = 64;        // rows of the other axis per step
constexpr int kBwdThreads = 256;

__device__ __forceinline__ u32x2 bwd_lds_read_tr16(const char *lds_ptr)
{
    typedef __attribute__((ext_vector_type(4))) short s16x4;
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(lds_ptr));
    return __builtin_bit_cast(u32x2, v);
}

// What the three kinds of workgroup share: the geometry of a 64-row step in LDS.
template<int HEAD>
struct BwdTile
{
    static constexpr int KSTEPS = HEAD / 16;       // MFMA steps along head
    static constexpr int DBLOCKS = HEAD / 32;      // 32-row blocks of a transposed gradient
    static constexpr int RB = HEAD * 2;            // bytes per row
    static constexpr int CPR = HEAD / 8;           // 16-byte chunks per row
    static constexpr int RPL = 16 / CPR;           // rows per 256-byte line of LDS banks
    static constexpr int ROWS_PER_LOAD = 1024 / RB;
    static constexpr int LOADS = kBwdStep / ROWS_PER_LOAD;
    static constexpr int LOADS_PER_WAVE = LOADS / 4;
    static constexpr int BYTES = kBwdStep * RB;
    static_assert(LOADS_PER_WAVE >= 1, "head size does not fit this tiling");

    // Chunk c of row r sits at chunk position c ^ swz(r).  Every tile is read
    // both ways: 16 lanes read the same chunk of 16 consecutive rows (they
    // need 16 different positions: swz must be one-to-one on 16 rows), and 32
    // lanes of a transposing read take 4 neighbouring chunks of 4 consecutive
    // rows (the 4 rows need different groups of 4 positions: the low bits of
    // the line number must land in the top bits).  Both hold for the line
    // number (r / RPL) % CPR rotated right by log2(CPR) - 2 bits.
    static __device__ __forceinline__ int swz(int r)
    {
        constexpr int ROT = CPR == 16 ? 2 : (CPR == 8 ? 1 : 0);
        constexpr int BITS = CPR == 16 ? 4 : (CPR == 8 ? 3 : 2);
        const int line = (r / RPL) % CPR;
#if NNTILE_BWD_SWIZZLE_ROTATED
        return ((line >> ROT) | (line << (BITS - ROT))) & (CPR - 1);
#else
        return line;
#endif
    }
};

// The registers of a 32x32 accumulator tile of lane (col, half): register r is
// row 8*(r/4) + 4*half + r%4 of the tile, column col.
// Workgroup number -> (batch entry, block along the sequence).  Workgroups
// go to the 8 XCDs round robin: the entries of the batch are dealt so that
// all blocks of one entry run on one XCD and share its L2, and the blocks are
// taken in the order longest first (`last_first`: from the last block down).
__device__ __forceinline__ void map_workgroup(unsigned wg, int entries, int blocks,
        bool last_first, int &entry, int &block)
{
    int i;
    if((entries & 7) == 0)
    {
        const int per_xcd = entries >> 3;
        i = (int)(wg >> 3);
        entry = (int)(wg & 7u) * per_xcd + i % per_xcd;
        i /= per_xcd;
    }
    else
    {
        entry = (int)(wg % (unsigned)entries);
        i = (int)(wg / (unsigned)entries);
    }
    // (the same for every lane: into scalar registers, whatever the divisions
    // were computed with)
    entry = __builtin_amdgcn_readfirstlane(entry);
    block = __builtin_amdgcn_readfirstlane(last_first ? blocks - 1 - i : i);
}

// The lane's index within its wavefront, asked of the hardware where it is
// needed again after a long loop (the thread index the kernel started with
// would have to sit in a register all the way through, and at head 128 there
// is none to spare).  Does not depend on which lanes are active.
__device__ __forceinline__ int lane_index_again()
{
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
}

__device__ __forceinline__ int tile_row(int r, int half)
{
    return 8 * (r >> 2) + 4 * half + (r & 3);
}

// ---------------------------------------------------------------------------------
// Masks given as values: one pass writes the class of every 64 x 64 block of
// the mask (the reference hands the kernel a materialised tile even where it is
// causal, src/tile/flash_sdpa_bwd_cudnn.cc), so that the three kernels below skip
// the steps whose blocks hide everything - without fetching them - and read no
// mask values in the steps whose blocks mask nothing.
constexpr int kMaskMixed = 0, kMaskOpen = 1, kMaskHidden = 2;

template<typename T, int MODE>
__global__ __launch_bounds__(256)
void sdpa_bwd_mask_classes_kernel(const void *mask, int64_t mask_ld, int q_seq, int k_seq,
        uint8_t *table, int class_ld)
{
    const int qb = blockIdx.x / class_ld, kb = blockIdx.x % class_ld;
    const int row = qb * kBwdStep + (int)threadIdx.x / 4;
    const int col0 = kb * kBwdStep + ((int)threadIdx.x % 4) * 16;
    bool any_visible = false, any_masked = false;
    constexpr int ES = (MODE == NNTILE_HIP_MASK_ADDITIVE) ? 2 : 1;
    const bool wide = (mask_ld * ES) % 16 == 0 && reinterpret_cast<uintptr_t>(mask) % 16 == 0;
    if(row < q_seq && col0 < k_seq)
    {
        const char *src = static_cast<const char *>(mask) + ((int64_t)row * mask_ld + col0) * ES;
        if(wide && col0 + 16 <= k_seq)
        {
            // the thread's 16 values as 16-byte loads
#pragma unroll
            for(int i = 0; i < ES; ++i)
            {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(src + 16 * i);
#pragma unroll
                for(int w = 0; w < 4; ++w)
                {
                    if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                    {
                        any_masked |= v[w] != 0u;
                        any_visible |= v[w] != T::kNegInfPair;
                    }
                    else
                    {
                        any_masked |= v[w] != 0x01010101u;
                        any_visible |= v[w] != 0u;
                    }
                }
            }
        }
        else
        {
            for(int e = 0; e < 16 && col0 + e < k_seq; ++e)
            {
                if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                {
                    const uint16_t v = reinterpret_cast<const uint16_t *>(src)[e];
                    any_visible |= (T::to_float(v) != neg_inf());
                    any_masked |= (v != 0);         // anything but +0 changes the score
                }
                else
                {
                    const bool vis = reinterpret_cast<const uint8_t *>(src)[e] != 0;
                    any_visible |= vis;
                    any_masked |= !vis;
                }
            }
        }
    }
    const int vis = __syncthreads_or(any_visible ? 1 : 0);
    const int msk = __syncthreads_or(any_masked ? 1 : 0);
    if(threadIdx.x == 0)
    {
        table[blockIdx.x] = (uint8_t)(!msk ? kMaskOpen : (!vis ? kMaskHidden : kMaskMixed));
    }
}

// The steps a workgroup takes, as a bit set (up to 64 of them; longer walks
// take every step), and the subset in which nothing is masked.
struct StepSet
{
    unsigned long long active, open;
    bool use_bits;
    int first, last;        // [first, last): the walk without the table

    __device__ __forceinline__ int begin() const
    {
        if(!use_bits)
        {
            return first < last ? first : -1;
        }
        return active != 0ull ? __builtin_ctzll(active) : -1;
    }
    __device__ __forceinline__ int next(int g) const
    {
        if(!use_bits)
        {
            return g + 1 < last ? g + 1 : -1;
        }
        const unsigned long long rest = g >= 63 ? 0ull : (active >> (g + 1)) << (g + 1);
        return rest != 0ull ? __builtin_ctzll(rest) : -1;
    }
    __device__ __forceinline__ bool is_open(int g) const
    {
        return use_bits && ((open >> g) & 1ull) != 0ull;
    }
};

// Step set of a workgroup that owns the blocks [own0, own0 + n_own) of one axis
// and walks the blocks [first, last) of the other.  by_row: the owned blocks
// are query blocks (rows of the table).
__device__ __forceinline__ StepSet make_step_set(const BwdParams &p, bool explicit_mask,
        int own0, int n_own, int first, int last, bool by_row)
{
    StepSet s;
    s.first = first;
    s.last = last;
    s.use_bits = explicit_mask && p.mask_class != nullptr && last <= 64;
    s.active = 0ull;
    s.open = 0ull;
    if(s.use_bits)
    {
        // lane g looks at step g; the ballots make the two sets (every
        // wavefront computes the same)
        const int g = (int)(threadIdx.x & 63);
        const bool in_walk = g >= first && g < last;
        bool hidden = true, open = true;
        for(int o = 0; o < n_own; ++o)
        {
            const int idx = by_row ? (own0 + o) * p.class_ld + g : g * p.class_ld + own0 + o;
            const int c = in_walk ? p.mask_class[idx] : kMaskHidden;
            hidden = hidden && (c == kMaskHidden);
            open = open && (c == kMaskOpen);
        }
        s.active = __builtin_amdgcn_ballot_w64(in_walk && !hidden);
        s.open = __builtin_amdgcn_ballot_w64(in_walk && open);
    }
    return s;
}

// ---------------------------------------------------------------------------------
// D[b][q] = dA[b][q][:] . A[b][q][:] in fp32, for the workgroups below: 16-byte
// loads, HEAD/8 lanes a row, summed across those lanes.
template<typename T, int HEAD>
__global__ __launch_bounds__(256)
void sdpa_bwd_rowdot_kernel(const void *dA, const void *A, float *D, int64_t rows)
{
    constexpr int LANES = HEAD / 8;             // lanes per row: 16, 8 or 4
    const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LANES;
    const int part = (int)(threadIdx.x % LANES);
    float d = 0.0f;
    if(row < rows)
    {
        const u32x4 g = *reinterpret_cast<const u32x4 *>(
                static_cast<const uint16_t *>(dA) + row * HEAD + part * 8);
        const u32x4 a = *reinterpret_cast<const u32x4 *>(
                static_cast<const uint16_t *>(A) + row * HEAD + part * 8);
#pragma unroll
        for(int e = 0; e < 4; ++e)
        {
            d += T::to_float((uint16_t)(g[e] & 0xffffu)) * T::to_float((uint16_t)(a[e] & 0xffffu));
            d += T::to_float((uint16_t)(g[e] >> 16)) * T::to_float((uint16_t)(a[e] >> 16));
        }
    }
#pragma unroll
    for(int o = LANES / 2; o >= 1; o >>= 1)
    {
        d += __shfl_xor(d, o, 64);
    }
    if(row < rows && part == 0)
    {
        D[row] = d;
    }
}

// GRID: the rows of both sequence axes live in separately allocated tiles
// (BwdGridParams); a workgroup's own 128 rows lie in one tile and every 64-row
// step of the other axis does too, because tile sizes are multiples of 128.
template<typename T, int HEAD, int MODE, bool GRID>
__device__ __forceinline__ void sdpa_bwd_dq_body(
        const std::conditional_t<GRID, BwdGridParams, BwdParams> &p, unsigned wg,
        char *lds_k0, char *lds_k1, char *lds_v0, char *lds_v1)
{
    typedef typename T::vec8 vec8;
    typedef BwdTile<HEAD> G;
    constexpr int KSTEPS = G::KSTEPS, DBLOCKS = G::DBLOCKS, RB = G::RB, CPR = G::CPR;
    constexpr int LOADS_PER_WAVE = G::LOADS_PER_WAVE, ROWS_PER_LOAD = G::ROWS_PER_LOAD;
    constexpr bool EXPLICIT = (MODE == NNTILE_HIP_MASK_ADDITIVE
            || MODE == NNTILE_HIP_MASK_BOOL);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int col = lane & 31;
    const int half = lane >> 5;

    const int q_blocks = (int)((p.q_seq + kBwdRows - 1) / kBwdRows);
    // the last query blocks see the most keys under a causal mask: first
    int b, q_block;
    // (the grid form: the slab of the entry, whose tiles are allocations of
    // their own)
    int q_tile0 = 0, k_tile0 = 0;
    int64_t d_slab = 0;
    if constexpr(GRID)
    {
        map_workgroup(wg, p.batch * p.n_slabs, q_blocks, true, b, q_block);
        if(p.n_slabs > 1)
        {
            const int slab = b / p.batch;
            b -= slab * p.batch;
            q_tile0 = slab * p.n_q_tiles;
            k_tile0 = slab * p.n_kv_tiles;
            d_slab = (int64_t)slab * p.q_seq * p.batch;
        }
    }
    else
    {
        map_workgroup(wg, p.batch, q_blocks, true, b, q_block);
    }
    const int q_row0 = q_block * kBwdRows;
    const int kvb = kv_entry(b, p.n_batch, p.kv_group);
    const int q_seq = (int)p.q_seq, k_seq = (int)p.k_seq;
    const int my_q = q_row0 + wave * 32 + col;
    const bool q_ok = my_q < q_seq;
    // the lane's query: its row within the allocation that holds it (of Q, dA,
    // dQ, and of lse without the head axis), and its place among the row dots
    // (a function of the row, so that the stores at the end can work it out
    // again instead of keeping it through the loop)
    int own_t0 = 0, own_rows = q_seq;           // the tile that holds the block's rows
    if constexpr(GRID)
    {
        const int q_tile = (int)p.q_tile;
        own_t0 = __builtin_amdgcn_readfirstlane((q_row0 / q_tile) * q_tile);
        own_rows = min(q_tile, q_seq - own_t0);
    }
    auto row_elem = [&](int row, bool ok) __attribute__((always_inline)) -> int64_t
    {
        return (int64_t)b * own_rows + ((ok ? row : (GRID ? q_row0 : 0)) - own_t0);
    };
    const int64_t q_elem = row_elem(my_q, q_ok);
    int64_t d_idx = q_elem;
    const void *Q_own = p.Q, *dA_own = p.dA;
    void *dQ_own = p.dQ;
    const float *lse_own = p.lse;
    if constexpr(GRID)
    {
        const int q_tile = (int)p.q_tile;
        const int tq = q_row0 / q_tile, t0 = tq * q_tile;
        d_idx = d_slab + (int64_t)p.batch * t0 + q_elem;
        Q_own = p.Qt[q_tile0 + tq];
        dA_own = p.dAt[q_tile0 + tq];
        dQ_own = p.dQt[q_tile0 + tq];
        lse_own = p.lset[q_tile0 + tq];
    }
    const int64_t q_off = q_elem * HEAD;

    // Q and dA fragments (B operands); the row dot D = dA . A of the query
    vec8 qf[KSTEPS], gf[KSTEPS];
    {
        const uint16_t *qs = static_cast<const uint16_t *>(Q_own) + q_off + half * 8;
        const uint16_t *gs = static_cast<const uint16_t *>(dA_own) + q_off + half * 8;
#pragma unroll
        for(int ks = 0; ks < KSTEPS; ++ks)
        {
            u32x4 q = *reinterpret_cast<const u32x4 *>(qs + ks * 16);
            u32x4 g = *reinterpret_cast<const u32x4 *>(gs + ks * 16);
            if(!q_ok)
            {
                q = u32x4{0, 0, 0, 0};
                g = u32x4{0, 0, 0, 0};
            }
            qf[ks] = __builtin_bit_cast(vec8, q);
            gf[ks] = __builtin_bit_cast(vec8, g);
        }
    }
    const float d_row = q_ok ? p.D[d_idx] : 0.0f;
    const float lse_q = q_ok ? lse_own[q_elem] : neg_inf();
    // exponent offset in log2 units; a row that saw nothing has P = 0
    const float lse2 = (lse_q == neg_inf()) ? __builtin_huge_valf() : lse_q * kLog2e;

    // ---- which keys ---------------------------------------------------------------
    // key row kg is visible to query row q iff kg <= rel + q (causal)
    int64_t rel64 = p.q_pos0 + p.causal_offset - p.k_pos0;
    rel64 = max((int64_t)-(1 << 30), min(rel64, (int64_t)(1 << 30)));
    const int rel = (int)rel64;
    int n_steps = (k_seq + kBwdStep - 1) / kBwdStep;
    if(MODE == NNTILE_HIP_MASK_CAUSAL)
    {
        const int hi = min(rel + min(q_row0 + kBwdRows, q_seq) - 1, k_seq - 1);
        n_steps = hi < 0 ? 0 : min(n_steps, hi / kBwdStep + 1);
    }
    const int my_lim = rel + my_q;          // last visible key of this lane's query

    // ---- LDS addresses --------------------------------------------------------------
    uint32_t ld_goff[LOADS_PER_WAVE];
    const int ld_cpos = lane % CPR;
    const int ld_row0 = wave * LOADS_PER_WAVE * ROWS_PER_LOAD + lane / CPR;   // + i * ROWS_PER_LOAD
#pragma unroll
    for(int i = 0; i < LOADS_PER_WAVE; ++i)
    {
        const int r = ld_row0 + i * ROWS_PER_LOAD;
        ld_goff[i] = (uint32_t)(r * RB + (ld_cpos ^ G::swz(r)) * 16);
    }
    // (only the last step of the keys can be short: its rows past the end read
    // the last row that exists; the offsets of that step are kept beside the
    // others rather than computed per load)
    uint32_t ld_goff_end[LOADS_PER_WAVE];
    {
        const int last_of_end = (k_seq - 1) % kBwdStep;
#pragma unroll
        for(int i = 0; i < LOADS_PER_WAVE; ++i)
        {
            ld_goff_end[i] = ld_goff[i]
                - (uint32_t)(max(ld_row0 + i * ROWS_PER_LOAD - last_of_end, 0) * RB);
        }
    }
    // row operand: lane (col, half) reads row mb*32+col, logical chunk 2*ks+half;
    // 32 rows further on the swizzle is the same, so mb goes into the immediate
    uint32_t row_raddr[KSTEPS];
#pragma unroll
    for(int ks = 0; ks < KSTEPS; ++ks)
    {
        row_raddr[ks] = (uint32_t)(col * RB + ((2 * ks + half) ^ G::swz(col)) * 16);
    }
    // transposed operand: within a 16-lane block lane i addresses row j = i/4 and
    // head values 4*(i%4)..+3 of the block's 16; lanes 16..31 take the upper 16
    // head values of a 32-row block, the lane half the rows 4..7.  For the
    // 16-row sub-step t the two reads cover rows 16t + 4*half + j and + 8; the
    // swizzle of a row does not depend on t, so 16t goes into the immediate.
    uint32_t tr_raddr[2][DBLOCKS];
    {
        const int i16 = lane & 15, dblk = (lane >> 4) & 1;
        const int j = i16 >> 2, r4 = i16 & 3;
#pragma unroll
        for(int a = 0; a < 2; ++a)
        {
            const int r = 4 * half + j + 8 * a;
#pragma unroll
            for(int db = 0; db < DBLOCKS; ++db)
            {
                const int c = 4 * db + 2 * dblk + (r4 >> 1);
                tr_raddr[a][db] = (uint32_t)(r * RB + (c ^ G::swz(r)) * 16 + 8 * (r4 & 1));
            }
        }
    }

    const char *Kb = static_cast<const char *>(p.K) + (int64_t)kvb * k_seq * RB;
    const char *Vb = static_cast<const char *>(p.V) + (int64_t)kvb * k_seq * RB;
    // loads of key step g; rows past the end are clamped to the last row
    // (their probabilities are exactly 0)
    // (a wave gets one such load accepted every ~64 cycles and stands still
    // until then: inside the loop the loads go between the MFMAs, one K and
    // one V load at a time)
    struct KeyRows
    {
        const char *K, *V;      // the step's first row of the entry
        bool at_end;
    };
    auto key_rows = [&](int g) __attribute__((always_inline)) -> KeyRows
    {
        const int row0 = g * kBwdStep;
        const bool at_end = row0 + kBwdStep > k_seq;
        if constexpr(GRID)
        {
            const int k_tile = (int)p.k_tile;
            const int tk = row0 / k_tile, t0 = tk * k_tile;
            const int64_t off = ((int64_t)kvb * min(k_tile, k_seq - t0) + (row0 - t0)) * RB;
            return KeyRows{static_cast<const char *>(p.Kt[k_tile0 + tk]) + off,
                static_cast<const char *>(p.Vt[k_tile0 + tk]) + off, at_end};
        }
        else
        {
            return KeyRows{Kb + (int64_t)row0 * RB, Vb + (int64_t)row0 * RB, at_end};
        }
    };
    auto fetch_piece = [&](const KeyRows &at, char *kdst_base, char *vdst_base, int i)
        __attribute__((always_inline))
    {
        char *kdst = kdst_base + wave_u * LOADS_PER_WAVE * 1024;
        char *vdst = vdst_base + wave_u * LOADS_PER_WAVE * 1024;
        const uint32_t goff = at.at_end ? ld_goff_end[i] : ld_goff[i];
        load_to_lds16<0, false>(at.K, goff, kdst + i * 1024);
        load_to_lds16<0, false>(at.V, goff, vdst + i * 1024);
    };
    auto fetch = [&](int g, char *kdst_base, char *vdst_base)
    {
        const KeyRows at = key_rows(g);
#pragma unroll
        for(int i = 0; i < LOADS_PER_WAVE; ++i)
        {
            fetch_piece(at, kdst_base, vdst_base, i);
        }
    };
    constexpr int FETCH_STRIDE = (NNTILE_BWD_SPREAD == 2 ? 2 : 1) * KSTEPS / LOADS_PER_WAVE;
    static_assert(FETCH_STRIDE >= 1 && 1 + (LOADS_PER_WAVE - 1) * FETCH_STRIDE < 2 * KSTEPS,
            "the pieces of a fetch must fit between the MFMAs of a step");

    f32x16 acc[DBLOCKS];
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
#pragma unroll
        for(int r = 0; r < 16; ++r)
        {
            acc[db][r] = 0.0f;
        }
    }
    const float c = p.scale * kLog2e;
    // mask values: the workgroup's first row of the mask, and the byte offset
    // of the lane's row from there (the launcher keeps 128 rows of the mask
    // within 32 bits); mask_off is that of the lane's first key in a step
    constexpr uint32_t MASK_ES = MODE == NNTILE_HIP_MASK_ADDITIVE ? 2u : 1u;
    const char *mask_wg = static_cast<const char *>(p.mask)
        + (int64_t)q_row0 * p.mask_ld * (int64_t)MASK_ES;
    const uint32_t mask_row_off = (uint32_t)(q_ok ? my_q - q_row0 : 0) * (uint32_t)p.mask_ld * MASK_ES;
    const uint32_t mask_off_wg = mask_row_off + (uint32_t)(4 * half) * MASK_ES;

    // the workgroup's two query blocks of 64 against the key blocks 0 .. n_steps-1
    const StepSet steps = make_step_set(p, EXPLICIT, q_row0 / kBwdStep,
            min(2, (q_seq - q_row0 + kBwdStep - 1) / kBwdStep), 0, n_steps, true);
    int g_cur = steps.begin();
    if(g_cur >= 0)
    {
        fetch(g_cur, lds_k0, lds_v0);
    }
    // masked_tag: the step reads mask values (as a compile-time choice, so
    // that the reads of a step stay one batch of loads)
    auto step = [&](int g, int g_next, auto buf_tag, auto masked_tag)
        __attribute__((always_inline))
    {
        constexpr int BUF = decltype(buf_tag)::value;
        const char *Ks = BUF ? lds_k1 : lds_k0;
        const char *Vs = BUF ? lds_v1 : lds_v0;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        // the last step loads its own tile once more, rather than branch
        // (wave-common, computed once here: the loads between the MFMAs below
        // only add their offsets)
        const KeyRows at_f = key_rows(g_next >= 0 ? g_next : g);
        if(NNTILE_BWD_SPREAD == 0 && g_next >= 0)
        {
            fetch(g_next, BUF ? lds_k0 : lds_k1, BUF ? lds_v0 : lds_v1);
        }
        constexpr bool use_mask = EXPLICIT && decltype(masked_tag)::value;
        const int kg0 = g * kBwdStep;
        const int keys_here = min(kBwdStep, k_seq - kg0);
        const char *mask_step = mask_wg + (int64_t)kg0 * MASK_ES;
        const uint32_t mask_off_last = mask_row_off + (uint32_t)(keys_here - 1) * MASK_ES;
        // (through an empty asm statement: the 32 offsets that a step adds
        // constants to are then made where the step uses them instead of once
        // before the loop and kept, which at head 128 means spilled)
        uint32_t mask_off = mask_off_wg;
        if(use_mask)
        {
            asm volatile("" : "+v"(mask_off));
        }

        // ---- S^T = K Q^T, dP^T = V dA^T -------------------------------------------------
        // (one 32-key block at a time: half the accumulators live)
        // ---- P^T, dS^T: register r of block mb is key mb*32 + tile_row(r, half) ------------
        int lim = keys_here - 1;
        if(MODE == NNTILE_HIP_MASK_CAUSAL)
        {
            lim = min(lim, my_lim - kg0);
        }
        const int lim_less_half = lim - 4 * half;
        // (wave-common: the last key of the step against the last key that
        // exists and the last key the workgroup's first query sees)
        const bool bounds = keys_here < kBwdStep
            || (MODE == NNTILE_HIP_MASK_CAUSAL && kg0 + kBwdStep - 1 > rel + q_row0);
        if constexpr(EXPLICIT || NNTILE_BWD_PIPE_DQ == 0)
        {
#pragma unroll
            for(int mb = 0; mb < 2; ++mb)
            {
                f32x16 sv, dpv;
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    sv[r] = 0.0f;
                    dpv[r] = 0.0f;
                }
#pragma unroll
                for(int ks = 0; ks < KSTEPS; ++ks)
                {
                    const vec8 ka = *reinterpret_cast<const vec8 *>(Ks + row_raddr[ks] + mb * 32 * RB);
                    const vec8 va = *reinterpret_cast<const vec8 *>(Vs + row_raddr[ks] + mb * 32 * RB);
                    sv = T::mfma(ka, qf[ks], sv);
                    dpv = T::mfma(va, gf[ks], dpv);
#pragma unroll
                    for(int j = 0; j < LOADS_PER_WAVE; ++j)
                    {
                        if(NNTILE_BWD_SPREAD != 0 && mb * KSTEPS + ks == 1 + j * FETCH_STRIDE)
                        {
                            fetch_piece(at_f, BUF ? lds_k0 : lds_k1, BUF ? lds_v0 : lds_v1, j);
                        }
                    }
                }
                // Keys past the end and keys the causal mask hides: their scores
                // become -inf in a pass of their own, which only the steps at the
                // end of the keys and on the diagonal run (a wave-common branch).
                if(bounds)
                {
#pragma unroll
                    for(int r = 0; r < 16; ++r)
                    {
                        // (key mb*32 + tile_row(r, half) <= lim, the lane's part on the right)
                        sv[r] = mb * 32 + tile_row(r, 0) <= lim_less_half ? sv[r] : neg_inf();
                    }
                }
                float dsv[16];
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    float e = fmaf(sv[r], c, -lse2);        // -inf: hidden, or a row that saw nothing
                    bool visible = true;
                    if(use_mask)
                    {
                        // wave-common address of the step's first key in the
                        // workgroup's first row + the lane's 32-bit offset;
                        // keys past the end read the last key, and are hidden
                        const uint32_t key_off = (uint32_t)(mb * 32 + tile_row(r, 0)) * MASK_ES;
                        const char *mp = mask_step + min(mask_off + key_off, mask_off_last);
                        if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                        {
                            const float add = T::to_float(*reinterpret_cast<const uint16_t *>(mp));
                            visible = visible && (add != neg_inf());
                            e = fmaf(add, kLog2e, e);
                        }
                        else
                        {
                            const uint8_t shown = *reinterpret_cast<const uint8_t *>(mp);
                            visible = visible && (shown != 0);
                        }
                    }
                    const float pr = use_mask ? (visible ? fast_exp2(e) : 0.0f) : fast_exp2(e);
                    dsv[r] = pr * (dpv[r] - d_row);
                }
                uint32_t ds_pk[8];
#pragma unroll
                for(int k = 0; k < 8; ++k)
                {
                    ds_pk[k] = T::pack2(dsv[2 * k], dsv[2 * k + 1]);
                }
                // ---- dQ^T += K^T dS^T: the block's two sub-steps of 16 keys ------------------
#pragma unroll
                for(int tt = 0; tt < 2; ++tt)
                {
                    const int t = 2 * mb + tt;
                    const u32x4 braw = {ds_pk[4 * tt], ds_pk[4 * tt + 1], ds_pk[4 * tt + 2],
                        ds_pk[4 * tt + 3]};
                    const vec8 bop = __builtin_bit_cast(vec8, braw);
#pragma unroll
                    for(int db = 0; db < DBLOCKS; ++db)
                    {
                        const u32x2 lo = bwd_lds_read_tr16(Ks + tr_raddr[0][db] + (16 * t) * RB);
                        const u32x2 hi = bwd_lds_read_tr16(Ks + tr_raddr[1][db] + (16 * t) * RB);
                        const u32x4 araw = {lo[0], lo[1], hi[0], hi[1]};
                        acc[db] = T::mfma(__builtin_bit_cast(vec8, araw), bop, acc[db]);
                    }
                }
            }
        }
        else
        {
            // The step's two 32-key blocks in three phases each - A: the two
            // score products, B: dS on the vector ALU, C: dQ^T += K^T dS^T -
            // issued as A0 | A1 with B0 | C0 with B1 | C1 (see the dK / dV body).
            f32x16 sv[2], dpv[2];
            uint32_t ds_pk[2][8];
            constexpr int A_MFMAS = 2 * KSTEPS, C_MFMAS = 2 * DBLOCKS;
            constexpr int AHEAD = NNTILE_BWD_AHEAD;
            auto a_init = [&](int mb) __attribute__((always_inline))
            {
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    sv[mb][r] = 0.0f;
                    dpv[mb][r] = 0.0f;
                }
            };
            auto a_read = [&](int mb, int i, vec8 (&ring)[AHEAD + 1]) __attribute__((always_inline))
            {
                if(i >= A_MFMAS)
                {
                    return;
                }
                ring[i % (AHEAD + 1)] = *reinterpret_cast<const vec8 *>(((i & 1) ? Vs : Ks)
                        + row_raddr[i / 2] + mb * 32 * RB);
            };
            auto a_mfma = [&](int mb, int i, vec8 (&ring)[AHEAD + 1]) __attribute__((always_inline))
            {
                const int ks = i / 2;
                if(i & 1)
                {
                    dpv[mb] = T::mfma(ring[i % (AHEAD + 1)], gf[ks], dpv[mb]);
#pragma unroll
                    for(int j = 0; j < LOADS_PER_WAVE; ++j)
                    {
                        if(NNTILE_BWD_SPREAD != 0 && mb * KSTEPS + ks == 1 + j * FETCH_STRIDE)
                        {
                            fetch_piece(at_f, BUF ? lds_k0 : lds_k1, BUF ? lds_v0 : lds_v1, j);
                        }
                    }
                }
                else
                {
                    sv[mb] = T::mfma(ring[i % (AHEAD + 1)], qf[ks], sv[mb]);
                }
            };
            // Keys past the end and keys the causal mask hides: their scores
            // become -inf in a pass of their own, which only the steps at the
            // end of the keys and on the diagonal run (a wave-common branch).
            auto hide = [&](int mb) __attribute__((always_inline))
            {
                if(bounds)
                {
#pragma unroll
                    for(int r = 0; r < 16; ++r)
                    {
                        // (key mb*32 + tile_row(r, half) <= lim, the lane's part on the right)
                        sv[mb][r] = mb * 32 + tile_row(r, 0) <= lim_less_half ? sv[mb][r]
                            : neg_inf();
                    }
                }
            };
            float ds_even = 0.0f;
            auto b_item = [&](int mb, int r) __attribute__((always_inline))
            {
                const float e = fmaf(sv[mb][r], c, -lse2);        // -inf: hidden, or a row that saw nothing
                const float pr = fast_exp2(e);
                const float dsr = pr * (dpv[mb][r] - d_row);
                if(r % 2 == 0)
                {
                    ds_even = dsr;
                }
                else
                {
                    ds_pk[mb][r / 2] = T::pack2(ds_even, dsr);
                    asm volatile("" : "+v"(ds_pk[mb][r / 2]));
                }
            };
            // the block's two sub-steps of 16 keys
            auto c_read = [&](int mb, int i, vec8 (&ring)[AHEAD + 1]) __attribute__((always_inline))
            {
                if(i >= C_MFMAS)
                {
                    return;
                }
                const int t = 2 * mb + i / DBLOCKS, db = i % DBLOCKS;
                const u32x2 lo = bwd_lds_read_tr16(Ks + tr_raddr[0][db] + (16 * t) * RB);
                const u32x2 hi = bwd_lds_read_tr16(Ks + tr_raddr[1][db] + (16 * t) * RB);
                const u32x4 araw = {lo[0], lo[1], hi[0], hi[1]};
                ring[i % (AHEAD + 1)] = __builtin_bit_cast(vec8, araw);
            };
            auto c_mfma = [&](int mb, int i, vec8 (&ring)[AHEAD + 1]) __attribute__((always_inline))
            {
                const int tt = i / DBLOCKS, db = i % DBLOCKS;
                const u32x4 braw = {ds_pk[mb][4 * tt], ds_pk[mb][4 * tt + 1], ds_pk[mb][4 * tt + 2],
                    ds_pk[mb][4 * tt + 3]};
                acc[db] = T::mfma(ring[i % (AHEAD + 1)], __builtin_bit_cast(vec8, braw), acc[db]);
            };
            {
                vec8 ring[AHEAD + 1];
                a_init(0);
#pragma unroll
                for(int i = 0; i < AHEAD; ++i)
                {
                    a_read(0, i, ring);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(int i = 0; i < A_MFMAS; ++i)
                {
                    a_read(0, i + AHEAD, ring);
                    a_mfma(0, i, ring);
                    __builtin_amdgcn_sched_barrier(0);
                }
                hide(0);
                a_init(1);
#pragma unroll
                for(int i = 0; i < AHEAD; ++i)
                {
                    a_read(1, i, ring);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(int i = 0; i < A_MFMAS; ++i)
                {
                    a_read(1, i + AHEAD, ring);
                    a_mfma(1, i, ring);
#pragma unroll
                    for(int r = i * 16 / A_MFMAS; r < (i + 1) * 16 / A_MFMAS; ++r)
                    {
                        b_item(0, r);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                hide(1);
#pragma unroll
                for(int i = 0; i < AHEAD; ++i)
                {
                    c_read(0, i, ring);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(int i = 0; i < C_MFMAS; ++i)
                {
                    c_read(0, i + AHEAD, ring);
                    c_mfma(0, i, ring);
#pragma unroll
                    for(int r = i * 16 / C_MFMAS; r < (i + 1) * 16 / C_MFMAS; ++r)
                    {
                        b_item(1, r);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for(int i = 0; i < AHEAD; ++i)
                {
                    c_read(1, i, ring);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(int i = 0; i < C_MFMAS; ++i)
                {
                    c_read(1, i + AHEAD, ring);
                    c_mfma(1, i, ring);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };
    auto run = [&](int g, int g_next, auto buf_tag) __attribute__((always_inline))
    {
        if(EXPLICIT && !steps.is_open(g))
        {
            step(g, g_next, buf_tag, std::true_type{});
        }
        else
        {
            step(g, g_next, buf_tag, std::false_type{});
        }
    };
    while(g_cur >= 0)
    {
        int g_next = steps.next(g_cur);
        run(g_cur, g_next, std::integral_constant<int, 0>{});
        g_cur = g_next;
        if(g_cur < 0)
        {
            break;
        }
        g_next = steps.next(g_cur);
        run(g_cur, g_next, std::integral_constant<int, 1>{});
        g_cur = g_next;
    }
    // (the last step's spare loads into LDS must have landed before the
    // workgroup's LDS can be given away)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // ---- dQ (+)= scale acc: register r of block db is head value
    // db*32 + tile_row(r, half); four consecutive ones per 8-byte store ----------------
    if(!q_ok)
    {
        return;
    }
    const int lane_again = lane_index_again();
    const int my_q_again = q_row0 + wave_u * 32 + (lane_again & 31);
    const int half_again = lane_again >> 5;
    uint16_t *dst = static_cast<uint16_t *>(dQ_own) + row_elem(my_q_again, true) * HEAD;
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
#pragma unroll
        for(int rg = 0; rg < 4; ++rg)
        {
            uint16_t *ptr = dst + db * 32 + 8 * rg + 4 * half_again;
            float v[4];
#pragma unroll
            for(int e = 0; e < 4; ++e)
            {
                v[e] = acc[db][4 * rg + e] * p.scale;
            }
            if(!p.overwrite)
            {
                const u32x2 old = *reinterpret_cast<const u32x2 *>(ptr);
                v[0] += T::to_float((uint16_t)(old[0] & 0xffffu));
                v[1] += T::to_float((uint16_t)(old[0] >> 16));
                v[2] += T::to_float((uint16_t)(old[1] & 0xffffu));
                v[3] += T::to_float((uint16_t)(old[1] >> 16));
            }
            u32x2 out;
            out[0] = T::pack2(v[0], v[1]);
            out[1] = T::pack2(v[2], v[3]);
            *reinterpret_cast<u32x2 *>(ptr) = out;
        }
    }
}

// ---------------------------------------------------------------------------------
// PART says which gradient: K and V fragments plus both accumulators take 192
// registers of a lane at head 128, which leaves too few for two wavefronts
// per SIMD to run without spilling and without room to read operands ahead.
// One set of workgroups per gradient (dK: S, dP, dK^T; dV: S, dV^T - the
// scores are computed once more) fits two workgroups of 4 wavefronts on a CU.
enum { BWD_PART_DK = 1, BWD_PART_DV = 2 };
// Where one workgroup holds both gradients of its keys: at head sizes up to 64
// under every mask mode; at head 128 (K and V fragments and the two
// accumulators are 192 of a lane's 256 registers there) under the analytic
// modes, with the blocks of a step one after the other and a few registers
// spilled - 12 scratch accesses a step beside its 64 MFMAs.
#ifndef NNTILE_BWD_FUSED_KEYS_HEAD
#define NNTILE_BWD_FUSED_KEYS_HEAD 64
#endif
#ifndef NNTILE_BWD_GOFF_IN_LDS
#define NNTILE_BWD_GOFF_IN_LDS 1
#endif
#ifndef NNTILE_BWD_FUSED_ORDER
#define NNTILE_BWD_FUSED_ORDER 1      // 1: product by product at head 128; 0: S with dP, then dV with dK
#endif
#ifndef NNTILE_BWD_FUSED_KEYS_HEAD_ANALYTIC
#define NNTILE_BWD_FUSED_KEYS_HEAD_ANALYTIC 128
#endif
template<int HEAD, int MODE> constexpr bool kBwdFusedKeys = HEAD <= NNTILE_BWD_FUSED_KEYS_HEAD
    || (HEAD <= NNTILE_BWD_FUSED_KEYS_HEAD_ANALYTIC
            && (MODE == NNTILE_HIP_MASK_NONE || MODE == NNTILE_HIP_MASK_CAUSAL));
constexpr int kBwdCUs = 256;
constexpr int kDkvWaves = 4;
constexpr int kDkvThreads = kDkvWaves * 64;
constexpr int kDkvRows = kDkvWaves * 32;        // keys per workgroup

template<typename T, int HEAD, int MODE, int PART, bool GRID>
__device__ __forceinline__ void sdpa_bwd_dkv_body(
        const std::conditional_t<GRID, BwdGridParams, BwdParams> &p, unsigned wg,
        char *lds_q0, char *lds_q1, char *lds_g0, char *lds_g1,
        float (*lds_stat_arg)[2][kBwdStep])
{
    constexpr bool DO_DK = (PART & BWD_PART_DK) != 0, DO_DV = (PART & BWD_PART_DV) != 0;
    constexpr bool BOTH = DO_DK && DO_DV;
    BWD_TRACE_DECL
    typedef typename T::vec8 vec8;
    typedef BwdTile<HEAD> G;
    constexpr int KSTEPS = G::KSTEPS, DBLOCKS = G::DBLOCKS, RB = G::RB, CPR = G::CPR;
    constexpr int ROWS_PER_LOAD = G::ROWS_PER_LOAD;
    constexpr int LPW = G::LOADS >= kDkvWaves ? G::LOADS / kDkvWaves : 1;   // loads per loading wavefront
    constexpr int LOADERS = G::LOADS / LPW;                                  // wavefronts that load
    constexpr bool EXPLICIT = (MODE == NNTILE_HIP_MASK_ADDITIVE
            || MODE == NNTILE_HIP_MASK_BOOL);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int col = lane & 31;
    const int half = lane >> 5;

    const int q_seq = (int)p.q_seq, k_seq = (int)p.k_seq;
    const int k_blocks = (k_seq + kDkvRows - 1) / kDkvRows;
    // the first key blocks are seen by the most queries under a causal mask
    int kvb, k_block;                               // kvb = nb + n_batch*hkv
    int q_tile0 = 0, k_tile0 = 0;
    int64_t d_slab = 0;
    if constexpr(GRID)
    {
        const int kv_entries = p.batch / p.kv_group;
        map_workgroup(wg, kv_entries * p.n_slabs, k_blocks, false, kvb, k_block);
        if(p.n_slabs > 1)
        {
            const int slab = kvb / kv_entries;
            kvb -= slab * kv_entries;
            q_tile0 = slab * p.n_q_tiles;
            k_tile0 = slab * p.n_kv_tiles;
            d_slab = (int64_t)slab * p.q_seq * p.batch;
        }
    }
    else
    {
        map_workgroup(wg, p.batch / p.kv_group, k_blocks, false, kvb, k_block);
    }
    const int k_row0 = k_block * kDkvRows;
    const int nb = kvb % p.n_batch, hkv = kvb / p.n_batch;
    const int my_k = k_row0 + wave * 32 + col;
    const bool k_ok = my_k < k_seq;
    // key kg is visible to query q0 + qr + 4*half iff kg - 4*half <= rel + q0 + qr
    const int my_k_less_half = my_k - 4 * half;
    // the lane's key: its row within the allocation that holds it (of K, V, dK, dV)
    // (a function of the row, so that the stores at the end can work it out
    // again instead of keeping it through the loop)
    int own_t0 = 0, own_rows = k_seq;           // the tile that holds the block's rows
    if constexpr(GRID)
    {
        const int k_tile = (int)p.k_tile;
        own_t0 = __builtin_amdgcn_readfirstlane((k_row0 / k_tile) * k_tile);
        own_rows = min(k_tile, k_seq - own_t0);
    }
    auto row_elem = [&](int row, bool ok) __attribute__((always_inline)) -> int64_t
    {
        return (int64_t)kvb * own_rows + ((ok ? row : (GRID ? k_row0 : 0)) - own_t0);
    };
    const int64_t k_elem = row_elem(my_k, k_ok);
    const void *K_own = p.K, *V_own = p.V;
    void *dK_own = p.dK, *dV_own = p.dV;
    if constexpr(GRID)
    {
        const int k_tile = (int)p.k_tile;
        const int tk = k_row0 / k_tile;
        K_own = p.Kt[k_tile0 + tk];
        V_own = p.Vt[k_tile0 + tk];
        dK_own = p.dKt[k_tile0 + tk];
        dV_own = p.dVt[k_tile0 + tk];
    }
    const int64_t k_off = k_elem * HEAD;

    // K and V fragments (B operands): lane (col, half) holds head values 16*ks + 8*half..+7
    vec8 kf[KSTEPS], vf[KSTEPS];
    {
        const uint16_t *ks_ = static_cast<const uint16_t *>(K_own) + k_off + half * 8;
        const uint16_t *vs_ = static_cast<const uint16_t *>(V_own) + k_off + half * 8;
#pragma unroll
        for(int ks = 0; ks < KSTEPS; ++ks)
        {
            u32x4 k = *reinterpret_cast<const u32x4 *>(ks_ + ks * 16);
            u32x4 v = *reinterpret_cast<const u32x4 *>(vs_ + ks * 16);
            if(!k_ok)
            {
                k = u32x4{0, 0, 0, 0};
                v = u32x4{0, 0, 0, 0};
            }
            kf[ks] = __builtin_bit_cast(vec8, k);
            vf[ks] = __builtin_bit_cast(vec8, DO_DK ? v : u32x4{0, 0, 0, 0});
        }
    }

    // key row kg is visible to query row q iff kg <= rel + q (causal)
    int64_t rel64 = p.q_pos0 + p.causal_offset - p.k_pos0;
    rel64 = max((int64_t)-(1 << 30), min(rel64, (int64_t)(1 << 30)));
    const int rel = (int)rel64;
    const int n_steps = (q_seq + kBwdStep - 1) / kBwdStep;
    int first_step = 0;
    if(MODE == NNTILE_HIP_MASK_CAUSAL)
    {
        // the first query that sees the workgroup's first key
        const int q_lo = max(k_row0 - rel, 0);
        first_step = min(q_lo / kBwdStep, n_steps);
    }

    // (only the last step of the queries can be short: its rows past the end
    // read the last row that exists; the offsets of that step are kept beside
    // the others rather than computed per load)
    uint32_t ld_goff[LPW], ld_goff_end[LPW];
    const int ld_cpos = lane % CPR;
#pragma unroll
    for(int i = 0; i < LPW; ++i)
    {
        const int r = ((wave % LOADERS) * LPW + i) * ROWS_PER_LOAD + lane / CPR;
        ld_goff[i] = (uint32_t)(r * RB + (ld_cpos ^ G::swz(r)) * 16);
        ld_goff_end[i] = ld_goff[i] - (uint32_t)(max(r - (q_seq - 1) % kBwdStep, 0) * RB);
    }
    // Both gradients at head 128 leave no registers for these tables, and a
    // spilled entry is reloaded from scratch with a wait for every load in
    // flight, the next step's tile loads included: they go to LDS, whose reads
    // have a counter of their own.
    constexpr bool GOFF_IN_LDS = BOTH && HEAD > 64 && NNTILE_BWD_GOFF_IN_LDS != 0;
    // (the statistics of the two buffers behind them in the same array: one
    // register, the thread's place in the array, then addresses all of it)
    __shared__ __attribute__((aligned(16))) uint32_t lds_goff[GOFF_IN_LDS
        ? (2 * LPW + 1) * kDkvThreads : 1];
    static_assert(2 * 2 * kBwdStep <= kDkvThreads, "two buffers of statistics in one row of the table");
    float (*lds_stat)[2][kBwdStep] = GOFF_IN_LDS
        ? reinterpret_cast<float (*)[2][kBwdStep]>(lds_goff + 2 * LPW * kDkvThreads) : lds_stat_arg;
    if constexpr(GOFF_IN_LDS)
    {
#pragma unroll
        for(int i = 0; i < LPW; ++i)
        {
            lds_goff[i * kDkvThreads + tid] = ld_goff[i];
            lds_goff[(LPW + i) * kDkvThreads + tid] = ld_goff_end[i];
        }
        // (each thread reads back what it wrote: no barrier needed)
    }
    // row operand: lane (col, half) reads row mb*32+col, logical chunk 2*ks+half;
    // 32 rows further on the swizzle is the same, so mb goes into the immediate
    uint32_t row_raddr[KSTEPS];
#pragma unroll
    for(int ks = 0; ks < KSTEPS; ++ks)
    {
        row_raddr[ks] = (uint32_t)(col * RB + ((2 * ks + half) ^ G::swz(col)) * 16);
    }
    uint32_t tr_raddr[2][DBLOCKS];
    {
        const int i16 = lane & 15, dblk = (lane >> 4) & 1;
        const int j = i16 >> 2, r4 = i16 & 3;
#pragma unroll
        for(int a = 0; a < 2; ++a)
        {
            const int r = 4 * half + j + 8 * a;
#pragma unroll
            for(int db = 0; db < DBLOCKS; ++db)
            {
                const int c = 4 * db + 2 * dblk + (r4 >> 1);
                tr_raddr[a][db] = (uint32_t)(r * RB + (c ^ G::swz(r)) * 16 + 8 * (r4 & 1));
            }
        }
    }

    f32x16 dk[DBLOCKS], dv[DBLOCKS];
#pragma unroll
    for(int db = 0; db < DBLOCKS; ++db)
    {
#pragma unroll
        for(int r = 0; r < 16; ++r)
        {
            dk[db][r] = 0.0f;
            dv[db][r] = 0.0f;
        }
    }
    const float c = p.scale * kLog2e;
    // mask values: byte offsets of the lane's key within a row of the mask,
    // for the rows of the lower and of the upper half of the wave (the
    // launcher keeps 64 rows of the mask within 32 bits)
    constexpr uint32_t MASK_ES = MODE == NNTILE_HIP_MASK_ADDITIVE ? 2u : 1u;
    const uint32_t mask_row_bytes_wg = (uint32_t)p.mask_ld * MASK_ES;
    const uint32_t mask_off_lo = (uint32_t)(k_ok ? my_k : 0) * MASK_ES;
    const uint32_t mask_off_hi = mask_off_lo + (uint32_t)(4 * half) * mask_row_bytes_wg;
    // the workgroup's key blocks of 64 against the query blocks
    // first_step .. n_steps-1, once per head of the group: walk position
    // i = head * 64K + query step
    const StepSet steps = make_step_set(p, EXPLICIT, k_row0 / kBwdStep,
            min(kDkvRows / kBwdStep, (k_seq - k_row0 + kBwdStep - 1) / kBwdStep),
            first_step, n_steps, false);
    constexpr int kHeadStride = 1 << 16;
    auto locate = [&](int i, int &bq, int &qs)
    {
        const int g = i / kHeadStride;
        qs = i % kHeadStride;
        bq = nb + p.n_batch * (g + p.kv_group * hkv);
    };
    auto walk_begin = [&]() -> int
    {
        return steps.begin();       // head 0
    };
    auto walk_next = [&](int i) -> int
    {
        const int g = i / kHeadStride;
        const int nxt = steps.next(i % kHeadStride);
        if(nxt >= 0)
        {
            return g * kHeadStride + nxt;
        }
        const int b0 = steps.begin();
        return (g + 1 < p.kv_group && b0 >= 0) ? (g + 1) * kHeadStride + b0 : -1;
    };
    // loads of walk position i: the Q and dA rows straight into LDS, the
    // logsumexp and D of its queries through registers (threads 0..127)
    // (inside the loop the tile loads go between the MFMAs, one Q and one dA
    // load at a time: a wave stands still ~64 cycles per load)
    // the allocation that holds query row0 of entry bq, the row's index in it
    // (for lse; times HEAD for Q and dA) and in the row dots
    struct QueryRows
    {
        const void *Q, *dA;
        const float *lse;
        int64_t elem, d_idx;
    };
    auto query_rows = [&](int bq, int row0) __attribute__((always_inline)) -> QueryRows
    {
        if constexpr(GRID)
        {
            const int q_tile = (int)p.q_tile;
            const int tq = row0 / q_tile, t0 = tq * q_tile;
            const int64_t elem = (int64_t)bq * min(q_tile, q_seq - t0) + (row0 - t0);
            return QueryRows{p.Qt[q_tile0 + tq], p.dAt[q_tile0 + tq], p.lset[q_tile0 + tq], elem,
                d_slab + (int64_t)p.batch * t0 + elem};
        }
        else
        {
            const int64_t elem = (int64_t)bq * q_seq + row0;
            return QueryRows{p.Q, p.dA, p.lse, elem, elem};
        }
    };
    auto fetch_piece = [&](const QueryRows &at, bool at_end, char *qdst_base, char *gdst_base,
            int j) __attribute__((always_inline))
    {
        const char *Qp = static_cast<const char *>(at.Q) + at.elem * RB;
        const char *Gp = static_cast<const char *>(at.dA) + at.elem * RB;
        char *qdst = qdst_base + wave_u * LPW * 1024;
        char *gdst = gdst_base + wave_u * LPW * 1024;
        uint32_t goff;
        if constexpr(GOFF_IN_LDS)
        {
            goff = lds_goff[((at_end ? LPW : 0) + j) * kDkvThreads + tid];
        }
        else
        {
            goff = at_end ? ld_goff_end[j] : ld_goff[j];
        }
        load_to_lds16<0, false>(Qp, goff, qdst + j * 1024);
        load_to_lds16<0, false>(Gp, goff, gdst + j * 1024);
    };
    // The statistics of a step in two halves, so that the load's latency
    // passes behind the MFMAs of the step before: stat_load starts the read
    // of the thread's value (threads 0..63 a logsumexp, 64..127 a row dot),
    // stat_store turns it into what the step reads from LDS.
    auto stat_load = [&](const QueryRows &at, int last) __attribute__((always_inline)) -> float
    {
        float raw = 0.0f;
        if(tid < 2 * kBwdStep)
        {
            const int which = tid / kBwdStep, r = tid % kBwdStep;
            const float *src = which == 0 ? at.lse + at.elem : p.D + at.d_idx;
            raw = src[min(r, last)];
        }
        return raw;
    };
    auto stat_store = [&](float raw, int last, float (*stat)[kBwdStep])
        __attribute__((always_inline))
    {
        if(tid < 2 * kBwdStep)
        {
            const int which = tid / kBwdStep, r = tid % kBwdStep;
            float v;
            if(which == 0)
            {
                v = (r > last || raw == neg_inf()) ? __builtin_huge_valf() : raw * kLog2e;
            }
            else
            {
                v = r > last ? 0.0f : -raw;
            }
            (&stat[0][0])[tid] = v;        // = stat[which][r]
        }
    };
    auto fetch_stat = [&](const QueryRows &at, int last, float (*stat)[kBwdStep])
    {
        stat_store(stat_load(at, last), last, stat);
    };
    constexpr int FETCH_STRIDE = (NNTILE_BWD_SPREAD == 2 ? 2 : 1) * KSTEPS / LPW;
    static_assert(FETCH_STRIDE >= 1 && 1 + (LPW - 1) * FETCH_STRIDE < 2 * KSTEPS,
            "the pieces of a fetch must fit between the MFMAs of a step");
    auto fetch = [&](int i, char *qdst_base, char *gdst_base, float (*stat)[kBwdStep])
    {
        int bq, qs;
        locate(i, bq, qs);
        const int row0 = qs * kBwdStep;
        const int last = min(kBwdStep, q_seq - row0) - 1;
        const QueryRows at = query_rows(bq, row0);
        if(LOADERS == kDkvWaves || wave_u < LOADERS)
        {
#pragma unroll
            for(int j = 0; j < LPW; ++j)
            {
                fetch_piece(at, last + 1 < kBwdStep, qdst_base, gdst_base, j);
            }
        }
        fetch_stat(at, last, stat);
    };

    int i_cur = walk_begin();
    if(i_cur >= 0)
    {
        fetch(i_cur, lds_q0, lds_g0, lds_stat[0]);
    }
    BWD_WALL_AT(3);     // (developer trace: the workgroup is set up, its first tile requested)
    auto step = [&](int i, int i_next, auto buf_tag, auto masked_tag)
        __attribute__((always_inline))
    {
        constexpr int BUF = decltype(buf_tag)::value;
        const char *Qs = BUF ? lds_q1 : lds_q0;
        const char *Gs = BUF ? lds_g1 : lds_g0;
        const float (*stat)[kBwdStep] = lds_stat[BUF];
        BWD_TRACE_START();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        BWD_TRACE_MARK(0);
        BWD_TRACE_STEP();
        // the statistics of the next step now, its tiles between the MFMAs
        // below (the last step loads its own tiles once more, rather than
        // branch)
        int bq_f, qs_f;
        locate(i_next >= 0 ? i_next : i, bq_f, qs_f);
        const int row0_f = qs_f * kBwdStep;
        const int last_f = min(kBwdStep, q_seq - row0_f) - 1;
        const bool at_end_f = last_f + 1 < kBwdStep;
        // (wave-common, computed once here: the loads between the MFMAs below
        // only add their offsets)
        const QueryRows at_f = query_rows(bq_f, row0_f);
        float raw_next = 0.0f;
        if(i_next >= 0)
        {
            raw_next = stat_load(at_f, last_f);
            if(NNTILE_BWD_SPREAD == 0 && (LOADERS == kDkvWaves || wave_u < LOADERS))
            {
#pragma unroll
                for(int j = 0; j < LPW; ++j)
                {
                    fetch_piece(at_f, at_end_f, BUF ? lds_q0 : lds_q1,
                            BUF ? lds_g0 : lds_g1, j);
                }
            }
        }
        int bq, qs;
        locate(i, bq, qs);
        constexpr bool use_mask = EXPLICIT && decltype(masked_tag)::value;
        const int q0 = qs * kBwdStep;
        const int rows_here = min(kBwdStep, q_seq - q0);
        // (wave-common: the workgroup's last key against the last key that
        // exists and the last key the step's first query sees)
        const bool bounds = k_row0 + kDkvRows > k_seq
            || (MODE == NNTILE_HIP_MASK_CAUSAL && k_row0 + kDkvRows - 1 > rel + q0);
        // (the row stride through an empty asm statement: its multiples are
        // then computed where a step uses them - 32 scalar products - instead
        // of once before the loop and kept, which at head 128 means spilled)
        uint32_t mask_row_bytes = mask_row_bytes_wg;
        if(use_mask)
        {
            asm volatile("" : "+s"(mask_row_bytes));
        }
        const char *mask_step = static_cast<const char *>(p.mask)
            + (int64_t)q0 * (int64_t)mask_row_bytes;
        const uint32_t mask_last_row = (uint32_t)(rows_here - 1) * mask_row_bytes;

        if constexpr(!EXPLICIT && BOTH && HEAD > 64 && NNTILE_BWD_FUSED_ORDER == 1)
        {
            // Both gradients at head 128: 192 registers hold fragments and
            // accumulators, so a block goes product by product - S, P, dV, then
            // dP, dS, dK - and the probabilities in fp32 are all that crosses
            // from the first half to the second.
#pragma unroll
            for(int mb = 0; mb < 2; ++mb)
            {
                f32x16 sv;
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    sv[r] = 0.0f;
                }
#pragma unroll
                for(int ks = 0; ks < KSTEPS; ++ks)
                {
                    const vec8 qa = *reinterpret_cast<const vec8 *>(Qs + row_raddr[ks]
                            + mb * 32 * RB);
                    sv = T::mfma(qa, kf[ks], sv);
                    if(LOADERS == kDkvWaves || wave_u < LOADERS)
                    {
#pragma unroll
                        for(int j = 0; j < LPW; ++j)
                        {
                            if(NNTILE_BWD_SPREAD != 0 && mb * KSTEPS + ks == 1 + j * FETCH_STRIDE)
                            {
                                fetch_piece(at_f, at_end_f, BUF ? lds_q0 : lds_q1,
                                        BUF ? lds_g0 : lds_g1, j);
                            }
                        }
                    }
                }
                if(bounds)
                {
#pragma unroll
                    for(int r = 0; r < 16; ++r)
                    {
                        // (the lane's part on the left, the rest is wave-common)
                        const int qr = mb * 32 + tile_row(r, 0);
                        bool vis = k_ok;
                        if(MODE == NNTILE_HIP_MASK_CAUSAL)
                        {
                            vis = vis && (my_k_less_half <= rel + q0 + qr);
                        }
                        sv[r] = vis ? sv[r] : neg_inf();
                    }
                }
                // P in place of S
                uint32_t pk[8];
#pragma unroll
                for(int rg = 0; rg < 4; ++rg)
                {
                    const f32x4 lse4 = *reinterpret_cast<const f32x4 *>(
                            &stat[0][mb * 32 + 8 * rg + 4 * half]);
#pragma unroll
                    for(int e = 0; e < 4; ++e)
                    {
                        sv[4 * rg + e] = fast_exp2(fmaf(sv[4 * rg + e], c, -lse4[e]));
                    }
                }
#pragma unroll
                for(int k = 0; k < 8; ++k)
                {
                    pk[k] = T::pack2(sv[2 * k], sv[2 * k + 1]);
                }
                // dV^T += dA^T P
#pragma unroll
                for(int tt = 0; tt < 2; ++tt)
                {
                    const int t = 2 * mb + tt;
                    const u32x4 praw = {pk[4 * tt], pk[4 * tt + 1], pk[4 * tt + 2], pk[4 * tt + 3]};
                    const vec8 pb = __builtin_bit_cast(vec8, praw);
#pragma unroll
                    for(int db = 0; db < DBLOCKS; ++db)
                    {
                        const u32x2 glo = bwd_lds_read_tr16(Gs + tr_raddr[0][db] + (16 * t) * RB);
                        const u32x2 ghi = bwd_lds_read_tr16(Gs + tr_raddr[1][db] + (16 * t) * RB);
                        const u32x4 graw = {glo[0], glo[1], ghi[0], ghi[1]};
                        dv[db] = T::mfma(__builtin_bit_cast(vec8, graw), pb, dv[db]);
                    }
                }
                // dP - D
                f32x16 dpv;
#pragma unroll
                for(int rg = 0; rg < 4; ++rg)
                {
                    const f32x4 nd4 = *reinterpret_cast<const f32x4 *>(
                            &stat[1][mb * 32 + 8 * rg + 4 * half]);
#pragma unroll
                    for(int e = 0; e < 4; ++e)
                    {
                        dpv[4 * rg + e] = nd4[e];
                    }
                }
#pragma unroll
                for(int ks = 0; ks < KSTEPS; ++ks)
                {
                    const vec8 ga = *reinterpret_cast<const vec8 *>(Gs + row_raddr[ks]
                            + mb * 32 * RB);
                    dpv = T::mfma(ga, vf[ks], dpv);
                }
                // dS, in the registers of the packed P
#pragma unroll
                for(int k = 0; k < 8; ++k)
                {
                    pk[k] = T::pack2(sv[2 * k] * dpv[2 * k], sv[2 * k + 1] * dpv[2 * k + 1]);
                }
                // dK^T += Q^T dS
#pragma unroll
                for(int tt = 0; tt < 2; ++tt)
                {
                    const int t = 2 * mb + tt;
                    const u32x4 sraw = {pk[4 * tt], pk[4 * tt + 1], pk[4 * tt + 2], pk[4 * tt + 3]};
                    const vec8 sb = __builtin_bit_cast(vec8, sraw);
#pragma unroll
                    for(int db = 0; db < DBLOCKS; ++db)
                    {
                        const u32x2 qlo = bwd_lds_read_tr16(Qs + tr_raddr[0][db] + (16 * t) * RB);
                        const u32x2 qhi = bwd_lds_read_tr16(Qs + tr_raddr[1][db] + (16 * t) * RB);
                        const u32x4 qraw = {qlo[0], qlo[1], qhi[0], qhi[1]};
                        dk[db] = T::mfma(__builtin_bit_cast(vec8, qraw), sb, dk[db]);
                    }
                }
            }
        }
        else if constexpr(EXPLICIT || NNTILE_BWD_PIPE == 0 || (BOTH && HEAD > 64))
        {
            // (one 32-query block at a time: half the accumulators live)
            // ---- S = Q K^T, dP = dA V^T: rows are queries, the lane's column its key;
            // P, dS: register r of block mb is query q0 + mb*32 + tile_row(r, half) --------------
#pragma unroll
            for(int mb = 0; mb < 2; ++mb)
            {
                uint32_t p_pk[8], ds_pk[8];
                f32x16 sv, dpv;
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    sv[r] = 0.0f;
                    dpv[r] = 0.0f;
                }
                if(DO_DK)
                {
                    // dP - D: the accumulator starts at -D of its row (four
                    // consecutive queries per LDS read), the products add dP
#pragma unroll
                    for(int rg = 0; rg < 4; ++rg)
                    {
                        const f32x4 nd4 = *reinterpret_cast<const f32x4 *>(
                                &stat[1][mb * 32 + 8 * rg + 4 * half]);
#pragma unroll
                        for(int e = 0; e < 4; ++e)
                        {
                            dpv[4 * rg + e] = nd4[e];
                        }
                    }
                }
#pragma unroll
                for(int ks = 0; ks < KSTEPS; ++ks)
                {
                    const vec8 qa = *reinterpret_cast<const vec8 *>(Qs + row_raddr[ks] + mb * 32 * RB);
                    sv = T::mfma(qa, kf[ks], sv);
                    if(DO_DK)
                    {
                        const vec8 ga = *reinterpret_cast<const vec8 *>(Gs + row_raddr[ks]
                                + mb * 32 * RB);
                        dpv = T::mfma(ga, vf[ks], dpv);
                    }
                    if(LOADERS == kDkvWaves || wave_u < LOADERS)
                    {
#pragma unroll
                        for(int j = 0; j < LPW; ++j)
                        {
                            if(NNTILE_BWD_SPREAD != 0 && mb * KSTEPS + ks == 1 + j * FETCH_STRIDE)
                            {
                                fetch_piece(at_f, at_end_f, BUF ? lds_q0 : lds_q1,
                                        BUF ? lds_g0 : lds_g1, j);
                            }
                        }
                    }
                }
                // Keys past the end and pairs the causal mask hides: their scores
                // become -inf in a pass of their own, which only the workgroups at
                // the end of the keys and the steps on the diagonal run (a
                // wave-common branch).
                if(bounds)
                {
#pragma unroll
                    for(int r = 0; r < 16; ++r)
                    {
                        // (the lane's part on the left, the rest is wave-common)
                        const int qr = mb * 32 + tile_row(r, 0);
                        bool vis = k_ok;
                        if(MODE == NNTILE_HIP_MASK_CAUSAL)
                        {
                            vis = vis && (my_k_less_half <= rel + q0 + qr);
                        }
                        sv[r] = vis ? sv[r] : neg_inf();
                    }
                }
                float pv[16], dsv[16];
#pragma unroll
                for(int rg = 0; rg < 4; ++rg)
                {
                    // four consecutive queries: their statistics in one LDS read each
                    const int qr0 = mb * 32 + 8 * rg + 4 * half;
                    const f32x4 lse4 = *reinterpret_cast<const f32x4 *>(&stat[0][qr0]);
#pragma unroll
                    for(int e = 0; e < 4; ++e)
                    {
                        const int r = 4 * rg + e;
                        float ex = fmaf(sv[r], c, -lse4[e]);    // -inf: hidden, or a row past the end
                        bool visible = true;
                        if(use_mask)
                        {
                            // the row is the same for the lanes of one half: its
                            // address is wave-common, the lane adds its key (and
                            // four rows in the upper half, while those exist;
                            // rows past the end read a row that exists and are
                            // dropped by their logsumexp of +inf)
                            const int rb = mb * 32 + 8 * rg + e;
                            const char *mrow = mask_step
                                + min((uint32_t)rb * mask_row_bytes, mask_last_row);
                            const char *mp = mrow + (rb + 4 < rows_here ? mask_off_hi : mask_off_lo);
                            if(MODE == NNTILE_HIP_MASK_ADDITIVE)
                            {
                                const float add = T::to_float(
                                        *reinterpret_cast<const uint16_t *>(mp));
                                visible = visible && (add != neg_inf());
                                ex = fmaf(add, kLog2e, ex);
                            }
                            else
                            {
                                const uint8_t shown = *reinterpret_cast<const uint8_t *>(mp);
                            visible = visible && (shown != 0);
                            }
                        }
                        pv[r] = use_mask ? (visible ? fast_exp2(ex) : 0.0f) : fast_exp2(ex);
                        dsv[r] = pv[r] * dpv[r];
                    }
                }
#pragma unroll
                for(int k = 0; k < 8; ++k)
                {
                    p_pk[k] = T::pack2(pv[2 * k], pv[2 * k + 1]);
                    ds_pk[k] = T::pack2(dsv[2 * k], dsv[2 * k + 1]);
                }
                // ---- dV^T += dA^T P, dK^T += Q^T dS: the block's two sub-steps of 16 queries ----
#pragma unroll
                for(int tt = 0; tt < 2; ++tt)
                {
                    const int t = 2 * mb + tt;
                    const u32x4 praw = {p_pk[4 * tt], p_pk[4 * tt + 1], p_pk[4 * tt + 2],
                        p_pk[4 * tt + 3]};
                    const u32x4 sraw = {ds_pk[4 * tt], ds_pk[4 * tt + 1], ds_pk[4 * tt + 2],
                        ds_pk[4 * tt + 3]};
                    const vec8 pb = __builtin_bit_cast(vec8, praw);
                    const vec8 sb = __builtin_bit_cast(vec8, sraw);
#pragma unroll
                    for(int db = 0; db < DBLOCKS; ++db)
                    {
                        if(DO_DV)
                        {
                            const u32x2 glo = bwd_lds_read_tr16(Gs + tr_raddr[0][db] + (16 * t) * RB);
                            const u32x2 ghi = bwd_lds_read_tr16(Gs + tr_raddr[1][db] + (16 * t) * RB);
                            const u32x4 graw = {glo[0], glo[1], ghi[0], ghi[1]};
                            dv[db] = T::mfma(__builtin_bit_cast(vec8, graw), pb, dv[db]);
                        }
                        if(DO_DK)
                        {
                            const u32x2 qlo = bwd_lds_read_tr16(Qs + tr_raddr[0][db] + (16 * t) * RB);
                            const u32x2 qhi = bwd_lds_read_tr16(Qs + tr_raddr[1][db] + (16 * t) * RB);
                            const u32x4 qraw = {qlo[0], qlo[1], qhi[0], qhi[1]};
                            dk[db] = T::mfma(__builtin_bit_cast(vec8, qraw), sb, dk[db]);
                        }
                    }
                }
            }
        }
        else
        {
            // The step's two 32-query blocks in three phases each - A: S = Q K^T and
            // dP = dA V^T (rows are queries, the lane's column its key), B: P and dS
            // on the vector ALU, C: dV^T += dA^T P, dK^T += Q^T dS - issued as
            // A0 | A1 with B0 | C0 with B1 | C1, so that the matrix unit works
            // through a block's neighbours while the vector ALU turns its scores
            // into probabilities.  P, dS: register r of block mb is query
            // q0 + mb*32 + tile_row(r, half).
            f32x16 sv[2], dpv[2];
            uint32_t p_pk[2][8], ds_pk[2][8];
            // Keys past the end and pairs the causal mask hides: their scores
            // become -inf in a pass of their own, which only the workgroups at
            // the end of the keys and the steps on the diagonal run (a
            // wave-common branch).
            auto hide = [&](int mb) __attribute__((always_inline))
            {
                if(bounds)
                {
#pragma unroll
                    for(int r = 0; r < 16; ++r)
                    {
                        // (the lane's part on the left, the rest is wave-common)
                        const int qr = mb * 32 + tile_row(r, 0);
                        bool vis = k_ok;
                        if(MODE == NNTILE_HIP_MASK_CAUSAL)
                        {
                            vis = vis && (my_k_less_half <= rel + q0 + qr);
                        }
                        sv[mb][r] = vis ? sv[mb][r] : neg_inf();
                    }
                }
            };
            // The overlapped order, written out slot by slot (one MFMA, the operand
            // read of a later slot, a slice of the vector work) with a scheduling
            // barrier after each, or the compiler regroups it into phases.
            constexpr int A_MFMAS = (DO_DK ? 2 : 1) * KSTEPS, C_MFMAS = (BOTH ? 2 : 1) * 2 * DBLOCKS;
            constexpr int AHEAD = NNTILE_BWD_AHEAD;
            auto a_read = [&](int mb, int i, vec8 (&ring)[AHEAD + 1]) __attribute__((always_inline))
            {
                if(i >= A_MFMAS)
                {
                    return;
                }
                const int ks = DO_DK ? i / 2 : i;
                const char *src = (DO_DK && (i & 1)) ? Gs : Qs;
                ring[i % (AHEAD + 1)] = *reinterpret_cast<const vec8 *>(src + row_raddr[ks]
                        + mb * 32 * RB);
            };
            auto a_mfma = [&](int mb, int i, vec8 (&ring)[AHEAD + 1]) __attribute__((always_inline))
            {
                const int ks = DO_DK ? i / 2 : i;
                if(DO_DK && (i & 1))
                {
                    dpv[mb] = T::mfma(ring[i % (AHEAD + 1)], vf[ks], dpv[mb]);
                }
                else
                {
                    sv[mb] = T::mfma(ring[i % (AHEAD + 1)], kf[ks], sv[mb]);
                }
                // the tile loads of the next step, spread over the products
                if((LOADERS == kDkvWaves || wave_u < LOADERS) && NNTILE_BWD_SPREAD != 0
                        && (!DO_DK || (i & 1)))
                {
#pragma unroll
                    for(int j = 0; j < LPW; ++j)
                    {
                        if(mb * KSTEPS + ks == 1 + j * FETCH_STRIDE)
                        {
                            fetch_piece(at_f, at_end_f, BUF ? lds_q0 : lds_q1,
                                    BUF ? lds_g0 : lds_g1, j);
                        }
                    }
                }
            };
            auto a_init = [&](int mb) __attribute__((always_inline))
            {
#pragma unroll
                for(int r = 0; r < 16; ++r)
                {
                    sv[mb][r] = 0.0f;
                    dpv[mb][r] = 0.0f;
                }
                if(DO_DK)
                {
#pragma unroll
                    for(int rg = 0; rg < 4; ++rg)
                    {
                        const f32x4 nd4 = *reinterpret_cast<const f32x4 *>(
                                &stat[1][mb * 32 + 8 * rg + 4 * half]);
#pragma unroll
                        for(int e = 0; e < 4; ++e)
                        {
                            dpv[mb][4 * rg + e] = nd4[e];
                        }
                    }
                }
            };
            auto c_read = [&](int mb, int i, vec8 (&ring)[AHEAD + 1]) __attribute__((always_inline))
            {
                if(i >= C_MFMAS)
                {
                    return;
                }
                // (both gradients: dV and dK products alternate)
                const int j = BOTH ? i / 2 : i;
                const bool for_dv = BOTH ? (i & 1) == 0 : DO_DV;
                const int t = 2 * mb + j / DBLOCKS, db = j % DBLOCKS;
                const char *src = (for_dv ? Gs : Qs) + (16 * t) * RB;
                const u32x2 lo = bwd_lds_read_tr16(src + tr_raddr[0][db]);
                const u32x2 hi = bwd_lds_read_tr16(src + tr_raddr[1][db]);
                const u32x4 raw = {lo[0], lo[1], hi[0], hi[1]};
                ring[i % (AHEAD + 1)] = __builtin_bit_cast(vec8, raw);
            };
            auto c_mfma = [&](int mb, int i, vec8 (&ring)[AHEAD + 1]) __attribute__((always_inline))
            {
                const int j = BOTH ? i / 2 : i;
                const bool for_dv = BOTH ? (i & 1) == 0 : DO_DV;
                const int tt = j / DBLOCKS, db = j % DBLOCKS;
                const uint32_t (&pk)[8] = for_dv ? p_pk[mb] : ds_pk[mb];
                const u32x4 braw = {pk[4 * tt], pk[4 * tt + 1], pk[4 * tt + 2], pk[4 * tt + 3]};
                if(for_dv)
                {
                    dv[db] = T::mfma(ring[i % (AHEAD + 1)], __builtin_bit_cast(vec8, braw), dv[db]);
                }
                else
                {
                    dk[db] = T::mfma(ring[i % (AHEAD + 1)], __builtin_bit_cast(vec8, braw), dk[db]);
                }
            };
            // vector work of query r of block mb (statistics of four queries per
            // LDS read, read one group ahead)
            f32x4 lse_cur = {0.0f, 0.0f, 0.0f, 0.0f}, lse_nxt = lse_cur;
            float pv_even = 0.0f, ds_even = 0.0f;
            auto b_begin = [&](int mb) __attribute__((always_inline))
            {
                lse_nxt = *reinterpret_cast<const f32x4 *>(&stat[0][mb * 32 + 4 * half]);
            };
            // (in three stages a tick apart - exponent, exponential, products and
            // packing - so that a lone wavefront does not wait for its own
            // results: tick t takes query t, t-1 and t-2 through one stage each)
            float ex_stage[2] = {0.0f, 0.0f}, pr_stage[2] = {0.0f, 0.0f};
            auto b_tick = [&](int mb, int t) __attribute__((always_inline))
            {
                if(t - 2 >= 0 && t - 2 < 16)
                {
                    const int r = t - 2;
                    const float pr = pr_stage[r % 2];
                    const float dsr = pr * dpv[mb][r];
                    if(r % 2 == 0)
                    {
                        pv_even = pr;
                        ds_even = dsr;
                    }
                    else
                    {
                        if(DO_DV)
                        {
                            p_pk[mb][r / 2] = T::pack2(pv_even, pr);
                            asm volatile("" : "+v"(p_pk[mb][r / 2]));
                        }
                        if(DO_DK)
                        {
                            ds_pk[mb][r / 2] = T::pack2(ds_even, dsr);
                            asm volatile("" : "+v"(ds_pk[mb][r / 2]));
                        }
                    }
                }
                if(t - 1 >= 0 && t - 1 < 16)
                {
                    const int r = t - 1;
                    pr_stage[r % 2] = fast_exp2(ex_stage[r % 2]);
                }
                if(t < 16)
                {
                    const int r = t;
                    if(r % 4 == 0)
                    {
                        lse_cur = lse_nxt;
                        if(r + 4 < 16)
                        {
                            lse_nxt = *reinterpret_cast<const f32x4 *>(
                                    &stat[0][mb * 32 + 8 * (r / 4 + 1) + 4 * half]);
                        }
                    }
                    ex_stage[r % 2] = fmaf(sv[mb][r], c, -lse_cur[r % 4]);
                }
            };
            constexpr int B_TICKS = 18;
            {
                vec8 ring[AHEAD + 1];
                // A0
                a_init(0);
#pragma unroll
                for(int i = 0; i < AHEAD; ++i)
                {
                    a_read(0, i, ring);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(int i = 0; i < A_MFMAS; ++i)
                {
                    a_read(0, i + AHEAD, ring);
                    a_mfma(0, i, ring);
                    __builtin_amdgcn_sched_barrier(0);
                }
                BWD_TRACE_MARK(1);
                hide(0);
                // A1 with B0
                a_init(1);
                b_begin(0);
#pragma unroll
                for(int i = 0; i < AHEAD; ++i)
                {
                    a_read(1, i, ring);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(int i = 0; i < A_MFMAS; ++i)
                {
                    a_read(1, i + AHEAD, ring);
                    a_mfma(1, i, ring);
#pragma unroll
                    for(int t = i * B_TICKS / A_MFMAS; t < (i + 1) * B_TICKS / A_MFMAS; ++t)
                    {
                        b_tick(0, t);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                BWD_TRACE_MARK(2);
                hide(1);
                // C0 with B1
                b_begin(1);
#pragma unroll
                for(int i = 0; i < AHEAD; ++i)
                {
                    c_read(0, i, ring);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(int i = 0; i < C_MFMAS; ++i)
                {
                    c_read(0, i + AHEAD, ring);
                    c_mfma(0, i, ring);
#pragma unroll
                    for(int t = i * B_TICKS / C_MFMAS; t < (i + 1) * B_TICKS / C_MFMAS; ++t)
                    {
                        b_tick(1, t);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                BWD_TRACE_MARK(3);
                // C1
#pragma unroll
                for(int i = 0; i < AHEAD; ++i)
                {
                    c_read(1, i, ring);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(int i = 0; i < C_MFMAS; ++i)
                {
                    c_read(1, i + AHEAD, ring);
                    c_mfma(1, i, ring);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        BWD_TRACE_MARK(4);
        // (the other buffer's readers passed this step's barrier; the next
        // step's barrier orders these writes before its reads)
        __builtin_amdgcn_sched_barrier(0);
        if(i_next >= 0)
        {
            stat_store(raw_next, last_f, lds_stat[BUF ^ 1]);
        }
        BWD_TRACE_MARK(5);
    };
    auto run = [&](int i, int i_next, auto buf_tag) __attribute__((always_inline))
    {
        if(EXPLICIT && !steps.is_open(i % kHeadStride))
        {
            step(i, i_next, buf_tag, std::true_type{});
        }
        else
        {
            step(i, i_next, buf_tag, std::false_type{});
        }
    };
    while(i_cur >= 0)
    {
        int i_next = walk_next(i_cur);
        run(i_cur, i_next, std::integral_constant<int, 0>{});
        i_cur = i_next;
        if(i_cur < 0)
        {
            break;
        }
        i_next = walk_next(i_cur);
        run(i_cur, i_next, std::integral_constant<int, 1>{});
        i_cur = i_next;
    }
    // (the last step's spare loads into LDS must have landed before the
    // workgroup's LDS can be given away)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    BWD_TRACE_FLUSH(PART);
    // ---- dK (+)= scale dk, dV (+)= dv -------------------------------------------------
    if(!k_ok)
    {
        return;
    }
    const int lane_again = lane_index_again();
    const int my_k_again = k_row0 + wave_u * 32 + (lane_again & 31);
    const int half_again = lane_again >> 5;
    const int64_t k_off_again = row_elem(my_k_again, true) * HEAD;
    auto store = [&](void *base, const f32x16 (&acc)[DBLOCKS], float factor)
    {
        uint16_t *dst = static_cast<uint16_t *>(base) + k_off_again;
#pragma unroll
        for(int db = 0; db < DBLOCKS; ++db)
        {
#pragma unroll
            for(int rg = 0; rg < 4; ++rg)
            {
                uint16_t *ptr = dst + db * 32 + 8 * rg + 4 * half_again;
                float v[4];
#pragma unroll
                for(int e = 0; e < 4; ++e)
                {
                    v[e] = acc[db][4 * rg + e] * factor;
                }
                if(!p.overwrite)
                {
                    const u32x2 old = *reinterpret_cast<const u32x2 *>(ptr);
                    v[0] += T::to_float((uint16_t)(old[0] & 0xffffu));
                    v[1] += T::to_float((uint16_t)(old[0] >> 16));
                    v[2] += T::to_float((uint16_t)(old[1] & 0xffffu));
                    v[3] += T::to_float((uint16_t)(old[1] >> 16));
                }
                u32x2 out;
                out[0] = T::pack2(v[0], v[1]);
                out[1] = T::pack2(v[2], v[3]);
                *reinterpret_cast<u32x2 *>(ptr) = out;
            }
        }
    };
    if(DO_DK)
    {
        store(dK_own, dk, p.scale);
    }
    if(DO_DV)
    {
        store(dV_own, dv, 1.0f);
    }
}

// One launch for the three gradients: workgroups [0, n_dkv) compute dK,
// the next n_dq dQ (three products a step each, the longer workgroups), the
// last n_dkv dV.  A tile-pair call has fewer workgroups per gradient than the
// chip has places (two a CU); together they fill it, and a long call loses
// the ends of two launches.
template<typename T, int HEAD, int MODE, bool GRID, bool FUSED_KEYS = false>
__global__ __launch_bounds__(kDkvThreads, 2)
void sdpa_bwd_kernel(const std::conditional_t<GRID, BwdGridParams, BwdParams> p, unsigned n_dkv,
        unsigned n_dq)
{
    BWD_WALL(0, blockIdx.x < n_dkv ? 1 : (blockIdx.x < n_dkv + n_dq ? 0 : 2));
    typedef BwdTile<HEAD> G;
    static_assert(kDkvThreads == kBwdThreads, "one block size for the three parts");
    __shared__ __attribute__((aligned(1024))) char lds_0[G::BYTES];
    __shared__ __attribute__((aligned(1024))) char lds_1[G::BYTES];
    __shared__ __attribute__((aligned(1024))) char lds_2[G::BYTES];
    __shared__ __attribute__((aligned(1024))) char lds_3[G::BYTES];
    // dK, dV parts, per query of a step: logsumexp in log2 units (+inf for a
    // row that saw nothing) and minus the row dot D; rows past the end hold +inf / 0
    __shared__ __attribute__((aligned(16))) float lds_stat[2][2][kBwdStep];
    if constexpr(FUSED_KEYS)
    {
        // (K and V fragments and both accumulators fit beside the rest: one
        // set of key-owning workgroups computes dK and dV from one pass over
        // the scores, seven products a call instead of eight)
        if(blockIdx.x < n_dkv)
        {
            sdpa_bwd_dkv_body<T, HEAD, MODE, BWD_PART_DK | BWD_PART_DV, GRID>(p, blockIdx.x, lds_0,
                    lds_1, lds_2, lds_3, lds_stat);
        }
        else
        {
            sdpa_bwd_dq_body<T, HEAD, MODE, GRID>(p, blockIdx.x - n_dkv, lds_0, lds_1, lds_2, lds_3);
        }
    }
    else if(blockIdx.x < n_dkv)
    {
        sdpa_bwd_dkv_body<T, HEAD, MODE, BWD_PART_DK, GRID>(p, blockIdx.x, lds_0, lds_1, lds_2,
                lds_3, lds_stat);
    }
    else if(blockIdx.x < n_dkv + n_dq)
    {
        sdpa_bwd_dq_body<T, HEAD, MODE, GRID>(p, blockIdx.x - n_dkv, lds_0, lds_1, lds_2, lds_3);
    }
    else
    {
        sdpa_bwd_dkv_body<T, HEAD, MODE, BWD_PART_DV, GRID>(p, blockIdx.x - n_dkv - n_dq, lds_0,
                lds_1, lds_2, lds_3, lds_stat);
    }
#ifdef NNTILE_BWD_TRACE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    BWD_WALL(1, blockIdx.x < n_dkv ? 1 : (blockIdx.x < n_dkv + n_dq ? 0 : 2));
#endif
}

template<typename T, int HEAD, int MODE>
static int launch_bwd_mode(hipStream_t stream, const BwdParams &p)
{
    const int64_t q_blocks = (p.q_seq + kBwdRows - 1) / kBwdRows;
    const int64_t k_blocks = (p.k_seq + kDkvRows - 1) / kDkvRows;
    const int64_t kv_batch = p.batch / p.kv_group;
    const int64_t n_dq = (int64_t)p.batch * q_blocks, n_dkv = kv_batch * k_blocks;
    if(n_dq <= 0 || n_dkv <= 0 || n_dq > 0x3fffffff || n_dkv > 0x3fffffff
            || (int64_t)p.batch * p.q_seq * (HEAD / 8) / 256 > 0x7ffffffe)
    {
        return NNTILE_HIP_EINVAL;
    }
    if((MODE == NNTILE_HIP_MASK_ADDITIVE || MODE == NNTILE_HIP_MASK_BOOL)
            && p.mask_class != nullptr)
    {
        const int64_t n_cls = ((p.q_seq + kBwdStep - 1) / kBwdStep) * p.class_ld;
        hipLaunchKernelGGL((sdpa_bwd_mask_classes_kernel<T, MODE>), dim3((unsigned)n_cls),
                dim3(256), 0, stream, p.mask, p.mask_ld, (int)p.q_seq, (int)p.k_seq,
                const_cast<uint8_t *>(p.mask_class), p.class_ld);
        if(hipGetLastError() != hipSuccess)
        {
            return NNTILE_HIP_ELAUNCH;
        }
    }
    const int64_t rows = (int64_t)p.batch * p.q_seq;
    hipLaunchKernelGGL((sdpa_bwd_rowdot_kernel<T, HEAD>),
            dim3((unsigned)((rows * (HEAD / 8) + 255) / 256)), dim3(256), 0, stream, p.dA, p.A,
            p.D, rows);
    if(hipGetLastError() != hipSuccess)
    {
        return NNTILE_HIP_ELAUNCH;
    }
    if constexpr(kBwdFusedKeys<HEAD, MODE>)
    {
        // One set of key-owning workgroups for both gradients (seven products
        // instead of eight) once the three sets would not all be resident at
        // the same time; below that the longest workgroup sets the time, and
        // the separate sets have the shorter ones.
        if(2 * n_dkv + n_dq > 2 * kBwdCUs)
        {
            hipLaunchKernelGGL((sdpa_bwd_kernel<T, HEAD, MODE, false, true>),
                    dim3((unsigned)(n_dkv + n_dq)), dim3(kDkvThreads), 0, stream, p,
                    (unsigned)n_dkv, (unsigned)n_dq);
            return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
        }
    }
    hipLaunchKernelGGL((sdpa_bwd_kernel<T, HEAD, MODE, false>),
            dim3((unsigned)(2 * n_dkv + n_dq)), dim3(kDkvThreads), 0, stream, p,
            (unsigned)n_dkv, (unsigned)n_dq);
    return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
}

// The grid form: the row dots tile by tile (each tile's A and dA are one
// allocation, and D follows the layout of lse), then the one gradient launch.
template<typename T, int HEAD, int MODE>
static int launch_bwd_grid_mode(hipStream_t stream, const BwdGridParams &p,
        const void *const *A_tiles, int n_q_tiles)
{
    const int64_t q_blocks = (p.q_seq + kBwdRows - 1) / kBwdRows;
    const int64_t k_blocks = (p.k_seq + kDkvRows - 1) / kDkvRows;
    const int64_t kv_batch = p.batch / p.kv_group * p.n_slabs;
    const int64_t n_dq = (int64_t)p.batch * p.n_slabs * q_blocks, n_dkv = kv_batch * k_blocks;
    if(n_dq <= 0 || n_dkv <= 0 || n_dq > 0x3fffffff || n_dkv > 0x3fffffff
            || (int64_t)p.batch * p.q_tile * (HEAD / 8) / 256 > 0x7ffffffe)
    {
        return NNTILE_HIP_EINVAL;
    }
    for(int s = 0; s < p.n_slabs; ++s)
    {
        for(int t = 0; t < n_q_tiles; ++t)
        {
            const int64_t t0 = (int64_t)t * p.q_tile;
            const int64_t rows = (int64_t)p.batch
                * (p.q_tile < p.q_seq - t0 ? p.q_tile : p.q_seq - t0);
            hipLaunchKernelGGL((sdpa_bwd_rowdot_kernel<T, HEAD>),
                    dim3((unsigned)((rows * (HEAD / 8) + 255) / 256)), dim3(256), 0, stream,
                    p.dAt[s * n_q_tiles + t], A_tiles[s * n_q_tiles + t],
                    p.D + (int64_t)s * p.q_seq * p.batch + (int64_t)p.batch * t0, rows);
            if(hipGetLastError() != hipSuccess)
            {
                return NNTILE_HIP_ELAUNCH;
            }
        }
    }
    if constexpr(kBwdFusedKeys<HEAD, MODE>)
    {
        // One set of key-owning workgroups for both gradients (seven products
        // instead of eight) once the three sets would not all be resident at
        // the same time; below that the longest workgroup sets the time, and
        // the separate sets have the shorter ones.
        if(2 * n_dkv + n_dq > 2 * kBwdCUs)
        {
            hipLaunchKernelGGL((sdpa_bwd_kernel<T, HEAD, MODE, true, true>),
                    dim3((unsigned)(n_dkv + n_dq)), dim3(kDkvThreads), 0, stream, p,
                    (unsigned)n_dkv, (unsigned)n_dq);
            return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
        }
    }
    hipLaunchKernelGGL((sdpa_bwd_kernel<T, HEAD, MODE, true>),
            dim3((unsigned)(2 * n_dkv + n_dq)), dim3(kDkvThreads), 0, stream, p,
            (unsigned)n_dkv, (unsigned)n_dq);
    return hipGetLastError() == hipSuccess ? NNTILE_HIP_OK : NNTILE_HIP_ELAUNCH;
}

template<typename T, int HEAD>
static int launch_bwd_grid_head(hipStream_t stream, const BwdGridParams &p,
        const void *const *A_tiles, int n_q_tiles, int mode)
{
    switch(mode)
    {
        case NNTILE_HIP_MASK_NONE:
            return launch_bwd_grid_mode<T, HEAD, NNTILE_HIP_MASK_NONE>(stream, p, A_tiles,
                    n_q_tiles);
        case NNTILE_HIP_MASK_CAUSAL:
            return launch_bwd_grid_mode<T, HEAD, NNTILE_HIP_MASK_CAUSAL>(stream, p, A_tiles,
                    n_q_tiles);
        default:
            return NNTILE_HIP_EINVAL;
    }
}

// The caller has checked: every tile but the last of an axis holds q_tile /
// k_tile rows, both multiples of 128 unless the axis is one tile.
template<typename T>
int launch_bwd_grid_16bit(hipStream_t stream, const BwdGridParams &p,
        const void *const *A_tiles, int n_q_tiles, int head, int mode)
{
    switch(head)
    {
        case 32:
            return launch_bwd_grid_head<T, 32>(stream, p, A_tiles, n_q_tiles, mode);
        case 64:
            return launch_bwd_grid_head<T, 64>(stream, p, A_tiles, n_q_tiles, mode);
        case 128:
            return launch_bwd_grid_head<T, 128>(stream, p, A_tiles, n_q_tiles, mode);
        default:
            return NNTILE_HIP_EUNSUPPORTED;
    }
}

template int launch_bwd_grid_16bit<Bf16>(hipStream_t, const BwdGridParams &, const void *const *,
        int, int, int);
template int launch_bwd_grid_16bit<Fp16>(hipStream_t, const BwdGridParams &, const void *const *,
        int, int, int);

template<typename T, int HEAD>
static int launch_bwd_head(hipStream_t stream, const BwdParams &p, int mode)
{
    switch(mode)
    {
        case NNTILE_HIP_MASK_ADDITIVE:
            return launch_bwd_mode<T, HEAD, NNTILE_HIP_MASK_ADDITIVE>(stream, p);
        case NNTILE_HIP_MASK_NONE:
            return launch_bwd_mode<T, HEAD, NNTILE_HIP_MASK_NONE>(stream, p);
        case NNTILE_HIP_MASK_CAUSAL:
            return launch_bwd_mode<T, HEAD, NNTILE_HIP_MASK_CAUSAL>(stream, p);
        case NNTILE_HIP_MASK_BOOL:
            return launch_bwd_mode<T, HEAD, NNTILE_HIP_MASK_BOOL>(stream, p);
        default:
            return NNTILE_HIP_EINVAL;
    }
}

template<typename T>
int launch_bwd_16bit(hipStream_t stream, const BwdParams &p, int head, int mode)
{
    switch(head)
    {
        case 32:
            return launch_bwd_head<T, 32>(stream, p, mode);
        case 64:
            return launch_bwd_head<T, 64>(stream, p, mode);
        case 128:
            return launch_bwd_head<T, 128>(stream, p, mode);
        default:
            return NNTILE_HIP_EUNSUPPORTED;
    }
}

template int launch_bwd_16bit<Bf16>(hipStream_t, const BwdParams &, int, int);
template int launch_bwd_16bit<Fp16>(hipStream_t, const BwdParams &, int, int);

} // namespace nntile_hip
