// Shared device-side definitions of the gfx950 attention kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/nntile_hip_sdpa.h"

// Developer hook: a diagnostic build may define these to record cycle counters
// at the phase boundaries of a kernel's main loop; they expand to nothing in
// the library.
#ifndef NNTILE_PHASE
#define NNTILE_PHASE(n)
#define NNTILE_PHASE_DUMP()
#endif
#ifndef PHASE_DECL
#define PHASE_DECL
#endif

namespace nntile_hip
{

constexpr int kMaxTiles = NNTILE_HIP_SDPA_MAX_TILES;
#ifndef NNTILE_DEC_KEYS
#define NNTILE_DEC_KEYS 64
#endif
constexpr int kDecKeys = NNTILE_DEC_KEYS;    // keys per step of the decode kernel
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// Kernel arguments of the prefill kernels (passed by value in the kernarg
// segment).  Query tile t holds rows [t*q_tile, min((t+1)*q_tile, q_seq)),
// the same for key tiles.
// Key ranges a mask is scanned in by mask_step_bits_kernel
constexpr int kMaskBitSplits = 8;

struct PrefillParams
{
    int64_t q_seq, k_seq, q_tile, k_tile;
    int64_t q_pos0, k_pos0, causal_offset;
    int64_t mask_ld;              // = k_seq of the single key tile (explicit masks)
    int64_t kv_rows;              // rows between two entries of K and V; 0: the tile's own rows
                                  // (a cache's capacity, single key tile only)
    const void *mask;
    // explicit masks, one query tile: what a scan of the mask rows of every
    // 128-query block found, written by mask_step_bits_kernel before the
    // launch - kMaskBitSplits pairs of 64-bit words per block (one pair per
    // range of keys, to be OR-ed): bit s of the first word: some value of
    // 64-key step s is not "open", of the second: not "hidden" (steps from 63
    // on share bit 63).  Null: every workgroup scans its own rows.
    unsigned long long *mask_bits;
    // The scan riding in the attention launch (n_scan_wgs > 0): the first
    // n_scan_wgs workgroups of the grid do the scan and publish, per (block,
    // key range), the two words and then a flag word holding mask_tag (unique
    // to the call); the attention workgroups wait for the flags of their block,
    // at most mask_spin_limit ticks of the 100 MHz clock (then they scan their
    // own rows).  Three words per (block, key range) in either form.
    unsigned long long mask_tag, mask_spin_limit;
    int32_t n_q_tiles, n_kv_tiles;
    int32_t n_slabs;              // slabs of `batch` entries each in this launch; slab s's tiles sit at
                                  // [s*n_q_tiles + t] / [s*n_kv_tiles + t] of the tables below
    int32_t batch, n_batch, kv_group;
    int32_t q_blocks_per_tile;    // ceil(q_tile / rows per workgroup)
    int32_t k_blocks_per_tile;    // ceil(k_tile / keys per step)
    int32_t xcd_remap;            // 1: regroup workgroups so a slab stays on one XCD
    int32_t overwrite;            // 1: ignore the running pair, write every row
    int32_t n_scan_wgs;
    int32_t form;                 // fp32 launcher: 0 pick by size, 1 shared key steps, 2 split key steps
                                  // 16-bit launcher: 0 pick by size, 1 128-query workgroups, 2 the same with the key steps split over two groups of wavefronts, 8 256-query
    float scale;                  // 1/sqrt(head)
    const void *K[kMaxTiles];
    const void *V[kMaxTiles];
    const void *Q[kMaxTiles];
    float *lse[kMaxTiles];
    void *A[kMaxTiles];
};

// Kernel arguments of the decode kernels.  K, V: [head, k_seq, n_batch,
// n_head_kv]; Q, A: [head, q_seq, n_batch, kv_group, n_head_kv].
struct DecodeParams
{
    int64_t q_seq, k_seq;
    int64_t kv_rows;    // rows between two entries of K and V (k_seq, or a cache's capacity)
    int64_t q_pos0, k_pos0, causal_offset;
    int64_t mask_ld;
    const void *mask;
    const void *K, *V, *Q;
    float *lse;
    void *A;
    float *part_o;      // [unit][split][rows][HEAD], fp32 or (normalised) in the tile type
    float *part_ml;     // [unit][split][rows][2]
    int32_t n_batch, kv_group, n_head_kv;
    int32_t rows;       // kv_group * q_seq
    int32_t n_splits, steps_per_split, n_steps;
    int32_t overwrite;
    float scale;
    // Merge inside the main launch (fused != 0): the grid holds n_main main
    // workgroups followed by merge_blocks_per_unit merge workgroups per unit.
    // sync: per unit sync_stride 64-bit words - word 0 is reserved, word
    // 1 + rb*n_splits + s is the flag that split s raises for merge workgroup
    // rb of the unit (the launch's tag; the merge workgroup sets it back to 0).
    unsigned long long *sync;
    unsigned long long tag;         // unique per call, never 0
    unsigned long long spin_limit;  // longest wait for a flag, in 100 MHz ticks
    int32_t fused, fenced;
    int32_t n_main, merge_blocks_per_unit, sync_stride;
    // The append riding in the launch (n_new > 0): K and V are caches whose
    // rows [k_seq - n_new, k_seq) of every entry have not been written yet;
    // they are k_new / v_new ([entry][n_new][head]).  The main workgroups read
    // those rows from k_new / v_new, and n_append workgroups at the end of the
    // grid (one per unit) copy them into the caches for the calls to come.
    const void *k_new, *v_new;
    int32_t n_new, n_append;
};

// Kernel arguments of the backward kernels.  K, V, dK, dV: [head, k_seq,
// n_batch, n_head_kv]; Q, A, dA, dQ: [head, q_seq, n_batch, kv_group,
// n_head_kv]; lse and the row dots D = sum_h dA*A: [q_seq, batch] fp32.
struct BwdParams
{
    int64_t q_seq, k_seq;
    int64_t q_pos0, k_pos0, causal_offset;
    int64_t mask_ld;
    const void *mask;
    const void *K, *Q, *V, *A, *dA;
    const float *lse;
    float *D;               // workspace: the row dots dA . A, written before the gradient launch
    // explicit masks: class of every 64 x 64 block of the mask, row = query
    // block, class_ld entries per row (0 mixed, 1 nothing masked, 2 all
    // hidden); null when the workspace has no room for it
    const uint8_t *mask_class;
    int32_t class_ld;
    void *dK, *dQ, *dV;
    int32_t batch, n_batch, kv_group;
    int32_t overwrite;      // 1: write the gradients, 0: add to what is there
    float scale;
};

// The same over a grid of separately allocated tiles along the two sequence
// axes (analytic masks only): tile t of the query axis holds rows
// [t*q_tile, min((t+1)*q_tile, q_seq)) of every batch entry, an entry's rows
// contiguous inside it; likewise the key axis.  The single pointers of the
// base are unused; D holds the row dots tile after tile in the layout of lse.
constexpr int kBwdMaxTiles = NNTILE_HIP_SDPA_BWD_MAX_TILES;
struct BwdGridParams : BwdParams
{
    int64_t q_tile, k_tile;
    // slabs of `batch` entries each: slab s's tiles sit at [s*n_q_tiles + t] /
    // [s*n_kv_tiles + t] of the tables, its row dots at D + s*q_seq*batch
    int32_t n_slabs, n_q_tiles, n_kv_tiles;
    const void *Kt[kBwdMaxTiles];
    const void *Vt[kBwdMaxTiles];
    const void *Qt[kBwdMaxTiles];
    const void *dAt[kBwdMaxTiles];
    const float *lset[kBwdMaxTiles];
    void *dKt[kBwdMaxTiles];
    void *dQt[kBwdMaxTiles];
    void *dVt[kBwdMaxTiles];
};

// 16 bytes per lane from global memory straight into LDS: lane l reads
// gaddr + OFF (its own address) and its bytes land at lds_dst + OFF + 16*l
// (lds_dst is the same for the whole wavefront; it travels in M0).  Written
// as assembly text on purpose: the compiler takes the builtin form for an
// access that may touch both memories, and while one is in flight it turns
// every wait for an LDS read into a wait for all LDS reads, which undoes
// reading operands ahead of their use.  The caller waits (vmcnt) and
// synchronises before anyone reads the target; nothing else here uses M0.
#ifndef NNTILE_DMA_NT_BITS
#define NNTILE_DMA_NT_BITS "nt"     // cache-policy bits of the streaming (NT) form
#endif
template<int OFF, bool NT>
__device__ __forceinline__ void load_to_lds16(const void *gaddr, char *lds_dst)
{
    typedef char __attribute__((address_space(3))) *lds_ptr;
    const uint32_t base = (uint32_t)(uintptr_t)(lds_ptr)lds_dst;
    if(NT)
    {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                "global_load_lds_dwordx4 %1, off offset:%2 " NNTILE_DMA_NT_BITS
                :: "s"(base), "v"(gaddr), "n"(OFF) : "memory");
    }
    else
    {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                "global_load_lds_dwordx4 %1, off offset:%2"
                :: "s"(base), "v"(gaddr), "n"(OFF) : "memory");
    }
}

// The same with the address as a base common to the wavefront plus a 32-bit
// offset per lane (no 64-bit address arithmetic on the vector unit).
template<int OFF, bool NT>
__device__ __forceinline__ void load_to_lds16(const void *gbase_in, uint32_t lane_off,
        char *lds_dst)
{
    typedef char __attribute__((address_space(3))) *lds_ptr;
    const uint32_t base = (uint32_t)(uintptr_t)(lds_ptr)lds_dst;
    // (the base is the same in every lane; this makes the compiler see it)
    const uint64_t g64 = reinterpret_cast<uint64_t>(gbase_in);
    // (the builtin returns a signed int: widen it as unsigned, or a set bit 31
    // of the low half would fill the high half)
    const uint32_t g_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)g64);
    const uint32_t g_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(g64 >> 32));
    const uint64_t g_uni = (uint64_t)g_lo | ((uint64_t)g_hi << 32);
    const void *gbase = reinterpret_cast<const void *>(g_uni);
    if(NT)
    {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                "global_load_lds_dwordx4 %1, %2 offset:%3 " NNTILE_DMA_NT_BITS
                :: "s"(base), "v"(lane_off), "s"(gbase), "n"(OFF) : "memory");
    }
    else
    {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                "global_load_lds_dwordx4 %1, %2 offset:%3"
                :: "s"(base), "v"(lane_off), "s"(gbase), "n"(OFF) : "memory");
    }
}

__device__ __forceinline__ float fast_exp2(float x)
{
    return __builtin_amdgcn_exp2f(x);
}

__device__ __forceinline__ float neg_inf()
{
    return -__builtin_huge_valf();
}

// Storage <-> float for the 16-bit tile types.
struct Bf16
{
    typedef bf16x8 vec8;
    static constexpr uint32_t kNegInfPair = 0xFF80FF80u;    // two -inf values
    static __device__ __forceinline__ float to_float(uint16_t v)
    {
        return __uint_as_float(static_cast<uint32_t>(v) << 16);
    }
    static __device__ __forceinline__ uint16_t from_float(float f)
    {
        __bf16 h = static_cast<__bf16>(f);   // round to nearest even
        return __builtin_bit_cast(uint16_t, h);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
        typedef __attribute__((ext_vector_type(2))) float f32x2;
        f32x2 v = {lo, hi};
        bf16x2 h = __builtin_convertvector(v, bf16x2);
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    // acc + lo + hi of a packed pair, in fp32
    static __device__ __forceinline__ float add_pair(uint32_t packed, float acc)
    {
        typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
        const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
        return __builtin_amdgcn_fdot2_f32_bf16(
                __builtin_bit_cast(bf16x2, packed), ones, acc, false);
    }
};

struct Fp16
{
    typedef f16x8 vec8;
    static constexpr uint32_t kNegInfPair = 0xFC00FC00u;    // two -inf values
    static __device__ __forceinline__ float to_float(uint16_t v)
    {
        return static_cast<float>(__builtin_bit_cast(_Float16, v));
    }
    static __device__ __forceinline__ uint16_t from_float(float f)
    {
        _Float16 h = static_cast<_Float16>(f);
        return __builtin_bit_cast(uint16_t, h);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
        typedef __attribute__((ext_vector_type(2))) float f32x2;
        f32x2 v = {lo, hi};
        f16x2 h = __builtin_convertvector(v, f16x2);
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float add_pair(uint32_t packed, float acc)
    {
        typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
        const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, packed), ones,
                acc, false);
    }
};

// max(x, value of x in lane ^ 32): v_permlane32_swap exchanges the upper half
// of one register with the lower half of another without going through LDS.
__device__ __forceinline__ float max_across_halves(float x)
{
    typedef __attribute__((ext_vector_type(2))) uint32_t pair;
    const uint32_t u = __float_as_uint(x);
    const pair r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// (No inline assembly on values that an MFMA may have produced: the wait
// states between an MFMA's write and a VALU read are only inserted for real
// instructions, not for assembly text.)
__device__ __forceinline__ float max3(float a, float b, float c)
{
    return fmaxf(fmaxf(a, b), c);
}

// max(m, x, value of x in lane ^ 32)
__device__ __forceinline__ float max_with_other_half(float m, float x)
{
    typedef __attribute__((ext_vector_type(2))) uint32_t pair;
    const uint32_t u = __float_as_uint(x);
    const pair r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return max3(m, __uint_as_float(r[0]), __uint_as_float(r[1]));
}

__device__ __forceinline__ float sum_across_halves(float x)
{
    typedef __attribute__((ext_vector_type(2))) uint32_t pair;
    const uint32_t u = __float_as_uint(x);
    const pair r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Key/value batch entry read by query batch entry b.
__device__ __forceinline__ int kv_entry(int b, int n_batch, int kv_group)
{
    return (b % n_batch) + n_batch * (b / (n_batch * kv_group));
}

// Merge of a fresh (lse_new, value) into the running pair, per row:
// returns the weights and the merged lse.  lse_new must be finite.
__device__ __forceinline__ void merge_weights(float lse_old, float lse_new,
        float &w_old, float &w_new, float &lse_out)
{
    if(lse_old == neg_inf())
    {
        w_old = 0.0f;
        w_new = 1.0f;
        lse_out = lse_new;
        return;
    }
    const float top = fmaxf(lse_old, lse_new);
    const float e_old = __expf(lse_old - top), e_new = __expf(lse_new - top);
    const float sum = e_old + e_new;
    const float inv = 1.0f / sum;
    w_old = e_old * inv;
    w_new = e_new * inv;
    lse_out = top + __logf(sum);
}

} // namespace nntile_hip
