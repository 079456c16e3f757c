// Global -> LDS tile staging and the flag-driven tile lists shared by the
// forward and backward kernels.
#pragma once
#include "bam_common.h"
#include "bam_launch.h"

namespace bam {

// LDS byte address of a __shared__ object (what the LDS-DMA base register M0 wants).
__device__ __forceinline__ unsigned lds_addr(const void* p) {
    return (unsigned)(unsigned long long)(const __attribute__((address_space(3))) void*)p;
}

// One direct global -> LDS copy instruction.  Lane l fetches `bytes` (16 or 4) from
// sbase + voff and the hardware writes them to LDS byte address lds_base + l * bytes;
// sbase and lds_base must be wave-uniform.  The LDS base travels in M0: it is handed to the asm
// statement as an input operand bound to that register, so the compiler writes M0 itself and knows
// it is occupied; the s_nop is the wait state the hardware wants between an M0 write and its use.  Issued as inline asm on purpose: the compiler
// then neither tracks the copy in vmcnt nor makes later LDS reads wait for it, which is what
// lets a tile load stay in flight across a whole loop iteration.  The price is that the
// caller owns the synchronization: wait_async() (or wait_async_but<N>()) + a workgroup
// barrier before anyone reads the destination.
// SITE only labels the instruction (as an assembler comment): copies issued from different places of a
// kernel get different labels, which keeps the compiler from merging them into one hoisted copy and so
// keeps each where the schedule wants it.
template <int SITE = 0>
__device__ __forceinline__ void dma_b128(const void* sbase, unsigned voff, unsigned lds_base) {
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 ; site %3" ::"v"(voff), "s"(sbase), "{m0}"(lds_base),
                 "n"(SITE)
                 : "memory");
}
template <int SITE = 0>
__device__ __forceinline__ void dma_b32(const void* sbase, unsigned voff, unsigned lds_base) {
    asm volatile("s_nop 0\n\tglobal_load_lds_dword %0, %1 ; site %3" ::"v"(voff), "s"(sbase), "{m0}"(lds_base),
                 "n"(SITE)
                 : "memory");
}

// All direct global-to-LDS copies this wave has issued have landed (pair with a barrier).
__device__ __forceinline__ void wait_async() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// ROWS x D tile of 2-byte elements copied global -> LDS by THREADS threads, 16 bytes per lane.
// Full tiles use the direct global-to-LDS load (no staging registers, no LDS write
// instructions): a wave's 64 lanes fill 64 consecutive chunk slots of the LDS tile, so the
// XOR swizzle is applied on the SOURCE side -- lane `id` fetches the chunk that belongs in
// slot `id`.  `setup` fixes those source offsets once per kernel; `issue(i, ...)` emits copy
// instruction i of CPT so that callers can spread a tile's copies between other work.
// The last, ragged tile of a sequence takes the synchronous path (`load_ragged`), which
// zero-fills the rows past the end.  Row strides are limited to 2^23 elements by the host
// checks, so the offsets fit 32 bits.
template <int D, int ROWS, int THREADS>
struct TileStage {
    static constexpr int NCH = D / 8;
    static constexpr int CHUNKS = ROWS * NCH;
    static constexpr int CPT = (CHUNKS + THREADS - 1) / THREADS;
    static constexpr bool EXACT = (CHUNKS % THREADS) == 0;
    unsigned goff[CPT];
    int wave_first;  // first chunk slot this wave fills with instruction 0

    __device__ __forceinline__ void setup(int64_t row_stride_bytes, int tid) {
        wave_first = __builtin_amdgcn_readfirstlane(tid & ~63);
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int id = tid + THREADS * i;
            const int row = id / NCH, pc = id % NCH;
            goff[i] = (unsigned)(row * row_stride_bytes + (pc ^ swz<D>(row)) * 16);
        }
    }
    // tile_base: first row of the tile in global memory, tile_lds: lds_addr() of the LDS tile
    // (both wave-uniform)
    template <int SITE = 0>
    __device__ __forceinline__ void issue(int i, const char* tile_base, unsigned tile_lds) const {
        if (EXACT || wave_first + THREADS * i < CHUNKS)
            dma_b128<SITE>(tile_base, goff[i], tile_lds + (unsigned)(THREADS * i + wave_first) * 16u);
    }
    __device__ __forceinline__ void load_full(const char* tile_base, unsigned tile_lds) const {
#pragma unroll
        for (int i = 0; i < CPT; ++i) issue(i, tile_base, tile_lds);
    }
    // synchronous, zero-filling copy of a tile with only rows_valid (< ROWS) rows in range
    __device__ __forceinline__ void load_ragged(const char* tile_base, u32x4* tile, int rows_valid, int tid) const {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int id = tid + THREADS * i;
            u32x4 z = {0u, 0u, 0u, 0u};
            if ((EXACT || id < CHUNKS) && id / NCH < rows_valid) z = *(const u32x4*)(tile_base + goff[i]);
            if (EXACT || id < CHUNKS) tile[id] = z;
        }
    }
    // tile_base / rows_valid wave-uniform
    __device__ __forceinline__ void load(const char* tile_base, u32x4* tile, int rows_valid, int tid) const {
        if (rows_valid >= ROWS)
            load_full(tile_base, lds_addr(tile));
        else
            load_ragged(tile_base, tile, rows_valid, tid);
    }
};

// One wave copies `DWORDS` consecutive dwords (a multiple of 64) global -> LDS asynchronously.
template <int DWORDS>
__device__ __forceinline__ void copy_dwords_async(const void* src, void* dst_lds, int lane) {
    const unsigned dst = lds_addr(dst_lds);
#pragma unroll
    for (int i = 0; i < DWORDS / 64; ++i) dma_b32(src, (unsigned)(lane * 4 + 256 * i), dst + 256u * i);
}

// List, in ascending order, the 64-key tiles a 128-row query block has to visit.
// entry = (tile << 2) | cls ; cls 1: evaluate the mask, cls 2: every pair allowed.
// A tile is "full" only when both of its 32-column flags say so AND it has no column past
// the end of the sequence (those columns must still be masked out of the softmax).
// Executed by wave 0; the caller synchronizes before reading.
__device__ __forceinline__ void build_key_tile_list(const int8_t* flag_row, int num_n, int S, int lane,
                                                    int* list, int* count_out) {
    const int nkt = (S + 63) >> 6;
    int count = 0;
    for (int base = 0; base < nkt; base += 64) {
        const int kt = base + lane;
        int cls = 0;
        if (kt < nkt) {
            const int f0 = flag_row[2 * kt];
            const int f1 = (2 * kt + 1 < num_n) ? flag_row[2 * kt + 1] : 0;
            if (f0 > 0 || f1 > 0) cls = (f0 == 2 && f1 == 2 && (kt + 1) * 64 <= S) ? 2 : 1;
        }
        const unsigned long long bal = __ballot(cls != 0);
        if (cls) list[count + __popcll(bal & ((1ull << lane) - 1ull))] = (kt << 2) | cls;
        count += __popcll(bal);
    }
    if (lane == 0) *count_out = count;
}

// List the 128-row query blocks that have work for a 128-key tile (4 flag columns).
// entry = (m << 8) | cls0 | cls1 << 2 | cls2 << 4 | cls3 << 6, cls_w = flag of key column w.
__device__ __forceinline__ void build_query_block_list(const int8_t* flags_b, int64_t flags_sm, int num_m,
                                                       int num_n, int nt, int lane, int* list,
                                                       int* count_out) {
    int count = 0;
    for (int base = 0; base < num_m; base += 64) {
        const int m = base + lane;
        int packed = 0;
        if (m < num_m) {
            const int8_t* f = flags_b + (int64_t)m * flags_sm + 4 * nt;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const int fw = (4 * nt + w < num_n) ? f[w] : 0;
                packed |= (fw & 3) << (2 * w);
            }
        }
        const unsigned long long bal = __ballot(packed != 0);
        if (packed) list[count + __popcll(bal & ((1ull << lane) - 1ull))] = (m << 8) | packed;
        count += __popcll(bal);
    }
    if (lane == 0) *count_out = count;
}

}  // namespace bam
