// Global -> register -> LDS tile staging and the flag-driven tile lists shared by the
// forward and backward kernels.
#pragma once
#include "bam_common.h"
#include "bam_launch.h"

namespace bam {

// ROWS x D tile of 2-byte elements copied global -> LDS by THREADS threads, 16 bytes per lane.
// Full tiles use the direct global-to-LDS load (no staging registers, no LDS write
// instructions): a wave's 64 lanes fill 64 consecutive chunk slots of the LDS tile, so the
// XOR swizzle is applied on the SOURCE side -- lane `id` fetches the chunk that belongs in
// slot `id`.  `setup` fixes those source offsets once per kernel.  The copy is asynchronous:
// the caller waits with wait_async() and a workgroup barrier before anyone reads the tile.
// The last, ragged tile of a sequence takes the synchronous path, which zero-fills the rows
// past the end.  Row strides are limited to 2^24 elements by the host checks, so the
// offsets fit 32 bits.
template <int D, int ROWS, int THREADS>
struct TileStage {
    static constexpr int NCH = D / 8;
    static constexpr int CHUNKS = ROWS * NCH;
    static constexpr int CPT = (CHUNKS + THREADS - 1) / THREADS;
    static constexpr bool EXACT = (CHUNKS % THREADS) == 0;
    unsigned goff[CPT];

    __device__ __forceinline__ void setup(int64_t row_stride_bytes, int tid) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int id = tid + THREADS * i;
            const int row = id / NCH, pc = id % NCH;
            goff[i] = (unsigned)(row * row_stride_bytes + (pc ^ swz<D>(row)) * 16);
        }
    }
    // tile_base: first row of the tile in global memory (wave-uniform); rows_valid: rows of it
    // inside the sequence (wave-uniform)
    __device__ __forceinline__ void load(const char* tile_base, u32x4* tile, int rows_valid, int tid) const {
        typedef __attribute__((address_space(1))) const void* gptr;
        typedef __attribute__((address_space(3))) void* lptr;
        if (rows_valid >= ROWS) {
            const int wave_first = __builtin_amdgcn_readfirstlane(tid & ~63);
#pragma unroll
            for (int i = 0; i < CPT; ++i)
                if (EXACT || wave_first + THREADS * i < CHUNKS)
                    __builtin_amdgcn_global_load_lds((gptr)(tile_base + goff[i]),
                                                     (lptr)(tile + THREADS * i + wave_first), 16, 0, 0);
        } else {
#pragma unroll
            for (int i = 0; i < CPT; ++i) {
                const int id = tid + THREADS * i;
                u32x4 z = {0u, 0u, 0u, 0u};
                if ((EXACT || id < CHUNKS) && id / NCH < rows_valid) z = *(const u32x4*)(tile_base + goff[i]);
                if (EXACT || id < CHUNKS) tile[id] = z;
            }
        }
    }
};

// One wave copies `DWORDS` consecutive dwords (a multiple of 64) global -> LDS asynchronously.
template <int DWORDS>
__device__ __forceinline__ void copy_dwords_async(const void* src, void* dst_lds, int lane) {
    typedef __attribute__((address_space(1))) const void* gptr;
    typedef __attribute__((address_space(3))) void* lptr;
#pragma unroll
    for (int i = 0; i < DWORDS / 64; ++i)
        __builtin_amdgcn_global_load_lds((gptr)((const unsigned*)src + 64 * i + lane),
                                         (lptr)((unsigned*)dst_lds + 64 * i), 4, 0, 0);
}

// All direct global-to-LDS copies this wave has issued have landed (pair with a barrier).
__device__ __forceinline__ void wait_async() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

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
