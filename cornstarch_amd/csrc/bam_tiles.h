// Global -> register -> LDS tile staging and the flag-driven tile lists shared by the
// forward and backward kernels.
#pragma once
#include "bam_common.h"
#include "bam_launch.h"

namespace bam {

// ROWS x D tile of 2-byte elements moved by THREADS threads, 16 bytes per access.  `load`
// only issues the global reads (rows past `S` read zeros); `store` writes the registers
// into the swizzled LDS tile, so the two can be separated by a whole tile of MFMA work.
template <int D, int ROWS, int THREADS>
struct TileStage {
    static constexpr int NCH = D / 8;
    static constexpr int CHUNKS = ROWS * NCH;
    static constexpr int CPT = (CHUNKS + THREADS - 1) / THREADS;
    u32x4 r[CPT];

    __device__ __forceinline__ void load(const char* base, int64_t row_stride_bytes, int row0, int S, int tid) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int id = tid + THREADS * i;
            const int row = id / NCH, c = id % NCH;
            const int grow = row0 + row;
            u32x4 z = {0u, 0u, 0u, 0u};
            if ((CHUNKS % THREADS == 0 || id < CHUNKS) && grow < S)
                z = *(const u32x4*)(base + (int64_t)grow * row_stride_bytes + c * 16);
            r[i] = z;
        }
    }
    __device__ __forceinline__ void store(u32x4* tile, int tid) const {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int id = tid + THREADS * i;
            const int row = id / NCH, c = id % NCH;
            if (CHUNKS % THREADS == 0 || id < CHUNKS) tile[chunk_slot<D>(row, c)] = r[i];
        }
    }
};

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
