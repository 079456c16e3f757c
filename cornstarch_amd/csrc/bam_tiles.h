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
// The same with the non-temporal hint: data that is read once (it should not displace what other workgroups re-read
// from the L2).
template <int SITE = 0>
__device__ __forceinline__ void dma_b128_stream(const void* sbase, unsigned voff, unsigned lds_base) {
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt ; site %3" ::"v"(voff), "s"(sbase), "{m0}"(lds_base),
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

// All LDS accesses this wave has issued are complete.  The compiler puts this wait in front of a barrier by itself --
// except, as the generated code showed, in front of a barrier at the head of a loop that is reached over the back
// edge with LDS stores still in flight (the list rebuilt for the next pass over a long sequence: other waves then
// read the old count or old entries).  So whoever writes LDS ahead of such a barrier states the wait.
__device__ __forceinline__ void wait_lds() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

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

// 64-row tile made of two 32-row slices that sit anywhere in global memory: LDS rows [0, 32) come from slice
// `lo`, rows [32, 64) from slice `hi` (the LDS layout is that of TileStage<D, 64, THREADS>).  Every copy
// instruction of a wave covers 64 / (D / 8) <= 16 consecutive rows starting at a multiple of that, so it stays
// inside one slice and only its (wave-uniform) base pointer depends on which.
template <int D, int THREADS>
struct SliceStage {
    static constexpr int NCH = D / 8;
    static constexpr int CHUNKS = 64 * NCH;
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
            goff[i] = (unsigned)((row & 31) * row_stride_bytes + (pc ^ swz<D>(row)) * 16);
        }
    }
    // lo / hi: first row of the two slices in global memory, tile_lds: lds_addr() of the LDS tile (wave-uniform)
    template <int SITE = 0>
    __device__ __forceinline__ void issue(int i, const char* lo, const char* hi, unsigned tile_lds) const {
        if (EXACT || wave_first + THREADS * i < CHUNKS) {
            const bool upper = (wave_first + THREADS * i) / NCH >= 32;
            dma_b128<SITE>(upper ? hi : lo, goff[i], tile_lds + (unsigned)(THREADS * i + wave_first) * 16u);
        }
    }
    // Does copy instruction i of this wave fill LDS rows 32..63 (slice `hi`)?  Wave-uniform, and a compile-time
    // constant where every instruction covers whole 32-row halves (D = 128 with 512 threads).
    __device__ __forceinline__ bool upper(int i) const {
        if ((THREADS * (i + 1)) / NCH <= 32) return false;
        if ((THREADS * i) / NCH >= 32) return true;
        return (wave_first + THREADS * i) / NCH >= 32;
    }
    // As issue(), with the slice's base pointer already chosen by the caller (see upper()).
    template <int SITE = 0>
    __device__ __forceinline__ void issue_from(int i, const char* slice_base, unsigned tile_lds) const {
        if (EXACT || wave_first + THREADS * i < CHUNKS)
            dma_b128<SITE>(slice_base, goff[i], tile_lds + (unsigned)(THREADS * i + wave_first) * 16u);
    }
    // synchronous, zero-filling copy of ONE slice with only rows_valid (<= 32) rows in range into LDS rows
    // [0, 32); rows [32, 64) are zeroed
    __device__ __forceinline__ void load_ragged(const char* slice_base, u32x4* tile, int rows_valid, int tid) const {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int id = tid + THREADS * i;
            u32x4 z = {0u, 0u, 0u, 0u};
            if ((EXACT || id < CHUNKS) && id / NCH < rows_valid) z = *(const u32x4*)(slice_base + goff[i]);
            if (EXACT || id < CHUNKS) tile[id] = z;
        }
    }
};

// One wave copies `DWORDS` consecutive dwords (a multiple of 64) global -> LDS asynchronously.
template <int DWORDS>
__device__ __forceinline__ void copy_dwords_async(const void* src, void* dst_lds, int lane) {
    const unsigned dst = lds_addr(dst_lds);
#pragma unroll
    for (int i = 0; i < DWORDS / 64; ++i) dma_b32(src, (unsigned)(lane * 4 + 256 * i), dst + 256u * i);
}

// The 32-row slice each of the four waves of a forward / dQ workgroup works on, and the row of tile classes
// (one byte per 32-key column tile: 0 empty, 1 partial, 2 full) that says which keys that slice needs.
// Without a plan the workgroup is a 128-row block in natural order and every wave reads the block's flag row;
// with one, group `grp` takes the next four slices of the sorted order and every slice has a class row of its own.
struct WaveSlices {
    int slice[4];             // -1: no slice (the wave idles through the key loop)
    const int8_t* cls_row[4]; // null where slice is -1
};

__device__ __forceinline__ WaveSlices pick_wave_slices(const AttnParams& p, int b, int grp) {
    WaveSlices w;
    if (p.fine != nullptr) {
        const int* ord = p.order + (int64_t)b * p.order_sb + 4 * grp;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            w.slice[x] = ord[x];
            w.cls_row[x] = w.slice[x] >= 0
                               ? (const int8_t*)p.fine + (int64_t)b * p.fine_sb + (int64_t)w.slice[x] * p.fine_ss
                               : nullptr;
        }
    } else {
        const int m = p.num_m - 1 - grp;  // late query blocks (most keys under causality) first
        const int8_t* row = p.flags + (int64_t)b * p.flags_sb + (int64_t)m * p.flags_sm;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            w.slice[x] = 4 * m + x;
            w.cls_row[x] = row;
        }
    }
    return w;
}

// List, in ascending order, the 64-key tiles the four slices of a workgroup have to visit, among the (at most
// MAX_LIST) tiles starting at tile kt_begin; longer sequences are walked in several passes.
// entry = (tile << 8) | c0 | c1 << 2 | c2 << 4 | c3 << 6 ; c_w is the class of the tile for wave w's slice:
// 0 nothing to do, 1 evaluate the mask, 2 every pair allowed.
// A tile is "full" for a slice only when both of its 32-column classes say so AND it has no column past
// the end of the sequence (those columns must still be masked out of the softmax).
// Executed by wave 0; the caller synchronizes before reading.
__device__ __forceinline__ void build_key_tile_list(const WaveSlices& ws, int num_n, int S, int lane, int kt_begin,
                                                    int* list, int* count_out) {
    const int nkt = min((S + 63) >> 6, kt_begin + MAX_LIST);
    int count = 0;
    for (int base = kt_begin; base < nkt; base += 64) {
        const int kt = base + lane;
        int packed = 0;
        if (kt < nkt) {
            const bool second = 2 * kt + 1 < num_n, inside = (kt + 1) * 64 <= S;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                if (ws.cls_row[x] == nullptr) continue;  // wave-uniform
                const int f0 = ws.cls_row[x][2 * kt];
                const int f1 = second ? ws.cls_row[x][2 * kt + 1] : 0;
                int cls = 0;
                if (f0 > 0 || f1 > 0) cls = (f0 == 2 && f1 == 2 && inside) ? 2 : 1;
                packed |= cls << (2 * x);
            }
        }
        const unsigned long long bal = __ballot(packed != 0);
        if (packed) list[count + __popcll(bal & ((1ull << lane) - 1ull))] = (kt << 8) | packed;
        count += __popcll(bal);
    }
    if (lane == 0) *count_out = count;
    wait_lds();
}

// List, in ascending order, the 32-row slices among [s_begin, s_end) (at most MAX_SLICE_LIST of them; longer
// sequences are walked in several passes) that have work for a 128-key tile (4 class columns).
// entry = (slice << 8) | c0 | c1 << 2 | c2 << 4 | c3 << 6, c_w = class of (slice, key column 4 nt + w).
// With a plan the classes are those of the 32 x 32 tiles; without one a slice inherits the flags of its
// 128-row block.
__device__ __forceinline__ void build_slice_list(const AttnParams& p, int b, int nt, int lane, int s_begin, int s_end,
                                                 int* list, int* count_out) {
    const int ns = s_end;
    int count = 0;
    for (int base = s_begin; base < ns; base += 64) {
        const int s = base + lane;
        int packed = 0;
        if (s < ns) {
            const int8_t* f = p.fine != nullptr
                                  ? (const int8_t*)p.fine + (int64_t)b * p.fine_sb + (int64_t)s * p.fine_ss + 4 * nt
                                  : p.flags + (int64_t)b * p.flags_sb + (int64_t)(s >> 2) * p.flags_sm + 4 * nt;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const int fw = (4 * nt + w < p.num_n) ? f[w] : 0;
                packed |= (fw & 3) << (2 * w);
            }
        }
        const unsigned long long bal = __ballot(packed != 0);
        if (packed) list[count + __popcll(bal & ((1ull << lane) - 1ull))] = (s << 8) | packed;
        count += __popcll(bal);
    }
    // list[-1] (the caller leaves room for it) repeats the first entry with all classes cleared: a consumer that
    // takes the entries in pairs from the end finds a harmless partner for the first entry of an odd count there.
    if (lane == 0) {
        *count_out = count;
        if (count > 0) list[-1] = list[0] & ~0xFF;
    }
    wait_lds();
}

}  // namespace bam
