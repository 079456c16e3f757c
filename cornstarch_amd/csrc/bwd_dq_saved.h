// dQ from saved dS: the second half of the backward that does NOT recompute S and dP for dQ.
// Reference semantics: cornstarch/kernel/bitfield_attention.py:877-898 (ds rounded to the input dtype, dq += ds k); the
// reference adds every 128 x 32 tile's contribution to dq with fp32 atomics, here the dK/dV kernel (SAVE form) leaves
// its 32 x 32 blocks of -dS / scale in a workspace and this kernel, which owns whole query rows, sums them up:
// dQ^T = K^T dS^T over the key tiles that have work for the slice.  One GEMM instead of three, no exponentials, no
// mask logic (masked pairs were stored as zeros); the price is reading the workspace once.
//
// Work decomposition: as the forward -- a workgroup is four 32-row slices of one (batch, q head), one per wave (taken
// from the plan's slice order), and walks the 64-key tiles any of them needs; K tiles are shared through LDS (double
// buffered), every wave copies its own dS blocks (two 2 KiB blocks per tile, one per 32-key half) into a wave-private
// LDS area, two tiles ahead: a buffer is refilled as soon as its operands are in registers.  Both MFMA operands come
// from transposing LDS reads: K^T (d x keys) from the row-major K tile, dS^T (keys x rows) from the block, which the
// dK/dV lanes wrote key by key.
#pragma once
#include "bam_common.h"
#include "bam_launch.h"
#include "bam_tiles.h"
#include <type_traits>

namespace bam {

constexpr int DQS_KT = 64;
constexpr int DQS_THREADS = 256;

// List, in ascending order, the 64-key tiles the four slices of a workgroup have to visit (at most MAX_LIST).
// entry = (tile << 16) | sum_w (c0_w | c1_w << 2) << (4 w), c0 / c1 = class of the tile's two 32-key halves for wave
// w's slice.  Executed by wave 0; the caller synchronizes before reading.
__device__ __forceinline__ void build_key_half_list(const WaveSlices& ws, int num_n, int S, int lane, int* list,
                                                    int* count_out) {
    const int nkt = (S + 63) >> 6;
    int count = 0;
    for (int base = 0; base < nkt; base += 64) {
        const int kt = base + lane;
        int packed = 0;
        if (kt < nkt) {
            const bool second = 2 * kt + 1 < num_n;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                if (ws.cls_row[x] == nullptr) continue;  // wave-uniform
                const int f0 = ws.cls_row[x][2 * kt] & 3;
                const int f1 = second ? (ws.cls_row[x][2 * kt + 1] & 3) : 0;
                packed |= (f0 | (f1 << 2)) << (4 * x);
            }
        }
        const unsigned long long bal = __ballot(packed != 0);
        if (packed) list[count + __popcll(bal & ((1ull << lane) - 1ull))] = (kt << 16) | packed;
        count += __popcll(bal);
    }
    if (lane == 0) *count_out = count;
    wait_lds();
}

// Transposed MFMA operand out of a dS block: 32 keys x 32 columns of 2 bytes, 64 bytes per key, no swizzle.  The lane
// gets column colbase16 + (lane & 15) of keys row0 + {0,1,2,3} and row0 + 8 + {0,1,2,3} (row0 includes 4 * hi).
__device__ __forceinline__ u32x4 ds_block_read_transposed(const char* block, int lane, int row0, int colbase16) {
    const int i = lane & 15;
    const int col = colbase16 + 4 * (i & 3);
    const int r_a = row0 + (i >> 2);
    typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
    const char* pa = block + r_a * 64 + col * 2;
    s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(pa));
    s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(pa + 8 * 64));
    u32x2 ua = __builtin_bit_cast(u32x2, a), ub = __builtin_bit_cast(u32x2, b);
    u32x4 r;
    r[0] = ua[0];
    r[1] = ua[1];
    r[2] = ub[0];
    r[3] = ub[1];
    return r;
}

template <typename T, int D>
__global__ __launch_bounds__(DQS_THREADS, 2) void bwd_dq_saved_kernel(const AttnParams p) {
    constexpr int NCH = D / 8, DB = D / 32;
    __shared__ u32x4 sK[2][DQS_KT * NCH];
    __shared__ u32x4 sDS[DQS_THREADS / 64][2][256];  // per wave and buffer: two 2 KiB blocks (key halves 0 and 1)
    __shared__ int sList[MAX_LIST];
    __shared__ int sCount;

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hi = lane >> 5, l32 = lane & 31, half16 = (lane >> 4) & 1;
    const int wave_lane = tid >> 6;
    const int Sq = p.Sq, Sk = p.Sk;
    const int G = p.Hq / p.Hkv;

    int ub, hk, g;
    head_unit_map(blockIdx.x, p.num_m * p.B, p.Hkv, G, ub, hk, g);
    int b = ub % p.B, grp = ub / p.B;
    if (p.group_order != nullptr) {  // with a plan: the groups of all sequences by falling length of their tile lists
        const int code = p.group_order[ub];
        b = code / p.num_m;
        grp = code - b * p.num_m;
    }
    const int h = hk * G + g;
    const WaveSlices ws = pick_wave_slices(p, b, grp);  // the plan's order (the launcher requires a plan)

    if (wave == 0) build_key_half_list(ws, p.num_n, Sk, lane, sList, &sCount);

    const int slice = __builtin_amdgcn_readfirstlane(wave == 0 ? ws.slice[0] : wave == 1 ? ws.slice[1] : wave == 2 ? ws.slice[2] : ws.slice[3]);
    // column n of a dS block holds query row 8 * ((n & 15) >> 2) + 4 * (n >> 4) + (n & 3) of the slice
    const int qrow = (slice < 0 ? 0 : slice) * 32 + 8 * ((l32 & 15) >> 2) + 4 * (l32 >> 4) + (l32 & 3);
    const bool qvalid = slice >= 0 && qrow < Sq;

    f32x16 dq[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) dq[db][i] = 0.f;

    const char* kbase = (const char*)p.k.ptr + 2 * ((int64_t)b * p.k.sb + (int64_t)hk * p.k.sh);
    const int64_t k_ts = 2 * p.k.ss * DQS_KT;  // bytes per tile
    typedef TileStage<D, DQS_KT, DQS_THREADS> Stage;
    constexpr int CPT = Stage::CPT;
    Stage stK;
    stK.setup(2 * p.k.ss, tid);
    const unsigned ldsK = lds_addr(sK), ldsDS = lds_addr(sDS) + wave * 8192u;
    constexpr unsigned TILE_BYTES = DQS_KT * NCH * 16;
    // records of this q head; record e (a slice x 128-key tile pair) is 8 KiB = four 2 KiB blocks
    const char* ds_head = (const char*)p.ds_ws + (((int64_t)h * p.ds_capacity) << 13);
    const int* entry_row = p.ds_entry + (int64_t)b * p.ds_entry_sb + (int64_t)(slice < 0 ? 0 : slice) * p.num_kt;

    // record numbers of the coming list entries, 64 at a time: lane j holds the one of list entry base + j.
    // The loaded value is handed on through an instruction of its own, so that the compiler's wait for the load sits
    // right here (once per 64 tiles) and not in front of every later use: a wait for this load is a wait for every
    // tile copy in flight.
    int ent_vec = 0;
    auto load_entries = [&](int base, int n) {
        const int j = base + lane;
        int e = 0;
        if (j < n && slice >= 0) e = entry_row[sList[j] >> 17];  // 64-key tile kt -> 128-key tile kt / 2
        asm volatile("v_mov_b32 %0, %1" : "=v"(ent_vec) : "v"(e));
    };

    // copy of the K tile of list entry `entry` into buffer buf (shared by the four waves)
    auto issue_k = [&](int entry, int buf) {
#pragma unroll
        for (int j = 0; j < CPT; ++j) stK.issue(j, kbase + (entry >> 16) * k_ts, ldsK + buf * TILE_BYTES);
    };
    // copies of this wave's dS blocks of tile `entry` (record e), the halves that have work, into its buffer buf;
    // returns the number of copy instructions issued (wave-uniform)
    auto issue_ds = [&](int entry, int e, int buf) -> int {
        const int kt = entry >> 16;
        const int c = (entry >> (4 * wave)) & 15;  // wave-uniform
        const char* rec = ds_head + ((int64_t)e << 13) + (kt & 1) * 4096;
        int issued = 0;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
            if ((c >> (2 * kb)) & 3) {
                dma_b128_stream<1>(rec + kb * 2048, (unsigned)(lane * 16), ldsDS + buf * 4096u + kb * 2048u);
                dma_b128_stream<2>(rec + kb * 2048, (unsigned)(lane * 16 + 1024), ldsDS + buf * 4096u + kb * 2048u + 1024u);
                issued += 2;
            }
        return issued;
    };

    // One 64-key tile.  The dS operands are read first; the wave's buffer is then free again and takes the blocks of
    // the tile after next (`entry2`, record `e2`; negative entry2 = nothing left), so that two tiles' worth of
    // workspace reads are in flight per wave: the kernel waits for HBM, not for the MFMAs.  Returns the number of
    // copies issued.
    auto tile_step = [&](int cur, int entry, int entry2, int e2) -> int {
        // (per-lane copy of the wave number: a skip branch the compiler can prove wave-uniform makes it restructure the loop)
        const int c = (entry >> (4 * wave_lane)) & 15;
        const u32x4* tK = sK[cur];
        const char* tDS = (const char*)sDS[wave][cur];
        u32x4 bop[2][2];
        if (c != 0) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    if ((c >> (2 * kb)) & 3) bop[kb][t] = ds_block_read_transposed(tDS + kb * 2048, lane, 16 * t + 4 * hi, 16 * half16);
            wait_lds();  // the copies below overwrite what was just read
        }
        const int issued = entry2 >= 0 ? issue_ds(entry2, e2, cur) : 0;
        if (c == 0) return issued;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (((c >> (2 * kb)) & 3) == 0) continue;
            u32x4 ta[2][DB];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int db = 0; db < DB; ++db)
                    ta[t][db] = lds_read_transposed<D>(tK, lane, 32 * kb + 16 * t + 4 * hi, 32 * db + 16 * half16);
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int db = 0; db < DB; ++db) dq[db] = T::mfma(ta[t][db], bop[kb][t], dq[db]);
        }
        return issued;
    };

    __syncthreads();
    const int n_all = sCount;
    // A tile that holds the end of a sequence whose length is not a multiple of 64 is always the last entry of the
    // list; its K rows are staged synchronously (zero fill past the end) after the main loop.
    const bool ragged = (Sk & (DQS_KT - 1)) != 0 && n_all > 0 &&
                        (__builtin_amdgcn_readfirstlane(sList[n_all > 0 ? n_all - 1 : 0]) >> 16) == ((Sk - 1) >> 6);
    const int n = n_all - (ragged ? 1 : 0);
    if (n > 0) {
        load_entries(0, n_all);
        int entry = __builtin_amdgcn_readfirstlane(sList[0]);
        int next = __builtin_amdgcn_readfirstlane(sList[n > 1 ? 1 : 0]);
        issue_k(entry, 0);
        issue_ds(entry, __builtin_amdgcn_readlane(ent_vec, 0), 0);
        if (n > 1) issue_ds(next, __builtin_amdgcn_readlane(ent_vec, 1), 1);
        wait_async();
        __syncthreads();
        for (int it = 0; it < n; ++it) {
            const int cur = it & 1;
            // the K tile of the next entry (past the end the last tile is copied again: nobody reads it)
            issue_k(next, cur ^ 1);
            // the dS blocks of the entry after next
            const int i2 = it + 2;
            int entry2 = -1, e2 = 0;
            if (i2 < n) {
                if ((i2 & 63) == 0) load_entries(i2, n_all);
                entry2 = __builtin_amdgcn_readfirstlane(sList[i2]);
                e2 = __builtin_amdgcn_readlane(ent_vec, i2 & 63);
            }
            const int issued = tile_step(cur, entry, entry2, e2);
            entry = next;
            next = entry2 >= 0 ? entry2 : next;
            // everything but the copies of the entry after next has to have landed: copies complete in order
            if (issued == 4)
                asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
            else if (issued == 2)
                asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
            else
                wait_async();
            __syncthreads();
        }
    }
    if (ragged) {
        const int entry = __builtin_amdgcn_readfirstlane(sList[n_all - 1]);
        const int kt = entry >> 16, rows = Sk - kt * DQS_KT;
        __syncthreads();
        stK.load_ragged(kbase + kt * k_ts, sK[0], rows, tid);
        const int c = (entry >> (4 * wave)) & 15;
        if (c != 0) {
            const int e = entry_row[kt >> 1];
            const char* rec = ds_head + ((int64_t)e << 13) + (kt & 1) * 4096;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
                if ((c >> (2 * kb)) & 3) {
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        sDS[wave][0][kb * 128 + j * 64 + lane] = *(const u32x4*)(rec + kb * 2048 + j * 1024 + lane * 16);
                }
        }
        __syncthreads();
        tile_step(0, entry, -1, 0);
    }

    // ---- epilogue: dq holds -dQ / scale (C fragment: lane = query column, registers = head dims 8 g + 4 hi + x)
    const float factor = -p.scale;
    if (qvalid && p.grad_typed) {
        char* dqp = (char*)p.dq.ptr + 2 * ((int64_t)b * p.dq.sb + (int64_t)qrow * p.dq.ss + (int64_t)h * p.dq.sh);
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int grp = 0; grp < 4; ++grp) {
                u32x2 w;
                w[0] = T::pack2(dq[db][4 * grp + 0] * factor, dq[db][4 * grp + 1] * factor);
                w[1] = T::pack2(dq[db][4 * grp + 2] * factor, dq[db][4 * grp + 3] * factor);
                *(u32x2*)(dqp + (32 * db + 8 * grp + 4 * hi) * 2) = w;
            }
    } else if (qvalid) {
        float* dqp = (float*)p.dq.ptr + ((int64_t)b * p.dq.sb + (int64_t)qrow * p.dq.ss + (int64_t)h * p.dq.sh);
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int grp = 0; grp < 4; ++grp) {
                const int d0 = 32 * db + 8 * grp + 4 * hi;
                f32x4 a = *(f32x4*)(dqp + d0);
#pragma unroll
                for (int x = 0; x < 4; ++x) a[x] = fmaf(dq[db][4 * grp + x], factor, a[x]);
                *(f32x4*)(dqp + d0) = a;
            }
    }
}

}  // namespace bam
