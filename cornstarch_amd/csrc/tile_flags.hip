// Tile-summary kernel: int64 bitfields -> int8 flag per (128-row, 32-column) tile, and the
// dense-mask utility.  Integer work only; results are bit exact by construction.
// Reference: cornstarch/kernel/bitfield_attention.py:60-156.
#include "bam_common.h"
#include "bam_launch.h"

namespace bam {

// One workgroup = one 128-row block x FLAG_COLS_PER_BLOCK key tiles.  Each wave takes one
// 128x32 tile at a time: lane l owns key column (l & 31) and the 64 query rows of half
// (l >> 5); the per-lane counts are summed over the wave.
// Shortcut: when the 128 rows carry one bitfield and the 32 columns carry one bitfield (and the
// tile lies inside the sequence) the class follows from one evaluation of the bit test plus the
// position of the tile relative to the diagonal; long runs of equal bitfields are the common case.
constexpr int FLAG_WAVES = 4;
constexpr int FLAG_TILES_PER_WAVE = 2;  // few tiles per wave: the grid, not the wave, covers the row of tiles
constexpr int FLAG_COLS_PER_BLOCK = FLAG_WAVES * FLAG_TILES_PER_WAVE;
constexpr int FLAG_MAX_BLOCKS_X = 64;  // workgroups per 128-row block; longer rows of tiles are walked in a loop

// ---------------------------------------------------------------------------------------------------------
// Slice order.  The forward and dQ kernels give each of the four waves of a workgroup one 32-row slice and walk
// the union of the key tiles those slices need, so four slices that need the same keys should sit together:
//   * slices holding a text row first, by descending position (they see their whole past; the latest see most),
//   * then the slices made of modality rows only, grouped by the OR of their bitfields (equal value = same
//     modality = same keys), by ascending position inside a group.
// Every slice gets a two-word sort key and is ranked against all others of its sequence (at most
// MAX_PLAN_SLICES of them); slots past the last slice are set to -1.  The work rides in the launch of the flag
// kernel, as extra workgroups of its grid (it needs the bitfields only): workgroup `part` of sequence b ranks
// slices [256 part, +256).
// Ranks the slices [256 part, +256) of one sequence among all `ns` slices by two-word keys (distinct for distinct
// slices; slices >= ns get the largest key) and writes order_row[rank] = slice; the slots past the last slice are set
// to -1.  `fill(base, sk)` puts the keys of slices [base, base + 256) into sk[2 i], sk[2 i + 1] (all 256 threads take
// part).  The compares read the keys eight at a time, so that the loop runs at the rate of the LDS and not at its
// latency.
typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
template <typename FillFn>
__device__ __forceinline__ void slice_order_ranked(FillFn fill, int ns, int slots, int part, int* __restrict__ order_row) {
    __shared__ __attribute__((aligned(16))) unsigned long long sk[2 * 256];
    const int tid = threadIdx.x, s = part * 256 + tid;
    unsigned long long my1 = 0, my2 = 0;
    int rank = 0;
    // this workgroup's own slices first (their keys are what the others are compared with), then the other chunks
    const int nchunks = (ns + 255) / 256;
    for (int c = 0; c < nchunks; ++c) {
        const int base = 256 * (c == 0 ? part : c <= part ? c - 1 : c);
        __syncthreads();
        fill(base, sk);
        __syncthreads();
        if (c == 0) {
            my1 = sk[2 * tid];
            my2 = sk[2 * tid + 1];
        }
        for (int j0 = 0; j0 < 256; j0 += 8) {  // entries past the last slice hold the largest key: never smaller
            u64x2 o[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) o[u] = *(const u64x2*)&sk[2 * (j0 + u)];
#pragma unroll
            for (int u = 0; u < 8; ++u) rank += (o[u][0] < my1 || (o[u][0] == my1 && o[u][1] < my2)) ? 1 : 0;
        }
    }
    if (s < ns)
        order_row[rank] = s;
    else if (s < slots)
        order_row[s] = -1;
}

// OR over the 16 lanes of a DPP row, result in every lane (quad swaps, then the two mirror patterns).
__device__ __forceinline__ unsigned row_or(unsigned x) {
    x |= (unsigned)__builtin_amdgcn_mov_dpp((int)x, 0xB1, 0xF, 0xF, false);   // quad_perm [1,0,3,2]
    x |= (unsigned)__builtin_amdgcn_mov_dpp((int)x, 0x4E, 0xF, 0xF, false);   // quad_perm [2,3,0,1]
    x |= (unsigned)__builtin_amdgcn_mov_dpp((int)x, 0x141, 0xF, 0xF, false);  // row_half_mirror
    x |= (unsigned)__builtin_amdgcn_mov_dpp((int)x, 0x140, 0xF, 0xF, false);  // row_mirror
    return x;
}

// Keys of slices [base, base + 256) from the bitfields (k1 = 0 for a slice with a text row, else bit 62 + the OR of
// its bitfields; k2 = the position rank inside the class), read in order: 16 lanes take the 32 rows of one slice (two
// each) and OR them together; bit 0 of the OR says whether the slice holds a text row.
__device__ __forceinline__ void slice_keys_chunk(const int64_t* __restrict__ row, int S, int ns, int base,
                                                 unsigned long long* sk) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t M = (((int64_t)1) << 62) - 1;
#pragma unroll 4
    for (int pass = 0; pass < 16; ++pass) {
        const int local = 64 * wave + 4 * pass + (lane >> 4);  // slice within the chunk
        const int s = base + local;
        const int i = s * 32 + 2 * (lane & 15);
        const int64_t f0 = i < S ? row[i] : 0, f1 = i + 1 < S ? row[i + 1] : 0;
        const uint64_t f = (uint64_t)(f0 | f1);
        const unsigned lo = row_or((unsigned)f), hi = row_or((unsigned)(f >> 32));
        if ((lane & 15) == 0) {
            const bool text = (lo & 1u) != 0;
            const unsigned long long sig = (((unsigned long long)hi << 32) | lo) & (unsigned long long)M;
            unsigned long long k1 = text ? 0ull : (1ull << 62) | sig;
            unsigned long long k2 = text ? (unsigned long long)(ns - 1 - s) : (unsigned long long)s;
            if (s >= ns) k1 = k2 = ~0ull;
            sk[2 * local] = k1;
            sk[2 * local + 1] = k2;
        }
    }
}

__device__ __forceinline__ void slice_order_part(const int64_t* __restrict__ row, int S, int part,
                                                 int* __restrict__ order_row) {
    const int ns = (S + 31) / 32, slots = 4 * ((S + BLOCK_M - 1) / BLOCK_M);
    slice_order_ranked([&](int base, unsigned long long* sk) { slice_keys_chunk(row, S, ns, base, sk); }, ns, slots, part,
                       order_row);
}

// The same ordering idea for index-tensor attention, where a local row's position is pos[row]: slices holding a
// text row first, by descending largest position; then modality-only slices grouped by the OR of their bitfields,
// by ascending smallest position.  The slice number in the low bits keeps the keys distinct whatever the positions.
__device__ __forceinline__ void slice_sort_key_indexed(const int64_t* __restrict__ bits, const int* __restrict__ pos,
                                                       int S, int ns, int s, unsigned long long& k1,
                                                       unsigned long long& k2) {
    k1 = ~0ull;
    k2 = ~0ull;
    if (s >= ns) return;
    const int64_t M = (((int64_t)1) << 62) - 1;
    int64_t sig = 0;
    bool text = false;
    int pmax = 0, pmin = 0x7FFFFFFF;
#pragma unroll
    for (int r = 0; r < 32; ++r) {
        const int i = s * 32 + r;
        const int64_t f = i < S ? bits[i] : 0;
        const int q = i < S ? pos[i] : 0;
        sig |= f & M;
        text |= (f & 1) != 0;
        if (i < S) {
            pmax = max(pmax, q);
            pmin = min(pmin, q);
        }
    }
    k1 = text ? 0ull : (1ull << 62) | (unsigned long long)sig;
    k2 = ((unsigned long long)(text ? 0x7FFFFFFF - pmax : pmin) << 20) | (unsigned long long)s;
}

// FINE: also write the class of every 32-row x 32-column tile (the four row slices of each flag tile) to
// fine[b][4 m + w][n]; same 0 / 1 / 2 meaning, "full" again over the in-range cells only.
template <bool FINE>
__global__ __launch_bounds__(FLAG_WAVES * 64) void tile_flags_kernel(const int64_t* __restrict__ bf,
                                                                    int64_t bf_stride_b,
                                                                    int8_t* __restrict__ flags,
                                                                    int64_t flags_stride_b,
                                                                    int64_t flags_stride_m, int S, int num_n,
                                                                    uint8_t* __restrict__ fine, int64_t fine_sb,
                                                                    int64_t fine_ss, int* __restrict__ order,
                                                                    int64_t order_sb, int flag_blocks_x,
                                                                    int flag_groups, int* __restrict__ pair_count) {
    // (the pair counter of the numbering kernel that follows in the stream starts from zero)
    if (FINE && pair_count != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0)
        *pair_count = 0;
    if (FINE && (int)blockIdx.x >= flag_blocks_x) {  // the workgroups that sort the slices (see slice_order_part)
        const int part = blockIdx.y;
        if (part * 256 < 4 * (int)gridDim.y)
            slice_order_part(bf + (int64_t)blockIdx.z * bf_stride_b, S, part, order + (int64_t)blockIdx.z * order_sb);
        return;
    }
    __shared__ int64_t q_bits[BLOCK_M];
    // classes of this workgroup's eight column tiles: row 0 the flag, rows 1..4 the four row slices; written out
    // together at the end (eight bytes per row in one store where the layout guarantees alignment)
    // (two copies: a workgroup that takes several groups of column tiles fills one while the other is stored)
    __shared__ __attribute__((aligned(8))) uint8_t s_out_buf[2][5][FLAG_COLS_PER_BLOCK];
    const int b = blockIdx.z, m = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t* row = bf + (int64_t)b * bf_stride_b;
    if (tid < BLOCK_M) {
        const int i = m * BLOCK_M + tid;
        q_bits[tid] = (i < S) ? row[i] : 0;  // out-of-range positions read 0 (reference :86-87)
    }
    __syncthreads();
    const int rows_in_range = min(BLOCK_M, S - m * BLOCK_M);
    const int half = lane >> 5, l32 = lane & 31;
    // Runs of equal bitfields inside each of the four 32-row slices: bit r of slice_starts[w] = row r starts a run
    // (rows past the end of the sequence read 0 and make a run of their own).  The count of a column over a run
    // follows from one evaluation of the bit test, so a tile costs one evaluation per run, not one per row.
    int64_t slice_q[4];
    unsigned slice_starts[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        slice_q[w] = q_bits[32 * w];
        slice_starts[w] = (unsigned)__ballot(l32 == 0 || q_bits[32 * w + l32] != q_bits[32 * w + max(l32, 1) - 1]);
    }
    const int64_t q0 = slice_q[0];
    const bool rows_uniform = rows_in_range == BLOCK_M && slice_starts[0] == 1u && slice_starts[1] == 1u &&
                              slice_starts[2] == 1u && slice_starts[3] == 1u && slice_q[1] == q0 && slice_q[2] == q0 &&
                              slice_q[3] == q0;
    // A workgroup takes the groups of eight column tiles bx = blockIdx.x, blockIdx.x + flag_blocks_x, ...: one group
    // for sequences of up to 16384 keys, several for longer ones (the setup above is then paid once).
    int it = 0;
    for (int bx = blockIdx.x; bx < flag_groups; bx += flag_blocks_x, ++it) {
        uint8_t (*s_out)[FLAG_COLS_PER_BLOCK] = s_out_buf[it & 1];
        if (tid < 5 * FLAG_COLS_PER_BLOCK) s_out[0][tid] = 0;
        __syncthreads();
        static_assert(FLAG_TILES_PER_WAVE == 2, "the counting path gives each half of a wave one tile");
        // the key bitfields of both tiles of this wave, requested together (one memory latency instead of one per tile)
        int64_t kfs[FLAG_TILES_PER_WAVE];
#pragma unroll
        for (int t = 0; t < FLAG_TILES_PER_WAVE; ++t) {
            const int j = (bx * FLAG_COLS_PER_BLOCK + wave * FLAG_TILES_PER_WAVE + t) * BLOCK_N + l32;
            kfs[t] = (j < S) ? row[j] : 0;
        }
        bool counted[FLAG_TILES_PER_WAVE];  // wave-uniform: the tile still needs the counting path
#pragma unroll
        for (int t = 0; t < FLAG_TILES_PER_WAVE; ++t) {
            const int n = bx * FLAG_COLS_PER_BLOCK + wave * FLAG_TILES_PER_WAVE + t;
            counted[t] = n < num_n;
            if (n >= num_n) continue;  // wave-uniform
            const int64_t kf = kfs[t];
            if (rows_uniform && (n + 1) * BLOCK_N <= S) {
                const unsigned klo = __builtin_amdgcn_readfirstlane((unsigned)kf);
                const unsigned khi = __builtin_amdgcn_readfirstlane((unsigned)((uint64_t)kf >> 32));
                const int64_t k0 = (int64_t)(((uint64_t)khi << 32) | klo);
                if (__all(kf == k0)) {
                    const int64_t M = (((int64_t)1) << 62) - 1;
                    const int64_t qb = q0 & M, kb = k0 & M;
                    int8_t f;
                    const int r0 = m * BLOCK_M, c0 = n * BLOCK_N;
                    if (q0 & 1) {  // text rows: causal over keys that share a bit
                        f = (qb & kb) == 0 ? 0 : r0 >= c0 + BLOCK_N - 1 ? 2 : r0 + BLOCK_M - 1 < c0 ? 0 : 1;
                    } else {
                        f = (qb == kb && qb != 0) ? 2 : 0;
                    }
                    const int col = wave * FLAG_TILES_PER_WAVE + t;
                    if (lane == 0) s_out[0][col] = (uint8_t)f;
                    if (FINE && lane < 4) {  // the same closed form for the 32 rows of slice `lane`
                        const int rs = r0 + 32 * lane;
                        int8_t fw = f;
                        if (q0 & 1) fw = (qb & kb) == 0 ? 0 : rs >= c0 + BLOCK_N - 1 ? 2 : rs + 31 < c0 ? 0 : 1;
                        s_out[1 + lane][col] = (uint8_t)fw;
                    }
                    counted[t] = false;
                }
            }
        }
        if (counted[0] || counted[1]) {
            // Counting path, both tiles at once: lanes [0, 32) own the columns of tile 0, lanes [32, 64) those of tile 1.
            const int t = half;
            const int n = bx * FLAG_COLS_PER_BLOCK + wave * FLAG_TILES_PER_WAVE + t;
            const int j = n * BLOCK_N + l32;
            const int64_t kf = half ? kfs[1] : kfs[0];
            const int64_t M = (((int64_t)1) << 62) - 1;
            const int64_t kb = kf & M;
            int cnt[4];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const int r0 = m * BLOCK_M + 32 * w;
                unsigned starts = slice_starts[w];  // wave-uniform, bit 0 set
                int c = 0;
                while (starts != 0u) {
                    const int a = __builtin_ctz(starts);
                    starts &= starts - 1u;
                    const int e = starts != 0u ? __builtin_ctz(starts) : 32;  // the run is rows [a, e) of the slice
                    const int64_t qf = q_bits[32 * w + a];
                    const int64_t qb = qf & M;
                    if (qf & 1)  // text rows: those at or after column j (reference :93-97)
                        c += (qb & kb) != 0 ? min(e - a, max(0, r0 + e - max(r0 + a, j))) : 0;
                    else
                        c += (qb == kb && qb != 0) ? e - a : 0;
                }
                cnt[w] = c;
            }
#pragma unroll
            for (int off = 16; off > 0; off >>= 1)  // over the 32 columns, inside each half of the wave
#pragma unroll
                for (int w = 0; w < 4; ++w) cnt[w] += __shfl_xor(cnt[w], off);
            const bool mine = half ? counted[1] : counted[0];
            if (l32 == 0 && mine) {
                const int cols_in_range = min(BLOCK_N, S - n * BLOCK_N);
                const int col = wave * FLAG_TILES_PER_WAVE + t;
                if (FINE) {
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const int rows = max(0, min(32, S - (m * BLOCK_M + 32 * w)));
                        s_out[1 + w][col] = (uint8_t)(cnt[w] == 0 ? 0 : cnt[w] == rows * cols_in_range ? 2 : 1);
                    }
                }
                const int total = cnt[0] + cnt[1] + cnt[2] + cnt[3];
                // full over in-range cells (:149-153)
                s_out[0][col] = (uint8_t)(total == 0 ? 0 : total == rows_in_range * cols_in_range ? 2 : 1);
            }
        }
        __syncthreads();
        const int n0 = bx * FLAG_COLS_PER_BLOCK;
        if (tid < FLAG_COLS_PER_BLOCK && n0 + tid < num_n)  // the flag row may start anywhere: single bytes
            flags[(int64_t)b * flags_stride_b + (int64_t)m * flags_stride_m + n0 + tid] = (int8_t)s_out[0][tid];
        if (FINE && tid >= 64 && tid < 68) {  // rows of the class matrix are padded to 16 bytes: one 8-byte store
            static_assert(FLAG_COLS_PER_BLOCK == 8, "one 64-bit word per row");
            const int w = tid - 64;
            *(unsigned long long*)(fine + (int64_t)b * fine_sb + (int64_t)(4 * m + w) * fine_ss + n0) =
                *(const unsigned long long*)s_out[1 + w];
        }
    }
}

__global__ __launch_bounds__(256) void materialize_mask_kernel(const int64_t* __restrict__ bf,
                                                               int64_t bf_stride_b,
                                                               uint8_t* __restrict__ out, int S) {
    const int b = blockIdx.z, i = blockIdx.y;
    const int64_t* row = bf + (int64_t)b * bf_stride_b;
    const int64_t qf = row[i];
    for (int j = blockIdx.x * blockDim.x + threadIdx.x; j < S; j += gridDim.x * blockDim.x)
        out[((int64_t)b * S + i) * S + j] = allow_rule(qf, row[j], i, j) ? 1 : 0;
}

// Index-tensor attention, step 0: the bitfield and the 32-bit position of every local row (or key),
// out_bits[b][i] = bf[b][idx[i]] (0 when idx[i] is outside [0, L)), out_pos[i] = idx[i].
// Restates the index branch of the reference's mask block (bitfield_attention.py:71-87), hoisted out
// of the attention kernels so that they read both with unit stride.
__global__ __launch_bounds__(256) void gather_bitfields_kernel(const int64_t* __restrict__ bf, int64_t bf_stride_b,
                                                               int L, const int64_t* __restrict__ idx, int n,
                                                               int64_t* __restrict__ out_bits,
                                                               int64_t out_stride_b, int* __restrict__ out_pos) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    if (i >= n) return;
    const int64_t pos = idx[i];
    const bool inside = pos >= 0 && pos < L;
    out_bits[(int64_t)b * out_stride_b + i] = inside ? bf[(int64_t)b * bf_stride_b + pos] : 0;
    if (b == 0) out_pos[i] = (int)(pos < 0 ? 0 : pos > 0x7FFFFFFE ? 0x7FFFFFFE : pos);
}

int launch_gather_bitfields(const int64_t* bf, int64_t bf_stride_b, int L, const int64_t* idx, int n, int64_t* out_bits,
                            int64_t out_stride_b, int* out_pos, int B, hipStream_t stream) {
    dim3 grid((n + 255) / 256, B);
    hipLaunchKernelGGL(gather_bitfields_kernel, grid, dim3(256), 0, stream, bf, bf_stride_b, L, idx, n, out_bits,
                       out_stride_b, out_pos);
    return (int)hipGetLastError();
}

// Tile flags of a materialized bool mask (B, Sq, Sk), one byte per pair: the same 0 / 1 / 2 classification
// over 128 x 32 tiles that the bitfield path uses, so that the attention kernels skip empty tiles and
// read the mask only in partial ones.  (The reference's materialized-mask kernel decides per tile, inside
// the attention loop, whether anything is unmasked: cornstarch/kernel/attention.py:188-200.)
// One workgroup = one row block x 8 column tiles; thread = one column, 128 rows, coalesced byte reads.
__global__ __launch_bounds__(256) void mask_tile_flags_kernel(const uint8_t* __restrict__ mask, int8_t* __restrict__ flags,
                                                              int64_t flags_stride_b, int64_t flags_stride_m, int Sq,
                                                              int Sk, int num_n) {
    const int b = blockIdx.z, m = blockIdx.y, tid = threadIdx.x;
    const int col = blockIdx.x * 256 + tid;
    const int r0 = m * BLOCK_M, r1 = min(r0 + BLOCK_M, Sq);
    int count = 0;
    if (col < Sk) {
        const uint8_t* pcol = mask + (int64_t)b * Sq * Sk + col;
        for (int r = r0; r < r1; ++r) count += pcol[(int64_t)r * Sk] != 0;
    }
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) count += __shfl_xor(count, off);  // over the 32 columns of a tile
    const int n = blockIdx.x * 8 + (tid >> 5);
    if ((tid & 31) == 0 && n < num_n) {
        const int cells = (r1 - r0) * min(BLOCK_N, Sk - n * BLOCK_N);
        flags[(int64_t)b * flags_stride_b + (int64_t)m * flags_stride_m + n] = count == 0 ? 0 : count == cells ? 2 : 1;
    }
}

int launch_mask_tile_flags(const uint8_t* mask, int8_t* flags, int64_t flags_stride_b, int64_t flags_stride_m, int B,
                           int Sq, int Sk, hipStream_t stream) {
    const int num_m = (Sq + BLOCK_M - 1) / BLOCK_M, num_n = (Sk + BLOCK_N - 1) / BLOCK_N;
    dim3 grid((num_n + 7) / 8, num_m, B);
    hipLaunchKernelGGL(mask_tile_flags_kernel, grid, dim3(256), 0, stream, mask, flags, flags_stride_b, flags_stride_m,
                       Sq, Sk, num_n);
    return (int)hipGetLastError();
}

// Work per 128-row block for the makespan-minimizing sequence split: the number of non-empty 128x32
// tiles of each row block, summed over the batch -- `torch.sum(compressed_mask > 0, dim=(0, 2))` of
// the reference (shardformer/layers/utils.py:161-166), computed where the flags already are instead
// of after a copy to the host.  One workgroup per row block, no atomics.
__global__ __launch_bounds__(256) void flag_row_workloads_kernel(const int8_t* __restrict__ flags, int64_t flags_stride_b,
                                                                 int64_t flags_stride_m, int B, int num_n,
                                                                 int* __restrict__ out) {
    __shared__ int partial[4];
    const int m = blockIdx.x, tid = threadIdx.x;
    int count = 0;
    for (int b = 0; b < B; ++b) {
        const int8_t* row = flags + (int64_t)b * flags_stride_b + (int64_t)m * flags_stride_m;
        for (int n = tid; n < num_n; n += 256) count += row[n] > 0;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) count += __shfl_xor(count, off);
    if ((tid & 63) == 0) partial[tid >> 6] = count;
    __syncthreads();
    if (tid == 0) out[m] = partial[0] + partial[1] + partial[2] + partial[3];
}

int launch_flag_row_workloads(const int8_t* flags, int64_t flags_stride_b, int64_t flags_stride_m, int B, int num_m,
                              int num_n, int* out, hipStream_t stream) {
    hipLaunchKernelGGL(flag_row_workloads_kernel, dim3(num_m), dim3(256), 0, stream, flags, flags_stride_b,
                       flags_stride_m, B, num_n, out);
    return (int)hipGetLastError();
}

// Plan for index-tensor attention: the class of every 32-row x 32-key tile of the LOCAL score matrix (rows and keys
// are gathered subsets of a global sequence: bits / positions per local row and key, as bam_gather_bitfields
// delivers them) and a slice order.  Brute force over the pairs of each tile, same wave layout as the flag kernel:
// lane = key column (lane & 31) x 64-row half (lane >> 5).  The extra column of workgroups ranks the slices.
__global__ __launch_bounds__(FLAG_WAVES * 64) void indexed_plan_kernel(
    const int64_t* __restrict__ qbits, int64_t qbits_sb, const int64_t* __restrict__ kbits, int64_t kbits_sb,
    const int* __restrict__ qpos, const int* __restrict__ kpos, int Sq, int Sk, int num_n, uint8_t* __restrict__ fine,
    int64_t fine_sb, int64_t fine_ss, int* __restrict__ order, int64_t order_sb, int flag_blocks_x,
    int* __restrict__ pair_count) {
    const int b = blockIdx.z;
    const int64_t* qrow = qbits + (int64_t)b * qbits_sb;
    if (pair_count != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0) *pair_count = 0;
    if ((int)blockIdx.x >= flag_blocks_x) {
        const int part = blockIdx.y;
        const int ns = (Sq + 31) / 32, slots = 4 * (int)gridDim.y;
        if (part * 256 < slots)
            slice_order_ranked(
                [&](int base, unsigned long long* sk) {
                    slice_sort_key_indexed(qrow, qpos, Sq, ns, base + (int)threadIdx.x, sk[2 * threadIdx.x], sk[2 * threadIdx.x + 1]);
                },
                ns, slots, part, order + (int64_t)b * order_sb);
        return;
    }
    __shared__ int64_t q_bits[BLOCK_M];
    __shared__ int q_pos[BLOCK_M];
    __shared__ __attribute__((aligned(8))) uint8_t s_out[4][FLAG_COLS_PER_BLOCK];
    const int m = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
    if (tid < 4 * FLAG_COLS_PER_BLOCK) s_out[0][tid] = 0;
    if (tid < BLOCK_M) {
        const int i = m * BLOCK_M + tid;
        q_bits[tid] = (i < Sq) ? qrow[i] : 0;
        q_pos[tid] = (i < Sq) ? qpos[i] : 0;
    }
    __syncthreads();
    const int64_t* krow = kbits + (int64_t)b * kbits_sb;
#pragma unroll
    for (int t = 0; t < FLAG_TILES_PER_WAVE; ++t) {
        const int n = blockIdx.x * FLAG_COLS_PER_BLOCK + wave * FLAG_TILES_PER_WAVE + t;
        if (n >= num_n) break;  // wave-uniform
        const int j = n * BLOCK_N + (lane & 31);
        const int64_t kf = (j < Sk) ? krow[j] : 0;
        const int64_t kp = (j < Sk) ? kpos[j] : 0;
        int cnt_a = 0, cnt_b = 0;  // rows [64 half, +32) and [64 half + 32, +32)
#pragma unroll 8
        for (int r = 0; r < 32; ++r) {
            const int ri = half * 64 + r;
            cnt_a += allow_rule(q_bits[ri], kf, q_pos[ri], kp) ? 1 : 0;
            cnt_b += allow_rule(q_bits[ri + 32], kf, q_pos[ri + 32], kp) ? 1 : 0;
        }
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) {
            cnt_a += __shfl_xor(cnt_a, off);
            cnt_b += __shfl_xor(cnt_b, off);
        }
        const int cols_in_range = min(BLOCK_N, Sk - n * BLOCK_N);
        const int col = wave * FLAG_TILES_PER_WAVE + t;
        if ((lane & 31) == 0) {
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                const int w = 2 * half + x, c = x ? cnt_b : cnt_a;
                const int rows = max(0, min(32, Sq - (m * BLOCK_M + 32 * w)));
                s_out[w][col] = (uint8_t)(c == 0 ? 0 : c == rows * cols_in_range ? 2 : 1);
            }
        }
    }
    __syncthreads();
    const int n0 = blockIdx.x * FLAG_COLS_PER_BLOCK;
    if (tid < 4) {
        static_assert(FLAG_COLS_PER_BLOCK == 8, "one 64-bit word per row");
        *(unsigned long long*)(fine + (int64_t)b * fine_sb + (int64_t)(4 * m + tid) * fine_ss + n0) =
            *(const unsigned long long*)s_out[tid];
    }
}

int launch_indexed_plan(const int64_t* qbits, int64_t qbits_sb, const int64_t* kbits, int64_t kbits_sb, const int* qpos,
                        const int* kpos, int Sq, int Sk, uint8_t* fine, int64_t fine_sb, int64_t fine_ss, int* order,
                        int64_t order_sb, int* pair_count, int B, hipStream_t stream) {
    const int num_m = (Sq + BLOCK_M - 1) / BLOCK_M, num_n = (Sk + BLOCK_N - 1) / BLOCK_N;
    const int flag_blocks_x = (num_n + FLAG_COLS_PER_BLOCK - 1) / FLAG_COLS_PER_BLOCK;
    dim3 grid(flag_blocks_x + 1, num_m, B);
    hipLaunchKernelGGL(indexed_plan_kernel, grid, dim3(FLAG_WAVES * 64), 0, stream, qbits, qbits_sb, kbits, kbits_sb, qpos,
                       kpos, Sq, Sk, num_n, fine, fine_sb, fine_ss, order, order_sb, flag_blocks_x, pair_count);
    return (int)hipGetLastError();
}

// Flags and plan of a materialized bool mask in one launch: as mask_tile_flags_kernel, with the count kept per
// 32-row slice, so that the four slice classes of every flag tile come out of the same pass over the mask.  The
// slice order is simply "last slice first" (under a causal-like mask the late rows see the most keys); it is
// written by the workgroups of column 0.
// The same pass packs the mask to bits, once per orientation, for the attention kernels (which then never touch the
// mask bytes): thread = key column, so the 32 rows of a slice make one word of col_bits in a register, and a ballot
// over the 32 columns of a tile makes one word of row_bits per row.  Cells outside the mask are 0; the arrays cover
// num_m * 128 rows, ceil(Sk / 128) * 128 keys and an even number of 32-key blocks.
__global__ __launch_bounds__(256) void mask_tile_plan_kernel(const uint8_t* __restrict__ mask, int8_t* __restrict__ flags,
                                                             int64_t flags_stride_b, int64_t flags_stride_m, int Sq,
                                                             int Sk, int num_n, uint8_t* __restrict__ fine,
                                                             int64_t fine_sb, int64_t fine_ss, int* __restrict__ order,
                                                             int64_t order_sb, int* __restrict__ pair_count,
                                                             unsigned* __restrict__ row_bits, int64_t row_bits_sb,
                                                             int64_t row_bits_sn, unsigned* __restrict__ col_bits,
                                                             int64_t col_bits_sb, int64_t col_bits_ss) {
    const int b = blockIdx.z, m = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
    if (pair_count != nullptr && blockIdx.x == 0 && m == 0 && b == 0 && tid == 0) *pair_count = 0;
    if (blockIdx.x == 0 && tid < 4) {
        const int ns = (Sq + 31) / 32, slot = 4 * m + tid;
        order[(int64_t)b * order_sb + slot] = slot < ns ? ns - 1 - slot : -1;
    }
    const int col = blockIdx.x * 256 + tid;
    const int r0 = m * BLOCK_M;
    const int n = blockIdx.x * 8 + (tid >> 5);  // this thread's 32-key block
    const int num_n_bits = (num_n + 1) & ~1, sk_pad = ((Sk + 127) >> 7) << 7;
    const bool in = col < Sk;
    const uint8_t* pcol = mask + (int64_t)b * Sq * Sk + (in ? col : 0);
    // lanes 0 and 32 of a wave write the row words of its two 32-key blocks
    unsigned* rb_out = (row_bits != nullptr && (lane & 31) == 0 && n < num_n_bits)
                           ? row_bits + (int64_t)b * row_bits_sb + (int64_t)n * row_bits_sn + r0
                           : nullptr;
    unsigned cw[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        cw[w] = 0;
        const int ra = r0 + 32 * w;
        if (row_bits == nullptr) {
            const int rb = min(ra + 32, Sq);
            for (int r = ra; r < rb; ++r) cw[w] |= (unsigned)(in && pcol[(int64_t)r * Sk] != 0) << (r - ra);
        } else {
            for (int r = ra; r < ra + 32; ++r) {
                const bool a = in && r < Sq && pcol[(int64_t)r * Sk] != 0;
                cw[w] |= (unsigned)a << (r - ra);
                const unsigned long long bal = __ballot(a);
                if (rb_out != nullptr) rb_out[r - r0] = (unsigned)(lane == 0 ? bal : bal >> 32);
            }
        }
    }
    if (col_bits != nullptr && col < sk_pad) {
#pragma unroll
        for (int w = 0; w < 4; ++w) col_bits[(int64_t)b * col_bits_sb + (int64_t)(4 * m + w) * col_bits_ss + col] = cw[w];
    }
    int count[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) count[w] = __popc(cw[w]);
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) {  // over the 32 columns of a tile
#pragma unroll
        for (int w = 0; w < 4; ++w) count[w] += __shfl_xor(count[w], off);
    }
    if ((tid & 31) == 0 && n < num_n) {
        const int cols = min(BLOCK_N, Sk - n * BLOCK_N);
        int total = 0, cells = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const int rows = max(0, min(32, Sq - (r0 + 32 * w)));
            fine[(int64_t)b * fine_sb + (int64_t)(4 * m + w) * fine_ss + n] =
                (uint8_t)(count[w] == 0 ? 0 : count[w] == rows * cols ? 2 : 1);
            total += count[w];
            cells += rows * cols;
        }
        flags[(int64_t)b * flags_stride_b + (int64_t)m * flags_stride_m + n] = total == 0 ? 0 : total == cells ? 2 : 1;
    }
}

// The same for masks whose rows are 4-byte aligned (Sk a multiple of four): a lane takes FOUR key columns and reads
// them as one word per row, a wave takes one 32-row slice, so a workgroup reads 1 KiB per load instruction instead of
// 256 bytes.  The bytes are reduced to one bit each in the word; the four column words of the lane collect them row
// by row, the row word of a 32-key block is the OR of the nibbles of its eight lanes (DPP), staged in LDS and stored
// as runs of 32 rows.
__device__ __forceinline__ unsigned oct_or(unsigned x) {  // OR over groups of eight lanes, result in every lane
    x |= (unsigned)__builtin_amdgcn_mov_dpp((int)x, 0xB1, 0xF, 0xF, false);   // quad_perm [1,0,3,2]
    x |= (unsigned)__builtin_amdgcn_mov_dpp((int)x, 0x4E, 0xF, 0xF, false);   // quad_perm [2,3,0,1]
    x |= (unsigned)__builtin_amdgcn_mov_dpp((int)x, 0x141, 0xF, 0xF, false);  // row_half_mirror
    return x;
}
__global__ __launch_bounds__(256) void mask_tile_plan_words_kernel(
    const uint8_t* __restrict__ mask, int8_t* __restrict__ flags, int64_t flags_stride_b, int64_t flags_stride_m, int Sq,
    int Sk, int num_n, uint8_t* __restrict__ fine, int64_t fine_sb, int64_t fine_ss, int* __restrict__ order,
    int64_t order_sb, int* __restrict__ pair_count, unsigned* __restrict__ row_bits, int64_t row_bits_sb,
    int64_t row_bits_sn, unsigned* __restrict__ col_bits, int64_t col_bits_sb, int64_t col_bits_ss) {
    __shared__ unsigned s_rows[4][8][32];  // [slice][32-key block][row]: row words of this workgroup
    __shared__ int s_cnt[4][8];
    const int b = blockIdx.z, m = blockIdx.y, tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    if (pair_count != nullptr && blockIdx.x == 0 && m == 0 && b == 0 && tid == 0) *pair_count = 0;
    if (blockIdx.x == 0 && tid < 4) {
        const int ns = (Sq + 31) / 32, slot = 4 * m + tid;
        order[(int64_t)b * order_sb + slot] = slot < ns ? ns - 1 - slot : -1;
    }
    const int col0 = blockIdx.x * 256 + 4 * lane;  // first of this lane's four columns (all inside or all outside)
    const int ra = m * BLOCK_M + 32 * w;           // first row of this wave's slice
    const int nb = lane >> 3, n = blockIdx.x * 8 + nb;
    const int num_n_bits = (num_n + 1) & ~1, sk_pad = ((Sk + 127) >> 7) << 7;
    const uint8_t* prow = mask + ((int64_t)b * Sq + ra) * Sk + (col0 < Sk ? col0 : 0);
    unsigned v[32];
#pragma unroll
    for (int r = 0; r < 32; ++r) v[r] = (col0 < Sk && ra + r < Sq) ? *(const unsigned*)(prow + (int64_t)r * Sk) : 0u;
    unsigned cw[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int r = 0; r < 32; ++r) {
        unsigned t = v[r] | (v[r] >> 4);  // any bit of a byte -> its bit 0
        t |= t >> 2;
        t |= t >> 1;
        t &= 0x01010101u;
#pragma unroll
        for (int c = 0; c < 4; ++c) cw[c] |= ((t >> (8 * c)) & 1u) << r;
        const unsigned nib = (t | (t >> 7) | (t >> 14) | (t >> 21)) & 0xFu;  // the four bits side by side
        const unsigned word = oct_or(nib << (4 * (lane & 7)));
        if ((lane & 7) == 0) s_rows[w][nb][r] = word;
    }
    if (col0 < sk_pad) {
        u32x4 out = {cw[0], cw[1], cw[2], cw[3]};
        *(u32x4*)(col_bits + (int64_t)b * col_bits_sb + (int64_t)(4 * m + w) * col_bits_ss + col0) = out;
    }
    // this wave's row words: 8 blocks x 32 rows, each block a run of 32 consecutive words
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int idx = 64 * k + lane, nb2 = idx >> 5, rr = idx & 31, n2 = blockIdx.x * 8 + nb2;
        if (n2 < num_n_bits)
            row_bits[(int64_t)b * row_bits_sb + (int64_t)n2 * row_bits_sn + ra + rr] = s_rows[w][nb2][rr];
    }
    int cnt = __popc(cw[0]) + __popc(cw[1]) + __popc(cw[2]) + __popc(cw[3]);
    cnt += __shfl_xor(cnt, 1);
    cnt += __shfl_xor(cnt, 2);
    cnt += __shfl_xor(cnt, 4);
    if ((lane & 7) == 0) {
        s_cnt[w][nb] = cnt;
        if (n < num_n) {
            const int cols = min(BLOCK_N, Sk - n * BLOCK_N), rows = max(0, min(32, Sq - ra));
            fine[(int64_t)b * fine_sb + (int64_t)(4 * m + w) * fine_ss + n] = (uint8_t)(cnt == 0 ? 0 : cnt == rows * cols ? 2 : 1);
        }
    }
    __syncthreads();
    if (tid < 8 && blockIdx.x * 8 + tid < num_n) {
        const int nn = blockIdx.x * 8 + tid, cols = min(BLOCK_N, Sk - nn * BLOCK_N);
        int total = 0, cells = 0;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            total += s_cnt[x][tid];
            cells += max(0, min(32, Sq - (m * BLOCK_M + 32 * x))) * cols;
        }
        flags[(int64_t)b * flags_stride_b + (int64_t)m * flags_stride_m + nn] = total == 0 ? 0 : total == cells ? 2 : 1;
    }
}

int launch_mask_tile_plan(const uint8_t* mask, int8_t* flags, int64_t flags_stride_b, int64_t flags_stride_m,
                          uint8_t* fine, int64_t fine_sb, int64_t fine_ss, int* order, int64_t order_sb, int* pair_count,
                          unsigned* row_bits, int64_t row_bits_sb, int64_t row_bits_sn, unsigned* col_bits,
                          int64_t col_bits_sb, int64_t col_bits_ss, int B, int Sq, int Sk, hipStream_t stream) {
    const int num_m = (Sq + BLOCK_M - 1) / BLOCK_M, num_n = (Sk + BLOCK_N - 1) / BLOCK_N;
    dim3 grid((num_n + 7) / 8, num_m, B);
    if (row_bits != nullptr && col_bits != nullptr && (Sk & 3) == 0 && (reinterpret_cast<uintptr_t>(mask) & 3u) == 0)
        hipLaunchKernelGGL(mask_tile_plan_words_kernel, grid, dim3(256), 0, stream, mask, flags, flags_stride_b,
                           flags_stride_m, Sq, Sk, num_n, fine, fine_sb, fine_ss, order, order_sb, pair_count, row_bits,
                           row_bits_sb, row_bits_sn, col_bits, col_bits_sb, col_bits_ss);
    else
        hipLaunchKernelGGL(mask_tile_plan_kernel, grid, dim3(256), 0, stream, mask, flags, flags_stride_b, flags_stride_m,
                           Sq, Sk, num_n, fine, fine_sb, fine_ss, order, order_sb, pair_count, row_bits, row_bits_sb,
                           row_bits_sn, col_bits, col_bits_sb, col_bits_ss);
    return (int)hipGetLastError();
}

// Numbering of the (32-row slice, 128-key tile) pairs that have work, for the backward that hands dS from the dK/dV
// kernel to the dQ kernel through memory.  The pairs of one key tile -- exactly the slices a dK/dV workgroup lists --
// get consecutive numbers, by ascending slice; the tiles themselves take their blocks of numbers in the order their
// workgroups arrive (one atomic add per tile on *count, which the plan kernels reset):
//   entry[b][s][t]  = number of pair (b, s, t), or -1 where its four classes are all "empty"  (what the dQ kernel looks up)
//   tile_base[b][t] = number of the first pair of key tile (b, t)                             (what dK/dV starts from)
//   *count          = how many pairs there are.
// Which tile gets which block of numbers only decides where a record sits in the workspace, never a result.
// tile_count[b][t] (optional) = number of pairs of key tile (b, t): what tile_order_kernel ranks the tiles by.
// One workgroup per (key tile, batch); thread = slice, 256 slices per sweep.
constexpr int DS_NUM_THREADS = 256;
constexpr int DS_MAX_ORDERED_TILES = MAX_RANKED;  // counts staged in LDS: 32 KiB
__global__ __launch_bounds__(DS_NUM_THREADS) void ds_entries_kernel(const uint8_t* __restrict__ fine, int64_t fine_sb,
                                                                   int64_t fine_ss, int slots, int nkt, int num_n,
                                                                   int* __restrict__ entry, int64_t entry_sb,
                                                                   int* __restrict__ tile_base, int* __restrict__ count,
                                                                   int* __restrict__ tile_count,
                                                                   const int* __restrict__ order, int64_t order_sb,
                                                                   int* __restrict__ group_count, int group_blocks,
                                                                   long long* __restrict__ row_workloads) {
    __shared__ int wave_sum[DS_NUM_THREADS / 64];
    __shared__ int s_base;
    const int b = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if ((int)blockIdx.x >= nkt + group_blocks) {
        // Extra workgroups, one per 128-row block m (those of batch entry 0 do the work): in how many of the block's
        // 128 x 32 tiles, over the whole batch, some pair is allowed -- the sum of (flags > 0) over batch and key
        // columns (reference shardformer/layers/utils.py:161-166).  A 128 x 32 flag is non-zero exactly when one of the
        // classes of its four 32 x 32 tiles is.
        if (b != 0) return;
        const int m = blockIdx.x - nkt - group_blocks, nb = gridDim.y;
        int tiles = 0;
        for (int bb = 0; bb < nb; ++bb) {
            const uint8_t* rows = fine + (int64_t)bb * fine_sb + (int64_t)(4 * m) * fine_ss;
            for (int n = tid; n < num_n; n += DS_NUM_THREADS)
                tiles += (rows[n] | rows[fine_ss + n] | rows[2 * fine_ss + n] | rows[3 * fine_ss + n]) != 0 ? 1 : 0;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) tiles += __shfl_xor(tiles, off);
        if (lane == 0) wave_sum[wave] = tiles;
        __syncthreads();
        if (tid == 0) {
            long long total = 0;
            for (int w = 0; w < DS_NUM_THREADS / 64; ++w) total += wave_sum[w];
            row_workloads[m] = total;
        }
        return;
    }
    if ((int)blockIdx.x >= nkt) {
        // Extra workgroups, one per group of four slices of the slice order: how many 64-key tiles the forward / dQ
        // workgroup of that group visits (the union over its slices), which is what group_order ranks the groups by.
        const int grp = blockIdx.x - nkt, num_m = slots / 4;
        const int* ord = order + (int64_t)b * order_sb + 4 * grp;
        const uint8_t* rows[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) rows[x] = ord[x] >= 0 ? fine + (int64_t)b * fine_sb + (int64_t)ord[x] * fine_ss : nullptr;
        int visits = 0;
        for (int kt = tid; 2 * kt < num_n; kt += DS_NUM_THREADS) {
            unsigned any = 0;
#pragma unroll
            for (int x = 0; x < 4; ++x)
                if (rows[x] != nullptr) any |= rows[x][2 * kt] | (2 * kt + 1 < num_n ? rows[x][2 * kt + 1] : 0);
            visits += any != 0 ? 1 : 0;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) visits += __shfl_xor(visits, off);
        if (lane == 0) wave_sum[wave] = visits;
        __syncthreads();
        if (tid == 0) {
            int total = 0;
            for (int w = 0; w < DS_NUM_THREADS / 64; ++w) total += wave_sum[w];
            group_count[b * num_m + grp] = total;
        }
        return;
    }
    const int t = blockIdx.x;
    const uint8_t* col = fine + (int64_t)b * fine_sb + 4 * t;
    unsigned valid = 0;  // which of the tile's four 32-key columns exist
#pragma unroll
    for (int w = 0; w < 4; ++w)
        if (4 * t + w < num_n) valid |= 0xFFu << (8 * w);
    auto has_work = [&](int sl) { return sl < slots && (*(const unsigned*)(col + (int64_t)sl * fine_ss) & valid) != 0; };
    int mine = 0;
    for (int sl = tid; sl < slots; sl += DS_NUM_THREADS) mine += has_work(sl) ? 1 : 0;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mine += __shfl_xor(mine, off);
    if (lane == 0) wave_sum[wave] = mine;
    __syncthreads();
    if (tid == 0) {
        int total = 0;
        for (int w = 0; w < DS_NUM_THREADS / 64; ++w) total += wave_sum[w];
        const int base = atomicAdd(count, total);
        s_base = base;
        tile_base[(int64_t)b * nkt + t] = base;
        if (tile_count != nullptr) tile_count[b * nkt + t] = total;
    }
    __syncthreads();
    int next = s_base;
    int* out = entry + (int64_t)b * entry_sb + t;
    for (int s0 = 0; s0 < slots; s0 += DS_NUM_THREADS) {
        const int sl = s0 + tid;
        const bool h = has_work(sl);
        const unsigned long long bal = __ballot(h);
        __syncthreads();  // wave_sum is free again
        if (lane == 0) wave_sum[wave] = __popcll(bal);
        __syncthreads();
        int before = 0, all = 0;
        for (int w = 0; w < DS_NUM_THREADS / 64; ++w) {
            if (w < wave) before += wave_sum[w];
            all += wave_sum[w];
        }
        if (sl < slots) out[(int64_t)sl * nkt] = h ? next + before + __popcll(bal & ((1ull << lane) - 1ull)) : -1;
        next += all;
    }
}

// The key tiles (code b * nkt + t) sorted by their number of pairs, most first (ties: lower code first): the order in
// which the dK/dV kernel takes them, so that the long workgroups start first whatever the mask looks like.
// 64 tiles per workgroup, four threads per tile, each comparing against a quarter of all counts (staged in LDS).
// blockIdx.y = 1 ranks a second, independent array the same way (the groups of four slices, for the forward and dQ
// kernels); either array may be absent (n = 0).
__global__ __launch_bounds__(256) void tile_order_kernel(const int* __restrict__ tile_count, int n_tiles,
                                                         int* __restrict__ tile_order,
                                                         const int* __restrict__ group_count, int n_groups,
                                                         int* __restrict__ group_order) {
    __shared__ __attribute__((aligned(16))) int s_cnt[DS_MAX_ORDERED_TILES];
    const int tid = threadIdx.x;
    if (blockIdx.y == 1) {
        tile_count = group_count;
        n_tiles = n_groups;
        tile_order = group_order;
    }
    if ((int)blockIdx.x * 64 >= n_tiles) return;  // (workgroup-uniform)
    const int padded = (n_tiles + 15) & ~15;
    for (int i = tid; i < padded; i += 256) s_cnt[i] = i < n_tiles ? tile_count[i] : -1;  // padding ranks behind everything
    __syncthreads();
    const int i = blockIdx.x * 64 + (tid >> 2), sub = tid & 3;
    const int c = i < n_tiles ? s_cnt[i] : 0;
    int rank = 0;
    // thread `sub` of a tile takes the groups of four counts number sub, sub + 4, ...
    for (int j4 = sub; 4 * j4 < padded; j4 += 4) {
        const int4 v = *(const int4*)&s_cnt[4 * j4];
        const int j = 4 * j4;
        rank += (v.x > c) | ((v.x == c) & (j < i));
        rank += (v.y > c) | ((v.y == c) & (j + 1 < i));
        rank += (v.z > c) | ((v.z == c) & (j + 2 < i));
        rank += (v.w > c) | ((v.w == c) & (j + 3 < i));
    }
    rank += __shfl_xor(rank, 1);
    rank += __shfl_xor(rank, 2);
    if (sub == 0 && i < n_tiles) tile_order[rank] = i;
}

int launch_ds_entries(const uint8_t* fine, int64_t fine_sb, int64_t fine_ss, int B, int Sq, int Sk, int* entry,
                      int64_t entry_sb, int* tile_base, int* count, int* tile_count, int* tile_order, const int* order,
                      int64_t order_sb, int* group_count, int* group_order, int64_t* row_workloads, hipStream_t stream) {
    const int num_m = (Sq + BLOCK_M - 1) / BLOCK_M;
    const int slots = 4 * num_m, nkt = (Sk + 127) / 128, num_n = (Sk + BLOCK_N - 1) / BLOCK_N;
    const int n_tiles = nkt * B, n_groups = num_m * B;
    if (n_tiles > DS_MAX_ORDERED_TILES || tile_count == nullptr) tile_order = nullptr;
    if (n_groups > DS_MAX_ORDERED_TILES || group_count == nullptr || order == nullptr) group_order = nullptr;
    const int group_blocks = group_order != nullptr ? num_m : 0;
    hipLaunchKernelGGL(ds_entries_kernel, dim3(nkt + group_blocks + (row_workloads != nullptr ? num_m : 0), B),
                       dim3(DS_NUM_THREADS), 0, stream, fine, fine_sb, fine_ss, slots, nkt, num_n, entry, entry_sb,
                       tile_base, count, tile_order != nullptr ? tile_count : nullptr, order, order_sb, group_count,
                       group_blocks, (long long*)row_workloads);
    if (tile_order != nullptr || group_order != nullptr) {
        const int nt = tile_order != nullptr ? n_tiles : 0, ng = group_order != nullptr ? n_groups : 0;
        hipLaunchKernelGGL(tile_order_kernel, dim3((max(nt, ng) + 63) / 64, group_order != nullptr ? 2 : 1), dim3(256), 0,
                           stream, tile_count, nt, tile_order, group_count, ng, group_order);
    }
    return (int)hipGetLastError();
}

int launch_tile_flags(const int64_t* bf, int64_t bf_stride_b, int8_t* flags, int64_t flags_stride_b,
                      int64_t flags_stride_m, int B, int S, hipStream_t stream) {
    const int num_m = (S + BLOCK_M - 1) / BLOCK_M, num_n = (S + BLOCK_N - 1) / BLOCK_N;
    const int flag_groups = (num_n + FLAG_COLS_PER_BLOCK - 1) / FLAG_COLS_PER_BLOCK;
    const int flag_blocks_x = min(flag_groups, FLAG_MAX_BLOCKS_X);
    dim3 grid(flag_blocks_x, num_m, B);
    hipLaunchKernelGGL(tile_flags_kernel<false>, grid, dim3(FLAG_WAVES * 64), 0, stream, bf, bf_stride_b, flags,
                       flags_stride_b, flags_stride_m, S, num_n, (uint8_t*)nullptr, (int64_t)0, (int64_t)0, (int*)nullptr,
                       (int64_t)0, flag_blocks_x, flag_groups, (int*)nullptr);
    return (int)hipGetLastError();
}

int launch_tile_plan(const int64_t* bf, int64_t bf_stride_b, int8_t* flags, int64_t flags_stride_b,
                     int64_t flags_stride_m, uint8_t* fine, int64_t fine_sb, int64_t fine_ss, int* order,
                     int64_t order_sb, int* pair_count, int B, int S, hipStream_t stream) {
    const int num_m = (S + BLOCK_M - 1) / BLOCK_M, num_n = (S + BLOCK_N - 1) / BLOCK_N;
    const int flag_groups = (num_n + FLAG_COLS_PER_BLOCK - 1) / FLAG_COLS_PER_BLOCK;
    const int flag_blocks_x = min(flag_groups, FLAG_MAX_BLOCKS_X);
    // one more column of workgroups: (flag_blocks_x, part, b) ranks 256 slices; 4 num_m slots need
    // ceil(4 num_m / 256) <= num_m parts
    dim3 grid(flag_blocks_x + 1, num_m, B);
    hipLaunchKernelGGL(tile_flags_kernel<true>, grid, dim3(FLAG_WAVES * 64), 0, stream, bf, bf_stride_b, flags,
                       flags_stride_b, flags_stride_m, S, num_n, fine, fine_sb, fine_ss, order, order_sb, flag_blocks_x,
                       flag_groups, pair_count);
    return (int)hipGetLastError();
}

int launch_materialize_mask(const int64_t* bf, int64_t bf_stride_b, uint8_t* out, int B, int S,
                            hipStream_t stream) {
    dim3 grid(min((S + 255) / 256, 64), S, B);
    hipLaunchKernelGGL(materialize_mask_kernel, grid, dim3(256), 0, stream, bf, bf_stride_b, out, S);
    return (int)hipGetLastError();
}

}  // namespace bam
