// Host-side launch interface between the C ABI (bam_abi.hip) and the kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bam {

// Where the allow / deny decision of a (query, key) pair comes from.
constexpr int MASK_BITFIELD = 0;  // bitfield rule, position = row / column number
constexpr int MASK_INDEXED = 1;   // bitfield rule on gathered bitfields and explicit global positions
constexpr int MASK_DENSE = 2;     // a materialized bool mask (B, Sq, Sk), one byte per pair (or none: all pairs allowed)

// A workgroup lists its 64-key tiles (forward, dQ) or its 32-row slices (dK/dV) in LDS, this many at a time;
// sequences beyond 131072 tokens take several passes.
constexpr int MAX_LIST = 2048;         // 64-key tiles per pass
constexpr int MAX_RANKED = 8192;       // key tiles / groups of slices of a batch that the plan ranks by their work
constexpr int MAX_SLICE_LIST = 4096;   // 32-row slices per pass
// Longest sequence the entry points accept (tile numbers are packed with eight class bits into 32-bit list entries,
// positions are 32-bit; the bound leaves a wide margin to both).
constexpr int MAX_SEQLEN = 1 << 22;
// A plan (fine classes + slice order) is only built for sequences up to this many 32-row slices.
constexpr int MAX_PLAN_SLICES = 4096;

struct Tensor4 {  // logical (B, S, H, D), unit stride along D, strides in elements
    const void* ptr;
    int64_t sb, ss, sh;
};

struct AttnParams {
    Tensor4 q, k, v, o, dout;  // 16-bit tensors
    Tensor4 dq, dk, dv;        // gradients: fp32 accumulated into, or (grad_typed) input dtype, overwritten
    int grad_typed;
    float* lse;                // (B, Hq, Sq_rounded)
    float* delta;              // (B, Hq, Sq_rounded)
    // Bitfields of the query rows (B, Sq) and of the keys (B, Sk), and their global positions.  Plain
    // attention: both point at the one bitfield tensor and the positions are null (position = row /
    // column number).  Index-tensor attention (context-parallel shards): gathered copies and positions.
    const int64_t* bfq;
    const int64_t* bfk;
    int64_t bfq_sb, bfk_sb;
    const int* posq;
    const int* posk;
    // MASK_DENSE: bool mask (B, Sq, Sk), contiguous, one byte per pair; null = every in-range pair allowed
    const uint8_t* mask;
    int mask_mode;             // MASK_BITFIELD / MASK_INDEXED / MASK_DENSE
    // Additive attention bias (reference bitfield_attention.py:321-329, :410-434): a logical (B, Hq, Sq, Sk)
    // view with unit stride along the keys, added to scale * q.k before the softmax; null = none.  A stride of
    // 0 broadcasts (the per-key "vector" form has bias_sm == 0).
    const void* bias;
    int64_t bias_sb, bias_sh, bias_sm;  // in elements
    int bias_f32;              // element type: 1 = fp32, 0 = the dtype of q
    int bias_vec;              // every group of four keys starting at a multiple of four is one aligned, in-range access
    const int8_t* flags;       // (B, num_m, num_n)
    int64_t flags_sb, flags_sm;
    // Optional plan (null = none; every mask mode has a builder of its own).  fine: class 0 / 1 / 2 of every 32-row x 32-key
    // tile, (B, 4 * num_m, fine_ss) bytes; order: the 32-row slices of each sequence sorted so that four
    // neighbours need about the same keys, heaviest first, (B, 4 * num_m) ints, -1 = no slice.
    const uint8_t* fine;
    int64_t fine_sb, fine_ss;
    const int* order;
    int64_t order_sb;
    // Optional hand-over of dS from the dK/dV kernel to the dQ kernel (needs the plan; null = none).  ds_entry:
    // number of every (slice, 128-key tile) pair that has work, (B, 4 * num_m, num_kt) ints, -1 = none.  ds_ws: one
    // 8 KiB record per (q head, pair), record (h, e) at ((h * ds_capacity + e) * 8 KiB); inside it four 2 KiB blocks,
    // one per 32-key group; a block holds, for each of its 32 keys, 32 values of -dS / scale in the input dtype.
    const int* ds_entry;
    int64_t ds_entry_sb;
    const int* ds_tile_base;   // (B, num_kt): number of the first pair of each 128-key tile; the pairs of a tile are
                               // numbered consecutively, by ascending slice
    void* ds_ws;
    int64_t ds_capacity;
    // Optional (plan): the key tiles of all sequences (code b * num_kt + t) by falling number of (slice, tile) pairs
    // with work; the dK/dV kernel takes its workgroups in this order (null: early tiles first).
    const int* tile_order;
    // Optional (plan): the groups of four slices of all sequences (code b * num_m + group) by falling number of
    // 64-key tiles their workgroup visits; the forward and dQ kernels take their workgroups in this order (null:
    // group by group, the sequences of the batch side by side).
    const int* group_order;
    // MASK_DENSE with a plan: the mask packed to bits, once per orientation (null = read the mask bytes).
    // row_bits (B, row_bits_sn-strided 32-key blocks, rows): bit c of word (n, r) = mask[r][32 n + c];
    // col_bits (B, 32-row slices, keys): bit r of word (s, k) = mask[32 s + r][k].  Out-of-range cells are 0.
    const unsigned* row_bits;
    int64_t row_bits_sb, row_bits_sn;
    const unsigned* col_bits;
    int64_t col_bits_sb, col_bits_ss;
    int B, Sq, Sk, Hq, Hkv, D;
    int Sq_rounded, num_m, num_n, num_kt;  // ceil(Sq/128)*128, ceil(Sq/128), ceil(Sk/32), ceil(Sk/128)
    float scale;
};

// Single-token decode step (one query row per batch element and head, no mask); strides in elements.
struct DecodeParams {
    const void *q, *k, *v;         // q (B, Hq, D): q_sb, q_sh; k / v (B, Sk, Hkv, D): *_sb, *_ss, *_sh
    void* o;                       // (B, Hq, D) in the dtype of q
    int64_t q_sb, q_sh, k_sb, k_ss, k_sh, v_sb, v_ss, v_sh, o_sb, o_sh;
    int B, Sk, Hq, Hkv, D;
    int window;                    // > 0: only the last `window` keys are attended to
    float scale, softcap;          // softcap > 0: scores become softcap * tanh(score / softcap)
    // How the keys are split over workgroups (decode_split_plan) and where the splits leave their partial results:
    // ws_o (B, Hq, nsplit, D) unnormalized outputs, ws_ml (B, Hq, nsplit, 2) maximum (log2 domain) and sum; unused
    // when nsplit == 1.  row_groups = ceil((Hq / Hkv) / 32): q heads of one kv head per workgroup, 32 at a time.
    float* ws_o;
    float* ws_ml;
    int nsplit, tiles_per_split, row_groups;
};
void decode_split_plan(int B, int Hq, int Hkv, int Sk, int window, int* nsplit, int* tiles_per_split, int* row_groups);

int launch_tile_flags(const int64_t* bf, int64_t bf_stride_b, int8_t* flags, int64_t flags_stride_b,
                      int64_t flags_stride_m, int B, int S, hipStream_t stream);
// Flags plus plan in one launch: fine (B, 4 * num_m, fine_ss) bytes, order (B, 4 * num_m) ints.
// (pair_count: the counter launch_ds_entries adds to, reset here)
int launch_tile_plan(const int64_t* bf, int64_t bf_stride_b, int8_t* flags, int64_t flags_stride_b,
                     int64_t flags_stride_m, uint8_t* fine, int64_t fine_sb, int64_t fine_ss, int* order,
                     int64_t order_sb, int* pair_count, int B, int S, hipStream_t stream);
int launch_materialize_mask(const int64_t* bf, int64_t bf_stride_b, uint8_t* out, int B, int S,
                            hipStream_t stream);
int launch_flag_row_workloads(const int8_t* flags, int64_t flags_stride_b, int64_t flags_stride_m, int B, int num_m,
                              int num_n, int* out, hipStream_t stream);
int launch_mask_tile_flags(const uint8_t* mask, int8_t* flags, int64_t flags_stride_b, int64_t flags_stride_m, int B,
                           int Sq, int Sk, hipStream_t stream);
int launch_gather_bitfields(const int64_t* bf, int64_t bf_stride_b, int L, const int64_t* idx, int n, int64_t* out_bits,
                            int64_t out_stride_b, int* out_pos, int B, hipStream_t stream);
// Plan (fine classes + slice order) of index-tensor attention, from the gathered bitfields and positions.
int launch_indexed_plan(const int64_t* qbits, int64_t qbits_sb, const int64_t* kbits, int64_t kbits_sb, const int* qpos,
                        const int* kpos, int Sq, int Sk, uint8_t* fine, int64_t fine_sb, int64_t fine_ss, int* order,
                        int64_t order_sb, int* pair_count, int B, hipStream_t stream);
// Flags plus plan of a materialized bool mask.
int launch_mask_tile_plan(const uint8_t* mask, int8_t* flags, int64_t flags_stride_b, int64_t flags_stride_m,
                          uint8_t* fine, int64_t fine_sb, int64_t fine_ss, int* order, int64_t order_sb, int* pair_count,
                          unsigned* row_bits, int64_t row_bits_sb, int64_t row_bits_sn, unsigned* col_bits,
                          int64_t col_bits_sb, int64_t col_bits_ss, int B, int Sq, int Sk, hipStream_t stream);
// Numbers the (slice, 128-key tile) pairs that have work: entry (B, 4 * num_m, ceil(Sk/128)) ints, -1 = none.
// tile_base (B, ceil(Sk/128)) ints: number of the first pair of each key tile (pairs are numbered tile by tile).
// *count must be zero when the kernel starts (the plan kernels reset it).  tile_count (B, ceil(Sk/128)) scratch and
// tile_order (B * ceil(Sk/128)): the key tiles by falling number of pairs, written by a second small launch; both may
// be null, and no order is written beyond MAX_RANKED tiles.  The same for the groups of four slices in the plan's slice
// order (order, order_sb): group_count (B * num_m) scratch, group_order (B * num_m) = the groups by falling number of
// 64-key tiles they visit.  row_workloads (num_m int64, or null): per 128-row block, the number of its 128 x 32 tiles
// with an allowed pair, summed over the batch.
int launch_ds_entries(const uint8_t* fine, int64_t fine_sb, int64_t fine_ss, int B, int Sq, int Sk, int* entry,
                      int64_t entry_sb, int* tile_base, int* count, int* tile_count, int* tile_order, const int* order,
                      int64_t order_sb, int* group_count, int* group_order, int64_t* row_workloads, hipStream_t stream);
int launch_fwd(const AttnParams& p, int dtype, hipStream_t stream);
int launch_bwd_preprocess(const AttnParams& p, int dtype, hipStream_t stream);
int launch_bwd_dkdv(const AttnParams& p, int dtype, hipStream_t stream);
int launch_bwd_dq(const AttnParams& p, int dtype, hipStream_t stream);
int launch_decode(const DecodeParams& p, int dtype, hipStream_t stream);
// dK/dV that also stores dS (p.ds_ws), and the dQ kernel that consumes it; D = 128, plan required
int launch_bwd_dkdv_save(const AttnParams& p, int dtype, hipStream_t stream);
int launch_bwd_dq_saved(const AttnParams& p, int dtype, hipStream_t stream);

}  // namespace bam
