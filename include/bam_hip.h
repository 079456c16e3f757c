/*
 * C ABI of libbam_hip.so: bitfield-masked attention for AMD MI355X (gfx950).
 *
 * Every entry point replaces one Triton launch site of the reference file
 * cornstarch/kernel/bitfield_attention.py (cited per function).  Conventions:
 *   - all pointers are DEVICE pointers owned by the caller; nothing is allocated or freed;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*); no call synchronizes;
 *   - q/k/v/o/do/dq/dk/dv are logically (B, S, H, D) with element strides for b, s, h and
 *     unit stride along D; 16-bit tensors need 16-byte aligned rows (pointer % 16 == 0,
 *     strides % 8 == 0), fp32 gradient buffers need pointer % 16 == 0, strides % 4 == 0;
 *   - D is 32, 64 or 128; Hq % Hkv == 0; kv head of q head h is h / (Hq / Hkv);
 *   - dtype: BAM_DTYPE_F16 or BAM_DTYPE_BF16;
 *   - flags: int8 (B, ceil(S/128), ceil(S/32)), unit stride along the last axis,
 *     0 = empty, 1 = partial, 2 = every in-range pair allowed;
 *   - lse / delta: fp32 (B, Hq, S_rounded), S_rounded = ceil(S/128)*128, contiguous;
 *   - return value: BAM_OK or a negative BAM_ERR_* code; bam_last_error() gives the text
 *     of the calling thread's last failure.
 */
#ifndef BAM_HIP_H
#define BAM_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BAM_OK 0
#define BAM_ERR_INVALID_ARGUMENT (-1) /* shape / stride / alignment / dtype violation */
#define BAM_ERR_UNSUPPORTED (-2)      /* valid request this build does not implement */
#define BAM_ERR_LAUNCH (-3)           /* the HIP runtime refused the launch */

#define BAM_DTYPE_F16 0
#define BAM_DTYPE_BF16 1

/* Upper bound on S accepted by the attention kernels (a sanity bound: the kernels walk sequences beyond 131072
 * tokens in several passes, so there is no structural limit short of 32-bit tile numbers). */
#define BAM_MAX_SEQLEN 4194304

/*
 * Index-tensor attention (context-parallel shards): the local query rows and keys are arbitrary
 * subsets / permutations of a global sequence.  The reference passes `offsets_q` / `offsets_k`
 * down to its mask block, which gathers bitfield[offsets] and compares the gathered positions
 * (bitfield_attention.py:71-101, 938-939, 1085-1086).  Here the gather is a step of its own
 * (bam_gather_bitfields) and the attention entry points take its outputs:
 *   q_bits int64 (B, Sq): bitfield of each local query row,   q_pos int32 (Sq): its global position
 *   k_bits int64 (B, Sk): bitfield of each local key,         k_pos int32 (Sk): its global position
 * The struct lives in host memory; the arrays it points at are device memory.
 */
typedef struct bam_index_view {
    const int64_t* q_bits;
    const int64_t* k_bits;
    const int32_t* q_pos;
    const int32_t* k_pos;
    int64_t q_bits_stride_b;
    int64_t k_bits_stride_b;
    int32_t Sq;
    int32_t Sk;
} bam_index_view;

/*
 * Additive attention bias (`bias` of `_bitfield_attn_forward` / `_bitfield_attn_backward` and of the
 * materialized-mask `_flash_attn_forward` / `_flash_attn_backward`; reference bitfield_attention.py:952-972,
 * 321-329, 410-434, 815-835): the scores become scale * q k^T + bias before mask and softmax; the log-sum-exp
 * includes it; it receives no gradient.  `ptr` is a logical (B, Hq, Sq, Sk) view with unit stride along the keys
 * and element strides for batch, head and query row; a stride of 0 broadcasts, so the reference's "vector" form
 * (.., 1, Sk) has stride_m == 0 and its "matrix" form (.., Sq, Sk) a real one.  Elements are fp32 (is_f32 != 0)
 * or have the dtype of q.  Pointer alignment: one element.  Every attention entry point takes a
 * `const bam_bias*` that may be null (no bias).  The struct lives in host memory.
 */
typedef struct bam_bias {
    const void* ptr;
    int64_t stride_b;
    int64_t stride_h;
    int64_t stride_m;
    int32_t is_f32;
} bam_bias;

/*
 * Plan: what the attention kernels can use beyond the 128 x 32 flags to avoid work on masked pairs.  It has no
 * counterpart in the reference (whose kernels decide per 128 x 32 flag tile, bitfield_attention.py:360-361,
 * 395-408); the flags stay exactly the reference's, the plan is derived from the same bitfields at the same time:
 *   fine : uint8 (B, 4 * ceil(S/128), fine_stride_s) -- class 0 / 1 / 2 of every 32-row x 32-key tile (row slice
 *          s = rows [32 s, 32 s + 32)), same meaning as the flags, "2" again over in-range cells only;
 *   order: int32 (B, 4 * ceil(S/128)) -- the row slices of each sequence sorted so that four neighbours need
 *          about the same keys (slices holding text rows first, latest first; then modality-only slices grouped
 *          by modality), -1 in the unused tail.
 * bam_tile_plan fills the arrays (inside a caller-provided device workspace) and this host struct; bam_plan_indexed
 * and bam_mask_tile_plan do the same for index-tensor attention and for a materialized mask (rows and keys may then
 * differ in number).  Every attention entry point takes a `const bam_plan*` that may be null.
 * With a plan, the forward and dQ kernels build their workgroups from four slices of `order` and every wave skips
 * the key tiles its own slice does not need; dK/dV walks the slices that have work for its keys, two at a time.
 * Results do not depend on whether a plan is given (same pairs, same arithmetic per pair; only the order in which
 * fp32 partial sums meet can differ in dK/dV).
 *
 * dS hand-over.  The reference's backward computes dS once per tile and adds dS k to dq with fp32 atomics
 * (bitfield_attention.py:877-898); the atomic-free split used here (dK/dV kernel, dQ kernel) recomputes S and dP in
 * the dQ kernel.  When the caller provides a workspace (plan->ds_workspace, plan->ds_capacity >= *plan->ds_count,
 * head dim 128, at most 131072 keys), the dK/dV kernel also stores every 32 x 32 block of dS it computes
 * (input dtype, as the reference rounds it, :877) and the dQ kernel becomes one GEMM over those blocks: 8 KiB per
 * (q head, pair).  With bam_bwd both kernels run in that order; with the separate entry points bam_bwd_dkdv* must be
 * called before bam_bwd_dq* with the same plan and workspace.  dq is then the sum of the very dS values that went
 * into dk (instead of a recomputation that may differ in the last bit).  The count is device data: read it (for
 * instance with an asynchronous copy enqueued right after the plan builder) before sizing the workspace.
 */
typedef struct bam_plan {
    const uint8_t* fine;
    int64_t fine_stride_b;
    int64_t fine_stride_s;
    const int32_t* order;
    int64_t order_stride_b;
    /* Hand-over of dS from the dK/dV kernel to the dQ kernel (described above).  ds_entry / ds_count are filled by the plan
     * builders; ds_workspace / ds_capacity are the caller's to set before a backward call (null / 0 = not used). */
    const int32_t* ds_entry;   /* device, (B, 4 * ceil(Sq/128), ceil(Sk/128)): number of each (slice, 128-key tile) pair
                                  that has work, numbered in (batch, tile, slice) order; -1 = the pair has none */
    int64_t ds_entry_stride_b;
    const int32_t* ds_tile_base; /* device, (B, ceil(Sk/128)): number of the first pair of each key tile */
    const int32_t* ds_count;   /* device, one int: how many such pairs there are */
    const int32_t* ds_tile_order; /* device, B * ceil(Sk/128) ints, or null (more than 8192 key tiles): the key tiles
                                     (code b * ceil(Sk/128) + t) by falling number of pairs, the order in which the
                                     dK/dV kernel takes its workgroups so that the longest start first */
    const int32_t* group_order; /* device, B * ceil(Sq/128) ints, or null (more than 8192 groups): the groups of four
                                   slices of `order` (code b * ceil(Sq/128) + group) by falling number of 64-key tiles
                                   they visit, the order in which the forward and dQ kernels take their workgroups, so
                                   that the longest start first whatever the sequences of a batch look like */
    const int64_t* row_workloads; /* device, ceil(Sq/128) int64: per 128-row block, the number of its 128 x 32 tiles in
                                     which some pair is allowed, summed over the batch -- sum(flags > 0) over batch and
                                     key columns, the workloads the reference's makespan-minimizing sequence split sorts
                                     by (shardformer/layers/utils.py:161-166); written by the plan builders' numbering
                                     launch, so a caller that builds a plan needs no bam_flag_row_workloads call */
    void* ds_workspace;        /* device, at least bam_ds_workspace_bytes(Hq, pairs) bytes, 16-byte aligned */
    int64_t ds_capacity;       /* pairs the workspace has room for: at least *ds_count */
    /* Materialized masks only (bam_mask_tile_plan; null otherwise): the mask packed to bits, once per orientation, so
     * that the attention kernels never read the mask bytes.  row_bits: bit c of word
     * [b * row_bits_stride_b + n * row_bits_stride_n + r] = mask[b][r][32 n + c]; col_bits: bit r of word
     * [b * col_bits_stride_b + s * col_bits_stride_s + k] = mask[b][32 s + r][k]; cells outside the mask are 0. */
    const uint32_t* row_bits;
    int64_t row_bits_stride_b;
    int64_t row_bits_stride_n;
    const uint32_t* col_bits;
    int64_t col_bits_stride_b;
    int64_t col_bits_stride_s;
    int32_t B;
    int32_t Sq;         /* query rows and keys the plan was built for (equal for plain bitfield attention) */
    int32_t Sk;
    int32_t generation; /* 0: caller-provided workspace; otherwise the call of bam_tile_plan_static that wrote it */
} bam_plan;

const char* bam_last_error(void);

/* ABI version of this library (bumped on any signature change). */
int bam_abi_version(void);

/*
 * Tile flags ("compressed mask").  Replaces the `_materialize_compressed_mask[shape](...)`
 * launch in BitfieldUtils.materialize_compressed_mask_from_bitfield_mask
 * (bitfield_attention.py:105-156, 176-212).
 *   bf: int64 (B, S), row stride bf_stride_b, unit column stride.
 *   flags: int8, strides flags_stride_b / flags_stride_m, unit stride along key tiles.
 */
int bam_tile_flags(const int64_t* bf, int64_t bf_stride_b, int8_t* flags, int64_t flags_stride_b,
                   int64_t flags_stride_m, int B, int S, void* stream);

/*
 * Tile flags plus plan in one call.  workspace: device memory of at least bam_plan_workspace_bytes(B, S) bytes,
 * 256-byte aligned, owned by the caller and alive as long as the plan is used; the library lays `fine` and `order`
 * out inside it.  bam_plan_workspace_bytes returns 0 when no plan is built for that size
 * (S above 131072); bam_tile_plan then refuses, and the caller uses bam_tile_flags and passes no plan.
 */
int64_t bam_plan_workspace_bytes(int B, int S);
/* The same for Sq query rows against Sk keys (index-tensor attention, materialized masks); 0 above 131072 rows. */
int64_t bam_plan_workspace_bytes_rect(int B, int Sq, int Sk);
int bam_tile_plan(const int64_t* bf, int64_t bf_stride_b, int8_t* flags, int64_t flags_stride_b,
                  int64_t flags_stride_m, void* workspace, int64_t workspace_bytes, int B, int S, bam_plan* plan,
                  void* stream);

/*
 * bam_tile_plan without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The plan is laid out in a device array built into the library (BAM_STATIC_PLAN_BYTES per GPU, held until the
 * process ends); the call allocates nothing and launches the same kernel as bam_tile_plan.  Sizes whose plan does
 * not fit (bam_plan_workspace_bytes(B, S) > BAM_STATIC_PLAN_BYTES, e.g. one sequence above ~90k tokens) are refused
 * with BAM_ERR_UNSUPPORTED.  Every call on a GPU reuses that GPU's array: the plan it returns is valid until the
 * next call of this function on the same GPU, and calls whose work overlaps on one GPU (two streams, two threads)
 * race.  Nothing in the array has to start at zero: every byte a later kernel reads is rewritten by each call.
 * A plan of an earlier call is refused by the attention entry points once a later call has reused the array
 * (bam_plan.generation).  The first call on a GPU resolves the array's address (hipGetSymbolAddress, which may load
 * the library's code onto that GPU): make one call outside graph capture before relying on "allocates nothing".
 */
#define BAM_STATIC_PLAN_BYTES (8 << 20)
int bam_tile_plan_static(const int64_t* bf, int64_t bf_stride_b, int8_t* flags, int64_t flags_stride_b,
                         int64_t flags_stride_m, int B, int S, bam_plan* plan, void* stream);

/* Bytes of a dS workspace for Hq query heads and `pairs` (slice, 128-key tile) pairs: 8192 * Hq * pairs. */
int64_t bam_ds_workspace_bytes(int Hq, int64_t pairs);

/*
 * Plan for index-tensor attention: classes of the 32 x 32 tiles of the LOCAL score matrix (iv->Sq rows against
 * iv->Sk keys, bitfields and positions as bam_gather_bitfields delivers them) and a slice order, laid out in
 * `workspace` (at least bam_plan_workspace_bytes_rect(B, iv->Sq, iv->Sk) bytes, 256-byte aligned).  No counterpart
 * in the reference, whose context-parallel shards work from the re-indexed 128 x 32 flags alone
 * (shardformer/layers/utils.py:331-353); with this plan a shard skips masked work at 32-row granularity like the
 * unsharded path.  The flags the caller passes to the attention entry points are then not consulted.
 */
int bam_plan_indexed(const bam_index_view* iv, void* workspace, int64_t workspace_bytes, int B, bam_plan* plan,
                     void* stream);

/*
 * Dense bool mask, uint8 (B, S, S) contiguous: the allow rule for every pair
 * (device function `_materialize_bitfield_mask_block`, bitfield_attention.py:60-101,
 * which the reference's test wraps in a kernel of its own,
 * tests/test_kernel/test_bitfield_attention.py:16-52).  Test/diagnostic utility.
 */
int bam_materialize_mask(const int64_t* bf, int64_t bf_stride_b, uint8_t* out, int B, int S, void* stream);

/*
 * Non-empty tiles per 128-row block, summed over the batch: out[m] = sum_{b,n} (flags[b,m,n] > 0), int32 (num_m).
 * This is the input of the makespan-minimizing sequence split, which the reference computes on the host
 * after copying the flags there (`torch.sum(compressed_mask > 0, dim=(0, 2))`,
 * shardformer/layers/utils.py:161-166).
 */
int bam_flag_row_workloads(const int8_t* flags, int64_t flags_stride_b, int64_t flags_stride_m, int B, int num_m,
                           int num_n, int32_t* out, void* stream);

/*
 * Gather for index-tensor attention: out_bits[b][i] = bf[b][idx[i]], or 0 where idx[i] is outside
 * [0, L) (the `other=0` of the reference's masked loads, bitfield_attention.py:86-87), and
 * out_pos[i] = idx[i] as int32.  bf: int64 (B, L); idx: int64 (n); out_bits: int64 (B, n) with row
 * stride out_stride_b; out_pos: int32 (n).
 */
int bam_gather_bitfields(const int64_t* bf, int64_t bf_stride_b, int L, const int64_t* idx, int n, int64_t* out_bits,
                         int64_t out_stride_b, int32_t* out_pos, int B, void* stream);

/*
 * Forward.  Replaces `_fwd_kernel[grid]` + `_aggregate_partial_outputs[grid]` in
 * `_bitfield_attn_forward` (bitfield_attention.py:236-523, 932-1069, 1292-1436):
 *   o = softmax_allowed(scale * q k^T) v,  lse = log sum_allowed exp(scale * q k^T);
 *   rows that allow no key give o = 0, lse = -inf.
 * o has q's dtype.  scale must be > 0.
 */
int bam_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int64_t* bf,
            const int8_t* flags, int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
            int64_t k_stride_b, int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b,
            int64_t v_stride_s, int64_t v_stride_h, int64_t o_stride_b, int64_t o_stride_s,
            int64_t o_stride_h, int64_t bf_stride_b, int64_t flags_stride_b, int64_t flags_stride_m, int B,
            int S, int Hq, int Hkv, int D, float scale, int dtype, const bam_bias* bias, const bam_plan* plan,
            void* stream);

/*
 * Forward with index tensors (`offsets_q` / `offsets_k` of `_bitfield_attn_forward`,
 * bitfield_attention.py:938-939, as used by
 * shardformer/layers/context_parallel_bitfield_attention.py:137-147).  q is (B, Sq, Hq, D),
 * k / v are (B, Sk, Hkv, D), flags are (B, ceil(Sq/128), ceil(Sk/32)) over LOCAL tiles,
 * lse is (B, Hq, ceil(Sq/128)*128).
 */
int bam_fwd_indexed(const void* q, const void* k, const void* v, void* o, float* lse, const bam_index_view* iv,
                    const int8_t* flags, int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                    int64_t k_stride_b, int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b,
                    int64_t v_stride_s, int64_t v_stride_h, int64_t o_stride_b, int64_t o_stride_s,
                    int64_t o_stride_h, int64_t flags_stride_b, int64_t flags_stride_m, int B, int Hq, int Hkv,
                    int D, float scale, int dtype, const bam_bias* bias, const bam_plan* plan,
        void* stream);

/*
 * delta[b,h,i] = sum_d o[b,i,h,d] * do[b,i,h,d] in fp32.  Replaces
 * `_bwd_preprocess_do_o_dot[grid]` (bitfield_attention.py:527-572, 1105-1122).
 */
int bam_bwd_preprocess(const void* o, const void* dout, float* delta, int64_t o_stride_b, int64_t o_stride_s,
                       int64_t o_stride_h, int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h,
                       int B, int S, int Hq, int D, int dtype, void* stream);

/*
 * Backward.  Replaces `_bwd_kernel[grid]` (bitfield_attention.py:598-929, 1145-1199).
 * accumulate != 0: dq, dk, dv are fp32 and are ACCUMULATED INTO (the caller zeroes them,
 *   bitfield_attention.py:1248-1250) -- the contract of `_bitfield_attn_backward`.
 * accumulate == 0: dq, dk, dv have the input dtype (16-byte aligned rows like q) and are
 *   OVERWRITTEN with the final gradients, which spares the autograd path
 *   (BitfieldAttentionFunction.backward, bitfield_attention.py:1240-1266) the zero fill and
 *   the fp32 -> dtype cast.
 * dk/dv receive the sum over the q heads of a group.  No atomics are used: each output
 * element is owned by exactly one workgroup, so the result is deterministic.
 */
int bam_bwd(const void* q, const void* k, const void* v, const void* dout, const float* lse,
            const float* delta, void* dq, void* dk, void* dv, const int64_t* bf, const int8_t* flags,
            int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b,
            int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s,
            int64_t v_stride_h, int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h,
            int64_t dq_stride_b, int64_t dq_stride_s, int64_t dq_stride_h, int64_t dk_stride_b,
            int64_t dk_stride_s, int64_t dk_stride_h, int64_t dv_stride_b, int64_t dv_stride_s,
            int64_t dv_stride_h, int64_t bf_stride_b, int64_t flags_stride_b, int64_t flags_stride_m, int B,
            int S, int Hq, int Hkv, int D, float scale, int dtype, int accumulate, const bam_bias* bias,
            const bam_plan* plan, void* stream);

/*
 * The two halves of bam_bwd as separate launches (same reference kernel,
 * bitfield_attention.py:598-929): bam_bwd_dkdv accumulates dk/dv only, bam_bwd_dq
 * accumulates dq only.  bam_bwd == bam_bwd_dkdv followed by bam_bwd_dq.  They exist so
 * that each kernel can be timed on its own and so that a caller that needs only one side
 * (frozen encoder outputs, for instance) does not pay for the other.
 */
int bam_bwd_dkdv(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                 const float* delta, void* dk, void* dv, const int64_t* bf, const int8_t* flags,
                 int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b,
                 int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s,
                 int64_t v_stride_h, int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h,
                 int64_t dk_stride_b, int64_t dk_stride_s, int64_t dk_stride_h, int64_t dv_stride_b,
                 int64_t dv_stride_s, int64_t dv_stride_h, int64_t bf_stride_b, int64_t flags_stride_b,
                 int64_t flags_stride_m, int B, int S, int Hq, int Hkv, int D, float scale, int dtype,
                 int accumulate, const bam_bias* bias, const bam_plan* plan, void* stream);

int bam_bwd_dq(const void* q, const void* k, const void* v, const void* dout, const float* lse,
               const float* delta, void* dq, const int64_t* bf, const int8_t* flags, int64_t q_stride_b,
               int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b, int64_t k_stride_s,
               int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s, int64_t v_stride_h,
               int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h, int64_t dq_stride_b,
               int64_t dq_stride_s, int64_t dq_stride_h, int64_t bf_stride_b, int64_t flags_stride_b,
               int64_t flags_stride_m, int B, int S, int Hq, int Hkv, int D, float scale, int dtype,
               int accumulate, const bam_bias* bias, const bam_plan* plan, void* stream);

/*
 * bam_bwd_dkdv / bam_bwd_dq with index tensors (`offsets_q` / `offsets_k` of
 * `_bitfield_attn_backward`, bitfield_attention.py:1085-1086, as used by
 * shardformer/layers/context_parallel_bitfield_attention.py:270-294).  dk / dv are (B, Sk, Hkv, D)
 * in LOCAL key order; dq is (B, Sq, Hq, D).
 */
int bam_bwd_dkdv_indexed(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                         const float* delta, void* dk, void* dv, const bam_index_view* iv, const int8_t* flags,
                         int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b,
                         int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s,
                         int64_t v_stride_h, int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h,
                         int64_t dk_stride_b, int64_t dk_stride_s, int64_t dk_stride_h, int64_t dv_stride_b,
                         int64_t dv_stride_s, int64_t dv_stride_h, int64_t flags_stride_b, int64_t flags_stride_m,
                         int B, int Hq, int Hkv, int D, float scale, int dtype, int accumulate, const bam_bias* bias, const bam_plan* plan,
        void* stream);

int bam_bwd_dq_indexed(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                       const float* delta, void* dq, const bam_index_view* iv, const int8_t* flags,
                       int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b,
                       int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s,
                       int64_t v_stride_h, int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h,
                       int64_t dq_stride_b, int64_t dq_stride_s, int64_t dq_stride_h, int64_t flags_stride_b,
                       int64_t flags_stride_m, int B, int Hq, int Hkv, int D, float scale, int dtype,
                       int accumulate, const bam_bias* bias, const bam_plan* plan,
        void* stream);

/*
 * Materialized-mask attention: the sibling path of the reference,
 * cornstarch/kernel/attention.py (`flash_attn_func(q, k, v, bias, mask)`, `_flash_attn_forward` :855-949,
 * `_flash_attn_backward` :952-1069, forward kernel :77-345, backward kernels :438-852), served by the same
 * forward / dK,dV / dQ kernels with the allow decision read from a bool mask instead of derived from bitfields.
 *   mask: uint8 / bool (B, Sq, Sk), contiguous, nonzero = attend; NULL = every pair allowed (then flags
 *         must be 2 everywhere).
 *   flags: int8 (B, ceil(Sq/128), ceil(Sk/32)) from bam_mask_tile_flags (0 empty, 1 partial, 2 full).
 * q is (B, Sq, Hq, D), k / v are (B, Sk, Hkv, D) (the reference requires Hkv == Hq, :867-868; grouped kv heads
 * work as in the bitfield path), lse / delta are (B, Hq, ceil(Sq/128)*128).
 */
int bam_mask_tile_flags(const uint8_t* mask, int8_t* flags, int64_t flags_stride_b, int64_t flags_stride_m, int B,
                        int Sq, int Sk, void* stream);

int bam_fwd_masked(const void* q, const void* k, const void* v, void* o, float* lse, const uint8_t* mask,
                   const int8_t* flags, int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                   int64_t k_stride_b, int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b,
                   int64_t v_stride_s, int64_t v_stride_h, int64_t o_stride_b, int64_t o_stride_s,
                   int64_t o_stride_h, int64_t flags_stride_b, int64_t flags_stride_m, int B, int Sq, int Sk, int Hq,
                   int Hkv, int D, float scale, int dtype, const bam_bias* bias, const bam_plan* plan,
        void* stream);

int bam_bwd_dkdv_masked(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                        const float* delta, void* dk, void* dv, const uint8_t* mask, const int8_t* flags,
                        int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b,
                        int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s,
                        int64_t v_stride_h, int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h,
                        int64_t dk_stride_b, int64_t dk_stride_s, int64_t dk_stride_h, int64_t dv_stride_b,
                        int64_t dv_stride_s, int64_t dv_stride_h, int64_t flags_stride_b, int64_t flags_stride_m,
                        int B, int Sq, int Sk, int Hq, int Hkv, int D, float scale, int dtype, int accumulate,
                        const bam_bias* bias, const bam_plan* plan,
        void* stream);

int bam_bwd_dq_masked(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                      const float* delta, void* dq, const uint8_t* mask, const int8_t* flags, int64_t q_stride_b,
                      int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b, int64_t k_stride_s,
                      int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s, int64_t v_stride_h,
                      int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h, int64_t dq_stride_b,
                      int64_t dq_stride_s, int64_t dq_stride_h, int64_t flags_stride_b, int64_t flags_stride_m, int B,
                      int Sq, int Sk, int Hq, int Hkv, int D, float scale, int dtype, int accumulate, const bam_bias* bias, const bam_plan* plan,
        void* stream);

/*
 * bam_mask_tile_flags plus a plan, in one pass over the mask: the four 32-row classes of every flag tile, a slice
 * order (last slice first) and the mask packed to bits in both orientations (plan->row_bits, plan->col_bits: an
 * eighth of the mask's size each), which is what the attention kernels consult in partial tiles when they are given
 * the plan -- without one they read the mask bytes.  workspace: at least bam_mask_plan_workspace_bytes(B, Sq, Sk)
 * bytes (0 = no plan is built for that size), 256-byte aligned.
 * Serves `_flash_attn_forward` / `_flash_attn_backward` of the reference's cornstarch/kernel/attention.py:855-1146,
 * whose kernels decide per 128 x 32 tile inside the attention loop (:188-200) and load the mask bytes there (:217-232).
 */
int64_t bam_mask_plan_workspace_bytes(int B, int Sq, int Sk);
int bam_mask_tile_plan(const uint8_t* mask, int8_t* flags, int64_t flags_stride_b, int64_t flags_stride_m, void* workspace,
                       int64_t workspace_bytes, int B, int Sq, int Sk, bam_plan* plan, void* stream);

/*
 * Single-token decode step of a model in eval mode: one query row per batch element and head against the whole
 * key / value cache, no bitfield consulted.  The reference hands this case to flash-attn through transformers'
 * `flash_attention_forward(module, q, k, v, attention_mask=None, dropout=, scaling=, sliding_window=, softcap=)`
 * (cornstarch/kernel/interface.py:71-83); with one query at the last position that is
 *   s_j = scale * q . k_j ;  s_j = softcap * tanh(s_j / softcap) when softcap > 0 ;
 *   keys j < Sk - window are dropped when 0 < window < Sk ;  o = softmax(s) v.
 * q, o: (B, Hq, D) with element strides for batch and head, unit stride along D, 2-byte aligned; k, v: (B, Sk, Hkv, D)
 * under the common layout rules.  window = 0 / softcap = 0 mean "none".
 * The keys are split over many workgroups (there is only one query row per head) whose partial results meet in
 * `workspace`: device memory of at least bam_decode_workspace_bytes(...) bytes for the same sizes, 16-byte aligned,
 * free again once the stream has passed the call; 0 bytes (short caches: one split) means no workspace is needed
 * and null may be passed.
 */
int64_t bam_decode_workspace_bytes(int B, int Sk, int Hq, int Hkv, int D, int window);
int bam_decode(const void* q, const void* k, const void* v, void* o, int64_t q_stride_b, int64_t q_stride_h,
               int64_t k_stride_b, int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s,
               int64_t v_stride_h, int64_t o_stride_b, int64_t o_stride_h, int B, int Sk, int Hq, int Hkv, int D, float scale,
               int dtype, int window, float softcap, void* workspace, int64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BAM_HIP_H */
