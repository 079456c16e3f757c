// extern "C" boundary of libbam_hip.so: argument validation + kernel launches.
// The declarations (with the reference call sites they replace) are in include/bam_hip.h.
#include "../../include/bam_hip.h"

#include <atomic>
#include <cstdarg>
#include <cstdio>

#include "bam_launch.h"

// Built-in plan workspace of bam_tile_plan_static: device memory that exists once per GPU for as long as the
// process lives.  In host code this name is only a handle for hipGetSymbolAddress; kernels and the other entry
// points are handed the address that call returns for the current device (g_static_plan_ptr).
static __device__ __align__(256) unsigned char g_static_plan_scratch[BAM_STATIC_PLAN_BYTES];

namespace {

constexpr int kMaxDevices = 64;
// per device, resolved on first use (two host threads that get there together both store the same address)
std::atomic<void*> g_static_plan_ptr[kMaxDevices] = {};
// Every bam_tile_plan_static call on a device starts a new generation of that device's array; the plan it returns
// carries the number, and a plan of an older generation (its arrays have been overwritten since) is refused.
std::atomic<int32_t> g_static_plan_generation[kMaxDevices] = {};

thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_half_tensor(const char* name, const void* ptr, int64_t sb, int64_t ss, int64_t sh) {
    if (ptr == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: null pointer", name);
    if (!aligned16(ptr)) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: pointer is not 16-byte aligned", name);
    if ((sb % 8) || (ss % 8) || (sh % 8))
        return fail(BAM_ERR_INVALID_ARGUMENT, "%s: strides (%lld, %lld, %lld) must be multiples of 8 elements", name,
                    (long long)sb, (long long)ss, (long long)sh);
    // tile copies hold row * stride as 32-bit byte offsets, for up to 128 rows of 2-byte elements
    if (ss < 0 || ss >= (1ll << 23))
        return fail(BAM_ERR_UNSUPPORTED, "%s: sequence stride %lld is outside [0, 2^23) elements", name, (long long)ss);
    return BAM_OK;
}

int check_f32_tensor(const char* name, const void* ptr, int64_t sb, int64_t ss, int64_t sh) {
    if (ptr == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: null pointer", name);
    if (!aligned16(ptr)) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: pointer is not 16-byte aligned", name);
    if ((sb % 4) || (ss % 4) || (sh % 4))
        return fail(BAM_ERR_INVALID_ARGUMENT, "%s: strides (%lld, %lld, %lld) must be multiples of 4 elements", name,
                    (long long)sb, (long long)ss, (long long)sh);
    return BAM_OK;
}

int check_problem(int B, int Sq, int Sk, int Hq, int Hkv, int D, int dtype) {
    if (B <= 0 || Sq <= 0 || Sk <= 0 || Hq <= 0 || Hkv <= 0)
        return fail(BAM_ERR_INVALID_ARGUMENT, "B, S, Hq, Hkv must be positive (got B %d, Sq %d, Sk %d, Hq %d, Hkv %d)", B,
                    Sq, Sk, Hq, Hkv);
    if (Hq % Hkv) return fail(BAM_ERR_INVALID_ARGUMENT, "Hq (%d) must be a multiple of Hkv (%d)", Hq, Hkv);
    if (D != 32 && D != 64 && D != 128)
        return fail(BAM_ERR_UNSUPPORTED, "head dimension %d is not supported (32, 64 or 128)", D);
    if (dtype != BAM_DTYPE_F16 && dtype != BAM_DTYPE_BF16)
        return fail(BAM_ERR_INVALID_ARGUMENT, "dtype %d is neither BAM_DTYPE_F16 nor BAM_DTYPE_BF16", dtype);
    static_assert(BAM_MAX_SEQLEN == bam::MAX_SEQLEN, "header and kernels disagree on the longest sequence");
    if (Sq > BAM_MAX_SEQLEN || Sk > BAM_MAX_SEQLEN)
        return fail(BAM_ERR_UNSUPPORTED, "S = %d exceeds BAM_MAX_SEQLEN = %d", Sq > Sk ? Sq : Sk, BAM_MAX_SEQLEN);
    if ((int64_t)((Sq + 127) / 128) * B * Hq > 0x7FFFFFFFll || (int64_t)((Sk + 127) / 128) * B * Hkv > 0x7FFFFFFFll)
        return fail(BAM_ERR_UNSUPPORTED, "grid too large");
    return BAM_OK;
}

int launched(int hip_err, const char* what) {
    if (hip_err != 0)
        return fail(BAM_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString((hipError_t)hip_err));
    return BAM_OK;
}

// Where the kernels find bitfields and positions: one (B, S) tensor for plain attention, gathered
// per-row / per-key arrays plus positions for index-tensor attention.
struct MaskSource {
    int mode;
    const int64_t *bfq, *bfk;
    int64_t bfq_sb, bfk_sb;
    const int *posq, *posk;
    const uint8_t* mask;
    int Sq, Sk;
};

MaskSource plain_source(const int64_t* bf, int64_t bf_stride_b, int S) {
    return MaskSource{bam::MASK_BITFIELD, bf, bf, bf_stride_b, bf_stride_b, nullptr, nullptr, nullptr, S, S};
}

MaskSource dense_source(const uint8_t* mask, int Sq, int Sk) {
    return MaskSource{bam::MASK_DENSE, nullptr, nullptr, 0, 0, nullptr, nullptr, mask, Sq, Sk};
}

// the kernels read the mask four bytes at a time when rows are a multiple of four bytes long
int check_mask(const char* who, const uint8_t* mask) {
    if (reinterpret_cast<uintptr_t>(mask) & 3u) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: mask is not 4-byte aligned", who);
    return BAM_OK;
}

int indexed_source(const bam_index_view* iv, MaskSource& m) {
    if (iv == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "index view: null pointer");
    if (iv->q_bits == nullptr || iv->k_bits == nullptr || iv->q_pos == nullptr || iv->k_pos == nullptr)
        return fail(BAM_ERR_INVALID_ARGUMENT, "index view: q_bits, k_bits, q_pos and k_pos must not be null");
    if ((reinterpret_cast<uintptr_t>(iv->q_bits) & 7u) || (reinterpret_cast<uintptr_t>(iv->k_bits) & 7u) ||
        (reinterpret_cast<uintptr_t>(iv->q_pos) & 3u) || (reinterpret_cast<uintptr_t>(iv->k_pos) & 3u))
        return fail(BAM_ERR_INVALID_ARGUMENT, "index view: misaligned array");
    m = MaskSource{bam::MASK_INDEXED, iv->q_bits, iv->k_bits, iv->q_bits_stride_b, iv->k_bits_stride_b,
                   iv->q_pos,         iv->k_pos,  nullptr,             iv->Sq,              iv->Sk};
    return BAM_OK;
}

// bias may be null.  The kernels read groups of four keys with one access when base and strides allow it.
int fill_bias(bam::AttnParams& p, const char* who, const bam_bias* bias, int Sk) {
    if (bias == nullptr) return BAM_OK;  // p.bias stays null
    if (bias->ptr == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: bias: null pointer", who);
    const int esz = bias->is_f32 ? 4 : 2;
    if (reinterpret_cast<uintptr_t>(bias->ptr) % esz) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: bias: misaligned pointer", who);
    p.bias = bias->ptr;
    p.bias_sb = bias->stride_b;
    p.bias_sh = bias->stride_h;
    p.bias_sm = bias->stride_m;
    p.bias_f32 = bias->is_f32 ? 1 : 0;
    p.bias_vec = (reinterpret_cast<uintptr_t>(bias->ptr) % (4 * esz) == 0) && (bias->stride_b % 4 == 0) &&
                 (bias->stride_h % 4 == 0) && (bias->stride_m % 4 == 0) && (Sk % 4 == 0);
    return BAM_OK;
}

// plan may be null.  It must have been built for this very (B, Sq, Sk).
int fill_plan(bam::AttnParams& p, const char* who, const bam_plan* plan, int B, int Sq, int Sk) {
    if (plan == nullptr) return BAM_OK;  // p.fine stays null
    if (plan->fine == nullptr || plan->order == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: plan: null array", who);
    if (plan->B != B || plan->Sq != Sq || plan->Sk != Sk)
        return fail(BAM_ERR_INVALID_ARGUMENT, "%s: plan was built for B = %d, Sq = %d, Sk = %d, not B = %d, Sq = %d, Sk = %d",
                    who, plan->B, plan->Sq, plan->Sk, B, Sq, Sk);
    if (plan->generation != 0) {  // laid out in the built-in array of bam_tile_plan_static
        int dev = -1;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices ||
            plan->fine != (const uint8_t*)g_static_plan_ptr[dev].load() ||
            plan->generation != g_static_plan_generation[dev].load())
            return fail(BAM_ERR_INVALID_ARGUMENT,
                        "%s: plan of bam_tile_plan_static is stale (a later call on this GPU has reused the built-in array)",
                        who);
    }
    if (reinterpret_cast<uintptr_t>(plan->order) & 3u) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: plan: misaligned order", who);
    p.fine = plan->fine;
    p.fine_sb = plan->fine_stride_b;
    p.fine_ss = plan->fine_stride_s;
    p.order = plan->order;
    p.order_sb = plan->order_stride_b;
    p.tile_order = plan->ds_tile_order;  // may be null
    if (reinterpret_cast<uintptr_t>(plan->group_order) & 3u)
        return fail(BAM_ERR_INVALID_ARGUMENT, "%s: plan: misaligned group order", who);
    p.group_order = plan->group_order;   // may be null
    // hand-over of dS from dK/dV to dQ: only with a workspace, for the head dim and lengths its kernels cover
    if (plan->ds_workspace != nullptr && plan->ds_entry != nullptr && plan->ds_tile_base != nullptr && p.D == 128 &&
        Sk <= bam::MAX_LIST * 64) {
        if (reinterpret_cast<uintptr_t>(plan->ds_workspace) & 15u)
            return fail(BAM_ERR_INVALID_ARGUMENT, "%s: plan: dS workspace is not 16-byte aligned", who);
        if (plan->ds_capacity <= 0) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: plan: dS workspace without a capacity", who);
        if ((int64_t)p.Hq * plan->ds_capacity > 0x7FFFFFFFll)  // record numbers are 32-bit in the kernels
            return fail(BAM_ERR_UNSUPPORTED, "%s: plan: dS workspace of %lld pairs x %d heads has too many records", who,
                        (long long)plan->ds_capacity, p.Hq);
        p.ds_entry = plan->ds_entry;
        p.ds_entry_sb = plan->ds_entry_stride_b;
        p.ds_tile_base = plan->ds_tile_base;
        p.ds_ws = plan->ds_workspace;
        p.ds_capacity = plan->ds_capacity;
    }
    if (p.mask_mode == bam::MASK_DENSE && plan->row_bits != nullptr && plan->col_bits != nullptr) {
        if ((reinterpret_cast<uintptr_t>(plan->row_bits) | reinterpret_cast<uintptr_t>(plan->col_bits)) & 3u)
            return fail(BAM_ERR_INVALID_ARGUMENT, "%s: plan: misaligned mask bits", who);
        p.row_bits = plan->row_bits;
        p.row_bits_sb = plan->row_bits_stride_b;
        p.row_bits_sn = plan->row_bits_stride_n;
        p.col_bits = plan->col_bits;
        p.col_bits_sb = plan->col_bits_stride_b;
        p.col_bits_ss = plan->col_bits_stride_s;
    }
    return BAM_OK;
}

void fill_sizes(bam::AttnParams& p, const MaskSource& m, int B, int Hq, int Hkv, int D, float scale) {
    p.bfq = m.bfq;
    p.bfk = m.bfk;
    p.bfq_sb = m.bfq_sb;
    p.bfk_sb = m.bfk_sb;
    p.posq = m.posq;
    p.posk = m.posk;
    p.mask = m.mask;
    p.mask_mode = m.mode;
    p.B = B;
    p.Sq = m.Sq;
    p.Sk = m.Sk;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.D = D;
    p.num_m = (m.Sq + 127) / 128;
    p.num_n = (m.Sk + 31) / 32;
    p.num_kt = (m.Sk + 127) / 128;
    p.Sq_rounded = p.num_m * 128;
    p.scale = scale;
}

int fwd_impl(const char* who, const void* q, const void* k, const void* v, void* o, float* lse, const MaskSource& m,
             const int8_t* flags, const int64_t* st, int64_t flags_stride_b, int64_t flags_stride_m, int B, int Hq,
             int Hkv, int D, float scale, int dtype, const bam_bias* bias, const bam_plan* plan, void* stream);
int bwd_params(bam::AttnParams& p, const char* who, const void* q, const void* k, const void* v, const void* dout,
               const float* lse, const float* delta, void* dq, void* dk, void* dv, const MaskSource& m,
               const int8_t* flags, const int64_t* st, int B, int Hq, int Hkv, int D, float scale, int dtype,
               int accumulate, bool need_dq, bool need_dkdv, const bam_bias* bias, const bam_plan* plan);

}  // namespace

#define BAM_TRY(expr)             \
    do {                          \
        int rc_ = (expr);         \
        if (rc_ != BAM_OK) return rc_; \
    } while (0)

namespace {

int fwd_impl(const char* who, const void* q, const void* k, const void* v, void* o, float* lse, const MaskSource& m,
             const int8_t* flags, const int64_t* st, int64_t flags_stride_b, int64_t flags_stride_m, int B, int Hq,
             int Hkv, int D, float scale, int dtype, const bam_bias* bias, const bam_plan* plan, void* stream) {
    BAM_TRY(check_problem(B, m.Sq, m.Sk, Hq, Hkv, D, dtype));
    BAM_TRY(check_half_tensor("q", q, st[0], st[1], st[2]));
    BAM_TRY(check_half_tensor("k", k, st[3], st[4], st[5]));
    BAM_TRY(check_half_tensor("v", v, st[6], st[7], st[8]));
    BAM_TRY(check_half_tensor("o", o, st[9], st[10], st[11]));
    if (lse == nullptr || flags == nullptr || (m.mode != bam::MASK_DENSE && (m.bfq == nullptr || m.bfk == nullptr)))
        return fail(BAM_ERR_INVALID_ARGUMENT, "%s: lse, bitfields and flags must not be null", who);
    if (!(scale > 0.f)) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: softmax scale must be > 0 (got %g)", who, scale);
    bam::AttnParams p = {};
    p.q = {q, st[0], st[1], st[2]};
    p.k = {k, st[3], st[4], st[5]};
    p.v = {v, st[6], st[7], st[8]};
    p.o = {o, st[9], st[10], st[11]};
    p.lse = lse;
    p.flags = flags;
    p.flags_sb = flags_stride_b;
    p.flags_sm = flags_stride_m;
    fill_sizes(p, m, B, Hq, Hkv, D, scale);
    BAM_TRY(fill_bias(p, who, bias, m.Sk));
    BAM_TRY(fill_plan(p, who, plan, B, m.Sq, m.Sk));
    return launched(bam::launch_fwd(p, dtype, (hipStream_t)stream), who);
}

// st: strides of q, k, v, do, dq, dk, dv (3 each), then flags_stride_b, flags_stride_m
int bwd_params(bam::AttnParams& p, const char* who, const void* q, const void* k, const void* v, const void* dout,
               const float* lse, const float* delta, void* dq, void* dk, void* dv, const MaskSource& m,
               const int8_t* flags, const int64_t* st, int B, int Hq, int Hkv, int D, float scale, int dtype,
               int accumulate, bool need_dq, bool need_dkdv, const bam_bias* bias, const bam_plan* plan) {
    BAM_TRY(check_problem(B, m.Sq, m.Sk, Hq, Hkv, D, dtype));
    BAM_TRY(check_half_tensor("q", q, st[0], st[1], st[2]));
    BAM_TRY(check_half_tensor("k", k, st[3], st[4], st[5]));
    BAM_TRY(check_half_tensor("v", v, st[6], st[7], st[8]));
    BAM_TRY(check_half_tensor("do", dout, st[9], st[10], st[11]));
    if (accumulate) {
        if (need_dq) BAM_TRY(check_f32_tensor("dq", dq, st[12], st[13], st[14]));
        if (need_dkdv) {
            BAM_TRY(check_f32_tensor("dk", dk, st[15], st[16], st[17]));
            BAM_TRY(check_f32_tensor("dv", dv, st[18], st[19], st[20]));
        }
    } else {
        if (need_dq) BAM_TRY(check_half_tensor("dq", dq, st[12], st[13], st[14]));
        if (need_dkdv) {
            BAM_TRY(check_half_tensor("dk", dk, st[15], st[16], st[17]));
            BAM_TRY(check_half_tensor("dv", dv, st[18], st[19], st[20]));
        }
    }
    p.grad_typed = accumulate ? 0 : 1;
    if (lse == nullptr || delta == nullptr || flags == nullptr ||
        (m.mode != bam::MASK_DENSE && (m.bfq == nullptr || m.bfk == nullptr)))
        return fail(BAM_ERR_INVALID_ARGUMENT, "%s: lse, delta, bitfields and flags must not be null", who);
    if (!(scale > 0.f)) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: softmax scale must be > 0 (got %g)", who, scale);
    p.q = {q, st[0], st[1], st[2]};
    p.k = {k, st[3], st[4], st[5]};
    p.v = {v, st[6], st[7], st[8]};
    p.dout = {dout, st[9], st[10], st[11]};
    p.dq = {dq, st[12], st[13], st[14]};
    p.dk = {dk, st[15], st[16], st[17]};
    p.dv = {dv, st[18], st[19], st[20]};
    p.lse = const_cast<float*>(lse);
    p.delta = const_cast<float*>(delta);
    p.flags = flags;
    p.flags_sb = st[21];
    p.flags_sm = st[22];
    fill_sizes(p, m, B, Hq, Hkv, D, scale);
    BAM_TRY(fill_plan(p, who, plan, B, m.Sq, m.Sk));
    return fill_bias(p, who, bias, m.Sk);
}

// with a dS workspace in the plan, dK/dV stores its dS blocks and dQ is computed from them
int launch_dkdv(const bam::AttnParams& p, int dtype, void* stream) {
    return p.ds_ws != nullptr ? bam::launch_bwd_dkdv_save(p, dtype, (hipStream_t)stream)
                              : bam::launch_bwd_dkdv(p, dtype, (hipStream_t)stream);
}
int launch_dq(const bam::AttnParams& p, int dtype, void* stream) {
    return p.ds_ws != nullptr ? bam::launch_bwd_dq_saved(p, dtype, (hipStream_t)stream)
                              : bam::launch_bwd_dq(p, dtype, (hipStream_t)stream);
}

}  // namespace

extern "C" {

const char* bam_last_error(void) { return g_error; }

int bam_abi_version(void) { return 10; }

int bam_tile_flags(const int64_t* bf, int64_t bf_stride_b, int8_t* flags, int64_t flags_stride_b,
                   int64_t flags_stride_m, int B, int S, void* stream) {
    if (bf == nullptr || flags == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_tile_flags: null pointer");
    if (B <= 0 || S <= 0) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_tile_flags: B and S must be positive");
    if (B > 65535 || (S + 127) / 128 > 65535)
        return fail(BAM_ERR_UNSUPPORTED, "bam_tile_flags: grid too large (B = %d, S = %d)", B, S);
    return launched(bam::launch_tile_flags(bf, bf_stride_b, flags, flags_stride_b, flags_stride_m, B, S,
                                           (hipStream_t)stream),
                    "bam_tile_flags");
}

namespace {
// workspace layout: fine | order, each part 256-byte aligned
struct PlanLayout {
    int64_t fine_ss, fine_sb, order_sb, entry_sb, fine_off, order_off, entry_off, base_off, count_off, bytes;
    int64_t row_sn, row_sb, col_ss, col_sb, row_off, col_off, bytes_with_bits, tile_count_off, tile_order_off;
    int64_t group_count_off, group_order_off, row_workloads_off;
};
PlanLayout plan_layout(int B, int Sq, int Sk) {
    const int64_t num_m = (Sq + 127) / 128, num_n = (Sk + 31) / 32, slots = 4 * num_m;
    auto up = [](int64_t x, int64_t a) { return (x + a - 1) / a * a; };
    PlanLayout l;
    l.fine_ss = up(num_n, 16);
    l.fine_sb = slots * l.fine_ss;
    l.order_sb = slots;
    l.fine_off = 0;
    l.order_off = up(B * l.fine_sb, 256);
    l.entry_sb = slots * ((Sk + 127) / 128);
    l.entry_off = l.order_off + up(B * slots * 4, 256);
    l.base_off = l.entry_off + up(B * l.entry_sb * 4, 256);
    l.count_off = l.base_off + up(B * ((Sk + 127) / 128) * 4, 256);
    l.tile_count_off = l.count_off + 256;
    l.tile_order_off = l.tile_count_off + up(B * ((Sk + 127) / 128) * 4, 256);
    l.group_count_off = l.tile_order_off + up(B * ((Sk + 127) / 128) * 4, 256);
    l.group_order_off = l.group_count_off + up(B * num_m * 4, 256);
    l.row_workloads_off = l.group_order_off + up(B * num_m * 4, 256);
    l.bytes = l.row_workloads_off + up(num_m * 8, 256);
    // the packed mask of bam_mask_tile_plan: rows padded to 128, keys to 128, 32-key blocks to an even number
    l.row_sn = num_m * 128;
    l.row_sb = ((num_n + 1) & ~(int64_t)1) * l.row_sn;
    l.col_ss = ((Sk + 127) / 128) * 128;
    l.col_sb = slots * l.col_ss;
    l.row_off = l.bytes;
    l.col_off = l.row_off + up(B * l.row_sb * 4, 256);
    l.bytes_with_bits = l.col_off + up(B * l.col_sb * 4, 256);
    return l;
}
}  // namespace

int64_t bam_plan_workspace_bytes_rect(int B, int Sq, int Sk) {
    if (B <= 0 || Sq <= 0 || Sk <= 0 || (Sq + 31) / 32 > bam::MAX_PLAN_SLICES || Sk > BAM_MAX_SEQLEN) return 0;
    return plan_layout(B, Sq, Sk).bytes;
}

int64_t bam_plan_workspace_bytes(int B, int S) { return bam_plan_workspace_bytes_rect(B, S, S); }

int64_t bam_mask_plan_workspace_bytes(int B, int Sq, int Sk) {
    if (bam_plan_workspace_bytes_rect(B, Sq, Sk) == 0) return 0;
    return plan_layout(B, Sq, Sk).bytes_with_bits;
}

namespace {
// Checks the workspace and lays the plan's arrays out in it.
int place_plan(const char* who, void* workspace, int64_t workspace_bytes, int B, int Sq, int Sk, bam_plan* plan,
               PlanLayout& l, bool with_bits = false) {
    if (workspace == nullptr || plan == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    const int64_t need = with_bits ? bam_mask_plan_workspace_bytes(B, Sq, Sk) : bam_plan_workspace_bytes_rect(B, Sq, Sk);
    if (need == 0) return fail(BAM_ERR_UNSUPPORTED, "%s: no plan is built for Sq = %d, Sk = %d", who, Sq, Sk);
    if (workspace_bytes < need)
        return fail(BAM_ERR_INVALID_ARGUMENT, "%s: workspace of %lld bytes, %lld needed", who, (long long)workspace_bytes,
                    (long long)need);
    if (reinterpret_cast<uintptr_t>(workspace) & 255u)
        return fail(BAM_ERR_INVALID_ARGUMENT, "%s: workspace is not 256-byte aligned", who);
    l = plan_layout(B, Sq, Sk);
    char* w = (char*)workspace;
    plan->fine = (const uint8_t*)(w + l.fine_off);
    plan->fine_stride_b = l.fine_sb;
    plan->fine_stride_s = l.fine_ss;
    plan->order = (const int32_t*)(w + l.order_off);
    plan->order_stride_b = l.order_sb;
    plan->ds_entry = (const int32_t*)(w + l.entry_off);
    plan->ds_entry_stride_b = l.entry_sb;
    plan->ds_tile_base = (const int32_t*)(w + l.base_off);
    plan->ds_count = (const int32_t*)(w + l.count_off);
    plan->ds_tile_order = (int64_t)B * ((Sk + 127) / 128) <= bam::MAX_RANKED ? (const int32_t*)(w + l.tile_order_off) : nullptr;
    plan->group_order = (int64_t)B * ((Sq + 127) / 128) <= bam::MAX_RANKED ? (const int32_t*)(w + l.group_order_off) : nullptr;
    plan->row_workloads = (const int64_t*)(w + l.row_workloads_off);
    plan->ds_workspace = nullptr;
    plan->ds_capacity = 0;
    plan->row_bits = with_bits ? (const uint32_t*)(w + l.row_off) : nullptr;
    plan->row_bits_stride_b = with_bits ? l.row_sb : 0;
    plan->row_bits_stride_n = with_bits ? l.row_sn : 0;
    plan->col_bits = with_bits ? (const uint32_t*)(w + l.col_off) : nullptr;
    plan->col_bits_stride_b = with_bits ? l.col_sb : 0;
    plan->col_bits_stride_s = with_bits ? l.col_ss : 0;
    plan->B = B;
    plan->Sq = Sq;
    plan->Sk = Sk;
    plan->generation = 0;
    return BAM_OK;
}

// second launch of every plan builder: numbers the (slice, 128-key tile) pairs that have work
int number_pairs(const char* who, const bam_plan* plan, const PlanLayout& l, void* workspace, void* stream) {
    return launched(bam::launch_ds_entries(plan->fine, plan->fine_stride_b, plan->fine_stride_s, plan->B, plan->Sq, plan->Sk,
                                           const_cast<int*>(plan->ds_entry), plan->ds_entry_stride_b,
                                           const_cast<int*>(plan->ds_tile_base),
                                           const_cast<int*>(plan->ds_count),
                                           (int*)((char*)workspace + l.tile_count_off),
                                           const_cast<int*>(plan->ds_tile_order), plan->order, plan->order_stride_b,
                                           (int*)((char*)workspace + l.group_count_off),
                                           const_cast<int*>(plan->group_order),
                                           const_cast<int64_t*>(plan->row_workloads), (hipStream_t)stream),
                    who);
}
}  // namespace

int bam_tile_plan(const int64_t* bf, int64_t bf_stride_b, int8_t* flags, int64_t flags_stride_b,
                  int64_t flags_stride_m, void* workspace, int64_t workspace_bytes, int B, int S, bam_plan* plan,
                  void* stream) {
    if (bf == nullptr || flags == nullptr || workspace == nullptr || plan == nullptr)
        return fail(BAM_ERR_INVALID_ARGUMENT, "bam_tile_plan: null pointer");
    if (B <= 0 || S <= 0) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_tile_plan: B and S must be positive");
    if (B > 65535 || (S + 127) / 128 > 65535)
        return fail(BAM_ERR_UNSUPPORTED, "bam_tile_plan: grid too large (B = %d, S = %d)", B, S);
    PlanLayout l;
    BAM_TRY(place_plan("bam_tile_plan", workspace, workspace_bytes, B, S, S, plan, l));
    char* w = (char*)workspace;
    BAM_TRY(launched(bam::launch_tile_plan(bf, bf_stride_b, flags, flags_stride_b, flags_stride_m, (uint8_t*)(w + l.fine_off),
                                           l.fine_sb, l.fine_ss, (int*)(w + l.order_off), l.order_sb,
                                           (int*)(w + l.count_off), B, S, (hipStream_t)stream),
                     "bam_tile_plan"));
    return number_pairs("bam_tile_plan", plan, l, workspace, stream);
}

int bam_tile_plan_static(const int64_t* bf, int64_t bf_stride_b, int8_t* flags, int64_t flags_stride_b,
                         int64_t flags_stride_m, int B, int S, bam_plan* plan, void* stream) {
    if (B <= 0 || S <= 0) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_tile_plan_static: B and S must be positive");
    const int64_t need = bam_plan_workspace_bytes(B, S);
    if (need == 0 || need > BAM_STATIC_PLAN_BYTES)
        return fail(BAM_ERR_UNSUPPORTED,
                    "bam_tile_plan_static: B = %d, S = %d needs a plan workspace of %lld bytes, the built-in one holds %lld "
                    "(use bam_tile_plan with a workspace of your own)",
                    B, S, (long long)need, (long long)BAM_STATIC_PLAN_BYTES);
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return fail(BAM_ERR_LAUNCH, "bam_tile_plan_static: no current device (or more than %d devices)", kMaxDevices);
    void* ptr = g_static_plan_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        // once per device, with that device current: the array's own address on this GPU
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_plan_scratch));
        if (e != hipSuccess || ptr == nullptr)
            return fail(BAM_ERR_LAUNCH, "bam_tile_plan_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        g_static_plan_ptr[dev].store(ptr, std::memory_order_release);
    }
    BAM_TRY(bam_tile_plan(bf, bf_stride_b, flags, flags_stride_b, flags_stride_m, ptr, BAM_STATIC_PLAN_BYTES, B, S, plan,
                          stream));
    int32_t gen = g_static_plan_generation[dev].fetch_add(1) + 1;
    if (gen <= 0) g_static_plan_generation[dev].store(gen = 1);
    plan->generation = gen;
    return BAM_OK;
}

int bam_plan_indexed(const bam_index_view* iv, void* workspace, int64_t workspace_bytes, int B, bam_plan* plan,
                     void* stream) {
    MaskSource m;
    BAM_TRY(indexed_source(iv, m));
    if (B <= 0 || m.Sq <= 0 || m.Sk <= 0) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_plan_indexed: B, Sq and Sk must be positive");
    if (B > 65535) return fail(BAM_ERR_UNSUPPORTED, "bam_plan_indexed: B is limited to 65535 (got %d)", B);
    PlanLayout l;
    BAM_TRY(place_plan("bam_plan_indexed", workspace, workspace_bytes, B, m.Sq, m.Sk, plan, l));
    char* w = (char*)workspace;
    BAM_TRY(launched(bam::launch_indexed_plan(m.bfq, m.bfq_sb, m.bfk, m.bfk_sb, m.posq, m.posk, m.Sq, m.Sk,
                                              (uint8_t*)(w + l.fine_off), l.fine_sb, l.fine_ss, (int*)(w + l.order_off),
                                              l.order_sb, (int*)(w + l.count_off), B, (hipStream_t)stream),
                     "bam_plan_indexed"));
    return number_pairs("bam_plan_indexed", plan, l, workspace, stream);
}

int bam_mask_tile_plan(const uint8_t* mask, int8_t* flags, int64_t flags_stride_b, int64_t flags_stride_m, void* workspace,
                       int64_t workspace_bytes, int B, int Sq, int Sk, bam_plan* plan, void* stream) {
    if (mask == nullptr || flags == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_mask_tile_plan: null pointer");
    if (B <= 0 || Sq <= 0 || Sk <= 0) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_mask_tile_plan: B, Sq and Sk must be positive");
    if (B > 65535 || (Sq + 127) / 128 > 65535)
        return fail(BAM_ERR_UNSUPPORTED, "bam_mask_tile_plan: grid too large (B = %d, Sq = %d)", B, Sq);
    PlanLayout l;
    BAM_TRY(place_plan("bam_mask_tile_plan", workspace, workspace_bytes, B, Sq, Sk, plan, l, true));
    char* w = (char*)workspace;
    BAM_TRY(launched(bam::launch_mask_tile_plan(mask, flags, flags_stride_b, flags_stride_m, (uint8_t*)(w + l.fine_off),
                                                l.fine_sb, l.fine_ss, (int*)(w + l.order_off), l.order_sb,
                                                (int*)(w + l.count_off), (unsigned*)(w + l.row_off), l.row_sb, l.row_sn,
                                                (unsigned*)(w + l.col_off), l.col_sb, l.col_ss, B, Sq, Sk,
                                                (hipStream_t)stream),
                     "bam_mask_tile_plan"));
    return number_pairs("bam_mask_tile_plan", plan, l, workspace, stream);
}

int64_t bam_ds_workspace_bytes(int Hq, int64_t pairs) {
    if (Hq <= 0 || pairs <= 0) return 0;
    return (int64_t)Hq * pairs * 8192;
}

int bam_materialize_mask(const int64_t* bf, int64_t bf_stride_b, uint8_t* out, int B, int S, void* stream) {
    if (bf == nullptr || out == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_materialize_mask: null pointer");
    if (B <= 0 || S <= 0) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_materialize_mask: B and S must be positive");
    if (B > 65535 || S > 65535)
        return fail(BAM_ERR_UNSUPPORTED, "bam_materialize_mask: B and S are limited to 65535 (got %d, %d)", B, S);
    return launched(bam::launch_materialize_mask(bf, bf_stride_b, out, B, S, (hipStream_t)stream),
                    "bam_materialize_mask");
}

int bam_flag_row_workloads(const int8_t* flags, int64_t flags_stride_b, int64_t flags_stride_m, int B, int num_m,
                           int num_n, int32_t* out, void* stream) {
    if (flags == nullptr || out == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_flag_row_workloads: null pointer");
    if (B <= 0 || num_m <= 0 || num_n <= 0)
        return fail(BAM_ERR_INVALID_ARGUMENT, "bam_flag_row_workloads: B, num_m and num_n must be positive");
    return launched(bam::launch_flag_row_workloads(flags, flags_stride_b, flags_stride_m, B, num_m, num_n, out,
                                                   (hipStream_t)stream),
                    "bam_flag_row_workloads");
}

int bam_gather_bitfields(const int64_t* bf, int64_t bf_stride_b, int L, const int64_t* idx, int n, int64_t* out_bits,
                         int64_t out_stride_b, int32_t* out_pos, int B, void* stream) {
    if (bf == nullptr || idx == nullptr || out_bits == nullptr || out_pos == nullptr)
        return fail(BAM_ERR_INVALID_ARGUMENT, "bam_gather_bitfields: null pointer");
    if (B <= 0 || L <= 0 || n <= 0) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_gather_bitfields: B, L and n must be positive");
    if (B > 65535) return fail(BAM_ERR_UNSUPPORTED, "bam_gather_bitfields: B is limited to 65535 (got %d)", B);
    return launched(bam::launch_gather_bitfields(bf, bf_stride_b, L, idx, n, out_bits, out_stride_b, out_pos, B,
                                                 (hipStream_t)stream),
                    "bam_gather_bitfields");
}

#define BAM_FWD_STRIDES                                                                                     \
    {q_stride_b, q_stride_s, q_stride_h, k_stride_b, k_stride_s, k_stride_h, v_stride_b, v_stride_s, v_stride_h, \
     o_stride_b, o_stride_s, o_stride_h}

int bam_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int64_t* bf,
            const int8_t* flags, int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
            int64_t k_stride_b, int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b,
            int64_t v_stride_s, int64_t v_stride_h, int64_t o_stride_b, int64_t o_stride_s,
            int64_t o_stride_h, int64_t bf_stride_b, int64_t flags_stride_b, int64_t flags_stride_m, int B,
            int S, int Hq, int Hkv, int D, float scale, int dtype, const bam_bias* bias, const bam_plan* plan,
            void* stream) {
    const int64_t st[12] = BAM_FWD_STRIDES;
    return fwd_impl("bam_fwd", q, k, v, o, lse, plain_source(bf, bf_stride_b, S), flags, st, flags_stride_b,
                    flags_stride_m, B, Hq, Hkv, D, scale, dtype, bias, plan, stream);
}

int bam_fwd_indexed(const void* q, const void* k, const void* v, void* o, float* lse, const bam_index_view* iv,
                    const int8_t* flags, int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                    int64_t k_stride_b, int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b,
                    int64_t v_stride_s, int64_t v_stride_h, int64_t o_stride_b, int64_t o_stride_s,
                    int64_t o_stride_h, int64_t flags_stride_b, int64_t flags_stride_m, int B, int Hq, int Hkv,
                    int D, float scale, int dtype, const bam_bias* bias, const bam_plan* plan,
        void* stream) {
    MaskSource m;
    BAM_TRY(indexed_source(iv, m));
    const int64_t st[12] = BAM_FWD_STRIDES;
    return fwd_impl("bam_fwd_indexed", q, k, v, o, lse, m, flags, st, flags_stride_b, flags_stride_m, B, Hq, Hkv, D,
                    scale, dtype, bias, plan, stream);
}

int bam_bwd_preprocess(const void* o, const void* dout, float* delta, int64_t o_stride_b, int64_t o_stride_s,
                       int64_t o_stride_h, int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h,
                       int B, int S, int Hq, int D, int dtype, void* stream) {
    BAM_TRY(check_problem(B, S, S, Hq, Hq, D, dtype));
    BAM_TRY(check_half_tensor("o", o, o_stride_b, o_stride_s, o_stride_h));
    BAM_TRY(check_half_tensor("do", dout, do_stride_b, do_stride_s, do_stride_h));
    if (delta == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_bwd_preprocess: delta must not be null");
    bam::AttnParams p = {};
    p.o = {o, o_stride_b, o_stride_s, o_stride_h};
    p.dout = {dout, do_stride_b, do_stride_s, do_stride_h};
    p.delta = delta;
    fill_sizes(p, plain_source(nullptr, 0, S), B, Hq, Hq, D, 1.f);  // the preprocess kernel never looks at the mask
    return launched(bam::launch_bwd_preprocess(p, dtype, (hipStream_t)stream), "bam_bwd_preprocess");
}

#define BAM_BWD_STRIDES                                                                                      \
    {q_stride_b,  q_stride_s,  q_stride_h,  k_stride_b,  k_stride_s,  k_stride_h,  v_stride_b,  v_stride_s,  \
     v_stride_h,  do_stride_b, do_stride_s, do_stride_h, dq_stride_b, dq_stride_s, dq_stride_h, dk_stride_b, \
     dk_stride_s, dk_stride_h, dv_stride_b, dv_stride_s, dv_stride_h, flags_stride_b, flags_stride_m}

int bam_bwd(const void* q, const void* k, const void* v, const void* dout, const float* lse,
            const float* delta, void* dq, void* dk, void* dv, const int64_t* bf, const int8_t* flags,
            int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b,
            int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s,
            int64_t v_stride_h, int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h,
            int64_t dq_stride_b, int64_t dq_stride_s, int64_t dq_stride_h, int64_t dk_stride_b,
            int64_t dk_stride_s, int64_t dk_stride_h, int64_t dv_stride_b, int64_t dv_stride_s,
            int64_t dv_stride_h, int64_t bf_stride_b, int64_t flags_stride_b, int64_t flags_stride_m, int B,
            int S, int Hq, int Hkv, int D, float scale, int dtype, int accumulate, const bam_bias* bias,
            const bam_plan* plan, void* stream) {
    const int64_t st[23] = BAM_BWD_STRIDES;
    bam::AttnParams p = {};
    BAM_TRY(bwd_params(p, "bam_bwd", q, k, v, dout, lse, delta, dq, dk, dv, plain_source(bf, bf_stride_b, S), flags, st, B,
                       Hq, Hkv, D, scale, dtype, accumulate, true, true, bias, plan));
    BAM_TRY(launched(launch_dkdv(p, dtype, stream), "bam_bwd (dk/dv)"));
    return launched(launch_dq(p, dtype, stream), "bam_bwd (dq)");
}

int bam_bwd_dkdv(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                 const float* delta, void* dk, void* dv, const int64_t* bf, const int8_t* flags,
                 int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b,
                 int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s,
                 int64_t v_stride_h, int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h,
                 int64_t dk_stride_b, int64_t dk_stride_s, int64_t dk_stride_h, int64_t dv_stride_b,
                 int64_t dv_stride_s, int64_t dv_stride_h, int64_t bf_stride_b, int64_t flags_stride_b,
                 int64_t flags_stride_m, int B, int S, int Hq, int Hkv, int D, float scale, int dtype,
                 int accumulate, const bam_bias* bias, const bam_plan* plan, void* stream) {
    void* dq = nullptr;
    const int64_t dq_stride_b = 0, dq_stride_s = 0, dq_stride_h = 0;
    const int64_t st[23] = BAM_BWD_STRIDES;
    bam::AttnParams p = {};
    BAM_TRY(bwd_params(p, "bam_bwd_dkdv", q, k, v, dout, lse, delta, dq, dk, dv, plain_source(bf, bf_stride_b, S), flags,
                       st, B, Hq, Hkv, D, scale, dtype, accumulate, false, true, bias, plan));
    return launched(launch_dkdv(p, dtype, stream), "bam_bwd_dkdv");
}

int bam_bwd_dq(const void* q, const void* k, const void* v, const void* dout, const float* lse,
               const float* delta, void* dq, const int64_t* bf, const int8_t* flags, int64_t q_stride_b,
               int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b, int64_t k_stride_s,
               int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s, int64_t v_stride_h,
               int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h, int64_t dq_stride_b,
               int64_t dq_stride_s, int64_t dq_stride_h, int64_t bf_stride_b, int64_t flags_stride_b,
               int64_t flags_stride_m, int B, int S, int Hq, int Hkv, int D, float scale, int dtype,
               int accumulate, const bam_bias* bias, const bam_plan* plan, void* stream) {
    void *dk = nullptr, *dv = nullptr;
    const int64_t dk_stride_b = 0, dk_stride_s = 0, dk_stride_h = 0, dv_stride_b = 0, dv_stride_s = 0, dv_stride_h = 0;
    const int64_t st[23] = BAM_BWD_STRIDES;
    bam::AttnParams p = {};
    BAM_TRY(bwd_params(p, "bam_bwd_dq", q, k, v, dout, lse, delta, dq, dk, dv, plain_source(bf, bf_stride_b, S), flags, st,
                       B, Hq, Hkv, D, scale, dtype, accumulate, true, false, bias, plan));
    return launched(launch_dq(p, dtype, stream), "bam_bwd_dq");
}

int bam_bwd_dkdv_indexed(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                         const float* delta, void* dk, void* dv, const bam_index_view* iv, const int8_t* flags,
                         int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b,
                         int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s,
                         int64_t v_stride_h, int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h,
                         int64_t dk_stride_b, int64_t dk_stride_s, int64_t dk_stride_h, int64_t dv_stride_b,
                         int64_t dv_stride_s, int64_t dv_stride_h, int64_t flags_stride_b, int64_t flags_stride_m,
                         int B, int Hq, int Hkv, int D, float scale, int dtype, int accumulate, const bam_bias* bias, const bam_plan* plan,
        void* stream) {
    MaskSource m;
    BAM_TRY(indexed_source(iv, m));
    void* dq = nullptr;
    const int64_t dq_stride_b = 0, dq_stride_s = 0, dq_stride_h = 0;
    const int64_t st[23] = BAM_BWD_STRIDES;
    bam::AttnParams p = {};
    BAM_TRY(bwd_params(p, "bam_bwd_dkdv_indexed", q, k, v, dout, lse, delta, dq, dk, dv, m, flags, st, B, Hq, Hkv, D, scale,
                       dtype, accumulate, false, true, bias, plan));
    return launched(launch_dkdv(p, dtype, stream), "bam_bwd_dkdv_indexed");
}

int bam_bwd_dq_indexed(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                       const float* delta, void* dq, const bam_index_view* iv, const int8_t* flags,
                       int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b,
                       int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s,
                       int64_t v_stride_h, int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h,
                       int64_t dq_stride_b, int64_t dq_stride_s, int64_t dq_stride_h, int64_t flags_stride_b,
                       int64_t flags_stride_m, int B, int Hq, int Hkv, int D, float scale, int dtype,
                       int accumulate, const bam_bias* bias, const bam_plan* plan,
        void* stream) {
    MaskSource m;
    BAM_TRY(indexed_source(iv, m));
    void *dk = nullptr, *dv = nullptr;
    const int64_t dk_stride_b = 0, dk_stride_s = 0, dk_stride_h = 0, dv_stride_b = 0, dv_stride_s = 0, dv_stride_h = 0;
    const int64_t st[23] = BAM_BWD_STRIDES;
    bam::AttnParams p = {};
    BAM_TRY(bwd_params(p, "bam_bwd_dq_indexed", q, k, v, dout, lse, delta, dq, dk, dv, m, flags, st, B, Hq, Hkv, D, scale,
                       dtype, accumulate, true, false, bias, plan));
    return launched(launch_dq(p, dtype, stream), "bam_bwd_dq_indexed");
}

int64_t bam_decode_workspace_bytes(int B, int Sk, int Hq, int Hkv, int D, int window) {
    if (B <= 0 || Sk <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || D <= 0 || window < 0) return 0;
    int nsplit = 1, tps = 1, rgs = 1;
    bam::decode_split_plan(B, Hq, Hkv, Sk, window, &nsplit, &tps, &rgs);
    return nsplit > 1 ? (int64_t)B * Hq * nsplit * (D + 2) * 4 : 0;
}

int bam_decode(const void* q, const void* k, const void* v, void* o, int64_t q_stride_b, int64_t q_stride_h,
               int64_t k_stride_b, int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s,
               int64_t v_stride_h, int64_t o_stride_b, int64_t o_stride_h, int B, int Sk, int Hq, int Hkv, int D, float scale,
               int dtype, int window, float softcap, void* workspace, int64_t workspace_bytes, void* stream) {
    BAM_TRY(check_problem(B, 1, Sk, Hq, Hkv, D, dtype));
    BAM_TRY(check_half_tensor("k", k, k_stride_b, k_stride_s, k_stride_h));
    BAM_TRY(check_half_tensor("v", v, v_stride_b, v_stride_s, v_stride_h));
    if (q == nullptr || o == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_decode: null pointer");
    if ((reinterpret_cast<uintptr_t>(q) & 1u) || (reinterpret_cast<uintptr_t>(o) & 1u))
        return fail(BAM_ERR_INVALID_ARGUMENT, "bam_decode: q / o are not 2-byte aligned");
    if (!(scale > 0.f)) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_decode: softmax scale must be > 0 (got %g)", scale);
    if (window < 0) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_decode: window must be >= 0 (0 = none), got %d", window);
    if (!(softcap >= 0.f)) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_decode: softcap must be >= 0 (0 = none), got %g", softcap);
    if ((int64_t)B * Hq > 0x7FFFFFFFll) return fail(BAM_ERR_UNSUPPORTED, "bam_decode: grid too large");
    bam::DecodeParams p = {};
    bam::decode_split_plan(B, Hq, Hkv, Sk, window, &p.nsplit, &p.tiles_per_split, &p.row_groups);
    if ((int64_t)B * p.row_groups > 65535 || Hkv > 65535)
        return fail(BAM_ERR_UNSUPPORTED, "bam_decode: grid too large (B = %d, Hkv = %d)", B, Hkv);
    if (p.nsplit > 1) {
        const int64_t need = bam_decode_workspace_bytes(B, Sk, Hq, Hkv, D, window);
        if (workspace == nullptr || workspace_bytes < need)
            return fail(BAM_ERR_INVALID_ARGUMENT, "bam_decode: workspace of %lld bytes, %lld needed",
                        (long long)(workspace == nullptr ? 0 : workspace_bytes), (long long)need);
        if (reinterpret_cast<uintptr_t>(workspace) & 15u)
            return fail(BAM_ERR_INVALID_ARGUMENT, "bam_decode: workspace is not 16-byte aligned");
        p.ws_o = (float*)workspace;
        p.ws_ml = p.ws_o + (int64_t)B * Hq * p.nsplit * D;
    }
    p.q = q;
    p.k = k;
    p.v = v;
    p.o = o;
    p.q_sb = q_stride_b;
    p.q_sh = q_stride_h;
    p.k_sb = k_stride_b;
    p.k_ss = k_stride_s;
    p.k_sh = k_stride_h;
    p.v_sb = v_stride_b;
    p.v_ss = v_stride_s;
    p.v_sh = v_stride_h;
    p.o_sb = o_stride_b;
    p.o_sh = o_stride_h;
    p.B = B;
    p.Sk = Sk;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.D = D;
    p.window = window;
    p.scale = scale;
    p.softcap = softcap;
    return launched(bam::launch_decode(p, dtype, (hipStream_t)stream), "bam_decode");
}

int bam_mask_tile_flags(const uint8_t* mask, int8_t* flags, int64_t flags_stride_b, int64_t flags_stride_m, int B,
                        int Sq, int Sk, void* stream) {
    if (mask == nullptr || flags == nullptr) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_mask_tile_flags: null pointer");
    if (B <= 0 || Sq <= 0 || Sk <= 0) return fail(BAM_ERR_INVALID_ARGUMENT, "bam_mask_tile_flags: B, Sq and Sk must be positive");
    if (B > 65535 || (Sq + 127) / 128 > 65535)
        return fail(BAM_ERR_UNSUPPORTED, "bam_mask_tile_flags: grid too large (B = %d, Sq = %d)", B, Sq);
    return launched(bam::launch_mask_tile_flags(mask, flags, flags_stride_b, flags_stride_m, B, Sq, Sk, (hipStream_t)stream),
                    "bam_mask_tile_flags");
}

int bam_fwd_masked(const void* q, const void* k, const void* v, void* o, float* lse, const uint8_t* mask,
                   const int8_t* flags, int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                   int64_t k_stride_b, int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b,
                   int64_t v_stride_s, int64_t v_stride_h, int64_t o_stride_b, int64_t o_stride_s,
                   int64_t o_stride_h, int64_t flags_stride_b, int64_t flags_stride_m, int B, int Sq, int Sk, int Hq,
                   int Hkv, int D, float scale, int dtype, const bam_bias* bias, const bam_plan* plan,
        void* stream) {
    BAM_TRY(check_mask("bam_fwd_masked", mask));
    const int64_t st[12] = BAM_FWD_STRIDES;
    return fwd_impl("bam_fwd_masked", q, k, v, o, lse, dense_source(mask, Sq, Sk), flags, st, flags_stride_b,
                    flags_stride_m, B, Hq, Hkv, D, scale, dtype, bias, plan, stream);
}

int bam_bwd_dkdv_masked(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                        const float* delta, void* dk, void* dv, const uint8_t* mask, const int8_t* flags,
                        int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b,
                        int64_t k_stride_s, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s,
                        int64_t v_stride_h, int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h,
                        int64_t dk_stride_b, int64_t dk_stride_s, int64_t dk_stride_h, int64_t dv_stride_b,
                        int64_t dv_stride_s, int64_t dv_stride_h, int64_t flags_stride_b, int64_t flags_stride_m,
                        int B, int Sq, int Sk, int Hq, int Hkv, int D, float scale, int dtype, int accumulate,
                        const bam_bias* bias, const bam_plan* plan,
        void* stream) {
    BAM_TRY(check_mask("bam_bwd_dkdv_masked", mask));
    void* dq = nullptr;
    const int64_t dq_stride_b = 0, dq_stride_s = 0, dq_stride_h = 0;
    const int64_t st[23] = BAM_BWD_STRIDES;
    bam::AttnParams p = {};
    BAM_TRY(bwd_params(p, "bam_bwd_dkdv_masked", q, k, v, dout, lse, delta, dq, dk, dv, dense_source(mask, Sq, Sk), flags,
                       st, B, Hq, Hkv, D, scale, dtype, accumulate, false, true, bias, plan));
    return launched(launch_dkdv(p, dtype, stream), "bam_bwd_dkdv_masked");
}

int bam_bwd_dq_masked(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                      const float* delta, void* dq, const uint8_t* mask, const int8_t* flags, int64_t q_stride_b,
                      int64_t q_stride_s, int64_t q_stride_h, int64_t k_stride_b, int64_t k_stride_s,
                      int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_s, int64_t v_stride_h,
                      int64_t do_stride_b, int64_t do_stride_s, int64_t do_stride_h, int64_t dq_stride_b,
                      int64_t dq_stride_s, int64_t dq_stride_h, int64_t flags_stride_b, int64_t flags_stride_m, int B,
                      int Sq, int Sk, int Hq, int Hkv, int D, float scale, int dtype, int accumulate, const bam_bias* bias, const bam_plan* plan,
        void* stream) {
    BAM_TRY(check_mask("bam_bwd_dq_masked", mask));
    void *dk = nullptr, *dv = nullptr;
    const int64_t dk_stride_b = 0, dk_stride_s = 0, dk_stride_h = 0, dv_stride_b = 0, dv_stride_s = 0, dv_stride_h = 0;
    const int64_t st[23] = BAM_BWD_STRIDES;
    bam::AttnParams p = {};
    BAM_TRY(bwd_params(p, "bam_bwd_dq_masked", q, k, v, dout, lse, delta, dq, dk, dv, dense_source(mask, Sq, Sk), flags, st,
                       B, Hq, Hkv, D, scale, dtype, accumulate, true, false, bias, plan));
    return launched(launch_dq(p, dtype, stream), "bam_bwd_dq_masked");
}

}  // extern "C"
