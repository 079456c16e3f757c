// Shared device helpers for the bitfield-masked attention kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bam {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int BLOCK_M = 128;  // flag tile rows   (reference bitfield_attention.py:53)
constexpr int BLOCK_N = 32;   // flag tile cols   (reference bitfield_attention.py:54)
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
constexpr unsigned HI_MODALITY_MASK = 0x3FFFFFFFu;  // bits 62, 63 are never consulted

// ---------------------------------------------------------------------------------
// The allow rule (reference bitfield_attention.py:86-101).  i, j are global positions.
__device__ __forceinline__ bool allow_rule(int64_t qf, int64_t kf, int64_t i, int64_t j) {
    const int64_t M = (((int64_t)1) << 62) - 1;
    const int64_t qb = qf & M, kb = kf & M;
    const bool text = (qf & 1) != 0;
    return text ? (i >= j && (qb & kb) != 0) : (qb == kb && qb != 0);
}

// Per-query constants of the rule, split in 32-bit halves and arranged so that the
// per-pair test is branch free and identical for text and modality queries:
//   v = ((k & a) ^ x)  over both halves
//   text query     : a = q,  x = 0  -> v = q & k ; allowed iff v != 0 and kpos <= qpos
//   modality query : a = M,  x = q  -> v = q ^ k ; allowed iff v == 0 and q != 0
// where M keeps the modality bits (everything but bits 62 and 63), so the key words can be
// the raw halves of the int64 bitfield.  `lim` folds the position test and the q != 0 test
// into one compare (kpos <= lim).
struct QueryBits {
    unsigned a_lo, a_hi, x_lo, x_hi;
    int lim;    // qpos for text rows, INT_MAX for live modality rows, -1 for rows that see nothing
    bool text;
};

__device__ __forceinline__ QueryBits make_query_bits(int64_t qf, int qpos) {
    const unsigned lo = (unsigned)(qf & 0xFFFFFFFFll);
    const unsigned hi = ((unsigned)((uint64_t)qf >> 32)) & HI_MODALITY_MASK;
    QueryBits q;
    q.text = (lo & 1u) != 0;
    q.a_lo = q.text ? lo : 0xFFFFFFFFu;
    q.a_hi = q.text ? hi : HI_MODALITY_MASK;
    q.x_lo = q.text ? 0u : lo;
    q.x_hi = q.text ? 0u : hi;
    q.lim = q.text ? qpos : (((lo | hi) != 0) ? 0x7FFFFFFF : -1);
    return q;
}

// klo/khi: the two halves of the key's int64 bitfield (bits 62/63 may be set), kpos: its position.
__device__ __forceinline__ bool allow_pair(const QueryBits& q, unsigned klo, unsigned khi, int kpos) {
    const unsigned v = ((klo & q.a_lo) ^ q.x_lo) | ((khi & q.a_hi) ^ q.x_hi);
    const bool nz = v != 0u;
    const bool pos_ok = kpos <= q.lim;
    return (nz == q.text) & pos_ok;
}

// The part of the rule that does not depend on the key's position.
__device__ __forceinline__ bool allow_bits(const QueryBits& q, unsigned klo, unsigned khi) {
    const unsigned v = ((klo & q.a_lo) ^ q.x_lo) | ((khi & q.a_hi) ^ q.x_hi);
    return (v != 0u) == q.text;
}

// ---------------------------------------------------------------------------------
// Element types: raw 16-byte operands, MFMA and float -> T conversion.
struct BF16 {
    static __device__ __forceinline__ f32x16 mfma(const u32x4& a, const u32x4& b, const f32x16& c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ unsigned pack2(float x, float y) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        bf16x2 v;
        v[0] = (__bf16)x;
        v[1] = (__bf16)y;
        return __builtin_bit_cast(unsigned, v);
    }
    static __device__ __forceinline__ float to_float(unsigned short raw) {
        return __builtin_bit_cast(float, ((unsigned)raw) << 16);
    }
    // acc + the two elements of a packed pair
    static __device__ __forceinline__ float add_pair(unsigned packed, float acc) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, packed), __builtin_bit_cast(bf16x2, 0x3F803F80u), acc, false);
    }
};

struct F16 {
    static __device__ __forceinline__ f32x16 mfma(const u32x4& a, const u32x4& b, const f32x16& c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ unsigned pack2(float x, float y) {
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        f16x2 v;
        v[0] = (_Float16)x;
        v[1] = (_Float16)y;
        return __builtin_bit_cast(unsigned, v);
    }
    static __device__ __forceinline__ float to_float(unsigned short raw) {
        return (float)__builtin_bit_cast(_Float16, raw);
    }
    static __device__ __forceinline__ float add_pair(unsigned packed, float acc) {
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, packed), __builtin_bit_cast(f16x2, 0x3C003C00u), acc, false);
    }
};

// Eight consecutive C-fragment values -> one 16-byte MFMA operand of type T.
template <typename T>
__device__ __forceinline__ u32x4 pack8(const f32x16& c, int base) {
    u32x4 r;
    r[0] = T::pack2(c[base + 0], c[base + 1]);
    r[1] = T::pack2(c[base + 2], c[base + 3]);
    r[2] = T::pack2(c[base + 4], c[base + 5]);
    r[3] = T::pack2(c[base + 6], c[base + 7]);
    return r;
}

// Four consecutive elements key .. key + 3 of one row of an attention bias, as floats.  `row` points at the
// row's element for key 0; keys at or past Sk read as 0.  `vec`: the group is one aligned access that lies
// completely inside or completely outside the row (key is a multiple of four).
template <typename T>
__device__ __forceinline__ f32x4 load_bias4(const void* row, int key, int Sk, bool f32, bool vec) {
    f32x4 r = {0.f, 0.f, 0.f, 0.f};
    if (f32) {
        const float* pf = (const float*)row + key;
        if (vec) {
            if (key < Sk) r = *(const f32x4*)pf;
        } else {
#pragma unroll
            for (int x = 0; x < 4; ++x)
                if (key + x < Sk) r[x] = pf[x];
        }
    } else {
        const unsigned short* ph = (const unsigned short*)row + key;
        if (vec) {
            if (key < Sk) {
                const u32x2 w = *(const u32x2*)ph;
                r[0] = T::to_float((unsigned short)(w[0] & 0xFFFFu));
                r[1] = T::to_float((unsigned short)(w[0] >> 16));
                r[2] = T::to_float((unsigned short)(w[1] & 0xFFFFu));
                r[3] = T::to_float((unsigned short)(w[1] >> 16));
            }
        } else {
#pragma unroll
            for (int x = 0; x < 4; ++x)
                if (key + x < Sk) r[x] = T::to_float(ph[x]);
        }
    }
    return r;
}

// One element of an attention bias as float.
template <typename T>
__device__ __forceinline__ float load_bias1(const void* base, int64_t index, bool f32) {
    return f32 ? ((const float*)base)[index] : T::to_float(((const unsigned short*)base)[index]);
}

// ---------------------------------------------------------------------------------
// LDS tile layout.  A tile is ROWS x D elements of 2 bytes, stored as 16-byte chunks;
// chunk c of row r lives at chunk slot  r * (D/8) + (c ^ swz(r)).  The XOR pattern is a
// one-bit rotation of the 256-byte line number.  Access shapes used by the kernels:
//   * natural read  : 16 lanes read the same chunk column of 16 consecutive rows (conflict free);
//   * transposed read (ds_read_b64_tr_b16): 16 lanes read a 4-row x 32-byte block (conflict free
//     within the 16 lanes; the two blocks of a half wave overlap in two bank groups, which costs
//     two cycles per instruction, hidden inside the four cycles a wave-wide LDS instruction takes).
template <int D>
__device__ __forceinline__ int swz(int row) {
    constexpr int NCH = D / 8;                                       // chunks per row: 4, 8, 16
    constexpr int CB = (NCH == 16) ? 4 : (NCH == 8) ? 3 : 2;         // log2(NCH)
    const int line = (row >> (4 - CB)) & (NCH - 1);
    return ((line << 1) & (NCH - 1)) | (line >> (CB - 1));
}

template <int D>
__device__ __forceinline__ int chunk_slot(int row, int c) {
    return row * (D / 8) + (c ^ swz<D>(row));
}

// Natural MFMA operand: 8 consecutive elements (one chunk) of one row.
template <int D>
__device__ __forceinline__ u32x4 lds_read_chunk(const u32x4* tile, int row, int c) {
    return tile[chunk_slot<D>(row, c)];
}

// Transposed MFMA operand.  The caller wants, for column `col` of the tile, the elements
// of rows  row0+{0,1,2,3}  and  row0+8+{0,1,2,3}  (the k-slot order the 32x32 C fragment
// produces).  Within each group of 16 lanes the hardware hands lane i element i of the
// four 16-element rows assembled from the 8-byte pieces the lanes address, so lane i
// must address row (row0 + i/4), columns colbase16 + 4*(i%4) .. +3.
//   lane: lane id; row0: first row for THIS lane's half (already includes hi*4);
//   colbase16: first column of this lane's 16-column group.
template <int D>
__device__ __forceinline__ u32x4 lds_read_transposed(const u32x4* tile, int lane, int row0, int colbase16) {
    const int i = lane & 15;
    const int col = colbase16 + 4 * (i & 3);
    const int c = col >> 3;
    const int sub = (col & 4) ? 8 : 0;  // byte offset inside the chunk
    const int r_a = row0 + (i >> 2);
    const int r_b = r_a + 8;
    typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
    const char* base = (const char*)tile;
    const char* pa = base + chunk_slot<D>(r_a, c) * 16 + sub;
    const char* pb = base + chunk_slot<D>(r_b, c) * 16 + sub;
    s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(pa));
    s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(pb));
    u32x2 ua = __builtin_bit_cast(u32x2, a), ub = __builtin_bit_cast(u32x2, b);
    u32x4 r;
    r[0] = ua[0];
    r[1] = ua[1];
    r[2] = ub[0];
    r[3] = ub[1];
    return r;
}

// max / sum with the lane that holds the other half of the same row (lane ^ 32).
// v_permlane32_swap exchanges the upper 32 lanes of its first register with the lower 32
// lanes of its second one; started from two copies of x, every lane ends up holding both
// halves' values.  Written as inline asm with both registers read-write so that the two
// results stay distinct values for the compiler; the s_nop cover the VALU hazards around
// the instruction, which the compiler cannot see inside an asm block.
__device__ __forceinline__ void half_swap(float x, float& lo, float& hi) {
    lo = x;
    hi = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
}
__device__ __forceinline__ float half_swap_max(float x) {
    float a, b;
    half_swap(x, a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float half_swap_sum(float x) {
    float a, b;
    half_swap(x, a, b);
    return a + b;
}

// Scheduling hint: interleave `n` MFMAs with the LDS reads that feed them so that reads run
// `ahead` operands in front of their MFMA (reads_per_op LDS instructions per operand).  Must
// follow, in the same basic block, the n operand reads and the n MFMAs it orders.
template <int N, int AHEAD, int READS_PER_OP>
__device__ __forceinline__ void sched_pipeline_mfma_lds() {
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) __builtin_amdgcn_sched_group_barrier(0x100, READS_PER_OP, 0);
#pragma unroll
    for (int i = 0; i < N - AHEAD; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, READS_PER_OP, 0);
    }
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
}

// x as the sum of three values of the 16-bit type (for bf16: x to its full fp32 precision), packed into the first three
// of a lane's eight k-slots of an MFMA operand; the other slots are zero.  Multiplied by ones in the same slots of the
// other operand, an MFMA adds x to a whole row or column of its accumulator.  An infinite x stays infinite (one slot).
template <typename T>
__device__ __forceinline__ u32x4 split3_operand(float x) {
    const unsigned h = T::pack2(x, 0.f) & 0xFFFFu;
    const float fh = T::to_float((unsigned short)h);
    const float r1 = fabsf(fh) < INFINITY ? x - fh : 0.f;  // exact
    const unsigned l = T::pack2(r1, 0.f) & 0xFFFFu;
    const float r2 = r1 - T::to_float((unsigned short)l);
    const unsigned l2 = T::pack2(r2, 0.f) & 0xFFFFu;
    u32x4 r = {h | (l << 16), l2, 0u, 0u};
    return r;
}
// The matching operand of ones (1.0 in the 16-bit type, three slots).
template <typename T>
__device__ __forceinline__ u32x4 ones3_operand() {
    const unsigned one = T::pack2(1.f, 0.f) & 0xFFFFu;
    u32x4 r = {one | (one << 16), one, 0u, 0u};
    return r;
}

// Workgroups are dealt round-robin to the 8 XCDs.  Map a linear block id onto
// (unit, member) so that the `G` members of one unit land on the same XCD back to back
// (they share K/V through that XCD's L2) while consecutive units spread over all XCDs.
__device__ __forceinline__ void xcd_group_map(int bid, int num_units, int G, int& unit, int& member) {
    const int chunk = bid / (8 * G);
    const int r = bid - chunk * 8 * G;
    if ((chunk + 1) * 8 <= num_units) {
        unit = chunk * 8 + (r & 7);
        member = r >> 3;
    } else {
        unit = chunk * 8 + r / G;
        member = r % G;
    }
}

// Which (batch x row-group index, kv head, member of the kv group) a workgroup of the forward / dQ kernels takes.
// Within an XCD the hardware deals consecutive workgroups to the four shader engines in turn and starts them strictly
// in order, so four consecutive workgroups of an XCD should carry the same amount of work or the engines with the
// lighter ones idle behind the others.  With four (or a multiple of four) q heads per kv head they do: the heads of
// one kv head on the same rows.  Smaller groups are filled up with neighbouring kv heads (4 kv heads for G = 1, 2 for
// G = 2) -- same rows, same mask, other K / V -- instead of the next batch element or row group.
__device__ __forceinline__ void head_unit_map(int bid, int rows_units, int Hkv, int G, int& ub, int& hk, int& g) {
    int V = (G & 3) == 0 ? 1 : (G & 1) == 0 ? 2 : 4;  // kv heads per run of workgroups
    if (Hkv % V != 0) V = 1;
    const int HV = Hkv / V;
    int unit, member;
    xcd_group_map(bid, rows_units * HV, G * V, unit, member);
    ub = unit / HV;
    hk = (unit - ub * HV) * V + member / G;
    g = member % G;
}

}  // namespace bam
