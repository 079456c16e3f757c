// Forward kernel of bitfield-masked attention for gfx950 (template; instantiated by fwd.hip and fwd_long.hip).
// Reference semantics: cornstarch/kernel/bitfield_attention.py:236-523 (+ the split-KV merge
// :1292-1436, which a single pass over the keys makes unnecessary).
//
// Work decomposition
//   workgroup  = four 32-row slices of one (batch, q head), one per wave: a 128-row block, or, with a plan,
//                four slices that need about the same keys (sorted slice order).
//   key loop   = 64-key tiles taken from the class rows of those slices: tiles no slice needs are never
//                touched; a wave skips the tiles its own slice does not need, skips the mask where every
//                pair of its slice is allowed, and evaluates the bitfield rule in registers otherwise.
//   K/V tiles  = double buffered in LDS; the next tile is copied global -> LDS directly while
//                the current one is consumed.
// Math layout
//   S^T = K Q^T on v_mfma_f32_32x32x16 with K rows as the A operand (LDS) and Q as the B
//   operand (registers).  In the C fragment a lane owns ONE query (lane & 31) and 16 of the
//   32 keys of a block, so the running max / sum / rescale factors are per-lane scalars and
//   the only cross-lane traffic is one exchange with lane ^ 32.  P^T then feeds
//   O^T = V^T P^T straight from registers as the B operand; V^T comes from the row-major V
//   tile through the transposing LDS read.
#pragma once
#include "bam_common.h"
#include "bam_launch.h"
#include "bam_tiles.h"
#include <type_traits>

namespace bam {

constexpr int FWD_KT = 64;
constexpr int FWD_THREADS = 256;

// MODE (MASK_*): where allow / deny comes from.  MASK_INDEXED: query rows and keys carry explicit global
// positions (p.posq, p.posk) and the bitfield arrays are already gathered per local row / key
// (context-parallel shards, reference bitfield_attention.py:71-81).  MASK_DENSE: a materialized bool mask
// (the reference's sibling kernel, cornstarch/kernel/attention.py:184-232), read from global memory in the
// tiles the flags call partial.
// BIAS: an additive bias p.bias (reference bitfield_attention.py:410-434) is added to scale * q.k.
// LONG: sequences of more than MAX_LIST 64-key tiles (131072 keys), walked in several passes; the short form has no
// pass loop at all (a loop around the main loop costs registers and a few per cent).
template <typename T, int D, int MODE, bool BIAS, bool LONG>
__global__ __launch_bounds__(FWD_THREADS, D == 128 ? 2 : 3) void fwd_kernel(const AttnParams p) {
    constexpr int NCH = D / 8, KK = D / 16, DB = D / 32;
    __shared__ u32x4 sK[2][FWD_KT * NCH];
    __shared__ u32x4 sV[2][FWD_KT * NCH];
    __shared__ __attribute__((aligned(16))) int64_t sKbf[2][FWD_KT];  // raw bitfields of the tile's keys
    __shared__ __attribute__((aligned(16))) int sKpos[2][FWD_KT];     // their global positions (IDX only)
    __shared__ int sList[MAX_LIST];
    __shared__ int sCount;
    constexpr bool IDX = MODE == MASK_INDEXED, DENSE = MODE == MASK_DENSE;
    // DENSE with packed mask bits: per wave, the words of its 32 rows for the tile's two 32-key blocks
    __shared__ unsigned sRowBits[DENSE ? 2 : 1][4][DENSE ? 64 : 1];
    // BIAS in its per-key ("vector") form: the 64 values of the tile (raw words; 16-bit elements fill half)
    __shared__ __attribute__((aligned(16))) unsigned sBias[BIAS ? 2 : 1][BIAS ? 64 : 1];

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
    const WaveSlices ws = pick_wave_slices(p, b, grp);  // group 0 is the heaviest

    if (wave == 0) build_key_tile_list(ws, p.num_n, Sk, lane, 0, sList, &sCount);  // first pass (usually the only one)

    // ---- per-lane query state -------------------------------------------------------
    const int slice = __builtin_amdgcn_readfirstlane(wave == 0 ? ws.slice[0] : wave == 1 ? ws.slice[1] : wave == 2 ? ws.slice[2] : ws.slice[3]);
    const int qrow = (slice < 0 ? 0 : slice) * 32 + l32;
    const bool qvalid = slice >= 0 && qrow < Sq;
    u32x4 qreg[KK];
    {
        const char* qp = (const char*)p.q.ptr + 2 * ((int64_t)b * p.q.sb + (int64_t)qrow * p.q.ss + (int64_t)h * p.q.sh);
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            u32x4 z = {0u, 0u, 0u, 0u};
            if (qvalid) z = *(const u32x4*)(qp + (16 * kk + 8 * hi) * 2);
            qreg[kk] = z;
        }
    }
    const int64_t qf = (!DENSE && qvalid) ? p.bfq[(int64_t)b * p.bfq_sb + qrow] : 0;
    const QueryBits qb = make_query_bits(qf, (IDX && qvalid) ? p.posq[qrow] : qrow);

    f32x16 o[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
    // Online softmax state.  m_i is the reference maximum the exponentials are taken against;
    // it is only moved (and O, l rescaled) when a tile raises a row's maximum by more than
    // RESCALE_LOG2 in the exponent, so most tiles skip the rescale entirely.  Until then the
    // probabilities are at most 2^RESCALE_LOG2, harmless in fp32 / bf16 and cancelled by the
    // final division by l.
    constexpr float RESCALE_LOG2 = 8.f;
    float m_i = -INFINITY, l_i = 0.f, nb = 0.f;  // nb = -m_i * c2 (0 while m_i is -inf)
    // with a bias the scores are turned into scale * s + bias right after the S phase, and only log2(e) is left
    // to fold into the exponent
    // A per-key bias whose groups of four keys are aligned, in-range accesses travels with the tile copies: 64 values
    // per tile, one word per lane (16-bit elements: lanes 32..63 repeat lanes 0..31).
    const bool bias_lds = BIAS && p.bias_sm == 0 && p.bias_vec != 0;
    // ... and with bf16 operands it is added by the matrix cores: bias / scale, split into three bf16 values, rides in
    // one more MFMA of the S phase against an operand of ones, so that the scores come out as q.k + bias / scale and
    // the exponent is taken exactly as without a bias (no multiply-add per score, no bias reads per score).
    const bool bias_fold = bias_lds && std::is_same<T, BF16>::value;
    const float c2 = (BIAS && !bias_fold) ? LOG2E : p.scale * LOG2E;
    const float inv_scale = 1.f / p.scale;
    const char* bias_row = nullptr;  // this lane's row of the bias
    if (BIAS)
        bias_row = (const char*)p.bias + (p.bias_f32 ? 4 : 2) * ((int64_t)b * p.bias_sb + (int64_t)h * p.bias_sh +
                                                                (int64_t)(qvalid ? qrow : 0) * p.bias_sm);
    const float rescale_thr = RESCALE_LOG2 / c2;
    f32x16 zero16;
#pragma unroll
    for (int i = 0; i < 16; ++i) zero16[i] = 0.f;

    const char* kbase = (const char*)p.k.ptr + 2 * ((int64_t)b * p.k.sb + (int64_t)hk * p.k.sh);
    const char* vbase = (const char*)p.v.ptr + 2 * ((int64_t)b * p.v.sb + (int64_t)hk * p.v.sh);
    const int64_t k_ts = 2 * p.k.ss * FWD_KT, v_ts = 2 * p.v.ss * FWD_KT;  // bytes per tile
    const int64_t* bfrow = p.bfk + (int64_t)b * p.bfk_sb;

    typedef TileStage<D, FWD_KT, FWD_THREADS> Stage;
    constexpr int CPT = Stage::CPT;
    // copy instructions per wave and tile: K, V, the key bitfields (DENSE: the mask bits of the wave's rows) and
    // (IDX) the key positions
    constexpr int NLOADS = 2 * CPT + 1 + (IDX ? 1 : 0) + (BIAS ? 1 : 0);
    static_assert(NLOADS <= 2 * KK + 1, "one copy per MFMA of the S phase (and at most one behind it)");
    Stage stK, stV;
    stK.setup(2 * p.k.ss, tid);
    stV.setup(2 * p.v.ss, tid);
    const unsigned ldsK = lds_addr(sK), ldsV = lds_addr(sV), ldsB = lds_addr(sKbf), ldsP = lds_addr(sKpos);
    const unsigned ldsR = lds_addr(sRowBits);
    const char* bias_head = BIAS ? (const char*)p.bias + (p.bias_f32 ? 4 : 2) * ((int64_t)b * p.bias_sb + (int64_t)h * p.bias_sh) : nullptr;
    const unsigned bias_voff = (unsigned)((p.bias_f32 ? lane : (lane & 31)) * 4);
    const int bias_tile_bytes = FWD_KT * (p.bias_f32 ? 4 : 2);
    // DENSE: the packed mask rows of this wave's slice (null: no plan, the mask bytes are read instead)
    const unsigned* row_bits_w = (DENSE && p.row_bits != nullptr)
                                     ? p.row_bits + (int64_t)b * p.row_bits_sb + (slice < 0 ? 0 : slice) * 32
                                     : nullptr;
    const unsigned row_bits_voff = DENSE ? (unsigned)(hi * (int)p.row_bits_sn * 4 + l32 * 4) : 0u;
    constexpr unsigned TILE_BYTES = FWD_KT * NCH * 16, BITS_BYTES = FWD_KT * 8;
    // Copy instruction j (0 <= j < NLOADS) of full tile kt into buffer buf.  The 128 dwords of key
    // bitfields are copied 64 dwords per wave (waves 2, 3 repeat what waves 0, 1 write), so that every
    // wave issues the same number of copies.
    auto issue_copy = [&](int j, int kt, int buf) {
        if (j < CPT)
            stK.issue(j, kbase + kt * k_ts, ldsK + buf * TILE_BYTES);
        else if (j < 2 * CPT)
            stV.issue(j - CPT, vbase + kt * v_ts, ldsV + buf * TILE_BYTES);
        else if (j == 2 * CPT) {
            if (DENSE) {  // lanes 0..31: block 2 kt, lanes 32..63: block 2 kt + 1, rows of this wave's slice
                if (row_bits_w != nullptr)
                    dma_b32(row_bits_w + (int64_t)(2 * kt) * p.row_bits_sn, row_bits_voff, ldsR + (unsigned)(buf * 4 + wave) * 256u);
            } else {
                dma_b32(bfrow + kt * FWD_KT, (unsigned)((wave & 1) * 256 + lane * 4), ldsB + buf * BITS_BYTES + (wave & 1) * 256u);
            }
        }
        else if (IDX && j == 2 * CPT + 1)  // 64 positions; every wave writes the same values
            dma_b32(p.posk + kt * FWD_KT, (unsigned)(lane * 4), ldsP + buf * (FWD_KT * 4u));
        else if (bias_lds)  // BIAS: the tile's 64 bias values; every wave writes the same values
            dma_b32(bias_head + (int64_t)kt * bias_tile_bytes, bias_voff, lds_addr(sBias) + buf * 256u);
    };

    // One 64-key tile held in buffer `cur`.  With PREFETCH the copies of tile `kt_next` into the other
    // buffer are issued one per MFMA of the S phase, where the wave has nothing else to wait for.
    auto tile_step = [&](auto prefetch, int cur, int entry, int kt_next) {
        constexpr bool PREFETCH = decltype(prefetch)::value;
        // (the class is extracted with a per-lane copy of the wave number on purpose: with a skip branch the
        // compiler can prove wave-uniform it lays the loop out around that branch and the kernel loses ~8 %)
        const int kt = entry >> 8, cls = (entry >> (2 * wave_lane)) & 3;
        if (cls == 0) {  // nothing for this wave's slice in the tile: only keep the copies of the next one going
            if (PREFETCH) {
#pragma unroll
                for (int j = 0; j < NLOADS; ++j) issue_copy(j, kt_next, cur ^ 1);
            }
            return;
        }
        const u32x4* tK = sK[cur];
        const u32x4* tV = sV[cur];

        // ---- S^T = K Q^T : 64 keys x 32 queries per wave ----------------------------------
        // two independent accumulator chains (key blocks 0 and 1) alternate; operand reads run AHEAD
        // MFMAs in front of their use; the first MFMA of a chain takes C = 0
        // (the MFMA phases run at raised wave priority: when the SIMD's other wave is in its softmax phase, this
        // wave's next MFMA is picked first and the MFMA pipe does not idle behind a queue of VALU instructions)
        f32x16 s[2];
        u32x4 bias_a[2];  // bias_fold: this lane's key of either 32-key block, as an operand (keys are the rows of S^T)
        if (BIAS && PREFETCH && bias_fold) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const float bv = p.bias_f32 ? ((const float*)sBias[cur])[32 * kb + l32]
                                            : T::to_float(((const unsigned short*)sBias[cur])[32 * kb + l32]);
                const u32x4 z = {0u, 0u, 0u, 0u};
                bias_a[kb] = hi == 0 ? split3_operand<T>(bv * inv_scale) : z;
            }
        }
        __builtin_amdgcn_s_setprio(1);
        {
            constexpr int NOP = 2 * KK, AHEAD = 4;
            u32x4 ka[NOP];
#pragma unroll
            for (int j = 0; j < AHEAD; ++j) ka[j] = lds_read_chunk<D>(tK, 32 * (j & 1) + l32, 2 * (j >> 1) + hi);
#pragma unroll
            for (int j = 0; j < NOP; ++j) {
                __builtin_amdgcn_sched_barrier(0);
                if (j + AHEAD < NOP)
                    ka[j + AHEAD] = lds_read_chunk<D>(tK, 32 * ((j + AHEAD) & 1) + l32, 2 * ((j + AHEAD) >> 1) + hi);
                s[j & 1] = T::mfma(ka[j], qreg[j >> 1], j < 2 ? zero16 : s[j & 1]);
                if (PREFETCH && j < NLOADS) issue_copy(j, kt_next, cur ^ 1);
            }
            if (PREFETCH) {
#pragma unroll
                for (int j = NOP; j < NLOADS; ++j) issue_copy(j, kt_next, cur ^ 1);
            }
            if (BIAS && PREFETCH && bias_fold) {
                const u32x4 z = {0u, 0u, 0u, 0u};
                const u32x4 ones = hi == 0 ? ones3_operand<T>() : z;
                s[0] = T::mfma(bias_a[0], ones, s[0]);
                s[1] = T::mfma(bias_a[1], ones, s[1]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_setprio(0);

        if (BIAS && PREFETCH && bias_fold) {
            // (added by the MFMA above)
        } else if (BIAS && PREFETCH && bias_lds) {  // (the ragged last tile is staged without the bias)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int grp = 0; grp < 4; ++grp) {
                    const int koff = 32 * kb + 8 * grp + 4 * hi;
                    f32x4 b4;
                    if (p.bias_f32) {
                        b4 = *(const f32x4*)&sBias[cur][koff];
                    } else {
                        const u32x2 w = *(const u32x2*)((const char*)sBias[cur] + 2 * koff);
                        b4[0] = T::to_float((unsigned short)(w[0] & 0xFFFFu));
                        b4[1] = T::to_float((unsigned short)(w[0] >> 16));
                        b4[2] = T::to_float((unsigned short)(w[1] & 0xFFFFu));
                        b4[3] = T::to_float((unsigned short)(w[1] >> 16));
                    }
#pragma unroll
                    for (int x = 0; x < 4; ++x) s[kb][4 * grp + x] = fmaf(s[kb][4 * grp + x], p.scale, b4[x]);
                }
        } else if (BIAS) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int grp = 0; grp < 4; ++grp) {
                    const f32x4 b4 = load_bias4<T>(bias_row, kt * FWD_KT + 32 * kb + 8 * grp + 4 * hi, Sk, p.bias_f32 != 0, p.bias_vec != 0);
#pragma unroll
                    for (int x = 0; x < 4; ++x)
                        s[kb][4 * grp + x] = bias_fold ? fmaf(b4[x], inv_scale, s[kb][4 * grp + x])  // (c2 holds the scale)
                                                       : fmaf(s[kb][4 * grp + x], p.scale, b4[x]);
                }
        }

        // ---- bitfield rule in registers (partial tiles only) ------------------------------
        if (DENSE) {
            if (cls == 1 && row_bits_w != nullptr) {
                // (shifted by this lane's first key, 4 hi, once: the bit numbers tested are then constants)
                const unsigned w01[2] = {sRowBits[cur][wave][l32] >> (4 * hi), sRowBits[cur][wave][32 + l32] >> (4 * hi)};
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        s[kb][i] = ((w01[kb] >> (8 * (i >> 2) + (i & 3))) & 1u) ? s[kb][i] : -INFINITY;
            } else if (cls == 1) {
                // mask bytes of this lane's query row: 4 consecutive keys per C-fragment group
                const int kt0 = kt * FWD_KT;
                const uint8_t* mrow = p.mask + ((int64_t)b * Sq + (qvalid ? qrow : 0)) * Sk + kt0;
                const bool dwords = (Sk & 3) == 0;  // rows start 4-byte aligned
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int grp = 0; grp < 4; ++grp) {
                        const int koff = 32 * kb + 8 * grp + 4 * hi;
                        unsigned m4 = 0;
                        if (p.mask == nullptr) {
                            m4 = 0x01010101u;
                        } else if (qvalid) {
                            if (dwords) {
                                if (kt0 + koff < Sk) m4 = *(const unsigned*)(mrow + koff);
                            } else {
#pragma unroll
                                for (int x = 0; x < 4; ++x)
                                    if (kt0 + koff + x < Sk) m4 |= (unsigned)mrow[koff + x] << (8 * x);
                            }
                        }
#pragma unroll
                        for (int x = 0; x < 4; ++x) {
                            const bool a = ((m4 >> (8 * x)) & 0xFFu) != 0 && kt0 + koff + x < Sk;
                            s[kb][4 * grp + x] = a ? s[kb][4 * grp + x] : -INFINITY;
                        }
                    }
            }
        } else if (cls == 1) {
            // Most partial tiles are partial only through causality: all 64 keys carry the same bitfield (and,
            // with index tensors, sit at consecutive positions).  Then the bit test is a per-query constant and
            // the rule reduces to one position compare.
            const int64_t mine = sKbf[cur][lane];
            const unsigned mlo = (unsigned)mine, mhi = (unsigned)((uint64_t)mine >> 32);
            const unsigned flo = __builtin_amdgcn_readfirstlane(mlo), fhi = __builtin_amdgcn_readfirstlane(mhi);
            bool uniform = (mlo == flo) & (mhi == fhi);
            int kt0 = kt * FWD_KT;  // position of the tile's first key
            if (IDX) {
                const int rel0 = sKpos[cur][lane] - lane;
                kt0 = __builtin_amdgcn_readfirstlane(rel0);
                uniform &= rel0 == kt0;
            }
            if (__all(uniform)) {
                // last allowed key, relative to the first key this lane holds (4 hi): what it is compared with are
                // then compile-time constants, which occupy no registers
                const int rel = allow_bits(qb, flo, fhi) ? qb.lim - kt0 - 4 * hi : -1;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        s[kb][i] = (32 * kb + 8 * (i >> 2) + (i & 3) <= rel) ? s[kb][i] : -INFINITY;
            } else {
                // natural positions: the row's limit relative to the first key this lane holds, so that the position
                // test compares with compile-time constants
                const int lim_rel = qb.lim - (kt * FWD_KT + 4 * hi);
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int grp = 0; grp < 4; ++grp) {
                        const int koff = 32 * kb + 8 * grp + 4 * hi;
                        const u32x4 k01 = *(const u32x4*)&sKbf[cur][koff];      // lo0 hi0 lo1 hi1
                        const u32x4 k23 = *(const u32x4*)&sKbf[cur][koff + 2];  // lo2 hi2 lo3 hi3
                        const unsigned klo[4] = {k01[0], k01[2], k23[0], k23[2]};
                        const unsigned khi[4] = {k01[1], k01[3], k23[1], k23[3]};
                        u32x4 kp = {0u, 0u, 0u, 0u};
                        if (IDX) kp = *(const u32x4*)&sKpos[cur][koff];
#pragma unroll
                        for (int x = 0; x < 4; ++x) {
                            const bool pos_ok = IDX ? (int)kp[x] <= qb.lim : 32 * kb + 8 * grp + x <= lim_rel;
                            const bool a = allow_bits(qb, klo[x], khi[x]) & pos_ok;
                            s[kb][4 * grp + x] = a ? s[kb][4 * grp + x] : -INFINITY;
                        }
                    }
            }
        }

        // ---- online softmax (per-lane scalars) ----------------------------------------------
        // (four short chains instead of one long one: the wave issues in order and would sit out the latency of
        // every link)
        float mx[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            mx[c] = fmaxf(s[0][4 * c], s[1][4 * c]);
#pragma unroll
            for (int i = 1; i < 4; ++i) mx[c] = fmaxf(fmaxf(mx[c], s[0][4 * c + i]), s[1][4 * c + i]);
        }
        float mloc = half_swap_max(fmaxf(fmaxf(mx[0], mx[1]), fmaxf(mx[2], mx[3])));
        if (__any(mloc > m_i + rescale_thr)) {  // wave-uniform; rare after the first tiles
            const float mnew = fmaxf(m_i, mloc);
            const float muse = (mnew == -INFINITY) ? 0.f : mnew;
            const float alpha = __builtin_amdgcn_exp2f((m_i - muse) * c2);  // 0 when m_i = -inf
            m_i = mnew;
            nb = -muse * c2;
            l_i *= alpha;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s[0][i] = __builtin_amdgcn_exp2f(fmaf(s[0][i], c2, nb));
            s[1][i] = __builtin_amdgcn_exp2f(fmaf(s[1][i], c2, nb));
        }
        u32x4 pb[2][2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int t = 0; t < 2; ++t) pb[kb][t] = pack8<T>(s[kb], 8 * t);
        // row sum of the probabilities as the P V product sees them (rounded to T), two per instruction
        {
            float ps[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int x = 0; x < 4; ++x) ps[kb][t] = T::add_pair(pb[kb][t][x], ps[kb][t]);
            l_i += (ps[0][0] + ps[0][1]) + (ps[1][0] + ps[1][1]);
        }

        // ---- O^T += V^T P^T -------------------------------------------------------------------
        __builtin_amdgcn_s_setprio(1);
        {
            u32x4 va[2][2][DB];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int db = 0; db < DB; ++db)
                        va[kb][t][db] = lds_read_transposed<D>(tV, lane, 32 * kb + 16 * t + 4 * hi, 32 * db + 16 * half16);
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int db = 0; db < DB; ++db) o[db] = T::mfma(va[kb][t][db], pb[kb][t], o[db]);
            sched_pipeline_mfma_lds<4 * DB, (DB >= 2 ? 3 : 2), 2>();
        }
        __builtin_amdgcn_s_setprio(0);
    };

    // Sequences of more than MAX_LIST 64-key tiles are walked in several passes, each with a list of its own; the
    // softmax state lives in registers and simply carries over.
    const int nkt_total = (Sk + FWD_KT - 1) / FWD_KT;
    for (int kt_begin = 0;;) {
        __syncthreads();
        const int n_all = sCount;
        // A tile that holds the end of a sequence whose length is not a multiple of 64 is always the last
        // entry of the list; it is staged synchronously (zero fill past the end) after the main loop.
        const bool ragged = (Sk & (FWD_KT - 1)) != 0 && n_all > 0 &&
                            (__builtin_amdgcn_readfirstlane(sList[n_all > 0 ? n_all - 1 : 0]) >> 8) == ((Sk - 1) >> 6);
        const int n = n_all - (ragged ? 1 : 0);
        if (n > 0) {
            int entry = __builtin_amdgcn_readfirstlane(sList[0]);
            int next = __builtin_amdgcn_readfirstlane(sList[n > 1 ? 1 : 0]);
    #pragma unroll
            for (int j = 0; j < NLOADS; ++j) issue_copy(j, entry >> 8, 0);
            wait_async();
            __syncthreads();
            for (int it = 0; it < n; ++it) {
                const int cur = it & 1;
                // entry after next, requested now and picked up at the end of the iteration; past the end of the
                // list the last tile is simply copied again (into the buffer nobody reads any more)
                const int after = sList[it + 2 < n ? it + 2 : n - 1];
                tile_step(std::true_type{}, cur, entry, next >> 8);
                entry = next;
                next = __builtin_amdgcn_readfirstlane(after);
                wait_async();
                __syncthreads();
            }
        }
        if (ragged) {
            const int entry = __builtin_amdgcn_readfirstlane(sList[n_all - 1]);
            const int kt = entry >> 8, rows = Sk - kt * FWD_KT;
            stK.load_ragged(kbase + kt * k_ts, sK[0], rows, tid);
            stV.load_ragged(vbase + kt * v_ts, sV[0], rows, tid);
            if (!DENSE && tid < FWD_KT) {
                sKbf[0][tid] = (tid < rows) ? bfrow[kt * FWD_KT + tid] : 0;
                if (IDX) sKpos[0][tid] = (tid < rows) ? p.posk[kt * FWD_KT + tid] : 0;
            }
            if (DENSE && row_bits_w != nullptr)
                sRowBits[0][wave][lane] = row_bits_w[(int64_t)(2 * kt + hi) * p.row_bits_sn + l32];
            __syncthreads();
            tile_step(std::false_type{}, 0, entry, 0);
        }
        if (!LONG) break;
        kt_begin += MAX_LIST;
        if (kt_begin >= nkt_total) break;
        __syncthreads();  // everybody has read the list of the pass that just ended
        if (wave == 0) build_key_tile_list(ws, p.num_n, Sk, lane, kt_begin, sList, &sCount);
    }

    // ---- epilogue: normalize, write O (q dtype) and LSE (natural log) -------------------
    const float ltot = half_swap_sum(l_i);
    const float inv = ltot > 0.f ? 1.f / ltot : 0.f;
    if (hi == 0 && slice >= 0)
        p.lse[((int64_t)b * p.Hq + h) * p.Sq_rounded + qrow] =
            ltot > 0.f ? (m_i * c2 + __builtin_amdgcn_logf(ltot)) * LN2 : -INFINITY;
    // A wave without a slice (plan: slot 4 grp + wave of the order lies past the last slice) owns the 32 padding rows
    // of that slot, so that every row of the rounded lse is written whether or not a plan is given.
    if (hi == 0 && slice < 0 && 32 * (4 * grp + wave) + 31 < p.Sq_rounded)
        p.lse[((int64_t)b * p.Hq + h) * p.Sq_rounded + 32 * (4 * grp + wave) + l32] = -INFINITY;
    if (qvalid) {
        char* op = (char*)p.o.ptr + 2 * ((int64_t)b * p.o.sb + (int64_t)qrow * p.o.ss + (int64_t)h * p.o.sh);
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int grp = 0; grp < 4; ++grp) {
                u32x2 w;
                w[0] = T::pack2(o[db][4 * grp + 0] * inv, o[db][4 * grp + 1] * inv);
                w[1] = T::pack2(o[db][4 * grp + 2] * inv, o[db][4 * grp + 3] * inv);
                *(u32x2*)(op + (32 * db + 8 * grp + 4 * hi) * 2) = w;
            }
    }
}


// Launches every (mask mode, bias) instantiation of one (element type, head dim, LONG) combination.
template <typename T, int D, bool BIAS, bool LONG>
static int launch_fwd_b(const AttnParams& p, hipStream_t stream) {
    const int blocks = p.num_m * p.B * p.Hq;
    if (p.mask_mode == MASK_INDEXED)
        hipLaunchKernelGGL((fwd_kernel<T, D, MASK_INDEXED, BIAS, LONG>), dim3(blocks), dim3(FWD_THREADS), 0, stream, p);
    else if (p.mask_mode == MASK_DENSE)
        hipLaunchKernelGGL((fwd_kernel<T, D, MASK_DENSE, BIAS, LONG>), dim3(blocks), dim3(FWD_THREADS), 0, stream, p);
    else
        hipLaunchKernelGGL((fwd_kernel<T, D, MASK_BITFIELD, BIAS, LONG>), dim3(blocks), dim3(FWD_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}
template <typename T, int D, bool LONG>
static int launch_fwd_t(const AttnParams& p, hipStream_t stream) {
    return p.bias != nullptr ? launch_fwd_b<T, D, true, LONG>(p, stream) : launch_fwd_b<T, D, false, LONG>(p, stream);
}
template <bool LONG>
static int launch_fwd_all(const AttnParams& p, int dtype, hipStream_t stream) {
    if (dtype == 1) {
        if (p.D == 128) return launch_fwd_t<BF16, 128, LONG>(p, stream);
        if (p.D == 64) return launch_fwd_t<BF16, 64, LONG>(p, stream);
        return launch_fwd_t<BF16, 32, LONG>(p, stream);
    }
    if (p.D == 128) return launch_fwd_t<F16, 128, LONG>(p, stream);
    if (p.D == 64) return launch_fwd_t<F16, 64, LONG>(p, stream);
    return launch_fwd_t<F16, 32, LONG>(p, stream);
}

}  // namespace bam
