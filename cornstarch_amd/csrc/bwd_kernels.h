// Backward kernels of bitfield-masked attention for gfx950 (templates; instantiated by bwd_dkdv.hip, bwd_dq.hip
// and bwd_long.hip).
// Reference semantics: cornstarch/kernel/bitfield_attention.py:527-572 (delta) and :598-929
// (dQ, dK, dV).  The reference accumulates dQ, dK and dV with fp32 atomics; here every output
// element has exactly one owner, so nothing is atomic and the sums are deterministic:
//   dkdv kernel : one workgroup per (batch, kv head, 128-key tile); it loops over the q heads
//                 of the group and over the query blocks its flag column lists.
//   dq kernel   : one workgroup per (batch, q head, 128-query block), looping over key tiles
//                 exactly like the forward kernel.
// Both recompute P = exp(scale * s - lse) from the saved log-sum-exp.
#pragma once
#include "bam_common.h"
#include "bam_launch.h"
#include "bam_tiles.h"
#include <type_traits>

namespace bam {

// ---------------------------------------------------------------------------------------
// delta[b,h,i] = sum_d o * do   (fp32).  D/8 lanes per row, 16 bytes per lane per tensor.
template <typename T, int D>
__global__ __launch_bounds__(256) void bwd_preprocess_kernel(const AttnParams p) {
    constexpr int LPR = D / 8;
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t row = gid / LPR;
    const int c = (int)(gid % LPR);
    const int64_t total = (int64_t)p.B * p.Sq * p.Hq;
    const bool valid = row < total;
    int h = 0, i = 0, b = 0;
    float acc = 0.f;
    if (valid) {
        h = (int)(row % p.Hq);
        const int64_t bi = row / p.Hq;
        i = (int)(bi % p.Sq);
        b = (int)(bi / p.Sq);
        const u32x4 ov = *(const u32x4*)((const char*)p.o.ptr +
                                         2 * ((int64_t)b * p.o.sb + (int64_t)i * p.o.ss + (int64_t)h * p.o.sh) + c * 16);
        const u32x4 gv = *(const u32x4*)((const char*)p.dout.ptr +
                                         2 * ((int64_t)b * p.dout.sb + (int64_t)i * p.dout.ss + (int64_t)h * p.dout.sh) + c * 16);
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            acc += T::to_float((unsigned short)(ov[x] & 0xFFFFu)) * T::to_float((unsigned short)(gv[x] & 0xFFFFu));
            acc += T::to_float((unsigned short)(ov[x] >> 16)) * T::to_float((unsigned short)(gv[x] >> 16));
        }
    }
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (valid && c == 0) p.delta[((int64_t)b * p.Hq + h) * p.Sq_rounded + i] = acc;
}

// ---------------------------------------------------------------------------------------
// dK, dV.  One workgroup = one 128-key tile of one (batch, kv head), 8 waves: wave w owns keys
// [32 (w & 3), +32) and works on rows [32 (w >> 2), +32) of every 64-row tile of Q / dO that streams
// through LDS (double buffered), so each SIMD holds two waves whose MFMA and softmax phases
// interleave.  A 64-row tile is a PAIR of 32-row slices taken from the list of slices that have work
// for this key tile (they need not be neighbours in the sequence), one slice per row stream; a wave
// whose own 32 x 32 class is "empty" sits the tile out.  K and V of the tile sit in LDS for the whole kernel and are
// read as MFMA B operands; dK^T and dV^T (d x keys) stay in accumulators.
// With S = Q K^T computed as queries x keys, a lane of the C fragment owns ONE key and 16
// query rows, so P and dS feed dV^T = dO^T P and dK^T = Q^T dS as B operands from registers;
// Q^T and dO^T come from the transposing LDS read of the same row-major tiles.
// The two waves that share a key group hold partial sums; they add them to the caller's
// buffers one after the other (workgroup barrier in between), so the result stays
// deterministic and atomic free.
constexpr int DKDV_QT = 64;
constexpr int DKDV_THREADS = 512;

// MODE (MASK_*): MASK_INDEXED = explicit global positions p.posq / p.posk and gathered bitfield arrays;
// MASK_DENSE = a materialized bool mask read from global memory in partial tiles.
// BIAS: the forward added p.bias to scale * q.k (reference bitfield_attention.py:815-835); P is recomputed with it.
// LONG: sequences of more than MAX_SLICE_LIST 32-row slices (131072 rows), walked in several passes; the short form has
// no pass loop at all (a loop around the main loop costs registers and a few per cent).
// SAVE: every wave also stores its 32 x 32 block of -dS / scale (the packed operand of the dK product) to p.ds_ws, where
// the dQ kernel of bwd_dq_saved.h picks it up instead of recomputing S and dP.  Record and block layout: AttnParams.
template <typename T, int D, int MODE, bool BIAS, bool LONG, bool SAVE = false>
__global__ __launch_bounds__(DKDV_THREADS, 2) void bwd_dkdv_kernel(const AttnParams p) {
    constexpr bool IDX = MODE == MASK_INDEXED, DENSE = MODE == MASK_DENSE;
    constexpr int NCH = D / 8, KK = D / 16, DB = D / 32;
    __shared__ u32x4 sK[128 * NCH];
    __shared__ u32x4 sV[128 * NCH];
    __shared__ u32x4 sQ[2][DKDV_QT * NCH];
    __shared__ u32x4 sDO[2][DKDV_QT * NCH];
    __shared__ __attribute__((aligned(16))) float sLse[2][DKDV_QT];      // natural-log lse of the rows
    __shared__ __attribute__((aligned(16))) float sDelta[2][DKDV_QT];
    __shared__ __attribute__((aligned(16))) int64_t sQbf[2][DKDV_QT];    // raw bitfields of the rows
    __shared__ __attribute__((aligned(16))) int sQpos[2][DKDV_QT];       // their global positions (IDX only)
    __shared__ __attribute__((aligned(16))) unsigned sWq[DKDV_THREADS / 64][5][32];  // per-wave rule constants
    // DENSE with packed mask bits: for the two slices of the tile, one word per key of the workgroup's 128 keys
    __shared__ unsigned sColBits[MODE == MASK_DENSE ? 2 : 1][2][MODE == MASK_DENSE ? 128 : 1];
    __shared__ int sListStore[MAX_SLICE_LIST + 1];  // entry -1: partner of the first entry of an odd count
    int* const sList = sListStore + 1;
    __shared__ int sCount;

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kg = wave & 3, st = wave >> 2;
    const int hi = lane >> 5, l32 = lane & 31, half16 = (lane >> 4) & 1;
    const int Sq = p.Sq, Sk = p.Sk;
    const int G = p.Hq / p.Hkv;

    const int unit = blockIdx.x;
    const int hk = unit % p.Hkv;
    int ub = unit / p.Hkv;  // position of the (batch, key tile) in the order of falling work
    {
        // The hardware deals the workgroups of an XCD to its four shader engines in turn and launches them strictly
        // in order: a workgroup waits for a free compute unit on ITS engine while free units of the other engines sit
        // idle behind it.  In a plainly sorted list one engine would get the heaviest workgroup of every four and
        // hold everybody back (measured: units idle 19 us at the median, up to 90 us, before their second workgroup),
        // so every other run of 32 workgroups -- four per XCD, one per engine -- takes its tiles in reverse.
        const int P = (p.Hkv <= 32 && 32 % p.Hkv == 0) ? 32 / p.Hkv : 1;
        const int g = ub / P, r = ub - g * P;
        if ((g & 1) && (g + 1) * P <= p.num_kt * p.B) ub = g * P + (P - 1 - r);
    }
    int b = ub % p.B;
    int nt = ub / p.B;  // early key tiles (most queries under causality) first
    if (p.tile_order != nullptr) {  // with a plan: the tiles by falling amount of work, whatever the mask looks like
        const int code = p.tile_order[ub];
        b = code / p.num_kt;
        nt = code - b * p.num_kt;
    }

    const int ns_total = (Sq + 31) >> 5;
    // first pass (usually the only one): the last MAX_SLICE_LIST slices
    if (wave == 0) build_slice_list(p, b, nt, lane, max(0, ns_total - MAX_SLICE_LIST), ns_total, sList, &sCount);

    // ---- K, V of the tile -> LDS (once) ---------------------------------------------------
    {
        TileStage<D, 128, DKDV_THREADS> stK, stV;
        stK.setup(2 * p.k.ss, tid);
        stV.setup(2 * p.v.ss, tid);
        const char* kb = (const char*)p.k.ptr + 2 * ((int64_t)b * p.k.sb + (int64_t)hk * p.k.sh + (int64_t)nt * 128 * p.k.ss);
        const char* vb = (const char*)p.v.ptr + 2 * ((int64_t)b * p.v.sb + (int64_t)hk * p.v.sh + (int64_t)nt * 128 * p.v.ss);
        stK.load(kb, sK, Sk - nt * 128, tid);
        stV.load(vb, sV, Sk - nt * 128, tid);
    }
    const int key = nt * 128 + kg * 32 + l32;
    const bool kvalid = key < Sk;
    const int64_t* bfrow = p.bfq + (int64_t)b * p.bfq_sb;  // bitfields of the query rows
    const int64_t kf = (!DENSE && kvalid) ? p.bfk[(int64_t)b * p.bfk_sb + key] : 0;
    int kpos = (IDX && kvalid) ? p.posk[key] : key;  // global position of this lane's key
    unsigned klo = (unsigned)(kf & 0xFFFFFFFFll);
    unsigned khi = (unsigned)((uint64_t)kf >> 32);
    // Pin the arrival of this load here.  Left alone, the compiler waits for it at the first use inside the
    // main loop, with a vmcnt that also (and every time round) drains the tile copies it does not know about.
    asm volatile("" : "+v"(klo), "+v"(khi), "+v"(kpos));

    f32x16 dk[DB], dv[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            dk[db][i] = 0.f;
            dv[db][i] = 0.f;
        }
    f32x16 zero16;
#pragma unroll
    for (int i = 0; i < 16; ++i) zero16[i] = 0.f;
    const float c2 = BIAS ? LOG2E : p.scale * LOG2E;  // with a bias the scores become scale * s + bias first

    // Flip the sign of every element of the V tile in LDS (once per workgroup, after the tile has landed and
    // before anybody reads it; the caller brackets it with workgroup barriers).
    auto negate_v_tile = [&]() {
#pragma unroll
        for (int i = 0; i < (128 * NCH) / DKDV_THREADS; ++i) {
            u32x4 x = sV[tid + DKDV_THREADS * i];
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] ^= 0x80008000u;
            sV[tid + DKDV_THREADS * i] = x;
        }
    };
    bool v_negated = false;
    // Head dims up to 64 leave room for this wave's K and (negated) V operands of the S / dP phase in registers:
    // they are the same for every tile, and the phase then reads half as much from LDS.
    constexpr bool KV_REGS = D <= 64;
    u32x4 kfrag[KV_REGS ? KK : 1], vfrag[KV_REGS ? KK : 1];
    bool kv_loaded = false;
    auto load_kv_operands = [&]() {  // after the V tile has been negated and a barrier has published it
        if (KV_REGS && !kv_loaded) {
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                kfrag[kk] = lds_read_chunk<D>(sK, 32 * kg + l32, 2 * kk + hi);
                vfrag[kk] = lds_read_chunk<D>(sV, 32 * kg + l32, 2 * kk + hi);
            }
            kv_loaded = true;
        }
    };

    typedef SliceStage<D, DKDV_THREADS> Stage;
    constexpr int CPT = Stage::CPT;
    // copy instructions per wave and tile: Q, dO, one of the four small rows and (IDX) the row positions
    constexpr int NLOADS = 2 * CPT + 1 + (IDX ? 1 : 0);
    static_assert(NLOADS <= 2 * KK, "one copy per MFMA of the S / dP phase");
    Stage stQ, stDO;
    stQ.setup(2 * p.q.ss, tid);
    stDO.setup(2 * p.dout.ss, tid);
    const unsigned ldsQ = lds_addr(sQ), ldsDO = lds_addr(sDO);
    constexpr unsigned TILE_BYTES = DKDV_QT * NCH * 16;
    // small rows of a tile: lse, delta and the two halves of the 64 int64 bitfields, 64 dwords each;
    // wave w copies row w & 3 (waves 4..7 repeat what waves 0..3 write, so that every wave issues the same
    // number of copies)
    // (DENSE: rows 2 and 3 are the packed mask words of keys 0..63 / 64..127 of the tile, for the slice of the
    // copying wave's row stream; without packed bits, waves 2, 3, 6, 7 repeat lse / delta instead)
    const bool col_bits_on = DENSE && p.col_bits != nullptr;
    const int small = (DENSE && !col_bits_on) ? (wave & 1) : (wave & 3);
    const unsigned ldsSmall = small == 0   ? lds_addr(sLse)
                              : small == 1 ? lds_addr(sDelta)
                              : DENSE      ? lds_addr(sColBits) + (unsigned)(st * 128 + (small - 2) * 64) * 4u
                                           : lds_addr(sQbf) + (small - 2) * 256u;
    const unsigned smallBytes = small < 2 ? DKDV_QT * 4u : DENSE ? 2 * 128 * 4u : DKDV_QT * 8u;  // per buffer
    // Where the copies of a tile read.  The scalar unit is shared by the whole compute unit, so the address
    // arithmetic is kept short: per-head base pointers are carried along and bumped when the head changes, row
    // offsets are 32 x 32 -> 64 bit unsigned products (rows < 2^22, row strides < 2^25 bytes by the host checks).
    struct HeadBase {
        const char* q;      // first row of the head in q
        const char* g;      // ... in dout
        const char* small;  // this wave's small row: lse / delta of the head, or the bitfields (head independent)
    };
    const unsigned q_rs = (unsigned)(2 * p.q.ss), g_rs = (unsigned)(2 * p.dout.ss);  // row strides in bytes
    const int64_t small_head_step = small < 2 ? (int64_t)p.Sq_rounded * 4 : 0;
    auto head_base = [&](int h) {
        HeadBase hb;
        hb.q = (const char*)p.q.ptr + 2 * ((int64_t)b * p.q.sb + (int64_t)h * p.q.sh);
        hb.g = (const char*)p.dout.ptr + 2 * ((int64_t)b * p.dout.sb + (int64_t)h * p.dout.sh);
        hb.small = small == 0   ? (const char*)(p.lse + ((int64_t)b * p.Hq + h) * p.Sq_rounded)
                   : small == 1 ? (const char*)(p.delta + ((int64_t)b * p.Hq + h) * p.Sq_rounded)
                   : DENSE      ? (const char*)(p.col_bits + (int64_t)b * p.col_bits_sb + nt * 128 + (small - 2) * 64)
                                : (const char*)bfrow;
        return hb;
    };
    auto next_head = [&](HeadBase& hb) {
        hb.q += 2 * (int64_t)p.q.sh;
        hb.g += 2 * (int64_t)p.dout.sh;
        hb.small += small_head_step;
    };
    // lanes 32..63 of a copy of 2 x 32 consecutive floats / ints take the second slice: their byte offset moves
    // from "the rows after the first slice" to it
    const unsigned upper_lanes = lane >= 32 ? 0xFFFFFFFFu : 0u;
    struct TileSource {
        const char* q[CPT];
        const char* g[CPT];
        const char* small;
        const int* pos;
        unsigned small_voff, pos_voff;
    };
    // the 64-row tile made of the slices starting at rows row_lo (LDS rows 0..31) and row_hi (LDS rows 32..63)
    auto tile_source = [&](const HeadBase& hb, int row_lo, int row_hi) {
        TileSource t;
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const unsigned row = (unsigned)(stQ.upper(i) ? row_hi : row_lo);
            t.q[i] = hb.q + (uint64_t)row * q_rs;
            t.g[i] = hb.g + (uint64_t)row * g_rs;
        }
        // lse / delta (small < 2): 32 floats of each slice.  Bitfields: 32 int64 = 64 dwords of slice lo
        // (small == 2) or hi (small == 3).
        const unsigned srow = (unsigned)(small == 3 ? row_hi : row_lo);
        if (DENSE && small >= 2)  // the words of the slice this wave's row stream works on
            t.small = hb.small + (uint64_t)((unsigned)(st ? row_hi : row_lo) >> 5) * (uint64_t)(p.col_bits_ss * 4);
        else
            t.small = hb.small + (small < 2 ? srow * 4u : srow * 8u);
        const unsigned shift = (unsigned)((row_hi - row_lo - 32) * 4);
        t.pos_voff = (unsigned)(lane * 4) + (shift & upper_lanes);
        t.small_voff = small < 2 ? t.pos_voff : (unsigned)(lane * 4);
        t.pos = IDX ? p.posq + row_lo : nullptr;
        return t;
    };
    // copy instruction j of a tile into buffer buf
    auto issue_copy = [&](int j, const TileSource& t, int buf) {
        if (j < CPT)
            stQ.issue_from(j, t.q[j], ldsQ + buf * TILE_BYTES);
        else if (j < 2 * CPT)
            stDO.issue_from(j - CPT, t.g[j - CPT], ldsDO + buf * TILE_BYTES);
        else if (j == 2 * CPT)
            dma_b32(t.small, t.small_voff, ldsSmall + buf * smallBytes);
        else  // 2 x 32 row positions; every wave writes the same values
            dma_b32(t.pos, t.pos_voff, lds_addr(sQpos) + buf * (DKDV_QT * 4u));
    };

    // One 64-row tile held in buffer cur against this wave's 32 keys; the wave's 32 rows sit at sequence
    // rows myrow0.. and its class for them is cls.  With PREFETCH the copies of the next tile into the other buffer
    // are issued one per MFMA of the S / dP phase, or back to back when this wave has nothing to compute.
    const int qr = 32 * st;  // this wave's rows inside the 64-row tile
    // The wave's flag class is extracted with a per-lane copy of the key group number on purpose: a branch
    // condition the compiler can prove wave-uniform makes it restructure the loop around that branch, and the
    // result needs far more registers than a wave has.
    const int kg_lane = (tid >> 6) & 3;
    // SAVE: where this lane's 32 bytes sit inside a 2 KiB block (key l32: 64 bytes, rows 4 hi + {0..3, 8..11, ...} first)
    const unsigned ds_lane_off = (unsigned)(kg * 2048 + l32 * 64 + hi * 32);
    // SAVE: the pairs (slice, this key tile) that have work are numbered consecutively from ds_base, by ascending slice,
    // i.e. in the order of the slice list: pair number = ds_base + position in the list
    int ds_base = 0;
    if (SAVE) ds_base = __builtin_amdgcn_readfirstlane(p.ds_tile_base[(int64_t)b * p.num_kt + nt]);
    // BIAS, per-key form (row stride 0): this lane's bias value for the head in work
    float bias_key = 0.f;
    int bias_head = -1;
    auto fetch_bias_key = [&](int h) {
        if (BIAS && p.bias_sm == 0 && h != bias_head) {
            bias_head = h;
            bias_key = kvalid ? load_bias1<T>(p.bias, (int64_t)b * p.bias_sb + (int64_t)h * p.bias_sh + key, p.bias_f32 != 0) : 0.f;
            asm volatile("" : "+v"(bias_key));  // arrives here, not at its first use between the tile copies
        }
    };
    // ds_pos: position of the wave's slice in the slice list.
    // returns true when the wave has issued its two dS stores (they may stay in flight over the end of the iteration)
    auto tile_step = [&](auto prefetch, int cur, int cls, int h_cur, int myrow0, int ds_pos, const TileSource& next) -> bool {
        constexpr bool PREFETCH = decltype(prefetch)::value;
        if (cls == 0) {
            if (PREFETCH) {
#pragma unroll
                for (int j = 0; j < NLOADS; ++j) issue_copy(j, next, cur ^ 1);
            }
            return false;
        }
        const int ds_e = ds_base + ds_pos;
        const u32x4* tQ = sQ[cur];
        const u32x4* tG = sDO[cur];
        // ---- S = Q K^T and dP = dO V^T : 32 queries x 32 keys, two accumulator chains; both operands of
        // every MFMA come from LDS and are requested AHEAD MFMAs in front of their use
        // The V tile in LDS is NEGATED (see negate_v_tile), and the dP accumulator starts from delta instead of
        // zero: the chain then delivers delta - dO V^T = -(dP - delta) with no subtraction left for the VALU.
        // The sign is carried through dS into dK and taken back by the epilogue.
        f32x16 s, dp;
        {
            constexpr int NOP = 2 * KK, AHEAD = 3;  // MFMA j: S (j even) or dP (j odd), k-slice j / 2
            u32x4 a[NOP], bb[NOP];
            a[0] = lds_read_chunk<D>(tQ, qr + l32, hi);  // the operands of the first MFMA go first
            bb[0] = KV_REGS ? kfrag[0] : lds_read_chunk<D>(sK, 32 * kg + l32, hi);
#pragma unroll
            for (int grp = 0; grp < 4; ++grp) {
                const f32x4 d4 = *(const f32x4*)&sDelta[cur][qr + 8 * grp + 4 * hi];
#pragma unroll
                for (int x = 0; x < 4; ++x) dp[4 * grp + x] = d4[x];
            }
#pragma unroll
            for (int j = 1; j < AHEAD; ++j) {
                a[j] = lds_read_chunk<D>((j & 1) ? tG : tQ, qr + l32, 2 * (j >> 1) + hi);
                bb[j] = KV_REGS ? ((j & 1) ? vfrag[j >> 1] : kfrag[j >> 1])
                                : lds_read_chunk<D>((j & 1) ? sV : sK, 32 * kg + l32, 2 * (j >> 1) + hi);
            }
#pragma unroll
            for (int j = 0; j < NOP; ++j) {
                __builtin_amdgcn_sched_barrier(0);
                if (j + AHEAD < NOP) {
                    a[j + AHEAD] = lds_read_chunk<D>(((j + AHEAD) & 1) ? tG : tQ, qr + l32, 2 * ((j + AHEAD) >> 1) + hi);
                    bb[j + AHEAD] = KV_REGS ? (((j + AHEAD) & 1) ? vfrag[(j + AHEAD) >> 1] : kfrag[(j + AHEAD) >> 1])
                                            : lds_read_chunk<D>(((j + AHEAD) & 1) ? sV : sK, 32 * kg + l32, 2 * ((j + AHEAD) >> 1) + hi);
                }
                if (j & 1)
                    dp = T::mfma(a[j], bb[j], dp);
                else
                    s = T::mfma(a[j], bb[j], j < 2 ? zero16 : s);
                if (PREFETCH && j < NLOADS) issue_copy(j, next, cur ^ 1);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- P = exp(scale s - lse) on allowed pairs, -dS/scale = P (delta - dP)   (the factor `-scale` of dS
        // is applied once to dK in the epilogue).  C fragment: register i <-> query row
        // 8*(i/4) + 4*hi + i%4 of this wave's 32 rows.
        if (BIAS && p.bias_sm == 0) {
            // the per-key ("vector") form: one value per key and head, fetched when the head changes
#pragma unroll
            for (int i = 0; i < 16; ++i) s[i] = fmaf(s[i], p.scale, bias_key);
        } else if (BIAS) {
            // column `key` of the bias, one element per row of the C fragment
            const int64_t col = (int64_t)b * p.bias_sb + (int64_t)h_cur * p.bias_sh + key;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int row = myrow0 + 8 * (i >> 2) + 4 * hi + (i & 3);
                float bv = 0.f;
                if (kvalid && row < Sq) bv = load_bias1<T>(p.bias, col + (int64_t)row * p.bias_sm, p.bias_f32 != 0);
                s[i] = fmaf(s[i], p.scale, bv);
            }
        }
#pragma unroll
        for (int grp = 0; grp < 4; ++grp) {
            const f32x4 l4 = *(const f32x4*)&sLse[cur][qr + 8 * grp + 4 * hi];
#pragma unroll
            for (int x = 0; x < 4; ++x) s[4 * grp + x] = __builtin_amdgcn_exp2f(fmaf(s[4 * grp + x], c2, l4[x] * -LOG2E));
        }
        if (DENSE) {
            if (cls == 1 && col_bits_on) {
                // (shifted by this lane's first row, 4 hi, once: the bit numbers tested are then constants)
                const unsigned w = sColBits[cur][st][32 * kg + l32] >> (4 * hi);
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = ((w >> (8 * (i >> 2) + (i & 3))) & 1u) ? s[i] : 0.f;
            } else if (cls == 1) {
                // mask bytes of this lane's key column, one per row of the C fragment
                const uint8_t* mcol = p.mask + ((int64_t)b * Sq + myrow0) * Sk + key;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int r = 8 * (i >> 2) + 4 * hi + (i & 3);
                    bool a = kvalid && myrow0 + r < Sq;
                    if (a && p.mask != nullptr) a = mcol[(int64_t)r * Sk] != 0;
                    s[i] = a ? s[i] : 0.f;
                }
            }
        } else if (cls == 1) {
            // Most partial tiles are partial only through causality: the 32 rows carry the same bitfield.
            // Then the bit test is a per-key constant and the rule reduces to one position compare.
            const int64_t mine = sQbf[cur][qr + l32];
            const unsigned mlo = (unsigned)mine, mhi = (unsigned)((uint64_t)mine >> 32);
            const unsigned flo = __builtin_amdgcn_readfirstlane(mlo), fhi = __builtin_amdgcn_readfirstlane(mhi);
            bool uniform = (mlo == flo) & (mhi == fhi);
            int qpos0 = myrow0;  // position of this wave's first row
            if (IDX) {              // ... and the 32 rows must sit at consecutive positions
                const int rel0 = sQpos[cur][qr + l32] - l32;
                qpos0 = __builtin_amdgcn_readfirstlane(rel0);
                uniform &= rel0 == qpos0;
            }
            if (__all(uniform)) {
                const QueryBits qu = make_query_bits(((int64_t)fhi << 32) | (int64_t)flo, 0);
                const bool ok = allow_bits(qu, klo, khi) & (qu.text | (qu.lim >= 0));
                // allowed iff krel <= 8 * grp + x  (text rows: key position <= row position)
                const int krel = !ok ? 0x7FFFFFFF : qu.text ? kpos - qpos0 - 4 * hi : (int)0x80000000;
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = (krel <= 8 * (i >> 2) + (i & 3)) ? s[i] : 0.f;
            } else {
                // rule constants of this wave's 32 rows, derived once per row (lane r < 32 takes row r) and
                // handed to all lanes through a wave-private LDS scratch
                {
                    const QueryBits qb = make_query_bits(mine, IDX ? sQpos[cur][qr + l32] : myrow0 + l32);
                    if (hi == 0) {
                        sWq[wave][0][l32] = qb.a_lo;
                        sWq[wave][1][l32] = qb.a_hi;
                        sWq[wave][2][l32] = qb.x_lo;
                        sWq[wave][3][l32] = qb.x_hi;
                        sWq[wave][4][l32] = (unsigned)qb.lim;
                    }
                }
#pragma unroll
                for (int grp = 0; grp < 4; ++grp) {
                    const int roff = 8 * grp + 4 * hi;
                    const u32x4 qalo = *(const u32x4*)&sWq[wave][0][roff];
                    const u32x4 qahi = *(const u32x4*)&sWq[wave][1][roff];
                    const u32x4 qxlo = *(const u32x4*)&sWq[wave][2][roff];
                    const u32x4 qxhi = *(const u32x4*)&sWq[wave][3][roff];
                    const u32x4 qlim = *(const u32x4*)&sWq[wave][4][roff];
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        QueryBits qb;
                        qb.a_lo = qalo[x];
                        qb.a_hi = qahi[x];
                        qb.x_lo = qxlo[x];
                        qb.x_hi = qxhi[x];
                        qb.lim = (int)qlim[x];
                        qb.text = qlim[x] < 0x7FFFFFFFu;  // text rows carry their position, modality rows INT_MAX or -1
                        s[4 * grp + x] = allow_pair(qb, klo, khi, kpos) ? s[4 * grp + x] : 0.f;
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) dp[i] = s[i] * dp[i];  // -dS / scale
        u32x4 pb[2], dsb[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            pb[t] = pack8<T>(s, 8 * t);
            dsb[t] = pack8<T>(dp, 8 * t);
        }
        // ---- dV^T += dO^T P ; dK^T += Q^T dS -------------------------------------------------
        {
            u32x4 tg[2][DB], tq[2][DB];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    tg[t][db] = lds_read_transposed<D>(tG, lane, qr + 16 * t + 4 * hi, 32 * db + 16 * half16);
                    tq[t][db] = lds_read_transposed<D>(tQ, lane, qr + 16 * t + 4 * hi, 32 * db + 16 * half16);
                }
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    dv[db] = T::mfma(tg[t][db], pb[t], dv[db]);
                    dk[db] = T::mfma(tq[t][db], dsb[t], dk[db]);
                }
            sched_pipeline_mfma_lds<4 * DB, 4, 2>();
        }
        if (SAVE) {
            // Issued after the MFMAs of the tile (in front of them they cost the kernel 2 % more).  Record number and
            // record address are wave-uniform (kept in scalar registers); the two 16-byte stores are inline asm so that
            // they take the scalar-base form and stay out of the compiler's load / store bookkeeping, like the tile
            // copies (the caller waits with explicit counts); non-temporal: the blocks are read once, by another
            // kernel, and should not push the Q / dO rows the other workgroups re-read out of L2
            const unsigned rec_no = (unsigned)__builtin_amdgcn_readfirstlane(h_cur * (int)p.ds_capacity + ds_e);
            const char* rec = (const char*)p.ds_ws + ((uint64_t)rec_no << 13);
            asm volatile("global_store_dwordx4 %0, %1, %3 nt\n\tglobal_store_dwordx4 %0, %2, %3 offset:16 nt"
                         :
                         : "v"(ds_lane_off), "v"(dsb[0]), "v"(dsb[1]), "s"(rec)
                         : "memory");
        }
        return SAVE;
    };

    // Sequences of more than MAX_SLICE_LIST slices are walked in several passes, from the end, each with a list
    // of its own; dK and dV live in registers and simply carry over.
    for (int s_end = ns_total;;) {
        __syncthreads();
        const int n_all = sCount;
        // The last slice of a sequence whose length is not a multiple of 32 (always the last list entry) is
        // staged synchronously, with neutral values for the rows past the end, after the main loop.
        const bool ragged = (Sq & 31) != 0 && n_all > 0 &&
                            (__builtin_amdgcn_readfirstlane(sList[n_all > 0 ? n_all - 1 : 0]) >> 8) == ((Sq - 1) >> 5);
        const int n = n_all - (ragged ? 1 : 0);
        // Main loop: the listed slices are taken in pairs from the END of the list (the workgroups of one kv head
        // that are resident together then read the same Q / dO rows at about the same time, and all but the first
        // of them find them in L2); pair r = entries n - 2 - 2 r (row stream 0) and n - 1 - 2 r (row stream 1).
        // An odd count leaves the first entry alone: its pair repeats it with all classes cleared for stream 0.
        // The q heads of the group follow one another: tile t = (head t / npairs, pair t % npairs).
        const int npairs = (n + 1) >> 1;
        const int total = npairs * G;
        if (total > 0) {
            auto entry_hi = [&](int r) { return sList[n - 1 - 2 * r]; };
            auto entry_lo = [&](int r) { return sList[n - 2 - 2 * r]; };  // entry -1 where the count is odd
            // current tile (g_cur, entries e_*), next tile (g_nxt, r_nxt, entries n_*, head base hb_nxt); past the
            // last tile "next" keeps walking through pairs of the last head, whose copies nobody reads
            int g_cur = 0, g_nxt = 0, r_nxt = 0, r_cur = 0;
            HeadBase hb_nxt = head_base(hk * G);
            int e_lo = __builtin_amdgcn_readfirstlane(entry_lo(0)), e_hi = __builtin_amdgcn_readfirstlane(entry_hi(0));
            {
                const TileSource first = tile_source(hb_nxt, (e_lo >> 8) * 32, (e_hi >> 8) * 32);
#pragma unroll
                for (int j = 0; j < NLOADS; ++j) issue_copy(j, first, 0);
            }
            auto advance = [&]() {
                if (++r_nxt == npairs) {
                    r_nxt = 0;
                    if (++g_nxt < G) next_head(hb_nxt);
                }
            };
            advance();
            int n_lo = __builtin_amdgcn_readfirstlane(entry_lo(r_nxt)), n_hi = __builtin_amdgcn_readfirstlane(entry_hi(r_nxt));
            wait_async();
            __syncthreads();
            if (!v_negated) {  // K, V and the first tile have landed
                negate_v_tile();
                v_negated = true;
                __syncthreads();
            }
            load_kv_operands();
            for (int it = 0; it < total; ++it) {
                const int cur = it & 1;
                // pair after next: its list entries are requested now and picked up at the end of the iteration
                const int r_aft = r_nxt + 1 == npairs ? 0 : r_nxt + 1;
                const int a_lo = entry_lo(r_aft), a_hi = entry_hi(r_aft);
                const TileSource next = tile_source(hb_nxt, (n_lo >> 8) * 32, (n_hi >> 8) * 32);
                const int mine = st ? e_hi : e_lo;
                fetch_bias_key(hk * G + g_cur);
                const bool stored = tile_step(std::true_type{}, cur, (mine >> (2 * kg_lane)) & 3, hk * G + g_cur,
                                              (mine >> 8) * 32, n - 2 - 2 * r_cur + st, next);
                g_cur = g_nxt;
                r_cur = r_nxt;
                e_lo = n_lo;
                e_hi = n_hi;
                advance();
                n_lo = __builtin_amdgcn_readfirstlane(a_lo);
                n_hi = __builtin_amdgcn_readfirstlane(a_hi);
                // the copies of the next tile must have landed; the two dS stores, issued after them, may stay in flight
                if (SAVE && stored)
                    asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
                else
                    wait_async();
                __syncthreads();
            }
        }
        if (ragged) {
            wait_async();  // K, V of the tile, in case the main loop had nothing to do
            if (!v_negated) {
                __syncthreads();
                negate_v_tile();
                v_negated = true;  // (the barrier at the top of the loop below publishes it)
            }
            const int entry = __builtin_amdgcn_readfirstlane(sList[n_all - 1]);
            const int row0 = (entry >> 8) * 32;
            const int rows = Sq - row0;  // rows of the slice inside the sequence (1..31)
            for (int g = 0; g < G; ++g) {
                const int h = hk * G + g;
                __syncthreads();  // everybody is done with buffer 0
                stQ.load_ragged((const char*)p.q.ptr + 2 * ((int64_t)b * p.q.sb + (int64_t)h * p.q.sh + (int64_t)row0 * p.q.ss), sQ[0], rows, tid);
                stDO.load_ragged((const char*)p.dout.ptr + 2 * ((int64_t)b * p.dout.sb + (int64_t)h * p.dout.sh + (int64_t)row0 * p.dout.ss), sDO[0], rows, tid);
                if (tid < DKDV_QT) {
                    const int64_t off = ((int64_t)b * p.Hq + h) * p.Sq_rounded + row0;
                    const bool ok = tid < rows;
                    sLse[0][tid] = ok ? p.lse[off + tid] : INFINITY;  // lse = +inf gives P = 0
                    sDelta[0][tid] = ok ? p.delta[off + tid] : 0.f;
                    if (!DENSE) sQbf[0][tid] = ok ? bfrow[row0 + tid] : 0;
                    if (IDX) sQpos[0][tid] = ok ? p.posq[row0 + tid] : 0;
                }
                if (col_bits_on && tid < 128)  // the slice sits in row stream 0
                    sColBits[0][0][tid] = p.col_bits[(int64_t)b * p.col_bits_sb + (int64_t)(row0 >> 5) * p.col_bits_ss + nt * 128 + tid];
                __syncthreads();
                load_kv_operands();
                fetch_bias_key(h);
                // the slice sits in LDS rows 0..31: row stream 0 computes it, row stream 1 has nothing to do
                tile_step(std::false_type{}, 0, st ? 0 : (entry >> (2 * kg_lane)) & 3, h, row0, n_all - 1, TileSource{});
            }
        }
        if (!LONG) break;
        s_end = max(0, s_end - MAX_SLICE_LIST);
        if (s_end == 0) break;
        __syncthreads();  // everybody has read the list of the pass that just ended
        if (wave == 0) build_slice_list(p, b, nt, lane, max(0, s_end - MAX_SLICE_LIST), s_end, sList, &sCount);
    }
    // every copy has landed and every wave is done with the tiles: the epilogue reuses the tile arrays
    wait_async();
    __syncthreads();

    // ---- epilogue.  The two waves of a key group hold partial sums.
    if (p.grad_typed) {
        // Overwrite mode: dk/dv have the input dtype.  The K, V, Q, dO tiles are dead now; the
        // stream-1 wave of key group kg parks its partial sums in tile array number kg (exactly
        // the right size: 2 * D/32 * 16 floats per lane), its stream-0 partner adds its own and
        // stores the converted result.
        float* park = (float*)(kg == 0 ? sK : kg == 1 ? sV : kg == 2 ? &sQ[0][0] : &sDO[0][0]);
        if (st == 1) {
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    park[(db * 16 + i) * 64 + lane] = dk[db][i];
                    park[((DB + db) * 16 + i) * 64 + lane] = dv[db][i];
                }
        }
        __syncthreads();
        if (st == 0 && kvalid) {
            char* dkp = (char*)p.dk.ptr + 2 * ((int64_t)b * p.dk.sb + (int64_t)key * p.dk.ss + (int64_t)hk * p.dk.sh);
            char* dvp = (char*)p.dv.ptr + 2 * ((int64_t)b * p.dv.sb + (int64_t)key * p.dv.ss + (int64_t)hk * p.dv.sh);
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int grp = 0; grp < 4; ++grp) {
                    float a[4], c[4];
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        const int i = 4 * grp + x;
                        a[x] = (dk[db][i] + park[(db * 16 + i) * 64 + lane]) * -p.scale;  // dk holds -dK / scale
                        c[x] = dv[db][i] + park[((DB + db) * 16 + i) * 64 + lane];
                    }
                    const int d0 = 32 * db + 8 * grp + 4 * hi;
                    u32x2 wk, wv;
                    wk[0] = T::pack2(a[0], a[1]);
                    wk[1] = T::pack2(a[2], a[3]);
                    wv[0] = T::pack2(c[0], c[1]);
                    wv[1] = T::pack2(c[2], c[3]);
                    *(u32x2*)(dkp + d0 * 2) = wk;
                    *(u32x2*)(dvp + d0 * 2) = wv;
                }
        }
        return;
    }
    // Accumulate mode: both waves add to the caller's fp32 buffers in turn (this workgroup is
    // the sole owner of these rows).
    float* dkp = (float*)p.dk.ptr + ((int64_t)b * p.dk.sb + (int64_t)key * p.dk.ss + (int64_t)hk * p.dk.sh);
    float* dvp = (float*)p.dv.ptr + ((int64_t)b * p.dv.sb + (int64_t)key * p.dv.ss + (int64_t)hk * p.dv.sh);
#pragma unroll
    for (int turn = 0; turn < 2; ++turn) {
        if (st == turn && kvalid) {
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int grp = 0; grp < 4; ++grp) {
                    const int d0 = 32 * db + 8 * grp + 4 * hi;
                    f32x4 a = *(f32x4*)(dkp + d0), c = *(f32x4*)(dvp + d0);
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        a[x] = fmaf(dk[db][4 * grp + x], -p.scale, a[x]);  // dk holds -dK / scale
                        c[x] += dv[db][4 * grp + x];
                    }
                    *(f32x4*)(dkp + d0) = a;
                    *(f32x4*)(dvp + d0) = c;
                }
        }
        __threadfence_block();
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------------------
// dQ.  Same decomposition and S^T layout as the forward kernel: a lane owns one query, so
// lse and delta are per-lane scalars; dS^T feeds dQ^T = K^T dS^T from registers and K^T comes
// from the transposing LDS read of the K tile that also serves S^T = K Q^T.
constexpr int DQ_KT = 64;
constexpr int DQ_THREADS = 256;

// LONG: as in the dK/dV kernel, for more than MAX_LIST 64-key tiles.
template <typename T, int D, int MODE, bool BIAS, bool LONG>
__global__ __launch_bounds__(DQ_THREADS, D == 128 ? 2 : 3) void bwd_dq_kernel(const AttnParams p) {
    constexpr bool IDX = MODE == MASK_INDEXED, DENSE = MODE == MASK_DENSE;
    constexpr int NCH = D / 8, KK = D / 16, DB = D / 32;
    __shared__ u32x4 sK[2][DQ_KT * NCH];
    __shared__ u32x4 sV[2][DQ_KT * NCH];
    __shared__ __attribute__((aligned(16))) int64_t sKbf[2][DQ_KT];  // raw bitfields of the tile's keys
    __shared__ __attribute__((aligned(16))) int sKpos[2][DQ_KT];     // their global positions (IDX only)
    __shared__ int sList[MAX_LIST];
    __shared__ int sCount;
    // DENSE with packed mask bits: per wave, the words of its 32 rows for the tile's two 32-key blocks
    __shared__ unsigned sRowBits[DENSE ? 2 : 1][4][DENSE ? 64 : 1];

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

    const int slice = __builtin_amdgcn_readfirstlane(wave == 0 ? ws.slice[0] : wave == 1 ? ws.slice[1] : wave == 2 ? ws.slice[2] : ws.slice[3]);
    const int qrow = (slice < 0 ? 0 : slice) * 32 + l32;
    const bool qvalid = slice >= 0 && qrow < Sq;
    u32x4 qreg[KK], greg[KK];
    {
        const char* qp = (const char*)p.q.ptr + 2 * ((int64_t)b * p.q.sb + (int64_t)qrow * p.q.ss + (int64_t)h * p.q.sh);
        const char* gp = (const char*)p.dout.ptr + 2 * ((int64_t)b * p.dout.sb + (int64_t)qrow * p.dout.ss + (int64_t)h * p.dout.sh);
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            u32x4 zq = {0u, 0u, 0u, 0u}, zg = {0u, 0u, 0u, 0u};
            if (qvalid) {
                zq = *(const u32x4*)(qp + (16 * kk + 8 * hi) * 2);
                zg = *(const u32x4*)(gp + (16 * kk + 8 * hi) * 2);
            }
            qreg[kk] = zq;
            greg[kk] = zg;
        }
    }
    const int64_t qf = (!DENSE && qvalid) ? p.bfq[(int64_t)b * p.bfq_sb + qrow] : 0;
    float lse_row = 0.f, dlt = 0.f;
    if (qvalid) {
        const int64_t off = ((int64_t)b * p.Hq + h) * p.Sq_rounded + qrow;
        lse_row = p.lse[off];
        dlt = p.delta[off];
    }
    // (the row loads above are in flight while wave 0 reads the class rows)
    if (wave == 0) build_key_tile_list(ws, p.num_n, Sk, lane, 0, sList, &sCount);  // first pass (usually the only one)
    const QueryBits qb = make_query_bits(qf, (IDX && qvalid) ? p.posq[qrow] : qrow);
    const float lse2 = (!qvalid || lse_row == -INFINITY) ? INFINITY : lse_row * LOG2E;

    f32x16 dq[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) dq[db][i] = 0.f;
    f32x16 zero16;
#pragma unroll
    for (int i = 0; i < 16; ++i) zero16[i] = 0.f;
    const float c2 = BIAS ? LOG2E : p.scale * LOG2E;  // with a bias the scores become scale * s + bias first
    const char* bias_row = nullptr;  // this lane's row of the bias
    if (BIAS)
        bias_row = (const char*)p.bias + (p.bias_f32 ? 4 : 2) * ((int64_t)b * p.bias_sb + (int64_t)h * p.bias_sh +
                                                                (int64_t)(qvalid ? qrow : 0) * p.bias_sm);

    const char* kbase = (const char*)p.k.ptr + 2 * ((int64_t)b * p.k.sb + (int64_t)hk * p.k.sh);
    const char* vbase = (const char*)p.v.ptr + 2 * ((int64_t)b * p.v.sb + (int64_t)hk * p.v.sh);
    const int64_t k_ts = 2 * p.k.ss * DQ_KT, v_ts = 2 * p.v.ss * DQ_KT;  // bytes per tile
    const int64_t* bfrow = p.bfk + (int64_t)b * p.bfk_sb;

    typedef TileStage<D, DQ_KT, DQ_THREADS> Stage;
    constexpr int CPT = Stage::CPT;
    // copy instructions per wave and tile: K, V, the key bitfields and (IDX) the key positions
    constexpr int NLOADS = 2 * CPT + 1 + (IDX ? 1 : 0);
    static_assert(NLOADS <= 2 * KK, "one copy per MFMA of the first S / dP block");
    Stage stK, stV;
    stK.setup(2 * p.k.ss, tid);
    stV.setup(2 * p.v.ss, tid);
    const unsigned ldsK = lds_addr(sK), ldsV = lds_addr(sV), ldsB = lds_addr(sKbf), ldsP = lds_addr(sKpos);
    const unsigned ldsR = lds_addr(sRowBits);
    // DENSE: the packed mask rows of this wave's slice (null: no plan, the mask bytes are read instead)
    const unsigned* row_bits_w = (DENSE && p.row_bits != nullptr)
                                     ? p.row_bits + (int64_t)b * p.row_bits_sb + (slice < 0 ? 0 : slice) * 32
                                     : nullptr;
    const unsigned row_bits_voff = DENSE ? (unsigned)(hi * (int)p.row_bits_sn * 4 + l32 * 4) : 0u;
    constexpr unsigned TILE_BYTES = DQ_KT * NCH * 16, BITS_BYTES = DQ_KT * 8;
    // copy instruction j of full tile kt into buffer buf (key bitfields: 64 dwords per wave, waves 2, 3
    // repeat what waves 0, 1 write, so that every wave issues the same number of copies)
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
                dma_b32(bfrow + kt * DQ_KT, (unsigned)((wave & 1) * 256 + lane * 4), ldsB + buf * BITS_BYTES + (wave & 1) * 256u);
            }
        }
        else  // 64 positions; every wave writes the same values
            dma_b32(p.posk + kt * DQ_KT, (unsigned)(lane * 4), ldsP + buf * (DQ_KT * 4u));
    };

    // One 64-key tile held in buffer `cur`; with PREFETCH the copies of tile kt_next into the other buffer
    // are issued one per MFMA of the first S / dP block.
    auto tile_step = [&](auto prefetch, int cur, int entry, int kt_next) {
        constexpr bool PREFETCH = decltype(prefetch)::value;
        // (the class is extracted with a per-lane copy of the wave number on purpose: a skip branch the compiler
        // can prove wave-uniform makes it restructure the loop around it at the price of ~90 spilled registers)
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
        // partial tile whose 64 keys all carry the same bitfield: the rule is one position compare
        bool uniform_keys = false;
        int rel = 0;
        if (!DENSE && cls == 1) {
            const int64_t mine = sKbf[cur][lane];
            const unsigned mlo = (unsigned)mine, mhi = (unsigned)((uint64_t)mine >> 32);
            const unsigned flo = __builtin_amdgcn_readfirstlane(mlo), fhi = __builtin_amdgcn_readfirstlane(mhi);
            bool uniform = (mlo == flo) & (mhi == fhi);
            int kt0 = kt * DQ_KT;  // position of the tile's first key
            if (IDX) {             // ... and the 64 keys must sit at consecutive positions
                const int rel0 = sKpos[cur][lane] - lane;
                kt0 = __builtin_amdgcn_readfirstlane(rel0);
                uniform &= rel0 == kt0;
            }
            uniform_keys = __all(uniform);
            // last allowed key, relative to the first key this lane holds (4 hi): what it is compared with are then
            // compile-time constants, which occupy no registers
            rel = allow_bits(qb, flo, fhi) ? qb.lim - kt0 - 4 * hi : -1;
        }
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            // ---- S^T = K Q^T and dP^T = V dO^T : 32 keys x 32 queries, two accumulator chains
            f32x16 s, dp;
            {
                constexpr int NOP = 2 * KK, AHEAD = 4;  // operand j: K chunk (j even) or V chunk (j odd) of k-slice j / 2
                u32x4 a[NOP];
#pragma unroll
                for (int j = 0; j < AHEAD; ++j) a[j] = lds_read_chunk<D>((j & 1) ? tV : tK, 32 * kb + l32, 2 * (j >> 1) + hi);
#pragma unroll
                for (int j = 0; j < NOP; ++j) {
                    __builtin_amdgcn_sched_barrier(0);
                    if (j + AHEAD < NOP)
                        a[j + AHEAD] = lds_read_chunk<D>(((j + AHEAD) & 1) ? tV : tK, 32 * kb + l32, 2 * ((j + AHEAD) >> 1) + hi);
                    if (j & 1)
                        dp = T::mfma(a[j], greg[j >> 1], j < 2 ? zero16 : dp);
                    else
                        s = T::mfma(a[j], qreg[j >> 1], j < 2 ? zero16 : s);
                    if (PREFETCH && kb == 0 && j < NLOADS) issue_copy(j, kt_next, cur ^ 1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (BIAS) {
#pragma unroll
                for (int grp = 0; grp < 4; ++grp) {
                    const f32x4 b4 = load_bias4<T>(bias_row, kt * DQ_KT + 32 * kb + 8 * grp + 4 * hi, Sk, p.bias_f32 != 0, p.bias_vec != 0);
#pragma unroll
                    for (int x = 0; x < 4; ++x) s[4 * grp + x] = fmaf(s[4 * grp + x], p.scale, b4[x]);
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float e = __builtin_amdgcn_exp2f(fmaf(s[i], c2, -lse2));
                dp[i] = e * (dp[i] - dlt);  // the factor `scale` of dS is applied to dQ in the epilogue
            }
            if (DENSE) {
                if (cls == 1 && row_bits_w != nullptr) {
                    // (shifted by this lane's first key, 4 hi, once: the bit numbers tested are then constants)
                    const unsigned w = sRowBits[cur][wave][32 * kb + l32] >> (4 * hi);
#pragma unroll
                    for (int i = 0; i < 16; ++i) dp[i] = ((w >> (8 * (i >> 2) + (i & 3))) & 1u) ? dp[i] : 0.f;
                } else if (cls == 1) {
                    const int kt0 = kt * DQ_KT;
                    const uint8_t* mrow = p.mask + ((int64_t)b * Sq + (qvalid ? qrow : 0)) * Sk + kt0;
                    const bool dwords = (Sk & 3) == 0;  // rows start 4-byte aligned
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
                            dp[4 * grp + x] = a ? dp[4 * grp + x] : 0.f;
                        }
                    }
                }
            } else if (cls == 1) {
                if (uniform_keys) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) dp[i] = (32 * kb + 8 * (i >> 2) + (i & 3) <= rel) ? dp[i] : 0.f;
                } else {
                    // natural positions: the row's limit relative to the first key this lane holds
                    const int lim_rel = qb.lim - (kt * DQ_KT + 4 * hi);
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
                            dp[4 * grp + x] = (allow_bits(qb, klo[x], khi[x]) & pos_ok) ? dp[4 * grp + x] : 0.f;
                        }
                    }
                }
            }
            u32x4 dsb[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) dsb[t] = pack8<T>(dp, 8 * t);
            // ---- dQ^T += K^T dS^T
            {
                u32x4 ta[2][DB];
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int db = 0; db < DB; ++db)
                        ta[t][db] = lds_read_transposed<D>(tK, lane, 32 * kb + 16 * t + 4 * hi, 32 * db + 16 * half16);
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int db = 0; db < DB; ++db) dq[db] = T::mfma(ta[t][db], dsb[t], dq[db]);
                sched_pipeline_mfma_lds<2 * DB, 2, 2>();
            }
        }
    };

    // Sequences of more than MAX_LIST 64-key tiles are walked in several passes, each with a list of its own.
    const int nkt_total = (Sk + DQ_KT - 1) / DQ_KT;
    for (int kt_begin = 0;;) {
        __syncthreads();
        const int n_all = sCount;
        // A tile that holds the end of a sequence whose length is not a multiple of 64 is always the last
        // entry of the list; it is staged synchronously (zero fill past the end) after the main loop.
        const bool ragged = (Sk & (DQ_KT - 1)) != 0 && n_all > 0 &&
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
            const int kt = entry >> 8, rows = Sk - kt * DQ_KT;
            stK.load_ragged(kbase + kt * k_ts, sK[0], rows, tid);
            stV.load_ragged(vbase + kt * v_ts, sV[0], rows, tid);
            if (!DENSE && tid < DQ_KT) {
                sKbf[0][tid] = (tid < rows) ? bfrow[kt * DQ_KT + tid] : 0;
                if (IDX) sKpos[0][tid] = (tid < rows) ? p.posk[kt * DQ_KT + tid] : 0;
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

    if (qvalid && p.grad_typed) {  // overwrite mode: dq has the input dtype
        char* dqp = (char*)p.dq.ptr + 2 * ((int64_t)b * p.dq.sb + (int64_t)qrow * p.dq.ss + (int64_t)h * p.dq.sh);
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int grp = 0; grp < 4; ++grp) {
                u32x2 w;
                w[0] = T::pack2(dq[db][4 * grp + 0] * p.scale, dq[db][4 * grp + 1] * p.scale);
                w[1] = T::pack2(dq[db][4 * grp + 2] * p.scale, dq[db][4 * grp + 3] * p.scale);
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
                for (int x = 0; x < 4; ++x) a[x] = fmaf(dq[db][4 * grp + x], p.scale, a[x]);
                *(f32x4*)(dqp + d0) = a;
            }
    }
}


// ---------------------------------------------------------------------------------------
template <typename T, int D, bool BIAS, bool LONG>
static int launch_dkdv_b(const AttnParams& p, hipStream_t stream) {
    const int blocks = p.num_kt * p.B * p.Hkv;  // one workgroup per 128-key tile
    if (p.mask_mode == MASK_INDEXED)
        hipLaunchKernelGGL((bwd_dkdv_kernel<T, D, MASK_INDEXED, BIAS, LONG>), dim3(blocks), dim3(DKDV_THREADS), 0, stream, p);
    else if (p.mask_mode == MASK_DENSE)
        hipLaunchKernelGGL((bwd_dkdv_kernel<T, D, MASK_DENSE, BIAS, LONG>), dim3(blocks), dim3(DKDV_THREADS), 0, stream, p);
    else
        hipLaunchKernelGGL((bwd_dkdv_kernel<T, D, MASK_BITFIELD, BIAS, LONG>), dim3(blocks), dim3(DKDV_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}
template <typename T, int D, bool BIAS>
static int launch_dkdv_save_b(const AttnParams& p, hipStream_t stream) {
    const int blocks = p.num_kt * p.B * p.Hkv;
    if (p.mask_mode == MASK_INDEXED)
        hipLaunchKernelGGL((bwd_dkdv_kernel<T, D, MASK_INDEXED, BIAS, false, true>), dim3(blocks), dim3(DKDV_THREADS), 0, stream, p);
    else if (p.mask_mode == MASK_DENSE)
        hipLaunchKernelGGL((bwd_dkdv_kernel<T, D, MASK_DENSE, BIAS, false, true>), dim3(blocks), dim3(DKDV_THREADS), 0, stream, p);
    else
        hipLaunchKernelGGL((bwd_dkdv_kernel<T, D, MASK_BITFIELD, BIAS, false, true>), dim3(blocks), dim3(DKDV_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}
template <typename T, int D, bool BIAS, bool LONG>
static int launch_dq_b(const AttnParams& p, hipStream_t stream) {
    const int blocks = p.num_m * p.B * p.Hq;
    if (p.mask_mode == MASK_INDEXED)
        hipLaunchKernelGGL((bwd_dq_kernel<T, D, MASK_INDEXED, BIAS, LONG>), dim3(blocks), dim3(DQ_THREADS), 0, stream, p);
    else if (p.mask_mode == MASK_DENSE)
        hipLaunchKernelGGL((bwd_dq_kernel<T, D, MASK_DENSE, BIAS, LONG>), dim3(blocks), dim3(DQ_THREADS), 0, stream, p);
    else
        hipLaunchKernelGGL((bwd_dq_kernel<T, D, MASK_BITFIELD, BIAS, LONG>), dim3(blocks), dim3(DQ_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}

// fn<T, D>(p, stream) for the element type and head dimension of the call
#define BAM_DISPATCH(fn)                                       \
    if (dtype == 1) {                                          \
        if (p.D == 128) return fn<BF16, 128>(p, stream);       \
        if (p.D == 64) return fn<BF16, 64>(p, stream);         \
        return fn<BF16, 32>(p, stream);                        \
    }                                                          \
    if (p.D == 128) return fn<F16, 128>(p, stream);            \
    if (p.D == 64) return fn<F16, 64>(p, stream);              \
    return fn<F16, 32>(p, stream);

}  // namespace bam
