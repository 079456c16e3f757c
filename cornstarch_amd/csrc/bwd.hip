// Backward kernels of bitfield-masked attention for gfx950.
// Reference semantics: cornstarch/kernel/bitfield_attention.py:527-572 (delta) and :598-929
// (dQ, dK, dV).  The reference accumulates dQ, dK and dV with fp32 atomics; here every output
// element has exactly one owner, so nothing is atomic and the sums are deterministic:
//   dkdv kernel : one workgroup per (batch, kv head, 128-key tile); it loops over the q heads
//                 of the group and over the query blocks its flag column lists.
//   dq kernel   : one workgroup per (batch, q head, 128-query block), looping over key tiles
//                 exactly like the forward kernel.
// Both recompute P = exp(scale * s - lse) from the saved log-sum-exp.
#include "bam_common.h"
#include "bam_launch.h"
#include "bam_tiles.h"

namespace bam {

// ---------------------------------------------------------------------------------------
// delta[b,h,i] = sum_d o * do   (fp32).  D/8 lanes per row, 16 bytes per lane per tensor.
template <typename T, int D>
__global__ __launch_bounds__(256) void bwd_preprocess_kernel(const AttnParams p) {
    constexpr int LPR = D / 8;
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t row = gid / LPR;
    const int c = (int)(gid % LPR);
    const int64_t total = (int64_t)p.B * p.S * p.Hq;
    const bool valid = row < total;
    int h = 0, i = 0, b = 0;
    float acc = 0.f;
    if (valid) {
        h = (int)(row % p.Hq);
        const int64_t bi = row / p.Hq;
        i = (int)(bi % p.S);
        b = (int)(bi / p.S);
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
    if (valid && c == 0) p.delta[((int64_t)b * p.Hq + h) * p.S_rounded + i] = acc;
}

// ---------------------------------------------------------------------------------------
// dK, dV.  One workgroup = one 128-key tile of one (batch, kv head), 8 waves: wave w owns keys
// [32 (w & 3), +32) and works on query rows [32 (w >> 2), +32) of every 64-row tile of Q / dO
// that streams through LDS (double buffered), so each SIMD holds two waves whose MFMA and
// softmax phases interleave.  K and V of the tile sit in LDS for the whole kernel and are
// read as MFMA B operands; dK^T and dV^T (d x keys) stay in accumulators.
// With S = Q K^T computed as queries x keys, a lane of the C fragment owns ONE key and 16
// query rows, so P and dS feed dV^T = dO^T P and dK^T = Q^T dS as B operands from registers;
// Q^T and dO^T come from the transposing LDS read of the same row-major tiles.
// The two waves that share a key group hold partial sums; they add them to the caller's
// buffers one after the other (workgroup barrier in between), so the result stays
// deterministic and atomic free.
constexpr int DKDV_QT = 64;
constexpr int DKDV_THREADS = 512;

template <typename T, int D>
__global__ __launch_bounds__(DKDV_THREADS, 2) void bwd_dkdv_kernel(const AttnParams p) {
    constexpr int NCH = D / 8, KK = D / 16, DB = D / 32;
    __shared__ u32x4 sK[128 * NCH];
    __shared__ u32x4 sV[128 * NCH];
    __shared__ u32x4 sQ[2][DKDV_QT * NCH];
    __shared__ u32x4 sDO[2][DKDV_QT * NCH];
    __shared__ __attribute__((aligned(16))) float sLse[2][DKDV_QT];      // natural-log lse of the rows
    __shared__ __attribute__((aligned(16))) float sDelta[2][DKDV_QT];
    __shared__ __attribute__((aligned(16))) int64_t sQbf[2][DKDV_QT];    // raw bitfields of the rows
    __shared__ __attribute__((aligned(16))) unsigned sWq[DKDV_THREADS / 64][5][32];  // per-wave rule constants
    __shared__ int sList[MAX_LIST / 2];
    __shared__ int sCount;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kg = wave & 3, st = wave >> 2;
    const int hi = lane >> 5, l32 = lane & 31, half16 = (lane >> 4) & 1;
    const int S = p.S;
    const int G = p.Hq / p.Hkv;

    const int unit = blockIdx.x;
    const int hk = unit % p.Hkv;
    const int ub = unit / p.Hkv;
    const int b = ub % p.B;
    const int nt = ub / p.B;  // early key tiles (most queries under causality) first

    if (wave == 0)
        build_query_block_list(p.flags + (int64_t)b * p.flags_sb, p.flags_sm, p.num_m, p.num_n, nt, lane, sList,
                               &sCount);

    // ---- K, V of the tile -> LDS (once) ---------------------------------------------------
    {
        TileStage<D, 128, DKDV_THREADS> stK, stV;
        stK.setup(2 * p.k.ss, tid);
        stV.setup(2 * p.v.ss, tid);
        const char* kb = (const char*)p.k.ptr + 2 * ((int64_t)b * p.k.sb + (int64_t)hk * p.k.sh + (int64_t)nt * 128 * p.k.ss);
        const char* vb = (const char*)p.v.ptr + 2 * ((int64_t)b * p.v.sb + (int64_t)hk * p.v.sh + (int64_t)nt * 128 * p.v.ss);
        stK.load(kb, sK, S - nt * 128, tid);
        stV.load(vb, sV, S - nt * 128, tid);
    }
    const int key = nt * 128 + kg * 32 + l32;
    const bool kvalid = key < S;
    const int64_t* bfrow = p.bf + (int64_t)b * p.bf_sb;
    const int64_t kf = kvalid ? bfrow[key] : 0;
    const unsigned klo = (unsigned)(kf & 0xFFFFFFFFll);
    const unsigned khi = (unsigned)((uint64_t)kf >> 32);

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
    const float c2 = p.scale * LOG2E;

    TileStage<D, DKDV_QT, DKDV_THREADS> stQ, stDO;
    stQ.setup(2 * p.q.ss, tid);
    stDO.setup(2 * p.dout.ss, tid);

    // iteration `it` -> (q head of the group, list entry, 64-row half of the 128-row block).
    // Query blocks are visited from the LAST one down: the workgroups of one kv head that are
    // resident together then read the same Q / dO tile at about the same time, and all but the
    // first of them find it in L2.
    auto list_at = [&](int rem, int n) { return __builtin_amdgcn_readfirstlane(sList[n - 1 - (rem >> 1)]); };
    auto tile_row0 = [&](int rem, int n) { return (list_at(rem, n) >> 8) * BLOCK_M + (1 - (rem & 1)) * DKDV_QT; };
    // Everything a tile needs (Q, dO rows, their lse, delta and bitfields) is copied global -> LDS
    // without passing through registers; only the ragged last tile of a sequence is staged
    // synchronously, with neutral values for the rows past the end (lse = +inf gives P = 0).
    auto stage = [&](int it, int n, int buf) {
        const int g = it / (2 * n);
        const int row0 = tile_row0(it - g * 2 * n, n);
        const int h = hk * G + g;
        const char* qbase = (const char*)p.q.ptr + 2 * ((int64_t)b * p.q.sb + (int64_t)h * p.q.sh);
        const char* gbase = (const char*)p.dout.ptr + 2 * ((int64_t)b * p.dout.sb + (int64_t)h * p.dout.sh);
        stQ.load(qbase + (int64_t)row0 * 2 * p.q.ss, sQ[buf], S - row0, tid);
        stDO.load(gbase + (int64_t)row0 * 2 * p.dout.ss, sDO[buf], S - row0, tid);
        const int64_t off = ((int64_t)b * p.Hq + h) * p.S_rounded + row0;
        if (S - row0 >= DKDV_QT) {
            if (wave == 1) copy_dwords_async<DKDV_QT>(p.lse + off, sLse[buf], lane);
            if (wave == 2) copy_dwords_async<DKDV_QT>(p.delta + off, sDelta[buf], lane);
            if (wave == 3) copy_dwords_async<2 * DKDV_QT>(bfrow + row0, sQbf[buf], lane);
        } else if (tid < DKDV_QT) {
            const bool ok = row0 + tid < S;
            sLse[buf][tid] = ok ? p.lse[off + tid] : INFINITY;
            sDelta[buf][tid] = ok ? p.delta[off + tid] : 0.f;
            sQbf[buf][tid] = ok ? bfrow[row0 + tid] : 0;
        }
    };

    __syncthreads();
    const int n = sCount;
    const int total = n * 2 * G;
    if (total > 0) {
        stage(0, n, 0);
        wait_async();
        __syncthreads();
        const int qr = 32 * st;  // this wave's rows inside the 64-row tile
        for (int it = 0; it < total; ++it) {
            const int cur = it & 1;
            if (it + 1 < total) stage(it + 1, n, cur ^ 1);

            const int rem = it % (2 * n);
            const int entry = list_at(rem, n);
            const int cls = (entry >> (2 * kg)) & 3;  // this wave's own 128x32 flag
            if (cls != 0) {
                // ---- S = Q K^T and dP = dO V^T : 32 queries x 32 keys; both operands of every MFMA
                // come from LDS and are requested a few MFMAs ahead of their use
                f32x16 s, dp;
                {
                    u32x4 aq[KK], ag[KK], bk[KK], bv[KK];
#pragma unroll
                    for (int kk = 0; kk < KK; ++kk) {
                        aq[kk] = lds_read_chunk<D>(sQ[cur], qr + l32, 2 * kk + hi);
                        bk[kk] = lds_read_chunk<D>(sK, 32 * kg + l32, 2 * kk + hi);
                        ag[kk] = lds_read_chunk<D>(sDO[cur], qr + l32, 2 * kk + hi);
                        bv[kk] = lds_read_chunk<D>(sV, 32 * kg + l32, 2 * kk + hi);
                    }
                    s = T::mfma(aq[0], bk[0], zero16);
                    dp = T::mfma(ag[0], bv[0], zero16);
#pragma unroll
                    for (int kk = 1; kk < KK; ++kk) {
                        s = T::mfma(aq[kk], bk[kk], s);
                        dp = T::mfma(ag[kk], bv[kk], dp);
                    }
                    sched_pipeline_mfma_lds<2 * KK, 2, 2>();
                }
                // ---- P = exp(scale s - lse), dS/scale = P (dP - delta)   (the factor `scale` of dS
                // is applied once to dK in the epilogue).  C fragment: register i <-> query row
                // 8*(i/4) + 4*hi + i%4 of this wave's 32 rows.
#pragma unroll
                for (int grp = 0; grp < 4; ++grp) {
                    const int roff = qr + 8 * grp + 4 * hi;
                    const f32x4 l4 = *(const f32x4*)&sLse[cur][roff];
                    const f32x4 d4 = *(const f32x4*)&sDelta[cur][roff];
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        const float e = __builtin_amdgcn_exp2f(fmaf(s[4 * grp + x], c2, l4[x] * -LOG2E));
                        s[4 * grp + x] = e;
                        dp[4 * grp + x] = e * (dp[4 * grp + x] - d4[x]);
                    }
                }
                if (cls == 1) {
                    // rule constants of this wave's 32 rows, derived once per row (lane r < 32 takes
                    // row r) and handed to all lanes through a wave-private LDS scratch
                    {
                        const int row0 = tile_row0(rem, n);
                        const QueryBits qb = make_query_bits(sQbf[cur][qr + l32], row0 + qr + l32);
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
                            const bool a = allow_pair(qb, klo, khi, key);
                            s[4 * grp + x] = a ? s[4 * grp + x] : 0.f;
                            dp[4 * grp + x] = a ? dp[4 * grp + x] : 0.f;
                        }
                    }
                }
                u32x4 pb[2], dsb[2];
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    pb[t] = pack8<T>(s, 8 * t);
                    dsb[t] = pack8<T>(dp, 8 * t);
                }
                // ---- dV^T += dO^T P ; dK^T += Q^T dS -------------------------------------------
                {
                    u32x4 tg[2][DB], tq[2][DB];
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int db = 0; db < DB; ++db) {
                            tg[t][db] = lds_read_transposed<D>(sDO[cur], lane, qr + 16 * t + 4 * hi, 32 * db + 16 * half16);
                            tq[t][db] = lds_read_transposed<D>(sQ[cur], lane, qr + 16 * t + 4 * hi, 32 * db + 16 * half16);
                        }
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int db = 0; db < DB; ++db) {
                            dv[db] = T::mfma(tg[t][db], pb[t], dv[db]);
                            dk[db] = T::mfma(tq[t][db], dsb[t], dk[db]);
                        }
                    sched_pipeline_mfma_lds<4 * DB, 3, 2>();
                }
            }
            wait_async();
            __syncthreads();
        }
    }

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
                        a[x] = (dk[db][i] + park[(db * 16 + i) * 64 + lane]) * p.scale;
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
                        a[x] = fmaf(dk[db][4 * grp + x], p.scale, a[x]);
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

template <typename T, int D>
__global__ __launch_bounds__(DQ_THREADS, 2) void bwd_dq_kernel(const AttnParams p) {
    constexpr int NCH = D / 8, KK = D / 16, DB = D / 32;
    __shared__ u32x4 sK[2][DQ_KT * NCH];
    __shared__ u32x4 sV[2][DQ_KT * NCH];
    __shared__ __attribute__((aligned(16))) int64_t sKbf[2][DQ_KT];  // raw bitfields of the tile's keys
    __shared__ int sList[MAX_LIST];
    __shared__ int sCount;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int hi = lane >> 5, l32 = lane & 31, half16 = (lane >> 4) & 1;
    const int S = p.S;
    const int G = p.Hq / p.Hkv;

    int unit, g;
    xcd_group_map(blockIdx.x, p.num_m * p.B * p.Hkv, G, unit, g);
    const int hk = unit % p.Hkv;
    const int ub = unit / p.Hkv;
    const int b = ub % p.B;
    const int m = p.num_m - 1 - ub / p.B;
    const int h = hk * G + g;

    if (wave == 0)
        build_key_tile_list(p.flags + (int64_t)b * p.flags_sb + (int64_t)m * p.flags_sm, p.num_n, S, lane,
                            sList, &sCount);

    const int qrow = m * BLOCK_M + wave * 32 + l32;
    const bool qvalid = qrow < S;
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
    const int64_t qf = qvalid ? p.bf[(int64_t)b * p.bf_sb + qrow] : 0;
    const QueryBits qb = make_query_bits(qf, qrow);
    float lse2 = INFINITY, dlt = 0.f;
    if (qvalid) {
        const int64_t off = ((int64_t)b * p.Hq + h) * p.S_rounded + qrow;
        const float l = p.lse[off];
        lse2 = (l == -INFINITY) ? INFINITY : l * LOG2E;
        dlt = p.delta[off];
    }

    f32x16 dq[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) dq[db][i] = 0.f;
    const float c2 = p.scale * LOG2E;

    const char* kbase = (const char*)p.k.ptr + 2 * ((int64_t)b * p.k.sb + (int64_t)hk * p.k.sh);
    const char* vbase = (const char*)p.v.ptr + 2 * ((int64_t)b * p.v.sb + (int64_t)hk * p.v.sh);
    const int64_t k_ts = 2 * p.k.ss * DQ_KT, v_ts = 2 * p.v.ss * DQ_KT;  // bytes per tile
    const int64_t* bfrow = p.bf + (int64_t)b * p.bf_sb;

    TileStage<D, DQ_KT, DQ_THREADS> stK, stV;
    stK.setup(2 * p.k.ss, tid);
    stV.setup(2 * p.v.ss, tid);
    // bitfields of a tile's keys: direct global -> LDS copy by wave 1; the ragged last tile is
    // staged synchronously with 0 (never allowed) for the keys past the end
    auto stage_key_bits = [&](int kt, int buf) {
        if (S - kt * DQ_KT >= DQ_KT) {
            if (wave == 1) copy_dwords_async<2 * DQ_KT>(bfrow + kt * DQ_KT, sKbf[buf], lane);
        } else if (tid < DQ_KT) {
            sKbf[buf][tid] = (kt * DQ_KT + tid < S) ? bfrow[kt * DQ_KT + tid] : 0;
        }
    };

    __syncthreads();
    const int n = sCount;
    if (n > 0) {
        {
            const int kt = __builtin_amdgcn_readfirstlane(sList[0]) >> 2;
            stK.load(kbase + kt * k_ts, sK[0], S - kt * DQ_KT, tid);
            stV.load(vbase + kt * v_ts, sV[0], S - kt * DQ_KT, tid);
            stage_key_bits(kt, 0);
        }
        wait_async();
        __syncthreads();
        for (int it = 0; it < n; ++it) {
            const int cur = it & 1;
            const int entry = __builtin_amdgcn_readfirstlane(sList[it]);
            const int kt = entry >> 2, cls = entry & 3;
            const bool more = it + 1 < n;
            if (more) {
                const int kt1 = __builtin_amdgcn_readfirstlane(sList[it + 1]) >> 2;
                stK.load(kbase + kt1 * k_ts, sK[cur ^ 1], S - kt1 * DQ_KT, tid);
                stV.load(vbase + kt1 * v_ts, sV[cur ^ 1], S - kt1 * DQ_KT, tid);
                stage_key_bits(kt1, cur ^ 1);
            }
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                f32x16 s, dp;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    s[i] = 0.f;
                    dp[i] = 0.f;
                }
                {
                    u32x4 ka[KK], va[KK];
#pragma unroll
                    for (int kk = 0; kk < KK; ++kk) {
                        ka[kk] = lds_read_chunk<D>(sK[cur], 32 * kb + l32, 2 * kk + hi);
                        va[kk] = lds_read_chunk<D>(sV[cur], 32 * kb + l32, 2 * kk + hi);
                    }
#pragma unroll
                    for (int kk = 0; kk < KK; ++kk) {
                        s = T::mfma(ka[kk], qreg[kk], s);
                        dp = T::mfma(va[kk], greg[kk], dp);
                    }
                    sched_pipeline_mfma_lds<2 * KK, 4, 1>();
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float e = __builtin_amdgcn_exp2f(fmaf(s[i], c2, -lse2));
                    dp[i] = e * (dp[i] - dlt);  // the factor `scale` of dS is applied to dQ in the epilogue
                }
                if (cls == 1) {
                    const int kt0 = kt * DQ_KT;
#pragma unroll
                    for (int grp = 0; grp < 4; ++grp) {
                        const int koff = 32 * kb + 8 * grp + 4 * hi;
                        const u32x4 k01 = *(const u32x4*)&sKbf[cur][koff];      // lo0 hi0 lo1 hi1
                        const u32x4 k23 = *(const u32x4*)&sKbf[cur][koff + 2];  // lo2 hi2 lo3 hi3
                        const unsigned klo[4] = {k01[0], k01[2], k23[0], k23[2]};
                        const unsigned khi[4] = {k01[1], k01[3], k23[1], k23[3]};
#pragma unroll
                        for (int x = 0; x < 4; ++x)
                            dp[4 * grp + x] = allow_pair(qb, klo[x], khi[x], kt0 + koff + x) ? dp[4 * grp + x] : 0.f;
                    }
                }
                u32x4 dsb[2];
#pragma unroll
                for (int t = 0; t < 2; ++t) dsb[t] = pack8<T>(dp, 8 * t);
                {
                    u32x4 ta[2][DB];
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int db = 0; db < DB; ++db)
                            ta[t][db] = lds_read_transposed<D>(sK[cur], lane, 32 * kb + 16 * t + 4 * hi,
                                                               32 * db + 16 * half16);
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int db = 0; db < DB; ++db) dq[db] = T::mfma(ta[t][db], dsb[t], dq[db]);
                    sched_pipeline_mfma_lds<2 * DB, 2, 2>();
                }
            }
            wait_async();
            __syncthreads();
        }
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
template <typename T, int D>
static int launch_pre_t(const AttnParams& p, hipStream_t stream) {
    const int64_t threads = (int64_t)p.B * p.S * p.Hq * (D / 8);
    const int64_t blocks = (threads + 255) / 256;
    hipLaunchKernelGGL((bwd_preprocess_kernel<T, D>), dim3((unsigned)blocks), dim3(256), 0, stream, p);
    return (int)hipGetLastError();
}
template <typename T, int D>
static int launch_dkdv_t(const AttnParams& p, hipStream_t stream) {
    const int blocks = p.num_m * p.B * p.Hkv;  // ceil(S/128) key tiles
    hipLaunchKernelGGL((bwd_dkdv_kernel<T, D>), dim3(blocks), dim3(DKDV_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}
template <typename T, int D>
static int launch_dq_t(const AttnParams& p, hipStream_t stream) {
    const int blocks = p.num_m * p.B * p.Hq;
    hipLaunchKernelGGL((bwd_dq_kernel<T, D>), dim3(blocks), dim3(DQ_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}

#define BAM_DISPATCH(fn)                                       \
    if (dtype == 1) {                                          \
        if (p.D == 128) return fn<BF16, 128>(p, stream);       \
        if (p.D == 64) return fn<BF16, 64>(p, stream);         \
        return fn<BF16, 32>(p, stream);                        \
    }                                                          \
    if (p.D == 128) return fn<F16, 128>(p, stream);            \
    if (p.D == 64) return fn<F16, 64>(p, stream);              \
    return fn<F16, 32>(p, stream);

int launch_bwd_preprocess(const AttnParams& p, int dtype, hipStream_t stream) { BAM_DISPATCH(launch_pre_t) }
int launch_bwd_dkdv(const AttnParams& p, int dtype, hipStream_t stream) { BAM_DISPATCH(launch_dkdv_t) }
int launch_bwd_dq(const AttnParams& p, int dtype, hipStream_t stream) { BAM_DISPATCH(launch_dq_t) }

}  // namespace bam
