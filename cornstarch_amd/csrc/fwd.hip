// Forward kernel of bitfield-masked attention for gfx950.
// Reference semantics: cornstarch/kernel/bitfield_attention.py:236-523 (+ the split-KV merge
// :1292-1436, which a single pass over the keys makes unnecessary).
//
// Work decomposition
//   workgroup  = 128 query rows of one (batch, q head); 4 waves x 32 rows.
//   key loop   = 64-key tiles taken from the flag row of this query block: empty tiles are
//                never touched, "full" tiles skip the mask, "partial" tiles evaluate the
//                bitfield rule in registers.
//   K/V tiles  = double buffered in LDS; the next tile is copied global -> LDS directly while
//                the current one is consumed.
// Math layout
//   S^T = K Q^T on v_mfma_f32_32x32x16 with K rows as the A operand (LDS) and Q as the B
//   operand (registers).  In the C fragment a lane owns ONE query (lane & 31) and 16 of the
//   32 keys of a block, so the running max / sum / rescale factors are per-lane scalars and
//   the only cross-lane traffic is one exchange with lane ^ 32.  P^T then feeds
//   O^T = V^T P^T straight from registers as the B operand; V^T comes from the row-major V
//   tile through the transposing LDS read.
#include "bam_common.h"
#include "bam_launch.h"
#include "bam_tiles.h"

namespace bam {

constexpr int FWD_KT = 64;
constexpr int FWD_THREADS = 256;

template <typename T, int D>
__global__ __launch_bounds__(FWD_THREADS, 2) void fwd_kernel(const AttnParams p) {
    constexpr int NCH = D / 8, KK = D / 16, DB = D / 32;
    __shared__ u32x4 sK[2][FWD_KT * NCH];
    __shared__ u32x4 sV[2][FWD_KT * NCH];
    __shared__ __attribute__((aligned(16))) int64_t sKbf[2][FWD_KT];  // raw bitfields of the tile's keys
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
    const int m = p.num_m - 1 - ub / p.B;  // late query blocks (most keys under causality) first
    const int h = hk * G + g;

    if (wave == 0)
        build_key_tile_list(p.flags + (int64_t)b * p.flags_sb + (int64_t)m * p.flags_sm, p.num_n, S, lane,
                            sList, &sCount);

    // ---- per-lane query state -------------------------------------------------------
    const int qrow = m * BLOCK_M + wave * 32 + l32;
    const bool qvalid = qrow < S;
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
    const int64_t qf = qvalid ? p.bf[(int64_t)b * p.bf_sb + qrow] : 0;
    const QueryBits qb = make_query_bits(qf, qrow);

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
    const float c2 = p.scale * LOG2E;
    const float rescale_thr = RESCALE_LOG2 / c2;
    f32x16 zero16;
#pragma unroll
    for (int i = 0; i < 16; ++i) zero16[i] = 0.f;

    const char* kbase = (const char*)p.k.ptr + 2 * ((int64_t)b * p.k.sb + (int64_t)hk * p.k.sh);
    const char* vbase = (const char*)p.v.ptr + 2 * ((int64_t)b * p.v.sb + (int64_t)hk * p.v.sh);
    const int64_t k_ts = 2 * p.k.ss * FWD_KT, v_ts = 2 * p.v.ss * FWD_KT;  // bytes per tile
    const int64_t* bfrow = p.bf + (int64_t)b * p.bf_sb;

    TileStage<D, FWD_KT, FWD_THREADS> stK, stV;
    stK.setup(2 * p.k.ss, tid);
    stV.setup(2 * p.v.ss, tid);
    // bitfields of a tile's keys: direct global -> LDS copy by wave 1; the ragged last tile is
    // staged synchronously with 0 (never allowed) for the keys past the end
    auto stage_key_bits = [&](int kt, int buf) {
        if (S - kt * FWD_KT >= FWD_KT) {
            if (wave == 1) copy_dwords_async<2 * FWD_KT>(bfrow + kt * FWD_KT, sKbf[buf], lane);
        } else if (tid < FWD_KT) {
            sKbf[buf][tid] = (kt * FWD_KT + tid < S) ? bfrow[kt * FWD_KT + tid] : 0;
        }
    };

    __syncthreads();
    const int n = sCount;
    if (n > 0) {
        {
            const int kt = __builtin_amdgcn_readfirstlane(sList[0]) >> 2;
            stK.load(kbase + kt * k_ts, sK[0], S - kt * FWD_KT, tid);
            stV.load(vbase + kt * v_ts, sV[0], S - kt * FWD_KT, tid);
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
                stK.load(kbase + kt1 * k_ts, sK[cur ^ 1], S - kt1 * FWD_KT, tid);
                stV.load(vbase + kt1 * v_ts, sV[cur ^ 1], S - kt1 * FWD_KT, tid);
                stage_key_bits(kt1, cur ^ 1);
            }

            // ---- S^T = K Q^T : 64 keys x 32 queries per wave ----------------------------
            // two independent accumulator chains (key blocks 0 and 1) alternate; operand reads
            // run a few MFMAs ahead of their use; the first MFMA of a chain takes C = 0
            f32x16 s[2];
            {
                u32x4 ka[KK][2];
#pragma unroll
                for (int kk = 0; kk < KK; ++kk)
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb) ka[kk][kb] = lds_read_chunk<D>(sK[cur], 32 * kb + l32, 2 * kk + hi);
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) s[kb] = T::mfma(ka[0][kb], qreg[0], zero16);
#pragma unroll
                for (int kk = 1; kk < KK; ++kk)
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb) s[kb] = T::mfma(ka[kk][kb], qreg[kk], s[kb]);
                sched_pipeline_mfma_lds<2 * KK, 4, 1>();
            }

            // ---- bitfield rule in registers (partial tiles only) ------------------------
            if (cls == 1) {
                const int kt0 = kt * FWD_KT;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int grp = 0; grp < 4; ++grp) {
                        const int koff = 32 * kb + 8 * grp + 4 * hi;
                        const u32x4 k01 = *(const u32x4*)&sKbf[cur][koff];      // lo0 hi0 lo1 hi1
                        const u32x4 k23 = *(const u32x4*)&sKbf[cur][koff + 2];  // lo2 hi2 lo3 hi3
                        const unsigned klo[4] = {k01[0], k01[2], k23[0], k23[2]};
                        const unsigned khi[4] = {k01[1], k01[3], k23[1], k23[3]};
#pragma unroll
                        for (int x = 0; x < 4; ++x) {
                            const bool a = allow_pair(qb, klo[x], khi[x], kt0 + koff + x);
                            s[kb][4 * grp + x] = a ? s[kb][4 * grp + x] : -INFINITY;
                        }
                    }
            }

            // ---- online softmax (per-lane scalars) ----------------------------------------
            float mloc = fmaxf(s[0][0], s[1][0]);
#pragma unroll
            for (int i = 1; i < 16; ++i) mloc = fmaxf(mloc, fmaxf(s[0][i], s[1][i]));
            mloc = half_swap_max(mloc);
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
            float psum0 = 0.f, psum1 = 0.f;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float e0 = __builtin_amdgcn_exp2f(fmaf(s[0][i], c2, nb));
                const float e1 = __builtin_amdgcn_exp2f(fmaf(s[1][i], c2, nb));
                s[0][i] = e0;
                s[1][i] = e1;
                psum0 += e0;
                psum1 += e1;
            }
            l_i += psum0 + psum1;

            u32x4 pb[2][2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int t = 0; t < 2; ++t) pb[kb][t] = pack8<T>(s[kb], 8 * t);

            // ---- O^T += V^T P^T ---------------------------------------------------------------
            {
                u32x4 va[2][2][DB];
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int db = 0; db < DB; ++db)
                            va[kb][t][db] = lds_read_transposed<D>(sV[cur], lane, 32 * kb + 16 * t + 4 * hi,
                                                                   32 * db + 16 * half16);
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int db = 0; db < DB; ++db) o[db] = T::mfma(va[kb][t][db], pb[kb][t], o[db]);
                sched_pipeline_mfma_lds<4 * DB, (DB >= 2 ? 3 : 2), 2>();
            }

            wait_async();
            __syncthreads();
        }
    }

    // ---- epilogue: normalize, write O (q dtype) and LSE (natural log) -------------------
    const float ltot = half_swap_sum(l_i);
    const float inv = ltot > 0.f ? 1.f / ltot : 0.f;
    if (hi == 0)
        p.lse[((int64_t)b * p.Hq + h) * p.S_rounded + qrow] =
            ltot > 0.f ? (m_i * c2 + __builtin_amdgcn_logf(ltot)) * LN2 : -INFINITY;
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

template <typename T, int D>
static int launch_fwd_t(const AttnParams& p, hipStream_t stream) {
    const int blocks = p.num_m * p.B * p.Hq;
    hipLaunchKernelGGL((fwd_kernel<T, D>), dim3(blocks), dim3(FWD_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}

int launch_fwd(const AttnParams& p, int dtype, hipStream_t stream) {
    if (dtype == 1) {
        if (p.D == 128) return launch_fwd_t<BF16, 128>(p, stream);
        if (p.D == 64) return launch_fwd_t<BF16, 64>(p, stream);
        return launch_fwd_t<BF16, 32>(p, stream);
    }
    if (p.D == 128) return launch_fwd_t<F16, 128>(p, stream);
    if (p.D == 64) return launch_fwd_t<F16, 64>(p, stream);
    return launch_fwd_t<F16, 32>(p, stream);
}

}  // namespace bam
