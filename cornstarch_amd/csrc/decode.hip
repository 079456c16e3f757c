// Single-token decode step: one query row per (batch, head) against the whole key / value cache.
// Reference: cornstarch/kernel/interface.py:71-83 hands this case (eval mode, q_len == 1) to flash-attn through
// transformers' flash_attention_forward with attention_mask=None, forwarding `scaling`, `sliding_window` and
// `softcap`.  With one query at the last position, flash-attn's semantics reduce to
//   s_j = scale * q.k_j ;  s_j = softcap * tanh(s_j / softcap)  (if softcap > 0)
//   keys j < Sk - window are dropped                            (if 0 < window < Sk)
//   o = softmax(s) V
// No bitfield is consulted.
//
// The step is bound by reading K and V once; there is one query row per head, so the parallelism has to come from the
// keys.  decode_split_kernel: one wave per (range of 32-key tiles, kv head, batch element); the q heads of the kv
// head (up to 32 per workgroup) are the 32 "query rows" of the attention kernels' S^T = K Q^T layout, so the tile is
// read once for all of them:
//   S^T (32 keys x 32 heads) = K Q^T with the K rows of the tile (copied global -> LDS) as the A operand,
//   a lane owns one head (softmax state = per-lane scalars), P^T feeds O^T = V^T P^T from registers,
//   V^T comes from the V tile (copied global -> LDS) through the transposing LDS read.
// Every split writes its unnormalized output, maximum and sum for the heads that exist; decode_combine_kernel merges
// them.  A single split writes the result itself.
#include "bam_common.h"
#include "bam_launch.h"
#include "bam_tiles.h"

namespace bam {

constexpr int DEC_KT = 32;  // keys per tile

template <typename T, int D>
__global__ __launch_bounds__(64, 2) void decode_split_kernel(const DecodeParams p) {
    constexpr int NCH = D / 8, KK = D / 16, DB = D / 32;
    // one K tile (refilled as soon as its rows are in registers) and two V tiles (the copy of tile t + 1 runs under the
    // arithmetic of tile t); before the loop the V tiles' memory stages a q that is not 16-byte aligned
    __shared__ u32x4 sK[DEC_KT * NCH];
    __shared__ u32x4 sV[2][DEC_KT * (NCH < 8 ? 8 : NCH)];
    static_assert(sizeof(sV) >= 32 * D * 2, "the q staging area fits");

    const int lane = threadIdx.x, hi = lane >> 5, l32 = lane & 31, half16 = (lane >> 4) & 1;
    const int split = blockIdx.x, hk = blockIdx.y;
    const int b = blockIdx.z / p.row_groups, rg = blockIdx.z % p.row_groups;
    const int G = p.Hq / p.Hkv;
    const int h0 = hk * G + 32 * rg;         // first q head of this workgroup
    const int rows = min(32, G - 32 * rg);   // q heads it holds
    const int first = (p.window > 0 && p.window < p.Sk) ? p.Sk - p.window : 0;
    const int n_tiles = (p.Sk - first + DEC_KT - 1) / DEC_KT;
    const int t0 = split * p.tiles_per_split, t1 = min(n_tiles, t0 + p.tiles_per_split);

    // ---- Q: rows = heads, zero rows past the last head ----
    u32x4 qreg[KK];
    const bool q_aligned = ((reinterpret_cast<uintptr_t>(p.q) | (uintptr_t)(2 * p.q_sb) | (uintptr_t)(2 * p.q_sh)) & 15u) == 0;
    if (q_aligned) {  // wave-uniform: the lane's 16-byte pieces straight from global memory
        const char* qrow = (const char*)p.q + 2 * ((int64_t)b * p.q_sb + (int64_t)(h0 + min(l32, rows - 1)) * p.q_sh);
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const u32x4 x = *(const u32x4*)(qrow + (2 * kk + hi) * 16);
            const u32x4 z = {0u, 0u, 0u, 0u};
            qreg[kk] = l32 < rows ? x : z;
        }
    } else {  // element-wise loads through LDS (a view of q may be only 2-byte aligned)
        unsigned short* sQ = (unsigned short*)sV;
        for (int i = lane; i < rows * D; i += 64) {
            const int r = i / D, d = i % D;
            sQ[i] = ((const unsigned short*)p.q)[(int64_t)b * p.q_sb + (int64_t)(h0 + r) * p.q_sh + d];
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const u32x4 z = {0u, 0u, 0u, 0u};
            qreg[kk] = l32 < rows ? *(const u32x4*)&sQ[l32 * D + 16 * kk + 8 * hi] : z;
        }
        wait_lds();  // the staging area becomes the V tiles
    }

    const char* kbase = (const char*)p.k + 2 * ((int64_t)b * p.k_sb + (int64_t)hk * p.k_sh);
    const char* vbase = (const char*)p.v + 2 * ((int64_t)b * p.v_sb + (int64_t)hk * p.v_sh);
    TileStage<D, DEC_KT, 64> stK, stV;
    stK.setup(2 * p.k_ss, lane);
    stV.setup(2 * p.v_ss, lane);

    f32x16 o[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
    f32x16 zero16;
#pragma unroll
    for (int i = 0; i < 16; ++i) zero16[i] = 0.f;
    float m_i = -INFINITY, l_i = 0.f;  // maximum in the log2 domain; this lane's share of the sum (16 of 32 keys)

    // Tile t: its K rows into the K buffer, its V rows into V buffer buf (zero rows past the end of the cache).  Both
    // travel as 1 KiB pieces, global -> LDS; the K rows are the A operand of S^T = K Q^T (one 16-byte LDS read per MFMA).
    auto fetch = [&](int t, int buf) {
        const int key0 = first + t * DEC_KT;
        const int nvalid = min(DEC_KT, p.Sk - key0);
        stK.load(kbase + 2 * (int64_t)key0 * p.k_ss, sK, nvalid, lane);
        stV.load(vbase + 2 * (int64_t)key0 * p.v_ss, sV[buf], nvalid, lane);
    };

    if (t0 < t1) {
        fetch(t0, 0);
        wait_async();
        wait_lds();
    }
    for (int t = t0; t < t1; ++t) {
        const int cur = (t - t0) & 1;
        const int nvalid = min(DEC_KT, p.Sk - (first + t * DEC_KT));
        u32x4 ka[KK];
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) ka[kk] = lds_read_chunk<D>(sK, l32, 2 * kk + hi);
        wait_lds();
        // The next tile is requested as soon as this one's K rows are in registers: its latency runs under this
        // tile's arithmetic and under the other waves of the compute unit.  (The reads of that V buffer ended before
        // the previous iteration did.)
        if (t + 1 < t1) fetch(t + 1, cur ^ 1);
        f32x16 s = zero16;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) s = T::mfma(ka[kk], qreg[kk], s);

        // scores in the log2 domain: scale, cap, keys past the end
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int koff = 8 * (i >> 2) + 4 * hi + (i & 3);
            float x = s[i] * p.scale;
            if (p.softcap > 0.f) x = p.softcap * tanhf(x / p.softcap);
            x = koff < nvalid ? x * LOG2E : -INFINITY;
            s[i] = x;
            mx = fmaxf(mx, x);
        }
        const float mloc = half_swap_max(mx);        // finite: every tile holds at least one key
        const float mnew = fmaxf(m_i, mloc);
        const float alpha = __builtin_amdgcn_exp2f(m_i - mnew);  // 0 for the first tile
        m_i = mnew;
        float ls = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s[i] = __builtin_amdgcn_exp2f(s[i] - mnew);
            ls += s[i];
        }
        l_i = l_i * alpha + ls;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
        u32x4 pb[2];
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) pb[h2] = pack8<T>(s, 8 * h2);

#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const u32x4 va = lds_read_transposed<D>(sV[cur], lane, 16 * h2 + 4 * hi, 32 * db + 16 * half16);
                o[db] = T::mfma(va, pb[h2], o[db]);
            }
        // the next tile has landed (one wave: no barrier needed, LDS reads follow in program order), this tile's
        // reads of its V buffer are done, and so are the synchronous stores of a ragged next tile
        wait_async();
        wait_lds();
    }

    // ---- this split's result for head h0 + l32: O^T fragment register i of block db <-> column 32 db + 8 (i/4) + 4 hi + i%4
    const float ltot = half_swap_sum(l_i);
    if (l32 >= rows) return;
    const int h = h0 + l32;
    if (p.nsplit == 1) {
        const float inv = 1.f / ltot;
        unsigned short* op = (unsigned short*)p.o + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i)
                op[32 * db + 8 * (i >> 2) + 4 * hi + (i & 3)] = (unsigned short)(T::pack2(o[db][i] * inv, 0.f) & 0xFFFFu);
        return;
    }
    const int64_t rec = ((int64_t)b * p.Hq + h) * p.nsplit + split;
    float* wo = p.ws_o + rec * D;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int grp = 0; grp < 4; ++grp) {
            f32x4 w = {o[db][4 * grp], o[db][4 * grp + 1], o[db][4 * grp + 2], o[db][4 * grp + 3]};
            *(f32x4*)(wo + 32 * db + 8 * grp + 4 * hi) = w;
        }
    if (hi == 0) {
        p.ws_ml[2 * rec] = m_i;
        p.ws_ml[2 * rec + 1] = ltot;
    }
}

// Merges the splits of one (batch, head).  Thread = four output columns x one of COMBINE_LANES interleaved subsets of
// the splits, merged with the usual running maximum / rescale; the subsets then meet in LDS.
constexpr int COMBINE_THREADS = 256;
template <typename T>
__global__ __launch_bounds__(COMBINE_THREADS) void decode_combine_kernel(const DecodeParams p) {
    __shared__ float s_m[COMBINE_THREADS], s_l[COMBINE_THREADS];
    __shared__ __attribute__((aligned(16))) float s_acc[COMBINE_THREADS][4];
    const int bh = blockIdx.x, tid = threadIdx.x;
    const int cols = p.D / 4;                 // threads across the columns: 8, 16 or 32
    const int lanes = COMBINE_THREADS / cols; // subsets of the splits
    const int c4 = tid % cols, sl = tid / cols;
    const float* ml = p.ws_ml + 2 * (int64_t)bh * p.nsplit;
    const float* wo = p.ws_o + (int64_t)bh * p.nsplit * p.D + 4 * c4;
    float m = -INFINITY, l = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int s = sl; s < p.nsplit; s += lanes) {
        const float ms = ml[2 * s], ls = ml[2 * s + 1];
        const f32x4 o4 = *(const f32x4*)(wo + (int64_t)s * p.D);
        const float mnew = fmaxf(m, ms);
        const float a = __builtin_amdgcn_exp2f(m - mnew), w = __builtin_amdgcn_exp2f(ms - mnew);  // a = 0 at first
        m = mnew;
        l = l * a + ls * w;
#pragma unroll
        for (int x = 0; x < 4; ++x) acc[x] = acc[x] * a + o4[x] * w;
    }
    s_m[tid] = m;
    s_l[tid] = l;
    *(f32x4*)s_acc[tid] = acc;
    __syncthreads();
    if (sl != 0) return;
    for (int j = 1; j < lanes; ++j) {
        const int t = j * cols + c4;
        const float ms = s_m[t];
        if (ms == -INFINITY) continue;  // a subset without splits
        const float mnew = fmaxf(m, ms);
        const float a = __builtin_amdgcn_exp2f(m - mnew), w = __builtin_amdgcn_exp2f(ms - mnew);
        m = mnew;
        l = l * a + s_l[t] * w;
#pragma unroll
        for (int x = 0; x < 4; ++x) acc[x] = acc[x] * a + s_acc[t][x] * w;
    }
    const int b = bh / p.Hq, h = bh % p.Hq;
    unsigned short* op = (unsigned short*)p.o + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + 4 * c4;
    const float inv = 1.f / l;
#pragma unroll
    for (int x = 0; x < 4; ++x) op[x] = (unsigned short)(T::pack2(acc[x] * inv, 0.f) & 0xFFFFu);
}

template <typename T>
static int launch_decode_t(const DecodeParams& p, hipStream_t stream) {
    const dim3 grid(p.nsplit, p.Hkv, p.B * p.row_groups), block(64);
    if (p.D == 128)
        hipLaunchKernelGGL((decode_split_kernel<T, 128>), grid, block, 0, stream, p);
    else if (p.D == 64)
        hipLaunchKernelGGL((decode_split_kernel<T, 64>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((decode_split_kernel<T, 32>), grid, block, 0, stream, p);
    if (p.nsplit > 1)
        hipLaunchKernelGGL((decode_combine_kernel<T>), dim3(p.B * p.Hq), dim3(COMBINE_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}

int launch_decode(const DecodeParams& p, int dtype, hipStream_t stream) {
    return dtype == 1 ? launch_decode_t<BF16>(p, stream) : launch_decode_t<F16>(p, stream);
}

// How the keys of one decode step are split over workgroups: about four waves per compute unit, all resident at once
// (1024 workgroups; more of them only add per-workgroup set-up and partial results to merge: 2560 measured 10 % slower,
// 512 leave too little in flight), at least two tiles per split where the cache is long enough.  Shared by the
// workspace size and the launch.
void decode_split_plan(int B, int Hq, int Hkv, int Sk, int window, int* nsplit, int* tiles_per_split, int* row_groups) {
    const int G = Hq / Hkv;
    const int rgs = (G + 31) / 32;
    const int keys = (window > 0 && window < Sk) ? window : Sk;
    const int n_tiles = (keys + DEC_KT - 1) / DEC_KT;
    const int64_t units = (int64_t)B * Hkv * rgs;
    int64_t want = (1024 + units - 1) / units;
    const int most = n_tiles >= 2 ? n_tiles / 2 : 1;
    if (want > most) want = most;
    if (want < 1) want = 1;
    const int tps = (int)((n_tiles + want - 1) / want);
    *tiles_per_split = tps;
    *nsplit = (n_tiles + tps - 1) / tps;
    *row_groups = rgs;
}

}  // namespace bam
