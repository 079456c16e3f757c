// Single-token decode step: one query row per (batch, head) against the whole key / value cache.
// Reference: cornstarch/kernel/interface.py:71-83 hands this case (eval mode, q_len == 1) to flash-attn through
// transformers' flash_attention_forward with attention_mask=None, forwarding `scaling`, `sliding_window` and
// `softcap`.  With one query at the last position, flash-attn's semantics reduce to
//   s_j = scale * q.k_j ;  s_j = softcap * tanh(s_j / softcap)  (if softcap > 0)
//   keys j < Sk - window are dropped                            (if 0 < window < Sk)
//   o = softmax(s) V
// No bitfield is consulted.  The kernel is bound by reading K and V once per q head (HBM / L2), not by arithmetic.
#include "bam_common.h"
#include "bam_launch.h"

namespace bam {

constexpr int DEC_THREADS = 256;
constexpr int DEC_CHUNK = 1024;  // keys whose scores sit in LDS at a time

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x = fmaxf(x, __shfl_xor(x, off));
    return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off);
    return x;
}

template <typename T, int D>
__global__ __launch_bounds__(DEC_THREADS) void decode_kernel(const DecodeParams p) {
    constexpr int LPR = D / 8;               // lanes that share one key row, 16 bytes each
    constexpr int NK = DEC_THREADS / LPR;    // keys in flight per sweep
    __shared__ float sQ[D];
    __shared__ float sS[DEC_CHUNK];
    __shared__ float sRed[DEC_THREADS / 64];
    __shared__ float sAcc[NK][D + 1];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int b = blockIdx.x / p.Hq, h = blockIdx.x % p.Hq, hk = h / (p.Hq / p.Hkv);
    const int dg = tid % LPR, kl = tid / LPR;

    if (tid < D)
        sQ[tid] = T::to_float(((const unsigned short*)p.q)[(int64_t)b * p.q_sb + (int64_t)h * p.q_sh + tid]);
    __syncthreads();
    float qv[8];
#pragma unroll
    for (int x = 0; x < 8; ++x) qv[x] = sQ[8 * dg + x];

    const char* kbase = (const char*)p.k + 2 * ((int64_t)b * p.k_sb + (int64_t)hk * p.k_sh) + 16 * dg;
    const char* vbase = (const char*)p.v + 2 * ((int64_t)b * p.v_sb + (int64_t)hk * p.v_sh) + 16 * dg;
    const int first = (p.window > 0 && p.window < p.Sk) ? p.Sk - p.window : 0;

    auto block_reduce = [&](float x, bool is_max) {
        x = is_max ? wave_max(x) : wave_sum(x);
        __syncthreads();  // sRed is free again
        if (lane == 0) sRed[wave] = x;
        __syncthreads();
        float r = sRed[0];
#pragma unroll
        for (int w = 1; w < DEC_THREADS / 64; ++w) r = is_max ? fmaxf(r, sRed[w]) : r + sRed[w];
        return r;
    };

    float m = -INFINITY, l = 0.f, acc[8];
#pragma unroll
    for (int x = 0; x < 8; ++x) acc[x] = 0.f;

    for (int c0 = first; c0 < p.Sk; c0 += DEC_CHUNK) {
        const int n = min(DEC_CHUNK, p.Sk - c0);
        // scores of the chunk: LPR neighbouring lanes share a key
        for (int j0 = 0; j0 < n; j0 += NK) {
            const int j = j0 + kl;
            float part = 0.f;
            if (j < n) {
                const u32x4 kv = *(const u32x4*)(kbase + 2 * (int64_t)(c0 + j) * p.k_ss);
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    part = fmaf(T::to_float((unsigned short)(kv[x] & 0xFFFFu)), qv[2 * x], part);
                    part = fmaf(T::to_float((unsigned short)(kv[x] >> 16)), qv[2 * x + 1], part);
                }
            }
#pragma unroll
            for (int off = LPR / 2; off > 0; off >>= 1) part += __shfl_xor(part, off);
            if (j < n && dg == 0) {
                float s = part * p.scale;
                if (p.softcap > 0.f) s = p.softcap * tanhf(s / p.softcap);
                sS[j] = s;
            }
        }
        __syncthreads();
        float cm = -INFINITY;
        for (int j = tid; j < n; j += DEC_THREADS) cm = fmaxf(cm, sS[j]);
        cm = block_reduce(cm, true);
        const float mnew = fmaxf(m, cm);            // finite: every chunk holds at least one key
        const float alpha = __expf(m - mnew);       // 0 for the first chunk
        float ls = 0.f;
        for (int j = tid; j < n; j += DEC_THREADS) {
            const float e = __expf(sS[j] - mnew);
            sS[j] = e;
            ls += e;
        }
        ls = block_reduce(ls, false);               // (its barriers also publish the probabilities)
        l = l * alpha + ls;
        m = mnew;
#pragma unroll
        for (int x = 0; x < 8; ++x) acc[x] *= alpha;
        for (int j = kl; j < n; j += NK) {
            const float pj = sS[j];
            const u32x4 vv = *(const u32x4*)(vbase + 2 * (int64_t)(c0 + j) * p.v_ss);
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                acc[2 * x] = fmaf(pj, T::to_float((unsigned short)(vv[x] & 0xFFFFu)), acc[2 * x]);
                acc[2 * x + 1] = fmaf(pj, T::to_float((unsigned short)(vv[x] >> 16)), acc[2 * x + 1]);
            }
        }
        __syncthreads();  // everybody is done with this chunk's probabilities
    }
#pragma unroll
    for (int x = 0; x < 8; ++x) sAcc[kl][8 * dg + x] = acc[x];
    __syncthreads();
    if (tid < D) {
        float r = 0.f;
        for (int k2 = 0; k2 < NK; ++k2) r += sAcc[k2][tid];
        r /= l;
        unsigned short* op = (unsigned short*)p.o + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + tid;
        *op = (unsigned short)(T::pack2(r, 0.f) & 0xFFFFu);
    }
}

template <typename T>
static int launch_decode_t(const DecodeParams& p, hipStream_t stream) {
    const dim3 grid(p.B * p.Hq), block(DEC_THREADS);
    if (p.D == 128)
        hipLaunchKernelGGL((decode_kernel<T, 128>), grid, block, 0, stream, p);
    else if (p.D == 64)
        hipLaunchKernelGGL((decode_kernel<T, 64>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((decode_kernel<T, 32>), grid, block, 0, stream, p);
    return (int)hipGetLastError();
}

int launch_decode(const DecodeParams& p, int dtype, hipStream_t stream) {
    return dtype == 1 ? launch_decode_t<BF16>(p, stream) : launch_decode_t<F16>(p, stream);
}

}  // namespace bam
