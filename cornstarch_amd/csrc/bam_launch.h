// Host-side launch interface between the C ABI (bam_abi.hip) and the kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bam {

// Number of 64-key (forward, dQ) or 128-row (dK/dV) tiles a workgroup can list in LDS.
constexpr int MAX_LIST = 2048;

struct Tensor4 {  // logical (B, S, H, D), unit stride along D, strides in elements
    const void* ptr;
    int64_t sb, ss, sh;
};

struct AttnParams {
    Tensor4 q, k, v, o, dout;  // 16-bit tensors
    Tensor4 dq, dk, dv;        // gradients: fp32 accumulated into, or (grad_typed) input dtype, overwritten
    int grad_typed;
    float* lse;                // (B, Hq, S_rounded)
    float* delta;              // (B, Hq, S_rounded)
    const int64_t* bf;
    int64_t bf_sb;
    const int8_t* flags;
    int64_t flags_sb, flags_sm;
    int B, S, Hq, Hkv, D;
    int S_rounded, num_m, num_n;  // ceil(S/128)*128, ceil(S/128), ceil(S/32)
    float scale;
};

int launch_tile_flags(const int64_t* bf, int64_t bf_stride_b, int8_t* flags, int64_t flags_stride_b,
                      int64_t flags_stride_m, int B, int S, hipStream_t stream);
int launch_materialize_mask(const int64_t* bf, int64_t bf_stride_b, uint8_t* out, int B, int S,
                            hipStream_t stream);
int launch_fwd(const AttnParams& p, int dtype, hipStream_t stream);
int launch_bwd_preprocess(const AttnParams& p, int dtype, hipStream_t stream);
int launch_bwd_dkdv(const AttnParams& p, int dtype, hipStream_t stream);
int launch_bwd_dq(const AttnParams& p, int dtype, hipStream_t stream);

}  // namespace bam
