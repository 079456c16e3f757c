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
    float* lse;                // (B, Hq, Sq_rounded)
    float* delta;              // (B, Hq, Sq_rounded)
    // Bitfields of the query rows (B, Sq) and of the keys (B, Sk), and their global positions.  Plain
    // attention: both point at the one bitfield tensor and the positions are null (position = row /
    // column number).  Index-tensor attention (context-parallel shards): gathered copies and positions.
    const int64_t* bfq;
    const int64_t* bfk;
    int64_t bfq_sb, bfk_sb;
    const int* posq;
    const int* posk;
    const int8_t* flags;       // (B, num_m, num_n)
    int64_t flags_sb, flags_sm;
    int B, Sq, Sk, Hq, Hkv, D;
    int Sq_rounded, num_m, num_n, num_kt;  // ceil(Sq/128)*128, ceil(Sq/128), ceil(Sk/32), ceil(Sk/128)
    float scale;
};

int launch_tile_flags(const int64_t* bf, int64_t bf_stride_b, int8_t* flags, int64_t flags_stride_b,
                      int64_t flags_stride_m, int B, int S, hipStream_t stream);
int launch_materialize_mask(const int64_t* bf, int64_t bf_stride_b, uint8_t* out, int B, int S,
                            hipStream_t stream);
int launch_gather_bitfields(const int64_t* bf, int64_t bf_stride_b, int L, const int64_t* idx, int n, int64_t* out_bits,
                            int64_t out_stride_b, int* out_pos, int B, hipStream_t stream);
int launch_fwd(const AttnParams& p, int dtype, hipStream_t stream);
int launch_bwd_preprocess(const AttnParams& p, int dtype, hipStream_t stream);
int launch_bwd_dkdv(const AttnParams& p, int dtype, hipStream_t stream);
int launch_bwd_dq(const AttnParams& p, int dtype, hipStream_t stream);

}  // namespace bam
