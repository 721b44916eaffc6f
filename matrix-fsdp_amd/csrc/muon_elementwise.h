// Element-wise stages of the Muon update (see muon_elementwise.hip).  Internal to libmfsdp_hip.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace mfsdp {

constexpr int kMuonMaxPartials = 1 << 18;  // workgroups of the momentum kernel = partial sums of squares (1 MiB of fp32)

// xraw <- bf16(u), partials <- per-block sums of bf16(u)^2, where u is the momentum/Nesterov update
// (with_momentum; buf updated in place) or grad itself.  dtype: MFSDP_F32 / MFSDP_BF16 of grad and buf.
int muon_momentum(const void* grad, void* buf, int dtype, int64_t numel, double momentum, int nesterov, bool with_momentum,
                  void* xraw, float* partials, int* n_partials, hipStream_t stream);
// scalars[0] <- max(bf16(sqrt(sum partials)), bf16(eps))
int muon_norm(const float* partials, int n_partials, float eps, float* scalars, hipStream_t stream);
// same[rows_pad x cols_pad] <- bf16(xraw / scalars[0]) zero-padded; trans[cols_pad x rows_pad] <- its transpose
int muon_scale_transpose(const void* xraw, int rows, int cols, const float* scalars, void* same, void* trans, int rows_pad,
                         int cols_pad, hipStream_t stream);
// param <- round(round(param*decay) + neg_lr*ortho), ortho bf16 with leading dimension ldo
int muon_apply(void* param, int dtype, const void* ortho, int rows, int cols, int ldo, float decay, float neg_lr,
               hipStream_t stream);
// out <- bf16(scale * in) over numel contiguous bf16 (whole 16-byte groups)
int muon_scale_bf16(void* out, const void* in, int64_t numel, float scale, hipStream_t stream);
// out[rows x cols] contiguous bf16 <- ortho (leading dimension ldo)
int muon_extract(void* out, const void* ortho, int rows, int cols, int ldo, hipStream_t stream);

}  // namespace mfsdp
