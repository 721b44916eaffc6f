// bf16 MFMA GEMM used by the Newton-Schulz iteration (gfx950).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace mfsdp {

// C = bf16( alpha * (P * Q^T) + beta * D ), fp32 accumulation.
//   P: M x K row-major (ldp), Q: N x K row-major (ldq), D / C: M x N row-major (ldd / ldc).
//   M, N multiples of 256 and K a multiple of 64 (callers zero-pad their operands).
//   D may be null (beta ignored).  CT, when non-null, also receives the transpose: CT[n][m] = C[m][n]
//   (ldct).  symmetric: P*Q^T is known to be symmetric (M == N); only tiles on or below the diagonal are
//   computed and each off-diagonal tile is also written mirrored into C.
struct GemmNtArgs {
  const void* P;
  const void* Q;
  const void* D;
  void* C;
  void* CT;
  int M, N, K;
  int ldp, ldq, ldd, ldc, ldct;
  float alpha, beta;
  int symmetric;
};

// Enqueues the GEMM on `stream`; returns an MFSDP_* status.
int gemm_nt_bf16(const GemmNtArgs& args, hipStream_t stream);

// Tile variant selection for experiments: 0 = default heuristic, 1 = 256x256 tiles, 2 = 128x128 tiles.
void set_gemm_variant(int variant);

}  // namespace mfsdp
