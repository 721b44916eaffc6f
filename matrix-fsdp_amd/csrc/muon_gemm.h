// bf16 MFMA GEMM used by the Newton-Schulz iteration (gfx950).  Internal to libmfsdp_hip.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace mfsdp {

// C = bf16( alpha * (P * Q^T) + beta * D ), fp32 accumulation.
//   P: M x K row-major (ldp), Q: N x K row-major (ldq), D / C: M x N row-major (ldd / ldc).
//   M, N multiples of 256 and K a multiple of 64 (callers zero-pad their operands).
//   D may be null (beta ignored); with D, Q must hold its transpose (d_transposed_is_q, K >= M).  CT, when non-null, also receives the transpose: CT[n][m] = C[m][n]
//   (ldct); with skip_c only CT is written.  symmetric: P*Q^T is known to be symmetric (M == N); only tiles on or below the diagonal are
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
  int skip_c;  // general product with CT set: write only the transposed output
  int d_transposed_is_q;  // the caller's word that Q holds D^T (Q[n][k] == D[k][n] for k < M): required with D, whose
                          // values whole tiles pick out of the Q slabs on their way through LDS (the fix-up of K-split
                          // pieces reads D itself)
  // Parameter update in the epilogue (the last product of a Muon step): when update_param is set, nothing is stored to
  // C / CT; every element o = bf16(alpha P Q^T + beta D) of the update_rows x update_cols corner instead goes into
  //     param <- round(param * update_decay) + update_neg_lr * o        (torch/optim/_muon.py:313-315)
  // on the contiguous row-major parameter of dtype update_dtype (MFSDP_F32 / MFSDP_BF16).  update_transposed: the
  // parameter holds the transpose of C (update_rows counts C's columns then).  General products only.
  void* update_param;
  int update_dtype;
  int update_rows, update_cols;
  int update_transposed;
  float update_decay, update_neg_lr;
  int update_vectors;  // set by gemm_nt_bf16: groups of eight parameter elements may use 16-byte accesses
  int shared;  // other matrices' products run beside this one on other streams: a symmetric product then takes the
               // 256 x 256 tiles even where their triangle fills only part of the CUs (the rest works for the others)
};

// Device scratch for the K-split pieces of the last partial round of tiles (fp32 partial tiles).
struct GemmScratch {
  void* partials = nullptr;
  int64_t partials_bytes = 0;
};
constexpr int64_t kGemmPartialsBytes = 64ll << 20;

struct GemmTuning {
  int general_variant = 1;    // 1: 256x256 tile / 8 waves / one workgroup per CU, 2: 128x128 tile / 4 waves / two per CU
  int symmetric_variant = 3;  // 1, 2 as above; 3: whichever fills the CUs better for the product at hand
  int group_m = 4;            // general products: tile rows walked together (the workgroups of one XCD share their P panels)
  int split_remainder = 1;    // split the tiles of the last partial round along K
  int max_splits = 16;
};
void set_gemm_tuning(const GemmTuning& tuning);
GemmTuning get_gemm_tuning();

// Flops the kernels execute for this product with the current tuning: 2 * tile area * K per computed tile (a symmetric
// product computes the tiles on or below the diagonal only).
int64_t gemm_nt_executed_flops(const GemmNtArgs& args);

// Enqueues the GEMM on `stream`; returns an MFSDP_* status.
int gemm_nt_bf16(const GemmNtArgs& args, const GemmScratch& scratch, hipStream_t stream);

}  // namespace mfsdp
