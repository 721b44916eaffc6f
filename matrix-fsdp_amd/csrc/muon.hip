// Owner-rank Muon update of one matrix: momentum -> Newton-Schulz (bf16 MFMA GEMMs) -> parameter update.
//
// The iteration keeps X (m x n, m <= n) AND X^T (n x m) so that all three products of a step are
// K-contiguous "NT" GEMMs:
//     A  = X X^T                    P = Q = X          (symmetric: lower-triangle tiles, mirrored store)
//     B  = b A + c A A = b A + c A A^T   P = Q = A     (symmetric)
//     X' = a X + B X                P = B, Q = X^T     (writes X' and X'^T)
// Every product is rounded to bf16, as the reference's bf16 addmm / mm do.  Buffers are zero-padded to
// multiples of 256 so the GEMM needs no edge handling; zero rows and columns stay zero through the iteration.
#include "mfsdp_common.h"
#include "muon_elementwise.h"
#include "muon_gemm.h"

#include <algorithm>
#include <cmath>

namespace mfsdp {
namespace {

constexpr int64_t kPad = 256;
constexpr int64_t kAlign = 256;  // byte alignment of every workspace region

int64_t round_up(int64_t v, int64_t to) { return (v + to - 1) / to * to; }

struct Workspace {
  int m, n, mp, np;        // short / long side and their padded sizes
  bool tall;               // rows > cols: the iteration runs on the transpose
  uint16_t* X[2];          // mp x np
  uint16_t* XT[2];         // np x mp
  uint16_t* A;             // mp x mp
  uint16_t* B;             // mp x mp
  uint16_t* xraw;          // rows x cols unscaled bf16 update (aliases X[1])
  float* partials;
  float* scalars;
  GemmScratch gemm;        // fp32 partial tiles of K-split GEMM pieces
  int64_t bytes;
};

bool plan_workspace(int64_t rows, int64_t cols, void* base, Workspace* w) {
  if (rows <= 0 || cols <= 0 || rows > (1 << 30) || cols > (1 << 30)) return false;
  w->tall = rows > cols;
  w->m = static_cast<int>(std::min(rows, cols));
  w->n = static_cast<int>(std::max(rows, cols));
  w->mp = static_cast<int>(round_up(w->m, kPad));
  w->np = static_cast<int>(round_up(w->n, kPad));
  const int64_t x_bytes = round_up(static_cast<int64_t>(w->mp) * w->np * 2, kAlign);
  const int64_t a_bytes = round_up(static_cast<int64_t>(w->mp) * w->mp * 2, kAlign);
  char* p = static_cast<char*>(base);
  int64_t off = 0;
  auto take = [&](int64_t bytes) { char* r = p ? p + off : nullptr; off += bytes; return r; };
  w->X[0] = reinterpret_cast<uint16_t*>(take(x_bytes));
  w->X[1] = reinterpret_cast<uint16_t*>(take(x_bytes));
  w->XT[0] = reinterpret_cast<uint16_t*>(take(x_bytes));
  w->XT[1] = reinterpret_cast<uint16_t*>(take(x_bytes));
  w->A = reinterpret_cast<uint16_t*>(take(a_bytes));
  w->B = reinterpret_cast<uint16_t*>(take(a_bytes));
  w->scalars = reinterpret_cast<float*>(take(kAlign));
  w->gemm.partials = take(kGemmPartialsBytes);
  w->gemm.partials_bytes = kGemmPartialsBytes;
  // the sums of squares of the momentum kernel are consumed by the norm before the first product runs
  static_assert(kMuonMaxPartials * 4 <= kGemmPartialsBytes, "the partial sums borrow the products' scratch");
  w->partials = reinterpret_cast<float*>(w->gemm.partials);
  w->xraw = w->X[1];
  w->bytes = off;
  return true;
}

// Newton-Schulz on the update already sitting in w.xraw (rows x cols bf16) with per-block sums of squares in
// w.partials.  Leaves O in param layout at *ortho with leading dimension *ldo.
// The parameter update of the step, handed to the last product (see GemmNtArgs::update_param).
struct ParamUpdate {
  void* param = nullptr;
  int dtype = MFSDP_F32;
  float decay = 1.0f, neg_lr = 0.0f;
};

// With `update` and at least one step the last product writes the parameter itself and *ortho stays null.
int run_newton_schulz(const Workspace& w, int rows, int cols, int n_partials, float a, float b, float c, int steps,
                      float eps, bool shared, const ParamUpdate* update, const uint16_t** ortho, int* ldo, hipStream_t stream) {
  if (int rc = muon_norm(w.partials, n_partials, eps, w.scalars, stream)) return rc;
  // the input is rows x cols; the iteration wants the short side first
  uint16_t* same = w.tall ? w.XT[0] : w.X[0];   // rows_pad x cols_pad
  uint16_t* trans = w.tall ? w.X[0] : w.XT[0];  // cols_pad x rows_pad
  const int rows_pad = w.tall ? w.np : w.mp;
  const int cols_pad = w.tall ? w.mp : w.np;
  if (int rc = muon_scale_transpose(w.xraw, rows, cols, w.scalars, same, trans, rows_pad, cols_pad, stream)) return rc;
  for (int s = 0; s < steps; ++s) {
    const int cur = s & 1, nxt = cur ^ 1;
    GemmNtArgs g{};
    g.P = w.X[cur]; g.Q = w.X[cur]; g.D = nullptr; g.C = w.A; g.CT = nullptr;
    g.M = w.mp; g.N = w.mp; g.K = w.np;
    g.ldp = w.np; g.ldq = w.np; g.ldd = 0; g.ldc = w.mp; g.ldct = 0;
    g.alpha = 1.0f; g.beta = 0.0f; g.symmetric = 1; g.shared = shared;
    if (int rc = gemm_nt_bf16(g, w.gemm, stream)) return rc;
    if (c == 0.0f) {
      // addmm with alpha = 0 leaves beta * A (the product is not formed at all, torch/optim/_muon.py:61 with a
      // quadratic polynomial); the GEMM's D path needs alpha != 0 (it adds (beta / alpha) D to the accumulators)
      if (int rc = muon_scale_bf16(w.B, w.A, static_cast<int64_t>(w.mp) * w.mp, b, stream)) return rc;
    } else {
      g = GemmNtArgs{};
      g.P = w.A; g.Q = w.A; g.D = w.A; g.C = w.B; g.CT = nullptr;
      g.d_transposed_is_q = 1;  // A is symmetric
      g.M = w.mp; g.N = w.mp; g.K = w.mp;
      g.ldp = w.mp; g.ldq = w.mp; g.ldd = w.mp; g.ldc = w.mp; g.ldct = 0;
      g.alpha = c; g.beta = b; g.symmetric = 1; g.shared = shared;
      if (int rc = gemm_nt_bf16(g, w.gemm, stream)) return rc;
    }
    g = GemmNtArgs{};
    g.P = w.B; g.Q = w.XT[cur]; g.D = w.X[cur]; g.C = w.X[nxt]; g.CT = w.XT[nxt];
    g.d_transposed_is_q = 1;  // Q = X^T
    g.M = w.mp; g.N = w.np; g.K = w.mp;
    g.ldp = w.mp; g.ldq = w.mp; g.ldd = w.np; g.ldc = w.np; g.ldct = w.mp;
    g.alpha = 1.0f; g.beta = a; g.symmetric = 0;
    if (s + 1 == steps) {  // the last step only has to leave O in the parameter's orientation
      if (w.tall) g.skip_c = 1;
      else g.CT = nullptr;
      if (update != nullptr) {  // ... or take it straight into the parameter: O is never stored
        g.update_param = update->param;
        g.update_dtype = update->dtype;
        g.update_rows = rows;
        g.update_cols = cols;
        g.update_transposed = w.tall ? 1 : 0;
        g.update_decay = update->decay;
        g.update_neg_lr = update->neg_lr;
      }
    }
    if (int rc = gemm_nt_bf16(g, w.gemm, stream)) return rc;
  }
  const int fin = steps & 1;
  *ortho = (update != nullptr && steps > 0) ? nullptr : (w.tall ? w.XT[fin] : w.X[fin]);
  *ldo = w.tall ? w.mp : w.np;
  return MFSDP_OK;
}

int check_common(int64_t rows, int64_t cols, float a, float b, float c, int steps, const void* workspace, int64_t workspace_bytes, Workspace* w) {
  // everything that can be refused is refused here, before the first kernel is enqueued (a step must not be left half applied)
  if (!std::isfinite(a) || !std::isfinite(b) || !std::isfinite(c) || (c != 0.0f && !std::isfinite(b / c)))
    return fail(MFSDP_ERR_INVALID, "Newton-Schulz coefficients must be finite (and b / c representable), got (%g, %g, %g)", a, b, c);
  if (steps < 0 || steps >= 100) return fail(MFSDP_ERR_INVALID, "Number of steps must be less than 100 for computational efficiency");
  if (!plan_workspace(rows, cols, const_cast<void*>(workspace), w))
    return fail(MFSDP_ERR_INVALID, "Input tensor gradient must be a 2D matrix with positive sizes, got %lld x %lld",
                static_cast<long long>(rows), static_cast<long long>(cols));
  if (workspace == nullptr || workspace_bytes < w->bytes)
    return fail(MFSDP_ERR_INVALID, "workspace of %lld bytes needed, got %lld", static_cast<long long>(w->bytes),
                static_cast<long long>(workspace_bytes));
  if (reinterpret_cast<uintptr_t>(workspace) % kAlign) return fail(MFSDP_ERR_INVALID, "workspace must be %lld-byte aligned", static_cast<long long>(kAlign));
  return MFSDP_OK;
}

}  // namespace
}  // namespace mfsdp

using namespace mfsdp;

extern "C" int64_t mfsdp_muon_workspace_bytes(int64_t rows, int64_t cols) {
  Workspace w;
  return plan_workspace(rows, cols, nullptr, &w) ? w.bytes : 0;
}

extern "C" int64_t mfsdp_muon_executed_flops(int64_t rows, int64_t cols, int steps, int flags) {
  Workspace w;
  if (steps < 0 || !plan_workspace(rows, cols, nullptr, &w)) return 0;
  GemmNtArgs gram{}, poly{}, update{};
  gram.M = gram.N = w.mp; gram.K = w.np; gram.symmetric = 1;
  poly.M = poly.N = poly.K = w.mp; poly.symmetric = 1;
  gram.shared = poly.shared = (flags & MFSDP_MUON_SHARED_MACHINE) != 0;
  update.M = w.mp; update.N = w.np; update.K = w.mp;
  return steps * (gemm_nt_executed_flops(gram) + gemm_nt_executed_flops(poly) + gemm_nt_executed_flops(update));
}

extern "C" int mfsdp_newton_schulz(const void* update, int update_dtype, int64_t rows, int64_t cols, float a, float b, float c,
                                   int steps, float eps, void* out_bf16, void* workspace, int64_t workspace_bytes, void* stream) {
  Workspace w;
  if (int rc = check_common(rows, cols, a, b, c, steps, workspace, workspace_bytes, &w)) return rc;
  if (update_dtype != MFSDP_F32 && update_dtype != MFSDP_BF16) return fail(MFSDP_ERR_INVALID, "update dtype must be f32 or bf16");
  if (!update || !out_bf16) return fail(MFSDP_ERR_INVALID, "null tensor pointer");
  hipStream_t s = as_stream(stream);
  int n_partials = 0;
  if (int rc = muon_momentum(update, nullptr, update_dtype, rows * cols, 0.0, 0, false, w.xraw, w.partials, &n_partials, s)) return rc;
  const uint16_t* ortho = nullptr;
  int ldo = 0;
  if (int rc = run_newton_schulz(w, static_cast<int>(rows), static_cast<int>(cols), n_partials, a, b, c, steps, eps, false, nullptr, &ortho, &ldo, s)) return rc;
  return muon_extract(out_bf16, ortho, static_cast<int>(rows), static_cast<int>(cols), ldo, s);
}

extern "C" int mfsdp_muon_step_ex(void* param, const void* grad, void* momentum_buf, int dtype, int64_t rows, int64_t cols, double lr,
                                  double weight_decay, double momentum, int nesterov, float a, float b, float c, int steps, float eps,
                                  double adjusted_lr, int flags, void* workspace, int64_t workspace_bytes, void* stream) {
  Workspace w;
  if (int rc = check_common(rows, cols, a, b, c, steps, workspace, workspace_bytes, &w)) return rc;
  if (dtype != MFSDP_F32 && dtype != MFSDP_BF16) return fail(MFSDP_ERR_INVALID, "dtype must be f32 or bf16");
  if (!param || !grad || !momentum_buf) return fail(MFSDP_ERR_INVALID, "null tensor pointer");
  if (!(lr >= 0.0)) return fail(MFSDP_ERR_INVALID, "Learning rate should be >= 0 but is: %g", lr);
  if (!(momentum >= 0.0)) return fail(MFSDP_ERR_INVALID, "momentum should be >= 0 but is: %g", momentum);
  if (!(weight_decay >= 0.0)) return fail(MFSDP_ERR_INVALID, "weight decay should be >= 0 but is: %g", weight_decay);
  if (flags & ~MFSDP_MUON_SHARED_MACHINE) return fail(MFSDP_ERR_INVALID, "unknown flags 0x%x", flags);
  hipStream_t s = as_stream(stream);
  int n_partials = 0;
  if (int rc = muon_momentum(grad, momentum_buf, dtype, rows * cols, momentum, nesterov, true, w.xraw, w.partials, &n_partials, s)) return rc;
  const uint16_t* ortho = nullptr;
  int ldo = 0;
  // the host scalars are doubles, as in Python: 1 - lr * wd and -adjusted_lr are rounded to fp32 once, where the
  // tensor operation takes them
  ParamUpdate update;
  update.param = param;
  update.dtype = dtype;
  update.decay = static_cast<float>(1.0 - lr * weight_decay);
  update.neg_lr = static_cast<float>(-adjusted_lr);
  if (int rc = run_newton_schulz(w, static_cast<int>(rows), static_cast<int>(cols), n_partials, a, b, c, steps, eps,
                                 (flags & MFSDP_MUON_SHARED_MACHINE) != 0, &update, &ortho, &ldo, s))
    return rc;
  if (ortho == nullptr) return MFSDP_OK;  // the last product has updated the parameter
  return muon_apply(param, dtype, ortho, static_cast<int>(rows), static_cast<int>(cols), ldo, update.decay, update.neg_lr, s);
}

extern "C" int mfsdp_muon_step(void* param, const void* grad, void* momentum_buf, int dtype, int64_t rows, int64_t cols, double lr,
                               double weight_decay, double momentum, int nesterov, float a, float b, float c, int steps, float eps,
                               double adjusted_lr, void* workspace, int64_t workspace_bytes, void* stream) {
  return mfsdp_muon_step_ex(param, grad, momentum_buf, dtype, rows, cols, lr, weight_decay, momentum, nesterov, a, b, c, steps, eps,
                            adjusted_lr, 0, workspace, workspace_bytes, stream);
}

extern "C" int mfsdp_gemm_nt_bf16(const void* p, const void* q, void* c, int m, int n, int k, void* partials, int64_t partials_bytes, void* stream) {
  GemmNtArgs g{};
  g.P = p; g.Q = q; g.C = c;
  g.M = m; g.N = n; g.K = k;
  g.ldp = k; g.ldq = k; g.ldc = n;
  g.alpha = 1.0f;
  GemmScratch scratch;
  scratch.partials = partials;
  scratch.partials_bytes = partials ? partials_bytes : 0;
  return gemm_nt_bf16(g, scratch, as_stream(stream));
}

extern "C" void mfsdp_set_muon_tuning(int general_variant, int symmetric_variant, int group_m, int split_remainder,
                                      int max_splits) {
  GemmTuning t = get_gemm_tuning();
  if (general_variant > 0) t.general_variant = general_variant;
  if (symmetric_variant > 0) t.symmetric_variant = symmetric_variant;
  if (group_m > 0) t.group_m = group_m;
  if (split_remainder > 0) t.split_remainder = split_remainder == 1;
  if (max_splits > 0) t.max_splits = max_splits;
  set_gemm_tuning(t);
}
