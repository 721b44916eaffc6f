// Fused AdamW over a flat fp32 shard: one launch reads param, grad and both moments once and writes
// param and both moments once (28 B per element with fp32 grads; amsgrad adds the running maximum of the
// second moment, 8 B more).
#include "mfsdp_common.h"

#include <algorithm>
#include <cmath>

namespace mfsdp {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct AdamWArgs {
  float decay;       // 1 - lr * weight_decay
  float beta1;
  float one_minus_beta1;
  float beta2;
  float one_minus_beta2;
  float neg_step_size;  // -lr / (1 - beta1^t)
  float bc2_sqrt;    // sqrt(1 - beta2^t)
  float eps;
  float grad_sign;   // -1 with maximize, else +1
};

// Tensor.lerp as ATen evaluates it.
__device__ __forceinline__ float lerp_aten(float start, float end, float weight) {
  // one fused multiply-add from the nearer end point, the form ATen's vectorised kernel spells out
  // (fmadd(weight, end - start, start) / fmadd(weight - 1, end - start, end)); written explicitly so that the
  // compiler's contraction choices cannot differ between code paths
  const float diff = end - start;
  return fabsf(weight) < 0.5f ? __builtin_fmaf(weight, diff, start) : __builtin_fmaf(weight - 1.0f, diff, end);
}

// The operation order of the single-tensor path of torch.optim.AdamW:
//   g = -g (maximize);  p *= 1 - lr*wd;  m += (g - m)*(1 - b1);  v = v*b2 + (1 - b2)*g*g;
//   vmax = max(vmax, v) (amsgrad);  p += (-step_size * m) / (sqrt(amsgrad ? vmax : v)/sqrt(bc2) + eps)
// No multiply-add contraction: every operation rounds on its own, so an element gets the same bits whether it is
// updated in the vector body or in the scalar tail, alone or as part of a merged span.
template <bool AMSGRAD>
__device__ __forceinline__ void adamw_one(float& p, float g, float& m, float& v, float& vmax, const AdamWArgs& a) {
#pragma clang fp contract(off)
  g = g * a.grad_sign;
  p = p * a.decay;
  m = lerp_aten(m, g, a.one_minus_beta1);
  v = v * a.beta2 + (a.one_minus_beta2 * g) * g;
  float second = v;
  if constexpr (AMSGRAD) {
    vmax = (vmax != vmax || v != v) ? __builtin_nanf("") : fmaxf(vmax, v);  // torch.maximum propagates NaN
    second = vmax;
  }
  const float denom = sqrtf(second) / a.bc2_sqrt + a.eps;  // sqrtf is correctly rounded; __fsqrt_rn is the fast native one here
  p = p + (a.neg_step_size * m) / denom;
}

template <bool NT, typename T>
__device__ __forceinline__ T ld(const T* p) {
  if constexpr (NT) return __builtin_nontemporal_load(p);
  else return *p;
}
template <bool NT, typename T>
__device__ __forceinline__ void st(T* p, T v) {
  if constexpr (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

template <bool GRAD_BF16, int U, bool NT, bool AMSGRAD>
__global__ void __launch_bounds__(256)
adamw_kernel(float* __restrict__ param, const void* __restrict__ grad, float* __restrict__ exp_avg,
             float* __restrict__ exp_avg_sq, float* __restrict__ max_exp_avg_sq, int64_t n_vec, int64_t numel, AdamWArgs a) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  // U vectors per thread and iteration, all of their loads issued before the first use
  for (int64_t base = static_cast<int64_t>(blockIdx.x) * blockDim.x * U + threadIdx.x; base < n_vec; base += stride * U) {
    f32x4 p[U], m[U], v[U], g[U], vmax[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * blockDim.x;
      if (i < n_vec) {
        p[u] = ld<NT>(reinterpret_cast<const f32x4*>(param) + i);
        m[u] = ld<NT>(reinterpret_cast<const f32x4*>(exp_avg) + i);
        v[u] = ld<NT>(reinterpret_cast<const f32x4*>(exp_avg_sq) + i);
        if constexpr (AMSGRAD) vmax[u] = ld<NT>(reinterpret_cast<const f32x4*>(max_exp_avg_sq) + i);
        if constexpr (GRAD_BF16) {
          const u32x2 raw = ld<NT>(reinterpret_cast<const u32x2*>(grad) + i);
          g[u].x = __uint_as_float(raw.x << 16);
          g[u].y = __uint_as_float(raw.x & 0xffff0000u);
          g[u].z = __uint_as_float(raw.y << 16);
          g[u].w = __uint_as_float(raw.y & 0xffff0000u);
        } else {
          g[u] = ld<NT>(reinterpret_cast<const f32x4*>(grad) + i);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * blockDim.x;
      if (i < n_vec) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          float pk = p[u][k], mk = m[u][k], vk = v[u][k], xk = 0.0f;
          if constexpr (AMSGRAD) xk = vmax[u][k];
          adamw_one<AMSGRAD>(pk, g[u][k], mk, vk, xk, a);
          p[u][k] = pk; m[u][k] = mk; v[u][k] = vk;
          if constexpr (AMSGRAD) vmax[u][k] = xk;
        }
        st<NT>(reinterpret_cast<f32x4*>(param) + i, p[u]);
        st<NT>(reinterpret_cast<f32x4*>(exp_avg) + i, m[u]);
        st<NT>(reinterpret_cast<f32x4*>(exp_avg_sq) + i, v[u]);
        if constexpr (AMSGRAD) st<NT>(reinterpret_cast<f32x4*>(max_exp_avg_sq) + i, vmax[u]);
      }
    }
  }
  // scalar tail: the elements past the last whole vector (everything when the tensors are not 16-byte aligned)
  for (int64_t i = n_vec * 4 + static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < numel; i += stride) {
    float g;
    if constexpr (GRAD_BF16) g = __uint_as_float(static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(grad)[i]) << 16);
    else g = reinterpret_cast<const float*>(grad)[i];
    float p = param[i], m = exp_avg[i], v = exp_avg_sq[i], x = 0.0f;
    if constexpr (AMSGRAD) x = max_exp_avg_sq[i];
    adamw_one<AMSGRAD>(p, g, m, v, x, a);
    param[i] = p; exp_avg[i] = m; exp_avg_sq[i] = v;
    if constexpr (AMSGRAD) max_exp_avg_sq[i] = x;
  }
}

}  // namespace
}  // namespace mfsdp

using namespace mfsdp;

extern "C" int mfsdp_adamw_step_ex(float* param, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
                                   float* max_exp_avg_sq, int64_t numel, int64_t step, double lr, double beta1,
                                   double beta2, double eps, double weight_decay, int maximize, void* stream) {
  if (numel < 0) return fail(MFSDP_ERR_INVALID, "numel must be non-negative");
  if (step < 1) return fail(MFSDP_ERR_INVALID, "step must be >= 1, got %lld", static_cast<long long>(step));
  if (grad_dtype != MFSDP_F32 && grad_dtype != MFSDP_BF16) return fail(MFSDP_ERR_INVALID, "grad_dtype must be f32 or bf16");
  if (numel == 0) return MFSDP_OK;
  if (!param || !grad || !exp_avg || !exp_avg_sq) return fail(MFSDP_ERR_INVALID, "null tensor pointer");
  const uintptr_t align = reinterpret_cast<uintptr_t>(param) | reinterpret_cast<uintptr_t>(exp_avg) |
                          reinterpret_cast<uintptr_t>(exp_avg_sq) | reinterpret_cast<uintptr_t>(max_exp_avg_sq);
  const uintptr_t galign = reinterpret_cast<uintptr_t>(grad);
  const bool vec_ok = (align % 16 == 0) && (galign % (grad_dtype == MFSDP_BF16 ? 8 : 16) == 0);
  AdamWArgs a;
  // every scalar is computed in double from the hyper-parameters as given, as Python does, and rounded to fp32 once
  // (1 - beta2 formed from an fp32 beta2 = 0.999 would already be off by 1.3e-5)
  const double bc1 = 1.0 - std::pow(beta1, static_cast<double>(step));
  const double bc2 = 1.0 - std::pow(beta2, static_cast<double>(step));
  a.decay = static_cast<float>(1.0 - lr * weight_decay);
  a.beta1 = static_cast<float>(beta1);
  a.one_minus_beta1 = static_cast<float>(1.0 - beta1);
  a.beta2 = static_cast<float>(beta2);
  a.one_minus_beta2 = static_cast<float>(1.0 - beta2);
  a.neg_step_size = static_cast<float>(-lr / bc1);
  a.bc2_sqrt = static_cast<float>(std::sqrt(bc2));
  a.eps = static_cast<float>(eps);
  a.grad_sign = maximize ? -1.0f : 1.0f;
  const int64_t n_vec = vec_ok ? numel / 4 : 0;
  // Non-temporal accesses (every byte is touched once) and one small workgroup per block of each stream rather than a
  // persistent grid: workgroups are dispatched in order, so the ones running at any moment sweep neighbouring
  // addresses of all seven streams, and the finer the workgroups the more evenly loads and stores mix.  41 M
  // elements: one wavefront per workgroup with two vectors per thread 6.22 TB/s (one vector 5.55, four 6.01; 256 threads
  // with four vectors 5.93, with two 5.94; 16 persistent workgroups per CU 5.71); 5.1-5.5 TB/s with cached loads or
  // stores.
  constexpr int threads = 64, per_thread = 2;
  const int64_t work = std::max<int64_t>((n_vec + per_thread - 1) / per_thread, numel - n_vec * 4);
  const int64_t want = std::max<int64_t>(1, (work + threads - 1) / threads);
  const int64_t cap = (int64_t{1} << 31) - 1;  // the loops stride by the grid, so a capped grid stays correct
  const dim3 grid(static_cast<uint32_t>(std::min(want, cap)));
#define MFSDP_ADAMW_U(BF16_, AMS_, U_)                                                                                  \
  hipLaunchKernelGGL((adamw_kernel<BF16_, U_, true, AMS_>), grid, dim3(threads), 0, as_stream(stream), \
                     param, grad, exp_avg, exp_avg_sq, max_exp_avg_sq, n_vec, numel, a)
#define MFSDP_ADAMW(BF16_, AMS_) MFSDP_ADAMW_U(BF16_, AMS_, per_thread)
  const bool bf16 = grad_dtype == MFSDP_BF16;
  if (max_exp_avg_sq != nullptr) {
    if (bf16) MFSDP_ADAMW(true, true); else MFSDP_ADAMW(false, true);
  } else {
    if (bf16) MFSDP_ADAMW(true, false); else MFSDP_ADAMW(false, false);
  }
#undef MFSDP_ADAMW
#undef MFSDP_ADAMW_U
  MFSDP_CHECK_LAUNCH("adamw_kernel");
  return MFSDP_OK;
}

extern "C" int mfsdp_adamw_step(float* param, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
                                int64_t numel, int64_t step, double lr, double beta1, double beta2, double eps,
                                double weight_decay, void* stream) {
  return mfsdp_adamw_step_ex(param, grad, grad_dtype, exp_avg, exp_avg_sq, nullptr, numel, step, lr, beta1, beta2, eps,
                             weight_decay, 0, stream);
}
