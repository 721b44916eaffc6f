// Fused AdamW over a flat fp32 shard: one launch reads param, grad and both moments once and writes
// param and both moments once (28 B per element with fp32 grads).
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
};

// Tensor.lerp as ATen evaluates it: the form that is exact at the nearer end point.
__device__ __forceinline__ float lerp_aten(float start, float end, float weight) {
  const float diff = end - start;
  return weight < 0.5f ? start + weight * diff : end - diff * (1.0f - weight);
}

// The operation order of the single-tensor path of torch.optim.AdamW:
//   p *= 1 - lr*wd;  m += (g - m)*(1 - b1);  v = v*b2 + (1 - b2)*g*g;
//   p += (-step_size * m) / (sqrt(v)/sqrt(bc2) + eps)
__device__ __forceinline__ void adamw_one(float& p, float g, float& m, float& v, const AdamWArgs& a) {
  p = p * a.decay;
  m = lerp_aten(m, g, a.one_minus_beta1);
  v = v * a.beta2 + (a.one_minus_beta2 * g) * g;
  const float denom = __fsqrt_rn(v) / a.bc2_sqrt + a.eps;
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

template <bool GRAD_BF16, int U, bool NT>
__global__ void __launch_bounds__(256)
adamw_kernel(float* __restrict__ param, const void* __restrict__ grad, float* __restrict__ exp_avg,
             float* __restrict__ exp_avg_sq, int64_t n_vec, int64_t numel, AdamWArgs a) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  // U vectors per thread and iteration, all of their loads issued before the first use
  for (int64_t base = static_cast<int64_t>(blockIdx.x) * blockDim.x * U + threadIdx.x; base < n_vec; base += stride * U) {
    f32x4 p[U], m[U], v[U], g[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * 256;
      if (i < n_vec) {
        p[u] = ld<NT>(reinterpret_cast<const f32x4*>(param) + i);
        m[u] = ld<NT>(reinterpret_cast<const f32x4*>(exp_avg) + i);
        v[u] = ld<NT>(reinterpret_cast<const f32x4*>(exp_avg_sq) + i);
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
      const int64_t i = base + u * 256;
      if (i < n_vec) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          float pk = p[u][k], mk = m[u][k], vk = v[u][k];
          adamw_one(pk, g[u][k], mk, vk, a);
          p[u][k] = pk; m[u][k] = mk; v[u][k] = vk;
        }
        st<NT>(reinterpret_cast<f32x4*>(param) + i, p[u]);
        st<NT>(reinterpret_cast<f32x4*>(exp_avg) + i, m[u]);
        st<NT>(reinterpret_cast<f32x4*>(exp_avg_sq) + i, v[u]);
      }
    }
  }
  // scalar tail: the elements past the last whole vector (everything when the tensors are not 16-byte aligned)
  for (int64_t i = n_vec * 4 + static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < numel; i += stride) {
    float g;
    if constexpr (GRAD_BF16) g = __uint_as_float(static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(grad)[i]) << 16);
    else g = reinterpret_cast<const float*>(grad)[i];
    float p = param[i], m = exp_avg[i], v = exp_avg_sq[i];
    adamw_one(p, g, m, v, a);
    param[i] = p; exp_avg[i] = m; exp_avg_sq[i] = v;
  }
}

}  // namespace
}  // namespace mfsdp

using namespace mfsdp;

extern "C" int mfsdp_adamw_step(float* param, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
                                int64_t numel, int64_t step, float lr, float beta1, float beta2, float eps,
                                float weight_decay, void* stream) {
  if (numel < 0) return fail(MFSDP_ERR_INVALID, "numel must be non-negative");
  if (step < 1) return fail(MFSDP_ERR_INVALID, "step must be >= 1, got %lld", static_cast<long long>(step));
  if (grad_dtype != MFSDP_F32 && grad_dtype != MFSDP_BF16) return fail(MFSDP_ERR_INVALID, "grad_dtype must be f32 or bf16");
  if (numel == 0) return MFSDP_OK;
  if (!param || !grad || !exp_avg || !exp_avg_sq) return fail(MFSDP_ERR_INVALID, "null tensor pointer");
  const uintptr_t align = reinterpret_cast<uintptr_t>(param) | reinterpret_cast<uintptr_t>(exp_avg) |
                          reinterpret_cast<uintptr_t>(exp_avg_sq);
  const uintptr_t galign = reinterpret_cast<uintptr_t>(grad);
  const bool vec_ok = (align % 16 == 0) && (galign % (grad_dtype == MFSDP_BF16 ? 8 : 16) == 0);
  AdamWArgs a;
  // scalars in double, as Python computes them, then rounded once to fp32
  const double bc1 = 1.0 - std::pow(static_cast<double>(beta1), static_cast<double>(step));
  const double bc2 = 1.0 - std::pow(static_cast<double>(beta2), static_cast<double>(step));
  a.decay = static_cast<float>(1.0 - static_cast<double>(lr) * static_cast<double>(weight_decay));
  a.beta1 = beta1;
  a.one_minus_beta1 = static_cast<float>(1.0 - static_cast<double>(beta1));
  a.beta2 = beta2;
  a.one_minus_beta2 = static_cast<float>(1.0 - static_cast<double>(beta2));
  a.neg_step_size = static_cast<float>(-static_cast<double>(lr) / bc1);
  a.bc2_sqrt = static_cast<float>(std::sqrt(bc2));
  a.eps = eps;
  const int64_t n_vec = vec_ok ? numel / 4 : 0;
  // four vectors per thread with non-temporal accesses (every byte is touched once): 5.7 TB/s against 4.9 TB/s for one
  // cached vector per thread on 41 M elements
  constexpr int kVectorsPerThread = 4;
  const int64_t work = std::max<int64_t>((n_vec + kVectorsPerThread - 1) / kVectorsPerThread, numel - n_vec * 4);
  const int64_t want = std::max<int64_t>(1, (work + 255) / 256);
  const int64_t cap = static_cast<int64_t>(device_cu_count()) * 16;
  const dim3 grid(static_cast<uint32_t>(std::min(want, cap)));
  if (grad_dtype == MFSDP_BF16)
    hipLaunchKernelGGL((adamw_kernel<true, kVectorsPerThread, true>), grid, dim3(256), 0, as_stream(stream), param, grad, exp_avg, exp_avg_sq, n_vec, numel, a);
  else
    hipLaunchKernelGGL((adamw_kernel<false, kVectorsPerThread, true>), grid, dim3(256), 0, as_stream(stream), param, grad, exp_avg, exp_avg_sq, n_vec, numel, a);
  MFSDP_CHECK_LAUNCH("adamw_kernel");
  return MFSDP_OK;
}
