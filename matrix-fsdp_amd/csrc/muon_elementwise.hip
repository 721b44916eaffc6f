// Element-wise stages of the owner-rank Muon update (everything around the Newton-Schulz GEMMs):
//   1. momentum + Nesterov + bf16 rounding + partial sums of squares,
//   2. Frobenius norm (rounded to bf16 and clamped, as the bf16 tensor ops of the reference do),
//   3. division by the norm, written both as X (short side first) and X^T into zero-padded buffers,
//   4. the parameter update  p <- p*(1 - lr*wd) - adjusted_lr * O.
// All are HBM-bound and small next to the GEMMs.
#include "muon_elementwise.h"

#include "mfsdp_common.h"

#include <algorithm>

namespace mfsdp {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float(static_cast<uint32_t>(b) << 16); }

// round to nearest even; inputs here are finite
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  const uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  return static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// Tensor.lerp as ATen evaluates it.
__device__ __forceinline__ float lerp_aten(float start, float end, float weight) {
  // one fused multiply-add from the nearer end point, the form ATen's vectorised kernel spells out
  // (fmadd(weight, end - start, start) / fmadd(weight - 1, end - start, end)); written explicitly so that the
  // compiler's contraction choices cannot differ between code paths
  const float diff = end - start;
  return fabsf(weight) < 0.5f ? __builtin_fmaf(weight, diff, start) : __builtin_fmaf(weight - 1.0f, diff, end);
}

template <typename T>
struct Elem;
template <>
struct Elem<float> {
  static __device__ __forceinline__ float load(const float* p, int64_t i) { return p[i]; }
  static __device__ __forceinline__ void store(float* p, int64_t i, float v) { p[i] = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};
template <>
struct Elem<uint16_t> {  // bf16 storage
  static __device__ __forceinline__ float load(const uint16_t* p, int64_t i) { return bf16_to_f32(p[i]); }
  static __device__ __forceinline__ void store(uint16_t* p, int64_t i, float v) { p[i] = f32_to_bf16(v); }
  static __device__ __forceinline__ float round(float v) { return bf16_to_f32(f32_to_bf16(v)); }
};

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// four consecutive elements at index 4*v (the caller guarantees the alignment)
template <typename T>
struct Quad;
template <>
struct Quad<float> {
  static __device__ __forceinline__ void load(const float* p, int64_t v, float (&out)[4]) {
    const f32x4 q = reinterpret_cast<const f32x4*>(p)[v];
    out[0] = q.x; out[1] = q.y; out[2] = q.z; out[3] = q.w;
  }
  static __device__ __forceinline__ void store(float* p, int64_t v, const float (&in)[4]) {
    const f32x4 q = {in[0], in[1], in[2], in[3]};
    reinterpret_cast<f32x4*>(p)[v] = q;
  }
};
template <>
struct Quad<uint16_t> {
  static __device__ __forceinline__ void load(const uint16_t* p, int64_t v, float (&out)[4]) {
    const u32x2 q = reinterpret_cast<const u32x2*>(p)[v];
    out[0] = __uint_as_float(q.x << 16); out[1] = __uint_as_float(q.x & 0xffff0000u);
    out[2] = __uint_as_float(q.y << 16); out[3] = __uint_as_float(q.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(uint16_t* p, int64_t v, const float (&in)[4]) {
    const u32x2 q = {static_cast<uint32_t>(f32_to_bf16(in[0])) | (static_cast<uint32_t>(f32_to_bf16(in[1])) << 16),
                     static_cast<uint32_t>(f32_to_bf16(in[2])) | (static_cast<uint32_t>(f32_to_bf16(in[3])) << 16)};
    reinterpret_cast<u32x2*>(p)[v] = q;
  }
};

// MOMENTUM: buf <- lerp(buf, g, 1-mu); u = nesterov ? lerp(g, buf, mu) : buf.   !MOMENTUM: u = g.
// xraw <- bf16(u); partials[block] = sum of bf16(u)^2 over the block's elements.
template <typename T, bool MOMENTUM>
__device__ __forceinline__ float momentum_one(float g, float b_old, float momentum, float one_minus_momentum, int nesterov,
                                              float* b_new, uint16_t* xb) {
  float u = g;
  if constexpr (MOMENTUM) {
    const float b = Elem<T>::round(lerp_aten(b_old, g, one_minus_momentum));
    *b_new = b;
    u = nesterov ? Elem<T>::round(lerp_aten(g, b, momentum)) : b;
  }
  *xb = f32_to_bf16(u);
  const float xf = bf16_to_f32(*xb);
  return xf * xf;
}

template <bool NT, typename V>
__device__ __forceinline__ V ld(const V* p) {
  if constexpr (NT) return __builtin_nontemporal_load(p);
  else return *p;
}
template <bool NT, typename V>
__device__ __forceinline__ void st(V* p, V v) {
  if constexpr (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}
template <typename T>
struct QuadOf;
template <>
struct QuadOf<float> { typedef f32x4 type; };
template <>
struct QuadOf<uint16_t> { typedef u32x2 type; };
template <typename T>
__device__ __forceinline__ float quad_elem(const typename QuadOf<T>::type& q, int e) {
  if constexpr (sizeof(T) == 4) return q[e];
  else return __uint_as_float(e & 1 ? (q[e >> 1] & 0xffff0000u) : (q[e >> 1] << 16));
}
template <typename T>
__device__ __forceinline__ typename QuadOf<T>::type quad_pack(const float (&v)[4]) {
  if constexpr (sizeof(T) == 4) {
    return f32x4{v[0], v[1], v[2], v[3]};
  } else {
    return u32x2{static_cast<uint32_t>(f32_to_bf16(v[0])) | (static_cast<uint32_t>(f32_to_bf16(v[1])) << 16),
                 static_cast<uint32_t>(f32_to_bf16(v[2])) | (static_cast<uint32_t>(f32_to_bf16(v[3])) << 16)};
  }
}

constexpr int kMomentumThreads = 64;  // one wavefront per workgroup
constexpr int kMomentumQuads = 2;     // groups of four elements per thread, all of their loads issued before the first use

// n_quads groups of four elements are processed with 128-bit (fp32) / 64-bit (bf16) accesses, the rest one by one.
// One small workgroup per 512 elements rather than a persistent grid (the grid-stride loop only runs when the grid
// is capped): workgroups are dispatched in order, so the ones in flight sweep neighbouring addresses of the four
// streams, and every byte but the bf16 update (read again by the next kernel) is touched once and bypasses the caches.
// 12288 x 4096 fp32: 113-118 us against 147 us for 2048 persistent workgroups of 256 threads.
template <typename T, bool MOMENTUM, bool NTX>
__global__ void __launch_bounds__(kMomentumThreads)
momentum_kernel(const T* __restrict__ grad, T* __restrict__ buf, uint16_t* __restrict__ xraw, float* __restrict__ partials,
                int64_t numel, int64_t n_quads, float momentum, float one_minus_momentum, int nesterov) {
  typedef typename QuadOf<T>::type Q;
  constexpr int U = kMomentumQuads;
  float sumsq = 0.0f;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kMomentumThreads;
  for (int64_t base = static_cast<int64_t>(blockIdx.x) * kMomentumThreads * U + threadIdx.x; base < n_quads; base += stride * U) {
    Q g[U], b[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t v = base + u * kMomentumThreads;
      if (v < n_quads) {
        g[u] = ld<true>(reinterpret_cast<const Q*>(grad) + v);
        if constexpr (MOMENTUM) b[u] = ld<true>(reinterpret_cast<const Q*>(buf) + v);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t v = base + u * kMomentumThreads;
      if (v < n_quads) {
        float bn[4];
        uint16_t xb[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          sumsq += momentum_one<T, MOMENTUM>(quad_elem<T>(g[u], e), MOMENTUM ? quad_elem<T>(b[u], e) : 0.0f, momentum, one_minus_momentum,
                                             nesterov, &bn[e], &xb[e]);
        if constexpr (MOMENTUM) st<true>(reinterpret_cast<Q*>(buf) + v, quad_pack<T>(bn));
        const u32x2 packed = {static_cast<uint32_t>(xb[0]) | (static_cast<uint32_t>(xb[1]) << 16),
                              static_cast<uint32_t>(xb[2]) | (static_cast<uint32_t>(xb[3]) << 16)};
        st<NTX>(reinterpret_cast<u32x2*>(xraw) + v, packed);
      }
    }
  }
  for (int64_t i = n_quads * 4 + static_cast<int64_t>(blockIdx.x) * kMomentumThreads + threadIdx.x; i < numel; i += stride) {
    float bn = 0.0f;
    uint16_t xb;
    sumsq += momentum_one<T, MOMENTUM>(Elem<T>::load(grad, i), MOMENTUM ? Elem<T>::load(buf, i) : 0.0f, momentum, one_minus_momentum,
                                       nesterov, &bn, &xb);
    if constexpr (MOMENTUM) Elem<T>::store(buf, i, bn);
    xraw[i] = xb;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sumsq += __shfl_down(sumsq, off, 64);
  if (threadIdx.x == 0) partials[blockIdx.x] = sumsq;
}

constexpr int kNormThreads = 1024;

// scalars[0] = max(bf16(sqrt(sum partials)), bf16(eps)); one workgroup, the sum in double and in a fixed order
__global__ void __launch_bounds__(kNormThreads)
norm_kernel(const float* __restrict__ partials, int n_partials, float eps, float* __restrict__ scalars) {
  __shared__ double lds[kNormThreads];
  double s = 0.0;
  const int n_vec = n_partials / 4;
  // eight loads in flight per thread: the partial sums come from memory (other XCDs wrote them), one at a time the
  // kernel would wait a memory latency per 16 KiB
  constexpr int kInFlight = 8;
  for (int i0 = threadIdx.x; i0 < n_vec; i0 += kNormThreads * kInFlight) {
    f32x4 v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int i = i0 + u * kNormThreads;
      v[u] = i < n_vec ? reinterpret_cast<const f32x4*>(partials)[i] : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int u = 0; u < kInFlight; ++u)
      s += (static_cast<double>(v[u].x) + static_cast<double>(v[u].y)) + (static_cast<double>(v[u].z) + static_cast<double>(v[u].w));
  }
  for (int i = n_vec * 4 + threadIdx.x; i < n_partials; i += kNormThreads) s += static_cast<double>(partials[i]);
  lds[threadIdx.x] = s;
  __syncthreads();
  for (int off = kNormThreads / 2; off > 0; off >>= 1) {
    if (static_cast<int>(threadIdx.x) < off) lds[threadIdx.x] += lds[threadIdx.x + off];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const float norm = bf16_to_f32(f32_to_bf16(sqrtf(static_cast<float>(lds[0]))));
    const float floor_ = bf16_to_f32(f32_to_bf16(eps));
    scalars[0] = norm > floor_ ? norm : floor_;
  }
}

// 64 x 64 tile of the zero-padded outputs per block:
//   same [r][c]  = bf16(x[r][c] / norm)   (rows_pad x cols_pad, ld = cols_pad)
//   trans[c][r]  = same[r][c]             (cols_pad x rows_pad, ld = rows_pad)
// with x = 0 outside rows x cols.  Every thread handles groups of four consecutive elements: 64-bit stores on
// both outputs (the padded buffers are 256-element aligned); the input is read 64 bits at a time when quads is set.
__global__ void __launch_bounds__(kThreads)
scale_transpose_kernel(const uint16_t* __restrict__ xraw, int rows, int cols, int quads, const float* __restrict__ scalars,
                       uint16_t* __restrict__ same, uint16_t* __restrict__ trans, int rows_pad, int cols_pad) {
  __shared__ uint16_t tile[64][68];
  const float norm = scalars[0];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  for (int e = threadIdx.x; e < 64 * 16; e += kThreads) {
    const int lr = e >> 4, lc = (e & 15) * 4;
    const int r = r0 + lr, c = c0 + lc;
    uint16_t raw[4] = {0, 0, 0, 0};
    if (r < rows) {
      if (quads && c + 3 < cols) {
        const u32x2 q = *reinterpret_cast<const u32x2*>(xraw + static_cast<int64_t>(r) * cols + c);
        raw[0] = static_cast<uint16_t>(q.x); raw[1] = static_cast<uint16_t>(q.x >> 16);
        raw[2] = static_cast<uint16_t>(q.y); raw[3] = static_cast<uint16_t>(q.y >> 16);
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (c + k < cols) raw[k] = xraw[static_cast<int64_t>(r) * cols + c + k];
      }
    }
    uint16_t v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[k] = (r < rows && c + k < cols) ? f32_to_bf16(__fdiv_rn(bf16_to_f32(raw[k]), norm)) : static_cast<uint16_t>(0);
      tile[lr][lc + k] = v[k];
    }
    const u32x2 packed = {static_cast<uint32_t>(v[0]) | (static_cast<uint32_t>(v[1]) << 16),
                          static_cast<uint32_t>(v[2]) | (static_cast<uint32_t>(v[3]) << 16)};
    *reinterpret_cast<u32x2*>(same + static_cast<int64_t>(r) * cols_pad + c) = packed;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 64 * 16; e += kThreads) {
    const int lc = e >> 4, lr = (e & 15) * 4;  // a row of trans = a column of the tile, four rows of the tile at a time
    const u32x2 packed = {static_cast<uint32_t>(tile[lr][lc]) | (static_cast<uint32_t>(tile[lr + 1][lc]) << 16),
                          static_cast<uint32_t>(tile[lr + 2][lc]) | (static_cast<uint32_t>(tile[lr + 3][lc]) << 16)};
    *reinterpret_cast<u32x2*>(trans + static_cast<int64_t>(c0 + lc) * rows_pad + r0 + lr) = packed;
  }
}

// p <- round(round(p * decay) + neg_lr * o) over rows x cols, o read with leading dimension ldo.  col_quads
// groups of four columns per row use vector accesses (the caller guarantees their alignment).
template <typename T>
__global__ void __launch_bounds__(kThreads)
apply_kernel(T* __restrict__ param, const uint16_t* __restrict__ ortho, int rows, int cols, int ldo, int col_quads, float decay,
             float neg_lr) {
  for (int r = blockIdx.y; r < rows; r += gridDim.y) {
    T* prow = param + static_cast<int64_t>(r) * cols;
    const uint16_t* orow = ortho + static_cast<int64_t>(r) * ldo;
    for (int v = blockIdx.x * kThreads + threadIdx.x; v < col_quads; v += gridDim.x * kThreads) {
      float p[4], o[4];
      Quad<T>::load(prow, v, p);
      Quad<uint16_t>::load(orow, v, o);
#pragma unroll
      for (int e = 0; e < 4; ++e) p[e] = Elem<T>::round(p[e] * decay) + neg_lr * o[e];
      Quad<T>::store(prow, v, p);
    }
    for (int c = col_quads * 4 + blockIdx.x * kThreads + threadIdx.x; c < cols; c += gridDim.x * kThreads)
      Elem<T>::store(prow, c, Elem<T>::round(Elem<T>::load(prow, c) * decay) + neg_lr * bf16_to_f32(orow[c]));
  }
}

__global__ void __launch_bounds__(kThreads)
extract_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ ortho, int rows, int cols, int ldo) {
  for (int r = blockIdx.y; r < rows; r += gridDim.y)
    for (int c = blockIdx.x * kThreads + threadIdx.x; c < cols; c += gridDim.x * kThreads)
      out[static_cast<int64_t>(r) * cols + c] = ortho[static_cast<int64_t>(r) * ldo + c];
}

// out <- bf16(scale * in) over n contiguous bf16 (n a multiple of 8, both 16-byte aligned)
__global__ void __launch_bounds__(kThreads)
scale_bf16_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out, int64_t groups, float scale) {
  for (int64_t g = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x; g < groups; g += static_cast<int64_t>(gridDim.x) * kThreads) {
    const u32x4 v = in[g];
    u32x4 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t lo = f32_to_bf16(scale * bf16_to_f32(static_cast<uint16_t>(v[e])));
      const uint32_t hi = f32_to_bf16(scale * bf16_to_f32(static_cast<uint16_t>(v[e] >> 16)));
      r[e] = lo | (hi << 16);
    }
    out[g] = r;
  }
}

int partial_blocks(int64_t numel, int64_t n_quads) {
  // one workgroup per kMomentumQuads * 64 groups of four, or per 64 of the elements left over (everything, when the
  // tensors are not aligned for vector accesses)
  const int64_t work = std::max<int64_t>((n_quads + kMomentumQuads - 1) / kMomentumQuads, numel - n_quads * 4);
  const int64_t want = (work + kMomentumThreads - 1) / kMomentumThreads;
  return static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(want, kMuonMaxPartials)));
}

}  // namespace

int muon_momentum(const void* grad, void* buf, int dtype, int64_t numel, double momentum, int nesterov, bool with_momentum,
                  void* xraw, float* partials, int* n_partials, hipStream_t stream) {
  // the scalars torch hands to lerp_ are the Python doubles 1 - momentum and momentum, rounded to fp32 by the kernel
  const float one_minus = static_cast<float>(1.0 - momentum);
  const float weight = static_cast<float>(momentum);
  auto x = static_cast<uint16_t*>(xraw);
  const uintptr_t need = dtype == MFSDP_F32 ? 16 : 8;  // alignment of a group of four elements
  const bool aligned = reinterpret_cast<uintptr_t>(grad) % need == 0 && (!with_momentum || reinterpret_cast<uintptr_t>(buf) % need == 0) &&
                       reinterpret_cast<uintptr_t>(xraw) % 8 == 0;
  const int64_t n_quads = aligned ? numel / 4 : 0;
  const int blocks = partial_blocks(numel, n_quads);
  *n_partials = blocks;
  // the bf16 update is stored through the caches: the next kernel reads it (non-temporal stores of it, and of the scaled
  // matrices behind it, were measured no faster in the step)
#define MFSDP_MOMENTUM(T_, MOM_)                                                                                                  \
  hipLaunchKernelGGL((momentum_kernel<T_, MOM_, false>), dim3(blocks), dim3(kMomentumThreads), 0, stream, static_cast<const T_*>(grad), \
                     static_cast<T_*>(buf), x, partials, numel, n_quads, weight, one_minus, nesterov)
  if (dtype == MFSDP_F32) {
    if (with_momentum) MFSDP_MOMENTUM(float, true); else MFSDP_MOMENTUM(float, false);
  } else {
    if (with_momentum) MFSDP_MOMENTUM(uint16_t, true); else MFSDP_MOMENTUM(uint16_t, false);
  }
#undef MFSDP_MOMENTUM
  MFSDP_CHECK_LAUNCH("momentum_kernel");
  return MFSDP_OK;
}

int muon_norm(const float* partials, int n_partials, float eps, float* scalars, hipStream_t stream) {
  hipLaunchKernelGGL(norm_kernel, dim3(1), dim3(kNormThreads), 0, stream, partials, n_partials, eps, scalars);
  MFSDP_CHECK_LAUNCH("norm_kernel");
  return MFSDP_OK;
}

int muon_scale_transpose(const void* xraw, int rows, int cols, const float* scalars, void* same, void* trans, int rows_pad,
                         int cols_pad, hipStream_t stream) {
  const dim3 grid(cols_pad / 64, rows_pad / 64);
  const int quads = (cols % 4 == 0 && reinterpret_cast<uintptr_t>(xraw) % 8 == 0) ? 1 : 0;
  hipLaunchKernelGGL(scale_transpose_kernel, grid, dim3(kThreads), 0, stream, static_cast<const uint16_t*>(xraw), rows, cols, quads,
                     scalars, static_cast<uint16_t*>(same), static_cast<uint16_t*>(trans), rows_pad, cols_pad);
  MFSDP_CHECK_LAUNCH("scale_transpose_kernel");
  return MFSDP_OK;
}

int muon_apply(void* param, int dtype, const void* ortho, int rows, int cols, int ldo, float decay, float neg_lr,
               hipStream_t stream) {
  auto o = static_cast<const uint16_t*>(ortho);
  const uintptr_t need = dtype == MFSDP_F32 ? 16 : 8;
  const bool aligned = cols % 4 == 0 && ldo % 4 == 0 && reinterpret_cast<uintptr_t>(param) % need == 0 && reinterpret_cast<uintptr_t>(ortho) % 8 == 0;
  const int col_quads = aligned ? cols / 4 : 0;
  const int per_row = aligned ? col_quads : cols;
  const dim3 grid(std::max(1, std::min((per_row + kThreads - 1) / kThreads, 64)), std::min(rows, 65535));
  if (dtype == MFSDP_F32)
    hipLaunchKernelGGL((apply_kernel<float>), grid, dim3(kThreads), 0, stream, static_cast<float*>(param), o, rows, cols, ldo, col_quads, decay, neg_lr);
  else
    hipLaunchKernelGGL((apply_kernel<uint16_t>), grid, dim3(kThreads), 0, stream, static_cast<uint16_t*>(param), o, rows, cols, ldo, col_quads, decay, neg_lr);
  MFSDP_CHECK_LAUNCH("apply_kernel");
  return MFSDP_OK;
}

int muon_scale_bf16(void* out, const void* in, int64_t numel, float scale, hipStream_t stream) {
  if (numel % 8 || reinterpret_cast<uintptr_t>(out) % 16 || reinterpret_cast<uintptr_t>(in) % 16)
    return fail(MFSDP_ERR_INVALID, "muon_scale_bf16: whole 16-byte groups only");
  const int64_t groups = numel / 8;
  const int blocks = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>((groups + kThreads - 1) / kThreads, 65535)));
  hipLaunchKernelGGL(scale_bf16_kernel, dim3(blocks), dim3(kThreads), 0, stream, static_cast<const u32x4*>(in), static_cast<u32x4*>(out), groups, scale);
  MFSDP_CHECK_LAUNCH("scale_bf16_kernel");
  return MFSDP_OK;
}

int muon_extract(void* out, const void* ortho, int rows, int cols, int ldo, hipStream_t stream) {
  const dim3 grid(std::max(1, std::min((cols + kThreads - 1) / kThreads, 64)), std::min(rows, 65535));
  hipLaunchKernelGGL(extract_kernel, grid, dim3(kThreads), 0, stream, static_cast<uint16_t*>(out),
                     static_cast<const uint16_t*>(ortho), rows, cols, ldo);
  MFSDP_CHECK_LAUNCH("extract_kernel");
  return MFSDP_OK;
}

}  // namespace mfsdp
