// bf16 MFMA GEMM for the Newton-Schulz iteration: C = bf16(alpha * P Q^T + beta * D) on gfx950.
//
// Both operands are K-contiguous (an "NT" product), which is what every Newton-Schulz product
// reduces to once X and X^T are both kept: X X^T, A A^T (A symmetric) and B (X^T)^T.  A workgroup owns
// a BM x BN tile of C; its waves each own a (BM/WM) x (BN/WN) sub-tile built from 32x32x16 bf16 MFMAs
// with fp32 accumulators.  K is walked in slabs of 64: the slab of P and Q is staged in LDS as rows of
// 128 bytes whose eight 16-byte chunks are XOR-swizzled with the row index, so that the 128-bit
// fragment reads of 32 consecutive rows are bank-conflict free.  Two LDS stages: the next slab is
// fetched from HBM into registers while the current one feeds the MFMAs.
#include "muon_gemm.h"

#include "mfsdp_common.h"

namespace mfsdp {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kBK = 64;            // K slab, bf16 elements (128 bytes per row)
constexpr int kChunksPerRow = 8;   // 16-byte chunks per slab row
constexpr int kXcds = 8;

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const __bf16 l = static_cast<__bf16>(lo);
  const __bf16 h = static_cast<__bf16>(hi);
  return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, l)) | (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, h)) << 16);
}

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) { return __uint_as_float(static_cast<uint32_t>(b) << 16); }

// Maps the hardware block id to a tile so that (a) the blocks that land on one XCD (ids congruent
// mod 8) work on a contiguous range of logical tiles and share that XCD's L2, and (b) consecutive
// logical tiles walk down GROUP_M tile rows before moving to the next tile column.
template <int GROUP_M>
__device__ __forceinline__ void tile_of_block(int block, int n_blocks, int tiles_m, int tiles_n, bool symmetric,
                                              int* tm, int* tn) {
  int logical = block;
  if (n_blocks % kXcds == 0) logical = (block % kXcds) * (n_blocks / kXcds) + block / kXcds;
  if (symmetric) {
    // logical enumerates the lower triangle row by row: t = i(i+1)/2 + j, j <= i
    int i = static_cast<int>((__fsqrt_rn(8.0f * static_cast<float>(logical) + 1.0f) - 1.0f) * 0.5f);
    while ((i + 1) * (i + 2) / 2 <= logical) ++i;
    while (i * (i + 1) / 2 > logical) --i;
    *tm = i;
    *tn = logical - i * (i + 1) / 2;
    return;
  }
  const int per_group = GROUP_M * tiles_n;
  const int group = logical / per_group;
  const int first_m = group * GROUP_M;
  const int rows = min(GROUP_M, tiles_m - first_m);
  const int in_group = logical - group * per_group;
  *tm = first_m + in_group % rows;
  *tn = in_group / rows;
}

template <int BM, int BN, int WM, int WN>
__global__ void __launch_bounds__(WM * WN * 64)
gemm_nt_kernel(GemmNtArgs a, int tiles_m, int tiles_n) {
  constexpr int kThreads = WM * WN * 64;
  constexpr int kWaveM = BM / WM;     // rows of C per wave
  constexpr int kWaveN = BN / WN;
  constexpr int TM = kWaveM / 32;     // 32x32 MFMA tiles per wave
  constexpr int TN = kWaveN / 32;
  constexpr int kPChunks = BM * kChunksPerRow / kThreads;  // 16-byte chunks of the P slab per thread
  constexpr int kQChunks = BN * kChunksPerRow / kThreads;
  static_assert(BM * kChunksPerRow % kThreads == 0 && BN * kChunksPerRow % kThreads == 0, "slab must divide over threads");
  constexpr int kStageElems = (BM + BN) * kBK;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __bf16* smem = reinterpret_cast<__bf16*>(smem_raw);

  int tm, tn;
  tile_of_block<4>(blockIdx.x, gridDim.x, tiles_m, tiles_n, a.symmetric != 0, &tm, &tn);
  const int row0 = tm * BM;
  const int col0 = tn * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave / WN;
  const int wave_n = wave % WN;

  const __bf16* __restrict__ P = static_cast<const __bf16*>(a.P) + static_cast<int64_t>(row0) * a.ldp;
  const __bf16* __restrict__ Q = static_cast<const __bf16*>(a.Q) + static_cast<int64_t>(col0) * a.ldq;

  // slab chunk c = i * kThreads + tid  ->  row c / 8, 16-byte chunk c % 8
  u32x4 pre_p[kPChunks], pre_q[kQChunks];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < kPChunks; ++i) {
      const int c = i * kThreads + tid;
      pre_p[i] = *reinterpret_cast<const u32x4*>(P + static_cast<int64_t>(c >> 3) * a.ldp + k0 + (c & 7) * 8);
    }
#pragma unroll
    for (int i = 0; i < kQChunks; ++i) {
      const int c = i * kThreads + tid;
      pre_q[i] = *reinterpret_cast<const u32x4*>(Q + static_cast<int64_t>(c >> 3) * a.ldq + k0 + (c & 7) * 8);
    }
  };
  auto stash = [&](int stage) {
    __bf16* sp = smem + stage * kStageElems;
    __bf16* sq = sp + BM * kBK;
#pragma unroll
    for (int i = 0; i < kPChunks; ++i) {
      const int c = i * kThreads + tid;
      const int r = c >> 3;
      *reinterpret_cast<u32x4*>(sp + r * kBK + (((c & 7) ^ (r & 7)) << 3)) = pre_p[i];
    }
#pragma unroll
    for (int i = 0; i < kQChunks; ++i) {
      const int c = i * kThreads + tid;
      const int r = c >> 3;
      *reinterpret_cast<u32x4*>(sq + r * kBK + (((c & 7) ^ (r & 7)) << 3)) = pre_q[i];
    }
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int frag_row = lane & 31;   // row of the 32-row MFMA operand this lane supplies
  const int frag_half = lane >> 5;  // which 8 of the 16 k values

  const int k_slabs = a.K / kBK;
  fetch(0);
  stash(0);
  __syncthreads();
  for (int ks = 0; ks < k_slabs; ++ks) {
    const int stage = ks & 1;
    if (ks + 1 < k_slabs) fetch((ks + 1) * kBK);
    const __bf16* sp = smem + stage * kStageElems + (wave_m * kWaveM) * kBK;
    const __bf16* sq = smem + stage * kStageElems + BM * kBK + (wave_n * kWaveN) * kBK;
#pragma unroll
    for (int kk = 0; kk < kBK / 16; ++kk) {
      const int chunk = kk * 2 + frag_half;
      bf16x8 fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int r = i * 32 + frag_row;
        fa[i] = *reinterpret_cast<const bf16x8*>(sp + r * kBK + ((chunk ^ (r & 7)) << 3));
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int r = j * 32 + frag_row;
        fb[j] = *reinterpret_cast<const bf16x8*>(sq + r * kBK + ((chunk ^ (r & 7)) << 3));
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (ks + 1 < k_slabs) stash(stage ^ 1);
    __syncthreads();
  }

  // Epilogue.  Accumulator register r of lane l holds C[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32x32 tile.
  const uint16_t* __restrict__ D = static_cast<const uint16_t*>(a.D);
  uint16_t* __restrict__ C = static_cast<uint16_t*>(a.C);
  uint16_t* __restrict__ CT = static_cast<uint16_t*>(a.CT);
  int ldct = a.ldct;
  if (a.symmetric && tm != tn) {  // mirror the off-diagonal tile
    CT = C;
    ldct = a.ldc;
  } else if (a.symmetric) {
    CT = nullptr;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = col0 + wave_n * kWaveN + j * 32 + (lane & 31);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = row0 + wave_m * kWaveM + i * 32 + q * 8 + frag_half * 4;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = a.alpha * acc[i][j][q * 4 + e];
          if (D != nullptr) v[e] += a.beta * bf16_bits_to_float(D[static_cast<int64_t>(row + e) * a.ldd + col]);
        }
        const uint32_t lo = pack_bf16x2(v[0], v[1]);
        const uint32_t hi = pack_bf16x2(v[2], v[3]);
        C[static_cast<int64_t>(row) * a.ldc + col] = static_cast<uint16_t>(lo);
        C[static_cast<int64_t>(row + 1) * a.ldc + col] = static_cast<uint16_t>(lo >> 16);
        C[static_cast<int64_t>(row + 2) * a.ldc + col] = static_cast<uint16_t>(hi);
        C[static_cast<int64_t>(row + 3) * a.ldc + col] = static_cast<uint16_t>(hi >> 16);
        if (CT != nullptr) {
          u32x2 packed = {lo, hi};
          *reinterpret_cast<u32x2*>(CT + static_cast<int64_t>(col) * ldct + row) = packed;
        }
      }
    }
  }
}

int g_variant = 0;

template <int BM, int BN, int WM, int WN>
int launch(const GemmNtArgs& a, hipStream_t stream) {
  const int tiles_m = a.M / BM, tiles_n = a.N / BN;
  const int blocks = a.symmetric ? tiles_m * (tiles_m + 1) / 2 : tiles_m * tiles_n;
  constexpr size_t smem = 2 * static_cast<size_t>(BM + BN) * kBK * sizeof(uint16_t);
  auto kernel = gemm_nt_kernel<BM, BN, WM, WN>;
  static bool configured = false;  // raising the dynamic LDS limit is needed once per kernel
  if (!configured) {
    MFSDP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(smem)));
    configured = true;
  }
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(WM * WN * 64), smem, stream, a, tiles_m, tiles_n);
  MFSDP_CHECK_LAUNCH("gemm_nt_kernel");
  return MFSDP_OK;
}

}  // namespace

void set_gemm_variant(int variant) { g_variant = variant; }

int gemm_nt_bf16(const GemmNtArgs& a, hipStream_t stream) {
  if (a.M <= 0 || a.N <= 0 || a.K <= 0 || a.M % 256 || a.N % 256 || a.K % kBK)
    return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: M=%d N=%d must be multiples of 256 and K=%d of %d", a.M, a.N, a.K, kBK);
  if (a.symmetric && a.M != a.N) return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: symmetric product needs M == N");
  if (!a.P || !a.Q || !a.C) return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: null operand");
  if (a.ldp < a.K || a.ldq < a.K || a.ldc < a.N || (a.D && a.ldd < a.N) || (a.CT && a.ldct < a.M))
    return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: leading dimension smaller than the row length");
  if ((a.ldp | a.ldq) % 8 || (reinterpret_cast<uintptr_t>(a.P) | reinterpret_cast<uintptr_t>(a.Q)) % 16)
    return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: operands must be 16-byte aligned with leading dimensions multiple of 8");
  if (a.CT && ((a.ldct % 4) || reinterpret_cast<uintptr_t>(a.CT) % 8))
    return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: transposed output must be 8-byte aligned");
  if (a.symmetric && ((a.ldc % 4) || reinterpret_cast<uintptr_t>(a.C) % 8))
    return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: symmetric output must be 8-byte aligned");
  int variant = g_variant;
  if (variant == 0) variant = a.symmetric ? 2 : 1;
  if (variant == 2) return launch<128, 128, 2, 2>(a, stream);
  return launch<256, 256, 2, 4>(a, stream);
}

}  // namespace mfsdp
