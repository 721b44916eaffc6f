// Segment programs: one persistent, bandwidth-bound gfx950 kernel that replays a
// whole shard layout's copy (every rank, every segment, pad zero-fill, optional
// bf16<->fp32 conversion) in a single launch.
//
// Work is cut by BYTES, not by segment: every run is divided into tiles of
// 64*U vector groups and each wavefront walks the tile table with a grid
// stride.  Within a tile lane l moves groups l, l+64, ... so every wave-level
// load / store touches one contiguous 1 KiB span (16 B per lane) whenever a
// tile lies inside a row; U independent 128-bit loads are in flight per lane
// before the first store.  Strided 2-D runs (block shards) find their row with
// a multiply-high by a host-computed reciprocal instead of a division.
#include "mfsdp_common.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

namespace mfsdp {
namespace {

constexpr int kMaxSources = 128;  // pointer table passed by value in the kernel arguments
constexpr int kWaveSize = 64;
constexpr int kBlockThreads = 256;
constexpr int64_t kMaxGrid = (int64_t{1} << 31) - 1;  // grid-stride loops keep a capped grid correct
constexpr int kWavesPerBlock = kBlockThreads / kWaveSize;
constexpr uint32_t kMaxGroupsPerRun = 0x7fffffffu;  // reciprocal division is exact below 2^31

struct SourceTable {
  const char* p[kMaxSources];
};

// One run in units of vector groups (device copy).
struct DevRun {
  int64_t src_off;
  int64_t dst_off;
  int64_t src_stride;
  int64_t dst_stride;
  uint32_t row_groups;
  uint32_t n_groups;
  uint32_t magic;  // row = umulhi(magic, g) >> shift   (unused when rows == 1 or row_groups == 1)
  uint32_t shift;
  int32_t src_id;
  uint32_t multi_row;
};

struct DevTile {
  uint32_t run;
  uint32_t tile;  // first group = tile * 64 * U
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int NB>
struct Words {
  uint32_t w[(NB + 3) / 4];
};

template <int NB, bool NT>
__device__ __forceinline__ Words<NB> load_bytes(const char* p) {
  Words<NB> r;
  if constexpr (NB == 32) {
    u32x4 a, b;
    if constexpr (NT) {
      a = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
      b = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p) + 1);
    } else {
      a = *reinterpret_cast<const u32x4*>(p);
      b = *(reinterpret_cast<const u32x4*>(p) + 1);
    }
    r.w[0] = a.x; r.w[1] = a.y; r.w[2] = a.z; r.w[3] = a.w;
    r.w[4] = b.x; r.w[5] = b.y; r.w[6] = b.z; r.w[7] = b.w;
  } else if constexpr (NB == 16) {
    u32x4 a;
    if constexpr (NT) a = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    else a = *reinterpret_cast<const u32x4*>(p);
    r.w[0] = a.x; r.w[1] = a.y; r.w[2] = a.z; r.w[3] = a.w;
  } else if constexpr (NB == 8) {
    u32x2 a;
    if constexpr (NT) a = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    else a = *reinterpret_cast<const u32x2*>(p);
    r.w[0] = a.x; r.w[1] = a.y;
  } else if constexpr (NB == 4) {
    if constexpr (NT) r.w[0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p));
    else r.w[0] = *reinterpret_cast<const uint32_t*>(p);
  } else if constexpr (NB == 2) {
    r.w[0] = *reinterpret_cast<const uint16_t*>(p);
  } else {
    r.w[0] = *reinterpret_cast<const uint8_t*>(p);
  }
  return r;
}

template <int NB, bool NT>
__device__ __forceinline__ void store_bytes(char* p, const Words<NB>& v) {
  if constexpr (NB == 32) {
    u32x4 a = {v.w[0], v.w[1], v.w[2], v.w[3]};
    u32x4 b = {v.w[4], v.w[5], v.w[6], v.w[7]};
    if constexpr (NT) {
      __builtin_nontemporal_store(a, reinterpret_cast<u32x4*>(p));
      __builtin_nontemporal_store(b, reinterpret_cast<u32x4*>(p) + 1);
    } else {
      *reinterpret_cast<u32x4*>(p) = a;
      *(reinterpret_cast<u32x4*>(p) + 1) = b;
    }
  } else if constexpr (NB == 16) {
    u32x4 a = {v.w[0], v.w[1], v.w[2], v.w[3]};
    if constexpr (NT) __builtin_nontemporal_store(a, reinterpret_cast<u32x4*>(p));
    else *reinterpret_cast<u32x4*>(p) = a;
  } else if constexpr (NB == 8) {
    u32x2 a = {v.w[0], v.w[1]};
    if constexpr (NT) __builtin_nontemporal_store(a, reinterpret_cast<u32x2*>(p));
    else *reinterpret_cast<u32x2*>(p) = a;
  } else if constexpr (NB == 4) {
    if constexpr (NT) __builtin_nontemporal_store(v.w[0], reinterpret_cast<uint32_t*>(p));
    else *reinterpret_cast<uint32_t*>(p) = v.w[0];
  } else if constexpr (NB == 2) {
    *reinterpret_cast<uint16_t*>(p) = static_cast<uint16_t>(v.w[0]);
  } else {
    *reinterpret_cast<uint8_t*>(p) = static_cast<uint8_t>(v.w[0]);
  }
}

// fp32 bits -> bf16 bits, round to nearest even; every NaN becomes the quiet
// NaN 0x7FC0.  This is the rounding Tensor.to(torch.bfloat16) performs.
__device__ __forceinline__ uint32_t f32_bits_to_bf16_bits(uint32_t u) {
  const uint32_t rounded = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  return ((u & 0x7fffffffu) > 0x7f800000u) ? 0x7fc0u : rounded;
}

// fp16 <-> fp32 through the hardware conversions: widening is exact (fp16 denormals included), narrowing rounds to
// nearest even (overflow to infinity, underflow through the fp16 denormals to zero); every NaN becomes the quiet NaN
// 0x7E00 with its sign kept.
__device__ __forceinline__ uint32_t f16_bits_to_f32_bits(uint32_t h) {
  return __float_as_uint(static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(h))));
}
__device__ __forceinline__ uint32_t f32_bits_to_f16_bits(uint32_t u) {
  if ((u & 0x7fffffffu) > 0x7f800000u) return ((u >> 16) & 0x8000u) | 0x7e00u;
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(__uint_as_float(u)));
}

// SRC_B bytes in, DST_B bytes out.  Equal sizes: raw move.  DST_B = 2*SRC_B: bf16 (HALF: fp16) -> fp32.
// SRC_B = 2*DST_B: fp32 -> bf16 (HALF: fp16).
template <int SRC_B, int DST_B, bool HALF = false>
__device__ __forceinline__ Words<DST_B> convert_group(const Words<SRC_B>& in) {
  Words<DST_B> out;
  if constexpr (SRC_B == DST_B) {
#pragma unroll
    for (int i = 0; i < (DST_B + 3) / 4; ++i) out.w[i] = in.w[i];
  } else if constexpr (DST_B == 2 * SRC_B) {
    constexpr int n = SRC_B / 2;  // elements
#pragma unroll
    for (int i = 0; i < n; ++i) {
      const uint32_t word = in.w[i / 2];
      if constexpr (HALF) out.w[i] = f16_bits_to_f32_bits((i & 1) ? (word >> 16) : (word & 0xffffu));
      else out.w[i] = (i & 1) ? (word & 0xffff0000u) : (word << 16);
    }
  } else {
    constexpr int n = DST_B / 2;
#pragma unroll
    for (int i = 0; i < (DST_B + 3) / 4; ++i) out.w[i] = 0;
#pragma unroll
    for (int i = 0; i < n; ++i) out.w[i / 2] |= (HALF ? f32_bits_to_f16_bits(in.w[i]) : f32_bits_to_bf16_bits(in.w[i])) << (16 * (i & 1));
  }
  return out;
}

template <int SRC_B, int DST_B, int U, bool NT, bool NTS = NT, bool HALF = false>
__global__ void __launch_bounds__(kBlockThreads)
segment_program_kernel(SourceTable srcs, char* __restrict__ dst, const DevRun* __restrict__ runs,
                       const DevTile* __restrict__ tiles, uint32_t n_tiles) {
  const uint32_t lane = threadIdx.x & (kWaveSize - 1);
  const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6));
  const uint32_t n_waves = gridDim.x * kWavesPerBlock;
  for (uint32_t t = wave; t < n_tiles; t += n_waves) {
    const DevTile tile = tiles[t];
    const DevRun run = runs[tile.run];
    const uint32_t first = tile.tile * (kWaveSize * U);
    const char* sbase = run.src_id >= 0 ? srcs.p[run.src_id] : nullptr;
    Words<SRC_B> data[U];
    int64_t doff[U];
    bool live[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t g = first + u * kWaveSize + lane;
      live[u] = g < run.n_groups;
      uint32_t row = 0, col = g;
      if (run.multi_row) {
        row = run.row_groups == 1 ? g : (__umulhi(run.magic, g) >> run.shift);
        col = g - row * run.row_groups;
      }
      doff[u] = run.dst_off + static_cast<int64_t>(row) * run.dst_stride + col;
      if (live[u] && sbase != nullptr) {
        const int64_t soff = run.src_off + static_cast<int64_t>(row) * run.src_stride + col;
        data[u] = load_bytes<SRC_B, NT>(sbase + soff * SRC_B);
      } else {
#pragma unroll
        for (int i = 0; i < (SRC_B + 3) / 4; ++i) data[u].w[i] = 0;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (live[u]) store_bytes<DST_B, NTS>(dst + doff[u] * DST_B, convert_group<SRC_B, DST_B, HALF>(data[u]));
    }
  }
}

struct Tuning {
  int blocks_per_cu = 2;        // persistent grid of the segment kernel: 2 workgroups (8 waves) per CU measured best
  int nontemporal = 1;
  int unroll = 4;
  // elements per lane when converting: 4 keeps the wider side at one 16-byte access per lane, so that every wave-level
  // access is one contiguous span (8 elements would make the 32-byte side two half-dense accesses: 51 % vs 67 % of HBM peak)
  int convert_group = 4;
};
Tuning g_tuning;

bool is_half_conversion(int convert) { return convert == MFSDP_CONVERT_F16_TO_F32 || convert == MFSDP_CONVERT_F32_TO_F16; }

// ---- host side -------------------------------------------------------------------------------

struct Compiled {  // tables for one vector width
  int group_units = 0;  // G
  DevRun* runs = nullptr;
  DevTile* tiles = nullptr;
  uint32_t n_tiles = 0;
  int unroll = 0;
};

// floor(g / d) for g < 2^31 as umulhi(magic, g) >> shift  (round-up reciprocal, d >= 2).
void reciprocal(uint32_t d, uint32_t* magic, uint32_t* shift) {
  uint32_t l = 0;
  while ((1ull << l) < d) ++l;  // l = ceil(log2 d) >= 1
  const unsigned __int128 num = static_cast<unsigned __int128>(1) << (31 + l);
  *magic = static_cast<uint32_t>(num / d + 1);
  *shift = l - 1;
}

int64_t gcd_pow2(int64_t v, int64_t cap) {  // largest power of two <= cap dividing v (v == 0 -> cap)
  int64_t g = cap;
  while (g > 1 && (v % g) != 0) g >>= 1;
  return g;
}

}  // namespace
}  // namespace mfsdp

using namespace mfsdp;

struct mfsdp_segment_program {
  std::vector<mfsdp_copy_run> runs;  // validated, rows>=1, row_len>=1
  std::vector<int64_t> src_numels;
  int64_t dst_numel = 0;
  int convert = 0;
  int src_unit = 1;  // bytes per unit on the source side
  int dst_unit = 1;
  int max_group = 16;  // widest vector group in units
  int64_t bytes_moved = 0;
  int device = 0;
  std::mutex mu;
  std::map<int, std::vector<Compiled>> variants;  // pointer alignment cap (units) -> one Compiled per group width in use
};

namespace {

void free_compiled(std::vector<Compiled>& v) {
  for (auto& c : v) {
    if (c.runs) (void)hipFree(c.runs);
    if (c.tiles) (void)hipFree(c.tiles);
  }
  v.clear();
}

// Builds the device tables for pointer-alignment cap `cap` (in units).
int compile_variant(mfsdp_segment_program* prog, int cap, std::vector<Compiled>* out) {
  const int unroll = g_tuning.unroll == 8 ? 8 : 4;
  std::map<int, std::pair<std::vector<DevRun>, std::vector<DevTile>>> by_group;
  for (const auto& r : prog->runs) {
    int64_t g = std::min<int64_t>(cap, prog->max_group);
    g = gcd_pow2(r.row_len, g);
    g = gcd_pow2(r.dst_off, g);
    if (r.src_id >= 0) g = gcd_pow2(r.src_off, g);
    if (r.rows > 1) {
      g = gcd_pow2(r.dst_stride, g);
      if (r.src_id >= 0) g = gcd_pow2(r.src_stride, g);
    }
    auto& bucket = by_group[static_cast<int>(g)];
    const int64_t row_groups = r.row_len / g;
    // split so that every device run holds fewer than 2^31 groups
    int64_t rows_per_part = r.rows;
    int64_t len_parts = 1;
    if (row_groups > kMaxGroupsPerRun) {
      rows_per_part = 1;
      len_parts = (row_groups + kMaxGroupsPerRun - 1) / kMaxGroupsPerRun;
    } else if (row_groups * r.rows > kMaxGroupsPerRun) {
      rows_per_part = kMaxGroupsPerRun / row_groups;
    }
    for (int64_t row0 = 0; row0 < r.rows; row0 += rows_per_part) {
      const int64_t nrows = std::min(rows_per_part, r.rows - row0);
      for (int64_t part = 0; part < len_parts; ++part) {
        const int64_t col0 = part * static_cast<int64_t>(kMaxGroupsPerRun);
        const int64_t ncols = std::min<int64_t>(kMaxGroupsPerRun, row_groups - col0);
        DevRun d{};
        d.src_off = (r.src_id >= 0 ? (r.src_off + row0 * r.src_stride) / g : 0) + col0;
        d.dst_off = (r.dst_off + row0 * r.dst_stride) / g + col0;
        d.src_stride = nrows > 1 && r.src_id >= 0 ? r.src_stride / g : 0;
        d.dst_stride = nrows > 1 ? r.dst_stride / g : 0;
        d.row_groups = static_cast<uint32_t>(ncols);
        d.n_groups = static_cast<uint32_t>(ncols * nrows);
        d.multi_row = nrows > 1 ? 1u : 0u;
        d.src_id = r.src_id;
        d.magic = 0;
        d.shift = 0;
        if (d.multi_row && d.row_groups > 1) reciprocal(d.row_groups, &d.magic, &d.shift);
        const uint32_t run_index = static_cast<uint32_t>(bucket.first.size());
        bucket.first.push_back(d);
        const uint32_t tile_groups = kWaveSize * unroll;
        const uint32_t ntiles = (d.n_groups + tile_groups - 1) / tile_groups;
        for (uint32_t t = 0; t < ntiles; ++t) bucket.second.push_back(DevTile{run_index, t});
      }
    }
  }
  for (auto& kv : by_group) {
    Compiled c;
    c.group_units = kv.first;
    c.unroll = unroll;
    auto& runs = kv.second.first;
    auto& tiles = kv.second.second;
    if (tiles.size() > 0xffffffffull) {
      free_compiled(*out);
      return fail(MFSDP_ERR_UNSUPPORTED, "segment program needs %zu tiles, more than one launch can address", tiles.size());
    }
    c.n_tiles = static_cast<uint32_t>(tiles.size());
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&c.runs), runs.size() * sizeof(DevRun));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&c.tiles), tiles.size() * sizeof(DevTile));
    if (e == hipSuccess) e = hipMemcpy(c.runs, runs.data(), runs.size() * sizeof(DevRun), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(c.tiles, tiles.data(), tiles.size() * sizeof(DevTile), hipMemcpyHostToDevice);
    out->push_back(c);
    if (e != hipSuccess) {
      free_compiled(*out);
      return fail(MFSDP_ERR_HIP, "uploading segment program tables failed: %s", hipGetErrorString(e));
    }
  }
  return MFSDP_OK;
}

template <int SRC_B, int DST_B, bool HALF = false>
int launch_one(const Compiled& c, const SourceTable& srcs, char* dst, hipStream_t stream) {
  const int cus = device_cu_count();
  const uint32_t want = (c.n_tiles + kWavesPerBlock - 1) / kWavesPerBlock;
  // widening programs (bf16 -> fp32 copy-in) write twice what they read and like more workgroups in flight:
  // 5.55 TB/s with 32 per CU against 5.38 with 2 on the hidden2048 gradient fill; plain copies are best at 2
  const int per_cu = DST_B > SRC_B ? std::max(32, g_tuning.blocks_per_cu) : std::max(1, g_tuning.blocks_per_cu);
  const uint32_t cap = static_cast<uint32_t>(cus) * static_cast<uint32_t>(per_cu);
  const dim3 grid(std::max(1u, std::min(want, cap)));
  const dim3 block(kBlockThreads);
  const int nt = g_tuning.nontemporal;  // 0 none, 1 loads and stores, 2 loads only, 3 stores only
#define MFSDP_LAUNCH(U_, NTL_, NTS_)                                                                             \
  hipLaunchKernelGGL((segment_program_kernel<SRC_B, DST_B, U_, NTL_, NTS_, HALF>), grid, block, 0, stream, srcs, dst, \
                     c.runs, c.tiles, c.n_tiles)
#define MFSDP_LAUNCH_NT(U_)                      \
  switch (nt) {                                  \
    case 0: MFSDP_LAUNCH(U_, false, false); break; \
    case 2: MFSDP_LAUNCH(U_, true, false); break;  \
    case 3: MFSDP_LAUNCH(U_, false, true); break;  \
    default: MFSDP_LAUNCH(U_, true, true); break;  \
  }
  if (c.unroll == 8) { MFSDP_LAUNCH_NT(8) } else { MFSDP_LAUNCH_NT(4) }
#undef MFSDP_LAUNCH_NT
#undef MFSDP_LAUNCH
  MFSDP_CHECK_LAUNCH("segment_program_kernel");
  return MFSDP_OK;
}

int launch_compiled(const mfsdp_segment_program* prog, const Compiled& c, const SourceTable& srcs, char* dst,
                    hipStream_t stream) {
  if (c.n_tiles == 0) return MFSDP_OK;
  const int sb = c.group_units * prog->src_unit;
  const int db = c.group_units * prog->dst_unit;
#define MFSDP_CASE(S_, D_) \
  if (sb == S_ && db == D_) return launch_one<S_, D_>(c, srcs, dst, stream)
#define MFSDP_CONVERTING(S_, D_) \
  if (sb == S_ && db == D_) return half ? launch_one<S_, D_, true>(c, srcs, dst, stream) : launch_one<S_, D_, false>(c, srcs, dst, stream)
  const bool half = is_half_conversion(prog->convert);
  MFSDP_CASE(16, 16); MFSDP_CASE(8, 8); MFSDP_CASE(4, 4); MFSDP_CASE(2, 2); MFSDP_CASE(1, 1);
  MFSDP_CONVERTING(16, 32); MFSDP_CONVERTING(8, 16); MFSDP_CONVERTING(4, 8); MFSDP_CONVERTING(2, 4);
  MFSDP_CONVERTING(32, 16); MFSDP_CONVERTING(16, 8); MFSDP_CONVERTING(8, 4); MFSDP_CONVERTING(4, 2);
#undef MFSDP_CONVERTING
#undef MFSDP_CASE
  return fail(MFSDP_ERR_UNSUPPORTED, "no kernel for %d -> %d byte groups", sb, db);
}

int pointer_alignment_units(const void* p, int unit_bytes, int max_group) {
  // largest power-of-two group (in units) whose byte size (capped at 16) divides the address
  int g = max_group;
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  while (g > 1 && (a % static_cast<uintptr_t>(std::min(g * unit_bytes, 16))) != 0) g >>= 1;
  return g;
}

int setup_units(int convert, int elem_bytes, int* src_unit, int* dst_unit, int* max_group, int* scale) {
  switch (convert) {
    case MFSDP_CONVERT_NONE:
      if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8)
        return fail(MFSDP_ERR_INVALID, "elem_bytes must be 1, 2, 4 or 8, got %d", elem_bytes);
      *src_unit = 1; *dst_unit = 1; *max_group = 16; *scale = elem_bytes;  // units are bytes
      return MFSDP_OK;
    case MFSDP_CONVERT_BF16_TO_F32:
    case MFSDP_CONVERT_F16_TO_F32:
      *src_unit = 2; *dst_unit = 4; *max_group = g_tuning.convert_group; *scale = 1;
      return MFSDP_OK;
    case MFSDP_CONVERT_F32_TO_BF16:
    case MFSDP_CONVERT_F32_TO_F16:
      *src_unit = 4; *dst_unit = 2; *max_group = g_tuning.convert_group; *scale = 1;
      return MFSDP_OK;
    default:
      return fail(MFSDP_ERR_INVALID, "unknown conversion code %d", convert);
  }
}

}  // namespace

extern "C" void mfsdp_set_copy_tuning(int blocks_per_cu, int nontemporal, int unroll) {
  g_tuning.blocks_per_cu = blocks_per_cu > 0 ? blocks_per_cu : 2;
  g_tuning.nontemporal = (nontemporal < 0 || nontemporal > 3) ? 1 : nontemporal;
  g_tuning.unroll = unroll == 8 ? 8 : 4;
}

extern "C" int64_t mfsdp_merge_segment_runs(const mfsdp_copy_run* segs, int64_t n_segs, mfsdp_copy_run* out) {
  int64_t n_out = 0;
  for (int64_t i = 0; i < n_segs; ++i) {
    mfsdp_copy_run s = segs[i];
    if (s.rows <= 0 || s.row_len <= 0) continue;
    if (s.src_id < 0) s.src_id = -1;
    if (s.rows == 1) s.src_stride = s.dst_stride = 0;
    if (n_out > 0 && s.rows == 1 && out[n_out - 1].src_id == s.src_id) {
      mfsdp_copy_run& cur = out[n_out - 1];
      const bool fill = s.src_id < 0;
      const int64_t dst_step = s.dst_off - cur.dst_off;
      const int64_t src_step = fill ? 0 : s.src_off - cur.src_off;
      if (cur.rows == 1) {
        if (dst_step == cur.row_len && (fill || src_step == cur.row_len)) {
          cur.row_len += s.row_len;  // back to back on both sides: one longer segment
          continue;
        }
        if (s.row_len == cur.row_len && dst_step >= cur.row_len && (fill || src_step > 0)) {
          cur.rows = 2;  // equal lengths at a constant pitch: start a 2-D run
          cur.dst_stride = dst_step;
          cur.src_stride = src_step;
          continue;
        }
      } else if (s.row_len == cur.row_len && dst_step == cur.rows * cur.dst_stride &&
                 (fill || src_step == cur.rows * cur.src_stride)) {
        cur.rows += 1;
        continue;
      }
    }
    out[n_out++] = s;
  }
  return n_out;
}

extern "C" int mfsdp_segment_program_create(const mfsdp_copy_run* runs, int64_t n_runs, const int64_t* src_numels,
                                            int32_t n_srcs, int64_t dst_numel, int convert, int elem_bytes,
                                            mfsdp_segment_program** out) {
  if (out == nullptr) return fail(MFSDP_ERR_INVALID, "out is null");
  *out = nullptr;
  if (n_runs < 0 || (n_runs > 0 && runs == nullptr)) return fail(MFSDP_ERR_INVALID, "runs is null or n_runs negative");
  if (n_srcs < 0 || n_srcs > kMaxSources)
    return fail(MFSDP_ERR_INVALID, "n_srcs must be in [0, %d], got %d", kMaxSources, n_srcs);
  if (n_srcs > 0 && src_numels == nullptr) return fail(MFSDP_ERR_INVALID, "src_numels is null");
  if (dst_numel < 0) return fail(MFSDP_ERR_INVALID, "dst_numel must be non-negative");
  int src_unit, dst_unit, max_group, scale;
  if (int rc = setup_units(convert, elem_bytes, &src_unit, &dst_unit, &max_group, &scale)) return rc;
  for (int32_t i = 0; i < n_srcs; ++i)
    if (src_numels[i] < 0) return fail(MFSDP_ERR_INVALID, "src_numels[%d] is negative", i);

  auto prog = new mfsdp_segment_program();
  prog->convert = convert;
  prog->src_unit = src_unit;
  prog->dst_unit = dst_unit;
  prog->max_group = max_group;
  prog->dst_numel = dst_numel * scale;
  for (int32_t i = 0; i < n_srcs; ++i) prog->src_numels.push_back(src_numels[i] * scale);
  (void)hipGetDevice(&prog->device);

  // validate extents; collect destination intervals to reject overlapping writes
  std::vector<std::pair<int64_t, int64_t>> spans;
  for (int64_t i = 0; i < n_runs; ++i) {
    mfsdp_copy_run r = runs[i];
    if (r.rows < 0 || r.row_len < 0) {
      delete prog;
      return fail(MFSDP_ERR_INVALID, "run %lld: negative size", static_cast<long long>(i));
    }
    if (r.rows == 0 || r.row_len == 0) continue;
    if (r.src_id >= n_srcs) {
      delete prog;
      return fail(MFSDP_ERR_INVALID, "run %lld: src_id %d out of range", static_cast<long long>(i), r.src_id);
    }
    if (r.src_id < 0) r.src_id = -1;
    if (r.rows == 1) r.src_stride = r.dst_stride = 0;
    if (r.rows > 1 && (r.dst_stride < r.row_len || (r.src_id >= 0 && r.src_stride < 0))) {
      delete prog;
      return fail(MFSDP_ERR_INVALID, "run %lld: destination rows overlap or negative source pitch", static_cast<long long>(i));
    }
    const int64_t dst_last = r.dst_off + (r.rows - 1) * r.dst_stride + r.row_len;
    if (r.dst_off < 0 || dst_last > dst_numel) {
      delete prog;
      return fail(MFSDP_ERR_INVALID, "run %lld: destination range [%lld, %lld) leaves the output of %lld elements",
                  static_cast<long long>(i), static_cast<long long>(r.dst_off), static_cast<long long>(dst_last),
                  static_cast<long long>(dst_numel));
    }
    if (r.src_id >= 0) {
      const int64_t src_last = r.src_off + (r.rows - 1) * r.src_stride + r.row_len;
      if (r.src_off < 0 || src_last > src_numels[r.src_id]) {
        delete prog;
        return fail(MFSDP_ERR_INVALID, "run %lld: source range [%lld, %lld) leaves source %d of %lld elements",
                    static_cast<long long>(i), static_cast<long long>(r.src_off), static_cast<long long>(src_last),
                    r.src_id, static_cast<long long>(src_numels[r.src_id]));
      }
    }
    spans.emplace_back(r.dst_off, dst_last);
    prog->bytes_moved += r.rows * r.row_len * ((r.src_id >= 0 ? src_unit : 0) + dst_unit) * scale;
    // to units
    r.src_off *= scale; r.dst_off *= scale; r.row_len *= scale; r.src_stride *= scale; r.dst_stride *= scale;
    prog->runs.push_back(r);
  }
  // Bounding spans of different runs may interleave legally (two column blocks of one matrix), so only
  // exact duplicates of a start offset are rejected here; full disjointness is the caller's contract.
  std::sort(spans.begin(), spans.end());
  for (size_t i = 1; i < spans.size(); ++i) {
    if (spans[i].first == spans[i - 1].first) {
      delete prog;
      return fail(MFSDP_ERR_INVALID, "two runs write destination offset %lld", static_cast<long long>(spans[i].first));
    }
  }
  std::vector<Compiled> compiled;
  if (int rc = compile_variant(prog, max_group, &compiled)) {
    delete prog;
    return rc;
  }
  prog->variants[max_group] = compiled;
  *out = prog;
  return MFSDP_OK;
}

extern "C" void mfsdp_segment_program_destroy(mfsdp_segment_program* program) {
  if (program == nullptr) return;
  for (auto& kv : program->variants) free_compiled(kv.second);
  delete program;
}

extern "C" int64_t mfsdp_segment_program_bytes(const mfsdp_segment_program* program) {
  return program ? program->bytes_moved : 0;
}

extern "C" int64_t mfsdp_segment_program_num_runs(const mfsdp_segment_program* program) {
  return program ? static_cast<int64_t>(program->runs.size()) : 0;
}

extern "C" int mfsdp_segment_program_run(mfsdp_segment_program* program, const void* const* srcs, int32_t n_srcs,
                                         void* dst, void* stream) {
  if (program == nullptr) return fail(MFSDP_ERR_INVALID, "program is null");
  if (n_srcs != static_cast<int32_t>(program->src_numels.size()))
    return fail(MFSDP_ERR_INVALID, "program was created for %zu sources, got %d", program->src_numels.size(), n_srcs);
  if (program->runs.empty()) return MFSDP_OK;
  if (dst == nullptr) return fail(MFSDP_ERR_INVALID, "dst is null");
  SourceTable table;
  std::memset(&table, 0, sizeof(table));
  int cap = pointer_alignment_units(dst, program->dst_unit, program->max_group);
  for (int32_t i = 0; i < n_srcs; ++i) {
    if (srcs == nullptr || (srcs[i] == nullptr && program->src_numels[i] > 0))
      return fail(MFSDP_ERR_INVALID, "source %d is null", i);
    table.p[i] = static_cast<const char*>(srcs[i]);
    if (program->src_numels[i] > 0) cap = std::min(cap, pointer_alignment_units(srcs[i], program->src_unit, program->max_group));
  }
  const std::vector<Compiled>* compiled = nullptr;
  {
    std::lock_guard<std::mutex> lock(program->mu);
    auto it = program->variants.find(cap);
    if (it == program->variants.end()) {
      std::vector<Compiled> fresh;
      if (int rc = compile_variant(program, cap, &fresh)) return rc;
      it = program->variants.emplace(cap, std::move(fresh)).first;
    }
    compiled = &it->second;
  }
  for (const auto& c : *compiled)
    if (int rc = launch_compiled(program, c, table, static_cast<char*>(dst), as_stream(stream))) return rc;
  return MFSDP_OK;
}

extern "C" int mfsdp_copy_rank_segments_to_full(const void* local, int64_t local_numel, void* output,
                                                int64_t output_numel, const int64_t* global_starts,
                                                const int64_t* local_starts, const int64_t* numels,
                                                int64_t n_segments, int elem_bytes, void* stream) {
  if (n_segments < 0) return fail(MFSDP_ERR_INVALID, "n_segments must be non-negative");
  if (n_segments == 0) return MFSDP_OK;
  if (!global_starts || !local_starts || !numels) return fail(MFSDP_ERR_INVALID, "segment metadata is null");
  if (local_numel < 0 || output_numel < 0) return fail(MFSDP_ERR_INVALID, "tensor sizes must be non-negative");
  std::vector<mfsdp_copy_run> segs(n_segments), merged(n_segments);
  for (int64_t i = 0; i < n_segments; ++i) {
    if (numels[i] < 0) return fail(MFSDP_ERR_INVALID, "segment %lld has negative numel", static_cast<long long>(i));
    segs[i] = mfsdp_copy_run{local_starts[i], global_starts[i], numels[i], 1, 0, 0, 0, 0};
  }
  const int64_t n = mfsdp_merge_segment_runs(segs.data(), n_segments, merged.data());
  if (n == 0) return MFSDP_OK;
  if (local == nullptr || output == nullptr) return fail(MFSDP_ERR_INVALID, "local or output is null");
  mfsdp_segment_program* prog = nullptr;
  if (int rc = mfsdp_segment_program_create(merged.data(), n, &local_numel, 1, output_numel, MFSDP_CONVERT_NONE,
                                            elem_bytes, &prog))
    return rc;
  const void* srcs[1] = {local};
  int rc = mfsdp_segment_program_run(prog, srcs, 1, output, stream);
  if (rc == MFSDP_OK) {
    // the tables must outlive the kernel: wait before freeing them
    hipError_t e = hipStreamSynchronize(as_stream(stream));
    if (e != hipSuccess) rc = fail(MFSDP_ERR_HIP, "hipStreamSynchronize failed: %s", hipGetErrorString(e));
  }
  mfsdp_segment_program_destroy(prog);
  return rc;
}

// ---- contiguous range copy / cast ---------------------------------------------------------------

namespace {

// dst[g] = convert(src[g]) over n_groups contiguous vector groups, persistent grid-stride.
template <int SRC_B, int DST_B, int U, bool NT, bool HALF = false>
__global__ void __launch_bounds__(kBlockThreads)
linear_kernel(const char* __restrict__ src, char* __restrict__ dst, int64_t n_groups) {
  const int64_t span = static_cast<int64_t>(kBlockThreads) * U;
  for (int64_t base = static_cast<int64_t>(blockIdx.x) * span; base < n_groups;
       base += static_cast<int64_t>(gridDim.x) * span) {
    Words<SRC_B> data[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t g = base + u * kBlockThreads + threadIdx.x;
      if (g < n_groups) data[u] = load_bytes<SRC_B, NT>(src + g * SRC_B);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t g = base + u * kBlockThreads + threadIdx.x;
      if (g < n_groups) store_bytes<DST_B, NT>(dst + g * DST_B, convert_group<SRC_B, DST_B, HALF>(data[u]));
    }
  }
}

template <int SRC_B, int DST_B, bool HALF = false>
int launch_linear(const char* src, char* dst, int64_t n_groups, hipStream_t stream) {
  if (n_groups <= 0) return MFSDP_OK;
  constexpr int U = 4;
  const int64_t span = static_cast<int64_t>(kBlockThreads) * U;
  const int64_t want = (n_groups + span - 1) / span;
  // one workgroup per block of the tensor, not a persistent grid: workgroups are dispatched in order, so those in
  // flight sweep neighbouring addresses (bf16 -> fp32 of 202 M elements 5.83 against 5.65 TB/s with 16 per CU)
  const dim3 grid(static_cast<uint32_t>(std::max<int64_t>(1, std::min(want, kMaxGrid))));
  if (g_tuning.nontemporal)
    hipLaunchKernelGGL((linear_kernel<SRC_B, DST_B, U, true, HALF>), grid, dim3(kBlockThreads), 0, stream, src, dst, n_groups);
  else
    hipLaunchKernelGGL((linear_kernel<SRC_B, DST_B, U, false, HALF>), grid, dim3(kBlockThreads), 0, stream, src, dst, n_groups);
  MFSDP_CHECK_LAUNCH("linear_kernel");
  return MFSDP_OK;
}

// Moves `units` contiguous units: a wide body sized by the pointers' common alignment, then a
// unit-wide tail for the remainder.
int linear_dispatch(const char* src, char* dst, int64_t units, int src_unit, int dst_unit, int max_group,
                    hipStream_t stream, bool half = false) {
  int g = std::min(pointer_alignment_units(src, src_unit, max_group), pointer_alignment_units(dst, dst_unit, max_group));
  const int64_t body = units / g;
  const int64_t tail = units - body * g;
  const int sb = g * src_unit, db = g * dst_unit;
  int rc = MFSDP_ERR_UNSUPPORTED;
#define MFSDP_CASE(S_, D_) \
  if (sb == S_ && db == D_) rc = launch_linear<S_, D_>(src, dst, body, stream)
#define MFSDP_CONVERTING(S_, D_) \
  if (sb == S_ && db == D_) rc = half ? launch_linear<S_, D_, true>(src, dst, body, stream) : launch_linear<S_, D_, false>(src, dst, body, stream)
  MFSDP_CASE(16, 16); MFSDP_CASE(8, 8); MFSDP_CASE(4, 4); MFSDP_CASE(2, 2); MFSDP_CASE(1, 1);
  MFSDP_CONVERTING(16, 32); MFSDP_CONVERTING(8, 16); MFSDP_CONVERTING(4, 8); MFSDP_CONVERTING(2, 4);
  MFSDP_CONVERTING(32, 16); MFSDP_CONVERTING(16, 8); MFSDP_CONVERTING(8, 4); MFSDP_CONVERTING(4, 2);
#undef MFSDP_CONVERTING
#undef MFSDP_CASE
  if (rc == MFSDP_ERR_UNSUPPORTED) return fail(rc, "no kernel for %d -> %d byte groups", sb, db);
  if (rc != MFSDP_OK || tail == 0) return rc;
  const char* ts = src + body * sb;
  char* td = dst + body * db;
  if (src_unit == 1) return launch_linear<1, 1>(ts, td, tail, stream);
  if (src_unit == 2) return half ? launch_linear<2, 4, true>(ts, td, tail, stream) : launch_linear<2, 4, false>(ts, td, tail, stream);
  return half ? launch_linear<4, 2, true>(ts, td, tail, stream) : launch_linear<4, 2, false>(ts, td, tail, stream);
}

}  // namespace

extern "C" int mfsdp_copy_range(const void* in, int64_t in_numel, void* out, int64_t out_numel, int64_t input_offset,
                                int elem_bytes, void* stream) {
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8)
    return fail(MFSDP_ERR_INVALID, "elem_bytes must be 1, 2, 4 or 8, got %d", elem_bytes);
  if (in_numel < 0 || out_numel < 0) return fail(MFSDP_ERR_INVALID, "tensor sizes must be non-negative");
  if (input_offset < 0) return fail(MFSDP_ERR_INVALID, "input_offset must be non-negative");
  if (input_offset + out_numel > in_numel) return fail(MFSDP_ERR_INVALID, "copy range exceeds input tensor");
  if (out_numel == 0) return MFSDP_OK;
  if (in == nullptr || out == nullptr) return fail(MFSDP_ERR_INVALID, "in or out is null");
  const char* src = static_cast<const char*>(in) + input_offset * elem_bytes;
  return linear_dispatch(src, static_cast<char*>(out), out_numel * elem_bytes, 1, 1, 16, as_stream(stream));
}

extern "C" int mfsdp_cast(const void* src, void* dst, int64_t numel, int convert, void* stream) {
  if (numel < 0) return fail(MFSDP_ERR_INVALID, "numel must be non-negative");
  if (convert != MFSDP_CONVERT_BF16_TO_F32 && convert != MFSDP_CONVERT_F32_TO_BF16 && !is_half_conversion(convert))
    return fail(MFSDP_ERR_INVALID, "mfsdp_cast converts bf16 / f16 -> f32 or f32 -> bf16 / f16, got code %d", convert);
  if (numel == 0) return MFSDP_OK;
  if (src == nullptr || dst == nullptr) return fail(MFSDP_ERR_INVALID, "src or dst is null");
  const bool widen = convert == MFSDP_CONVERT_BF16_TO_F32 || convert == MFSDP_CONVERT_F16_TO_F32;
  return linear_dispatch(static_cast<const char*>(src), static_cast<char*>(dst), numel, widen ? 2 : 4, widen ? 4 : 2,
                         g_tuning.convert_group, as_stream(stream), is_half_conversion(convert));
}

// ---- accumulate: dst += src --------------------------------------------------------------------------------------

namespace {

// FMT 0: fp32, 1: bf16, 2: fp16.  16-bit formats add in fp32 and round to nearest even once, as Tensor.add_ does.
template <int FMT>
__device__ __forceinline__ uint32_t add_word(uint32_t a, uint32_t b) {
  if constexpr (FMT == 0) {
    return __float_as_uint(__uint_as_float(a) + __uint_as_float(b));
  } else if constexpr (FMT == 1) {
    const float lo = __uint_as_float(a << 16) + __uint_as_float(b << 16);
    const float hi = __uint_as_float(a & 0xffff0000u) + __uint_as_float(b & 0xffff0000u);
    return f32_bits_to_bf16_bits(__float_as_uint(lo)) | (f32_bits_to_bf16_bits(__float_as_uint(hi)) << 16);
  } else {
    const float lo = __uint_as_float(f16_bits_to_f32_bits(a & 0xffffu)) + __uint_as_float(f16_bits_to_f32_bits(b & 0xffffu));
    const float hi = __uint_as_float(f16_bits_to_f32_bits(a >> 16)) + __uint_as_float(f16_bits_to_f32_bits(b >> 16));
    return f32_bits_to_f16_bits(__float_as_uint(lo)) | (f32_bits_to_f16_bits(__float_as_uint(hi)) << 16);
  }
}

// n_vec 16-byte groups, then `tail` single elements starting at element `tail_first`
template <int FMT>
__global__ void __launch_bounds__(kBlockThreads)
accumulate_kernel(char* __restrict__ dst, const char* __restrict__ src, int64_t n_vec, int64_t tail_first, int64_t tail) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlockThreads;
  for (int64_t g = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x; g < n_vec; g += stride) {
    const Words<16> b = load_bytes<16, true>(src + g * 16);
    Words<16> a = load_bytes<16, false>(dst + g * 16);
#pragma unroll
    for (int i = 0; i < 4; ++i) a.w[i] = add_word<FMT>(a.w[i], b.w[i]);
    store_bytes<16, false>(dst + g * 16, a);
  }
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x; i < tail; i += stride) {
    const int64_t e = tail_first + i;
    if constexpr (FMT == 0) {
      reinterpret_cast<float*>(dst)[e] += reinterpret_cast<const float*>(src)[e];
    } else {
      uint16_t* d = reinterpret_cast<uint16_t*>(dst) + e;
      *d = static_cast<uint16_t>(add_word<FMT>(*d, reinterpret_cast<const uint16_t*>(src)[e]));
    }
  }
}

}  // namespace

extern "C" int mfsdp_accumulate(void* dst, const void* src, int64_t numel, int dtype, void* stream) {
  if (numel < 0) return fail(MFSDP_ERR_INVALID, "numel must be non-negative");
  if (dtype != MFSDP_F32 && dtype != MFSDP_BF16 && dtype != MFSDP_F16) return fail(MFSDP_ERR_INVALID, "dtype must be f32, bf16 or f16");
  if (numel == 0) return MFSDP_OK;
  if (dst == nullptr || src == nullptr) return fail(MFSDP_ERR_INVALID, "dst or src is null");
  const int elem = dtype == MFSDP_F32 ? 4 : 2;
  const bool aligned = (reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) % 16 == 0;
  const int64_t per_vec = 16 / elem;
  const int64_t n_vec = aligned ? numel / per_vec : 0;
  const int64_t tail_first = n_vec * per_vec, tail = numel - tail_first;
  const int64_t work = std::max(n_vec, tail);
  const int64_t want = (work + kBlockThreads - 1) / kBlockThreads;
  // one workgroup per block, as launch_linear: 6.27 against 4.78 TB/s with 16 persistent workgroups per CU (fp32, 202 M elements)
  const dim3 grid(static_cast<uint32_t>(std::max<int64_t>(1, std::min(want, kMaxGrid))));
  char* d = static_cast<char*>(dst);
  const char* s = static_cast<const char*>(src);
  if (dtype == MFSDP_F32) hipLaunchKernelGGL((accumulate_kernel<0>), grid, dim3(kBlockThreads), 0, as_stream(stream), d, s, n_vec, tail_first, tail);
  else if (dtype == MFSDP_BF16) hipLaunchKernelGGL((accumulate_kernel<1>), grid, dim3(kBlockThreads), 0, as_stream(stream), d, s, n_vec, tail_first, tail);
  else hipLaunchKernelGGL((accumulate_kernel<2>), grid, dim3(kBlockThreads), 0, as_stream(stream), d, s, n_vec, tail_first, tail);
  MFSDP_CHECK_LAUNCH("accumulate_kernel");
  return MFSDP_OK;
}
