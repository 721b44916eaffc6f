// Rank-segment copy driven by DEVICE-resident metadata: the enqueue-only form of copy_rank_segments_to_full.
//
//     output[global_starts[s] + o] = local[local_starts[s] + o]      for o < numels[s], every segment s
//
// The three int64 arrays live in device memory (the caller caches them per layout), so the host sees neither the
// segment sizes nor their alignment: everything a segment needs is derived inside the kernels.
//
// Addressing.  For segment s let S and D be the byte addresses of its first source and destination element.  The
// widest vector both sides can use is V = the largest power of two <= 16 dividing S - D; the copy then runs on the
// destination's V-byte grid: vector k covers destination bytes [D - lead + kV, D - lead + (k+1)V) with
// lead = D mod V, so every full vector is V-aligned on both sides, and only the first and the last vector of a segment
// can be partial (moved byte by byte).  A wavefront moves a tile of 64 * 4 vectors (4 KiB at V = 16) with four
// independent loads in flight per lane, each wave-level access one contiguous 64 V-byte span.
//
// Two launch shapes:
//   * uniform: one tile slot per (segment, tile index up to the longest segment), as the reference's
//     (tiles, segments) grid; needs no memory besides the arguments, slots past a segment's end exit at once;
//   * balanced: two small kernels write the running tile counts of the segments (per block of 1024 segments, plus one
//     offset per block) into a caller-provided (or the library's static) scratch array, and the waves of the copy
//     grid take one tile each (striding on when the grid is capped) and find its segment by bisection -- the work
//     is cut by bytes, so one very long segment beside many short ones costs no empty slots.
#include "mfsdp_common.h"

#include <algorithm>
#include <mutex>

namespace mfsdp {
namespace {

constexpr int kWave = 64;
constexpr int kUnroll = 4;  // loads in flight per lane = 1 KiB spans per tile; on 4.7 KiB row segments: 1 -> 65 us, 2 -> 45, 4 -> 36, 8 -> 48
constexpr int kTileVectors = kWave * kUnroll;
constexpr int kCopyThreads = 64;  // one wavefront per workgroup
constexpr int kWavesPerBlock = kCopyThreads / kWave;
constexpr int kCountThreads = 256;
constexpr int kCountPerThread = 4;
constexpr int kBlockSegments = kCountThreads * kCountPerThread;  // segments whose tile counts one workgroup sums
constexpr int kBlockShift = 10;
static_assert(kBlockSegments == 1 << kBlockShift, "block of segments");
// Consecutive tiles one bisection serves, and the workgroups (of one wavefront each) per CU the balanced grid is capped at.
// Measured on the 21 250 row segments of a hidden4096 rank shard, waves per CU = 4 x the figure given for workgroups of
// four waves: (8 tiles, 16 waves per CU) 50 us, (4, 64) 48 us, (1, 256) 45 us, (1, 1024) 59 us; eight segments of 50 MB:
// 163, 176, 148, 155 us.  Many short-lived waves beat few long-lived ones, as in the other copy kernels, until the empty
// workgroups of the upper-bound grid cost more than they hide.  One wavefront per workgroup (dispatch in index order
// sweeps neighbouring addresses) took the uniform shape from 5.4-5.7 to 5.6-5.8 TB/s on that shard, close to the
// compiled segment program; the balanced shape stays at 46 us there (its two count kernels are 9 us of that, and a
// ballot search over the running counts in place of the bisection was slower still: 87 us -- the set-up of a wave that
// moves 4 KiB is what costs), so it is the shape for layouts whose segment lengths differ widely, not for this one.
constexpr int kChunkTiles = 1;
constexpr int kBalancedBlocksPerCu = 256;
constexpr int kMaxDevices = 64;

// Scratch of the entry point that allocates nothing: the tile-count tables of up to kStaticMaxSegments segments.
constexpr int64_t kStaticScratchBytes = (1 << 20) + 2048;
constexpr int64_t kStaticMaxSegments = MFSDP_NOALLOC_MAX_SEGMENTS;
// entries of 8 bytes the tile-count tables of n segments take: n + 1 running counts, one offset per block of segments + 1
constexpr int64_t table_entries(int64_t n) { return n + 1 + (n + kBlockSegments - 1) / kBlockSegments + 1; }
static_assert(table_entries(kStaticMaxSegments) * 8 <= kStaticScratchBytes, "the header states the limit");
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct SegmentCopyArgs {
  const char* local;
  char* output;
  const int64_t* global_starts;
  const int64_t* local_starts;
  const int64_t* numels;
  int64_t local_numel;
  int64_t output_numel;
  int64_t n_segments;
  int64_t limit;  // elements copied per segment at most (the reference's grid covers max_numel rounded up to 256)
  int elem_bytes;
};

struct Geometry {
  const char* src;   // first source byte
  char* dst;         // first destination byte
  int64_t nbytes;
  uint32_t vec;      // V
  uint32_t lead;     // D mod V
  uint64_t n_vec;    // vectors on the destination's V-byte grid that hold at least one byte of the segment
  uint64_t tiles;
};

// What the addresses of a segment allow, from the low 32 bits of its first source and destination byte (V <= 16, so
// the low four bits decide): V and the destination's offset inside its V-byte vector.
__device__ __forceinline__ void vector_shape(uint32_t src_lo, uint32_t dst_lo, uint32_t* vec, uint32_t* lead) {
  const uint32_t d = (src_lo - dst_lo) & 15u;
  *vec = d ? (d & (0u - d)) : 16u;  // lowest set bit of the difference, 16 when the two are congruent mod 16
  *lead = dst_lo & (*vec - 1);
}

// True when the segment is copied at all: not empty, and inside both tensors.
__device__ __forceinline__ bool segment_is_live(const SegmentCopyArgs& a, int64_t gs, int64_t ls, int64_t n) {
  return n > 0 && gs >= 0 && ls >= 0 && ls <= a.local_numel - n && gs <= a.output_numel - n;
}

// Tiles of a segment from its three metadata values (zero when it is not copied): the part of the geometry the scan
// needs, in 32-bit arithmetic wherever the low bits decide.
__device__ __forceinline__ uint64_t segment_tiles(const SegmentCopyArgs& a, int64_t gs, int64_t ls, int64_t n) {
  if (!segment_is_live(a, gs, ls, n)) return 0;
  n = n < a.limit ? n : a.limit;
  const uint32_t eb = static_cast<uint32_t>(a.elem_bytes);
  uint32_t vec, lead;
  vector_shape(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(a.local)) + static_cast<uint32_t>(ls) * eb,
               static_cast<uint32_t>(reinterpret_cast<uintptr_t>(a.output)) + static_cast<uint32_t>(gs) * eb, &vec, &lead);
  const uint64_t n_vec = (static_cast<uint64_t>(n) * eb + lead + vec - 1) >> __builtin_ctz(vec);
  return (n_vec + kTileVectors - 1) / kTileVectors;
}

// Geometry of segment s; a segment that is empty or leaves either tensor gets zero tiles (it is not copied).
__device__ __forceinline__ Geometry segment_geometry(const SegmentCopyArgs& a, int64_t s) {
  Geometry g{};
  const int64_t gs = a.global_starts[s], ls = a.local_starts[s];
  int64_t n = a.numels[s];
  if (!segment_is_live(a, gs, ls, n)) return g;
  n = n < a.limit ? n : a.limit;
  g.src = a.local + ls * a.elem_bytes;
  g.dst = a.output + gs * a.elem_bytes;
  g.nbytes = n * a.elem_bytes;
  vector_shape(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(g.src)), static_cast<uint32_t>(reinterpret_cast<uintptr_t>(g.dst)), &g.vec, &g.lead);
  g.n_vec = (static_cast<uint64_t>(g.nbytes) + g.lead + g.vec - 1) >> __builtin_ctz(g.vec);  // V is a power of two
  g.tiles = (g.n_vec + kTileVectors - 1) / kTileVectors;
  return g;
}

template <int V>
struct Vec {
  uint32_t w[(V + 3) / 4];
};

template <int V>
__device__ __forceinline__ Vec<V> load_vec(const char* p) {
  Vec<V> r;
  if constexpr (V == 16) {
    const u32x4 a = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    r.w[0] = a.x; r.w[1] = a.y; r.w[2] = a.z; r.w[3] = a.w;
  } else if constexpr (V == 8) {
    const u32x2 a = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    r.w[0] = a.x; r.w[1] = a.y;
  } else if constexpr (V == 4) {
    r.w[0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p));
  } else if constexpr (V == 2) {
    r.w[0] = *reinterpret_cast<const uint16_t*>(p);
  } else {
    r.w[0] = *reinterpret_cast<const uint8_t*>(p);
  }
  return r;
}

template <int V>
__device__ __forceinline__ void store_vec(char* p, const Vec<V>& v) {
  if constexpr (V == 16) {
    const u32x4 a = {v.w[0], v.w[1], v.w[2], v.w[3]};
    __builtin_nontemporal_store(a, reinterpret_cast<u32x4*>(p));
  } else if constexpr (V == 8) {
    const u32x2 a = {v.w[0], v.w[1]};
    __builtin_nontemporal_store(a, reinterpret_cast<u32x2*>(p));
  } else if constexpr (V == 4) {
    __builtin_nontemporal_store(v.w[0], reinterpret_cast<uint32_t*>(p));
  } else if constexpr (V == 2) {
    *reinterpret_cast<uint16_t*>(p) = static_cast<uint16_t>(v.w[0]);
  } else {
    *reinterpret_cast<uint8_t*>(p) = static_cast<uint8_t>(v.w[0]);
  }
}

// Tiles [tile_begin, tile_end) of one segment, by one wavefront.
template <int V>
__device__ __forceinline__ void copy_tiles(const Geometry& g, uint64_t tile_begin, uint64_t tile_end, uint32_t lane) {
  for (uint64_t tile = tile_begin; tile < tile_end; ++tile) {
    Vec<V> data[kUnroll];
    int64_t at[kUnroll];  // byte offset of the vector from the segment's first byte; < 0 or cut at the end: partial
    bool full[kUnroll], partial[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const uint64_t k = tile * kTileVectors + static_cast<uint64_t>(u) * kWave + lane;
      at[u] = static_cast<int64_t>(k) * V - static_cast<int64_t>(g.lead);
      const bool live = k < g.n_vec;
      full[u] = live && at[u] >= 0 && at[u] + V <= g.nbytes;
      partial[u] = live && !full[u];
      if (full[u]) data[u] = load_vec<V>(g.src + at[u]);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      if (full[u]) store_vec<V>(g.dst + at[u], data[u]);
      if (partial[u]) {  // the first or the last vector of the segment
        const int64_t b0 = at[u] < 0 ? 0 : at[u];
        const int64_t b1 = at[u] + V < g.nbytes ? at[u] + V : g.nbytes;
        for (int64_t b = b0; b < b1; ++b) g.dst[b] = g.src[b];
      }
    }
  }
}

__device__ __forceinline__ void copy_tiles_any(const Geometry& g, uint64_t tile_begin, uint64_t tile_end, uint32_t lane) {
  switch (g.vec) {
    case 16: copy_tiles<16>(g, tile_begin, tile_end, lane); break;
    case 8: copy_tiles<8>(g, tile_begin, tile_end, lane); break;
    case 4: copy_tiles<4>(g, tile_begin, tile_end, lane); break;
    case 2: copy_tiles<2>(g, tile_begin, tile_end, lane); break;
    default: copy_tiles<1>(g, tile_begin, tile_end, lane); break;
  }
}

// ---- uniform launch shape: slot = (segment, j) with j < slots_per_segment, the tile count of the longest segment at
// V = 16; the slot's wave moves tiles j, j + slots_per_segment, ... of its segment (more than one only when the
// segment's addresses force a narrower vector).
// One wavefront per workgroup: workgroups are dispatched in index order, so the waves in flight sweep neighbouring
// addresses (as in the other copy kernels, small short-lived workgroups serve HBM best).
// FAST: fewer than 2^31 slots, so the slot's segment comes from a multiply-high by a host-computed reciprocal
// (slots_per_segment >= 2; magic == 0 says one slot per segment) instead of a 64-bit division in every workgroup.
template <bool FAST>
__global__ void __launch_bounds__(kWave)
segment_copy_uniform_kernel(SegmentCopyArgs a, uint64_t slots_per_segment, uint64_t n_slots, uint32_t magic, uint32_t shift) {
  const uint32_t lane = threadIdx.x;
  for (uint64_t slot = blockIdx.x; slot < n_slots; slot += gridDim.x) {
    uint64_t s, first;
    if constexpr (FAST) {
      const uint32_t slot32 = static_cast<uint32_t>(slot);
      const uint32_t s32 = magic == 0 ? slot32 : (__umulhi(magic, slot32) >> shift);
      s = s32;
      first = slot32 - s32 * static_cast<uint32_t>(slots_per_segment);
    } else {
      s = slot / slots_per_segment;
      first = slot - s * slots_per_segment;
    }
    const Geometry g = segment_geometry(a, static_cast<int64_t>(s));
    for (uint64_t tile = first; tile < g.tiles; tile += slots_per_segment) copy_tiles_any(g, tile, tile + 1, lane);
  }
}

// ---- balanced launch shape, step 1.  The running tile counts are kept in two levels, so that many workgroups can
// build them: counts[s + 1] = tiles of the segments from the start of s's block of 1024 up to and including s, and
// block_offsets[b] = tiles of all blocks before b (block_offsets[n_blocks] = all tiles).  running_count() below puts
// the two together: tiles of the segments before s.
__global__ void __launch_bounds__(kCountThreads)
segment_tile_count_kernel(SegmentCopyArgs a, uint64_t* __restrict__ counts, uint64_t* __restrict__ block_offsets) {
  __shared__ uint64_t wave_sums[kCountThreads / kWave];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kBlockSegments + static_cast<int64_t>(tid) * kCountPerThread;
  if (blockIdx.x == 0 && tid == 0) {
    counts[0] = 0;
    block_offsets[0] = 0;
  }
  uint64_t mine[kCountPerThread];
  uint64_t sum = 0;
#pragma unroll
  for (int i = 0; i < kCountPerThread; ++i) {
    const int64_t at = first + i < a.n_segments ? first + i : a.n_segments - 1;
    mine[i] = first + i < a.n_segments ? segment_tiles(a, a.global_starts[at], a.local_starts[at], a.numels[at]) : 0;
    sum += mine[i];
  }
  // inclusive scan of the per-thread sums: within the wave by shuffles, across the waves through LDS
  uint64_t incl = sum;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const uint64_t up = __shfl_up(incl, d, kWave);
    if (lane >= d) incl += up;
  }
  if (lane == kWave - 1) wave_sums[wave] = incl;
  __syncthreads();
  uint64_t before = 0;
  for (int w = 0; w < wave; ++w) before += wave_sums[w];
  uint64_t running = before + incl - sum;  // tiles of the block's segments before this thread's first
#pragma unroll
  for (int i = 0; i < kCountPerThread; ++i) {
    running += mine[i];
    if (first + i < a.n_segments) counts[first + i + 1] = running;
  }
  if (tid == kCountThreads - 1) block_offsets[blockIdx.x + 1] = before + incl;  // the block's total, summed up by the next kernel
}

// One wavefront turns the block totals (entries 1 .. n_blocks) into running sums, 64 at a time.
__global__ void __launch_bounds__(kWave)
block_offset_kernel(uint64_t* __restrict__ block_offsets, int64_t n_blocks) {
  const int lane = threadIdx.x;
  uint64_t carry = 0;
  for (int64_t base = 0; base < n_blocks; base += kWave) {
    const int64_t at = base + lane;
    uint64_t incl = at < n_blocks ? block_offsets[at + 1] : 0;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const uint64_t up = __shfl_up(incl, d, kWave);
      if (lane >= d) incl += up;
    }
    if (at < n_blocks) block_offsets[at + 1] = carry + incl;
    carry += __shfl(incl, kWave - 1, kWave);
  }
}

// Tiles of the segments before s, 0 <= s <= n_segments.
__device__ __forceinline__ uint64_t running_count(const uint64_t* __restrict__ counts, const uint64_t* __restrict__ block_offsets, int64_t s) {
  return s == 0 ? 0 : counts[s] + block_offsets[(s - 1) >> kBlockShift];
}

// ---- balanced launch shape, step 2: every wave takes chunks of chunk_tiles consecutive tiles, chunk = wave, wave + waves, ...
__global__ void __launch_bounds__(kCopyThreads)
segment_copy_balanced_kernel(SegmentCopyArgs a, const uint64_t* __restrict__ counts, const uint64_t* __restrict__ block_offsets,
                             uint32_t chunk_tiles) {
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint64_t wave = static_cast<uint64_t>(blockIdx.x) * kWavesPerBlock + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint64_t n_waves = static_cast<uint64_t>(gridDim.x) * kWavesPerBlock;
  auto prefix = [&](int64_t at) { return running_count(counts, block_offsets, at); };
  const uint64_t total = prefix(a.n_segments);
  const uint64_t n_chunks = (total + chunk_tiles - 1) / chunk_tiles;
  for (uint64_t chunk = wave; chunk < n_chunks; chunk += n_waves) {
    uint64_t t = chunk * chunk_tiles;
    const uint64_t t_end = t + chunk_tiles < total ? t + chunk_tiles : total;
    // the segment holding tile t: prefix(s) <= t < prefix(s + 1)  (prefix(0) = 0 <= t < total = prefix(n_segments))
    int64_t lo = 0, hi = a.n_segments;
    while (hi - lo > 1) {
      const int64_t mid = lo + ((hi - lo) >> 1);
      if (prefix(mid) <= t) lo = mid; else hi = mid;
    }
    int64_t s = lo;
    while (t < t_end && s < a.n_segments) {
      const uint64_t seg_begin = prefix(s), seg_end = prefix(s + 1);
      if (t >= seg_end) { ++s; continue; }
      const Geometry g = segment_geometry(a, s);
      const uint64_t upto = t_end < seg_end ? t_end : seg_end;
      copy_tiles_any(g, t - seg_begin, upto - seg_begin, lane);
      t = upto;
    }
  }
}

int check_args(const void* local, int64_t local_numel, void* output, int64_t output_numel, const int64_t* d_global_starts,
               const int64_t* d_local_starts, const int64_t* d_numels, int64_t n_segments, int64_t max_numel, int elem_bytes) {
  if (n_segments < 0) return fail(MFSDP_ERR_INVALID, "n_segments must be non-negative");
  if (max_numel < 0) return fail(MFSDP_ERR_INVALID, "max_numel must be non-negative");
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8)
    return fail(MFSDP_ERR_INVALID, "elem_bytes must be 1, 2, 4 or 8, got %d", elem_bytes);
  if (local_numel < 0 || output_numel < 0) return fail(MFSDP_ERR_INVALID, "tensor sizes must be non-negative");
  if (n_segments > 0 && max_numel > 0) {
    if (!d_global_starts || !d_local_starts || !d_numels) return fail(MFSDP_ERR_INVALID, "segment metadata is null");
    if (!local || !output) return fail(MFSDP_ERR_INVALID, "local or output is null");
    if ((reinterpret_cast<uintptr_t>(local) | reinterpret_cast<uintptr_t>(output)) % elem_bytes)
      return fail(MFSDP_ERR_INVALID, "local and output must be aligned to the element size");
  }
  return MFSDP_OK;
}

SegmentCopyArgs make_args(const void* local, int64_t local_numel, void* output, int64_t output_numel,
                          const int64_t* d_global_starts, const int64_t* d_local_starts, const int64_t* d_numels,
                          int64_t n_segments, int64_t max_numel, int elem_bytes) {
  SegmentCopyArgs a{};
  a.local = static_cast<const char*>(local);
  a.output = static_cast<char*>(output);
  a.global_starts = d_global_starts;
  a.local_starts = d_local_starts;
  a.numels = d_numels;
  a.local_numel = local_numel;
  a.output_numel = output_numel;
  a.n_segments = n_segments;
  // the reference launches ceil(max_numel / 256) blocks of 256 threads per segment (matrix_copy_cuda.cu:45-51):
  // offsets below that many elements are copied, whatever numels[s] says
  a.limit = (max_numel + 255) / 256 * 256;
  a.elem_bytes = elem_bytes;
  return a;
}

// Upper bound of the tiles one segment can need: V >= elem_bytes, plus one vector for a misaligned start.
uint64_t max_tiles_per_segment(const SegmentCopyArgs& a) {
  const uint64_t vectors = static_cast<uint64_t>(a.limit) + 1;
  return (vectors + kTileVectors - 1) / kTileVectors;
}

int launch_balanced(const SegmentCopyArgs& a, uint64_t* tables, hipStream_t stream) {
  uint64_t* counts = tables;                          // n_segments + 1 entries
  uint64_t* block_offsets = tables + a.n_segments + 1;  // n_blocks + 1 entries
  const int64_t n_blocks = (a.n_segments + kBlockSegments - 1) / kBlockSegments;
  if (n_blocks > (int64_t{1} << 31) - 1) return fail(MFSDP_ERR_UNSUPPORTED, "%lld segments are beyond the grid", static_cast<long long>(a.n_segments));
  hipLaunchKernelGGL(segment_tile_count_kernel, dim3(static_cast<uint32_t>(n_blocks)), dim3(kCountThreads), 0, stream, a, counts, block_offsets);
  MFSDP_CHECK_LAUNCH("segment_tile_count_kernel");
  const uint64_t bound = static_cast<uint64_t>(a.n_segments) * max_tiles_per_segment(a);
  hipLaunchKernelGGL(block_offset_kernel, dim3(1), dim3(kWave), 0, stream, block_offsets, n_blocks);
  MFSDP_CHECK_LAUNCH("block_offset_kernel");
  // one tile per wave while the grid can hold them all (excess waves leave at once; beyond that the waves stride on)
  const uint64_t want = (bound + kChunkTiles * kWavesPerBlock - 1) / (kChunkTiles * kWavesPerBlock);
  const uint64_t cap = static_cast<uint64_t>(device_cu_count()) * kBalancedBlocksPerCu;
  const dim3 grid(static_cast<uint32_t>(std::max<uint64_t>(1, std::min(want, cap))));
  hipLaunchKernelGGL(segment_copy_balanced_kernel, grid, dim3(kCopyThreads), 0, stream, a, counts, block_offsets, static_cast<uint32_t>(kChunkTiles));
  MFSDP_CHECK_LAUNCH("segment_copy_balanced_kernel");
  return MFSDP_OK;
}

// Device address of the static scratch array, looked up once per device (each device holds its own copy).
int static_scratch(uint64_t** out) {
  static std::mutex mu;
  static uint64_t* cached[kMaxDevices] = {nullptr};
  int dev = 0;
  MFSDP_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(MFSDP_ERR_UNSUPPORTED, "device index %d is beyond the %d devices the static scratch covers", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(mu);
  if (cached[dev] == nullptr) {
    void* ptr = nullptr;
    MFSDP_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) return fail(MFSDP_ERR_HIP, "hipGetSymbolAddress returned a null address for the static scratch");
    cached[dev] = static_cast<uint64_t*>(ptr);
  }
  *out = cached[dev];
  return MFSDP_OK;
}

}  // namespace
}  // namespace mfsdp

using namespace mfsdp;

extern "C" int64_t mfsdp_copy_rank_segments_workspace_bytes(int64_t n_segments) {
  return n_segments < 0 ? 0 : table_entries(n_segments) * 8;
}

extern "C" int mfsdp_copy_rank_segments_to_full_device(const void* local, int64_t local_numel, void* output, int64_t output_numel,
                                                       const int64_t* d_global_starts, const int64_t* d_local_starts,
                                                       const int64_t* d_numels, int64_t n_segments, int64_t max_numel,
                                                       int elem_bytes, void* workspace, int64_t workspace_bytes, void* stream) {
  if (int rc = check_args(local, local_numel, output, output_numel, d_global_starts, d_local_starts, d_numels, n_segments, max_numel, elem_bytes)) return rc;
  if (n_segments == 0 || max_numel == 0) return MFSDP_OK;
  const SegmentCopyArgs a = make_args(local, local_numel, output, output_numel, d_global_starts, d_local_starts, d_numels, n_segments, max_numel, elem_bytes);
  if (workspace != nullptr) {
    if (workspace_bytes < mfsdp_copy_rank_segments_workspace_bytes(n_segments))
      return fail(MFSDP_ERR_INVALID, "workspace of %lld bytes needed for %lld segments, got %lld",
                  static_cast<long long>(mfsdp_copy_rank_segments_workspace_bytes(n_segments)), static_cast<long long>(n_segments),
                  static_cast<long long>(workspace_bytes));
    if (reinterpret_cast<uintptr_t>(workspace) % 8) return fail(MFSDP_ERR_INVALID, "workspace must be 8-byte aligned");
    return launch_balanced(a, static_cast<uint64_t*>(workspace), as_stream(stream));
  }
  // tiles of the longest segment when its addresses allow 16-byte vectors (one more vector for a misaligned start)
  const uint64_t per_segment = (static_cast<uint64_t>(a.limit) * elem_bytes / 16 + kTileVectors) / kTileVectors;
  const uint64_t n_slots = static_cast<uint64_t>(n_segments) * per_segment;
  const dim3 grid(static_cast<uint32_t>(std::min<uint64_t>(n_slots, (uint64_t{1} << 31) - 1)));
  if (n_slots < (uint64_t{1} << 31)) {
    // floor(slot / d) for slot < 2^31 as umulhi(magic, slot) >> shift, with the round-up reciprocal of d >= 2
    uint32_t magic = 0, shift = 0;
    if (per_segment >= 2) {
      uint32_t l = 0;
      while ((uint64_t{1} << l) < per_segment) ++l;  // ceil(log2 d) >= 1
      magic = static_cast<uint32_t>((static_cast<unsigned __int128>(1) << (31 + l)) / per_segment + 1);
      shift = l - 1;
    }
    hipLaunchKernelGGL(segment_copy_uniform_kernel<true>, grid, dim3(kWave), 0, as_stream(stream), a, per_segment, n_slots, magic, shift);
  } else {
    hipLaunchKernelGGL(segment_copy_uniform_kernel<false>, grid, dim3(kWave), 0, as_stream(stream), a, per_segment, n_slots, 0u, 0u);
  }
  MFSDP_CHECK_LAUNCH("segment_copy_uniform_kernel");
  return MFSDP_OK;
}

extern "C" int mfsdp_copy_rank_segments_to_full_noalloc(const void* local, int64_t local_numel, void* output, int64_t output_numel,
                                                        const int64_t* d_global_starts, const int64_t* d_local_starts,
                                                        const int64_t* d_numels, int64_t n_segments, int64_t max_numel,
                                                        int elem_bytes, void* stream) {
  if (int rc = check_args(local, local_numel, output, output_numel, d_global_starts, d_local_starts, d_numels, n_segments, max_numel, elem_bytes)) return rc;
  if (n_segments > kStaticMaxSegments)
    return fail(MFSDP_ERR_UNSUPPORTED, "the static scratch holds the tile counts of at most %lld segments, got %lld",
                static_cast<long long>(kStaticMaxSegments), static_cast<long long>(n_segments));
  if (n_segments == 0 || max_numel == 0) return MFSDP_OK;
  uint64_t* prefix = nullptr;
  if (int rc = static_scratch(&prefix)) return rc;
  const SegmentCopyArgs a = make_args(local, local_numel, output, output_numel, d_global_starts, d_local_starts, d_numels, n_segments, max_numel, elem_bytes);
  return launch_balanced(a, prefix, as_stream(stream));
}
