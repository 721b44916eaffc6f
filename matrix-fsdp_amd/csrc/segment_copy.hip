// Segment programs: one bandwidth-bound gfx950 kernel that replays a whole shard layout's copy (every rank,
// every segment, pad zero-fill, optional bf16 / fp16 <-> fp32 conversion) in a single launch.
//
// Work is cut by BYTES, not by segment: every run is divided into tiles of 256 * U vector groups (4 KiB of 16-byte
// groups at U = 1) and a workgroup moves one tile, thread i taking groups i, i + 256, ..., so every wave-level load
// / store touches one contiguous 1 KiB span whenever the tile lies inside a row.  Strided 2-D runs (block shards)
// find their row with a multiply-high by a host-computed reciprocal instead of a division.  By default there is one
// workgroup per tile and no grid-stride loop; a persistent grid is a tuning option.
#include "mfsdp_common.h"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <queue>
#include <type_traits>
#include <vector>

namespace mfsdp {
namespace {

constexpr int kMaxSources = 128;  // source pointers one launch carries by value in its kernel arguments
constexpr int kMaxBatch = 64;     // destination pointers (buffers) one launch carries
constexpr int kDefaultBlocksPerCu = 0;  // one workgroup per tile
constexpr int kDefaultBlockThreads = 64;
constexpr int kBlockThreads = 256;
constexpr int kFillTileSpans = 8;  // spans of 256 * U groups a zero-fill tile covers (its group count must stay below 2^16)
constexpr int64_t kMaxGrid = (int64_t{1} << 31) - 1;  // grid-stride loops keep a capped grid correct
constexpr int64_t kMaxUnitsPerRun = 0x7fffffff;  // a device run holds fewer than 2^31 units: the reciprocal division is exact below 2^31 groups, at any group width

struct SourceTable {
  const char* p[kMaxSources];  // buffer b's source i at p[b * sources_per_buffer + i]
};
struct DestTable {
  char* p[kMaxBatch];
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

// One tile = the work of one workgroup, 16 bytes.  A tile that lies inside one row of its run is DIRECT: it carries
// its own offsets, so the workgroup needs no run descriptor (one dependent scalar load before its data loads instead
// of two, and no row arithmetic).  Runs whose rows are short get GENERIC tiles of 256 * U consecutive groups of the
// run, which may span rows and go through the run descriptor.
//   direct : a = source group offset | (source id + 1) << 48  (0: zero fill),  b = destination group offset | groups << 48
//   generic: a = 1 << 63 | run index,                                           b = tile index within the run
struct DevTile {
  uint64_t a;
  uint64_t b;
};
constexpr uint64_t kTileGeneric = uint64_t{1} << 63;
constexpr uint64_t kTileOffsetMask = (uint64_t{1} << 48) - 1;

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

// One launch replays the program over `batch` buffers (base pointers differ, tables are shared): the global tile
// index T = b * n_tiles + t walks buffer after buffer.  A tile is 256 * U vector groups moved by one workgroup,
// thread i taking groups i, i + 256, ...: at U = 1 a workgroup lives for one 4 KiB span, and with one workgroup per
// tile (no grid-stride loop) the workgroups in flight sweep neighbouring addresses in dispatch order, loads and
// stores finely interleaved -- what HBM serves best (a plain copy: 6.5 TB/s against 5.9 for a persistent grid); and the
// finer the better: by default the 256 lanes of a tile are four workgroups of one wavefront each (THREADS = 64), which
// all read the same 16-byte tile entry.
// narrow_shift s > 0 runs the tables at a vector group 2^s times narrower than the one they were compiled for (base
// pointers less aligned than the layout): a tile is then 2^s sub-tiles, and group g of the narrow grid lies in natural
// group g >> s.
template <int SRC_B, int DST_B, int U, bool NT, bool NTS = NT, bool HALF = false, int THREADS = kBlockThreads>
__global__ void __launch_bounds__(THREADS)
segment_program_kernel(SourceTable srcs, DestTable dsts, const DevRun* __restrict__ runs, const DevTile* __restrict__ tiles,
                       uint32_t n_tiles, uint32_t total_tiles, uint32_t srcs_per_buffer, uint32_t narrow_shift, uint32_t tiles_per_xcd_turn) {
  const uint32_t s = narrow_shift;
  constexpr uint32_t kTileGroups = kBlockThreads * U;
  // a tile's 256 lanes may be spread over several smaller workgroups: lane = part * THREADS + threadIdx.x
  constexpr uint32_t kParts = kBlockThreads / THREADS;
  const uint32_t n_slots = total_tiles * kParts;
  // Workgroups whose ids are congruent mod 8 run on one XCD.  With tiles_per_xcd_turn = 4 the workgroups of a tile, and
  // of the four tiles whose entries share a 64-byte line of the tile table, are handed ids 8 apart: one XCD's L2 then
  // fetches that line once instead of every L2 fetching every line (6 % more bytes read otherwise), and consecutive
  // XCDs take consecutive 16 KiB of the copy.  Slots behind the last whole group keep the plain order, as do all
  // slots with tiles_per_xcd_turn = 0.
  constexpr uint32_t kXcds = 8;
  const uint32_t kGroup = kXcds * tiles_per_xcd_turn * kParts;
  const uint32_t grouped = tiles_per_xcd_turn == 0 ? 0 : n_slots / kGroup * kGroup;
  for (uint32_t slot = blockIdx.x; slot < n_slots; slot += gridDim.x) {
    uint32_t T = slot / kParts, part = slot % kParts;
    if (slot < grouped) {
      const uint32_t in_group = slot % kGroup, index = in_group / kXcds;  // index: this XCD's share of the group
      T = (slot / kGroup * kXcds + in_group % kXcds) * tiles_per_xcd_turn + index / kParts;
      part = index % kParts;
    }
    const uint32_t tile_lane = part * THREADS + threadIdx.x;
    uint32_t b = 0, t = T;
    if (total_tiles != n_tiles) {
      b = T / n_tiles;
      t = T - b * n_tiles;
    }
    // with one source per buffer its base pointer does not depend on the tile: fetched beside the tile, not behind it
    const char* only_source = srcs.p[b];
    char* dst = dsts.p[b];
    const DevTile tile = tiles[t];
    if (!(tile.a & kTileGeneric)) {
      const uint32_t id1 = static_cast<uint32_t>(tile.a >> 48);
      const char* sbase = id1 == 0 ? nullptr : (srcs_per_buffer == 1 ? only_source : srcs.p[b * srcs_per_buffer + id1 - 1]);
      const int64_t soff = static_cast<int64_t>(tile.a & kTileOffsetMask) << s;
      const int64_t doff = static_cast<int64_t>(tile.b & kTileOffsetMask) << s;
      const uint32_t n_groups = static_cast<uint32_t>(tile.b >> 48) << s;
      for (uint32_t first = 0; first < n_groups; first += kTileGroups) {
        Words<SRC_B> data[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t g = first + u * kBlockThreads + tile_lane;
          if (g < n_groups && sbase != nullptr) {
            data[u] = load_bytes<SRC_B, NT>(sbase + (soff + g) * SRC_B);
          } else {
#pragma unroll
            for (int i = 0; i < (SRC_B + 3) / 4; ++i) data[u].w[i] = 0;
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t g = first + u * kBlockThreads + tile_lane;
          if (g < n_groups) store_bytes<DST_B, NTS>(dst + (doff + g) * DST_B, convert_group<SRC_B, DST_B, HALF>(data[u]));
        }
      }
      continue;
    }
    const DevRun run = runs[static_cast<uint32_t>(tile.a)];
    const uint32_t tile_index = static_cast<uint32_t>(tile.b);
    const char* sbase = run.src_id >= 0 ? srcs.p[b * srcs_per_buffer + run.src_id] : nullptr;
    const uint32_t n_groups = run.n_groups << s;
    for (uint32_t sub = 0; sub < (1u << s); ++sub) {
      const uint32_t first = ((tile_index << s) + sub) * kTileGroups;
      if (first >= n_groups) break;
      Words<SRC_B> data[U];
      int64_t doff[U];
      bool live[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t g = first + u * kBlockThreads + tile_lane;
        live[u] = g < n_groups;
        uint32_t row = 0, col = g;
        if (run.multi_row) {
          const uint32_t natural = g >> s;
          row = run.row_groups == 1 ? natural : (__umulhi(run.magic, natural) >> run.shift);
          col = g - ((row * run.row_groups) << s);
        }
        doff[u] = (run.dst_off << s) + static_cast<int64_t>(row) * (run.dst_stride << s) + col;
        if (live[u] && sbase != nullptr) {
          const int64_t soff = (run.src_off << s) + static_cast<int64_t>(row) * (run.src_stride << s) + col;
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
}

// Launch tuning.  Set through the C ABI from any thread while other threads launch: plain atomics, every launch
// reads each field once.
struct Tuning {
  std::atomic<int> blocks_per_cu{-1};  // -1: library default, 0: one workgroup per tile (no grid-stride), n > 0: persistent grid of n per CU
  std::atomic<int> nontemporal{1};
  std::atomic<int> block_threads{0};  // threads per workgroup: 64, 128 or 256 (a tile's 256 lanes over 4, 2 or 1 workgroups); 0: default
  std::atomic<int> unroll{0};  // loads in flight per lane: 1, 2 or 4; 0: library default per kernel
  // elements per lane when converting: 4 keeps the wider side at one 16-byte access per lane, so that every wave-level
  // access is one contiguous span (8 elements would make the 32-byte side two half-dense accesses: 51 % vs 67 % of HBM peak)
  static constexpr int convert_group = 4;
};
Tuning g_tuning;

bool is_half_conversion(int convert) { return convert == MFSDP_CONVERT_F16_TO_F32 || convert == MFSDP_CONVERT_F32_TO_F16; }

// ---- host side -------------------------------------------------------------------------------

// Tables of one launch: the runs of one natural vector width whose sources fall into one block of kMaxSources.
struct Compiled {
  int group_units = 0;   // natural group width G, in units
  int source_base = 0;   // first source id the launch's pointer table holds (a multiple of kMaxSources)
  int n_sources = 0;     // pointers per buffer in that table
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
  std::vector<mfsdp_copy_run> runs;  // validated, rows>=1, row_len>=1, in units
  std::vector<int64_t> src_numels;
  int64_t dst_numel = 0;
  int convert = 0;
  int src_unit = 1;  // bytes per unit on the source side
  int dst_unit = 1;
  int max_group = 16;  // widest vector group in units
  int64_t bytes_moved = 0;
  int device = 0;
  std::vector<Compiled> compiled;  // built once at create time; run() only reads it
};

namespace {

void free_compiled(std::vector<Compiled>& v) {
  for (auto& c : v) {
    if (c.runs) (void)hipFree(c.runs);
    if (c.tiles) (void)hipFree(c.tiles);
  }
  v.clear();
}

// Builds the device tables: runs bucketed by (natural vector width, block of kMaxSources sources), one tile per workgroup.
int compile_tables(mfsdp_segment_program* prog, std::vector<Compiled>* out) {
  int unroll = g_tuning.unroll.load(std::memory_order_relaxed);
  // plain copies: one 16-byte load per lane (pack / unpack of the hidden4096 block layout with workgroups of one
  // wavefront: 6.56 / 6.39 TB/s against 6.22 / 6.14 with two loads; with 256 threads 6.06 / 6.20); converting programs move
  // half as much on their narrow side and like two (bf16 -> fp32 gradient fill of the hidden2048 layer 6.09 against 6.00)
  if (unroll != 1 && unroll != 2 && unroll != 4) unroll = prog->src_unit != prog->dst_unit ? 2 : 1;
  const uint32_t tile_groups = kBlockThreads * unroll;
  std::map<std::pair<int, int>, std::pair<std::vector<DevRun>, std::vector<DevTile>>> buckets;
  for (const auto& r : prog->runs) {
    int64_t g = prog->max_group;
    g = gcd_pow2(r.row_len, g);
    g = gcd_pow2(r.dst_off, g);
    if (r.src_id >= 0) g = gcd_pow2(r.src_off, g);
    if (r.rows > 1) {
      g = gcd_pow2(r.dst_stride, g);
      if (r.src_id >= 0) g = gcd_pow2(r.src_stride, g);
    }
    const int block = r.src_id >= 0 ? r.src_id / kMaxSources : 0;
    auto& bucket = buckets[{static_cast<int>(g), block}];
    const int64_t row_groups = r.row_len / g;
    const int32_t local_id = r.src_id >= 0 ? r.src_id - block * kMaxSources : -1;
    const int64_t src_off = r.src_id >= 0 ? r.src_off / g : 0, dst_off = r.dst_off / g;
    const int64_t src_stride = r.rows > 1 && r.src_id >= 0 ? r.src_stride / g : 0, dst_stride = r.rows > 1 ? r.dst_stride / g : 0;
    if (r.rows == 1 || row_groups >= tile_groups / 2) {
      // direct tiles: every row is cut into equal pieces of at most one tile, a multiple of 128 bytes long where
      // the row allows it, so that no workgroup is left with a sliver
      // Zero fill only stores: a wavefront that writes 1 KiB is gone before the next can be dispatched and the launch
      // runs at the dispatch rate (pad tails of the hidden5120 owner layouts: 4.2-4.6 TB/s); eight times the span per
      // workgroup, walked in the kernel's loop over a direct tile, lifts the fill to 5.3 TB/s (pack of such a layer
      // buffer 6.09 TB/s against 5.55-5.78; 32 spans no better; fill tiles spread evenly among the copying tiles
      // instead of behind each rank's segments: slower, 5.85-5.95).
      const int64_t tile_cap = r.src_id < 0 ? kFillTileSpans * tile_groups : tile_groups;
      const int64_t per_row = (row_groups + tile_cap - 1) / tile_cap;
      const int64_t piece = std::min<int64_t>(tile_cap, ((row_groups + per_row - 1) / per_row + 7) / 8 * 8);
      for (int64_t row = 0; row < r.rows; ++row) {
        for (int64_t col = 0; col < row_groups; col += piece) {
          const uint64_t n = static_cast<uint64_t>(std::min(piece, row_groups - col));
          bucket.second.push_back(DevTile{static_cast<uint64_t>(src_off + row * src_stride + col) | (static_cast<uint64_t>(local_id + 1) << 48),
                                          static_cast<uint64_t>(dst_off + row * dst_stride + col) | (n << 48)});
        }
      }
      continue;
    }
    // generic tiles: short rows, several per tile; a device run holds fewer than 2^31 units so that the reciprocal
    // division stays exact at any vector width (row_groups < tile_groups here, so only the row count is ever cut)
    const int64_t rows_per_part = std::max<int64_t>(1, kMaxUnitsPerRun / g / row_groups);
    for (int64_t row0 = 0; row0 < r.rows; row0 += rows_per_part) {
      const int64_t nrows = std::min(rows_per_part, r.rows - row0);
      DevRun d{};
      d.src_off = src_off + row0 * src_stride;
      d.dst_off = dst_off + row0 * dst_stride;
      d.src_stride = nrows > 1 ? src_stride : 0;
      d.dst_stride = nrows > 1 ? dst_stride : 0;
      d.row_groups = static_cast<uint32_t>(row_groups);
      d.n_groups = static_cast<uint32_t>(row_groups * nrows);
      d.multi_row = nrows > 1 ? 1u : 0u;
      d.src_id = local_id;
      d.magic = 0;
      d.shift = 0;
      if (d.multi_row && d.row_groups > 1) reciprocal(d.row_groups, &d.magic, &d.shift);
      const uint64_t run_index = bucket.first.size();
      bucket.first.push_back(d);
      const uint32_t ntiles = (d.n_groups + tile_groups - 1) / tile_groups;
      for (uint32_t t = 0; t < ntiles; ++t) bucket.second.push_back(DevTile{kTileGeneric | run_index, t});
    }
  }
  const int n_srcs = static_cast<int>(prog->src_numels.size());
  for (auto& kv : buckets) {
    Compiled c;
    c.group_units = kv.first.first;
    c.source_base = kv.first.second * kMaxSources;
    c.n_sources = std::max(0, std::min(kMaxSources, n_srcs - c.source_base));
    c.unroll = unroll;
    auto& runs = kv.second.first;
    auto& tiles = kv.second.second;
    if (tiles.size() > 0xffffffffull) {
      free_compiled(*out);
      return fail(MFSDP_ERR_UNSUPPORTED, "segment program needs %zu tiles, more than one launch can address", tiles.size());
    }
    c.n_tiles = static_cast<uint32_t>(tiles.size());
    hipError_t e = hipSuccess;
    if (!runs.empty()) e = hipMalloc(reinterpret_cast<void**>(&c.runs), runs.size() * sizeof(DevRun));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&c.tiles), tiles.size() * sizeof(DevTile));
    if (e == hipSuccess && !runs.empty()) e = hipMemcpy(c.runs, runs.data(), runs.size() * sizeof(DevRun), hipMemcpyHostToDevice);
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
int launch_one(const Compiled& c, const SourceTable& srcs, const DestTable& dsts, uint32_t batch, uint32_t narrow_shift,
               hipStream_t stream) {
  const int cus = device_cu_count();
  const uint64_t total64 = static_cast<uint64_t>(c.n_tiles) * batch;
  if (total64 > 0xffffffffull) return fail(MFSDP_ERR_UNSUPPORTED, "a batch of %u buffers needs %llu tiles, more than one launch can address", batch, static_cast<unsigned long long>(total64));
  const uint32_t total = static_cast<uint32_t>(total64);
  int threads = g_tuning.block_threads.load(std::memory_order_relaxed);
  if (threads != 64 && threads != 128 && threads != 256) threads = kDefaultBlockThreads;
  const uint64_t want64 = static_cast<uint64_t>(total) * (kBlockThreads / threads);
  if (want64 > static_cast<uint64_t>(kMaxGrid)) return fail(MFSDP_ERR_UNSUPPORTED, "launch of %llu workgroups is beyond the grid limit", static_cast<unsigned long long>(want64));
  const uint32_t want = static_cast<uint32_t>(want64);
  int per_cu = g_tuning.blocks_per_cu.load(std::memory_order_relaxed);
  if (per_cu < 0) per_cu = kDefaultBlocksPerCu;
  const uint32_t cap = per_cu == 0 ? want : static_cast<uint32_t>(std::min<uint64_t>(static_cast<uint64_t>(cus) * per_cu, kMaxGrid));
  const dim3 grid(std::max(1u, std::min(want, cap)));
  // one buffer: XCD-grouped workgroup order (exact read traffic, pack + unpack 6.41 against 6.38 TB/s); several buffers
  // in one grid run faster in the plain order (hidden2048: 6.51 against 6.26 TB/s, the widening fill 6.32 against 5.83)
  const uint32_t tpl = batch == 1 ? 4u : 0u;
  const int nt = g_tuning.nontemporal.load(std::memory_order_relaxed);  // 0 none, 1 loads and stores, 2 loads only, 3 stores only
#define MFSDP_LAUNCH(U_, NTL_, NTS_, T_)                                                                                  \
  hipLaunchKernelGGL((segment_program_kernel<SRC_B, DST_B, U_, NTL_, NTS_, HALF, T_>), grid, dim3(T_), 0, stream, srcs, dsts, \
                     c.runs, c.tiles, c.n_tiles, total, static_cast<uint32_t>(c.n_sources), narrow_shift, tpl)
#define MFSDP_LAUNCH_T(U_, NTL_, NTS_)                                        \
  if (threads == 64) MFSDP_LAUNCH(U_, NTL_, NTS_, 64);                        \
  else if (threads == 128) MFSDP_LAUNCH(U_, NTL_, NTS_, 128);                 \
  else MFSDP_LAUNCH(U_, NTL_, NTS_, kBlockThreads)
#define MFSDP_LAUNCH_NT(U_)                        \
  switch (nt) {                                    \
    case 0: MFSDP_LAUNCH_T(U_, false, false); break; \
    case 2: MFSDP_LAUNCH_T(U_, true, false); break;  \
    case 3: MFSDP_LAUNCH_T(U_, false, true); break;  \
    default: MFSDP_LAUNCH_T(U_, true, true); break;  \
  }
  switch (c.unroll) {
    case 2: MFSDP_LAUNCH_NT(2) break;
    case 4: MFSDP_LAUNCH_NT(4) break;
    default: MFSDP_LAUNCH_NT(1) break;
  }
#undef MFSDP_LAUNCH_NT
#undef MFSDP_LAUNCH_T
#undef MFSDP_LAUNCH
  MFSDP_CHECK_LAUNCH("segment_program_kernel");
  return MFSDP_OK;
}

// `cap` is the widest group (in units) the base pointers of this launch allow.
int launch_compiled(const mfsdp_segment_program* prog, const Compiled& c, const SourceTable& srcs, const DestTable& dsts,
                    uint32_t batch, int cap, hipStream_t stream) {
  if (c.n_tiles == 0) return MFSDP_OK;
  const int group = std::min(c.group_units, cap);
  uint32_t narrow_shift = 0;
  while ((group << narrow_shift) < c.group_units) ++narrow_shift;
  const int sb = group * prog->src_unit;
  const int db = group * prog->dst_unit;
#define MFSDP_CASE(S_, D_) \
  if (sb == S_ && db == D_) return launch_one<S_, D_>(c, srcs, dsts, batch, narrow_shift, stream)
#define MFSDP_CONVERTING(S_, D_) \
  if (sb == S_ && db == D_) return half ? launch_one<S_, D_, true>(c, srcs, dsts, batch, narrow_shift, stream) : launch_one<S_, D_, false>(c, srcs, dsts, batch, narrow_shift, stream)
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
      *src_unit = 2; *dst_unit = 4; *max_group = Tuning::convert_group; *scale = 1;
      return MFSDP_OK;
    case MFSDP_CONVERT_F32_TO_BF16:
    case MFSDP_CONVERT_F32_TO_F16:
      *src_unit = 4; *dst_unit = 2; *max_group = Tuning::convert_group; *scale = 1;
      return MFSDP_OK;
    default:
      return fail(MFSDP_ERR_INVALID, "unknown conversion code %d", convert);
  }
}

// Do any two destination rows of the runs overlap?  Every run is a sequence of disjoint row intervals in
// increasing order (dst_stride >= row_len), so a k-way merge by row start visits the intervals in address order
// and only neighbours need comparing; a run whose remaining rows all end before the next run's current row is
// dropped in one step, rows that end before it are skipped arithmetically, so runs that do not interleave cost
// O(log n) each and interleaved ones (column blocks of one matrix) one step per row.
bool find_destination_overlap(const std::vector<mfsdp_copy_run>& runs, int64_t* where) {
  struct Cursor {
    int64_t start;  // start of the current row
    size_t run;
    int64_t row;
  };
  auto later = [](const Cursor& a, const Cursor& b) { return a.start > b.start; };
  std::priority_queue<Cursor, std::vector<Cursor>, decltype(later)> heap(later);
  for (size_t i = 0; i < runs.size(); ++i) heap.push(Cursor{runs[i].dst_off, i, 0});
  while (!heap.empty()) {
    Cursor c = heap.top();
    heap.pop();
    if (heap.empty()) return false;
    const mfsdp_copy_run& r = runs[c.run];
    const int64_t next_start = heap.top().start;
    if (c.start + r.row_len > next_start) {
      *where = next_start;
      return true;
    }
    if (c.row + 1 >= r.rows) continue;
    const int64_t last_end = r.dst_off + (r.rows - 1) * r.dst_stride + r.row_len;
    if (last_end <= next_start) continue;  // the whole rest of this run lies before every other run's current row
    // skip the rows that end at or before next_start: off + k * stride + len <= next_start
    int64_t k = c.row + 1;
    const int64_t room = next_start - r.dst_off - r.row_len;
    if (room >= 0) k = std::max(k, room / r.dst_stride + 1);
    if (k >= r.rows) continue;
    heap.push(Cursor{r.dst_off + k * r.dst_stride, c.run, k});
  }
  return false;
}

}  // namespace

extern "C" void mfsdp_set_copy_tuning(int blocks_per_cu, int nontemporal, int unroll, int block_threads) {
  g_tuning.block_threads.store((block_threads == 64 || block_threads == 128 || block_threads == 256) ? block_threads : 0, std::memory_order_relaxed);
  g_tuning.blocks_per_cu.store(blocks_per_cu < 0 ? -1 : blocks_per_cu, std::memory_order_relaxed);
  g_tuning.nontemporal.store((nontemporal < 0 || nontemporal > 3) ? 1 : nontemporal, std::memory_order_relaxed);
  g_tuning.unroll.store((unroll == 1 || unroll == 2 || unroll == 4) ? unroll : 0, std::memory_order_relaxed);
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
  if (n_srcs < 0) return fail(MFSDP_ERR_INVALID, "n_srcs must be non-negative, got %d", n_srcs);
  if (n_srcs > 0 && src_numels == nullptr) return fail(MFSDP_ERR_INVALID, "src_numels is null");
  if (dst_numel < 0) return fail(MFSDP_ERR_INVALID, "dst_numel must be non-negative");
  int src_unit, dst_unit, max_group, scale;
  if (int rc = setup_units(convert, elem_bytes, &src_unit, &dst_unit, &max_group, &scale)) return rc;
  for (int32_t i = 0; i < n_srcs; ++i)
    if (src_numels[i] < 0) return fail(MFSDP_ERR_INVALID, "src_numels[%d] is negative", i);

  std::unique_ptr<mfsdp_segment_program> prog(new mfsdp_segment_program());
  prog->convert = convert;
  prog->src_unit = src_unit;
  prog->dst_unit = dst_unit;
  prog->max_group = max_group;
  prog->dst_numel = dst_numel * scale;
  for (int32_t i = 0; i < n_srcs; ++i) prog->src_numels.push_back(src_numels[i] * scale);
  (void)hipGetDevice(&prog->device);

  for (int64_t i = 0; i < n_runs; ++i) {
    mfsdp_copy_run r = runs[i];
    if (r.rows < 0 || r.row_len < 0) return fail(MFSDP_ERR_INVALID, "run %lld: negative size", static_cast<long long>(i));
    if (r.rows == 0 || r.row_len == 0) continue;
    if (r.src_id >= n_srcs) return fail(MFSDP_ERR_INVALID, "run %lld: src_id %d out of range", static_cast<long long>(i), r.src_id);
    if (r.src_id < 0) r.src_id = -1;
    if (r.rows == 1) r.src_stride = r.dst_stride = 0;
    if (r.rows > 1 && (r.dst_stride < r.row_len || (r.src_id >= 0 && r.src_stride < 0)))
      return fail(MFSDP_ERR_INVALID, "run %lld: destination rows overlap or negative source pitch", static_cast<long long>(i));
    const int64_t dst_last = r.dst_off + (r.rows - 1) * r.dst_stride + r.row_len;
    if (r.dst_off < 0 || dst_last > dst_numel)
      return fail(MFSDP_ERR_INVALID, "run %lld: destination range [%lld, %lld) leaves the output of %lld elements",
                  static_cast<long long>(i), static_cast<long long>(r.dst_off), static_cast<long long>(dst_last),
                  static_cast<long long>(dst_numel));
    if (r.src_id >= 0) {
      const int64_t src_last = r.src_off + (r.rows - 1) * r.src_stride + r.row_len;
      if (r.src_off < 0 || src_last > src_numels[r.src_id])
        return fail(MFSDP_ERR_INVALID, "run %lld: source range [%lld, %lld) leaves source %d of %lld elements",
                    static_cast<long long>(i), static_cast<long long>(r.src_off), static_cast<long long>(src_last),
                    r.src_id, static_cast<long long>(src_numels[r.src_id]));
    }
    prog->bytes_moved += r.rows * r.row_len * ((r.src_id >= 0 ? src_unit : 0) + dst_unit) * scale;
    // to units
    r.src_off *= scale; r.dst_off *= scale; r.row_len *= scale; r.src_stride *= scale; r.dst_stride *= scale;
    prog->runs.push_back(r);
  }
  // The reference's sequential slice writes make overlapping destinations well defined (the last one wins); the
  // waves of one launch write in no particular order, so a program whose runs overlap is refused.
  int64_t where = 0;
  if (find_destination_overlap(prog->runs, &where))
    return fail(MFSDP_ERR_INVALID, "two runs write destination offset %lld", static_cast<long long>(where / scale));
  if (int rc = compile_tables(prog.get(), &prog->compiled)) return rc;
  *out = prog.release();
  return MFSDP_OK;
}

extern "C" void mfsdp_segment_program_destroy(mfsdp_segment_program* program) {
  if (program == nullptr) return;
  free_compiled(program->compiled);
  delete program;
}

extern "C" int64_t mfsdp_segment_program_bytes(const mfsdp_segment_program* program) {
  return program ? program->bytes_moved : 0;
}

extern "C" int64_t mfsdp_segment_program_num_runs(const mfsdp_segment_program* program) {
  return program ? static_cast<int64_t>(program->runs.size()) : 0;
}

extern "C" int mfsdp_segment_program_run_many(mfsdp_segment_program* program, int32_t n_buffers, const void* const* srcs,
                                              int32_t n_srcs, void* const* dsts, void* stream) {
  if (program == nullptr) return fail(MFSDP_ERR_INVALID, "program is null");
  if (n_buffers < 0) return fail(MFSDP_ERR_INVALID, "n_buffers must be non-negative");
  if (n_srcs != static_cast<int32_t>(program->src_numels.size()))
    return fail(MFSDP_ERR_INVALID, "program was created for %zu sources, got %d", program->src_numels.size(), n_srcs);
  if (program->runs.empty() || n_buffers == 0) return MFSDP_OK;
  if (dsts == nullptr || (n_srcs > 0 && srcs == nullptr)) return fail(MFSDP_ERR_INVALID, "pointer array is null");
  // the narrowest alignment among all base pointers decides the vector width of every launch
  int cap = program->max_group;
  for (int32_t b = 0; b < n_buffers; ++b) {
    if (dsts[b] == nullptr) return fail(MFSDP_ERR_INVALID, "dst is null (buffer %d)", b);
    cap = std::min(cap, pointer_alignment_units(dsts[b], program->dst_unit, program->max_group));
    for (int32_t i = 0; i < n_srcs; ++i) {
      const void* p = srcs[static_cast<int64_t>(b) * n_srcs + i];
      if (program->src_numels[i] == 0) continue;
      if (p == nullptr) return fail(MFSDP_ERR_INVALID, "source %d is null (buffer %d)", i, b);
      cap = std::min(cap, pointer_alignment_units(p, program->src_unit, program->max_group));
    }
  }
  hipStream_t s = as_stream(stream);
  for (const auto& c : program->compiled) {
    // buffers per launch: both pointer tables travel by value in the kernel arguments
    const int32_t per_launch = std::min<int32_t>(kMaxBatch, kMaxSources / std::max(1, c.n_sources));
    for (int32_t b0 = 0; b0 < n_buffers; b0 += per_launch) {
      const int32_t batch = std::min(per_launch, n_buffers - b0);
      SourceTable st;
      DestTable dt;
      std::memset(&st, 0, sizeof(st));
      std::memset(&dt, 0, sizeof(dt));
      for (int32_t b = 0; b < batch; ++b) {
        dt.p[b] = static_cast<char*>(dsts[b0 + b]);
        for (int i = 0; i < c.n_sources; ++i)
          st.p[b * c.n_sources + i] = static_cast<const char*>(srcs[static_cast<int64_t>(b0 + b) * n_srcs + c.source_base + i]);
      }
      if (int rc = launch_compiled(program, c, st, dt, static_cast<uint32_t>(batch), cap, s)) return rc;
    }
  }
  return MFSDP_OK;
}

extern "C" int mfsdp_segment_program_run(mfsdp_segment_program* program, const void* const* srcs, int32_t n_srcs,
                                         void* dst, void* stream) {
  if (program == nullptr) return fail(MFSDP_ERR_INVALID, "program is null");
  if (dst == nullptr && !program->runs.empty()) return fail(MFSDP_ERR_INVALID, "dst is null");
  void* const dsts[1] = {dst};
  return mfsdp_segment_program_run_many(program, 1, srcs, n_srcs, dsts, stream);
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

// Threads per workgroup of the contiguous streaming kernels below (they index with blockDim.x).
int stream_threads() {
  const int threads = g_tuning.block_threads.load(std::memory_order_relaxed);
  return (threads == 64 || threads == 128 || threads == 256) ? threads : kDefaultBlockThreads;
}

// dst[g] = convert(src[g]) over n_groups contiguous vector groups.
template <int SRC_B, int DST_B, int U, bool NT, bool HALF = false>
__global__ void __launch_bounds__(kBlockThreads)
linear_kernel(const char* __restrict__ src, char* __restrict__ dst, int64_t n_groups) {
  const int64_t span = static_cast<int64_t>(blockDim.x) * U;
  for (int64_t base = static_cast<int64_t>(blockIdx.x) * span; base < n_groups;
       base += static_cast<int64_t>(gridDim.x) * span) {
    Words<SRC_B> data[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t g = base + u * blockDim.x + threadIdx.x;
      if (g < n_groups) data[u] = load_bytes<SRC_B, NT>(src + g * SRC_B);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t g = base + u * blockDim.x + threadIdx.x;
      if (g < n_groups) store_bytes<DST_B, NT>(dst + g * DST_B, convert_group<SRC_B, DST_B, HALF>(data[u]));
    }
  }
}

template <int SRC_B, int DST_B, bool HALF = false>
int launch_linear(const char* src, char* dst, int64_t n_groups, hipStream_t stream) {
  if (n_groups <= 0) return MFSDP_OK;
  // one workgroup per block of the tensor, not a persistent grid: workgroups are dispatched in order, so those in
  // flight sweep neighbouring addresses (bf16 -> fp32 of 202 M elements 5.83 against 5.65 TB/s with 16 per CU)
  // workgroups of one wavefront, one 16-byte load per lane for a plain copy (202 M bf16 elements: 6.55 TB/s; two loads 6.39,
  // four 6.21; 256 threads: 6.42 / 6.13 / 5.91), two for the conversions (bf16 -> fp32 6.44 against 6.23, fp32 -> bf16
  // 6.60 against 6.08)
  int unroll = g_tuning.unroll.load(std::memory_order_relaxed);
  if (unroll != 1 && unroll != 2 && unroll != 4) unroll = SRC_B != DST_B ? 2 : 1;
  const bool nt = g_tuning.nontemporal.load(std::memory_order_relaxed) != 0;
  auto go = [&](auto u_tag) {
    constexpr int U = decltype(u_tag)::value;
    const int threads = stream_threads();
    const int64_t span = static_cast<int64_t>(threads) * U;
    const int64_t want = (n_groups + span - 1) / span;
    const dim3 grid(static_cast<uint32_t>(std::max<int64_t>(1, std::min(want, kMaxGrid))));
    if (nt) hipLaunchKernelGGL((linear_kernel<SRC_B, DST_B, U, true, HALF>), grid, dim3(threads), 0, stream, src, dst, n_groups);
    else hipLaunchKernelGGL((linear_kernel<SRC_B, DST_B, U, false, HALF>), grid, dim3(threads), 0, stream, src, dst, n_groups);
  };
  if (unroll == 1) go(std::integral_constant<int, 1>{});
  else if (unroll == 2) go(std::integral_constant<int, 2>{});
  else go(std::integral_constant<int, 4>{});
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
                         Tuning::convert_group, as_stream(stream), is_half_conversion(convert));
}

// ---- HBM probes: what the part sustains for pure reads and pure writes, measured with this library's own launch shape
// (one workgroup of 256 threads per 4 KiB, non-temporal accesses) so that a copy's rate can be read against them.

namespace {

__global__ void __launch_bounds__(kBlockThreads)
probe_read_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ sink, int64_t n_groups) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (g >= n_groups) return;
  const u32x4 v = __builtin_nontemporal_load(src + g);
  // never true for the probe's input (the caller fills it with small values); keeps the load alive
  if ((v.x & v.y & v.z & v.w) == 0xffffffffu) sink[threadIdx.x] = v;
}

__global__ void __launch_bounds__(kBlockThreads)
probe_write_kernel(u32x4* __restrict__ dst, int64_t n_groups) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (g >= n_groups) return;
  const u32x4 v = {1u, 2u, 3u, 4u};
  __builtin_nontemporal_store(v, dst + g);
}

}  // namespace

extern "C" int mfsdp_hbm_probe(int kind, const void* src, void* dst, int64_t bytes, void* stream) {
  if (kind != 0 && kind != 1) return fail(MFSDP_ERR_INVALID, "probe kind must be 0 (read) or 1 (write), got %d", kind);
  if (bytes < 4096 || bytes % 16) return fail(MFSDP_ERR_INVALID, "probe size must be a multiple of 16 bytes, at least 4096");
  if (dst == nullptr || (kind == 0 && src == nullptr)) return fail(MFSDP_ERR_INVALID, "null pointer");
  if ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) % 16) return fail(MFSDP_ERR_INVALID, "probe buffers must be 16-byte aligned");
  const int64_t n_groups = bytes / 16;
  // one-directional passes are limited by the rate at which workgroups can be dispatched when each of them moves
  // only 1 KiB (4.3 / 4.6 TB/s with 64 threads against 6.9 / 6.6 with 256); a copy holds its workgroups twice as long
  const int threads = kBlockThreads;
  const int64_t want = (n_groups + threads - 1) / threads;
  if (want > kMaxGrid) return fail(MFSDP_ERR_UNSUPPORTED, "probe size beyond one launch");
  const dim3 grid(static_cast<uint32_t>(want));
  if (kind == 0)
    hipLaunchKernelGGL(probe_read_kernel, grid, dim3(threads), 0, as_stream(stream), static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), n_groups);
  else
    hipLaunchKernelGGL(probe_write_kernel, grid, dim3(threads), 0, as_stream(stream), static_cast<u32x4*>(dst), n_groups);
  MFSDP_CHECK_LAUNCH("probe kernel");
  return MFSDP_OK;
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
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t g = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; g < n_vec; g += stride) {
    const Words<16> b = load_bytes<16, true>(src + g * 16);
    Words<16> a = load_bytes<16, false>(dst + g * 16);
#pragma unroll
    for (int i = 0; i < 4; ++i) a.w[i] = add_word<FMT>(a.w[i], b.w[i]);
    store_bytes<16, false>(dst + g * 16, a);
  }
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < tail; i += stride) {
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
  const int threads = stream_threads();
  const int64_t want = (work + threads - 1) / threads;
  // one workgroup per block, as launch_linear: 6.27 against 4.78 TB/s with 16 persistent workgroups per CU (fp32, 202 M elements)
  const dim3 grid(static_cast<uint32_t>(std::max<int64_t>(1, std::min(want, kMaxGrid))));
  char* d = static_cast<char*>(dst);
  const char* s = static_cast<const char*>(src);
  if (dtype == MFSDP_F32) hipLaunchKernelGGL((accumulate_kernel<0>), grid, dim3(threads), 0, as_stream(stream), d, s, n_vec, tail_first, tail);
  else if (dtype == MFSDP_BF16) hipLaunchKernelGGL((accumulate_kernel<1>), grid, dim3(threads), 0, as_stream(stream), d, s, n_vec, tail_first, tail);
  else hipLaunchKernelGGL((accumulate_kernel<2>), grid, dim3(threads), 0, as_stream(stream), d, s, n_vec, tail_first, tail);
  MFSDP_CHECK_LAUNCH("accumulate_kernel");
  return MFSDP_OK;
}
