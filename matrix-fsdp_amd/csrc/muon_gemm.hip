// bf16 MFMA GEMM for the Newton-Schulz iteration: C = bf16(alpha * P Q^T + beta * D) on gfx950.
//
// Both operands are K-contiguous (an "NT" product), which is what every Newton-Schulz product
// reduces to once X and X^T are both kept: X X^T, A A^T (A symmetric) and B (X^T)^T.  A workgroup owns
// a BM x BN tile of C; its waves each own a (BM/WM) x (BN/WN) sub-tile built from 16x16x32 bf16 MFMAs
// with fp32 accumulators.  K is walked in slabs of BK = 64: the slab of P and Q is staged in LDS as
// rows of BK bf16 whose 16-byte chunks are XOR-swizzled with the row index: the LDS has 64 banks of 4
// bytes, 256 / (2 BK) rows span them once, so any 16 consecutive rows read at one logical chunk touch every
// bank exactly once and the 128-bit fragment reads are bank-conflict free.  STAGES slabs are resident: the
// next ones stream from HBM straight into LDS (buffer_load ... lds, no register round trip) while the
// current one feeds the MFMAs.
//
// Tile scheduling.  Tiles are handed to workgroups so that the groups sharing an XCD (block ids
// congruent mod 8) work on neighbouring tiles and reuse that XCD's L2, whatever the tile count.  When the tile count is not a
// multiple of the number of resident workgroups, the tiles of the last, partial round are split along
// K into pieces that fill the machine once more for a fraction of a tile's time; each piece leaves an
// fp32 partial tile in a workspace and a small fix-up kernel sums the pieces in split order and runs
// the epilogue (the kernel boundary is the only synchronisation: no fences, no spinning).
#include "muon_gemm.h"

#include "mfsdp_common.h"

#include <algorithm>
#include <mutex>
#include <type_traits>
#include <utility>

namespace mfsdp {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kXcds = 8;
constexpr int kSlabK = 64;  // K granularity of the schedule (operands are padded to it); a slab is BK <= 64 wide

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const __bf16 l = static_cast<__bf16>(lo);
  const __bf16 h = static_cast<__bf16>(hi);
  return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, l)) | (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, h)) << 16);
}

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) { return __uint_as_float(static_cast<uint32_t>(b) << 16); }

// param[prow][pcol .. pcol + count - 1] <- round(param * decay) + neg_lr * o for the first `count` bf16 values o of `eight`
// (those inside the parameter's update_rows x update_cols); a.update_vectors says that whole groups of eight may use
// 16-byte accesses.
__device__ __forceinline__ void update_param8(const GemmNtArgs& a, int prow, int pcol, const u32x4& eight, int count = 8) {
  if (prow >= a.update_rows || pcol >= a.update_cols) return;
  const int n = a.update_cols - pcol < count ? a.update_cols - pcol : count;
  const int64_t at = static_cast<int64_t>(prow) * a.update_cols + pcol;
  float o[8];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    o[2 * e] = __uint_as_float(eight[e] << 16);
    o[2 * e + 1] = __uint_as_float(eight[e] & 0xffff0000u);
  }
  const float decay = a.update_decay, neg_lr = a.update_neg_lr;
  if (a.update_dtype == MFSDP_F32) {
    float* p = static_cast<float*>(a.update_param) + at;
    if (n == 8 && a.update_vectors) {
      f32x4 lo = reinterpret_cast<const f32x4*>(p)[0], hi = reinterpret_cast<const f32x4*>(p)[1];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo[e] = lo[e] * decay + neg_lr * o[e];
        hi[e] = hi[e] * decay + neg_lr * o[4 + e];
      }
      reinterpret_cast<f32x4*>(p)[0] = lo;
      reinterpret_cast<f32x4*>(p)[1] = hi;
    } else {
      for (int e = 0; e < n; ++e) p[e] = p[e] * decay + neg_lr * o[e];
    }
  } else {
    uint16_t* p = static_cast<uint16_t*>(a.update_param) + at;
    auto one = [&](uint16_t old, float ov) {
      const float scaled = bf16_bits_to_float(__builtin_bit_cast(uint16_t, static_cast<__bf16>(bf16_bits_to_float(old) * decay)));
      return __builtin_bit_cast(uint16_t, static_cast<__bf16>(scaled + neg_lr * ov));
    };
    if (n == 8 && a.update_vectors) {
      u32x4 v = *reinterpret_cast<const u32x4*>(p);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        v[e] = static_cast<uint32_t>(one(static_cast<uint16_t>(v[e]), o[2 * e])) | (static_cast<uint32_t>(one(static_cast<uint16_t>(v[e] >> 16), o[2 * e + 1])) << 16);
      *reinterpret_cast<u32x4*>(p) = v;
    } else {
      for (int e = 0; e < n; ++e) p[e] = one(p[e], o[e]);
    }
  }
}

struct Schedule {
  int tiles_m, tiles_n;
  int full_tiles;   // tiles computed whole, one per workgroup (block ids [0, full_tiles))
  int splits;       // K pieces per remaining tile (block ids from full_tiles on); 1 when nothing remains
  float* partials;  // [remaining tiles][splits][BM][BN] fp32
  int group_m;      // tile rows per group of the general products' tile order
};

// logical tile index -> (tm, tn)
__device__ __forceinline__ void tile_coords(int group_m, int logical, int tiles_m, int tiles_n, bool symmetric, int* tm, int* tn) {
  if (symmetric) {
    // the lower triangle row by row: t = i(i+1)/2 + j, j <= i
    int i = static_cast<int>((__fsqrt_rn(8.0f * static_cast<float>(logical) + 1.0f) - 1.0f) * 0.5f);
    while ((i + 1) * (i + 2) / 2 <= logical) ++i;
    while (i * (i + 1) / 2 > logical) --i;
    *tm = i;
    *tn = logical - i * (i + 1) / 2;
    return;
  }
  // group_m tile rows at a time, walking down the rows before moving to the next tile column
  const int per_group = group_m * tiles_n;
  const int group = logical / per_group;
  const int first_m = group * group_m;
  const int rows = min(group_m, tiles_m - first_m);
  const int in_group = logical - group * per_group;
  *tm = first_m + in_group % rows;
  *tn = in_group / rows;
}

// OCC workgroups are meant to share a CU: the register budget per wave is set for OCC * WM * WN / 4 waves per SIMD.
template <int BM, int BN, int WM, int WN, int BK, int STAGES, int OCC>
__global__ void __launch_bounds__(WM * WN * 64, (OCC * WM * WN + 3) / 4)
gemm_nt_kernel(GemmNtArgs a, Schedule sched) {
  constexpr int kThreads = WM * WN * 64;
  constexpr int kWaves = WM * WN;
  constexpr int kWaveM = BM / WM;     // rows of C per wave
  constexpr int kWaveN = BN / WN;
  constexpr int TM = kWaveM / 16;     // 16x16 MFMA tiles per wave
  constexpr int TN = kWaveN / 16;
  constexpr int TMH = TM / 2;         // tile rows one half step covers
  constexpr int kChunks = BK / 8;               // 16-byte chunks per slab row (row = BK bf16)
  constexpr int kRowsPerSweep = 128 / BK;       // slab rows that together span the 64 LDS banks once (256 bytes)
  constexpr int kRowsPerLoad = 512 / BK;        // slab rows one wave-level 1 KiB load fills
  constexpr int kSteps = BK / 32;               // k32 MFMA steps per slab, each run as two half steps of TMH tile rows
  constexpr int kLoadsP = BM / kRowsPerLoad / kWaves, kLoadsQ = BN / kRowsPerLoad / kWaves;
  constexpr int kLoadsPerSlab = kLoadsP + kLoadsQ;  // direct-to-LDS loads one wave issues per slab
  static_assert(BM % (kRowsPerLoad * kWaves) == 0 && BN % (kRowsPerLoad * kWaves) == 0, "slab must divide over the waves");
  static_assert(kSteps % 2 == 0 && TM % 2 == 0 && STAGES >= 2 && (STAGES - 1) * kLoadsPerSlab < 64, "pipeline shape");
  constexpr int kStageElems = (BM + BN) * BK;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __bf16* smem = reinterpret_cast<__bf16*>(smem_raw);

  // ---- which tile, which K range
  const int block = blockIdx.x;
  const bool whole = block < sched.full_tiles;
  int logical, split = 0, piece_tile = 0;
  if (whole) {
    // workgroup ids congruent mod 8 run on one XCD: hand each XCD one contiguous eighth of the tile order (the first
    // full_tiles % 8 of them one tile more), so that the workgroups sharing an L2 work on neighbouring tiles
    const int xcd = block % kXcds, each = sched.full_tiles / kXcds, extra = sched.full_tiles % kXcds;
    logical = xcd * each + (xcd < extra ? xcd : extra) + block / kXcds;
  } else {
    const int piece = block - sched.full_tiles;
    piece_tile = piece / sched.splits;
    split = piece - piece_tile * sched.splits;
    logical = sched.full_tiles + piece_tile;
  }
  int tm, tn;
  tile_coords(sched.group_m, logical, sched.tiles_m, sched.tiles_n, a.symmetric != 0, &tm, &tn);
  const int row0 = tm * BM;
  const int col0 = tn * BN;
  const int k_slabs_total = a.K / BK;
  const int ks_begin = whole ? 0 : static_cast<int>(static_cast<int64_t>(k_slabs_total) * split / sched.splits);
  const int ks_end = whole ? k_slabs_total : static_cast<int>(static_cast<int64_t>(k_slabs_total) * (split + 1) / sched.splits);

  // Every tile walks its K range from its first slab on: the tiles of an XCD that share a panel then share its slabs in
  // L2 (walks that start at different slabs were measured 3 to 37 % slower).
  const int n_slabs = ks_end - ks_begin;
  auto k0_of = [&](int i) { return (ks_begin + i) * BK; };

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction: keeps LDS slab addresses scalar
  const int wave_m = wave / WN;
  const int wave_n = wave % WN;

  const __bf16* __restrict__ P = static_cast<const __bf16*>(a.P) + static_cast<int64_t>(row0) * a.ldp;
  const __bf16* __restrict__ Q = static_cast<const __bf16*>(a.Q) + static_cast<int64_t>(col0) * a.ldq;

  // ---- slab loader.  A slab row holds BK bf16 = kChunks 16-byte chunks; chunk c of row r is stored at chunk
  // position c ^ ((r / kRowsPerSweep) % kChunks).  One wave-level direct-to-LDS load fills 1 KiB = kRowsPerLoad
  // rows: lane l lands at row l / kChunks, position l % kChunks, and therefore fetches the global chunk the
  // swizzle maps there.  Wave w takes the row groups w, w + kWaves, ...
  // The loads are buffer loads: the tile's first row is the descriptor's base, a lane's offset inside a row group (row
  // l / kChunks, the chunk the swizzle maps to position l % kChunks) is one loop-invariant register per operand --
  // the swizzle term does not depend on which of the wave's row groups it is -- and everything that changes from
  // load to load (row group, k) is a scalar offset: no vector address arithmetic in the loop.
  static_assert((kWaves * kRowsPerLoad / kRowsPerSweep) % kChunks == 0, "the swizzle must repeat from one row group of a wave to the next");
  const int dl_row = wave * kRowsPerLoad + lane / kChunks;
  const int dl_chunk = (lane % kChunks) ^ ((dl_row / kRowsPerSweep) % kChunks);
  const uint32_t lane_offset_p = static_cast<uint32_t>(dl_row * a.ldp + dl_chunk * 8) * 2u;
  const uint32_t lane_offset_q = static_cast<uint32_t>(dl_row * a.ldq + dl_chunk * 8) * 2u;
  auto operand_rsrc = [](const __bf16* base, int64_t rows, int ld) {
    const int64_t bytes = rows * ld * 2;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<__bf16*>(base), 0, static_cast<int>(bytes < 0x7fffffff ? bytes : 0x7fffffff), 0x00020000);
  };
  const __amdgpu_buffer_rsrc_t rsrc_p = operand_rsrc(P, a.M - row0, a.ldp);
  const __amdgpu_buffer_rsrc_t rsrc_q = operand_rsrc(Q, a.N - col0, a.ldq);
  typedef __attribute__((address_space(3))) void* LdsPtr;
  // One load at a time: a wave that issues several of these back to back stalls on the address queue, and its
  // MFMAs wait with it, so the main loop slips them in between MFMAs.
  auto load_p = [&](int k0, int stage, int i) {
    const int r0 = (i * kWaves + wave) * kRowsPerLoad;
    const int scalar_offset = (i * kWaves * kRowsPerLoad * a.ldp + k0) * 2;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_p, (LdsPtr)(smem + stage * kStageElems + r0 * BK), 16, lane_offset_p, scalar_offset, 0, 0);
  };
  auto load_q = [&](int k0, int stage, int i) {
    const int r0 = (i * kWaves + wave) * kRowsPerLoad;
    const int scalar_offset = (i * kWaves * kRowsPerLoad * a.ldq + k0) * 2;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_q, (LdsPtr)(smem + stage * kStageElems + BM * BK + r0 * BK), 16, lane_offset_q, scalar_offset, 0, 0);
  };
  auto stream_p = [&](int k0, int stage) {
#pragma unroll
    for (int i = 0; i < kLoadsP; ++i) load_p(k0, stage, i);
  };
  auto stream_q = [&](int k0, int stage) {
#pragma unroll
    for (int i = 0; i < kLoadsQ; ++i) load_q(k0, stage, i);
  };

  // Accumulator register r of lane l holds C[4*(l/16) + r][l%16] of its 16x16 tile.
  const int lcol = wave_n * kWaveN + (lane & 15);
  const int lrow = wave_m * kWaveM + (lane >> 4) * 4;
  // A whole tile whose D operand is also at hand transposed starts from it instead of adding it at the end:
  // acc = (beta / alpha) D, so that alpha * acc is alpha P Q^T + beta D with one rounding, as before.  The four
  // registers of an MFMA tile are four consecutive rows of one column, i.e. four consecutive elements (8 bytes) of a
  // row of D^T, which come straight from global memory in the accumulator's layout and go out with the first slabs.
  // (A D tile fetched behind the main loop has to be staged through LDS, since its rows do not match the accumulator
  // layout, and picked up with 2-byte LDS reads: 5 of the 121 microseconds of a 256x256 tile with K = 4096.  The
  // fetch itself stays what it is wherever it sits: every CU wants its 128 KiB at the same moment.)
  // A whole tile takes its D operand on the way: D^T is the Q operand itself in both products that have one (X^T in
  // the update product, the symmetric A in A A), and K spans the rows of C there, so the Q slabs with k in
  // [row0, row0 + BM) hold D[k - row0][0 .. BN) of this tile as they pass through LDS.  The waves pick their values
  // out of those slabs (see the slab loop) and add (beta / alpha) D to the accumulators, so that alpha * acc is
  // alpha P Q^T + beta D with one rounding; nothing is fetched for D.  (Fetched behind the main loop the D tile
  // cost a 256 x 256 tile with K = 4096 11 of its 121 microseconds: every CU wants its 128 KiB from HBM at the same
  // moment, and the tile has to be staged through LDS because its rows do not match the accumulator layout.)
  const bool d_in_slabs = whole && a.D != nullptr;
  const float d_scale = d_in_slabs ? a.beta / a.alpha : 0.0f;
  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;

  // 16x16x32 MFMA operands: lane l supplies row l % 16 of its 16-row block and the 8 k values of chunk l / 16 of
  // the 32 wide step.  (At equal peak rate this shape draws less power than 32x32x16 on operands with random
  // bits, and under sustained load the chip's clock is set by power: measured 2.0 against 1.8 PFLOP/s for bare
  // MFMA streams.)
  const int frag_row = lane & 15;
  const int frag_chunk = lane >> 4;

  // LDS offsets of this lane's fragment chunk for the k32 steps of a slab (the row part of the swizzle only
  // depends on frag_row: every 16-row block starts at a multiple of 16 rows)
  const __bf16* frag_p = smem + (wave_m * kWaveM + frag_row) * BK;
  const __bf16* frag_q = smem + BM * BK + (wave_n * kWaveN + frag_row) * BK;
  auto frag_off = [&](int stage, int kk) {
    return stage * kStageElems + (((kk * 4 + frag_chunk) ^ ((frag_row / kRowsPerSweep) % kChunks)) << 3);
  };
  // Software pipeline.  STAGES slabs are resident or in flight: the slab being multiplied and the next
  // STAGES - 1, streamed HBM -> LDS while the MFMAs run.  A k32 step runs as two half steps of TMH x TN MFMAs
  // (the upper and the lower tile rows of the wave).  Fragments: the Q side (all TN of a step) is double
  // buffered, the P side holds one buffer per half; the first half of a step reads the P fragments of its second
  // half, the second half reads the next step's Q fragments and first-half P fragments, so every 128-bit LDS read
  // has half a step of MFMAs to come back (it is waited for at the start of the next half step).  The one barrier
  // per slab sits before the slab's last half step: by then every wave has its last fragments of the current
  // stage in registers (the stage can be refilled with the slab STAGES ahead) and its share of the next slab has
  // landed, so the next slab's first fragments are fetched under this slab's last MFMAs.
  constexpr int kWaitLds = 0xC07F;  // s_waitcnt lgkmcnt(0), vmcnt / expcnt fields at their maxima
  // s_waitcnt lgkmcnt(0) vmcnt(N): loads return in order, so this leaves the N most recent ones in flight
  constexpr int kInFlight = (STAGES - 2) * kLoadsPerSlab;
  constexpr int kWaitNextSlab = 0x0070 | (kInFlight & 0xF) | ((kInFlight >> 4) << 14);
  bf16x8 fa_lo[TMH], fa_hi[TMH], fb0[TN], fb1[TN];
  // Loads are issued unconditionally, for a slab number clamped to the last one: past the end of the walk they
  // fetch the last slab once more into a stage nobody reads again.  (A branch around a load in the middle of the
  // MFMAs makes the register allocator spill the accumulators.)
  auto k0_clamped = [&](int i) { return k0_of(i < n_slabs ? i : n_slabs - 1); };
  if (n_slabs > 0) {
#pragma unroll
    for (int sidx = 0; sidx < STAGES; ++sidx) {
      stream_p(k0_clamped(sidx), sidx);
      if (sidx + 1 < STAGES) stream_q(k0_clamped(sidx), sidx);  // the Q rows of the last one go out under the first MFMAs
    }
    constexpr int kAfterFirst = (STAGES - 2) * kLoadsPerSlab + kLoadsP;
    __builtin_amdgcn_s_waitcnt(0x0F70 | (kAfterFirst & 0xF) | ((kAfterFirst >> 4) << 14));
    __syncthreads();
    const int off = frag_off(0, 0);
#pragma unroll
    for (int i = 0; i < TMH; ++i) fa_lo[i] = *reinterpret_cast<const bf16x8*>(frag_p + off + i * 16 * BK);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb0[j] = *reinterpret_cast<const bf16x8*>(frag_q + off + j * 16 * BK);
  }
  // One half step: the TMH x TN MFMAs on the fragments in hand (use_a for tile rows row0.., use_b), kReads LDS
  // reads (read(r), one behind each of the first MFMAs) and kLoads slab loads, interleaved instruction by
  // instruction: MFMA, LDS read, MFMA, LDS read, ..., slab load, ...  The matrix pipe is handed to the oldest wave
  // that has an MFMA ready, so whenever one of the two waves of a SIMD sits at the barrier the other runs alone,
  // and then every clump of other instructions between two MFMAs is a bubble in the pipe.
  auto half_step = [&](auto row0_tag, const bf16x8 (&use_a)[TMH], const bf16x8 (&use_b)[TN], auto reads_tag, auto&& read,
                       auto loads_tag, auto&& load) {
    constexpr int kRow0 = decltype(row0_tag)::value;
    constexpr int kReads = decltype(reads_tag)::value;
    constexpr int kLoads = decltype(loads_tag)::value;
    constexpr int kMfma = TMH * TN;
    constexpr int kChunks_ = kLoads > 0 ? kLoads : 1;
    constexpr int kPer = kMfma / kChunks_;
    static_assert(kMfma % kChunks_ == 0 && kReads <= kMfma, "half step shape");
#pragma unroll
    for (int c = 0; c < kChunks_; ++c) {
#pragma unroll
      for (int n = c * kPer; n < (c + 1) * kPer; ++n) {
        if (n < kReads) read(n);
        acc[kRow0 + n / TN][n % TN] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(use_a[n / TN], use_b[n % TN], acc[kRow0 + n / TN][n % TN], 0, 0, 0);
      }
#pragma unroll
      for (int n = c * kPer; n < (c + 1) * kPer; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
        if (n < kReads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
      }
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (kLoads > 0) {
        load(c);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  using Zero = std::integral_constant<int, 0>;
  using Upper = std::integral_constant<int, TMH>;
  // first half of step kk (fragments in fa_lo / use_b): reads the second half's P fragments
  auto first_half = [&](const bf16x8 (&use_b)[TN], int read_stage, int kk, auto loads_tag, auto&& load) {
    const int off = frag_off(read_stage, kk);
    half_step(Zero{}, fa_lo, use_b, std::integral_constant<int, TMH>{},
              [&](int r) { fa_hi[r] = *reinterpret_cast<const bf16x8*>(frag_p + off + (TMH + r) * 16 * BK); }, loads_tag, load);
  };
  // second half (fa_hi / use_b): reads the Q fragments and the first-half P fragments of the step after it
  auto second_half = [&](const bf16x8 (&use_b)[TN], bf16x8 (&next_b)[TN], int read_stage, int read_kk, auto loads_tag, auto&& load) {
    const int off = frag_off(read_stage, read_kk);
    half_step(Upper{}, fa_hi, use_b, std::integral_constant<int, TN + TMH>{},
              [&](int r) {
                // Q fragments first: the next step's first MFMAs need every one of them but only the first P fragment
                if (r < TN) next_b[r] = *reinterpret_cast<const bf16x8*>(frag_q + off + r * 16 * BK);
                else fa_lo[r - TN] = *reinterpret_cast<const bf16x8*>(frag_p + off + (r - TN) * 16 * BK);
              },
              loads_tag, load);
  };
  // D values out of a Q slab (see d_in_slabs above).  Slab q of the BM / BK slabs that hold the tile's D rows carries
  // the rows of kTilesPerSlab MFMA tile rows of the waves with wave_m == q / kSlabsPerWave; a lane's four rows of one
  // column are four consecutive k of one slab row: one 64-bit LDS read per MFMA tile, in three batches at the starts
  // of the slab's first three half steps (the values wait in registers for half a step, and all reads are back before
  // the barrier that releases the stage).
  constexpr int kTilesPerSlab = BK / 16;
  constexpr int kSlabsPerWave = kWaveM / BK;
  constexpr int kDSlabs = BM / BK;
  constexpr int kDPairs = kTilesPerSlab * TN, kDBatches = 3, kDBatch = (kDPairs + kDBatches - 1) / kDBatches;
  static_assert(kWaveM % BK == 0 && TM == kSlabsPerWave * kTilesPerSlab && kSteps == 2, "D slabs must divide over the waves and the half steps");
  const int d_base = BM * BK + lcol * BK + 4 * ((lane >> 4) & 1);  // slab row lcol (+ 16 j), first or second half of a chunk
  const int d_swizzle = (lcol / kRowsPerSweep) % kChunks;          // the same for lcol + 16 j
  u32x2 d_vals[kDBatch];
  auto d_read = [&](int stage, int batch) {
#pragma unroll
    for (int n = 0; n < kDBatch; ++n) {
      const int pair = batch * kDBatch + n, ii = pair / TN, j = pair % TN;
      if (pair >= kDPairs) break;
      const int chunk = (2 * ii + (lane >> 5)) ^ d_swizzle;
      d_vals[n] = *reinterpret_cast<const u32x2*>(smem + stage * kStageElems + d_base + j * 16 * BK + (chunk << 3));
    }
  };
  auto d_add = [&](auto qq_tag, int batch, float scale) {
    constexpr int kFirstTile = decltype(qq_tag)::value * kTilesPerSlab;
#pragma unroll
    for (int n = 0; n < kDBatch; ++n) {
      const int pair = batch * kDBatch + n, i = kFirstTile + pair / TN, j = pair % TN;
      if (pair >= kDPairs) break;
      acc[i][j][0] += scale * __uint_as_float(d_vals[n].x << 16);
      acc[i][j][1] += scale * __uint_as_float(d_vals[n].x & 0xffff0000u);
      acc[i][j][2] += scale * __uint_as_float(d_vals[n].y << 16);
      acc[i][j][3] += scale * __uint_as_float(d_vals[n].y & 0xffff0000u);
    }
  };
  int stage = 0;
  // One slab.  d_tag: -1, or which of the tile's D slabs this one is.
  auto slab = [&](int it, auto d_tag) {
    constexpr int kD = decltype(d_tag)::value;
    constexpr int kOwner = kD < 0 ? 0 : kD / kSlabsPerWave;
    using Part = std::integral_constant<int, kD < 0 ? 0 : kD % kSlabsPerWave>;
    const float scale = (kD >= 0 && wave_m == kOwner) ? d_scale : 0.0f;  // the other waves add zero times a finite value
    const int next_stage = stage + 1 == STAGES ? 0 : stage + 1;
    const int prev_stage = stage == 0 ? STAGES - 1 : stage - 1;
#pragma unroll
    for (int kk = 0; kk < kSteps; kk += 2) {
      __builtin_amdgcn_s_waitcnt(kWaitLds);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (kD >= 0) {
        d_read(stage, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (kk == 0) {
        // second half of the refill of the stage the previous slab's barrier released (its P rows went out there)
        const int k0 = k0_clamped(it - 1 + STAGES);
        first_half(fb0, stage, kk, std::integral_constant<int, kLoadsQ>{}, [&](int l) { load_q(k0, prev_stage, l); });
      } else {
        first_half(fb0, stage, kk, Zero{}, [](int) {});
      }
      __builtin_amdgcn_s_waitcnt(kWaitLds);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (kD >= 0) {
        d_add(Part{}, 0, scale);
        d_read(stage, 1);
        __builtin_amdgcn_sched_barrier(0);
      }
      second_half(fb0, fb1, stage, kk + 1, Zero{}, [](int) {});
      __builtin_amdgcn_s_waitcnt(kWaitLds);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (kD >= 0) {
        d_add(Part{}, 1, scale);
        d_read(stage, 2);
        __builtin_amdgcn_sched_barrier(0);
      }
      first_half(fb1, stage, kk + 1, Zero{}, [](int) {});
      if (kk + 2 < kSteps) {
        __builtin_amdgcn_s_waitcnt(kWaitLds);
        __builtin_amdgcn_sched_barrier(0);
        second_half(fb1, fb0, stage, kk + 2, Zero{}, [](int) {});
      } else {
        // last half step of the slab: the slab after it must have landed (the STAGES - 2 younger ones may be in
        // flight); behind the barrier this slab's stage is free and its refill starts with the P rows
        __builtin_amdgcn_s_waitcnt(kWaitNextSlab);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (kD >= 0) {
          d_add(Part{}, 2, scale);
          __builtin_amdgcn_sched_barrier(0);
        }
        const int k0 = k0_clamped(it + STAGES);
        second_half(fb1, fb0, next_stage, 0, std::integral_constant<int, kLoadsP>{}, [&](int l) { load_p(k0, stage, l); });
      }
    }
    stage = next_stage;
  };
  using NoD = std::integral_constant<int, -1>;
  if (d_in_slabs) {
    // the slabs with k in [row0, row0 + BM) are peeled out of the walk (whole tiles walk all of K from slab 0)
    const int first_d = row0 / BK;
    for (int it = 0; it < first_d; ++it) slab(it, NoD{});
    auto d_slabs = [&](auto&& self, auto q_tag) -> void {
      constexpr int kQ = decltype(q_tag)::value;
      slab(first_d + kQ, q_tag);
      if constexpr (kQ + 1 < kDSlabs) self(self, std::integral_constant<int, kQ + 1>{});
    };
    d_slabs(d_slabs, Zero{});
    for (int it = first_d + kDSlabs; it < n_slabs; ++it) slab(it, NoD{});
  } else {
    for (int it = 0; it < n_slabs; ++it) slab(it, NoD{});
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // the loads past the end of the walk have landed too; LDS is free

  // ---- K pieces: park the fp32 partial tile (row-major BM x BN); the fix-up kernel sums the pieces and
  // runs the epilogue.
  if (!whole) {
    float* mine = sched.partials + (static_cast<int64_t>(piece_tile) * sched.splits + split) * (BM * BN);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) mine[(lrow + i * 16 + r) * BN + lcol + j * 16] = acc[i][j][r];
    return;
  }


  // ---- epilogue, staged through LDS so that HBM only sees whole 16-byte-per-lane, row-contiguous accesses.
  // Accumulator register r of lane l holds C[4*(l/16) + r][l%16] of its 16x16 tile: written
  // straight from registers that would be 2-byte stores for C and 8-byte stores scattered over 16 rows for
  // the transpose.  Instead: C tile -> LDS -> HBM, transposed tile -> LDS -> HBM.  (The D operand is already in the
  // accumulators.)
  uint16_t* __restrict__ C = static_cast<uint16_t*>(a.C);
  uint16_t* __restrict__ CT = static_cast<uint16_t*>(a.CT);
  int ldct = a.ldct;
  if (a.symmetric) {  // mirror the off-diagonal tile
    CT = tm != tn ? C : nullptr;
    ldct = a.ldc;
  }
  uint16_t* stage_c = reinterpret_cast<uint16_t*>(smem_raw);
  constexpr int kLdS = BN + 8;  // row pitch of the staged C tile (elements); +8 keeps rows 16-byte aligned and skews banks
  constexpr int kLdT = BM + 8;  // row pitch of the staged transposed tile
  constexpr int kRowChunks = BN / 8, kColChunks = BM / 8;
  __syncthreads();  // every wave is done reading the slab stages
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = a.alpha * acc[i][j][r];
  if (a.update_param != nullptr) {
    // the last product of a Muon step: the tile goes into the parameter (in the parameter's orientation) and nowhere else
    if (!a.update_transposed) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            stage_c[(lrow + i * 16 + r) * kLdS + lcol + j * 16] = __builtin_bit_cast(uint16_t, static_cast<__bf16>(acc[i][j][r]));
      __syncthreads();
      for (int c = tid; c < BM * kRowChunks; c += kThreads) {
        const int r = c / kRowChunks, cc = c - r * kRowChunks;
        update_param8(a, row0 + r, col0 + cc * 8, *reinterpret_cast<const u32x4*>(stage_c + r * kLdS + cc * 8));
      }
    } else {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          u32x2 four = {pack_bf16x2(acc[i][j][0], acc[i][j][1]), pack_bf16x2(acc[i][j][2], acc[i][j][3])};
          *reinterpret_cast<u32x2*>(stage_c + (lcol + j * 16) * kLdT + lrow + i * 16) = four;
        }
      __syncthreads();
      for (int c = tid; c < BN * kColChunks; c += kThreads) {
        const int r = c / kColChunks, cc = c - r * kColChunks;
        update_param8(a, col0 + r, row0 + cc * 8, *reinterpret_cast<const u32x4*>(stage_c + r * kLdT + cc * 8));
      }
    }
    return;
  }
  if (!a.skip_c) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          stage_c[(lrow + i * 16 + r) * kLdS + lcol + j * 16] = __builtin_bit_cast(uint16_t, static_cast<__bf16>(acc[i][j][r]));
    __syncthreads();
    for (int c = tid; c < BM * kRowChunks; c += kThreads) {
      const int r = c / kRowChunks, cc = c - r * kRowChunks;
      *reinterpret_cast<u32x4*>(C + static_cast<int64_t>(row0 + r) * a.ldc + col0 + cc * 8) =
          *reinterpret_cast<const u32x4*>(stage_c + r * kLdS + cc * 8);
    }
    if (CT == nullptr) return;
    __syncthreads();
  }
  if (CT == nullptr) return;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
    {
      // the four registers of a tile are four consecutive rows of one column: four consecutive elements of a transposed row
      u32x2 four = {pack_bf16x2(acc[i][j][0], acc[i][j][1]), pack_bf16x2(acc[i][j][2], acc[i][j][3])};
      *reinterpret_cast<u32x2*>(stage_c + (lcol + j * 16) * kLdT + lrow + i * 16) = four;
    }
  __syncthreads();
  for (int c = tid; c < BN * kColChunks; c += kThreads) {
    const int r = c / kColChunks, cc = c - r * kColChunks;
    *reinterpret_cast<u32x4*>(CT + static_cast<int64_t>(col0 + r) * ldct + row0 + cc * 8) =
        *reinterpret_cast<const u32x4*>(stage_c + r * kLdT + cc * 8);
  }
}

// Sums the K pieces of every split tile in split order and applies the epilogue of gemm_nt_kernel.  A workgroup of
// 1024 threads finishes a 64 x 64 block of a tile, thread t four consecutive columns of row t / 16; the transposed /
// mirrored copy goes through LDS so that both orientations leave in whole 16-byte, row-contiguous stores.
constexpr int kFixupThreads = 1024;
template <int BM, int BN>
__global__ void __launch_bounds__(kFixupThreads)
splitk_fixup_kernel(GemmNtArgs a, Schedule sched) {
  constexpr int kSub = 64;
  constexpr int kSubsPerTile = (BM / kSub) * (BN / kSub);
  __shared__ __attribute__((aligned(16))) uint16_t transposed[kSub][kSub + 8];
  const int tile = blockIdx.x / kSubsPerTile;
  const int sub = blockIdx.x % kSubsPerTile;
  const int sub_row0 = (sub / (BN / kSub)) * kSub, sub_col0 = (sub % (BN / kSub)) * kSub;
  int tm, tn;
  tile_coords(sched.group_m, sched.full_tiles + tile, sched.tiles_m, sched.tiles_n, a.symmetric != 0, &tm, &tn);
  const uint16_t* __restrict__ D = static_cast<const uint16_t*>(a.D);
  uint16_t* __restrict__ C = static_cast<uint16_t*>(a.C);
  uint16_t* __restrict__ CT = static_cast<uint16_t*>(a.CT);
  int ldct = a.ldct;
  if (a.symmetric) {  // mirror the off-diagonal tile
    CT = tm != tn ? C : nullptr;
    ldct = a.ldc;
  }
  const int t = threadIdx.x;
  const int r = t / 16, c = (t % 16) * 4;  // position inside the 64 x 64 block
  const int lrow = sub_row0 + r, lcol = sub_col0 + c;
  const float* base = sched.partials + static_cast<int64_t>(tile) * sched.splits * (BM * BN) + lrow * BN + lcol;
  // four loads in flight at a time; the sum itself stays in split order
  f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
  int s = 0;
  for (; s + 4 <= sched.splits; s += 4) {
    f32x4 piece[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) piece[u] = *reinterpret_cast<const f32x4*>(base + static_cast<int64_t>(s + u) * (BM * BN));
#pragma unroll
    for (int u = 0; u < 4; ++u) sum += piece[u];
  }
  for (; s < sched.splits; ++s) sum += *reinterpret_cast<const f32x4*>(base + static_cast<int64_t>(s) * (BM * BN));
  const int row = tm * BM + lrow, col = tn * BN + lcol;
  float v[4] = {a.alpha * sum.x, a.alpha * sum.y, a.alpha * sum.z, a.alpha * sum.w};
  if (D != nullptr) {
    const u32x2 d = *reinterpret_cast<const u32x2*>(D + static_cast<int64_t>(row) * a.ldd + col);
    v[0] += a.beta * bf16_bits_to_float(static_cast<uint16_t>(d.x));
    v[1] += a.beta * bf16_bits_to_float(static_cast<uint16_t>(d.x >> 16));
    v[2] += a.beta * bf16_bits_to_float(static_cast<uint16_t>(d.y));
    v[3] += a.beta * bf16_bits_to_float(static_cast<uint16_t>(d.y >> 16));
  }
  const uint32_t lo = pack_bf16x2(v[0], v[1]);
  const uint32_t hi = pack_bf16x2(v[2], v[3]);
  if (a.update_param != nullptr) {  // uniform over the grid: the parameter update in place of the stores (see gemm_nt_kernel)
    if (!a.update_transposed) {
      const u32x4 packed = {lo, hi, 0u, 0u};  // this thread's four columns
      update_param8(a, row, col, packed, 4);
      return;
    }
    transposed[c][r] = static_cast<uint16_t>(lo);
    transposed[c + 1][r] = static_cast<uint16_t>(lo >> 16);
    transposed[c + 2][r] = static_cast<uint16_t>(hi);
    transposed[c + 3][r] = static_cast<uint16_t>(hi >> 16);
    __syncthreads();
    if (t < kSub * 8) {
      const int tr = t / 8, chunk = t % 8;
      update_param8(a, tn * BN + sub_col0 + tr, tm * BM + sub_row0 + chunk * 8, *reinterpret_cast<const u32x4*>(&transposed[tr][chunk * 8]));
    }
    return;
  }
  if (!a.skip_c) {
    const u32x2 packed = {lo, hi};
    *reinterpret_cast<u32x2*>(C + static_cast<int64_t>(row) * a.ldc + col) = packed;
  }
  if (CT == nullptr) return;  // uniform over the workgroup
  transposed[c][r] = static_cast<uint16_t>(lo);
  transposed[c + 1][r] = static_cast<uint16_t>(lo >> 16);
  transposed[c + 2][r] = static_cast<uint16_t>(hi);
  transposed[c + 3][r] = static_cast<uint16_t>(hi >> 16);
  __syncthreads();
  if (t < kSub * 8) {
    const int tr = t / 8, chunk = t % 8;  // row of the transposed block = column of the tile
    *reinterpret_cast<u32x4*>(CT + static_cast<int64_t>(tn * BN + sub_col0 + tr) * ldct + tm * BM + sub_row0 + chunk * 8) =
        *reinterpret_cast<const u32x4*>(&transposed[tr][chunk * 8]);
  }
}

GemmTuning g_tuning;
std::mutex g_tuning_mutex;  // the setter may be called while other threads launch: every launch works on one snapshot

GemmTuning tuning_snapshot() {
  std::lock_guard<std::mutex> lock(g_tuning_mutex);
  return g_tuning;
}

// Tiles a product computes: every tile of a general product, the tiles on or below the diagonal of a symmetric one.
int tile_count(const GemmNtArgs& a, int bm, int bn) {
  const int tm = a.M / bm, tn = a.N / bn;
  return a.symmetric ? tm * (tm + 1) / 2 : tm * tn;
}

template <int BM, int BN, int WM, int WN, int BK, int STAGES, int OCC>
int launch(const GemmNtArgs& a, const GemmScratch& scratch, const GemmTuning& tuning, hipStream_t stream) {
  constexpr int blocks_per_cu = OCC;
  Schedule s{};
  s.tiles_m = a.M / BM;
  s.tiles_n = a.N / BN;
  const int tiles = tile_count(a, BM, BN);
  const int slots = device_cu_count() * blocks_per_cu;
  const int k_slabs = a.K / BK;
  s.full_tiles = tiles;
  s.splits = 1;
  s.partials = static_cast<float*>(scratch.partials);
  s.group_m = std::max(1, tuning.group_m);
  const int rem = tiles % slots;
  if (tuning.split_remainder && rem != 0 && scratch.partials != nullptr) {
    // fill the machine once more with pieces of the leftover tiles; cap the pieces per tile so that the summing stays short
    int splits = std::min({slots / rem, k_slabs, tuning.max_splits});
    const int64_t tile_bytes = static_cast<int64_t>(BM) * BN * 4;
    while (splits > 1 && static_cast<int64_t>(rem) * splits * tile_bytes > scratch.partials_bytes) --splits;
    if (splits > 1) {
      s.full_tiles = tiles - rem;
      s.splits = splits;
    }
  }
  const int blocks = s.full_tiles + (tiles - s.full_tiles) * s.splits;
  constexpr size_t smem_loop = static_cast<size_t>(STAGES) * (BM + BN) * BK * sizeof(uint16_t);
  constexpr size_t smem_c = static_cast<size_t>(BM) * (BN + 8) * sizeof(uint16_t), smem_ct = static_cast<size_t>(BN) * (BM + 8) * sizeof(uint16_t);
  constexpr size_t smem_epilogue = smem_c > smem_ct ? smem_c : smem_ct;
  constexpr size_t smem = smem_loop > smem_epilogue ? smem_loop : smem_epilogue;
  auto kernel = gemm_nt_kernel<BM, BN, WM, WN, BK, STAGES, OCC>;
  {
    // raising the dynamic LDS limit is needed once per kernel and device
    static std::mutex mu;
    static bool configured[64] = {false};
    int dev = 0;
    MFSDP_HIP_TRY(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(mu);
    if (dev < 0 || dev >= 64 || !configured[dev]) {
      MFSDP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        static_cast<int>(smem)));
      if (dev >= 0 && dev < 64) configured[dev] = true;
    }
  }
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(WM * WN * 64), smem, stream, a, s);
  MFSDP_CHECK_LAUNCH("gemm_nt_kernel");
  if (s.splits > 1) {
    const int fix_blocks = (tiles - s.full_tiles) * (BM / 64) * (BN / 64);
    hipLaunchKernelGGL((splitk_fixup_kernel<BM, BN>), dim3(fix_blocks), dim3(kFixupThreads), 0, stream, a, s);
    MFSDP_CHECK_LAUNCH("splitk_fixup_kernel");
  }
  return MFSDP_OK;
}

// Which tiling a product runs with: 1 = 256 x 256, 2 = 128 x 128.
int choose_variant(const GemmNtArgs& a, const GemmTuning& tuning) {
  int variant = a.symmetric ? tuning.symmetric_variant : tuning.general_variant;
  if (a.symmetric && variant == 3) {
    // The triangle of a symmetric product rarely tiles the machine evenly.  Compare the two tilings in rounds of
    // resident workgroups, the last partial round counting 1/splits (plus the partial-tile traffic, which grows with
    // the splits) when its tiles are split along K: a round of 128x128 tiles (two per CU) takes about 0.6 of a round
    // of 256x256 tiles.  m = 4096 on 256 CUs: 136 big tiles are one half-empty round (1.0) against 528 small ones in
    // 1 + 1/16 rounds (0.83); m = 5120: 210 big tiles in one round (1.0) against 820 small ones in two (1.2) --
    // measured 15 % faster with the big tiles.  Below three quarters of a round of big tiles (m <= 4096 on 256 CUs)
    // only K-splitting would fill the machine and the small tiles win (m = 3072: 0.89 ms against 1.15 ms for the five
    // iterations; m = 2048, k = 8192: 0.88 against 0.99).
    auto rounds = [&](int tile, int per_cu) {
      const int t = a.M / tile, tiles = t * (t + 1) / 2, slots = device_cu_count() * per_cu;
      const int rem = tiles % slots;
      double r = tiles / slots;
      if (rem != 0) {
        const int splits = tuning.split_remainder ? std::min({slots / rem, a.K / kSlabK, tuning.max_splits}) : 1;
        r += splits > 1 ? 1.0 / splits + 0.02 * splits : 1.0;
      }
      return r;
    };
    const int big = a.M / 256, big_tiles = big * (big + 1) / 2;
    variant = (4 * big_tiles >= 3 * device_cu_count() && rounds(256, 1) <= 0.6 * rounds(128, 2)) ? 1 : 2;
    // On a machine shared with other matrices' kernels the CUs a part-filling triangle of big tiles leaves idle are
    // not lost, and a big tile moves fewer LDS bytes per flop: three hidden4096 matrices on three streams take 7.97 ms
    // with big tiles against 8.73 ms with small ones (8.47 ms one after the other).
    if (a.shared && 4 * big_tiles >= device_cu_count()) variant = 1;
  }
  return variant;
}

}  // namespace

void set_gemm_tuning(const GemmTuning& t) {
  std::lock_guard<std::mutex> lock(g_tuning_mutex);
  g_tuning = t;
}
GemmTuning get_gemm_tuning() { return tuning_snapshot(); }

int64_t gemm_nt_executed_flops(const GemmNtArgs& a) {
  const GemmTuning tuning = tuning_snapshot();
  const int tile = choose_variant(a, tuning) == 2 ? 128 : 256;
  return 2 * static_cast<int64_t>(tile) * tile * a.K * tile_count(a, tile, tile);
}

int gemm_nt_bf16(const GemmNtArgs& a, const GemmScratch& scratch, hipStream_t stream) {
  if (a.M <= 0 || a.N <= 0 || a.K <= 0 || a.M % 256 || a.N % 256 || a.K % kSlabK)
    return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: M=%d N=%d must be multiples of 256 and K=%d of %d", a.M, a.N, a.K, kSlabK);
  if (a.symmetric && a.M != a.N) return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: symmetric product needs M == N");
  if (a.skip_c && (a.symmetric || !a.CT)) return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: skip_c needs a transposed output and a general product");
  if (!a.P || !a.Q || !a.C) return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: null operand");
  if (a.ldp < a.K || a.ldq < a.K || a.ldc < a.N || (a.D && a.ldd < a.N) || (a.CT && a.ldct < a.M))
    return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: leading dimension smaller than the row length");
  if ((a.ldp | a.ldq) % 8 || (reinterpret_cast<uintptr_t>(a.P) | reinterpret_cast<uintptr_t>(a.Q)) % 16)
    return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: operands must be 16-byte aligned with leading dimensions multiple of 8");
  if ((a.ldc % 8) || reinterpret_cast<uintptr_t>(a.C) % 16 || (a.D && ((a.ldd % 8) || reinterpret_cast<uintptr_t>(a.D) % 16)) ||
      (a.CT && ((a.ldct % 8) || reinterpret_cast<uintptr_t>(a.CT) % 16)))
    return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: C, D and the transposed output must be 16-byte aligned with leading dimensions multiple of 8");
  if (a.D && (!a.d_transposed_is_q || a.K < a.M || a.alpha == 0.0f))
    return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: a D operand needs D^T == Q (K >= M) and alpha != 0");
  if (a.ldp > (1 << 22) || a.ldq > (1 << 22)) return fail(MFSDP_ERR_UNSUPPORTED, "gemm_nt_bf16: leading dimensions beyond 2^22 elements");
  GemmNtArgs b = a;
  if (a.update_param != nullptr) {
    const int elem = a.update_dtype == MFSDP_F32 ? 4 : 2;
    if (a.symmetric || (a.update_dtype != MFSDP_F32 && a.update_dtype != MFSDP_BF16) || a.update_rows <= 0 || a.update_cols <= 0 ||
        a.update_rows > (a.update_transposed ? a.N : a.M) || a.update_cols > (a.update_transposed ? a.M : a.N) ||
        reinterpret_cast<uintptr_t>(a.update_param) % elem)
      return fail(MFSDP_ERR_INVALID, "gemm_nt_bf16: parameter update needs a general product, an f32 / bf16 parameter inside the result and an aligned pointer");
    // groups of eight elements start at multiples of eight columns: whole 16-byte accesses when the rows keep that alignment
    b.update_vectors = a.update_cols % 8 == 0 && reinterpret_cast<uintptr_t>(a.update_param) % 16 == 0;
  }
  const GemmTuning tuning = tuning_snapshot();
  // Slabs of 32 (three to five deep) were measured too: each slab row is then half a 128-byte line, the vector
  // cache looks every line up twice, and the products run 15-25 % slower than with slabs of 64 two deep.
  if (choose_variant(b, tuning) == 2)  // 128x128 tile, 4 waves of 64x64, two workgroups per CU
    return launch<128, 128, 2, 2, 64, 2, 2>(b, scratch, tuning, stream);
  return launch<256, 256, 2, 4, 64, 2, 1>(b, scratch, tuning, stream);  // 256x256 tile, 8 waves of 128x64, one workgroup per CU
}

}  // namespace mfsdp
