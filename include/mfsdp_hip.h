/*
 * mfsdp_hip.h -- C ABI of libmfsdp_hip.so: MatrixFSDP's per-rank copy-in /
 * copy-out path and owner-rank optimizer update as hand-written gfx950 (CDNA4)
 * HIP kernels.
 *
 * Conventions (all entry points):
 *   - plain pointers and sizes; device pointers are raw HBM addresses on the
 *     current HIP device; `stream` is a hipStream_t passed as void* (NULL = the
 *     default stream);
 *   - every call validates its arguments on the host, enqueues its kernels on
 *     `stream` and returns without synchronising; tensors are borrowed for the
 *     duration of the enqueued work;
 *   - return value 0 = success; any other value is an error code and
 *     mfsdp_last_error() holds a message for the calling thread.  A binding
 *     turns non-zero into the host language's exception (the reference's
 *     TORCH_CHECK -> RuntimeError convention, matrix_copy.cpp:60-78, 86-94);
 *   - only the *_create / *_destroy calls and the host-metadata mfsdp_copy_rank_segments_to_full allocate or
 *     free device memory.
 *
 * Element offsets, not bytes, everywhere; `elem_bytes` in {1, 2, 4, 8}.
 */
#ifndef MFSDP_HIP_H_
#define MFSDP_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MFSDP_OK 0
#define MFSDP_ERR_INVALID 1   /* bad argument (null pointer, negative size, out of range, misaligned) */
#define MFSDP_ERR_HIP 2       /* a HIP runtime call failed */
#define MFSDP_ERR_UNSUPPORTED 3

/* dtype codes used by the cast / optimizer entry points */
#define MFSDP_F32 0
#define MFSDP_BF16 1
#define MFSDP_F16 2 /* mfsdp_accumulate only */

/* flag of mfsdp_muon_step_ex / mfsdp_muon_executed_flops */
#define MFSDP_MUON_SHARED_MACHINE 1

/* conversion a segment program applies while copying */
#define MFSDP_CONVERT_NONE 0         /* raw element move, any elem_bytes */
#define MFSDP_CONVERT_BF16_TO_F32 1  /* exact widening (Tensor.to(float32)) */
#define MFSDP_CONVERT_F32_TO_BF16 2  /* round-to-nearest-even, NaN -> 0x7FC0 (Tensor.to(bfloat16)) */
#define MFSDP_CONVERT_F16_TO_F32 3   /* exact widening, fp16 denormals included (Tensor.to(float32)) */
#define MFSDP_CONVERT_F32_TO_F16 4   /* round-to-nearest-even, NaN -> sign | 0x7E00 (Tensor.to(float16)) */

const char* mfsdp_last_error(void);
/* ABI version of the library; bumped on any signature change. */
int mfsdp_abi_version(void);

/* ------------------------------------------------------------------ copy */

/*
 * out[o] = in[input_offset + o] for o < out_numel.
 * Replaces copy_range (matrix_fsdp/kernels/native/matrix_copy.cpp:85-99,
 * matrix_copy_cuda.cu:25-36, 69-87).  Errors as the reference: negative
 * offset, range exceeding the input.  out_numel == 0 returns at once.
 */
int mfsdp_copy_range(const void* in, int64_t in_numel, void* out, int64_t out_numel,
                     int64_t input_offset, int elem_bytes, void* stream);

/*
 * out[global_starts[s] + o] = local[local_starts[s] + o] for o < numels[s].
 * Replaces copy_rank_segments_to_full (matrix_copy.cpp:53-83,
 * matrix_copy_cuda.cu:8-23, 38-67).  The three metadata arrays are HOST arrays
 * of n_segments int64 each (the reference passes device tensors it caches per
 * layout, kernels/native.py:470-489; here the cached object is the segment
 * program below, and this call is the uncached convenience form: it builds a
 * throw-away program, so it allocates and synchronises -- use a program on hot
 * paths).  n_segments == 0 returns at once.
 */
int mfsdp_copy_rank_segments_to_full(const void* local, int64_t local_numel, void* output, int64_t output_numel,
                                     const int64_t* global_starts, const int64_t* local_starts,
                                     const int64_t* numels, int64_t n_segments, int elem_bytes, void* stream);

/*
 * The same copy with the reference's own metadata contract: the three arrays are DEVICE arrays of n_segments int64
 * each (the tensors kernels/native.py:470-489 builds once per layout and caches) and max_numel is the longest
 * segment.  Replaces copy_rank_segments_to_full (matrix_copy.cpp:53-83, matrix_copy_cuda.cu:8-23, 38-67) argument
 * for argument; enqueue-only: no allocation, no host read of the metadata, no synchronisation, so it may be
 * captured into a HIP graph.  Offsets o < ceil(max_numel / 256) * 256 of every segment are copied, as the
 * reference's (tiles, segments) grid does.  The host cannot see the metadata, so the kernel validates it: a segment
 * with a negative start or size, or one that leaves `local` or `output`, is skipped (the reference would access
 * out of bounds).  n_segments == 0 or max_numel == 0 returns at once.
 *
 * workspace == NULL: one tile slot per (segment, tile index up to max_numel), the reference's launch shape; needs
 * nothing besides the arguments and is safe on concurrent streams.  workspace != NULL (8-byte aligned, at least
 * mfsdp_copy_rank_segments_workspace_bytes(n_segments) bytes, not shared by calls that may overlap): two small
 * kernels write the segments' running tile counts there (per block of 1024 segments, plus one offset per block) and
 * the copy grid is cut by bytes instead of by segment -- the shape to use when segment lengths differ widely.
 */
int64_t mfsdp_copy_rank_segments_workspace_bytes(int64_t n_segments);
int mfsdp_copy_rank_segments_to_full_device(const void* local, int64_t local_numel, void* output, int64_t output_numel,
                                            const int64_t* d_global_starts, const int64_t* d_local_starts,
                                            const int64_t* d_numels, int64_t n_segments, int64_t max_numel,
                                            int elem_bytes, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * The device-metadata copy above in its byte-balanced launch shape, for callers that cannot allocate: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The
 * segments' running tile counts go into an array of 1 MiB + 2 KiB that is part of the library's device image (every GPU the
 * library runs on holds its own copy until the process ends) instead of a caller's workspace, so the call neither
 * allocates nor frees anything; more than MFSDP_NOALLOC_MAX_SEGMENTS segments are rejected with
 * MFSDP_ERR_UNSUPPORTED.  Every call on a GPU shares that GPU's array: calls that may overlap on one GPU (two
 * streams) race and must use mfsdp_copy_rank_segments_to_full_device with their own workspaces instead.  The first
 * call on a device looks the array's address up (and loads the code object it lives in): make it outside a graph
 * capture; from the second call on the entry point only enqueues kernels.
 */
#define MFSDP_NOALLOC_MAX_SEGMENTS 131071
int mfsdp_copy_rank_segments_to_full_noalloc(const void* local, int64_t local_numel, void* output, int64_t output_numel,
                                             const int64_t* d_global_starts, const int64_t* d_local_starts,
                                             const int64_t* d_numels, int64_t n_segments, int64_t max_numel,
                                             int elem_bytes, void* stream);

/*
 * Segment program: a layout's whole copy (every rank, every segment, pad
 * zero-fill, optional dtype conversion) compiled once into device-resident
 * tables and replayed with ONE kernel launch per buffer.
 *
 * A run is a 2-D strided block, in elements:
 *     for r < rows, c < row_len:
 *         dst[dst_off + r*dst_stride + c] = convert(src[src_id][src_off + r*src_stride + c])
 * src_id = -1 writes zeros instead (pad tails: new_zeros / packed.zero_() in
 * matrix_fsdp/runtime/collectives.py:236-237 and runtime/grad_bucket.py:106).
 * A plain segment is a run with rows = 1.  It covers
 *   pack    _pack_full_tensor_by_rank_segments  (runtime/flat_buffer.py:1304-1316) fused with the
 *           zero-padded all-gather staging       (runtime/collectives.py:236-237, 248-249),
 *   unpack  un-pad                               (runtime/collectives.py:264-272) fused with
 *           _unpack_rank_shards_to_full_tensor   (runtime/flat_buffer.py:1318-1333),
 *   owner self-copy _copy_local_rank_segments    (runtime/collectives.py:495-503),
 *   grad copy-in    fill_reduce_scatter_input    (runtime/grad_bucket.py:71-116, 200-225),
 *                   compact owner fill           (runtime/flat_buffer.py:1232-1252),
 *   with the dtype casts of runtime/flat_buffer.py:1186-1206 folded in.
 * Destination runs of one program must not overlap each other.
 */
typedef struct mfsdp_copy_run {
  int64_t src_off;
  int64_t dst_off;
  int64_t row_len;
  int64_t rows;
  int64_t src_stride;
  int64_t dst_stride;
  int32_t src_id;   /* index into the srcs[] array given at run time; -1 = zero fill */
  int32_t reserved;
} mfsdp_copy_run;

typedef struct mfsdp_segment_program mfsdp_segment_program;

/*
 * Merges consecutive segments with equal length and constant source /
 * destination pitch into 2-D runs (a 2x2 block shard of an R x C matrix: R/2
 * row segments -> one run).  `segs` holds n_segs plain runs (rows == 1);
 * `out` has room for n_segs runs; returns the number written (host only).
 */
int64_t mfsdp_merge_segment_runs(const mfsdp_copy_run* segs, int64_t n_segs, mfsdp_copy_run* out);

/*
 * Validates the runs against the extents (src_numels[n_srcs], dst_numel), refuses runs whose destination rows
 * overlap (the reference's sequential slice writes make an overlap well defined; the waves of one launch write in
 * no particular order), compiles the tables for every vector width a later run may need and uploads them.
 * Allocates device memory; synchronous.  `convert` is one of MFSDP_CONVERT_*; elem_bytes is the element size for
 * MFSDP_CONVERT_NONE (ignored otherwise: 2 -> 4 or 4 -> 2 bytes: bf16 or fp16 on the 2-byte side).  Any number of
 * sources: fill_reduce_scatter_input (runtime/grad_bucket.py:71-116) takes any number of gradients; a launch
 * carries 128 source pointers, so a program over more sources replays as one launch per block of 128.
 */
int mfsdp_segment_program_create(const mfsdp_copy_run* runs, int64_t n_runs,
                                 const int64_t* src_numels, int32_t n_srcs, int64_t dst_numel,
                                 int convert, int elem_bytes, mfsdp_segment_program** out);
void mfsdp_segment_program_destroy(mfsdp_segment_program* program);
/* Algorithmic bytes one run of the program moves: bytes read + bytes written (zero fill counts as written). */
int64_t mfsdp_segment_program_bytes(const mfsdp_segment_program* program);
int64_t mfsdp_segment_program_num_runs(const mfsdp_segment_program* program);

/*
 * Replays the program: srcs[i] is the device base of source i and must hold
 * at least the src_numels[i] elements given at create time, dst at least
 * dst_numel.  One kernel launch per vector width in use (one for a layout whose
 * offsets are all 16-byte multiples); never allocates, never synchronises.  Base
 * pointers less aligned than the layout run the same tables at a narrower
 * vector width.
 */
int mfsdp_segment_program_run(mfsdp_segment_program* program, const void* const* srcs, int32_t n_srcs,
                              void* dst, void* stream);

/*
 * The same program over n_buffers buffers of one layout in ONE grid (the layer buffers of a step that are
 * due together: prefetched all-gather outputs, the gradient buckets of a backward window): buffer b reads
 * srcs[b * n_srcs + i] and writes dsts[b].  The per-launch ramp and tail are paid once instead of n_buffers times.
 * Both pointer tables travel in the kernel arguments (128 source pointers, 64 destinations): larger batches are
 * split into several launches.  Never allocates, never synchronises.
 */
int mfsdp_segment_program_run_many(mfsdp_segment_program* program, int32_t n_buffers, const void* const* srcs,
                                   int32_t n_srcs, void* const* dsts, void* stream);

/* ------------------------------------------------------------------ cast */

/*
 * dst = convert(src) element-wise over `numel` contiguous elements: the
 * Tensor.to(dtype) of _maybe_to_param_dtype / _maybe_to_reduce_dtype /
 * _maybe_to_local_dtype (matrix_fsdp/runtime/flat_buffer.py:1186-1206).
 */
int mfsdp_cast(const void* src, void* dst, int64_t numel, int convert, void* stream);

/*
 * dst += src over `numel` contiguous elements of one dtype (MFSDP_F32, MFSDP_BF16
 * or MFSDP_F16; 16-bit formats add in fp32 and round once): a backward that finds
 * the previous one's reduced gradient shard still in place adds to it,
 * MatrixFlatBuffer.accumulate_local_grad_shard (matrix_fsdp/runtime/flat_buffer.py:886-900).
 */
int mfsdp_accumulate(void* dst, const void* src, int64_t numel, int dtype, void* stream);

/* ------------------------------------------------------------------ Muon */

/*
 * Bytes of device workspace mfsdp_muon_step / mfsdp_newton_schulz need for an
 * rows x cols matrix (0 on invalid shape).
 */
int64_t mfsdp_muon_workspace_bytes(int64_t rows, int64_t cols);

/*
 * Quintic Newton-Schulz orthogonalisation of one matrix, the arithmetic of
 * torch.optim._muon._zeropower_via_newtonschulz (torch/optim/_muon.py:31-70)
 * that MixedMuonAdamWOptimizer.step reaches through torch.optim.Muon
 * (matrix_fsdp/optim/wrapper.py:497-516): bf16 operands, fp32 accumulation,
 * every product rounded to bf16, Frobenius normalisation with max(norm, eps).
 * `update` is rows x cols row-major of dtype `update_dtype` (MFSDP_F32 or
 * MFSDP_BF16); `out` is rows x cols bf16.
 */
int mfsdp_newton_schulz(const void* update, int update_dtype, int64_t rows, int64_t cols,
                        float a, float b, float c, int steps, float eps,
                        void* out_bf16, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * One matrix of torch.optim._muon._single_tensor_muon (torch/optim/_muon.py:285-318):
 *   buf <- buf + (1-momentum)*(grad - buf);  U = nesterov ? grad + momentum*(buf - grad) : buf
 *   O = NewtonSchulz(U);  param <- param*(1 - lr*weight_decay) - adjusted_lr*O
 * param / grad / momentum buffer share one dtype (`dtype`), as the reference's
 * local shard, local grad shard and zeros_like(grad) state do
 * (matrix_fsdp/runtime/flat_buffer.py:790-803).  adjusted_lr is the caller's
 * _adjust_lr(lr, fn, shape) (torch/optim/_muon.py:73-84).
 */
int mfsdp_muon_step(void* param, const void* grad, void* momentum_buf, int dtype, int64_t rows, int64_t cols,
                    double lr, double weight_decay, double momentum, int nesterov,
                    float a, float b, float c, int steps, float eps, double adjusted_lr,
                    void* workspace, int64_t workspace_bytes, void* stream);

/*
 * mfsdp_muon_step with flags.  MFSDP_MUON_SHARED_MACHINE: the caller updates other matrices at the same time on
 * other streams (each with its own workspace; a rank's whole matrices are independent of each other,
 * torch/optim/_muon.py:285-318 loops over them).  The symmetric products X X^T and A A then take the tile shape that
 * is best when the CUs they leave idle work for the other streams.  Results do not depend on the flag beyond the
 * summation order inside a product.
 */
int mfsdp_muon_step_ex(void* param, const void* grad, void* momentum_buf, int dtype, int64_t rows, int64_t cols,
                       double lr, double weight_decay, double momentum, int nesterov,
                       float a, float b, float c, int steps, float eps, double adjusted_lr, int flags,
                       void* workspace, int64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ AdamW */

/*
 * Fused single-launch AdamW over a flat fp32 shard (the arithmetic of
 * torch/optim/adam.py:347-547 with decoupled weight decay, reached through
 * matrix_fsdp/optim/wrapper.py:439, 497-516; state laid out flat as in
 * matrix_fsdp/optim/adamw_state.py:177-218).  `step` is the 1-based step
 * count after this update.  grad_dtype: MFSDP_F32 or MFSDP_BF16.  The
 * hyper-parameters are doubles, as Python holds them: 1 - beta, lr / (1 - beta1^t)
 * and the like are formed in double and rounded to fp32 once, as torch does.
 */
int mfsdp_adamw_step(float* param, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
                     int64_t numel, int64_t step, double lr, double beta1, double beta2, double eps,
                     double weight_decay, void* stream);

/*
 * The same update with the two remaining switches of torch.optim.AdamW's
 * single-tensor path (torch/optim/adam.py:398-399, 470-481): `maximize`
 * negates the gradient; a non-null `max_exp_avg_sq` turns on amsgrad (the
 * running element-wise maximum of the second moment, updated in place, takes
 * the second moment's place in the denominator; the reference lays it out
 * flat beside the moments, matrix_fsdp/optim/adamw_state.py:24-28).
 */
int mfsdp_adamw_step_ex(float* param, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
                        float* max_exp_avg_sq, int64_t numel, int64_t step, double lr, double beta1, double beta2,
                        double eps, double weight_decay, int maximize, void* stream);

/* ------------------------------------------------------------------ measurement and experiments
 *
 * Nothing below is part of the drop-in surface: the reference has no counterpart for any of it and a binding of the
 * reference needs none of it.  bench.py and the tests use these entry points to state what the part sustains beside
 * what the kernels reach, to count the flops the kernels execute, and to force kernel variants.
 */

/*
 * Flops the Newton-Schulz kernels execute for `steps` iterations on a rows x cols matrix with the current tuning
 * and the flags of mfsdp_muon_step_ex (operands zero-padded to multiples of 256; the two symmetric products of a step compute only the tiles on or below
 * the diagonal).  The reference executes full products: steps * (4 m^2 n + 2 m^3) with m the short side.
 */
int64_t mfsdp_muon_executed_flops(int64_t rows, int64_t cols, int steps, int flags);

/*
 * Measurement aid (no counterpart in the reference): one pass of pure reads (kind 0: `bytes` of src are loaded
 * and discarded; dst is a 4 KiB sink that is never written as long as src holds no all-ones 16-byte group) or pure
 * writes (kind 1: `bytes` of dst are filled with a constant), one workgroup per 4 KiB like the copy kernels, so that a
 * benchmark can state what the part sustains in each direction beside the copy it measures.
 */
int mfsdp_hbm_probe(int kind, const void* src, void* dst, int64_t bytes, void* stream);

/*
 * One plain product C = bf16(P Q^T) through the Newton-Schulz GEMM kernel (P: m x k, Q: n x k, C: m x n, all bf16
 * row-major and contiguous, m and n multiples of 256, k of 64), so that a benchmark can time the kernel on a shape of
 * its choice beside a library GEMM.  `partials` (may be NULL) is scratch for the K-split pieces of a last partial
 * round of tiles.
 */
int mfsdp_gemm_nt_bf16(const void* p, const void* q, void* c, int m, int n, int k, void* partials, int64_t partials_bytes, void* stream);

/* Launch tuning for experiments (safe to call while other threads launch): workgroups per CU of the copy grid
 * (-1 = library default, 0 = one workgroup per four tiles without a grid-stride loop, n > 0 = persistent grid of n
 * per CU), non-temporal hints (0 none, 1 loads and stores, 2 loads only, 3 stores only, -1 = default); and, for
 * programs created afterwards, 128-bit loads in flight per lane (1, 2 or 4; 0 = default); threads per workgroup (64, 128
 * or 256: the 256 lanes of a tile spread over 4, 2 or 1 workgroups; 0 = default). */
void mfsdp_set_copy_tuning(int blocks_per_cu, int nontemporal, int unroll, int block_threads);

/* Kernel selection for experiments (values <= 0 keep the current setting):
 * tile variant of the general and of the symmetric Newton-Schulz products (1: 256x256 tile / 8 waves / one
 * workgroup per CU, 2: 128x128 tile / 4 waves / two per CU; for the symmetric products also 3, the default:
 * whichever of the two fills the CUs better for the size at hand), the tile rows the general products walk together
 * (default 4), K-splitting of the last partial round of tiles on (1) / off (2), and its cap. */
void mfsdp_set_muon_tuning(int general_variant, int symmetric_variant, int group_m, int split_remainder, int max_splits);

#ifdef __cplusplus
}
#endif
#endif /* MFSDP_HIP_H_ */
