/*
 * C ABI of libgact_hip.so: GACT's saved-activation compression path on MI355X (gfx950).
 *
 * Every entry point takes plain device pointers and sizes, launches on the HIP stream it
 * is given (0 = the null stream), allocates no device memory and returns 0 or a negative
 * GACT_E* code (gact_strerror() names it).  The current HIP device must be the one the
 * pointers live on.  Calls are asynchronous; nothing synchronises the stream.
 *
 * "Reference" below is LiuXiaoxuanPKU/GACT-ICML; paths are relative to its root.
 */
#ifndef GACT_HIP_H
#define GACT_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GACT_ABI_VERSION 7

/* element types of activations, min, max and scale */
#define GACT_F32 0
#define GACT_F16 1
/* bfloat16 activations (no counterpart in the reference, which knows float and half).  Taken by
 * gact_quantize, gact_dequantize and the batched launches only.  min and max are bfloat16, the scale is
 * FLOAT32: the codes, the scale and the minimum are those of the float path on the widened values, and
 * dequantize rounds float(code) / scale + min to bfloat16, to nearest even. */
#define GACT_BF16 2

/* where the stochastic-rounding uniform u of each element comes from */
#define GACT_NOISE_CONST 0  /* u = 0.5: deterministic round-to-nearest                          */
#define GACT_NOISE_INJECT 1 /* u read from a float tensor laid out like the (padded) data        */
#define GACT_NOISE_REF 2    /* the reference's stream: one Philox4x32-10 state per output byte,  */
                            /* (seed, subsequence = byte index, offset 0), cuRAND uniform map    */
#define GACT_NOISE_FAST 3   /* one Philox4x32-7 block per 32 elements, 8-bit centred noise (ours)  */

#define GACT_OK 0
#define GACT_EINVAL (-1) /* bad argument (bits not in {1,2,4,8}, negative size, null pointer ...) */
#define GACT_EALIGN (-2) /* a pointer is not aligned as the kernels need (16 bytes)               */
#define GACT_ESHAPE (-3) /* shape not supported by this entry point                               */
#define GACT_ELAUNCH (-4) /* the HIP runtime reported an error at launch                          */
#define GACT_EBUDGET (-5) /* calc_precision: every tensor is at 1 bit and the budget is not met   */
#define GACT_ELIMIT (-6)  /* beyond the size limit of an entry point that brings its own workspace */

const char* gact_strerror(int code);
int gact_abi_version(void);

/* Bytes the pack kernels write for N groups rows of G*D elements: bits*N_round*G*D/8 with N rounded
 * up to a multiple of 8/bits.  The reference allocates one byte more and never writes it
 * (gact/gact/cpp_extension/quantization_cuda_kernel.cu:88-91). */
int64_t gact_packed_bytes(int bits, int64_t N, int64_t G, int64_t D);

/* Per-row minimum and maximum of a contiguous [N, D] tensor; D % 32 == 0 and D > 32.
 * Replaces minimax_cuda (gact/gact/cpp_extension/minimax_cuda_kernel.cu:70-89, bound at
 * minimax.cc:7-14). */
int gact_minimax(const void* data, int dtype, int64_t N, int64_t D, void* mn, void* mx, void* stream);

/* scale = T(2^bits-1)/(max-min+2e-6) for N*G entries, then the packed codes of data[N,G,D].
 * Writes gact_packed_bytes() bytes to `packed` and N*G values to `scale`.
 * Replaces pack_single_precision_cuda (quantization_cuda_kernel.cu:74-146, bound at
 * quantization.cc:51-61).  `noise` is only read in GACT_NOISE_INJECT mode. */
int gact_pack(const void* data, const void* mn, const void* mx, int dtype, int bits, int64_t N, int64_t G,
              int64_t D, int noise_mode, uint64_t seed, const float* noise, void* packed, void* scale,
              void* stream);

/* out[N,G,D] = T(code)/scale + min.  Replaces unpack_single_precision_cuda
 * (quantization_cuda_kernel.cu:180-221, bound at quantization.cc:36-49). */
int gact_unpack(const void* packed, int bits, const void* scale, const void* mn, int dtype, int64_t N,
                int64_t G, int64_t D, void* out, void* stream);

/* The whole of no_scheme_quantize_pack (gact/gact/ops.py:11-32) for group size 256 in one pass over
 * the data: `x` holds `numel` contiguous elements, treated as zero-padded to N = ceil(numel/256)
 * groups; writes min[N], scale[N] (and max[N] when `mx` is not null) and gact_packed_bytes(bits,N,1,256)
 * bytes.  Same results as gact_minimax + gact_pack on the padded tensor.  (GACT_BF16: scale is float32.) */
int gact_quantize(const void* x, int dtype, int64_t numel, int bits, int noise_mode, uint64_t seed,
                  const float* noise, void* packed, void* scale, void* mn, void* mx, void* stream);

/* gact_quantize with a second part of the seed that is read from device memory when the kernel runs: the
 * streams are seeded with seed + *seed_add (seed_add: one uint64 in device memory, 8-byte aligned; null = 0).
 * For launches recorded in a HIP graph, whose host arguments are frozen at capture: the caller rewrites the
 * device word between replays (gact/gact/quantizer.py:119-124 adds the iteration count to every tensor's seed)
 * and every replay draws fresh noise.  No counterpart in the reference. */
int gact_quantize_seeded(const void* x, int dtype, int64_t numel, int bits, int noise_mode, uint64_t seed,
                         const uint64_t* seed_add, const float* noise, void* packed, void* scale, void* mn,
                         void* mx, void* stream);

/* The whole of dequantize_and_unpack + the slice of op_dequantize (gact/gact/ops.py:34-47,61-69) for
 * group size 256: writes exactly `numel` elements. */
int gact_dequantize(const void* packed, int bits, const void* scale, const void* mn, int dtype,
                    int64_t numel, void* out, void* stream);

/* What a gact_quantize (kind 0; fast, deterministic or injected noise) or gact_dequantize (kind 1) launch of a tensor of
 * N groups is made of, without launching anything: the threads of a workgroup, the dynamic LDS the launch asks for -
 * on large tensors some kernels ask for LDS they never touch, which is how the library caps their occupancy - and
 * the workgroups of that kernel a compute unit holds under both (hipOccupancyMaxActiveBlocksPerMultiprocessor).
 * Any of the three pointers may be null.  No counterpart in the reference; for tests and tuning. */
int gact_launch_geometry(int kind, int dtype, int bits, int64_t N, int* threads, int* lds_bytes,
                         int* workgroups_per_cu);

/* Dropout-mask bit packing: n bytes (nonzero = 1) <-> ceil(n/32) int32 words.
 * Replace act_quantize_dropout_mask_cuda / act_dequantize_dropout_mask_cuda
 * (quantization_cuda_kernel.cu:254-303, bound at quantization.cc:26-33). */
int gact_mask_pack(const uint8_t* data, int64_t n, int32_t* mask, void* stream);
int gact_mask_unpack(const int32_t* mask, int64_t n, uint8_t* out, void* stream);

/* Greedy bit allocation on host memory; mutates b.  Replaces calc_precision
 * (gact/gact/cpp_extension/calc_precision.cc:66-118, bound at :120-123). */
int gact_calc_precision(int32_t* b, const float* C, const int64_t* w, int64_t L, double target);

/* The same allocation computed on the GPU from device arrays (b is updated in place), so that the
 * sensitivities never leave the device.  `status` (device int32, may be null) receives 0 or GACT_EBUDGET.
 * No counterpart in the reference, which runs calc_precision on the host. */
int gact_calc_precision_device(int32_t* b, const float* C, const int64_t* w, int64_t L, double target,
                               int32_t* status, void* stream);

/* One saved tensor of a batched launch.  The table itself lives in device memory. */
typedef struct gact_batch_entry {
  const void* x;      /* activation (quantize input / dequantize output), numel elements          */
  int64_t numel;
  int32_t dtype;      /* GACT_F32 / GACT_F16 / GACT_BF16                                           */
  int32_t reserved;
  uint64_t seed;      /* per-tensor seed: seeds[tid] + seed_iter (gact/gact/quantizer.py:119-124)  */
  int64_t first_block; /* exclusive prefix sum of ceil(N/128) over the table (128 groups per block) */
  int64_t packed_offset; /* byte offset of this tensor's codes in the packed arena (written by     */
                         /* gact_batch_plan from the device-resident bits)                          */
  int64_t stats_offset;  /* element offset of this tensor's scale/min rows in the stats arenas      */
} gact_batch_entry;

/* Bytes of device workspace gact_batch_plan fills for a table of L tensors whose grid has total_blocks
 * blocks (the sum of ceil(N_i/128): a block is 128 groups whatever the width).  16-byte aligned memory.
 * The batched entry points take L <= 2^30 and total_blocks < 2^29 (GACT_EINVAL beyond). */
int64_t gact_batch_workspace_bytes(int64_t L, int64_t total_blocks);

/* Plan a batched launch from device-resident bits: fills packed_offset of every table entry (256-byte
 * aligned, in table order) and the workspace - a header of 32 int64 ([0] the arena bytes the table needs,
 * [1] 1 when every bits[i] is in {1,2,4,8}, every dtype is known and [0] <= capacity, else 0: the batched
 * kernels then do nothing, [2..5] the number of tensors at width 1, 2, 4, 8) and the tensor of every block.
 * One small launch; nothing is read back.  No counterpart in the reference. */
int gact_batch_plan(gact_batch_entry* table, const int32_t* bits, int64_t L, int64_t total_blocks,
                    int64_t capacity, void* workspace, void* stream);

/* Quantize / dequantize all L tensors of the table, each at its own bits[i] read from device memory: one
 * launch over the grid of blocks per element type (quantize) or for all of them (dequantize), the width of
 * a block's tensor selecting the code path.  Scale and min of tensor i
 * are written at byte offset 4*stats_offset of their arenas (keep stats_offset a multiple of 8 so that
 * the rows stay 32-byte aligned).  Results equal a loop of
 * gact_quantize / gact_dequantize over the tensors (gact/gact/quantizer.py:95-142 drives the reference
 * one tensor at a time).  `workspace` is what gact_batch_plan filled for the same table, bits, L and
 * total_blocks.  `dtypes` says which element types
 * occur in the table, which the host that built it knows: bit 0 float, bit 1 half, bit 2 bfloat16 (GACT_DTYPES_*); quantize
 * launches only the kernels of those types, so a tensor whose type is missing from the mask is left unquantized. */
#define GACT_DTYPES_F32 1
#define GACT_DTYPES_F16 2
#define GACT_DTYPES_BF16 4
#define GACT_DTYPES_ALL 7
int gact_quantize_batched(const gact_batch_entry* table, const int32_t* bits, int64_t L, int64_t total_blocks,
                          int noise_mode, int dtypes, const void* workspace, void* packed_arena,
                          void* scale_arena, void* min_arena, void* stream);
int gact_dequantize_batched(const gact_batch_entry* table, const int32_t* bits, int64_t L,
                            int64_t total_blocks, const void* workspace, const void* packed_arena,
                            const void* scale_arena, const void* min_arena, void* stream);

/* gact_batch_plan followed by gact_quantize_batched, with the workspace in a device array that is part of
 * the library (1 MB per GPU the library runs on, held until the process ends) instead of memory the
 * caller brings: nothing is allocated, by the library or on its behalf.  No counterpart in the reference; it
 * is for callers that cannot allocate - code under HIP graph capture, tight serving loops, harnesses that
 * forbid it.  Same results as the two calls it stands for (packed_offset of every table entry is filled, the
 * arenas are written).  The plan's verdict lives in the library's array, out of the caller's reach, so the plan
 * also writes it to `verdict` (two int64 in device memory, 8-byte aligned; may be null): [0] the arena bytes the
 * table needs, [1] 1 when the launch went ahead, 0 when it was void (a width outside {1,2,4,8}, an unknown
 * element type, or [0] > capacity: the arenas are then left untouched).  Read it whenever the caller may
 * synchronise.  Limit: total_blocks <= 262144 (33.5 M groups, 8.6 G elements),
 * GACT_ELIMIT beyond.  All calls on one GPU share the array: calls that overlap on one GPU (two streams, two
 * threads) race, the caller serialises them.  The first call on a GPU looks the array's address up; make it
 * outside a stream capture.  Dequantize with gact_batch_plan + gact_dequantize_batched as usual. */
int gact_quantize_batched_static(gact_batch_entry* table, const int32_t* bits, int64_t L, int64_t total_blocks,
                                 int64_t capacity, int noise_mode, int dtypes, void* packed_arena,
                                 void* scale_arena, void* min_arena, int64_t* verdict, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* GACT_HIP_H */
