/*
 * C ABI of the MI355X (gfx950) fused-embedding path.
 *
 * Two kinds of shared library implement it:
 *
 *  1. librecom.so -- one per emitted model (the code emitter writes process.hip, hipcc builds
 *     it).  It holds the fused kernel `FusedKnl` specialised to the model's feature list and
 *     exports the recom_* entry points below.  It replaces the reference's generated torch
 *     extension (TORCH_LIBRARY(recom): RecFlex/code_emitter/codegen.py:454-461).
 *     Several such libraries can be loaded into one process (dlopen / ctypes.CDLL), each
 *     with its own handle.
 *
 *  2. librecflex_host.so -- model independent, CPU only.  It exports the recom_host_* entry
 *     points: the text front end that turns the reference's dataset lines into indices and
 *     offsets and packs them.  It replaces the generated pybind module `recom_host`
 *     (RecFlex/code_emitter/codegen.py:90-218) and the per-schedule string parsers
 *     (examples/csrc/{warp_per_sample,one_block_multi_sample,onehot}_preprocess.cu).
 *
 * All functions return 0 on success.  recom_* functions return the hipError_t of the first
 * failing HIP call otherwise (never exit(), never synchronise the device, never allocate or
 * free device memory); recom_host_* functions return a negative RECOM_HOST_E* code.
 * Plain pointers and sizes only: no torch types cross this boundary.
 */
#ifndef RECFLEX_HIP_H_
#define RECFLEX_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------
 * librecom.so (generated, GPU)
 * ---------------------------------------------------------------------------------------- */

/* table element types (MetaData.data_type: "float", "half", "int8") */
#define RECOM_DTYPE_F32 0
#define RECOM_DTYPE_F16 1
/* row = dim unsigned 8-bit codes + fp16 scale + fp16 bias, row stride rounded up to 16 B;
 * value = code * scale + bias */
#define RECOM_DTYPE_I8 2

typedef struct recom_info {
  int32_t abi_version;    /* RECOM_ABI_VERSION */
  int32_t num_features;   /* F */
  int32_t embed_dim_sum;  /* columns of the pooled output */
  int32_t block_threads;  /* workgroup size the kernel was emitted for */
  int32_t occupancy;      /* workgroups per CU the kernel was emitted for (0 = not limited) */
  int32_t num_bodies;     /* distinct schedule bodies after de-duplication */
  int32_t timing;         /* 1 if built with per-feature device timers */
  int32_t tile_bytes;     /* default memory traffic per tile of the run-time binding; 0 = chosen
                           * per batch on the device from the batch's total traffic */
  int32_t static_binding; /* 1 if the tile count per feature was fixed at emit time */
  int32_t num_candidates; /* schedules compiled in; == num_features unless a tuning build */
  int32_t xcd_segments;   /* default of recom_process_args.xcd_segments (0 = flat tile walk) */
  int32_t outliers;       /* 1 if emitted with outlier tiles: recom_process first launches a kernel
                           * that lists the bags too long for their feature's schedule, and the
                           * fused kernel runs them as tiles of their own, several workgroups each */
  int32_t static_workspace; /* 1 if the workspace fits the library's static device array, i.e.
                             * recom_process_static_workspace can be used */
  int32_t reserved[3];
} recom_info;

#define RECOM_ABI_VERSION 6     /* 4: recom_process_static_workspace; the once-per-launch binding
                                 * table of very wide models moved into the workspace
                                 * 5: recom_process_args.start_event / stop_event
                                 * 6: recom_process_args.d_lookup_counts */

/* largest workspace recom_process_static_workspace serves from the library's static array */
#define RECOM_STATIC_WORKSPACE_MAX_BYTES (32 * 1024 * 1024)
/* returned by recom_process_static_workspace of a library whose workspace is larger than that
 * (negative: not a hipError_t) */
#define RECOM_ESTATIC_WORKSPACE (-5)

/* Static description of the emitted kernel.  No reference counterpart as a function: the
 * reference bakes the same numbers into process.cu (EMBED_DIM_SUM, block_threads,
 * RecFlex/code_emitter/codegen.py:227-231,318-319). */
int recom_get_info(recom_info *out);

/* Per-feature static tables, each `num_features` long; any pointer may be NULL.
 * embed_dims / embed_dim_offsets: RecFlex/code_emitter/codegen.py:227-231,289-292
 * (d_embed_dim_offsets).  dtypes: RECOM_DTYPE_*.  row_strides: bytes between table rows. */
int recom_get_feature_tables(int32_t *embed_dims, int32_t *embed_dim_offsets, int32_t *dtypes,
                             int32_t *row_strides);

/* Number of schedules compiled in for each feature (`num_features` entries): 1 in a production
 * build; in a tuning build the whole candidate list of the feature, from which each launch
 * picks one through recom_process_args.d_schedule_choice.  No reference counterpart: the
 * reference compiles one library per (feature, occupancy) with the candidates laid out as
 * separate features (RecFlex/tuning/tuner.py:112-126). */
int recom_get_candidate_counts(int32_t *counts);

/* Workgroups of FusedKnl that are resident at once on the current device
 * (= CUs x workgroups per CU at the emitted occupancy); this is also the size of the
 * persistent grid.  Replaces torch.ops.recom.get_max_concurrent_blocks
 * (RecFlex/code_emitter/codegen.py:446-452, RecFlex/sched_basic_csrc/include/utils.cuh:6-21). */
int recom_get_max_concurrent_blocks(int32_t *out);

/* Bytes of recom_process_args.d_workspace this library needs: 0 unless a feature runs a
 * schedule that splits bags over workgroups, then 2048 * (D_f + 1) * 4 bytes for each such
 * feature (rounded up to 128); a library with outlier tiles adds its list of outliers and
 * their partial sums (entries * (36 + 16 * max dim) + 128 bytes; 4 096 entries up to 128
 * features, 16 384 beyond); a library whose last tile passes are drawn from ticket counters
 * adds those (1 152 bytes); a library that is bound once per launch (by default one of more
 * than 3072 features) adds the table into which a one-workgroup kernel binds the model (12 bytes
 * per feature).  Replaces the
 * extra-buffer sizes the reference's host preprocessors report per batch
 * (RecFlex/code_emitter/codegen.py:149-160, extra_buffer_offsets). */
int recom_get_workspace_bytes(int64_t *out);

typedef struct recom_launch_info {
  int32_t compute_units;      /* CUs of the current device */
  int32_t occupancy;          /* workgroups per CU the persistent grid is sized for */
  int32_t dyn_lds_bytes;      /* dynamic-LDS pad per workgroup that keeps further ones off a CU */
  int32_t natural_occupancy;  /* workgroups per CU the kernel's registers and LDS allow */
  int32_t api_occupancy;      /* hipOccupancyMaxActiveBlocksPerMultiprocessor, for comparison */
  int32_t num_vgprs;          /* vector registers per lane */
  int32_t static_lds_bytes;
  int32_t lds_bytes_per_cu;
  int32_t padded_api_occupancy; /* hipOccupancyMaxActiveBlocksPerMultiprocessor with the pad */
  int32_t reserved[3];
} recom_launch_info;

/* How FusedKnl is launched on the current device: the pieces of the reference's
 * get_max_concurrent_blocks / get_dyn_smem_size (RecFlex/sched_basic_csrc/include/utils.cuh:6-58),
 * made visible. */
int recom_get_launch_info(recom_launch_info *out);

typedef struct recom_process_args {
  /* device int64[F]: base address of each feature's table
   * (RecFlex/sched_basic_csrc/gpu_pointers_array.cc:16-25) */
  const int64_t *d_embed_table_ptrs;
  /* Input, form A: device int64[2F], [2f] = address of feature f's int32 indices[L_f],
   * [2f+1] = address of its int32 offsets[batch+1].  NULL selects form B. */
  const int64_t *d_io_ptrs;
  /* Input, form B (the packed buffer of RecFlex/rec_modules.py:40-42): feature f's data
   * start at d_arg_buffers + d_arg_buffer_offsets[f] (bytes, device int64[F+1]):
   * int32 offsets[batch+1], padded to 128 B, then int32 indices[L_f], padded to 128 B. */
  const void *d_arg_buffers;
  const int64_t *d_arg_buffer_offsets;
  /* device fp32 [batch, embed_dim_sum], row-major, caller allocated; every element is
   * written (empty bag -> zeros).  The reference allocates it inside the op
   * (RecFlex/code_emitter/codegen.py:416-421). */
  float *d_output;
  int32_t batch;
  /* memory traffic per tile for the run-time binding; 0 = the emitted default
   * (recom_info.tile_bytes; if that is 0 too, the device sizes the tiles from the batch:
   * total traffic / (64 tiles per workgroup of the grid), within 64..256 KiB) */
  int32_t tile_bytes;
  /* persistent grid size; 0 = recom_get_max_concurrent_blocks() */
  int32_t grid_blocks;
  /* L2 locality of the tile walk: > 0 cuts the (feature-ordered) tile space into 8 * xcd_segments
   * equal segments and gives segment s to the workgroups of XCD s % 8, so that the rows a
   * feature's bags share are cached by one or two of the eight L2s instead of all; 0 = the
   * emitted default; < 0 = flat walk (tile t to workgroup t % grid) */
  int32_t xcd_segments;
  /* tuning builds: device int32[F], the candidate schedule each feature runs in this launch
   * (clamped to the feature's candidate count); NULL = candidate 0 everywhere */
  const int32_t *d_schedule_choice;
  /* timing builds only: device uint64[F + 2], the kernel ADDS each feature's workgroup-ticks
   * (s_memtime, shader cycles) to entries 0..F-1 and, in units of 10 ns (the constant 100 MHz
   * clock, s_memrealtime), the time every workgroup spends before its first tile (the run-time
   * binding) to entry F and every workgroup's time from start to end to entry F + 1;
   * caller zeroes it.  Replaces the per-block clock() array
   * (RecFlex/code_emitter/codegen.py:301-316,388-401).  NULL runs a timing build untimed;
   * must be NULL for other builds. */
  unsigned long long *d_times;
  /* hipStream_t to launch on (NULL = the null stream) */
  void *stream;
  /* floats between the starts of consecutive output rows; 0 = embed_dim_sum (a dense
   * [batch, embed_dim_sum] output, the only form the reference has).  A larger stride lets
   * several libraries -- a model split by features over libraries or GPUs -- write their column
   * slabs into one [batch, sum of all] buffer.  Must be a multiple of 4 when embed_dim_sum is
   * (the kernel then stores 16 bytes at a time), and d_output aligned likewise. */
  int64_t output_row_stride;
  /* Workspace of the schedules that give one bag to several workgroups (batches of few, very
   * long bags), of the outlier tiles, of a drawn end of the tile walk and of the once-per-launch
   * binding of very wide models:
   * device memory of at least recom_get_workspace_bytes() bytes, 16-byte aligned,
   * caller allocated.  It must be all zero before the first launch that uses it; every launch
   * leaves its arrival counters at zero again, so it is cleared once, not per launch.  Launches
   * that may overlap (different streams) need a workspace each.  Ignored (may be NULL) by a
   * library whose recom_get_workspace_bytes() is 0.  The reference's counterparts are the
   * extra_buffers / task_barriers tensors of torch.ops.recom.process
   * (RecFlex/code_emitter/codegen.py:403-444, RecFlex/rec_modules.py:44-52). */
  void *d_workspace;
  int64_t workspace_bytes;
  /* hipEvent_t (created by the caller with timing enabled) or NULL.  When either is given, the
   * kernels are launched with hipExtLaunchKernel: start_event receives the begin of the call's
   * first dispatch (the fused kernel, or the kernel launched ahead of it: outlier search,
   * once-per-launch binding), stop_event the end of the fused kernel's -- the call's own
   * duration on the device, without the dispatch latency and the marker packets that a pair of
   * hipEventRecord calls around the call adds (about two microseconds, which matter for a kernel
   * of ten).  Not for use under stream capture.  The reference times with the profiler only (RecFlex/cuda_helper.py:33-51). */
  void *start_event;
  void *stop_event;
  /* Optional hint for the run-time binding: device int32[F], the number of lookups of each
   * feature in this batch as far as the caller knows (the length of its index array).  NULL: the
   * binding reads offsets[batch] of every feature itself -- one scattered cache line per feature
   * and workgroup, half of the binding's time for a model of a thousand features.  The figures
   * only size the tiles (and tell the row-copy schedule that a feature may hold one lookup per
   * bag, which it verifies bag by bag): a wrong figure costs balance, never correctness.  The
   * reference has no counterpart (its binding runs on the host). */
  const int32_t *d_lookup_counts;
} recom_process_args;

/* Launch the fused kernel: for every feature f and sample b,
 *   output[b, off_f : off_f + D_f] = sum_{p in [offsets_f[b], offsets_f[b+1])} row(table_f, indices_f[p])
 * Asynchronous.  Replaces torch.ops.recom.process (RecFlex/code_emitter/codegen.py:403-444)
 * and FusedKnl (RecFlex/code_emitter/codegen.py:318-383).
 * Never allocates.  A library emitted with outlier tiles (recom_info.outliers) launches a small
 * kernel ahead that walks the offsets and lists the outlier bags in the workspace.
 * A library that is bound once per launch (by default one of more than 3072 features)
 * launches a one-workgroup kernel ahead of the fused one that binds the model for this batch
 * into a table in the workspace. */
int recom_process(const recom_process_args *args);

/* recom_process for callers that cannot allocate device memory at all, not even once: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  Same arguments, same kernels, same result bits as
 * recom_process, except that d_workspace / workspace_bytes are ignored: the workspace is a
 * file-scope device array of the library (recom_get_workspace_bytes() bytes, at most
 * RECOM_STATIC_WORKSPACE_MAX_BYTES; every device the library runs on holds its copy until the
 * process ends).  A library that needs more returns RECOM_ESTATIC_WORKSPACE
 * (recom_info.static_workspace == 0) and launches nothing.  Calls no hipMalloc / hipFree or
 * other allocating routine; a small fill kernel ahead of the others puts the array's arrival
 * counters and list header back to zero (no hipMemsetAsync, so the call can be captured).
 * The first call on a device also resolves the array's address and queries the kernel's
 * launch state (neither belongs inside a capture): make one eager call per device before
 * capturing this entry point in a graph.
 * All calls of one library on one device share the one array: calls that may overlap (two
 * streams, two threads) race and must be serialised by the caller.  A library whose
 * recom_get_workspace_bytes() is 0 behaves exactly like recom_process. */
int recom_process_static_workspace(const recom_process_args *args);

/* ------------------------------------------------------------------------------------------
 * librecflex_host.so (CPU)
 * ---------------------------------------------------------------------------------------- */

#define RECOM_HOST_EINVAL (-1)   /* NULL pointer / negative size */
#define RECOM_HOST_ENOSPC (-2)   /* output capacity too small */
#define RECOM_HOST_ELINES (-3)   /* text holds a different number of lines than expected */
#define RECOM_HOST_ERANGE (-4)   /* value does not fit in int32 */

/* Parse `num_lines` '\n'-separated sample lines of one feature.  Inside a line any byte that
 * is not a decimal digit separates two indices and a non-empty line always ends an index, so
 * "3,,5" gives 3,0,5 and "" gives an empty bag
 * (examples/csrc/warp_per_sample_preprocess.cu:14-32; the one-hot parser
 * examples/csrc/onehot_preprocess.cu:9-11 is the single-index case).
 * offsets_out[num_lines+1] receives the exclusive prefix sum of the bag lengths,
 * indices_out[0..*num_indices_out) the indices.  A final '\n' after the last line is allowed. */
int recom_host_parse_lines(const char *text, int64_t text_len, int32_t num_lines,
                           int32_t *indices_out, int64_t indices_capacity,
                           int32_t *offsets_out, int64_t *num_indices_out);

/* Upper bound of the number of indices a text of this length can hold. */
int64_t recom_host_max_indices(int64_t text_len);

/* 128-byte alignment used inside the packed argument buffer
 * (RecFlex/sched_basic_csrc/include/utils.cuh:60-68). */
int64_t recom_host_alignmem(int64_t nbytes);

/* Bytes feature f occupies in the packed buffer (form B above). */
int64_t recom_host_packed_size(int32_t batch, int64_t num_indices);

/* Pack F features into form B.  offsets[f] -> int32[batch+1], indices[f] -> int32[n_f].
 * dst has room for dst_capacity bytes; byte_offsets_out[F+1] receives each feature's start
 * (RecFlex/code_emitter/codegen.py:149-160 computes the same offsets for the reference's
 * layout).  Padding bytes are zeroed. */
int recom_host_pack(int32_t num_features, int32_t batch, const int32_t *const *offsets,
                    const int32_t *const *indices, const int64_t *num_indices, void *dst,
                    int64_t dst_capacity, int64_t *byte_offsets_out);

#ifdef __cplusplus
}
#endif

#endif /* RECFLEX_HIP_H_ */
