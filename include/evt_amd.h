/*
 * C ABI of one fused GEMM/BMM + epilogue-visitor-tree kernel module for MI355X
 * (gfx950).
 *
 * Every fused kernel the code generator emits is compiled into its own shared
 * object that exports exactly the symbols declared here (fixed names, loaded
 * with RTLD_LOCAL so many modules can coexist in one process).  The caller owns
 * every buffer: inputs, outputs and the workspace; a module never allocates
 * device memory, never synchronises the device and never reads device memory
 * from the host, so `evt_launch` can be recorded into a HIP graph.
 *
 * What each entry point replaces in the reference (apuaaChen/EVT_AE):
 *   - the per-kernel `extern "C"` trio `${op}_get_param_size`,
 *     `${op}_shared_memory_size`, `${op}_get_params` plus the
 *     `extern "C" __global__ ${op}(Params)` entry that the Python side launches
 *     (python/gtl/ops/reduce_apply_operation.py:44-86), and
 *   - for the GEMM/BMM anchors, `GemmArguments(...)` / `BmmArguments2x(...)` +
 *     `operation.run(arguments, stream)` of the un-vendored CUTLASS Python
 *     package (python/gtl/compiler/passes/evt_fuser.py:539-546, :674-680,
 *     python/gtl/ops/bmm.py:23-64).
 */
#ifndef EVT_AMD_H_
#define EVT_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EVT_ABI_VERSION 5
#define EVT_MAX_TENSORS 16
#define EVT_MAX_SCALARS 16

/* EvtArgs.flags: finish every cross-tile reduction in the separate finalize
 * kernel, also where the last workgroup to arrive could do it inside the GEMM
 * kernel (a test switch: both forms give the same bits). */
#define EVT_FLAG_TWO_KERNEL_REDUCE 1
/* EvtArgs.flags bits 8..15, row-wise modules only (GEMM modules ignore them):
 * workgroups per CU before the waves of a row kernel walk over several rows,
 * stored plus one (0 = the module's own default; EVT_FLAG_ROW_WG_PER_CU(0) = a
 * workgroup per group of rows, no walking).  The workspace size of a row module
 * with a per-column reduction depends on it: pass the same flags to
 * evt_workspace_bytes and evt_launch.  The modules read no environment. */
#define EVT_FLAG_ROW_WG_PER_CU(n) ((((n) + 1) & 0xff) << 8)
#define EVT_FLAG_ROW_WG_PER_CU_MASK 0xff00

/* Error codes returned by evt_launch / evt_workspace_bytes (negative); a
 * positive value is a hipError_t reported by the runtime at launch. */
#define EVT_OK 0
#define EVT_ERR_BAD_ARGS (-1)      /* null pointer, wrong tensor/scalar count   */
#define EVT_ERR_ALIGNMENT (-2)     /* operand not aligned for this module       */
#define EVT_ERR_WORKSPACE (-3)     /* workspace missing or too small            */
#define EVT_ERR_RANGE (-4)         /* a dimension exceeds what the kernel holds */
#define EVT_ERR_SCRATCH (-5)       /* evt_launch_static: the partial results of this problem exceed the static array */

/* One epilogue tensor (load or store).  Element (l, m, n) of the logical
 * [L, M, N] iteration space lives at
 *     ptr + (lb / l_div) * stride_l + (lb % l_div) * stride_l2
 *         + m * stride_m + n * stride_n                              (elements),
 *     lb = l_mod > 0 ? l % l_mod : l.
 * A broadcast dimension has stride 0.  l_div > 1 with stride_l2 = 0: l_div
 * consecutive batches share elements (a [B, ...] tensor against L = B*H
 * batches); with stride_l2 != 0 the batch index has two levels (a [B, S, H, D]
 * tensor read or written as L = B*H batches of [S, D]: the head split of an
 * attention layer without a copy); l_mod > 0: batches
 * that agree modulo l_mod share elements (an [H, ...] tensor against the same L).  For the
 * output of a per-row reduction, batches that share elements are summed into
 * them (the reduction then runs over N and over those batches).  Replaces the (M, N, L)-strided
 * tensor arguments of VisitorAuxLoad / VisitorRowBroadcast / VisitorRowStore
 * (src/cuda/epilogue/threadblock/visitor_load.hpp:364-571,
 *  visitor_store.hpp:46-145).
 * A slot the module spec lists with kind "rand" (rand_like) has no storage:
 * `ptr` is ignored and the strides give the element index e that seeds the
 * generator -- the value is word (e & 3) of Philox4x32-10(counter = (e >> 2
 * as two words, offset, slot index + 16 * stream id), key = seed), mapped to
 * [0, 1) as (word >> 8) * 2^-24.  Takes the place of VisitorRand's {seed, offset}
 * arguments (visitor_load.hpp:79-151). */
typedef struct EvtTensorArg {
  void* ptr;
  int64_t stride_l;
  int64_t stride_m;
  int64_t stride_n;
  int64_t l_div;
  int64_t l_mod;
  int64_t stride_l2;
} EvtTensorArg;

/* Launch arguments.  A is [L, M, K], B is [L, K, N]; which of the two
 * dimensions of each operand is contiguous is a compile-time property of the
 * module (see evt_module_spec).  `lda`/`ldb` are the strides, in elements, of
 * the non-contiguous dimension; batch strides are in elements and may be 0.
 * Modules with "tile"."dma": true in their spec move 16-byte chunks: A, B, lda, ldb
 * and the batch strides must be multiples of 8 elements (16 bytes), and so
 * must K where an operand is contiguous along K.  An operand that is
 * contiguous along M (A) or N (B) is read in whole chunks of 8 along that
 * dimension: if M (N) is not a multiple of 8, lda (ldb) must be at least M (N)
 * rounded up to 8 and every row, the last one included, readable to that
 * extent (what lies there does not reach the output).  Anything else is
 * refused with EVT_ERR_ALIGNMENT; modules with "tile"."dma": false take any
 * alignment.
 * Replaces GemmArguments / BmmArguments2x (evt_fuser.py:539-544, bmm.py:23-64).
 *
 * Row-wise modules (module spec has "anchor": softmax, softmax_backward,
 * layernorm, layernorm_backward; they replace SoftmaxArguments /
 * SoftmaxBackwardArguments / LayerNormArguments / LayerNormBackwardArguments,
 * evt_fuser.py:755-760, :818-824, :893-900, :960-968) use the same block: the
 * operand is viewed as [L, M, N] with rows of N contiguous elements; A is the
 * input (backward modules: the incoming gradient) and B the second operand of
 * the backward modules (softmax output / forward input), `lda`/`ldb` their row
 * strides and the batch strides their strides between batches, in elements;
 * K is ignored.  N may not exceed the module's "row"."max_n"
 * ("row"."waves_per_row" > 1: one workgroup per row).  Rows are read with
 * 16-byte accesses when A / B and their strides are 4-byte aligned.  A layer norm's
 * eps is scalars["anchor_scalars"]; layer norm backward reads the forward
 * pass's mean and rstd (fp32, one per row, contiguous) and optionally the
 * weight from the tensor slots listed under "anchor_tensors".  These modules
 * need a workspace only when the epilogue reduces over the rows (per-column
 * sum / max: one partial per workgroup and column; L must then be 1); it holds
 * no counters, so evt_workspace_init has nothing to do.
 */
typedef struct EvtArgs {
  int32_t M, N, K, L;
  const void* A;
  int64_t lda;
  int64_t batch_stride_A;
  const void* B;
  int64_t ldb;
  int64_t batch_stride_B;
  /* two-level batch index of an operand: batch l starts at
   *   (l / batch_div_X) * batch_stride_X + (l % batch_div_X) * batch_stride2_X
   * elements (batch_div_X = 0 or 1: one level, batch_stride2_X ignored).  Lets a [B, S, H, D] tensor serve as
   * L = B*H batches of [S, D] with row stride H*D (reference: the permuted
   * BMM operands of BmmArguments2x, python/gtl/ops/bmm.py:23-64). */
  int64_t batch_div_A;
  int64_t batch_stride2_A;
  int64_t batch_div_B;
  int64_t batch_stride2_B;
  int32_t num_tensors;
  int32_t num_scalars;
  /* Split-K of a GEMM module: 0 = the module decides (splits only when the
   * output tiles cannot fill the chip, K is long and the output is small),
   * 1 = never, n >= 2 = n splits (capped at the number of k-tiles).  The
   * workspace size depends on it: pass the same value to evt_workspace_bytes
   * and evt_launch.  Row-wise modules ignore it. */
  int32_t split_k;
  /* EVT_FLAG_* bits. */
  int32_t flags;
  EvtTensorArg tensors[EVT_MAX_TENSORS];
  /* immediates of the epilogue, in module-spec order.  A module with a "rand"
   * slot reads four of them as 32-bit patterns, not as float values:
   * scalars[rng_scalars + 0..3] = seed low word, seed high word, offset,
   * stream id (below 2^28; distinct per fused op, so that two ops whose
   * rand_like tensors have equal shapes draw unrelated numbers). */
  float scalars[EVT_MAX_SCALARS];
} EvtArgs;

/* ABI version the module was built against (== EVT_ABI_VERSION). */
int evt_abi_version(void);

/* Static JSON text describing the module: kernel name, tile shape, operand
 * layouts, alignment requirements, and the name / dtype / role of every tensor
 * and scalar slot.  Replaces the reference's emitted-source introspection
 * (`${op}_get_param_size`, reduce_apply_operation.py:44-58). */
const char* evt_module_spec(void);

/* Bytes of device workspace `evt_launch` needs for these arguments (0 when the
 * epilogue has no reduction that spans several workgroup tiles).  It holds the
 * per-tile partial results of the two-phase reduction and one arrival counter
 * per row / column block; when the module splits K over several workgroups per
 * output tile (few tiles, long K) also one fp32 accumulator tile per split and
 * one counter per tile.  The counters must be zero before the first launch
 * (evt_workspace_init) and every launch leaves them zero; launches that share
 * a workspace must not overlap in time.  The workspace is 16-byte aligned.  Takes the place of the host-side
 * pre-zeroing of reduction outputs (evt_fuser.py:217-225). */
int64_t evt_workspace_bytes(const EvtArgs* args);

/* Zero-fill a fresh workspace on `stream` with a fill kernel (no memset node,
 * so the call may be captured in a HIP graph). */
int evt_workspace_init(void* workspace, int64_t bytes, void* stream);

/* Enqueue the fused kernel (and, for reductions that span more than 64 tiles,
 * its small finalize kernel) on `stream` (a hipStream_t).  Asynchronous; returns
 * EVT_OK, a negative EVT_ERR_* code, or a positive hipError_t.  Replaces
 * `operation.run(arguments, stream=stream.cuda_stream)` (evt_fuser.py:546). */
int evt_launch(const EvtArgs* args, void* workspace, int64_t workspace_bytes,
               void* stream);

/* `evt_launch` for callers that cannot allocate device memory or be handed a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It has no counterpart in the reference.
 * The partial results, arrival counters and split-K tiles that `evt_launch`
 * keeps in the caller's workspace live in a device array that is part of the
 * module ("static_scratch_bytes" in the module spec: 1 MiB, or 0 for a module
 * whose kernels never use a workspace and which therefore carries no array),
 * which every GPU the module runs on holds from the first such call until the
 * process ends; the call itself allocates nothing and frees nothing.  A
 * problem whose workspace (evt_workspace_bytes) exceeds the array is refused
 * with EVT_ERR_SCRATCH before anything is enqueued.  The array used is the one
 * of the GPU `stream` belongs to (the current GPU for the null stream).  All
 * calls on one GPU share that GPU's array, so calls that may overlap in time
 * (different streams) race; each call clears the arrival counters it uses on
 * `stream` first (fill kernels, no memset node).  The first call on each GPU
 * looks the array's address up and must happen outside a stream capture;
 * later calls may be captured.  Inputs and outputs are passed as for
 * `evt_launch`. */
int evt_launch_static(const EvtArgs* args, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* EVT_AMD_H_ */
