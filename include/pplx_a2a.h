/*
 * pplx_a2a.h -- C ABI of the MI355X (gfx950) MoE dispatch / combine library.
 *
 * This is the boundary a host-language binding attaches to.  Every entry point
 * takes plain pointers, sizes and strides; no torch / C++ types cross it.  The
 * library replaces the host classes and kernels of ppl-ai/pplx-kernels'
 * intranode all-to-all for a single-GPU loopback: all `world_size` simulated
 * expert-parallel (EP) ranks live in one process and one GPU's HBM.
 *
 * Reference interfaces replaced (paths relative to the reference tree):
 *   csrc/all_to_all/all_to_all.h:9-13    SplitMode                -> pplx_a2a_split_mode
 *   csrc/all_to_all/all_to_all.h:29-39   AllToAll ctor arguments  -> pplx_a2a_config_t
 *   csrc/all_to_all/intranode.h:23-63    AllToAllIntraNode        -> pplx_a2a_t + dispatch/combine
 *   csrc/core/buffer.h:116-161           Strided1D/2D/3D views    -> pointer + stride fields
 *   csrc/bindings/all_to_all_ops.cpp:54-108,122-196,238-311  create/destroy/dispatch/combine ops
 *
 * Conventions
 *   - Every function returns a pplx_a2a_status; 0 is success.  The library never
 *     exits or traps; pplx_a2a_last_error() returns the message of the calling
 *     thread's last failure.
 *   - Device pointers are HBM addresses on the world's device.  `stream` is a
 *     hipStream_t passed as void* (NULL = the legacy default stream).
 *   - Only *_create, *_destroy and pplx_a2a_world_reserve_split allocate, free
 *     or synchronise (pplx_a2a_world_faults synchronises the stream it reads
 *     behind); dispatch / combine only enqueue kernels, so they may be captured
 *     in a hipGraph and replayed.
 *   - Outputs of a send+recv step made of per-rank calls are valid once the
 *     LAST rank's call has returned, in stream order of any stream a rank of
 *     the step called on.
 */
#ifndef PPLX_A2A_H_
#define PPLX_A2A_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum pplx_a2a_status {
  PPLX_A2A_OK = 0,
  PPLX_A2A_INVALID_ARGUMENT = 1, /* a precondition on the arguments does not hold */
  PPLX_A2A_INVALID_STATE = 2,    /* call order violated (e.g. RECV before every SEND) */
  PPLX_A2A_HIP_ERROR = 3,        /* a HIP runtime call failed */
  PPLX_A2A_UNSUPPORTED = 4       /* valid request that this build cannot serve */
} pplx_a2a_status;

/* csrc/all_to_all/all_to_all.h:9-13 */
typedef enum pplx_a2a_split_mode {
  PPLX_A2A_SPLIT_NONE = 0, /* send and receive in one call */
  PPLX_A2A_SPLIT_SEND = 1,
  PPLX_A2A_SPLIT_RECV = 2
} pplx_a2a_split_mode;

/* element types of combine: csrc/bindings/all_to_all_ops.cpp:265-310 */
typedef enum pplx_a2a_dtype {
  PPLX_A2A_F32 = 0,
  PPLX_A2A_BF16 = 1,
  PPLX_A2A_F16 = 2
} pplx_a2a_dtype;

/* The AllToAll constructor arguments, csrc/all_to_all/all_to_all.h:29-39.
 * Invariants checked at world creation (csrc/all_to_all/all_to_all.cpp:32-39):
 * hidden_dim_bytes % 16 == 0, hidden_dim_scale_bytes % 16 == 0,
 * hidden_dim_scale_bytes <= hidden_dim_bytes, num_experts % world_size == 0,
 * world_size % dp_size == 0.  Unlike the reference a single DP group
 * (world_size == dp_size) is accepted. */
typedef struct pplx_a2a_config {
  uint64_t max_num_tokens;         /* M: max tokens per DP group per step */
  uint64_t num_experts;            /* E: global expert count */
  uint64_t experts_per_token;      /* K: top-k */
  uint32_t world_size;             /* R: number of simulated EP ranks */
  uint32_t dp_size;                /* ranks per DP group (hold identical tokens) */
  uint64_t hidden_dim;             /* H: elements per token row */
  uint64_t hidden_dim_bytes;       /* bytes of one dispatched activation row */
  uint64_t hidden_dim_scale_bytes; /* bytes of one row of fp32 block scales, 0 if none */
} pplx_a2a_config_t;

/* Owner of the state shared by all simulated ranks (routing tables, slot map,
 * staging for split mode).  Takes the place of the IPC-mapped peer buffers set
 * up in csrc/all_to_all/intranode.cpp:11-137. */
typedef struct pplx_a2a_world pplx_a2a_world_t;
/* One simulated EP rank; takes the place of an AllToAllIntraNode object. */
typedef struct pplx_a2a pplx_a2a_t;
/* An instantiated hipGraph. */
typedef struct pplx_a2a_graph pplx_a2a_graph_t;

/* Arguments of one rank's dispatch: the views built in
 * csrc/bindings/all_to_all_ops.cpp:165-195 for AllToAllIntraNode::dispatch
 * (csrc/all_to_all/intranode.h:39-50). */
typedef struct pplx_a2a_dispatch_args {
  int32_t *out_expert_num_tokens;        /* [L] */
  int64_t out_expert_num_tokens_stride;  /* elements */
  void *out_expert_x;                    /* [L, rows, hidden_dim_bytes] */
  int64_t out_expert_x_stride_row;       /* bytes between rows */
  int64_t out_expert_x_stride_expert;    /* bytes between local experts */
  int64_t out_expert_x_rows;             /* size(1): row capacity per expert; 0 = M * num_dp_groups */
  float *out_expert_x_scale;             /* [L, rows, S] or NULL */
  int64_t out_expert_x_scale_stride_elem;   /* floats */
  int64_t out_expert_x_scale_stride_row;    /* floats */
  int64_t out_expert_x_scale_stride_expert; /* floats */
  const void *dp_x;                      /* [m, hidden_dim_bytes] */
  int64_t dp_x_stride_row;               /* bytes */
  const float *dp_x_scale;               /* [m, S] or NULL */
  int64_t dp_x_scale_stride_elem;        /* floats */
  int64_t dp_x_scale_stride_row;         /* floats */
  const uint32_t *indices;               /* [m, K] contiguous */
  uint32_t m;                            /* rows of dp_x / indices */
  const uint32_t *bound_m;               /* device scalar: tokens actually present, or NULL (= m) */
} pplx_a2a_dispatch_args_t;

/* Arguments of one rank's combine: the views built in
 * csrc/bindings/all_to_all_ops.cpp:222-235 for AllToAllIntraNode::combine<T,U>
 * (csrc/all_to_all/intranode.h:53-63).  Strides are in elements. */
typedef struct pplx_a2a_combine_args {
  void *out_tokens;                 /* [>= m, H] of out_dtype */
  int64_t out_tokens_stride_row;
  int32_t out_dtype;                /* pplx_a2a_dtype: BF16 or F16 */
  const uint32_t *indices;          /* [m, K] contiguous */
  const float *weights;             /* [m, K] */
  int64_t weights_stride_row;
  const void *expert_y;             /* [L, rows, H] of in_dtype */
  int64_t expert_y_stride_row;
  int64_t expert_y_stride_expert;
  int64_t expert_y_rows;            /* size(1); 0 = M * num_dp_groups */
  int32_t in_dtype;                 /* pplx_a2a_dtype: F32, BF16 or F16 */
  uint32_t m;
  const uint32_t *bound_m;          /* device scalar or NULL (= m) */
} pplx_a2a_combine_args_t;

/* ---- lifecycle ------------------------------------------------------- */

/* Allocates the world's device state on `device` (a HIP device ordinal): with
 * T = world_size / dp_size * max_num_tokens, a slot map of T * experts_per_token * 4
 * bytes and routing tables of about T * num_experts / 8 bytes (the 8192-token
 * DSv3 shape: 2 MiB + 2.3 MiB), plus rank tables for worlds of more than 64 ranks.
 * Replaces the buffer set-up of csrc/all_to_all/intranode.cpp:11-137. */
int pplx_a2a_world_create(const pplx_a2a_config_t *cfg, int device, pplx_a2a_world_t **out);
/* Frees the world.  Fails with INVALID_STATE while rank handles are attached. */
int pplx_a2a_world_destroy(pplx_a2a_world_t *world);

/* Attaches simulated rank `rank`; replaces create_intranode,
 * csrc/bindings/all_to_all_ops.cpp:79-106. */
int pplx_a2a_create(pplx_a2a_world_t *world, uint32_t rank, pplx_a2a_t **out);
/* Replaces destroy, csrc/bindings/all_to_all_ops.cpp:108. */
int pplx_a2a_destroy(pplx_a2a_t *handle);
/* AllToAll::getNumExpertsPerToken, csrc/all_to_all/all_to_all.h:44. */
uint64_t pplx_a2a_num_experts_per_token(const pplx_a2a_t *handle);
uint32_t pplx_a2a_rank(const pplx_a2a_t *handle);

/* ---- per-rank calls (the reference API) ------------------------------ */

/* AllToAllIntraNode::dispatch, csrc/all_to_all/intranode_dispatch.cu:288-390.
 * The call is collective over the world, like the reference's: with
 * PPLX_A2A_SPLIT_NONE the kernels are enqueued when the last of the world_size
 * ranks has made its call for the step, on that call's `stream`, and every
 * rank's outputs are complete once they finish.  Ranks may call on different
 * streams (csrc/bindings/all_to_all_ops.cpp:163,194 runs each rank on its own
 * current stream): the launching stream first waits for the work the other
 * streams held when the last call came in, and those streams then wait for the
 * kernels; work a rank enqueues BETWEEN its own call and the last rank's call
 * is not ordered against the step.  The ranks of a captured step must share
 * one stream (PPLX_A2A_INVALID_STATE otherwise).
 * SEND and RECV are collective in the same way, phase by phase: the last
 * rank's SEND enqueues the sends of all ranks (inputs may be reused once it has
 * returned, in stream order; no output is touched), the last rank's RECV the
 * receives (outputs are those named by the RECV calls).  A SEND takes over
 * everything its call's inputs hold: dispatch SEND copies every present token
 * (row, scales, picks) and the groups' token counts into the staging area and
 * RECV routes and places them; combine SEND reads expert_y, indices, weights
 * and bound_m and leaves the combined rows in the staging area, and RECV copies
 * them to out_tokens (the reference reads indices and weights in its RECV,
 * csrc/all_to_all/intranode_combine.cu:127-169: pass the same ones to both
 * calls, as its callers do).  Every rank's SEND must
 * come before the first RECV, and staging must have been reserved with
 * pplx_a2a_world_reserve_split (PPLX_A2A_INVALID_STATE otherwise).
 * Without bound_m, m may not exceed max_num_tokens
 * (csrc/all_to_all/intranode_dispatch.cu:65); the members of a DP group must
 * pass the same m. */
int pplx_a2a_dispatch(pplx_a2a_t *handle, const pplx_a2a_dispatch_args_t *args,
                      int split_mode, void *stream);
/* AllToAllIntraNode::combine<T,U>, csrc/all_to_all/intranode_combine.cu:190-266. */
int pplx_a2a_combine(pplx_a2a_t *handle, const pplx_a2a_combine_args_t *args,
                     int split_mode, void *stream);

/* ---- all ranks in one call ------------------------------------------- */

/* One step for all ranks: `per_rank` is a host array of world_size entries,
 * entry r holding rank r's arguments.  Equivalent to world_size calls of
 * pplx_a2a_dispatch(..., PPLX_A2A_SPLIT_NONE, stream). */
int pplx_a2a_world_dispatch(pplx_a2a_world_t *world, const pplx_a2a_dispatch_args_t *per_rank,
                            void *stream);
int pplx_a2a_world_combine(pplx_a2a_world_t *world, const pplx_a2a_combine_args_t *per_rank,
                           void *stream);

/* One step (dispatch, combine, or dispatch then combine) for all ranks without a
 * world and without any allocation.  It has no counterpart in the reference; it
 * is for callers that cannot allocate device memory around the call: code under
 * hipGraph capture that has no world yet, tight serving loops, harnesses that
 * forbid hipMalloc.  `dispatch_per_rank` / `combine_per_rank` are host arrays
 * of world_size entries as for pplx_a2a_world_dispatch / _combine (either may be
 * NULL to skip that half); the kernels and the results are the same.  The state
 * a world would own (slot map, routing tables) lives in an 8 MiB array that
 * is part of the library's code object on every GPU; a geometry that needs more
 * (world_size / dp_size * max_num_tokens * experts_per_token * 4 bytes of slot
 * map plus about world_size / dp_size * max_num_tokens * num_experts / 8 bytes of
 * routing tables), or more than 64 ranks, is refused with
 * PPLX_A2A_INVALID_ARGUMENT / PPLX_A2A_UNSUPPORTED.  The slot map written by a
 * dispatch stays there for the combine of a later call.  All calls on one GPU
 * share the array: calls that overlap in time on one GPU (different streams or
 * threads) race, and a step of a different geometry overwrites the slot map.
 * `fault_bits`: optional device word that the kernels OR the fault bits of
 * pplx_a2a_world_faults into (the caller clears and reads it); NULL discards them.
 * Calls no hipMalloc / hipFree and never synchronises.  The first call on a device looks the
 * array's address up (pplx_a2a_world_create on that device does the same): it cannot be made
 * under stream capture and returns PPLX_A2A_INVALID_STATE there. */
int pplx_a2a_static_step(const pplx_a2a_config_t *cfg, int device,
                         const pplx_a2a_dispatch_args_t *dispatch_per_rank,
                         const pplx_a2a_combine_args_t *combine_per_rank, uint32_t *fault_bits,
                         void *stream);

/* Parts of a step for pplx_a2a_world_abandon_step. */
#define PPLX_A2A_ABANDON_DISPATCH 1u
#define PPLX_A2A_ABANDON_COMBINE 2u

/* Drops the calls recorded so far for the dispatch and / or combine step (or split phase)
 * that is being assembled and returns that half of the world to idle, so that every rank can
 * call again.  For the caller whose rank r fails its argument checks after other ranks of the
 * step have called: nothing of a step reaches the GPU before its last rank has called, so the
 * recorded calls are forgotten and no kernel runs.  A split step between its SEND and RECV
 * phases is given up as a whole (what SEND staged is overwritten by the next SEND).
 * `dropped_calls` (optional) receives the number of recorded calls that were dropped.  The
 * reference has no such exit because it has no such state: a failed check there ends the
 * process (csrc/core/cuda_utils.h:7-14, csrc/core/utils.h:16-24).  Only host state changes:
 * no allocation, no synchronisation. */
int pplx_a2a_world_abandon_step(pplx_a2a_world_t *world, uint32_t which, uint32_t *dropped_calls);
/* Number of per-rank calls of `op` (0 = dispatch, 1 = combine) in `split_mode` that the world
 * has recorded and not launched yet; 0 once the last rank's call has enqueued the phase.  A
 * binding that keeps the callers' buffers alive for the ranks that called early reads this to
 * know when to let them go. */
int pplx_a2a_world_recorded_calls(pplx_a2a_world_t *world, int op, int split_mode, uint32_t *out);
/* The world a rank handle is attached to. */
pplx_a2a_world_t *pplx_a2a_world_of(const pplx_a2a_t *handle);

/* Allocates the staging that split send / recv calls go through (the reference
 * allocates its inboxes in the constructor, csrc/all_to_all/intranode.cpp:37-136;
 * here a world that never splits does not pay for them).  With G = world_size /
 * dp_size DP groups and M = max_num_tokens: G*M * (hidden_dim_bytes +
 * hidden_dim_scale_bytes + 4 * experts_per_token) bytes for dispatch (one copy
 * of every token, its scales and its picks) and, when expert_y_elem_bytes is not
 * 0, world_size*M * hidden_dim * 2 bytes for combine (one combined row per rank
 * and token, in the 2-byte dtype of out_tokens whatever expert_y holds; 2 and 4
 * ask for the same).  May be called again: what has been allocated stays where
 * it is until the world is destroyed, so graphs that recorded split calls remain
 * valid.  The first call (and the first that asks for combine staging)
 * allocates and clears memory, which synchronises the device. */
int pplx_a2a_world_reserve_split(pplx_a2a_world_t *world, uint32_t expert_y_elem_bytes);

/* Reads and clears the world's device-side fault word (synchronises `stream`):
 * bit 0 = a routed row did not fit out_expert_x_rows and was dropped,
 * bit 1 = an expert index >= num_experts was ignored,
 * bit 2 = combine met a slot beyond expert_y_rows,
 * bit 3 = an expert id repeated inside one token: the repeat took no row, was
 *         not counted and adds nothing in combine (the reference gives every
 *         pick a slot, csrc/all_to_all/intranode_dispatch.cu:139-144; top-k
 *         routing never repeats an expert),
 * bit 4 = a bound_m beyond max_num_tokens (or beyond m) was clamped
 *         (csrc/all_to_all/intranode_dispatch.cu:65 asserts). */
int pplx_a2a_world_faults(pplx_a2a_world_t *world, void *stream, uint32_t *out_bits);

/* ---- hipGraph plumbing ------------------------------------------------ */

/* Thin wrappers over stream capture so that a binding without HIP access can
 * record a dispatch+combine step once and replay it
 * (the reference's "CUDA graph support", README.md:5). */
int pplx_a2a_graph_begin_capture(void *stream);
int pplx_a2a_graph_end_capture(void *stream, pplx_a2a_graph_t **out);
int pplx_a2a_graph_launch(pplx_a2a_graph_t *graph, void *stream);
int pplx_a2a_graph_destroy(pplx_a2a_graph_t *graph);

/* ---- misc -------------------------------------------------------------- */

const char *pplx_a2a_last_error(void);
/* "major.minor.patch" of this library. */
const char *pplx_a2a_version(void);
/* Hash of the sources the library was built from (a binding can tell a stale build). */
const char *pplx_a2a_build_id(void);

#ifdef __cplusplus
}
#endif
#endif /* PPLX_A2A_H_ */
