/*
 * mlora.h — C-ABI of the MI355X (gfx950) multi-LoRA batched apply library.
 *
 * One shared library, plain pointers and sizes, no torch types.  Every entry
 * point enqueues work on the HIP stream it is given and returns without
 * synchronising, so all of them are legal under HIP graph capture.  Device
 * pointers are borrowed for the duration of the enqueued work only.
 *
 * Return value of every int-returning entry point: 0 on success, a negative
 * MLORA_E_* code for an argument the library rejects before launching
 * anything, or a positive hipError_t when a launch failed.  The text of the
 * last failure on the calling thread is available from mlora_last_error().
 *
 * Weight layout is the reference's: A_i is [slots, r, K] contiguous (K
 * fastest), B_i is [slots, N_i, r] contiguous (r fastest)
 * (reference: nanovllm_voxcpm/layers/lora.py:289-297,507-511,703-705,828-829).
 */
#ifndef MLORA_H_
#define MLORA_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLORA_ABI_VERSION 4

/* element types of x / y / A / B */
#define MLORA_DTYPE_F32 0
#define MLORA_DTYPE_F16 1
#define MLORA_DTYPE_BF16 2

/* which kernel family mlora_add_lora uses */
#define MLORA_FORM_AUTO 0  /* library chooses from shapes and the plan */
#define MLORA_FORM_TOKEN 1 /* one workgroup per token, any shape or dtype; needs no plan */
#define MLORA_FORM_BGMV 2  /* small tiles (<= 16 tokens of one slot), packed dot2 + wave64 reductions */
#define MLORA_FORM_SGMV 3  /* shrink launch + expand launch through the workspace: 64-token MFMA tiles for
                              segments >= threshold, one short tile each for the rest */
#define MLORA_FORM_MFMA 4  /* small tiles for every segment, both products on the matrix cores; one workgroup
                              per (tile, column range), each repeating its tile's shrink */
#define MLORA_FORM_SPLIT 5 /* small tiles, one launch: producer workgroups compute the rank-r intermediate of a
                              (tile, slice, K part) and publish it in the workspace, consumer workgroups take a
                              column range each, pick the intermediate up and expand; needs an initialised workspace */
#define MLORA_FORM_FUSED 6 /* the tiles of MLORA_FORM_SGMV in one launch: the workgroups of a group of tiles share
                              out its shrink, seal what they wrote to the workspace, wait for each other's seals
                              and expand a column range each; needs an initialised workspace */
#define MLORA_FORM_SLOT 7  /* MLORA_FORM_MFMA with the grid laid over the slots instead of the tiles: the workgroup of
                              (slot, column range) requests A[slot] from its own index alone, before the record of the
                              slot's first sixteen tokens has arrived; further tiles of a slot are
                              taken by extra workgroups of the same launch */

#define MLORA_FORM_WIDE 8  /* the tiles of MLORA_FORM_SGMV in one launch without anything passing between workgroups:
                              one workgroup per (tile, column range) multiplies the tile's x rows by A[slot] of the
                              range's slice over the whole of K, keeps the result in LDS and expands it into its
                              range; needs no workspace */

/* error codes (negative) */
#define MLORA_E_INVALID (-1)     /* malformed argument (NULL pointer, negative size, bad dtype) */
#define MLORA_E_UNSUPPORTED (-2) /* well-formed but outside what the selected form handles */
#define MLORA_E_TOO_LARGE (-3)   /* exceeds a compile-time capacity (slices, slots, rank) */

#define MLORA_MAX_SLICES 8
#define MLORA_MAX_SLOTS 1024 /* valid slot ids are [0, max_slots), max_slots <= this */
#define MLORA_MAX_RANK 256

/* One LoRA-wrapped slice of a stacked projection (q / k / v, gate / up, or
 * the only slice of o / down).  Replaces the per-slice pointer, stride and
 * column-start tables the reference uploads to the device
 * (reference: nanovllm_voxcpm/lora_ops/triton_ops/utils.py:15-116). */
typedef struct MloraSlice {
  const void* a;      /* A_i: [slots, r, K] contiguous */
  const void* b;      /* B_i: [slots, n, r] contiguous */
  int32_t n;          /* output columns of this slice */
  int32_t y_col;      /* first column of this slice inside y */
} MloraSlice;

/* Arguments of the fused apply:  for every token t with s = token_to_slot[t] >= 0
 * and every slice i:  y[t, y_col_i : y_col_i + n_i] += scaling * (x[t] . A_i[s]^T) . B_i[s]^T
 * with fp32 accumulation and a single rounding to the element type.  Rows with
 * s < 0 are not touched.
 * Replaces LoRABackend.add_lora (reference: nanovllm_voxcpm/lora.py:43-54, body
 * :241-381) including its shrink/expand grouping (:195-239, :299-381). */
typedef struct MloraAddArgs {
  void* stream;           /* hipStream_t */
  const void* x;          /* [T, K], row stride x_stride elements, unit column stride */
  void* y;                /* [T, >= max(y_col_i + n_i)], row stride y_stride elements */
  int64_t x_stride;
  int64_t y_stride;
  const int32_t* token_to_slot; /* [T] on device */
  const int32_t* plan;    /* workspace filled by mlora_meta_build for this token_to_slot, or NULL
                             (NULL is accepted by MLORA_FORM_TOKEN and makes AUTO choose it).  Read-only
                             for mlora_add_lora too, but for the header word MLORA_PLAN_REJECTED (an
                             atomic count): calls on any number of streams may share one plan.  A return
                             value of 0 does not say that the plan matched the call: see that word */
  int32_t num_tokens;     /* T */
  int32_t k;              /* K, input features */
  int32_t r;              /* rank dimension of the A/B buffers (max_lora_rank) */
  int32_t num_slots;      /* first dimension of A_i / B_i */
  int32_t num_slices;     /* <= MLORA_MAX_SLICES */
  int32_t dtype;          /* MLORA_DTYPE_* of x, y, A and B */
  int32_t form;           /* MLORA_FORM_* */
  float scaling;
  MloraSlice slices[MLORA_MAX_SLICES];
  void* workspace;        /* device scratch for the rank-r intermediate: between the producer and the
                             consumer workgroups of MLORA_FORM_SPLIT and between the two launches of
                             MLORA_FORM_SGMV; 256-byte aligned and at least MLORA_WORKSPACE_HEAD_BYTES
                             long, or NULL (AUTO then keeps to MLORA_FORM_MFMA).  Counterpart of the
                             [S, T, r] buffer the reference allocates between its two kernels
                             (reference: nanovllm_voxcpm/lora.py:299-381).  Pass it to
                             mlora_workspace_init once after allocating it; calls that share a
                             workspace must be ordered on one stream. */
  int64_t workspace_bytes; /* >= mlora_add_workspace_bytes(T, num_slices, r, dtype) lets every form be used */
  const int32_t* effective_rank; /* [num_slots] on device, or NULL: rank of the adapter resident in each slot
                             of THESE buffers (0: none).  Rows of A_i[s] and columns of B_i[s] at or
                             above effective_rank[s] are then neither read nor multiplied, so a slot
                             costs what its own rank costs, not what the padded rank costs.  The
                             reference keeps this vector per layer
                             (reference: nanovllm_voxcpm/layers/lora.py:409-417) and relies on the
                             padding being zero; with NULL this library does the same. */
} MloraAddArgs;

int mlora_add_lora(const MloraAddArgs* args);

/* The same fused apply for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  args->workspace and args->workspace_bytes are ignored: the scratch is an array of
 * MLORA_STATIC_SCRATCH_BYTES bytes that lives in the library's device image, one copy per GPU, held
 * until the process ends.  The call allocates and frees nothing.  It returns MLORA_E_TOO_LARGE when
 * one fp32 copy of the rank-r intermediate (num_tokens x num_slices x r x 4 bytes) does not fit the
 * array, whatever form the call would take.  Every call on a GPU shares that GPU's array: calls that
 * overlap in time on one GPU (two streams, two threads) race on it and must be ordered by the
 * caller.  The first call on a device looks the array's address up and must be made outside stream
 * capture (a call with num_tokens = 0 is enough); a first call inside a capture is refused. */
#define MLORA_STATIC_SCRATCH_BYTES (16u << 20)
int mlora_add_lora_static(const MloraAddArgs* args);

/* Bytes of MloraAddArgs.workspace that let mlora_add_lora use every form it has for this shape
 * (a smaller workspace of at least MLORA_WORKSPACE_HEAD_BYTES is legal: the two-launch form then
 * splits K less, or AUTO does not choose it). */
size_t mlora_add_workspace_bytes(int32_t num_tokens, int32_t num_slices, int32_t r, int32_t dtype);

/* A workspace starts with a head of MLORA_WORKSPACE_HEAD_BYTES bytes: a signature word, the
 * workspace's {generation, arrivals} pair (advanced once per launch that uses the head), the area
 * in which producer workgroups of MLORA_FORM_SPLIT leave the intermediate for the consumers, every
 * word tagged with the generation, and the seals (generation and XCD of the writer) that the
 * workgroups of MLORA_FORM_FUSED put on the partial sums they wrote.  mlora_workspace_init enqueues one kernel that clears the head and writes the
 * signature; call it once after allocation (it is a kernel, not a memset, so it may be recorded
 * into a graph).  Launches leave the head ready for the next launch.  A workspace whose head
 * is not in the state the initialisation or a launch left it in (no signature, or a generation,
 * arrival count and check word that do not fit each other) is still safe to pass: the kernels
 * then compute every intermediate locally and never read the exchange area.  Initialise every
 * workspace once all the same: memory that held a workspace before is not told apart from one
 * by more than those words.  No counterpart in the reference. */
#define MLORA_WORKSPACE_HEAD_BYTES (16384 + (4 << 20) + (64 << 10))
int mlora_workspace_init(void* workspace, int64_t workspace_bytes, void* stream);

/* Unfused shrink:  out[i, t, 0:r] = scaling * x[t] . A_i[s_t]^T  for s_t >= 0, and 0
 * for rows with s_t < 0 (the reference zero-fills the buffer first).
 * Replaces lora_shrink (reference:
 * nanovllm_voxcpm/lora_ops/triton_ops/lora_shrink_op.py:257-341). */
typedef struct MloraShrinkArgs {
  void* stream;
  const void* x;          /* [T, K] */
  void* out;              /* [S, T, r] contiguous, element type out_dtype */
  int64_t x_stride;
  const int32_t* token_to_slot;
  int32_t num_tokens, k, r, num_slots, num_slices;
  int32_t dtype;          /* of x and A */
  int32_t out_dtype;      /* of out */
  float scaling;
  const void* a[MLORA_MAX_SLICES];
} MloraShrinkArgs;

int mlora_shrink(const MloraShrinkArgs* args);

/* Unfused expand:  y[t, c_i : c_i + n_i] (+)= h[i, t] . B_i[s_t]^T for s_t >= 0 where
 * c_i = offset_start + n_0 + ... + n_{i-1}.  The product is rounded to B's element type
 * before it is added (add_inputs != 0) or stored (add_inputs == 0), as the reference does.
 * Replaces lora_expand (reference:
 * nanovllm_voxcpm/lora_ops/triton_ops/lora_expand_op.py:94-170). */
typedef struct MloraExpandArgs {
  void* stream;
  const void* h;          /* [S, T, r] contiguous, element type h_dtype */
  void* y;                /* [T, *], row stride y_stride elements, element type dtype */
  int64_t y_stride;
  const int32_t* token_to_slot;
  int32_t num_tokens, r, num_slots, num_slices;
  int32_t dtype;          /* of B and y */
  int32_t h_dtype;
  int32_t offset_start;
  int32_t add_inputs;
  const void* b[MLORA_MAX_SLICES];
  int32_t n[MLORA_MAX_SLICES];
} MloraExpandArgs;

int mlora_expand(const MloraExpandArgs* args);

/* ---- segment metadata built on the device from the slot-id vector ------------------ */

/* Bytes of plan workspace needed for num_tokens tokens and max_slots slots. */
size_t mlora_plan_workspace_bytes(int32_t num_tokens, int32_t max_slots);

/* Header words of a plan workspace (int32 index). */
#define MLORA_PLAN_MAGIC 0
#define MLORA_PLAN_NUM_TOKENS 1
#define MLORA_PLAN_MAX_SLOTS 2
#define MLORA_PLAN_NUM_LORA_TOKENS 3 /* tokens with a valid slot */
#define MLORA_PLAN_NUM_ACTIVE 4      /* distinct valid slots in use */
#define MLORA_PLAN_NO_LORA 5         /* 1 iff no token has a valid slot */
#define MLORA_PLAN_BAD_SLOT 6        /* 1 iff some slot id was >= max_slots (treated as -1) */
#define MLORA_PLAN_TILES_SHORT 7     /* small tiles of segments below the threshold */
#define MLORA_PLAN_TILES_LONG_SMALL 8 /* small tiles of segments at or above the threshold */
#define MLORA_PLAN_TILES_LONG_BIG 9  /* big tiles of segments at or above the threshold */
#define MLORA_PLAN_MAX_SEGMENT 10    /* longest segment */
#define MLORA_PLAN_TILES_OVER 11     /* small tiles that are not the first tile of their slot */
#define MLORA_PLAN_REJECTED 12       /* launches of mlora_add_lora that found this plan built for another
                                        (num_tokens, max_slots) or not built at all and therefore left y as it
                                        was: the one word of a plan that the apply kernels write (atomically) */
#define MLORA_PLAN_HEADER_WORDS 16
#define MLORA_PLAN_MAGIC_VALUE 0x4d4c5031 /* "MLP1" */

/* Segment length from which a segment gets big (prefill) tiles, and the two tile heights. */
#define MLORA_SEGMENT_THRESHOLD 16
#define MLORA_TILE_SMALL 16
#define MLORA_TILE_BIG 64
/* A small tile is a self-contained 128-byte record, so that a workgroup learns everything it
 * needs from one load: words {slot, token count, first position in sorted_idx, 0}, then 16
 * token indices (the tile's tokens in order; entries past the count repeat them cyclically, so
 * all sixteen name rows of the tile itself), then padding.
 * A big tile is four words {slot, first position in sorted_idx, token count, 0}; behind the
 * big-tile records lies one list of MLORA_TILE_BIG token indices per big tile (its tokens in
 * order, 0 past the count: a valid row to read), at a place that follows from the tile's place
 * alone: a workgroup requests it together with the record.  The list of big tiles (capacity: with
 * most = num_tokens / 64 + min(max_slots, num_tokens) and root the smallest integer with
 * 8 root^2 >= most, (most + 8 (root + 2) + 31) & ~31) is cut into eight equal blocks, one per
 * XCD (workgroup (x, ., z) of a launch takes place x * capacity / 8 + z).  The big tiles of a plan are
 * sorted by slot; runs of consecutive tiles go to the blocks in turn (tile t of run i = t / run at
 * (i % 8) * capacity / 8 + (i / 8) * run + t % run), where run = ceil(n / (8 k)) for n tiles and
 * k = ceil(n / (8 * floor(n / slots that have big tiles))): runs about as long as a slot's segment
 * has tiles, so that a slot meets few XCDs and its weights are fetched into few L2s, and of one tile
 * when the slots have one tile each.  Places without a tile hold {-1, 0, 0, 0}. */
#define MLORA_SMALL_TILE_WORDS 32
#define MLORA_SMALL_TILE_ROWS 4 /* word index of the first token index inside a record */
#define MLORA_BIG_TILE_WORDS 4
/* Behind the row lists of the big tiles the same small tiles are listed a second time, by slot: one
 * 128-byte record per slot id (its place follows from the slot id alone: a workgroup that serves a
 * slot can request the slot's weights before it knows the slot's tokens) for the slot's first
 * sixteen tokens, then one record for every further small tile of every slot (unused ones carry
 * count 0).  Words {slot, token count, first position in sorted_idx, MLORA_PLAN_CHECK(T, L)}, then
 * the sixteen token indices as in a small-tile record. */
#define MLORA_PLAN_CHECK(num_tokens, max_slots) \
  (0x4d4c5031u ^ (uint32_t)(num_tokens) ^ ((uint32_t)(max_slots) << 20))

/* Arguments of the on-device metadata build: a stable counting sort of the tokens by
 * slot id.  The plan workspace (always written when non-NULL) feeds mlora_add_lora; the
 * optional outputs reproduce, bit for bit, the three index layouts the reference builds
 * on the host:
 *   compact, -1 left out   — engine path (reference: nanovllm_voxcpm/engine/lora_manager.py:77-91)
 *                            and torch builder (nanovllm_voxcpm/utils/context.py:77-116)
 *   compact, -1 as a bucket — LoRAKernelMeta.prepare_tensors
 *                            (nanovllm_voxcpm/lora_ops/triton_ops/lora_kernel_metadata.py:46-68)
 *   dense by slot id        — graph buffers (nanovllm_voxcpm/engine/model_runner.py:743-797)
 * Any output pointer may be NULL. */
typedef struct MloraMetaArgs {
  void* stream;
  const int32_t* token_to_slot; /* [T] on device */
  int32_t num_tokens;           /* T */
  int32_t max_slots;            /* L <= MLORA_MAX_SLOTS */
  int32_t no_lora_bucket;       /* 0: tokens with slot -1 are left out of every output;
                                   1: they form the first bucket (id -1) of sorted_idx and the
                                      compact arrays (not of the plan) */
  int32_t* plan;                /* mlora_plan_workspace_bytes(T, L) bytes, or NULL */
  int32_t* sorted_idx;          /* token indices grouped by slot, ascending inside a slot */
  int32_t* compact_ids;         /* [compact_capacity], unused tail filled with -1 */
  int32_t* compact_counts;      /* [compact_capacity], unused tail filled with 0 */
  int32_t* compact_offsets;     /* [compact_capacity + 1]: 0, running totals, unused tail 0 */
  int32_t compact_capacity;
  int32_t* dense_counts;        /* [L + 1], index slot + 1; entry 0 (slot -1) is always 0 */
  int32_t* dense_offsets;       /* [L + 2]: 0 followed by the running totals of dense_counts */
  int32_t* padded_token_to_slot; /* [padded_len]: copy of token_to_slot, tail filled with -1 */
  int32_t padded_len;
  int32_t* scalars;             /* [4]: number of buckets written to the compact arrays, number
                                   of entries written to sorted_idx, no_lora flag, bad_slot flag */
} MloraMetaArgs;

int mlora_meta_build(const MloraMetaArgs* args);

/* Fused slot install:  A[slot, :, :] = 0; A[slot, 0:rank, :] = a_src[0:rank, :];
 * B[slot, :, :] = 0; B[slot, :, 0:rank] = b_src[:, 0:rank] * scaling  in one launch.
 * Replaces the zero / copy / scale sequence of set_slot_lora
 * (reference: nanovllm_voxcpm/layers/lora.py:395-417, 599-621, 744-762, 851-869). */
typedef struct MloraInstallArgs {
  void* stream;
  void* a_dst;            /* [slots, r, K] */
  void* b_dst;            /* [slots, n, r] */
  const void* a_src;      /* [>= rank, K], row stride a_src_stride elements */
  const void* b_src;      /* [n, >= rank], row stride b_src_stride elements */
  int64_t a_src_stride, b_src_stride;
  int32_t slot, k, n, r, rank;
  int32_t dtype;          /* of the destination buffers */
  int32_t src_dtype;      /* of a_src and b_src */
  float scaling;
  int32_t num_slots;      /* first dimension of a_dst / b_dst: slot >= num_slots is rejected */
} MloraInstallArgs;

int mlora_install_slot(const MloraInstallArgs* args);

/* Identifier of the graph capture in progress on `stream`, 0 when the stream is not
 * capturing.  No counterpart in the reference: lets a host-side cache tell work recorded
 * into one capture from work run eagerly or recorded into another capture. */
uint64_t mlora_stream_capture_id(void* stream);

/* Library identification and diagnostics. */
int mlora_abi_version(void);
const char* mlora_last_error(void);
const char* mlora_build_info(void);

#ifdef __cplusplus
}
#endif
#endif /* MLORA_H_ */
