/*
 * fsta.h -- C ABI of libfsta: fused sparse tree attention for AMD MI355X (gfx950).
 *
 * Every pointer is a DEVICE pointer unless its comment says "host".  `stream`
 * is a hipStream_t passed as void* (NULL = the null stream).  All entry points
 * only enqueue work on `stream`; none synchronises, allocates or frees memory.
 * Return value: FSTA_OK or a negative FSTA_E* code; fsta_last_error() then
 * gives a message for the calling thread.
 *
 * Tensors are dense row-major ("contiguous") with the shapes given below.
 * Conventions shared with the reference: node ids are int64, -1 marks an empty
 * slot, ancestor_mask is one byte per entry (0/1).
 */
#ifndef FSTA_H
#define FSTA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FSTA_ABI_VERSION 2

/* element types of q/k/v/o */
#define FSTA_F32  0
#define FSTA_F16  1
#define FSTA_BF16 2
#define FSTA_F64  3  /* fsta_medusa_tree's probabilities only */

/* return codes */
#define FSTA_OK            0
#define FSTA_EINVAL       -1  /* argument outside the documented domain      */
#define FSTA_EUNSUPPORTED -2  /* valid but not built (head_dim, block size)   */
#define FSTA_EHIP         -3  /* the HIP runtime reported an error            */

/* flags of fsta_attention_fwd */
#define FSTA_FLAG_FAST_PV   1u /* bf16 only: feed P to the matrix cores as one bf16
                                  value instead of a hi+lo pair (about 2^-9 relative
                                  error per weight instead of 2^-17)            */
#define FSTA_FLAG_GENERIC   2u /* force the scalar-ALU kernel (any dtype)      */
#define FSTA_FLAG_WIDE_WAVES 4u /* matrix-core kernel with 32 query rows per wave
                                  (32x32x16 MFMA, 2 waves per SIMD) instead of 16
                                  rows per wave (16x16x32 MFMA, 4 waves per SIMD) */

#define FSTA_FLAG_SHARE_TILES 8u /* tuning: where two waves share a group of 16 query rows they
                                  always take alternate key tiles (and merge at the end), never
                                  halves of the head dimension                              */
#define FSTA_FLAG_STREAM 16u    /* tuning/tests: workgroups that stay and walk a list of query blocks
                                  * (the streaming kernel, one launch of as many workgroups as the GPU
                                  * holds) wherever the shape allows: block_m 64/128, head_dim 64/128,
                                  * 16-bit types, no prefix, a block plan.  Measured slower than one
                                  * workgroup per block, so the library never takes it by itself. */
#define FSTA_FLAG_KEY_SPLITS(n) (((uint32_t)(n) & 0xffu) << 8)
                               /* fsta_attention_fwd_ws / fsta_attention_workspace_bytes:
                                  cut the shared prefix into n runs of keys (n = 1: never
                                  split; n = 0, i.e. no such flag: the library decides)   */

/* bits of the status word written by fsta_precompute */
#define FSTA_PRE_TOO_MANY_ANCESTORS 1u /* a block has more than max_ancestors unique ancestors */
#define FSTA_PRE_BAD_NODE_ID        2u /* lineage entry < -1 or >= n_nodes                      */
#define FSTA_PRE_BAD_LEVEL          4u /* level_lookup entry outside [-width, width)            */
/* bit of the status word written by fsta_medusa_tree */
#define FSTA_TREE_NOT_PREFIX_CLOSED 8u /* a kept path's parent path was not kept (probabilities
                                          above 1 or not numbers)                                */

int fsta_abi_version(void);

/* Message of the last failing call made by this thread ("" if none). */
const char* fsta_last_error(void);

/* Which attention kernel the last fsta_attention_fwd* call of this thread launched, as
 * "name<template arguments>" in the spelling profilers show (e.g. rocprofv3's kernel trace),
 * followed by launch options; "" before the first launch.  For benchmarks and profiles. */
const char* fsta_last_attention_kernel(void);

/* Number of 32-bit words per (block, query row) in the packed tree mask. */
int32_t fsta_mask_words(int32_t max_ancestors);

/*
 * Size in bytes of the block plan of a tree (0 when block_m is not 32, 64 or
 * 128: the kernel that reads plans takes no other block size).  The plan is the
 * same information as ancestor_idx / leaf_idx / mask_bits / anc_count in the
 * form the matrix-core attention kernel consumes without any per-launch
 * preparation: per query block a record of 32-bit words
 *   [0] anc_count  [1..3] 0  [4..7] leaf validity, one word per 32 rows
 *   [8 ..)  32 * T ancestor keys (T = ceil(max_ancestors / 32)): K/V row of
 *           every slot; an empty slot repeats a valid row of the block
 *   then per group of 32 query rows: 32 leaf keys (K/V row of each row's own
 *           key, an empty slot repeats a valid row), then T x 32 mask words
 *           (word t of row r: bit b = row r attends ancestor slot 32 t + b;
 *           bits of empty slots are 0)
 * Records are 16-byte aligned and follow each other block by block.  No
 * counterpart in the reference, whose kernel re-reads the int64 lists and the
 * byte mask in every program (fstattention.py:61-67).
 */
size_t fsta_block_plan_bytes(int32_t num_blocks, int32_t block_m, int32_t max_ancestors);

/*
 * Per-block tree precompute on the GPU; replaces the host loop of
 * create_fst_attention_kernel_inputs (reference utils.py:104-129) and is
 * bit-exact with it:
 *   ancestor_idx  [num_blocks, max_ancestors]           int64  (utils.py:112,119-120)
 *   ancestor_mask [num_blocks, block_m, max_ancestors]  bool   (utils.py:113,126-127)
 *   leaf_idx      [num_blocks, block_m]                 int64  (utils.py:114,121-122)
 * with num_blocks = ceil(n_nodes / block_m); ancestor_mask may be NULL when only
 * the packed form is wanted.  Extra outputs for the attention kernels (each
 * may be NULL):
 *   mask_bits     [num_blocks, fsta_mask_words(A), block_m] uint32, bit b of
 *                 word w of row r = ancestor_mask[j, r, 32*w + b]
 *   anc_count     [num_blocks] int32, number of valid entries of ancestor_idx[j]
 *   block_plan    fsta_block_plan_bytes(num_blocks, block_m, A) bytes, 16-byte
 *                 aligned (block_m 32, 64 or 128 only, else it must be NULL)
 * lineage [n_nodes, width] int64 and level_lookup [n_nodes] int64 follow the
 * layout of utils.py:43-44,66-75.  With mutate_lineage != 0 each node id is
 * written into its own level column of `lineage`, as utils.py:124-125 does to
 * the caller's tensor.  `status` (one uint32, must be zero on entry) receives
 * FSTA_PRE_* bits; where the reference raises (utils.py:120) the bit
 * FSTA_PRE_TOO_MANY_ANCESTORS is set and the surplus ancestors are dropped.
 * Alignment: lineage, level_lookup, ancestor_idx, leaf_idx 8 bytes; mask_bits,
 * anc_count, status 4 bytes.
 */
int fsta_precompute(int64_t* lineage, const int64_t* level_lookup,
                    int64_t n_nodes, int64_t width,
                    int32_t block_m, int32_t max_ancestors, int32_t mutate_lineage,
                    int64_t* ancestor_idx, uint8_t* ancestor_mask, int64_t* leaf_idx,
                    uint32_t* mask_bits, int32_t* anc_count, uint32_t* block_plan,
                    uint32_t* status, void* stream);

/*
 * Packs a boolean ancestor_mask [num_blocks, block_m, max_ancestors] (one byte
 * per entry, the tensor utils.py:104-129 returns) into mask_bits (layout above)
 * and counts, per block, the leading slots of ancestor_idx up to and including
 * the last non-negative one into anc_count.  Bits of slots whose ancestor_idx
 * is negative are cleared.  With block_plan != NULL (then leaf_idx
 * [num_blocks, block_m] int64 is required, block_m 32, 64 or 128) the block
 * plan of these lists is written as well; ids outside [0, key_limit) count as
 * empty slots there (key_limit = number of K/V rows the lists address).
 * Alignment: ancestor_idx, leaf_idx 8 bytes; mask_bits, anc_count 4 bytes;
 * block_plan 16 bytes.
 */
int fsta_pack_mask(const int64_t* ancestor_idx, const uint8_t* ancestor_mask,
                   const int64_t* leaf_idx,
                   int32_t num_blocks, int32_t block_m, int32_t max_ancestors, int64_t key_limit,
                   uint32_t* mask_bits, int32_t* anc_count, uint32_t* block_plan, void* stream);

/*
 * Fused sparse tree attention forward; replaces fst_attention/_fwd_kernel
 * (reference fstattention.py:153-181, 21-151).
 *   q [batch, heads, nq, head_dim], k, v [batch, heads, nk, head_dim] of `dtype`;
 *   o [batch, heads, nq, head_dim] of `out_dtype` (= dtype, or FSTA_F32);
 *   lse [batch*heads, nq] float32 or NULL: base-2 log-sum-exp of the scaled
 *   scores times log2(e) (fstattention.py:139-141).
 * Query block j = rows [j*block_m, (j+1)*block_m) attends, per row r, to
 *   - K/V rows ancestor_idx[j, c] for the columns c whose mask bit is set,
 *   - K/V row leaf_idx[j, r] if that is >= 0 (fstattention.py:86-91,104-107),
 *   - K/V rows [0, nk - nq), the shared dense prefix (fstattention.py:113-136),
 * with weights softmax(q.k * sm_scale) over that set.  Negative indices and
 * indices >= nk are skipped.  nq need not be a multiple of block_m (the rows
 * past nq are neither read nor written) and the prefix may have any length;
 * num_blocks must equal ceil(nq / block_m).  A row that attends to nothing
 * gets o = 0 and lse = -inf.
 * head_dim in {16,32,64,128}; block_m in {16,32,64,128}; max_ancestors >= 1.
 * block_plan (may be NULL): the block plan of the same lists, as written by
 * fsta_precompute or fsta_pack_mask with these block_m / max_ancestors;
 * plan_key_shift is added to the plan's keys (the caller has added it to the
 * valid entries of ancestor_idx and leaf_idx since the plan was made, e.g. the
 * prefix length, fstattention.py:211-212).  The fastest kernel (16-bit types,
 * head_dim >= 32, block_m >= 32) reads the plan only; without a plan a slower
 * matrix-core kernel reads the lists themselves.  With a plan, the lists are
 * still read by the kernels that serve the shapes the fast one does not take.
 * Alignment: q, k, v, o and block_plan 16 bytes (rows are moved 16 bytes at a
 * time); ancestor_idx and leaf_idx 8 bytes; mask_bits, anc_count and lse 4 bytes.
 * batch * heads <= 65535.  The matrix-core kernels address one (batch, head)
 * slice of K or V with 32-bit byte offsets: slices of 4 GiB and more
 * (nk * head_dim * 2 bytes) are served by the slower vector-ALU kernel.
 */
int fsta_attention_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                       const int64_t* ancestor_idx, const uint32_t* mask_bits,
                       const int32_t* anc_count, const int64_t* leaf_idx,
                       const uint32_t* block_plan, int32_t plan_key_shift,
                       int32_t batch, int32_t heads, int32_t nq, int32_t nk, int32_t head_dim,
                       int32_t dtype, int32_t out_dtype,
                       int32_t block_m, int32_t max_ancestors, int32_t num_blocks,
                       float sm_scale, uint32_t flags, void* stream);

/*
 * The same operation with a device workspace, which lets the library cut a long
 * shared prefix (fstattention.py:113-136: every query block walks all nk - nq
 * prefix keys on its own) into runs of keys that separate workgroups take
 * ("flash decoding"): when batch * heads * num_blocks workgroups cannot fill
 * the GPU, e.g. one sequence with a long KV cache in front of a small tree, the
 * prefix is read several times faster.  Each run yields a float32 partial
 * result with its log-sum-exp in the workspace; the launch that takes the tree
 * part (or a small second kernel, where that launch cannot) joins them into o
 * (and lse).  Results are those of fsta_attention_fwd up to float32 rounding of
 * the join.
 *   fsta_attention_workspace_bytes: bytes of device memory (256-byte aligned
 *     start) fsta_attention_fwd_ws wants for this problem; 0 when it would not
 *     split (short or no prefix, enough blocks, dtype/shape of the scalar kernel).
 *   fsta_attention_fwd_ws: `workspace` of at least that many bytes, or NULL / a
 *     smaller size to run without splitting (then identical to
 *     fsta_attention_fwd).  The workspace is free again when the work queued on
 *     `stream` has run; calls that share one workspace must not overlap.
 * `flags` must be the same in both calls; FSTA_FLAG_KEY_SPLITS(n) forces n runs.
 * Both the runs of keys and the dense prefix kernel read the block plan: a call
 * with block_plan = NULL ignores the workspace and walks the prefix unsplit in one
 * launch (correct, slower), whatever fsta_attention_workspace_bytes said -- that
 * function has no plan argument and answers for a caller that passes one.
 */
size_t fsta_attention_workspace_bytes(int32_t batch, int32_t heads, int32_t nq, int32_t nk,
                                      int32_t head_dim, int32_t dtype, int32_t block_m,
                                      int32_t max_ancestors, float sm_scale, uint32_t flags);
int fsta_attention_fwd_ws(const void* q, const void* k, const void* v, void* o, float* lse,
                          const int64_t* ancestor_idx, const uint32_t* mask_bits,
                          const int32_t* anc_count, const int64_t* leaf_idx,
                          const uint32_t* block_plan, int32_t plan_key_shift,
                          int32_t batch, int32_t heads, int32_t nq, int32_t nk, int32_t head_dim,
                          int32_t dtype, int32_t out_dtype,
                          int32_t block_m, int32_t max_ancestors, int32_t num_blocks,
                          float sm_scale, uint32_t flags,
                          void* workspace, size_t workspace_bytes, void* stream);

/*
 * The same operation on K and V stored as 8-bit floats: k8, v8 [batch, heads, nk,
 * head_dim] bytes in the OCP e4m3 format ("float8_e4m3fn": 1 sign, 4 exponent, 3
 * mantissa bits, no infinities), with one float32 scale per (batch, head) slice
 * each (k_scale, v_scale [batch*heads], NULL = 1): the keys are k8 * k_scale, the
 * values v8 * v_scale.  q and o stay 16-bit (dtype FSTA_F16 / FSTA_BF16; out_dtype
 * = dtype or FSTA_F32) and all arithmetic is that of fsta_attention_fwd: the rows
 * are widened exactly in the kernel, so the result is fsta_attention_fwd's on the
 * widened K and V.  Half the K/V bytes travel.  No counterpart in the reference
 * (16-bit tensors only).  Needs the block plan (no index lists are read);
 * head_dim 64 or 128, block_m 32, 64 or 128, sm_scale > 0; other shapes are
 * refused with FSTA_EUNSUPPORTED.  Alignment: q, k8, v8, o, block_plan 16 bytes;
 * k_scale, v_scale, lse 4 bytes.
 */
int fsta_attention_fwd_kv8(const void* q, const void* k8, const void* v8, const float* k_scale,
                           const float* v_scale, void* o, float* lse, const uint32_t* block_plan,
                           int32_t plan_key_shift, int32_t batch, int32_t heads, int32_t nq, int32_t nk,
                           int32_t head_dim, int32_t dtype, int32_t out_dtype, int32_t block_m,
                           int32_t max_ancestors, int32_t num_blocks, float sm_scale, void* stream);

/*
 * parent[n_nodes] int64 (parent[i] < i, -1 for roots) -> level_lookup [n_nodes]
 * and lineage [n_nodes, width] in the layout of utils.py:66-75 (strict ancestor
 * a of i at lineage[i, level(a)], -1 elsewhere).  `status` (zero on entry) gets
 * FSTA_PRE_BAD_NODE_ID for an entry outside [-1, i) and FSTA_PRE_BAD_LEVEL when
 * a node is deeper than width-1.  With lineage == NULL only level_lookup is
 * written (to size `width` first).  Front-end for trees that are rebuilt on the
 * GPU every decoding step; the reference builds lineage on the host only
 * (utils.py:66-75).
 */
int fsta_lineage_from_parents(const int64_t* parent, int64_t n_nodes, int64_t width,
                              int64_t* lineage, int64_t* level_lookup, uint32_t* status,
                              void* stream);

/*
 * fsta_lineage_from_parents and fsta_precompute in one launch, for the trees of a
 * decoding step that is rebuilt every step (README.md:15-16): every workgroup
 * copies parent[n_nodes] into its LDS, builds the lineage rows of its own query
 * block there (layout of utils.py:66-75, `width` columns) and goes on as
 * fsta_precompute does (utils.py:104-129), without the lineage ever travelling
 * through memory.  Outputs and status bits are those of fsta_precompute on the
 * lineage of fsta_lineage_from_parents, bit for bit; lineage [n_nodes, width] and
 * level_lookup [n_nodes] are optional outputs here (NULL: not written), lineage
 * with each node's id in its own level column when insert_self != 0 (what
 * fsta_precompute leaves in the caller's tensor).  A tree deeper than width - 1
 * sets FSTA_PRE_BAD_LEVEL, a parent entry outside [-1, i) FSTA_PRE_BAD_NODE_ID
 * (such a node counts as a root).  Everything lives in one workgroup's LDS:
 * 4 * (n_nodes + block_m * width) bytes beside fsta_precompute's tables, 160 KB in
 * all -- about 16000 nodes at width 64, block_m 128; larger problems are refused
 * with FSTA_EUNSUPPORTED (use the two calls).  No counterpart in the reference.
 * Alignment as fsta_precompute; parent 8 bytes.
 */
int fsta_precompute_from_parents(const int64_t* parent, int64_t n_nodes, int64_t width, int32_t block_m,
                                 int32_t max_ancestors, int32_t insert_self, int64_t* lineage,
                                 int64_t* level_lookup, int64_t* ancestor_idx, uint8_t* ancestor_mask,
                                 int64_t* leaf_idx, uint32_t* mask_bits, int32_t* anc_count,
                                 uint32_t* block_plan, uint32_t* status, void* stream);

/*
 * Depth-first (pre-order) renumbering of a forest, the node order the reference
 * names as its open item (README.md:19-20: blocks of consecutive ids then share
 * lineage and their ancestor lists shrink).  parent[n_nodes] int64 as above ->
 * perm[new_id] = old_id and rank[old_id] = new_id, both int64 [n_nodes].
 * Siblings (and roots) are visited by ascending id, or smallest subtree first
 * (ties by id) when light_first != 0.  workspace:
 * FSTA_DFS_ORDER_WORKSPACE_INTS(n_nodes) int32 of device scratch.  `status` gets
 * FSTA_PRE_BAD_NODE_ID for a parent entry outside [-1, i); perm and rank are then
 * the identity.  Bits already set in `status` on entry (earlier stages of a
 * front-end chain may share the word) are left alone and do not change the result.  n_nodes <= FSTA_DFS_ORDER_MAX_NODES (2^17, the
 * largest entry of the reference's size table, utils.py:4-13).  Work is
 * O(n_nodes * depth + sum over parents of children^2).
 */
#define FSTA_DFS_ORDER_MAX_NODES 131072
#define FSTA_DFS_ORDER_WORKSPACE_INTS(n) (6 * (size_t)(n) + 8)
int fsta_dfs_order(const int64_t* parent, int64_t n_nodes, int32_t light_first, int64_t* perm,
                   int64_t* rank, int32_t* workspace, uint32_t* status, void* stream);

/*
 * fsta_dfs_order without a workspace argument and without any allocation: the
 * scratch is an array inside the library, one copy per GPU, held until the
 * process ends (384 KiB).  No counterpart in the reference; for
 * callers that cannot allocate device memory: code under HIP graph capture,
 * serving loops and harnesses that forbid hipMalloc.  Same arguments, results
 * and status bits as fsta_dfs_order; n_nodes <= FSTA_DFS_ORDER_STATIC_MAX_NODES,
 * larger trees are refused with FSTA_EUNSUPPORTED.  All calls on one GPU share
 * that GPU's array: calls that overlap on one GPU (two streams, two threads)
 * race, queue them on one stream or order them with events.  The first call on
 * a device looks the array's address up (hipGetSymbolAddress under a mutex; no
 * memory is allocated): make that first call outside stream capture, later calls
 * may be captured.  The array used is the one of the CURRENT device, which must be
 * the device `stream` belongs to.
 */
#define FSTA_DFS_ORDER_STATIC_MAX_NODES 16384
int fsta_dfs_order_static(const int64_t* parent, int64_t n_nodes, int32_t light_first, int64_t* perm,
                          int64_t* rank, uint32_t* status, void* stream);

/*
 * Joins two partial attention results of the same queries over disjoint key
 * sets: o = (o_a 2^lse_a + o_b 2^lse_b) / (2^lse_a + 2^lse_b) per row, lse_out
 * (may be NULL) = log2 of the denominator.  o_*: [rows, head_dim] of `dtype`,
 * lse_*: float32 [rows], base 2 as written by fsta_attention_fwd (reference
 * fstattention.py:139-141, which computes L and drops it).  A part with
 * lse = -inf carries no keys and is ignored.  With it the dense shared prefix
 * of fstattention.py:113-136 can come from any kernel that reports its
 * log-sum-exp.  o_out may alias o_a or o_b.  head_dim a multiple of 8.
 */
int fsta_merge_states(const void* o_a, const float* lse_a, const void* o_b, const float* lse_b,
                      void* o_out, float* lse_out, int64_t rows, int32_t head_dim, int32_t dtype,
                      void* stream);

/*
 * new_parent[rank[i]] = rank[parent[i]] (-1 for roots): the parent array of the same
 * forest after node i has been renamed rank[i], e.g. with the rank of
 * fsta_dfs_order.  No counterpart in the reference (see fsta_dfs_order).  rank must
 * be a permutation of 0 .. n_nodes-1; new_parent must not alias parent.
 */
int fsta_renumber_parents(const int64_t* parent, const int64_t* rank, int64_t n_nodes,
                          int64_t* new_parent, void* stream);

/*
 * Draft-head probabilities -> parent array of the tree of the most probable candidate
 * paths (a Medusa-style static tree), on the device.  No counterpart in the reference,
 * which builds its trees on the host (utils.py:27-77); with fsta_dfs_order,
 * fsta_lineage_from_parents and fsta_precompute a tree goes from model output to
 * kernel inputs on the stream, without a host round trip (README.md:16: the inputs
 * are rebuilt once per decoding step).
 *   probs [depths, topk] float32 or float64 (probs_dtype FSTA_F32 / FSTA_F64), row d
 *   = probabilities of the ranked candidates of draft depth d, descending.
 * A path of ranks (r1..rd) scores probs[0][r1] * ... * probs[d-1][rd] (float64,
 * left to right).  Node 0 is the empty path; the other n_nodes - 1 nodes are the
 * best-scoring paths (ties: shallower first, then smaller ranks), numbered by
 * (depth, ranks) ascending, so parent[i] < i.  parent [n_nodes] int64, -1 for the
 * root.  `status` (zero on entry) gets FSTA_TREE_NOT_PREFIX_CLOSED where a kept
 * path's prefix is not kept.  At most 16384 candidate paths (sum of topk^d) and
 * depths * topk <= 1024; n_nodes - 1 must not exceed the number of paths.
 */
int fsta_medusa_tree(const void* probs, int32_t probs_dtype, int32_t depths, int32_t topk,
                     int32_t n_nodes, int64_t* parent, uint32_t* status, void* stream);

/*
 * The same with a device workspace, for more candidate paths than one workgroup's
 * LDS holds: up to 2^24 paths (e.g. five draft depths of 10 ranks = 111110, six =
 * 1111110), scores and node ids in the workspace, one launch per step of the
 * selection (scores, up to eight radix passes, numbering, parents).  Same tree,
 * bit for bit, as fsta_medusa_tree gives where both apply; no counterpart in the
 * reference either.
 *   fsta_medusa_workspace_bytes: bytes of device memory (8-byte aligned) that
 *     fsta_medusa_tree_ws wants for (depths, topk); 0 when fsta_medusa_tree takes
 *     the problem (then the workspace may be NULL) or when it is out of range.
 *   The workspace is free again when the work queued on `stream` has run; calls
 *   that share one workspace must not overlap.
 */
size_t fsta_medusa_workspace_bytes(int32_t depths, int32_t topk);
int fsta_medusa_tree_ws(const void* probs, int32_t probs_dtype, int32_t depths, int32_t topk,
                        int32_t n_nodes, int64_t* parent, uint32_t* status,
                        void* workspace, size_t workspace_bytes, void* stream);

/*
 * Measuring aids (no counterpart in the reference; bench.py reports them beside
 * the attention kernels' figures as this GPU's own ceilings).
 *   fsta_probe_empty_launch: one launch of a kernel that does nothing, `workgroups`
 *     workgroups of `threads` threads: what a launch of that shape costs by itself.
 *   fsta_probe_hbm_read: a kernel that only reads: `bytes` (a multiple of 16) from
 *     src (16-byte aligned), 16 bytes per lane, consecutive lanes consecutive
 *     addresses, `workgroups` workgroups of 256 threads; `variant` 0..7: bit 0 = 16
 *     instead of 8 loads per lane in flight, bit 1 = non-temporal loads, bit 2 =
 *     every workgroup walks a contiguous piece instead of striding with the grid;
 *     `sink` (may be NULL) is never written in practice.
 */
int fsta_probe_empty_launch(int32_t workgroups, int32_t threads, void* stream);
int fsta_probe_hbm_read(const void* src, size_t bytes, int32_t workgroups, int32_t variant, uint32_t* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FSTA_H */
