/*
 * torchgt_hip.h — C ABI of the MI355X (gfx950) sparse-attention library.
 *
 * The reference (zxmeng98/torchgt) has no FFI layer: its hot path is the Python
 * method CoreAttention.sparse_attention / sparse_attention_bias, a chain of a
 * dozen ATen / torch_scatter kernels.  These entry points are what a binding for
 * that path attaches to; each comment names the reference code it replaces.
 *
 * Conventions
 *   - every pointer named d_* is DEVICE memory of the current HIP device; h_* is
 *     host memory; `stream` is a hipStream_t passed as void*.
 *   - all functions return 0 (TGT_OK) or a negative error code and write no
 *     output on error; tgt_last_error() gives a per-thread message.
 *   - inputs are borrowed and never modified; nothing here synchronises the
 *     stream except tgt_plan_create / tgt_plan_export.
 *   - node features are row-major [N, H, d] (the reference's [b, S, H, d] view
 *     flattened over b*S, attn_module.py:141-143).
 */
#ifndef TORCHGT_HIP_H
#define TORCHGT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TGT_OK                 0
#define TGT_ERR_INVALID_ARG   -1   /* null pointer, negative size, bad enum        */
#define TGT_ERR_INDEX_RANGE   -2   /* an edge endpoint is outside [0, N)            */
#define TGT_ERR_UNSUPPORTED   -3   /* (H, d, dtype) combination has no kernel       */
#define TGT_ERR_HIP           -4   /* a HIP runtime call failed                     */
#define TGT_ERR_WORKSPACE     -5   /* workspace too small / misaligned              */

/* element type of q, k, v, out, bias and the gradients */
#define TGT_DTYPE_F32   0
#define TGT_DTYPE_BF16  1
/* dense attention only: float32 tensors whose matrix products run on the bf16 matrix cores (operands
 * rounded to bf16, fp32 accumulation and softmax): about 2e-2 instead of 1e-5, for callers that ask for it */
#define TGT_DTYPE_F32_BF16_PRODUCTS 2

/* how the additive attention bias is supplied (added AFTER the +-5 clamp,
 * models/graphormer_dist_graph_level.py:262-267) */
#define TGT_BIAS_NONE      0
#define TGT_BIAS_EDGE_HEAD 1   /* [E, H], one value per edge and head, caller's edge order */
#define TGT_BIAS_EDGE      2   /* [E], one value per edge broadcast over heads
                                  (graphormer_dist_node_level.py:384)                     */
/* OR'ed to TGT_BIAS_EDGE_HEAD / TGT_BIAS_EDGE: bias and dbias rows are in the plan's
 * destination-sorted edge order (row i belongs to the caller's edge
 * tgt_plan_edge_order()[i]) instead of the caller's order.  The walks by destination then
 * read the bias and write dbias sequentially instead of through the edge permutation
 * (random 16 / 32-byte accesses that cost as much as the K/V row gathers on large graphs);
 * a bias shared by several layers is permuted once.  Needs tgt_plan_enable_bias_order(). */
#define TGT_BIAS_PLAN_ORDER 0x10
/* OR'ed to TGT_BIAS_PLAN_ORDER: d_bias holds the bias twice, 2 * E rows: first in
 * destination-sorted order, then in source-sorted order (tgt_plan_sort_rows with
 * direction 0 and 2).  The backward's walk by source then streams its copy as well: no
 * walk gathers the bias any more, and tgt_plan_enable_bias_order is not needed.  The
 * forward reads the first copy only; d_dbias is [E] / [E, H] in destination-sorted order. */
#define TGT_BIAS_BOTH_ORDERS 0x20

typedef struct tgt_plan tgt_plan_t;   /* opaque, owns device memory */

/* ---- device memory of the library's own ----------------------------------
 * Plans, tile sets and the scratch buffers of the edge preparation come from hipMalloc / hipFree
 * unless the host gives an allocator: `alloc(bytes, stream, user)` returns device memory that is
 * safe to use on `stream` (NULL on failure), `free_fn(ptr, user)` takes it back and may hand it
 * out again to later allocations for the same stream while kernels already launched there still
 * read it (what a stream-ordered caching allocator does).  The PyTorch extension registers torch's
 * caching allocator when it is loaded, so that building a plan per training iteration - the
 * reference moves edge_index to the GPU in every iteration, main_sp_sparse_node_level.py:178-183 -
 * costs no hipMalloc / hipFree (both synchronise the device).  Give both functions, or NULL for
 * both to return to hipMalloc; memory goes back to the allocator it came from.  No counterpart in
 * the reference (torch owns all of its memory). */
typedef void* (*tgt_alloc_fn)(size_t bytes, void* stream, void* user);
typedef void (*tgt_free_fn)(void* ptr, void* user);
int tgt_set_allocator(tgt_alloc_fn alloc, tgt_free_fn free_fn, void* user);

int          tgt_version(void);
const char*  tgt_error_string(int code);
const char*  tgt_last_error(void);

/* ---- graph plan ---------------------------------------------------------
 * Replaces the per-call gathers `k[edge_index[0]]`, `q[edge_index[1]]` and the
 * atomic scatter-adds `scatter(msg, edge_index[1], ...)` (attn_module.py:146-147,
 * 180, 185) by two sorted views of the edge list built ONCE per edge_index:
 *   CSR by destination: rowptr_dst[N+1], col_dst[E] (= source of the edge),
 *                       eid_dst[E] (= index of the edge in the caller's order)
 *   CSC by source:      rowptr_src[N+1], col_src[E] (= destination), eid_src[E]
 * Both orders are the STABLE sort of the caller's edge list (ties keep the
 * caller's order), i.e. what `argsort(kind='stable')` gives — the same contract
 * as the reference's edge sort (gt_sp/utils.py:354-356).  On top of that the
 * plan holds a degree-binned row schedule (long rows split into segments).
 *
 * d_src / d_dst: int64 device arrays of length E (edge_index[0], edge_index[1]).
 * Synchronises `stream` (once; a second time if the graph has rows of more than 256 edges,
 * a third for the launch descriptors).  TGT_ERR_INDEX_RANGE if any endpoint is outside [0,N).
 */
int tgt_plan_create(const int64_t* d_src, const int64_t* d_dst, int64_t E, int64_t N,
                    void* stream, tgt_plan_t** out_plan);
int tgt_plan_destroy(tgt_plan_t* plan);
/* The same for the edges that remain beside a tile set (tgt_block_attn_*; the reference's reordering
 * leaves them as the tail of its edge list, gt_sp/utils.py:284-299): the schedules hold only the rows
 * that have edges, the tile kernels write the others (most rows, when the tiles hold most edges: the
 * sparse kernels then start a fraction of the waves).  Accepted by tgt_block_attn_* and every tgt_plan_*
 * call; tgt_sparse_attn_* refuse such a plan with TGT_ERR_INVALID_ARG, since on their own they would
 * leave the rows without edges unwritten. */
int tgt_plan_create_remaining(const int64_t* d_src, const int64_t* d_dst, int64_t E, int64_t N,
                              void* stream, tgt_plan_t** out_plan);
/* A 128-bit content key of an edge list (values and their positions), for caches of plans that must
 * recognise an edge_index they have seen at another address: the reference's training loops move the
 * same CPU-resident edge_index to the GPU in every iteration (main_sp_sparse_node_level.py:178-183,
 * gt_sp/utils.py:455-458), and its layers and iterations are meant to share one plan.  Two small
 * kernels on `stream`, a 16-byte copy to h_key and one synchronisation of the stream; the key does
 * not depend on the launch shape. */
int tgt_edge_index_hash(const int64_t* d_src, const int64_t* d_dst, int64_t E, void* stream, uint64_t h_key[2]);
/* The attention kernels of a (H, d) shape read launch descriptors that are made on the first call
 * with that shape (a few small allocations, copies and one synchronisation of the stream, once per
 * plan and H * d / 8); tgt_plan_create makes those of H * d = 64 (the reference's hidden size 64
 * with 8 x 8 or 4 x 16 heads).  Call this for any other shape before capturing attention calls
 * into a HIP graph.  Later calls with the same shape return at once. */
int tgt_plan_prepare(tgt_plan_t* plan, int H, int d, void* stream);

/* info[0]=N, [1]=E, [2]=#schedule items (dst side), [3]=#split rows (dst),
 * [4]=#partial segments (dst), [5..7]= the same for the src side,
 * [8]=segment length limit, [9]=longest row one wave walks, [10],[11]=#workgroup
 * items (dst, src), [12..15] reserved (0). */
int tgt_plan_info(const tgt_plan_t* plan, int64_t info[16]);

#define TGT_PLAN_ROWPTR_DST 0
#define TGT_PLAN_COL_DST    1
#define TGT_PLAN_EID_DST    2
#define TGT_PLAN_ROWPTR_SRC 3
#define TGT_PLAN_COL_SRC    4
#define TGT_PLAN_EID_SRC    5
#define TGT_PLAN_ITEMS_DST  6   /* int32 x4 per item: row, first edge, length, partial slot (-1 = whole row) */
#define TGT_PLAN_ITEMS_SRC  7
#define TGT_PLAN_POS_SRC    8   /* after tgt_plan_enable_bias_order: destination-sorted position of every edge of the source-sorted order */
/* number of int32 values in array `which` */
int64_t tgt_plan_array_len(const tgt_plan_t* plan, int which);
/* copy array `which` to host memory (capacity in int32 elements); synchronous */
int tgt_plan_export(const tgt_plan_t* plan, int which, int32_t* h_out, int64_t capacity);

/* Support for TGT_BIAS_PLAN_ORDER.  tgt_plan_enable_bias_order builds (once; later calls return
 * at once) the map from the source-sorted to the destination-sorted edge order that the walk by
 * source needs; it allocates 4 bytes per edge and synchronises `stream`.  Call it before the
 * first attention call that uses the flag (not from a graph capture).  tgt_plan_edge_order writes
 * the permutation itself, int64 [E] on the device: d_out[i] = caller's index of the i-th edge in
 * destination-sorted order (stable), so  bias_sorted = bias[d_out]  and  dbias[d_out] = dbias_sorted. */
int tgt_plan_enable_bias_order(tgt_plan_t* plan, void* stream);
int tgt_plan_edge_order(const tgt_plan_t* plan, int64_t* d_out, void* stream);
/* the same for the source-sorted (stable) order */
int tgt_plan_edge_order_src(const tgt_plan_t* plan, int64_t* d_out, void* stream);
/* Rows of row_bytes bytes, one per edge, between the orders.  direction 0: d_out[i] =
 * d_in[edge_order[i]] (caller's order -> destination-sorted: a bias); 1: d_out[edge_order[i]] =
 * d_in[i] (destination-sorted -> caller's order: its gradient); 2: caller's order ->
 * source-sorted (the second copy of TGT_BIAS_BOTH_ORDERS).  d_in != d_out. */
int tgt_plan_sort_rows(const tgt_plan_t* plan, const void* d_in, int row_bytes, void* d_out, int direction, void* stream);

/* ---- sparse attention ---------------------------------------------------
 * Workspace (device memory, 256-byte aligned) needed by fwd/bwd for partial
 * sums of split rows, their arrival counters and per-node side vectors; depends
 * on the plan and H*d.  The caller ZEROES it once after allocating it; after that
 * only this library writes it (the counters return to zero at the end of every
 * call).  Calls that share a workspace must be ordered on one stream.  The attention
 * calls themselves only launch kernels (see tgt_plan_prepare for the one exception). */
int64_t tgt_sparse_attn_workspace_bytes(const tgt_plan_t* plan, int H, int d);

/* Forward of CoreAttention.sparse_attention (attn_module.py:133-189) /
 * sparse_attention_bias (models/graphormer_dist_node_level.py:69-127):
 *   s_e   = clamp(sum_c k[src,h,c] q[dst,h,c] / sqrt(d), -5, 5) + bias_e[h]
 *   w_e   = exp(s_e)                       (no max subtraction)
 *   Z_i   = sum_{e: dst=i} w_e ;  out_i = sum_e w_e v[src] / (Z_i + 1e-6)
 * d_out: [N, H, d] dtype;  d_Z: [N, H] float32 (saved for backward).
 */
int tgt_sparse_attn_fwd(const tgt_plan_t* plan,
                        const void* d_q, const void* d_k, const void* d_v,
                        const void* d_bias, int bias_mode,
                        int H, int d, int dtype,
                        void* d_out, float* d_Z,
                        void* d_workspace, int64_t workspace_bytes, void* stream);

/* The same forward for callers that cannot allocate device memory or pass a workspace (code under
 * HIP-graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in
 * the reference.  The partial sums and arrival counters of split rows live in a fixed array of
 * 4 MiB per GPU inside the library (held until the process ends); a graph whose split rows need
 * more is refused with TGT_ERR_WORKSPACE (a few thousand segments of long rows fit; use
 * tgt_sparse_attn_fwd with a workspace beyond that).  The call allocates nothing and frees nothing:
 * the launch descriptors of the (H, d) shape must exist already (tgt_plan_create makes those of
 * H * d = 64; tgt_plan_prepare any other), else TGT_ERR_INVALID_ARG.  Every call on a GPU
 * uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race.
 * Results are bit-identical to tgt_sparse_attn_fwd. */
int tgt_sparse_attn_fwd_noalloc(const tgt_plan_t* plan,
                                const void* d_q, const void* d_k, const void* d_v,
                                const void* d_bias, int bias_mode,
                                int H, int d, int dtype,
                                void* d_out, float* d_Z, void* stream);

/* Backward of the same function (autograd in the reference).  d_dout, d_dq,
 * d_dk, d_dv: [N, H, d] dtype; d_dbias: same shape/dtype as d_bias or NULL.
 * Every gradient is written exactly once (no atomics, no pre-zeroing needed). */
int tgt_sparse_attn_bwd(const tgt_plan_t* plan,
                        const void* d_q, const void* d_k, const void* d_v,
                        const void* d_bias, int bias_mode,
                        int H, int d, int dtype,
                        const void* d_out, const float* d_Z, const void* d_dout,
                        void* d_dq, void* d_dk, void* d_dv, void* d_dbias,
                        void* d_workspace, int64_t workspace_bytes, void* stream);

/* ---- dense biased attention (graph-level batches) -------------------------
 * CoreAttention.forward of models/graphormer_graph_level.py:186-214 (same body:
 * attn_module.py:99-127):  x = (q * sqrt(d)) k^T + bias ; softmax over keys ; x v.
 * d_q, d_k, d_v: [b, S, H, d]; d_bias: [b, H, S, S] (may hold -inf on padded
 * keys) or NULL; d_out: [b, S, H*d]; all of `dtype`.  d_lse: [b, H, S] float32
 * (log-sum-exp of every score row, saved for the backward).  TGT_DTYPE_BF16 and
 * TGT_DTYPE_F32_BF16_PRODUCTS: bf16 matrix instructions with fp32 accumulation and fp32 softmax
 * (S <= 256).  TGT_DTYPE_F32: float32 arithmetic throughout, like the reference (vector units; any S
 * whose four head images and one bias strip fit the LDS, S * (4 d + 35) <= 40 000).  d in {8, 16, 32}.  No dropout (see tgt_dense_attn_dropout_fwd);
 * the reference's unused `mask` argument is not applied. */
int tgt_dense_attn_fwd(const void* d_q, const void* d_k, const void* d_v, const void* d_bias,
                       int b, int S, int H, int d, int dtype,
                       void* d_out, float* d_lse, void* stream);
/* Backward (autograd in the reference).  d_dbias: [b, H, S, S] or NULL. */
int tgt_dense_attn_bwd(const void* d_q, const void* d_k, const void* d_v, const void* d_bias,
                       int b, int S, int H, int d, int dtype,
                       const void* d_out, const float* d_lse, const void* d_dout,
                       void* d_dq, void* d_dk, void* d_dv, void* d_dbias, void* stream);

/* The same with attention dropout (models/graphormer_graph_level.py:207-209, attn_module.py:121: Dropout(p) on the
 * softmax output, kept probabilities scaled by 1 / (1 - p); the reference's defaults are p = 0.1 / 0.5,
 * utils/parser_graph_level.py:20, utils/parser_node_level.py:20).  Whether the probability of (graph, head,
 * query, key) is kept is a counter-based hash of (seed, graph, head, query, key): the backward regenerates the
 * forward's choice from the same (p_drop, seed), nothing is stored.  p_drop in [0, 1); p_drop = 0 is
 * tgt_dense_attn_fwd / _bwd.  d_lse is the log-sum-exp of the undropped scores. */
int tgt_dense_attn_dropout_fwd(const void* d_q, const void* d_k, const void* d_v, const void* d_bias,
                               int b, int S, int H, int d, int dtype, float p_drop, uint64_t seed,
                               void* d_out, float* d_lse, void* stream);
int tgt_dense_attn_dropout_bwd(const void* d_q, const void* d_k, const void* d_v, const void* d_bias,
                               int b, int S, int H, int d, int dtype, float p_drop, uint64_t seed,
                               const void* d_out, const float* d_lse, const void* d_dout,
                               void* d_dq, void* d_dk, void* d_dv, void* d_dbias, void* stream);
/* d_keep: uint8 [b, H, S, S], 1 where the kernels keep the probability for (p_drop, seed) - what torch's
 * Dropout would hold as its mask; for tests and for callers that want to inspect it. */
int tgt_dense_attn_dropout_mask(int b, int S, int H, float p_drop, uint64_t seed, uint8_t* d_keep, void* stream);

/* ---- dense attention with the bias formed in the kernels from ids and tables -----------------
 * GraphAttnBias.forward (models/graphormer_graph_level.py:94-156, edge_type other than 'multi_hop') feeding
 * CoreAttention.forward (:186-214) without the [b, H, S, S] bias tensor in memory in either direction:
 *   bias[g,h,i,j] = 2 attn_bias[g,i,j] + spatial_table[sp[g,i,j]][h] + mean_f edge_table[et[g,i,j,f]][h]
 * over the padded index space S = s + 1 (virtual node first), i.e. the tensor tgt_graph_attn_bias_fwd would
 * write (the kernels round it to bf16, as a bf16 bias tensor is).
 *
 * tgt_dense_ids_pack: once per batch, the reference's int64 spatial_pos [b, s, s] and attn_edge_type
 * [b, s, s, F] to 16-bit ids over [b, S, S] and [b, S, S, F]: clamped to their tables like
 * tgt_graph_attn_bias_fwd does; on the virtual node's row and column the spatial id is num_spatial (the
 * kernels read the virtual distance there) and the edge id num_edges (reads as 0).  Table sizes 1..65534. */
int tgt_dense_ids_pack(const int64_t* d_spatial_pos, const int64_t* d_edge_type, int b, int s, int F, int num_spatial,
                       int num_edges, uint16_t* d_sp16, uint16_t* d_et16, void* stream);
/* Forward.  d_attn_bias: [b, S, S] of `dtype` (0 / -inf padding mask of the collator, any values allowed) or
 * NULL; tables [num_spatial, H], [num_edges, H], [H] of `dtype`; everything else as
 * tgt_dense_attn_dropout_fwd.  dtype TGT_DTYPE_BF16 or TGT_DTYPE_F32_BF16_PRODUCTS (the float32-arithmetic
 * kernels take a bias tensor: TGT_ERR_UNSUPPORTED); H <= 32; the [S, S] bias of one (graph, head) as bf16 plus
 * one column of both tables as float must fit the LDS next to the q/k/v images (S = 129 with the molecule
 * tables, 512 + 1537 rows: 52 KB forward, 79 KB backward), else TGT_ERR_UNSUPPORTED.  The forward applies the
 * backward's (larger) need: a shape it accepts is a shape tgt_dense_attn_ids_bwd accepts.  The same holds for
 * tgt_dense_attn_fwd / _bwd. */
int tgt_dense_attn_ids_fwd(const void* d_q, const void* d_k, const void* d_v, const void* d_attn_bias,
                           const uint16_t* d_sp16, const uint16_t* d_et16, int F, const void* d_spatial_table, int num_spatial,
                           const void* d_edge_table, int num_edges, const void* d_virtual_dist, int b, int S, int H, int d,
                           int dtype, float p_drop, uint64_t seed, void* d_out, float* d_lse, void* stream);
/* Backward: dq, dk, dv as tgt_dense_attn_dropout_bwd, and the gradients of the three tables (all three or
 * all NULL; autograd of the embedding lookups in the reference, row 0 of the spatial and edge tables is the
 * padding index and gets zero) summed over this call's batch: workgroups add dS into fixed-point LDS
 * accumulators (integer atomics, one power-of-two scale per (graph, head) from a bound B on a row's sum of |dS|:
 * no spatial accumulator exceeds S B, no edge accumulator F S B - a position adds its dS once per edge feature -
 * and one unit is at most 2^-21 B, for the edge table 2^-21 B times F rounded up to a power of two) and their
 * partials are added in a fixed order: results are reproducible bit for bit.  d_workspace: tgt_dense_attn_ids_bwd_workspace_bytes(...) bytes, 16-byte aligned,
 * needed only with table gradients. */
int64_t tgt_dense_attn_ids_bwd_workspace_bytes(int b, int H, int num_spatial, int num_edges);
int tgt_dense_attn_ids_bwd(const void* d_q, const void* d_k, const void* d_v, const void* d_attn_bias,
                           const uint16_t* d_sp16, const uint16_t* d_et16, int F, const void* d_spatial_table, int num_spatial,
                           const void* d_edge_table, int num_edges, const void* d_virtual_dist, int b, int S, int H, int d,
                           int dtype, float p_drop, uint64_t seed, const void* d_out, const float* d_lse, const void* d_dout,
                           void* d_dq, void* d_dk, void* d_dv, void* d_dspatial_table, void* d_dedge_table,
                           void* d_dvirtual_dist, void* d_workspace, int64_t workspace_bytes, void* stream);

/* ---- block path: dense 16 x 16 tiles + remaining edges, one softmax per node ----
 * A tile (r0, c0) stands for the 256 edges a -> b, a in [r0, r0+16), b in
 * [c0, c0+16) that the reference's cluster reordering emits as an expanded edge
 * list (gt_sp/utils.py:284-299, create_pairs :218-220) and then feeds to
 * sparse_attention (attn_module.py:133-189).  The result equals sparse attention
 * over the expanded tiles plus the edges of `plan` (tiles carry no bias, like the
 * reference, which forces attn_bias to None on this path, gt_sp/utils.py:465,470).
 * Tile products run on bf16 matrix instructions with fp32 accumulation (float32
 * inputs are rounded to bf16 for them); the remaining edges run on the sparse
 * kernels.  h_tiles: HOST int32 [T, 2]; destination blocks (and source blocks) of
 * different tiles must be identical or disjoint.  `plan` holds the remaining edges
 * (it may have E = 0) and fixes N.  Workspace: as for tgt_sparse_attn_*, zeroed once. */
typedef struct tgt_tiles tgt_tiles_t;
int tgt_tiles_create(const int32_t* h_tiles, int64_t T, int block_size, int64_t N, void* stream,
                     tgt_tiles_t** out);
int tgt_tiles_destroy(tgt_tiles_t* tiles);
int64_t tgt_block_attn_workspace_bytes(const tgt_tiles_t* tiles, const tgt_plan_t* plan, int H, int d);
int tgt_block_attn_fwd(const tgt_tiles_t* tiles, const tgt_plan_t* plan,
                       const void* d_q, const void* d_k, const void* d_v,
                       const void* d_bias, int bias_mode, int H, int d, int dtype,
                       void* d_out, float* d_Z, void* d_workspace, int64_t workspace_bytes, void* stream);
int tgt_block_attn_bwd(const tgt_tiles_t* tiles, const tgt_plan_t* plan,
                       const void* d_q, const void* d_k, const void* d_v,
                       const void* d_bias, int bias_mode, int H, int d, int dtype,
                       const void* d_out, const float* d_Z, const void* d_dout,
                       void* d_dq, void* d_dk, void* d_dv, void* d_dbias,
                       void* d_workspace, int64_t workspace_bytes, void* stream);

/* ---- edge construction and ordering ------------------------------------
 * fix_edge_index (gt_sp/utils.py:34-50): d_edge_index int64 [2, E0] over real
 * nodes 0..num_node-1 -> d_out int64 [2, E0 + 2*num_node]: real nodes shift by +1,
 * then num_node edges (i+1 -> 0), then num_node edges (0 -> i+1).  Global node 0
 * gets no self-loop. */
int tgt_fix_edge_index(const int64_t* d_edge_index, int64_t E0, int64_t num_node, int64_t* d_out, void* stream);

/* gen_sub_edge_index (gt_sp/utils.py:202-215): the edges among the nodes of a
 * batch, renamed to batch positions.  The reference calls torch_geometric
 * 2.0.0 (requirements.txt:208): remove_self_loops, add_self_loops(num_nodes=N),
 * subgraph(idx_batch, relabel_nodes=True).  Result, in this order: every edge
 * (s, d) of d_edge_index (int64 [2, E]) with s != d and both ends in
 * d_idx_batch (int64 [S], values in [0, N)), in the input's edge order; then one
 * self-loop per distinct batch node in ascending ORIGINAL node id.  Node
 * idx_batch[p] is renamed p; a node listed more than once takes its last
 * position.  d_out: int64, row 0 (sources) at d_out, row 1 (destinations) at
 * d_out + capacity; capacity >= E + min(S, N) always suffices.  *h_num_edges
 * (HOST) receives the number of edges written.  Synchronises `stream`.
 * TGT_ERR_INDEX_RANGE for ids outside [0, N), TGT_ERR_WORKSPACE if capacity is
 * too small (*h_num_edges then holds the needed size). */
int tgt_sub_edge_index(const int64_t* d_edge_index, int64_t E, int64_t N, const int64_t* d_idx_batch, int64_t S,
                       int64_t* d_out, int64_t capacity, int64_t* h_num_edges, void* stream);

/* reformat_graph (gt_sp/utils.py:319-359) with the METIS call replaced by the
 * explicit d_partition_ids int64 [N] in [0, k):
 *   relabel: parts in order 0..k-1, members in ascending old id (:329-335);
 *   blockize != 0: generate_new_edges_optimized (:223-305) - the edges of every
 *     partition pair are REPLACED by int(count/bs^2)+1 random dense bs x bs blocks
 *     drawn from numpy's legacy MT19937 stream exactly as the reference draws them
 *     (including its compact-count quirk and p hard-wired to 1);
 *   blockize == 0: keep the real edges (the alternative commented out at :347);
 *   stable sort of the new edge list by source (:354-356).
 * Synchronises `stream`.  Results are read with tgt_reformat_export:
 * d_edge_index int64 [2, E'] (E' = tgt_reformat_num_edges), d_sorted_indices
 * int64 [N] = argsort(new_id_mapping) (new id -> old id, :352). */
typedef struct tgt_reformat tgt_reformat_t;
int tgt_reformat_create(const int64_t* d_src, const int64_t* d_dst, int64_t E, int64_t N,
                        const int64_t* d_partition_ids, int k, int block_size, int blockize,
                        void* stream, tgt_reformat_t** out);
int64_t tgt_reformat_num_edges(const tgt_reformat_t* r);
int tgt_reformat_export(const tgt_reformat_t* r, int64_t* d_edge_index, int64_t* d_sorted_indices, void* stream);
int tgt_reformat_destroy(tgt_reformat_t* r);
/* The same result as a tile list: every emitted block as (first source, first
 * destination) in new ids (h_tiles, HOST int32 [T, 2], T = tgt_reformat_num_tiles)
 * plus the edges that were kept as they are (d_raw_edge_index, DEVICE int64
 * [2, E_raw], relabelled) - the input of tgt_block_attn_*. */
int64_t tgt_reformat_num_tiles(const tgt_reformat_t* r);
int64_t tgt_reformat_num_raw_edges(const tgt_reformat_t* r);
int tgt_reformat_export_tiles(const tgt_reformat_t* r, int32_t* h_tiles, int64_t* d_raw_edge_index, void* stream);

/* Host only: the n values np.random.randint(0, h_highs[i]) returns after
 * np.random.seed(seed) (legacy MT19937 stream used by gt_sp/utils.py:290-295). */
int tgt_np_legacy_randint(uint32_t seed, const int64_t* h_highs, int n, int64_t* h_out);

/* ---- projections around the attention -------------------------------------
 * MultiHeadAttention.forward (models/graphormer_dist_node_level.py:246-273; same
 * module in models/gt_dist_node_level.py and models/graphormer_dist_graph_level.py):
 * linear_q / linear_k / linear_v (:255-257, n_out = 3: one pass over x writes q, k
 * and v in the [N, H, d] layout the attention reads) and output_layer (:271,
 * n_out = 1).  y_j = x W_j^T + b_j for j < n_out.
 * d_x: [N, in_features]; d_W[j]: [out_features, in_features] row-major
 * (nn.Linear.weight); d_b[j]: [out_features] (d_b or an entry may be NULL: no
 * bias); d_y[j]: [N, out_features]; all of `dtype`, fp32 accumulation.  d_W, d_b,
 * d_y are HOST arrays of n_out device pointers.  in_features and out_features
 * must be multiples of 4 (fp32) or 8 (bf16): rows are read in 16-byte pieces. */
int tgt_linear_fwd(const void* d_x, const void* const* d_W, const void* const* d_b, void* const* d_y, int n_out,
                   int64_t N, int in_features, int out_features, int dtype, void* stream);

/* Backward of the same (autograd of nn.Linear in the reference):
 *   dx = sum_j dy_j W_j ;  dW_j = dy_j^T x ;  db_j = column sums of dy_j.
 * d_dx: [N, in_features] or NULL (not wanted).  d_dW: HOST array of n_out device
 * pointers [out_features, in_features], or NULL (then d_db must be NULL too);
 * d_db: HOST array of n_out device pointers [out_features] (or NULL, entries may
 * be NULL).  The weight gradients are summed in a fixed order (same inputs give
 * the same bits).  d_workspace: tgt_linear_bwd_workspace_bytes(...) bytes,
 * 16-byte aligned, needed when d_dW is given; contents need no initialisation. */
int64_t tgt_linear_bwd_workspace_bytes(int n_out, int in_features, int out_features);
/* A sum over per-workgroup partials that a *_deferred call leaves to its caller: element e of the result is the sum
 * over w of partial[w * n + e], added in a fixed order, and goes to out[i] + (e - begin[i]) for the last i with
 * begin[i] <= e (an out[i] of NULL: not wanted).  The caller only carries descriptors from a *_deferred call to
 * tgt_reduce_partials; the workspace the call was given must live until that launch has run. */
typedef struct {
    const float* partial;
    int32_t workers, n, n_out;
    void* out[6];
    int32_t begin[6];
} tgt_reduce_desc;
/* Up to eight such sums in one launch (a layer's backward has six: four linears, two LayerNorms, each a few
 * microseconds of launch latency on its own).  The result of a sum does not depend on what else is in the launch:
 * tgt_linear_bwd is tgt_linear_bwd_deferred followed by tgt_reduce_partials of its one descriptor.  dtype: of the
 * outputs.  No counterpart in the reference (autograd of nn.Linear / nn.LayerNorm reduces inside its own kernels). */
int tgt_reduce_partials(const tgt_reduce_desc* descs, int count, int dtype, void* stream);
/* tgt_linear_bwd without its last step: dx is complete on return (in stream order), the weight and bias gradients
 * are the sum `desc` describes.  d_dW must be given. */
int tgt_linear_bwd_deferred(const void* d_x, const void* const* d_W, const void* const* d_dy, int n_out, int64_t N,
                            int in_features, int out_features, int dtype, void* d_dx, void* const* d_dW, void* const* d_db,
                            void* d_workspace, int64_t workspace_bytes, void* stream, tgt_reduce_desc* desc);
/* FeedForwardNetwork's first layer with its activation (models/graphormer_dist_node_level.py:36-37:
 * x = self.layer1(x); x = self.gelu(x)) in one pass: u = x W^T + b goes to d_u and act(u) to d_h, both [N, out_features].
 * act: TGT_ACT_GELU (exact erf form, as tgt_gelu_fwd) or TGT_ACT_RELU.  The same bits as tgt_linear_fwd followed by
 * tgt_gelu_fwd / tgt_relu_fwd (which is what runs for shapes whose kernel has no such epilogue: only 64 -> 64 has). */
#define TGT_ACT_GELU 1
#define TGT_ACT_RELU 2
int tgt_linear_act_fwd(const void* d_x, const void* d_W, const void* d_b, int64_t N, int in_features, int out_features, int dtype,
                       int act, void* d_u, void* d_h, void* stream);
/* Backward of the layer that follows such an activation (FeedForwardNetwork.layer2, :38): its input was h = act(u)
 * [N, in_features].  d_du = (dy W) * act'(u), the gradient of u, instead of the gradient of h; d_dW = dy^T h and
 * d_db (may be NULL) as in tgt_linear_bwd.  The same bits as tgt_linear_bwd followed by tgt_gelu_bwd / tgt_relu_bwd.
 * desc: NULL, or a descriptor to fill instead of summing the weight-gradient partials (see tgt_reduce_partials). */
int tgt_linear_act_bwd(const void* d_h, const void* d_W, const void* d_dy, const void* d_u, int64_t N, int in_features,
                       int out_features, int dtype, int act, void* d_du, void* d_dW, void* d_db, void* d_workspace,
                       int64_t workspace_bytes, void* stream, tgt_reduce_desc* desc);
int tgt_linear_bwd(const void* d_x, const void* const* d_W, const void* const* d_dy, int n_out, int64_t N,
                   int in_features, int out_features, int dtype, void* d_dx, void* const* d_dW, void* const* d_db,
                   void* d_workspace, int64_t workspace_bytes, void* stream);

/* ---- the rest of the encoder layer ------------------------------------------
 * EncoderLayer.forward (models/graphormer_dist_node_level.py:296-314): each residual
 * block is  x = x + f(LayerNorm(x)).  One pass forms the residual sum and the
 * LayerNorm that follows it:
 *   s = x (+ r when d_r != NULL), written to d_sum when d_sum != NULL;
 *   y = (s - mean) / sqrt(var + eps) * gamma + beta   (nn.LayerNorm: biased variance
 *   over the C features of a row), written to d_y when d_y != NULL.
 * d_x, d_r, d_sum, d_y: [N, C]; d_gamma, d_beta: [C]; all of `dtype`, statistics in
 * fp32.  d_mean, d_rstd: float32 [N], saved for the backward (may be NULL).
 * C must be 16-byte vectors times a power of two of at most 64 lanes
 * (fp32: 8, 16, ..., 256; bf16: 16, 32, ..., 512). */
int tgt_add_layer_norm_fwd(const void* d_x, const void* d_r, const void* d_gamma, const void* d_beta, int64_t N, int C,
                           float eps, int dtype, void* d_sum, void* d_y, float* d_mean, float* d_rstd, void* stream);
/* Backward of y = LayerNorm(s) (autograd of nn.LayerNorm in the reference):
 *   ds = LayerNorm-backward(dy) (+ d_ds_extra when != NULL: the gradient that reaches s
 *   through the residual path), dgamma = sum_rows dy * xhat, dbeta = sum_rows dy.
 * The column sums are formed per workgroup and added in a fixed order.
 * d_workspace: tgt_layer_norm_bwd_workspace_bytes(C) bytes, 16-byte aligned. */
int64_t tgt_layer_norm_bwd_workspace_bytes(int C);
/* (tgt_layer_norm_bwd_deferred: the same with dgamma and dbeta left as the sum `desc` describes, see tgt_reduce_partials) */
int tgt_layer_norm_bwd(const void* d_s, const void* d_gamma, const float* d_mean, const float* d_rstd, const void* d_dy,
                       const void* d_ds_extra, int64_t N, int C, int dtype, void* d_ds, void* d_dgamma, void* d_dbeta,
                       void* d_workspace, int64_t workspace_bytes, void* stream);
int tgt_layer_norm_bwd_deferred(const void* d_s, const void* d_gamma, const float* d_mean, const float* d_rstd, const void* d_dy,
                       const void* d_ds_extra, int64_t N, int C, int dtype, void* d_ds, void* d_dgamma, void* d_dbeta,
                       void* d_workspace, int64_t workspace_bytes, void* stream, tgt_reduce_desc* desc);
/* nn.GELU() of FeedForwardNetwork (models/graphormer_dist_node_level.py:32,37), exact
 * erf form, on n elements (n a multiple of 4 for fp32, 8 for bf16):
 * h = 0.5 u (1 + erf(u / sqrt 2));  backward: du = dh * dh/du evaluated at u. */
int tgt_gelu_fwd(const void* d_u, int64_t n, int dtype, void* d_h, void* stream);
int tgt_gelu_bwd(const void* d_u, const void* d_dh, int64_t n, int dtype, void* d_du, void* stream);
/* F.relu of the GT layers (models/gt_dist_node_level.py:258,285; MLPReadout :272), same shapes
 * and limits as tgt_gelu_*: h = max(u, 0);  backward: du = dh where u > 0, else 0.  The kernel
 * time is booked under the gelu slot of the per-kernel timing. */
int tgt_relu_fwd(const void* d_u, int64_t n, int dtype, void* d_h, void* stream);
int tgt_relu_bwd(const void* d_u, const void* d_dh, int64_t n, int dtype, void* d_du, void* stream);
/* F.nll_loss(log_probs, target) of the node-level training and evaluation loops (main_sp_sparse_node_level.py:200,
 * gt_sp/evaluate.py:52,77): reduction 'mean', no class weights.  log_probs [N, C] (float32 or bf16), target [N]
 * int64:  loss = - sum_i log_probs[i, target_i] / count over the rows with target_i != ignore_index (torch's default
 * is -100), count = their number (0 rows: nan, like torch).  A target outside [0, C) other than ignore_index counts
 * as ignored (torch raises a device-side assertion there).  d_loss: one element of dtype; d_count: one float, kept
 * for the backward.  The sum is formed per workgroup and then in a fixed order: the same inputs give the same bits.
 * d_workspace: tgt_nll_loss_workspace_bytes(N) bytes, 4-byte aligned.
 * Backward: d_dlog_probs[i, c] = - dloss / count where c == target_i (and the row counts), else 0; d_dloss is one
 * element of dtype on the device. */
int64_t tgt_nll_loss_workspace_bytes(int64_t N);
int tgt_nll_loss_fwd(const void* d_log_probs, const int64_t* d_target, int64_t N, int C, int dtype, int64_t ignore_index, void* d_loss,
                     float* d_count, void* d_workspace, int64_t workspace_bytes, void* stream);
int tgt_nll_loss_bwd(const int64_t* d_target, const void* d_dloss, const float* d_count, int64_t N, int C, int dtype, int64_t ignore_index,
                     void* d_dlog_probs, void* stream);

/* ---- graph-level attention bias ---------------------------------------------
 * GraphAttnBias.forward (models/graphormer_graph_level.py:94-156), edge_type other than
 * 'multi_hop' (:148-150).  With S1 = s + 1 (virtual node first):
 *   out[g,h,i,j] = 2 * attn_bias[g,i,j]                                   (:104 and :153)
 *                + spatial_table[spatial_pos[g,i-1,j-1]][h]               (i, j >= 1; :110-111)
 *                + mean_f edge_table[edge_type[g,i-1,j-1,f]][h]           (i, j >= 1; :150-152)
 *                + virtual_dist[h]                                         (i == 0 or j == 0; :115-117)
 * d_attn_bias: [b, S1, S1]; d_spatial_pos: int64 [b, s, s]; d_edge_type: int64
 * [b, s, s, F]; tables [num_spatial, H], [num_edges, H], [H]; d_out: [b, H, S1, S1];
 * float tensors of `dtype`.  Ids outside a table are clamped to its range (the
 * reference's embedding lookup would raise). */
int tgt_graph_attn_bias_fwd(const void* d_attn_bias, const int64_t* d_spatial_pos, const int64_t* d_edge_type, int F,
                            const void* d_spatial_table, int num_spatial, const void* d_edge_table, int num_edges,
                            const void* d_virtual_dist, int b, int s, int H, int dtype, void* d_out, void* stream);
/* Gradients of the three tables for the upstream gradient d_dout [b, H, S1, S1]
 * (autograd of the embedding lookups in the reference; row 0 of the spatial and edge
 * tables is the padding index and gets zero).  Sums are formed in LDS per workgroup
 * with floating-point atomics and the workgroup partials are added in a fixed order:
 * results agree to rounding between runs, not bit for bit.
 * (num_spatial + num_edges + 1) * H must not exceed 32 768 (128 KB of LDS: the molecule tables
 * of the reference, 512 spatial ids and 1 537 edge types, fit with up to 15 heads). */
int64_t tgt_graph_attn_bias_bwd_workspace_bytes(int num_spatial, int num_edges, int H);
int tgt_graph_attn_bias_bwd(const void* d_dout, const int64_t* d_spatial_pos, const int64_t* d_edge_type, int F,
                            int num_spatial, int num_edges, int b, int s, int H, int dtype, void* d_dspatial_table,
                            void* d_dedge_table, void* d_dvirtual_dist, void* d_workspace, int64_t workspace_bytes,
                            void* stream);
/* GraphNodeFeature.forward (models/graphormer_graph_level.py:18-60): the input rows of the
 * graph-level model, virtual node first:
 *   out[g, 0, :]     = graph_token
 *   out[g, 1 + i, :] = sum_f atom_table[x[g,i,f]] + in_table[in_degree[g,i]] + out_table[out_degree[g,i]]
 * d_x: int64 [b, s, Fx]; d_in_degree, d_out_degree: int64 [b, s]; tables [num_*, C], d_graph_token
 * [C], d_out [b, s + 1, C] of `dtype`.  Ids outside a table are clamped to its range (the
 * reference's embedding lookup would raise). */
int tgt_graph_node_feature_fwd(const int64_t* d_x, const int64_t* d_in_degree, const int64_t* d_out_degree, int Fx,
                               const void* d_atom_table, int num_atoms, const void* d_in_table, int num_in,
                               const void* d_out_table, int num_out, const void* d_graph_token, int b, int s, int C, int dtype,
                               void* d_out, void* stream);
/* Gradients of the four tables for the upstream gradient d_dout [b, s + 1, C] (autograd of the
 * embedding lookups in the reference; row 0 of the three lookup tables is the padding index and
 * gets zero).  Sums are formed in float with memory atomics: results agree to rounding between
 * runs, not bit for bit.  d_workspace: tgt_graph_node_feature_bwd_workspace_bytes(...) bytes. */
int64_t tgt_graph_node_feature_bwd_workspace_bytes(int num_atoms, int num_in, int num_out, int C);
int tgt_graph_node_feature_bwd(const void* d_dout, const int64_t* d_x, const int64_t* d_in_degree, const int64_t* d_out_degree,
                               int Fx, int num_atoms, int num_in, int num_out, int b, int s, int C, int dtype, void* d_datom_table,
                               void* d_din_table, void* d_dout_table, void* d_dgraph_token, void* d_workspace,
                               int64_t workspace_bytes, void* stream);
/* The input rows of the graph-level GT, `embedding_h(x).sum(dim=-2)` (models/gt_graph_level.py:301,334):
 *   out[g, i, :] = sum_f table[x[g,i,f]]
 * d_x: int64 [b, s, Fx]; d_table [num_rows, C]; d_out [b, s, C] of `dtype`.  No padding index: the
 * backward gives every row its gradient (float sums with memory atomics, as above).  Ids outside
 * the table are clamped to its range. */
int tgt_embedding_sum_fwd(const int64_t* d_x, int Fx, const void* d_table, int num_rows, int b, int s, int C, int dtype, void* d_out,
                          void* stream);
int64_t tgt_embedding_sum_bwd_workspace_bytes(int num_rows, int C);
int tgt_embedding_sum_bwd(const void* d_dout, const int64_t* d_x, int Fx, int num_rows, int b, int s, int C, int dtype, void* d_dtable,
                          void* d_workspace, int64_t workspace_bytes, void* stream);
/* GraphAttnBias.forward with edge_type == 'multi_hop' (models/graphormer_graph_level.py:94-156,
 * the path-encoding branch :119-147).  As tgt_graph_attn_bias_fwd, with the edge term replaced by
 *   (1 / hops) * sum_dd  mean_f edge_table[edge_input[g,i-1,j-1,dd,f]]  x  W[dd]        (i, j >= 1)
 * where W = edge_dis_weight viewed as [num_edge_dis, H, H] (:137), dd runs over the first
 * D = min(D0, multi_hop_max_dist) hops (all D0 when multi_hop_max_dist is 0; :125-127) and
 * hops = 1 for spatial ids 0 and 1, id - 1 above, at most multi_hop_max_dist when that is set
 * (:121-126).  d_edge_input: int64 [b, s, s, D0, F]; d_edge_dis_weight: [num_edge_dis * H * H]
 * of `dtype`.  D must not exceed num_edge_dis (the reference's bmm would raise); H <= 32. */
int tgt_graph_attn_bias_multi_hop_fwd(const void* d_attn_bias, const int64_t* d_spatial_pos, const int64_t* d_edge_input, int D0,
                                      int F, const void* d_spatial_table, int num_spatial, const void* d_edge_table,
                                      int num_edges, const void* d_edge_dis_weight, int num_edge_dis, const void* d_virtual_dist,
                                      int multi_hop_max_dist, int b, int s, int H, int dtype, void* d_out, void* stream);
/* Gradients of the four parameter tensors of that branch for the upstream gradient d_dout
 * [b, H, S1, S1] (autograd in the reference): spatial table, edge table (row 0 of both is the
 * padding index and gets zero), the hop matrices ([num_edge_dis * H * H]; matrices beyond the D
 * hops in use get zero) and the virtual distance.  Workgroup sums are formed in LDS (floating-point
 * atomics) and added in a fixed order: results agree to rounding between runs, not bit for bit.
 * D = min(D0, multi_hop_max_dist) (D0 when the limit is 0) sizes the workspace. */
int64_t tgt_graph_attn_bias_multi_hop_bwd_workspace_bytes(int num_spatial, int num_edges, int H, int D);
int tgt_graph_attn_bias_multi_hop_bwd(const void* d_dout, const int64_t* d_spatial_pos, const int64_t* d_edge_input, int D0, int F,
                                      const void* d_edge_table, int num_spatial, int num_edges, const void* d_edge_dis_weight,
                                      int num_edge_dis, int multi_hop_max_dist, int b, int s, int H, int dtype,
                                      void* d_dspatial_table, void* d_dedge_table, void* d_dedge_dis_weight,
                                      void* d_dvirtual_dist, void* d_workspace, int64_t workspace_bytes, void* stream);
/* gen_edge_input (data/algos.pyx:64-92) for a batch of graphs of at most 256 nodes.
 * d_path: int32 [num_graphs, n_max, n_max] as tgt_floyd_warshall writes it; d_edge_feat:
 * [num_graphs, n_max, n_max, F], int64 (feat_is_int64 != 0) or int32; d_n_nodes as there.
 * d_out: int64 [num_graphs, n_max, n_max, max_dist, F]; entry (i, j, k) = features of the k-th
 * edge on the recorded shortest path from i to j (the reference's recursive expansion of the
 * intermediate nodes, :56-61), -1 where there is none: i == j, unreachable pairs, hops past the
 * end of the path, padding nodes.  Hops at or beyond max_dist are dropped. */
int tgt_gen_edge_input(const int32_t* d_path, const void* d_edge_feat, int feat_is_int64, int F, const int32_t* d_n_nodes,
                       int num_graphs, int n_max, int max_dist, int64_t* d_out, void* stream);
/* floyd_warshall (data/algos.pyx:9-54) for a batch of graphs of at most 256 nodes.
 * d_adj: uint8 [num_graphs, n_max, n_max], entry = edge weight, 0 = no edge;
 * d_n_nodes: int32 [num_graphs] node counts (NULL: all n_max).  d_dist, d_path:
 * int32 [num_graphs, n_max, n_max]; entries with i or j >= n_nodes[g] are left
 * untouched.  dist = shortest distance (0 on the diagonal, 510 if unreachable),
 * path = the intermediate node recorded by the last strict improvement (-1 for
 * direct edges, 510 if unreachable): both exactly what the reference's loop yields. */
int tgt_floyd_warshall(const uint8_t* d_adj, const int32_t* d_n_nodes, int num_graphs, int n_max, int32_t* d_dist,
                       int32_t* d_path, void* stream);

/* ---- per-kernel timing --------------------------------------------------
 * The reference times this path with torch.profiler around whole iterations
 * (attn_module.py:415-438).  When enabled, every kernel the library launches is
 * bracketed by two hipEvents on the launch stream; tgt_timing_read waits for the
 * recorded pairs and returns the summed duration and launch count of one kernel
 * slot (0 <= slot < tgt_timing_slots()).  Off by default. */
int tgt_timing_enable(int on);
int tgt_timing_reset(void);
int tgt_timing_slots(void);
int tgt_timing_read(int slot, const char** name, double* total_ms, int64_t* launches);

#ifdef __cplusplus
}
#endif
#endif /* TORCHGT_HIP_H */
