/*
 * graphiler_amd.h -- C ABI of the MI355X (gfx950) sparse graph-primitive layer.
 *
 * These entry points are what the operator wrappers behind the reference's
 * TorchScript boundary (torch.ops.my_ops.* / torch.classes.my_classes.DGLGraph)
 * bind to.  Each declaration cites the reference function it replaces
 * (paths relative to the reference repository).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the comment says "host";
 *   - sizes are int64_t, graph index arrays keep the reference's layout
 *     (include/dglgraph.h:54-74): int32 row pointer / neighbour id / edge id,
 *     int64 COO endpoints and type columns;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); all
 *     work is enqueued on it and nothing synchronises;
 *   - entry points never allocate, never throw and return GA_OK (0), a negative
 *     GA_E* code for rejected arguments, or a positive hipError_t from a launch;
 *   - feature matrices are row-major and contiguous; GA_BF16 data is read and
 *     written as bf16, accumulated in fp32; per-edge scalars (attention logits
 *     and weights) are always fp32;
 *   - results are deterministic: no atomics are used, and the order of every
 *     floating-point reduction is a function of the graph and sizes only.
 */
#ifndef GRAPHILER_AMD_H_
#define GRAPHILER_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GA_OK 0
#define GA_EINVAL (-1)       /* null / negative / inconsistent argument      */
#define GA_EUNSUPPORTED (-2) /* valid request this build has no kernel for   */
#define GA_EWORKSPACE (-3)   /* workspace missing, too small or misaligned   */
#define GA_EALIGN (-4)       /* pointer not aligned to its element size      */
#define GA_ESCRATCH (-5)     /* problem needs more than the library's static scratch */

typedef void *ga_stream_t;

enum ga_dtype { GA_F32 = 0, GA_BF16 = 1 };
/* message = u[nbr] | e[eid] | u[nbr] * w[eid]   (functor.cuh:18-121)         */
enum ga_sddmm_op { GA_SDDMM_ADD = 0, GA_SDDMM_SUB = 1, GA_SDDMM_MUL = 2, GA_SDDMM_DIV = 3 };
enum ga_spmm_op {
  GA_COPY_U = 0, GA_COPY_E = 1,
  GA_U_MUL_E = 2, GA_U_ADD_E = 3, GA_U_SUB_E = 4, GA_U_DIV_E = 5 /* u[src] (op) w[edge] */
};
/* binary operators of the general (broadcasting) forms, functor.cuh:19-116 */
enum ga_bcast_op {
  GA_BCAST_ADD = 0, GA_BCAST_SUB = 1, GA_BCAST_MUL = 2, GA_BCAST_DIV = 3,
  GA_BCAST_COPY_LHS = 4, GA_BCAST_COPY_RHS = 5, GA_BCAST_DOT = 6 /* SDDMM only */
};
/* functor.cuh:125-213: sum starts at 0, max at -inf, min at +inf             */
enum ga_reduce { GA_SUM = 0, GA_MAX = 1, GA_MIN = 2 };
/* activation applied to an output row before it is stored (the *_act entry points) */
enum ga_activation { GA_ACT_NONE = 0, GA_ACT_RELU = 1, GA_ACT_ELU = 2 };

/* Library version (major*10000 + minor*100 + patch). */
int ga_version(void);
/* Static, human-readable text for a return code of this library. */
const char *ga_error_string(int code);

/* ------------------------------------------------------------------ graph --
 * Slot -> row map of a grouped adjacency: row_of_slot[i] = v for every
 * i in [pointer[v], pointer[v+1]).  It is the schedule every row-reduction
 * kernel below balances its work with (equal-sized runs of slots instead of
 * whole rows), built once per graph next to the arrays that
 * python/graphiler/utils/setup.py:116-146 (prepare_graph) fills in.
 */
int ga_csr_row_ids(const int32_t *pointer, int64_t n_rows, int64_t n_edges,
                   int32_t *row_of_slot, ga_stream_t stream);

/* Stable grouping of items by key on the device: the construction of the
 * in_* / out_* columns (python/graphiler/utils/setup.py:116-146: key = COO_dst,
 * other = COO_src for the in-adjacency; key = COO_src, other = COO_dst for the
 * out-adjacency) and of the type pointers (setup.py:147-161 with
 * include/dglgraph.h:68-71: key = type of each item, nbr = NULL; eid is then
 * the stable permutation that makes types contiguous).
 *   key, other  (n_items) int64      pointer (n_keys+1) int32
 *   nbr         (n_items) int32 or NULL: other[eid[i]]
 *   eid         (n_items) int32: item ids, ascending inside one key
 *   status      one int32 on the device: 0, or 1 when a key lies outside
 *               [0, n_keys) (the outputs are then meaningless but in bounds)
 *   workspace   ga_group_edges_workspace_bytes() bytes, 256-byte aligned
 */
size_t ga_group_edges_workspace_bytes(int64_t n_keys, int64_t n_items);
int ga_group_edges(const int64_t *key, const int64_t *other, int64_t n_keys,
                   int64_t n_items, int32_t *pointer, int32_t *nbr, int32_t *eid,
                   int32_t *status, void *workspace, size_t workspace_bytes,
                   ga_stream_t stream);

/* ------------------------------------------------------------------- SpMM --
 * out[v, h, d] = reduce_{i in [pointer[v], pointer[v+1])} msg_i[h, d]
 * Replaces SpMMSrc (spmm.cu:375-389; op GA_COPY_U, gather by nbr),
 * SpMMEdge (spmm.cu:359-373; op GA_COPY_E, gather rows of the (E, feat) matrix
 * `u` by eid), src_mul_e_sum / dst_mul_e_sum (spmm.cu:286-356; op GA_U_MUL_E,
 * pass the in- or the out-adjacency) and the generic SpMMCsrKernel with its
 * add / sub / mul / div binary operators (functor.cuh:19-72; GA_U_ADD_E ..
 * GA_U_DIV_E, w per head like U_MUL_E) and Max / Min reducers (spmm.cuh:30-71).
 *   pointer      (n_rows+1) int32     nbr (n_edges) int32, unused for COPY_E
 *   row_of_slot  (n_edges)  int32     from ga_csr_row_ids
 *   eid          (n_edges)  int32 or NULL when eid[i] == i
 *   u            (n_src, feat)  or (n_edges, feat) for COPY_E, `dtype`
 *   w            (n_edges, heads) fp32, the U_*_E operators only; feat % heads == 0
 *   out          (n_rows, feat) `dtype`; every row is written (rows without
 *                edges get 0, -inf or +inf by reducer)
 *   workspace    ga_spmm_workspace_bytes() bytes, 16-byte aligned
 */
size_t ga_spmm_workspace_bytes(int64_t n_edges, int64_t feat);
int ga_spmm_csr(const int32_t *pointer, const int32_t *row_of_slot,
                const int32_t *nbr, const int32_t *eid, const void *u,
                const float *w, void *out, int64_t n_rows, int64_t n_edges,
                int64_t feat, int64_t heads, int op, int reduce, int dtype,
                void *workspace, size_t workspace_bytes, ga_stream_t stream);

/* Sum SpMM of copied rows (GA_COPY_U or GA_COPY_E) with the row-wise tail of a GCN
 * layer in its store: out[v, :] = act(row_scale[v] * sum_i msg_i), i.e. SpMMSrc
 * (spmm.cu:375-389) followed by the destination-side normalisation and the relu of
 * examples/GCN/GCN.py:26 (`torch.relu(torch.sum(mailbox, 1))`) without a pass over
 * the (n_rows, feat) result for either.  row_scale (n_rows) fp32 or NULL (no
 * factor); activation one of ga_activation, applied to the fp32 value before it is
 * rounded.  Rows without edges get act(row_scale[v] * 0).  Everything else as
 * ga_spmm_csr; with row_scale == NULL and GA_ACT_NONE the result is that of
 * ga_spmm_csr, bit for bit.  workspace: ga_spmm_scaled_workspace_bytes() bytes,
 * 16-byte aligned (the factor travels with the partial sums of a row).
 */
size_t ga_spmm_scaled_workspace_bytes(int64_t n_edges, int64_t feat);
int ga_spmm_csr_scaled(const int32_t *pointer, const int32_t *row_of_slot,
                       const int32_t *nbr, const int32_t *eid, const void *u, void *out,
                       const float *row_scale, int activation, int64_t n_rows,
                       int64_t n_edges, int64_t feat, int op, int dtype, void *workspace,
                       size_t workspace_bytes, ga_stream_t stream);

/* SpMM with max / min and the position of each extremum: the arg_u / arg_e
 * outputs of the reference's generic kernel (SpMMCsrKernel, spmm.cuh:30-71,
 * reducers functor.cuh:148-213: strict comparison, so the first extremum in
 * adjacency order wins; the locals start at 0, so a row whose extremum is never
 * replaced - no edges, only NaN - reports 0).
 *   arg_u  (n_rows, feat) int32 or NULL: neighbour id that supplied out[v, f];
 *          COPY_U and U_MUL_E only (operators that read u)
 *   arg_e  (n_rows, feat) int32 or NULL: edge id that supplied out[v, f];
 *          COPY_E and U_MUL_E only (operators that read edge data)
 *   reduce GA_MAX or GA_MIN; everything else as ga_spmm_csr
 *   workspace  ga_spmm_arg_workspace_bytes() bytes, 16-byte aligned
 */
size_t ga_spmm_arg_workspace_bytes(int64_t n_edges, int64_t feat);
int ga_spmm_csr_arg(const int32_t *pointer, const int32_t *row_of_slot,
                    const int32_t *nbr, const int32_t *eid, const void *u,
                    const float *w, void *out, int32_t *arg_u, int32_t *arg_e,
                    int64_t n_rows, int64_t n_edges, int64_t feat, int64_t heads,
                    int op, int reduce, int dtype, void *workspace,
                    size_t workspace_bytes, ga_stream_t stream);

/* SpMM whose operands broadcast against each other: the UseBcast = true form of
 * the reference's generic kernel (SpMMCsrKernel, spmm.cuh:30-71) fed by the offset
 * tables of CalcBcastOff (bcast.cc:19-71):
 *   out[v, k] = reduce_{i in row v} op(u[nbr[i], u_off[k]], w[eid[i], w_off[k]])
 * u (n_src, u_len), w (n_edges, w_len), out (n_rows, out_len), all fp32;
 * u_off / w_off (out_len) int64 on the device, NULL = the identity (k).
 * op: ga_bcast_op without DOT; reduce: ga_reduce; arg_u / arg_e as in
 * ga_spmm_csr_arg (NULL when not wanted; max / min only).  Edges of a row are
 * folded in adjacency order by one thread per output element: the general path,
 * not a tuned one.  eid NULL when eid[i] == i. */
int ga_spmm_csr_bcast(const int32_t *pointer, const int32_t *nbr, const int32_t *eid,
                      const float *u, const float *w, float *out, int32_t *arg_u,
                      int32_t *arg_e, int64_t n_rows, int64_t n_edges, const int64_t *u_off,
                      const int64_t *w_off, int64_t u_len, int64_t w_len, int64_t out_len,
                      int op, int reduce, ga_stream_t stream);

/* ------------------------------------------------------------------ SDDMM --
 * out[i, k] = u[lhs[i], k] + v[rhs[i], k], fp32 output (E, feat).
 * Replaces SDDMMCoo_u_add_v_mul_alpha (sddmm.cu:118-129, kernel
 * sddmm.cuh:34-71); `alpha` of the reference is accepted by the operator
 * wrapper and ignored there, as in the reference.  (lhs, rhs) are either the
 * int64 COO columns (idx_bits 64: output in edge-id order) or the int32
 * (nbr, row_of_slot) columns of an adjacency (idx_bits 32: output in slot
 * order, equal to edge-id order when eid[i] == i).
 */
int ga_sddmm_u_add_v(const void *lhs, const void *rhs, int idx_bits,
                     const void *u, const void *v, float *out, int64_t n_edges,
                     int64_t feat, int dtype, ga_stream_t stream);

/* The same kernel with the other binary functors of the reference's generic
 * SDDMM (SDDMMCooKernel<..., BinaryOp, ...>, sddmm.cuh:34-71 with
 * functor.cuh:19-72): out[i, k] = u[lhs[i], k] (op) v[rhs[i], k], one fp32
 * operation per element.  op: GA_SDDMM_ADD / SUB / MUL / DIV. */
int ga_sddmm_u_op_v(const void *lhs, const void *rhs, int idx_bits,
                    const void *u, const void *v, float *out, int64_t n_edges,
                    int64_t feat, int op, int dtype, ga_stream_t stream);

/* The same operators over a grouped adjacency, for graphs whose edge ids are slot
 * numbers (eid[i] == i, e.g. edges stored by destination): out[i, k] =
 * u[nbr[i], k] (op) v[row(i), k] for every slot i, i.e. the reference's
 * SDDMMCoo_u_add_v_mul_alpha (sddmm.cu:118-129) with lhs target = the neighbour
 * column, rhs target = the row (selector.h:30-60).  The row of a slot comes from the
 * row pointer, so no second index column is read and v is read once per row:
 * 4 + 8 feat bytes per edge instead of 8 + 12 feat.  fp32, feat 1, 2 or 4
 * (GA_EUNSUPPORTED otherwise: use ga_sddmm_u_op_v); nbr and out 16-byte aligned,
 * u and v aligned to a row (GA_EALIGN otherwise).  row_of_slot is read at two
 * slots per 256 - 1024 only.  Bit-exact with ga_sddmm_u_op_v. */
int ga_sddmm_u_op_v_adj(const int32_t *pointer, const int32_t *row_of_slot,
                        const int32_t *nbr, const float *u, const float *v, float *out,
                        int64_t n_rows, int64_t n_edges, int64_t feat, int op,
                        ga_stream_t stream);

/* Typed neighbour sum: out[v, :] = sum over in-edges e of v of
 * row_scale[e] * (x[src(e), :] @ W[type(e)]), the operator chain BroadcastSrcNode ->
 * SegmentMMEdge -> mul -> SpMMEdge of an RGCN layer (broadcast.cu:58-63,
 * segment_mm.cu:29-33, spmm.cu:359-373; examples/RGCN/RGCN.py:25-33) in one pass, with
 * no (E, M) message tensor.
 *
 * ga_typed_tiles_build prepares the graph once: the slots of the in-adjacency
 * (row_of_slot = destination, nbr = source, eid = edge id or null when slot = edge id;
 * type_pointer: n_types + 1 entries over the edge ids, include/dglgraph.h:24-27) are
 * ordered by (destination / tile_rows, relation) and every such group is padded to
 * chunks of 16 slots.  tile_rows is 128 or 144: ga_typed_tile_rows(n_rows) names the one
 * whose tiles fill whole rounds of this device's CUs best; the same value goes to every
 * call for the graph.  Outputs: tile_chunk_pointer (tiles + 1, tiles =
 * ceil(n_rows / tile_rows)), chunk_type (capacity: relation | mask of the chunk's 16-row
 * blocks << 16; at most 65535 relations), slot_src and slot_edge
 * (16 * capacity, -1 in pad slots), slot_dst (16 * capacity bytes: destination - tile
 * start, 255 in pad slots; 4-byte aligned), capacity =
 * ga_typed_tiles_chunk_capacity(...).  Everything runs on `stream`; nothing is read
 * back.
 *
 * ga_typed_spmm: x (n_src, K), W (n_types, K, M), out (n_rows, M) of `dtype`;
 * row_scale (n_edges,) fp32 in edge-id order or null.  M must be 8, 16, 32 or 64, K one
 * of 16, 32, 48, 64, and x and row_scale smaller than 4 GiB (GA_EUNSUPPORTED otherwise:
 * use ga_segment_mm_gather + ga_spmm_csr, which are also the faster pair from about
 * K * M = 4096 on).  The sum over the in-edges runs on the matrix
 * cores with fp32 accumulation: bf16 messages enter as the two-operator chain rounds
 * them, fp32 messages as three bf16 terms that carry 24 bits.  The order of the
 * additions is fixed by the prepared layout, so repeated calls give identical bits;
 * against the chain only that order differs.  Messages that are not finite reach
 * exactly the rows the chain would give them to. */
int64_t ga_typed_tile_rows(int64_t n_rows);
int64_t ga_typed_tiles_chunk_capacity(int64_t n_rows, int64_t n_edges, int64_t n_types,
                                      int64_t tile_rows);
size_t ga_typed_tiles_workspace_bytes(int64_t n_rows, int64_t n_edges, int64_t n_types,
                                      int64_t tile_rows);
int ga_typed_tiles_build(const int32_t *row_of_slot, const int32_t *nbr, const int32_t *eid,
                         const int32_t *type_pointer, int64_t n_rows, int64_t n_edges,
                         int64_t n_types, int64_t tile_rows, int32_t *tile_chunk_pointer,
                         int32_t *chunk_type, int32_t *slot_src, unsigned char *slot_dst,
                         int32_t *slot_edge, void *workspace, size_t workspace_bytes,
                         ga_stream_t stream);
int ga_typed_spmm(const int32_t *tile_chunk_pointer, const int32_t *chunk_type,
                  const int32_t *slot_src, const unsigned char *slot_dst,
                  const int32_t *slot_edge, const void *x, const void *W,
                  const float *row_scale, void *out, int64_t n_rows, int64_t n_src,
                  int64_t n_edges, int64_t n_types, int64_t tile_rows, int64_t K, int64_t M,
                  int dtype, ga_stream_t stream);

/* ga_typed_spmm with the activation that follows the layer (relu between the layers of
 * examples/RGCN/RGCN.py:69; GA_ACT_RELU, GA_ACT_ELU with alpha = 1) applied to the fp32
 * sums before they are rounded and stored.  GA_ACT_NONE is ga_typed_spmm. */
int ga_typed_spmm_act(const int32_t *tile_chunk_pointer, const int32_t *chunk_type,
                      const int32_t *slot_src, const unsigned char *slot_dst,
                      const int32_t *slot_edge, const void *x, const void *W,
                      const float *row_scale, void *out, int64_t n_rows, int64_t n_src,
                      int64_t n_edges, int64_t n_types, int64_t tile_rows, int64_t K, int64_t M,
                      int activation, int dtype, ga_stream_t stream);

/* The general SDDMM of the reference (SDDMMCooKernel / SDDMMCooTreeReduceKernel,
 * sddmm.cuh:34-120): operands on the source nodes (target 0), on the edges (1) or on
 * the destination nodes (2) in any combination (selector.h:30-60), feature shapes
 * that broadcast (offset tables of CalcBcastOff, bcast.cc:19-71), and the dot
 * product over the last dimension:
 *   out[e, k] = op(lhs[id_l(e), lhs_off[k] * reduce_size ...],
 *                  rhs[id_r(e), rhs_off[k] * reduce_size ...])
 * with id = src[e] | e | dst[e] by target; GA_BCAST_DOT sums reduce_size products,
 * every other operator needs reduce_size == 1.  src / dst int64 (the COO columns),
 * lhs (*, lhs_len), rhs (*, rhs_len), out (n_edges, out_len) fp32 in edge-id order;
 * lhs_off / rhs_off (out_len) int64 on the device, NULL = the identity. */
int ga_sddmm_bcast(const int64_t *src, const int64_t *dst, const float *lhs, const float *rhs,
                   float *out, int64_t n_edges, int lhs_target, int rhs_target,
                   const int64_t *lhs_off, const int64_t *rhs_off, int64_t lhs_len,
                   int64_t rhs_len, int64_t out_len, int64_t reduce_size, int op,
                   ga_stream_t stream);

/* out[i, h] = sum_d u[lhs[i], h, d] * v[rhs[i], h, d], fp32 output (E, heads).
 * The Dot functor (functor.cuh:103-116) with the reduction over the last
 * dimension (bcast.cc:37-39,57-60; kernel sddmm.cuh:80-120), which the
 * reference compiles but never registers. */
int ga_sddmm_u_dot_v(const void *lhs, const void *rhs, int idx_bits,
                     const void *u, const void *v, float *out, int64_t n_edges,
                     int64_t heads, int64_t dim, int dtype, ga_stream_t stream);

/* ---------------------------------------------------------- edge softmax --
 * y[e, h] = softmax of x[., h] over the edges e = eid[i] (or i when eid is
 * NULL), i in [pointer[v], pointer[v+1]), for every row v.  fp32 in and out.
 * Replaces SegmentSoftmaxForward / softmax_v (segment_softmax.cu:3-24,
 * segment_softmax_kernel.cu:4-49) and supplies the multi-head case the
 * reference leaves empty (softmax_m, segment_softmax_kernel.cu:52-53).
 * Uses the true segment maximum (the reference clamps it at >= 0, which only
 * changes results once every logit of a segment is below about -87).
 * y entries of edges that belong to no row are left untouched: pass y zeroed
 * to match the reference's zeros_like output when eid is not a permutation.
 * y may be x itself (in place); any other overlap of the two is GA_EINVAL.
 * workspace: ga_softmax_workspace_bytes() bytes (partial maxima / sums and
 * descriptors of the rows that leave a tile of 8192 values), 16-byte aligned.
 */
size_t ga_softmax_workspace_bytes(int64_t n_edges, int64_t heads);
int ga_segment_softmax(const int32_t *pointer, const int32_t *row_of_slot,
                       const int32_t *eid, const float *x, float *y,
                       int64_t n_rows, int64_t n_edges, int64_t heads,
                       void *workspace, size_t workspace_bytes,
                       ga_stream_t stream);

/* ------------------------------------------------------------ segment_mm --
 * Y[r, h, :] = X[r, h, :] @ W[t, h, :, :] for r in [type_pointer[t],
 * type_pointer[t+1]).  Replaces SegmentMMBase / SegmentMMNode / SegmentMMEdge
 * (segment_mm.cu:4-33) for heads == 1; heads > 1 applies one K x M block per
 * head.  type_pointer stays on the device (the reference copies it to the host
 * every call, segment_mm.cu:10).  X (rows, heads*K), W (n_types, heads, K, M),
 * Y (rows, heads*M), all `dtype`; fp32 accumulation on the matrix cores.
 */
int ga_segment_mm(const int32_t *type_pointer, int64_t n_types, const void *X,
                  const void *W, void *Y, int64_t rows, int64_t heads,
                  int64_t K, int64_t M, int dtype, ga_stream_t stream);

/* Several typed products of the same rows in one pass: Y[i] = segment_mm(X, W[i]) for
 * i < n_weights (1 .. 4), every W[i] (n_types, K, M) and Y[i] (rows, M); W and Y are
 * host arrays of device pointers.  The K | Q | V projections of an HGT layer
 * (examples/HGT/HGT.py:35-44, three calls of segment_mm.cu:29-33 on one input) read X
 * once this way.  bf16 with K % 8 == 0, K <= 256 (or K % 4 == 0, K <= 128, two groups
 * at most), M % 128 == 0 and n_weights * M / 128 groups of 128 columns within the LDS
 * of a CU runs as one launch; every other shape ga_segment_mm takes runs as n_weights
 * launches with the same results. */
int ga_segment_mm_stacked(const int32_t *type_pointer, int64_t n_types, const void *X,
                          const void *const *W, void *const *Y, int64_t n_weights,
                          int64_t rows, int64_t K, int64_t M, int dtype, ga_stream_t stream);

/* Y[r] = (X[r] @ W[type(r)]) * g(gate[type(r)]), g the identity or, with gate_sigmoid != 0,
 * 1 / (1 + exp(-x)): SegmentMMNode (segment_mm.cu:23-27) with the per-node-type gate of
 * examples/HGT/HGT.py:58-60 (`trans_out * sigmoid(skip[ntype])`) applied to the fp32 sums
 * before they are rounded, so that neither the sigmoid, nor its copy to the nodes
 * (BroadcastNodeType, broadcast.cu:67-72), nor the multiplication is a pass of its own.
 * gate: (n_types,) fp32.  bf16 shapes of the wide kernel only (see ga_segment_mm_stacked);
 * GA_EUNSUPPORTED, having launched nothing, otherwise: the caller then forms the per-row
 * factor itself and passes it as row_scale of ga_segment_mm_gather. */
int ga_segment_mm_gated(const int32_t *type_pointer, int64_t n_types, const void *X,
                        const void *W, void *Y, const float *gate, int gate_sigmoid,
                        int64_t rows, int64_t K, int64_t M, int dtype, ga_stream_t stream);

/* out[b, j, i] = W[b, i, j] * scale[b] * factor over n_blocks square D x D blocks (scale
 * NULL: 1), computed in fp32 and rounded once to `dtype`: the relation matrices of
 * examples/HGT/HGT.py:39-45 transposed and carrying `relation_pri / sqrt(D)`, as the query
 * side of the scores needs them when the product is moved from the keys to the queries
 * (ga_dot_attention_sum).  out must not be W. */
int ga_transpose_scale_blocks(const void *W, const float *scale, float factor, void *out,
                              int64_t n_blocks, int64_t D, int dtype, ga_stream_t stream);
/* The same with `scale` stored as scale_dtype (GA_F32 or GA_BF16): a prior kept in the
 * model's bf16 needs no conversion pass of its own (bf16 -> fp32 is exact). */
int ga_transpose_scale_blocks_as(const void *W, const void *scale, int scale_dtype, float factor,
                                 void *out, int64_t n_blocks, int64_t D, int dtype,
                                 ga_stream_t stream);

/* Per-edge typed linear whose operand lives on the nodes, without the per-edge
 * copy: Y[r] = X[x_index[r]] @ W[type(r)] (x_index NULL: X[r]).  Replaces the
 * pair BroadcastSrcNode / BroadcastDstNode (broadcast.cu:58-66) -> SegmentMMEdge
 * (segment_mm.cu:29-33) that the reference's plans execute for
 * examples/RGCN/RGCN.py:26-28 and examples/HGT/HGT.py:35-44.  Exactly one of
 * two results:
 *   Y   (rows, heads*M) `dtype`, with Q / q_index / dot NULL; row_scale, when
 *       not NULL, is (rows,) fp32 and multiplies row r of Y (the per-edge norm
 *       of examples/RGCN/RGCN.py:29, read in edge order with the rows; with x_index
 *       NULL and the node type pointer it is the gate of examples/HGT/HGT.py:58-60
 *       on the output projection).  The factor multiplies the fp32 sums before they
 *       are rounded;
 *   dot (rows, heads) fp32 with Y NULL: dot[r, h] = <Y[r, h, :], Q[q_index[r], h, :]>
 *       (q_index NULL: Q[r]); Q (*, heads*M) `dtype`.  The product rows stay in
 *       registers (HGT's sum(k * q, dim=1), HGT.py:44-45).  scale, when not
 *       NULL, is (n_types, heads) fp32 and multiplies dot[r, h] by
 *       scale[type(r), h] (the relation_pri factor of HGT.py:45).
 * x_index / q_index are int64 (the COO columns of the graph); entries are not
 * checked on the device.  Returns GA_EUNSUPPORTED, having launched nothing, for
 * shapes outside the matrix-core tile (heads*K > 128 fp32 / 256 bf16,
 * heads*M > 128, K % 4 (fp32) or K % 8 (bf16) != 0; for dot also a head width M
 * that is not c, 2c, 4c, 8c or 16c with c = ceil(heads*M / 16) rounded up to a
 * power of two (at least 2 for bf16)); the caller then gathers with
 * ga_gather_rows.  Without index columns and dot operand, bf16 shapes of the wide
 * kernel (see ga_segment_mm_stacked) are taken as well; a call with row_scale whose
 * shape no matrix-core kernel takes also returns GA_EUNSUPPORTED (ga_segment_mm, then
 * the factor).
 */
int ga_segment_mm_gather(const int32_t *type_pointer, int64_t n_types, const void *X,
                         const int64_t *x_index, const void *W, void *Y,
                         const void *Q, const int64_t *q_index, const float *scale,
                         float *dot, const float *row_scale, int64_t rows,
                         int64_t heads, int64_t K, int64_t M, int dtype,
                         ga_stream_t stream);

/* ---------------------------------------------------------------- gather --
 * y[i, :] = x[idx[i], :], a bit-exact row copy of row_bytes bytes.
 * Replaces BroadcastSrcNode / DstNode / NodeType / EdgeType
 * (broadcast.cu:58-100: features.index({COO_src | COO_dst | ntype_COO |
 * etype_COO})).  idx is int64 (idx_bits 64) or int32 (idx_bits 32); entries
 * must lie in [0, n_in) -- they are not checked on the device.
 */
int ga_gather_rows(const void *idx, int idx_bits, const void *x, void *y,
                   int64_t n_out, int64_t row_bytes, ga_stream_t stream);

/* ------------------------------------------------- fused GAT aggregation --
 * The chain the reference's optimised GAT plan executes as four operators
 * (examples/GAT/GAT.py:25-36 after fusion.cpp:37-47,67-77):
 * gsddmm_u_add_v -> leaky_relu -> SegmentSoftmax -> gspmm_src_mul_e_sum,
 *   s_i = leaky_relu(el[nbr[i], h] + er[v, h], slope),  a = softmax_v(s),
 *   out[v, h, :] = sum_i a_i * z[nbr[i], h, :]
 * in one pass over the edges without materialising per-edge tensors.
 * el, er (n, heads) fp32; z, out (n, heads*dim) `dtype`.  Rows without edges
 * get 0.  workspace: ga_gat_workspace_bytes() bytes, 16-byte aligned.
 */
size_t ga_gat_workspace_bytes(int64_t n_edges, int64_t feat, int64_t heads);
int ga_gat_aggregate(const int32_t *pointer, const int32_t *row_of_slot,
                     const int32_t *nbr, const float *el, const float *er,
                     const void *z, void *out, int64_t n_rows, int64_t n_edges,
                     int64_t heads, int64_t dim, float slope, int dtype,
                     void *workspace, size_t workspace_bytes,
                     ga_stream_t stream);

/* ga_gat_aggregate for callers that cannot allocate device memory or hand over
 * a workspace: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It has no counterpart in the reference.  Same arguments,
 * kernels and results (bit for bit) as ga_gat_aggregate, but the partial rows of
 * destination rows that span workgroups go to a buffer of
 * GA_STATIC_SCRATCH_BYTES that the library holds in device memory itself (a
 * file-scope array: every GPU the library runs on keeps it until the process
 * ends).  The call allocates nothing and calls no allocating routine.
 *   - GA_ESCRATCH (nothing launched) when the graph and width need more partial
 *     rows than the buffer holds: 2 rows of heads*dim features per workgroup, with
 *     the softmax state beside every feature: x 1.5 for 16-byte lanes of fp32
 *     (4 features + maximum + denominator per lane), x 1.25 for 16-byte lanes of
 *     bf16 (8 features), and x 3 for rows that 16-byte accesses do not tile with
 *     several heads (one feature per lane, each with its own maximum and
 *     denominator).  64.3 M edges x 256 bf16 features need 20 MB, 11.6 M edges x
 *     64 fp32 features 4.3 MB.  ga_gat_static_scratch_needed gives the exact
 *     figure for a shape without touching the device.
 *   - All calls on one GPU share that GPU's buffer: calls that overlap on one
 *     GPU (two streams, two threads) race; calls on one stream are ordered.
 *   - The first call on a device looks the buffer's address up
 *     (hipGetSymbolAddress, once per device); make that call outside a stream
 *     capture.
 */
#define GA_STATIC_SCRATCH_BYTES (32u << 20)
int ga_gat_aggregate_static(const int32_t *pointer, const int32_t *row_of_slot,
                            const int32_t *nbr, const float *el, const float *er,
                            const void *z, void *out, int64_t n_rows, int64_t n_edges,
                            int64_t heads, int64_t dim, float slope, int dtype,
                            ga_stream_t stream);

/* Host arithmetic only (no device call, no pointer read): the bytes of the static
 * buffer that ga_gat_aggregate_static uses for a graph of n_edges edges and rows of
 * heads x dim values of `dtype`, stored at 16-byte aligned addresses or not (the
 * lane layout depends on it).  The call fits when the result is at most
 * GA_STATIC_SCRATCH_BYTES.  Negative: a GA_E* code for arguments the entry point
 * would reject.  No counterpart in the reference. */
int64_t ga_gat_static_scratch_needed(int64_t n_edges, int64_t heads, int64_t dim, int dtype,
                                     int rows_16_byte_aligned);

/* The same chain with the source term recomputed from the gathered row:
 *   s_i = leaky_relu(<z[nbr[i], h, :], a_l[h, :]> + er[v, h], slope)
 * instead of reading el[nbr[i], h].  Same result as ga_gat_aggregate with
 * el = z . a_l (up to fp32 summation order; for bf16 z the products use the
 * stored, rounded rows, as the reference's plan does when it evaluates
 * mm(z, attn_weight) on the stored z, examples/GAT/GAT.py:27-29).  It saves the
 * separate (n, heads) gather, one more memory sector per edge once that table
 * outgrows the caches (2.4 M nodes x 4 heads: 15 % of the traffic).  a_l is
 * (heads, dim) fp32.  GA_EUNSUPPORTED when the lanes that share a head
 * (dim / 8 for bf16, dim / 4 for fp32 with 16-byte aligned rows, else dim) are
 * not a power of two <= 16.
 */
int ga_gat_aggregate_from_z(const int32_t *pointer, const int32_t *row_of_slot,
                            const int32_t *nbr, const float *a_l, const float *er,
                            const void *z, void *out, int64_t n_rows, int64_t n_edges,
                            int64_t heads, int64_t dim, float slope, int dtype,
                            void *workspace, size_t workspace_bytes,
                            ga_stream_t stream);

/* ga_gat_aggregate / ga_gat_aggregate_from_z followed by the layer's activation
 * (`h = F.elu(h)` between the layers of the reference's GAT network,
 * examples/GAT/GAT.py; relu for GA_ACT_RELU; elu with alpha = 1) applied to the fp32
 * row before it is rounded and stored, so the (n, heads * dim) result is not written,
 * read and written again for it.  activation = GA_ACT_NONE is the plain entry point. */
int ga_gat_aggregate_act(const int32_t *pointer, const int32_t *row_of_slot,
                         const int32_t *nbr, const float *el, const float *er,
                         const void *z, void *out, int64_t n_rows, int64_t n_edges,
                         int64_t heads, int64_t dim, float slope, int activation, int dtype,
                         void *workspace, size_t workspace_bytes, ga_stream_t stream);
int ga_gat_aggregate_from_z_act(const int32_t *pointer, const int32_t *row_of_slot,
                                const int32_t *nbr, const float *a_l, const float *er,
                                const void *z, void *out, int64_t n_rows, int64_t n_edges,
                                int64_t heads, int64_t dim, float slope, int activation,
                                int dtype, void *workspace, size_t workspace_bytes,
                                ga_stream_t stream);

/* Dot-product attention over an adjacency, in one pass:
 *   s_i[h]       = <k[nbr[i], h, :], q[qrow[i], h, :]>      for the slots i of row r,
 *   out[r, h, :] = sum_i softmax_r(s)[i, h] * v[nbr[i], h, :],
 *   lse[r, h]    = log sum_i exp(s_i[h])                     (lse may be NULL; with lse_index,
 *                                                              int32 (n_rows), written to row
 *                                                              lse_index[r] instead of r)
 * i.e. sum(k * q) -> SegmentSoftmax -> mul -> SpMM of examples/HGT/HGT.py:44-53 with the
 * keys and values gathered from node rows and no per-edge tensor.  With the rows being
 * the (destination, relation) pairs of a graph (qrow: the pair's transformed query
 * row), lse is what combines the pairs of a destination into its softmax afterwards.
 * nbr, qrow (n_edges) int32; k, v (*, heads*dim), q (*, heads*dim) `dtype`; out
 * (n_rows, heads*dim) `dtype`, lse (n_rows, heads) fp32; rows without slots get 0 and
 * -inf.  Needs 16-byte aligned k, q, v, out and dim a multiple of 4 (fp32) / 8 (bf16)
 * with dim / that a power of two up to 16 (GA_EUNSUPPORTED otherwise).  workspace:
 * ga_gat_workspace_bytes(n_edges, heads*dim, heads) bytes, 16-byte aligned. */
int ga_dot_attention_sum(const int32_t *pointer, const int32_t *row_of_slot,
                         const int32_t *nbr, const int32_t *qrow, const void *k, const void *q,
                         const void *v, void *out, float *lse, const int32_t *lse_index,
                         int64_t n_rows, int64_t n_edges, int64_t heads, int64_t dim, int dtype,
                         void *workspace, size_t workspace_bytes, ga_stream_t stream);

/* The softmax-weighted reduction with per-edge operands:
 *   a = softmax_v(logit[e, h] over the in-edges e of v),
 *   out[v, h, :] = sum_e a_e * m[e, h, :]
 * replacing the tail SegmentSoftmax -> mul -> SpMMEdge (segment_softmax.cu:3-24,
 * spmm.cu:359-373) of the reference's HGT plan (examples/HGT/HGT.py:50-53) in
 * one pass, with no (E, heads) attention tensor.  logit (E, heads) fp32 and
 * m (E, heads*dim) `dtype` are in edge-id order and are read through `eid`
 * (NULL when slot i holds edge i).  Rows without edges get 0.  workspace:
 * ga_gat_workspace_bytes(n_edges, heads*dim, heads) bytes, 16-byte aligned.
 */
int ga_edge_softmax_sum(const int32_t *pointer, const int32_t *row_of_slot,
                        const int32_t *eid, const float *logit, const void *m,
                        void *out, int64_t n_rows, int64_t n_edges, int64_t heads,
                        int64_t dim, int dtype, void *workspace,
                        size_t workspace_bytes, ga_stream_t stream);

/* ------------------------------------------- dense projection (fp32) ------
 * Z = X @ W and, optionally, the per-head attention terms of a GAT layer
 * el[n, h] = <Z[n, h, :], a_l[h, :]>, er likewise, in the same kernel.
 * Replaces the dense operators in front of the graph chain in the reference's
 * GAT plan: mm(h, fc_weight) and the two halves of mm(z2, attn_weight)
 * (examples/GAT/GAT.py:25-29 after the split and reorder passes,
 * src/optimizer/split.cpp:5-34); with el == er == NULL it is the plain node
 * projection of examples/GCN/GCN.py:39.  X (rows, K), W (K, M), Z (rows, M),
 * a_l / a_r (heads, M/heads), el / er (rows, heads), all fp32.
 * Every fp32 product is formed exactly, from bf16 pieces of its operands on the
 * matrix unit, and summed in fp32: the result is as close to the exact product
 * as plain fp32 arithmetic gets; a non-finite input gives NaN.
 * GA_EUNSUPPORTED when the attention terms are requested with M/heads not in
 * {16, 32, 64}, when K > 2^22 or when K * M >= 2^30.
 */
int ga_linear_attn(const float *X, const float *W, const float *a_l,
                   const float *a_r, float *Z, float *el, float *er,
                   int64_t rows, int64_t K, int64_t M, int64_t heads,
                   ga_stream_t stream);

/* The plain projection with a factor per row: Z[n, :] = (X[n, :] @ W) * row_scale[n]
 * (row_scale (rows) fp32, NULL for none) -- the projection of examples/GCN/GCN.py:39
 * together with the source-side norm of the message (`edges.src['h'] * norm`,
 * GCN.py:22-23), which multiplies exactly these rows.  The product is rounded to
 * fp32 first and then multiplied, as the two separate operators do.  Limits as
 * ga_linear_attn.
 */
int ga_linear_rows_scaled(const float *X, const float *W, const float *row_scale, float *Z,
                          int64_t rows, int64_t K, int64_t M, ga_stream_t stream);

/* The same projection with the attention terms for fp32 or bf16 storage (fp32
 * accumulation; el / er are fp32 and are taken from the accumulators, before Z
 * is rounded): the 100 -> 256 (4 heads x 64, bf16) layer of the larger GAT
 * configuration as one operator instead of three GEMMs.  fp32 with M/heads in
 * {16, 32, 64} runs ga_linear_attn; other cases run the typed-linear tile
 * kernel with a single type, column passes of 128 inside one launch.  X (rows, K),
 * W (K, M), Z (rows, M) `dtype`; a_l / a_r (heads, M/heads), el / er
 * (rows, heads) fp32, all required.  GA_EUNSUPPORTED (nothing launched) when
 * K > 128 (fp32) / 256 (bf16, K % 8 == 0) / 128 (bf16, K % 4 == 0), K % 4 != 0,
 * M/heads > 128, or M/heads not a multiple of 16 (fp32) / of 32 and not 16 (bf16).
 */
int ga_project_attn(const void *X, const void *W, const float *a_l,
                    const float *a_r, void *Z, float *el, float *er,
                    int64_t rows, int64_t K, int64_t M, int64_t heads, int dtype,
                    ga_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* GRAPHILER_AMD_H_ */
