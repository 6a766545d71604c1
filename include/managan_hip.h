/*
 * managan_hip.h — C ABI of the MI355X (gfx950) implementation of the
 * equivariant message-passing hot path: periodic cell-list neighbour search,
 * fused Cartesian tensor products + per-irrep channel-mixing linears, and the
 * edge->node segment sum.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the comment says "host";
 *   - every tensor is dense row-major float32 (indices int32) unless stated;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - every entry point returns an mg_status; nothing is thrown, nothing
 *     terminates the process; mg_last_error() gives the text of the last
 *     failure on the calling thread;
 *   - no entry point allocates or frees device memory: callers own outputs and
 *     pass workspaces whose sizes the *_workspace_bytes functions report;
 *   - entry points only enqueue work on `stream`; they synchronise nothing.
 *
 * Each declaration names the reference interface it stands in for
 * (file:line relative to the pb1729/learned-dynamics checkout).
 */
#ifndef MANAGAN_HIP_H
#define MANAGAN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* mg_stream_t;

enum mg_status {
    MG_OK = 0,
    MG_ERR_INVALID_ARGUMENT = 1, /* bad shape / size / null pointer / alignment */
    MG_ERR_HIP = 2,              /* a HIP runtime call failed, see mg_last_error() */
    MG_ERR_BOX_TOO_SMALL = 3,    /* "box dimension must be greater than 3*cutoff" */
    MG_ERR_WORKSPACE = 4,        /* workspace smaller than *_workspace_bytes reports */
    MG_ERR_UNSUPPORTED = 5       /* e.g. tensor rank > 2 */
};

const char* mg_status_string(int status);
const char* mg_last_error(void);
int mg_abi_version(void);

/* ------------------------------------------------------------------------
 * Stage A — periodic radius graph.
 * Stands in for get_neighbours / get_edges
 * (extensions/neighbour_grid/neighbour_grid.cpp:59-103,170-195) and the kernels
 * assignParticlesToCells, createNeighbourListsKern, writeSrcDstKern
 * (extensions/neighbour_grid/neighbour_grid_kern.cu:57-150,334-352).
 * Two phases so the caller can size the edge arrays:
 *   count: bins atoms, walks the 3x3x3 cell window, writes the CSR row_ptr
 *          (batch*nodes+1, exclusive prefix), edge_counts (batch, inclusive
 *          prefix per box, as the reference's edgeCounts) and stats[4] =
 *          {E, max atoms in a cell, max degree, flags: bit 0 = E overflowed int32},
 *          each word stored exactly once per call (a caller may point stats at
 *          device-visible pinned host memory preset to -1 and poll it);
 *   fill:  writes src[e] = b*nodes+i and dst[e] = b*nodes+j, rows ordered by
 *          (b,i); order inside a row is deterministic.  n_edges is the CAPACITY of
 *          src and dst in edges: an edge whose position row_ptr[row] + k is not
 *          below n_edges is dropped (nothing is ever written past the arrays).  A
 *          caller that sized the arrays without reading stats[0] back (no host
 *          synchronisation, e.g. under stream capture) compares stats[0] with its
 *          capacity afterwards: the first min(stats[0], n_edges) entries are the
 *          complete rows, in order, that fit.
 * The reference's listmax / neighboursmax caps are not needed (exact-size CSR);
 * callers that want the reference's overflow errors compare stats[1], stats[2]
 * with their caps.
 * ---------------------------------------------------------------------- */
int mg_neighbour_ndiv(float cutoff, float box_x, float box_y, float box_z, int ndiv[3] /* host */);

/* The workspace holds the wrapped and cell-sorted atoms, the cell table and one row per atom that collects the
 * atom's neighbours between the two phases (box-local ids: 16 bits each when a box has at most 65536 atoms, else
 * 32).  mg_neighbour_workspace_bytes reports the preferred size: rows of 256 entries.  The count, fill and
 * cell-order calls also accept a smaller workspace (the same pointer and size in all of them) and then use the
 * longest rows that fit, down to 32 entries; an atom with more neighbours than a row holds costs a second sweep
 * of its window in the fill pass, nothing else.  Below that the calls return MG_ERR_WORKSPACE. */
int mg_neighbour_workspace_bytes(int batch, int nodes, float cutoff,
                                 float box_x, float box_y, float box_z, size_t* bytes /* host */);

int mg_neighbour_count(const float* x /* (batch,nodes,3) */, int batch, int nodes, float cutoff,
                       float box_x, float box_y, float box_z,
                       void* workspace, size_t workspace_bytes,
                       int* row_ptr /* batch*nodes+1 */, int* edge_counts /* batch */,
                       int* stats /* 4 */, mg_stream_t stream);

int mg_neighbour_fill(const void* workspace, size_t workspace_bytes, int batch, int nodes,
                      float cutoff, float box_x, float box_y, float box_z,
                      const int* row_ptr, int n_edges, int* src, int* dst, mg_stream_t stream);

/* Both phases in one call for a caller that sizes src / dst itself (`capacity` edges each) and does not want to read
 * the edge count back in between: get_edges (extensions/neighbour_grid/neighbour_grid.cpp:170-195) without its
 * device->host copies.  What the caller gets is the graph truncated at `capacity` edges: edges beyond the capacity
 * are dropped as in mg_neighbour_fill, and row_ptr / edge_counts entries above the capacity are lowered to it, so a
 * kernel that walks the edges through row_ptr never leaves the edge arrays (the rows that did not fit are short or
 * empty).  stats[0] holds the true count and stats[3] has bit 1 (value 2) set when edges were dropped: read them
 * after the work that used the graph to know whether its result is that of the whole graph.
 * Nothing in it synchronises or allocates, so the call can be recorded into a HIP graph. */
int mg_neighbour_edges(const float* x /* (batch,nodes,3) */, int batch, int nodes, float cutoff,
                       float box_x, float box_y, float box_z, void* workspace, size_t workspace_bytes,
                       int* row_ptr /* batch*nodes+1 */, int* edge_counts /* batch */, int* stats /* 4 */,
                       int capacity, int* src /* capacity */, int* dst /* capacity */, mg_stream_t stream);

/* mg_neighbour_edges without a workspace argument, for callers that cannot allocate one (code under HIP graph
 * capture, tight serving loops, harnesses that forbid allocation).  No counterpart in the reference.  The workspace
 * is a 64 MiB buffer built into the library (one per GPU, held until the process ends), used with the longest
 * neighbour rows that fit (see mg_neighbour_workspace_bytes: 8 boxes of 16384 atoms get rows of 224 entries); a
 * search that does not fit with rows of 32 entries (116 bytes per atom plus 8 per cell: beyond about 500 000 atoms
 * over all boxes) is refused with MG_ERR_WORKSPACE and a message.  The call allocates and frees nothing and
 * synchronises nothing;
 * inputs and outputs are the caller's.
 * All calls on one GPU share the buffer: calls that overlap in time on the same GPU (two streams, two threads)
 * race, calls ordered on one stream do not.  The first call on a device looks the buffer's address up
 * (hipGetSymbolAddress): make that call outside stream capture. */
int mg_neighbour_edges_static(const float* x /* (batch,nodes,3) */, int batch, int nodes, float cutoff,
                              float box_x, float box_y, float box_z,
                              int* row_ptr /* batch*nodes+1 */, int* edge_counts /* batch */, int* stats /* 4 */,
                              int capacity, int* src /* capacity */, int* dst /* capacity */, mg_stream_t stream);

/* After mg_neighbour_count on the same workspace: order[k] = global id (b*nodes + i) of the k-th atom in
 * cell order (boxes, then cells x-major, then atom id).  Processing the rows of the fused edge kernels
 * in this order keeps the gathered neighbours of consecutive rows close together in time (cache
 * locality) when atom ids carry no spatial meaning.  No counterpart in the reference. */
int mg_neighbour_cell_order(const void* workspace, size_t workspace_bytes, int batch, int nodes,
                            float cutoff, float box_x, float box_y, float box_z,
                            int* order /* batch*nodes */, mg_stream_t stream);

/* First step of the search on its own: wrapped positions (batch,nodes,3) and box-local
 * linear cell ids (batch,nodes), as assignParticlesToCells computes them
 * (extensions/neighbour_grid/neighbour_grid_kern.cu:75-82).  Diagnostic / test entry. */
int mg_neighbour_wrap_cells(const float* x, int batch, int nodes, float cutoff,
                            float box_x, float box_y, float box_z,
                            float* wrapped, int* cell, mg_stream_t stream);

/* CSR -> the reference's padded table (get_neighbours,
 * extensions/neighbour_grid/neighbour_grid.cpp:59-103): neighbours
 * (batch,nodes,neighboursmax) holds box-local indices, entries >= count are
 * left untouched; counts (batch,nodes). */
int mg_neighbour_pad(const int* row_ptr, const int* dst, int batch, int nodes, int neighboursmax,
                     int* neighbours, int* counts, mg_stream_t stream);

/* Padded gather / reduce (edges_read, edges_reduce:
 * extensions/neighbour_grid/neighbour_grid.cpp:105-167; kernels
 * neighbour_grid_kern.cu:226-306). */
int mg_padded_edges_read(const int* counts, const int* neighbours, const float* x /* (batch,nodes,chan) */,
                         int batch, int nodes, int neighboursmax, int chan,
                         float* edge_data /* (batch,nodes,neighboursmax,chan) */, mg_stream_t stream);
int mg_padded_edges_reduce(const int* counts, const float* edge_data, int batch, int nodes,
                           int neighboursmax, int chan, float* out /* (batch,nodes,chan) */,
                           mg_stream_t stream);

/* r_ij[e] = boxwrap(box, x[dst[e]] - x[src[e]]) with floor-mod, fp32
 * (managan/graph_layers.py:62-66 applied as in archs/meanflow_painn8.py:167-172)
 * and, if shift != NULL, the periodic image rint(((x_j - x_i) - r_ij)/box) as int8 x3. */
int mg_edge_vectors(const float* x /* (batch*nodes,3) */, const int* src, const int* dst, long n_edges,
                    float box_x, float box_y, float box_z, float* r_ij /* (E,3) */,
                    int8_t* shift /* (E,3) or NULL */, mg_stream_t stream);

/* ------------------------------------------------------------------------
 * Stage C — gather to edges and sum edges -> nodes.
 * Stand in for x_node[graph.dst] (managan/graph_layers.py:37-52) and
 * torch_scatter.segment_coo(x_edge, graph.src, dim_size=batch*nodes)
 * (managan/graph_layers.py:54-59).
 * ---------------------------------------------------------------------- */
/* row_ptr[r] = first e with index[e] >= r, r = 0..n_rows (index sorted ascending).
 * index_is_int64 selects the element type of `index`. */
int mg_segment_row_ptr(const void* index, int index_is_int64, long n_edges, int n_rows,
                       int* row_ptr /* n_rows+1 */, mg_stream_t stream);
/* out[r, :] = sum over e in [row_ptr[r], row_ptr[r+1]) of x_edge[e, :], in edge order. */
int mg_segment_sum_csr(const float* x_edge /* (E,feat) */, const int* row_ptr, int n_rows, int feat,
                       float* out /* (n_rows,feat) */, mg_stream_t stream);
/* The same for an index that is not sorted: perm (E ints) lists the rows of x_edge in the sorted order of the index
 * (a stable sort), row_ptr is that of the sorted index, and out[r, :] = sum over e in [row_ptr[r], row_ptr[r+1]) of
 * x_edge[perm[e], :]: the adjoint of a gather by an unsorted index (torch's index backward under
 * managan/graph_layers.py:37-52), without a permuted copy of x_edge.  perm == NULL: mg_segment_sum_csr. */
int mg_segment_sum_csr_perm(const float* x_edge /* (E,feat) */, const int* perm, const int* row_ptr, int n_rows,
                            int feat, float* out /* (n_rows,feat) */, mg_stream_t stream);
/* out[e, :] = x[index[e], :] */
int mg_gather_rows(const float* x /* (n_rows,feat) */, const void* index, int index_is_int64,
                   long n_edges, int n_rows, int feat, float* out /* (E,feat) */, mg_stream_t stream);

/* ------------------------------------------------------------------------
 * Stage B — Cartesian tensor products (elementwise over rows x chan).
 * Operand layouts (rows,chan), (rows,chan,3), (rows,chan,3,3).
 * ---------------------------------------------------------------------- */
/* bee_fwd_cuda (extensions/codegen_tensops/codegen_tensops.cpp:1519-1573, kernel
 * codegen_tensops_kern.cu:3800-3875).  y: host array of 13 device pointers in the
 * order 000,110,220,011,101,121,211,022,202,112,222,111,212. */
int mg_bee_fwd(const float* l_0, const float* l_1, const float* l_2,
               const float* r_0, const float* r_1, const float* r_2,
               long rows, int chan, float* const y[13] /* host array */, mg_stream_t stream);
/* bee_bwl_cuda / bee_bwr_cuda (codegen_tensops.cpp:1575-1769): gradient with respect to
 * the left (resp. right) operands given the OTHER side's operands o_0,o_1,o_2 and the 13
 * output gradients.  side = 0: o = r, outputs dl; side = 1: o = l, outputs dr. */
int mg_bee_bwd(int side, const float* o_0, const float* o_1, const float* o_2,
               const float* const dy[13] /* host array */, long rows, int chan,
               float* d_0, float* d_1, float* d_2, mg_stream_t stream);
/* The same with operands given per node and read through an index (a gather folded into the kernel; chan a multiple
 * of 256: mg_bee_indexed_supported).  mg_bee_fwd_indexed: l_* hold l_rows rows and product row e reads row l_index[e]
 * (Messages: the destination's L0 x_a, L1 x_v, L2 x_d, archs/diffuser_atoms15.py:244-247).  mg_bee_bwd_indexed: the
 * other side's operands through o_index (or NULL), and the output gradients dy[k] with bit k of dy_indexed set hold
 * dy_rows rows and are read at row dy_index[e] (products that were summed over the edges of a node: the gradient of an
 * edge's row is its node's).  Indices outside the operand are clamped.  The reference gathers first
 * (managan/graph_layers.py:37-52). */
int mg_bee_indexed_supported(int chan);   /* returns 0 / 1, not a status */
int mg_bee_fwd_indexed(const float* l_0, const float* l_1, const float* l_2, const int* l_index, long l_rows,
                       const float* r_0, const float* r_1, const float* r_2, long rows, int chan,
                       float* const y[13] /* host array */, mg_stream_t stream);
int mg_bee_bwd_indexed(int side, const float* o_0, const float* o_1, const float* o_2, const int* o_index, long o_rows,
                       const float* const dy[13] /* host array */, const int* dy_index, long dy_rows,
                       unsigned dy_indexed, long rows, int chan, float* d_0, float* d_1, float* d_2,
                       mg_stream_t stream);
/* cow_o0_fwd_cuda: products 000,110 (codegen_tensops.cpp:1771-1802). */
int mg_cow_o0_fwd(const float* l_0, const float* l_1, const float* r_0, const float* r_1,
                  long rows, int chan, float* y_000, float* y_110, mg_stream_t stream);
/* cow_o1_fwd_cuda: products 011,101,111 (codegen_tensops.cpp:1868-1900). */
int mg_cow_o1_fwd(const float* l_0, const float* l_1, const float* r_0, const float* r_1,
                  long rows, int chan, float* y_011, float* y_101, float* y_111, mg_stream_t stream);
/* cow_o0_bw{l,r}_cuda, cow_o1_bw{l,r}_cuda (codegen_tensops.cpp:1804-1866,1902-1978). */
int mg_cow_o0_bwd(int side, const float* o_0, const float* o_1, const float* dy_000, const float* dy_110,
                  long rows, int chan, float* d_0, float* d_1, mg_stream_t stream);
int mg_cow_o1_bwd(int side, const float* o_0, const float* o_1, const float* dy_011, const float* dy_101,
                  const float* dy_111, long rows, int chan, float* d_0, float* d_1, mg_stream_t stream);
/* TensorProdBare.forward (managan/tensor_products.py:91-106) for one non-chiral
 * (inds_l, inds_r, inds_o) with all ranks <= 2. */
int mg_tensor_prod_bare(int inds_l, int inds_r, int inds_o, const float* x_l, const float* x_r,
                        long rows, int chan, float* y, mg_stream_t stream);
/* TensorProds.forward in one launch (managan/tensor_products.py:109-121):
 *   y = lin_o(prod(lin_l(x_l), lin_r(x_r))),  lin_l: W_l (rank, dim_l), lin_r: W_r (rank, dim_r), lin_o: W_o (dim_o, rank),
 * weights with row strides ldl / ldr / ldo (unit stride along a row), x_l (rows, dim_l, (3,)^inds_l),
 * x_r (rows, dim_r, (3,)^inds_r), y (rows, dim_o, (3,)^inds_o) dense and 16-byte aligned.  Needs channel counts that are
 * multiples of 16 and weights that fit 64 KB of LDS: mg_tensor_prods_supported returns 1 if a problem qualifies
 * (a yes/no answer, not a status); otherwise compose mg_tensor_linear and mg_tensor_prod_bare. */
int mg_tensor_prods_supported(int inds_l, int inds_r, int inds_o, int dim_l, int dim_r, int rank, int dim_o);
int mg_tensor_prods(int inds_l, int inds_r, int inds_o, const float* W_l, long ldl, const float* W_r, long ldr,
                    const float* W_o, long ldo, const float* x_l, const float* x_r, long rows, int dim_l, int dim_r,
                    int rank, int dim_o, float* y, mg_stream_t stream);
/* The three products the vector/scalar pair of one TensorProds stack needs in one pass:
 * y_110 = v.v', y_011 = a v', y_112 = v (x) v' with v = left vector, v' = right vector,
 * a = scalar (managan/tensor_products.py:91-121 applied three times). */
int mg_tensor_prods_avd(const float* a, const float* v_l, const float* v_r, long rows, int chan,
                        float* y_110, float* y_011, float* y_112, mg_stream_t stream);

/* ------------------------------------------------------------------------
 * Stage B — per-irrep channel-mixing linear (dense contraction, MFMA).
 * tensor_linear (extensions/tensor_ops/tensor_ops.cpp:31-93; kernel
 * tensor_ops_kern.cu:6-42): y[r,o,t] = sum_i W[o,i] x[r,i,t], t < 3^inds;
 * W is read with element strides (w_stride_o, w_stride_i) so a transposed view costs nothing.
 * Optional fused epilogue (used for nn.Linear inside the MLPs, inds = 0):
 *   y = act(y + bias[o]); act: 0 none, 1 SiLU, 2 LeakyReLU(0.1); bias may be NULL.
 * accumulate != 0 adds into y instead of overwriting it.
 * ---------------------------------------------------------------------- */
int mg_tensor_linear(int inds, const float* W, long w_stride_o, long w_stride_i,
                     const float* x, long rows, int dim_in, int dim_out,
                     const float* bias, int act, int accumulate, float* y, mg_stream_t stream);
/* The same contraction with explicit memory layouts of x and y:
 *   0 = (row, chan, comp), how the reference stores every tensor;
 *   1 = (row, comp, chan), component-major: what the fused edge kernels gather from and
 *       accumulate into, so that a wave's accesses are unit-stride. */
int mg_tensor_linear_layout(int inds, const float* W, long w_stride_o, long w_stride_i,
                            const float* x, long rows, int dim_in, int dim_out,
                            const float* bias, int act, int accumulate,
                            int x_layout, int y_layout, float* y, mg_stream_t stream);
/* Arithmetic used by the wide plain-row GEMMs (inds = 0 or component-major x, dim_in % 32 == 0):
 *   0  fp32 MFMA (v_mfma_f32_32x32x2_f32);
 *   1  operands split exactly into three bf16 pieces, six bf16 MFMAs per product, fp32
 *      accumulation: same accuracy class as fp32 (dropped terms < 2^-24 |a||b|), ~2.7x the rate;
 *   2  as 1 for callers of mg_tensor_linear*; the host side additionally routes wide plain-row
 *      layers through mg_tensor_linear_f16x2 (below).
 * Process-wide setting; no counterpart in the reference (its kernel is a plain fp32 dot product,
 * extensions/tensor_ops/tensor_ops_kern.cu:6-42). */
int mg_set_linear_mode(int mode);
int mg_get_linear_mode(void);
/* Pre-split weights for mode 1: W (dim_out, dim_in, any strides) -> three bf16 planes (hi, mid, lo),
 * dim_out rounded up to 128 rows, in caller-owned memory of mg_linear_packed_weight_bytes bytes
 * (16-byte aligned).  mg_tensor_linear_packed then computes, for plain rows x (rows, dim_in),
 * y = act(x W^T + bias) with x split on the fly; out_comps = 1 writes y (rows, dim_out); out_comps =
 * 3 or 9 treats the rows as (row, comp) pairs and writes y (rows/out_comps, dim_out, out_comps).
 * dim_in % 32 == 0, x 16-byte aligned.  Same contraction as tensor_linear
 * (extensions/tensor_ops/tensor_ops.cpp:31-93); the packing has no counterpart in the reference. */
int mg_linear_packed_weight_bytes(int dim_in, int dim_out, size_t* bytes /* host */);
int mg_linear_pack_weight(const float* W, long w_stride_o, long w_stride_i, int dim_in, int dim_out,
                          void* packed, mg_stream_t stream);
int mg_tensor_linear_packed(const void* packed_W, const float* x, long rows, int dim_in, int dim_out,
                            const float* bias, int act, int accumulate, int out_comps, float* y,
                            mg_stream_t stream);
/* Mode 2: two-piece fp16 split with per-row power-of-two scales, three fp16 MFMAs per product,
 * fp32 accumulation (a few fp32 ulps per product; half the matrix work of mode 1).
 * mg_linear_f16x2_pack_weight: W -> hi / lo fp16 planes (dim_out rounded up to 256 rows) followed by
 * one fp32 inverse scale per row, in caller-owned memory of mg_linear_f16x2_packed_weight_bytes bytes.
 * mg_tensor_linear_f16x2: y = act(x W^T + bias) for plain rows x (rows, dim_in), dim_in % 32 == 0;
 * x_rowmax[(r / x_rows_per_bound) * x_rowmax_stride + p], p < x_rowmax_parts, holds upper bounds of
 * max_i |x[r,i]| (the largest part is used; any bound within a factor 2^14 of the true maximum keeps
 * full accuracy; stride 0 = one bound for all rows; x_rows_per_bound = 3 or 9 when the rows are the
 * components of a node that carries one bound): the y_rowmax output of the call that produced x,
 * mg_row_absmax(x) (one part), or a bound the caller derives from the producing layer's weights.  y_rowmax, if not NULL,
 * receives (rows, mg_tensor_linear_f16x2_rowmax_parts(rows, dim_in, dim_out)) partial row maxima of |y|
 * (out_comps must be 1).  out_comps / accumulate / act as in mg_tensor_linear_packed.
 * Same contraction as tensor_linear (extensions/tensor_ops/tensor_ops.cpp:31-93); packing, scales
 * and row maxima have no counterpart in the reference. */
int mg_linear_f16x2_packed_weight_bytes(int dim_in, int dim_out, size_t* bytes /* host */);
int mg_linear_f16x2_pack_weight(const float* W, long w_stride_o, long w_stride_i, int dim_in, int dim_out,
                                void* packed, mg_stream_t stream);
int mg_row_absmax(const float* x, long rows, int dim, float* out /* (rows) */, mg_stream_t stream);
int mg_tensor_linear_f16x2_rowmax_parts(long rows, int dim_in, int dim_out);   /* returns the count, not a status */
int mg_tensor_linear_f16x2(const void* packed_W, const float* x, const float* x_rowmax, int x_rowmax_parts,
                           long x_rowmax_stride, long x_rows_per_bound, long rows, int dim_in, int dim_out, const float* bias, int act, int accumulate,
                           int out_comps, float* y, float* y_rowmax, mg_stream_t stream);
/* The same with the bound of row r given as bound_mul * x_rowmax[r] + bound_add (both >= 0): lets a caller carry one
 * array of row maxima through a chain of layers, |act(x W^T + b)| <= |x|max * max_o sum_i |W[o,i]| + max|b|, without a
 * launch per layer to update it.  No counterpart in the reference. */
int mg_tensor_linear_f16x2_scaled_bound(const void* packed_W, const float* x, const float* x_rowmax, int x_rowmax_parts,
                                        long x_rowmax_stride, long x_rows_per_bound, long rows, int dim_in, int dim_out,
                                        const float* bias, int act, int accumulate, int out_comps, float* y,
                                        float* y_rowmax, float bound_mul, float bound_add, mg_stream_t stream);
/* y = act(x W^T + bias) in float64 arithmetic: W (dim_out, dim_in) and bias are the float32 parameters, widened
 * exactly; x (rows, dim_in), every product and sum, the activation and y (rows, dim_out) are double.  The same
 * contraction as nn.Linear inside the reference's MLPs (archs/meanflow_painn8.py:38-51); float64 has no counterpart
 * in the reference.  It exists to measure approximations of a float32 MLP against exact arithmetic on the device
 * (the acceptance test of the PaiNN filter grid), not as a compute path. */
int mg_linear_f64(const float* W, const float* bias /* may be NULL */, const double* x, long rows, int dim_in,
                  int dim_out, int act, double* y, mg_stream_t stream);
/* dW[o,i] = sum_{r,t} dy[r,o,t] x[r,i,t]  (tensor_ops_kern.cu:45-71), dW dense (dim_out,dim_in).  The rows are
 * reduced in slices whose partial results go to `workspace` (mg_tensor_linear_wgrad_workspace_bytes) and are added
 * in slice order: no atomics, the same bits on every run. */
int mg_tensor_linear_wgrad_workspace_bytes(long rows, int dim_in, int dim_out, size_t* bytes /* host */);
int mg_tensor_linear_wgrad(int inds, const float* dy, const float* x, long rows, int dim_in, int dim_out,
                           void* workspace, float* dW, mg_stream_t stream);
/* The same for plain rows (inds = 0) on the fp16 matrix cores with two-piece operands: dy and x are each scaled by one
 * power of two and split into hi + lo fp16 pieces, three matrix instructions per step, fp32 accumulation; the error
 * is a few fp32 ulps of sum |dy| |x|, as for mg_tensor_linear_f16x2.  dy_bound / x_bound: device arrays of
 * n_dy_bound / n_x_bound floats whose largest magnitude is an upper bound of |dy| / |x| (for instance the row maxima
 * from mg_row_absmax; how tight does not matter within a factor 2^14), or NULL: the operand itself is scanned first.
 * db, if not NULL, receives the bias gradient db[o] = sum_r dy[r,o] (plain fp32 sums, slices added in order) from the
 * same pass.  Needs mg_tensor_linear_wgrad_f16x2_supported(rows, dim_in, dim_out) != 0 and 16-byte aligned dy, x;
 * workspace as for mg_tensor_linear_wgrad.  Same sum as tensor_ops_kern.cu:45-71; scales and bounds have no counterpart there. */
int mg_tensor_linear_wgrad_f16x2_supported(long rows, int dim_in, int dim_out);   /* returns 0 / 1, not a status */
int mg_tensor_linear_wgrad_f16x2(const float* dy, const float* x, const float* dy_bound, long n_dy_bound,
                                 const float* x_bound, long n_x_bound, long rows, int dim_in, int dim_out,
                                 void* workspace, float* dW, float* db /* (dim_out) or NULL */, mg_stream_t stream);

/* ------------------------------------------------------------------------
 * Ant16 (managan/codegen_tensor_products.py:19-34; ant16_o0_cuda / ant16_o1_cuda / ant16_o2_cuda /
 * ant16_oc_cuda, extensions/codegen_tensops/codegen_tensops.cpp:610-667,823-890,1072-1140,1327-1390):
 *   y[b,o,:] (+)= sum_t sum_{i<dim_l, j<dim_r} P_t[o,i,j] * (left_t[b,i,:] (x) x_r[b,j,:])
 * over n_terms <= 6 product types that share the output rank rank_o.  labels[t] indexes the order
 * 000 110 220 011 101 121 211 022 202 112 222 111 212; P_t (dim_o, dim_l, dim_r) and
 * left_t (rows, dim_l, (3,)^rank_l) dense; x_k (rows, dim_k, (3,)^k); y (rows, dim_o, (3,)^rank_o).
 * labels, P and left are HOST arrays of n_terms entries (device pointers inside).  accumulate != 0
 * adds into y.  One call per reference function (o0: 000 110 220; o1: 011 101 121 211;
 * o2: 022 202 112 222; oc: 111 into y_1c and 212 into y_2c as two calls). */
int mg_ant16_fwd(int rank_o, int n_terms, const int* labels, const float* const* P, const float* const* left,
                 const float* x_0, const float* x_1, const float* x_2, long rows, int dim_0, int dim_1, int dim_2,
                 int dim_l, int accumulate, float* y, mg_stream_t stream);
/* Gradient for x of rank rank_r (ant16_o{0,1,2,c}_backward_cuda, codegen_tensops.cpp:669-821 and the oc variant
 * at 1374-1420): dx[b,j,:] (+)= sum_t sum_{o,i} P_t[o,i,j] * C(left_t[b,i,:], dy_o[b,o,:]) over n_terms <= 6 product
 * types whose right operand has rank rank_r (they may differ in output rank: dy_k is the gradient of the rank-k
 * output, null if no term needs it).  Tables as for mg_ant16_fwd.  dx (rows, dim_{rank_r}, (3,)^rank_r). */
int mg_ant16_grad_x(int rank_r, int n_terms, const int* labels, const float* const* P, const float* const* left,
                    const float* dy_0, const float* dy_1, const float* dy_2, long rows, int dim_0, int dim_1, int dim_2,
                    int dim_l, int accumulate, float* dx, mg_stream_t stream);
/* Gradient for the left operand of one product type (ant16_o*_backleft_cuda, codegen_tensops.cpp:892-1070,
 * 1421-1470): dleft[b,i,:] = sum_{o,j} P[o,i,j] * C(x[b,j,:], dy[b,o,:]); x of the type's right rank, dy of its
 * output rank; dleft (rows, dim_l, (3,)^rank_l). */
int mg_ant16_grad_left(int label, const float* P, const float* x, const float* dy, long rows, int dim_0, int dim_1,
                       int dim_2, int dim_l, float* dleft, mg_stream_t stream);
/* Gradient for P of one product type (ant16_o*_wtsback_cuda, codegen_tensops.cpp:1142-1325, 1471-1517):
 * dP[o,i,j] = sum_{b} <dy[b,o,:], left[b,i,:] (x) x[b,j,:]>.  The rows are reduced in slices whose partial results go
 * to `workspace` (mg_ant16_grad_weight_workspace_bytes, with dim_o / dim_r the channel counts of the type's output /
 * right rank) and are added in slice order: no atomics, the same bits on every run. */
int mg_ant16_grad_weight_workspace_bytes(long rows, int dim_o, int dim_l, int dim_r, size_t* bytes /* host */);
int mg_ant16_grad_weight(int label, const float* left, const float* x, const float* dy, long rows, int dim_0, int dim_1,
                         int dim_2, int dim_l, void* workspace, float* dP, mg_stream_t stream);

/* ------------------------------------------------------------------------
 * PaiNN message passing (archs/meanflow_painn8.py:25-35,77-100).
 * ---------------------------------------------------------------------- */
/* radial_encode(r, n, rmax) (archs/meanflow_painn8.py:25-35): out (E,n) =
 * [cos(k_m d)]_{m<hn} | [sin(k_m d)]_{m<n-hn}, k_m = (pi/rmax)(1 + m/2), hn = (n+1)/2, d = |r|. */
int mg_painn_radial_encode(const float* r_ij /* (E,3) */, long n_edges, int n, float rmax,
                           float* out /* (E,n) */, mg_stream_t stream);
/* First layer of Message.mlp_dist applied to the encoding without materialising it
 * (archs/meanflow_painn8.py:25-35 feeding :38-51 at :92):
 *   y[e,o] = act(bias[o] + sum_m W[o,m] radial_encode(r_ij[e], n, rmax)[m]),  y (E,dim_out).
 * n <= 32; dim_out = 4 * 2^k <= 1024.  act as in mg_tensor_linear_layout. */
int mg_painn_radial_linear(const float* r_ij /* (E,3) */, long n_edges, int n, float rmax, const float* W,
                           long w_stride_o, long w_stride_i, const float* bias, int dim_out, int act,
                           float* y, mg_stream_t stream);
/* mg_painn_message with the filter taken from a table instead of one row per edge.  The radial MLP of
 * Message.forward (archs/meanflow_painn8.py:92) sees an edge only through d = |r_ij|, and its input
 * radial_encode(r, n, rmax) (:25-35) consists of cos / sin (k pi d / rmax) with integer k, so the filter is a smooth
 * function of d with period 2 rmax.  table (table_rows, 4n): that function at d = k * period / table_rows, k = 0 ..
 * table_rows - 1 (table_rows a power of two, period = 2 rmax); every edge interpolates its filter between the four
 * rows around d (4-point Lagrange, indices wrapped), error <= 0.0234 (period / table_rows)^4 max |d^4 filter / dd^4|.
 * Everything else as mg_painn_message. */
int mg_painn_table_message(const int* row_ptr, const int* dst, const int* node_order, int n_nodes, long n_edges,
                           const float* r_ij, const float* table, int table_rows, float period, const float* actv,
                           const float* x_v, int n, float epsilon, const float* res_a, const float* res_v, float* out_a,
                           float* out_v, mg_stream_t stream);
/* mg_painn_table_message with the table in LDS: table_rows <= 512, n % 16 == 0.  A workgroup keeps the filter columns of
 * one slice of 16 channels for every table row in LDS, so only node rows are gathered through the caches.
 * What an edge contributes apart from its node rows (its first table row, the four interpolation weights, the
 * direction r / sqrt(epsilon + |r|^2)) is written once per edge by mg_painn_edge_records into `records` (n_edges x 8
 * floats, 16-byte aligned) and read by every slice.
 * actv_sliced (n_nodes, n / 16, 4, 16): actv with its columns regrouped slice by slice, element (s, k, c) = column
 * k n + 16 s + c of mg_painn_message's actv.  node_order as in mg_painn_message.  Same results as
 * mg_painn_table_message up to fp32 summation order. */
int mg_painn_edge_records(const float* r_ij /* (E,3) */, long n_edges, int table_rows, float period, float epsilon,
                          float* records /* (E,8) */, mg_stream_t stream);
int mg_painn_table_message_sliced(const int* row_ptr, const int* dst, const int* node_order, int n_nodes, long n_edges,
                                  const float* records, const float* table, int table_rows, const float* actv_sliced,
                                  const float* x_v, int n, const float* res_a, const float* res_v,
                                  float* out_a, float* out_v, mg_stream_t stream);
/* Message.forward after the two MLPs (archs/meanflow_painn8.py:91-100), fused over CSR rows:
 *   P = filt[e] * actv[dst[e]];  u = r_ij[e] / sqrt(epsilon + |r_ij[e]|^2);  v = x_v[dst[e]]
 *   out_v[i] = res_v[i] + sum_{e in row i} v*P[0:n] + (v x u)*P[n:2n] + u (x) P[2n:3n]
 *   out_a[i] = res_a[i] + sum_{e in row i} P[3n:4n]
 * filt (E,4n) is the radial MLP output per edge; actv (n_nodes,4n) is mlp_actv applied per
 * NODE (a row-wise function commutes with the gather); res_a/res_v may be NULL.
 * node_order (n_nodes ints, or NULL) is the order in which rows are processed (e.g. the cell order
 * of the neighbour search, for cache locality of the gathers); results do not depend on it. */
int mg_painn_message(const int* row_ptr /* n_nodes+1 */, const int* dst /* E */, const int* node_order,
                     int n_nodes, long n_edges,
                     const float* r_ij /* (E,3) */, const float* filt /* (E,4n) */,
                     const float* actv /* (n_nodes,4n) */, const float* x_v /* (n_nodes,n,3) */,
                     int n, float epsilon, const float* res_a, const float* res_v,
                     float* out_a /* (n_nodes,n) */, float* out_v /* (n_nodes,n,3) */, mg_stream_t stream);

/* Training side of the same message: its elementwise middle, between the per-edge MLP / the gathers and the sums over
 * edges (archs/meanflow_painn8.py:94-100), as one pass, and the adjoint of that pass.  dist, actv (E, 4n); v (E, n, 3)
 * the gathered vectors; dir (E, 3) = r_ij / sqrt(epsilon + |r_ij|^2):
 *   p = dist * actv;  m[e,c,:] = v[e,c,:] p[e,c] + (v[e,c,:] x dir[e]) p[e,n+c] + dir[e] p[e,2n+c];  a[e,c] = p[e,3n+c]
 * node (E ints) or NULL: with an index, actv is (n_rows, 4n) and v (n_rows, n, 3) and edge e reads row node[e] of both
 * (the gather by destination folded into the pass; an index outside 0..n_rows-1 is clamped); NULL: row e.
 * mg_painn_combine_bwd takes the gradients dm (E, n, 3), da (E, n), or with grad_row (E ints) dm (n_grad_rows, n, 3),
 * da (n_grad_rows, n) read at row grad_row[e] (m and a were summed over the edges of a source node: the gradient of an
 * edge is its node's), and writes those of the four inputs (any of the four output pointers may be NULL), all per edge
 * (d_actv (E, 4n), dv (E, n, 3): with an index the caller sums them over the edges of a row).  n: a power of two in
 * 4..256 (mg_painn_combine_supported); arrays contiguous and 16-byte aligned.  The reference evaluates these lines as
 * separate tensor operations.
 * terms: 15 for the message.  Bit k keeps the term that contains p[e, k n + c] (bits 0, 1: the terms with v; bits 1, 2:
 * those with dir).  sum (dm . m + da . a) is linear in dm / da, dist and actv, and in v and dir once restricted to
 * their terms, so a gradient of a gradient is the same pair of kernels with a cotangent in one argument's place and
 * that argument's mask: the operations are differentiable any number of times on these two kernels. */
int mg_painn_combine_supported(int n);   /* returns 0 / 1, not a status */
int mg_painn_combine_fwd(const float* dist, const float* actv, const float* v, const float* dir, const int* node,
                         long n_rows, long E, int n, int terms, float* m, float* a, mg_stream_t stream);
/* mg_painn_combine_fwd with the sums over the edges of a source node inside: the edge arrays are sorted by that node and
 * row_ptr (n_out_rows + 1) is their CSR; out_v (n_out_rows, n, 3) and out_a (n_out_rows, n) are the sums of m and a over
 * each row's edges, added in edge order (the same on every run).  Replaces mg_painn_combine_fwd followed by two
 * segment sums (torch_scatter.segment_coo at managan/graph_layers.py:54-59). */
int mg_painn_combine_fwd_rows(const float* dist, const float* actv, const float* v, const float* dir, const int* node,
                              long n_rows, const int* row_ptr, long n_out_rows, long E, int n, int terms, float* out_v,
                              float* out_a, mg_stream_t stream);
int mg_painn_combine_bwd(const float* dist, const float* actv, const float* v, const float* dir, const int* node,
                         long n_rows, const float* dm, const float* da, const int* grad_row, long n_grad_rows, long E,
                         int n, int terms, float* d_dist, float* d_actv, float* dv, float* d_dir, mg_stream_t stream);
/* mg_painn_combine_bwd with dist given by its grid: table (table_rows, 4n) is the filter at d = k period / table_rows
 * and edge e takes the 4-point Lagrange interpolation at len[e] (mg_painn_table_interp_fwd's arithmetic), so the
 * (E, 4n) filter is not stored between the forward and the backward pass (the forward pass being
 * mg_painn_table_message).  d_dist is still per edge, (E, 4n): mg_painn_table_interp_bwd sums it into the grid. */
int mg_painn_combine_bwd_grid(const float* table, int table_rows, float period, const float* len /* (E) */,
                              const float* actv, const float* v, const float* dir, const int* node, long n_rows,
                              const float* dm, const float* da, const int* grad_row, long n_grad_rows, long E, int n,
                              int terms, float* d_dist, float* d_actv, float* dv, float* d_dir, mg_stream_t stream);

/* The same gradients with those of actv and v summed inside the kernel, for actv (n_rows, 4n) and v (n_rows, n, 3) read
 * by every edge at one row (its destination): row r is read by the edges order[row_ptr[r]] .. order[row_ptr[r + 1] - 1]
 * (order NULL: by the edge positions themselves, edges sorted by that row), the caller's CSR of the index that
 * mg_painn_combine_bwd takes as `node`.  d_actv (n_rows, 4n) and dv (n_rows, n, 3) come out per row, summed in the
 * order of `order` (the same on every run); d_dist (E, 4n) and d_dir (E, 3) stay per edge; any of the four may be NULL.
 * The filter is dist (E, 4n), or (dist NULL) table (table_rows, 4n) interpolated at len[e] as in
 * mg_painn_combine_bwd_grid.  Replaces mg_painn_combine_bwd followed by two segment sums over (E, 4n) and (E, n, 3). */
int mg_painn_combine_bwd_rows(const float* dist, const float* table, int table_rows, float period, const float* len,
                              const float* actv, const float* v, const float* dir, const int* row_ptr, const int* order,
                              long n_rows, const float* dm, const float* da, const int* grad_row, long n_grad_rows,
                              long E, int n, int terms, float* d_dist, float* d_actv, float* dv, float* d_dir,
                              mg_stream_t stream);

/* The filter from its grid, for training (the grid itself: mg_painn_table_message above).  table (table_rows, cols):
 * the filter at d = k period / table_rows; table_rows and cols powers of two, cols <= 1024.
 *   mg_painn_table_interp_fwd:  out[e, :] = the 4-point Lagrange interpolation of the grid at d[e] (as the inference kernels do).
 *   mg_painn_table_buckets:     bucket[e] = the grid row floor(d[e] table_rows / period) mod table_rows.
 *   mg_painn_table_interp_bwd:  d_table = the adjoint of that interpolation applied to g (E, cols); perm (E ints) lists the
 *     edges in the order of a stable sort by bucket and bucket_ptr (table_rows + 1 ints) is the row pointer of the sorted
 *     buckets: the sums run in that order, in pieces added in a fixed order (same bits on every run; workspace from the
 *     _bytes call).  dd (E) or NULL: the gradient for the lengths, sum_c g[e, c] d out[e, c] / d d[e].
 * order (0 .. 3): the interpolant's order-th derivative with respect to d in place of the interpolant (its weights are
 * cubics in d): the derivatives of these operations are the same operations at other orders, which is what makes them
 * differentiable any number of times.
 * The reference evaluates the filter MLP on every edge (archs/meanflow_painn8.py:92); differentiating through the grid
 * moves the MLP's backward pass from E rows to table_rows rows. */
int mg_painn_table_interp_supported(int table_rows, int cols);   /* returns 0 / 1, not a status */
int mg_painn_table_interp_fwd(const float* table, int table_rows, int cols, float period, const float* d, long E,
                              int order, float* out, mg_stream_t stream);
int mg_painn_table_buckets(const float* d, long E, int table_rows, float period, int* bucket, mg_stream_t stream);
int mg_painn_table_interp_bwd_workspace_bytes(int table_rows, int cols, size_t* bytes /* host */);
int mg_painn_table_interp_bwd(const float* g, const float* table, int table_rows, int cols, float period, const float* d,
                              const int* perm, const int* bucket_ptr, long E, int order, void* workspace,
                              float* d_table, float* dd, mg_stream_t stream);

/* The edge filters of Messages for its training path (archs/diffuser_atoms15.py:240-243): from enc (E, chan) and
 * rh (E, 3), phi_v[e,c,i] = enc[e,c] rh[e,i] (E, chan, 3) and phi_d[e,c,i,j] = (enc[e,c] rh[e,j]) rh[e,i] (E, chan, 3, 3), and
 * the adjoint: d_enc (E, chan) and d_rh (E, 3) from the gradients g_v, g_d of the two (sums over channels in a fixed
 * order).  The reference writes them as broadcasting products. */
int mg_bee_edge_filters_fwd(const float* enc, const float* rh, long E, int chan, float* phi_v, float* phi_d,
                            mg_stream_t stream);
int mg_bee_edge_filters_bwd(const float* enc, const float* rh, const float* g_v, const float* g_d, long E, int chan,
                            float* d_enc, float* d_rh, mg_stream_t stream);

/* SiLU and its derivatives for the MLPs' training path (nn.SiLU in archs/meanflow_painn8.py:38-51, differentiated up
 * to three times by the meanflow loss, :274-296): out[k] = SiLU^(order)(z[k]) (* mul[k] if mul is not null), order 0..4,
 * n floats, 16-byte aligned.  The reference leaves these derivatives to autograd's elementwise formulas. */
int mg_silu_order(const float* z, const float* mul, long n, int order, float* out, mg_stream_t stream);

/* The first two layers of the radial MLP from the edge vectors (archs/meanflow_painn8.py:25-35 feeding :38-51):
 *   y[e] = SiLU(b2 + W2 SiLU(b1 + W1 radial_encode(r_ij[e], 16, rmax))),   y (E, hidden)
 * in one kernel; the first layer's output is produced chunk by chunk on the matrix cores and never stored.
 * 16 radial functions; hidden = 256 or 512.  W1 (hidden, 16) float32 with the given strides; packed_W2:
 * mg_linear_f16x2_pack_weight of W2 (hidden, hidden) with its INPUT channels permuted inside every group of 32:
 * position 16 g + p (g = 0, 1; p = 0..15) holds channel 8 (p / 4) + 4 g + p % 4.  h1_bound (1 float, device): an
 * upper bound of |SiLU(b1 + W1 enc)| (e.g. max_o sum_i |W1[o,i]| + max |b1|: the encodings are at most 1). */
int mg_painn_filter_hidden(const float* r_ij, long n_edges, float rmax, const float* W1, long w1_stride_o,
                           long w1_stride_i, const float* b1, const void* packed_W2, const float* b2, int hidden,
                           const float* h1_bound, float* y, mg_stream_t stream);

/* mg_painn_message with the LAST layer of the radial MLP folded in (archs/meanflow_painn8.py:38-51 at :92,
 * then :93-100): filt[e] = bias3 + W3 h[e] is produced on the matrix cores (split-fp16 arithmetic, as
 * mg_tensor_linear_f16x2) and consumed in the same kernel, so the (E,4n) filter is never stored.
 *   h (E,hidden): the MLP's second layer output (after its SiLU); h_rowmax: upper bounds of max_k |h[e,k]| as for
 *   mg_tensor_linear_f16x2 (h_rowmax_parts values per row, row stride h_rowmax_stride floats, 0 = one shared row).
 *   packed_W3: mg_linear_f16x2_pack_weight of W3 with its 4n rows PERMUTED to (c / 64, k, c % 64) for filter
 *   column k n + c (k = 0..3), i.e. packed row 256 (c / 64) + 64 k + c % 64; bias3 (4n) in the same order.
 *   src (E): the receiving node of every edge (sorted ascending; row_ptr is its CSR form).
 *   workspace: mg_painn_filter_message_workspace_bytes(n_edges, n) bytes, 16-byte aligned (partial sums).
 * n % 64 == 0, hidden % 32 == 0 and >= 64.  Sums run in edge order within blocks of 32 edges and then in
 * block order: deterministic, and equal to mg_painn_message up to fp32 summation order. */
int mg_painn_filter_message_workspace_bytes(long n_edges, int n, size_t* bytes);
int mg_painn_filter_message(const void* packed_W3, const float* bias3, const float* h, const float* h_rowmax,
                            int h_rowmax_parts, long h_rowmax_stride, int hidden, const int* row_ptr,
                            const int* src, const int* dst, const float* r_ij, const float* actv, const float* x_v,
                            long n_nodes, long n_edges, int n, float epsilon, const float* res_a,
                            const float* res_v, void* workspace, float* out_a, float* out_v, mg_stream_t stream);

/* mg_tensor_linear_f16x2_rowsum on bf16 storage: x (rows, dim_in) and the optional y (rows, dim_out) bfloat16,
 * packed_W as for mg_tensor_linear_bf16, out (n_out, dim_out) float32 = scale * sum over the rows of each segment
 * of the bfloat16-rounded act(bias + W x[r]) (the values y holds), accumulated in fp32.  dim_out % 128 == 0. */
int mg_tensor_linear_bf16_rowsum_workspace_bytes(long rows, int dim_out, size_t* bytes);
int mg_tensor_linear_bf16_rowsum(const void* packed_W, const void* x, long rows, int dim_in, int dim_out,
                                 const float* bias, int act, const int* row_ptr, const int* seg, long n_out, float scale,
                                 void* workspace, void* y, float* out, mg_stream_t stream);

/* The per-edge part of the scalar messages on bf16 storage (archs/diffuser_atoms15.py:98-110 MLP.forward applied
 * at :244-246 to psi_a = Y P0) reduced to the two sums over edges that the layers after the sum need:
 *   psi = Y x (rows, 128);  h1 = act(b1 + W1 psi) (rows, 256);  h2 = act(b2 + W2 h1) (rows, 256)
 *   sum_psi (n_out, 128) float32 = sum over the rows of each segment of bfloat16(psi)
 *   sum_h2  (n_out, 256) float32 = sum over the rows of each segment of bfloat16(h2)
 * with every intermediate rounded to bfloat16 exactly where mg_tensor_linear_bf16 rounds it when it stores, so
 * the result equals three mg_tensor_linear_bf16[_rowsum] calls up to fp32 summation order; no per-row tensor is
 * written.  x (rows, dim_in) bfloat16, dim_in % 32 == 0; packed_Y, packed_W1, packed_W2 as for
 * mg_tensor_linear_bf16, where the INPUT channels of W1 and W2 are permuted inside every group of 32 so that
 * position 16 g + p holds channel 8 (p / 4) + 4 g + p % 4 (g = 0, 1; p = 0..15).  seg, row_ptr as for
 * mg_tensor_linear_bf16_rowsum. */
int mg_mlp_chain_bf16_workspace_bytes(long rows, size_t* bytes);
int mg_mlp_chain_bf16(const void* x, long rows, int dim_in, const void* packed_Y, const void* packed_W1,
                      const float* b1, const void* packed_W2, const float* b2, int act, const int* row_ptr,
                      const int* seg, long n_out, void* workspace, float* sum_psi, float* sum_h2, mg_stream_t stream);

/* The three edge sums of DisplacementTensors.forward (archs/diffuser_atoms15.py:218-224) over CSR rows: with
 * u = s r / sqrt(1 + |s r|^2), s = scale (7 / r0 in the reference, tens_sigmoid of managan/tensor_products.py:167-182),
 *   out_a[i,c] = sum_e phi[e,c];  out_v[i,c,x] = sum_e phi[e,c] u_x;  out_d[i,c,x,y] = sum_e phi[e,c] u_x u_y
 * phi (E, chan) is the radial MLP's output per edge; the per-edge tensors phi (x) u, phi (x) u (x) u are never stored. */
int mg_displacement_sums(const int* row_ptr, long n_nodes, long n_edges, const float* r_ij, const float* phi, int chan,
                         float scale, float* out_a, float* out_v, float* out_d, mg_stream_t stream);

/* repel5_sim (extensions/polymer_sims_cuda/polymer_sims_kern.cu:145-164, bound as polymer_sim(SimId.REPEL5, ...) in
 * polymer_sims.cpp:17-47): Langevin dynamics of batch_size chains of n beads, x and v (batch_size, n, 3) float32
 * updated in place, drag (n).  Per call: half velocity update, max(nsteps, 1) position updates with full velocity
 * updates between them, half velocity update.  Forces: harmonic bonds (K 20, r0 0.8) to the chain neighbours and
 * 20 d / (|d|^2 + 0.2)^6 from every bead that is not a cyclic neighbour.  One workgroup per chain, n <= 2048; unlike
 * the reference's 256-thread blocks, every force is computed from the positions of one step.  The normals of bead
 * b = chain * n + i at velocity update first_kick + s are Box-Muller transforms of Philox4x32-10(counter (b,
 * first_kick + s, 0, 0), key seed): a call with first_kick advanced by max(nsteps, 1) + 1 continues the stream
 * (the reference reseeds XORWOW from the wall clock on every call). */
int mg_repel5_sim(float* x, float* v, const float* drag, float T, float dt, int nsteps, int batch_size, int n,
                  unsigned long long seed, unsigned int first_kick, mg_stream_t stream);

/* x (rows, dim, comps) in the reference's tensor layout (managan/tensor_products.py:17-24: channel, then the 3^k
 * components) -> xt (rows * comps, dim_pad): one plain GEMM row per (row, component) with the channels zero-padded
 * to dim_pad (a power of two, 32..256), and rowmax (rows * comps): max |xt| per output row.  What
 * mg_tensor_linear_f16x2 needs to apply a TensLinear to many rows with component-major output. */
int mg_components_to_rows(const float* x, long rows, int dim, int comps, int dim_pad, float* xt, float* rowmax,
                          mg_stream_t stream);

/* SelfTensProds.forward after its six input linears (archs/diffuser_atoms15.py:82-94), one output rank per call:
 *   y[node, o, comp] = sum over the product types `lab` of output rank rank_o, channels c of
 *                      Y[o, (lab, c)] * p_lab(l, r)[node, comp, c]
 * with the product types in the order 000 110 220 (rank 0), 011 101 121 211 111 (rank 1), 022 202 112 222 212
 * (rank 2) (managan/codegen_tensor_products.py:235-249), so Y = [Y_lab ...] concatenated along its input axis,
 * packed with mg_linear_f16x2_pack_weight (dim_out x n_types*chan).  The products are built in registers and
 * never stored.  l_k, r_k: component-major (nodes, 3^k, chan); node_bound (nodes): an upper bound of every
 * |product component| of the node (e.g. 9 max|l| max|r|; any bound within 2^14 of the largest keeps fp32
 * accuracy); y: (nodes, dim_out, 3^rank_o), the reference's layout.  chan % 32 == 0.
 * k_order 0: the columns of Y are ordered (type, channel) as above.  k_order 1 (rank_o == 2, dim_out <= 64):
 * (channel / 32, type, channel % 32); the kernel then stages the operands of 32 channels in LDS for all types. */
int mg_bee_products_linear(int rank_o, const float* l_0, const float* l_1, const float* l_2, const float* r_0,
                           const float* r_1, const float* r_2, const float* node_bound, long n_nodes, int chan,
                           const void* packed_W, int k_order, int dim_out, float* y, mg_stream_t stream);

/* A per-edge nn.Linear followed by the sum over the edges of each node, in one kernel: the pattern
 * `edges_reduce_src(graph, mlp(...))` of archs/diffuser_atoms15.py:244-246 (managan/graph_layers.py:54-59) for a
 * layer of the MLP whose output is only needed summed.
 *   out[s] = scale * sum_{rows r with seg[r] == s} act(bias + W x[r]),   out (n_out, dim_out)
 * x (rows, dim_in) with rows sorted by seg (ascending; row_ptr is the CSR form of seg, n_out + 1 entries);
 * packed_W / x_rowmax as for mg_tensor_linear_f16x2 (bounds per row, stride 0 = one shared row of parts);
 * y (rows, dim_out) also receives the per-row values when it is not NULL.  dim_out % 256 == 0, dim_in % 32 == 0
 * and >= 64.  workspace: mg_tensor_linear_f16x2_rowsum_workspace_bytes(rows, dim_out) bytes, 16-byte aligned.
 * Sums run in row order within blocks of 32 rows, then in block order (no atomics). */
int mg_tensor_linear_f16x2_rowsum_workspace_bytes(long rows, int dim_out, size_t* bytes);
int mg_tensor_linear_f16x2_rowsum(const void* packed_W, const float* x, const float* x_rowmax, int x_rowmax_parts,
                                  long x_rowmax_stride, long rows, int dim_in, int dim_out, const float* bias, int act,
                                  const int* row_ptr, const int* seg, long n_out, float scale, void* workspace,
                                  float* y, float* out, mg_stream_t stream);
/* The same with the bound of row r given as bound_mul * x_rowmax[r] + bound_add (see mg_tensor_linear_f16x2_scaled_bound). */
int mg_tensor_linear_f16x2_rowsum_scaled_bound(const void* packed_W, const float* x, const float* x_rowmax,
                                               int x_rowmax_parts, long x_rowmax_stride, long rows, int dim_in,
                                               int dim_out, const float* bias, int act, const int* row_ptr,
                                               const int* seg, long n_out, float scale, void* workspace, float* y,
                                               float* out, float bound_mul, float bound_add, mg_stream_t stream);

/* Update.forward (archs/meanflow_painn8.py:63-75), elementwise parts around its GEMMs.
 * lrv = [lin_l | lin_r | lin_v] applied to x_v (one stacked tensor_linear), stored (rows, 3n, 3) as the reference
 * stores tensors (lrv_comp_major = 0) or component-major (rows, 3, 3n) (lrv_comp_major = 1).
 *   pre:  ip[r,c] = sum_x l[c,x] r[c,x];  cat[r] = [x_a[r] | |r[c]|]  (rows, 2n), the MLP input
 *   vec:  v = lin_v(x_v) * y[:, 0:n];  out_v (rows, n, 3) = res_v + v / sqrt(1 + |v|^2)   (y: (rows, 3n) MLP output)
 * The scalar output is mg_group_norm(mode 1) of ip * y[:, n:2n] plus y[:, 2n:3n]. */
int mg_painn_update_pre(const float* lrv, int lrv_comp_major, const float* x_a, long rows, int n, float* ip, float* cat,
                        float* cat_rowmax /* (rows) max |cat[r,:]|, or NULL; n <= 256 */, mg_stream_t stream);
int mg_painn_update_vec(const float* lrv, int lrv_comp_major, const float* y, const float* res_v /* or NULL */, long rows, int n,
                        float* out_v, mg_stream_t stream);

/* ------------------------------------------------------------------------
 * Norms, squash, remaining radial encodings (node- or edge-sized streaming kernels).
 * ---------------------------------------------------------------------- */
/* Group norms over the nodes of a box and the channels of a group.
 *   mode 0  TensGroupNorm (managan/tensor_products.py:215-232):
 *           out = gamma[c] * v / sqrt(eps + mean_{nodes, group chans}(sum_comp v^2))
 *   mode 1  ScalGroupNorm (managan/layers_common.py:201-223), comps = 1:
 *           out = beta[c] + gamma[c] * (v - mean) / sqrt(eps + var)
 * v = x (* mul if mul != NULL); element (b, i, c, t) of x at x[((b*nodes + i)*x_stride + c)*comps + t]
 * (x_stride = channels per row of the underlying buffer, so a channel slice needs no copy), same for
 * mul / add with their strides; out (batch, nodes, chan, comps) dense; out += add, out += res when
 * given.  scratch: mg_group_norm_scratch_bytes bytes of device memory (fp64 partial sums, folded in
 * a fixed order: results are deterministic). */
int mg_group_norm_scratch_bytes(int batch, int groups, size_t* bytes /* host */);
int mg_group_norm(int mode, const float* x, long x_stride, const float* mul, long mul_stride,
                  int batch, int nodes, int chan, int groups, int comps, float eps,
                  const float* gamma, const float* beta, const float* add, long add_stride,
                  const float* res, void* scratch, float* out, mg_stream_t stream);
/* tens_sigmoid (managan/tensor_products.py:167-182): x / sqrt(1 + sum_comp x^2) per (row, chan). */
int mg_tens_sigmoid(int inds, const float* x, long rows_times_chan, float* out, mg_stream_t stream);
/* kind 1: sq_radial_encode(normed_sq_dist(r, rmax), n) (archs/diffuser_atoms14.py:32-48);
 * kind 2: radial_encode_edge(r, n, rmax) (archs/diffuser_atoms5.py:25-30).  out (E, n). */
int mg_radial_encode(int kind, const float* r_ij, long n_edges, int n, float rmax, float* out,
                     mg_stream_t stream);

/* ------------------------------------------------------------------------
 * Rank-0/1/2 message passing with the 13 products (archs/diffuser_atoms15.py:227-253).
 * ---------------------------------------------------------------------- */
/* Per-edge geometry of Messages.forward (archs/diffuser_atoms15.py:239-240):
 * enc (E,8) = radial_encode_8(r_ij, r0) (managan/jacobi_radenc.py:24-37), evaluated in fp64 and
 * rounded to fp32; rhat (E,3) = tens_sigmoid(1, r_ij * 7 / r0) (managan/tensor_products.py:167-182). */
int mg_bee_edge_geometry(const float* r_ij /* (E,3) */, long n_edges, float r0,
                         float* enc /* (E,8) */, float* rhat /* (E,3) */, mg_stream_t stream);
/* Messages.forward lines 241-247 and the edge sums of lines 250-252, fused over CSR rows.
 * phi_a[e,c] = enc_b[c] + sum_m enc_W[c,m] enc[e,m]; phi_v, phi_d as in the reference;
 * left operands La (N,chan), Lv (N,3,chan), Ld (N,9,chan) are L_k x_k in component-major layout.
 *   P0 (E,3,chan)    = [y_000 | y_110 | y_220] per edge
 *   S1 (N,3,5,chan)  = sum over the edges of each node of [y_011, y_101, y_121, y_211, y_111]
 *   S2 (N,9,5,chan)  = ... of [y_022, y_202, y_112, y_222, y_212]
 * node_order (N ints, or NULL) is the order in which rows are processed (e.g. cell order, for
 * cache locality of the gathers); results do not depend on it. */
int mg_bee_message(const int* row_ptr, const int* dst, const int* node_order, int n_nodes, long n_edges,
                   const float* rhat, const float* enc, const float* La, const float* Lv, const float* Ld,
                   int chan, const float* enc_W /* (chan,8) */, const float* enc_b /* (chan) */,
                   float* P0, float* S1, float* S2, float* node_max, float* edge_max, mg_stream_t stream);
/* mg_bee_message with the bias-free rank-2 output linear of Messages.forward (the Y_022 .. Y_212 of line 245,
 * which commute with the edge sum of line 252) applied inside the kernel: Y2 (dim_d, 5 chan) = the five Y_lab.W side
 * by side in the label order of S2, packed by mg_bee_pack_rank2_weight into mg_bee_rank2_weight_bytes(chan) bytes;
 * out_d (N, dim_d, 9) = Y2 S2 replaces S2, which is never stored.  For chan = 64, 128 or 256 and dim_d <= 16
 * (mg_bee_message_rank2_supported); the packing has no counterpart in the reference. */
int mg_bee_message_rank2_supported(int chan, int dim_d);
int mg_bee_rank2_weight_bytes(int chan, size_t* bytes);
int mg_bee_pack_rank2_weight(const float* Y2, long row_stride, int chan, int dim_d, float* packed, mg_stream_t stream);
int mg_bee_message_rank2(const int* row_ptr, const int* dst, const int* node_order, int n_nodes, long n_edges,
                         const float* rhat, const float* enc, const float* La, const float* Lv, const float* Ld,
                         int chan, const float* enc_W, const float* enc_b, const float* packed_Y2, int dim_d,
                         float* P0, float* S1, float* out_d, int accumulate /* out_d += Y2 S2 instead of = */,
                         float* node_max, float* edge_max, mg_stream_t stream);
/* The rank-2 part of SelfTensProds.forward (archs/diffuser_atoms15.py:82-94) in one pass over the nodes: the five
 * rank-2 products of l = L_k x_k and r = R_k x_k (component-major operands as for mg_bee_node_products) and their
 * output linears Y_022 .. Y_212, packed as for mg_bee_message_rank2; out_d (N, dim_d, 9).  Same domain.
 * P0 (N,3,chan), P1 (N,3,5,chan) (both or neither; may be NULL): the scalar and vector products as
 * mg_bee_node_products stores them, written in the same pass; node_max (N, chan/64; may be NULL): their partial
 * maxima per node.
 * x_d (N, dim_in2, 9) with L2t, R2t (dim_in2, chan) = the transposed weights of L2 and R2, dim_in2 <= 16 (or all
 * NULL / 0): l2 = L2 x_d and r2 = R2 x_d are formed inside the kernel and the arguments l2, r2 are not read. */
int mg_bee_node_products_rank2(long n_nodes, int chan, const float* l0, const float* l1, const float* l2,
                               const float* r0, const float* r1, const float* r2, const float* packed_Y2, int dim_d,
                               float* out_d, float* P0, float* P1, float* node_max, const float* x_d,
                               const float* L2t, const float* R2t, int dim_in2, mg_stream_t stream);
/* node_max (above and below; may be NULL): (N, ceil(chan/64)) partial maxima of |S1|, |S2| (of |P0|,
 * |P1|, |P2| below) per node, which mg_tensor_linear_f16x2 accepts as row bounds of those tensors
 * (x_rows_per_bound = 3 or 9); edge_max (may be NULL): (E, ceil(chan/64)) partial maxima of the rows
 * of P0; no counterpart in the reference. */

/* The 13 products of SelfTensProds.forward (archs/diffuser_atoms15.py:86-88; formulas of
 * managan/codegen_tensor_products.py:235-249) on node rows in component-major layout:
 * l0/r0 (N,chan), l1/r1 (N,3,chan), l2/r2 (N,9,chan) ->
 * P0 (N,3,chan) [000,110,220], P1 (N,3,5,chan) [011,101,121,211,111], P2 (N,9,5,chan)
 * [022,202,112,222,212]: the layout of S1/S2 above, so each rank's output linears are one GEMM. */
int mg_bee_node_products(long n_nodes, int chan, const float* l0, const float* l1, const float* l2,
                         const float* r0, const float* r1, const float* r2, float* P0, float* P1, float* P2,
                         float* node_max /* needs chan % 64 == 0 */, mg_stream_t stream);

/* ------------------------------------------------------------------------
 * bf16-storage configuration: feature tensors are bf16 in memory (void* below), every
 * sum and product is fp32.  Same math and layouts as the fp32 entry points of the same name.
 * ---------------------------------------------------------------------- */
/* y = act(bias + x W^T): x bf16 (rows, dim_in), dim_in % 32 == 0; W = the buffer written by
 * mg_linear_pack_weight (its hi and mid planes are used: 16 significand bits); y bf16
 * (y_is_bf16 != 0) or fp32; out_comps / accumulate / act as mg_tensor_linear_packed
 * (tensor_linear of extensions/tensor_ops/tensor_ops.cpp:31-93 on bf16 storage). */
int mg_tensor_linear_bf16(const void* packed_W, const void* x, long rows, int dim_in, int dim_out,
                          const float* bias, int act, int accumulate, int out_comps, int y_is_bf16, void* y,
                          mg_stream_t stream);
/* mg_bee_message with La, Lv, Ld, P0, S1, S2 stored as bf16 (enc, rhat, enc_W, enc_b fp32). */
int mg_bee_message_bf16(const int* row_ptr, const int* dst, const int* node_order, int n_nodes, long n_edges,
                        const float* rhat, const float* enc, const void* La, const void* Lv, const void* Ld,
                        int chan, const float* enc_W, const float* enc_b, void* P0, void* S1, void* S2,
                        mg_stream_t stream);
/* mg_bee_node_products on bf16 storage. */
int mg_bee_node_products_bf16(long n_nodes, int chan, const void* l0, const void* l1, const void* l2,
                              const void* r0, const void* r1, const void* r2, void* P0, void* P1, void* P2,
                              mg_stream_t stream);
/* out[r,:] = scale * sum_{e in row r} x_edge[e,:]  (segment_coo at managan/graph_layers.py:54-59 on bf16
 * storage, fp32 accumulation); feat % 4 == 0. */
int mg_segment_sum_csr_bf16(const void* x_edge /* (E,feat) bf16 */, const int* row_ptr, int n_rows, int feat,
                            float scale, void* out /* (n_rows,feat) bf16 */, mg_stream_t stream);

/* TensGroupNorm (managan/tensor_products.py:215-232) on bf16 storage, component-major: y, res (optional), out
 * (batch * nodes, comps, chan) bfloat16,
 *   out = gamma[c] * y / sqrt(eps + mean over (nodes, channels of the group) of sum_comps y^2) (+ res).
 * chan % 8 == 0, comps * chan <= 4608.  scratch: mg_tens_group_norm_bf16_scratch_bytes(batch, groups) bytes,
 * 8-byte aligned.  Statistics are summed in a fixed order. */
int mg_tens_group_norm_bf16_scratch_bytes(int batch, int groups, size_t* bytes);
int mg_tens_group_norm_bf16(const void* y, const void* res, int batch, int nodes, int comps, int chan, int groups, float eps,
                            const float* gamma, void* scratch, void* out, mg_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MANAGAN_HIP_H */
