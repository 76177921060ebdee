/*
 * e3x — C ABI of the MI355X-native equivariant message-passing hot path.
 *
 * Plain pointers and sizes only.  Every device pointer is caller-owned memory on the
 * current HIP device; the library allocates no device memory and frees nothing it did
 * not create.  All launches are asynchronous on the `stream` argument (a hipStream_t
 * passed as void*; NULL is the default stream).  Functions return 0 on success and a
 * negative E3X_ERR_* code otherwise; e3x_last_error() gives the message for the calling
 * thread.  Feature layout is the reference's: irreps concatenated in order, each block
 * row-major [mul, 2l+1] (reference e3nn/o3/_tensor_product/_codegen.py:82-94, :314).
 *
 * File:line citations name the reference function each entry point replaces
 * (paths relative to the e3nn source tree).
 */
#ifndef E3X_H
#define E3X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* the library is built with hidden visibility: only what this header declares is exported */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

#define E3X_OK 0
#define E3X_ERR_INVALID (-1)     /* bad argument / unsupported instruction set */
#define E3X_ERR_COMPILE (-2)     /* kernel specialisation could not be built */
#define E3X_ERR_HIP (-3)         /* a HIP runtime call failed */
#define E3X_ERR_INDEX (-4)       /* edge index out of range */

/* storage type of features / weights / outputs; accumulation is always fp32 */
#define E3X_F32 0
#define E3X_BF16 1

/* connection modes (reference _tensor_product.py:245-254) */
#define E3X_MODE_UVW 0
#define E3X_MODE_UVU 1
#define E3X_MODE_UVV 2
#define E3X_MODE_UUW 3
#define E3X_MODE_UUU 4
#define E3X_MODE_UVUV 5
#define E3X_MODE_UVU_LT_V 6 /* "uvu<v" */
#define E3X_MODE_U_LT_VW 7  /* "u<vw" */

/* spherical-harmonics output normalisation (reference _spherical_harmonics.py:103-110) */
#define E3X_NORM_INTEGRAL 0
#define E3X_NORM_COMPONENT 1
#define E3X_NORM_NORM 2

typedef struct {
  int32_t mul; /* multiplicity */
  int32_t l;   /* degree */
  int32_t p;   /* parity, +1 or -1 */
} e3x_irrep;

/* One row of TensorProduct.instructions (reference _tensor_product/_instruction.py:4-11)
 * after normalisation: path_weight is sqrt(alpha) of _tensor_product.py:289-324. */
typedef struct {
  int32_t i_in1, i_in2, i_out;
  int32_t mode;       /* E3X_MODE_* */
  int32_t has_weight; /* 0 / 1 */
  double path_weight;
} e3x_instruction;

typedef struct {
  int32_t n_in1, n_in2, n_out, n_ins;
  const e3x_irrep* in1;
  const e3x_irrep* in2;
  const e3x_irrep* out;
  const e3x_instruction* ins;
  int32_t shared_weights; /* 1: w is [weight_numel]; 0: w is [Z, weight_numel] */
  int32_t dtype;          /* E3X_F32 / E3X_BF16 storage of x1, x2, w, out */
} e3x_tp_desc;

/* activation functions of e3x_gate_* */
#define E3X_ACT_IDENTITY 0
#define E3X_ACT_SILU 1
#define E3X_ACT_TANH 2
#define E3X_ACT_SIGMOID 3
#define E3X_ACT_ABS 4
#define E3X_ACT_RELU 5

/* `count` scalar channels: out[offset_out + c] = cst * act(x[offset_in + c]) */
typedef struct {
  int32_t offset_in, offset_out, count, act;
  float cst;
} e3x_act_block;

/* `mul` copies of an irrep of dimension `dim`, copy u gated by scalar u of a run of `mul` gate scalars:
 * out[offset_out + u*dim + m] = cst * act(x[gate_offset_in + u]) * x[gated_offset_in + u*dim + m] */
typedef struct {
  int32_t gate_offset_in, gated_offset_in, offset_out, mul, dim, act;
  float cst;
} e3x_gate_block;

typedef struct e3x_plan e3x_plan;

const char* e3x_last_error(void);
int e3x_version(void);

/* Real-basis Wigner 3j tensor, out[(2l1+1)(2l2+1)(2l3+1)] row-major doubles, Frobenius
 * norm 1.  Host only.  Replaces o3.wigner_3j (e3nn/o3/_wigner.py:102-164). */
int e3x_wigner_3j(int l1, int l2, int l3, double* out);

/* Builds (or finds in the on-disk kernel cache) the fused kernel specialised to one
 * instruction set: the role of codegen_tensor_product_left_right
 * (e3nn/o3/_tensor_product/_codegen.py:24-395) behind the provider hook
 * _CODEGEN_PROVIDERS_LEFT_RIGHT (e3nn/o3/_tensor_product/_tensor_product.py:17-21,348-361).
 * Needs a HIP compiler only on a cache miss; needs no GPU (the code object is loaded on
 * first launch).  The cache directory is $E3X_KERNEL_CACHE or <library dir>/../kernel_cache. */
int e3x_tp_plan_create(const e3x_tp_desc* desc, e3x_plan** out);
int e3x_tp_plan_destroy(e3x_plan* plan);
/* weight_numel (reference _tensor_product.py:403), in1/in2/out dims, and the kernel family
 * name ("uvu", "uvw_small", "uvw_mfma", "uvw_node"); any out pointer may be NULL. */
int e3x_tp_plan_info(const e3x_plan* plan, int64_t* weight_numel, int64_t* in1_dim, int64_t* in2_dim,
                     int64_t* out_dim, const char** family, const char** cache_key);

/* Which instruction forms the products of the plan's kernels: "fp32 vector ALU", "fp32 matrix instruction",
 * "bf16 matrix instruction" (bf16 storage) or "bf16 matrix instruction, six products of three-way split operands"
 * (fp32 storage, fp32-accurate; see e3x_tp_forward).  which = 0: forward; which = 1: the "uvw" weight gradient on the
 * matrix cores, "" until that kernel has been built (e3x_tp_plan_prepare_backward_w).  No counterpart in the
 * reference; benchmarks use it to state the peak a kernel is measured against.  The string lives as long as the plan. */
const char* e3x_tp_plan_arithmetic(const e3x_plan* plan, int which);

/* out[Z, out_dim] = TP(x1[Z, in1_dim], x2[Z, in2_dim], w).  Replaces the generated
 * module called at e3nn/o3/_tensor_product/_tensor_product.py:554
 * (contraction: _codegen.py:148-187, path weights :312, sum/cat :327-343).
 * `out` is fully overwritten (output irreps no instruction reaches become 0).
 * fp32 plans of the "uvw_mfma" family whose blocks are all multiples of 64 wide form their products on the
 * bf16 matrix instruction from operands split into three bf16 pieces each (six cross products, fp32 accumulation):
 * the results have the accuracy of fp32 products and are reproducible, but negating an input changes last bits
 * (scaling by a power of two does not), and a row holding +-inf, or a finite value above 3.39e38 in magnitude (inf in
 * bf16), comes out NaN where the fp32 instruction gives +-inf: the split forms x - bf16(x).  Rows are independent.  E3X_UVW_SPLIT=0 in the environment at plan creation keeps the fp32
 * instruction; the "uvw" weight gradient (E3X_DW_SPLIT) and the dense layers of scalars do the same. */
int e3x_tp_forward(e3x_plan* plan, const void* x1, const void* x2, const void* w, void* out, int64_t Z,
                   void* stream);
/* The same with caller-owned device scratch.  Plans of the "uvw_mfma" family in bf16 storage repack the
 * weights for the matrix cores on every call and need e3x_tp_forward_workspace_bytes(plan) bytes (16-byte
 * aligned, as x1 and x2 must be); every other plan needs none and e3x_tp_forward is enough. */
size_t e3x_tp_forward_workspace_bytes(const e3x_plan* plan);
int e3x_tp_forward_ws(e3x_plan* plan, const void* x1, const void* x2, const void* w, void* out, int64_t Z,
                      void* workspace, size_t workspace_bytes, void* stream);

/* Destination-sorted edge list for the fused scatter: stable sort of edge ids by dst.
 * rowptr[num_nodes+1], perm[E] are int32 device arrays owned by the caller;
 * `workspace` is device scratch of at least e3x_csr_workspace_bytes(E, num_nodes).
 * Indices are int32 (idx_bits = 32) or int64 (idx_bits = 64) and must lie in
 * [0, num_nodes): scatter_add_ semantics (e3nn/nn/models/v2106/points_convolution.py:13-17).
 * Synchronises the stream once to report E3X_ERR_INDEX for out-of-range indices. */
size_t e3x_csr_workspace_bytes(int64_t E, int64_t num_nodes);
int e3x_csr_build(const void* dst, int idx_bits, int64_t E, int64_t num_nodes, int32_t* rowptr, int32_t* perm,
                  void* workspace, size_t workspace_bytes, void* stream);
/* e3x_csr_build for callers that cannot allocate device memory or hand over a workspace (tight serving loops that
 * rebuild the neighbour list every few steps, harnesses that forbid hipMalloc, set-up code that runs before a HIP
 * graph is captured).  Like e3x_csr_build it copies the range-check flag back and synchronises the stream before it
 * returns, so it must not be issued while the stream is capturing.  No counterpart in the reference.  The sort buffers live in a file-scope device array of
 * e3x_csr_static_scratch_bytes() = 64 MiB that every GPU the library runs on holds until the process ends; its
 * address is looked up once per device, on the first call there.  The call allocates and frees nothing.  Limit: the
 * buffers of e3x_csr_workspace_bytes(E, num_nodes) must fit the array (2 097 152 edges always do); larger edge lists
 * return E3X_ERR_INVALID.  All calls on one GPU share the array; the library makes the host threads of a process take
 * turns (a per-device lock held from the first launch to the final synchronisation), so only callers outside its
 * reach -- another process's library has an array of its own; the same array used through a stale pointer -- could
 * overlap.  Results are bit-identical to e3x_csr_build. */
size_t e3x_csr_static_scratch_bytes(void);
int e3x_csr_build_static(const void* dst, int idx_bits, int64_t E, int64_t num_nodes, int32_t* rowptr, int32_t* perm,
                         void* stream);
/* Checks gather indices the way torch advanced indexing does (x[edge_src],
 * points_convolution.py:105): values in [-num_nodes, num_nodes) are valid, negative
 * ones wrap.  Synchronises the stream. */
int e3x_index_check(const void* idx, int idx_bits, int64_t E, int64_t num_nodes, void* stream);

/* out[n, out_dim] = sum over edges e with dst[e] == n of TP(node_x[src[e]], edge_attr[e], w[e]),
 * i.e. scatter(tp(node_features[edge_src], edge_attr, weight), edge_dst, N) of
 * e3nn/nn/models/v2106/points_convolution.py:105-106, with neither [E, .] tensor
 * materialised.  rowptr / perm come from e3x_csr_build (perm may be NULL when the
 * edges are already grouped by destination in rowptr order).  Within a row, edges are
 * summed in perm order by a fixed reduction tree: results are bit-reproducible.
 * `out` is fully overwritten; rows without in-edges become 0.  Only for plans whose
 * instructions are all `uvu`. */
int e3x_tp_gather_scatter(e3x_plan* plan, const void* node_x, const void* edge_attr, const void* w,
                          const void* src, int idx_bits, const int32_t* rowptr, const int32_t* perm, void* out,
                          int64_t E, int64_t num_src_nodes, int64_t num_out_nodes, void* stream);

/* e3x_tp_gather_scatter with the per-edge weights computed inside the kernel by a two-layer radial network,
 *   w[e, :] = act(edge_scalars[e, :] @ W1 / sqrt(n_in variance_in)) * act_cst @ W2 / sqrt(n_hidden / variance_out),
 * i.e. weight = fc(edge_length_embedded) followed by the scatter of the tensor product
 * (e3nn/nn/models/v2106/points_convolution.py:99-106, network e3nn/nn/_fc.py:38-88 with hs = {n_in, n_hidden,
 * weight_numel}, out_act = False); the [E, weight_numel] weights are never stored.  w1 [n_in, n_hidden] and
 * w2 [n_hidden, weight_numel] are the reference's layer0.weight / layer1.weight, edge_scalars [E, n_in].
 * For fp32 all-uvu plans with per-edge weights on every instruction, multiplicity 32 on the first input and the
 * output and 1 on the second, n_hidden a multiple of 16 (E3X_ERR_INVALID otherwise: run the network and
 * e3x_tp_gather_scatter instead).  `out` is fully overwritten.  Every row is summed in the order of the sorted
 * edge list by one worker of the kernel: results are bit-reproducible.  The kernel is built on first use (one per
 * network shape). */
int e3x_tp_gather_scatter_radial(e3x_plan* plan, const void* node_x, const void* edge_attr, const void* edge_scalars,
                                 const void* w1, const void* w2, int32_t n_in, int32_t n_hidden, int32_t act,
                                 double act_cst, double variance_in, double variance_out, const void* src, int idx_bits,
                                 const int32_t* rowptr, const int32_t* perm, void* out, int64_t E,
                                 int64_t num_src_nodes, int64_t num_out_nodes, void* stream);

/* Builds the kernel of e3x_tp_gather_scatter_radial for one network description ahead of the first call (no GPU
 * needed); E3X_ERR_INVALID when the plan or the network is outside what the kernel takes. */
int e3x_tp_plan_prepare_radial(e3x_plan* plan, int32_t n_in, int32_t n_hidden, int32_t act, double act_cst,
                               double variance_in, double variance_out);

/* Processing order of the output rows for e3x_tp_gather_scatter_ordered: row_order[num_nodes] (int32 device array owned
 * by the caller) is the permutation of the rows sorted, stably, by the smallest source row among their in-edges (with
 * num_src_nodes == num_nodes, one node set, the sort key is (k3, k2, k1): k1 the smallest source of the row, k2 = k1 of
 * node k1, k3 = k1 of node k2).  Rows
 * that share their smallest source share most of their sources (a one-permutation min-hash of the neighbour sets), so
 * rows processed next to each other gather the same rows of the node table and find them in L2, whatever the
 * caller's node numbering; the results are bit-identical to the unordered call.  No counterpart in the reference
 * (torch scatter_add_ has no processing order to choose).  rowptr / perm as built by e3x_csr_build; `workspace` is
 * device scratch of at least e3x_row_order_workspace_bytes(num_nodes).  With a non-NULL `shared_pairs` (a HOST int)
 * the call also counts the rows that agree with their successor in the order in their TWO smallest sources and
 * synchronises the stream to return it: on a graph without neighbourhood structure (uniformly random edges) the
 * count is a vanishing fraction of the rows, the order is a random permutation of them and is better not used. */
size_t e3x_row_order_workspace_bytes(int64_t num_nodes);
int e3x_row_order_build(const void* src, int idx_bits, const int32_t* rowptr, const int32_t* perm, int64_t E,
                        int64_t num_nodes, int64_t num_src_nodes, int32_t* row_order, int32_t* shared_pairs,
                        void* workspace, size_t workspace_bytes, void* stream);
/* e3x_tp_gather_scatter with the output rows walked in `row_order` (NULL: in row order). */
int e3x_tp_gather_scatter_ordered(e3x_plan* plan, const void* node_x, const void* edge_attr, const void* w,
                                  const void* src, int idx_bits, const int32_t* rowptr, const int32_t* perm,
                                  const int32_t* row_order, void* out, int64_t E, int64_t num_src_nodes,
                                  int64_t num_out_nodes, void* stream);

/* e3x_tp_gather_scatter_ordered with caller-owned device scratch.  Plans in bf16 storage whose instruction set fits
 * the matrix-core message kernel (per-edge weights on every instruction, multiplicity 128 on the first input and
 * the output, 1 on the second, at most 16 components per multiplicity index, one instruction per output irrep:
 * what the reference's convolution builds, e3nn/nn/models/v2106/points_convolution.py:60-76) take that kernel
 * when given e3x_tp_gather_scatter_workspace_bytes(plan, num_src_nodes) bytes (16-byte aligned; the call writes a
 * copy of the node table in matrix-operand order there); the Clebsch-Gordan contraction then runs in bf16 on the
 * matrix cores with fp32 accumulation (the per-edge matrices are rounded to bf16 once more than in the other
 * kernels).  Every other plan needs no workspace (the function returns 0) and runs as e3x_tp_gather_scatter_ordered;
 * so does a call without workspace. */
size_t e3x_tp_gather_scatter_workspace_bytes(const e3x_plan* plan, int64_t num_src_nodes);
/* `src_rows` (may be NULL): the source rows in the order of the destination-sorted list, as e3x_src_rows_build writes
 * them; the kernels then read it in place of `src` (which is still required).  Results are bit-identical. */
int e3x_tp_gather_scatter_ws(e3x_plan* plan, const void* node_x, const void* edge_attr, const void* w, const void* src,
                             int idx_bits, const int32_t* rowptr, const int32_t* perm, const int32_t* row_order,
                             const int32_t* src_rows, void* out, int64_t E, int64_t num_src_nodes,
                             int64_t num_out_nodes, void* workspace, size_t workspace_bytes, void* stream);
/* src_rows[k] = src[perm[k]] (perm NULL: src[k]) as int32, negative values wrapped by num_src_nodes: the gather
 * indices of x[edge_src] (points_convolution.py:105) laid out in the order the fused kernels walk the edges.  Read
 * through `perm`, an index costs the kernels a cache line of its own per edge; this list is read sequentially.  It
 * depends on the graph only (built once per edge list, E * 4 bytes, caller-owned).  Indices must have been
 * validated (e3x_index_check). */
int e3x_src_rows_build(const void* src, int idx_bits, const int32_t* perm, int64_t E, int64_t num_src_nodes,
                       int32_t* src_rows, void* stream);

/* e3x_tp_gather_scatter_ws for plans whose second input is the spherical harmonics of the edge vectors,
 * irreps_in2 = 0e + 1o + ... up to lmax <= 3 with multiplicity 1 (what the reference's convolutions feed it:
 * edge_attr = o3.spherical_harmonics(range(lmax + 1), edge_vec, normalize, normalization), e.g.
 * e3nn/nn/models/gate_points_2101.py:329): the kernel reads edge_vec[E, 3] (always fp32, 12 bytes per edge) and
 * forms the harmonics itself, with the arithmetic of e3x_sh_forward (e3nn/o3/_spherical_harmonics.py:93-112,
 * :194-226), instead of reading a stored [E, (lmax + 1)^2] tensor.  Equal to e3x_sh_forward followed by
 * e3x_tp_gather_scatter_ws up to the rounding of the fused multiply-adds.  `normalize` / `normalization`
 * (E3X_NORM_*) as in e3x_sh_forward.  A code object of its own per (normalize, normalization), built on first use or
 * ahead of time (no GPU needed) by e3x_tp_plan_prepare_gather_scatter_sh, which returns E3X_ERR_INVALID for plans
 * this does not apply to (not all-uvu, shared weights, another second input).  Vector-ALU kernels in either
 * storage type; no workspace. */
int e3x_tp_plan_prepare_gather_scatter_sh(e3x_plan* plan, int32_t normalize, int32_t normalization);
int e3x_tp_gather_scatter_sh(e3x_plan* plan, const void* node_x, const float* edge_vec, const void* w, const void* src,
                             int idx_bits, const int32_t* rowptr, const int32_t* perm, const int32_t* row_order,
                             const int32_t* src_rows, void* out, int64_t E, int64_t num_src_nodes,
                             int64_t num_out_nodes, int32_t normalize, int32_t normalization, void* stream);

/* Gradients of the `uvu` product (plain: src = dst = NULL, row e of every table; fused: the edge lists
 * of e3x_tp_gather_scatter, unsorted) with respect to the per-sample weights and the second input:
 *   grad_w[E, weight_numel] (shared weights: one [weight_numel] vector summed over the edges with fp32 atomics),
 *   grad_x2[E, in2_dim]  from  grad_out[num_out_nodes, out_dim].
 * Either output may be NULL.  The reference obtains these by autograd through the einsums of
 * e3nn/o3/_tensor_product/_codegen.py:166-187.  The gradient with respect to the first input is the
 * forward entry point applied to a transposed plan (inputs grad_out and x2, output irreps_in1, same
 * weights) with source and destination exchanged; no separate entry point is needed for it.
 * Only for all-`uvu` plans; bf16 storage only for per-sample weights and plans of a single kernel.
 * x2 may be NULL when grad_w is (only the weight gradient reads it), per-sample w when grad_x2 is. */
int e3x_tp_backward_w_x2(e3x_plan* plan, const void* x1, const void* x2, const void* w, const void* grad_out,
                         const void* src, const void* dst, int idx_bits, void* grad_w, void* grad_x2, int64_t E,
                         int64_t num_src_nodes, int64_t num_out_nodes, void* stream);

/* The backward pass of a message step in ONE kernel, called on the TRANSPOSED plan (first input: the messages'
 * irreps, output: the node features' irreps, same second input and weights) with source and destination exchanged:
 *   out[n]    = sum over the edges e leaving node n of  plan(table[gather_idx[e]], edge_attr[e], w[e])   (= d/dnode_x)
 *   grad_w[e] = the gradient of the per-edge weights, which needs the forward input row of the source node:
 *               row_x[num_out_rows, out_dim] (the node features the forward pass gathered from)
 * from table = grad_out[num_table_rows, in1_dim] of the forward call.  rowptr / perm (/ row_order) group the edges
 * by SOURCE node (e3x_csr_build on edge_src); gather_idx = edge_dst, src_rows (may be NULL) = e3x_src_rows_build of
 * it.  One pass over the weights and one gather of the
 * output gradient per edge, where e3x_tp_gather_scatter on this plan followed by e3x_tp_backward_w_x2 on the forward
 * plan makes two of each; out agrees with e3x_tp_gather_scatter_ordered to rounding (the same sums per lane group; the groups of a
 * wavefront are combined by a shuffle butterfly, there sometimes through LDS in another order).  grad_x2[E, in2_dim]
 * (may be NULL: not computed) is the gradient of edge_attr, summed over the multiplicity indices inside the kernel.
 * The reference obtains all of this by autograd through points_convolution.py:105-106 and the einsums of
 * e3nn/o3/_tensor_product/_codegen.py:166-187.  fp32, per-edge weights, multiplicities that one lane group of a
 * wavefront covers (instruction sets that run as several kernels over disjoint output irreps launch as many here)
 * (e3x_tp_plan_prepare_gather_scatter_grad_w builds the code objects and returns E3X_ERR_INVALID, without a message,
 * for plans that do not fit); grad_w[E, weight_numel] 16-byte aligned. */
int e3x_tp_plan_prepare_gather_scatter_grad_w(e3x_plan* plan);
int e3x_tp_gather_scatter_grad_w(e3x_plan* plan, const void* table, const void* edge_attr, const void* w,
                                 const void* row_x, const void* gather_idx, int idx_bits, const int32_t* rowptr,
                                 const int32_t* perm, const int32_t* row_order, const int32_t* src_rows, void* out,
                                 void* grad_w, void* grad_x2, int64_t E, int64_t num_table_rows, int64_t num_out_rows,
                                 void* stream);

/* Weight gradient of the `uvw` product: grad_w[weight_numel] (shared weights, summed over the batch with
 * fp32 atomics, so the last bits depend on the order) or grad_w[Z, weight_numel] (per-sample weights), from
 * x1[Z, in1_dim], x2[Z, in2_dim], grad_out[Z, out_dim].  The reference obtains it by autograd through
 * einsum("uvw,ijk,zuvij->zwk") (e3nn/o3/_tensor_product/_codegen.py:148-165).  fp32 storage only.  Plans
 * of the "uvw_mfma" family need x1, x2 and grad_out 16-byte aligned and build a second code object on first
 * use; e3x_tp_plan_prepare_backward_w builds it ahead of time (no GPU needed), so that a later call finds
 * it in the kernel cache. */
int e3x_tp_plan_prepare_backward_w(e3x_plan* plan);
int e3x_tp_backward_w_uvw(e3x_plan* plan, const void* x1, const void* x2, const void* grad_out, void* grad_w,
                          int64_t Z, void* stream);

/* out[n, sum(2l+1 for l in ls)] = spherical harmonics of xyz[n, 3].  Replaces
 * SphericalHarmonics.forward (e3nn/o3/_spherical_harmonics.py:93-112) and the polynomial
 * chain _spherical_harmonics (:193-249 for l <= 3, recurrence of
 * _spherical_harmonics_generator.py:57-65 above).  max(ls) <= 12. */
int e3x_sh_forward(const int32_t* ls, int32_t n_ls, int32_t normalize, int32_t normalization, const void* xyz,
                   void* out, int64_t n, int32_t dtype, void* stream);

/* grad_xyz[n, 3] from grad_out[n, sum(2 l + 1)] for the same l list: the backward pass of e3x_sh_forward (the
 * reference differentiates the polynomial chain of e3nn/o3/_spherical_harmonics.py:93-112,193-249 by autograd).
 * ls = 0..lmax with lmax <= 3 runs on closed forms, any other list (l <= 12) on the reverse sweep of the
 * recurrence. */
int e3x_sh_backward(const int32_t* ls, int32_t n_ls, int32_t normalize, int32_t normalization, const void* xyz,
                    const void* grad_out, void* grad_xyz, int64_t n, int32_t dtype, void* stream);

/* The derivative of e3x_sh_backward, for training on quantities that are themselves gradients (forces): with
 * phi(x) = <grad_out, Y(x)>, whose gradient e3x_sh_backward returns, and a cotangent cot_xyz[n, 3] on that gradient,
 *   grad_grad_out[n, n_out] = d<cot, grad phi>/d grad_out = the directional derivative of Y along cot,
 *   grad_xyz[n, 3]          = d<cot, grad phi>/d xyz      = the Hessian of phi applied to cot
 * (the normalisation of the vectors is part of the differentiated function).  The reference obtains both by
 * differentiating its polynomial chain twice (e3nn/o3/_spherical_harmonics.py:193-249).  Implemented for the l lists
 * 0 .. lmax <= 3 (the closed forms); E3X_ERR_INVALID for any other list. */
int e3x_sh_backward2(const int32_t* ls, int32_t n_ls, int32_t normalize, int32_t normalization, const void* xyz,
                     const void* grad_out, const void* cot_xyz, void* grad_grad_out, void* grad_xyz, int64_t n,
                     int32_t dtype, void* stream);

/* Gated non-linearity on rows x[Z, in_dim] -> out[Z, out_dim] (stored as fp32 or bf16, `dtype`; fp32 arithmetic), at
 * most 16 blocks of each kind; columns of `out`
 * that no block covers become 0.  Replaces nn.Gate.forward (e3nn/nn/_gate.py:121-144: Extract, Activation,
 * ElementwiseTensorProduct, cat) and, with n_gates = 0, nn.Activation.forward (e3nn/nn/_activation.py:78-104);
 * `cst` is the second-moment normalisation of e3nn/math/_normalize_activation.py:22-57.  e3x_gate_backward writes
 * grad_x[Z, in_dim] from grad_out[Z, out_dim] (the reference differentiates the same graph by autograd). */
int e3x_gate_forward(const e3x_act_block* acts, int32_t n_acts, const e3x_gate_block* gates, int32_t n_gates, const void* x,
                     void* out, int64_t Z, int64_t in_dim, int64_t out_dim, int32_t dtype, void* stream);
int e3x_gate_backward(const e3x_act_block* acts, int32_t n_acts, const e3x_gate_block* gates, int32_t n_gates, const void* x,
                      const void* grad_out, void* grad_x, int64_t Z, int64_t in_dim, int64_t out_dim, int32_t dtype,
                      void* stream);
/* The derivative of e3x_gate_backward: for a cotangent cot_x[Z, in_dim] on its result,
 * grad_grad_out[Z, out_dim] = d<cot_x, grad_x>/d grad_out and grad_x[Z, in_dim] = d<cot_x, grad_x>/dx (second
 * derivatives of the activations; 0 for abs and relu away from 0).  The reference differentiates
 * e3nn/nn/_gate.py:121-144 and e3nn/nn/_activation.py:78-104 twice by autograd. */
int e3x_gate_backward2(const e3x_act_block* acts, int32_t n_acts, const e3x_gate_block* gates, int32_t n_gates,
                       const void* x, const void* grad_out, const void* cot_x, void* grad_grad_out, void* grad_x,
                       int64_t Z, int64_t in_dim, int64_t out_dim, int32_t dtype, void* stream);

/* Fully-connected network of scalars hs[0] -> hs[1] -> ... -> hs[n_hs-1] in ONE kernel (fp32, matrix cores):
 *   layer l:  x <- act(x @ W_l / sqrt(hs[l] var_in)) * act_cst * sqrt(var_out)      (with activation)
 *             x <- x @ W_l / sqrt(hs[l] var_in / var_out)                           (without)
 * Replaces nn.FullyConnectedNet.forward (e3nn/nn/_fc.py:38-48 for a layer, :70-88 for which layers carry the
 * activation and which variances: every layer but the last has the activation and var_out = 1, the last has
 * var_out = variance_out and the activation only with out_act != 0).  `act` is an E3X_ACT_* code
 * (E3X_ACT_IDENTITY for the reference's act=None) and `act_cst` its second-moment normalisation
 * (e3nn/math/_normalize_activation.py:22-57).  The hidden activations never leave the registers.
 * Limits (E3X_ERR_INVALID beyond them): 1..8 layers; with widths rounded up to 32 (hs[0] to 8), the input of the last
 * layer <= 384, the input plus the output of every other layer <= 384, and all weights together <= 150 KB.
 * e3x_fc_forward: x[Z, hs[0]] -> out[Z, hs[n_hs-1]]; `weights` is a HOST array of n_hs-1 device pointers,
 * weights[l] = W_l[hs[l], hs[l+1]] row-major (the reference's `layer{l}.weight`); `workspace` is device memory of
 * e3x_fc_workspace_bytes(plan) bytes, 16-byte aligned like x, that the call overwrites. */
typedef struct e3x_fc_plan e3x_fc_plan;
int e3x_fc_plan_create(const int32_t* hs, int32_t n_hs, int32_t act, double act_cst, int32_t out_act, double variance_in,
                       double variance_out, int32_t dtype, e3x_fc_plan** out);
/* The same network with an activation fused at either end, for the layer-by-layer path under autograd (one-layer
 * plans): input_act != E3X_ACT_IDENTITY: the rows given are pre-activations and the network starts from
 * input_cst * act(x) -- also in e3x_fc_backward_w -- so the activated tensor is never stored; epilogue_act: the
 * outputs are multiplied by epilogue_cst * act'(z), z[Z, hs[n_hs-1]] given at launch: with hs = {h_out, h_in} and the
 * transposed weights this is the input gradient of a dense layer taken through the normalised activation in front of
 * it (autograd of e3nn/nn/_fc.py:38-48 over two layers) in one kernel.  e3x_fc_forward on a plan with an epilogue
 * is an error; e3x_fc_forward_epilogue on a plan without one ignores z. */
int e3x_fc_plan_create_fused(const int32_t* hs, int32_t n_hs, int32_t act, double act_cst, int32_t out_act,
                             double variance_in, double variance_out, int32_t dtype, int32_t input_act, double input_cst,
                             int32_t epilogue_act, double epilogue_cst, e3x_fc_plan** out);
int e3x_fc_forward_epilogue(e3x_fc_plan* plan, const void* x, const void* const* weights, const void* z, void* out,
                            int64_t Z, void* workspace, size_t workspace_bytes, void* stream);
int e3x_fc_plan_destroy(e3x_fc_plan* plan);
size_t e3x_fc_workspace_bytes(const e3x_fc_plan* plan);
/* name of the plan's code object in the kernel cache */
const char* e3x_fc_plan_key(const e3x_fc_plan* plan);
int e3x_fc_forward(e3x_fc_plan* plan, const void* x, const void* const* weights, void* out, int64_t Z, void* workspace,
                   size_t workspace_bytes, void* stream);
/* One-layer plans (n_hs = 2, no activation) only: grad_w[hs[0], hs[1]] = s * x^T grad_out with the layer's factor
 * s = 1 / sqrt(hs[0] variance_in / variance_out), i.e. the gradient autograd derives for `weight` from
 * `x @ (weight * s)` (e3nn/nn/_fc.py:38-48).  Batch slices are added with fp32 atomics (last-bit run-to-run
 * variation); grad_w is fully overwritten.  hs[0] <= 256.  e3x_fc_plan_prepare_backward_w builds the kernel ahead of
 * the first call (no GPU needed). */
int e3x_fc_plan_prepare_backward_w(e3x_fc_plan* plan);
int e3x_fc_backward_w(e3x_fc_plan* plan, const void* x, const void* grad_out, void* grad_w, int64_t Z, void* stream);

/* Plain device copy dst[i] = src[i], n_bytes multiple of 16: the calibration kernel
 * for bandwidth counters (known traffic: n_bytes read + n_bytes written). */
int e3x_copy_bytes(const void* src, void* dst, size_t n_bytes, void* stream);
/* The memory traffic of a fused message kernel without its arithmetic and without its gather: one wavefront per row
 * reads in_bytes_per_row consecutive bytes (row r at in + r * in_bytes_per_row, non-temporal 16-byte loads) and
 * writes out_bytes_per_row bytes (row r at out + r * out_bytes_per_row; 0: nothing is written).  Sizes are multiples
 * of 16.  No counterpart in the reference: a calibration kernel like e3x_copy_bytes, for the rate this chip sustains
 * on a read stream that carries a few per cent of row-sized writes (it is well below the rate of the read stream
 * alone), against which the message kernels are to be read. */
int e3x_stream_rows(const void* in, size_t in_bytes_per_row, int64_t n_rows, void* out, size_t out_bytes_per_row,
                    void* stream);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* E3X_H */
