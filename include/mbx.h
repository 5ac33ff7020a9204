/*
 * mbx.h — C ABI of libmbx.so: the dropless-MoE hot path for AMD MI355X (gfx950).
 *
 * Every entry point takes raw device pointers, explicit sizes and a HIP stream, enqueues
 * its kernels on that stream and returns without synchronising.  Nothing here allocates
 * device memory: outputs and scratch are caller-provided (the *_scratch_bytes functions
 * say how much).  Return value: 0 on success, a positive hipError_t if the HIP runtime
 * reported one, or a negative MBX_E* code for a rejected argument.
 *
 * All index tensors of the permutation ops (indices, bin_ids, bins, padded_bins) are
 * int32.  "bins" are inclusive cumulative sums: expert e owns sorted slots
 * [bins[e-1], bins[e]) with bins[-1] := 0.
 *
 * Each declaration names the interface of databricks/megablocks it stands in for.
 */
#ifndef MBX_H_
#define MBX_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* mbx_stream_t; /* a hipStream_t; NULL = the default stream */

enum mbx_itype { MBX_I16 = 0, MBX_I32 = 1, MBX_I64 = 2 };
enum mbx_dtype { MBX_BF16 = 0, MBX_F16 = 1, MBX_F32 = 2 };
enum mbx_layout { MBX_NN = 0, MBX_NT = 1, MBX_TN = 2 };
enum mbx_activation { MBX_ACT_SILU = 0, MBX_ACT_GELU_TANH = 1 };

#define MBX_EINVAL (-1)   /* bad enum / negative size / null pointer */
#define MBX_ESCRATCH (-2) /* scratch buffer too small */
#define MBX_ERANGE (-3)   /* size beyond what the kernels index with 32 bits */
#define MBX_EUNSUPPORTED (-4) /* this entry point does not handle the shape / type; use the general form */
#define MBX_ECAPTURE (-5) /* the call needs a one-time set-up that cannot run under stream capture: mbx_init() first */

/* Human-readable text for a return code (static storage). */
const char* mbx_error_string(int code);
/* ABI version of the loaded library. */
int mbx_version(void);
/* One-time set-up for the current device (hipSetDevice first), outside stream capture: looks up the addresses of the
 * device memory that is part of the library image (the buffer of mbx_scatter_static).  Optional -- the entry points
 * that need it do it on their first call on a device -- except ahead of a first call under stream capture, which
 * returns MBX_ECAPTURE instead.  Idempotent, thread-safe.  No counterpart in the reference. */
int mbx_init(void);

/* ------------------------------------------------------------------ routing ops */

/* csrc/histogram.h:61-81 `histogram(x, num_bins)`: out[r, b] = #{c : x[r, c] == b},
 * b in [0, num_bins); values outside the range are counted nowhere.  x is
 * [rows, n] of `itype`, out is int32 [rows, num_bins].  All rows in one call. */
int mbx_histogram(const void* x, int itype, int64_t rows, int64_t n, int num_bins,
                  int32_t* out, mbx_stream_t stream);

/* csrc/sort.h:59-86 `sort(x, end_bit, x_out, iota_out)`: stable LSD radix sort of n keys
 * on bits [0, end_bit); the payload is 0..n-1 in the key type.  keys_out[i] =
 * x[perm_out[i]].  With end_bit equal to the key width the order is the signed order. */
size_t mbx_sort_scratch_bytes(int64_t n, int itype, int end_bit);
int mbx_sort(const void* x, int itype, int64_t n, int end_bit, void* keys_out,
             void* perm_out, void* scratch, size_t scratch_bytes, mbx_stream_t stream);

/* The routing bookkeeping of one layer step, megablocks/layers/moe.py:152-183 (`indices_and_bins`) and
 * megablocks/layers/dmoe.py:131-154 (`indices_and_padded_bins`), in three launches instead of the seven of
 * sort + histogram + the cumsums + mbx_slot_rows.  For int32 expert ids [n] in [0, num_experts):
 *   bin_ids, indices      = sort(expert_ids, end_bit)                      (csrc/sort.h:59)
 *   tokens_per_expert     = histogram(expert_ids, num_experts)             (csrc/histogram.h:61)
 *   bins                  = inclusive_cumsum(tokens_per_expert)            (csrc/cumsum.h:131)
 *   padded_bins           = inclusive_cumsum(round_up(tokens_per_expert, pad))   if pad > 0 (else not written; may be NULL)
 *   slot_rows (or NULL)   = what mbx_slot_rows builds from these (with padded_bins if pad > 0)
 * bit for bit what the separate entry points give.  An id outside [0, num_experts) is a caller's error here; it is
 * taken by its low end_bit bits throughout (the order, the counts and the row map agree): one more row of the expert
 * those bits name, or, if they name none, sorted behind the last bin with row -1 -- where mbx_histogram would drop it
 * and leave the bins short of the sorted order.  No row inside a bin is left without a slot or padding.
 * scratch: mbx_sort_scratch_bytes(n, MBX_I32, end_bit) bytes.  MBX_EUNSUPPORTED (use the separate entry points):
 * end_bit above 8 or num_experts above 2^end_bit. */
int mbx_route(const int32_t* expert_ids, int64_t n, int num_experts, int end_bit, int pad, int32_t* indices,
              int32_t* bin_ids, int32_t* tokens_per_expert, int32_t* bins, int32_t* padded_bins,
              int32_t* slot_rows, void* scratch, size_t scratch_bytes, mbx_stream_t stream);

/* csrc/cumsum.h:104-156 `inclusive_cumsum / exclusive_cumsum(x, dim=1, out)`: scan of
 * every row of x [rows, n]. */
int mbx_cumsum(const void* x, int itype, int64_t rows, int64_t n, int exclusive, void* out,
               mbx_stream_t stream);

/* csrc/indices.h:69-93 `indices(padded_bins, block_size, block_rows, block_cols, out)`:
 * column indices (int16) of the block-diagonal topology; block-rows past the last bin
 * are written as 0. */
int mbx_topology(const int32_t* padded_bins, int num_bins, int block_size, int block_rows,
                 int block_cols, int16_t* out, mbx_stream_t stream);

/* csrc/replicate.h:130-183 `replicate_forward(x, bins, out)`: out[b, bins[i-1]:bins[i]] =
 * x[b, i]; columns at or past bins[-1] are written as 0.  elem_bytes is 2 or 4. */
int mbx_replicate_forward(const void* x, int elem_bytes, int64_t batch, int num_bins,
                          const int32_t* bins, void* out, int64_t columns, mbx_stream_t stream);

/* csrc/replicate.h:185-206 `replicate_backward(grad, bins, out)`: out[b, i] =
 * sum(grad[b, bins[i-1]:bins[i]]) with fp32 accumulation. */
int mbx_replicate_backward(const void* grad, int dtype, int64_t batch, int64_t columns,
                           const int32_t* bins, int num_bins, void* out, mbx_stream_t stream);

/* --------------------------------------------------------------- permutation ops */

/* megablocks/backend/kernels.py:107-170 `gather` / `padded_gather` (_padded_copy,
 * A_TO_B): out row r of expert e (r counted from padded_bins[e-1], or bins[e-1] when
 * padded_bins is NULL) receives x[indices[i] / top_k] for the i-th sorted slot of e,
 * times weights[indices[i]] (fp32 product, rounded once) when weights is not NULL.
 * out has out_rows rows; rows owned by no slot (padding) are written as zeros.
 * x is [tokens, hidden].  slot_rows: optional, the map mbx_slot_rows() made of the same routing;
 * with it (and rows that are 16-byte multiples at 16-byte aligned bases) every token's row is
 * read once and written to its top_k places; without it one wave copies one output row. */
int mbx_gather(const void* x, int dtype, int64_t tokens, int hidden, int top_k,
               const int32_t* indices, const int32_t* bins, const int32_t* padded_bins,
               int num_bins, const void* weights, int w_dtype, void* out, int64_t out_rows,
               const int32_t* slot_rows, mbx_stream_t stream);

/* The index algebra of megablocks/backend/kernels.py:60-76 turned round: slot_rows[s] = the row of
 * the expert-major (optionally padded) buffer that holds slot s = t * top_k + j, -1 if none
 * does.  indices[i] is the slot at sorted position i; its row is i - bins[e-1] + padded_bins[e-1]
 * for the expert e of that position (bin_ids[i], or found in bins when bin_ids is NULL), or i
 * when padded_bins is NULL.  One map serves every gather and scatter of a layer step (forward and
 * backward): n_slots entries. */
int mbx_slot_rows(const int32_t* indices, const int32_t* bin_ids, const int32_t* bins,
                  const int32_t* padded_bins, int num_bins, int64_t n_slots, int32_t* slot_rows,
                  mbx_stream_t stream);

/* megablocks/backend/kernels.py:173-207 `scatter` / `padded_scatter` (_padded_copy,
 * !A_TO_B, then sum over top_k): out[t] = sum_j round(x[row(t*top_k+j)] * w[t*top_k+j]),
 * each product rounded to the storage type and the sum taken in fp32, like the
 * reference's two passes but without the [tokens, top_k, hidden] temporary.
 * slot_rows: the map of mbx_slot_rows(), or NULL to have it built here in scratch
 * (4 * tokens * top_k bytes; not used otherwise).  x has padded_bins[num_bins-1] rows, or
 * tokens * top_k if padded_bins is NULL: an entry of slot_rows at or past that reads as "no row". */
int mbx_scatter(const void* x, int dtype, int64_t tokens, int hidden, int top_k,
                const int32_t* indices, const int32_t* bin_ids, const int32_t* bins,
                const int32_t* padded_bins, int num_bins, const void* weights, int w_dtype,
                void* out, const int32_t* slot_rows, void* scratch, size_t scratch_bytes,
                mbx_stream_t stream);

/* mbx_scatter for callers that cannot allocate device memory and have no buffer to lend: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose
 * scatter allocates its [tokens, top_k, hidden] temporary through torch).  Same arguments and results as
 * mbx_scatter with slot_rows = NULL, except that the slot -> row map is built in a buffer that is part of the
 * library image (MBX_STATIC_SCATTER_MAX_SLOTS int32 entries = 4 MiB on every GPU the library runs on, held until the
 * process ends) instead of in caller-provided scratch.  It calls no allocator.  tokens * top_k above
 * MBX_STATIC_SCATTER_MAX_SLOTS returns MBX_ERANGE.  All calls on one GPU share that one buffer: calls that may
 * overlap on a GPU (different streams, different threads) race and must be ordered by the caller.  The buffer's
 * address is looked up by mbx_init() or on the first call on each device; a first call on a stream that is being
 * captured returns MBX_ECAPTURE and enqueues nothing (call mbx_init() on that device beforehand). */
#define MBX_STATIC_SCATTER_MAX_SLOTS (1 << 20)
int mbx_scatter_static(const void* x, int dtype, int64_t tokens, int hidden, int top_k,
                       const int32_t* indices, const int32_t* bin_ids, const int32_t* bins,
                       const int32_t* padded_bins, int num_bins, const void* weights, int w_dtype,
                       void* out, mbx_stream_t stream);

/* megablocks/backend/kernels.py:217-307 `scatter_wgrad` / `padded_scatter_wgrad`:
 * wgrad[indices[i]] = <x[row(i)], grad[indices[i] / top_k]> (fp32 accumulate, stored
 * in the type of x). */
int mbx_scatter_wgrad(const void* x, const void* grad, int dtype, int64_t tokens, int hidden,
                      int top_k, const int32_t* indices, const int32_t* bin_ids,
                      const int32_t* bins, const int32_t* padded_bins, int num_bins,
                      void* wgrad, mbx_stream_t stream);

/* The backward of `scatter` / `padded_scatter` with weights, megablocks/ops/scatter.py:34-62 and
 * megablocks/ops/padded_scatter.py:49-80 (a weighted gather of the output gradient, then
 * `scatter_wgrad`), in one pass over grad[tokens, hidden]:
 *   grad_x[row(s)] = round(grad[s / top_k] * weights[s]),   wgrad[s] = <x[row(s)], grad[s / top_k]>
 * for every slot s with a row in slot_rows (the map of mbx_slot_rows(), required); the other
 * rows of grad_x[out_rows, hidden] are written as zeros, the other entries of wgrad are left
 * alone.  Same values as mbx_gather + mbx_scatter_wgrad.  MBX_EUNSUPPORTED (the caller makes the
 * two calls): no map, top_k above 8, rows that are not 16-byte multiples at aligned bases. */
int mbx_scatter_backward(const void* grad, const void* x, int dtype, int64_t tokens, int hidden,
                         int top_k, const int32_t* indices, const int32_t* bins,
                         const int32_t* padded_bins, int num_bins, const void* weights,
                         int w_dtype, const int32_t* slot_rows, void* grad_x, int64_t out_rows,
                         void* wgrad, mbx_stream_t stream);

/* megablocks/backend/kernels.py:392-418 `binned_gather`: out [num_bins, capacity, hidden];
 * entry j of expert e = x[indices[bins[e-1]+j] / top_k] (* weight) for j < min(count_e,
 * capacity), zeros otherwise. */
int mbx_binned_gather(const void* x, int dtype, int64_t tokens, int hidden, int top_k,
                      const int32_t* indices, const int32_t* bins, int num_bins, int capacity,
                      const void* weights, int w_dtype, void* out, mbx_stream_t stream);

/* megablocks/backend/kernels.py:421-449 `binned_scatter`: the inverse of the above with the
 * sum over top_k; slots that were dropped contribute zero.  x is [num_bins, capacity,
 * hidden]; scratch: 4 * tokens * top_k bytes. */
int mbx_binned_scatter(const void* x, int dtype, int64_t tokens, int hidden, int top_k,
                       const int32_t* indices, const int32_t* bins, int num_bins, int capacity,
                       const void* weights, int w_dtype, void* out, void* scratch,
                       size_t scratch_bytes, mbx_stream_t stream);

/* megablocks/backend/kernels.py:521-543 `binned_scatter_wgrad`: wgrad[slot] =
 * <x[e, j], grad[slot / top_k]> for kept slots, 0 for dropped ones. */
int mbx_binned_scatter_wgrad(const void* x, const void* grad, int dtype, int64_t tokens,
                             int hidden, int top_k, const int32_t* indices, const int32_t* bins,
                             int num_bins, int capacity, void* wgrad, mbx_stream_t stream);

/* ------------------------------------------------------------------ grouped GEMM */

/* grouped_gemm.backend.gmm(a, b, batch_sizes, trans_a, trans_b, c) as called through
 * megablocks/grouped_gemm_util.py:25-26 (call sites megablocks/layers/mlp.py:414-523,
 * megablocks/layers/glu.py:84-205).  Row groups are given on the device as inclusive
 * int32 `bins` (no host copy of the sizes is needed); group e owns rows
 * [bins[e-1], bins[e]) of a.
 *   MBX_NN: c[r_e, :n] = a[r_e, :k] @ b[e] (b is [E, k, n])          rows = a.rows
 *   MBX_NT: c[r_e, :n] = a[r_e, :k] @ b[e]^T (b is [E, n, k])
 *   MBX_TN: c[e] = a[r_e, :k]^T @ b[r_e, :n] (c is [E, k, n]; all-zero for an empty group)
 * fp32 accumulation; a, b, c share `dtype`.  Rows of c at or past bins[E-1] are not
 * written (NN / NT). */
int mbx_gmm(const void* a, const void* b, void* c, int dtype, const int32_t* bins,
            int num_groups, int64_t rows, int k, int n, int layout, mbx_stream_t stream);

/* The input gradient of the GLU experts, megablocks/layers/glu.py:160-166
 * (`gmm(dsdd_out, w1, c=dx); dx += gmm(dv1_out, v1)`), as one reduction over both operand pairs:
 *   MBX_NN: c[r_e] = a[r_e] @ b[e] + a2[r_e] @ b2[e]      MBX_NT: ... @ b[e]^T + ... @ b2[e]^T
 * with a2 / b2 shaped like a / b.  One rounding of the fp32 sum instead of the reference's three.
 * Handles bf16 / f16 with k a multiple of 64 and at least 256, 16-byte aligned operands (n a multiple
 * of 8 for MBX_NN), any number of rows, one expert's weights below 2 GiB; anything else returns MBX_EUNSUPPORTED and the caller issues the
 * two mbx_gmm calls and the addition itself. */
int mbx_gmm_dual(const void* a, const void* b, const void* a2, const void* b2, void* c, int dtype,
                 const int32_t* bins, int num_groups, int64_t rows, int k, int n, int layout,
                 mbx_stream_t stream);

/* mbx_gmm (a2 == b2 == NULL) / mbx_gmm_dual with a workspace: device memory the launch may use to cut the tiles of its
 * last, partly filled round of workgroups along the reduction (MBX_NN with long reductions: a Mixtral-shaped second
 * product has 4.25 rounds of tiles on 256 compute units, and the quarter round costs as much as a whole one).  Parts
 * of a tile are summed in a fixed order: results do not change from run to run, but differ in the last bits from
 * those of a launch without workspace.  grouped_gemm.backend.gmm allocates what it needs through torch; this library
 * allocates nothing, so the caller lends the memory:
 *   workspace: mbx_gmm_workspace_bytes() bytes, 16-byte aligned (less: fewer tiles are cut; NULL: none are), whose
 *   first 4096 bytes are zero before the first launch that uses it.  Every launch leaves them zero again.  Launches
 *   that may run at the same time (different streams) need workspaces of their own. */
size_t mbx_gmm_workspace_bytes(void);
int mbx_gmm_ws(const void* a, const void* b, const void* a2, const void* b2, void* c, int dtype, const int32_t* bins,
               int num_groups, int64_t rows, int k, int n, int layout, void* workspace, size_t workspace_bytes,
               mbx_stream_t stream);

/* The first product of the expert MLP with its activation, megablocks/layers/mlp.py:521-522 / 414-416
 * (`x = gmm(x, w1, batch_sizes, trans_b=True); x = activation_fn(x)`), in one launch:
 *   c[r_e] = a[r_e] @ b[e]^T (b is [E, n, k]),   c_act = act(c)
 * where act is applied in the product's epilogue to c as stored (rounded to `dtype`), i.e. to the value the
 * reference's separate activation kernel reads.  Both outputs are [rows, n].  act: MBX_ACT_GELU_TANH.
 * MBX_EUNSUPPORTED (the caller runs mbx_gmm and the activation itself): fp32, another activation, k not a multiple of 64,
 * n not a multiple of 8, operands or outputs not 16-byte aligned, one expert's weights of 2 GiB or more. */
int mbx_gmm_act(const void* a, const void* b, void* c, void* c_act, int dtype, const int32_t* bins,
                int num_groups, int64_t rows, int k, int n, int act, mbx_stream_t stream);

/* The activation gradient of the expert MLP's backward, megablocks/layers/mlp.py:478-483 with
 * megablocks/layers/gelu.py:9-13 (`dact = gmm(ddsd_out, w2, trans_b=True); dsdd_out = gelu_backward_(dact, sdd_out)`),
 * in one launch:   c[r_e] = round(a[r_e] @ b[e]^T) * act'(pre[r_e])
 * with `pre` the saved first product ([rows, n], read in the epilogue).  The product is rounded to `dtype` before the
 * multiplication, as the reference's two steps round it.  Same restrictions and return codes as mbx_gmm_act. */
int mbx_gmm_dact(const void* a, const void* b, const void* pre, void* c, int dtype, const int32_t* bins,
                 int num_groups, int64_t rows, int k, int n, int act, mbx_stream_t stream);

/* The two first products of the GLU experts and their gated activation, megablocks/layers/glu.py:201-204
 * (`x1 = gmm(x, w1, trans_b=True); x2 = gmm(x, v1, trans_b=True); x1 = activation_fn(x1) * x2`), in one launch:
 *   x1[r_e] = a[r_e] @ b1[e]^T,   x2[r_e] = a[r_e] @ b2[e]^T   (b1, b2: [E, n, k]),   h = round(round(act(x1)) * x2)
 * every workgroup computes the same 128 columns of both products side by side and gates them in the epilogue, from the
 * values as stored (rounded to `dtype`).  All three outputs are [rows, n].  act: MBX_ACT_SILU or MBX_ACT_GELU_TANH.
 * MBX_EUNSUPPORTED (the caller runs two mbx_gmm and mbx_glu_forward): as for mbx_gmm_dglu. */
int mbx_gmm_glu(const void* a, const void* b1, const void* b2, void* x1, void* x2, void* h, int dtype,
                const int32_t* bins, int num_groups, int64_t rows, int k, int n, int act, mbx_stream_t stream);

/* The token gather and the experts' first product(s) in one launch: megablocks/layers/dmoe.py:219 / :273
 * (`x = ops.padded_gather(x, indices, bin_ids, bins, padded_bins, top_k)` / `ops.gather(...)`) followed by
 * megablocks/layers/mlp.py:521 (`gmm(x, w1, trans_b=True)`, then the activation) or glu.py:201-204.  The rows of the
 * product's first operand are read from the ungathered x through the row map, so the gathered copy is never written:
 *   A[first(e) + r] = x[indices[x_first(e) + r] / top_k]  for r < x_bins[e] - x_first(e),   zeros for the other rows of e
 * (first(e) = bins[e - 1], x_first(e) = x_bins[e - 1], 0 for e = 0: `bins` are the row bins of the products, `x_bins`
 * the bins of the sorted assignments `indices` -- padded_bins and bins of dmoe.py:131-154; x_bins NULL = `bins`), then
 *   b2 == NULL, h == NULL:  c = A[r_e] @ b1[e]^T
 *   b2 == NULL, h != NULL:  the same and h = act(c) as mbx_gmm_act writes it (act: MBX_ACT_GELU_TANH)
 *   b2 != NULL:             c, c2, h = x1, x2, h of mbx_gmm_glu (act: MBX_ACT_SILU or MBX_ACT_GELU_TANH)
 * x: [x_rows, k]; b1, b2: [E, n, k]; c, c2, h: [rows, n].  The results are bit-identical to mbx_gather / mbx_padded_gather
 * followed by mbx_gmm / mbx_gmm_act / mbx_gmm_glu.  An assignment outside [0, x_rows * top_k) reads as a row of zeros.
 * MBX_EUNSUPPORTED (the caller gathers and multiplies in two steps): what mbx_gmm_act / mbx_gmm_glu do not take, x of
 * 2 GiB or more, x_rows * top_k above INT32_MAX. */
int mbx_gmm_gather(const void* x, int64_t x_rows, const int32_t* indices, int top_k, const int32_t* x_bins,
                   const void* b1, const void* b2, void* c, void* c2, void* h, int dtype, const int32_t* bins,
                   int num_groups, int64_t rows, int k, int n, int act, mbx_stream_t stream);

/* The experts' second product and the weighted combine in one launch, for top_k = 1: megablocks/layers/mlp.py:523 /
 * glu.py:205 (`gmm(x, w2, batch_sizes)`) followed by megablocks/layers/dmoe.py:280 (`ops.scatter(x, indices, bin_ids,
 * expert_weights, bins, top_k)`, megablocks/backend/kernels.py:173-207).  With one expert per token an output row is one
 * product row times the token's weight -- no sum over top_k, no two tiles that write the same row -- so the store phase
 * of the product writes it:
 *   y = a[r_e] @ b[e]        (MBX_NN; a: [rows, k], b: [E, k, n])
 *   c[r] = y[r]                                  (c: [rows, n], or NULL: not wanted -- the backward pass reads it)
 *   out[indices[r]] = round(weights[indices[r]] * round(y[r]))        (out: [tokens, n]; weights NULL: 1)
 * for every row r of the product (rows == tokens * 1: the unpadded grouped layout).  indices: the sorted assignments
 * (int32 [rows]); weights: [tokens] of type w_dtype (an mbx_dtype).  The roundings are those of mbx_gmm followed by
 * mbx_scatter: the results are bit-identical.  A row whose assignment is outside [0, tokens) is not combined.  out rows
 * that no assignment names are left as they are.  MBX_EUNSUPPORTED: fp32, k not a multiple of 64, unaligned, an
 * expert's weights of 2 GiB or more -- multiply, then scatter. */
int mbx_gmm_scatter(const void* a, const void* b, void* c, void* out, int dtype, const int32_t* bins, int num_groups,
                    int64_t rows, int k, int n, const int32_t* indices, const void* weights, int w_dtype, int64_t tokens,
                    mbx_stream_t stream);

/* The weight gradient of the experts' first product(s) on token rows that were never gathered: the backward's
 * `gmm(dsdd_out, x, batch_sizes, trans_a=True)` of megablocks/layers/mlp.py:485-491 / glu.py:154-159, where x is what
 * megablocks/layers/dmoe.py:219 / :273 gathered (`ops.padded_gather` / `ops.gather`), with that gather done by the
 * operand loads -- the counterpart of mbx_gmm_gather for the training step, so that the gathered copy exists in neither
 * pass:
 *   c[e] = a[r_e]^T @ X[r_e],   X[first(e) + r] = x[indices[x_first(e) + r] / top_k] for r < x_bins[e] - x_first(e), else 0
 * (a: [rows, k]; x: [x_rows, n]; c: [E, k, n]; bins, x_bins, first, x_first as for mbx_gmm_gather).  Bit-identical to
 * mbx_gather / mbx_padded_gather followed by mbx_gmm(MBX_TN).
 * row_table: scratch of mbx_gmm_tn_gather_table_bytes(x_rows, top_k, num_groups) bytes (16-byte aligned) in which the
 * call builds the byte offset of every assignment's row, in the order the kernel's loads want them; table_ready != 0:
 * an earlier call with the same indices, x_bins, top_k, x_rows, num_groups and n has left it there (the two weight
 * gradients of a GLU layer share one).  MBX_ESCRATCH: no table, or too small or misaligned a one.
 * MBX_EUNSUPPORTED (the caller gathers and calls mbx_gmm): fp32, k or n not multiples of 8, operands not 16-byte
 * aligned, k of 128 or less, x or an operand of 2 GiB or more. */
size_t mbx_gmm_tn_gather_table_bytes(int64_t x_rows, int top_k, int num_groups);
int mbx_gmm_tn_gather(const void* a, const void* x, int64_t x_rows, const int32_t* indices, int top_k, const int32_t* x_bins,
                      void* c, int dtype, const int32_t* bins, int num_groups, int64_t rows, int k, int n, void* row_table,
                      size_t row_table_bytes, int table_ready, mbx_stream_t stream);

/* The backward of the GLU experts' gated activation on the product that feeds it, megablocks/layers/glu.py:135-153
 * (`gmm(ddsd_out, w2, trans_b=True, c=dactivation_fn_out)`, then autograd's gradient of
 * `activation_fn(sdd_out) * v1_out`, glu.py:120-124), in one launch:
 *   g = round(a[r_e] @ b[e]^T)        (a = ddsd_out, b = w2 as [E, n, k]: `gmm(ddsd_out, w2, trans_b=True)`)
 *   d1 = round(g * x2) * act'(x1)     (the gradient of sdd_out;  x1 = sdd_out, x2 = v1_out, all [rows, n])
 *   d2 = g * round(act(x1))           (the gradient of v1_out)
 * with the roundings of the separate steps; g itself is not stored.  act: MBX_ACT_SILU or MBX_ACT_GELU_TANH.
 * MBX_EUNSUPPORTED (the caller runs mbx_gmm and mbx_glu_backward): the cases of mbx_gmm_act. */
int mbx_gmm_dglu(const void* a, const void* b, const void* x1, const void* x2, void* d1, void* d2, int dtype,
                 const int32_t* bins, int num_groups, int64_t rows, int k, int n, int act, mbx_stream_t stream);

/* megablocks/layers/gelu.py:9-13 `_gelu_backward_inplace(g, x)`: g *= d/dx gelu_tanh(x). */
int mbx_gelu_backward_inplace(void* g, const void* x, int dtype, int64_t numel,
                              mbx_stream_t stream);

/* The gated activation of the GLU experts, megablocks/layers/glu.py:89,204
 * (`activation_fn(x1) * x2`) in one pass: out = round(round(act(a)) * b), i.e. with the same two
 * roundings as the reference's two element-wise ops.  act: 0 = SiLU, 1 = tanh-GELU.  numel must be a
 * multiple of 16 bytes' worth of elements and the buffers 16-byte aligned (else MBX_EINVAL). */
int mbx_glu_forward(const void* a, const void* b, void* out, int dtype, int act, int64_t numel,
                    mbx_stream_t stream);

/* Backward of the above as autograd derives it for glu.py:89 / glu.py:120-151:
 * db = g * round(act(a)), da = round(g * b) * act'(a). */
int mbx_glu_backward(const void* g, const void* a, const void* b, void* da, void* db, int dtype,
                     int act, int64_t numel, mbx_stream_t stream);

/* ---- router post-processing (megablocks/layers/router.py:87-106) ----
 * What LearnedRouter.forward does after the linear layer, for `tokens` rows of `num_experts` logits:
 *   scores  = softmax(logits, dim=-1)                                   router.py:98   [tokens, num_experts]
 *   weights, indices = scores.max(-1) (top_k == 1) / torch.topk(scores, top_k)  router.py:87-90  [tokens, top_k]
 *   weights = weights / norm(weights, p = norm_p, dim=-1)   if norm_p > 0        router.py:100-106
 * computed in fp32 and rounded to `dtype` where torch's operations round (scores; the norm; the quotient).
 * Weights come out in descending order; equal scores are taken in ascending expert index.  indices are
 * int64 like torch.topk's; indices32 (NULL: not wanted) receives the same values as int32, which saves the layer the
 * `top_expert.int()` pass of megablocks/layers/moe.py:160.  lse (NULL: not wanted) receives logsumexp(logits, dim=1) in
 * fp32, [tokens]: the term of the router z-loss, megablocks/layers/router.py:37, which the softmax has at hand.
 * num_experts up to 512 and top_k up to 64, else MBX_EUNSUPPORTED. */
int mbx_router_forward(const void* logits, int dtype, int64_t tokens, int num_experts, int top_k, float norm_p,
                       void* scores, void* weights, int64_t* indices, int32_t* indices32, float* lse,
                       mbx_stream_t stream);

/* Backward of the above as autograd derives it for router.py:98-106: grad_logits from grad_weights
 * [tokens, top_k] (NULL: none) and, optionally, a gradient that reaches `scores` directly (NULL: none;
 * e.g. from the load-balancing loss, moe.py:32-89), given the forward's scores and indices.  grad_lse (NULL: none): a
 * gradient that reaches the forward's `lse` ([tokens], fp32; from the z-loss, router.py:25-42); it adds
 * grad_lse[t] * scores[t, :] to the row. */
int mbx_router_backward(const void* grad_weights, const void* grad_scores, const void* scores, const int64_t* indices,
                        int dtype, int64_t tokens, int num_experts, int top_k, float norm_p, void* grad_logits,
                        const float* grad_lse, mbx_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MBX_H_ */
