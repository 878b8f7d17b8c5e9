/*
 * slora_hip.h -- C ABI of libslora_hip.so: heterogeneous multi-LoRA batching
 * over a unified paged adapter pool, for AMD MI355X (gfx950).
 *
 * Every pointer is a DEVICE pointer unless stated otherwise.  Nothing is
 * retained after a call returns; no call allocates, frees or synchronises.
 * Kernels are enqueued on `stream` (a hipStream_t passed as void*, NULL = the
 * default stream).  Every function returns SLORA_OK or a negative SLORA_ERR_*
 * code; slora_strerror() gives the message.  Shape checks happen on the host
 * before anything is launched; indices read on the device (adapter ids, page
 * ids) are range-checked against n_adapters / n_loc / n_pages and a token or
 * row whose index is out of range is skipped instead of faulting.
 *
 * Pool layout (reference: slora/common/mem_allocator.py:229-234,
 * slora/models/peft/layer_weights/lora_layer_weight.py:84-93): `w` is one
 * layer's buffer of `n_pages` pages of `page_elems` 16-bit elements.  An
 * adapter a of rank r owns the 4r page ids a_loc[a_start[a] .. +4r), a_len[a]
 * = 4r, grouped by projection p in (q,k,v,o):
 *   A side (key_buffer):   page a_loc[a_start[a] + p*r + j] = column j of A_p
 *                          (h_in elements).
 *   B side (value_buffer): the (h_out, r) row-major matrix B_p^T laid end to
 *                          end over pages a_loc[a_start[a] + p*r + 0..): element
 *                          (n, d) is at flat index n*r + d, page flat /
 *                          page_elems, offset flat % page_elems.
 * The reference ties page_elems to h_in (shrink) / h_out (expand); here it is
 * explicit so an output narrower than a page (grouped-query k/v) works.
 */
#ifndef SLORA_HIP_H
#define SLORA_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* major * 100 + minor.  The major number changes when an entry point is removed or its
 * signature changes (callers built against an older major must be rebuilt), the minor one when
 * entry points are added.
 *   2.0 (200): slora_bgmv_lora_planned (shrink and expand in one launch) has a new signature and a
 *              new plan layout behind it -- the 1.0 form was removed in 1.1 without a major bump,
 *              which this number corrects; plans hold hand-over counters (slora_bgmv_plan_bytes
 *              grew); + slora_pool_page_xor, slora_plan_status.
 *   1.2 (102): + slora_sgmm_expand_qkv.
 *   1.1 (101): + slora_sgmm_shrink_qkv, slora_pool_page_checksums, slora_pool_pack_transposed,
 *              slora_pool_alloc_contiguous_static; - slora_bgmv_lora_planned. */
#define SLORA_VERSION 200

#define SLORA_API __attribute__((visibility("default")))

/* storage types of x / y / w / scales */
#define SLORA_DTYPE_F16 0
#define SLORA_DTYPE_BF16 1
#define SLORA_DTYPE_F32 2 /* scales only */

#define SLORA_OK 0
#define SLORA_ERR_NULL_POINTER -1  /* a required pointer is NULL */
#define SLORA_ERR_BAD_DTYPE -2     /* dtype is not F16/BF16 (scales: F16/BF16/F32) */
#define SLORA_ERR_BAD_SHAPE -3     /* negative size, qkvo outside 0..3, stride too small, page ids over an empty pool */
#define SLORA_ERR_UNSUPPORTED -4   /* "No suitable kernel": width not a multiple of 8, rank above 512, ... */
#define SLORA_ERR_ALIGNMENT -5     /* a buffer the kernels read 16 bytes at a time is not 16-byte aligned */
#define SLORA_ERR_LAUNCH -6        /* the HIP runtime refused the launch */
#define SLORA_ERR_TOO_LARGE -7     /* a size exceeds the fixed capacity of an entry point that allocates nothing */

#define SLORA_MAX_RANK 512

SLORA_API int slora_version(void);
SLORA_API const char* slora_strerror(int code);

/* Index tables shared by every entry point
 * (reference: slora/server/router/model_infer/infer_adapter.py:11-24). */
typedef struct slora_tables {
  const int64_t* a_start; /* [n_adapters] offset of the adapter's block in a_loc */
  const int64_t* a_len;   /* [n_adapters] 4 * rank */
  const int64_t* a_loc;   /* [n_loc]      page ids */
  int64_t n_adapters;
  int64_t n_loc;
} slora_tables;

/* Decode shrink.  Replaces dispatch_bgmv with h_in >= h_out
 * (slora/csrc/lora_ops.cc:76-126 -> bgmv_multi_lora_rank_shrink_kernel,
 * slora/csrc/bgmv/bgmv_impl.cuh:14-149).
 *   y[b, j] = T( sum_k f32(w[page(a,p,j), k]) * f32(x[b, k]) ),  j < min(r_a, y_cols)
 * with a = bins[b], r_a = a_len[a]/4, p = qkvo.  Columns j >= r_a are left
 * untouched, nothing is scaled.  x is [batch, h_in] contiguous, y is
 * [batch, y_cols] contiguous. */
SLORA_API int slora_bgmv_shrink(void* y, const void* x, const void* w, const slora_tables* tables,
                      const int64_t* bins, int64_t batch, int64_t h_in, int64_t y_cols,
                      int64_t page_elems, int64_t n_pages, int qkvo, int dtype, void* stream);

/* Decode expand.  Replaces dispatch_bgmv with h_in < h_out
 * (slora/csrc/lora_ops.cc:76-126 -> bgmv_multi_lora_rank_expand_kernel,
 * slora/csrc/bgmv/bgmv_impl.cuh:152-208).
 *   y[b, n] = T( y[b, n] + T( sum_{d < min(r_a, x_cols)} f32(Bt[n*r_a + d]) * f32(x[b, d]) * f32(scales[a]) ) )
 * x is [batch, x_cols] contiguous, y is [batch, h_out] contiguous.  `scales`
 * is read in ITS OWN type scales_dtype (the reference reinterprets the fp16
 * scaling table as bf16 on the bf16 path, lora_ops.cc:118). */
SLORA_API int slora_bgmv_expand(void* y, const void* x, const void* w, const slora_tables* tables,
                      const int64_t* bins, const void* scales, int scales_dtype, int64_t batch,
                      int64_t x_cols, int64_t h_out, int64_t page_elems, int64_t n_pages,
                      int qkvo, int dtype, void* stream);

/* Decode shrink of q, k and v in ONE launch: the three calls of
 * slora/models/peft/lora_unordered_batch_infer.py:267-270, 287-290, 307-310
 * read the same x, so x is staged once.  y_q/y_k/y_v are three [batch, y_cols]
 * buffers; semantics per projection are those of slora_bgmv_shrink with
 * qkvo = 0, 1, 2. */
SLORA_API int slora_bgmv_shrink_qkv(void* y_q, void* y_k, void* y_v, const void* x, const void* w,
                          const slora_tables* tables, const int64_t* bins, int64_t batch,
                          int64_t h_in, int64_t y_cols, int64_t page_elems, int64_t n_pages,
                          int dtype, void* stream);

/* Decode expand of q, k and v in ONE launch (the calls of
 * lora_unordered_batch_infer.py:271-273, 291-295, 311-315).  x_* are the three
 * [batch, x_cols] shrink outputs, y_* are [batch, h_out_*] with their own
 * widths (k/v may be narrower than q). */
SLORA_API int slora_bgmv_expand_qkv(void* y_q, void* y_k, void* y_v, const void* x_q, const void* x_k,
                          const void* x_v, const void* w, const slora_tables* tables,
                          const int64_t* bins, const void* scales, int scales_dtype,
                          int64_t batch, int64_t x_cols, int64_t h_out_q, int64_t h_out_k,
                          int64_t h_out_v, int64_t page_elems, int64_t n_pages, int dtype,
                          void* stream);

/* ---- per-batch plan (no counterpart in the reference) ----------------------
 * The reference rebuilds nothing per call because it launches one block per
 * (token, rank row) and lets most of them exit; here a call walks
 * bins -> a_len/a_start -> a_loc before it can touch a weight.  Those tables do
 * not change between the 8 x n_layers calls of one decode step
 * (lora_unordered_batch_infer.py:254-318 passes the same req_bins and
 * infer_adapter tables to every call), so a caller may build a plan once per
 * step and pass it to the *_planned entry points, which then reach the weights
 * in one table read.  The plan lists the batch's work items: a "run" (up to 4
 * tokens that share an adapter) times a block of 8 rows, with the tokens and
 * the page ids of those rows for q, k, v and o.  It is valid as long as bins and the adapter tables keep their
 * contents.  rank_cap bounds the ranks whose page ids are stored (larger ranks
 * still work through a_loc).  Results are identical to the stateless calls. */

/* Bytes a plan for `batch` tokens needs (negative: SLORA_ERR_*). */
SLORA_API int64_t slora_bgmv_plan_bytes(int64_t batch, int64_t rank_cap);

/* Enqueue the plan build on `stream`.  `plan` is a 16-byte aligned device
 * buffer of at least slora_bgmv_plan_bytes(batch, rank_cap) bytes.  Word 1 of
 * the finished plan (int32) is the number of items, word 2 the largest rank in
 * the batch, word 6 the number of runs; a caller may read word 1 back and pass
 * it as n_items so that a launch has exactly one workgroup per item. */
SLORA_API int slora_bgmv_plan_build(void* plan, int64_t plan_bytes, const slora_tables* tables,
                                    const int64_t* bins, int64_t batch, int64_t rank_cap,
                                    int64_t n_pages, void* stream);

/* Status word of a plan (of slora_bgmv_plan_build or slora_sgmm_plan_build), copied to the host;
 * WAITS for the work queued on `stream`.  0 after a build.  Bit 0: a launch was given this plan
 * with another batch size, rank cap or launch shape than the plan was built for -- such a launch
 * does nothing (the outputs keep their values) and leaves this mark instead of an error code,
 * because only the device can tell.  Bit 1: a hand-over inside slora_bgmv_lora_planned was
 * abandoned after its poll limit.  The mark covers a wrong plan in a large enough buffer only: a
 * planned launch reads its item records before it has seen the header, so the buffer it is given
 * must hold slora_bgmv_plan_bytes(batch, rank_cap) bytes for the batch and rank cap OF THE LAUNCH,
 * whatever the plan in it was built for.  Not to be called on a stream that is being captured
 * into a graph (it copies to the host and waits).  No counterpart in the reference. */
SLORA_API int slora_plan_status(const void* plan, int* status, void* stream);

/* slora_bgmv_shrink / slora_bgmv_shrink_qkv with a plan.  nproj = 1: y0 and
 * qkvo as in slora_bgmv_shrink; nproj = 3: y0,y1,y2 = q,k,v and qkvo = 0.
 * n_items: the item count a caller read back (one workgroup per item), or 0:
 * the launch then has a quarter of the plan's capacity in workgroups, which
 * walk the items in strides of the grid -- right for any batch the plan may
 * hold, and the form to record into a graph that is replayed over new batches. */
SLORA_API int slora_bgmv_shrink_planned(const void* plan, int64_t rank_cap, int64_t n_items, int nproj,
                                        void* y0, void* y1, void* y2, const void* x, const void* w,
                                        const slora_tables* tables, const int64_t* bins,
                                        int64_t batch, int64_t h_in, int64_t y_cols,
                                        int64_t page_elems, int64_t n_pages, int qkvo, int dtype,
                                        void* stream);

/* slora_bgmv_expand / slora_bgmv_expand_qkv with a plan. */
SLORA_API int slora_bgmv_expand_planned(const void* plan, int64_t rank_cap, int64_t n_items, int nproj,
                                        void* y0, void* y1, void* y2, const void* x0, const void* x1,
                                        const void* x2, const void* w, const slora_tables* tables,
                                        const int64_t* bins, const void* scales, int scales_dtype,
                                        int64_t batch, int64_t x_cols, int64_t h_out0,
                                        int64_t h_out1, int64_t h_out2, int64_t page_elems,
                                        int64_t n_pages, int qkvo, int dtype, void* stream);

/* Shrink and expand of a projection (nproj = 1) or of q, k and v (nproj = 3, qkvo = 0) in ONE
 * launch, with a plan.  The reference issues the two back to back for every projection
 * (slora/models/peft/lora_unordered_batch_infer.py:267-273, 287-293, 307-313, 438-444); here one
 * workgroup per plan item computes its 8 rows of delta = x A, hands them to the other
 * workgroups of its run through counters behind the plan (device-scope stores and loads, no
 * second launch), and then updates y with its 8 pages of B^T:
 *   delta_i[b, j] = T(sum_k w_a[page(a,p,j), k] * x[b, k])                    as slora_bgmv_shrink
 *   y_i[b, n]     = T(y_i[b, n] + T(scales[a] * sum_d Bt[n*r+d] * delta_i[b, d]))  as slora_bgmv_expand
 * bit for bit what the two calls give.  delta_i ([batch, delta_cols], delta_cols a multiple of 8
 * and at least every rank in the batch for the usual result) is left filled as after the
 * shrink call.  w_a / w_b are the pools of the A side and the B side (key_buffer[l],
 * value_buffer[l]), which share page ids.  `plan` is written to (its counters): launches that
 * use one plan must not overlap, e.g. stay on one stream.  A hand-over that is not complete
 * after 65536 polls is abandoned (the workgroup goes on and a flag is set behind the plan)
 * rather than waited for for ever; it never is unless workgroups are not handed out in order. */
SLORA_API int slora_bgmv_lora_planned(void* plan, int64_t rank_cap, int64_t n_items, int nproj, void* y0, void* y1,
                                      void* y2, void* delta0, void* delta1, void* delta2, const void* x,
                                      const void* w_a, const void* w_b, const slora_tables* tables,
                                      const int64_t* bins, const void* scales, int scales_dtype, int64_t batch,
                                      int64_t h_in, int64_t delta_cols, int64_t h_out0, int64_t h_out1,
                                      int64_t h_out2, int64_t page_elems, int64_t n_pages, int qkvo, int dtype,
                                      void* stream);

/* Prefill (segmented) shrink.  Replaces lora_get_qkvo_fwd_shrink + _shrink_fwd_kernel
 * (slora/models/peft/triton_kernel/lora/lora_prefill.py:139-164, 57-102).
 * Request i owns token rows b_start_loc[i] + [0, b_seq_len[i]) and uses
 * adapter a = b_indicies[i]:
 *   o[row, j] = T( sum_k f32(x[row, k]) * f32(w[page(a,p,j), k]) )  for j < r_a
 *   o[row, j] = 0                                                    for r_a <= j < max_rank
 * x, w, o are addressed with element strides (row stride, and unit column
 * stride required). */
SLORA_API int slora_sgmm_shrink(void* o, const void* x, const void* w, const slora_tables* tables,
                      const int32_t* b_start_loc, const int32_t* b_seq_len,
                      const int64_t* b_indicies, int64_t n_requests, int64_t max_input_len,
                      int64_t n_tokens, int64_t h_in, int64_t max_rank, int64_t x_row_stride,
                      int64_t w_row_stride, int64_t o_row_stride, int64_t n_pages, int qkvo,
                      int dtype, void* stream);

/* Prefill shrink with a per-step plan.  No counterpart in the reference: its Triton
 * kernel (lora_prefill.py:57-102) looks up request and adapter in every program of every
 * one of the 4 x n_layers shrink launches of a prefill step
 * (lora_unordered_batch_infer.py:358-410), all with the same b_start_loc / b_seq_len /
 * b_indicies.  slora_sgmm_plan_build computes the split of the requests over the
 * workgroups once (it depends on the request lengths and adapter ranks only, not on
 * layer or projection) into `plan` (device memory, slora_sgmm_plan_bytes() bytes, 16-byte
 * aligned, owned by the caller); slora_sgmm_shrink_planned is slora_sgmm_shrink reading
 * that split: same arguments, same results bit for bit.
 *   *usable = 1: the plan was built.  0: this batch shape takes no plan (more than 256
 *   requests, more requests than workgroups, or nothing to do) -- call slora_sgmm_shrink.
 * slora_sgmm_shrink_planned returns SLORA_ERR_BAD_SHAPE for such a shape.  The sizes
 * (n_requests, max_input_len, n_tokens, max_rank) must be those of the build call; a plan
 * of another launch shape makes the kernel leave `o` untouched. */
SLORA_API int64_t slora_sgmm_plan_bytes(void);
SLORA_API int slora_sgmm_plan_build(void* plan, int64_t plan_bytes, const slora_tables* tables,
                          const int32_t* b_start_loc, const int32_t* b_seq_len,
                          const int64_t* b_indicies, int64_t n_requests, int64_t max_input_len,
                          int64_t n_tokens, int64_t max_rank, int* usable, void* stream);
SLORA_API int slora_sgmm_shrink_planned(const void* plan, void* o, const void* x, const void* w,
                              const slora_tables* tables, const int32_t* b_start_loc,
                              const int32_t* b_seq_len, const int64_t* b_indicies,
                              int64_t n_requests, int64_t max_input_len, int64_t n_tokens,
                              int64_t h_in, int64_t max_rank, int64_t x_row_stride,
                              int64_t w_row_stride, int64_t o_row_stride, int64_t n_pages,
                              int qkvo, int dtype, void* stream);

/* Prefill shrink of q, k and v in ONE launch.  The reference issues three shrink calls per
 * layer with the same x (slora/models/peft/lora_unordered_batch_infer.py:334-347, 374-381,
 * 400-407); here every 64-row tile of x is read once and multiplied with the weight rows of
 * the three projections in turn.  o_q / o_k / o_v are three [n_tokens, >= max_rank] outputs
 * with one row stride; per projection the results are those of slora_sgmm_shrink with qkvo =
 * 0, 1, 2, bit for bit.  plan: NULL, or a plan of slora_sgmm_plan_build for this batch
 * (SLORA_ERR_BAD_SHAPE if the batch shape takes no plan, as for slora_sgmm_shrink_planned). */
SLORA_API int slora_sgmm_shrink_qkv(const void* plan, void* o_q, void* o_k, void* o_v, const void* x, const void* w,
                          const slora_tables* tables, const int32_t* b_start_loc, const int32_t* b_seq_len,
                          const int64_t* b_indicies, int64_t n_requests, int64_t max_input_len,
                          int64_t n_tokens, int64_t h_in, int64_t max_rank, int64_t x_row_stride,
                          int64_t w_row_stride, int64_t o_row_stride, int64_t n_pages, int dtype, void* stream);

/* Prefill (segmented) expand.  Replaces lora_get_qkvo_fwd_expand + _expand_fwd_kernel
 * (lora_prefill.py:105-136, 10-54).
 *   o[row, n] = T( f32(o[row, n]) + (sum_{d < r_a} f32(x[row, d]) * f32(Bt[n*r_a + d])) * f32(scales[a]) )
 * `feat_out` is both the output width and the page width, as in the reference
 * (BLOCK_DMODEL, lora_prefill.py:42-43) unless page_elems > 0 overrides the
 * page width. */
SLORA_API int slora_sgmm_expand(void* o, const void* x, const void* w, const slora_tables* tables,
                      const void* scales, int scales_dtype, const int32_t* b_start_loc,
                      const int32_t* b_seq_len, const int64_t* b_indicies, int64_t n_requests,
                      int64_t max_input_len, int64_t n_tokens, int64_t feat_out,
                      int64_t page_elems, int64_t max_rank, int64_t x_row_stride,
                      int64_t w_row_stride, int64_t o_row_stride, int64_t n_pages, int qkvo,
                      int dtype, void* stream);

/* Prefill expand of q, k and v in ONE launch.  The reference issues three expand calls per
 * layer (slora/models/peft/lora_unordered_batch_infer.py:349-372, 383-398, 409-424); here the
 * output groups of the three projections share one grid, so a layer pays one launch instead of
 * three.  x_q / x_k / x_v are three [n_tokens, >= max_rank] inputs with one row stride; o_k and
 * o_v share width (feat_out_kv, narrower than feat_out_q in grouped-query models) and row
 * stride.  Per projection the results are those of slora_sgmm_expand with qkvo = 0, 1, 2 and
 * the same page_elems, bit for bit.  page_elems == 0: feat_out_q. */
SLORA_API int slora_sgmm_expand_qkv(void* o_q, void* o_k, void* o_v, const void* x_q, const void* x_k, const void* x_v,
                          const void* w, const slora_tables* tables, const void* scales, int scales_dtype,
                          const int32_t* b_start_loc, const int32_t* b_seq_len, const int64_t* b_indicies,
                          int64_t n_requests, int64_t max_input_len, int64_t n_tokens, int64_t feat_out_q,
                          int64_t feat_out_kv, int64_t page_elems, int64_t max_rank, int64_t x_row_stride,
                          int64_t w_row_stride, int64_t o_row_stride_q, int64_t o_row_stride_kv, int64_t n_pages,
                          int dtype, void* stream);

/* ---- moving adapters in and out of the pool --------------------------------- */

/* pool[loc[i]] = rows[i], i < n_rows, for n_bufs pool buffers in one go.
 * Replaces the per-layer index_put of the adapter loader,
 * `key_buffer[l][loc] = w_combined[0]` and `value_buffer[l][loc] = w_combined[1]`
 * (slora/server/router/model_infer/infer_adapter.py:56-57, 81-82).
 * dst_bufs / src_bufs are HOST arrays of n_bufs device pointers (e.g. the
 * key_buffer and value_buffer of every layer, and the two halves of every
 * layer's w_combined): src_bufs[b] holds n_rows rows of row_bytes bytes at
 * src_row_stride_bytes, dst_bufs[b] holds n_pages pages at
 * dst_row_stride_bytes.  loc is a device array of n_rows page ids shared by all
 * buffers; a page id outside [0, n_pages) is skipped.  Duplicate page ids give
 * an unspecified winner, as with index_put. */
SLORA_API int slora_pool_scatter_rows(void* const* dst_bufs, const void* const* src_bufs, int n_bufs,
                            const int64_t* loc, int64_t n_rows, int64_t row_bytes, int64_t dst_row_stride_bytes,
                            int64_t src_row_stride_bytes, int64_t n_pages, void* stream);

/* One adapter's LoRA matrices written straight into its pool pages, n_mats matrices per
 * call (e.g. A_q, A_k, A_v, A_o into the key_buffer and B_q .. B_o into the value_buffer of
 * every layer).  Replaces building w_combined on the host
 * (slora/models/peft/layer_weights/lora_layer_weight.py:84-93, 215-224) and the index_put
 * of its rows (slora/server/router/model_infer/infer_adapter.py:56-57, 81-82) with one pass.
 * Matrix i is a (rows[i] x cols[i]) row-major device array of 16-bit elements -- A_p as the
 * reference keeps it at home, (hidden x r), or B_p, (r x h_out).  It is written TRANSPOSED:
 * element (k, c) goes to flat position c * dst_pitch[i] + k of the slot formed by the pages
 * loc[first[i] .. first[i] + n_slot[i]) of dst_bufs[i], page flat / page_elems, offset flat
 * % page_elems.  dst_pitch = page_elems for A_p (column j of A_p becomes page j), dst_pitch
 * = rows = r for B_p (the dense (h_out, r) matrix B_p^T end to end); n_slot = r for both.
 * Positions of the slot no source element reaches are zeroed (what index_put of the
 * zero-padded w_combined leaves there).  first, rows, cols, dst_pitch, n_slot, dst_bufs and
 * src_mats are HOST arrays of n_mats entries; loc is the device array of page ids (n_loc
 * entries); a page id outside [0, n_pages) is skipped. */
SLORA_API int slora_pool_pack_transposed(void* const* dst_bufs, const void* const* src_mats, const int64_t* first,
                                         const int64_t* rows, const int64_t* cols, const int64_t* dst_pitch,
                                         const int64_t* n_slot, int n_mats, const int64_t* loc, int64_t n_loc,
                                         int64_t page_elems, int64_t n_pages, void* stream);

/* new_a_loc[new_a_start[i] + k] = old_a_loc[old_a_start[i] + k], k < old_a_len[i],
 * i < n_adapters.  Replaces launch_var_len_copy_triton
 * (slora/server/router/model_infer/infer_adapter.py:261-280); copies exactly
 * old_a_len[i] entries (the reference's mask over-copies lists longer than its
 * block of 256 into the next adapter's range).  A list that does not fit its
 * table (n_old_loc / n_new_loc entries) is skipped. */
SLORA_API int slora_var_len_copy(const int64_t* old_a_start, const int64_t* old_a_len, const int64_t* old_a_loc,
                       const int64_t* new_a_start, int64_t* new_a_loc, int64_t n_adapters, int64_t n_old_loc,
                       int64_t n_new_loc, void* stream);

/* The index tables after dropping the adapters with keep[i] == 0, in one launch.
 * Replaces the table rebuild of InferAdapter.offload_adapters
 * (slora/server/router/model_infer/infer_adapter.py:186-258: a_len[left_ind],
 * cumsum, a_scaling[left_ind], var_len_copy, torch.cat of the removed lists).
 * Kept adapters keep their order; new_a_start is the running sum of their
 * lengths; new_a_loc holds their page lists back to back; removed_pages holds the
 * page lists of the dropped adapters back to back, in order (what goes back to
 * the allocator).  counts[0..3] = kept adapters, kept page ids, dropped adapters,
 * dropped page ids.  Output arrays must have room for the worst case
 * (n_adapters / n_loc entries); work is n_adapters int64 of scratch owned by the
 * caller.  a_scaling / new_a_scaling are scales_dtype (2 or 4 bytes per entry). */
SLORA_API int slora_tables_compact(const slora_tables* tables, const void* a_scaling, int scales_dtype,
                         const uint8_t* keep, int64_t* new_a_start, int64_t* new_a_len, int64_t* new_a_loc,
                         void* new_a_scaling, int64_t* removed_pages, int64_t* counts, int64_t* work,
                         void* stream);

/* A_p of one adapter as a dense row-major (h, out_cols) matrix of 16-bit elements:
 * out[k, d] = pool[a_loc[first + d]][k] for d < rank, 0 for rank <= d < out_cols.
 * `first` = a_start[adapter] + qkvo * rank.  This is the unpacking of
 * slora/models/peft/lora_single_batch_infer.py:38-46
 * (`key_buffer[l][loc[p r:(p+1) r]].reshape(r, H).transpose(0, 1)`), the left
 * operand when an adapter is merged into the base weights (:60-93): with it,
 * W_p += scaling * A_p B_p is slora_sgmm_expand with x = A_p, o = W_p, one request
 * covering all h rows, and unmerging is the same call with the scale negated. */
SLORA_API int slora_pool_gather_a(void* out, int64_t out_cols, const void* pool, const int64_t* a_loc, int64_t n_loc,
                        int64_t first, int64_t rank, int64_t h, int64_t page_elems, int64_t n_pages, void* stream);

/* Checksums of pool pages: out[i] = xor of the 32-bit words of page loc[i] of `pool` (pages of
 * page_bytes bytes, a multiple of 16; an id outside [0, n_pages) gives 0).  No counterpart in
 * the reference, which has no way to tell whether the pages an adapter was copied into
 * (slora/server/router/model_infer/infer_adapter.py:43-88) still hold it.  The kernel is one
 * wavefront per page and only reads: the benchmark times it over the pages a LoRA launch
 * reads and reports that as the streaming ceiling of the launch. */
SLORA_API int slora_pool_page_checksums(uint32_t* out, const void* pool, const int64_t* loc, int64_t n,
                                        int64_t page_bytes, int64_t n_pages, void* stream);

/* In-place xor of pool pages: every 32-bit word of page loc[i] of `pool` ^= key (ids outside
 * [0, n_pages) are skipped; a page listed twice is undefined).  No counterpart in the reference.
 * Like slora_pool_page_checksums it is a measurement aid as much as a tool: one wavefront per
 * page, loads then stores and nothing else, so with key = 0 its duration over the rows of an
 * output is the read-modify-write floor the benchmark reports next to the expand kernels. */
SLORA_API int slora_pool_page_xor(void* pool, const int64_t* loc, int64_t n, int64_t page_bytes, int64_t n_pages,
                                  uint32_t key, void* stream);

/* ---- page allocator over the pool's free map ---------------------------------
 * mem_state: one byte per pool page, 1 = free (the reference's torch.bool
 * `mem_state`, slora/common/mem_allocator.py:222).  `workspace` is device memory of
 * slora_pool_alloc_workspace_bytes(tot_size) bytes owned by the caller; `result`
 * is two device int64.  The host keeps the free-page count itself, as the
 * reference does (`can_use_mem_size`). */
SLORA_API int64_t slora_pool_alloc_workspace_bytes(int64_t tot_size);

/* MemoryAllocator.alloc (mem_allocator.py:30-39): the first `need` free pages in
 * index order are written to out_index (ascending) and marked used; result[0] =
 * pages handed out (fewer than `need` only if the map has fewer free pages). */
SLORA_API int slora_pool_alloc(uint8_t* mem_state, int64_t tot_size, int64_t need, int64_t* out_index,
                     int64_t* result, void* workspace, void* stream);

/* MemoryAllocator.alloc_contiguous (mem_allocator.py:42-59): the first start s with
 * pages [s, s + need) all free; they are marked used and listed in out_index.
 * result[0] = s or -1 if there is no such run (nothing is changed then),
 * result[1] = pages handed out. */
SLORA_API int slora_pool_alloc_contiguous(uint8_t* mem_state, int64_t tot_size, int64_t need, int64_t* out_index,
                                int64_t* result, void* workspace, void* stream);

/* slora_pool_alloc_contiguous without a workspace argument, for callers that cannot
 * allocate device memory (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * workspace is an array inside the library's device image (about 48 KiB, held by
 * every GPU the library runs on until the process ends), good for maps of up to
 * SLORA_POOL_STATIC_MAX_PAGES pages; a larger tot_size returns SLORA_ERR_TOO_LARGE.
 * Arguments and results are those of slora_pool_alloc_contiguous.  All calls on
 * one GPU share the array: calls that overlap on one GPU (two streams) race. */
#define SLORA_POOL_STATIC_MAX_PAGES (1 << 24)
SLORA_API int slora_pool_alloc_contiguous_static(uint8_t* mem_state, int64_t tot_size, int64_t need,
                                                 int64_t* out_index, int64_t* result, void* stream);

/* MemoryAllocator.free (mem_allocator.py:185-199): mem_state[free_index] = 1;
 * ids outside the map are skipped. */
SLORA_API int slora_pool_free(uint8_t* mem_state, int64_t tot_size, const int64_t* free_index, int64_t n,
                    void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SLORA_HIP_H */
