/*
 * come_hip.h — C ABI of libcome_hip.so, the MI355X (gfx950) implementation of the
 * Co-Me accelerated-inference hot path: confidence-guided token merge, unmerge and
 * the forward varlen attention with an additive per-key bias.
 *
 * Every entry point takes plain device pointers and sizes, enqueues its kernels on
 * the HIP stream passed in `stream` (a hipStream_t; NULL = the null stream) and
 * returns without synchronising.  Nothing here allocates device memory: outputs and
 * small work buffers are supplied by the caller.  The device that owns the pointers
 * must be the current HIP device of the calling thread.
 *
 * Return value: COME_OK (0) or a come_status error code; come_last_error() then
 * holds a message for the calling thread.
 *
 * Each declaration cites the interface of the reference (co-me-tokens/CoMe, paths
 * relative to its root) that the entry point stands in for.
 */
#ifndef COME_HIP_H
#define COME_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum come_status {
    COME_OK = 0,
    COME_ERR_INVALID = 1,     /* bad argument (null pointer, negative size, inconsistent shape) */
    COME_ERR_UNSUPPORTED = 2, /* a combination this library does not implement                 */
    COME_ERR_HIP = 3          /* a HIP runtime call or kernel launch failed                    */
} come_status;

typedef enum come_dtype {
    COME_F32 = 0,
    COME_F16 = 1,
    COME_BF16 = 2
} come_dtype;

/*
 * Bits of the `flags` argument of come_attn_varlen_fwd / _ws / _static (head_dim 64; the other widths always use
 * the arithmetic of flags = 0).  They are per call: nothing in the library remembers them.
 *
 *   0                      softmax_scale is applied in fp32 to every score, q enters the matrix unit as it is and
 *                          bias / scale is added to the raw scores: the reference's arithmetic
 *                          (src/cuda_extension/flash_attn/src/flash_fwd_kernel.h:30-55, src/softmax.h:76-88).
 *   COME_ATTN_FOLD_SCALE   q is multiplied by softmax_scale * log2(e) once and rounded back to `dtype`, which saves
 *                          one vector instruction per score (about 10 % of the run time) and moves a logit by up to
 *                          2^-9 of its size: inside 1e-2 max-abs / 1e-3 mean-abs for logits within about +-10 nats
 *                          (q / k LayerNorm with gains near 1), outside it from about +-20 nats on.  A caller that
 *                          knows such a bound for its logits may set it; nothing else should.
 *   COME_ATTN_WORK_QUEUE   (come_attn_varlen_fwd_ws / _static, segments of at most 2048 keys, at most 65 536
 *                          (segment, head) units) the launch is two resident workgroups per CU which take their
 *                          256-query blocks from a queue in the work buffer - a one-workgroup kernel builds it from
 *                          cu_seqlens first: lists of (unit, block) items without empty entries - and stage the
 *                          first tiles of their next item during the last iterations of the current one.  Needs
 *                          come_attn_queue_bytes(...) bytes of buffer; without them the flag is ignored.  Same bits
 *                          as the default launch (one workgroup per query block).  Measured 5 - 12 % SLOWER than the
 *                          default on every shape tried: the hardware's own dispatch staggers and re-ages the two
 *                          workgroups of a CU, which a resident pair cannot.  Kept for callers whose segment mix
 *                          defeats a static grid (max_seqlen far above most lengths costs nothing here).
 */
enum { COME_ATTN_FOLD_SCALE = 1, COME_ATTN_WORK_QUEUE = 2 };

/* Library version (major * 10000 + minor * 100 + patch); 200 = 0.2.0, the first with `flags` on the attention entry points; 201 adds come_attn_varlen_fwd_qp. */
int come_version(void);

/* Message of the last failing call made by this thread ("" if none). */
const char *come_last_error(void);

/*
 * come_merge_plan — from the merge mask to packed-row bookkeeping.
 *
 *   merge_mask   [rows, groups] bytes, non-zero = merge that group into one row
 *   offsets      [rows + 1] int32 out: offsets[0] = 0,
 *                offsets[b+1] - offsets[b] = start_index + tail + sum_m (mask ? 1 : group_size)
 *   group_prefix [rows, groups] int32 out: exclusive prefix of (mask ? 1 : group_size)
 *                inside the row
 *
 * Stands in for block_prefix_scan_kernel + the cumsum glue of the reference
 * (src/cuda_extension/co_me/src/kernel_token_merge.cu:12-46, 271-286) and for
 * `offsets` of func_token_merge (src/accelerate/token_merger/co_me.py:177-182).
 * `tail` (tokens behind the groups that are always copied) is 0 in the reference.
 */
int come_merge_plan(const uint8_t *merge_mask, int64_t rows, int64_t groups,
                    int64_t start_index, int64_t group_size, int64_t tail,
                    int32_t *offsets, int32_t *group_prefix, void *stream);

/*
 * come_token_merge — gather-mean of the selected windows into packed rows.
 *
 *   tokens   [rows, n_tok, chans] of `dtype`, contiguous;
 *            n_tok = start_index + grid_h * grid_w
 *   windows  group_h x group_w over the grid_h x grid_w token grid, block-row-major,
 *            row-major inside a window; a 1-D merge of `M` groups of `G` tokens is
 *            grid_h = 1, grid_w = M * G, group_h = 1, group_w = G.
 *            Grid positions outside the (grid_h / group_h) x (grid_w / group_w) full
 *            windows are copied behind the windows in image row-major order.
 *   merge_mask, offsets, group_prefix   as produced by / passed to come_merge_plan
 *            (same rows, groups = full windows per row, start_index,
 *            group_size = group_h * group_w, tail = positions outside full windows)
 *   out      [out_rows, chans] of `dtype`; rows at or beyond out_rows are not written
 *   rev_i64 / rev_i32   [rows * n_tok] packed row of every source token, in the
 *            original (image row-major) token order; either may be NULL
 *   weight_f32 / count_i32   [out_rows] number of source tokens per packed row;
 *            either may be NULL
 *
 * Packed layout per row block: [specials | window 0 | window 1 | ... | leftover positions];
 * a merged window is one row = mean of its tokens (fp32 accumulation, one rounding).
 *
 * Stands in for co_me_token_merge_cuda (src/cuda_extension/co_me/src/binding.cpp:33-42,
 * kernel_token_merge.cu:50-191, 239-348), for func_token_merge
 * (src/accelerate/token_merger/co_me.py:153-222) and, with group_h > 1, for
 * func_token_merge_2d (src/accelerate/token_merger/co_me_2d.py:174-211) without its
 * permuted copy of the tokens.
 */
int come_token_merge(const void *tokens, int dtype, int64_t rows, int64_t n_tok, int64_t chans,
                     int64_t start_index, int64_t group_h, int64_t group_w,
                     int64_t grid_h, int64_t grid_w,
                     const uint8_t *merge_mask, const int32_t *offsets, const int32_t *group_prefix,
                     void *out, int64_t out_rows,
                     int64_t *rev_i64, int32_t *rev_i32, float *weight_f32, int32_t *count_i32,
                     void *stream);

/*
 * come_token_split — unmerge: out[i, :] = merged[rev[i], :].
 *
 *   merged  [merged_rows, chans] of `dtype`, contiguous
 *   rev     [total] int64 (rev_i64) or int32 (rev_i32); exactly one is non-NULL
 *   out     [total, chans] of `dtype`
 * An index outside [0, merged_rows) yields a row of zeros.
 *
 * Stands in for co_me_token_split_cuda (src/cuda_extension/co_me/src/binding.cpp:44-51,
 * kernel_token_merge.cu:195-233, 354-398) and func_token_split
 * (src/accelerate/token_merger/co_me.py:241-254).
 */
int come_token_split(const void *merged, int dtype, int64_t merged_rows, int64_t chans,
                     const int64_t *rev_i64, const int32_t *rev_i32, int64_t total,
                     void *out, void *stream);

/*
 * come_token_split_pair — unmerge two packed tensors that share one index map into one
 * dense tensor with their channels side by side:
 *   out[i, :chans] = merged_a[rev[i], :],  out[i, chans:] = merged_b[rev[i], :].
 *
 *   merged_a, merged_b  [merged_rows, chans] of `dtype`, contiguous
 *   out                 [total, 2 * chans] of `dtype`
 * Other arguments and the out-of-range rule as for come_token_split.
 *
 * Stands in for the two token splits followed by torch.cat(dim=-1) at the retained layers
 * of the fused aggregator (src/accelerate/vggt/fused.py:157-165): one launch and one pass
 * over the output instead of two splits plus a concatenation.
 */
int come_token_split_pair(const void *merged_a, const void *merged_b, int dtype,
                          int64_t merged_rows, int64_t chans,
                          const int64_t *rev_i64, const int32_t *rev_i32, int64_t total,
                          void *out, void *stream);

/*
 * come_select_windows — per-window confidence mean and lowest-confidence selection.
 *
 *   conf     [batch * frames, grid_h, grid_w] of `dtype` (COME_BF16 or COME_F32), contiguous
 *   mode     0 = ranking: per batch element, over its frames * windows means jointly,
 *                mask = mean < quantile(float(mean), threshold) with torch.quantile's
 *                linear interpolation;
 *            1 = absolute: mask = mean < threshold (threshold rounded to `dtype` first, as a
 *                comparison of a `dtype` tensor with a scalar does)
 *            2 = normalised: the confidence of a batch element is first turned into
 *                z = (x - mean) / (std + 1e-3) over all its positions (unbiased std, every
 *                step rounded to `dtype`), then mask = window mean of z < threshold (rounded likewise)
 *   means_f32 [batch * frames, windows] float out (the means, rounded to `dtype` first);
 *            may be NULL
 *   merge_mask [batch * frames, windows] bytes out (1 = merge)
 *   work     device scratch that holds the means when means_f32 is NULL: at least
 *            come_select_work_bytes(...) bytes; not used (may be NULL) when means_f32 is given
 *
 * Stands in for the window-mean + torch.quantile + compare sequence of
 * _CoMe_2D_Base.build_ctx (src/accelerate/token_merger/co_me_2d.py:268-298; mode 2:
 * :275-283).
 */
int come_select_windows(const void *conf, int dtype, int64_t batch, int64_t frames,
                        int64_t grid_h, int64_t grid_w, int64_t group_h, int64_t group_w,
                        int mode, float threshold,
                        float *means_f32, uint8_t *merge_mask, void *work, int64_t work_bytes,
                        void *stream);
int64_t come_select_work_bytes(int64_t batch, int64_t frames, int64_t grid_h, int64_t grid_w,
                               int64_t group_h, int64_t group_w);

/*
 * come_select_plan — come_select_windows followed by come_merge_plan of the selected mask, in one launch when
 * batch == 1 (the mask never leaves the workgroup that made it; with batch > 1 a second, one-wavefront launch scans
 * the row lengths into offsets).
 *
 *   arguments up to merge_mask as for come_select_windows; start_index as for come_merge_plan
 *   offsets      [batch * frames + 1] int32 out, group_prefix [batch * frames, windows] int32 out: exactly what
 *                come_merge_plan(merge_mask, batch * frames, windows, start_index, group_h * group_w,
 *                grid_h * grid_w - windows * group_h * group_w, ...) writes
 * The grid must hold at least one full window.
 *
 * Stands in for build_ctx's selection (src/accelerate/token_merger/co_me_2d.py:268-298) plus the scan + cumsum
 * front end of the merge (src/cuda_extension/co_me/src/kernel_token_merge.cu:12-46, 271-286), which the reference
 * runs as torch.quantile's sort, a dozen small tensor kernels and two host reads.
 */
int come_select_plan(const void *conf, int dtype, int64_t batch, int64_t frames,
                     int64_t grid_h, int64_t grid_w, int64_t group_h, int64_t group_w,
                     int mode, float threshold, int64_t start_index,
                     float *means_f32, uint8_t *merge_mask, int32_t *offsets, int32_t *group_prefix,
                     void *work, int64_t work_bytes, void *stream);

/*
 * come_attn_varlen_fwd — softmax(Q K^T * softmax_scale + bias[key]) V per packed
 * segment and head, forward only, no causal mask, no dropout.
 *
 *   q, k, v   [total, n_heads, head_dim] views of `dtype` (COME_BF16 or COME_F16) with
 *             unit stride in the last dimension; *_row_stride / *_head_stride in elements
 *             (q/k/v are usually slices of one packed [total, 3, n_heads, head_dim] tensor)
 *   cu_seqlens [n_seq + 1] int32 segment boundaries, cu_seqlens[n_seq] <= total
 *   perkey_bias [total] of `dtype`, or NULL for plain attention
 *   max_seqlen  upper bound of the segment lengths (sizes the launch grid)
 *   out       [total, n_heads, head_dim] of `dtype`, strides in elements
 *   lse       [n_heads, total] float: logsumexp of the biased, scaled scores; may be NULL
 *   flags     0 or COME_ATTN_FOLD_SCALE (above)
 * head_dim is 32, 64 or 128 (the reference instantiates 32 ... 256 in steps of 32,
 * src/cuda_extension/flash_attn/src/flash_fwd_launch_template.h:174-330; callers pad other widths up to 128 with
 * zero columns, which changes neither q . k nor the other output columns).
 * head_dim 64, the width of the shipped models: probabilities are kept relative to a lazily moved reference point
 * of their row and stored in `dtype`; a workgroup that meets a key beating everything its rows have seen by more than
 * that type can hold within one 32-key step (2^127 for COME_BF16, about 2^15 for COME_F16) computes its query block
 * again with a running maximum, so the result is right for any finite scores.
 * head_dim 32 and 128: one 32-query tile per wavefront, scale and bias applied to the fp32 scores (as with
 * flags = 0), running maximum per row; no work buffer is used.
 *
 * Stands in for varlen_fwd / varlen_fwd_w_perkey_bias
 * (src/cuda_extension/flash_attn/flash_api.cpp:291-607; kernel
 * src/cuda_extension/flash_attn/src/flash_fwd_kernel.h:30-55, 80-545) as reached from
 * flash_attn_varlen_qkvpacked_func[_w_perkey_bias]
 * (src/cuda_extension/flash_attn/__init__.py:235-295, 439-477).
 */
int come_attn_varlen_fwd(const void *q, const void *k, const void *v, int dtype,
                         int64_t q_row_stride, int64_t q_head_stride,
                         int64_t k_row_stride, int64_t k_head_stride,
                         int64_t v_row_stride, int64_t v_head_stride,
                         const int32_t *cu_seqlens, int64_t n_seq, int64_t total,
                         int64_t n_heads, int64_t head_dim,
                         const void *perkey_bias, int64_t max_seqlen, float softmax_scale,
                         void *out, int64_t o_row_stride, int64_t o_head_stride,
                         float *lse, int flags, void *stream);

/*
 * come_attn_varlen_fwd_ws — the same operator with a caller-supplied work buffer.  When the launch would end
 * in a partly filled last round of workgroups (long segments), the query blocks of that round are computed as
 * several workgroups each, every one over its share of the keys, into `work`, and combined by a second small
 * kernel: the result is the same up to rounding, the tail of the launch is shorter.
 *
 *   work, work_bytes   device buffer, 16-byte aligned, of at least come_attn_work_bytes(...) bytes; NULL or a
 *                      smaller buffer makes the call identical to come_attn_varlen_fwd
 * come_attn_work_bytes returns 0 when a launch of that shape would not use a buffer.  The buffer is used for
 * head_dim 64 only: the size query does not know the head width, so callers of the 32- and 128-wide instances pass
 * NULL / 0 instead of allocating what it returns.
 *
 * No counterpart in the reference (its kernel has a split-KV variant for decoding only,
 * src/cuda_extension/flash_attn/src/flash_fwd_launch_template.h:99-157, unreachable from the varlen forward).
 */
int64_t come_attn_work_bytes(int64_t n_seq, int64_t total, int64_t n_heads, int64_t max_seqlen);
/* Buffer size for COME_ATTN_WORK_QUEUE (0: that shape never uses a queue).  No counterpart in the reference, whose
 * grid is (ceil(max_seqlen / 128), batch, heads) (src/cuda_extension/flash_attn/src/flash_fwd_launch_template.h:63-64). */
int64_t come_attn_queue_bytes(int64_t n_seq, int64_t n_heads, int64_t max_seqlen);
int come_attn_varlen_fwd_ws(const void *q, const void *k, const void *v, int dtype,
                            int64_t q_row_stride, int64_t q_head_stride,
                            int64_t k_row_stride, int64_t k_head_stride,
                            int64_t v_row_stride, int64_t v_head_stride,
                            const int32_t *cu_seqlens, int64_t n_seq, int64_t total,
                            int64_t n_heads, int64_t head_dim,
                            const void *perkey_bias, int64_t max_seqlen, float softmax_scale,
                            void *out, int64_t o_row_stride, int64_t o_head_stride,
                            float *lse, void *work, int64_t work_bytes, int flags, void *stream);

/*
 * come_attn_varlen_fwd_static — come_attn_varlen_fwd_ws without a buffer argument and without any allocation:
 * the pieces of the key-split tail go to a fixed array of come_attn_static_work_bytes() bytes (64 MiB) that is part
 * of the library's device image, one copy per GPU, held until the process ends.  Same kernels, same launch shape
 * and therefore the same results as come_attn_varlen_fwd_ws with a buffer of come_attn_work_bytes(...) bytes.
 *
 * A launch whose come_attn_work_bytes(...) exceeds come_attn_static_work_bytes() fails with COME_ERR_UNSUPPORTED
 * (nothing is enqueued).  All calls on one GPU share that GPU's array: calls that may run concurrently there (on
 * different streams or from different threads) race on it and must be serialised by the caller; calls on one
 * stream are ordered by the stream.  Nothing in the array has to be cleared between calls: every piece is
 * written in full before the combining kernel of the same call reads it.
 *
 * come_attn_static_work_bytes() also looks up the address of the current device's copy of the array (-1 if that
 * fails); a caller that records launches into a graph calls it once per device before the capture, so that the
 * entry point itself makes nothing but kernel launches.
 *
 * No counterpart in the reference.  It is for callers that cannot allocate device memory around the call: code
 * under HIP graph capture, tight serving loops, harnesses that forbid allocation.
 */
int64_t come_attn_static_work_bytes(void);
int come_attn_varlen_fwd_static(const void *q, const void *k, const void *v, int dtype,
                                int64_t q_row_stride, int64_t q_head_stride,
                                int64_t k_row_stride, int64_t k_head_stride,
                                int64_t v_row_stride, int64_t v_head_stride,
                                const int32_t *cu_seqlens, int64_t n_seq, int64_t total,
                                int64_t n_heads, int64_t head_dim,
                                const void *perkey_bias, int64_t max_seqlen, float softmax_scale,
                                void *out, int64_t o_row_stride, int64_t o_head_stride,
                                float *lse, int flags, void *stream);

/*
 * come_qk_norm_rope — attention prologue, in place on the packed projection output:
 * LayerNorm over the head dimension of every q and k head, then the 2-D rotary position
 * embedding.
 *
 *   q, k      [total, n_heads, head_dim] views of `dtype` (COME_BF16 or COME_F16), unit stride
 *             inside a head, *_row_stride / *_head_stride in elements; overwritten.  One of them may be
 *             NULL: that tensor is skipped (its strides are not looked at)
 *   apply_norm  0 = no normalisation; otherwise y = (x - mean) * rsqrt(var + eps) * weight + bias
 *             over the head_dim elements of a head (biased variance, fp32 arithmetic, one
 *             rounding to `dtype`); q_weight / q_bias / k_weight / k_bias are [head_dim] of
 *             `dtype`, NULL = 1 resp. 0
 *   positions [total, 2] int64 (y, x) per row, or NULL = no rotation.  The first half of a
 *             head rotates with y, the second with x; inside a half h of H = head_dim / 2
 *             elements, out[j] = h[j] cos[j mod H/2] - h[j + H/2] sin[j mod H/2] for j < H/2
 *             and out[j] = h[j] cos[j mod H/2] + h[j - H/2] sin[j mod H/2] otherwise, products
 *             and sum each rounded to `dtype`.
 *   cos_table, sin_table  [n_pos, head_dim / 4] of `dtype`: cos / sin of
 *             position * base^(-i / (head_dim / 4)); positions are clamped to [0, n_pos)
 * Only head_dim == 64 is implemented.
 *
 * Stands in for the inference branch of prepare_packed_self_attention_qkv
 * (src/accelerate/common/qkv.py:31-39): q_norm / k_norm of
 * src/thirdparty/vggt/layers/attention.py:40-41 and RotaryPositionEmbedding2D.forward
 * (src/thirdparty/vggt/layers/rope.py:100-187), which the reference runs as eight tensor
 * passes over q and k.
 */
int come_qk_norm_rope(void *q, void *k, int dtype,
                      int64_t q_row_stride, int64_t q_head_stride,
                      int64_t k_row_stride, int64_t k_head_stride,
                      int64_t total, int64_t n_heads, int64_t head_dim,
                      int apply_norm, const void *q_weight, const void *q_bias,
                      const void *k_weight, const void *k_bias, float eps,
                      const int64_t *positions, const void *cos_table, const void *sin_table,
                      int64_t n_pos, void *stream);

/*
 * come_attn_varlen_fwd_qp — come_attn_varlen_fwd_ws with the q half of come_qk_norm_rope applied to the query rows
 * as the kernel loads them: q in memory is the raw projection (it is not written), k has been through
 * come_qk_norm_rope (which skips a NULL q), and the result is bit for bit what come_attn_varlen_fwd_ws returns after
 * come_qk_norm_rope on both - the kernel runs the same arithmetic in the same order on its query fragments.  Saves
 * the read and the write of q in the prologue pass (half its traffic).
 *
 *   prologue  the q-side arguments of come_qk_norm_rope with the same meaning (weight / bias may be NULL;
 *             positions NULL = no rotation, otherwise cos_table / sin_table [n_pos, 16] of `dtype`); pointers
 *             16-byte aligned.  NULL makes the call identical to come_attn_varlen_fwd_ws.
 * head_dim must be 64, and COME_ATTN_WORK_QUEUE is refused (COME_ERR_UNSUPPORTED).
 *
 * In the reference the prologue is a separate step of the caller (src/accelerate/common/qkv.py:31-39, called at
 * src/accelerate/vggt/module/bias_attention.py:100-106 right in front of the operator); this entry point is for a
 * caller that hands the q-side step to the operator.
 */
typedef struct come_q_prologue {
    int apply_norm;                 /* 0 = no LayerNorm */
    float eps;
    const void *weight, *bias;      /* [64] of dtype, NULL = 1 resp. 0 */
    const int64_t *positions;       /* [total, 2] (y, x), NULL = no rotation */
    const void *cos_table, *sin_table;
    int64_t n_pos;
} come_q_prologue;
int come_attn_varlen_fwd_qp(const void *q, const void *k, const void *v, int dtype,
                            int64_t q_row_stride, int64_t q_head_stride,
                            int64_t k_row_stride, int64_t k_head_stride,
                            int64_t v_row_stride, int64_t v_head_stride,
                            const int32_t *cu_seqlens, int64_t n_seq, int64_t total,
                            int64_t n_heads, int64_t head_dim,
                            const void *perkey_bias, int64_t max_seqlen, float softmax_scale,
                            void *out, int64_t o_row_stride, int64_t o_head_stride,
                            float *lse, void *work, int64_t work_bytes,
                            const come_q_prologue *prologue, int flags, void *stream);

/*
 * come_jagged_add_suffix / come_jagged_split_suffix — append `count` dense rows to every packed
 * segment, or strip the last `count` rows of every segment again.
 *
 *   tokens   [rows, chans] of `dtype`, weight [rows] float (may be NULL together with out_weight)
 *   offsets  [n_seg + 1] int64 segment boundaries of the input, offsets[n_seg] == rows
 *   add:     suffix [n_seg, count, chans]; out_tokens [rows + n_seg * count, chans]: segment m
 *            followed by suffix[m]; appended rows get weight 1; out_offsets[m] = offsets[m] + m * count
 *   split:   out_tokens [rows - n_seg * count, chans], out_suffix [n_seg, count, chans] = the last
 *            `count` rows of each segment, out_offsets[m] = offsets[m] - m * count.  Every segment
 *            must hold at least `count` rows (the caller checks: it needs the offsets on the host).
 *
 * Stand in for JaggedTokens.add_suffix / split_suffix (src/interface/token_merger.py:23-58, 60-100),
 * which the reference runs as arange / searchsorted / index_copy_ / index_select tensor passes.
 */
int come_jagged_add_suffix(const void *tokens, const float *weight, int dtype, int64_t rows, int64_t chans,
                           const int64_t *offsets, int64_t n_seg, const void *suffix, int64_t count,
                           void *out_tokens, float *out_weight, int64_t *out_offsets, void *stream);
int come_jagged_split_suffix(const void *tokens, const float *weight, int dtype, int64_t rows, int64_t chans,
                             const int64_t *offsets, int64_t n_seg, int64_t count,
                             void *out_tokens, float *out_weight, int64_t *out_offsets, void *out_suffix,
                             void *stream);

#ifdef __cplusplus
}
#endif
#endif /* COME_HIP_H */
