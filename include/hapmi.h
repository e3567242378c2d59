/*
 * libhapmi -- flat C ABI of the MI355X (gfx950) kernels that execute one
 * device's shard of a HAP SPMD program.
 *
 * The reference (alibaba/hap) has no native kernels and no FFI for this path:
 * its emitted torch.fx graph calls PyTorch ops (cuBLAS/cuDNN below them) and
 * collectives.py.  Each entry point below therefore cites the reference NODE
 * FORM (the call the synthesizer emits, /root/reference/hap.rs) or the
 * Python function (/root/reference/collectives.py, models.py) it replaces.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *     the caller owns all memory, nothing is allocated or freed here;
 *   - all work is enqueued on `stream` (a hipStream_t passed as void*); no
 *     entry point synchronises with the host;
 *   - return value 0 = success, negative = HAPMI_E* code; hapmi_last_error()
 *     returns a thread-local message for the last failure;
 *   - tensors are row-major and contiguous unless a leading dimension (ld*)
 *     or stride is given; `dtype` is HAPMI_F32 or HAPMI_BF16.
 */
#ifndef HAPMI_H
#define HAPMI_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *hapmi_stream_t;

enum { HAPMI_F32 = 0, HAPMI_BF16 = 1 };
enum { HAPMI_ACT_NONE = 0, HAPMI_ACT_RELU = 1, HAPMI_ACT_GELU = 2, HAPMI_ACT_SIGMOID = 3 };
enum {
    HAPMI_OK = 0,
    HAPMI_EINVAL = -1,   /* bad shape / argument            */
    HAPMI_EALIGN = -2,   /* pointer or stride not aligned   */
    HAPMI_EARCH = -3,    /* device is not gfx950            */
    HAPMI_ELAUNCH = -4,  /* HIP reported a launch error     */
    HAPMI_ELIMIT = -5    /* size beyond a documented limit  */
};
#define HAPMI_MAX_RANKS 64

/* ---- host side -------------------------------------------------------
 * hapmi_init: once per process and per device, with that device current: checks that it is gfx950 and looks up the
 * device's copy of the scratch array that hapmi_sumsq_static uses. */
int hapmi_init(void);
const char *hapmi_last_error(void);
int hapmi_version(void);

/* hap.rs:3536-3559 sharding_round (exported to Python at hap.rs:211-218):
 * integer shard lengths for `full_length` units under `ratios`. Host only. */
int hapmi_sharding_round(int64_t full_length, const double *ratios_host, int64_t n_ranks,
                         int64_t *lengths_host);

/* ---- uneven-collective local halves (collectives.py) ------------------
 * A tensor is seen as [outer, len, inner] with the sharded dimension in the
 * middle; `inner_bytes` = inner * element size.                           */

/* collectives.py:9-12 padded(): dst[outer, padded_len, inner] <- src[outer, len, inner];
 * the tail rows are left untouched (the reference leaves them uninitialised). */
int hapmi_pad_rows(const void *src, void *dst, int64_t outer, int64_t len, int64_t padded_len,
                   int64_t inner_bytes, hapmi_stream_t stream);

/* collectives.py:20 / :102: cut the pad off W padded slices [outer, padded_len, inner]
 * and concatenate them along the sharded dimension into dst[outer, sum(lengths), inner].  A slice that already lies at its place in dst (outer = 1 and
 * slices[i] == dst + offset of shard i) is left where it is. */
int hapmi_unpad_concat(const void *const *slices_host, const int64_t *lengths_host, int n_ranks, void *dst,
                       int64_t outer, int64_t padded_len, int64_t inner_bytes, hapmi_stream_t stream);

/* collectives.py:24-25 / :92-93: split src[outer, sum(lengths), inner] along the
 * sharded dimension and pad every piece into its own [outer, padded_len, inner] buffer.  A NULL slice is skipped. */
int hapmi_split_pad(const void *src, void *const *slices_host, const int64_t *lengths_host, int n_ranks,
                    int64_t outer, int64_t padded_len, int64_t inner_bytes, hapmi_stream_t stream);

/* collectives.py:146-148 dynamic_slice, and the slice-off-pad of :28 / :96:
 * dst[outer, len, inner] <- src[outer, src_len, inner][:, offset:offset+len, :]. */
int hapmi_slice_rows(const void *src, void *dst, int64_t outer, int64_t src_len, int64_t offset, int64_t len,
                     int64_t inner_bytes, hapmi_stream_t stream);

/* inverse of hapmi_slice_rows: dst[:, offset:offset+len, :] <- src (rest of dst untouched). */
int hapmi_place_rows(const void *src, void *dst, int64_t outer, int64_t dst_len, int64_t offset, int64_t len,
                     int64_t inner_bytes, hapmi_stream_t stream);

/* collectives.py:156-158 / :163-165: split src[outer, sum(lengths), inner] into W
 * contiguous unpadded pieces (the all_to_all send buffers). */
int hapmi_split_rows(const void *src, void *const *pieces_host, const int64_t *lengths_host, int n_ranks,
                     int64_t outer, int64_t inner_bytes, hapmi_stream_t stream);

/* hapmi_split_rows of src * (fwd_out > 0), fwd_out having src's shape and dtype: the backward of a relu whose
 * only reader's gradient goes straight into an all_to_all (the FFN's F.relu -- the default activation of the
 * nn.TransformerEncoderLayer built at models.py:74, emitted at hap.rs:1417 -- behind collectives.py:156-165 in
 * the column-sharded FFN), without a separate pass over the gradient.  Every piece, src and fwd_out 16-byte aligned
 * with inner_bytes * lengths a multiple of 16. */
int hapmi_split_rows_relu_bwd(const void *src, const void *fwd_out, void *const *pieces_host,
                              const int64_t *lengths_host, int n_ranks, int64_t outer, int64_t inner_bytes,
                              int dtype, hapmi_stream_t stream);
/* The same with the kept elements multiplied by `scale`: the backward of F.relu followed by F.dropout(p)
 * (hap.rs:1417, 1464; the FFN's activation and the dropout behind it: `self.dropout` in `_ff_block` of torch's
 * nn.TransformerEncoderLayer, torch:nn/modules/transformer.py:981, which models.py:74, 100 build), given the DROPPED forward
 * output as fwd_out -- it is positive exactly where relu passed the element and dropout kept it -- and
 * scale = 1 / (1 - p); no random numbers are needed backward. */
int hapmi_split_rows_relu_bwd_scaled(const void *src, const void *fwd_out, void *const *pieces_host,
                                     const int64_t *lengths_host, int n_ranks, int64_t outer, int64_t inner_bytes,
                                     float scale, int dtype, hapmi_stream_t stream);

/* collectives.py:159 / :166: concatenate W contiguous pieces [outer, lengths[i], inner]
 * into dst[outer, sum(lengths), inner]; `act` != NONE applies the activation to
 * every element on the way (dtype needed then).  A piece that already lies at its place in dst
 * (act = NONE, outer = 1 and pieces[i] == dst + offset of piece i) is left where it is. */
int hapmi_concat_rows(const void *const *pieces_host, const int64_t *lengths_host, int n_ranks, void *dst,
                      int64_t outer, int64_t inner_bytes, int act, int dtype, hapmi_stream_t stream);
/* hapmi_concat_rows with F.relu and then F.dropout(p) (hap.rs:1417, 1464) applied on the way: dst =
 * dropout(relu(cat(pieces))), with the keep decisions hapmi_dropout takes for dst as a whole under the same p,
 * RNG state and stream id.  Pieces and dst 16-byte aligned with inner_bytes * lengths a multiple of 16. */
int hapmi_concat_rows_relu_dropout(const void *const *pieces_host, const int64_t *lengths_host, int n_ranks, void *dst,
                                   int64_t outer, int64_t inner_bytes, float p, const int64_t *rng_state_dev,
                                   int64_t stream_id, int dtype, hapmi_stream_t stream);
/* The same without concatenating, for a linear that reads the pieces of an all_to_all where they lie (A_segments of
 * hapmi_gemm): dst[i][rows, widths[i]] = the columns of dropout(relu(cat(src, dim 1))) that piece i holds, every
 * piece contiguous; the keep decisions are those hapmi_dropout takes for the [rows, sum(widths)] tensor as a whole.
 * dst[i] may be src[i].  Pieces 16-byte aligned, widths * element size multiples of 16. */
int hapmi_relu_dropout_pieces(const void *const *src_host, void *const *dst_host, const int64_t *widths_host,
                              int n_pieces, int64_t rows, float p, const int64_t *rng_state_dev, int64_t stream_id,
                              int dtype, hapmi_stream_t stream);

/* the local sum of dist.reduce_scatter / dist.all_reduce (collectives.py:27, :95, :77):
 * dst[outer, len, inner] = sum_w contribs[w][outer, src_len, inner][:, offset:offset+len, :]
 * accumulated in float32 in rank order. */
int hapmi_ragged_reduce(const void *const *contribs_host, int n_ranks, void *dst, int64_t outer, int64_t src_len,
                        int64_t offset, int64_t len, int64_t inner, int dtype, hapmi_stream_t stream);

/* hapmi_ragged_reduce with one more term, added last: dst = addend + sum_w contribs[w][...]; addend has dst's
 * layout and may be dst itself.  The gradient that all_gather's backward (AllGather.backward, collectives.py:22-29) contributes
 * to a value that already holds a gradient from another consumer, in one pass. */
int hapmi_ragged_reduce_add(const void *const *contribs_host, int n_ranks, void *dst, const void *addend,
                            int64_t outer, int64_t src_len, int64_t offset, int64_t len, int64_t inner, int dtype,
                            hapmi_stream_t stream);

/* The same sum for several output shards in ONE launch (every rank's piece of a reduce_scatter when the
 * ranks' tensors share one device): dsts[r][outer, lengths[r], inner] = sum_w contribs[w][:, offsets[r]:offsets[r]+lengths[r], :]. */
int hapmi_ragged_reduce_multi(const void *const *contribs_host, int n_ranks, void *const *dsts_host,
                              const int64_t *offsets_host, const int64_t *lengths_host, int n_outputs, int64_t outer,
                              int64_t src_len, int64_t inner, int dtype, hapmi_stream_t stream);

/* collectives.py:9-12 padded() for several shards in ONE launch: dsts[i][outer, padded_len, inner] <- srcs[i][outer, lengths[i], inner]. */
int hapmi_pad_rows_multi(const void *const *srcs_host, void *const *dsts_host, const int64_t *lengths_host, int n_shards,
                         int64_t outer, int64_t padded_len, int64_t inner_bytes, hapmi_stream_t stream);

/* ---- GEMM: F.linear (hap.rs:1032) and the expert einsums (hap.rs:2273) --
 * C[z] = op(A[z]) * op(B[z]) (+ bias[N]) (act) (+ C[z] if accumulate)
 * op(A) is [M,K]: transA=0 -> A stored [M,K] (lda), transA=1 -> A stored [K,M];
 * op(B) is [K,N]: transB=0 -> B stored [K,N] (ldb), transB=1 -> B stored [N,K].
 * z = z1 * batch2 + z2 addresses X + z1*strideX1 + z2*strideX2 (elements).
 * Accumulation is float32; in/out element types are given separately. */
/* An operand or result that exists as SEGMENTS along one of its dimensions instead of as one matrix: the pieces an
 * all_to_all delivers, which collectives.py:159 / :166 would first concatenate (torch.cat) into one tensor.
 * Segment s covers the index range [begin[s], begin[s + 1]) of the segmented dimension and is a row-major matrix
 * [rows, begin[s + 1] - begin[s]] at base[s] with leading dimension ld[s]; begin[0] = 0, begin[n] = the full extent. */
#define HAPMI_GEMM_MAX_SEGMENTS 8
typedef struct {
    int n;                                           /* 1 .. HAPMI_GEMM_MAX_SEGMENTS */
    int64_t begin[HAPMI_GEMM_MAX_SEGMENTS + 1];
    int64_t ld[HAPMI_GEMM_MAX_SEGMENTS];
    const void *base[HAPMI_GEMM_MAX_SEGMENTS];
} hapmi_gemm_segments;

typedef struct {
    const void *A, *B;
    void *C;
    const void *bias;            /* float32[N] or NULL */
    int64_t M, N, K;
    int64_t lda, ldb, ldc;
    int transA, transB;
    int in_dtype, out_dtype;
    int accumulate;              /* 1: C += result (C read in out_dtype) */
    int act;
    float alpha;                 /* result scaled before bias */
    int64_t batch1, batch2;      /* >= 1 */
    int64_t strideA1, strideA2, strideB1, strideB2, strideC1, strideC2;
    void *workspace;             /* optional float32 scratch (16-byte aligned) or NULL: partial sums of a split    */
    int64_t workspace_bytes;     /* reduction (M * roundup(N, 4) * 4 bytes per split; no split when batch > 1), and,
                                  * with a_rowsum / a_rowsum_list, partial row sums in its second half (at most
                                  * batch * 32 * ceil(N / 64) * M * 4 bytes; HAPMI_ELIMIT if they do not fit)        */
    float *a_rowsum;             /* optional: a_rowsum[m] += sum over k of op(A)[m, k]: the bias gradient of F.linear
                                  * when the call is the weight gradient dW = dY^T X, i.e. the column sum that
                                  * autograd takes of dY (hap.rs:1032 F.linear with bias).  The blocks write partial
                                  * sums to the workspace and a second kernel adds them in a fixed order (no atomics:
                                  * the same call gives the same bits every time).  Needs transA = 1, batch 1 and a
                                  * workspace; NULL = off */
    const void *c_relu_mask;     /* optional: [M][ldc] in out_dtype; elements of the result (before accumulation)
                                  * whose mask value is <= 0 are written as 0: the backward of F.relu
                                  * (hap.rs:1417) when the call is the data gradient of the next F.linear and
                                  * the mask is relu's output.  With a batch, problem z's mask lies at C's batch
                                  * offsets from this pointer; NULL = off */
    const void *c_addend;        /* optional, with accumulate = 1: the result is added to c_addend[M][ldc] (out_dtype)
                                  * instead of C's old content, and C is only written: a gradient contribution
                                  * added to a buffer that other launches still read.  Needs batch 1; NULL = off */
    /* Several problems of one shape behind arbitrary pointers in ONE launch (the same linear's weight gradient
     * for a run of layers: each is too small to fill the chip without splitting K, together they are not):
     * host arrays of batch1 device pointers (batch1 <= HAPMI_GEMM_MAX_LIST, batch2 = 1); problem z uses
     * A_list[z], B_list[z], C_list[z] and, if a_rowsum_list is given, a_rowsum_list[z] (entries may be NULL).
     * A, B, C, the batch strides, a_rowsum, c_relu_mask and c_addend must be NULL / 0 then.  NULL = off */
    const void *const *A_list, *const *B_list;
    void *const *C_list;
    float *const *a_rowsum_list;
    /* Segmented operands (bf16 operands, NULL = off).  They let the linear behind an all_to_all (hap.rs:2713-2744,
     * then F.relu hap.rs:1417, then F.linear hap.rs:1032) read the received pieces where they were received, with
     * relu applied as the operand is loaded, and let its backward write the pieces of the backward all_to_all
     * directly, so no concatenating / splitting copy runs on either side:
     *   A_segments    A stored [M, K] (transA = 0) in pieces along K (begin: multiples of 64; K a multiple of 64,
     *                 transB = 1, batch 1, no split); A itself is ignored.  The forward of that linear.
     *   B_segments    B stored [K, N] (transB = 0) in pieces along N; B is ignored.  With pointer lists,
     *                 B_segments_list[z] describes problem z (all with the same n, begin and ld).  Its weight gradient.
     *   C_segments    C in pieces along N; C is ignored; c_mask_segments: c_relu_mask in pieces with the same n,
     *                 begin and ld (piece s of the mask has the layout of piece s of the result).  No accumulate / c_addend.  Its data gradient, written as the backward pieces.
     *   a_relu / b_relu   max(., 0) applied to op(A) (with A_segments) / op(B) (with transA = 1, transB = 0) on load.
     * A block tile must not straddle a piece: the tile configuration is chosen among those whose N extent divides
     * every begin of B_segments / C_segments (HAPMI_EINVAL if none does). */
    const hapmi_gemm_segments *A_segments, *B_segments, *C_segments, *c_mask_segments;
    const hapmi_gemm_segments *const *B_segments_list;
    int a_relu, b_relu;
    /* F.dropout(., p) behind the activation (hap.rs:1464 after 1417: the dropout that follows the FFN's activation,
     * torch:nn/modules/transformer.py:981 in the layers built at models.py:74, 100), applied by the epilogue with the decisions hapmi_dropout takes for C as a whole under the same
     * p, RNG state and stream id.  One contiguous problem (transA = 0, transB = 1, batch 1, ldc = N, N even), no
     * accumulate, no pieces; the reduction is not split.  drop_state = NULL: off */
    const int64_t *drop_state;
    int64_t drop_stream_id;
    float drop_p;
} hapmi_gemm_args;
#define HAPMI_GEMM_MAX_LIST 16
int hapmi_gemm(const hapmi_gemm_args *args_host, hapmi_stream_t stream);

/* PROCESS-WIDE STATE.  hapmi_gemm_tuning, the plan table below and hapmi_prof_gemm_* keep state inside the library
 * that every later hapmi_gemm call of the process reads: they are set-up and measurement hooks, not part of a
 * step.  Calling them while another thread launches GEMMs is safe (the table and the instrumentation are locked)
 * but changes what that thread's next call does; every other entry point of this header is stateless and
 * re-entrant (all work goes to the stream passed in, all memory is the caller's).
 *
 * Tuning hook for measurements: force tile configuration `tile_config` (block tile / waves: 0: 128x128 / 2x2,
 * 1: 256x256 / 2x4, 2: 384x192 / 4x2, 3: 192x256 / 2x4, 4: 256x192 / 4x2, 5: 256x128 / 4x2, 6: 128x256 / 2x4,
 * 7: 192x128 / 2x4, 8: 256x128 / 2x2, 9: 128x192 / 4x2, 10: 64x64 / 2x2, 11: 64x128 / 2x2; 5..9 keep three
 * k-tiles in LDS (two in flight); 1..9 take bf16 operands only, 10 and 11 float32 operands only; a configuration
 * that does not fit the call's operand type is ignored; -1 = automatic) and `k_splits` (0 = automatic). */
int hapmi_gemm_tuning(int tile_config, int k_splits);

/* Plan table: pin the tile configuration and K split that hapmi_gemm uses for one problem signature
 * (shape, batch = batch1 * batch2, transposes, element types).  A caller that has timed the candidates on
 * its own operands (hap_amd.ops.autotune_gemm does) stores the winner here; signatures without a plan fall
 * back to the built-in cost model.  tile_config < 0 removes the entry; hapmi_gemm_plan_clear empties the
 * table.  No counterpart in the reference (its GEMMs are cuBLAS calls behind F.linear, hap.rs:1032). */
int hapmi_gemm_plan_set(int64_t M, int64_t N, int64_t K, int64_t batch, int transA, int transB, int in_dtype,
                        int out_dtype, int tile_config, int k_splits);
int hapmi_gemm_plan_clear(void);

/* ---- row-wise kernels ------------------------------------------------- */
/* operator.add + F.layer_norm(x, (width,)) without affine, eps (hap.rs:1515, 1653):
 * y = LN(x + res); res may be NULL; rstd[rows] (float32) is kept for backward. */
int hapmi_add_layernorm_fwd(const void *x, const void *res, void *y, float *rstd, int64_t rows, int64_t width,
                            float eps, int dtype, hapmi_stream_t stream);
/* dx = rstd * (dy - mean(dy) - y * mean(dy * y)) (+ dx_add if not NULL) */
int hapmi_layernorm_bwd(const void *dy, const void *y, const float *rstd, const void *dx_add, void *dx,
                        int64_t rows, int64_t width, int dtype, hapmi_stream_t stream);
/* F.dropout(x, p) -> operator.add(., res) -> F.layer_norm in one pass (hap.rs:1464, 1515, 1653: the residual
 * connections of the encoder layer: dropout1 / dropout2 and norm1 / norm2 of torch's nn.TransformerEncoderLayer,
 * torch:nn/modules/transformer.py:952-956, 977, 982, in the layers built at models.py:74, 100): y = LN(dropout(x) + res).  The keep decisions are those
 * hapmi_dropout takes for x as a whole [rows, width] tensor under the same p, RNG state and stream id.  Backward
 * gives dx (the gradient of the sum: res's) and dx_drop = dropout's backward of dx (x's), regenerating the mask;
 * dx_drop must not alias dx. */
int hapmi_dropout_add_layernorm_fwd(const void *x, const void *res, void *y, float *rstd, int64_t rows, int64_t width,
                                    float eps, float p, const int64_t *rng_state_dev, int64_t stream_id, int dtype,
                                    hapmi_stream_t stream);
int hapmi_layernorm_bwd_dropout(const void *dy, const void *y, const float *rstd, const void *dx_add, void *dx,
                                void *dx_drop, int64_t rows, int64_t width, float p, const int64_t *rng_state_dev,
                                int64_t stream_id, int dtype, hapmi_stream_t stream);

/* softmax over the last dimension of [rows, width] (row stride ld elements, the same for
 * input and output) with an optional additive float32 mask[mask_rows, width] (contiguous;
 * row r uses mask row r % mask_rows), in place allowed:
 * the explicit attention path of torch's multi_head_attention_forward (hap.rs:1301). */
int hapmi_softmax_fwd(const void *x, const float *mask, void *p, int64_t rows, int64_t width, int64_t ld,
                      int64_t mask_rows, int dtype, hapmi_stream_t stream);
/* ds = p * (dp - sum(dp * p)) */
int hapmi_softmax_bwd(const void *dp, const void *p, void *ds, int64_t rows, int64_t width, int64_t ld, int dtype,
                      hapmi_stream_t stream);

/* fused scaled-dot-product attention on packed projections (the explicit baddbmm / softmax / bmm path of
 * F.multi_head_attention_forward, hap.rs:1301-1327; bf16 only, head_dim 64):
 * qkv[b, S, 3*H*64] -> out[b, S, H*64]; lse[b, H, S] float32 (log-sum-exp of every score row) is kept for
 * backward; mask is NULL or an additive float32 [S, S].  causal != 0 (mask must then be NULL) stands for the
 * mask torch.triu(full(-inf), diagonal=1) that the language models register as src_mask (models.py:72, 97): the
 * same result without reading a mask, and the key tiles above the diagonal are skipped.  Backward writes
 * dqkv[b, S, 3*H*64] completely; delta_ws is float32 scratch of b*H*S elements. */
int hapmi_attention_fwd(const void *qkv, const float *mask, int causal, void *out, float *lse, int64_t b, int64_t S,
                        int64_t H, float scale, hapmi_stream_t stream);
int hapmi_attention_bwd(const void *qkv, const void *out, const void *dout, const float *lse, const float *mask,
                        int causal, void *dqkv, float *delta_ws, int64_t b, int64_t S, int64_t H, float scale,
                        hapmi_stream_t stream);

/* The same with dropout of the probabilities (dropout_p > 0 of F.multi_head_attention_forward, hap.rs:1257, 1307:
 * out = dropout(softmax(scores)) V).  The keep decisions are those F.dropout's kernel (hapmi_dropout) takes for the
 * elements of a [b*H, S, row_len] tensor of probabilities (row_len even, >= S) under the same p, RNG state and
 * stream id, so this path and one that materialises the probabilities drop the same entries.
 * hapmi_attention_keep_bits packs them into bit words in the two orders the kernels read them in:
 *   keep_rows: b*H*S*2*ceil(S/64) uint32, read by forward and by backward
 *              (per query: the tile's 64 keys in the lane's accumulator-register order);
 *   keep_cols: the same count, read by backward (per key: one bit per query).
 * Both are 8-byte aligned, written completely for the rows / columns below S, and belong to one (step, stream id):
 * backward must be given the words its forward ran with.  p lies in [0, 1). */
int hapmi_attention_keep_bits(uint32_t *keep_rows, uint32_t *keep_cols, int64_t b, int64_t S, int64_t H,
                              int64_t row_len, float p, const int64_t *rng_state_dev, int64_t stream_id,
                              hapmi_stream_t stream);
int hapmi_attention_fwd_dropout(const void *qkv, const float *mask, int causal, void *out, float *lse, int64_t b,
                                int64_t S, int64_t H, float scale, const uint32_t *keep_rows, float p,
                                hapmi_stream_t stream);
int hapmi_attention_bwd_dropout(const void *qkv, const void *out, const void *dout, const float *lse,
                                const float *mask, int causal, void *dqkv, float *delta_ws, int64_t b, int64_t S,
                                int64_t H, float scale, const uint32_t *keep_rows, const uint32_t *keep_cols, float p,
                                hapmi_stream_t stream);

/* torch.log_softmax + F.nll_loss(reduction='sum', ignore_index) (hap.rs:1829, 1881) and their
 * backward in one pass: row_loss[rows] float32, dlogits = (softmax - onehot) * grad_scale for
 * counted rows and 0 for ignored rows; dlogits may alias logits; rows of both are ld elements apart. */
int hapmi_logsoftmax_nll(const void *logits, const int64_t *targets, int64_t ignore_index, float *row_loss,
                         void *dlogits, int64_t rows, int64_t width, int64_t ld, float grad_scale, int dtype,
                         hapmi_stream_t stream);
/* out[0] = sum of x[0..n) in a fixed order (deterministic) */
int hapmi_sum_f32(const float *x, int64_t n, float *out, hapmi_stream_t stream);

/* ---- elementwise ------------------------------------------------------- */
/* F.relu (hap.rs:1417) / F.gelu / torch.sigmoid (hap.rs:1088) */
int hapmi_act_fwd(const void *x, void *y, int64_t n, int act, int dtype, hapmi_stream_t stream);
/* relu, sigmoid: ref = y (output); gelu: ref = x (input) */
int hapmi_act_bwd(const void *dy, const void *ref, void *dx, int64_t n, int act, int dtype, hapmi_stream_t stream);
/* out = a + b (operator.add, hap.rs:1515; also gradient accumulation) */
int hapmi_add(const void *a, const void *b, void *out, int64_t n, int dtype, hapmi_stream_t stream);
/* out[i] = value: the gradient of torch.sum(x) (hap.rs:1133) with respect to x */
int hapmi_fill_value(void *out, float value, int64_t n, int dtype, hapmi_stream_t stream);
/* out = a * s (operator.mul with a number, hap.rs:1563) */
int hapmi_scale(const void *a, float s, void *out, int64_t n, int dtype, hapmi_stream_t stream);
/* out[r, :] = a[r, :] + b[r % b_rows, :] (broadcast add of pe / pos_embed, hap.rs:3821-3837) */
int hapmi_add_bcast_rows(const void *a, const void *b, void *out, int64_t rows, int64_t b_rows, int64_t width,
                         int dtype, hapmi_stream_t stream);
/* column sums: out[N] (float32) (+)= sum_m x[m, :]; bias gradient of F.linear; also sums over samples.
 * Rows are summed in slabs whose partial sums go to `workspace` (float32, up to ceil(M / 128) * N elements are
 * used; NULL or too small: fewer, longer slabs) and are added in slab order: no atomics, reproducible bits. */
int hapmi_colsum(const void *x, float *out, int64_t M, int64_t N, int64_t ldx, int accumulate, int dtype,
                 float *workspace, int64_t workspace_elems, hapmi_stream_t stream);
int hapmi_fill_zero(void *p, int64_t bytes, hapmi_stream_t stream);
int hapmi_cast(const void *src, int src_dtype, void *dst, int dst_dtype, int64_t n, hapmi_stream_t stream);

/* F.dropout(input, p) as the emitted program calls it, i.e. in training mode (hap.rs:1464; also the dropout of the
 * attention probabilities, hap.rs:1307): y = x * keep / (1 - p), in place allowed.  keep is a counter-based function
 * of (rng_state_dev[0] = seed, rng_state_dev[1] = step, stream_id, element index): nothing is stored, the
 * backward of the node is the same call on the gradient, and hapmi_dropout_mask writes the same decisions as
 * bytes (1 = kept).  stream_id names the dropout node inside a program.  The reference draws from torch's
 * generator instead; the two streams of random numbers cannot be made equal, so results are compared on exported
 * masks and statistically. */
int hapmi_dropout(const void *x, void *y, int64_t n, float p, const int64_t *rng_state_dev, int64_t stream_id,
                  int dtype, hapmi_stream_t stream);
int hapmi_dropout_mask(uint8_t *mask, int64_t n, float p, const int64_t *rng_state_dev, int64_t stream_id,
                       hapmi_stream_t stream);
/* rng_state_dev[1] += 1: once per training step, as a kernel, so that a step replayed from a HIP graph draws new masks */
int hapmi_rng_advance(int64_t *rng_state_dev, hapmi_stream_t stream);

/* F.embedding (hap.rs:2041) fused with `* scale` and `+ pe[S, d]` (models.py:79-81):
 * out[t, :] = table[ids[t], :] * scale + pe[t % S, :]   (pe may be NULL) */
int hapmi_embedding_fwd(const int64_t *ids, const void *table, const void *pe, void *out, int64_t n_tokens,
                        int64_t d, int64_t S, int64_t vocab, float scale, int dtype, hapmi_stream_t stream);
/* dtable[ids[t], :] += dout[t, :] * scale, the tokens of one id added in token order by one wave (no atomics,
 * reproducible bits); dtable zeroed by the caller; d <= 2048 */
int hapmi_embedding_bwd(const int64_t *ids, const void *dout, float *dtable, int64_t n_tokens, int64_t d,
                        int64_t vocab, float scale, int dtype, hapmi_stream_t stream);

/* ---- ViT leaves -------------------------------------------------------- */
/* F.conv2d with kernel = stride, no padding (hap.rs:1723) as patch rows for a GEMM:
 * cols[b * gh * gw, C * ph * pw] <- x[b, C, gh*ph, gw*pw] (float32 in, `dtype` out) */
int hapmi_patchify(const float *x, void *cols, int64_t b, int64_t C, int64_t gh, int64_t gw, int64_t ph,
                   int64_t pw, int dtype, hapmi_stream_t stream);
/* models.append_cls_token (models.py:443-445) fused with `+ pos_embed` (models.py:167):
 * out[b, 0, :] = cls + pos[0]; out[b, 1 + t, :] = patches[b, t, :] + pos[1 + t]; pos may be NULL (the bare
 * append_cls_token) */
int hapmi_append_cls_pos(const void *patches, const void *cls, const void *pos, void *out, int64_t b, int64_t T,
                         int64_t d, int dtype, hapmi_stream_t stream);

/* ---- MoE: models.top_2_gating (models.py:477-502) in index form --------
 * logits[B, S, E] float32 -> probs[B, S, E] float32, index[B, S, 2] int32,
 * slot[B, S, 2] int32 (0 = dropped, usable slots 1..C-1; a choice whose gate is exactly 0
 * counts as dropped, as models.py:500 derives dispatch from combine > 0), gate[B, S, 2] float32,
 * token_of_slot[B, E, C] int32 (-1 = empty). */
int hapmi_top2_gate(const float *logits, float *probs, int32_t *index, int32_t *slot, float *gate,
                    int32_t *token_of_slot, int64_t B, int64_t S, int64_t E, int64_t C, hapmi_stream_t stream);
/* models.switch_gating (models.py:436-437, 452-475; the reference's synthesizer has no handler for it, its
 * single-device models RSwitch / VSwitch call it): the same records with one choice per token -- position
 * = 1-based rank among the earlier tokens of the same expert, kept while < C, combine weight = the softmax
 * probability of the chosen expert.  The second entry of every record is a dropped choice (gate 0, slot 0),
 * so every entry point below takes these records unchanged. */
int hapmi_switch_gate(const float *logits, float *probs, int32_t *index, int32_t *slot, float *gate,
                      int32_t *token_of_slot, int64_t B, int64_t S, int64_t E, int64_t C, hapmi_stream_t stream);
/* dlogits = softmax backward of the two kept gate gradients */
int hapmi_top2_gate_bwd(const float *probs, const int32_t *index, const int32_t *slot, const float *dgate,
                        float *dlogits, int64_t B, int64_t S, int64_t E, hapmi_stream_t stream);
/* dense [B, S, E, C] tensors exactly as models.py:495-500 lays them out */
int hapmi_top2_densify(const int32_t *index, const int32_t *slot, const float *gate, float *dispatch,
                       float *combine, int64_t B, int64_t S, int64_t E, int64_t C, hapmi_stream_t stream);
/* The four MoE einsums (hap.rs:2273, models.py:356-364) on index-form routing.  The device's share of the dense
 * [B, S, E, C] dispatch / combine tensors is a window of experts [e_lo, e_lo + E_loc) (the expert split of the
 * einsums, hap.rs:3312-3316, 3325-3329, 3356-3360, 3393-3397), of capacity slots [c_lo, c_lo + C_loc) (the capacity
 * split, hap.rs:3318-3322, 3349-3353, 3380-3384, 3399-3403) and of positions [s_lo, s_lo + S_loc) (the split along the
 * sequence, hap.rs:3300-3304 for the dispatch): dynamic_slice of the gating outputs along dim 2 / dim 3 / dim 1.
 * Expert-major activations are [E_loc, B, C_loc, d], token tensors (x, out, dout, dx) [B, S_loc, d]; the routing
 * records and dgate always cover all S positions.  The whole tensor is e_lo = c_lo = s_lo = 0, E_loc = E, C_loc = C,
 * S_loc = S.
 *
 * einsum "bsd,bsec->becd" as a row gather into expert_in[E_loc, B, C_loc, d] (zero rows for empty slots and for
 * tokens outside the window of positions: the result is then a partial sum over the devices) */
int hapmi_moe_dispatch(const void *x, const int32_t *token_of_slot, void *expert_in, int64_t B, int64_t S,
                       int64_t E, int64_t C, int64_t d, int64_t e_lo, int64_t E_loc, int64_t c_lo, int64_t C_loc,
                       int64_t s_lo, int64_t S_loc, int dtype, hapmi_stream_t stream);
/* einsum "becd,bsec->bsd" (models.py:364) as a weighted row gather:
 * out[b, s - s_lo, :] = sum_k gate_k * expert_out[e_k - e_lo, b, slot_k - c_lo, :] over kept choices inside the windows */
int hapmi_moe_combine(const void *expert_out, const int32_t *index, const int32_t *slot, const float *gate,
                      void *out, int64_t B, int64_t S, int64_t C, int64_t d, int64_t e_lo, int64_t E_loc,
                      int64_t c_lo, int64_t C_loc, int64_t s_lo, int64_t S_loc, int dtype, hapmi_stream_t stream);
/* backward of combine: d_expert_out[e, b, c, :] = gate * dout[b, token - s_lo, :] (0 for empty slots and tokens outside
 * the window); dgate[b, s, k] = <dout[b, s - s_lo, :], expert_out[e_k - e_lo, b, slot_k - c_lo, :]> (0 if not kept /
 * outside the windows) */
int hapmi_moe_combine_bwd(const void *dout, const void *expert_out, const int32_t *index, const int32_t *slot,
                          const float *gate, const int32_t *token_of_slot, void *d_expert_out, float *dgate,
                          int64_t B, int64_t S, int64_t E, int64_t C, int64_t d, int64_t e_lo, int64_t E_loc,
                          int64_t c_lo, int64_t C_loc, int64_t s_lo, int64_t S_loc, int dtype, hapmi_stream_t stream);
/* backward of dispatch: dx[b, s - s_lo, :] (+)= sum_k d_expert_in[e_k - e_lo, b, slot_k - c_lo, :] */
int hapmi_moe_dispatch_bwd(const void *d_expert_in, const int32_t *index, const int32_t *slot, const float *gate,
                           void *dx, int64_t B, int64_t S, int64_t C, int64_t d, int64_t e_lo, int64_t E_loc,
                           int64_t c_lo, int64_t C_loc, int64_t s_lo, int64_t S_loc, int accumulate, int dtype,
                           hapmi_stream_t stream);

/* ---- optimizer (worker.py:47, 74-76; profiler.py:18) --------------------
 * Flat float32 master parameters and gradients; `shadow` (bf16 copy of the
 * updated parameters) may be NULL; `grad_scale_dev` (device float, e.g. the
 * clipping coefficient) may be NULL. */
int hapmi_sgd_step(float *param, const float *grad, void *shadow, int64_t n, float lr,
                   const float *grad_scale_dev, hapmi_stream_t stream);
int hapmi_adam_step(float *param, const float *grad, float *exp_avg, float *exp_avg_sq, void *shadow, int64_t n,
                    float lr, float beta1, float beta2, float eps, float bias_corr1, float bias_corr2,
                    const float *grad_scale_dev, hapmi_stream_t stream);
/* The same update with the step count and bias corrections held on the device: state_dev[0..2] = {step,
 * 1 - beta1^step, 1 - beta2^step} (zero-initialised by the caller) is advanced by one and then used, so the
 * call can be captured in a HIP graph and replayed. */
int hapmi_adam_step_dev(float *param, const float *grad, float *exp_avg, float *exp_avg_sq, void *shadow, int64_t n,
                        float lr, float beta1, float beta2, float eps, float *state_dev,
                        const float *grad_scale_dev, hapmi_stream_t stream);
/* The two halves of hapmi_adam_step_dev, for a caller that updates the parameters in several pieces per step
 * (e.g. each piece as soon as its gradients are final, on another stream): hapmi_adam_advance advances
 * state_dev once per step, hapmi_adam_apply_dev applies the update to one piece with the state as it is. */
int hapmi_adam_advance(float *state_dev, float beta1, float beta2, hapmi_stream_t stream);
int hapmi_adam_apply_dev(float *param, const float *grad, float *exp_avg, float *exp_avg_sq, void *shadow, int64_t n,
                         float lr, float beta1, float beta2, float eps, const float *state_dev,
                         const float *grad_scale_dev, hapmi_stream_t stream);
/* out[0] = sum g^2, the square of the norm that torch.nn.utils.clip_grad_norm_ takes (worker.py:74), in two
 * stages through `workspace` (the number of floats that hapmi_sumsq_workspace_elems reports for n: one partial sum per 16384 elements, added in
 * order by one block): no atomics, reproducible bits */
int hapmi_sumsq_workspace_elems(int64_t n, int64_t *elems_host);
int hapmi_sumsq(const float *g, int64_t n, float *out, float *workspace, int64_t workspace_elems,
                hapmi_stream_t stream);
/* hapmi_sumsq without a workspace argument and without any allocation.  No counterpart in the reference; it is for
 * callers that cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses that
 * forbid it.  The partial sums go to a 256 KiB array inside the library's device code (each GPU the library runs
 * on holds its copy until the process ends), so n is limited to 2^30 elements (HAPMI_ELIMIT beyond).  Calls that
 * overlap on one GPU (different streams) share that array and race; calls on one stream are ordered and give the
 * bits of hapmi_sumsq.  The array used is that of the stream's device (the current device for the null stream);
 * hapmi_init() must have run with that device current (HAPMI_EINVAL otherwise), so that this call is nothing but
 * kernel launches on `stream` and may be recorded by a stream capture. */
int hapmi_sumsq_static(const float *g, int64_t n, float *out, hapmi_stream_t stream);
/* torch.nn.utils.clip_grad_norm_ coefficient (worker.py:74): coef = min(1, max_norm / (sqrt(sumsq) + 1e-6)) */
int hapmi_clip_coef(const float *sumsq, float max_norm, float *coef, hapmi_stream_t stream);

/* ---- instrumentation ---------------------------------------------------
 * When enabled, every hapmi_gemm call is bracketed by HIP events on its own stream, followed by an empty bracket
 * (two event records with nothing between them).  hapmi_prof_gemm_collect synchronises those events and returns,
 * since enable: the summed bracket time around the calls (ms), the summed time of the empty brackets (ms: what
 * the event records themselves add to a bracket; NULL = not wanted), the call count and the algorithmic FLOPs. */
int hapmi_prof_gemm_enable(int on);
int hapmi_prof_gemm_collect(double *ms_host, int64_t *launches_host, double *flops_host, double *empty_ms_host);

#ifdef __cplusplus
}
#endif
#endif /* HAPMI_H */
