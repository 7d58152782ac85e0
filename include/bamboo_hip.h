/* bamboo_hip.h -- C ABI of libbamboo_hip.so, the gfx950 (MI355X) kernel library under
 * one Bamboo pipeline stage.
 *
 * Conventions (every entry point):
 *   - returns 0 on success, a negative BB_E* code otherwise; never throws, never exits.
 *     bb_last_error() gives a thread-local human-readable message for the last failure.
 *   - all data pointers are DEVICE pointers owned by the caller (any allocator), 16-byte
 *     aligned, row-major; leading dimensions and strides are in ELEMENTS.
 *   - `stream` is a hipStream_t passed as void*; work is stream-ordered, no hidden
 *     synchronisation, no allocation (workspaces are caller-provided).
 *   - results are deterministic: no atomics in reductions, partial sums (split contractions,
 *     per-block partials) added in a fixed order, so running the same call twice on the same
 *     inputs gives bit-identical outputs (this is what makes the redundant forward of shadow
 *     layers bit-exact with the normal forward).
 *   - dtype codes: BB_F32 = 0, BB_BF16 = 1.
 *
 * The reference has exactly one native entry point on this path, the torch extension
 *   multi_tensor_adam(chunk_size, noop_flag, [[g],[p],[m],[v]], lr, b1, b2, eps, step, mode,
 *                     bias_correction, wd)   (csrc/adam/fused_adam_frontend.cpp:3-20);
 * bb_adam_multi replaces it.  All other layer arithmetic of the reference runs through
 * ATen operators called from Python (DeepSpeedExamples/pipeline_parallelism/transformer.py:77-172,
 * resnet.py:49-75); each entry point below names the call site it stands in for.
 */
#ifndef BAMBOO_HIP_H
#define BAMBOO_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BB_F32 0
#define BB_BF16 1

#define BB_OK 0
#define BB_EINVAL (-1)  /* bad argument / unsupported shape */
#define BB_EHIP (-2)    /* a HIP runtime call failed */
#define BB_ENOSPC (-3)  /* caller workspace too small */

/* GEMM operand layouts (row-major storage):
 *   BB_NT  C[M,N] = A[M,K] * B[N,K]^T   y = x W^T        (nn.Linear forward, Q K^T, dctx V^T)
 *   BB_NN  C[M,N] = A[M,K] * B[K,N]     dx = dy W        (linear dgrad, P V, dS K)
 *   BB_TN  C[M,N] = A[K,M]^T * B[K,N]   dW = dy^T x      (linear wgrad, P^T dctx, dS^T Q)   */
#define BB_NT 0
#define BB_NN 1
#define BB_TN 2

/* GEMM epilogues, applied to v = alpha * acc (+ bias[n] if bias != NULL):
 *   BB_EPI_NONE      C = v
 *   BB_EPI_ACT       aux_out = v (if aux_out != NULL);  C = act(v)
 *   BB_EPI_DACT      C = v * act'(aux_in[m,n])
 *   BB_EPI_RESIDUAL  C = v + resid[m,n]
 *   BB_EPI_MUL       C = v * aux_in[m,n]  (e.g. aux_in = act'(u) kept by BB_EPI_ACT_DACT or bb_act_fwd)
 *   BB_EPI_ACT_DACT  aux_out = act'(v);  C = act(v)   (forward of an FFN whose backward then needs no
 *                    transcendental: its input gradient is a BB_EPI_MUL product with aux_out)
 *   BB_EPI_MUL_POS   C = v (+ resid[m,n] if resid != NULL) where aux_in[m,n] > 0, else 0  (input gradient through a
 *                    ReLU whose OUTPUT was kept: relu'(u) = [relu(u) > 0], so the forward stores nothing beside
 *                    its output; a dropout factor 1/(1-p) on that output goes into alpha; with resid: the
 *                    gradient that meets a skip connection's before it passes the ReLU of the block in front)
 * `accumulate` != 0 adds the result to the existing contents of C (C must be fp32).       */
#define BB_EPI_NONE 0
#define BB_EPI_ACT 1
#define BB_EPI_DACT 2
#define BB_EPI_RESIDUAL 3
#define BB_EPI_MUL 4
#define BB_EPI_ACT_DACT 5
#define BB_EPI_MUL_POS 6

#define BB_ACT_RELU 0
#define BB_ACT_GELU_TANH 1

/* attention / softmax mask kinds (reference hook: scores.masked_fill(mask == 0, -1e9),
 * transformer.py:122-123) */
#define BB_MASK_NONE 0
#define BB_MASK_CAUSAL 1      /* keep col <= row */
#define BB_MASK_KEY_PADDING 2 /* keep col < key_len[batch] */

/* LayerNorm flavours */
#define BB_LN_STANDARD 0  /* (x-mean) * rsqrt(var_biased + eps) */
#define BB_LN_ANNOTATED 1 /* (x-mean) / (std_unbiased + eps), transformer.py:77-88 */

typedef struct bb_gemm_desc {
    int32_t layout;     /* BB_NT / BB_NN / BB_TN */
    int32_t dtype;      /* dtype of A, B, bias, aux, resid (BB_F32 / BB_BF16) */
    int32_t c_dtype;    /* dtype of C (same as dtype, or BB_F32) */
    int32_t M, N, K;
    const void* A; int64_t lda;
    const void* B; int64_t ldb;
    void* C; int64_t ldc;
    /* batching: grid z = nb1 * nb2, operand offset = i1 * s?1 + i2 * s?2 (elements) */
    int32_t nb1, nb2;
    int64_t sA1, sA2, sB1, sB2, sC1, sC2;
    float alpha;
    int32_t epilogue;   /* BB_EPI_* */
    int32_t act;        /* BB_ACT_* */
    int32_t accumulate; /* C += ... (c_dtype must be BB_F32) */
    const void* bias;   /* [N] or NULL */
    const void* aux_in; /* [M,N], leading dim ldaux, batch strides as C */
    void* aux_out;      /* [M,N], leading dim ldaux */
    const void* resid;  /* [M,N], leading dim ldaux */
    int64_t ldaux;
    /* BB_TN only: colsum_out[m] += sum_k A[k,m] (fp32, [M]) -- with A = dy this is the bias gradient
     * of the linear layer whose weight gradient the GEMM computes.  Fused into the GEMM where the
     * kernel allows; otherwise computed by bb_colsum_acc with colsum_ws (>= bb_colsum_workspace(M)
     * floats, may be NULL only if the fused path is certain).  Same result either way up to the
     * fp32 summation order.                                                                */
    float* colsum_out;
    float* colsum_ws;
    /* BB_TN, bf16, unbatched only: with conv_c > 0, B is not a matrix in memory but the 3x3 / pad 1 patch
     * matrix [K pixels, N = 9 * conv_c] of the NHWC tensor at B ([pixels, conv_c], images of conv_h x conv_w;
     * column tap * conv_c + c of row p = the tensor at pixel p + shift(tap), zero outside the image), gathered
     * by the operand loader: with A = dy this is the weight gradient of nn.Conv2d(k=3, padding=1)
     * (resnet.py:58) in [out, 3, 3, in] order.  ldb is ignored; conv_c % 128 == 0; K % 32 == 0; B points at
     * pixel 0 of the tensor and the K rows of the problem are its pixels conv_row0 .. conv_row0 + K - 1 (A's
     * rows start at A as usual).  All four zero: an ordinary B.                                        */
    int32_t conv_h, conv_w, conv_c, conv_row0;
    /* bb_gemm only, where bb_gemm_strip_stats_supported() says so: the kernel also leaves, per strip of 32
     * consecutive rows of C and per column, the triple (pivot = the strip's first row, sum (c - pivot),
     * sum (c - pivot)^2) of the stored bf16 values: strip_stats[(strip * 3 + j) * N + n], fp32,
     * >= bb_strip_stats_workspace(M, N) floats.  bb_batchnorm_fwd_strips turns them into the batch statistics
     * of nn.BatchNorm2d without reading C again (resnet.py:55-62: every convolution feeds a BatchNorm).    */
    float* strip_stats;
    /* Dropout on the product, after bias and activation and before the residual is added
     * (nn.Dropout of SublayerConnection and PositionwiseFeedForward, transformer.py:98-103,154-158):
     * element (m, n) is kept and scaled by 1 / (1 - dropout_p) when bb_dropout_keep(key, m * N + n) says so
     * (the decision function of bb_dropout_apply), else zero; with BB_EPI_ACT_DACT the stored derivative gets
     * the same factor.  dropout_p = 0: none.  Not with BB_EPI_DACT / BB_EPI_MUL / BB_EPI_MUL_POS, not batched.            */
    float dropout_p;
    uint32_t dropout_k0, dropout_k1;
} bb_gemm_desc;

/* library ------------------------------------------------------------------------------ */
int bb_version(void);
const char* bb_last_error(void);
/* Device name check: fails with BB_EHIP when the current device is not a gfx950 part.    */
int bb_init(void);

/* GEMM (MFMA, LDS-tiled).  Stands in for every F.linear / torch.matmul call of the reference
 * layer (transformer.py:121,127,136-146,158) and for their autograd backward
 * (engine.py:1701-1709 torch.autograd.backward).  bf16 needs K, lda, ldb, ldc % 8 == 0;
 * fp32 needs them % 4 == 0.                                                               */
int bb_gemm(const bb_gemm_desc* desc, void* stream);
int bb_gemm_strip_stats_supported(const bb_gemm_desc* desc);
int64_t bb_strip_stats_workspace(int rows, int cols);
/* `count` independent GEMMs of one layout/dtype; results are identical to calling bb_gemm on
 * each descriptor in turn.  When all are unbatched bf16 problems they share one launch, which
 * is how the four weight-gradient products of a layer (autograd of transformer.py:136-146,158)
 * fill the GPU although each has few output tiles.                                         */
int bb_gemm_grouped(const bb_gemm_desc* descs, int count, void* stream);
/* bb_gemm_grouped for problems with an fp32 C, few output tiles and a long contraction (weight
 * gradients dW += dy^T x of narrow layers, e.g. the three convolutions of resnet.py:49-75 over
 * K = N*H*W rows): the contraction is cut into chunks that run as problems of their own into fp32
 * partial products in `workspace` (>= bb_gemm_splitk_workspace(descs, count) bytes, 16-byte
 * aligned), then added to C in chunk order -- deterministic, and equal to bb_gemm_grouped up to
 * the fp32 summation order.  Falls back to bb_gemm_grouped when cutting does not pay.          */
int64_t bb_gemm_splitk_workspace(const bb_gemm_desc* descs, int count);
int bb_gemm_grouped_splitk(const bb_gemm_desc* descs, int count, void* workspace,
                           int64_t workspace_bytes, void* stream);
/* Name of the kernel variant bb_gemm would launch for this descriptor ("bf16_nt_256x256", ...),
 * written NUL-terminated into out; for correlating launches with profiler output.        */
int bb_gemm_variant(const bb_gemm_desc* desc, char* out, int out_len);

/* LayerNorm over the last dimension (transformer.py:77-88 custom LayerNorm, or the standard
 * one).  x, y: [rows, cols] of `dtype`; gain, shift: [cols] of `dtype`; mean, rinv: [rows]
 * fp32 saved for backward (rinv = 1/(std+eps) or rsqrt(var+eps)).  cols <= 8192.          */
int bb_layernorm_fwd(int dtype, int kind, int rows, int cols, float eps, const void* x,
                     const void* gain, const void* shift, void* y, float* mean, float* rinv,
                     void* stream);
/* Backward: dx = dLN(dy) (+ dres if dres != NULL, the residual branch's gradient);
 * dgain/dshift (fp32, [cols]) are ACCUMULATED.  workspace: fp32, at least
 * bb_layernorm_bwd_workspace(cols) elements.                                              */
int64_t bb_layernorm_bwd_workspace(int cols);
int bb_layernorm_bwd(int dtype, int kind, int rows, int cols, float eps, const void* x,
                     const void* gain, const float* mean, const float* rinv, const void* dy,
                     const void* dres, void* dx, float* dgain, float* dshift,
                     float* workspace, void* stream);
/* The same without a workspace, for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * per-block partial sums live in an array inside the library's device image (4 MiB per GPU, held until
 * the process ends); the call allocates nothing.  cols <= BB_LN_BWD_STATIC_MAX_COLS, else BB_EINVAL.
 * All calls on one GPU share that array: calls that overlap in time on one GPU (two streams, two
 * threads) race; calls on one stream are ordered and independent (nothing of an earlier call's contents
 * is read).  bb_init() on a device completes the one-time set-up; otherwise the first call on that
 * device does (do not make that first call under stream capture).                                  */
#define BB_LN_BWD_STATIC_MAX_COLS 2048
int bb_layernorm_bwd_static(int dtype, int kind, int rows, int cols, float eps, const void* x,
                            const void* gain, const float* mean, const float* rinv, const void* dy,
                            const void* dres, void* dx, float* dgain, float* dshift, void* stream);

/* Sum over the last dimension and its backward: y[r] = sum_c x[r, c]; dx[r, c] = dy[r]
 * (the ``lambda x: x.sum(-1)`` tail layer of transformer.py:250 and its autograd).
 * x, dx: [rows, cols]; y, dy: [rows], all of `dtype`.                                      */
int bb_rowsum_fwd(int dtype, int rows, int cols, const void* x, void* y, void* stream);
int bb_rowsum_bwd(int dtype, int rows, int cols, const void* dy, void* dx, void* stream);

/* dst[i] = src[i] / (1 - p) where element i is kept, else 0 (F.dropout in training mode with the mask of
 * key (k0, k1)): i counts the n elements of a contiguous tensor.  The decision for element i is a pure
 * function of (k0, k1, i) -- see bb_dropout_keep_host -- shared by the GEMM epilogues (i = m * N + n) and the
 * attention kernels (i = ((batch * heads + head) * seq + query) * seq + key).  src == dst allowed.
 * The backward of dropout is the same call on the gradient.                                         */
int bb_dropout_apply(int dtype, int64_t n, const void* src, void* dst, float p, uint32_t k0, uint32_t k1,
                     void* stream);
/* The decision itself, on the host (1 = keep): for tests and for callers that need the mask. */
int bb_dropout_keep_host(float p, uint32_t k0, uint32_t k1, uint64_t index);

/* Column sums of a [rows, cols] matrix accumulated into an fp32 vector: the bias gradient of
 * nn.Linear (autograd of transformer.py:136-146,158).  workspace: fp32, at least
 * bb_colsum_workspace(cols) elements.                                                     */
int64_t bb_colsum_workspace(int cols);
int bb_colsum_acc(int dtype, int rows, int cols, const void* x, int64_t ldx, float* out,
                  float* workspace, void* stream);

/* Masked softmax over the last dimension, in place (transformer.py:121-124).
 * s: [batch, heads, sq, sk] contiguous of `dtype`; key_len: int32 [batch] for
 * BB_MASK_KEY_PADDING.  Masked scores are replaced by -1e9 before the softmax.            */
int bb_softmax_fwd(int dtype, int mask, int batch, int heads, int sq, int sk, void* s,
                   const int32_t* key_len, void* stream);
/* In place on dp: dp <- p * (dp - sum_j dp*p).                                            */
int bb_softmax_bwd(int dtype, int batch, int heads, int sq, int sk, const void* p, void* dp,
                   void* stream);

/* Fused masked softmax-attention (bf16; head_dim d = 64 or 128, or d = 32 with an even number of heads -- the kernels
 * then take two neighbouring heads per block; gpt2.py:212-214 defaults to 512 / 16 = 32):
 * out = softmax(Q K^T / sqrt(d), mask) V for every (batch, head), without materialising the score matrix
 * (transformer.py:117-127).
 * q, k, v point at head 0 of batch 0; rows are tokens (batch-major), head j occupies columns
 * j*d.. of each pointer, row stride ld_qkv (the three pointers may alias one [rows, 3h] buffer).
 * out: [rows, heads*d] with row stride ld_out.  lse: fp32 [batch, heads, seq] log-sum-exp (base 2,
 * scaled scores) kept for the backward.
 * dropout_p > 0: dropout on the probabilities (transformer.py:125-126), out = (P o mask / (1 - p)) V with the
 * decisions of key (dropout_k0, dropout_k1) at element ((batch * heads + head) * seq + query) * seq + key;
 * the backward is given the same p and key and makes the same decisions again.                          */
int bb_attention_fwd(int dtype, int mask, int batch, int heads, int seq, int head_dim, const void* q,
                     const void* k, const void* v, int64_t ld_qkv, void* out, int64_t ld_out, float* lse,
                     const int32_t* key_len, float dropout_p, uint32_t dropout_k0, uint32_t dropout_k1, void* stream);
/* Backward of bb_attention_fwd: dq, dk, dv (same addressing as q, k, v with row stride ld_dqkv)
 * from d_out, the forward's out and lse.  delta: fp32 workspace [batch, heads, seq].
 * Deterministic (no atomics): dK/dV and dQ are produced by two passes over the score tiles. */
int bb_attention_bwd(int dtype, int mask, int batch, int heads, int seq, int head_dim, const void* q,
                     const void* k, const void* v, int64_t ld_qkv, const void* out, const void* d_out,
                     int64_t ld_out, const float* lse, float* delta, void* dq, void* dk, void* dv,
                     int64_t ld_dqkv, const int32_t* key_len, float dropout_p, uint32_t dropout_k0, uint32_t dropout_k1, void* stream);

/* out = a + b, elementwise (SublayerConnection residual, transformer.py:103).             */
int bb_residual_add(int dtype, int64_t n, const void* a, const void* b, void* out,
                    void* stream);

/* m = sqrt(1 - x), elementwise: the stand-in memory of DecoderLayerSimple.forward
 * (DeepSpeedExamples/pipeline_parallelism/gpt2.py:31), and its backward dx (+)= dm * (-1 / (2 m))
 * (accumulate != 0 adds to dx).  n a multiple of 8 (bf16) / 4 (fp32).                       */
int bb_sqrt_one_minus_fwd(int dtype, int64_t n, const void* x, void* m, void* stream);
int bb_sqrt_one_minus_bwd(int dtype, int64_t n, const void* dm, const void* m, void* dx,
                          int accumulate, void* stream);

/* out = act(x), elementwise: the activation of PositionwiseFeedForward (transformer.py:158) as a
 * bandwidth-bound pass of its own.  If dact != NULL it also receives act'(x), the factor autograd
 * applies in the backward pass; dact may be x itself (each element is read before it is
 * replaced), so keeping the derivative instead of the pre-activation costs no memory.         */
int bb_act_fwd(int dtype, int act, int64_t n, const void* x, void* out, void* dact, void* stream);

/* BatchNorm2d in training mode on an NHWC activation viewed as [rows = N*H*W, cols = channels]
 * (resnet.py:56,59,62): per-channel batch mean and biased variance (one pass, sums shifted by row 0), then
 * y = gamma * (x - mean) * rstd + beta (+ resid) with optional ReLU (the block's final
 * ReLU(residual_function(x) + shortcut(x)), resnet.py:75).  mean / rstd: fp32 [cols], kept for the
 * backward.  running_mean / running_var (both or neither; may be NULL for a redundant forward,
 * which must not update them) follow nn.BatchNorm2d (momentum, unbiased running variance).
 * workspace: fp32, >= bb_bn_workspace(cols).                                                  */
int64_t bb_bn_workspace(int cols);
int bb_batchnorm_fwd(int dtype, int rows, int cols, float eps, float momentum, int relu, const void* x,
                     const void* gamma, const void* beta, const void* resid, void* y, float* mean,
                     float* rstd, float* running_mean, float* running_var, float* workspace, void* stream);
/* bb_batchnorm_fwd with the statistics pass replaced by the strip statistics of x that the kernel which
 * produced x left behind (bb_gemm_desc.strip_stats, bb_conv3x3): same outputs up to the fp32 rounding of the
 * statistics (strips are merged with the pairwise update of Chan et al., no cancellation).  bf16 only.      */
int bb_batchnorm_fwd_strips(int dtype, int rows, int cols, float eps, float momentum, int relu, const void* x,
                            const void* gamma, const void* beta, const void* resid, void* y, float* mean,
                            float* rstd, float* running_mean, float* running_var, const float* strip_stats,
                            void* stream);
/* Backward through (optional ReLU given by its output relu_out) and the batch normalisation:
 * g = dy * (relu_out > 0); dgamma += sum g*xhat; dbeta += sum g;
 * dx = gamma * rstd * (g - mean(g) - xhat * mean(g*xhat)); g_out (optional) receives g.       */
int bb_batchnorm_bwd(int dtype, int rows, int cols, const void* x, const void* gamma, const float* mean,
                     const float* rstd, const void* dy, const void* relu_out, void* dx, void* g_out,
                     float* dgamma, float* dbeta, float* workspace, void* stream);
/* 3x3 / stride 1 / pad 1 patch matrix of an NHWC tensor: col[p, tap*C + c] = x[n, y+dy, x+dx, c]
 * (adjoint = 0), or its adjoint dx[p, c] = sum of the patch entries that read x[p, c]
 * (adjoint = 1); turns nn.Conv2d(k=3, padding=1) (resnet.py:58) and its input gradient into GEMMs. */
int bb_patch3x3(int dtype, int adjoint, int n, int h, int w, int c, const void* src, void* dst, void* stream);
/* The same with a stride (nn.Conv2d(k=3, stride=s, padding=1) of a down-sampling bottleneck, resnet.py:58 with
 * stride = 2): col has one row per output pixel of the [(h-1)/s + 1, (w-1)/s + 1] grid; the adjoint writes the
 * [n*h*w, c] input gradient from it.  stride 1..4.                                                           */
int bb_patch3x3_strided(int dtype, int adjoint, int n, int h, int w, int c, int stride, const void* src, void* dst,
                        void* stream);
/* What a 1x1 convolution with stride s reads (the projection shortcut, resnet.py:69): adjoint = 0:
 * dst[n, oy, ox, :] = src[n, s*oy, s*ox, :]; adjoint = 1, in place: dst[n, s*oy, s*ox, :] += src[n, oy, ox, :]
 * (dst [n*h*w, c] keeps its other pixels).                                                                    */
int bb_subsample(int dtype, int adjoint, int n, int h, int w, int c, int stride, const void* src, void* dst,
                 void* stream);
/* nn.Conv2d(cin, cout, kernel_size=3, padding=1, bias=False) (resnet.py:58) on NHWC rows as an implicit
 * GEMM on the matrix cores: the patch matrix is never written, the operand loader gathers it.
 *   BB_CONV_FWD    dst[p, o] = sum_{t, i} src[p + shift(t), i] * weight[o, t, i]     src [n*h*w, cin], dst [n*h*w, cout]
 *   BB_CONV_DGRAD  dst[p, i] = sum_{t, o} src[p - shift(t), o] * weight[o, t, i]     src [n*h*w, cout], dst [n*h*w, cin]
 * with tap t = (dy + 1) * 3 + (dx + 1), shift(t) = dy * w + dx inside one image and zero outside it, and
 * weight [cout, 3, 3, cin] (tap-major, channel-minor).  bf16 only; bb_conv3x3_supported() says (1 / 0) whether
 * a problem is taken (channel counts: gathered side a multiple of 64), bb_conv3x3 refuses the others.     */
#define BB_CONV_FWD 0
#define BB_CONV_DGRAD 1
int bb_conv3x3_supported(int dtype, int mode, int n, int h, int w, int cin, int cout);
int bb_conv3x3(int dtype, int mode, int n, int h, int w, int cin, int cout, const void* src, const void* weight,
               void* dst, float* strip_stats /* BB_CONV_FWD: as bb_gemm_desc.strip_stats, or NULL */, void* stream);

/* The backward pass of "BatchNorm2d, ReLU, Conv2d" (resnet.py:56-61: each of the two inner normalisations of a
 * bottleneck feeds a ReLU and a convolution; autograd's backward of that chain, engine.py:1701-1709) without a
 * reduction pass over the tensor: the kernel that computes the convolution's input gradient dy also masks it with
 * the ReLU (g = dy * (relu_out > 0), stored as C / dst) and leaves, per strip of 32 consecutive rows and per
 * column, sum g and sum g * xhat of the stored bf16 values, xhat = (x - mean) * rstd of the normalisation's input
 * x ([M, N] contiguous like C): strips[(strip * 2 + j) * N + n], fp32, >= bb_bn_bwd_strips_workspace(M, N) floats.
 * bb_batchnorm_bwd_strips adds the strips up in a fixed order and applies
 * dx = gamma * rstd * (g - mean(g) - xhat * mean(g * xhat)); dgamma += sum g * xhat; dbeta += sum g
 * (bb_batchnorm_bwd's result up to the fp32 summation order).  bf16 only.
 *   bb_gemm_bn_bwd       the input gradient of a 1x1 convolution: a BB_NN problem (C = dy_next W) with epilogue
 *                        BB_EPI_MUL_POS and aux_in = relu_out (or BB_EPI_NONE / BB_EPI_RESIDUAL: no ReLU);
 *                        bb_gemm_bn_bwd_supported() says (1 / 0) whether the problem is taken.  With resid this
 *                        is also the gradient a bottleneck hands to the block in front of it (resnet.py:75: the
 *                        sum of the residual function's and the shortcut's, then that block's last ReLU and
 *                        BatchNorm): x, mean, rstd, relu_out are then that block's
 *   bb_conv3x3_dgrad_bn  bb_conv3x3(BB_CONV_DGRAD) with the same additions (relu_out may be NULL)               */
typedef struct bb_bn_bwd_stats {
    const void* x;      /* [M, N] input of the normalisation */
    const float* mean;  /* [N] */
    const float* rstd;  /* [N] */
    float* strips;      /* out */
} bb_bn_bwd_stats;
int64_t bb_bn_bwd_strips_workspace(int rows, int cols);
int bb_gemm_bn_bwd_supported(const bb_gemm_desc* desc);
int bb_gemm_bn_bwd(const bb_gemm_desc* desc, const bb_bn_bwd_stats* bn, void* stream);
int bb_conv3x3_dgrad_bn(int dtype, int n, int h, int w, int cin, int cout, const void* src, const void* weight,
                        void* dst, const void* relu_out, const bb_bn_bwd_stats* bn, void* stream);
/* The same strip sums where no such kernel wrote the gradient (it arrived from another stage, or the shape is not
 * one they take): one pass over x, dy and relu_out (NULL: no ReLU) that writes g = dy * (relu_out > 0) to g_out (may be
 * dy itself; may be NULL without a ReLU) and the sums to strips, added up in the order of those epilogues: whichever
 * way the sums were made, bb_batchnorm_bwd_strips gives the same bits.                                             */
int bb_batchnorm_bwd_strip_sums(int dtype, int rows, int cols, const void* x, const float* mean, const float* rstd,
                                const void* dy, const void* relu_out, void* g_out, float* strips, void* stream);
int bb_batchnorm_bwd_strips(int dtype, int rows, int cols, const void* x, const void* gamma, const float* mean,
                            const float* rstd, const void* g, const float* strips, void* dx, float* dgamma,
                            float* dbeta, void* stream);

/* Mean-squared-error head (nn.MSELoss, transformer.py:264) fused with its gradient:
 * loss_out[0] (+)= mean((y-t)^2);  dy = grad_scale * 2 (y-t) / n.  Deterministic two-pass
 * reduction; workspace: fp32, at least bb_mse_workspace() elements.                       */
int64_t bb_mse_workspace(void);
int bb_mse_fwd_bwd(int dtype, int64_t n, const void* y, const void* target, void* dy,
                   float grad_scale, float* loss_out, int accumulate_loss, float* workspace,
                   void* stream);

/* Fused multi-tensor Adam / AdamW; replaces multi_tensor_adam
 * (csrc/adam/fused_adam_frontend.cpp:3-20, kernel csrc/adam/multi_tensor_adam.cu:28-121).
 * All of g, p, m, v are fp32; `lowp` (may be NULL, entries may be NULL) receives a bf16 copy
 * of the updated parameter (the compute weights of the bf16 configurations).
 * The pointer tables are HOST arrays of n_tensors device pointers; `sizes` are element counts.
 * mode: 0 = L2 (g += wd*p), 1 = decoupled weight decay (AdamW).  step >= 1.
 * zero_grad != 0 also clears g after use (the engine's zero_grad, fused).                 */
int bb_adam_multi(int n_tensors, void* const* g, void* const* p, void* const* m,
                  void* const* v, void* const* lowp, const int64_t* sizes, float lr,
                  float beta1, float beta2, float eps, int step, int mode,
                  int bias_correction, float weight_decay, int zero_grad, void* stream);

/* Gradient clipping by the global norm: clip_grad_norm_ (deepspeed/runtime/utils.py:259-326) as
 * _take_model_step calls it before optimizer.step() (deepspeed/runtime/engine.py:1526-1531,
 * clip_fp32_gradients :1521-1524).  bb_grad_clip_coef leaves out[0] = sqrt(sum of squares of all
 * the listed fp32 gradient tensors) and out[1] = min(1, max_norm / (out[0] + 1e-6)) in device
 * memory (fixed summation order, no atomics); bb_adam_multi_scaled is bb_adam_multi with every
 * gradient multiplied by the device scalar *grad_scale (NULL: by nothing) before the update, so
 * the clipped gradients never make a pass of their own through memory and the host never waits
 * for the norm.  workspace: bb_grad_clip_workspace(n_tensors, sizes) floats, 8-byte aligned.   */
int64_t bb_grad_clip_workspace(int n_tensors, const int64_t* sizes);
int bb_grad_clip_coef(int n_tensors, void* const* g, const int64_t* sizes, float max_norm,
                      float* out, float* workspace, void* stream);
int bb_adam_multi_scaled(int n_tensors, void* const* g, void* const* p, void* const* m,
                         void* const* v, void* const* lowp, const int64_t* sizes, float lr,
                         float beta1, float beta2, float eps, int step, int mode,
                         int bias_correction, float weight_decay, int zero_grad,
                         const float* grad_scale, void* stream);

/* dtype conversion / fill helpers used when (re)materialising compute weights.            */
int bb_cast(int src_dtype, int dst_dtype, int64_t n, const void* src, void* dst, void* stream);
int bb_fill_f32(float* dst, int64_t n, float value, void* stream);

/* Replay of a fixed launch sequence as a HIP graph.  The reference replays nothing: its engine
 * issues every ATen kernel of a micro-batch from Python on each step (engine.py:1626-1727); on
 * static buffers the same sequence is captured once and launched as one graph.
 *   bb_graph_begin   starts capturing `stream` (not the default stream; thread-local mode).  Calls
 *                    of this library on that stream are recorded, not run, until bb_graph_end.
 *   bb_graph_end     ends the capture and returns an executable graph in *exec_out.
 *   bb_graph_launch  runs it on a stream.   bb_graph_destroy  releases it.
 * Every kernel of the sequence must have been launched once before it is captured.            */
int bb_graph_begin(void* stream);
int bb_graph_end(void* stream, void** exec_out);
int bb_graph_launch(void* exec, void* stream);
int bb_graph_destroy(void* exec);

#ifdef __cplusplus
}
#endif
#endif /* BAMBOO_HIP_H */
