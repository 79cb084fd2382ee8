/*
 * C ABI of libterapipe_hip.so -- the MI355X (gfx950) kernels behind the sliced GPT-layer hot path.
 *
 * The reference (zhuohan123/terapipe) is pure Python on PyTorch and has no FFI layer; each entry
 * point below replaces the ATen call(s) the reference makes at the cited lines.  Conventions:
 *   - every pointer is a raw device pointer owned by the caller (PyTorch owns all memory); the
 *     library never allocates or frees device memory and keeps no state between calls
 *     (one exception, stated at its declaration: tp_gemm_static_ws keeps its k-split partial sums in a
 *     device array of the library's own);
 *   - `stream` is a hipStream_t passed as void*; launches are asynchronous on it, no internal syncs;
 *   - every function returns 0 on success or a tp_status code; tp_last_error() gives the message of
 *     the calling thread's last failure.  Nothing throws, nothing aborts;
 *   - dtype is a tp_dtype; fp16/bf16 compute with fp32 accumulation on MFMA, fp32 uses fp32 MFMA.
 *   - rows of every matrix are contiguous; leading dimensions and the contiguous extents must be
 *     multiples of 16 bytes worth of elements (8 for fp16/bf16, 4 for fp32) and pointers 16-byte aligned.
 */
#ifndef TERAPIPE_HIP_H_
#define TERAPIPE_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { TP_F32 = 0, TP_F16 = 1, TP_BF16 = 2 } tp_dtype;

typedef enum {
    TP_OK = 0,
    TP_ERR_ARG = 1,         /* null pointer, bad shape, misalignment */
    TP_ERR_UNSUPPORTED = 2, /* shape or dtype outside what the kernels cover */
    TP_ERR_WORKSPACE = 3,   /* workspace missing or too small */
    TP_ERR_LAUNCH = 4       /* HIP reported a launch error */
} tp_status;

int tp_version(void);
const char* tp_last_error(void);

/* ------------------------------------------------------------------------------------------------
 * LayerNorm over the last dimension of x[M, E]  (replaces nn.LayerNorm at transformer_models.py:275
 * and :280; modules built at :323, :325).  Statistics in fp32; mean/rstd [M] are saved for backward.
 */
int tp_layernorm_fwd(const void* x, const void* gamma, const void* beta, void* y, float* mean,
                     float* rstd, int M, int E, float eps, int dtype, void* stream);

/* Backward of the above fused with the residual-path add that follows it in the layer
 * (transformer_models.py:277, :284 are `x += y`, so the gradient of the LayerNorm input is
 * LN'(dy) + dres).  dres may be NULL.  The parameter gradients are ADDED into fp32 accumulators
 * (dgamma_acc and dbeta_acc may both be NULL to skip them, see tp_ln_param_grads):
 *   dgamma_acc[E] += sum_m dy * xhat,   dbeta_acc[E] += sum_m dy,
 *   colsum_dres_acc[E] += sum_m dres    (NULL to skip; this is the bias gradient of the
 *                                        row-parallel linear whose output fed the residual add),
 *   colsum_dx_acc[E]  += sum_m dx       (NULL to skip; bias gradient of the linear that produced
 *                                        the LayerNorm's input branch).
 */
int tp_layernorm_bwd(const void* dy, const void* x, const float* mean, const float* rstd,
                     const void* gamma, const void* dres, void* dx, float* dgamma_acc,
                     float* dbeta_acc, float* colsum_dres_acc, float* colsum_dx_acc, int M, int E,
                     int dtype, void* stream);

/* The same two kernels fed from the partial sums a k-split tp_gemm with defer_reduce left in its workspace
 * (partials[z][m][e], z < nsplit, fp32): the input row is sum_z partials (+ bias[e]) (+ residual[m][e]),
 * rounded to dtype exactly as the GEMM's own reduce would have, written to x_out / dy_out (the tensor the
 * GEMM was asked for) and normalised from there.  Saves the reduce launch and one pass over the tensor. */
int tp_layernorm_fwd_partials(const float* partials, int nsplit, const void* bias, const void* residual,
                              void* x_out, const void* gamma, const void* beta, void* y, float* mean,
                              float* rstd, int M, int E, float eps, int dtype, void* stream);
int tp_layernorm_bwd_partials(const float* partials, int nsplit, void* dy_out, const void* x,
                              const float* mean, const float* rstd, const void* gamma, const void* dres,
                              void* dx, float* dgamma_acc, float* dbeta_acc, float* colsum_dres_acc,
                              float* colsum_dx_acc, int M, int E, int dtype, void* stream);

/* LayerNorm parameter gradients over a block of rows (used once per layer over ALL tokens of a step
 * when the per-slice tp_layernorm_bwd calls pass NULL accumulators):
 *   dgamma_acc[E] += sum_m dy[m] * (x[m] - mean[m]) * rstd[m],   dbeta_acc[E] += sum_m dy[m].
 * Same sums autograd accumulates into nn.LayerNorm's weight.grad / bias.grad across slices. */
int tp_ln_param_grads(const void* dy, const void* x, const float* mean, const float* rstd,
                      float* dgamma_acc, float* dbeta_acc, int M, int E, int dtype, void* stream);

/* Every vector-parameter gradient of a layer in one launch: the sums autograd accumulates over the slices of a step
 * into the four bias .grad (mpu/layers.py:256, :346-347: column sums of the linears' output gradients) and the two
 * nn.LayerNorm weight / bias .grad pairs (transformer_models.py:275, :280), each taken over ALL rows of the step.
 * Up to 8 problems; a problem with x == NULL is a column sum (acc0[N] += sum_m dy[m, :]), otherwise the LayerNorm
 * pair (acc0[N] += sum_m dy * (x - mean) * rstd, acc1[N] += sum_m dy).  fp32 accumulators, added to. */
typedef struct tp_vecgrad_desc {
    const void* dy;             /* [M, ld] rows of `dtype` */
    const void* x;              /* [M, ld] LayerNorm input, or NULL for a column sum */
    const float* mean; const float* rstd;   /* [M], with x */
    float* acc0; float* acc1;   /* [N] fp32; acc1 only with x */
    int64_t ld;
    int32_t M, N;
} tp_vecgrad_desc;
int tp_vec_param_grads(const tp_vecgrad_desc* descs, int n, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------------
 * GEMMs that mpu.ColumnParallelLinear / RowParallelLinear reduce to at tensor-parallel size 1
 * (F.linear at mpu/layers.py:256 and :335, and their autograd backward), with the elementwise work
 * around them fused into the epilogue.
 */
typedef enum {
    TP_GEMM_NT = 0, /* C[M,N] = A[M,K] . B[N,K]^T   forward  Y = X W^T        (W stored [out,in]) */
    TP_GEMM_NN = 1, /* C[M,N] = A[M,K] . B[K,N]     data grad dX = dY W                          */
    TP_GEMM_TN = 2  /* C[M,N] = A[K,M]^T . B[K,N]   weight grad dW = dY^T X                      */
} tp_gemm_op;

typedef enum {
    TP_EPI_STORE = 0,         /* C = acc                                                            */
    TP_EPI_ACCUMULATE = 1,    /* C += acc            (parameter .grad accumulation across slices)   */
    TP_EPI_BIAS = 2,          /* C = acc + bias[n]   (ColumnParallelLinear, mpu/layers.py:256)      */
    TP_EPI_BIAS_RELU = 3,     /* C = relu(acc + bias[n])   (fc1 + relu_, transformer_models.py:282) */
    TP_EPI_BIAS_GELU = 4,     /* C = gelu_erf(acc + bias[n]); aux_out (if set) = acc + bias[n]      */
    TP_EPI_BIAS_RESIDUAL = 5, /* C = acc + bias[n] + residual[m,n] (RowParallelLinear bias add
                                 mpu/layers.py:346-347 + `x += y` transformer_models.py:277, :284)  */
    TP_EPI_QKV_SCATTER = 6,   /* in_proj output split per head into q (scaled), k, v and written
                                 straight to q[B*H,T,Dh] and rows [P, P+T) of the K/V caches
                                 (transformer_models.py:217-219 and _AssignCache.forward :181-184)  */
    TP_EPI_RELU_GRAD = 7,     /* C = acc * (aux[m,n] > 0)   backward of relu_ on its saved output   */
    TP_EPI_GELU_GRAD = 8      /* C = acc * gelu_erf'(aux[m,n])   aux = saved pre-activation         */
} tp_gemm_epilogue;

typedef struct tp_gemm_desc {
    int32_t op;       /* tp_gemm_op */
    int32_t dtype;    /* tp_dtype of A, B, C, bias, residual, aux, q, caches */
    int32_t epilogue; /* tp_gemm_epilogue */
    int32_t M, N, K;
    const void* A; int64_t lda;
    const void* B; int64_t ldb;
    void* C; int64_t ldc;               /* unused by TP_EPI_QKV_SCATTER */
    const void* bias;                   /* [N] */
    const void* residual; int64_t ldr;  /* [M, ldr] */
    const void* aux; int64_t ldaux;     /* [M, ldaux] */
    void* aux_out; int64_t ldauxo;      /* [M, ldauxo] */
    float* colsum_acc;                  /* optional [N] fp32: += column sums of the values written to C
                                           (bias gradient of the linear whose output gradient C is) */
    /* TP_EPI_QKV_SCATTER: row m of C is (t, b) = (m / batch, m % batch); column n is
       head n / (3*head_dim), then [q | k | v] inside the head. */
    void* q; void* k_cache; void* v_cache;
    int32_t batch, heads, head_dim, cache_len;
    int64_t cache_rows;                 /* L_max: rows per (b,h) in the caches */
    float q_scale;
    int32_t reserved;                   /* 0 = automatic; bits 0-7: tile configuration + 1, bits 8-15: k splits (tuning, tests) */
    int64_t q_bh_rows;                  /* rows per (b,h) block of q: 0 = T (compact [B*H,T,Dh]); a runner that
                                           keeps the queries of every slice passes L_max and q offset to row P */
    int32_t defer_reduce;               /* 1 (STORE / BIAS_RESIDUAL epilogues only): when the plan splits k
                                           (tp_gemm_splits > 1) leave the fp32 partial sums [splits][M][N] in the
                                           workspace and write nothing else; the LayerNorm that consumes C sums them,
                                           applies bias / residual and writes C (tp_layernorm_fwd/bwd_partials).
                                           Without a split the GEMM completes as usual. */
    int32_t reserved4;
} tp_gemm_desc;

/* number of k splits the plan uses for this product (1 = none; 0 = invalid descriptor) */
int tp_gemm_splits(const tp_gemm_desc* d);
/* The plan tp_gemm would run the product with: the tile configuration's number (the kernel and tile shape, as listed
 * in csrc/gemm.hip) and the number of k splits.  Host code only; for tuning, tests and logs. */
int tp_gemm_plan(const tp_gemm_desc* d, int* tile_cfg, int* nsplit);
size_t tp_gemm_workspace_bytes(const tp_gemm_desc* d);
int tp_gemm(const tp_gemm_desc* d, void* workspace, size_t workspace_bytes, void* stream);
/* n independent products as if by n tp_gemm calls in order on the stream (the four weight gradients of a layer,
   which autograd's backward of the four linears of transformer_models.py:273-285 produces one by one).  Up to four
   16-bit TP_GEMM_TN products of one dtype, k a multiple of 64, whose largest plans to 256 x 256 tiles with unsplit
   k share ONE launch, so that together they fill whole rounds of the chip's CUs; any other group runs member by
   member.  workspace: the largest member's tp_gemm_workspace_bytes. */
int tp_gemm_grouped(const tp_gemm_desc* descs, int n, void* workspace, size_t workspace_bytes, void* stream);
/* the tile configuration of the single launch tp_gemm_grouped makes for this group; 0 = member by member */
int tp_gemm_group_cfg(const tp_gemm_desc* descs, int n);

/* tp_gemm for callers that cannot allocate device memory or pass a workspace (code under HIP-graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference: it exists for those
 * callers only.  The k-split partial sums go to a TP_GEMM_STATIC_WS_BYTES array that the library holds in every
 * GPU's memory from load to process exit; the call allocates and frees nothing.  Same kernels, same plan, same
 * result bits as tp_gemm with a caller workspace.  A product whose plan needs more than the array holds is
 * refused with TP_ERR_WORKSPACE (tp_gemm_workspace_bytes(d) > tp_gemm_static_ws_capacity()), defer_reduce with
 * TP_ERR_ARG.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two
 * threads) race on the partial sums; nothing in it needs to start at zero.  The array's address on a device is
 * looked up once, by the first call of either function with that device current (a module and symbol lookup):
 * a caller that captures tp_gemm_static_ws into a HIP graph calls tp_gemm_static_ws_capacity() on the device
 * BEFORE the capture opens. */
#define TP_GEMM_STATIC_WS_BYTES (64u << 20)
size_t tp_gemm_static_ws_capacity(void);
int tp_gemm_static_ws(const tp_gemm_desc* d, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Prefix-cached causal attention (attn_helper, transformer_models.py:235-245, with the mask of :220
 * and :229 applied as an index comparison, and the gradient contract of _AssignCache.backward
 * :186-190).  Query row t of the slice attends to cache rows [0, cache_len + t].
 */
typedef struct tp_attn_desc {
    int32_t dtype;
    int32_t batch, heads, head_dim;     /* 16, 32, 64, 80, 96 or 128 */
    int32_t T;                          /* slice length */
    int32_t cache_len;                  /* P: rows of the caches filled by earlier slices */
    int64_t cache_rows;                 /* L_max */
    const void* q;                      /* [B*H, T, Dh], already multiplied by Dh^-0.5 */
    const void* k_cache;                /* [B*H, L_max, Dh]; rows [0, P+T) valid */
    const void* v_cache;
    void* o;                            /* [T, B, H*Dh]  (heads concatenated, transformer_models.py:244) */
    float* lse;                         /* [B*H, T] log-sum-exp of the scaled, masked scores */
    /* backward only */
    const void* d_o;                    /* [T, B, H*Dh] */
    float* delta;                       /* [B*H, T] scratch: rowsum(dO * O) */
    void* dqkv;                         /* [T*B, 3*H*Dh] gradient of the in_proj output (per-head
                                           [q|k|v] order); the q part includes the Dh^-0.5 factor */
    void* dk_cache; void* dv_cache;     /* [B*H, L_max, Dh] gradient caches */
    int32_t grad_cache_dtype;           /* tp_dtype of dk_cache/dv_cache: `dtype` or TP_F32 */
    int32_t accumulate_prefix;          /* 1: rows [0,P) += dK, dV;  0: rows [0,P) = dK, dV */
    int32_t has_incoming;               /* 1: rows [P,P+T) hold the gradient handed back by later
                                           slices and are added to this slice's dK, dV */
    int32_t zero_slice_rows;            /* 1: rows [P,P+T) are set to zero after being consumed
                                           (grad_cache.data[index] = 0, transformer_models.py:189) */
    float q_scale;
    float* colsum_dqkv_acc;             /* optional [3*H*Dh] fp32: += column sums of dqkv (in_proj bias grad) */
    int32_t reserved;                   /* 0 = automatic; bits 0-7: number of workgroups (fp32: splits) that share the key
                                           range of a query block in the forward (tuning, tests) */
    int32_t reserved2;                  /* tuning, tests.  bit 1 / bit 2: force the eight-wave / the four-wave form of the
                                           16-bit forward kernel; bit 3 / bit 4: force its workgroups of 32 / of 64 queries
                                           (64 needs T >= 64) */
    int64_t q_bh_rows;                  /* rows per (b,h) block of q: 0 = T; see tp_gemm_desc.q_bh_rows */
    int64_t stat_bh_rows;               /* entries per (b,h) block of lse and delta: 0 = T */
    int32_t dq_only;                    /* backward: 1 = compute delta and the q part of dqkv only; dK/dV of the
                                           slice are left to tp_attn_suffix_dkdv and no gradient cache is touched */
    int32_t reserved3;
} tp_attn_desc;

/* A forward call with few (batch, head) x 32-query blocks and a long key range spreads each block's keys over
 * several workgroups; their fp32 partial results go through the caller's workspace and a second launch of the same
 * call merges them.  The size query returns 0 when the call does not split. */
size_t tp_attn_fwd_workspace_bytes(const tp_attn_desc* d);
int tp_attn_prefix_fwd(const tp_attn_desc* d, void* workspace, size_t workspace_bytes, void* stream);
size_t tp_attn_bwd_workspace_bytes(const tp_attn_desc* d);
int tp_attn_prefix_bwd(const tp_attn_desc* d, void* workspace, size_t workspace_bytes, void* stream);

/* dK / dV of one slice's keys against EVERY query that can see them, in one pass: the sum that
 * _AssignCache.backward (transformer_models.py:186-190) builds up slice by slice in the gradient caches
 * when the later slices run their backward first (terapipe.py:182-191).  A stage that keeps q, dO, lse
 * and delta of all its slices (position-indexed, as the K/V caches are) calls this when slice [P, P+T)
 * runs its backward -- every later slice has then left its dO and delta -- and needs no gradient cache.
 * Query position t in [key_begin, q_end) sees key position s <= t.  Writes the k and v parts of dqkv. */
typedef struct tp_attn_suffix_desc {
    int32_t dtype;                      /* TP_F16 or TP_BF16 */
    int32_t batch, heads, head_dim;     /* head_dim 64 or 128 */
    int32_t key_begin, key_count;       /* P, T of the slice whose keys these are */
    int32_t q_end;                      /* queries [key_begin, q_end) take part */
    int32_t reserved;
    int64_t cache_rows;                 /* rows per (b,h) of k_cache, v_cache */
    int64_t q_bh_rows;                  /* rows per (b,h) of q_all */
    int64_t stat_bh_rows;               /* entries per (b,h) of lse_all, delta_all */
    const void* k_cache; const void* v_cache;
    const void* q_all;                  /* [B*H, q_bh_rows, Dh], row = position, scaled as in tp_attn_desc.q */
    const void* d_o_all;                /* [q_end.., B, H*Dh], row = position */
    const float* lse_all; const float* delta_all;   /* [B*H, stat_bh_rows], entry = position */
    void* dqkv;                         /* [T*B, 3*H*Dh] of the slice; the k and v parts are written */
} tp_attn_suffix_desc;
int tp_attn_suffix_dkdv(const tp_attn_suffix_desc* d, void* stream);

/* tp_attn_prefix_bwd with dq_only = 1 and tp_attn_suffix_dkdv of the SAME slice as one launch (fp16 / bf16): the backward
 * of attn_helper for one slice (transformer_models.py:229-240 under autograd, driven by terapipe.py:182-191) on a stage
 * that keeps no gradient caches.  Half of the workgroups stream the keys before the slice (dQ, delta), the other half
 * the queries after it (dK, dV) at the same time; the two descriptors must name the same slice (d->cache_len =
 * sd->key_begin, d->T = sd->key_count, same caches and dqkv).  The dK/dV half reads sd->delta_all only for positions
 * at or past own_delta_end and takes delta of [key_begin, own_delta_end) itself from d_o_all and o_all (the attention
 * output, row = position, laid out as d_o_all): own_delta_end = end of the slice when every later slice's backward
 * has completed, later when the launches that write the delta of the next slices may still be running (at most 4096
 * positions from key_begin).  Same results as the two calls. */
int tp_attn_bwd_fused(const tp_attn_desc* d, const tp_attn_suffix_desc* sd, const void* o_all, int32_t own_delta_end,
                      void* stream);

/* ------------------------------------------------------------------------------------------------
 * The two ends of the layer stack in the reference's end-to-end configuration (token ids in, next-token
 * cross-entropy out), at tensor-parallel size 1.
 */
/* out[m, :] = weight[ids[m], :]   (F.embedding inside VocabParallelEmbedding.forward, mpu/layers.py:126-141;
 * ids outside [0, V) give a zero row, as the reference's masked rows do). */
int tp_embedding_fwd(const int64_t* ids, const void* weight, void* out, int M, int E, int V, int dtype, void* stream);
/* dweight_acc[ids[m], :] += dout[m, :]   (fp32 accumulators; autograd's embedding backward) */
int tp_embedding_bwd(const int64_t* ids, const void* dout, float* dweight_acc, int M, int E, int V, int dtype, void* stream);
/* _VocabParallelCrossEntropy (mpu/cross_entropy.py:25-104) forward and backward in one pass over logits
 * [M, ld] whose first V columns are the vocabulary (columns [V, Vpad) are alignment padding of the LM-head
 * GEMM): loss[m] = logsumexp(logits[m, :V]) - logits[m, target[m]], and logits is overwritten IN PLACE with
 * its gradient (softmax - onehot(target)) * grad_scale (padding columns 0), the way the reference overwrites
 * its input with the softmax (:65-74) and returns it scaled as grad_input (:79-99). */
int tp_cross_entropy(void* logits, int64_t ld, const int64_t* target, float* loss, int M, int V, int Vpad,
                     float grad_scale, int dtype, void* stream);
/* x[m, :N] *= scale[m] in place: the per-token grad_output factor of the cross-entropy backward (:97) */
int tp_scale_rows(void* x, int64_t ld, const float* scale, int M, int N, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Slice planner (host code, no GPU work): `planning` of latency_model.py:97-152.
 * latency_grid[bs][step][ctx], bs <= total_batch_size, step, ctx <= n_steps (row-major doubles): latency of
 * one slice of `step` sequence steps after `ctx` steps of context at batch size bs.  Minimises the sum of
 * slice latencies + (pipeline_len - 1) * the largest one with every slice latency <= max_latency.
 * Output: *final_time (infinity and *n_groups = 0 when no plan is feasible), the batch groups in the order the
 * reference emits them, and for each group its slices in steps, LAST slice of the sequence first (as the
 * reference's list before analysis_model reverses it, :172-173).  group_batch, group_nslices hold up to
 * total_batch_size entries, slice_steps up to total_batch_size * n_steps. */
int tp_plan_slices(const double* latency_grid, int total_batch_size, int n_steps, int pipeline_len,
                   double max_latency, double* final_time, int* n_groups, int* group_batch, int* group_nslices,
                   int* slice_steps);

/* ------------------------------------------------------------------------------------------------
 * Mixed-precision optimizer step: `update_weights` of test_transformer_terapipe.py:245-266 in one launch
 * (gradient copy to fp32 with 1/loss-scale :248-252, FusedAdam on the fp32 master weights :255 as constructed
 * at :92-97, zero_grad :256-260, master -> 16-bit model copy :262-266).  The update follows apex's
 * multi_tensor_adam (adam_w_mode 1 = decoupled weight decay, 0 = L2), which with weight_decay 0 is
 * torch.optim.Adam.  All state is fp32; every pointer is 16-byte aligned.
 */
typedef struct tp_adam_tensor {
    void* master;       /* fp32 [n] weights, updated in place */
    void* grad;         /* [n] gradient of desc.grad_dtype; zeroed when desc.zero_grad */
    void* exp_avg;      /* fp32 [n] first moment, updated in place */
    void* exp_avg_sq;   /* fp32 [n] second moment, updated in place */
    void* model;        /* [n] weights of desc.model_dtype, overwritten with the new master; unused when -1 */
    int64_t n;
} tp_adam_tensor;

typedef struct tp_adam_desc {
    int32_t n_tensors;          /* <= 65535 */
    int32_t grad_dtype;         /* tp_dtype of every gradient in the table */
    int32_t model_dtype;        /* TP_F16 / TP_BF16, or -1: no 16-bit copy is written */
    int32_t adam_w_mode;
    int32_t bias_correction;
    int32_t zero_grad;
    int32_t step;               /* 1 for the first update */
    int32_t blocks_per_tensor;  /* 0 = default (256) */
    double lr, beta1, beta2, eps, weight_decay;   /* doubles: 1 - beta and the bias corrections are formed in
                                                     double and rounded once, as torch.optim does */
    double grad_scale;          /* gradients are multiplied by this first (1 / loss scale) */
    const tp_adam_tensor* tensors;  /* DEVICE memory, n_tensors records */
} tp_adam_desc;

/* validates a HOST copy of the table (null pointers, alignment, lengths) before it is uploaded */
int tp_adam_check_table(const tp_adam_tensor* host_table, int n_tensors, int model_dtype);
int tp_adam_step(const tp_adam_desc* desc, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Small helpers around the kernels above.
 */
/* dst[n] (dtype) = (accumulate ? dst[n] : 0) + src[n] (fp32): folds the fp32 accumulators of the
 * LayerNorm / bias gradients into parameter .grad tensors (autograd's sum over slices). */
int tp_accum_cast(void* dst, const float* src, int64_t n, int accumulate, int dtype, void* stream);
/* acc[N] += column sums of x[M, N] (fp32 accumulators). */
int tp_colsum_acc(const void* x, int64_t ldx, float* acc, int M, int N, int dtype, void* stream);
/* fills n 32-bit words with zero (a kernel, so it can be recorded into a HIP graph) */
int tp_zero_words(void* dst, int64_t n_words, void* stream);
/* Measurement aid, no counterpart in the reference: `workgroups` workgroups of four waves each stream
   batches_per_wave batches of 8192 bytes per wave into LDS with global_load_lds_dwordx4 (128 KB of LDS and four
   batches in flight per wave: one workgroup per CU) and do nothing else.  hits_per_miss < 0: every batch from
   small_region (which the L2 holds); 0: every batch from the wave's own stretch of big (HBM); n > 0: one batch of
   big after every n of small_region.  row_stride 0: a batch is 8192 consecutive bytes; else a batch is a tile of 64
   rows x 128 bytes of a row-major matrix with row_stride bytes between rows, and consecutive batches of a source
   walk along the rows -- the access pattern of a GEMM's k loop over a k-major operand.  Bytes moved:
   workgroups * 4 * batches_per_wave * 8192.  bench.py --fill-path times it: the rates bound every kernel here that
   stages operand tiles through LDS. */
int tp_fill_probe(const void* big, int64_t big_bytes, const void* small_region, int64_t small_bytes,
                  int hits_per_miss, int workgroups, int batches_per_wave, int64_t row_stride, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TERAPIPE_HIP_H_ */
