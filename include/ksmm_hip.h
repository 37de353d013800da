/* C ABI of libksmm_hip.so: Kronecker-sparse matrix multiplication on MI355X (gfx950).
 *
 * A factor with pattern (a, b, c, d) holds a*b*c*d weights and maps a*c*d input features to
 * a*b*d output features:
 *
 *     y[a_i, b_i, d_i, n] = scale * sum_{c_i} W[a_i, b_i, c_i, d_i] * x[a_i, c_i, d_i, n]
 *
 * Tensors are plain device pointers:
 *   x  input,  bs_last ? (a*c*d, batch) : (batch, a*c*d), row-major, contiguous
 *   w  weight in the reference's "kernel" format (a*d*c, b), row-major: element
 *      (a_i, b_i, c_i, d_i) at row (a_i*d + d_i)*c + c_i, column b_i
 *      (reference: src/ksmm_py/layer/kronecker_sparse/interface.py:65-69)
 *   y  output, bs_last ? (a*b*d, batch) : (batch, a*b*d); never aliases x
 * All accumulation is fp32.  Supported (x, w, y) element types:
 *   (F32, F32, F32)   (F16, F16, F16)   (FP8_E4M3, FP8_E4M3, F16)   (F16, FP8_E4M3, F16)
 * FP8_E4M3 is the OCP e4m3fn encoding (torch.float8_e4m3fn); `scale` carries the product of
 * the per-tensor dequantisation scales and is applied to the fp32 accumulator before the
 * result is rounded to the output type.
 *
 * Alignment: x, w and y that start on 16-byte boundaries run on the vector kernels; tensors
 * that do not are still computed, by the one-thread-per-output kernel (a forced family
 * refuses them with KSMM_ERR_BAD_ALGO).  A bias vector needs the alignment of its element
 * type only.  Workspaces must be 16-byte aligned.
 *
 * The library never allocates device memory and keeps no caller-visible mutable state (it
 * remembers which kernels had their LDS limit raised, and ksmm_chain_forward_static owns one
 * fixed device buffer per GPU).  All launches go to the stream the caller passes (a
 * hipStream_t cast to void*; NULL is the legacy default stream).  Every entry point returns
 * KSMM_OK or a negative error code; ksmm_strerror() names it.  Only ksmm_factor_forward*,
 * ksmm_chain_forward* and ksmm_factor_backward* touch the GPU.
 */
#ifndef KSMM_HIP_H
#define KSMM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KSMM_VERSION 2

typedef enum ksmm_dtype {
    KSMM_F32 = 0,
    KSMM_F16 = 1,
    KSMM_FP8_E4M3 = 2
} ksmm_dtype;

typedef enum ksmm_status {
    KSMM_OK = 0,
    KSMM_ERR_NULL_POINTER = -1,   /* x, w or y is NULL                                        */
    KSMM_ERR_BAD_PATTERN = -2,    /* a, b, c or d < 1                                         */
    KSMM_ERR_BAD_BATCH = -3,      /* batch < 1                                                */
    KSMM_ERR_BAD_DTYPE = -4,      /* (x, w, y) type combination not in the list above         */
    KSMM_ERR_TOO_LARGE = -5,      /* a tensor has 2^31 elements or more                       */
    KSMM_ERR_BAD_ALGO = -6,       /* forced kernel id unknown, or it cannot run this problem  */
    KSMM_ERR_LAUNCH = -7,         /* HIP reported an error at launch                          */
    KSMM_ERR_CHAIN_MISMATCH = -8, /* output size of factor i != input size of factor i+1      */
    KSMM_ERR_WORKSPACE = -9,      /* workspace missing or smaller than ksmm_chain_workspace   */
    KSMM_ERR_BAD_CHAIN = -10,     /* n_factors < 1 or > KSMM_MAX_FACTORS                      */
    KSMM_ERR_ALIAS = -11,         /* y overlaps x, or the workspace overlaps x or y           */
    KSMM_ERR_BAD_EPILOGUE = -12   /* ksmm_epilogue.act is not a ksmm_act                      */
} ksmm_status;

/* Kernel families.  KSMM_ALGO_AUTO lets the tile table decide. */
typedef enum ksmm_algo {
    KSMM_ALGO_AUTO = 0,
    KSMM_ALGO_GENERIC = 1, /* one thread per output element group; any shape              */
    KSMM_ALGO_WAVE = 2,    /* weights stationary in registers, one wavefront per group    */
    KSMM_ALGO_TILE = 3     /* LDS-staged MFMA tiles                                       */
} ksmm_algo;

/* What the tile table chose for a problem.  Replaces the reference's generated
 * `best_kernel_bs_{first,last}_{float,half}` if-chains
 * (src/ksmm_py/layer/kronecker_sparse/kernel_bs_first_float.cuh:8-21) and the rows of
 * kernel_bs_*.best (batch a b c d TILEX TILEK TILEY TX TY VSIZE ms std mse). */
typedef struct ksmm_tile {
    int algo;         /* ksmm_algo actually used                                           */
    int variant;      /* index of the template instance inside that family                 */
    int tile_m;       /* outputs of one (a_i, d_i) block computed by a workgroup           */
    int tile_n;       /* batch columns per workgroup iteration                             */
    int tile_k;       /* slab of c staged per step                                         */
    int tile_d;       /* consecutive d_i handled by one workgroup                          */
    int threads;      /* workgroup size                                                    */
    int lds_bytes;    /* LDS per workgroup                                                 */
    int64_t grid;     /* number of workgroups                                              */
} ksmm_tile;

/* What the last factor of a call does to its fp32 accumulator before rounding to y's type:
 *     y = act(scale * acc + bias[output feature]).
 * Replaces the separate bias pass of KSLinear.post_process
 * (src/ksmm_py/layer/kronecker_sparse/interface.py:457-466) and the GELU between the two
 * projections of the ViT feed-forward block (src/ksmm_py/model/vit.py:416-431). */
typedef enum ksmm_act {
    KSMM_ACT_NONE = 0,
    KSMM_ACT_GELU = 1 /* x * Phi(x), the erf form (torch.nn.GELU() default)                 */
} ksmm_act;

typedef struct ksmm_epilogue {
    const void *bias; /* NULL, or a*b*d values of y's element type on the device           */
    int act;          /* ksmm_act                                                          */
} ksmm_epilogue;

typedef struct ksmm_factor_desc {
    const void *w;    /* kernel-format weight (a*d*c, b)                                   */
    int a, b, c, d;
    int w_dtype;      /* ksmm_dtype                                                        */
    float scale;      /* multiplies this factor's fp32 accumulator                         */
} ksmm_factor_desc;

#define KSMM_MAX_FACTORS 16

int ksmm_version(void);
const char *ksmm_strerror(int status);

/* Host-only argument check (no GPU needed).  Mirrors the checks of the reference binding
 * (src/ksmm_py/layer/kronecker_sparse/kernel.cpp:36-42, kernel.cu:123-125), as codes. */
int ksmm_validate(int64_t batch, int a, int b, int c, int d, int x_dtype, int w_dtype,
                  int y_dtype, int bs_last);

/* Tile-table lookup (host only).  `algo` = KSMM_ALGO_AUTO or a forced family. */
int ksmm_query_tile(int64_t batch, int a, int b, int c, int d, int x_dtype, int w_dtype,
                    int y_dtype, int bs_last, int algo, ksmm_tile *out);

/* The same for one forced instance: `variant` as in ksmm_factor_forward_algo; with
 * KSMM_ALGO_AUTO, -1 = measured table first, then the heuristics, -3 = heuristics only. */
int ksmm_query_tile_variant(int64_t batch, int a, int b, int c, int d, int x_dtype, int w_dtype,
                            int y_dtype, int bs_last, int algo, int variant, ksmm_tile *out);

/* The measured table KSMM_ALGO_AUTO consults for batches of 8192 and more: the counterpart
 * of the reference's tuned `*.best` files and the if-chains generated from them
 * (src/ksmm_py/layer/kronecker_sparse/kernel.py:151-257).  Row i is
 * {a, b, c, d, combo, bs_last, algo, instance id, parameter, variant}, combo 0 = fp32,
 * 1 = fp16, 2 = e4m3 -> fp16; rows are sorted by (a, b, c, d, combo, bs_last).  The table
 * stores (instance id, parameter): the id is a hash of the instance's own parameters, so rows
 * keep naming the same kernel when instances are added or reordered; `variant` is what that
 * resolves to in this build (-1: the instance no longer exists, the heuristics take over).
 * Patterns without a row use the heuristic order of kernel families. */
int ksmm_tuned_count(void);
int ksmm_tuned_row(int index, int row[10]);

/* The stable name of the instance a (family, variant) pair selects for these element types
 * and layout, and back.  The tuner writes ids; forcing a kernel still takes a variant. */
int ksmm_variant_id(int algo, int variant, int x_dtype, int w_dtype, int y_dtype, int bs_last,
                    uint32_t *id, int *param);
int ksmm_variant_from_id(int algo, uint32_t id, int param, int x_dtype, int w_dtype, int y_dtype,
                         int bs_last, int *variant);

/* One factor.  Replaces `kernel.forward(input, factor, bs_last, a, b, c, d, dtype, vsize)`
 * (src/ksmm_py/layer/kronecker_sparse/kernel.cpp:25-45 -> kernel.cu:40-127); the caller
 * allocates y. */
int ksmm_factor_forward(const void *x, const void *w, void *y, int64_t batch, int a, int b,
                        int c, int d, int x_dtype, int w_dtype, int y_dtype, int bs_last,
                        float scale, void *stream);

/* Same, with the kernel family (and optionally a variant, -1 = the family's own choice) forced;
 * used by the tuner and by tests that must exercise one family.  Variants: KSMM_ALGO_GENERIC
 * 0 = one thread per output, 1 = 16-byte vector form (batch-size-last); KSMM_ALGO_WAVE
 * instance | tiles-per-wave << 8 | round-robin << 16, 1000 + i = batch-size-first row kernel i;
 * KSMM_ALGO_TILE sub-family << 24 | instance (0 k-loop, 1 weight-stationary, 2 stream,
 * 3 batch-size-first d > 1, 4 direct-to-LDS GEMM); KSMM_ALGO_AUTO -1 = measured table, then
 * heuristics, -3 = heuristics only.  An instance that cannot run the problem returns
 * KSMM_ERR_BAD_ALGO. */
int ksmm_factor_forward_algo(const void *x, const void *w, void *y, int64_t batch, int a,
                             int b, int c, int d, int x_dtype, int w_dtype, int y_dtype,
                             int bs_last, float scale, int algo, int variant, void *stream);

/* Batch-size-first factors with d > 1 whose shape has no kernel of its own in that layout run
 * in batch-size-last layout between two transposes when the caller lends a workspace.
 * ksmm_factor_workspace returns the bytes ksmm_factor_forward_ws can use for a problem (0: a
 * direct kernel exists, the workspace is ignored).  With a smaller workspace (or NULL) it
 * returns KSMM_ERR_WORKSPACE; ksmm_factor_forward (no workspace) falls back to the generic
 * kernel for such shapes.  The reference has no counterpart: its batch-size-first kernels
 * gather with strided scalar loads (template_kernels_float.cuh:156-161).
 * The same pair serves batch-size-last problems whose batch is not a multiple of the 16-byte
 * vector (rows that are not vector-aligned): the workspace holds the input and the output with
 * rows zero-filled to the next multiple of 16 columns, the factor runs there with the kernel of
 * the padded batch, and the result rows are cut back.  The reference refuses batch sizes its
 * hyper-parameters do not divide (kernel.py:241-244). */
int64_t ksmm_factor_workspace(int64_t batch, int a, int b, int c, int d, int x_dtype, int w_dtype,
                              int y_dtype, int bs_last);
int ksmm_factor_forward_ws(const void *x, const void *w, void *y, int64_t batch, int a, int b,
                           int c, int d, int x_dtype, int w_dtype, int y_dtype, int bs_last,
                           float scale, void *workspace, int64_t workspace_bytes, void *stream);

/* ksmm_factor_forward_ws with an epilogue (NULL: none) on the accumulator.  The bias add of
 * KSLinear.post_process (src/ksmm_py/layer/kronecker_sparse/interface.py:457-466) and an
 * activation that follows the layer (src/ksmm_py/model/vit.py:416-431) then cost no pass
 * over y of their own. */
int ksmm_factor_forward_ep(const void *x, const void *w, void *y, int64_t batch, int a, int b,
                           int c, int d, int x_dtype, int w_dtype, int y_dtype, int bs_last,
                           float scale, const ksmm_epilogue *epilogue, void *workspace,
                           int64_t workspace_bytes, void *stream);

/* Bytes of device workspace ksmm_chain_forward needs for these factors in batch-size-last
 * layout (two ping-pong intermediates; 0 for a single factor).  Intermediates have type
 * y_dtype. */
int64_t ksmm_chain_workspace(const ksmm_factor_desc *factors, int n_factors, int64_t batch,
                             int y_dtype);

/* The same for a given layout and input type: a batch-size-first chain with a factor that
 * needs the transposed route asks for room for the transposed input and for ping-pong buffers
 * that also hold the (transposed) final output.  ksmm_chain_forward returns
 * KSMM_ERR_WORKSPACE when the workspace it is given is smaller than this (or NULL while this
 * is not 0), like ksmm_factor_forward_ws: it never falls back to a slower route silently.
 * A batch-size-last chain whose batch is not a multiple of the 16-byte vector asks for the same
 * buffers with rows padded to a multiple of 16 columns and runs the whole chain there. */
int64_t ksmm_chain_workspace_layout(const ksmm_factor_desc *factors, int n_factors, int64_t batch,
                                    int x_dtype, int y_dtype, int bs_last);

/* A chain K_n ... K_1 x: factors[0] acts first.  Replaces the Python loop of
 * KSLinear.forward_bs_first / forward_bs_last
 * (src/ksmm_py/layer/kronecker_sparse/interface.py:193-211, 269-291).  The first factor
 * reads x in x_dtype; intermediates and y have y_dtype.  `fuse` != 0 allows kernels that
 * keep intermediates in LDS when the table has one for this chain. */
int ksmm_chain_forward(const ksmm_factor_desc *factors, int n_factors, const void *x, void *y,
                       void *workspace, int64_t workspace_bytes, int64_t batch, int x_dtype,
                       int y_dtype, int bs_last, int fuse, void *stream);

/* ksmm_chain_forward with an epilogue (NULL: none) applied by the last factor:
 * y = act(scale_n * acc + bias).  Replaces the chain loop plus the bias pass of
 * KSLinear.post_process (src/ksmm_py/layer/kronecker_sparse/interface.py:269-291, 457-466). */
int ksmm_chain_forward_ep(const ksmm_factor_desc *factors, int n_factors, const void *x, void *y,
                          void *workspace, int64_t workspace_bytes, int64_t batch, int x_dtype,
                          int y_dtype, int bs_last, int fuse, const ksmm_epilogue *epilogue,
                          void *stream);

/* Backward pass of one factor y = scale_fwd * K x, for F32 and F16 tensors (all three of one
 * type).  The reference has none that works (src/ksmm_py/layer/kronecker_sparse/kernel.py:319-329
 * names an undefined symbol, forward_bmm.py:12-15 is `pass`); these are the adjoints of its
 * forward product (interface.py:108-113):
 *   ksmm_factor_backward_input :  dx = scale * K^T dy, the KS factor with pattern (a, c, b, d)
 *                                 and every b x c block transposed, on the forward kernels;
 *   ksmm_factor_backward_weight:  dw[a_i,b_i,c_i,d_i] = scale * sum_n dy[a_i,b_i,d_i,n] x[a_i,c_i,d_i,n],
 *                                 written in kernel format (a*d*c, b) like w.
 * dy has y's shape and layout, dx has x's.  Both need ksmm_factor_backward_workspace() bytes of
 * 16-byte aligned device memory (transposed blocks, fp32 partial sums of the reduction over the
 * batch, one slice per batch split, and the forward kernels' own workspace for the transposed
 * factor).  The weight gradient adds its partial sums in a fixed order: two calls on the same
 * inputs give the same bits. */
int64_t ksmm_factor_backward_workspace(int64_t batch, int a, int b, int c, int d, int dtype,
                                       int bs_last);
int ksmm_factor_backward_input(const void *dy, const void *w, void *dx, int64_t batch, int a, int b,
                               int c, int d, int dtype, int bs_last, float scale, void *workspace,
                               int64_t workspace_bytes, void *stream);
int ksmm_factor_backward_weight(const void *dy, const void *x, void *dw, int64_t batch, int a, int b,
                                int c, int d, int dtype, int bs_last, float scale, void *workspace,
                                int64_t workspace_bytes, void *stream);

/* ksmm_chain_forward_ep for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the ping-pong intermediates
 * and the transposed-route and padded-rows buffers live in a fixed device array inside the library,
 * ksmm_static_scratch_bytes() = 32 MiB per GPU, instead of a caller's workspace.  It has no
 * counterpart in the reference: it exists for the callers named above, those that cannot
 * allocate.  Chains whose ksmm_chain_workspace_layout() exceeds the array return
 * KSMM_ERR_WORKSPACE.  Allocates nothing and frees nothing.  All calls on one GPU share the
 * array (every intermediate is fully written before it is read, so nothing has to be cleared
 * between calls): calls that overlap in time on one GPU race. */
int64_t ksmm_static_scratch_bytes(void);
int ksmm_chain_forward_static(const ksmm_factor_desc *factors, int n_factors, const void *x, void *y,
                              int64_t batch, int x_dtype, int y_dtype, int bs_last, int fuse,
                              const ksmm_epilogue *epilogue, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* KSMM_HIP_H */
