/*
 * endia_hip.h -- C ABI of libendia_hip.so: the MI355X (gfx950) implementation of
 * Endia's reverse-mode dense-layer training step.
 *
 * Conventions (they mirror the data contract of the reference's op plug-in seam,
 * endia/functional/_utils.mojo:208-327 and endia/_array/_array.mojo:523-536):
 *   - every tensor is fp32, row-major; a complex64 tensor is interleaved (re, im) fp32 pairs;
 *   - every data pointer is a DEVICE pointer obtained from endia_hip_malloc (or any
 *     hipMalloc'ed memory of the current device); host pointers appear only in the
 *     memcpy calls and in small descriptor arrays (shapes, strides);
 *   - sizes, leading dimensions and strides are int64 counts of ELEMENTS (complex: of
 *     complex elements), never bytes, except where the name says "bytes";
 *   - every call returns 0 on success or a negative endia_hip_status; the text of the last
 *     failure on the calling thread is returned by endia_hip_last_error();
 *   - work is enqueued on one internal HIP stream in call order and is asynchronous to the
 *     host; endia_hip_sync() (and the d2h copy) block until it has drained;
 *   - the library keeps one global context and is not thread-safe, like the reference,
 *     whose hot path is single-threaded (matmul_op.mojo:168-169).
 */
#ifndef ENDIA_HIP_H
#define ENDIA_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ENDIA_API __attribute__((visibility("default")))

typedef enum {
  ENDIA_HIP_OK = 0,
  ENDIA_HIP_ERR_INVALID = -1,     /* bad argument: null pointer, negative size, bad enum, bad shape */
  ENDIA_HIP_ERR_NOT_INIT = -2,    /* endia_hip_init has not succeeded */
  ENDIA_HIP_ERR_RUNTIME = -3,     /* a HIP runtime call failed */
  ENDIA_HIP_ERR_NOMEM = -4,       /* device allocation failed */
  ENDIA_HIP_ERR_UNSUPPORTED = -5  /* valid request outside what this build implements */
} endia_hip_status;

/* Unary operators. Replaces the per-op forward bodies and VJP rules of
 * endia/functional/unary_ops/<name>_op.mojo. Real arrays take the reference's complex body at
 * imag = 0 (unary_ops/_utils.mojo:113-118), which is why LOG is log|x| and SQRT is 0 for x < 0. */
typedef enum {
  ENDIA_OP_RELU = 0,   /* relu_op.mojo:115-117 ; vjp greater(x,0)*g  relu_op.mojo:95  */
  ENDIA_OP_TANH = 1,   /* tanh_op.mojo:112-115 ; vjp (1-tanh(x)^2)*g tanh_op.mojo:92  */
  ENDIA_OP_SIN = 2,    /* sin_op.mojo:112-114  ; vjp cos(x)*g        sin_op.mojo:92   */
  ENDIA_OP_COS = 3,    /* cos_op.mojo:113-115  ; vjp -sin(x)*g       cos_op.mojo:93   */
  ENDIA_OP_NEG = 4,    /* neg_op.mojo:111-113  ; vjp -g              neg_op.mojo:91   */
  ENDIA_OP_SQUARE = 5, /* square_op.mojo:117-119; vjp 2*x*g          square_op.mojo:96 */
  ENDIA_OP_SQRT = 6,   /* sqrt_op.mojo:111-114 (0 for x<0) ; vjp g/(2*sqrt(x)) sqrt_op.mojo:91 */
  ENDIA_OP_ABS = 7,    /* abs_op.mojo:114-115,157 ; vjp sign(x)*g    abs_op.mojo:93   */
  ENDIA_OP_IDENTITY = 8,
  ENDIA_OP_GREATER0 = 9, /* 1.0 where x > 0 else 0.0: greater_op.mojo:46-60 against a zero operand */
  ENDIA_OP_EXP = 10,     /* exp_op.mojo:113-114 ; vjp exp(x)*g            exp_op.mojo:92     */
  ENDIA_OP_LOG = 11,     /* log_op.mojo:111-114 (log|x|) ; vjp g/x        log_op.mojo:91     */
  ENDIA_OP_SIGMOID = 12, /* sigmoid_op.mojo:118-121 ; vjp out*(1-out)*g   sigmoid_op.mojo:98 */
  ENDIA_OP_SINH = 13,    /* sinh_op.mojo:108-109 ; vjp cosh(x)*g          sinh_op.mojo:88    */
  ENDIA_OP_COSH = 14,    /* cosh_op.mojo:109-110 ; vjp sinh(x)*g          cosh_op.mojo:89    */
  ENDIA_OP_TAN = 15,     /* tan_op.mojo (real) ; vjp g*(1+out^2)          tan_op.mojo:81     */
  ENDIA_OP_ASIN = 16,    /* asin_op.mojo:103 ; vjp g/sqrt(1-x^2)          asin_op.mojo:83    */
  ENDIA_OP_ACOS = 17,    /* acos_op.mojo:111 ; vjp -1/sqrt(1-x^2)*g       acos_op.mojo:91    */
  ENDIA_OP_ATAN = 18,    /* atan_op.mojo:105 ; vjp g/(1+x^2)              atan_op.mojo:85    */
  ENDIA_OP_RECIPROCAL = 19, /* reciprocal_op.mojo:115-117 (x/x^2) ; vjp -g/x^2  reciprocal_op.mojo:95 */
  ENDIA_OP_SIGN = 20     /* sign_op.mojo:78-81 (x/|x|, NaN at 0) ; vjp passes g on (sign_op.mojo:58) */
} endia_hip_unary_op;
#define ENDIA_OP_COUNT 21

/* Binary operators: endia/functional/binary_ops/{add,sub,mul,div,pow}_op.mojo and the comparisons of
 * endia/functional/comparison_ops (1.0 / 0.0 results, real only, not differentiable). */
typedef enum {
  ENDIA_BIN_ADD = 0,
  ENDIA_BIN_SUB = 1,
  ENDIA_BIN_MUL = 2,
  ENDIA_BIN_DIV = 3,
  ENDIA_BIN_GREATER = 4,       /* greater_op.mojo:46-60 */
  ENDIA_BIN_POW = 5,           /* exp(log|a|*b) * cos(arg(a)*b), complex form likewise: pow_op.mojo:139-146 */
  ENDIA_BIN_GREATER_EQUAL = 6, /* greater_equal_op.mojo */
  ENDIA_BIN_LESS = 7,          /* less_op.mojo */
  ENDIA_BIN_LESS_EQUAL = 8,    /* less_equal_op.mojo */
  ENDIA_BIN_EQUAL = 9,         /* equal_op.mojo */
  ENDIA_BIN_NOT_EQUAL = 10     /* not_equal_op.mojo */
} endia_hip_binary_op;
#define ENDIA_BIN_COUNT 11

/* GEMM epilogues (what is applied to the accumulator tile before it is stored). */
typedef enum {
  ENDIA_EPI_NONE = 0,      /* C = AB */
  ENDIA_EPI_BIAS = 1,      /* C = AB + bias[n]                       (x @ W + b, _mlp.mojo:50) */
  ENDIA_EPI_BIAS_ACT = 2,  /* Z = AB + bias[n]; aux_out = Z if non-null; C = act(Z)   (_mlp.mojo:50-52) */
  ENDIA_EPI_ACT_GRAD = 3   /* C = (AB) * act'(aux_in)  -- activation VJP fused into dX = dZ W^T.
                              aux_in is the PRE-activation Z unless ENDIA_ACT_FROM_OUTPUT is or'ed into
                              `act`, in which case it is the stored activation output A = act(Z)
                              (valid for relu and tanh only). */
} endia_hip_epilogue;
#define ENDIA_ACT_FROM_OUTPUT 0x100
#define ENDIA_GEMM_ACCUMULATE 0x200 /* or'ed into `epilogue`: C += result instead of C = result */
#define ENDIA_GEMM_COLSUM_B 0x400  /* or'ed into `epilogue` (with ENDIA_EPI_NONE, transB = 0, batch = 1, ldb = N): aux_out[n] also
                                      receives sum_k B[k][n]. With C = A^T dY this is the bias gradient, the VJP of the broadcast
                                      bias add (expand_op.mojo:121-126), produced by the weight-gradient launch itself */

typedef enum { ENDIA_CGEMM_4M = 0, ENDIA_CGEMM_3M = 1 } endia_hip_cgemm_algo;

/* ---- context ------------------------------------------------------------------------------- */
/* No counterpart in the reference (it has no device); creates the stream and buffer pool. */
ENDIA_API int32_t endia_hip_init(int32_t device);
ENDIA_API int32_t endia_hip_shutdown(void);
ENDIA_API const char* endia_hip_last_error(void);
ENDIA_API int32_t endia_hip_sync(void);
/* Writes a short description of the device ("gfx950 ... CUs ... MHz") into buf. */
ENDIA_API int32_t endia_hip_device_info(char* buf, int64_t buf_bytes, int32_t* cu_count, int32_t* clock_mhz);

/* ---- memory: replaces Node buffer allocation, setup_shape_and_data (functional/_utils.mojo:319-327)
 *      and Node.__del__ (_array.mojo:177-179). Buffers come from a size-bucketed pool, so a freed
 *      buffer is reused by later calls without hipMalloc. malloc does NOT zero the buffer. */
ENDIA_API int32_t endia_hip_malloc(int64_t bytes, void** out);
ENDIA_API int32_t endia_hip_free(void* p);
ENDIA_API int32_t endia_hip_memcpy_h2d(void* dst, const void* src, int64_t bytes);
ENDIA_API int32_t endia_hip_memcpy_d2h(void* dst, const void* src, int64_t bytes); /* blocks */
ENDIA_API int32_t endia_hip_memcpy_d2d(void* dst, const void* src, int64_t bytes);
ENDIA_API int32_t endia_hip_memset0(void* p, int64_t bytes);
ENDIA_API int32_t endia_hip_fill(float* p, int64_t n, float value); /* init_ops.mojo full/ones/zeros */
ENDIA_API int32_t endia_hip_pool_stats(int64_t* bytes_in_use, int64_t* bytes_cached, int64_t* n_device_allocs);
ENDIA_API int32_t endia_hip_pool_trim(void);

/* ---- timing on the library's stream (hipEvent pairs); slots 0..63 ---------------------------- */
ENDIA_API int32_t endia_hip_timer_start(int32_t slot);
ENDIA_API int32_t endia_hip_timer_stop(int32_t slot);
ENDIA_API int32_t endia_hip_timer_elapsed_ms(int32_t slot, float* ms); /* blocks until the stop event */

/* ---- captured steps (HIP graphs). No counterpart in the reference. Calls made between begin and end are
 *      recorded, not executed; endia_hip_graph_launch replays them on the library's stream with one launch.
 *      While capturing, host<->device copies, endia_hip_sync and the timers return ENDIA_HIP_ERR_UNSUPPORTED.
 *      Buffers handed out during the capture stay reserved for the graph until endia_hip_graph_destroy, even
 *      after their holders free them, because the recorded kernels keep their addresses. Scalar arguments
 *      (learning rate, Adam's step counter) are frozen at capture time. */
ENDIA_API int32_t endia_hip_graph_begin(void);
ENDIA_API int32_t endia_hip_graph_end(int64_t* handle);
ENDIA_API int32_t endia_hip_graph_launch(int64_t handle);
ENDIA_API int32_t endia_hip_graph_destroy(int64_t handle);

/* ---- per-launch timing of the MFMA GEMM kernel. Between begin and end every launch of the tiled
 *      fp32 GEMM kernel is bracketed by a pair of HIP events on the library's stream; end blocks, then
 *      reports the number of launches, the sum of their durations and of their 2*M*N*K*batch flops.
 *      Used by the benchmark to state achieved TFLOP/s of the dominant kernel inside the timed region. */
ENDIA_API int32_t endia_hip_gemm_timing_begin(void);
ENDIA_API int32_t endia_hip_gemm_timing_end(int64_t* launches, double* total_ms, double* total_flops);

/* ---- several independent fp32 products in one call. No counterpart in the reference, whose backward pass issues its
 *      matmul VJPs one at a time (autograd/functional.mojo:46-65, matmul_op.mojo:278-283): a second-order pass holds many
 *      products of 1024 x 2048 x 2048 that do not depend on each other, each too small to fill the chip, and members that
 *      fit together share one launch of the 256 x 128 one-wave-per-SIMD tile (one tile per CU); the others run as
 *      endia_hip_sgemm would run them. Results are those of endia_hip_sgemm on every member in turn (the order of the
 *      additions along K may differ). No member's C may overlap another member's A, B or C. epilogue: ENDIA_EPI_NONE
 *      or ENDIA_EPI_BIAS (bias[n] added), optionally | ENDIA_GEMM_ACCUMULATE. count <= 64.
 *      need = -1 runs every member. need = i (a caller that keeps a list of products it has put off and now has to
 *      have member i) runs member i and whichever other members make its launch a better one, and leaves the rest to
 *      the caller. launched (may be null when need = -1) receives one flag per member: 1 = it has been run. */
typedef struct endia_hip_sgemm_desc {
  int32_t transA, transB;
  int64_t M, N, K;
  const float* A;
  int64_t lda;
  const float* B;
  int64_t ldb;
  float* C;
  int64_t ldc;
  int32_t epilogue;
  const float* bias;
} endia_hip_sgemm_desc;
ENDIA_API int32_t endia_hip_sgemm_grouped(int32_t count, const endia_hip_sgemm_desc* members, int32_t need, int32_t* launched);

/* Tile choice of the fp32 matrix-core kernels behind endia_hip_sgemm (and everything built on it). No counterpart in the
 * reference: a hook for tests and tuning. tile = 0 (the default) lets every call choose by shape; 64, 128, 256 or 256128
 * makes every later call that runs on the matrix cores use the 64 x 64, 128 x 128, 256 x 256 or 256 x 128 tile (all
 * transpose forms and epilogues; a call that no matrix-core kernel takes, e.g. unaligned operands, keeps its own path). Results do not
 * depend on the tile beyond the order of the additions along K. Process-wide, not thread-safe against concurrent
 * sgemm calls. */
ENDIA_API int32_t endia_hip_gemm_force_tile(int32_t tile);

/* ---- strided gather copy: execute_copy_raw / contiguous (functional/_utils.mojo:79-205).
 *      dst is contiguous row-major of `shape`; src element (i0..i_{r-1}) is at
 *      src[offset + sum i_d*stride_d]; stride 0 broadcasts. ndim <= 8. is_complex copies pairs. */
ENDIA_API int32_t endia_hip_strided_copy(int32_t ndim, const int64_t* shape, const int64_t* src_strides,
                               int64_t src_offset, const float* src, float* dst, int32_t is_complex);

/* ---- strided scatter, the store side of a view: Pad.__call__ (view_ops/pad_op.mojo:115-142) writes its
 *      argument through a slice view of a zeroed target (this is also the gradient of a slice,
 *      array_slice_op.mojo:104-120), and AsStridedInv.__call__ (view_ops/as_strided_op.mojo:169-190), the
 *      gradient of as_strided, adds it through an as_strided view of a zeroed target.
 *      dst[dst_offset + sum i_d*stride_d] = src[i0..i_{r-1}] (+= when accumulate), src contiguous row-major
 *      of `shape`, strides >= 0, ndim <= 8; dst is not cleared. accumulate = 0 requires a view whose
 *      elements are distinct (checked); accumulate = 1 allows overlapping windows: the additions are
 *      atomic and their order, hence the last bit of a sum, is not fixed. is_complex moves pairs. */
ENDIA_API int32_t endia_hip_strided_scatter(int32_t ndim, const int64_t* shape, const int64_t* dst_strides,
                                  int64_t dst_offset, const float* src, float* dst, int32_t accumulate,
                                  int32_t is_complex);

/* ---- fp32 GEMM: matmul_fwd (binary_ops/matmul_op.mojo:93-254) and both products of matmul_vjp
 *      (matmul_op.mojo:278-283). C[b] = opA(A[b]) . opB(B[b]), C is M x N with row stride ldc.
 *      transA = 0: A is M x K, element (m,k) at A[m*lda + k];  transA = 1: A is stored K x M, element
 *      (m,k) at A[k*lda + m]. Same for B (K x N, or stored N x K when transB = 1). The transposed
 *      forms replace the reference's materialised .T() copies (matmul_op.mojo:111-136).
 *      batch >= 1; a batch stride of 0 broadcasts that operand (matmul_op.mojo:162-165).
 *      epilogue: endia_hip_epilogue, optionally | ENDIA_GEMM_ACCUMULATE | ENDIA_GEMM_COLSUM_B.
 *      act: endia_hip_unary_op in {RELU,TANH,SIN,IDENTITY}, optionally | ENDIA_ACT_FROM_OUTPUT.
 *      bias: N floats (BIAS, BIAS_ACT) else null.  aux_in: M x N, row stride ldc (ACT_GRAD) else null.
 *      aux_out: M x N, row stride ldc, or null (BIAS_ACT); N floats (COLSUM_B). */
ENDIA_API int32_t endia_hip_sgemm(int32_t transA, int32_t transB, int64_t M, int64_t N, int64_t K,
                        const float* A, int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                        int64_t batch, int64_t strideA, int64_t strideB, int64_t strideC,
                        int32_t epilogue, int32_t act, const float* bias, const float* aux_in,
                        float* aux_out);

/* ---- backward of one dense layer y = act(x W + b) in one call: both products of matmul_vjp
 *      (matmul_op.mojo:278-283), the bias gradient (Expand.vjp, expand_op.mojo:121-126) and the activation
 *      derivative of the layer BELOW on the way out (relu_op.mojo:95, tanh_op.mojo:92, sin_op.mojo:92).
 *      x [B,K], W [K,N], g [B,N] = cotangent of x W + b (contiguous, row-major).
 *        dx [B,K] = (g W^T) * act'(aux)   when aux [B,K] is given (act as in endia_hip_sgemm's ACT_GRAD epilogue,
 *                                          optionally | ENDIA_ACT_FROM_OUTPUT), else g W^T
 *        dW [K,N] = x^T g,   db [N] = sum over rows of g.        Any of dx, dW, db may be null.
 *      When all three are wanted and the layer is small (B and N at most 128) they come from ONE launch; otherwise
 *      the call is the corresponding endia_hip_sgemm calls. The results are those calls' results either way. */
ENDIA_API int32_t endia_hip_linear_bwd(int64_t B, int64_t K, int64_t N, const float* x, const float* W, const float* g,
                             int32_t act, const float* aux, float* dx, float* dW, float* db);

/* ---- a whole small dense model per call: nn.MLP.forward (nn/modules/_mlp.mojo:47-53: h_l = act(h_{l-1} W_l + b_l), no
 *      activation after the last layer) and the backward pass of that chain (matmul_vjp matmul_op.mojo:278-283,
 *      Expand.vjp expand_op.mojo:121-126, relu_op.mojo:95 / tanh_op.mojo:92), for models whose layers are at most
 *      ENDIA_MLP_MAX_WIDTH wide, like the reference's own benchmark model (benchmarks/mlp_benchmarks/mlp_imp.mojo:35-37).
 *      Every row of the batch is independent through all layers, so the forward pass is ONE launch (a work-group keeps
 *      16 rows' activations in LDS from the first layer to the last) and the backward pass two (the chain of cotangents
 *      the same way, then every dW_l and db_l at once), instead of one to three launches per layer.
 *      widths[0..layers]: input width, then each layer's output width. W[l] is [widths[l], widths[l+1]] row-major, b[l]
 *      is [widths[l+1]], x is [batch, widths[0]], all contiguous. act in {RELU, TANH, IDENTITY} follows every layer but
 *      the last. A weight matrix may start at any float; every other array (x, b, h, target, delta, dW, db, dx) must
 *      start on a 16-byte boundary (ENDIA_HIP_ERR_INVALID otherwise): they are read and written 16 bytes at a time.
 *      fwd: h[l] receives layer l's output [batch, widths[l+1]] (h[layers-1] is the model's output; the others are what
 *           the backward pass needs).
 *      bwd: delta[layers-1] holds the cotangent of the output on entry; delta[l] for l < layers-1 are buffers
 *           [batch, widths[l+1]] that receive the cotangents of the pre-activations. dW[l] = h[l-1]^T delta[l] (x for
 *           l = 0), db[l] = column sums of delta[l]; entries of dW / db may be null. dx [batch, widths[0]] or null. */
#define ENDIA_MLP_MAX_LAYERS 16
#define ENDIA_MLP_MAX_WIDTH 128
typedef struct endia_hip_mlp_desc {
  int32_t layers;
  int32_t act; /* endia_hip_unary_op */
  int64_t batch;
  int64_t widths[ENDIA_MLP_MAX_LAYERS + 1];
} endia_hip_mlp_desc;
ENDIA_API int32_t endia_hip_mlp_fwd(const endia_hip_mlp_desc* desc, const float* x, const float* const* W, const float* const* b,
                          float* const* h);
/* endia_hip_mlp_fwd with the MSE loss of the reference's training script on top (mlp_imp.mojo:56-60: forward, then
 * mse_op.mojo:17-20), in the same launch: loss (one device float) = mean((h[layers-1] - target)^2), and dpred
 * [batch, widths[layers]] (may be null) = 2 (h[layers-1] - target) / n, which is what endia_hip_mlp_bwd takes as
 * delta[layers-1]. The work-groups' partial sums are added in row order by the last one to finish. */
ENDIA_API int32_t endia_hip_mlp_fwd_mse(const endia_hip_mlp_desc* desc, const float* x, const float* const* W,
                              const float* const* b, const float* target, float* const* h, float* dpred, float* loss);
ENDIA_API int32_t endia_hip_mlp_bwd(const endia_hip_mlp_desc* desc, const float* x, const float* const* W, const float* const* h,
                          float* const* delta, float* const* dW, float* const* db, float* dx);
/* The training step of mlp_imp.mojo:56-66 (forward, mse, backward) split so that the backward pass is one launch:
 * endia_hip_mlp_fwd_mse_delta is endia_hip_mlp_fwd_mse that goes on, in the same launch for batches of up to 2048 rows,
 * to the cotangents of ALL layers for the loss gradient 2 (h[layers-1] - target) / n (every row of the batch is
 * independent through the whole chain): delta[l] [batch, widths[l+1]], none null, and dx [batch, widths[0]] when not
 * null, exactly what endia_hip_mlp_bwd leaves there when its delta[layers-1] is that loss gradient.
 * endia_hip_mlp_wgrad is the rest of endia_hip_mlp_bwd: dW[l] = h[l-1]^T delta[l] (h[-1] = x) and db[l] = the column
 * sums of delta[l], for the layers whose pointers are not null. */
ENDIA_API int32_t endia_hip_mlp_fwd_mse_delta(const endia_hip_mlp_desc* desc, const float* x, const float* const* W,
                                    const float* const* b, const float* target, float* const* h, float* const* delta,
                                    float* loss, float* dx);
ENDIA_API int32_t endia_hip_mlp_wgrad(const endia_hip_mlp_desc* desc, const float* x, const float* const* h,
                            const float* const* delta, float* const* dW, float* const* db);

/* ---- complex64 GEMM: the complex branch of matmul_fwd (matmul_op.mojo:201-238). Interleaved
 *      operands; lda/ldb/ldc and strides count complex elements. conjA/conjB conjugate the operand
 *      (the reference's VJP does not conjugate, matmul_op.mojo:278-283; the Wirtinger convention does).
 *      algo 4M forms the four real products of matmul_op.mojo:216-217; 3M uses three. */
ENDIA_API int32_t endia_hip_cgemm(int32_t transA, int32_t conjA, int32_t transB, int32_t conjB, int64_t M,
                        int64_t N, int64_t K, const float* A, int64_t lda, const float* B, int64_t ldb,
                        float* C, int64_t ldc, int64_t batch, int64_t strideA, int64_t strideB,
                        int64_t strideC, int32_t algo, int32_t accumulate);

/* ---- elementwise: execute_unary_op (unary_ops/_utils.mojo:77-134) and the VJP rules listed at
 *      endia_hip_unary_op. n counts elements (complex: complex elements). In-place (y == x) allowed.
 *      Complex forward is implemented for NEG, SQUARE, IDENTITY, SIN, COS, TANH, EXP, LOG, SINH, COSH,
 *      SQRT, RECIPROCAL and SIGN; ABS with is_complex writes n REAL values |z| (abs_op.mojo:114-115,157). */
ENDIA_API int32_t endia_hip_unary_fwd(int32_t op, int64_t n, const float* x, float* y, int32_t is_complex);
/* dx = g * op'(x). Complex: NEG, SQUARE, IDENTITY, and ABS, for which g is real (n floats) and x and dx
 * are complex: dx = g*z/|z|. */
ENDIA_API int32_t endia_hip_unary_vjp(int32_t op, int64_t n, const float* x, const float* g, float* dx,
                            int32_t is_complex);

/* dx = g * op'(x) computed from the stored OUTPUT y = op(x) instead of x: RELU (y > 0), TANH (1 - y^2),
 * SQRT (1 / (2y)), EXP (y), SIGMOID (y(1-y)), TAN (1 + y^2), IDENTITY. Equal to endia_hip_unary_vjp where the reference recomputes the forward
 * (tanh_op.mojo:92) but without the second transcendental pass. Real only. */
ENDIA_API int32_t endia_hip_unary_vjp_from_output(int32_t op, int64_t n, const float* y, const float* g, float* dx);

/* ---- fused elementwise program: a run of elementwise ops in one pass over memory. Replaces the
 *      reference's fused unary runs (simd_op_list + execute_fwds, endia/_array/_array.mojo:90-101,756-782)
 *      and stands in for its JIT-compiled elementwise subgraphs (endia/compile/fx.mojo:105-159).
 *      Every lane interprets `steps` on an accumulator `acc` (0 at the start) and 4 save slots:
 *        LOAD     acc = operand            UNARY    acc = op(acc)           (endia_hip_unary_op)
 *        BINARY   acc = op(acc, operand)   RBINARY  acc = op(operand, acc)  (endia_hip_binary_op)
 *        SAVE     slot[src_index] = acc    STORE    outputs[src_index][i] = acc
 *      An operand is input `src_index` (src_kind INPUT), slot `src_index` (SLOT; an earlier step must
 *      have saved it) or `imm` (IMM).
 *      Inputs are real fp32: FULL = [rows*cols] contiguous, ROW_VECTOR = [cols] broadcast over rows,
 *      SCALAR = one element. Outputs are [rows*cols]; every output must be stored by some step. */
typedef enum { ENDIA_EW_LOAD = 0, ENDIA_EW_UNARY = 1, ENDIA_EW_BINARY = 2, ENDIA_EW_RBINARY = 3, ENDIA_EW_SAVE = 4,
               ENDIA_EW_STORE = 5 } endia_hip_ew_kind;
typedef enum { ENDIA_EW_SRC_INPUT = 0, ENDIA_EW_SRC_SLOT = 1, ENDIA_EW_SRC_IMM = 2 } endia_hip_ew_src;
typedef enum { ENDIA_EW_FULL = 0, ENDIA_EW_ROW_VECTOR = 1, ENDIA_EW_SCALAR = 2 } endia_hip_ew_mode;
typedef struct endia_hip_ew_step {
  int32_t kind;      /* endia_hip_ew_kind */
  int32_t op;        /* unary or binary op code, for UNARY / BINARY / RBINARY */
  int32_t src_kind;  /* endia_hip_ew_src, for LOAD / BINARY / RBINARY */
  int32_t src_index; /* input, slot or output index */
  float imm;
} endia_hip_ew_step;
#define ENDIA_EW_MAX_INPUTS 8
#define ENDIA_EW_MAX_OUTPUTS 4
#define ENDIA_EW_MAX_SLOTS 4
#define ENDIA_EW_MAX_STEPS 48
ENDIA_API int32_t endia_hip_ew_program(int64_t rows, int64_t cols, int32_t n_inputs, const float* const* inputs,
                             const int32_t* input_modes, int32_t n_outputs, float* const* outputs,
                             int32_t n_steps, const endia_hip_ew_step* steps);

/* ---- broadcasting binary op: binary_op_array + execute_binary_op (binary_ops/_utils.mojo:57-177).
 *      out is contiguous row-major of `shape`; a and b are addressed through element strides
 *      (0 = broadcast axis) so the reference's materialised expand copies are never made. ndim <= 8. */
ENDIA_API int32_t endia_hip_binary(int32_t op, int32_t ndim, const int64_t* shape, const int64_t* a_strides,
                         const int64_t* b_strides, const float* a, const float* b, float* out,
                         int32_t is_complex);
/* out[i] = alpha * a[i] + beta * b[i]  (gradient accumulation `add`, autograd/functional.mojo:55-57,
 * and scalar scaling such as Div by a full([1], n) operand, _array.mojo:1041-1043). b may be null. */
ENDIA_API int32_t endia_hip_axpby(int64_t n, float alpha, const float* a, float beta, const float* b, float* out);

/* out[i] = (re[i], im[i]) as interleaved complex; im may be null (imaginary part 0). Replaces
 * complex(real, imag) (init_ops.mojo:419-433), which Real.vjp uses (view_ops/real_op.mojo:74-77). */
ENDIA_API int32_t endia_hip_complex_pack(int64_t n, const float* re, const float* im, float* out);

/* ---- reductions: ReduceAdd.__call__ (reduce_ops/reduce_add_op.mojo:65-210) -- also Expand.vjp, the
 *      bias gradient (view_ops/expand_op.mojo:121-126) -- and sum / mean (sum_op.mojo:35-62,
 *      mean_op.mojo:35-65). x is contiguous row-major of `shape`; axes with reduce_mask bit d set are
 *      summed and kept as size 1; out is contiguous of the reduced shape. scale multiplies the result
 *      (1/count for mean). ndim <= 8. is_complex reduces pairs. */
ENDIA_API int32_t endia_hip_reduce_add(int32_t ndim, const int64_t* shape, uint32_t reduce_mask, const float* x,
                             float* out, float scale, int32_t is_complex);

/* ---- column sums without any allocation. No counterpart in the reference: a variant of endia_hip_reduce_add for
 *      callers that cannot allocate device memory (code under HIP-graph capture, tight serving loops, harnesses that
 *      forbid hipMalloc). out[c] = scale * sum_r x[r][c] for a contiguous row-major x of R rows and C columns: the
 *      bias gradient db = 1^T dZ, i.e. endia_hip_reduce_add with ndim = 2 and reduce_mask = 1, and the same result bit
 *      for bit (the row splits that call chooses on a 256-CU device never need more than 262144 partial sums; on a
 *      device where they would, the rows are cut into fewer pieces and the last bits may differ). The partial sums of its first stage live in a 1 MiB array
 *      that is part of the library's device image instead of the library's growing workspace, so the call performs no
 *      hipMalloc / hipFree. C above 262144 is refused with ENDIA_HIP_ERR_INVALID. Every call on a device uses that
 *      device's one array: calls that overlap on one device (two host threads, two processes' worth of streams)
 *      race; calls on the library's single stream, the only kind this ABI issues, are ordered. */
ENDIA_API int32_t endia_hip_col_sum_static(int64_t R, int64_t C, const float* x, float* out, float scale);
/* Several column sums in one call: out[c] = scale * sum_r x[r][c] for every member, each the result, bit for bit, of
 * endia_hip_reduce_add(2, {R, C}, 1, x, out, scale, 0). No counterpart in the reference, whose reverse walk reduces one
 * bias gradient at a time (expand_op.mojo:121-126 from autograd/functional.mojo:46-65): a second-order pass over a
 * few 2048-wide layers leaves eight such sums of [1024, 2048] that nothing reads until the pass is over, each a
 * launch of 7 us that is mostly launch; members of that size share one launch, the others run as the single call
 * runs them. No member's output may be another member's output or input (members run concurrently). count <= 64. */
typedef struct endia_hip_col_sum_desc {
  int64_t R, C;
  const float* x;
  float* out;
  float scale;
} endia_hip_col_sum_desc;
ENDIA_API int32_t endia_hip_col_sum_multi(int32_t count, const endia_hip_col_sum_desc* members);
/* How a column sum of R rows and C columns cuts its rows on a device of cu_count CUs when scratch_floats floats are
 * there for first-stage partial sums (0: no limit, what endia_hip_reduce_add has; 262144: endia_hip_col_sum_static).
 * aligned16: x and out start on 16-byte boundaries. No counterpart in the reference; pure arithmetic, needs no device
 * and no endia_hip_init. splits = 0: one launch without a first stage (small inputs, and aligned inputs of up to 2^22
 * elements and 2048 rows); -1: C does not fit the scratch; otherwise `splits` pieces of rows_per_split rows. Two calls
 * that get the same plan add in the same order and agree bit for bit. */
ENDIA_API int32_t endia_hip_col_sum_plan(int64_t R, int64_t C, int64_t cu_count, int64_t scratch_floats, int32_t aligned16,
                                         int64_t* splits, int64_t* rows_per_split);

/* ---- the other reductions: ReduceMax / ReduceMin / ReduceMul .__call__ (reduce_ops/reduce_max_op.mojo:66-190,
 *      reduce_min_op.mojo:66-190, reduce_mul_op.mojo:65-210) and ReduceArgMax / ReduceArgMin .__call__
 *      (reduce_argmax_op.mojo:66-163, reduce_argmin_op.mojo:66-163). Same layout contract as
 *      endia_hip_reduce_add (kept axes of size 1, ndim <= 8, real arrays). The arg variants reduce exactly one
 *      axis and write the position along it as a float (the reference's arrays hold fp32 only): the first
 *      position whose value is strictly greater (smaller) than everything before it, -1 when no value exceeds
 *      the starting value -inf (+inf), as the reference's loop leaves it. An empty reduction yields the
 *      starting value: -inf, +inf, 1, -1. */
typedef enum {
  ENDIA_REDUCE_MAX = 0,
  ENDIA_REDUCE_MIN = 1,
  ENDIA_REDUCE_MUL = 2,
  ENDIA_REDUCE_ARGMAX = 3,
  ENDIA_REDUCE_ARGMIN = 4
} endia_hip_reduce_op;
ENDIA_API int32_t endia_hip_reduce(int32_t op, int32_t ndim, const int64_t* shape, uint32_t reduce_mask, const float* x,
                         float* out);

/* ---- loss: mse (loss_ops/mse_op.mojo:17-20) and its gradient 2(p-t)/n as produced by the
 *      sub/mul/sum/div VJP chain. loss is one device float; dpred may be null (forward only);
 *      loss may be null (gradient only). */
ENDIA_API int32_t endia_hip_mse_fwd_bwd(int64_t n, const float* pred, const float* target, float* loss,
                              float* dpred);

/* ---- conv2d, NCHW, groups = 1: Conv2d.__call__ (spacial_ops/conv2d_op.mojo:88-196), output shape
 *      rule conv2d_op.mojo:31-85. The three gradients have no counterpart in the reference, whose
 *      Conv2d.vjp is default_vjp (conv2d_op.mojo:198-200); they are the adjoints of that forward loop.
 *      x [N,C,H,W], w [K,C,R,S], bias [K] or null, y/dy [N,K,P,Q]. */
typedef struct {
  int64_t N, C, H, W, K, R, S;
  int64_t stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, groups;
} endia_hip_conv2d_desc;
ENDIA_API int32_t endia_hip_conv2d_out_shape(const endia_hip_conv2d_desc* d, int64_t* P, int64_t* Q);
/* act in {IDENTITY, RELU}: y = act(conv(x,w)+bias). */
ENDIA_API int32_t endia_hip_conv2d_fwd(const endia_hip_conv2d_desc* d, const float* x, const float* w,
                             const float* bias, float* y, int32_t act);
ENDIA_API int32_t endia_hip_conv2d_bwd_data(const endia_hip_conv2d_desc* d, const float* dy, const float* w,
                                  float* dx);
ENDIA_API int32_t endia_hip_conv2d_bwd_weight(const endia_hip_conv2d_desc* d, const float* x, const float* dy,
                                    float* dw);
ENDIA_API int32_t endia_hip_conv2d_bwd_bias(const endia_hip_conv2d_desc* d, const float* dy, float* db);
/* Every gradient of y = relu(conv(x,w)+bias) in one call, from the stored y (what endia_hip_conv2d_fwd wrote with
 * act = RELU): the ReLU's derivative [y > 0] (relu_op.mojo:51-53) is applied to dy inside the gradient kernels, as
 * they load it, where that is faster than a pass of its own (always for a scalar dy, and for the weight and bias
 * gradients of a tensor dy), and db comes out of the weight-gradient launch.
 * dy_is_scalar != 0: dy points at ONE device float that stands for every element of the cotangent (the gradient
 * of a mean or a sum). dx, dw, db may each be null; x is read only for dw, w only for dx. */
ENDIA_API int32_t endia_hip_conv2d_bwd_relu(const endia_hip_conv2d_desc* d, const float* x, const float* w,
                                  const float* y, const float* dy, int32_t dy_is_scalar, float* dx, float* dw,
                                  float* db);

/* Kernel choice of the 3 x 3 weight gradient. No counterpart in the reference: a hook for tests and tuning, like
 * endia_hip_gemm_force_tile. path = 0 (the default) chooses by shape; 1 keeps every weight gradient on the gather
 * kernels; 2 runs the cached-rows kernel on every shape it can compute, also where few channels would leave most of
 * its tile multiplying zeros. Results do not depend on the path beyond the order of the additions. Process-wide, not
 * thread-safe against concurrent convolution calls. */
ENDIA_API int32_t endia_hip_conv_force_path(int32_t path);

/* ---- conv3d, [N,C,D,H,W] with kernel [K,C,T,R,S], groups = 1: Conv3d.__call__ (spacial_ops/conv3d_op.mojo:104-259),
 *      output extents per axis (in + 2*pad - dil*(k-1) - 1) / stride + 1 (conv3d_op.mojo:71-101). Conv1d
 *      (spacial_ops/conv1d_op.mojo) is conv2d on a height-1 image. Same kernels as conv2d, which is the case
 *      D = T = 1; the three gradients are the adjoints of the forward loop (the reference has none:
 *      Conv3d.vjp = default_vjp). Array order in stride / padding / dilation: depth, height, width. */
typedef struct endia_hip_conv3d_desc {
  int64_t N, C, D, H, W, K, T, R, S;
  int64_t stride[3], padding[3], dilation[3];
  int64_t groups;
} endia_hip_conv3d_desc;
ENDIA_API int32_t endia_hip_conv3d_out_shape(const endia_hip_conv3d_desc* desc, int64_t* out_dhw);
ENDIA_API int32_t endia_hip_conv3d_fwd(const endia_hip_conv3d_desc* desc, const float* x, const float* w, const float* bias,
                             float* y, int32_t act);
ENDIA_API int32_t endia_hip_conv3d_bwd_data(const endia_hip_conv3d_desc* desc, const float* dy, const float* w, float* dx);
ENDIA_API int32_t endia_hip_conv3d_bwd_weight(const endia_hip_conv3d_desc* desc, const float* x, const float* dy, float* dw);
ENDIA_API int32_t endia_hip_conv3d_bwd_bias(const endia_hip_conv3d_desc* desc, const float* dy, float* db);

/* ---- pooling over 1, 2 or 3 spatial axes of a contiguous [N, C, D, H, W] array (set the unused leading
 *      axes to extent 1 with kernel 1, stride 1, padding 0, dilation 1). Forward: MaxPool{1,2,3}d.__call__
 *      (spacial_ops/max_pool2d_op.mojo:88-150 and siblings), AvgPool{1,2,3}d.__call__
 *      (spacial_ops/avg_pool2d_op.mojo:84-140 and siblings); output extent per axis
 *      (in + 2*pad - dil*(k-1) - 1) / stride + 1 (max_pool2d_op.mojo:57-82). Taps outside the array are
 *      skipped: max over the taps inside (-inf if none), average = sum / number of taps inside (0 if none).
 *      The reference has no backward rule for pooling (vjp = default_vjp, max_pool2d_op.mojo:152-154);
 *      endia_hip_pool_bwd is the adjoint of the forward loop. For max pooling the forward writes, per
 *      output, the flat (d*H + h)*W + w position of the first tap that attains the maximum into `argmax`
 *      (may be null if no gradient is needed) and the backward reads it; average pooling ignores it. */
typedef enum { ENDIA_POOL_MAX = 0, ENDIA_POOL_AVG = 1 } endia_hip_pool_mode;
typedef struct endia_hip_pool_desc {
  int64_t N, C, D, H, W;
  int64_t kernel[3], stride[3], padding[3], dilation[3]; /* order: depth, height, width */
} endia_hip_pool_desc;
ENDIA_API int32_t endia_hip_pool_out_shape(const endia_hip_pool_desc* desc, int64_t* out_dhw);
ENDIA_API int32_t endia_hip_pool_fwd(const endia_hip_pool_desc* desc, int32_t mode, const float* x, float* y,
                           int32_t* argmax);
ENDIA_API int32_t endia_hip_pool_bwd(const endia_hip_pool_desc* desc, int32_t mode, const float* dy,
                           const int32_t* argmax, float* dx);

/* ---- optimizers: SGD.step plain path (optim/sgd.mojo:61-62) and Adam.step (optim/adam.mojo:47-65),
 *      each as one pass over the parameter. t is Adam's fp32 step counter (starts at 1, adam.mojo:40). */
ENDIA_API int32_t endia_hip_sgd_step(int64_t n, float* p, const float* g, float lr);
/* The same update for `count` parameter tensors in one launch (n, p, g are host arrays of length count): a model
 * of many small tensors, like the reference's sine-fit MLP, is bound by launch latency rather than bandwidth. */
ENDIA_API int32_t endia_hip_sgd_step_multi(int32_t count, const int64_t* n, float* const* p, const float* const* g, float lr);
/* Adam.step for `count` tensors with the step counter t in DEVICE memory (`step`: one float, 1 before the first
 * step): the kernels read it, compute 1 - beta^t themselves, and a last tiny kernel adds 1 to it after all
 * parameters (adam.mojo:65). No argument changes from one step to the next, so the call can be recorded into a
 * captured step and replayed. beta^t comes from the device's powf here and from the host's in endia_hip_adam_step:
 * the two may differ in the last bit of the bias corrections (1e-7 relative in the update). */
ENDIA_API int32_t endia_hip_adam_step_multi(int32_t count, const int64_t* n, float* const* p, const float* const* g,
                                  float* const* m, float* const* v, float lr, float beta1, float beta2, float eps,
                                  float* step);
/* SGD with momentum and / or weight decay (optim/sgd.mojo:42-60): vel = momentum*vel - lr*(g + wd*p); p += vel
 * (without momentum: p -= lr*(g + wd*p); vel may then be null). Adagrad (optim/adagrad.mojo:36-45):
 * cache += g*g; p -= lr*g / (sqrt(cache) + eps). RMSprop (optim/rmsprop.mojo:39-53):
 * cache = alpha*cache + (1-alpha)*g*g; p -= lr*g / (sqrt(cache) + eps). One pass each. */
ENDIA_API int32_t endia_hip_sgd_momentum_step(int64_t n, float* p, const float* g, float* vel, float lr, float momentum,
                                    float weight_decay);
ENDIA_API int32_t endia_hip_adagrad_step(int64_t n, float* p, const float* g, float* cache, float lr, float eps);
ENDIA_API int32_t endia_hip_rmsprop_step(int64_t n, float* p, const float* g, float* cache, float lr, float alpha, float eps);
ENDIA_API int32_t endia_hip_adam_step(int64_t n, float* p, const float* g, float* m, float* v, float lr,
                            float beta1, float beta2, float eps, float t);

#ifdef __cplusplus
}
#endif
#endif /* ENDIA_HIP_H */
