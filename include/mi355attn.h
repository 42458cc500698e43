/*
 * mi355attn -- C ABI of the MI355X (gfx950) attention library.
 *
 * This is the boundary a host language binds with its FFI (Julia `ccall`, Python
 * `ctypes`, ...).  Plain pointers and sizes only.  It replaces, for device arrays,
 * the following pieces of NNlib.jl (paths relative to the NNlib.jl source tree):
 *
 *   dot_product_attention / _dot_product_attention      src/attention.jl:40-101
 *   dot_product_attention_scores                        src/attention.jl:112-127
 *   apply_attn_bias / apply_attn_mask                   src/attention.jl:129-138
 *   make_causal_mask                                    src/attention.jl:149-153
 *   softmax / softmax! / _softmax! (dims = 1)           src/softmax.jl:56-79
 *   batched_mul! -> _batched_gemm! backend hook         src/batched/batchedmul.jl:238-298
 *   batched_gemm! (CPU backend being replaced)          src/gemm.jl:89-188
 *   rocBLAS hook of the AMDGPU extension                ext/NNlibAMDGPUExt/batched_mul.jl:11-24
 *
 * Conventions
 *   - Every array is column-major (Julia layout).  A (E, L, B) array stores element
 *     (d, i, b) at d + i*E + b*E*L.  Heads are feature slices: head h owns features
 *     [h*D, (h+1)*D), D = E / H  (split_heads, src/attention.jl:158).
 *   - All pointers passed to op entry points are DEVICE pointers owned by the caller.
 *     Op entry points never allocate or free device memory and are asynchronous on
 *     the given stream (NULL = the default stream).
 *   - Every function returns an int32 status; 0 = MI_OK.  No exception crosses the
 *     boundary.  mi_last_error_string() gives a thread-local message for the last
 *     non-zero status returned on the calling thread.
 */
#ifndef MI355ATTN_H
#define MI355ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355ATTN_VERSION 100 /* major*10000 + minor*100 + patch */

/* ---- status codes ---------------------------------------------------------------- */
enum {
    MI_OK = 0,
    MI_EINVAL = 1,       /* null pointer, negative size, bad flag                       */
    MI_EDTYPE = 2,       /* dtype not one of MI_F32 / MI_F16 / MI_BF16                  */
    MI_ESHAPE = 3,       /* sizes inconsistent (the reference throws ArgumentError /    */
                         /* DimensionMismatch for the same conditions)                  */
    MI_EHIP = 4,         /* a HIP runtime call failed; message carries hipGetErrorString */
    MI_ENOMEM = 5,       /* device allocation failed (mi_malloc only)                   */
    MI_EWORKSPACE = 6    /* workspace missing or smaller than mi_attention_workspace_size */
};

/* ---- element types --------------------------------------------------------------- */
enum {
    MI_F32 = 0, MI_F16 = 1, MI_BF16 = 2,
    /* MI_F64: mi_batched_gemm_f64 / mi_batched_mul_generic, the softmax family (mi_softmax*, mi_logsumexp*), the forward
     * attention calls (mi_attention_fwd / _plan / _fwd_static; double-precision vector kernels, what the reference computes
     * for Float64 arrays: src/softmax.jl:56, test/attention.jl:17-34) and mi_convert.  The others: mi_batched_mul_generic
     * only, and the integers as a source of mi_convert (float(T) of an integer array is Float64).  Every other entry
     * point answers MI_EDTYPE for them. */
    MI_F64 = 3, MI_C64 = 4 /* ComplexF32 */, MI_C128 = 5 /* ComplexF64 */, MI_I32 = 6, MI_I64 = 7
};

typedef void *mi_stream; /* a hipStream_t */
typedef void *mi_event;  /* a hipEvent_t  */

/* ---- runtime: device memory, streams, events ------------------------------------- */
/* The reference has no counterpart: its CPU path uses Julia's GC'd Arrays.  These exist
 * so that a host language without a HIP binding can own device buffers. */
int32_t mi_version(void);
const char *mi_last_error_string(void);
int32_t mi_init(int32_t device); /* select device, verify it is gfx950; idempotent */
int32_t mi_device_count(int32_t *count);
int32_t mi_device_name(char *buf, size_t buflen);
int32_t mi_malloc(void **ptr, size_t bytes);
int32_t mi_free(void *ptr);
int32_t mi_memcpy_h2d(void *dst, const void *src, size_t bytes, mi_stream stream);
int32_t mi_memcpy_d2h(void *dst, const void *src, size_t bytes, mi_stream stream);
int32_t mi_memcpy_d2d(void *dst, const void *src, size_t bytes, mi_stream stream);
int32_t mi_fill_zero(void *ptr, size_t bytes, mi_stream stream); /* fill kernel, graph-capture safe */
int32_t mi_stream_create(mi_stream *stream);
int32_t mi_stream_destroy(mi_stream stream);
int32_t mi_stream_sync(mi_stream stream);
int32_t mi_device_sync(void);
int32_t mi_event_create(mi_event *event);
int32_t mi_event_destroy(mi_event event);
int32_t mi_event_record(mi_event event, mi_stream stream);
int32_t mi_event_sync(mi_event event);
int32_t mi_event_elapsed_ms(mi_event start, mi_event stop, float *ms);

/* ---- attention ------------------------------------------------------------------- */

/* Which kernel family mi_attention_fwd picked (reported by mi_attention_plan). */
enum {
    MI_ATTN_KERNEL_GENERIC = 0,  /* any shape / dtype, scalar FMA                        */
    MI_ATTN_KERNEL_FLASH16 = 1,  /* f16 / bf16 MFMA flash forward, head dims 8..256 (x8) */
    MI_ATTN_KERNEL_FLASH32 = 2,  /* f32 MFMA flash forward, head dims 4..128 (x4): Float32 in, out and accumulation;
                                    products as six bf16 matrix instructions on three bf16 planes per operand (Float32
                                    accuracy), or the Float32 instruction if MI355ATTN_F32_MFMA=1 is in the environment
                                    (the gradient kernels of this family: the same for calls without bias / mask arrays
                                    and dropout, the Float32 instruction otherwise).  On the planes a finite q, k or v
                                    entry above the largest bf16 (|x| > 3.3895e38) gives NaN products; calls with a
                                    128-wide head tile, a bias or mask array and the weights output always use the
                                    Float32 instruction */
    MI_ATTN_KERNEL_DECODE = 3    /* split-kv bandwidth-bound path for one to four queries (L_q <= 4) */
};

/* flags */
#define MI_ATTN_FORCE_GENERIC 1u /* use the generic kernel regardless of shape (testing) */

/*
 * One call of dot_product_attention(q, k, v, bias; mask, nheads) with fdrop = identity
 * (src/attention.jl:52-84), or of dot_product_attention_scores when `out` is NULL
 * (src/attention.jl:112-127; the 4-D (D, H, L, B) inputs of that function have the
 * same memory layout as the 3-D (D*H, L, B) ones).
 *
 *   q   (E,  Lq,  B)       k (E, Lkv, B)       v (Ev, Lkv, B)      all of `dtype`
 *   out (Ev, Lq,  B) of `dtype`, or NULL to compute weights only (then v may be NULL)
 *   weights (Lkv, Lq, H, B) of `weights_dtype`, or NULL to not materialise them
 *   bias   : NULL, or `dtype` array with element strides for the (kv, q, head, batch)
 *            dims of the score tensor; stride 0 = broadcast along that dim
 *            (apply_attn_bias, src/attention.jl:131: logits .+ bias)
 *   mask   : NULL, or uint8 array (0 = drop, non-zero = keep) with strides as for bias
 *            (apply_attn_mask, src/attention.jl:133-138: dropped logits become -Inf)
 *   causal : non-zero = additionally apply make_causal_mask's pattern
 *            keep(kv, q) = kv <= q (src/attention.jl:145) without reading a mask array;
 *            requires Lq == Lkv as a (len, len) mask would.
 *
 * Scores are sum_d k[d]*(q[d]/sqrt(D)) + bias, masked, softmax over kv, as the
 * reference orders them (bias before mask).  A query whose kv positions are all
 * dropped yields NaN weights and NaN output, as the reference's softmax does.
 *
 * weights_dtype must be `dtype` or MI_F32.
 * workspace: device scratch of at least mi_attention_workspace_size() bytes (may be
 * NULL when that size is 0).
 */
typedef struct mi_attn_desc {
    int32_t struct_size; /* = sizeof(mi_attn_desc); guards against ABI drift */
    int32_t dtype;
    int32_t weights_dtype;
    int32_t causal;
    uint32_t flags;
    int32_t reserved;
    int64_t E, Ev, Lq, Lkv, H, B;
    const void *q;
    const void *k;
    const void *v;
    void *out;
    void *weights;
    const void *bias;
    int64_t bias_strides[4];
    const uint8_t *mask;
    int64_t mask_strides[4];
    void *workspace;
    size_t workspace_bytes;
    /* fdrop = dropout(., p) fused into the kernel (src/dropout.jl:38-53 applied at
     * src/attention.jl:126): each weight is zeroed with probability dropout_p, else multiplied by
     * 1/(1 - dropout_p), after the softmax and before the value product; returned weights are
     * post-dropout, as the reference returns them.  The keep decision of weight (kv, q, h, b) is
     * that of mi_dropout() at linear index kv + Lkv*(q + Lq*(h + H*b)) with the same seed, so the
     * fused and the unfused route give the same result.  0 = no dropout. */
    float dropout_p;
    uint32_t reserved2;
    uint64_t dropout_seed;
    /* Optional: softmax row statistics saved for mi_attention_bwd (what an AD rule keeps between the
     * forward and the backward call).  NULL, or a buffer of mi_attention_stats_size() bytes, 16-byte
     * aligned.  Written only by calls that mi_attention_plan() reports as MI_ATTN_KERNEL_FLASH16 or
     * MI_ATTN_KERNEL_FLASH32 (such calls then do not split the key range); other kernels leave it
     * untouched.  Contents are private
     * to the library.  In mi_attn_bwd_desc.fwd: pass the buffer such a forward call of the same
     * arguments filled (the backward call also writes into it), or NULL to have the statistics
     * recomputed. */
    float *stats;
} mi_attn_desc;

/* Validates shapes the way src/attention.jl:55-78 does (MI_ESHAPE on failure) and
 * reports the kernel family and workspace need without touching the device.  A call that is given less
 * workspace than planned fails with MI_EWORKSPACE, with one exception: a 16-bit call without bias and mask
 * whose plan splits the key range (few queries, many keys) is then run unsplit, which needs no workspace
 * and is slower, not wrong. */
int32_t mi_attention_plan(const mi_attn_desc *desc, int32_t *kernel, size_t *workspace_bytes);
int32_t mi_attention_workspace_size(const mi_attn_desc *desc, size_t *bytes);
int32_t mi_attention_fwd(const mi_attn_desc *desc, mi_stream stream);
int32_t mi_attention_stats_size(const mi_attn_desc *desc, size_t *bytes);

/* mi_attention_fwd for callers that cannot allocate device memory: code under stream (graph) capture, serving loops
 * and harnesses that forbid it.  No counterpart in the reference.  Same arguments and results as mi_attention_fwd,
 * except that desc.workspace / workspace_bytes are ignored: the partial results of split-kv calls, the raw scores of
 * single-query calls that return weights and the context lengths of key-padding masks go into an array of
 * MI_ATTN_STATIC_WORKSPACE_BYTES that is part of the library's device image (each GPU the library runs on holds one
 * copy until the process ends).  A call whose mi_attention_workspace_size() exceeds that returns MI_EWORKSPACE.  The
 * call allocates and frees nothing.  All calls on one GPU share the array: calls that may run at the same time on one
 * GPU (different streams) race and must be ordered by the caller.  mi_init(device) looks the array's address up for
 * that device; without it the first call on a device does. */
#define MI_ATTN_STATIC_WORKSPACE_BYTES (32u << 20)
int32_t mi_attention_fwd_static(const mi_attn_desc *desc, mi_stream stream);

/*
 * Gradient of one dot_product_attention call (fdrop = identity or fused dropout).  The reference has no hand-written
 * rule: reverse-mode AD walks src/attention.jl:86-127 backwards through the rrule of batched_mul
 * (src/batched/batchedmul.jl:96-110) and _∇softmax! (src/softmax.jl:107-110); this entry point is
 * that chain fused, never materialising the (Lkv, Lq, H, B) tensors.  Its results are checked the
 * way the reference checks its gradients (test/attention.jl:70-76: against finite differences).
 *
 *   fwd      : the forward call (dtype, sizes, q, k, v, bias, mask, causal, flags, and dropout_p /
 *              dropout_seed when the forward call dropped weights: the keep decisions are redrawn
 *              from the same stream, and the pullback of dropout multiplies by them).  fwd.out holds the
 *              forward RESULT x, or NULL when the caller did not keep it: the MFMA kernels (f16 / bf16: head dim a
 *              multiple of 8 up to 256; f32: of 4 up to 128) need it, and where they can take the call the library
 *              recomputes it with one forward call into the workspace (mi_attention_bwd_plan sizes the workspace for
 *              that, and it must then be 256-byte aligned); otherwise the generic kernels run.  fwd.weights and
 *              fwd.workspace are ignored.
 *   dout     : (Ev, Lq, B) cotangent of x, `dtype`.
 *   dweights : NULL, or (Lkv, Lq, H, B) cotangent of the returned weights, `dtype`.
 *   dq, dk, dv : gradients with the shapes of q, k, v, `dtype`; any may be NULL (not computed).
 *   dbias    : NULL, or FLOAT32 array addressed with fwd.bias_strides; the gradient is ADDED into
 *              it (dims with stride 0 receive the sum over that dim), so the caller zero-fills it.
 *   workspace: at least mi_attention_bwd_plan()'s size, 16-byte aligned (256-byte aligned when q / k and v have
 *              different head dims: the narrower side is zero-padded inside it for the matrix-core kernels).
 * A query whose keys are all dropped has NaN weights in the forward pass and NaN gradients here.
 */
typedef struct mi_attn_bwd_desc {
    int32_t struct_size; /* = sizeof(mi_attn_bwd_desc) */
    int32_t reserved;
    mi_attn_desc fwd;
    const void *dout;
    const void *dweights;
    void *dq;
    void *dk;
    void *dv;
    float *dbias;
    void *workspace;
    size_t workspace_bytes;
} mi_attn_bwd_desc;
int32_t mi_attention_bwd_plan(const mi_attn_bwd_desc *desc, int32_t *kernel, size_t *workspace_bytes);
int32_t mi_attention_bwd(const mi_attn_bwd_desc *desc, mi_stream stream);

/* make_causal_mask (src/attention.jl:149-153): m (len, len) uint8, m[i,j] = (i <= j). */
int32_t mi_make_causal_mask(uint8_t *m, int64_t len, mi_stream stream);

/* ---- dropout --------------------------------------------------------------------- */
/* y[i] = keep_i ? x[i] / (1 - p) : 0 with keep_i ~ Bernoulli(1 - p) from a counter-based generator:
 * dropout(x, p; dims = :) of src/dropout.jl:38-53 with a reproducible stream in place of Julia's RNG.
 * The 64-bit word of counter i >> 2 (splitmix64 of a key derived from the seed) serves elements
 * 4(i >> 2) .. +3 with 16 bits each; keep_i = (that field >= ceil(p * 65536)), so p has a resolution of
 * 2^-16.  y may alias x.  0 <= p <= 1 (p = 1 zeroes everything). */
int32_t mi_dropout(int32_t dtype, const void *x, void *y, int64_t n, float p, uint64_t seed,
                   mi_stream stream);
/* dropout(x, p; dims) of src/dropout.jl:38-53 for dims other than `:`: one keep decision per index along the
 * dimensions in dims_mask (bit d = dimension d + 1), shared along every other dimension, as the reference's
 * random array has extent 1 there (_dropout_shape).  The decision is that of mi_dropout() at the column-major
 * linear index within that smaller array.  sizes: ndim (<= 8) extents of x, a HOST array.  y may alias x. */
int32_t mi_dropout_dims(int32_t dtype, const void *x, void *y, int32_t ndim, const int64_t *sizes,
                        uint32_t dims_mask, float p, uint64_t seed, mi_stream stream);

/* ---- softmax over the first dimension -------------------------------------------- */
/* y[:, c] = softmax(x[:, c]) for a (rows, cols) column-major matrix; y may alias x
 * (softmax!(x), src/softmax.jl:64).  Arithmetic in fp32 (Float64 arrays: in double); +-Inf / NaN rules of
 * src/softmax.jl:69-79 (a +Inf maximum turns the column into an indicator of its
 * +Inf entries, normalised; NaN poisons its column; an all -Inf column is NaN). */
int32_t mi_softmax_dim1(int32_t dtype, const void *x, void *y, int64_t rows, int64_t cols,
                        mi_stream stream);

/* ---- softmax family over any run of adjacent dimensions --------------------------- */
/* The array is viewed as (inner, len, outer): element (i, j, o) at i + inner*(j + len*o), and the
 * reduction runs over j.  `dims = d` of an N-d column-major array gives inner = prod(size[1:d-1]),
 * len = size[d], outer = prod(size[d+1:N]); `dims = :` gives (1, length, 1); a tuple of adjacent
 * dims multiplies their extents into len.  y may alias x.  Arithmetic in fp32 (Float64 arrays: in double). */
enum { MI_SOFTMAX = 0, MI_LOGSOFTMAX = 1 };
/* op = MI_SOFTMAX: softmax(x; dims) (src/softmax.jl:56-79).  op = MI_LOGSOFTMAX: logsoftmax(x; dims)
 * (src/softmax.jl:133-147), including its +Inf rule: a column whose maximum is +Inf gives 0 at the
 * +Inf entries and -Inf elsewhere before the log-sum is subtracted. */
int32_t mi_softmax(int32_t op, int32_t dtype, const void *x, void *y, int64_t inner, int64_t len,
                   int64_t outer, mi_stream stream);
/* logsumexp(x; dims) (src/softmax.jl:200-203): y (inner, outer) = max + log(sum(exp(x - max))). */
int32_t mi_logsumexp(int32_t dtype, const void *x, void *y, int64_t inner, int64_t len,
                     int64_t outer, mi_stream stream);
/* Gradients given the forward RESULT y and the cotangent dy; dx may alias dy.
 * op = MI_SOFTMAX:    dx = dy*y - y*sum(dy*y)   (_∇softmax!, src/softmax.jl:107-110)
 * op = MI_LOGSOFTMAX: dx = dy - sum(dy)*exp(y)  (_∇logsoftmax!, src/softmax.jl:175-177) */
int32_t mi_softmax_bwd(int32_t op, int32_t dtype, const void *dy, const void *y, void *dx,
                       int64_t inner, int64_t len, int64_t outer, mi_stream stream);
/* Pullback of logsumexp (rrule at src/softmax.jl:205-212: dy .* tmp ./ sum(tmp)) given x and the forward
 * RESULT lse: dx[i,j,o] = dy[i,o] * exp(x[i,j,o] - lse[i,o]); dy and lse are (inner, outer), x and dx
 * (inner, len, outer).  A column whose lse is not finite gets NaN, as the reference's formula does. */
int32_t mi_logsumexp_bwd(int32_t dtype, const void *dy, const void *x, const void *lse, void *dx,
                         int64_t inner, int64_t len, int64_t outer, mi_stream stream);

/* The same four operations over ANY set of dimensions of an N-d column-major array (N <= 8), as the reference's
 * `dims` keyword takes (src/softmax.jl:56, 133, 200; Base's reductions accept any dims).  sizes: the N extents, a HOST
 * array; dims_mask: bit d set = dimension d + 1 is reduced over (dimensions past N are ignored, having extent 1).  A
 * set that is a run of adjacent dimensions goes straight to the kernels above; any other set is permuted to the front,
 * reduced and permuted back inside the library (what permutedims does for the reference), through a caller workspace
 * of mi_softmax_dims_workspace() bytes (0 for a run), 16-byte aligned.  y of mi_logsumexp_dims and dy / lse of
 * mi_logsumexp_bwd_dims have the size of x with extent 1 along the reduced dimensions. */
int32_t mi_softmax_dims_workspace(int32_t dtype, int32_t ndim, const int64_t *sizes, uint32_t dims_mask, size_t *bytes);
int32_t mi_softmax_dims(int32_t op, int32_t dtype, const void *x, void *y, int32_t ndim, const int64_t *sizes,
                        uint32_t dims_mask, void *workspace, size_t workspace_bytes, mi_stream stream);
int32_t mi_logsumexp_dims(int32_t dtype, const void *x, void *y, int32_t ndim, const int64_t *sizes, uint32_t dims_mask,
                          void *workspace, size_t workspace_bytes, mi_stream stream);
int32_t mi_softmax_bwd_dims(int32_t op, int32_t dtype, const void *dy, const void *y, void *dx, int32_t ndim,
                            const int64_t *sizes, uint32_t dims_mask, void *workspace, size_t workspace_bytes,
                            mi_stream stream);
int32_t mi_logsumexp_bwd_dims(int32_t dtype, const void *dy, const void *x, const void *lse, void *dx, int32_t ndim,
                              const int64_t *sizes, uint32_t dims_mask, void *workspace, size_t workspace_bytes,
                              mi_stream stream);

/* ---- batched GEMM ---------------------------------------------------------------- */
/* C[:,:,b] = alpha * op(A[:,:,b]) * op(B[:,:,b]) + beta * C[:,:,b],  b in [0, batch).
 * The signature follows the backend hook NNlib._batched_gemm!(transA, transB, alpha,
 * A, B, beta, C) (src/batched/batchedmul.jl:298) flattened to BLAS-style arguments as
 * src/gemm.jl:141-149 passes them: trans flags are the characters 'N' or 'T' ('C' is
 * accepted as 'T': all supported element types are real); op(A) is m x k, op(B) is
 * k x n; lda/ldb/ldc are column strides in elements; strideA/strideB = 0 broadcasts a
 * single slice over the batch (src/gemm.jl:117-118).  beta == 0 overwrites C without
 * reading it.  Accumulation is fp32 for every dtype. */
int32_t mi_batched_gemm(int32_t dtype, char transA, char transB, int64_t m, int64_t n, int64_t k,
                        float alpha, const void *A, int64_t lda, int64_t strideA, const void *B,
                        int64_t ldb, int64_t strideB, float beta, void *C, int64_t ldc,
                        int64_t strideC, int64_t batch, mi_stream stream);

/* ComplexF32 batched_mul: C = alpha * op(A) * op(B) + beta * C per batch slice, complex alpha and beta.
 * Arrays hold interleaved (re, im) Float32 pairs, as Julia stores ComplexF32.  Every operand is given
 * by the ELEMENT strides of its (row, column, batch) indices AFTER op: op(A) is m x k, op(B) is k x n;
 * conj_a / conj_b conjugate the operand.  'N' is (1, ld), 'T' is (ld, 1), 'C' is 'T' with conj: what the
 * reference passes to cgemm (src/gemm.jl:31, flags chosen at src/batched/batchedmul.jl:261-296, 'C' for
 * a BatchedAdjoint{<:Complex}); any other strides are the layouts it gives to batched_mul_generic!
 * (src/batched/batchedmul.jl:306-325).  A batch stride of 0 shares one slice (src/gemm.jl:117-118).
 * beta == 0 overwrites C without reading it. */
int32_t mi_batched_mul_c32(int64_t m, int64_t n, int64_t k, float alpha_re, float alpha_im, const void *A,
                           int64_t a_row_stride, int64_t a_col_stride, int64_t a_batch_stride, int32_t conj_a,
                           const void *B, int64_t b_row_stride, int64_t b_col_stride, int64_t b_batch_stride,
                           int32_t conj_b, float beta_re, float beta_im, void *C, int64_t c_row_stride,
                           int64_t c_col_stride, int64_t c_batch_stride, int64_t batch, mi_stream stream);

/* Float64 batched_mul!: the same call as mi_batched_gemm for the element type the reference hands to dgemm_
 * (src/gemm.jl:27-32, 141-149; ext/NNlibAMDGPUExt/batched_mul.jl:22 lists Float64 among the rocBLAS types), on the
 * fp64 matrix cores.  alpha and beta are doubles; beta == 0 overwrites C without reading it. */
int32_t mi_batched_gemm_f64(char transA, char transB, int64_t m, int64_t n, int64_t k, double alpha, const void *A,
                            int64_t lda, int64_t strideA, const void *B, int64_t ldb, int64_t strideB, double beta,
                            void *C, int64_t ldc, int64_t strideC, int64_t batch, mi_stream stream);

/* batched_mul_generic! (src/batched/batchedmul.jl:306-325): what the reference falls back to when no BLAS routine
 * takes the call: element types that differ between A, B and C (test/batchedmul.jl:41-73: Float64 x Float32,
 * integers, complex x real), Int32 / Int64, ComplexF64, and layouts that are neither 'N' nor 'T'.  Operands are
 * given by their element types and by the ELEMENT strides of the (row, column, batch) indices after op, as in
 * mi_batched_mul_c32; conj_a / conj_b conjugate a complex operand.  dtype_c is the promoted type (Julia's
 * promote_type of the two): A and B are converted to it element by element and the arithmetic is that type's
 * (integer products and sums wrap like Julia's).  dtype_c: MI_F32, MI_F64, MI_I32, MI_I64, MI_C64 or MI_C128.
 * alpha_im / beta_im must be 0 for a real C, alpha and beta integers for an integer C.  A batch stride of 0
 * shares one slice; beta == 0 overwrites C without reading it. */
int32_t mi_batched_mul_generic(int32_t dtype_c, int32_t dtype_a, int32_t dtype_b, int64_t m, int64_t n, int64_t k,
                               double alpha_re, double alpha_im, const void *A, int64_t a_row_stride,
                               int64_t a_col_stride, int64_t a_batch_stride, int32_t conj_a, const void *B,
                               int64_t b_row_stride, int64_t b_col_stride, int64_t b_batch_stride, int32_t conj_b,
                               double beta_re, double beta_im, void *C, int64_t c_row_stride, int64_t c_col_stride,
                               int64_t c_batch_stride, int64_t batch, mi_stream stream);

/* ---- materialising lazy views ------------------------------------------------------ */
/* dst (contiguous column-major d0 x d1 x d2) = src read with element strides (s0, s1, s2): the copy(X)
 * the reference makes of a PermutedDimsArray / transposed view before a BLAS call cannot address it
 * (_copy_if_faster, src/batched/batchedmul.jl:76-83).  elem_bytes is 1, 2, 4, 8 or 16. */
int32_t mi_strided_copy(void *dst, const void *src, int32_t elem_bytes, int64_t d0, int64_t d1, int64_t d2,
                        int64_t s0, int64_t s1, int64_t s2, mi_stream stream);
/* The same for up to 8 dimensions: permutedims of an N-d array (what Base does for the reference when
 * softmax and friends reduce over dimensions that are not neighbours).  sizes / strides: HOST arrays. */
int32_t mi_strided_copy_nd(void *dst, const void *src, int32_t elem_bytes, int32_t ndim, const int64_t *sizes,
                           const int64_t *strides, mi_stream stream);

/* ---- reproducible inputs --------------------------------------------------------- */
/* ptr[i] = dtype(scale * z_i), z_i ~ N(0,1) from a counter-based generator keyed by
 * (seed, stream_id, i); the same call always produces the same bits.  No counterpart
 * in the reference (its tests use Julia's rand/randn). */
int32_t mi_randn_fill(void *ptr, int32_t dtype, int64_t n, uint64_t seed, uint64_t stream_id,
                      float scale, mi_stream stream);
/* mask[i] = (u_i < keep_prob) as uint8, same generator. */
int32_t mi_bernoulli_fill(uint8_t *mask, int64_t n, uint64_t seed, uint64_t stream_id,
                          float keep_prob, mi_stream stream);
/* dst[i] = dtype_dst(src[i]) with round-to-nearest-even: between MI_F32, MI_F16 and MI_BF16; to MI_F64 from those and
 * from MI_I32 / MI_I64; from MI_F64 to the three narrower floating-point types. */
int32_t mi_convert(void *dst, int32_t dtype_dst, const void *src, int32_t dtype_src, int64_t n,
                   mi_stream stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355ATTN_H */
