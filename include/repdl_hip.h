/*
 * repdl_hip.h -- C ABI of the MI355X (gfx950) backend for RepDL's reproducible
 * operators.
 *
 * This is the drop-in boundary: one entry point per function that RepDL's
 * device backend module exports to repdl/ops.py (backend/cuda/bind.cpp:6-18 and
 * the m.def lists cited below), plus the elementwise operators that RepDL
 * composes from PyTorch calls (repdl/ops.py:98-103, 122-123) or keeps internal
 * (backend/cpu/math.h:14-15).  Plain pointers and sizes only; no PyTorch types.
 *
 * Conventions
 *   - All pointers are DEVICE pointers to contiguous row-major float32 data
 *     (int64 for class labels) on the device that is current when the call is
 *     made.  Outputs are caller-allocated.  Inputs are never written
 *     (the optimizer steps update their state tensors in place and say so).
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *     Calls enqueue work and return without synchronising.
 *   - Return value: 0 on success; a positive value is a hipError_t from the
 *     runtime; a negative value is one of the REPDL_E_* codes below.
 *     repdl_hip_error_string() describes either kind.
 *   - Arithmetic contract: binary32, round to nearest even, subnormals kept;
 *     one accumulator per output element starting at +0.0f, updated by single
 *     fused multiply-adds in the loop order of RepDL's CPU backend (whether a
 *     v_fma_f32 or a matrix instruction performs them, see "Matrix path"); results are
 *     bit-identical to that backend for finite data.  (When a NaN is produced
 *     inside a multiply-accumulate chain its sign and payload are unspecified;
 *     the elementwise operators below define NaN bits exactly.)
 */
#ifndef REPDL_HIP_H
#define REPDL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define REPDL_OK 0
#define REPDL_E_ARG (-1)         /* null pointer, negative size, size out of range */
#define REPDL_E_UNSUPPORTED (-2) /* a combination the reference itself does not define */
#define REPDL_E_WORKSPACE (-3)   /* workspace missing or too small */
#define REPDL_E_TOO_LARGE (-4)   /* input beyond the fixed capacity of an entry point that allocates nothing */

const char *repdl_hip_error_string(int code);
int repdl_hip_abi_version(void);

/* Scratch memory.  No counterpart in the reference, whose device functions allocate their output
 * and nothing else (backend/cuda/convolution.cu:153-183, 259-287, 359-383; summation.cu:33-147).
 * Some entry points here need scratch for the duration of a call (they say so below).  Each of them
 * comes in two forms:
 *   repdl_hip_<op>_ws(..., workspace, workspace_bytes, stream) with
 *   repdl_hip_<op>_workspace_bytes(...): the caller provides the memory -- device memory of at least
 *     the size the query returns for the same arguments, any alignment, any contents.  The call
 *     allocates, frees and keeps nothing, so it can be captured into a graph, and the memory can come
 *     from the caller's own allocator (PyTorch's, in this library's bindings).  A workspace that is
 *     missing or too small gives REPDL_E_WORKSPACE (nothing is written outside the workspace; the
 *     output is then undefined).  A query is host arithmetic
 *     only (it runs the entry point's own choice of kernels with the launches switched off; no device
 *     is needed); where it takes operand pointers they are only looked at for their alignment, which
 *     some kernels depend on, and may be NULL for a bound that holds for any pointers.  The bound
 *     covers both settings of the matrix path.
 *   repdl_hip_<op>(..., stream): the library's scratch cache provides it -- a list of buffers per
 *     device and stream: hipMalloc on first use and when a larger size is asked for (a blocking
 *     call), the same buffer for later calls on that stream (whose work is ordered, so the next call
 *     cannot touch it early), held until repdl_hip_scratch_trim() or the end of the process; at most
 *     4 GiB + 25 % per buffer (larger requests go to hipMallocAsync / hipFreeAsync on `stream`).  Two
 *     host threads may use one stream at once (they get different buffers).  While `stream` is being
 *     captured into a graph the cache neither allocates nor frees: the call succeeds only if a buffer
 *     of sufficient size is already there -- from an earlier call with the same arguments on that
 *     stream -- and fails with hipErrorStreamCaptureUnsupported (900) otherwise; a buffer used under
 *     capture is never freed or moved afterwards, since the graph holds its address.  Nothing else
 *     that takes scratch should run on the capture stream while such a graph replays.
 *   repdl_hip_scratch_trim: frees every cache buffer that no call and no captured graph is using
 *     (waits for the device).  repdl_hip_scratch_bytes: bytes the cache holds now. */
int repdl_hip_scratch_trim(void);
size_t repdl_hip_scratch_bytes(void);

/* Which kernels ran.  No counterpart in the reference.  The operators choose among several kernel
 * families by shape, alignment and the matrix path; every family that launches sets its bit in a
 * process-wide mask.  repdl_hip_routes_taken returns the mask (and clears it when `reset` is not 0);
 * repdl_hip_route_name names bit `route` (NULL past the last).  For tests that must reach every family. */
uint64_t repdl_hip_routes_taken(int reset);
const char *repdl_hip_route_name(int route);

/* Matrix path.  No counterpart in the reference: its CUDA kernels use one FMA per
 * term (backend/cuda/matrix_multiplication.cu:18-60, convolution.cu:62-151).
 * mm and the three convolutions have two implementations of the same chains: one on
 * the binary32 matrix instructions of gfx950 (v_mfma_f32_32x32x2_f32 /
 * v_mfma_f32_16x16x4_f32) and one on v_fma_f32.  The matrix instructions are used
 * only on a device where a check run on that device has found them bit-identical to
 * chains of single-rounding FMAs, k ascending; no setting overrides a failed check.
 *   repdl_hip_init: runs that check (about a million comparisons) for the current
 *     device, once, and waits for it.  It works on a stream of its own, created
 *     non-blocking at the default priority, with memory from the stream-ordered
 *     allocator: it neither waits for nor delays the null stream or any stream of the
 *     caller.  Returns 0 when the check could run, whatever its verdict.  Call it at
 *     start-up, outside any stream capture.
 *   First-call behaviour without repdl_hip_init: the first GEMM-shaped call on a device
 *     runs the same check in the same way (the calling thread waits about 0.2 ms; the
 *     caller's stream is not touched).  If the check cannot run at that moment -- the
 *     thread is capturing a graph, say -- that call takes the v_fma_f32 kernels (same
 *     bits, slower) and the check is tried again at the next call.
 *   repdl_hip_mfma_selftest: runs waves*trials further comparisons of each
 *     instruction (operand classes cycle with the trial number) and writes the
 *     number of differing results to mismatches[0] (32x32x2) and mismatches[1]
 *     (16x16x4), HOST memory.  Synchronous, on a stream of its own.
 *   repdl_hip_set_matrix_path: 0 = always the v_fma_f32 kernels; -1 (default) and 1 =
 *     the matrix kernels wherever the check has passed.  Mode 1 also runs the check for
 *     the current device and returns REPDL_E_UNSUPPORTED, changing nothing, if it did
 *     not pass there.  Process-wide.
 *   repdl_hip_matrix_path: 1 if GEMM-shaped calls on the current device now take the
 *     matrix kernels, else 0 (runs the check if it has not run yet). */
int repdl_hip_init(void);
int repdl_hip_mfma_selftest(int64_t waves, int64_t trials, uint64_t seed, uint64_t *mismatches);
int repdl_hip_set_matrix_path(int mode);
int repdl_hip_matrix_path(void);

/* mm -- backend/cuda/matrix_multiplication.cu:234-260 (bound at :267);
 * semantics backend/cpu/matrix_multiplication.cpp:12-36.
 * C[M,N] = op(A) op(B); A is [M,K] (or [K,M] when transA), B is [K,N] (or [N,K]
 * when transB); C(i,j) = fma(a_{K-1}, b_{K-1}, ... fma(a_0, b_0, +0)). */
int repdl_hip_mm(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K,
                 int transA, int transB, void *stream);

/* mm with the bias of a linear layer -- repdl/nn/linear.py:21-22, 37: `mm(x, W, transB)`
 * followed by `+= bias`.  The reference makes the addition a second pass over the
 * output; here it is the last operation on each output's register: C(i,j) =
 * RN(chain(i,j) + bias[j]), one IEEE addition after the complete chain, the same bits.
 * bias is [N] (NULL: no bias, exactly repdl_hip_mm). */
int repdl_hip_mm_bias(const float *A, const float *B, const float *bias, float *C, int64_t M, int64_t N,
                      int64_t K, int transA, int transB, void *stream);

/* conv2d -- backend/cuda/convolution.cu:153-183 (bound at :385); semantics
 * backend/cpu/convolution.cpp:12-52.  NCHW; kernel is [OC, IC/groups, KH, KW];
 * output is [N, OC, OH, OW] with OH = (H + 2 pH - KH) / sH + 1.
 * Scratch (see "Scratch memory" above): 17 KiB whenever the geometry
 * makes the reference skip taps (padding, strides of grad-input, kernels wider than one
 * tap in grad-input); on the matrix path also a copy of the kernel in the order the matrix
 * instruction reads it (3x3 kernels at stride 1 in grad-input, and 1x1 kernels with chains of
 * at most 64 terms; 3x3 forward and the other 1x1 kernels at stride 1 take nothing else), or for the
 * remaining shapes a zero-padded copy of the gathered operand
 * of conv2d / conv2d_grad_input with two small offset tables (or, for images of at most
 * 100 pixels with many channels, its im2col: output elements x IC*KH*KW floats), and for conv2d_grad_kernel
 * copies of grad_output / input with rows rounded up to a multiple of 4 floats when
 * their widths are not one -- at most the size of the operands with their borders -- or,
 * for layers with many short chains (OC*IC*KH*KW large, N*OH*OW small), grad_output with
 * the batch outermost and the im2col of the input (N*OH*OW * IC*KH*KW floats, below 2^31). */
int repdl_hip_conv2d(const float *input, const float *kernel, float *output, int64_t N, int64_t IC,
                     int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t sH,
                     int64_t sW, int64_t pH, int64_t pW, int64_t groups, void *stream);

/* conv2d with the layer's bias -- repdl/nn/conv.py:27-28: conv2d followed by
 * `+= bias` broadcast over [N, OC, OH, OW].  output(n,oc,oh,ow) = RN(chain + bias[oc]):
 * one IEEE addition after the complete chain, made in the kernel's epilogue instead of
 * a second pass over the output.  bias is [OC] (NULL: none, exactly repdl_hip_conv2d). */
int repdl_hip_conv2d_bias(const float *input, const float *kernel, const float *bias, float *output, int64_t N,
                          int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t sH,
                          int64_t sW, int64_t pH, int64_t pW, int64_t groups, void *stream);

/* conv2d / conv2d_bias with the caller's workspace (bias may be NULL). */
size_t repdl_hip_conv2d_workspace_bytes(const float *input, const float *kernel, int64_t N, int64_t IC, int64_t H,
                                        int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t sH, int64_t sW,
                                        int64_t pH, int64_t pW, int64_t groups);
int repdl_hip_conv2d_ws(const float *input, const float *kernel, const float *bias, float *output, int64_t N,
                        int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t sH,
                        int64_t sW, int64_t pH, int64_t pW, int64_t groups, void *workspace,
                        size_t workspace_bytes, void *stream);

/* conv2d_grad_input -- backend/cuda/convolution.cu:259-287 (bound at :386);
 * semantics backend/cpu/convolution.cpp:54-90.  groups == 1.
 * grad_output is [N, OC, OH, OW], kernel [OC, IC, KH, KW], grad_input [N, IC, H, W]. */
int repdl_hip_conv2d_grad_input(const float *grad_output, const float *kernel, float *grad_input,
                                int64_t N, int64_t OC, int64_t OH, int64_t OW, int64_t IC,
                                int64_t KH, int64_t KW, int64_t H, int64_t W, int64_t sH,
                                int64_t sW, int64_t pH, int64_t pW, void *stream);

size_t repdl_hip_conv2d_grad_input_workspace_bytes(const float *grad_output, const float *kernel, int64_t N,
                                                   int64_t OC, int64_t OH, int64_t OW, int64_t IC, int64_t KH,
                                                   int64_t KW, int64_t H, int64_t W, int64_t sH, int64_t sW,
                                                   int64_t pH, int64_t pW);
int repdl_hip_conv2d_grad_input_ws(const float *grad_output, const float *kernel, float *grad_input, int64_t N,
                                   int64_t OC, int64_t OH, int64_t OW, int64_t IC, int64_t KH, int64_t KW,
                                   int64_t H, int64_t W, int64_t sH, int64_t sW, int64_t pH, int64_t pW,
                                   void *workspace, size_t workspace_bytes, void *stream);

/* conv2d_grad_kernel -- backend/cuda/convolution.cu:359-383 (bound at :387);
 * semantics backend/cpu/convolution.cpp:92-128.  groups == 1.
 * grad_kernel is [OC, IC, KH, KW]. */
int repdl_hip_conv2d_grad_kernel(const float *grad_output, const float *input, float *grad_kernel,
                                 int64_t N, int64_t IC, int64_t H, int64_t W, int64_t OC,
                                 int64_t OH, int64_t OW, int64_t KH, int64_t KW, int64_t sH,
                                 int64_t sW, int64_t pH, int64_t pW, void *stream);
size_t repdl_hip_conv2d_grad_kernel_workspace_bytes(const float *grad_output, const float *input, int64_t N,
                                                    int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t OH,
                                                    int64_t OW, int64_t KH, int64_t KW, int64_t sH, int64_t sW,
                                                    int64_t pH, int64_t pW);
int repdl_hip_conv2d_grad_kernel_ws(const float *grad_output, const float *input, float *grad_kernel, int64_t N,
                                    int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t OH, int64_t OW,
                                    int64_t KH, int64_t KW, int64_t sH, int64_t sW, int64_t pH, int64_t pW,
                                    void *workspace, size_t workspace_bytes, void *stream);

/* sums -- backend/cuda/summation.cu:33-147 (bound at :149-155); semantics
 * backend/cpu/summation.cpp:12-78: strict left-to-right binary32 chains from
 * +0.0f, then one multiply by (float)(average ? 1.0/count : 1.0).
 *   sum1d:        out[0]    = sum_i in[i]                       (count n)
 *   sum2d_dim0:   out[j]    = sum_i in[i][j],  in [M,N]         (count M)
 *   sum2d_dim1:   out[i]    = sum_j in[i][j],  in [M,N]         (count N)
 *   sum4d_dim023: out[c]    = sum_{n,h,w} in[n][c][h][w]        (count N*H*W) */
int repdl_hip_sum1d(const float *in, float *out, int64_t n, int average, void *stream);
/* sum1d with caller-provided scratch memory (same result).  Long inputs are evaluated in
 * parallel -- exactly: the result is the sequential chain's, bit for bit -- which needs
 * repdl_hip_sum1d_workspace_bytes(n) bytes of 16-byte aligned device memory (about 5n/8
 * bytes; 0 for short inputs).  The memory may hold anything on entry.  repdl_hip_sum1d itself
 * takes it from the library's scratch cache (see "Scratch memory" above). */
size_t repdl_hip_sum1d_workspace_bytes(int64_t n);
int repdl_hip_sum1d_ws(const float *in, float *out, int64_t n, int average, void *workspace,
                       size_t workspace_bytes, void *stream);
/* sum1d for callers that cannot allocate (code under graph capture, serving loops, harnesses
 * that forbid hipMalloc).  No counterpart in the reference.  Same result as repdl_hip_sum1d, bit
 * for bit, but the scratch memory of the parallel evaluation is a fixed 8 MiB array inside the
 * library (one per device, held until the process ends) instead of an allocation: the call
 * makes no hipMalloc / hipFree / stream-ordered allocation.  n may not exceed
 * repdl_hip_sum1d_static_max_n() (about 13 million elements; REPDL_E_TOO_LARGE beyond).  All
 * calls on one device share that array: calls that overlap in time on one device (two
 * streams, two threads) race and must be serialised by the caller. */
int64_t repdl_hip_sum1d_static_max_n(void);
int repdl_hip_sum1d_static(const float *in, float *out, int64_t n, int average, void *stream);
int repdl_hip_sum2d_dim0(const float *in, float *out, int64_t M, int64_t N, int average,
                         void *stream);
/* sum2d_dim1 and sum4d_dim023 with few long chains (at most 512 chains of at least 49152
 * elements, or at most 64 of at least 24576; for sum4d_dim023 also H*W a multiple of 16) take the same parallel evaluation,
 * all chains at once, with about half the input's size in bytes from the scratch cache;
 * otherwise they allocate nothing. */
int repdl_hip_sum2d_dim1(const float *in, float *out, int64_t M, int64_t N, int average,
                         void *stream);
int repdl_hip_sum4d_dim023(const float *in, float *out, int64_t N, int64_t C, int64_t H, int64_t W,
                           int average, void *stream);
size_t repdl_hip_sum2d_dim1_workspace_bytes(int64_t M, int64_t N);
int repdl_hip_sum2d_dim1_ws(const float *in, float *out, int64_t M, int64_t N, int average, void *workspace,
                            size_t workspace_bytes, void *stream);
size_t repdl_hip_sum4d_dim023_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W);
int repdl_hip_sum4d_dim023_ws(const float *in, float *out, int64_t N, int64_t C, int64_t H, int64_t W, int average,
                              void *workspace, size_t workspace_bytes, void *stream);

/* exp, log -- backend/cuda/math.cu:15-18, 42-45 (drivers :30-39, :56-65; declared
 * backend/cuda/math.h, not bound to Python by the reference); semantics
 * backend/cpu/math.cpp:14-17, 32-35: (float)exp((double)x), (float)log((double)x)
 * with glibc's binary64 routines.  Any number of elements. */
int repdl_hip_exp(const float *in, float *out, int64_t n, void *stream);
int repdl_hip_log(const float *in, float *out, int64_t n, void *stream);

/* sqrt -- repdl/ops.py:122-123: float32(sqrt(float64(x))) == IEEE binary32 sqrt.
 * Negative arguments give the quiet NaN 0x7FC00000 (PyTorch's CPU convention);
 * NaN arguments keep sign and payload, quieted; sqrt(-0) = -0. */
int repdl_hip_sqrt(const float *in, float *out, int64_t n, void *stream);

/* div -- repdl/ops.py:98-103: IEEE binary32 quotient, elementwise, either by a
 * second tensor of the same length or by one binary32 scalar (a true division,
 * never a multiplication by the reciprocal).  NaN dividend wins over NaN
 * divisor; 0/0 and inf/inf give 0xFFC00000. */
int repdl_hip_div(const float *a, const float *b, float *out, int64_t n, void *stream);
int repdl_hip_div_scalar(const float *a, float b, float *out, int64_t n, void *stream);

/* softmax -- backend/cuda/softmax.cpp:15-21 (bound at :28); semantics
 * backend/cpu/softmax.cpp:15-21.  in/out are [M,N]. */
int repdl_hip_softmax(const float *in, float *out, int64_t M, int64_t N, void *stream);

/* cross_entropy -- backend/cuda/cross_entropy.cpp:15-24 (bound at :31); semantics
 * backend/cpu/cross_entropy.cpp:15-24.  in is [M,N], target is [M] int64 class
 * indices in [0,N), out is one float.  workspace: M floats of device memory (the row
 * losses; their mean is repdl_hip_sum1d with average = 1, which from 12288 rows on takes
 * its own scratch from the scratch cache as described there). */
int repdl_hip_cross_entropy(const float *in, const int64_t *target, float *out, int64_t M,
                            int64_t N, float *workspace, void *stream);
/* cross_entropy with one caller's workspace for both the row losses and the scratch of their mean. */
size_t repdl_hip_cross_entropy_workspace_bytes(int64_t M, int64_t N);
int repdl_hip_cross_entropy_ws(const float *in, const int64_t *target, float *out, int64_t M, int64_t N,
                               void *workspace, size_t workspace_bytes, void *stream);

/* Batch normalisation, the elementwise passes -- the reference has no backend function for
 * these: repdl/nn/batchnorm.py:12-66 composes them from PyTorch tensor operations, one
 * rounding each.  Each entry point evaluates one of those compositions per element with the
 * same roundings in the same order, in one pass over memory.  Tensors are
 * [outer][channels][inner] (NCHW: outer = N, inner = H*W; [B,F]: outer = B, inner = 1); mean,
 * std, weight, bias and coef are [channels]; `/` is the IEEE quotient.
 *   bn_apply         y   = RN(RN(RN(RN(x - mean[c]) / std[c]) * weight[c]) + bias[c])   (batchnorm.py:25-32)
 *   bn_gvar_term     out = RN(RN(grad_y * RN(mean[c] - x)) * coef[c])                   (:56-58, before the sum)
 *   bn_gweight_term  out = RN(RN(RN(x - mean[c]) / std[c]) * grad_y)                    (:60-61, before the sum) */
int repdl_hip_bn_apply(const float *x, const float *mean, const float *std, const float *weight, const float *bias,
                       float *y, int64_t outer, int64_t channels, int64_t inner, void *stream);
int repdl_hip_bn_gvar_term(const float *grad_y, const float *x, const float *mean, const float *coef, float *out,
                           int64_t outer, int64_t channels, int64_t inner, void *stream);
int repdl_hip_bn_gweight_term(const float *x, const float *mean, const float *std, const float *grad_y, float *out,
                              int64_t outer, int64_t channels, int64_t inner, void *stream);

/* Optimizer steps -- the reference has no backend function for these: repdl/optim.py:56-83
 * writes Adam as a sequence of PyTorch tensor operations around ops.sqrt and a true
 * division (a dozen launches and temporaries per parameter).  These entry points evaluate
 * that same sequence per element, every rounding in the same place, in one pass over all
 * the tensors of a parameter group.  param, exp_avg, exp_avg_sq and max_exp_avg_sq are
 * updated in place; grad is read only; tensors must not overlap.  The scalars are the
 * binary32 roundings of the values the Python code computes in binary64 (PyTorch rounds a
 * Python number that meets a float32 tensor once, to binary32).  A NaN operand gives a NaN
 * result whose sign and payload are unspecified.
 *
 * Adam, per element (optim.py:64-83), with b1 = beta1, c1 = one_minus_beta1 = float(1 - beta1),
 * likewise b2 and c2:
 *   g' = weight_decay != 0 ? fma(weight_decay, p, g) : g
 *   m  = fma(c1, g', RN(m * b1))
 *   v  = RN(RN(v * b2) + RN(RN(g' * g') * c2))
 *   s  = max_exp_avg_sq ? (vmax = max(vmax, v), NaN if either is) : v
 *   d  = RN(RN(RN(sqrt(s)) / sqrt_bias_correction2) + eps), a true division
 *   p  = RN(p + RN(RN(m / d) * step_scale))
 * where sqrt_bias_correction2 = float(sqrt(1 - beta2^t)) and step_scale =
 * float(-(lr / (1 - beta1^t))) for the tensor's step count t (optim.py:60-61, 82).
 * max_exp_avg_sq == NULL means amsgrad is off for that tensor. */
typedef struct
{
    float *param;
    const float *grad;
    float *exp_avg;
    float *exp_avg_sq;
    float *max_exp_avg_sq;
    int64_t n;
    float sqrt_bias_correction2;
    float step_scale;
} repdl_adam_tensor;

/* tensors: HOST array of `count` descriptors (device pointers inside); read before the
 * call returns.  Empty tensors (n == 0) are skipped. */
int repdl_hip_adam_step(const repdl_adam_tensor *tensors, int count, float beta1, float one_minus_beta1,
                        float beta2, float one_minus_beta2, float eps, float weight_decay, void *stream);

/* Plain gradient descent with both roundings kept: p = RN(p - RN(g * lr)).  (PyTorch's own
 * update, param.add_(grad, alpha=-lr), rounds once on devices that fuse it and twice on
 * those that do not.) */
typedef struct
{
    float *param;
    const float *grad;
    int64_t n;
} repdl_sgd_tensor;

int repdl_hip_sgd_step(const repdl_sgd_tensor *tensors, int count, float lr, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* REPDL_HIP_H */
