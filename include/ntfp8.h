/* ntfp8 — C ABI of the MI355X (gfx950) FP8 linear hot path.
 *
 * This is the native plug-in point that stands where nanotron's `nanotron.fp8` package
 * calls NVIDIA Transformer Engine's pybind module (`transformer_engine_extensions as tex`).
 * Each entry point names the reference call it replaces (paths relative to the reference
 * checkout).
 *
 * Conventions
 *   - every data pointer is a DEVICE pointer owned by the caller (a torch tensor kept alive
 *     on the Python side); the library never allocates, frees or synchronises;
 *   - amax / scale / history values live in device memory: no host round trip;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *   - return value: 0 on success, a negative NTFP8_ERR_* code otherwise; argument errors are
 *     detected on the host before anything is launched, so a bad call never faults the GPU;
 *   - 2-D operands are row-major and contiguous; fp8 bytes are OCP e4m3fn / e5m2;
 *   - `workspace` is NTFP8_WORKSPACE_BYTES of device memory that must be zero before its first
 *     use; kernels leave it zero again, so it can be reused by stream-ordered calls.  Calls
 *     that may overlap (different streams) need distinct workspaces;
 *   - every scale argument is the SCALE (x_fp8 = x * scale) unless an entry point or descriptor field says
 *     that it takes the inverse scale, the form Transformer Engine's functions are handed by the reference
 *     (`meta.inverse_scale`, src/nanotron/fp8/meta.py:36-37).  For the power-of-two scales this path produces
 *     (src/nanotron/fp8/tensor.py:97-103) both forms give the same bits: 1 / (1 / s) == s exactly.
 */
#ifndef NTFP8_H
#define NTFP8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NTFP8_VERSION 3
#define NTFP8_WORKSPACE_BYTES 2048

/* FP8 storage formats.  Reference: DTypes.FP8E4M3 / DTypes.FP8E5M2 (src/nanotron/fp8/dtypes.py:4-7),
 * mapped to tex.DType.kFloat8E4M3 / kFloat8E5M2 at src/nanotron/fp8/tensor.py:39-55. */
enum { NTFP8_E4M3 = 0, NTFP8_E5M2 = 1 };

/* High-precision element types (tex.DType.kFloat32 / kFloat16 / kBFloat16, tensor.py:43-47). */
enum { NTFP8_F32 = 0, NTFP8_F16 = 1, NTFP8_BF16 = 2 };

enum {
    NTFP8_OK = 0,
    NTFP8_ERR_NULL = -1,        /* a required pointer is NULL */
    NTFP8_ERR_ENUM = -2,        /* unknown format / dtype value */
    NTFP8_ERR_SIZE = -3,        /* negative, zero or overflowing size */
    NTFP8_ERR_ALIGN = -4,       /* pointer not aligned to its element type */
    NTFP8_ERR_UNSUPPORTED = -5, /* valid request the library does not implement */
    NTFP8_ERR_LAUNCH = -6,      /* HIP reported an error at launch */
    NTFP8_ERR_ALIAS = -7        /* output overlaps an input */
};

int ntfp8_version(void);
const char* ntfp8_strerror(int code);

/* amax = max|x| (NaN-propagating) and the power-of-two scale derived from it.
 * Replaces `tensor.abs().max()` + `update_scaling_factor(amax, 1.0, dtype)`
 * (src/nanotron/fp8/tensor.py:25-26, 94-103), one launch instead of ~10.
 * old_scale may be NULL (= INITIAL_SCALING_FACTOR 1.0, src/nanotron/fp8/constants.py:8). */
int ntfp8_amax_scale(const void* x, int x_dtype, int64_t n, int fmt, int margin,
                     const float* old_scale, float* amax_out, float* scale_out,
                     void* workspace, void* stream);

/* Element-wise update_scaling_factor on device arrays of n amax values
 * (src/nanotron/fp8/tensor.py:77-105).  old_scale / out have n elements. */
int ntfp8_update_scaling_factor(const float* amax, const float* old_scale, int fmt, int margin,
                                float* out, int64_t n, void* stream);

/* The same function for one host value (no GPU involved): what the reference evaluates on CPU
 * tensors in FP8Linear.__init__ (src/nanotron/fp8/linear.py:33-42). */
float ntfp8_update_scaling_factor_host(float amax, float old_scale, int fmt, int margin);

/* out = saturating_rne_fp8(fp32(x) * *scale).  Replaces tex.cast_to_fp8
 * (src/nanotron/fp8/tensor.py:65).  x is [rows, cols]; out_t, when not NULL, also receives the
 * transposed bytes [cols, rows] (what tex.fp8_transpose, src/nanotron/fp8/kernel.py:43-44, would
 * produce from `out`), written in the same pass. */
int ntfp8_cast_to_fp8(const void* x, int x_dtype, int64_t rows, int64_t cols, const float* scale,
                      int fmt, void* out, void* out_t, void* stream);

/* tex.cast_to_fp8(input, scale, amax, scale_inv, otype) with all of its effects (src/nanotron/fp8/tensor.py:65; the
 * arithmetic lives in Transformer Engine, which the reference does not vendor: the effects below are its published
 * behaviour): out = saturating_rne_fp8(fp32(x) * *scale); *amax_inout = max(*amax_inout, max|x|) (a NaN on either
 * side is kept; Transformer Engine's own maximum drops NaN inputs, an un-pinned corner); *scale_inv_out = 1 / *scale.
 * amax_inout and scale_inv_out may each be NULL; with both NULL this is ntfp8_cast_to_fp8 without a transposed
 * copy and needs no workspace. */
int ntfp8_te_cast_to_fp8(const void* x, int x_dtype, int64_t n, const float* scale, float* amax_inout,
                         float* scale_inv_out, int fmt, void* out, void* workspace, void* stream);

/* FP8Tensor.__new__ in one call (src/nanotron/fp8/tensor.py:25-28): current scaling.
 * amax pass, scale from amax starting at 1.0, cast pass.  If amax_history is not NULL the
 * delayed-scaling state is updated as well (history rolled, *scale_state = next scale), which
 * is what the first use of a delayed-scaling role does. */
int ntfp8_quantize_current(const void* x, int x_dtype, int64_t rows, int64_t cols, int fmt, int margin,
                           float* amax_out, float* scale_used_out, void* out, void* out_t,
                           float* amax_history, int history_len, float* scale_state,
                           void* workspace, void* stream);

/* The quantisation of a delayed-scaling role that may or may not hold a scale yet, decided on the device (the host
 * reads nothing back, so the call can be captured in a HIP graph from a role's very first step): *initialised is a
 * flag in device memory, 0.0 until a finite positive amax has been recorded.
 *   *initialised == 0:  the result of ntfp8_quantize_current with the history arguments (the reference's scaling,
 *                       src/nanotron/fp8/tensor.py:25-28: the scale comes from this tensor's own amax);
 *   *initialised != 0:  the result of ntfp8_quantize_delayed, bit for bit (cast with *scale_state, history rolled,
 *                       next scale stored), from two launches instead of one (amax pass, then cast: 5 bytes per 16-bit
 *                       element instead of 3);
 * and *initialised becomes 1.0 if this tensor's amax is finite and positive.  A caller that knows the role holds a scale
 * calls ntfp8_quantize_delayed. */
int ntfp8_quantize_first_use(const void* x, int x_dtype, int64_t rows, int64_t cols, int fmt, int margin, float* scale_state,
                             float* amax_history, int history_len, float* initialised, float* amax_out,
                             float* scale_used_out, void* out, void* out_t, void* workspace, void* stream);

/* One delayed-scaling step in a single pass over x (no counterpart in the reference, which
 * has no amax history; semantics fixed by the benchmark configs: history 16, margin 0):
 *   a = amax(x); q = cast(x, *scale_state); roll amax_history, hist[0] = a;
 *   *scale_used_out = old *scale_state; *scale_state = update_scaling_factor(max(hist), old). */
int ntfp8_quantize_delayed(const void* x, int x_dtype, int64_t rows, int64_t cols, int fmt, int margin,
                           float* scale_state, float* amax_history, int history_len,
                           float* amax_out, float* scale_used_out, void* out, void* out_t,
                           void* workspace, void* stream);

/* One delayed-scaling step of TWO roles that quantise the same tensor, e4m3 and e5m2, in a single pass over x
 * (4 bytes of traffic per bf16 element instead of 2 x 3; no counterpart in the reference).  Results equal, bit for
 * bit, ntfp8_quantize_delayed called once per format: the amax is shared, each role keeps its own scale and
 * history.  scale_used_out_* may be NULL. */
int ntfp8_quantize_delayed_dual(const void* x, int x_dtype, int64_t n, int margin,
                                float* scale_state_e4m3, float* amax_history_e4m3,
                                float* scale_state_e5m2, float* amax_history_e5m2, int history_len,
                                float* amax_out, float* scale_used_out_e4m3, float* scale_used_out_e5m2,
                                void* out_e4m3, void* out_e5m2, void* workspace, void* stream);

/* ntfp8_quantize_delayed for several tensors in one call (each with a zeroed workspace of its own): same results
 * as the separate calls.  Tensors without a transposed copy that share source type and format share a launch, in
 * which the reduction and bookkeeping of one tensor run under the streaming of the next instead of in front of a
 * kernel boundary: the call for the fp8 copies of all weights after an optimizer step (the reference has no
 * counterpart: it quantises a weight once, src/nanotron/fp8/parameter.py:27). */
#define NTFP8_MAX_BATCH 64   /* problems / tensors per batched call */
typedef struct ntfp8_quant_desc {
    const void* x;
    int x_dtype, fmt, margin, history_len;
    int64_t rows, cols;
    float* scale_state;
    float* amax_history;
    float* amax_out;
    float* scale_used_out;   /* may be NULL */
    void* out;
    void* out_t;             /* may be NULL */
    void* workspace;
} ntfp8_quant_desc;
int ntfp8_quantize_delayed_batch(const ntfp8_quant_desc* tensors, int count, void* stream);

/* ntfp8_quantize_delayed_batch for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid it).  It has no counterpart in the reference.  The reduction workspaces come
 * from an array inside the library's device image (NTFP8_STATIC_MAX_TENSORS x NTFP8_WORKSPACE_BYTES = 32 KiB, held
 * by every GPU the library runs on until the process ends); the `workspace` members of the descriptors are ignored.
 * count above NTFP8_STATIC_MAX_TENSORS returns NTFP8_ERR_SIZE.  Nothing is allocated or freed, here or in any
 * routine it calls.  All calls on one GPU share that GPU's array: calls that may overlap in time (different
 * streams, different threads) race; order them, or use ntfp8_quantize_delayed_batch with workspaces of their own.
 * The per-device address of the array is resolved at the first call on a device (a host-side look-up, nothing is
 * launched: the array starts zeroed with the device image and every kernel leaves its workspace zero);
 * ntfp8_static_init does that ahead of time for the current device, e.g. before a graph capture begins (`stream` is
 * not used). */
#define NTFP8_STATIC_MAX_TENSORS 16
int ntfp8_static_init(void* stream);
int ntfp8_quantize_delayed_batch_static(const ntfp8_quant_desc* tensors, int count, void* stream);

/* out = out_dtype(fp32(fp8) * (1 / *scale)).  Replaces tex.cast_from_fp8
 * (src/nanotron/fp8/tensor.py:74) with meta.inverse_scale (src/nanotron/fp8/meta.py:36-37). */
int ntfp8_cast_from_fp8(const void* in, int fmt, const float* scale, int64_t n, void* out, int out_dtype,
                        void* stream);
/* The same with the inverse scale as argument, which is what tex.cast_from_fp8 receives at
 * src/nanotron/fp8/tensor.py:74: out = out_dtype(fp32(fp8) * *scale_inv). */
int ntfp8_cast_from_fp8_scale_inv(const void* in, int fmt, const float* scale_inv, int64_t n, void* out, int out_dtype,
                                  void* stream);

/* Byte transpose [rows, cols] -> [cols, rows].  Replaces tex.fp8_transpose
 * (src/nanotron/fp8/kernel.py:43-44). */
int ntfp8_transpose(const void* in, int64_t rows, int64_t cols, void* out, void* stream);

/* D[M,N] (+)= (A[M,K] . B[N,K]^T) * (1 / *scale_a) * (1 / *scale_b), fp32 accumulation.
 * Replaces tex.te_gemm in the only form the reference issues it (transa=True, transb=False:
 * both operands contiguous along the reduction dimension; src/nanotron/fp8/kernel.py:46-68).
 * d_dtype: NTFP8_F32 (reference default, kernel.py:24,28), NTFP8_BF16 or NTFP8_F16.
 * accumulate != 0 adds into D (fp32 only) before the single rounding: the fp32 master-gradient
 * accumulation of src/nanotron/optim/gradient_accumulator.py:222 folded into the epilogue. */
int ntfp8_gemm(const void* A, int fmt_a, const float* scale_a,
               const void* B, int fmt_b, const float* scale_b,
               void* D, int d_dtype, int64_t M, int64_t N, int64_t K, int accumulate, void* stream);

/* Several independent GEMMs in one call: no output may overlap an operand or output of another
 * problem.  Problems with the same operand formats share launches, which removes the partial last
 * round of tiles and the kernel boundary between them.  The reference issues the dgrad and wgrad of
 * a layer as two tex.te_gemm calls on the same stream (src/nanotron/fp8/linear.py:104-109); they
 * do not depend on each other.  Each problem means what it means for ntfp8_gemm. */
typedef struct ntfp8_gemm_desc {
    const void* A;
    const float* scale_a;
    const void* B;
    const float* scale_b;
    void* D;
    int64_t M, N, K;
    int fmt_a, fmt_b, d_dtype, accumulate;
    /* fp8 outputs only (d_dtype NTFP8_OUT_E4M3 / NTFP8_OUT_E5M2, below); ignored otherwise */
    const float* scale_d;   /* device scalar: the result is multiplied by it before the cast */
    void* D_t;              /* NULL, or [N, M] bytes: the transposed copy of D */
    void* amax_workspace;   /* NULL, or NTFP8_WORKSPACE_BYTES, all zero: collects max|result| */
    /* != 0: B points to the [K, N] row-major bytes of B's transpose, i.e. to a tensor whose row index is the
     * reduction index.  That is what the backward GEMMs of a linear layer have at hand (dgrad: W[N_out, K_in]
     * reduces over N_out; wgrad: X[tokens, K_in] reduces over tokens; src/nanotron/fp8/linear.py:104-109), and
     * where the reference calls tex.fp8_transpose first (src/nanotron/fp8/kernel.py:43) this library reads the
     * tensor as it is.  Served for N a multiple of 16, M and N above 128, K at least 256, operands below 2 GiB
     * (fp8 outputs in addition: M a multiple of 4, M N below 2^32, D_t aligned to 16 bytes); anything else returns
     * NTFP8_ERR_UNSUPPORTED (transpose B and pass 0). */
    int b_transposed;
    /* NULL, or bias[N] of type bias_dtype (NTFP8_F32 / NTFP8_F16 / NTFP8_BF16), added to the descaled fp32 result
     * before the single rounding to d_dtype: D = round(fp32(acc * descale) + bias[n]).  This is the `bias` /
     * `bias_type` pair of tex.te_gemm, which the reference leaves empty (src/nanotron/fp8/kernel.py:29-32) and adds
     * outside instead (src/nanotron/fp8/linear.py:62,65).  For an fp32 output the result equals the separate
     * addition bit for bit; for 16-bit and fp8 outputs it saves the intermediate rounding.  Not together with
     * b_transposed (NTFP8_ERR_UNSUPPORTED): the backward GEMMs that use it have no bias. */
    const void* bias;
    int bias_dtype;
    /* != 0: scale_a and scale_b point to INVERSE scales, the form tex.te_gemm is handed
     * (meta.inverse_scale, src/nanotron/fp8/kernel.py:48,52): the sum is multiplied by them, not divided. */
    int scales_are_inverse;
    /* != 0: A points to the [K, M] row-major bytes of A's transpose.  The wgrad of a linear layer,
     * dW = dY^T . X (src/nanotron/fp8/linear.py:107-109), reduces over the rows of both its operands: with
     * a_transposed and b_transposed set it reads dY[tokens, out] and X[tokens, in] as they are, where the reference
     * transposes both first (src/nanotron/fp8/kernel.py:43-44).  Only together with b_transposed, under its
     * conditions, and M a multiple of 16; anything else returns NTFP8_ERR_UNSUPPORTED. */
    int a_transposed;
} ntfp8_gemm_desc;
/* A call that returns an error has launched nothing: every problem is validated, and matched to a kernel, before
 * the first launch. */
int ntfp8_gemm_batch(const ntfp8_gemm_desc* problems, int count, void* stream);

/* fp8 GEMM output ("return an fp8 tensor as output", the TODO at src/nanotron/fp8/linear.py:63-64):
 * with d_dtype one of the two codes below, a problem of ntfp8_gemm_batch writes
 *   D[m,n] = sat_rne_fp8(r * *scale_d),  r = fp32 result as d_dtype NTFP8_F32 would store it,
 * i.e. the bytes ntfp8_cast_to_fp8 makes of the fp32 output, NaN -> sign|0x7F included, and the same
 * bytes transposed into D_t if given.  accumulate must be 0.  The amax of r cannot be known before
 * the GEMM has run, so the scale is one decided earlier (delayed scaling); the GEMM leaves max|r| in
 * amax_workspace, and ntfp8_amax_finalize, queued behind it on the same stream, turns that into the
 * bookkeeping of ntfp8_quantize_delayed:
 *   *amax_out = max|r| (NaN if any r is); hist <- roll(hist), hist[0] = amax;
 *   *scale_used_out = old *scale_state; *scale_state = update_scaling_factor(max(hist), old);
 * and zeroes the workspace again.  scale_d usually is scale_state.  amax_history may be NULL
 * (history_len 0): then only *amax_out and *scale_used_out are written. */
#define NTFP8_OUT_E4M3 3
#define NTFP8_OUT_E5M2 4
int ntfp8_amax_finalize(void* workspace, int fmt, int margin, float* scale_state, float* amax_history,
                        int history_len, float* amax_out, float* scale_used_out, void* stream);

/* Bandwidth yardstick: a kernel with the access pattern of the flat quantise kernels (same workgroup size, same grid,
 * 128-bit streaming loads and stores) and none of their arithmetic, so that a quantise figure can be set against what
 * the memory system gives that pattern on the same GPU in the same run.  It has no counterpart in the reference; it is
 * a measurement aid for the benchmark.  `bytes` (a multiple of 32) are read from src (16-byte aligned);
 * NTFP8_PROBE_READ writes nothing (dst: 16 bytes that are left alone in practice), NTFP8_PROBE_HALF writes bytes / 2
 * to dst (the traffic of a 16-bit -> fp8 cast), NTFP8_PROBE_COPY writes bytes. */
#define NTFP8_PROBE_READ 0
#define NTFP8_PROBE_HALF 1
#define NTFP8_PROBE_COPY 2
int ntfp8_stream_probe(int mode, const void* src, int64_t bytes, void* dst, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NTFP8_H */
