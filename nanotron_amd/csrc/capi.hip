// extern "C" entry points declared in include/ntfp8.h: argument validation on the host, then one or
// two kernel launches on the caller's stream.  Nothing here allocates, frees or synchronises.
#include "common.h"

namespace ntfp8 {

int run_quant(int mode, const void* x, int x_dtype, int64_t rows, int64_t cols, int fmt, uint8_t* out, uint8_t* out_t,
              const float* scale_ptr, Workspace* ws, const ScalarIO& io, hipStream_t st);
int run_dequant(const void* in, int fmt, const float* scale, int is_inverse, int64_t n, void* out, int out_dtype,
                hipStream_t st);
int run_quant_dual(const void* x, int x_dtype, int64_t n, uint8_t* out_e4m3, uint8_t* out_e5m2, Workspace* ws,
                   const ScalarIO& io_e4m3, const ScalarIO& io_e5m2, hipStream_t st);
int static_scratch(void** out, hipStream_t st);
int run_quant_delayed_batch_static(QuantDesc* q, int count, hipStream_t st);
int run_transpose(const void* in, int64_t rows, int64_t cols, void* out, hipStream_t st);
int run_update_scale(const float* amax, const float* old_scale, int fmt, int margin, float* out, int64_t n,
                     hipStream_t st);
int run_amax_finalize(Workspace* ws, const ScalarIO& io, hipStream_t st);
int run_stream_probe(int mode, const void* src, int64_t bytes, void* dst, hipStream_t st);
int run_quant_delayed_batch(const QuantDesc* q, int count, hipStream_t st);
int run_gemm(const GemmDesc& g, hipStream_t st);
int run_gemm_batch(const GemmDesc* g, int n, hipStream_t st);

namespace {

constexpr int kMaxHistory = 65536;
constexpr int kMaxMargin = 126;

bool fmt_ok(int f) { return f == NTFP8_E4M3 || f == NTFP8_E5M2; }
bool dtype_ok(int d) { return d == NTFP8_F32 || d == NTFP8_F16 || d == NTFP8_BF16; }
size_t dtype_size(int d) { return d == NTFP8_F32 ? 4 : (is_fp8_out(d) ? 1 : 2); }
bool is_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// rows * cols as a positive int64, or false
bool numel(int64_t rows, int64_t cols, int64_t* n) {
    if (rows <= 0 || cols <= 0) return false;
    long long r;
    if (__builtin_smulll_overflow((long long)rows, (long long)cols, &r)) return false;
    if (r > (1LL << 46)) return false;
    *n = r;
    return true;
}

bool overlap(const void* a, size_t an, const void* b, size_t bn) {
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return a0 < b0 + bn && b0 < a0 + an;
}

int check_quant_common(const void* x, int x_dtype, int64_t rows, int64_t cols, int fmt, int margin, int64_t* n) {
    if (!x) return NTFP8_ERR_NULL;
    if (!fmt_ok(fmt) || !dtype_ok(x_dtype)) return NTFP8_ERR_ENUM;
    if (!numel(rows, cols, n)) return NTFP8_ERR_SIZE;
    if (margin < -kMaxMargin || margin > kMaxMargin) return NTFP8_ERR_SIZE;
    if (!is_aligned(x, dtype_size(x_dtype))) return NTFP8_ERR_ALIGN;
    return NTFP8_OK;
}

int check_outputs(const void* x, int x_dtype, int64_t n, const void* out, const void* out_t) {
    const size_t xb = (size_t)n * dtype_size(x_dtype);
    if (out && overlap(x, xb, out, (size_t)n)) return NTFP8_ERR_ALIAS;
    if (out_t && overlap(x, xb, out_t, (size_t)n)) return NTFP8_ERR_ALIAS;
    if (out && out_t && overlap(out, (size_t)n, out_t, (size_t)n)) return NTFP8_ERR_ALIAS;
    return NTFP8_OK;
}

// argument checks of one GEMM problem; fills the launchers' descriptor
int check_gemm(const ntfp8_gemm_desc& p, GemmDesc* g) {
    if (!p.A || !p.B || !p.D || !p.scale_a || !p.scale_b) return NTFP8_ERR_NULL;
    const bool fp8_out = is_fp8_out(p.d_dtype);
    if (!fmt_ok(p.fmt_a) || !fmt_ok(p.fmt_b) || !(dtype_ok(p.d_dtype) || fp8_out)) return NTFP8_ERR_ENUM;
    if (fp8_out && !p.scale_d) return NTFP8_ERR_NULL;
    const int64_t M = p.M, N = p.N, K = p.K;
    if (M <= 0 || N <= 0 || K <= 0 || M > 0x7fffff00LL || N > 0x7fffff00LL || K > 0x7fffff00LL) return NTFP8_ERR_SIZE;
    int64_t mn, mk, nk;
    if (!numel(M, N, &mn) || !numel(M, K, &mk) || !numel(N, K, &nk)) return NTFP8_ERR_SIZE;
    if (((M + 127) / 128) * ((N + 127) / 128) > 0x7fffffffLL) return NTFP8_ERR_SIZE;
    if (p.accumulate && p.d_dtype != NTFP8_F32) return NTFP8_ERR_UNSUPPORTED;
    if (!is_aligned(p.scale_a, 4) || !is_aligned(p.scale_b, 4) || !is_aligned(p.D, dtype_size(p.d_dtype)))
        return NTFP8_ERR_ALIGN;
    const size_t db = (size_t)mn * dtype_size(p.d_dtype);
    if (overlap(p.A, (size_t)mk, p.D, db) || overlap(p.B, (size_t)nk, p.D, db)) return NTFP8_ERR_ALIAS;
    if (p.bias) {
        if (p.b_transposed) return NTFP8_ERR_UNSUPPORTED;
        if (!dtype_ok(p.bias_dtype)) return NTFP8_ERR_ENUM;
        if (!is_aligned(p.bias, dtype_size(p.bias_dtype))) return NTFP8_ERR_ALIGN;
        if (overlap(p.bias, (size_t)N * dtype_size(p.bias_dtype), p.D, db)) return NTFP8_ERR_ALIAS;
    }
    *g = GemmDesc{p.A, p.fmt_a, p.scale_a, p.B, p.fmt_b, p.scale_b, p.D, p.d_dtype, (int)M, (int)N, (int)K, p.accumulate ? 1 : 0,
                  nullptr, nullptr, nullptr, p.b_transposed ? 1 : 0, p.bias, p.bias ? p.bias_dtype : NTFP8_F32,
                  p.scales_are_inverse ? 1 : 0, p.a_transposed ? 1 : 0};
    if (p.a_transposed && !p.b_transposed) return NTFP8_ERR_UNSUPPORTED;
    if (fp8_out) {
        if (!is_aligned(p.scale_d, 4) || (p.amax_workspace && !is_aligned(p.amax_workspace, 4))) return NTFP8_ERR_ALIGN;
        if (p.D_t && (overlap(p.A, (size_t)mk, p.D_t, db) || overlap(p.B, (size_t)nk, p.D_t, db) || overlap(p.D, db, p.D_t, db)))
            return NTFP8_ERR_ALIAS;
        if (p.amax_workspace &&
            (overlap(p.amax_workspace, NTFP8_WORKSPACE_BYTES, p.D, db) || (p.D_t && overlap(p.amax_workspace, NTFP8_WORKSPACE_BYTES, p.D_t, db))))
            return NTFP8_ERR_ALIAS;
        g->sd = p.scale_d;
        g->Dt = p.D_t;
        g->ws = p.amax_workspace;
    }
    return NTFP8_OK;
}

}  // namespace
}  // namespace ntfp8

using namespace ntfp8;

extern "C" {

int ntfp8_version(void) { return NTFP8_VERSION; }

const char* ntfp8_strerror(int code) {
    switch (code) {
        case NTFP8_OK: return "ok";
        case NTFP8_ERR_NULL: return "a required pointer is NULL";
        case NTFP8_ERR_ENUM: return "unknown format or dtype";
        case NTFP8_ERR_SIZE: return "size, history length or margin out of range";
        case NTFP8_ERR_ALIGN: return "pointer is not aligned to its element type";
        case NTFP8_ERR_UNSUPPORTED: return "request not supported";
        case NTFP8_ERR_LAUNCH: return "HIP reported an error at kernel launch";
        case NTFP8_ERR_ALIAS: return "an output overlaps an input or another output";
        default: return "unknown error code";
    }
}

int ntfp8_amax_scale(const void* x, int x_dtype, int64_t n, int fmt, int margin, const float* old_scale,
                     float* amax_out, float* scale_out, void* workspace, void* stream) {
    int64_t nn;
    if (!amax_out || !scale_out || !workspace) return NTFP8_ERR_NULL;
    int rc = check_quant_common(x, x_dtype, n, 1, fmt, margin, &nn);
    if (rc) return rc;
    if (!is_aligned(amax_out, 4) || !is_aligned(scale_out, 4) || !is_aligned(workspace, 4) ||
        (old_scale && !is_aligned(old_scale, 4)))
        return NTFP8_ERR_ALIGN;
    ScalarIO io = {old_scale, amax_out, scale_out, nullptr, nullptr, 0, fmt, margin};
    return run_quant(kModeAmaxOnly, x, x_dtype, nn, 1, fmt, nullptr, nullptr, nullptr, static_cast<Workspace*>(workspace),
                     io, static_cast<hipStream_t>(stream));
}

int ntfp8_update_scaling_factor(const float* amax, const float* old_scale, int fmt, int margin, float* out, int64_t n,
                                void* stream) {
    if (!amax || !old_scale || !out) return NTFP8_ERR_NULL;
    if (!fmt_ok(fmt)) return NTFP8_ERR_ENUM;
    if (n <= 0 || n > (1LL << 40) || margin < -kMaxMargin || margin > kMaxMargin) return NTFP8_ERR_SIZE;
    if (!is_aligned(amax, 4) || !is_aligned(old_scale, 4) || !is_aligned(out, 4)) return NTFP8_ERR_ALIGN;
    return run_update_scale(amax, old_scale, fmt, margin, out, n, static_cast<hipStream_t>(stream));
}

float ntfp8_update_scaling_factor_host(float amax, float old_scale, int fmt, int margin) {
    if (!fmt_ok(fmt) || margin < -kMaxMargin || margin > kMaxMargin) return bits_f32(kNanBits);
    return update_scale(amax, old_scale, fmt, margin);
}

int ntfp8_cast_to_fp8(const void* x, int x_dtype, int64_t rows, int64_t cols, const float* scale, int fmt, void* out,
                      void* out_t, void* stream) {
    int64_t n;
    if (!scale || (!out && !out_t)) return NTFP8_ERR_NULL;
    int rc = check_quant_common(x, x_dtype, rows, cols, fmt, 0, &n);
    if (rc) return rc;
    if (!is_aligned(scale, 4)) return NTFP8_ERR_ALIGN;
    rc = check_outputs(x, x_dtype, n, out, out_t);
    if (rc) return rc;
    ScalarIO io = {nullptr, nullptr, nullptr, nullptr, nullptr, 0, fmt, 0};
    return run_quant(kModeCastOnly, x, x_dtype, rows, cols, fmt, static_cast<uint8_t*>(out), static_cast<uint8_t*>(out_t),
                     scale, nullptr, io, static_cast<hipStream_t>(stream));
}

int ntfp8_quantize_current(const void* x, int x_dtype, int64_t rows, int64_t cols, int fmt, int margin, float* amax_out,
                           float* scale_used_out, void* out, void* out_t, float* amax_history, int history_len,
                           float* scale_state, void* workspace, void* stream) {
    int64_t n;
    if (!amax_out || !scale_used_out || !workspace || (!out && !out_t)) return NTFP8_ERR_NULL;
    int rc = check_quant_common(x, x_dtype, rows, cols, fmt, margin, &n);
    if (rc) return rc;
    if (amax_history) {
        if (!scale_state) return NTFP8_ERR_NULL;
        if (history_len < 1 || history_len > kMaxHistory) return NTFP8_ERR_SIZE;
        if (!is_aligned(amax_history, 4) || !is_aligned(scale_state, 4)) return NTFP8_ERR_ALIGN;
    }
    if (!is_aligned(amax_out, 4) || !is_aligned(scale_used_out, 4) || !is_aligned(workspace, 4)) return NTFP8_ERR_ALIGN;
    rc = check_outputs(x, x_dtype, n, out, out_t);
    if (rc) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    ScalarIO io = {nullptr, amax_out, scale_used_out, amax_history ? scale_state : nullptr, amax_history,
                   amax_history ? history_len : 0, fmt, margin};
    rc = run_quant(kModeAmaxOnly, x, x_dtype, n, 1, fmt, nullptr, nullptr, nullptr, static_cast<Workspace*>(workspace), io,
                   st);
    if (rc) return rc;
    ScalarIO none = {nullptr, nullptr, nullptr, nullptr, nullptr, 0, fmt, 0};
    return run_quant(kModeCastOnly, x, x_dtype, rows, cols, fmt, static_cast<uint8_t*>(out), static_cast<uint8_t*>(out_t),
                     scale_used_out, nullptr, none, st);
}

int ntfp8_quantize_first_use(const void* x, int x_dtype, int64_t rows, int64_t cols, int fmt, int margin, float* scale_state,
                             float* amax_history, int history_len, float* initialised, float* amax_out,
                             float* scale_used_out, void* out, void* out_t, void* workspace, void* stream) {
    int64_t n;
    if (!scale_state || !amax_history || !initialised || !amax_out || !scale_used_out || !workspace || (!out && !out_t))
        return NTFP8_ERR_NULL;
    int rc = check_quant_common(x, x_dtype, rows, cols, fmt, margin, &n);
    if (rc) return rc;
    if (history_len < 1 || history_len > kMaxHistory) return NTFP8_ERR_SIZE;
    if (!is_aligned(scale_state, 4) || !is_aligned(amax_history, 4) || !is_aligned(initialised, 4) || !is_aligned(amax_out, 4) ||
        !is_aligned(scale_used_out, 4) || !is_aligned(workspace, 4))
        return NTFP8_ERR_ALIGN;
    rc = check_outputs(x, x_dtype, n, out, out_t);
    if (rc) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // launch 1: amax, the decision between this tensor's scale and the held one, history roll, next scale
    ScalarIO io = {nullptr, amax_out, scale_used_out, scale_state, amax_history, history_len, fmt, margin, nullptr, nullptr,
                   initialised};
    rc = run_quant(kModeAmaxOnly, x, x_dtype, n, 1, fmt, nullptr, nullptr, nullptr, static_cast<Workspace*>(workspace), io,
                   st);
    if (rc) return rc;
    // launch 2: the cast with the scale launch 1 chose
    ScalarIO none = {nullptr, nullptr, nullptr, nullptr, nullptr, 0, fmt, 0};
    return run_quant(kModeCastOnly, x, x_dtype, rows, cols, fmt, static_cast<uint8_t*>(out), static_cast<uint8_t*>(out_t),
                     scale_used_out, nullptr, none, st);
}

int ntfp8_quantize_delayed(const void* x, int x_dtype, int64_t rows, int64_t cols, int fmt, int margin,
                           float* scale_state, float* amax_history, int history_len, float* amax_out,
                           float* scale_used_out, void* out, void* out_t, void* workspace, void* stream) {
    int64_t n;
    if (!scale_state || !amax_history || !amax_out || !workspace || (!out && !out_t)) return NTFP8_ERR_NULL;
    int rc = check_quant_common(x, x_dtype, rows, cols, fmt, margin, &n);
    if (rc) return rc;
    if (history_len < 1 || history_len > kMaxHistory) return NTFP8_ERR_SIZE;
    if (!is_aligned(scale_state, 4) || !is_aligned(amax_history, 4) || !is_aligned(amax_out, 4) ||
        !is_aligned(workspace, 4) || (scale_used_out && !is_aligned(scale_used_out, 4)))
        return NTFP8_ERR_ALIGN;
    rc = check_outputs(x, x_dtype, n, out, out_t);
    if (rc) return rc;
    ScalarIO io = {nullptr, amax_out, scale_used_out, scale_state, amax_history, history_len, fmt, margin};
    return run_quant(kModeDelayed, x, x_dtype, rows, cols, fmt, static_cast<uint8_t*>(out), static_cast<uint8_t*>(out_t),
                     scale_state, static_cast<Workspace*>(workspace), io, static_cast<hipStream_t>(stream));
}

// validation of a batched quantise call; fills q[0 .. count)
static int check_quant_batch(const ntfp8_quant_desc* tensors, int count, int max_count, bool own_workspaces, QuantDesc* q) {
    if (!tensors) return NTFP8_ERR_NULL;
    if (count <= 0 || count > max_count) return NTFP8_ERR_SIZE;
    for (int i = 0; i < count; ++i) {
        const ntfp8_quant_desc& t = tensors[i];
        int64_t n;
        if (!t.scale_state || !t.amax_history || !t.amax_out || (own_workspaces && !t.workspace) || (!t.out && !t.out_t))
            return NTFP8_ERR_NULL;
        int rc = check_quant_common(t.x, t.x_dtype, t.rows, t.cols, t.fmt, t.margin, &n);
        if (rc) return rc;
        if (t.history_len < 1 || t.history_len > kMaxHistory) return NTFP8_ERR_SIZE;
        if (!is_aligned(t.scale_state, 4) || !is_aligned(t.amax_history, 4) || !is_aligned(t.amax_out, 4) ||
            (own_workspaces && !is_aligned(t.workspace, 4)) || (t.scale_used_out && !is_aligned(t.scale_used_out, 4)))
            return NTFP8_ERR_ALIGN;
        rc = check_outputs(t.x, t.x_dtype, n, t.out, t.out_t);
        if (rc) return rc;
        for (int j = 0; j < i; ++j)   // the tensors run concurrently: nothing one of them writes may be shared
            if ((own_workspaces && tensors[j].workspace == t.workspace) || tensors[j].scale_state == t.scale_state ||
                tensors[j].amax_history == t.amax_history || tensors[j].amax_out == t.amax_out ||
                (t.out && tensors[j].out == t.out) || (t.out_t && tensors[j].out_t == t.out_t))
                return NTFP8_ERR_ALIAS;
        q[i] = QuantDesc{t.x, t.x_dtype, t.rows, t.cols, t.fmt, t.out, t.out_t, own_workspaces ? t.workspace : nullptr,
                         ScalarIO{nullptr, t.amax_out, t.scale_used_out, t.scale_state, t.amax_history, t.history_len, t.fmt,
                                  t.margin}};
    }
    return NTFP8_OK;
}

int ntfp8_quantize_delayed_batch(const ntfp8_quant_desc* tensors, int count, void* stream) {
    QuantDesc q[NTFP8_MAX_BATCH];
    const int rc = check_quant_batch(tensors, count, NTFP8_MAX_BATCH, true, q);
    if (rc) return rc;
    return run_quant_delayed_batch(q, count, static_cast<hipStream_t>(stream));
}

/* BEGIN static-scratch entry points */
int ntfp8_static_init(void* stream) {
    void* p = nullptr;
    return static_scratch(&p, static_cast<hipStream_t>(stream));
}

int ntfp8_quantize_delayed_batch_static(const ntfp8_quant_desc* tensors, int count, void* stream) {
    QuantDesc q[NTFP8_STATIC_MAX_TENSORS];
    const int rc = check_quant_batch(tensors, count, NTFP8_STATIC_MAX_TENSORS, false, q);
    if (rc) return rc;
    return run_quant_delayed_batch_static(q, count, static_cast<hipStream_t>(stream));
}
/* END static-scratch entry points */

int ntfp8_te_cast_to_fp8(const void* x, int x_dtype, int64_t n, const float* scale, float* amax_inout, float* scale_inv_out,
                         int fmt, void* out, void* workspace, void* stream) {
    int64_t nn;
    if (!scale || !out) return NTFP8_ERR_NULL;
    const bool bookkeeping = amax_inout || scale_inv_out;
    if (bookkeeping && !workspace) return NTFP8_ERR_NULL;
    int rc = check_quant_common(x, x_dtype, n, 1, fmt, 0, &nn);
    if (rc) return rc;
    if (!is_aligned(scale, 4) || (amax_inout && !is_aligned(amax_inout, 4)) || (scale_inv_out && !is_aligned(scale_inv_out, 4)) ||
        (workspace && !is_aligned(workspace, 4)))
        return NTFP8_ERR_ALIGN;
    rc = check_outputs(x, x_dtype, nn, out, nullptr);
    if (rc) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (!bookkeeping) {
        ScalarIO io = {nullptr, nullptr, nullptr, nullptr, nullptr, 0, fmt, 0};
        return run_quant(kModeCastOnly, x, x_dtype, nn, 1, fmt, static_cast<uint8_t*>(out), nullptr, scale, nullptr, io, st);
    }
    // the fused pass: cast with *scale, amax of x, no history
    ScalarIO io = {nullptr, amax_inout, nullptr, const_cast<float*>(scale), nullptr, 0, fmt, 0, amax_inout, scale_inv_out};
    rc = run_quant(kModeDelayed, x, x_dtype, nn, 1, fmt, static_cast<uint8_t*>(out), nullptr, scale,
                   static_cast<Workspace*>(workspace), io, st);
    return rc;
}

int ntfp8_quantize_delayed_dual(const void* x, int x_dtype, int64_t n, int margin, float* scale_state_e4m3,
                                float* amax_history_e4m3, float* scale_state_e5m2, float* amax_history_e5m2, int history_len,
                                float* amax_out, float* scale_used_out_e4m3, float* scale_used_out_e5m2, void* out_e4m3,
                                void* out_e5m2, void* workspace, void* stream) {
    int64_t nn;
    if (!scale_state_e4m3 || !amax_history_e4m3 || !scale_state_e5m2 || !amax_history_e5m2 || !amax_out || !out_e4m3 ||
        !out_e5m2 || !workspace)
        return NTFP8_ERR_NULL;
    int rc = check_quant_common(x, x_dtype, n, 1, NTFP8_E4M3, margin, &nn);
    if (rc) return rc;
    if (history_len < 1 || history_len > kMaxHistory) return NTFP8_ERR_SIZE;
    if (!is_aligned(scale_state_e4m3, 4) || !is_aligned(amax_history_e4m3, 4) || !is_aligned(scale_state_e5m2, 4) ||
        !is_aligned(amax_history_e5m2, 4) || !is_aligned(amax_out, 4) || !is_aligned(workspace, 4) ||
        (scale_used_out_e4m3 && !is_aligned(scale_used_out_e4m3, 4)) || (scale_used_out_e5m2 && !is_aligned(scale_used_out_e5m2, 4)))
        return NTFP8_ERR_ALIGN;
    rc = check_outputs(x, x_dtype, nn, out_e4m3, out_e5m2);
    if (rc) return rc;
    if (scale_state_e4m3 == scale_state_e5m2 || amax_history_e4m3 == amax_history_e5m2 ||
        (scale_used_out_e4m3 && scale_used_out_e4m3 == scale_used_out_e5m2))
        return NTFP8_ERR_ALIAS;
    ScalarIO io0 = {nullptr, amax_out, scale_used_out_e4m3, scale_state_e4m3, amax_history_e4m3, history_len, NTFP8_E4M3, margin};
    ScalarIO io1 = {nullptr, amax_out, scale_used_out_e5m2, scale_state_e5m2, amax_history_e5m2, history_len, NTFP8_E5M2, margin};
    return run_quant_dual(x, x_dtype, nn, static_cast<uint8_t*>(out_e4m3), static_cast<uint8_t*>(out_e5m2),
                          static_cast<Workspace*>(workspace), io0, io1, static_cast<hipStream_t>(stream));
}

int ntfp8_cast_from_fp8(const void* in, int fmt, const float* scale, int64_t n, void* out, int out_dtype, void* stream) {
    if (!in || !scale || !out) return NTFP8_ERR_NULL;
    if (!fmt_ok(fmt) || !dtype_ok(out_dtype)) return NTFP8_ERR_ENUM;
    if (n <= 0 || n > (1LL << 46)) return NTFP8_ERR_SIZE;
    if (!is_aligned(scale, 4) || !is_aligned(out, dtype_size(out_dtype))) return NTFP8_ERR_ALIGN;
    if (overlap(in, (size_t)n, out, (size_t)n * dtype_size(out_dtype))) return NTFP8_ERR_ALIAS;
    return run_dequant(in, fmt, scale, 0, n, out, out_dtype, static_cast<hipStream_t>(stream));
}

int ntfp8_cast_from_fp8_scale_inv(const void* in, int fmt, const float* scale_inv, int64_t n, void* out, int out_dtype,
                                  void* stream) {
    if (!in || !scale_inv || !out) return NTFP8_ERR_NULL;
    if (!fmt_ok(fmt) || !dtype_ok(out_dtype)) return NTFP8_ERR_ENUM;
    if (n <= 0 || n > (1LL << 46)) return NTFP8_ERR_SIZE;
    if (!is_aligned(scale_inv, 4) || !is_aligned(out, dtype_size(out_dtype))) return NTFP8_ERR_ALIGN;
    if (overlap(in, (size_t)n, out, (size_t)n * dtype_size(out_dtype))) return NTFP8_ERR_ALIAS;
    return run_dequant(in, fmt, scale_inv, 1, n, out, out_dtype, static_cast<hipStream_t>(stream));
}

int ntfp8_transpose(const void* in, int64_t rows, int64_t cols, void* out, void* stream) {
    int64_t n;
    if (!in || !out) return NTFP8_ERR_NULL;
    if (!numel(rows, cols, &n)) return NTFP8_ERR_SIZE;
    if (overlap(in, (size_t)n, out, (size_t)n)) return NTFP8_ERR_ALIAS;
    return run_transpose(in, rows, cols, out, static_cast<hipStream_t>(stream));
}

int ntfp8_gemm(const void* A, int fmt_a, const float* scale_a, const void* B, int fmt_b, const float* scale_b, void* D,
               int d_dtype, int64_t M, int64_t N, int64_t K, int accumulate, void* stream) {
    if (is_fp8_out(d_dtype)) return NTFP8_ERR_UNSUPPORTED;   // fp8 outputs carry more arguments: ntfp8_gemm_batch
    const ntfp8_gemm_desc p = {A, scale_a, B, scale_b, D, M, N, K, fmt_a, fmt_b, d_dtype, accumulate, nullptr, nullptr, nullptr, 0,
                               nullptr, NTFP8_F32, 0, 0};
    GemmDesc g;
    const int rc = check_gemm(p, &g);
    if (rc) return rc;
    return run_gemm(g, static_cast<hipStream_t>(stream));
}

int ntfp8_gemm_batch(const ntfp8_gemm_desc* problems, int count, void* stream) {
    if (!problems) return NTFP8_ERR_NULL;
    if (count <= 0 || count > NTFP8_MAX_BATCH) return NTFP8_ERR_SIZE;
    GemmDesc g[NTFP8_MAX_BATCH];
    for (int i = 0; i < count; ++i) {
        const int rc = check_gemm(problems[i], &g[i]);
        if (rc) return rc;
    }
    // independence: an output (D, its transposed copy, its amax slots) overlaps nothing of any other problem
    for (int i = 0; i < count; ++i) {
        const size_t di = (size_t)g[i].M * g[i].N * dtype_size(g[i].d_dtype);
        const void* outs_i[3] = {g[i].D, g[i].Dt, g[i].ws};
        const size_t size_i[3] = {di, di, NTFP8_WORKSPACE_BYTES};
        for (int j = 0; j < count; ++j) {
            if (i == j) continue;
            const size_t dj = (size_t)g[j].M * g[j].N * dtype_size(g[j].d_dtype);
            const void* outs_j[3] = {g[j].D, g[j].Dt, g[j].ws};
            const size_t size_j[3] = {dj, dj, NTFP8_WORKSPACE_BYTES};
            for (int a = 0; a < 3; ++a) {
                if (!outs_i[a]) continue;
                if (overlap(outs_i[a], size_i[a], g[j].A, (size_t)g[j].M * g[j].K) ||
                    overlap(outs_i[a], size_i[a], g[j].B, (size_t)g[j].N * g[j].K))
                    return NTFP8_ERR_ALIAS;
                for (int b = 0; b < 3; ++b)
                    if (i < j && outs_j[b] && overlap(outs_i[a], size_i[a], outs_j[b], size_j[b])) return NTFP8_ERR_ALIAS;
            }
        }
    }
    return run_gemm_batch(g, count, static_cast<hipStream_t>(stream));
}

int ntfp8_amax_finalize(void* workspace, int fmt, int margin, float* scale_state, float* amax_history, int history_len,
                        float* amax_out, float* scale_used_out, void* stream) {
    if (!workspace || !scale_state || !amax_out) return NTFP8_ERR_NULL;
    if (!fmt_ok(fmt)) return NTFP8_ERR_ENUM;
    if (margin < -kMaxMargin || margin > kMaxMargin) return NTFP8_ERR_SIZE;
    if (amax_history ? (history_len < 1 || history_len > kMaxHistory) : history_len != 0) return NTFP8_ERR_SIZE;
    if (!is_aligned(workspace, 4) || !is_aligned(scale_state, 4) || !is_aligned(amax_out, 4) ||
        (amax_history && !is_aligned(amax_history, 4)) || (scale_used_out && !is_aligned(scale_used_out, 4)))
        return NTFP8_ERR_ALIGN;
    ScalarIO io = {nullptr, amax_out, scale_used_out, scale_state, amax_history, history_len, fmt, margin};
    return run_amax_finalize(static_cast<Workspace*>(workspace), io, static_cast<hipStream_t>(stream));
}

int ntfp8_stream_probe(int mode, const void* src, int64_t bytes, void* dst, void* stream) {
    if (!src || !dst) return NTFP8_ERR_NULL;
    if (mode < NTFP8_PROBE_READ || mode > NTFP8_PROBE_COPY) return NTFP8_ERR_ENUM;
    if (bytes < 32 || bytes % 32 != 0 || bytes > (1LL << 46)) return NTFP8_ERR_SIZE;
    if (!is_aligned(src, 16) || !is_aligned(dst, 16)) return NTFP8_ERR_ALIGN;
    const size_t written = mode == NTFP8_PROBE_READ ? 16 : (mode == NTFP8_PROBE_HALF ? (size_t)bytes / 2 : (size_t)bytes);
    if (overlap(src, (size_t)bytes, dst, written)) return NTFP8_ERR_ALIAS;
    return run_stream_probe(mode, src, bytes, dst, static_cast<hipStream_t>(stream));
}

}  // extern "C"
