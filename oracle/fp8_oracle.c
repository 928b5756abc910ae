/* CPU oracle, C restatement, for the nanotron.fp8 hot path.  TEST INFRASTRUCTURE ONLY:
 * linked/loaded by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg as
 * the checker; never by the product library.
 *
 * It is written independently of oracle/fp8_oracle.py (integer-only fp8 encoder instead
 * of torch's cast) so that the two restatements pin each other.
 *
 * Reference lines followed (paths relative to the reference checkout):
 *   orc_amax            src/nanotron/fp8/tensor.py:25        amax = tensor.abs().max()
 *   orc_update_scale    src/nanotron/fp8/tensor.py:94-103    update_scaling_factor._inner
 *   orc_cast_to_fp8     src/nanotron/fp8/tensor.py:60-65     tex.cast_to_fp8 (TE, un-vendored):
 *                       out = sat_rne_fp8(fp32(x) * scale), OCP e4m3fn / e5m2
 *   orc_cast_from_fp8   src/nanotron/fp8/tensor.py:68-74     tex.cast_from_fp8: fp32(fp8) * (1/scale)
 *   orc_transpose       src/nanotron/fp8/kernel.py:43-44     tex.fp8_transpose
 *   orc_gemm_nt         src/nanotron/fp8/kernel.py:46-68     tex.te_gemm, TN form, fp32 accumulate,
 *                       one multiply by (1/scale_a)(1/scale_b)
 *   orc_delayed_step    build-defined amax-history roll (the reference has none)
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

enum { ORC_E4M3 = 0, ORC_E5M2 = 1 };
enum { ORC_F32 = 0, ORC_F16 = 1, ORC_BF16 = 2 };

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

static float half_to_float(uint16_t h) {
    uint32_t s = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1f, m = h & 0x3ff;
    if (e == 31) return u2f(s | 0x7f800000u | (m << 13));
    if (e == 0) {
        if (m == 0) return u2f(s);
        float v = (float)m * 5.9604644775390625e-08f; /* m * 2^-24, exact */
        return (s ? -v : v);
    }
    return u2f(s | ((e + 112) << 23) | (m << 13));
}

static inline float load_elem(const void* x, int dtype, int64_t i) {
    if (dtype == ORC_F32) return ((const float*)x)[i];
    if (dtype == ORC_BF16) return u2f((uint32_t)((const uint16_t*)x)[i] << 16);
    return half_to_float(((const uint16_t*)x)[i]);
}

float orc_fp8_max(int fmt) { return fmt == ORC_E4M3 ? 448.0f : 57344.0f; }

/* max |x|, NaN-propagating like torch.max. */
float orc_amax(const void* x, int dtype, int64_t n) {
    uint32_t best = 0; /* |x| compared as unsigned bit patterns: NaN (>0x7f800000) wins */
    for (int64_t i = 0; i < n; ++i) {
        uint32_t a = f2u(load_elem(x, dtype, i)) & 0x7fffffffu;
        if (a > best) best = a;
    }
    if (best > 0x7f800000u) return u2f(0x7fc00000u);
    return u2f(best);
}

/* tensor.py:97-103.  log2 is taken in double and rounded once to float, i.e. a correctly
 * rounded log2f; margin restricted to integers (pow(2,|exp|) is then an exact power of two
 * and round() is the identity). */
float orc_update_scale(float amax, float old_scale, int fmt, int margin) {
    float ratio = orc_fp8_max(fmt) / amax;           /* :97 */
    float l2 = (float)log2((double)ratio);
    float e = floorf(l2) - (float)margin;            /* :98 */
    float sf = roundf(powf(2.0f, fabsf(e)));         /* :99 */
    if (!(amax > 0.0f)) sf = old_scale;              /* :100 */
    if (!isfinite(amax)) sf = old_scale;             /* :101 */
    if (e < 0.0f) sf = 1.0f / sf;                    /* :102 */
    return sf;
}

/* Integer-only saturating round-to-nearest-even encoder from an fp32 bit pattern. */
uint8_t orc_encode_fp8(float y, int fmt) {
    const int M = (fmt == ORC_E4M3) ? 3 : 2;
    const int BIAS = (fmt == ORC_E4M3) ? 7 : 15;
    const uint8_t MAXCODE = (fmt == ORC_E4M3) ? 0x7e : 0x7b;
    const uint32_t MAXBITS = f2u(orc_fp8_max(fmt));
    uint32_t u = f2u(y);
    uint8_t sign = (uint8_t)((u >> 31) << 7);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return sign | 0x7f;  /* NaN */
    if (a >= MAXBITS) return sign | MAXCODE;  /* clamp (covers +-Inf) */
    int e32 = (int)(a >> 23);
    if (e32 == 0) return sign;                /* fp32 zero / denormal: far below half the smallest fp8 subnormal */
    uint32_t m24 = (a & 0x7fffffu) | 0x800000u;
    int e = e32 - 127;
    int emin = 1 - BIAS;
    int shift = 23 - M;
    uint32_t code_exp;
    if (e >= emin) {
        code_exp = (uint32_t)(e + BIAS);
    } else {
        shift += emin - e;
        code_exp = 0;
    }
    uint32_t q, rem, half;
    if (shift >= 32) { q = 0; rem = 1; half = 2; }
    else {
        q = m24 >> shift;
        rem = m24 & ((1u << shift) - 1u);
        half = 1u << (shift - 1);
    }
    if (rem > half || (rem == half && (q & 1u))) q += 1;
    uint32_t code;
    if (code_exp) code = ((code_exp - 1) << M) + q;  /* q carries the implicit one: (1<<M)+frac */
    else code = q;                                   /* subnormal; q may reach 1<<M = smallest normal */
    if (code > MAXCODE) code = MAXCODE;
    return sign | (uint8_t)code;
}

float orc_decode_fp8(uint8_t b, int fmt) {
    const int M = (fmt == ORC_E4M3) ? 3 : 2;
    const int BIAS = (fmt == ORC_E4M3) ? 7 : 15;
    const int EMAX = (fmt == ORC_E4M3) ? 15 : 31;
    int e = (b & 0x7f) >> M, m = b & ((1 << M) - 1);
    float v;
    if (fmt == ORC_E4M3 && e == EMAX && m == 7) v = NAN;
    else if (fmt == ORC_E5M2 && e == EMAX) v = m ? NAN : INFINITY;
    else if (e == 0) v = ldexpf((float)m, 1 - BIAS - M);
    else v = ldexpf((float)((1 << M) + m), e - BIAS - M);
    return (b & 0x80) ? -v : v;
}

void orc_cast_to_fp8(const void* x, int dtype, int64_t n, float scale, int fmt, uint8_t* out) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        volatile float y = load_elem(x, dtype, i) * scale; /* one fp32 RN multiply, no contraction */
        out[i] = orc_encode_fp8(y, fmt);
    }
}

void orc_cast_from_fp8(const uint8_t* q, int64_t n, float scale, int fmt, float* out) {
    float inv = 1.0f / scale;
    for (int64_t i = 0; i < n; ++i) out[i] = orc_decode_fp8(q[i], fmt) * inv;
}

void orc_transpose(const uint8_t* in, int64_t rows, int64_t cols, uint8_t* out) {
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) out[c * rows + r] = in[r * cols + c];
}

/* D[M,N] (+)= (sum_k A[m,k] B[n,k]) * (1/sa)(1/sb); fp32 accumulate in k order. */
void orc_gemm_nt(const uint8_t* A, int fmt_a, float scale_a, const uint8_t* B, int fmt_b, float scale_b,
                 float* D, int64_t M, int64_t N, int64_t K, int accumulate) {
    float ta[256], tb[256];
    for (int i = 0; i < 256; ++i) { ta[i] = orc_decode_fp8((uint8_t)i, fmt_a); tb[i] = orc_decode_fp8((uint8_t)i, fmt_b); }
    float alpha = (1.0f / scale_a) * (1.0f / scale_b);
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            float acc = 0.0f;
            const uint8_t* a = A + m * K;
            const uint8_t* b = B + n * K;
            for (int64_t k = 0; k < K; ++k) acc += ta[a[k]] * tb[b[k]];
            float v = acc * alpha;
            D[m * N + n] = accumulate ? D[m * N + n] + v : v;
        }
}

/* One delayed-scaling step: state = {scale, initialised flag}, hist[H].  Returns the
 * amax of x; writes the bytes, the scale used and updates hist / *scale_io. */
float orc_delayed_step(const void* x, int dtype, int64_t n, int fmt, int margin, float* hist, int H,
                       float* scale_io, int* initialised_io, uint8_t* out, float* scale_used) {
    float a = orc_amax(x, dtype, n);
    float s = *initialised_io ? *scale_io : orc_update_scale(a, 1.0f, fmt, margin);
    orc_cast_to_fp8(x, dtype, n, s, fmt, out);
    for (int i = H - 1; i > 0; --i) hist[i] = hist[i - 1];
    hist[0] = a;
    uint32_t best = 0;
    for (int i = 0; i < H; ++i) { uint32_t b = f2u(hist[i]) & 0x7fffffffu; if (b > best) best = b; }
    float hmax = best > 0x7f800000u ? u2f(0x7fc00000u) : u2f(best);
    *scale_io = orc_update_scale(hmax, s, fmt, margin);
    if (isfinite(a) && a > 0.0f) *initialised_io = 1;
    *scale_used = s;
    return a;
}
