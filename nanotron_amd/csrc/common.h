// Shared device helpers for the gfx950 FP8 kernels.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/ntfp8.h"

namespace ntfp8 {

constexpr int kE4M3 = NTFP8_E4M3;
constexpr int kE5M2 = NTFP8_E5M2;

constexpr uint32_t kInfBits = 0x7f800000u;
constexpr uint32_t kNanBits = 0x7fc00000u;

// Reduction scratch shared by the blocks of one launch.  All zero between launches.
// Every counter sits on its own 128-byte line: atomics on one address serialise (~10 ns each on
// MI355X), atomics on different lines proceed in parallel.
constexpr int kMaxSlots = 8;
struct Workspace {
    uint32_t ticket;  // number of slot groups whose last block has arrived
    uint32_t pad0[31];
    struct {
        uint32_t bits;    // running max of |x| as an unsigned bit pattern (NaN patterns compare above Inf)
        uint32_t ticket;  // number of blocks of this slot's group (blockIdx % kMaxSlots) that have published
        uint32_t pad[30];
    } slot[kMaxSlots];
    uint32_t pad1[(NTFP8_WORKSPACE_BYTES - 128 - 128 * kMaxSlots) / 4];
};
static_assert(sizeof(Workspace) == NTFP8_WORKSPACE_BYTES, "workspace size is part of the ABI");

enum Mode { kModeAmaxOnly = 0, kModeCastOnly = 1, kModeDelayed = 2 };

// Scalar bookkeeping written by the last block of a launch.
struct ScalarIO {
    const float* old_scale;  // amax-only mode: previous scale (NULL = 1.0)
    float* amax_out;         // amax of this tensor
    float* scale_out;        // scale the bytes are / will be produced with
    float* scale_state;      // delayed scaling: scale for the next step (in/out)
    float* hist;             // amax history, newest first (may be NULL)
    int hist_len;
    int fmt;
    int margin;
    // Transformer-Engine-shaped cast (tex.cast_to_fp8 takes `amax` and `scale_inv` tensors and updates both):
    const float* amax_in;    // not NULL: *amax_out = max(*amax_in, amax of this tensor), NaN from either side kept
    float* scale_inv_out;    // not NULL: receives 1 / (scale the bytes were produced with)
    // First use of a delayed-scaling role (amax-only mode): 0.0 = no usable amax recorded yet, scale from this tensor's
    // amax; anything else = the role holds a scale, *scale_state is used.  Set to 1.0 when this amax is finite and > 0.
    float* init_flag;
};

// one tensor of a batched quantise call as the launchers see it (validated by the C entry point)
struct QuantDesc {
    const void* x;
    int x_dtype;
    int64_t rows, cols;
    int fmt;
    void* out;
    void* out_t;
    void* ws;
    ScalarIO io;
};

template <int F>
struct Fmt;
template <>
struct Fmt<kE4M3> {
    static constexpr float kMax = 448.0f;
};
template <>
struct Fmt<kE5M2> {
    static constexpr float kMax = 57344.0f;
};

__host__ __device__ inline float fp8_max_of(int fmt) { return fmt == kE4M3 ? 448.0f : 57344.0f; }

__host__ __device__ inline uint32_t f32_bits(float f) { return __builtin_bit_cast(uint32_t, f); }
__host__ __device__ inline float bits_f32(uint32_t u) { return __builtin_bit_cast(float, u); }

// update_scaling_factor of the reference (src/nanotron/fp8/tensor.py:97-103), for integer margins:
//   ratio = fp8_max / amax; exp = floor(log2(ratio)) - margin; sf = round(2^|exp|);
//   sf = old unless amax > 0 and finite; sf = 1/sf if exp < 0.
// log2 is evaluated in double and rounded once to float (a correctly rounded log2f), so quotients a
// few ulps below a power of two land on that power exactly as the float formula does.
__host__ __device__ inline float update_scale(float amax, float old_scale, int fmt, int margin) {
    const uint32_t ab = f32_bits(amax);
    const uint32_t mag = ab & 0x7fffffffu;
    if (mag > kInfBits) return old_scale;            // NaN: every comparison false, scale held
    if (mag == kInfBits) return 1.0f / old_scale;    // +-Inf: ratio = +-0, log2 = -inf < 0 -> 1/old
    if ((ab >> 31) || mag == 0u) return old_scale;   // amax <= 0: scale held
    const float ratio = fp8_max_of(fmt) / amax;      // IEEE round-to-nearest division
    if ((f32_bits(ratio) & 0x7fffffffu) >= kInfBits) return bits_f32(kInfBits);
    // floor(float(log2(ratio))).  Rounded to float, the logarithm reaches the next integer only for a ratio within a few
    // tens of mantissa steps below a power of two (the spacing of floats near |k| <= 128 is at most 44 steps of
    // d log2 / d mantissa = 8.6e-8): every other normal ratio gives its own exponent, read off the bits.  The double
    // logarithm, a long software routine that the last workgroup of a quantise launch runs on one lane while the
    // whole GPU waits for it, is only evaluated for those few and for subnormal ratios.
    const uint32_t rb = f32_bits(ratio);
    int fl;
    if ((rb >> 23) != 0u && (rb & 0x7fffffu) < 0x7fff00u) fl = (int)(rb >> 23) - 127;
    else fl = (int)floorf((float)log2((double)ratio));
    const int e = fl - margin;
    const int ae = e < 0 ? -e : e;
    if (ae >= 128) return e < 0 ? 0.0f : bits_f32(kInfBits);
    // 2^e as a bit pattern (normal for e >= -126, subnormal below)
    if (e >= -126) return bits_f32((uint32_t)(e + 127) << 23);
    return bits_f32(1u << (149 + e));
}

// Two packed conversions: 4 floats -> 4 fp8 bytes (little-endian order a,b,c,d).
template <int F>
__device__ __forceinline__ uint32_t cvt4(float a, float b, float c, float d) {
    int r = 0;
    if constexpr (F == kE4M3) {
        r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, r, false);
        r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
    } else {
        r = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, r, false);
        r = __builtin_amdgcn_cvt_pk_bf8_f32(c, d, r, true);
    }
    return (uint32_t)r;
}

// y -> clamp to +-max (exact for every non-NaN y).  NaN lanes are patched by the caller.
template <int F>
__device__ __forceinline__ float sat(float y) {
    return __builtin_amdgcn_fmed3f(y, -Fmt<F>::kMax, Fmt<F>::kMax);
}

// NaN -> sign|0x7F in both formats.
__device__ __forceinline__ uint32_t patch_nan(uint32_t word, int lane_byte, float y) {
    if (y != y) {
        const uint32_t b = ((__float_as_uint(y) >> 24) & 0x80u) | 0x7fu;
        word = (word & ~(0xffu << (8 * lane_byte))) | (b << (8 * lane_byte));
    }
    return word;
}

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __uint_as_float(b << 16); }

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
    return __half2float(__ushort_as_half((unsigned short)h));
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)v, off, 64);
        v = o > v ? o : v;
    }
    return v;
}

// one GEMM problem as the launchers see it (validated by the C entry points)
struct GemmDesc {
    const void* A;
    int fmt_a;
    const float* sa;
    const void* B;
    int fmt_b;
    const float* sb;
    void* D;
    int d_dtype;
    int M, N, K;
    int accumulate;
    // fp8 outputs (d_dtype NTFP8_OUT_*): scale applied before the cast, optional transposed copy, optional amax slots
    const float* sd;
    void* Dt;
    void* ws;
    int tb;   // B is given as [K, N] row-major (its transpose)
    // optional bias[N] added to the descaled fp32 result before the single rounding (NULL: none)
    const void* bias;
    int bias_dtype;
    int scale_inv;   // scale_a / scale_b point to inverse scales (what tex.te_gemm receives): multiplied, not divided by
    int ta;          // A is given as [K, M] row-major (its transpose); only together with tb
};

__host__ __device__ inline bool is_fp8_out(int d_dtype) { return d_dtype == NTFP8_OUT_E4M3 || d_dtype == NTFP8_OUT_E5M2; }

// compute units of the current device (cached per device; threads may race to fill an entry, with the same value)
inline int cu_count() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int v = cached[dev].load(std::memory_order_relaxed);
    if (v == 0) {
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
        cached[dev].store(v, std::memory_order_relaxed);
    }
    return v;
}

}  // namespace ntfp8
