// Helpers shared by the FP8 GEMM kernels: vector types, output conversion, LDS/buffer primitives,
// tile ordering and the epilogue for 32 x 32 accumulator blocks.
#pragma once
#include <type_traits>

#include "common.h"

namespace ntfp8 {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr;

constexpr int kBK = 128;     // bytes of K per LDS stage
// Tile order: groups of kGroupM row-tiles, swept along N.  With 32 consecutive tiles of a round on one XCD (one per
// CU), an XCD then works on a block of 4 row-tiles x 8 column-tiles: 4 A panels and 8 B panels per K step in its L2.
// The transposed block (8 x 4, kGroupM = 8) moves the same number of panels and measured 2-6 % slower on the
// one-round shapes (4096^3: 56.2 -> 52.8 us), 2 x 16 and 16 x 2 slower still on the long and wide ones.
constexpr int kGroupM = 4;
constexpr int kXcds = 8;     // workgroups are dealt round-robin to the 8 XCDs, each with its own L2

// 16-byte chunk `kc` (0..7) of tile row `row`, swizzled so that the 16 lanes of a 128-bit LDS access
// that read the same chunk of 16 consecutive rows touch 16 distinct 16-byte bank groups.
__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int lds_off(int row, int kc) { return row * kBK + ((kc ^ swz(row)) << 4); }

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float v) {
    const uint32_t u = __float_as_uint(v);
    if ((u & 0x7fffffffu) > kInfBits) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

// Output element types.  cvt() rounds one value, pack2() two values into one 32-bit word (first value
// in the low half) with the packed hardware conversions (V_CVT_PK_BF16_F32 / V_CVT_PK_F16_F32, both
// round-to-nearest-even).
template <int D>
struct OutT;
template <>
struct OutT<NTFP8_F32> {
    typedef float type;
    __device__ static __forceinline__ float cvt(float v) { return v; }
};
template <>
struct OutT<NTFP8_BF16> {
    typedef uint16_t type;
    __device__ static __forceinline__ uint16_t cvt(float v) { return f32_to_bf16_rne(v); }
    __device__ static __forceinline__ uint32_t pack2(float a, float b) {
        return __builtin_bit_cast(uint32_t, __builtin_convertvector((v2f){a, b}, v2bf));
    }
};
template <>
struct OutT<NTFP8_F16> {
    typedef uint16_t type;
    __device__ static __forceinline__ uint16_t cvt(float v) {
        asm volatile("" : "+v"(v));  // no folding of the descale multiply into a mixed-precision fma (-0 would become +0)
        return __half_as_ushort(__float2half_rn(v));
    }
    __device__ static __forceinline__ uint32_t pack2(float a, float b) {
        asm volatile("" : "+v"(a), "+v"(b));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector((v2f){a, b}, v2h));
    }
};

// Device-only builtins live in __device__ helpers: written directly inside a __global__ template they
// are non-dependent expressions that the host pass cannot resolve.
__device__ __forceinline__ void wg_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}
// x of lanes 32..63 <-> y of lanes 0..31 (V_PERMLANE32_SWAP)
__device__ __forceinline__ void swap_halves(uint32_t& x, uint32_t& y) {
    typedef unsigned v2u __attribute__((ext_vector_type(2)));
    const v2u r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
    x = r.x;
    y = r.y;
}
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}
// 16 bytes per lane from global memory straight into LDS: lane i lands at dst + 16 * i.  Offsets past
// the descriptor's size read as zero.
__device__ __forceinline__ void lds_load16(__amdgpu_buffer_rsrc_t r, lds_ptr dst, uint32_t voff, int soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, dst, 16, voff, soff, 0, 0);
}
template <int FA, int FB>
__device__ __forceinline__ v16f mfma_32x32x64(v8i b_frag, v8i a_frag, v16f c) {
    // The B-matrix fragment is the first source, so the 32x32 result block is indexed [n][m]: each
    // lane then owns 4 consecutive n of one output row m.
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b_frag, a_frag, c, FB, FA, 0, 0, 0, 0);
}

// scale product applied to the accumulated sum: the operands' scales divide it; inverse scales (the form
// tex.te_gemm is handed, src/nanotron/fp8/kernel.py:48,52) multiply it
__device__ __forceinline__ float descale_factor(const float* scale_a, const float* scale_b, int scale_inv) {
    const float sa = *scale_a, sb = *scale_b;
    return scale_inv ? sa * sb : (1.0f / sa) * (1.0f / sb);
}

// element n of a bias vector of any supported type, as fp32 (exact)
__device__ __forceinline__ float bias_at(const void* bias, int dtype, int n) {
    if (dtype == NTFP8_F32) return static_cast<const float*>(bias)[n];
    const uint32_t h = static_cast<const uint16_t*>(bias)[n];
    return dtype == NTFP8_BF16 ? bf16_bits_to_float(h) : half_bits_to_float(h);
}

// Bias in the epilogue: D = round(fp32(acc * alpha) + bias[n]), two separately rounded fp32 operations before the
// single rounding to the output type (what `output + bias` does to an fp32 GEMM output, src/nanotron/fp8/linear.py:65).
// load_bias16: the bias values of the columns a lane owns in 16 x 16 accumulator blocks, bv[j][e] = bias of column
// n_base + 16 j + 4 (lane / 16) + e (zero past N: those columns are never stored).
template <int NJ>
__device__ __forceinline__ void load_bias16(float (&bv)[NJ][4], const void* bias, int bias_dtype, int N, int n_base, int lane) {
    const int q = lane >> 4;
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int n = n_base + j * 16 + q * 4 + e;
            bv[j][e] = n < N ? bias_at(bias, bias_dtype, n) : 0.0f;
        }
}
// 32 x 32 accumulator blocks (the small kernel, off the fast path): acc <- fp32(acc * alpha) + bias[n] in place, after
// which the store routines run unchanged with alpha = 1 (a multiplication by one changes nothing).
template <int MI, int NJ>
__device__ __forceinline__ void add_bias32(v16f (&acc)[MI][NJ], float alpha, const void* bias, int bias_dtype, int N,
                                           int n_base, int lane) {
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float b[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int n = n_base + j * 32 + g * 8 + (lane >> 5) * 4 + e;
                b[e] = n < N ? bias_at(bias, bias_dtype, n) : 0.0f;
            }
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[i][j][g * 4 + e] = acc[i][j][g * 4 + e] * alpha + b[e];
        }
}

// what a problem carries beside its operands and output
struct GemmExtras {
    const void* bias;   // NULL, or bias[N]
    int bias_dtype;     // NTFP8_F32 / NTFP8_F16 / NTFP8_BF16
    int scale_inv;      // the scale pointers hold inverse scales
};

// tile order: XCD-contiguous, then kGroupM row-tiles swept before moving along N
__device__ __forceinline__ void tile_of_block(int tiles_m, int tiles_n, int& pid_m, int& pid_n) {
    int pid = blockIdx.x;
    const int nwg = gridDim.x;
    if (nwg % kXcds == 0) pid = (pid % kXcds) * (nwg / kXcds) + pid / kXcds;
    const int in_group = kGroupM * tiles_n;
    const int group = pid / in_group;
    const int first_m = group * kGroupM;
    const int gsz = min(tiles_m - first_m, kGroupM);
    pid_m = first_m + (pid % in_group) % gsz;
    pid_n = (pid % in_group) / gsz;
}

// Epilogue of one wave: MI x NJ accumulator blocks of 32 x 32, block (i, j) at rows m_base + 32 i,
// columns n_base + 32 j.  Descale, optional fp32 accumulate, one rounding, store.
template <int DT, bool kAcc, int MI, int NJ>
__device__ __forceinline__ void store_wave_tile(const v16f (&acc)[MI][NJ], void* __restrict__ Dv, float alpha, int M,
                                                int N, int m_base, int n_base, int lane) {
    typedef typename OutT<DT>::type O;
    O* D = static_cast<O*>(Dv);
    if constexpr (DT != NTFP8_F32) {
        // 16-bit outputs: a lane's 4 consecutive n are only 8 bytes, and the two 32-lane halves of the
        // wave hold adjacent groups of 4.  Swapping registers between the halves gives every lane 8
        // consecutive n (16 bytes), and lanes l / l + 32 together a full 32-byte sector per row, which
        // is what the memory side writes without read-modify-write traffic.
        if ((N & 7) == 0) {
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                const int m = m_base + i * 32 + (lane & 31);
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
#pragma unroll
                    for (int q = 0; q < 2; ++q) {
                        uint32_t w[4];
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const int g = 2 * q + h;
                            w[2 * h] = OutT<DT>::pack2(acc[i][j][g * 4 + 0] * alpha, acc[i][j][g * 4 + 1] * alpha);
                            w[2 * h + 1] = OutT<DT>::pack2(acc[i][j][g * 4 + 2] * alpha, acc[i][j][g * 4 + 3] * alpha);
                        }
                        swap_halves(w[0], w[2]);
                        swap_halves(w[1], w[3]);
                        const int n = n_base + j * 32 + (2 * q + (lane >> 5)) * 8;
                        if (m < M && n < N)
                            *reinterpret_cast<v4i*>(D + (int64_t)m * N + n) = (v4i){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
                    }
                }
            }
            return;
        }
    }
    const bool vec_ok = (N & 3) == 0;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int m = m_base + i * 32 + (lane & 31);
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n_base + j * 32 + g * 8 + (lane >> 5) * 4;
                if (n >= N) continue;
                O* dp = D + (int64_t)m * N + n;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc[i][j][g * 4 + e] * alpha;
                if (vec_ok && n + 3 < N) {
                    if constexpr (DT == NTFP8_F32) {
                        v4f o = {v[0], v[1], v[2], v[3]};
                        if constexpr (kAcc) {
                            const v4f old = *reinterpret_cast<const v4f*>(dp);
                            o = o + old;
                        }
                        *reinterpret_cast<v4f*>(dp) = o;
                    } else {
                        const uint32_t lo = OutT<DT>::pack2(v[0], v[1]);
                        const uint32_t hi = OutT<DT>::pack2(v[2], v[3]);
                        *reinterpret_cast<uint2*>(dp) = make_uint2(lo, hi);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (n + e < N) {
                            if constexpr (DT == NTFP8_F32) {
                                float o = v[e];
                                if constexpr (kAcc) o = o + dp[e];
                                dp[e] = o;
                            } else {
                                dp[e] = OutT<DT>::cvt(v[e]);
                            }
                        }
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// fp8 outputs: bytes = sat_rne_fp8(r * scale_d) of the descaled fp32 results r, optionally also
// transposed, and max|r| for the delayed-scaling bookkeeping of the output.
struct Fp8Out {
    const float* scale;   // device scalar applied before the cast
    uint8_t* Dt;          // NULL, or the [N, M] transposed copy
    Workspace* ws;        // NULL, or the slots that collect max|r|
};

__device__ __forceinline__ bool scale_is_degenerate(float s) {   // 0, Inf or NaN: products can be NaN
    const uint32_t b = __float_as_uint(s) & 0x7fffffffu;
    return b == 0u || b >= kInfBits;
}

// Four results -> one word of fp8 bytes (first value in the low byte); amax_bits collects |r| as unsigned
// bit patterns (NaN patterns compare above Inf).  The clamp turns a NaN into a number, so NaN bytes are patched
// in afterwards; that is rare and sits behind a branch the whole wave takes or skips: `slow` (the scale is
// degenerate, any product may be NaN) or some lane holding a NaN result.
template <int F>
__device__ __forceinline__ uint32_t quant4(float r0, float r1, float r2, float r3, float scale_d, bool slow,
                                           uint32_t& amax_bits) {
    const uint32_t a01 = max(__float_as_uint(r0) & 0x7fffffffu, __float_as_uint(r1) & 0x7fffffffu);
    const uint32_t a23 = max(__float_as_uint(r2) & 0x7fffffffu, __float_as_uint(r3) & 0x7fffffffu);
    const uint32_t a = max(a01, a23);
    amax_bits = max(amax_bits, a);
    const float y0 = r0 * scale_d, y1 = r1 * scale_d, y2 = r2 * scale_d, y3 = r3 * scale_d;
    uint32_t w = cvt4<F>(sat<F>(y0), sat<F>(y1), sat<F>(y2), sat<F>(y3));
    if (slow || __any(a > kInfBits)) {
        w = patch_nan(w, 0, y0);
        w = patch_nan(w, 1, y1);
        w = patch_nan(w, 2, y2);
        w = patch_nan(w, 3, y3);
    }
    return w;
}

// 4 x 4 byte transpose inside every quad of lanes: lane 4 a + k receives byte k of the words of lanes
// 4 a .. 4 a + 3, in lane order from the low byte up.
__device__ __forceinline__ uint32_t quad_transpose_bytes(uint32_t w, int lane) {
    const uint32_t x0 = (uint32_t)__builtin_amdgcn_mov_dpp((int)w, 0x00, 0xf, 0xf, true);   // quad_perm [0,0,0,0]
    const uint32_t x1 = (uint32_t)__builtin_amdgcn_mov_dpp((int)w, 0x55, 0xf, 0xf, true);   // [1,1,1,1]
    const uint32_t x2 = (uint32_t)__builtin_amdgcn_mov_dpp((int)w, 0xaa, 0xf, 0xf, true);   // [2,2,2,2]
    const uint32_t x3 = (uint32_t)__builtin_amdgcn_mov_dpp((int)w, 0xff, 0xf, 0xf, true);   // [3,3,3,3]
    const uint32_t k = lane & 3;
    const uint32_t sel = k | ((4u + k) << 8);   // V_PERM_B32: selector values 0-3 pick bytes of the second source, 4-7 of the first
    const uint32_t t01 = __builtin_amdgcn_perm(x1, x0, sel);
    const uint32_t t23 = __builtin_amdgcn_perm(x3, x2, sel);
    return __builtin_amdgcn_perm(t23, t01, 0x05040100u);
}

// a word of 4 bytes to dst, whole if it may be (`vec`: dst + offsets are 4-byte aligned), else the bytes below `count`
__device__ __forceinline__ void store_bytes4(uint8_t* dst, uint32_t w, bool vec, int count) {
    if (vec && count >= 4) {
        *reinterpret_cast<uint32_t*>(dst) = w;
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (e < count) dst[e] = (uint8_t)(w >> (8 * e));
    }
}

// one wave's share of max|r| into the launch's slots (slots of different workgroups sit on different lines)
__device__ __forceinline__ void publish_amax(uint32_t lane_bits, Workspace* ws) {
    if (!ws) return;
    const uint32_t wm = wave_max_u32(lane_bits);
    if ((threadIdx.x & 63) == 0 && wm != 0u)
        __hip_atomic_fetch_max(&ws->slot[blockIdx.x % kMaxSlots].bits, wm, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// fp8 epilogue of one wave for 32 x 32 accumulator blocks (layout as store_wave_tile); returns the lane's max|r| bits
template <int F, int MI, int NJ>
__device__ __forceinline__ uint32_t store_wave_tile_fp8(const v16f (&acc)[MI][NJ], uint8_t* __restrict__ D,
                                                        uint8_t* __restrict__ Dt, float alpha, float scale_d, bool slow,
                                                        int M, int N, int m_base, int n_base, int lane) {
    uint32_t amax = 0;
    const bool d_vec = (N & 3) == 0;   // rows of D start 4-byte aligned (the launcher checks D itself)
    const bool t_vec = (M & 3) == 0 && (reinterpret_cast<uintptr_t>(Dt) & 3) == 0;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int m = m_base + i * 32 + (lane & 31);
        const int mq = m & ~3;   // first row of this lane's quad
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n_base + j * 32 + g * 8 + (lane >> 5) * 4;
                const uint32_t w = quant4<F>(acc[i][j][g * 4 + 0] * alpha, acc[i][j][g * 4 + 1] * alpha,
                                             acc[i][j][g * 4 + 2] * alpha, acc[i][j][g * 4 + 3] * alpha, scale_d, slow, amax);
                if (m < M && n < N) store_bytes4(D + (int64_t)m * N + n, w, d_vec, N - n);
                if (Dt) {   // uniform
                    const uint32_t t = quad_transpose_bytes(w, lane);
                    const int nt = n + (lane & 3);
                    if (nt < N && mq < M) store_bytes4(Dt + (int64_t)nt * M + mq, t, t_vec, M - mq);
                }
            }
        }
    }
    return amax;
}

}  // namespace ntfp8
