// FP8 GEMM for gfx950:  D[M,N] (+)= (A[M,K] . B[N,K]^T) * (1/scale_a)(1/scale_b)
// Both operands are contiguous along K (the only form the reference issues).  fp32 accumulation on
// the matrix cores with V_MFMA_F32_32X32X64_F8F6F4 (e4m3 / e5m2 selectable per operand), operands
// staged through XOR-swizzled LDS tiles, descale + one rounding in the epilogue.
#include "common.h"

namespace ntfp8 {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kBM = 128, kBN = 128, kBK = 128;  // block tile; kBK bytes of K per stage
constexpr int kGemmThreads = 256;               // 4 waves, 2 x 2, each 64 x 64
constexpr int kGroupM = 8;                      // tile-order grouping for L2 reuse

// 16-byte chunk `kc` (0..7) of tile row `row`, swizzled so that the 16 lanes of a 128-bit LDS access
// that read the same chunk of 16 consecutive rows touch 16 distinct 16-byte bank groups.
__device__ __forceinline__ int lds_off(int row, int kc) { return row * kBK + ((kc ^ ((row >> 1) & 7)) << 4); }

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float v) {
    const uint32_t u = __float_as_uint(v);
    if ((u & 0x7fffffffu) > kInfBits) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

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
};
template <>
struct OutT<NTFP8_F16> {
    typedef uint16_t type;
    __device__ static __forceinline__ uint16_t cvt(float v) {
        asm volatile("" : "+v"(v));  // no folding of the descale multiply into a mixed-precision fma (-0 would become +0)
        return __half_as_ushort(__float2half_rn(v));
    }
};

template <int FA, int FB, int DT, bool kAcc>
__global__ __launch_bounds__(kGemmThreads) void gemm_nt_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                               void* __restrict__ Dv, const float* __restrict__ scale_a,
                                                               const float* __restrict__ scale_b, int M, int N, int K,
                                                               int tiles_m, int tiles_n) {
    __shared__ __attribute__((aligned(16))) uint8_t sA[kBM * kBK];
    __shared__ __attribute__((aligned(16))) uint8_t sB[kBN * kBK];

    // tile order: consecutive ids sweep kGroupM row-tiles before moving along N
    const int pid = blockIdx.x;
    const int in_group = kGroupM * tiles_n;
    const int group = pid / in_group;
    const int first_m = group * kGroupM;
    const int gsz = min(tiles_m - first_m, kGroupM);
    const int pid_m = first_m + (pid % in_group) % gsz;
    const int pid_n = (pid % in_group) / gsz;
    const int m0 = pid_m * kBM, n0 = pid_n * kBN;

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

    // global -> LDS assignment: 1024 16-byte chunks per operand tile, 4 per thread
    int ld_row[4], ld_kc[4];
    const uint8_t* a_ptr[4];
    const uint8_t* b_ptr[4];
    bool a_ok[4], b_ok[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = t + kGemmThreads * i;
        ld_row[i] = c >> 3;
        ld_kc[i] = c & 7;
        a_ok[i] = m0 + ld_row[i] < M;
        b_ok[i] = n0 + ld_row[i] < N;
        a_ptr[i] = A + (int64_t)(a_ok[i] ? m0 + ld_row[i] : 0) * K + ld_kc[i] * 16;
        b_ptr[i] = B + (int64_t)(b_ok[i] ? n0 + ld_row[i] : 0) * K + ld_kc[i] * 16;
    }

    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    v4i ra[4], rb[4];
    const v4i zero = {0, 0, 0, 0};
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool kin = k0 + ld_kc[i] * 16 < K;
            ra[i] = (a_ok[i] && kin) ? *reinterpret_cast<const v4i*>(a_ptr[i] + k0) : zero;
            rb[i] = (b_ok[i] && kin) ? *reinterpret_cast<const v4i*>(b_ptr[i] + k0) : zero;
        }
    };

    const int frow = lane & 31;        // fragment row within a 32-row block
    const int fk = (lane >> 5) * 2;    // first of the lane's two 16-byte chunks within a 64-byte k-step

    fetch(0);
    for (int k0 = 0; k0 < K; k0 += kBK) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<v4i*>(&sA[lds_off(ld_row[i], ld_kc[i])]) = ra[i];
            *reinterpret_cast<v4i*>(&sB[lds_off(ld_row[i], ld_kc[i])]) = rb[i];
        }
        __syncthreads();
        if (k0 + kBK < K) fetch(k0 + kBK);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            v8i fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int ra_row = wm + i * 32 + frow, rb_row = wn + i * 32 + frow;
                const v4i a0 = *reinterpret_cast<const v4i*>(&sA[lds_off(ra_row, ks * 4 + fk)]);
                const v4i a1 = *reinterpret_cast<const v4i*>(&sA[lds_off(ra_row, ks * 4 + fk + 1)]);
                const v4i b0 = *reinterpret_cast<const v4i*>(&sB[lds_off(rb_row, ks * 4 + fk)]);
                const v4i b1 = *reinterpret_cast<const v4i*>(&sB[lds_off(rb_row, ks * 4 + fk + 1)]);
                fa[i] = (v8i){a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
                fb[i] = (v8i){b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
            }
            // The B-matrix fragment is the MFMA's first source so that the 32x32 result block is
            // indexed [n][m]: each lane then owns 4 consecutive n of one output row m.
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j], fa[i], acc[i][j], FB, FA, 0, 0, 0, 0);
        }
    }

    // epilogue: descale, optional fp32 accumulate, one rounding, store
    typedef typename OutT<DT>::type O;
    O* D = static_cast<O*>(Dv);
    const float alpha = (1.0f / *scale_a) * (1.0f / *scale_b);
    const bool vec_ok = (N & 3) == 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int m = m0 + wm + i * 32 + (lane & 31);
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wn + j * 32 + g * 8 + (lane >> 5) * 4;
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
                        const uint32_t lo = (uint32_t)OutT<DT>::cvt(v[0]) | ((uint32_t)OutT<DT>::cvt(v[1]) << 16);
                        const uint32_t hi = (uint32_t)OutT<DT>::cvt(v[2]) | ((uint32_t)OutT<DT>::cvt(v[3]) << 16);
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

// Any K / alignment: one output element per thread, table-free decode through the hardware
// fp8 -> fp32 conversion.  Only meant for tiny or odd shapes.
template <int FA, int FB, int DT, bool kAcc>
__global__ void gemm_nt_naive_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, void* __restrict__ Dv,
                                     const float* __restrict__ scale_a, const float* __restrict__ scale_b, int M, int N,
                                     int K) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)M * N) return;
    const int m = (int)(idx / N), n = (int)(idx % N);
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) {
        const float a = FA == kE4M3 ? __builtin_amdgcn_cvt_f32_fp8((int)A[(int64_t)m * K + k], 0)
                                    : __builtin_amdgcn_cvt_f32_bf8((int)A[(int64_t)m * K + k], 0);
        const float b = FB == kE4M3 ? __builtin_amdgcn_cvt_f32_fp8((int)B[(int64_t)n * K + k], 0)
                                    : __builtin_amdgcn_cvt_f32_bf8((int)B[(int64_t)n * K + k], 0);
        acc += a * b;
    }
    typedef typename OutT<DT>::type O;
    O* D = static_cast<O*>(Dv);
    float v = acc * ((1.0f / *scale_a) * (1.0f / *scale_b));
    if constexpr (DT == NTFP8_F32) {
        if constexpr (kAcc) v = v + D[idx];
        D[idx] = v;
    } else {
        D[idx] = OutT<DT>::cvt(v);
    }
}

template <int FA, int FB, int DT, bool kAcc>
static int launch_gemm(const void* A, const float* sa, const void* B, const float* sb, void* D, int M, int N, int K,
                       bool fast, hipStream_t st) {
    const uint8_t* a = static_cast<const uint8_t*>(A);
    const uint8_t* b = static_cast<const uint8_t*>(B);
    if (fast) {
        const int tm = (M + kBM - 1) / kBM, tn = (N + kBN - 1) / kBN;
        hipLaunchKernelGGL((gemm_nt_kernel<FA, FB, DT, kAcc>), dim3(tm * tn), dim3(kGemmThreads), 0, st, a, b, D, sa, sb,
                           M, N, K, tm, tn);
    } else {
        const int64_t blocks = ((int64_t)M * N + 255) / 256;
        hipLaunchKernelGGL((gemm_nt_naive_kernel<FA, FB, DT, kAcc>), dim3((int)blocks), dim3(256), 0, st, a, b, D, sa, sb,
                           M, N, K);
    }
    return hipGetLastError() == hipSuccess ? NTFP8_OK : NTFP8_ERR_LAUNCH;
}

template <int FA, int FB>
static int dispatch_out(const void* A, const float* sa, const void* B, const float* sb, void* D, int d_dtype, int M,
                        int N, int K, int accumulate, bool fast, hipStream_t st) {
    if (d_dtype == NTFP8_F32)
        return accumulate ? launch_gemm<FA, FB, NTFP8_F32, true>(A, sa, B, sb, D, M, N, K, fast, st)
                          : launch_gemm<FA, FB, NTFP8_F32, false>(A, sa, B, sb, D, M, N, K, fast, st);
    if (d_dtype == NTFP8_BF16) return launch_gemm<FA, FB, NTFP8_BF16, false>(A, sa, B, sb, D, M, N, K, fast, st);
    return launch_gemm<FA, FB, NTFP8_F16, false>(A, sa, B, sb, D, M, N, K, fast, st);
}

int run_gemm(const void* A, int fmt_a, const float* sa, const void* B, int fmt_b, const float* sb, void* D, int d_dtype,
             int M, int N, int K, int accumulate, hipStream_t st) {
    const bool fast = (K % 16 == 0) && ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 &&
                      (reinterpret_cast<uintptr_t>(D) & 15) == 0;
    if (fmt_a == kE4M3)
        return fmt_b == kE4M3 ? dispatch_out<kE4M3, kE4M3>(A, sa, B, sb, D, d_dtype, M, N, K, accumulate, fast, st)
                              : dispatch_out<kE4M3, kE5M2>(A, sa, B, sb, D, d_dtype, M, N, K, accumulate, fast, st);
    return fmt_b == kE4M3 ? dispatch_out<kE5M2, kE4M3>(A, sa, B, sb, D, d_dtype, M, N, K, accumulate, fast, st)
                          : dispatch_out<kE5M2, kE5M2>(A, sa, B, sb, D, d_dtype, M, N, K, accumulate, fast, st);
}

}  // namespace ntfp8
