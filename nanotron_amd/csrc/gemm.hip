// FP8 GEMM for gfx950:  D[M,N] (+)= (A[M,K] . B[N,K]^T) * (1/scale_a)(1/scale_b)
//
// Both operands are contiguous along K (the only form the reference issues).  fp32 accumulation on
// the matrix cores with V_MFMA_F32_32X32X64_F8F6F4 (e4m3 / e5m2 selectable per operand), operand
// tiles staged in XOR-swizzled LDS, descale + one rounding in the epilogue.
//
// Two kernels:
//   gemm_nt_big_kernel    256 x 256 x 128 tiles, 8 waves, direct global->LDS buffer loads, two LDS
//                         stages, and two staggered groups of four waves ("ping-pong"): while one
//                         group issues its MFMAs the other reads fragments from LDS and queues the
//                         next tile's loads.  Used for every shape with at least one full-ish tile.
//   gemm_nt_kernel        128 x 128 x 128 tiles, 4 waves, loads through registers; small shapes and
//                         operands beyond the 2 GiB reach of a buffer descriptor's 32-bit offsets.
//   gemm_nt_naive_kernel  any K / alignment, one output per thread.
#include "common.h"

namespace ntfp8 {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr;

constexpr int kBK = 128;     // bytes of K per LDS stage
constexpr int kGroupM = 8;   // tile-order grouping for L2 reuse
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

// Device-only builtins live in __device__ helpers: written directly inside a __global__ template they
// are non-dependent expressions that the host pass cannot resolve.
__device__ __forceinline__ void wg_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}
__device__ __forceinline__ void mfma_priority(bool high) {
    if (high) __builtin_amdgcn_s_setprio(1);
    else __builtin_amdgcn_s_setprio(0);
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
                            w[2 * h] = (uint32_t)OutT<DT>::cvt(acc[i][j][g * 4 + 0] * alpha) |
                                       ((uint32_t)OutT<DT>::cvt(acc[i][j][g * 4 + 1] * alpha) << 16);
                            w[2 * h + 1] = (uint32_t)OutT<DT>::cvt(acc[i][j][g * 4 + 2] * alpha) |
                                           ((uint32_t)OutT<DT>::cvt(acc[i][j][g * 4 + 3] * alpha) << 16);
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

// ---------------------------------------------------------------------------------------------
// 256 x 256 x 128, 8 waves in two staggered groups.
constexpr int kBigM = 256, kBigN = 256;
constexpr int kBigWaves = 8, kBigThreads = kBigWaves * 64;
constexpr int kBigWGN = 2;                 // waves along N: each wave owns 64 (M) x 128 (N)
constexpr int kBigWTM = 64, kBigWTN = 128;
constexpr int kBigMI = kBigWTM / 32, kBigNJ = kBigWTN / 32;
constexpr int kBigLoads = kBigM / 8 / kBigWaves;  // 1 KB wave-level loads per operand per stage per wave

template <int FA, int FB, int DT, bool kAcc>
__global__ __launch_bounds__(kBigThreads) void gemm_nt_big_kernel(const uint8_t* __restrict__ A,
                                                                  const uint8_t* __restrict__ B, void* __restrict__ Dv,
                                                                  const float* __restrict__ scale_a,
                                                                  const float* __restrict__ scale_b, int M, int N, int K,
                                                                  int tiles_m, int tiles_n) {
    __shared__ __attribute__((aligned(1024))) uint8_t sA[2][kBigM * kBK];
    __shared__ __attribute__((aligned(1024))) uint8_t sB[2][kBigN * kBK];

    int pid_m, pid_n;
    tile_of_block(tiles_m, tiles_n, pid_m, pid_n);
    const int m0 = pid_m * kBigM, n0 = pid_n * kBigN;

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int grp = wave >> 2;  // waves w and w + 4 share a SIMD: one from each group
    const int wm = (wave / kBigWGN) * kBigWTM, wn = (wave % kBigWGN) * kBigWTN;

    const __amdgpu_buffer_rsrc_t ra = make_rsrc(A, (uint32_t)((int64_t)M * K));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(B, (uint32_t)((int64_t)N * K));

    // One wave-level load fills 8 tile rows (1 KB of LDS, lane i at byte 16 i).  The lane that lands on
    // chunk position p of row r fetches global chunk p ^ swz(r), which gives the swizzled layout.
    uint32_t a_off[kBigLoads], b_off[kBigLoads];
    int ld_kc[kBigLoads];
#pragma unroll
    for (int i = 0; i < kBigLoads; ++i) {
        const int row = (wave + kBigWaves * i) * 8 + (lane >> 3);
        ld_kc[i] = ((lane & 7) ^ swz(row)) << 4;
        a_off[i] = (uint32_t)(m0 + row) * (uint32_t)K + ld_kc[i];   // rows >= M fall past the descriptor: zeros
        b_off[i] = (uint32_t)(n0 + row) * (uint32_t)K + ld_kc[i];
    }

    v16f acc[kBigMI][kBigNJ];
#pragma unroll
    for (int i = 0; i < kBigMI; ++i)
#pragma unroll
        for (int j = 0; j < kBigNJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const int KT = (K + kBK - 1) / kBK;
    const bool ktail = (K % kBK) != 0;
    auto issue = [&](int s, int kt) {
        const int k0 = kt * kBK;
        const bool tail = ktail && kt == KT - 1;  // chunks at k >= K must read as zero, not as the next row
#pragma unroll
        for (int i = 0; i < kBigLoads; ++i) {
            const bool dead = tail && k0 + ld_kc[i] >= K;
            lds_load16(ra, (lds_ptr)(uintptr_t)&sA[s][(wave + kBigWaves * i) * 1024], dead ? 0xfffffff0u : a_off[i], k0);
            lds_load16(rb, (lds_ptr)(uintptr_t)&sB[s][(wave + kBigWaves * i) * 1024], dead ? 0xfffffff0u : b_off[i], k0);
        }
    };

    const int frow = lane & 31;      // fragment row within a 32-row block
    const int fk = (lane >> 5) * 2;  // first of the lane's two 16-byte chunks within a 64-byte k-step
    v8i fa[kBigMI], fb[kBigNJ];
    auto read_frags = [&](int s, int ks) {
#pragma unroll
        for (int i = 0; i < kBigMI; ++i) {
            const int row = wm + i * 32 + frow;
            const v4i x0 = *reinterpret_cast<const v4i*>(&sA[s][lds_off(row, ks * 4 + fk)]);
            const v4i x1 = *reinterpret_cast<const v4i*>(&sA[s][lds_off(row, ks * 4 + fk + 1)]);
            fa[i] = (v8i){x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
        }
#pragma unroll
        for (int j = 0; j < kBigNJ; ++j) {
            const int row = wn + j * 32 + frow;
            const v4i x0 = *reinterpret_cast<const v4i*>(&sB[s][lds_off(row, ks * 4 + fk)]);
            const v4i x1 = *reinterpret_cast<const v4i*>(&sB[s][lds_off(row, ks * 4 + fk + 1)]);
            fb[j] = (v8i){x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
        }
    };
    auto mma = [&]() {
        mfma_priority(true);
#pragma unroll
        for (int i = 0; i < kBigMI; ++i)
#pragma unroll
            for (int j = 0; j < kBigNJ; ++j) acc[i][j] = mfma_32x32x64<FA, FB>(fb[j], fa[i], acc[i][j]);
        mfma_priority(false);
    };

    // Phases alternate "memory" (LDS fragment reads, and once per tile the next tile's global->LDS
    // loads) and "compute" (8 MFMAs), separated by workgroup barriers.  Group 1 takes one extra barrier
    // up front, so it runs one phase behind group 0: the matrix pipe of every SIMD always has one wave
    // in its compute phase while the other wave of that SIMD is in its memory phase.  Every wave
    // executes the same number of barriers.
    //   tile kt lives in stage kt & 1; its loads are issued in the first memory phase of tile kt - 1,
    //   after every wave has finished reading tile kt - 2 from that stage, and each wave waits for its
    //   own loads before the barrier that precedes the first read of tile kt.
    issue(0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    wg_barrier();
    if (grp == 1) wg_barrier();
    for (int kt = 0; kt < KT; ++kt) {
        const int s = kt & 1;
        read_frags(s, 0);
        if (kt + 1 < KT) issue(s ^ 1, kt + 1);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wg_barrier();
        mma();
        wg_barrier();
        read_frags(s, 1);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (grp == 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        wg_barrier();
        mma();
        if (grp == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        wg_barrier();
    }
    if (grp == 0) wg_barrier();

    const float alpha = (1.0f / *scale_a) * (1.0f / *scale_b);
    store_wave_tile<DT, kAcc, kBigMI, kBigNJ>(acc, Dv, alpha, M, N, m0 + wm, n0 + wn, lane);
}

// ---------------------------------------------------------------------------------------------
// 128 x 128 x 128, 4 waves (2 x 2, each 64 x 64), loads staged through registers.
constexpr int kBM = 128, kBN = 128;
constexpr int kGemmThreads = 256;

template <int FA, int FB, int DT, bool kAcc>
__global__ __launch_bounds__(kGemmThreads) void gemm_nt_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                               void* __restrict__ Dv, const float* __restrict__ scale_a,
                                                               const float* __restrict__ scale_b, int M, int N, int K,
                                                               int tiles_m, int tiles_n) {
    __shared__ __attribute__((aligned(16))) uint8_t sA[kBM * kBK];
    __shared__ __attribute__((aligned(16))) uint8_t sB[kBN * kBK];

    int pid_m, pid_n;
    tile_of_block(tiles_m, tiles_n, pid_m, pid_n);
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

    const int frow = lane & 31;
    const int fk = (lane >> 5) * 2;

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
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = mfma_32x32x64<FA, FB>(fb[j], fa[i], acc[i][j]);
        }
    }

    const float alpha = (1.0f / *scale_a) * (1.0f / *scale_b);
    store_wave_tile<DT, kAcc, 2, 2>(acc, Dv, alpha, M, N, m0 + wm, n0 + wn, lane);
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

// ---------------------------------------------------------------------------------------------
enum GemmPath { kPathNaive = 0, kPathSmall = 1, kPathBig = 2 };

template <int FA, int FB, int DT, bool kAcc>
static int launch_gemm(const void* A, const float* sa, const void* B, const float* sb, void* D, int M, int N, int K,
                       int path, hipStream_t st) {
    const uint8_t* a = static_cast<const uint8_t*>(A);
    const uint8_t* b = static_cast<const uint8_t*>(B);
    if (path == kPathBig) {
        const int tm = (M + kBigM - 1) / kBigM, tn = (N + kBigN - 1) / kBigN;
        hipLaunchKernelGGL((gemm_nt_big_kernel<FA, FB, DT, kAcc>), dim3(tm * tn), dim3(kBigThreads), 0, st, a, b, D, sa,
                           sb, M, N, K, tm, tn);
    } else if (path == kPathSmall) {
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
                        int N, int K, int accumulate, int path, hipStream_t st) {
    if (d_dtype == NTFP8_F32)
        return accumulate ? launch_gemm<FA, FB, NTFP8_F32, true>(A, sa, B, sb, D, M, N, K, path, st)
                          : launch_gemm<FA, FB, NTFP8_F32, false>(A, sa, B, sb, D, M, N, K, path, st);
    if (d_dtype == NTFP8_BF16) return launch_gemm<FA, FB, NTFP8_BF16, false>(A, sa, B, sb, D, M, N, K, path, st);
    return launch_gemm<FA, FB, NTFP8_F16, false>(A, sa, B, sb, D, M, N, K, path, st);
}

int run_gemm(const void* A, int fmt_a, const float* sa, const void* B, int fmt_b, const float* sb, void* D, int d_dtype,
             int M, int N, int K, int accumulate, hipStream_t st) {
    const bool aligned16 = (K % 16 == 0) &&
                           ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 &&
                           (reinterpret_cast<uintptr_t>(D) & 15) == 0;
    int path = kPathNaive;
    if (aligned16) {
        // the big kernel addresses its operands with 32-bit buffer offsets and wants enough tiles to matter
        const bool fits32 = (int64_t)(M + kBigM) * K < (1LL << 31) && (int64_t)(N + kBigN) * K < (1LL << 31);
        const bool worth = M > kBM && N > kBN && K >= 2 * kBK;
        path = (fits32 && worth) ? kPathBig : kPathSmall;
    }
    if (fmt_a == kE4M3)
        return fmt_b == kE4M3 ? dispatch_out<kE4M3, kE4M3>(A, sa, B, sb, D, d_dtype, M, N, K, accumulate, path, st)
                              : dispatch_out<kE4M3, kE5M2>(A, sa, B, sb, D, d_dtype, M, N, K, accumulate, path, st);
    return fmt_b == kE4M3 ? dispatch_out<kE5M2, kE4M3>(A, sa, B, sb, D, d_dtype, M, N, K, accumulate, path, st)
                          : dispatch_out<kE5M2, kE5M2>(A, sa, B, sb, D, d_dtype, M, N, K, accumulate, path, st);
}

}  // namespace ntfp8
