// FP8 GEMM for gfx950:  D[M,N] (+)= (A[M,K] . B[N,K]^T) * (1/scale_a)(1/scale_b)
//
// Both operands are contiguous along K (the only form the reference issues); the big kernel also takes B as
// its transpose, a [K, N] tensor.  fp32 accumulation on the matrix cores (e4m3 / e5m2 selectable per
// operand), operand tiles staged in XOR-swizzled LDS, descale + one rounding in the epilogue to fp32
// (optionally added to what is there), bf16, fp16 or fp8 bytes.
//
// Three kernels:
//   gemm_nt_big_kernel    (gemm_big.h) 256 x 256 x 128 tiles, 4 waves of 128 x 128 with 16x16x128 MFMAs,
//                         loads staged through registers, two LDS stages, one barrier per K-tile.  The
//                         partial last round of tiles over the CUs is cut into 128-row half tiles.
//   gemm_nt_kernel        128 x 128 x 128 tiles, 4 waves, loads through registers; small shapes and
//                         operands beyond the 2 GiB reach of a buffer descriptor's 32-bit offsets.
//   gemm_nt_naive_kernel  any K / alignment, one output per thread.
#include "gemm_common.h"
#include "gemm_big.h"

namespace ntfp8 {

// ---------------------------------------------------------------------------------------------
// 128 x 128 x 128, 4 waves (2 x 2, each 64 x 64), loads staged through registers.
constexpr int kBM = 128, kBN = 128;
constexpr int kGemmThreads = 256;

template <int FA, int FB, int DT, bool kAcc>
__global__ __launch_bounds__(kGemmThreads) void gemm_nt_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                               void* __restrict__ Dv, const float* __restrict__ scale_a,
                                                               const float* __restrict__ scale_b, int M, int N, int K,
                                                               int tiles_m, int tiles_n, Fp8Out fp8, GemmExtras ex) {
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

    float alpha = descale_factor(scale_a, scale_b, ex.scale_inv);
    if (ex.bias) {   // uniform
        add_bias32<2, 2>(acc, alpha, ex.bias, ex.bias_dtype, N, n0 + wn, lane);
        alpha = 1.0f;
    }
    if constexpr (DT == NTFP8_OUT_E4M3 || DT == NTFP8_OUT_E5M2) {
        constexpr int F = DT == NTFP8_OUT_E4M3 ? kE4M3 : kE5M2;
        const float scale_d = *fp8.scale;
        const uint32_t amax = store_wave_tile_fp8<F, 2, 2>(acc, static_cast<uint8_t*>(Dv), fp8.Dt, alpha, scale_d,
                                                           scale_is_degenerate(scale_d), M, N, m0 + wm, n0 + wn, lane);
        publish_amax(amax, fp8.ws);
    } else {
        store_wave_tile<DT, kAcc, 2, 2>(acc, Dv, alpha, M, N, m0 + wm, n0 + wn, lane);
    }
}

// Any K / alignment: one output element per thread, table-free decode through the hardware
// fp8 -> fp32 conversion.  Only meant for tiny or odd shapes.
template <int FA, int FB, int DT, bool kAcc>
__global__ void gemm_nt_naive_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, void* __restrict__ Dv,
                                     const float* __restrict__ scale_a, const float* __restrict__ scale_b, int M, int N,
                                     int K, Fp8Out fp8, GemmExtras ex) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const bool live = idx < (int64_t)M * N;
    if (!live && !(DT == NTFP8_OUT_E4M3 || DT == NTFP8_OUT_E5M2)) return;
    const int m = live ? (int)(idx / N) : 0, n = live ? (int)(idx % N) : 0;
    float acc = 0.0f;
    for (int k = 0; live && k < K; ++k) {
        const float a = FA == kE4M3 ? __builtin_amdgcn_cvt_f32_fp8((int)A[(int64_t)m * K + k], 0)
                                    : __builtin_amdgcn_cvt_f32_bf8((int)A[(int64_t)m * K + k], 0);
        const float b = FB == kE4M3 ? __builtin_amdgcn_cvt_f32_fp8((int)B[(int64_t)n * K + k], 0)
                                    : __builtin_amdgcn_cvt_f32_bf8((int)B[(int64_t)n * K + k], 0);
        acc += a * b;
    }
    float v = acc * descale_factor(scale_a, scale_b, ex.scale_inv);
    if (ex.bias && live) v = v + bias_at(ex.bias, ex.bias_dtype, n);
    if constexpr (DT == NTFP8_OUT_E4M3 || DT == NTFP8_OUT_E5M2) {
        // whole waves get here (the amax reduction runs over all 64 lanes); lanes past the end hold zeros
        constexpr int F = DT == NTFP8_OUT_E4M3 ? kE4M3 : kE5M2;
        uint32_t amax = 0;
        const uint32_t w = quant4<F>(v, 0.0f, 0.0f, 0.0f, *fp8.scale, true, amax);
        if (live) {
            static_cast<uint8_t*>(Dv)[idx] = (uint8_t)w;
            if (fp8.Dt) fp8.Dt[(int64_t)n * M + m] = (uint8_t)w;
        }
        publish_amax(amax, fp8.ws);
    } else {
        typedef typename OutT<DT>::type O;
        O* D = static_cast<O*>(Dv);
        if constexpr (DT == NTFP8_F32) {
            if constexpr (kAcc) v = v + D[idx];
            D[idx] = v;
        } else {
            D[idx] = OutT<DT>::cvt(v);
        }
    }
}

// ---------------------------------------------------------------------------------------------
enum GemmPath { kPathNone = -1, kPathNaive = 0, kPathSmall = 1, kPathBig = 2 };

// which kernel serves a problem
static int path_of(const GemmDesc& g) {
    const bool aligned16 = (g.K % 16 == 0) &&
                           ((reinterpret_cast<uintptr_t>(g.A) | reinterpret_cast<uintptr_t>(g.B)) & 15) == 0 &&
                           (reinterpret_cast<uintptr_t>(g.D) & 15) == 0;
    if (!aligned16) return g.tb ? kPathNone : kPathNaive;
    // the big kernel addresses its operands with 32-bit buffer offsets and wants enough tiles to matter
    const bool fits32 = (int64_t)(g.M + 256) * g.K < (1LL << 31) && (int64_t)(g.N + kBigN) * g.K < (1LL << 31);
    const bool worth = g.M > kBM && g.N > kBN && g.K >= 2 * kBK;
    // its fp8 epilogue stores whole words through 32-bit buffer offsets
    const bool fp8_ok = !is_fp8_out(g.d_dtype) ||
                        (g.N % 16 == 0 && g.M % 4 == 0 && (int64_t)g.M * g.N < (1LL << 32) - 16 &&
                         (reinterpret_cast<uintptr_t>(g.Dt) & 15) == 0);
    // an operand given as its transpose, [K, N] or [K, M], is loaded in 16-byte pieces of its rows; only the big
    // kernel reads it, and a transposed A only next to a transposed B (the wgrad form)
    if (g.ta && (!g.tb || g.M % 16 != 0)) return kPathNone;
    if (g.tb) return (g.N % 16 == 0 && fits32 && worth && fp8_ok) ? kPathBig : kPathNone;
    return (fits32 && worth && fp8_ok) ? kPathBig : kPathSmall;
}

// One launch (plus one for the half-tile tail) of the big kernel over up to kBigMaxProblems problems of the
// same operand formats.  Tiles are listed problem by problem, longest K first: the long tiles start together and
// the shorter ones fill the rounds behind them.
template <int FA, int FB, bool kFp8Out, bool kBT>
static int launch_big(const GemmDesc* const* g, int n, hipStream_t st) {
    int order[kBigMaxProblems];
    for (int i = 0; i < n; ++i) order[i] = i;
    for (int i = 1; i < n; ++i)   // insertion sort, stable, K descending
        for (int j = i; j > 0 && g[order[j]]->K > g[order[j - 1]]->K; --j) {
            const int t = order[j];
            order[j] = order[j - 1];
            order[j - 1] = t;
        }
    BigLaunch L = {};
    L.count = n;
    int tiles = 0;
    for (int i = 0; i < n; ++i) {
        const GemmDesc& d = *g[order[i]];
        BigProblem& p = L.p[i];
        p.A = static_cast<const uint8_t*>(d.A);
        p.B = static_cast<const uint8_t*>(d.B);
        p.D = d.D;
        p.scale_a = d.sa;
        p.scale_b = d.sb;
        p.M = d.M;
        p.N = d.N;
        p.K = d.K;
        p.tiles_m = (d.M + 255) / 256;
        p.tiles_n = (d.N + kBigN - 1) / kBigN;
        p.tile_begin = tiles;
        p.d_dtype = d.d_dtype;
        p.accumulate = d.accumulate;
        p.fp8 = Fp8Out{d.sd, static_cast<uint8_t*>(d.Dt), static_cast<Workspace*>(d.ws)};
        p.ex = GemmExtras{d.bias, d.bias_dtype, d.scale_inv};
        p.at = d.ta;
        tiles += p.tiles_m * p.tiles_n;
    }
    const int rem = tiles % cu_count();
    L.tail_tiles = (rem != 0 && 2 * rem <= cu_count()) ? rem : 0;
    L.full_blocks = tiles - L.tail_tiles;
    L.round_size = cu_count();
    (void)hipGetLastError();   // an error left behind by an unrelated earlier call is not this launch's
    if (L.full_blocks > 0)
        hipLaunchKernelGGL((gemm_nt_big_kernel<FA, FB, 8, kFp8Out, kBT>), dim3(L.full_blocks), dim3(kBigThreads), 0, st, L);
    if (L.tail_tiles > 0)
        hipLaunchKernelGGL((gemm_nt_big_kernel<FA, FB, 4, kFp8Out, kBT>), dim3(2 * L.tail_tiles), dim3(kBigThreads), 0, st, L);
    return hipGetLastError() == hipSuccess ? NTFP8_OK : NTFP8_ERR_LAUNCH;
}

template <int FA, int FB, int DT, bool kAcc>
static int launch_small(const GemmDesc& g, int path, hipStream_t st) {
    const uint8_t* a = static_cast<const uint8_t*>(g.A);
    const uint8_t* b = static_cast<const uint8_t*>(g.B);
    const Fp8Out fp8 = {g.sd, static_cast<uint8_t*>(g.Dt), static_cast<Workspace*>(g.ws)};
    const GemmExtras ex = {g.bias, g.bias_dtype, g.scale_inv};
    (void)hipGetLastError();   // an error left behind by an unrelated earlier call is not this launch's
    if (path == kPathSmall) {
        const int tm = (g.M + kBM - 1) / kBM, tn = (g.N + kBN - 1) / kBN;
        hipLaunchKernelGGL((gemm_nt_kernel<FA, FB, DT, kAcc>), dim3(tm * tn), dim3(kGemmThreads), 0, st, a, b, g.D, g.sa,
                           g.sb, g.M, g.N, g.K, tm, tn, fp8, ex);
    } else {
        const int64_t blocks = ((int64_t)g.M * g.N + 255) / 256;
        hipLaunchKernelGGL((gemm_nt_naive_kernel<FA, FB, DT, kAcc>), dim3((int)blocks), dim3(256), 0, st, a, b, g.D, g.sa,
                           g.sb, g.M, g.N, g.K, fp8, ex);
    }
    return hipGetLastError() == hipSuccess ? NTFP8_OK : NTFP8_ERR_LAUNCH;
}

template <int FA, int FB>
static int dispatch_fmt(const GemmDesc* const* g, int n, int path, hipStream_t st) {
    if (path == kPathNone) return NTFP8_ERR_UNSUPPORTED;
    if (path == kPathBig) {
        if (g[0]->tb)
            return is_fp8_out(g[0]->d_dtype) ? launch_big<FA, FB, true, true>(g, n, st) : launch_big<FA, FB, false, true>(g, n, st);
        return is_fp8_out(g[0]->d_dtype) ? launch_big<FA, FB, true, false>(g, n, st) : launch_big<FA, FB, false, false>(g, n, st);
    }
    const GemmDesc& d = *g[0];   // the small kernels take one problem
    if (d.d_dtype == NTFP8_F32)
        return d.accumulate ? launch_small<FA, FB, NTFP8_F32, true>(d, path, st)
                            : launch_small<FA, FB, NTFP8_F32, false>(d, path, st);
    if (d.d_dtype == NTFP8_BF16) return launch_small<FA, FB, NTFP8_BF16, false>(d, path, st);
    if (d.d_dtype == NTFP8_OUT_E4M3) return launch_small<FA, FB, NTFP8_OUT_E4M3, false>(d, path, st);
    if (d.d_dtype == NTFP8_OUT_E5M2) return launch_small<FA, FB, NTFP8_OUT_E5M2, false>(d, path, st);
    return launch_small<FA, FB, NTFP8_F16, false>(d, path, st);
}

static int dispatch(const GemmDesc* const* g, int n, int path, hipStream_t st) {
    const int fa = g[0]->fmt_a, fb = g[0]->fmt_b;
#ifdef NTFP8_PROFILE_NARROW
    // experiment builds of the profiling library carry one instantiation only: e4m3 x e4m3, K-contiguous operands,
    // 16-bit or fp32 output (what the loop experiments launch); everything else is refused
    if (fa != kE4M3 || fb != kE4M3 || path != kPathBig || g[0]->tb || is_fp8_out(g[0]->d_dtype)) return NTFP8_ERR_UNSUPPORTED;
    return launch_big<kE4M3, kE4M3, false, false>(g, n, st);
#else
    if (fa == kE4M3) return fb == kE4M3 ? dispatch_fmt<kE4M3, kE4M3>(g, n, path, st) : dispatch_fmt<kE4M3, kE5M2>(g, n, path, st);
    return fb == kE4M3 ? dispatch_fmt<kE5M2, kE4M3>(g, n, path, st) : dispatch_fmt<kE5M2, kE5M2>(g, n, path, st);
#endif
}

int run_gemm(const GemmDesc& g, hipStream_t st) {
    const GemmDesc* one[1] = {&g};
    return dispatch(one, 1, path_of(g), st);
}

// Independent problems (no output of one is an operand of another).  Problems that qualify for the big kernel
// and share their operand formats go out together, up to kBigMaxProblems per launch; the rest one by one.
int run_gemm_batch(const GemmDesc* g, int n, hipStream_t st) {
    bool done[64] = {false};
    if (n > 64) return NTFP8_ERR_SIZE;
    // a problem no kernel serves fails the whole call before anything is launched
    for (int i = 0; i < n; ++i)
        if (path_of(g[i]) == kPathNone) return NTFP8_ERR_UNSUPPORTED;
    for (int i = 0; i < n; ++i) {
        if (done[i]) continue;
        const GemmDesc* group[kBigMaxProblems];
        int cnt = 0;
        const int path = path_of(g[i]);
        group[cnt++] = &g[i];
        done[i] = true;
        if (path == kPathBig) {
            for (int j = i + 1; j < n && cnt < kBigMaxProblems; ++j)
                if (!done[j] && g[j].fmt_a == g[i].fmt_a && g[j].fmt_b == g[i].fmt_b && path_of(g[j]) == kPathBig &&
                    is_fp8_out(g[j].d_dtype) == is_fp8_out(g[i].d_dtype) && g[j].tb == g[i].tb) {
                    group[cnt++] = &g[j];
                    done[j] = true;
                }
        }
        const int rc = dispatch(group, cnt, path, st);
        if (rc != NTFP8_OK) return rc;
    }
    return NTFP8_OK;
}

}  // namespace ntfp8

#ifdef NTFP8_STAMPS
// Profiling build only: copies the per-workgroup time stamps of the last gemm_nt_big_kernel launches to host memory
// (8 x uint64 per workgroup index, see gemm_big.h).  Synchronises the device.
extern "C" __attribute__((visibility("default"))) int ntfp8_debug_stamps(void* dst, size_t bytes) {
    if (!dst || bytes > sizeof(unsigned long long) * ntfp8::kStampSlots * 8) return dst ? NTFP8_ERR_SIZE : NTFP8_ERR_NULL;
    return hipMemcpyFromSymbol(dst, HIP_SYMBOL(ntfp8::g_stamps), bytes) == hipSuccess ? NTFP8_OK : NTFP8_ERR_LAUNCH;
}
extern "C" __attribute__((visibility("default"))) int ntfp8_debug_set_tile_order(int plain) {
    const int v = plain ? 1 : 0;
    return hipMemcpyToSymbol(HIP_SYMBOL(ntfp8::g_plain_tile_order), &v, sizeof(v)) == hipSuccess ? NTFP8_OK : NTFP8_ERR_LAUNCH;
}
#endif
