// amax reduction, delayed-scaling history roll + scale update, saturating casts to OCP FP8,
// dequantisation and byte transpose for gfx950.  All kernels are HBM-bandwidth bound: one pass
// over the input with 128-bit loads and stores, a wavefront reduction for the amax, one atomic per
// block and a last-block epilogue that finishes the scalar bookkeeping in the same launch.
#include "common.h"

namespace ntfp8 {

constexpr int kThreads = 256;       // dequant / transpose / scalar kernels
constexpr int kFlatThreads = 1024;  // streaming quantise kernel: one block per CU, 16 waves
constexpr int kTileThreads = 256;   // tile (transposing) quantise kernel
constexpr int kVec = 16;  // elements per thread per step: 16 fp8 bytes = one 128-bit store

typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));


// ---------------------------------------------------------------------------------------------
// 16-element loads.  `m16` receives max|x| of the 16 elements as a comparable unsigned pattern in
// the *source* format (fp32 bits for float, 16-bit patterns for half / bf16).
template <typename T>
struct Src;

template <>
struct Src<float> {
    static constexpr int kDtype = NTFP8_F32;
    __device__ static __forceinline__ void load16(const float* p, float (&v)[16], uint32_t& m16) {
        const f4* q = reinterpret_cast<const f4*>(p);
        uint32_t m = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const f4 t = __builtin_nontemporal_load(q + i);
            v[4 * i + 0] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t a = __float_as_uint(v[i]) & 0x7fffffffu;
            m = a > m ? a : m;
        }
        m16 = m;
    }
    __device__ static __forceinline__ float load1(const float* p, uint32_t& m) {
        const float x = *p;
        m = __float_as_uint(x) & 0x7fffffffu;
        return x;
    }
    __device__ static __forceinline__ bool has_nan(uint32_t m) { return m > kInfBits; }
    __device__ static __forceinline__ uint32_t to_f32_bits(uint32_t m) { return m; }
};

template <bool kBf16>
struct Src16 {
    __device__ static __forceinline__ float cvt(uint32_t h) {
        if constexpr (kBf16) return bf16_bits_to_float(h);
        else return half_bits_to_float(h);
    }
    __device__ static __forceinline__ void load16(const uint16_t* p, float (&v)[16], uint32_t& m16) {
        const u4* q = reinterpret_cast<const u4*>(p);
        const u4 a = __builtin_nontemporal_load(q);
        const u4 b = __builtin_nontemporal_load(q + 1);
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        typedef unsigned short us2 __attribute__((ext_vector_type(2)));
        us2 m = {0, 0};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if constexpr (kBf16) {
                v[2 * i] = __uint_as_float(w[i] << 16);
                v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
            } else {
                v[2 * i] = half_bits_to_float(w[i] & 0xffffu);
                v[2 * i + 1] = half_bits_to_float(w[i] >> 16);
            }
            const uint32_t ab = w[i] & 0x7fff7fffu;
            us2 t;
            __builtin_memcpy(&t, &ab, 4);
            m = __builtin_elementwise_max(m, t);
        }
        m16 = m.x > m.y ? m.x : m.y;
    }
    __device__ static __forceinline__ float load1(const uint16_t* p, uint32_t& m) {
        const uint32_t h = *p;
        m = h & 0x7fffu;
        return cvt(h);
    }
    __device__ static __forceinline__ bool has_nan(uint32_t m) { return m > (kBf16 ? 0x7f80u : 0x7c00u); }
    __device__ static __forceinline__ uint32_t to_f32_bits(uint32_t m) { return __float_as_uint(cvt(m)); }
};

struct bf16_tag {};
struct f16_tag {};
template <>
struct Src<bf16_tag> : Src16<true> {
    static constexpr int kDtype = NTFP8_BF16;
    typedef uint16_t elem;
};
template <>
struct Src<f16_tag> : Src16<false> {
    static constexpr int kDtype = NTFP8_F16;
    typedef uint16_t elem;
};
template <typename T>
struct ElemOf {
    typedef uint16_t type;
};
template <>
struct ElemOf<float> {
    typedef float type;
};

// 16 scaled values -> 16 fp8 bytes.  `slow` = this group may contain a NaN (NaN input or a
// degenerate scale): patch the NaN bytes to sign|0x7F.
template <int F>
__device__ __forceinline__ u4 encode16(const float (&v)[16], float scale, bool slow) {
    float y[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) y[i] = v[i] * scale;
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        w[i] = cvt4<F>(sat<F>(y[4 * i]), sat<F>(y[4 * i + 1]), sat<F>(y[4 * i + 2]), sat<F>(y[4 * i + 3]));
    if (slow) {
#pragma unroll
        for (int i = 0; i < 16; ++i) w[i >> 2] = patch_nan(w[i >> 2], i & 3, y[i]);
    }
    return (u4){w[0], w[1], w[2], w[3]};
}

template <int F>
__device__ __forceinline__ uint8_t encode1(float x, float scale) {
    const float y = x * scale;
    uint32_t w = cvt4<F>(sat<F>(y), 0.0f, 0.0f, 0.0f);
    w = patch_nan(w, 0, y);
    return (uint8_t)(w & 0xffu);
}

// ---------------------------------------------------------------------------------------------
// Block reduction of the partial max, publication, and the last-block epilogue.
//
// Inter-block traffic uses relaxed device-scope atomics only (they execute at the level where all
// XCDs agree) and orders them with the wave's own memory counter: the partial max is folded in with
// a returning atomic, the wave waits for it, then takes a ticket.  A release fence here would write
// back the whole L2 once per block, which costs more than the streaming pass itself.
// What the last block's epilogue will read, requested by the first wave of every block while the
// tensor is still streaming: the history entry that moves into this lane's slot and the scale in
// force.  It takes one round trip out of the dependent chain at the end of the kernel.
struct EpiloguePrefetch {
    float hist_prev;  // hist[lane - 1] (lanes 1 .. hist_len-1; histories of up to 64 entries)
    float scale;      // *scale_state; amax-only mode: *old_scale (1.0 if there is none)
};
__device__ __forceinline__ EpiloguePrefetch prefetch_epilogue(const ScalarIO& io, int mode) {
    EpiloguePrefetch p = {0.0f, 1.0f};
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        if (io.hist && io.hist_len <= 64 && lane >= 1 && lane < io.hist_len) p.hist_prev = io.hist[lane - 1];
        if (mode != kModeAmaxOnly) p.scale = *io.scale_state;
        else if (io.old_scale) p.scale = *io.old_scale;
    }
    return p;
}

// Bookkeeping of one launch, run by one wave (lanes 0..63 of a workgroup) once every workgroup's maximum is in
// the slots: amax, history roll, next scale; leaves the workspace zeroed.  Every global access is one round
// trip for the whole wave instead of one per history entry.
//
// collect_amax: the maximum over the slots as a bit pattern (NaN patterns normalised to the quiet NaN).
__device__ inline uint32_t collect_amax(Workspace* ws) {
    const int lane = threadIdx.x;
    uint32_t bits = 0;
    if (lane < kMaxSlots) bits = __hip_atomic_load(&ws->slot[lane].bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    bits = wave_max_u32(bits);
    if (bits > kInfBits) bits = kNanBits;
    return bits;
}

// bookkeep: what one tensor role learns from the amax `bits` of this launch.
__device__ inline void bookkeep(uint32_t bits, const ScalarIO& io, int mode, const EpiloguePrefetch& pre) {
    const int lane = threadIdx.x;
    const float a = __uint_as_float(bits);
    float used;
    if (mode == kModeAmaxOnly) {
        // (the flag and the held scale are read here, before lane 0 writes either below)
        if (io.init_flag && *io.init_flag != 0.0f) used = *io.scale_state;
        else used = update_scale(a, pre.scale, io.fmt, io.margin);
    } else {
        used = pre.scale;
    }
    uint32_t hm = bits;
    if (io.hist && io.hist_len <= 64) {
        const bool ok = lane < io.hist_len;
        const float h = lane == 0 ? a : pre.hist_prev;
        if (ok) io.hist[lane] = h;
        const uint32_t hb = wave_max_u32(ok ? (__float_as_uint(h) & 0x7fffffffu) : 0u);
        hm = hb > hm ? hb : hm;
        if (hm > kInfBits) hm = kNanBits;
    } else if (io.hist) {
        // hist[i] <- hist[i-1], hist[0] <- a; 64 entries per trip, highest chunk first so that an entry is
        // read before the chunk below overwrites it
        for (int base = ((io.hist_len - 1) / 64) * 64; base >= 0; base -= 64) {
            const int i = base + lane;
            const bool ok = i < io.hist_len;
            float h = 0.0f;
            if (ok) h = (i == 0) ? a : io.hist[i - 1];
            if (ok) io.hist[i] = h;
            const uint32_t hb = wave_max_u32(ok ? (__float_as_uint(h) & 0x7fffffffu) : 0u);
            hm = hb > hm ? hb : hm;
        }
        if (hm > kInfBits) hm = kNanBits;
    }
    if (lane == 0) {
        uint32_t out_bits = bits;
        if (io.amax_in) {   // running maximum kept by the caller (NaN patterns compare above everything)
            uint32_t prev = __float_as_uint(*io.amax_in) & 0x7fffffffu;
            if (prev > kInfBits) prev = kNanBits;
            out_bits = prev > out_bits ? prev : out_bits;
        }
        if (io.amax_out) *io.amax_out = __uint_as_float(out_bits);
        if (io.scale_out) *io.scale_out = used;
        if (io.scale_inv_out) *io.scale_inv_out = 1.0f / used;
        if (io.hist) *io.scale_state = update_scale(__uint_as_float(hm), used, io.fmt, io.margin);
        if (io.init_flag && bits != 0u && bits < kInfBits) *io.init_flag = 1.0f;
    }
}

__device__ inline void clear_workspace(Workspace* ws) {
    const int lane = threadIdx.x;
    if (lane == 0) __hip_atomic_store(&ws->ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (lane < kMaxSlots) {
        __hip_atomic_store(&ws->slot[lane].bits, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&ws->slot[lane].ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// `io2` / `pre2`: a second tensor role fed by the same amax (one source tensor quantised to both formats).
__device__ inline void finalize_wave(Workspace* ws, const ScalarIO& io, int mode, const EpiloguePrefetch& pre,
                                     const ScalarIO* io2 = nullptr, const EpiloguePrefetch* pre2 = nullptr) {
    const uint32_t bits = collect_amax(ws);
    bookkeep(bits, io, mode, pre);
    if (io2) bookkeep(bits, *io2, mode, *pre2);
    clear_workspace(ws);
}

// `bid` of `nblocks`: this workgroup's place among the workgroups that reduce the same tensor (the whole grid,
// except in a launch that carries several tensors).
template <int THREADS>
__device__ inline void publish_and_finalize(uint32_t m_f32bits, Workspace* ws, const ScalarIO& io, int mode,
                                            const EpiloguePrefetch& pre, uint32_t bid = blockIdx.x,
                                            uint32_t nblocks = gridDim.x, const ScalarIO* io2 = nullptr,
                                            const EpiloguePrefetch* pre2 = nullptr) {
    __shared__ uint32_t s_part[THREADS / 64];
    __shared__ bool s_last;
    const uint32_t wm = wave_max_u32(m_f32bits);
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = wm;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t bm = 0;
#pragma unroll
        for (int i = 0; i < THREADS / 64; ++i) bm = s_part[i] > bm ? s_part[i] : bm;
        // Two-level arrival count: a block publishes into the slot of its group and draws a ticket there; the
        // last block of a group draws a ticket of the launch.  All blocks finish at about the same time, and
        // their atomics on one address would queue one behind the other.
        const uint32_t grp = bid % kMaxSlots;
        const uint32_t old = __hip_atomic_fetch_max(&ws->slot[grp].bits, bm, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::"v"(old) : "memory");   // the max is in place before the ticket is drawn
        const uint32_t in_group = (nblocks - grp + kMaxSlots - 1) / kMaxSlots;
        const uint32_t t = __hip_atomic_fetch_add(&ws->slot[grp].ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        bool last = false;
        if (t == in_group - 1) {
            const uint32_t groups = nblocks < (uint32_t)kMaxSlots ? nblocks : (uint32_t)kMaxSlots;
            const uint32_t t2 = __hip_atomic_fetch_add(&ws->ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last = (t2 == groups - 1);
        }
        s_last = last;
    }
    __syncthreads();
    // the epilogue runs on the first wave of the block that drew the last ticket
    if (!s_last || threadIdx.x >= 64) return;
    finalize_wave(ws, io, mode, pre, io2, pre2);
}

// The same bookkeeping for maxima that another kernel (the fp8-output GEMM epilogue) left in the slots.
__global__ __launch_bounds__(64) void amax_finalize_kernel(Workspace* ws, ScalarIO io) {
    const EpiloguePrefetch pre = prefetch_epilogue(io, kModeDelayed);
    finalize_wave(ws, io, kModeDelayed, pre);
}

__device__ __forceinline__ bool degenerate_scale(float s) {
    const uint32_t b = __float_as_uint(s) & 0x7fffffffu;
    return b == 0u || b >= kInfBits;
}

// ---------------------------------------------------------------------------------------------
// Flat (no transpose) kernel: amax only, cast only, or both (delayed scaling).
template <typename S, int F, int MODE>
__device__ __forceinline__ void quant_flat_body(const typename ElemOf<S>::type* __restrict__ x, int64_t n_vec, int64_t n,
                                                uint8_t* __restrict__ out, const float* __restrict__ scale_ptr,
                                                Workspace* ws, const ScalarIO& io, uint32_t bid, uint32_t nblocks) {
    typedef Src<S> L;
    constexpr bool kCast = MODE != kModeAmaxOnly;
    constexpr bool kAmax = MODE != kModeCastOnly;
    float scale = 1.0f;
    bool degen = false;
    if constexpr (kCast) {
        scale = *scale_ptr;
        degen = degenerate_scale(scale);
    }
    EpiloguePrefetch pre = {0.0f, 1.0f};
    if constexpr (kAmax) pre = prefetch_epilogue(io, MODE);
    uint32_t m_run = 0;  // in source-format bits
    const int64_t stride = (int64_t)nblocks * kFlatThreads;
    int64_t i = (int64_t)bid * kFlatThreads + threadIdx.x;
    // two groups per trip: four (bf16) or eight (fp32) 128-bit loads in flight per lane
    for (; i + stride < n_vec; i += 2 * stride) {
        float v0[16], v1[16];
        uint32_t m0, m1;
        L::load16(x + i * kVec, v0, m0);
        L::load16(x + (i + stride) * kVec, v1, m1);
        if constexpr (kAmax) {
            m_run = m0 > m_run ? m0 : m_run;
            m_run = m1 > m_run ? m1 : m_run;
        }
        if constexpr (kCast) {
            const u4 q0 = encode16<F>(v0, scale, degen || L::has_nan(m0));
            const u4 q1 = encode16<F>(v1, scale, degen || L::has_nan(m1));
            __builtin_nontemporal_store(q0, reinterpret_cast<u4*>(out + i * kVec));
            __builtin_nontemporal_store(q1, reinterpret_cast<u4*>(out + (i + stride) * kVec));
        }
    }
    if (i < n_vec) {
        float v0[16];
        uint32_t m0;
        L::load16(x + i * kVec, v0, m0);
        if constexpr (kAmax) m_run = m0 > m_run ? m0 : m_run;
        if constexpr (kCast) {
            const u4 q0 = encode16<F>(v0, scale, degen || L::has_nan(m0));
            __builtin_nontemporal_store(q0, reinterpret_cast<u4*>(out + i * kVec));
        }
    }
    // elements the vector body does not cover (tail, or everything when a pointer is misaligned)
    for (int64_t j = n_vec * kVec + (int64_t)bid * kFlatThreads + threadIdx.x; j < n; j += stride) {
        uint32_t m;
        const float xv = L::load1(x + j, m);
        if constexpr (kAmax) m_run = m > m_run ? m : m_run;
        if constexpr (kCast) out[j] = encode1<F>(xv, scale);
    }
    if constexpr (kAmax) publish_and_finalize<kFlatThreads>(L::to_f32_bits(m_run), ws, io, MODE, pre, bid, nblocks);
}

template <typename S, int F, int MODE>
__global__ __launch_bounds__(kFlatThreads) void quant_flat_kernel(const typename ElemOf<S>::type* __restrict__ x,
                                                              int64_t n_vec, int64_t n, uint8_t* __restrict__ out,
                                                              const float* __restrict__ scale_ptr, Workspace* ws,
                                                              ScalarIO io) {
    quant_flat_body<S, F, MODE>(x, n_vec, n, out, scale_ptr, ws, io, blockIdx.x, gridDim.x);
}

// One source tensor, both formats, one pass: the fused delayed-scaling step of an e4m3 role and an e5m2 role that
// quantise the same tensor (4 bytes per bf16 element instead of 2 x 3).  The amax is shared; each role has its own
// scale, history and output.
template <typename S>
__global__ __launch_bounds__(kFlatThreads) void quant_flat_dual_kernel(const typename ElemOf<S>::type* __restrict__ x,
                                                                   int64_t n_vec, int64_t n, uint8_t* __restrict__ out0,
                                                                   uint8_t* __restrict__ out1, Workspace* ws, ScalarIO io0,
                                                                   ScalarIO io1) {
    typedef Src<S> L;
    const float s0 = *io0.scale_state, s1 = *io1.scale_state;
    const bool d0 = degenerate_scale(s0), d1 = degenerate_scale(s1);
    const EpiloguePrefetch pre0 = prefetch_epilogue(io0, kModeDelayed);
    const EpiloguePrefetch pre1 = prefetch_epilogue(io1, kModeDelayed);
    uint32_t m_run = 0;
    const int64_t stride = (int64_t)gridDim.x * kFlatThreads;
    int64_t i = (int64_t)blockIdx.x * kFlatThreads + threadIdx.x;
    for (; i + stride < n_vec; i += 2 * stride) {
        float v0[16], v1[16];
        uint32_t m0, m1;
        L::load16(x + i * kVec, v0, m0);
        L::load16(x + (i + stride) * kVec, v1, m1);
        m_run = m0 > m_run ? m0 : m_run;
        m_run = m1 > m_run ? m1 : m_run;
        const bool n0 = L::has_nan(m0), n1 = L::has_nan(m1);
        __builtin_nontemporal_store(encode16<kE4M3>(v0, s0, d0 || n0), reinterpret_cast<u4*>(out0 + i * kVec));
        __builtin_nontemporal_store(encode16<kE5M2>(v0, s1, d1 || n0), reinterpret_cast<u4*>(out1 + i * kVec));
        __builtin_nontemporal_store(encode16<kE4M3>(v1, s0, d0 || n1), reinterpret_cast<u4*>(out0 + (i + stride) * kVec));
        __builtin_nontemporal_store(encode16<kE5M2>(v1, s1, d1 || n1), reinterpret_cast<u4*>(out1 + (i + stride) * kVec));
    }
    if (i < n_vec) {
        float v0[16];
        uint32_t m0;
        L::load16(x + i * kVec, v0, m0);
        m_run = m0 > m_run ? m0 : m_run;
        const bool n0 = L::has_nan(m0);
        __builtin_nontemporal_store(encode16<kE4M3>(v0, s0, d0 || n0), reinterpret_cast<u4*>(out0 + i * kVec));
        __builtin_nontemporal_store(encode16<kE5M2>(v0, s1, d1 || n0), reinterpret_cast<u4*>(out1 + i * kVec));
    }
    for (int64_t j = n_vec * kVec + (int64_t)blockIdx.x * kFlatThreads + threadIdx.x; j < n; j += stride) {
        uint32_t m;
        const float xv = L::load1(x + j, m);
        m_run = m > m_run ? m : m_run;
        out0[j] = encode1<kE4M3>(xv, s0);
        out1[j] = encode1<kE5M2>(xv, s1);
    }
    publish_and_finalize<kFlatThreads>(L::to_f32_bits(m_run), ws, io0, kModeDelayed, pre0, blockIdx.x, gridDim.x, &io1, &pre1);
}

// Several tensors, one launch (the fused delayed-scaling step of each): the workgroups of tensor t follow those of
// tensor t - 1, so the tail of one tensor (its last loads, its reduction, its bookkeeping) runs under the streaming
// of the next instead of in front of a kernel boundary.  Every tensor has its own workspace.
constexpr int kMaxMulti = 16;
struct MultiQuant {
    struct Tensor {
        const void* x;
        uint8_t* out;
        int64_t n_vec, n;
        Workspace* ws;
        ScalarIO io;
        int first_block, blocks;
    } t[kMaxMulti];
    int count;
};

template <typename S, int F>
__global__ __launch_bounds__(kFlatThreads) void quant_flat_multi_kernel(const MultiQuant Q) {
    int which = 0;
#pragma unroll
    for (int i = 1; i < kMaxMulti; ++i)
        if (i < Q.count && (int)blockIdx.x >= Q.t[i].first_block) which = i;
    const MultiQuant::Tensor& T = Q.t[which];
    quant_flat_body<S, F, kModeDelayed>(static_cast<const typename ElemOf<S>::type*>(T.x), T.n_vec, T.n, T.out,
                                        T.io.scale_state, T.ws, T.io, blockIdx.x - T.first_block, T.blocks);
}

// ---------------------------------------------------------------------------------------------
// Cast (+ optional amax) that also writes the transposed bytes.  One 128x128 tile per block, staged
// through 16 KB of LDS.  LDS holds the tile transposed, [col][row], the 16-byte row chunks of each
// column XOR-swizzled with the column's 16-wide chunk index so that both the byte stores of phase 1
// and the 128-bit loads of phase 2 are bank-conflict free.
constexpr int kTile = 128;

template <typename S, int F, bool kAmax>
__global__ __launch_bounds__(kTileThreads) void quant_transpose_kernel(const typename ElemOf<S>::type* __restrict__ x,
                                                                   int64_t rows, int64_t cols,
                                                                   uint8_t* __restrict__ out,
                                                                   uint8_t* __restrict__ out_t,
                                                                   const float* __restrict__ scale_ptr,
                                                                   Workspace* ws, ScalarIO io) {
    typedef Src<S> L;
    __shared__ __attribute__((aligned(16))) uint8_t tile[kTile * kTile];
    const float scale = *scale_ptr;
    const bool degen = degenerate_scale(scale);
    const int64_t tiles_c = cols / kTile;
    const int64_t tiles = (rows / kTile) * tiles_c;
    const int t = threadIdx.x;
    const int cchunk = t & 7;   // 16-column chunk inside the tile
    const int rsub = t >> 3;    // 0..31
    const int rchunk = t & 7;
    EpiloguePrefetch pre = {0.0f, 1.0f};
    if constexpr (kAmax) pre = prefetch_epilogue(io, kModeDelayed);
    uint32_t m_run = 0;
    // persistent over tiles: the number of blocks (and so of reduction atomics) stays ~2 per CU
    for (int64_t tile_id = blockIdx.x; tile_id < tiles; tile_id += gridDim.x) {
    const int64_t row0 = (tile_id / tiles_c) * kTile, col0 = (tile_id % tiles_c) * kTile;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int r = rsub + 32 * it;
        const int64_t g = (row0 + r) * cols + col0 + cchunk * 16;
        float v[16];
        uint32_t m16;
        L::load16(x + g, v, m16);
        if constexpr (kAmax) m_run = m16 > m_run ? m16 : m_run;
        const u4 q = encode16<F>(v, scale, degen || L::has_nan(m16));
        if (out) __builtin_nontemporal_store(q, reinterpret_cast<u4*>(out + g));
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        const int rsw = r ^ (cchunk << 4);  // swizzled row position inside a column
#pragma unroll
        for (int j = 0; j < 16; ++j)
            tile[(cchunk * 16 + j) * kTile + rsw] = (uint8_t)(w[j >> 2] >> (8 * (j & 3)));
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int c = rsub + 32 * it;
        const int pos = (rchunk ^ (c >> 4)) << 4;
        const u4 q = *reinterpret_cast<const u4*>(&tile[c * kTile + pos]);
        __builtin_nontemporal_store(q, reinterpret_cast<u4*>(out_t + (col0 + c) * rows + row0 + rchunk * 16));
    }
    __syncthreads();  // the tile buffer is reused by the next trip
    }
    if constexpr (kAmax) publish_and_finalize<kTileThreads>(L::to_f32_bits(m_run), ws, io, kModeDelayed, pre);
}

// Any shape: one element per thread step, transposed store.  Used when the tile kernel's
// 128-multiples / alignment requirements are not met.
template <typename S, int F, bool kAmax>
__global__ __launch_bounds__(kThreads) void quant_transpose_scalar_kernel(
    const typename ElemOf<S>::type* __restrict__ x, int64_t rows, int64_t cols, uint8_t* __restrict__ out,
    uint8_t* __restrict__ out_t, const float* __restrict__ scale_ptr, Workspace* ws, ScalarIO io) {
    typedef Src<S> L;
    const float scale = *scale_ptr;
    const int64_t n = rows * cols;
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    EpiloguePrefetch pre = {0.0f, 1.0f};
    if constexpr (kAmax) pre = prefetch_epilogue(io, kModeDelayed);
    uint32_t m_run = 0;
    for (int64_t j = (int64_t)blockIdx.x * kThreads + threadIdx.x; j < n; j += stride) {
        uint32_t m;
        const float xv = L::load1(x + j, m);
        if constexpr (kAmax) m_run = m > m_run ? m : m_run;
        const uint8_t b = encode1<F>(xv, scale);
        if (out) out[j] = b;
        const int64_t r = j / cols, c = j % cols;
        out_t[c * rows + r] = b;
    }
    if constexpr (kAmax) publish_and_finalize<kThreads>(L::to_f32_bits(m_run), ws, io, kModeDelayed, pre);
}

// ---------------------------------------------------------------------------------------------
// Dequantise: out = out_dtype(decode(byte) * (1 / scale)).
template <int F>
__device__ __forceinline__ float decode1(uint32_t b) {
    if constexpr (F == kE4M3) return __builtin_amdgcn_cvt_f32_fp8((int)b, 0);
    else return __builtin_amdgcn_cvt_f32_bf8((int)b, 0);
}

// `is_inverse`: scale_ptr holds 1 / scale already (the form tex.cast_from_fp8 is handed, src/nanotron/fp8/tensor.py:74)
template <int F, int OUT>
__global__ __launch_bounds__(kThreads) void dequant_kernel(const uint8_t* __restrict__ in, int64_t n,
                                                           const float* __restrict__ scale_ptr, void* __restrict__ out,
                                                           int is_inverse) {
    const float inv = is_inverse ? *scale_ptr : 1.0f / *scale_ptr;
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    for (int64_t j = (int64_t)blockIdx.x * kThreads + threadIdx.x; j < n; j += stride) {
        float v = decode1<F>(in[j]) * inv;
        // keep the fp32 product a value of its own: folded into a mixed-precision fma (x*y + 0) the
        // conversion would turn -0 into +0
        asm volatile("" : "+v"(v));
        if constexpr (OUT == NTFP8_F32) ((float*)out)[j] = v;
        else if constexpr (OUT == NTFP8_F16) ((__half*)out)[j] = __float2half_rn(v);
        else {
            // bf16 round-to-nearest-even with NaN kept quiet
            uint32_t u = __float_as_uint(v);
            uint16_t r;
            if ((u & 0x7fffffffu) > kInfBits) r = (uint16_t)((u >> 16) | 0x40u);
            else r = (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
            ((uint16_t*)out)[j] = r;
        }
    }
}

// Byte transpose through a 64x64 LDS tile (pitch 65 breaks the bank pattern); any shape.
__global__ __launch_bounds__(kThreads) void transpose_kernel(const uint8_t* __restrict__ in, int64_t rows, int64_t cols,
                                                             uint8_t* __restrict__ out) {
    __shared__ uint8_t tile[64][65];
    const int64_t tiles_c = (cols + 63) / 64;
    const int64_t r0 = (blockIdx.x / tiles_c) * 64, c0 = (blockIdx.x % tiles_c) * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int r = ty; r < 64; r += 4)
        if (r0 + r < rows && c0 + tx < cols) tile[r][tx] = in[(r0 + r) * cols + c0 + tx];
    __syncthreads();
    for (int c = ty; c < 64; c += 4)
        if (c0 + c < cols && r0 + tx < rows) out[(c0 + c) * rows + r0 + tx] = tile[tx][c];
}

// ---------------------------------------------------------------------------------------------
// Bandwidth yardsticks: the access pattern of the flat quantise kernel (one 1024-thread workgroup per CU, two
// 16-element groups per lane and trip, 128-bit non-temporal accesses) with the arithmetic and the reduction taken
// out.  kProbeRead: 32 bytes read per group, nothing written.  kProbeHalf: 32 bytes read, 16 written (the traffic of
// a bf16 -> fp8 cast).  kProbeCopy: 32 read, 32 written.
enum ProbeMode { kProbeRead = NTFP8_PROBE_READ, kProbeHalf = NTFP8_PROBE_HALF, kProbeCopy = NTFP8_PROBE_COPY };
template <int MODE>
__global__ __launch_bounds__(kFlatThreads) void stream_probe_kernel(const u4* __restrict__ src, int64_t n_vec, u4* __restrict__ dst) {
    const int64_t stride = (int64_t)gridDim.x * kFlatThreads;
    int64_t i = (int64_t)blockIdx.x * kFlatThreads + threadIdx.x;
    u4 seen = {0u, 0u, 0u, 0u};
    auto one = [&](int64_t k) {
        const u4 a = __builtin_nontemporal_load(src + 2 * k), b = __builtin_nontemporal_load(src + 2 * k + 1);
        if constexpr (MODE == kProbeRead) seen = seen | (a ^ b);
        else if constexpr (MODE == kProbeHalf) __builtin_nontemporal_store(a ^ b, dst + k);
        else {
            __builtin_nontemporal_store(a, dst + 2 * k);
            __builtin_nontemporal_store(b, dst + 2 * k + 1);
        }
    };
    for (; i + stride < n_vec; i += 2 * stride) {
        one(i);
        one(i + stride);
    }
    if (i < n_vec) one(i);
    if constexpr (MODE == kProbeRead) {
        // keeps the loads alive; a word of dst is written only if every bit of some lane's xor came out set
        if ((seen.x & seen.y & seen.z & seen.w) == 0xffffffffu) reinterpret_cast<uint32_t*>(dst)[0] = 1u;
    }
}

__global__ void update_scale_kernel(const float* amax, const float* old_scale, int fmt, int margin, float* out,
                                    int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = update_scale(amax[i], old_scale[i], fmt, margin);
}

// ---------------------------------------------------------------------------------------------
// Host-side launchers.
// blocks for `work_items` thread-steps with `threads` per block, at most `per_cu_blocks` per CU
static int grid_for(int64_t work_items, int threads = kThreads, int per_cu_blocks = 8) {
    int64_t want = (work_items + threads - 1) / threads;
    int64_t cap = (int64_t)cu_count() * per_cu_blocks;
    if (want < 1) want = 1;
    return (int)(want < cap ? want : cap);
}

// The launch macro reports through the thread's last-error slot.  hipGetLastError() reads and clears it; an error
// left there by an unrelated earlier call of this thread is dropped by clear_stale_error() before a launch, so that
// check_launch() speaks for this library's launch only.
static void clear_stale_error() { (void)hipGetLastError(); }
static int check_launch() { return hipGetLastError() == hipSuccess ? NTFP8_OK : NTFP8_ERR_LAUNCH; }

template <typename S, int F>
static int launch_flat(int mode, const void* x, int64_t n, bool vec_ok, uint8_t* out, const float* scale_ptr,
                       Workspace* ws, const ScalarIO& io, hipStream_t st) {
    typedef typename ElemOf<S>::type E;
    const int64_t n_vec = vec_ok ? n / kVec : 0;
    // two 16-element groups per lane per trip
    const int grid = grid_for(n_vec > 0 ? (n_vec + 1) / 2 : n, kFlatThreads, 1);
    const E* xp = static_cast<const E*>(x);
    if (mode == kModeAmaxOnly)
        hipLaunchKernelGGL((quant_flat_kernel<S, F, kModeAmaxOnly>), dim3(grid), dim3(kFlatThreads), 0, st, xp, n_vec, n, out,
                           scale_ptr, ws, io);
    else if (mode == kModeCastOnly)
        hipLaunchKernelGGL((quant_flat_kernel<S, F, kModeCastOnly>), dim3(grid), dim3(kFlatThreads), 0, st, xp, n_vec, n, out,
                           scale_ptr, ws, io);
    else
        hipLaunchKernelGGL((quant_flat_kernel<S, F, kModeDelayed>), dim3(grid), dim3(kFlatThreads), 0, st, xp, n_vec, n, out,
                           scale_ptr, ws, io);
    return check_launch();
}

template <typename S, int F>
static int launch_transpose(bool with_amax, const void* x, int64_t rows, int64_t cols, bool tile_ok, uint8_t* out,
                            uint8_t* out_t, const float* scale_ptr, Workspace* ws, const ScalarIO& io, hipStream_t st) {
    typedef typename ElemOf<S>::type E;
    const E* xp = static_cast<const E*>(x);
    if (tile_ok) {
        const int64_t tiles = (rows / kTile) * (cols / kTile);
        const int64_t cap = (int64_t)cu_count() * (with_amax ? 2 : 8);
        const int tgrid = (int)(tiles < cap ? tiles : cap);
        if (with_amax)
            hipLaunchKernelGGL((quant_transpose_kernel<S, F, true>), dim3(tgrid), dim3(kTileThreads), 0, st, xp, rows,
                               cols, out, out_t, scale_ptr, ws, io);
        else
            hipLaunchKernelGGL((quant_transpose_kernel<S, F, false>), dim3(tgrid), dim3(kTileThreads), 0, st, xp, rows,
                               cols, out, out_t, scale_ptr, ws, io);
    } else {
        const int grid = grid_for(rows * cols);
        if (with_amax)
            hipLaunchKernelGGL((quant_transpose_scalar_kernel<S, F, true>), dim3(grid), dim3(kThreads), 0, st, xp, rows,
                               cols, out, out_t, scale_ptr, ws, io);
        else
            hipLaunchKernelGGL((quant_transpose_scalar_kernel<S, F, false>), dim3(grid), dim3(kThreads), 0, st, xp, rows,
                               cols, out, out_t, scale_ptr, ws, io);
    }
    return check_launch();
}

template <typename S>
static int dispatch_fmt_flat(int fmt, int mode, const void* x, int64_t n, bool vec_ok, uint8_t* out,
                             const float* scale_ptr, Workspace* ws, const ScalarIO& io, hipStream_t st) {
    return fmt == kE4M3 ? launch_flat<S, kE4M3>(mode, x, n, vec_ok, out, scale_ptr, ws, io, st)
                        : launch_flat<S, kE5M2>(mode, x, n, vec_ok, out, scale_ptr, ws, io, st);
}

template <typename S>
static int dispatch_fmt_tr(int fmt, bool with_amax, const void* x, int64_t rows, int64_t cols, bool tile_ok,
                           uint8_t* out, uint8_t* out_t, const float* scale_ptr, Workspace* ws, const ScalarIO& io,
                           hipStream_t st) {
    return fmt == kE4M3 ? launch_transpose<S, kE4M3>(with_amax, x, rows, cols, tile_ok, out, out_t, scale_ptr, ws, io, st)
                        : launch_transpose<S, kE5M2>(with_amax, x, rows, cols, tile_ok, out, out_t, scale_ptr, ws, io, st);
}

static bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// mode: kModeAmaxOnly / kModeCastOnly / kModeDelayed.  out_t may be NULL.
int run_quant(int mode, const void* x, int x_dtype, int64_t rows, int64_t cols, int fmt, uint8_t* out, uint8_t* out_t,
              const float* scale_ptr, Workspace* ws, const ScalarIO& io, hipStream_t st) {
    clear_stale_error();
    const int64_t n = rows * cols;
    if (mode != kModeAmaxOnly && out_t != nullptr) {
        const bool tile_ok = rows % kTile == 0 && cols % kTile == 0 && aligned(x, 16) && aligned(out_t, 16) &&
                             (out == nullptr || aligned(out, 16));
        const bool with_amax = mode == kModeDelayed;
        switch (x_dtype) {
            case NTFP8_F32: return dispatch_fmt_tr<float>(fmt, with_amax, x, rows, cols, tile_ok, out, out_t, scale_ptr, ws, io, st);
            case NTFP8_F16: return dispatch_fmt_tr<f16_tag>(fmt, with_amax, x, rows, cols, tile_ok, out, out_t, scale_ptr, ws, io, st);
            default: return dispatch_fmt_tr<bf16_tag>(fmt, with_amax, x, rows, cols, tile_ok, out, out_t, scale_ptr, ws, io, st);
        }
    }
    const bool vec_ok = aligned(x, 16) && (mode == kModeAmaxOnly || aligned(out, 16));
    switch (x_dtype) {
        case NTFP8_F32: return dispatch_fmt_flat<float>(fmt, mode, x, n, vec_ok, out, scale_ptr, ws, io, st);
        case NTFP8_F16: return dispatch_fmt_flat<f16_tag>(fmt, mode, x, n, vec_ok, out, scale_ptr, ws, io, st);
        default: return dispatch_fmt_flat<bf16_tag>(fmt, mode, x, n, vec_ok, out, scale_ptr, ws, io, st);
    }
}

template <typename S, int F>
static int launch_flat_multi(const QuantDesc* const* q, int count, hipStream_t st) {
    clear_stale_error();
    MultiQuant Q = {};
    Q.count = count;
    int blocks = 0;
    for (int i = 0; i < count; ++i) {
        const QuantDesc& d = *q[i];
        const int64_t n = d.rows * d.cols;
        const bool vec_ok = aligned(d.x, 16) && aligned(d.out, 16);
        MultiQuant::Tensor& T = Q.t[i];
        T.x = d.x;
        T.out = static_cast<uint8_t*>(d.out);
        T.n = n;
        T.n_vec = vec_ok ? n / kVec : 0;
        T.ws = static_cast<Workspace*>(d.ws);
        T.io = d.io;
        T.first_block = blocks;
        T.blocks = grid_for(T.n_vec > 0 ? (T.n_vec + 1) / 2 : n, kFlatThreads, 1);
        blocks += T.blocks;
    }
    hipLaunchKernelGGL((quant_flat_multi_kernel<S, F>), dim3(blocks), dim3(kFlatThreads), 0, st, Q);
    return check_launch();
}

template <typename S>
static int dispatch_flat_multi(int fmt, const QuantDesc* const* q, int count, hipStream_t st) {
    return fmt == kE4M3 ? launch_flat_multi<S, kE4M3>(q, count, st) : launch_flat_multi<S, kE5M2>(q, count, st);
}

// The fused delayed-scaling step of several tensors.  Tensors without a transposed copy that share source type and
// format go out together, up to kMaxMulti per launch; the others one by one.
int run_quant_delayed_batch(const QuantDesc* q, int count, hipStream_t st) {
    bool done[NTFP8_MAX_BATCH] = {false};
    for (int i = 0; i < count; ++i) {
        if (done[i]) continue;
        done[i] = true;
        if (q[i].out_t != nullptr || q[i].out == nullptr) {
            const int rc = run_quant(kModeDelayed, q[i].x, q[i].x_dtype, q[i].rows, q[i].cols, q[i].fmt,
                                     static_cast<uint8_t*>(q[i].out), static_cast<uint8_t*>(q[i].out_t), q[i].io.scale_state,
                                     static_cast<Workspace*>(q[i].ws), q[i].io, st);
            if (rc != NTFP8_OK) return rc;
            continue;
        }
        const QuantDesc* group[kMaxMulti];
        int cnt = 0;
        group[cnt++] = &q[i];
        for (int j = i + 1; j < count && cnt < kMaxMulti; ++j)
            if (!done[j] && q[j].out_t == nullptr && q[j].out != nullptr && q[j].x_dtype == q[i].x_dtype && q[j].fmt == q[i].fmt) {
                group[cnt++] = &q[j];
                done[j] = true;
            }
        int rc;
        switch (q[i].x_dtype) {
            case NTFP8_F32: rc = dispatch_flat_multi<float>(q[i].fmt, group, cnt, st); break;
            case NTFP8_F16: rc = dispatch_flat_multi<f16_tag>(q[i].fmt, group, cnt, st); break;
            default: rc = dispatch_flat_multi<bf16_tag>(q[i].fmt, group, cnt, st); break;
        }
        if (rc != NTFP8_OK) return rc;
    }
    return NTFP8_OK;
}

// Both formats from one pass over x (flat layout only).
int run_quant_dual(const void* x, int x_dtype, int64_t n, uint8_t* out_e4m3, uint8_t* out_e5m2, Workspace* ws,
                   const ScalarIO& io_e4m3, const ScalarIO& io_e5m2, hipStream_t st) {
    clear_stale_error();
    const bool vec_ok = aligned(x, 16) && aligned(out_e4m3, 16) && aligned(out_e5m2, 16);
    const int64_t n_vec = vec_ok ? n / kVec : 0;
    const int grid = grid_for(n_vec > 0 ? (n_vec + 1) / 2 : n, kFlatThreads, 1);
    switch (x_dtype) {
        case NTFP8_F32:
            hipLaunchKernelGGL((quant_flat_dual_kernel<float>), dim3(grid), dim3(kFlatThreads), 0, st,
                               static_cast<const float*>(x), n_vec, n, out_e4m3, out_e5m2, ws, io_e4m3, io_e5m2);
            break;
        case NTFP8_F16:
            hipLaunchKernelGGL((quant_flat_dual_kernel<f16_tag>), dim3(grid), dim3(kFlatThreads), 0, st,
                               static_cast<const uint16_t*>(x), n_vec, n, out_e4m3, out_e5m2, ws, io_e4m3, io_e5m2);
            break;
        default:
            hipLaunchKernelGGL((quant_flat_dual_kernel<bf16_tag>), dim3(grid), dim3(kFlatThreads), 0, st,
                               static_cast<const uint16_t*>(x), n_vec, n, out_e4m3, out_e5m2, ws, io_e4m3, io_e5m2);
            break;
    }
    return check_launch();
}

// ---------------------------------------------------------------------------------------------
// Reduction workspaces that live in the library's own device image, for callers that cannot allocate device
// memory (HIP graph capture, serving loops): one Workspace per tensor of a batched call.  Every GPU the library
// runs on holds its own copy of the array, at its own address, until the process ends; the name below is only a
// host-side handle of it, the address comes from hipGetSymbolAddress with that device current.
static __device__ __align__(256) unsigned char scratch[NTFP8_STATIC_MAX_TENSORS * NTFP8_WORKSPACE_BYTES];

// Device address of `scratch` on the current device, resolved at the first call for that device.  Nothing is launched:
// a device image starts with the array zeroed and every kernel leaves its workspace zero, so there is nothing to
// clear, and a clearing kernel on the first caller's stream would race with a first user on another stream.
int static_scratch(void** out, hipStream_t) {
    static std::atomic<void*> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return NTFP8_ERR_LAUNCH;
    void* p = cached[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        // (threads that race here resolve the same address)
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return NTFP8_ERR_LAUNCH;
        cached[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return NTFP8_OK;
}

// run_quant_delayed_batch with the workspaces taken from the static array (count <= NTFP8_STATIC_MAX_TENSORS)
int run_quant_delayed_batch_static(QuantDesc* q, int count, hipStream_t st) {
    void* base = nullptr;
    const int rc = static_scratch(&base, st);
    if (rc != NTFP8_OK) return rc;
    for (int i = 0; i < count; ++i) q[i].ws = static_cast<unsigned char*>(base) + (size_t)i * NTFP8_WORKSPACE_BYTES;
    return run_quant_delayed_batch(q, count, st);
}

int run_dequant(const void* in, int fmt, const float* scale, int is_inverse, int64_t n, void* out, int out_dtype,
                hipStream_t st) {
    clear_stale_error();
    const int grid = grid_for(n);
    const uint8_t* p = static_cast<const uint8_t*>(in);
#define NT_DQ(F, O) hipLaunchKernelGGL((dequant_kernel<F, O>), dim3(grid), dim3(kThreads), 0, st, p, n, scale, out, is_inverse)
    if (fmt == kE4M3) {
        if (out_dtype == NTFP8_F32) NT_DQ(kE4M3, NTFP8_F32);
        else if (out_dtype == NTFP8_F16) NT_DQ(kE4M3, NTFP8_F16);
        else NT_DQ(kE4M3, NTFP8_BF16);
    } else {
        if (out_dtype == NTFP8_F32) NT_DQ(kE5M2, NTFP8_F32);
        else if (out_dtype == NTFP8_F16) NT_DQ(kE5M2, NTFP8_F16);
        else NT_DQ(kE5M2, NTFP8_BF16);
    }
#undef NT_DQ
    return check_launch();
}

int run_transpose(const void* in, int64_t rows, int64_t cols, void* out, hipStream_t st) {
    clear_stale_error();
    const int64_t tiles = ((rows + 63) / 64) * ((cols + 63) / 64);
    if (tiles > 0x7fffffff) return NTFP8_ERR_SIZE;
    hipLaunchKernelGGL(transpose_kernel, dim3((int)tiles), dim3(kThreads), 0, st, static_cast<const uint8_t*>(in), rows,
                       cols, static_cast<uint8_t*>(out));
    return check_launch();
}

int run_stream_probe(int mode, const void* src, int64_t bytes, void* dst, hipStream_t st) {
    clear_stale_error();
    const int64_t n_vec = bytes / 32;
    const int grid = grid_for((n_vec + 1) / 2, kFlatThreads, 1);
    const u4* s = static_cast<const u4*>(src);
    u4* d = static_cast<u4*>(dst);
    if (mode == kProbeRead) hipLaunchKernelGGL((stream_probe_kernel<kProbeRead>), dim3(grid), dim3(kFlatThreads), 0, st, s, n_vec, d);
    else if (mode == kProbeHalf) hipLaunchKernelGGL((stream_probe_kernel<kProbeHalf>), dim3(grid), dim3(kFlatThreads), 0, st, s, n_vec, d);
    else hipLaunchKernelGGL((stream_probe_kernel<kProbeCopy>), dim3(grid), dim3(kFlatThreads), 0, st, s, n_vec, d);
    return check_launch();
}

int run_amax_finalize(Workspace* ws, const ScalarIO& io, hipStream_t st) {
    clear_stale_error();
    hipLaunchKernelGGL(amax_finalize_kernel, dim3(1), dim3(64), 0, st, ws, io);
    return check_launch();
}

int run_update_scale(const float* amax, const float* old_scale, int fmt, int margin, float* out, int64_t n,
                     hipStream_t st) {
    clear_stale_error();
    const int64_t blocks = (n + 255) / 256;
    if (blocks > 0x7fffffff) return NTFP8_ERR_SIZE;
    hipLaunchKernelGGL(update_scale_kernel, dim3((int)blocks), dim3(256), 0, st, amax, old_scale, fmt, margin, out, n);
    return check_launch();
}

}  // namespace ntfp8
