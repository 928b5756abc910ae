// Large-tile FP8 GEMM kernel for gfx950; included by gemm.hip after the shared helpers.
//
// Block tile (32 MI) x 256 x 128 bytes of K, four waves in a 2 x 2 arrangement, one wave per
// SIMD.  Each wave owns (16 MI) x 128 outputs as MI x 8 accumulator blocks of V_MFMA_F32_16X16X128_F8F6F4
// (MI = 8: 256-row block tile, 256 accumulator registers per lane; MI = 4: 128-row block tile).
//
// Data movement per K-tile: every wave brings a quarter of the A and B tiles from global memory into
// LDS (16 bytes per lane, XOR-swizzled), reads its MI A fragments from LDS once and keeps them in
// registers, and streams its 8 B fragments from LDS two MFMA groups ahead of their use.  One MFMA
// group = the MI MFMAs that share one B fragment.
//
// Pipeline, two LDS stages, ONE workgroup barrier per K-tile placed after MFMA group 5:
//   * before the barrier a wave has read every fragment of the current tile into registers, so the
//     barrier releases the current stage for tile kt + 2 and publishes tile kt + 1 at once;
//   * groups 6 and 7 are issued interleaved, two MFMAs per A fragment; the fragment register is dead
//     after them and is refilled with the same fragment of tile kt + 1, so one set of A registers
//     suffices.
// Global loads: whole tiles (MI = 8) keep one K-tile in flight in registers and write it to LDS a
// K-tile later, so that every load has a full K-tile of MFMA time to arrive; half tiles (MI = 4) have
// no registers to spare and load straight into the released LDS stage.
//
// Instantiations beside the operand formats and MI: kFp8Out (the outputs are fp8 bytes, cast in the
// epilogue, with an optional transposed copy and the amax of the results) and kBT (the B operands are
// given as their transposes, [K, N] tensors, and gathered from LDS with the transposing read).
#pragma once

namespace ntfp8 {

// Profiling build (-DNTFP8_STAMPS, libntfp8_stamps.so): every workgroup of gemm_nt_big_kernel leaves five readings of
// the 100 MHz wall clock (kernel entry, first tile published, end of the K loop, last store issued, stores drained), the
// shader-clock cycle counter at both ends of the K loop and the identity of its CU in a table that
// ntfp8_debug_stamps() copies out.  The product library is built without it.
#ifdef NTFP8_STAMPS
constexpr int kStampSlots = 16384;
__device__ unsigned long long g_stamps[kStampSlots * 8];
// 1: workgroups take the tiles in launch order, i.e. every XCD gets every eighth tile and touches all operand panels
// (an experiment on what the fetch traffic costs; set with ntfp8_debug_set_tile_order)
__device__ int g_plain_tile_order = 0;
#define NTFP8_STAMP(var) var = wall_clock64()
#define NTFP8_CYCLES(var) var = __builtin_readcyclecounter()
// Timing experiments on the K loop of whole tiles, chosen when a profiling build is compiled (the results of such a
// build are wrong, only its stamps mean something).  -DNTFP8_KNOCKOUT=<bits> leaves parts of the loop out: 1 the global
// loads (the registers of the first K-tile are deposited again and again), 2 the deposits into LDS, 4 the workgroup barrier, 8 the LDS reads of the B
// fragments, 16 those of the A fragments.  -DNTFP8_IDLE=<n> lets every wave sleep 64 n cycles behind the barrier of
// every K-tile.  -DNTFP8_COLUMNS=<6 | 7> runs the K loop of a tile that is 192 or 224 columns wide instead of 256 (that
// many of a wave's eight block columns, B loads and B fragments; the schedule is the same with the last front groups
// left out): what a tile width that divides N = 6144 or 14336 into a whole number of rounds would cost per K-tile.
// -DNTFP8_MFMA32=1 (with -DNTFP8_KNOCKOUT=31) issues 32 V_MFMA_F32_32X32X64_F8F6F4 per K-tile in place of the 64
// 16x16x128 ones (the same FLOPs and matrix-pipe cycles, half the operand registers read per FLOP, twice the accumulator
// registers touched): what the other instruction shape draws.
#ifndef NTFP8_KNOCKOUT
#define NTFP8_KNOCKOUT 0
#endif
#ifndef NTFP8_IDLE
#define NTFP8_IDLE 0
#endif
#ifndef NTFP8_COLUMNS
#define NTFP8_COLUMNS 8
#endif
#ifndef NTFP8_MFMA32
#define NTFP8_MFMA32 0
#endif
constexpr int kKnockout = NTFP8_KNOCKOUT, kIdle = NTFP8_IDLE, kColumns = NTFP8_COLUMNS;
constexpr bool kMfma32 = NTFP8_MFMA32 != 0;
#else
#define NTFP8_STAMP(var) (void)0
#define NTFP8_CYCLES(var) (void)0
constexpr int kKnockout = 0, kIdle = 0, kColumns = 8;
constexpr bool kMfma32 = false;
#endif
constexpr bool kNoLoads = kKnockout & 1, kNoDeposits = kKnockout & 2, kNoBarrier = kKnockout & 4, kNoBReads = kKnockout & 8,
               kNoAReads = kKnockout & 16;


constexpr int kBigN = 256;
constexpr int kBigWaves = 4, kBigThreads = kBigWaves * 64;
constexpr int kBigNJ = 8;              // 16-column accumulator blocks per wave: 128 columns
constexpr int kBigLB = kBigN / 8 / kBigWaves;   // 1 KB wave-level loads of the B tile per wave per stage

// Swizzle for 16-row fragments: the 16 lanes that read chunk c of rows r .. r + 15 hit 16 distinct
// 16-byte bank groups when the chunk index is XORed with (row mod 8) ^ (bit 3 of row).
__device__ __forceinline__ int swz16(int row) { return (row & 7) ^ ((row >> 3) & 1); }
__device__ __forceinline__ int lds_off16(int row, int kc) { return row * kBK + ((kc ^ swz16(row)) << 4); }

template <int FA, int FB>
__device__ __forceinline__ v4f mfma_16x16x128(v8i b_frag, v8i a_frag, v4f c) {
    // B fragment first: the 16 x 16 result block is indexed [n][m], so a lane owns 4 consecutive n
    // (n = 4 (lane / 16) + r) of one output row m = lane % 16.
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b_frag, a_frag, c, FB, FA, 0, 0, 0, 0);
}
// rows (groups of 16 lanes) 1 and 3 of x <-> rows 0 and 2 of y (V_PERMLANE16_SWAP)
__device__ __forceinline__ void swap_rows16(uint32_t& x, uint32_t& y) {
    typedef unsigned v2u __attribute__((ext_vector_type(2)));
    const v2u r = __builtin_amdgcn_permlane16_swap(x, y, false, false);
    x = r.x;
    y = r.y;
}
// 16 bytes per lane from global memory into registers; offsets past the descriptor read as zero
__device__ __forceinline__ v4i reg_load16(__amdgpu_buffer_rsrc_t r, uint32_t voff, int soff) {
    return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
__device__ __forceinline__ void sched_fence() { __builtin_amdgcn_sched_barrier(0); }
// 16 bytes of output to global memory, written through to memory as they are issued (sc0 sc1) and marked streaming
// (nt).  An ordinary store leaves its line dirty in the XCD's L2; a tile's worth of output per CU then fills that L2,
// and the lines are written back in one burst when the kernel ends.  Written through, the output drains while the
// other waves still compute: 2.5 us less per round of tiles (4096^3: 58.0 -> 55.5 us; `nt` alone changes nothing).
__device__ __forceinline__ void store16_through(void* p, v4i v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt" ::"v"(p), "v"(v) : "memory");
}

// Epilogue of one wave: MI x NJ accumulator blocks of 16 x 16, block (i, j) at rows m_base + 16 i,
// columns n_base + 16 j.  Descale, optional fp32 accumulate, one rounding, store.
// kBias: bv[j][e] = bias of column n_base + 16 j + 4 (lane / 16) + e, added to the descaled value before the rounding.
template <int DT, bool kAcc, int MI, int NJ, bool kBias = false>
__device__ __forceinline__ void store_wave_tile16(const v4f (&acc)[MI][NJ], void* __restrict__ Dv, float alpha, int M,
                                                  int N, int m_base, int n_base, int lane, const float (*bv)[4] = nullptr) {
    typedef typename OutT<DT>::type O;
    O* D = static_cast<O*>(Dv);
    const int mrow = lane & 15, q = lane >> 4;
    // element e of block (i, j): descaled, plus bias if there is one (two separately rounded fp32 operations)
    auto val = [&](int i, int j, int e) -> float {
        if constexpr (kBias) return acc[i][j][e] * alpha + bv[j][e];
        else return acc[i][j][e] * alpha;
    };
    if constexpr (DT != NTFP8_F32) {
        // 16-bit outputs: a lane's 4 consecutive n are only 8 bytes.  Exchanging registers of two
        // neighbouring blocks between lane rows gives every lane 8 consecutive n (16 bytes) of one
        // block, and lane rows r / r + 2 together a full 32-byte sector per output row, which the
        // memory side writes without read-modify-write traffic.
        if ((N & 7) == 0) {
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                const int m = m_base + i * 16 + mrow;
#pragma unroll
                for (int j = 0; j < NJ; j += 2) {
                    uint32_t x0 = OutT<DT>::pack2(val(i, j, 0), val(i, j, 1));
                    uint32_t x1 = OutT<DT>::pack2(val(i, j, 2), val(i, j, 3));
                    uint32_t y0 = OutT<DT>::pack2(val(i, j + 1, 0), val(i, j + 1, 1));
                    uint32_t y1 = OutT<DT>::pack2(val(i, j + 1, 2), val(i, j + 1, 3));
                    swap_rows16(x0, y0);
                    swap_rows16(x1, y1);
                    // lane row q now holds n 8 (q / 2) .. + 7 of block j + (q & 1): x = first four, y = last four
                    const int n = n_base + (j + (q & 1)) * 16 + (q >> 1) * 8;
                    if (m < M && n < N)
                        store16_through(D + (int64_t)m * N + n, (v4i){(int)x0, (int)x1, (int)y0, (int)y1});
                }
            }
            return;
        }
    }
    const bool vec_ok = (N & 3) == 0;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int m = m_base + i * 16 + mrow;
        if (m >= M) continue;
        // accumulate: all of a row block's old values are requested before the first one is needed
        v4f old[NJ];
        if constexpr (kAcc) {
            if (vec_ok) {
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const int n = n_base + j * 16 + q * 4;
                    old[j] = n + 3 < N ? *reinterpret_cast<const v4f*>(static_cast<const float*>(Dv) + (int64_t)m * N + n)
                                       : (v4f){0.f, 0.f, 0.f, 0.f};
                }
            }
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int n = n_base + j * 16 + q * 4;
            if (n >= N) continue;
            O* dp = D + (int64_t)m * N + n;
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = val(i, j, e);
            if (vec_ok && n + 3 < N) {
                if constexpr (DT == NTFP8_F32) {
                    v4f o = {v[0], v[1], v[2], v[3]};
                    if constexpr (kAcc) o = o + old[j];
                    // (fp32 outputs keep the ordinary store: written through they measured the same or slower)
                    *reinterpret_cast<v4f*>(dp) = o;
                } else {
                    *reinterpret_cast<uint2*>(dp) = make_uint2(OutT<DT>::pack2(v[0], v[1]), OutT<DT>::pack2(v[2], v[3]));
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

// 16 / 4 bytes per lane to global memory through a buffer descriptor; offsets past its size are dropped.  Cache policy
// of the builtin's last argument on gfx950: bit 0 = sc0, bit 1 = nt, bit 4 = sc1 (written through, as store16_through).
constexpr int kStoreThrough = 1 | 2 | 16;
__device__ __forceinline__ void reg_store16(__amdgpu_buffer_rsrc_t r, uint32_t voff, v4i data) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, data), r, voff, 0, kStoreThrough);
}
__device__ __forceinline__ void reg_store4(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t data) {
    __builtin_amdgcn_raw_buffer_store_b32(data, r, voff, 0, kStoreThrough);
}

// fp8 epilogue of one wave (layout as store_wave_tile16); returns the lane's max|r| as a bit pattern.
// Shapes: N a multiple of 16, M a multiple of 4, M N < 2^32 (the launcher sends other shapes to the small kernel).
// A lane's 4 consecutive n of a block are one word of D.  Row-major bytes: a 4 x 4 exchange of words between the
// four lane rows and four neighbouring blocks gives lane row q the 16 consecutive n of block j0 + q, one 16-byte
// store per lane and 64 contiguous bytes per output row and instruction.  Transposed bytes: a 4 x 4 byte transpose
// inside each quad of lanes (4 consecutive m) turns the word into 4 consecutive m of one n.
// All stores go through buffer descriptors of M N bytes: rows past the end fall outside and are dropped, columns
// past the end get an offset that does; nothing is predicated, which keeps the scalar registers of the epilogue
// (and with them the register budget of the K loop before it) small.
// kMask: accumulator blocks past N (and past M if `mask_rows`: A given as its transpose) hold arbitrary values,
// because an operand read through the transposing loads wraps into its next row there instead of reading zeros, and
// must stay out of the amax.  N (and M, with a transposed A) is a multiple of 16 then, so whole blocks are in or
// out, uniformly for the wave.  Rows past M of an ordinary A operand read as zeros and need no mask.
template <int F, int MI, int NJ, bool kBias = false, bool kMask = false>
__device__ __forceinline__ uint32_t store_wave_tile16_fp8(const v4f (&acc)[MI][NJ], uint8_t* __restrict__ D,
                                                          uint8_t* __restrict__ Dt, float alpha, float scale_d, bool slow,
                                                          int M, int N, int m_base, int n_base, int lane,
                                                          const float (*bv)[4] = nullptr, bool mask_rows = false) {
    auto val = [&](int i, int j, int e) -> float {
        if constexpr (kBias) return acc[i][j][e] * alpha + bv[j][e];
        else return acc[i][j][e] * alpha;
    };
    static_assert(NJ % 4 == 0, "blocks are exchanged four at a time");
    const int mrow = lane & 15, q = lane >> 4;
    uint32_t amax = 0;
    const uint32_t bytes = (uint32_t)M * (uint32_t)N;
    const __amdgpu_buffer_rsrc_t rd = make_rsrc(D, bytes);
    const __amdgpu_buffer_rsrc_t rt = make_rsrc(Dt, Dt ? bytes : 0u);
    constexpr uint32_t kDropped = 0xfffffff0u;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int m = m_base + i * 16 + mrow;
        const int mq = m & ~3;
        uint32_t w[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            if constexpr (kMask) {
                uint32_t a = amax;
                w[j] = quant4<F>(val(i, j, 0), val(i, j, 1), val(i, j, 2), val(i, j, 3), scale_d, slow, a);
                if ((!mask_rows || m_base + i * 16 < M) && n_base + j * 16 < N) amax = a;
            } else {
                w[j] = quant4<F>(val(i, j, 0), val(i, j, 1), val(i, j, 2), val(i, j, 3), scale_d, slow, amax);
            }
        }
        if (Dt) {   // uniform
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const uint32_t t = quad_transpose_bytes(w[j], lane);
                const int nt = n_base + j * 16 + q * 4 + (lane & 3);
                // nt >= N lies past the end of the [N, M] bytes by itself
                reg_store4(rt, mq < M ? (uint32_t)nt * (uint32_t)M + (uint32_t)mq : kDropped, t);
            }
        }
#pragma unroll
        for (int j0 = 0; j0 < NJ; j0 += 4) {
            uint32_t x0 = w[j0], x1 = w[j0 + 1], x2 = w[j0 + 2], x3 = w[j0 + 3];
            swap_rows16(x0, x1);   // lane rows 1, 3 of a word <-> rows 0, 2 of the next block's word
            swap_rows16(x2, x3);
            swap_halves(x0, x2);   // lane rows 2, 3 <-> rows 0, 1 two blocks further on
            swap_halves(x1, x3);
            // lane row q now holds n 0-3, 4-7, 8-11, 12-15 of block j0 + q; m >= M lies past the end by itself
            const int n = n_base + (j0 + q) * 16;
            reg_store16(rd, n < N ? (uint32_t)m * (uint32_t)N + (uint32_t)n : kDropped, (v4i){(int)x0, (int)x1, (int)x2, (int)x3});
        }
    }
    return amax;
}

// Launch geometry, computed on the host.  The first `full_blocks` tiles (in grouped order) are computed
// whole by the MI = 8 kernel.  If the tile count leaves a partial last round over the CUs, the
// remaining `tail_tiles` tiles are cut into two 128-row halves and computed by a second launch of
// the MI = 4 kernel with 2 tail_tiles workgroups, so that the last round is half as long.
//
// One launch can carry several independent GEMMs of the same operand formats (the dgrad and wgrad of a
// layer, say): their tiles form one list, longest K first, so that the rounds of one problem fill up
// with tiles of the next instead of ending in a partial round and a kernel boundary each.
struct BigProblem {
    const uint8_t* A;
    const uint8_t* B;
    void* D;
    const float* scale_a;
    const float* scale_b;
    int M, N, K;
    int tiles_m, tiles_n;   // 256 x 256 tiles
    int tile_begin;         // position of this problem's first tile in the launch's tile list
    int d_dtype;            // NTFP8_F32 / NTFP8_F16 / NTFP8_BF16 / NTFP8_OUT_E4M3 / NTFP8_OUT_E5M2
    int accumulate;         // fp32 outputs only: D += result
    Fp8Out fp8;             // fp8 outputs only
    GemmExtras ex;          // bias, inverse-scale flag
    int at;                 // A is given as [K, M] row-major (its transpose); kBT launches only
};
constexpr int kBigMaxProblems = 4;
struct BigLaunch {
    BigProblem p[kBigMaxProblems];
    int count;
    int full_blocks;        // tiles (of the whole list) computed whole
    int tail_tiles;         // tiles at the end of the list computed as two halves
    int round_size;         // workgroups resident at once: one per CU
};

// MI = 8 needs the whole register file of a SIMD for one wave (256 accumulators + fragments).  The
// MI = 4 variant is held to half of it by declaring a launch bound of twice its real workgroup
// size: given more registers than it needs, the compiler keeps its accumulators in a second
// register set and copies them back and forth inside the K loop.
// kFp8Out: every problem of the launch has an fp8 output (a kernel of its own: the other outputs' code stays as
// the register allocator likes it).
// kBT: the B operands are given transposed, as [K, N] row-major bytes (what a caller has when the reduction index is
// the row index of its tensor: W for dgrad, X for wgrad).  A K-tile of such an operand lies in LDS as it lies in
// memory, 128 rows of k with 256 bytes of n each, and the 16 x 128 fragments are gathered with the transposing
// LDS read DS_READ_B64_TR_B8: within 16 lanes, lane 2 u supplies the address of 8 bytes that lanes 0-7 receive one
// byte each of (byte i to lane i, as their byte u), lane 2 u + 1 the same for lanes 8-15.  With lane 2 u on row
// k0 + u, columns c .. c + 7, and lane 2 u + 1 on the same row, columns c + 8 .. c + 15, lane r receives k0 .. k0 + 7
// of column c + r: a quarter of its fragment.  16-byte chunk c of row k is stored at chunk
// c ^ ((k mod 8) | 8 (k / 32 mod 2)), so that the 8 rows one read touches (and the two 16-lane groups that go
// through LDS together) use different banks.
template <int FA, int FB, int MI, bool kFp8Out = false, bool kBT = false>
__global__ __launch_bounds__(MI == 8 ? kBigThreads : 2 * kBigThreads)
void gemm_nt_big_kernel(const BigLaunch L) {
    // whole tiles: 2 stages of 64 KB; half tiles: 3 stages of 48 KB (their loads go straight to LDS and need the
    // extra stage to have two K-tiles of flight time, see below)
    constexpr int NS = MI == 8 ? 2 : 3;
    __shared__ __attribute__((aligned(1024))) uint8_t sA[NS][32 * MI * kBK];
    __shared__ __attribute__((aligned(1024))) uint8_t sB[NS][kBigN * kBK];

    // ---- which tile (or half tile) of which problem is this workgroup's ----------------------------
    [[maybe_unused]] unsigned long long st_entry = 0, st_first = 0, st_loop = 0, cy_first = 0, cy_loop = 0;
    NTFP8_STAMP(st_entry);
    int pid = blockIdx.x;
    int half = 0;
    if constexpr (MI == 8) {
        // Workgroups are dealt to the XCDs round robin.  Within each round of `round_size` workgroups (one per
        // CU) an XCD gets a contiguous run of the tile list, so its L2 sees few operand panels; across rounds
        // the list is walked in order, so that the long tiles at its head start together on the whole chip.
        const int round0 = (pid / L.round_size) * L.round_size;
        const int in_round = min(L.round_size, L.full_blocks - round0);
        const int local = pid - round0;
#ifdef NTFP8_STAMPS
        if (g_plain_tile_order) {
        } else
#endif
        if (in_round % kXcds == 0) pid = round0 + (local % kXcds) * (in_round / kXcds) + local / kXcds;
    } else {
        const int nb = 2 * L.tail_tiles;
        if (nb % kXcds == 0) pid = (pid % kXcds) * (nb / kXcds) + pid / kXcds;
        half = pid & 1;
        pid = L.full_blocks + (pid >> 1);
    }
    int which = 0;
#pragma unroll
    for (int i = 1; i < kBigMaxProblems; ++i)
        if (i < L.count && pid >= L.p[i].tile_begin) which = i;
    const BigProblem& P = L.p[which];
    const uint8_t* __restrict__ A = P.A;
    const uint8_t* __restrict__ B = P.B;
    void* __restrict__ Dv = P.D;
    const int M = P.M, N = P.N, K = P.K;
    pid -= P.tile_begin;
    int pid_m, pid_n;
    {
        const int in_group = kGroupM * P.tiles_n;
        const int group = pid / in_group;
        const int first_m = group * kGroupM;
        const int gsz = min(P.tiles_m - first_m, kGroupM);
        pid_m = first_m + (pid % in_group) % gsz;
        pid_n = (pid % in_group) / gsz;
    }
    const int n0 = pid_n * kBigN;
    const int m0 = pid_m * 256 + half * 128;
    if (m0 >= M) return;   // second half of a bottom-edge tile with nothing in it (uniform for the workgroup)

    const int t = threadIdx.x;
    const int lane = t & 63;
    // the wave index as a scalar: LDS destinations of the loads (M0) and every other per-wave offset then
    // live in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(A, (uint32_t)((int64_t)M * K));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(B, (uint32_t)((int64_t)N * K));
    const int KT = (K + kBK - 1) / kBK;   // >= 2 (host)
    // A wave-level load fills 8 tile rows (1 KB of LDS, lane i at byte 16 i); the lane landing on
    // chunk position p of row r fetches global chunk p ^ swz16(r).  For the rows a lane serves
    // (8 (wave + 4 i) + lane / 8) that is the same chunk for every i.
    const int ld_kc = ((lane & 7) ^ (lane >> 3) ^ (wave & 1)) << 4;
    // chunks of the last K-tile at k >= K must read as zero, not as the start of the next row
    const bool tail_dead = (KT - 1) * kBK + ld_kc >= K;
    const float alpha = descale_factor(P.scale_a, P.scale_b, P.ex.scale_inv);

    constexpr int LA = MI * 2 * 16 / 8 / kBigWaves;  // wave-level loads of the A tile per wave per stage
    constexpr int NJe = MI == 8 ? kColumns : kBigNJ;   // block columns the K loop computes (8 outside experiments)
    constexpr int LB = MI == 8 ? kBigLB - (kBigNJ - NJe) : kBigLB;
    constexpr int NL = LA + LB;                      // loads per wave per K-tile
    static_assert(NL % 4 == 0 || NJe != kBigNJ, "the loads are queued in four equal portions");
    const int wm = (wave >> 1) * (MI * 16), wn = (wave & 1) * 128;

    v4f acc[MI][kBigNJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < kBigNJ; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
    // (experiment builds only: the accumulators of the 32 x 32 instruction shape)
    [[maybe_unused]] v16f big[kMfma32 ? MI / 2 : 1][kMfma32 ? kBigNJ / 2 : 1];
    if constexpr (kMfma32) {
#pragma unroll
        for (int i = 0; i < MI / 2; ++i)
#pragma unroll
            for (int j = 0; j < kBigNJ / 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) big[i][j][e] = 0.f;
    }
    // one step of the MFMA loop: block (i, j) of the wave tile; in the 32 x 32 experiment every fourth step issues the
    // two instructions (K = 2 x 64) of the 32 x 32 block it belongs to, on whatever fragments are at hand
    auto mma = [&](int i, int j, const v8i b, const v8i a) {
        if constexpr (kMfma32) {
            if (!(i & 1) && !(j & 1)) {
                big[i >> 1][j >> 1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a, big[i >> 1][j >> 1], FB, FA, 0, 0, 0, 0);
                big[i >> 1][j >> 1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, big[i >> 1][j >> 1], FB, FA, 0, 0, 0, 0);
            }
        } else {
            acc[i][j] = mfma_16x16x128<FA, FB>(b, a, acc[i][j]);
        }
    };

    // The K loop.  kAT: the A operand is given as its transpose, a [K, M] tensor (what wgrad has of dY: its reduction
    // index, the token, is the row index).  Its K-tiles lie in LDS as they lie in memory, 128 rows of k with 256 (whole
    // tiles) or 128 (half tiles) bytes of m each, and the 16 x 128 fragments are gathered with the transposing LDS read,
    // exactly as for a transposed B operand.  Operand layout is a property of the problem, decided per workgroup: a
    // launch mixes dgrad (A plain) and wgrad (A transposed) tiles.
    auto kloop = [&](auto at_tag) {
        constexpr bool kAT = decltype(at_tag)::value;
        uint32_t a_off[LA], b_off[LB];
#pragma unroll
        for (int i = 0; i < LA; ++i) {
            if constexpr (kAT && MI == 8) {
                // as the transposed B below: 4 rows of k per wave-level load, 16 chunks of m each
                const int k = (wave + kBigWaves * i) * 4 + (lane >> 4);
                const int chunk = (lane & 15) ^ ((k & 7) | (((k >> 5) & 1) << 3));
                a_off[i] = (uint32_t)k * (uint32_t)M + (uint32_t)(m0 + chunk * 16);
            } else if constexpr (kAT) {
                // half tiles: 128 bytes of m per row of k, 8 rows of k per wave-level load; chunk c of row k is stored
                // at chunk c ^ ((k / 2 mod 4) | 4 (k / 32 mod 2)): the 8 rows one transposing read touches, and the
                // two 16-lane groups that go through LDS together, then use 16 different 16-byte bank groups
                const int k = (wave + kBigWaves * i) * 8 + (lane >> 3);
                const int chunk = (lane & 7) ^ (((k >> 1) & 3) | (((k >> 5) & 1) << 2));
                a_off[i] = (uint32_t)k * (uint32_t)M + (uint32_t)(m0 + chunk * 16);
            } else {
                // rows >= M fall past the descriptor: zeros
                a_off[i] = (uint32_t)(m0 + (wave + kBigWaves * i) * 8 + (lane >> 3)) * (uint32_t)K + ld_kc;
            }
        }
#pragma unroll
        for (int i = 0; i < LB; ++i) {
            if constexpr (kBT) {
                // a wave-level load fills 4 rows of k (lane / 16) with 16 chunks of n (lane % 16) each; rows k >= K fall
                // past the descriptor (zeros); chunks past N wrap into the next row and only reach outputs that are
                // never stored
                const int k = (wave + kBigWaves * i) * 4 + (lane >> 4);
                const int chunk = (lane & 15) ^ ((k & 7) | (((k >> 5) & 1) << 3));
                b_off[i] = (uint32_t)k * (uint32_t)N + (uint32_t)(n0 + chunk * 16);
            } else {
                b_off[i] = (uint32_t)(n0 + (wave + kBigWaves * i) * 8 + (lane >> 3)) * (uint32_t)K + ld_kc;
            }
        }
        // byte distance between K-tiles in memory
        const int a_step = kAT ? kBK * M : kBK, b_step = kBT ? kBK * N : kBK;

        // load number `l` (0 .. NL-1, A loads first) of K-tile `ktile` straight into its LDS stage, ktile mod NS
        auto issue = [&](int ktile, int l) {
            const int s = ktile % NS;
            if (l < LA)
                lds_load16(ra, (lds_ptr)(uintptr_t)&sA[s][(wave + kBigWaves * l) * 1024], a_off[l], ktile * a_step);
            else
                lds_load16(rb, (lds_ptr)(uintptr_t)&sB[s][(wave + kBigWaves * (l - LA)) * 1024], b_off[l - LA], ktile * b_step);
        };
        // Called once, before the first load of the last K-tile is queued (no other tile is loaded after it):
        // lanes whose chunk lies at k >= K get an offset past the descriptor and so read zeros.
        auto poison_tail = [&]() {
            if (tail_dead) {
                if constexpr (!kAT) {   // (rows k >= K of a transposed operand fall past its descriptor by themselves)
#pragma unroll
                    for (int i = 0; i < LA; ++i) a_off[i] = 0xfffffff0u;
                }
                if constexpr (!kBT) {
#pragma unroll
                    for (int i = 0; i < LB; ++i) b_off[i] = 0xfffffff0u;
                }
            }
        };

        // fragment reads: lane -> row (lane % 16) of a 16-row block, two 16-byte chunks 2 (lane / 16) + {0, 1};
        // block i of the wave is 16 i rows = 2048 i bytes further on (the swizzle only looks at row bits 0-3)
        const int frow = lane & 15;
        const int fk = (lane >> 4) * 2;
        const int a_rd0 = lds_off16(wm + frow, fk), a_rd1 = lds_off16(wm + frow, fk + 1);
        const int b_rd0 = lds_off16(wn + frow, fk), b_rd1 = lds_off16(wn + frow, fk + 1);
        // transposed operands: lane u of a 16-lane group (which serves k 32 (lane / 16) .. + 31) addresses row k0 + u / 2,
        // half u % 2 of the block's 16-byte chunk; quarter t of the fragment is k0 = 32 (lane / 16) + 8 t
        const int bt_row = (lane & 15) >> 1;
        const int bt_base = ((lane >> 4) * 32 + bt_row) * 256 + ((((wave & 1) ^ ((lane >> 4) & 1))) << 7) + (lane & 1) * 8;
        const int bt_x = bt_row << 4;
        // the same for A: the wave's blocks are chunks 8 (wave / 2) + i of a 256-byte row (whole tiles), chunks
        // 4 (wave / 2) + i of a 128-byte row (half tiles, swizzle (k / 2 mod 4) | 4 (k / 32 mod 2))
        const int at_base = MI == 8 ? ((lane >> 4) * 32 + bt_row) * 256 + ((((wave >> 1) ^ ((lane >> 4) & 1))) << 7) + (lane & 1) * 8
                                    : ((lane >> 4) * 32 + bt_row) * 128 + ((((wave >> 1) ^ ((lane >> 4) & 1))) << 6) + (lane & 1) * 8;
        const int at_x = MI == 8 ? bt_row << 4 : ((bt_row >> 1) & 3) << 4;
        constexpr int at_pitch = MI == 8 ? 256 : 128;
        // half h (0 / 1) of a fragment = one 128-bit LDS read, or two transposing 64-bit reads
        auto rd_a = [&](int s, int i, int h) -> v4i {
            if constexpr (kAT) {
                typedef int v2i __attribute__((ext_vector_type(2)));
                typedef __attribute__((address_space(3))) v2i* tr_ptr;
                int x = at_x;
                if constexpr (MI == 4) asm volatile("" : "+v"(x));
                uint8_t* p = &sA[s][at_base + ((i << 4) ^ x) + h * (2 * 8 * at_pitch)];
                const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((tr_ptr)p);
                const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((tr_ptr)(p + 8 * at_pitch));
                return (v4i){lo.x, lo.y, hi.x, hi.y};
            } else {
                return *reinterpret_cast<const v4i*>(&sA[s][(h ? a_rd1 : a_rd0) + i * 2048]);
            }
        };
        auto rd_b = [&](int s, int j, int h) -> v4i {
            if constexpr (kBT) {
                typedef int v2i __attribute__((ext_vector_type(2)));
                typedef __attribute__((address_space(3))) v2i* tr_ptr;
                // (address-space cast, not a round trip through an integer: the compiler must see that these reads
                // come from sB, or it waits for every direct-to-LDS load in flight before each of them)
                int x = bt_x;
                // half tiles: recomputed at every use, eight block offsets kept across the K loop do not fit their
                // register budget; whole tiles keep them (1 % faster than recomputing)
                if constexpr (MI == 4) asm volatile("" : "+v"(x));
                uint8_t* p = &sB[s][bt_base + ((j << 4) ^ x) + h * (2 * 8 * 256)];
                const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((tr_ptr)p);
                const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((tr_ptr)(p + 8 * 256));
                return (v4i){lo.x, lo.y, hi.x, hi.y};
            } else {
                return *reinterpret_cast<const v4i*>(&sB[s][(h ? b_rd1 : b_rd0) + j * 2048]);
            }
        };
        auto frag = [](const v4i (&x)[2]) -> v8i { return (v8i){x[0].x, x[0].y, x[0].z, x[0].w, x[1].x, x[1].y, x[1].z, x[1].w}; };

        v4i fa[MI][2], fb[4][2];

        // A K-tile kt lives in LDS stage kt mod NS and is computed in two parts:
        //   front(kt): MFMA groups 0-5.  Entered with fa[] = the tile's A fragments and fb[0], fb[1] = its first
        //              two B fragments; streams B fragments 2..7; ends with the barrier that publishes tile
        //              kt + 1 and releases the stage of tile kt.
        //   back(kt):  MFMA groups 6-7, interleaved per A fragment; refills fa[] / fb[0], fb[1] from tile kt + 1.
        // The K loop runs back(kt); front(kt + 1), so that its back edge sits right behind the barrier, where no
        // LDS read is outstanding.  With direct-to-LDS loads (half tiles) the stage released by the barrier of
        // tile kt is refilled with tile kt + NS between that barrier and the next: half of the loads under
        // back(kt), the rest under groups 0-1 of front(kt + 1).
        //
        // An MFMA occupies the matrix pipe for 32 cycles and the wave issues in order, so whatever stands between
        // two MFMAs must issue within that time or the pipe idles.  The code below therefore puts at most one
        // memory instruction (two LDS reads at most) behind each MFMA, and a scheduling fence behind each such
        // pair keeps the compiler from regrouping them.
        constexpr int kBackLoads = NL / 2;
        constexpr int kFrontLoads = NL - kBackLoads;   // half under group 0, half under group 1
        // loads: queue the second half of tile kt + NS - 1; WAIT (>= 0): barrier, after all but the newest WAIT
        // loads of this wave have landed (-1: no barrier)
        auto front = [&](auto loads_tag, auto wait_tag, int kt) {
            constexpr bool loads = decltype(loads_tag)::value;
            constexpr int WAIT = decltype(wait_tag)::value;
            const int s = kt % NS;
            sched_fence();
#pragma unroll
            for (int j = 0; j < 6; ++j) {
                int l = kBackLoads + j * (kFrontLoads / 2);           // next load to queue
                const int lend = (loads && j < 2) ? l + kFrontLoads / 2 : l;
#pragma unroll
                for (int i = 0; i < MI; ++i) {
                    mma(i, j, frag(fb[j & 3]), frag(fa[i]));
                    if (i == 0) fb[(j + 2) & 3][0] = rd_b(s, j + 2, 0);
                    else if (i == 2) fb[(j + 2) & 3][1] = rd_b(s, j + 2, 1);
                    else if (l < lend) issue(kt + NS - 1, l++);
                    if (i == MI - 1) {   // whatever did not get a slot of its own
                        for (; l < lend; ++l) issue(kt + NS - 1, l);
                    }
                    sched_fence();
                }
            }
            if constexpr (WAIT >= 0) {
                // Every fragment of tile kt is in registers (or in flight): after the barrier its stage may be
                // overwritten, and tile kt + 1 is complete in the next stage.
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(WAIT) : "memory");
                wg_barrier();
            }
        };
        auto back = [&](auto loads_tag, auto prefetch_tag, int kt) {
            constexpr bool loads = decltype(loads_tag)::value, prefetch = decltype(prefetch_tag)::value;
            const int s1 = (kt + 1) % NS;
            sched_fence();
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                // fa[i] is dead after its two MFMAs; it is refilled with the fragment of the next tile one step later
                mma(i, NJe - 2, frag(fb[(NJe - 2) & 3]), frag(fa[i]));
                if (prefetch && !kNoAReads && i > 0) {
                    fa[i - 1][0] = rd_a(s1, i - 1, 0);
                    fa[i - 1][1] = rd_a(s1, i - 1, 1);
                }
                sched_fence();
                mma(i, NJe - 1, frag(fb[(NJe - 1) & 3]), frag(fa[i]));
                if constexpr (loads) {   // loads [i kBackLoads / MI, (i + 1) kBackLoads / MI) ride on this step
#pragma unroll
                    for (int l = i * kBackLoads / MI; l < (i + 1) * kBackLoads / MI; ++l) issue(kt + NS, l);
                }
                if (prefetch && !kNoBReads && i < 4) fb[i >> 1][i & 1] = rd_b(s1, i >> 1, i & 1);
                sched_fence();
            }
            if constexpr (prefetch && !kNoAReads) {
                fa[MI - 1][0] = rd_a(s1, MI - 1, 0);
                fa[MI - 1][1] = rd_a(s1, MI - 1, 1);
            }
            sched_fence();
        };
        using Yes = std::true_type;
        using No = std::false_type;

        if constexpr (MI == 8) {
            // ---- whole tiles: loads staged through registers ------------------------------------------
            // g[] always holds one K-tile in flight.  front(f) runs between the barriers B(f-1) and B(f); there
            // g[l] (tile f + 1, requested one K-tile earlier) is written to the stage released by B(f-1) and
            // at once re-requested for tile f + 2.  Every load so has a full K-tile of MFMA time to arrive
            // whatever its position, and the requests are spread evenly over the K-tile; with direct-to-LDS
            // loads (which can only be issued once their stage is free) operands that come from HBM rather
            // than from the memory-side cache stalled the barrier.
            v4i g[NL];
            const int wr_lane = wave * 1024 + lane * 16;   // a wave-level load covers 1 KB of a stage: 16 bytes per lane
            auto load_now = [&](int ktile, int l) {
                g[l] = l < LA ? reg_load16(ra, a_off[l], ktile * a_step) : reg_load16(rb, b_off[l - LA], ktile * b_step);
            };
            if constexpr (kNoLoads) {
                // one real K-tile, deposited again and again: operand bytes of the real distribution (what the matrix
                // cores draw depends on the data: zeros would make this build look far cheaper than it is)
#pragma unroll
                for (int l = 0; l < NL; ++l) load_now(0, l);
            }
            auto request = [&](int ktile, int l) {
                if constexpr (!kNoLoads) load_now(ktile, l);
            };
            auto deposit = [&](int s, int l) {
                if constexpr (kNoDeposits) return;
                if (l < LA) *reinterpret_cast<v4i*>(&sA[s][wr_lane + l * (kBigWaves * 1024)]) = g[l];
                else *reinterpret_cast<v4i*>(&sB[s][wr_lane + (l - LA) * (kBigWaves * 1024)]) = g[l];
            };
            // MFMA groups 0-5 of tile f.  W: deposit tile f + 1; L: request tile f + 2; B: barrier that publishes
            // tile f + 1.  A group has 8 MFMA slots: two carry the LDS reads of B fragment j + 2, the other six
            // take deposit / request pairs (three pairs in groups 0-4, the sixteenth pair in group 5).
            auto front_st = [&](auto w_tag, auto l_tag, auto b_tag, int f) {
                constexpr bool W = decltype(w_tag)::value, L = decltype(l_tag)::value, B = decltype(b_tag)::value;
                const int s = f & 1;
                sched_fence();
                int l = 0;
#pragma unroll
                for (int j = 0; j < NJe - 2; ++j) {
#pragma unroll
                    for (int i = 0; i < MI; ++i) {
                        mma(i, j, frag(fb[j & 3]), frag(fa[i]));
                        if (i == 0) { if constexpr (!kNoBReads) fb[(j + 2) & 3][0] = rd_b(s, j + 2, 0); }
                        else if (i == 2) { if constexpr (!kNoBReads) fb[(j + 2) & 3][1] = rd_b(s, j + 2, 1); }
                        else if (l < NL) {
                            const bool second = i == 3 || i == 5 || i == 7;   // slots 1,3 / 4,5 / 6,7 form the pairs
                            if (!second) { if (W) deposit(s ^ 1, l); }
                            else { if (L) request(f + 2, l); ++l; }
                        }
                        sched_fence();
                    }
                }
                if constexpr (B) {
                    // Every fragment of tile f is in registers (or in flight) and this wave's part of tile f + 1 is
                    // written: after the barrier stage s may be overwritten and tile f + 1 is complete in s ^ 1.
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    // the first front publishes tile 1, which the prologue sent straight to LDS: its loads are
                    // older than the NL requests of tile 2 queued above
                    if constexpr (!W) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(L ? NL : 0) : "memory");
                    if constexpr (!kNoBarrier) wg_barrier();
                    if constexpr (kIdle > 0) __builtin_amdgcn_s_sleep(kIdle);
                }
            };
            // prologue: tiles 0 and 1 straight into LDS
#pragma unroll
            for (int l = 0; l < NL; ++l) issue(0, l);
            if (KT == 2) poison_tail();
#pragma unroll
            for (int l = 0; l < NL; ++l) issue(1, l);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NL) : "memory");   // tile 0 has landed, tile 1 may still be in flight
            wg_barrier();
            NTFP8_STAMP(st_first);
            NTFP8_CYCLES(cy_first);
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                fa[i][0] = rd_a(0, i, 0);
                fa[i][1] = rd_a(0, i, 1);
            }
#pragma unroll
            for (int h = 0; h < 4; ++h) fb[h >> 1][h & 1] = rd_b(0, h >> 1, h & 1);

            // (poison_tail() runs right before the front that requests the last tile, KT - 1 = f + 2)
            if (KT == 3) poison_tail();
            if (KT > 2) front_st(No{}, Yes{}, Yes{}, 0);   // nothing to deposit: tile 1 is on its way to LDS already
            else front_st(No{}, No{}, Yes{}, 0);
            int f = 1;
            for (; f + 3 < KT; ++f) {
                back(No{}, Yes{}, f - 1);
                front_st(Yes{}, Yes{}, Yes{}, f);
            }
            if (f + 2 < KT) {   // f = KT - 3 >= 1
                poison_tail();
                back(No{}, Yes{}, f - 1);
                front_st(Yes{}, Yes{}, Yes{}, f);
                ++f;
            }
            if (f + 1 < KT) {   // f = KT - 2 >= 1: the last tile is deposited, nothing left to request
                back(No{}, Yes{}, f - 1);
                front_st(Yes{}, No{}, Yes{}, f);
                ++f;
            }
            back(No{}, Yes{}, f - 1);   // f = KT - 1
            front_st(No{}, No{}, No{}, f);
            back(No{}, No{}, f);
        } else {
        // ---- half tiles: loads go straight into LDS (the register budget has no room for staging) --------
        // Three stages: the loads of tile t are queued while tile t - 3's stage is the one just released, i.e.
        // two K-tiles before tile t is published.  A half-tile K-tile is only 32 MFMAs (about 0.55 us): with
        // two stages the loads had half a K-tile to arrive, less than an L2 hit takes.
        using Wait = std::integral_constant<int, NL>;   // the NL loads of the newest tile may still be in flight
        using WaitAll = std::integral_constant<int, 0>;
        using NoBarrier = std::integral_constant<int, -1>;
        // prologue: tiles 0, 1 and (if there is one) 2
#pragma unroll
        for (int l = 0; l < NL; ++l) issue(0, l);
        if (KT == 2) poison_tail();
#pragma unroll
        for (int l = 0; l < NL; ++l) issue(1, l);
        if (KT > 2) {
            if (KT == 3) poison_tail();
#pragma unroll
            for (int l = 0; l < NL; ++l) issue(2, l);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NL) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NL) : "memory");
        }
        wg_barrier();
        NTFP8_STAMP(st_first);
        NTFP8_CYCLES(cy_first);
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            fa[i][0] = rd_a(0, i, 0);
            fa[i][1] = rd_a(0, i, 1);
        }
#pragma unroll
        for (int h = 0; h < 4; ++h) fb[h >> 1][h & 1] = rd_b(0, h >> 1, h & 1);

        // front(0) queues nothing (tile 3 goes into the stage that front(0) itself still reads)
        if (KT > 2) front(No{}, Wait{}, 0);
        else front(No{}, WaitAll{}, 0);
        int f = 1;
        for (; f + 2 < KT; ++f) {   // tile f + 2 is loaded during back(f - 1); front(f)
            if (f + 3 == KT) poison_tail();
            back(Yes{}, Yes{}, f - 1);
            front(Yes{}, Wait{}, f);
        }
        if (f + 1 < KT) {   // f = KT - 2 >= 1: nothing left to load
            back(No{}, Yes{}, f - 1);
            front(No{}, WaitAll{}, f);
            ++f;
        }
        back(No{}, Yes{}, f - 1);   // f = KT - 1
        front(No{}, NoBarrier{}, f);
        back(No{}, No{}, f);
        }
    };
    if constexpr (kBT) {
        if (P.at) kloop(std::true_type{});   // uniform for the workgroup
        else kloop(std::false_type{});
    } else {
        kloop(std::false_type{});
    }

    NTFP8_STAMP(st_loop);
    NTFP8_CYCLES(cy_loop);
    if constexpr (kMfma32) {   // the experiment's results must reach memory, or its MFMAs are dead code
#pragma unroll
        for (int i = 0; i < MI / 2; ++i)
#pragma unroll
            for (int j = 0; j < kBigNJ / 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[2 * i + (e >> 3)][2 * j + ((e >> 2) & 1)][e & 3] += big[i][j][e];
    }
    {
        // output type, accumulation and bias are properties of the problem, not of the kernel (fp8 outputs apart)
        auto epilogue = [&](auto bias_tag, const float (*bv)[4]) {
            constexpr bool kBias = decltype(bias_tag)::value;
            if constexpr (kFp8Out) {
                const float scale_d = *P.fp8.scale;
                const bool slow = scale_is_degenerate(scale_d);
                const uint32_t amax =
                    P.d_dtype == NTFP8_OUT_E4M3
                        ? store_wave_tile16_fp8<kE4M3, MI, kBigNJ, kBias, kBT>(acc, static_cast<uint8_t*>(Dv), P.fp8.Dt, alpha, scale_d,
                                                                          slow, M, N, m0 + wm, n0 + wn, lane, bv, kBT && P.at)
                        : store_wave_tile16_fp8<kE5M2, MI, kBigNJ, kBias, kBT>(acc, static_cast<uint8_t*>(Dv), P.fp8.Dt, alpha, scale_d,
                                                                          slow, M, N, m0 + wm, n0 + wn, lane, bv, kBT && P.at);
                publish_amax(amax, P.fp8.ws);
            } else if (P.d_dtype == NTFP8_BF16) {
                store_wave_tile16<NTFP8_BF16, false, MI, kBigNJ, kBias>(acc, Dv, alpha, M, N, m0 + wm, n0 + wn, lane, bv);
            } else if (P.d_dtype == NTFP8_F16) {
                store_wave_tile16<NTFP8_F16, false, MI, kBigNJ, kBias>(acc, Dv, alpha, M, N, m0 + wm, n0 + wn, lane, bv);
            } else if (P.accumulate) {
                store_wave_tile16<NTFP8_F32, true, MI, kBigNJ, kBias>(acc, Dv, alpha, M, N, m0 + wm, n0 + wn, lane, bv);
            } else {
                store_wave_tile16<NTFP8_F32, false, MI, kBigNJ, kBias>(acc, Dv, alpha, M, N, m0 + wm, n0 + wn, lane, bv);
            }
        };
        // (no bias together with a transposed B operand: the backward GEMMs that read one have none, and their
        // instantiation has no registers to spare for the second set of epilogues)
        bool with_bias = false;
        if constexpr (!kBT) with_bias = P.ex.bias != nullptr;   // uniform
        if (with_bias) {
            float bv[kBigNJ][4];
            load_bias16<kBigNJ>(bv, P.ex.bias, P.ex.bias_dtype, N, n0 + wn, lane);
            epilogue(std::true_type{}, bv);
        } else {
            epilogue(std::false_type{}, nullptr);
        }
    }
#ifdef NTFP8_STAMPS
    {
        const unsigned long long st_issued = wall_clock64();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const unsigned long long st_drained = wall_clock64();
        if (threadIdx.x == 0) {
            unsigned long long* o = g_stamps + (size_t)(blockIdx.x % kStampSlots) * 8;
            o[0] = st_entry, o[1] = st_first, o[2] = st_loop, o[3] = st_issued, o[4] = st_drained;
            // HW_ID (cu 11:8, sh 12, se 15:13) | XCC_ID << 32 | MI << 40
            o[5] = (unsigned long long)__builtin_amdgcn_s_getreg((31 << 11) | 4) |
                   ((unsigned long long)(__builtin_amdgcn_s_getreg((31 << 11) | 20) & 0xf) << 32) | ((unsigned long long)MI << 40);
            o[6] = cy_first, o[7] = cy_loop;
        }
    }
#endif
}

}  // namespace ntfp8
