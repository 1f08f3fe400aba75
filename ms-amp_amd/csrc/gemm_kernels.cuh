// FP8 GEMM for gfx950: D[N][M] = (B[N][K] . A[M][K]^T) * a_scale_inv * b_scale_inv (+bias) (+D).
//
// Both operands are K-contiguous, which is the layout the 32x32x64 FP8 MFMA wants: a lane holds
// 32 consecutive K bytes of one row.  Inside the kernel the operand that supplies D's rows is X
// (= B of the API, N rows) and the one that supplies D's columns is Y (= A of the API, M rows).
//
// Block tile BR x BC over K slices of 128 bytes, four wavefronts in a 2 x 2 arrangement, LDS
// double-buffered with a 16-byte-chunk XOR swizzle that keeps both the 128-bit tile writes and
// the 128-bit fragment reads off shared banks.  Tiles are handed to workgroups so that the
// workgroups of one XCD (one L2) work on neighbouring tiles.
#pragma once
#include "common.cuh"
#include "gemm_call.h"

#include <atomic>

#include <type_traits>

namespace msamp {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kGemmThreads = 256;

__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row & 7) ^ ((row >> 3) & 1)); }

template <int ROWS, bool KGUARD>
struct TileLoader {
    static constexpr int kIters = ROWS * 8 / kGemmThreads;
    uint4 regs[kIters];

    // rows beyond `nrows` are clamped (their products land in output rows that are never stored);
    // with KGUARD, K chunks beyond `K` read as zero (without it K is a multiple of the stage).
    __device__ __forceinline__ void gload(const uint8_t* __restrict__ base, int row0, int nrows, int K, int k0) {
        const int t = threadIdx.x;
#pragma unroll
        for (int i = 0; i < kIters; ++i) {
            const int idx = t + kGemmThreads * i;
            const int r = idx >> 3, c = idx & 7;
            int gr = row0 + r;
            gr = gr < nrows ? gr : nrows - 1;
            const int kk = k0 + c * 16;
            if (!KGUARD || kk < K) {
                regs[i] = *reinterpret_cast<const uint4*>(base + static_cast<size_t>(gr) * K + kk);
            } else {
                regs[i] = make_uint4(0, 0, 0, 0);
            }
        }
    }
    __device__ __forceinline__ void lstore(uint8_t* lds) const {
        const int t = threadIdx.x;
#pragma unroll
        for (int i = 0; i < kIters; ++i) {
            const int idx = t + kGemmThreads * i;
            const int r = idx >> 3, c = idx & 7;
            *reinterpret_cast<uint4*>(lds + r * kBK + (swz(r, c) << 4)) = regs[i];
        }
    }
};

// 32 K-bytes of one tile row for this lane: chunks 2*kc, 2*kc+1 of the 128-byte row
__device__ __forceinline__ v8i read_frag(const uint8_t* lds, int row, int kc) {
    const v4i lo = *reinterpret_cast<const v4i*>(lds + row * kBK + (swz(row, 2 * kc) << 4));
    const v4i hi = *reinterpret_cast<const v4i*>(lds + row * kBK + (swz(row, 2 * kc + 1) << 4));
    v8i f;
    f[0] = lo[0], f[1] = lo[1], f[2] = lo[2], f[3] = lo[3];
    f[4] = hi[0], f[5] = hi[1], f[6] = hi[2], f[7] = hi[3];
    return f;
}

typedef float v4f __attribute__((ext_vector_type(4)));

// 16 x 16 x 128 FP8 MFMA (the non-scaled form: block scales 0).  On this part it sustains about a tenth more
// throughput under the power limit than the 32 x 32 x 64 form on the same data.
template <int XF, int YF>
__device__ __forceinline__ v4f mfma16(const v8i& x, const v8i& y, const v4f& c) {
    constexpr int cb = (XF == MSAMP_DT_E4M3) ? 0 : 1;
    constexpr int bl = (YF == MSAMP_DT_E4M3) ? 0 : 1;
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(x, y, c, cb, bl, 0, 0, 0, 0);
}

template <typename OT>
__device__ __forceinline__ void store_out(OT* p, float v, bool accumulate) {
    if (accumulate) v += Elem<OT>::load(p);
    Elem<OT>::store(p, v);
}

__device__ __forceinline__ float load_bias(const void* bias, int dt, int i) {
    if (dt == MSAMP_DT_F32) return static_cast<const float*>(bias)[i];
    if (dt == MSAMP_DT_F16) return f16_bits_to_float(static_cast<const uint16_t*>(bias)[i]);
    return bf16_bits_to_float(static_cast<const uint16_t*>(bias)[i]);
}

// workgroup id -> tile, keeping the workgroups of one XCD on adjacent tiles and walking groups of `kGroup` tile rows
// column by column (or, with `by_columns`, groups of tile columns row by row): the 32 CUs of an XCD then work on an
// 8 x 4 patch of tiles and share its 12 operand panels through that L2.
__device__ __forceinline__ void tile_of_id(int id, int tiles_r, int tiles_c, bool by_columns, bool wide, int& tr, int& tc) {
    constexpr int kXcd = 8, kGroup = 8;
    const int n_a = by_columns ? tiles_c : tiles_r, n_b = by_columns ? tiles_r : tiles_c;    // a: grouped, b: walked
    const int nt = tiles_r * tiles_c;
    // XCD x runs the workgroups x, x + 8, ...: they get the contiguous ids that start where those of XCDs 0 .. x-1 end
    // (the first nt % 8 XCDs run one workgroup more than the others)
    const int x = id % kXcd, extra = nt % kXcd;
    id = x * (nt / kXcd) + (x < extra ? x : extra) + id / kXcd;
    const int per_group = kGroup * n_b;
    const int g = id / per_group;
    const int first_a = g * kGroup;
    const int here = (n_a - first_a) < kGroup ? (n_a - first_a) : kGroup;
    const int in_g = id - g * per_group;
    int a = first_a + in_g % here, b = in_g / here;
    if (wide && here == kGroup) {
        // the patch of an XCD the other way round: 32 consecutive ids are 4 of the grouped dimension x 8 of the walked one
        const int blk = in_g / (8 * kGroup), r = in_g % (8 * kGroup);
        if ((blk + 1) * 8 <= n_b) {
            a = first_a + (r / 32) * 4 + (r % 4);
            b = blk * 8 + (r % 32) / 4;
        }
    }
    tr = by_columns ? b : a;
    tc = by_columns ? a : b;
}
__device__ __forceinline__ void tile_of_block(int tiles_r, int tiles_c, int& tr, int& tc) {
    tile_of_id(blockIdx.x, tiles_r, tiles_c, false, false, tr, tc);
}

// Which operand the walk of 256 x 256 tiles groups.  The panels of the grouped operand (eight per group, one group per
// XCD at a time) are read again for every few tiles of the walk, out of the memory-side cache if they are still
// there; the other operand streams past and is swept once per group.  Between two sweeps the cache has to hold the
// grouped panels in flight plus all of the other operand.  When that fits, grouping the larger operand is better (each
// of its panels comes from HBM once, in a burst at the start of a group; a streamed large operand puts HBM latency into
// every tile); when it does not, the grouped panels of a large operand are evicted between two reads, and grouping the
// smaller one loses less.  Measured on 64 shapes (4096 .. 32768 squared, K 4096 .. 28672): up to 16 % between the two
// walks, and this rule picks the faster one wherever they differ by more than 3 %.
__device__ __forceinline__ bool walk_by_columns(int tiles_r, int tiles_c, int K) {
    constexpr long long kCacheBudget = 288ll << 20;    // a little above the 256 MiB: eviction is not strictly LRU
    const long long panel = static_cast<long long>(kDmaTile) * K;
    const bool tall = tiles_r > tiles_c;
    const long long big = (tall ? tiles_r : tiles_c) * panel, small = (tall ? tiles_c : tiles_r) * panel;
    const long long in_flight = 64 * panel;
    const bool fits = (big < in_flight ? big : in_flight) + small <= kCacheBudget;
    return fits ? !tall : tall;
}

template <int BR, int BC, int XF, int YF, typename OT, bool KGUARD>
__global__ __launch_bounds__(kGemmThreads) void fp8_gemm_kernel(const uint8_t* __restrict__ X,
                                                                 const uint8_t* __restrict__ Y, OT* __restrict__ D,
                                                                 int NR, int NC, int K,
                                                                 const float* __restrict__ x_scale_inv,
                                                                 const float* __restrict__ y_scale_inv, int accumulate,
                                                                 const void* __restrict__ bias, int bias_dt) {
    constexpr int WR = BR / 2, WC = BC / 2;    // wave tile
    constexpr int TR = WR / 16, TC = WC / 16;  // MFMA tiles per wave
    constexpr int kStage = (BR + BC) * kBK;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    int tr, tc;
    tile_of_block((NR + BR - 1) / BR, (NC + BC - 1) / BC, tr, tc);
    const int row0 = tr * BR, col0 = tc * BC;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wr = wave >> 1, wc = wave & 1;
    const int l16 = lane & 15, g4 = lane >> 4;

    v4f acc[TR][TC];
#pragma unroll
    for (int i = 0; i < TR; ++i)
#pragma unroll
        for (int j = 0; j < TC; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;

    TileLoader<BR, KGUARD> lx;
    TileLoader<BC, KGUARD> ly;
    const int nk = (K + kBK - 1) / kBK;
    // The K slices are walked in ascending order, 128 bytes of K per MFMA, exactly as the direct-to-LDS kernel below
    // walks them: the two kernels add up the same blocks in the same order and agree to the bit.  (Walking them in
    // an order rotated per workgroup, to spread the memory channels, was measured slower: 2-4 % at 2048 x 2048 x 4096,
    // 10-14 % at 4096 x 4096 x 4112.)
    auto slice = [&](int kt) { return kt * kBK; };
    lx.gload(X, row0, NR, K, slice(0));
    ly.gload(Y, col0, NC, K, slice(0));
    lx.lstore(smem);
    ly.lstore(smem + BR * kBK);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
        const uint8_t* sx = smem + (kt & 1) * kStage;
        const uint8_t* sy = sx + BR * kBK;
        if (kt + 1 < nk) {
            lx.gload(X, row0, NR, K, slice(kt + 1));
            ly.gload(Y, col0, NC, K, slice(kt + 1));
        }
        {
            // a lane holds, for row lane % 16 of a 16-row block, the 32 K-bytes (lane / 16) * 32 .. + 31 of the slice
            v8i fx[TR], fy[TC];
#pragma unroll
            for (int i = 0; i < TR; ++i) fx[i] = read_frag(sx, wr * WR + i * 16 + l16, g4);
#pragma unroll
            for (int j = 0; j < TC; ++j) fy[j] = read_frag(sy, wc * WC + j * 16 + l16, g4);
#pragma unroll
            for (int i = 0; i < TR; ++i)
#pragma unroll
                for (int j = 0; j < TC; ++j) acc[i][j] = mfma16<XF, YF>(fx[i], fy[j], acc[i][j]);
        }
        if (kt + 1 < nk) {
            uint8_t* nx = smem + ((kt + 1) & 1) * kStage;
            lx.lstore(nx);
            ly.lstore(nx + BR * kBK);
        }
        __syncthreads();
    }

    // srcA = X rows: a lane holds D column (Y row) lane % 16 of a block and the four D rows (lane / 16) * 4 .. + 3
    const float alpha = (*x_scale_inv) * (*y_scale_inv);
#pragma unroll
    for (int j = 0; j < TC; ++j) {
        const int col = col0 + wc * WC + j * 16 + l16;
        if (col >= NC) continue;
        const float bv = bias != nullptr ? load_bias(bias, bias_dt, col) : 0.0f;
#pragma unroll
        for (int i = 0; i < TR; ++i) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = row0 + wr * WR + i * 16 + g4 * 4 + r;
                if (row < NR) {
                    store_out<OT>(D + static_cast<size_t>(row) * NC + col, fmaf(acc[i][j][r], alpha, bv), accumulate != 0);
                }
            }
        }
    }
}



// two floats -> packed 16-bit pair with the hardware's round-to-nearest-even converters
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ uint32_t pack_f16(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}

template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// four consecutive elements of an output row straight from the accumulators, one by one: ragged edges,
// bias and accumulation, all in float32 with a single rounding to the output type
template <typename OT>
__device__ __noinline__ void store_quad_slow(OT* D, int row, int col, int NR, int NC, float alpha, float v0, float v1,
                                             float v2, float v3, int accumulate, const void* bias, int bias_dt) {
    if (row >= NR) return;
    const float v[4] = {v0, v1, v2, v3};
    for (int e = 0; e < 4; ++e) {
        if (col + e >= NC) break;
        const float bv = bias != nullptr ? load_bias(bias, bias_dt, col + e) : 0.0f;
        store_out<OT>(D + static_cast<size_t>(row) * NC + col + e, fmaf(v[e], alpha, bv), accumulate != 0);
    }
}


// 16 bytes of output, stored past the caches (non-temporal).  A round of tiles writes 128 KiB per CU, 4 MiB per XCD: as
// ordinary stores that is the whole L2, and the operand panels that the next tiles are about to read get evicted for
// data nobody reads again soon.  Measured on the Llama-7B shapes: 3 to 9 % off the whole GEMM.
__device__ __forceinline__ void store_out16(void* p, const uint4& v) {
    typedef uint32_t v4u_t __attribute__((ext_vector_type(4)));
    const v4u_t vv = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(vv, static_cast<v4u_t*>(p));
}

// the old output of an accumulating GEMM is read once: past the caches as well
__device__ __forceinline__ uint4 load_out16(const void* p) {
    typedef uint32_t v4u_t __attribute__((ext_vector_type(4)));
    const v4u_t v = __builtin_nontemporal_load(static_cast<const v4u_t*>(p));
    return make_uint4(v[0], v[1], v[2], v[3]);
}

// ---------------------------------------------------------------------------------------------
// Main kernel: 256 x 256 output tile over 128-byte K slices, four wavefronts each owning a 128 x 128
// quadrant (8 x 8 accumulators of the 16x16x128 FP8 MFMA = 256 accumulation registers per lane).
//  * Tiles travel global -> LDS with the direct-to-LDS load: no staging registers, no LDS stores.  A
//    lane group of 8 fetches one whole 128-byte line (full-line requests are what the L2 serves best).
//  * Two 64 KiB LDS stages.  A slice is computed in four quarters of 16 MFMAs (X half x Y half); the fragment
//    half the next quarters need is read while the current one executes.
//  * One workgroup barrier per slice, after the second quarter: by then every wave holds the whole slice
//    in registers, so the stage is refilled right away with the slice after next (its 16 loads spread over
//    the last two quarters, which leaves them half a slice to land).
//  * LDS reads and tile loads are interleaved with the MFMAs one at a time, so that neither the LDS nor
//    the vector-memory queue backs up and stalls the MFMA stream.
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

constexpr int kDmaStage = 2 * kDmaTile * kBK;    // X + Y slice: 64 KiB

// s_waitcnt vmcnt(N), leaving the other counters unconstrained (gfx9 encoding: vmcnt = [3:0] and [15:14])
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

//  * XT / YT: that operand is handed over K-major, T[K][rows] with the rows contiguous (the transpose of
//    what the product needs), so that callers need not materialize transposed copies.  Its slice sits in
//    LDS as 128 k-rows of 256 bytes (same 32 KiB), filled by the same eight 1 KiB loads, and its
//    fragments come from the transposing LDS read: a 16-lane group reads eight k-rows of 16 bytes and
//    lane i receives byte i of each, i.e. eight consecutive k for its row -- four such reads make the
//    32-byte operand of the MFMA.  The 16-byte position inside a k-row is XOR-ed with k % 8 (on the global
//    side again) so that the eight k-rows of one read fall into different banks.  Needs that operand's
//    row count to be a multiple of 256.
typedef int v2i __attribute__((ext_vector_type(2)));

//  * QF (an FP8 format, or 0): the output is not stored in OT but cast on to FP8 with in-time scaling in the same
//    launch, the way cast_to_fp8 of the stored output would: D is rounded to OT in registers, max |D| is taken over
//    the whole matrix, the scale follows from it, and the codes of D * scale are what reaches memory -- bit for
//    bit what the two steps give, without D's trip through memory.  Every workgroup holds its tile in registers
//    while the maxima meet (slots in the workspace, as in the one-pass in-time cast), so the launch must have all
//    its workgroups on the chip at once: the host only takes this path for at most one tile per CU.
//  * QSPEC: the cast to FP8 rides along on speculation instead, for any number of tiles.  The output is stored in OT as
//    usual and, next to it, the codes of the rounded output times the scale the meta holds before the call; every
//    workgroup folds the maximum of its rounded outputs into one word of the workspace, and the workgroup that
//    finishes last (a ticket counter tells) applies the scale rule, rewrites the meta and leaves a flag that says
//    whether the rule arrived at another scale than the one used.  Only then does the caller's next kernel read the
//    stored output again and cast it with the new scale; otherwise the codes stand, bit for bit what the two steps
//    give, and the stored output is never read back.  No workgroup waits for another.
// QuantArgs (the meta pointers, meeting slots and workspace words of the fused casts) is declared in gemm_call.h

// a * b rounded to OT (as the plain epilogue stores it) and widened again
template <typename OT>
__device__ __forceinline__ void round_pair(float a, float b, float& ra, float& rb) {
    if constexpr (sizeof(OT) == 4) {
        ra = a, rb = b;
    } else if constexpr (__is_same(OT, bf16_t)) {
        const uint32_t p = pack_bf16(a, b);
        ra = __uint_as_float(p << 16), rb = __uint_as_float(p & 0xffff0000u);
    } else {
        const f32x2 v = {a, b};
        const f16x2 h = __builtin_convertvector(v, f16x2);
        ra = static_cast<float>(h[0]), rb = static_cast<float>(h[1]);
    }
}

// element-wise unsigned maximum of two packed 16-bit pairs
__device__ __forceinline__ uint32_t pk_umax16(uint32_t a, uint32_t b) {
    typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b)));
}

// ---- the accumulators of the DMA kernel live in fixed AGPRs: block (i, j) of the wave's 8 x 8 in a[4n .. 4n+3], n = i * 8 + j.
// The register allocator never sees them.  Left to it, they are renumbered between the K loop, its straight-line tail
// and the epilogue, which costs copies between the MFMAs or spills once all 256 are taken.
#define MSAMP_A10(p) "a" #p "0", "a" #p "1", "a" #p "2", "a" #p "3", "a" #p "4", "a" #p "5", "a" #p "6", "a" #p "7", "a" #p "8", "a" #p "9"
#define MSAMP_ALL_AGPRS                                                                                                \
    "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", MSAMP_A10(1), MSAMP_A10(2), MSAMP_A10(3), MSAMP_A10(4),  \
        MSAMP_A10(5), MSAMP_A10(6), MSAMP_A10(7), MSAMP_A10(8), MSAMP_A10(9), MSAMP_A10(10), MSAMP_A10(11), MSAMP_A10(12), \
        MSAMP_A10(13), MSAMP_A10(14), MSAMP_A10(15), MSAMP_A10(16), MSAMP_A10(17), MSAMP_A10(18), MSAMP_A10(19),          \
        MSAMP_A10(20), MSAMP_A10(21), MSAMP_A10(22), MSAMP_A10(23), MSAMP_A10(24), "a250", "a251", "a252", "a253", "a254", \
        "a255"

// a[4N .. 4N+3] += srcA x srcB.  No clobber list: the compiler follows a clobbered register with a wait state, one per
// MFMA.  It learns of the AGPRs from acc_clear() and acc_fence(), which name them all.
template <int N, int CB, int BL>
__device__ __forceinline__ void mfma_fixed(const v8i& a, const v8i& b) {
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 a[%2:%3], %0, %1, a[%2:%3] cbsz:%4 blgp:%5"
                 :
                 : "v"(a), "v"(b), "n"(N * 4), "n"(N * 4 + 3), "n"(CB), "n"(BL));
}
__device__ __forceinline__ void acc_clear() {
    static_for<64>([&](auto nc) {
        constexpr int n = decltype(nc)::value;
        asm volatile("v_accvgpr_write_b32 a[%0], 0\n\tv_accvgpr_write_b32 a[%1], 0\n\tv_accvgpr_write_b32 a[%2], 0\n\t"
                     "v_accvgpr_write_b32 a[%3], 0"
                     :
                     : "n"(n * 4), "n"(n * 4 + 1), "n"(n * 4 + 2), "n"(n * 4 + 3));
    });
    asm volatile("s_nop 4" : : : MSAMP_ALL_AGPRS);
}
// After the last MFMA: waits out the MFMA pipe (a 16-pass MFMA's result may be read 18 wait states later) and hands out
// the token that ties the reads below to this point of the program.
__device__ __forceinline__ uint32_t acc_fence() {
    uint32_t token;
    asm volatile("s_nop 15\n\ts_nop 7\n\tv_mov_b32 %0, 0" : "=v"(token) : : MSAMP_ALL_AGPRS);
    return token;
}
__device__ __forceinline__ uint32_t acc_refence(uint32_t token) {
    asm volatile("" : "+v"(token));
    return token;
}
// Not volatile: the compiler may place the read where it likes after the fence that made the token.
template <int N>
__device__ __forceinline__ v4f acc_quad(uint32_t token) {
    v4f r;
    float x, y, z, w;
    asm("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(N * 4), "v"(token));
    asm("v_accvgpr_read_b32 %0, a[%1]" : "=v"(y) : "n"(N * 4 + 1), "v"(token));
    asm("v_accvgpr_read_b32 %0, a[%1]" : "=v"(z) : "n"(N * 4 + 2), "v"(token));
    asm("v_accvgpr_read_b32 %0, a[%1]" : "=v"(w) : "n"(N * 4 + 3), "v"(token));
    r[0] = x, r[1] = y, r[2] = z, r[3] = w;
    return r;
}

template <int XF, int YF, typename OT, bool XT = false, bool YT = false, int QF = 0, bool ODD_NK = false, bool QSPEC = false,
          bool SPLIT = false>
__global__ __launch_bounds__(kGemmThreads) void fp8_gemm_dma_kernel(const uint8_t* __restrict__ X,
                                                                     const uint8_t* __restrict__ Y, OT* __restrict__ D,
                                                                     int NR, int NC, int K,
                                                                     const float* __restrict__ x_scale_inv,
                                                                     const float* __restrict__ y_scale_inv, int accumulate,
                                                                     const void* __restrict__ bias, int bias_dt,
                                                                     QuantArgs qa) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    const int tiles_r = (NR + kDmaTile - 1) / kDmaTile, tiles_c = (NC + kDmaTile - 1) / kDmaTile;
    bool by_columns = walk_by_columns(tiles_r, tiles_c, K);
    int tr, tc;
    // Which way round the 32 tiles of an XCD lie.  A K-major operand with a long leading dimension that is a multiple
    // of 4 KiB is hard on that XCD's L2: the 128 k-rows of a tile's 256-byte strip lie a multiple of 4 KiB apart, L2
    // misses double (TCC_MISS, FETCH_SIZE x 2.4 on 8192 x 28672 x 16384 with Y as [K, 28672]) and the CUs that share
    // the strip all wait.  Eight such strips shared by four CUs each then beat four shared by eight: the patch is turned
    // so that this operand gets the eight (that shape: 2.82 -> 3.07 PFLOP/s; with X K-major as well 2.73 -> 3.09;
    // 28672 x 8192 x 16384, both K-major: 2.88 -> 3.02).  Measured only where it is applied: K of 16384 and more, one
    // such operand (with two, or at K = 8192, turning the patch lost 1 to 7 %).
    auto strips = [](int n) { return n % 4096 == 0 && n >= 12288; };
    const bool strips_x = XT && strips(NR), strips_y = YT && strips(NC);
    bool wide = K >= 16384 && strips_x != strips_y && (strips_y ? !by_columns : by_columns);
    // Weight gradients (both operands K-major) over 16384 .. 24576 tokens: the longer operand gets the eight whenever its
    // leading dimension is 10240 or more and a multiple of 256, whichever walk the cache rule above prefers.  Measured
    // at K = 16384 on 41 shapes (long side 5120 .. 28672, short side 4096 / 5120 / 8192, either way round) against
    // the three other walks: 10240 x 8192 +7 %, 8192 x 10240 +11 %, 14336 x 4096 +13 %, 4096 x 14336 +14 %,
    // 8192 x 14336 +11 %, 8192 x 22016 +8 %, 13824 x 4096 +6 %, 11008 x 4096 +3 %, the multiples of 4096 that the rule above already turned
    // unchanged, nothing below -2 % (5120 x 13824); +2 to 5 % at K = 20480, +1 to 3 % at 24576; nothing at K = 12288, and
    // at K = 32768 the turned patch loses 3 to 6 %.
    // Input gradients (only Y K-major) with 12288 or more columns and K of 8192 or more: Y gets the eight, walking
    // groups of tile rows.  Measured on 35 shapes (8192 .. 32768 rows, 12288 .. 28672 columns, K 8192 .. 28672) against
    // the three other walks: up to +9 % (8192 x 14336 x 12288 and x 16384), 16384 x 28672 x 8192 +4 %, nothing below -0.7 %;
    // with 8192 columns (x 28672) it loses 3 %, at K = 4096 nothing moves.
    if (!XT && YT && NC >= 12288 && K >= 8192) by_columns = false, wide = true;
    if (XT && YT && K >= 16384 && K <= 24576 && NR != NC) {
        const bool x_long = NR > NC;
        const int long_n = x_long ? NR : NC, short_n = x_long ? NC : NR;
        if (long_n >= 10240 && long_n % 256 == 0 && short_n <= 8192) by_columns = x_long, wide = true;
    }
    // Split waits (template flag SPLIT, row-major operands only; the host picks the instantiation: bit 2 of a registered
    // walk, else by rule).  In the plain form a slice's sixteen tile loads are issued during the second half of a step
    // (the stage they fill is read until then) and all awaited at the one barrier in the middle of the next step: the
    // last of them has half a step to arrive.  But a row-major load brings whole rows, and the rows of blocks 0..3 of
    // every wave's quadrant were already read at the end of the step before.  In the split form the loads go out in the
    // order of need, four per quarter of the step: X and Y blocks 0..3 of slice kt + 2 during the first half of step kt
    // (after a barrier of its own at the start of the step: everybody has read those rows of slice kt), Y and X blocks
    // 4..7 during the second half; the first part is awaited in the middle of step kt + 1, the second at the start of
    // step kt + 2, each with sixteen younger loads in flight behind it: every load has one to one and a half steps.  That
    // pays where the loads miss the L2 and the memory-side cache -- the longer K, the more: 16384 x 8192 x K at K = 12288
    // +1 %, 14336 +5 %, 16384 +2 %, 20480 +5 %, 28672 +8 %, 16384 cubed +5 % -- and is level below (-0.8 to +0.8 % at K
    // of 4096 .. 11008: the second barrier), hence the host's rule K >= 12288.  (A flag read at run time instead of a
    // second instantiation cost the plain form 3 to 7 %: the selects between the two orders sat in the K loop.)
    static_assert(!SPLIT || (!XT && !YT && QF == 0 && !QSPEC), "split waits: plain row-major form only");
    // a walk registered for this problem (timed on this machine) overrides the rules
    if (qa.walk_plus_one > 0) by_columns = (qa.walk_plus_one - 1) & 1, wide = ((qa.walk_plus_one - 1) >> 1) & 1;
    tile_of_id(blockIdx.x, tiles_r, tiles_c, by_columns, wide, tr, tc);
    const int row0 = tr * kDmaTile, col0 = tc * kDmaTile;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wr = wave >> 1, wc = wave & 1;
    // the output factor is fetched now: left to the epilogue, the two scalar loads sit on its critical path
    float alpha_early = (*x_scale_inv) * (*y_scale_inv);
    asm volatile("" : "+v"(alpha_early));
    // QSPEC: the scale the codes are written with, as the meta holds it now (the last workgroup rewrites the meta)
    float guess = 1.0f;
    if constexpr (QSPEC) {
        guess = *qa.scale;
        asm volatile("" : "+v"(guess));
    }

    // ---- global -> LDS.  A stage holds 256 X rows then 256 Y rows, 128 bytes per row.  One wave
    // instruction fills 8 rows (1 KiB, lane-contiguous): lane l lands in row l/8, 16-byte position l%8,
    // and therefore fetches the logical chunk position ^ swizzle(row).  Rows past the end of the matrix
    // are clamped to its last row (their results are never stored).
    const int chunk = (lane & 7) ^ (lane >> 3) ^ (wave & 1);
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)smem)));
    // K-major operand: one wave instruction fills 4 k-rows of 256 bytes; lane l lands in k-row l/16,
    // position l%16, and fetches the logical chunk position ^ (k-row % 8)
    const int chunk_t = (lane & 15) ^ ((wave & 1) * 4 + (lane >> 4));
    uint32_t xoff[8], yoff[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = (i * 4 + wave) * 8 + (lane >> 3);
        int gx = row0 + r, gy = col0 + r;
        gx = gx < NR ? gx : NR - 1;
        gy = gy < NC ? gy : NC - 1;
        const int krow = (i * 4 + wave) * 4 + (lane >> 4);
        xoff[i] = XT ? static_cast<uint32_t>(krow) * static_cast<uint32_t>(NR) + row0 + chunk_t * 16
                     : static_cast<uint32_t>(gx) * static_cast<uint32_t>(K) + chunk * 16;
        yoff[i] = YT ? static_cast<uint32_t>(krow) * static_cast<uint32_t>(NC) + col0 + chunk_t * 16
                     : static_cast<uint32_t>(gy) * static_cast<uint32_t>(K) + chunk * 16;
    }
    // one of the 16 loads of a slice (0..7: X rows, 8..15: Y rows), so they can be spread between MFMAs
    auto dma = [&](int kt, int stage, int i) __attribute__((always_inline)) {
        // the i-th load of a slice is load i, or in the split form the i-th in order of need
        constexpr int by_need[16] = {0, 1, 4, 5, 8, 9, 12, 13, 10, 11, 14, 15, 2, 3, 6, 7};
        const int which = SPLIT ? by_need[i] : i;
        const bool is_x = which < 8;
        const size_t slice = static_cast<size_t>(kt) * kBK;
        const uint8_t* src = is_x ? X + (XT ? slice * NR : slice) : Y + (YT ? slice * NC : slice);
        const uint32_t off = which < 8 ? xoff[which] : yoff[which - 8];
        // (wave-uniform by construction; the readfirstlane keeps it in a scalar register whatever the compiler makes of it)
        const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_base + stage * kDmaStage + (which < 8 ? 0 : kDmaTile * kBK) +
                                                            ((which & 7) * 4 + wave) * 1024);
        // Written as assembly so that the compiler does not see an LDS write it cannot tell apart from
        // the fragment reads: it would otherwise make every LDS read wait for all loads in flight.
        // Completion is tracked by hand with wait_vmcnt<>() before the barriers below.  M0 holds the
        // wave's LDS destination.  The address is a scalar base (operand + slice) plus the lane's 32-bit
        // offset, so no vector instruction is spent on it.
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(dst), "v"(off), "s"(src) : "memory", "m0");
    };

    // ---- LDS -> fragments of the 16x16x128 MFMA: a lane holds, for row lane % 16 of a 16-row block, the 32 K-bytes
    // (lane / 16) * 32 .. + 31 of the 128-byte slice.  Row-major operand: two 16-byte reads at the swizzled chunks
    // 2 * (lane / 16) and + 1.  K-major operand: four transposing reads, each handing a 16-lane group eight
    // consecutive k of 16 rows.
    const int fsw = (lane & 7) ^ ((lane >> 3) & 1);
    const int l16 = lane & 15, g4 = lane >> 4;
    const int off_lo = ((2 * g4) ^ fsw) << 4;    // low 16 bytes of this lane's 32; the high ones are at ^ 16
    const int xrow = (wr * 128 + l16) * kBK;
    const int yrow = kDmaTile * kBK + (wc * 128 + l16) * kBK;
    const int tj = l16 >> 1;
    const int t_lane = (g4 * 32 + tj) * 256 + (l16 & 1) * 8;    // k-row and 8-byte half of this lane's address
    // The wave's 128 x 128 quadrant is 8 x 8 blocks of 16 x 16.  Fragments are kept by halves: fx[h] / fy[h] hold the
    // four 16-row blocks 4h .. 4h+3 of X / Y (8 registers each).  A half arrives in pieces: two 16-byte reads per
    // block of a row-major operand, four 8-byte transposing reads otherwise.
    constexpr int kPX = XT ? 16 : 8, kPY = YT ? 16 : 8;
    auto read_piece = [&](int* dst, int stage, bool is_x, int half, int p) __attribute__((always_inline)) {
        const uint8_t* base = smem + stage * kDmaStage;
        if ((is_x && !XT) || (!is_x && !YT)) {
            const int b = p >> 1, hf = p & 1;
            const v4i val = *reinterpret_cast<const v4i*>(base + (is_x ? xrow : yrow) + (half * 4 + b) * 16 * kBK +
                                                          (off_lo ^ (hf * 16)));
            int* d = dst + b * 8 + hf * 4;
            d[0] = val[0], d[1] = val[1], d[2] = val[2], d[3] = val[3];
        } else {
            const int b = p >> 2, qq = p & 3;
            const int wq = is_x ? wr : wc;
            const int addr = (is_x ? 0 : kDmaTile * kBK) + t_lane + (qq * 8) * 256 + wq * 128 + (((half * 4 + b) ^ tj) << 4);
            const v2i val = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                (__attribute__((address_space(3))) v2i*)(base + addr));
            int* d = dst + b * 8 + qq * 2;
            d[0] = val[0], d[1] = val[1];
        }
    };

    // accumulator block (i, j): D rows i * 16 + lane % 16, D columns j * 16 + (lane / 16) * 4 .. + 3 of the quadrant
    acc_clear();

    const int nk = K / kBK;
    int fx[2][32], fy[2][32];

    // One quarter of a slice: the 16 MFMAs of X half hx against Y half hy, with the reads of one fragment half
    // (rd_x / rd_half from rd_stage into rd_dst) spread between them and, if asked for, eight of the 16 tile loads
    // of slice ld_kt (ld_first .. ld_first + 7), one every other MFMA.
    // srcA = Y rows (columns of D), srcB = X rows (rows of D): a lane then holds, for D row lane % 16 of a block, four
    // consecutive D columns -- the layout the epilogue wants.
    auto quarter = [&](auto hxc, auto hyc, int* rd_dst, int rd_stage, bool rd_x, int rd_half, bool do_read, int ld_kt,
                       int ld_stage, int ld_first, bool do_load) __attribute__((always_inline)) {
        constexpr int cb = (YF == MSAMP_DT_E4M3) ? 0 : 1;
        constexpr int bl = (XF == MSAMP_DT_E4M3) ? 0 : 1;
        const int np = rd_x ? kPX : kPY;
        constexpr int hx = decltype(hxc)::value, hy = decltype(hyc)::value;
        static_for<4>([&](auto jc) {    // the Y fragment stays for four MFMAs in a row
            static_for<4>([&](auto ic) {
                constexpr int i = decltype(ic)::value, j = decltype(jc)::value;
                constexpr int n = j * 4 + i;
                const int* cx = fx[hx] + i * 8;
                const int* cy = fy[hy] + j * 8;
                const v8i vx = {cx[0], cx[1], cx[2], cx[3], cx[4], cx[5], cx[6], cx[7]};
                const v8i vy = {cy[0], cy[1], cy[2], cy[3], cy[4], cy[5], cy[6], cy[7]};
                mfma_fixed<(hx * 4 + i) * 8 + hy * 4 + j, cb, bl>(vy, vx);
                if (do_read) {
#pragma unroll
                    for (int p = n * np / 16; p < (n + 1) * np / 16; ++p) read_piece(rd_dst, rd_stage, rd_x, rd_half, p);
                }
                if constexpr (SPLIT) {    // four loads per quarter, all four quarters
                    if (do_load && (n & 3) == 3) dma(ld_kt, ld_stage, ld_first + (n >> 2));
                } else {    // eight per quarter in the second half of the step
                    if (do_load && (n & 1)) dma(ld_kt, ld_stage, ld_first + (n >> 1));
                }
                // Nothing moves across: one MFMA, then the reads and the load that go with it, so that the LDS reads and
                // the tile loads stay spread evenly between the MFMAs as written.
                __builtin_amdgcn_sched_barrier(0);
            });
        });
    };
    // Slice kt sits in stage st and slice kt + 1 is on its way into the other stage; X half 0 and Y half 0 of slice
    // kt are in registers.  Quarters 1, 2: X0 x Y0 while Y half 1 arrives, X0 x Y1 while X half 1 arrives -- all of
    // slice kt is in registers now.  Barrier: slice kt + 1 has landed and nobody needs the LDS copy of slice kt.
    // Quarters 3, 4: X1 x Y0 while X half 0 of slice kt + 1 arrives, X1 x Y1 while its Y half 0 arrives; the stage of
    // slice kt is refilled with slice kt + 2 meanwhile.
    // Split form: at the start of the step the second part of slice kt's loads has landed (behind it in the queue, if the
    // step before issued loads -- prev_loaded --, the sixteen of slice kt + 1) and everybody is past the reads of the
    // step before; the first part of slice kt + 2 then goes out during quarters 1 and 2, into the rows of blocks 0..3.
    auto slice = [&](int st, bool has_next, int ld_kt, bool do_load, bool prev_loaded = true) __attribute__((always_inline)) {
        constexpr std::integral_constant<int, 0> c0{};
        constexpr std::integral_constant<int, 1> c1{};
        if constexpr (SPLIT) {
            if (prev_loaded) wait_vmcnt<16>();
            else wait_vmcnt<0>();
            __syncthreads();
        }
        quarter(c0, c0, fy[1], st, false, 1, true, ld_kt, st, 0, SPLIT && do_load);
        quarter(c0, c1, fx[1], st, true, 1, true, ld_kt, st, 4, SPLIT && do_load);
        if (SPLIT && has_next) {
            // the first part of slice kt + 1; behind it its second part and, if this step loads, the first of slice kt + 2
            if (do_load) wait_vmcnt<16>();
            else wait_vmcnt<8>();
        } else {
            wait_vmcnt<0>();
        }
        __syncthreads();
        quarter(c1, c0, fx[0], st ^ 1, true, 0, has_next, ld_kt, st, SPLIT ? 8 : 0, do_load);
        quarter(c1, c1, fy[0], st ^ 1, false, 0, has_next, ld_kt, st, SPLIT ? 12 : 8, do_load);
    };

    // prologue: slices 0 and 1 (the host sends no problem with fewer than two slices here); wait for slice 0; read
    // its first fragment halves
#pragma unroll
    for (int w = 0; w < 16; ++w) dma(0, 0, w);
#pragma unroll
    for (int w = 0; w < 16; ++w) dma(1, 1, w);
    wait_vmcnt<16>();
    __syncthreads();
#pragma unroll
    for (int p = 0; p < kPX; ++p) read_piece(fx[0], 0, true, 0, p);
#pragma unroll
    for (int p = 0; p < kPY; ++p) read_piece(fy[0], 0, false, 0, p);
    // Two slices per turn of the loop (stage 0, stage 1).  What is left afterwards -- two slices when the slice count is
    // even, three when it is odd (ODD_NK, chosen by the host) -- follows as straight-line code: the last slices load
    // nothing and the last one reads no fragments for a successor, which the compiler then knows.
    int kt = 0;
    for (; kt + 3 < nk; kt += 2) {
        slice(0, true, kt + 2, true);
        slice(1, true, kt + 3, true);
    }
    if constexpr (ODD_NK) {
        slice(0, true, kt + 2, true);
        slice(1, true, 0, false);
        slice(0, false, 0, false, false);
    } else {
        slice(0, true, 0, false);
        slice(1, false, 0, false, false);
    }
    // The workgroup that follows this one on the CU is, as a rule, the one 256 ids on (same XCD).  Touch the first two K
    // slices of its tile now -- one 4-byte load per 128-byte line, dropped into an LDS corner that nothing reads -- so that
    // its prologue finds them in this XCD's L2 instead of waiting for HBM with the MFMA pipe idle.  The loads have no
    // register destination, so nothing has to wait for them; the hardware drains them before the wave ends.
    {
        const int nid = blockIdx.x + 256;
        if (nid < tiles_r * tiles_c) {
            int ntr, ntc;
            tile_of_id(nid, tiles_r, tiles_c, by_columns, wide, ntr, ntc);
            const int nr0 = ntr * kDmaTile, nc0 = ntc * kDmaTile;
            // line L of an operand's 512: row-major, half L % 2 of row L / 2 (clamped like the tile loads); K-major (whole
            // tiles only), half L % 2 of the tile's 256 bytes in k-row L / 2 (K >= 256 here)
            auto line = [&](int L, bool is_x) __attribute__((always_inline)) -> const uint8_t* {
                const int r = L >> 1, hf = (L & 1) * 128;
                const uint8_t* base = is_x ? X : Y;
                const int n = is_x ? NR : NC, first = is_x ? nr0 : nc0;
                if (is_x ? XT : YT) return base + static_cast<size_t>(r) * n + first + hf;
                const int row = first + r < n ? first + r : n - 1;
                return base + static_cast<size_t>(row) * K + hf;
            };
            const int t = threadIdx.x;
            const uint32_t dump = __builtin_amdgcn_readfirstlane(lds_base + 2 * kDmaStage - 256);
            asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off\n\tglobal_load_lds_dword %2, off\n\t"
                         "global_load_lds_dword %3, off\n\tglobal_load_lds_dword %4, off"
                         : : "s"(dump), "v"(line(t, true)), "v"(line(t + 256, true)), "v"(line(t, false)), "v"(line(t + 256, false))
                         : "memory", "m0");
        }
    }
    const uint32_t acc_token = acc_fence();
    // No barrier here: the last LDS reads of every wave were issued (and awaited) before the barrier of the last
    // slice, and no load is in flight, so each wave may start on its patch as soon as its own MFMAs are done.

    // The epilogues below handle the quadrant in four units of 32 rows (two 16-row blocks): unit u, half h, column
    // block j -> acc[2u + h][j], patch row h * 16 + lane % 16, patch columns j * 16 + (lane / 16) * 4 .. + 3.
    if constexpr (QF != 0) {
        // ---- fused in-time cast (whole tiles only, no bias, no accumulation: the host sees to that)
        __shared__ uint32_t q_red[kGemmThreads / kWave];
        __shared__ uint32_t q_scale, q_amax;
        const float alpha = alpha_early;
        // max |acc| as an ordered bit pattern: NaN above Inf above everything finite, so a NaN reaches the amax
        // as it does through abs().max()
        uint32_t m = 0;
        static_for<64>([&](auto nc) {
            const v4f a = acc_quad<decltype(nc)::value>(acc_token);
#pragma unroll
            for (int r = 0; r < 4; ++r) m = umax(m, __float_as_uint(a[r]) & 0x7fffffffu);
        });
        m = block_max_u32(m, q_red);    // valid in lane 0 of wave 0
        const int tid = threadIdx.x;
        if (tid == 0) {
            // Scaling by |alpha| and rounding to OT never reorder magnitudes, so the maximum of the rounded outputs
            // is the rounded, scaled maximum.
            float am, unused;
            round_pair<OT>(__uint_as_float(m) * fabsf(alpha), 0.0f, am, unused);
            m = __float_as_uint(am) & 0x7fffffffu;
            __hip_atomic_store(qa.slots + blockIdx.x, (static_cast<uint64_t>(qa.token) << 32) | m, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        }
        // Workgroup 0 collects the slots (its first wave), derives amax and scale and posts
        // both, tagged with the token, in the two words behind the slots; the other workgroups poll only those.
        // Every wait is bounded.  Workgroup 0 posts even when it gives up (NaN amax, old scale), and the others wait
        // longer for the post than it waits for them; whoever gives up sets the sticky error word of the workspace.
        uint64_t* post = qa.slots + kMaxSlots;
        if (blockIdx.x == 0) {
            if (tid < kWave) {
                uint32_t mm = 0;
                bool all_in = false;
                for (uint32_t spins = 0; !all_in && spins < qa.spin_limit; ++spins) {
                    uint64_t sv[kMaxSlots / kWave];
#pragma unroll
                    for (int j = 0; j < kMaxSlots / kWave; ++j)
                        sv[j] = __hip_atomic_load(qa.slots + tid + j * kWave, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    bool ok = true;
                    mm = 0;
#pragma unroll
                    for (int j = 0; j < kMaxSlots / kWave; ++j) {
                        const bool live = static_cast<uint32_t>(tid + j * kWave) < gridDim.x;
                        ok = ok && (!live || static_cast<uint32_t>(sv[j] >> 32) == qa.token);
                        mm = umax(mm, live ? static_cast<uint32_t>(sv[j]) : 0u);
                    }
                    all_in = __all(ok);
                }
                mm = wave_max_u32(mm);
                if (tid == 0) {
                    float am = __uint_as_float(mm);
                    if (!all_in) {    // gave up: NaN amax, old scale, both still posted, sticky error word set
                        am = __uint_as_float(0x7fc00000u);
                        report_wait_expired(qa.error_word, kErrCollectorGaveUp);
                    } else if ((qa.flags & MSAMP_FLAG_NAN_TO_INF) && !(am < __uint_as_float(0x7f800000u))) {
                        am = __uint_as_float(0x7f800000u);
                    }
                    const float sc = scale_rule(am, *qa.scale, qa.fp_max, qa.margin);
                    const uint64_t tag = static_cast<uint64_t>(qa.token) << 32;
                    __hip_atomic_store(post, tag | __float_as_uint(am), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(post + 1, tag | __float_as_uint(sc), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    q_scale = __float_as_uint(sc);
                    q_amax = __float_as_uint(am);
                    *qa.amax = am;
                    *qa.scale = sc;
                    *qa.scale_inv = 1.0f / sc;
                }
            }
        } else {
            if (tid == 0) {
                uint64_t pa = 0, ps = 0;
                bool posted = false;
                const uint64_t follower_limit = static_cast<uint64_t>(qa.spin_limit) * kFollowerSpinFactor;
                for (uint64_t spins = 0; !posted && spins < follower_limit; ++spins) {
                    pa = __hip_atomic_load(post, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    ps = __hip_atomic_load(post + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    posted = static_cast<uint32_t>(pa >> 32) == qa.token && static_cast<uint32_t>(ps >> 32) == qa.token;
                }
                if (!posted) report_wait_expired(qa.error_word, kErrFollowerGaveUp);
                q_amax = posted ? static_cast<uint32_t>(pa) : 0x7fc00000u;
                q_scale = posted ? static_cast<uint32_t>(ps) : 0x7fc00000u;
            }
        }
        __syncthreads();    // also: every wave is through with the stages, which the patches below reuse
        const float sc = __uint_as_float(q_scale);
        const uint32_t acc_token2 = acc_refence(acc_token);    // a second round of reads, not the first one kept alive
        // with a positive finite amax and the scale derived from it nothing leaves the format and nothing is NaN:
        // the clamp and the NaN patch of the general conversion can go
        const bool in_range = __uint_as_float(q_amax) * sc <= qa.fp_max && __uint_as_float(q_amax) > 0.0f;
        constexpr int kQPitch = 128 + 16;    // bytes per patch row: 128 codes and padding that staggers the banks
        uint8_t* qpatch = smem + wave * (32 * kQPitch);
        auto emit = [&](auto checked) {
            constexpr bool kChecked = decltype(checked)::value;
            static_for<4>([&](auto uc) {
                constexpr int u = decltype(uc)::value;
                static_for<2>([&](auto hc) {
                    constexpr int h = decltype(hc)::value;
                    static_for<8>([&](auto jc) {
                        constexpr int j = decltype(jc)::value;
                        // the outputs as OT would hold them, then scaled
                        const v4f a = acc_quad<(2 * u + h) * 8 + j>(acc_token2);
                        float r0, r1, r2, r3;
                        round_pair<OT>(a[0] * alpha, a[1] * alpha, r0, r1);
                        round_pair<OT>(a[2] * alpha, a[3] * alpha, r2, r3);
                        uint32_t w;
                        if constexpr (kChecked) w = quant4<QF>(r0 * sc, r1 * sc, r2 * sc, r3 * sc);
                        else w = quant4_in_range<QF>(r0 * sc, r1 * sc, r2 * sc, r3 * sc);
                        *reinterpret_cast<uint32_t*>(qpatch + (h * 16 + l16) * kQPitch + j * 16 + g4 * 4) = w;
                    });
                });
                // the patch is private to this wave and the LDS serves one wave's requests in order: no waits here
                auto rd = [&](int t) {
                    return *reinterpret_cast<const uint4*>(qpatch + (t * 8 + (lane >> 3)) * kQPitch + (lane & 7) * 16);
                };
                const uint4 val0 = rd(0), val1 = rd(1), val2 = rd(2), val3 = rd(3);
                auto st = [&](int t, const uint4& v) {
                    const int grow = row0 + wr * 128 + u * 32 + t * 8 + (lane >> 3);
                    const int gcol = col0 + wc * 128 + (lane & 7) * 16;
                    store_out16(qa.q + static_cast<size_t>(grow) * NC + gcol, v);
                };
                st(0, val0), st(1, val1), st(2, val2), st(3, val3);
            });
        };
        if (in_range) emit(std::false_type{}); else emit(std::true_type{});
        return;
    }

    // ---- epilogue: per 32-row unit, accumulators -> this wave's LDS patch -> 16-byte row stores
    constexpr int kEsz = static_cast<int>(sizeof(OT));
    constexpr int kPitch = 128 * kEsz + 16;    // bytes per patch row (padding staggers the banks)
    uint8_t* patch = smem + wave * (32 * kPitch);
    const float alpha = alpha_early;
    const bool vec_ok = (NC % (16 / kEsz) == 0) && ((reinterpret_cast<uintptr_t>(D) & 15) == 0);
    const bool plain = !accumulate && bias == nullptr;    // (rows that 16-byte stores do not fit go out element by element)
    const bool pairs_ok = (NC % 2 == 0) && ((reinterpret_cast<uintptr_t>(D) & 3) == 0);
    constexpr int kChunksPerRow = 128 * kEsz / 16;      // 16 (2-byte) or 32 (float)
    constexpr int kRowsPerPass = 64 / kChunksPerRow;    // 4 or 2
    constexpr int kElemsPerChunk = 16 / kEsz;           // 8 or 4
    // QSPEC: the codes of a unit leave through a second per-wave patch, behind the room of the four largest (float32)
    // output patches; spec_max is the running maximum of the rounded outputs' magnitudes, as float32 bit patterns or
    // as two packed 16-bit patterns (NaN patterns compare above Inf, so a NaN reaches the amax as through abs().max())
    constexpr int kCPitch = 128 + 16;
    uint8_t* cpatch = smem + 4 * (32 * (128 * 4 + 16)) + wave * (32 * kCPitch);
    uint32_t spec_max = 0;
    // the values a packed pair of 16-bit outputs stands for
    auto widen_pair = [&](uint32_t pk, float& lo, float& hi) __attribute__((always_inline)) {
        if constexpr (__is_same(OT, bf16_t)) {
            lo = __uint_as_float(pk << 16), hi = __uint_as_float(pk & 0xffff0000u);
        } else {
            lo = f16_bits_to_float(pk & 0xffffu), hi = f16_bits_to_float(pk >> 16);
        }
    };
    auto emit_fused_rows = [&]() __attribute__((always_inline)) {
        // ---- bias and / or accumulation with 16-byte row accesses: the raw float32 accumulators of a 32-row unit go
        // through a per-wave float32 patch, each lane picks up one 16-byte segment of an output row, reads the old
        // output there if it is to be added, and stores fma(acc, alpha, bias) (+ old) rounded once -- the expression of
        // the element-wise path below and of the generic kernel.  A lane's columns are the same in every pass, so
        // its bias values are fetched once.
        constexpr int kFPitch = 128 * 4 + 16;    // bytes per float32 patch row
        uint8_t* fpatch = smem + wave * (32 * kFPitch);
        const int pc = lane % kChunksPerRow, prl = lane / kChunksPerRow;
        const int gcol = col0 + wc * 128 + pc * kElemsPerChunk;
        const bool col_ok = gcol < NC;
        float bv[kElemsPerChunk];
#pragma unroll
        for (int e = 0; e < kElemsPerChunk; ++e) bv[e] = (bias != nullptr && col_ok) ? load_bias(bias, bias_dt, gcol + e) : 0.0f;
        constexpr int kPasses = 32 / kRowsPerPass;    // 8 or 16
        constexpr int kGroup = 4;                     // passes whose old outputs are in flight together
        static_for<4>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            static_for<2>([&](auto hc) {
                constexpr int h = decltype(hc)::value;
                static_for<8>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    const v4f a = acc_quad<(2 * u + h) * 8 + j>(acc_token);
                    *reinterpret_cast<float4*>(fpatch + (h * 16 + l16) * kFPitch + (j * 16 + g4 * 4) * 4) =
                        make_float4(a[0], a[1], a[2], a[3]);
                });
            });
            // the patch is private to this wave and the LDS serves one wave's requests in order: no waits needed
            static_for<kPasses / kGroup>([&](auto gc) {
                constexpr int p0 = decltype(gc)::value * kGroup;
                uint4 old[kGroup];
                bool ok[kGroup];
#pragma unroll
                for (int t = 0; t < kGroup; ++t) {
                    const int grow = row0 + wr * 128 + u * 32 + (p0 + t) * kRowsPerPass + prl;
                    ok[t] = col_ok && grow < NR;
                    old[t] = make_uint4(0, 0, 0, 0);
                    if (accumulate && ok[t]) old[t] = load_out16(D + static_cast<size_t>(grow) * NC + gcol);
                }
#pragma unroll
                for (int t = 0; t < kGroup; ++t) {
                    const int pr = (p0 + t) * kRowsPerPass + prl;
                    const int grow = row0 + wr * 128 + u * 32 + pr;
                    const float* src = reinterpret_cast<const float*>(fpatch + pr * kFPitch + pc * kElemsPerChunk * 4);
                    float r[kElemsPerChunk], o[kElemsPerChunk];
                    const float4 a0 = *reinterpret_cast<const float4*>(src);
                    r[0] = a0.x, r[1] = a0.y, r[2] = a0.z, r[3] = a0.w;
                    if constexpr (kElemsPerChunk == 8) {
                        const float4 a1 = *reinterpret_cast<const float4*>(src + 4);
                        r[4] = a1.x, r[5] = a1.y, r[6] = a1.z, r[7] = a1.w;
                    }
                    if constexpr (kEsz == 4) {
                        o[0] = __uint_as_float(old[t].x), o[1] = __uint_as_float(old[t].y);
                        o[2] = __uint_as_float(old[t].z), o[3] = __uint_as_float(old[t].w);
                    } else {
                        In16<OT>::decode(old[t], o);
                    }
#pragma unroll
                    for (int e = 0; e < kElemsPerChunk; ++e) {
                        r[e] = fmaf(r[e], alpha, bv[e]);
                        if (accumulate) r[e] += o[e];
                    }
                    uint4 v;
                    if constexpr (kEsz == 4) {
                        v = make_uint4(__float_as_uint(r[0]), __float_as_uint(r[1]), __float_as_uint(r[2]), __float_as_uint(r[3]));
                    } else if constexpr (__is_same(OT, bf16_t)) {
                        v = make_uint4(pack_bf16(r[0], r[1]), pack_bf16(r[2], r[3]), pack_bf16(r[4], r[5]), pack_bf16(r[6], r[7]));
                    } else {
                        v = make_uint4(pack_f16(r[0], r[1]), pack_f16(r[2], r[3]), pack_f16(r[4], r[5]), pack_f16(r[6], r[7]));
                    }
                    if (ok[t]) store_out16(D + static_cast<size_t>(grow) * NC + gcol, v);
                    if constexpr (QSPEC) {
                        // the codes of the eight (four) outputs just rounded: 8 (4) bytes of a row of q per lane
                        float rr[kElemsPerChunk];
                        if constexpr (kEsz == 4) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) rr[e] = r[e], spec_max = umax(spec_max, __float_as_uint(r[e]) & 0x7fffffffu);
                        } else {
                            const uint32_t pk[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                spec_max = pk_umax16(spec_max, pk[e] & 0x7fff7fffu);
                                widen_pair(pk[e], rr[2 * e], rr[2 * e + 1]);
                            }
                        }
                        uint8_t* qo = qa.q + static_cast<size_t>(grow) * NC + gcol;
                        const uint32_t c0 = quant4_in_range<MSAMP_DT_E4M3>(rr[0] * guess, rr[1] * guess, rr[2] * guess, rr[3] * guess);
                        if constexpr (kEsz == 4) {
                            if (ok[t]) __builtin_nontemporal_store(c0, reinterpret_cast<uint32_t*>(qo));
                        } else {
                            const uint32_t c1 = quant4_in_range<MSAMP_DT_E4M3>(rr[4] * guess, rr[5] * guess, rr[6] * guess, rr[7] * guess);
                            typedef uint32_t v2u_t __attribute__((ext_vector_type(2)));
                            const v2u_t cc = {c0, c1};
                            if (ok[t]) __builtin_nontemporal_store(cc, reinterpret_cast<v2u_t*>(qo));
                        }
                    }
                }
            });
        });
    };
    if (!QSPEC && !plain && vec_ok) {
        emit_fused_rows();
        return;
    }
    if (!QSPEC && !plain) {
        static_for<8>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            static_for<8>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const v4f a = acc_quad<i * 8 + j>(acc_token);
                store_quad_slow<OT>(D, row0 + wr * 128 + i * 16 + l16, col0 + wc * 128 + j * 16 + g4 * 4, NR, NC, alpha, a[0], a[1],
                                    a[2], a[3], accumulate, bias, bias_dt);
            });
        });
        return;
    }
    // Three copies of the plain epilogue, chosen once per workgroup so that the one that runs is straight-line code:
    // whole tile with 16-byte row stores (no bounds checks; the address is a scalar row base plus one per-lane offset),
    // 16-byte row stores with bounds checks (tiles on the right or bottom edge), and rows that 16-byte stores do not fit.
    // (With the choice made per store, every store dragged three variants and their branches along.)
    auto emit_plain = [&](auto vec_c, auto inside_c) __attribute__((always_inline)) {
        constexpr bool kVec = decltype(vec_c)::value, kInside = decltype(inside_c)::value;
        const int pc = lane % kChunksPerRow, prl = lane / kChunksPerRow;
        const int gcol = col0 + wc * 128 + pc * kElemsPerChunk;
        // whole tile: byte offset of this lane's segment from the first element of its pass's first row
        const uint32_t lane_off = (static_cast<uint32_t>(prl) * static_cast<uint32_t>(NC) + static_cast<uint32_t>(pc * kElemsPerChunk)) * kEsz;
        static_for<4>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            static_for<2>([&](auto hc) {
                constexpr int h = decltype(hc)::value;
                static_for<8>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    const v4f a = acc_quad<(2 * u + h) * 8 + j>(acc_token);
                    // 8-byte writes of 16 rows at a time: rows r and r + 8 are 8 * (pitch mod 128 bytes) = 128 bytes apart in
                    // bank terms, the same 8-byte slot; the upper eight rows swap each pair of slots (undone when read back)
                    uint8_t* dst = patch + (h * 16 + l16) * kPitch + (((j * 16 + g4 * 4) * kEsz) ^ (kEsz == 2 ? ((l16 >> 3) & 1) << 3 : 0));
                    const float v0 = a[0] * alpha, v1 = a[1] * alpha, v2 = a[2] * alpha, v3 = a[3] * alpha;
                    float r0 = v0, r1 = v1, r2 = v2, r3 = v3;    // QSPEC: the outputs as OT holds them
                    if constexpr (kEsz == 4) {
                        *reinterpret_cast<float4*>(dst) = make_float4(v0, v1, v2, v3);
                        if constexpr (QSPEC)
                            spec_max = umax(umax(spec_max, __float_as_uint(v0) & 0x7fffffffu),
                                            umax(umax(__float_as_uint(v1) & 0x7fffffffu, __float_as_uint(v2) & 0x7fffffffu),
                                                 __float_as_uint(v3) & 0x7fffffffu));
                    } else {
                        uint32_t p01, p23;
                        if constexpr (__is_same(OT, bf16_t)) p01 = pack_bf16(v0, v1), p23 = pack_bf16(v2, v3);
                        else p01 = pack_f16(v0, v1), p23 = pack_f16(v2, v3);
                        *reinterpret_cast<uint2*>(dst) = make_uint2(p01, p23);
                        if constexpr (QSPEC) {
                            spec_max = pk_umax16(spec_max, pk_umax16(p01 & 0x7fff7fffu, p23 & 0x7fff7fffu));
                            widen_pair(p01, r0, r1);
                            widen_pair(p23, r2, r3);
                        }
                    }
                    if constexpr (QSPEC)
                        *reinterpret_cast<uint32_t*>(cpatch + (h * 16 + l16) * kCPitch + j * 16 + g4 * 4) =
                            quant4_in_range<MSAMP_DT_E4M3>(r0 * guess, r1 * guess, r2 * guess, r3 * guess);
                });
            });
            // no wait between the writes above and the reads below, nor before the next unit's writes: the patch is
            // private to this wave and the LDS serves one wave's requests in order
            constexpr int kPasses = 32 / kRowsPerPass;    // 8 or 16
            static_for<kPasses / 8>([&](auto gc) {
                constexpr int p0 = decltype(gc)::value * 8;
                // eight reads in flight together, then the eight stores (named values: an array here ends up in scratch)
                auto rd = [&](int t) {
                    const int pr = (p0 + t) * kRowsPerPass + prl;
                    const uint4 v = *reinterpret_cast<const uint4*>(patch + pr * kPitch + pc * 16);
                    const bool swapped = kEsz == 2 && (((p0 + t) * kRowsPerPass) >> 3) & 1;    // the same for all lanes of a pass
                    return swapped ? make_uint4(v.z, v.w, v.x, v.y) : v;
                };
                const uint4 val0 = rd(0), val1 = rd(1), val2 = rd(2), val3 = rd(3), val4 = rd(4), val5 = rd(5), val6 = rd(6),
                            val7 = rd(7);
                auto st = [&](int t, const uint4& v) {
                    const int first_row = row0 + wr * 128 + u * 32 + (p0 + t) * kRowsPerPass;    // wave-uniform
                    if constexpr (kVec && kInside) {
                        uint8_t* row_base = reinterpret_cast<uint8_t*>(D + static_cast<size_t>(first_row) * NC + (col0 + wc * 128));
                        store_out16(row_base + lane_off, v);
                    } else if constexpr (kVec) {
                        const int grow = first_row + prl;
                        if (grow < NR && gcol < NC) store_out16(D + static_cast<size_t>(grow) * NC + gcol, v);
                    } else {
                        // an output whose rows are not 16-byte aligned, or end inside a segment: the lane's segment one
                        // element at a time (still whole rows side by side: the 64 stores of a wave instruction touch few lines)
                        const int grow = first_row + prl;
                        if (grow < NR) {
                            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
                            OT* out = D + static_cast<size_t>(grow) * NC + gcol;
                            if (kEsz == 4 || pairs_ok) {    // 4-byte stores: float32, or 2-byte elements in aligned pairs
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    if (gcol + e * (4 / kEsz) < NC) reinterpret_cast<uint32_t*>(out)[e] = w[e];
                            } else {
#pragma unroll
                                for (int e = 0; e < kElemsPerChunk; ++e)
                                    if (gcol + e < NC) reinterpret_cast<uint16_t*>(out)[e] = static_cast<uint16_t>(w[e >> 1] >> ((e & 1) * 16));
                            }
                        }
                    }
                };
                st(0, val0), st(1, val1), st(2, val2), st(3, val3), st(4, val4), st(5, val5), st(6, val6), st(7, val7);
            });
            if constexpr (QSPEC) {
                // the unit's codes: 32 rows of 128 bytes, eight rows per pass, 16 bytes per lane (whole tiles only)
                auto crd = [&](int t) {
                    return *reinterpret_cast<const uint4*>(cpatch + (t * 8 + (lane >> 3)) * kCPitch + (lane & 7) * 16);
                };
                const uint4 c0 = crd(0), c1 = crd(1), c2 = crd(2), c3 = crd(3);
                auto cst = [&](int t, const uint4& v) {
                    const int grow = row0 + wr * 128 + u * 32 + t * 8 + (lane >> 3);
                    const int gcol = col0 + wc * 128 + (lane & 7) * 16;
                    store_out16(qa.q + static_cast<size_t>(grow) * NC + gcol, v);
                };
                cst(0, c0), cst(1, c1), cst(2, c2), cst(3, c3);
            }
        });
    };
    if constexpr (QSPEC) {
        // whole tiles and 16-byte rows only, no bias (the host sees to that): the output in OT and its codes side by side
        if (accumulate) emit_fused_rows();
        else emit_plain(std::true_type{}, std::true_type{});
        uint32_t m = spec_max;
        if constexpr (kEsz == 2) {
            m = umax(m & 0xffffu, m >> 16);
            if constexpr (__is_same(OT, bf16_t)) m <<= 16;
            else m = __float_as_uint(f16_bits_to_float(m));
        }
        __shared__ uint32_t spec_red[kGemmThreads / kWave];
        m = block_max_u32(m, spec_red);    // valid in lane 0 of wave 0
        if (threadIdx.x == 0) {
            // Fold into the call's one word, then draw a ticket.  Both are atomics of agent scope on neighbouring words,
            // carried out where all XCDs meet; the maximum's old value has come back before the ticket is asked for, so
            // whoever draws the last ticket finds every workgroup's maximum in the word.  No fence: at agent scope a
            // fence writes this XCD's L2 back, outputs of the other compute units included, once per workgroup.
            uint32_t* w = qa.spec_words;
            uint32_t before = 0;
            if (m > __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
                before = __hip_atomic_fetch_max(w, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(before) : : "memory");
            const uint32_t ticket = __hip_atomic_fetch_add(w + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (ticket == gridDim.x - 1) {
                const uint32_t mm = __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(w, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);    // ready for the next call
                __hip_atomic_store(w + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                float am = __uint_as_float(mm);
                if ((qa.flags & MSAMP_FLAG_NAN_TO_INF) && !(am < __uint_as_float(0x7f800000u))) am = __uint_as_float(0x7f800000u);
                const float sc = scale_rule(am, guess, qa.fp_max, qa.margin);
                *qa.amax = am;
                *qa.scale = sc;
                *qa.scale_inv = 1.0f / sc;
                // The codes stand if the rule confirms the scale they were written with and every output times that scale
                // is finite and inside the format (they were converted without clamp or NaN patch); otherwise the
                // caller's next kernel writes them again from the stored output.
                const bool stand = __float_as_uint(sc) == __float_as_uint(guess) && am * guess <= qa.fp_max;
                w[2] = stand ? 0u : 1u;
            }
        }
        return;
    }
    const bool inside = row0 + kDmaTile <= NR && col0 + kDmaTile <= NC;
    // (the per-lane offset of the whole-tile form is 32 bits: four rows of the output)
    if (vec_ok && inside && static_cast<unsigned long long>(NC) * kEsz * 4 < (1ull << 31)) emit_plain(std::true_type{}, std::true_type{});
    else if (vec_ok) emit_plain(std::true_type{}, std::false_type{});
    else emit_plain(std::false_type{}, std::false_type{});
}

// The kernel is built once for an even and once for an odd number of K slices (its last slices are straight-line
// code); ODD picks the one that fits K.
template <int XF, int YF, typename OT, bool XT, bool YT, bool ODD, bool SPLIT = false>
static int launch_gemm_dma_parity(const uint8_t* X, const uint8_t* Y, void* D, int NR, int NC, int K, const float* xs,
                                  const float* ys, int accumulate, const void* bias, int bias_dt, hipStream_t st) {
    constexpr int smem = 2 * kDmaStage;
    static std::atomic<bool> configured{false};    // setting the attribute twice is harmless
    auto kern = fp8_gemm_dma_kernel<XF, YF, OT, XT, YT, 0, ODD, false, SPLIT>;
    if (!configured.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(fp8_gemm_dma_kernel)");
        configured.store(true, std::memory_order_release);
    }
    const int tiles = ((NR + kDmaTile - 1) / kDmaTile) * ((NC + kDmaTile - 1) / kDmaTile);
    QuantArgs qa = {};
    qa.walk_plus_one = registered_walk(NR, NC, K, XT, YT) + 1;
    hipLaunchKernelGGL(kern, dim3(tiles), dim3(kGemmThreads), smem, st, X, Y, static_cast<OT*>(D), NR, NC, K, xs, ys,
                       accumulate, bias, bias_dt, qa);
    MSAMP_CHECK_LAUNCH("fp8_gemm_dma_kernel");
    return MSAMP_OK;
}

template <int XF, int YF, typename OT, bool XT = false, bool YT = false>
static int launch_gemm_dma(const uint8_t* X, const uint8_t* Y, void* D, int NR, int NC, int K, const float* xs,
                           const float* ys, int accumulate, const void* bias, int bias_dt, hipStream_t st) {
    if constexpr (!XT && !YT) {
        // split waits: bit 2 of a walk registered for the problem, else from K = 12288 on (see the kernel)
        const int walk = registered_walk(NR, NC, K, XT, YT);
        if (walk >= 0 ? (walk & 4) != 0 : K >= 12288) {
            constexpr int d_dtype = std::is_same<OT, float>::value ? MSAMP_DT_F32 : std::is_same<OT, f16_t>::value ? MSAMP_DT_F16 : MSAMP_DT_BF16;
            return run_gemm_split<XF, YF>(X, Y, D, d_dtype, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
        }
    }
    if ((K / kBK) & 1) return launch_gemm_dma_parity<XF, YF, OT, XT, YT, true>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
    return launch_gemm_dma_parity<XF, YF, OT, XT, YT, false>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
}

// the same kernel with the in-time cast to FP8 fused in (see QF above); the caller has checked the shape
template <int XF, int YF, typename OT, bool XT, bool YT, int QF, bool ODD>
static int launch_gemm_dma_quant_parity(const uint8_t* X, const uint8_t* Y, int NR, int NC, int K, const float* xs,
                                        const float* ys, const QuantArgs& qa, hipStream_t st) {
    constexpr int smem = 2 * kDmaStage;
    static std::atomic<bool> configured{false};    // setting the attribute twice is harmless
    auto kern = fp8_gemm_dma_kernel<XF, YF, OT, XT, YT, QF, ODD>;
    if (!configured.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(fp8_gemm_dma_kernel, fused cast)");
        configured.store(true, std::memory_order_release);
    }
    // its workgroups wait for each other, one per CU: the runtime must confirm that one fits (asked once per instantiation)
    static std::atomic<int> resident{-1};
    int fits = resident.load(std::memory_order_acquire);
    if (fits < 0) {
        int blocks = 0;
        fits = hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, reinterpret_cast<const void*>(kern), kGemmThreads, smem) == hipSuccess &&
               blocks >= 1;
        resident.store(fits, std::memory_order_release);
    }
    if (!fits) return MSAMP_NOT_FUSED;
    const int tiles = (NR / kDmaTile) * (NC / kDmaTile);
    QuantArgs qw = qa;
    qw.walk_plus_one = registered_walk(NR, NC, K, XT, YT) + 1;
    hipLaunchKernelGGL(kern, dim3(tiles), dim3(kGemmThreads), smem, st, X, Y, static_cast<OT*>(nullptr), NR, NC, K, xs, ys, 0,
                       static_cast<const void*>(nullptr), 0, qw);
    MSAMP_CHECK_LAUNCH("fp8_gemm_dma_kernel (fused cast)");
    return MSAMP_OK;
}

template <int XF, int YF, typename OT, bool XT, bool YT, int QF>
static int launch_gemm_dma_quant(const uint8_t* X, const uint8_t* Y, int NR, int NC, int K, const float* xs, const float* ys,
                                 const QuantArgs& qa, hipStream_t st) {
    if ((K / kBK) & 1) return launch_gemm_dma_quant_parity<XF, YF, OT, XT, YT, QF, true>(X, Y, NR, NC, K, xs, ys, qa, st);
    return launch_gemm_dma_quant_parity<XF, YF, OT, XT, YT, QF, false>(X, Y, NR, NC, K, xs, ys, qa, st);
}

// the same kernel with the cast to FP8 riding along on speculation (see QSPEC above); the caller has checked the shape
template <int XF, int YF, typename OT, bool XT, bool YT, bool ODD>
static int launch_gemm_dma_spec_parity(const uint8_t* X, const uint8_t* Y, void* D, int NR, int NC, int K, const float* xs,
                                       const float* ys, int accumulate, const QuantArgs& qa, hipStream_t st) {
    constexpr int smem = 2 * kDmaStage;
    static std::atomic<bool> configured{false};    // setting the attribute twice is harmless
    auto kern = fp8_gemm_dma_kernel<XF, YF, OT, XT, YT, 0, ODD, true>;
    if (!configured.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(fp8_gemm_dma_kernel, speculative cast)");
        configured.store(true, std::memory_order_release);
    }
    const int tiles = (NR / kDmaTile) * (NC / kDmaTile);
    QuantArgs qw = qa;
    qw.walk_plus_one = registered_walk(NR, NC, K, XT, YT) + 1;
    hipLaunchKernelGGL(kern, dim3(tiles), dim3(kGemmThreads), smem, st, X, Y, static_cast<OT*>(D), NR, NC, K, xs, ys, accumulate,
                       static_cast<const void*>(nullptr), 0, qw);
    MSAMP_CHECK_LAUNCH("fp8_gemm_dma_kernel (speculative cast)");
    return MSAMP_OK;
}

template <int XF, int YF, typename OT, bool XT, bool YT>
static int launch_gemm_dma_spec(const uint8_t* X, const uint8_t* Y, void* D, int NR, int NC, int K, const float* xs,
                                const float* ys, int accumulate, const QuantArgs& qa, hipStream_t st) {
    if ((K / kBK) & 1) return launch_gemm_dma_spec_parity<XF, YF, OT, XT, YT, true>(X, Y, D, NR, NC, K, xs, ys, accumulate, qa, st);
    return launch_gemm_dma_spec_parity<XF, YF, OT, XT, YT, false>(X, Y, D, NR, NC, K, xs, ys, accumulate, qa, st);
}

template <int BR, int BC, int XF, int YF, typename OT, bool KGUARD>
static int launch_gemm_k(const uint8_t* X, const uint8_t* Y, void* D, int NR, int NC, int K, const float* xs,
                       const float* ys, int accumulate, const void* bias, int bias_dt, hipStream_t st) {
    constexpr int smem = 2 * (BR + BC) * kBK;
    static std::atomic<bool> configured{false};    // setting the attribute twice is harmless
    auto kern = fp8_gemm_kernel<BR, BC, XF, YF, OT, KGUARD>;
    if (!configured.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(fp8_gemm_kernel)");
        configured.store(true, std::memory_order_release);
    }
    const int tiles = ((NR + BR - 1) / BR) * ((NC + BC - 1) / BC);
    hipLaunchKernelGGL(kern, dim3(tiles), dim3(kGemmThreads), smem, st, X, Y, static_cast<OT*>(D), NR, NC, K, xs, ys,
                       accumulate, bias, bias_dt);
    MSAMP_CHECK_LAUNCH("fp8_gemm_kernel");
    return MSAMP_OK;
}

template <int BR, int BC, int XF, int YF, typename OT>
static int launch_gemm(const uint8_t* X, const uint8_t* Y, void* D, int NR, int NC, int K, const float* xs,
                       const float* ys, int accumulate, const void* bias, int bias_dt, hipStream_t st) {
    if (K % kBK == 0) return launch_gemm_k<BR, BC, XF, YF, OT, false>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
    return launch_gemm_k<BR, BC, XF, YF, OT, true>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
}

}    // namespace msamp
#include "gemm_small_tile.cuh"
namespace msamp {

// few 256 x 256 tiles leave most compute units idle: 128 x 128 tiles then (takes_small_tiles(), gemm_small_tile.cuh)

template <int XF, int YF, typename OT>
static int pick_tile(const uint8_t* X, const uint8_t* Y, void* D, int NR, int NC, int K, const float* xs,
                     const float* ys, int accumulate, const void* bias, int bias_dt, hipStream_t st) {
    // the direct-to-LDS kernel needs whole 128-byte K slices, at least two of them, and 32-bit row offsets; where it can run it is the
    // faster one at every size (measured 2.2x from a single 256 x 256 tile up to 121 tiles).  Everything else takes
    // the generic register-staged kernel with 128 x 128 tiles.
    const bool fits32 = static_cast<unsigned long long>(NR) * K < (1ull << 32) && static_cast<unsigned long long>(NC) * K < (1ull << 32);
    if (fits32 && takes_small_tiles(NR, NC, K))
        return launch_gemm_dma128<XF, YF, OT>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
    if (K % kBK == 0 && K >= 2 * kBK && fits32)
        return launch_gemm_dma<XF, YF, OT>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
    return launch_gemm<128, 128, XF, YF, OT>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
}

template <int XF, int YF>
static int pick_out(const uint8_t* X, const uint8_t* Y, void* D, int d_dtype, int NR, int NC, int K, const float* xs,
                    const float* ys, int accumulate, const void* bias, int bias_dt, hipStream_t st) {
    switch (d_dtype) {
        case MSAMP_DT_F32:
            return pick_tile<XF, YF, float>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
        case MSAMP_DT_F16:
            return pick_tile<XF, YF, f16_t>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
        default:
            return pick_tile<XF, YF, bf16_t>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
    }
}

template <int XF, int YF, typename OT, bool XT, bool YT>
static int pick_tile_kmajor(const uint8_t* X, const uint8_t* Y, void* D, int NR, int NC, int K, const float* xs, const float* ys,
                            int accumulate, const void* bias, int bias_dt, hipStream_t st) {
    // (the entry point has checked the shape: whole 256-row tiles of every K-major operand, 32-bit offsets)
    if (takes_small_tiles(NR, NC, K))
        return launch_gemm_dma128<XF, YF, OT, XT, YT>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
    return launch_gemm_dma<XF, YF, OT, XT, YT>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
}

template <int XF, int YF, bool XT, bool YT>
static int pick_out_kmajor(const uint8_t* X, const uint8_t* Y, void* D, int d_dtype, int NR, int NC, int K, const float* xs,
                           const float* ys, int accumulate, const void* bias, int bias_dt, hipStream_t st) {
    switch (d_dtype) {
        case MSAMP_DT_F32:
            return pick_tile_kmajor<XF, YF, float, XT, YT>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
        case MSAMP_DT_F16:
            return pick_tile_kmajor<XF, YF, f16_t, XT, YT>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
        default:
            return pick_tile_kmajor<XF, YF, bf16_t, XT, YT>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
    }
}

template <int XF, int YF, bool T>
static int pick_out_quant(const uint8_t* X, const uint8_t* Y, int d_dtype, int NR, int NC, int K, const float* xs, const float* ys,
                          const QuantArgs& qa, hipStream_t st) {
    switch (d_dtype) {
        case MSAMP_DT_F32:
            return launch_gemm_dma_quant<XF, YF, float, T, T, MSAMP_DT_E4M3>(X, Y, NR, NC, K, xs, ys, qa, st);
        case MSAMP_DT_F16:
            return launch_gemm_dma_quant<XF, YF, f16_t, T, T, MSAMP_DT_E4M3>(X, Y, NR, NC, K, xs, ys, qa, st);
        default:
            return launch_gemm_dma_quant<XF, YF, bf16_t, T, T, MSAMP_DT_E4M3>(X, Y, NR, NC, K, xs, ys, qa, st);
    }
}

template <int XF, int YF, bool T>
static int pick_out_spec(const uint8_t* X, const uint8_t* Y, void* D, int d_dtype, int NR, int NC, int K, const float* xs,
                         const float* ys, int accumulate, const QuantArgs& qa, hipStream_t st) {
    switch (d_dtype) {
        case MSAMP_DT_F32:
            // a float32 product takes the two steps: with four-byte outputs the epilogue that also emits codes does not
            // fit the vector registers left beside the accumulators
            return MSAMP_NOT_FUSED;
        case MSAMP_DT_F16:
            return launch_gemm_dma_spec<XF, YF, f16_t, T, T>(X, Y, D, NR, NC, K, xs, ys, accumulate, qa, st);
        default:
            return launch_gemm_dma_spec<XF, YF, bf16_t, T, T>(X, Y, D, NR, NC, K, xs, ys, accumulate, qa, st);
    }
}

#ifdef MSAMP_GEMM_SPLIT_UNIT
template <int XF, int YF>
int run_gemm_split(const uint8_t* X, const uint8_t* Y, void* D, int d_dtype, int NR, int NC, int K, const float* xs,
                   const float* ys, int accumulate, const void* bias, int bias_dt, hipStream_t st) {
    const bool odd = (K / kBK) & 1;
#define MSAMP_SPLIT_LAUNCH(OT)                                                                                                         \
    return odd ? launch_gemm_dma_parity<XF, YF, OT, false, false, true, true>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st) \
               : launch_gemm_dma_parity<XF, YF, OT, false, false, false, true>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st)
    switch (d_dtype) {
        case MSAMP_DT_F32: MSAMP_SPLIT_LAUNCH(float);
        case MSAMP_DT_F16: MSAMP_SPLIT_LAUNCH(f16_t);
        default: MSAMP_SPLIT_LAUNCH(bf16_t);
    }
#undef MSAMP_SPLIT_LAUNCH
}
#endif

// Everything behind the C entry points for one pair of operand formats.  gemm_inst.hip instantiates it once per
// pair (four translation units, so that they compile side by side).
template <int XF, int YF>
int run_gemm_pair(const GemmCall& c) {
    if (c.qa != nullptr && c.qspec) {
        if (c.xt) return pick_out_spec<XF, YF, true>(c.X, c.Y, c.D, c.d_dtype, c.NR, c.NC, c.K, c.xs, c.ys, c.accumulate, *c.qa, c.st);
        return pick_out_spec<XF, YF, false>(c.X, c.Y, c.D, c.d_dtype, c.NR, c.NC, c.K, c.xs, c.ys, c.accumulate, *c.qa, c.st);
    }
    if (c.qa != nullptr) {
        if (c.xt) return pick_out_quant<XF, YF, true>(c.X, c.Y, c.d_dtype, c.NR, c.NC, c.K, c.xs, c.ys, *c.qa, c.st);
        return pick_out_quant<XF, YF, false>(c.X, c.Y, c.d_dtype, c.NR, c.NC, c.K, c.xs, c.ys, *c.qa, c.st);
    }
    if (c.xt && c.yt)
        return pick_out_kmajor<XF, YF, true, true>(c.X, c.Y, c.D, c.d_dtype, c.NR, c.NC, c.K, c.xs, c.ys, c.accumulate, c.bias, c.bias_dt, c.st);
    if (c.yt)
        return pick_out_kmajor<XF, YF, false, true>(c.X, c.Y, c.D, c.d_dtype, c.NR, c.NC, c.K, c.xs, c.ys, c.accumulate, c.bias, c.bias_dt, c.st);
    return pick_out<XF, YF>(c.X, c.Y, c.D, c.d_dtype, c.NR, c.NC, c.K, c.xs, c.ys, c.accumulate, c.bias, c.bias_dt, c.st);
}

}    // namespace msamp
