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
#include "common.cuh"

namespace msamp {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kGemmThreads = 256;
constexpr int kBK = 128;    // K bytes per stage

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

template <int XF, int YF>
__device__ __forceinline__ v16f mfma(const v8i& x, const v8i& y, const v16f& c) {
    constexpr int cb = (XF == MSAMP_DT_E4M3) ? 0 : 1;
    constexpr int bl = (YF == MSAMP_DT_E4M3) ? 0 : 1;
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(x, y, c, cb, bl, 0, 0, 0, 0);
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

// workgroup id -> tile, keeping the workgroups of one XCD on adjacent tiles and walking groups of
// `kGroup` tile rows column by column so that the X and Y panels of a group stay in that L2
__device__ __forceinline__ void tile_of_block(int tiles_r, int tiles_c, int& tr, int& tc) {
    constexpr int kXcd = 8, kGroup = 8;
    const int nt = tiles_r * tiles_c;
    int id = blockIdx.x;
    if (nt % kXcd == 0) id = (id % kXcd) * (nt / kXcd) + id / kXcd;
    const int per_group = kGroup * tiles_c;
    const int g = id / per_group;
    const int first_r = g * kGroup;
    const int rows_here = (tiles_r - first_r) < kGroup ? (tiles_r - first_r) : kGroup;
    const int in_g = id - g * per_group;
    tr = first_r + in_g % rows_here;
    tc = in_g / rows_here;
}

template <int BR, int BC, int XF, int YF, typename OT, bool KGUARD>
__global__ __launch_bounds__(kGemmThreads) void fp8_gemm_kernel(const uint8_t* __restrict__ X,
                                                                 const uint8_t* __restrict__ Y, OT* __restrict__ D,
                                                                 int NR, int NC, int K,
                                                                 const float* __restrict__ x_scale_inv,
                                                                 const float* __restrict__ y_scale_inv, int accumulate,
                                                                 const void* __restrict__ bias, int bias_dt) {
    constexpr int WR = BR / 2, WC = BC / 2;    // wave tile
    constexpr int TR = WR / 32, TC = WC / 32;  // MFMA tiles per wave
    constexpr int kStage = (BR + BC) * kBK;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    int tr, tc;
    tile_of_block((NR + BR - 1) / BR, (NC + BC - 1) / BC, tr, tc);
    const int row0 = tr * BR, col0 = tc * BC;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wr = wave >> 1, wc = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;

    v16f acc[TR][TC];
#pragma unroll
    for (int i = 0; i < TR; ++i)
#pragma unroll
        for (int j = 0; j < TC; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    TileLoader<BR, KGUARD> lx;
    TileLoader<BC, KGUARD> ly;
    const int nk = (K + kBK - 1) / kBK;
    lx.gload(X, row0, NR, K, 0);
    ly.gload(Y, col0, NC, K, 0);
    lx.lstore(smem);
    ly.lstore(smem + BR * kBK);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
        const uint8_t* sx = smem + (kt & 1) * kStage;
        const uint8_t* sy = sx + BR * kBK;
        if (kt + 1 < nk) {
            lx.gload(X, row0, NR, K, (kt + 1) * kBK);
            ly.gload(Y, col0, NC, K, (kt + 1) * kBK);
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            v8i fx[TR], fy[TC];
#pragma unroll
            for (int i = 0; i < TR; ++i) fx[i] = read_frag(sx, wr * WR + i * 32 + l32, ks * 2 + lh);
#pragma unroll
            for (int j = 0; j < TC; ++j) fy[j] = read_frag(sy, wc * WC + j * 32 + l32, ks * 2 + lh);
#pragma unroll
            for (int i = 0; i < TR; ++i)
#pragma unroll
                for (int j = 0; j < TC; ++j) acc[i][j] = mfma<XF, YF>(fx[i], fy[j], acc[i][j]);
        }
        if (kt + 1 < nk) {
            uint8_t* nx = smem + ((kt + 1) & 1) * kStage;
            lx.lstore(nx);
            ly.lstore(nx + BR * kBK);
        }
        __syncthreads();
    }

    const float alpha = (*x_scale_inv) * (*y_scale_inv);
#pragma unroll
    for (int j = 0; j < TC; ++j) {
        const int col = col0 + wc * WC + j * 32 + l32;
        if (col >= NC) continue;
        const float bv = bias != nullptr ? load_bias(bias, bias_dt, col) : 0.0f;
#pragma unroll
        for (int i = 0; i < TR; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = row0 + wr * WR + i * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                if (row < NR) {
                    store_out<OT>(D + static_cast<size_t>(row) * NC + col, acc[i][j][r] * alpha + bv, accumulate != 0);
                }
            }
        }
    }
}

template <int BR, int BC, int XF, int YF, typename OT, bool KGUARD>
static int launch_gemm_k(const uint8_t* X, const uint8_t* Y, void* D, int NR, int NC, int K, const float* xs,
                       const float* ys, int accumulate, const void* bias, int bias_dt, hipStream_t st) {
    constexpr int smem = 2 * (BR + BC) * kBK;
    static bool configured = false;
    auto kern = fp8_gemm_kernel<BR, BC, XF, YF, OT, KGUARD>;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(fp8_gemm_kernel)");
        configured = true;
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

template <int XF, int YF, typename OT>
static int pick_tile(const uint8_t* X, const uint8_t* Y, void* D, int NR, int NC, int K, const float* xs,
                     const float* ys, int accumulate, const void* bias, int bias_dt, hipStream_t st) {
    // large tiles once they fill the chip at least once; otherwise smaller ones for more workgroups
    const long big = static_cast<long>((NR + 255) / 256) * ((NC + 255) / 256);
    if (big >= cu_count()) return launch_gemm<256, 256, XF, YF, OT>(X, Y, D, NR, NC, K, xs, ys, accumulate, bias, bias_dt, st);
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

}    // namespace msamp

using namespace msamp;

extern "C" int msamp_fp8_gemm(const uint8_t* a, int a_type, const float* a_scale_inv, const uint8_t* b, int b_type,
                              const float* b_scale_inv, void* d, int d_dtype, int m, int n, int k, int accumulate,
                              const void* bias, int bias_dtype, msamp_stream_t stream) {
    MSAMP_REQUIRE(is_fp8(a_type) && is_fp8(b_type), MSAMP_ERR_DTYPE, "msamp_fp8_gemm: operand types %d, %d", a_type, b_type);
    MSAMP_REQUIRE(is_hp(d_dtype), MSAMP_ERR_DTYPE, "msamp_fp8_gemm: output dtype %d", d_dtype);
    MSAMP_REQUIRE(bias == nullptr || is_hp(bias_dtype), MSAMP_ERR_DTYPE, "msamp_fp8_gemm: bias dtype %d", bias_dtype);
    MSAMP_REQUIRE(m >= 0 && n >= 0 && k >= 0, MSAMP_ERR_SHAPE, "msamp_fp8_gemm: m=%d n=%d k=%d", m, n, k);
    if (m == 0 || n == 0) return MSAMP_OK;
    MSAMP_REQUIRE(k > 0 && k % 16 == 0, MSAMP_ERR_SHAPE, "msamp_fp8_gemm: k=%d must be a positive multiple of 16", k);
    MSAMP_REQUIRE(a && b && d && a_scale_inv && b_scale_inv, MSAMP_ERR_NULL, "msamp_fp8_gemm: null pointer");
    MSAMP_REQUIRE(aligned(a, 16) && aligned(b, 16), MSAMP_ERR_SHAPE, "msamp_fp8_gemm: operands must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    // X = b (rows of D), Y = a (columns of D)
    if (b_type == MSAMP_DT_E4M3 && a_type == MSAMP_DT_E4M3)
        return pick_out<MSAMP_DT_E4M3, MSAMP_DT_E4M3>(b, a, d, d_dtype, n, m, k, b_scale_inv, a_scale_inv, accumulate, bias, bias_dtype, st);
    if (b_type == MSAMP_DT_E4M3)
        return pick_out<MSAMP_DT_E4M3, MSAMP_DT_E5M2>(b, a, d, d_dtype, n, m, k, b_scale_inv, a_scale_inv, accumulate, bias, bias_dtype, st);
    if (a_type == MSAMP_DT_E4M3)
        return pick_out<MSAMP_DT_E5M2, MSAMP_DT_E4M3>(b, a, d, d_dtype, n, m, k, b_scale_inv, a_scale_inv, accumulate, bias, bias_dtype, st);
    return pick_out<MSAMP_DT_E5M2, MSAMP_DT_E5M2>(b, a, d, d_dtype, n, m, k, b_scale_inv, a_scale_inv, accumulate, bias, bias_dtype, st);
}
