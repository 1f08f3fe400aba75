// What the C entry points of the FP8 GEMM hand to the kernels' translation units.
#pragma once

#include "common.cuh"

namespace msamp {

constexpr int kBK = 128;         // K bytes per LDS stage
constexpr int kDmaTile = 256;    // output tile edge of the direct-to-LDS kernel

struct QuantArgs {
    uint8_t* q;          // [NR][NC] FP8 codes
    float* scale;        // in: the fallback of the scale rule; out: the scale used
    float* amax;         // out: max |D|
    float* scale_inv;    // out: 1 / scale
    uint64_t* slots;     // kMaxSlots meeting slots and two post words
    float fp_max;
    int margin;
    int flags;
    uint32_t token;
    uint32_t spin_limit;
    uint32_t* error_word;    // sticky: set when a bounded wait runs out
    uint32_t* spec_words;    // speculative form: [0] running maximum, [1] ticket counter (both zero between calls), [2] out: 1 = cast again
    int walk_plus_one;       // every form of the kernel: 0 = the tile walk the built-in rule picks, 1..4 = walk 0..3 (see registered_walk)
};

// One product D[NR][NC] = X[NR][K] . Y[NC][K]^T * *xs * *ys.  xt / yt: that operand is handed over K-major.
// qa != nullptr: the output is cast on to FP8 in the same launch; D is not written, unless `qspec` asks for the
// speculative form, which stores D as usual and the codes of D times the scale in force next to it.
struct GemmCall {
    const uint8_t* X;
    const uint8_t* Y;
    void* D;
    int d_dtype;
    int NR, NC, K;
    const float* xs;
    const float* ys;
    int accumulate;
    const void* bias;
    int bias_dt;
    bool xt, yt;
    const QuantArgs* qa;
    hipStream_t st;
    bool qspec = false;
};

template <int XF, int YF>
int run_gemm_pair(const GemmCall& c);
// The split-wait instantiations of the 256 x 256-tile kernel for one pair of formats (row-major operands, all three
// output types, both parities of the slice count).  They live in translation units of their own (gemm_inst.hip built
// with -DMSAMP_GEMM_SPLIT_UNIT) so that they compile beside the others instead of after them.
template <int XF, int YF>
int run_gemm_split(const uint8_t* X, const uint8_t* Y, void* D, int d_dtype, int NR, int NC, int K, const float* xs,
                   const float* ys, int accumulate, const void* bias, int bias_dt, hipStream_t st);

// Problems of at most this many 256 x 256 tiles take the kernel with 128 x 128 tiles (msamp_set_small_tile_limit) ...
int small_tile_limit();
// The tile walk registered for this problem of the 256 x 256-tile kernel (msamp_fp8_gemm_set_walk / _tune), or -1: bit 0 =
// groups of tile columns walked row by row instead of groups of tile rows, bit 1 = the XCD's patch of 32 tiles turned (4 of
// the grouped dimension x 8 of the walked one).  Any walk gives the same output bits: it only decides which workgroup
// takes which tile.  Bit 2 (row-major operands only): the tile loads awaited in two parts, see the kernel.
int registered_walk(int NR, int NC, int K, bool XT, bool YT);
// ... which is this rule: K in whole slices, at least four of them; up to half the limit always (one small tile per
// compute unit with the default limit), up to the limit where K is long enough for the second round of small tiles to
// pay (measured: 128 large tiles level at K = 2048, 15 % ahead at 4096).
inline bool takes_small_tiles(int NR, int NC, int K) {
    const long big_tiles = static_cast<long>((NR + kDmaTile - 1) / kDmaTile) * ((NC + kDmaTile - 1) / kDmaTile);
    const int limit = small_tile_limit();
    return K % kBK == 0 && K >= 4 * kBK && (big_tiles <= limit / 2 || (big_tiles <= limit && K >= 3072));
}

// Implemented with the cast kernels: q = FP8(d * *scale) over n elements, unless *redo is zero (then nothing is done).
int cast_again_if_flagged(const void* d, int d_dtype, size_t n, const float* scale, uint8_t* q, int q_type, const uint32_t* redo,
                          hipStream_t st);

extern template int run_gemm_pair<MSAMP_DT_E4M3, MSAMP_DT_E4M3>(const GemmCall&);
extern template int run_gemm_pair<MSAMP_DT_E4M3, MSAMP_DT_E5M2>(const GemmCall&);
extern template int run_gemm_pair<MSAMP_DT_E5M2, MSAMP_DT_E4M3>(const GemmCall&);
extern template int run_gemm_pair<MSAMP_DT_E5M2, MSAMP_DT_E5M2>(const GemmCall&);
#define MSAMP_SPLIT_ARGS const uint8_t*, const uint8_t*, void*, int, int, int, int, const float*, const float*, int, const void*, int, hipStream_t
extern template int run_gemm_split<MSAMP_DT_E4M3, MSAMP_DT_E4M3>(MSAMP_SPLIT_ARGS);
extern template int run_gemm_split<MSAMP_DT_E4M3, MSAMP_DT_E5M2>(MSAMP_SPLIT_ARGS);
extern template int run_gemm_split<MSAMP_DT_E5M2, MSAMP_DT_E4M3>(MSAMP_SPLIT_ARGS);
extern template int run_gemm_split<MSAMP_DT_E5M2, MSAMP_DT_E5M2>(MSAMP_SPLIT_ARGS);

}    // namespace msamp
