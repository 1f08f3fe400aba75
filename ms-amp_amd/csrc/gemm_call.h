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
};

// One product D[NR][NC] = X[NR][K] . Y[NC][K]^T * *xs * *ys.  xt / yt: that operand is handed over K-major.
// qa != nullptr: the output is cast on to FP8 in the same launch and D is not written.
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
};

template <int XF, int YF>
int run_gemm_pair(const GemmCall& c);

extern template int run_gemm_pair<MSAMP_DT_E4M3, MSAMP_DT_E4M3>(const GemmCall&);
extern template int run_gemm_pair<MSAMP_DT_E4M3, MSAMP_DT_E5M2>(const GemmCall&);
extern template int run_gemm_pair<MSAMP_DT_E5M2, MSAMP_DT_E4M3>(const GemmCall&);
extern template int run_gemm_pair<MSAMP_DT_E5M2, MSAMP_DT_E5M2>(const GemmCall&);

}    // namespace msamp
