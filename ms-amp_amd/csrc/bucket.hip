// Quantizing a bucket of high-precision gradients into one flat FP8 buffer, many tensors per launch: the
// compute steps of the FP8 gradient reducer (msamp/nn/distributed.py:143-184) either side of its amax
// all-reduce.  One workgroup handles one 16384-element chunk of one tensor; a device table describes the
// tensors and a block map assigns the chunks, as in the fused AdamW step.
#include "common.cuh"

namespace msamp {

constexpr int kBucketThreads = 256;

// max |x| of one chunk, as the bit pattern of the float (a NaN pattern compares above every number, so it wins)
// FMT != 0: the chunk is also quantized, with the scale the item has now, into its place in the flat buffer.  That
// scale is what the previous round's msamp_bucket_cast left there, and it is a power of two times a constant, so it is
// as a rule the scale this round will arrive at; msamp_bucket_cast then finds its work done (see bucket_scale_kernel).
template <typename IT, int FMT>
__global__ __launch_bounds__(kBucketThreads) void bucket_amax_kernel(msamp_bucket_item* __restrict__ items,
                                                                     const int32_t* __restrict__ block_map, int stream) {
    constexpr int EPT = In16<IT>::EPT;
    constexpr int kVecs = MSAMP_BUCKET_CHUNK / (kBucketThreads * EPT);    // 16 (fp32) or 8 (16-bit)
    __shared__ uint32_t red[kBucketThreads / kWave];
    const int t = block_map[2 * blockIdx.x], chunk = block_map[2 * blockIdx.x + 1];
    msamp_bucket_item& d = items[t];
    const IT* x = static_cast<const IT*>(d.src);
    const size_t n = d.numel, base = static_cast<size_t>(chunk) * MSAMP_BUCKET_CHUNK;
    uint32_t m = 0;
    uint8_t* out = d.dst;
    const float s = FMT != 0 ? *d.scale : 1.0f;
    const bool vec_out = FMT == 0 || (reinterpret_cast<uintptr_t>(out) & (EPT - 1)) == 0;
    if (base + MSAMP_BUCKET_CHUNK <= n && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && vec_out) {
        float v[kVecs][EPT];
#pragma unroll
        for (int u = 0; u < kVecs; ++u)
            In16<IT>::load(x + base + (static_cast<size_t>(u) * kBucketThreads + threadIdx.x) * EPT, v[u], stream != 0);
#pragma unroll
        for (int u = 0; u < kVecs; ++u) {
#pragma unroll
            for (int j = 0; j < EPT; ++j) {
                const uint32_t a = __float_as_uint(v[u][j]) & 0x7fffffffu;
                m = a > m ? a : m;
            }
            if constexpr (FMT != 0) {
                uint32_t w[EPT / 4];
#pragma unroll
                for (int j = 0; j < EPT / 4; ++j)
                    w[j] = quant4<FMT>(v[u][4 * j] * s, v[u][4 * j + 1] * s, v[u][4 * j + 2] * s, v[u][4 * j + 3] * s);
                uint8_t* o = out + base + (static_cast<size_t>(u) * kBucketThreads + threadIdx.x) * EPT;
                if constexpr (EPT == 4) {
                    *reinterpret_cast<uint32_t*>(o) = w[0];
                } else {
                    *reinterpret_cast<uint2*>(o) = make_uint2(w[0], w[1]);
                }
            }
        }
    } else {
        for (size_t i = base + threadIdx.x; i < n && i < base + MSAMP_BUCKET_CHUNK; i += kBucketThreads) {
            const float xi = Elem<IT>::load(x + i);
            const uint32_t a = __float_as_uint(xi) & 0x7fffffffu;
            m = a > m ? a : m;
            if constexpr (FMT != 0) out[i] = static_cast<uint8_t>(quant1<FMT>(xi * s));
        }
    }
    m = block_max_u32(m, red);
    if (threadIdx.x == 0 && m) atomicMax(&d.acc, m);
}

// amax[0] of every tensor from the accumulated pattern (NaN and +Inf become +Inf when asked: the all-reduce that
// follows in the reducer ignores NaN); the accumulator goes back to zero
constexpr uint32_t kBucketDone = 0xffffffffu;    // item.reserved: the buffer already holds this round's codes

__global__ void bucket_amax_finish_kernel(msamp_bucket_item* items, int n_items, int flags, int speculative) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_items) return;
    msamp_bucket_item& d = items[t];
    float a = __uint_as_float(d.acc);
    d.acc = 0u;
    // the scale the codes were written with, if they were (a positive finite one: anything else is no guess)
    const float guess = *d.scale;
    d.reserved = (speculative && guess > 0.0f && guess < __uint_as_float(0x7f800000u)) ? __float_as_uint(guess) : 0u;
    if ((flags & MSAMP_FLAG_NAN_TO_INF) && !(a < __uint_as_float(0x7f800000u))) a = __uint_as_float(0x7f800000u);
    *d.amax = a;
}

// scale = rule(amax[0], fallback = the scale in force) * pre_scale, scale_inv = (1 / scale) / inv_div (the reducer
// divides the finished ScalingTensor by the world size, which is a division of scale_inv: two roundings, kept)
__global__ void bucket_scale_kernel(msamp_bucket_item* items, int n_items, float fp_max, int margin, float pre_scale,
                                    float inv_div) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_items) return;
    msamp_bucket_item& d = items[t];
    const float sf = scale_rule(*d.amax, *d.scale, fp_max, margin) * pre_scale;
    // after msamp_bucket_amax_speculative: did the codes go out with this very scale?  (A mark left by an earlier cast
    // of the same round is no guess: a second cast without a new amax pass writes the codes again.)
    if (d.reserved != 0u) d.reserved = (d.reserved != kBucketDone && __float_as_uint(sf) == d.reserved) ? kBucketDone : 0u;
    *d.scale = sf;
    const float inv = 1.0f / sf;
    *d.scale_inv = inv / inv_div;
}

template <typename IT, int FMT>
__global__ __launch_bounds__(kBucketThreads) void bucket_cast_kernel(const msamp_bucket_item* __restrict__ items,
                                                                     const int32_t* __restrict__ block_map, int stream) {
    constexpr int EPT = In16<IT>::EPT;
    constexpr int kVecs = MSAMP_BUCKET_CHUNK / (kBucketThreads * EPT);
    const int t = block_map[2 * blockIdx.x], chunk = block_map[2 * blockIdx.x + 1];
    const msamp_bucket_item& d = items[t];
    if (d.reserved == kBucketDone) return;    // written by the speculative first pass with the scale that came out
    const IT* x = static_cast<const IT*>(d.src);
    uint8_t* out = d.dst;
    const float s = *d.scale;
    const size_t n = d.numel, base = static_cast<size_t>(chunk) * MSAMP_BUCKET_CHUNK;
    // a tensor's place in the flat buffer follows from the sizes before it: vector stores only where it allows
    const bool vec = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & (EPT - 1)) == 0;
    if (base + MSAMP_BUCKET_CHUNK <= n && vec) {
        float v[kVecs][EPT];
#pragma unroll
        for (int u = 0; u < kVecs; ++u)
            In16<IT>::load(x + base + (static_cast<size_t>(u) * kBucketThreads + threadIdx.x) * EPT, v[u], stream != 0);
#pragma unroll
        for (int u = 0; u < kVecs; ++u) {
            uint32_t w[EPT / 4];
#pragma unroll
            for (int j = 0; j < EPT / 4; ++j)
                w[j] = quant4<FMT>(v[u][4 * j] * s, v[u][4 * j + 1] * s, v[u][4 * j + 2] * s, v[u][4 * j + 3] * s);
            uint8_t* o = out + base + (static_cast<size_t>(u) * kBucketThreads + threadIdx.x) * EPT;
            if constexpr (EPT == 4) {
                *reinterpret_cast<uint32_t*>(o) = w[0];
            } else {
                *reinterpret_cast<uint2*>(o) = make_uint2(w[0], w[1]);
            }
        }
    } else {
        for (size_t i = base + threadIdx.x; i < n && i < base + MSAMP_BUCKET_CHUNK; i += kBucketThreads)
            out[i] = static_cast<uint8_t>(quant1<FMT>(Elem<IT>::load(x + i) * s));
    }
}

// ---- norms of FP8 gradients (clip_grad_norm_) ----------------------------------------------------------------
// sum |q|^p (p = 1, 2) or max |q| over the codes of each tensor, accumulated in double (four elements at a time are
// summed in float32 first): the dequantization factor
// is constant per tensor and is applied once at the end, so a tensor is read at one byte per element and never
// expanded to float32 in memory.
template <int FMT, int KIND>    // KIND: 1, 2, or 0 for the maximum
__global__ __launch_bounds__(kBucketThreads) void fp8_norm_kernel(msamp_norm_item* __restrict__ items,
                                                                   const int32_t* __restrict__ block_map) {
    __shared__ double red[kBucketThreads / kWave];
    const int t = block_map[2 * blockIdx.x], chunk = block_map[2 * blockIdx.x + 1];
    msamp_norm_item& d = items[t];
    const uint8_t* q = d.q;
    const size_t n = d.numel, base = static_cast<size_t>(chunk) * MSAMP_BUCKET_CHUNK;
    double acc = 0.0;
    auto take = [&](float v) {
        const double a = fabs(static_cast<double>(v));
        if constexpr (KIND == 0) {
            acc = (a != a || acc != acc) ? (a != a ? a : acc) : (a > acc ? a : acc);    // NaN stays
        } else if constexpr (KIND == 1) {
            acc += a;
        } else {
            acc = fma(a, a, acc);
        }
    };
    if (base + MSAMP_BUCKET_CHUNK <= n && (reinterpret_cast<uintptr_t>(q) & 15) == 0) {
        constexpr int kVecs = MSAMP_BUCKET_CHUNK / (kBucketThreads * 16);    // 4
        uint4 w[kVecs];
#pragma unroll
        for (int u = 0; u < kVecs; ++u)
            w[u] = *reinterpret_cast<const uint4*>(q + base + (static_cast<size_t>(u) * kBucketThreads + threadIdx.x) * 16);
#pragma unroll
        for (int u = 0; u < kVecs; ++u) {
            const uint32_t words[4] = {w[u].x, w[u].y, w[u].z, w[u].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float a, b, c, e;
                dequant4<FMT>(words[j], a, b, c, e);
                if constexpr (KIND == 0) {
                    take(a), take(b), take(c), take(e);
                } else if constexpr (KIND == 1) {
                    // four values at a time in float32 (three roundings of 2^-24 each), then into the double sum: a
                    // double conversion and addition per element kept the vector units busier than the memory
                    acc += static_cast<double>((fabsf(a) + fabsf(b)) + (fabsf(c) + fabsf(e)));
                } else {
                    // the square of an FP8 value is exact in float32
                    acc += static_cast<double>(fmaf(a, a, b * b) + fmaf(c, c, e * e));
                }
            }
        }
    } else {
        for (size_t i = base + threadIdx.x; i < n && i < base + MSAMP_BUCKET_CHUNK; i += kBucketThreads) take(dequant1<FMT>(q[i]));
    }
    // workgroup total (maximum): lanes, then wavefronts
#pragma unroll
    for (int o = 32; o; o >>= 1) {
        const double other = __shfl_xor(acc, o);
        if constexpr (KIND == 0) {
            acc = (other != other || acc != acc) ? (other != other ? other : acc) : (other > acc ? other : acc);
        } else {
            acc += other;
        }
    }
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double total = red[0];
        for (int w = 1; w < kBucketThreads / kWave; ++w) {
            if constexpr (KIND == 0) {
                total = (red[w] != red[w] || total != total) ? (red[w] != red[w] ? red[w] : total) : (red[w] > total ? red[w] : total);
            } else {
                total += red[w];
            }
        }
        if constexpr (KIND == 0) {
            // bit patterns of non-negative doubles order like the values, NaN patterns above all of them
            atomicMax(reinterpret_cast<unsigned long long*>(&d.acc), static_cast<unsigned long long>(__double_as_longlong(total)));
        } else {
            atomicAdd(&d.acc, total);
        }
    }
}

// out[i] = |scale_inv| * acc^(1/p) (the maximum itself for KIND 0), rounded to float once; the accumulator goes back to zero
__global__ void fp8_norm_finish_kernel(msamp_norm_item* items, int n_items, int kind) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_items) return;
    msamp_norm_item& d = items[t];
    const double acc = d.acc;
    d.acc = 0.0;
    const double root = kind == 2 ? sqrt(acc) : acc;
    *d.out = static_cast<float>(fabs(static_cast<double>(*d.scale_inv)) * root);
}

static int check_bucket_args(const char* who, const msamp_bucket_item* items, int n_items, const int32_t* block_map,
                             int n_blocks, int in_dtype) {
    MSAMP_REQUIRE(n_items >= 0 && n_blocks >= 0, MSAMP_ERR_SHAPE, "%s: n_items=%d n_blocks=%d", who, n_items, n_blocks);
    MSAMP_REQUIRE(is_hp(in_dtype), MSAMP_ERR_DTYPE, "%s: in_dtype %d", who, in_dtype);
    MSAMP_REQUIRE(n_items == 0 || items != nullptr, MSAMP_ERR_NULL, "%s: null descriptor table", who);
    MSAMP_REQUIRE(n_blocks == 0 || block_map != nullptr, MSAMP_ERR_NULL, "%s: null block map", who);
    return MSAMP_OK;
}

}    // namespace msamp

using namespace msamp;

extern "C" {

static int bucket_amax_launch(const char* who, msamp_bucket_item* items, int n_items, const int32_t* block_map, int n_blocks,
                              int in_dtype, int fp8_type, int flags, msamp_stream_t stream) {
    const int rc = check_bucket_args(who, items, n_items, block_map, n_blocks, in_dtype);
    if (rc != MSAMP_OK || n_items == 0) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // more bytes than the caches keep: read them as a stream
    const int in_size = in_dtype == MSAMP_DT_F32 ? 4 : 2;
    const int streams = static_cast<size_t>(n_blocks) * MSAMP_BUCKET_CHUNK * in_size >= kStreamBytes ? 1 : 0;
    if (n_blocks > 0) {
#define BUCKET_AMAX(IT)                                                                                                 \
    do {                                                                                                              \
        if (fp8_type == MSAMP_DT_E4M3)                                                                                \
            hipLaunchKernelGGL((bucket_amax_kernel<IT, MSAMP_DT_E4M3>), dim3(n_blocks), dim3(kBucketThreads), 0, st, items, block_map, streams); \
        else if (fp8_type == MSAMP_DT_E5M2)                                                                           \
            hipLaunchKernelGGL((bucket_amax_kernel<IT, MSAMP_DT_E5M2>), dim3(n_blocks), dim3(kBucketThreads), 0, st, items, block_map, streams); \
        else                                                                                                          \
            hipLaunchKernelGGL((bucket_amax_kernel<IT, 0>), dim3(n_blocks), dim3(kBucketThreads), 0, st, items, block_map, streams); \
    } while (0)
        if (in_dtype == MSAMP_DT_F32) BUCKET_AMAX(float);
        else if (in_dtype == MSAMP_DT_F16) BUCKET_AMAX(f16_t);
        else BUCKET_AMAX(bf16_t);
#undef BUCKET_AMAX
        MSAMP_CHECK_LAUNCH("bucket_amax_kernel");
    }
    hipLaunchKernelGGL(bucket_amax_finish_kernel, dim3((n_items + 63) / 64), dim3(64), 0, st, items, n_items, flags,
                       fp8_type != 0 ? 1 : 0);
    MSAMP_CHECK_LAUNCH("bucket_amax_finish_kernel");
    return MSAMP_OK;
}

int msamp_bucket_amax(msamp_bucket_item* items, int n_items, const int32_t* block_map, int n_blocks, int in_dtype, int flags,
                      msamp_stream_t stream) {
    return bucket_amax_launch("msamp_bucket_amax", items, n_items, block_map, n_blocks, in_dtype, 0, flags, stream);
}

int msamp_bucket_amax_speculative(msamp_bucket_item* items, int n_items, const int32_t* block_map, int n_blocks, int in_dtype,
                                  int fp8_type, int flags, msamp_stream_t stream) {
    MSAMP_REQUIRE(is_fp8(fp8_type), MSAMP_ERR_DTYPE, "msamp_bucket_amax_speculative: fp8_type %d", fp8_type);
    return bucket_amax_launch("msamp_bucket_amax_speculative", items, n_items, block_map, n_blocks, in_dtype, fp8_type, flags,
                              stream);
}

int msamp_bucket_cast(msamp_bucket_item* items, int n_items, const int32_t* block_map, int n_blocks, int in_dtype,
                      int fp8_type, float pre_scale, float scale_inv_div, int margin, msamp_stream_t stream) {
    const int rc = check_bucket_args("msamp_bucket_cast", items, n_items, block_map, n_blocks, in_dtype);
    if (rc != MSAMP_OK) return rc;
    MSAMP_REQUIRE(is_fp8(fp8_type), MSAMP_ERR_DTYPE, "msamp_bucket_cast: fp8_type %d", fp8_type);
    if (n_items == 0) return MSAMP_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(bucket_scale_kernel, dim3((n_items + 63) / 64), dim3(64), 0, st, items, n_items, fp8_max(fp8_type),
                       margin, pre_scale, scale_inv_div);
    MSAMP_CHECK_LAUNCH("bucket_scale_kernel");
    if (n_blocks == 0) return MSAMP_OK;
    const int in_size = in_dtype == MSAMP_DT_F32 ? 4 : 2;
    const int streams = static_cast<size_t>(n_blocks) * MSAMP_BUCKET_CHUNK * in_size >= kStreamBytes ? 1 : 0;
#define BUCKET_CAST(IT)                                                                                                  \
    do {                                                                                                               \
        if (fp8_type == MSAMP_DT_E4M3)                                                                                 \
            hipLaunchKernelGGL((bucket_cast_kernel<IT, MSAMP_DT_E4M3>), dim3(n_blocks), dim3(kBucketThreads), 0, st, items, block_map, streams); \
        else                                                                                                           \
            hipLaunchKernelGGL((bucket_cast_kernel<IT, MSAMP_DT_E5M2>), dim3(n_blocks), dim3(kBucketThreads), 0, st, items, block_map, streams); \
    } while (0)
    if (in_dtype == MSAMP_DT_F32) BUCKET_CAST(float);
    else if (in_dtype == MSAMP_DT_F16) BUCKET_CAST(f16_t);
    else BUCKET_CAST(bf16_t);
#undef BUCKET_CAST
    MSAMP_CHECK_LAUNCH("bucket_cast_kernel");
    return MSAMP_OK;
}

int msamp_fp8_norms(msamp_norm_item* items, int n_items, const int32_t* block_map, int n_blocks, int fp8_type, int norm_kind,
                    msamp_stream_t stream) {
    MSAMP_REQUIRE(n_items >= 0 && n_blocks >= 0, MSAMP_ERR_SHAPE, "msamp_fp8_norms: n_items=%d n_blocks=%d", n_items, n_blocks);
    MSAMP_REQUIRE(is_fp8(fp8_type), MSAMP_ERR_DTYPE, "msamp_fp8_norms: fp8_type %d", fp8_type);
    MSAMP_REQUIRE(norm_kind >= 0 && norm_kind <= 2, MSAMP_ERR_SHAPE, "msamp_fp8_norms: norm_kind %d (1, 2, or 0 for the maximum)",
                  norm_kind);
    if (n_items == 0) return MSAMP_OK;
    MSAMP_REQUIRE(items != nullptr && (n_blocks == 0 || block_map != nullptr), MSAMP_ERR_NULL, "msamp_fp8_norms: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (n_blocks > 0) {
#define NORM_LAUNCH(FMT)                                                                                                \
    do {                                                                                                              \
        if (norm_kind == 0)                                                                                           \
            hipLaunchKernelGGL((fp8_norm_kernel<FMT, 0>), dim3(n_blocks), dim3(kBucketThreads), 0, st, items, block_map); \
        else if (norm_kind == 1)                                                                                      \
            hipLaunchKernelGGL((fp8_norm_kernel<FMT, 1>), dim3(n_blocks), dim3(kBucketThreads), 0, st, items, block_map); \
        else                                                                                                          \
            hipLaunchKernelGGL((fp8_norm_kernel<FMT, 2>), dim3(n_blocks), dim3(kBucketThreads), 0, st, items, block_map); \
    } while (0)
        if (fp8_type == MSAMP_DT_E4M3) NORM_LAUNCH(MSAMP_DT_E4M3); else NORM_LAUNCH(MSAMP_DT_E5M2);
#undef NORM_LAUNCH
        MSAMP_CHECK_LAUNCH("fp8_norm_kernel");
    }
    hipLaunchKernelGGL(fp8_norm_finish_kernel, dim3((n_items + 63) / 64), dim3(64), 0, st, items, n_items, norm_kind);
    MSAMP_CHECK_LAUNCH("fp8_norm_finish_kernel");
    return MSAMP_OK;
}

}    // extern "C"
