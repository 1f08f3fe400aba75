// Shared device/host helpers for the gfx950 FP8 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <math.h>

#include "../../include/msamp_hip.h"

namespace msamp {

constexpr int kWave = 64;

// ---- error reporting -------------------------------------------------------------------------
void set_error(const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);
// true if a kernel whose workgroups wait for each other may be launched on this stream now
bool waiting_kernels_allowed(hipStream_t st);
// `count` consecutive non-zero tokens, unique in this process
uint32_t next_tokens(uint32_t count);
// device address of the library's own workspace (the one msamp_cast_to_fp8_intime_static uses) on the current device
int static_workspace(void** ws);
// how many times the collecting workgroup of a waiting kernel polls before it gives up (msamp_set_spin_limit)
uint32_t collector_spin_limit();

#define MSAMP_REQUIRE(cond, code, ...)  \
    do {                                \
        if (!(cond)) {                  \
            msamp::set_error(__VA_ARGS__); \
            return (code);              \
        }                               \
    } while (0)

#define MSAMP_CHECK_LAUNCH(what)                         \
    do {                                                 \
        hipError_t e__ = hipGetLastError();              \
        if (e__ != hipSuccess) return msamp::hip_fail(e__, what); \
    } while (0)

inline bool is_fp8(int dt) { return dt == MSAMP_DT_E4M3 || dt == MSAMP_DT_E5M2; }
inline bool is_hp(int dt) { return dt == MSAMP_DT_F32 || dt == MSAMP_DT_F16 || dt == MSAMP_DT_BF16; }
inline float fp8_max(int dt) { return dt == MSAMP_DT_E4M3 ? 448.0f : 57344.0f; }
inline int hp_size(int dt) { return dt == MSAMP_DT_F32 ? 4 : 2; }
inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// ---- element types ---------------------------------------------------------------------------
struct bf16_t {
    uint16_t bits;
};
struct f16_t {
    uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ float f16_bits_to_float(uint32_t b) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(b)));
}
// round-to-nearest-even float -> bf16 bits, NaN kept quiet (same rule torch uses)
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}
__device__ __forceinline__ uint32_t float_to_f16_bits(float f) {
    return static_cast<uint32_t>(__half_as_ushort(__float2half_rn(f)));
}

template <typename T>
struct Elem;    // load/store of one element as float
template <>
struct Elem<float> {
    static __device__ __forceinline__ float load(const float* p) { return *p; }
    static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <>
struct Elem<bf16_t> {
    static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_bits_to_float(p->bits); }
    static __device__ __forceinline__ void store(bf16_t* p, float v) {
        p->bits = static_cast<uint16_t>(float_to_bf16_bits(v));
    }
};
template <>
struct Elem<f16_t> {
    static __device__ __forceinline__ float load(const f16_t* p) { return f16_bits_to_float(p->bits); }
    static __device__ __forceinline__ void store(f16_t* p, float v) {
        p->bits = static_cast<uint16_t>(float_to_f16_bits(v));
    }
};

template <typename IT>
struct In16;    // one 16-byte load = EPT elements as float
// A 16-byte load, optionally marked as streaming (the `nt` bit): for inputs that are larger than the caches and read
// once.  Plain streaming reads of 2 GiB reach 6.4 TB/s on this part with ordinary loads and 7.1 TB/s with the mark; on
// data that a cache still holds the mark costs (the transposes, 64 MiB casts: 6 to 25 % slower), so the callers set it
// by size.
constexpr size_t kStreamBytes = 96ull << 20;
__device__ __forceinline__ uint4 ld16(const void* p, bool stream = false) {
    if (stream) {
        typedef uint32_t v4u_t __attribute__((ext_vector_type(4)));
        const v4u_t t = __builtin_nontemporal_load(static_cast<const v4u_t*>(p));
        return make_uint4(t.x, t.y, t.z, t.w);
    }
    return *static_cast<const uint4*>(p);
}
template <>
struct In16<float> {
    static constexpr int EPT = 4;
    static __device__ __forceinline__ void decode(const uint4& t, float* v) {
        v[0] = __uint_as_float(t.x), v[1] = __uint_as_float(t.y), v[2] = __uint_as_float(t.z), v[3] = __uint_as_float(t.w);
    }
    static __device__ __forceinline__ void load(const float* p, float* v, bool stream = false) { decode(ld16(p, stream), v); }
};
template <>
struct In16<bf16_t> {
    static constexpr int EPT = 8;
    static __device__ __forceinline__ void load(const bf16_t* p, float* v, bool stream = false) { decode(ld16(p, stream), v); }
    static __device__ __forceinline__ void decode(const uint4& t, float* v) {
        v[0] = __uint_as_float(t.x << 16), v[1] = __uint_as_float(t.x & 0xffff0000u);
        v[2] = __uint_as_float(t.y << 16), v[3] = __uint_as_float(t.y & 0xffff0000u);
        v[4] = __uint_as_float(t.z << 16), v[5] = __uint_as_float(t.z & 0xffff0000u);
        v[6] = __uint_as_float(t.w << 16), v[7] = __uint_as_float(t.w & 0xffff0000u);
    }
};
template <>
struct In16<f16_t> {
    static constexpr int EPT = 8;
    static __device__ __forceinline__ void load(const f16_t* p, float* v, bool stream = false) { decode(ld16(p, stream), v); }
    static __device__ __forceinline__ void decode(const uint4& t, float* v) {
        v[0] = f16_bits_to_float(t.x & 0xffffu), v[1] = f16_bits_to_float(t.x >> 16);
        v[2] = f16_bits_to_float(t.y & 0xffffu), v[3] = f16_bits_to_float(t.y >> 16);
        v[4] = f16_bits_to_float(t.z & 0xffffu), v[5] = f16_bits_to_float(t.z >> 16);
        v[6] = f16_bits_to_float(t.w & 0xffffu), v[7] = f16_bits_to_float(t.w >> 16);
    }
};

// ---- FP8 conversion --------------------------------------------------------------------------
// FMT: MSAMP_DT_E4M3 or MSAMP_DT_E5M2.  Saturating round-to-nearest-even through the gfx950
// OCP converters; the clamp makes saturation independent of the wave's overflow mode and
// NaN is patched to sign|0x7F afterwards (the clamp would otherwise turn it into -max).
template <int FMT>
__device__ __forceinline__ float sat(float v) {
    constexpr float mx = (FMT == MSAMP_DT_E4M3) ? 448.0f : 57344.0f;
    return __builtin_amdgcn_fmed3f(v, -mx, mx);
}

template <int FMT>
__device__ __forceinline__ uint32_t cvt_pk(float a, float b, uint32_t old, bool hi) {
    if constexpr (FMT == MSAMP_DT_E4M3) {
        return hi ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, false);
    } else {
        return hi ? __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, false);
    }
}

__device__ __forceinline__ uint32_t nan_byte(float v) { return 0x7fu | ((__float_as_uint(v) >> 24) & 0x80u); }

// four floats (already multiplied by the scale) -> four packed FP8 bytes, byte i = element i
template <int FMT>
__device__ __forceinline__ uint32_t quant4(float a, float b, float c, float d) {
    uint32_t w = 0;
    w = cvt_pk<FMT>(sat<FMT>(a), sat<FMT>(b), w, false);
    w = cvt_pk<FMT>(sat<FMT>(c), sat<FMT>(d), w, true);
    if (__builtin_expect((a != a) | (b != b) | (c != c) | (d != d), 0)) {
        if (a != a) w = (w & 0xffffff00u) | nan_byte(a);
        if (b != b) w = (w & 0xffff00ffu) | (nan_byte(b) << 8);
        if (c != c) w = (w & 0xff00ffffu) | (nan_byte(c) << 16);
        if (d != d) w = (w & 0x00ffffffu) | (nan_byte(d) << 24);
    }
    return w;
}

// the same for values known to be finite and within the format's range: no clamp, no NaN patch
template <int FMT>
__device__ __forceinline__ uint32_t quant4_in_range(float a, float b, float c, float d) {
    uint32_t w = 0;
    w = cvt_pk<FMT>(a, b, w, false);
    w = cvt_pk<FMT>(c, d, w, true);
    return w;
}

template <int FMT>
__device__ __forceinline__ uint32_t quant1(float a) {
    uint32_t w = cvt_pk<FMT>(sat<FMT>(a), 0.0f, 0u, false) & 0xffu;
    if (a != a) w = nan_byte(a);
    return w;
}

// packed FP8 word -> floats (exact)
template <int FMT>
__device__ __forceinline__ void dequant4(uint32_t w, float& a, float& b, float& c, float& d) {
    typedef float v2f __attribute__((ext_vector_type(2)));
    v2f lo, hi;
    if constexpr (FMT == MSAMP_DT_E4M3) {
        lo = __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
        hi = __builtin_amdgcn_cvt_pk_f32_fp8(w, true);
    } else {
        lo = __builtin_amdgcn_cvt_pk_f32_bf8(w, false);
        hi = __builtin_amdgcn_cvt_pk_f32_bf8(w, true);
    }
    a = lo.x;
    b = lo.y;
    c = hi.x;
    d = hi.y;
}

template <int FMT>
__device__ __forceinline__ float dequant1(uint32_t byte) {
    float a, b, c, d;
    dequant4<FMT>(byte & 0xffu, a, b, c, d);
    return a;
}

// ---- meeting place of the kernels whose workgroups wait for each other --------------------------------
// `kMaxSlots` eight-byte {token, max} slots start at byte kWsSlotBytes of the workspace; two post words follow.
// Word kWsErrorWord of the workspace is sticky: a kernel whose bounded wait runs out stores a non-zero code there
// (a vector store), and msamp_check_async_error reports and clears it.  The collecting workgroup (0) gives up
// after `spin_limit` polls and then still posts (a NaN amax and the old scale), so that every workgroup that sees
// the post quantizes with the same scale; the others wait kFollowerSpinFactor times as long for that post, and a
// workgroup that never sees it writes NaN codes.  Either way the error word is set.
constexpr int kWsErrorWord = 8;
constexpr uint32_t kFollowerSpinFactor = 4;
constexpr uint32_t kErrCollectorGaveUp = 1, kErrFollowerGaveUp = 2;
__device__ __forceinline__ void report_wait_expired(uint32_t* error_word, uint32_t code) {
    __hip_atomic_fetch_or(error_word, code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
constexpr int kWsSlotBytes = 8192;
constexpr int kMaxSlots = 512;
static_assert(kWsSlotBytes + (kMaxSlots + 2) * 8 <= MSAMP_WORKSPACE_BYTES, "slots exceed the workspace");

__device__ __forceinline__ uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }

// ---- reductions ------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        uint32_t o = static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), off, 64));
        v = v > o ? v : o;
    }
    return v;
}

// max over the block of a non-negative-float bit pattern (or any u32); result valid in thread 0.
// `smem` must hold blockDim.x/64 words.
__device__ __forceinline__ uint32_t block_max_u32(uint32_t v, uint32_t* smem) {
    v = wave_max_u32(v);
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) smem[wid] = v;
    __syncthreads();
    if (wid == 0) {
        v = lane < nw ? smem[lane] : 0u;
        v = wave_max_u32(v);
    }
    return v;
}

// The pow-2 scale rule, evaluated the way float32 torch evaluates it: `fp_max / amax` with a Python
// float on the left is reciprocal(amax) * fp_max (two roundings, in eager mode and under TorchScript
// alike), log2 is the correctly rounded float log2 (double log2 narrowed once), 2^|e| overflows to
// +Inf from |e| = 128.
__device__ __forceinline__ float scale_rule(float amax, float fallback, float fp_max, int margin) {
    const float recip = 1.0f / amax;
    const float q = recip * fp_max;
    // e = floor(float(log2(q))).  For a positive normal q whose mantissa is not within 2^-17 of the
    // next power of two, the float rounding of log2(q) cannot reach the next integer (half an ulp of
    // any float of magnitude <= 128 is below 2^-17 / ln 2), so e is the exponent field.  Otherwise
    // take the long road: double log2, narrowed by hand -- keeping the double result live in double
    // arithmetic stops the compiler from shrinking the call to the (not correctly rounded) float
    // log2; if narrowing d to float reaches the next integer, the floor is that integer.
    const uint32_t qb = __float_as_uint(q);
    const uint32_t qe = (qb >> 23) & 0xffu;
    float e;
    if ((qb >> 31) == 0u && qe != 0u && qe != 255u && (qb & 0x7fffffu) < 0x7fff80u) {
        e = static_cast<float>(static_cast<int>(qe) - 127 - margin);
    } else {
        const double d = log2(static_cast<double>(q));
        double fl = floor(d);
        if (static_cast<float>(d) >= static_cast<float>(fl + 1.0)) fl += 1.0;
        e = static_cast<float>(fl) - static_cast<float>(margin);
    }
    float ae = fabsf(e);
    float sf;
    if (ae != ae) {
        sf = ae;    // NaN
    } else if (ae >= 128.0f) {
        sf = __uint_as_float(0x7f800000u);
    } else {
        sf = __uint_as_float(static_cast<uint32_t>(static_cast<int>(ae) + 127) << 23);
    }
    if (!(amax > 0.0f)) sf = fallback;
    if (!(fabsf(amax) < __uint_as_float(0x7f800000u))) sf = fallback;    // not finite (NaN or Inf)
    if (e < 0.0f) sf = 1.0f / sf;
    return sf;
}

inline int cu_count() {
    static int n = 0;
    if (n == 0) {
        int dev = 0;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess)
            n = p.multiProcessorCount;
        if (n <= 0) n = 256;
    }
    return n;
}

}    // namespace msamp
