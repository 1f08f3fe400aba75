// Cast group: amax, pow-2 scale rule, FP8 quantize / dequantize, cast+transpose, byte transpose,
// amax-window update.  All bandwidth-bound: 16-byte lane-contiguous loads, packed FP8 converters,
// wavefront shuffle reductions, one atomic per block.
#include "common.cuh"
#include "gemm_call.h"

#include <atomic>
#include <mutex>

namespace msamp {

constexpr int kCastThreads = 256;
constexpr int kCastUnroll = 4;

// issue an atomic max on a non-negative float cell only when it can change the cell
__device__ __forceinline__ void amax_publish(float* amax, float v) {
    int vb = __float_as_int(v);
    int cur = __hip_atomic_load(reinterpret_cast<int*>(amax), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (vb > cur) atomicMax(reinterpret_cast<int*>(amax), vb);
}

// ---------------------------------------------------------------------------------------------
// Quantize with a given scale.  WITH_AMAX: also fold max|x| (NaN skipped) into *amax.
// reverse != 0 walks the tiles back to front (second pass of the in-time cast).
// Workspace of the two-pass (in-time) casts, in 32-bit words: [0] scale in force before the call,
// [1] number of partial maxima, [kWsPartials...] per-workgroup partial maxima of the first pass
// (float bit patterns of |x|, NaN patterns included).
constexpr int kWsPartials = 16;
constexpr int kMaxPartials = 1024;
// word kWsSpecDone: non-zero when the first pass of an in-time cast also wrote the output, quantized with the scale
// in force before the call (word 0); the second pass then only has to run when the rule gives another scale
constexpr int kWsSpecDone = 9;

struct InTimeArgs {
    const uint32_t* ws;    // nullptr: the scale comes from *scale_p
    float* scale_out;
    float* amax_out;
    float fp_max;
    int margin;
    int flags;
    const float* known_amax;       // kRescale: amax window of the real values, already known
    const float* old_scale_inv;    // kRescale: reciprocal scale of the stored payload
    float* amax_copy;              // kRescale, nullable: receives a copy of the amax window
    int window;
    int32_t* counter_out;          // kRescale, nullable: set to 0 (the new meta's update count)
    int speculative;               // kInTime: the first pass may already have written the output (see kWsSpecDone)
};

// Warm-up gate: the amax kernels of a gated cast run only while *counter < window (in-time scaling);
// once the window is full they return at once and the cast that follows uses the stored scale.
struct Gate {
    const int32_t* counter;    // nullptr: always run
    int window;
};
__device__ __forceinline__ bool gate_closed(const Gate& g) { return g.counter != nullptr && *g.counter >= g.window; }

// where cast_to_fp8_kernel takes its scale from
// (kGivenIfFlagged: as kGivenScale, but the launch does nothing unless the word it.ws points at is non-zero)
enum ScaleSource { kGivenScale = 0, kInTime = 1, kRescale = 2, kGivenIfFlagged = 3 };

// every workgroup of the second pass derives the same amax and scale from the partial maxima
__device__ __forceinline__ float resolve_in_time_scale(const InTimeArgs& a, uint32_t* red, float* scale_inv) {
    __shared__ float s_scale;
    const int np = static_cast<int>(a.ws[1]);
    uint32_t m = 0;
    for (int i = threadIdx.x; i < np; i += blockDim.x) {
        const uint32_t v = a.ws[kWsPartials + i];
        m = v > m ? v : m;
    }
    m = block_max_u32(m, red);
    if (threadIdx.x == 0) {
        float am = __uint_as_float(m);
        if ((a.flags & MSAMP_FLAG_NAN_TO_INF) && !(am < __uint_as_float(0x7f800000u))) am = __uint_as_float(0x7f800000u);
        const float s = scale_rule(am, __uint_as_float(a.ws[0]), a.fp_max, a.margin);
        s_scale = s;
        if (blockIdx.x == 0 && blockIdx.y == 0) {
            *a.amax_out = am;
            *a.scale_out = s;
            *scale_inv = 1.0f / s;
        }
    }
    __syncthreads();
    return s_scale;
}

// kRescale: the payload holds value * old_scale and max|value| is known, so the new scale is the rule of
// that amax (fallback 1), the payload is multiplied by new_scale * old_scale_inv, and the meta gets
// scale = that factor, scale_inv = 1 / new_scale.
// Every workgroup ends with one atomic on the amax cell, and atomics on one address are served one
// at a time (about 10 ns each): the launch with WITH_AMAX uses few, large workgroups (THREADS = 512,
// two per CU) so that they stay a small part of the run time.
template <typename IT, int FMT, bool WITH_AMAX, int INTIME, int THREADS = kCastThreads>
__global__ __launch_bounds__(THREADS) void cast_to_fp8_kernel(const IT* __restrict__ x,
                                                                    uint8_t* __restrict__ out, size_t n,
                                                                    const float* __restrict__ scale_p, float* amax,
                                                                    float* scale_inv, int vec_ok, int reverse,
                                                                    InTimeArgs it) {
    constexpr int EPT = In16<IT>::EPT;
    constexpr size_t TILE = static_cast<size_t>(THREADS) * EPT * kCastUnroll;
    __shared__ uint32_t red[THREADS / kWave];
    float s;
    if constexpr (INTIME == kInTime) {
        s = resolve_in_time_scale(it, red, scale_inv);
        // the first pass quantized with the scale it found in the meta, and the rule confirms that scale: done
        if (it.speculative && it.ws[kWsSpecDone] != 0u && __float_as_uint(s) == it.ws[0]) return;
    } else if constexpr (INTIME == kRescale) {
        const float s_new = scale_rule(*it.known_amax, 1.0f, it.fp_max, it.margin);
        s = s_new * *it.old_scale_inv;
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            *it.scale_out = s;
            *scale_inv = 1.0f / s_new;
            if (it.counter_out != nullptr) *it.counter_out = 0;
        }
        if (blockIdx.x == 0 && it.amax_copy != nullptr) {
            for (int j = threadIdx.x; j < it.window; j += blockDim.x) it.amax_copy[j] = it.known_amax[j];
        }
    } else if constexpr (INTIME == kGivenIfFlagged) {
        if (*it.ws == 0u) return;    // the codes written on speculation stand
        s = *scale_p;
    } else {
        s = *scale_p;
    }
    const int tid = threadIdx.x;
    float mx = 0.0f;
    const size_t ntiles = (n + TILE - 1) / TILE;
    for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const size_t tile = reverse ? (ntiles - 1 - t) : t;
        const size_t base = tile * TILE;
        if ((vec_ok & 1) && base + TILE <= n) {
            float v[kCastUnroll][EPT];
#pragma unroll
            for (int u = 0; u < kCastUnroll; ++u)
                In16<IT>::load(x + base + (static_cast<size_t>(u) * THREADS + tid) * EPT, v[u], (vec_ok & 2) != 0);
#pragma unroll
            for (int u = 0; u < kCastUnroll; ++u) {
                uint32_t w[EPT / 4];
#pragma unroll
                for (int j = 0; j < EPT / 4; ++j) {
                    const float a = v[u][4 * j], b = v[u][4 * j + 1], c = v[u][4 * j + 2], d = v[u][4 * j + 3];
                    if (WITH_AMAX) mx = fmaxf(fmaxf(mx, fabsf(a)), fmaxf(fmaxf(fabsf(b), fabsf(c)), fabsf(d)));
                    w[j] = quant4<FMT>(a * s, b * s, c * s, d * s);
                }
                uint8_t* o = out + base + (static_cast<size_t>(u) * THREADS + tid) * EPT;
                if constexpr (EPT == 4) {
                    *reinterpret_cast<uint32_t*>(o) = w[0];
                } else {
                    *reinterpret_cast<uint2*>(o) = make_uint2(w[0], w[1]);
                }
            }
        } else {
            const size_t end = (base + TILE < n) ? base + TILE : n;
            for (size_t i = base + tid; i < end; i += THREADS) {
                const float a = Elem<IT>::load(x + i);
                if (WITH_AMAX) mx = fmaxf(mx, fabsf(a));
                out[i] = static_cast<uint8_t>(quant1<FMT>(a * s));
            }
        }
    }
    if (WITH_AMAX) {
        uint32_t m = block_max_u32(__float_as_uint(mx), red);
        if (tid == 0) amax_publish(amax, __uint_as_float(m));
    }
    if constexpr (INTIME == kGivenScale) {
        if (scale_inv != nullptr && blockIdx.x == 0 && tid == 0) *scale_inv = 1.0f / s;
    }
}

// ---------------------------------------------------------------------------------------------
// First pass of the in-time casts: NaN-propagating max|x| per workgroup, written to the workspace
// (no atomics, no fences: the kernel boundary orders it before the second pass).

// With fin.amax set, the workgroup that finishes last (a ticket counter in the workspace tells) also
// reduces the partial maxima and applies the scale rule, which saves the finalize launch.
struct Finish {
    float* amax;    // nullptr: leave the reduction to a later kernel
    float* scale;
    float* scale_inv;
    float fp_max;
    int margin;
    int flags;
};
constexpr int kWsTicket = 2;

template <typename IT>
__global__ __launch_bounds__(kCastThreads) void amax_partial_kernel(const IT* __restrict__ x, size_t n, uint32_t* ws,
                                                                     const float* scale, int vec_ok, Gate gate,
                                                                     Finish fin) {
    if (gate_closed(gate)) return;
    constexpr int EPT = 16 / sizeof(IT);
    constexpr int UNROLL = 8;
    constexpr size_t TILE = static_cast<size_t>(kCastThreads) * EPT * UNROLL;
    __shared__ uint32_t red[kCastThreads / kWave];
    const int tid = threadIdx.x;
    // running max of the |x| bit pattern; for 2-byte inputs kept in the high half-word
    uint32_t m = 0;
    const size_t ntiles = (n + TILE - 1) / TILE;
    for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const size_t base = t * TILE;
        if (vec_ok && base + TILE <= n) {
            uint4 v[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u)
                v[u] = *reinterpret_cast<const uint4*>(x + base + (static_cast<size_t>(u) * kCastThreads + tid) * EPT);
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if constexpr (sizeof(IT) == 4) {
                        m = umax(m, w[j] & 0x7fffffffu);
                    } else {
                        m = umax(m, umax((w[j] << 16) & 0x7fff0000u, w[j] & 0x7fff0000u));
                    }
                }
            }
        } else {
            const size_t end = (base + TILE < n) ? base + TILE : n;
            for (size_t i = base + tid; i < end; i += kCastThreads) {
                if constexpr (sizeof(IT) == 4) {
                    m = umax(m, reinterpret_cast<const uint32_t*>(x)[i] & 0x7fffffffu);
                } else {
                    m = umax(m, (static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(x)[i]) << 16) & 0x7fff0000u);
                }
            }
        }
    }
    m = block_max_u32(m, red);
    if (tid == 0) {
        // to a float32 bit pattern (order-preserving for bf16 already; fp16 needs widening)
        if constexpr (sizeof(IT) == 2 && !__is_same(IT, bf16_t)) {
            m = __float_as_uint(f16_bits_to_float(m >> 16));
        }
        ws[kWsPartials + blockIdx.x] = m;
        if (blockIdx.x == 0) {
            ws[0] = scale != nullptr ? __float_as_uint(*scale) : __float_as_uint(1.0f);
            ws[1] = gridDim.x;
        }
    }
    if (fin.amax == nullptr) return;
    __shared__ uint32_t s_last;
    if (tid == 0) {
        __threadfence();    // the partial maximum above is visible before the ticket is taken
        const uint32_t ticket = atomicAdd(ws + kWsTicket, 1u);
        s_last = ticket == gridDim.x - 1;
        if (s_last) ws[kWsTicket] = 0;    // ready for the next call
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();    // see every other workgroup's partial maximum
    uint32_t mm = 0;
    for (int i = tid; i < static_cast<int>(gridDim.x); i += kCastThreads) {
        const uint32_t v = __hip_atomic_load(ws + kWsPartials + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        mm = v > mm ? v : mm;
    }
    mm = block_max_u32(mm, red);
    if (tid == 0) {
        float a = __uint_as_float(mm);
        if ((fin.flags & MSAMP_FLAG_NAN_TO_INF) && !(a < __uint_as_float(0x7f800000u))) a = __uint_as_float(0x7f800000u);
        const float sc = scale_rule(a, *fin.scale, fin.fp_max, fin.margin);
        *fin.amax = a;
        *fin.scale = sc;
        *fin.scale_inv = 1.0f / sc;
    }
}

// First pass of the in-time cast of a tensor too large for the one-pass kernel, with the output written on
// speculation: max|x| per workgroup as above, and every element quantized with the scale the meta holds before the
// call.  A power-of-two scale rarely changes between two calls on the same meta; when the second pass finds that
// the rule confirms it, it returns at once and x has been read once (sizeof(in) + 1 bytes per element instead of
// 2 * sizeof(in) + 1).  Otherwise the second pass quantizes again with the new scale: the same bytes as without
// speculation, since the output is not an input.  A meta that has never been used (amax 0, scale 1) is not
// speculated on: the pass then only takes the maxima.
constexpr int kSpecThreads = 512;

template <typename IT, int FMT>
__global__ __launch_bounds__(kSpecThreads) void cast_speculative_kernel(const IT* __restrict__ x, uint8_t* __restrict__ out,
                                                                         size_t n, const float* scale, const float* amax,
                                                                         uint32_t* ws, int vec_ok) {
    constexpr int EPT = In16<IT>::EPT;
    constexpr size_t TILE = static_cast<size_t>(kSpecThreads) * EPT * kCastUnroll;
    __shared__ uint32_t red[kSpecThreads / kWave];
    const int tid = threadIdx.x;
    const float guess = *scale;
    const bool spec = !(*amax == 0.0f && guess == 1.0f);
    uint32_t m = 0;
    const size_t ntiles = (n + TILE - 1) / TILE;
    for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const size_t base = t * TILE;
        if ((vec_ok & 1) && base + TILE <= n) {
            uint4 raw[kCastUnroll];
#pragma unroll
            for (int u = 0; u < kCastUnroll; ++u)
                raw[u] = ld16(x + base + (static_cast<size_t>(u) * kSpecThreads + tid) * EPT, (vec_ok & 2) != 0);
#pragma unroll
            for (int u = 0; u < kCastUnroll; ++u) {
                const uint32_t w[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if constexpr (sizeof(IT) == 4) m = umax(m, w[j] & 0x7fffffffu);
                    else m = umax(m, umax((w[j] << 16) & 0x7fff0000u, w[j] & 0x7fff0000u));
                }
                if (spec) {
                    float f[EPT];
                    In16<IT>::decode(raw[u], f);
                    uint32_t q[EPT / 4];
#pragma unroll
                    for (int j = 0; j < EPT / 4; ++j)
                        q[j] = quant4<FMT>(f[4 * j] * guess, f[4 * j + 1] * guess, f[4 * j + 2] * guess, f[4 * j + 3] * guess);
                    uint8_t* o = out + base + (static_cast<size_t>(u) * kSpecThreads + tid) * EPT;
                    if constexpr (EPT == 4) *reinterpret_cast<uint32_t*>(o) = q[0];
                    else *reinterpret_cast<uint2*>(o) = make_uint2(q[0], q[1]);
                }
            }
        } else {
            const size_t end = (base + TILE < n) ? base + TILE : n;
            for (size_t i = base + tid; i < end; i += kSpecThreads) {
                if constexpr (sizeof(IT) == 4) {
                    m = umax(m, reinterpret_cast<const uint32_t*>(x)[i] & 0x7fffffffu);
                } else {
                    m = umax(m, (static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(x)[i]) << 16) & 0x7fff0000u);
                }
                if (spec) out[i] = static_cast<uint8_t>(quant1<FMT>(Elem<IT>::load(x + i) * guess));
            }
        }
    }
    m = block_max_u32(m, red);
    if (tid == 0) {
        if constexpr (sizeof(IT) == 2 && !__is_same(IT, bf16_t)) m = __float_as_uint(f16_bits_to_float(m >> 16));
        ws[kWsPartials + blockIdx.x] = m;
        if (blockIdx.x == 0) {
            ws[0] = __float_as_uint(guess);
            ws[1] = gridDim.x;
            ws[kWsSpecDone] = spec ? 1u : 0u;
        }
    }
}

// reduce the partial maxima into amax[0] (and, if asked, run the scale rule) in one workgroup
__global__ __launch_bounds__(kCastThreads) void amax_finalize_kernel(const uint32_t* ws, float* amax, float* scale,
                                                                      float* scale_inv, float fp_max, int margin, int flags,
                                                                      int update_scale, Gate gate) {
    if (gate_closed(gate)) return;
    __shared__ uint32_t red[kCastThreads / kWave];
    const int np = static_cast<int>(ws[1]);
    uint32_t m = 0;
    for (int i = threadIdx.x; i < np; i += blockDim.x) {
        const uint32_t v = ws[kWsPartials + i];
        m = v > m ? v : m;
    }
    m = block_max_u32(m, red);
    if (threadIdx.x == 0) {
        float a = __uint_as_float(m);
        if ((flags & MSAMP_FLAG_NAN_TO_INF) && !(a < __uint_as_float(0x7f800000u))) a = __uint_as_float(0x7f800000u);
        *amax = a;
        if (update_scale) {
            const float s = scale_rule(a, __uint_as_float(ws[0]), fp_max, margin);
            *scale = s;
            *scale_inv = 1.0f / s;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// One-pass in-time cast for tensors that fit the register file of the chip: each 512-lane workgroup
// (two per CU) keeps a contiguous run of x in registers (up to kResVecs 16-byte vectors per lane),
// publishes max|x| of its run, waits until every workgroup has published, and quantizes from
// registers, so x is read once.
// The grid-wide meeting uses no atomics and no fences: workgroup b stores {token, max} as one
// 8-byte word into slot b of the workspace (slots start at byte kWsSlotBytes), then the first wave
// of every workgroup polls all slots until each carries this call's token, reducing the maxima on
// the way; every workgroup then derives the same scale by itself.  Tokens come from a host counter,
// so slots never need clearing.  All workgroups must be resident together: the host launches at most
// two per CU and keeps the kernel to one stream per device; the wait is bounded all the same, and a
// wait that runs out sets the workspace's sticky error word (and, when it is workgroup 0's, NaN as the amax).
constexpr int kResThreads = 512;
constexpr int kResVecs = 16;
constexpr int kResBlocksPerCu = 2;

template <typename IT>
__device__ __forceinline__ uint32_t abs_bits_hi(uint32_t raw) {    // raw element bits -> ordered key
    if constexpr (sizeof(IT) == 4) return raw & 0x7fffffffu;
    else return (raw << 16) & 0x7fff0000u;
}

// R = vectors per lane the kernel is built for (the host picks the smallest of 4 / 8 / 16 that covers the
// tensor, so that a small tensor does not pay for loads it has no use for).
// SPEC: quantize with the scale in force *before* the meeting and store, then meet: a power-of-two scale rarely
// changes between two calls on the same meta, and when the rule confirms it the output is already in place --
// the workgroups never sit idle between an all-loads and an all-stores phase, and early finishers' stores overlap
// the late ones' loads.  When the scale did change, the run is quantized again from the registers, as without
// SPEC.  Same bytes either way (the output is not an input).  A meta that has never been used (amax 0, scale 1)
// is not speculated on.
template <typename IT, int FMT, int R, bool SPEC>
__global__ __launch_bounds__(kResThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void cast_intime_resident_kernel(const IT* __restrict__ x,
                                                                           uint8_t* __restrict__ out, size_t n,
                                                                           float* scale, float* amax, float* scale_inv,
                                                                           uint64_t* slots, float fp_max, int margin,
                                                                           int flags, int rounds, uint32_t token,
                                                                           uint32_t spin_limit, uint32_t* error_word) {
    constexpr int EPT = 16 / sizeof(IT);
    using Raw = typename std::conditional<sizeof(IT) == 4, uint32_t, uint16_t>::type;
    __shared__ uint32_t red[kResThreads / kWave];
    __shared__ uint32_t s_scale, s_amax;
    const int tid = threadIdx.x;
    // the host keeps the vector count within 32 bits (at most one register file of vectors)
    const uint32_t nvec = static_cast<uint32_t>(n / EPT);
    // each workgroup owns one contiguous run of rounds * kResThreads vectors
    const uint32_t v0 = blockIdx.x * static_cast<uint32_t>(rounds) * kResThreads + tid;
    // read before any workgroup can pass the meeting and replace them
    const float old_scale = *scale;
    const float old_amax = *amax;

    uint4 v[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        // unconditional (clamped) loads, so that all of them are in flight together; a vector read
        // twice changes no maximum, and the store phase skips the duplicates
        const uint32_t idx = v0 + r * kResThreads;
        v[r] = ld16(reinterpret_cast<const uint4*>(x) + (idx < nvec ? idx : nvec - 1), true);    // read once: as a stream
    }
    // the ragged end (fewer than EPT elements) rides with the first lanes of workgroup 0
    const size_t tail0 = static_cast<size_t>(nvec) * EPT;
    const bool has_tail = blockIdx.x == 0 && tail0 + tid < n;
    Raw tail_raw = 0;
    if (has_tail) tail_raw = reinterpret_cast<const Raw*>(x)[tail0 + tid];

    uint32_t m = abs_bits_hi<IT>(tail_raw);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t w[4] = {v[r].x, v[r].y, v[r].z, v[r].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (sizeof(IT) == 4) m = umax(m, w[j] & 0x7fffffffu);
            else m = umax(m, umax((w[j] << 16) & 0x7fff0000u, w[j] & 0x7fff0000u));
        }
    }
    m = block_max_u32(m, red);    // valid in lane 0 of wave 0
    if (tid == 0) {
        if constexpr (sizeof(IT) == 2 && !__is_same(IT, bf16_t)) m = __float_as_uint(f16_bits_to_float(m >> 16));
        __hip_atomic_store(slots + blockIdx.x, (static_cast<uint64_t>(token) << 32) | m, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }

    // quantize this lane's vectors (and the ragged end) with scale q and store them
    auto emit = [&](float q, auto in_range_c, auto fenced_c) {
        constexpr bool kInRange = decltype(in_range_c)::value, kFenced = decltype(fenced_c)::value;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            // after the meeting: keep only the raw words live across it, not values derived from them before it
            if constexpr (kFenced) asm volatile("" : "+v"(v[r].x), "+v"(v[r].y), "+v"(v[r].z), "+v"(v[r].w));
            const uint32_t idx = v0 + r * kResThreads;
            if (r < rounds && idx < nvec) {
                float f[EPT];
                In16<IT>::decode(v[r], f);
                uint32_t w[EPT / 4];
#pragma unroll
                for (int j = 0; j < EPT / 4; ++j) {
                    if constexpr (kInRange) w[j] = quant4_in_range<FMT>(f[4 * j] * q, f[4 * j + 1] * q, f[4 * j + 2] * q, f[4 * j + 3] * q);
                    else w[j] = quant4<FMT>(f[4 * j] * q, f[4 * j + 1] * q, f[4 * j + 2] * q, f[4 * j + 3] * q);
                }
                if constexpr (EPT == 4) reinterpret_cast<uint32_t*>(out)[idx] = w[0];
                else reinterpret_cast<uint2*>(out)[idx] = make_uint2(w[0], w[1]);
            }
        }
        if (has_tail) {
            float a;
            if constexpr (sizeof(IT) == 4) a = __uint_as_float(tail_raw);
            else if constexpr (__is_same(IT, bf16_t)) a = __uint_as_float(static_cast<uint32_t>(tail_raw) << 16);
            else a = f16_bits_to_float(tail_raw);
            out[tail0 + tid] = static_cast<uint8_t>(quant1<FMT>(a * q));
        }
    };
    bool speculated = false;
    if constexpr (SPEC) {
        speculated = !(old_amax == 0.0f && old_scale == 1.0f);
        if (speculated) emit(old_scale, std::false_type{}, std::false_type{});
    }

    if (tid < kWave) {
        // Workgroup 0 collects: it alone polls the slots (everyone polling them costs the workgroups still
        // loading a good part of their bandwidth), derives amax and scale and posts both, tagged with the
        // token, in two words behind the slots; the others poll only those.
        uint64_t* post = slots + kMaxSlots;
        if (blockIdx.x == 0) {
            uint32_t mm = 0;
            bool all_in = false;
            for (uint32_t spins = 0; !all_in && spins < spin_limit; ++spins) {
                // all slots of one poll are requested together; the ones past the grid are read and ignored
                uint64_t sv[kMaxSlots / kWave];
#pragma unroll
                for (int j = 0; j < kMaxSlots / kWave; ++j)
                    sv[j] = __hip_atomic_load(slots + tid + j * kWave, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                bool ok = true;
                mm = 0;
#pragma unroll
                for (int j = 0; j < kMaxSlots / kWave; ++j) {
                    const bool live = static_cast<uint32_t>(tid + j * kWave) < gridDim.x;
                    ok = ok && (!live || static_cast<uint32_t>(sv[j] >> 32) == token);
                    mm = umax(mm, live ? static_cast<uint32_t>(sv[j]) : 0u);
                }
                all_in = __all(ok);
            }
            mm = wave_max_u32(mm);
            if (tid == 0) {
                float am = __uint_as_float(mm);
                // The wait ran out: the amax becomes NaN, the rule then keeps the old scale, and both are still posted,
                // so every workgroup that sees the post quantizes with one and the same scale; the sticky error word
                // tells the host.
                if (!all_in) {
                    am = __uint_as_float(0x7fc00000u);
                    report_wait_expired(error_word, kErrCollectorGaveUp);
                } else if ((flags & MSAMP_FLAG_NAN_TO_INF) && !(am < __uint_as_float(0x7f800000u))) {
                    am = __uint_as_float(0x7f800000u);
                }
                const float s = scale_rule(am, old_scale, fp_max, margin);
                const uint64_t tag = static_cast<uint64_t>(token) << 32;
                __hip_atomic_store(post, tag | __float_as_uint(am), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(post + 1, tag | __float_as_uint(s), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                s_scale = __float_as_uint(s);
                s_amax = __float_as_uint(am);
                *amax = am;
                *scale = s;
                *scale_inv = 1.0f / s;
            }
        } else if (tid == 0) {
            // wait for workgroup 0's post, longer than it waits itself: it posts even when it gives up
            uint64_t pa = 0, ps = 0;
            bool posted = false;
            const uint64_t follower_limit = static_cast<uint64_t>(spin_limit) * kFollowerSpinFactor;
            for (uint64_t spins = 0; !posted && spins < follower_limit; ++spins) {
                pa = __hip_atomic_load(post, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ps = __hip_atomic_load(post + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                posted = static_cast<uint32_t>(pa >> 32) == token && static_cast<uint32_t>(ps >> 32) == token;
            }
            if (!posted) report_wait_expired(error_word, kErrFollowerGaveUp);    // no post at all: NaN codes from here
            s_amax = posted ? static_cast<uint32_t>(pa) : 0x7fc00000u;
            s_scale = posted ? static_cast<uint32_t>(ps) : 0x7fc00000u;
        }
    }
    __syncthreads();
    const float s = __uint_as_float(s_scale);
    if constexpr (SPEC) {
        // the scale the output was written with stands: done.  Otherwise let those stores land before writing again.
        if (speculated && __float_as_uint(s) == __float_as_uint(old_scale)) return;
        if (speculated) __builtin_amdgcn_s_waitcnt(0x0F70);    // vmcnt(0): loads and stores share the counter here
    }
    // With a positive finite amax and the scale the rule derived from it, every |x| * s stays within the
    // format and nothing is NaN: the clamp and the NaN patch can go.
    const bool in_range = __uint_as_float(s_amax) * s <= fp_max && __uint_as_float(s_amax) > 0.0f;
    if (in_range) emit(s, std::true_type{}, std::true_type{});
    else emit(s, std::false_type{}, std::true_type{});
}

// ---------------------------------------------------------------------------------------------
template <int FMT, typename OT>
__global__ __launch_bounds__(kCastThreads) void cast_from_fp8_kernel(const uint8_t* __restrict__ q,
                                                                      OT* __restrict__ out, size_t n,
                                                                      const float* __restrict__ scale_inv_p,
                                                                      int vec_ok) {
    constexpr int EPT = 16 / sizeof(OT);    // codes per thread per step: 4 (fp32 out) or 8
    constexpr int UNROLL = 4;
    constexpr size_t TILE = static_cast<size_t>(kCastThreads) * EPT * UNROLL;
    const float si = *scale_inv_p;
    const int tid = threadIdx.x;
    const size_t ntiles = (n + TILE - 1) / TILE;
    for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const size_t base = t * TILE;
        if (vec_ok && base + TILE <= n) {
            uint32_t w[UNROLL][EPT / 4];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const uint8_t* p = q + base + (static_cast<size_t>(u) * kCastThreads + tid) * EPT;
                if constexpr (EPT == 4) {
                    w[u][0] = *reinterpret_cast<const uint32_t*>(p);
                } else {
                    uint2 t2 = *reinterpret_cast<const uint2*>(p);
                    w[u][0] = t2.x, w[u][1] = t2.y;
                }
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                float f[EPT];
#pragma unroll
                for (int j = 0; j < EPT / 4; ++j) {
                    dequant4<FMT>(w[u][j], f[4 * j], f[4 * j + 1], f[4 * j + 2], f[4 * j + 3]);
                }
#pragma unroll
                for (int j = 0; j < EPT; ++j) f[j] *= si;
                OT* o = out + base + (static_cast<size_t>(u) * kCastThreads + tid) * EPT;
                if constexpr (sizeof(OT) == 4) {
                    *reinterpret_cast<float4*>(o) = make_float4(f[0], f[1], f[2], f[3]);
                } else {
                    uint32_t pk[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if constexpr (__is_same(OT, bf16_t)) {
                            pk[j] = float_to_bf16_bits(f[2 * j]) | (float_to_bf16_bits(f[2 * j + 1]) << 16);
                        } else {
                            pk[j] = float_to_f16_bits(f[2 * j]) | (float_to_f16_bits(f[2 * j + 1]) << 16);
                        }
                    }
                    *reinterpret_cast<uint4*>(o) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
                }
            }
        } else {
            const size_t end = (base + TILE < n) ? base + TILE : n;
            for (size_t i = base + tid; i < end; i += kCastThreads) {
                Elem<OT>::store(out + i, dequant1<FMT>(q[i]) * si);
            }
        }
    }
}

// out = OT(float(x) * scale), IEEE overflow
template <typename IT, typename OT>
__global__ __launch_bounds__(kCastThreads) void scale_cast_kernel(const IT* __restrict__ x, OT* __restrict__ out,
                                                                   size_t n, const float* __restrict__ scale_p) {
    const float s = *scale_p;
    const size_t stride = static_cast<size_t>(gridDim.x) * kCastThreads;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kCastThreads + threadIdx.x; i < n; i += stride) {
        Elem<OT>::store(out + i, Elem<IT>::load(x + i) * s);
    }
}

// ---------------------------------------------------------------------------------------------
// 64x64 tile: quantize (or pass bytes through), write the row-major copy, stage the packed words
// in LDS, transpose 4x4 byte blocks in registers and write the transposed copy.
template <typename IT>
struct TileLoad {    // 4 consecutive elements of a row as floats
    static __device__ __forceinline__ void load(const IT* p, int vec, int valid, float* v) {
        if (vec && valid == 4) {
            if constexpr (sizeof(IT) == 4) {
                float4 t = *reinterpret_cast<const float4*>(p);
                v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
            } else {
                uint2 t = *reinterpret_cast<const uint2*>(p);
                if constexpr (__is_same(IT, bf16_t)) {
                    v[0] = __uint_as_float(t.x << 16), v[1] = __uint_as_float(t.x & 0xffff0000u);
                    v[2] = __uint_as_float(t.y << 16), v[3] = __uint_as_float(t.y & 0xffff0000u);
                } else {
                    v[0] = f16_bits_to_float(t.x & 0xffffu), v[1] = f16_bits_to_float(t.x >> 16);
                    v[2] = f16_bits_to_float(t.y & 0xffffu), v[3] = f16_bits_to_float(t.y >> 16);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = j < valid ? Elem<IT>::load(p + j) : 0.0f;
        }
    }
};

template <typename IT, int FMT, bool CAST, bool WITH_AMAX>
__global__ __launch_bounds__(kCastThreads) void cast_transpose_kernel(const IT* __restrict__ x,
                                                                       uint8_t* __restrict__ out,
                                                                       uint8_t* __restrict__ out_t, int R, int C,
                                                                       const float* __restrict__ scale_p,
                                                                       float* amax, float* scale_inv, int vec_in,
                                                                       int vec_out, int vec_t) {
    __shared__ uint32_t tile[64][17];
    __shared__ uint32_t red[kCastThreads / kWave];
    const int tid = threadIdx.x;
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    float s = 1.0f;
    if constexpr (CAST) s = *scale_p;
    float mx = 0.0f;
    const int wc = tid & 15;    // word column: columns c0 + 4*wc .. +3
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int lr = (tid >> 4) + 16 * i;
        const int r = r0 + lr, c = c0 + 4 * wc;
        uint32_t w = 0;
        int valid = C - c;
        valid = valid > 4 ? 4 : valid;
        if (r < R && valid > 0) {
            const size_t off = static_cast<size_t>(r) * C + c;
            if constexpr (CAST) {
                float v[4];
                TileLoad<IT>::load(x + off, vec_in, valid, v);
                if (WITH_AMAX) mx = fmaxf(fmaxf(mx, fabsf(v[0])), fmaxf(fmaxf(fabsf(v[1]), fabsf(v[2])), fabsf(v[3])));
                w = quant4<FMT>(v[0] * s, v[1] * s, v[2] * s, v[3] * s);
                if (out != nullptr) {
                    if (vec_out && valid == 4) {
                        *reinterpret_cast<uint32_t*>(out + off) = w;
                    } else {
                        for (int j = 0; j < valid; ++j) out[off + j] = static_cast<uint8_t>(w >> (8 * j));
                    }
                }
            } else {
                const uint8_t* p = reinterpret_cast<const uint8_t*>(x) + off;
                if (vec_in && valid == 4) {
                    w = *reinterpret_cast<const uint32_t*>(p);
                } else {
                    for (int j = 0; j < valid; ++j) w |= static_cast<uint32_t>(p[j]) << (8 * j);
                }
            }
        }
        tile[lr][wc] = w;
    }
    __syncthreads();
    {
        const int tr = tid & 15, tc = tid >> 4;    // rows 4*tr..+3 of the tile, word column tc
        const uint32_t w0 = tile[4 * tr][tc], w1 = tile[4 * tr + 1][tc], w2 = tile[4 * tr + 2][tc],
                       w3 = tile[4 * tr + 3][tc];
        const int row = r0 + 4 * tr;
        int rvalid = R - row;
        rvalid = rvalid > 4 ? 4 : rvalid;
        if (rvalid > 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int col = c0 + 4 * tc + i;
                if (col < C) {
                    const int sh = 8 * i;
                    const uint32_t t = ((w0 >> sh) & 0xffu) | (((w1 >> sh) & 0xffu) << 8) |
                                       (((w2 >> sh) & 0xffu) << 16) | (((w3 >> sh) & 0xffu) << 24);
                    const size_t off = static_cast<size_t>(col) * R + row;
                    if (vec_t && rvalid == 4) {
                        *reinterpret_cast<uint32_t*>(out_t + off) = t;
                    } else {
                        for (int j = 0; j < rvalid; ++j) out_t[off + j] = static_cast<uint8_t>(t >> (8 * j));
                    }
                }
            }
        }
    }
    if constexpr (CAST && WITH_AMAX) {
        uint32_t m = block_max_u32(__float_as_uint(mx), red);
        if (tid == 0) amax_publish(amax, __uint_as_float(m));
    }
    if constexpr (CAST) {
        if (scale_inv != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && tid == 0) *scale_inv = 1.0f / s;
    }
}

// ---------------------------------------------------------------------------------------------
// Byte transpose with 16-byte accesses on both sides: a 128x128 tile goes through LDS (rows rotated
// by their index so that neither side piles up on a bank), each lane gathers a 4-byte-wide, 16-row
// column strip, transposes its four 4x4 byte blocks with byte permutes and writes 16 bytes of four
// output rows.  Eight neighbouring lanes fill one 128-byte line on the way in and on the way out.
// Needs R % 16 == 0, C % 16 == 0 and 16-byte aligned pointers.
__device__ __forceinline__ void transpose4x4_bytes(uint32_t a, uint32_t b, uint32_t c, uint32_t d, uint32_t* o) {
    const uint32_t t0 = __builtin_amdgcn_perm(b, a, 0x05010400u), t1 = __builtin_amdgcn_perm(b, a, 0x07030602u);
    const uint32_t t2 = __builtin_amdgcn_perm(d, c, 0x05010400u), t3 = __builtin_amdgcn_perm(d, c, 0x07030602u);
    o[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    o[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    o[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    o[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

__global__ __launch_bounds__(kCastThreads) void byte_transpose128_kernel(const uint8_t* __restrict__ in,
                                                                          uint8_t* __restrict__ out_t, int R, int C) {
    __shared__ uint4 tile[128 * 8];    // [row][8 chunks of 16 bytes], chunk index rotated per row
    const int tid = threadIdx.x;
    const int r0 = blockIdx.y * 128, c0 = blockIdx.x * 128;
    {
        const int ch = tid & 7;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int row = p * 32 + (tid >> 3);
            uint4 t = make_uint4(0, 0, 0, 0);
            if (r0 + row < R && c0 + ch * 16 < C)
                t = *reinterpret_cast<const uint4*>(in + static_cast<size_t>(r0 + row) * C + c0 + ch * 16);
            tile[row * 8 + ((ch + (row >> 4) + (row & 7)) & 7)] = t;
        }
    }
    __syncthreads();
    const int g = tid & 7, w = tid >> 3;    // rows 16g..16g+15 of the tile, byte columns 4w..4w+3
    const uint32_t* words = reinterpret_cast<const uint32_t*>(tile);
    uint32_t o[4][4];                       // o[q][i]: column 4w+i, rows 16g+4q..+3
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        uint32_t a[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = 4 * q + j, row = 16 * g + k;
            a[j] = words[row * 32 + ((w + 4 * (g + (k & 7))) & 31)];
        }
        transpose4x4_bytes(a[0], a[1], a[2], a[3], o[q]);
    }
    if (r0 + 16 * g < R) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = c0 + 4 * w + i;
            if (c < C)
                *reinterpret_cast<uint4*>(out_t + static_cast<size_t>(c) * R + r0 + 16 * g) =
                    make_uint4(o[0][i], o[1][i], o[2][i], o[3][i]);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Cast + transpose with 16-byte loads and 128x128 tiles, for R % 16 == 0, C % 16 == 0 and 16-byte
// aligned pointers.  A workgroup walks tiles in a grid-stride loop: it quantizes eight 16-byte loads
// per lane at a time, writes the row-major bytes, parks them in LDS (same rotated layout as the byte
// transpose), then each lane gathers a 4-byte-wide, 16-row strip, transposes its 4x4 byte blocks and
// writes 16 bytes of four output rows.  Few long-lived workgroups mean few atomics on the amax cell.
template <typename IT, int FMT, bool WITH_AMAX>
__global__ __launch_bounds__(kCastThreads) void cast_transpose128_kernel(const IT* __restrict__ x,
                                                                          uint8_t* __restrict__ out,
                                                                          uint8_t* __restrict__ out_t, int R, int C,
                                                                          const float* __restrict__ scale_p,
                                                                          float* amax, float* scale_inv, int tiles_x,
                                                                          int ntiles) {
    constexpr int EPT = 16 / sizeof(IT);          // elements per 16-byte load: 8 or 4
    constexpr int TPR = 128 / EPT;                // lanes per tile row: 16 or 32
    constexpr int RPP = kCastThreads / TPR;       // rows per pass: 16 or 8
    constexpr int PASSES = 128 / RPP;             // 8 or 16
    constexpr int UNROLL = 8;
    __shared__ uint4 tile[128 * 8];
    __shared__ uint32_t red[kCastThreads / kWave];
    uint32_t* words = reinterpret_cast<uint32_t*>(tile);
    const int tid = threadIdx.x;
    const float s = *scale_p;
    float mx = 0.0f;
    const int lc = tid % TPR, lr = tid / TPR;     // this lane's column group and row within a pass
    const int g = tid & 7, w = tid >> 3;          // transposed side: rows 16g..16g+15, byte columns 4w..4w+3
    for (int t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const int r0 = (t / tiles_x) * 128, c0 = (t % tiles_x) * 128;
        const bool col_ok = c0 + lc * EPT < C;
#pragma unroll
        for (int p0 = 0; p0 < PASSES; p0 += UNROLL) {
            uint4 v[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int row = (p0 + u) * RPP + lr;
                v[u] = make_uint4(0, 0, 0, 0);
                if (col_ok && r0 + row < R)
                    v[u] = *reinterpret_cast<const uint4*>(x + static_cast<size_t>(r0 + row) * C + c0 + lc * EPT);
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int row = (p0 + u) * RPP + lr;
                float f[EPT];
                In16<IT>::decode(v[u], f);
                uint32_t q[EPT / 4];
#pragma unroll
                for (int j = 0; j < EPT / 4; ++j) {
                    const float a = f[4 * j], b = f[4 * j + 1], c = f[4 * j + 2], d = f[4 * j + 3];
                    if (WITH_AMAX) mx = fmaxf(fmaxf(mx, fabsf(a)), fmaxf(fmaxf(fabsf(b), fabsf(c)), fabsf(d)));
                    q[j] = quant4<FMT>(a * s, b * s, c * s, d * s);
                }
                const bool ok = col_ok && r0 + row < R;
                const int word = lc * (EPT / 4);    // word column of this lane's bytes within the tile row
                const int pw = ((((word >> 2) + (row >> 4) + (row & 7)) & 7) << 2) | (word & 3);
                if constexpr (EPT == 8) {
                    if (ok && out != nullptr)
                        *reinterpret_cast<uint2*>(out + static_cast<size_t>(r0 + row) * C + c0 + lc * EPT) = make_uint2(q[0], q[1]);
                    *reinterpret_cast<uint2*>(words + row * 32 + pw) = make_uint2(q[0], q[1]);
                } else {
                    if (ok && out != nullptr)
                        *reinterpret_cast<uint32_t*>(out + static_cast<size_t>(r0 + row) * C + c0 + lc * EPT) = q[0];
                    words[row * 32 + pw] = q[0];
                }
            }
        }
        __syncthreads();
        uint32_t o[4][4];    // o[q][i]: column 4w+i, rows 16g+4q..+3
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t a[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int k = 4 * q + j, row = 16 * g + k;
                a[j] = words[row * 32 + ((w + 4 * (g + (k & 7))) & 31)];
            }
            transpose4x4_bytes(a[0], a[1], a[2], a[3], o[q]);
        }
        if (r0 + 16 * g < R) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int c = c0 + 4 * w + i;
                if (c < C)
                    *reinterpret_cast<uint4*>(out_t + static_cast<size_t>(c) * R + r0 + 16 * g) =
                        make_uint4(o[0][i], o[1][i], o[2][i], o[3][i]);
            }
        }
        __syncthreads();    // the tile is free for the next round
    }
    if constexpr (WITH_AMAX) {
        uint32_t m = block_max_u32(__float_as_uint(mx), red);
        if (tid == 0) amax_publish(amax, __uint_as_float(m));
    }
    if (scale_inv != nullptr && blockIdx.x == 0 && tid == 0) *scale_inv = 1.0f / s;
}

// ---------------------------------------------------------------------------------------------
__global__ void scaling_factor_kernel(const float* amax, const float* scale_in, int scale_in_n, float* scale_out, int n,
                                      float fp_max, int margin) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) scale_out[i] = scale_rule(amax[i], scale_in[scale_in_n == 1 ? 0 : i], fp_max, margin);
}

__device__ __forceinline__ float nanmax(float a, float b) { return (a != a) ? a : ((b != b) ? b : fmaxf(a, b)); }

// One wavefront per meta (window <= 64): lane j holds amaxs[i][j], so the row is read and written
// with one load and one store per lane instead of a chain of dependent accesses; the scale and the
// counter are fetched with the row, not after the reduction.
__device__ __forceinline__ void scale_update_row(float* scales, float* amaxs, uint8_t* bad, int32_t* counters, int i,
                                                 int window, float fp_max, int margin) {
    const int lane = threadIdx.x & 63;
    float* row = amaxs + static_cast<size_t>(i) * window;
    float v = lane < window ? row[lane] : 0.0f;
    const float old_scale = scales[i];
    const int32_t old_count = counters != nullptr ? counters[i] : 0;
    const float a0_raw = __shfl(v, 0);
    const bool is_bad = !(fabsf(a0_raw) < __uint_as_float(0x7f800000u));
    const float a0 = is_bad ? 0.0f : a0_raw;
    if (lane == 0) v = a0;
    // NaN-propagating maximum over the window, as torch.max does
    float mx = v;
#pragma unroll
    for (int o = 32; o; o >>= 1) mx = nanmax(mx, __shfl_xor(mx, o));
    // shift: row[j] <- row[j-1] for j >= 1 (row[1] gets the cleaned current value), row[0] <- 0
    const float left = __shfl_up(v, 1);
    if (lane < window) row[lane] = lane == 0 ? 0.0f : left;
    if (lane == 0) {
        scales[i] = scale_rule(mx, old_scale, fp_max, margin);
        if (bad != nullptr) bad[i] = is_bad ? 1 : 0;
        if (counters != nullptr) counters[i] = is_bad ? 0 : old_count + 1;
    }
}

__global__ __launch_bounds__(256) void scale_update_kernel(float* scales, float* amaxs, uint8_t* bad,
                                                            int32_t* counters, int n, int window, float fp_max,
                                                            int margin) {
    const int i = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (i >= n) return;
    scale_update_row(scales, amaxs, bad, counters, i, window, fp_max, margin);
}

// several groups of metas (one format and window each) in one launch: blockIdx.y picks the group
struct ScaleGroups {
    msamp_scale_group g[MSAMP_MAX_SCALE_GROUPS];
};
__global__ __launch_bounds__(256) void scale_update_groups_kernel(ScaleGroups groups, int margin) {
    const msamp_scale_group& g = groups.g[blockIdx.y];
    const int i = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (i >= g.n) return;
    scale_update_row(g.scales, g.amaxs, g.bad, g.counters, i, g.window, g.fp_max, margin);
}

// any window: one lane per meta
__global__ void scale_update_wide_kernel(float* scales, float* amaxs, uint8_t* bad, int32_t* counters, int n, int window,
                                         float fp_max, int margin) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float* row = amaxs + static_cast<size_t>(i) * window;
    float a0 = row[0];
    const bool is_bad = !(fabsf(a0) < __uint_as_float(0x7f800000u));
    if (is_bad) a0 = 0.0f;
    float mx = a0;
    for (int j = 1; j < window; ++j) mx = nanmax(mx, row[j]);
    const float sf = scale_rule(mx, scales[i], fp_max, margin);
    for (int j = window - 1; j >= 2; --j) row[j] = row[j - 1];
    if (window > 1) row[1] = a0;
    row[0] = 0.0f;
    scales[i] = sf;
    if (bad != nullptr) bad[i] = is_bad ? 1 : 0;
    if (counters != nullptr) counters[i] = is_bad ? 0 : counters[i] + 1;
}

// ---------------------------------------------------------------------------------------------
static int grid_for(size_t n, size_t tile) {
    size_t tiles = (n + tile - 1) / tile;
    size_t cap = static_cast<size_t>(cu_count()) * 8;
    if (tiles < 1) tiles = 1;
    return static_cast<int>(tiles < cap ? tiles : cap);
}

template <typename IT>
static int launch_cast(const IT* x, size_t n, const float* scale, float* amax, float* scale_inv, uint8_t* out,
                       int fp8_type, const InTimeArgs* it, hipStream_t st) {
    constexpr int EPT = In16<IT>::EPT;
    // bit 0: 16-byte accesses fit; bit 1: the input is larger than the caches keep, read it as a stream
    const int vec_only = aligned(x, 16) && aligned(out, EPT);
    const int vec_ok = vec_only | (n * sizeof(IT) >= kStreamBytes ? 2 : 0);
    int grid = grid_for(n, static_cast<size_t>(kCastThreads) * EPT * kCastUnroll);
    const InTimeArgs none = {nullptr, nullptr, nullptr, 0.0f, 0, 0, nullptr, nullptr, nullptr, 0, nullptr};
#define LAUNCH(FMT, AM, INT) \
    hipLaunchKernelGGL((cast_to_fp8_kernel<IT, FMT, AM, INT>), dim3(grid), dim3(kCastThreads), 0, st, x, out, n, scale, amax, scale_inv, INT == kInTime ? vec_only : vec_ok, INT == kInTime ? 1 : 0, INT != kGivenScale ? *it : none)
    if (it != nullptr && it->known_amax != nullptr) {
        // few, large, long-lived workgroups (two of 512 lanes per CU, grid-stride), like the cast that publishes an amax
        constexpr int kBigThreads = 512;
        int g2 = grid_for(n, static_cast<size_t>(kBigThreads) * EPT * kCastUnroll);
        const int cap = cu_count() * 2;
        g2 = g2 < cap ? g2 : cap;
#define LAUNCH_RESCALE(FMT) \
    hipLaunchKernelGGL((cast_to_fp8_kernel<IT, FMT, false, kRescale, kBigThreads>), dim3(g2), dim3(kBigThreads), 0, st, x, out, n, scale, amax, scale_inv, vec_ok, 0, *it)
        if (fp8_type == MSAMP_DT_E4M3) LAUNCH_RESCALE(MSAMP_DT_E4M3); else LAUNCH_RESCALE(MSAMP_DT_E5M2);
#undef LAUNCH_RESCALE
    } else if (it != nullptr) {
        // second pass of an in-time cast: fewer, longer-lived workgroups (each one re-derives the scale),
        // walking the tensor back to front to meet what the first pass left in the caches
        const int cap = cu_count() * 4;
        grid = grid < cap ? grid : cap;
        if (fp8_type == MSAMP_DT_E4M3) LAUNCH(MSAMP_DT_E4M3, false, kInTime); else LAUNCH(MSAMP_DT_E5M2, false, kInTime);
    } else if (amax != nullptr) {
        constexpr int kAmaxThreads = 512;
        int g2 = grid_for(n, static_cast<size_t>(kAmaxThreads) * EPT * kCastUnroll);
        const int cap = cu_count() * 2;
        g2 = g2 < cap ? g2 : cap;
#define LAUNCH_AMAX(FMT) \
    hipLaunchKernelGGL((cast_to_fp8_kernel<IT, FMT, true, kGivenScale, kAmaxThreads>), dim3(g2), dim3(kAmaxThreads), 0, st, x, out, n, scale, amax, scale_inv, vec_ok, 0, none)
        if (fp8_type == MSAMP_DT_E4M3) LAUNCH_AMAX(MSAMP_DT_E4M3); else LAUNCH_AMAX(MSAMP_DT_E5M2);
#undef LAUNCH_AMAX
    } else if (fp8_type == MSAMP_DT_E4M3) {
        LAUNCH(MSAMP_DT_E4M3, false, kGivenScale);
    } else {
        LAUNCH(MSAMP_DT_E5M2, false, kGivenScale);
    }
#undef LAUNCH
    MSAMP_CHECK_LAUNCH("cast_to_fp8_kernel");
    return MSAMP_OK;
}

template <typename IT>
static int launch_amax(const IT* x, size_t n, uint32_t* ws, const float* scale, Gate gate, Finish fin, hipStream_t st) {
    constexpr int EPT = 16 / sizeof(IT);
    const int vec_ok = aligned(x, 16);
    int grid = grid_for(n, static_cast<size_t>(kCastThreads) * EPT * 8);
    const int cap = cu_count() * 4 < kMaxPartials ? cu_count() * 4 : kMaxPartials;
    grid = grid < cap ? grid : cap;
    hipLaunchKernelGGL((amax_partial_kernel<IT>), dim3(grid), dim3(kCastThreads), 0, st, x, n, ws, scale, vec_ok, gate, fin);
    MSAMP_CHECK_LAUNCH("amax_partial_kernel");
    return MSAMP_OK;
}

template <typename IT>
static int launch_cast_if_flagged(const IT* d, size_t n, const float* scale, uint8_t* q, int q_type, const uint32_t* redo,
                                  hipStream_t st) {
    constexpr int EPT = In16<IT>::EPT;
    const int vec_ok = (aligned(d, 16) && aligned(q, EPT) ? 1 : 0) | (n * sizeof(IT) >= kStreamBytes ? 2 : 0);
    // as a rule every workgroup returns at once: few of them, grid-stride
    int grid = grid_for(n, static_cast<size_t>(kCastThreads) * EPT * kCastUnroll);
    const int cap = cu_count() * 4;
    grid = grid < cap ? grid : cap;
    const InTimeArgs flag = {redo, nullptr, nullptr, 0.0f, 0, 0, nullptr, nullptr, nullptr, 0, nullptr, 0};
    if (q_type == MSAMP_DT_E4M3)
        hipLaunchKernelGGL((cast_to_fp8_kernel<IT, MSAMP_DT_E4M3, false, kGivenIfFlagged>), dim3(grid), dim3(kCastThreads), 0, st, d, q, n,
                           scale, static_cast<float*>(nullptr), static_cast<float*>(nullptr), vec_ok, 0, flag);
    else
        hipLaunchKernelGGL((cast_to_fp8_kernel<IT, MSAMP_DT_E5M2, false, kGivenIfFlagged>), dim3(grid), dim3(kCastThreads), 0, st, d, q, n,
                           scale, static_cast<float*>(nullptr), static_cast<float*>(nullptr), vec_ok, 0, flag);
    MSAMP_CHECK_LAUNCH("cast_to_fp8_kernel (if flagged)");
    return MSAMP_OK;
}

// first pass: partial maxima of |x| into the workspace (plus the scale in force, for the rule's fallback)
constexpr Gate kNoGate = {nullptr, 0};

constexpr Finish kNoFinish = {nullptr, nullptr, nullptr, 0.0f, 0, 0};

static int dispatch_amax(const void* x, int dtype, size_t n, void* ws, const float* scale, hipStream_t st,
                         Gate gate = kNoGate, Finish fin = kNoFinish) {
    uint32_t* w = static_cast<uint32_t*>(ws);
    switch (dtype) {
        case MSAMP_DT_F32:
            return launch_amax(static_cast<const float*>(x), n, w, scale, gate, fin, st);
        case MSAMP_DT_F16:
            return launch_amax(static_cast<const f16_t*>(x), n, w, scale, gate, fin, st);
        case MSAMP_DT_BF16:
            return launch_amax(static_cast<const bf16_t*>(x), n, w, scale, gate, fin, st);
    }
    set_error("unsupported input dtype %d", dtype);
    return MSAMP_ERR_DTYPE;
}

// true if the runtime confirms kResBlocksPerCu workgroups of this kernel fit one CU; `state` is the caller's
// function-local cache for one instantiation (-1 = not asked yet)
static bool fits_resident(const void* fn, std::atomic<int>& state) {
    int fits = state.load(std::memory_order_acquire);
    if (fits < 0) {
        int blocks = 0;
        fits = hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, fn, kResThreads, 0) == hipSuccess && blocks >= kResBlocksPerCu;
        state.store(fits, std::memory_order_release);
    }
    return fits != 0;
}

// One-pass (register-resident) in-time cast; returns 1 if it does not apply and the two-pass path must run.
template <typename IT, bool SPEC>
static int launch_resident(const IT* x, size_t n, float* scale, float* amax, float* scale_inv, uint8_t* out,
                           int fp8_type, int margin, int flags, void* ws, hipStream_t st) {
    constexpr int EPT = 16 / sizeof(IT);
    if (flags & MSAMP_FLAG_TWO_PASS) return 1;
    if (!aligned(x, 16) || !aligned(out, EPT)) return 1;
    const size_t nvec = n / EPT;
    size_t max_blocks = static_cast<size_t>(cu_count()) * kResBlocksPerCu;
    if (max_blocks > static_cast<size_t>(kMaxSlots)) max_blocks = kMaxSlots;
    if (nvec == 0 || nvec > max_blocks * kResThreads * kResVecs) return 1;
    if (!waiting_kernels_allowed(st)) return 1;
    // as many workgroups as there are runs of kResThreads vectors, up to the resident limit
    size_t g = (nvec + kResThreads - 1) / kResThreads;
    g = g > max_blocks ? max_blocks : g;
    int rounds = static_cast<int>((nvec + g * kResThreads - 1) / (g * kResThreads));
    g = (nvec + static_cast<size_t>(rounds) * kResThreads - 1) / (static_cast<size_t>(rounds) * kResThreads);
    const uint32_t token = next_tokens(1);
    uint64_t* slots = reinterpret_cast<uint64_t*>(static_cast<char*>(ws) + kWsSlotBytes);
    const float fp_max = fp8_max(fp8_type);
    const uint32_t spin_limit = collector_spin_limit();
    uint32_t* error_word = static_cast<uint32_t*>(ws) + kWsErrorWord;
    // the runtime must confirm, for the very instantiation that is launched, that kResBlocksPerCu workgroups fit a CU
    bool fits = true;
#define LAUNCH(FMT, R) \
    do { \
        static std::atomic<int> fits_state{-1}; \
        fits = fits_resident(reinterpret_cast<const void*>(&cast_intime_resident_kernel<IT, FMT, R, SPEC>), fits_state); \
        if (fits) hipLaunchKernelGGL((cast_intime_resident_kernel<IT, FMT, R, SPEC>), dim3(static_cast<unsigned>(g)), dim3(kResThreads), 0, st, x, out, n, scale, amax, scale_inv, slots, fp_max, margin, flags, rounds, token, spin_limit, error_word); \
    } while (0)
#define LAUNCH_R(FMT) \
    do { if (rounds <= 4) LAUNCH(FMT, 4); else if (rounds <= 8) LAUNCH(FMT, 8); else LAUNCH(FMT, kResVecs); } while (0)
    if (fp8_type == MSAMP_DT_E4M3) LAUNCH_R(MSAMP_DT_E4M3); else LAUNCH_R(MSAMP_DT_E5M2);
#undef LAUNCH_R
#undef LAUNCH
    if (!fits) return 1;
    MSAMP_CHECK_LAUNCH("cast_intime_resident_kernel");
    return MSAMP_OK;
}

static int dispatch_resident(const void* x, int dtype, size_t n, float* scale, float* amax, float* scale_inv, uint8_t* out,
                             int fp8_type, int margin, int flags, void* ws, hipStream_t st) {
    const bool spec = !(flags & MSAMP_FLAG_NO_SPECULATION);
#define RESIDENT(T) \
    (spec ? launch_resident<T, true>(static_cast<const T*>(x), n, scale, amax, scale_inv, out, fp8_type, margin, flags, ws, st) \
          : launch_resident<T, false>(static_cast<const T*>(x), n, scale, amax, scale_inv, out, fp8_type, margin, flags, ws, st))
    switch (dtype) {
        case MSAMP_DT_F32:
            return RESIDENT(float);
        case MSAMP_DT_F16:
            return RESIDENT(f16_t);
        case MSAMP_DT_BF16:
            return RESIDENT(bf16_t);
    }
#undef RESIDENT
    return 1;
}

template <typename IT>
static int launch_speculative(const IT* x, size_t n, const float* scale, const float* amax, uint8_t* out, int fp8_type,
                              uint32_t* ws, hipStream_t st) {
    constexpr int EPT = In16<IT>::EPT;
    // bit 1: stream the input (this pass reads it once; measured faster at 64 MiB as well as at 470 MiB)
    const int vec_ok = (aligned(x, 16) && aligned(out, EPT) ? 1 : 0) | 2;
    int grid = grid_for(n, static_cast<size_t>(kSpecThreads) * EPT * kCastUnroll);
    const int cap = cu_count() * 2 < kMaxPartials ? cu_count() * 2 : kMaxPartials;
    grid = grid < cap ? grid : cap;
    if (fp8_type == MSAMP_DT_E4M3)
        hipLaunchKernelGGL((cast_speculative_kernel<IT, MSAMP_DT_E4M3>), dim3(grid), dim3(kSpecThreads), 0, st, x, out, n, scale, amax, ws, vec_ok);
    else
        hipLaunchKernelGGL((cast_speculative_kernel<IT, MSAMP_DT_E5M2>), dim3(grid), dim3(kSpecThreads), 0, st, x, out, n, scale, amax, ws, vec_ok);
    MSAMP_CHECK_LAUNCH("cast_speculative_kernel");
    return MSAMP_OK;
}

static int dispatch_speculative(const void* x, int dtype, size_t n, const float* scale, const float* amax, uint8_t* out,
                                int fp8_type, void* ws, hipStream_t st) {
    uint32_t* w = static_cast<uint32_t*>(ws);
    switch (dtype) {
        case MSAMP_DT_F32:
            return launch_speculative(static_cast<const float*>(x), n, scale, amax, out, fp8_type, w, st);
        case MSAMP_DT_F16:
            return launch_speculative(static_cast<const f16_t*>(x), n, scale, amax, out, fp8_type, w, st);
        case MSAMP_DT_BF16:
            return launch_speculative(static_cast<const bf16_t*>(x), n, scale, amax, out, fp8_type, w, st);
    }
    set_error("unsupported input dtype %d", dtype);
    return MSAMP_ERR_DTYPE;
}

static int finalize_amax(void* ws, float* amax, float* scale, float* scale_inv, float fp_max, int margin, int flags,
                         int update_scale, hipStream_t st, Gate gate = kNoGate) {
    hipLaunchKernelGGL(amax_finalize_kernel, dim3(1), dim3(kCastThreads), 0, st, static_cast<const uint32_t*>(ws), amax, scale,
                       scale_inv, fp_max, margin, flags, update_scale, gate);
    MSAMP_CHECK_LAUNCH("amax_finalize_kernel");
    return MSAMP_OK;
}

static int dispatch_cast(const void* x, int dtype, size_t n, const float* scale, float* amax, float* scale_inv,
                         uint8_t* out, int fp8_type, const InTimeArgs* it, hipStream_t st) {
    switch (dtype) {
        case MSAMP_DT_F32:
            return launch_cast(static_cast<const float*>(x), n, scale, amax, scale_inv, out, fp8_type, it, st);
        case MSAMP_DT_F16:
            return launch_cast(static_cast<const f16_t*>(x), n, scale, amax, scale_inv, out, fp8_type, it, st);
        case MSAMP_DT_BF16:
            return launch_cast(static_cast<const bf16_t*>(x), n, scale, amax, scale_inv, out, fp8_type, it, st);
    }
    set_error("unsupported input dtype %d", dtype);
    return MSAMP_ERR_DTYPE;
}

template <typename IT, bool CAST>
static int launch_ct(const IT* x, int rows, int cols, const float* scale, float* amax, float* scale_inv, uint8_t* out,
                     uint8_t* out_t, int fp8_type, hipStream_t st) {
    const int esz = CAST ? static_cast<int>(sizeof(IT)) : 1;
    const int vec_in = (cols % 4 == 0) && aligned(x, 4 * esz);
    const int vec_out = (cols % 4 == 0) && (out == nullptr || aligned(out, 4));
    const int vec_t = (rows % 4 == 0) && aligned(out_t, 4);
    if constexpr (CAST) {
        if (rows % 16 == 0 && cols % 16 == 0 && aligned(x, 16) && (out == nullptr || aligned(out, 16)) && aligned(out_t, 16)) {
            const int tiles_x = (cols + 127) / 128;
            const long long ntiles_ll = static_cast<long long>(tiles_x) * ((rows + 127) / 128);
            if (ntiles_ll <= 0x7fffffffLL) {
                const int ntiles = static_cast<int>(ntiles_ll);
                const int cap = cu_count() * 2;
                const int g = ntiles < cap ? ntiles : cap;
#define LAUNCH128(FMT, AM) \
    hipLaunchKernelGGL((cast_transpose128_kernel<IT, FMT, AM>), dim3(g), dim3(kCastThreads), 0, st, x, out, out_t, rows, cols, scale, amax, scale_inv, tiles_x, ntiles)
                if (fp8_type == MSAMP_DT_E4M3) {
                    if (amax) LAUNCH128(MSAMP_DT_E4M3, true); else LAUNCH128(MSAMP_DT_E4M3, false);
                } else {
                    if (amax) LAUNCH128(MSAMP_DT_E5M2, true); else LAUNCH128(MSAMP_DT_E5M2, false);
                }
#undef LAUNCH128
                MSAMP_CHECK_LAUNCH("cast_transpose128_kernel");
                return MSAMP_OK;
            }
        }
    }
    dim3 grid((cols + 63) / 64, (rows + 63) / 64);
    MSAMP_REQUIRE(grid.y <= 65535u, MSAMP_ERR_SHAPE, "too many rows for one launch: %d", rows);
#define LAUNCH(FMT, AM) \
    hipLaunchKernelGGL((cast_transpose_kernel<IT, FMT, CAST, AM>), grid, dim3(kCastThreads), 0, st, x, out, out_t, rows, cols, scale, amax, scale_inv, vec_in, vec_out, vec_t)
    if (fp8_type == MSAMP_DT_E4M3) {
        if (amax) LAUNCH(MSAMP_DT_E4M3, true); else LAUNCH(MSAMP_DT_E4M3, false);
    } else {
        if (amax) LAUNCH(MSAMP_DT_E5M2, true); else LAUNCH(MSAMP_DT_E5M2, false);
    }
#undef LAUNCH
    MSAMP_CHECK_LAUNCH("cast_transpose_kernel");
    return MSAMP_OK;
}

static int dispatch_ct(const void* x, int dtype, int rows, int cols, const float* scale, float* amax, float* scale_inv,
                       uint8_t* out, uint8_t* out_t, int fp8_type, hipStream_t st) {
    switch (dtype) {
        case MSAMP_DT_F32:
            return launch_ct<float, true>(static_cast<const float*>(x), rows, cols, scale, amax, scale_inv, out, out_t, fp8_type, st);
        case MSAMP_DT_F16:
            return launch_ct<f16_t, true>(static_cast<const f16_t*>(x), rows, cols, scale, amax, scale_inv, out, out_t, fp8_type, st);
        case MSAMP_DT_BF16:
            return launch_ct<bf16_t, true>(static_cast<const bf16_t*>(x), rows, cols, scale, amax, scale_inv, out, out_t, fp8_type, st);
    }
    set_error("unsupported input dtype %d", dtype);
    return MSAMP_ERR_DTYPE;
}

template <typename IT>
static int launch_scale_cast_out(const IT* x, size_t n, const float* scale, void* out, int out_dtype, hipStream_t st) {
    const int grid = grid_for(n, kCastThreads * 4);
    switch (out_dtype) {
        case MSAMP_DT_F32:
            hipLaunchKernelGGL((scale_cast_kernel<IT, float>), dim3(grid), dim3(kCastThreads), 0, st, x, static_cast<float*>(out), n, scale);
            break;
        case MSAMP_DT_F16:
            hipLaunchKernelGGL((scale_cast_kernel<IT, f16_t>), dim3(grid), dim3(kCastThreads), 0, st, x, static_cast<f16_t*>(out), n, scale);
            break;
        case MSAMP_DT_BF16:
            hipLaunchKernelGGL((scale_cast_kernel<IT, bf16_t>), dim3(grid), dim3(kCastThreads), 0, st, x, static_cast<bf16_t*>(out), n, scale);
            break;
        default:
            set_error("unsupported output dtype %d", out_dtype);
            return MSAMP_ERR_DTYPE;
    }
    MSAMP_CHECK_LAUNCH("scale_cast_kernel");
    return MSAMP_OK;
}

// ---------------------------------------------------------------------------------------------
// add_to_fp8: q <- cast_in_time(IT(dequant(q)) + other), in place (operators/arithmetic/arithmetic.py:15-35,
// vectorized_pointwise.h:184-301).  t = IT(float(q) * scale_inv) + other with the sum rounded to IT, as
// torch adds two IT tensors; amax = max|t|; scale by the rule; q = fp8(float(t) * scale).  Two passes over
// q and other; the old scale_inv travels in workspace word kWsOldScaleInv because the second pass replaces it.
constexpr int kWsOldScaleInv = 6;

template <typename IT>
__device__ __forceinline__ float round_to(float v) {
    if constexpr (sizeof(IT) == 4) return v;
    else if constexpr (__is_same(IT, bf16_t)) return bf16_bits_to_float(float_to_bf16_bits(v));
    else return f16_bits_to_float(float_to_f16_bits(v));
}

template <typename IT, int FMT>
__device__ __forceinline__ float add_term(uint32_t code, float other, float si) {
    return round_to<IT>(round_to<IT>(dequant1<FMT>(code) * si) + other);
}

template <typename IT, int FMT>
__global__ __launch_bounds__(kCastThreads) void add_amax_partial_kernel(const uint8_t* __restrict__ q,
                                                                         const IT* __restrict__ other, size_t n,
                                                                         uint32_t* ws, const float* scale,
                                                                         const float* scale_inv, int vec_ok) {
    __shared__ uint32_t red[kCastThreads / kWave];
    const float si = *scale_inv;
    uint32_t m = 0;
    const size_t stride = static_cast<size_t>(gridDim.x) * kCastThreads * 4;
    for (size_t i = (static_cast<size_t>(blockIdx.x) * kCastThreads + threadIdx.x) * 4; i < n; i += stride) {
        if (i + 4 <= n && vec_ok) {
            const uint32_t w = *reinterpret_cast<const uint32_t*>(q + i);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float t = add_term<IT, FMT>((w >> (8 * j)) & 0xffu, Elem<IT>::load(other + i + j), si);
                m = umax(m, __float_as_uint(t) & 0x7fffffffu);
            }
        } else {
            for (size_t e = i; e < n && e < i + 4; ++e) {
                const float t = add_term<IT, FMT>(q[e], Elem<IT>::load(other + e), si);
                m = umax(m, __float_as_uint(t) & 0x7fffffffu);
            }
        }
    }
    m = block_max_u32(m, red);
    if (threadIdx.x == 0) {
        ws[kWsPartials + blockIdx.x] = m;
        if (blockIdx.x == 0) {
            ws[0] = __float_as_uint(*scale);
            ws[1] = gridDim.x;
            ws[kWsOldScaleInv] = __float_as_uint(si);
        }
    }
}

template <typename IT, int FMT>
__global__ __launch_bounds__(kCastThreads) void add_cast_kernel(uint8_t* __restrict__ q, const IT* __restrict__ other,
                                                                 size_t n, float* scale_inv, InTimeArgs it, int vec_ok) {
    __shared__ uint32_t red[kCastThreads / kWave];
    const float si = __uint_as_float(it.ws[kWsOldScaleInv]);
    const float s = resolve_in_time_scale(it, red, scale_inv);
    const size_t stride = static_cast<size_t>(gridDim.x) * kCastThreads * 4;
    for (size_t i = (static_cast<size_t>(blockIdx.x) * kCastThreads + threadIdx.x) * 4; i < n; i += stride) {
        if (i + 4 <= n && vec_ok) {
            const uint32_t w = *reinterpret_cast<const uint32_t*>(q + i);
            float t[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) t[j] = add_term<IT, FMT>((w >> (8 * j)) & 0xffu, Elem<IT>::load(other + i + j), si);
            *reinterpret_cast<uint32_t*>(q + i) = quant4<FMT>(t[0] * s, t[1] * s, t[2] * s, t[3] * s);
        } else {
            for (size_t e = i; e < n && e < i + 4; ++e)
                q[e] = static_cast<uint8_t>(quant1<FMT>(add_term<IT, FMT>(q[e], Elem<IT>::load(other + e), si) * s));
        }
    }
}

template <typename IT>
static int launch_add_to_fp8(uint8_t* q, int fp8_type, const IT* other, size_t n, float* scale, float* scale_inv, float* amax,
                             uint32_t* ws, hipStream_t st) {
    int grid = grid_for(n, static_cast<size_t>(kCastThreads) * 4 * 4);
    const int cap = cu_count() * 4 < kMaxPartials ? cu_count() * 4 : kMaxPartials;
    grid = grid < cap ? grid : cap;
    const InTimeArgs it = {ws, scale, amax, fp8_max(fp8_type), 0, 0, nullptr, nullptr, nullptr, 0, nullptr};
    const int vec_ok = aligned(q, 4);
    if (fp8_type == MSAMP_DT_E4M3) {
        hipLaunchKernelGGL((add_amax_partial_kernel<IT, MSAMP_DT_E4M3>), dim3(grid), dim3(kCastThreads), 0, st, q, other, n, ws, scale, scale_inv, vec_ok);
        hipLaunchKernelGGL((add_cast_kernel<IT, MSAMP_DT_E4M3>), dim3(grid), dim3(kCastThreads), 0, st, q, other, n, scale_inv, it, vec_ok);
    } else {
        hipLaunchKernelGGL((add_amax_partial_kernel<IT, MSAMP_DT_E5M2>), dim3(grid), dim3(kCastThreads), 0, st, q, other, n, ws, scale, scale_inv, vec_ok);
        hipLaunchKernelGGL((add_cast_kernel<IT, MSAMP_DT_E5M2>), dim3(grid), dim3(kCastThreads), 0, st, q, other, n, scale_inv, it, vec_ok);
    }
    MSAMP_CHECK_LAUNCH("add_to_fp8 kernels");
    return MSAMP_OK;
}

// ---------------------------------------------------------------------------------------------
// Workspace of msamp_cast_to_fp8_intime_static: the same MSAMP_WORKSPACE_BYTES the other in-time entry points
// are handed by their caller, but owned by the library, so that the call needs no allocation anywhere.  Every
// GPU holds its own copy of the array at its own address; host code never uses the array's name as a pointer,
// only the address hipGetSymbolAddress reports for the device that is current.
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[MSAMP_WORKSPACE_BYTES];

int static_workspace(void** ws) {
    static std::mutex mu;
    static void* ptrs[64];
    static bool known[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    MSAMP_REQUIRE(dev >= 0 && dev < 64, MSAMP_ERR_SHAPE, "static workspace: device index %d", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!known[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
        MSAMP_REQUIRE(p != nullptr, MSAMP_ERR_WORKSPACE, "no address for the static workspace");
        ptrs[dev] = p;
        known[dev] = true;
    }
    *ws = ptrs[dev];
    return MSAMP_OK;
}

int cast_again_if_flagged(const void* d, int d_dtype, size_t n, const float* scale, uint8_t* q, int q_type, const uint32_t* redo,
                          hipStream_t st) {
    switch (d_dtype) {
        case MSAMP_DT_F32:
            return launch_cast_if_flagged(static_cast<const float*>(d), n, scale, q, q_type, redo, st);
        case MSAMP_DT_F16:
            return launch_cast_if_flagged(static_cast<const f16_t*>(d), n, scale, q, q_type, redo, st);
        case MSAMP_DT_BF16:
            return launch_cast_if_flagged(static_cast<const bf16_t*>(d), n, scale, q, q_type, redo, st);
    }
    set_error("unsupported dtype %d", d_dtype);
    return MSAMP_ERR_DTYPE;
}

}    // namespace msamp

using namespace msamp;

extern "C" {

int msamp_amax(const void* x, int dtype, size_t n, float* amax, void* workspace, msamp_stream_t stream) {
    MSAMP_REQUIRE(amax != nullptr && (x != nullptr || n == 0), MSAMP_ERR_NULL, "msamp_amax: null pointer");
    MSAMP_REQUIRE(workspace != nullptr, MSAMP_ERR_WORKSPACE, "msamp_amax: workspace required");
    MSAMP_REQUIRE(is_hp(dtype), MSAMP_ERR_DTYPE, "msamp_amax: unsupported dtype %d", dtype);
    hipStream_t st = static_cast<hipStream_t>(stream);
    int rc = dispatch_amax(x, dtype, n, workspace, nullptr, st);
    if (rc != MSAMP_OK) return rc;
    return finalize_amax(workspace, amax, nullptr, nullptr, 0.0f, 0, 0, 0, st);
}

int msamp_compute_scaling_factor(const float* amax, const float* scale_in, int scale_in_n, float* scale_out, int n,
                                 float fp_max, int margin, msamp_stream_t stream) {
    MSAMP_REQUIRE(n >= 0 && (scale_in_n == 1 || scale_in_n == n), MSAMP_ERR_SHAPE,
                  "msamp_compute_scaling_factor: n=%d scale_in_n=%d", n, scale_in_n);
    if (n == 0) return MSAMP_OK;
    MSAMP_REQUIRE(amax && scale_in && scale_out, MSAMP_ERR_NULL, "msamp_compute_scaling_factor: null pointer");
    hipLaunchKernelGGL(scaling_factor_kernel, dim3((n + 127) / 128), dim3(128), 0, static_cast<hipStream_t>(stream), amax,
                       scale_in, scale_in_n, scale_out, n, fp_max, margin);
    MSAMP_CHECK_LAUNCH("scaling_factor_kernel");
    return MSAMP_OK;
}

int msamp_cast_to_fp8(const void* x, int in_dtype, size_t n, const float* scale, float* amax, float* scale_inv,
                      uint8_t* out, int fp8_type, msamp_stream_t stream) {
    MSAMP_REQUIRE(is_fp8(fp8_type), MSAMP_ERR_DTYPE, "msamp_cast_to_fp8: fp8_type %d", fp8_type);
    MSAMP_REQUIRE(is_hp(in_dtype), MSAMP_ERR_DTYPE, "msamp_cast_to_fp8: in_dtype %d", in_dtype);
    MSAMP_REQUIRE(scale != nullptr && ((x != nullptr && out != nullptr) || n == 0), MSAMP_ERR_NULL,
                  "msamp_cast_to_fp8: null pointer");
    return dispatch_cast(x, in_dtype, n, scale, amax, scale_inv, out, fp8_type, nullptr, static_cast<hipStream_t>(stream));
}

int msamp_cast_to_fp8_intime(const void* x, int in_dtype, size_t n, float* scale, float* amax, float* scale_inv,
                             uint8_t* out, int fp8_type, int margin, int flags, void* workspace,
                             msamp_stream_t stream) {
    MSAMP_REQUIRE(is_fp8(fp8_type), MSAMP_ERR_DTYPE, "msamp_cast_to_fp8_intime: fp8_type %d", fp8_type);
    MSAMP_REQUIRE(is_hp(in_dtype), MSAMP_ERR_DTYPE, "msamp_cast_to_fp8_intime: in_dtype %d", in_dtype);
    MSAMP_REQUIRE(scale && amax && scale_inv && ((x && out) || n == 0), MSAMP_ERR_NULL,
                  "msamp_cast_to_fp8_intime: null pointer");
    MSAMP_REQUIRE(workspace != nullptr, MSAMP_ERR_WORKSPACE, "msamp_cast_to_fp8_intime: workspace required");
    hipStream_t st = static_cast<hipStream_t>(stream);
    int rc = dispatch_resident(x, in_dtype, n, scale, amax, scale_inv, out, fp8_type, margin, flags, workspace, st);
    if (rc <= 0) return rc;
    const int speculative = (flags & MSAMP_FLAG_NO_SPECULATION) ? 0 : 1;
    if (speculative) rc = dispatch_speculative(x, in_dtype, n, scale, amax, out, fp8_type, workspace, st);
    else rc = dispatch_amax(x, in_dtype, n, workspace, scale, st);
    if (rc != MSAMP_OK) return rc;
    const InTimeArgs it = {static_cast<const uint32_t*>(workspace), scale, amax, fp8_max(fp8_type), margin, flags, nullptr, nullptr, nullptr, 0, nullptr, speculative};
    return dispatch_cast(x, in_dtype, n, scale, nullptr, scale_inv, out, fp8_type, &it, st);
}

int msamp_cast_to_fp8_intime_static(const void* x, int in_dtype, size_t n, float* scale, float* amax, float* scale_inv,
                                    uint8_t* out, int fp8_type, int margin, int flags, msamp_stream_t stream) {
    MSAMP_REQUIRE(n <= MSAMP_STATIC_MAX_ELEMS, MSAMP_ERR_SHAPE,
                  "msamp_cast_to_fp8_intime_static: n=%zu exceeds the limit of %llu elements", n,
                  static_cast<unsigned long long>(MSAMP_STATIC_MAX_ELEMS));
    void* ws = nullptr;
    const int rc = static_workspace(&ws);
    if (rc != MSAMP_OK) return rc;
    // Nothing in the workspace has to start at zero for this path: the header words and the partial maxima are
    // rewritten by every call's first kernel before its second reads them, and the slots through which the
    // one-pass kernel's workgroups meet are tagged with a token that is new for every call.
    return msamp_cast_to_fp8_intime(x, in_dtype, n, scale, amax, scale_inv, out, fp8_type, margin, flags, ws, stream);
}

int msamp_cast_scaled_to_fp8(const void* x, int in_dtype, size_t n, const float* amax, const float* old_scale_inv,
                             float* scale, float* scale_inv, float* amax_out, int window, int32_t* counter_out,
                             uint8_t* out, int fp8_type, int margin, msamp_stream_t stream) {
    MSAMP_REQUIRE(is_fp8(fp8_type), MSAMP_ERR_DTYPE, "msamp_cast_scaled_to_fp8: fp8_type %d", fp8_type);
    MSAMP_REQUIRE(is_hp(in_dtype), MSAMP_ERR_DTYPE, "msamp_cast_scaled_to_fp8: in_dtype %d", in_dtype);
    MSAMP_REQUIRE(amax && old_scale_inv && scale && scale_inv && ((x && out) || n == 0), MSAMP_ERR_NULL,
                  "msamp_cast_scaled_to_fp8: null pointer");
    MSAMP_REQUIRE(amax_out == nullptr || window >= 1, MSAMP_ERR_SHAPE, "msamp_cast_scaled_to_fp8: window %d", window);
    const InTimeArgs it = {nullptr, scale, nullptr, fp8_max(fp8_type), margin, 0, amax, old_scale_inv, amax_out, window, counter_out};
    return dispatch_cast(x, in_dtype, n, nullptr, nullptr, scale_inv, out, fp8_type, &it, static_cast<hipStream_t>(stream));
}

int msamp_add_to_fp8(uint8_t* q, int fp8_type, size_t n, float* scale, float* scale_inv, float* amax, const void* other,
                     int other_dtype, void* workspace, msamp_stream_t stream) {
    MSAMP_REQUIRE(is_fp8(fp8_type), MSAMP_ERR_DTYPE, "msamp_add_to_fp8: fp8_type %d", fp8_type);
    MSAMP_REQUIRE(is_hp(other_dtype), MSAMP_ERR_DTYPE, "msamp_add_to_fp8: other_dtype %d", other_dtype);
    MSAMP_REQUIRE(scale && scale_inv && amax && ((q && other) || n == 0), MSAMP_ERR_NULL, "msamp_add_to_fp8: null pointer");
    MSAMP_REQUIRE(workspace != nullptr, MSAMP_ERR_WORKSPACE, "msamp_add_to_fp8: workspace required");
    hipStream_t st = static_cast<hipStream_t>(stream);
    uint32_t* ws = static_cast<uint32_t*>(workspace);
    switch (other_dtype) {
        case MSAMP_DT_F32:
            return launch_add_to_fp8(q, fp8_type, static_cast<const float*>(other), n, scale, scale_inv, amax, ws, st);
        case MSAMP_DT_F16:
            return launch_add_to_fp8(q, fp8_type, static_cast<const f16_t*>(other), n, scale, scale_inv, amax, ws, st);
        default:
            return launch_add_to_fp8(q, fp8_type, static_cast<const bf16_t*>(other), n, scale, scale_inv, amax, ws, st);
    }
}

int msamp_cast_from_fp8(const uint8_t* q, int fp8_type, size_t n, const float* scale_inv, void* out, int out_dtype,
                        msamp_stream_t stream) {
    MSAMP_REQUIRE(is_fp8(fp8_type), MSAMP_ERR_DTYPE, "msamp_cast_from_fp8: fp8_type %d", fp8_type);
    MSAMP_REQUIRE(is_hp(out_dtype), MSAMP_ERR_DTYPE, "msamp_cast_from_fp8: out_dtype %d", out_dtype);
    MSAMP_REQUIRE(scale_inv && ((q && out) || n == 0), MSAMP_ERR_NULL, "msamp_cast_from_fp8: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int ept = 16 / hp_size(out_dtype);
    const int vec_ok = aligned(out, 16) && aligned(q, ept);
    const int grid = grid_for(n, static_cast<size_t>(kCastThreads) * ept * 4);
#define LAUNCH(FMT, OT) \
    hipLaunchKernelGGL((cast_from_fp8_kernel<FMT, OT>), dim3(grid), dim3(kCastThreads), 0, st, q, static_cast<OT*>(out), n, scale_inv, vec_ok)
    if (fp8_type == MSAMP_DT_E4M3) {
        if (out_dtype == MSAMP_DT_F32) LAUNCH(MSAMP_DT_E4M3, float);
        else if (out_dtype == MSAMP_DT_F16) LAUNCH(MSAMP_DT_E4M3, f16_t);
        else LAUNCH(MSAMP_DT_E4M3, bf16_t);
    } else {
        if (out_dtype == MSAMP_DT_F32) LAUNCH(MSAMP_DT_E5M2, float);
        else if (out_dtype == MSAMP_DT_F16) LAUNCH(MSAMP_DT_E5M2, f16_t);
        else LAUNCH(MSAMP_DT_E5M2, bf16_t);
    }
#undef LAUNCH
    MSAMP_CHECK_LAUNCH("cast_from_fp8_kernel");
    return MSAMP_OK;
}

int msamp_cast_transpose(const void* x, int in_dtype, int rows, int cols, const float* scale, float* amax,
                         float* scale_inv, uint8_t* out, uint8_t* out_t, int fp8_type, msamp_stream_t stream) {
    MSAMP_REQUIRE(is_fp8(fp8_type), MSAMP_ERR_DTYPE, "msamp_cast_transpose: fp8_type %d", fp8_type);
    MSAMP_REQUIRE(is_hp(in_dtype), MSAMP_ERR_DTYPE, "msamp_cast_transpose: in_dtype %d", in_dtype);
    MSAMP_REQUIRE(rows >= 0 && cols >= 0, MSAMP_ERR_SHAPE, "msamp_cast_transpose: shape %d x %d", rows, cols);
    if (rows == 0 || cols == 0) return MSAMP_OK;
    MSAMP_REQUIRE(x && scale && out_t, MSAMP_ERR_NULL, "msamp_cast_transpose: null pointer");
    return dispatch_ct(x, in_dtype, rows, cols, scale, amax, scale_inv, out, out_t, fp8_type, static_cast<hipStream_t>(stream));
}

int msamp_cast_transpose_intime(const void* x, int in_dtype, int rows, int cols, float* scale, float* amax,
                                float* scale_inv, uint8_t* out, uint8_t* out_t, int fp8_type, int margin, int flags,
                                void* workspace, msamp_stream_t stream) {
    MSAMP_REQUIRE(is_fp8(fp8_type), MSAMP_ERR_DTYPE, "msamp_cast_transpose_intime: fp8_type %d", fp8_type);
    MSAMP_REQUIRE(is_hp(in_dtype), MSAMP_ERR_DTYPE, "msamp_cast_transpose_intime: in_dtype %d", in_dtype);
    MSAMP_REQUIRE(rows >= 0 && cols >= 0, MSAMP_ERR_SHAPE, "msamp_cast_transpose_intime: shape %d x %d", rows, cols);
    MSAMP_REQUIRE(scale && amax && scale_inv, MSAMP_ERR_NULL, "msamp_cast_transpose_intime: null meta pointer");
    MSAMP_REQUIRE(workspace != nullptr, MSAMP_ERR_WORKSPACE, "msamp_cast_transpose_intime: workspace required");
    MSAMP_REQUIRE((x && out_t) || rows == 0 || cols == 0, MSAMP_ERR_NULL, "msamp_cast_transpose_intime: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t n = static_cast<size_t>(rows) * cols;
    int rc = dispatch_amax(x, in_dtype, n, workspace, scale, st);
    if (rc != MSAMP_OK) return rc;
    rc = finalize_amax(workspace, amax, scale, scale_inv, fp8_max(fp8_type), margin, flags, 1, st);
    if (rc != MSAMP_OK || n == 0) return rc;
    return dispatch_ct(x, in_dtype, rows, cols, scale, nullptr, nullptr, out, out_t, fp8_type, st);
}

int msamp_cast_to_fp8_gated(const void* x, int in_dtype, size_t n, float* scale, float* amax, float* scale_inv,
                            uint8_t* out, int fp8_type, int margin, int flags, const int32_t* warmup_counter, int window,
                            void* workspace, msamp_stream_t stream) {
    MSAMP_REQUIRE(is_fp8(fp8_type), MSAMP_ERR_DTYPE, "msamp_cast_to_fp8_gated: fp8_type %d", fp8_type);
    MSAMP_REQUIRE(is_hp(in_dtype), MSAMP_ERR_DTYPE, "msamp_cast_to_fp8_gated: in_dtype %d", in_dtype);
    MSAMP_REQUIRE(scale && amax && scale_inv && warmup_counter && ((x && out) || n == 0), MSAMP_ERR_NULL,
                  "msamp_cast_to_fp8_gated: null pointer");
    MSAMP_REQUIRE(workspace != nullptr, MSAMP_ERR_WORKSPACE, "msamp_cast_to_fp8_gated: workspace required");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const Gate gate = {warmup_counter, window};
    // while warming up: amax[0] and the scale from this tensor; afterwards both kernels return at once
    const Finish fin = {amax, scale, scale_inv, fp8_max(fp8_type), margin, flags};
    int rc = dispatch_amax(x, in_dtype, n, workspace, scale, st, gate, fin);
    if (rc != MSAMP_OK) return rc;
    // the delayed cast serves both cases: folding max|x| into an amax[0] that already holds it changes nothing
    return dispatch_cast(x, in_dtype, n, scale, amax, scale_inv, out, fp8_type, nullptr, st);
}

int msamp_cast_transpose_gated(const void* x, int in_dtype, int rows, int cols, float* scale, float* amax,
                               float* scale_inv, uint8_t* out, uint8_t* out_t, int fp8_type, int margin, int flags,
                               const int32_t* warmup_counter, int window, void* workspace, msamp_stream_t stream) {
    MSAMP_REQUIRE(is_fp8(fp8_type), MSAMP_ERR_DTYPE, "msamp_cast_transpose_gated: fp8_type %d", fp8_type);
    MSAMP_REQUIRE(is_hp(in_dtype), MSAMP_ERR_DTYPE, "msamp_cast_transpose_gated: in_dtype %d", in_dtype);
    MSAMP_REQUIRE(rows >= 0 && cols >= 0, MSAMP_ERR_SHAPE, "msamp_cast_transpose_gated: shape %d x %d", rows, cols);
    MSAMP_REQUIRE(scale && amax && scale_inv && warmup_counter, MSAMP_ERR_NULL, "msamp_cast_transpose_gated: null meta pointer");
    MSAMP_REQUIRE(workspace != nullptr, MSAMP_ERR_WORKSPACE, "msamp_cast_transpose_gated: workspace required");
    MSAMP_REQUIRE((x && out_t) || rows == 0 || cols == 0, MSAMP_ERR_NULL, "msamp_cast_transpose_gated: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t n = static_cast<size_t>(rows) * cols;
    const Gate gate = {warmup_counter, window};
    const Finish fin = {amax, scale, scale_inv, fp8_max(fp8_type), margin, flags};
    int rc = dispatch_amax(x, in_dtype, n, workspace, scale, st, gate, fin);
    if (rc != MSAMP_OK || n == 0) return rc;
    return dispatch_ct(x, in_dtype, rows, cols, scale, amax, scale_inv, out, out_t, fp8_type, st);
}

int msamp_fp8_transpose(const uint8_t* q, int rows, int cols, uint8_t* out, msamp_stream_t stream) {
    MSAMP_REQUIRE(rows >= 0 && cols >= 0, MSAMP_ERR_SHAPE, "msamp_fp8_transpose: shape %d x %d", rows, cols);
    if (rows == 0 || cols == 0) return MSAMP_OK;
    MSAMP_REQUIRE(q && out, MSAMP_ERR_NULL, "msamp_fp8_transpose: null pointer");
    if (rows % 16 == 0 && cols % 16 == 0 && aligned(q, 16) && aligned(out, 16) && (rows + 127) / 128 <= 65535) {
        hipLaunchKernelGGL(byte_transpose128_kernel, dim3((cols + 127) / 128, (rows + 127) / 128), dim3(kCastThreads), 0,
                           static_cast<hipStream_t>(stream), q, out, rows, cols);
        MSAMP_CHECK_LAUNCH("byte_transpose128_kernel");
        return MSAMP_OK;
    }
    return launch_ct<uint8_t, false>(q, rows, cols, nullptr, nullptr, nullptr, nullptr, out, MSAMP_DT_E4M3,
                                     static_cast<hipStream_t>(stream));
}

int msamp_scale_cast(const void* x, int in_dtype, size_t n, const float* scale, void* out, int out_dtype,
                     msamp_stream_t stream) {
    MSAMP_REQUIRE(is_hp(in_dtype) && is_hp(out_dtype), MSAMP_ERR_DTYPE, "msamp_scale_cast: dtypes %d -> %d", in_dtype, out_dtype);
    MSAMP_REQUIRE(scale && ((x && out) || n == 0), MSAMP_ERR_NULL, "msamp_scale_cast: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (n == 0) return MSAMP_OK;
    switch (in_dtype) {
        case MSAMP_DT_F32:
            return launch_scale_cast_out(static_cast<const float*>(x), n, scale, out, out_dtype, st);
        case MSAMP_DT_F16:
            return launch_scale_cast_out(static_cast<const f16_t*>(x), n, scale, out, out_dtype, st);
        default:
            return launch_scale_cast_out(static_cast<const bf16_t*>(x), n, scale, out, out_dtype, st);
    }
}

int msamp_scale_update(float* scales, float* amaxs, uint8_t* bad, int32_t* counters, int n, int window, float fp_max,
                       int margin, msamp_stream_t stream) {
    MSAMP_REQUIRE(n >= 0 && window >= 1, MSAMP_ERR_SHAPE, "msamp_scale_update: n=%d window=%d", n, window);
    if (n == 0) return MSAMP_OK;
    MSAMP_REQUIRE(scales && amaxs, MSAMP_ERR_NULL, "msamp_scale_update: null pointer");
    if (window <= 64) {
        hipLaunchKernelGGL(scale_update_kernel, dim3((n + 3) / 4), dim3(256), 0, static_cast<hipStream_t>(stream), scales,
                           amaxs, bad, counters, n, window, fp_max, margin);
    } else {
        hipLaunchKernelGGL(scale_update_wide_kernel, dim3((n + 63) / 64), dim3(64), 0, static_cast<hipStream_t>(stream),
                           scales, amaxs, bad, counters, n, window, fp_max, margin);
    }
    MSAMP_CHECK_LAUNCH("scale_update_kernel");
    return MSAMP_OK;
}

int msamp_scale_update_groups(const msamp_scale_group* groups, int n_groups, int margin, msamp_stream_t stream) {
    MSAMP_REQUIRE(n_groups >= 0 && n_groups <= MSAMP_MAX_SCALE_GROUPS, MSAMP_ERR_SHAPE,
                  "msamp_scale_update_groups: n_groups=%d (at most %d)", n_groups, MSAMP_MAX_SCALE_GROUPS);
    if (n_groups == 0) return MSAMP_OK;
    MSAMP_REQUIRE(groups, MSAMP_ERR_NULL, "msamp_scale_update_groups: null pointer");
    ScaleGroups packed = {};
    int n_max = 0, used = 0;
    bool narrow = true;
    for (int k = 0; k < n_groups; ++k) {
        const msamp_scale_group& g = groups[k];
        MSAMP_REQUIRE(g.n >= 0 && g.window >= 1, MSAMP_ERR_SHAPE, "msamp_scale_update_groups: group %d: n=%d window=%d", k,
                      g.n, g.window);
        if (g.n == 0) continue;
        MSAMP_REQUIRE(g.scales && g.amaxs, MSAMP_ERR_NULL, "msamp_scale_update_groups: group %d: null pointer", k);
        narrow = narrow && g.window <= 64;
        n_max = g.n > n_max ? g.n : n_max;
        packed.g[used++] = g;
    }
    if (used == 0) return MSAMP_OK;
    if (!narrow) {    // a window wider than a wavefront: group by group through the single-group entry point
        for (int k = 0; k < used; ++k) {
            const msamp_scale_group& g = packed.g[k];
            const int rc = msamp_scale_update(g.scales, g.amaxs, g.bad, g.counters, g.n, g.window, g.fp_max, margin, stream);
            if (rc != MSAMP_OK) return rc;
        }
        return MSAMP_OK;
    }
    hipLaunchKernelGGL(scale_update_groups_kernel, dim3((n_max + 3) / 4, used), dim3(256), 0, static_cast<hipStream_t>(stream),
                       packed, margin);
    MSAMP_CHECK_LAUNCH("scale_update_groups_kernel");
    return MSAMP_OK;
}

}    // extern "C"
