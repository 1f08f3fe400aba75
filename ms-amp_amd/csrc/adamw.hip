// FP8 AdamW: the reference-shaped stage-1 / stage-2 entry points on fp32 param/grad, and the fused
// multi-tensor step that works on the quantized tensors directly (5 bytes read, 4 written per
// parameter).  Arithmetic is plain float32, left to right, never contracted into fused
// multiply-adds, so the second pass reproduces the first one bit for bit.
#include "common.cuh"

#include <type_traits>

#include <cmath>
#include <limits>

namespace msamp {

constexpr int kAdamThreads = 256;

struct AdamConsts {
    float beta1, beta2, omb1, omb2, eps, step_size, sbc2, inv_sbc2, decay, wd;
    float bound_rsq, bound_eps;    // first pass: |update| <= step_size * |m'| * min(bound_rsq * rsq(v'), bound_eps)
    int adam_mode, maximize, use_decay;
    int rule_scales;    // the moments' scales follow the scale rule (tensor_scale): what the clamp-free fast path needs
};

// float step_size and sqrt(bias_correction2) from float betas and a double pow, then narrowed
static void host_consts(float lr, float beta1, float beta2, int step, int bias_correction, float* step_size,
                        float* sbc2) {
    float bc1 = bias_correction ? static_cast<float>(1.0 - pow(static_cast<double>(beta1), step)) : 1.0f;
    float bc2 = bias_correction ? static_cast<float>(1.0 - pow(static_cast<double>(beta2), step)) : 1.0f;
    *step_size = lr / bc1;
    *sbc2 = sqrtf(bc2);
}

// m' and v' from the stored moments (already widened to float)
__device__ __forceinline__ void moments(float mf, float vf, float g, float inv_m, float inv_v, const AdamConsts& k,
                                        float& m_new, float& v_new) {
#pragma clang fp contract(off)
    const float t1 = k.beta1 * mf;
    const float t2 = t1 * inv_m;
    const float t3 = k.omb1 * g;
    m_new = t2 + t3;
    const float u1 = k.beta2 * vf;
    const float u2 = u1 * inv_v;
    const float gg = g * g;
    const float u3 = k.omb2 * gg;
    v_new = u2 + u3;
}

__device__ __forceinline__ float param_update(float p, float m_new, float v_new, const AdamConsts& k) {
#pragma clang fp contract(off)
    const float root = sqrtf(v_new);
    const float q = root / k.sbc2;
    const float denom = q + k.eps;
    const float r = m_new / denom;
    const float d = k.step_size * r;
    return p - d;
}

// ---- generic moment storage for the single-tensor entry points ---------------------------------
template <int DT>
struct State;
template <>
struct State<MSAMP_DT_E4M3> {
    typedef uint8_t T;
    static __device__ __forceinline__ float load(const T* p, size_t i) { return dequant1<MSAMP_DT_E4M3>(p[i]); }
    static __device__ __forceinline__ void store(T* p, size_t i, float v) {
        p[i] = static_cast<uint8_t>(quant1<MSAMP_DT_E4M3>(v));
    }
};
template <>
struct State<MSAMP_DT_E5M2> {
    typedef uint8_t T;
    static __device__ __forceinline__ float load(const T* p, size_t i) { return dequant1<MSAMP_DT_E5M2>(p[i]); }
    static __device__ __forceinline__ void store(T* p, size_t i, float v) {
        p[i] = static_cast<uint8_t>(quant1<MSAMP_DT_E5M2>(v));
    }
};
template <>
struct State<MSAMP_DT_F16> {
    typedef uint16_t T;
    static __device__ __forceinline__ float load(const T* p, size_t i) { return f16_bits_to_float(p[i]); }
    static __device__ __forceinline__ void store(T* p, size_t i, float v) {
        p[i] = static_cast<uint16_t>(float_to_f16_bits(v));
    }
};
template <>
struct State<MSAMP_DT_F32> {
    typedef float T;
    static __device__ __forceinline__ float load(const T* p, size_t i) { return p[i]; }
    static __device__ __forceinline__ void store(T* p, size_t i, float v) { p[i] = v; }
};

template <int MDT, int VDT>
__global__ __launch_bounds__(kAdamThreads) void stage1_kernel(float* __restrict__ param, const float* __restrict__ grad,
                                                               size_t n, const typename State<MDT>::T* __restrict__ m,
                                                               float inv_m, float* m_amax,
                                                               const typename State<VDT>::T* __restrict__ v,
                                                               float inv_v, float* v_amax, AdamConsts k) {
    __shared__ uint32_t red[kAdamThreads / kWave];
    float mxm = 0.0f, mxv = 0.0f;
    const size_t stride = static_cast<size_t>(gridDim.x) * kAdamThreads;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kAdamThreads + threadIdx.x; i < n; i += stride) {
        float m_new, v_new;
        moments(State<MDT>::load(m, i), State<VDT>::load(v, i), grad[i], inv_m, inv_v, k, m_new, v_new);
        mxm = fmaxf(mxm, fabsf(m_new));
        mxv = fmaxf(mxv, fabsf(v_new));
        param[i] = param_update(param[i], m_new, v_new, k);
    }
    uint32_t a = block_max_u32(__float_as_uint(mxm), red);
    uint32_t b = block_max_u32(__float_as_uint(mxv), red);
    if (threadIdx.x == 0) {
        atomicMax(reinterpret_cast<int*>(m_amax), static_cast<int>(a));
        atomicMax(reinterpret_cast<int*>(v_amax), static_cast<int>(b));
    }
}

template <int MDT, int VDT>
__global__ __launch_bounds__(kAdamThreads) void stage2_kernel(const float* __restrict__ grad, size_t n,
                                                               typename State<MDT>::T* __restrict__ m, float inv_m,
                                                               float new_m, typename State<VDT>::T* __restrict__ v,
                                                               float inv_v, float new_v, AdamConsts k) {
    const size_t stride = static_cast<size_t>(gridDim.x) * kAdamThreads;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kAdamThreads + threadIdx.x; i < n; i += stride) {
        float m_new, v_new;
        moments(State<MDT>::load(m, i), State<VDT>::load(v, i), grad[i], inv_m, inv_v, k, m_new, v_new);
        State<MDT>::store(m, i, m_new * new_m);
        State<VDT>::store(v, i, v_new * new_v);
    }
}

// ---- fused multi-tensor step -------------------------------------------------------------------
constexpr int kEPT = 16;                                   // elements per thread per step
constexpr int kSteps = MSAMP_ADAMW_CHUNK / (kAdamThreads * kEPT);    // 4

template <int WDT>
__device__ __forceinline__ void load_w16(const void* base, size_t i, float* f) {
    if constexpr (WDT == MSAMP_DT_F16) {
        const uint4* p = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(base) + i);
        uint4 a = p[0], b = p[1];
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            f[2 * j] = f16_bits_to_float(w[j] & 0xffffu);
            f[2 * j + 1] = f16_bits_to_float(w[j] >> 16);
        }
    } else {
        uint4 a = *reinterpret_cast<const uint4*>(static_cast<const uint8_t*>(base) + i);
        dequant4<WDT>(a.x, f[0], f[1], f[2], f[3]);
        dequant4<WDT>(a.y, f[4], f[5], f[6], f[7]);
        dequant4<WDT>(a.z, f[8], f[9], f[10], f[11]);
        dequant4<WDT>(a.w, f[12], f[13], f[14], f[15]);
    }
}

template <int WDT>
__device__ __forceinline__ float load_w1(const void* base, size_t i) {
    if constexpr (WDT == MSAMP_DT_F16) {
        return f16_bits_to_float(static_cast<const uint16_t*>(base)[i]);
    } else {
        return dequant1<WDT>(static_cast<const uint8_t*>(base)[i]);
    }
}

// ---- element-wise pieces shared by both passes ------------------------------------------------
// Exact part: dequantized weight (decayed), gradient (negated / with the Adam-mode L2 term) and the
// new moments, all as the reference evaluates them.  Two uniform choices are folded into factors, which
// changes no bit: `g_si` arrives negated when the step maximizes (negation commutes with rounding), and
// `k.decay` is 1 when no decoupled decay applies.  L2 (Adam mode with a non-zero weight decay) is a
// template parameter: it adds the decay term to the gradient instead.
template <bool L2>
__device__ __forceinline__ void prepare(float w_raw, float g_raw, float m_old, float v_old, float w_si, float g_si,
                                        float inv_m, float inv_v, const AdamConsts& k, float& pj, float& g_plain,
                                        float& m_new, float& v_new) {
#pragma clang fp contract(off)
    pj = w_raw * w_si;
    float gj = g_raw * g_si;
    g_plain = gj;
    if constexpr (L2) {
        const float t = k.wd * pj;
        gj = gj + t;
    } else {
        pj = pj * k.decay;
    }
    moments(m_old, v_old, gj, inv_m, inv_v, k, m_new, v_new);
}

// Cheap estimate of p' = p - step * m' / (sqrt(v') / sbc2 + eps) with the hardware's 1-ulp sqrt and
// reciprocal, and a bound on its distance from the exactly rounded chain of param_update():
// the update term is off by at most 13 unit roundoffs, the subtraction adds one rounding on each side.
// Non-finite inputs make the bound NaN, which every caller treats as "take the exact path".
// `eps_v` is k.eps held in a vector register (an instruction takes one scalar operand only: with eps in a scalar
// register next to inv_sbc2 every element would pay for a move).
__device__ __forceinline__ void estimate(float pj, float m_new, float v_new, const AdamConsts& k, float eps_v, float& p_est,
                                         float& err) {
    const float root = __builtin_amdgcn_sqrtf(v_new);
    const float den = fmaf(root, k.inv_sbc2, eps_v);
    const float r = m_new * __builtin_amdgcn_rcpf(den);
    const float d = k.step_size * r;
    p_est = pj - d;
    err = fmaf(1.0e-6f, fabsf(d), 2.0e-7f * fabsf(p_est));
}

template <int WDT, int GDT>
__device__ __forceinline__ void load16(const msamp_adamw_tensor& d, size_t i, float* p, float* g, float* m,
                                       float* v) {
    load_w16<WDT>(d.weight, i, p);
    load_w16<GDT>(d.grad, i, g);
    load_w16<MSAMP_DT_E4M3>(d.exp_avg, i, m);
    load_w16<MSAMP_DT_F16>(d.exp_avg_sq, i, v);
}

// One lane's 16 elements of the first pass (p, g, m, v hold the dequantized stored values on entry).
// Only bounds on |p'| are needed here: |p| - D <= |p'| <= |p| + D with D >= |step * m' / (sqrt(v') / sbc2 + eps)|,
// and since eps >= 0 the quotient is at most sbc2 / sqrt(v') and at most 1 / eps.  k.bound_rsq and k.bound_eps hold
// |step| times those two factors, widened by 4e-6 for the roundings of both chains (the exact one has six, the
// hardware reciprocal square root is good to one ulp).  A NaN or negative v' keeps its NaN through the selection.
template <bool L2>
__device__ __forceinline__ void amax_step(float* p, const float* g, float* m, float* v, float w_si, float g_si, float inv_m,
                                          float inv_v, const AdamConsts& k, float& floor_p, uint32_t& mxp, float& mxm,
                                          float& mxv) {
    float hi[kEPT];
    float lo_max = 0.0f;
#pragma unroll
    for (int j = 0; j < kEPT; ++j) {
        float pj, g_plain, m_new, v_new;
        prepare<L2>(p[j], g[j], m[j], v[j], w_si, g_si, inv_m, inv_v, k, pj, g_plain, m_new, v_new);
        const float t = k.bound_rsq * __builtin_amdgcn_rsqf(v_new);
        const float lim = k.bound_eps < t ? k.bound_eps : t;
        const float dmax = fabsf(m_new) * lim;
        mxm = fmaxf(mxm, fabsf(m_new));
        mxv = fmaxf(mxv, fabsf(v_new));
        p[j] = pj, m[j] = m_new, v[j] = v_new;
        hi[j] = fabsf(pj) + dmax;
        lo_max = fmaxf(lo_max, fabsf(pj) - dmax);    // NaN bounds are skipped here, caught below
    }
    floor_p = fmaxf(floor_p, __uint_as_float(wave_max_u32(__float_as_uint(lo_max))));
    // the additions above and the last subtraction of the exact chain round once each: leave room for them
    const float skip_below = floor_p * 0.999999f;
#pragma unroll
    for (int j = 0; j < kEPT; ++j) {
        if (!(hi[j] < skip_below)) {
            const uint32_t ab = __float_as_uint(param_update(p[j], m[j], v[j], k)) & 0x7fffffffu;
            mxp = ab > mxp ? ab : mxp;
        }
    }
}

// First pass: exact max |m'| and |v'| (they are cheap), and the exact max |p'| found by bounding:
// every element gets cheap bounds; only elements whose upper bound reaches the best lower bound
// seen so far (by this wavefront, or already published for the tensor) are evaluated exactly.  The
// element that attains the true maximum always passes that test, so the result is the exact maximum.
template <int WDT, int GDT, bool L2>
__global__ __launch_bounds__(kAdamThreads) void fused_amax_kernel(msamp_adamw_tensor* __restrict__ tensors,
                                                                   const int32_t* __restrict__ block_map,
                                                                   AdamConsts k) {
    __shared__ uint32_t red[kAdamThreads / kWave];
    const int t = block_map[2 * blockIdx.x], chunk = block_map[2 * blockIdx.x + 1];
    msamp_adamw_tensor& d = tensors[t];
    const size_t n = d.numel;
    const size_t base = static_cast<size_t>(chunk) * MSAMP_ADAMW_CHUNK;
    const float w_si = *d.w_scale_inv, g_si = k.maximize ? -*d.g_scale_inv : *d.g_scale_inv;
    const float inv_m = 1.0f / *d.m_scale, inv_v = 1.0f / *d.v_scale;
    uint32_t mxp = 0;    // exact |p'| bit patterns of the candidates (NaN patterns compare highest)
    float mxm = 0.0f, mxv = 0.0f;
    // lower bound on the tensor's max |p'|: what other workgroups have published so far
    float floor_p = __uint_as_float(__hip_atomic_load(&d.acc[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    if (!(floor_p >= 0.0f)) floor_p = 0.0f;    // a NaN already published: everything is exact from here on
    if (base + MSAMP_ADAMW_CHUNK <= n) {
#pragma unroll 1
        for (int s = 0; s < kSteps; ++s) {
            const size_t i = base + (static_cast<size_t>(s) * kAdamThreads + threadIdx.x) * kEPT;
            float p[kEPT], g[kEPT], m[kEPT], v[kEPT];
            load16<WDT, GDT>(d, i, p, g, m, v);
            amax_step<L2>(p, g, m, v, w_si, g_si, inv_m, inv_v, k, floor_p, mxp, mxm, mxv);
        }
    } else {
        for (size_t i = base + threadIdx.x; i < n; i += kAdamThreads) {
            float pj, g_plain, m_new, v_new;
            prepare<L2>(load_w1<WDT>(d.weight, i), load_w1<GDT>(d.grad, i), load_w1<MSAMP_DT_E4M3>(d.exp_avg, i),
                    load_w1<MSAMP_DT_F16>(d.exp_avg_sq, i), w_si, g_si, inv_m, inv_v, k, pj, g_plain, m_new, v_new);
            const uint32_t ab = __float_as_uint(param_update(pj, m_new, v_new, k)) & 0x7fffffffu;
            mxp = ab > mxp ? ab : mxp;
            mxm = fmaxf(mxm, fabsf(m_new));
            mxv = fmaxf(mxv, fabsf(v_new));
        }
    }
    const uint32_t a = block_max_u32(mxp, red);
    const uint32_t b = block_max_u32(__float_as_uint(mxm), red);
    const uint32_t c = block_max_u32(__float_as_uint(mxv), red);
    if (threadIdx.x == 0) {
        if (a) atomicMax(&d.acc[0], a);
        if (b) atomicMax(&d.acc[1], b);
        if (c) atomicMax(&d.acc[2], c);
    }
}

__global__ void fused_scales_kernel(msamp_adamw_tensor* tensors, int n_tensors, float w_fp_max, int tensor_scale,
                                    int32_t* redo) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;    // `tensors` is pre-offset to the group's first tensor
    if (t >= n_tensors) return;
    msamp_adamw_tensor& d = tensors[t];
    const float ap = __uint_as_float(d.acc[0]), am = __uint_as_float(d.acc[1]), av = __uint_as_float(d.acc[2]);
    d.acc[0] = 0u, d.acc[1] = 0u, d.acc[2] = 0u;
    d.saved[0] = *d.w_scale_inv;
    d.saved[1] = 1.0f / *d.m_scale;
    d.saved[2] = 1.0f / *d.v_scale;
    const float ws = scale_rule(ap, *d.w_scale, w_fp_max, 0);
    const float ms = tensor_scale ? scale_rule(am, 1.0f, 448.0f, 0) : 1.0f;
    const float vs = tensor_scale ? scale_rule(av, 1.0f, 65504.0f, 0) : 1.0f;
    // after the speculative pass (which used the scales as they were): is any of them different now?
    if (redo != nullptr)
        redo[t] = (__float_as_uint(ws) != __float_as_uint(*d.w_scale) || __float_as_uint(ms) != __float_as_uint(*d.m_scale) ||
                   __float_as_uint(vs) != __float_as_uint(*d.v_scale))
                      ? 1
                      : 0;
    *d.w_scale = ws;
    *d.w_scale_inv = 1.0f / ws;
    *d.w_amax = ap;
    *d.m_scale = ms;
    *d.m_scale_inv = 1.0f / ms;
    *d.m_amax = am;
    *d.v_scale = vs;
    *d.v_scale_inv = 1.0f / vs;
    *d.v_amax = av;
}

template <int WDT>
__device__ __forceinline__ void store_w16(void* base, size_t i, const float* f) {
    if constexpr (WDT == MSAMP_DT_F16) {
        uint32_t w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = float_to_f16_bits(f[2 * j]) | (float_to_f16_bits(f[2 * j + 1]) << 16);
        uint4* p = reinterpret_cast<uint4*>(static_cast<uint16_t*>(base) + i);
        p[0] = make_uint4(w[0], w[1], w[2], w[3]);
        p[1] = make_uint4(w[4], w[5], w[6], w[7]);
    } else {
        uint4 o;
        o.x = quant4<WDT>(f[0], f[1], f[2], f[3]);
        o.y = quant4<WDT>(f[4], f[5], f[6], f[7]);
        o.z = quant4<WDT>(f[8], f[9], f[10], f[11]);
        o.w = quant4<WDT>(f[12], f[13], f[14], f[15]);
        *reinterpret_cast<uint4*>(static_cast<uint8_t*>(base) + i) = o;
    }
}

template <int WDT>
__device__ __forceinline__ void store_w1(void* base, size_t i, float f) {
    if constexpr (WDT == MSAMP_DT_F16) {
        static_cast<uint16_t*>(base)[i] = static_cast<uint16_t>(float_to_f16_bits(f));
    } else {
        static_cast<uint8_t*>(base)[i] = static_cast<uint8_t>(quant1<WDT>(f));
    }
}

// weight payload of one element from the exact p' (slow path of the second pass)
template <int WDT>
__device__ __forceinline__ uint32_t quant_weight_exact(float pj, float m_new, float v_new, float ws, const AdamConsts& k) {
    const float pe = param_update(pj, m_new, v_new, k) * ws;
    if constexpr (WDT == MSAMP_DT_F16) {
        return float_to_f16_bits(pe);
    } else {
        return quant1<WDT>(pe);
    }
}

// One lane's 16 elements of the second pass: requantized weight, exp_avg and exp_avg_sq are stored at element i.
template <int WDT, bool L2>
__device__ __forceinline__ void write_step(void* w_out, uint8_t* m_out, uint16_t* v_out, size_t i, float* p, const float* g,
                                           float* m, float* v, float w_si, float g_si, float inv_m, float inv_v, float ws,
                                           float ms, float vs, const AdamConsts& k) {
    uint32_t wq[kEPT];
    float eps_v = k.eps;
    asm volatile("" : "+v"(eps_v));
#pragma unroll
    for (int j = 0; j < kEPT; ++j) {
        float pj, g_plain, m_new, v_new, p_est, err;
        prepare<L2>(p[j], g[j], m[j], v[j], w_si, g_si, inv_m, inv_v, k, pj, g_plain, m_new, v_new);
        estimate(pj, m_new, v_new, k, eps_v, p_est, err);
        const float lo = (p_est - err) * ws, hi = (p_est + err) * ws;
        bool same;
        uint32_t code;
        if constexpr (WDT == MSAMP_DT_F16) {
            code = float_to_f16_bits(lo);
            same = code == float_to_f16_bits(hi);
        } else {
            const uint32_t two = cvt_pk<WDT>(sat<WDT>(lo), sat<WDT>(hi), 0u, false);
            code = two & 0xffu;
            same = code == ((two >> 8) & 0xffu);
        }
        if (!(same && err < __uint_as_float(0x7f800000u))) code = quant_weight_exact<WDT>(pj, m_new, v_new, ws, k);
        wq[j] = code;
        if constexpr (L2) moments(m[j], v[j], g_plain, inv_m, inv_v, k, m_new, v_new);    // stored moments ignore the L2 term
        m[j] = m_new * ms;
        v[j] = v_new * vs;
    }
    if constexpr (WDT == MSAMP_DT_F16) {
        uint4* o = reinterpret_cast<uint4*>(static_cast<uint16_t*>(w_out) + i);
        o[0] = make_uint4(wq[0] | (wq[1] << 16), wq[2] | (wq[3] << 16), wq[4] | (wq[5] << 16), wq[6] | (wq[7] << 16));
        o[1] = make_uint4(wq[8] | (wq[9] << 16), wq[10] | (wq[11] << 16), wq[12] | (wq[13] << 16), wq[14] | (wq[15] << 16));
    } else {
        uint4 o;
        o.x = wq[0] | (wq[1] << 8) | (wq[2] << 16) | (wq[3] << 24);
        o.y = wq[4] | (wq[5] << 8) | (wq[6] << 16) | (wq[7] << 24);
        o.z = wq[8] | (wq[9] << 8) | (wq[10] << 16) | (wq[11] << 24);
        o.w = wq[12] | (wq[13] << 8) | (wq[14] << 16) | (wq[15] << 24);
        *reinterpret_cast<uint4*>(static_cast<uint8_t*>(w_out) + i) = o;
    }
    store_w16<MSAMP_DT_E4M3>(m_out, i, m);
    store_w16<MSAMP_DT_F16>(v_out, i, v);
}

// Second pass: recompute m', v' exactly and requantize them; for the weight, quantize both ends of the
// estimate's error interval -- when they give the same code (rounding is monotonic) that code is the
// exact answer, otherwise (or for anything non-finite) the element takes the exact chain.
// One chunk of the second pass: the tensor's inputs at d.weight / d.grad / d.exp_avg / d.exp_avg_sq, requantized with
// the given scales into w_out / m_out / v_out (which may be the inputs' own places).
template <int WDT, int GDT, bool L2>
__device__ __forceinline__ void write_chunk(const msamp_adamw_tensor& d, int chunk, void* w_out, uint8_t* m_out, uint16_t* v_out,
                                            float w_si, float g_si, float inv_m, float inv_v, float ws, float ms, float vs,
                                            const AdamConsts& k) {
    const size_t n = d.numel;
    const size_t base = static_cast<size_t>(chunk) * MSAMP_ADAMW_CHUNK;
    if (base + MSAMP_ADAMW_CHUNK <= n) {
#pragma unroll 1
        for (int s = 0; s < kSteps; ++s) {
            const size_t i = base + (static_cast<size_t>(s) * kAdamThreads + threadIdx.x) * kEPT;
            float p[kEPT], g[kEPT], m[kEPT], v[kEPT];
            load16<WDT, GDT>(d, i, p, g, m, v);
            write_step<WDT, L2>(w_out, m_out, v_out, i, p, g, m, v, w_si, g_si, inv_m, inv_v, ws, ms, vs, k);
        }
    } else {
        for (size_t i = base + threadIdx.x; i < n; i += kAdamThreads) {
            const float m_old = load_w1<MSAMP_DT_E4M3>(d.exp_avg, i), v_old = load_w1<MSAMP_DT_F16>(d.exp_avg_sq, i);
            float pj, g_plain, m_new, v_new;
            prepare<L2>(load_w1<WDT>(d.weight, i), load_w1<GDT>(d.grad, i), m_old, v_old, w_si, g_si, inv_m, inv_v, k, pj,
                    g_plain, m_new, v_new);
            store_w1<WDT>(w_out, i, param_update(pj, m_new, v_new, k) * ws);
            if constexpr (L2) moments(m_old, v_old, g_plain, inv_m, inv_v, k, m_new, v_new);
            store_w1<MSAMP_DT_E4M3>(m_out, i, m_new * ms);
            store_w1<MSAMP_DT_F16>(v_out, i, v_new * vs);
        }
    }
}

// Second pass: recompute m', v' exactly and requantize them; for the weight, quantize both ends of the
// estimate's error interval -- when they give the same code (rounding is monotonic) that code is the
// exact answer, otherwise (or for anything non-finite) the element takes the exact chain.
template <int WDT, int GDT, bool L2>
__global__ __launch_bounds__(kAdamThreads) void fused_write_kernel(msamp_adamw_tensor* __restrict__ tensors,
                                                                    const int32_t* __restrict__ block_map,
                                                                    AdamConsts k,
                                                                    const msamp_adamw_buffers* __restrict__ outs,
                                                                    const int32_t* __restrict__ redo) {
    const int b = gridDim.x - 1 - blockIdx.x;    // back to front: most recently read chunks first
    const int t = block_map[2 * b], chunk = block_map[2 * b + 1];
    // after the speculative pass: only the tensors whose scales it guessed wrong are done again, from the untouched
    // inputs, into the same output buffers
    if (redo != nullptr && redo[t] == 0) return;
    msamp_adamw_tensor& d = tensors[t];
    void* w_out = outs ? outs[t].weight : d.weight;
    uint8_t* m_out = outs ? outs[t].exp_avg : d.exp_avg;
    uint16_t* v_out = outs ? outs[t].exp_avg_sq : d.exp_avg_sq;
    const float w_si = d.saved[0], g_si = k.maximize ? -*d.g_scale_inv : *d.g_scale_inv, inv_m = d.saved[1], inv_v = d.saved[2];
    const float ws = *d.w_scale, ms = *d.m_scale, vs = *d.v_scale;
    write_chunk<WDT, GDT, L2>(d, chunk, w_out, m_out, v_out, w_si, g_si, inv_m, inv_v, ws, ms, vs, k);
}

// ---- speculative single pass -------------------------------------------------------------------
// The scales of a tensor are powers of two and seldom change from one step to the next.  With separate output
// buffers the step can therefore be taken in ONE pass over the data: quantize p', m', v' with the scales the tensor
// has now, find the three maxima on the way, and let fused_scales_kernel compare the scales the rule gives with the
// ones used.  Where they agree the output is what the two passes above produce, bit for bit; a tensor where they do
// not is done again by fused_write_kernel from its inputs, which this pass does not touch.
//
// A lane works on eight consecutive elements at a time (one 8-byte load each of weight, gradient and exp_avg codes,
// one 16-byte load of exp_avg_sq; 2-byte weights: 16 bytes), two such groups per step, 2048 elements apart, so that
// every load and store instruction of a wavefront covers one contiguous run of whole cache lines.  |m'| and |v'| are
// exact.  For |p'| the estimate gives |p_est| - err <= |p'| <= |p_est| + err; only elements whose upper end reaches the
// best lower end seen so far are evaluated exactly, and the element that attains the maximum always is.  Elements that
// took the exact chain for their code (an estimate too close to a rounding boundary, anything non-finite) have their
// exact |p'| already.
constexpr int kGroup = 8;                                              // elements per lane and group
constexpr int kGroupSpan = kAdamThreads * kGroup;                      // 2048 elements per workgroup and group
constexpr int kSpecSteps = MSAMP_ADAMW_CHUNK / (2 * kGroupSpan);       // 4 steps of two groups

// Stores of the fused kernels' outputs.  THRU: written through to where every compute unit of the GPU sees them (the
// `sc1` stores that an agent-scope atomic store is made of), which the shifting step needs: there a chunk may be
// written twice, by workgroups on different dies with an L2 each, and a line left dirty in one of them would be
// written back over the later store.  The stores are assembly because no builtin makes a 16-byte one; the kernel
// waits for them by hand (s_waitcnt) where their completion matters.
template <bool THRU>
__device__ __forceinline__ void put16(void* p, const uint4& v) {
    if constexpr (THRU) {
        typedef uint32_t v4u_t __attribute__((ext_vector_type(4)));
        const v4u_t vv = {v.x, v.y, v.z, v.w};
        // (the wait states after it: a store of more than 8 bytes reads its data registers over several cycles, and the
        // compiler, which does not know this is one, would not keep the next instruction off them)
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(vv) : "memory");
    } else {
        *static_cast<uint4*>(p) = v;
    }
}
template <bool THRU, typename T>
__device__ __forceinline__ void put1(T* p, T v) {
    if constexpr (THRU) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *p = v;
}

template <bool THRU>
__device__ __forceinline__ void put8(void* p, uint32_t lo, uint32_t hi) {
    if constexpr (THRU) {
        __hip_atomic_store(static_cast<uint64_t*>(p), (static_cast<uint64_t>(hi) << 32) | lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        *static_cast<uint2*>(p) = make_uint2(lo, hi);
    }
}
template <int WDT, bool THRU>
__device__ __forceinline__ void store_one(void* base, size_t i, float f) {
    if constexpr (WDT == MSAMP_DT_F16) put1<THRU>(static_cast<uint16_t*>(base) + i, static_cast<uint16_t>(float_to_f16_bits(f)));
    else put1<THRU>(static_cast<uint8_t*>(base) + i, static_cast<uint8_t>(quant1<WDT>(f)));
}

// eight raw elements of one lane, as loaded: 2 words of FP8 codes or 4 words of float16
template <int DT>
struct Raw8 {
    static constexpr int kWords = DT == MSAMP_DT_F16 ? 4 : 2;
    uint32_t w[kWords];
    __device__ __forceinline__ void load(const void* base, size_t i) {
        if constexpr (DT == MSAMP_DT_F16) {
            const uint4 a = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(base) + i);
            w[0] = a.x, w[1] = a.y, w[2] = a.z, w[3] = a.w;
        } else {
            const uint2 a = *reinterpret_cast<const uint2*>(static_cast<const uint8_t*>(base) + i);
            w[0] = a.x, w[1] = a.y;
        }
    }
    // elements 4q .. 4q+3 as floats (exact)
    __device__ __forceinline__ void quad(int q, float* f) const {
        if constexpr (DT == MSAMP_DT_F16) {
            f[0] = f16_bits_to_float(w[2 * q] & 0xffffu), f[1] = f16_bits_to_float(w[2 * q] >> 16);
            f[2] = f16_bits_to_float(w[2 * q + 1] & 0xffffu), f[3] = f16_bits_to_float(w[2 * q + 1] >> 16);
        } else {
            dequant4<DT>(w[q], f[0], f[1], f[2], f[3]);
        }
    }
    template <bool THRU>
    __device__ __forceinline__ void store(void* base, size_t i) const {
        if constexpr (DT == MSAMP_DT_F16) put16<THRU>(static_cast<uint16_t*>(base) + i, make_uint4(w[0], w[1], w[2], w[3]));
        else put8<THRU>(static_cast<uint8_t*>(base) + i, w[0], w[1]);
    }
};

// what the speculative pass carries along a chunk
struct SpecState {
    float floor_p;    // a lower bound of the tensor's max |p'|
    uint32_t mxp;     // exact |p'| bit patterns of the candidates (NaN patterns compare highest)
    float mxm, mxv;
};

// One group of eight elements at element i: new codes of the weight, exp_avg and exp_avg_sq from the raw inputs, the
// maxima folded into `st` (TRACK; without it only the codes are made: the other round of a chunk).  Nothing is stored.
// ---- the step with the dequantization factors folded into the coefficients ------------------------------------------
// With all four factors (weight, gradient, exp_avg, exp_avg_sq scale_inv) exact powers of two -- what the scale rule
// produces -- multiplying by them is exact, so it commutes with the roundings of the chain:
//   (w * w_si) * decay            = w * (w_si * decay)
//   (beta1 * m) * inv_m           = (beta1 * inv_m) * m
//   omb1 * (g * g_si)             = (omb1 * g_si) * g
//   (beta2 * v) * inv_v           = (beta2 * inv_v) * v
//   omb2 * ((g * g_si)(g * g_si)) = (omb2 * g_si^2) * (g * g)      (g * g is exact: an FP8 code has at most 4 significant bits)
// bit for bit, as long as nothing underflows or overflows on the way: 8 instructions per element instead of 12.
// fold_ok() admits factors 2^-40 .. 2^40 and coefficients of ordinary size; the smallest intermediates are then
// 2^-16 (E5M2) * 2^-40 * 2^-20 and its like, far from the denormals.  Anything else takes the plain chain.
struct Folded {
    float cw, cm, cg1, cv, c3;
};
__device__ __forceinline__ bool pow2_in_range(float x) {
    const uint32_t b = __float_as_uint(x) & 0x7fffffffu;
    const uint32_t e = b >> 23;
    return (b & 0x007fffffu) == 0u && e >= 127u - 40u && e <= 127u + 40u;
}
__device__ __forceinline__ bool ordinary(float c) { return c >= 0x1.0p-20f && c <= 2.0f; }
__device__ __forceinline__ bool fold_ok(float w_si, float g_si, float inv_m, float inv_v, const AdamConsts& k) {
    return pow2_in_range(w_si) && pow2_in_range(g_si) && pow2_in_range(inv_m) && pow2_in_range(inv_v) && ordinary(k.beta1) &&
           ordinary(k.beta2) && ordinary(k.omb1) && ordinary(k.omb2) && ordinary(k.decay);
}
__device__ __forceinline__ Folded fold(float w_si, float g_si, float inv_m, float inv_v, const AdamConsts& k) {
    Folded f;
    // (the same in every lane; this part has no scalar float arithmetic, so they are worked out in a vector register and
    // handed to scalar ones, where they cost the loop nothing)
    auto uniform = [](float x) { return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(x))); };
    f.cw = uniform(w_si * k.decay), f.cm = uniform(k.beta1 * inv_m), f.cg1 = uniform(k.omb1 * g_si);
    f.cv = uniform(k.beta2 * inv_v), f.c3 = uniform(k.omb2 * (g_si * g_si));
    return f;
}
// pj, m', v' of one element from its raw codes (decoupled decay only: the L2 form needs the plain gradient)
__device__ __forceinline__ void prepare_folded(float w_raw, float g_raw, float m_raw, float v_raw, const Folded& f, float& pj,
                                               float& m_new, float& v_new) {
#pragma clang fp contract(off)
    pj = w_raw * f.cw;
    const float t2 = f.cm * m_raw;
    const float t3 = f.cg1 * g_raw;
    m_new = t2 + t3;
    const float u2 = f.cv * v_raw;
    const float gg = g_raw * g_raw;
    const float u3 = f.c3 * gg;
    v_new = u2 + u3;
}
// any of the four packed FP8 codes all ones below the sign: what the converter makes of NaN, Inf and values beyond the
// format (E4M3; the codes of finite values in range end at 0x7e)
__device__ __forceinline__ bool any_code_7f(uint32_t w) { return (((w & 0x7f7f7f7fu) + 0x01010101u) & 0x80808080u) != 0u; }

template <int WDT, int GDT, bool L2, bool TRACK = true, bool FAST = false>
__device__ __forceinline__ void spec_group(const msamp_adamw_tensor& d, size_t i, const Raw8<WDT>& rw, const Raw8<GDT>& rg,
                                           const Raw8<MSAMP_DT_E4M3>& rm, const Raw8<MSAMP_DT_F16>& rv, float w_si, float g_si,
                                           float inv_m, float inv_v, float ws, float ms, float vs, const AdamConsts& k,
                                           SpecState& st, Raw8<WDT>& ow, Raw8<MSAMP_DT_E4M3>& om, Raw8<MSAMP_DT_F16>& ov,
                                           const Folded& fc = Folded{}) {
    // FAST (the caller has checked fold_ok(), decoupled decay and scales that follow the rule): folded factors; no clamp
    // in front of the converters -- with the guessed scales confirmed nothing leaves the formats, and a tensor whose
    // scales are not confirmed is done again through the plain path -- and the codes of exp_avg looked at once per
    // four for what the converter makes of NaN and Inf, which then take the plain conversion.
    static_assert(!(FAST && L2), "the folded chain has no plain gradient");
    float hi[kGroup];
    float lo_max = 0.0f, hi_max = 0.0f;
    float eps_v = k.eps;
    asm volatile("" : "+v"(eps_v));
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        float p4[4], g4[4], m4[4], v4[4];
        rw.quad(q, p4), rg.quad(q, g4), rm.quad(q, m4), rv.quad(q, v4);
        uint32_t code4[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float pj, g_plain = 0.0f, m_new, v_new, p_est, err;
            if constexpr (FAST) prepare_folded(p4[e], g4[e], m4[e], v4[e], fc, pj, m_new, v_new);
            else prepare<L2>(p4[e], g4[e], m4[e], v4[e], w_si, g_si, inv_m, inv_v, k, pj, g_plain, m_new, v_new);
            if constexpr (TRACK) {
                st.mxm = fmaxf(st.mxm, fabsf(m_new));
                st.mxv = fmaxf(st.mxv, fabsf(v_new));
            }
            estimate(pj, m_new, v_new, k, eps_v, p_est, err);
            const float lo = (p_est - err) * ws, up = (p_est + err) * ws;
            bool same;
            uint32_t code;
            if constexpr (WDT == MSAMP_DT_F16) {
                code = float_to_f16_bits(lo);
                same = code == float_to_f16_bits(up);
            } else {
                const uint32_t two = FAST ? cvt_pk<WDT>(lo, up, 0u, false) : cvt_pk<WDT>(sat<WDT>(lo), sat<WDT>(up), 0u, false);
                code = two & 0xffu;
                same = code == ((two >> 8) & 0xffu);
            }
            float a_hi = fabsf(p_est) + err, a_lo = fabsf(p_est) - err;    // both finite whenever err is
            if (!(same && err < __uint_as_float(0x7f800000u))) {
                // the exact chain: its |p'| goes straight into the maximum, and the element leaves the bounds
                const float pe = param_update(pj, m_new, v_new, k);
                if constexpr (TRACK) {
                    const uint32_t ab = __float_as_uint(pe) & 0x7fffffffu;
                    st.mxp = ab > st.mxp ? ab : st.mxp;
                }
                const float scaled = pe * ws;
                if constexpr (WDT == MSAMP_DT_F16) code = float_to_f16_bits(scaled);
                else code = quant1<WDT>(scaled);
                a_hi = 0.0f, a_lo = 0.0f;
            }
            code4[e] = code;
            if constexpr (TRACK) {
                hi[4 * q + e] = a_hi;
                hi_max = fmaxf(hi_max, a_hi);
                lo_max = fmaxf(lo_max, a_lo);
            }
            if constexpr (L2) moments(m4[e], v4[e], g_plain, inv_m, inv_v, k, m_new, v_new);    // stored moments ignore the L2 term
            m4[e] = m_new * ms;
            v4[e] = v_new * vs;
        }
        if constexpr (WDT == MSAMP_DT_F16) {
            ow.w[2 * q] = code4[0] | (code4[1] << 16), ow.w[2 * q + 1] = code4[2] | (code4[3] << 16);
        } else {
            ow.w[q] = code4[0] | (code4[1] << 8) | (code4[2] << 16) | (code4[3] << 24);
        }
        if constexpr (FAST) {
            uint32_t mc = quant4_in_range<MSAMP_DT_E4M3>(m4[0], m4[1], m4[2], m4[3]);
            if (__builtin_expect(any_code_7f(mc), 0)) mc = quant4<MSAMP_DT_E4M3>(m4[0], m4[1], m4[2], m4[3]);
            om.w[q] = mc;
        } else {
            om.w[q] = quant4<MSAMP_DT_E4M3>(m4[0], m4[1], m4[2], m4[3]);
        }
        ov.w[2 * q] = float_to_f16_bits(v4[0]) | (float_to_f16_bits(v4[1]) << 16);
        ov.w[2 * q + 1] = float_to_f16_bits(v4[2]) | (float_to_f16_bits(v4[3]) << 16);
    }
    if constexpr (!TRACK) return;
    st.floor_p = fmaxf(st.floor_p, __uint_as_float(wave_max_u32(__float_as_uint(lo_max))));
    const float skip_below = st.floor_p * 0.999999f;    // room for the roundings of the bounds themselves
    if (hi_max >= skip_below) {    // few lanes get here: the ones that hold an element next to the maximum
#pragma unroll
        for (int j = 0; j < kGroup; ++j) {
            if (hi[j] >= skip_below) {
                // the inputs are still in memory (this pass writes elsewhere): fetching the element again costs less
                // than keeping more values per lane alive for the few that come here
                float pj, g_plain, m_new, v_new;
                prepare<L2>(load_w1<WDT>(d.weight, i + j), load_w1<GDT>(d.grad, i + j), load_w1<MSAMP_DT_E4M3>(d.exp_avg, i + j),
                            load_w1<MSAMP_DT_F16>(d.exp_avg_sq, i + j), w_si, g_si, inv_m, inv_v, k, pj, g_plain, m_new, v_new);
                const uint32_t ab = __float_as_uint(param_update(pj, m_new, v_new, k)) & 0x7fffffffu;
                st.mxp = ab > st.mxp ? ab : st.mxp;
            }
        }
    }
}

// the element-wise tail of a chunk that is not whole (speculative pass)
template <int WDT, int GDT, bool L2, bool THRU>
__device__ __forceinline__ void spec_ragged(const msamp_adamw_tensor& d, size_t first, size_t stride, void* w_out, uint8_t* m_out,
                                            uint16_t* v_out, float w_si, float g_si, float inv_m, float inv_v, float ws, float ms,
                                            float vs, const AdamConsts& k, SpecState& st) {
    for (size_t i = first; i < d.numel; i += stride) {
        const float m_old = load_w1<MSAMP_DT_E4M3>(d.exp_avg, i), v_old = load_w1<MSAMP_DT_F16>(d.exp_avg_sq, i);
        float pj, g_plain, m_new, v_new;
        prepare<L2>(load_w1<WDT>(d.weight, i), load_w1<GDT>(d.grad, i), m_old, v_old, w_si, g_si, inv_m, inv_v, k, pj, g_plain,
                    m_new, v_new);
        const float pn = param_update(pj, m_new, v_new, k);
        const uint32_t ab = __float_as_uint(pn) & 0x7fffffffu;
        st.mxp = ab > st.mxp ? ab : st.mxp;
        st.mxm = fmaxf(st.mxm, fabsf(m_new));
        st.mxv = fmaxf(st.mxv, fabsf(v_new));
        store_one<WDT, THRU>(w_out, i, pn * ws);
        if constexpr (L2) moments(m_old, v_old, g_plain, inv_m, inv_v, k, m_new, v_new);
        store_one<MSAMP_DT_E4M3, THRU>(m_out, i, m_new * ms);
        store_one<MSAMP_DT_F16, THRU>(v_out, i, v_new * vs);
    }
}

// The speculative pass between two sets of buffers works on sixteen consecutive elements per lane (16-byte accesses
// throughout; measured 6 % faster there than the groups of eight that the shifting step below needs for its
// written-through stores), one lane's sixteen elements at a time:
template <int WDT, int GDT, bool L2, bool FAST = false>
__device__ __forceinline__ void spec_step16(const msamp_adamw_tensor& d, void* w_out, uint8_t* m_out, uint16_t* v_out, size_t i,
                                          float* p, const float* g,
                                          float* m, float* v, float w_si, float g_si, float inv_m, float inv_v, float ws,
                                          float ms, float vs, const AdamConsts& k, float& floor_p, uint32_t& mxp,
                                          float& mxm, float& mxv, const Folded& fc = Folded{}) {
    static_assert(!(FAST && L2), "the folded chain has no plain gradient");    // FAST: as in spec_group
    uint32_t wq[kEPT];
    float hi[kEPT];
    float lo_max = 0.0f, hi_max = 0.0f;
    float eps_v = k.eps;
    asm volatile("" : "+v"(eps_v));
#pragma unroll
    for (int j = 0; j < kEPT; ++j) {
        float pj, g_plain = 0.0f, m_new, v_new, p_est, err;
        if constexpr (FAST) prepare_folded(p[j], g[j], m[j], v[j], fc, pj, m_new, v_new);
        else prepare<L2>(p[j], g[j], m[j], v[j], w_si, g_si, inv_m, inv_v, k, pj, g_plain, m_new, v_new);
        mxm = fmaxf(mxm, fabsf(m_new));
        mxv = fmaxf(mxv, fabsf(v_new));
        estimate(pj, m_new, v_new, k, eps_v, p_est, err);
        const float lo = (p_est - err) * ws, up = (p_est + err) * ws;
        bool same;
        uint32_t code;
        if constexpr (WDT == MSAMP_DT_F16) {
            code = float_to_f16_bits(lo);
            same = code == float_to_f16_bits(up);
        } else {
            const uint32_t two = FAST ? cvt_pk<WDT>(lo, up, 0u, false) : cvt_pk<WDT>(sat<WDT>(lo), sat<WDT>(up), 0u, false);
            code = two & 0xffu;
            same = code == ((two >> 8) & 0xffu);
        }
        float a_hi = fabsf(p_est) + err, a_lo = fabsf(p_est) - err;    // both finite whenever err is
        if (!(same && err < __uint_as_float(0x7f800000u))) {
            // the exact chain: its |p'| goes straight into the maximum, and the element leaves the bounds
            const float pe = param_update(pj, m_new, v_new, k);
            const uint32_t ab = __float_as_uint(pe) & 0x7fffffffu;
            mxp = ab > mxp ? ab : mxp;
            const float scaled = pe * ws;
            if constexpr (WDT == MSAMP_DT_F16) {
                code = float_to_f16_bits(scaled);
            } else {
                code = quant1<WDT>(scaled);
            }
            a_hi = 0.0f, a_lo = 0.0f;
        }
        wq[j] = code;
        hi[j] = a_hi;
        hi_max = fmaxf(hi_max, a_hi);
        lo_max = fmaxf(lo_max, a_lo);
        if constexpr (L2) moments(m[j], v[j], g_plain, inv_m, inv_v, k, m_new, v_new);    // stored moments ignore the L2 term
        m[j] = m_new * ms;
        v[j] = v_new * vs;
    }
    if constexpr (WDT == MSAMP_DT_F16) {
        uint4* o = reinterpret_cast<uint4*>(static_cast<uint16_t*>(w_out) + i);
        o[0] = make_uint4(wq[0] | (wq[1] << 16), wq[2] | (wq[3] << 16), wq[4] | (wq[5] << 16), wq[6] | (wq[7] << 16));
        o[1] = make_uint4(wq[8] | (wq[9] << 16), wq[10] | (wq[11] << 16), wq[12] | (wq[13] << 16), wq[14] | (wq[15] << 16));
    } else {
        uint4 o;
        o.x = wq[0] | (wq[1] << 8) | (wq[2] << 16) | (wq[3] << 24);
        o.y = wq[4] | (wq[5] << 8) | (wq[6] << 16) | (wq[7] << 24);
        o.z = wq[8] | (wq[9] << 8) | (wq[10] << 16) | (wq[11] << 24);
        o.w = wq[12] | (wq[13] << 8) | (wq[14] << 16) | (wq[15] << 24);
        *reinterpret_cast<uint4*>(static_cast<uint8_t*>(w_out) + i) = o;
    }
    if constexpr (FAST) {
        uint32_t o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            o[q] = quant4_in_range<MSAMP_DT_E4M3>(m[4 * q], m[4 * q + 1], m[4 * q + 2], m[4 * q + 3]);
            if (__builtin_expect(any_code_7f(o[q]), 0)) o[q] = quant4<MSAMP_DT_E4M3>(m[4 * q], m[4 * q + 1], m[4 * q + 2], m[4 * q + 3]);
        }
        *reinterpret_cast<uint4*>(m_out + i) = make_uint4(o[0], o[1], o[2], o[3]);
    } else {
        store_w16<MSAMP_DT_E4M3>(m_out, i, m);
    }
    store_w16<MSAMP_DT_F16>(v_out, i, v);
    floor_p = fmaxf(floor_p, __uint_as_float(wave_max_u32(__float_as_uint(lo_max))));
    const float skip_below = floor_p * 0.999999f;    // room for the roundings of the bounds themselves
    if (hi_max >= skip_below) {    // few lanes get here: the ones that hold an element next to the maximum
#pragma unroll
        for (int j = 0; j < kEPT; ++j) {
            if (hi[j] >= skip_below) {
                // the inputs are still in memory (this pass writes elsewhere): fetching the element again costs less
                // than keeping 48 more values per lane alive for the few that come here
                float pj, g_plain, m_new, v_new;
                prepare<L2>(load_w1<WDT>(d.weight, i + j), load_w1<GDT>(d.grad, i + j), load_w1<MSAMP_DT_E4M3>(d.exp_avg, i + j),
                            load_w1<MSAMP_DT_F16>(d.exp_avg_sq, i + j), w_si, g_si, inv_m, inv_v, k, pj, g_plain, m_new, v_new);
                const uint32_t ab = __float_as_uint(param_update(pj, m_new, v_new, k)) & 0x7fffffffu;
                mxp = ab > mxp ? ab : mxp;
            }
        }
    }
}

template <int WDT, int GDT, bool L2>
__global__ __launch_bounds__(kAdamThreads) void fused_spec_kernel(msamp_adamw_tensor* __restrict__ tensors,
                                                                   const int32_t* __restrict__ block_map, AdamConsts k,
                                                                   const msamp_adamw_buffers* __restrict__ outs) {
    __shared__ uint32_t red[kAdamThreads / kWave];
    const int t = block_map[2 * blockIdx.x], chunk = block_map[2 * blockIdx.x + 1];
    msamp_adamw_tensor& d = tensors[t];
    void* w_out = outs[t].weight;
    uint8_t* m_out = outs[t].exp_avg;
    uint16_t* v_out = outs[t].exp_avg_sq;
    const size_t n = d.numel;
    const size_t base = static_cast<size_t>(chunk) * MSAMP_ADAMW_CHUNK;
    const float w_si = *d.w_scale_inv, g_si = k.maximize ? -*d.g_scale_inv : *d.g_scale_inv;
    const float ws = *d.w_scale, ms = *d.m_scale, vs = *d.v_scale;    // the guess: the scales in force
    const float inv_m = 1.0f / ms, inv_v = 1.0f / vs;
    uint32_t mxp = 0;
    float mxm = 0.0f, mxv = 0.0f;
    float floor_p = __uint_as_float(__hip_atomic_load(&d.acc[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    if (!(floor_p >= 0.0f)) floor_p = 0.0f;
    if (base + MSAMP_ADAMW_CHUNK <= n) {
        // the folded, clamp-free form of the step where the tensor's factors allow it (see spec_group)
        bool fast = !L2 && k.rule_scales && fold_ok(w_si, g_si, inv_m, inv_v, k);
        fast = __builtin_amdgcn_readfirstlane(fast);
        const Folded fc = fold(w_si, g_si, inv_m, inv_v, k);
        if (!L2 && fast) {
            if constexpr (!L2) {
#pragma unroll 1
                for (int s = 0; s < kSteps; ++s) {
                    const size_t i = base + (static_cast<size_t>(s) * kAdamThreads + threadIdx.x) * kEPT;
                    float p[kEPT], g[kEPT], m[kEPT], v[kEPT];
                    load16<WDT, GDT>(d, i, p, g, m, v);
                    spec_step16<WDT, GDT, L2, true>(d, w_out, m_out, v_out, i, p, g, m, v, w_si, g_si, inv_m, inv_v, ws, ms, vs, k,
                                                    floor_p, mxp, mxm, mxv, fc);
                }
            }
        } else {
#pragma unroll 1
            for (int s = 0; s < kSteps; ++s) {
                const size_t i = base + (static_cast<size_t>(s) * kAdamThreads + threadIdx.x) * kEPT;
                float p[kEPT], g[kEPT], m[kEPT], v[kEPT];
                load16<WDT, GDT>(d, i, p, g, m, v);
                spec_step16<WDT, GDT, L2>(d, w_out, m_out, v_out, i, p, g, m, v, w_si, g_si, inv_m, inv_v, ws, ms, vs, k, floor_p,
                                          mxp, mxm, mxv);
            }
        }
    } else {
        for (size_t i = base + threadIdx.x; i < n; i += kAdamThreads) {
            const float m_old = load_w1<MSAMP_DT_E4M3>(d.exp_avg, i), v_old = load_w1<MSAMP_DT_F16>(d.exp_avg_sq, i);
            float pj, g_plain, m_new, v_new;
            prepare<L2>(load_w1<WDT>(d.weight, i), load_w1<GDT>(d.grad, i), m_old, v_old, w_si, g_si, inv_m, inv_v, k, pj,
                    g_plain, m_new, v_new);
            const float pn = param_update(pj, m_new, v_new, k);
            const uint32_t ab = __float_as_uint(pn) & 0x7fffffffu;
            mxp = ab > mxp ? ab : mxp;
            mxm = fmaxf(mxm, fabsf(m_new));
            mxv = fmaxf(mxv, fabsf(v_new));
            store_w1<WDT>(w_out, i, pn * ws);
            if constexpr (L2) moments(m_old, v_old, g_plain, inv_m, inv_v, k, m_new, v_new);
            store_w1<MSAMP_DT_E4M3>(m_out, i, m_new * ms);
            store_w1<MSAMP_DT_F16>(v_out, i, v_new * vs);
        }
    }
    const uint32_t a = block_max_u32(mxp, red);
    const uint32_t b = block_max_u32(__float_as_uint(mxm), red);
    const uint32_t c = block_max_u32(__float_as_uint(mxv), red);
    if (threadIdx.x == 0) {
        if (a) atomicMax(&d.acc[0], a);
        if (b) atomicMax(&d.acc[1], b);
        if (c) atomicMax(&d.acc[2], c);
    }
}

// ---- the one-pass step inside shifting arenas -------------------------------------------------------------
// The speculative pass needs its outputs away from its inputs (a tensor whose scales it guessed wrong is done again
// from the inputs), but not a whole second set of buffers.  Here the payloads of all tensors lie back to back in one
// arena per kind (weights, exp_avg, exp_avg_sq), each tensor padded to whole chunks, with `slack` chunks of room at
// one end, and a step moves everything by `slack` chunks towards the room: the workgroup of chunk j writes where the
// chunk `slack` positions earlier in the walk used to be.  That earlier chunk's tensor must be through by then.
// Every wavefront marks its quarter of a chunk when it is stored.  The workgroup about to overwrite the FIRST chunk
// of a tensor waits for the marks of all that tensor's chunks, applies the scale rule (what fused_scales_kernel does
// for the other forms) and posts the outcome; every wavefront about to overwrite any of the tensor's chunks waits for
// that post.  Nobody ever waits for anything but tensors that lie wholly earlier in the walk, whose workgroups the
// hardware started earlier, so nobody waits for a workgroup that cannot run; and with the room a few thousand chunks
// larger than the largest tensor nobody waits at all in practice: the post is asked for when a wavefront starts and
// looked at when its first outputs are ready to be stored.  If the post says the tensor takes another round, the
// wavefront does its quarter of that chunk again first, from the inputs it is about to overwrite (the same lanes
// read there that write there afterwards).  The tensors at the end of the walk, which nobody overwrites, are left to
// fused_shift_scales_kernel and fused_shift_tail_kernel.  The next step walks the other way and moves everything
// back.  Extra memory: `slack` chunks per arena instead of a second copy.
//
// What crosses between workgroups, and how, without a fence (a release or acquire at agent scope writes back or
// invalidates a whole L2 on this part), without an atomic that every workgroup would have to take in turn, and
// without a workgroup barrier (the wavefronts of a workgroup come and go on their own):
//  * a maximum goes out as an agent-scope atomic, only where it raises the word, and the wavefront's mark takes the
//    returned values as an operand, so it is issued only when those atomics have been performed;
//  * a mark or a post is one agent-scope store of this call's token, or of {token, value}: whoever reads the token
//    beside a value reads that value;
//  * payload stores are written through (THRU) and a wavefront waits for its own before it marks, so its part of the
//    chunk is in memory before the mark -- and before anybody who then writes the same places a second time (the
//    other round, possibly from another die) issues its stores;
//  * inputs are read with ordinary loads: nothing writes them during the launch until their own overwriting.
constexpr int kWavesPerChunk = kAdamThreads / kWave;
// sync buffer of a call, in 8-byte words: per tensor kShiftPostWords post words; then per chunk one verdict word
// {token, another round?} (what the wavefronts about to overwrite that chunk read: one word per chunk, so that no single
// address is asked for by a whole tensor's wavefronts); then per chunk and wavefront kMarkWords mark words
// {token, max |p'|}, {token, max |m'|}, {token, max |v'|} (a wavefront's maxima travel in its marks: no atomics)
constexpr int kMarkWords = 4;
struct ShiftArgs {
    long long shift;        // output element = input element + shift (its sign is the direction of the walk)
    int slack;              // |shift| in chunks
    int lead;               // how many chunks ahead of a tensor's first overwriting its outcome is decided
    int n_chunks;
    int n_tensors;
    uint32_t token;
    uint32_t spin_limit;
    uint32_t* error_word;
    int32_t* redo;
    uint64_t* posts;        // kShiftPostWords words per tensor
    uint64_t* verdicts;     // one word per chunk
    uint64_t* marks;        // kWavesPerChunk * kMarkWords words per chunk
    float w_fp_max;
    int tensor_scale;
};
constexpr uint32_t kErrShiftGaveUp = 4, kErrShiftLayout = 8;
// post words of a tensor: [0] 1 = another round; then the factors that round needs: the old weight scale_inv, the old
// reciprocal moment scales, the new weight and moment scales
constexpr int kShiftPostWords = MSAMP_ADAMW_POST_WORDS;

__device__ __forceinline__ void post_word(uint64_t* p, uint32_t token, uint32_t value) {
    __hip_atomic_store(p, (static_cast<uint64_t>(token) << 32) | value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool anybody_gave_up(const ShiftArgs& a) {
    return __hip_atomic_load(a.error_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
}
// the value posted beside this call's token; `ok` is cleared if it does not show up within the limit
__device__ __forceinline__ uint32_t await_post(const uint64_t* p, const ShiftArgs& a, bool& ok) {
    for (uint32_t spins = 0; ok; ++spins) {
        const uint64_t w = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (static_cast<uint32_t>(w >> 32) == a.token) return static_cast<uint32_t>(w);
        // the limit, or somebody else has given up already: nobody waits any longer
        if (spins >= a.spin_limit || anybody_gave_up(a)) ok = false;
        else __builtin_amdgcn_s_sleep(8);
    }
    return 0u;
}

template <int WDT>
__device__ __forceinline__ void* shifted_weight(void* p, long long shift) {
    if constexpr (WDT == MSAMP_DT_F16) return static_cast<uint16_t*>(p) + shift;
    else return static_cast<uint8_t*>(p) + shift;
}

// The maxima of a tensor from the marks of its wavefronts, gathered by a whole workgroup (valid in its first lane);
// returns false if a mark of this call does not show up within the limit.  first_chunk: index of the tensor's first
// chunk in the launch.  Every lane asks for all its marks at once, a dozen loads in flight: this sits between a
// tensor and everybody who writes over it.
__device__ __forceinline__ bool gather_marks(const ShiftArgs& a, int first_chunk, int chunks, uint32_t* red, uint32_t& mp,
                                             uint32_t& mm, uint32_t& mv) {
    const uint64_t* marks = a.marks + static_cast<size_t>(first_chunk) * (kWavesPerChunk * kMarkWords);
    const int n_waves = chunks * kWavesPerChunk;
    mp = 0, mm = 0, mv = 0;
    bool mine = true;
    constexpr int kBatch = 4;    // wavefronts per lane and round: 12 loads in flight
    for (int w0 = threadIdx.x; w0 < n_waves; w0 += kAdamThreads * kBatch) {
        uint64_t word[kBatch][3];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const int w = w0 + u * kAdamThreads;
#pragma unroll
            for (int i = 0; i < 3; ++i)
                word[u][i] = w < n_waves ? __hip_atomic_load(marks + static_cast<size_t>(w) * kMarkWords + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                         : (static_cast<uint64_t>(a.token) << 32);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const int w = w0 + u * kAdamThreads;
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                // not there yet (rare: the tensor has only just been finished): wait for it
                for (uint32_t spins = 0; static_cast<uint32_t>(word[u][i] >> 32) != a.token; ++spins) {
                    if (spins >= a.spin_limit || anybody_gave_up(a)) {
                        mine = false;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(8);
                    word[u][i] = __hip_atomic_load(marks + static_cast<size_t>(w) * kMarkWords + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            mp = umax(mp, static_cast<uint32_t>(word[u][0])), mm = umax(mm, static_cast<uint32_t>(word[u][1]));
            mv = umax(mv, static_cast<uint32_t>(word[u][2]));
        }
    }
    const bool all = __syncthreads_and(mine) != 0;
    mp = block_max_u32(mp, red), mm = block_max_u32(mm, red), mv = block_max_u32(mv, red);
    return all;
}

// What fused_scales_kernel does, for one tensor whose maxima are known to the workgroup's first lane (the whole
// workgroup comes here).  in_launch: also tell the wavefronts of this launch that will overwrite the tensor's chunks --
// the factors another round needs in the tensor's post words, the verdict in every chunk's own word.
__device__ __forceinline__ void decide_tensor(msamp_adamw_tensor& d, int t, const ShiftArgs& a, int first_chunk, int chunks,
                                              uint32_t mp, uint32_t mm, uint32_t mv, bool in_launch, uint32_t* red) {
    if (threadIdx.x == 0) {
        const float ap = __uint_as_float(mp), am = __uint_as_float(mm), av = __uint_as_float(mv);
        const float old_ws = *d.w_scale, old_ms = *d.m_scale, old_vs = *d.v_scale;
        const float old_wsi = *d.w_scale_inv, old_inv_m = 1.0f / old_ms, old_inv_v = 1.0f / old_vs;
        d.saved[0] = old_wsi, d.saved[1] = old_inv_m, d.saved[2] = old_inv_v;
        const float ws = scale_rule(ap, old_ws, a.w_fp_max, 0);
        const float ms = a.tensor_scale ? scale_rule(am, 1.0f, 448.0f, 0) : 1.0f;
        const float vs = a.tensor_scale ? scale_rule(av, 1.0f, 65504.0f, 0) : 1.0f;
        const uint32_t again = (__float_as_uint(ws) != __float_as_uint(old_ws) || __float_as_uint(ms) != __float_as_uint(old_ms) ||
                                __float_as_uint(vs) != __float_as_uint(old_vs))
                                   ? 1u
                                   : 0u;
        red[0] = again;
        // for the kernels and the host that come after this launch
        a.redo[t] = static_cast<int32_t>(again);
        *d.w_scale = ws;
        *d.w_scale_inv = 1.0f / ws;
        *d.w_amax = ap;
        *d.m_scale = ms;
        *d.m_scale_inv = 1.0f / ms;
        *d.m_amax = am;
        *d.v_scale = vs;
        *d.v_scale_inv = 1.0f / vs;
        *d.v_amax = av;
        uint64_t* post = a.posts + static_cast<size_t>(t) * kShiftPostWords;
        if (in_launch && again) {
            post_word(post + 1, a.token, __float_as_uint(old_wsi));
            post_word(post + 2, a.token, __float_as_uint(old_inv_m));
            post_word(post + 3, a.token, __float_as_uint(old_inv_v));
            post_word(post + 4, a.token, __float_as_uint(ws));
            post_word(post + 5, a.token, __float_as_uint(ms));
            post_word(post + 6, a.token, __float_as_uint(vs));
        }
        post_word(post, a.token, again);    // also what tells fused_shift_scales_kernel that the tensor is settled
    }
    if (in_launch) {
        __syncthreads();
        const uint32_t again = red[0];
        for (int c = threadIdx.x; c < chunks; c += kAdamThreads) post_word(a.verdicts + first_chunk + c, a.token, again);
    }
}

// This wavefront's quarter of the other round of one chunk: what write_chunk does, by the same element functions, in
// the groups of eight of the speculative pass (whose registers it shares here), written through.  f: the old weight
// scale_inv, the old reciprocal moment scales, the new weight and moment scales.
template <int WDT, int GDT, bool L2>
__device__ __forceinline__ void redo_quarter(const msamp_adamw_tensor& d, int chunk, long long shift, const float (&f)[6],
                                             const AdamConsts& k) {
    void* w_out = shifted_weight<WDT>(d.weight, shift);
    uint8_t* m_out = d.exp_avg + shift;
    uint16_t* v_out = d.exp_avg_sq + shift;
    const float g_si0 = *d.g_scale_inv, g_si = k.maximize ? -g_si0 : g_si0;
    const size_t base = static_cast<size_t>(chunk) * MSAMP_ADAMW_CHUNK;
    SpecState unused;
    if (base + MSAMP_ADAMW_CHUNK <= d.numel) {
#pragma unroll 1
        for (int s = 0; s < 2 * kSpecSteps; ++s) {
            const size_t i = base + static_cast<size_t>(s) * kGroupSpan + threadIdx.x * kGroup;
            Raw8<WDT> rw, ow;
            Raw8<GDT> rg;
            Raw8<MSAMP_DT_E4M3> rm, om;
            Raw8<MSAMP_DT_F16> rv, ov;
            rw.load(d.weight, i), rg.load(d.grad, i), rm.load(d.exp_avg, i), rv.load(d.exp_avg_sq, i);
            spec_group<WDT, GDT, L2, false>(d, i, rw, rg, rm, rv, f[0], g_si, f[1], f[2], f[3], f[4], f[5], k, unused, ow, om, ov);
            ow.template store<true>(w_out, i), om.template store<true>(m_out, i), ov.template store<true>(v_out, i);
        }
    } else {
        for (size_t i = base + threadIdx.x; i < d.numel; i += kAdamThreads) {
            const float m_old = load_w1<MSAMP_DT_E4M3>(d.exp_avg, i), v_old = load_w1<MSAMP_DT_F16>(d.exp_avg_sq, i);
            float pj, g_plain, m_new, v_new;
            prepare<L2>(load_w1<WDT>(d.weight, i), load_w1<GDT>(d.grad, i), m_old, v_old, f[0], g_si, f[1], f[2], k, pj, g_plain,
                        m_new, v_new);
            store_one<WDT, true>(w_out, i, param_update(pj, m_new, v_new, k) * f[3]);
            if constexpr (L2) moments(m_old, v_old, g_plain, f[1], f[2], k, m_new, v_new);
            store_one<MSAMP_DT_E4M3, true>(m_out, i, m_new * f[4]);
            store_one<MSAMP_DT_F16, true>(v_out, i, v_new * f[5]);
        }
    }
}

template <int WDT, int GDT, bool L2>
__global__ __launch_bounds__(kAdamThreads) void fused_shift_kernel(msamp_adamw_tensor* __restrict__ tensors,
                                                                    const int32_t* __restrict__ block_map, AdamConsts k,
                                                                    ShiftArgs a) {
    const int b = blockIdx.x;
    const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const bool up = a.shift > 0;    // moving up: walk from the top, so that the room is always ahead
    const int j = up ? a.n_chunks - 1 - b : b;
    const int t = block_map[2 * j], chunk = block_map[2 * j + 1];
    // the chunk that lies where this one's outputs go, if any
    const bool overwrites = b >= a.slack;
    const int jv = overwrites ? (up ? j + a.slack : j - a.slack) : j;
    const int tv = block_map[2 * jv], cv = block_map[2 * jv + 1];
    msamp_adamw_tensor& d = tensors[t];
    msamp_adamw_tensor& dv = tensors[tv];
    const uint64_t* post = a.posts + static_cast<size_t>(tv) * kShiftPostWords;
    // Who decides a tensor's outcome: the workgroup `lead` chunks ahead of the one that overwrites the tensor's first chunk
    // (in the order of the walk), so that the outcome is posted by the time anybody needs it -- if the tensor is short
    // enough to lie wholly before that workgroup; else the workgroup that overwrites its first chunk.
    __shared__ uint32_t red[kAdamThreads / kWave];
    auto decides_ahead = [&](int chunks) { return chunks <= a.slack - a.lead; };
    auto decide = [&](int jt) {    // jt: index of any chunk of the tensor
        const int tt = block_map[2 * jt], first = jt - block_map[2 * jt + 1];
        msamp_adamw_tensor& dt = tensors[tt];
        const int chunks_t = static_cast<int>((dt.numel + MSAMP_ADAMW_CHUNK - 1) / MSAMP_ADAMW_CHUNK);
        uint32_t gp, gm, gv;
        if (gather_marks(a, first, chunks_t, red, gp, gm, gv)) decide_tensor(dt, tt, a, first, chunks_t, gp, gm, gv, true, red);
        else if (threadIdx.x == 0) report_wait_expired(a.error_word, kErrShiftGaveUp);
    };
    auto first_walked = [&](int jt) {    // is this the chunk of its tensor that the walk meets first?
        const int ct = block_map[2 * jt + 1];
        if (!up) return ct == 0;
        const msamp_adamw_tensor& dt = tensors[block_map[2 * jt]];
        return ct == static_cast<int>((dt.numel + MSAMP_ADAMW_CHUNK - 1) / MSAMP_ADAMW_CHUNK) - 1;
    };
    {
        const int q = b - (a.slack - a.lead);    // position in the walk of the chunk overwritten `lead` workgroups from here
        if (a.lead > 0 && q >= 0) {
            const int jq = up ? a.n_chunks - 1 - q : q;
            if (first_walked(jq)) {
                const msamp_adamw_tensor& dq = tensors[block_map[2 * jq]];
                if (decides_ahead(static_cast<int>((dq.numel + MSAMP_ADAMW_CHUNK - 1) / MSAMP_ADAMW_CHUNK))) decide(jq);
            }
        }
    }
    uint64_t posted = 0;    // first lane: what the verdict word of the chunk underneath held when this wavefront started
    if (overwrites) {
        if (tv == t) {
            // a tensor longer than the room: the layout is not what this kernel needs
            if (threadIdx.x == 0) report_wait_expired(a.error_word, kErrShiftLayout);
            return;
        }
        const int chunks_v = static_cast<int>((dv.numel + MSAMP_ADAMW_CHUNK - 1) / MSAMP_ADAMW_CHUNK);
        if (first_walked(jv) && !(a.lead > 0 && decides_ahead(chunks_v))) decide(jv);
    }

    void* w_out = shifted_weight<WDT>(d.weight, a.shift);
    uint8_t* m_out = d.exp_avg + a.shift;
    uint16_t* v_out = d.exp_avg_sq + a.shift;
    const size_t base = static_cast<size_t>(chunk) * MSAMP_ADAMW_CHUNK;
    const float w_si = *d.w_scale_inv, g_si = k.maximize ? -*d.g_scale_inv : *d.g_scale_inv;
    const float ws = *d.w_scale, ms = *d.m_scale, vs = *d.v_scale;    // the guess: the scales in force
    const float inv_m = 1.0f / ms, inv_v = 1.0f / vs;
    SpecState st;
    st.mxp = 0, st.mxm = 0.0f, st.mxv = 0.0f, st.floor_p = 0.0f;

    // Before this wavefront's first store: what became of the tensor underneath.  Returns 0 = go on, 1 = its chunk
    // has just been done again by these lanes (whatever they held is gone), negative = gave up.
    bool gate_open = !overwrites;
    auto gate = [&]() -> int {
        int verdict = 0;
        float f[6] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        if (lane == 0) {
            bool ok = true;
            const uint32_t again = static_cast<uint32_t>(posted >> 32) == a.token ? static_cast<uint32_t>(posted) : await_post(a.verdicts + jv, a, ok);
            if (ok && again) {
#pragma unroll
                for (int i = 0; i < 6; ++i) f[i] = __uint_as_float(await_post(post + 1 + i, a, ok));
            }
            if (!ok) report_wait_expired(a.error_word, kErrShiftGaveUp);
            verdict = ok ? static_cast<int>(again) : -1;
        }
        verdict = __builtin_amdgcn_readfirstlane(verdict);
        if (verdict > 0) {
#pragma unroll
            for (int i = 0; i < 6; ++i) f[i] = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(f[i])));
            redo_quarter<WDT, GDT, L2>(dv, cv, a.shift, f, k);
            // A whole chunk and a partly filled one are shared out among the lanes differently: if one of the two chunks
            // is of each kind, these lanes' outputs land on what other wavefronts of the workgroup read for the other
            // round, and all four must be through with it first (all four come here: the verdict is the tensor's).
            const bool own_whole = base + MSAMP_ADAMW_CHUNK <= d.numel;
            const bool other_whole = static_cast<size_t>(cv) * MSAMP_ADAMW_CHUNK + MSAMP_ADAMW_CHUNK <= dv.numel;
            if (own_whole != other_whole) __syncthreads();
        }
        return verdict;
    };

    if (base + MSAMP_ADAMW_CHUNK <= d.numel) {
        // the folded, clamp-free form of the step where the tensor's factors allow it (see spec_group)
        bool fast = !L2 && a.tensor_scale && fold_ok(w_si, g_si, inv_m, inv_v, k);
        fast = __builtin_amdgcn_readfirstlane(fast);
        const Folded fc = fold(w_si, g_si, inv_m, inv_v, k);
        // (the loop twice, as a macro: behind a generic lambda the kernel's argument structures moved to the stack)
#define MSAMP_SHIFT_WALK(FASTV)                                                                                                  \
    _Pragma("unroll 1") for (int s = 0; s < kSpecSteps;) {                                                                       \
        const size_t i0 = base + static_cast<size_t>(s) * (2 * kGroupSpan) + threadIdx.x * kGroup, i1 = i0 + kGroupSpan;          \
        Raw8<WDT> w0, w1, ow;                                                                                                     \
        Raw8<GDT> g0, g1;                                                                                                         \
        Raw8<MSAMP_DT_E4M3> m0, m1, om;                                                                                           \
        Raw8<MSAMP_DT_F16> v0, v1, ov;                                                                                            \
        w0.load(d.weight, i0), g0.load(d.grad, i0), m0.load(d.exp_avg, i0), v0.load(d.exp_avg_sq, i0);                            \
        w1.load(d.weight, i1), g1.load(d.grad, i1), m1.load(d.exp_avg, i1), v1.load(d.exp_avg_sq, i1);                            \
        /* the verdict on the chunk underneath: asked for behind this wavefront's own loads (it comes from further away  */      \
        /* than they do, and loads return in order), looked at when the first outputs are ready                          */      \
        if (!gate_open && lane == 0) posted = __hip_atomic_load(a.verdicts + jv, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);     \
        const SpecState before = st;                                                                                              \
        spec_group<WDT, GDT, L2, true, FASTV>(d, i0, w0, g0, m0, v0, w_si, g_si, inv_m, inv_v, ws, ms, vs, k, st, ow, om, ov, fc); \
        if (!gate_open) {                                                                                                         \
            const int verdict = gate();                                                                                           \
            /* gave up: this chunk is left as it was; the call has failed and the error word says so */                          \
            if (verdict < 0) return;                                                                                              \
            gate_open = true;                                                                                                     \
            if (verdict > 0) { /* start the step again */                                                                         \
                st = before;                                                                                                      \
                continue;                                                                                                         \
            }                                                                                                                     \
        }                                                                                                                         \
        ow.template store<true>(w_out, i0), om.template store<true>(m_out, i0), ov.template store<true>(v_out, i0);               \
        spec_group<WDT, GDT, L2, true, FASTV>(d, i1, w1, g1, m1, v1, w_si, g_si, inv_m, inv_v, ws, ms, vs, k, st, ow, om, ov, fc); \
        ow.template store<true>(w_out, i1), om.template store<true>(m_out, i1), ov.template store<true>(v_out, i1);               \
        ++s;                                                                                                                      \
    }
        if constexpr (L2) {
            MSAMP_SHIFT_WALK(false)
        } else {
            if (fast) {
                MSAMP_SHIFT_WALK(true)
            } else {
                MSAMP_SHIFT_WALK(false)
            }
        }
#undef MSAMP_SHIFT_WALK
    } else {
        // the tensor's last, partly filled chunk: element by element, a lane's elements the same in both rounds
        if (!gate_open && gate() < 0) return;
        spec_ragged<WDT, GDT, L2, true>(d, base + threadIdx.x, kAdamThreads, w_out, m_out, v_out, w_si, g_si, inv_m, inv_v, ws, ms, vs,
                                        k, st);
    }
    // this wavefront's stores have arrived before anything its first lane publishes
    __builtin_amdgcn_s_waitcnt(0x0F70);    // vmcnt(0)
    const uint32_t mp = wave_max_u32(st.mxp), mm = wave_max_u32(__float_as_uint(st.mxm)), mv = wave_max_u32(__float_as_uint(st.mxv));
    if (lane == 0) {
        uint64_t* mark = a.marks + (static_cast<size_t>(j) * kWavesPerChunk + wave) * kMarkWords;
        post_word(mark, a.token, mp);
        post_word(mark + 1, a.token, mm);
        post_word(mark + 2, a.token, mv);
    }
}

// after the walk: the tensors nobody has decided (their first chunk lies where nothing is written over it); one
// workgroup per tensor, which finds the tensor's first chunk in the block map (tensors in order there) by bisection
__global__ __launch_bounds__(kAdamThreads) void fused_shift_scales_kernel(msamp_adamw_tensor* tensors, const int32_t* block_map,
                                                                           ShiftArgs a) {
    __shared__ uint32_t red[kAdamThreads / kWave];
    const int t = blockIdx.x;
    if (static_cast<uint32_t>(a.posts[static_cast<size_t>(t) * kShiftPostWords] >> 32) == a.token) return;
    int lo = 0, hi = a.n_chunks;    // first chunk whose tensor is >= t
    while (lo < hi) {
        const int mid = lo + (hi - lo) / 2;
        if (block_map[2 * mid] < t) lo = mid + 1;
        else hi = mid;
    }
    if (lo >= a.n_chunks || block_map[2 * lo] != t) return;    // a tensor without elements has no chunk
    msamp_adamw_tensor& d = tensors[t];
    const int chunks = static_cast<int>((d.numel + MSAMP_ADAMW_CHUNK - 1) / MSAMP_ADAMW_CHUNK);
    uint32_t gp, gm, gv;
    if (gather_marks(a, lo, chunks, red, gp, gm, gv)) decide_tensor(d, t, a, lo, chunks, gp, gm, gv, false, red);
    else if (threadIdx.x == 0) report_wait_expired(a.error_word, kErrShiftGaveUp);
}

// the last `slack` chunks of the walk: nothing is written over them, so nobody has looked at their tensors' marks
// (a launch of its own: everything the earlier ones stored is in memory by now, ordinary loads and stores do)
template <int WDT, int GDT, bool L2>
__global__ __launch_bounds__(kAdamThreads) void fused_shift_tail_kernel(msamp_adamw_tensor* __restrict__ tensors,
                                                                         const int32_t* __restrict__ block_map, AdamConsts k,
                                                                         ShiftArgs a) {
    const int first = a.n_chunks > a.slack ? a.n_chunks - a.slack : 0;
    const int b = first + blockIdx.x;    // position in the walk
    const int j = a.shift > 0 ? a.n_chunks - 1 - b : b;
    const int t = block_map[2 * j], chunk = block_map[2 * j + 1];
    if (a.redo[t] == 0) return;
    msamp_adamw_tensor& d = tensors[t];
    const float g_si = k.maximize ? -*d.g_scale_inv : *d.g_scale_inv;
    write_chunk<WDT, GDT, L2>(d, chunk, shifted_weight<WDT>(d.weight, a.shift), d.exp_avg + a.shift, d.exp_avg_sq + a.shift,
                              d.saved[0], g_si, d.saved[1], d.saved[2], *d.w_scale, *d.m_scale, *d.v_scale, k);
}

static int adam_grid(size_t n) {
    size_t blocks = (n + kAdamThreads * 4 - 1) / (kAdamThreads * 4);
    size_t cap = static_cast<size_t>(cu_count()) * 8;
    if (blocks < 1) blocks = 1;
    return static_cast<int>(blocks < cap ? blocks : cap);
}

static bool state_dt_ok(int dt) {
    return dt == MSAMP_DT_E4M3 || dt == MSAMP_DT_E5M2 || dt == MSAMP_DT_F16 || dt == MSAMP_DT_F32;
}

// call F<MDT, VDT>() for the runtime pair
#define MSAMP_STATE_SWITCH(mdt, vdt, ...)                                 \
    switch (mdt) {                                                          \
        case MSAMP_DT_E4M3: { constexpr int MDT = MSAMP_DT_E4M3; MSAMP_STATE_SWITCH_V(vdt, __VA_ARGS__) } break; \
        case MSAMP_DT_E5M2: { constexpr int MDT = MSAMP_DT_E5M2; MSAMP_STATE_SWITCH_V(vdt, __VA_ARGS__) } break; \
        case MSAMP_DT_F16: { constexpr int MDT = MSAMP_DT_F16; MSAMP_STATE_SWITCH_V(vdt, __VA_ARGS__) } break;   \
        default: { constexpr int MDT = MSAMP_DT_F32; MSAMP_STATE_SWITCH_V(vdt, __VA_ARGS__) } break;             \
    }
#define MSAMP_STATE_SWITCH_V(vdt, ...)                                    \
    switch (vdt) {                                                          \
        case MSAMP_DT_E4M3: { constexpr int VDT = MSAMP_DT_E4M3; __VA_ARGS__ } break; \
        case MSAMP_DT_E5M2: { constexpr int VDT = MSAMP_DT_E5M2; __VA_ARGS__ } break; \
        case MSAMP_DT_F16: { constexpr int VDT = MSAMP_DT_F16; __VA_ARGS__ } break;   \
        default: { constexpr int VDT = MSAMP_DT_F32; __VA_ARGS__ } break;             \
    }

// ---- the step for parameters kept in high precision ---------------------------------------------------------------
// Biases, norm weights and the like: a plain float32 / float16 / bfloat16 parameter with a gradient of such a type,
// exp_avg in E4M3 and exp_avg_sq in scaled float16.  The reference (and the per-tensor path here) takes them one by one
// through stage 1, a look at the two amaxs on the host, and stage 2: a dozen launches and two round trips to the host
// per parameter, for tensors of a few thousand elements.  Here one workgroup takes one parameter through both
// stages: m', v', p' with the expressions of the stages, p' stored in the parameter's type, max |m'| and max |v'| over
// the workgroup, the scale rule, and the moments again from the still untouched stored ones with the new scales
// (Adam mode: without the L2 term, as stage 2 has it).  Uses the weight, grad, exp_avg, exp_avg_sq, m_* and v_* fields
// of the descriptor.
template <typename PT, typename GT, bool L2>
__global__ __launch_bounds__(kAdamThreads) void plain_step_kernel(msamp_adamw_tensor* __restrict__ tensors, AdamConsts k) {
    __shared__ uint32_t red[kAdamThreads / kWave];
    __shared__ float s_scales[2];
    msamp_adamw_tensor& d = tensors[blockIdx.x];
    const size_t n = d.numel;
    PT* param = static_cast<PT*>(d.weight);
    const GT* grad = reinterpret_cast<const GT*>(d.grad);
    const float inv_m = 1.0f / *d.m_scale, inv_v = 1.0f / *d.v_scale;
    float mxm = 0.0f, mxv = 0.0f;
    for (size_t i = threadIdx.x; i < n; i += kAdamThreads) {
#pragma clang fp contract(off)
        float pj = Elem<PT>::load(param + i);
        float gj = Elem<GT>::load(grad + i);
        if (k.maximize) gj = -gj;
        if constexpr (L2) {
            gj = fmaf(k.wd, pj, gj);    // torch's add(other, alpha=) on the GPU, which the per-tensor path takes: one rounding
        } else {
            pj = pj * k.decay;
        }
        float m_new, v_new;
        moments(dequant1<MSAMP_DT_E4M3>(d.exp_avg[i]), f16_bits_to_float(d.exp_avg_sq[i]), gj, inv_m, inv_v, k, m_new, v_new);
        mxm = fmaxf(mxm, fabsf(m_new));
        mxv = fmaxf(mxv, fabsf(v_new));
        Elem<PT>::store(param + i, param_update(pj, m_new, v_new, k));
    }
    const uint32_t a = block_max_u32(__float_as_uint(mxm), red);
    const uint32_t b = block_max_u32(__float_as_uint(mxv), red);
    if (threadIdx.x == 0) {
        const float am = __uint_as_float(a), av = __uint_as_float(b);
        const float ms = k.rule_scales ? scale_rule(am, 1.0f, 448.0f, 0) : 1.0f;
        const float vs = k.rule_scales ? scale_rule(av, 1.0f, 65504.0f, 0) : 1.0f;
        s_scales[0] = ms, s_scales[1] = vs;
        *d.m_scale = ms, *d.m_scale_inv = 1.0f / ms, *d.m_amax = am;
        *d.v_scale = vs, *d.v_scale_inv = 1.0f / vs, *d.v_amax = av;
    }
    __syncthreads();
    const float ms = s_scales[0], vs = s_scales[1];
    for (size_t i = threadIdx.x; i < n; i += kAdamThreads) {
        float gj = Elem<GT>::load(grad + i);
        if (k.maximize) gj = -gj;
        float m_new, v_new;
        moments(dequant1<MSAMP_DT_E4M3>(d.exp_avg[i]), f16_bits_to_float(d.exp_avg_sq[i]), gj, inv_m, inv_v, k, m_new, v_new);
        d.exp_avg[i] = static_cast<uint8_t>(quant1<MSAMP_DT_E4M3>(m_new * ms));
        d.exp_avg_sq[i] = static_cast<uint16_t>(float_to_f16_bits(v_new * vs));
    }
}

// The same step for parameters of any size, in three launches over 16 Ki-element chunks (`block_map` as in the fused FP8
// step): stage 1 with its maxima into the descriptors' accumulators, the scale rule per tensor (the old dequantization
// factors are kept in `saved` for the last launch), stage 2.  Payload pointers must be aligned for four elements.
template <typename T>
__device__ __forceinline__ void load4(const T* p, float* f) {
    if constexpr (sizeof(T) == 4) {
        const float4 t = *reinterpret_cast<const float4*>(p);
        f[0] = t.x, f[1] = t.y, f[2] = t.z, f[3] = t.w;
    } else {
        const uint2 t = *reinterpret_cast<const uint2*>(p);
        const T* h = reinterpret_cast<const T*>(&t);
        for (int j = 0; j < 4; ++j) f[j] = Elem<T>::load(h + j);
    }
}
template <typename T>
__device__ __forceinline__ void store4(T* p, const float* f) {
    if constexpr (sizeof(T) == 4) {
        *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
    } else {
        uint2 t;
        T* h = reinterpret_cast<T*>(&t);
        for (int j = 0; j < 4; ++j) Elem<T>::store(h + j, f[j]);
        *reinterpret_cast<uint2*>(p) = t;
    }
}

template <typename PT, typename GT, bool L2>
__device__ __forceinline__ void plain_stage1(float& pj, float gj, float m_old, float v_old, float inv_m, float inv_v,
                                             const AdamConsts& k, float& mxm, float& mxv) {
#pragma clang fp contract(off)
    if (k.maximize) gj = -gj;
    if constexpr (L2) gj = fmaf(k.wd, pj, gj);    // as in plain_step_kernel
    else pj = pj * k.decay;
    float m_new, v_new;
    moments(m_old, v_old, gj, inv_m, inv_v, k, m_new, v_new);
    mxm = fmaxf(mxm, fabsf(m_new));
    mxv = fmaxf(mxv, fabsf(v_new));
    pj = param_update(pj, m_new, v_new, k);
}

template <typename PT, typename GT, bool L2>
__global__ __launch_bounds__(kAdamThreads) void plain_amax_kernel(msamp_adamw_tensor* __restrict__ tensors,
                                                                   const int32_t* __restrict__ block_map, AdamConsts k) {
    __shared__ uint32_t red[kAdamThreads / kWave];
    msamp_adamw_tensor& d = tensors[block_map[2 * blockIdx.x]];
    const size_t n = d.numel, first = static_cast<size_t>(block_map[2 * blockIdx.x + 1]) * MSAMP_ADAMW_CHUNK;
    const size_t last = first + MSAMP_ADAMW_CHUNK < n ? first + MSAMP_ADAMW_CHUNK : n;
    PT* param = static_cast<PT*>(d.weight);
    const GT* grad = reinterpret_cast<const GT*>(d.grad);
    const float inv_m = 1.0f / *d.m_scale, inv_v = 1.0f / *d.v_scale;
    float mxm = 0.0f, mxv = 0.0f;
    for (size_t i = first + threadIdx.x * 4; i < last; i += kAdamThreads * 4) {
        if (i + 4 <= last) {
            float p[4], g[4], m[4];
            load4<PT>(param + i, p);
            load4<GT>(grad + i, g);
            dequant4<MSAMP_DT_E4M3>(*reinterpret_cast<const uint32_t*>(d.exp_avg + i), m[0], m[1], m[2], m[3]);
            const uint2 vv = *reinterpret_cast<const uint2*>(d.exp_avg_sq + i);
            const float v[4] = {f16_bits_to_float(vv.x & 0xffffu), f16_bits_to_float(vv.x >> 16), f16_bits_to_float(vv.y & 0xffffu),
                                f16_bits_to_float(vv.y >> 16)};
#pragma unroll
            for (int j = 0; j < 4; ++j) plain_stage1<PT, GT, L2>(p[j], g[j], m[j], v[j], inv_m, inv_v, k, mxm, mxv);
            store4<PT>(param + i, p);
        } else {
            for (size_t e = i; e < last; ++e) {
                float pj = Elem<PT>::load(param + e);
                plain_stage1<PT, GT, L2>(pj, Elem<GT>::load(grad + e), dequant1<MSAMP_DT_E4M3>(d.exp_avg[e]),
                                         f16_bits_to_float(d.exp_avg_sq[e]), inv_m, inv_v, k, mxm, mxv);
                Elem<PT>::store(param + e, pj);
            }
        }
    }
    const uint32_t a = block_max_u32(__float_as_uint(mxm), red);
    const uint32_t b = block_max_u32(__float_as_uint(mxv), red);
    if (threadIdx.x == 0) {
        atomicMax(&d.acc[1], a);
        atomicMax(&d.acc[2], b);
    }
}

__global__ void plain_scales_kernel(msamp_adamw_tensor* tensors, int n_tensors, int tensor_scale) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_tensors) return;
    msamp_adamw_tensor& d = tensors[t];
    const float am = __uint_as_float(d.acc[1]), av = __uint_as_float(d.acc[2]);
    d.acc[1] = 0u, d.acc[2] = 0u;
    d.saved[1] = 1.0f / *d.m_scale;
    d.saved[2] = 1.0f / *d.v_scale;
    const float ms = tensor_scale ? scale_rule(am, 1.0f, 448.0f, 0) : 1.0f;
    const float vs = tensor_scale ? scale_rule(av, 1.0f, 65504.0f, 0) : 1.0f;
    *d.m_scale = ms, *d.m_scale_inv = 1.0f / ms, *d.m_amax = am;
    *d.v_scale = vs, *d.v_scale_inv = 1.0f / vs, *d.v_amax = av;
}

template <typename GT>
__global__ __launch_bounds__(kAdamThreads) void plain_write_kernel(msamp_adamw_tensor* __restrict__ tensors,
                                                                    const int32_t* __restrict__ block_map, AdamConsts k) {
    msamp_adamw_tensor& d = tensors[block_map[2 * blockIdx.x]];
    const size_t n = d.numel, first = static_cast<size_t>(block_map[2 * blockIdx.x + 1]) * MSAMP_ADAMW_CHUNK;
    const size_t last = first + MSAMP_ADAMW_CHUNK < n ? first + MSAMP_ADAMW_CHUNK : n;
    const GT* grad = reinterpret_cast<const GT*>(d.grad);
    const float inv_m = d.saved[1], inv_v = d.saved[2], ms = *d.m_scale, vs = *d.v_scale;
    for (size_t i = first + threadIdx.x * 4; i < last; i += kAdamThreads * 4) {
        if (i + 4 <= last) {
            float g[4], m[4], mn[4], vn[4];
            load4<GT>(grad + i, g);
            dequant4<MSAMP_DT_E4M3>(*reinterpret_cast<const uint32_t*>(d.exp_avg + i), m[0], m[1], m[2], m[3]);
            const uint2 vv = *reinterpret_cast<const uint2*>(d.exp_avg_sq + i);
            const float v[4] = {f16_bits_to_float(vv.x & 0xffffu), f16_bits_to_float(vv.x >> 16), f16_bits_to_float(vv.y & 0xffffu),
                                f16_bits_to_float(vv.y >> 16)};
#pragma unroll
            for (int j = 0; j < 4; ++j) moments(m[j], v[j], k.maximize ? -g[j] : g[j], inv_m, inv_v, k, mn[j], vn[j]);
            *reinterpret_cast<uint32_t*>(d.exp_avg + i) = quant4<MSAMP_DT_E4M3>(mn[0] * ms, mn[1] * ms, mn[2] * ms, mn[3] * ms);
            uint2 out;
            out.x = float_to_f16_bits(vn[0] * vs) | (float_to_f16_bits(vn[1] * vs) << 16);
            out.y = float_to_f16_bits(vn[2] * vs) | (float_to_f16_bits(vn[3] * vs) << 16);
            *reinterpret_cast<uint2*>(d.exp_avg_sq + i) = out;
        } else {
            for (size_t e = i; e < last; ++e) {
                const float gj = Elem<GT>::load(grad + e);
                float m_new, v_new;
                moments(dequant1<MSAMP_DT_E4M3>(d.exp_avg[e]), f16_bits_to_float(d.exp_avg_sq[e]), k.maximize ? -gj : gj, inv_m, inv_v, k,
                        m_new, v_new);
                d.exp_avg[e] = static_cast<uint8_t>(quant1<MSAMP_DT_E4M3>(m_new * ms));
                d.exp_avg_sq[e] = static_cast<uint16_t>(float_to_f16_bits(v_new * vs));
            }
        }
    }
}

// ---- float32 moments ------------------------------------------------------------------------------------------------
// The branch of LBAdamW.adamw_fn for float32 exp_avg / exp_avg_sq (msamp/optim/adamw.py:200-232) is a chain of a dozen
// element-wise torch calls per parameter; this kernel is that chain in one pass, with every intermediate rounded where
// the chain rounds it on the GPU: a.add(b, alpha=c) is one fused multiply-add, a division by a Python number is a
// multiplication by its reciprocal (taken in double, then narrowed), everything else rounds per operation.
// (adamw.cu:20-28, the kernel the reference binds as adamw_compute but never calls, divides by sqrt(bc2) instead.)
struct F32Consts {
    float beta1, omb1, beta2, omb2, inv_sbc2, eps, neg_step, wd, decay;
    int maximize;
};

template <bool L2>
__device__ __forceinline__ void f32_element(float& p, float g, float& m, float& v, const F32Consts& k) {
#pragma clang fp contract(off)
    if (k.maximize) g = -g;
    if constexpr (L2) g = fmaf(k.wd, p, g);
    else p = p * k.decay;    // (1 when there is no decay)
    const float m_scaled = k.beta1 * m;
    m = fmaf(k.omb1, g, m_scaled);
    const float v_scaled = k.beta2 * v;
    const float gg = g * g;
    v = fmaf(k.omb2, gg, v_scaled);
    const float root = sqrtf(v);
    const float q = root * k.inv_sbc2;
    const float denom = q + k.eps;
    const float r = m / denom;
    p = fmaf(k.neg_step, r, p);
}

// VEC: every pointer is aligned for four elements
template <typename GT, bool L2, bool VEC>
__global__ __launch_bounds__(kAdamThreads) void f32_step_kernel(float* __restrict__ param, const GT* __restrict__ grad,
                                                                 float* __restrict__ exp_avg, float* __restrict__ exp_avg_sq,
                                                                 size_t n, F32Consts k) {
    const size_t tid = static_cast<size_t>(blockIdx.x) * kAdamThreads + threadIdx.x;
    const size_t threads = static_cast<size_t>(gridDim.x) * kAdamThreads;
    size_t done = 0;
    if constexpr (VEC) {
        const size_t quads = n / 4;
        for (size_t q = tid; q < quads; q += threads) {
            const size_t i = q * 4;
            float4 p4 = *reinterpret_cast<const float4*>(param + i);
            float4 m4 = *reinterpret_cast<const float4*>(exp_avg + i);
            float4 v4 = *reinterpret_cast<const float4*>(exp_avg_sq + i);
            float g[4];
            load4<GT>(grad + i, g);
            f32_element<L2>(p4.x, g[0], m4.x, v4.x, k);
            f32_element<L2>(p4.y, g[1], m4.y, v4.y, k);
            f32_element<L2>(p4.z, g[2], m4.z, v4.z, k);
            f32_element<L2>(p4.w, g[3], m4.w, v4.w, k);
            *reinterpret_cast<float4*>(param + i) = p4;
            *reinterpret_cast<float4*>(exp_avg + i) = m4;
            *reinterpret_cast<float4*>(exp_avg_sq + i) = v4;
        }
        done = quads * 4;
    }
    for (size_t i = done + tid; i < n; i += threads) {
        float p = param[i], m = exp_avg[i], v = exp_avg_sq[i];
        f32_element<L2>(p, Elem<GT>::load(grad + i), m, v, k);
        param[i] = p, exp_avg[i] = m, exp_avg_sq[i] = v;
    }
}

}    // namespace msamp

using namespace msamp;

extern "C" {

int msamp_adamw_fp8_stage1(float* param, const float* grad, size_t n, const void* exp_avg, int exp_avg_dtype,
                           float exp_avg_factor, float* exp_avg_amax, float beta1, const void* exp_avg_sq,
                           int exp_avg_sq_dtype, float exp_avg_sq_factor, float* exp_avg_sq_amax, float beta2,
                           float eps, int step, float lr, int bias_correction, msamp_stream_t stream) {
    MSAMP_REQUIRE(state_dt_ok(exp_avg_dtype) && state_dt_ok(exp_avg_sq_dtype), MSAMP_ERR_DTYPE,
                  "msamp_adamw_fp8_stage1: state dtypes %d/%d", exp_avg_dtype, exp_avg_sq_dtype);
    MSAMP_REQUIRE(exp_avg_amax && exp_avg_sq_amax, MSAMP_ERR_NULL, "msamp_adamw_fp8_stage1: null amax");
    if (n == 0) return MSAMP_OK;
    MSAMP_REQUIRE(param && grad && exp_avg && exp_avg_sq, MSAMP_ERR_NULL, "msamp_adamw_fp8_stage1: null pointer");
    AdamConsts k = {};
    k.beta1 = beta1, k.beta2 = beta2, k.omb1 = 1.0f - beta1, k.omb2 = 1.0f - beta2, k.eps = eps;
    host_consts(lr, beta1, beta2, step, bias_correction, &k.step_size, &k.sbc2);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int grid = adam_grid(n);
    MSAMP_STATE_SWITCH(exp_avg_dtype, exp_avg_sq_dtype, {
        hipLaunchKernelGGL((stage1_kernel<MDT, VDT>), dim3(grid), dim3(kAdamThreads), 0, st, param, grad, n,
                           static_cast<const typename State<MDT>::T*>(exp_avg), exp_avg_factor, exp_avg_amax,
                           static_cast<const typename State<VDT>::T*>(exp_avg_sq), exp_avg_sq_factor, exp_avg_sq_amax, k);
    })
    MSAMP_CHECK_LAUNCH("stage1_kernel");
    return MSAMP_OK;
}

int msamp_adamw_fp8_stage2(const float* grad, size_t n, void* exp_avg, int exp_avg_dtype, float exp_avg_factor,
                           float new_exp_avg_factor, float beta1, void* exp_avg_sq, int exp_avg_sq_dtype,
                           float exp_avg_sq_factor, float new_exp_avg_sq_factor, float beta2, msamp_stream_t stream) {
    MSAMP_REQUIRE(state_dt_ok(exp_avg_dtype) && state_dt_ok(exp_avg_sq_dtype), MSAMP_ERR_DTYPE,
                  "msamp_adamw_fp8_stage2: state dtypes %d/%d", exp_avg_dtype, exp_avg_sq_dtype);
    if (n == 0) return MSAMP_OK;
    MSAMP_REQUIRE(grad && exp_avg && exp_avg_sq, MSAMP_ERR_NULL, "msamp_adamw_fp8_stage2: null pointer");
    AdamConsts k = {};
    k.beta1 = beta1, k.beta2 = beta2, k.omb1 = 1.0f - beta1, k.omb2 = 1.0f - beta2;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int grid = adam_grid(n);
    MSAMP_STATE_SWITCH(exp_avg_dtype, exp_avg_sq_dtype, {
        hipLaunchKernelGGL((stage2_kernel<MDT, VDT>), dim3(grid), dim3(kAdamThreads), 0, st, grad, n,
                           static_cast<typename State<MDT>::T*>(exp_avg), exp_avg_factor, new_exp_avg_factor,
                           static_cast<typename State<VDT>::T*>(exp_avg_sq), exp_avg_sq_factor, new_exp_avg_sq_factor, k);
    })
    MSAMP_CHECK_LAUNCH("stage2_kernel");
    return MSAMP_OK;
}

// hyper-parameters of the fused step, narrowed the way the reference narrows them; returns whether the decay is an
// L2 term on the gradient (Adam mode)
static bool fused_consts(double lr, double beta1, double beta2, double eps, double weight_decay, int step,
                         int bias_correction, int adam_mode, int maximize, AdamConsts& k) {
    k = AdamConsts{};
    k.beta1 = static_cast<float>(beta1), k.beta2 = static_cast<float>(beta2);
    k.omb1 = 1.0f - k.beta1, k.omb2 = 1.0f - k.beta2;
    k.eps = static_cast<float>(eps);
    host_consts(static_cast<float>(lr), k.beta1, k.beta2, step, bias_correction, &k.step_size, &k.sbc2);
    k.inv_sbc2 = 1.0f / k.sbc2;
    k.wd = static_cast<float>(weight_decay);
    k.adam_mode = adam_mode, k.maximize = maximize, k.use_decay = weight_decay != 0.0;
    const bool l2 = k.use_decay && adam_mode;    // Adam mode: the decay joins the gradient, the weight is not decayed
    k.decay = (k.use_decay && !adam_mode) ? static_cast<float>(1.0 - lr * weight_decay) : 1.0f;
    // factors of the first pass' bound on |update|, rounded up and widened; a negative eps (the bound assumes
    // eps >= 0) or anything non-finite makes them infinite, and then every element takes the exact chain
    const float inf = std::numeric_limits<float>::infinity();
    const double widen = 1.0 + 4e-6, abs_step = fabs(static_cast<double>(k.step_size));
    k.bound_rsq = k.eps >= 0.0f ? nextafterf(static_cast<float>(abs_step * k.sbc2 * widen), inf) : inf;
    k.bound_eps = k.eps > 0.0f ? nextafterf(static_cast<float>(abs_step / k.eps * widen), inf) : inf;
    if (!(k.bound_rsq >= 0.0f)) k.bound_rsq = inf;
    if (!(k.bound_eps >= 0.0f)) k.bound_eps = inf;
    return l2;
}

static int fused_args_ok(const char* who, const void* tensors, int n_tensors, const void* block_map, int n_blocks,
                         int weight_dtype, int grad_dtype) {
    MSAMP_REQUIRE(n_tensors >= 0 && n_blocks >= 0, MSAMP_ERR_SHAPE, "%s: n_tensors=%d n_blocks=%d", who, n_tensors, n_blocks);
    if (n_tensors == 0 || n_blocks == 0) return MSAMP_OK;
    MSAMP_REQUIRE(tensors && block_map, MSAMP_ERR_NULL, "%s: null pointer", who);
    MSAMP_REQUIRE(weight_dtype == MSAMP_DT_E4M3 || weight_dtype == MSAMP_DT_E5M2 || weight_dtype == MSAMP_DT_F16,
                  MSAMP_ERR_DTYPE, "%s: weight dtype %d", who, weight_dtype);
    MSAMP_REQUIRE(is_fp8(grad_dtype), MSAMP_ERR_DTYPE, "%s: grad dtype %d", who, grad_dtype);
    return MSAMP_OK;
}

// launch KERNEL<weight type, gradient type, l2> for the runtime types
#define FUSED_LAUNCH_WG(KERNEL, NB, W, G, ...)                                                                        \
    do {                                                                                                              \
        if (l2)                                                                                                       \
            hipLaunchKernelGGL((KERNEL<W, G, true>), dim3(NB), dim3(kAdamThreads), 0, st, __VA_ARGS__);               \
        else                                                                                                          \
            hipLaunchKernelGGL((KERNEL<W, G, false>), dim3(NB), dim3(kAdamThreads), 0, st, __VA_ARGS__);              \
    } while (0)
#define FUSED_LAUNCH(KERNEL, NB, ...)                                                                                 \
    do {                                                                                                              \
        if (weight_dtype == MSAMP_DT_E4M3 && grad_dtype == MSAMP_DT_E4M3)                                             \
            FUSED_LAUNCH_WG(KERNEL, NB, MSAMP_DT_E4M3, MSAMP_DT_E4M3, __VA_ARGS__);                                   \
        else if (weight_dtype == MSAMP_DT_E4M3)                                                                       \
            FUSED_LAUNCH_WG(KERNEL, NB, MSAMP_DT_E4M3, MSAMP_DT_E5M2, __VA_ARGS__);                                   \
        else if (weight_dtype == MSAMP_DT_E5M2 && grad_dtype == MSAMP_DT_E4M3)                                        \
            FUSED_LAUNCH_WG(KERNEL, NB, MSAMP_DT_E5M2, MSAMP_DT_E4M3, __VA_ARGS__);                                   \
        else if (weight_dtype == MSAMP_DT_E5M2)                                                                       \
            FUSED_LAUNCH_WG(KERNEL, NB, MSAMP_DT_E5M2, MSAMP_DT_E5M2, __VA_ARGS__);                                   \
        else if (grad_dtype == MSAMP_DT_E4M3)                                                                         \
            FUSED_LAUNCH_WG(KERNEL, NB, MSAMP_DT_F16, MSAMP_DT_E4M3, __VA_ARGS__);                                    \
        else                                                                                                          \
            FUSED_LAUNCH_WG(KERNEL, NB, MSAMP_DT_F16, MSAMP_DT_E5M2, __VA_ARGS__);                                    \
    } while (0)

int msamp_adamw_fp8_fused(msamp_adamw_tensor* tensors, int n_tensors, const int32_t* block_map, int n_blocks,
                          int weight_dtype, int grad_dtype, double lr, double beta1, double beta2, double eps,
                          double weight_decay, int step, int bias_correction, int adam_mode, int maximize,
                          int tensor_scale, const int32_t* blocks_per_tensor, int group_blocks, msamp_stream_t stream) {
    const int rc = fused_args_ok("msamp_adamw_fp8_fused", tensors, n_tensors, block_map, n_blocks, weight_dtype, grad_dtype);
    if (rc != MSAMP_OK || n_tensors == 0 || n_blocks == 0) return rc;
    AdamConsts k;
    const bool l2 = fused_consts(lr, beta1, beta2, eps, weight_decay, step, bias_correction, adam_mode, maximize, k);
    const float w_fp_max = weight_dtype == MSAMP_DT_F16 ? 65504.0f : fp8_max(weight_dtype);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const msamp_adamw_buffers* in_place = nullptr;
    const int32_t* every_tensor = nullptr;
    // Groups of whole tensors, each small enough that what the first pass read (5 B/param) and what
    // the second writes (4 B/param) stay in the 256 MB Infinity Cache: the second pass then re-reads
    // from cache and HBM sees 9 B/param.  Without the per-tensor block counts everything is one group.
    int t0 = 0, b0 = 0;
    while (t0 < n_tensors) {
        int t1 = t0, b1 = b0;
        if (blocks_per_tensor == nullptr || group_blocks <= 0) {
            t1 = n_tensors, b1 = n_blocks;
        } else {
            do {
                b1 += blocks_per_tensor[t1];
                ++t1;
            } while (t1 < n_tensors && b1 - b0 + blocks_per_tensor[t1] <= group_blocks);
        }
        MSAMP_REQUIRE(b1 <= n_blocks, MSAMP_ERR_SHAPE, "msamp_adamw_fp8_fused: blocks_per_tensor exceeds n_blocks");
        const int nb = b1 - b0, nt = t1 - t0;
        if (nb > 0) {
            FUSED_LAUNCH(fused_amax_kernel, nb, tensors, block_map + 2 * b0, k);
            MSAMP_CHECK_LAUNCH("fused_amax_kernel");
        }
        hipLaunchKernelGGL(fused_scales_kernel, dim3((nt + 63) / 64), dim3(64), 0, st, tensors + t0, nt, w_fp_max,
                           tensor_scale, static_cast<int32_t*>(nullptr));
        MSAMP_CHECK_LAUNCH("fused_scales_kernel");
        if (nb > 0) {
            FUSED_LAUNCH(fused_write_kernel, nb, tensors, block_map + 2 * b0, k, in_place, every_tensor);
            MSAMP_CHECK_LAUNCH("fused_write_kernel");
        }
        t0 = t1, b0 = b1;
    }
    return MSAMP_OK;
}

int msamp_adamw_fp8_fused_speculative(msamp_adamw_tensor* tensors, const msamp_adamw_buffers* outputs, int32_t* redo,
                                      int n_tensors, const int32_t* block_map, int n_blocks, int weight_dtype,
                                      int grad_dtype, double lr, double beta1, double beta2, double eps,
                                      double weight_decay, int step, int bias_correction, int adam_mode, int maximize,
                                      int tensor_scale, msamp_stream_t stream) {
    const int rc = fused_args_ok("msamp_adamw_fp8_fused_speculative", tensors, n_tensors, block_map, n_blocks, weight_dtype,
                                 grad_dtype);
    if (rc != MSAMP_OK || n_tensors == 0 || n_blocks == 0) return rc;
    MSAMP_REQUIRE(outputs && redo, MSAMP_ERR_NULL, "msamp_adamw_fp8_fused_speculative: null outputs or redo");
    AdamConsts k;
    const bool l2 = fused_consts(lr, beta1, beta2, eps, weight_decay, step, bias_correction, adam_mode, maximize, k);
    k.rule_scales = tensor_scale != 0;
    const float w_fp_max = weight_dtype == MSAMP_DT_F16 ? 65504.0f : fp8_max(weight_dtype);
    hipStream_t st = static_cast<hipStream_t>(stream);
    FUSED_LAUNCH(fused_spec_kernel, n_blocks, tensors, block_map, k, outputs);
    MSAMP_CHECK_LAUNCH("fused_spec_kernel");
    hipLaunchKernelGGL(fused_scales_kernel, dim3((n_tensors + 63) / 64), dim3(64), 0, st, tensors, n_tensors, w_fp_max,
                       tensor_scale, redo);
    MSAMP_CHECK_LAUNCH("fused_scales_kernel");
    // the tensors whose scales changed, again, with the scales just written; every other workgroup returns at once
    const int32_t* redo_in = redo;
    FUSED_LAUNCH(fused_write_kernel, n_blocks, tensors, block_map, k, outputs, redo_in);
    MSAMP_CHECK_LAUNCH("fused_write_kernel");
    return MSAMP_OK;
}
int msamp_adamw_f32(float* param, const void* grad, int grad_dtype, size_t n, float* exp_avg, float* exp_avg_sq, double lr,
                    double beta1, double beta2, double eps, double weight_decay, int step, int bias_correction, int adam_mode,
                    int maximize, msamp_stream_t stream) {
    if (n == 0) return MSAMP_OK;
    MSAMP_REQUIRE(param && grad && exp_avg && exp_avg_sq, MSAMP_ERR_NULL, "msamp_adamw_f32: null pointer");
    MSAMP_REQUIRE(is_hp(grad_dtype), MSAMP_ERR_DTYPE, "msamp_adamw_f32: grad dtype %d", grad_dtype);
    // the Python numbers of the chain, each narrowed where torch narrows it (to the tensors' float32)
    const double bc1 = bias_correction ? 1.0 - pow(beta1, step) : 1.0;
    const double bc2 = bias_correction ? 1.0 - pow(beta2, step) : 1.0;
    F32Consts k;
    k.beta1 = static_cast<float>(beta1), k.omb1 = static_cast<float>(1.0 - beta1);
    k.beta2 = static_cast<float>(beta2), k.omb2 = static_cast<float>(1.0 - beta2);
    k.inv_sbc2 = static_cast<float>(1.0 / sqrt(bc2));
    k.eps = static_cast<float>(eps);
    k.neg_step = static_cast<float>(-(lr / bc1));
    k.wd = static_cast<float>(weight_decay);
    const bool l2 = weight_decay != 0.0 && adam_mode;
    k.decay = (weight_decay != 0.0 && !adam_mode) ? static_cast<float>(1.0 - lr * weight_decay) : 1.0f;
    k.maximize = maximize;
    const size_t grad_bytes = grad_dtype == MSAMP_DT_F32 ? 4 : 2;
    const bool vec = (reinterpret_cast<uintptr_t>(param) | reinterpret_cast<uintptr_t>(exp_avg) |
                      reinterpret_cast<uintptr_t>(exp_avg_sq)) % 16 == 0 && reinterpret_cast<uintptr_t>(grad) % (4 * grad_bytes) == 0;
    const size_t per_group = static_cast<size_t>(kAdamThreads) * 4;
    const int grid = static_cast<int>(std::min<size_t>((n + per_group - 1) / per_group, static_cast<size_t>(cu_count()) * 16));
    hipStream_t st = static_cast<hipStream_t>(stream);
#define F32_LAUNCH(GT, L2V, VECV)                                                                                          \
    hipLaunchKernelGGL((f32_step_kernel<GT, L2V, VECV>), dim3(grid), dim3(kAdamThreads), 0, st, param, static_cast<const GT*>(grad), \
                       exp_avg, exp_avg_sq, n, k)
#define F32_FORMS(GT)                                 \
    do {                                              \
        if (l2 && vec) F32_LAUNCH(GT, true, true);    \
        else if (l2) F32_LAUNCH(GT, true, false);     \
        else if (vec) F32_LAUNCH(GT, false, true);    \
        else F32_LAUNCH(GT, false, false);            \
    } while (0)
    if (grad_dtype == MSAMP_DT_F32) F32_FORMS(float);
    else if (grad_dtype == MSAMP_DT_F16) F32_FORMS(f16_t);
    else F32_FORMS(bf16_t);
#undef F32_FORMS
#undef F32_LAUNCH
    MSAMP_CHECK_LAUNCH("f32_step_kernel");
    return MSAMP_OK;
}

int msamp_adamw_plain_fused(msamp_adamw_tensor* tensors, int n_tensors, const int32_t* block_map, int n_blocks, int param_dtype,
                            int grad_dtype, double lr, double beta1, double beta2, double eps, double weight_decay, int step,
                            int bias_correction, int adam_mode, int maximize, int tensor_scale, msamp_stream_t stream) {
    MSAMP_REQUIRE(n_tensors >= 0 && n_blocks >= 0, MSAMP_ERR_SHAPE, "msamp_adamw_plain_fused: n_tensors=%d n_blocks=%d", n_tensors,
                  n_blocks);
    if (n_tensors == 0 || (block_map && n_blocks == 0)) return MSAMP_OK;
    MSAMP_REQUIRE(tensors, MSAMP_ERR_NULL, "msamp_adamw_plain_fused: null pointer");
    MSAMP_REQUIRE(is_hp(param_dtype) && is_hp(grad_dtype), MSAMP_ERR_DTYPE, "msamp_adamw_plain_fused: dtypes %d, %d", param_dtype,
                  grad_dtype);
    AdamConsts k;
    const bool l2 = fused_consts(lr, beta1, beta2, eps, weight_decay, step, bias_correction, adam_mode, maximize, k);
    k.rule_scales = tensor_scale != 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // block_map == NULL: one workgroup per tensor, one launch
#define PLAIN_LAUNCH(PT, GT)                                                                                                    \
    do {                                                                                                                        \
        if (!block_map) {                                                                                                       \
            if (l2) hipLaunchKernelGGL((plain_step_kernel<PT, GT, true>), dim3(n_tensors), dim3(kAdamThreads), 0, st, tensors, k);   \
            else hipLaunchKernelGGL((plain_step_kernel<PT, GT, false>), dim3(n_tensors), dim3(kAdamThreads), 0, st, tensors, k);     \
        } else {                                                                                                                \
            if (l2) hipLaunchKernelGGL((plain_amax_kernel<PT, GT, true>), dim3(n_blocks), dim3(kAdamThreads), 0, st, tensors, block_map, k);  \
            else hipLaunchKernelGGL((plain_amax_kernel<PT, GT, false>), dim3(n_blocks), dim3(kAdamThreads), 0, st, tensors, block_map, k);    \
            hipLaunchKernelGGL(plain_scales_kernel, dim3((n_tensors + 63) / 64), dim3(64), 0, st, tensors, n_tensors, tensor_scale);  \
            hipLaunchKernelGGL((plain_write_kernel<GT>), dim3(n_blocks), dim3(kAdamThreads), 0, st, tensors, block_map, k);     \
        }                                                                                                                       \
    } while (0)
#define PLAIN_GRAD(PT)                                                   \
    do {                                                                 \
        if (grad_dtype == MSAMP_DT_F32) PLAIN_LAUNCH(PT, float);         \
        else if (grad_dtype == MSAMP_DT_F16) PLAIN_LAUNCH(PT, f16_t);    \
        else PLAIN_LAUNCH(PT, bf16_t);                                   \
    } while (0)
    if (param_dtype == MSAMP_DT_F32) PLAIN_GRAD(float);
    else if (param_dtype == MSAMP_DT_F16) PLAIN_GRAD(f16_t);
    else PLAIN_GRAD(bf16_t);
#undef PLAIN_GRAD
#undef PLAIN_LAUNCH
    MSAMP_CHECK_LAUNCH("msamp_adamw_plain_fused");
    return MSAMP_OK;
}

int msamp_adamw_fp8_fused_shift(msamp_adamw_tensor* tensors, int32_t* redo, void* sync, int n_tensors, const int32_t* block_map,
                                int n_blocks, long long shift_elems, int weight_dtype, int grad_dtype, double lr, double beta1,
                                double beta2, double eps, double weight_decay, int step, int bias_correction, int adam_mode,
                                int maximize, int tensor_scale, void* workspace, msamp_stream_t stream) {
    const int rc = fused_args_ok("msamp_adamw_fp8_fused_shift", tensors, n_tensors, block_map, n_blocks, weight_dtype, grad_dtype);
    if (rc != MSAMP_OK || n_tensors == 0 || n_blocks == 0) return rc;
    MSAMP_REQUIRE(redo != nullptr && sync != nullptr, MSAMP_ERR_NULL, "msamp_adamw_fp8_fused_shift: null redo or sync");
    MSAMP_REQUIRE(aligned(sync, 8), MSAMP_ERR_ALIGNMENT, "msamp_adamw_fp8_fused_shift: sync must be 8-byte aligned");
    MSAMP_REQUIRE(workspace != nullptr, MSAMP_ERR_WORKSPACE, "msamp_adamw_fp8_fused_shift: workspace required");
    const long long mag = shift_elems < 0 ? -shift_elems : shift_elems;
    MSAMP_REQUIRE(mag > 0 && mag % MSAMP_ADAMW_CHUNK == 0 && mag / MSAMP_ADAMW_CHUNK <= 0x7fffffffLL, MSAMP_ERR_SHAPE,
                  "msamp_adamw_fp8_fused_shift: shift_elems=%lld must be a non-zero multiple of %d", shift_elems, MSAMP_ADAMW_CHUNK);
    AdamConsts k;
    const bool l2 = fused_consts(lr, beta1, beta2, eps, weight_decay, step, bias_correction, adam_mode, maximize, k);
    hipStream_t st = static_cast<hipStream_t>(stream);
    ShiftArgs a;
    a.shift = shift_elems;
    a.slack = static_cast<int>(mag / MSAMP_ADAMW_CHUNK);
    a.lead = a.slack / 2 < 512 ? a.slack / 2 : 512;
    a.n_chunks = n_blocks;
    a.n_tensors = n_tensors;
    a.token = next_tokens(1);
    a.spin_limit = collector_spin_limit();
    a.error_word = static_cast<uint32_t*>(workspace) + kWsErrorWord;
    a.redo = redo;
    a.posts = static_cast<uint64_t*>(sync);
    a.verdicts = a.posts + static_cast<size_t>(n_tensors) * kShiftPostWords;
    a.marks = a.verdicts + n_blocks;
    a.w_fp_max = weight_dtype == MSAMP_DT_F16 ? 65504.0f : fp8_max(weight_dtype);
    a.tensor_scale = tensor_scale;
    FUSED_LAUNCH(fused_shift_kernel, n_blocks, tensors, block_map, k, a);
    MSAMP_CHECK_LAUNCH("fused_shift_kernel");
    hipLaunchKernelGGL(fused_shift_scales_kernel, dim3(n_tensors), dim3(kAdamThreads), 0, st, tensors, block_map, a);
    MSAMP_CHECK_LAUNCH("fused_shift_scales_kernel");
    const int tail = n_blocks < a.slack ? n_blocks : a.slack;
    FUSED_LAUNCH(fused_shift_tail_kernel, tail, tensors, block_map, k, a);
    MSAMP_CHECK_LAUNCH("fused_shift_tail_kernel");
    return MSAMP_OK;
}
#undef FUSED_LAUNCH
#undef FUSED_LAUNCH_WG

}    // extern "C"
