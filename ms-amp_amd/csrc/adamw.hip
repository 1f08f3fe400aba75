// FP8 AdamW: the reference-shaped stage-1 / stage-2 entry points on fp32 param/grad, and the fused
// multi-tensor step that works on the quantized tensors directly (5 bytes read, 4 written per
// parameter).  Arithmetic is plain float32, left to right, never contracted into fused
// multiply-adds, so the second pass reproduces the first one bit for bit.
#include "common.cuh"

namespace msamp {

constexpr int kAdamThreads = 256;

struct AdamConsts {
    float beta1, beta2, omb1, omb2, eps, step_size, sbc2, decay, wd;
    int adam_mode, maximize, use_decay;
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

// the element-wise update shared by both passes.  RAW_MOMENTS (write pass): the moments that get
// stored are recomputed from the gradient without the Adam-mode L2 term, as the reference's second
// stage does (msamp/optim/adamw.py:186-199), while p' keeps the term.
template <int NE, bool RAW_MOMENTS>
__device__ __forceinline__ void update(float* p, const float* g_in, float* m, float* v, float w_si, float g_si,
                                       float inv_m, float inv_v, const AdamConsts& k) {
#pragma clang fp contract(off)
#pragma unroll
    for (int j = 0; j < NE; ++j) {
        float pj = p[j] * w_si;
        float gj = g_in[j] * g_si;
        if (k.maximize) gj = -gj;
        const float g_raw = gj;
        if (k.use_decay) {
            if (k.adam_mode) {
                const float t = k.wd * pj;
                gj = gj + t;
            } else {
                pj = pj * k.decay;
            }
        }
        float m_new, v_new;
        moments(m[j], v[j], gj, inv_m, inv_v, k, m_new, v_new);
        p[j] = param_update(pj, m_new, v_new, k);
        if (RAW_MOMENTS && k.use_decay && k.adam_mode) moments(m[j], v[j], g_raw, inv_m, inv_v, k, m_new, v_new);
        m[j] = m_new;
        v[j] = v_new;
    }
}

template <int WDT, int GDT>
__device__ __forceinline__ void load16(const msamp_adamw_tensor& d, size_t i, float* p, float* g, float* m,
                                       float* v) {
    load_w16<WDT>(d.weight, i, p);
    load_w16<GDT>(d.grad, i, g);
    load_w16<MSAMP_DT_E4M3>(d.exp_avg, i, m);
    load_w16<MSAMP_DT_F16>(d.exp_avg_sq, i, v);
}

template <int WDT, int GDT>
__global__ __launch_bounds__(kAdamThreads) void fused_amax_kernel(msamp_adamw_tensor* __restrict__ tensors,
                                                                   const int32_t* __restrict__ block_map,
                                                                   AdamConsts k) {
    __shared__ uint32_t red[kAdamThreads / kWave];
    const int t = block_map[2 * blockIdx.x], chunk = block_map[2 * blockIdx.x + 1];
    msamp_adamw_tensor& d = tensors[t];
    const size_t n = d.numel;
    const size_t base = static_cast<size_t>(chunk) * MSAMP_ADAMW_CHUNK;
    const float w_si = *d.w_scale_inv, g_si = *d.g_scale_inv;
    const float inv_m = 1.0f / *d.m_scale, inv_v = 1.0f / *d.v_scale;
    uint32_t mxp = 0;
    float mxm = 0.0f, mxv = 0.0f;
    if (base + MSAMP_ADAMW_CHUNK <= n) {
#pragma unroll 2
        for (int s = 0; s < kSteps; ++s) {
            const size_t i = base + (static_cast<size_t>(s) * kAdamThreads + threadIdx.x) * kEPT;
            float p[kEPT], g[kEPT], m[kEPT], v[kEPT];
            load16<WDT, GDT>(d, i, p, g, m, v);
            update<kEPT, false>(p, g, m, v, w_si, g_si, inv_m, inv_v, k);
#pragma unroll
            for (int j = 0; j < kEPT; ++j) {
                const uint32_t ab = __float_as_uint(p[j]) & 0x7fffffffu;
                mxp = ab > mxp ? ab : mxp;
                mxm = fmaxf(mxm, fabsf(m[j]));
                mxv = fmaxf(mxv, fabsf(v[j]));
            }
        }
    } else {
        for (size_t i = base + threadIdx.x; i < n; i += kAdamThreads) {
            float p = load_w1<WDT>(d.weight, i), g = load_w1<GDT>(d.grad, i);
            float m = load_w1<MSAMP_DT_E4M3>(d.exp_avg, i), v = load_w1<MSAMP_DT_F16>(d.exp_avg_sq, i);
            update<1, false>(&p, &g, &m, &v, w_si, g_si, inv_m, inv_v, k);
            const uint32_t ab = __float_as_uint(p) & 0x7fffffffu;
            mxp = ab > mxp ? ab : mxp;
            mxm = fmaxf(mxm, fabsf(m));
            mxv = fmaxf(mxv, fabsf(v));
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

__global__ void fused_scales_kernel(msamp_adamw_tensor* tensors, int n_tensors, float w_fp_max, int tensor_scale) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_tensors) return;
    msamp_adamw_tensor& d = tensors[t];
    const float ap = __uint_as_float(d.acc[0]), am = __uint_as_float(d.acc[1]), av = __uint_as_float(d.acc[2]);
    d.acc[0] = 0u, d.acc[1] = 0u, d.acc[2] = 0u;
    d.saved[0] = *d.w_scale_inv;
    d.saved[1] = 1.0f / *d.m_scale;
    d.saved[2] = 1.0f / *d.v_scale;
    const float ws = scale_rule(ap, *d.w_scale, w_fp_max, 0);
    *d.w_scale = ws;
    *d.w_scale_inv = 1.0f / ws;
    *d.w_amax = ap;
    const float ms = tensor_scale ? scale_rule(am, 1.0f, 448.0f, 0) : 1.0f;
    const float vs = tensor_scale ? scale_rule(av, 1.0f, 65504.0f, 0) : 1.0f;
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

template <int WDT, int GDT>
__global__ __launch_bounds__(kAdamThreads) void fused_write_kernel(msamp_adamw_tensor* __restrict__ tensors,
                                                                    const int32_t* __restrict__ block_map,
                                                                    AdamConsts k) {
    const int b = gridDim.x - 1 - blockIdx.x;    // back to front: most recently read chunks first
    const int t = block_map[2 * b], chunk = block_map[2 * b + 1];
    msamp_adamw_tensor& d = tensors[t];
    const size_t n = d.numel;
    const size_t base = static_cast<size_t>(chunk) * MSAMP_ADAMW_CHUNK;
    const float w_si = d.saved[0], g_si = *d.g_scale_inv, inv_m = d.saved[1], inv_v = d.saved[2];
    const float ws = *d.w_scale, ms = *d.m_scale, vs = *d.v_scale;
    if (base + MSAMP_ADAMW_CHUNK <= n) {
#pragma unroll 2
        for (int s = 0; s < kSteps; ++s) {
            const size_t i = base + (static_cast<size_t>(s) * kAdamThreads + threadIdx.x) * kEPT;
            float p[kEPT], g[kEPT], m[kEPT], v[kEPT];
            load16<WDT, GDT>(d, i, p, g, m, v);
            update<kEPT, true>(p, g, m, v, w_si, g_si, inv_m, inv_v, k);
#pragma unroll
            for (int j = 0; j < kEPT; ++j) {
                p[j] *= ws;
                m[j] *= ms;
                v[j] *= vs;
            }
            store_w16<WDT>(d.weight, i, p);
            store_w16<MSAMP_DT_E4M3>(d.exp_avg, i, m);
            store_w16<MSAMP_DT_F16>(d.exp_avg_sq, i, v);
        }
    } else {
        for (size_t i = base + threadIdx.x; i < n; i += kAdamThreads) {
            float p = load_w1<WDT>(d.weight, i), g = load_w1<GDT>(d.grad, i);
            float m = load_w1<MSAMP_DT_E4M3>(d.exp_avg, i), v = load_w1<MSAMP_DT_F16>(d.exp_avg_sq, i);
            update<1, true>(&p, &g, &m, &v, w_si, g_si, inv_m, inv_v, k);
            store_w1<WDT>(d.weight, i, p * ws);
            store_w1<MSAMP_DT_E4M3>(d.exp_avg, i, m * ms);
            store_w1<MSAMP_DT_F16>(d.exp_avg_sq, i, v * vs);
        }
    }
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

int msamp_adamw_fp8_fused(msamp_adamw_tensor* tensors, int n_tensors, const int32_t* block_map, int n_blocks,
                          int weight_dtype, int grad_dtype, double lr, double beta1, double beta2, double eps,
                          double weight_decay, int step, int bias_correction, int adam_mode, int maximize,
                          int tensor_scale, msamp_stream_t stream) {
    MSAMP_REQUIRE(n_tensors >= 0 && n_blocks >= 0, MSAMP_ERR_SHAPE, "msamp_adamw_fp8_fused: n_tensors=%d n_blocks=%d",
                  n_tensors, n_blocks);
    if (n_tensors == 0 || n_blocks == 0) return MSAMP_OK;
    MSAMP_REQUIRE(tensors && block_map, MSAMP_ERR_NULL, "msamp_adamw_fp8_fused: null pointer");
    MSAMP_REQUIRE(weight_dtype == MSAMP_DT_E4M3 || weight_dtype == MSAMP_DT_E5M2 || weight_dtype == MSAMP_DT_F16,
                  MSAMP_ERR_DTYPE, "msamp_adamw_fp8_fused: weight dtype %d", weight_dtype);
    MSAMP_REQUIRE(is_fp8(grad_dtype), MSAMP_ERR_DTYPE, "msamp_adamw_fp8_fused: grad dtype %d", grad_dtype);
    AdamConsts k = {};
    k.beta1 = static_cast<float>(beta1), k.beta2 = static_cast<float>(beta2);
    k.omb1 = 1.0f - k.beta1, k.omb2 = 1.0f - k.beta2;
    k.eps = static_cast<float>(eps);
    host_consts(static_cast<float>(lr), k.beta1, k.beta2, step, bias_correction, &k.step_size, &k.sbc2);
    k.decay = static_cast<float>(1.0 - lr * weight_decay);
    k.wd = static_cast<float>(weight_decay);
    k.adam_mode = adam_mode, k.maximize = maximize, k.use_decay = weight_decay != 0.0;
    const float w_fp_max = weight_dtype == MSAMP_DT_F16 ? 65504.0f : fp8_max(weight_dtype);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define FUSED_LAUNCH(KERNEL)                                                                                          \
    do {                                                                                                              \
        if (weight_dtype == MSAMP_DT_E4M3 && grad_dtype == MSAMP_DT_E4M3)                                             \
            hipLaunchKernelGGL((KERNEL<MSAMP_DT_E4M3, MSAMP_DT_E4M3>), dim3(n_blocks), dim3(kAdamThreads), 0, st, tensors, block_map, k); \
        else if (weight_dtype == MSAMP_DT_E4M3)                                                                       \
            hipLaunchKernelGGL((KERNEL<MSAMP_DT_E4M3, MSAMP_DT_E5M2>), dim3(n_blocks), dim3(kAdamThreads), 0, st, tensors, block_map, k); \
        else if (weight_dtype == MSAMP_DT_E5M2 && grad_dtype == MSAMP_DT_E4M3)                                        \
            hipLaunchKernelGGL((KERNEL<MSAMP_DT_E5M2, MSAMP_DT_E4M3>), dim3(n_blocks), dim3(kAdamThreads), 0, st, tensors, block_map, k); \
        else if (weight_dtype == MSAMP_DT_E5M2)                                                                       \
            hipLaunchKernelGGL((KERNEL<MSAMP_DT_E5M2, MSAMP_DT_E5M2>), dim3(n_blocks), dim3(kAdamThreads), 0, st, tensors, block_map, k); \
        else if (grad_dtype == MSAMP_DT_E4M3)                                                                         \
            hipLaunchKernelGGL((KERNEL<MSAMP_DT_F16, MSAMP_DT_E4M3>), dim3(n_blocks), dim3(kAdamThreads), 0, st, tensors, block_map, k); \
        else                                                                                                          \
            hipLaunchKernelGGL((KERNEL<MSAMP_DT_F16, MSAMP_DT_E5M2>), dim3(n_blocks), dim3(kAdamThreads), 0, st, tensors, block_map, k); \
    } while (0)
    FUSED_LAUNCH(fused_amax_kernel);
    MSAMP_CHECK_LAUNCH("fused_amax_kernel");
    hipLaunchKernelGGL(fused_scales_kernel, dim3((n_tensors + 63) / 64), dim3(64), 0, st, tensors, n_tensors, w_fp_max,
                       tensor_scale);
    MSAMP_CHECK_LAUNCH("fused_scales_kernel");
    FUSED_LAUNCH(fused_write_kernel);
    MSAMP_CHECK_LAUNCH("fused_write_kernel");
#undef FUSED_LAUNCH
    return MSAMP_OK;
}

}    // extern "C"
