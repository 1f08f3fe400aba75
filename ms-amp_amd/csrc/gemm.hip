// C entry points of the FP8 GEMM: D[N][M] = (B[N][K] . A[M][K]^T) * a_scale_inv * b_scale_inv (+bias) (+D).
// The kernels live in gemm_kernels.cuh and are compiled once per pair of operand formats (gemm_inst.hip); this
// file checks the arguments and hands the call over.  Inside the kernels the operand that supplies D's rows is
// X (= B of the API, N rows) and the one that supplies D's columns is Y (= A of the API, M rows).
#include "gemm_call.h"

#include <algorithm>
#include <atomic>
#include <map>
#include <mutex>
#include <tuple>

namespace msamp {

static int dispatch_pair(int x_type, int y_type, const GemmCall& c) {
    if (x_type == MSAMP_DT_E4M3 && y_type == MSAMP_DT_E4M3) return run_gemm_pair<MSAMP_DT_E4M3, MSAMP_DT_E4M3>(c);
    if (x_type == MSAMP_DT_E4M3) return run_gemm_pair<MSAMP_DT_E4M3, MSAMP_DT_E5M2>(c);
    if (y_type == MSAMP_DT_E4M3) return run_gemm_pair<MSAMP_DT_E5M2, MSAMP_DT_E4M3>(c);
    return run_gemm_pair<MSAMP_DT_E5M2, MSAMP_DT_E5M2>(c);
}

// K-major operands: only the direct-to-LDS kernel reads them, so the shape must suit it
static bool kmajor_shape_ok(int NR, int NC, int K, bool xt, bool yt) {
    const bool fits32 = static_cast<unsigned long long>(NR) * K < (1ull << 32) && static_cast<unsigned long long>(NC) * K < (1ull << 32);
    return K % kBK == 0 && K >= 2 * kBK && fits32 && (!xt || NR % kDmaTile == 0) && (!yt || NC % kDmaTile == 0);
}

// tile walks registered per problem (kernel-side naming: NR x NC output, K, which operands are K-major)
static std::mutex g_walk_mutex;
static std::map<std::tuple<int, int, int, int>, int> g_walks;
static thread_local int t_forced_walk = -2;    // -2: none; msamp_fp8_gemm_tune times its candidates through this
int registered_walk(int NR, int NC, int K, bool XT, bool YT) {
    if (t_forced_walk != -2) return t_forced_walk;
    std::lock_guard<std::mutex> lock(g_walk_mutex);
    if (g_walks.empty()) return -1;
    const auto it = g_walks.find(std::make_tuple(NR, NC, K, (XT ? 1 : 0) | (YT ? 2 : 0)));
    return it == g_walks.end() ? -1 : it->second;
}

static std::atomic<int> g_small_tile_limit{128};
int small_tile_limit() { return g_small_tile_limit.load(std::memory_order_relaxed); }

}    // namespace msamp

using namespace msamp;

extern "C" void msamp_set_small_tile_limit(int big_tiles) {
    msamp::g_small_tile_limit.store(big_tiles < 0 ? 0 : big_tiles, std::memory_order_relaxed);
}

extern "C" int msamp_fp8_gemm_set_walk(int m, int n, int k, int a_kmajor, int b_kmajor, int walk) {
    MSAMP_REQUIRE(walk >= -1 && walk <= 7, MSAMP_ERR_SHAPE, "msamp_fp8_gemm_set_walk: walk=%d", walk);
    // X = b (n rows of D), Y = a (m columns of D)
    const auto key = std::make_tuple(n, m, k, (b_kmajor ? 1 : 0) | (a_kmajor ? 2 : 0));
    std::lock_guard<std::mutex> lock(msamp::g_walk_mutex);
    if (walk < 0) msamp::g_walks.erase(key);
    else msamp::g_walks[key] = walk;
    return MSAMP_OK;
}

extern "C" int msamp_fp8_gemm_get_walk(int m, int n, int k, int a_kmajor, int b_kmajor) {
    std::lock_guard<std::mutex> lock(msamp::g_walk_mutex);
    const auto it = msamp::g_walks.find(std::make_tuple(n, m, k, (b_kmajor ? 1 : 0) | (a_kmajor ? 2 : 0)));
    return it == msamp::g_walks.end() ? -1 : it->second;
}

extern "C" int msamp_fp8_gemm_tune(const uint8_t* a, int a_type, const float* a_scale_inv, int a_kmajor, const uint8_t* b,
                                   int b_type, const float* b_scale_inv, int b_kmajor, void* d, int d_dtype, int m, int n,
                                   int k, const void* bias, int bias_dtype, int* chosen, msamp_stream_t stream) {
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto run = [&]() {
        return msamp_fp8_gemm_kmajor(a, a_type, a_scale_inv, a_kmajor, b, b_type, b_scale_inv, b_kmajor, d, d_dtype, m, n, k, 0, bias,
                                     bias_dtype, stream);
    };
    if (chosen) *chosen = -1;
    // Only problems of the 256 x 256-tile kernel with at least two rounds of tiles have a walk worth timing, and timing
    // needs a stream that is not being captured; everything else is the plain product.
    const long tiles = (static_cast<long>(n) + kDmaTile - 1) / kDmaTile * ((static_cast<long>(m) + kDmaTile - 1) / kDmaTile);
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &capturing) != hipSuccess) capturing = hipStreamCaptureStatusActive, (void)hipGetLastError();
    const bool candidate = m > 0 && n > 0 && k >= 4 * kBK && k % kBK == 0 && tiles >= 2L * cu_count() && !takes_small_tiles(n, m, k) &&
                           capturing == hipStreamCaptureStatusNone;
    if (!candidate) return run();
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        if (e0) (void)hipEventDestroy(e0);
        (void)hipGetLastError();
        return run();
    }
    // the rule's walk first and last, the four explicit ones between: two untimed launches, then as many as fill about four
    // milliseconds (at least four) between one pair of events
    float best_ms = 0.0f, rule_ms = 0.0f;
    int best = -1, rc = MSAMP_OK;
    // (row-major operands: the fastest of the four once more with split waits, bit 2)
    const bool can_split = !a_kmajor && !b_kmajor;
    float explicit_ms[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const int turns = can_split ? 7 : 6;
    for (int turn = 0; turn < turns && rc == MSAMP_OK; ++turn) {
        int walk = turn - 1;
        if (turn == turns - 1) walk = -1;    // (the rule's walk once more at the end: a cold start must not cost it the comparison)
        else if (turn == 5) walk = 4 + static_cast<int>(std::min_element(explicit_ms, explicit_ms + 4) - explicit_ms);
        msamp::t_forced_walk = walk;
        for (int i = 0; i < 2 && rc == MSAMP_OK; ++i) rc = run();
        int reps = 4;
        if (walk >= 0 && rule_ms > 0.0f) reps = std::max(4, std::min(64, static_cast<int>(4.0f / rule_ms)));
        if (rc == MSAMP_OK && hipEventRecord(e0, st) != hipSuccess) rc = MSAMP_ERR_HIP;
        for (int i = 0; i < reps && rc == MSAMP_OK; ++i) rc = run();
        float ms = 0.0f;
        if (rc == MSAMP_OK && (hipEventRecord(e1, st) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
                               hipEventElapsedTime(&ms, e0, e1) != hipSuccess))
            rc = MSAMP_ERR_HIP;
        ms /= reps;
        if (walk >= 0 && walk < 4) explicit_ms[walk] = ms;
        if (turn == 0) rule_ms = best_ms = ms;
        else if (walk < 0) rule_ms = std::min(rule_ms, ms);
        else if (ms < best_ms) best_ms = ms, best = walk;
    }
    msamp::t_forced_walk = -2;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc != MSAMP_OK) {
        (void)hipGetLastError();
        return run();
    }
    // an explicit walk is kept only where it beats the rule's by more than the timing's noise
    if (best >= 0 && best_ms > 0.95f * rule_ms) best = -1;
    msamp_fp8_gemm_set_walk(m, n, k, a_kmajor, b_kmajor, best);
    if (chosen) *chosen = best;
    return MSAMP_OK;    // (d holds the product: every timed launch wrote it)
}

// words of the workspace that the speculative form of msamp_fp8_gemm_cast uses: running maximum, ticket counter (both
// left at zero by every call) and the flag its second launch reads
constexpr int kWsGemmSpec = 10;

extern "C" int msamp_fp8_gemm_cast(const uint8_t* a, int a_type, const float* a_scale_inv, int a_kmajor, const uint8_t* b,
                                   int b_type, const float* b_scale_inv, int b_kmajor, void* d, int d_dtype, int accumulate,
                                   uint8_t* q, int q_type, float* scale, float* amax, float* scale_inv, int m, int n, int k,
                                   int margin, int flags, void* workspace, msamp_stream_t stream) {
    MSAMP_REQUIRE(is_fp8(a_type) && is_fp8(b_type) && is_fp8(q_type), MSAMP_ERR_DTYPE, "msamp_fp8_gemm_cast: types %d, %d -> %d",
                  a_type, b_type, q_type);
    MSAMP_REQUIRE(is_hp(d_dtype), MSAMP_ERR_DTYPE, "msamp_fp8_gemm_cast: intermediate dtype %d", d_dtype);
    MSAMP_REQUIRE(m > 0 && n > 0 && k > 0, MSAMP_ERR_SHAPE, "msamp_fp8_gemm_cast: m=%d n=%d k=%d", m, n, k);
    MSAMP_REQUIRE(a && b && q && a_scale_inv && b_scale_inv && scale && amax && scale_inv, MSAMP_ERR_NULL,
                  "msamp_fp8_gemm_cast: null pointer");
    MSAMP_REQUIRE(!accumulate || d != nullptr, MSAMP_ERR_NULL, "msamp_fp8_gemm_cast: accumulate needs d");
    MSAMP_REQUIRE(aligned(a, 16) && aligned(b, 16) && aligned(q, 16) && aligned(d, 16), MSAMP_ERR_ALIGNMENT,
                  "msamp_fp8_gemm_cast: operands and outputs must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool both = a_kmajor && b_kmajor, neither = !a_kmajor && !b_kmajor;
    const long tiles = static_cast<long>(n / kDmaTile) * (m / kDmaTile);
    const bool fits32 = static_cast<unsigned long long>(n) * k < (1ull << 32) && static_cast<unsigned long long>(m) * k < (1ull << 32);
    if (q_type != MSAMP_DT_E4M3 || !(both || neither) || m % kDmaTile || n % kDmaTile || k % kBK || k < 2 * kBK || !fits32 ||
        workspace == nullptr)
        return MSAMP_NOT_FUSED;
    // A problem small enough for the 128 x 128 tiles is better off with the two steps: both forms below run 256 x 256
    // tiles, a few of them on a few compute units, where the small-tile GEMM and the one-pass cast of its (small) output
    // take less (1024 x 1024 x 8192: 38 against 70 us; 2048 x 2048 x 2048: 22 against 27).
    if (takes_small_tiles(n, m, k)) return MSAMP_NOT_FUSED;
    QuantArgs qa = {};
    qa.q = q, qa.scale = scale, qa.amax = amax, qa.scale_inv = scale_inv;
    qa.slots = reinterpret_cast<uint64_t*>(static_cast<char*>(workspace) + kWsSlotBytes);
    qa.fp_max = fp8_max(q_type), qa.margin = margin, qa.flags = flags;
    qa.error_word = static_cast<uint32_t*>(workspace) + kWsErrorWord;
    qa.spec_words = static_cast<uint32_t*>(workspace) + kWsGemmSpec;
    // one launch, D never stored: at most one tile per compute unit, on a stream that may run waiting kernels
    if (!accumulate && tiles <= cu_count() && tiles <= kMaxSlots && !(flags & MSAMP_FLAG_TWO_PASS) && waiting_kernels_allowed(st)) {
        qa.token = next_tokens(1);
        qa.spin_limit = collector_spin_limit();
        // X = b (rows of D), Y = a (columns of D)
        const GemmCall c = {b, a, nullptr, d_dtype, n, m, k, b_scale_inv, a_scale_inv, 0, nullptr, 0, both, both, &qa, st};
        const int rc = dispatch_pair(b_type, a_type, c);
        if (rc != MSAMP_NOT_FUSED) return rc;
    }
    if (d == nullptr || (flags & MSAMP_FLAG_NO_SPECULATION)) return MSAMP_NOT_FUSED;
    // on speculation: D and the codes for the scale in force side by side, then (only if the rule arrives at another
    // scale) the cast of D again
    GemmCall c = {b, a, d, d_dtype, n, m, k, b_scale_inv, a_scale_inv, accumulate, nullptr, 0, both, both, &qa, st};
    c.qspec = true;
    const int rc = dispatch_pair(b_type, a_type, c);
    if (rc != MSAMP_OK) return rc;
    return cast_again_if_flagged(d, d_dtype, static_cast<size_t>(n) * m, scale, q, q_type, qa.spec_words + 2, st);
}

extern "C" int msamp_fp8_gemm_kmajor(const uint8_t* a, int a_type, const float* a_scale_inv, int a_kmajor, const uint8_t* b,
                                     int b_type, const float* b_scale_inv, int b_kmajor, void* d, int d_dtype, int m, int n,
                                     int k, int accumulate, const void* bias, int bias_dtype, msamp_stream_t stream) {
    if (!a_kmajor && !b_kmajor)
        return msamp_fp8_gemm(a, a_type, a_scale_inv, b, b_type, b_scale_inv, d, d_dtype, m, n, k, accumulate, bias, bias_dtype, stream);
    MSAMP_REQUIRE(is_fp8(a_type) && is_fp8(b_type), MSAMP_ERR_DTYPE, "msamp_fp8_gemm_kmajor: operand types %d, %d", a_type, b_type);
    MSAMP_REQUIRE(is_hp(d_dtype), MSAMP_ERR_DTYPE, "msamp_fp8_gemm_kmajor: output dtype %d", d_dtype);
    MSAMP_REQUIRE(bias == nullptr || is_hp(bias_dtype), MSAMP_ERR_DTYPE, "msamp_fp8_gemm_kmajor: bias dtype %d", bias_dtype);
    MSAMP_REQUIRE(a_kmajor, MSAMP_ERR_SHAPE, "msamp_fp8_gemm_kmajor: b may be K-major only together with a");
    MSAMP_REQUIRE(m > 0 && n > 0 && k > 0 && kmajor_shape_ok(n, m, k, b_kmajor != 0, true), MSAMP_ERR_SHAPE,
                  "msamp_fp8_gemm_kmajor: m=%d n=%d k=%d (k must be a multiple of 128 and at least 256, the K-major operands' rows multiples of 256)", m, n, k);
    MSAMP_REQUIRE(a && b && d && a_scale_inv && b_scale_inv, MSAMP_ERR_NULL, "msamp_fp8_gemm_kmajor: null pointer");
    MSAMP_REQUIRE(aligned(a, 16) && aligned(b, 16), MSAMP_ERR_ALIGNMENT, "msamp_fp8_gemm_kmajor: operands must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    // X = b (rows of D), Y = a (columns of D)
    const GemmCall c = {b, a, d, d_dtype, n, m, k, b_scale_inv, a_scale_inv, accumulate, bias, bias_dtype, b_kmajor != 0, true, nullptr, st};
    return dispatch_pair(b_type, a_type, c);
}

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
    MSAMP_REQUIRE(aligned(a, 16) && aligned(b, 16), MSAMP_ERR_ALIGNMENT, "msamp_fp8_gemm: operands must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    // X = b (rows of D), Y = a (columns of D)
    const GemmCall c = {b, a, d, d_dtype, n, m, k, b_scale_inv, a_scale_inv, accumulate, bias, bias_dtype, false, false, nullptr, st};
    return dispatch_pair(b_type, a_type, c);
}

// Calibration aid: what the matrix pipes of this device sustain when nothing else moves.  Every wavefront issues
// 16x16x128 FP8 MFMAs on registers it loaded once; the sum is stored only if it equals a value it cannot take, so
// the loop is not optimised away and nothing is written.  FRAGS = 1: the same two operands for every MFMA (the
// operand buses never toggle); FRAGS = 8: eight X and eight Y fragments, every pair once per turn as in a K slice of
// the GEMM, so that consecutive MFMAs see different operands.
namespace msamp {
typedef int mfma_probe_v8i __attribute__((ext_vector_type(8)));
typedef float mfma_probe_v4f __attribute__((ext_vector_type(4)));
template <int FRAGS>
__global__ __launch_bounds__(256) void mfma_probe_kernel(const int* __restrict__ seed, float* __restrict__ sink, int iters) {
    mfma_probe_v8i a[FRAGS], b[FRAGS];
    for (int f = 0; f < FRAGS; ++f)
        for (int i = 0; i < 8; ++i) {
            a[f][i] = seed[(threadIdx.x * 8 + i + f * 37) & 1023];
            b[f][i] = seed[(threadIdx.x * 8 + i + 512 + f * 53) & 1023];
        }
    mfma_probe_v4f acc[16];
    for (int i = 0; i < 16; ++i) acc[i] = mfma_probe_v4f{0, 0, 0, 0};
    constexpr int kTurns = FRAGS == 1 ? 1 : 4;    // 16 or 64 MFMAs per turn of the loop
    for (int it = 0; it < iters; it += kTurns) {
#pragma unroll
        for (int n = 0; n < 16 * kTurns; ++n) {
            const int i = (n / FRAGS) % FRAGS, j = n % FRAGS;
            acc[n % 16] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i], b[j], acc[n % 16], 0, 0, 0, 0, 0, 0);
        }
    }
    float s = 0;
    for (int i = 0; i < 16; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    if (s == 12345.678f) sink[0] = s;
}
}    // namespace msamp

extern "C" int msamp_mfma_probe(const void* seed, float* sink, int iters, int workgroups, int distinct_operands, double* flop,
                                msamp_stream_t stream) {
    MSAMP_REQUIRE(seed && sink, MSAMP_ERR_NULL, "msamp_mfma_probe: null pointer");
    MSAMP_REQUIRE(iters > 0 && iters % 4 == 0 && workgroups > 0 && workgroups <= 65536, MSAMP_ERR_SHAPE,
                  "msamp_mfma_probe: iters=%d (a positive multiple of 4) workgroups=%d", iters, workgroups);
    if (distinct_operands)
        hipLaunchKernelGGL(mfma_probe_kernel<8>, dim3(workgroups), dim3(256), 0, static_cast<hipStream_t>(stream),
                           static_cast<const int*>(seed), sink, iters);
    else
        hipLaunchKernelGGL(mfma_probe_kernel<1>, dim3(workgroups), dim3(256), 0, static_cast<hipStream_t>(stream),
                           static_cast<const int*>(seed), sink, iters);
    if (flop) *flop = 4.0 * workgroups * iters * 16.0 * 2.0 * 16 * 16 * 128;
    MSAMP_CHECK_LAUNCH("msamp_mfma_probe");
    return MSAMP_OK;
}
