/*
 * libmsamp_hip.so -- C ABI of the MI355X (gfx950) FP8 hot path.
 *
 * Every entry point borrows raw device pointers for the duration of the enqueue, allocates
 * nothing, enqueues on the caller's stream and returns without synchronising.  Return value:
 * 0 on success, negative on error (MSAMP_ERR_*); msamp_last_error() gives a thread-local
 * message.  Data-type codes are the reference's QType values
 * (msamp/common/dtype/dtypes.py:30-36).
 *
 * The functions replace, one for one, the native calls the reference makes for this path:
 * the five TransformerEngine extension calls behind
 * msamp/common/utils/transformer_engine_wrapper.py:93-176, the jit-scripted scale rule
 * (msamp/common/tensor/meta.py:37-56), the amax-window update
 * (msamp/optim/optimizer.py:83-108) and the msamp_adamw extension
 * (msamp/optim/adamw.cu:77-153).
 */
#ifndef MSAMP_HIP_H_
#define MSAMP_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* stream handle: a hipStream_t passed as an opaque pointer (NULL = the null stream) */
typedef void* msamp_stream_t;

enum {
    MSAMP_DT_BYTE = 0,
    MSAMP_DT_INT32 = 1,
    MSAMP_DT_F32 = 2,
    MSAMP_DT_F16 = 3,
    MSAMP_DT_BF16 = 4,
    MSAMP_DT_E4M3 = 5,
    MSAMP_DT_E5M2 = 6
};

enum {
    MSAMP_OK = 0,
    MSAMP_ERR_DTYPE = -1,     /* unsupported data type code            */
    MSAMP_ERR_SHAPE = -2,     /* bad size or shape                     */
    MSAMP_ERR_NULL = -3,      /* required pointer is NULL              */
    MSAMP_ERR_WORKSPACE = -4, /* workspace missing or too small        */
    MSAMP_ERR_TIMEOUT = -5,   /* a kernel's bounded wait ran out (msamp_check_async_error) */
    MSAMP_ERR_ALIGNMENT = -6, /* a pointer is not aligned as the entry point requires */
    MSAMP_ERR_HIP = -100      /* -100 - hipError_t of the failing call */
};

/* flags of msamp_cast_to_fp8_intime / msamp_cast_transpose_intime */
enum {
    MSAMP_FLAG_NAN_TO_INF = 1, /* amax: NaN/+Inf -> +Inf before the scale rule (cast.py:37-40, sync=True) */
    MSAMP_FLAG_TWO_PASS = 2,   /* never take the one-pass (register-resident, grid-barrier) kernel */
    MSAMP_FLAG_NO_SPECULATION = 4 /* in-time casts: do not quantize with the old scale before the new one is known */
};

/* bytes of device workspace the amax and in-time entry points (msamp_amax, *_intime) need: partial
 * maxima of a first pass, or the per-workgroup slots through which the one-pass kernel's
 * workgroups meet.  Zero it once after allocating it (every call leaves it ready for the next);
 * calls that share one workspace must be ordered on one stream. */
#define MSAMP_WORKSPACE_BYTES 16384

int msamp_hip_version(void);
const char* msamp_last_error(void);

/* The one-pass in-time cast and the fused GEMM + cast are kernels whose workgroups wait for each other, with a bounded
 * wait.  A wait that runs out cannot be reported by the call that enqueued the kernel: the kernel then leaves a sticky
 * non-zero code in the workspace (and a NaN amax when the collecting workgroup gave up), and this call reports it.  It
 * copies the word to the host -- it SYNCHRONISES `stream` -- and returns MSAMP_OK, or MSAMP_ERR_TIMEOUT after clearing
 * the word; the tensor and meta written by the failed kernel are invalid then, and the caller repeats the operation with
 * MSAMP_FLAG_TWO_PASS.  No counterpart in the reference (its casts have no such kernels). */
int msamp_check_async_error(void* workspace, msamp_stream_t stream);

/* Number of polls after which the collecting workgroup of such a kernel gives up (default 2^20, a fraction of a second;
 * the other workgroups wait four times as long for its post).  0 makes every wait give up at once without polling: a
 * hook for testing the failure path with kernels that still exit normally. */
void msamp_set_spin_limit(uint32_t polls);

/* amax[0] = max|x| over n elements, NaN propagating (torch abs().max(), cast.py:34).
 * dtype: F32/F16/BF16.  workspace: MSAMP_WORKSPACE_BYTES. */
int msamp_amax(const void* x, int dtype, size_t n, float* amax, void* workspace, msamp_stream_t stream);

/* out[i] = rule(amax[i], fallback scale_in[i]) for i < n; the pow-2 scale rule of
 * ScalingMeta.compute_scaling_factor (meta.py:37-56).  scale_in may have 1 element
 * (scale_in_n == 1, broadcast) or n.  out may alias scale_in. */
int msamp_compute_scaling_factor(const float* amax, const float* scale_in, int scale_in_n, float* scale_out, int n,
                                 float fp_max, int margin, msamp_stream_t stream);

/* Delayed-scaling cast: tex.cast_to_fp8 (transformer_engine_wrapper.py:106-120).
 * out[i] = fp8_sat_rne(float(x[i]) * *scale); if amax != NULL: *amax = atomic-max(*amax, max|x|)
 * (NaN elements skipped); if scale_inv != NULL: *scale_inv = 1 / *scale. */
int msamp_cast_to_fp8(const void* x, int in_dtype, size_t n, const float* scale, float* amax, float* scale_inv,
                      uint8_t* out, int fp8_type, msamp_stream_t stream);

/* In-time cast: the whole of TypeCast.cast_to_fp8's in-time branch (cast.py:33-62) --
 * amax[0] = max|x|, *scale = rule(amax[0], *scale, fp_max(fp8_type), margin), quantize,
 * *scale_inv = 1 / *scale.  A tensor of up to 64 MiB (16-byte aligned) is read once by a
 * kernel that holds it in registers while its workgroups agree on the amax; that kernel runs on
 * one stream per device (the first to ask) and can be switched off with MSAMP_FLAG_TWO_PASS or
 * MSAMP_INTIME_MODE=0 in the environment.  Otherwise two passes over x, the second back to
 * front so that it meets the cache lines the first left behind.  Same results either way. */
int msamp_cast_to_fp8_intime(const void* x, int in_dtype, size_t n, float* scale, float* amax, float* scale_inv,
                             uint8_t* out, int fp8_type, int margin, int flags, void* workspace,
                             msamp_stream_t stream);

/* msamp_cast_to_fp8_intime without the workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): it has no counterpart in
 * the reference.  The MSAMP_WORKSPACE_BYTES of scratch live in a static device array inside the library (each GPU
 * the library runs on holds its own copy until the process ends); the call allocates and frees nothing.  Same
 * kernels and same results as msamp_cast_to_fp8_intime.  n above MSAMP_STATIC_MAX_ELEMS is rejected with
 * MSAMP_ERR_SHAPE.  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two
 * streams, two threads) race on it -- order them on one stream. */
#define MSAMP_STATIC_MAX_ELEMS ((size_t)1 << 32)
int msamp_cast_to_fp8_intime_static(const void* x, int in_dtype, size_t n, float* scale, float* amax, float* scale_inv,
                                    uint8_t* out, int fp8_type, int margin, int flags, msamp_stream_t stream);

/* ScalingTensor.cast from a scaled 16/32-bit payload to FP8 (msamp/common/tensor/tensor.py:223-265):
 * x holds value * old_scale and *amax = max|value| is known, so no reduction is needed:
 * s = rule(amax[0], 1, fp_max(fp8_type), margin); out[i] = fp8_sat_rne(float(x[i]) * (s * *old_scale_inv));
 * *scale = s * *old_scale_inv; *scale_inv = 1 / s.  The rest of the new meta can be filled in the same
 * launch: amax_out (nullable) receives amax[0..window), *counter_out (nullable) = 0. */
int msamp_cast_scaled_to_fp8(const void* x, int in_dtype, size_t n, const float* amax, const float* old_scale_inv,
                             float* scale, float* scale_inv, float* amax_out, int window, int32_t* counter_out,
                             uint8_t* out, int fp8_type, int margin, msamp_stream_t stream);

/* TypeCast.cast_to_fp8 with the warm-up test of ScalingMeta.is_in_time_scaling (meta.py:58-72,
 * cast.py:33) taken on the device: while *warmup_counter < window the call is the in-time cast,
 * afterwards the delayed one (stored scale, max|x| folded into amax[0]).  The host needs no copy of
 * the counter, so a training step has no device-to-host synchronisation. */
int msamp_cast_to_fp8_gated(const void* x, int in_dtype, size_t n, float* scale, float* amax, float* scale_inv,
                            uint8_t* out, int fp8_type, int margin, int flags, const int32_t* warmup_counter, int window,
                            void* workspace, msamp_stream_t stream);

/* Arithmetic.add_to_fp8 (msamp/operators/arithmetic/arithmetic.py:15-35, vectorized_pointwise.h:184-301): in place,
 * q <- in-time cast of (T(dequant(q)) + other), T = other's dtype, the sum rounded to T as torch adds two T tensors;
 * amax[0] = max|sum|, *scale by the rule (fallback the old *scale), *scale_inv = 1 / *scale.  Equal, bit for bit, to
 * (q.to(T) + other).cast(qtype, meta) -- the identity the reference's own test demands (tests/operators/
 * test_arithmetic.py:25-42). */
int msamp_add_to_fp8(uint8_t* q, int fp8_type, size_t n, float* scale, float* scale_inv, float* amax, const void* other,
                     int other_dtype, void* workspace, msamp_stream_t stream);

/* tex.cast_from_fp8 (transformer_engine_wrapper.py:123-137): out[i] = otype(float(q[i]) * *scale_inv). */
int msamp_cast_from_fp8(const uint8_t* q, int fp8_type, size_t n, const float* scale_inv, void* out, int out_dtype,
                        msamp_stream_t stream);

/* tex.fused_cast_transpose (transformer_engine_wrapper.py:140-162), any rows/cols (the reference
 * pads to multiples of 16 and slices; the result is the same): out[r][c] and out_t[c][r]. */
int msamp_cast_transpose(const void* x, int in_dtype, int rows, int cols, const float* scale, float* amax,
                         float* scale_inv, uint8_t* out, uint8_t* out_t, int fp8_type, msamp_stream_t stream);

/* in-time variant of the above (cast.py:33-52 with fuse_transpose=True) */
int msamp_cast_transpose_intime(const void* x, int in_dtype, int rows, int cols, float* scale, float* amax,
                                float* scale_inv, uint8_t* out, uint8_t* out_t, int fp8_type, int margin, int flags,
                                void* workspace, msamp_stream_t stream);

/* msamp_cast_transpose with the same device-side warm-up test as msamp_cast_to_fp8_gated. */
int msamp_cast_transpose_gated(const void* x, int in_dtype, int rows, int cols, float* scale, float* amax,
                               float* scale_inv, uint8_t* out, uint8_t* out_t, int fp8_type, int margin, int flags,
                               const int32_t* warmup_counter, int window, void* workspace, msamp_stream_t stream);

/* tex.fp8_transpose (transformer_engine_wrapper.py:165-176): out[c][r] = q[r][c]. */
int msamp_fp8_transpose(const uint8_t* q, int rows, int cols, uint8_t* out, msamp_stream_t stream);

/* Scaled 16/32-bit "ScalingTensor" payloads (cast.py:68-95,122-136):
 * out[i] = otype(float(x[i]) * *scale) with IEEE overflow (no saturation). */
int msamp_scale_cast(const void* x, int in_dtype, size_t n, const float* scale, void* out, int out_dtype,
                     msamp_stream_t stream);

/* LBOptimizer._update_scaling_factors (optimizer.py:83-108) on flattened metas: scales (n),
 * amaxs (n x window, row-major).  A non-finite amaxs[i][0] is dropped, the scale comes from the
 * window maximum, the window shifts.  bad[i] (nullable, n bytes) = 1 where amaxs[i][0] was not
 * finite; counters[i] (nullable, n int32 on the device) += 1, or = 0 where bad. */
int msamp_scale_update(float* scales, float* amaxs, uint8_t* bad, int32_t* counters, int n, int window, float fp_max,
                       int margin, msamp_stream_t stream);

/* The same for several groups of metas in one launch -- the optimizer updates the `input` and the `ograd`
 * group (different formats, possibly different windows) once per step (optimizer.py:75-82 loops over them).
 * `groups` is a HOST array of n_groups <= MSAMP_MAX_SCALE_GROUPS descriptors whose pointers are device
 * pointers with the meaning they have above. */
#define MSAMP_MAX_SCALE_GROUPS 4
typedef struct msamp_scale_group {
    float* scales;
    float* amaxs;
    uint8_t* bad;         /* nullable */
    int32_t* counters;    /* nullable */
    int32_t n;
    int32_t window;
    float fp_max;
    int32_t reserved;
} msamp_scale_group;
int msamp_scale_update_groups(const msamp_scale_group* groups, int n_groups, int margin, msamp_stream_t stream);

/* ---- a bucket of gradients into one flat FP8 buffer -------------------------------------------------
 * The compute steps of the FP8 gradient reducer (nn/distributed.py:143-184) for all tensors of a bucket at
 * once; the two collectives between and after them are the caller's.  `items` is a DEVICE array of
 * descriptors (acc is scratch: zero it once, the library leaves it zero), `block_map` a DEVICE array of
 * n_blocks {item index, chunk index} int32 pairs, chunks of MSAMP_BUCKET_CHUNK elements, every chunk of every
 * item listed once.  in_dtype: F32/F16/BF16 for all items. */
#define MSAMP_BUCKET_CHUNK 16384
typedef struct msamp_bucket_item {
    const void* src;     /* the gradient, in_dtype                                             */
    uint8_t* dst;        /* where its FP8 codes go inside the flat buffer                       */
    float* amax;         /* meta.amax[0]                                                        */
    float* scale;        /* meta.scale: read as the rule's fallback, then rewritten             */
    float* scale_inv;    /* meta.scale_inv: rewritten                                           */
    uint64_t numel;
    uint32_t acc;        /* scratch                                                             */
    uint32_t reserved;   /* scratch (zero it once with acc)                                     */
} msamp_bucket_item;

/* amax[0] = max|src| per item, NaN propagating (distributed.py:156: g.abs().max()); with
 * MSAMP_FLAG_NAN_TO_INF a NaN or +Inf result becomes +Inf (distributed.py:159: the MAX all-reduce that
 * follows ignores NaN). */
int msamp_bucket_amax(msamp_bucket_item* items, int n_items, const int32_t* block_map, int n_blocks, int in_dtype,
                      int flags, msamp_stream_t stream);

/* msamp_bucket_amax that also writes, into each item's dst, the FP8 codes of src times the scale the item has NOW (no
 * counterpart in the reference, which quantizes after the scales are known: distributed.py:163-185).  After a round
 * of msamp_bucket_cast that scale is rule(amax) * pre_scale of that round, a power of two times a constant that
 * seldom changes from one round to the next.  msamp_bucket_cast compares the scale it arrives at with the one the
 * codes were written with and leaves the items where the two agree alone: the bucket is then read once instead of
 * twice (3 instead of 5 bytes per bf16 element), with the same bytes in the buffer either way.  The codes of an item
 * are final only after msamp_bucket_cast.  fp8_type must be the one msamp_bucket_cast is then called with. */
int msamp_bucket_amax_speculative(msamp_bucket_item* items, int n_items, const int32_t* block_map, int n_blocks,
                                  int in_dtype, int fp8_type, int flags, msamp_stream_t stream);

/* scale = rule(amax[0], fallback scale, fp_max, margin) * pre_scale (distributed.py:163-170, pre_scale =
 * 1/sqrt(world size)), dst = FP8 codes of src * scale (distributed.py:179-185), scale_inv = (1/scale) /
 * scale_inv_div (distributed.py:186 followed by :192, the division of the finished tensor by the world size;
 * pass 1 for none).  amax[0] is read as the caller left it (reduced over the ranks or not). */
int msamp_bucket_cast(msamp_bucket_item* items, int n_items, const int32_t* block_map, int n_blocks, int in_dtype,
                      int fp8_type, float pre_scale, float scale_inv_div, int margin, msamp_stream_t stream);

/* Norms of FP8 tensors without dequantizing them to memory: what clip_grad_norm_ computes per gradient
 * (nn/clip_grad.py:29-41: `g.to(float32)` then `abs().max()` or `torch.norm(g, p)`), for many tensors per launch.
 * out[i] = |scale_inv| * (sum |q|^p)^(1/p) for norm_kind 1 or 2, |scale_inv| * max|q| for norm_kind 0 (the
 * infinity norm), accumulated in double and rounded to float once; NaN codes give NaN.  `items`: DEVICE array
 * (acc is scratch: zero it once); block_map as for the bucket entry points, chunks of MSAMP_BUCKET_CHUNK codes. */
typedef struct msamp_norm_item {
    const uint8_t* q;
    const float* scale_inv;
    float* out;
    uint64_t numel;
    double acc;          /* scratch */
} msamp_norm_item;
int msamp_fp8_norms(msamp_norm_item* items, int n_items, const int32_t* block_map, int n_blocks, int fp8_type,
                    int norm_kind, msamp_stream_t stream);

/* tex.te_gemm as Gemm.fp8_gemm calls it (gemm.py:121-144; transa=True, transb=False):
 * D[N][M] = (B[N][K] . A[M][K]^T) * *a_scale_inv * *b_scale_inv (+ bias[M]) (+ D if accumulate).
 * A, B: FP8 bytes, row-major, K contiguous, K % 16 == 0, 16-byte aligned.  d_dtype: F32/F16/BF16.
 * bias: nullable, bias_dtype F32/F16/BF16. */
int msamp_fp8_gemm(const uint8_t* a, int a_type, const float* a_scale_inv, const uint8_t* b, int b_type,
                   const float* b_scale_inv, void* d, int d_dtype, int m, int n, int k, int accumulate,
                   const void* bias, int bias_dtype, msamp_stream_t stream);

/* The same product with operands handed over K-major: a_kmajor != 0 means `a` points at A^T, i.e. [K][M]
 * with M contiguous, likewise b_kmajor for [K][N].  The backward GEMMs of a linear layer
 * (nn/functional.py:84-111 of the reference) then read W, x and dy as they are, and the explicit FP8
 * transposes (transformer_engine_wrapper.py:165-176) are not needed.  Results are bit-identical to
 * msamp_fp8_gemm on transposed copies (every kernel behind these entry points adds up the same 128-byte blocks of K
 * in ascending order).  Supported: a K-major alone, or both; k a multiple of 128 and at least 256, and the row
 * count of every K-major operand (m, and n if b_kmajor) a multiple of 256; otherwise MSAMP_ERR_SHAPE. */
int msamp_fp8_gemm_kmajor(const uint8_t* a, int a_type, const float* a_scale_inv, int a_kmajor, const uint8_t* b,
                          int b_type, const float* b_scale_inv, int b_kmajor, void* d, int d_dtype, int m, int n, int k,
                          int accumulate, const void* bias, int bias_dtype, msamp_stream_t stream);

/* The weight-gradient GEMM of a linear layer followed by its cast to FP8 (nn/functional.py:100-111 followed by
 * :121-123 of the reference: `wgrad = Gemm.fp8_gemm(...)`, then `wgrad.cast(Dtypes.kfloat8_e4m3, meta=..., sync=True)`)
 * without the second trip over the product: q = FP8 codes of round_to_d_dtype(D) * scale, with
 * *amax = max |round_to_d_dtype(D)|, *scale from the pow-2 rule of that amax (fallback: the old *scale) and
 * *scale_inv = 1 / *scale -- bit for bit what msamp_fp8_gemm_kmajor into a d_dtype buffer followed by
 * msamp_cast_to_fp8_intime of that buffer gives.  flags and workspace as for msamp_cast_to_fp8_intime.  Two forms:
 *  - one launch, the product never leaves the chip: at most one 256 x 256 output tile per compute unit (the workgroups
 *    wait for each other), accumulate == 0, a stream on which such kernels are allowed (not capturing, no other stream
 *    of the device busy with them), no MSAMP_FLAG_TWO_PASS;
 *  - on speculation, any number of tiles, any stream, also under capture: needs d, a buffer of n x m d_dtype elements
 *    (16-byte aligned).  The GEMM stores the product there as msamp_fp8_gemm_kmajor would (added to what d holds if
 *    accumulate != 0: gradient accumulation, functional.py:100-111) and beside it the codes for the scale the meta
 *    holds before the call; the workgroup that finishes last applies the rule, and only if the rule arrives at another
 *    scale does a second launch read d again and rewrite the codes.  On return d holds the (accumulated) product.
 *    Not taken with MSAMP_FLAG_NO_SPECULATION, nor for d_dtype float32.
 * Both need m and n multiples of 256, k a multiple of 128 and at least 256, q_type E4M3, both operands K-major or
 * neither, and a problem too large for the GEMM with 128 x 128 tiles (msamp_set_small_tile_limit): below that size the
 * two steps are the faster way.  d may be null: then only the first form is considered.
 * Returns MSAMP_NOT_FUSED (1), having done nothing, when neither form applies and the caller has to take the two steps. */
#define MSAMP_NOT_FUSED 1
int msamp_fp8_gemm_cast(const uint8_t* a, int a_type, const float* a_scale_inv, int a_kmajor, const uint8_t* b, int b_type,
                        const float* b_scale_inv, int b_kmajor, void* d, int d_dtype, int accumulate, uint8_t* q, int q_type,
                        float* scale, float* amax, float* scale_inv, int m, int n, int k, int margin, int flags,
                        void* workspace, msamp_stream_t stream);

/* Tile walks of the 256 x 256-tile kernel (no counterpart in the reference, whose GEMM is cuBLASLt behind
 * transformer_engine_wrapper.py:63-103).  Which workgroup takes which output tile decides what the 32 compute units of
 * an XCD share through their L2; the library picks a walk from the shape by rules measured on Llama shapes, and the
 * best one for another shape can be up to 13 % faster.  A walk is a number 0..7: bit 0 = groups of eight tile columns
 * walked row by row (instead of groups of tile rows walked column by column), bit 1 = the XCD's patch of 32 tiles
 * turned, 4 of the grouped dimension by 8 of the walked one; with both operands row-major a third bit (walks 4..7) makes
 * the K loop issue a slice's tile loads in the order of need over a whole step and await them in two parts at two
 * barriers (1 to 8 % faster at K of 12288 and more, where the built-in rule takes it; level below).  Every walk gives the same output bits.
 * msamp_fp8_gemm_set_walk registers a walk for one problem -- (m, n, k) and operand layouts as in msamp_fp8_gemm_kmajor --
 * for all later calls of every GEMM entry point, walk = -1 removes it; msamp_fp8_gemm_get_walk returns it, -1 if none.
 * msamp_fp8_gemm_tune computes the product like msamp_fp8_gemm_kmajor with accumulate = 0 and, when the problem has at
 * least two rounds of tiles and `stream` is not being captured, times the rule's walk and the explicit ones on the
 * operands given (some forty launches between HIP events; it synchronises with the stream) and registers the fastest if
 * it beats the rule's by more than 5 %; *chosen (nullable) receives the registered walk or -1.  Process-wide. */
int msamp_fp8_gemm_set_walk(int m, int n, int k, int a_kmajor, int b_kmajor, int walk);
int msamp_fp8_gemm_get_walk(int m, int n, int k, int a_kmajor, int b_kmajor);
int msamp_fp8_gemm_tune(const uint8_t* a, int a_type, const float* a_scale_inv, int a_kmajor, const uint8_t* b, int b_type,
                        const float* b_scale_inv, int b_kmajor, void* d, int d_dtype, int m, int n, int k, const void* bias,
                        int bias_dtype, int* chosen, msamp_stream_t stream);

/* msamp_fp8_gemm with row-major operands runs 256 x 256 output tiles, one workgroup each; a problem with few of them
 * (a 2048 x 2048 output has 64, a quarter of the compute units) runs 128 x 128 tiles instead when it has at most
 * `big_tiles` of the large ones (at most half that many if K < 3072), K is a multiple of 128 and at least 512.  Same
 * bits either way.  Default 128 (up to two small tiles per compute unit: measured faster up to there); 0 = the large
 * tile always.  Process-wide; no counterpart in the reference. */
void msamp_set_small_tile_limit(int big_tiles);

/* Calibration aid, no counterpart in the reference: `workgroups` workgroups of four wavefronts each issue
 * iters x 16 FP8 16x16x128 MFMAs (iters a multiple of 4) on registers loaded once from seed (4096 bytes of FP8 codes,
 * device memory); nothing else moves and nothing is written (sink: one float of device memory, never stored to in
 * practice).  distinct_operands == 0: every MFMA takes the same two operands; != 0: eight X and eight Y fragments,
 * every pair in turn as in a K slice of the GEMM, so that the operand buses toggle as they do there.  *flop (host,
 * may be null) receives the floating-point operations of the launch.  Timed, it gives the rate the matrix pipes
 * sustain on this device under its power limit, the practical ceiling beside the nominal peak. */
int msamp_mfma_probe(const void* seed, float* sink, int iters, int workgroups, int distinct_operands, double* flop,
                     msamp_stream_t stream);

/* msamp_adamw.adamw_fp8_stage1_compute (adamw.cu:99-127): fp32 param/grad, quantized moments;
 * updates param in place and atomically maxes |m'|, |v'| into the two amax cells.
 * exp_avg_dtype: E4M3/E5M2/F16/F32, exp_avg_sq_dtype: F16/F32/E4M3/E5M2. */
int msamp_adamw_fp8_stage1(float* param, const float* grad, size_t n, const void* exp_avg, int exp_avg_dtype,
                           float exp_avg_factor, float* exp_avg_amax, float beta1, const void* exp_avg_sq,
                           int exp_avg_sq_dtype, float exp_avg_sq_factor, float* exp_avg_sq_amax, float beta2,
                           float eps, int step, float lr, int bias_correction, msamp_stream_t stream);

/* msamp_adamw.adamw_fp8_stage2_compute (adamw.cu:129-153): rewrite the moments with new scales. */
int msamp_adamw_fp8_stage2(const float* grad, size_t n, void* exp_avg, int exp_avg_dtype, float exp_avg_factor,
                           float new_exp_avg_factor, float beta1, void* exp_avg_sq, int exp_avg_sq_dtype,
                           float exp_avg_sq_factor, float new_exp_avg_sq_factor, float beta2, msamp_stream_t stream);

/* One tensor of the fused multi-tensor step below.  The array of descriptors lives in DEVICE
 * memory and is written by the kernels (acc/saved are scratch: zero-initialise acc once; the
 * library leaves it zero). */
typedef struct msamp_adamw_tensor {
    void* weight;            /* weight_dtype payload (FP8 codes or scaled fp16), updated in place */
    const uint8_t* grad;     /* FP8 codes (grad_dtype)                                            */
    uint8_t* exp_avg;        /* E4M3 codes, updated in place                                      */
    uint16_t* exp_avg_sq;    /* scaled fp16, updated in place                                     */
    float* w_scale;          /* weight meta: scale, scale_inv, amax[0] -- read, then rewritten    */
    float* w_scale_inv;
    float* w_amax;
    const float* g_scale_inv;
    float* m_scale;          /* exp_avg meta                                                      */
    float* m_scale_inv;
    float* m_amax;
    float* v_scale;          /* exp_avg_sq meta                                                   */
    float* v_scale_inv;
    float* v_amax;
    uint64_t numel;
    uint32_t acc[3];         /* scratch: running max bit patterns of |p'|, |m'|, |v'|             */
    float saved[3];          /* scratch: dequantization factors in force before this step         */
    uint32_t reserved[2];
} msamp_adamw_tensor;

/* The whole FP8 branch of LBAdamW.adamw_fn (adamw.py:148-199) for n_tensors tensors in three
 * launches: (1) dequantize w/g/m/v, AdamW (or Adam-mode L2) update, fresh amax of p', m', v';
 * (2) pow-2 scales (weight: fallback = old scale; moments: fallback 1.0; all moment scales 1 when
 * tensor_scale == 0) and meta rewrite; (3) recompute and requantize w (weight_dtype), m (E4M3),
 * v (scaled fp16), walking the blocks back to front so the re-read meets the cache.
 * `tensors`: DEVICE array of descriptors; `block_map`: DEVICE array of n_blocks
 * {tensor index, chunk index} int32 pairs (chunks of MSAMP_ADAMW_CHUNK elements, tensors in order)
 * built by the caller once per parameter set.  `blocks_per_tensor` (HOST array of n_tensors counts,
 * nullable) with `group_blocks` > 0 makes the library process whole tensors in groups of at most
 * group_blocks chunks, so that a group's second pass re-reads from the Infinity Cache instead of HBM.
 * weight_dtype: E4M3/E5M2/F16; grad_dtype: E4M3/E5M2.
 * Hyper-parameters arrive as doubles and are narrowed the way the reference narrows them
 * (adamw.cu:99-107, adamw.py:160-164). */
#define MSAMP_ADAMW_CHUNK 16384
int msamp_adamw_fp8_fused(msamp_adamw_tensor* tensors, int n_tensors, const int32_t* block_map, int n_blocks,
                          int weight_dtype, int grad_dtype, double lr, double beta1, double beta2, double eps,
                          double weight_decay, int step, int bias_correction, int adam_mode, int maximize,
                          int tensor_scale, const int32_t* blocks_per_tensor, int group_blocks,
                          msamp_stream_t stream);

/* Output buffers of one tensor for the speculative form below: same sizes and types as the descriptor's weight,
 * exp_avg and exp_avg_sq payloads, not overlapping them. */
typedef struct msamp_adamw_buffers {
    void* weight;
    uint8_t* exp_avg;
    uint16_t* exp_avg_sq;
    uint64_t reserved;
} msamp_adamw_buffers;

/* msamp_adamw_fp8_fused with separate output buffers, in ONE pass over the data when the scales hold (not in the
 * reference, whose optimizer is LBAdamW.adamw_fn, adamw.py:148-199, with two passes over every tensor).  Scales are
 * powers of two and seldom change between steps, so the first launch reads w/g/m/v once, quantizes p', m', v' with
 * the scales each tensor has NOW into outputs[t], and collects the three maxima; the second derives the scales from
 * them as msamp_adamw_fp8_fused does, rewrites the metas and sets redo[t] = 1 where a scale differs from the one
 * used; the third repeats exactly those tensors from their (untouched) inputs with the new scales.  On return the
 * new payloads of EVERY tensor are in outputs[t] -- the same bits msamp_adamw_fp8_fused leaves in place -- the metas
 * are updated, and the descriptors' weight / exp_avg / exp_avg_sq buffers still hold the old state: the caller swaps
 * the two sets of buffers.  9 instead of 14 bytes of HBM traffic per parameter, at the price of 4 bytes per parameter
 * of memory.  `outputs`: DEVICE array of n_tensors entries; `redo`: DEVICE array of n_tensors int32 written by the
 * call (1 = the tensor took the second round).  Other arguments as for msamp_adamw_fp8_fused. */
int msamp_adamw_fp8_fused_speculative(msamp_adamw_tensor* tensors, const msamp_adamw_buffers* outputs, int32_t* redo,
                                      int n_tensors, const int32_t* block_map, int n_blocks, int weight_dtype,
                                      int grad_dtype, double lr, double beta1, double beta2, double eps,
                                      double weight_decay, int step, int bias_correction, int adam_mode, int maximize,
                                      int tensor_scale, msamp_stream_t stream);

/* The one-pass step of msamp_adamw_fp8_fused_speculative without the second set of buffers (not in the reference,
 * whose optimizer is LBAdamW.adamw_fn, adamw.py:148-199).  The caller keeps the payloads of all n_tensors tensors
 * back to back, in the order of `block_map`, each padded to whole chunks of MSAMP_ADAMW_CHUNK elements, in three arenas
 * (weights, exp_avg, exp_avg_sq) that have |shift_elems| elements of room at one end; the descriptors point at the
 * payloads where they are now.  The call writes every tensor's new payloads shift_elems elements away from the old
 * ones (the same element offset in all three arenas): with a negative shift it walks the chunks front to back, with a
 * positive one back to front, so that the room is always ahead of the walk, and it sees to it that a chunk is
 * overwritten only once its tensor's scales are known and, where they came out different from the ones used, the
 * chunk has been done again from its inputs.  The caller alternates the sign from step to step (with descriptors that
 * point at the new places).  No tensor may have more chunks than the room holds (sticky error word otherwise, see
 * below); for the workgroups never to wait for each other in practice, make the room a few thousand chunks larger
 * than the largest tensor.  Results, metas and `redo` as for msamp_adamw_fp8_fused_speculative: the same bits that
 * msamp_adamw_fp8_fused leaves in place.  `sync`: DEVICE buffer of MSAMP_ADAMW_SYNC_BYTES(n_tensors, n_blocks) bytes,
 * 8-byte aligned, zeroed once by the caller, through which the workgroups of a call tell each other which chunks are
 * stored and how a tensor came out.  The descriptors' acc words must be zero before the first call (the library
 * leaves them at zero).  `workspace`: the MSAMP_WORKSPACE_BYTES buffer of the other entry points; a wait that
 * runs out (msamp_set_spin_limit) or a layout that breaks the rule above sets its sticky error word, reported by
 * msamp_check_async_error: the state is then partly updated and must be restored from a copy. */
/* The float32-moment branch of LBAdamW.adamw_fn (adamw.py:200-232) for one parameter in one pass: the reference runs it
 * as about a dozen element-wise torch calls (its own one-pass kernel, adamw.cu:20-28 bound as adamw_compute :77-97, is
 * never called from its Python).  `param`, `exp_avg`, `exp_avg_sq`: float32, updated in place; `grad`: F32 / F16 / BF16.
 * Every intermediate is rounded where the torch chain rounds it on the GPU (add with alpha = one fused multiply-add,
 * division by the Python number sqrt(bias_correction2) = multiplication by its narrowed reciprocal), so the results are
 * the chain's, bit for bit.  adam_mode: weight decay as an L2 term on the gradient instead of a decay of the weight. */
int msamp_adamw_f32(float* param, const void* grad, int grad_dtype, size_t n, float* exp_avg, float* exp_avg_sq, double lr,
                    double beta1, double beta2, double eps, double weight_decay, int step, int bias_correction, int adam_mode,
                    int maximize, msamp_stream_t stream);

/* The same step (adamw.py:148-199: stage 1, the scale rule on the two amaxs, stage 2) for parameters kept in high
 * precision -- biases, norm weights, embeddings: a plain F32 / F16 / BF16 parameter and gradient, exp_avg in E4M3, exp_avg_sq
 * in scaled F16 -- for n_tensors of them at once, with nothing read back by the host (the reference takes a dozen launches
 * and two host round trips per parameter).  Uses the weight (the parameter, updated in place in param_dtype), grad
 * (grad_dtype, passed through the uint8_t pointer), exp_avg, exp_avg_sq, m_* and v_* fields of the descriptors.
 * block_map == NULL: one launch, one workgroup per parameter (which walks its parameter twice: for small tensors).
 * Otherwise `block_map` / `n_blocks` as for msamp_adamw_fp8_fused and three launches over the chunks (stage 1, scales,
 * stage 2), for tensors of any size; the four payload pointers of a tensor must then be aligned for four elements, and
 * the descriptors' `acc` words zero between calls (the call leaves them so).  Same bits as msamp_adamw_fp8_stage1 /
 * _stage2 with the parameter rounded to its type in between. */
int msamp_adamw_plain_fused(msamp_adamw_tensor* tensors, int n_tensors, const int32_t* block_map, int n_blocks, int param_dtype,
                            int grad_dtype, double lr, double beta1, double beta2, double eps, double weight_decay, int step,
                            int bias_correction, int adam_mode, int maximize, int tensor_scale, msamp_stream_t stream);

#define MSAMP_ADAMW_POST_WORDS 8
#define MSAMP_ADAMW_SYNC_BYTES(n_tensors, n_blocks) ((size_t)(n_tensors) * MSAMP_ADAMW_POST_WORDS * 8 + (size_t)(n_blocks) * 136)
int msamp_adamw_fp8_fused_shift(msamp_adamw_tensor* tensors, int32_t* redo, void* sync, int n_tensors, const int32_t* block_map,
                                int n_blocks, long long shift_elems, int weight_dtype, int grad_dtype, double lr, double beta1,
                                double beta2, double eps, double weight_decay, int step, int bias_correction, int adam_mode,
                                int maximize, int tensor_scale, void* workspace, msamp_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MSAMP_HIP_H_ */
