// The direct-to-LDS FP8 GEMM with 128 x 128 output tiles, for problems that leave most compute units idle with
// 256 x 256 tiles (a 2048 x 2048 output is 64 of those, a quarter of the chip, and 256 of these).  K a multiple of 128
// and at least 512; operands row-major (K-contiguous) or, with XT / YT, K-major ([K][rows], rows a multiple of 128):
// the slice then lies in LDS as 128 k-rows of 128 bytes, the 16-byte position XOR-ed with k % 8, and the fragments
// come from the transposing LDS read, as in the large tile.
//
// Four wavefronts, each owning a 64 x 64 quadrant as 4 x 4 accumulators of the 16x16x128 FP8 MFMA, in fixed AGPRs like
// those of the large tile (block (i, j) in a[16i + 4j .. + 3]; left to the register allocator they were renumbered
// from slice to slice, with copies and wait states between the MFMAs).  A K slice is 128 X rows
// and 128 Y rows of 128 bytes, 32 KiB, brought in by eight direct-to-LDS loads per wavefront with the same swizzle
// as the large tile; five stages -- the whole LDS -- so that three slices are on their way while one is being read and
// another worked on (a slice is only 16 MFMAs per wavefront, a fifth of a microsecond, and the way to L2 is close to
// a microsecond).  The fragments of slice kt + 1 are read from LDS between the first eight MFMAs of slice kt, and the
// eight loads of slice kt + 4 go out one every other MFMA (issued in one go after the barrier they held the wave, and
// its MFMAs, while the memory pipe accepted them: 0.54 against 0.43 us per slice); one barrier per slice.
//
// Per flop this tile needs twice the L2 -> LDS bytes of the large one (32 KiB per 16 MFMAs per wavefront against
// 64 KiB per 64), which is what bounds it once every compute unit runs one: 2048 x 2048 x 4096 takes 16.7 us with the
// MFMAs and 15.5 us without them (an ablation), 95 GB/s per compute unit where a bare loop of such loads reaches 121.
// It is the faster kernel only while the large tile leaves compute units idle, and the host picks it only then.
//
// Every output element is accumulated over the 128-byte blocks of K in ascending order, one MFMA per block, and
// scaled, biased, summed and rounded with the expressions of the large tile: the two kernels agree to the bit.
#pragma once

namespace msamp {

constexpr int kSmallTile = 128;
constexpr int kSmallStage = 2 * kSmallTile * kBK;    // 32 KiB
constexpr int kSmallStages = 5;    // all 160 KiB of the LDS

template <int XF, int YF, typename OT, bool XT = false, bool YT = false>
__global__ __launch_bounds__(kGemmThreads) void fp8_gemm_dma128_kernel(const uint8_t* __restrict__ X, const uint8_t* __restrict__ Y,
                                                                        OT* __restrict__ D, int NR, int NC, int K,
                                                                        const float* __restrict__ x_scale_inv,
                                                                        const float* __restrict__ y_scale_inv, int accumulate,
                                                                        const void* __restrict__ bias, int bias_dt) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    const int tiles_r = (NR + kSmallTile - 1) / kSmallTile, tiles_c = (NC + kSmallTile - 1) / kSmallTile;
    int tr, tc;
    tile_of_id(blockIdx.x, tiles_r, tiles_c, false, false, tr, tc);
    const int row0 = tr * kSmallTile, col0 = tc * kSmallTile;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wr = wave >> 1, wc = wave & 1;
    float alpha = (*x_scale_inv) * (*y_scale_inv);
    asm volatile("" : "+v"(alpha));

    // ---- global -> LDS: one wave instruction fills 8 rows of 128 bytes (lane l: row l / 8, 16-byte position l % 8,
    // fetching the logical chunk position ^ swizzle(row)); rows past the end of the matrix are clamped to its last row
    // K-major operand: one wave instruction fills 8 k-rows of 128 bytes (lane l: k-row l / 8, position l % 8, fetching
    // the logical chunk position ^ (k-row % 8))
    const int chunk = (lane & 7) ^ (lane >> 3) ^ (wave & 1);
    const int chunk_t = (lane & 7) ^ (lane >> 3);
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)smem)));
    uint32_t xoff[4], yoff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = (i * 4 + wave) * 8 + (lane >> 3);
        int gx = row0 + r, gy = col0 + r;
        gx = gx < NR ? gx : NR - 1;
        gy = gy < NC ? gy : NC - 1;
        const int krow = (i * 4 + wave) * 8 + (lane >> 3);
        xoff[i] = XT ? static_cast<uint32_t>(krow) * static_cast<uint32_t>(NR) + row0 + chunk_t * 16
                     : static_cast<uint32_t>(gx) * static_cast<uint32_t>(K) + chunk * 16;
        yoff[i] = YT ? static_cast<uint32_t>(krow) * static_cast<uint32_t>(NC) + col0 + chunk_t * 16
                     : static_cast<uint32_t>(gy) * static_cast<uint32_t>(K) + chunk * 16;
    }
    // one of the 8 loads of a slice (0..3: X rows, 4..7: Y rows); assembly for the reason given at the large tile
    auto dma = [&](int kt, int which) __attribute__((always_inline)) {
        const bool is_x = which < 4;
        const size_t slice = static_cast<size_t>(kt) * kBK;
        const uint8_t* src = is_x ? X + (XT ? slice * NR : slice) : Y + (YT ? slice * NC : slice);
        const uint32_t off = is_x ? xoff[which] : yoff[which - 4];
        const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_base + (kt % kSmallStages) * kSmallStage +
                                                            (is_x ? 0 : kSmallTile * kBK) + ((which & 3) * 4 + wave) * 1024);
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(dst), "v"(off), "s"(src) : "memory", "m0");
    };
    auto dma_slice = [&](int kt) __attribute__((always_inline)) {
#pragma unroll
        for (int w = 0; w < 8; ++w) dma(kt, w);
    };

    // ---- LDS -> fragments: for row lane % 16 of a 16-row block a lane holds the K-bytes (lane / 16) * 32 .. + 31 of the
    // slice, two 16-byte reads at the swizzled chunks
    const int l16 = lane & 15, g4 = lane >> 4;
    const int fsw = (lane & 7) ^ ((lane >> 3) & 1);
    const int off_lo = ((2 * g4) ^ fsw) << 4;
    const int xrow = (wr * 64 + l16) * kBK;
    const int yrow = kSmallTile * kBK + (wc * 64 + l16) * kBK;
    const int tj = l16 >> 1;
    const int t_lane = (g4 * 32 + tj) * kBK + (l16 & 1) * 8;    // k-row and 8-byte half of this lane's transposing reads
    // A slice's fragments arrive in pieces: two 16-byte reads per 16-row block of a row-major operand (block p / 2, half
    // p % 2), four 8-byte transposing reads per block of a K-major one (block p / 4, eight k each); X pieces first.
    constexpr int kPX = XT ? 16 : 8, kPY = YT ? 16 : 8, kPieces = kPX + kPY;
    auto read_piece = [&](int* fxd, int* fyd, int kt, int p) __attribute__((always_inline)) {
        const uint8_t* base = smem + (kt % kSmallStages) * kSmallStage;
        const bool is_x = p < kPX;
        const int q = is_x ? p : p - kPX;
        if ((is_x && !XT) || (!is_x && !YT)) {
            const int b = q >> 1, hf = q & 1;
            const v4i val = *reinterpret_cast<const v4i*>(base + (is_x ? xrow : yrow) + b * 16 * kBK + (off_lo ^ (hf * 16)));
            int* d = (is_x ? fxd : fyd) + b * 8 + hf * 4;
            d[0] = val[0], d[1] = val[1], d[2] = val[2], d[3] = val[3];
        } else {
            const int b = q >> 2, qq = q & 3;
            const int wq = is_x ? wr : wc;
            const int addr = (is_x ? 0 : kSmallTile * kBK) + t_lane + (qq * 8) * kBK + (((wq * 4 + b) ^ tj) << 4);
            const v2i val = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i*)(base + addr));
            int* d = (is_x ? fxd : fyd) + b * 8 + qq * 2;
            d[0] = val[0], d[1] = val[1];
        }
    };

    acc_clear();
    int fx[2][32], fy[2][32];

    // the 16 MFMAs of the slice held in fragment set `cur`, with the 16 fragment reads of slice rd_kt (into the other
    // set) between them.  srcA = Y rows, srcB = X rows: a lane then holds, for D row lane % 16 of a block, four
    // consecutive D columns.
    auto step = [&](auto curc, int rd_kt, bool do_read, int ld_kt, bool do_load) __attribute__((always_inline)) {
        constexpr int cur = decltype(curc)::value;
        constexpr int cb = (YF == MSAMP_DT_E4M3) ? 0 : 1;
        constexpr int bl = (XF == MSAMP_DT_E4M3) ? 0 : 1;
        static_for<4>([&](auto jc) {
            static_for<4>([&](auto ic) {
                constexpr int i = decltype(ic)::value, j = decltype(jc)::value;
                const int* cx = fx[cur] + i * 8;
                const int* cy = fy[cur] + j * 8;
                const v8i vx = {cx[0], cx[1], cx[2], cx[3], cx[4], cx[5], cx[6], cx[7]};
                const v8i vy = {cy[0], cy[1], cy[2], cy[3], cy[4], cy[5], cy[6], cy[7]};
                mfma_fixed<i * 4 + j, cb, bl>(vy, vx);
                // the fragment reads go with the first eight MFMAs (two to four each) and have come back by the barrier that
                // follows the last one; nothing moves across, so they stay spread as written
                constexpr int n = j * 4 + i;
                if (do_read && n < 8) {
#pragma unroll
                    for (int p = n * kPieces / 8; p < (n + 1) * kPieces / 8; ++p) read_piece(fx[cur ^ 1], fy[cur ^ 1], rd_kt, p);
                }
                // the eight tile loads of slice ld_kt, one every other MFMA: issued in one go they hold the wave, and with
                // it its MFMAs, for as long as the memory pipe takes to accept them
                if (do_load && (n & 1)) dma(ld_kt, n >> 1);
                __builtin_amdgcn_sched_barrier(0);
            });
        });
    };
    constexpr std::integral_constant<int, 0> c0{};
    constexpr std::integral_constant<int, 1> c1{};

    const int nk = K / kBK;    // at least 4 (the host sees to that)
    dma_slice(0);
    dma_slice(1);
    dma_slice(2);
    dma_slice(3);
    wait_vmcnt<24>();
    __syncthreads();
#pragma unroll
    for (int p = 0; p < kPieces; ++p) read_piece(fx[0], fy[0], 0, p);

    // Before the step of slice kt: slices kt + 1 .. kt + 3 are on their way (24 loads of this wave), slice kt is in
    // registers.  Wait for slice kt + 1, meet (it has landed in every wave's part of the stage, and nobody reads the
    // stage of slice kt - 1 any more), compute slice kt while reading kt + 1 and sending for slice kt + 4 into that stage.
    auto turn = [&](auto curc, int kt) __attribute__((always_inline)) {
        wait_vmcnt<16>();
        __syncthreads();
        step(curc, kt + 1, true, kt + 4, true);
    };
    int kt = 0;
    for (; kt + 5 < nk; kt += 2) {
        turn(c0, kt);
        turn(c1, kt + 1);
    }
    // four or five slices are left; the last four load nothing
    auto tail4 = [&](auto ac, auto bc, int k0) __attribute__((always_inline)) {
        wait_vmcnt<16>();
        __syncthreads();
        step(ac, k0 + 1, true, 0, false);
        wait_vmcnt<8>();
        __syncthreads();
        step(bc, k0 + 2, true, 0, false);
        wait_vmcnt<0>();
        __syncthreads();
        step(ac, k0 + 3, true, 0, false);
        step(bc, 0, false, 0, false);
    };
    if (kt + 5 == nk) {
        turn(c0, kt);
        tail4(c1, c0, kt + 1);
    } else {
        tail4(c0, c1, kt);
    }
    const uint32_t acc_token = acc_fence();
    __syncthreads();    // every wave is through with the stages, which the patches below reuse

    // ---- epilogue: the raw accumulators of a 16-row block go through a per-wave float32 patch; each lane then picks up
    // one 16-byte segment of an output row and applies the factor (bias, old output) with one rounding
    constexpr int kEsz = static_cast<int>(sizeof(OT));
    constexpr int kElems = 16 / kEsz;              // outputs per 16-byte segment: 8 or 4
    constexpr int kSegs = 64 / kElems;             // segments per 64-column row: 8 or 16
    constexpr int kRowsPerPass = 64 / kSegs;       // 8 or 4
    constexpr int kFPitch = 64 * 4 + 16;           // bytes per patch row
    uint8_t* patch = smem + wave * (16 * kFPitch);
    const bool vec_ok = (NC % kElems == 0) && ((reinterpret_cast<uintptr_t>(D) & 15) == 0);
    const bool plain = !accumulate && bias == nullptr;
    const int seg = lane % kSegs, prl = lane / kSegs;
    const int gcol = col0 + wc * 64 + seg * kElems;
    float bv[kElems];
#pragma unroll
    for (int e = 0; e < kElems; ++e) bv[e] = (bias != nullptr && gcol + e < NC) ? load_bias(bias, bias_dt, gcol + e) : 0.0f;
    static_for<4>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        static_for<4>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const v4f a = acc_quad<i * 4 + j>(acc_token);
            *reinterpret_cast<float4*>(patch + l16 * kFPitch + (j * 16 + g4 * 4) * 4) = make_float4(a[0], a[1], a[2], a[3]);
        });
        // (the patch is private to this wave and the LDS serves one wave's requests in order: no waits needed)
#pragma unroll
        for (int pass = 0; pass < 16 / kRowsPerPass; ++pass) {
            const int pr = pass * kRowsPerPass + prl;
            const int grow = row0 + wr * 64 + i * 16 + pr;
            const float* src = reinterpret_cast<const float*>(patch + pr * kFPitch + seg * kElems * 4);
            float r[kElems];
            const float4 a0 = *reinterpret_cast<const float4*>(src);
            r[0] = a0.x, r[1] = a0.y, r[2] = a0.z, r[3] = a0.w;
            if constexpr (kElems == 8) {
                const float4 a1 = *reinterpret_cast<const float4*>(src + 4);
                r[4] = a1.x, r[5] = a1.y, r[6] = a1.z, r[7] = a1.w;
            }
            if (grow >= NR || gcol >= NC) continue;
            OT* out = D + static_cast<size_t>(grow) * NC + gcol;
            if (vec_ok && gcol + kElems <= NC) {
                if (plain) {
#pragma unroll
                    for (int e = 0; e < kElems; ++e) r[e] = r[e] * alpha;
                } else {
                    float o[kElems];
#pragma unroll
                    for (int e = 0; e < kElems; ++e) o[e] = 0.0f;
                    if (accumulate) {
                        const uint4 old = load_out16(out);
                        if constexpr (kEsz == 4) {
                            o[0] = __uint_as_float(old.x), o[1] = __uint_as_float(old.y);
                            o[2] = __uint_as_float(old.z), o[3] = __uint_as_float(old.w);
                        } else {
                            In16<OT>::decode(old, o);
                        }
                    }
#pragma unroll
                    for (int e = 0; e < kElems; ++e) {
                        r[e] = fmaf(r[e], alpha, bv[e]);
                        if (accumulate) r[e] += o[e];
                    }
                }
                uint4 v;
                if constexpr (kEsz == 4) {
                    v = make_uint4(__float_as_uint(r[0]), __float_as_uint(r[1]), __float_as_uint(r[2]), __float_as_uint(r[3]));
                } else if constexpr (__is_same(OT, bf16_t)) {
                    v = make_uint4(pack_bf16(r[0], r[1]), pack_bf16(r[2], r[3]), pack_bf16(r[4], r[5]), pack_bf16(r[6], r[7]));
                } else {
                    v = make_uint4(pack_f16(r[0], r[1]), pack_f16(r[2], r[3]), pack_f16(r[4], r[5]), pack_f16(r[6], r[7]));
                }
                store_out16(out, v);
            } else {
                // rows that 16-byte accesses do not fit, or a segment that ends past the last column: one by one
#pragma unroll
                for (int e = 0; e < kElems; ++e) {
                    if (gcol + e < NC) {
                        if (plain) Elem<OT>::store(out + e, r[e] * alpha);
                        else store_out<OT>(out + e, fmaf(r[e], alpha, bv[e]), accumulate != 0);
                    }
                }
            }
        }
    });
}

template <int XF, int YF, typename OT, bool XT = false, bool YT = false>
static int launch_gemm_dma128(const uint8_t* X, const uint8_t* Y, void* D, int NR, int NC, int K, const float* xs, const float* ys,
                              int accumulate, const void* bias, int bias_dt, hipStream_t st) {
    constexpr int smem = kSmallStages * kSmallStage;
    static std::atomic<bool> configured{false};    // setting the attribute twice is harmless
    auto kern = fp8_gemm_dma128_kernel<XF, YF, OT, XT, YT>;
    if (!configured.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(fp8_gemm_dma128_kernel)");
        configured.store(true, std::memory_order_release);
    }
    const int tiles = ((NR + kSmallTile - 1) / kSmallTile) * ((NC + kSmallTile - 1) / kSmallTile);
    hipLaunchKernelGGL(kern, dim3(tiles), dim3(kGemmThreads), smem, st, X, Y, static_cast<OT*>(D), NR, NC, K, xs, ys, accumulate,
                       bias, bias_dt);
    MSAMP_CHECK_LAUNCH("fp8_gemm_dma128_kernel");
    return MSAMP_OK;
}

}    // namespace msamp
