// Convolution for layers whose whole filter fits in LDS: 64 input channels, at most 64 output
// channels, stride 1, no dilation (the 3x3 and 1x1 64->64 layers of ResNet; BASELINE config 1).
//
// Such layers have so little reduction per output (K*R*S = 576 MACs) that an implicit GEMM which
// re-gathers the input once per filter tap is bound by its loads and address arithmetic, not by
// the matrix cores.  Here a workgroup instead
//   * keeps the packed filter [K][R*S*64] resident in LDS for its whole life (persistent grid),
//   * loads one band of the input -- TP output rows plus the halo, every byte once -- into LDS,
//     biased to signed (x ^ 0x80) with the padding materialised, and
//   * runs the full reduction out of LDS with no global access and no barrier: per 32-byte step of
//     the reduction a wavefront reads 2 weight fragments and up to 4 pixel fragments and issues up
//     to 8 v_mfma_i32_32x32x32_i8 on its 128 pixel x 64 channel tile.
// The activations feed MFMA source A, so a lane owns one output channel (its scale, bias and
// sign-bias correction are per-lane constants) and four consecutive pixels per accumulator group.
// 8-bit results are staged through LDS so that every global store is a full 16-byte line piece in
// either output layout.
#include <type_traits>

#include "hipq_igemm.h"

// Optional phase clocks (development builds only): lane 0 of workgroup 0 records the shader clock
// at each HIPQ_PHASE(i); hipq_debug_band_phases copies them out.
#ifdef HIPQ_PHASE_CLOCKS
static __device__ long long g_phase_clock[32];
#define HIPQ_PHASE(i)                                                                              \
    do                                                                                             \
    {                                                                                              \
        if (blockIdx.x == 0 && threadIdx.x == 0)                                                   \
            g_phase_clock[(i) < 3 ? (i) : (i) + 6 * phase_iter] = clock64();                                                      \
    } while (0)
#define HIPQ_PHASE_NEXT() (++phase_iter)
#define HIPQ_PHASE_INIT() int phase_iter = 0
extern "C" HIPQ_API int hipq_debug_band_phases(long long* out32)
{
    return hipMemcpyFromSymbol(out32, HIP_SYMBOL(g_phase_clock), sizeof(long long) * 32) == hipSuccess ? 0 : 1;
}
#else
#define HIPQ_PHASE(i) ((void)0)
#define HIPQ_PHASE_NEXT() ((void)0)
#define HIPQ_PHASE_INIT() ((void)0)
#endif

namespace hipq
{
    constexpr int kBandC = 64;          // input channels (bytes per pixel slot)
    constexpr int kBandStagePitch = 144; // NCHW staging: bytes per channel row (128 pixels + pad, 16-byte multiple)
    constexpr int kBandStageWave = 64 * kBandStagePitch; // 9216 bytes per wavefront

    struct BandParams
    {
        const uint8_t* x; // [N][H][W][64]
        uint32_t x_bytes;
        int32_t H, W, P, Q, R, S, pbh, pbw, K;
        int32_t TP;    // output rows per band
        int32_t bands; // bands per image
        int32_t items; // N * bands
        int32_t BW;    // band width in pixel slots: Q + S - 1
        int32_t x_lds; // byte offset of the band buffer in LDS
        int32_t sink;  // byte offset of 16 spare LDS bytes that absorb the copies' out-of-range lanes
        int64_t PQ;
    };

    constexpr int kBandBatch = 10; // 16-byte loads a lane keeps in flight while filling LDS

    __device__ __forceinline__ int band_slot_offset(int slot, int chunk)
    {
        return slot * kBandC + ((chunk ^ ((slot >> 1) & 3)) << 4);
    }

    // Copies into LDS go in batches: all loads of a batch are issued before any is stored, and
    // issue and store recompute the addresses so that only the data stays in registers between.
    struct BandBatch
    {
        v4i v[kBandBatch];
    };

    // Filter: 4 lanes per row n = tid / 4, lane tid % 4 takes every fourth 16-byte chunk of the
    // row; batch element u is chunk tid % 4 + 4 * (u0 + u).
    template <bool STORE>
    __device__ __forceinline__ void band_w_copy(BandBatch& b, __amdgpu_buffer_rsrc_t wrs, uint8_t* lds, int u0, int taps, int kred, int K, int sink)
    {
        const int n = static_cast<int>(threadIdx.x) >> 2;
        const int sub = static_cast<int>(threadIdx.x) & 3;
#pragma unroll
        for (int u = 0; u < kBandBatch; ++u)
        {
            const int c = sub + 4 * (u0 + u);
            const bool in = u0 + u < taps;
            if (STORE) // LDS: [tap][64 rows][64 bytes], chunks swizzled like the band's
                *reinterpret_cast<v4i*>(lds + (in ? (u0 + u) * (64 * kBandC) + band_slot_offset(n, sub) : sink)) = b.v[u];
            else
                b.v[u] = buffer_load16(wrs, (in && n < K) ? n * kred + c * 16 : kOob); // rows beyond K read as zeros
        }
    }

    // Band: lane takes chunk cx = cx0 + tid of a row of BW pixel slots (4 chunks a slot); batch
    // element u is band row sy0 + u.
    template <bool STORE>
    __device__ __forceinline__ void band_x_copy(BandBatch& b, __amdgpu_buffer_rsrc_t xrs, uint8_t* lds, const BandParams& p, int cx0, int sy0, int band_rows, int img_base, int p0, int fill, int xor_mask)
    {
        const int cx = cx0 + static_cast<int>(threadIdx.x);
        const int sx = cx >> 2;
        const int c4 = cx & 3;
        const int ix = sx - p.pbw;
        const bool col_in = sx < p.BW;
        const bool col_ok = col_in & (static_cast<uint32_t>(ix) < static_cast<uint32_t>(p.W));
#pragma unroll
        for (int u = 0; u < kBandBatch; ++u)
        {
            const int sy = sy0 + u;
            const int iy = p0 + sy - p.pbh;
            const bool in = col_in & (sy < band_rows);
            const bool ok = col_ok & (sy < band_rows) & (static_cast<uint32_t>(iy) < static_cast<uint32_t>(p.H));
            if (STORE)
            {
                v4i t = b.v[u];
                if (fill != 0) // uniform: a non-zero data zero point pads with that byte
                    t = v4i{ok ? t[0] : fill, ok ? t[1] : fill, ok ? t[2] : fill, ok ? t[3] : fill};
                *reinterpret_cast<v4i*>(lds + (in ? p.x_lds + band_slot_offset(sy * p.BW + sx, c4) : p.sink)) =
                    v4i{t[0] ^ xor_mask, t[1] ^ xor_mask, t[2] ^ xor_mask, t[3] ^ xor_mask};
            }
            else
                b.v[u] = buffer_load16(xrs, ok ? img_base + (iy * p.W + ix) * kBandC + c4 * 16 : kOob);
        }
    }

    // Reduction of T pixel tiles x 2 channel tiles over all taps, out of LDS: per 32-byte half of a
    // tap 2 weight fragments, T pixel fragments, 2T MFMAs; no barrier, no global access.  Two
    // fragment sets alternate (statically indexed) so that the reads of one half overlap the MFMAs
    // of the other.  wl: this lane's weight row at tap 0, chunk lane/32.
    template <int T>
    __device__ __forceinline__ void band_reduce(v16i (&acc)[4][2], const uint8_t* xs, const uint8_t* wl, const int (&slot0)[4], int half, int R, int S, int BW)
    {
        v4i xa[T], xb[T], wa[2], wb[2];
        int xoff[T];
        auto addr = [&](int tap_slot) {
#pragma unroll
            for (int ti = 0; ti < T; ++ti)
                xoff[ti] = band_slot_offset(slot0[ti] + tap_slot, half);
        };
        // chunks 2,3 of a 64-byte row are chunks 0,1 with offset bit 5 flipped
        auto load = [&](const uint8_t* wp, int flip, v4i(&xf)[T], v4i(&wf)[2]) {
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
                wf[ni] = *reinterpret_cast<const v4i*>(reinterpret_cast<const uint8_t*>(reinterpret_cast<uintptr_t>(wp) ^ flip) + ni * 32 * kBandC);
#pragma unroll
            for (int ti = 0; ti < T; ++ti)
                xf[ti] = *reinterpret_cast<const v4i*>(xs + (xoff[ti] ^ flip));
        };
        auto mac = [&](const v4i(&xf)[T], const v4i(&wf)[2]) {
#pragma unroll
            for (int ti = 0; ti < T; ++ti)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    acc[ti][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[ti], wf[ni], acc[ti][ni], 0, 0, 0);
        };
        addr(0);
        load(wl, 0, xa, wa);
        const uint8_t* wp = wl;
        int r = 0, s = 0;
        const int taps = R * S;
#pragma unroll 1
        for (int tap = 0; tap < taps; ++tap)
        {
            load(wp, 32, xb, wb);
            mac(xa, wa);
            // the next tap; after the last one this wraps to tap 0, a harmless re-read that keeps
            // the loop free of conditional loads
            wp += 64 * kBandC;
            ++s;
            if (s == S)
            {
                s = 0;
                ++r;
            }
            if (r == R)
            {
                r = 0;
                wp = wl;
            }
            addr(r * BW + s);
            load(wp, 0, xa, wa);
            mac(xb, wb);
        }
    }

    template <int MODE, int KIND, bool OUT_NCX>
    __global__ __launch_bounds__(256, 2) void conv_band_kernel(BandParams p,
                                                               ConvX xl,
                                                               const int8_t* __restrict__ w,
                                                               const int32_t* __restrict__ wsum,
                                                               int32_t x_unsigned,
                                                               ZeroPoints zp,
                                                               Epilogue epi,
                                                               void* __restrict__ out)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int half = lane >> 5;
        const int l32 = lane & 31;
        uint8_t* const xs = lds + p.x_lds;

        HIPQ_PHASE_INIT();
        HIPQ_PHASE(0);
        const int taps = p.R * p.S;
        const int kred = taps * kBandC;
        const __amdgpu_buffer_rsrc_t xrs = make_rsrc(p.x, p.x_bytes);
        const __amdgpu_buffer_rsrc_t wrs = make_rsrc(w, static_cast<uint32_t>(p.K) * static_cast<uint32_t>(kred));

        auto item_geom = [&](int item, int& img, int& p0, int& rows) {
            img = item / p.bands;
            p0 = (item - img * p.bands) * p.TP;
            rows = min(p.TP, p.P - p0);
        };

        // the first loads of the filter and of the first band go out before anything waits
        BandBatch wb0, xb0;
        int item = blockIdx.x; // the grid never exceeds the item count
        int img, p0, rows;
        item_geom(item, img, p0, rows);
        band_w_copy<false>(wb0, wrs, lds, 0, taps, kred, p.K, p.sink);
        band_x_copy<false>(xb0, xrs, lds, p, 0, 0, rows + p.R - 1, img * p.H * p.W * kBandC, p0, 0, 0);

        const int32_t xzp = load_zp(zp.data_zp, zp.data_t);
        const int32_t wzp = load_zp(zp.filter_zp, zp.filter_t);
        if (wzp != 0) // uniform; w - wzp does not fit a signed byte: exact, slow
        {
            const OutMap om{OUT_NCX ? 1 : 0, p.K, p.PQ};
            for (; item < p.items; item += gridDim.x)
            {
                item_geom(item, img, p0, rows);
                slow_tile(xl, w, static_cast<int64_t>(p.items) * p.PQ, kred, x_unsigned, xzp, wzp, epi, om, out,
                          static_cast<int64_t>(img) * p.PQ + static_cast<int64_t>(p0) * p.Q, 0, rows * p.Q, p.K);
            }
            return;
        }
        const int xor_mask = x_unsigned ? static_cast<int>(0x80808080u) : 0;
        const int fill = (xzp & 0xFF) * 0x01010101;
        const int32_t mult = (x_unsigned ? 128 : 0) - xzp;

        // ---- per-lane channel constants (a lane owns channels lane%32 and 32 + lane%32) ---------
        const EpiConst ec = epi_const(epi);
        const bool has_sum = MODE == EPI_FUSED && epi.sum_in != nullptr;
        const bool relu = epi.relu != 0;
        int32_t corr[2];
        float bias[2], scale[2];
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
        {
            const int n = ni * 32 + l32;
            const bool ok = n < p.K;
            corr[ni] = ok ? mult * wsum[n] : 0;
            bias[ni] = (MODE == EPI_FUSED && epi.bias && ok) ? static_cast<float>(epi.bias[n]) : 0.0f;
            scale[ni] = (MODE == EPI_FUSED && epi.per_channel && ok) ? epi.scale[n] : ec.scale;
        }
        // INTERPRETER requantization in fixed point needs |acc * scale| * 256 < 2^31
        const float acc_max = static_cast<float>(kred) * (255.0f * 128.0f);
        const bool fast_interp = fabsf(ec.scale) * acc_max < 4194304.0f;

        HIPQ_PHASE(1);
        for (int u0 = 0; u0 < taps; u0 += kBandBatch)
        {
            if (u0)
                band_w_copy<false>(wb0, wrs, lds, u0, taps, kred, p.K, p.sink);
            band_w_copy<true>(wb0, wrs, lds, u0, taps, kred, p.K, p.sink);
        }
        HIPQ_PHASE(2);

        for (; item < p.items; item += gridDim.x)
        {
            item_geom(item, img, p0, rows);
            const int npix = rows * p.Q;
            const int ntiles = (npix + 31) >> 5;
            const int band_rows = rows + p.R - 1;
            const int img_base = img * p.H * p.W * kBandC;

            HIPQ_PHASE(3);
            __syncthreads(); // the previous item's staging reads are done
            HIPQ_PHASE(4);

            // ---- the band, every input byte once ----------------------------------------------
            for (int cx0 = 0; cx0 < p.BW * 4; cx0 += 256)
                for (int sy0 = 0; sy0 < band_rows; sy0 += kBandBatch)
                {
                    if (cx0 | sy0) // the first batch was issued ahead of time
                        band_x_copy<false>(xb0, xrs, lds, p, cx0, sy0, band_rows, img_base, p0, fill, xor_mask);
                    band_x_copy<true>(xb0, xrs, lds, p, cx0, sy0, band_rows, img_base, p0, fill, xor_mask);
                }
            __syncthreads();
            HIPQ_PHASE(5);
            // the next band's first loads fly while this one is reduced and requantized
            if (item + static_cast<int>(gridDim.x) < p.items)
            {
                int nimg, np0, nrows;
                item_geom(item + gridDim.x, nimg, np0, nrows);
                band_x_copy<false>(xb0, xrs, lds, p, 0, 0, nrows + p.R - 1, nimg * p.H * p.W * kBandC, np0, 0, 0);
            }

            // ---- reduction out of LDS: wavefront `wave` owns tiles 4*wave .. 4*wave+3 ---------------
            const int my_tiles = max(0, min(4, ntiles - 4 * wave));
            v16i acc[4][2];
#pragma unroll
            for (int ti = 0; ti < 4; ++ti)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        acc[ti][ni][r] = corr[ni];

            if (my_tiles > 0)
            {
                int slot0[4];
#pragma unroll
                for (int ti = 0; ti < 4; ++ti)
                {
                    // tiles past the end re-read the last pixel; their results are never stored
                    const int pix = min((4 * wave + ti) * 32 + l32, npix - 1);
                    const int py = pix / p.Q;
                    slot0[ti] = py * p.BW + (pix - py * p.Q);
                }
                const uint8_t* const wl = lds + band_slot_offset(l32, half);
                if (my_tiles > 2)
                    band_reduce<4>(acc, xs, wl, slot0, half, p.R, p.S, p.BW);
                else
                    band_reduce<2>(acc, xs, wl, slot0, half, p.R, p.S, p.BW);
            }

            HIPQ_PHASE(6);
            // ---- epilogue ------------------------------------------------------------------------
            // lane: channel ni*32 + lane%32; accumulator register 4g+e of tile ti is pixel
            // (4*wave + ti)*32 + 8g + 4*(lane/32) + e of the band
            const int64_t img_pix0 = static_cast<int64_t>(img) * p.PQ + static_cast<int64_t>(p0) * p.Q; // first pixel of the band, image-major
            if (KIND == OUT_Q8)
                __syncthreads(); // every wavefront is done reading the band: staging may overwrite it
            uint8_t* const stage = xs + wave * kBandStageWave;

            // FAST: requantization without a float rounding step (see the two branches below)
            auto epilogue = [&](auto fast_c, auto sum_c) {
                constexpr bool FAST = decltype(fast_c)::value;
                constexpr bool SUM = decltype(sum_c)::value;
                const float s256 = __fmul_rn(ec.scale, 256.0f);
                const int32_t c256 = 128 + 256 * ec.ozp;
                const float lo = fmaxf(ec.lo, ec.relu_floor);
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                {
                    const int n = ni * 32 + l32;
#pragma unroll
                    for (int ti = 0; ti < 4; ++ti)
                    {
#pragma unroll
                        for (int g = 0; g < 4; ++g)
                        {
                            const int lpix = ti * 32 + 8 * g + 4 * half; // pixel within the wavefront's 128
                            const int bpix = wave * 128 + lpix;         // pixel within the band
                            float s4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                            if (SUM && n < p.K && bpix < npix)
                            {
                                if (OUT_NCX)
                                    sum4(epi.sum_in, epi.sum_t, (static_cast<int64_t>(img) * p.K + n) * p.PQ + static_cast<int64_t>(p0) * p.Q + bpix, true, s4);
                                else
                                {
#pragma unroll
                                    for (int e = 0; e < 4; ++e)
                                        if (bpix + e < npix)
                                            s4[e] = static_cast<float>(load_q(epi.sum_in, epi.sum_t, (img_pix0 + bpix + e) * p.K + n));
                                }
                            }
                            // x[e]: the output byte sits in byte BYTE of x[e]
                            constexpr int BYTE = (MODE == EPI_INTERP && FAST && KIND == OUT_Q8) ? 1 : 0;
                            int32_t x[4];
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                            {
                                const int32_t a = acc[ti][ni][4 * g + e];
                                if (KIND != OUT_Q8)
                                    x[e] = epi_interp<KIND>(ec, a);
                                else if (MODE == EPI_INTERP && FAST)
                                {
                                    // t = trunc(256 v); round-half-away(v) = (t + 128 - (t < 0)) >> 8, exactly:
                                    // for t >= 0 it is floor(v + 1/2), for t < 0 it is ceil(v - 1/2)
                                    const int32_t t = static_cast<int32_t>(__fmul_rn(static_cast<float>(a), s256));
                                    x[e] = t + (t >> 31) + c256;
                                }
                                else if (MODE == EPI_INTERP)
                                    x[e] = epi_interp<KIND>(ec, a);
                                else
                                {
                                    float v = __fmul_rn(__fadd_rn(static_cast<float>(a), bias[ni]), scale[ni]);
                                    if (SUM)
                                        v = fmaf(ec.sum_scale, s4[e], v);
                                    v = __builtin_amdgcn_fmed3f(v, lo, ec.hi);
                                    // 1.5 * 2^23 + v rounds half-to-even into the low mantissa bits
                                    x[e] = __float_as_int(__fadd_rn(v, 12582912.0f));
                                }
                            }
                            if (KIND == OUT_Q8)
                            {
                                if (OUT_NCX)
                                {
                                    constexpr uint32_t sel = BYTE ? 0x0c0c0501u : 0x0c0c0400u;
                                    const uint32_t lo2 = __builtin_amdgcn_perm(x[1], x[0], sel);
                                    const uint32_t hi2 = __builtin_amdgcn_perm(x[3], x[2], sel);
                                    *reinterpret_cast<uint32_t*>(stage + n * kBandStagePitch + lpix) = (hi2 << 16) | lo2;
                                }
                                else
                                {
#pragma unroll
                                    for (int e = 0; e < 4; ++e)
                                        stage[(lpix + e) * 64 + n] = static_cast<uint8_t>(BYTE ? (x[e] >> 8) : x[e]);
                                }
                            }
                            else if (n < p.K && bpix < npix)
                            {
                                int32_t* o32 = static_cast<int32_t*>(out);
                                if (OUT_NCX) // npix, PQ and the band start are multiples of 4 (checked by the launcher)
                                    *reinterpret_cast<v4i*>(o32 + (static_cast<int64_t>(img) * p.K + n) * p.PQ + static_cast<int64_t>(p0) * p.Q + bpix) =
                                        v4i{x[0], x[1], x[2], x[3]};
                                else
                                {
#pragma unroll
                                    for (int e = 0; e < 4; ++e)
                                        if (bpix + e < npix)
                                            o32[(img_pix0 + bpix + e) * p.K + n] = x[e];
                                }
                            }
                        }
                    }
                }
            };
            using std::false_type;
            using std::true_type;
            if (MODE == EPI_FUSED)
            {
                if (has_sum)
                    epilogue(true_type{}, true_type{});
                else
                    epilogue(true_type{}, false_type{});
            }
            else if (KIND == OUT_Q8 && fast_interp)
                epilogue(true_type{}, false_type{});
            else
                epilogue(false_type{}, false_type{});

            HIPQ_PHASE(7);
            if (KIND == OUT_Q8)
            {
                // staging regions are wavefront-private and a wavefront's LDS accesses complete in order: no barrier
                uint8_t* o8 = static_cast<uint8_t*>(out);
                if (OUT_NCX)
                {
                    // 64 channel rows of 128 pixels: a lane moves 16 consecutive pixels of one channel
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                    {
                        const int id = j * 64 + lane;
                        const int ch = id >> 3;
                        const int part = id & 7;
                        const int bpix = wave * 128 + part * 16;
                        if (ch < p.K && bpix < npix)
                        {
                            const uint8_t* src = stage + ch * kBandStagePitch + part * 16;
                            uint8_t* dst = o8 + (static_cast<int64_t>(img) * p.K + ch) * p.PQ + static_cast<int64_t>(p0) * p.Q + bpix;
                            if (bpix + 16 <= npix)
                                __builtin_nontemporal_store(*reinterpret_cast<const v4i*>(src), reinterpret_cast<v4i*>(dst));
                            else
                                for (int e = 0; bpix + e < npix; ++e)
                                    dst[e] = src[e];
                        }
                    }
                }
                else
                {
                    // 128 pixel rows of 64 channels: a lane moves 16 consecutive channels of one pixel
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                    {
                        const int id = j * 64 + lane;
                        const int px = id >> 2;
                        const int part = id & 3;
                        const int bpix = wave * 128 + px;
                        if (bpix < npix && part * 16 < p.K)
                            __builtin_nontemporal_store(*reinterpret_cast<const v4i*>(stage + px * 64 + part * 16),
                                                        reinterpret_cast<v4i*>(o8 + (img_pix0 + bpix) * p.K + part * 16));
                    }
                }
            }
            HIPQ_PHASE(8);
            HIPQ_PHASE_NEXT();
        }
    }

    // rows per band and LDS bytes; false when the layer does not fit this kernel
    static bool band_plan(const ConvGeom& g, bool out_ncx, BandParams* bp, size_t* lds_bytes)
    {
        if (g.in[0] != 1 || g.f[0] != 1 || g.out[0] != 1)
            return false;
        if (g.C != kBandC || g.K > 64 || g.K % 16 != 0)
            return false;
        for (int i = 0; i < 3; ++i)
            if (g.st[i] != 1 || g.dl[i] != 1 || g.dd[i] != 1)
                return false;
        if (g.filter_t != HIPQ_I8 || (g.data_t != HIPQ_U8 && g.data_t != HIPQ_I8))
            return false;
        if (g.out_t != HIPQ_U8 && g.out_t != HIPQ_I8 && g.out_t != HIPQ_I32)
            return false;
        const int64_t R = g.f[1], S = g.f[2], P = g.out[1], Q = g.out[2];
        if (R * S > 25 || Q > 512 || Q < 1)
            return false;
        if (g.in_count() >= (1ll << 31) || g.out_count() >= (1ll << 31) || g.N * P >= (1ll << 30))
            return false;
        const int64_t wbytes = R * S * 64 * kBandC; // [tap][64][64]
        const int64_t BW = Q + S - 1;
        const int64_t budget = 79 * 1024; // two workgroups per CU
        int64_t best = 0;
        for (int64_t tp = 1; tp <= P && tp * Q <= 512; ++tp)
        {
            const int64_t band_bytes = (tp + R - 1) * BW * kBandC;
            const int64_t need = wbytes + (band_bytes > 4 * kBandStageWave ? band_bytes : 4 * kBandStageWave) + 16;
            if (need > budget)
                break;
            // full 32-pixel tiles and (for NCHW output) 16-byte aligned band starts
            const bool tidy = (tp * Q) % 32 == 0 || tp == P;
            if (tidy || best == 0)
                best = tp;
        }
        if (best == 0)
            return false;
        if (out_ncx && ((P * Q) % 16 != 0 || (best * Q) % 16 != 0))
            return false;
        if ((best * Q) % 4 != 0 && best != P)
            return false;
        const int64_t band_bytes = (best + R - 1) * BW * kBandC;
        bp->H = static_cast<int32_t>(g.in[1]);
        bp->W = static_cast<int32_t>(g.in[2]);
        bp->P = static_cast<int32_t>(P);
        bp->Q = static_cast<int32_t>(Q);
        bp->R = static_cast<int32_t>(R);
        bp->S = static_cast<int32_t>(S);
        bp->pbh = static_cast<int32_t>(g.pb[1]);
        bp->pbw = static_cast<int32_t>(g.pb[2]);
        bp->K = static_cast<int32_t>(g.K);
        bp->TP = static_cast<int32_t>(best);
        bp->bands = static_cast<int32_t>((P + best - 1) / best);
        bp->items = static_cast<int32_t>(g.N * bp->bands);
        bp->BW = static_cast<int32_t>(BW);
        bp->x_lds = static_cast<int32_t>(wbytes);
        bp->sink = static_cast<int32_t>(wbytes + (band_bytes > 4 * kBandStageWave ? band_bytes : 4 * kBandStageWave));
        bp->PQ = P * Q;
        bp->x_bytes = static_cast<uint32_t>(g.in_count());
        *lds_bytes = static_cast<size_t>(bp->sink) + 16;
        return true;
    }

    bool conv_band_eligible(const ConvGeom& g, bool out_ncx)
    {
        BandParams bp;
        size_t lds_bytes;
        return band_plan(g, out_ncx, &bp, &lds_bytes);
    }

    template <int MODE, int KIND, bool OUT_NCX>
    static int launch_band(const BandParams& bp, const ConvX& xl, size_t lds_bytes, const int8_t* w, const int32_t* wsum, int xu, const ZeroPoints& zp, const Epilogue& epi, void* out, hipStream_t s)
    {
        auto kernel = conv_band_kernel<MODE, KIND, OUT_NCX>;
        static size_t configured[16] = {};
        int dev = 0;
        HIPQ_HIP(hipGetDevice(&dev));
        if (dev >= 0 && dev < 16 && configured[dev] < lds_bytes)
        {
            HIPQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024));
            configured[dev] = 80 * 1024;
        }
        hipDeviceProp_t prop;
        static int cus[16] = {};
        if (dev >= 0 && dev < 16 && cus[dev] == 0)
        {
            HIPQ_HIP(hipGetDeviceProperties(&prop, dev));
            cus[dev] = prop.multiProcessorCount;
        }
        const int slots = 2 * (dev >= 0 && dev < 16 && cus[dev] > 0 ? cus[dev] : 256);
        const unsigned grid = static_cast<unsigned>(bp.items < slots ? bp.items : slots);
        kernel<<<grid, 256, lds_bytes, s>>>(bp, xl, w, wsum, xu, zp, epi, out);
        return check_launch("conv_band_i8_32x32x32");
    }

    int launch_conv_band(const ConvGeom& g,
                         const void* data_nxc,
                         const void* packed,
                         const ZeroPoints& zp,
                         const Epilogue& epi,
                         void* out,
                         bool out_ncx,
                         hipStream_t s)
    {
        BandParams bp;
        size_t lds_bytes = 0;
        HIPQ_REQUIRE(band_plan(g, out_ncx, &bp, &lds_bytes), "layer does not fit the band convolution");
        HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(data_nxc) & 15) == 0 && (reinterpret_cast<uintptr_t>(packed) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(out) & 15) == 0,
                     "band convolution needs 16-byte aligned tensors");
        bp.x = static_cast<const uint8_t*>(data_nxc);
        ConvX xl;
        xl.x = bp.x;
        xl.H = bp.H;
        xl.W = bp.W;
        xl.C = kBandC;
        xl.Q = bp.Q;
        xl.R = bp.R;
        xl.S = bp.S;
        xl.sh = xl.sw = xl.dh = xl.dw = 1;
        xl.pbh = bp.pbh;
        xl.pbw = bp.pbw;
        xl.PQ = bp.PQ;
        xl.bytes = bp.x_bytes;
        const int kred = bp.R * bp.S * kBandC;
        const int8_t* w = static_cast<const int8_t*>(packed);
        const int32_t* wsum = reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(packed) + align_up(static_cast<size_t>(g.K) * kred, 256));
        const int xu = g.data_t == HIPQ_U8 ? 1 : 0;
        const bool q8 = g.out_t == HIPQ_U8 || g.out_t == HIPQ_I8;
#define BAND(MODE, KIND)                                                                           \
    (out_ncx ? launch_band<MODE, KIND, true>(bp, xl, lds_bytes, w, wsum, xu, zp, epi, out, s)          \
             : launch_band<MODE, KIND, false>(bp, xl, lds_bytes, w, wsum, xu, zp, epi, out, s))
        if (epi.mode == EPI_INTERP)
            return q8 ? BAND(EPI_INTERP, OUT_Q8) : BAND(EPI_INTERP, OUT_I32);
        if (q8)
            return BAND(EPI_FUSED, OUT_Q8);
#undef BAND
        return fail(HIPQ_ERR_UNSUPPORTED, "no band kernel for this epilogue / output type");
    }
}
