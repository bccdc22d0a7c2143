// A network's first convolution -- at most four input channels, 64 output channels, a filter of up
// to 8 x 8 taps walking two pixels a step -- with the oneDNN-style epilogue (bias, scale per channel,
// ReLU, round half to even, saturate to u8), optionally followed by a MaxPool over its own output,
// as one kernel with the image band resident in LDS:
//
//   * a work item is a band of output rows of one image; persistent workgroups of eight wavefronts
//     walk the items;
//   * the band's input rows are read straight from the [N][C][H][W] bytes (one dword of four pixels
//     from each channel plane a lane), interleaved to four bytes a pixel, sign-flipped for the
//     signed MFMA and written to LDS with the padding materialised; the next band's loads are issued
//     before the current band is multiplied and land in the second buffer after it;
//   * the filter lives in registers for the whole kernel as MFMA fragments: row r of the filter is
//     one 32-byte reduction step (8 taps x 4 channels, taps past S and channels past C weigh zero),
//     so an output pixel's operand for step r is 32 contiguous bytes of LDS row (y * stride + r);
//   * v_mfma_i32_32x32x32_i8 with the filter as the first operand: a lane ends up with four
//     consecutive channels of one pixel per accumulator group, requantizes them with one
//     v_cvt_pk_u8_f32 each, trades halves with the other half-wavefront (v_permlane32_swap) and
//     holds 32 contiguous bytes of its pixel's channels-last row;
//   * without a pool those leave for global memory; with one they go to a band of convolution rows
//     in LDS, from which the pooled rows are reduced (sixteen channels a lane) and written.  The
//     convolution's own output never reaches memory.  Bands overlap by the pool window's overhang
//     (one convolution row in nine for 3 x 3 / 2), which is recomputed.
//
// The accumulators start from (128 * sum of the channel's weights + bias): the correction for
// running u8 data as signed bytes and the bias join the MFMA's addend, which is exact while
// |accumulator| and |bias| stay within 2^24 (float(a) + float(b) is then float(a + b)); a bias beyond
// that sends the band through a scalar loop with the reference arithmetic instead.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include "hipq_igemm.h"

namespace hipq
{
    namespace
    {
        constexpr int kStemThreads = 512;
        constexpr int kConvPixel = 80;  // bytes between the pixels of a band's convolution rows in LDS
        constexpr size_t kStemLdsLimit = 159 * 1024; // dynamic LDS a workgroup may ask for (the kernel has a little static LDS of its own)

        struct StemParams
        {
            const uint8_t* x;    // [N][C][H][W]
            const int8_t* w;     // row-packed filter [64][kp]
            const int32_t* wsum; // [64]
            uint8_t* out;        // [N][P][Q][64], or [N][PH][PW][64] with a pool
            int32_t C, H, W, R, S, sh, pad_h, pad_w, P, Q, kp;
            int32_t x_unsigned;
            int32_t band_rows; // rows of the result (pooled rows with a pool) a band produces
            int32_t bands;     // bands an image
            int32_t CR, IR;    // convolution rows / input rows a band holds
            int32_t pitch;     // bytes of an input row in LDS
            int32_t quads;     // W / 4
            int32_t n_tiles;   // 32-pixel tiles of a band's convolution rows
            int32_t items;     // N * bands
            FastDiv by_q, by_bands, by_quads, by_units, by_c;
            uint32_t x_bytes;  // N * C * H * W
            int32_t raw_bytes; // LDS staging area: IR * C * W, rounded up to whole wavefront loads
            // pool (window wh x ww, strides, padding above / left) and its result's extent
            int32_t PH, PW, wh, ww, psh, psw, ppt, ppl;
            FastDiv by_pw;
            // epilogue (fused policy, u8 output): bias may be null
            const int32_t* bias;
            const float* scale;
            int32_t per_channel, relu;
        };

        // byte-wise unsigned maximum of dwords: even and odd bytes in 16-bit lanes (the low byte of
        // an odd lane is along for the ride: it cannot change which high byte wins)
        typedef unsigned short stem_u16x2 __attribute__((ext_vector_type(2)));
        struct ByteMax
        {
            stem_u16x2 e = {0, 0}, o = {0, 0};
            __device__ __forceinline__ void add(uint32_t x)
            {
                e = __builtin_elementwise_max(e, __builtin_bit_cast(stem_u16x2, x & 0x00ff00ffu));
                o = __builtin_elementwise_max(o, __builtin_bit_cast(stem_u16x2, x));
            }
            __device__ __forceinline__ uint32_t bytes() const { return (__builtin_bit_cast(uint32_t, e) & 0x00ff00ffu) | (__builtin_bit_cast(uint32_t, o) & 0xff00ff00u); }
        };

        typedef int stem_v2i __attribute__((ext_vector_type(2)));

        // KS: reduction steps (filter rows, rounded up to a step count the kernel is built for; the
        // rows past R weigh zero and read LDS rows the band holds for that purpose)
        // UNIT: bytes a lane stages per load (16 when the image rows are whole 16-byte pieces, else 4)
        template <bool POOL, int KS, int UNIT>
        __global__ __launch_bounds__(kStemThreads) void conv_stem_kernel(const StemParams p)
        {
            extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
            const int tid = static_cast<int>(threadIdx.x);
            const int lane = tid & 63;
            const int half = lane >> 5;
            const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
            const int in_bytes = p.IR * p.pitch;
            uint8_t* const raw = lds + in_bytes;           // staged plane rows of the next band: [IR][C][W]
            uint8_t* const conv_rows = raw + p.raw_bytes;  // POOL: [CR][Q] pixels of kConvPixel bytes (64 channels, then a gap that spreads the pixels over the banks)
            int32_t* const consts = reinterpret_cast<int32_t*>(conv_rows + (POOL ? p.CR * p.Q * kConvPixel : 0)); // [64] start values, [64] scales
            const uint32_t flip = p.x_unsigned ? 0x80808080u : 0u;

            // ---- per-channel constants ----------------------------------------------------------
            bool fold;
            {
                int32_t b = 0;
                if (tid < 64)
                {
                    b = p.bias ? p.bias[tid] : 0;
                    consts[tid] = (p.x_unsigned ? 128 : 0) * p.wsum[tid] + b;
                    reinterpret_cast<float*>(consts)[64 + tid] = p.per_channel ? p.scale[tid] : p.scale[0];
                }
                fold = __syncthreads_and(b >= -(1 << 24) && b <= (1 << 24)) != 0;
            }
            // the band's rows start as padding everywhere; the loader only ever rewrites the columns of
            // the image, so the margins stay
            {
                const v4i fill4 = {static_cast<int>(flip), static_cast<int>(flip), static_cast<int>(flip), static_cast<int>(flip)};
                for (int i = tid; i < in_bytes / 16; i += kStemThreads)
                    reinterpret_cast<v4i*>(lds)[i] = fill4;
            }
            // the filter as MFMA fragments: lane (c = lane % 32, half) of block ni holds bytes
            // [32 r + 16 half, + 16) of filter row 32 ni + c
            v4i wf[KS][2];
#pragma unroll
            for (int r = 0; r < KS; ++r)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    wf[r][ni] = r < p.R ? *reinterpret_cast<const v4i*>(p.w + (ni * 32 + (lane & 31)) * p.kp + r * 32 + half * 16) : v4i{0, 0, 0, 0};
            // a lane's accumulator register 4 g + e of block ni is channel 32 ni + 8 g + 4 half + e
            // the fragments have arrived before the first tile: a wait for them inside the tile loop
            // would also wait for the next band's rows, which the compiler does not know are in flight
#pragma unroll
            for (int r = 0; r < KS; ++r)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    asm volatile("" ::"v"(wf[r][ni]));
            // (the start values stay in registers; the scales are read back from LDS tile by tile)
            v16i start[2];
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                {
                    const v4i c4 = *reinterpret_cast<const v4i*>(consts + ni * 32 + 8 * g + 4 * half);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        start[ni][4 * g + e] = c4[e];
                }
            const float* const scales = reinterpret_cast<const float*>(consts) + 64 + 4 * half;

            // ---- loader ------------------------------------------------------------------------
            // A band's input rows travel in two steps.  (1) The raw bytes of its C x IR plane rows go
            // from global memory straight into an LDS staging area (loads with the lds modifier, one
            // dword or -- rows of whole 16-byte pieces -- four a lane), issued for the next band before
            // the current one is multiplied: no registers hold them, and the compiler, which does
            // not see them, has nothing to wait for in front of the tile loop.  A row outside the
            // image is out of the buffer's range and arrives as zeros, the fused ops' zero point.
            // (2) After the band's last tile the staged rows are interleaved to four bytes a pixel,
            // sign-flipped and written over the band's rows in place.
            const int raw_row = p.C * p.W; // staged bytes of one input row: its C plane rows
            const int raw_units = p.IR * raw_row / UNIT;
            const int units_a_row = p.W / UNIT;
            const v4i xrs = rsrc_words(p.x, p.x_bytes);
            const uint32_t raw_lds = lds_address(raw);
            auto band_of = [&](int item, int& n, int& first_row) {
                n = static_cast<int>(p.by_bands.div(static_cast<uint32_t>(item)));
                first_row = (item - n * p.bands) * p.band_rows;
            };
            // first convolution row a band holds (may lie above the image with a pool)
            auto conv_row0 = [&](int first_row) { return POOL ? first_row * p.psh - p.ppt : first_row; };
            auto issue = [&](int item) {
                int n, first_row;
                band_of(item, n, first_row);
                const int iy0 = conv_row0(first_row) * p.sh - p.pad_h;
                for (int k = wave; k * 64 < raw_units; k += kStemThreads / 64)
                {
                    const int u = k * 64 + lane; // unit u of the staging area: plane row u / units_a_row, piece u % units_a_row
                    const int pr = static_cast<int>(p.by_units.div(static_cast<uint32_t>(u)));
                    const int piece = u - pr * units_a_row;
                    const int r = static_cast<int>(p.by_c.div(static_cast<uint32_t>(pr)));
                    const int c = pr - r * p.C;
                    const int iy = iy0 + r;
                    const bool live = u < raw_units && iy >= 0 && iy < p.H;
                    const int32_t off = live ? ((n * p.C + c) * p.H + iy) * p.W + piece * UNIT : kOob;
                    const uint32_t base = __builtin_amdgcn_readfirstlane(raw_lds + static_cast<uint32_t>(k) * (64 * UNIT));
                    if (UNIT == 16)
                        lds_dma16(xrs, off, base);
                    else
                        asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, 0 offen lds" ::"s"(base), "v"(off), "s"(xrs) : "memory");
                }
            };
            auto commit = [&]() {
                for (int id = tid; id < p.IR * p.quads; id += kStemThreads)
                {
                    const int r = static_cast<int>(p.by_quads.div(static_cast<uint32_t>(id)));
                    const int q = id - r * p.quads;
                    const uint8_t* const src = raw + r * raw_row + 4 * q;
                    uint32_t ch[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        ch[c] = c < p.C ? *reinterpret_cast<const uint32_t*>(src + c * p.W) : 0u;
                    uint32_t* const o = reinterpret_cast<uint32_t*>(lds + r * p.pitch) + (4 * q + p.pad_w);
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                    {
                        const uint32_t lo = __builtin_amdgcn_perm(ch[1], ch[0], 0x0c0c0400u + 0x0101u * t); // bytes t of channels 0, 1
                        const uint32_t hi = __builtin_amdgcn_perm(ch[3], ch[2], 0x0c0c0400u + 0x0101u * t); // ... of channels 2, 3
                        o[t] = (lo | (hi << 16)) ^ flip;
                    }
                }
            };

            // ---- the slow, exact band (a bias the accumulators cannot carry) ---------------------
            auto slow_band = [&](int n, int cy0) {
                Epilogue epi;
                memset(&epi, 0, sizeof(epi));
                epi.mode = EPI_FUSED;
                epi.out_t = HIPQ_U8;
                epi.bias = p.bias;
                epi.scale = p.scale;
                epi.per_channel = p.per_channel;
                epi.relu = p.relu;
                const EpiRegs er = epi_load(epi);
                const uint8_t* const src = lds;
                const int total = p.CR * p.Q * 64;
                for (int i = tid; i < total; i += kStemThreads)
                {
                    const int ch = i & 63;
                    const uint32_t pix = static_cast<uint32_t>(i >> 6);
                    const int ly = static_cast<int>(p.by_q.div(pix));
                    const int x = static_cast<int>(pix) - ly * p.Q;
                    int32_t acc = 0;
                    for (int r = 0; r < p.R; ++r)
                        for (int s = 0; s < p.S; ++s)
                            for (int c = 0; c < p.C; ++c)
                            {
                                const uint8_t b = src[(ly * p.sh + r) * p.pitch + (2 * x + s) * 4 + c] ^ static_cast<uint8_t>(flip);
                                const int32_t a = p.x_unsigned ? static_cast<int32_t>(b) : static_cast<int32_t>(static_cast<int8_t>(b));
                                acc += a * static_cast<int32_t>(p.w[ch * p.kp + r * 32 + s * 4 + c]);
                            }
                    const uint8_t v = static_cast<uint8_t>(epi_apply(epi, er, acc, ch, 0));
                    if (POOL)
                        conv_rows[pix * kConvPixel + ch] = v;
                    else if (cy0 + ly < p.P)
                        p.out[((static_cast<int64_t>(n) * p.P + cy0 + ly) * p.Q + x) * 64 + ch] = v;
                }
            };

            // ---- items ---------------------------------------------------------------------------
            int item = static_cast<int>(blockIdx.x);
            if (item >= p.items)
                return;
            issue(item);
            wait_vmcnt<0>();
            __syncthreads(); // the padding fill is complete, the first band's rows are staged
            commit();
            __syncthreads();
            const int band_pixels = p.CR * p.Q;
            for (; item < p.items; item += static_cast<int>(gridDim.x))
            {
                const int next = item + static_cast<int>(gridDim.x);
                const bool has_next = next < p.items; // uniform
                if (has_next)
                    issue(next);
                int n, first_row;
                band_of(item, n, first_row);
                const int cy0 = conv_row0(first_row);
                const uint8_t* const src = lds;
                if (!fold)
                    slow_band(n, cy0);
                else
                    for (int t = wave; t < p.n_tiles; t += kStemThreads / 64)
                    {
                        const int pix_raw = t * 32 + (lane & 31);
                        const uint32_t pix = static_cast<uint32_t>(pix_raw < band_pixels ? pix_raw : band_pixels - 1);
                        const int ly = static_cast<int>(p.by_q.div(pix));
                        const int x = static_cast<int>(pix) - ly * p.Q;
                        const uint8_t* const a0 = src + ly * p.sh * p.pitch + 8 * x + 16 * half;
                        v16i acc[2];
                        v4i xf[KS];
#pragma unroll
                        for (int r = 0; r < KS; ++r)
                        {
                            const stem_v2i lo = *reinterpret_cast<const stem_v2i*>(a0 + r * p.pitch);
                            const stem_v2i hi = *reinterpret_cast<const stem_v2i*>(a0 + r * p.pitch + 8);
                            xf[r] = v4i{lo[0], lo[1], hi[0], hi[1]};
                        }
#pragma unroll
                        for (int r = 0; r < KS; ++r)
#pragma unroll
                            for (int ni = 0; ni < 2; ++ni)
                                acc[ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[r][ni], xf[r], r == 0 ? start[ni] : acc[ni], 0, 0, 0);
                        // requantize: dword (ni, g) of a lane is channels 32 ni + 8 g + 4 half .. + 3 of its pixel
                        uint32_t d[2][4];
#pragma unroll
                        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                            for (int g = 0; g < 4; ++g)
                            {
                                const v4f s4 = *reinterpret_cast<const v4f*>(scales + ni * 32 + 8 * g);
                                uint32_t packed = 0;
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    packed = __builtin_amdgcn_cvt_pk_u8_f32(__fmul_rn(static_cast<float>(acc[ni][4 * g + e]), s4[e]), e, packed);
                                d[ni][g] = packed;
                            }
                        // the lower half-wavefront collects channels 0 .. 31 of its pixel, the upper 32 .. 63
                        v4i piece[2];
#pragma unroll
                        for (int g = 0; g < 4; ++g)
                        {
                            const auto sw = __builtin_amdgcn_permlane32_swap(d[0][g], d[1][g], false, false);
                            piece[g >> 1][(g & 1) * 2] = static_cast<int>(sw[0]);
                            piece[g >> 1][(g & 1) * 2 + 1] = static_cast<int>(sw[1]);
                        }
                        if (pix_raw < band_pixels)
                        {
                            if (POOL)
                            {
                                v4i* const o = reinterpret_cast<v4i*>(conv_rows + pix * kConvPixel + 32 * half);
                                o[0] = piece[0];
                                o[1] = piece[1];
                            }
                            else if (cy0 + ly < p.P)
                            {
                                v4i* const o = reinterpret_cast<v4i*>(p.out + ((static_cast<int64_t>(n) * p.P + cy0 + ly) * p.Q + x) * 64 + 32 * half);
                                o[0] = piece[0];
                                o[1] = piece[1];
                            }
                        }
                    }
                wait_vmcnt<0>(); // this wavefront's share of the next band's rows has landed
                __syncthreads(); // the band's convolution rows are in LDS; its input rows are free
                if (has_next)
                    commit();
                if (POOL)
                {
                    const int rows = p.PH - first_row < p.band_rows ? p.PH - first_row : p.band_rows;
                    const int tasks = rows * p.PW * 4; // (pooled row, pooled column, 16 channels)
                    for (int t = tid; t < tasks; t += kStemThreads)
                    {
                        const int cg = t & 3;
                        const uint32_t pp = static_cast<uint32_t>(t >> 2);
                        const int pr = static_cast<int>(p.by_pw.div(pp));
                        const int pc = static_cast<int>(pp) - pr * p.PW;
                        const int r0 = (first_row + pr) * p.psh - p.ppt; // convolution row / column of the window's corner
                        const int c0 = pc * p.psw - p.ppl;
                        // a cell outside the window or the tensor is replaced by the nearest one inside both
                        // (every window holds one): a maximum does not mind seeing a cell twice, and
                        // the nine reads go out together
                        const int ylo = r0 < 0 ? 0 : r0, yhi = (r0 + p.wh < p.P ? r0 + p.wh : p.P) - 1;
                        const int xlo = c0 < 0 ? 0 : c0, xhi = (c0 + p.ww < p.Q ? c0 + p.ww : p.Q) - 1;
                        v4i cell[9];
#pragma unroll
                        for (int wy = 0; wy < 3; ++wy)
#pragma unroll
                            for (int wx = 0; wx < 3; ++wx)
                            {
                                int cy = r0 + wy, cx = c0 + wx;
                                cy = cy < ylo ? ylo : (cy > yhi ? yhi : cy);
                                cx = cx < xlo ? xlo : (cx > xhi ? xhi : cx);
                                cell[wy * 3 + wx] = *reinterpret_cast<const v4i*>(conv_rows + ((cy - cy0) * p.Q + cx) * kConvPixel + 16 * cg);
                            }
                        ByteMax m[4];
#pragma unroll
                        for (int c = 0; c < 9; ++c)
#pragma unroll
                            for (int j = 0; j < 4; ++j)
                                m[j].add(static_cast<uint32_t>(cell[c][j]));
                        const v4i r = {static_cast<int>(m[0].bytes()), static_cast<int>(m[1].bytes()), static_cast<int>(m[2].bytes()), static_cast<int>(m[3].bytes())};
                        *reinterpret_cast<v4i*>(p.out + ((static_cast<int64_t>(n) * p.PH + first_row + pr) * p.PW + pc) * 64 + 16 * cg) = r;
                    }
                }
                __syncthreads(); // the next band is in place; nobody reads this band's convolution rows any more
            }
        }

        // reduction steps the kernel is built for: 3, 5, 7 or 8
        int stem_steps(int R) { return R <= 3 ? 3 : (R <= 5 ? 5 : (R <= 7 ? 7 : 8)); }

        bool stem_plan(const ConvGeom& g, const Epilogue& epi, const ZeroPoints& zp, const PoolFuse* pool, StemParams* out, size_t* lds_bytes)
        {
            if (g.in[0] != 1 || g.f[0] != 1 || g.out[0] != 1)
                return false;
            for (int i = 0; i < 3; ++i)
                if (g.dd[i] != 1 || g.dl[i] != 1)
                    return false;
            if (g.filter_t != HIPQ_I8 || (g.data_t != HIPQ_U8 && g.data_t != HIPQ_I8) || g.out_t != HIPQ_U8)
                return false;
            if (epi.mode != EPI_FUSED || epi.sum_in != nullptr || epi.post_scale != nullptr || zp.data_zp != nullptr || zp.filter_zp != nullptr)
                return false;
            if (g.data_layout != HIPQ_LAYOUT_NCX || g.out_layout != HIPQ_LAYOUT_NXC)
                return false;
            if (g.C < 1 || g.C > 4 || g.K != 64 || g.f[1] < 1 || g.f[1] > 8 || g.f[2] < 1 || g.f[2] > 8 || g.st[2] != 2 || g.st[1] < 1 || g.st[1] > 2)
                return false;
            if (g.pb[1] < 0 || g.pb[2] < 0 || g.pb[1] > 8 || g.pb[2] > 8 || g.in[2] % 4 != 0 || g.out[1] < 1 || g.out[2] < 1 || g.N < 1)
                return false;
            if (g.in_count() >= (1ll << 31) || g.out_count() >= (1ll << 31) || g.in[2] > 4096 || g.in[1] > (1 << 20))
                return false;
            if (getenv("HIPQ_NO_STEM") != nullptr)
                return false;
            StemParams p;
            memset(&p, 0, sizeof(p));
            p.C = static_cast<int32_t>(g.C);
            p.H = static_cast<int32_t>(g.in[1]);
            p.W = static_cast<int32_t>(g.in[2]);
            p.R = static_cast<int32_t>(g.f[1]);
            p.S = static_cast<int32_t>(g.f[2]);
            p.sh = static_cast<int32_t>(g.st[1]);
            p.pad_h = static_cast<int32_t>(g.pb[1]);
            p.pad_w = static_cast<int32_t>(g.pb[2]);
            p.P = static_cast<int32_t>(g.out[1]);
            p.Q = static_cast<int32_t>(g.out[2]);
            p.kp = static_cast<int32_t>(align_up(static_cast<size_t>(g.f[1] * 32), 64));
            p.x_unsigned = g.data_t == HIPQ_U8 ? 1 : 0;
            p.quads = p.W / 4;
            const int64_t lds_pixels = std::max<int64_t>((p.Q - 1) * 2 + 8, p.pad_w + p.W);
            p.pitch = static_cast<int32_t>(align_up(static_cast<size_t>(lds_pixels * 4), 16) + 16);
            int64_t out_rows;
            if (pool)
            {
                if (pool->wh < 1 || pool->wh > 3 || pool->ww < 1 || pool->ww > 3 || pool->sh < 1 || pool->sh > 3 || pool->sw < 1 || pool->sw > 3 || pool->pt < 0 || pool->pl < 0 ||
                    pool->pt >= pool->wh || pool->pl >= pool->ww || pool->out_h < 1 || pool->out_w < 1)
                    return false;
                // every window must hold a cell of the convolution's output
                if ((pool->out_h - 1) * pool->sh - pool->pt >= p.P || (pool->out_w - 1) * pool->sw - pool->pl >= p.Q)
                    return false;
                if (g.N * pool->out_h * pool->out_w * 64 >= (1ll << 31))
                    return false;
                p.PH = static_cast<int32_t>(pool->out_h);
                p.PW = static_cast<int32_t>(pool->out_w);
                p.wh = static_cast<int32_t>(pool->wh);
                p.ww = static_cast<int32_t>(pool->ww);
                p.psh = static_cast<int32_t>(pool->sh);
                p.psw = static_cast<int32_t>(pool->sw);
                p.ppt = static_cast<int32_t>(pool->pt);
                p.ppl = static_cast<int32_t>(pool->pl);
                p.by_pw = fast_div(p.PW);
                out_rows = p.PH;
            }
            else
                out_rows = p.P;
            // the largest band that fits LDS and the loader's registers
            bool found = false;
            for (int rows = pool ? 4 : 8; rows >= 1; rows >>= 1)
            {
                const int64_t CR = pool ? static_cast<int64_t>(rows - 1) * p.psh + p.wh : rows;
                const int64_t IR = (CR - 1) * p.sh + stem_steps(p.R);
                const size_t raw_bytes = align_up(static_cast<size_t>(IR * p.C * p.W), 1024);
                const size_t need = static_cast<size_t>(IR * p.pitch) + raw_bytes + (pool ? static_cast<size_t>(CR * p.Q * kConvPixel) : 0) + 512;
                if (need > kStemLdsLimit)
                    continue;
                p.raw_bytes = static_cast<int32_t>(raw_bytes);
                p.band_rows = rows;
                p.CR = static_cast<int32_t>(CR);
                p.IR = static_cast<int32_t>(IR);
                *lds_bytes = need;
                found = true;
                break;
            }
            if (!found)
                return false;
            p.bands = static_cast<int32_t>((out_rows + p.band_rows - 1) / p.band_rows);
            p.n_tiles = (p.CR * p.Q + 31) / 32;
            if (g.N * p.bands >= (1ll << 30))
                return false;
            p.items = static_cast<int32_t>(g.N * p.bands);
            p.by_q = fast_div(p.Q);
            p.by_bands = fast_div(p.bands);
            p.by_quads = fast_div(p.quads);
            p.by_c = fast_div(p.C);
            p.x_bytes = static_cast<uint32_t>(g.in_count());
            *out = p;
            return true;
        }
    }

    bool conv_stem_eligible(const ConvGeom& g, const Epilogue& epi, const ZeroPoints& zp, const PoolFuse* pool)
    {
        StemParams p;
        size_t lds_bytes = 0;
        return stem_plan(g, epi, zp, pool, &p, &lds_bytes);
    }

    int launch_conv_stem(const ConvGeom& g, const void* data, const void* packed, const ZeroPoints& zp, const Epilogue& epi, const PoolFuse* pool, void* out, hipStream_t s)
    {
        StemParams p;
        size_t lds_bytes = 0;
        HIPQ_REQUIRE(stem_plan(g, epi, zp, pool, &p, &lds_bytes), "layer does not fit the first-layer band convolution");
        HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(data) & 3) == 0 && (reinterpret_cast<uintptr_t>(packed) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0,
                     "first-layer band convolution: data must be 4-byte aligned, packed filter and output 16-byte aligned");
        p.x = static_cast<const uint8_t*>(data);
        p.w = static_cast<const int8_t*>(packed);
        p.wsum = reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(packed) + align_up(static_cast<size_t>(g.K) * p.kp, 256));
        p.out = static_cast<uint8_t*>(out);
        p.bias = epi.bias;
        p.scale = epi.scale;
        p.per_channel = epi.per_channel;
        p.relu = epi.relu;
        const unsigned grid = static_cast<unsigned>(std::min<int64_t>(p.items, device_compute_units()));
        int rc = HIPQ_OK;
        auto go = [&](auto kernel, int slot) {
            static bool configured[16][16] = {};
            int dev = 0;
            if (hipGetDevice(&dev) != hipSuccess)
            {
                rc = fail(HIPQ_ERR_HIP, "hipGetDevice failed");
                return;
            }
            if (dev >= 0 && dev < 16 && !configured[slot][dev])
            {
                if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kStemLdsLimit)) != hipSuccess)
                {
                    rc = fail(HIPQ_ERR_HIP, "cannot raise the LDS limit of the first-layer kernel");
                    return;
                }
                configured[slot][dev] = true;
            }
            kernel<<<grid, kStemThreads, lds_bytes, s>>>(p);
        };
        const int ks = stem_steps(p.R);
        const bool wide = p.W % 16 == 0 && (reinterpret_cast<uintptr_t>(data) & 15) == 0; // image rows in whole 16-byte pieces
        p.by_units = fast_div(p.W / (wide ? 16 : 4));
        auto pick = [&](auto pooled, int slot0) {
            constexpr bool P = decltype(pooled)::value;
            switch (ks)
            {
            case 3: wide ? go(conv_stem_kernel<P, 3, 16>, slot0 + 0) : go(conv_stem_kernel<P, 3, 4>, slot0 + 1); break;
            case 5: wide ? go(conv_stem_kernel<P, 5, 16>, slot0 + 2) : go(conv_stem_kernel<P, 5, 4>, slot0 + 3); break;
            case 7: wide ? go(conv_stem_kernel<P, 7, 16>, slot0 + 4) : go(conv_stem_kernel<P, 7, 4>, slot0 + 5); break;
            default: wide ? go(conv_stem_kernel<P, 8, 16>, slot0 + 6) : go(conv_stem_kernel<P, 8, 4>, slot0 + 7); break;
            }
        };
        if (pool)
        {
            pick(std::true_type{}, 0);
            return rc ? rc : check_launch("conv_stem_pool_i8_32x32x32");
        }
        pick(std::false_type{}, 8);
        return rc ? rc : check_launch("conv_stem_i8_32x32x32");
    }
}
