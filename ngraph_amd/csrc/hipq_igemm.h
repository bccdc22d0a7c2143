// int8 GEMM and implicit-GEMM convolution on the CDNA4 i8 matrix cores (v_mfma_i32_32x32x32_i8).
//
// out[m][n] = epilogue( sum_k (x[m][k] - x_zp) * w[n][k] )
//   x : the activation operand.  GEMM: a row-major [M][K] matrix.  Convolution: gathered on the
//       fly from channels-last data, m = (image, out_y, out_x), k = (filter_y, filter_x, channel).
//   w : the weights as [N][K] int8, K contiguous (for convolution: K,spatial,C order).
//
// The matrix cores multiply signed by signed bytes only, so unsigned activations are biased:
// x' = x ^ 0x80 = x - 128, and since  sum (x - zp) w = sum x' w + (128 - zp) * sum w  the
// kernel adds (128 - zp) * wsum[n] to each accumulator.  Padding taps are materialised as the
// byte `zp` (a real element equal to the zero point), which contributes (zp - zp) * w = 0 exactly
// as the reference's skipped tap does.
//
// Work split: a workgroup of 4 wavefronts computes a BM (m) x BN (n) tile; each wavefront owns
// WM x WN MFMA tiles of 32 x 32.  Large per-wave tiles keep LDS reads (the scarce resource next to
// the matrix cores) low: a 128 x 64 wave tile reads 6 KiB of LDS per 8 MFMAs.  Operands are staged
// through LDS in 64-byte K slices, double buffered: global loads of slice i+1 are in flight while
// slice i feeds the MFMAs.  LDS rows are 64 bytes with the 16-byte chunk index XOR-swizzled by
// (row >> 1) & 3, which makes both the 16-byte stores and the 16-byte fragment reads free of bank
// conflicts.
//
// Which operand feeds MFMA source A decides what a lane's four consecutive accumulator registers
// are: with the weights on A they are four consecutive output channels of one pixel (one 4-byte
// store into a channels-last / row-major output); with the activations on A they are four
// consecutive pixels of one channel (one 4-byte store into an NCHW output).
//
// Workgroup ids are remapped so that each of the 8 XCDs (which receive consecutive ids round-robin
// and have private L2s) works on a contiguous range of m tiles.
#pragma once
#include <type_traits>

#include "hipq_common.h"
#include "hipq_quant_math.h"
#include "hipq_row_math.h"

namespace hipq
{
    typedef int v4i __attribute__((ext_vector_type(4)));
    typedef float v4f __attribute__((ext_vector_type(4)));
    typedef int v16i __attribute__((ext_vector_type(16)));

    constexpr int BK = 64; // reduction bytes per LDS slice

    // A ds_read_b128 is served 16 lanes at a time from 64 banks: full rate needs 16 consecutive rows
    // at one chunk index in 16 different 16-byte columns of a 256-byte line.  Rows r, r+4, r+8, r+12
    // share a 64-byte column group, hence the rotation by (r / 4) % 4 (measured 190 B/clk/CU; a
    // rotation by (r / 2) % 4 gives 128, none 64).
    __device__ __forceinline__ int lds_offset(int row, int chunk)
    {
        return row * BK + ((chunk ^ ((row >> 2) & 3)) << 4);
    }

    // ---- activation loaders ---------------------------------------------------------------------
    // All tile loads are raw buffer loads: the hardware range check returns zeros for an offset
    // beyond the buffer, so an out-of-range chunk (row beyond M, tap in the padding, K tail) is
    // simply given the offset kOob -- no branch, and all loads of a slice issue back to back.
    constexpr int32_t kOob = static_cast<int32_t>(0x80000000u);

    __device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes)
    {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, static_cast<int>(bytes), 0x00020000);
    }

    __device__ __forceinline__ v4i buffer_load16(__amdgpu_buffer_rsrc_t r, int32_t off)
    {
        return __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    }

    // Division of a value below 2^31 by a divisor fixed at launch (1 <= d < 2^31), exact:
    // with l = ceil(log2 d) and m = 2^(31 + l) / d + 1, n / d = hi32(n * m) >> (l - 1).
    struct FastDiv
    {
        uint32_t m, sh; // m == 0: d == 1
        __device__ __forceinline__ uint32_t div(uint32_t n) const { return m ? __umulhi(n, m) >> sh : n; }
    };
    static inline FastDiv fast_div(int64_t d)
    {
        FastDiv r{0u, 0u};
        if (d <= 1)
            return r;
        int l = 0;
        while ((1ll << l) < d)
            ++l;
        r.m = static_cast<uint32_t>((1ull << (31 + l)) / static_cast<uint64_t>(d) + 1);
        r.sh = static_cast<uint32_t>(l - 1);
        return r;
    }

    // ---- loads straight into LDS -----------------------------------------------------------------
    __device__ __forceinline__ v4i rsrc_words(const void* p, uint32_t bytes)
    {
        const uint64_t a = reinterpret_cast<uint64_t>(p);
        return v4i{static_cast<int>(a), static_cast<int>((a >> 32) & 0xffffu), static_cast<int>(bytes), 0x00020000};
    }
    __device__ __forceinline__ uint32_t lds_address(const void* p)
    {
        return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const uint8_t*)p));
    }
    // every lane's 16 bytes at `off` of the buffer go to LDS address lds_base + 16 * lane (zeros
    // when `off` is out of range); lds_base is uniform.  Counted by vmcnt like any load.
    __device__ __forceinline__ void lds_dma16(v4i rsrc, int32_t off, uint32_t lds_base)
    {
        asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_base), "v"(off), "s"(rsrc) : "memory");
    }
    // The same load without the compiler-level memory barrier, for kernels that bracket their LDS
    // traffic with barriers of their own (every fragment read sits behind a wait_vmcnt, every load
    // that overwrites a region behind the waited-for reads of that region).  A barrier on every load
    // makes the compiler treat all of memory as changed behind it: uniform loads that follow can no
    // longer go through the scalar cache and land in the vector queue behind the operand stream.
    __device__ __forceinline__ void lds_dma16_unfenced(v4i rsrc, int32_t off, uint32_t lds_base)
    {
        asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_base), "v"(off), "s"(rsrc));
    }
    template <int N>
    __device__ __forceinline__ void wait_vmcnt()
    {
        static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
    }

    struct GemmX
    {
        const uint8_t* x;
        int32_t K;
        uint32_t bytes; // M * K
        static constexpr bool kUniform = false;
        static constexpr bool kFloatOut = false;
        static constexpr bool kPads = false; // (only read by the kernels that load straight into LDS)

        struct Row
        {
            int32_t off; // byte offset of the row, kOob when beyond M
        };
        struct Cursor
        {
            int32_t kbyte;
        };
        __device__ __forceinline__ void init_row(Row& r, int64_t m, int64_t M) const { r.off = m < M ? static_cast<int32_t>(m) * K : kOob; }
        __device__ __forceinline__ void init_cursor(Cursor& c, int kbyte) const { c.kbyte = kbyte; }
        __device__ __forceinline__ void advance(Cursor& c, int bytes_) const { c.kbyte += bytes_; }
        __device__ __forceinline__ int32_t offset(const Row& r, const Cursor& c) const
        {
            return (r.off != kOob && c.kbyte < K) ? r.off + c.kbyte : kOob;
        }
        // slow path: exact accumulator of one output, any zero points
        __device__ __forceinline__ int32_t direct(int64_t m, const int8_t* wrow, int32_t xzp, int32_t wzp, bool x_unsigned) const
        {
            const uint8_t* p = x + m * static_cast<int64_t>(K);
            int32_t acc = 0;
            for (int32_t k = 0; k < K; ++k)
            {
                int32_t a = x_unsigned ? static_cast<int32_t>(p[k]) : static_cast<int32_t>(static_cast<int8_t>(p[k]));
                acc += (a - xzp) * (static_cast<int32_t>(wrow[k]) - wzp);
            }
            return acc;
        }
    };

    struct ConvX
    {
        static constexpr bool kUniform = false;
        static constexpr bool kFloatOut = false;
        static constexpr bool kPads = false; // (only read by the kernels that load straight into LDS)
        const uint8_t* x; // [N][H][W][C]
        int32_t H, W, C, Q, R, S, sh, sw, dh, dw, pbh, pbw;
        int64_t PQ;
        uint32_t bytes; // N * H * W * C
        FastDiv by_pq, by_q, by_c, by_s; // by_pq.sh == 0xffffffff: more than 2^31 output pixels, plain division

        struct Row
        {
            int32_t base; // byte offset of the image, kOob when beyond M
            int32_t yx;   // (top input row << 16) | (left input column & 0xffff) of the window
        };
        struct Cursor
        {
            int32_t r, s, c;
        };
        __device__ __forceinline__ void init_row(Row& rw, int64_t m, int64_t M) const
        {
            const bool valid = m < M;
            const int64_t mm = valid ? m : 0;
            int32_t n, rem;
            if (by_pq.sh == 0xffffffffu) // uniform
            {
                const int64_t n64 = mm / PQ;
                n = static_cast<int32_t>(n64);
                rem = static_cast<int32_t>(mm - n64 * PQ);
            }
            else
            {
                n = static_cast<int32_t>(by_pq.div(static_cast<uint32_t>(mm)));
                rem = static_cast<int32_t>(mm) - n * static_cast<int32_t>(PQ);
            }
            const int32_t p = static_cast<int32_t>(by_q.div(static_cast<uint32_t>(rem)));
            const int32_t q = rem - p * Q;
            rw.base = valid ? n * H * W * C : kOob;
            rw.yx = ((p * sh - pbh) << 16) | ((q * sw - pbw) & 0xffff);
        }
        __device__ __forceinline__ void init_cursor(Cursor& c, int kbyte) const
        {
            const int tap = static_cast<int>(by_c.div(static_cast<uint32_t>(kbyte)));
            c.c = kbyte - tap * C;
            c.r = static_cast<int>(by_s.div(static_cast<uint32_t>(tap)));
            c.s = tap - c.r * S;
        }
        __device__ __forceinline__ void advance(Cursor& c, int bytes_) const
        {
            c.c += bytes_;
            while (c.c >= C)
            {
                c.c -= C;
                if (++c.s == S)
                {
                    c.s = 0;
                    ++c.r;
                }
            }
        }
        __device__ __forceinline__ int32_t offset(const Row& rw, const Cursor& c) const
        {
            const int32_t y = (rw.yx >> 16) + c.r * dh;
            const int32_t xx = static_cast<int16_t>(rw.yx & 0xffff) + c.s * dw;
            const bool ok = (rw.base != kOob) & (c.r < R) & (static_cast<uint32_t>(y) < static_cast<uint32_t>(H)) &
                            (static_cast<uint32_t>(xx) < static_cast<uint32_t>(W));
            return ok ? rw.base + (y * W + xx) * C + c.c : kOob;
        }
        __device__ __forceinline__ int32_t direct(int64_t m, const int8_t* wrow, int32_t xzp, int32_t wzp, bool x_unsigned) const
        {
            Row rw;
            init_row(rw, m, m + 1);
            const int32_t iy0 = rw.yx >> 16, ix0 = static_cast<int16_t>(rw.yx & 0xffff);
            int32_t acc = 0;
            for (int32_t r = 0; r < R; ++r)
                for (int32_t s = 0; s < S; ++s)
                {
                    int32_t y = iy0 + r * dh, xx = ix0 + s * dw;
                    if (static_cast<uint32_t>(y) >= static_cast<uint32_t>(H) || static_cast<uint32_t>(xx) >= static_cast<uint32_t>(W))
                        continue;
                    const uint8_t* p = x + rw.base + (y * W + xx) * C;
                    const int8_t* wp = wrow + (r * S + s) * C;
                    for (int32_t c = 0; c < C; ++c)
                    {
                        int32_t a = x_unsigned ? static_cast<int32_t>(p[c]) : static_cast<int32_t>(static_cast<int8_t>(p[c]));
                        acc += (a - xzp) * (static_cast<int32_t>(wp[c]) - wzp);
                    }
                }
            return acc;
        }
    };

    // ---- loaders of the kernels that load straight into LDS -------------------------------------
    // Their reduction cursor is the same for every lane of the workgroup (scalar registers); a lane
    // adds the offset of its own 16-byte chunk.
    struct RowsU
    {
        const uint8_t* x;
        int32_t K;
        uint32_t bytes; // M * K
        static constexpr bool kUniform = true;
        static constexpr bool kFloatOut = true; // GEMM outputs may be floats; also: the loader is light enough on registers for three workgroups per compute unit
        static constexpr bool kDeep = true;     // 128-byte-deep slices are possible
        bool deep_ok() const { return true; }
        static constexpr bool kPads = false; // no reads of padding: an out-of-range chunk is never used
        struct Row
        {
            int32_t off;
        };
        struct Cursor
        {
            int32_t kbyte;
        };
        __device__ __forceinline__ void init_row(Row& r, int64_t m, int64_t M) const { r.off = m < M ? static_cast<int32_t>(m) * K : kOob; }
        __device__ __forceinline__ void init_cursor(Cursor& c, int kbyte) const { c.kbyte = kbyte; }
        __device__ __forceinline__ void advance(Cursor& c, int bytes_) const { c.kbyte += bytes_; }
        __device__ __forceinline__ int32_t offset(const Row& r, const Cursor& c, int lane_bytes) const
        {
            return (r.off != kOob && c.kbyte + lane_bytes < K) ? r.off + c.kbyte + lane_bytes : kOob;
        }
        __device__ __forceinline__ int32_t direct(int64_t m, const int8_t* wrow, int32_t xzp, int32_t wzp, bool x_unsigned) const
        {
            GemmX g{x, K, bytes};
            return g.direct(m, wrow, xzp, wzp, x_unsigned);
        }
    };

    // channels-last convolution whose channel count is a multiple of 64: a 64-byte slice lies inside one tap
    struct ConvU
    {
        ConvX cx;
        const uint8_t* x; // = cx.x
        uint32_t bytes;   // = cx.bytes
        static constexpr bool kUniform = true;
        static constexpr bool kFloatOut = false;
        static constexpr bool kDeep = true;
        bool deep_ok() const { return cx.C % 128 == 0; } // a 128-byte slice then lies inside one tap
        static constexpr bool kPads = true;
        struct Row
        {
            int32_t pix; // byte offset of the window's first tap (may lie before the image), kOob when beyond M
            int32_t yx;  // (top input row << 16) | (left input column & 0xffff) of the window
        };
        struct Cursor
        {
            int32_t r, s, c;  // tap and channel offset of the slice
            int32_t ry, sx;   // r * dh, s * dw
            int32_t tap_off;  // ((r * dh) * W + s * dw) * C + c
        };
        __device__ __forceinline__ void init_row(Row& rw, int64_t m, int64_t M) const
        {
            ConvX::Row r;
            cx.init_row(r, m, M);
            rw.yx = r.yx;
            rw.pix = r.base == kOob ? kOob : r.base + ((r.yx >> 16) * cx.W + static_cast<int16_t>(r.yx & 0xffff)) * cx.C;
        }
        __device__ __forceinline__ void set(Cursor& c) const
        {
            c.ry = c.r * cx.dh;
            c.sx = c.s * cx.dw;
            c.tap_off = (c.ry * cx.W + c.sx) * cx.C + c.c;
        }
        __device__ __forceinline__ void init_cursor(Cursor& c, int kbyte) const
        {
            const int tap = static_cast<int>(cx.by_c.div(static_cast<uint32_t>(kbyte)));
            c.c = kbyte - tap * cx.C;
            c.r = static_cast<int>(cx.by_s.div(static_cast<uint32_t>(tap)));
            c.s = tap - c.r * cx.S;
            set(c);
        }
        __device__ __forceinline__ void advance(Cursor& c, int bytes_) const
        {
            c.c += bytes_;
            if (c.c >= cx.C) // at most one tap further: bytes_ <= C
            {
                c.c -= cx.C;
                if (++c.s == cx.S)
                {
                    c.s = 0;
                    ++c.r;
                }
            }
            set(c);
        }
        __device__ __forceinline__ int32_t offset(const Row& rw, const Cursor& c, int lane_bytes) const
        {
            const int32_t y = (rw.yx >> 16) + c.ry;
            const int32_t xx = static_cast<int16_t>(rw.yx & 0xffff) + c.sx;
            const bool ok = (rw.pix != kOob) & (c.r < cx.R) & (static_cast<uint32_t>(y) < static_cast<uint32_t>(cx.H)) &
                            (static_cast<uint32_t>(xx) < static_cast<uint32_t>(cx.W));
            return ok ? rw.pix + c.tap_off + lane_bytes : kOob;
        }
        __device__ __forceinline__ int32_t direct(int64_t m, const int8_t* wrow, int32_t xzp, int32_t wzp, bool x_unsigned) const
        {
            return cx.direct(m, wrow, xzp, wzp, x_unsigned);
        }
    };

    // Convolution over at most four channels (a network's first layer), on a staged copy of the
    // data: [image][Hp][Wp][4] with the padding materialised (data zero point) so that every window
    // lies inside it.  A filter row is one 32-byte run of the copy -- 8 taps x 4 channels, the taps
    // and channels beyond the filter's meeting zero weights -- so the reduction is R runs of 32
    // bytes instead of R x S taps padded to 16 channels each (a 7 x 7 filter: 224 bytes, not 784).
    struct ConvR
    {
        const uint8_t* x;
        uint32_t bytes;
        int32_t R, S, C;                 // filter rows, taps per row (<= 8), channels (<= 4)
        int32_t row_pitch, img_pitch;    // Wp * 4, Hp * Wp * 4
        int32_t sh_pitch, sw4;           // stride_h * Wp * 4, stride_w * 4
        int32_t Q, PQ;
        FastDiv by_pq, by_q;
        static constexpr bool kUniform = true;
        static constexpr bool kFloatOut = false;
        static constexpr bool kDeep = false;
        static constexpr bool kPads = false;
        struct Row
        {
            int32_t off;
        };
        struct Cursor
        {
            int32_t kbyte;
        };
        __device__ __forceinline__ void init_row(Row& r, int64_t m, int64_t M) const
        {
            const bool valid = m < M;
            const uint32_t mm = valid ? static_cast<uint32_t>(m) : 0u;
            const int32_t n = static_cast<int32_t>(by_pq.div(mm));
            const int32_t rem = static_cast<int32_t>(mm) - n * PQ;
            const int32_t p = static_cast<int32_t>(by_q.div(static_cast<uint32_t>(rem)));
            const int32_t q = rem - p * Q;
            r.off = valid ? n * img_pitch + p * sh_pitch + q * sw4 : kOob;
        }
        __device__ __forceinline__ void init_cursor(Cursor& c, int kbyte) const { c.kbyte = kbyte; }
        __device__ __forceinline__ void advance(Cursor& c, int bytes_) const { c.kbyte += bytes_; }
        __device__ __forceinline__ int32_t offset(const Row& r, const Cursor& c, int lane_bytes) const
        {
            const int32_t q = (c.kbyte + lane_bytes) >> 4; // 16-byte piece of the packed reduction: filter row q / 2, half q % 2
            const int32_t fr = q >> 1;
            return (r.off != kOob && fr < R) ? r.off + fr * row_pitch + (q & 1) * 16 : kOob;
        }
        // exact accumulator over the filter's own taps and channels; wrow is the packed row [R][8][4]
        __device__ __forceinline__ int32_t direct(int64_t m, const int8_t* wrow, int32_t xzp, int32_t wzp, bool x_unsigned) const
        {
            Row rw;
            init_row(rw, m, m + 1);
            int32_t acc = 0;
            for (int32_t fr = 0; fr < R; ++fr)
                for (int32_t fs = 0; fs < S; ++fs)
                    for (int32_t c = 0; c < C; ++c)
                    {
                        const uint8_t b = x[rw.off + fr * row_pitch + fs * 4 + c];
                        const int32_t a = x_unsigned ? static_cast<int32_t>(b) : static_cast<int32_t>(static_cast<int8_t>(b));
                        acc += (a - xzp) * (static_cast<int32_t>(wrow[fr * 32 + fs * 4 + c]) - wzp);
                    }
            return acc;
        }
    };

    // Exact but slow tile for a non-zero weight zero point (w - wzp does not fit a signed byte).
    struct OutMap
    {
        int32_t ncx;  // 1: out is [image][n][pixel], 0: out is [m][n]
        int32_t N;
        int64_t PQ;   // pixels per image (ncx only)
        __device__ __forceinline__ int64_t index(int64_t m, int32_t n) const
        {
            if (!ncx)
                return m * N + n;
            int64_t img = m / PQ;
            return (img * N + n) * PQ + (m - img * PQ);
        }
    };

    // Inlined: as a call its by-value descriptors travelled on the stack, which gave every kernel 96
    // bytes of scratch a lane (set up at every launch although only this path touched it); inlined it
    // costs the MFMA path at most two registers, the branch being uniform and the loops scalar.
    template <class XL>
    __device__ __attribute__((always_inline)) void slow_tile(const XL xl,
                                           const int8_t* __restrict__ w,
                                           int64_t M,
                                           int32_t Kred,
                                           int32_t x_unsigned,
                                           int32_t xzp,
                                           int32_t wzp,
                                           const Epilogue epi,
                                           const OutMap om,
                                           void* __restrict__ out,
                                           int64_t m0,
                                           int32_t n0,
                                           int bm,
                                           int bn)
    {
        const EpiRegs er = epi_load(epi);
        for (int i = threadIdx.x; i < bm * bn; i += blockDim.x)
        {
            const int64_t m = m0 + i / bn;
            const int32_t n = n0 + i % bn;
            if (m < M && n < om.N)
            {
                int32_t a = xl.direct(m, w + static_cast<int64_t>(n) * Kred, xzp, wzp, x_unsigned != 0);
                const int64_t o = om.index(m, n);
                store_out(out, epi.out_t, o, epi_apply(epi, er, a, n, o));
            }
        }
    }

    // ---- lean, branch-free epilogues ------------------------------------------------------------
    // MODE: EPI_INTERP / EPI_FUSED.  KIND: what an output element is.
    enum
    {
        OUT_Q8 = 0, // u8 or i8, packed four to a dword by the caller
        OUT_I32 = 1,
        OUT_F32 = 2,
        OUT_GELU_Q8 = 3 // the float result through Gelu and Quantize: only the 8-bit tensor is written
    };

    struct EpiConst
    {
        float scale;      // interp scale, or the scalar fused scale
        float sum_scale;  // fused
        float lo, hi;     // fused saturation bounds
        float relu_floor; // fused: 0 with relu, -inf without
        int32_t ozp;      // interp
        bool slow_cvt;    // interp: |round| may reach 2^31, take the x86 out-of-range rule
    };

    __device__ __forceinline__ EpiConst epi_const(const Epilogue& e)
    {
        EpiConst c;
        const EpiRegs r = epi_load(e);
        c.scale = r.scale;
        c.sum_scale = r.sum_scale;
        c.ozp = r.ozp;
        c.lo = (e.out_t == HIPQ_U8) ? 0.0f : (e.out_t == HIPQ_I8 ? -128.0f : -2147483648.0f);
        c.hi = (e.out_t == HIPQ_U8) ? 255.0f : (e.out_t == HIPQ_I8 ? 127.0f : 2147483520.0f);
        c.relu_floor = e.relu ? 0.0f : -__builtin_huge_valf();
        // |acc| <= 2^31, so |acc * scale| < 2^31 whenever |scale| < 1 (false for NaN)
        c.slow_cvt = !(fabsf(r.scale) < 1.0f);
        return c;
    }

    // The scalars of a kernel's head -- both accumulation zero points and everything epi_const reads
    // -- fetched by loads that are all issued at once.  epi_const / load_zp branch on modes, types and
    // null pointers, and a load behind a branch waits for the loads in front of it: a chain of
    // memory latencies where one is enough.  Here a pointer the call does not use (or a null one) is
    // replaced by `safe` (any readable, 4-byte aligned address) and its value discarded; a byte is
    // read through the aligned word that holds it (the word lies in the byte's own page), so that
    // every load is a uniform word load: those go through the scalar cache and its own counter,
    // where they neither wait for nor hold up the vector loads around them.  8-bit data and filter
    // zero points only (what the MFMA kernels take).
    //   head_scalars_load    at the very top of a kernel (behind an asm statement the compiler can no
    //                        longer prove memory unchanged and falls back to vector loads)
    //   head_scalars_settle  where the kernel is ready to wait for them (behind its operand loads):
    //                        pins the first use of the raw words to this point
    //   head_scalars_finish  the arithmetic
    struct HeadWords
    {
        uint32_t x, w, o, sd, sf, so, s0, ss; // raw words: zero points (data, filter, output), scales
    };
    struct HeadScalars
    {
        int32_t xzp, wzp;
        EpiConst ec;
    };
    __device__ __forceinline__ HeadWords head_scalars_load(const ZeroPoints& zp, const Epilogue& e, const void* safe)
    {
        const bool interp = e.mode == EPI_INTERP;
        auto word_at = [&](const void* p, bool used) {
            const uint8_t* q = static_cast<const uint8_t*>((used && p != nullptr) ? p : safe);
            return *reinterpret_cast<const uint32_t*>(q - (reinterpret_cast<uintptr_t>(q) & 3)); // (pointer arithmetic, not an integer cast: the load stays a global one)
        };
        HeadWords h;
        h.x = word_at(zp.data_zp, true);
        h.w = word_at(zp.filter_zp, true);
        h.o = word_at(e.out_zp, interp);
        h.sd = word_at(e.s_data, interp);
        h.sf = word_at(e.s_filter, interp);
        h.so = word_at(e.s_out, interp);
        h.s0 = word_at(e.scale, !interp);
        h.ss = word_at(e.sum_scale, !interp && e.sum_in != nullptr);
        return h;
    }
    __device__ __forceinline__ void head_scalars_settle(HeadWords& h)
    {
        asm volatile("" : "+s"(h.x), "+s"(h.w), "+s"(h.o), "+s"(h.sd), "+s"(h.sf), "+s"(h.so), "+s"(h.s0), "+s"(h.ss));
    }
    __device__ __forceinline__ HeadScalars head_scalars_finish(const HeadWords& h, const ZeroPoints& zp, const Epilogue& e)
    {
        const bool interp = e.mode == EPI_INTERP;
        auto as_zp = [](uint32_t word, const void* p, int t) {
            const uint32_t b = (word >> (8 * static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p) & 3))) & 0xFFu;
            return t == HIPQ_U8 ? static_cast<int32_t>(b) : static_cast<int32_t>(static_cast<int8_t>(b));
        };
        HeadScalars r;
        r.xzp = zp.data_zp ? as_zp(h.x, zp.data_zp, zp.data_t) : 0;
        r.wzp = zp.filter_zp ? as_zp(h.w, zp.filter_zp, zp.filter_t) : 0;
        EpiConst& c = r.ec;
        // src/ngraph/runtime/reference/convolution.hpp:254 : two f32 roundings, this order
        c.scale = interp ? __fdiv_rn(__fmul_rn(__uint_as_float(h.sd), __uint_as_float(h.sf)), __uint_as_float(h.so)) : __uint_as_float(h.s0);
        c.sum_scale = (!interp && e.sum_in != nullptr) ? __uint_as_float(h.ss) : 0.0f;
        c.ozp = (interp && e.out_zp != nullptr) ? ((e.out_t == HIPQ_U8 || e.out_t == HIPQ_I8) ? as_zp(h.o, e.out_zp, e.out_t) : static_cast<int32_t>(h.o)) : 0;
        c.lo = (e.out_t == HIPQ_U8) ? 0.0f : (e.out_t == HIPQ_I8 ? -128.0f : -2147483648.0f);
        c.hi = (e.out_t == HIPQ_U8) ? 255.0f : (e.out_t == HIPQ_I8 ? 127.0f : 2147483520.0f);
        c.relu_floor = e.relu ? 0.0f : -__builtin_huge_valf();
        c.slow_cvt = !(fabsf(c.scale) < 1.0f);
        return r;
    }

    // INTERPRETER: (OUT) roundf(float(acc) * scale) + ozp; the caller keeps the low byte for 8-bit types
    template <int KIND>
    __device__ __forceinline__ int32_t epi_interp(const EpiConst& c, int32_t acc)
    {
        const float v = __fmul_rn(static_cast<float>(acc), c.scale);
        // half away from zero from round-half-even: the two differ only at exact .5 ties that
        // round-half-even took toward zero, i.e. where the residual d = v - r0 is +-0.5 with the
        // sign of v; there the correction 2*d is exactly +-1 (d is exact: r0 is within 0.5 of v)
        const float r0 = rintf(v);
        const float d = __fsub_rn(v, r0);
        const float r = (d == copysignf(0.5f, v)) ? __fadd_rn(r0, __fadd_rn(d, d)) : r0;
        int32_t t = static_cast<int32_t>(r);
        if (c.slow_cvt)
            t = (!(fabsf(r) < 2147483648.0f)) ? INT32_MIN : t;
        if (KIND == OUT_I32)
            return static_cast<int32_t>(static_cast<uint32_t>(t) + static_cast<uint32_t>(c.ozp));
        // narrowing first and adding the zero point afterwards is the same low byte
        return t + c.ozp;
    }

    // oneDNN: sat(rne(relu(scale * (float(acc) + bias) (+ sum_scale * sum))))
    template <int KIND>
    __device__ __forceinline__ int32_t epi_fused(const EpiConst& c, int32_t acc, float bias, float scale, bool has_sum, float sum_v, bool relu)
    {
        float v = __fmul_rn(__fadd_rn(static_cast<float>(acc), bias), scale);
        if (has_sum)
            v = fmaf(c.sum_scale, sum_v, v);
        if (KIND == OUT_F32)
        {
            if (relu)
                v = (v > 0.0f) ? v : __fmul_rn(v, -0.0f);
            return __float_as_int(v);
        }
        v = fmaxf(v, c.relu_floor);
        v = fminf(fmaxf(v, c.lo), c.hi);
        return static_cast<int32_t>(rintf(v));
    }

    __device__ __forceinline__ uint32_t pack4(const int32_t v[4])
    {
        return (v[0] & 0xFF) | ((v[1] & 0xFF) << 8) | ((v[2] & 0xFF) << 16) | (static_cast<uint32_t>(v[3]) << 24);
    }

    // sum input bytes of four consecutive elements -> floats
    __device__ __forceinline__ void sum4(const void* sum_in, int sum_t, int64_t idx, bool aligned, float out[4])
    {
        uint32_t w;
        if (aligned)
            w = *reinterpret_cast<const uint32_t*>(static_cast<const uint8_t*>(sum_in) + idx);
        else
        {
            const uint8_t* p = static_cast<const uint8_t*>(sum_in) + idx;
            w = p[0] | (p[1] << 8) | (p[2] << 16) | (static_cast<uint32_t>(p[3]) << 24);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e)
        {
            const uint32_t b = (w >> (8 * e)) & 0xFFu;
            out[e] = sum_t == HIPQ_I8 ? static_cast<float>(static_cast<int8_t>(b)) : static_cast<float>(b);
        }
    }

    // WM x WN MFMA tiles per wavefront, WAVES_M x WAVES_N wavefronts per workgroup (= 4).
    // X_ON_A: activations feed MFMA source A (NCHW output) instead of the weights.
    template <class XL, int WM, int WN, int WAVES_M, int WAVES_N, bool X_ON_A, int MODE, int KIND>
    __global__ __launch_bounds__(256, (WM * WN <= 4 ? 4 : 2)) void igemm_i8_kernel(XL xl,
                                                              const int8_t* __restrict__ w,
                                                              const int32_t* __restrict__ wsum,
                                                              int64_t M,
                                                              int32_t Kred,
                                                              int32_t x_unsigned,
                                                              int32_t m_tiles,
                                                              ZeroPoints zp,
                                                              Epilogue epi,
                                                              OutMap om,
                                                              void* __restrict__ out)
    {
        static_assert(WAVES_M * WAVES_N == 4, "four wavefronts per workgroup");
        constexpr int BM = WAVES_M * WM * 32;
        constexpr int BN = WAVES_N * WN * 32;
        constexpr int XLOADS = BM * 4 / 256; // 16-byte chunks per lane and slice
        constexpr int WLOADS = (BN * 4 + 255) / 256;
        constexpr int STAGE = (BM + BN) * BK;
        extern __shared__ __attribute__((aligned(16))) uint8_t lds[]; // [2][x tile | w tile]

        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int wn = wave % WAVES_N;
        const int wm = wave / WAVES_N;
        const int N = om.N;

        // XCD-aware tile order: ids i, i+8, i+16, ... land on one XCD; give it consecutive m tiles
        const int per_xcd = (m_tiles + 7) >> 3;
        const int mt = static_cast<int>(blockIdx.x & 7) * per_xcd + static_cast<int>(blockIdx.x >> 3);
        if (mt >= m_tiles)
            return;
        const int64_t m0 = static_cast<int64_t>(mt) * BM;
        const int32_t n0 = static_cast<int32_t>(blockIdx.y) * BN;

        const int32_t xzp = load_zp(zp.data_zp, zp.data_t);
        const int32_t wzp = load_zp(zp.filter_zp, zp.filter_t);
        if (wzp != 0) // uniform across the grid
        {
            slow_tile(xl, w, M, Kred, x_unsigned, xzp, wzp, epi, om, out, m0, n0, BM, BN);
            return;
        }

        // Accumulators start at the sign-bias correction (128 - zp) * sum(w[n]) of their channel.
        // MFMA result layout: lane holds column (source B index) lane % 32 and rows (source A
        // index) 8*(r/4) + 4*(lane/32) + r%4 for accumulator register r.
        const int32_t mult = (x_unsigned ? 128 : 0) - xzp;
        v16i acc[WM][WN];
#pragma unroll
        for (int ni = 0; ni < WN; ++ni)
        {
            v16i init;
            if (X_ON_A)
            {
                const int32_t n = n0 + (wn * WN + ni) * 32 + (lane & 31);
                const int32_t c = n < N ? mult * wsum[n] : 0;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    init[r] = c;
            }
            else
            {
#pragma unroll
                for (int r = 0; r < 16; ++r)
                {
                    const int32_t n = n0 + (wn * WN + ni) * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r & 3);
                    init[r] = n < N ? mult * wsum[n] : 0;
                }
            }
#pragma unroll
            for (int mi = 0; mi < WM; ++mi)
                acc[mi][ni] = init;
        }

        {
            const int lrow = tid >> 2;
            const int lchunk = tid & 3;
            const int xor_mask = x_unsigned ? static_cast<int>(0x80808080u) : 0;
            const int fill = (xzp & 0xFF) * 0x01010101;

            typename XL::Row xr[XLOADS];
            typename XL::Cursor cur;
#pragma unroll
            for (int i = 0; i < XLOADS; ++i)
                xl.init_row(xr[i], m0 + lrow + 64 * i, M);
            xl.init_cursor(cur, lchunk * 16);
            const __amdgpu_buffer_rsrc_t xrs = make_rsrc(xl.x, xl.bytes);
            const __amdgpu_buffer_rsrc_t wrs = make_rsrc(w, static_cast<uint32_t>(N) * static_cast<uint32_t>(Kred));
            int32_t woff[WLOADS]; // byte offset of this lane's weight row, kOob when beyond N
#pragma unroll
            for (int i = 0; i < WLOADS; ++i)
            {
                const int32_t r = lrow + 64 * i;
                const int32_t n = n0 + r;
                woff[i] = (n < N && r < BN) ? n * Kred : kOob;
            }
            int32_t kb = lchunk * 16;

            v4i xreg[XLOADS], wreg[WLOADS];
            uint32_t oob_mask = 0; // bit i: chunk i of the slice in flight was out of range
            // nothing between the loads and the MFMAs may touch the loaded registers: the fix-ups
            // (padding byte, sign bias) happen in lstore, one slice later
            auto gload = [&]() {
                oob_mask = 0;
#pragma unroll
                for (int i = 0; i < XLOADS; ++i)
                {
                    const int32_t off = xl.offset(xr[i], cur);
                    oob_mask |= (off == kOob ? 1u : 0u) << i;
                    xreg[i] = buffer_load16(xrs, off);
                }
#pragma unroll
                for (int i = 0; i < WLOADS; ++i)
                    wreg[i] = buffer_load16(wrs, (woff[i] != kOob && kb < Kred) ? woff[i] + kb : kOob);
            };
            auto lstore = [&](int buf) {
                uint8_t* xs = lds + buf * STAGE;
                uint8_t* ws = xs + BM * BK;
#pragma unroll
                for (int i = 0; i < XLOADS; ++i)
                {
                    v4i v = xreg[i];
                    if (fill != 0) // uniform: a non-zero data zero point pads with that byte
                    {
                        const bool oob = (oob_mask >> i) & 1u;
                        v = v4i{oob ? fill : v[0], oob ? fill : v[1], oob ? fill : v[2], oob ? fill : v[3]};
                    }
                    *reinterpret_cast<v4i*>(xs + lds_offset(lrow + 64 * i, lchunk)) =
                        v4i{v[0] ^ xor_mask, v[1] ^ xor_mask, v[2] ^ xor_mask, v[3] ^ xor_mask};
                }
#pragma unroll
                for (int i = 0; i < WLOADS; ++i)
                    if (lrow + 64 * i < BN)
                        *reinterpret_cast<v4i*>(ws + lds_offset(lrow + 64 * i, lchunk)) = wreg[i];
            };

            const int KT = (Kred + BK - 1) / BK;
            gload();
            lstore(0);
            __syncthreads();
            for (int kt = 0; kt < KT; ++kt)
            {
                const int buf = kt & 1;
                const bool more = kt + 1 < KT;
                if (more)
                {
                    xl.advance(cur, BK);
                    kb += BK;
                    gload();
                }
                const uint8_t* xs = lds + buf * STAGE;
                const uint8_t* ws = xs + BM * BK;
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
                {
                    v4i wf[WN], xf[WM];
                    const int chunk = ks * 2 + (lane >> 5);
#pragma unroll
                    for (int i = 0; i < WN; ++i)
                        wf[i] = *reinterpret_cast<const v4i*>(ws + lds_offset((wn * WN + i) * 32 + (lane & 31), chunk));
#pragma unroll
                    for (int i = 0; i < WM; ++i)
                        xf[i] = *reinterpret_cast<const v4i*>(xs + lds_offset((wm * WM + i) * 32 + (lane & 31), chunk));
#pragma unroll
                    for (int mi = 0; mi < WM; ++mi)
#pragma unroll
                        for (int ni = 0; ni < WN; ++ni)
                        {
                            if (X_ON_A)
                                acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[mi], wf[ni], acc[mi][ni], 0, 0, 0);
                            else
                                acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[ni], xf[mi], acc[mi][ni], 0, 0, 0);
                        }
                }
                if (more)
                    lstore(buf ^ 1);
                __syncthreads();
            }
        }

        // ---- epilogue on the accumulators in registers -----------------------------------------
        const EpiConst ec = epi_const(epi);
        const bool has_sum = MODE == EPI_FUSED && epi.sum_in != nullptr;
        const bool relu = epi.relu != 0;
        if (!X_ON_A)
        {
            // rows = output channels: 4 consecutive channels of one m -> out[m][n..n+3]
            const bool vec_ok = (N & 3) == 0;
            // 8-bit outputs whose rows are whole 16-byte pieces leave through LDS (the operand buffers
            // are free now): a lane's dword of four channels goes into a [BM][BN + 16] byte tile, and
            // the tile is written out 16 bytes a lane with neighbouring lanes on neighbouring pieces
            // of a row -- full lines instead of 64 scattered dwords per store instruction
            constexpr int SP = BN + 16; // staging pitch: 16-byte aligned rows, two-way bank conflicts at worst
            constexpr bool kCanStage = KIND == OUT_Q8 && BM * SP <= 2 * STAGE;
            const bool staged = kCanStage && (N & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
#pragma unroll
            for (int ni = 0; ni < WN; ++ni)
            {
#pragma unroll
                for (int g = 0; g < 4; ++g)
                {
                    const int32_t nb = n0 + (wn * WN + ni) * 32 + 8 * g + 4 * (lane >> 5);
                    if (nb >= N)
                        continue;
                    // per-channel parameters of the four channels this lane holds
                    float bias4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                    float scale4[4] = {ec.scale, ec.scale, ec.scale, ec.scale};
                    if (MODE == EPI_FUSED)
                    {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (nb + e < N)
                            {
                                if (epi.bias)
                                    bias4[e] = static_cast<float>(epi.bias[nb + e]);
                                if (epi.per_channel)
                                    scale4[e] = epi.scale[nb + e];
                            }
                    }
#pragma unroll
                    for (int mi = 0; mi < WM; ++mi)
                    {
                        const int64_t m = m0 + (wm * WM + mi) * 32 + (lane & 31);
                        if (m >= M)
                            continue;
                        const int64_t o = m * N + nb;
                        float s4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                        if (has_sum)
                        {
                            if (vec_ok)
                                sum4(epi.sum_in, epi.sum_t, o, true, s4);
                            else
                            {
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    if (nb + e < N)
                                        s4[e] = static_cast<float>(load_q(epi.sum_in, epi.sum_t, o + e));
                            }
                        }
                        int32_t v[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                        {
                            const int32_t a = acc[mi][ni][4 * g + e];
                            v[e] = MODE == EPI_INTERP ? epi_interp<KIND>(ec, a) : epi_fused<KIND>(ec, a, bias4[e], scale4[e], has_sum, s4[e], relu);
                        }
                        if (kCanStage && staged)
                            *reinterpret_cast<uint32_t*>(lds + ((wm * WM + mi) * 32 + (lane & 31)) * SP + (nb - n0)) = pack4(v);
                        else if (vec_ok) // nb is a multiple of 4, so nb + 3 < N and the store is aligned
                        {
                            if (KIND == OUT_Q8)
                                *reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(out) + o) = pack4(v);
                            else
                                *reinterpret_cast<v4i*>(static_cast<int32_t*>(out) + o) = v4i{v[0], v[1], v[2], v[3]};
                        }
                        else
                        {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if (nb + e < N)
                                    store_out(out, KIND == OUT_Q8 ? HIPQ_U8 : HIPQ_I32, o + e, v[e]);
                        }
                    }
                }
            }
            if (kCanStage && staged) // uniform
            {
                __syncthreads();
                constexpr int PIECES = BN / 16; // per row
                uint8_t* o8 = static_cast<uint8_t*>(out);
#pragma unroll
                for (int i = 0; i < BM * PIECES / 256; ++i)
                {
                    const int id = i * 256 + tid;
                    const int row = id / PIECES;
                    const int piece = id % PIECES;
                    const int64_t m = m0 + row;
                    const int32_t n = n0 + piece * 16;
                    if (m < M && n < N)
                        *reinterpret_cast<v4i*>(o8 + m * N + n) = *reinterpret_cast<const v4i*>(lds + row * SP + piece * 16);
                }
            }
        }
        else
        {
            // rows = m: 4 consecutive pixels of one channel -> out[image][n][pixel..pixel+3]
            const bool vec_ok = om.ncx && (om.PQ & 3) == 0;
#pragma unroll
            for (int ni = 0; ni < WN; ++ni)
            {
                const int32_t n = n0 + (wn * WN + ni) * 32 + (lane & 31);
                if (n >= N)
                    continue;
                float bias = 0.0f, scale = ec.scale;
                if (MODE == EPI_FUSED)
                {
                    if (epi.bias)
                        bias = static_cast<float>(epi.bias[n]);
                    if (epi.per_channel)
                        scale = epi.scale[n];
                }
#pragma unroll
                for (int mi = 0; mi < WM; ++mi)
                {
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                    {
                        const int64_t mb = m0 + (wm * WM + mi) * 32 + 8 * g + 4 * (lane >> 5);
                        if (mb >= M)
                            continue;
                        if (vec_ok) // mb % 4 == 0 and PQ % 4 == 0: same image, aligned, mb + 3 < M
                        {
                            const int64_t o = om.index(mb, n);
                            float s4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                            if (has_sum)
                                sum4(epi.sum_in, epi.sum_t, o, true, s4);
                            int32_t v[4];
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                            {
                                const int32_t a = acc[mi][ni][4 * g + e];
                                v[e] = MODE == EPI_INTERP ? epi_interp<KIND>(ec, a) : epi_fused<KIND>(ec, a, bias, scale, has_sum, s4[e], relu);
                            }
                            if (KIND == OUT_Q8)
                                *reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(out) + o) = pack4(v);
                            else
                                *reinterpret_cast<v4i*>(static_cast<int32_t*>(out) + o) = v4i{v[0], v[1], v[2], v[3]};
                        }
                        else
                        {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if (mb + e < M)
                                {
                                    const int64_t o = om.index(mb + e, n);
                                    const int32_t a = acc[mi][ni][4 * g + e];
                                    const float sv = has_sum ? static_cast<float>(load_q(epi.sum_in, epi.sum_t, o)) : 0.0f;
                                    const int32_t v = MODE == EPI_INTERP ? epi_interp<KIND>(ec, a) : epi_fused<KIND>(ec, a, bias, scale, has_sum, sv, relu);
                                    store_out(out, KIND == OUT_Q8 ? HIPQ_U8 : HIPQ_I32, o, v);
                                }
                        }
                    }
                }
            }
        }
    }



    // ---- persistent, software-pipelined variant ---------------------------------------------------
    // For 8-bit channels-last / row-major outputs whose rows are whole 16-byte pieces.  A workgroup
    // walks its tiles (tile = vb + j * grid) and treats all their 64-byte reduction slices as one
    // sequence: while slice s feeds the MFMAs out of LDS, slice s+1 waits in registers and the loads
    // of slice s+2 -- possibly the next tile's -- are in flight, so short reductions (1x1
    // convolutions over 64 channels are a single slice) overlap their loads with the neighbouring
    // tiles' arithmetic and epilogues, and long ones have two slices of latency cover.  Each
    // wavefront requantizes its own 64 x 64 sub-tile into a private swizzled LDS region and writes it
    // out 16 bytes a lane; per-channel constants of the current column tile sit in LDS.
    // (That is the register-staged variant; the one below prefetches one or two slices and is
    // written as a loop nest per tile.)
    //
    // DMA variant (loaders with a uniform cursor): the slices go from global memory straight into
    // LDS (buffer loads with the lds modifier, 16 bytes a lane, a wavefront's 64 lanes filling one
    // contiguous KiB, so the swizzle is applied to what a lane reads instead of where it writes),
    // three buffers deep (two where LDS is better spent on a third workgroup per compute unit: the
    // kernels with a residual input, the narrow tiles, the deep slices): no staging registers, no
    // LDS stores, and the sign flip of unsigned data moves to the MFMA fragments.  These loads are
    // written in assembly, so the waits for them are explicit: a wait for "at most n operations in
    // flight" only ever errs on the long side when the compiler's own loads and stores are in the
    // queue as well.
    // KIND OUT_F32 (fused policy without a residual, loaders with a uniform cursor): the scaled sums
    // leave as floats, 16 bytes a lane straight from the accumulators.
    // BKT = 128 (loads straight into LDS, no residual, reductions -- per tap -- in whole 128-byte pieces): slices twice
    // as deep, two operand buffers.  A row piece is then a whole 128-byte line, which the path from
    // L2 into LDS moves half again as fast as two 64-byte halves, and a slice has half the barriers.
    template <class XL, int WM, int WN, int WAVES_M, int WAVES_N, int MODE, bool HAS_SUM, bool DMA, int KIND = OUT_Q8, int BKT = BK>
    __global__ __launch_bounds__(256, (DMA && !HAS_SUM && XL::kFloatOut && BKT == BK) ? 3 : 2) void igemm_pipe_kernel(XL xl,
                                                                const int8_t* __restrict__ w,
                                                                const int32_t* __restrict__ wsum,
                                                                int64_t M,
                                                                int32_t Kred,
                                                                int32_t x_unsigned,
                                                                int32_t m_tiles,
                                                                int32_t n_tiles,
                                                                int32_t split_shift,
                                                                FastDiv by_m_tiles,
                                                                FastDiv by_group,
                                                                int32_t group_shift,
                                                                int32_t* __restrict__ partials,
                                                                uint32_t* __restrict__ counters,
                                                                ZeroPoints zp,
                                                                Epilogue epi,
                                                                OutMap om,
                                                                void* __restrict__ out)
    {
        static_assert(WAVES_M * WAVES_N == 4, "four wavefronts per workgroup");
        constexpr int BM = WAVES_M * WM * 32;
        constexpr int BN = WAVES_N * WN * 32;
        constexpr int TM = WM * 32, TN = WN * 32; // a wavefront's sub-tile
        static_assert(BKT == BK || (BKT == 2 * BK && DMA && !HAS_SUM), "deep slices: loads straight into LDS, no residual");
        constexpr int LPR = BKT / 16;  // lanes that load one row's piece of a slice
        constexpr int RPI = 256 / LPR; // rows one load instruction of the workgroup covers
        constexpr int XLOADS = BM / RPI;
        constexpr int WLOADS = (BN + RPI - 1) / RPI;
        constexpr int STAGE = (BM + BN) * BKT;
        constexpr int OUT_STAGE = TM * TN; // per wavefront
        static_assert(TN == 64, "the output staging swizzle is written for 64-byte rows");
        constexpr int NSTAGE = DMA && BKT == BK && !HAS_SUM && WAVES_N > 1 ? 3 : 2; // (with a residual the output regions need room of their own: two buffers, so that three workgroups fit a compute unit)
        extern __shared__ __attribute__((aligned(16))) uint8_t lds[]; // [NSTAGE][x | w] operands, 4 output regions, per-channel constants
        // Without a residual input the output regions need no room of their own: a tile's outputs are
        // staged in the operand buffer that its last slice has just been multiplied out of (one more
        // barrier per tile), which lets a third workgroup fit on a compute unit.
        constexpr bool ALIAS_OUT = DMA && !HAS_SUM;
        static_assert(!ALIAS_OUT || 4 * OUT_STAGE <= STAGE, "the output regions must fit an operand buffer");
        uint8_t* ostage = lds + NSTAGE * STAGE + (threadIdx.x >> 6) * OUT_STAGE;
        float* const params = reinterpret_cast<float*>(lds + NSTAGE * STAGE + (ALIAS_OUT ? 0 : 4 * OUT_STAGE)); // [3][BN]: correction (as int), bias, scale

        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int wn = wave % WAVES_N;
        const int wm = wave / WAVES_N;
        const int N = om.N;
        const int grid = static_cast<int>(gridDim.x);
        // With `splits` > 1 the reduction of every tile is cut into that many equal runs of slices,
        // each a work item of its own (neighbouring ids: they finish together); the items of a tile
        // leave their raw sums in `partials` and the last one to arrive adds them up and finishes.
        const int splits = 1 << split_shift;
        const int total_tiles = (m_tiles * n_tiles) << split_shift;
        const int vb = (grid & 7) == 0 ? (static_cast<int>(blockIdx.x) & 7) * (grid >> 3) + (static_cast<int>(blockIdx.x) >> 3) : static_cast<int>(blockIdx.x);
        if (vb >= total_tiles)
            return;
        const int my_tiles = (total_tiles - vb + grid - 1) / grid;
        // Tile order: column blocks go in groups of 2^group_shift; inside a group the tiles run
        // along the group's column blocks first, then down the rows.  The workgroups of one compute
        // die work on consecutive tiles (see `vb`), so with groups of eight they cover a square of
        // 8 x 8 tiles and fetch 16 operand tiles into their L2 where the plain order (group_shift
        // 0: down the rows of one column block) fetches 65.  The launcher only groups when the grid
        // is a multiple of the group, so a workgroup keeps its column block from tile to tile;
        // a last, narrower group runs in the plain order.
        auto tile_index = [&](int j, int& tile, int& split) {
            const int t = vb + j * grid;
            tile = t >> split_shift;
            split = t & (splits - 1);
        };
        auto tile_origin = [&](int j, int64_t& m0, int32_t& n0) {
            int t, ks;
            tile_index(j, t, ks);
            const int g = static_cast<int>(by_group.div(static_cast<uint32_t>(t)));
            const int r = t - g * (m_tiles << group_shift);
            int mt, nt;
            if (((g + 1) << group_shift) <= n_tiles) // uniform
            {
                mt = r >> group_shift;
                nt = (g << group_shift) + (r & ((1 << group_shift) - 1));
            }
            else
            {
                const int c = static_cast<int>(by_m_tiles.div(static_cast<uint32_t>(r)));
                mt = r - c * m_tiles;
                nt = (g << group_shift) + c;
            }
            m0 = static_cast<int64_t>(mt) * BM;
            n0 = nt * BN;
        };

        const int32_t xzp = load_zp(zp.data_zp, zp.data_t);
        const int32_t wzp = load_zp(zp.filter_zp, zp.filter_t);
        if (wzp != 0) // uniform across the grid
        {
            for (int j = 0; j < my_tiles; ++j)
            {
                int64_t m0;
                int32_t n0;
                tile_origin(j, m0, n0);
                int t, ks;
                tile_index(j, t, ks);
                if (ks == 0)
                    slow_tile(xl, w, M, Kred, x_unsigned, xzp, wzp, epi, om, out, m0, n0, BM, BN);
            }
            return;
        }
        const int32_t mult = (x_unsigned ? 128 : 0) - xzp;
        const EpiConst ec = epi_const(epi);
        constexpr bool has_sum = HAS_SUM; // residual input (fused policy only)
        static_assert(!HAS_SUM || MODE == EPI_FUSED, "only the fused policy adds a residual");
        static_assert(KIND == OUT_Q8 || ((KIND == OUT_F32 || KIND == OUT_GELU_Q8) && DMA && MODE == EPI_FUSED && !HAS_SUM),
                      "float outputs: fused policy, no residual, loads straight into LDS");

        // ---- loader --------------------------------------------------------------------------
        const int lrow = tid / LPR;
        // (DMA: the lane's LDS slot is fixed, chunk position tid % LPR of row lrow: it reads the chunk that belongs there)
        const int lchunk = !DMA ? (tid & 3) : BKT == BK ? ((tid & 3) ^ ((lrow >> 2) & 3)) : ((tid & 7) ^ ((lrow >> 1) & 7));
        const int xor_mask = x_unsigned ? static_cast<int>(0x80808080u) : 0;
        const int fill = (xzp & 0xFF) * 0x01010101;
        const __amdgpu_buffer_rsrc_t xrs = make_rsrc(xl.x, xl.bytes);
        const __amdgpu_buffer_rsrc_t wrs = make_rsrc(w, static_cast<uint32_t>(N) * static_cast<uint32_t>(Kred));
        const int KT = ((Kred + BKT - 1) / BKT) >> split_shift; // slices per work item (the launcher makes the split even)
        // Every slice issues the loads of the slice after next and stores the next one's into LDS,
        // without conditions (a condition the compiler cannot see through makes it wait for loads in
        // flight before their registers are loaded again): past the end the loader reads nothing
        // (every offset out of range), and an odd sequence gets one idle slice whose tile stores nothing.
        const int total = DMA ? my_tiles * KT : ((my_tiles * KT + 1) & ~1);
        typename XL::Row xr[XLOADS];
        typename XL::Cursor cur;
        int32_t woff[WLOADS];
        int32_t kb = 0;
        int lj = 0, lkt = 0;
        auto loader_tile = [&](int j) {
            int64_t m0;
            int32_t n0;
            tile_origin(j, m0, n0);
            int t, ks;
            tile_index(j, t, ks);
            const int kbyte0 = ks * KT * BKT + (DMA ? 0 : lchunk * 16);
#pragma unroll
            for (int i = 0; i < XLOADS; ++i)
                xl.init_row(xr[i], m0 + lrow + RPI * i, M);
            xl.init_cursor(cur, kbyte0);
#pragma unroll
            for (int i = 0; i < WLOADS; ++i)
            {
                const int32_t r = lrow + RPI * i;
                woff[i] = (n0 + r < N && r < BN) ? (n0 + r) * Kred : kOob;
            }
            kb = kbyte0;
        };
        struct Regs
        {
            v4i x[XLOADS];
            v4i w[WLOADS];
            uint32_t oob;
        };
        auto gload = [&](Regs& r) {
            r.oob = 0;
            if constexpr (!DMA)
            {
#pragma unroll
                for (int i = 0; i < XLOADS; ++i)
                {
                    const int32_t off = xl.offset(xr[i], cur);
                    r.oob |= (off == kOob ? 1u : 0u) << i;
                    r.x[i] = buffer_load16(xrs, off);
                }
#pragma unroll
                for (int i = 0; i < WLOADS; ++i)
                    r.w[i] = buffer_load16(wrs, (woff[i] != kOob && kb < Kred) ? woff[i] + kb : kOob);
            }
            if (++lkt == KT)
            {
                lkt = 0;
                if (++lj < my_tiles)
                    loader_tile(lj);
                else
                {
#pragma unroll
                    for (int i = 0; i < XLOADS; ++i)
                        xl.init_row(xr[i], M, M);
#pragma unroll
                    for (int i = 0; i < WLOADS; ++i)
                        woff[i] = kOob;
                }
            }
            else
            {
                xl.advance(cur, BK);
                kb += BK;
            }
        };
        auto lstore = [&](const Regs& r, int buf) {
            uint8_t* xs = lds + buf * STAGE;
            uint8_t* ws = xs + BM * BK;
#pragma unroll
            for (int i = 0; i < XLOADS; ++i)
            {
                v4i v = r.x[i];
                if (fill != 0) // uniform: a non-zero data zero point pads with that byte
                {
                    const bool oob = (r.oob >> i) & 1u;
                    v = v4i{oob ? fill : v[0], oob ? fill : v[1], oob ? fill : v[2], oob ? fill : v[3]};
                }
                *reinterpret_cast<v4i*>(xs + lds_offset(lrow + 64 * i, lchunk)) = v4i{v[0] ^ xor_mask, v[1] ^ xor_mask, v[2] ^ xor_mask, v[3] ^ xor_mask};
            }
#pragma unroll
            for (int i = 0; i < WLOADS; ++i)
                if (lrow + 64 * i < BN)
                    *reinterpret_cast<v4i*>(ws + lds_offset(lrow + 64 * i, lchunk)) = r.w[i];
        };

        // DMA: the next slice of the loader's sequence goes into operand buffer `buf`; returns which
        // of the lane's data chunks were out of range (they arrive as zeros)
        const v4i xrs_words = rsrc_words(xl.x, xl.bytes);
        const v4i wrs_words = rsrc_words(w, static_cast<uint32_t>(N) * static_cast<uint32_t>(Kred));
        const uint32_t lds_wave = lds_address(lds) + static_cast<uint32_t>(wave) * 1024u;
        auto dma_load = [&](int buf) -> uint32_t {
            uint32_t oob = 0;
            if constexpr (DMA)
            {
                const uint32_t base = __builtin_amdgcn_readfirstlane(lds_wave + static_cast<uint32_t>(buf) * STAGE);
#pragma unroll
                for (int i = 0; i < XLOADS; ++i)
                {
                    const int32_t off = xl.offset(xr[i], cur, lchunk * 16);
                    oob |= (off == kOob ? 1u : 0u) << i;
                    lds_dma16(xrs_words, off, base + i * 4096);
                }
#pragma unroll
                for (int i = 0; i < WLOADS; ++i)
                    lds_dma16(wrs_words, (woff[i] != kOob && kb + lchunk * 16 < Kred) ? woff[i] + kb + lchunk * 16 : kOob, base + BM * BKT + i * 4096);
                if (++lkt == KT)
                {
                    lkt = 0;
                    if (++lj < my_tiles)
                        loader_tile(lj);
                }
                else
                {
                    xl.advance(cur, BKT);
                    kb += BKT;
                }
            }
            return oob;
        };
        // byte offset of 16-byte chunk `chunk` of operand row `row` inside its LDS block
        auto frag_offset = [](int row, int chunk) { return BKT == BK ? lds_offset(row, chunk) : row * BKT + ((chunk ^ ((row >> 1) & 7)) << 4); };
        // DMA with a non-zero data zero point: chunks in the padding must hold that byte, not zero
        auto fill_fix = [&](int buf, uint32_t oob) {
            if constexpr (DMA && XL::kPads)
            {
                if (fill != 0 && oob != 0)
                {
#pragma unroll
                    for (int i = 0; i < XLOADS; ++i)
                        if ((oob >> i) & 1u)
                            *reinterpret_cast<v4i*>(lds + buf * STAGE + frag_offset(lrow + RPI * i, lchunk)) = v4i{fill, fill, fill, fill};
                }
            }
        };

        // ---- consumer ------------------------------------------------------------------------
        v16i acc[WM][WN];
        // The accumulators start from the zero-point correction of their channels (a register row of
        // an MFMA result is one output channel), so nothing is cleared and the epilogue adds nothing:
        // the first slice of a tile multiplies onto `corrv`, read from the per-channel constants.
        v16i corrv[WN];
        auto corr_load = [&](bool zero) {
#pragma unroll
            for (int ni = 0; ni < WN; ++ni)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                {
                    const v4i c4 = zero ? v4i{0, 0, 0, 0} : *reinterpret_cast<const v4i*>(reinterpret_cast<const int32_t*>(params) + wn * TN + ni * 32 + 8 * g + 4 * (lane >> 5));
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        corrv[ni][4 * g + e] = c4[e];
                }
        };
        auto compute = [&](int buf, auto first) {
            const uint8_t* xs = lds + buf * STAGE;
            const uint8_t* ws = xs + BM * BKT;
#pragma unroll
            for (int ks = 0; ks < BKT / 32; ++ks)
            {
                v4i wf[WN], xf[WM];
                const int chunk = ks * 2 + (lane >> 5);
#pragma unroll
                for (int i = 0; i < WN; ++i)
                    wf[i] = *reinterpret_cast<const v4i*>(ws + frag_offset((wn * WN + i) * 32 + (lane & 31), chunk));
#pragma unroll
                for (int i = 0; i < WM; ++i)
                {
                    xf[i] = *reinterpret_cast<const v4i*>(xs + frag_offset((wm * WM + i) * 32 + (lane & 31), chunk));
                    if constexpr (DMA) // the data sits in LDS as it came: unsigned bytes become signed here
                        xf[i] = v4i{xf[i][0] ^ xor_mask, xf[i][1] ^ xor_mask, xf[i][2] ^ xor_mask, xf[i][3] ^ xor_mask};
                }
#pragma unroll
                for (int mi = 0; mi < WM; ++mi)
#pragma unroll
                    for (int ni = 0; ni < WN; ++ni)
                        acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[ni], xf[mi], (decltype(first)::value && ks == 0) ? corrv[ni] : acc[mi][ni], 0, 0, 0);
            }
        };
        int cj = 0, ckt = 0;
        int64_t cm0;
        int32_t cn0, params_n0 = -1;
        tile_origin(0, cm0, cn0);
        // per-channel constants of column block n0 -> LDS; callers put a barrier behind it
        // With a short reduction (|accumulator| <= 2^24) and biases of that size, float(acc) +
        // float(bias) is float(acc + bias): no rounding happens before the sum's own.  The bias of such
        // a column block joins the correction in the accumulators' start value and the epilogue
        // skips its add (decided per column block; every lane of the workgroup calls this).
        // (only in the kernels that load straight into LDS: they take the short reductions, and the
        // register-staged ones have no registers to spare for a second epilogue)
        constexpr bool kFold = DMA && MODE == EPI_FUSED;
        const bool fold_possible = kFold && static_cast<int64_t>(Kred) * (255 * 128) <= (1 << 24);
        bool bias_folded = false;
        auto load_params = [&](int32_t n0) {
            int32_t corr = 0, b = 0;
            float sc = ec.scale;
            if (tid < BN)
            {
                const int32_t n = n0 + tid;
                const bool ok = n < N;
                corr = ok ? mult * wsum[n] : 0;
                b = (MODE == EPI_FUSED && epi.bias && ok) ? epi.bias[n] : 0;
                sc = (MODE == EPI_FUSED && epi.per_channel && ok) ? epi.scale[n] : ec.scale;
            }
            bool fold = false;
            if (fold_possible) // uniform
                fold = __syncthreads_and(b >= -(1 << 24) && b <= (1 << 24)) != 0;
            if (tid < BN)
            {
                reinterpret_cast<int32_t*>(params)[tid] = fold ? corr + b : corr;
                params[BN + tid] = fold ? 0.0f : static_cast<float>(b);
                params[2 * BN + tid] = sc;
            }
            bias_folded = fold;
            params_n0 = n0;
        };
        // requantizes the wavefront's sub-tile into its staging region and writes it out
        const float clamp_lo = fmaxf(ec.lo, ec.relu_floor);
        const float magic = 12582912.0f; // 1.5 * 2^23: adding it rounds half to even into the low mantissa bits
        const float s256 = __fmul_rn(ec.scale, 256.0f);
        const int32_t c256 = 128 + 256 * ec.ozp;
        // (Gelu + Quantize of a float result: the Quantize's scale and zero point)
        const float post_scale = KIND == OUT_GELU_Q8 ? *epi.post_scale : 1.0f;
        const int32_t post_zp_i = KIND == OUT_GELU_Q8 ? load_zp(epi.post_zp, epi.post_t) : 0;
        const float post_zp = static_cast<float>(post_zp_i);
        // the fixed-point form needs |acc * scale| * 256 < 2^31 with room to spare
        const bool fast_interp = fabsf(ec.scale) * (static_cast<float>(Kred) * (255.0f * 128.0f)) < 4194304.0f;
        constexpr int SUM_LOADS = TM * TN / 16 / 64;
        v4i sum_regs[SUM_LOADS];
        const __amdgpu_buffer_rsrc_t srs = make_rsrc(epi.sum_in, has_sum ? static_cast<uint32_t>(M * N) : 0u);
        const v4i srs_words = rsrc_words(epi.sum_in, has_sum ? static_cast<uint32_t>(M * N) : 0u);
        const uint32_t ostage_lds = lds_address(lds) + NSTAGE * STAGE + static_cast<uint32_t>(wave) * OUT_STAGE;
        bool loads_behind_sum = false; // DMA: operand loads were issued after the residual's
        auto sum_fetch = [&]() {
            if constexpr (DMA)
            {
                // straight into the wavefront's staging region, in the layout the epilogue reads: the
                // lane's slot is piece id % 4 of row id / 4, so it fetches the piece that belongs there
                const uint32_t base = __builtin_amdgcn_readfirstlane(ostage_lds);
#pragma unroll
                for (int i = 0; i < SUM_LOADS; ++i)
                {
                    const int id = i * 64 + lane;
                    const int row = id >> 2;
                    const int piece = (id & 3) ^ ((row >> 2) & 3);
                    const int64_t m = cm0 + wm * TM + row;
                    const int32_t n = cn0 + wn * TN + piece * 16;
                    lds_dma16(srs_words, (m < M && n < N) ? static_cast<int32_t>(m * N + n) : kOob, base + i * 1024);
                }
            }
            else
            {
#pragma unroll
                for (int i = 0; i < SUM_LOADS; ++i)
                {
                    const int id = i * 64 + lane;
                    const int row = id >> 2;
                    const int piece = id & 3;
                    const int64_t m = cm0 + wm * TM + row;
                    const int32_t n = cn0 + wn * TN + piece * 16;
                    sum_regs[i] = buffer_load16(srs, (m < M && n < N) ? static_cast<int32_t>(m * N + n) : kOob);
                }
            }
        };
        auto epilogue = [&](auto folded, auto to_u8) {
            constexpr bool FOLD = decltype(folded)::value; // the bias is already in the accumulators
            constexpr bool PK_U8 = decltype(to_u8)::value; // fused policy, u8 output: one instruction saturates, rounds and packs
            if constexpr (KIND == OUT_F32)
            {
                float* const of = static_cast<float*>(out);
                const bool relu = epi.relu != 0;
#pragma unroll
                for (int ni = 0; ni < WN; ++ni)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                    {
                        const int nt = wn * TN + ni * 32 + 8 * g + 4 * (lane >> 5); // within the column block
                        v4f bias4 = v4f{0.0f, 0.0f, 0.0f, 0.0f};
                        if (!FOLD)
                            bias4 = *reinterpret_cast<const v4f*>(params + BN + nt);
                        const v4f scale4 = *reinterpret_cast<const v4f*>(params + 2 * BN + nt);
                        const int32_t n = cn0 + nt;
#pragma unroll
                        for (int mi = 0; mi < WM; ++mi)
                        {
                            const int64_t m = cm0 + wm * TM + mi * 32 + (lane & 31);
                            v4f v;
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                            {
                                const float a = static_cast<float>(acc[mi][ni][4 * g + e]);
                                const float x = __fmul_rn(FOLD ? a : __fadd_rn(a, bias4[e]), scale4[e]);
                                v[e] = relu ? ((x > 0.0f) ? x : __fmul_rn(x, -0.0f)) : x;
                            }
                            if (m < M && n < N)
                                *reinterpret_cast<v4f*>(of + m * N + n) = v;
                        }
                    }
                return;
            }
            uint8_t* o8 = static_cast<uint8_t*>(out);
            if (has_sum)
            {
                // the residual input of the sub-tile comes in the way the output leaves: 16 bytes a
                // lane along the rows, fetched before the tile's last slice was multiplied -- into
                // registers and from there into the staging region, or (DMA) straight into it; each
                // lane then picks up the dword that its own output dword will replace
                if constexpr (DMA)
                {
                    if (loads_behind_sum) // uniform
                        wait_vmcnt<XLOADS + WLOADS>();
                    else
                        wait_vmcnt<0>();
                }
                else
                {
#pragma unroll
                    for (int i = 0; i < SUM_LOADS; ++i)
                    {
                        const int id = i * 64 + lane;
                        const int row = id >> 2;
                        const int piece = id & 3;
                        *reinterpret_cast<v4i*>(ostage + row * TN + ((piece ^ ((row >> 2) & 3)) << 4)) = sum_regs[i];
                    }
                }
            }
#pragma unroll
            for (int ni = 0; ni < WN; ++ni)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                {
                    const int nl = ni * 32 + 8 * g + 4 * (lane >> 5); // channel within the wavefront's 64
                    const int nt = wn * TN + nl;                     // within the column block
                    v4f bias4 = v4f{0.0f, 0.0f, 0.0f, 0.0f};
                    if (!FOLD)
                        bias4 = *reinterpret_cast<const v4f*>(params + BN + nt);
                    const v4f scale4 = *reinterpret_cast<const v4f*>(params + 2 * BN + nt);
#pragma unroll
                    for (int mi = 0; mi < WM; ++mi)
                    {
                        const int row = mi * 32 + (lane & 31);
                        uint32_t* const cell = reinterpret_cast<uint32_t*>(ostage + row * TN + ((((nl >> 4) ^ ((row >> 2) & 3))) << 4) + (nl & 15));
                        float s4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                        if (has_sum)
                        {
                            const uint32_t sw = *cell;
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                            {
                                const uint32_t b = (sw >> (8 * e)) & 0xFFu;
                                s4[e] = epi.sum_t == HIPQ_I8 ? static_cast<float>(static_cast<int8_t>(b)) : static_cast<float>(b);
                            }
                        }
                        // the output byte ends up in byte BYTE of x[e]: fused policy -- clamp (the ReLU is
                        // the clamp's lower bound), then 1.5 * 2^23 + v rounds half to even into the low
                        // mantissa bits; INTERPRETER policy in fixed point -- t = trunc(256 v), and
                        // round-half-away(v) = (t + 128 - (t < 0)) >> 8 exactly
                        int32_t x[4];
                        uint32_t packed = 0;
                        if constexpr (KIND == OUT_GELU_Q8)
                        {
                            // the float result exactly as the float kernel computes it, then Gelu and
                            // Quantize with the arithmetic of their own kernels (gelu1, quantize4 /
                            // quantize_one): the bytes equal the three launches'
                            v4f r4;
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                            {
                                const float a = static_cast<float>(acc[mi][ni][4 * g + e]);
                                const float y = __fmul_rn(FOLD ? a : __fadd_rn(a, bias4[e]), scale4[e]);
                                r4[e] = gelu1(epi.relu ? ((y > 0.0f) ? y : __fmul_rn(y, -0.0f)) : y);
                            }
                            if (epi.post_mode == HIPQ_ROUND_NEAREST_TOWARD_EVEN) // uniform
                                packed = epi.post_t == HIPQ_U8 ? quantize4<uint8_t, true>(r4, post_scale, post_zp, epi.post_mode) : quantize4<int8_t, true>(r4, post_scale, post_zp, epi.post_mode);
                            else
                            {
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    packed |= (epi.post_t == HIPQ_U8 ? static_cast<uint32_t>(quantize_one<float, uint8_t>(r4[e], post_scale, static_cast<uint8_t>(post_zp_i), epi.post_mode))
                                                                     : static_cast<uint32_t>(static_cast<uint8_t>(quantize_one<float, int8_t>(r4[e], post_scale, static_cast<int8_t>(post_zp_i), epi.post_mode))))
                                              << (8 * e);
                            }
                            *cell = packed;
                            continue;
                        }
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                        {
                            const int32_t a = acc[mi][ni][4 * g + e];
                            if (MODE == EPI_FUSED)
                            {
                                float v = __fmul_rn(FOLD ? static_cast<float>(a) : __fadd_rn(static_cast<float>(a), bias4[e]), scale4[e]);
                                if (has_sum)
                                    v = fmaf(ec.sum_scale, s4[e], v);
                                if constexpr (PK_U8)
                                {
                                    // float -> u8 with saturation to [0, 255] (the ReLU included) and
                                    // round half to even, written into byte e of the word; a NaN gives 0
                                    packed = __builtin_amdgcn_cvt_pk_u8_f32(v, e, packed);
                                    continue;
                                }
                                v = __builtin_amdgcn_fmed3f(v, clamp_lo, ec.hi);
                                // the rounding add drops its low byte straight into byte e of the word
                                if (e == 0)
                                    packed = __float_as_uint(__fadd_rn(v, magic)); // the bytes above are replaced below
                                else if (e == 1)
                                    asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(packed) : "v"(v), "v"(magic));
                                else if (e == 2)
                                    asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(packed) : "v"(v), "v"(magic));
                                else
                                    asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(packed) : "v"(v), "v"(magic));
                            }
                            else if (fast_interp)
                            {
                                const int32_t t = static_cast<int32_t>(__fmul_rn(static_cast<float>(a), s256));
                                x[e] = t + (t >> 31) + c256;
                            }
                            else
                                x[e] = epi_interp<OUT_Q8>(ec, a) << 8;
                        }
                        if (MODE == EPI_FUSED)
                            *cell = packed;
                        else
                            *cell = (__builtin_amdgcn_perm(x[3], x[2], 0x0c0c0501u) << 16) | __builtin_amdgcn_perm(x[1], x[0], 0x0c0c0501u);
                    }
                }
#pragma unroll
            for (int i = 0; i < TM * TN / 16 / 64; ++i)
            {
                const int id = i * 64 + lane;
                const int row = id >> 2;
                const int piece = id & 3;
                const int64_t m = cm0 + wm * TM + row;
                const int32_t n = cn0 + wn * TN + piece * 16;
                if (m < M && n < N)
                    *reinterpret_cast<v4i*>(o8 + m * N + n) = *reinterpret_cast<const v4i*>(ostage + row * TN + ((piece ^ ((row >> 2) & 3)) << 4));
            }
        };
        // (the variants exist in the kernels that load straight into LDS; see kFold)
        constexpr bool kPackU8 = DMA && MODE == EPI_FUSED && KIND == OUT_Q8;
        const bool pack_u8 = kPackU8 && epi.out_t == HIPQ_U8;
        auto run_epilogue = [&]() {
            if (kFold && bias_folded) // uniform
            {
                if (kPackU8 && pack_u8) // uniform
                    epilogue(std::true_type{}, std::true_type{});
                else
                    epilogue(std::true_type{}, std::false_type{});
            }
            else
            {
                if (kPackU8 && pack_u8) // uniform
                    epilogue(std::false_type{}, std::true_type{});
                else
                    epilogue(std::false_type{}, std::false_type{});
            }
        };
        // split reductions: leaves this item's raw sums in `partials`; the last item of the tile to
        // arrive (counted in `counters`, which it resets) adds all of them into its accumulators and
        // returns true: it runs the epilogue.  Every wavefront of the workgroup takes the same path.
        // The sums travel between compute dies, each with an L2 of its own: they are stored and
        // loaded at device scope (sc1: written through to, and fetched from, the memory side), so no
        // whole-cache write-back or invalidate is needed.  A workgroup barrier does not wait for
        // stores in flight, so every wavefront drains its own (vmcnt 0: acknowledged by the memory
        // side) before the barrier in front of the counter update.
        uint32_t* const arrival = reinterpret_cast<uint32_t*>(params + 3 * BN);
        constexpr int kDeviceScope = 16; // the sc1 bit of a buffer instruction
        auto gather_splits = [&]() {
            int tile, ks;
            tile_index(cj, tile, ks);
            const __amdgpu_buffer_rsrc_t prs = make_rsrc(partials + static_cast<size_t>(tile) * splits * (BM * BN), static_cast<uint32_t>(splits) * BM * BN * 4u);
            // register order: a wavefront's store covers 1 KiB in one piece
            const int32_t lane_off = (wave * (WM * WN * 4) * 64 + lane) * 16;
#pragma unroll
            for (int mi = 0; mi < WM; ++mi)
#pragma unroll
                for (int ni = 0; ni < WN; ++ni)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        __builtin_amdgcn_raw_buffer_store_b128(v4i{acc[mi][ni][4 * g], acc[mi][ni][4 * g + 1], acc[mi][ni][4 * g + 2], acc[mi][ni][4 * g + 3]},
                                                               prs,
                                                               ks * (BM * BN * 4) + lane_off + ((mi * WN + ni) * 4 + g) * 1024,
                                                               0,
                                                               kDeviceScope);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // this wavefront's partial sums have reached memory
            __syncthreads();                                 // ... and so have the other wavefronts'
            if (tid == 0)
            {
                const uint32_t seen = atomicAdd(counters + tile, 1u);
                if (seen == static_cast<uint32_t>(splits - 1))
                    atomicExch(counters + tile, 0u);
                *arrival = seen;
            }
            __syncthreads();
            const bool last = *arrival == static_cast<uint32_t>(splits - 1);
            __syncthreads(); // `arrival` may be rewritten by the next tile
            if (!last)
                return false;
            // the other items' sums, a batch of loads at a time (all issued before the first is added;
            // the register-staged kernels can spare registers for two)
            constexpr int GB = DMA ? 4 : 2;
            for (int k = 0; k < splits; ++k)
            {
                if (k == ks)
                    continue;
#pragma unroll
                for (int mi = 0; mi < WM; ++mi)
#pragma unroll
                    for (int ni = 0; ni < WN; ++ni)
#pragma unroll
                        for (int g0 = 0; g0 < 4; g0 += GB)
                        {
                            v4i p4[GB];
#pragma unroll
                            for (int g = 0; g < GB; ++g)
                                p4[g] = __builtin_amdgcn_raw_buffer_load_b128(prs, k * (BM * BN * 4) + lane_off + ((mi * WN + ni) * 4 + g0 + g) * 1024, 0, kDeviceScope);
#pragma unroll
                            for (int g = 0; g < GB; ++g)
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    acc[mi][ni][4 * (g0 + g) + e] += p4[g][e];
                        }
            }
            return true;
        };
        // one slice: LDS buffer `buf` feeds the MFMAs, `next` (slice s+1) moves into the other
        // buffer, `free_regs` takes the loads of slice s+2
        auto multiply = [&](int buf) {
            if (ckt == 0) // uniform
            {
                int t, ks = 0;
                if (splits > 1)
                    tile_index(cj, t, ks);
                corr_load(ks != 0); // the correction enters a split reduction once
                compute(buf, std::true_type{});
            }
            else
                compute(buf, std::false_type{});
        };
        auto step = [&](int s, int buf, const Regs& next, Regs& free_regs) {
            const bool tile_done = ckt + 1 == KT;
            if (tile_done) // uniform; the residual is fetched and used inside one branch
            {
                if (has_sum)
                    sum_fetch();
                gload(free_regs);
                multiply(buf);
                if (splits == 1 || (cm0 < M && gather_splits())) // uniform
                {
                    run_epilogue();
                }
                ckt = 0;
                if (++cj < my_tiles)
                    tile_origin(cj, cm0, cn0);
                else
                    cm0 = M; // the idle slice's tile: nothing fetched, nothing stored
            }
            else
            {
                gload(free_regs);
                multiply(buf);
                ++ckt;
            }
            lstore(next, buf ^ 1);
            __syncthreads();
            if (tile_done && cj < my_tiles && cn0 != params_n0) // uniform
            {
                load_params(cn0);
                __syncthreads();
            }
        };

        if constexpr (DMA)
        {
            constexpr int L = XLOADS + WLOADS; // operand loads of one slice per lane
            constexpr int PF = NSTAGE - 1;     // slices in flight ahead of the one being multiplied
            loader_tile(0);
            uint32_t oob_next = dma_load(0);
            uint32_t oob_new = (PF > 1 && total > 1) ? dma_load(1) : 0u;
            load_params(cn0);
            if (PF > 1 && total > 1)
                wait_vmcnt<L>();
            else
                wait_vmcnt<0>();
            fill_fix(0, oob_next);
            oob_next = oob_new;
            __syncthreads();
            int cb = 0, lb = PF; // buffer of the slice being multiplied, buffer the loads go to
            int s = 0;          // position in the workgroup's sequence of slices
            // One loop nest per tile, the tile's middle slices in a loop of their own that holds
            // nothing but loads, waits and MFMAs: the accumulators then have one definition per
            // tile (the first slice's product onto the correction) and the compiler neither copies
            // them around a merged loop nor puts waits of its own into the steady state.
            auto issue = [&]() {
                loads_behind_sum = s + PF < total;
                if (s + PF < total) // uniform
                    oob_new = dma_load(lb);
            };
            // the slice after this one has landed once at most the loads of the one after it are in flight
            auto slice_end = [&]() {
                cb = cb == NSTAGE - 1 ? 0 : cb + 1;
                lb = lb == NSTAGE - 1 ? 0 : lb + 1;
                if (PF > 1 && s + 2 < total)
                    wait_vmcnt<L>();
                else
                    wait_vmcnt<0>();
                fill_fix(cb, PF > 1 ? oob_next : oob_new); // the flags of the slice that has just landed
                oob_next = oob_new;
                ++s;
                __syncthreads();
            };
            for (cj = 0; cj < my_tiles; ++cj)
            {
                int t, ks = 0;
                if (splits > 1)
                    tile_index(cj, t, ks);
                if (has_sum && KT == 1) // ahead of the operand loads, so that waiting for it leaves them in flight
                    sum_fetch();
                issue();
                corr_load(ks != 0); // the correction enters a split reduction once
                compute(cb, std::true_type{});
                if (KT > 1) // uniform
                {
                    slice_end();
                    for (int kt = 1; kt + 1 < KT; ++kt)
                    {
                        issue();
                        compute(cb, std::false_type{});
                        slice_end();
                    }
                    if (has_sum)
                        sum_fetch();
                    issue();
                    compute(cb, std::false_type{});
                }
                if constexpr (ALIAS_OUT)
                {
                    __syncthreads(); // every wavefront has read its last fragments
                    ostage = lds + cb * STAGE + wave * OUT_STAGE;
                }
                if (splits == 1 || gather_splits()) // uniform
                {
                    run_epilogue();
                }
                if (cj + 1 < my_tiles)
                    tile_origin(cj + 1, cm0, cn0);
                slice_end();
                if (cj + 1 < my_tiles && cn0 != params_n0) // uniform
                {
                    load_params(cn0);
                    __syncthreads();
                }
            }
        }
        else
        {
            Regs r0, r1;
            loader_tile(0);
            gload(r0);
            gload(r1);
            load_params(cn0);
            lstore(r0, 0);
            __syncthreads();
            for (int s = 0; s < total; s += 2)
            {
                step(s, 0, r1, r0);
                step(s + 1, 1, r0, r1);
            }
        }
    }

    static inline bool fits_i32(int64_t v) { return v >= 0 && v < (1ll << 31); }

    // one instantiation = one tile shape; sets the dynamic LDS limit on first use
    template <class XL, int WM, int WN, int WAVES_M, int WAVES_N, bool X_ON_A, int MODE, int KIND>
    static int launch_tile(const XL& xl,
                           const int8_t* w,
                           const int32_t* wsum,
                           int64_t M,
                           int32_t N,
                           int32_t Kred,
                           int x_unsigned,
                           const ZeroPoints& zp,
                           const Epilogue& epi,
                           const OutMap& om,
                           void* out,
                           hipStream_t s,
                           const char* name)
    {
        constexpr int BM = WAVES_M * WM * 32;
        constexpr int BN = WAVES_N * WN * 32;
        constexpr size_t lds_bytes = 2 * static_cast<size_t>(BM + BN) * BK;
        auto kernel = igemm_i8_kernel<XL, WM, WN, WAVES_M, WAVES_N, X_ON_A, MODE, KIND>;
        static bool configured[16] = {};
        int dev = 0;
        HIPQ_HIP(hipGetDevice(&dev));
        if (dev >= 0 && dev < 16 && !configured[dev])
        {
            HIPQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
            configured[dev] = true;
        }
        const int64_t m_tiles = (M + BM - 1) / BM;
        HIPQ_REQUIRE(fits_i32(m_tiles * 8), "too many row tiles");
        dim3 grid(static_cast<unsigned>(((m_tiles + 7) / 8) * 8), static_cast<unsigned>((N + BN - 1) / BN));
        kernel<<<grid, 256, lds_bytes, s>>>(xl, w, wsum, M, Kred, x_unsigned, static_cast<int32_t>(m_tiles), zp, epi, om, out);
        return check_launch(name);
    }

    template <class XL, int WAVES_M, int WAVES_N, int MODE, bool HAS_SUM, int KIND = OUT_Q8, int BKT = BK, int WM = 2>
    static int launch_pipe(const XL& xl,
                           const int8_t* w,
                           const int32_t* wsum,
                           int64_t M,
                           int32_t N,
                           int32_t Kred,
                           int x_unsigned,
                           const ZeroPoints& zp,
                           const Epilogue& epi,
                           const OutMap& om,
                           void* out,
                           hipStream_t s,
                           const char* name)
    {
        constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * 64;
        constexpr bool DMA = XL::kUniform;
        // (the kernels that load into LDS and take no residual stage their outputs in an operand buffer)
        constexpr size_t lds_bytes = (DMA && BKT == BK && !HAS_SUM && WAVES_N > 1 ? 3 : 2) * static_cast<size_t>(BM + BN) * BKT + (DMA && !HAS_SUM ? 0 : 4 * WM * 32 * 64) + 3 * BN * sizeof(float) + 16;
        auto kernel = igemm_pipe_kernel<XL, WM, 2, WAVES_M, WAVES_N, MODE, HAS_SUM, DMA, KIND, BKT>;
        static bool configured[16] = {};
        static int cus[16] = {};
        static int per_cu[16] = {}; // workgroups of this kernel that fit a compute unit (LDS and registers)
        int dev = 0;
        HIPQ_HIP(hipGetDevice(&dev));
        if (dev >= 0 && dev < 16 && !configured[dev])
        {
            HIPQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
            hipDeviceProp_t prop;
            HIPQ_HIP(hipGetDeviceProperties(&prop, dev));
            cus[dev] = prop.multiProcessorCount;
            int fit = 0;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&fit, reinterpret_cast<const void*>(kernel), 256, lds_bytes) != hipSuccess)
            {
                (void)hipGetLastError(); // no answer: size the grid by LDS alone
                fit = 0;
            }
            const int by_lds = static_cast<int>(160 * 1024 / lds_bytes);
            per_cu[dev] = fit >= 1 && fit < by_lds ? fit : by_lds;
            configured[dev] = true;
        }
        const int64_t m_tiles = (M + BM - 1) / BM;
        const int64_t n_tiles = (N + BN - 1) / BN;
        HIPQ_REQUIRE(fits_i32(m_tiles * n_tiles), "too many tiles");
        const int64_t resident = static_cast<int64_t>(dev >= 0 && dev < 16 && cus[dev] > 0 ? cus[dev] : 256) * (dev >= 0 && dev < 16 && per_cu[dev] > 0 ? per_cu[dev] : static_cast<int>(160 * 1024 / lds_bytes));
        const int64_t tiles = m_tiles * n_tiles;
        // Few tiles with long reductions leave most of the chip idle: cut every reduction into
        // `splits` runs of whole slices.
        int splits = 1;
        const int64_t slices = (Kred + BKT - 1) / BKT;
        constexpr int64_t kDeep = BKT / BK; // the thresholds below are in 64-byte slices
        const char* const split_env = getenv("HIPQ_SPLIT_K");
        if (split_env)
        {
            const int want = atoi(split_env);
            splits = want > 0 && (want & (want - 1)) == 0 && slices % want == 0 ? want : 1;
        }
        else
        {
            // doubled while the items leave a quarter of the compute units free and keep eight
            // slices, or find a resident slot each and keep sixteen (gathering the partial sums
            // costs what about eight slices do, more when workgroups share a compute unit);
            // measured on ResNet-50's layers at batches 1, 32 and 128 and on GEMMs of 128 to 512 rows
            const int64_t units = dev >= 0 && dev < 16 && cus[dev] > 0 ? cus[dev] : 256;
            while (splits < 16 && slices % (splits * 2) == 0 &&
                   ((tiles * splits * 2 * 4 <= units * 3 && slices * kDeep / (splits * 2) >= 8) || (WM == 2 && tiles * splits * 2 <= resident && slices * kDeep / (splits * 2) >= 16)))
                splits *= 2;
        }
        int32_t* partials = nullptr;
        uint32_t* counters = nullptr;
        if (splits > 1 && tiles * sizeof(uint32_t) <= kSplitCounterBytes)
        {
            void* p = nullptr;
            int rc = split_workspace(static_cast<size_t>(tiles) * splits * BM * BN * sizeof(int32_t), s, &counters, &p);
            if (rc != HIPQ_OK)
                return rc;
            partials = static_cast<int32_t*>(p);
        }
        else
            splits = 1;
        const int64_t items = tiles * splits;
        int split_shift = 0;
        while ((1 << split_shift) < splits)
            ++split_shift;
        const unsigned grid = static_cast<unsigned>(items < resident ? items : resident);
        // column blocks in groups of up to eight (a power of two that divides the grid: a workgroup
        // then stays in its column block), for operand reuse inside each compute die's L2
        int group_shift = 0;
        if (getenv("HIPQ_NO_TILE_GROUPS") == nullptr)
            while (group_shift < 3 && (2ll << group_shift) <= n_tiles && ((grid >> split_shift) % (2u << group_shift)) == 0 && (grid & ((1u << split_shift) - 1)) == 0)
                ++group_shift;
        kernel<<<grid, 256, lds_bytes, s>>>(xl, w, wsum, M, Kred, x_unsigned, static_cast<int32_t>(m_tiles), static_cast<int32_t>(n_tiles), split_shift, fast_div(m_tiles), fast_div(m_tiles << group_shift), group_shift, partials, counters, zp, epi, om, out);
        return check_launch(name);
    }

    // The kernels that load straight into LDS, for 8-bit channels-last outputs in whole 16-byte
    // pieces; returns HIPQ_ERR_UNSUPPORTED (nothing launched, no error text) when the call is not of that kind.
    template <class XL>
    static int launch_uniform(const XL& xl,
                              const int8_t* w,
                              const int32_t* wsum,
                              int64_t M,
                              int32_t N,
                              int32_t Kred,
                              int x_unsigned,
                              const ZeroPoints& zp,
                              const Epilogue& epi,
                              const OutMap& om,
                              void* out,
                              hipStream_t s,
                              const char* name)
    {
        const bool q8 = epi.out_t == HIPQ_U8 || epi.out_t == HIPQ_I8;
        const bool f32 = epi.out_t == HIPQ_F32 && epi.mode == EPI_FUSED && epi.sum_in == nullptr;
        if ((!q8 && !f32) || om.ncx || (N & 15) != 0 || (reinterpret_cast<uintptr_t>(out) & 15) != 0 || getenv("HIPQ_NO_DMA") != nullptr || getenv("HIPQ_NO_PIPE") != nullptr)
            return HIPQ_ERR_UNSUPPORTED;
        if (f32 && !XL::kFloatOut)
            return HIPQ_ERR_UNSUPPORTED;
        // Gelu + Quantize in the epilogue: the wide float-output kernels only
        const bool gelu_q8 = epi.post_scale != nullptr;
        if (gelu_q8 && (!f32 || N <= 64))
            return HIPQ_ERR_UNSUPPORTED;
        // row matrices with reductions in whole 128-byte pieces, no residual, wide outputs: deep slices
        bool deep = false;
        if constexpr (XL::kDeep)
        {
            deep = xl.deep_ok() && Kred % (2 * BK) == 0 && Kred >= 4 * BK && N > 64 && epi.sum_in == nullptr && getenv("HIPQ_NO_DEEP_SLICES") == nullptr;
            // two of those workgroups fit a compute unit where three of the regular ones do: a
            // tile count that the regular kernel takes in one round and the deep one in two stays
            // regular (4096 x 2304 outputs, 576 tiles on 256 units: 18.9 us against 22.9)
            const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
            const int64_t units = device_compute_units();
            if (tiles > 2 * units && tiles <= 3 * units)
                deep = false;
            // few tiles with long reductions are split over workgroups, which then hold few slices
            // each: three buffers of regular slices do better there (config 2 at 256 rows: 19.5 us
            // against 20.9)
            if (tiles * 8 <= units * 3 && Kred >= 16 * BK)
                deep = false;
        }
        // 128 x 128 tiles that leave compute units idle (and would have their reductions split over
        // workgroups, partial sums through memory): 64 x 128 tiles, twice as many, no split.
        // Row matrices only: a 3 x 3 filter's long reduction over gathered rows does better split
        // (512 -> 512 channels on 128 x 7 x 7 pixels: 34 us split, 40 us in half tiles)
        bool half_height = false;
        if constexpr (XL::kDeep && !XL::kPads)
        {
            const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
            half_height = deep && M > 64 && tiles <= device_compute_units() && getenv("HIPQ_NO_HALF_TILES") == nullptr;
        }
        if constexpr (XL::kFloatOut)
            if (f32)
            {
                if (half_height && gelu_q8)
                    return launch_pipe<XL, 2, 2, EPI_FUSED, false, OUT_GELU_Q8, 2 * BK, 1>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
                if (half_height)
                    return launch_pipe<XL, 2, 2, EPI_FUSED, false, OUT_F32, 2 * BK, 1>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
                if (gelu_q8)
                {
                    if (deep)
                        return launch_pipe<XL, 2, 2, EPI_FUSED, false, OUT_GELU_Q8, 2 * BK>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
                    return launch_pipe<XL, 2, 2, EPI_FUSED, false, OUT_GELU_Q8>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
                }
                if (N <= 64)
                    return launch_pipe<XL, 4, 1, EPI_FUSED, false, OUT_F32>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
                if (deep)
                    return launch_pipe<XL, 2, 2, EPI_FUSED, false, OUT_F32, 2 * BK>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
                return launch_pipe<XL, 2, 2, EPI_FUSED, false, OUT_F32>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
            }
        if constexpr (XL::kDeep)
            if (deep)
            {
                if (half_height && epi.mode == EPI_FUSED)
                    return launch_pipe<XL, 2, 2, EPI_FUSED, false, OUT_Q8, 2 * BK, 1>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
                if (epi.mode == EPI_INTERP)
                    return launch_pipe<XL, 2, 2, EPI_INTERP, false, OUT_Q8, 2 * BK>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
                return launch_pipe<XL, 2, 2, EPI_FUSED, false, OUT_Q8, 2 * BK>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
            }
        if (epi.mode == EPI_INTERP)
        {
            if (N <= 64)
                return launch_pipe<XL, 4, 1, EPI_INTERP, false>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
            return launch_pipe<XL, 2, 2, EPI_INTERP, false>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
        }
        if (epi.sum_in != nullptr)
        {
            if (N <= 64)
                return launch_pipe<XL, 4, 1, EPI_FUSED, true>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
            return launch_pipe<XL, 2, 2, EPI_FUSED, true>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
        }
        if (N <= 64)
            return launch_pipe<XL, 4, 1, EPI_FUSED, false>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
        return launch_pipe<XL, 2, 2, EPI_FUSED, false>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
    }

    // tile choice: narrow outputs (N <= 64) take 512 x 64 so each wavefront still owns 128 x 64
    template <class XL, bool X_ON_A, int MODE, int KIND>
    static int launch_best(const XL& xl,
                           const int8_t* w,
                           const int32_t* wsum,
                           int64_t M,
                           int32_t N,
                           int32_t Kred,
                           int x_unsigned,
                           const ZeroPoints& zp,
                           const Epilogue& epi,
                           const OutMap& om,
                           void* out,
                           hipStream_t s,
                           const char* name)
    {
        // 8-bit channels-last outputs in whole 16-byte pieces: the persistent pipelined kernel
        if (!X_ON_A && KIND == OUT_Q8 && (N & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 && getenv("HIPQ_NO_PIPE") == nullptr)
        {
            if (MODE == EPI_FUSED && epi.sum_in != nullptr)
            {
                if (N <= 64)
                    return launch_pipe<XL, 4, 1, EPI_FUSED, true>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
                return launch_pipe<XL, 2, 2, EPI_FUSED, true>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
            }
            if (N <= 64)
                return launch_pipe<XL, 4, 1, MODE, false>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
            return launch_pipe<XL, 2, 2, MODE, false>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
        }
        // short reductions are bound by latency, not by LDS traffic: small wavefront tiles (64 x 64)
        // take half the registers, so twice as many workgroups are resident to hide it; and when the
        // large tiles are too few to give every compute unit two (a 4096 x 768 output is 96 of them),
        // the small ones fill the chip better than the large ones use it
        const int64_t large_tiles = ((M + 255) / 256) * ((N + 127) / 128);
        if ((Kred <= 512 || large_tiles < 512) && N > 64 && getenv("HIPQ_NO_SMALL_TILE") == nullptr)
            return launch_tile<XL, 2, 2, 2, 2, X_ON_A, MODE, KIND>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
        if (N <= 64)
            return launch_tile<XL, 4, 2, 4, 1, X_ON_A, MODE, KIND>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
        return launch_tile<XL, 4, 2, 2, 2, X_ON_A, MODE, KIND>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
    }

    // epilogue policy x output kind -> instantiation
    template <class XL, bool X_ON_A>
    static int launch_epilogue(const XL& xl,
                               const int8_t* w,
                               const int32_t* wsum,
                               int64_t M,
                               int32_t N,
                               int32_t Kred,
                               int x_unsigned,
                               const ZeroPoints& zp,
                               const Epilogue& epi,
                               const OutMap& om,
                               void* out,
                               hipStream_t s,
                               const char* name)
    {
        const bool q8 = epi.out_t == HIPQ_U8 || epi.out_t == HIPQ_I8;
        if (epi.mode == EPI_INTERP)
        {
            if (q8)
                return launch_best<XL, X_ON_A, EPI_INTERP, OUT_Q8>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
            if (epi.out_t == HIPQ_I32)
                return launch_best<XL, X_ON_A, EPI_INTERP, OUT_I32>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
        }
        else
        {
            if (q8)
                return launch_best<XL, X_ON_A, EPI_FUSED, OUT_Q8>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
            if (epi.out_t == HIPQ_F32)
                return launch_best<XL, X_ON_A, EPI_FUSED, OUT_F32>(xl, w, wsum, M, N, Kred, x_unsigned, zp, epi, om, out, s, name);
        }
        return fail(HIPQ_ERR_UNSUPPORTED, "no MFMA kernel for this epilogue / output type");
    }
}
