// int8 GEMM on the i8 matrix cores: eligibility and launch (kernel in hipq_igemm.h).
#include <cstdlib>
#include <type_traits>

#include "hipq_igemm.h"

namespace hipq
{
    // ---- skinny GEMM: M <= 256 ------------------------------------------------------------------
    // With a handful of rows the product is a stream over the weights: every weight byte must come
    // from HBM once and is used for at most 64 MACs.  One workgroup owns 16 output columns and the
    // whole reduction, so no partial sums leave the CU; its four wavefronts split K four ways, each
    // lane loads its v_mfma_i32_16x16x64_i8 fragments straight from global memory (16 bytes a lane,
    // sixteen 64-byte steps in flight before the first MFMA), and the four partial 16x16 tiles meet in
    // LDS.  N / 16 workgroups: 256 for N = 4096, one per CU.
    typedef int v4acc __attribute__((ext_vector_type(4)));

    // Requantization and store of one lane's finished outputs (column n, rows m[i]), with the
    // policy and output kind resolved once instead of per element.
    template <int COUNT, class RowOf, class AccOf>
    __device__ __forceinline__ void skinny_finish(const Epilogue& epi, int32_t M, int32_t N, int n, RowOf row_of, AccOf acc_of, void* __restrict__ out)
    {
        const EpiConst ec = epi_const(epi);
        const float bias = (epi.mode == EPI_FUSED && epi.bias) ? static_cast<float>(epi.bias[n]) : 0.0f;
        const float scale = (epi.mode == EPI_FUSED && epi.per_channel) ? epi.scale[n] : ec.scale;
        const bool relu = epi.relu != 0;
        auto run = [&](auto mode_c, auto kind_c) {
            constexpr int MODE = decltype(mode_c)::value;
            constexpr int KIND = decltype(kind_c)::value;
#pragma unroll
            for (int i = 0; i < COUNT; ++i)
            {
                const int m = row_of(i);
                if (m < M)
                {
                    const int32_t a = acc_of(i);
                    const int64_t o = static_cast<int64_t>(m) * N + n;
                    // (a convolution routed here may carry a residual sum input, indexed like the output)
                    const bool has_sum = MODE == EPI_FUSED && epi.sum_in != nullptr;
                    const float sv = has_sum ? static_cast<float>(load_q(epi.sum_in, epi.sum_t, o)) : 0.0f;
                    const int32_t v = MODE == EPI_INTERP ? epi_interp<KIND>(ec, a) : epi_fused<KIND>(ec, a, bias, scale, has_sum, sv, relu);
                    if (KIND == OUT_Q8)
                        static_cast<uint8_t*>(out)[o] = static_cast<uint8_t>(v);
                    else
                        static_cast<int32_t*>(out)[o] = v;
                }
            }
        };
        using std::integral_constant;
        const bool q8 = epi.out_t == HIPQ_U8 || epi.out_t == HIPQ_I8;
        if (epi.mode == EPI_INTERP)
        {
            if (q8)
                run(integral_constant<int, EPI_INTERP>{}, integral_constant<int, OUT_Q8>{});
            else
                run(integral_constant<int, EPI_INTERP>{}, integral_constant<int, OUT_I32>{});
        }
        else if (q8)
            run(integral_constant<int, EPI_FUSED>{}, integral_constant<int, OUT_Q8>{});
        else if (epi.out_t == HIPQ_F32)
            run(integral_constant<int, EPI_FUSED>{}, integral_constant<int, OUT_F32>{});
        else
            run(integral_constant<int, EPI_FUSED>{}, integral_constant<int, OUT_I32>{});
    }

    template <int MT, int STEPS>
    __global__ __launch_bounds__(256) void dot_skinny_kernel(const uint8_t* __restrict__ a,
                                                             const int8_t* __restrict__ w,
                                                             const int32_t* __restrict__ wsum,
                                                             int32_t M,
                                                             int32_t N,
                                                             int32_t K,
                                                             int32_t x_unsigned,
                                                             ZeroPoints zp,
                                                             Epilogue epi,
                                                             void* __restrict__ out)
    {
        __shared__ int32_t red[3][MT][4][64];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int r16 = lane & 15; // A: row within the m-tile, B: column within the n-tile
        const int kc = lane >> 4;  // 16-byte chunk of a 64-byte step
        const int n0 = blockIdx.x * 16;
        const int32_t xzp = load_zp(zp.data_zp, zp.data_t);
        const int32_t wzp = load_zp(zp.filter_zp, zp.filter_t);
        const EpiRegs er = epi_load(epi);
        if (wzp != 0) // uniform; w - wzp does not fit a signed byte: exact, slow
        {
            for (int i = tid; i < 16 * M; i += 256)
            {
                const int m = i >> 4, n = n0 + (i & 15);
                if (n < N)
                {
                    int32_t acc = 0;
                    for (int k = 0; k < K; ++k)
                    {
                        const int32_t xv = x_unsigned ? static_cast<int32_t>(a[static_cast<int64_t>(m) * K + k])
                                                      : static_cast<int32_t>(static_cast<int8_t>(a[static_cast<int64_t>(m) * K + k]));
                        acc += (xv - xzp) * (static_cast<int32_t>(w[static_cast<int64_t>(n) * K + k]) - wzp);
                    }
                    const int64_t o = static_cast<int64_t>(m) * N + n;
                    store_out(out, epi.out_t, o, epi_apply(epi, er, acc, n, o));
                }
            }
            return;
        }
        const int xor_mask = x_unsigned ? static_cast<int>(0x80808080u) : 0;
        const __amdgpu_buffer_rsrc_t ars = make_rsrc(a, static_cast<uint32_t>(M) * static_cast<uint32_t>(K));
        const __amdgpu_buffer_rsrc_t wrs = make_rsrc(w, static_cast<uint32_t>(N) * static_cast<uint32_t>(K));
        const int kq = ((K / 64 + 3) / 4) * 64; // bytes of K per wavefront, whole 64-byte steps
        // (rotated by workgroup: in lockstep all workgroups would queue on the same activation lines in L2)
        const int k_begin = ((wave + static_cast<int>(blockIdx.x)) & 3) * kq;
        const int k_end = min(K, k_begin + kq);
        const int32_t wrow = n0 + r16 < N ? (n0 + r16) * K + kc * 16 : kOob;
        int32_t arow[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            arow[mt] = mt * 16 + r16 < M ? (mt * 16 + r16) * K + kc * 16 : kOob;

        v4acc acc[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            acc[mt] = v4acc{0, 0, 0, 0};
        for (int kb = k_begin; kb < k_end; kb += 64 * STEPS)
        {
            v4i bf[STEPS], af[MT][STEPS];
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
            {
                const int k = kb + st * 64;
                bf[st] = buffer_load16(wrs, (wrow != kOob && k < k_end) ? wrow + k : kOob);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    af[mt][st] = buffer_load16(ars, (arow[mt] != kOob && k < k_end) ? arow[mt] + k : kOob);
            }
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                {
                    // out-of-range fragments read zeros; a zero weight fragment cancels whatever the
                    // sign bias makes of a zero activation fragment
                    const v4i x = v4i{af[mt][st][0] ^ xor_mask, af[mt][st][1] ^ xor_mask, af[mt][st][2] ^ xor_mask, af[mt][st][3] ^ xor_mask};
                    acc[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x, bf[st], acc[mt], 0, 0, 0);
                }
        }
        // ---- the four partial tiles meet in LDS; wavefront 0 requantizes ----------------------------
        if (wave > 0)
        {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    red[wave - 1][mt][r][lane] = acc[mt][r];
        }
        __syncthreads();
        if (wave > 0)
            return;
        const int n = n0 + r16;
        if (n >= N)
            return;
        const int32_t corr = ((x_unsigned ? 128 : 0) - xzp) * wsum[n];
        // lane: column lane % 16; accumulator register r is row 4 * (lane / 16) + r of the tile
        skinny_finish<MT * 4>(
            epi, M, N, n, [&](int i) { return (i >> 2) * 16 + 4 * kc + (i & 3); },
            [&](int i) { return acc[i >> 2][i & 3] + red[0][i >> 2][i & 3][lane] + red[1][i >> 2][i & 3][lane] + red[2][i >> 2][i & 3][lane] + corr; }, out);
    }

    // The same idea for up to 256 rows: the weight fragments of a 256-byte piece of K stay in
    // registers while the row tiles stream past them (activations come from L2, where all
    // workgroups share them); the activation fragments run four row tiles ahead of the MFMAs.
    template <int MT>
    __global__ __launch_bounds__(256) void dot_skinny_wide_kernel(const uint8_t* __restrict__ a,
                                                                  const int8_t* __restrict__ w,
                                                                  const int32_t* __restrict__ wsum,
                                                                  int32_t M,
                                                                  int32_t N,
                                                                  int32_t K,
                                                                  int32_t x_unsigned,
                                                                  ZeroPoints zp,
                                                                  Epilogue epi,
                                                                  void* __restrict__ out)
    {
        constexpr int D = 4;     // row tiles in flight
        constexpr int STEPS = 4; // 64-byte steps per piece of K
        __shared__ int32_t red[3][MT][4][64];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int r16 = lane & 15;
        const int kc = lane >> 4;
        const int n0 = blockIdx.x * 16;
        const int32_t xzp = load_zp(zp.data_zp, zp.data_t);
        const int32_t wzp = load_zp(zp.filter_zp, zp.filter_t);
        const EpiRegs er = epi_load(epi);
        if (wzp != 0) // uniform; exact, slow
        {
            for (int i = tid; i < 16 * M; i += 256)
            {
                const int m = i >> 4, n = n0 + (i & 15);
                if (n < N)
                {
                    int32_t acc = 0;
                    for (int k = 0; k < K; ++k)
                    {
                        const int32_t xv = x_unsigned ? static_cast<int32_t>(a[static_cast<int64_t>(m) * K + k])
                                                      : static_cast<int32_t>(static_cast<int8_t>(a[static_cast<int64_t>(m) * K + k]));
                        acc += (xv - xzp) * (static_cast<int32_t>(w[static_cast<int64_t>(n) * K + k]) - wzp);
                    }
                    const int64_t o = static_cast<int64_t>(m) * N + n;
                    store_out(out, epi.out_t, o, epi_apply(epi, er, acc, n, o));
                }
            }
            return;
        }
        const int xor_mask = x_unsigned ? static_cast<int>(0x80808080u) : 0;
        const __amdgpu_buffer_rsrc_t ars = make_rsrc(a, static_cast<uint32_t>(M) * static_cast<uint32_t>(K));
        const __amdgpu_buffer_rsrc_t wrs = make_rsrc(w, static_cast<uint32_t>(N) * static_cast<uint32_t>(K));
        // All workgroups read the same activations: in lockstep they would queue on the same L2
        // lines.  Each workgroup therefore gives its wavefronts another quarter of K and walks the
        // quarter's pieces from another starting piece.
        const int kq = ((K / 64 + 3) / 4) * 64;
        const int k_begin = ((wave + static_cast<int>(blockIdx.x)) & 3) * kq;
        const int k_end = min(K, k_begin + kq);
        const int pieces = (max(k_end - k_begin, 0) + 64 * STEPS - 1) / (64 * STEPS);
        const int rot = pieces > 0 ? (static_cast<int>(blockIdx.x) >> 2) % pieces : 0;
        auto piece_k = [&](int c) { // byte offset of the c-th piece in this workgroup's order
            int q = c + rot;
            q = q >= pieces ? q - pieces : q;
            return c < pieces ? k_begin + q * 64 * STEPS : k_end; // past the end: everything out of range
        };
        const int32_t wrow = n0 + r16 < N ? (n0 + r16) * K + kc * 16 : kOob;
        const int32_t arow0 = r16 * K + kc * 16; // row r16 of row tile 0

        auto load_b = [&](int kb, v4i(&bf)[STEPS]) {
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
            {
                const int k = kb + st * 64;
                bf[st] = buffer_load16(wrs, (wrow != kOob && k < k_end) ? wrow + k : kOob);
            }
        };
        auto load_a = [&](int kb, int mt, v4i(&af)[STEPS]) {
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
            {
                const int k = kb + st * 64;
                af[st] = buffer_load16(ars, (mt * 16 + r16 < M && k < k_end) ? arow0 + mt * 16 * K + k : kOob);
            }
        };

        v4acc acc[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            acc[mt] = v4acc{0, 0, 0, 0};
        v4i bf[STEPS], bfn[STEPS], af[D][STEPS];
        load_b(piece_k(0), bf);
#pragma unroll
        for (int d = 0; d < D; ++d)
            load_a(piece_k(0), d, af[d]);
        for (int c = 0; c < pieces; ++c)
        {
            const int kb = piece_k(c), kb_next = piece_k(c + 1);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
            {
                v4i x[STEPS];
#pragma unroll
                for (int st = 0; st < STEPS; ++st)
                    x[st] = v4i{af[mt % D][st][0] ^ xor_mask, af[mt % D][st][1] ^ xor_mask, af[mt % D][st][2] ^ xor_mask, af[mt % D][st][3] ^ xor_mask};
                // refill the slot with the row tile D ahead (of the next piece of K past the last tile)
                if (mt + D < MT)
                    load_a(kb, mt + D, af[mt % D]);
                else
                    load_a(kb_next, mt + D - MT, af[mt % D]);
                if (mt == MT - D)
                    load_b(kb_next, bfn);
#pragma unroll
                for (int st = 0; st < STEPS; ++st)
                    acc[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x[st], bf[st], acc[mt], 0, 0, 0);
            }
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
                bf[st] = bfn[st];
        }
        if (wave > 0)
        {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    red[wave - 1][mt][r][lane] = acc[mt][r];
        }
        __syncthreads();
        if (wave > 0)
            return;
        const int n = n0 + r16;
        if (n >= N)
            return;
        const int32_t corr = ((x_unsigned ? 128 : 0) - xzp) * wsum[n];
        // lane: column lane % 16; accumulator register r is row 4 * (lane / 16) + r of the tile
        skinny_finish<MT * 4>(
            epi, M, N, n, [&](int i) { return (i >> 2) * 16 + 4 * kc + (i & 3); },
            [&](int i) { return acc[i >> 2][i & 3] + red[0][i >> 2][i & 3][lane] + red[1][i >> 2][i & 3][lane] + red[2][i >> 2][i & 3][lane] + corr; }, out);
    }

    static bool dot_skinny_eligible(const hipq_dot_desc_t& d)
    {
        return d.M <= 256 && d.K % 64 == 0 && d.K >= 256 && d.M * d.K < (1ll << 31);
    }

    template <int MT, int STEPS>
    static int launch_skinny(const hipq_dot_desc_t& d, const void* a, const void* w_nk, const int32_t* wsum, const ZeroPoints& zp, const Epilogue& epi, void* out, hipStream_t s)
    {
        const unsigned grid = static_cast<unsigned>((d.N + 15) / 16);
        dot_skinny_kernel<MT, STEPS><<<grid, 256, 0, s>>>(static_cast<const uint8_t*>(a), static_cast<const int8_t*>(w_nk), wsum, static_cast<int32_t>(d.M),
                                                      static_cast<int32_t>(d.N), static_cast<int32_t>(d.K), d.a_t == HIPQ_U8 ? 1 : 0, zp, epi, out);
        return check_launch("dot_skinny_i8_16x16x64");
    }

    template <int MT>
    static int launch_skinny_wide(const hipq_dot_desc_t& d, const void* a, const void* w_nk, const int32_t* wsum, const ZeroPoints& zp, const Epilogue& epi, void* out, hipStream_t s)
    {
        const unsigned grid = static_cast<unsigned>((d.N + 15) / 16);
        dot_skinny_wide_kernel<MT><<<grid, 256, 0, s>>>(static_cast<const uint8_t*>(a), static_cast<const int8_t*>(w_nk), wsum, static_cast<int32_t>(d.M),
                                                   static_cast<int32_t>(d.N), static_cast<int32_t>(d.K), d.a_t == HIPQ_U8 ? 1 : 0, zp, epi, out);
        return check_launch("dot_skinny_wide_i8_16x16x64");
    }

    // rows of `a` ([M][K] bytes) against packed weights, channels-last 8-bit or wider output: the
    // tile kernels with the row-matrix loader (also the path of 1 x 1 convolutions, whose
    // channels-last data is such a matrix)
    int launch_rows_mfma(const void* a, bool a_unsigned, const int8_t* w_nk, const int32_t* wsum, int64_t M, int32_t N, int32_t K,
                         const ZeroPoints& zp, const Epilogue& epi, void* out, hipStream_t s, const char* name)
    {
        OutMap om{0, N, 1};
        {
            RowsU xu;
            xu.x = static_cast<const uint8_t*>(a);
            xu.K = K;
            xu.bytes = static_cast<uint32_t>(M * K);
            const int rc = launch_uniform(xu, w_nk, wsum, M, N, K, a_unsigned ? 1 : 0, zp, epi, om, out, s, name);
            if (rc != HIPQ_ERR_UNSUPPORTED)
                return rc;
        }
        GemmX xl;
        xl.x = static_cast<const uint8_t*>(a);
        xl.K = K;
        xl.bytes = static_cast<uint32_t>(M * K);
        return launch_epilogue<GemmX, false>(xl, w_nk, wsum, M, N, K, a_unsigned ? 1 : 0, zp, epi, om, out, s, name);
    }

    bool dot_mfma_eligible(const hipq_dot_desc_t& d)
    {
        if (d.b_t != HIPQ_I8 || (d.a_t != HIPQ_U8 && d.a_t != HIPQ_I8))
            return false;
        if (d.K % 16 != 0 || d.K <= 0 || d.M <= 0 || d.N <= 0)
            return false;
        if (!fits_i32(d.K) || !fits_i32(d.N) || d.N > 65535ll * 64 || !fits_i32(d.M * d.K) || !fits_i32(d.N * d.K))
            return false;
        return true;
    }

    int launch_dot_mfma(const hipq_dot_desc_t& d,
                        const void* a,
                        const void* w_nk,
                        const int32_t* wsum,
                        const ZeroPoints& zp,
                        const Epilogue& epi,
                        void* out,
                        hipStream_t s)
    {
        HIPQ_REQUIRE(dot_mfma_eligible(d), "shape not eligible for the MFMA dot");
        HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w_nk) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(out) & 15) == 0,
                     "MFMA dot needs 16-byte aligned tensors");
        if (dot_skinny_eligible(d) && getenv("HIPQ_NO_SKINNY") == nullptr)
        {
            if (d.M <= 16)
                return launch_skinny<1, 16>(d, a, w_nk, wsum, zp, epi, out, s);
            if (d.M <= 32)
                return launch_skinny<2, 16>(d, a, w_nk, wsum, zp, epi, out, s);
            if (d.M <= 64)
                return launch_skinny<4, 8>(d, a, w_nk, wsum, zp, epi, out, s);
            // above 64 rows an 8-bit or (fused policy) float output is faster on the tile kernels,
            // whose reductions are split over workgroups when the tiles are few (config 2, 256 rows:
            // 22 us against 44)
            const bool q8 = epi.out_t == HIPQ_U8 || epi.out_t == HIPQ_I8;
            const bool f32 = epi.out_t == HIPQ_F32 && epi.mode == EPI_FUSED && epi.sum_in == nullptr;
            if (!((q8 || f32) && d.N % 16 == 0) || getenv("HIPQ_NO_PIPE") != nullptr || (f32 && getenv("HIPQ_NO_DMA") != nullptr))
            {
                if (d.M <= 128)
                    return launch_skinny_wide<8>(d, a, w_nk, wsum, zp, epi, out, s);
                return launch_skinny_wide<16>(d, a, w_nk, wsum, zp, epi, out, s);
            }
        }
        return launch_rows_mfma(a, d.a_t == HIPQ_U8, static_cast<const int8_t*>(w_nk), wsum, d.M, static_cast<int32_t>(d.N), static_cast<int32_t>(d.K), zp, epi,
                                out, s, "dot_mfma_i8_32x32x32");
    }
}

#ifdef HIPQ_PIPE_CLOCKS
extern "C" HIPQ_API int hipq_debug_pipe_clocks_rows(long long* out384)
{
    return hipMemcpyFromSymbol(out384, HIP_SYMBOL(hipq::g_pipe_clock), sizeof(long long) * 384) == hipSuccess ? 0 : 1;
}
#endif
