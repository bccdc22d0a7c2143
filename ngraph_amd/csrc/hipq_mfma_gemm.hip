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
    // policy and output kind resolved once instead of per element.  The caller brings the scalars
    // (ec) and its column's bias and scale: it asks memory for them before its main loop.
    struct SkinnyColumn
    {
        EpiConst ec;
        float bias, scale;
        int32_t wsum;
    };
    __device__ __forceinline__ SkinnyColumn skinny_column(const Epilogue& epi, const int32_t* __restrict__ wsum, int n, int32_t N)
    {
        SkinnyColumn c;
        c.ec = epi_const(epi);
        const bool ok = n < N;
        c.wsum = ok ? wsum[n] : 0;
        c.bias = (epi.mode == EPI_FUSED && epi.bias && ok) ? static_cast<float>(epi.bias[n]) : 0.0f;
        c.scale = (epi.mode == EPI_FUSED && epi.per_channel && ok) ? epi.scale[n] : c.ec.scale;
        return c;
    }
    template <int COUNT, class RowOf, class AccOf>
    __device__ __forceinline__ void skinny_finish(const Epilogue& epi, const EpiConst& ec, float bias, float scale, int32_t M, int32_t N, int n, RowOf row_of, AccOf acc_of,
                                                  void* __restrict__ out)
    {
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
        v4i bf[STEPS], af[MT][STEPS];
        auto load = [&](int kb) {
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
            {
                const int k = kb + st * 64;
                bf[st] = buffer_load16(wrs, (wrow != kOob && k < k_end) ? wrow + k : kOob);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    af[mt][st] = buffer_load16(ars, (arow[mt] != kOob && k < k_end) ? arow[mt] + k : kOob);
            }
        };
        // the weights and activations of the first steps are asked for before anything else; the
        // scalars and this lane's column constants (needed at the very end) right behind them
        load(k_begin);
        const int32_t xzp = load_zp(zp.data_zp, zp.data_t);
        const int32_t wzp = load_zp(zp.filter_zp, zp.filter_t);
        const SkinnyColumn col = skinny_column(epi, wsum, n0 + r16, N);
        if (wzp != 0) // uniform; w - wzp does not fit a signed byte: exact, slow
        {
            const EpiRegs er = epi_load(epi);
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

        v4acc acc[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            acc[mt] = v4acc{0, 0, 0, 0};
        for (int kb = k_begin; kb < k_end; kb += 64 * STEPS)
        {
            if (kb != k_begin)
                load(kb);
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
        const int32_t corr = ((x_unsigned ? 128 : 0) - xzp) * col.wsum;
        // lane: column lane % 16; accumulator register r is row 4 * (lane / 16) + r of the tile
        skinny_finish<MT * 4>(
            epi, col.ec, col.bias, col.scale, M, N, n, [&](int i) { return (i >> 2) * 16 + 4 * kc + (i & 3); },
            [&](int i) { return acc[i >> 2][i & 3] + red[0][i >> 2][i & 3][lane] + red[1][i >> 2][i & 3][lane] + red[2][i >> 2][i & 3][lane] + corr; }, out);
    }

    // dot_skinny_kernel for prepacked weights (at most 32 rows): every load whole cache lines.  A
    // fragment read from a row-major matrix puts consecutive lanes in sixteen different lines, and the
    // texture path looks up one line a clock: 16 bytes a clock instead of 64.  Here
    //  * the weights come from the blob's copy in fragment order: a wavefront's B fragment of (its 16
    //    columns, a 64-byte reduction step) is 1 KB of contiguous memory, and the steps of its quarter
    //    of K follow one another -- the workgroup's weights are four contiguous streams;
    //  * the activations go through LDS: a wavefront fetches its quarter of K of every row with loads
    //    that cover 1 KB of one row each (straight into LDS, all of them in flight at once: at most
    //    32 KB a wavefront) and reads the A fragments back.  Position p of row r holds chunk p ^ (r % 16)
    //    of the row's piece, so the sixteen lanes of a fragment read hit sixteen different columns.
    // SEG: 1 KB segments of a row's quarter of K (1: K <= 4096, 2: K <= 8192 with MT = 1).
    constexpr size_t kSkinnyfLds = 4 * 32768 + 3 * 2 * 4 * 64 * 4;

    template <int MT, int SEG>
    __global__ __launch_bounds__(256) void dot_skinnyf_kernel(const uint8_t* __restrict__ a,
                                                              const int8_t* __restrict__ w,
                                                              const v4i* __restrict__ wfrag,
                                                              const int32_t* __restrict__ wsum,
                                                              int32_t M,
                                                              int32_t N,
                                                              int32_t K,
                                                              int32_t x_unsigned,
                                                              ZeroPoints zp,
                                                              Epilogue epi,
                                                              void* __restrict__ out)
    {
        static_assert(MT * 16 * SEG * 1024 <= 32768, "a wavefront's activations fit its 32 KB of LDS");
        constexpr int STEPS = SEG * 16; // 64-byte steps of a wavefront's quarter of K
        extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int r16 = lane & 15;
        const int kc = lane >> 4;
        const int cb = static_cast<int>(blockIdx.x); // column block: 16 output columns
        const int n0 = cb * 16;
        const int ksteps = K >> 6;
        const int sq = (ksteps + 3) >> 2; // steps a wavefront (at most STEPS)
        // (rotated by workgroup: in lockstep all workgroups would queue on the same activation lines in L2)
        const int s_begin = ((wave + cb) & 3) * sq;
        const int s_end = min(ksteps, s_begin + sq);
        const v4i arsw = rsrc_words(a, static_cast<uint32_t>(M) * static_cast<uint32_t>(K));
        const __amdgpu_buffer_rsrc_t frs = make_rsrc(wfrag, static_cast<uint32_t>((N + 15) >> 4) * static_cast<uint32_t>(ksteps) * 1024u);
        uint8_t* const mine = lds + wave * 32768;
        const uint32_t ring = lds_address(mine);

        // the column constants of the epilogue first (they complete first and hold nothing up), then the
        // scalars through the scalar cache, then the operands: activations, then weights
        const int n = n0 + r16;
        const int nn = n < N ? n : 0;
        const bool with_bias = epi.mode == EPI_FUSED && epi.bias != nullptr, per_channel = epi.mode == EPI_FUSED && epi.per_channel != 0;
        const int32_t col_wsum = wsum[nn];
        const int32_t col_bias_raw = (with_bias ? epi.bias : wsum)[nn];
        const float col_scale_pc = (per_channel ? epi.scale : reinterpret_cast<const float*>(wsum))[nn];
        HeadWords hw = head_scalars_load(zp, epi, wsum);
#pragma unroll
        for (int r = 0; r < MT * 16; ++r)
#pragma unroll
            for (int sg = 0; sg < SEG; ++sg)
            {
                // lane p of (row r, segment sg) fetches chunk p ^ (r % 16) of the segment
                const int c = sg * 64 + (lane ^ (r & 15));
                const bool ok = (r < M) & (s_begin * 4 + c < s_end * 4);
                lds_dma16_unfenced(arsw, ok ? r * K + s_begin * 64 + c * 16 : kOob, ring + (r * SEG + sg) * 1024);
            }
        __builtin_amdgcn_sched_barrier(0);
        v4i bf[STEPS];
#pragma unroll
        for (int st = 0; st < STEPS; ++st)
            bf[st] = buffer_load16(frs, s_begin + st < s_end ? (cb * ksteps + s_begin + st) * 1024 + lane * 16 : kOob);
        __builtin_amdgcn_sched_barrier(0);

        const int xor_mask = x_unsigned ? static_cast<int>(0x80808080u) : 0;
        v4acc acc[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            acc[mt] = v4acc{0, 0, 0, 0};
        wait_vmcnt<STEPS>(); // the activations have landed (only the weights, asked for behind them, may be in flight)
#pragma unroll
        for (int st = 0; st < STEPS; ++st)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
            {
                // fragment (row tile mt, step st) of lane (row r16, chunk kc): chunk 4 st + kc of the row's piece.
                // Steps past the wavefront's range read zeros on the weight side, which cancel whatever is here.
                const int c = st * 4 + kc;
                const v4i t = *reinterpret_cast<const v4i*>(mine + ((mt * 16 + r16) * SEG + (c >> 6)) * 1024 + (((c & 63) ^ r16) << 4));
                const v4i x = v4i{t[0] ^ xor_mask, t[1] ^ xor_mask, t[2] ^ xor_mask, t[3] ^ xor_mask};
                acc[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x, bf[st], acc[mt], 0, 0, 0);
            }
        // the scalars are first looked at here, behind the whole reduction
        head_scalars_settle(hw);
        const HeadScalars hs = head_scalars_finish(hw, zp, epi);
        const int32_t xzp = hs.xzp, wzp = hs.wzp;
        const EpiConst ec = hs.ec;
        if (wzp != 0) // uniform; w - wzp does not fit a signed byte: exact, slow
        {
            const EpiRegs er = epi_load(epi);
            for (int i = tid; i < 16 * M; i += 256)
            {
                const int m = i >> 4, nx = n0 + (i & 15);
                if (nx < N)
                {
                    int32_t sum = 0;
                    for (int k = 0; k < K; ++k)
                    {
                        const int32_t xv = x_unsigned ? static_cast<int32_t>(a[static_cast<int64_t>(m) * K + k])
                                                      : static_cast<int32_t>(static_cast<int8_t>(a[static_cast<int64_t>(m) * K + k]));
                        sum += (xv - xzp) * (static_cast<int32_t>(w[static_cast<int64_t>(nx) * K + k]) - wzp);
                    }
                    const int64_t o = static_cast<int64_t>(m) * N + nx;
                    store_out(out, epi.out_t, o, epi_apply(epi, er, sum, nx, o));
                }
            }
            return;
        }
        // ---- the four partial tiles meet in LDS (behind the activation regions); wavefront 0 requantizes
        int32_t* const red = reinterpret_cast<int32_t*>(lds + 4 * 32768); // [3][MT][4][64]
        if (wave > 0)
        {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    red[(((wave - 1) * MT + mt) * 4 + r) * 64 + lane] = acc[mt][r];
        }
        __syncthreads();
        if (wave > 0 || n >= N)
            return;
        const int32_t corr = ((x_unsigned ? 128 : 0) - xzp) * col_wsum;
        // lane: column lane % 16; accumulator register r is row 4 * (lane / 16) + r of the tile
        skinny_finish<MT * 4>(
            epi, ec, with_bias ? static_cast<float>(col_bias_raw) : 0.0f, per_channel ? col_scale_pc : ec.scale, M, N, n, [&](int i) { return (i >> 2) * 16 + 4 * kc + (i & 3); },
            [&](int i) {
                const int mt = i >> 2, r = i & 3;
                return acc[mt][r] + red[((0 * MT + mt) * 4 + r) * 64 + lane] + red[((1 * MT + mt) * 4 + r) * 64 + lane] + red[((2 * MT + mt) * 4 + r) * 64 + lane] + corr;
            },
            out);
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
        // (the scalars and this lane's column constants are asked for behind the first fragments)
        const int32_t xzp = load_zp(zp.data_zp, zp.data_t);
        const int32_t wzp = load_zp(zp.filter_zp, zp.filter_t);
        const SkinnyColumn col = skinny_column(epi, wsum, n0 + r16, N);
        if (wzp != 0) // uniform; exact, slow
        {
            const EpiRegs er = epi_load(epi);
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
        const int32_t corr = ((x_unsigned ? 128 : 0) - xzp) * col.wsum;
        // lane: column lane % 16; accumulator register r is row 4 * (lane / 16) + r of the tile
        skinny_finish<MT * 4>(
            epi, col.ec, col.bias, col.scale, M, N, n, [&](int i) { return (i >> 2) * 16 + 4 * kc + (i & 3); },
            [&](int i) { return acc[i >> 2][i & 3] + red[0][i >> 2][i & 3][lane] + red[1][i >> 2][i & 3][lane] + red[2][i >> 2][i & 3][lane] + corr; }, out);
    }

    // Between the skinny kernels and the tile kernels: a few hundred rows against a weight matrix that
    // must stream from HBM once (config 2 at 256 rows).  The tile kernels would have too few 128 x 128
    // tiles for the chip and split each reduction over workgroups, which costs a round trip of partial
    // sums through memory.  Here a workgroup owns a 64 x 64 output tile and the WHOLE reduction: its
    // eight wavefronts split K eight ways (128-byte pieces dealt round robin).  A wavefront brings
    // its piece of the 64 activation rows and the 64 weight rows straight into a 16 KB LDS region of
    // its own -- every load instruction is 8 rows x 128 bytes, eight whole cache lines (loads shaped
    // like an MFMA fragment, 16 rows x 64 bytes, run at less than half the rate) -- and reads the
    // v_mfma_i32_16x16x64_i8 fragments back 16 bytes a lane; the next piece is on its way while this
    // one multiplies.  No barrier in the loop: nothing is shared between wavefronts until the
    // eight partial tiles meet in LDS (each in its wavefront's region), after which every wavefront
    // requantizes two 16 x 16 blocks.  Everything the epilogue needs from memory (zero points,
    // scales, bias, weight sums) is asked for before the loop.  Workgroups of one compute die share
    // a run of column tiles, so each die's L2 fetches its part of the weights from HBM once.
    constexpr int kRows64Threads = 512;
    constexpr size_t kRows64Lds = 8 * 16384;

    __global__ __launch_bounds__(kRows64Threads) void dot_rows64_kernel(const uint8_t* __restrict__ a,
                                                                        const int8_t* __restrict__ w,
                                                                        const int32_t* __restrict__ wsum,
                                                                        int32_t M,
                                                                        int32_t N,
                                                                        int32_t K,
                                                                        int32_t tiles_m,
                                                                        int32_t x_unsigned,
                                                                        ZeroPoints zp,
                                                                        Epilogue epi,
                                                                        void* __restrict__ out)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int r16 = lane & 15;
        const int kc = lane >> 4;
        // workgroups are dealt round robin to the eight compute dies: renumber so that a die's
        // workgroups are consecutive tiles (row tiles of one column tile next to each other)
        const int grid = static_cast<int>(gridDim.x);
        const int id = (grid & 7) == 0 ? (static_cast<int>(blockIdx.x) & 7) * (grid >> 3) + (static_cast<int>(blockIdx.x) >> 3) : static_cast<int>(blockIdx.x);
        const int ct = id / tiles_m, rt = id - ct * tiles_m;
        const int m0 = rt * 64, n0 = ct * 64;
        const v4i arsw = rsrc_words(a, static_cast<uint32_t>(M) * static_cast<uint32_t>(K));
        const v4i wrsw = rsrc_words(w, static_cast<uint32_t>(N) * static_cast<uint32_t>(K));
        // One load instruction brings 8 rows x 128 bytes (eight whole cache lines) into a 1 KB block of
        // this wavefront's 16 KB region: [A, B][block of 8 rows][64 pieces of 16 bytes].  Which piece
        // (row rho, chunk c of the 128 bytes) a lane fetches decides where it lands (at 16 * lane), so
        // the block's order is free: piece (rho, c) sits at 16 * (c / 2) + 8 * ((c % 2) ^ (block % 2)) + rho,
        // which makes the fragment reads below conflict-free (16 lanes of one chunk index read rows of
        // an even and an odd block from 16 different 16-byte columns).
        const int rho = lane & 7;
        int32_t arow[8], wrow[8];
#pragma unroll
        for (int blk = 0; blk < 8; ++blk)
        {
            const int c = 2 * (lane >> 4) + (((lane >> 3) & 1) ^ (blk & 1));
            arow[blk] = m0 + blk * 8 + rho < M ? (m0 + blk * 8 + rho) * K + c * 16 : kOob;
            wrow[blk] = n0 + blk * 8 + rho < N ? (n0 + blk * 8 + rho) * K + c * 16 : kOob;
        }
        uint8_t* const mine = lds + wave * 16384;
        const uint32_t ring = lds_address(mine);
        auto issue = [&](int pc) {
            const int k = pc * 128;
#pragma unroll
            for (int blk = 0; blk < 8; ++blk)
            {
                // (K is a multiple of 64: a chunk of the second half of the last piece may be past the end)
                const int c16 = (2 * (lane >> 4) + (((lane >> 3) & 1) ^ (blk & 1))) * 16;
                const bool in_k = k + c16 < K;
                lds_dma16(wrsw, (in_k && wrow[blk] != kOob) ? wrow[blk] + k : kOob, ring + 8192 + blk * 1024);
                lds_dma16(arsw, (in_k && arow[blk] != kOob) ? arow[blk] + k : kOob, ring + blk * 1024);
            }
        };
        // fragment (16-row block i, 64-byte half h) of lane (row r16, chunk kc): at frag0 + 2048 i + 512 h
        const int frag0 = (r16 >> 3) * 1024 + (16 * (kc >> 1) + 8 * ((kc & 1) ^ (r16 >> 3)) + (r16 & 7)) * 16;
        // wavefront v takes pieces v, v + 8, ... (rotated by workgroup: in lockstep all workgroups of
        // a row tile would queue on the same activation lines in L2)
        const int pieces = (K + 127) >> 7;
        const int first = (wave + id) & 7;
        if (first < pieces) // uniform
            issue(first);

        // what the epilogue needs, asked for now: two blocks (i, j) = (blk / 4, blk % 4) a wavefront
        const int32_t xzp = load_zp(zp.data_zp, zp.data_t);
        const int32_t wzp = load_zp(zp.filter_zp, zp.filter_t);
        const EpiConst ec = epi_const(epi);
        int32_t col_wsum[2];
        float col_bias[2], col_scale[2];
#pragma unroll
        for (int b = 0; b < 2; ++b)
        {
            const int n = n0 + ((wave * 2 + b) & 3) * 16 + r16;
            const bool ok = n < N;
            col_wsum[b] = ok ? wsum[n] : 0;
            col_bias[b] = (epi.mode == EPI_FUSED && epi.bias && ok) ? static_cast<float>(epi.bias[n]) : 0.0f;
            col_scale[b] = (epi.mode == EPI_FUSED && epi.per_channel && ok) ? epi.scale[n] : ec.scale;
        }
        if (wzp != 0) // uniform; w - wzp does not fit a signed byte: exact, slow
        {
            wait_vmcnt<0>(); // nothing may still be on its way into LDS when the wavefront ends
            const EpiRegs er = epi_load(epi);
            for (int i = tid; i < 64 * 64; i += kRows64Threads)
            {
                const int m = m0 + (i >> 6), n = n0 + (i & 63);
                if (m < M && n < N)
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
        v4acc acc[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = v4acc{0, 0, 0, 0};
        for (int pc = first; pc < pieces; pc += 8)
        {
            wait_vmcnt<0>(); // the piece has landed
            v4i x[2][4], bf[2][4];
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    // out-of-range fragments read zeros; a zero weight fragment cancels whatever the
                    // sign bias makes of a zero activation fragment
                    const v4i t = *reinterpret_cast<const v4i*>(mine + frag0 + i * 2048 + h * 512);
                    x[h][i] = v4i{t[0] ^ xor_mask, t[1] ^ xor_mask, t[2] ^ xor_mask, t[3] ^ xor_mask};
                    bf[h][i] = *reinterpret_cast<const v4i*>(mine + 8192 + frag0 + i * 2048 + h * 512);
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the region is in registers: the next piece may overwrite it
            if (pc + 8 < pieces) // uniform
                issue(pc + 8);
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x[h][i], bf[h][j], acc[i][j], 0, 0, 0);
        }
        // ---- the eight partial tiles meet in LDS (each in its wavefront's region); every wavefront
        // finishes two 16 x 16 blocks --------------------------------------------------------------------
        v4acc* const red = reinterpret_cast<v4acc*>(lds);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                red[(wave * 16 + i * 4 + j) * 64 + lane] = acc[i][j];
        __syncthreads();
#pragma unroll
        for (int b = 0; b < 2; ++b)
        {
            const int blk = wave * 2 + b;
            v4acc sum = red[blk * 64 + lane];
#pragma unroll
            for (int v = 1; v < 8; ++v)
            {
                const v4acc t = red[(v * 16 + blk) * 64 + lane];
                sum = v4acc{sum[0] + t[0], sum[1] + t[1], sum[2] + t[2], sum[3] + t[3]};
            }
            const int n = n0 + (blk & 3) * 16 + r16;
            if (n >= N)
                continue;
            const int32_t corr = ((x_unsigned ? 128 : 0) - xzp) * col_wsum[b];
            const int mb = m0 + (blk >> 2) * 16 + 4 * kc;
            // lane: column lane % 16; accumulator register r is row 4 * (lane / 16) + r of the block
            skinny_finish<4>(
                epi, ec, col_bias[b], col_scale[b], M, N, n, [&](int i) { return mb + i; }, [&](int i) { return sum[i] + corr; }, out);
        }
    }

    // dot_rows64_kernel for prepacked weights and reductions of at most 8 * PW pieces of 128 bytes
    // (K <= 4096 at PW = 4), built on what bounds the kernel above:
    //  * The texture path looks up one cache line a clock.  A load whose consecutive lanes lie in
    //    different lines (an MFMA fragment read from a row-major matrix: sixteen rows, four lanes
    //    apart; or the kernel above, whose lane % 8 is the row) spends a lookup on every 16 bytes and
    //    takes a compute unit to ~40 GB/s; with consecutive lanes inside one line it takes whole lines
    //    at ~125 GB/s (measured: libhipq_probe, intake).  So the weights come from the blob's copy in
    //    fragment order -- a lane's B fragment is 16 bytes of a contiguous 1 KB block -- and the
    //    activation rows are fetched eight lanes a row, a row a line.
    //  * The weights, the operand that comes from HBM, bypass LDS: a lane asks for its B fragments of
    //    ALL the wavefront's pieces before anything else (32 loads of 16 bytes at PW = 4: the whole
    //    weight stream of the launch is requested in the kernel's first microsecond).  The
    //    activations, which every workgroup shares and the L2s serve, take the wavefront's LDS region
    //    as two halves, two pieces in flight.
    template <int PW>
    __global__ __launch_bounds__(kRows64Threads) void dot_rows64w_kernel(const uint8_t* __restrict__ a,
                                                                         const int8_t* __restrict__ w,
                                                                         const v4i* __restrict__ wfrag,
                                                                         const int32_t* __restrict__ wsum,
                                                                         int32_t M,
                                                                         int32_t N,
                                                                         int32_t K,
                                                                         int32_t tiles_m,
                                                                         int32_t x_unsigned,
                                                                         ZeroPoints zp,
                                                                         Epilogue epi,
                                                                         void* __restrict__ out)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int r16 = lane & 15;
        const int kc = lane >> 4;
        const int grid = static_cast<int>(gridDim.x);
        const int id = (grid & 7) == 0 ? (static_cast<int>(blockIdx.x) & 7) * (grid >> 3) + (static_cast<int>(blockIdx.x) >> 3) : static_cast<int>(blockIdx.x);
        const int ct = id / tiles_m, rt = id - ct * tiles_m;
        const int m0 = rt * 64, n0 = ct * 64;
        const v4i arsw = rsrc_words(a, static_cast<uint32_t>(M) * static_cast<uint32_t>(K));
        const int ksteps = K >> 6; // 64-byte reduction steps (K is a multiple of 64)
        const __amdgpu_buffer_rsrc_t frs = make_rsrc(wfrag, static_cast<uint32_t>((N + 15) >> 4) * static_cast<uint32_t>(ksteps) * 1024u);
        const int pieces = (K + 127) >> 7;
        const int first = (wave + id) & 7; // this wavefront's pieces: first, first + 8, ...

        // The column constants of the epilogue (two blocks (i, j) = (blk / 4, blk % 4) a wavefront) are
        // asked for first: loads complete in issue order, so waiting for these few at the end never
        // waits for anything else, and asked for last they would hold the operand stream in front of
        // them.  Unconditional loads from a safe index: no branch, no wait here.
        int32_t col_wsum[2], col_bias_raw[2];
        float col_scale_pc[2];
        const bool with_bias = epi.mode == EPI_FUSED && epi.bias != nullptr, per_channel = epi.mode == EPI_FUSED && epi.per_channel != 0;
#pragma unroll
        for (int b = 0; b < 2; ++b)
        {
            const int n = n0 + ((wave * 2 + b) & 3) * 16 + r16;
            const bool ok = n < N;
            const int nn = ok ? n : 0;
            // (raw values: a select on them here would wait for them here)
            col_wsum[b] = wsum[nn];
            col_bias_raw[b] = (with_bias ? epi.bias : wsum)[nn];
            col_scale_pc[b] = (per_channel ? epi.scale : reinterpret_cast<const float*>(wsum))[nn];
        }

        // Activations: a piece of the 64 rows (8 KB) into one half of the wavefront's 16 KB region, eight
        // blocks of 8 rows x 128 bytes.  A load instruction is one block: lanes 8 q ... 8 q + 7 fetch
        // row q, the eight 16-byte chunks of its line, and land at 16 * lane.  Which chunk a lane
        // fetches -- position p of row q in block blk holds chunk p ^ (q / 2 + 4 * (blk % 2)) -- makes the
        // fragment reads below conflict-free: sixteen lanes of one chunk index read rows of an even and
        // an odd block from sixteen different 16-byte columns.
        const int q8 = lane >> 3, p8 = lane & 7;
        int32_t arow[8];
        int c16[8];
#pragma unroll
        for (int blk = 0; blk < 8; ++blk)
        {
            c16[blk] = (p8 ^ ((q8 >> 1) | ((blk & 1) << 2))) * 16;
            arow[blk] = m0 + blk * 8 + q8 < M ? (m0 + blk * 8 + q8) * K + c16[blk] : kOob;
        }
        uint8_t* const mine = lds + wave * 16384;
        const uint32_t ring = lds_address(mine);
        // (a piece past the end is asked for all the same, out of range: it arrives as zeros and keeps
        // the count of loads in flight the same for every wavefront)
        auto issue_a = [&](int j) {
            const int pc = first + 8 * j;
            const int k = pc * 128;
#pragma unroll
            for (int blk = 0; blk < 8; ++blk)
            {
                const bool ok = (pc < pieces) & (k + c16[blk] < K) & (arow[blk] != kOob); // (no short-circuit: selects, not branches)
                lds_dma16_unfenced(arsw, ok ? arow[blk] + k : kOob, ring + (j & 1) * 8192 + blk * 1024);
            }
        };
        // weights: B fragment (column block jb, 64-byte half h) of piece j: 16 bytes of the 1 KB block
        // (column block, reduction step) of the fragment-ordered copy
        v4i bf[PW][2][4];
        auto load_w = [&](int j) {
            const int pc = first + 8 * j;
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int jb = 0; jb < 4; ++jb)
                {
                    const int ks = pc * 2 + h;
                    const bool ok = (ks < ksteps) & (n0 + jb * 16 < N);
                    bf[j][h][jb] = buffer_load16(frs, ok ? (((n0 >> 4) + jb) * ksteps + ks) * 1024 + lane * 16 : kOob);
                }
        };
        // The scalars (zero points, scales) are asked for just ahead of the operands, through the scalar
        // cache (a counter of their own: nothing waits for them until they are used, and they wait for
        // nothing; every address above is computed, so no wait for a kernel argument catches them)
        HeadWords hw = head_scalars_load(zp, epi, wsum);
        // issue order: [A0 W0] [A1 W1] W2 W3; A2 and A3 follow when their halves of the region are free
        // (fenced piece by piece: the waits below count loads in this order, and the scheduler is
        // otherwise free to issue a fragment of the first piece last)
#pragma unroll
        for (int j = 0; j < PW; ++j)
        {
            if (j < 2)
                issue_a(j);
            load_w(j);
            __builtin_amdgcn_sched_barrier(0);
        }

        const int xor_mask = x_unsigned ? static_cast<int>(0x80808080u) : 0;
        // fragment (16-row block i, 64-byte half h) of lane (row r16, chunk kc): block 2 i + r16 / 8, row r16 % 8,
        // chunk 4 h + kc at position chunk ^ (row / 2 + 4 * (block % 2))
        const int fswz = ((r16 & 7) >> 1) | ((r16 >> 3) << 2);
        const int frag_h[2] = {(r16 >> 3) * 1024 + (r16 & 7) * 128 + ((kc ^ fswz) << 4), (r16 >> 3) * 1024 + (r16 & 7) * 128 + (((4 + kc) ^ fswz) << 4)};
        v4acc acc[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = v4acc{0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < PW; ++j)
        {
            // Piece j's activations have landed once at most `later` younger loads are in flight
            // (vmcnt counts in issue order; the scalars asked for above only make the true count
            // larger).  Upfront pieces: everything issued behind [A_j W_j] at the start plus the
            // activation pieces issued by earlier steps; later pieces: only the next activation piece.
            constexpr int kLoadsA = 8, kLoadsW = 8;
            const int later = j < 2 ? (j == 0 ? (PW > 1 ? kLoadsA + kLoadsW : 0) + (PW > 2 ? (PW - 2) * kLoadsW : 0) : (PW - 2) * kLoadsW + (PW > 2 ? kLoadsA : 0))
                                    : (j + 1 < PW ? kLoadsA : 0);
            if (later >= 32)
                wait_vmcnt<32>();
            else if (later >= 24)
                wait_vmcnt<24>();
            else if (later >= 16)
                wait_vmcnt<16>();
            else if (later >= 8)
                wait_vmcnt<8>();
            else
                wait_vmcnt<0>();
            v4i x[2][4];
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    // out-of-range fragments read zeros; a zero weight fragment cancels whatever the
                    // sign bias makes of a zero activation fragment
                    const v4i t = *reinterpret_cast<const v4i*>(mine + (j & 1) * 8192 + frag_h[h] + i * 2048);
                    x[h][i] = v4i{t[0] ^ xor_mask, t[1] ^ xor_mask, t[2] ^ xor_mask, t[3] ^ xor_mask};
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the half is in registers: the piece after next may overwrite it
            if (j + 2 < PW)
                issue_a(j + 2);
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int jb = 0; jb < 4; ++jb)
                        acc[i][jb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x[h][i], bf[j][h][jb], acc[i][jb], 0, 0, 0);
        }
        // The scalars are first looked at here, behind the whole reduction: a wait for them (or the
        // exact path's own loads) in front of the loop would sit in front of every fragment of the loop.
        // A non-zero filter zero point discards the products and takes the exact path.
        head_scalars_settle(hw);
        const HeadScalars hs = head_scalars_finish(hw, zp, epi);
        const int32_t xzp = hs.xzp, wzp = hs.wzp;
        const EpiConst ec = hs.ec;
        if (wzp != 0) // uniform; w - wzp does not fit a signed byte: exact, slow
        {
            wait_vmcnt<0>(); // nothing may still be on its way into LDS when the wavefront ends
            const EpiRegs er = epi_load(epi);
            for (int i = tid; i < 64 * 64; i += kRows64Threads)
            {
                const int m = m0 + (i >> 6), n = n0 + (i & 63);
                if (m < M && n < N)
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
        // ---- the eight partial tiles meet in LDS (each in its wavefront's region); every wavefront
        // finishes two 16 x 16 blocks --------------------------------------------------------------------
        v4acc* const red = reinterpret_cast<v4acc*>(lds);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                red[(wave * 16 + i * 4 + j) * 64 + lane] = acc[i][j];
        __syncthreads();
#pragma unroll
        for (int b = 0; b < 2; ++b)
        {
            const int blk = wave * 2 + b;
            v4acc sum = red[blk * 64 + lane];
#pragma unroll
            for (int v = 1; v < 8; ++v)
            {
                const v4acc t = red[(v * 16 + blk) * 64 + lane];
                sum = v4acc{sum[0] + t[0], sum[1] + t[1], sum[2] + t[2], sum[3] + t[3]};
            }
            const int n = n0 + (blk & 3) * 16 + r16;
            if (n >= N)
                continue;
            const int32_t corr = ((x_unsigned ? 128 : 0) - xzp) * col_wsum[b];
            const int mb = m0 + (blk >> 2) * 16 + 4 * kc;
            skinny_finish<4>(
                epi, ec, with_bias ? static_cast<float>(col_bias_raw[b]) : 0.0f, per_channel ? col_scale_pc[b] : ec.scale, M, N, n, [&](int i) { return mb + i; },
                [&](int i) { return sum[i] + corr; }, out);
        }
    }

    // More than 64 rows, a long reduction, and too few 128 x 128 tiles to give every compute unit one
    // without splitting reductions; at most two rounds of 64 x 64 tiles.
    static bool dot_rows64_eligible(const hipq_dot_desc_t& d)
    {
        if (getenv("HIPQ_NO_ROWS64") != nullptr || d.M <= 64 || d.K % 64 != 0 || d.K < 1024)
            return false;
        const int64_t tiles64 = ((d.M + 63) / 64) * ((d.N + 63) / 64);
        const int64_t tiles128 = ((d.M + 127) / 128) * ((d.N + 127) / 128);
        const int cus = device_compute_units();
        return tiles128 * 4 < 3 * cus && tiles64 <= 2 * cus && d.M * d.K < (1ll << 31) && d.N * d.K < (1ll << 31);
    }

    static int launch_rows64(const hipq_dot_desc_t& d, const void* a, const void* w_nk, const void* w_frag, const int32_t* wsum, const ZeroPoints& zp, const Epilogue& epi, void* out, hipStream_t s)
    {
        static bool configured[16] = {};
        int dev = 0;
        HIPQ_HIP(hipGetDevice(&dev));
        if (dev >= 0 && dev < 16 && !configured[dev])
        {
            HIPQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dot_rows64_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kRows64Lds)));
            configured[dev] = true;
        }
        const int32_t tiles_m = static_cast<int32_t>((d.M + 63) / 64);
        const unsigned grid = static_cast<unsigned>(tiles_m * ((d.N + 63) / 64));
        // prepacked weights (fragment-ordered copy) and at most 32 pieces of 128 bytes: every byte asked
        // for up front, consecutive lanes in one cache line (HIPQ_ROWS64_PLAIN=1 keeps the kernel below)
        const int64_t pieces = (d.K + 127) / 128;
        if (w_frag && pieces <= 32 && getenv("HIPQ_ROWS64_PLAIN") == nullptr)
        {
            const int pw = static_cast<int>((pieces + 7) / 8);
            auto go = [&](auto kernel) {
                static bool set[16] = {};
                if (dev >= 0 && dev < 16 && !set[dev])
                {
                    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kRows64Lds)) != hipSuccess)
                        return fail(HIPQ_ERR_HIP, "cannot raise the LDS limit of dot_rows64w");
                    set[dev] = true;
                }
                kernel<<<grid, kRows64Threads, kRows64Lds, s>>>(static_cast<const uint8_t*>(a), static_cast<const int8_t*>(w_nk), static_cast<const v4i*>(w_frag), wsum,
                                                               static_cast<int32_t>(d.M), static_cast<int32_t>(d.N), static_cast<int32_t>(d.K), tiles_m, d.a_t == HIPQ_U8 ? 1 : 0, zp, epi, out);
                return check_launch("dot_rows64w_i8_16x16x64");
            };
            switch (pw)
            {
            case 1: return go(dot_rows64w_kernel<1>);
            case 2: return go(dot_rows64w_kernel<2>);
            case 3: return go(dot_rows64w_kernel<3>);
            default: return go(dot_rows64w_kernel<4>);
            }
        }
        dot_rows64_kernel<<<grid, kRows64Threads, kRows64Lds, s>>>(static_cast<const uint8_t*>(a), static_cast<const int8_t*>(w_nk), wsum, static_cast<int32_t>(d.M),
                                                                  static_cast<int32_t>(d.N), static_cast<int32_t>(d.K), tiles_m, d.a_t == HIPQ_U8 ? 1 : 0, zp, epi, out);
        return check_launch("dot_rows64_i8_16x16x64");
    }

    static bool dot_skinny_eligible(const hipq_dot_desc_t& d)
    {
        return d.M <= 256 && d.K % 64 == 0 && d.K >= 256 && d.M * d.K < (1ll << 31);
    }

    // products whose packed weights carry a copy in MFMA fragment order (the weight-streaming kernels
    // for prepacked weights read it)
    bool dot_fragments_eligible(const hipq_dot_desc_t& d)
    {
        return dot_mfma_eligible(d) && dot_skinny_eligible(d) && ((d.N + 15) / 16) * d.K * 16 < (1ll << 31);
    }
    size_t dot_fragment_bytes(const hipq_dot_desc_t& d) { return static_cast<size_t>((d.N + 15) / 16) * static_cast<size_t>(d.K / 64) * 1024; }

    template <int MT, int SEG>
    static int launch_skinnyf(const hipq_dot_desc_t& d, const void* a, const void* w_nk, const void* w_frag, const int32_t* wsum, const ZeroPoints& zp, const Epilogue& epi, void* out,
                              hipStream_t s)
    {
        auto kernel = dot_skinnyf_kernel<MT, SEG>;
        static bool set[16] = {};
        int dev = 0;
        HIPQ_HIP(hipGetDevice(&dev));
        if (dev >= 0 && dev < 16 && !set[dev])
        {
            HIPQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kSkinnyfLds)));
            set[dev] = true;
        }
        const unsigned grid = static_cast<unsigned>((d.N + 15) / 16);
        kernel<<<grid, 256, kSkinnyfLds, s>>>(static_cast<const uint8_t*>(a), static_cast<const int8_t*>(w_nk), static_cast<const v4i*>(w_frag), wsum, static_cast<int32_t>(d.M),
                                             static_cast<int32_t>(d.N), static_cast<int32_t>(d.K), d.a_t == HIPQ_U8 ? 1 : 0, zp, epi, out);
        return check_launch("dot_skinnyf_i8_16x16x64");
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

    // Quantize(Gelu(rows x weights -> f32)) with Gelu and Quantize in the epilogue of the kernels that
    // load straight into LDS; HIPQ_ERR_UNSUPPORTED (nothing launched, no error text) when the call is
    // not of their kind.  epi carries the Quantize in its post_* fields; out is the 8-bit tensor.
    int launch_rows_gelu_q8(const void* a, bool a_unsigned, const int8_t* w_nk, const int32_t* wsum, int64_t M, int32_t N, int32_t K, const ZeroPoints& zp, const Epilogue& epi,
                            void* out, hipStream_t s)
    {
        OutMap om{0, N, 1};
        RowsU xu;
        xu.x = static_cast<const uint8_t*>(a);
        xu.K = K;
        xu.bytes = static_cast<uint32_t>(M * K);
        return launch_uniform(xu, w_nk, wsum, M, N, K, a_unsigned ? 1 : 0, zp, epi, om, out, s, "dot_gelu_q8_mfma_i8_32x32x32");
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
                        hipStream_t s,
                        const void* w_frag)
    {
        HIPQ_REQUIRE(dot_mfma_eligible(d), "shape not eligible for the MFMA dot");
        HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w_nk) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(out) & 15) == 0,
                     "MFMA dot needs 16-byte aligned tensors");
        if (dot_skinny_eligible(d) && getenv("HIPQ_NO_SKINNY") == nullptr)
        {
            // prepacked weights: whole-line loads (fragment-ordered weights, activations through LDS)
            if (w_frag && d.M <= 32 && getenv("HIPQ_SKINNY_PLAIN") == nullptr)
            {
                if (d.M <= 16 && d.K <= 4096)
                    return launch_skinnyf<1, 1>(d, a, w_nk, w_frag, wsum, zp, epi, out, s);
                if (d.M <= 16 && d.K <= 8192)
                    return launch_skinnyf<1, 2>(d, a, w_nk, w_frag, wsum, zp, epi, out, s);
                if (d.K <= 4096)
                    return launch_skinnyf<2, 1>(d, a, w_nk, w_frag, wsum, zp, epi, out, s);
            }
            if (d.M <= 16)
                return launch_skinny<1, 16>(d, a, w_nk, wsum, zp, epi, out, s);
            if (d.M <= 32)
                return launch_skinny<2, 16>(d, a, w_nk, wsum, zp, epi, out, s);
            if (d.M <= 64)
                return launch_skinny<4, 8>(d, a, w_nk, wsum, zp, epi, out, s);
            if (dot_rows64_eligible(d))
                return launch_rows64(d, a, w_nk, w_frag, wsum, zp, epi, out, s);
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
