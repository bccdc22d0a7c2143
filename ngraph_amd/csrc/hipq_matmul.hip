// f32 batched matrix product (attention scores and contexts of a transformer encoder; op::v0::Dot on
// two matrices is the batch of one).  64 x 64 output tiles, the reduction in stages of 64 through
// LDS (f32), every wavefront a 32 x 32 quarter as 2 x 2 blocks of v_mfma_f64_16x16x4_f64.  The reference accumulates
// f32 products in double, k ascending (src/ngraph/runtime/reference/dot.hpp:34-37 with widen<float> =
// double, convolution.hpp:34-44), and rounds the sum to f32 once.  A product of two floats is exact
// in double, so a fused multiply-add rounds exactly as the reference's separate multiply and add;
// and the f64 matrix instruction accumulates its four products as a chain of such multiply-adds in
// k order (checked on the device against the chain: a million outputs over uniform, wide-range,
// integer-valued and cancelling operands, no bit differed -- and every parity test of this kernel
// is bit-exact against the oracle's sequential sum): the results are the reference's bit for bit.
// Operands are converted to double as fragments, one element a lane and matrix instruction, which
// is what makes the matrix instruction pay: the vector form converts eight operands for sixteen
// multiply-adds and is bound by the conversions.
#include <algorithm>

#include "hipq_common.h"
#include "hipq_quant_math.h"
#include "hipq_row_math.h"

namespace hipq
{
    namespace
    {
        typedef float f4 __attribute__((ext_vector_type(4)));
        typedef double d4 __attribute__((ext_vector_type(4)));
        constexpr int TM = 64, TN = 64, TK = 64, TKS = 16; // a stage is TK of the reduction, fetched and laid into LDS in pieces of TKS

        // where the matrices of batch element (outer, inner) start and how far apart their rows are (in
        // elements): the plain op has one batch level and dense matrices; views of a larger tensor
        // (the heads of a fused QKV projection, a context written head-interleaved) have two
        struct MatView
        {
            int64_t batch_inner;
            int64_t a_outer, a_inner, lda;
            int64_t b_outer, b_inner, ldb;
            int64_t o_outer, o_inner, ldo;
        };
        struct MatQuant
        {
            void* out; // null: none
            const float* scale;
            const void* zero_point;
            int32_t quant_t, mode;
        };

        // out[b] = op(A[b]) * op(B[b]): A is [M][K] (or [K][M] with ta), B is [K][N] (or [N][K] with tb).
        // A workgroup walks tiles item, item + grid, ...; the operands of the next stage -- the next
        // tile's first one after a tile's last -- are on their way into registers while this stage
        // multiplies, and a tile's stores drain under the next tile's products.  (One tile a workgroup,
        // all resident at once, runs the whole grid in lockstep: everyone loads, then everyone
        // multiplies, then everyone stores, and the three times add up.)
#ifndef BMM_PER_CU
#define BMM_PER_CU 3
#endif
#ifndef BMM_OCC
#define BMM_OCC __attribute__((amdgpu_waves_per_eu(3, 3)))
#endif
        struct TileAt
        {
            const float* A;
            const float* B;
            int64_t o_base;
            int m0, n0;
        };

        // WHOLE: every tile is full (M, N multiples of 64, K of TK) and every row 16-byte aligned, so
        // fetches and stores carry no bounds checks or scalar alternatives (uniform, chosen by the host)
        template <bool WHOLE, bool ta, bool tb>
        __global__ __launch_bounds__(256) BMM_OCC void batch_matmul_f32_kernel(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ out, MatView view, MatQuant mq, int32_t M,
                                                                       int32_t K, int32_t N, int32_t m_tiles, int32_t n_tiles, int32_t tiles, int32_t vec_a, int32_t vec_b)
        {
            // An operand lies in LDS the way it lies in memory, so that every piece goes in as one 16-byte
            // write: [row][k] when its rows run along the reduction (A as given, B transposed), [k][row]
            // otherwise.  The pitches spread a fragment read (16 rows x 4 consecutive k a wavefront)
            // over all 64 banks: 68 floats a row ([row][k]: bank 4 row + k), 80 floats a k ([k][row]: bank 16 k + row).
            constexpr int PR = TK + 4, PK = TM + 16;
            constexpr int OPERAND = TM * PR > TK * PK ? TM * PR : TK * PK;
            __shared__ __attribute__((aligned(16))) float as[OPERAND];
            __shared__ __attribute__((aligned(16))) float bs[OPERAND];
            auto a_at = [](int k, int m) { return ta ? k * PK + m : m * PR + k; };
            auto b_at = [](int k, int n) { return tb ? n * PR + k : k * PK + n; };
            const int tid = threadIdx.x;
            const int64_t lda = view.lda, ldb = view.ldb, ldo = view.ldo;
            const int lane = tid & 63, wave = tid >> 6;
            const int r16 = lane & 15, kq = lane >> 4;          // fragment element: row / column r16 of a block, k = 4 * step + kq
            const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32; // this wavefront's quarter of the tile
            // workgroups are dealt round-robin to the 8 XCDs (an L2 each): renumbered so that
            // neighbouring tiles, which share operand rows, meet in one L2
            const int grid = static_cast<int>(gridDim.x);
            const int item = (grid & 7) == 0 ? (static_cast<int>(blockIdx.x) & 7) * (grid >> 3) + (static_cast<int>(blockIdx.x) >> 3) : static_cast<int>(blockIdx.x);
            const uint32_t batch_inner = static_cast<uint32_t>(view.batch_inner < (1ll << 31) ? view.batch_inner : (1ll << 31)); // (there are fewer than 2^31 tiles)
            auto tile_at = [&](int t) -> TileAt {
                const int nt = t % n_tiles;
                t /= n_tiles;
                const int mt = t % m_tiles;
                const uint32_t batch = static_cast<uint32_t>(t / m_tiles);
                const int64_t bo = batch / batch_inner, bi = batch - bo * batch_inner; // (32-bit division)
                return TileAt{a + bo * view.a_outer + bi * view.a_inner, b + bo * view.b_outer + bi * view.b_inner, bo * view.o_outer + bi * view.o_inner, mt * TM, nt * TN};
            };
            // 64 x 16 elements of each operand a piece, four a lane, contiguous along the operand's rows in memory
            auto fetch_a = [&](const TileAt& w, int k0) -> f4 {
                f4 v = f4{0.0f, 0.0f, 0.0f, 0.0f};
                if (!ta)
                {
                    const int r = tid >> 2, kq = (tid & 3) * 4; // A[m0 + r][k0 + kq ..]
                    if (WHOLE || (vec_a && w.m0 + r < M && k0 + kq + 3 < K))
                        v = *reinterpret_cast<const f4*>(w.A + static_cast<int64_t>(w.m0 + r) * lda + k0 + kq);
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            v[i] = (w.m0 + r < M && k0 + kq + i < K) ? w.A[static_cast<int64_t>(w.m0 + r) * lda + k0 + kq + i] : 0.0f;
                    }
                }
                else
                {
                    const int kk = tid >> 4, mq = (tid & 15) * 4; // A[k0 + kk][m0 + mq ..]
                    if (WHOLE || (vec_a && k0 + kk < K && w.m0 + mq + 3 < M))
                        v = *reinterpret_cast<const f4*>(w.A + static_cast<int64_t>(k0 + kk) * lda + w.m0 + mq);
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            v[i] = (k0 + kk < K && w.m0 + mq + i < M) ? w.A[static_cast<int64_t>(k0 + kk) * lda + w.m0 + mq + i] : 0.0f;
                    }
                }
                return v;
            };
            auto put_a = [&](f4 v, int kbase) {
                if (!ta)
                {
                    const int r = tid >> 2, kq = (tid & 3) * 4;
                    *reinterpret_cast<f4*>(&as[a_at(kbase + kq, r)]) = v;
                }
                else
                {
                    const int kk = tid >> 4, mq = (tid & 15) * 4;
                    *reinterpret_cast<f4*>(&as[a_at(kbase + kk, mq)]) = v;
                }
            };
            auto fetch_b = [&](const TileAt& w, int k0) -> f4 {
                f4 v = f4{0.0f, 0.0f, 0.0f, 0.0f};
                if (!tb)
                {
                    const int kk = tid >> 4, nq = (tid & 15) * 4; // B[k0 + kk][n0 + nq ..]
                    if (WHOLE || (vec_b && k0 + kk < K && w.n0 + nq + 3 < N))
                        v = *reinterpret_cast<const f4*>(w.B + static_cast<int64_t>(k0 + kk) * ldb + w.n0 + nq);
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            v[i] = (k0 + kk < K && w.n0 + nq + i < N) ? w.B[static_cast<int64_t>(k0 + kk) * ldb + w.n0 + nq + i] : 0.0f;
                    }
                }
                else
                {
                    const int r = tid >> 2, kq = (tid & 3) * 4; // B[n0 + r][k0 + kq ..]
                    if (WHOLE || (vec_b && w.n0 + r < N && k0 + kq + 3 < K))
                        v = *reinterpret_cast<const f4*>(w.B + static_cast<int64_t>(w.n0 + r) * ldb + k0 + kq);
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            v[i] = (w.n0 + r < N && k0 + kq + i < K) ? w.B[static_cast<int64_t>(w.n0 + r) * ldb + k0 + kq + i] : 0.0f;
                    }
                }
                return v;
            };
            auto put_b = [&](f4 v, int kbase) {
                if (!tb)
                {
                    const int kk = tid >> 4, nq = (tid & 15) * 4;
                    *reinterpret_cast<f4*>(&bs[b_at(kbase + kk, nq)]) = v;
                }
                else
                {
                    const int r = tid >> 2, kq = (tid & 3) * 4;
                    *reinterpret_cast<f4*>(&bs[b_at(kbase + kq, r)]) = v;
                }
            };
            // (the optional quantized copy: Quantize of the f32 result, the arithmetic of hipq_quantize)
            const float qs = mq.out ? *mq.scale : 1.0f;
            const int32_t qz = mq.out ? load_zp(mq.zero_point, mq.quant_t) : 0;
            auto q1 = [&](float v) -> uint32_t {
                return mq.quant_t == HIPQ_U8 ? static_cast<uint32_t>(quantize_one<float, uint8_t>(v, qs, static_cast<uint8_t>(qz), mq.mode))
                                             : static_cast<uint32_t>(static_cast<uint8_t>(quantize_one<float, int8_t>(v, qs, static_cast<int8_t>(qz), mq.mode)));
            };
            d4 acc[2][2];
            auto clear = [&]() {
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = d4{0.0, 0.0, 0.0, 0.0};
            };
            // block (i, j), register e of lane (r16, kq): row wm + 16 i + 4 e + kq, column wn + 16 j + r16.
            // A finished tile is rounded to f32 into `res` and stored one stage later, after the next
            // tile's operands have arrived: loads and stores share one counter, so stores issued just
            // before that wait would have to be acknowledged before the next tile could start.
            float res[2][2][4];
            auto round_tile = [&]() {
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            res[i][j][e] = static_cast<float>(acc[i][j][e]);
            };
            auto each_result = [&](const TileAt& w, auto&& f) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                    {
                        const int m = w.m0 + wm + i * 16 + 4 * e + kq;
                        if (!WHOLE && m >= M)
                            continue;
#pragma unroll
                        for (int j = 0; j < 2; ++j)
                        {
                            const int n = w.n0 + wn + j * 16 + r16;
                            if (!WHOLE && n >= N)
                                continue;
                            f(w.o_base + static_cast<int64_t>(m) * ldo + n, res[i][j][e]);
                        }
                    }
            };
            auto store_tile = [&](const TileAt& w) {
                if (out) // uniform
                    each_result(w, [&](int64_t at, float r) { out[at] = r; });
                if (mq.out) // uniform
                    each_result(w, [&](int64_t at, float r) { static_cast<uint8_t*>(mq.out)[at] = static_cast<uint8_t>(q1(r)); });
            };

            if (item >= tiles) // uniform
                return;
            // a stage is TK of the reduction (the whole reduction of an attention score), asked for at once
            constexpr int PIECES = TK / TKS;
            int t_fetch = item, k_fetch = 0, k_done = 0;
            TileAt ft = tile_at(t_fetch); // the tile whose operands are being fetched
            TileAt ct = ft;               // the tile being multiplied
            TileAt st = ft;               // the finished tile waiting in `res`
            bool unsaved = false;         // uniform
            f4 va[PIECES], vb[PIECES];
#pragma unroll
            for (int q = 0; q < PIECES; ++q)
            {
                va[q] = fetch_a(ft, q * TKS);
                vb[q] = fetch_b(ft, q * TKS);
            }
            clear();
            for (;;)
            {
#pragma unroll
                for (int q = 0; q < PIECES; ++q)
                {
                    put_a(va[q], q * TKS);
                    put_b(vb[q], q * TKS);
                }
                __syncthreads();
                // the stage after this one: of this tile, or the first of the workgroup's next tile
                bool more = true; // uniform
                k_fetch += TK;
                if (k_fetch >= K)
                {
                    k_fetch = 0;
                    t_fetch += grid;
                    more = t_fetch < tiles;
                    if (more)
                        ft = tile_at(t_fetch);
                }
                if (more)
                {
#pragma unroll
                    for (int q = 0; q < PIECES; ++q)
                    {
                        va[q] = fetch_a(ft, k_fetch + q * TKS);
                        vb[q] = fetch_b(ft, k_fetch + q * TKS);
                    }
                }
                if (unsaved)
                {
                    store_tile(st);
                    unsaved = false;
                }
#pragma unroll
                for (int k = 0; k < TK; k += 4)
                {
                    // (past K both operands hold zeros: + 0 * 0 leaves a sum as it is -- a sum that started from +0 is never -0)
                    double ad[2], bd[2];
#pragma unroll
                    for (int i = 0; i < 2; ++i)
                    {
                        ad[i] = static_cast<double>(as[a_at(k + kq, wm + i * 16 + r16)]);
                        bd[i] = static_cast<double>(bs[b_at(k + kq, wn + i * 16 + r16)]);
                    }
#pragma unroll
                    for (int i = 0; i < 2; ++i)
#pragma unroll
                        for (int j = 0; j < 2; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(ad[i], bd[j], acc[i][j], 0, 0, 0);
                }
                __syncthreads();
                k_done += TK;
                if (k_done >= K) // the tile's last stage: the fetch cursor stands on the next tile
                {
                    round_tile();
                    st = ct;
                    if (!more)
                        break;
                    unsaved = true;
                    clear();
                    k_done = 0;
                    ct = ft;
                }
            }
            store_tile(st);
        }

        // ---- attention of one head in one kernel -------------------------------------------------------
        // out = BatchMatMul(Softmax(Multiply(BatchMatMulTranspose(Q, K), factor)), V), every op rounding
        // as the separate kernels round (the products through the same matrix instruction chain, the
        // Softmax through softmax_piece with the same lanes on the same pieces), so the result equals
        // the three launches bit for bit while the scores never leave the compute unit.
        // A work item is 32 query rows of one head against its 128 keys of depth 64.  LDS: Q [32][64],
        // K [128][64], V [128][64] as f32; the scores and probabilities [32][132] take K's place once K
        // has been multiplied.  Rows of Q and K are swizzled by k ^ 4 (row % 16), rows of V by
        // n ^ 16 (key % 4): fragment reads (16 rows x 4 consecutive k a wavefront) and the 16-byte
        // writes touch every bank once, without padding, which is what lets two workgroups share a
        // compute unit's 160 KB.
        // A workgroup walks items: V is asked for when the item starts and laid into LDS after the
        // scores, the next item's Q and K are asked for before the second product, and an item's
        // results wait in registers until the next item's operands have arrived (loads and stores
        // share one counter).
        constexpr int AQ = 32, AKEYS = 128, AD = 64, ASP = AKEYS + 4;
        constexpr size_t kAttnLdsBytes = static_cast<size_t>(AQ * AD + 2 * AKEYS * AD) * sizeof(float);
        static_assert(AQ * ASP <= AKEYS * AD, "the scores must fit K's region");
        struct AttnView
        {
            int64_t batch_inner;
            int64_t q_outer, q_inner, ldq;
            int64_t k_outer, k_inner, ldk;
            int64_t v_outer, v_inner, ldv;
            int64_t o_outer, o_inner, ldo;
        };
        struct AttnItem
        {
            const float* Q;
            const float* K;
            const float* V;
            int64_t o_base;
        };

        __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void attention_f32_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                                                                                 const float* __restrict__ v, const float* __restrict__ factor,
                                                                                                                 float* __restrict__ out, AttnView view, MatQuant mq, int32_t row_blocks,
                                                                                                                 int32_t items)
        {
            extern __shared__ __attribute__((aligned(16))) float attn_lds[];
            float* const Qs = attn_lds;
            float* const Ks = Qs + AQ * AD;
            float* const Vs = Ks + AKEYS * AD;
            float* const Ss = Ks;
            const int tid = threadIdx.x;
            const int lane = tid & 63, wave = tid >> 6;
            const int r16 = lane & 15, kq = lane >> 4;
            const int64_t ldq = view.ldq, ldk = view.ldk, ldv = view.ldv, ldo = view.ldo;
            const bool scaled = factor != nullptr;
            const float c = scaled ? *factor : 1.0f;
            const int grid = static_cast<int>(gridDim.x);
            // (workgroups are dealt round-robin to the 8 XCDs: renumbered so that the row blocks of a head meet in one L2)
            const int first = (grid & 7) == 0 ? (static_cast<int>(blockIdx.x) & 7) * (grid >> 3) + (static_cast<int>(blockIdx.x) >> 3) : static_cast<int>(blockIdx.x);
            if (first >= items) // uniform
                return;
            const uint32_t batch_inner = static_cast<uint32_t>(view.batch_inner < (1ll << 31) ? view.batch_inner : (1ll << 31));
            auto item_at = [&](int t) -> AttnItem {
                const int rb = t % row_blocks;
                const uint32_t batch = static_cast<uint32_t>(t / row_blocks);
                const int64_t bo = batch / batch_inner, bi = batch - bo * batch_inner;
                return AttnItem{q + bo * view.q_outer + bi * view.q_inner + static_cast<int64_t>(rb) * AQ * ldq, k + bo * view.k_outer + bi * view.k_inner,
                                v + bo * view.v_outer + bi * view.v_inner, bo * view.o_outer + bi * view.o_inner + static_cast<int64_t>(rb) * AQ * ldo};
            };
            // a thread's 16-byte pieces: row tid / 16 (+ 16 a piece), columns 4 (tid % 16) ..
            const int prow = tid >> 4, pcol = (tid & 15) * 4;
            f4 rq[2], rk[8], rv[8];
            auto fetch_qk = [&](const AttnItem& w) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    rq[i] = *reinterpret_cast<const f4*>(w.Q + static_cast<int64_t>(prow + 16 * i) * ldq + pcol);
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    rk[i] = *reinterpret_cast<const f4*>(w.K + static_cast<int64_t>(prow + 16 * i) * ldk + pcol);
            };
            auto fetch_v = [&](const AttnItem& w) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    rv[i] = *reinterpret_cast<const f4*>(w.V + static_cast<int64_t>(prow + 16 * i) * ldv + pcol);
            };
            auto put_qk = [&]() {
                const int at = prow * AD + (pcol ^ (4 * prow)); // (row % 16 = tid / 16 for every piece of the thread)
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    *reinterpret_cast<f4*>(Qs + at + i * 16 * AD) = rq[i];
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    *reinterpret_cast<f4*>(Ks + at + i * 16 * AD) = rk[i];
            };
            auto put_v = [&]() {
                const int at = prow * AD + (pcol ^ (16 * (prow & 3))); // (key % 4 = (tid / 16) % 4 for every piece)
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    *reinterpret_cast<f4*>(Vs + at + i * 16 * AD) = rv[i];
            };
            const float qs = mq.out ? *mq.scale : 1.0f;
            const int32_t qz = mq.out ? load_zp(mq.zero_point, mq.quant_t) : 0;
            auto q1 = [&](float x) -> uint32_t {
                return mq.quant_t == HIPQ_U8 ? static_cast<uint32_t>(quantize_one<float, uint8_t>(x, qs, static_cast<uint8_t>(qz), mq.mode))
                                             : static_cast<uint32_t>(static_cast<uint8_t>(quantize_one<float, int8_t>(x, qs, static_cast<int8_t>(qz), mq.mode)));
            };
            // second product: block i, register e of lane (r16, kq) = row 16 i + 4 e + kq, column 16 wave + r16
            float res[2][4];
            auto store_item = [&](const AttnItem& w) {
                if (out) // uniform
                {
#pragma unroll
                    for (int i = 0; i < 2; ++i)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            out[w.o_base + static_cast<int64_t>(16 * i + 4 * e + kq) * ldo + 16 * wave + r16] = res[i][e];
                }
                if (mq.out) // uniform
                {
                    const bool rne = mq.mode == HIPQ_ROUND_NEAREST_TOWARD_EVEN; // uniform: the Quantize kernels' four-at-a-time arithmetic
#pragma unroll
                    for (int i = 0; i < 2; ++i)
                    {
                        uint32_t four = 0;
                        if (rne)
                        {
                            const f4 x = f4{res[i][0], res[i][1], res[i][2], res[i][3]};
                            four = mq.quant_t == HIPQ_U8 ? quantize4<uint8_t, true>(x, qs, static_cast<float>(qz), mq.mode) : quantize4<int8_t, true>(x, qs, static_cast<float>(qz), mq.mode);
                        }
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            static_cast<uint8_t*>(mq.out)[w.o_base + static_cast<int64_t>(16 * i + 4 * e + kq) * ldo + 16 * wave + r16] =
                                static_cast<uint8_t>(rne ? (four >> (8 * e)) & 0xFFu : q1(res[i][e]));
                    }
                }
            };

            int t = first;
            AttnItem cur = item_at(t);
            AttnItem done = cur;
            bool unsaved = false; // uniform
            fetch_qk(cur);
            for (;;)
            {
                put_qk();
                __syncthreads();
                fetch_v(cur);
                if (unsaved)
                {
                    store_item(done);
                    unsaved = false;
                }
                // ---- scores: 32 x 128 over depth 64; this wavefront the 32 keys 32 wave .. as 2 x 2 blocks
                d4 acc[2][2];
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = d4{0.0, 0.0, 0.0, 0.0};
                {
                    const float* const qa = Qs + r16 * AD + kq;
                    const float* const kb = Ks + (32 * wave + r16) * AD + kq;
#pragma unroll
                    for (int s = 0; s < AD / 4; ++s)
                    {
                        const int off = (4 * s) ^ (4 * r16);
                        double ad[2], bd[2];
#pragma unroll
                        for (int i = 0; i < 2; ++i)
                        {
                            ad[i] = static_cast<double>(qa[off + i * 16 * AD]);
                            bd[i] = static_cast<double>(kb[off + i * 16 * AD]);
                        }
#pragma unroll
                        for (int i = 0; i < 2; ++i)
#pragma unroll
                            for (int j = 0; j < 2; ++j)
                                acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(ad[i], bd[j], acc[i][j], 0, 0, 0);
                    }
                }
                __syncthreads(); // every wavefront has read K: the scores take its place
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            Ss[(16 * i + 4 * e + kq) * ASP + 32 * wave + 16 * j + r16] = static_cast<float>(acc[i][j][e]);
                put_v();
                __syncthreads();
                // ---- Softmax of the rows: this wavefront rows 8 wave .., two at a time, 32 lanes a row
#pragma unroll
                for (int it = 0; it < 4; ++it)
                {
                    f4* const piece = reinterpret_cast<f4*>(Ss + (8 * wave + 2 * it + (lane >> 5)) * ASP) + (lane & 31);
                    *piece = softmax_piece<32>(*piece, true, scaled, c);
                }
                __syncthreads();
                // the next item's Q and K
                const int t_next = t + grid;
                const bool more = t_next < items; // uniform
                AttnItem next = cur;
                if (more)
                {
                    next = item_at(t_next);
                    fetch_qk(next);
                }
                // ---- context: 32 x 64 over the 128 keys; this wavefront columns 16 wave .. as 2 x 1 blocks
                d4 ctx[2] = {d4{0.0, 0.0, 0.0, 0.0}, d4{0.0, 0.0, 0.0, 0.0}};
                {
                    const float* const pa = Ss + r16 * ASP + kq;
                    const float* const vb = Vs + kq * AD + ((16 * wave + r16) ^ (16 * kq));
#pragma unroll
                    for (int s = 0; s < AKEYS / 4; ++s)
                    {
                        const double bd = static_cast<double>(vb[4 * s * AD]);
#pragma unroll
                        for (int i = 0; i < 2; ++i)
                            ctx[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(static_cast<double>(pa[4 * s + i * 16 * ASP]), bd, ctx[i], 0, 0, 0);
                    }
                }
                __syncthreads(); // every wavefront has read Q's, the probabilities' and V's regions
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        res[i][e] = static_cast<float>(ctx[i][e]);
                done = cur;
                if (!more)
                    break;
                unsaved = true;
                cur = next;
                t = t_next;
            }
            store_item(done);
        }
    }
}

using namespace hipq;

static int launch_batch_matmul(const float* a, const float* b, float* out, const MatView& view, const MatQuant& mq, int64_t batch, int64_t M, int64_t K, int64_t N, int32_t transpose_a,
                               int32_t transpose_b, void* stream)
{
    HIPQ_REQUIRE(M < (1ll << 31) && K < (1ll << 31) && N < (1ll << 31), "extent too large");
    const int64_t m_tiles = (M + TM - 1) / TM, n_tiles = (N + TN - 1) / TN;
    // 16-byte accesses along the rows when every row of every matrix starts aligned
    auto all4 = [](int64_t x, int64_t y, int64_t z) { return x % 4 == 0 && y % 4 == 0 && z % 4 == 0; };
    const int vec_a = (reinterpret_cast<uintptr_t>(a) & 15) == 0 && all4(view.lda, view.a_outer, view.a_inner);
    const int vec_b = (reinterpret_cast<uintptr_t>(b) & 15) == 0 && all4(view.ldb, view.b_outer, view.b_inner);
    HIPQ_REQUIRE(batch * m_tiles * n_tiles < (1ll << 31) - (1 << 20), "too many tiles for one launch");
    const int64_t tiles = batch * m_tiles * n_tiles;
    // three workgroups a compute unit (their LDS and the 12 wavefronts they make fit), each walking its share of the tiles
    const int64_t grid = std::min<int64_t>(tiles, static_cast<int64_t>(BMM_PER_CU) * device_compute_units());
    const bool whole = M % TM == 0 && N % TN == 0 && K % TK == 0 && K > 0 && vec_a && vec_b;
#define BMM_LAUNCH(W, TA, TB)                                                                                                                                                            \
    batch_matmul_f32_kernel<W, TA, TB><<<static_cast<unsigned>(grid), 256, 0, as_stream(stream)>>>(a, b, out, view, mq, static_cast<int32_t>(M), static_cast<int32_t>(K), static_cast<int32_t>(N), \
                                                                                                     static_cast<int32_t>(m_tiles), static_cast<int32_t>(n_tiles), static_cast<int32_t>(tiles), vec_a, vec_b)
#define BMM_T(W) (transpose_a ? (transpose_b ? BMM_LAUNCH(W, true, true) : BMM_LAUNCH(W, true, false)) : (transpose_b ? BMM_LAUNCH(W, false, true) : BMM_LAUNCH(W, false, false)))
    if (whole)
        BMM_T(true);
    else
        BMM_T(false);
#undef BMM_T
#undef BMM_LAUNCH
    return check_launch("batch_matmul_f32");
}

int hipq_batch_matmul_f32(const float* a, const float* b, float* out, int64_t batch, int64_t M, int64_t K, int64_t N, int32_t transpose_a, int32_t transpose_b, void* stream)
{
    HIPQ_REQUIRE(batch >= 0 && M >= 0 && K >= 0 && N >= 0, "negative extent");
    if (batch == 0 || M == 0 || N == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(out && (K == 0 || (a && b)), "null pointer");
    HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(out) & 15) == 0, "the output must be 16-byte aligned");
    const MatView view{1, M * K, 0, transpose_a ? M : K, K * N, 0, transpose_b ? K : N, M * N, 0, N};
    return launch_batch_matmul(a, b, out, view, MatQuant{nullptr, nullptr, nullptr, HIPQ_I8, HIPQ_ROUND_NEAREST_TOWARD_EVEN}, batch, M, K, N, transpose_a, transpose_b, stream);
}

int hipq_batch_matmul_view_f32(const float* a, const float* b, float* out, const hipq_matmul_view_t* v, const hipq_quant_out_t* q, int64_t batch, int64_t M, int64_t K, int64_t N,
                               int32_t transpose_a, int32_t transpose_b, void* stream)
{
    HIPQ_REQUIRE(v, "null view");
    HIPQ_REQUIRE(batch >= 0 && M >= 0 && K >= 0 && N >= 0, "negative extent");
    if (batch == 0 || M == 0 || N == 0)
        return HIPQ_OK;
    MatQuant mq{nullptr, nullptr, nullptr, HIPQ_I8, HIPQ_ROUND_NEAREST_TOWARD_EVEN};
    if (q)
    {
        HIPQ_REQUIRE(q->out && q->scale, "quantized output: null pointer");
        HIPQ_REQUIRE(q->quant_t == HIPQ_I8 || q->quant_t == HIPQ_U8, "quantized output: i8 or u8");
        HIPQ_REQUIRE(q->round_mode >= HIPQ_ROUND_NEAREST_TOWARD_INFINITY && q->round_mode <= HIPQ_ROUND_DOWN, "quantized output: unknown round mode");
        mq = MatQuant{q->out, q->scale, q->zero_point, q->quant_t, q->round_mode};
    }
    HIPQ_REQUIRE((out || mq.out) && (K == 0 || (a && b)), "null pointer");
    HIPQ_REQUIRE(v->batch_inner >= 1, "batch_inner must be at least 1");
    HIPQ_REQUIRE(v->lda >= (transpose_a ? M : K) && v->ldb >= (transpose_b ? K : N) && v->ldo >= N, "a row stride is shorter than the row");
    HIPQ_REQUIRE(v->a_outer >= 0 && v->a_inner >= 0 && v->b_outer >= 0 && v->b_inner >= 0 && v->o_outer >= 0 && v->o_inner >= 0, "negative batch stride");
    const MatView view{v->batch_inner, v->a_outer, v->a_inner, v->lda, v->b_outer, v->b_inner, v->ldb, v->o_outer, v->o_inner, v->ldo};
    return launch_batch_matmul(a, b, out, view, mq, batch, M, K, N, transpose_a, transpose_b, stream);
}

int hipq_attention_f32(const float* q, const float* k, const float* v, const float* factor, float* out, const hipq_attention_view_t* view, const hipq_quant_out_t* quant, int64_t batch,
                       int64_t queries, int64_t keys, int64_t depth, void* stream)
{
    HIPQ_REQUIRE(view, "null view");
    HIPQ_REQUIRE(batch >= 0 && queries >= 0 && keys >= 0 && depth >= 0, "negative extent");
    if (keys != AKEYS || depth != AD || queries % AQ != 0)
        return fail(HIPQ_ERR_UNSUPPORTED, "the one-kernel attention takes 128 keys of depth 64 and query rows in multiples of 32 (run the three ops otherwise)");
    if (batch == 0 || queries == 0)
        return HIPQ_OK;
    MatQuant mq{nullptr, nullptr, nullptr, HIPQ_I8, HIPQ_ROUND_NEAREST_TOWARD_EVEN};
    if (quant)
    {
        HIPQ_REQUIRE(quant->out && quant->scale, "quantized output: null pointer");
        HIPQ_REQUIRE(quant->quant_t == HIPQ_I8 || quant->quant_t == HIPQ_U8, "quantized output: i8 or u8");
        HIPQ_REQUIRE(quant->round_mode >= HIPQ_ROUND_NEAREST_TOWARD_INFINITY && quant->round_mode <= HIPQ_ROUND_DOWN, "quantized output: unknown round mode");
        mq = MatQuant{quant->out, quant->scale, quant->zero_point, quant->quant_t, quant->round_mode};
    }
    HIPQ_REQUIRE(q && k && v && (out || mq.out), "null pointer");
    HIPQ_REQUIRE(view->batch_inner >= 1, "batch_inner must be at least 1");
    HIPQ_REQUIRE(view->ldq >= depth && view->ldk >= depth && view->ldv >= depth && view->ldo >= depth, "a row stride is shorter than the row");
    HIPQ_REQUIRE(view->q_outer >= 0 && view->q_inner >= 0 && view->k_outer >= 0 && view->k_inner >= 0 && view->v_outer >= 0 && view->v_inner >= 0 && view->o_outer >= 0 && view->o_inner >= 0,
                 "negative batch stride");
    auto rows16 = [](const float* p, int64_t ld, int64_t outer, int64_t inner) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0 && ld % 4 == 0 && outer % 4 == 0 && inner % 4 == 0; };
    HIPQ_REQUIRE(rows16(q, view->ldq, view->q_outer, view->q_inner) && rows16(k, view->ldk, view->k_outer, view->k_inner) && rows16(v, view->ldv, view->v_outer, view->v_inner),
                 "rows of Q, K and V must start 16-byte aligned");
    const int64_t row_blocks = queries / AQ;
    HIPQ_REQUIRE(batch * row_blocks < (1ll << 31) - (1 << 20), "too many work items for one launch");
    static bool configured[16] = {};
    int dev = 0;
    HIPQ_HIP(hipGetDevice(&dev));
    if (dev >= 0 && dev < 16 && !configured[dev])
    {
        HIPQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(attention_f32_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kAttnLdsBytes)));
        configured[dev] = true;
    }
    const AttnView av{view->batch_inner, view->q_outer, view->q_inner, view->ldq, view->k_outer, view->k_inner, view->ldk,
                      view->v_outer, view->v_inner, view->ldv, view->o_outer, view->o_inner, view->ldo};
    const int64_t items = batch * row_blocks;
    // two workgroups a compute unit (their LDS fits twice), each walking its share of the items
    const int64_t grid = std::min<int64_t>(items, 2ll * device_compute_units());
    attention_f32_kernel<<<static_cast<unsigned>(grid), 256, kAttnLdsBytes, as_stream(stream)>>>(q, k, v, factor, out, av, mq, static_cast<int32_t>(row_blocks), static_cast<int32_t>(items));
    return check_launch("attention_f32");
}
