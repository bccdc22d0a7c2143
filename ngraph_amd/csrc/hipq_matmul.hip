// f32 batched matrix product (attention scores and contexts of a transformer encoder; op::v0::Dot on
// two matrices is the batch of one).  64 x 64 output tiles, 16-deep steps through LDS, 4 x 4 outputs a
// lane in registers.  The reference accumulates f32 products in double, k ascending
// (src/ngraph/runtime/reference/dot.hpp:34-37 with widen<float> = double,
// convolution.hpp:34-44), and rounds the sum to f32 once; so does this kernel: a product of two
// floats is exact in double, hence the fused multiply-add rounds exactly as the reference's separate
// multiply and add, and the results are the reference's bit for bit.
#include "hipq_common.h"
#include "hipq_quant_math.h"

namespace hipq
{
    namespace
    {
        typedef float f4 __attribute__((ext_vector_type(4)));
        constexpr int TM = 64, TN = 64, TK = 16;

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

        // out[b] = op(A[b]) * op(B[b]): A is [M][K] (or [K][M] with ta), B is [K][N] (or [N][K] with tb)
        __global__ __launch_bounds__(256) void batch_matmul_f32_kernel(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ out, MatView view, MatQuant mq, int32_t M,
                                                                       int32_t K, int32_t N, int32_t ta, int32_t tb, int32_t m_tiles, int32_t n_tiles, int32_t vec_a, int32_t vec_b,
                                                                       int32_t vec_o)
        {
            __shared__ __attribute__((aligned(16))) float as[TK][TM + 4]; // [k][m]
            __shared__ __attribute__((aligned(16))) float bs[TK][TN + 4]; // [k][n]
            const int tid = threadIdx.x;
            int t = blockIdx.x;
            const int nt = t % n_tiles;
            t /= n_tiles;
            const int mt = t % m_tiles;
            const int64_t batch = t / m_tiles;
            const int64_t bo = batch / view.batch_inner, bi = batch - bo * view.batch_inner;
            const float* A = a + bo * view.a_outer + bi * view.a_inner;
            const float* B = b + bo * view.b_outer + bi * view.b_inner;
            const int64_t o_base = bo * view.o_outer + bi * view.o_inner;
            float* O = out ? out + o_base : nullptr;
            const int64_t lda = view.lda, ldb = view.ldb, ldo = view.ldo;
            const int m0 = mt * TM, n0 = nt * TN;
            const int tm = (tid >> 4) * 4, tn = (tid & 15) * 4; // this lane's 4 x 4 outputs within the tile
            double acc[4][4] = {};
            // 64 x 16 elements of each operand, four a lane, contiguous along the operand's rows in
            // memory; the next step's elements are fetched into registers while this step multiplies
            auto fetch_a = [&](int k0) -> f4 {
                f4 v = f4{0.0f, 0.0f, 0.0f, 0.0f};
                if (!ta)
                {
                    const int r = tid >> 2, kq = (tid & 3) * 4; // A[m0 + r][k0 + kq ..]
                    if (vec_a && m0 + r < M && k0 + kq + 3 < K)
                        v = *reinterpret_cast<const f4*>(A + static_cast<int64_t>(m0 + r) * lda + k0 + kq);
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            v[i] = (m0 + r < M && k0 + kq + i < K) ? A[static_cast<int64_t>(m0 + r) * lda + k0 + kq + i] : 0.0f;
                    }
                }
                else
                {
                    const int kk = tid >> 4, mq = (tid & 15) * 4; // A[k0 + kk][m0 + mq ..]
                    if (vec_a && k0 + kk < K && m0 + mq + 3 < M)
                        v = *reinterpret_cast<const f4*>(A + static_cast<int64_t>(k0 + kk) * lda + m0 + mq);
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            v[i] = (k0 + kk < K && m0 + mq + i < M) ? A[static_cast<int64_t>(k0 + kk) * lda + m0 + mq + i] : 0.0f;
                    }
                }
                return v;
            };
            auto put_a = [&](f4 v) {
                if (!ta)
                {
                    const int r = tid >> 2, kq = (tid & 3) * 4;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        as[kq + i][r] = v[i];
                }
                else
                {
                    const int kk = tid >> 4, mq = (tid & 15) * 4;
                    *reinterpret_cast<f4*>(&as[kk][mq]) = v;
                }
            };
            auto fetch_b = [&](int k0) -> f4 {
                f4 v = f4{0.0f, 0.0f, 0.0f, 0.0f};
                if (!tb)
                {
                    const int kk = tid >> 4, nq = (tid & 15) * 4; // B[k0 + kk][n0 + nq ..]
                    if (vec_b && k0 + kk < K && n0 + nq + 3 < N)
                        v = *reinterpret_cast<const f4*>(B + static_cast<int64_t>(k0 + kk) * ldb + n0 + nq);
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            v[i] = (k0 + kk < K && n0 + nq + i < N) ? B[static_cast<int64_t>(k0 + kk) * ldb + n0 + nq + i] : 0.0f;
                    }
                }
                else
                {
                    const int r = tid >> 2, kq = (tid & 3) * 4; // B[n0 + r][k0 + kq ..]
                    if (vec_b && n0 + r < N && k0 + kq + 3 < K)
                        v = *reinterpret_cast<const f4*>(B + static_cast<int64_t>(n0 + r) * ldb + k0 + kq);
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            v[i] = (n0 + r < N && k0 + kq + i < K) ? B[static_cast<int64_t>(n0 + r) * ldb + k0 + kq + i] : 0.0f;
                    }
                }
                return v;
            };
            auto put_b = [&](f4 v) {
                if (!tb)
                {
                    const int kk = tid >> 4, nq = (tid & 15) * 4;
                    *reinterpret_cast<f4*>(&bs[kk][nq]) = v;
                }
                else
                {
                    const int r = tid >> 2, kq = (tid & 3) * 4;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        bs[kq + i][r] = v[i];
                }
            };
            f4 va = fetch_a(0), vb = fetch_b(0);
            for (int k0 = 0; k0 < K; k0 += TK)
            {
                put_a(va);
                put_b(vb);
                __syncthreads();
                if (k0 + TK < K) // uniform
                {
                    va = fetch_a(k0 + TK);
                    vb = fetch_b(k0 + TK);
                }
#pragma unroll
                for (int k = 0; k < TK; ++k)
                {
                    // (past K both operands hold zeros: + 0 * 0 leaves a sum as it is -- a sum that started from +0 is never -0)
                    const f4 av = *reinterpret_cast<const f4*>(&as[k][tm]);
                    const f4 bv = *reinterpret_cast<const f4*>(&bs[k][tn]);
                    double ad[4], bd[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        ad[i] = static_cast<double>(av[i]);
                        bd[i] = static_cast<double>(bv[i]);
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i)
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            acc[i][j] = fma(ad[i], bd[j], acc[i][j]);
                }
                __syncthreads();
            }
            // (the optional quantized copy: Quantize of the f32 result, the arithmetic of hipq_quantize)
            const float qs = mq.out ? *mq.scale : 1.0f;
            const int32_t qz = mq.out ? load_zp(mq.zero_point, mq.quant_t) : 0;
            auto q1 = [&](float v) -> uint32_t {
                return mq.quant_t == HIPQ_U8 ? static_cast<uint32_t>(quantize_one<float, uint8_t>(v, qs, static_cast<uint8_t>(qz), mq.mode))
                                             : static_cast<uint32_t>(static_cast<uint8_t>(quantize_one<float, int8_t>(v, qs, static_cast<int8_t>(qz), mq.mode)));
            };
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                const int m = m0 + tm + i;
                if (m >= M)
                    continue;
                const int64_t at = static_cast<int64_t>(m) * ldo + n0 + tn;
                const f4 r = f4{static_cast<float>(acc[i][0]), static_cast<float>(acc[i][1]), static_cast<float>(acc[i][2]), static_cast<float>(acc[i][3])};
                if (n0 + tn + 3 < N && vec_o)
                {
                    if (O)
                        *reinterpret_cast<f4*>(O + at) = r;
                    if (mq.out)
                        *reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(mq.out) + o_base + at) = q1(r[0]) | (q1(r[1]) << 8) | (q1(r[2]) << 16) | (q1(r[3]) << 24);
                }
                else
                {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (n0 + tn + j < N)
                        {
                            if (O)
                                O[at + j] = r[j];
                            if (mq.out)
                                static_cast<uint8_t*>(mq.out)[o_base + at + j] = static_cast<uint8_t>(q1(r[j]));
                        }
                }
            }
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
    const int vec_o = (!out || (reinterpret_cast<uintptr_t>(out) & 15) == 0) && (!mq.out || (reinterpret_cast<uintptr_t>(mq.out) & 3) == 0) && all4(view.ldo, view.o_outer, view.o_inner);
    HIPQ_REQUIRE(batch * m_tiles * n_tiles < (1ll << 31), "too many tiles for one launch");
    batch_matmul_f32_kernel<<<static_cast<unsigned>(batch * m_tiles * n_tiles), 256, 0, as_stream(stream)>>>(a, b, out, view, mq, static_cast<int32_t>(M), static_cast<int32_t>(K),
                                                                                                              static_cast<int32_t>(N), transpose_a ? 1 : 0, transpose_b ? 1 : 0,
                                                                                                              static_cast<int32_t>(m_tiles), static_cast<int32_t>(n_tiles), vec_a, vec_b, vec_o);
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
