// 1 x 1 convolutions that widen 64 or 128 channels to a multiple of 256 (a bottleneck block's last layer
// and its projection shortcut at the first stages of a ResNet), fused policy, channels-last, optionally
// with the residual input: layers that move 9 bytes through HBM for every 64 multiply-adds and are
// bound by that traffic.  What the general tile kernel leaves on the table there is overlap -- a
// workgroup loads, multiplies, requantizes and stores one tile after the other -- so this kernel is
// arranged around keeping the memory system busy:
//
//   * the weights of a wavefront's 128 output channels (8 or 16 KiB) stay in its registers as MFMA
//     fragments for the whole launch; a tile's operands are 64 pixels x C bytes of data (4 or 8 KiB,
//     shared by the four wavefronts through LDS) and, per wavefront, 32 pixels x 128 bytes of
//     residual;
//   * both arrive by loads straight into LDS, whole 128-byte lines an instruction for the
//     residual; the loads of tile j + 1 are issued before tile j is multiplied, into second
//     buffers, so a workgroup always has a tile's worth of reads in flight behind its stores;
//   * a wavefront owns 32 pixels x 128 channels: it requantizes in place over the residual it
//     has just read (one dword a lane and step, swizzled so that neighbouring pixels fall into
//     different banks) and writes whole 128-byte rows, eight lanes a row;
//   * one barrier a tile (the shared data tile), one wait: at most the previous tile's four
//     stores may still be in flight.
//
// Arithmetic: that of the tile kernels' fused epilogue (hipq_igemm.h) -- the accumulators start
// from 128 * sum(w) (+ the bias when it can be carried exactly), v = scale * (acc + bias)
// (+ sum_scale * residual, fused multiply-add), ReLU, round half to even, saturate.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include "hipq_igemm.h"

namespace hipq
{
    namespace
    {
        struct PwParams
        {
            const uint8_t* x;      // [M][C], C = 64 or 128
            const int8_t* w;       // [N][C]
            const int32_t* wsum;   // [N]
            uint8_t* out;          // [M][N]
            const uint8_t* sum_in; // [M][N] or null
            const int32_t* bias;   // [N] or null
            const float* scale;    // [N] or [1]
            const float* sum_scale;
            uint32_t x_bytes, out_bytes;
            int32_t M, N;
            int32_t tiles;     // 64-pixel tiles
            int32_t col_tiles; // N / 256
            int32_t x_unsigned, per_channel, relu, out_t, sum_t;
        };

        constexpr int kPwRows = 64;    // pixels of a workgroup's tile
        constexpr int kPwCols = 256;   // output channels of a workgroup's tile
        constexpr int kPwStage = 4096; // bytes of a wavefront's residual / output region

        // CIN: input channels, 64 or 128 (reduction steps of 32 bytes: 2 or 4; with 128 the weight
        // fragments take 64 registers)
        template <int CIN, bool HAS_SUM>
        __global__ __launch_bounds__(256, 3) void conv_pw64_kernel(const PwParams p)
        {
            constexpr int KS = CIN / 32;
            constexpr int NB = CIN == 64 ? 2 : 1; // accumulator blocks of 32 channels live at a time (registers: the weight fragments take 8 KS)
            constexpr int kPwData = kPwRows * CIN; // bytes of a tile's data in LDS
            extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
            constexpr int NSTAGE = HAS_SUM ? 2 : 1; // regions a wavefront: the residual of the next tile lands while this one is worked on
            uint8_t* const data = lds;                                       // [2][64 pixels][CIN bytes], swizzled like the tile kernels' operands
            uint8_t* const stage = lds + 2 * kPwData;                        // [4 wavefronts][NSTAGE][32 pixels][128 bytes]
            float* const consts = reinterpret_cast<float*>(stage + 4 * NSTAGE * kPwStage); // [3][256]: start values (as int), bias, scale
            const int tid = static_cast<int>(threadIdx.x);
            const int lane = tid & 63;
            const int half = lane >> 5;
            const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
            const int ph = wave & 1;  // pixels 32 ph .. of the tile
            const int cg = wave >> 1; // channels 128 cg .. of the workgroup's 256
            // a workgroup keeps its column block: the launcher makes the grid a multiple of col_tiles
            const int col = static_cast<int>(blockIdx.x) % p.col_tiles;
            const int first = static_cast<int>(blockIdx.x) / p.col_tiles;
            const int stride = static_cast<int>(gridDim.x) / p.col_tiles;
            if (first >= p.tiles)
                return;
            const int my_tiles = (p.tiles - first + stride - 1) / stride;
            const int n_wg = col * kPwCols;     // the workgroup's first channel
            const int n_wave = n_wg + cg * 128; // the wavefront's

            // ---- per-channel constants ----------------------------------------------------------
            bool fold;
            {
                const int32_t b = p.bias ? p.bias[n_wg + tid] : 0;
                fold = __syncthreads_and(b >= -(1 << 24) && b <= (1 << 24)) != 0;
                reinterpret_cast<int32_t*>(consts)[tid] = (p.x_unsigned ? 128 : 0) * p.wsum[n_wg + tid] + (fold ? b : 0);
                consts[256 + tid] = fold ? 0.0f : static_cast<float>(b);
                consts[512 + tid] = p.per_channel ? p.scale[n_wg + tid] : p.scale[0];
            }
            const float sum_scale = HAS_SUM ? *p.sum_scale : 0.0f;
            // the wavefront's weights as fragments: lane (c = lane % 32, half) of block ni, step ks holds
            // bytes [32 ks + 16 half, + 16) of weight row n_wave + 32 ni + c
            v4i wf[KS][4];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int ni = 0; ni < 4; ++ni)
                    wf[ks][ni] = *reinterpret_cast<const v4i*>(p.w + (n_wave + ni * 32 + (lane & 31)) * CIN + ks * 32 + half * 16);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int ni = 0; ni < 4; ++ni)
                    asm volatile("" ::"v"(wf[ks][ni])); // arrived before the loop: a wait for them inside it would also wait for the tile loads
            const int xor_mask = p.x_unsigned ? static_cast<int>(0x80808080u) : 0;

            // ---- loads --------------------------------------------------------------------------
            const v4i xrs = rsrc_words(p.x, p.x_bytes);
            const v4i srs = rsrc_words(p.sum_in, HAS_SUM ? p.out_bytes : 0u);
            const uint32_t data_lds = lds_address(data) + static_cast<uint32_t>(wave) * 1024u;
            constexpr int LPR = CIN / 16; // lanes that load one row of the data tile
            const uint32_t stage_lds = lds_address(stage) + static_cast<uint32_t>(wave) * (NSTAGE * kPwStage);
            // data: lane tid fills slot tid % LPR of row tid / LPR (and of the rows 256 / LPR further on) with the chunk that belongs there
            const int drow = tid / LPR;
            const int dchunk = CIN == 64 ? ((tid & 3) ^ ((drow >> 2) & 3)) : ((tid & 7) ^ ((drow >> 1) & 7));
            // residual / output rows: eight lanes a row, slot s of row r holds channels 16 (s ^ (r / 2 % 8)) ..
            auto issue = [&](int j) { // tile j of the workgroup's sequence (anything past the end loads nothing)
                const int64_t m0 = j < my_tiles ? static_cast<int64_t>(first + j * stride) * kPwRows : static_cast<int64_t>(p.M);
#pragma unroll
                for (int i = 0; i < CIN / 64; ++i) // (rows 32 apart share the swizzle of their slots)
                {
                    const int64_t m = m0 + drow + i * (256 / LPR);
                    const int32_t off = m < p.M ? static_cast<int32_t>(m) * CIN + dchunk * 16 : kOob;
                    lds_dma16(xrs, off, __builtin_amdgcn_readfirstlane(data_lds + static_cast<uint32_t>(j & 1) * kPwData + i * 4096));
                }
                if constexpr (HAS_SUM)
                {
                    const uint32_t base = __builtin_amdgcn_readfirstlane(stage_lds + static_cast<uint32_t>(j & 1) * kPwStage);
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        const int id = i * 64 + lane;
                        const int row = id >> 3;
                        const int piece = (id & 7) ^ ((row >> 1) & 7);
                        const int64_t m = m0 + ph * 32 + row;
                        lds_dma16(srs, m < p.M ? static_cast<int32_t>(m * p.N + n_wave + piece * 16) : kOob, base + i * 1024);
                    }
                }
            };

            const float magic = 12582912.0f; // 1.5 * 2^23: adding it rounds half to even into the low mantissa bits
            const float lo = p.out_t == HIPQ_U8 ? 0.0f : -128.0f, hi = p.out_t == HIPQ_U8 ? 255.0f : 127.0f;
            const float clamp_lo = p.relu ? fmaxf(lo, 0.0f) : lo;
            const float* const start_at = consts + cg * 128 + 4 * half;

            auto tile = [&](int j, auto folded, auto to_u8) {
                constexpr bool FOLD = decltype(folded)::value;
                constexpr bool PK_U8 = decltype(to_u8)::value;
                const uint8_t* const xs = data + (j & 1) * kPwData;
                uint8_t* const region = stage + (wave * NSTAGE + (HAS_SUM ? (j & 1) : 0)) * kPwStage;
                v4i xf[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                {
                    const int frow = ph * 32 + (lane & 31), fchunk = ks * 2 + half;
                    const v4i f = *reinterpret_cast<const v4i*>(xs + (CIN == 64 ? lds_offset(frow, fchunk) : frow * 128 + ((fchunk ^ ((frow >> 1) & 7)) << 4)));
                    xf[ks] = v4i{f[0] ^ xor_mask, f[1] ^ xor_mask, f[2] ^ xor_mask, f[3] ^ xor_mask};
                }
                const int row = lane & 31;
                // NB blocks of 32 channels at a time, not all four: registers
#pragma unroll
                for (int nh = 0; nh < 4 / NB; ++nh)
                {
                    __builtin_amdgcn_sched_barrier(0); // (the next blocks' reads stay behind these blocks' epilogue)
                    v16i acc[NB];
#pragma unroll
                    for (int i = 0; i < NB; ++i)
#pragma unroll
                        for (int g = 0; g < 4; ++g)
                        {
                            const v4i c4 = *reinterpret_cast<const v4i*>(start_at + (nh * NB + i) * 32 + 8 * g);
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                acc[i][4 * g + e] = c4[e];
                        }
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                        for (int i = 0; i < NB; ++i)
                            acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[ks][nh * NB + i], xf[ks], acc[i], 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < NB; ++i)
#pragma unroll
                        for (int g = 0; g < 4; ++g)
                        {
                            const int nl = (nh * NB + i) * 32 + 8 * g + 4 * half; // channel within the wavefront's 128
                            v4f bias4 = v4f{0.0f, 0.0f, 0.0f, 0.0f};
                            if (!FOLD)
                                bias4 = *reinterpret_cast<const v4f*>(consts + 256 + cg * 128 + nl);
                            const v4f scale4 = *reinterpret_cast<const v4f*>(consts + 512 + cg * 128 + nl);
                            uint32_t* const cell = reinterpret_cast<uint32_t*>(region + row * 128 + (((nl >> 4) ^ ((row >> 1) & 7)) << 4) + (nl & 15));
                            float s4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                            if (HAS_SUM)
                            {
                                const uint32_t sw = *cell;
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                {
                                    const uint32_t b = (sw >> (8 * e)) & 0xFFu;
                                    s4[e] = p.sum_t == HIPQ_I8 ? static_cast<float>(static_cast<int8_t>(b)) : static_cast<float>(b);
                                }
                            }
                            uint32_t packed = 0;
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                            {
                                const float a = static_cast<float>(acc[i][4 * g + e]);
                                float v = __fmul_rn(FOLD ? a : __fadd_rn(a, bias4[e]), scale4[e]);
                                if (HAS_SUM)
                                    v = fmaf(sum_scale, s4[e], v);
                                if constexpr (PK_U8)
                                {
                                    // float -> u8 with saturation to [0, 255] (the ReLU included) and round half to even
                                    packed = __builtin_amdgcn_cvt_pk_u8_f32(v, e, packed);
                                    continue;
                                }
                                v = __builtin_amdgcn_fmed3f(v, clamp_lo, hi);
                                if (e == 0)
                                    packed = __float_as_uint(__fadd_rn(v, magic));
                                else if (e == 1)
                                    asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(packed) : "v"(v), "v"(magic));
                                else if (e == 2)
                                    asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(packed) : "v"(v), "v"(magic));
                                else
                                    asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(packed) : "v"(v), "v"(magic));
                            }
                            *cell = packed;
                        }
                }
                // whole rows out: eight lanes a 128-byte row
                const int64_t m0 = static_cast<int64_t>(first + j * stride) * kPwRows + ph * 32;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    const int id = i * 64 + lane;
                    const int r = id >> 3;
                    const int piece = (id & 7) ^ ((r >> 1) & 7);
                    const int64_t m = m0 + r;
                    if (m < p.M)
                        *reinterpret_cast<v4i*>(p.out + m * p.N + n_wave + piece * 16) = *reinterpret_cast<const v4i*>(region + r * 128 + (id & 7) * 16);
                }
            };

            // ---- tiles ----------------------------------------------------------------------------
            const bool pack_u8 = p.out_t == HIPQ_U8;
            issue(0);
            for (int j = 0; j < my_tiles; ++j)
            {
                // everything but the previous tile's four stores has landed: this tile's data and residual
                if (j == 0)
                    wait_vmcnt<0>();
                else
                    wait_vmcnt<4>();
                __syncthreads(); // the data tile is whole; nobody reads the other data buffer any more
                issue(j + 1);
                if (fold) // uniform
                {
                    if (pack_u8) // uniform
                        tile(j, std::true_type{}, std::true_type{});
                    else
                        tile(j, std::true_type{}, std::false_type{});
                }
                else
                {
                    if (pack_u8) // uniform
                        tile(j, std::false_type{}, std::true_type{});
                    else
                        tile(j, std::false_type{}, std::false_type{});
                }
            }
            wait_vmcnt<0>(); // (the loads issued past the end land in LDS before the workgroup leaves)
        }
    }

    bool conv_pw64_eligible(const ConvGeom& g, const Epilogue& epi, const ZeroPoints& zp)
    {
        if (g.in[0] != 1 || g.f[0] != 1 || g.f[1] != 1 || g.f[2] != 1)
            return false;
        for (int i = 0; i < 3; ++i)
            if (g.dd[i] != 1 || g.dl[i] != 1 || g.st[i] != 1 || g.pb[i] != 0)
                return false;
        if (g.out[1] != g.in[1] || g.out[2] != g.in[2])
            return false;
        if (g.filter_t != HIPQ_I8 || (g.data_t != HIPQ_U8 && g.data_t != HIPQ_I8) || (g.out_t != HIPQ_U8 && g.out_t != HIPQ_I8))
            return false;
        if (epi.mode != EPI_FUSED || epi.post_scale != nullptr || zp.data_zp != nullptr || zp.filter_zp != nullptr)
            return false;
        if (g.data_layout != HIPQ_LAYOUT_NXC || g.out_layout != HIPQ_LAYOUT_NXC)
            return false;
        if ((g.C != 64 && g.C != 128) || g.K % kPwCols != 0 || g.K > 2048)
            return false;
        if (g.C == 128 && getenv("HIPQ_NO_PW128") != nullptr)
            return false;
        const int64_t M = g.N * g.in[1] * g.in[2];
        // few pixels: the tile kernels split their work better (HIPQ_PW64_MIN_ROWS moves the threshold)
        const char* const min_rows = getenv("HIPQ_PW64_MIN_ROWS");
        if (M < (min_rows ? atoll(min_rows) : 64 * 1024) || M * g.K >= (1ll << 31))
            return false;
        return getenv("HIPQ_NO_PW64") == nullptr;
    }

    int launch_conv_pw64(const ConvGeom& g, const void* data, const void* packed, const Epilogue& epi, void* out, hipStream_t s)
    {
        HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(data) & 15) == 0 && (reinterpret_cast<uintptr_t>(packed) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(epi.sum_in) & 15) == 0,
                     "MFMA convolution needs 16-byte aligned tensors");
        PwParams p;
        memset(&p, 0, sizeof(p));
        const int64_t M = g.N * g.in[1] * g.in[2];
        p.x = static_cast<const uint8_t*>(data);
        p.w = static_cast<const int8_t*>(packed);
        p.wsum = reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(packed) + align_up(static_cast<size_t>(g.K * g.C), 256));
        p.out = static_cast<uint8_t*>(out);
        p.sum_in = static_cast<const uint8_t*>(epi.sum_in);
        p.bias = epi.bias;
        p.scale = epi.scale;
        p.sum_scale = epi.sum_scale;
        p.x_bytes = static_cast<uint32_t>(M * g.C);
        p.out_bytes = static_cast<uint32_t>(M * g.K);
        p.M = static_cast<int32_t>(M);
        p.N = static_cast<int32_t>(g.K);
        p.tiles = static_cast<int32_t>((M + kPwRows - 1) / kPwRows);
        p.col_tiles = static_cast<int32_t>(g.K / kPwCols);
        p.x_unsigned = g.data_t == HIPQ_U8 ? 1 : 0;
        p.per_channel = epi.per_channel;
        p.relu = epi.relu;
        p.out_t = epi.out_t;
        p.sum_t = epi.sum_t;
        const bool has_sum = epi.sum_in != nullptr;
        const size_t lds_bytes = 2 * static_cast<size_t>(kPwRows * g.C) + 4 * (has_sum ? 2 : 1) * kPwStage + 3 * 256 * sizeof(float);
        const int64_t slots = static_cast<int64_t>(device_compute_units()) * 3 / p.col_tiles * p.col_tiles;
        const int64_t items = static_cast<int64_t>(p.tiles) * p.col_tiles;
        const unsigned grid = static_cast<unsigned>(std::min<int64_t>(items, std::max<int64_t>(slots, p.col_tiles)));
        if (g.C == 64)
        {
            if (has_sum)
                conv_pw64_kernel<64, true><<<grid, 256, lds_bytes, s>>>(p);
            else
                conv_pw64_kernel<64, false><<<grid, 256, lds_bytes, s>>>(p);
        }
        else
        {
            if (has_sum)
                conv_pw64_kernel<128, true><<<grid, 256, lds_bytes, s>>>(p);
            else
                conv_pw64_kernel<128, false><<<grid, 256, lds_bytes, s>>>(p);
        }
        return check_launch("conv_pw64_i8_32x32x32");
    }
}
