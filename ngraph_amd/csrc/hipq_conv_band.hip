// Convolution for layers whose whole filter fits in LDS: 64 input channels, at most 64 output
// channels, stride 1, no dilation (the 3x3 and 1x1 64->64 layers of ResNet; BASELINE config 1).
//
// Such layers have so little reduction per output (K*R*S = 576 MACs) that an implicit GEMM which
// re-gathers the input once per filter tap is bound by its loads and address arithmetic, and the
// requantization of an output costs as many VALU cycles as its share of the MFMAs.  Here one
// persistent workgroup per CU (8 wavefronts)
//   * keeps the packed filter resident in LDS for its whole life,
//   * loads a band of the input -- TP output rows plus the halo, every byte once -- into LDS, biased
//     to signed (x ^ 0x80) with the padding materialised,
//   * runs the full reduction out of LDS with no global access and no barrier: per 32-byte step a
//     wavefront reads 2 weight fragments and 4 pixel fragments and issues 8 v_mfma_i32_32x32x32_i8
//     on its 128 pixel x 64 channel tile, and
//   * works as two groups of 4 wavefronts in opposite phase, each with a band buffer of its own:
//     while one group multiplies, the other requantizes its previous band, writes it out and moves
//     its next band (loaded into registers at the start of that phase) into LDS.  Wavefront w of either
//     group sits on SIMD w, so the matrix core of a SIMD works for one group while its VALU works
//     for the other.  The phases are separated by workgroup barriers only.
// The activations feed MFMA source A, so a lane owns one output channel (its scale, bias and
// sign-bias correction are per-lane constants) and four consecutive pixels per accumulator group.
// 8-bit results are staged through LDS so that every global store is a full 16-byte piece of a
// line in either output layout.
#include <cstdlib>
#include <type_traits>

#include "hipq_igemm.h"


namespace hipq
{
    constexpr int kBandC = 64;           // input channels (bytes per pixel slot)
    // Output stores carry the device-scope bit (sc1): written through to the memory side as they are
    // issued instead of sitting dirty in the compute dies' L2s until the write-back that ends the
    // kernel (batch 128, channels-last: 26.1 -> 23.1 us).
    constexpr int kBandStoreScope = 16;
    constexpr int kBandGroupThreads = 256; // a group: four wavefronts, one per SIMD
    constexpr int kBandStagePitch = 144; // NCHW staging: bytes per channel row (128 pixels + pad, 16-byte multiple)
    constexpr int kBandStageWave = 64 * kBandStagePitch; // 9216 bytes per wavefront
    constexpr int kBandBatch = 10;       // 16-byte loads a lane keeps in flight while filling LDS

    struct BandParams
    {
        const uint8_t* x; // [N][H][W][64]
        uint32_t x_bytes;
        uint32_t out_bytes; // size of the output tensor (8-bit outputs: the copy-out uses buffer stores)
        int32_t H, W, P, Q, R, S, pbh, pbw, K;
        int32_t TP;         // output rows per band
        int32_t bands;      // bands per image
        int32_t items;      // N * bands
        int32_t BW;         // slots per band row in LDS: Q + S - 1 rounded up to a multiple of 16, so that
                            // the chunk rotation of a slot does not depend on its row
        int32_t BWr;        // slots per band row that hold data: Q + S - 1
        int32_t q_magic;    // ceil(2^20 / Q): pix / Q = (pix * q_magic) >> 20 for pix < 2048
        int32_t xcd_map;     // renumber workgroups so that each XCD gets a contiguous run of items
        uint32_t bands_magic; // 2^32 / bands + 1: item / bands = hi32(item * bands_magic), exact while items * bands < 2^32 (0: one band)
        int32_t x_lds;      // LDS byte offset of band buffer 0 (the filter sits in front of it)
        int32_t band_bytes; // bytes of one band buffer
        int32_t stage_lds;  // LDS byte offset of the output staging area (one region per wavefront)
        int32_t sink;       // LDS byte offset of 16 spare bytes that absorb the copies' out-of-range lanes
        int64_t PQ;
    };

    // LDS layout of a row of 64-byte cells (the pixel slots of a band row, the 64 filter rows of a
    // tap): two planes of 32-byte half cells, plane h holding the 16-byte chunks 2h and 2h+1 of
    // every cell.  An MFMA fragment read takes chunk 2h + lane/32 of 32 consecutive cells, so both
    // halves of a 64-byte step are one per-lane address plus a constant.  A ds_read_b128 is served
    // 16 lanes at a time from 64 banks: 16 consecutive cells at one chunk index must land in 16
    // different 16-byte columns of a 256-byte line; cells x and x+8 share a column pair, so the
    // chunk within the half cell is flipped by (x / 8) % 2.  (Measured on 64-byte cells: 190
    // B/clk/CU conflict-free against 128 with two-way and 64 with four-way conflicts.)
    __device__ __forceinline__ int band_cell(int x, int chunk, int plane_bytes)
    {
        return (chunk >> 1) * plane_bytes + x * 32 + (((chunk & 1) ^ ((x >> 3) & 1)) << 4);
    }
    constexpr int kTapBytes = 64 * kBandC; // a filter tap in LDS: two planes of 64 x 32 bytes

    // Copies into LDS go in batches: all loads of a batch are issued before any is stored, and
    // issue and store recompute the addresses so that only the data stays in registers between.
    struct BandBatch
    {
        v4i v[kBandBatch];
    };

    // Filter (all 512 lanes): 8 lanes per row n = tid / 8, lane tid % 8 takes every eighth 16-byte
    // chunk of the row; batch element u is chunk tid % 8 + 8 * (u0 + u).  LDS: [tap][plane][64 rows].
    template <bool STORE>
    __device__ __forceinline__ void band_w_copy(BandBatch& b, __amdgpu_buffer_rsrc_t wrs, uint8_t* lds, int u0, int taps, int kred, int K, int sink)
    {
        if (threadIdx.x >= 512) // 64 rows x 8 lanes; a third group has no part in it
            return;
        const int n = static_cast<int>(threadIdx.x) >> 3;
        const int sub = static_cast<int>(threadIdx.x) & 7;
#pragma unroll
        for (int u = 0; u < kBandBatch; ++u)
        {
            const int c = sub + 8 * (u0 + u);
            const bool in = c < taps * 4;
            if (STORE)
                *reinterpret_cast<v4i*>(lds + (in ? (c >> 2) * kTapBytes + band_cell(n, c & 3, kTapBytes / 2) : sink)) = b.v[u];
            else
                b.v[u] = buffer_load16(wrs, (in && n < K) ? n * kred + c * 16 : kOob); // rows beyond K read as zeros
        }
    }

    // Band (the 256 lanes of a group): lane takes chunk cx = cx0 + gtid of a row of BW pixel slots
    // (4 chunks a slot); batch element u < NB is band row sy0 + u.  xs_off: LDS offset of the group's
    // buffer.  A lane's column and a batch element's row are each valid or not on their own (the row
    // uniformly), so an address is the sum of a per-lane and a per-row part, and either part being
    // half of the out-of-range offset puts the sum out of range: one scalar select and one add per
    // load.  (The tensor is at most 2^30 bytes, checked by the launcher.)
    // FILL: padding is a non-zero byte (out-of-range loads give zeros, which is the padding otherwise)
    // PLAIN: the batch is the whole band and every row of it lies inside the image (all bands but an
    // image's first and last): row offsets ride in the scalar offset of the load (which the range
    // check ignores -- the rows are known to be valid), no per-row tests.  PITCH: bytes per band row
    // in LDS when known at compile time (row offsets become immediates), else 0.
    constexpr int kHalfOob = 0x40000000;
    template <bool STORE, bool FILL, int NB, bool PLAIN, int PITCH>
    __device__ __forceinline__ void band_x_copy(BandBatch& b, __amdgpu_buffer_rsrc_t xrs, uint8_t* lds, const BandParams& p, int xs_off, int cx0, int sy0, int band_rows, int img_base, int p0, int fill, int xor_mask)
    {
        const int cx = cx0 + (static_cast<int>(threadIdx.x) & 255);
        const int sx = cx >> 2;
        const int c4 = cx & 3;
        const int ix = sx - p.pbw;
        const bool col_in = sx < p.BWr;
        const bool col_ok = col_in & (static_cast<uint32_t>(ix) < static_cast<uint32_t>(p.W));
        const int pitch = PITCH ? PITCH : p.BW * kBandC;
        if (!STORE)
        {
            const int v_col = col_ok ? img_base + ix * kBandC + c4 * 16 : kHalfOob;
#pragma unroll
            for (int u = 0; u < NB; ++u)
            {
                const int sy = sy0 + u;
                const int iy = p0 + sy - p.pbh;
                if (PLAIN)
                    b.v[u] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(xrs, v_col, iy * p.W * kBandC, 0));
                else
                {
                    const bool row_ok = (sy < band_rows) & (static_cast<uint32_t>(iy) < static_cast<uint32_t>(p.H));
                    const int s_row = row_ok ? iy * p.W * kBandC : kHalfOob;
                    b.v[u] = buffer_load16(xrs, v_col + s_row);
                }
            }
        }
        else if (col_in)
        {
            const int v_cell = xs_off + band_cell(sx, c4, pitch / 2);
#pragma unroll
            for (int u = 0; u < NB; ++u)
            {
                const int sy = sy0 + u;
                if (PLAIN || sy < band_rows) // uniform
                {
                    v4i t = b.v[u];
                    if (FILL)
                    {
                        const int iy = p0 + sy - p.pbh;
                        const bool ok = col_ok & (static_cast<uint32_t>(iy) < static_cast<uint32_t>(p.H));
                        t = v4i{ok ? t[0] : fill, ok ? t[1] : fill, ok ? t[2] : fill, ok ? t[3] : fill};
                    }
                    *reinterpret_cast<v4i*>(lds + v_cell + sy * pitch) = v4i{t[0] ^ xor_mask, t[1] ^ xor_mask, t[2] ^ xor_mask, t[3] ^ xor_mask};
                }
            }
        }
    }

    // Reduction of T pixel tiles x 2 channel tiles over all taps, out of LDS: per 32-byte half of a
    // tap 2 weight fragments, T pixel fragments, 2T MFMAs; no barrier, no global access.  Two
    // fragment sets alternate (statically indexed) so that the reads of one half overlap the MFMAs
    // of the other.  woff: LDS offset of this lane's filter row in plane 0 of tap 0; xrow0 / xcol0:
    // LDS offset of the band row and the slot in it of each tile's pixel (tap 0,0).
    // U taps per loop trip; the tap count must be a multiple of U.
    template <int T, int U>
    __device__ __forceinline__ void band_reduce(v16i (&acc)[T][2], const uint8_t* lds, int woff, const int (&xrow0)[T], const int (&xcol0)[T], int half, int R, int S, int BW)
    {
        const int plane = BW * 32, rowp = BW * kBandC;
        v4i xa[T], xb[T], wa[2], wb[2];
        int xoff[T], xnext[T];
        auto addr = [&](int r, int sx, int(&xo)[T]) {
#pragma unroll
            for (int ti = 0; ti < T; ++ti)
                xo[ti] = xrow0[ti] + r * rowp + band_cell(xcol0[ti] + sx, half, 0);
        };
        auto load = [&](int wp, const int(&xo)[T], int h, v4i(&xf)[T], v4i(&wf)[2]) {
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
                wf[ni] = *reinterpret_cast<const v4i*>(lds + wp + h * (kTapBytes / 2) + ni * 32 * 32);
#pragma unroll
            for (int ti = 0; ti < T; ++ti)
                xf[ti] = *reinterpret_cast<const v4i*>(lds + xo[ti] + h * plane);
        };
        auto mac = [&](const v4i(&xf)[T], const v4i(&wf)[2]) {
#pragma unroll
            for (int ti = 0; ti < T; ++ti)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    acc[ti][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[ti], wf[ni], acc[ti][ni], 0, 0, 0);
        };
        // One wavefront issues in order: an MFMA occupies the matrix core for 32 cycles and anything
        // issued behind it runs in its shadow, but 2T MFMAs back to back leave no shadow for the
        // reads and address arithmetic of the next half.  Ask for MFMA, LDS read, a few VALU, MFMA, ...
        auto interleave = [&]() {
#pragma unroll
            for (int i = 0; i < 2 * T; ++i)
            {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // DS read
                __builtin_amdgcn_sched_group_barrier(0x002, 3, 0); // VALU
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        // The pipeline, per tap: while half 0 multiplies, half 1 is read and the next tap's LDS
        // offsets are computed; while half 1 multiplies, the next tap's half 0 is read.
        addr(0, 0, xoff);
        load(woff, xoff, 0, xa, wa);
        __builtin_amdgcn_sched_barrier(0);
        int wp = woff;
        int r = 0, sx = 0;
        const int taps = R * S;
#pragma unroll 1
        for (int tap = 0; tap < taps; tap += U)
        {
#pragma unroll
            for (int u = 0; u < U; ++u)
            {
                load(wp, xoff, 1, xb, wb);
                // the next tap; after the last one this wraps to tap 0, a harmless re-read that
                // keeps the loop free of conditional loads
                wp += kTapBytes;
                ++sx;
                if (sx == S)
                {
                    sx = 0;
                    ++r;
                }
                if (r == R)
                {
                    r = 0;
                    wp = woff;
                }
                addr(r, sx, xnext);
                mac(xa, wa);
                interleave();
#pragma unroll
                for (int ti = 0; ti < T; ++ti)
                    xoff[ti] = xnext[ti];
                load(wp, xoff, 0, xa, wa);
                mac(xb, wb);
                interleave();
            }
        }
    }

    // The same reduction for a 3x3 filter over band rows of 64 slots: every LDS address is a
    // per-lane base (one per pixel tile and filter column, computed once per band) plus a
    // compile-time offset (filter row, half, tap, channel tile), so the 144 MFMAs and 108 reads run
    // as straight-line code without address arithmetic, loop branches or register shuffles.
    template <int T, bool ADD_CORR>
    __device__ __forceinline__ void band_reduce_33(v16i (&acc)[T][2], const uint8_t* lds, int woff, const int (&xrow0)[T], const int (&xcol0)[T], int half, const int32_t (&corr)[2])
    {
        constexpr int kRow = 64 * kBandC; // bytes of a band row of 64 slots (two planes of 2048)
        int xbase[T][3];
#pragma unroll
        for (int ti = 0; ti < T; ++ti)
#pragma unroll
            for (int sx = 0; sx < 3; ++sx)
                xbase[ti][sx] = xrow0[ti] + band_cell(xcol0[ti] + sx, half, 0);
        v4i xa[T], xb[T], wa[2], wb[2];
        auto load = [&](int k, v4i(&xf)[T], v4i(&wf)[2]) {
            const int tap = k >> 1, h = k & 1, r = tap / 3, sx = tap % 3;
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
                wf[ni] = *reinterpret_cast<const v4i*>(lds + woff + tap * kTapBytes + h * (kTapBytes / 2) + ni * 32 * 32);
#pragma unroll
            for (int ti = 0; ti < T; ++ti)
                xf[ti] = *reinterpret_cast<const v4i*>(lds + xbase[ti][sx] + r * kRow + h * (kRow / 2));
        };
        // the first step starts the accumulators from the constant 0 (no initialisation moves; tuples
        // preloaded with the correction made the register allocator spill); the sign-bias correction
        // is added after the last MFMA, still in the multiply phase, which is the shorter one
        auto mac = [&](const v4i(&xf)[T], const v4i(&wf)[2], bool first) {
            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int ti = 0; ti < T; ++ti)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    acc[ti][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[ti], wf[ni], first ? zero : acc[ti][ni], 0, 0, 0);
        };
        auto interleave = [&]() {
#pragma unroll
            for (int i = 0; i < 2 * T; ++i)
            {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // DS read
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        load(0, xa, wa);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < 18; k += 2)
        {
            load(k + 1, xb, wb);
            mac(xa, wa, k == 0);
            interleave();
            if (k + 2 < 18)
                load(k + 2, xa, wa);
            mac(xb, wb, false);
            interleave();
        }
        if (ADD_CORR)
        {
#pragma unroll
            for (int ti = 0; ti < T; ++ti)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        acc[ti][ni][r] += corr[ni];
        }
    }

    // U: filter taps per trip of the reduction loop (the tap count is a multiple of it); 0: the
    // straight-line 3x3 reduction over 64-slot band rows
    // T: 32-pixel tiles per wavefront (4: items of up to 512 pixels; 2: items of up to 256 pixels,
    // which fill and drain the two-group pipeline in half the time and split a layer more evenly)
    // G: groups of four wavefronts.  Two groups alternate between multiplying and requantizing; three
    // groups (two-tile items only: the registers allow three wavefronts a SIMD) rotate through
    // multiply / requantize first half / requantize second half, which keeps a third wavefront on
    // every SIMD to fill the gaps the other two leave.
    template <int MODE, int KIND, bool OUT_NCX, int U, int T, int G>
    __global__ __launch_bounds__(kBandGroupThreads * G) void conv_band_kernel(BandParams p,
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
        // wavefront-uniform values, told so to the compiler: item geometry and loop control then run
        // on the scalar unit instead of in vector registers under exec masks
        const int wave_id = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int grp = wave_id >> 2; // group of four wavefronts
        const int gw = wave_id & 3;   // wavefront within the group (= its SIMD)
        const int half = lane >> 5;
        const int l32 = lane & 31;
        const int xs_off = p.x_lds + grp * p.band_bytes;

        // ---- small loads first: they must not queue behind the bulk loads ------------------------
        const int32_t xzp = load_zp(zp.data_zp, zp.data_t);
        const int32_t wzp = load_zp(zp.filter_zp, zp.filter_t);
        const EpiConst ec = epi_const(epi);
        const bool has_sum = MODE == EPI_FUSED && epi.sum_in != nullptr;
        int32_t wsum_n[2];
        float bias[2], scale[2]; // a lane owns channels lane%32 and 32 + lane%32
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
        {
            const int n = ni * 32 + l32;
            const bool ok = n < p.K;
            wsum_n[ni] = ok ? wsum[n] : 0;
            bias[ni] = (MODE == EPI_FUSED && epi.bias && ok) ? static_cast<float>(epi.bias[n]) : 0.0f;
            scale[ni] = (MODE == EPI_FUSED && epi.per_channel && ok) ? epi.scale[n] : ec.scale;
        }

        const int taps = p.R * p.S;
        const int kred = taps * kBandC;
        const __amdgpu_buffer_rsrc_t xrs = make_rsrc(p.x, p.x_bytes);
        const __amdgpu_buffer_rsrc_t wrs = make_rsrc(w, static_cast<uint32_t>(p.K) * static_cast<uint32_t>(kred));
        const int grid = static_cast<int>(gridDim.x);
        // this workgroup's items are blockIdx.x + j * grid, j = 0 .. my_items-1; item j belongs to
        // group j % 2, is reduced in phase j and requantized in phase j + 1
        // Workgroups are dealt round-robin to the 8 XCDs, each with an L2 of its own: workgroup b works as
        // number vb, which gives every XCD a contiguous run of items in each round, so that the halo
        // rows neighbouring bands share are fetched into one L2 (grids that are not a multiple of 8 keep
        // the plain numbering).
        const int vb = ((grid & 7) == 0 && p.xcd_map) ? (static_cast<int>(blockIdx.x) & 7) * (grid >> 3) + (static_cast<int>(blockIdx.x) >> 3) : static_cast<int>(blockIdx.x);
        const int my_items = (p.items - vb + grid - 1) / grid;

        auto item_geom = [&](int j, int& img, int& p0, int& rows) {
            const int item = vb + j * grid;
            img = p.bands_magic ? static_cast<int>(__umulhi(static_cast<uint32_t>(item), p.bands_magic)) : item;
            p0 = (item - img * p.bands) * p.TP;
            rows = min(p.TP, p.P - p0);
        };

        // ---- the filter and each group's first band ---------------------------------------------
        // Both groups fetch their first band together with the filter: group 1 multiplies one phase
        // later, but a fetch started then would not be back before group 0 is done.
        BandBatch wb0, xb0;
        int img, p0, rows;
        band_w_copy<false>(wb0, wrs, lds, 0, taps, kred, p.K, p.sink);
        if (grp < my_items)
        {
            item_geom(grp, img, p0, rows);
            band_x_copy<false, false, (T == 2 ? 6 : kBandBatch), false, 0>(xb0, xrs, lds, p, xs_off, 0, 0, rows + p.R - 1, img * p.H * p.W * kBandC, p0, 0, 0);
        }

        if (wzp != 0) // uniform; w - wzp does not fit a signed byte: exact, slow, one output a lane
        {
            const EpiRegs er = epi_load(epi);
            for (int j = 0; j < my_items; ++j)
            {
                item_geom(j, img, p0, rows);
                for (int i = tid; i < rows * p.Q * p.K; i += kBandGroupThreads * G)
                {
                    const int n = i % p.K, pix = i / p.K;
                    const int py = p0 + pix / p.Q, px = pix % p.Q;
                    int32_t a = 0;
                    for (int r = 0; r < p.R; ++r)
                        for (int sx = 0; sx < p.S; ++sx)
                        {
                            const int iy = py + r - p.pbh, ix = px + sx - p.pbw;
                            if (static_cast<uint32_t>(iy) >= static_cast<uint32_t>(p.H) || static_cast<uint32_t>(ix) >= static_cast<uint32_t>(p.W))
                                continue; // padding is the data zero point: contributes nothing
                            const uint8_t* xp = p.x + (static_cast<int64_t>(img) * p.H * p.W + iy * p.W + ix) * kBandC;
                            const int8_t* wp = w + static_cast<int64_t>(n) * kred + (r * p.S + sx) * kBandC;
                            for (int c = 0; c < kBandC; ++c)
                            {
                                const int32_t xv = x_unsigned ? static_cast<int32_t>(xp[c]) : static_cast<int32_t>(static_cast<int8_t>(xp[c]));
                                a += (xv - xzp) * (static_cast<int32_t>(wp[c]) - wzp);
                            }
                        }
                    const int64_t gp = static_cast<int64_t>(img) * p.PQ + static_cast<int64_t>(p0) * p.Q + pix;
                    const int64_t o = OUT_NCX ? (static_cast<int64_t>(img) * p.K + n) * p.PQ + static_cast<int64_t>(p0) * p.Q + pix : gp * p.K + n;
                    store_out(out, epi.out_t, o, epi_apply(epi, er, a, n, o));
                }
            }
            return;
        }
        const int xor_mask = x_unsigned ? static_cast<int>(0x80808080u) : 0;
        const int fill = (xzp & 0xFF) * 0x01010101;
        const int32_t mult = (x_unsigned ? 128 : 0) - xzp;
        const int32_t corr[2] = {mult * wsum_n[0], mult * wsum_n[1]};
        // INTERPRETER requantization in fixed point needs |acc * scale| * 256 < 2^31
        const float acc_max = static_cast<float>(kred) * (255.0f * 128.0f);
        const bool fast_interp = fabsf(ec.scale) * acc_max < 4194304.0f;

        // moves a band into the group's buffer; the first batch is already in xb0
        // rows of a band a lane fetches in one go: the bands of two-tile items are short
        constexpr int NB = T == 2 ? 6 : kBandBatch;
        constexpr int PITCH = U == 0 ? 64 * kBandC : 0; // the straight-line kernel runs on 64-slot band rows
        // every row of item j's band inside the image, and the band exactly one batch: no per-row tests
        auto band_plain = [&]() { return p.BWr * 4 <= 256 && rows + p.R - 1 == NB && p0 >= p.pbh && p0 - p.pbh + NB <= p.H; };
        auto band_fetch = [&](BandBatch& xb, int j) {
            item_geom(j, img, p0, rows);
            if (band_plain())
                band_x_copy<false, false, NB, true, PITCH>(xb, xrs, lds, p, xs_off, 0, 0, NB, img * p.H * p.W * kBandC, p0, 0, 0);
            else
                band_x_copy<false, false, NB, false, PITCH>(xb, xrs, lds, p, xs_off, 0, 0, rows + p.R - 1, img * p.H * p.W * kBandC, p0, 0, 0);
        };
        auto band_store = [&](BandBatch& xb0, int j) {
            item_geom(j, img, p0, rows);
            const int band_rows = rows + p.R - 1;
            const int img_base = img * p.H * p.W * kBandC;
            if (fill == 0 && band_plain())
            {
                band_x_copy<true, false, NB, true, PITCH>(xb0, xrs, lds, p, xs_off, 0, 0, NB, img_base, p0, fill, xor_mask);
                return;
            }
            if (fill == 0)
                band_x_copy<true, false, NB, false, PITCH>(xb0, xrs, lds, p, xs_off, 0, 0, band_rows, img_base, p0, fill, xor_mask);
            else
                band_x_copy<true, true, NB, false, PITCH>(xb0, xrs, lds, p, xs_off, 0, 0, band_rows, img_base, p0, fill, xor_mask);
            if (p.BWr * 4 > 256 || band_rows > NB) // wide or tall bands: the rest, batch by batch
                for (int cx0 = 0; cx0 < p.BWr * 4; cx0 += 256)
                    for (int sy0 = 0; sy0 < band_rows; sy0 += NB)
                        if (cx0 | sy0)
                        {
                            band_x_copy<false, false, NB, false, PITCH>(xb0, xrs, lds, p, xs_off, cx0, sy0, band_rows, img_base, p0, fill, xor_mask);
                            band_x_copy<true, true, NB, false, PITCH>(xb0, xrs, lds, p, xs_off, cx0, sy0, band_rows, img_base, p0, fill, xor_mask);
                        }
        };

        for (int u0 = 0; u0 * 8 < taps * 4; u0 += kBandBatch)
        {
            if (u0)
                band_w_copy<false>(wb0, wrs, lds, u0, taps, kred, p.K, p.sink);
            band_w_copy<true>(wb0, wrs, lds, u0, taps, kred, p.K, p.sink);
        }
        // group 0's first band is awaited here; the later groups move theirs into LDS just before the
        // barrier that precedes their first multiply phase, so that the first phase does not wait for them
        if (grp == 0 && 0 < my_items)
            band_store(xb0, 0);
        __syncthreads();

        // Phase p multiplies item p and requantizes item p - 1; item j belongs to group j % 2.  Both
        // groups run the same multiply / barrier / requantize / barrier loop over their own items,
        // group 1 one barrier behind group 0, and whichever finishes first keeps arriving at the
        // barrier until my_items + 1 phases have passed.  The accumulators never cross a loop trip.
        int phases_done = 0;
        for (; phases_done < grp; ++phases_done)
        {
            if (phases_done == grp - 1 && grp < my_items)
                band_store(xb0, grp);
            __syncthreads();
        }
        // staging holds a whole wavefront tile (two groups) or half of one (three groups: LDS is short)
        constexpr bool kStageHalf = G == 3;
        constexpr int kStagePitch = kStageHalf ? 16 * T + 16 : kBandStagePitch;
        constexpr int kStageWave = kStageHalf ? 64 * kStagePitch : kBandStageWave;
        // Three groups: the group's next band is fetched at the start of its second phase and enters the
        // band buffer at the end of its third (nobody reads the buffer in between, and two phases
        // cover the round trip to memory); the multiply phase carries no fetch registers.
        constexpr bool kCarryFetch = G == 3;
        // three groups: the multiply phase is the long one, the sign-bias correction moves to the requantization
        constexpr bool kCorrLate = G == 3 && U == 0;
        BandBatch nb;
        for (int sp = grp; sp < my_items; sp += G)
        {
            v16i acc[T][2];
            // The group's next band travels through registers: fetched during this multiply phase,
            // moved into the band buffer in the requantize phase that follows (when nobody reads the
            // buffer).  With two tiles a wavefront the registers are free from the start of the
            // phase and the data is back before the barrier; with four the fetch starts once the
            // fragment registers are free and is awaited at the end of the requantize phase.
            constexpr bool kEarlyFetch = T == 2;
            if (kEarlyFetch && !kCarryFetch && sp + G < my_items)
                band_fetch(nb, sp + G);
            {
                // ================= multiply: item sp =================
                // The SIMD's arbiter favours its older wavefront; without a hint group 1 starves in
                // either role.  The multiply phase has few, long instructions: it gets priority and the
                // requantizing wavefront fills the gaps.
                __builtin_amdgcn_s_setprio(3);
                {
                    item_geom(sp, img, p0, rows);
                    const int npix = rows * p.Q;
                    const int ntiles = (npix + 31) >> 5;
                    // wavefront gw owns tiles T*gw .. T*gw+T-1
                    if (U != 0) // the straight-line reduction brings the correction in with its first MFMAs
                    {
#pragma unroll
                        for (int ti = 0; ti < T; ++ti)
#pragma unroll
                            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                                for (int r = 0; r < 16; ++r)
                                    acc[ti][ni][r] = corr[ni];
                    }
                    if (T * gw < ntiles)
                    {
                        int xrow0[T], xcol0[T];
#pragma unroll
                        for (int ti = 0; ti < T; ++ti)
                        {
                            // tiles past the end re-read the last pixel; their results are never stored
                            const int pix = min((T * gw + ti) * 32 + l32, npix - 1);
                            const int py = (pix * p.q_magic) >> 20;
                            xrow0[ti] = xs_off + py * (p.BW * kBandC);
                            xcol0[ti] = pix - py * p.Q;
                        }
                        const int woff = band_cell(l32, half, 0);
                        if (U == 0)
                            band_reduce_33<T, !kCorrLate>(acc, lds, woff, xrow0, xcol0, half, corr);
                        else
                            band_reduce<T, U == 0 ? 1 : U>(acc, lds, woff, xrow0, xcol0, half, p.R, p.S, p.BW);
                    }
                }
            }
            __builtin_amdgcn_s_setprio(0);
            if (!kEarlyFetch && sp + G < my_items)
                band_fetch(nb, sp + G);
            __syncthreads();
            ++phases_done;
            {
                // ================= requantize and write out: item sp =================
                // per-lane indices are recomputed from an opaque copy of the lane id: hoisted out of the
                // item loop they would occupy registers through the multiply phase and spill
                int lane_v = lane;
                asm volatile("" : "+v"(lane_v));
                const int half = lane_v >> 5;
                const int l32 = lane_v & 31;
                uint8_t* const stage = lds + p.stage_lds + (G == 3 ? wave_id : gw) * kStageWave;
                item_geom(sp, img, p0, rows);
                const int npix = rows * p.Q;
                // lane: channel ni*32 + lane%32; accumulator register 4g+e of tile ti is pixel
                // (4*gw + ti)*32 + 8g + 4*(lane/32) + e of the band
                const int64_t img_pix0 = static_cast<int64_t>(img) * p.PQ + static_cast<int64_t>(p0) * p.Q; // first pixel of the band, image-major
                if (kEarlyFetch && !kCarryFetch && sp + G < my_items)
                    band_store(nb, sp + G);
                if (kCarryFetch && sp + G < my_items)
                    band_fetch(nb, sp + G);
                if (kEarlyFetch)
                    item_geom(sp, img, p0, rows);

                auto epilogue = [&](auto fast_c, auto sum_c, auto ti0_c, auto ti1_c) {
                    constexpr int ti0 = decltype(ti0_c)::value, ti1 = decltype(ti1_c)::value;
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
                        for (int ti = ti0; ti < ti1; ++ti)
                        {
#pragma unroll
                            for (int g = 0; g < 4; ++g)
                            {
                                const int lpix = ti * 32 + 8 * g + 4 * half; // pixel within the wavefront's 32 * T
                                const int bpix = gw * (32 * T) + lpix;      // pixel within the band
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
                                    const int32_t a = acc[ti][ni][4 * g + e] + (kCorrLate ? corr[ni] : 0);
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
                                        *reinterpret_cast<uint32_t*>(stage + n * kStagePitch + lpix - (kStageHalf ? ti0 * 32 : 0)) = (hi2 << 16) | lo2;
                                    }
                                    else
                                    {
#pragma unroll
                                        for (int e = 0; e < 4; ++e)
                                            stage[(lpix - (kStageHalf ? ti0 * 32 : 0) + e) * 64 + n] = static_cast<uint8_t>(BYTE ? (x[e] >> 8) : x[e]);
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
                auto requantize = [&](auto ti0, auto ti1) {
                    if (MODE == EPI_FUSED)
                    {
                        if (has_sum)
                            epilogue(true_type{}, true_type{}, ti0, ti1);
                        else
                            epilogue(true_type{}, false_type{}, ti0, ti1);
                    }
                    else if (KIND == OUT_Q8 && fast_interp)
                        epilogue(true_type{}, false_type{}, ti0, ti1);
                    else
                        epilogue(false_type{}, false_type{}, ti0, ti1);
                };
                // Staging regions are wavefront-private and a wavefront's LDS accesses complete in order:
                // no barrier.  Lanes with nothing to store get an out-of-range offset, which the buffer
                // store drops: no branches.  The tile is written out in two halves of 16 * T pixels; the
                // staging reads of the first half are in flight while the second half is requantized.
                const __amdgpu_buffer_rsrc_t ors = make_rsrc(out, p.out_bytes);
                v4i piece[T];
                auto stage_read = [&](int h) {
#pragma unroll
                    for (int j = 0; j < T; ++j)
                    {
                        const int id = j * 64 + lane_v;
                        if (OUT_NCX) // 64 channel rows: a lane moves 16 consecutive pixels of one channel
                            piece[j] = *reinterpret_cast<const v4i*>(stage + (id / T) * kStagePitch + ((kStageHalf ? 0 : h * T) + id % T) * 16);
                        else // 16 * T pixel rows of 64 channels: a lane moves 16 consecutive channels of one pixel
                            piece[j] = *reinterpret_cast<const v4i*>(stage + ((kStageHalf ? 0 : 16 * T * h) + (id >> 2)) * 64 + (id & 3) * 16);
                    }
                };
                auto stage_write_out = [&](int h) {
#pragma unroll
                    for (int j = 0; j < T; ++j)
                    {
                        const int id = j * 64 + lane_v;
                        if (OUT_NCX)
                        {
                            // bands and images hold multiples of 16 pixels (checked by the launcher)
                            const int ch = id / T;
                            const int part = h * T + id % T;
                            const int band0 = (img * p.K) * static_cast<int>(p.PQ) + p0 * p.Q + gw * (32 * T);
                            const bool ok = (ch < p.K) & (gw * (32 * T) + part * 16 < npix);
                            __builtin_amdgcn_raw_buffer_store_b128(piece[j], ors, ok ? band0 + ch * static_cast<int>(p.PQ) + part * 16 : kOob, 0, kBandStoreScope);
                        }
                        else
                        {
                            const int px = 16 * T * h + (id >> 2);
                            const int part = id & 3;
                            const int band0 = (img * static_cast<int>(p.PQ) + p0 * p.Q + gw * (32 * T)) * p.K;
                            const bool ok = (gw * (32 * T) + px < npix) & (part * 16 < p.K);
                            __builtin_amdgcn_raw_buffer_store_b128(piece[j], ors, ok ? band0 + px * p.K + part * 16 : kOob, 0, kBandStoreScope);
                        }
                    }
                };
                if (KIND == OUT_Q8)
                {
                    requantize(std::integral_constant<int, 0>{}, std::integral_constant<int, T / 2>{});
                    __builtin_amdgcn_sched_barrier(0);
                    stage_read(0);
                    __builtin_amdgcn_sched_barrier(0);
                    if (G == 3) // the second half of the tile is the group's third phase
                    {
                        __syncthreads();
                        ++phases_done;
                    }
                    if (kStageHalf) // the first half leaves the staging area before the second half enters
                    {
                        stage_write_out(0);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    requantize(std::integral_constant<int, T / 2>{}, std::integral_constant<int, T>{});
                    __builtin_amdgcn_sched_barrier(0);
                    if (!kStageHalf)
                        stage_write_out(0);
                    stage_read(1);
                    __builtin_amdgcn_sched_barrier(0);
                    stage_write_out(1);
                }
                else
                {
                    requantize(std::integral_constant<int, 0>{}, std::integral_constant<int, T / 2>{});
                    if (G == 3)
                    {
                        __syncthreads();
                        ++phases_done;
                    }
                    requantize(std::integral_constant<int, T / 2>{}, std::integral_constant<int, T>{});
                }
                if (!kEarlyFetch && sp + G < my_items)
                    band_store(nb, sp + G);
                if (kCarryFetch && sp + G < my_items)
                    band_store(nb, sp + G);
            }
            __syncthreads();
            ++phases_done;
        }
        for (; phases_done < my_items + G - 1; ++phases_done)
        {
            __syncthreads();
        }
    }

    // rows per band and LDS bytes; false when the layer does not fit this kernel
    static bool band_plan(const ConvGeom& g, bool out_ncx, int tiles, int groups, BandParams* bp, size_t* lds_bytes)
    {
        const int64_t stage_wave = groups == 3 ? 64 * (16 * tiles + 16) : kBandStageWave;
        // two groups: only one requantizes at a time, a region per SIMD; three: two do, a region per wavefront
        const int64_t stage_regions = groups == 3 ? 12 : 4;
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
        if (g.in_count() > (1ll << 30) || g.out_count() >= (1ll << 31) || g.N * P >= (1ll << 30))
            return false;
        const int64_t wbytes = R * S * 64 * kBandC; // [tap][64][64]
        const int64_t BWr = Q + S - 1;
        const int64_t BW = (BWr + 15) / 16 * 16;
        const int64_t budget = 160 * 1024; // one workgroup per CU: filter, two band buffers, staging
        int64_t best = 0;
        for (int64_t tp = 1; tp <= P && tp * Q <= 4 * 32 * tiles; ++tp)
        {
            const int64_t band_bytes = (tp + R - 1) * BW * kBandC;
            const int64_t need = wbytes + groups * band_bytes + stage_regions * stage_wave + 16;
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
        bp->BWr = static_cast<int32_t>(BWr);
        bp->q_magic = static_cast<int32_t>(((1 << 20) + Q - 1) / Q);
        bp->bands_magic = bp->bands > 1 ? static_cast<uint32_t>((1ull << 32) / static_cast<uint64_t>(bp->bands) + 1) : 0u;
        if (static_cast<int64_t>(bp->items) * bp->bands >= (1ll << 32))
            return false;
        bp->xcd_map = tiles == 2 ? 1 : 0; // short bands share more halo rows; measured neutral to harmful for tall ones
        bp->x_lds = static_cast<int32_t>(wbytes);
        bp->band_bytes = static_cast<int32_t>(band_bytes);
        bp->stage_lds = static_cast<int32_t>(wbytes + groups * band_bytes);
        bp->sink = bp->stage_lds + static_cast<int32_t>(stage_regions * stage_wave);
        bp->PQ = P * Q;
        bp->x_bytes = static_cast<uint32_t>(g.in_count());
        bp->out_bytes = static_cast<uint32_t>(g.out_count() * static_cast<int64_t>(dtype_size(g.out_t)));
        *lds_bytes = static_cast<size_t>(bp->sink) + 16;
        return true;
    }

    bool conv_band_eligible(const ConvGeom& g, bool out_ncx)
    {
        BandParams bp;
        size_t lds_bytes;
        return band_plan(g, out_ncx, 4, 2, &bp, &lds_bytes);
    }

    static int band_slots()
    {
        static int cus[16] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16)
            return 256;
        if (cus[dev] == 0)
        {
            hipDeviceProp_t prop;
            cus[dev] = hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        }
        return cus[dev]; // one persistent workgroup per CU
    }

    template <int MODE, int KIND, bool OUT_NCX, int U, int T, int G>
    static int launch_band(const BandParams& bp, size_t lds_bytes, const int8_t* w, const int32_t* wsum, int xu, const ZeroPoints& zp, const Epilogue& epi, void* out, hipStream_t s)
    {
        auto kernel = conv_band_kernel<MODE, KIND, OUT_NCX, U, T, G>;
        static bool configured[16] = {};
        int dev = 0;
        HIPQ_HIP(hipGetDevice(&dev));
        if (dev >= 0 && dev < 16 && !configured[dev])
        {
            HIPQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            configured[dev] = true;
        }
        const int slots = band_slots();
        const unsigned grid = static_cast<unsigned>(bp.items < slots ? bp.items : slots);
        kernel<<<grid, kBandGroupThreads * G, lds_bytes, s>>>(bp, w, wsum, xu, zp, epi, out);
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
        HIPQ_REQUIRE(band_plan(g, out_ncx, 4, 2, &bp, &lds_bytes), "layer does not fit the band convolution");
        // Items of half the size (two tiles a wavefront) for the straight-line 3x3 kernel when that is
        // estimated faster: time ~ (phases + fill and drain) x tiles, a phase being one item per group
        // and the small items paying about a tenth more per pixel (filter fragments reused half as often)
        int tiles = 4;
        {
            BandParams b2;
            size_t l2 = 0;
            const char* force = getenv("HIPQ_BAND_TILES");
            if (bp.R == 3 && bp.S == 3 && bp.BW == 64 && getenv("HIPQ_BAND_LOOP") == nullptr && band_plan(g, out_ncx, 2, 3, &b2, &l2))
            {
                const int slots = band_slots();
                auto cost = [slots](const BandParams& b, double fill, double per_phase) {
                    const int grid = b.items < slots ? b.items : slots;
                    return ((b.items + grid - 1) / grid + fill) * per_phase;
                };
                // measured: a phase of the three-group kernel takes about 0.4 of a four-tile phase
                const bool small = force ? atoi(force) == 2 : cost(b2, 3.0, 0.4) < cost(bp, 1.6, 1.0);
                if (small)
                {
                    bp = b2;
                    lds_bytes = l2;
                    tiles = 2;
                }
            }
        }
        HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(data_nxc) & 15) == 0 && (reinterpret_cast<uintptr_t>(packed) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(out) & 15) == 0,
                     "band convolution needs 16-byte aligned tensors");
        bp.x = static_cast<const uint8_t*>(data_nxc);
        const int kred = bp.R * bp.S * kBandC;
        const int8_t* w = static_cast<const int8_t*>(packed);
        const int32_t* wsum = reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(packed) + align_up(static_cast<size_t>(g.K) * kred, 256));
        const int xu = g.data_t == HIPQ_U8 ? 1 : 0;
        const bool q8 = g.out_t == HIPQ_U8 || g.out_t == HIPQ_I8;
        // straight-line reduction for 3x3 filters over 64-slot band rows, else a loop of 3 or 1 taps a trip
        const int u = (bp.R == 3 && bp.S == 3 && bp.BW == 64 && getenv("HIPQ_BAND_LOOP") == nullptr) ? 0 : ((bp.R * bp.S) % 3 == 0 ? 3 : 1);
#define BAND_U(MODE, KIND, NCX)                                                                    \
    (u == 0 ? (tiles == 2 ? launch_band<MODE, KIND, NCX, 0, 2, 3>(bp, lds_bytes, w, wsum, xu, zp, epi, out, s)                   \
                          : launch_band<MODE, KIND, NCX, 0, 4, 2>(bp, lds_bytes, w, wsum, xu, zp, epi, out, s))                  \
            : (u == 3 ? launch_band<MODE, KIND, NCX, 3, 4, 2>(bp, lds_bytes, w, wsum, xu, zp, epi, out, s)                       \
                      : launch_band<MODE, KIND, NCX, 1, 4, 2>(bp, lds_bytes, w, wsum, xu, zp, epi, out, s)))
#define BAND(MODE, KIND) (out_ncx ? BAND_U(MODE, KIND, true) : BAND_U(MODE, KIND, false))
        if (epi.mode == EPI_INTERP)
            return q8 ? BAND(EPI_INTERP, OUT_Q8) : BAND(EPI_INTERP, OUT_I32);
        if (q8)
            return BAND(EPI_FUSED, OUT_Q8);
#undef BAND
#undef BAND_U
        return fail(HIPQ_ERR_UNSUPPORTED, "no band kernel for this epilogue / output type");
    }
}
