// 3x3 convolution over 64 input channels with the whole filter in registers (BASELINE config 1:
// u8 [N,64,56,56] x i8 [64,64,3,3], stride 1, pad 1; ResNet's 64 -> 64 layers).
//
// The layer has 576 multiply-accumulates per output: too few to amortise a filter that is re-read
// from LDS for every pixel tile, and its requantization costs a wavefront as many issue slots as
// its matrix instructions.  Here
//   * every wavefront keeps the packed filter (64 x 576 bytes) in 144 registers for its whole life
//     as the B fragments of v_mfma_i32_32x32x32_i8, so a 32-pixel x 64-channel tile costs 18 LDS
//     reads (the pixel fragments) for 36 MFMAs;
//   * a workgroup (8 wavefronts, two a SIMD, 256 registers each) owns a band of output rows of one
//     image.  Four wavefronts (one a SIMD) start as loaders: they read the input band (rows + halo)
//     from memory exactly once, in the tensor's own layout, with four rounds of loads in flight from
//     the first cycle on -- NCHW rows are transposed to channels-last 16-byte pieces in registers
//     with v_perm_b32 on the way, so the reference's layout needs no separate transposition pass --
//     bias the bytes to signed (x ^ 0x80) and lay them into LDS with the padding materialised, four
//     band rows a round, each round announced through an LDS counter;
//   * the other four wavefronts multiply from the start: they draw tile numbers from an LDS counter,
//     wait only for the rounds their tile needs, and overlap the MFMAs of one tile with the
//     requantization and the stores of the previous one in a single instruction stream (two
//     accumulator sets).  A loader that has delivered its last round joins them;
//   * tiles are runs of 32 consecutive pixels of the band (rows of 56 pixels leave no padding
//     slots in a tile); a lane owns one output channel, requantizes its 16 pixels of a tile in
//     registers, gathers 16 consecutive pixels of its channel with v_permlane32_swap_b32 and stores
//     them as one 16-byte piece of an NCHW row.
#include <cstdlib>

#include "hipq_igemm.h"


namespace hipq
{
    constexpr int kRwThreads = 512;
    constexpr int kRwRoundRows = 4; // band rows per load round
    // (measured at batch 128: two loaders 21.3 us, four 20.6; 2 / 4 / 8 rounds in flight 20.35 / 20.1 / 21.3 us --
    // a deeper queue delays the first rounds, which the multiplying wavefronts are waiting for)
    constexpr int kRwLoaders = 4;               // wavefronts that start as loaders (the last ones of the workgroup)
    constexpr int kRwGroups = 4 / kRwLoaders;   // 16-channel groups (NCHW) or piece quarters (NHWC) a loader brings per round
    constexpr int kRwMulThreads = (8 - kRwLoaders) * 64; // lanes of the wavefronts that multiply from the start
    constexpr int kRwMaxRounds = 24;
    constexpr int kRwDepth = 4;     // rounds of loads a loader keeps in flight
    constexpr int kRwAhead = 3;     // pixel fragments on their way from LDS while a tile multiplies and the previous one requantizes
    constexpr int kRwKred = 576;    // 9 taps x 64 channels
    // Output stores carry the device-scope bit (sc1): they are written through to the memory side as
    // they are issued.  Each compute die has an L2 of its own, and what a kernel leaves dirty there is
    // written back when it ends, behind the last wavefront; this kernel's 25 MB of output would
    // otherwise mostly still sit in the L2s at that point (batch 128: 23.4 -> 21.9 us).
    constexpr int kRwStoreScope = 16;

    struct RegwParams
    {
        const uint8_t* x;
        uint32_t x_bytes;
        uint32_t out_bytes;
        int32_t H, W, K;
        int32_t TP;          // output rows per band (divides H)
        int32_t bands;       // bands per image
        int32_t items;       // N * bands
        int32_t pitch;       // bytes of a band row in one plane: (W + 2) * 32 + 16
        int32_t plane_bytes; // bytes of a plane; = 128 mod 256 so that the two planes use different banks
        int32_t flags_lds;   // LDS offset of the round counters (kRwMaxRounds), the tile counter and the slow-path flag
        uint32_t bands_magic; // 2^32 / bands + 1 (0: one band an image)
        FastDiv div_w;
    };

    // LDS: two planes (channels 0..31, 32..63); a plane row holds W + 2 half cells of 32 bytes (slot 0
    // and slot W + 1 are the horizontal padding); the two 16-byte chunks of a half cell are flipped
    // where (slot / 8) is odd, which spreads 16 consecutive slots over all 64 banks.
    __device__ __forceinline__ int regw_cell(int slot, int chunk) { return slot * 32 + (((chunk ^ (slot >> 3)) & 1) << 4); }

    // bytes of one LDS plane for a band of `rows` output rows of a layer `w` pixels wide
    // (= 128 mod 256, so that the two planes use different banks)
    __host__ __device__ constexpr int regw_plane_bytes(int w, int rows) { return ((rows + 2) * ((w + 2) * 32 + 16) + 255) / 256 * 256 + 128; }
    constexpr int kRwMaxRowsCT = 28; // band rows the compile-time geometry leaves room for (56-wide layers: 2 x 56448 + 36864 bytes)

    struct RegwRaw
    {
        int v[16];
    };

    template <int MODE, bool IN_NCX, bool SUM, int WCT>
    __global__ __launch_bounds__(kRwThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv_regw_kernel(RegwParams p,
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
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int half = lane >> 5;
        const int l32 = lane & 31;
        // WCT != 0: a layer WCT pixels wide with the LDS geometry fixed at compile time, so that every
        // fragment address is a per-lane base plus an immediate offset (no address arithmetic between
        // the MFMAs); WCT == 0: any width, geometry from the parameters
        const int W_ = WCT ? WCT : p.W;
        const int pitch = WCT ? (WCT + 2) * 32 + 16 : p.pitch;
        const int plane = WCT ? regw_plane_bytes(WCT, kRwMaxRowsCT) : p.plane_bytes;
        auto div_w = [&](int v) { return WCT ? static_cast<int>(static_cast<uint32_t>(v) / static_cast<uint32_t>(WCT ? WCT : 1)) : static_cast<int>(p.div_w.div(static_cast<uint32_t>(v))); };

        // ---- which band ----------------------------------------------------------------------------
        // workgroups are dealt round-robin to the 8 XCDs (an L2 each): renumbered so that the bands of
        // an image, which share halo rows, meet in one L2
        const int grid = static_cast<int>(gridDim.x);
        const int item = (grid & 7) == 0 ? (static_cast<int>(blockIdx.x) & 7) * (grid >> 3) + (static_cast<int>(blockIdx.x) >> 3) : static_cast<int>(blockIdx.x);
        const int img = p.bands_magic ? static_cast<int>(__umulhi(static_cast<uint32_t>(item), p.bands_magic)) : item;
        const int h0 = (item - img * p.bands) * p.TP;
        const int rows = p.TP;
        const int band_rows = rows + 2;
        const int npix = rows * W_;
        const int PQ = p.H * W_;

        const __amdgpu_buffer_rsrc_t xrs = make_rsrc(p.x, p.x_bytes);
        const __amdgpu_buffer_rsrc_t ors = make_rsrc(out, p.out_bytes);
        const bool loader = wave >= 8 - kRwLoaders; // uniform
        const int lw0 = (wave - (8 - kRwLoaders)) * kRwGroups; // first group of this loader
        const int nrounds = (band_rows + kRwRoundRows - 1) / kRwRoundRows;
        const int ntiles = (npix + 31) >> 5;
        const int xor_mask = x_unsigned ? static_cast<int>(0x80808080u) : 0;
        uint32_t* const flags = reinterpret_cast<uint32_t*>(lds + p.flags_lds);
        uint32_t* const tile_ctr = flags + kRwMaxRounds;
        uint32_t* const slow_flag = flags + kRwMaxRounds + 1;
        uint8_t* const wlds = lds + p.flags_lds + (kRwMaxRounds + 8) * 4;

        // ---- the band loader -----------------------------------------------------------------------
        // A round is four band rows.  NCHW: loader wavefront lw takes channels 16 lw .. 16 lw + 15; a
        // lane takes 4 consecutive pixels of one row for those channels (16 dword loads, each covering
        // four whole rows = 4 W contiguous bytes a wavefront), transposes four 4x4 byte blocks with
        // v_perm_b32 and writes four 16-byte pieces (one pixel, 16 channels each).  The pixel a lane
        // writes at step e is rotated by lane / 4, which spreads the 16 lanes of an LDS write over all
        // banks; the rotation rides in the selectors of the first permutation stage.
        // NHWC: a lane takes four 16-byte pieces (pixel, channel quarter) as they lie in memory.
        const int n4 = W_ >> 2; // 4-pixel groups a row (NCHW)
        const int rot = (lane >> 2) & 3;
        uint32_t sel_lo, sel_hi;
        {
            const uint32_t r0 = rot, r1 = (rot + 1) & 3, r2 = (rot + 2) & 3, r3 = (rot + 3) & 3;
            sel_lo = r0 | ((4 + r0) << 8) | (r1 << 16) | ((4 + r1) << 24);
            sel_hi = r2 | ((4 + r2) << 8) | (r3 << 16) | ((4 + r3) << 24);
        }
        auto issue = [&](RegwRaw& raw, int k, int lw) {
            if (IN_NCX)
            {
                const int j = lane & 15;
                const int r = k * kRwRoundRows + (lane >> 4);
                const int y = h0 - 1 + r;
                const bool ok = (j < n4) & (r < band_rows) & (static_cast<uint32_t>(y) < static_cast<uint32_t>(p.H));
                const int base = ok ? ((img * 64 + lw * 16) * p.H + y) * W_ + 4 * j : kOob;
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    raw.v[i] = __builtin_amdgcn_raw_buffer_load_b32(xrs, base, i * PQ, 0);
            }
            else
            {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    const int id = i * 256 + lw * 64 + lane;
                    const int pl = id >> 2, c4 = id & 3;
                    const int rr = div_w(pl);
                    const int col = pl - rr * W_;
                    const int r = k * kRwRoundRows + rr;
                    const int y = h0 - 1 + r;
                    const bool ok = (rr < kRwRoundRows) & (r < band_rows) & (static_cast<uint32_t>(y) < static_cast<uint32_t>(p.H));
                    const v4i t = buffer_load16(xrs, ok ? ((img * p.H + y) * W_ + col) * 64 + c4 * 16 : kOob);
                    raw.v[4 * i] = t[0];
                    raw.v[4 * i + 1] = t[1];
                    raw.v[4 * i + 2] = t[2];
                    raw.v[4 * i + 3] = t[3];
                }
            }
        };
        auto commit = [&](const RegwRaw& raw, int k, int lw) {
            if (IN_NCX)
            {
                const int j = lane & 15;
                const int r = k * kRwRoundRows + (lane >> 4);
                const int y = h0 - 1 + r;
                const bool ok = (j < n4) & (r < band_rows) & (static_cast<uint32_t>(y) < static_cast<uint32_t>(p.H));
                int o[4][4]; // [channel quad][step]: bytes = channels 4m..4m+3 of pixel (step + rot) % 4
#pragma unroll
                for (int m = 0; m < 4; ++m)
                {
                    const uint32_t a = raw.v[4 * m], b = raw.v[4 * m + 1], c = raw.v[4 * m + 2], d = raw.v[4 * m + 3];
                    const uint32_t t_lo = __builtin_amdgcn_perm(b, a, sel_lo), t_hi = __builtin_amdgcn_perm(b, a, sel_hi);
                    const uint32_t u_lo = __builtin_amdgcn_perm(d, c, sel_lo), u_hi = __builtin_amdgcn_perm(d, c, sel_hi);
                    o[m][0] = static_cast<int>(__builtin_amdgcn_perm(u_lo, t_lo, 0x05040100u)) ^ xor_mask;
                    o[m][1] = static_cast<int>(__builtin_amdgcn_perm(u_lo, t_lo, 0x07060302u)) ^ xor_mask;
                    o[m][2] = static_cast<int>(__builtin_amdgcn_perm(u_hi, t_hi, 0x05040100u)) ^ xor_mask;
                    o[m][3] = static_cast<int>(__builtin_amdgcn_perm(u_hi, t_hi, 0x07060302u)) ^ xor_mask;
                }
                if (ok)
                {
                    uint8_t* const row = lds + (lw >> 1) * plane + r * pitch;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                    {
                        const int slot = 4 * j + ((e + rot) & 3) + 1;
                        *reinterpret_cast<v4i*>(row + regw_cell(slot, lw & 1)) = v4i{o[0][e], o[1][e], o[2][e], o[3][e]};
                    }
                }
            }
            else
            {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    const int id = i * 256 + lw * 64 + lane;
                    const int pl = id >> 2, c4 = id & 3;
                    const int rr = div_w(pl);
                    const int col = pl - rr * W_;
                    const int r = k * kRwRoundRows + rr;
                    const int y = h0 - 1 + r;
                    const bool ok = (rr < kRwRoundRows) & (r < band_rows) & (static_cast<uint32_t>(y) < static_cast<uint32_t>(p.H));
                    if (ok)
                        *reinterpret_cast<v4i*>(lds + (c4 >> 1) * plane + r * pitch + regw_cell(col + 1, c4 & 1)) =
                            v4i{raw.v[4 * i] ^ xor_mask, raw.v[4 * i + 1] ^ xor_mask, raw.v[4 * i + 2] ^ xor_mask, raw.v[4 * i + 3] ^ xor_mask};
                }
            }
        };

        // ---- start-up ---------------------------------------------------------------------------------
        // loaders: the first rounds of the band are asked for before anything else, and nothing the
        // loaders do before the barrier waits for memory.  The others: filter into LDS (fragment order),
        // scalars, the constant parts of the band (horizontal padding, rows outside the image).
        RegwRaw raw[kRwDepth][kRwGroups];
        int32_t xzp = 0, wzp = 0;
        if (loader)
        {
#pragma unroll
            for (int d = 0; d < kRwDepth; ++d)
                if (d < nrounds)
#pragma unroll
                    for (int g = 0; g < kRwGroups; ++g)
                        issue(raw[d][g], d, lw0 + g);
        }
        // what the requantization needs from memory is asked for now, behind the band (loaders) or
        // ahead of the filter (the others), and used long after it has arrived
        const EpiConst ec = epi_const(epi);
        int32_t wsum_n[2];
        float bias[2], scale[2]; // a lane owns channels lane % 32 and 32 + lane % 32
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
        {
            const int n = ni * 32 + l32;
            const bool ok = n < p.K;
            wsum_n[ni] = ok ? wsum[n] : 0;
            bias[ni] = (MODE == EPI_FUSED && epi.bias && ok) ? static_cast<float>(epi.bias[n]) : 0.0f;
            scale[ni] = (MODE == EPI_FUSED && epi.per_channel && ok) ? epi.scale[n] : ec.scale;
        }
        if (!loader)
        {
            constexpr int kFilterPieces = 64 * kRwKred / 16; // 2304 16-byte pieces
            constexpr int kFilterLoads = kFilterPieces / kRwMulThreads;
            static_assert(kFilterPieces % kRwMulThreads == 0, "filter pieces divide over the wavefronts that fetch them");
            v4i fpiece[kFilterLoads];
            const __amdgpu_buffer_rsrc_t wrs = make_rsrc(w, static_cast<uint32_t>(p.K) * kRwKred);
#pragma unroll
            for (int i = 0; i < kFilterLoads; ++i)
                fpiece[i] = buffer_load16(wrs, (i * kRwMulThreads + tid) * 16); // rows beyond K read as zeros
            xzp = load_zp(zp.data_zp, zp.data_t);
            wzp = load_zp(zp.filter_zp, zp.filter_t);
            if (tid < kRwMaxRounds + 2)
                flags[tid] = (tid == kRwMaxRounds + 1 && wzp != 0) ? 1u : 0u; // round counters, tile counter, slow-path flag
            const int fill = ((xzp & 0xFF) * 0x01010101) ^ xor_mask;
            const v4i f4 = {fill, fill, fill, fill};
            // slots 0 and W + 1 of every row: 2 planes x 2 slots x 2 chunks pieces a row
            for (int i = tid; i < band_rows * 8; i += kRwMulThreads)
            {
                const int r = i >> 3, pl = (i >> 2) & 1, sl = (i & 2) ? W_ + 1 : 0, c = i & 1;
                *reinterpret_cast<v4i*>(lds + pl * plane + r * pitch + regw_cell(sl, c)) = f4;
            }
            const int per_row = (W_ + 2) * 4; // pieces of a whole row in both planes
            if (h0 == 0)
                for (int i = tid; i < per_row; i += kRwMulThreads)
                    *reinterpret_cast<v4i*>(lds + (i & 1) * plane + regw_cell(i >> 2, (i >> 1) & 1)) = f4;
            if (h0 + rows == p.H)
                for (int i = tid; i < per_row; i += kRwMulThreads)
                    *reinterpret_cast<v4i*>(lds + (i & 1) * plane + (band_rows - 1) * pitch + regw_cell(i >> 2, (i >> 1) & 1)) = f4;
            // the filter in fragment order: piece ((ks * 2 + ni) * 64 + lane) is what `lane` feeds the MFMAs
            // of step ks, channel tile ni: row ni * 32 + lane % 32, bytes ks * 32 + 16 * (lane / 32) ...
#pragma unroll
            for (int i = 0; i < kFilterLoads; ++i)
            {
                const int g = i * kRwMulThreads + tid;
                const int n = g / 36, r = g - n * 36; // 36 pieces a filter row
                const int ks = r >> 1, hf = r & 1;
                *reinterpret_cast<v4i*>(wlds + (((ks * 2 + (n >> 5)) * 2 + hf) * 32 + (n & 31)) * 16) = fpiece[i];
            }
        }
        __syncthreads();

        if (*reinterpret_cast<volatile uint32_t*>(slow_flag) != 0) // uniform; w - wzp does not fit a signed byte: exact, slow, one output a lane
        {
            xzp = load_zp(zp.data_zp, zp.data_t);
            wzp = load_zp(zp.filter_zp, zp.filter_t);
            const EpiRegs er = epi_load(epi);
            for (int i = tid; i < npix * p.K; i += kRwThreads)
            {
                const int n = i / npix, pix = i - n * npix;
                const int py = h0 + div_w(pix);
                const int px = pix - (py - h0) * W_;
                int32_t a = 0;
                for (int r = 0; r < 3; ++r)
                    for (int sx = 0; sx < 3; ++sx)
                    {
                        const int iy = py + r - 1, ix = px + sx - 1;
                        if (static_cast<uint32_t>(iy) >= static_cast<uint32_t>(p.H) || static_cast<uint32_t>(ix) >= static_cast<uint32_t>(W_))
                            continue; // padding is the data zero point: contributes nothing
                        const int8_t* wp = w + n * kRwKred + (r * 3 + sx) * 64;
                        for (int c = 0; c < 64; ++c)
                        {
                            const int64_t xi = IN_NCX ? (static_cast<int64_t>(img) * 64 + c) * PQ + iy * W_ + ix : (static_cast<int64_t>(img) * PQ + iy * W_ + ix) * 64 + c;
                            const int32_t xv = x_unsigned ? static_cast<int32_t>(p.x[xi]) : static_cast<int32_t>(static_cast<int8_t>(p.x[xi]));
                            a += (xv - xzp) * (static_cast<int32_t>(wp[c]) - wzp);
                        }
                    }
                const int64_t o = (static_cast<int64_t>(img) * p.K + n) * PQ + h0 * W_ + pix;
                store_out(out, epi.out_t, o, epi_apply(epi, er, a, n, o));
            }
            return;
        }

        // ---- loaders: every round into LDS, kRwDepth rounds of loads in flight -----------------------
        if (loader)
        {
            for (int base = 0; base < nrounds; base += kRwDepth)
            {
#pragma unroll
                for (int d = 0; d < kRwDepth; ++d)
                {
                    const int k = base + d;
                    if (k < nrounds) // uniform
                    {
#pragma unroll
                        for (int g = 0; g < kRwGroups; ++g)
                            commit(raw[d][g], k, lw0 + g);
                        // this wavefront's share of round k is in LDS: count it in (a round is complete at 4)
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        if (lane == 0)
                            __hip_atomic_fetch_add(flags + k, static_cast<uint32_t>(kRwGroups), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        if (k + kRwDepth < nrounds)
#pragma unroll
                            for (int g = 0; g < kRwGroups; ++g)
                                issue(raw[d][g], k + kRwDepth, lw0 + g);
                    }
                }
            }
            xzp = load_zp(zp.data_zp, zp.data_t);
        }

        // ---- everyone multiplies from here on ---------------------------------------------------------
        const int32_t mult = (x_unsigned ? 128 : 0) - xzp;
        const int32_t corr[2] = {mult * wsum_n[0], mult * wsum_n[1]};
        // INTERPRETER requantization in fixed point needs |acc * scale| * 256 < 2^31
        const bool fast_interp = fabsf(ec.scale) * (static_cast<float>(kRwKred) * (255.0f * 128.0f)) < 4194304.0f;
        const float s256 = __fmul_rn(ec.scale, 256.0f);
        const int32_t c256 = 128 + 256 * ec.ozp;
        const float lo = fmaxf(ec.lo, ec.relu_floor);
        v4i wf[18][2];
#pragma unroll
        for (int ks = 0; ks < 18; ++ks)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
                wf[ks][ni] = *reinterpret_cast<const v4i*>(wlds + ((ks * 2 + ni) * 64 + lane) * 16);

        // next tile of the band, dealt out by an LDS counter
        auto grab = [&]() {
            uint32_t v = 0;
            if (lane == 0)
                v = __hip_atomic_fetch_add(tile_ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            return __builtin_amdgcn_readfirstlane(static_cast<int>(v));
        };
        int ready = 0; // rounds 0 .. ready-1 are known to be complete
        auto await_rows = [&](int t) {
            // the tile's last pixel is in band-relative output row ro_max and needs band rows up to ro_max + 2
            const int last = min(t * 32 + 31, npix - 1);
            const int ro_max = div_w(last);
            const int need = min((ro_max + 3 + kRwRoundRows - 1) / kRwRoundRows, nrounds);
            while (ready < need)
            {
                while (__builtin_amdgcn_readfirstlane(static_cast<int>(__hip_atomic_load(flags + ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP))) < 4)
                    __builtin_amdgcn_s_sleep(1);
                ++ready;
            }
            asm volatile("" ::: "memory");
        };

        // the multiply half of a tile: 36 MFMAs over 18 pixel fragments
        auto tile_mfma = [&](int t, v16i (&acc)[2]) {
            // tiles past the end re-read the last pixel; their results are never stored
            const int pix = min(t * 32 + l32, npix - 1);
            const int ro = div_w(pix);
            const int col = pix - ro * W_;
            int xb[3];
#pragma unroll
            for (int sx = 0; sx < 3; ++sx)
                xb[sx] = ro * pitch + regw_cell(col + sx, half);
            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            auto frag = [&](int ks) {
                const int tap = ks >> 1, h = ks & 1, r = tap / 3, sx = tap % 3;
                return *reinterpret_cast<const v4i*>(lds + xb[sx] + r * pitch + h * plane);
            };
            constexpr int kAhead = 6; // no requantization in this stream: registers to spare
            v4i xf[kAhead + 1];
#pragma unroll
            for (int i = 0; i < kAhead; ++i)
                xf[i] = frag(i);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < 18; ++ks)
            {
                if (ks + kAhead < 18)
                    xf[(ks + kAhead) % (kAhead + 1)] = frag(ks + kAhead);
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    acc[ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[ks % (kAhead + 1)], wf[ks][ni], ks == 0 ? zero : acc[ni], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // the other half: requantize and store.  Accumulator register 4g + e is pixel 32t + 8g + 4 * (lane / 32) + e,
        // channel ni * 32 + lane % 32.  FAST: the INTERPRETER policy in fixed point (a compile-time choice: a
        // uniform branch per output would cost more than the arithmetic)
        auto tile_store = [&](int t, const v16i (&acc)[2], auto fast_c) {
            constexpr bool FAST = decltype(fast_c)::value;
            const int gpix0 = h0 * W_ + t * 32; // first pixel of the tile within the image
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
            {
                const int n = ni * 32 + l32;
                uint32_t d[4];
#pragma unroll
                for (int g = 0; g < 4; ++g)
                {
                    float s4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                    if (SUM)
                    {
                        const int lp = t * 32 + 8 * g + 4 * half;
                        if (n < p.K && lp < npix)
                            sum4(epi.sum_in, epi.sum_t, (static_cast<int64_t>(img) * p.K + n) * PQ + gpix0 + 8 * g + 4 * half, true, s4);
                    }
                    int32_t x[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                    {
                        const int32_t a = acc[ni][4 * g + e] + corr[ni];
                        if (MODE == EPI_INTERP && FAST)
                        {
                            // t = trunc(256 v); round-half-away(v) = (t + 128 - (t < 0)) >> 8, exactly
                            const int32_t tt = static_cast<int32_t>(__fmul_rn(static_cast<float>(a), s256));
                            x[e] = tt + (tt >> 31) + c256;
                        }
                        else if (MODE == EPI_INTERP)
                            x[e] = epi_interp<OUT_Q8>(ec, a);
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
                    constexpr uint32_t sel = (MODE == EPI_INTERP && FAST) ? 0x0c0c0501u : 0x0c0c0400u;
                    const uint32_t lo2 = __builtin_amdgcn_perm(x[1], x[0], sel);
                    const uint32_t hi2 = __builtin_amdgcn_perm(x[3], x[2], sel);
                    d[g] = (hi2 << 16) | lo2;
                }
                // the lower half of the wavefront holds pixels 8g .. 8g+3, the upper 8g+4 .. 8g+7: after the
                // two swaps a lane holds 16 consecutive pixels of its channel (lower: 0..15, upper: 16..31)
                const auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
                const auto s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
                const v4i piece = {static_cast<int>(s02[0]), static_cast<int>(s02[1]), static_cast<int>(s13[0]), static_cast<int>(s13[1])};
                const bool ok = (n < p.K) & (t * 32 + 16 * half < npix);
                __builtin_amdgcn_raw_buffer_store_b128(piece, ors, ok ? (img * p.K + n) * PQ + gpix0 + 16 * half : kOob, 0, kRwStoreScope);
            }
        };
        // One instruction stream for the MFMAs of tile t and the requantization of tile tp: an MFMA
        // occupies the matrix core for 32 cycles and what is issued behind it runs in its shadow.  The
        // order is written out -- behind each of the 36 MFMAs the requantization of one output of the
        // previous tile (six VALU instructions), the pack of four, the gather and the store of sixteen
        // -- and fenced step by step, because the scheduler, short of registers, would otherwise put
        // all MFMAs first.
        auto tile_both = [&](int t, v16i (&acc)[2], int tp, const v16i (&accp)[2], auto fast_c) {
            constexpr bool FAST = decltype(fast_c)::value;
            const int pix = min(t * 32 + l32, npix - 1);
            const int ro = div_w(pix);
            const int col = pix - ro * W_;
            int xb[3];
#pragma unroll
            for (int sx = 0; sx < 3; ++sx)
                xb[sx] = ro * pitch + regw_cell(col + sx, half);
            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const int gpix0 = h0 * W_ + tp * 32; // first pixel of the previous tile within the image
            auto frag = [&](int ks) {
                const int tap = ks >> 1, h = ks & 1, r = tap / 3, sx = tap % 3;
                return *reinterpret_cast<const v4i*>(lds + xb[sx] + r * pitch + h * plane);
            };
            int32_t x[4];
            uint32_t d[4];
            float s4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            // slot s of 36: output (ni, g, e) = (s / 16, (s / 4) % 4, s % 4) of the previous tile
            // slot sl of 36 (one behind every MFMA): stage sl % 4 of the four outputs (ni, g) = (sl / 16,
            // (sl / 4) % 4) of the previous tile.  The four outputs of a group go through each stage
            // together, so an instruction's input is four instructions old instead of one: a wavefront
            // that shares its SIMD issues dependent arithmetic a third slower than independent.
            auto requant = [&](int sl) {
                if (sl >= 32)
                    return;
                const int ni = sl >> 4, g = (sl >> 2) & 3, stage = sl & 3;
                const int n = ni * 32 + l32;
                if (stage == 0)
                {
                    if (SUM)
                    {
                        const int lp = tp * 32 + 8 * g + 4 * half;
                        s4[0] = s4[1] = s4[2] = s4[3] = 0.0f;
                        if (n < p.K && lp < npix)
                            sum4(epi.sum_in, epi.sum_t, (static_cast<int64_t>(img) * p.K + n) * PQ + gpix0 + 8 * g + 4 * half, true, s4);
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        x[e] = accp[ni][4 * g + e] + corr[ni];
                    if (MODE == EPI_FUSED || FAST)
                    {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            x[e] = __float_as_int(static_cast<float>(x[e]));
                    }
                }
                else if (stage == 1)
                {
                    if (MODE == EPI_INTERP && FAST)
                    {
                        // t = trunc(256 v); round-half-away(v) = (t + 128 - (t < 0)) >> 8, exactly
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            x[e] = __float_as_int(__fmul_rn(__int_as_float(x[e]), s256));
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            x[e] = static_cast<int32_t>(__int_as_float(x[e]));
                    }
                    else if (MODE == EPI_FUSED)
                    {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            x[e] = __float_as_int(__fadd_rn(__int_as_float(x[e]), bias[ni]));
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            x[e] = __float_as_int(__fmul_rn(__int_as_float(x[e]), scale[ni]));
                    }
                }
                else if (stage == 2)
                {
                    if (MODE == EPI_INTERP && FAST)
                    {
                        int32_t sg[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            sg[e] = x[e] >> 31;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            x[e] = x[e] + sg[e] + c256;
                    }
                    else if (MODE == EPI_INTERP)
                    {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            x[e] = epi_interp<OUT_Q8>(ec, x[e]);
                    }
                    else
                    {
                        if (SUM)
                        {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                x[e] = __float_as_int(fmaf(ec.sum_scale, s4[e], __int_as_float(x[e])));
                        }
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            x[e] = __float_as_int(__builtin_amdgcn_fmed3f(__int_as_float(x[e]), lo, ec.hi));
                        // 1.5 * 2^23 + v rounds half-to-even into the low mantissa bits
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            x[e] = __float_as_int(__fadd_rn(__int_as_float(x[e]), 12582912.0f));
                    }
                }
                else
                {
                    constexpr uint32_t sel = (MODE == EPI_INTERP && FAST) ? 0x0c0c0501u : 0x0c0c0400u;
                    const uint32_t lo2 = __builtin_amdgcn_perm(x[1], x[0], sel);
                    const uint32_t hi2 = __builtin_amdgcn_perm(x[3], x[2], sel);
                    d[g] = (hi2 << 16) | lo2;
                    if (g == 3)
                    {
                        // the lower half of the wavefront holds pixels 8g .. 8g+3, the upper 8g+4 .. 8g+7: after the
                        // two swaps a lane holds 16 consecutive pixels of its channel (lower: 0..15, upper: 16..31)
                        const auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
                        const auto s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
                        const v4i piece = {static_cast<int>(s02[0]), static_cast<int>(s02[1]), static_cast<int>(s13[0]), static_cast<int>(s13[1])};
                        const bool ok = (n < p.K) & (tp * 32 + 16 * half < npix);
                        __builtin_amdgcn_raw_buffer_store_b128(piece, ors, ok ? (img * p.K + n) * PQ + gpix0 + 16 * half : kOob, 0, kRwStoreScope);
                    }
                }
            };
            // an LDS read takes about three MFMA pairs to come back: kRwAhead fragments are on their way
            v4i xf[kRwAhead + 1];
#pragma unroll
            for (int i = 0; i < kRwAhead; ++i)
                xf[i] = frag(i);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < 18; ++ks)
            {
                if (ks + kRwAhead < 18)
                    xf[(ks + kRwAhead) % (kRwAhead + 1)] = frag(ks + kRwAhead);
                acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[ks % (kRwAhead + 1)], wf[ks][0], ks == 0 ? zero : acc[0], 0, 0, 0);
                requant(2 * ks);
                __builtin_amdgcn_sched_barrier(0);
                acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[ks % (kRwAhead + 1)], wf[ks][1], ks == 0 ? zero : acc[1], 0, 0, 0);
                requant(2 * ks + 1);
                __builtin_amdgcn_sched_barrier(0);
            }
        };

        auto run = [&](auto fast_c) {
            v16i acc_a[2], acc_b[2];
            int ta = grab();
            if (ta >= ntiles)
                return;
            await_rows(ta);
            tile_mfma(ta, acc_a);
            if (SUM) // the residual's loads and conversions leave no registers for a second accumulator set
            {
                for (;;)
                {
                    tile_store(ta, acc_a, fast_c);
                    ta = grab();
                    if (ta >= ntiles)
                        break;
                    await_rows(ta);
                    tile_mfma(ta, acc_a);
                }
                return;
            }
            for (;;)
            {
                const int tb = grab();
                if (tb >= ntiles)
                {
                    tile_store(ta, acc_a, fast_c);
                    break;
                }
                await_rows(tb);
                tile_both(tb, acc_b, ta, acc_a, fast_c);
                ta = grab();
                if (ta >= ntiles)
                {
                    tile_store(tb, acc_b, fast_c);
                    break;
                }
                await_rows(ta);
                tile_both(ta, acc_a, tb, acc_b, fast_c);
            }
        };
        if (MODE == EPI_INTERP && fast_interp) // uniform
            run(std::true_type{});
        else
            run(std::false_type{});
    }

    // rows per band and LDS bytes; false when the layer is not of this kernel's kind
    static bool regw_plan(const ConvGeom& g, bool out_ncx, int slots, RegwParams* rp, size_t* lds_bytes)
    {
        if (g.in[0] != 1 || g.f[0] != 1 || g.out[0] != 1)
            return false;
        if (!out_ncx) // channels-last outputs stay with the band kernel
            return false;
        if (g.C != 64 || g.K > 64 || g.K % 16 != 0 || g.f[1] != 3 || g.f[2] != 3)
            return false;
        for (int i = 0; i < 3; ++i)
            if (g.st[i] != 1 || g.dl[i] != 1 || g.dd[i] != 1)
                return false;
        if (g.pb[1] != 1 || g.pb[2] != 1 || g.out[1] != g.in[1] || g.out[2] != g.in[2])
            return false;
        if (g.filter_t != HIPQ_I8 || (g.data_t != HIPQ_U8 && g.data_t != HIPQ_I8) || (g.out_t != HIPQ_U8 && g.out_t != HIPQ_I8))
            return false;
        const int64_t H = g.in[1], W = g.in[2];
        if (W % 4 != 0 || W > 64 || W < 4 || g.in_count() >= (1ll << 31) || g.out_count() >= (1ll << 31))
            return false;
        const int64_t pitch = (W + 2) * 32 + 16;
        // a band: TP divides H, bands start on 16-pixel boundaries of the image (the 16-byte output pieces)
        int64_t best = 0;
        double best_cost = 0;
        for (int64_t tp = 1; tp <= H; ++tp)
        {
            if (H % tp != 0 || (tp * W) % 16 != 0)
                continue;
            const int64_t plane = (W == 56 && tp <= kRwMaxRowsCT) ? regw_plane_bytes(56, kRwMaxRowsCT) : ((tp + 2) * pitch + 255) / 256 * 256 + 128;
            if (2 * plane + (kRwMaxRounds + 8) * 4 + 64 * kRwKred > 160 * 1024 || (tp + 2 + kRwRoundRows - 1) / kRwRoundRows > kRwMaxRounds)
                break;
            const int64_t items = g.N * (H / tp);
            // rounds of workgroups x (rows of a band + what a band costs to start and to drain)
            const double cost = static_cast<double>((items + slots - 1) / slots) * static_cast<double>(tp + 3);
            if (best == 0 || cost < best_cost)
            {
                best = tp;
                best_cost = cost;
            }
        }
        if (best == 0)
            return false;
        rp->H = static_cast<int32_t>(H);
        rp->W = static_cast<int32_t>(W);
        rp->K = static_cast<int32_t>(g.K);
        rp->TP = static_cast<int32_t>(best);
        rp->bands = static_cast<int32_t>(H / best);
        rp->items = static_cast<int32_t>(g.N * rp->bands);
        rp->pitch = static_cast<int32_t>(pitch);
        rp->plane_bytes = static_cast<int32_t>((W == 56 && best <= kRwMaxRowsCT) ? regw_plane_bytes(56, kRwMaxRowsCT) : ((best + 2) * pitch + 255) / 256 * 256 + 128);
        rp->flags_lds = 2 * rp->plane_bytes;
        rp->bands_magic = rp->bands > 1 ? static_cast<uint32_t>((1ull << 32) / static_cast<uint64_t>(rp->bands) + 1) : 0u;
        if (static_cast<int64_t>(rp->items) * rp->bands >= (1ll << 32))
            return false;
        rp->div_w = fast_div(W);
        rp->x_bytes = static_cast<uint32_t>(g.in_count());
        rp->out_bytes = static_cast<uint32_t>(g.out_count());
        *lds_bytes = static_cast<size_t>(rp->flags_lds) + (kRwMaxRounds + 8) * 4 + 64 * kRwKred; // band planes, chunk counters, the filter on its way into registers
        return true;
    }

    bool conv_regw_eligible(const ConvGeom& g, bool out_ncx)
    {
        RegwParams rp;
        size_t lds_bytes;
        return getenv("HIPQ_NO_REGW") == nullptr && regw_plan(g, out_ncx, 256, &rp, &lds_bytes);
    }

    template <int MODE, bool IN_NCX, bool SUM, int WCT>
    static int launch_regw(const RegwParams& rp, size_t lds_bytes, const int8_t* w, const int32_t* wsum, int xu, const ZeroPoints& zp, const Epilogue& epi, void* out, hipStream_t s)
    {
        auto kernel = conv_regw_kernel<MODE, IN_NCX, SUM, WCT>;
        static bool configured[16] = {};
        int dev = 0;
        HIPQ_HIP(hipGetDevice(&dev));
        if (dev >= 0 && dev < 16 && !configured[dev])
        {
            HIPQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            configured[dev] = true;
        }
        kernel<<<static_cast<unsigned>(rp.items), kRwThreads, lds_bytes, s>>>(rp, w, wsum, xu, zp, epi, out);
        return check_launch("conv_regw_i8_32x32x32");
    }

    int launch_conv_regw(const ConvGeom& g, const void* data, const void* packed, const ZeroPoints& zp, const Epilogue& epi, void* out, bool out_ncx, hipStream_t s)
    {
        RegwParams rp;
        size_t lds_bytes = 0;
        HIPQ_REQUIRE(regw_plan(g, out_ncx, device_compute_units(), &rp, &lds_bytes), "layer does not fit the filter-in-registers convolution");
        HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(data) & 15) == 0 && (reinterpret_cast<uintptr_t>(packed) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0,
                     "convolution needs 16-byte aligned tensors");
        rp.x = static_cast<const uint8_t*>(data);
        const int8_t* w = static_cast<const int8_t*>(packed);
        const int32_t* wsum = reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(packed) + align_up(static_cast<size_t>(g.K) * kRwKred, 256));
        const int xu = g.data_t == HIPQ_U8 ? 1 : 0;
        const bool in_ncx = g.data_layout == HIPQ_LAYOUT_NCX;
        const bool sum = epi.mode == EPI_FUSED && epi.sum_in != nullptr;
        HIPQ_REQUIRE(!sum || (reinterpret_cast<uintptr_t>(epi.sum_in) & 3) == 0, "sum input must be 4-byte aligned");
        // 56-wide layers (ResNet's first stage, config 1) with the compile-time LDS geometry
        const bool w56 = rp.W == 56 && rp.TP <= kRwMaxRowsCT && rp.plane_bytes == regw_plane_bytes(56, kRwMaxRowsCT) && getenv("HIPQ_REGW_NO_CT") == nullptr;
#define REGW_W(MODE, IN, SUM) (w56 ? launch_regw<MODE, IN, SUM, 56>(rp, lds_bytes, w, wsum, xu, zp, epi, out, s) : launch_regw<MODE, IN, SUM, 0>(rp, lds_bytes, w, wsum, xu, zp, epi, out, s))
#define REGW(MODE, SUM) (in_ncx ? REGW_W(MODE, true, SUM) : REGW_W(MODE, false, SUM))
        if (epi.mode == EPI_INTERP)
            return REGW(EPI_INTERP, false);
        return sum ? REGW(EPI_FUSED, true) : REGW(EPI_FUSED, false);
#undef REGW
#undef REGW_W
    }
}
