// MaxPool / AvgPool / Concat: the integer glue between the quantized convolutions of a network.
// One output element per lane; channels-last tensors put consecutive lanes on consecutive
// channels of a pixel, NCHW tensors on consecutive pixels of a row -- coalesced either way.
#include <cmath>
#include <cstdlib>
#include <limits>

#include "hipq_common.h"

namespace hipq
{
    struct PoolGeom
    {
        int64_t N, C;
        int64_t in[3], win[3], st[3], pb[3], out[3];
        int32_t nxc;
        int32_t include_padding;
        int64_t count;
    };

    template <typename T, bool AVG>
    __global__ __launch_bounds__(256) void pool_kernel(PoolGeom g, const T* __restrict__ in, T* __restrict__ out)
    {
        const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
        if (i >= g.count)
            return;
        // flat output index -> (n, c, o0, o1, o2) in the tensor's layout
        int64_t n, c, o[3];
        int64_t t = i;
        if (g.nxc)
        {
            c = t % g.C;
            t /= g.C;
        }
        o[2] = t % g.out[2];
        t /= g.out[2];
        o[1] = t % g.out[1];
        t /= g.out[1];
        o[0] = t % g.out[0];
        t /= g.out[0];
        if (!g.nxc)
        {
            c = t % g.C;
            t /= g.C;
        }
        n = t;
        const int64_t in_sp = g.in[0] * g.in[1] * g.in[2];
        // src/ngraph/runtime/reference/max_pool.hpp:209 : lowest(); avg_pool.hpp:216 : T result = 0
        T best = std::numeric_limits<T>::lowest();
        T sum = 0;
        int64_t cnt = 0;
        for (int64_t w0 = 0; w0 < g.win[0]; ++w0)
            for (int64_t w1 = 0; w1 < g.win[1]; ++w1)
                for (int64_t w2 = 0; w2 < g.win[2]; ++w2)
                {
                    const int64_t y0 = o[0] * g.st[0] + w0 - g.pb[0];
                    const int64_t y1 = o[1] * g.st[1] + w1 - g.pb[1];
                    const int64_t y2 = o[2] * g.st[2] + w2 - g.pb[2];
                    const bool inb = y0 >= 0 && y0 < g.in[0] && y1 >= 0 && y1 < g.in[1] && y2 >= 0 && y2 < g.in[2];
                    if (inb)
                    {
                        const int64_t sp = (y0 * g.in[1] + y1) * g.in[2] + y2;
                        const T v = g.nxc ? in[(n * in_sp + sp) * g.C + c] : in[(n * g.C + c) * in_sp + sp];
                        if (AVG)
                        {
                            sum = static_cast<T>(sum + v); // the reference sums in T: 8-bit sums wrap
                            ++cnt;
                        }
                        else
                            best = v > best ? v : best;
                    }
                    else if (AVG && g.include_padding)
                        ++cnt;
                }
        if (AVG)
        {
            // avg_pool.hpp:238-246 : nearbyint(float(sum) / count) for 8-bit types, plain division else
            if (sizeof(T) == 1)
                out[i] = static_cast<T>(rintf(static_cast<float>(sum) / static_cast<float>(static_cast<uint64_t>(cnt))));
            else
                out[i] = static_cast<T>(sum / static_cast<T>(static_cast<uint64_t>(cnt)));
        }
        else
            out[i] = best;
    }

    // out[(o * total + offset + e) * inner + j] = in[(o * extent + e) * inner + j], one byte group per lane
    template <typename T>
    __global__ __launch_bounds__(256) void concat_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t count, int64_t piece, int64_t total, int64_t offset)
    {
        const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
        if (i >= count)
            return;
        const int64_t o = i / piece;
        const int64_t r = i - o * piece;
        out[o * total + offset + r] = in[i];
    }


    // ------------------------------------------------------------------ 8-bit fast paths
    // Four bytes of a dword are reduced at once: the even and the odd bytes are spread into two
    // pairs of 16-bit lanes, where packed 16-bit max / add work on them.  Signed bytes are biased by
    // 0x80 first, which keeps their order as unsigned bytes; 8-bit sums wrap exactly as the
    // reference's sum in T does, because 2^16 is a multiple of 2^8.
    typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

    template <bool AVG>
    struct Bytes4
    {
        // e: even bytes in the low byte of each 16-bit lane; o: odd bytes in the high byte (for the
        // maximum the low byte of o is along for the ride: it cannot change which high byte wins)
        u16x2 e = {0, 0}, o = {0, 0};
        __device__ __forceinline__ void add(uint32_t x)
        {
            const u16x2 xe = __builtin_bit_cast(u16x2, x & 0x00ff00ffu);
            if (AVG)
            {
                e += xe;
                o += __builtin_bit_cast(u16x2, x & 0xff00ff00u);
            }
            else
            {
                e = __builtin_elementwise_max(e, xe);
                o = __builtin_elementwise_max(o, __builtin_bit_cast(u16x2, x));
            }
        }
        __device__ __forceinline__ uint32_t bytes() const
        {
            return (__builtin_bit_cast(uint32_t, e) & 0x00ff00ffu) | (__builtin_bit_cast(uint32_t, o) & 0xff00ff00u);
        }
    };

    // avg_pool.hpp:238-246 for one 8-bit sum: nearbyint(float(T(sum)) / count)
    template <bool SIGNED>
    __device__ __forceinline__ uint32_t avg_byte(uint32_t sum_byte, float cnt)
    {
        const float v = SIGNED ? static_cast<float>(static_cast<int8_t>(sum_byte)) : static_cast<float>(sum_byte);
        return static_cast<uint32_t>(static_cast<int32_t>(rintf(v / cnt))) & 0xffu;
    }

    template <bool SIGNED>
    __device__ __forceinline__ uint32_t avg_bytes4(uint32_t sums, float cnt)
    {
        return avg_byte<SIGNED>(sums & 0xffu, cnt) | (avg_byte<SIGNED>((sums >> 8) & 0xffu, cnt) << 8) |
               (avg_byte<SIGNED>((sums >> 16) & 0xffu, cnt) << 16) | (avg_byte<SIGNED>(sums >> 24, cnt) << 24);
    }

    // valid window positions of output o on an axis: [lo, hi) in window coordinates
    __device__ __forceinline__ void window_range(int o, int stride, int pb, int win, int extent, int& lo, int& hi)
    {
        const int start = o * stride - pb;
        lo = start < 0 ? -start : 0;
        hi = extent - start < win ? extent - start : win;
        if (hi < lo)
            hi = lo;
    }

    struct Pool8Geom
    {
        int N, C;
        int in[3], win[3], st[3], pb[3], out[3];
        int include_padding;
    };

    // Channels-last: one lane per (output pixel, group of 4*VEC channels).  A pixel's channels are
    // contiguous, so a lane's VEC dwords are one load and neighbouring lanes read neighbouring addresses.
    template <bool AVG, bool SIGNED, int VEC>
    __global__ __launch_bounds__(256) void pool8_nxc_kernel(Pool8Geom g, const uint32_t* __restrict__ in, uint32_t* __restrict__ out, uint32_t tasks)
    {
        typedef uint32_t vec_t __attribute__((ext_vector_type(VEC)));
        const uint32_t bias = (!AVG && SIGNED) ? 0x80808080u : 0u;
        // workgroups are dealt round-robin to the 8 XCDs, each with an L2 of its own: give every XCD a
        // contiguous run of the output so that the input rows two neighbouring output rows share are
        // fetched into one L2
        const uint32_t per_xcd = gridDim.x >> 3;
        const uint32_t t = ((blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3)) * 256u + threadIdx.x;
        if (t >= tasks)
            return;
        const uint32_t groups = g.C / (4 * VEC);
        uint32_t pix = t / groups;
        const uint32_t cg = t - pix * groups;
        const int o2 = pix % g.out[2];
        pix /= g.out[2];
        const int o1 = pix % g.out[1];
        pix /= g.out[1];
        const int o0 = pix % g.out[0];
        const int n = pix / g.out[0];
        int lo0, hi0, lo1, hi1, lo2, hi2;
        window_range(o0, g.st[0], g.pb[0], g.win[0], g.in[0], lo0, hi0);
        window_range(o1, g.st[1], g.pb[1], g.win[1], g.in[1], lo1, hi1);
        window_range(o2, g.st[2], g.pb[2], g.win[2], g.in[2], lo2, hi2);
        // The cells of the two inner window axes are fetched kBatch at a time, all loads of a batch in
        // flight together: a loop that loads a cell, waits and reduces pays one memory latency a cell
        // (49 in a row for a 7 x 7 average).  A slot past the window's end holds the reduction's
        // identity (the byte pattern whose biased form is zero).
        constexpr int kBatch = VEC == 4 ? 8 : 16;
        Bytes4<AVG> acc[VEC];
        const int span2 = hi2 - lo2;
        const int cells = (hi1 - lo1) * span2;
        for (int w0 = lo0; w0 < hi0; ++w0)
        {
            const size_t plane = static_cast<size_t>(n) * g.in[0] + (o0 * g.st[0] - g.pb[0] + w0);
            int r = lo1, c = lo2; // cell (r, c) is slot `first` of the next batch
            for (int first = 0; first < cells; first += kBatch)
            {
                vec_t v[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; ++u)
                {
                    const bool in_window = first + u < cells;
                    const size_t line = plane * g.in[1] + (o1 * g.st[1] - g.pb[1] + r);
                    const vec_t* p = reinterpret_cast<const vec_t*>(in) + (line * g.in[2] + (o2 * g.st[2] - g.pb[2] + c)) * groups + cg;
                    vec_t ident;
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        ident[j] = bias;
                    v[u] = in_window ? *p : ident;
                    const bool wrap = c + 1 == hi2;
                    c = wrap ? lo2 : c + 1;
                    r += (wrap && in_window) ? 1 : 0; // (a row past the window is never formed: its address would lie outside the tensor)
                }
#pragma unroll
                for (int u = 0; u < kBatch; ++u)
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        acc[j].add(v[u][j] ^ bias);
            }
        }
        vec_t r;
        if (AVG)
        {
            const int n_el = g.include_padding ? g.win[0] * g.win[1] * g.win[2] : (hi0 - lo0) * (hi1 - lo1) * (hi2 - lo2);
            const float cnt = static_cast<float>(n_el);
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                r[j] = avg_bytes4<SIGNED>(acc[j].bytes(), cnt);
        }
        else
        {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                r[j] = acc[j].bytes() ^ bias;
        }
        reinterpret_cast<vec_t*>(out)[t] = r;
    }

    // division of a small task index by a divisor fixed at launch: q = hi32(t * m), exact for
    // t, d < 2^16 with m = 2^32 / d + 1
    struct SmallDiv
    {
        uint32_t d, m;
        __device__ __forceinline__ uint32_t div(uint32_t t) const { return d == 1 ? t : __umulhi(t, m); }
    };
    static SmallDiv small_div(int64_t d)
    {
        SmallDiv r;
        r.d = static_cast<uint32_t>(d);
        r.m = d > 1 ? static_cast<uint32_t>((1ull << 32) / static_cast<uint64_t>(d) + 1) : 0;
        return r;
    }

    // Channel-major, one or two spatial axes: a workgroup takes G whole planes (contiguous bytes) into
    // LDS, reduces the window's rows into an intermediate row per output row (VW dwords of columns
    // per lane, or single bytes when the width is not a multiple of 4), then reduces along each row.
    // The intermediate rows carry a margin on both sides that holds the reduction's identity (zero:
    // the lowest biased byte, the empty sum), so the second pass needs no bounds on its window.
    struct Pool8Planes
    {
        int planes;       // N * C
        int H, W, OH, OW; // a single spatial axis is W with H = 1
        int win_h, win_w, st_h, st_w, pb_h, pb_w;
        int include_padding;
        int G;            // planes per workgroup
        int pitch;        // bytes per intermediate row, margins included; a multiple of 16
        int margin;       // left margin, >= pb_w, a multiple of 16
        int mid_offset;   // LDS byte offset of the intermediate rows
        int lds_bytes;
        SmallDiv by_cols, by_oh, by_ocols;
    };

    template <bool AVG, bool SIGNED, int VW, bool OUT4>
    __global__ __launch_bounds__(256) void pool8_ncx_kernel(Pool8Planes g, const uint8_t* __restrict__ in, uint8_t* __restrict__ out, uint32_t in_bytes)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
        const uint32_t bias = (!AVG && SIGNED) ? 0x80808080u : 0u;
        const int HW = g.H * g.W;
        const int g0 = blockIdx.x * g.G;
        const int here = g.planes - g0 < g.G ? g.planes - g0 : g.G;
        // planes [g0, g0 + G) as dwords; bytes past the tensor read as zero and belong to planes that are not stored
        {
            const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(in), 0, in_bytes, 0x00020000);
            const uint32_t base = static_cast<uint32_t>(g0) * HW;
            const int dwords = (g.G * HW + 3) >> 2;
            uint32_t* l32 = reinterpret_cast<uint32_t*>(lds);
            for (int i = threadIdx.x; i < dwords; i += 256)
                l32[i] = __builtin_amdgcn_raw_buffer_load_b32(rs, base + 4u * i, 0, 0);
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            u32x4* m128 = reinterpret_cast<u32x4*>(lds + g.mid_offset);
            const int quads = (g.lds_bytes - g.mid_offset) >> 4;
            for (int i = threadIdx.x; i < quads; i += 256)
                m128[i] = u32x4{0, 0, 0, 0};
        }
        __syncthreads();
        uint8_t* mid = lds + g.mid_offset + g.margin;
        // rows of the window -> one intermediate row per output row
        if constexpr (VW > 0)
        {
            typedef uint32_t vec_t __attribute__((ext_vector_type(VW)));
            const uint32_t tasks = static_cast<uint32_t>(here) * g.OH * g.by_cols.d;
            for (uint32_t t = threadIdx.x; t < tasks; t += 256)
            {
                const uint32_t r = g.by_cols.div(t);
                const int k = t - r * g.by_cols.d;
                const uint32_t p = g.by_oh.div(r);
                const int oh = r - p * g.OH;
                int lo, hi;
                window_range(oh, g.st_h, g.pb_h, g.win_h, g.H, lo, hi);
                Bytes4<AVG> acc[VW];
                const uint8_t* src = lds + p * HW + (oh * g.st_h - g.pb_h + lo) * g.W + 4 * VW * k;
                for (int w = lo; w < hi; ++w, src += g.W)
                {
                    const vec_t v = *reinterpret_cast<const vec_t*>(src);
#pragma unroll
                    for (int j = 0; j < VW; ++j)
                        acc[j].add(v[j] ^ bias);
                }
                vec_t res;
#pragma unroll
                for (int j = 0; j < VW; ++j)
                    res[j] = acc[j].bytes();
                *reinterpret_cast<vec_t*>(mid + r * g.pitch + 4 * VW * k) = res;
            }
        }
        else
        {
            const uint32_t tasks = static_cast<uint32_t>(here) * g.OH * g.W;
            for (uint32_t t = threadIdx.x; t < tasks; t += 256)
            {
                const uint32_t r = g.by_cols.div(t);
                const int x = t - r * g.W;
                const uint32_t p = g.by_oh.div(r);
                const int oh = r - p * g.OH;
                int lo, hi;
                window_range(oh, g.st_h, g.pb_h, g.win_h, g.H, lo, hi);
                uint32_t acc = 0;
                const uint8_t* src = lds + p * HW + (oh * g.st_h - g.pb_h + lo) * g.W + x;
                for (int w = lo; w < hi; ++w, src += g.W)
                {
                    const uint32_t v = *src ^ (bias & 0xffu);
                    acc = AVG ? acc + v : (v > acc ? v : acc);
                }
                mid[r * g.pitch + x] = static_cast<uint8_t>(acc);
            }
        }
        __syncthreads();
        // along each intermediate row
        constexpr int PER = OUT4 ? 4 : 1;
        const uint32_t tasks = static_cast<uint32_t>(here) * g.OH * g.by_ocols.d;
        for (uint32_t t = threadIdx.x; t < tasks; t += 256)
        {
            const uint32_t r = g.by_ocols.div(t);
            const int oc = t - r * g.by_ocols.d;
            const uint8_t* src = mid + r * g.pitch + (oc * PER * g.st_w - g.pb_w);
            uint32_t acc[PER];
#pragma unroll
            for (int j = 0; j < PER; ++j)
                acc[j] = 0;
            for (int w = 0; w < g.win_w; ++w, ++src)
            {
#pragma unroll
                for (int j = 0; j < PER; ++j)
                {
                    const uint32_t v = src[j * g.st_w];
                    acc[j] = AVG ? acc[j] + v : (v > acc[j] ? v : acc[j]);
                }
            }
            uint32_t packed = 0;
            if (AVG)
            {
                const int oh = r - g.by_oh.div(r) * g.OH;
                int lo_h, hi_h;
                window_range(oh, g.st_h, g.pb_h, g.win_h, g.H, lo_h, hi_h);
#pragma unroll
                for (int j = 0; j < PER; ++j)
                {
                    int lo, hi;
                    window_range(oc * PER + j, g.st_w, g.pb_w, g.win_w, g.W, lo, hi);
                    const int n_el = g.include_padding ? g.win_h * g.win_w : (hi_h - lo_h) * (hi - lo);
                    packed |= avg_byte<SIGNED>(acc[j] & 0xffu, static_cast<float>(n_el)) << (8 * j);
                }
            }
            else
            {
#pragma unroll
                for (int j = 0; j < PER; ++j)
                    packed |= acc[j] << (8 * j);
                packed ^= bias;
            }
            const size_t o = (static_cast<size_t>(g0) * g.OH + r) * g.OW + oc * PER;
            if (OUT4)
                *reinterpret_cast<uint32_t*>(out + o) = packed;
            else
                out[o] = static_cast<uint8_t>(packed);
        }
    }

    template <bool AVG, bool SIGNED>
    static void launch_pool8_ncx(const Pool8Planes& p, int vw, bool out4, unsigned grid, const void* in, void* out, uint32_t in_bytes, hipStream_t s)
    {
        const uint8_t* i8 = static_cast<const uint8_t*>(in);
        uint8_t* o8 = static_cast<uint8_t*>(out);
        const size_t lds_bytes = static_cast<size_t>(p.lds_bytes);
#define HIPQ_POOL8_CASE(VW, OUT4)                                                                  \
    if (vw == VW && out4 == OUT4)                                                                  \
        pool8_ncx_kernel<AVG, SIGNED, VW, OUT4><<<grid, 256, lds_bytes, s>>>(p, i8, o8, in_bytes);
        HIPQ_POOL8_CASE(4, true)
        HIPQ_POOL8_CASE(4, false)
        HIPQ_POOL8_CASE(1, true)
        HIPQ_POOL8_CASE(1, false)
        HIPQ_POOL8_CASE(0, true)
        HIPQ_POOL8_CASE(0, false)
#undef HIPQ_POOL8_CASE
    }

    template <bool AVG, bool SIGNED>
    static void launch_pool8_nxc(const Pool8Geom& p, int vec, uint32_t tasks, const void* in, void* out, hipStream_t s)
    {
        const uint32_t* i32 = static_cast<const uint32_t*>(in);
        uint32_t* o32 = static_cast<uint32_t*>(out);
        const unsigned grid = ((tasks + 255) / 256 + 7) / 8 * 8;
        if (vec == 4)
            pool8_nxc_kernel<AVG, SIGNED, 4><<<grid, 256, 0, s>>>(p, i32, o32, tasks);
        else
            pool8_nxc_kernel<AVG, SIGNED, 1><<<grid, 256, 0, s>>>(p, i32, o32, tasks);
    }

    // -> true when one of the 8-bit kernels took the call
    static bool try_pool8(const PoolGeom& g, int op, bool is_signed, const void* in, void* out, hipStream_t s, int& rc)
    {
        if (getenv("HIPQ_NO_FAST_POOL"))
            return false;
        const int64_t lim = 1ll << 30;
        const int64_t in_bytes = g.N * g.C * g.in[0] * g.in[1] * g.in[2];
        if (in_bytes >= (1ll << 32) || g.N * g.C >= lim)
            return false;
        for (int i = 0; i < 3; ++i)
            if (g.in[i] >= lim || g.win[i] >= (1 << 15) || g.st[i] >= lim || g.pb[i] >= lim || g.out[i] >= lim)
                return false;
        const bool avg = op == HIPQ_POOL_AVG;
        const uintptr_t ai = reinterpret_cast<uintptr_t>(in), ao = reinterpret_cast<uintptr_t>(out);
        if (g.nxc)
        {
            const int64_t out_dwords = g.count / 4;
            if (g.C % 4 != 0 || (ai | ao) % 4 != 0 || out_dwords >= (1ll << 31))
                return false;
            Pool8Geom p;
            p.N = static_cast<int>(g.N);
            p.C = static_cast<int>(g.C);
            for (int i = 0; i < 3; ++i)
            {
                p.in[i] = static_cast<int>(g.in[i]);
                p.win[i] = static_cast<int>(g.win[i]);
                p.st[i] = static_cast<int>(g.st[i]);
                p.pb[i] = static_cast<int>(g.pb[i]);
                p.out[i] = static_cast<int>(g.out[i]);
            }
            p.include_padding = g.include_padding;
            // 16 bytes per lane unless that leaves the device short of lanes (a global pool over few pixels)
            const int vec = (g.C % 16 == 0 && (ai | ao) % 16 == 0 && out_dwords / 4 >= 256 * 1024) ? 4 : 1;
            const uint32_t grid = static_cast<uint32_t>(out_dwords / vec);
            if (avg)
                is_signed ? launch_pool8_nxc<true, true>(p, vec, grid, in, out, s) : launch_pool8_nxc<true, false>(p, vec, grid, in, out, s);
            else
                is_signed ? launch_pool8_nxc<false, true>(p, vec, grid, in, out, s) : launch_pool8_nxc<false, false>(p, vec, grid, in, out, s);
            rc = check_launch(avg ? "avg_pool8_nxc" : "max_pool8_nxc");
            return true;
        }
        if (g.in[0] != 1 || g.out[0] != 1 || in_bytes % 4 != 0 || ai % 4 != 0)
            return false;
        const int64_t HW = g.in[1] * g.in[2];
        const int64_t unit = HW % 4 == 0 ? 1 : (HW % 2 == 0 ? 2 : 4);
        int64_t G = unit * (4096 / (HW * unit) > 1 ? 4096 / (HW * unit) : 1);
        // margins of the intermediate rows: the window of the first output starts pb columns left of
        // the data, the window of the last output may end past it
        const int64_t margin = (g.pb[2] + 15) / 16 * 16;
        const int64_t over = (g.out[2] - 1) * g.st[2] - g.pb[2] + g.win[2] - g.in[2];
        const int64_t pitch = (margin + g.in[2] + (over > 0 ? over : 0) + 15) / 16 * 16;
        const int64_t mid_offset = (G * HW + 15) / 16 * 16;
        const int64_t lds_bytes = mid_offset + G * g.out[1] * pitch;
        if (lds_bytes > 64 * 1024)
            return false;
        Pool8Planes p;
        p.planes = static_cast<int>(g.N * g.C);
        p.H = static_cast<int>(g.in[1]);
        p.W = static_cast<int>(g.in[2]);
        p.OH = static_cast<int>(g.out[1]);
        p.OW = static_cast<int>(g.out[2]);
        p.win_h = static_cast<int>(g.win[1]);
        p.win_w = static_cast<int>(g.win[2]);
        p.st_h = static_cast<int>(g.st[1]);
        p.st_w = static_cast<int>(g.st[2]);
        p.pb_h = static_cast<int>(g.pb[1]);
        p.pb_w = static_cast<int>(g.pb[2]);
        p.include_padding = g.include_padding;
        p.G = static_cast<int>(G);
        p.pitch = static_cast<int>(pitch);
        p.margin = static_cast<int>(margin);
        p.mid_offset = static_cast<int>(mid_offset);
        p.lds_bytes = static_cast<int>(lds_bytes);
        const int vw = g.in[2] % 16 == 0 ? 4 : (g.in[2] % 4 == 0 ? 1 : 0);
        const bool out4 = g.out[2] % 4 == 0 && ao % 4 == 0;
        p.by_cols = small_div(vw ? g.in[2] / (4 * vw) : g.in[2]);
        p.by_oh = small_div(g.out[1]);
        p.by_ocols = small_div(out4 ? g.out[2] / 4 : g.out[2]);
        const unsigned grid = static_cast<unsigned>((p.planes + G - 1) / G);
        if (avg)
            is_signed ? launch_pool8_ncx<true, true>(p, vw, out4, grid, in, out, static_cast<uint32_t>(in_bytes), s)
                      : launch_pool8_ncx<true, false>(p, vw, out4, grid, in, out, static_cast<uint32_t>(in_bytes), s);
        else
            is_signed ? launch_pool8_ncx<false, true>(p, vw, out4, grid, in, out, static_cast<uint32_t>(in_bytes), s)
                      : launch_pool8_ncx<false, false>(p, vw, out4, grid, in, out, static_cast<uint32_t>(in_bytes), s);
        rc = check_launch(avg ? "avg_pool8_ncx" : "max_pool8_ncx");
        return true;
    }

    template <typename T>
    static int launch_pool(const PoolGeom& g, int op, const void* in, void* out, hipStream_t s)
    {
        const unsigned grid = static_cast<unsigned>((g.count + 255) / 256);
        if (op == HIPQ_POOL_AVG)
            pool_kernel<T, true><<<grid, 256, 0, s>>>(g, static_cast<const T*>(in), static_cast<T*>(out));
        else
            pool_kernel<T, false><<<grid, 256, 0, s>>>(g, static_cast<const T*>(in), static_cast<T*>(out));
        return check_launch(op == HIPQ_POOL_AVG ? "avg_pool" : "max_pool");
    }
}

using namespace hipq;

extern "C" {

int hipq_pool_infer_output(hipq_pool_desc_t* d)
{
    HIPQ_REQUIRE(d, "descriptor is null");
    HIPQ_REQUIRE(d->n_spatial >= 1 && d->n_spatial <= HIPQ_MAX_SPATIAL, "n_spatial %d out of range", d->n_spatial);
    for (int i = 0; i < d->n_spatial; ++i)
    {
        HIPQ_REQUIRE(d->in_sp[i] >= 1 && d->window[i] >= 1 && d->stride[i] >= 1 && d->pad_below[i] >= 0 && d->pad_above[i] >= 0,
                     "non-positive extent, window or stride, or negative padding on spatial axis %d", i);
        const int64_t padded = d->in_sp[i] + d->pad_below[i] + d->pad_above[i];
        HIPQ_REQUIRE(padded >= d->window[i], "window larger than padded data on spatial axis %d", i);
        d->out_sp[i] = (padded - d->window[i]) / d->stride[i] + 1;
    }
    return HIPQ_OK;
}

int hipq_pool(const hipq_pool_desc_t* d, const void* in, void* out, void* stream)
{
    HIPQ_REQUIRE(d, "descriptor is null");
    hipq_pool_desc_t chk = *d;
    int rc = hipq_pool_infer_output(&chk);
    if (rc)
        return rc;
    HIPQ_REQUIRE(d->op == HIPQ_POOL_MAX || d->op == HIPQ_POOL_AVG, "pool op %d unknown", d->op);
    HIPQ_REQUIRE(d->layout == HIPQ_LAYOUT_NCX || d->layout == HIPQ_LAYOUT_NXC, "layout %d unknown", d->layout);
    HIPQ_REQUIRE(d->N >= 0 && d->C >= 0, "negative extent");
    PoolGeom g;
    g.N = d->N;
    g.C = d->C;
    g.nxc = d->layout == HIPQ_LAYOUT_NXC;
    g.include_padding = d->include_padding;
    // normalise to three spatial axes, leading ones of extent 1
    const int lead = 3 - d->n_spatial;
    for (int i = 0; i < 3; ++i)
    {
        const bool real = i >= lead;
        g.in[i] = real ? d->in_sp[i - lead] : 1;
        g.win[i] = real ? d->window[i - lead] : 1;
        g.st[i] = real ? d->stride[i - lead] : 1;
        g.pb[i] = real ? d->pad_below[i - lead] : 0;
        g.out[i] = real ? chk.out_sp[i - lead] : 1;
        HIPQ_REQUIRE(!real || d->out_sp[i - lead] == chk.out_sp[i - lead], "out_sp[%d] does not match the window geometry", i - lead);
    }
    g.count = g.N * g.C * g.out[0] * g.out[1] * g.out[2];
    if (g.count == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(in && out, "null tensor pointer");
    HIPQ_REQUIRE((g.count + 255) / 256 < (1ll << 31), "tensor too large for one launch");
    if (d->op == HIPQ_POOL_AVG)
    {
        // a window that sees neither data nor counted padding has no average: the reference throws
        for (int i = 0; i < 3; ++i)
            HIPQ_REQUIRE(d->include_padding || (g.pb[i] < g.win[i] && (g.out[i] - 1) * g.st[i] - g.pb[i] < g.in[i]),
                         "AvgPool window wholly inside the padding (elements == 0)");
    }
    hipStream_t s = as_stream(stream);
    if ((d->dtype == HIPQ_U8 || d->dtype == HIPQ_I8) && try_pool8(g, d->op, d->dtype == HIPQ_I8, in, out, s, rc))
        return rc;
    switch (d->dtype)
    {
    case HIPQ_U8: return launch_pool<uint8_t>(g, d->op, in, out, s);
    case HIPQ_I8: return launch_pool<int8_t>(g, d->op, in, out, s);
    case HIPQ_F32: return launch_pool<float>(g, d->op, in, out, s);
    case HIPQ_I32:
        if (d->op == HIPQ_POOL_MAX)
            return launch_pool<int32_t>(g, d->op, in, out, s);
        return fail(HIPQ_ERR_UNSUPPORTED, "AvgPool on i32 is not supported");
    default: return fail(HIPQ_ERR_UNSUPPORTED, "pooling on dtype %d", d->dtype);
    }
}

int hipq_concat(int32_t elem_bytes,
                int32_t n_inputs,
                const void* const* inputs,
                const int64_t* extents,
                int64_t outer,
                int64_t inner,
                void* out,
                void* stream)
{
    HIPQ_REQUIRE(n_inputs >= 0 && outer >= 0 && inner >= 0, "negative extent");
    HIPQ_REQUIRE(elem_bytes == 1 || elem_bytes == 4 || elem_bytes == 8, "concat of %d-byte elements", elem_bytes);
    HIPQ_REQUIRE(n_inputs == 0 || (inputs && extents), "null input table");
    int64_t total = 0;
    for (int i = 0; i < n_inputs; ++i)
    {
        HIPQ_REQUIRE(extents[i] >= 0, "negative extent of input %d", i);
        total += extents[i];
    }
    hipStream_t s = as_stream(stream);
    // widest unit (up to 16 bytes) that divides every piece, the output pitch and every pointer
    int64_t unit = 16;
    auto narrow = [&unit](int64_t v) {
        while (unit > 1 && v % unit != 0)
            unit >>= 1;
    };
    narrow(total * inner * elem_bytes);
    narrow(static_cast<int64_t>(reinterpret_cast<uintptr_t>(out) % 16));
    for (int i = 0; i < n_inputs; ++i)
    {
        narrow(extents[i] * inner * elem_bytes);
        if (outer * extents[i] * inner > 0)
            narrow(static_cast<int64_t>(reinterpret_cast<uintptr_t>(inputs[i]) % 16));
    }
    const int64_t per = unit / (unit % elem_bytes == 0 ? elem_bytes : unit); // elements per unit
    int64_t offset = 0;
    for (int i = 0; i < n_inputs; ++i)
    {
        const int64_t piece = extents[i] * inner / per;
        const int64_t count = outer * piece;
        if (count > 0)
        {
            HIPQ_REQUIRE(inputs[i] && out, "null tensor pointer");
            HIPQ_REQUIRE((count + 255) / 256 < (1ll << 31), "tensor too large for one launch");
            const unsigned grid = static_cast<unsigned>((count + 255) / 256);
            const int64_t pitch = total * inner / per, at = offset * inner / per;
            const int64_t width = per * elem_bytes;
            if (width == 1)
                concat_kernel<uint8_t><<<grid, 256, 0, s>>>(static_cast<const uint8_t*>(inputs[i]), static_cast<uint8_t*>(out), count, piece, pitch, at);
            else if (width == 2)
                concat_kernel<uint16_t><<<grid, 256, 0, s>>>(static_cast<const uint16_t*>(inputs[i]), static_cast<uint16_t*>(out), count, piece, pitch, at);
            else if (width == 4)
                concat_kernel<uint32_t><<<grid, 256, 0, s>>>(static_cast<const uint32_t*>(inputs[i]), static_cast<uint32_t*>(out), count, piece, pitch, at);
            else if (width == 8)
                concat_kernel<uint64_t><<<grid, 256, 0, s>>>(static_cast<const uint64_t*>(inputs[i]), static_cast<uint64_t*>(out), count, piece, pitch, at);
            else
                concat_kernel<uint4><<<grid, 256, 0, s>>>(static_cast<const uint4*>(inputs[i]), static_cast<uint4*>(out), count, piece, pitch, at);
            int rc = check_launch("concat");
            if (rc)
                return rc;
        }
        offset += extents[i];
    }
    return HIPQ_OK;
}
}
