// Division of a 31-bit index by a divisor fixed at launch, as the Quantize / Dequantize kernels use it
// for their scale index.
#pragma once
#include <cstdint>

#ifndef __HIPCC__
#define __host__
#define __device__
#define __forceinline__ inline
#endif

namespace hipq
{
    // ---- division of a 31-bit index by a run-time constant -----------------------------------
    // q = (n * magic) >> (31 + shift) with shift = ceil(log2 d), magic = ceil(2^(31+shift) / d)
    // is exact for every 0 <= n < 2^31 (Granlund & Montgomery, N = 31).
    struct IndexDiv
    {
        uint32_t magic;
        uint32_t shift;
        uint32_t d;
    };

    inline IndexDiv make_fastdiv(uint32_t d)
    {
        IndexDiv f;
        f.d = d;
        uint32_t s = 0;
        while ((1ull << s) < d)
            ++s;
        f.shift = s;
        unsigned __int128 num = static_cast<unsigned __int128>(1) << (31 + s);
        f.magic = static_cast<uint32_t>((num + d - 1) / d);
        return f;
    }

    __host__ __device__ __forceinline__ uint32_t fastdiv(uint32_t n, const IndexDiv& f)
    {
        return static_cast<uint32_t>((static_cast<uint64_t>(n) * f.magic) >> (31 + f.shift));
    }
}
