// Division of a workgroup index by the (runtime) number of node tiles without the integer-division sequence.
// Usable from host code (the divisor is prepared there) and from device code.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define BBHIP_HD __host__ __device__
#else
#define BBHIP_HD
#endif

namespace bbhip {

// mul = ceil(2^(31+L) / d), L = ceil(log2 d)  gives  n / d == (n * mul) >> (31 + L)  exactly for 0 <= n < 2^31
// (the error term n * (mul * d - 2^(31+L)) is below 2^(31+L) because mul * d - 2^(31+L) < d <= 2^L).
struct TileDivisor {
    int      count;
    uint32_t mul;
    uint32_t shift;      // 31 + L
};

inline TileDivisor make_tile_divisor(int d)
{
    TileDivisor t;
    t.count = d;
    uint32_t L = 0;
    while ((1ull << L) < (unsigned long long)d) { ++L; }
    t.shift = 31 + L;
    t.mul = (uint32_t)(((1ull << t.shift) + (unsigned long long)d - 1) / (unsigned long long)d);
    return t;
}

// lid = outer * tiles.count + tile
BBHIP_HD inline void split_tile(int lid, TileDivisor const &tiles, int &outer, int &tile)
{
    outer = (int)(((unsigned long long)(uint32_t)lid * tiles.mul) >> tiles.shift);
    tile  = lid - outer * tiles.count;
}

}  // namespace bbhip
