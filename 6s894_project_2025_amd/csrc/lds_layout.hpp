// Compile-time checks of LDS access patterns: a swizzle that would serialise a 16-byte LDS access is
// a build error rather than a slow kernel.  The idea follows the reference's static layout checks
// (csrc/frag.cuh:94-160 bank-conflict freedom, :437-474 coalescing), restated for wave64 and
// 16-byte accesses.
//
// Model: a wavefront's ds_read_b128 / ds_write_b128 is served eight lanes at a time, 128 bytes per
// pass; the eight lanes of a pass proceed together when their 16-byte pieces fall into eight
// different 16-byte columns of the 128-byte LDS row, i.e. when (address / 16) % 8 takes eight
// different values.  Every pattern below that passes this test measured SQ_LDS_BANK_CONFLICT = 0
// on the device.
#pragma once
#include <cstdint>

namespace mi {
namespace lds {

// `addr(lane)` = byte address of lane's 16-byte piece, lane = 0..63
template <class AddrOfLane>
constexpr bool conflict_free_b128(AddrOfLane addr)
{
    for (uint32_t pass = 0; pass < 8; ++pass) {
        uint32_t seen = 0;
        for (uint32_t l = 0; l < 8; ++l) {
            const uint32_t a = addr(8u * pass + l);
            if (a % 16u != 0) return false;  // must be a single 16-byte access
            const uint32_t column = (a / 16u) % 8u;
            if (seen & (1u << column)) return false;
            seen |= 1u << column;
        }
    }
    return true;
}

// The same when only some lanes take part (`active(lane)`): the others are masked off and touch
// nothing.
template <class AddrOfLane, class Active>
constexpr bool conflict_free_b128_masked(AddrOfLane addr, Active active)
{
    for (uint32_t pass = 0; pass < 8; ++pass) {
        uint32_t seen = 0;
        for (uint32_t l = 0; l < 8; ++l) {
            if (!active(8u * pass + l)) continue;
            const uint32_t a = addr(8u * pass + l);
            if (a % 16u != 0) return false;
            const uint32_t column = (a / 16u) % 8u;
            if (seen & (1u << column)) return false;
            seen |= 1u << column;
        }
    }
    return true;
}

}  // namespace lds
}  // namespace mi
