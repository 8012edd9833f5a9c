// Scan over the 64 lanes of a wavefront with lane-to-lane moves (data-parallel-primitive modifiers of the vector ALU),
// shared by the hand-written and the generated reassociating row scans.
#ifndef OVL_WAVE_SCAN_H_
#define OVL_WAVE_SCAN_H_

#include <stdint.h>

// Lane-to-lane move with a row mask: rows of 16 lanes whose bit is clear in ROW_MASK, and lanes the pattern gives no
// source, receive `old`.  CTRL: 0x110 + n = row_shr:n, 0x138 = wave_shr:1, 0x142 = row_bcast:15, 0x143 = row_bcast:31.
template <int CTRL, int ROW_MASK, typename T>
__device__ __forceinline__ T ovl_masked_lane_move(T old, T src) {
    if constexpr (sizeof(T) == 8) {
        const uint64_t o = __builtin_bit_cast(uint64_t, old), v = __builtin_bit_cast(uint64_t, src);
        const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp((int)(uint32_t)o, (int)(uint32_t)v, CTRL, ROW_MASK, 0xf, false);
        const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp((int)(uint32_t)(o >> 32), (int)(uint32_t)(v >> 32), CTRL,
                                                                  ROW_MASK, 0xf, false);
        return __builtin_bit_cast(T, ((uint64_t)hi << 32) | lo);
    } else {
        static_assert(sizeof(T) == 4, "lane moves carry 4 or 8 bytes");
        return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, src),
                                                                 CTRL, ROW_MASK, 0xf, false));
    }
}

// Inclusive scan in six steps: lanes 1, 2, 4 and 8 below within each row of sixteen (row_shr), then the last lane of
// row 0 into row 1 and of row 2 into row 3 (row_bcast:15), then lane 31 into rows 2 and 3 (row_bcast:31).  `unit` is
// the value with op(unit, x) == x: a lane without a partner combines with it and stays unchanged.
template <typename T, typename F>
__device__ __forceinline__ T ovl_wave_inclusive_scan(T v, T unit, F op) {
    v = op(ovl_masked_lane_move<0x111, 0xf>(unit, v), v);
    v = op(ovl_masked_lane_move<0x112, 0xf>(unit, v), v);
    v = op(ovl_masked_lane_move<0x114, 0xf>(unit, v), v);
    v = op(ovl_masked_lane_move<0x118, 0xf>(unit, v), v);
    v = op(ovl_masked_lane_move<0x142, 0xa>(unit, v), v);
    v = op(ovl_masked_lane_move<0x143, 0xc>(unit, v), v);
    return v;
}

// The inclusive value of the lane below (wave_shr:1); lane 0 receives `unit`.
template <typename T>
__device__ __forceinline__ T ovl_wave_shift_up(T inclusive, T unit) {
    return ovl_masked_lane_move<0x138, 0xf>(unit, inclusive);
}

#endif  // OVL_WAVE_SCAN_H_
