/*
 * Cross-lane arithmetic that stays in the vector ALU on gfx950: DPP moves
 * inside a 16-lane row, the row swaps v_permlane16_swap / v_permlane32_swap
 * across rows.  Nothing here goes through the LDS crossbar (ds_bpermute), so
 * nothing waits on lgkmcnt.  64-lane wavefronts.
 */
#ifndef FBLT_AMD_LANE_OPS_H
#define FBLT_AMD_LANE_OPS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float x) {
    return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), CTRL, 0xf, 0xf, true));
}
constexpr int DPP_XOR1 = 0xB1, DPP_XOR2 = 0x4E, DPP_HALF_MIRROR = 0x141, DPP_ROW_MIRROR = 0x140;
constexpr int DPP_ROR1 = 0x121, DPP_ROR2 = 0x122, DPP_ROR4 = 0x124, DPP_ROR8 = 0x128;

struct OpSum {
    __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
struct OpMax {
    __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};

/* x combined over lanes l ^ 16 (rows of 16 lanes pairwise), result in both */
template <typename Op>
__device__ __forceinline__ float swap16(float x, Op op) {
    const unsigned u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return op(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
/* x combined over lanes l ^ 32 */
template <typename Op>
__device__ __forceinline__ float swap32(float x, Op op) {
    const unsigned u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return op(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

/* Sum over the G consecutive lanes of a key (G a power of two up to 32); every lane gets it.
 * After the two quad steps all four lanes of a quad agree, so the mirrored reads of the next
 * two steps fetch the other quad's / the other half row's sum whatever lane they land on. */
template <int G>
__device__ __forceinline__ float key_sum(float x) {
    if (G >= 2) x += dpp_mov<DPP_XOR1>(x);
    if (G >= 4) x += dpp_mov<DPP_XOR2>(x);
    if (G >= 8) x += dpp_mov<DPP_HALF_MIRROR>(x);
    if (G >= 16) x += dpp_mov<DPP_ROW_MIRROR>(x);
    if (G >= 32) x = swap16(x, OpSum());
    return x;
}

/* Combination over the 64 / G keys a wave holds at once, lane g of every key with lane g of
 * every other key: rotations inside a 16-lane row (a rotation by a multiple of G keeps g), then
 * the row swaps.  Every lane gets the result. */
template <int G, typename Op>
__device__ __forceinline__ float across_keys(float x, Op op) {
    if (G <= 8) x = op(x, dpp_mov<DPP_ROR8>(x));
    if (G <= 4) x = op(x, dpp_mov<DPP_ROR4>(x));
    if (G <= 2) x = op(x, dpp_mov<DPP_ROR2>(x));
    if (G <= 1) x = op(x, dpp_mov<DPP_ROR1>(x));
    if (G <= 16) x = swap16(x, op);
    return swap32(x, op);
}

/* Combination over the first 16 lanes of a wave (lanes 16.. hold the identity); lane 0's row
 * gets the result. */
template <typename Op>
__device__ __forceinline__ float row0_all(float x, Op op) {
    x = op(x, dpp_mov<DPP_XOR1>(x));
    x = op(x, dpp_mov<DPP_XOR2>(x));
    x = op(x, dpp_mov<DPP_HALF_MIRROR>(x));
    x = op(x, dpp_mov<DPP_ROW_MIRROR>(x));
    return x;
}

/* the lane-read builtins take and return integers: pass the bit pattern, not the value */
__device__ __forceinline__ float first_lane(float x) {
    return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(x)));
}
__device__ __forceinline__ float lane_value(float x, int l) {
    return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(x), l));
}

#endif
