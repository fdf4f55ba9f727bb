// Compare-and-pack primitives shared by the quantizer kernels and the fused 1x1 conv kernel: sixteen lanes (one
// DPP row) turn one row of 64 consecutive channels, read as 16 float4, into its packed element.
#pragma once
#include "tab_common.h"

namespace tab {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t uintx4 __attribute__((ext_vector_type(4)));
typedef uint32_t uintx2 __attribute__((ext_vector_type(2)));

// OR over the 8 lanes of each half of a 16-lane DPP row; every lane gets the result.
__device__ __forceinline__ uint32_t or_reduce8(uint32_t v)
{
    v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
    v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
    v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, true);  // row_half_mirror
    return v;
}

// value of the lane 8 positions further round the 16-lane DPP row (row_ror:8)
__device__ __forceinline__ uint32_t rotate_row8(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x128, 0xF, 0xF, true);
}

// Compare one float4 against the threshold; bit e of the result belongs to element e.
// MODE 2, ternary: first test v > t (+1), only then v < -t (-1); both are strict and ordered, so
// ties and NaN give 0 (TAB_GEMM.cu:184-192).  MODE 1, binary: bit = v < t (TAB_GEMM.cu:231).
// MODE 5 (RTN fields) compares like MODE 2.  MODE 4 (2-bit levels): `sign` gets the weight-2 bit and
// `nz` the weight-1 bit of level = (v >= 0.5t) + (v >= 1.5t) + (v >= 2.5t).
template <int MODE>
__device__ __forceinline__ void compare4(const floatx4 v, const float t, uint32_t &sign, uint32_t &nz)
{
    const float e[4] = {v[0], v[1], v[2], v[3]};
    sign = 0;
    nz = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        if (MODE == 2 || MODE == 5) {
            const bool pos = e[i] > t;
            const bool neg = !pos && (e[i] < -t);
            nz |= (uint32_t)(pos || neg) << i;
            sign |= (uint32_t)neg << i;
        } else if (MODE == 4) {
            const int level = (int)(e[i] >= 0.5f * t) + (int)(e[i] >= 1.5f * t) + (int)(e[i] >= 2.5f * t);
            sign |= (uint32_t)(level >> 1) << i;
            nz |= (uint32_t)(level & 1) << i;
        } else {
            sign |= (uint32_t)(e[i] < t) << i;
        }
    }
}

// The packed output of one 64-channel row from the compare bits of lane l of its 16-lane DPP row; all
// lanes of the row take part, lane 0 gets the complete result: out[0..1] for MODE 1, out[0..3] else.
// MODE 1/2/4: the lane's nibble goes to bit 4*(l%8) and an OR over 8 lanes yields the low (lanes 0-7)
// or high (lanes 8-15) 32 bits of a plane word; a rotate by 8 within the row hands lane 0 the other
// half: (plane 0 low, plane 0 high, plane 1 low, plane 1 high).
// MODE 5: the row is two words of 32 two-bit fields (TAB_CPU.cpp:364-379); the lane's four fields
// (8 bits, even bit = nonzero, odd bit = sign) go to byte l%4 of the low (l%8 < 4) or high half of the
// word lanes 0-7 (channels 0-31) or lanes 8-15 (channels 32-63) build: (word 0 low, high, word 1 low, high).
template <int MODE>
__device__ __forceinline__ void pack_row(uint32_t sign, uint32_t nz, int l, uint32_t (&out)[4])
{
    if (MODE == 5) {
        uint32_t fields = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) fields |= (((nz >> i) & 1u) | (((sign >> i) & 1u) << 1)) << (2 * i);
        const uint32_t placed = fields << (8 * (l & 3));
        const uint32_t lo = or_reduce8((l & 4) ? 0u : placed), hi = or_reduce8((l & 4) ? placed : 0u);
        out[0] = lo; out[1] = hi; out[2] = rotate_row8(lo); out[3] = rotate_row8(hi);
        return;
    }
    const int shift = 4 * (l & 7);
    const uint32_t sign_half = or_reduce8(sign << shift);
    out[0] = sign_half;
    out[1] = rotate_row8(sign_half);
    if (MODE != 1) {
        const uint32_t nz_half = or_reduce8(nz << shift);
        out[2] = nz_half;
        out[3] = rotate_row8(nz_half);
    }
}

}  // namespace
}  // namespace tab
