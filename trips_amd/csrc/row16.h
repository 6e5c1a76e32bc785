// Cross-lane primitives inside one DPP row (16 consecutive lanes of a wave64). A row holds one pixel list:
// lane j of the row owns entry j. Everything here is a v_mov_dpp, no LDS crossbar traffic. The callers keep every
// row either fully active or fully inactive, so a DPP source lane is never masked off by EXEC.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace trips
{
using u64 = unsigned long long;

// DPP controls (gfx9 encoding)
constexpr int kDppXor1       = 0xB1;   // quad_perm [1,0,3,2]
constexpr int kDppXor2       = 0x4E;   // quad_perm [2,3,0,1]
constexpr int kDppQuadRev    = 0x1B;   // quad_perm [3,2,1,0]      lane ^ 3
constexpr int kDppHalfMirror = 0x141;  // row_half_mirror          lane ^ 7
constexpr int kDppMirror     = 0x140;  // row_mirror               lane ^ 15
constexpr int kDppRor8       = 0x128;  // row_ror:8                lane ^ 8
constexpr int kDppShr1       = 0x111;  // row_shr:1                lane i reads lane i-1

// full permutations inside a row: every source lane exists, so `old` is irrelevant (bound_ctrl avoids a copy)
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return __int_as_float(dpp_i<CTRL>(__float_as_int(v)));
}
template <int CTRL>
__device__ __forceinline__ u64 dpp_u64(u64 v)
{
    const unsigned lo = (unsigned)dpp_i<CTRL>((int)(unsigned)v);
    const unsigned hi = (unsigned)dpp_i<CTRL>((int)(unsigned)(v >> 32));
    return ((u64)hi << 32) | lo;
}

// value of lane (i ^ M) of the same row, M in {1, 2, 4, 8, 15}
template <int M>
__device__ __forceinline__ u64 row_xor_u64(u64 v)
{
    static_assert(M == 1 || M == 2 || M == 4 || M == 8 || M == 15, "unsupported row xor");
    if (M == 1) return dpp_u64<kDppXor1>(v);
    if (M == 2) return dpp_u64<kDppXor2>(v);
    if (M == 4) return dpp_u64<kDppQuadRev>(dpp_u64<kDppHalfMirror>(v));  // (i ^ 3) ^ 7 = i ^ 4
    if (M == 8) return dpp_u64<kDppRor8>(v);
    return dpp_u64<kDppMirror>(v);
}

// 64-bit lane mask with bit (16 r + i) set for the row positions i whose bit in `pattern16` is set
__host__ __device__ constexpr u64 rows4(unsigned pattern16)
{
    return (u64)pattern16 | ((u64)pattern16 << 16) | ((u64)pattern16 << 32) | ((u64)pattern16 << 48);
}

// row positions that keep the LARGER key in step (K, J) of an ascending bitonic sort of 16
template <int K, int J>
__host__ __device__ constexpr unsigned want_max_pattern()
{
    unsigned m = 0;
    for (int i = 0; i < 16; ++i)
    {
        const bool up    = (i & K) == 0 || K == 16;
        const bool lower = (i & J) == 0;
        if (lower != up) m |= 1u << i;
    }
    return m;
}

// One compare-exchange step: keys are distinct (or both the +inf filler), so "take the partner's key" is
// (partner < mine) xor (this position keeps the larger one). The position pattern is a compile-time lane mask,
// which leaves one 64-bit compare, one scalar xor and two selects per step.
template <int K, int J>
__device__ __forceinline__ u64 bitonic_step(u64 v)
{
    const u64 o        = row_xor_u64<J>(v);
    constexpr u64 kMax = rows4(want_max_pattern<K, J>());
    const u64 lt       = __builtin_amdgcn_ballot_w64(o < v);
    const bool take    = __builtin_amdgcn_inverse_ballot_w64(lt ^ kMax);
    return take ? o : v;
}

// ascending bitonic sort of the 16 keys of a row (lanes outside active rows see EXEC = 0 and are untouched)
__device__ __forceinline__ u64 row_sort16(u64 v)
{
    v = bitonic_step<2, 1>(v);
    v = bitonic_step<4, 2>(v);
    v = bitonic_step<4, 1>(v);
    v = bitonic_step<8, 4>(v);
    v = bitonic_step<8, 2>(v);
    v = bitonic_step<8, 1>(v);
    v = bitonic_step<16, 8>(v);
    v = bitonic_step<16, 4>(v);
    v = bitonic_step<16, 2>(v);
    v = bitonic_step<16, 1>(v);
    return v;
}

// v is bitonic over the row: ascending merge
__device__ __forceinline__ u64 row_merge16(u64 v)
{
    v = bitonic_step<16, 8>(v);
    v = bitonic_step<16, 4>(v);
    v = bitonic_step<16, 2>(v);
    v = bitonic_step<16, 1>(v);
    return v;
}

// ---- the same row split into two independent lists of 8 lanes (two short pixel lists per DPP row) ----
// final merge stage of an ascending sort of 8: every 8-lane group ascends, so position i keeps the larger key
// when its bit J is set
template <int J>
__device__ __forceinline__ u64 bitonic_step_half_ascending(u64 v)
{
    static_assert(J == 1 || J == 2 || J == 4, "inside 8 lanes");
    const u64 o = row_xor_u64<J>(v);
    unsigned m  = 0;
    for (int i = 0; i < 16; ++i)
        if (i & J) m |= 1u << i;
    const u64 kMax  = rows4(m);
    const u64 lt    = __builtin_amdgcn_ballot_w64(o < v);
    const bool take = __builtin_amdgcn_inverse_ballot_w64(lt ^ kMax);
    return take ? o : v;
}

// ascending sort of the 8 keys of each half row (the 2- and 4-stages of the sort of 16 already treat the halves alike)
__device__ __forceinline__ u64 half_sort8(u64 v)
{
    v = bitonic_step<2, 1>(v);
    v = bitonic_step<4, 2>(v);
    v = bitonic_step<4, 1>(v);
    v = bitonic_step_half_ascending<4>(v);
    v = bitonic_step_half_ascending<2>(v);
    v = bitonic_step_half_ascending<1>(v);
    return v;
}

// ---- and into four lists of 4 lanes (the DPP quads) ----
// ascending sort of the 4 keys of each quad
__device__ __forceinline__ u64 quad_sort4(u64 v)
{
    v = bitonic_step<2, 1>(v);
    v = bitonic_step_half_ascending<2>(v);
    v = bitonic_step_half_ascending<1>(v);
    return v;
}

// sum over each quad, valid in its lane 0; the first two steps of row_sum_to_lane0
__device__ __forceinline__ float quad_sum_to_lane0(float v)
{
    v = v + dpp_f<kDppXor1>(v);
    v = v + dpp_f<kDppXor2>(v);
    return v;
}

// sum over each half row, valid in its lane 0; same pairing as row_sum_to_lane0 without the last step
__device__ __forceinline__ float half_sum_to_lane0(float v)
{
    v = v + dpp_f<kDppXor1>(v);
    v = v + dpp_f<kDppXor2>(v);
    v = v + dpp_f<kDppHalfMirror>(v);
    return v;
}

// lane i reads lane i-1 of the row; lane 0 of the row reads `fill`
__device__ __forceinline__ float row_shr1(float v, float fill)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(v), kDppShr1, 0xf, 0xf, false));
}

// lane i reads lane i-S of the row; the first S lanes of the row read `fill`
template <int S>
__device__ __forceinline__ float row_shr(float v, float fill)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(v), 0x110 + S, 0xf, 0xf, false));
}

// lane i reads lane i+S of the row; lanes past the end read 0
template <int S>
__device__ __forceinline__ float row_shl0(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x100 + S, 0xf, 0xf, true));
}

// Sum over the row, valid in lane 0 of the row (other lanes hold partial sums). The additions pair up as the
// butterfly (0+1)+(2+3), ... does, which is the order the colour of a pixel is accumulated in.
__device__ __forceinline__ float row_sum_to_lane0(float v)
{
    v = v + dpp_f<kDppXor1>(v);
    v = v + dpp_f<kDppXor2>(v);
    v = v + dpp_f<kDppHalfMirror>(v);  // every lane of a quad holds the quad sum: lane 0 adds lane 7 = quad 1
    v = v + dpp_f<kDppMirror>(v);      // lane 0 adds lane 15 = upper half
    return v;
}

// exclusive product chain: lane j gets prod_{k<j} f_k, multiplied left to right (lane 0 gets 1).
// `steps` (wave-uniform, 1..16) = number of leading row positions whose result is needed.
__device__ __forceinline__ float row_exclusive_product(float f, int steps)
{
    float pre = 1.f, T = 1.f;
    u64 latch = rows4(1u << 1);
    for (int s = 1; s < steps; ++s)
    {
        pre = row_shr1(pre * f, 1.f);
        T   = __builtin_amdgcn_inverse_ballot_w64(latch) ? pre : T;  // position s latches its product
        latch <<= 1;
    }
    return T;
}

// the same per half row (steps 1..8): positions 0 and 8 of a row start a chain
__device__ __forceinline__ float half_exclusive_product(float f, int steps)
{
    float pre = 1.f, T = 1.f;
    u64 latch = rows4((1u << 1) | (1u << 9));
    constexpr u64 kFirst = rows4(0x0101u);
    for (int s = 1; s < steps; ++s)
    {
        pre = row_shr1(pre * f, 1.f);
        pre = __builtin_amdgcn_inverse_ballot_w64(kFirst) ? 1.f : pre;  // position 8 must not see position 7
        T   = __builtin_amdgcn_inverse_ballot_w64(latch) ? pre : T;
        latch <<= 1;
    }
    return T;
}

// the same per quad (steps 1..4)
__device__ __forceinline__ float quad_exclusive_product(float f, int steps)
{
    float pre = 1.f, T = 1.f;
    u64 latch = rows4(0x2222u);
    constexpr u64 kFirst = rows4(0x1111u);
    for (int s = 1; s < steps; ++s)
    {
        pre = row_shr1(pre * f, 1.f);
        pre = __builtin_amdgcn_inverse_ballot_w64(kFirst) ? 1.f : pre;  // a quad's first position must not see the quad before
        T   = __builtin_amdgcn_inverse_ballot_w64(latch) ? pre : T;
        latch <<= 1;
    }
    return T;
}

// exclusive suffix sum: lane j gets sum_{i>j} v_i
__device__ __forceinline__ float row_exclusive_suffix_sum(float v)
{
    float s = row_shl0<1>(v);
    s += row_shl0<1>(s);
    s += row_shl0<2>(s);
    s += row_shl0<4>(s);
    s += row_shl0<8>(s);
    return s;
}

// the same per half row
__device__ __forceinline__ float half_exclusive_suffix_sum(float v)
{
    // positions whose source (i + S) lies in the same half: S = 1 -> all but 7 and 15, S = 2 -> 0..5 and 8..13,
    // S = 4 -> 0..3 and 8..11
    constexpr u64 k1 = rows4(0x7F7Fu), k2 = rows4(0x3F3Fu), k4 = rows4(0x0F0Fu);
    float t = row_shl0<1>(v);
    float s = __builtin_amdgcn_inverse_ballot_w64(k1) ? t : 0.f;
    t       = row_shl0<1>(s);
    s += __builtin_amdgcn_inverse_ballot_w64(k1) ? t : 0.f;
    t = row_shl0<2>(s);
    s += __builtin_amdgcn_inverse_ballot_w64(k2) ? t : 0.f;
    t = row_shl0<4>(s);
    s += __builtin_amdgcn_inverse_ballot_w64(k4) ? t : 0.f;
    return s;
}

}  // namespace trips
