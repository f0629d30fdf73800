// Device-side building blocks shared by the QVB8 kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qvb8 {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr int kFieldsPerLane = 32;                     // a lane owns 32 consecutive ids of a row = NB dwords
constexpr int kChunk = kWave * kFieldsPerLane;         // 2048 columns per wave pass
constexpr int kMaxFastNb = 8;                          // widths 4..8 take the dword-sliced path

// ---- number formats ---------------------------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {      // round to nearest even, NaN kept quiet
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x0040u;
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
    _Float16 h = (_Float16)f;                                         // v_cvt_f16_f32, round to nearest even
    return (uint32_t)__builtin_bit_cast(uint16_t, h);
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
}

// Activation narrowing: clamp to fp16's finite range, then round; NaN passes through (comparisons, not min/max).
__device__ __forceinline__ uint32_t sat_half_bits(float v) {
    v = v > 65504.0f ? 65504.0f : (v < -65504.0f ? -65504.0f : v);
    return f32_to_f16_bits(v);
}

template <int DT> __device__ __forceinline__ float load_as_f32(const void* p, int64_t i);
template <> __device__ __forceinline__ float load_as_f32<0>(const void* p, int64_t i) { return ((const float*)p)[i]; }
template <> __device__ __forceinline__ float load_as_f32<1>(const void* p, int64_t i) {
    return f16_bits_to_f32(((const uint16_t*)p)[i]);
}
template <> __device__ __forceinline__ float load_as_f32<2>(const void* p, int64_t i) {
    return bf16_bits_to_f32(((const uint16_t*)p)[i]);
}
__device__ __forceinline__ float load_as_f32(const void* p, int64_t i, int dt) {
    return dt == 0 ? load_as_f32<0>(p, i) : dt == 1 ? load_as_f32<1>(p, i) : load_as_f32<2>(p, i);
}

template <int DT> __device__ __forceinline__ void store_from_f32(void* p, int64_t i, float v);
template <> __device__ __forceinline__ void store_from_f32<0>(void* p, int64_t i, float v) { ((float*)p)[i] = v; }
template <> __device__ __forceinline__ void store_from_f32<1>(void* p, int64_t i, float v) {
    ((uint16_t*)p)[i] = (uint16_t)f32_to_f16_bits(v);
}
template <> __device__ __forceinline__ void store_from_f32<2>(void* p, int64_t i, float v) {
    ((uint16_t*)p)[i] = (uint16_t)f32_to_bf16_bits(v);
}

// ---- packed ids -------------------------------------------------------------------------------------------
// One id of width nb at absolute bit position `bit`: two aligned dwords and a 64-bit shift.  Touches bytes up to
// (bit >> 3) + 7, which the 8 pad bytes after the payload cover; `last_dword` (byte offset of the last whole
// dword of the buffer minus 4) clamps the address so that inconsistent metadata can never read outside `ids`.
__device__ __forceinline__ uint32_t load_field(const uint8_t* __restrict__ ids, int64_t bit, int nb, int64_t clamp_byte) {
    int64_t a = (bit >> 3) & ~(int64_t)3;
    a = a > clamp_byte ? clamp_byte : a;
    const uint32_t* p = reinterpret_cast<const uint32_t*>(ids + a);
    const uint64_t v = (uint64_t)p[0] | ((uint64_t)p[1] << 32);
    const uint32_t sh = (uint32_t)(bit - a * 8) & 63u;
    return (uint32_t)(v >> sh) & ((1u << nb) - 1u);
}

// Field J (NB bits) of a lane's NB-dword slice, every shift a compile-time constant.
template <int NB, int J>
__device__ __forceinline__ uint32_t field_of(const uint32_t (&w)[kMaxFastNb]) {
    constexpr int bit = J * NB, d = bit >> 5, s = bit & 31;
    constexpr uint32_t mask = (1u << NB) - 1u;
    if constexpr (s + NB <= 32) return __builtin_amdgcn_ubfe(w[d], s, NB);
    else return __builtin_amdgcn_alignbit(w[d + 1], w[d], s) & mask;
}

// The three steps of turning two adjacent ids into a biased fp16 pair are written as single instructions: left
// to itself the compiler splits the 2*NB-bit extract into two masked halves and spends one to two more
// operations per pair.
template <int S, int W>
__device__ __forceinline__ uint32_t bfe_const(uint32_t w) {
    uint32_t r;
    asm("v_bfe_u32 %0, %1, %2, %3" : "=v"(r) : "v"(w), "n"(S), "n"(W));
    return r;
}
template <int SH>
__device__ __forceinline__ uint32_t shl_or_self(uint32_t e) {      // (e << SH) | e
    uint32_t r;
    asm("v_lshl_or_b32 %0, %1, %2, %1" : "=v"(r) : "v"(e), "n"(SH));
    return r;
}
__device__ __forceinline__ uint32_t and_or(uint32_t t, uint32_t mask, uint32_t bias) {   // (t & mask) | bias
    uint32_t r;
    asm("v_bitop3_b32 %0, %1, %2, %3 bitop3:0xea" : "=v"(r) : "v"(t), "v"(mask), "v"(bias));
    return r;
}

// Ids 2*PR and 2*PR+1 of the lane's slice as a | b << 16, plus bits the caller masks off (a << (16-NB) below
// bit 16).
template <int NB, int PR>
__device__ __forceinline__ uint32_t pair_of(const uint32_t (&w)[kMaxFastNb]) {
    constexpr int bit = PR * 2 * NB, d = bit >> 5, s = bit & 31, W = 2 * NB;
    uint32_t e;
    if constexpr (s + W <= 32) e = bfe_const<s, W>(w[d]);
    else e = __builtin_amdgcn_alignbit(w[d + 1], w[d], s) & ((1u << W) - 1u);
    return shl_or_self<16 - NB>(e);
}

// The lane's NB dwords, 4-byte aligned.
template <int NB>
__device__ __forceinline__ void load_slice(const uint32_t* __restrict__ p, uint32_t (&w)[kMaxFastNb]) {
#pragma unroll
    for (int k = 0; k < NB; ++k) w[k] = p[k];
}

// ---- wave64 sum -------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true);
    return v + __int_as_float(moved);
}

// Sum over the 64 lanes, same value returned to every lane.  Fixed order: bit-reproducible.
__device__ __forceinline__ float wave_sum(float v) {
    v = dpp_add<0xB1>(v);     // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);     // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);    // row_half_mirror
    v = dpp_add<0x140>(v);    // row_mirror: every lane of a 16-lane row holds the row sum
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (r0 + r1) + (r2 + r3);
}

}  // namespace qvb8
