// Device pieces shared by the matrix-core kernels (the tile kernel, the decode + GEMM kernel, the one-token MoE
// kernels): operand formats, the way activations are read, and the decode of a lane's 32-id slice into MFMA operands.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "qvb8_device.h"

namespace qvb8 {

typedef _Float16 v8h_t __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf_t __attribute__((ext_vector_type(8)));
typedef float v4f_t __attribute__((ext_vector_type(4)));
typedef uint32_t v4u_t __attribute__((ext_vector_type(4)));
typedef float v16f_t __attribute__((ext_vector_type(16)));

constexpr int kTileRows = 16;
constexpr int kStepCols = 128;          // columns one wave step covers (4 lane groups x 32 ids)

template <bool BF> struct Fmt;
template <> struct Fmt<false> {          // fp16: 0x6400 | id == 1024 + id for id < 1024
    static constexpr uint32_t bias_bits = 0x64006400u, one_bits = 0x3C003C00u;
    static constexpr float bias = 1024.0f;
    static constexpr int max_nb = 8;
    static __device__ __forceinline__ v4f_t mfma(const v4u_t& a, const v4u_t& b, const v4f_t& c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h_t, a), __builtin_bit_cast(v8h_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ v16f_t mfma32(const v4u_t& a, const v4u_t& b, const v16f_t& c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h_t, a), __builtin_bit_cast(v8h_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(uint32_t h) { return f16_bits_to_f32(h); }
};
template <> struct Fmt<true> {           // bf16: 0x4300 | id == 128 + id for id < 128
    static constexpr uint32_t bias_bits = 0x43004300u, one_bits = 0x3F803F80u;
    static constexpr float bias = 128.0f;
    static constexpr int max_nb = 7;
    static __device__ __forceinline__ v4f_t mfma(const v4u_t& a, const v4u_t& b, const v4f_t& c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf_t, a), __builtin_bit_cast(v8bf_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ v16f_t mfma32(const v4u_t& a, const v4u_t& b, const v16f_t& c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf_t, a), __builtin_bit_cast(v8bf_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(uint32_t h) { return bf16_bits_to_f32(h); }
};

// How the kernels read an activation.  XC = false: X is already in the operand format (fp16 for Fmt<false>, bf16 for
// Fmt<true>).  XC = true (fp16 operands only): X is bf16 in memory and is narrowed on the way in exactly as
// saturating_half does it -- clamp to +-65504, round to fp16, NaN kept -- so a bf16 caller gets what the fp16 paths of
// the reference multiply without a separate pass over X.
template <bool BF, bool XC> struct XIn {
    static __device__ __forceinline__ float scalar(uint32_t bits) {
        if constexpr (XC) return f16_bits_to_f32(sat_half_bits(bf16_bits_to_f32(bits)));
        else return Fmt<BF>::to_f32(bits);
    }
    // Two activations in one dword.  Round first (v_cvt_pk_f16_f32, nearest even; beyond 65520 gives infinity), clamp
    // after with the NaN-propagating packed minimum / maximum: the same value as clamping first, in five instructions.
    static __device__ __forceinline__ uint32_t pair(uint32_t w) {
        if constexpr (XC) {
            typedef float v2f_t __attribute__((ext_vector_type(2)));
            typedef _Float16 v2h_t __attribute__((ext_vector_type(2)));
            const v2f_t f = {__uint_as_float(w << 16), __uint_as_float(w & 0xFFFF0000u)};
            v2h_t h = __builtin_convertvector(f, v2h_t);
            const v2h_t top = {(_Float16)65504.0f, (_Float16)65504.0f};
            h = __builtin_elementwise_minimum(h, top);
            h = __builtin_elementwise_maximum(h, -top);
            return __builtin_bit_cast(uint32_t, h);
        } else {
            return w;
        }
    }
};

// the 16 pairs of a lane's slice -> 4 operand registers for each of the 4 MFMA steps, stage by stage: all
// extracts, then all spreads, then all mask-and-bias steps, so that no instruction waits for its predecessor
template <int NB, int PR>
__device__ __forceinline__ void stage_extract(const uint32_t (&w)[kMaxFastNb], uint32_t (&e)[16]) {
    if constexpr (PR < 16) { e[PR] = pair_extract<NB, PR>(w); stage_extract<NB, PR + 1>(w, e); }
}
template <int NB, int PR>
__device__ __forceinline__ void stage_spread(uint32_t (&e)[16]) {
    if constexpr (PR < 16) { e[PR] = pair_spread<NB, PR>(e[PR]); stage_spread<NB, PR + 1>(e); }
}

template <int NB>
__device__ __forceinline__ void slice_pairs(const uint4& lo, const uint4& hi, uint32_t (&e)[16]) {
    const uint32_t l[4] = {lo.x, lo.y, lo.z, lo.w}, h[4] = {hi.x, hi.y, hi.z, hi.w};
    uint32_t w[kMaxFastNb];
#pragma unroll
    for (int k = 0; k < 4; ++k) w[k] = l[k];
#pragma unroll
    for (int k = 4; k < NB; ++k) w[k] = h[k - (NB - 4)];
    stage_extract<NB, 0>(w, e);
    stage_spread<NB, 0>(e);
}

template <int NB, bool BF>
__device__ __forceinline__ void decode_slice(const uint4& lo, const uint4& hi, v4u_t (&b)[4]) {
    constexpr int KEEP = (BF && NB > 7) ? 7 : NB;            // bf16 holds 7 id bits next to the bias
    constexpr uint32_t mask = ((1u << KEEP) - 1u) * 0x00010001u;
    uint32_t e[16];
    slice_pairs<NB>(lo, hi, e);
    // the two constants as registers (opaque to constant folding): the last step is then ONE v_and_or_b32 per pair, a
    // real instruction of the compiler's, so that it keeps the wait states the matrix instruction needs after it
    uint32_t m = mask, bias = Fmt<BF>::bias_bits;
    asm("" : "+v"(m), "+v"(bias));
#pragma unroll
    for (int p = 0; p < 16; ++p) b[p / 4][p % 4] = and_or3(e[p], m, bias);
}

// the value lane l + O of the same row of sixteen lanes holds (zero past the row's end): DPP row_shl, no trip to LDS
template <int O>
__device__ __forceinline__ double row16_from(double v) {
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)b, 0x100 + O, 0xF, 0xF, true);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(b >> 32), 0x100 + O, 0xF, 0xF, true);
    return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}
// the sum of a value over the sixteen lanes of a row, as a fixed tree (0+8)+(4+12)...: valid in the row's first lane
__device__ __forceinline__ double row16_sum(double v) {
    v += row16_from<8>(v);
    v += row16_from<4>(v);
    v += row16_from<2>(v);
    v += row16_from<1>(v);
    return v;
}

}  // namespace qvb8
