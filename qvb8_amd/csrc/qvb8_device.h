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
    // The fp32 value is rounded to fp16 as a step of its own: without the empty statement the compiler folds a preceding
    // fused multiply-add into v_fma_mixlo_f16, which rounds the exact sum ONCE to fp16 and differs from
    // fp16(fp32 result) where the fp32 rounding lands on an fp16 tie (about one value in 10^5).
    asm("" : "+v"(f));
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

// ---- rows stored in planes ------------------------------------------------------------------------------------
// A loader may store a 16-row tile of ONE width nb (4..8, P a multiple of 128) so that every request instruction of a
// wave reads one contiguous run: per 128-column step first plane A -- the first four dwords of every lane's slice, lane
// l = row + 16 * (column group of 32 within the step), 64 x 16 bytes -- then plane B, the remaining nb - 4 dwords of every
// lane, 64 x 4 (nb - 4) bytes.  A step takes 256 nb bytes and a tile n_steps x 256 nb = 16 rows' worth: the same bytes
// as 16 rows stored back to back, permuted inside the tile.  Such a row is marked in its bit offset:
//   bit 62 set, bits 0..47 = bit offset of the TILE's first byte, bits 48..51 = the row's number inside the tile.
constexpr int64_t kPlaneFlag = (int64_t)1 << 62;
constexpr int64_t kOffBitsMask = ((int64_t)1 << 48) - 1;
__host__ __device__ __forceinline__ bool off_is_plane(int64_t off) { return (off & kPlaneFlag) != 0; }
__host__ __device__ __forceinline__ int off_plane_row(int64_t off) { return (int)((off >> 48) & 15); }
// byte offset (from the tile's first byte) of dword d of the 32-id slice `cg` (column group of 32) of row r
__host__ __device__ __forceinline__ uint64_t plane_dword_at(int r, uint32_t nb, int cg, int d) {
    const uint64_t sb = (uint64_t)(cg >> 2) * (256u * nb);
    const uint32_t lane = (uint32_t)r + 16u * (uint32_t)(cg & 3);
    return d < 4 ? sb + lane * 16u + 4u * (uint32_t)d : sb + 1024u + lane * (4u * (nb - 4u)) + 4u * (uint32_t)(d - 4);
}
// One id of a row stored in planes (any column): at most two dwords.
__device__ __forceinline__ uint32_t plane_field(const uint8_t* __restrict__ ids, uint64_t tile_byte, int r, int nb, int col) {
    const int cg = col >> 5, bit = (col & 31) * nb, d = bit >> 5, sh = bit & 31;
    uint32_t v = *reinterpret_cast<const uint32_t*>(ids + tile_byte + plane_dword_at(r, (uint32_t)nb, cg, d)) >> sh;
    if (sh + nb > 32) v |= *reinterpret_cast<const uint32_t*>(ids + tile_byte + plane_dword_at(r, (uint32_t)nb, cg, d + 1)) << (32 - sh);
    return v & ((1u << nb) - 1u);
}
// One id of a row, however it is stored.  `off` = the row's bit offset word; in bounds by the caller's check.
__device__ __forceinline__ uint32_t row_field(const uint8_t* __restrict__ ids, int64_t off, int nb, int col, int64_t clamp_byte) {
    if (off_is_plane(off)) return plane_field(ids, (uint64_t)((off & kOffBitsMask) >> 3), off_plane_row(off), nb, col);
    return load_field(ids, off + (int64_t)col * nb, nb, clamp_byte);
}
// Whether the bytes a row's metadata points at lie inside the buffer (with the 8 pad bytes behind the payload).
__host__ __device__ __forceinline__ bool row_in_bounds(int64_t off, int nb, int64_t P, int64_t ids_bytes) {
    if (nb < 1 || nb > 14 || off < 0) return false;
    if (off_is_plane(off)) {
        const int64_t t0 = (off & kOffBitsMask) >> 3;
        return nb >= 4 && nb <= 8 && (P & 127) == 0 && (t0 & 3) == 0 && t0 + 2 * P * nb + 8 <= ids_bytes;     // 16 rows
    }
    return off < kOffBitsMask && ((off + (int64_t)nb * P + 7) >> 3) + 8 <= ids_bytes;
}
// The lane's NB dwords of slice `cg` of a row stored in planes.
template <int NB>
__device__ __forceinline__ void load_slice_planes(const uint8_t* __restrict__ ids, uint64_t tile_byte, int r, int cg, uint32_t (&w)[kMaxFastNb]) {
    const uint4 a = *reinterpret_cast<const uint4*>(ids + tile_byte + plane_dword_at(r, NB, cg, 0));
    w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w;
#pragma unroll
    for (int k = 4; k < NB; ++k) w[k] = *reinterpret_cast<const uint32_t*>(ids + tile_byte + plane_dword_at(r, NB, cg, k));
}

// Field J (NB bits) of a lane's NB-dword slice, every shift a compile-time constant.
template <int NB, int J>
__device__ __forceinline__ uint32_t field_of(const uint32_t (&w)[kMaxFastNb]) {
    constexpr int bit = J * NB, d = bit >> 5, s = bit & 31;
    constexpr uint32_t mask = (1u << NB) - 1u;
    if constexpr (s + NB <= 32) return __builtin_amdgcn_ubfe(w[d], s, NB);
    else return __builtin_amdgcn_alignbit(w[d + 1], w[d], s) & mask;
}

// Ids 2*PR and 2*PR+1 of a lane's slice as an fp16 pair with each id in the low mantissa bits of `bias`:
//   e = bits [2*PR*NB, +2*NB) of the slice          v_bfe_u32, or v_alignbit_b32 + v_and_b32 across a dword edge
//   t = (e << (16 - NB)) | e                        v_lshl_or_b32: the second id lands on bit 16
//   r = (t & mask) | bias                           v_bitop3_b32
// Written as one instruction sequence: left to itself the compiler splits the 2*NB-bit extract into two masked
// halves and spends one to two more operations per pair.
template <int NB, int PR>
__device__ __forceinline__ uint32_t pair_bits(const uint32_t (&w)[kMaxFastNb], uint32_t mask, uint32_t bias) {
    constexpr int bit = PR * 2 * NB, d = bit >> 5, s = bit & 31, W = 2 * NB;
    uint32_t r;
    if constexpr (s + W <= 32) {
        asm("v_bfe_u32 %0, %1, %4, %5\n\t"
            "v_lshl_or_b32 %0, %0, %6, %0\n\t"
            "v_bitop3_b32 %0, %0, %2, %3 bitop3:0xea"
            : "=&v"(r) : "v"(w[d]), "v"(mask), "v"(bias), "n"(s), "n"(W), "n"(16 - NB));
    } else {
        asm("v_alignbit_b32 %0, %2, %1, %5\n\t"
            "v_and_b32 %0, %6, %0\n\t"
            "v_lshl_or_b32 %0, %0, %7, %0\n\t"
            "v_bitop3_b32 %0, %0, %3, %4 bitop3:0xea"
            : "=&v"(r) : "v"(w[d]), "v"(w[d + 1]), "v"(mask), "v"(bias), "n"(s), "n"((1 << W) - 1), "n"(16 - NB));
    }
    return r;
}

// The same three steps as single instructions, for callers that want to interleave many pairs (stage by stage)
// so that dependent instructions are far apart in the instruction stream.
template <int NB, int PR>
__device__ __forceinline__ uint32_t pair_extract(const uint32_t (&w)[kMaxFastNb]) {      // e = 2*NB bits at pair PR
    constexpr int bit = PR * 2 * NB, d = bit >> 5, s = bit & 31, W = 2 * NB;
    uint32_t r;
    if constexpr (s + W <= 32) {
        asm("v_bfe_u32 %0, %1, %2, %3" : "=v"(r) : "v"(w[d]), "n"(s), "n"(W));
    } else {
        asm("v_alignbit_b32 %0, %2, %1, %3" : "=v"(r) : "v"(w[d]), "v"(w[d + 1]), "n"(s));
    }
    return r;
}
template <int NB, int PR>
__device__ __forceinline__ uint32_t pair_spread(uint32_t e) {                          // (e << (16-NB)) | e, e cleaned first if needed
    constexpr int bit = PR * 2 * NB, s = bit & 31, W = 2 * NB;
    uint32_t r;
    if constexpr (s + W <= 32) {
        asm("v_lshl_or_b32 %0, %1, %2, %1" : "=v"(r) : "v"(e), "n"(16 - NB));
    } else {
        // the window came from v_alignbit_b32 and still has bits above 2*NB: shifting it left by 16-NB puts id b on
        // bit 16 and pushes the junk above bit 16+NB, OR-ing the unshifted copy adds id a at bit 0 plus junk at
        // bits >= NB; everything outside the two id fields is removed by the mask of the final step, except bits
        // 16..16+NB-1 of the unshifted copy, which must be cleared here
        asm("v_and_b32 %0, %2, %1\n\tv_lshl_or_b32 %0, %0, %3, %0" : "=&v"(r) : "v"(e), "n"((1 << W) - 1), "n"(16 - NB));
    }
    return r;
}
// Written in C on purpose: the result is an MFMA operand, and the compiler keeps the wait states between a vector
// instruction's write and the matrix instruction that reads it only for instructions it can see.  As an inline-asm
// instruction the same operation was invisible to that check: an operand written two instructions before its MFMA was
// read stale (measured: the register's previous contents entered the product).
__device__ __forceinline__ uint32_t and_or3(uint32_t t, uint32_t mask, uint32_t bias) {   // (t & mask) | bias: v_and_or_b32
    return (t & mask) | bias;
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

// Sums of four values per lane over the 64 lanes at once: on return lane j (j < 4) holds the total of v[j].
// Two select-and-exchange steps leave lane l with the quad sum of v[l & 3]; the quads of a 16-lane row are
// combined with row rotations, the four rows with two cross-lane reads.  Fixed order: bit-reproducible.
__device__ __forceinline__ float wave_sum4(const float (&v)[4], int lane) {
    const bool b0 = lane & 1, b1 = lane & 2;
    const float k01 = b0 ? v[1] : v[0], s01 = b0 ? v[0] : v[1];
    const float k23 = b0 ? v[3] : v[2], s23 = b0 ? v[2] : v[3];
    const float r01 = k01 + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(s01), 0xB1, 0xF, 0xF, true));
    const float r23 = k23 + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(s23), 0xB1, 0xF, 0xF, true));
    const float kk = b1 ? r23 : r01, ss = b1 ? r01 : r23;
    float r = kk + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(ss), 0x4E, 0xF, 0xF, true));
    r += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(r), 0x124, 0xF, 0xF, true));   // row_ror:4
    r += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(r), 0x128, 0xF, 0xF, true));   // row_ror:8
    r += __int_as_float(__builtin_amdgcn_ds_bpermute((lane ^ 16) << 2, __float_as_int(r)));
    r += __int_as_float(__builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __float_as_int(r)));
    return r;
}

}  // namespace qvb8
