// QVB8 kernels for gfx950: dense restore, certificate check, activation narrowing, fused decode + GEMV (M = 1..8).
//
// Work decomposition common to the restore and the GEMV: an ITEM is one row x one chunk of 2048 columns, handled
// by one 64-lane wave; lane l owns the 32 consecutive ids at columns chunk*2048 + 32*l, which are exactly NB
// dwords of the row (32 ids * NB bits), dword aligned whenever the row itself starts on a dword (true for every
// row of a pack with P % 32 == 0).  The wave therefore reads a contiguous NB*256-byte span per item, the lane
// slices its ids with compile-time shifts, and nothing is exchanged between lanes until the final sum.
// Rows that do not fit that pattern (P % 32 != 0, a row starting off a dword, widths outside 4..8) take a
// per-element path inside the same kernel: any width 1..14, any bit offset.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string>

#include "../../include/qvb8_amd.h"
#include "qvb8_device.h"
#include "qvb8_host.h"

namespace qvb8 {

// ===========================================================================================================
// dense restore
// ===========================================================================================================
template <int DT> struct OutPack;     // 32 values of a lane -> vector stores
template <> struct OutPack<0> {
    static __device__ __forceinline__ void store(void* out, int64_t i, const float (&v)[32]) {
        float4* o = reinterpret_cast<float4*>((float*)out + i);
#pragma unroll
        for (int k = 0; k < 8; ++k) o[k] = make_float4(v[4 * k], v[4 * k + 1], v[4 * k + 2], v[4 * k + 3]);
    }
};
template <> struct OutPack<1> {
    static __device__ __forceinline__ void store(void* out, int64_t i, const float (&v)[32]) {
        uint4* o = reinterpret_cast<uint4*>((uint16_t*)out + i);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                w[j] = f32_to_f16_bits(v[8 * k + 2 * j]) | (f32_to_f16_bits(v[8 * k + 2 * j + 1]) << 16);
            o[k] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
};
template <> struct OutPack<2> {
    static __device__ __forceinline__ void store(void* out, int64_t i, const float (&v)[32]) {
        uint4* o = reinterpret_cast<uint4*>((uint16_t*)out + i);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                w[j] = f32_to_bf16_bits(v[8 * k + 2 * j]) | (f32_to_bf16_bits(v[8 * k + 2 * j + 1]) << 16);
            o[k] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
};

// FMA: the value of a linear layer's weight, fmaf(id, tau_s, min_s) (one rounding).  !FMA: the value the embedding
// lookup of the reference computes, min_s + id * tau_s as two fp32 operations (two roundings).
template <bool FMA>
__device__ __forceinline__ float band_value(uint32_t id, float ts, float m) {
#pragma clang fp contract(off)                  // the two-step form must stay a multiply and an add
    if constexpr (FMA) return __builtin_fmaf((float)id, ts, m);
    else { const float prod = (float)id * ts; return m + prod; }
}

template <int NB, bool FMA, int J0, int J1>
__device__ __forceinline__ void restore_fields(const uint32_t (&w)[kMaxFastNb], float ts, float m, float (&v)[32]) {
    if constexpr (J0 < J1) {
        v[J0] = band_value<FMA>(field_of<NB, J0>(w), ts, m);
        restore_fields<NB, FMA, J0 + 1, J1>(w, ts, m, v);
    }
}

template <int DT, int NB, bool FMA>
__device__ __forceinline__ void restore_item_fast(const uint8_t* __restrict__ ids, int64_t row_byte, int slice,
                                                  float ts, float m, void* out, int64_t out_index) {
    uint32_t w[kMaxFastNb];
    load_slice<NB>(reinterpret_cast<const uint32_t*>(ids + row_byte) + (int64_t)slice * NB, w);
    float v[32];
    restore_fields<NB, FMA, 0, 32>(w, ts, m, v);
    OutPack<DT>::store(out, out_index, v);
}

struct DecodeArgs {
    const uint8_t* ids; const float* min_s; const float* tau_s; const uint8_t* nbits; const int64_t* bit_off;
    void* out; int64_t ids_bytes; int64_t n_items; int Q; int P; int C;
    // row lookup only: the rows wanted (output row i is row rows[i] of the pack) and the escapes of the whole pack
    const int64_t* rows; const int64_t* esc_idx; const float* esc_vals; int64_t n_esc;
};

// One wave per item; 4 waves per workgroup.  LOOKUP: output row i is row rows[i] of the pack (any order, repeats allowed;
// a row number outside 0..Q-1 gives a row of NaN), values are min_s + id * tau_s in two roundings, and the escapes of
// the row overwrite the band values (a binary search of the ascending flat positions finds the item's range).
template <int DT, bool LOOKUP>
__global__ void __launch_bounds__(256) decode_kernel(DecodeArgs a) {
    constexpr bool FMA = !LOOKUP;
    const int lane = threadIdx.x & 63;
    const int64_t item = (int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (item >= a.n_items) return;
    const int64_t orow = item / a.C;
    const int c = (int)(item - orow * a.C);
    int64_t q64 = orow;
    if constexpr (LOOKUP) q64 = a.rows[orow];
    const bool row_ok = q64 >= 0 && q64 < a.Q;
    const int q = row_ok ? (int)q64 : 0;
    const int nb = __builtin_amdgcn_readfirstlane((int)a.nbits[q]);
    const int64_t bit0 = a.bit_off[q];
    const float ts = a.tau_s[q], m = a.min_s[q];
    const int col0 = c * kChunk;
    const int64_t clamp_byte = (a.ids_bytes - 8) & ~(int64_t)3;
    const bool in_bounds = row_ok && row_in_bounds(bit0, nb, a.P, a.ids_bytes);
    // the lane's 32 values go out as 16-byte stores: the output row must start on 16 bytes as well
    const bool planes = off_is_plane(bit0);
    const bool fast = in_bounds && !planes && (a.P % kFieldsPerLane) == 0 && (bit0 & 31) == 0 && nb >= 4 && nb <= kMaxFastNb;
    const int col_end = min(a.P, col0 + kChunk);
    if (in_bounds && planes) {
        // a row stored in planes: the lane's slice comes from two places of its tile
        const int col = col0 + lane * kFieldsPerLane;
        if (col < a.P) {
            const uint64_t tile_byte = (uint64_t)((bit0 & kOffBitsMask) >> 3);
            const int r = off_plane_row(bit0), cg = col / kFieldsPerLane;
            uint32_t w[kMaxFastNb];
            float v[32];
            switch (nb) {
                case 4: load_slice_planes<4>(a.ids, tile_byte, r, cg, w); restore_fields<4, FMA, 0, 32>(w, ts, m, v); break;
                case 5: load_slice_planes<5>(a.ids, tile_byte, r, cg, w); restore_fields<5, FMA, 0, 32>(w, ts, m, v); break;
                case 6: load_slice_planes<6>(a.ids, tile_byte, r, cg, w); restore_fields<6, FMA, 0, 32>(w, ts, m, v); break;
                case 7: load_slice_planes<7>(a.ids, tile_byte, r, cg, w); restore_fields<7, FMA, 0, 32>(w, ts, m, v); break;
                default: load_slice_planes<8>(a.ids, tile_byte, r, cg, w); restore_fields<8, FMA, 0, 32>(w, ts, m, v); break;
            }
            OutPack<DT>::store(a.out, orow * a.P + col, v);
        }
    } else if (fast) {
        const int col = col0 + lane * kFieldsPerLane;
        if (col < a.P) {
            const int64_t oi = orow * a.P + col;
            const int slice = col / kFieldsPerLane;
            switch (nb) {
                case 4: restore_item_fast<DT, 4, FMA>(a.ids, bit0 >> 3, slice, ts, m, a.out, oi); break;
                case 5: restore_item_fast<DT, 5, FMA>(a.ids, bit0 >> 3, slice, ts, m, a.out, oi); break;
                case 6: restore_item_fast<DT, 6, FMA>(a.ids, bit0 >> 3, slice, ts, m, a.out, oi); break;
                case 7: restore_item_fast<DT, 7, FMA>(a.ids, bit0 >> 3, slice, ts, m, a.out, oi); break;
                default: restore_item_fast<DT, 8, FMA>(a.ids, bit0 >> 3, slice, ts, m, a.out, oi); break;
            }
        }
    } else {
        for (int col = col0 + lane; col < col_end; col += kWave) {
            float v = __builtin_nanf("");
            if (in_bounds) v = band_value<FMA>(load_field(a.ids, bit0 + (int64_t)col * nb, nb, clamp_byte), ts, m);
            store_from_f32<DT>(a.out, orow * a.P + col, v);
        }
    }
    if constexpr (LOOKUP) {
        if (a.n_esc == 0 || !row_ok) return;
        const int64_t lo_pos = q64 * a.P + col0, hi_pos = q64 * a.P + col_end;
        int64_t lo = 0, hi = a.n_esc;                              // first escape at or after lo_pos
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (a.esc_idx[mid] < lo_pos) lo = mid + 1; else hi = mid;
        }
        if (lo >= a.n_esc || a.esc_idx[lo] >= hi_pos) return;
        // the band values of this item are the wave's own earlier stores: wait until all of them have been
        // acknowledged (vmcnt(0); the other counters stay unconstrained) before some are overwritten
        __builtin_amdgcn_s_waitcnt(0x0F70);
        for (int64_t e = lo + lane; e < a.n_esc; e += kWave) {
            const int64_t at = a.esc_idx[e];
            if (at >= hi_pos) break;
            store_from_f32<DT>(a.out, orow * a.P + (at - q64 * a.P), a.esc_vals[e]);
        }
    }
}

template <int DT>
__global__ void __launch_bounds__(256) scatter_escapes_kernel(void* out, int64_t n_out, const int64_t* __restrict__ idx,
                                                             const float* __restrict__ vals, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t at = idx[i];
    if (at >= 0 && at < n_out) store_from_f32<DT>(out, at, vals[i]);
}

// ===========================================================================================================
// certificate: max |restored - original| and the number of elements at or over tau
// ===========================================================================================================
__global__ void certify_init_kernel(uint32_t* result) {
    if (threadIdx.x < 2) result[threadIdx.x] = 0u;
}

__global__ void __launch_bounds__(256) certify_kernel(const void* __restrict__ a, int adt, const void* __restrict__ b, int bdt,
                                                      int64_t n, float tau, uint32_t* result) {
    float mx = 0.f;
    uint32_t bad = 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const float d = fabsf(load_as_f32(a, i, adt) - load_as_f32(b, i, bdt));
        if (!(d < tau)) ++bad;                       // also counts NaN / inf
        if (d == d) mx = fmaxf(mx, d);
        else mx = __builtin_inff();
    }
    // non-negative floats order like their bit patterns
    __shared__ uint32_t s_mx, s_bad;
    if (threadIdx.x == 0) { s_mx = 0; s_bad = 0; }
    __syncthreads();
    atomicMax(&s_mx, __float_as_uint(mx));
    if (bad) atomicAdd(&s_bad, bad);
    __syncthreads();
    if (threadIdx.x == 0) {
        atomicMax(&result[0], s_mx);
        if (s_bad) atomicAdd(&result[1], s_bad);
    }
}

// ===========================================================================================================
// activation narrowing
// ===========================================================================================================
template <int DT>
__global__ void __launch_bounds__(256) sat_half_kernel(const void* __restrict__ x, uint16_t* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = (uint16_t)sat_half_bits(load_as_f32<DT>(x, i));
}

template <int DT>
__global__ void __launch_bounds__(256) scale_sat_half_kernel(const void* __restrict__ x, float scale, uint16_t* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = (uint16_t)sat_half_bits(load_as_f32<DT>(x, i) * scale);
}

// ===========================================================================================================
// fused decode + GEMV, M = MB rows of X (1..8)
// ===========================================================================================================
// y[m][q] = tau_s[q] * sum_c x[m][c] * id[q][c] + min_s[q] * sum_c x[m][c]       (x = sat_half(X))
// The id sum runs on v_dot2_f32_f16: two ids are placed in the mantissas of an fp16 pair biased by 1024
// (0x6400 | id is exactly 1024 + id for id < 1024), multiplied with the fp16 pair of activations and accumulated
// in fp32; each lane removes its own bias term 1024 * sum(x) before the lanes are combined.
struct GemvArgs {
    const void* X; const uint8_t* ids; const float* min_s; const float* tau_s; const uint8_t* nbits;
    const int64_t* bit_off; float* Y; int64_t ids_bytes;
    int x_dtype; int Q; int P; int C;          // C = chunks of 2048 columns per row
    int W;                                     // waves of a workgroup that share a row (one chunk each per panel)
    int G;                                     // row groups per workgroup; waves = W * G
    int panels;                                // ceil(C / W)
    int RW;                                    // rows per workgroup (multiple of G)
};

constexpr float kBias = 1024.0f;
constexpr uint32_t kBiasBits = 0x64006400u;

template <int NB, int PR, int PR_END, int MB>
__device__ __forceinline__ void dot_pairs(const uint32_t (&w)[kMaxFastNb], const uint32_t (&xr)[MB][16], float (&acc)[MB][2],
                                          uint32_t mask, uint32_t bias) {
    if constexpr (PR < PR_END) {
        const uint32_t bits = pair_bits<NB, PR>(w, mask, bias);
        const half2_t wv = __builtin_bit_cast(half2_t, bits);
#pragma unroll
        for (int m = 0; m < MB; ++m)
            acc[m][PR & 1] = __builtin_amdgcn_fdot2(wv, __builtin_bit_cast(half2_t, xr[m][PR]), acc[m][PR & 1], false);
        dot_pairs<NB, PR + 1, PR_END, MB>(w, xr, acc, mask, bias);
    }
}

// A lane's slice is NB dwords.  It is fetched as two 16-byte loads whatever NB is: dwords [0, 4) and the LAST
// four dwords [NB-4, NB) (they overlap for NB < 8), so every row costs the same two in-bounds load
// instructions and the wait counters of the prefetch pipeline stay exact.
template <int NB, int MB>
__device__ __forceinline__ void gemv_item_fast(const uint4& lo, const uint4& hi, const uint32_t (&xr)[MB][16],
                                               const float (&sx)[MB], float (&d)[MB]) {
    const uint32_t l[4] = {lo.x, lo.y, lo.z, lo.w}, h[4] = {hi.x, hi.y, hi.z, hi.w};
    uint32_t w[kMaxFastNb];
#pragma unroll
    for (int k = 0; k < 4; ++k) w[k] = l[k];
#pragma unroll
    for (int k = 4; k < NB; ++k) w[k] = h[k - (NB - 4)];
    float acc[MB][2];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m][0] = acc[m][1] = 0.f;
    constexpr uint32_t mask = ((1u << NB) - 1u) * 0x00010001u;
    dot_pairs<NB, 0, 16, MB>(w, xr, acc, mask, kBiasBits);
#pragma unroll
    for (int m = 0; m < MB; ++m) d[m] = __builtin_fmaf(-kBias, sx[m], acc[m][0] + acc[m][1]);
}

template <int MB>
__device__ __forceinline__ void gemv_compute_fast(int nb, const uint4& lo, const uint4& hi, const uint32_t (&xr)[MB][16],
                                                  const float (&sx)[MB], float (&d)[MB]) {
    switch (nb) {
        case 4: gemv_item_fast<4, MB>(lo, hi, xr, sx, d); break;
        case 5: gemv_item_fast<5, MB>(lo, hi, xr, sx, d); break;
        case 6: gemv_item_fast<6, MB>(lo, hi, xr, sx, d); break;
        case 7: gemv_item_fast<7, MB>(lo, hi, xr, sx, d); break;
        default: gemv_item_fast<8, MB>(lo, hi, xr, sx, d); break;
    }
}

// kind of a row for the GEMV: 0 = metadata points outside the buffer, 1 = dword-sliced, 2 = per element
struct RowState { int nb; int kind; int64_t bit0; };

// FAST = false: no row can take the dword-sliced path (P % 32 != 0, or a buffer too small to prefetch from);
// the kernel then contains no prefetch at all.
template <int MB, int D, bool FAST>
__global__ void __launch_bounds__(512) gemv_kernel(GemvArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint16_t* xh = reinterpret_cast<uint16_t*>(smem);                                // [MB][P] sat-fp16 activations
    const size_t xh_bytes = (((size_t)MB * a.P * 2) + 15) & ~(size_t)15;
    float* sxc = reinterpret_cast<float*>(smem + xh_bytes);                          // [C][MB] chunk sums of x
    float* part = sxc + (size_t)a.C * MB;                                            // [RW][C][MB] partial id sums

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = wave / a.W, wc = wave - g * a.W;
    const int row0 = blockIdx.x * a.RW;
    const int rows_here = min(a.RW, a.Q - row0);
    const int64_t clamp_byte = (a.ids_bytes - 8) & ~(int64_t)3;
    // rows of this wave's group: row0 + g + G*k, k < n_rows (<= 64)
    const int n_rows = rows_here > g ? (rows_here - g + a.G - 1) / a.G : 0;

    // ---- row metadata of the whole group in one vector load: lane k holds row k's width, kind and bit offset.
    // kind: 0 = metadata points outside the buffer, 1 = dword-sliced, 2 = per element, 3 = no such row
    uint32_t my_info = 3u << 8;
    int64_t my_bit0 = 0;
    if (lane < n_rows) {
        const int q = row0 + g + a.G * lane;
        const int nb = a.nbits[q];
        my_bit0 = a.bit_off[q];
        const bool ok = row_in_bounds(my_bit0, nb, a.P, a.ids_bytes);
        // a row stored in planes is read element by element here (this kernel serves the shapes the matrix-core path does not)
        const int kind = !ok ? 0 : (FAST && !off_is_plane(my_bit0) && (my_bit0 & 31) == 0 && nb >= 4 && nb <= kMaxFastNb) ? 1 : 2;
        my_info = (uint32_t)nb | ((uint32_t)kind << 8);
    }
    uint32_t my_b_lo = (uint32_t)my_bit0, my_b_hi = (uint32_t)((uint64_t)my_bit0 >> 32);
    // The values are copied once (the copy is where the wait for the metadata happens); reading a lane of them
    // later never waits on the vector-memory queue again.
    asm volatile("v_mov_b32 %0, %0\n\tv_mov_b32 %1, %1\n\tv_mov_b32 %2, %2" : "+v"(my_info), "+v"(my_b_lo), "+v"(my_b_hi));

    bool active = false;      // whether this wave has a chunk in the current panel
    auto row_state = [&](int k) {
        RowState s;
        const uint32_t info = (uint32_t)__builtin_amdgcn_readlane((int)my_info, k & 63);
        const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readlane((int)my_b_lo, k & 63);
        const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readlane((int)my_b_hi, k & 63);
        s.nb = (int)(info & 0xFFu);
        s.kind = (active && k < 64) ? (int)(info >> 8) : 3;
        s.bit0 = (int64_t)(((uint64_t)b_hi << 32) | b_lo);
        return s;
    };

    uint4 wlo[D], whi[D];
    RowState st[D];
    int cur_col = 0;          // this lane's first column in the current panel
    bool cur_live = false;
    // Requests the two 16-byte pieces of row k's slice.  ALWAYS exactly two loads, never under a branch, from
    // addresses inside the buffer (rows or lanes that do not use them read the first 32 bytes of `ids`): the
    // number of loads in flight behind any slot is then the same on every path, which is what lets the
    // consumer wait for its own slot only.
    auto issue = [&](int slot, int k) {
        const RowState s = row_state(k);
        st[slot] = s;
        if constexpr (FAST) {
            const bool row_fast = s.kind == 1;                                   // uniform
            const unsigned char* rowp = a.ids + (row_fast ? (s.bit0 >> 3) : 0);  // uniform
            const uint32_t tail = row_fast ? 4u * (uint32_t)(s.nb - 4) : 16u;    // uniform
            const uint32_t off = (row_fast && cur_live) ? (uint32_t)(cur_col / kFieldsPerLane) * (4u * (uint32_t)s.nb) : 0u;
            wlo[slot] = *reinterpret_cast<const uint4*>(rowp + (uint64_t)off);
            whi[slot] = *reinterpret_cast<const uint4*>(rowp + tail + (uint64_t)off);
        }
    };

    for (int panel = 0; panel < a.panels; ++panel) {
        const int c = panel * a.W + wc;
        active = c < a.C;                                    // wave-uniform
        const int n_eff = active ? n_rows : 0;
        cur_col = c * kChunk + lane * kFieldsPerLane;
        cur_live = FAST && active && cur_col < a.P;
#pragma unroll
        for (int s = 0; s < D; ++s) issue(s, s);

        if (panel == 0) {
            // ---- activations: narrow once per workgroup (after the first ids are on their way) ----
            const int64_t n = (int64_t)MB * a.P;
            if ((a.P & 7) == 0) {
                for (int64_t i = (int64_t)tid * 8; i < n; i += (int64_t)blockDim.x * 8) {
                    uint32_t o[4];
                    if (a.x_dtype == QVB8_F32) {
                        const float4 v0 = *reinterpret_cast<const float4*>((const float*)a.X + i);
                        const float4 v1 = *reinterpret_cast<const float4*>((const float*)a.X + i + 4);
                        o[0] = sat_half_bits(v0.x) | (sat_half_bits(v0.y) << 16);
                        o[1] = sat_half_bits(v0.z) | (sat_half_bits(v0.w) << 16);
                        o[2] = sat_half_bits(v1.x) | (sat_half_bits(v1.y) << 16);
                        o[3] = sat_half_bits(v1.z) | (sat_half_bits(v1.w) << 16);
                    } else {
                        const uint4 v = *reinterpret_cast<const uint4*>((const uint16_t*)a.X + i);
                        const uint32_t u[4] = {v.x, v.y, v.z, v.w};
                        if (a.x_dtype == QVB8_F16) {
#pragma unroll
                            for (int k = 0; k < 4; ++k) o[k] = u[k];      // fp16 input is used as it is (no clamp: inf stays inf)
                        } else {
#pragma unroll
                            for (int k = 0; k < 4; ++k)
                                o[k] = sat_half_bits(__uint_as_float(u[k] << 16)) | (sat_half_bits(__uint_as_float(u[k] & 0xFFFF0000u)) << 16);
                        }
                    }
                    *reinterpret_cast<uint4*>(xh + i) = make_uint4(o[0], o[1], o[2], o[3]);
                }
            } else {
                for (int64_t i = tid; i < n; i += blockDim.x) {
                    const float v = load_as_f32(a.X, i, a.x_dtype);
                    xh[i] = a.x_dtype == QVB8_F16 ? ((const uint16_t*)a.X)[i] : (uint16_t)sat_half_bits(v);
                }
            }
            __syncthreads();
        }

        const int col = cur_col;
        const bool live = cur_live;
        // the lane's activations as fp16 pairs, and their sum
        uint32_t xr[MB][16];
        float sx[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                uint4 v = make_uint4(0, 0, 0, 0);
                if (live) v = *reinterpret_cast<const uint4*>(xh + (size_t)m * a.P + col + 8 * k);
                xr[m][4 * k] = v.x; xr[m][4 * k + 1] = v.y; xr[m][4 * k + 2] = v.z; xr[m][4 * k + 3] = v.w;
            }
            float s0 = 0.f, s1 = 0.f;
            const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
            for (int k = 0; k < 16; k += 2) {
                s0 = __builtin_amdgcn_fdot2(ones, __builtin_bit_cast(half2_t, xr[m][k]), s0, false);
                s1 = __builtin_amdgcn_fdot2(ones, __builtin_bit_cast(half2_t, xr[m][k + 1]), s1, false);
            }
            sx[m] = s0 + s1;
        }
        // chunk sum of x for the epilogue (per element when no lane owns whole slices)
        float sxw[MB];
        if constexpr (FAST) {
#pragma unroll
            for (int m = 0; m < MB; ++m) sxw[m] = wave_sum(sx[m]);
        } else {
            const int col_end = active ? min(a.P, (c + 1) * kChunk) : 0;
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                float s = 0.f;
                for (int cc = c * kChunk + lane; cc < col_end; cc += kWave) s += f16_bits_to_f32(xh[(size_t)m * a.P + cc]);
                sxw[m] = wave_sum(s);
            }
        }
        if (active && g == 0 && lane == 0) {
#pragma unroll
            for (int m = 0; m < MB; ++m) sxc[c * MB + m] = sxw[m];
        }

        // id sums of one row for this lane (before the lanes are combined)
        auto consume = [&](int slot, float (&d)[MB]) {
            const RowState s = st[slot];
#pragma unroll
            for (int m = 0; m < MB; ++m) d[m] = 0.f;
            if (FAST && s.kind == 1) {
                if (live) gemv_compute_fast<MB>(s.nb, wlo[slot], whi[slot], xr, sx, d);
            } else if (s.kind == 2) {
                const int col_end = min(a.P, (c + 1) * kChunk);
                for (int cc = c * kChunk + lane; cc < col_end; cc += kWave) {
                    const float idf = (float)row_field(a.ids, s.bit0, s.nb, cc, clamp_byte);
#pragma unroll
                    for (int m = 0; m < MB; ++m) d[m] = __builtin_fmaf(f16_bits_to_f32(xh[(size_t)m * a.P + cc]), idf, d[m]);
                }
            } else if (s.kind == 0) {
#pragma unroll
                for (int m = 0; m < MB; ++m) d[m] = __builtin_nanf("");
            }
        };
        static_assert(D == 4, "the row pipeline combines four rows at a time");
        const int n_iter = (n_eff + D - 1) / D;
        for (int it = 0; it < n_iter; ++it) {
            float d[D][MB];
#pragma unroll
            for (int s = 0; s < D; ++s) {
                consume(s, d[s]);
                issue(s, it * D + s + D);
            }
            // lanes 0..3 end up with the totals of rows it*4 + 0..3
            const int k = it * D + (lane & 3);
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                const float v4[4] = {d[0][m], d[1][m], d[2][m], d[3][m]};
                const float tot = wave_sum4(v4, lane);
                if (lane < 4 && k < n_eff) part[((size_t)(g + a.G * k) * a.C + c) * MB + m] = tot;
            }
        }
    }
    __syncthreads();

    // ---- epilogue: combine the chunks of each row in ascending order ----
    for (int i = tid; i < rows_here * MB; i += blockDim.x) {
        const int rl = i / MB, m = i - rl * MB;
        double dsum = 0.0, xsum = 0.0;
        for (int cc = 0; cc < a.C; ++cc) {
            dsum += (double)part[((size_t)rl * a.C + cc) * MB + m];
            xsum += (double)sxc[cc * MB + m];
        }
        const int q = row0 + rl;
        a.Y[(size_t)m * a.Q + q] = (float)((double)a.tau_s[q] * dsum + (double)a.min_s[q] * xsum);
    }
}

// Escapes: the main pass multiplied the banded value; add x * (exact - banded) for each escape, one thread per
// output row that has escapes, in ascending order, no atomics.
__global__ void __launch_bounds__(256) gemv_fix_escapes_kernel(const void* __restrict__ X, int x_dtype, int M,
        const uint8_t* __restrict__ ids, int64_t ids_bytes, const float* __restrict__ min_s, const float* __restrict__ tau_s,
        const uint8_t* __restrict__ nbits, const int64_t* __restrict__ bit_off, const int64_t* __restrict__ esc_idx,
        const float* __restrict__ esc_vals, int64_t n_esc, float* __restrict__ Y, int Q, int P) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_esc) return;
    const int64_t q = esc_idx[i] / P;
    if (q < 0 || q >= Q) return;
    if (i > 0 && esc_idx[i - 1] / P == q) return;
    const int nb = nbits[q];
    const int64_t bit0 = bit_off[q];
    const float ts = tau_s[q], mn = min_s[q];
    const int64_t clamp_byte = (ids_bytes - 8) & ~(int64_t)3;
    float acc[8];
#pragma unroll
    for (int m = 0; m < 8; ++m) acc[m] = 0.f;
    for (int64_t e = i; e < n_esc && esc_idx[e] / P == q; ++e) {
        const int c = (int)(esc_idx[e] - q * P);
        const float banded = __builtin_fmaf((float)row_field(ids, bit0, nb, c, clamp_byte), ts, mn);
        const float delta = esc_vals[e] - banded;
#pragma unroll
        for (int m = 0; m < 8; ++m)
            if (m < M) {
                const float xv = load_as_f32(X, (int64_t)m * P + c, x_dtype);
                const float xs = x_dtype == QVB8_F16 ? xv : f16_bits_to_f32(sat_half_bits(xv));
                acc[m] = __builtin_fmaf(xs, delta, acc[m]);
            }
    }
#pragma unroll
    for (int m = 0; m < 8; ++m)
        if (m < M) Y[(size_t)m * Q + q] += acc[m];
}

}  // namespace qvb8

// ===========================================================================================================
// C ABI
// ===========================================================================================================
using namespace qvb8;

extern "C" int qvb8_abi_version(void) { return QVB8_ABI_VERSION; }
extern "C" const char* qvb8_last_error(void) { return host::last_error().c_str(); }

static int check_pack(const uint8_t* ids, int64_t ids_bytes, const float* min_s, const float* tau_s, const uint8_t* nbits,
                      const int64_t* bit_off, int64_t Q, int64_t P, const char* who) {
    if (Q < 0 || P < 0 || Q > 0x7fffffff || P > 0x7fffffff) return host::fail(QVB8_ERR_ARG, "%s: Q=%lld P=%lld out of range", who, (long long)Q, (long long)P);
    if (Q > 0 && (!min_s || !tau_s || !nbits || !bit_off)) return host::fail(QVB8_ERR_ARG, "%s: null row metadata", who);
    if (Q > 0 && P > 0 && !ids) return host::fail(QVB8_ERR_ARG, "%s: null ids", who);
    if ((reinterpret_cast<uintptr_t>(ids) & 3u) != 0)
        return host::fail(QVB8_ERR_ARG, "%s: ids buffer must be 4-byte aligned (pass a contiguous copy, not an offset view)", who);
    if (Q > 0 && P > 0 && ids_bytes < 8) return host::fail(QVB8_ERR_ARG, "%s: ids buffer shorter than its 8 pad bytes", who);
    return QVB8_OK;
}

extern "C" int qvb8_decode(const uint8_t* ids, int64_t ids_bytes, const float* min_s, const float* tau_s,
                           const uint8_t* nbits, const int64_t* bit_off, int64_t Q, int64_t P,
                           int out_dtype, void* out, void* stream) {
    if (int rc = check_pack(ids, ids_bytes, min_s, tau_s, nbits, bit_off, Q, P, "qvb8_decode")) return rc;
    if (out_dtype < 0 || out_dtype > 2) return host::fail(QVB8_ERR_ARG, "qvb8_decode: out_dtype %d", out_dtype);
    if (Q == 0 || P == 0) return QVB8_OK;
    if (!out || (reinterpret_cast<uintptr_t>(out) & 15u)) return host::fail(QVB8_ERR_ARG, "qvb8_decode: out must be 16-byte aligned");
    DecodeArgs a;
    a.ids = ids; a.min_s = min_s; a.tau_s = tau_s; a.nbits = nbits; a.bit_off = bit_off; a.out = out;
    a.ids_bytes = ids_bytes; a.Q = (int)Q; a.P = (int)P; a.C = (int)((P + kChunk - 1) / kChunk);
    a.n_items = Q * a.C;
    a.rows = nullptr; a.esc_idx = nullptr; a.esc_vals = nullptr; a.n_esc = 0;
    const int64_t blocks = (a.n_items + 3) / 4;
    if (blocks > 0x7fffffff) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_decode: tensor too large for one launch");
    hipStream_t s = (hipStream_t)stream;
    switch (out_dtype) {
        case QVB8_F32: hipLaunchKernelGGL((decode_kernel<0, false>), dim3((unsigned)blocks), dim3(256), 0, s, a); break;
        case QVB8_F16: hipLaunchKernelGGL((decode_kernel<1, false>), dim3((unsigned)blocks), dim3(256), 0, s, a); break;
        default: hipLaunchKernelGGL((decode_kernel<2, false>), dim3((unsigned)blocks), dim3(256), 0, s, a); break;
    }
    return host::check_launch("qvb8_decode");
}

extern "C" int qvb8_lookup_rows(const int64_t* rows, int64_t n_rows, const uint8_t* ids, int64_t ids_bytes, const float* min_s,
                                const float* tau_s, const uint8_t* nbits, const int64_t* bit_off, int64_t Q, int64_t P,
                                const int64_t* esc_idx, const float* esc_vals, int64_t n_esc, int out_dtype, void* out,
                                void* stream) {
    if (int rc = check_pack(ids, ids_bytes, min_s, tau_s, nbits, bit_off, Q, P, "qvb8_lookup_rows")) return rc;
    if (out_dtype < 0 || out_dtype > 2) return host::fail(QVB8_ERR_ARG, "qvb8_lookup_rows: out_dtype %d", out_dtype);
    if (n_rows < 0 || n_esc < 0) return host::fail(QVB8_ERR_ARG, "qvb8_lookup_rows: negative size");
    if (n_rows == 0 || P == 0) return QVB8_OK;
    if (Q == 0) return host::fail(QVB8_ERR_ARG, "qvb8_lookup_rows: rows wanted from an empty table");
    if (!rows) return host::fail(QVB8_ERR_ARG, "qvb8_lookup_rows: null rows");
    if (n_esc > 0 && (!esc_idx || !esc_vals)) return host::fail(QVB8_ERR_ARG, "qvb8_lookup_rows: null escape arrays");
    if (!out || (reinterpret_cast<uintptr_t>(out) & 15u)) return host::fail(QVB8_ERR_ARG, "qvb8_lookup_rows: out must be 16-byte aligned");
    DecodeArgs a;
    a.ids = ids; a.min_s = min_s; a.tau_s = tau_s; a.nbits = nbits; a.bit_off = bit_off; a.out = out;
    a.ids_bytes = ids_bytes; a.Q = (int)Q; a.P = (int)P; a.C = (int)((P + kChunk - 1) / kChunk);
    a.n_items = n_rows * a.C;
    a.rows = rows; a.esc_idx = esc_idx; a.esc_vals = esc_vals; a.n_esc = n_esc;
    const int64_t blocks = (a.n_items + 3) / 4;
    if (blocks > 0x7fffffff) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_lookup_rows: too many rows for one launch");
    hipStream_t s = (hipStream_t)stream;
    switch (out_dtype) {
        case QVB8_F32: hipLaunchKernelGGL((decode_kernel<0, true>), dim3((unsigned)blocks), dim3(256), 0, s, a); break;
        case QVB8_F16: hipLaunchKernelGGL((decode_kernel<1, true>), dim3((unsigned)blocks), dim3(256), 0, s, a); break;
        default: hipLaunchKernelGGL((decode_kernel<2, true>), dim3((unsigned)blocks), dim3(256), 0, s, a); break;
    }
    return host::check_launch("qvb8_lookup_rows");
}

extern "C" int qvb8_scatter_escapes(void* out, int out_dtype, int64_t n_out, const int64_t* esc_idx,
                                    const float* esc_vals, int64_t n_esc, void* stream) {
    if (out_dtype < 0 || out_dtype > 2) return host::fail(QVB8_ERR_ARG, "qvb8_scatter_escapes: out_dtype %d", out_dtype);
    if (n_esc < 0 || n_out < 0) return host::fail(QVB8_ERR_ARG, "qvb8_scatter_escapes: negative size");
    if (n_esc == 0) return QVB8_OK;
    if (!out || !esc_idx || !esc_vals) return host::fail(QVB8_ERR_ARG, "qvb8_scatter_escapes: null pointer");
    const unsigned blocks = (unsigned)((n_esc + 255) / 256);
    hipStream_t s = (hipStream_t)stream;
    switch (out_dtype) {
        case QVB8_F32: hipLaunchKernelGGL(scatter_escapes_kernel<0>, dim3(blocks), dim3(256), 0, s, out, n_out, esc_idx, esc_vals, n_esc); break;
        case QVB8_F16: hipLaunchKernelGGL(scatter_escapes_kernel<1>, dim3(blocks), dim3(256), 0, s, out, n_out, esc_idx, esc_vals, n_esc); break;
        default: hipLaunchKernelGGL(scatter_escapes_kernel<2>, dim3(blocks), dim3(256), 0, s, out, n_out, esc_idx, esc_vals, n_esc); break;
    }
    return host::check_launch("qvb8_scatter_escapes");
}

extern "C" int qvb8_certify(const void* restored, int restored_dtype, const void* original, int original_dtype,
                            int64_t n, float tau, uint32_t* result, void* stream) {
    if (restored_dtype < 0 || restored_dtype > 2 || original_dtype < 0 || original_dtype > 2)
        return host::fail(QVB8_ERR_ARG, "qvb8_certify: dtype");
    if (n < 0 || !result) return host::fail(QVB8_ERR_ARG, "qvb8_certify: bad n or null result");
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(certify_init_kernel, dim3(1), dim3(64), 0, s, result);
    if (n > 0) {
        if (!restored || !original) return host::fail(QVB8_ERR_ARG, "qvb8_certify: null tensor");
        const int64_t want = (n + 255) / 256;
        const unsigned blocks = (unsigned)(want < 4096 ? want : 4096);
        hipLaunchKernelGGL(certify_kernel, dim3(blocks), dim3(256), 0, s, restored, restored_dtype, original, original_dtype, n, tau, result);
    }
    return host::check_launch("qvb8_certify");
}

extern "C" int qvb8_sat_half(const void* x, int x_dtype, int64_t n, void* out_f16, void* stream) {
    if (x_dtype < 0 || x_dtype > 2 || n < 0) return host::fail(QVB8_ERR_ARG, "qvb8_sat_half: bad argument");
    if (n == 0) return QVB8_OK;
    if (!x || !out_f16) return host::fail(QVB8_ERR_ARG, "qvb8_sat_half: null pointer");
    const int64_t blocks = (n + 255) / 256;
    if (blocks > 0x7fffffff) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_sat_half: too large");
    hipStream_t s = (hipStream_t)stream;
    switch (x_dtype) {
        case QVB8_F32: hipLaunchKernelGGL(sat_half_kernel<0>, dim3((unsigned)blocks), dim3(256), 0, s, x, (uint16_t*)out_f16, n); break;
        case QVB8_F16: hipLaunchKernelGGL(sat_half_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, s, x, (uint16_t*)out_f16, n); break;
        default: hipLaunchKernelGGL(sat_half_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, s, x, (uint16_t*)out_f16, n); break;
    }
    return host::check_launch("qvb8_sat_half");
}

extern "C" int qvb8_scale_sat_half(const void* x, int x_dtype, int64_t n, float scale, void* out_f16, void* stream) {
    if (x_dtype < 0 || x_dtype > 2 || n < 0) return host::fail(QVB8_ERR_ARG, "qvb8_scale_sat_half: bad argument");
    if (n == 0) return QVB8_OK;
    if (!x || !out_f16) return host::fail(QVB8_ERR_ARG, "qvb8_scale_sat_half: null pointer");
    const int64_t blocks = (n + 255) / 256;
    if (blocks > 0x7fffffff) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_scale_sat_half: too large");
    hipStream_t s = (hipStream_t)stream;
    switch (x_dtype) {
        case QVB8_F32: hipLaunchKernelGGL(scale_sat_half_kernel<0>, dim3((unsigned)blocks), dim3(256), 0, s, x, scale, (uint16_t*)out_f16, n); break;
        case QVB8_F16: hipLaunchKernelGGL(scale_sat_half_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, s, x, scale, (uint16_t*)out_f16, n); break;
        default: hipLaunchKernelGGL(scale_sat_half_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, s, x, scale, (uint16_t*)out_f16, n); break;
    }
    return host::check_launch("qvb8_scale_sat_half");
}

// ---- GEMV launch plan --------------------------------------------------------------------------------------
namespace {
struct GemvPlan { int C, W, G, panels, RW, threads; size_t lds; unsigned blocks; };

// LDS a workgroup may use for the narrowed activations plus partial sums.
constexpr size_t kGemvLdsLimit = 128 * 1024;

bool plan_gemv(int64_t M, int64_t Q, int64_t P, GemvPlan& pl) {
    pl.C = (int)((P + kChunk - 1) / kChunk);
    if (pl.C < 1) pl.C = 1;
    const int max_waves = 8;
    pl.panels = (pl.C + max_waves - 1) / max_waves;
    pl.W = (pl.C + pl.panels - 1) / pl.panels;
    pl.G = pl.panels == 1 ? max_waves / pl.W : 1;
    if (pl.G < 1) pl.G = 1;
    pl.threads = 64 * pl.W * pl.G;
    // rows per workgroup: aim at `per_cu` workgroups per compute unit, at least one row per group
    const int cus = host::device_cus();
    const int per_cu = host::env_int("QVB8_GEMV_WGS_PER_CU", 2);
    int64_t target = (int64_t)cus * (per_cu > 0 ? per_cu : 2);
    int64_t rw = (Q + target - 1) / target;
    rw = (rw + pl.G - 1) / pl.G * pl.G;
    if (rw < pl.G) rw = pl.G;
    const int64_t rw_max = 64LL * pl.G;
    if (rw > rw_max) rw = rw_max;
    pl.RW = (int)rw;
    pl.blocks = (unsigned)((Q + rw - 1) / rw);
    const size_t xh = (((size_t)M * P * 2) + 15) & ~(size_t)15;
    pl.lds = xh + (size_t)pl.C * M * 4 + (size_t)pl.RW * pl.C * M * 4;
    return pl.lds <= kGemvLdsLimit;
}

template <int MB, int D, bool FAST>
void launch_gemv_as(const GemvArgs& a, const GemvPlan& pl, hipStream_t s) {
    static bool attr = false;
    if (!attr) {
        (void)hipFuncSetAttribute((const void*)gemv_kernel<MB, D, FAST>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kGemvLdsLimit);
        attr = true;
    }
    hipLaunchKernelGGL((gemv_kernel<MB, D, FAST>), dim3(pl.blocks), dim3(pl.threads), pl.lds, s, a);
}

template <int MB>
void launch_gemv(const GemvArgs& a, const GemvPlan& pl, hipStream_t s) {
    constexpr int D = 4;
    const bool fast = (a.P % kFieldsPerLane) == 0 && a.ids_bytes >= 32;
    if (fast) launch_gemv_as<MB, D, true>(a, pl, s);
    else launch_gemv_as<MB, D, false>(a, pl, s);
}
}  // namespace

extern "C" int64_t qvb8_gemv_workspace_bytes(int64_t M, int64_t Q, int64_t P) {
    (void)M; (void)Q; (void)P;
    return 0;
}

extern "C" int qvb8_gemv(const void* X, int x_dtype, int64_t M,
                         const uint8_t* ids, int64_t ids_bytes, const float* min_s, const float* tau_s,
                         const uint8_t* nbits, const int64_t* bit_off, int64_t Q, int64_t P,
                         const int64_t* esc_idx, const float* esc_vals, int64_t n_esc,
                         float* Y, void* workspace, int64_t workspace_bytes, void* stream) {
    (void)workspace; (void)workspace_bytes;
    if (int rc = check_pack(ids, ids_bytes, min_s, tau_s, nbits, bit_off, Q, P, "qvb8_gemv")) return rc;
    if (M < 1 || M > 8)
        return host::fail(QVB8_ERR_ARG, "qvb8 GEMV-multi: M=%lld is outside the instantiated range 1..8; callers above this route M>8 to the small-M GEMM", (long long)M);
    if (x_dtype < 0 || x_dtype > 2) return host::fail(QVB8_ERR_ARG, "qvb8_gemv: x_dtype %d", x_dtype);
    if (n_esc < 0 || (n_esc > 0 && (!esc_idx || !esc_vals))) return host::fail(QVB8_ERR_ARG, "qvb8_gemv: bad escape list");
    if (Q == 0) return QVB8_OK;
    if (!Y) return host::fail(QVB8_ERR_ARG, "qvb8_gemv: null Y");
    if (P > 0 && (!X || (reinterpret_cast<uintptr_t>(X) & 15u))) return host::fail(QVB8_ERR_ARG, "qvb8_gemv: X must be 16-byte aligned");
    if (P > 0 && (P % 8) == 0 && ((P * (x_dtype == QVB8_F32 ? 4 : 2)) % 16) != 0)
        return host::fail(QVB8_ERR_ARG, "qvb8_gemv: rows of X must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    // the activations of one launch must fit in LDS: split M if they do not
    int64_t mb = M;
    GemvPlan pl;
    while (mb >= 1 && !plan_gemv(mb, Q, P, pl)) --mb;
    if (mb < 1) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_gemv: P=%lld is too wide for one workgroup's LDS", (long long)P);
    const size_t xrow = (size_t)P * (x_dtype == QVB8_F32 ? 4 : 2);
    for (int64_t m0 = 0; m0 < M; m0 += mb) {
        const int64_t mm = (M - m0) < mb ? (M - m0) : mb;
        if (mm != mb && !plan_gemv(mm, Q, P, pl)) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_gemv: planning failed");
        GemvArgs a;
        a.X = (const char*)X + (size_t)m0 * xrow; a.ids = ids; a.min_s = min_s; a.tau_s = tau_s; a.nbits = nbits; a.bit_off = bit_off;
        a.Y = Y + (size_t)m0 * Q; a.ids_bytes = ids_bytes; a.x_dtype = x_dtype; a.Q = (int)Q; a.P = (int)P;
        a.C = pl.C; a.W = pl.W; a.G = pl.G; a.panels = pl.panels; a.RW = pl.RW;
        switch (mm) {
            case 1: launch_gemv<1>(a, pl, s); break;
            case 2: launch_gemv<2>(a, pl, s); break;
            case 3: launch_gemv<3>(a, pl, s); break;
            case 4: launch_gemv<4>(a, pl, s); break;
            case 5: launch_gemv<5>(a, pl, s); break;
            case 6: launch_gemv<6>(a, pl, s); break;
            case 7: launch_gemv<7>(a, pl, s); break;
            default: launch_gemv<8>(a, pl, s); break;
        }
        if (int rc = host::check_launch("qvb8_gemv")) return rc;
        if (n_esc > 0) {
            hipLaunchKernelGGL(gemv_fix_escapes_kernel, dim3((unsigned)((n_esc + 255) / 256)), dim3(256), 0, s,
                               a.X, x_dtype, (int)mm, ids, ids_bytes, min_s, tau_s, nbits, bit_off, esc_idx, esc_vals, n_esc,
                               a.Y, (int)Q, (int)P);
            if (int rc = host::check_launch("qvb8_gemv escapes")) return rc;
        }
    }
    return QVB8_OK;
}
