// Attention of a block of query rows over a banded KV cache: keys and values stay in memory as 1- or 2-byte ids with
// one (centre value, step) per segment / kv head / channel and one id centre per segment / kv head,
//
//     k = fp16(kmid[c] + kstep[c] * (id - kc))          v likewise,
//
// and are restored tile by tile inside the kernel -- the full-precision K / V of the context never exist.  Semantics
// of the reference's kernel (kv/cuda_attn/qvattn_cuda.cu:97-255): one workgroup = one kv head x one split of the key
// tiles x one block of query rows (row r = token * G + g); tiles of at most 32 keys come from a table (first key,
// length, segment) and never straddle a segment; key position <= query position; online softmax with the
// probabilities rounded to fp16 before they are summed and multiplied; the result per split is the unnormalised
// accumulator plus (running max, running sum), which the caller combines.
//
// Shape of this kernel (gfx950): 256 threads = 4 waves per workgroup, 16 query rows (or 2 / 4 blocks of 16), 32 keys per tile.
//   * ids are requested TWO tiles ahead into two register sets (a trip to memory under load takes longer than one tile's
//     arithmetic): a wave reads whole key rows (64 lanes x 4 ids = 256 channels), every thread keeps the same four
//     channels for all its keys, so it holds 4 + 4 constants per operand; no request sits under a branch (a tile past
//     the split's end re-reads one cached line), so the counted waits leave the younger set in flight; the tile table
//     comes through the scalar unit;
//   * restored K goes to LDS as [key][channel], restored V as [channel][key] (a thread owns 4 keys x 4 channels, so the
//     transposition is free) with the 8-byte cells of a row swizzled by the channel group;
//   * S = Q K^T: wave w takes keys 16 (w % 2) .. + 15 and half w / 2 of the channels (v_mfma_f32_16x16x16_f16, its part
//     of Q kept in registers as the A operand); the two halves are added when S is read back;
//   * the softmax is computed once per workgroup (wave w rows 4 w .. 4 w + 3, sixteen lanes a row, two keys a lane, row
//     maxima and sums by data-parallel rotations inside the row); the probabilities, rounded to fp16, and the rows'
//     rescale factors reach the four waves through LDS in the A-operand layout of the second product;
//   * O += P V: wave w owns a quarter of the output channels.
#include <hip/hip_runtime.h>
#include <math.h>
#include <algorithm>
#include <type_traits>
#include <stdint.h>

#include "qvb8_amd.h"
#include "qvb8_host.h"

namespace qvb8 {
namespace {

typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef float f4_t __attribute__((ext_vector_type(4)));

constexpr int kRows = 16;          // query rows per workgroup
constexpr int kKeys = 32;          // keys per tile (the table's tiles are never longer)
constexpr int kAttnThreads = 256;
constexpr int kSStride = kKeys + 4;

struct AttnArgs {
    const uint16_t* q; int64_t sq_r, sq_h;
    const void* ki; const void* vi; int64_t s_n, s_h;           // strides in ids
    const float* kmid; const float* kstep; const float* vmid; const float* vstep; const float* kc; const float* vc;
    const int32_t* ts; const int32_t* tl; const int32_t* tseg;
    float* o; float* m; float* l;
    int q_pos0, n_tiles, tps, n_rows, G, nhkv;
    float scale;
};

// Four neighbouring channels of one key, as they lie in memory.
template <typename T> struct Quad;
template <> struct Quad<uint8_t> {
    typedef uint32_t type;
    static __device__ __forceinline__ float id(type w, int c) { return (float)((w >> (8 * c)) & 0xFFu); }
};
template <> struct Quad<uint16_t> {
    typedef uint2 type;
    static __device__ __forceinline__ float id(type w, int c) { return (float)(((c < 2 ? w.x : w.y) >> (16 * (c & 1))) & 0xFFFFu); }
};

// Two restored values as one dword of fp16: lo = fp16(fma(s0, d0, m0)), hi = fp16(fma(s1, d1, m1)), the fused
// multiply-add rounded to fp32 FIRST and then to fp16, as the reference's `__floats2half2_rn(md + sp * (v - c))` does.
// Written as `(_Float16)fmaf(...)` the compiler emits v_fma_mixlo_f16, which rounds the exact sum to fp16 in one step:
// one fp16 ulp off in about one value of 4000 (measured against the oracle).  The conversion is kept out of its sight.
__device__ __forceinline__ uint32_t restore_pair(float s0, float d0, float m0, float s1, float d1, float m1) {
    const float lo = __builtin_fmaf(s0, d0, m0), hi = __builtin_fmaf(s1, d1, m1);
    uint32_t r;
    asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
    return r;
}

// The value of the lane N places further on in its row of 16 lanes (a data-parallel move inside the vector unit; four of
// them -- 8, 4, 2, 1 -- leave a row's maximum or sum in every lane, without the LDS trips of a general shuffle).
template <int N>
__device__ __forceinline__ float row_rotate(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x120 + N, 0xF, 0xF, false));
}
__device__ __forceinline__ float row_max16(float v) {
    v = fmaxf(v, row_rotate<8>(v)); v = fmaxf(v, row_rotate<4>(v)); v = fmaxf(v, row_rotate<2>(v)); return fmaxf(v, row_rotate<1>(v));
}
__device__ __forceinline__ float row_sum16(float v) {
    v += row_rotate<8>(v); v += row_rotate<4>(v); v += row_rotate<2>(v); return v + row_rotate<1>(v);
}

// One entry of the tile table through the scalar unit.  A plain load would do, but behind a barrier the compiler turns
// it into a vector load, and waiting for that one (the youngest request) also waits for every id request still in
// flight -- the prefetch would be worth nothing.
struct TileRef { int start, nlen, seg; bool ok; };
__device__ __forceinline__ void tile_entry(const int32_t* ts, const int32_t* tl, const int32_t* tseg, int t, TileRef& r) {
    const uint32_t off = (uint32_t)__builtin_amdgcn_readfirstlane(t) * 4u;
    int start, nlen, seg;
    asm volatile("s_load_dword %0, %3, %6\n\ts_load_dword %1, %4, %6\n\ts_load_dword %2, %5, %6\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(start), "=&s"(nlen), "=&s"(seg) : "s"(ts), "s"(tl), "s"(tseg), "s"(off) : "memory");
    r.start = start; r.nlen = nlen; r.seg = seg;
}

// Three workgroups per compute unit (two with 16-bit ids and 256 channels, whose two register sets are twice as large):
// the third one is what hides a workgroup's barriers and dependent chains -- 74.9 against 82.3 us over 131072 keys.
// RB = blocks of 16 query rows a workgroup serves from one restored tile (1, 2 or 4): the restore, most of the work, is
// shared; every block has its own Q registers, scores, softmax state and accumulators (two workgroups per CU then).
template <int D, typename T, int RB>
__global__ __launch_bounds__(kAttnThreads, ((D == 256 && sizeof(T) == 2) || RB > 1) ? 2 : 3) void attn_kernel(const AttnArgs a) {
    constexpr int CG = D / 4;                  // channel groups (four channels each) of a key
    constexpr int KSTEP = kAttnThreads / CG;   // key groups (four keys each) that one pass of the workgroup covers
    constexpr int UNITS = D / 128;             // (4 keys x 4 channels) units per thread and tile
    constexpr int KROW = D + 4;                // halfs per key in LDS: 16 keys' 8-byte reads fall on all banks once
    constexpr int NF = D / 64;                 // 16-channel output fragments per wave
    constexpr int NKS = D / 32;                // 16-channel steps of S = Q K^T per wave
    using QD = Quad<T>;
    using U = typename QD::type;
    __shared__ __align__(16) _Float16 Ks[kKeys * KROW];
    __shared__ __align__(16) _Float16 Vt[D * kKeys];
    __shared__ __align__(16) float Ss[RB * 2 * kRows * kSStride];
    constexpr int kPStride = kKeys + 8;                       // halfs per row of P
    __shared__ __align__(16) _Float16 Ps[RB * kRows * kPStride];
    __shared__ __align__(16) float Al[RB * kRows];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n16 = lane & 15, kg = lane >> 4;
    const int kf = wave & 1, dh = wave >> 1;                  // this wave's 16 keys and its half of the channels in S
    const int h = blockIdx.x, sp = blockIdx.y, row0 = blockIdx.z * (RB * kRows);
    const int cg = tid % CG, kgp0 = tid / CG;

    // the lane's query rows (one per block) as the A operand of S = Q K^T: Q[row][16 ks + 4 kg .. + 3], ks in the wave's half
    h4_t qa[RB][NKS];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        const int row = row0 + rb * kRows + n16;
        const bool row_ok = row < a.n_rows;
        const int rr = row_ok ? row : 0;
        const uint16_t* qp = a.q + (int64_t)(rr / a.G) * a.sq_r + (int64_t)(h * a.G + rr % a.G) * a.sq_h + dh * (D / 2) + 4 * kg;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            const h4_t v = *reinterpret_cast<const h4_t*>(qp + 16 * ks);
            qa[rb][ks] = row_ok ? v : h4_t{0, 0, 0, 0};
        }
    }
    const int qmin = a.q_pos0 + row0 / a.G;                                   // first position of the block's rows
    // the softmax's own split of the block: this lane's row and pair of keys
    const int srow = 4 * wave + (lane >> 4), kpair = lane & 15;             // row within a block
    const int qmax = a.q_pos0 + (min(row0 + RB * kRows, a.n_rows) - 1) / a.G; // last position any row of the workgroup sees

    // the head's ids: a scalar base; the thread's four channels are part of its (32-bit) offset
    const T* ki = reinterpret_cast<const T*>(a.ki) + (int64_t)h * a.s_h;
    const T* vi = reinterpret_cast<const T*>(a.vi) + (int64_t)h * a.s_h;
    const uint32_t cg_off = (uint32_t)(4 * cg) * (uint32_t)sizeof(T);
    const int t0 = (int)min((int64_t)sp * a.tps, (int64_t)a.n_tiles), t1 = (int)min((int64_t)t0 + a.tps, (int64_t)a.n_tiles);
    // ids of tile t into one register set: always 8 UNITS requests, none under a branch; keys past the tile's length
    // re-read its last key, and a tile that is not wanted -- past the split's end, or starting behind the last visible
    // position (tiles ascend: so do all after it) -- re-reads key 0 of the head (one cached line); neither is used.
    // A request's address is the tile's first key (scalar) plus the thread's key offset, fixed for the whole kernel
    // and clamped to the tile's last key (host-checked: 32 keys' stride fits 31 bits).
    const uint32_t key_stride = (uint32_t)a.s_n * (uint32_t)sizeof(T);      // bytes from one key to the next
    const uint32_t key_off0 = (uint32_t)(4 * kgp0) * key_stride;            // the thread's first key; its others lie a scalar further
    const unsigned char* kbytes = reinterpret_cast<const unsigned char*>(ki);
    const unsigned char* vbytes = reinterpret_cast<const unsigned char*>(vi);
    auto fetch = [&](int t, U (&rk)[UNITS][4], U (&rv)[UNITS][4], TileRef& ref) {
        tile_entry(a.ts, a.tl, a.tseg, min(t, t1 - 1), ref);
        ref.ok = __builtin_amdgcn_readfirstlane((int)(t < t1 && ref.start <= qmax)) != 0;      // scalar: the loop's branches stay uniform
        const int start = ref.ok ? ref.start : 0, nlen = ref.ok ? ref.nlen : 1;
        const int64_t tile_byte = (int64_t)start * a.s_n * (int64_t)sizeof(T);
        const uint32_t last_off = (uint32_t)max(nlen - 1, 0) * (uint32_t)a.s_n * (uint32_t)sizeof(T);
        const unsigned char* kb = kbytes + tile_byte;
        const unsigned char* vb = vbytes + tile_byte;
#pragma unroll
        for (int u = 0; u < UNITS; ++u)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t off = min(key_off0 + (uint32_t)(4 * KSTEP * u + j) * key_stride, last_off) + cg_off;
                rk[u][j] = *reinterpret_cast<const U*>(kb + off);
                rv[u][j] = *reinterpret_cast<const U*>(vb + off);
            }
    };

    float m_run[RB], l_run[RB];
    f4_t acc[RB][NF];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        m_run[rb] = -INFINITY; l_run[rb] = 0.f;
#pragma unroll
        for (int f = 0; f < NF; ++f) acc[rb][f] = f4_t{0.f, 0.f, 0.f, 0.f};
    }

    int cur_seg = -1;
    float km[4] = {0.f, 0.f, 0.f, 0.f}, ks_[4] = {0.f, 0.f, 0.f, 0.f}, vm[4] = {0.f, 0.f, 0.f, 0.f}, vs_[4] = {0.f, 0.f, 0.f, 0.f}, kc = 0.f, vc = 0.f;
    // One tile: restore the ids of register set (rk, rv) into LDS, refill the set with tile t + 2, S, softmax, O.
    auto tile = [&](int t, U (&rk)[UNITS][4], U (&rv)[UNITS][4], TileRef& ref) {
        const int start = ref.start, nlen = ref.ok ? ref.nlen : 0, seg = ref.seg;      // a tile that is not wanted: no key counts
        if (seg != cur_seg) {
            // A new segment (every few thousand keys): its constants for this thread's four channels.  The wait stands
            // INSIDE the branch: the requests of the next tiles' ids are older than these, and a wait placed where the
            // constants are first used would hold every tile until its successors' ids had arrived.
            const int64_t pb = ((int64_t)seg * a.nhkv + h) * D + 4 * cg;
            const float4 kmid = *reinterpret_cast<const float4*>(a.kmid + pb), kstep = *reinterpret_cast<const float4*>(a.kstep + pb);
            const float4 vmid = *reinterpret_cast<const float4*>(a.vmid + pb), vstep = *reinterpret_cast<const float4*>(a.vstep + pb);
            kc = a.kc[seg * a.nhkv + h]; vc = a.vc[seg * a.nhkv + h];
            km[0] = kmid.x; km[1] = kmid.y; km[2] = kmid.z; km[3] = kmid.w;
            ks_[0] = kstep.x; ks_[1] = kstep.y; ks_[2] = kstep.z; ks_[3] = kstep.w;
            vm[0] = vmid.x; vm[1] = vmid.y; vm[2] = vmid.z; vm[3] = vmid.w;
            vs_[0] = vstep.x; vs_[1] = vstep.y; vs_[2] = vstep.z; vs_[3] = vstep.w;
            __builtin_amdgcn_s_waitcnt(0x0F70);               // vmcnt(0)
            cur_seg = seg;
        }
        // Keys past the tile's length hold a copy of its last key: their scores are replaced by -inf before any use, so K
        // needs no blanking; their V must be zero (0 * inf would poison the sums), done on the packed halves.
        const bool whole = nlen == kKeys;
#pragma unroll
        for (int u = 0; u < UNITS; ++u) {
            const int kgp = kgp0 + KSTEP * u;
            uint2 vcell[4];
            float dv[4][4];                                         // [key j][channel c]: id - centre of V
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int key = 4 * kgp + j;
                float dk[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) { dk[c] = QD::id(rk[u][j], c) - kc; dv[j][c] = QD::id(rv[u][j], c) - vc; }
                uint2 kv;
                kv.x = restore_pair(ks_[0], dk[0], km[0], ks_[1], dk[1], km[1]);
                kv.y = restore_pair(ks_[2], dk[2], km[2], ks_[3], dk[3], km[3]);
                *reinterpret_cast<uint2*>(Ks + key * KROW + 4 * cg) = kv;
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                vcell[c].x = restore_pair(vs_[c], dv[0][c], vm[c], vs_[c], dv[1][c], vm[c]);
                vcell[c].y = restore_pair(vs_[c], dv[2][c], vm[c], vs_[c], dv[3][c], vm[c]);
            }
            if (!whole) {
                const uint32_t m0 = (4 * kgp + 0 < nlen ? 0x0000FFFFu : 0u) | (4 * kgp + 1 < nlen ? 0xFFFF0000u : 0u);
                const uint32_t m1 = (4 * kgp + 2 < nlen ? 0x0000FFFFu : 0u) | (4 * kgp + 3 < nlen ? 0xFFFF0000u : 0u);
#pragma unroll
                for (int c = 0; c < 4; ++c) { vcell[c].x &= m0; vcell[c].y &= m1; }
            }
#pragma unroll
            for (int c = 0; c < 4; ++c)
                *reinterpret_cast<uint2*>(Vt + (4 * cg + c) * kKeys + 4 * (kgp ^ (cg & 7))) = vcell[c];
        }
        __syncthreads();
        fetch(t + 2, rk, rv, ref);

        // ---- S = Q K^T: this wave's 16 keys, its half of the channels; a K operand serves every row block ----
        {
            f4_t sc[RB];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) sc[rb] = f4_t{0.f, 0.f, 0.f, 0.f};
            const _Float16* kp = Ks + (16 * kf + n16) * KROW + dh * (D / 2) + 4 * kg;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                const h4_t kb = *reinterpret_cast<const h4_t*>(kp + 16 * ks);
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) sc[rb] = __builtin_amdgcn_mfma_f32_16x16x16f16(qa[rb][ks], kb, sc[rb], 0, 0, 0);
            }
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int e = 0; e < 4; ++e) Ss[((2 * rb + dh) * kRows + 4 * kg + e) * kSStride + 16 * kf + n16] = sc[rb][e];
        }
        __syncthreads();

        // ---- softmax, once per workgroup: wave w takes rows 4 w .. 4 w + 3 of every block, sixteen lanes a row, two keys
        //      a lane; the probabilities (fp16) and the rows' rescale factors go to LDS for all four waves ----
        {
            // every key of the tile counts for every row of the workgroup (rows past n_rows compute on zeros, never stored)
            const bool all_seen = nlen == kKeys && start + kKeys - 1 <= qmin;
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const int prow = rb * kRows + srow;                // row within the workgroup
                const bool srow_ok = row0 + prow < a.n_rows;
                const int sqpos = a.q_pos0 + (srow_ok ? (row0 + prow) / a.G : 0);
                const float2 sa = *reinterpret_cast<const float2*>(Ss + ((2 * rb) * kRows + srow) * kSStride + 2 * kpair);
                const float2 sb = *reinterpret_cast<const float2*>(Ss + ((2 * rb + 1) * kRows + srow) * kSStride + 2 * kpair);
                const bool ok0 = all_seen || (srow_ok && 2 * kpair < nlen && start + 2 * kpair <= sqpos);
                const bool ok1 = all_seen || (srow_ok && 2 * kpair + 1 < nlen && start + 2 * kpair + 1 <= sqpos);
                const float sv0 = ok0 ? (sa.x + sb.x) * a.scale : -INFINITY, sv1 = ok1 ? (sa.y + sb.y) * a.scale : -INFINITY;
                const float mx = row_max16(fmaxf(sv0, sv1));
                const float m_new = fmaxf(m_run[rb], mx);
                const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                const _Float16 p0 = (_Float16)(sv0 == -INFINITY ? 0.f : __expf(sv0 - m_safe));
                const _Float16 p1 = (_Float16)(sv1 == -INFINITY ? 0.f : __expf(sv1 - m_safe));
                const float sum = row_sum16((float)p0 + (float)p1);    // the rounded p, as the second product sees it
                const float alpha = m_run[rb] == -INFINITY ? 0.f : (m_new == m_run[rb] ? 1.f : __expf(m_run[rb] - m_safe));
                l_run[rb] = l_run[rb] * alpha + sum;
                m_run[rb] = m_new;
                typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
                *reinterpret_cast<h2_t*>(Ps + prow * kPStride + 2 * kpair) = h2_t{p0, p1};
                if (kpair == 0) Al[prow] = alpha;
            }
        }
        __syncthreads();
        // ---- O = alpha O + P V; the accumulator holds rows 4 kg + e of channel n16 of each fragment; a V operand serves
        //      every row block ----
        h4_t pa[RB][2];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            pa[rb][0] = *reinterpret_cast<const h4_t*>(Ps + (rb * kRows + n16) * kPStride + 4 * kg);
            pa[rb][1] = *reinterpret_cast<const h4_t*>(Ps + (rb * kRows + n16) * kPStride + 16 + 4 * kg);
            const f4_t ae = *reinterpret_cast<const f4_t*>(Al + rb * kRows + 4 * kg);
            if (__builtin_amdgcn_ballot_w64(ae[0] != 1.f || ae[1] != 1.f || ae[2] != 1.f || ae[3] != 1.f)) {
#pragma unroll
                for (int f = 0; f < NF; ++f)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[rb][f][e] *= ae[e];
            }
        }
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int f = 0; f < NF; ++f) {
                const int ch = wave * (D / 4) + 16 * f + n16;
                const h4_t b = *reinterpret_cast<const h4_t*>(Vt + ch * kKeys + 4 * ((4 * kk + kg) ^ ((ch >> 2) & 7)));
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) acc[rb][f] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa[rb][kk], b, acc[rb][f], 0, 0, 0);
            }
        __syncthreads();                                  // the tile in LDS is free again
    };

    if (t0 < t1) {
        U rk0[UNITS][4], rv0[UNITS][4], rk1[UNITS][4], rv1[UNITS][4];
        TileRef ref0, ref1;
        fetch(t0, rk0, rv0, ref0);
        __builtin_amdgcn_sched_barrier(0);                 // set 0 is the older one, as in every later round of the loop
        fetch(t0 + 1, rk1, rv1, ref1);
        __builtin_amdgcn_sched_barrier(0);
        // The loop has one way out, at its head, and takes tiles in pairs; when the last pair has no second tile, that
        // one is run as an empty tile (no key counts: nothing changes).  A way out of the middle would be turned into a
        // path through the loop's end back to its head, on which set 0 is the younger one, and the compiler would make
        // every round wait for both sets; a copy of the tile's code behind the loop costs registers that end in scratch.
        for (int t = t0; ref0.ok; t += 2) {
            tile(t, rk0, rv0, ref0);
            tile(t + 1, rk1, rv1, ref1);
        }
    }

    // Where the results go is worked out only now, from a thread index the compiler cannot connect with the one above:
    // otherwise it computes the addresses before the loop and, short of registers, parks them in scratch memory (measured:
    // 5.6 MB written and read back per launch).
    int tid_e = threadIdx.x;
    asm volatile("" : "+v"(tid_e));
    const int lane_e = tid_e & 63, wave_e = tid_e >> 6, n16_e = lane_e & 15, kg_e = lane_e >> 4;
    const int64_t base = ((int64_t)sp * a.nhkv + h) * a.n_rows;
    const int srow_e = 4 * wave_e + kg_e;                    // the row (of every block) whose softmax state this lane holds
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
        for (int f = 0; f < NF; ++f)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int r = row0 + rb * kRows + 4 * kg_e + e;
                if (r < a.n_rows) a.o[(base + r) * D + wave_e * (D / 4) + 16 * f + n16_e] = acc[rb][f][e];
            }
        const int r = row0 + rb * kRows + srow_e;
        if (n16_e == 0 && r < a.n_rows) {
            a.m[base + r] = m_run[rb];
            a.l[base + r] = l_run[rb];
        }
    }
}

// Splits -> the normalised result and the log-sum-exp.  One workgroup per (kv head, row, 16 channels): 64 groups of 4
// threads share the splits (group g takes splits g, g + 64, ...), a thread holds four channels; the groups' maxima,
// sums and partial results meet in LDS.  A thread has a few independent loads, so the launch costs a few trips to
// memory, not one per split.
__global__ __launch_bounds__(256) void attn_combine_kernel(const float* __restrict__ o, const float* __restrict__ m, const float* __restrict__ l,
                                                            int n_splits, int nhkv, int n_rows, int D, int G,
                                                            float* __restrict__ out, float* __restrict__ lse) {
    __shared__ float s_top[64], s_total[64];
    __shared__ __align__(16) float s_acc[64][16];
    const int h = blockIdx.x / n_rows, r = blockIdx.x % n_rows;
    const int grp = threadIdx.x >> 2, cl = threadIdx.x & 3, ch = blockIdx.y * 16 + cl * 4;
    const int64_t hr = (int64_t)h * n_rows + r, stride = (int64_t)nhkv * n_rows;
    float top = -INFINITY;
    for (int s = grp; s < n_splits; s += 64) top = fmaxf(top, m[s * stride + hr]);
    if (cl == 0) s_top[grp] = top;
    __syncthreads();
#pragma unroll
    for (int g = 0; g < 64; ++g) top = fmaxf(top, s_top[g]);
    if (top == -INFINITY) top = 0.f;
    float total = 0.f;
    f4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int s = grp; s < n_splits; s += 64) {
        const float w = expf(m[s * stride + hr] - top);
        total += (l ? l[s * stride + hr] : 1.f) * w;
        if (ch < D) acc += *reinterpret_cast<const f4_t*>(o + (s * stride + hr) * D + ch) * w;
    }
    if (cl == 0) s_total[grp] = total;
    *reinterpret_cast<f4_t*>(&s_acc[grp][cl * 4]) = acc;
    __syncthreads();
    if (grp == 0) {
        total = 0.f;
        acc = f4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
        for (int g = 0; g < 64; ++g) {                    // fixed order: the result does not depend on timing
            total += s_total[g];
            acc += *reinterpret_cast<const f4_t*>(&s_acc[g][cl * 4]);
        }
        const int tok = r / G, qh = h * G + r % G;
        const int64_t dst = (int64_t)tok * (nhkv * G) + qh;
        if (ch < D) *reinterpret_cast<f4_t*>(out + dst * D + ch) = acc * (1.f / fmaxf(total, 1e-30f));
        if (cl == 0 && blockIdx.y == 0) lse[dst] = total > 0.f ? top + logf(fmaxf(total, 1e-30f)) : -INFINITY;
    }
}

template <int D, typename T>
int launch_attn(const AttnArgs& a, int64_t n_splits, hipStream_t s) {
    // up to 16 rows: one block per workgroup; up to 32: two; beyond: four with 128 channels, two with 256 (four blocks'
    // accumulators and Q do not fit the registers there).  QVB8_ATTN_ROW_BLOCKS forces 1, 2 or 4.
    int rb = a.n_rows <= kRows ? 1 : a.n_rows <= 2 * kRows ? 2 : 4;
    const int forced = host::env_int("QVB8_ATTN_ROW_BLOCKS", 0);
    if (forced == 1 || forced == 2 || forced == 4) rb = forced;
    if (D == 256 && rb > 2) rb = 2;
    const dim3 grid((unsigned)a.nhkv, (unsigned)n_splits, (unsigned)((a.n_rows + rb * kRows - 1) / (rb * kRows)));
    if (grid.z > 65535u) return host::fail(-1, "qvb8_attn_fwd: %d rows are more than one launch takes", a.n_rows);
    if (rb == 1) hipLaunchKernelGGL((attn_kernel<D, T, 1>), grid, dim3(kAttnThreads), 0, s, a);
    else if (rb == 2) hipLaunchKernelGGL((attn_kernel<D, T, 2>), grid, dim3(kAttnThreads), 0, s, a);
    else if constexpr (D == 128) hipLaunchKernelGGL((attn_kernel<D, T, 4>), grid, dim3(kAttnThreads), 0, s, a);
    return host::check_launch("qvb8_attn_fwd");
}

bool aligned(const void* p, uintptr_t n) { return (reinterpret_cast<uintptr_t>(p) & (n - 1)) == 0; }

}  // namespace
}  // namespace qvb8

extern "C" int qvb8_attn_fwd(const void* q, int64_t sq_r, int64_t sq_h, const void* ki, const void* vi, int id_bytes,
                             int64_t s_n, int64_t s_h, const float* kmid, const float* kstep, const float* vmid,
                             const float* vstep, const float* kc, const float* vc, const int32_t* ts, const int32_t* tl,
                             const int32_t* tseg, int64_t n_tiles, float* o, float* m, float* l, int64_t n_splits,
                             int64_t n_rows, int64_t n_kv_heads, int64_t head_dim, int64_t q_pos0, int64_t tps,
                             double scale, int64_t G, void* stream) {
    using namespace qvb8;
    const char* who = "qvb8_attn_fwd";
    if (head_dim != 128 && head_dim != 256) return host::fail(-1, "%s: head_dim must be 128 or 256, got %lld", who, (long long)head_dim);
    if (id_bytes != 1 && id_bytes != 2) return host::fail(-1, "%s: ids are 1 or 2 bytes wide, got %d", who, id_bytes);
    if (n_rows < 0 || n_tiles < 0 || n_splits < 1 || tps < 1 || G < 1 || n_kv_heads < 1)
        return host::fail(-1, "%s: negative or zero size (rows %lld, tiles %lld, splits %lld, tiles per split %lld, G %lld, kv heads %lld)",
                          who, (long long)n_rows, (long long)n_tiles, (long long)n_splits, (long long)tps, (long long)G, (long long)n_kv_heads);
    if (n_rows % G != 0) return host::fail(-1, "%s: %lld rows are not whole tokens of %lld heads", who, (long long)n_rows, (long long)G);
    if (n_splits * tps < n_tiles) return host::fail(-1, "%s: %lld splits of %lld tiles do not cover %lld tiles", who, (long long)n_splits, (long long)tps, (long long)n_tiles);
    if (n_rows == 0) return 0;
    if (!q || !o || !m || !l) return host::fail(-1, "%s: null q / o / m / l", who);
    if (n_tiles > 0 && (!ki || !vi || !kmid || !kstep || !vmid || !vstep || !kc || !vc || !ts || !tl || !tseg))
        return host::fail(-1, "%s: null ids, constants or tile table", who);
    if (!aligned(q, 8) || (sq_r & 3) || (sq_h & 3)) return host::fail(-1, "%s: q must be 8-byte aligned with strides that are multiples of 4", who);
    if (n_tiles > 0) {
        if (!aligned(ki, 4 * id_bytes) || !aligned(vi, 4 * id_bytes) || (s_n & 3) || (s_h & 3))
            return host::fail(-1, "%s: ids must be aligned to four ids with strides that are multiples of 4", who);
        if (!aligned(kmid, 16) || !aligned(kstep, 16) || !aligned(vmid, 16) || !aligned(vstep, 16))
            return host::fail(-1, "%s: the per-channel constants must be 16-byte aligned", who);
    }
    if (n_tiles > 0 && (s_n < 0 || s_n * 32 * id_bytes > INT32_MAX)) return host::fail(-1, "%s: key stride %lld out of range", who, (long long)s_n);
    const int64_t row_blocks = (n_rows + kRows - 1) / kRows;
    if (n_splits > 65535 || row_blocks > 65535 || n_tiles > INT32_MAX || n_rows > INT32_MAX || q_pos0 > INT32_MAX / 2 || q_pos0 < INT32_MIN / 2)
        return host::fail(-1, "%s: size beyond what one launch takes", who);
    AttnArgs a;
    a.q = static_cast<const uint16_t*>(q); a.sq_r = sq_r; a.sq_h = sq_h;
    a.ki = ki; a.vi = vi; a.s_n = s_n; a.s_h = s_h;
    a.kmid = kmid; a.kstep = kstep; a.vmid = vmid; a.vstep = vstep; a.kc = kc; a.vc = vc;
    a.ts = ts; a.tl = tl; a.tseg = tseg; a.o = o; a.m = m; a.l = l;
    a.q_pos0 = (int)q_pos0; a.n_tiles = (int)n_tiles; a.tps = (int)std::min<int64_t>(INT32_MAX / 2, tps); a.n_rows = (int)n_rows;
    a.G = (int)G; a.nhkv = (int)n_kv_heads; a.scale = (float)scale;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (head_dim == 256) return id_bytes == 1 ? launch_attn<256, uint8_t>(a, n_splits, s) : launch_attn<256, uint16_t>(a, n_splits, s);
    return id_bytes == 1 ? launch_attn<128, uint8_t>(a, n_splits, s) : launch_attn<128, uint16_t>(a, n_splits, s);
}

extern "C" int qvb8_attn_combine(const float* o, const float* m, const float* l, int64_t n_splits, int64_t n_kv_heads,
                                 int64_t n_rows, int64_t head_dim, int64_t G, float* out, float* lse, void* stream) {
    using namespace qvb8;
    const char* who = "qvb8_attn_combine";
    if (n_splits < 1 || n_kv_heads < 1 || n_rows < 0 || G < 1 || head_dim < 4 || head_dim % 4 != 0)
        return host::fail(-1, "%s: bad size (splits %lld, kv heads %lld, rows %lld, G %lld, head_dim %lld)", who, (long long)n_splits,
                          (long long)n_kv_heads, (long long)n_rows, (long long)G, (long long)head_dim);
    if (n_rows % G != 0) return host::fail(-1, "%s: %lld rows are not whole tokens of %lld heads", who, (long long)n_rows, (long long)G);
    if (n_rows == 0) return 0;
    if (!o || !m || !out || !lse) return host::fail(-1, "%s: null pointer", who);
    if (!aligned(o, 16) || !aligned(out, 16)) return host::fail(-1, "%s: o and out must be 16-byte aligned", who);
    if (n_kv_heads * n_rows > INT32_MAX || n_splits > INT32_MAX) return host::fail(-1, "%s: size beyond what one launch takes", who);
    hipLaunchKernelGGL(attn_combine_kernel, dim3((unsigned)(n_kv_heads * n_rows), (unsigned)((head_dim + 15) / 16)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       o, m, l, (int)n_splits, (int)n_kv_heads, (int)n_rows, (int)head_dim, (int)G, out, lse);
    return host::check_launch(who);
}
