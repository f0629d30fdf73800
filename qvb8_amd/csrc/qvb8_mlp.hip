// One launch for the MLP of a decoder layer at decode (gfx950):  Y = down( act(gate(x)) * up(x) ),  1..4 rows of x.
//
// Launched one after the other, the gate+up product and the down product each pay a launch's fixed cost -- the gap between
// two kernels, the first trip for the activations, the first trip for the ids, the drain -- during which no weight byte
// moves.  Here both run in ONE grid of one workgroup per CU (all resident at once), and the hand-over happens inside it:
//
//   phase 1   every workgroup multiplies its share of the gate and up rows (16 gate rows and the 16 matching up rows are
//             a UNIT, multiplied by the two halves of the workgroup side by side, so gate and up of an output meet in one
//             workgroup) and, before it finishes them, REQUESTS the first ids of its down rows -- weights do not depend
//             on activations;
//   hand-over the workgroup writes its H = act(gate) * up values to memory, each 16-bit value in a dword of its own
//             together with a 16-bit tag of this call (one 4-byte store: a reader sees the value and its tag or neither);
//             four of its sixteen waves then read ALL of H (every workgroup's), asking again for the pieces whose tag is
//             not yet this call's, and leave it in LDS -- one trip through memory, no flag to wait for first, no fence.
//             The wait is BOUNDED: when a piece has not arrived after `wait_ticks` the workgroup gives up, writes NaN as
//             its results and raises the error word of the workspace -- it never spins without end;
//   phase 2   the sixteen waves multiply the workgroup's down rows against H from LDS (the ids asked for in phase 1 have
//             landed meanwhile) and write Y.
//
// Loads return to a wave in the order it asked, so a wave that has ids in flight cannot see H before those ids: the four
// waves that read H ask for their own ids only afterwards.
// Values are those of the separate launches: gate and up results rounded to the caller's type, act in fp32 rounded to it,
// the product rounded to it, then narrowed to saturated fp16 like every activation of the fp16 paths.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "../../include/qvb8_amd.h"
#include "qvb8_device.h"
#include "qvb8_host.h"
#include "qvb8_mma_device.h"

namespace qvb8 {

constexpr int kMlpWaves = 16, kMlpThreads = 64 * kMlpWaves;
constexpr int kMlpLoaders = 4;              // waves that read H for their workgroup
constexpr int kMlpPieces = 24;              // 8-byte pieces of H a lane of those waves holds at a time
constexpr int kMlpTileWaves = 8;            // phase 1: waves per 16-row tile (the gate tile and the up tile side by side)
// The workspace: 16 state words, then H as tagged dwords, one region per row count (rows of M: M x I dwords at
// I * M (M - 1) / 2), so that a region is rewritten completely by every call that reads it.
//   state[0] workgroups of the running call that are done reading H    state[1] error (sticky)   state[2 + M - 1] calls made with M rows
constexpr int kMlpStateWords = 16;

// One weight of the block: rows stored in planes, in position order (position -> output row through fin), at most three
// runs of one width each, every run a whole number of tiles.
struct MlpSide {
    const uint8_t* ids;
    const uint4* fin;             // per position: tau_s bits, min_s bits, output row, 0
    int Q, P;
    int first1, first2;           // positions where the second and the third width start (Q when there is none)
    uint32_t widths;              // nb0 | nb1 << 8 | nb2 << 16
};

struct MlpArgs {
    const uint16_t* X;            // (M, hidden) fp16, or bf16 with x_bf16
    MlpSide up, dn;
    uint32_t* state;
    void* Y;
    uint32_t wait_ticks;          // bound of the wait for H in ticks of the 100 MHz clock
    int M;
    int x_bf16;                   // X is bf16: narrowed to saturated fp16 on its way into LDS
    int act_dt;                   // type the block computes in between the products: 0 fp32, 1 fp16, 2 bf16
    int out_dt;                   // what Y holds: 0 fp32, 1 fp16, 2 bf16
    int flags;                    // bit 0: H is written with the tag of another call (exercises the bounded wait)
};

// byte offset of tile `tile` (16 positions) from the start of the side's ids, and its width
__device__ __forceinline__ uint64_t mlp_tile_byte(const MlpSide& s, int tile, uint32_t& nb) {
    const int pos = tile * kTileRows;
    const uint32_t nb0 = s.widths & 255u, nb1 = (s.widths >> 8) & 255u, nb2 = (s.widths >> 16) & 255u;
    const int c = (pos >= s.first1 ? 1 : 0) + (pos >= s.first2 ? 1 : 0);
    const uint64_t P64 = (uint64_t)s.P;
    const uint64_t base1 = (uint64_t)s.first1 * P64 * nb0;
    const uint64_t base2 = base1 + (uint64_t)(s.first2 - s.first1) * P64 * nb1;
    nb = c == 0 ? nb0 : c == 1 ? nb1 : nb2;
    const uint64_t bit0 = (c == 0 ? 0 : c == 1 ? base1 : base2) + (uint64_t)(pos - (c == 0 ? 0 : c == 1 ? s.first1 : s.first2)) * P64 * nb;
    return bit0 >> 3;
}

// The lane's slices of T steps of a tile in planes: 2 T non-temporal 16-byte loads, none under a branch, every address
// inside the buffer (a wave without the tile, and steps past the row's end, read the buffer's first 32 bytes).
template <int T>
__device__ __forceinline__ void mlp_issue(const uint8_t* __restrict__ ids, uint64_t tile_byte, uint32_t nb, int step0, int n_steps, bool has,
                                          int lane, uint4 (&lo)[T], uint4 (&hi)[T]) {
    const uint64_t lo0 = tile_byte + (uint64_t)lane * 16u;
    const uint64_t hi0 = tile_byte + 1024u + (uint64_t)lane * (4u * (nb - 4u)) + 4u * (nb - 4u) - 16u;
    const uint32_t step_bytes = 256u * nb;
#pragma unroll
    for (int it = 0; it < T; ++it) {
        const bool use = has && (step0 + it) < n_steps;
        const uint64_t at = (uint64_t)(step0 + it) * step_bytes;
        const v4u_t va = __builtin_nontemporal_load(reinterpret_cast<const v4u_t*>(ids + (use ? lo0 + at : 0)));
        const v4u_t vb = __builtin_nontemporal_load(reinterpret_cast<const v4u_t*>(ids + (use ? hi0 + at : 16)));
        lo[it] = uint4{va.x, va.y, va.z, va.w};
        hi[it] = uint4{vb.x, vb.y, vb.z, vb.w};
    }
}

// T steps of a tile against the activations in LDS (rows of `P` fp16 values; lanes without a row of X, and steps past the
// row's end, read the 64 bytes of zeros at x_zero).  `sums`: the row sums of X over these steps are added to sx as well.
template <int T>
__device__ __forceinline__ void mlp_multiply(uint32_t nb, const uint4 (&lo)[T], const uint4 (&hi)[T], const unsigned char* xs, uint32_t P,
                                             uint32_t x_zero, int M, int step0, int n_steps, bool sums, int r, int kg, v4f_t& sx, v4f_t& acc) {
    using F = Fmt<false>;
    const v4u_t ones = {F::one_bits, F::one_bits, F::one_bits, F::one_bits};
#pragma unroll
    for (int it = 0; it < T; ++it) {
        v4u_t xv[4], b[4];
        const bool on = r < M && (step0 + it) < n_steps;
        const uint32_t at = on ? 2u * ((uint32_t)r * P + (uint32_t)(step0 + it) * kStepCols + (uint32_t)kg * 32u) : x_zero;
#pragma unroll
        for (int j = 0; j < 4; ++j) xv[j] = *reinterpret_cast<const v4u_t*>(xs + at + 16 * j);
        if (sums) {
#pragma unroll
            for (int j = 0; j < 4; ++j) sx = F::mfma(xv[j], ones, sx);
        }
        switch (nb) {
            case 7: decode_slice<7, false>(lo[it], hi[it], b); break;
            case 6: decode_slice<6, false>(lo[it], hi[it], b); break;
            case 5: decode_slice<5, false>(lo[it], hi[it], b); break;
            case 4: decode_slice<4, false>(lo[it], hi[it], b); break;
            default: decode_slice<8, false>(lo[it], hi[it], b); break;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = F::mfma(xv[j], b[j], acc);
    }
}

__device__ __forceinline__ float mlp_round(float v, int dt) {
    if (dt == 1) return f16_bits_to_f32(f32_to_f16_bits(v));
    if (dt == 2) return bf16_bits_to_f32(f32_to_bf16_bits(v));
    return v;
}

// H of one output: gate and up results as the separate launches hand them on (rounded to the block's type), SiLU in fp32
// rounded to it, the product rounded to it, then saturated fp16 -- the chain gate_proj -> act_fn -> * up_proj -> down_proj's
// activation narrowing of the reference's MLP.
__device__ __forceinline__ uint32_t mlp_h_bits(float yg, float yu, int dt) {
    const float g = mlp_round(yg, dt), u = mlp_round(yu, dt);
    const float s = mlp_round(g / (1.0f + expf(-g)), dt);
    float h = s * u;
    asm("" : "+v"(h));                                          // the product is rounded on its own, never fused into what follows
    return sat_half_bits(mlp_round(h, dt));
}

__device__ __forceinline__ void mlp_bare_barrier() {
    // waits for this wave's LDS traffic only: __syncthreads() carries a fence that would also wait for the ids in flight
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

__device__ __forceinline__ void mlp_store_y(void* Y, int out_dt, int64_t i, float v) {
    if (out_dt == 0) store_from_f32<0>(Y, i, v);
    else if (out_dt == 1) store_from_f32<1>(Y, i, v);
    else store_from_f32<2>(Y, i, v);
}

// T1 / T2: steps of 128 columns a wave owns per panel in phase 1 / 2; XP: 16-byte pieces of X per thread.
template <int T1, int T2, int XP>
__global__ void __launch_bounds__(kMlpThreads) mlp_kernel(MlpArgs a) {
    using F = Fmt<false>;
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, kg = lane >> 4;
    const int M = a.M;
    // workgroup b runs on XCD b % 8: the workgroups of one XCD take neighbouring units and tiles
    const int nblk = (int)gridDim.x;
    const int vb = (nblk & 7) == 0 ? ((int)blockIdx.x & 7) * (nblk >> 3) + ((int)blockIdx.x >> 3) : (int)blockIdx.x;
    const int units = a.up.Q >> 5, tiles2 = a.dn.Q >> 4;
    const int n_units = vb < units ? (units - 1 - vb) / nblk + 1 : 0;        // local unit lu is global unit lu * nblk + vb
    const int n_tiles2 = vb < tiles2 ? (tiles2 - 1 - vb) / nblk + 1 : 0;
    const int U1 = (units + nblk - 1) / nblk, TW2 = (tiles2 + nblk - 1) / nblk;
    const int P1 = a.up.P, I = a.dn.P;
    const int n_steps1 = P1 >> 7, ranges1 = (n_steps1 + T1 - 1) / T1, panels1 = (ranges1 + kMlpTileWaves - 1) / kMlpTileWaves;
    const int n_steps2 = I >> 7, ranges2 = (n_steps2 + T2 - 1) / T2, panels2 = (ranges2 + kMlpWaves - 1) / kMlpWaves;

    // ---- LDS ----
    uint4* s_fin1 = reinterpret_cast<uint4*>(smem);                                      // [U1 * 32]
    uint4* s_fin2 = s_fin1 + U1 * 32;                                                    // [TW2 * 16]
    float* sxs1 = reinterpret_cast<float*>(s_fin2 + TW2 * 16);                           // [8][16]
    float* sxs2 = sxs1 + kMlpTileWaves * 16;                                             // [16][16]
    float* part1 = sxs2 + kMlpWaves * 16;                                                // [U1 * 32][8][M]
    float* part2 = part1 + (size_t)U1 * 32 * kMlpTileWaves * M;                          // [TW2 * 16][16][M]
    uint32_t* s_flag = reinterpret_cast<uint32_t*>(part2 + (size_t)TW2 * 16 * kMlpWaves * M);    // [4]
    unsigned char* xs1 = reinterpret_cast<unsigned char*>(s_flag + 4);                   // [M][P1] fp16, 64 bytes of zeros behind
    const uint32_t x1_zero = (uint32_t)M * (uint32_t)P1 * 2u;
    unsigned char* xs2 = xs1 + x1_zero + 64;                                             // [M][I] fp16, 64 bytes of zeros behind
    const uint32_t x2_zero = (uint32_t)M * (uint32_t)I * 2u;

    // ---- first requests: X, the rows' end-of-tile records, the call count, the first ids ----
    const int x_pieces = (M * P1) >> 3;
    v4u_t xg[XP];
    {
        const v4u_t* xsrc = reinterpret_cast<const v4u_t*>(a.X);
#pragma unroll
        for (int i = 0; i < XP; ++i) xg[i] = xsrc[min(tid + i * kMlpThreads, x_pieces - 1)];
        __builtin_amdgcn_sched_barrier(0);
    }
    uint4 f1 = {0u, 0u, 0xffffffffu, 0u}, f2 = {0u, 0u, 0xffffffffu, 0u};
    {
        const bool h1 = tid < n_units * 32;
        const uint4 v1 = a.up.fin[h1 ? ((tid >> 5) * nblk + vb) * 32 + (tid & 31) : 0];
        if (h1) f1 = v1;
        const bool h2 = tid < n_tiles2 * kTileRows;
        const uint4 v2 = a.dn.fin[h2 ? ((tid >> 4) * nblk + vb) * kTileRows + (tid & 15) : 0];
        if (h2) f2 = v2;
    }
    // calls made so far with this row count (one thread asks; the workgroup shares the answer through LDS)
    uint32_t calls_here = 0;
    if (tid == 0) calls_here = __hip_atomic_load(a.state + 2 + (M - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int g = wave >> 3, wc = wave & 7;                       // phase 1: g = 0 the unit's gate tile, 1 its up tile
    uint4 lo[T1], hi[T1];
    uint32_t nb_cur;
    {
        const uint64_t tb = mlp_tile_byte(a.up, 2 * vb + g, nb_cur);
        mlp_issue<T1>(a.up.ids, tb, nb_cur, wc * T1, n_steps1, n_units > 0, lane, lo, hi);
    }
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        const int idx = tid + i * kMlpThreads;
        v4u_t v = xg[i];
        if (a.x_bf16) {
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = XIn<false, true>::pair(v[k]);
        }
        if (idx < x_pieces) reinterpret_cast<v4u_t*>(xs1)[idx] = v;
        __builtin_amdgcn_sched_barrier(0);
    }
    if (tid < 16) {
        reinterpret_cast<uint32_t*>(xs1 + x1_zero)[tid] = 0u;
        reinterpret_cast<uint32_t*>(xs2 + x2_zero)[tid] = 0u;
    }
    if (tid < 4) s_flag[tid] = 0u;                                // [0] a wait for H ran out
    if (tid == 0) s_flag[1] = calls_here;                         // (the same thread's second store: it stays)
    if (tid < U1 * 32) s_fin1[tid] = f1;
    if (tid < TW2 * kTileRows) s_fin2[tid] = f2;
    mlp_bare_barrier();

    // ---- phase 1: gate and up ----
    for (int panel = 0; panel < panels1; ++panel) {
        const int range = panel * kMlpTileWaves + wc, step0 = range * T1;
        const int n_mine = step0 < n_steps1 ? n_units : 0;
        const bool first_panel = panel == 0;
        const bool more = n_units > 0 && panel + 1 < panels1 && (range + kMlpTileWaves) * T1 < n_steps1;
        v4f_t sx = {0.f, 0.f, 0.f, 0.f};
        for (int lu = 0; lu < n_mine; ++lu) {
            v4f_t acc = {0.f, 0.f, 0.f, 0.f};
            mlp_multiply<T1>(nb_cur, lo, hi, xs1, (uint32_t)P1, x1_zero, M, step0, n_steps1, lu == 0, r, kg, sx, acc);
            if (lu + 1 < n_mine) {
                const uint64_t tb = mlp_tile_byte(a.up, 2 * ((lu + 1) * nblk + vb) + g, nb_cur);
                mlp_issue<T1>(a.up.ids, tb, nb_cur, step0, n_steps1, true, lane, lo, hi);
            } else if (more) {
                const uint64_t tb = mlp_tile_byte(a.up, 2 * vb + g, nb_cur);
                mlp_issue<T1>(a.up.ids, tb, nb_cur, step0 + kMlpTileWaves * T1, n_steps1, true, lane, lo, hi);
            }
            if (lu == 0 && g == 0 && r == 0) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float* dst = sxs1 + wc * 16 + kg * 4 + e;
                    *dst = first_panel ? sx[e] : *dst + sx[e];
                }
            }
            const int lrow = lu * 32 + g * 16 + r;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int t = kg * 4 + e;
                const float v = __builtin_fmaf(-F::bias, sx[e], acc[e]);
                if (t < M) {
                    float* dst = part1 + ((size_t)lrow * kMlpTileWaves + wc) * M + t;
                    *dst = first_panel ? v : *dst + v;
                }
            }
        }
    }
    // ---- the first ids of the down rows, asked for before the hand-over by the waves that will not read H ----
    const bool loader = wave < kMlpLoaders;
    uint4 lo2[T2], hi2[T2];
    uint32_t nb2;
    const uint64_t tb2_first = mlp_tile_byte(a.dn, vb, nb2);
    if (!loader) mlp_issue<T2>(a.dn.ids, tb2_first, nb2, wave * T2, n_steps2, n_tiles2 > 0, lane, lo2, hi2);
    mlp_bare_barrier();

    // ---- hand-over, writing side: H of this workgroup's units, a thread per (output, token, column range) ----
    const uint32_t calls = s_flag[1];
    const uint32_t tag = calls % 65535u + 1u;                     // never 0: a workspace starts as zeros
    const uint32_t tag_w = ((a.flags & 1) ? (tag % 65535u + 1u) : tag) << 16;
    uint32_t* Hreg = a.state + kMlpStateWords + (size_t)I * (size_t)(M * (M - 1) / 2);
    {
        const int valid1 = ranges1 < kMlpTileWaves ? ranges1 : kMlpTileWaves;
        const int items1 = n_units * kTileRows * M;
        for (int first = wave * 4; first < items1; first += kMlpWaves * 4) {
            const int i = first + (lane >> 4), w = lane & 15;
            const bool item = i < items1;
            const int rl = item ? i / M : 0, t = item ? i - rl * M : 0;
            const int grow = (rl >> 4) * 32 + (rl & 15), urow = grow + 16;
            const bool live = item && w < valid1;
            const int wr = live ? w : 0;
            const float pg = part1[((size_t)grow * kMlpTileWaves + wr) * M + t], pu = part1[((size_t)urow * kMlpTileWaves + wr) * M + t];
            const float sv = sxs1[wr * 16 + t];
            const double dg = row16_sum(live ? (double)pg : 0.0), du = row16_sum(live ? (double)pu : 0.0), xsum = row16_sum(live ? (double)sv : 0.0);
            if (item && w == 0) {
                const uint4 fg = s_fin1[grow], fu = s_fin1[urow];
                const float yg = (float)((double)__uint_as_float(fg.x) * dg + (double)__uint_as_float(fg.y) * xsum);
                const float yu = (float)((double)__uint_as_float(fu.x) * du + (double)__uint_as_float(fu.y) * xsum);
                uint32_t h = mlp_h_bits(yg, yu, a.act_dt);
                if (fu.z != fg.z + (uint32_t)I) h = 0x7E00u;         // the up row of this place is not the gate row's partner
                if (fg.z < (uint32_t)I) __hip_atomic_store(Hreg + (size_t)t * I + fg.z, h | tag_w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    // ---- hand-over, reading side: four waves read all of H, piece by piece until every piece carries this call's tag ----
    if (loader && n_tiles2 > 0) {
        const uint64_t* H64 = reinterpret_cast<const uint64_t*>(Hreg);
        uint32_t* xw = reinterpret_cast<uint32_t*>(xs2);
        const int n64 = (M * I) >> 1;
        const uint64_t t0 = wall_clock64();
        bool failed = false;
        for (int base = 0; base < n64 && !failed; base += kMlpLoaders * 64 * kMlpPieces) {
            uint64_t v[kMlpPieces];
            uint32_t need = 0;
#pragma unroll
            for (int i = 0; i < kMlpPieces; ++i)
                if (base + (i * kMlpLoaders + wave) * 64 + lane < n64) need |= 1u << i;
            for (;;) {
#pragma unroll
                for (int i = 0; i < kMlpPieces; ++i)
                    if ((need >> i) & 1u) v[i] = __hip_atomic_load(H64 + base + (i * kMlpLoaders + wave) * 64 + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int i = 0; i < kMlpPieces; ++i) {
                    if ((need >> i) & 1u) {
                        const uint32_t d0 = (uint32_t)v[i], d1 = (uint32_t)(v[i] >> 32);
                        if ((d0 >> 16) == tag && (d1 >> 16) == tag) {
                            need &= ~(1u << i);
                            xw[base + (i * kMlpLoaders + wave) * 64 + lane] = (d0 & 0xFFFFu) | (d1 << 16);
                        }
                    }
                }
                if (__builtin_amdgcn_ballot_w64(need != 0u) == 0) break;
                if (wall_clock64() - t0 > (uint64_t)a.wait_ticks) { failed = true; break; }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        if (failed && lane == 0) s_flag[0] = 1u;
        mlp_issue<T2>(a.dn.ids, tb2_first, nb2, wave * T2, n_steps2, true, lane, lo2, hi2);
    }
    mlp_bare_barrier();
    const bool bad = s_flag[0] != 0u;
    // this workgroup needs H no more: count it (the answer is looked at when the kernel ends)
    uint32_t done_before = 0;
    if (tid == 0) done_before = __hip_atomic_fetch_add(a.state, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // ---- phase 2: down ----
    for (int panel = 0; panel < panels2; ++panel) {
        // odd panels start at wave 8: a last panel that is not full then goes to waves that had their first ids early
        const int range = panel * kMlpWaves + ((wave + 8 * panel) & 15), step0 = range * T2;
        const int next_step0 = ((panel + 1) * kMlpWaves + ((wave + 8 * (panel + 1)) & 15)) * T2;
        const int n_mine = step0 < n_steps2 ? n_tiles2 : 0;
        const bool first_panel = panel == 0;
        const bool more = n_tiles2 > 0 && panel + 1 < panels2 && next_step0 < n_steps2;
        v4f_t sx = {0.f, 0.f, 0.f, 0.f};
        for (int lt = 0; lt < n_mine; ++lt) {
            v4f_t acc = {0.f, 0.f, 0.f, 0.f};
            mlp_multiply<T2>(nb2, lo2, hi2, xs2, (uint32_t)I, x2_zero, M, step0, n_steps2, lt == 0, r, kg, sx, acc);
            if (lt + 1 < n_mine) {
                const uint64_t tb = mlp_tile_byte(a.dn, (lt + 1) * nblk + vb, nb2);
                mlp_issue<T2>(a.dn.ids, tb, nb2, step0, n_steps2, true, lane, lo2, hi2);
            } else if (more) {
                const uint64_t tb = mlp_tile_byte(a.dn, vb, nb2);
                mlp_issue<T2>(a.dn.ids, tb, nb2, next_step0, n_steps2, true, lane, lo2, hi2);
            }
            if (lt == 0 && r == 0) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float* dst = sxs2 + wave * 16 + kg * 4 + e;
                    *dst = first_panel ? sx[e] : *dst + sx[e];
                }
            }
            const int lrow = lt * kTileRows + r;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int t = kg * 4 + e;
                const float v = __builtin_fmaf(-F::bias, sx[e], acc[e]);
                if (t < M) {
                    float* dst = part2 + ((size_t)lrow * kMlpWaves + wave) * M + t;
                    *dst = first_panel ? v : *dst + v;
                }
            }
        }
    }
    __syncthreads();

    // ---- the down rows' results: a thread per (row, token, column range), sixteen lanes added up as a fixed tree ----
    {
        const int valid2 = ranges2 < kMlpWaves ? ranges2 : kMlpWaves;
        const int items2 = n_tiles2 * kTileRows * M;
        const int Q2 = a.dn.Q;
        for (int first = wave * 4; first < items2; first += kMlpWaves * 4) {
            const int i = first + (lane >> 4), w = lane & 15;
            const bool item = i < items2;
            const int rl = item ? i / M : 0, t = item ? i - rl * M : 0;
            const bool live = item && w < valid2;
            const int wr = live ? w : 0;
            const float pv = part2[((size_t)rl * kMlpWaves + wr) * M + t], sv = sxs2[wr * 16 + t];
            const double dsum = row16_sum(live ? (double)pv : 0.0), xsum = row16_sum(live ? (double)sv : 0.0);
            if (item && w == 0) {
                const uint4 f = s_fin2[rl];
                const float y = bad ? __builtin_nanf("") : (float)((double)__uint_as_float(f.x) * dsum + (double)__uint_as_float(f.y) * xsum);
                if (f.z < (uint32_t)Q2) mlp_store_y(a.Y, a.out_dt, (int64_t)t * Q2 + f.z, y);
            }
        }
    }
    if (tid == 0) {
        if (bad) __hip_atomic_store(a.state + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (done_before == (uint32_t)nblk - 1u) {
            // the last workgroup to let go of H closes the call: the count starts again, the next call gets the next tag
            __hip_atomic_store(a.state, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(a.state + 2 + (M - 1), calls + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

}  // namespace qvb8

using namespace qvb8;

namespace {

constexpr size_t kMlpLdsLimit = 160 * 1024;

struct MlpPlan { int T1, T2, XP, blocks; size_t lds; };

int pick_t2(int n_steps2) {
    const int forced = host::env_int("QVB8_MLP_T2", 0);
    if (forced == 3 || forced == 4) return forced;
    // the fewest padded steps over whole panels of sixteen waves; ties go to the longer burst (six steps per wave would
    // cover 12288 columns in one panel, but its 48 id registers next to the 48 of the waves that read H do not fit 128)
    int best = 4, best_cost = 1 << 30;
    for (int t : {4, 3}) {
        const int ranges = (n_steps2 + t - 1) / t, panels = (ranges + kMlpWaves - 1) / kMlpWaves;
        const int cost = panels * kMlpWaves * t;
        if (cost < best_cost) { best_cost = cost; best = t; }
    }
    return best;
}

bool side_ok(const qvb8_mma_layout* L, int64_t Q, int64_t P, int64_t ids_bytes, int unit_rows, MlpSide& s, const char** why) {
    const int n = L->n_classes;
    if (n < 1 || n > QVB8_MMA_MAX_CLASSES || L->first_pos[0] != 0 || L->first_pos[n] != Q) { *why = "bad row layout (1..3 classes that cover positions 0..Q)"; return false; }
    int64_t bits = 0;
    uint32_t widths = 0;
    for (int c = 0; c < n; ++c) {
        const int64_t rows = (int64_t)L->first_pos[c + 1] - L->first_pos[c], nbc = L->nbits[c];
        if (rows < 0 || (rows % unit_rows) != 0 || (L->first_pos[c] % unit_rows) != 0) { *why = "every run of one width must be whole tiles (whole gate/up units)"; return false; }
        if (nbc < 4 || nbc > 8) { *why = "widths 4..8 only"; return false; }
        bits += rows * P * nbc;
        widths |= (uint32_t)nbc << (8 * c);
    }
    for (int c = n; c < 3; ++c) widths |= (uint32_t)L->nbits[n - 1] << (8 * c);
    if ((bits >> 3) + 8 > ids_bytes) { *why = "the row layout does not fit the ids buffer"; return false; }
    s.Q = (int)Q; s.P = (int)P;
    s.first1 = n > 1 ? L->first_pos[1] : (int)Q;
    s.first2 = n > 2 ? L->first_pos[2] : (int)Q;
    s.widths = widths;
    return true;
}

template <int T1, int T2, int XP>
int launch_mlp(const MlpArgs& a, const MlpPlan& pl, hipStream_t s) {
    static bool attr[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return host::fail(QVB8_ERR_LAUNCH, "qvb8_mlp: no current device");
    if (!attr[dev]) {
        if (hipFuncSetAttribute((const void*)mlp_kernel<T1, T2, XP>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMlpLdsLimit) != hipSuccess)
            return host::fail(QVB8_ERR_LAUNCH, "qvb8_mlp: cannot raise the kernel's LDS limit");
        attr[dev] = true;
    }
    hipLaunchKernelGGL((mlp_kernel<T1, T2, XP>), dim3((unsigned)pl.blocks), dim3(kMlpThreads), pl.lds, s, a);
    return host::check_launch("qvb8_mlp");
}

template <int T1, int T2>
int launch_mlp_xp(const MlpArgs& a, const MlpPlan& pl, hipStream_t s) {
    return pl.XP == 1 ? launch_mlp<T1, T2, 1>(a, pl, s) : launch_mlp<T1, T2, 4>(a, pl, s);
}
template <int T1>
int launch_mlp_t2(const MlpArgs& a, const MlpPlan& pl, hipStream_t s) {
    return pl.T2 == 3 ? launch_mlp_xp<T1, 3>(a, pl, s) : launch_mlp_xp<T1, 4>(a, pl, s);
}

}  // namespace

extern "C" int64_t qvb8_mlp_workspace_bytes(int64_t inter) {
    if (inter <= 0) return 0;
    return (int64_t)kMlpStateWords * 4 + inter * 4 * (QVB8_MLP_MAX_ROWS * (QVB8_MLP_MAX_ROWS + 1) / 2);
}

extern "C" int qvb8_mlp(const void* X, int x_dtype, int64_t M, int64_t hidden, int64_t inter, int64_t out_features,
                        const uint8_t* gu_ids, int64_t gu_ids_bytes, const uint64_t* gu_rowinfo, const qvb8_mma_layout* gu_layout,
                        const uint8_t* dn_ids, int64_t dn_ids_bytes, const uint64_t* dn_rowinfo, const qvb8_mma_layout* dn_layout,
                        int act, int mid_dtype, void* Y, int y_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
    if (M < 1 || M > QVB8_MLP_MAX_ROWS) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp: 1..%d rows of X (M=%lld)", QVB8_MLP_MAX_ROWS, (long long)M);
    if (x_dtype != QVB8_F16 && x_dtype != QVB8_BF16) return host::fail(QVB8_ERR_ARG, "qvb8_mlp: X must be fp16 or bf16");
    if (mid_dtype < 0 || mid_dtype > 2 || y_dtype < 0 || y_dtype > 2) return host::fail(QVB8_ERR_ARG, "qvb8_mlp: bad dtype code");
    if ((act & 0xFF) != QVB8_MLP_SILU_GATED) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp: activation %d is not built (gated SiLU only)", act & 0xFF);
    if (hidden <= 0 || inter <= 0 || out_features <= 0 || hidden > 0x3fffffff || inter > 0x3fffffff || out_features > 0x3fffffff)
        return host::fail(QVB8_ERR_ARG, "qvb8_mlp: sizes out of range");
    if ((hidden % kStepCols) != 0 || (inter % kStepCols) != 0 || (out_features % kTileRows) != 0)
        return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp: needs hidden %% 128 == 0, inter %% 128 == 0 and out_features %% 16 == 0");
    if (!X || !Y || !gu_ids || !dn_ids || !gu_rowinfo || !dn_rowinfo || !gu_layout || !dn_layout || !workspace)
        return host::fail(QVB8_ERR_ARG, "qvb8_mlp: null pointer");
    if ((reinterpret_cast<uintptr_t>(X) & 15u) || (reinterpret_cast<uintptr_t>(gu_ids) & 15u) || (reinterpret_cast<uintptr_t>(dn_ids) & 15u)
        || (reinterpret_cast<uintptr_t>(workspace) & 15u))
        return host::fail(QVB8_ERR_ARG, "qvb8_mlp: X, ids and workspace must be 16-byte aligned");
    if (workspace_bytes < qvb8_mlp_workspace_bytes(inter))
        return host::fail(QVB8_ERR_WORKSPACE, "qvb8_mlp: needs %lld bytes of workspace (zeroed once before its first use)", (long long)qvb8_mlp_workspace_bytes(inter));
    MlpArgs a;
    const char* why = "";
    if (!side_ok(gu_layout, 2 * inter, hidden, gu_ids_bytes, 32, a.up, &why)) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp: gate+up: %s", why);
    if (!side_ok(dn_layout, out_features, inter, dn_ids_bytes, kTileRows, a.dn, &why)) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp: down: %s", why);
    a.X = (const uint16_t*)X;
    a.up.ids = gu_ids; a.up.fin = reinterpret_cast<const uint4*>(gu_rowinfo + ((2 * inter + 1) & ~(int64_t)1));
    a.dn.ids = dn_ids; a.dn.fin = reinterpret_cast<const uint4*>(dn_rowinfo + ((out_features + 1) & ~(int64_t)1));
    a.state = (uint32_t*)workspace; a.Y = Y;
    a.M = (int)M; a.x_bf16 = x_dtype == QVB8_BF16 ? 1 : 0; a.act_dt = mid_dtype; a.out_dt = y_dtype;
    a.flags = (act & QVB8_MLP_TEST_STALE_TAG) ? 1 : 0;
    const int wait_us = host::env_int("QVB8_MLP_WAIT_US", 20000);
    a.wait_ticks = (uint32_t)(wait_us < 1 ? 100 : (wait_us > 10000000 ? 1000000000u : (uint32_t)wait_us * 100u));

    MlpPlan pl;
    const int n_steps1 = (int)(hidden / kStepCols), n_steps2 = (int)(inter / kStepCols);
    pl.T1 = (n_steps1 > 32 && n_steps1 <= 40) ? 5 : 4;
    pl.T2 = pick_t2(n_steps2);
    const int64_t x_pieces = M * hidden / 8;
    if (x_pieces > 4 * kMlpThreads) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp: M * hidden beyond %d", 32 * kMlpThreads);
    pl.XP = x_pieces <= kMlpThreads ? 1 : 4;
    // one workgroup per CU, all resident at once: the hand-over inside the grid needs every workgroup running
    int cus = host::device_cus();
    const int forced = host::env_int("QVB8_MLP_WGS", 0);
    pl.blocks = forced > 0 && forced < cus ? forced : cus;
    const int64_t units = inter / kTileRows, tiles2 = out_features / kTileRows;
    const int64_t U1 = (units + pl.blocks - 1) / pl.blocks, TW2 = (tiles2 + pl.blocks - 1) / pl.blocks;
    if (U1 * 32 > kMlpThreads || TW2 * kTileRows > kMlpThreads)
        return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp: more than %d rows per workgroup", kMlpThreads);
    pl.lds = (size_t)(U1 * 32 + TW2 * 16) * 16 + (size_t)(kMlpTileWaves + kMlpWaves) * 16 * 4
             + (size_t)(U1 * 32 * kMlpTileWaves + TW2 * 16 * kMlpWaves) * (size_t)M * 4 + 16
             + (size_t)M * (size_t)hidden * 2 + 64 + (size_t)M * (size_t)inter * 2 + 64;
    if (pl.lds > kMlpLdsLimit) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp: %zu bytes of LDS per workgroup (limit %zu)", pl.lds, kMlpLdsLimit);
    hipStream_t s = (hipStream_t)stream;
    return pl.T1 == 5 ? launch_mlp_t2<5>(a, pl, s) : launch_mlp_t2<4>(a, pl, s);
}
