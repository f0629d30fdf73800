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
//             together with a 16-bit tag of this call (one 4-byte store: a reader sees the value and its tag or neither).
//             There is no flag to wait for first, no fence and no barrier across the grid: a reader asks for the values
//             themselves, again and again for the pieces whose tag is not yet this call's -- one trip through memory once
//             they are there.  The wait is BOUNDED: when a piece has not arrived after `wait_ticks` the workgroup gives up,
//             writes NaN as its results and raises the error word of the workspace -- it never spins without end;
//   phase 2   the sixteen waves share the workgroup's down rows by columns.  Each wave fetches the part of H that ITS
//             columns need, so it waits for the producers of those columns only (a sixteenth of the grid), not for the
//             slowest workgroup, and multiplies at once: the ids it asked for in phase 1 have landed meanwhile.  The ids of
//             a wave's second share of columns were asked for at the same time, straight into LDS (no registers needed).
//
// Loads return to a wave in the order it asked, so H reaches a wave only after the ids it asked for earlier: those were
// asked for microseconds before and are there by then.
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
constexpr int kMlpMaxM = QVB8_MLP_MAX_ROWS;
constexpr int kMlpMaxUnits = 32;            // units of 32 rows a workgroup may have (1024 threads hold their records)
constexpr int kMlpTileWaves = 8;            // phase 1: waves per 16-row tile (the gate tile and the up tile side by side)
// The workspace: 8 state words, the block's description (MlpDesc, written once by qvb8_mlp_init), then from byte 128 on H
// as tagged dwords, one region per row count (rows of M: M x I dwords at I * M (M - 1) / 2), so that a region is rewritten
// completely by every call that reads it.
//   state[1] error (sticky)   state[2 + M - 1] calls made with M rows
constexpr int kMlpStateWords = 32;           // dwords before H
constexpr int kMlpDescAt = 8;                // dword at which the description starts

// One weight of the block: rows stored in planes, in position order (position -> output row through fin), at most three
// runs of one width each, every run a whole number of tiles.
struct MlpSide {
    const uint8_t* ids;
    const uint4* fin;             // per position: tau_s bits, min_s bits, output row, 0
    int Q, P;
    int first1, first2;           // positions where the second and the third width start (Q when there is none)
    uint32_t widths;              // nb0 | nb1 << 8 | nb2 << 16
};

// What does not change from call to call lives in the workspace (device memory), so that a call's kernel arguments are the
// 14 dwords that arrive in registers: arguments beyond those are fetched from the kernel-argument buffer by the kernel's
// first instructions, and everything behind that fetch -- the activations' way into LDS, the first ids -- started
// 3 us late (measured with a 136-byte argument struct).
struct MlpDesc {
    const uint8_t* gu_ids; const uint4* gu_fin; const uint8_t* dn_ids; const uint4* dn_fin;
    int gu_first1, gu_first2; uint32_t gu_widths;
    int dn_first1, dn_first2; uint32_t dn_widths;
    int hidden, inter, out_features, pad;
};
static_assert(sizeof(MlpDesc) <= (kMlpStateWords - kMlpDescAt) * 4, "the description has its place before H");

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

// The two halves of mlp_multiply for a caller that decodes before its activations are there.
template <int T>
__device__ __forceinline__ void mlp_decode(uint32_t nb, const uint4 (&lo)[T], const uint4 (&hi)[T], v4u_t (&b)[T][4]) {
#pragma unroll
    for (int it = 0; it < T; ++it) {
        switch (nb) {
            case 7: decode_slice<7, false>(lo[it], hi[it], b[it]); break;
            case 6: decode_slice<6, false>(lo[it], hi[it], b[it]); break;
            case 5: decode_slice<5, false>(lo[it], hi[it], b[it]); break;
            case 4: decode_slice<4, false>(lo[it], hi[it], b[it]); break;
            default: decode_slice<8, false>(lo[it], hi[it], b[it]); break;
        }
    }
}
template <int T>
__device__ __forceinline__ void mlp_products(const v4u_t (&b)[T][4], const unsigned char* xs, uint32_t P, uint32_t x_zero, int M, int step0,
                                             int n_steps, bool sums, int r, int kg, v4f_t& sx, v4f_t& acc) {
    using F = Fmt<false>;
    const v4u_t ones = {F::one_bits, F::one_bits, F::one_bits, F::one_bits};
#pragma unroll
    for (int it = 0; it < T; ++it) {
        v4u_t xv[4];
        const bool on = r < M && (step0 + it) < n_steps;
        const uint32_t at = on ? 2u * ((uint32_t)r * P + (uint32_t)(step0 + it) * kStepCols + (uint32_t)kg * 32u) : x_zero;
#pragma unroll
        for (int j = 0; j < 4; ++j) xv[j] = *reinterpret_cast<const v4u_t*>(xs + at + 16 * j);
        if (sums) {
#pragma unroll
            for (int j = 0; j < 4; ++j) sx = F::mfma(xv[j], ones, sx);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = F::mfma(xv[j], b[it][j], acc);
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

// T1 / T2: steps of 128 columns a wave owns per panel in phase 1 / 2; XP: 16-byte pieces of X per thread; PRE: a wave decodes
// its first ids of phase 2 before it waits for H.
// `packed`: M | x_bf16 << 3 | act_dt << 4 | out_dt << 6 | flags << 8 (flags bit 0: H gets another call's tag).  nblk = the grid's size (an argument, because the
// grid size the hardware hands out is fetched from memory like a late argument).
template <int T1, int T2, int XP, bool PRE>
__global__ void __launch_bounds__(kMlpThreads) mlp_kernel(const uint16_t* __restrict__ X, const MlpDesc* __restrict__ desc, uint32_t* state,
                                                          void* Y, uint32_t packed, int hidden, int inter, int out_features, int nblk,
                                                          uint32_t wait_ticks) {
    using F = Fmt<false>;
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, kg = lane >> 4;
    MlpArgs a;
    a.X = X; a.state = state; a.Y = Y; a.wait_ticks = wait_ticks;
    a.M = (int)(packed & 7u); a.x_bf16 = (int)((packed >> 3) & 1u); a.act_dt = (int)((packed >> 4) & 3u); a.out_dt = (int)((packed >> 6) & 3u);
    a.flags = (int)(packed >> 8);
    a.up.Q = 2 * inter; a.up.P = hidden; a.dn.Q = out_features; a.dn.P = inter;
    a.up.ids = desc->gu_ids; a.up.fin = desc->gu_fin; a.up.first1 = desc->gu_first1; a.up.first2 = desc->gu_first2; a.up.widths = desc->gu_widths;
    a.dn.ids = desc->dn_ids; a.dn.fin = desc->dn_fin; a.dn.first1 = desc->dn_first1; a.dn.first2 = desc->dn_first2; a.dn.widths = desc->dn_widths;
    const int M = a.M;
    // workgroup b runs on XCD b % 8: the workgroups of one XCD take neighbouring units and tiles
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
    uint32_t* s_flag = reinterpret_cast<uint32_t*>(part2 + (size_t)TW2 * 16 * kMlpWaves * M);    // [4]: a wait ran out, the call count
    unsigned char* xs1 = reinterpret_cast<unsigned char*>(s_flag + 4);                   // [M][P1] fp16, 64 bytes of zeros behind
    const uint32_t x1_zero = (uint32_t)M * (uint32_t)P1 * 2u;
    unsigned char* xs2 = xs1 + x1_zero + 64;                                             // [M][I] fp16, 64 bytes of zeros behind
    const uint32_t x2_zero = (uint32_t)M * (uint32_t)I * 2u;

    // ---- first requests: X, the rows' end-of-tile records, the call count, the first ids ----
    // (a wave whose threads all lie past the last piece of X, or past the last row, asks for nothing and waits for nothing)
    const int x_pieces = (M * P1) >> 3;
    const bool wave_has_x = wave * 64 < x_pieces, wave_has_rows = wave * 64 < n_units * 32;
    v4u_t xg[XP];
    if (wave_has_x) {
        const v4u_t* xsrc = reinterpret_cast<const v4u_t*>(a.X);
#pragma unroll
        for (int i = 0; i < XP; ++i) xg[i] = xsrc[min(tid + i * kMlpThreads, x_pieces - 1)];
    }
    __builtin_amdgcn_sched_barrier(0);
    uint4 f1 = {0u, 0u, 0xffffffffu, 0u};
    if (wave_has_rows) {
        const bool h1 = tid < n_units * 32;
        const uint4 v1 = a.up.fin[h1 ? ((tid >> 5) * nblk + vb) * 32 + (tid & 31) : 0];
        if (h1) f1 = v1;
    }
    // calls made so far with this row count: written by the call before this one, so an input like any other; one
    // thread asks and shares the answer through LDS
    uint32_t calls_here = 0;
    if (tid == 0) calls_here = a.state[2 + (M - 1)];
    const int g = wave >> 3, wc = wave & 7;                       // phase 1: g = 0 the unit's gate tile, 1 its up tile
    uint4 lo[T1], hi[T1];
    uint32_t nb_cur;
    {
        const uint64_t tb = mlp_tile_byte(a.up, 2 * vb + g, nb_cur);
        mlp_issue<T1>(a.up.ids, tb, nb_cur, wc * T1, n_steps1, n_units > 0, lane, lo, hi);
    }
    if (wave_has_x) {
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const int idx = tid + i * kMlpThreads;
            v4u_t v = xg[i];
            if (a.x_bf16) {
#pragma unroll
                for (int k = 0; k < 4; ++k) v[k] = XIn<false, true>::pair(v[k]);
            }
            if (idx < x_pieces) reinterpret_cast<v4u_t*>(xs1)[idx] = v;
        }
    }
    if (tid < 16) {
        reinterpret_cast<uint32_t*>(xs1 + x1_zero)[tid] = 0u;
        reinterpret_cast<uint32_t*>(xs2 + x2_zero)[tid] = 0u;
    }
    if (tid < 4) s_flag[tid] = 0u;                                // [0] a wait for H ran out
    if (tid == 0) s_flag[1] = calls_here;
    if (tid < U1 * 32) s_fin1[tid] = f1;
    mlp_bare_barrier();

    // ---- hand-over, writing side: H of a unit, a thread per (output, token, column range); `first_item` / `stride` say which of
    //      the unit's 16 M (output, token) items the calling wave takes ----
    const uint32_t calls = s_flag[1];
    const uint32_t tag = calls % 65535u + 1u;                     // never 0: a workspace starts as zeros
    const uint32_t tag_w = ((a.flags & 1) ? (tag % 65535u + 1u) : tag) << 16;
    uint32_t* Hreg = a.state + kMlpStateWords + (size_t)I * (size_t)(M * (M - 1) / 2);
    auto publish = [&](int lu, int first_item, int stride) __attribute__((always_inline)) {
        const int valid1 = ranges1 < kMlpTileWaves ? ranges1 : kMlpTileWaves;
        const int items = kTileRows * M;
        for (int first = first_item; first < items; first += stride) {
            const int i = first + (lane >> 4), w = lane & 15;
            const bool item = i < items;
            const int rr = item ? i / M : 0, t = item ? i - rr * M : 0;
            const int grow = lu * 32 + rr, urow = grow + 16;
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
    };
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
    // Nothing of phase 1 is in flight any more.  Said to the compiler in a form it reads (a wait instruction of its own
    // kind, not inline assembly): otherwise it assumes loads of the loop above may still be pending and answers the first
    // use of a register behind the requests below with a wait for ALL of them.
    __builtin_amdgcn_s_waitcnt(0x0F70);                           // vmcnt(0)
    // the down rows' end-of-tile records (their pointer is one of the kernel arguments that arrive late: asked for at the
    // kernel's start they held up the activations' way into LDS by two trips)
    uint4 f2 = {0u, 0u, 0xffffffffu, 0u};
    {
        const bool h2 = tid < n_tiles2 * kTileRows;
        const uint4 v2 = a.dn.fin[h2 ? ((tid >> 4) * nblk + vb) * kTileRows + (tid & 15) : 0];
        if (h2) f2 = v2;
    }

    // ---- phase 2, down: the sixteen waves share the workgroup's rows by columns.  A wave's items: for each of its column
    //      ranges (one per panel) the workgroup's tiles, in that order ----
    auto step0_of = [&](int panel) { return (panel * kMlpWaves + ((wave + 8 * panel) & 15)) * T2; };   // odd panels start at wave 8
    int n_panels_mine = 0;
    for (int pn = 0; pn < panels2; ++pn) n_panels_mine += step0_of(pn) < n_steps2 ? 1 : 0;
    const int n_items = n_tiles2 * n_panels_mine;
    uint4 lo2[T2], hi2[T2];
    uint32_t nb2 = 4u;
    auto ask_item = [&](int k) __attribute__((always_inline)) {            // the ids of item k into lo2 / hi2
        const int panel = k / n_tiles2, lt = k - panel * n_tiles2;
        const uint64_t tb = mlp_tile_byte(a.dn, lt * nblk + vb, nb2);
        mlp_issue<T2>(a.dn.ids, tb, nb2, step0_of(panel), n_steps2, true, lane, lo2, hi2);
    };
    const uint64_t* H64 = reinterpret_cast<const uint64_t*>(Hreg);
    uint32_t* xw = reinterpret_cast<uint32_t*>(xs2);
    const uint64_t t_wait0 = wall_clock64();
    bool failed = false;
    // H of the columns of steps [s0, s0 + T2) into LDS, row by row (T2 * 128 tagged dwords = T2 pieces of 8 bytes per lane):
    // the wave asks again for the pieces whose tag is not yet this call's, for at most wait_ticks
    auto fetch_h = [&](int s0) __attribute__((always_inline)) {
        for (int m = 0; m < M && !failed; ++m) {
            const size_t piece0 = ((size_t)m * I + (size_t)s0 * kStepCols) / 2 + lane;
            uint64_t v[T2];
            uint32_t need = 0;
#pragma unroll
            for (int it = 0; it < T2; ++it)
                if (s0 + it < n_steps2) need |= 1u << it;
            for (;;) {
#pragma unroll
                for (int it = 0; it < T2; ++it)
                    if ((need >> it) & 1u) v[it] = __hip_atomic_load(H64 + piece0 + (size_t)it * (kStepCols / 2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int it = 0; it < T2; ++it) {
                    if ((need >> it) & 1u) {
                        const uint32_t d0 = (uint32_t)v[it], d1 = (uint32_t)(v[it] >> 32);
                        if (__builtin_amdgcn_ballot_w64((d0 >> 16) != tag || (d1 >> 16) != tag) == 0) {
                            need &= ~(1u << it);
                            xw[piece0 + (size_t)it * (kStepCols / 2)] = (d0 & 0xFFFFu) | (d1 << 16);
                        }
                    }
                }
                if (need == 0u) break;
                if (wall_clock64() - t_wait0 > (uint64_t)a.wait_ticks) { failed = true; break; }
                __builtin_amdgcn_s_sleep(1);
            }
        }
    };
    // a tile's sums of this wave's columns into its LDS slots (and, once per panel, the sums of H over those columns)
    auto put_away = [&](int lt, bool first_panel, const v4f_t& sx, const v4f_t& acc) __attribute__((always_inline)) {
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
            const float vv = __builtin_fmaf(-F::bias, sx[e], acc[e]);
            if (t < M) {
                float* dst = part2 + ((size_t)lrow * kMlpWaves + wave) * M + t;
                *dst = first_panel ? vv : *dst + vv;
            }
        }
    };
    v4f_t sx_panel = {0.f, 0.f, 0.f, 0.f};
    // Item k with its ids decoded AHEAD of H: while H is on its way the wave turns the ids it already has into operands
    // (vector work that does not need H) and asks for its next ids into the registers that this frees; when H is there only
    // the products are left.
    auto run_item_ahead = [&](int k) __attribute__((always_inline)) {
        const int panel = k / n_tiles2, lt = k - panel * n_tiles2, s0 = step0_of(panel);
        v4u_t b2[T2][4];
        mlp_decode<T2>(nb2, lo2, hi2, b2);
        if (k + 1 < n_items) ask_item(k + 1);
        if (lt == 0) { fetch_h(s0); sx_panel = v4f_t{0.f, 0.f, 0.f, 0.f}; }
        v4f_t acc = {0.f, 0.f, 0.f, 0.f};
        mlp_products<T2>(b2, xs2, (uint32_t)I, x2_zero, M, s0, n_steps2, lt == 0, r, kg, sx_panel, acc);
        put_away(lt, panel == 0, sx_panel, acc);
    };
    auto run_item = [&](int k) __attribute__((always_inline)) {
        const int panel = k / n_tiles2, lt = k - panel * n_tiles2, s0 = step0_of(panel);
        if (lt == 0) { fetch_h(s0); sx_panel = v4f_t{0.f, 0.f, 0.f, 0.f}; }
        v4f_t acc = {0.f, 0.f, 0.f, 0.f};
        mlp_multiply<T2>(nb2, lo2, hi2, xs2, (uint32_t)I, x2_zero, M, s0, n_steps2, lt == 0, r, kg, sx_panel, acc);
        if (k + 1 < n_items) ask_item(k + 1);
        put_away(lt, panel == 0, sx_panel, acc);
    };
    // The first ids are asked for BEFORE the hand-over (they do not depend on H).
    if (n_items > 0) ask_item(0);
    int k_done = 0;
    mlp_bare_barrier();
    if (tid < TW2 * kTileRows) s_fin2[tid] = f2;                  // read behind the last barrier of the kernel
    // H of this workgroup's units: the waves share the units' (output, token) items
    for (int u = 0; u < n_units; ++u) publish(u, ((wave + 4 * u) & 15) * 4, kMlpWaves * 4);
    if (PRE && k_done < n_items) { run_item_ahead(k_done); ++k_done; }
    for (int k = k_done; k < n_items; ++k) run_item(k);
    if (failed && lane == 0) s_flag[0] = 1u;
    __syncthreads();
    const bool bad = s_flag[0] != 0u;

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
        // The workgroup of the first down tile closes the call: its waves have seen ALL of H, so every workgroup of the grid
        // has read the call count by now, and the next call gets the next tag.  (A plain store: the kernel's end publishes it.)
        if (vb == 0) a.state[2 + (M - 1)] = calls + 1u;
    }
}

}  // namespace qvb8

using namespace qvb8;

namespace {

constexpr size_t kMlpLdsLimit = 160 * 1024;
constexpr int64_t kPlanMagic = 0x51564d4c50ll;                 // marks a qvb8_mlp_plan that qvb8_mlp_init filled

struct MlpLaunch { int T1, T2, XP, blocks; size_t lds; };

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

bool side_ok(const qvb8_mma_layout* L, int64_t Q, int64_t P, int64_t ids_bytes, int unit_rows, int& first1, int& first2, uint32_t& widths_out, const char** why) {
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
    first1 = n > 1 ? L->first_pos[1] : (int)Q;
    first2 = n > 2 ? L->first_pos[2] : (int)Q;
    widths_out = widths;
    return true;
}

// zeroes the workspace (state words and every tag of H) and writes the block's description into it
__global__ void __launch_bounds__(256) mlp_init_kernel(uint32_t* ws, int64_t words, MlpDesc d) {
    const int64_t n_desc = (int64_t)(sizeof(MlpDesc) + 3) / 4;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t k = i - kMlpDescAt;
        ws[i] = (k >= 0 && k < n_desc) ? reinterpret_cast<const uint32_t*>(&d)[k] : 0u;
    }
}

template <int T1, int T2, int XP, bool PRE>
int launch_mlp(const void* X, void* ws, void* Y, uint32_t packed, const qvb8_mlp_plan* p, uint32_t wait_ticks, const MlpLaunch& pl, hipStream_t s) {
    static bool attr[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return host::fail(QVB8_ERR_LAUNCH, "qvb8_mlp: no current device");
    if (!attr[dev]) {
        if (hipFuncSetAttribute((const void*)mlp_kernel<T1, T2, XP, PRE>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMlpLdsLimit) != hipSuccess)
            return host::fail(QVB8_ERR_LAUNCH, "qvb8_mlp: cannot raise the kernel's LDS limit");
        attr[dev] = true;
    }
    uint32_t* state = reinterpret_cast<uint32_t*>(ws);
    hipLaunchKernelGGL((mlp_kernel<T1, T2, XP, PRE>), dim3((unsigned)pl.blocks), dim3(kMlpThreads), pl.lds, s, (const uint16_t*)X,
                       reinterpret_cast<const MlpDesc*>(state + kMlpDescAt), state, Y, packed, (int)p->hidden, (int)p->inter,
                       (int)p->out_features, pl.blocks, wait_ticks);
    return host::check_launch("qvb8_mlp");
}

template <int T1, int T2>
int launch_mlp_xp(const void* X, void* ws, void* Y, uint32_t packed, const qvb8_mlp_plan* p, uint32_t wait_ticks, const MlpLaunch& pl, hipStream_t s) {
    // decoding ahead of H is built for three steps per wave (more decoded operands do not fit the registers)
    if (T2 == 3 && host::env_int("QVB8_MLP_PRE", 1) != 0)
        return pl.XP == 1 ? launch_mlp<T1, T2, 1, T2 == 3>(X, ws, Y, packed, p, wait_ticks, pl, s) : launch_mlp<T1, T2, 4, T2 == 3>(X, ws, Y, packed, p, wait_ticks, pl, s);
    return pl.XP == 1 ? launch_mlp<T1, T2, 1, false>(X, ws, Y, packed, p, wait_ticks, pl, s) : launch_mlp<T1, T2, 4, false>(X, ws, Y, packed, p, wait_ticks, pl, s);
}
template <int T1>
int launch_mlp_t2(const void* X, void* ws, void* Y, uint32_t packed, const qvb8_mlp_plan* p, uint32_t wait_ticks, const MlpLaunch& pl, hipStream_t s) {
    return pl.T2 == 3 ? launch_mlp_xp<T1, 3>(X, ws, Y, packed, p, wait_ticks, pl, s) : launch_mlp_xp<T1, 4>(X, ws, Y, packed, p, wait_ticks, pl, s);
}

}  // namespace

extern "C" int64_t qvb8_mlp_workspace_bytes(int64_t inter) {
    if (inter <= 0) return 0;
    return (int64_t)kMlpStateWords * 4 + inter * 4 * (QVB8_MLP_MAX_ROWS * (QVB8_MLP_MAX_ROWS + 1) / 2);
}

extern "C" int qvb8_mlp_init(int64_t hidden, int64_t inter, int64_t out_features,
                             const uint8_t* gu_ids, int64_t gu_ids_bytes, const uint64_t* gu_rowinfo, const qvb8_mma_layout* gu_layout,
                             const uint8_t* dn_ids, int64_t dn_ids_bytes, const uint64_t* dn_rowinfo, const qvb8_mma_layout* dn_layout,
                             void* workspace, int64_t workspace_bytes, qvb8_mlp_plan* plan, void* stream) {
    if (!plan) return host::fail(QVB8_ERR_ARG, "qvb8_mlp_init: null plan");
    plan->magic = 0;
    if (hidden <= 0 || inter <= 0 || out_features <= 0 || hidden > 0x3fffffff || inter > 0x3fffffff || out_features > 0x3fffffff)
        return host::fail(QVB8_ERR_ARG, "qvb8_mlp_init: sizes out of range");
    if ((hidden % kStepCols) != 0 || (inter % kStepCols) != 0 || (out_features % kTileRows) != 0)
        return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp_init: needs hidden %% 128 == 0, inter %% 128 == 0 and out_features %% 16 == 0");
    if (!gu_ids || !dn_ids || !gu_rowinfo || !dn_rowinfo || !gu_layout || !dn_layout || !workspace)
        return host::fail(QVB8_ERR_ARG, "qvb8_mlp_init: null pointer");
    if ((reinterpret_cast<uintptr_t>(gu_ids) & 15u) || (reinterpret_cast<uintptr_t>(dn_ids) & 15u) || (reinterpret_cast<uintptr_t>(workspace) & 15u))
        return host::fail(QVB8_ERR_ARG, "qvb8_mlp_init: ids and workspace must be 16-byte aligned");
    if (workspace_bytes < qvb8_mlp_workspace_bytes(inter))
        return host::fail(QVB8_ERR_WORKSPACE, "qvb8_mlp_init: needs %lld bytes of workspace", (long long)qvb8_mlp_workspace_bytes(inter));
    MlpDesc d;
    const char* why = "";
    if (!side_ok(gu_layout, 2 * inter, hidden, gu_ids_bytes, 32, d.gu_first1, d.gu_first2, d.gu_widths, &why)) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp_init: gate+up: %s", why);
    if (!side_ok(dn_layout, out_features, inter, dn_ids_bytes, kTileRows, d.dn_first1, d.dn_first2, d.dn_widths, &why)) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp_init: down: %s", why);
    d.gu_ids = gu_ids; d.gu_fin = reinterpret_cast<const uint4*>(gu_rowinfo + ((2 * inter + 1) & ~(int64_t)1));
    d.dn_ids = dn_ids; d.dn_fin = reinterpret_cast<const uint4*>(dn_rowinfo + ((out_features + 1) & ~(int64_t)1));
    d.hidden = (int)hidden; d.inter = (int)inter; d.out_features = (int)out_features; d.pad = 0;
    const int64_t words = qvb8_mlp_workspace_bytes(inter) / 4;
    hipLaunchKernelGGL(mlp_init_kernel, dim3((unsigned)((words + 255) / 256 < 1024 ? (words + 255) / 256 : 1024)), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<uint32_t*>(workspace), words, d);
    if (int rc = host::check_launch("qvb8_mlp_init")) return rc;
    plan->hidden = hidden; plan->inter = inter; plan->out_features = out_features;
    plan->magic = kPlanMagic ^ (int64_t)reinterpret_cast<uintptr_t>(workspace);
    return QVB8_OK;
}

extern "C" int qvb8_mlp(const qvb8_mlp_plan* plan, const void* X, int x_dtype, int64_t M, int act, int mid_dtype,
                        void* Y, int y_dtype, void* workspace, void* stream) {
    if (!plan || !workspace || plan->magic != (kPlanMagic ^ (int64_t)reinterpret_cast<uintptr_t>(workspace)))
        return host::fail(QVB8_ERR_ARG, "qvb8_mlp: the plan is not the one qvb8_mlp_init made for this workspace");
    if (M < 1 || M > QVB8_MLP_MAX_ROWS) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp: 1..%d rows of X (M=%lld)", QVB8_MLP_MAX_ROWS, (long long)M);
    if (x_dtype != QVB8_F16 && x_dtype != QVB8_BF16) return host::fail(QVB8_ERR_ARG, "qvb8_mlp: X must be fp16 or bf16");
    if (mid_dtype < 0 || mid_dtype > 2 || y_dtype < 0 || y_dtype > 2) return host::fail(QVB8_ERR_ARG, "qvb8_mlp: bad dtype code");
    if ((act & 0xFF) != QVB8_MLP_SILU_GATED) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp: activation %d is not built (gated SiLU only)", act & 0xFF);
    if (!X || !Y) return host::fail(QVB8_ERR_ARG, "qvb8_mlp: null pointer");
    if (reinterpret_cast<uintptr_t>(X) & 15u) return host::fail(QVB8_ERR_ARG, "qvb8_mlp: X must be 16-byte aligned");
    const int64_t hidden = plan->hidden, inter = plan->inter, out_features = plan->out_features;
    const int wait_us = host::env_int("QVB8_MLP_WAIT_US", 20000);
    const uint32_t wait_ticks = (uint32_t)(wait_us < 1 ? 100 : (wait_us > 10000000 ? 1000000000u : (uint32_t)wait_us * 100u));
    const uint32_t packed = (uint32_t)M | ((x_dtype == QVB8_BF16 ? 1u : 0u) << 3) | ((uint32_t)mid_dtype << 4) | ((uint32_t)y_dtype << 6)
                            | (((act & QVB8_MLP_TEST_STALE_TAG) ? 1u : 0u) << 8);

    MlpLaunch pl;
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
    if (U1 > kMlpMaxUnits || U1 * 32 > kMlpThreads || TW2 * kTileRows > kMlpThreads)
        return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp: more than %d rows per workgroup", kMlpThreads);
    pl.lds = (size_t)(U1 * 32 + TW2 * 16) * 16 + (size_t)(kMlpTileWaves + kMlpWaves) * 16 * 4
             + (size_t)(U1 * 32 * kMlpTileWaves + TW2 * 16 * kMlpWaves) * (size_t)M * 4 + 16
             + (size_t)M * (size_t)hidden * 2 + 64 + (size_t)M * (size_t)inter * 2 + 64;
    if (pl.lds > kMlpLdsLimit) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mlp: %zu bytes of LDS per workgroup (limit %zu)", pl.lds, kMlpLdsLimit);
    hipStream_t s = (hipStream_t)stream;
    return pl.T1 == 5 ? launch_mlp_t2<5>(X, workspace, Y, packed, plan, wait_ticks, pl, s) : launch_mlp_t2<4>(X, workspace, Y, packed, plan, wait_ticks, pl, s);
}
