// Fused QVB8 decode + small-M GEMM on the matrix cores (gfx950): M = 1..48 rows of X against the packed (Q, P) weight.
//
//   Y[t][q] = tau_s[q] * sum_c X[t][c] * id[q][c]  +  min_s[q] * sum_c X[t][c]
//
// The id sum is a matrix product with the ids as one MFMA operand.  A tile is 16 weight rows; per step a wave
// takes 128 columns of the tile: lane l owns the 32 consecutive ids of row l % 16 at columns 32 * (l / 16), which
// are NB dwords of that row, fetched as two 16-byte loads straight in the MFMA operand layout (16 row streams
// per wave; measured as fast as fully contiguous loads).  Each pair of ids is turned into two 16-bit floats
// `bias + id` (exact: 1024 + id in fp16, 128 + id in bf16) with three integer operations, four v_mfma 16x16x32
// consume the lane's 32 ids against the activations held in registers, and the bias is removed with one more
// MFMA per step against a matrix of ones (computed once per wave, not per tile).  Activations are used in
// their own 16-bit format: no conversion anywhere.
//
// A workgroup has W waves that share a tile and own T*128 columns each (repeated over `panels` when the row is
// longer), times G tile groups.  Per-row metadata of the workgroup's rows is staged in LDS once; partial sums
// meet in LDS and are combined in a fixed order (bit-reproducible, no atomics).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/qvb8_amd.h"
#include "qvb8_device.h"
#include "qvb8_host.h"
#include "qvb8_mma_device.h"

namespace qvb8 {

// Row records of the tile kernel, in TILE ORDER (position -> row through `perm`), two arrays back to back:
//   loc[pos]  u64   bits 0..47 absolute bit offset of the row's first id | bits 48..55 width | bits 56..57 kind
//             kind 0: the metadata points outside the buffer (the row yields NaN), 1: dword-aligned row of width
//             4..8 (sliced path), 2: anything else that is in bounds (read element by element), 3: no such row
//             bit 58: the row is stored in planes (then bits 0..47 = bit offset of its 16-row tile, bits 59..62 = its
//             number inside the tile; kind 1)
//   fin[pos]  4 x u32   tau_s bits, min_s bits, output row q (or 0xffffffff), 0 -- what the end of a tile needs
// loc has Q rounded up to even entries, so that fin is 16-byte aligned.
constexpr uint64_t kRowOffMask = (1ull << 48) - 1;
__host__ __device__ inline size_t rowinfo_loc_words(int64_t Q) { return (size_t)((Q + 1) & ~(int64_t)1); }

// a result into Y in the caller's format (wave-uniform choice)
__device__ __forceinline__ void store_y(float* Y, int out_dt, int64_t i, float v) {
    if (out_dt == 0) Y[i] = v;
    else if (out_dt == 1) store_from_f32<1>(Y, i, v);
    else store_from_f32<2>(Y, i, v);
}

struct TileArgs {
    const uint16_t* X;            // (M, P) fp16 or bf16 bits
    const uint8_t* ids;
    const uint64_t* loc;          // row records, see above
    const uint4* fin;
    float* Y;                     // (M, Q) fp32
    int64_t ids_bytes;
    int M, Q, P;
    int out_dt;                   // what Y holds: 0 fp32, 1 fp16, 2 bf16
    int n_steps;                  // P / 128
    int W, G, panels;             // waves per tile, tile groups per workgroup, column panels
    int TW;                       // tiles per workgroup (multiple of G)
    // Rows STORED in tile order from bit 0 of `ids`, one run per width (at most three): positions [0, first1) have width
    // nb[0], [first1, first2) nb[1], [first2, Q) nb[2].  n_classes == 0: addresses come from `loc`.
    int n_classes, first1, first2;
    int nb[3];
    int planes;                   // rows of whole 16-row tiles of one sliceable width are stored in planes (see qvb8_device.h)
};

__global__ void __launch_bounds__(256) rowinfo_kernel(const uint8_t* __restrict__ nbits, const int64_t* __restrict__ bit_off,
                                                      const float* __restrict__ tau_s, const float* __restrict__ min_s,
                                                      const int32_t* __restrict__ perm, int Q, int P, int64_t ids_bytes,
                                                      uint64_t* __restrict__ loc, uint4* __restrict__ fin) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= Q) return;
    const int q = perm ? perm[i] : i;
    uint64_t rec = 0;
    uint4 f = {0u, 0u, 0xffffffffu, 0u};
    if (q >= 0 && q < Q) {
        f = uint4{__float_as_uint(tau_s[q]), __float_as_uint(min_s[q]), (uint32_t)q, 0u};
        const int nb = nbits[q];
        const int64_t bit0 = bit_off[q];
        const bool ok = row_in_bounds(bit0, nb, P, ids_bytes);
        if (ok && off_is_plane(bit0)) {
            rec = (uint64_t)(bit0 & kOffBitsMask) | ((uint64_t)nb << 48) | (1ull << 56) | (1ull << 58) | ((uint64_t)off_plane_row(bit0) << 59);
        } else {
            const uint64_t kind = !ok ? 0 : ((bit0 & 31) == 0 && nb >= 4 && nb <= 8) ? 1 : 2;
            rec = (ok ? (uint64_t)bit0 : 0) | ((uint64_t)nb << 48) | (kind << 56);
        }
    }
    loc[i] = rec;
    fin[i] = f;
}

// bf16, width 8: the operand above carries id & 127 (plus the bias); bit 7 goes into a second operand as
// 2^-63 per set bit (a lone exponent bit), multiplied separately and scaled back in the epilogue.
constexpr uint32_t kTopBitBits = 0x20002000u;               // bf16 2^-63 in both halves
constexpr float kTopBitScale = 128.0f * 9223372036854775808.0f;   // 128 * 2^63

__device__ __forceinline__ void decode_slice8_top(const uint4& lo, const uint4& hi, v4u_t (&bt)[4]) {
    uint32_t e[16];
    slice_pairs<8>(lo, hi, e);
#pragma unroll
    for (int p = 0; p < 16; ++p) bt[p / 4][p % 4] = (e[p] << 6) & kTopBitBits;
}

// NT = token tiles of 16 (M <= 16 * NT); T = steps of 128 columns a wave owns per panel; BF = bf16 operands.
//
// Wave (g, wc) of a workgroup owns column range wc (T steps; further ranges in later panels) of the tiles of group
// g.  Its activations for that range stay in registers for the whole panel.  Per tile it requests its T slices in
// one burst (2T loads), turns them into MFMA operands as they arrive, and puts its partial sums into its own LDS
// slots.  After one barrier the whole workgroup combines the column ranges of each row in a fixed order.
// The kernel's arguments are 56 bytes of scalars (measured: every further 64 bytes of kernel arguments cost about a
// microsecond per launch): fin follows loc, n_steps follows P, the small counts share one word.
// Waves a workgroup of this variant may have: twelve (three per SIMD) where the registers allow it -- long rows then take
// fewer panels (12288 columns: two instead of three) --, else eight.
constexpr uint32_t kTileTransitRow = 272;                     // bytes between rows of a wave's transit region (256 + 16: see XT)
constexpr uint32_t kTileTransitBytes = 16 * kTileTransitRow;
template <int NT, int T, bool BF, bool PL> constexpr int tile_max_waves() { return (NT == 1 && T == 4 && PL && !BF) ? 12 : 8; }

template <int NT, int T, bool BF, bool XC, int XP = 0, bool PL = false>
__global__ void __launch_bounds__((64 * tile_max_waves<NT, T, BF, PL>())) tile_kernel(const uint16_t* __restrict__ X, const uint8_t* __restrict__ ids,
                                                   const uint64_t* __restrict__ loc, float* __restrict__ Y, int64_t ids_bytes,
                                                   int Q, int P, uint32_t counts, int TW, int first1, int first2, uint32_t widths) {
    static_assert(!(BF && XC), "narrowing on the way in exists for fp16 operands only");
    constexpr bool XL = XP > 0;                              // X goes through LDS, XP 16-byte pieces per thread
    TileArgs a;
    a.X = X; a.ids = ids; a.loc = loc; a.fin = reinterpret_cast<const uint4*>(loc + rowinfo_loc_words(Q)); a.Y = Y;
    a.ids_bytes = ids_bytes; a.Q = Q; a.P = P; a.n_steps = P / kStepCols; a.TW = TW;
    a.M = (int)(counts & 63u); a.out_dt = (int)((counts >> 6) & 3u); a.W = (int)((counts >> 8) & 15u); a.G = (int)((counts >> 12) & 15u); a.panels = (int)(counts >> 16);
    a.first1 = first1; a.first2 = first2; a.n_classes = (int)((widths >> 24) & 0x7Fu); a.planes = PL ? 1 : 0;
    a.nb[0] = (int)(widths & 255u); a.nb[1] = (int)((widths >> 8) & 255u); a.nb[2] = (int)((widths >> 16) & 255u);
    using F = Fmt<BF>;
    using XI = XIn<BF, XC>;
    constexpr int TM = 16 * NT;
    extern __shared__ __align__(16) unsigned char smem[];
    const int rows_cap = a.TW * kTileRows;
    const int ranges = a.W;                                   // partial-sum slots per row: one per wave of the tile; panels add up in place
    const int wave_rows = (a.TW / a.G) * kTileRows;           // rows a wave ever touches
    const int n_waves = a.W * a.G;
    // LDS: per-wave copies of the row records, what the end needs per row, column-range sums of x, partial sums
    uint4* s_fin = reinterpret_cast<uint4*>(smem);                                       // [rows_cap]
    uint64_t* s_loc = reinterpret_cast<uint64_t*>(s_fin + rows_cap);                     // [n_waves][wave_rows]
    float* sxs = reinterpret_cast<float*>(s_loc + (size_t)n_waves * wave_rows);          // [ranges][TM]
    // [rows_cap][ranges][M].  (The lanes of a store -- 16 rows x 4 tokens -- fall into few banks this way; a layout without those
    // conflicts, [ranges][M][rows_cap + 4], was measured and was 5 % slower at 8..16 rows of X: the stores are not waited for,
    // and its addresses cost more instructions.)
    float* part = sxs + (size_t)ranges * TM;
    const int MS = a.M;                                       // a row's partial sums hold M tokens, not the TM the tile could take

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = wave / a.W, wc = wave - g * a.W;
    const int r = lane & 15, kg = lane >> 4;
    // XL: the whole of X (at most XP 16-byte pieces per thread) goes through LDS once: every thread requests its
    // pieces before anything else, the first tile's ids follow at once, and the workgroup shares X after one barrier --
    // so the trip of the activations and the first trip of the ids overlap, and later panels need no trip for theirs.
    // [M][P] as in memory.  (Rows a multiple of 128 bytes apart put the lanes of an operand read, one row each, into the same
    // banks; moving the rows 16..80 bytes further apart was measured and changed nothing: those reads are not what the
    // launch waits for.)
    unsigned char* xs = reinterpret_cast<unsigned char*>(part + (size_t)rows_cap * ranges * MS);
    static_assert(!XL || NT == 1, "X as a whole in LDS exists for one token tile");
    // JIT: with one token tile and X in LDS a step's operands are read from LDS when the step is multiplied instead of being
    // held in 16 T registers for the whole panel (lanes without a row of X, and steps past the end, read 64 bytes of zeros)
    constexpr bool JIT = XL && NT == 1;
    // XT (one token tile, X not in LDS as a whole): a wave fetches the activations of its columns in memory order -- a load
    // instruction covers four rows of X, 256 contiguous bytes of each -- and turns them into operand order through a
    // 16 x 256-byte region of LDS of its own, step by step.  (Fetched in operand order, every lane reads 64 bytes of a row of
    // its own: 64 cache lines per instruction, and with 9..16 rows of X the CU's L1 spent more cycles on those accesses than
    // the launch needs for everything else.)
    constexpr bool XT = !XL && NT == 1;
    const int x_pieces = (a.M * a.P) >> 3;
    v4u_t xg[XL ? XP : 1];
    if constexpr (XL) {
        const v4u_t* xsrc = reinterpret_cast<const v4u_t*>(a.X);
#pragma unroll
        for (int i = 0; i < XP; ++i) xg[i] = xsrc[min(tid + i * (int)blockDim.x, x_pieces - 1)];
        __builtin_amdgcn_sched_barrier(0);                     // these requests stay where they are: ahead of everything
    }
    // The workgroup's local tile lt is global tile lt * gridDim.x + vb (vb: the workgroup's number, see below): at any moment the
    // workgroups of the grid read neighbouring tiles, so the whole chip walks through memory together (spread over all channels).
    const int total_tiles = (a.Q + kTileRows - 1) / kTileRows;
    // Workgroup b runs on XCD b % 8 (workgroups are dealt to the eight XCDs in turn): the workgroups of one XCD take
    // neighbouring tiles, so each XCD's L2 and its path to memory see one contiguous eighth of the window the chip is
    // reading (measured: 0.4 % of the 9B decode step, o and q+k+v 0.05-0.1 us each; nothing on the long launches).
    const int nblk = (int)gridDim.x;
    const int vb = (nblk & 7) == 0 ? ((int)blockIdx.x & 7) * (nblk >> 3) + ((int)blockIdx.x >> 3) : (int)blockIdx.x;
    const int tiles_here = vb < total_tiles ? min(a.TW, (total_tiles - 1 - vb) / nblk + 1) : 0;
    auto local_to_pos = [&](int lrow) { return ((lrow >> 4) * nblk + vb) * kTileRows + (lrow & 15); };
    const int n_tiles = tiles_here > g ? (tiles_here - g + a.G - 1) / a.G : 0;    // tiles of this wave's group

    // ---- the records of this wave's rows into its own LDS copy (a wave's LDS accesses stay in order, so the copy
    //      needs no barrier); a position past Q has no row ----
    uint64_t* my_loc = s_loc + (size_t)wave * wave_rows;
    for (int i = lane; i < n_tiles * kTileRows; i += kWave) {
        const int pos = local_to_pos((g + a.G * (i >> 4)) * kTileRows + (i & 15));
        uint64_t rec = 3ull << 56;
        if (pos < a.Q) {
            if (a.n_classes > 0) {
                // no request: where the row is follows from the layout in the kernel arguments
                const uint64_t P64 = (uint64_t)a.P;
                const uint64_t base1 = (uint64_t)a.first1 * P64 * (uint64_t)a.nb[0];
                const uint64_t base2 = base1 + (uint64_t)(a.first2 - a.first1) * P64 * (uint64_t)a.nb[1];
                const int c = (pos >= a.first1 ? 1 : 0) + (pos >= a.first2 ? 1 : 0);
                const uint64_t nbc = (uint64_t)(c == 0 ? a.nb[0] : c == 1 ? a.nb[1] : a.nb[2]);
                const uint64_t bit0 = (c == 0 ? 0 : c == 1 ? base1 : base2)
                                      + (uint64_t)(pos - (c == 0 ? 0 : c == 1 ? a.first1 : a.first2)) * P64 * nbc;
                rec = bit0 | (nbc << 48) | ((uint64_t)((nbc >= 4 && nbc <= 8) ? 1 : 2) << 56);
                if constexpr (PL) {
                    // a tile that lies inside one run of a sliceable width is stored in planes: the record then names the tile
                    const int first_c = c == 0 ? 0 : c == 1 ? a.first1 : a.first2;
                    const int end_c = c == 0 ? a.first1 : c == 1 ? a.first2 : a.Q;
                    const int t0 = pos & ~15;
                    if (nbc >= 4 && nbc <= 8 && t0 >= first_c && t0 + 16 <= end_c)
                        rec = (bit0 - (uint64_t)(pos & 15) * P64 * nbc) | (nbc << 48) | (1ull << 56) | (1ull << 58) | ((uint64_t)(pos & 15) << 59);
                }
            } else {
                rec = a.loc[pos];
                // a record that says "stored in planes" reaching the kernel variant for rows back to back (the caller left
                // QVB8_MMA_PLANES out): its offset names the tile, not the row -- the row comes out as NaN, not as another row's values
                if constexpr (!PL) { if ((rec >> 58) & 1ull) rec &= ~(3ull << 56); }
            }
        }
        my_loc[i] = rec;
    }
    // ---- what the end needs for row `tid`: requested now, parked in registers, put in LDS before the barrier ----
    uint4 e_fin = {0u, 0u, 0xffffffffu, 0u};
    if constexpr (XL) {
        // no request under a branch from here to the barrier: the counted waits for the activations must know exactly
        // how many requests follow them
        const bool has_row = tid < tiles_here * kTileRows && local_to_pos(tid) < a.Q;
        const uint4 f = a.fin[has_row ? local_to_pos(tid) : 0];
        if (has_row) e_fin = f;
    } else {
        if (tid < tiles_here * kTileRows && local_to_pos(tid) < a.Q) e_fin = a.fin[local_to_pos(tid)];
    }

    const int64_t clamp_byte = (a.ids_bytes - 8) & ~(int64_t)3;
    uint4 wlo[T], whi[T];
    uint32_t info = 0;
    // Requests the lane's slices of all T steps of the wave's tile number tk: 2T loads, none under a branch, all from
    // addresses inside the buffer (lanes whose row is not sliced, and steps past the end of the row, read the first
    // 32 bytes of `ids`).  Returns width | 1 << 8 for a sliced row, 0 otherwise.
    // Requests go out in a lane order that the L1 can merge: lane l asks for chunk l % 4 of row l / 4, so four
    // neighbouring lanes read 4 x 4*nb consecutive bytes of one row (in operand order -- lane = row + 16 * chunk --
    // every lane is a row of its own: measured 61 L1 accesses per request instruction against 25 this way, and about
    // 1.3 % of the decode step).  to_operand then moves a register from request order to operand order across the wave.
    // PL (the weight has rows stored in planes): every lane asks for its own operand's slice -- for a row in planes the two
    // requests of a wave are then one contiguous run each (plane A: 1024 bytes, plane B: 256 (nb - 4)), nothing is read
    // twice, and the loads can be non-temporal; the few rows that are not in planes (tiles across two widths, the last
    // rows) are asked for row by row in the same lane order.  No move across the wave afterwards.
    const int lr = PL ? r : lane >> 2, lk = PL ? kg : lane & 3;
    const int pull = 4 * (4 * r + kg);                         // byte address of the lane whose request holds this lane's operand
    auto to_operand = [&](const uint4& v) -> uint4 {
        if constexpr (PL) return v;
        return uint4{(uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.x), (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.y),
                     (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.z), (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.w)};
    };
    auto issue_tile = [&](int tk, int step0, uint4 (&wlo)[T], uint4 (&whi)[T], bool has_tile = true) -> uint32_t {
        const uint64_t rec_read = my_loc[tk * kTileRows + lr];
        const uint64_t rec = has_tile ? rec_read : 3ull << 56;  // a wave without tiles: no row, every request reads the buffer's start
        const uint32_t nb = (uint32_t)(rec >> 48) & 0xFFu, kind = (uint32_t)(rec >> 56) & 3u;
        const bool row_sliced = kind == 1u;
        if constexpr (PL) {
            const bool in_planes = ((rec >> 58) & 1ull) != 0;
            const uint32_t slot = (uint32_t)((rec >> 59) & 15ull) + 16u * (uint32_t)lk;      // the lane's place in a plane
            const uint64_t base = (rec & kRowOffMask) >> 3;
            // first / last four dwords of the slice: in planes the last four end with the lane's share of plane B
            const uint64_t lo0 = in_planes ? base + slot * 16u : base + (uint64_t)lk * (4u * nb);
            const uint64_t hi0 = in_planes ? base + 1024u + (uint64_t)slot * (4u * (nb - 4u)) + 4u * (nb - 4u) - 16u : lo0 + 4u * (nb - 4u);
            const uint32_t step_bytes = in_planes ? 256u * nb : 16u * nb;
#pragma unroll
            for (int it = 0; it < T; ++it) {
                const bool use = row_sliced && (step0 + it) < a.n_steps;
                const uint64_t at = (uint64_t)(step0 + it) * step_bytes;
                const v4u_t va = __builtin_nontemporal_load(reinterpret_cast<const v4u_t*>(a.ids + (use ? lo0 + at : 0)));
                const v4u_t vb = __builtin_nontemporal_load(reinterpret_cast<const v4u_t*>(a.ids + (use ? hi0 + at : 16)));
                wlo[it] = uint4{va.x, va.y, va.z, va.w};
                whi[it] = uint4{vb.x, vb.y, vb.z, vb.w};
            }
        } else {
            const uint64_t row_off = ((rec & kRowOffMask) >> 3) + (uint64_t)(step0 * 4 + lk) * (4u * nb);
            const uint32_t step_bytes = 16u * nb;
            const uint32_t tail = row_sliced ? 4u * (nb - 4u) : 16u;
#pragma unroll
            for (int it = 0; it < T; ++it) {
                const bool use = row_sliced && (step0 + it) < a.n_steps;
                const uint64_t off = use ? row_off + (uint64_t)it * step_bytes : 0;
                wlo[it] = *reinterpret_cast<const uint4*>(a.ids + off);
                whi[it] = *reinterpret_cast<const uint4*>(a.ids + off + tail);
            }
        }
        const uint64_t rec2 = my_loc[tk * kTileRows + r];       // what the lane will decode: its operand row's width
        return has_tile && ((uint32_t)(rec2 >> 56) & 3u) == 1u ? (((uint32_t)(rec2 >> 48) & 0xFFu) | (1u << 8)) : 0u;
    };

    const uint32_t x_row_bytes = (uint32_t)a.P * 2u, x_zero_at = (uint32_t)a.M * x_row_bytes;
    if constexpr (XL) {
        info = issue_tile(0, wc * T, wlo, whi, n_tiles > 0);   // steps past the row's end read the buffer's start as well
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const int idx = tid + i * (int)blockDim.x;
            v4u_t v = xg[i];
            if constexpr (XC) {
#pragma unroll
                for (int k = 0; k < 4; ++k) v[k] = XI::pair(v[k]);
            }
            if (idx < x_pieces) reinterpret_cast<v4u_t*>(xs)[idx] = v;
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (JIT) { if (tid < 16) reinterpret_cast<uint32_t*>(xs + x_zero_at)[tid] = 0u; }   // 64 bytes of zeros behind X
        // A bare barrier behind this wave's own LDS writes: __syncthreads() carries a release fence that would also wait
        // for the ids just requested.
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    }

    for (int panel = 0; panel < a.panels; ++panel) {
        const int step0 = (panel * a.W + wc) * T;             // first global step of this wave in this panel
        const bool active = step0 < a.n_steps;                          // wave-uniform
        const int range = wc;
        const bool first_panel = panel == 0;
        const int n_mine = active ? n_tiles : 0;
        const int step0_next = step0 + a.W * T;
        const bool more = n_mine > 0 && panel + 1 < a.panels && step0_next < a.n_steps;
        // ---- activations of this wave's columns, in MFMA operand layout: lane (t = l % 16, kg) holds
        //      X[16*nt + t][128*(step0+it) + 32*kg + 8*j + 0..7] ----
        v4u_t xa[NT][T][4];
        auto x_operand = [&](int it, v4u_t (&xv)[4]) __attribute__((always_inline)) {
            const bool on = active && r < a.M && (step0 + it) < a.n_steps;
            const uint32_t at = on ? (uint32_t)r * x_row_bytes + 2u * ((uint32_t)(step0 + it) * kStepCols + (uint32_t)kg * 32u) : x_zero_at;
#pragma unroll
            for (int j = 0; j < 4; ++j) xv[j] = *reinterpret_cast<const v4u_t*>(xs + at + 16 * j);
        };
        if constexpr (XT) {
            // lane l of load i: row 4 i + l / 16 (rows past the last one read the last one again: their products are never
            // stored; leaving those requests and their narrowing out under a test of the row count was measured and cost 7 %
            // at 16 rows, where nothing is left out: the tests break up the burst), bytes 16 (l % 16) .. of the step's 256; a
            // step past the end of the rows holds zeros
            const uint32_t row4 = (uint32_t)lane >> 4, last_row = (uint32_t)a.M - 1u;
            uint32_t lane_at[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) lane_at[i] = min(4u * i + row4, last_row) * (uint32_t)a.P * 2u + ((uint32_t)lane & 15u) * 16u;
#pragma unroll
            for (int it = 0; it < T; ++it) {
                if (active && (step0 + it) < a.n_steps) {                  // wave-uniform
                    const unsigned char* base = reinterpret_cast<const unsigned char*>(a.X) + (size_t)(step0 + it) * (kStepCols * 2);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const uint4 v = *reinterpret_cast<const uint4*>(base + lane_at[i]);
                        xa[0][it][i] = v4u_t{v.x, v.y, v.z, v.w};
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) xa[0][it][i] = v4u_t{0, 0, 0, 0};
                }
            }
        }
#pragma unroll
        for (int nt = 0; nt < ((JIT || XT) ? 0 : NT); ++nt) {
            const int t = nt * 16 + r;
#pragma unroll
            for (int it = 0; it < T; ++it) {
#pragma unroll
                for (int j = 0; j < 4; ++j) xa[nt][it][j] = v4u_t{0, 0, 0, 0};
                if (active && t < a.M && (step0 + it) < a.n_steps) {
                    const size_t at = (size_t)t * a.P + (size_t)(step0 + it) * kStepCols + kg * 32;
                    if constexpr (XL) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) xa[nt][it][j] = *reinterpret_cast<const v4u_t*>(xs + 2 * at + 16 * j);
                    } else {
                        const uint16_t* xp = a.X + at;
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const uint4 v = *reinterpret_cast<const uint4*>(xp + 8 * j);
                            xa[nt][it][j] = v4u_t{v.x, v.y, v.z, v.w};
                        }
                    }
                }
            }
        }
        if constexpr (XC && !XL) {          // after ALL requests are out: narrowing inside the branches above would wait per branch
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int it = 0; it < T; ++it)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int k = 0; k < 4; ++k) xa[nt][it][j][k] = XI::pair(xa[nt][it][j][k]);
        }
        if constexpr (XT) {
            // into operand order: piece (row, chunk) is written where lane (row, chunk / 4) finds it as its register chunk % 4;
            // rows are 272 bytes apart, so that the eight lanes LDS serves per cycle touch all banks both ways.  The region is
            // this wave's own and a wave's LDS accesses keep their order: no barrier, and the next step may overwrite it.
            unsigned char* tr = xs + (size_t)wave * kTileTransitBytes;
            const uint32_t put = (uint32_t)(lane >> 4) * kTileTransitRow + (uint32_t)(lane & 15) * 16u;
            const uint32_t get = (uint32_t)r * kTileTransitRow + (uint32_t)kg * 64u;
#pragma unroll
            for (int it = 0; it < T; ++it) {
#pragma unroll
                for (int i = 0; i < 4; ++i) *reinterpret_cast<v4u_t*>(tr + put + 4u * i * kTileTransitRow) = xa[0][it][i];
#pragma unroll
                for (int j = 0; j < 4; ++j) xa[0][it][j] = *reinterpret_cast<const v4u_t*>(tr + get + 16u * j);
            }
        }
        // sums of x over the wave's columns: the product with a matrix of ones, in the accumulator layout
        // (lane (row r, token group kg) register e <-> token 4*kg + e; identical for every r)
        const v4u_t ones = {F::one_bits, F::one_bits, F::one_bits, F::one_bits};
        v4f_t sx[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            sx[nt] = v4f_t{0.f, 0.f, 0.f, 0.f};
            if constexpr (!JIT) {
#pragma unroll
                for (int it = 0; it < T; ++it)
#pragma unroll
                    for (int j = 0; j < 4; ++j) sx[nt] = F::mfma(xa[nt][it][j], ones, sx[nt]);
            }
        }
        // JIT: the sums are taken while the wave's first tile is multiplied (its operands are in registers then)
        auto put_sums = [&]() __attribute__((always_inline)) {
            if (active && g == 0 && r == 0) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float* dst = sxs + range * TM + nt * 16 + kg * 4 + e;
                        *dst = first_panel ? sx[nt][e] : *dst + sx[nt][e];
                    }
            }
        };
        if constexpr (!JIT) put_sums();
        // The first tile's ids are requested only now, after the activations have ARRIVED: requesting them earlier --
        // before the activations, or right behind them -- was measured to cost about a microsecond per launch (the few
        // activation requests then compete with the flood of id requests of the whole chip).
        // (Measured again with the activations fetched in memory order, 16 rows of X: ids right behind the activations 0.532 ms
        // for 8 layers against 0.500 this way.)
        // Later panels' first ids are in flight already (requested at the end of the panel before).
        if constexpr (!XL) { if (n_mine > 0 && first_panel) info = issue_tile(0, step0, wlo, whi); }

        for (int tk = 0; tk < n_mine; ++tk) {
            v4f_t acc[NT], acc_top[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) { acc[nt] = v4f_t{0.f, 0.f, 0.f, 0.f}; acc_top[nt] = v4f_t{0.f, 0.f, 0.f, 0.f}; }
            const uint32_t nb = info & 0xFFu;
            const bool sliced = (info >> 8) == 1u;
            const uint32_t info0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)info);
            const bool uniform = __builtin_amdgcn_ballot_w64(info != info0) == 0 && (info0 >> 8) == 1u && !(BF && (info0 & 0xFFu) == 8u);
#pragma unroll
            for (int it = 0; it < T; ++it) {
                v4u_t b[4];
                const int xi = JIT ? 0 : it;
                if constexpr (JIT) {
                    x_operand(it, xa[0][0]);                       // this step's operands, in the first register set
                    if (tk == 0) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) sx[0] = F::mfma(xa[0][0][j], ones, sx[0]);
                    }
                }
                const uint4 lo = to_operand(wlo[it]), hi = to_operand(whi[it]);
                if (uniform) {
                    switch (info0 & 0xFFu) {
                        case 7: decode_slice<7, BF>(lo, hi, b); break;
                        case 6: decode_slice<6, BF>(lo, hi, b); break;
                        case 5: decode_slice<5, BF>(lo, hi, b); break;
                        case 4: decode_slice<4, BF>(lo, hi, b); break;
                        default: decode_slice<8, BF>(lo, hi, b); break;
                    }
                } else {
                    // mixed tile: one pass per width present; lanes without a sliced row multiply id 0
#pragma unroll
                    for (int j = 0; j < 4; ++j) b[j] = v4u_t{F::bias_bits, F::bias_bits, F::bias_bits, F::bias_bits};
                    if (__builtin_amdgcn_ballot_w64(sliced && nb == 7)) { if (sliced && nb == 7) decode_slice<7, BF>(lo, hi, b); }
                    if (__builtin_amdgcn_ballot_w64(sliced && nb == 6)) { if (sliced && nb == 6) decode_slice<6, BF>(lo, hi, b); }
                    if (__builtin_amdgcn_ballot_w64(sliced && nb == 5)) { if (sliced && nb == 5) decode_slice<5, BF>(lo, hi, b); }
                    if (__builtin_amdgcn_ballot_w64(sliced && nb == 4)) { if (sliced && nb == 4) decode_slice<4, BF>(lo, hi, b); }
                    if (__builtin_amdgcn_ballot_w64(sliced && nb == 8)) {
                        if (sliced && nb == 8) decode_slice<8, BF>(lo, hi, b);
                        if constexpr (BF) {
                            v4u_t bt[4];
#pragma unroll
                            for (int j = 0; j < 4; ++j) bt[j] = v4u_t{0, 0, 0, 0};
                            if (sliced && nb == 8) decode_slice8_top(lo, hi, bt);
#pragma unroll
                            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                                for (int j = 0; j < 4; ++j) acc_top[nt] = F::mfma(xa[nt][xi][j], bt[j], acc_top[nt]);
                        }
                    }
                }
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[nt] = F::mfma(xa[nt][xi][j], b[j], acc[nt]);
            }
            // the next tile's ids (after the last tile: the next panel's first) are requested before this tile's sums
            // are put away
            if (tk + 1 < n_mine) info = issue_tile(tk + 1, step0, wlo, whi);
            else if (more) info = issue_tile(0, step0_next, wlo, whi);
            if constexpr (JIT) { if (tk == 0) put_sums(); }

            // ---- tile done for this wave: remove the bias, store into the wave's own LDS slots ----
            const int lt = g + a.G * tk;                                // the workgroup's local tile
            const int lrow = lt * kTileRows + r;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int t = nt * 16 + kg * 4 + e;
                    float v = __builtin_fmaf(-F::bias, sx[nt][e], acc[nt][e]);
                    if constexpr (BF) v = __builtin_fmaf(kTopBitScale, acc_top[nt][e], v);
                    if (t < a.M) {
                        float* dst = part + ((size_t)lrow * ranges + range) * MS + t;
                        *dst = first_panel ? v : *dst + v;
                    }
                }
            }
            // rows the sliced path cannot read: redo them element by element
            const uint32_t kind_here = (uint32_t)(my_loc[tk * kTileRows + r] >> 56) & 3u;
            uint64_t odd = __builtin_amdgcn_ballot_w64(kg == 0 && (kind_here == 0u || kind_here == 2u));
            while (odd) {
                const int rr = __builtin_ctzll(odd);
                odd &= odd - 1;
                const int lr2 = lt * kTileRows + rr;
                const uint64_t rec = my_loc[tk * kTileRows + rr];
                const int nb2 = (int)((rec >> 48) & 0xFFu);
                const bool readable = ((rec >> 56) & 3u) != 0u;
                const int64_t bit0 = (int64_t)(rec & kRowOffMask);
                const int c_lo = step0 * kStepCols, c_hi = min(a.P, (step0 + T) * kStepCols);
                for (int t = 0; t < a.M; ++t) {
                    float sacc = 0.f;
                    if (readable) {
                        for (int c = c_lo + lane; c < c_hi; c += kWave) {
                            const float idf = (float)load_field(a.ids, bit0 + (int64_t)c * nb2, nb2, clamp_byte);
                            sacc = __builtin_fmaf(XI::scalar(a.X[(size_t)t * a.P + c]), idf, sacc);
                        }
                    } else {
                        sacc = __builtin_nanf("");
                    }
                    const float tot = wave_sum(sacc);
                    // the sliced pass stored this wave's value for the row already (zero contribution plus earlier panels)
                    if (lane == 0) part[((size_t)lr2 * ranges + range) * MS + t] += tot;
                }
            }
        }
    }
    if (tid < rows_cap) s_fin[tid] = e_fin;
    __syncthreads();

    // ---- combine the column ranges of each row in ascending order ----
    const int all_ranges = (a.n_steps + T - 1) / T;
    const int valid_ranges = all_ranges < ranges ? all_ranges : ranges;      // waves without any column never stored
    const int n_items = tiles_here * kTileRows * a.M;
    const int n_waves_here = (int)blockDim.x >> 6;
    if (n_items <= 4 * n_waves_here) {
        // Few results (one token, a few tiles): a thread per (result, range) instead of a thread per result that walks
        // the ranges one LDS trip after the other while every other wave idles.  Sixteen neighbouring lanes hold a result's
        // terms (zero past the last range) and add them up as a fixed tree -- (0+8)+(4+12) ... -- in double; four results
        // per wave and pass.
        for (int first = wave * 4; first < n_items; first += n_waves_here * 4) {
            const int i = first + (lane >> 4), w = lane & 15;
            const bool item = i < n_items;
            const int rl = item ? i / a.M : 0, t = item ? i - rl * a.M : 0;
            const bool live = item && w < valid_ranges;
            const int wr = live ? w : 0;
            const float pv = part[((size_t)rl * ranges + wr) * MS + t], sv = sxs[wr * TM + t];
            double dsum = live ? (double)pv : 0.0, xsum = live ? (double)sv : 0.0;
            dsum += row16_from<8>(dsum); xsum += row16_from<8>(xsum);
            dsum += row16_from<4>(dsum); xsum += row16_from<4>(xsum);
            dsum += row16_from<2>(dsum); xsum += row16_from<2>(xsum);
            dsum += row16_from<1>(dsum); xsum += row16_from<1>(xsum);
            const uint4 f = s_fin[rl];
            if (item && w == 0 && f.z < (uint32_t)a.Q)
                store_y(a.Y, a.out_dt, (int64_t)t * a.Q + f.z, (float)((double)__uint_as_float(f.x) * dsum + (double)__uint_as_float(f.y) * xsum));
        }
        return;
    }
    for (int i = tid; i < n_items; i += blockDim.x) {
        const int rl = i / a.M, t = i - rl * a.M;
        const uint4 f = s_fin[rl];
        if (f.z >= (uint32_t)a.Q) continue;
        double dsum = 0.0, xsum = 0.0;
        for (int w = 0; w < valid_ranges; ++w) {
            dsum += (double)part[((size_t)rl * ranges + w) * MS + t];
            xsum += (double)sxs[w * TM + t];
        }
        store_y(a.Y, a.out_dt, (int64_t)t * a.Q + f.z, (float)((double)__uint_as_float(f.x) * dsum + (double)__uint_as_float(f.y) * xsum));
    }
}

// Escape correction for any M: one thread per (output row with escapes, token), ascending order, no atomics.
template <bool BF, bool XC>
__global__ void __launch_bounds__(256) tile_fix_escapes_kernel(const uint16_t* __restrict__ X, int M,
        const uint8_t* __restrict__ ids, int64_t ids_bytes, const float* __restrict__ min_s, const float* __restrict__ tau_s,
        const uint8_t* __restrict__ nbits, const int64_t* __restrict__ bit_off, const int64_t* __restrict__ esc_idx,
        const float* __restrict__ esc_vals, int64_t n_esc, float* __restrict__ Y, int Q, int P) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int t = blockIdx.y;
    if (i >= n_esc || t >= M) return;
    const int64_t q = esc_idx[i] / P;
    if (q < 0 || q >= Q) return;
    if (i > 0 && esc_idx[i - 1] / P == q) return;
    const int nb = nbits[q];
    const int64_t bit0 = bit_off[q];
    const float ts = tau_s[q], mn = min_s[q];
    const int64_t clamp_byte = (ids_bytes - 8) & ~(int64_t)3;
    float acc = 0.f;
    for (int64_t e = i; e < n_esc && esc_idx[e] / P == q; ++e) {
        const int c = (int)(esc_idx[e] - q * P);
        const float banded = __builtin_fmaf((float)row_field(ids, bit0, nb, c, clamp_byte), ts, mn);
        acc = __builtin_fmaf(XIn<BF, XC>::scalar(X[(size_t)t * P + c]), esc_vals[e] - banded, acc);
    }
    Y[(size_t)t * Q + q] += acc;
}

// ---- fused decode + GEMM, M = 49..256 ---------------------------------------------------------------------------------
// For this many rows of X the activations no longer fit a wave's registers, and every byte of X must serve many weight
// rows: a workgroup (4 waves) takes 256 weight rows of ONE width x TMK = 32 * MT = 64 rows of X x one range of columns.  X goes
// through LDS in stages of 128 columns (double-buffered); the weights never touch LDS: lane (n = l % 32, kh = l / 32) of a
// wave owns the 32 consecutive ids of row n at columns 64 * step + 32 * kh, fetched as two 16-byte loads and decoded
// into the B operands of four v_mfma_f32_32x32x16 (the K order inside a step is a permutation that X follows).  The id
// registers form a ring of four steps: a step's registers are asked for the step four ahead as soon as it has been
// decoded, so about 256 columns of every row of the workgroup are in flight at any time.  A wave keeps 2 row tiles x MT
// token tiles of 32 x 32 sums (every X operand read from LDS feeds two MFMAs).  The main loop has no branch: a column
// range is a whole number of 256-column groups, and requests past its end read its last step again.
// A pass over X beforehand (gemm_prep_kernel) narrows bf16 activations once (XC) and adds up each row of X per column
// range: the sums remove the bias of `bias + id` and carry min_s.  Column ranges (blockIdx.z) write partial results that
// a last kernel adds in order.  Needs rows stored in width order (the layout of qvb8_mma), widths 4..8 (bf16 operands:
// 4..7) and P % 256 == 0.
constexpr int kGemmRows = 256, kGemmWaveRows = 64, kGemmStageCols = 128;
constexpr int kGemmXStride = kGemmStageCols * 2 + 16;              // bytes per row of X of one stage in LDS (padded: conflict-free 16-byte reads)

struct GemmArgs {
    const uint16_t* X;             // (M, P) in the operand format
    const uint8_t* ids; const uint4* fin;
    const float* sx;               // [splits][M] sums of X over each column range
    float* out;                    // Y (one column range) or the partial results [splits][M][Q]
    int M, Q, P;
    int out_dt;                    // what `out` holds when there is one column range: 0 fp32, 1 fp16, 2 bf16 (partial results are fp32)
    int stages_per_split;          // even
    int first1, first2;            // positions where the second and the third width start (Q when there is none)
    int blocks1, blocks2;          // row blocks before the second / the third width (blocks of 256 positions from a width's first)
    uint32_t widths;               // nb0 | nb1 << 8 | nb2 << 16
    int planes;                    // whole 16-row tiles inside a run are stored in planes (see qvb8_device.h)
};

// grid (M, splits): sx[z][m] = sum of row m of X over column range z, as the operands see it; XC: X16[m] = the row narrowed
// tile_rows > 0: X16 is written for every operand format, stage by stage -- [block of tile_rows rows][P / 64][tile_rows][64 columns] -- so that
// the 64 columns of all rows that a workgroup stages together are one contiguous run (rows of a row-major X are a
// multiple of 4 KB apart: the same few L2 channels for every row of a stage, asked by every workgroup at once)
template <bool BF, bool XC>
__global__ void __launch_bounds__(256) gemm_prep_kernel(const uint16_t* __restrict__ X, int M, int P, int cols_per_split,
                                                        uint16_t* __restrict__ X16, float* __restrict__ sx, int tile_rows) {
    __shared__ float red[4];
    const int m = blockIdx.x, z = blockIdx.y, tid = threadIdx.x;
    const int c_begin = z * cols_per_split, c_end = min(P, c_begin + cols_per_split);
    float part = 0.f;
    for (int c = c_begin + 8 * tid; c < c_end; c += 8 * 256) {
        const uint4 v = *reinterpret_cast<const uint4*>(X + (size_t)m * P + c);
        uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            w[k] = XIn<BF, XC>::pair(w[k]);
            part += Fmt<BF>::to_f32(w[k] & 0xFFFFu) + Fmt<BF>::to_f32(w[k] >> 16);
        }
        if (tile_rows > 0) *reinterpret_cast<uint4*>(X16 + (((size_t)(m / tile_rows) * (P >> 6) + (c >> 6)) * tile_rows + m % tile_rows) * 64 + (c & 63)) = uint4{w[0], w[1], w[2], w[3]};
        else if constexpr (XC) *reinterpret_cast<uint4*>(X16 + (size_t)m * P + c) = uint4{w[0], w[1], w[2], w[3]};
    }
    part = wave_sum(part);
    if ((tid & 63) == 0) red[tid >> 6] = part;
    __syncthreads();
    if (tid == 0) sx[(size_t)z * M + m] = (red[0] + red[1]) + (red[2] + red[3]);
}

// The workgroup's rows are positions [pos0, pos0 + 256) of a run of width NB that ends at pos_end and starts at byte
// run_byte0 (position run_first) of the ids buffer.
template <int MT, bool BF, bool XC, int NB, int RT>
__device__ __forceinline__ void gemm_run(const GemmArgs& a, int pos0, int pos_end, int run_first, uint64_t run_byte0, unsigned char* smem) {
    using F = Fmt<BF>;
    using XI = XIn<BF, XC>;
    constexpr int TMK = 32 * MT;                   // rows of X per workgroup
    constexpr int THREADS = 64 * (kGemmRows / (32 * RT));          // RT row tiles of 32 per wave: 4 waves (RT = 2) or 8 (RT = 1)
    constexpr int XROWS = THREADS / 16;            // rows of X staged per pass of the workgroup
    constexpr int XL = (TMK * 16 + THREADS - 1) / THREADS;          // 16-byte pieces of a stage per thread
    unsigned char* xs = smem;                                              // [2][TMK][kGemmXStride]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 31, kh = lane >> 5;
    const int tok0 = (int)blockIdx.y * TMK;
    const int s_begin = (int)blockIdx.z * a.stages_per_split;
    const int s_end = min(a.P / kGemmStageCols, s_begin + a.stages_per_split);
    const int u_begin = 2 * s_begin, u_end = 2 * s_end;                    // 64-column steps; u_end - u_begin is a multiple of 4
    if (u_begin >= u_end) return;

    // ---- this lane's RT rows; a position past the run reads the run's last row (finite operands, result not stored) ----
    const uint8_t* row_ptr[RT]; const uint8_t* row_hi[RT]; int row_pos[RT]; bool row_ok[RT], row_pl[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int pos = pos0 + wave * (32 * RT) + rt * 32 + n;
        row_ok[rt] = pos < pos_end;
        row_pos[rt] = row_ok[rt] ? pos : pos_end - 1;
        // requests go out in the order lane = 2 * row + half, so that neighbouring lanes read neighbouring bytes
        // (fewer L1 accesses per request); to_operand moves the registers into operand order (lane = row + 32 * half).
        // (With rows stored in planes, requests in operand order -- contiguous, no move afterwards -- were measured: no gain.)
        const int rpos = min(pos0 + wave * (32 * RT) + rt * 32 + (lane >> 1), pos_end - 1);
        const uint32_t rhalf = (uint32_t)(lane & 1);
        const uint64_t row_bytes = (uint64_t)a.P * NB / 8;
        // a row of a whole tile inside the run may be stored in planes: first / last four dwords of its slice then come
        // from the tile's two planes (the slice of 64-column step u, half h is column group 2 u + h of the row)
        const int t0 = rpos & ~15;
        row_pl[rt] = a.planes != 0 && t0 >= run_first && t0 + 16 <= pos_end;
        if (row_pl[rt]) {
            const uint8_t* tile = a.ids + run_byte0 + (uint64_t)(t0 - run_first) * row_bytes;
            const uint32_t slot = (uint32_t)(rpos & 15) + 16u * rhalf;
            row_ptr[rt] = tile + slot * 16u;
            row_hi[rt] = tile + 1024u + slot * (4u * (NB - 4u)) + 4u * (NB - 4u) - 16u;
        } else {
            row_ptr[rt] = a.ids + run_byte0 + (uint64_t)(rpos - run_first) * row_bytes + rhalf * (4u * NB);
            row_hi[rt] = row_ptr[rt] + 4u * (NB - 4u);
        }
    }
    const int pull = 4 * (2 * n + kh);
    auto to_operand = [pull](const uint4& v) -> uint4 {
        return uint4{(uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.x), (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.y),
                     (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.z), (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.w)};
    };
    uint4 raw[4][RT][2];                            // [step % 4][row tile][first / last four dwords]
    auto request_ids = [&](int u, uint4 (&w)[RT][2]) {
        const uint32_t uc = (uint32_t)min(u, u_end - 1);
        const uint32_t off = uc * (8u * NB);                               // a step is 64 columns = 8 NB bytes of a row
        const uint32_t pa = (uc >> 1) * (256u * NB) + (uc & 1u) * 512u;    // in planes: step u / 2, column groups 2 (u % 2) + half
        const uint32_t pb = (uc >> 1) * (256u * NB) + (uc & 1u) * (128u * (NB - 4u));
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            w[rt][0] = *reinterpret_cast<const uint4*>(row_ptr[rt] + (row_pl[rt] ? pa : off));
            w[rt][1] = *reinterpret_cast<const uint4*>(row_hi[rt] + (row_pl[rt] ? pb : off));
        }
    };
    // ---- X: thread tid stages piece tid % 16 (8 columns) of rows tid / 16 + 16 * i; rows past M read row M - 1 (not stored at the end) ----
    const int xch = tid & 15, xrow = tid >> 4;                  // with 512 threads a stage of 32 rows of X is one piece for every thread
    const uint16_t* const x_base = a.X + 8 * xch;
    const int M = a.M, P = a.P;
    v4u_t xg[XL];
    auto request_x = [=](int st, v4u_t (&g)[XL]) {
        const uint32_t c = (uint32_t)min(st, s_end - 1) * kGemmStageCols;
#pragma unroll
        for (int i = 0; i < XL; ++i) g[i] = *reinterpret_cast<const v4u_t*>(x_base + (size_t)min(tok0 + xrow + XROWS * i, M - 1) * P + c);
    };
    // XC: bf16 activations are narrowed like saturating_half on their way into LDS (every workgroup narrows the 16 KB it
    // stages; a pass of its own over X would be one more launch per product)
    auto store_x = [=](int buf, const v4u_t (&g)[XL]) {
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            v4u_t v = g[i];
            if constexpr (XC) {
#pragma unroll
                for (int k = 0; k < 4; ++k) v[k] = XI::pair(v[k]);
            }
            *reinterpret_cast<v4u_t*>(xs + ((size_t)buf * TMK + xrow + XROWS * i) * kGemmXStride + 16 * xch) = v;
        }
    };

    v16f_t acc[RT][MT];
    // sums of the rows of X over this workgroup's columns, as the operands see them: the product with a matrix of ones,
    // in the accumulator layout (register i of every lane <-> the token that acc[.][mt][i] belongs to).  (Added up on the
    // vector ALU while X is staged instead -- a third fewer matrix instructions -- was measured slower: M = 64 0.995 against
    // 0.951 ms per 8 layers.)
    v16f_t sxa[MT];
    const v4u_t ones = {F::one_bits, F::one_bits, F::one_bits, F::one_bits};
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sxa[mt][i] = 0.f;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[rt][mt][i] = 0.f;

    request_x(s_begin, xg);
#pragma unroll
    for (int k = 0; k < 4; ++k) request_ids(u_begin + k, raw[k]);
    store_x(0, xg);
    __syncthreads();
    for (int u0 = u_begin; u0 < u_end; u0 += 4) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int h = k & 1, buf = k >> 1;
            if (h == 0) request_x((u0 >> 1) + buf + 1, xg);
            v4u_t b[RT][4];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) decode_slice<NB, BF>(to_operand(raw[k][rt][0]), to_operand(raw[k][rt][1]), b[rt]);
            request_ids(u0 + k + 4, raw[k]);
            __builtin_amdgcn_sched_barrier(0);                             // the requests stay ahead of the products
            const unsigned char* xb = xs + (size_t)buf * TMK * kGemmXStride + (size_t)n * kGemmXStride + 2 * (64 * h + 32 * kh);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const uint4 v = *reinterpret_cast<const uint4*>(xb + (size_t)(32 * mt) * kGemmXStride + 16 * j);
                    const v4u_t av = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) acc[rt][mt] = F::mfma32(av, b[rt][j], acc[rt][mt]);
                    // eight waves: the sums are shared work -- wave w < 4 adds up the columns of operand j = w, joined at the end
                    if (RT == 2 || j == wave) sxa[mt] = F::mfma32(av, ones, sxa[mt]);
                }
            if (h == 1) {
                store_x(buf ^ 1, xg);
                __syncthreads();
            }
        }
    }
    // ---- the end: lane holds, for row n of each row tile, tokens 32 mt + 8 (i / 4) + 4 kh + i % 4 ----
    float* sxs = reinterpret_cast<float*>(smem);                           // [4][TMK]; the X stages are no longer read (barrier above)
    if constexpr (RT == 1) {
        if (wave < 4 && n == 0) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int i = 0; i < 16; ++i) sxs[wave * TMK + 32 * mt + 8 * (i >> 2) + 4 * kh + (i & 3)] = sxa[mt][i];
        }
        __syncthreads();
    }
    float* out = a.out + (size_t)blockIdx.z * (size_t)a.M * (size_t)a.Q;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (!row_ok[rt]) continue;
        const uint4 f = a.fin[row_pos[rt]];
        if (f.z >= (uint32_t)a.Q) continue;
        const double ts = (double)__uint_as_float(f.x), mn = (double)__uint_as_float(f.y);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int tl = 32 * mt + 8 * (i >> 2) + 4 * kh + (i & 3);
                const int t = tok0 + tl;
                if (t < a.M) {
                    const float sx = RT == 1 ? ((sxs[tl] + sxs[TMK + tl]) + sxs[2 * TMK + tl]) + sxs[3 * TMK + tl] : sxa[mt][i];
                    const float d = __builtin_fmaf(-F::bias, sx, acc[rt][mt][i]);
                    store_y(out, a.out_dt, (int64_t)t * a.Q + f.z, (float)(ts * (double)d + mn * (double)sx));
                }
            }
    }
}

template <int MT, bool BF, bool XC, int RT>
__global__ void __launch_bounds__(64 * (kGemmRows / (32 * RT))) gemm_kernel(GemmArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    // which run of equal widths this workgroup's 256 positions belong to
    const int bx = (int)blockIdx.x;
    const int c = (bx >= a.blocks1 ? 1 : 0) + (bx >= a.blocks2 ? 1 : 0);
    const uint32_t nb0 = a.widths & 255u, nb1 = (a.widths >> 8) & 255u, nb2 = (a.widths >> 16) & 255u;
    const uint64_t row0 = (uint64_t)a.P * nb0 / 8, row1 = (uint64_t)a.P * nb1 / 8;
    const int run_first = c == 0 ? 0 : c == 1 ? a.first1 : a.first2;
    const int run_end = c == 0 ? a.first1 : c == 1 ? a.first2 : a.Q;
    const uint64_t byte0 = c == 0 ? 0 : c == 1 ? (uint64_t)a.first1 * row0 : (uint64_t)a.first1 * row0 + (uint64_t)(a.first2 - a.first1) * row1;
    const int pos0 = run_first + (bx - (c == 0 ? 0 : c == 1 ? a.blocks1 : a.blocks2)) * kGemmRows;
    if (pos0 >= run_end) return;
    switch (c == 0 ? nb0 : c == 1 ? nb1 : nb2) {
        case 4: gemm_run<MT, BF, XC, 4, RT>(a, pos0, run_end, run_first, byte0, smem); break;
        case 5: gemm_run<MT, BF, XC, 5, RT>(a, pos0, run_end, run_first, byte0, smem); break;
        case 6: gemm_run<MT, BF, XC, 6, RT>(a, pos0, run_end, run_first, byte0, smem); break;
        case 7: gemm_run<MT, BF, XC, 7, RT>(a, pos0, run_end, run_first, byte0, smem); break;
        case 8: if constexpr (!BF) gemm_run<MT, BF, XC, 8, RT>(a, pos0, run_end, run_first, byte0, smem); break;
        default: break;
    }
}

// ---- fused decode + GEMM through LDS, M = 65..256 ----------------------------------------------------------------------
// With this many rows of X every weight must serve many of them once it has been read and decoded: a workgroup takes 128
// weight rows of ONE width x BM rows of X (256: all of X, or 128) x one range of columns, and every id it fetches is
// decoded once, into LDS.  Its 16 waves have two jobs:
//   waves 8..15 fill LDS.  X (stored stage by stage by gemm_prep_kernel): per 64-column stage, 16-byte pieces into the
//         stage's A buffer ([row of X][64 columns], two buffers), requested four stages before they are stored.  ids:
//         per 128-column block, a thread fetches the 32-id slice g of a row (two 16-byte loads; four neighbouring lanes
//         read 16 NB contiguous bytes), decodes it into 32 `bias + id` halves and writes them to the block's B buffer
//         ([weight row][128 columns], two buffers); requested two blocks before they are decoded.
//   waves 0..7 multiply.  Wave (wm, wn) owns 64 rows of X x 32 NT weight rows (NT = 2 for BM = 256, 1 for BM = 128): per
//         16 columns two A operands and NT B operands from LDS (rows padded by 16 bytes: conflict-free 16-byte reads)
//         feed 2 NT v_mfma_f32_32x32x16.  A wave issues in order and both the LDS requests (about 30 cycles each,
//         measured) and the matrix instructions (32 cycles) hold its issue, so two multiplying waves share a SIMD: one
//         requests operands while the other one's products run.
// One barrier per stage, met by all 16 waves.  The end is the end of gemm_run: bias and min_s through the row sums of X
// (gemm_prep_kernel), partial results per column range, added in order by gemm_reduce_kernel.
constexpr int kG2Rows = 128, kG2Cols = 64, kG2Mul = 8, kG2Waves = 16, kG2Fill = 512;   // multiplying waves, all waves, filling threads
constexpr int kG2AStride = kG2Cols * 2 + 16;                       // bytes per row of X of one stage
constexpr int kG2BStride = 2 * kG2Cols * 2 + 16;                   // bytes per weight row of one 128-column block

template <int WM, bool BF, int NB>
__device__ __forceinline__ void gemm2_run(const GemmArgs& a, int pos0, int pos_end, int run_first, uint64_t run_byte0, unsigned char* smem,
                                          int by, int bz) {
    using F = Fmt<BF>;
    constexpr int BM = 64 * WM, WN = kG2Mul / WM, NT = kG2Rows / (32 * WN);   // WM = 4: 256 rows of X, 64 x 64 sums per wave; WM = 2: 128 rows, 64 x 32
    constexpr int MT = 2;
    constexpr int XL = BM * 8 / kG2Fill;                           // 16-byte pieces of a stage per filling thread
    unsigned char* As = smem;                                      // [2][BM][kG2AStride]
    unsigned char* Bs = smem + (size_t)2 * BM * kG2AStride;        // [2][kG2Rows][kG2BStride]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tok0 = by * BM;
    const int s_begin = bz * a.stages_per_split * 2;  // stages_per_split counts 128-column stages
    const int s_end = min(a.P / kG2Cols, s_begin + a.stages_per_split * 2);
    const int n_st = s_end - s_begin;                              // a multiple of 4
    if (n_st <= 0) return;
    const int n_blk = n_st / 2;
    const int wm = wave / WN, wn = wave - wm * WN;                 // of the multiplying waves
    const int n = lane & 31, kh = lane >> 5;
    v16f_t acc[MT][NT];

    if (wave >= kG2Mul) {
        // ================= filling =================
        // Requests run far ahead of their use (X from L2, ids from HBM: one to two microseconds under load): four
        // register sets of X pieces (stage s in set s % 4, requested four stages before it is stored), two of id slices
        // (block b in set b % 2, requested two blocks before it is decoded).  Four stages per turn of the loop.
        const int p = tid - 64 * kG2Mul;
        // ids: slice g = p % 4 of row p / 4 (neighbouring lanes read neighbouring bytes of a row); with rows stored in planes
        // lane l of a wave takes entry l of its tile's planes -- row l % 16, slice l / 16 -- and a wave's request is one
        // contiguous run.  A position past the run reads the run's last row (never stored).
        const bool by_entry = a.planes != 0;
        const int dg = by_entry ? (p >> 4) & 3 : p & 3, drow = by_entry ? (p & 15) + 16 * (p >> 6) : p >> 2;
        const int dpos = min(pos0 + drow, pos_end - 1);
        const uint64_t row_bytes = (uint64_t)a.P * NB / 8;
        // a row of a whole tile inside the run may be stored in planes (a wave's 16 rows x 4 slices are then the tile's two
        // planes, one contiguous run per request)
        const int t0 = dpos & ~15;
        const bool in_planes = a.planes != 0 && t0 >= run_first && t0 + 16 <= pos_end;
        const uint32_t slot = (uint32_t)(dpos & 15) + 16u * (uint32_t)dg;
        const uint8_t* const tile = a.ids + run_byte0 + (uint64_t)(t0 - run_first) * row_bytes;
        const uint32_t blk_bytes = in_planes ? 256u * NB : 16u * NB;
        const uint8_t* const idp = (in_planes ? tile + slot * 16u
                                              : a.ids + run_byte0 + (uint64_t)(dpos - run_first) * row_bytes + (uint32_t)dg * (4u * NB))
                                   + (uint64_t)(s_begin / 2) * blk_bytes;
        const uint8_t* const idh = in_planes ? tile + 1024u + slot * (4u * (NB - 4u)) + 4u * (NB - 4u) - 16u + (uint64_t)(s_begin / 2) * blk_bytes
                                             : idp + 4u * (NB - 4u);
        uint4 raw[2][2];
        auto request_ids = [&](int blk, uint4 (&w)[2]) __attribute__((always_inline)) {
            const uint32_t off = (uint32_t)min(blk, n_blk - 1) * blk_bytes;
            w[0] = *reinterpret_cast<const uint4*>(idp + off);
            w[1] = *reinterpret_cast<const uint4*>(idh + off);
        };
        auto store_ids = [&](int buf, const uint4 (&w)[2]) __attribute__((always_inline)) {
            v4u_t b[4];
            decode_slice<NB, BF>(w[0], w[1], b);
            unsigned char* dst = Bs + ((size_t)buf * kG2Rows + drow) * kG2BStride + 64 * dg;
#pragma unroll
            for (int j = 0; j < 4; ++j) *reinterpret_cast<v4u_t*>(dst + 16 * j) = b[j];
        };
        // X, stored stage by stage ([block of BM rows][stage][BM rows][64 columns], gemm_prep_kernel): piece p % 8 (8
        // columns) of rows p / 8 + 64 i of the block; rows past M read row M - 1 (not stored at the end)
        const int xch = p & 7, xrow = p >> 3;
        const int M = a.M;
        const uint16_t* x_piece[XL];
#pragma unroll
        for (int i = 0; i < XL; ++i)
            x_piece[i] = a.X + (((size_t)by * (a.P / kG2Cols) + s_begin) * BM + min(xrow + 64 * i, M - 1 - tok0)) * kG2Cols + 8 * xch;
        v4u_t xg[4][XL];
        auto request_x = [&](int st, v4u_t (&g)[XL]) __attribute__((always_inline)) {
            const size_t c = (size_t)min(st, n_st - 1) * (BM * kG2Cols);
#pragma unroll
            for (int i = 0; i < XL; ++i) g[i] = *reinterpret_cast<const v4u_t*>(x_piece[i] + c);
        };
        auto store_x = [&](int buf, const v4u_t (&g)[XL]) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < XL; ++i)
                *reinterpret_cast<v4u_t*>(As + ((size_t)buf * BM + xrow + 64 * i) * kG2AStride + 16 * xch) = g[i];
        };
        request_x(0, xg[0]);
        request_ids(0, raw[0]);
        request_x(1, xg[1]);
        request_ids(1, raw[1]);
        request_x(2, xg[2]);
        request_x(3, xg[3]);
        store_x(0, xg[0]);
        request_x(4, xg[0]);
        store_ids(0, raw[0]);
        request_ids(2, raw[0]);
        __syncthreads();
        for (int ls = 0; ls < n_st; ls += 4) {
            const int blk = ls >> 1;                               // even
            // stage ls is multiplied: X of stage ls + 1, ids of block blk + 1 (set 1) into B buffer 1
            store_x(1, xg[1]);
            request_x(ls + 5, xg[1]);
            store_ids(1, raw[1]);
            request_ids(blk + 3, raw[1]);
            __syncthreads();
            store_x(0, xg[2]);                                     // stage ls + 2
            request_x(ls + 6, xg[2]);
            __syncthreads();
            store_x(1, xg[3]);                                     // stage ls + 3; ids of block blk + 2 (set 0) into B buffer 0
            request_x(ls + 7, xg[3]);
            store_ids(0, raw[0]);
            request_ids(blk + 4, raw[0]);
            __syncthreads();
            store_x(0, xg[0]);                                     // stage ls + 4
            request_x(ls + 8, xg[0]);
            __syncthreads();
        }
    } else {
        // ================= multiplying =================
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.f;
        // Operands of 16 columns ahead of their products, in two register sets: the requests for the next 16 columns go to
        // LDS before the matrix instructions of the current ones are issued (a wave issues in order, and the matrix
        // pipe holds the issue for 32 cycles per instruction), and the last 16 columns of a stage are multiplied after
        // the barrier, behind the first requests of the next stage.
        auto operands = [&](int ls, int q, v4u_t (&av)[MT], v4u_t (&bv)[NT]) __attribute__((always_inline)) {
            const unsigned char* Ab = As + ((size_t)(ls & 1) * BM + wm * (32 * MT) + n) * kG2AStride + 16 * kh + 32 * q;
            const unsigned char* Bb = Bs + ((size_t)((ls >> 1) & 1) * kG2Rows + wn * (32 * NT) + n) * kG2BStride + (ls & 1) * (2 * kG2Cols) + 16 * kh + 32 * q;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) av[mt] = *reinterpret_cast<const v4u_t*>(Ab + (size_t)(32 * mt) * kG2AStride);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) bv[nt] = *reinterpret_cast<const v4u_t*>(Bb + (size_t)(32 * nt) * kG2BStride);
        };
        auto products = [&](const v4u_t (&av)[MT], const v4u_t (&bv)[NT]) __attribute__((always_inline)) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = F::mfma32(av[mt], bv[nt], acc[mt][nt]);
        };
        v4u_t av0[MT], bv0[NT], av1[MT], bv1[NT];
        __syncthreads();
        operands(0, 0, av0, bv0);
        for (int ls = 0; ls < n_st; ++ls) {
            operands(ls, 1, av1, bv1);
            __builtin_amdgcn_sched_barrier(0);
            products(av0, bv0);
            __builtin_amdgcn_sched_barrier(0);
            operands(ls, 2, av0, bv0);
            __builtin_amdgcn_sched_barrier(0);
            products(av1, bv1);
            __builtin_amdgcn_sched_barrier(0);
            operands(ls, 3, av1, bv1);
            __builtin_amdgcn_sched_barrier(0);
            products(av0, bv0);
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            operands(ls + 1, 0, av0, bv0);                     // past the last stage: a buffer nobody writes any more, never used
            __builtin_amdgcn_sched_barrier(0);
            products(av1, bv1);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // ---- the end: a multiplying lane holds, for weight row n of each row tile, rows of X 32 mt + 8 (i / 4) + 4 kh + i % 4 ----
    float* sxs = reinterpret_cast<float*>(smem);                   // the buffers are no longer read (barrier above)
    if (tid < BM) sxs[tid] = tok0 + tid < a.M ? a.sx[(size_t)bz * a.M + tok0 + tid] : 0.f;
    __syncthreads();
    if (wave >= kG2Mul) return;
    float* out = a.out + (size_t)bz * (size_t)a.M * (size_t)a.Q;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int pos = pos0 + wn * (32 * NT) + 32 * nt + n;
        if (pos >= pos_end) continue;
        const uint4 f = a.fin[pos];
        if (f.z >= (uint32_t)a.Q) continue;
        const double ts = (double)__uint_as_float(f.x), mn = (double)__uint_as_float(f.y);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int tl = wm * (32 * MT) + 32 * mt + 8 * (i >> 2) + 4 * kh + (i & 3);
                const int t = tok0 + tl;
                if (t < a.M) {
                    const float sx = sxs[tl];
                    const float d = __builtin_fmaf(-F::bias, sx, acc[mt][nt][i]);
                    store_y(out, a.out_dt, (int64_t)t * a.Q + f.z, (float)(ts * (double)d + mn * (double)sx));
                }
            }
    }
}

template <int WM, bool BF>
__global__ void __launch_bounds__(64 * kG2Waves) gemm2_kernel(GemmArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    // Which block of weight rows (bx), block of rows of X (by) and column range (bz) this workgroup takes.  Workgroups go
    // to the eight XCDs in turn (flat number % 8), each XCD with an L2 of its own; dealt in the grid's order, every XCD
    // meets every column range and so fetches all of X (at 256 rows: 8 x 6.3 MB for `down`, more than its ids).  When the
    // number of column ranges divides 8, XCD j instead takes range j % nz only, both blocks of X of it, and every
    // (8 / nz)-th block of weight rows: X crosses the fabric 8 / nz times instead of 8, every id still once.  Measured, 8
    // layers of the 9B shapes: 192 rows of X 1.549 -> 1.521 ms, 256 rows 1.618 -> 1.568 ms, HBM-side traffic per layer
    // 437 -> 383 MB; with one block of X (up to 128 rows: X is 1 MB or less) the grid's own order is 1.5 % faster and is kept.
    int bx = (int)blockIdx.x, by = (int)blockIdx.y, bz = (int)blockIdx.z;
    {
        const int nx = (int)gridDim.x, ny = (int)gridDim.y, nz = (int)gridDim.z;
        const int per = nz <= 8 ? 8 / nz : 0;                      // XCDs that share a column range
        if (ny > 1 && nz > 1 && per * nz == 8 && nx % per == 0) {
            const int flat = bx + nx * (by + ny * bz);
            const int xcd = flat & 7, k = flat >> 3;               // k: the XCD's own count, 0 .. nx * ny / per - 1
            bz = xcd % nz;
            by = k % ny;
            bx = (k / ny) * per + xcd / nz;
        }
    }
    // which run of equal widths this workgroup's 128 positions belong to
    const int c = (bx >= a.blocks1 ? 1 : 0) + (bx >= a.blocks2 ? 1 : 0);
    const uint32_t nb0 = a.widths & 255u, nb1 = (a.widths >> 8) & 255u, nb2 = (a.widths >> 16) & 255u;
    const uint64_t row0 = (uint64_t)a.P * nb0 / 8, row1 = (uint64_t)a.P * nb1 / 8;
    const int run_first = c == 0 ? 0 : c == 1 ? a.first1 : a.first2;
    const int run_end = c == 0 ? a.first1 : c == 1 ? a.first2 : a.Q;
    const uint64_t byte0 = c == 0 ? 0 : c == 1 ? (uint64_t)a.first1 * row0 : (uint64_t)a.first1 * row0 + (uint64_t)(a.first2 - a.first1) * row1;
    const int pos0 = run_first + (bx - (c == 0 ? 0 : c == 1 ? a.blocks1 : a.blocks2)) * kG2Rows;
    if (pos0 >= run_end) return;
    switch (c == 0 ? nb0 : c == 1 ? nb1 : nb2) {
        case 4: gemm2_run<WM, BF, 4>(a, pos0, run_end, run_first, byte0, smem, by, bz); break;
        case 5: gemm2_run<WM, BF, 5>(a, pos0, run_end, run_first, byte0, smem, by, bz); break;
        case 6: gemm2_run<WM, BF, 6>(a, pos0, run_end, run_first, byte0, smem, by, bz); break;
        case 7: gemm2_run<WM, BF, 7>(a, pos0, run_end, run_first, byte0, smem, by, bz); break;
        case 8: if constexpr (!BF) gemm2_run<WM, BF, 8>(a, pos0, run_end, run_first, byte0, smem, by, bz); break;
        default: break;
    }
}

// Y = sum of the column ranges' partial results, in ascending order
__global__ void __launch_bounds__(256) gemm_reduce_kernel(const float* __restrict__ part, float* __restrict__ Y, int64_t n, int splits, int out_dt) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = part[i];
    for (int s = 1; s < splits; ++s) v += part[(int64_t)s * n + i];
    store_y(Y, out_dt, i, v);
}

}  // namespace qvb8

using namespace qvb8;

extern "C" int64_t qvb8_mma_rowinfo_bytes(int64_t Q);

namespace {
struct TilePlan { int W, G, panels, TW, threads; size_t lds; unsigned blocks; };

constexpr size_t kTileLdsLimit = 128 * 1024;
constexpr size_t kTileXLdsLimit = 64 * 1024;     // X through LDS: up to this many bytes of activations on top
constexpr size_t kTileXLdsMost = 140000;         // ... and up to this many for at most 8 rows of X
constexpr size_t kLdsPerWorkgroup = 160 * 1024;

bool plan_tile_for(int NT, int T, int64_t M, int64_t Q, int64_t P, TilePlan& pl, int wave_cap, int per_cu, size_t lds_limit = kTileLdsLimit) {
    const int n_steps = (int)(P / kStepCols);
    const int ranges = (n_steps + T - 1) / T;                 // column ranges of T steps
    // more than eight waves only where that saves a panel
    const int max_waves = (wave_cap > 8 && (ranges + wave_cap - 1) / wave_cap < (ranges + 7) / 8) ? wave_cap : 8;
    pl.panels = (ranges + max_waves - 1) / max_waves;
    pl.W = (ranges + pl.panels - 1) / pl.panels;
    pl.G = pl.panels == 1 ? max_waves / pl.W : 1;
    if (pl.G < 1) pl.G = 1;
    pl.threads = 64 * pl.W * pl.G;
    const int64_t tiles = (Q + kTileRows - 1) / kTileRows;
    const int cus = host::device_cus();
    int64_t target = (int64_t)cus * (per_cu > 0 ? per_cu : 1);
    int64_t tw = (tiles + target - 1) / target;
    tw = (tw + pl.G - 1) / pl.G * pl.G;
    if (tw < pl.G) tw = pl.G;
    while (tw > pl.G && tw * kTileRows > pl.threads) tw -= pl.G;     // the end needs one thread per row of the workgroup
    const size_t TM = 16 * (size_t)NT, rg = (size_t)pl.W;
    for (;;) {
        const size_t rows = (size_t)tw * kTileRows;
        pl.lds = rows * 16 + (size_t)pl.W * pl.G * (tw / pl.G) * kTileRows * 8 + rg * TM * 4 + rows * rg * (size_t)M * 4;
        if (pl.lds <= lds_limit || tw <= pl.G) break;
        tw -= pl.G;
    }
    if (pl.lds > lds_limit) return false;
    // more workgroups than the target (LDS or the thread count capped the tiles of one): a whole number of rounds over the
    // CUs, the tiles spread evenly -- 1035 workgroups on 256 CUs would leave the fifth round to 11 of them
    int64_t blocks = (tiles + tw - 1) / tw;
    if (blocks > target) {
        blocks = (blocks + target - 1) / target * target;
        int64_t even = (tiles + blocks - 1) / blocks;
        even = (even + pl.G - 1) / pl.G * pl.G;
        if (even < tw) tw = even;
        // the rounded number of workgroups is kept (tile t goes to workgroup t % blocks, so each gets tiles / blocks of them,
        // give or take one): ceil(tiles / tw) workgroups would again leave CUs idle in the last round
        if ((tiles + blocks - 1) / blocks > tw) blocks = (tiles + tw - 1) / tw;
    }
    pl.TW = (int)tw;
    pl.blocks = (unsigned)blocks;
    return true;
}
// Workgroups per CU the plan aims at: two where two fit a CU at the same time -- eight waves each (one panel), a kernel of
// at most 128 registers per lane (`pair_fits`: the one-token-tile kernel that reads its operands from LDS step by step),
// and LDS for both (`x_lds` = the activations' bytes on top of the plan's own) -- else one.  Two resident workgroups keep
// more requests in flight and let one's epilogue overlap the other's stream (9B gate+up 19.5 -> 18.4 us); where only one
// fits, twice the workgroups would just be a second round (27B down, twelve waves: 23.2 -> 26.7 us).
bool plan_tile(int NT, int T, int64_t M, int64_t Q, int64_t P, TilePlan& pl, int wave_cap = 8, bool pair_fits = false, size_t x_lds = 0,
               size_t lds_limit = kTileLdsLimit) {
    const int forced = host::env_int("QVB8_TILE_WGS_PER_CU", 0);
    if (forced > 0) return plan_tile_for(NT, T, M, Q, P, pl, wave_cap, forced, lds_limit);
    if (pair_fits && plan_tile_for(NT, T, M, Q, P, pl, wave_cap, 2, lds_limit) && pl.panels == 1 && pl.threads <= 512
        && 2 * (pl.lds + x_lds) <= kLdsPerWorkgroup) return true;
    // (Where two copies of X do not fit -- 5..8 rows of 4096 columns -- one workgroup of sixteen waves sharing one copy was
    // measured: no faster than one of eight, 0.464 against 0.460 ms for 8 layers at 8 rows.)
    return plan_tile_for(NT, T, M, Q, P, pl, wave_cap, 1, lds_limit);
}

// Whether the registers of this kernel let two workgroups of eight waves share a CU (asked of the runtime once per device).
template <int NT, int T, bool BF, bool XC, int XP, bool PL>
bool tile_pair_fits() {
    if constexpr (!(XP > 0 && NT == 1)) return false;
    static int known[64] = {0};                               // 0 not asked yet, 1 no, 2 yes
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
    if (known[dev] == 0) {
        int n = 0;
        const bool ok = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, (const void*)tile_kernel<NT, T, BF, XC, XP, PL>, 512, 0) == hipSuccess;
        if (!ok) (void)hipGetLastError();
        known[dev] = ok && n >= 2 ? 2 : 1;
    }
    return known[dev] == 2;
}

template <int NT, int T, bool BF, bool XC, int XP = 0, bool PL = false>
int launch_tile(TileArgs& a, hipStream_t s) {
    TilePlan pl;
    const bool jit = tile_pair_fits<NT, T, BF, XC, XP, PL>();
    // on top of the plan's own: all of X (XP > 0), or a transit region per wave (one token tile, X not in LDS as a whole)
    const size_t x_lds = XP > 0 ? (size_t)a.M * (size_t)a.P * 2 + 64 : (NT == 1 ? (size_t)tile_max_waves<NT, T, BF, PL>() * kTileTransitBytes : 0);
    const size_t limit = kLdsPerWorkgroup - x_lds < kTileLdsLimit ? kLdsPerWorkgroup - x_lds : kTileLdsLimit;   // what X or the transit regions leave
    if (!plan_tile(NT, T, a.M, a.Q, a.P, pl, host::env_int("QVB8_TILE_WAVES12", 1) ? tile_max_waves<NT, T, BF, PL>() : 8, jit, x_lds, limit))
        return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mma: shape does not fit a workgroup's LDS");
    pl.lds += x_lds;
    a.W = pl.W; a.G = pl.G; a.panels = pl.panels; a.TW = pl.TW;
    static bool attr[64] = {false};                           // per device: the attribute belongs to the device's copy of the kernel
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return host::fail(QVB8_ERR_LAUNCH, "qvb8_mma: no current device");
    if (!attr[dev]) {
        if (hipFuncSetAttribute((const void*)tile_kernel<NT, T, BF, XC, XP, PL>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsPerWorkgroup) != hipSuccess)
            return host::fail(QVB8_ERR_LAUNCH, "qvb8_mma: cannot raise the kernel's LDS limit");
        attr[dev] = true;
    }
    if (pl.panels > 0xffff) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mma: rows too long");
    const uint32_t counts = (uint32_t)a.M | ((uint32_t)a.out_dt << 6) | ((uint32_t)a.W << 8) | ((uint32_t)a.G << 12) | ((uint32_t)a.panels << 16);
    hipLaunchKernelGGL((tile_kernel<NT, T, BF, XC, XP, PL>), dim3(pl.blocks), dim3(pl.threads), pl.lds, s,
                       a.X, a.ids, a.loc, a.Y, a.ids_bytes, a.Q, a.P, counts, a.TW, a.first1, a.first2,
                       (uint32_t)a.nb[0] | ((uint32_t)a.nb[1] << 8) | ((uint32_t)a.nb[2] << 16) | ((uint32_t)a.n_classes << 24));
    return host::check_launch("qvb8_mma");
}
// One to sixteen rows of X on the NT = 1 kernel: X goes through LDS when all of it fits (the limits below, and the
// workgroup's LDS), with 1, 4, 8 or 16 pieces of 16 bytes per thread (a request past the end of X would be a wasted one:
// the count is exact to within those four variants).
template <int T, bool BF, bool XC, bool PL = false>
int launch_tile_rows16(TileArgs& a, hipStream_t s) {
    TilePlan pl;
    const size_t x_bytes = (size_t)a.M * (size_t)a.P * 2;
    // Up to 8 rows of X whatever fits (measured on the 9B `down`, 12288 columns: 3 rows 74 KB, 5 rows 123 KB of X in LDS
    // against fetched per wave: 8 layers 0.420 -> 0.385 ms at 3 rows, 0.428 -> 0.404 at 5); more rows only up to 64 KB (9..16
    // rows of 4096 columns through LDS as a whole leave room for three tiles per workgroup: 0.478 -> 0.543 ms at 16 rows).
    const size_t x_limit = a.M <= 8 ? (size_t)host::env_int("QVB8_TILE_X_LDS_LIMIT", (int)kTileXLdsMost) : kTileXLdsLimit;
    bool fits = x_bytes <= x_limit && x_bytes + 64 + 8192 <= kLdsPerWorkgroup && host::env_int("QVB8_TILE_X_LDS", 1) != 0;
    size_t per_thread = 0;
    if (fits) {
        // the plan as the kernel with X in LDS will make it: its own LDS within what X leaves
        const size_t left = kLdsPerWorkgroup - (x_bytes + 64);
        fits = plan_tile(1, T, a.M, a.Q, a.P, pl, host::env_int("QVB8_TILE_WAVES12", 1) ? tile_max_waves<1, T, BF, PL>() : 8,
                         tile_pair_fits<1, T, BF, XC, 1, PL>(), x_bytes + 64, left < kTileLdsLimit ? left : kTileLdsLimit);
        per_thread = fits ? (x_bytes / 16 + pl.threads - 1) / pl.threads : 0;
    }
    if (fits && per_thread <= 1) return launch_tile<1, T, BF, XC, 1, PL>(a, s);
    if (fits && per_thread <= 4) return launch_tile<1, T, BF, XC, 4, PL>(a, s);
    if (fits && per_thread <= 8) return launch_tile<1, T, BF, XC, 8, PL>(a, s);
    if (fits && per_thread <= 16) return launch_tile<1, T, BF, XC, 16, PL>(a, s);
    return launch_tile<1, T, BF, XC, 0, PL>(a, s);
}

struct GemmPlan {
    int MT, tok_blocks, row_blocks, splits, stages_per_split;
    size_t lds;
    int64_t x16_at, sx_at, part_at, bytes;      // workspace layout, bytes from its start (after the row records' place)
};
int64_t align256i(int64_t n) { return (n + 255) & ~(int64_t)255; }

// Column ranges of whole 256-column groups, enough of them for about three workgroups per four CUs (row blocks counted as
// ceil(Q / 256): up to two more exist when the rows have several widths).
GemmPlan plan_gemm(int64_t M, int64_t Q, int64_t P) {
    GemmPlan g;
    // 64 rows of X per workgroup (two waves per SIMD) up to 192 rows; beyond, 128 rows per workgroup read the ids half as
    // often (measured at M = 256: 10 % faster although only one wave per SIMD fits)
    const int mt_env = host::env_int("QVB8_GEMM_MT", 0);
    g.MT = mt_env == 2 || mt_env == 4 ? mt_env : (M > 192 ? 4 : 2);
    if (M <= 64) g.MT = 2;
    if (M <= host::env_int("QVB8_GEMM_MT1_UPTO", 32)) g.MT = 1;           // one token tile of 32: half the matrix instructions per step
    const int TMK = 32 * g.MT;
    g.tok_blocks = (int)((M + TMK - 1) / TMK);
    g.row_blocks = (int)((Q + kGemmRows - 1) / kGemmRows);
    const int64_t groups = P / (2 * kGemmStageCols);
    const int64_t base = (int64_t)g.tok_blocks * g.row_blocks;
    // measured: three workgroups per four CUs is the best trade between idle CUs and partial-result traffic
    const int64_t target = host::env_int("QVB8_GEMM_TARGET_WGS", 0) > 0 ? host::env_int("QVB8_GEMM_TARGET_WGS", 0) : 3 * (int64_t)host::device_cus() / 4;
    int64_t splits = (target + base - 1) / base;
    if (splits > groups) splits = groups;
    if (splits > 16) splits = 16;
    if (splits < 1) splits = 1;
    const int64_t groups_per_split = (groups + splits - 1) / splits;
    g.stages_per_split = (int)(2 * groups_per_split);
    g.splits = (int)((groups + groups_per_split - 1) / groups_per_split);
    g.lds = (size_t)2 * TMK * kGemmXStride;
    g.x16_at = align256i(qvb8_mma_rowinfo_bytes(Q));
    g.sx_at = g.x16_at + align256i(M * P * 2);
    g.part_at = g.sx_at + align256i((int64_t)g.splits * M * 4);
    g.bytes = g.part_at + (g.splits > 1 ? (int64_t)g.splits * M * Q * 4 : 0);
    return g;
}

// The kernel that stages decoded weights in LDS: one block of rows of X (M <= 256), 128 weight rows per workgroup, column
// ranges for about one workgroup per CU (it holds most of a CU's LDS).
int gemm2_from() { const int v = host::env_int("QVB8_GEMM_LDS_FROM", 65); return v < 33 ? 33 : v; }
GemmPlan plan_gemm2(int64_t M, int64_t Q, int64_t P) {
    GemmPlan g;
    g.row_blocks = (int)((Q + kG2Rows - 1) / kG2Rows);
    // All of X in one block of 256 rows when the weight alone has row blocks for most of the chip; otherwise blocks of 128
    // rows of X: twice the workgroups before any column range is split off, and half the partial results to add up.
    const int mt_env = host::env_int("QVB8_GEMM_MT", 0);
    g.MT = mt_env == 2 || mt_env == 4 ? mt_env : ((M > 128 && 2 * g.row_blocks >= (int)host::device_cus()) ? 4 : 2);
    const int BM = 64 * g.MT;
    g.tok_blocks = (int)((M + BM - 1) / BM);
    const int64_t groups = P / (2 * kGemmStageCols);
    const int64_t base = (int64_t)g.row_blocks * g.tok_blocks;
    const int64_t target = host::env_int("QVB8_GEMM_TARGET_WGS", 0) > 0 ? host::env_int("QVB8_GEMM_TARGET_WGS", 0) : (int64_t)host::device_cus();
    int64_t splits = (target + base / 2) / base;
    if (splits > groups) splits = groups;
    if (splits > 16) splits = 16;
    if (splits < 1) splits = 1;
    const int64_t groups_per_split = (groups + splits - 1) / splits;
    g.stages_per_split = (int)(2 * groups_per_split);
    g.splits = (int)((groups + groups_per_split - 1) / groups_per_split);
    g.lds = (size_t)2 * BM * kG2AStride + (size_t)2 * kG2Rows * kG2BStride;
    g.x16_at = align256i(qvb8_mma_rowinfo_bytes(Q));
    g.sx_at = g.x16_at + align256i((int64_t)g.tok_blocks * BM * P * 2);    // X stage by stage, in blocks of BM rows
    g.part_at = g.sx_at + align256i((int64_t)g.splits * M * 4);
    g.bytes = g.part_at + (g.splits > 1 ? (int64_t)g.splits * M * Q * 4 : 0);
    return g;
}
GemmPlan plan_gemm_for(int64_t M, int64_t Q, int64_t P) { return M >= gemm2_from() ? plan_gemm2(M, Q, P) : plan_gemm(M, Q, P); }

// Fewest rows of X that go to the workgroup-tiled kernel when it can read the weight (49..: always; below that the tile
// kernel is the alternative).
// from 17 rows of X on the register-decode kernel (one token tile of 32 up to 32 rows) is the faster one (measured on the 9B
// projections, 8 layers: M = 17 0.641 ms against 0.721 for the tile kernel with two token tiles, M = 32 0.70 / 0.87)
int gemm_from() { const int v = host::env_int("QVB8_MMA_GEMM_FROM", 17); return v < 17 ? 17 : (v > 49 ? 49 : v); }

template <int MT, bool BF, bool XC, int RT>
int launch_gemm_as(const GemmArgs& a, const GemmPlan& g, int row_blocks, hipStream_t s) {
    static bool attr[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return host::fail(QVB8_ERR_LAUNCH, "qvb8_mma: no current device");
    if (!attr[dev]) {
        if (hipFuncSetAttribute((const void*)gemm_kernel<MT, BF, XC, RT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)g.lds) != hipSuccess)
            return host::fail(QVB8_ERR_LAUNCH, "qvb8_mma: cannot raise the kernel's LDS limit");
        attr[dev] = true;
    }
    hipLaunchKernelGGL((gemm_kernel<MT, BF, XC, RT>), dim3((unsigned)row_blocks, (unsigned)g.tok_blocks, (unsigned)g.splits),
                       dim3(64 * (kGemmRows / (32 * RT))), g.lds, s, a);
    return host::check_launch("qvb8_mma");
}
// eight waves with one row tile each (two waves per SIMD: one decodes while the other's products run) or four with two
template <int MT, bool BF, bool XC>
int launch_gemm(const GemmArgs& a, const GemmPlan& g, int row_blocks, hipStream_t s) {
    if (host::env_int("QVB8_GEMM_WAVES", 8) == 8 && MT <= 2) return launch_gemm_as<MT, BF, XC, 1>(a, g, row_blocks, s);
    return launch_gemm_as<MT, BF, XC, 2>(a, g, row_blocks, s);
}

template <int WM, bool BF>
int launch_gemm2(const GemmArgs& a, const GemmPlan& g, int row_blocks, hipStream_t s) {
    static bool attr[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return host::fail(QVB8_ERR_LAUNCH, "qvb8_mma: no current device");
    if (!attr[dev]) {
        if (hipFuncSetAttribute((const void*)gemm2_kernel<WM, BF>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)g.lds) != hipSuccess)
            return host::fail(QVB8_ERR_LAUNCH, "qvb8_mma: cannot raise the kernel's LDS limit");
        attr[dev] = true;
    }
    hipLaunchKernelGGL((gemm2_kernel<WM, BF>), dim3((unsigned)row_blocks, (unsigned)g.tok_blocks, (unsigned)g.splits), dim3(64 * kG2Waves), g.lds, s, a);
    return host::check_launch("qvb8_mma");
}
}  // namespace

// A kernel of the tile kernel's launch shape (grid, workgroup size, dynamic LDS, 56 bytes of scalar arguments) that does
// nothing: what a launch costs before it moves a byte.
__global__ void __launch_bounds__(512) launch_probe_kernel(const uint16_t* X, const uint8_t* ids, const uint64_t* loc, float* Y, int64_t ids_bytes,
                                                           int Q, int P, uint32_t counts, int TW, int first1, int first2, uint32_t widths) {
    extern __shared__ __align__(16) unsigned char smem[];
    if (Q < 0) Y[threadIdx.x] = (float)(smem[threadIdx.x] + X[0] + ids[0] + loc[0] + ids_bytes + P + counts + TW + first1 + first2 + widths);
}

extern "C" int qvb8_launch_probe(int64_t blocks, int64_t threads, int64_t lds_bytes, void* stream) {
    if (blocks < 1 || blocks > 65535 || threads < 64 || threads > 512 || (threads & 63) || lds_bytes < 0 || lds_bytes > (int64_t)kLdsPerWorkgroup)
        return host::fail(QVB8_ERR_ARG, "qvb8_launch_probe: 1..65535 workgroups of 64..512 threads (whole waves), at most 160 KB of LDS");
    static bool attr[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return host::fail(QVB8_ERR_LAUNCH, "qvb8_launch_probe: no current device");
    if (!attr[dev]) {
        if (hipFuncSetAttribute((const void*)launch_probe_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsPerWorkgroup) != hipSuccess)
            return host::fail(QVB8_ERR_LAUNCH, "qvb8_launch_probe: cannot raise the kernel's LDS limit");
        attr[dev] = true;
    }
    hipLaunchKernelGGL(launch_probe_kernel, dim3((unsigned)blocks), dim3((unsigned)threads), (size_t)lds_bytes, (hipStream_t)stream,
                       nullptr, nullptr, nullptr, nullptr, (int64_t)0, 1, 1, 0u, 1, 1, 1, 0u);
    return host::check_launch("qvb8_launch_probe");
}

extern "C" int64_t qvb8_mma_rowinfo_bytes(int64_t Q) { return Q > 0 ? (int64_t)(rowinfo_loc_words(Q) * 8 + (size_t)Q * 16) : 0; }

extern "C" int qvb8_mma_prepare(const uint8_t* nbits, const int64_t* bit_off, const float* tau_s, const float* min_s,
                                const int32_t* perm, int64_t Q, int64_t P, int64_t ids_bytes, uint64_t* rowinfo, void* stream) {
    if (Q < 0 || P < 0 || Q > 0x7fffffff || P > 0x7fffffff) return host::fail(QVB8_ERR_ARG, "qvb8_mma_prepare: Q or P out of range");
    if (Q == 0) return QVB8_OK;
    if (!nbits || !bit_off || !tau_s || !min_s || !rowinfo) return host::fail(QVB8_ERR_ARG, "qvb8_mma_prepare: null pointer");
    hipLaunchKernelGGL(rowinfo_kernel, dim3((unsigned)((Q + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       nbits, bit_off, tau_s, min_s, perm, (int)Q, (int)P, ids_bytes, rowinfo,
                       reinterpret_cast<uint4*>(rowinfo + rowinfo_loc_words(Q)));
    return host::check_launch("qvb8_mma_prepare");
}

extern "C" int64_t qvb8_mma_workspace_bytes(int64_t M, int64_t Q, int64_t P) {
    if (M >= gemm_from() && M <= 256 && Q > 0 && P > 0 && (P % (2 * kGemmStageCols)) == 0) return plan_gemm_for(M, Q, P).bytes;
    return qvb8_mma_rowinfo_bytes(Q);
}

extern "C" int qvb8_mma(const void* X, int x_dtype, int64_t M,
                        const uint8_t* ids, int64_t ids_bytes, const float* min_s, const float* tau_s,
                        const uint8_t* nbits, const int64_t* bit_off, int64_t Q, int64_t P,
                        const int64_t* esc_idx, const float* esc_vals, int64_t n_esc,
                        const int32_t* perm, const uint64_t* rowinfo, const qvb8_mma_layout* layout, int flags, float* Y,
                        void* workspace, int64_t workspace_bytes, void* stream) {
    if (Q < 0 || P < 0 || Q > 0x7fffffff || P > 0x7fffffff) return host::fail(QVB8_ERR_ARG, "qvb8_mma: Q or P out of range");
    if (M < 1 || M > 256) return host::fail(QVB8_ERR_ARG, "qvb8 mma-multi: M=%lld outside 1..256", (long long)M);
    if (x_dtype != QVB8_F16 && x_dtype != QVB8_BF16) return host::fail(QVB8_ERR_ARG, "qvb8_mma: X must be fp16 or bf16 (narrow fp32 activations with qvb8_sat_half first)");
    if ((P % kStepCols) != 0 || (reinterpret_cast<uintptr_t>(ids) & 3u) != 0)
        return host::fail(QVB8_ERR_ARG, "qvb8 mma-multi: needs P%%128==0 and 4-byte-aligned ids");
    if (ids_bytes < 32) return host::fail(QVB8_ERR_ARG, "qvb8_mma: ids buffer shorter than 32 bytes");
    if (n_esc < 0 || (n_esc > 0 && (!esc_idx || !esc_vals))) return host::fail(QVB8_ERR_ARG, "qvb8_mma: bad escape list");
    if (Q == 0) return QVB8_OK;
    if (!X || !Y || !ids || !min_s || !tau_s || !nbits || !bit_off) return host::fail(QVB8_ERR_ARG, "qvb8_mma: null pointer");
    if (reinterpret_cast<uintptr_t>(X) & 15u) return host::fail(QVB8_ERR_ARG, "qvb8_mma: X must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    if (!rowinfo) {
        if (!workspace || workspace_bytes < qvb8_mma_rowinfo_bytes(Q))
            return host::fail(QVB8_ERR_WORKSPACE, "qvb8_mma: without row records the call needs %lld bytes of workspace", (long long)qvb8_mma_rowinfo_bytes(Q));
        if (int rc = qvb8_mma_prepare(nbits, bit_off, tau_s, min_s, perm, Q, P, ids_bytes, (uint64_t*)workspace, stream)) return rc;
        rowinfo = (const uint64_t*)workspace;
    }
    TileArgs a;
    a.X = (const uint16_t*)X; a.ids = ids; a.loc = rowinfo; a.fin = reinterpret_cast<const uint4*>(rowinfo + rowinfo_loc_words(Q));
    a.n_classes = 0; a.first1 = a.first2 = (int)Q; a.nb[0] = a.nb[1] = a.nb[2] = 0; a.planes = 0;
    if (layout) {
        if (!rowinfo) return host::fail(QVB8_ERR_ARG, "qvb8_mma: a row layout goes with the row records of the same order");
        const int n = layout->n_classes;
        if (n < 1 || n > QVB8_MMA_MAX_CLASSES || layout->first_pos[0] != 0 || layout->first_pos[n] != Q)
            return host::fail(QVB8_ERR_ARG, "qvb8_mma: bad row layout (1..3 classes that cover positions 0..Q)");
        int64_t bits = 0;
        for (int c = 0; c < n; ++c) {
            const int64_t rows = (int64_t)layout->first_pos[c + 1] - layout->first_pos[c], nbc = layout->nbits[c];
            if (rows < 0 || nbc < 1 || nbc > 14) return host::fail(QVB8_ERR_ARG, "qvb8_mma: bad row layout class %d", c);
            bits += rows * P * nbc;
            a.nb[c] = (int)nbc;
        }
        if ((bits >> 3) + 8 > ids_bytes) return host::fail(QVB8_ERR_ARG, "qvb8_mma: the row layout does not fit the ids buffer");
        a.first1 = n > 1 ? layout->first_pos[1] : (int)Q;
        a.first2 = n > 2 ? layout->first_pos[2] : (int)Q;
        a.n_classes = n;
    }
    const int out_dt = (flags & QVB8_MMA_Y_F16) ? 1 : (flags & QVB8_MMA_Y_BF16) ? 2 : 0;
    a.planes = (flags & QVB8_MMA_PLANES) ? 1 : 0;
    if (out_dt != 0 && n_esc > 0) return host::fail(QVB8_ERR_ARG, "qvb8_mma: fp16 / bf16 results need a weight without escapes (the correction adds to fp32 results)");
    a.Y = Y; a.out_dt = out_dt; a.ids_bytes = ids_bytes; a.M = (int)M; a.Q = (int)Q; a.P = (int)P; a.n_steps = (int)(P / kStepCols);
    // mode 0: fp16 X, fp16 operands; 1: bf16 X narrowed to saturated fp16 on the way in, fp16 operands; 2: bf16 operands
    const int mode = x_dtype == QVB8_F16 ? 0 : (flags & QVB8_MMA_SATURATE_X) ? 1 : 2;
    int rc;
    // Many rows of X: the workgroup-tiled kernel.  It addresses rows arithmetically and decodes whole slices only; from 17
    // rows on it is also the faster one (the tile kernel then keeps too few bytes in flight), so it is taken whenever it
    // can read the weight and the caller brought its workspace.
    bool tiled = M > 48;
    if (!tiled && M >= gemm_from() && layout && (P % (2 * kGemmStageCols)) == 0 && workspace
        && workspace_bytes >= plan_gemm_for(M, Q, P).bytes && (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0) {
        tiled = true;
        for (int c = 0; c < a.n_classes; ++c) tiled = tiled && a.nb[c] >= 4 && a.nb[c] <= (mode == 2 ? 7 : 8);
    }
    if (tiled) {
        if (!layout) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mma: M > 48 needs rows stored in width order (a row layout)");
        if ((P % (2 * kGemmStageCols)) != 0) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mma: M > 48 needs P %% 256 == 0");
        for (int c = 0; c < a.n_classes; ++c)
            if (a.nb[c] < 4 || a.nb[c] > (mode == 2 ? 7 : 8))
                return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_mma: M > 48 needs widths 4..8 (4..7 on bf16 operands), found %d", a.nb[c]);
        const bool staged = M >= gemm2_from();
        const GemmPlan g = plan_gemm_for(M, Q, P);
        if (!workspace || workspace_bytes < g.bytes || (reinterpret_cast<uintptr_t>(workspace) & 15u))
            return host::fail(QVB8_ERR_WORKSPACE, "qvb8_mma: M=%lld needs %lld bytes of 16-byte aligned workspace", (long long)M, (long long)g.bytes);
        unsigned char* ws = reinterpret_cast<unsigned char*>(workspace);
        uint16_t* x16 = reinterpret_cast<uint16_t*>(ws + g.x16_at);
        float* sx = reinterpret_cast<float*>(ws + g.sx_at);
        float* out = g.splits > 1 ? reinterpret_cast<float*>(ws + g.part_at) : Y;
        const int cols_per_split = g.stages_per_split * kGemmStageCols;
        const dim3 pgrid((unsigned)M, (unsigned)g.splits);
        const int tile_rows = staged ? 64 * g.MT : 0;                 // the staged kernel reads X stage by stage
        // the activation pass (narrowed copy stored stage by stage, sums per column range) is for the staged kernel only: the
        // register-decode kernel narrows what it stages and adds the rows of X up on the matrix cores itself
        if (staged) {
            if (mode == 0) hipLaunchKernelGGL((gemm_prep_kernel<false, false>), pgrid, dim3(256), 0, s, a.X, (int)M, (int)P, cols_per_split, x16, sx, tile_rows);
            else if (mode == 1) hipLaunchKernelGGL((gemm_prep_kernel<false, true>), pgrid, dim3(256), 0, s, a.X, (int)M, (int)P, cols_per_split, x16, sx, tile_rows);
            else hipLaunchKernelGGL((gemm_prep_kernel<true, false>), pgrid, dim3(256), 0, s, a.X, (int)M, (int)P, cols_per_split, x16, sx, tile_rows);
            if (int rc2 = host::check_launch("qvb8_mma activations")) return rc2;
        }
        GemmArgs ga;
        ga.X = staged ? x16 : a.X; ga.ids = ids; ga.fin = a.fin; ga.sx = staged ? sx : nullptr; ga.out = out;
        ga.M = (int)M; ga.Q = (int)Q; ga.P = (int)P; ga.stages_per_split = g.stages_per_split;
        ga.out_dt = g.splits > 1 ? 0 : out_dt;
        ga.planes = a.planes;
        ga.first1 = a.first1; ga.first2 = a.first2;
        const int rows0 = a.first1, rows1 = a.first2 - a.first1, rows2 = (int)Q - a.first2;
        const int br = staged ? kG2Rows : kGemmRows;                  // weight rows per workgroup
        ga.blocks1 = (rows0 + br - 1) / br;
        ga.blocks2 = ga.blocks1 + (rows1 + br - 1) / br;
        const int row_blocks = ga.blocks2 + (rows2 + br - 1) / br;
        ga.widths = (uint32_t)a.nb[0] | ((uint32_t)a.nb[1] << 8) | ((uint32_t)a.nb[2] << 16);
        if (staged) {
            if (g.MT == 4) rc = mode == 2 ? launch_gemm2<4, true>(ga, g, row_blocks, s) : launch_gemm2<4, false>(ga, g, row_blocks, s);
            else rc = mode == 2 ? launch_gemm2<2, true>(ga, g, row_blocks, s) : launch_gemm2<2, false>(ga, g, row_blocks, s);
        } else if (g.MT == 1) rc = mode == 2 ? launch_gemm<1, true, false>(ga, g, row_blocks, s) : mode == 1 ? launch_gemm<1, false, true>(ga, g, row_blocks, s) : launch_gemm<1, false, false>(ga, g, row_blocks, s);
        else if (g.MT == 4) rc = mode == 2 ? launch_gemm<4, true, false>(ga, g, row_blocks, s) : mode == 1 ? launch_gemm<4, false, true>(ga, g, row_blocks, s) : launch_gemm<4, false, false>(ga, g, row_blocks, s);
        else rc = mode == 2 ? launch_gemm<2, true, false>(ga, g, row_blocks, s) : mode == 1 ? launch_gemm<2, false, true>(ga, g, row_blocks, s) : launch_gemm<2, false, false>(ga, g, row_blocks, s);
        if (rc) return rc;
        if (g.splits > 1) {
            const int64_t n = M * Q;
            hipLaunchKernelGGL(gemm_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, out, Y, n, g.splits, out_dt);
            if (int rc2 = host::check_launch("qvb8_mma reduce")) return rc2;
        }
    } else {
#define QVB8_TILE_LAUNCH_P(NT_, T_, PL_) (mode == 0 ? launch_tile<NT_, T_, false, false, 0, PL_>(a, s) : mode == 1 ? launch_tile<NT_, T_, false, true, 0, PL_>(a, s) : launch_tile<NT_, T_, true, false, 0, PL_>(a, s))
#define QVB8_TILE_LAUNCH(NT_, T_) (a.planes ? QVB8_TILE_LAUNCH_P(NT_, T_, true) : QVB8_TILE_LAUNCH_P(NT_, T_, false))
    // rows of 33..40 steps (P = 5120): one panel of eight waves with five steps each instead of two panels of five waves
    // with four (measured on 27B-class shapes: 16 % faster; more steps per wave did not pay for longer rows)
    const int n_steps_all = (int)(P / kStepCols);
#define QVB8_TILE_LAUNCH_ROWS16_P(T_, PL_) (mode == 0 ? launch_tile_rows16<T_, false, false, PL_>(a, s) : mode == 1 ? launch_tile_rows16<T_, false, true, PL_>(a, s) : launch_tile_rows16<T_, true, false, PL_>(a, s))
#define QVB8_TILE_LAUNCH_ROWS16(T_) (a.planes ? QVB8_TILE_LAUNCH_ROWS16_P(T_, true) : QVB8_TILE_LAUNCH_ROWS16_P(T_, false))
        // (with twelve waves four steps each cover up to 48 steps in one panel: QVB8_TILE_T5=0 tries that instead)
        const bool five = n_steps_all > 32 && n_steps_all <= 40 && !(a.planes && mode != 2 && host::env_int("QVB8_TILE_T5", 1) == 0);
        // (eleven waves of three steps for 4096-column rows were measured as well: no difference)
        if (M <= 16) rc = five ? QVB8_TILE_LAUNCH_ROWS16(5) : QVB8_TILE_LAUNCH_ROWS16(4);
#undef QVB8_TILE_LAUNCH_ROWS16
#undef QVB8_TILE_LAUNCH_ROWS16_P
    else if (M <= 32) rc = QVB8_TILE_LAUNCH(2, 2);
    else rc = QVB8_TILE_LAUNCH(3, 2);
#undef QVB8_TILE_LAUNCH
#undef QVB8_TILE_LAUNCH_P
        if (rc) return rc;
    }
    if (n_esc > 0) {
        dim3 grid((unsigned)((n_esc + 255) / 256), (unsigned)M);
#define QVB8_FIX_ARGS grid, dim3(256), 0, s, (const uint16_t*)X, (int)M, ids, ids_bytes, min_s, tau_s, nbits, bit_off, esc_idx, esc_vals, n_esc, Y, (int)Q, (int)P
        if (mode == 0) hipLaunchKernelGGL((tile_fix_escapes_kernel<false, false>), QVB8_FIX_ARGS);
        else if (mode == 1) hipLaunchKernelGGL((tile_fix_escapes_kernel<false, true>), QVB8_FIX_ARGS);
        else hipLaunchKernelGGL((tile_fix_escapes_kernel<true, false>), QVB8_FIX_ARGS);
#undef QVB8_FIX_ARGS
        return host::check_launch("qvb8_mma escapes");
    }
    return QVB8_OK;
}
