// Routed MoE expert stack on packed QVB8 experts (decode: a few tokens, top-k experts each), gfx950.
//
//   pair p = (token t, j-th choice), expert e = idx[t][j]
//   gated (act 0):   Y = W_gu[e] . x_t ;  H[p][i] = silu(Y[i]) * Y[I + i]      (gate = first half of the rows)
//   relu2 (act 1):   Y = W_up[e] . x_t ;  H[p][i] = max(Y[i], 0)^2
//   Yd[p] = W_dn[e] . H[p] ;  out[t] = sum_j w[t][j] * Yd[t * k + j]           (j ascending, fused multiply-add)
//
// Three steps on the caller's stream: a one-workgroup routing plan (pairs grouped by expert, no host round trip), the
// up projection with the activation fused into its epilogue, the down projection, and the weighted combine.  The
// grouped products run over the experts that were actually selected, and an expert chosen by several tokens is read
// ONCE for all of them (up to 8 pairs share every decoded id): the bytes touched are those of the unique experts.
//
// Arithmetic: x is narrowed like saturating_half and widened again (what the reference multiplies), H stays fp32.
// A row's product is  tau_s * sum(x * id) + min_s * sum(x)  with fp32 fused multiply-adds per lane, a fixed-order wave
// sum, and the two terms joined in double: reproducible, and within rounding of  sum(x * fmaf(id, tau_s, min_s)).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <algorithm>
#include <mutex>
#include <type_traits>

#include "../../include/qvb8_amd.h"
#include "qvb8_device.h"
#include "qvb8_host.h"
#include "qvb8_mma_device.h"

namespace qvb8 {

constexpr int kMoeMB = 8;              // pairs that share one pass over an expert's rows
constexpr int kMoeThreads = 256;

// Workspace layout (bytes from the start): plan | H | Yd
//   plan: i32 n_bad, i32 slots in use (+2 pad), int4 slot[n_slots] = {expert, first pair, end pair, 0} for the experts that have pairs
//   (end == first for unused slots), i32 order[npairs] (pair numbers grouped by expert)
struct MoePlan {
    int32_t* n_bad; int4* slot; int32_t* order;
};
__host__ __device__ inline int64_t moe_slots(int64_t E, int64_t npairs) { return E < npairs ? E : npairs; }
__host__ __device__ inline size_t moe_plan_bytes(int64_t E, int64_t npairs) {
    return (size_t)(16 + moe_slots(E, npairs) * 16 + npairs * 4 + 255) & ~(size_t)255;
}
__host__ __device__ inline MoePlan moe_plan_at(void* ws, int64_t E, int64_t npairs) {
    unsigned char* p = reinterpret_cast<unsigned char*>(ws);
    return MoePlan{reinterpret_cast<int32_t*>(p), reinterpret_cast<int4*>(p + 16),
                   reinterpret_cast<int32_t*>(p + 16 + moe_slots(E, npairs) * 16)};
}

// One workgroup: pairs grouped by expert (counting sort), table of the experts that have pairs.  The two running
// sums over the experts (pairs before expert e, selected experts before e) are a workgroup scan, 256 experts per round.
// `cap`: the most pairs one expert may have for the path that follows (the grouped walk takes an expert's pairs as the token
// rows of ONE operand: at most one per token); an expert with more counts as a bad entry, so the results come out as NaN
// instead of sums with pairs missing.
__global__ void __launch_bounds__(kMoeThreads) moe_plan_kernel(const int64_t* __restrict__ idx, int npairs, int E, MoePlan pl, int cap) {
    extern __shared__ int32_t s_cnt[];                        // [E] counts, then cursors; [E .. E + 8) scan scratch
    int32_t* s_scan = s_cnt + E;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int e = tid; e < E; e += blockDim.x) s_cnt[e] = 0;
    if (tid == 0) *pl.n_bad = 0;
    __syncthreads();
    int bad = 0;
    for (int p = tid; p < npairs; p += blockDim.x) {
        const int64_t e = idx[p];
        if (e >= 0 && e < E) atomicAdd(&s_cnt[(int)e], 1); else ++bad;
    }
    if (bad) atomicAdd(pl.n_bad, bad);
    __syncthreads();
    const int n_slots = E < npairs ? E : npairs;
    int run_pairs = 0, run_active = 0;                        // totals of the rounds before this one (same in every thread)
    for (int e0 = 0; e0 < E; e0 += blockDim.x) {
        const int e = e0 + tid;
        const int c = e < E ? s_cnt[e] : 0;
        if (c > cap) atomicAdd(pl.n_bad, 1);
        // inclusive scan of (c, c > 0) packed as pairs * 2^16 + active: both stay below 2^15 per round... pairs can be
        // larger, so scan them separately
        int sc = c, sa = c > 0 ? 1 : 0;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int tc = __shfl_up(sc, o, 64), ta = __shfl_up(sa, o, 64);
            if (lane >= o) { sc += tc; sa += ta; }
        }
        if (lane == 63) { s_scan[wave] = sc; s_scan[4 + wave] = sa; }
        __syncthreads();
        int base_c = run_pairs, base_a = run_active, tot_c = 0, tot_a = 0;
        for (int w = 0; w < (int)(blockDim.x >> 6); ++w) {
            if (w < wave) { base_c += s_scan[w]; base_a += s_scan[4 + w]; }
            tot_c += s_scan[w]; tot_a += s_scan[4 + w];
        }
        const int first = base_c + sc - c;                    // pairs before expert e
        if (e < E) {
            if (c > 0) pl.slot[base_a + sa - 1] = int4{e, first, first + c, 0};
            s_cnt[e] = first;                                 // becomes the expert's cursor
        }
        run_pairs += tot_c; run_active += tot_a;
        __syncthreads();
    }
    for (int i = run_active + tid; i < n_slots; i += blockDim.x) pl.slot[i] = int4{0, 0, 0, 0};
    if (tid == 0) pl.n_bad[1] = run_active;                   // slots in use
    __syncthreads();
    for (int p = tid; p < npairs; p += blockDim.x) {
        const int64_t e = idx[p];
        if (e >= 0 && e < E) pl.order[atomicAdd(&s_cnt[(int)e], 1)] = p;
    }
}

struct MoeGemvArgs {
    const void* X;                 // stage 0: (tokens, P) activations in x_dtype; stage 1: H (npairs, P) f32
    const uint8_t* ids; int64_t ids_bytes;
    const float* min_s; const float* tau_s; const uint8_t* nbits; const int64_t* bit_off;   // (E, Q) each
    float* out;                    // stage 0: H (npairs, n_units); stage 1: Yd (npairs, Q)
    MoePlan plan;
    int Q, P, topk, x_dtype, act;  // act: 0 gated silu, 1 relu2 (stage 0 only)
    int units;                     // output columns per pair: stage 0 gated Q/2, relu2 Q; stage 1 Q
    int units_per_block;
    int x_rows;                    // activation rows a workgroup stages at a time: min(kMoeMB, tokens)
};

template <int NB, int J>
__device__ __forceinline__ void moe_fields(const uint32_t (&w)[kMaxFastNb], float (&idf)[32]) {
    if constexpr (J < 32) { idf[J] = (float)field_of<NB, J>(w); moe_fields<NB, J + 1>(w, idf); }
}

// acc[mb] += x[mb][c0 + j] * id_j over the lane's 32 consecutive ids, given as the first and the last four dwords of
// its NB-dword slice
template <int NB, typename XT>
__device__ __forceinline__ void moe_chunk(const uint4& lo, const uint4& hi, const XT* __restrict__ xs, int P, int c0, int n,
                                          float (&acc)[kMoeMB]) {
    uint32_t w[kMaxFastNb];
    const uint32_t l[4] = {lo.x, lo.y, lo.z, lo.w}, h[4] = {hi.x, hi.y, hi.z, hi.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) w[k] = l[k];
#pragma unroll
    for (int k = 4; k < NB; ++k) w[k] = h[k - (NB - 4)];
    float idf[32];
    moe_fields<NB, 0>(w, idf);
#pragma unroll
    for (int mb = 0; mb < kMoeMB; ++mb) {
        if (mb >= n) break;                                             // wave-uniform
        float a = acc[mb];
        if constexpr (sizeof(XT) == 4) {
            const float4* xp = reinterpret_cast<const float4*>(xs + (size_t)mb * P + c0);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const float4 xv = xp[k];
                a = __builtin_fmaf(xv.x, idf[4 * k + 0], a);
                a = __builtin_fmaf(xv.y, idf[4 * k + 1], a);
                a = __builtin_fmaf(xv.z, idf[4 * k + 2], a);
                a = __builtin_fmaf(xv.w, idf[4 * k + 3], a);
            }
        } else {
            typedef _Float16 v8h __attribute__((ext_vector_type(8)));
            const v8h* xp = reinterpret_cast<const v8h*>(xs + (size_t)mb * P + c0);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const v8h xv = xp[k];
#pragma unroll
                for (int j = 0; j < 8; ++j) a = __builtin_fmaf((float)xv[j], idf[8 * k + j], a);
            }
        }
        acc[mb] = a;
    }
}

template <typename XT>
__device__ __forceinline__ void moe_chunk_any(int nb, const uint4& lo, const uint4& hi, const XT* xs, int P, int c0, int n,
                                              float (&acc)[kMoeMB]) {
    switch (nb) {
        case 4: moe_chunk<4>(lo, hi, xs, P, c0, n, acc); break;
        case 5: moe_chunk<5>(lo, hi, xs, P, c0, n, acc); break;
        case 6: moe_chunk<6>(lo, hi, xs, P, c0, n, acc); break;
        case 7: moe_chunk<7>(lo, hi, xs, P, c0, n, acc); break;
        default: moe_chunk<8>(lo, hi, xs, P, c0, n, acc); break;
    }
}

// Row record a workgroup keeps in LDS for each of its rows: flags = width | ok << 8 | fast << 9
struct MoeRow { int64_t bit0; float ts, mn; int flags; int pad; };

// STAGE 0: up projection + activation -> H.  STAGE 1: down projection -> Yd.
// grid = (unit blocks, expert slots); a workgroup serves `units_per_block` output units of one selected expert for
// all pairs routed to it, kMoeMB pairs at a time, with those pairs' activation rows staged in LDS as fp32.  A wave
// walks through its rows with the next row's ids already requested while it multiplies the current one.
template <int STAGE>
__global__ void __launch_bounds__(kMoeThreads) moe_gemv_kernel(MoeGemvArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int rpu = (STAGE == 0 && a.act == 0) ? 2 : 1;             // rows per output unit (gate and up)
    // stage 0 multiplies activations that were narrowed to fp16: they are kept as fp16 (half the LDS and LDS traffic)
    using XT = std::conditional_t<STAGE == 0, _Float16, float>;
    XT* xs = reinterpret_cast<XT*>(smem);                           // [x_rows][P]
    float* sxs = reinterpret_cast<float*>(smem + (((size_t)a.x_rows * a.P * sizeof(XT) + 15) & ~(size_t)15));   // [kMoeMB] sums of the staged rows
    float* red = sxs + kMoeMB;                                      // [kMoeMB][waves]
    MoeRow* s_row = reinterpret_cast<MoeRow*>(red + kMoeMB * (kMoeThreads / 64));   // [units_per_block * rpu]
    const int4 slot = a.plan.slot[blockIdx.y];
    const int e = slot.x, p_begin = slot.y, p_end = slot.z;
    if (p_begin >= p_end) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n_waves = blockDim.x >> 6;
    const int u_begin = blockIdx.x * a.units_per_block, u_end = min(a.units, u_begin + a.units_per_block);
    const int gate_rows = a.Q / 2;
    const int n_rows_blk = (u_end - u_begin) * rpu;
    // local row lr -> row of the expert: unit u_begin + lr / rpu; in gated mode the even local rows are gate rows (u),
    // the odd ones the matching up rows (Q/2 + u)
    for (int lr = tid; lr < n_rows_blk; lr += blockDim.x) {
        const int u = u_begin + lr / rpu;
        const size_t mi = (size_t)e * a.Q + ((rpu == 2 && (lr & 1)) ? gate_rows + u : u);
        const int nb = a.nbits[mi];
        const int64_t bit0 = a.bit_off[mi];
        const bool ok = nb >= 1 && nb <= 14 && bit0 >= 0 && ((bit0 + (int64_t)nb * a.P + 7) >> 3) + 8 <= a.ids_bytes;
        const bool fast = ok && nb >= 4 && nb <= 8 && (bit0 & 31) == 0;
        s_row[lr] = MoeRow{ok ? bit0 : 0, a.tau_s[mi], a.min_s[mi], nb | (ok ? 256 : 0) | (fast ? 512 : 0), 0};
    }
    const int64_t clamp_byte = (a.ids_bytes - 8) & ~(int64_t)3;
    const int n_items = ((u_end - u_begin - wave + n_waves - 1) / n_waves) * rpu;   // rows this wave walks through
    auto local_row = [&](int i) { return ((wave + (i / rpu) * n_waves) * rpu) + (i % rpu); };
    // the lane's slice of the first 2048 columns of a row (fast rows; other lanes / rows read the buffer's first bytes)
    auto request = [&](const MoeRow& r, uint4& lo, uint4& hi) {
        const int nb = r.flags & 255;
        const bool use = (r.flags & 512) && lane * 32 < a.P;
        const uint8_t* p = a.ids + (use ? (r.bit0 >> 3) + (int64_t)lane * 4 * nb : 0);
        lo = *reinterpret_cast<const uint4*>(p);
        hi = *reinterpret_cast<const uint4*>(p + (use ? 4 * (nb - 4) : 16));
    };

    for (int pc = p_begin; pc < p_end; pc += a.x_rows) {
        const int n = min(a.x_rows, p_end - pc);                    // x_rows <= kMoeMB
        __syncthreads();                                            // the previous chunk's rows are no longer read; s_row is written
        uint4 lo, hi;
        MoeRow cur;
        if (n_items > 0) { cur = s_row[local_row(0)]; request(cur, lo, hi); }
        // ---- stage the chunk's activation rows and their sums ----
        for (int mb = 0; mb < n; ++mb) {
            const int p = a.plan.order[pc + mb];
            float part = 0.f;
            for (int c = tid; c < a.P; c += blockDim.x) {
                float v;
                if constexpr (STAGE == 0) {
                    const uint32_t hb = sat_half_bits(load_as_f32(a.X, (int64_t)(p / a.topk) * a.P + c, a.x_dtype));
                    v = f16_bits_to_f32(hb);
                    xs[(size_t)mb * a.P + c] = __builtin_bit_cast(XT, (uint16_t)hb);
                } else {
                    v = reinterpret_cast<const float*>(a.X)[(size_t)p * a.P + c];
                    xs[(size_t)mb * a.P + c] = v;
                }
                part += v;
            }
            part = wave_sum(part);
            if (lane == 0) red[mb * n_waves + wave] = part;
        }
        __syncthreads();
        if (tid < n) {
            float s = 0.f;
            for (int w = 0; w < n_waves; ++w) s += red[tid * n_waves + w];
            sxs[tid] = s;
        }
        __syncthreads();
        // ---- rows: the next row's slice is requested before the current one is multiplied ----
        float y_gate[kMoeMB];
#pragma unroll
        for (int mb = 0; mb < kMoeMB; ++mb) y_gate[mb] = 0.f;
        for (int i = 0; i < n_items; ++i) {
            uint4 lo_n = lo, hi_n = hi;
            MoeRow nxt = cur;
            if (i + 1 < n_items) { nxt = s_row[local_row(i + 1)]; request(nxt, lo_n, hi_n); }
            const int nb = cur.flags & 255;
            float acc[kMoeMB];
#pragma unroll
            for (int mb = 0; mb < kMoeMB; ++mb) acc[mb] = 0.f;
            if (cur.flags & 512) {
                if (lane * 32 < a.P) moe_chunk_any(nb, lo, hi, xs, a.P, lane * 32, n, acc);
                for (int c0 = (kWave + lane) * 32; c0 < a.P; c0 += kWave * 32) {          // rows longer than 2048 columns
                    const uint8_t* p = a.ids + (cur.bit0 >> 3) + (int64_t)(c0 >> 5) * 4 * nb;
                    moe_chunk_any(nb, *reinterpret_cast<const uint4*>(p), *reinterpret_cast<const uint4*>(p + 4 * (nb - 4)), xs, a.P, c0, n, acc);
                }
            } else if (cur.flags & 256) {
                for (int c = lane; c < a.P; c += kWave) {
                    const float idf = (float)load_field(a.ids, cur.bit0 + (int64_t)c * nb, nb, clamp_byte);
#pragma unroll
                    for (int mb = 0; mb < kMoeMB; ++mb)
                        if (mb < n) acc[mb] = __builtin_fmaf((float)xs[(size_t)mb * a.P + c], idf, acc[mb]);
                }
            }
            float y[kMoeMB];
#pragma unroll
            for (int mb = 0; mb < kMoeMB; ++mb) {
                y[mb] = 0.f;
                if (mb < n) {                                                            // wave-uniform
                    const float sum = wave_sum(acc[mb]);
                    y[mb] = (cur.flags & 256) ? (float)((double)cur.ts * (double)sum + (double)cur.mn * (double)sxs[mb]) : __builtin_nanf("");
                }
            }
            const bool unit_done = (i % rpu) == rpu - 1;
            if (unit_done) {
                const int u = u_begin + wave + (i / rpu) * n_waves;
                if (lane < n) {
                    float v = 0.f;
#pragma unroll
                    for (int mb = 0; mb < kMoeMB; ++mb) {           // lane mb takes result mb (no dynamic register index)
                        if (lane == mb) {
                            if constexpr (STAGE == 0) {
                                if (a.act == 0) v = (y_gate[mb] / (1.0f + __expf(-y_gate[mb]))) * y[mb];
                                else { const float r = fmaxf(y[mb], 0.f); v = r * r; }
                            } else {
                                v = y[mb];
                            }
                        }
                    }
                    a.out[(size_t)a.plan.order[pc + lane] * a.units + u] = v;
                }
            } else {
#pragma unroll
                for (int mb = 0; mb < kMoeMB; ++mb) y_gate[mb] = y[mb];
            }
            cur = nxt; lo = lo_n; hi = hi_n;
        }
    }
}

// ---- one token: both projections on the matrix cores ------------------------------------------------------------------
// With a single token every selected expert has exactly one pair, and nothing needs a routing plan: slot j is expert
// idx[j].  Two launches instead of four.  Both use the tile scheme of the dense kernels: a row tile is 16 rows of one
// expert, a wave owns T steps of 128 columns of it (W = ceil(steps / T) waves per tile, G = 8 / W tiles at a time),
// requests its activations and its ids in one burst (no request under a branch), decodes the ids into MFMA operands
// (ids exact in fp16 next to a bias of 1024, the token in row 0 of the other operand) and leaves its partial sums in LDS.
//   up:   a workgroup takes `tiles_per_wg` unit tiles (16 outputs of one slot; gated: the 16 gate rows and the 16
//         matching up rows, so the activation is applied here) and writes H as fp16, saturated like every activation.
//   down: workgroup b takes rows 16 b .. 16 b + 15 of EVERY slot (the token's H row of that slot as activations) and
//         adds the slots up in order with their routing weights: the combine needs no launch and no buffer.
// Rows the slicing cannot read (width outside 4..8, not dword aligned) are redone element by element; an expert number
// outside the stack gives NaN.
constexpr int kOneMaxTiles = 16;       // row tiles per workgroup
constexpr int kOneWaves = 8;

struct MoeOneArgs {
    const uint16_t* X;             // up: the token's activations (P), fp16 or bf16 bits; down: H (topk, P) fp16 bits
    const int64_t* idx;            // (topk) selected experts
    const float* w;                // (topk) routing weights (down)
    const uint8_t* ids; int64_t ids_bytes;
    const float* min_s; const float* tau_s; const uint8_t* nbits; const int64_t* bit_off;   // (E, Q)
    void* out;                     // up: H (topk, units) fp16 bits; down: out (Q) in the caller's dtype
    int E, Q, P, topk;
    int units, gated;              // up: outputs per expert; whether the rows come as (gate, up) halves
    int tiles_per_wg;              // up: unit tiles per workgroup
};

// REG: the caller states that every row of the stack has one width and that the rows lie at regular places (row q of
// expert e at bit_off[0] + e * (bit_off[Q] - bit_off[0]) + q * P * width): the kernel then works a row's place out
// instead of reading it, which takes one dependent memory trip out of every round.
template <int T, bool DOWN, bool XC, int DT, bool REG>
__global__ void __launch_bounds__(64 * kOneWaves) moe_one_kernel(MoeOneArgs a) {
    using F = Fmt<false>;
    using XI = XIn<false, XC>;
    __shared__ float s_part[kOneMaxTiles][kOneWaves][16];    // [row tile][column range][row]
    __shared__ float s_sx[kOneMaxTiles][kOneWaves];          // sum of the activations over the column range
    __shared__ float2 s_fin[kOneMaxTiles][16];               // tau_s, min_s of the tile's rows
    __shared__ int s_ok[kOneMaxTiles];                       // the slot's expert number is inside the stack
    __shared__ float s_y[kOneMaxTiles][16];                  // a row tile's finished values
    __shared__ __align__(16) uint16_t s_x[kOneWaves][T * kStepCols];   // each wave's activations, narrowed (private to the wave)
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, kg = lane >> 4;
    // blockIdx.y = token: every token is a problem of its own (its slots, its activations, its output row)
    const int tok = blockIdx.y;
    a.idx += (size_t)tok * a.topk; a.w += (size_t)tok * a.topk;
    if constexpr (DOWN) { a.X += (size_t)tok * a.topk * a.P; a.out = reinterpret_cast<unsigned char*>(a.out) + (size_t)tok * a.Q * (DT == 0 ? 4 : 2); }
    else { a.X += (size_t)tok * a.P; a.out = reinterpret_cast<uint16_t*>(a.out) + (size_t)tok * a.topk * a.units; }
    const int n_steps = a.P / kStepCols;
    const int W = (n_steps + T - 1) / T, G = kOneWaves / W;
    const int g = wave / W, wc = wave - g * W;
    const int step0 = wc * T;
    const int RT = (!DOWN && a.gated) ? 2 : 1;               // row tiles per unit tile
    const int UT = DOWN ? 1 : a.units / 16;                  // unit tiles per expert
    const int ut_first = DOWN ? 0 : (int)blockIdx.x * a.tiles_per_wg;
    const int n_rt = DOWN ? a.topk : min(a.tiles_per_wg, a.topk * UT - ut_first) * RT;
    auto slot_of = [&](int i) { return DOWN ? i : (ut_first + i / RT) / UT; };
    auto row0_of = [&](int i) { return DOWN ? (int)blockIdx.x * 16 : ((ut_first + i / RT) % UT) * 16 + (i % RT) * a.units; };
    const int64_t clamp_byte = (a.ids_bytes - 8) & ~(int64_t)3;
    const v4u_t ones = {F::one_bits, F::one_bits, F::one_bits, F::one_bits};
    // REG: the stack's width, first bit and bits from one expert to the next (three reads that depend on nothing)
    const int reg_nb = REG ? (int)a.nbits[0] : 0;
    const int64_t reg_base = REG ? a.bit_off[0] : 0;
    const int64_t reg_stride = REG ? a.bit_off[a.E > 1 ? a.Q : 0] - reg_base : 0;

    // A round = the row tiles the workgroup's waves work on at the same time.  (Two rounds of the up kernel in flight
    // together were measured: no faster -- a CU's share of the bytes, not the chain of trips, sets the time -- and the
    // registers cost occupancy.)  The up kernel loads its activations once, the down kernel per round: every slot has
    // activations of its own.
    constexpr int R = 1;
    struct Round { int i; bool has; int nb; int64_t bit0; float ts, mn; bool e_ok, ok, sliced; };
    Round rd[R];
    uint4 wlo[R][T], whi[R][T];
    // The wave's 128 T columns of the token are 16 T pieces of 16 bytes: a lane requests one (or two) of them, narrows it
    // like every activation when it arrives as bf16 (zero past the end of the row) and leaves it in the wave's own part
    // of LDS; multiply reads the MFMA operands from there just before it needs them (every operand row holds the token:
    // only result row 0 is used).  Four registers instead of the 16 T of operands held across the wait for the ids, and
    // one narrowing per value instead of sixteen.
    constexpr int XP = (16 * T + kWave - 1) / kWave;
    v4u_t xc[XP];
    auto request_x = [&](const uint16_t* xrow) {
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const int piece = lane + kWave * i;
            const bool on = piece < 16 * T && (step0 + (piece >> 4)) < n_steps;
            xc[i] = *reinterpret_cast<const v4u_t*>(xrow + (on ? (size_t)step0 * kStepCols + (size_t)piece * 8 : (size_t)0));
        }
    };
    auto finish_x = [&]() {
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const int piece = lane + kWave * i;
            const bool on = (step0 + (piece >> 4)) < n_steps;
            v4u_t v;
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = on ? XI::pair(xc[i][k]) : 0u;
            if (piece < 16 * T) *reinterpret_cast<v4u_t*>(&s_x[wave][piece * 8]) = v;
        }
    };
    // nothing here is under a branch: a wave without a tile in this round reads the metadata of tile 0 and the start of ids
    auto request_meta = [&](Round& q, int i) {
        q.has = g < G && i < n_rt;
        q.i = q.has ? i : 0;
        const int64_t e = a.idx[slot_of(q.i)];
        q.e_ok = e >= 0 && e < a.E;
        const size_t mi = (size_t)(q.e_ok ? e : 0) * a.Q + row0_of(q.i) + r;
        if constexpr (REG) {
            q.nb = reg_nb;
            q.bit0 = reg_base + (int64_t)(q.e_ok ? e : 0) * reg_stride + (int64_t)(row0_of(q.i) + r) * a.P * reg_nb;
        } else {
            q.nb = a.nbits[mi];
            q.bit0 = a.bit_off[mi];
        }
        q.ts = a.tau_s[mi]; q.mn = a.min_s[mi];
    };
    // REG: a row's place is arithmetic, so a lane can ask for ANOTHER row's bytes: requests go out in the order lane = 4 * row
    // + chunk (four neighbouring lanes read 16 nb consecutive bytes of one row: far fewer L1 accesses per request than a row
    // per lane) and to_operand moves the registers into operand order (lane = row + 16 * chunk) across the wave.
    const int pull = 4 * (4 * r + kg);
    auto to_operand = [&](const uint4& v) -> uint4 {
        if constexpr (!REG) return v;
        return uint4{(uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.x), (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.y),
                     (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.z), (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.w)};
    };
    auto request_ids = [&](Round& q, uint4 (&lo)[T], uint4 (&hi)[T]) {
        q.ok = q.e_ok && q.nb >= 1 && q.nb <= 14 && q.bit0 >= 0 && ((q.bit0 + (int64_t)q.nb * a.P + 7) >> 3) + 8 <= a.ids_bytes;
        q.sliced = q.ok && q.nb >= 4 && q.nb <= 8 && (q.bit0 & 31) == 0;
        // the row and chunk this lane asks for: its own (row r, chunk kg), or in REG mode row lane / 4, chunk lane % 4 of the
        // same tile (rows of a tile follow each other at P * nb bits; all 16 are usable or none is)
        const int64_t ask_bit0 = REG ? q.bit0 + (int64_t)((lane >> 2) - r) * a.P * q.nb : q.bit0;
        const int ask_chunk = REG ? (lane & 3) : kg;
        const bool ask_sliced = !REG ? q.sliced : (q.e_ok && q.nb >= 4 && q.nb <= 8 && ask_bit0 >= 0 && (ask_bit0 & 31) == 0
                                                   && ((ask_bit0 + (int64_t)q.nb * a.P + 7) >> 3) + 8 <= a.ids_bytes);
        const uint64_t row_off = (uint64_t)(ask_bit0 >> 3) + (uint64_t)(step0 * 4 + ask_chunk) * (4u * (uint32_t)q.nb);
#pragma unroll
        for (int it = 0; it < T; ++it) {
            const bool use = ask_sliced && (step0 + it) < n_steps;     // a wave without a tile reads tile 0's again: no address shared by the whole chip
            const uint64_t off = use ? row_off + (uint64_t)it * (16u * (uint32_t)q.nb) : 0;
            lo[it] = *reinterpret_cast<const uint4*>(a.ids + off);
            hi[it] = *reinterpret_cast<const uint4*>(a.ids + off + (use ? 4u * (uint32_t)(q.nb - 4) : 16u));
        }
    };
    auto multiply = [&](const Round& q, const uint4 (&lo_)[T], const uint4 (&hi_)[T], const uint16_t* xrow) {
        const int nb = q.nb;
        const bool sliced = q.sliced;
        v4f_t sx = {0.f, 0.f, 0.f, 0.f}, acc = {0.f, 0.f, 0.f, 0.f};
        const uint32_t info = sliced ? ((uint32_t)nb | 256u) : 0u;
        // REG: one width for the whole stack, known without looking at the lanes (rows that cannot be read -- an expert
        // number outside the stack -- decode whatever was loaded; their results are replaced by NaN below)
        const uint32_t info0 = REG ? ((uint32_t)reg_nb | ((reg_nb >= 4 && reg_nb <= 8) ? 256u : 0u)) : (uint32_t)__builtin_amdgcn_readfirstlane((int)info);
        // (a regular stack whose rows do not start on dword boundaries has no sliced row: its lanes then multiply id 0 here and
        // the rows are redone element by element below, as without the statement)
        const bool uniform = REG ? ((info0 >> 8) == 1u && __builtin_amdgcn_ballot_w64(q.e_ok && !sliced) == 0)
                                 : (__builtin_amdgcn_ballot_w64(info != info0) == 0 && (info0 >> 8) == 1u);
#pragma unroll
        for (int it = 0; it < T; ++it) {
            v4u_t b[4];
            const uint4 lo = to_operand(lo_[it]), hi = to_operand(hi_[it]);
            if (uniform) {
                switch (info0 & 0xFFu) {
                    case 7: decode_slice<7, false>(lo, hi, b); break;
                    case 6: decode_slice<6, false>(lo, hi, b); break;
                    case 5: decode_slice<5, false>(lo, hi, b); break;
                    case 4: decode_slice<4, false>(lo, hi, b); break;
                    default: decode_slice<8, false>(lo, hi, b); break;
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) b[j] = v4u_t{F::bias_bits, F::bias_bits, F::bias_bits, F::bias_bits};
                if constexpr (!REG) {
                    if (__builtin_amdgcn_ballot_w64(sliced && nb == 7)) { if (sliced && nb == 7) decode_slice<7, false>(lo, hi, b); }
                    if (__builtin_amdgcn_ballot_w64(sliced && nb == 6)) { if (sliced && nb == 6) decode_slice<6, false>(lo, hi, b); }
                    if (__builtin_amdgcn_ballot_w64(sliced && nb == 5)) { if (sliced && nb == 5) decode_slice<5, false>(lo, hi, b); }
                    if (__builtin_amdgcn_ballot_w64(sliced && nb == 4)) { if (sliced && nb == 4) decode_slice<4, false>(lo, hi, b); }
                    if (__builtin_amdgcn_ballot_w64(sliced && nb == 8)) { if (sliced && nb == 8) decode_slice<8, false>(lo, hi, b); }
                }
            }
            v4u_t xa[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) xa[j] = *reinterpret_cast<const v4u_t*>(&s_x[wave][it * kStepCols + kg * 32 + 8 * j]);
#pragma unroll
            for (int j = 0; j < 4; ++j) sx = F::mfma(xa[j], ones, sx);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc = F::mfma(xa[j], b[j], acc);
        }
        if (!q.has) return;                                   // wave-uniform
        const int i = q.i;
        // the token's sums (accumulator register 0 of lane group 0) into the wave's LDS slots
        if (kg == 0) s_part[i][wc][r] = __builtin_fmaf(-F::bias, sx[0], acc[0]);
        if (lane == 0) s_sx[i][wc] = sx[0];
        if (kg == 0 && wc == 0) s_fin[i][r] = float2{q.ts, q.mn};
        if (lane == 0 && wc == 0) s_ok[i] = q.e_ok ? 1 : 0;
        // rows the slicing cannot read: element by element over this wave's columns
        uint64_t odd = __builtin_amdgcn_ballot_w64(kg == 0 && !sliced);
        while (odd) {
            const int rr = __builtin_ctzll(odd);
            odd &= odd - 1;
            const int nb2 = __shfl(nb, rr, 64);
            const int64_t bit02 = ((int64_t)__shfl((int)(q.bit0 >> 32), rr, 64) << 32) | (uint32_t)__shfl((int)(uint32_t)q.bit0, rr, 64);
            const bool ok2 = __shfl((int)q.ok, rr, 64) != 0;
            const int c_lo = step0 * kStepCols, c_hi = min(a.P, (step0 + T) * kStepCols);
            float sacc = 0.f;
            if (ok2) {
                for (int c = c_lo + lane; c < c_hi; c += kWave)
                    sacc = __builtin_fmaf(XI::scalar(xrow[c]), (float)load_field(a.ids, bit02 + (int64_t)c * nb2, nb2, clamp_byte), sacc);
            } else {
                sacc = __builtin_nanf("");
            }
            const float tot = wave_sum(sacc);
            if (lane == 0) s_part[i][wc][rr] += tot;
        }
    };

    const int n_rounds = (n_rt + G - 1) / G;
    if constexpr (!DOWN) { request_x(a.X); }
    for (int r0 = 0; r0 < n_rounds; r0 += R) {
        if constexpr (DOWN) request_x(a.X + (size_t)slot_of(min(g + r0 * G, n_rt - 1) * (g < G ? 1 : 0)) * a.P);
#pragma unroll
        for (int k = 0; k < R; ++k) request_meta(rd[k], g + (r0 + k) * G);
#pragma unroll
        for (int k = 0; k < R; ++k) request_ids(rd[k], wlo[k], whi[k]);
        if (DOWN || r0 == 0) finish_x();
#pragma unroll
        for (int k = 0; k < R; ++k) multiply(rd[k], wlo[k], whi[k], a.X + (DOWN ? (size_t)slot_of(rd[k].i) * a.P : (size_t)0));
    }
    __syncthreads();

    // tau_s * sum(x * id) + min_s * sum(x) of every row the workgroup worked on, the ranges added in order: a thread per
    // row (not per output, which would leave one wave walking the slots' or the gate / up rows' ranges one LDS trip after
    // the other), the values handed on through LDS
    for (int o = tid; o < n_rt * 16; o += blockDim.x) {
        const int i = o >> 4, u = o & 15;
        double d = 0.0, xs = 0.0;
        for (int w = 0; w < W; ++w) { d += (double)s_part[i][w][u]; xs += (double)s_sx[i][w]; }
        const float2 f = s_fin[i][u];
        const float y = (float)((double)f.x * d + (double)f.y * xs);
        s_y[i][u] = s_ok[i] ? y : __builtin_nanf("");
    }
    __syncthreads();
    if constexpr (DOWN) {
        if (tid < 16) {
            float acc = 0.f;
            for (int j = 0; j < a.topk; ++j) acc = __builtin_fmaf(a.w[j], s_y[j][tid], acc);
            store_from_f32<DT>(a.out, (int64_t)blockIdx.x * 16 + tid, acc);
        }
    } else {
        const int n_ut = n_rt / RT;
        for (int o = tid; o < n_ut * 16; o += blockDim.x) {
            const int lut = o >> 4, u = o & 15, i0 = lut * RT;
            const float y0 = s_y[i0][u];
            float h;
            if (a.gated) h = (y0 / (1.0f + __expf(-y0))) * s_y[i0 + 1][u];
            else { const float p = fmaxf(y0, 0.f); h = y0 != y0 ? y0 : p * p; }
            const int ut = ut_first + lut;
            reinterpret_cast<uint16_t*>(a.out)[(size_t)(ut / UT) * a.units + (ut % UT) * 16 + u] = (uint16_t)sat_half_bits(h);
        }
    }
}

// ---- a few tokens (3..16): the tokens that chose an expert share one walk over it, on the matrix cores -------------------
// The routing plan groups the (token, choice) pairs by expert; a selected expert has at most one pair per token, so its
// pairs fit the 16 token rows of one MFMA operand, and every id that is read serves all of the expert's tokens: each
// selected expert's bytes are read once, however many tokens chose it.
//   up:   unit tiles of 16 outputs (gated: the 16 gate rows and the 16 matching up rows); H[pair] as saturated fp16.
//   down: tiles of 16 rows; Yd[pair] in fp32 for the weighted combine (moe_combine_kernel).
// work:    the workgroups are dealt to the experts in use, equally many each (the plan holds the number in use), and an
//          expert's tiles in equal runs to its workgroups; a run is walked in segments of as many tiles as the LDS holds.
// segment: the waves hold the activation rows as MFMA operands (row t = pair order[first + t]: the pair's token for the
//          up projection, the pair's own H row for the down projection).  The segment's rows are regrouped BY WIDTH in
//          LDS (a stable counting sort of at most 256 row records), so that the 16 rows a wave decodes together nearly
//          always share one width and take the single-width decode; a tile across a boundary takes each width in turn.
//          Then, per tile: T steps of 128 columns per wave (W = ceil(steps / T) waves per tile, G = 4 / W tiles at a
//          time), ids decoded into MFMA operands (exact in fp16 next to a bias of 1024), the next tile's ids in flight
//          meanwhile, partial sums in LDS, added in order in double.
// Rows the slicing cannot read (width outside 4..8, not dword aligned) are redone element by element; an expert number
// outside the stack gives NaN.
// (One token through this walk -- slot j = expert idx[j], the combine inside the down kernel -- was built and measured
// slower than moe_one_kernel: 28.7 against 24.7 us per layer; with so little work per workgroup the sort and its two
// barriers cost more than the single-width decode saves.)
struct MoeWalkArgs {
    const uint16_t* X;             // up: (tokens, P) fp16 or bf16 bits; down: H (npairs, P) fp16 bits
    MoePlan plan;
    const uint8_t* ids; int64_t ids_bytes;
    const float* min_s; const float* tau_s; const uint8_t* nbits; const int64_t* bit_off;   // (E, Q)
    void* out;                     // up: H (npairs, units) fp16 bits; down: Yd (npairs, Q) f32
    int E, Q, P, topk;
    int units, gated;              // up: outputs per expert; whether the rows come as (gate, up) halves
    int tiles_per_seg;             // unit tiles (up) / row tiles (down) per segment
    int max_tokens;                // most pairs an expert can have in this call (the LDS is laid out for it)
};
constexpr int kWalkWaves = 4;          // waves per workgroup: two workgroups share a CU
constexpr int kWalkMaxRowTiles = 16;   // row tiles per segment: one row record per thread

struct WalkRow { int64_t bit0; int flags; float ts, mn; int nat; };       // flags = width | usable << 8 | sliced << 9; nat = place before the sort

template <int T, bool DOWN, bool XC, bool TWO, bool REG>
__device__ __forceinline__ void moe_walk_body(const MoeWalkArgs& a) {
    using F = Fmt<false>;
    using XI = XIn<false, XC>;
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, kg = lane >> 4;
    const int n_steps = a.P / kStepCols;
    const int W = (n_steps + T - 1) / T, G = kWalkWaves / W;
    const int g = wave / W, wc = wave - g * W;
    const bool walker = g < G;                               // W = 3 leaves one wave without a column range
    const int step0 = wc * T;
    const int RT = (!DOWN && a.gated) ? 2 : 1;               // row tiles per unit tile
    const int UT = DOWN ? a.Q / 16 : a.units / 16;           // tiles per expert
    const int rt_cap = a.tiles_per_seg * RT;
    // LDS: partial sums [row tile][column range][row][token], sums of the activations [column range][token], per sorted
    // row its constants and its record, the counts of the sort, per natural row its sorted place
    float* s_part = reinterpret_cast<float*>(smem);
    float* s_sx = s_part + (size_t)rt_cap * W * 16 * a.max_tokens;                        // [W][16]
    float2* s_fin = reinterpret_cast<float2*>(s_sx + W * 16);                             // [rt_cap * 16]
    WalkRow* s_row = reinterpret_cast<WalkRow*>(s_fin + (size_t)rt_cap * 16);             // [rt_cap * 16]
    int* s_cls = reinterpret_cast<int*>(s_row + (size_t)rt_cap * 16);                     // [kWalkWaves][8]
    uint16_t* s_pos = reinterpret_cast<uint16_t*>(s_cls + kWalkWaves * 8);                // [rt_cap * 16]
    const int64_t clamp_byte = (a.ids_bytes - 8) & ~(int64_t)3;
    const v4u_t ones = {F::one_bits, F::one_bits, F::one_bits, F::one_bits};

    // REG (one width, rows at regular places, see moe_one_kernel): the stack's width, first bit, bits between experts
    const int reg_nb = REG ? (int)a.nbits[0] : 0;
    const int64_t reg_base = REG ? a.bit_off[0] : 0;
    const int64_t reg_stride = REG ? a.bit_off[a.E > 1 ? a.Q : 0] - reg_base : 0;
    const int n_active = a.plan.n_bad[1];
    const int per_expert = max(1, (int)gridDim.x / max(1, n_active));
    const int sl = (int)blockIdx.x / per_expert;
    if (sl >= n_active) return;                              // the whole workgroup
    const int run = (UT + per_expert - 1) / per_expert;
    int t0 = ((int)blockIdx.x - sl * per_expert) * run;
    const int t_end = min(UT, t0 + run);
    // the expert, its first pair and the number of its pairs (operand rows in use)
    const int4 slot = a.plan.slot[sl];
    const int e = slot.x, first = slot.y, n = max(1, min(slot.z - slot.y, min(16, a.max_tokens)));
    const bool e_ok = e >= 0 && e < a.E;
    auto pair_of = [&](int t) { return a.plan.order[first + t]; };

    v4u_t xa[T][4];
    v4f_t sx = {0.f, 0.f, 0.f, 0.f};
    while (t0 < t_end) {
        const int ut_first = t0;
        const int n_rt = min(a.tiles_per_seg, t_end - t0) * RT;
        t0 += n_rt / RT;
        auto row0_of = [&](int i) { return DOWN ? (ut_first + i) * 16 : (ut_first + i / RT) * 16 + (i % RT) * a.units; };
        // ---- the activation rows: operand row t = r (requested for every segment: from the caches after the first, and
        // never under a branch, so that the waits below are exact) ----
        const int pair = pair_of(min(r, n - 1));
        // ---- the segment's row records, regrouped by width (stable: rows of a width keep their order) ----
        const int n_rows = n_rt * 16;
        int key = 7, rank = 0;
        WalkRow mine{0, 0, 0.f, 0.f, 0};
        const int row_in_expert = tid < n_rows ? row0_of(tid >> 4) + (tid & 15) : 0;
        const size_t mi = (size_t)(e_ok ? e : 0) * a.Q + row_in_expert;
        int nb; int64_t bit0;
        if constexpr (REG) {
            nb = reg_nb;
            bit0 = reg_base + (int64_t)(e_ok ? e : 0) * reg_stride + (int64_t)row_in_expert * a.P * reg_nb;
        } else {
            nb = a.nbits[mi];
            bit0 = a.bit_off[mi];
        }
        const float row_ts = a.tau_s[mi], row_mn = a.min_s[mi];
        const uint16_t* xrow = a.X + (size_t)(DOWN ? pair : pair / a.topk) * a.P;
#pragma unroll
        for (int it = 0; it < T; ++it) {
            const bool on = (step0 + it) < n_steps;
            const uint16_t* xp = xrow + (on ? (size_t)(step0 + it) * kStepCols + kg * 32 : (size_t)0);
#pragma unroll
            for (int j = 0; j < 4; ++j) xa[it][j] = *reinterpret_cast<const v4u_t*>(xp + 8 * j);
        }
        bool row_usable = false;
        if (tid < n_rows) {
            const bool ok = e_ok && nb >= 1 && nb <= 14 && bit0 >= 0 && ((bit0 + (int64_t)nb * a.P + 7) >> 3) + 8 <= a.ids_bytes;
            const bool sliced = ok && nb >= 4 && nb <= 8 && (bit0 & 31) == 0;
            row_usable = ok;
            // REG: the record is complete without anything read from memory; tau_s and min_s go to LDS further down,
            // behind the first requests for ids
            mine = WalkRow{ok ? bit0 : 0, nb | (ok ? 256 : 0) | (sliced ? 512 : 0), REG ? 0.f : row_ts, REG ? 0.f : row_mn, tid};
            key = sliced ? nb - 4 : 5;
        }
        if constexpr (REG) {
            // one width: the rows stay where they are
            if (tid < n_rows) { s_row[tid] = mine; s_pos[tid] = (uint16_t)tid; }
            __syncthreads();
        } else {
#pragma unroll
        for (int c = 0; c < 6; ++c) {
            const uint64_t m = __builtin_amdgcn_ballot_w64(key == c);
            if (key == c) rank = __builtin_popcountll(m & ((1ull << lane) - 1ull));
            if (lane == 0) s_cls[wave * 8 + c] = __builtin_popcountll(m);
        }
        __syncthreads();
        if (tid < n_rows) {
            int base = 0;
#pragma unroll
            for (int c = 0; c < 6; ++c)
#pragma unroll
                for (int w = 0; w < kWalkWaves; ++w)
                    if (c < key || (c == key && w < wave)) base += s_cls[w * 8 + c];
            s_row[base + rank] = mine;
            s_pos[tid] = (uint16_t)(base + rank);
        }
        __syncthreads();
        }

        const int n_rounds = (n_rt + G - 1) / G;
        // Requests the lane's slices of the wave's tile of round `rnd` (clamped to the last round: nothing under a branch,
        // the repeated request at the end reads lines that are in the caches).  Returns the lane's row record.
        auto issue = [&](int rnd, uint4 (&lo)[T], uint4 (&hi)[T]) __attribute__((always_inline)) -> WalkRow {
            const int i = min(g + min(rnd, n_rounds - 1) * G, n_rt - 1);
            const WalkRow rec = s_row[i * 16 + r];
            // REG: the lane asks for chunk lane % 4 of row lane / 4 of the tile (neighbouring lanes, neighbouring bytes: far
            // fewer L1 accesses per request than a row per lane); to_operand brings the registers into operand order
            const WalkRow ask = REG ? s_row[i * 16 + (lane >> 2)] : rec;
            const int ask_chunk = REG ? (lane & 3) : kg;
            const uint32_t nbr = (uint32_t)ask.flags & 255u;
            const bool sliced = (ask.flags & 512) != 0;
            const uint64_t row_off = (uint64_t)(ask.bit0 >> 3) + (uint64_t)(step0 * 4 + ask_chunk) * (4u * nbr);
#pragma unroll
            for (int it = 0; it < T; ++it) {
                const bool use = sliced && (step0 + it) < n_steps;
                const uint64_t off = use ? row_off + (uint64_t)it * (16u * nbr) : 0;
                lo[it] = *reinterpret_cast<const uint4*>(a.ids + off);
                hi[it] = *reinterpret_cast<const uint4*>(a.ids + off + (use ? 4u * (nbr - 4u) : 16u));
            }
            return rec;
        };
        const int pull = 4 * (4 * r + kg);
        auto to_operand = [&](const uint4& v) __attribute__((always_inline)) -> uint4 {
            if constexpr (!REG) return v;
            return uint4{(uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.x), (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.y),
                         (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.z), (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.w)};
        };
        uint4 lo0[T], hi0[T], lo1[T], hi1[T];
        WalkRow rec0 = issue(0, lo0, hi0), rec1{0, 0, 0.f, 0.f, 0};     // by every wave: nothing under a branch
        if constexpr (REG) { if (tid < n_rows) s_fin[tid] = float2{row_usable ? row_ts : __builtin_nanf(""), row_mn}; }
        {
            // rows past the pairs and steps past the row multiply zeros; bf16 activations are narrowed like every activation
#pragma unroll
            for (int it = 0; it < T; ++it) {
                const bool on = (step0 + it) < n_steps && r < n;
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int k = 0; k < 4; ++k) xa[it][j][k] = on ? XI::pair(xa[it][j][k]) : 0u;
            }
            // sums of the activations over this wave's columns, per token: accumulator layout, lane (row r, token
            // group kg) register k <-> token 4 kg + k
            sx = v4f_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int it = 0; it < T; ++it)
#pragma unroll
                for (int j = 0; j < 4; ++j) sx = F::mfma(xa[it][j], ones, sx);
            if (g == 0 && r == 0) {
#pragma unroll
                for (int k = 0; k < 4; ++k) s_sx[wc * 16 + kg * 4 + k] = sx[k];
            }
        }
        auto compute = [&](int rnd, const WalkRow& rec, const uint4 (&lo_)[T], const uint4 (&hi_)[T]) __attribute__((always_inline)) {
            v4f_t acc = {0.f, 0.f, 0.f, 0.f};
            const int nbr = rec.flags & 255;
            const bool sliced = (rec.flags & 512) != 0;
            const uint32_t info = sliced ? ((uint32_t)nbr | 256u) : 0u;
            // REG: one width for the whole stack (rows that cannot be read decode what was loaded and end as NaN)
            const uint32_t info0 = REG ? ((uint32_t)reg_nb | ((reg_nb >= 4 && reg_nb <= 8) ? 256u : 0u)) : (uint32_t)__builtin_amdgcn_readfirstlane((int)info);
            // (usable rows of a regular stack that do not start on dword boundaries are not sliced: zero here, redone below)
            const bool uniform = REG ? ((info0 >> 8) == 1u && __builtin_amdgcn_ballot_w64((rec.flags & 256) != 0 && !sliced) == 0)
                                     : (__builtin_amdgcn_ballot_w64(info != info0) == 0 && (info0 >> 8) == 1u);
#pragma unroll
            for (int it = 0; it < T; ++it) {
                v4u_t b[4];
                const uint4 lo = to_operand(lo_[it]), hi = to_operand(hi_[it]);
                if (uniform) {
                    switch (info0 & 0xFFu) {
                        case 7: decode_slice<7, false>(lo, hi, b); break;
                        case 6: decode_slice<6, false>(lo, hi, b); break;
                        case 5: decode_slice<5, false>(lo, hi, b); break;
                        case 4: decode_slice<4, false>(lo, hi, b); break;
                        default: decode_slice<8, false>(lo, hi, b); break;
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) b[j] = v4u_t{F::bias_bits, F::bias_bits, F::bias_bits, F::bias_bits};
                    if constexpr (!REG) {
                        if (__builtin_amdgcn_ballot_w64(sliced && nbr == 7)) { if (sliced && nbr == 7) decode_slice<7, false>(lo, hi, b); }
                        if (__builtin_amdgcn_ballot_w64(sliced && nbr == 6)) { if (sliced && nbr == 6) decode_slice<6, false>(lo, hi, b); }
                        if (__builtin_amdgcn_ballot_w64(sliced && nbr == 5)) { if (sliced && nbr == 5) decode_slice<5, false>(lo, hi, b); }
                        if (__builtin_amdgcn_ballot_w64(sliced && nbr == 4)) { if (sliced && nbr == 4) decode_slice<4, false>(lo, hi, b); }
                        if (__builtin_amdgcn_ballot_w64(sliced && nbr == 8)) { if (sliced && nbr == 8) decode_slice<8, false>(lo, hi, b); }
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) acc = F::mfma(xa[it][j], b[j], acc);
            }
            const int i = g + rnd * G;                            // place of the tile among the sorted rows
            if (i < n_rt) {                                       // wave-uniform
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int t = kg * 4 + k;
                    if (t < n) s_part[(((size_t)i * W + wc) * 16 + r) * n + t] = __builtin_fmaf(-F::bias, sx[k], acc[k]);
                }
                if constexpr (!REG) { if (kg == 0 && wc == 0) s_fin[i * 16 + r] = float2{(rec.flags & 256) ? rec.ts : __builtin_nanf(""), rec.mn}; }
                // rows the slicing cannot read: element by element over this wave's columns, token by token
                uint64_t odd = __builtin_amdgcn_ballot_w64(kg == 0 && !sliced);
                while (odd) {
                    const int rr = __builtin_ctzll(odd);
                    odd &= odd - 1;
                    const WalkRow o = s_row[i * 16 + rr];
                    const int nb2 = o.flags & 255;
                    const int c_lo = step0 * kStepCols, c_hi = min(a.P, (step0 + T) * kStepCols);
                    for (int t = 0; t < n; ++t) {
                        const int pr = pair_of(t);
                        const uint16_t* xr = a.X + (size_t)(DOWN ? pr : pr / a.topk) * a.P;
                        float sacc = 0.f;
                        if (o.flags & 256) {
                            for (int c = c_lo + lane; c < c_hi; c += kWave)
                                sacc = __builtin_fmaf(XI::scalar(xr[c]), (float)load_field(a.ids, o.bit0 + (int64_t)c * nb2, nb2, clamp_byte), sacc);
                        }
                        const float tot = wave_sum(sacc);
                        if (lane == 0) s_part[(((size_t)i * W + wc) * 16 + rr) * n + t] += tot;
                    }
                }
            }
        };
        if (walker) {
            if constexpr (TWO) {
                // two register sets: the next tile's ids are in flight while a tile is decoded
                for (int r0 = 0; r0 < n_rounds; r0 += 2) {
                    rec1 = issue(r0 + 1, lo1, hi1);
                    compute(r0, rec0, lo0, hi0);
                    rec0 = issue(r0 + 2, lo0, hi0);
                    if (r0 + 1 < n_rounds) compute(r0 + 1, rec1, lo1, hi1);
                }
            } else {
                for (int r0 = 0; r0 < n_rounds; ++r0) {
                    compute(r0, rec0, lo0, hi0);
                    if (r0 + 1 < n_rounds) rec0 = issue(r0 + 1, lo0, hi0);
                }
            }
        }
        __syncthreads();

        // natural row j of the segment, operand row t: tau_s * sum(x * id) + min_s * sum(x), the column ranges added in order
        auto row_value = [&](int j, int t) {
            const int at = s_pos[j];
            double d = 0.0, xs = 0.0;
            for (int w = 0; w < W; ++w) {
                d += (double)s_part[(((size_t)(at >> 4) * W + w) * 16 + (at & 15)) * n + t];
                xs += (double)s_sx[w * 16 + t];
            }
            const float2 f = s_fin[at];
            return (float)((double)f.x * d + (double)f.y * xs);
        };
        if constexpr (DOWN) {
            float* Yd = reinterpret_cast<float*>(a.out);
            for (int o = tid; o < n_rows * n; o += blockDim.x) {
                const int t = o % n, j = o / n;
                Yd[(size_t)pair_of(t) * a.Q + row0_of(j >> 4) + (j & 15)] = row_value(j, t);
            }
        } else {
            const int n_ut = n_rt / RT;
            uint16_t* H = reinterpret_cast<uint16_t*>(a.out);
            for (int o = tid; o < n_ut * 16 * n; o += blockDim.x) {
                const int t = o % n, u = (o / n) & 15, lut = o / (16 * n), j0 = lut * RT * 16 + u;
                const float y0 = row_value(j0, t);
                float h;
                if (a.gated) h = (y0 / (1.0f + __expf(-y0))) * row_value(j0 + 16, t);
                else { const float pz = fmaxf(y0, 0.f); h = y0 != y0 ? y0 : pz * pz; }
                H[(size_t)pair_of(t) * a.units + (ut_first + lut) * 16 + u] = (uint16_t)sat_half_bits(h);
            }
        }
        __syncthreads();                                     // the next segment reuses the LDS
    }
}

// rows of up to 2048 columns: within 256 registers, two workgroups per CU (one starts while the other walks)
template <int T, bool DOWN, bool XC, bool TWO, bool REG>
__global__ void __launch_bounds__(64 * kWalkWaves) __attribute__((amdgpu_waves_per_eu(2, 2))) moe_walk_kernel(MoeWalkArgs a) {
    moe_walk_body<T, DOWN, XC, TWO, REG>(a);
}
// longer rows: eight steps of activations per wave need more registers, one workgroup per CU
template <bool DOWN, bool XC, bool REG>
__global__ void __launch_bounds__(64 * kWalkWaves) moe_walk_wide_kernel(MoeWalkArgs a) {
    moe_walk_body<8, DOWN, XC, false, REG>(a);
}

template <int DT>
__global__ void __launch_bounds__(256) moe_combine_kernel(const float* __restrict__ Yd, const float* __restrict__ w, void* __restrict__ out,
                                                          int topk, int D, int tokens, const int32_t* __restrict__ n_bad) {
    const int t = blockIdx.y;
    const int d = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= tokens || d >= D) return;
    float acc = 0.f;
    for (int j = 0; j < topk; ++j) acc = __builtin_fmaf(w[t * topk + j], Yd[((size_t)t * topk + j) * D + d], acc);
    if (*n_bad != 0) acc = __builtin_nanf("");                      // an expert index outside the stack: fail loudly
    store_from_f32<DT>(out, (int64_t)t * D + d, acc);
}

}  // namespace qvb8

using namespace qvb8;

namespace {
constexpr size_t kMoeLdsLimit = 144 * 1024;

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

int launch_moe_gemv(int stage, MoeGemvArgs a, int64_t slots, hipStream_t s) {
    // enough workgroups to fill the chip four times over the selected experts, at least one unit per wave
    const int waves = kMoeThreads / 64;
    // measured on the 35B-A3B shapes: four workgroups per CU are best for a handful of selected experts, eight for dozens
    const int64_t target_blocks = ((int64_t)host::env_int("QVB8_MOE_WGS_PER_CU", slots > 16 ? 8 : 4) * host::device_cus() + slots - 1) / slots;
    int64_t upb = (a.units + target_blocks - 1) / target_blocks;
    upb = (upb + waves - 1) / waves * waves;
    a.units_per_block = (int)upb;
    const size_t lds = (((size_t)a.x_rows * a.P * (stage == 0 ? 2 : 4) + 15) & ~(size_t)15) + (kMoeMB + kMoeMB * (kMoeThreads / 64)) * 4
                       + (size_t)upb * 2 * sizeof(MoeRow);
    if (lds > kMoeLdsLimit) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_moe_experts: P=%d does not fit the workgroup's LDS", a.P);
    static bool attr[2][64] = {{false}};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return host::fail(QVB8_ERR_LAUNCH, "qvb8_moe_experts: no current device");
    if (!attr[stage][dev]) {
        const void* f = stage == 0 ? (const void*)moe_gemv_kernel<0> : (const void*)moe_gemv_kernel<1>;
        if (hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMoeLdsLimit) != hipSuccess)
            return host::fail(QVB8_ERR_LAUNCH, "qvb8_moe_experts: cannot raise the kernel's LDS limit");
        attr[stage][dev] = true;
    }
    dim3 grid((unsigned)((a.units + upb - 1) / upb), (unsigned)slots);
    if (stage == 0) hipLaunchKernelGGL(moe_gemv_kernel<0>, grid, dim3(kMoeThreads), lds, s, a);
    else hipLaunchKernelGGL(moe_gemv_kernel<1>, grid, dim3(kMoeThreads), lds, s, a);
    return host::check_launch("qvb8_moe_experts");
}
// The matrix-core walk: what it needs.  H (fp16) takes the place of the fp32 H in the workspace.
bool moe_walk_shapes_ok(int64_t topk, int x_dtype, int64_t P_up, int64_t Q_dn, int64_t P_dn) {
    if (x_dtype != QVB8_F16 && x_dtype != QVB8_BF16) return false;
    if (P_up % kStepCols != 0 || P_dn % kStepCols != 0 || P_up > 4096 || P_dn > 4096) return false;
    return P_dn % 16 == 0 && Q_dn % 16 == 0 && topk >= 1;
}
// per token (no plan, the combine inside the down kernel): up to 8 slots, whose H rows are operand rows of one MFMA
bool moe_one_token_ok(int64_t tokens, int64_t topk, int x_dtype, int64_t P_up, int64_t Q_dn, int64_t P_dn) {
    if (tokens > host::env_int("QVB8_MOE_TILE_TOKENS", 16) || topk > 8) return false;
    return moe_walk_shapes_ok(topk, x_dtype, P_up, Q_dn, P_dn) && host::env_int("QVB8_MOE_ONE_TOKEN", 1) != 0;
}
// grouped by expert (7..16 tokens; fewer are faster one by one although an expert is then read once per token that chose it:
// 31 against 44 us per layer at 3 tokens, 53 against 56 at 6, 67 against 66 at 8 at the 35B-A3B shapes)
bool moe_group_ok(int64_t tokens, int64_t topk, int x_dtype, int64_t P_up, int64_t Q_dn, int64_t P_dn) {
    if (tokens < host::env_int("QVB8_MOE_GROUP_FROM", 7) || tokens > 16) return false;
    return moe_walk_shapes_ok(topk, x_dtype, P_up, Q_dn, P_dn) && host::env_int("QVB8_MOE_GROUPED", 1) != 0;
}

template <bool DOWN, bool XC, int DT, bool REG>
int launch_moe_one_as(const MoeOneArgs& a, unsigned blocks, unsigned tokens, hipStream_t s) {
    const int n_steps = a.P / kStepCols;
    // six steps per wave only for the down kernel (one round in flight): a whole row of up to 768 columns per wave, so
    // that eight slots are one round
    if constexpr (DOWN) {
        if (n_steps <= 6) {
            hipLaunchKernelGGL((moe_one_kernel<6, DOWN, XC, DT, REG>), dim3(blocks, tokens), dim3(64 * kOneWaves), 0, s, a);
            return host::check_launch("qvb8_moe_experts");
        }
    }
    hipLaunchKernelGGL((moe_one_kernel<4, DOWN, XC, DT, REG>), dim3(blocks, tokens), dim3(64 * kOneWaves), 0, s, a);
    return host::check_launch("qvb8_moe_experts");
}
template <bool DOWN, bool XC, int DT>
int launch_moe_one(const MoeOneArgs& a, bool regular, unsigned blocks, unsigned tokens, hipStream_t s) {
    return regular ? launch_moe_one_as<DOWN, XC, DT, true>(a, blocks, tokens, s) : launch_moe_one_as<DOWN, XC, DT, false>(a, blocks, tokens, s);
}

size_t moe_walk_lds(int64_t row_tiles, int W, int max_tokens) {
    return (size_t)row_tiles * W * 16 * max_tokens * 4 + (size_t)W * 16 * 4 + (size_t)row_tiles * 16 * (8 + sizeof(WalkRow) + 2)
           + (size_t)kWalkWaves * 8 * 4 + 16;
}

// `slots`: the plan's slots (experts that can be in use)
template <bool DOWN, bool XC, bool REG>
int launch_moe_walk_as(MoeWalkArgs a, int64_t slots, int64_t max_tokens, hipStream_t s) {
    const int n_steps = a.P / kStepCols;
    // steps per wave: four, with the next tile's ids in flight; a short down row (up to 768 columns) is one wave's; rows
    // beyond 2048 columns take eight steps per wave and one register set
    const int T = (DOWN && n_steps <= 6) ? 6 : (n_steps <= 4 * kWalkWaves ? 4 : 8);
    const int W = (n_steps + T - 1) / T;
    const int RT = (!DOWN && a.gated) ? 2 : 1;
    const int UT = DOWN ? a.Q / 16 : a.units / 16;
    a.max_tokens = (int)std::min<int64_t>(16, max_tokens);
    // tiles per segment: what the LDS of two workgroups per CU holds, one row record per thread
    int64_t per_seg = std::min<int64_t>(host::env_int("QVB8_MOE_GROUP_SEG_TILES", kWalkMaxRowTiles), kWalkMaxRowTiles / RT);
    per_seg = std::max<int64_t>(1, std::min<int64_t>(per_seg, UT));
    while (per_seg > 1 && moe_walk_lds(per_seg * RT, W, a.max_tokens) > 64 * 1024) --per_seg;
    a.tiles_per_seg = (int)per_seg;
    const size_t lds = moe_walk_lds(per_seg * RT, W, a.max_tokens);
    if (lds > 64 * 1024) return host::fail(QVB8_ERR_UNSUPPORTED, "qvb8_moe_experts: rows too long for the walk's LDS");
    // two workgroups per CU, at least one per slot (the kernel deals them to the experts in use)
    const int64_t wgs = std::max<int64_t>(slots, std::min<int64_t>((int64_t)host::env_int("QVB8_MOE_GROUP_WGS_PER_CU", 2) * host::device_cus(), slots * UT));
    dim3 grid((unsigned)wgs), block(64 * kWalkWaves);
    if constexpr (DOWN) {
        if (T == 6) {
            hipLaunchKernelGGL((moe_walk_kernel<6, true, XC, false, REG>), grid, block, lds, s, a);
            return host::check_launch("qvb8_moe_experts");
        }
    }
    if (T == 4) hipLaunchKernelGGL((moe_walk_kernel<4, DOWN, XC, true, REG>), grid, block, lds, s, a);
    else hipLaunchKernelGGL((moe_walk_wide_kernel<DOWN, XC, REG>), grid, block, lds, s, a);
    return host::check_launch("qvb8_moe_experts");
}
template <bool DOWN, bool XC>
int launch_moe_walk(const MoeWalkArgs& a, bool regular, int64_t slots, int64_t max_tokens, hipStream_t s) {
    return regular ? launch_moe_walk_as<DOWN, XC, true>(a, slots, max_tokens, s) : launch_moe_walk_as<DOWN, XC, false>(a, slots, max_tokens, s);
}
}  // namespace

extern "C" int64_t qvb8_moe_workspace_bytes(int64_t tokens, int64_t topk, int64_t n_experts, int64_t Q_up, int64_t P_dn, int64_t Q_dn) {
    (void)Q_up;
    if (tokens <= 0 || topk <= 0 || n_experts <= 0 || P_dn <= 0 || Q_dn <= 0) return 0;
    const int64_t np = tokens * topk;
    return (int64_t)(moe_plan_bytes(n_experts, np) + align256((size_t)np * P_dn * 4) + align256((size_t)np * Q_dn * 4));
}

extern "C" int qvb8_moe_experts(const void* X, int x_dtype, int64_t tokens, const int64_t* idx, const float* w, int64_t topk, int64_t n_experts,
                                const uint8_t* up_ids, int64_t up_ids_bytes, const float* up_min, const float* up_tau,
                                const uint8_t* up_nb, const int64_t* up_off, int64_t Q_up, int64_t P_up,
                                const uint8_t* dn_ids, int64_t dn_ids_bytes, const float* dn_min, const float* dn_tau,
                                const uint8_t* dn_nb, const int64_t* dn_off, int64_t Q_dn, int64_t P_dn,
                                int act, void* out, int out_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
    if (tokens < 0 || topk < 1 || n_experts < 1 || n_experts > 8192) return host::fail(QVB8_ERR_ARG, "qvb8_moe_experts: bad token / top-k / expert count");
    if ((act & ~(QVB8_MOE_UP_REGULAR | QVB8_MOE_DOWN_REGULAR)) != 0 && (act & ~(QVB8_MOE_UP_REGULAR | QVB8_MOE_DOWN_REGULAR)) != 1)
        return host::fail(QVB8_ERR_ARG, "qvb8_moe_experts: act must be 0 (gated SiLU) or 1 (ReLU squared), with the QVB8_MOE_*_REGULAR flags at most");
    const bool up_regular = (act & QVB8_MOE_UP_REGULAR) != 0, dn_regular = (act & QVB8_MOE_DOWN_REGULAR) != 0;
    act &= 0xFF;
    if (Q_up <= 0 || P_up <= 0 || Q_dn <= 0 || P_dn <= 0 || Q_up > 0x7fffffff || P_up > 0x7fffffff || Q_dn > 0x7fffffff || P_dn > 0x7fffffff)
        return host::fail(QVB8_ERR_ARG, "qvb8_moe_experts: bad shape");
    if (act == 0 ? (Q_up % 2 != 0 || Q_up / 2 != P_dn) : (Q_up != P_dn)) return host::fail(QVB8_ERR_ARG, "moe: gate_up/down shapes disagree");
    if (Q_dn != P_up) return host::fail(QVB8_ERR_ARG, "moe: down must map back to the hidden size");
    if (P_up % 32 != 0 || P_dn % 32 != 0) return host::fail(QVB8_ERR_UNSUPPORTED, "moe: P must be a multiple of 32");
    if (x_dtype < QVB8_F32 || x_dtype > QVB8_BF16 || out_dtype < QVB8_F32 || out_dtype > QVB8_BF16) return host::fail(QVB8_ERR_ARG, "qvb8_moe_experts: bad dtype");
    if (tokens == 0) return QVB8_OK;
    if (tokens * topk > 0x7fffffff / 4) return host::fail(QVB8_ERR_ARG, "qvb8_moe_experts: too many pairs");
    if (!X || !idx || !w || !up_ids || !up_min || !up_tau || !up_nb || !up_off || !dn_ids || !dn_min || !dn_tau || !dn_nb || !dn_off || !out)
        return host::fail(QVB8_ERR_ARG, "qvb8_moe_experts: null pointer");
    if ((reinterpret_cast<uintptr_t>(up_ids) & 15u) || (reinterpret_cast<uintptr_t>(dn_ids) & 15u)) return host::fail(QVB8_ERR_ARG, "moe: ids must be 16-byte aligned");
    if (up_ids_bytes < 32 || dn_ids_bytes < 32) return host::fail(QVB8_ERR_ARG, "qvb8_moe_experts: ids buffer shorter than 32 bytes");
    const int64_t need = qvb8_moe_workspace_bytes(tokens, topk, n_experts, Q_up, P_dn, Q_dn);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u))
        return host::fail(QVB8_ERR_WORKSPACE, "qvb8_moe_experts: needs %lld bytes of 16-byte aligned workspace", (long long)need);
    hipStream_t s = (hipStream_t)stream;
    const int64_t np = tokens * topk;
    unsigned char* ws = (unsigned char*)workspace;
    MoePlan pl = moe_plan_at(ws, n_experts, np);
    float* H = reinterpret_cast<float*>(ws + moe_plan_bytes(n_experts, np));
    float* Yd = reinterpret_cast<float*>(ws + moe_plan_bytes(n_experts, np) + align256((size_t)np * P_dn * 4));

    const bool grouped = moe_group_ok(tokens, topk, x_dtype, P_up, Q_dn, P_dn);
    if (!grouped && moe_one_token_ok(tokens, topk, x_dtype, P_up, Q_dn, P_dn)) {
        MoeOneArgs o;
        o.X = reinterpret_cast<const uint16_t*>(X); o.idx = idx; o.w = w; o.ids = up_ids; o.ids_bytes = up_ids_bytes;
        o.min_s = up_min; o.tau_s = up_tau; o.nbits = up_nb; o.bit_off = up_off; o.out = H;
        o.E = (int)n_experts; o.Q = (int)Q_up; o.P = (int)P_up; o.topk = (int)topk; o.units = (int)P_dn; o.gated = act == 0 ? 1 : 0;
        // unit tiles per workgroup: two workgroups fit a CU (at most 128 registers per lane), and a workgroup that takes its
        // tiles in one round has all its requests out at once -- so as few tiles each as 2 x CUs workgroups allow, within
        // what the rounds of a workgroup can take
        const int RT = o.gated ? 2 : 1;
        const int64_t total_ut = topk * (P_dn / 16);
        const int64_t places = (int64_t)host::device_cus() * host::env_int("QVB8_MOE_ONE_WGS_PER_CU", 2);
        int64_t per_wg = (total_ut + places - 1) / places;
        const int64_t cap = kOneMaxTiles / RT;
        if (per_wg > cap) per_wg = cap;
        if (per_wg < 1) per_wg = 1;
        o.tiles_per_wg = (int)per_wg;
        const unsigned up_blocks = (unsigned)((total_ut + per_wg - 1) / per_wg);
        const unsigned tk = (unsigned)tokens;
        if (int rc = x_dtype == QVB8_BF16 ? launch_moe_one<false, true, 0>(o, up_regular, up_blocks, tk, s) : launch_moe_one<false, false, 0>(o, up_regular, up_blocks, tk, s)) return rc;
        o.X = reinterpret_cast<const uint16_t*>(H); o.ids = dn_ids; o.ids_bytes = dn_ids_bytes;
        o.min_s = dn_min; o.tau_s = dn_tau; o.nbits = dn_nb; o.bit_off = dn_off; o.out = out;
        o.Q = (int)Q_dn; o.P = (int)P_dn; o.units = (int)Q_dn; o.gated = 0; o.tiles_per_wg = 0;
        const unsigned dn_blocks = (unsigned)(Q_dn / 16);
        if (out_dtype == QVB8_F32) return launch_moe_one<true, false, 0>(o, dn_regular, dn_blocks, tk, s);
        if (out_dtype == QVB8_F16) return launch_moe_one<true, false, 1>(o, dn_regular, dn_blocks, tk, s);
        return launch_moe_one<true, false, 2>(o, dn_regular, dn_blocks, tk, s);
    }

    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(kMoeThreads), (size_t)(n_experts + 8) * 4, s, idx, (int)np, (int)n_experts, pl,
                       grouped ? (int)(tokens < 16 ? tokens : 16) : (int)np);
    if (int rc = host::check_launch("qvb8_moe_experts plan")) return rc;
    const int64_t slots = moe_slots(n_experts, np);
    if (grouped) {
        MoeWalkArgs wa;
        wa.X = reinterpret_cast<const uint16_t*>(X); wa.plan = pl; wa.ids = up_ids; wa.ids_bytes = up_ids_bytes;
        wa.min_s = up_min; wa.tau_s = up_tau; wa.nbits = up_nb; wa.bit_off = up_off; wa.out = H;                // H as fp16 (pairs, P_dn)
        wa.E = (int)n_experts; wa.Q = (int)Q_up; wa.P = (int)P_up; wa.topk = (int)topk; wa.units = (int)P_dn; wa.gated = act == 0 ? 1 : 0;
        wa.tiles_per_seg = 1; wa.max_tokens = 1;
        if (int rc = x_dtype == QVB8_BF16 ? launch_moe_walk<false, true>(wa, up_regular, slots, tokens, s) : launch_moe_walk<false, false>(wa, up_regular, slots, tokens, s)) return rc;
        wa.X = reinterpret_cast<const uint16_t*>(H); wa.ids = dn_ids; wa.ids_bytes = dn_ids_bytes;
        wa.min_s = dn_min; wa.tau_s = dn_tau; wa.nbits = dn_nb; wa.bit_off = dn_off; wa.out = Yd;
        wa.Q = (int)Q_dn; wa.P = (int)P_dn; wa.units = (int)Q_dn; wa.gated = 0;
        if (int rc = launch_moe_walk<true, false>(wa, dn_regular, slots, tokens, s)) return rc;
        dim3 cgrid((unsigned)((Q_dn + 255) / 256), (unsigned)tokens);
        if (out_dtype == QVB8_F32) hipLaunchKernelGGL(moe_combine_kernel<0>, cgrid, dim3(256), 0, s, Yd, w, out, (int)topk, (int)Q_dn, (int)tokens, pl.n_bad);
        else if (out_dtype == QVB8_F16) hipLaunchKernelGGL(moe_combine_kernel<1>, cgrid, dim3(256), 0, s, Yd, w, out, (int)topk, (int)Q_dn, (int)tokens, pl.n_bad);
        else hipLaunchKernelGGL(moe_combine_kernel<2>, cgrid, dim3(256), 0, s, Yd, w, out, (int)topk, (int)Q_dn, (int)tokens, pl.n_bad);
        return host::check_launch("qvb8_moe_experts combine");
    }

    MoeGemvArgs a;
    a.X = X; a.ids = up_ids; a.ids_bytes = up_ids_bytes; a.min_s = up_min; a.tau_s = up_tau; a.nbits = up_nb; a.bit_off = up_off;
    a.out = H; a.plan = pl; a.Q = (int)Q_up; a.P = (int)P_up; a.topk = (int)topk; a.x_dtype = x_dtype; a.act = act;
    a.units = (int)P_dn; a.units_per_block = 0; a.x_rows = (int)(tokens < kMoeMB ? tokens : kMoeMB);
    if (int rc = launch_moe_gemv(0, a, slots, s)) return rc;
    a.X = H; a.ids = dn_ids; a.ids_bytes = dn_ids_bytes; a.min_s = dn_min; a.tau_s = dn_tau; a.nbits = dn_nb; a.bit_off = dn_off;
    a.out = Yd; a.Q = (int)Q_dn; a.P = (int)P_dn; a.x_dtype = QVB8_F32; a.units = (int)Q_dn;
    if (int rc = launch_moe_gemv(1, a, slots, s)) return rc;

    dim3 grid((unsigned)((Q_dn + 255) / 256), (unsigned)tokens);
    if (out_dtype == QVB8_F32) hipLaunchKernelGGL(moe_combine_kernel<0>, grid, dim3(256), 0, s, Yd, w, out, (int)topk, (int)Q_dn, (int)tokens, pl.n_bad);
    else if (out_dtype == QVB8_F16) hipLaunchKernelGGL(moe_combine_kernel<1>, grid, dim3(256), 0, s, Yd, w, out, (int)topk, (int)Q_dn, (int)tokens, pl.n_bad);
    else hipLaunchKernelGGL(moe_combine_kernel<2>, grid, dim3(256), 0, s, Yd, w, out, (int)topk, (int)Q_dn, (int)tokens, pl.n_bad);
    return host::check_launch("qvb8_moe_experts combine");
}

// ---- the same call for callers that cannot allocate ------------------------------------------------------------------
// The workspace of qvb8_moe_experts (routing plan, H, Yd) as a fixed array in the device image: every GPU the library
// runs on holds its own copy at its own address until the process ends.  Host code never uses the array's name as an
// address (there it is only a handle for the runtime): the device address is looked up once per device.
static __device__ __align__(256) unsigned char scratch[QVB8_MOE_STATIC_SCRATCH_BYTES];

namespace {
// device address of `scratch` on the current device, looked up on the first call there (with that device current)
int moe_static_scratch(void** out) {
    static void* ptr[64] = {nullptr};
    static std::mutex mu;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return host::fail(QVB8_ERR_LAUNCH, "qvb8_moe_experts_static: no current device");
    std::lock_guard<std::mutex> lock(mu);
    if (!ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return host::fail(QVB8_ERR_LAUNCH, "qvb8_moe_experts_static: cannot find the scratch array on device %d: %s", dev, hipGetErrorString(e));
        ptr[dev] = p;
    }
    *out = ptr[dev];
    return QVB8_OK;
}
}  // namespace

extern "C" int qvb8_moe_experts_static(const void* X, int x_dtype, int64_t tokens, const int64_t* idx, const float* w, int64_t topk, int64_t n_experts,
                                       const uint8_t* up_ids, int64_t up_ids_bytes, const float* up_min, const float* up_tau,
                                       const uint8_t* up_nb, const int64_t* up_off, int64_t Q_up, int64_t P_up,
                                       const uint8_t* dn_ids, int64_t dn_ids_bytes, const float* dn_min, const float* dn_tau,
                                       const uint8_t* dn_nb, const int64_t* dn_off, int64_t Q_dn, int64_t P_dn,
                                       int act, void* out, int out_dtype, void* stream) {
    const int64_t need = qvb8_moe_workspace_bytes(tokens, topk, n_experts, Q_up, P_dn, Q_dn);
    if (need > (int64_t)QVB8_MOE_STATIC_SCRATCH_BYTES)
        return host::fail(QVB8_ERR_WORKSPACE, "qvb8_moe_experts_static: this call needs %lld bytes of scratch, the built-in array holds %lld "
                          "(fewer tokens per call, or qvb8_moe_experts with a workspace)", (long long)need, (long long)QVB8_MOE_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    if (int rc = moe_static_scratch(&ws)) return rc;
    // nothing in the workspace has to start at zero: the plan kernel writes its counter before it is read, and H and Yd
    // are written completely before the next step reads them
    return qvb8_moe_experts(X, x_dtype, tokens, idx, w, topk, n_experts, up_ids, up_ids_bytes, up_min, up_tau, up_nb, up_off, Q_up, P_up,
                            dn_ids, dn_ids_bytes, dn_min, dn_tau, dn_nb, dn_off, Q_dn, P_dn, act, out, out_dtype, ws,
                            (int64_t)QVB8_MOE_STATIC_SCRATCH_BYTES, stream);
}
