// QVB8R on gfx950: band ids that are rANS-coded (32 interleaved streams per tile) are decoded on the fly.
//
// A tile is walked by HALF a wavefront: lane j of the half owns the 64-bit rANS state j.  Per step a lane looks its
// state up in the class's 4096-entry slot table (LDS, one class per workgroup), gets the symbol of column
// 32 * step + j and advances  x' = f * (x >> 12) + d.  Steps go in pairs: after two symbols the lanes whose state
// fell below 2^32 take the next 32-bit word of the tile's stream in lane order (ballot of the half + popcount).  Words
// come from a per-tile LDS ring that is refilled from registers loaded half a ring ahead.  A wave64 therefore walks
// TWO tiles at once, a workgroup of 256 threads eight: the block schedule of the format (runs of <= 8 tiles of one
// class) maps one block to one workgroup.  id = symbol + drow[row]; value = fmaf(id, tau_s[row], min_s[row]).
//
//   qvb8r_decode   dense rows (fp32 / fp16 / bf16 values, or the ids as int16), bit-exact with the QVB8 restore
//   qvb8r_gemv     Y = tau_s * (sum x * symbol + drow * sum x) + min_s * sum x.  M = 1: fp32 multiply-adds per lane.
//                  M = 2..48: the symbols of a workgroup's eight rows go through LDS as exact fp16 integers and meet X on
//                  the matrix cores (v_mfma_f32_16x16x32_f16, fp32 accumulate), so the cost of a launch is the walk and
//                  hardly depends on M.  X is scaled per row by a power of two into fp16 range and split hi + lo (lo only
//                  for fp32 X: fp16 / bf16 values are exact in hi), the scale is undone exactly at the end.
//   qvb8r_fix_escapes   Y[m, q] += sum over q's escapes of x[m, c] * delta, in stored order, one thread per output
//
// The walk is bound by the dependent LDS lookups and the 64-bit multiply per symbol, not by HBM (the stream is about
// 4.5 bits per weight).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/qvb8_amd.h"
#include "qvb8_device.h"
#include "qvb8_host.h"

namespace qvb8 {

constexpr int kRTiles = 8;             // tiles per workgroup (two per wave)
constexpr int kRThreads = 32 * kRTiles;
constexpr int kRing = 256;             // 32-bit words per tile ring: a pair takes <= 32, refilled every kRing / 2

struct RCore {
    const uint32_t* words; int64_t n_words;      // stream + at least 2048 zero words of pad (n_words counts the pad)
    const int64_t* tile_off;                     // [n_tiles + 1] in words
    const uint64_t* states;                      // [n_tiles][32]
    const int64_t* tiles;                        // [n_tiles][3] class, first sorted row, rows
    const int32_t* blocks;                       // [n_blocks][3] class, first tile, tiles (<= 8)
    const uint32_t* tab;                         // [K][4096]
    const int32_t* perm;                         // sorted row -> original row
    const float* min_s; const float* tau_s; const int32_t* drow;   // by original row
    int n_tiles, n_blocks, K, Q, P;
};

struct Walker {
    uint32_t xl, xh;
    int ptr, sb;
    uint32_t pre[kRing / 64];
    const uint32_t* wp;
};

// Returns the last word index (from the tile's first word) the walk may read ahead to: the end of the buffer, and -- when
// the next tile's words follow this tile's, as every writer lays them out -- the tile's own last word.  The ring always
// asks for 128..384 words more than the walk has used; past the tile's end those lines belong to a tile that another
// workgroup walks at another time, so they came from memory twice (measured at the 65B shapes, one row per tile of 1150
// words: 325 MB fetched for 267 MB of stream).  Requests past the bound read the bound's word again.
__device__ __forceinline__ int64_t walk_init(Walker& z, uint32_t* rg, const RCore& c, int tile, int l32) {
    int64_t off = c.tile_off[tile];
    const int64_t next = c.tile_off[tile + 1];
    const int64_t last = c.n_words - (kRing + kRing / 2);                  // the furthest start that keeps every read inside
    off = off < 0 ? 0 : (off > last ? last : off);
    z.wp = c.words + off;
    int64_t room = c.n_words - 1 - off;
    if (next > off && next - off - 1 < room) room = next - off - 1;
    const uint64_t s = c.states[(int64_t)tile * 32 + l32];
    z.xl = (uint32_t)s; z.xh = (uint32_t)(s >> 32);
    z.ptr = z.sb = 0;
#pragma unroll
    for (int q = 0; q < kRing / 32; ++q) {
        const int64_t i = 32 * q + l32;
        rg[32 * q + l32] = z.wp[i < room ? i : room];
    }
#pragma unroll
    for (int q = 0; q < kRing / 64; ++q) {
        const int64_t i = kRing + 32 * q + l32;
        z.pre[q] = z.wp[i < room ? i : room];
    }
    return room;
}

// one symbol: x' = f * (x >> 12) + d on the 64-bit state
// `st` holds the slot table re-packed for the walk (block_setup): frequency << 21 | (slot - cumulative) << 11 | symbol.
__device__ __forceinline__ uint32_t walk_dec(Walker& z, const uint32_t* st) {
    const uint32_t E = st[z.xl & 4095u];
    const uint32_t f = E >> 21, d = (E >> 11) & 1023u;
    const uint64_t q = (((uint64_t)z.xh << 32) | z.xl) >> 12;
    const uint64_t x = (uint64_t)f * q + d;
    z.xl = (uint32_t)x; z.xh = (uint32_t)(x >> 32);
    return E & 2047u;
}

// Two symbols, then one renormalisation.  Called by whole half-waves (the lanes of a tile are all in or all out).
// `room` = words the tile's stream may still be read ahead (clamps the read-ahead of a damaged stream inside the pad).
__device__ __forceinline__ void walk_pair(Walker& z, const uint32_t* st, uint32_t* rg, int l32, int half, int64_t room,
                                          uint32_t& s1, uint32_t& s2) {
    s1 = walk_dec(z, st);
    s2 = walk_dec(z, st);
    const bool need = z.xh == 0u;
    const uint64_t mk64 = __builtin_amdgcn_ballot_w64(need);
    const uint32_t mk = half ? (uint32_t)(mk64 >> 32) : (uint32_t)mk64;
    const uint32_t below = mk & ((1u << l32) - 1u);
    if (need) { z.xh = z.xl; z.xl = rg[(z.ptr + __builtin_popcount(below)) & (kRing - 1)]; }
    z.ptr += __builtin_popcount(mk);
    if (z.ptr - z.sb >= kRing / 2) {                                       // uniform within the half
#pragma unroll
        for (int q = 0; q < kRing / 64; ++q) rg[(z.sb + kRing + 32 * q + l32) & (kRing - 1)] = z.pre[q];
        z.sb += kRing / 2;
        const int64_t at = (int64_t)z.sb + kRing;
#pragma unroll
        for (int q = 0; q < kRing / 64; ++q) {
            const int64_t i = at + 32 * q + l32;
            z.pre[q] = z.wp[i < room ? i : room];
        }
    }
}

__device__ __forceinline__ float half_sum(float v) {                       // sum over the 32 lanes of a half, to every lane
    v = dpp_add<0xB1>(v);     // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);     // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);    // row_half_mirror
    v = dpp_add<0x140>(v);    // row_mirror: every lane of a 16-lane row holds the row sum
    return v + __shfl_xor(v, 16, 64);
}

// Per-workgroup set-up shared by the kernels: slot table into LDS, this half-wave's tile.
struct TileCtx { bool has; int tile, r0, nr; int64_t room; };
__device__ __forceinline__ TileCtx block_setup(const RCore& c, int block, uint32_t* st, int h8) {
    int cls = c.blocks[3 * block], tb = c.blocks[3 * block + 1], ntb = c.blocks[3 * block + 2];
    cls = cls < 0 ? 0 : (cls >= c.K ? c.K - 1 : cls);
    // the file's entry is (frequency - 1) << 22 | (slot - cumulative) << 11 | symbol with frequency <= 1024; the walk wants
    // the frequency itself, one instruction per symbol less
    for (int i = threadIdx.x; i < 4096; i += blockDim.x) {
        const uint32_t E = c.tab[(int64_t)cls * 4096 + i];
        st[i] = (((E >> 22) + 1u) << 21) | (E & 0x1FFFFFu);
    }
    TileCtx t;
    t.tile = tb + h8;
    t.has = h8 < ntb && t.tile >= 0 && t.tile < c.n_tiles;
    if (!t.has) t.tile = 0;
    t.r0 = (int)c.tiles[3 * (int64_t)t.tile + 1];
    t.nr = t.has ? (int)c.tiles[3 * (int64_t)t.tile + 2] : 0;
    if (t.r0 < 0 || t.r0 + t.nr > c.Q) { t.nr = 0; t.has = false; }
    t.room = 0;
    return t;
}

// ---- dense rows -----------------------------------------------------------------------------------------------------
// DT: 0 fp32, 1 fp16, 2 bf16 values; 3 the ids as int16.  row_base < 0: a row is written at its ORIGINAL index;
// row_base >= 0: at its sorted position - row_base (a contiguous block range fills a compact chunk of out_rows rows).
// `list` (or null): workgroup j walks block list[j] instead of block b0 + j and writes row r of the block's tile h at row
// (j * 8 + h) * T + r of `out` (a fixed slot per tile: what a lookup of scattered rows gathers from).
template <int DT>
__global__ void __launch_bounds__(kRThreads) r_decode_kernel(RCore c, int b0, int64_t row_base, int64_t out_rows, void* __restrict__ out, int T,
                                                             const int32_t* __restrict__ list) {
    __shared__ uint32_t st[4096];
    __shared__ uint32_t ring[kRTiles][kRing];
    const int lane = threadIdx.x & 63, l32 = lane & 31, half = lane >> 5, h8 = threadIdx.x >> 5;
    int block_no = b0 + (int)blockIdx.x;
    if (list) {
        block_no = list[blockIdx.x];
        if (block_no < 0 || block_no >= c.n_blocks) return;                   // the whole workgroup: a bad entry writes nothing
    }
    TileCtx t = block_setup(c, block_no, st, h8);
    uint32_t* rg = ring[h8];
    Walker z;
    t.room = walk_init(z, rg, c, t.tile, l32);
    __syncthreads();
    const int S = c.P >> 5;
    for (int r = 0; r < T; ++r) {
        if (!(t.has && r < t.nr)) continue;                                // per half-wave
        const int orow = c.perm[t.r0 + r];
        const bool row_ok = orow >= 0 && orow < c.Q;
        const float m = row_ok ? c.min_s[orow] : 0.f, ts = row_ok ? c.tau_s[orow] : 0.f;
        const int dr = row_ok ? c.drow[orow] : 0;
        const int64_t at = list ? ((int64_t)blockIdx.x * kRTiles + h8) * T + r : row_base < 0 ? (int64_t)orow : (int64_t)(t.r0 + r) - row_base;
        const bool store = row_ok && at >= 0 && at < out_rows;
        for (int s0 = 0; s0 < S; s0 += 2) {
            uint32_t s1, s2;
            walk_pair(z, st, rg, l32, half, t.room, s1, s2);
            if (store) {
                const int64_t i1 = at * c.P + (int64_t)s0 * 32 + l32, i2 = i1 + 32;
                const int id1 = (int)s1 + dr, id2 = (int)s2 + dr;
                if constexpr (DT == 3) {
                    reinterpret_cast<int16_t*>(out)[i1] = (int16_t)id1;
                    reinterpret_cast<int16_t*>(out)[i2] = (int16_t)id2;
                } else {
                    store_from_f32<DT>(out, i1, __builtin_fmaf((float)id1, ts, m));
                    store_from_f32<DT>(out, i2, __builtin_fmaf((float)id2, ts, m));
                }
            }
        }
    }
}

// ---- fused decode + product, one row of X ------------------------------------------------------------------------------
// WALK_ONLY (a measurement aid, qvb8r_walk_probe): the same launch with the activations not read and the two multiply-adds
// per pair replaced by an exclusive-or that keeps the symbols alive -- what the walk alone costs, the ceiling of this path.
template <int DT, bool WALK_ONLY = false>
__global__ void __launch_bounds__(kRThreads) r_gemv_kernel(RCore c, const void* __restrict__ X, float* __restrict__ Y, int T) {
    __shared__ uint32_t st[4096];
    __shared__ uint32_t ring[kRTiles][kRing];
    const int lane = threadIdx.x & 63, l32 = lane & 31, half = lane >> 5, h8 = threadIdx.x >> 5;
    TileCtx t = block_setup(c, blockIdx.x, st, h8);
    uint32_t* rg = ring[h8];
    Walker z;
    t.room = walk_init(z, rg, c, t.tile, l32);
    __syncthreads();
    const int S = c.P >> 5;
    float sx = 0.f;                  // sum of x over this lane's columns (the same for every row): taken while the first row is walked
    // one row: the walk with two multiply-adds per pair; FIRST also adds the activations up (a second copy of the loop
    // instead of a test per pair: the loop is bound by its instruction count)
    auto walk_row = [&](auto first) __attribute__((always_inline)) {
        constexpr bool FIRST = decltype(first)::value;
        if constexpr (WALK_ONLY) {
            uint32_t keep = 0;
            for (int s0 = 0; s0 < S; s0 += 2) {
                uint32_t s1, s2;
                walk_pair(z, st, rg, l32, half, t.room, s1, s2);
                keep ^= s1 + s2;
            }
            return (float)keep;
        } else {
            float acc = 0.f;
            float x1 = load_as_f32<DT>(X, l32), x2 = load_as_f32<DT>(X, 32 + l32);
            for (int s0 = 0; s0 < S; s0 += 2) {
                const int sn = s0 + 2 < S ? s0 + 2 : s0;                   // the last pair reloads itself (unused)
                const float n1 = load_as_f32<DT>(X, sn * 32 + l32), n2 = load_as_f32<DT>(X, (sn + 1) * 32 + l32);
                uint32_t s1, s2;
                walk_pair(z, st, rg, l32, half, t.room, s1, s2);
                acc = __builtin_fmaf(x1, (float)s1, acc);
                acc = __builtin_fmaf(x2, (float)s2, acc);
                if constexpr (FIRST) sx += x1 + x2;
                x1 = n1; x2 = n2;
            }
            if constexpr (FIRST) sx = half_sum(sx);
            return acc;
        }
    };
    for (int r = 0; r < T; ++r) {
        if (!(t.has && r < t.nr)) continue;                                // per half-wave
        const int orow = c.perm[t.r0 + r];
        const bool row_ok = orow >= 0 && orow < c.Q;
        const float acc = r == 0 ? walk_row(std::true_type{}) : walk_row(std::false_type{});
        const double m = row_ok ? (double)c.min_s[orow] : 0.0, ts = row_ok ? (double)c.tau_s[orow] : 0.0;
        const double dr = row_ok ? (double)c.drow[orow] : 0.0;
        const float a = half_sum(acc);
        if (l32 == 0 && row_ok) Y[orow] = (float)(ts * ((double)a + dr * (double)sx) + m * (double)sx);
    }
}

// ---- fused decode + product on the matrix cores, M = 2..48 ---------------------------------------------------------------
// A batch is 256 columns = four step pairs of every half-wave.  In LDS a pair's two symbols share a dword, so LDS
// position kk of a batch holds column  64 * (kk / 64) + 32 * (kk & 1) + (kk % 64) / 2  of the batch; X is packed in the
// same order, already in the A-operand layout: chunk (32 positions) x token tile x lane -> 8 halfs.
constexpr int kRBatchCols = 256;
constexpr int kRSymStride = kRBatchCols / 2 + 4;                           // dwords per row of a batch in LDS (padded)

constexpr int kRSlabCols = 1024;                                          // columns one workgroup of the packing kernel writes

struct RPacked {
    const uint4* hi; const uint4* lo;        // [chunks][NT][64]
    const double* sums;                      // [16 NT][slabs] sum of the scaled row, per slab, as the matrix cores see it
    const int* kexp;                         // [16 NT] the row was scaled by 2^kexp
    int slabs;
};

__device__ __forceinline__ int r_batch_col(int kk) { return 64 * (kk >> 6) + 32 * (kk & 1) + ((kk & 63) >> 1); }

// Workgroup (m, slab): the largest finite |x| of row m (every slab of the row finds it again: the row is a few KB of
// L2 hits), then this slab's columns scaled, split and laid out, and the slab's sum.
template <int DT, bool LO>
__global__ void __launch_bounds__(256) r_pack_x_kernel(const void* __restrict__ X, int M, int P, int NT,
                                                       uint4* __restrict__ hi, uint4* __restrict__ lo, double* __restrict__ sums, int* __restrict__ kexp) {
    __shared__ float s_max[256];
    __shared__ double s_sum[256];
    const int m = blockIdx.x, slab = blockIdx.y, tid = threadIdx.x;
    const bool valid = m < M;
    float mx = 0.f;
    if (valid) for (int c0 = tid * 8; c0 < P; c0 += 256 * 8) {            // P is a multiple of 128: whole groups of eight
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = __builtin_fabsf(load_as_f32<DT>(X, (int64_t)m * P + c0 + j));
#pragma unroll
        for (int j = 0; j < 8; ++j) mx = v[j] < __builtin_inff() ? __builtin_fmaxf(mx, v[j]) : mx;
    }
    s_max[tid] = mx;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) { if (tid < w) s_max[tid] = __builtin_fmaxf(s_max[tid], s_max[tid + w]); __syncthreads(); }
    mx = s_max[0];
    int k = 0;
    if (mx > 0.f) { int ex; (void)__builtin_frexpf(mx, &ex); k = 14 - ex; k = k < -100 ? -100 : (k > 100 ? 100 : k); }   // scaled max in [8192, 16384)
    const float scale = __builtin_ldexpf(1.f, k);
    const int Pp = (P + kRBatchCols - 1) / kRBatchCols * kRBatchCols;
    const int nt = m >> 4, r16 = m & 15;
    double sum = 0.0;
    const int g = slab * (kRSlabCols / 8) + tid;                            // eight LDS positions = one lane's share of a chunk
    if (tid < kRSlabCols / 8 && g < Pp / 8) {
        const int chunk = g >> 2, kg = g & 3;
        uint32_t h[4], l[4];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int kk = (chunk & 7) * 32 + kg * 8 + j;
            const int col = (chunk >> 3) * kRBatchCols + r_batch_col(kk);
            const float v = valid && col < P ? load_as_f32<DT>(X, (int64_t)m * P + col) * scale : 0.f;
            const _Float16 vh = (_Float16)v;
            const _Float16 vl = LO ? (_Float16)(v - (float)vh) : (_Float16)0.f;
            sum += (double)(float)vh + (double)(float)vl;
            const uint32_t bh = __builtin_bit_cast(uint16_t, vh), bl = __builtin_bit_cast(uint16_t, vl);
            if (j & 1) { h[j >> 1] |= bh << 16; l[j >> 1] |= bl << 16; } else { h[j >> 1] = bh; l[j >> 1] = bl; }
        }
        const int64_t at = ((int64_t)chunk * NT + nt) * 64 + kg * 16 + r16;
        hi[at] = make_uint4(h[0], h[1], h[2], h[3]);
        if (LO) lo[at] = make_uint4(l[0], l[1], l[2], l[3]);
    }
    s_sum[tid] = sum;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) { if (tid < w) s_sum[tid] += s_sum[tid + w]; __syncthreads(); }
    if (tid == 0) { sums[(int64_t)m * gridDim.y + slab] = s_sum[0]; if (slab == 0) kexp[m] = k; }
}

// fp16 bits (low half of the result) of an integer below 2048: exact
__device__ __forceinline__ uint32_t u16_to_half_bits(uint32_t v) {
    uint32_t r;
    asm("v_cvt_f16_u16_e32 %0, %1" : "=v"(r) : "v"(v));
    return r;
}

typedef _Float16 r_v8h_t __attribute__((ext_vector_type(8)));
typedef float r_v4f_t __attribute__((ext_vector_type(4)));

template <int NT, bool LO>
__global__ void __launch_bounds__(kRThreads) r_mma_kernel(RCore c, RPacked xp, int M, float* __restrict__ Y, int T) {
    __shared__ uint32_t st[4096];
    __shared__ uint32_t ring[kRTiles][kRing];
    __shared__ __align__(16) uint32_t sym[2][kRTiles][kRSymStride];
    __shared__ float red[kRThreads / 64][NT][256];
    __shared__ int s_row[kRTiles];
    __shared__ float s_ts[kRTiles], s_min[kRTiles], s_dr[kRTiles];
    __shared__ double s_sx[16 * NT];
    const int lane = threadIdx.x & 63, l32 = lane & 31, half = lane >> 5, h8 = threadIdx.x >> 5, wave = threadIdx.x >> 6;
    if (threadIdx.x < 16 * NT) {
        double a = 0.0;
        for (int i = 0; i < xp.slabs; ++i) a += xp.sums[threadIdx.x * xp.slabs + i];
        s_sx[threadIdx.x] = a;
    }
    TileCtx t = block_setup(c, blockIdx.x, st, h8);
    uint32_t* rg = ring[h8];
    Walker z;
    t.room = walk_init(z, rg, c, t.tile, l32);
    __syncthreads();
    const int S = c.P >> 5;
    const int n_batches = (c.P + kRBatchCols - 1) / kRBatchCols;
    const int n16 = lane & 15, kg = lane >> 4;
    int flip = 0;
    for (int r = 0; r < T; ++r) {
        const bool active = t.has && r < t.nr;                             // per half-wave
        r_v4f_t acc[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[nt] = r_v4f_t{0.f, 0.f, 0.f, 0.f};
        for (int b = 0; b < n_batches; ++b) {
            // this wave's two chunks of the batch: the X operands are requested before the walk
            uint4 xh[2][NT], xl[2][NT];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const int64_t at = ((int64_t)(b * 8 + wave * 2 + j) * NT + nt) * 64 + lane;
                    xh[j][nt] = xp.hi[at];
                    if (LO) xl[j][nt] = xp.lo[at];
                }
            uint32_t* sb = sym[flip][h8] + l32;
            const int pairs = (S - b * 8) >> 1;                            // step pairs left in the row: a short last batch ends in zeros
            if (active) {
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    uint32_t out = 0;
                    if (p < pairs) {                                       // uniform
                        uint32_t s1, s2;
                        walk_pair(z, st, rg, l32, half, t.room, s1, s2);
                        out = __builtin_amdgcn_perm(u16_to_half_bits(s2), u16_to_half_bits(s1), 0x05040100u);
                    }
                    sb[p * 32] = out;
                }
            } else {
#pragma unroll
                for (int p = 0; p < 4; ++p) sb[p * 32] = 0u;
            }
            __syncthreads();
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                uint4 w = make_uint4(0, 0, 0, 0);
                if (n16 < kRTiles) w = *reinterpret_cast<const uint4*>(&sym[flip][n16][(wave * 2 + j) * 16 + kg * 4]);
                const r_v8h_t bop = __builtin_bit_cast(r_v8h_t, w);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(r_v8h_t, xh[j][nt]), bop, acc[nt], 0, 0, 0);
                    if (LO) acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(r_v8h_t, xl[j][nt]), bop, acc[nt], 0, 0, 0);
                }
            }
            flip ^= 1;
        }
        // the row is done: lane holds tokens 4 kg + i of tile row n16; add the four waves' column shares
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave][nt][lane * 4 + i] = acc[nt][i];
        if (l32 == 0) {
            const int orow = active ? c.perm[t.r0 + r] : -1;
            const bool row_ok = orow >= 0 && orow < c.Q;
            s_row[h8] = row_ok ? orow : -1;
            s_ts[h8] = row_ok ? c.tau_s[orow] : 0.f;
            s_min[h8] = row_ok ? c.min_s[orow] : 0.f;
            s_dr[h8] = row_ok ? (float)c.drow[orow] : 0.f;
        }
        __syncthreads();
        for (int o = threadIdx.x; o < 16 * NT * kRTiles; o += kRThreads) {
            const int n = o & (kRTiles - 1), m = o >> 3, nt = m >> 4, m16 = m & 15;
            const int orow = s_row[n];
            if (orow < 0 || m >= M) continue;
            const int at = (((m16 >> 2) * 16 + n) << 2) + (m16 & 3);
            double a = 0.0;
#pragma unroll
            for (int w = 0; w < kRThreads / 64; ++w) a += (double)red[w][nt][at];
            const double sx = s_sx[m];
            const double v = (double)s_ts[n] * (a + (double)s_dr[n] * sx) + (double)s_min[n] * sx;
            Y[(int64_t)m * c.Q + orow] = (float)__builtin_ldexp(v, -xp.kexp[m]);
        }
        // red and s_row are written again only after the next row's batch barriers, which every thread reaches after this loop
    }
}

template <int DT>
__global__ void __launch_bounds__(256) r_fix_escapes_kernel(const void* __restrict__ X, const int64_t* __restrict__ uq, const int64_t* __restrict__ ptr,
        const int64_t* __restrict__ ec, const float* __restrict__ ed, float* __restrict__ Y, int64_t U, int M, int P, int Q) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= U * M) return;
    const int64_t u = i % U;
    const int m = (int)(i / U);
    const int64_t q = uq[u];
    if (q < 0 || q >= Q) return;
    float a = 0.f;
    for (int64_t e = ptr[u]; e < ptr[u + 1]; ++e) {
        const int64_t col = ec[e];
        if (col >= 0 && col < P) a = __builtin_fmaf(load_as_f32<DT>(X, (int64_t)m * P + col), ed[e], a);
    }
    Y[(int64_t)m * Q + q] += a;
}

}  // namespace qvb8

using namespace qvb8;

namespace {
int check_core(const char* who, const qvb8r_core* k, RCore& c) {
    if (!k) return host::fail(QVB8_ERR_ARG, "%s: null core", who);
    if (k->Q < 0 || k->P <= 0 || k->Q > 0x7fffffff || k->P > 0x7fffffff || (k->P % 128) != 0)
        return host::fail(QVB8_ERR_ARG, "%s: needs P %% 128 == 0 and Q, P below 2^31", who);
    if (k->n_tiles < 0 || k->n_tiles > 0x7fffffff || k->n_blocks < 0 || k->n_blocks > 0x7fffffff || k->n_classes < 1 || k->n_classes > 65535)
        return host::fail(QVB8_ERR_ARG, "%s: bad tile / block / class count", who);
    if (k->n_words < 2048) return host::fail(QVB8_ERR_ARG, "%s: the stream must end with at least 2048 zero words of pad", who);
    if (k->Q > 0 && (!k->words || !k->tile_off || !k->states || !k->tiles || !k->blocks || !k->tab || !k->perm || !k->min_s || !k->tau_s || !k->drow))
        return host::fail(QVB8_ERR_ARG, "%s: null pointer", who);
    c.words = k->words; c.n_words = k->n_words; c.tile_off = k->tile_off; c.states = k->states; c.tiles = k->tiles;
    c.blocks = k->blocks; c.tab = k->tab; c.perm = k->perm; c.min_s = k->min_s; c.tau_s = k->tau_s; c.drow = k->drow;
    c.n_tiles = (int)k->n_tiles; c.n_blocks = (int)k->n_blocks; c.K = (int)k->n_classes; c.Q = (int)k->Q; c.P = (int)k->P;
    return 0;
}
int64_t packed_cols(int64_t P) { return (P + kRBatchCols - 1) / kRBatchCols * kRBatchCols; }
int64_t packed_slabs(int64_t P) { return (packed_cols(P) + kRSlabCols - 1) / kRSlabCols; }
int64_t packed_plane_bytes(int64_t M, int64_t P) { return packed_cols(P) / 32 * ((M + 15) / 16) * 64 * 16; }
}  // namespace

extern "C" int qvb8r_decode(const qvb8r_core* core, int64_t max_tile_rows, int out_dtype, int64_t b0, int64_t nb, int64_t row_base,
                            void* out, int64_t out_rows, void* stream) {
    RCore c;
    if (int rc = check_core("qvb8r_decode", core, c)) return rc;
    if (out_dtype < 0 || out_dtype > 3) return host::fail(QVB8_ERR_ARG, "qvb8r_decode: out_dtype must be 0..3");
    if (b0 < 0 || nb < 0 || b0 + nb > c.n_blocks) return host::fail(QVB8_ERR_ARG, "qvb8r_decode: block range outside the schedule");
    if (max_tile_rows < 1 || max_tile_rows > 0x7fffffff) return host::fail(QVB8_ERR_ARG, "qvb8r_decode: bad rows-per-tile bound");
    if (nb == 0 || c.Q == 0) return QVB8_OK;
    if (!out || out_rows < 0) return host::fail(QVB8_ERR_ARG, "qvb8r_decode: null output");
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)nb), block(kRThreads);
    const int T = (int)max_tile_rows;
    switch (out_dtype) {
        case 0: hipLaunchKernelGGL(r_decode_kernel<0>, grid, block, 0, s, c, (int)b0, row_base, out_rows, out, T, (const int32_t*)nullptr); break;
        case 1: hipLaunchKernelGGL(r_decode_kernel<1>, grid, block, 0, s, c, (int)b0, row_base, out_rows, out, T, (const int32_t*)nullptr); break;
        case 2: hipLaunchKernelGGL(r_decode_kernel<2>, grid, block, 0, s, c, (int)b0, row_base, out_rows, out, T, (const int32_t*)nullptr); break;
        default: hipLaunchKernelGGL(r_decode_kernel<3>, grid, block, 0, s, c, (int)b0, row_base, out_rows, out, T, (const int32_t*)nullptr); break;
    }
    return host::check_launch("qvb8r_decode");
}

extern "C" int qvb8r_decode_blocks(const qvb8r_core* core, int64_t max_tile_rows, int out_dtype, const int32_t* block_list, int64_t n_list,
                                   void* out, int64_t out_rows, void* stream) {
    RCore c;
    if (int rc = check_core("qvb8r_decode_blocks", core, c)) return rc;
    if (out_dtype < 0 || out_dtype > 3) return host::fail(QVB8_ERR_ARG, "qvb8r_decode_blocks: out_dtype must be 0 (fp32), 1 (fp16), 2 (bf16) or 3 (ids)");
    if (max_tile_rows < 1 || max_tile_rows > 0x7fffffff) return host::fail(QVB8_ERR_ARG, "qvb8r_decode_blocks: bad rows-per-tile bound");
    if (n_list < 0 || n_list > 0x7fffffff) return host::fail(QVB8_ERR_ARG, "qvb8r_decode_blocks: bad list length");
    if (n_list == 0) return QVB8_OK;
    if (!block_list || !out) return host::fail(QVB8_ERR_ARG, "qvb8r_decode_blocks: null pointer");
    if (out_rows < n_list * kRTiles * max_tile_rows)
        return host::fail(QVB8_ERR_ARG, "qvb8r_decode_blocks: out needs %lld rows (blocks x 8 tiles x rows per tile)", (long long)(n_list * kRTiles * max_tile_rows));
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)n_list), block(kRThreads);
    const int T = (int)max_tile_rows;
    switch (out_dtype) {
        case 0: hipLaunchKernelGGL(r_decode_kernel<0>, grid, block, 0, s, c, 0, (int64_t)0, out_rows, out, T, block_list); break;
        case 1: hipLaunchKernelGGL(r_decode_kernel<1>, grid, block, 0, s, c, 0, (int64_t)0, out_rows, out, T, block_list); break;
        case 2: hipLaunchKernelGGL(r_decode_kernel<2>, grid, block, 0, s, c, 0, (int64_t)0, out_rows, out, T, block_list); break;
        default: hipLaunchKernelGGL(r_decode_kernel<3>, grid, block, 0, s, c, 0, (int64_t)0, out_rows, out, T, block_list); break;
    }
    return host::check_launch("qvb8r_decode_blocks");
}

extern "C" int qvb8r_walk_probe(const qvb8r_core* core, int64_t max_tile_rows, float* Y, void* stream) {
    RCore c;
    if (int rc = check_core("qvb8r_walk_probe", core, c)) return rc;
    if (max_tile_rows < 1 || max_tile_rows > 0x7fffffff) return host::fail(QVB8_ERR_ARG, "qvb8r_walk_probe: bad rows-per-tile bound");
    if (c.Q == 0 || c.n_blocks == 0) return QVB8_OK;
    if (!Y) return host::fail(QVB8_ERR_ARG, "qvb8r_walk_probe: null pointer");
    hipLaunchKernelGGL((r_gemv_kernel<0, true>), dim3((unsigned)c.n_blocks), dim3(kRThreads), 0, (hipStream_t)stream, c, (const void*)Y, Y, (int)max_tile_rows);
    return host::check_launch("qvb8r_walk_probe");
}

extern "C" int64_t qvb8r_gemv_workspace_bytes(int64_t M, int64_t P) {
    if (M < 1 || M > 48 || P <= 0) return 0;
    if (M == 1) return 16;                                                 // X is read in place
    return 2 * packed_plane_bytes(M, P) + 48 * 8 * packed_slabs(P) + 48 * 4;   // hi, lo, slab sums, row exponents
}

extern "C" int qvb8r_gemv(const void* X, int x_dtype, int64_t M, const qvb8r_core* core, int64_t max_tile_rows, float* Y,
                          void* workspace, int64_t workspace_bytes, void* stream) {
    RCore c;
    if (int rc = check_core("qvb8r_gemv", core, c)) return rc;
    if (M < 1 || M > 48) return host::fail(QVB8_ERR_ARG, "qvb8r_gemv: M=%lld outside 1..48", (long long)M);
    if (x_dtype < QVB8_F32 || x_dtype > QVB8_BF16) return host::fail(QVB8_ERR_ARG, "qvb8r_gemv: bad activation dtype");
    if (max_tile_rows < 1 || max_tile_rows > 0x7fffffff) return host::fail(QVB8_ERR_ARG, "qvb8r_gemv: bad rows-per-tile bound");
    if (c.Q == 0 || c.n_blocks == 0) return QVB8_OK;
    if (!X || !Y) return host::fail(QVB8_ERR_ARG, "qvb8r_gemv: null pointer");
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)c.n_blocks), block(kRThreads);
    const int T = (int)max_tile_rows;
    if (M == 1) {
        if (x_dtype == QVB8_F32) hipLaunchKernelGGL(r_gemv_kernel<0>, grid, block, 0, s, c, X, Y, T);
        else if (x_dtype == QVB8_F16) hipLaunchKernelGGL(r_gemv_kernel<1>, grid, block, 0, s, c, X, Y, T);
        else hipLaunchKernelGGL(r_gemv_kernel<2>, grid, block, 0, s, c, X, Y, T);
        return host::check_launch("qvb8r_gemv");
    }
    const int64_t need = qvb8r_gemv_workspace_bytes(M, c.P);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u))
        return host::fail(QVB8_ERR_WORKSPACE, "qvb8r_gemv: needs %lld bytes of 16-byte aligned workspace", (long long)need);
    const int NT = (int)((M + 15) / 16);
    const int64_t plane = packed_plane_bytes(M, c.P);
    uint8_t* ws = (uint8_t*)workspace;
    RPacked xp;
    const int slabs = (int)packed_slabs(c.P);
    uint4* hi = (uint4*)ws; uint4* lo = (uint4*)(ws + plane);
    double* sums = (double*)(ws + 2 * plane); int* kexp = (int*)(ws + 2 * plane + 48 * 8 * (int64_t)slabs);
    xp.hi = hi; xp.lo = lo; xp.sums = sums; xp.kexp = kexp; xp.slabs = slabs;
    const bool split = x_dtype == QVB8_F32;                                // fp16 / bf16 values, scaled by a power of two, are exact in hi
    const dim3 pgrid(16 * NT, slabs);
    if (split) hipLaunchKernelGGL((r_pack_x_kernel<0, true>), pgrid, dim3(256), 0, s, X, (int)M, c.P, NT, hi, lo, sums, kexp);
    else if (x_dtype == QVB8_F16) hipLaunchKernelGGL((r_pack_x_kernel<1, false>), pgrid, dim3(256), 0, s, X, (int)M, c.P, NT, hi, lo, sums, kexp);
    else hipLaunchKernelGGL((r_pack_x_kernel<2, false>), pgrid, dim3(256), 0, s, X, (int)M, c.P, NT, hi, lo, sums, kexp);
    if (int rc = host::check_launch("qvb8r_gemv pack")) return rc;
#define QVB8R_MMA(NT_) do { if (split) hipLaunchKernelGGL((r_mma_kernel<NT_, true>), grid, block, 0, s, c, xp, (int)M, Y, T); \
                            else hipLaunchKernelGGL((r_mma_kernel<NT_, false>), grid, block, 0, s, c, xp, (int)M, Y, T); } while (0)
    if (NT == 1) QVB8R_MMA(1); else if (NT == 2) QVB8R_MMA(2); else QVB8R_MMA(3);
#undef QVB8R_MMA
    return host::check_launch("qvb8r_gemv");
}

extern "C" int qvb8r_fix_escapes(const void* X, int x_dtype, int64_t M, const int64_t* uq, const int64_t* ptr, const int64_t* ec,
                                 const float* ed, int64_t U, float* Y, int64_t Q, int64_t P, void* stream) {
    if (M < 0 || U < 0 || Q < 0 || P < 0 || Q > 0x7fffffff || P > 0x7fffffff || M > 0x7fffffff) return host::fail(QVB8_ERR_ARG, "qvb8r_fix_escapes: bad shape");
    if (x_dtype < QVB8_F32 || x_dtype > QVB8_BF16) return host::fail(QVB8_ERR_ARG, "qvb8r_fix_escapes: bad activation dtype");
    if (U == 0 || M == 0) return QVB8_OK;
    if (!X || !uq || !ptr || !ec || !ed || !Y) return host::fail(QVB8_ERR_ARG, "qvb8r_fix_escapes: null pointer");
    const int64_t n = U * M;
    dim3 grid((unsigned)((n + 255) / 256)), block(256);
    hipStream_t s = (hipStream_t)stream;
    if (x_dtype == QVB8_F32) hipLaunchKernelGGL(r_fix_escapes_kernel<0>, grid, block, 0, s, X, uq, ptr, ec, ed, Y, U, (int)M, (int)P, (int)Q);
    else if (x_dtype == QVB8_F16) hipLaunchKernelGGL(r_fix_escapes_kernel<1>, grid, block, 0, s, X, uq, ptr, ec, ed, Y, U, (int)M, (int)P, (int)Q);
    else hipLaunchKernelGGL(r_fix_escapes_kernel<2>, grid, block, 0, s, X, uq, ptr, ec, ed, Y, U, (int)M, (int)P, (int)Q);
    return host::check_launch("qvb8r_fix_escapes");
}
