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
//   qvb8r_gemv     M = 1..16 rows of X (fp32 arithmetic): Y = tau_s * (sum x * symbol + drow * sum x) + min_s * sum x
//   qvb8r_fix_escapes   Y[m, q] += sum over q's escapes of x[m, c] * delta, in stored order, one thread per output
//
// The walk is bound by the dependent LDS lookups and the 64-bit multiply per symbol, not by HBM (the stream is about
// 4.5 bits per weight).
#include <hip/hip_runtime.h>
#include <stdint.h>

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

__device__ __forceinline__ void walk_init(Walker& z, uint32_t* rg, const RCore& c, int tile, int l32) {
    int64_t off = c.tile_off[tile];
    const int64_t last = c.n_words - (kRing + kRing / 2);                  // the furthest start that keeps every read inside
    off = off < 0 ? 0 : (off > last ? last : off);
    z.wp = c.words + off;
    const uint64_t s = c.states[(int64_t)tile * 32 + l32];
    z.xl = (uint32_t)s; z.xh = (uint32_t)(s >> 32);
    z.ptr = z.sb = 0;
#pragma unroll
    for (int q = 0; q < kRing / 32; ++q) rg[32 * q + l32] = z.wp[32 * q + l32];
#pragma unroll
    for (int q = 0; q < kRing / 64; ++q) z.pre[q] = z.wp[kRing + 32 * q + l32];
}

// one symbol: x' = f * (x >> 12) + d on the 64-bit state
__device__ __forceinline__ uint32_t walk_dec(Walker& z, const uint32_t* st) {
    const uint32_t E = st[z.xl & 4095u];
    const uint32_t f = (E >> 22) + 1u, d = (E >> 11) & 2047u;
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
    for (int i = threadIdx.x; i < 4096; i += blockDim.x) st[i] = c.tab[(int64_t)cls * 4096 + i];
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
template <int DT>
__global__ void __launch_bounds__(kRThreads) r_decode_kernel(RCore c, int b0, int64_t row_base, int64_t out_rows, void* __restrict__ out, int T) {
    __shared__ uint32_t st[4096];
    __shared__ uint32_t ring[kRTiles][kRing];
    const int lane = threadIdx.x & 63, l32 = lane & 31, half = lane >> 5, h8 = threadIdx.x >> 5;
    TileCtx t = block_setup(c, b0 + blockIdx.x, st, h8);
    uint32_t* rg = ring[h8];
    Walker z;
    walk_init(z, rg, c, t.tile, l32);
    t.room = c.n_words - 1 - (z.wp - c.words);
    __syncthreads();
    const int S = c.P >> 5;
    for (int r = 0; r < T; ++r) {
        if (!(t.has && r < t.nr)) continue;                                // per half-wave
        const int orow = c.perm[t.r0 + r];
        const bool row_ok = orow >= 0 && orow < c.Q;
        const float m = row_ok ? c.min_s[orow] : 0.f, ts = row_ok ? c.tau_s[orow] : 0.f;
        const int dr = row_ok ? c.drow[orow] : 0;
        const int64_t at = row_base < 0 ? (int64_t)orow : (int64_t)(t.r0 + r) - row_base;
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

// ---- activations, transposed: Xt[c][mb] fp32, mb < MB (rows past M are zero) ----------------------------------------
__global__ void __launch_bounds__(256) r_transpose_kernel(const void* __restrict__ X, int x_dtype, int M, int P, int MB, float* __restrict__ Xt) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)P * MB) return;
    const int c = (int)(i / MB), mb = (int)(i - (int64_t)c * MB);
    Xt[i] = mb < M ? load_as_f32(X, (int64_t)mb * P + c, x_dtype) : 0.f;
}

// ---- fused decode + product, M = 1..16 -------------------------------------------------------------------------------
template <int MB>
__device__ __forceinline__ void load_xt(const float* __restrict__ p, float (&v)[MB]) {
    if constexpr (MB >= 4) {
#pragma unroll
        for (int i = 0; i < MB; i += 4) {
            const float4 q = *reinterpret_cast<const float4*>(p + i);
            v[i] = q.x; v[i + 1] = q.y; v[i + 2] = q.z; v[i + 3] = q.w;
        }
    } else if constexpr (MB == 2) {
        const float2 q = *reinterpret_cast<const float2*>(p);
        v[0] = q.x; v[1] = q.y;
    } else {
        v[0] = p[0];
    }
}

template <int MB>
__global__ void __launch_bounds__(kRThreads) r_gemv_kernel(RCore c, const float* __restrict__ Xt, int M, float* __restrict__ Y, int T) {
    __shared__ uint32_t st[4096];
    __shared__ uint32_t ring[kRTiles][kRing];
    const int lane = threadIdx.x & 63, l32 = lane & 31, half = lane >> 5, h8 = threadIdx.x >> 5;
    TileCtx t = block_setup(c, blockIdx.x, st, h8);
    uint32_t* rg = ring[h8];
    Walker z;
    walk_init(z, rg, c, t.tile, l32);
    t.room = c.n_words - 1 - (z.wp - c.words);
    __syncthreads();
    const int S = c.P >> 5;
    // sums of x over this lane's columns (the same for every row): taken while the first row is walked
    float sx[MB];
#pragma unroll
    for (int i = 0; i < MB; ++i) sx[i] = 0.f;
    for (int r = 0; r < T; ++r) {
        if (!(t.has && r < t.nr)) continue;                                // per half-wave
        const int orow = c.perm[t.r0 + r];
        const bool row_ok = orow >= 0 && orow < c.Q;
        float acc[MB], x1[MB], x2[MB];
#pragma unroll
        for (int i = 0; i < MB; ++i) acc[i] = 0.f;
        load_xt<MB>(Xt + (int64_t)l32 * MB, x1);
        load_xt<MB>(Xt + (int64_t)(32 + l32) * MB, x2);
        for (int s0 = 0; s0 < S; s0 += 2) {
            float n1[MB], n2[MB];
            const int sn = s0 + 2 < S ? s0 + 2 : s0;                       // the last pair reloads itself (unused)
            load_xt<MB>(Xt + (int64_t)(sn * 32 + l32) * MB, n1);
            load_xt<MB>(Xt + (int64_t)((sn + 1) * 32 + l32) * MB, n2);
            uint32_t s1, s2;
            walk_pair(z, st, rg, l32, half, t.room, s1, s2);
            const float f1 = (float)s1, f2 = (float)s2;
#pragma unroll
            for (int i = 0; i < MB; ++i) {
                acc[i] = __builtin_fmaf(x1[i], f1, acc[i]);
                acc[i] = __builtin_fmaf(x2[i], f2, acc[i]);
                if (r == 0) sx[i] += x1[i] + x2[i];
                x1[i] = n1[i]; x2[i] = n2[i];
            }
        }
        if (r == 0) {
#pragma unroll
            for (int i = 0; i < MB; ++i) sx[i] = half_sum(sx[i]);
        }
        const double m = row_ok ? (double)c.min_s[orow] : 0.0, ts = row_ok ? (double)c.tau_s[orow] : 0.0;
        const double dr = row_ok ? (double)c.drow[orow] : 0.0;
#pragma unroll
        for (int i = 0; i < MB; ++i) {
            const float a = half_sum(acc[i]);
            if (l32 == 0 && i < M && row_ok)
                Y[(int64_t)i * c.Q + orow] = (float)(ts * ((double)a + dr * (double)sx[i]) + m * (double)sx[i]);
        }
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
int mb_for(int64_t M) { return M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16; }
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
        case 0: hipLaunchKernelGGL(r_decode_kernel<0>, grid, block, 0, s, c, (int)b0, row_base, out_rows, out, T); break;
        case 1: hipLaunchKernelGGL(r_decode_kernel<1>, grid, block, 0, s, c, (int)b0, row_base, out_rows, out, T); break;
        case 2: hipLaunchKernelGGL(r_decode_kernel<2>, grid, block, 0, s, c, (int)b0, row_base, out_rows, out, T); break;
        default: hipLaunchKernelGGL(r_decode_kernel<3>, grid, block, 0, s, c, (int)b0, row_base, out_rows, out, T); break;
    }
    return host::check_launch("qvb8r_decode");
}

extern "C" int64_t qvb8r_gemv_workspace_bytes(int64_t M, int64_t P) {
    if (M < 1 || M > 16 || P <= 0) return 0;
    return (int64_t)mb_for(M) * P * 4;
}

extern "C" int qvb8r_gemv(const void* X, int x_dtype, int64_t M, const qvb8r_core* core, int64_t max_tile_rows, float* Y,
                          void* workspace, int64_t workspace_bytes, void* stream) {
    RCore c;
    if (int rc = check_core("qvb8r_gemv", core, c)) return rc;
    if (M < 1 || M > 16) return host::fail(QVB8_ERR_ARG, "qvb8r_gemv: M=%lld outside 1..16", (long long)M);
    if (x_dtype < QVB8_F32 || x_dtype > QVB8_BF16) return host::fail(QVB8_ERR_ARG, "qvb8r_gemv: bad activation dtype");
    if (max_tile_rows < 1 || max_tile_rows > 0x7fffffff) return host::fail(QVB8_ERR_ARG, "qvb8r_gemv: bad rows-per-tile bound");
    if (c.Q == 0 || c.n_blocks == 0) return QVB8_OK;
    if (!X || !Y) return host::fail(QVB8_ERR_ARG, "qvb8r_gemv: null pointer");
    const int64_t need = qvb8r_gemv_workspace_bytes(M, c.P);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u))
        return host::fail(QVB8_ERR_WORKSPACE, "qvb8r_gemv: needs %lld bytes of 16-byte aligned workspace", (long long)need);
    hipStream_t s = (hipStream_t)stream;
    const int MB = mb_for(M);
    float* Xt = (float*)workspace;
    const int64_t n = (int64_t)c.P * MB;
    hipLaunchKernelGGL(r_transpose_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, X, x_dtype, (int)M, c.P, MB, Xt);
    if (int rc = host::check_launch("qvb8r_gemv transpose")) return rc;
    dim3 grid((unsigned)c.n_blocks), block(kRThreads);
    const int T = (int)max_tile_rows;
    switch (MB) {
        case 1: hipLaunchKernelGGL(r_gemv_kernel<1>, grid, block, 0, s, c, Xt, (int)M, Y, T); break;
        case 2: hipLaunchKernelGGL(r_gemv_kernel<2>, grid, block, 0, s, c, Xt, (int)M, Y, T); break;
        case 4: hipLaunchKernelGGL(r_gemv_kernel<4>, grid, block, 0, s, c, Xt, (int)M, Y, T); break;
        case 8: hipLaunchKernelGGL(r_gemv_kernel<8>, grid, block, 0, s, c, Xt, (int)M, Y, T); break;
        default: hipLaunchKernelGGL(r_gemv_kernel<16>, grid, block, 0, s, c, Xt, (int)M, Y, T); break;
    }
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
