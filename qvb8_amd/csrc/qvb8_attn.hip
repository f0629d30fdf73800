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
// Shape of this kernel (gfx950): 128 threads = 2 waves per workgroup, 16 query rows, 32 keys per tile.
//   * ids are requested one tile ahead into registers: a wave reads whole key rows (64 lanes x 4 ids = 256 channels),
//     every thread keeps the same four channels for all its keys, so it holds 4 + 4 constants per operand;
//   * restored K goes to LDS as [key][channel], restored V as [channel][key] (a thread owns 4 keys x 4 channels, so the
//     transposition is free) with the 8-byte cells of a row swizzled by the channel group;
//   * S = Q K^T: wave w takes keys 16 w .. 16 w + 15 (v_mfma_f32_16x16x16_f16, Q kept in registers as the A operand);
//   * both waves do the softmax of all 16 rows from S in LDS (same inputs, same results; no state in LDS) in the
//     A-operand layout of the second product, so P needs no trip through LDS;
//   * O += P V: wave w owns half of the output channels.
#include <hip/hip_runtime.h>
#include <math.h>
#include <algorithm>
#include <stdint.h>

#include "qvb8_amd.h"
#include "qvb8_host.h"

namespace qvb8 {
namespace {

typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef float f4_t __attribute__((ext_vector_type(4)));

constexpr int kRows = 16;          // query rows per workgroup
constexpr int kKeys = 32;          // keys per tile (the table's tiles are never longer)
constexpr int kAttnThreads = 128;
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

template <int D, typename T>
__global__ __launch_bounds__(kAttnThreads) void attn_kernel(const AttnArgs a) {
    constexpr int CG = D / 4;                  // channel groups (four channels each) of a key
    constexpr int KSTEP = kAttnThreads / CG;   // key groups (four keys each) that one pass of the workgroup covers
    constexpr int UNITS = D / 64;              // (4 keys x 4 channels) units per thread and tile
    constexpr int KROW = D + 8;                // halfs per key in LDS
    constexpr int NF = D / 32;                 // 16-channel output fragments per wave
    using QD = Quad<T>;
    using U = typename QD::type;
    __shared__ __align__(16) _Float16 Ks[kKeys * KROW];
    __shared__ __align__(16) _Float16 Vt[D * kKeys];
    __shared__ __align__(16) float Ss[kRows * kSStride];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n16 = lane & 15, kg = lane >> 4;
    const int h = blockIdx.x, sp = blockIdx.y, row0 = blockIdx.z * kRows;
    const int cg = tid % CG, kgp0 = tid / CG;

    // the lane's query row as the A operand of S = Q K^T: Q[row][16 ks + 4 kg .. + 3]
    const int row = row0 + n16;
    const bool row_ok = row < a.n_rows;
    const int qpos = a.q_pos0 + (row_ok ? row / a.G : 0);
    h4_t qa[D / 16];
    {
        const int rr = row_ok ? row : 0;
        const uint16_t* qp = a.q + (int64_t)(rr / a.G) * a.sq_r + (int64_t)(h * a.G + rr % a.G) * a.sq_h + 4 * kg;
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) {
            const h4_t v = *reinterpret_cast<const h4_t*>(qp + 16 * ks);
            qa[ks] = row_ok ? v : h4_t{0, 0, 0, 0};
        }
    }
    const int qmax = a.q_pos0 + (min(row0 + kRows, a.n_rows) - 1) / a.G;      // last position any row of the block sees

    const T* ki = reinterpret_cast<const T*>(a.ki) + (int64_t)h * a.s_h + 4 * cg;
    const T* vi = reinterpret_cast<const T*>(a.vi) + (int64_t)h * a.s_h + 4 * cg;
    U rk[UNITS][4], rv[UNITS][4];
    // ids of tile t into registers; keys past the tile's length re-read its last key (never used)
    auto fetch = [&](int t) {
        const int start = a.ts[t], nlen = a.tl[t];
#pragma unroll
        for (int u = 0; u < UNITS; ++u)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int key = max(0, min(4 * (kgp0 + KSTEP * u) + j, nlen - 1));
                const int64_t off = (int64_t)(start + key) * a.s_n;
                rk[u][j] = *reinterpret_cast<const U*>(ki + off);
                rv[u][j] = *reinterpret_cast<const U*>(vi + off);
            }
    };

    const int t0 = (int)min((int64_t)sp * a.tps, (int64_t)a.n_tiles), t1 = (int)min((int64_t)t0 + a.tps, (int64_t)a.n_tiles);
    float m_run = -INFINITY, l_run = 0.f;
    f4_t acc[NF];
#pragma unroll
    for (int f = 0; f < NF; ++f) acc[f] = f4_t{0.f, 0.f, 0.f, 0.f};

    bool have = t0 < t1 && a.ts[t0] <= qmax;            // tiles ascend: behind the first masked one all are masked
    if (have) fetch(t0);
    for (int t = t0; have; ++t) {
        const int start = a.ts[t], nlen = a.tl[t], seg = a.tseg[t];
        {
            const int64_t pb = ((int64_t)seg * a.nhkv + h) * D + 4 * cg;
            const float4 kmid = *reinterpret_cast<const float4*>(a.kmid + pb), kstep = *reinterpret_cast<const float4*>(a.kstep + pb);
            const float4 vmid = *reinterpret_cast<const float4*>(a.vmid + pb), vstep = *reinterpret_cast<const float4*>(a.vstep + pb);
            const float kc = a.kc[seg * a.nhkv + h], vc = a.vc[seg * a.nhkv + h];
            const float km[4] = {kmid.x, kmid.y, kmid.z, kmid.w}, ks_[4] = {kstep.x, kstep.y, kstep.z, kstep.w};
            const float vm[4] = {vmid.x, vmid.y, vmid.z, vmid.w}, vs_[4] = {vstep.x, vstep.y, vstep.z, vstep.w};
#pragma unroll
            for (int u = 0; u < UNITS; ++u) {
                const int kgp = kgp0 + KSTEP * u;
                h4_t vcell[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int key = 4 * kgp + j;
                    const bool live = key < nlen;
                    h4_t kv;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const float kf = __builtin_fmaf(ks_[c], QD::id(rk[u][j], c) - kc, km[c]);
                        const float vf = __builtin_fmaf(vs_[c], QD::id(rv[u][j], c) - vc, vm[c]);
                        kv[c] = live ? (_Float16)kf : (_Float16)0.f;
                        vcell[c][j] = live ? (_Float16)vf : (_Float16)0.f;
                    }
                    *reinterpret_cast<h4_t*>(Ks + key * KROW + 4 * cg) = kv;
                }
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    *reinterpret_cast<h4_t*>(Vt + (4 * cg + c) * kKeys + 4 * (kgp ^ (cg & 7))) = vcell[c];
            }
        }
        __syncthreads();
        const bool more = t + 1 < t1 && a.ts[t + 1] <= qmax;
        if (more) fetch(t + 1);

        // ---- S = Q K^T for this wave's 16 keys ----
        {
            f4_t s = {0.f, 0.f, 0.f, 0.f};
            const _Float16* kp = Ks + (16 * wave + n16) * KROW + 4 * kg;
#pragma unroll
            for (int ks = 0; ks < D / 16; ++ks)
                s = __builtin_amdgcn_mfma_f32_16x16x16f16(qa[ks], *reinterpret_cast<const h4_t*>(kp + 16 * ks), s, 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 4; ++e) Ss[(4 * kg + e) * kSStride + 16 * wave + n16] = s[e];
        }
        __syncthreads();

        // ---- softmax of row n16 over the tile: this lane holds keys 16 kk + 4 kg + i ----
        h4_t pa[2];
        float alpha;
        {
            float sv[8], mx = -INFINITY;
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                const f4_t s4 = *reinterpret_cast<const f4_t*>(Ss + n16 * kSStride + 16 * kk + 4 * kg);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int n = 16 * kk + 4 * kg + i;
                    const bool ok = row_ok && n < nlen && start + n <= qpos;
                    sv[4 * kk + i] = ok ? s4[i] * a.scale : -INFINITY;
                    mx = fmaxf(mx, sv[4 * kk + i]);
                }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16));
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run, mx);
            const float m_safe = m_new == -INFINITY ? 0.f : m_new;
            float sum = 0.f;
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float x = sv[4 * kk + i];
                    const _Float16 p = (_Float16)(x == -INFINITY ? 0.f : __expf(x - m_safe));
                    pa[kk][i] = p;
                    sum += (float)p;                    // the rounded p, as the second product sees it
                }
            sum += __shfl_xor(sum, 16);
            sum += __shfl_xor(sum, 32);
            alpha = m_run == -INFINITY ? 0.f : (m_new == m_run ? 1.f : __expf(m_run - m_safe));
            l_run = l_run * alpha + sum;
            m_run = m_new;
        }
        // ---- O = alpha O + P V; the accumulator holds rows 4 kg + e of channel n16 of each fragment ----
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
            float ae[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) ae[e] = __shfl(alpha, 4 * kg + e);
#pragma unroll
            for (int f = 0; f < NF; ++f)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[f][e] *= ae[e];
        }
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int f = 0; f < NF; ++f) {
                const int ch = wave * (D / 2) + 16 * f + n16;
                const h4_t b = *reinterpret_cast<const h4_t*>(Vt + ch * kKeys + 4 * ((4 * kk + kg) ^ ((ch >> 2) & 7)));
                acc[f] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa[kk], b, acc[f], 0, 0, 0);
            }
        __syncthreads();                                  // the tile in LDS is free again
        have = more;
    }

    const int64_t base = ((int64_t)sp * a.nhkv + h) * a.n_rows;
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int r = row0 + 4 * kg + e;
            if (r < a.n_rows) a.o[(base + r) * D + wave * (D / 2) + 16 * f + n16] = acc[f][e];
        }
    if (wave == 0 && kg == 0 && row_ok) {
        a.m[base + row] = m_run;
        a.l[base + row] = l_run;
    }
}

template <int D, typename T>
int launch_attn(const AttnArgs& a, int64_t n_splits, hipStream_t s) {
    const dim3 grid((unsigned)a.nhkv, (unsigned)n_splits, (unsigned)((a.n_rows + kRows - 1) / kRows));
    hipLaunchKernelGGL((attn_kernel<D, T>), grid, dim3(kAttnThreads), 0, s, a);
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
