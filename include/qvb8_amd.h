/* qvb8_amd.h -- C ABI of libqvb8_amd.so: QVB8 / QVB8R dequantize-inside-the-matmul on MI355X (gfx950).
 *
 * Every entry point takes raw DEVICE pointers, sizes and a HIP stream (hipStream_t passed as void*; NULL =
 * the default stream), launches asynchronously on that stream on the CURRENT device, never synchronises and
 * never allocates device memory (scratch is a caller-supplied workspace).  Return value: 0 on success, a
 * negative qvb8_status otherwise; qvb8_last_error() gives the message of the calling thread's last failure.
 * Inputs are borrowed and never written.  The functions are re-entrant; the only state is read-once
 * configuration (environment variables) and cached device properties.
 *
 * Each function names the interface of the reference extension it stands in for
 * (src/qv_band/formats/qvb8/backends/cuda_qvb8/qvb8_cuda.cu, pybind table at :2673-2691).
 *
 * Common operands ("the pack"), as the reference's tensors (qvb8_cuda.cu:1424-1431, formats/qvb8/decode.py:30-43):
 *   ids      u8[ids_bytes]  bit-packed row-major ids, LSB first, rows back to back, >= 8 pad bytes at the end,
 *                           base address 4-byte aligned
 *   min_s    f32[Q]         row origin          tau_s  f32[Q]   row step
 *   nbits    u8[Q]          row width, 1..14    bit_off i64[Q]  absolute bit of the row's first id
 *   esc_idx  i64[n_esc]     flat positions q*P+c, ascending     esc_vals f32[n_esc]  exact values
 * value(q, c) = fmaf((float)id, tau_s[q], min_s[q]) in fp32, escapes overwrite.
 *
 * Rows stored in planes (optional, made by a loader; no counterpart in the reference, whose rows are always back to
 * back).  16 rows of ONE width nb in 4..8 (P a multiple of 128) may share a TILE of 16 * P * nb / 8 bytes -- the bytes
 * of the 16 rows, permuted -- laid out so that each 16-byte and each 4 (nb - 4)-byte request of a 64-lane wave of the
 * matrix-core kernels is one contiguous run.  Call the nb dwords that hold ids 32 g .. 32 g + 31 of a row its slice g.
 * The tile is a sequence of P / 128 steps of 256 nb bytes; step s holds slices 4 s .. 4 s + 3 of the 16 rows as
 *   plane A, 64 x 16 bytes:          entry l = r + 16 (g mod 4) holds dwords 0..3 of slice g of row r;
 *   plane B, 64 x 4 (nb - 4) bytes:  entry l holds dwords 4..nb-1 of that slice (empty for nb = 4).
 * Row r of such a tile is marked in its bit_off word: bit 62 set, bits 0..47 = bit offset of the TILE's first byte (a
 * multiple of 32), bits 48..51 = r.  Every entry point that takes a pack reads such rows (qvb8_gemv and the escape
 * corrections id by id); qvb8_mma is told of them with QVB8_MMA_PLANES.  The expert stacks of qvb8_moe_experts do not
 * take them (a marked row there comes out as NaN, like any row whose metadata points outside its buffer).
 */
#ifndef QVB8_AMD_H
#define QVB8_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum qvb8_dtype { QVB8_F32 = 0, QVB8_F16 = 1, QVB8_BF16 = 2 };

enum qvb8_status {
    QVB8_OK = 0,
    QVB8_ERR_ARG = -1,        /* bad argument (shape, range, alignment, null pointer) */
    QVB8_ERR_WORKSPACE = -2,  /* workspace too small */
    QVB8_ERR_LAUNCH = -3,     /* the HIP runtime refused a launch */
    QVB8_ERR_UNSUPPORTED = -4 /* configuration this build does not cover */
};

/* Library identification: ABI version, bumped on any signature change or new entry point (3: row lookup, attention over
 * the banded KV cache, query preparation; 4: qvb8_moe_experts_static; 5: result-type flags of qvb8_mma; 6: rows stored
 * in planes, QVB8_MMA_PLANES; 7: qvb8_mlp, qvb8r_walk_probe).  A binding compares the loaded library's answer
 * with the QVB8_ABI_VERSION it was written for before it makes any other call. */
#define QVB8_ABI_VERSION 7
int qvb8_abi_version(void);
/* Message of the calling thread's most recent failure ("" if none). Valid until that thread's next call. */
const char* qvb8_last_error(void);

/* ---- dense restore ------------------------------------------------------------------------------------- */

/* Dense (Q, P) restore: out[q*P+c] = (T)fmaf(id, tau_s[q], min_s[q]) -- the fp32 result of the fused multiply-add,
 * then that fp32 value rounded to out_dtype (two roundings for fp16 / bf16, as a cast of the reference's fp32 value gives).
 * Bit-exact with the reference restore.  Escapes are NOT applied (see qvb8_scatter_escapes).
 * Replaces: qvb8_decode_launch / qvb8_decode_all(_v3)  qvb8_cuda.cu:535-649; out_dtype QVB8_F16 = ext.decode
 * (:651-699), QVB8_BF16 = ext.decode_bf16 (:1711-1727), QVB8_F32 = the fp32 band value of decode.py:196-209. */
int qvb8_decode(const uint8_t* ids, int64_t ids_bytes, const float* min_s, const float* tau_s,
                const uint8_t* nbits, const int64_t* bit_off, int64_t Q, int64_t P,
                int out_dtype, void* out, void* stream);

/* Row lookup (the embedding read): out[i*P + c] = (T)(min_s[r] + (float)id[r][c] * tau_s[r]) for r = rows[i], the
 * product and the sum rounded separately in fp32 as the reference's lookup does (NOT the single rounding of
 * qvb8_decode), then every escape of row r overwrites its column with (T)esc_vals[e].  rows: i64[n_rows] in device
 * memory, any order, repeats allowed; a row number outside 0..Q-1 gives a row of NaN.  esc_idx ascending flat
 * positions q*P+c of the whole table (may be null when n_esc = 0).  out: (n_rows, P) of out_dtype, 16-byte aligned.
 * Replaces QVBandEmbeddingV8._decode_rows + the escape loop of forward  formats/qvb8/embedding.py:92-119, 121-152
 * (there: torch byte gathers and a host loop over the looked-up rows). */
int qvb8_lookup_rows(const int64_t* rows, int64_t n_rows, const uint8_t* ids, int64_t ids_bytes, const float* min_s,
                     const float* tau_s, const uint8_t* nbits, const int64_t* bit_off, int64_t Q, int64_t P,
                     const int64_t* esc_idx, const float* esc_vals, int64_t n_esc, int out_dtype, void* out,
                     void* stream);

/* out[esc_idx[e]] = (T)esc_vals[e] for every escape: the overwrite the reference does with
 * index_copy_(0, esc_idx, esc_vals.to(dt))  qvb8_cuda.cu:689-697, 1721-1725.  n_out = Q*P (bounds check). */
int qvb8_scatter_escapes(void* out, int out_dtype, int64_t n_out, const int64_t* esc_idx,
                         const float* esc_vals, int64_t n_esc, void* stream);

/* Certificate re-check on the GPU: result[0] = max |restored[i] - original[i]| (as float bits),
 * result[1] = number of elements with |restored - original| >= tau or a non-finite difference.
 * `result` is u32[2] in device memory; the call initialises it.  Differences are taken in fp32 after exact
 * widening.  No counterpart in the reference's extension: the reference certifies at pack time on the CPU
 * (formats/qvb8/module.py:66-78 states the bound); this re-verifies it where the weights live. */
int qvb8_certify(const void* restored, int restored_dtype, const void* original, int original_dtype,
                 int64_t n, float tau, uint32_t* result, void* stream);

/* ---- activations ----------------------------------------------------------------------------------------- */

/* out_f16[i] = fp16(clamp(x[i], -65504, 65504)), NaN kept.  Replaces saturating_half  qvb8_cuda.cu:761-841. */
int qvb8_sat_half(const void* x, int x_dtype, int64_t n, void* out_f16, void* stream);

/* out_f16[i] = fp16(clamp((float)x[i] * scale, -65504, 65504)), NaN kept: the queries of the banded-KV attention with the
 * softmax scale folded in, one launch.  Replaces `(q.float() * scale).clamp_(-65504.0, 65504.0).to(torch.float16)` of
 * attend  kv/fused_attn.py:276-279. */
int qvb8_scale_sat_half(const void* x, int x_dtype, int64_t n, float scale, void* out_f16, void* stream);

/* ---- fused decode + GEMV, M = 1..8 ---------------------------------------------------------------------- */

/* Bytes of workspace qvb8_gemv needs for this shape (0 is possible). */
int64_t qvb8_gemv_workspace_bytes(int64_t M, int64_t Q, int64_t P);

/* Y[m, q] = sum_c sat_half(X[m, c]) * value(q, c), fp32 accumulate, Y is f32 (M, Q) row-major.
 * X is (M, P) row-major in x_dtype, rows 16-byte aligned; 1 <= M <= 8.  The band value is the fp32 one (not
 * narrowed); escapes are corrected after the main pass in ascending order without atomics, so results are
 * reproducible run to run.
 * Replaces: ext.gemv (M=1) qvb8_gemv_forward :1416-1512, ext.gemv_multi qvb8_gemv_multi_forward :1059-1166
 * (kernels qvb8_gemv_multi_v3 :375-453, qvb8_fix_escapes :507-533, qvb8_splitk_combine :463-470). */
int qvb8_gemv(const void* X, int x_dtype, int64_t M,
              const uint8_t* ids, int64_t ids_bytes, const float* min_s, const float* tau_s,
              const uint8_t* nbits, const int64_t* bit_off, int64_t Q, int64_t P,
              const int64_t* esc_idx, const float* esc_vals, int64_t n_esc,
              float* Y, void* workspace, int64_t workspace_bytes, void* stream);

/* ---- fused decode + small-M GEMM on the matrix cores, M = 1..48 (and 49..256, see qvb8_mma) ---------------- */

enum qvb8_mma_flags {
    QVB8_MMA_SATURATE_X = 1,  /* bf16 X is narrowed as saturating_half does (clamp to +-65504, round to fp16, NaN kept) while
                                 it is loaded, and the product runs on fp16 operands: what the fp16 paths of the reference
                                 multiply.  Without it bf16 X is used as it is, on bf16 operands (the reference's bf16
                                 mode).  No effect on fp16 X. */
    QVB8_MMA_Y_F16 = 2,       /* Y is (M, Q) fp16: each result rounded to nearest even from the fp32 value the call would */
    QVB8_MMA_Y_BF16 = 4,      /* otherwise store; likewise bf16.  Only for a weight without escapes (n_esc == 0): the escape
                                 correction adds to fp32 results.  Saves the caller's cast pass over Y (the reference's
                                 operator casts the extension's fp32 result, formats/qvb8/module.py:430-441). */
    QVB8_MMA_PLANES = 8       /* the pack has rows stored in planes (bit 62 of their bit_off, see "rows stored in planes"
                                 above): with a row layout these are the rows of every whole 16-row tile that lies inside
                                 one run of a width 4..8; without one, whatever rows the records mark.  The call then asks
                                 for ids in operand order with non-temporal loads. */
};

/* Row records of the matrix-core path: qvb8_mma_rowinfo_bytes(Q) bytes (24 per row, 8-byte aligned), in tile order
 * (position i describes row perm[i], or row i when perm is NULL): where the row's ids start and how wide they are,
 * then tau_s, min_s and the output row.  Built once per weight (at load) and passed to every qvb8_mma call, so that
 * a call never chases perm -> nbits/bit_off before it can request ids.  Counterpart of the per-weight launch metadata the
 * reference computes once in QVBandLinearV8._mma_order  formats/qvb8/module.py:230-277 (perm, tile_nb). */
int64_t qvb8_mma_rowinfo_bytes(int64_t Q);
int qvb8_mma_prepare(const uint8_t* nbits, const int64_t* bit_off, const float* tau_s, const float* min_s,
                     const int32_t* perm, int64_t Q, int64_t P, int64_t ids_bytes, uint64_t* rowinfo, void* stream);

/* Optional description of a pack whose rows are STORED in tile order from bit 0 of `ids`, back to back, one run per
 * width (what a loader gets by copying the rows once, sorted by width): positions [first_pos[c], first_pos[c+1]) have
 * width nbits[c] and row number perm[pos]; at most three runs.  A host struct, passed by pointer: with it the kernel
 * computes where a row's ids are instead of reading that from the row records, which takes one dependent memory round
 * trip off the start of every call. */
#define QVB8_MMA_MAX_CLASSES 3
typedef struct qvb8_mma_layout {
    int32_t n_classes;
    int32_t first_pos[QVB8_MMA_MAX_CLASSES + 1];
    int32_t nbits[QVB8_MMA_MAX_CLASSES];
} qvb8_mma_layout;

/* Workspace qvb8_mma needs: up to 16 rows of X only when it is called WITHOUT row records (it then builds them itself
 * first); from 17 rows on, when P % 256 == 0, what the workgroup-tiled kernels need (narrowed activations, their sums per
 * column range, partial results of the column ranges). */
int64_t qvb8_mma_workspace_bytes(int64_t M, int64_t Q, int64_t P);

/* Y[m, q] = sum_c X[m, c] * value(q, c), fp32 accumulate on v_mfma 16x16x32, Y f32 (M, Q) row-major.
 * X is (M, P) fp16 or bf16 (x_dtype QVB8_F16 / QVB8_BF16), 16-byte aligned, P % 128 == 0, 1 <= M <= 48 (up to 256 under the
 * conditions below).
 * The ids enter the matrix product exactly (as bias + id in X's own 16-bit format) and tau_s / min_s are applied
 * in fp32 afterwards, so the result equals X times the UN-narrowed fp32 band value, escapes exact.
 * `perm` (i32[Q], position -> row, or NULL): order in which rows are grouped into tiles of 16; rows sorted by
 * width keep each tile on one decode pass (any order is correct).  `rowinfo`: from qvb8_mma_prepare for the same
 * perm, or NULL (then `workspace` must hold qvb8_mma_workspace_bytes).  `layout`: NULL, or the description of rows stored
 * in tile order (needs `rowinfo`).  Widths 4..8 on dword-aligned rows take the fast path; other rows are read element
 * by element.
 * 49 <= M <= 256 runs a workgroup-tiled decode + GEMM (X staged in LDS, v_mfma 32x32x16, column ranges added in a fixed
 * order): it needs `layout` with widths 4..8 (4..7 for bf16 operands), P % 256 == 0 and `workspace`; otherwise
 * QVB8_ERR_UNSUPPORTED / QVB8_ERR_WORKSPACE.  17 <= M <= 48 takes the same kernel when those conditions hold and the
 * workspace is there (it is the faster one from 17 rows on), else the 16-row tile kernel.  Above 48 rows the reference
 * restores the weight and calls a library GEMM (formats/qvb8/module.py:402-457).
 * Replaces: ext.mma_multi  qvb8_mma_multi_forward qvb8_cuda.cu:2566-2671 (kernels :2321-2441, escape fix
 * :2503-2548), and, through the Python module, the M <= 8 GEMV of :1059-1166 when P % 128 == 0. */
int qvb8_mma(const void* X, int x_dtype, int64_t M,
             const uint8_t* ids, int64_t ids_bytes, const float* min_s, const float* tau_s,
             const uint8_t* nbits, const int64_t* bit_off, int64_t Q, int64_t P,
             const int64_t* esc_idx, const float* esc_vals, int64_t n_esc,
             const int32_t* perm, const uint64_t* rowinfo, const qvb8_mma_layout* layout, int flags, float* Y,
             void* workspace, int64_t workspace_bytes, void* stream);

/* Measurement aid: launches a kernel of the matrix-core path's launch shape (blocks x threads, lds_bytes of dynamic LDS,
 * the same 56 bytes of scalar arguments) that does nothing.  A graph of such launches gives the cost of a launch on this
 * machine before any byte moves, the floor under every per-launch figure of the benchmark (bench.py --workload floor).
 * No counterpart in the reference. */
int qvb8_launch_probe(int64_t blocks, int64_t threads, int64_t lds_bytes, void* stream);

/* ---- the MLP of a decoder layer in ONE launch (decode: 1..4 rows) ---------------------------------------------- */

/* Y = down( act(gate(x)) * up(x) ) for 1 <= M <= QVB8_MLP_MAX_ROWS rows of X, as one kernel: the gate+up product, the
 * activation and the down product run in one grid of one workgroup per CU (all resident at once), and H = act(gate) * up
 * is handed from its producers to the down rows' workgroups INSIDE the grid, through `workspace`, while the down
 * weight's first ids are already on their way.  Launched separately the two products each pay a launch's fixed cost;
 * this call pays it once.
 * Values are those of the separate calls and the caller's elementwise code between them: gate and up results rounded to
 * `mid_dtype` (QVB8_F32 = not rounded), SiLU computed in fp32 and rounded to it, the product rounded to it, then narrowed
 * to saturated fp16 (what qvb8_mma's QVB8_MMA_SATURATE_X does to the down product's input); Y rounded to `y_dtype`.
 *
 * qvb8_mlp_init, once per block (at load): checks the two weights, fills `plan` (a host struct the caller keeps) and
 * launches a small kernel that zeroes `workspace` and writes the block's description into it.  Both weights: rows stored
 * in planes in position order with a row layout (see qvb8_mma; widths 4..8, every run of one width whole tiles, no
 * escapes), row records from qvb8_mma_prepare for the same order.  gate+up is ONE pack of 2 * inter rows (rows
 * 0..inter-1 gate, the rest up) whose position order goes unit by unit: positions 32 u .. 32 u + 15 hold 16 gate rows,
 * 32 u + 16 .. 32 u + 31 the up rows of the same outputs (position 32 u + 16 + r is row inter + j when position 32 u + r is
 * row j; a pair that breaks this gives NaN for that output).  down: out_features rows of inter columns.
 * hidden % 128 == 0, inter % 128 == 0, out_features % 16 == 0; anything else: QVB8_ERR_UNSUPPORTED (call the products
 * separately).  The weights' buffers must stay where they are while the plan is in use.
 * `workspace`: qvb8_mlp_workspace_bytes(inter) bytes of device memory, 16-byte aligned, the library's from qvb8_mlp_init
 * on: it carries the description and the state of the hand-over from call to call, so calls that share it must not
 * overlap (one workspace per block, or per stream).  Its second word (int32 [1]) is the error word, sticky: nonzero once a
 * call's bounded wait for H ran out (QVB8_MLP_WAIT_US microseconds, default 20000; that call's Y is NaN) -- it can only run out when the grid is not resident as a whole, e.g. while
 * other kernels hold CUs for that long.
 *
 * qvb8_mlp, per call: X (M, hidden) fp16, or bf16 narrowed like QVB8_MMA_SATURATE_X, 16-byte aligned; Y (M,
 * out_features).  `act`: QVB8_MLP_SILU_GATED.  QVB8_MLP_TEST_STALE_TAG ORed in makes the producers label H as another
 * call's, so that the wait runs out: for tests of that path only.
 * No single counterpart in the reference, which launches the products separately (ext.gemv / ext.mma_multi,
 * qvb8_cuda.cu:1059-1166, 2566-2671, with the elementwise code of decode/fused_pointwise.py:60-67, 194-204 between them)
 * and removes the launch cost from the host's side by replaying the MLP as a graph (install_mlp_graphs
 * formats/qvb8/moe_graph.py:145-178). */
#define QVB8_MLP_MAX_ROWS 4
enum qvb8_mlp_act { QVB8_MLP_SILU_GATED = 0, QVB8_MLP_TEST_STALE_TAG = 0x100 };
typedef struct qvb8_mlp_plan {
    int64_t hidden, inter, out_features;
    int64_t magic;                          /* set by qvb8_mlp_init, checked by qvb8_mlp */
} qvb8_mlp_plan;
int64_t qvb8_mlp_workspace_bytes(int64_t inter);
int qvb8_mlp_init(int64_t hidden, int64_t inter, int64_t out_features,
                  const uint8_t* gu_ids, int64_t gu_ids_bytes, const uint64_t* gu_rowinfo, const qvb8_mma_layout* gu_layout,
                  const uint8_t* dn_ids, int64_t dn_ids_bytes, const uint64_t* dn_rowinfo, const qvb8_mma_layout* dn_layout,
                  void* workspace, int64_t workspace_bytes, qvb8_mlp_plan* plan, void* stream);
int qvb8_mlp(const qvb8_mlp_plan* plan, const void* X, int x_dtype, int64_t M, int act, int mid_dtype,
             void* Y, int y_dtype, void* workspace, void* stream);

/* ---- routed MoE expert stack (decode: a few tokens, top-k experts each) ---------------------------------------- */

enum qvb8_moe_act {
    QVB8_MOE_SILU_GATED = 0,  /* up rows = gate (first half) then up: H[i] = silu(Y[i]) * Y[I + i], Q_up == 2 * P_dn */
    QVB8_MOE_RELU2 = 1,       /* non-gated: H[i] = max(Y[i], 0)^2, Q_up == P_dn */
    /* Optional statements about a stack, ORed to the activation (a loader that stores the stack itself can make them true;
     * no counterpart in the reference).  "Regular": every row of the stack has the width nbits[0], and row q of expert e
     * starts at bit  bit_off[0] + e * (bit_off[Q] - bit_off[0]) + q * P * nbits[0].  The matrix-core paths (1..16 tokens)
     * then work a row's place out instead of reading nbits / bit_off, which takes one dependent memory trip out of every
     * launch; results are bit for bit those without the flag (also when the rows do not start on dword boundaries: they
     * are then read id by id, as without the flag).  A stack for which the statement is false gives wrong results (never
     * an access outside the ids buffer). */
    QVB8_MOE_UP_REGULAR = 0x100,
    QVB8_MOE_DOWN_REGULAR = 0x200
};

/* Bytes of workspace qvb8_moe_experts needs (routing plan + fp32 H (pairs, P_dn) + fp32 Yd (pairs, Q_dn)). */
int64_t qvb8_moe_workspace_bytes(int64_t tokens, int64_t topk, int64_t n_experts, int64_t Q_up, int64_t P_dn, int64_t Q_dn);

/* out[t] = sum_j w[t][j] * W_dn[e] . act(W_up[e] . sat_half(X[t])),  e = idx[t][j]; out is (tokens, Q_dn) in out_dtype.
 * Stacked layout of the reference (QVBandExpertsV8.build_stack, formats/qvb8/backends_experts.py:145-195): per
 * projection ONE ids buffer (16-byte aligned, every expert's ids concatenated) and (n_experts, Q) row metadata with
 * bit offsets made global; experts carry no escapes.  idx i64 (tokens, topk), w f32 (tokens, topk), X (tokens, P_up)
 * in x_dtype; P_up and P_dn multiples of 32; Q_dn == P_up.  No host round trip.  An index outside 0..n_experts-1 gives
 * NaN: in every output row of the token that holds it, and in the whole output on the paths that group by expert.
 * Up to 16 tokens with topk <= 8, fp16 / bf16 X, P_up and P_dn multiples of 128 up to 4096 and Q_dn a multiple of 16 run
 * on the matrix cores, H handed over as saturated fp16:
 *   1 .. 6 tokens: two launches, every token a problem of its own (slot j = expert idx[t][j]; an expert is read once per
 *     token that chose it); the down projection adds the slots up with their routing weights;
 *   7 .. 16 tokens: four launches (plan, up, down, combine): the (token, choice) pairs are grouped by expert, the tokens
 *     that chose an expert are the token rows of one MFMA operand, and every selected expert is read ONCE however many
 *     tokens chose it.  An expert's pairs are the rows of one operand, as many as there are tokens: an expert with more
 *     pairs than that (only possible when a token lists it twice) makes the whole output NaN instead of a sum with pairs
 *     missing; the other paths take such lists.
 * Everything else takes the general path (four launches, H in fp32, an expert read once for up to 8 of its tokens).
 * Replaces: ext.moe_experts  qvb8_moe_experts_forward qvb8_cuda.cu:937-992 (kernels qvb8_moe_gemv :860-907,
 * qvb8_moe_act :910-918, qvb8_moe_combine :924-935) with act QVB8_MOE_SILU_GATED, and ext.moe_experts_relu2
 * qvb8_moe_experts_relu2_forward :1002-1055 with QVB8_MOE_RELU2. */
int qvb8_moe_experts(const void* X, int x_dtype, int64_t tokens, const int64_t* idx, const float* w, int64_t topk,
                     int64_t n_experts,
                     const uint8_t* up_ids, int64_t up_ids_bytes, const float* up_min, const float* up_tau,
                     const uint8_t* up_nb, const int64_t* up_off, int64_t Q_up, int64_t P_up,
                     const uint8_t* dn_ids, int64_t dn_ids_bytes, const float* dn_min, const float* dn_tau,
                     const uint8_t* dn_nb, const int64_t* dn_off, int64_t Q_dn, int64_t P_dn,
                     int act, void* out, int out_dtype, void* workspace, int64_t workspace_bytes, void* stream);

/* qvb8_moe_experts for callers that cannot allocate device memory or bring a workspace: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  Same operands, same kernels and the same results bit for bit; the
 * workspace is an array of QVB8_MOE_STATIC_SCRATCH_BYTES inside the library's device image (one copy per GPU, held until
 * the process ends).  A call that would need more (qvb8_moe_workspace_bytes) fails with QVB8_ERR_WORKSPACE: 2 MiB covers
 * 16 tokens x top-8 of a 2048 / 768 expert stack.  The call allocates and frees nothing.  All calls on one GPU share the
 * array: calls that overlap on one GPU (two streams, two threads) race; calls in stream order do not.  The first call on a
 * device looks the array's address up (make that call outside a stream capture).
 * No counterpart in the reference, whose extension allocates its temporaries with torch on every call
 * (qvb8_cuda.cu:958-960). */
#define QVB8_MOE_STATIC_SCRATCH_BYTES (2 * 1024 * 1024)
int qvb8_moe_experts_static(const void* X, int x_dtype, int64_t tokens, const int64_t* idx, const float* w, int64_t topk,
                            int64_t n_experts,
                            const uint8_t* up_ids, int64_t up_ids_bytes, const float* up_min, const float* up_tau,
                            const uint8_t* up_nb, const int64_t* up_off, int64_t Q_up, int64_t P_up,
                            const uint8_t* dn_ids, int64_t dn_ids_bytes, const float* dn_min, const float* dn_tau,
                            const uint8_t* dn_nb, const int64_t* dn_off, int64_t Q_dn, int64_t P_dn,
                            int act, void* out, int out_dtype, void* stream);

/* ---- QVB8R: the same band ids, rANS-coded (32 interleaved streams per tile) ---------------------------------------- */

/* What every QVB8R kernel walks ("core" of the reference: qvb8r_cuda.cu:333-344), all device pointers:
 *   words     u32[n_words]   the streams of all tiles back to back, then >= 2048 zero words (n_words counts the pad)
 *   tile_off  i64[n_tiles+1] first word of each tile            states  u64[n_tiles][32]  initial rANS states
 *   tiles     i64[n_tiles][3] class, first sorted row, rows     blocks  i32[n_blocks][3]  class, first tile, tiles (<= 8)
 *   tab       u32[n_classes][4096] slot tables: symbol | offset << 11 | (freq - 1) << 22
 *   perm      i32[Q] sorted row -> original row                 min_s, tau_s f32[Q], drow i32[Q]  by original row
 * id = symbol + drow[row]; value = fmaf((float)id, tau_s[row], min_s[row]).  P % 128 == 0. */
typedef struct qvb8r_core {
    const uint32_t* words; int64_t n_words;
    const int64_t* tile_off; const uint64_t* states; const int64_t* tiles; int64_t n_tiles;
    const int32_t* blocks; int64_t n_blocks;
    const uint32_t* tab; int64_t n_classes;
    const int32_t* perm; const float* min_s; const float* tau_s; const int32_t* drow;
    int64_t Q, P;
} qvb8r_core;

/* Dense rows of blocks [b0, b0 + nb): out_dtype 0 fp32 / 1 fp16 / 2 bf16 values (rounded once), 3 the ids as int16.
 * row_base < 0: a row lands at its ORIGINAL index (out is the whole (Q, P) weight); row_base >= 0: at its sorted
 * position - row_base (a contiguous block range fills a compact chunk).  out has out_rows rows of P.  Escapes are not
 * applied.  max_tile_rows = most rows in any tile (the file's T).  Bit-exact with the QVB8 restore of the same ids.
 * Replaces: ext.decode  qvb8r_decode qvb8r_cuda.cu:279-306 (wrapper :398-424) and ext.ids (:426-444). */
int qvb8r_decode(const qvb8r_core* core, int64_t max_tile_rows, int out_dtype, int64_t b0, int64_t nb, int64_t row_base,
                 void* out, int64_t out_rows, void* stream);

/* The rows of a LIST of blocks (block numbers of the schedule in `core`, i32 in device memory, any order, repeats
 * allowed): block j of the list fills rows [j * 8 * max_tile_rows, (j + 1) * 8 * max_tile_rows) of `out`, row r of the
 * block's tile h at row (j * 8 + h) * max_tile_rows + r; slots of tiles the block does not have, or rows a tile does not
 * have, are left untouched.  out_dtype as qvb8r_decode; out has out_rows >= n_list * 8 * max_tile_rows rows of P.  A block
 * number outside the schedule writes nothing.  What a lookup of scattered rows (an embedding read) gathers from.
 * Replaces the per-row walk of embed_rows  qvb8r_cpu.cpp:13-51 (there on the CPU, one tile prefix per looked-up row). */
int qvb8r_decode_blocks(const qvb8r_core* core, int64_t max_tile_rows, int out_dtype, const int32_t* block_list,
                        int64_t n_list, void* out, int64_t out_rows, void* stream);

/* Bytes of workspace qvb8r_gemv needs: 16 for M = 1 (X is read in place); for M = 2..48 the activations packed as
 * fp16 hi + lo planes in matrix-core operand order plus one sum and one scale exponent per row. */
int64_t qvb8r_gemv_workspace_bytes(int64_t M, int64_t P);

/* Y[m, q] = sum_c X[m, c] * value(q, c) for M = 1..48, fp32 accumulate, Y f32 (M, Q) row-major, every row written.
 * M = 1: X in x_dtype is used in fp32 as it is.  M >= 2: one walk of the stream serves all rows on the matrix cores;
 * each row of X is scaled by a power of two into fp16 range and used as fp16 hi + lo (fp32 X: 22 significant bits;
 * fp16 / bf16 X: exact), the symbols are exact fp16 integers, so the product differs from fp32 arithmetic only by the
 * split of fp32 activations.  A row of X with a non-finite element gives non-finite outputs for that row.
 * Escapes are NOT corrected (qvb8r_fix_escapes).
 * Replaces: ext.gemv  qvb8r_gemv qvb8r_cuda.cu:88-131, ext.multi  qvb8r_multi :153-194 and ext.tc  qvb8r_tc :199-272
 * (which multiplies fp16-rounded weights; this one keeps the fp32 band value). */
int qvb8r_gemv(const void* X, int x_dtype, int64_t M, const qvb8r_core* core, int64_t max_tile_rows, float* Y,
               void* workspace, int64_t workspace_bytes, void* stream);

/* Measurement aid: the launch of qvb8r_gemv for one row of X with the activations not read and the two multiply-adds per
 * symbol pair replaced by an exclusive-or of the symbols -- the rANS walk alone (slot lookups, 64-bit state updates, word
 * hand-out, ring reads), the ceiling of the fused kernel on this hardware.  Y (f32, Q) receives values without meaning.
 * No counterpart in the reference. */
int qvb8r_walk_probe(const qvb8r_core* core, int64_t max_tile_rows, float* Y, void* stream);

/* Y[m, uq[u]] += sum_{e in [ptr[u], ptr[u+1])} X[m, ec[e]] * ed[e]: one thread per (m, u), stored order, no atomics.
 * Replaces: ext.fix_escapes  qvb8r_fix_escapes qvb8r_cuda.cu:311-320. */
int qvb8r_fix_escapes(const void* X, int x_dtype, int64_t M, const int64_t* uq, const int64_t* ptr, const int64_t* ec,
                      const float* ed, int64_t U, float* Y, int64_t Q, int64_t P, void* stream);

/* Attention of query rows over a banded KV cache whose keys and values stay ids in memory: per split of the key tiles
 * the unnormalised result and the softmax state, which the caller combines (o * exp(m - max m) summed, over the
 * likewise weighted l).
 *   q      fp16, (tokens, q heads, head_dim) with strides sq_r / sq_h in elements, head_dim contiguous; row r of a kv
 *          head is token r / G, q head h * G + r % G; the token's position is q_pos0 + r / G
 *   ki, vi ids, (capacity, kv heads, head_dim) with strides s_n / s_h in ids; id_bytes = 1 (uint8) or 2 (uint16)
 *   kmid, kstep, vmid, vstep  f32 (segments, kv heads, head_dim) contiguous; kc, vc f32 (segments, kv heads):
 *          k = fp16(kmid + kstep * ((float)id - kc)), one fused multiply-add in fp32; v likewise
 *   ts, tl, tseg  i32[n_tiles]: first key, length (1..32) and segment of each tile, first keys ascending; split s
 *          takes tiles s * tps .. min((s + 1) * tps, n_tiles) - 1; a key at position p counts for a row when
 *          p <= the row's position
 *   o (n_splits, kv heads, n_rows, head_dim), m and l (n_splits, kv heads, n_rows)  f32, written completely
 *          (a row that sees no key of a split: m = -inf, l = 0, o = 0)
 * S = q k^T is accumulated in fp32 from fp16 operands, multiplied by `scale`; the probabilities exp(s - m) are rounded
 * to fp16 before they are summed into l and multiplied with v (fp32 accumulate).  head_dim 128 or 256.
 * Replaces: ext.fwd  qvattn_fwd kv/cuda_attn/qvattn_cuda.cu:97-255, host :257-287 (called from attend,
 * kv/fused_attn.py:246-316, which also does the combination). */
int qvb8_attn_fwd(const void* q, int64_t sq_r, int64_t sq_h, const void* ki, const void* vi, int id_bytes,
                  int64_t s_n, int64_t s_h, const float* kmid, const float* kstep, const float* vmid,
                  const float* vstep, const float* kc, const float* vc, const int32_t* ts, const int32_t* tl,
                  const int32_t* tseg, int64_t n_tiles, float* o, float* m, float* l, int64_t n_splits,
                  int64_t n_rows, int64_t n_kv_heads, int64_t head_dim, int64_t q_pos0, int64_t tps,
                  double scale, int64_t G, void* stream);

/* Combination of the splits of qvb8_attn_fwd, one launch: with top = max over splits of m (0 when no split saw a key)
 * and w_s = exp(m_s - top):  total = sum_s l_s w_s,  out = sum_s o_s w_s / max(total, 1e-30),
 * lse = top + log(total) when total > 0, else -inf.  o / m / l as qvb8_attn_fwd writes them; out (tokens, q heads,
 * head_dim) and lse (tokens, q heads) f32 contiguous, row r of kv head h going to token r / G, q head h * G + r % G.
 * head_dim a multiple of 4; o and out 16-byte aligned.  l may be null: every l_s is then 1, which merges NORMALISED partial
 * results by their log-sum-exp (m = lse_s) -- the banded part and the dense residual of a layer, or the blocks of a
 * tiered cache (_merge_lse / _merge_lse_all  kv/fused_attn.py:769-788; n_kv_heads = 1, G = n_rows keeps the row order).
 * Replaces the torch expressions of attend  kv/fused_attn.py:302-316. */
int qvb8_attn_combine(const float* o, const float* m, const float* l, int64_t n_splits, int64_t n_kv_heads,
                      int64_t n_rows, int64_t head_dim, int64_t G, float* out, float* lse, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* QVB8_AMD_H */
