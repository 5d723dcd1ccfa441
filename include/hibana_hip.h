/*
 * hibana_hip.h - C ABI of the MI355X (gfx950) quantized-weight linear / MoE expert kernels.
 *
 * Plain pointers and sizes only. Every pointer is a DEVICE pointer unless its comment says "host". The caller owns
 * every buffer, including scratch ("workspace"); the library allocates nothing. `stream` is a hipStream_t passed as
 * void* (NULL = the default stream). Every function enqueues work on `stream` and returns without synchronizing;
 * kernels use no floating-point atomics, so results are bitwise repeatable and the calls are graph-capturable.
 * Return value: HB_OK (0) or a negative HB_E* code; hb_error_string() names it.
 *
 * Workspaces. A workspace begins with a few words that no launch initializes: arrival counters (of the launch whose
 * last workgroup plans a routed call; of the tiles whose K several workgroups share) and a fault word. The caller
 * hands a workspace over with its first min(bytes, HB_WORKSPACE_ZERO_BYTES) bytes ZERO, once, before its first use
 * (hipMemsetAsync, or hb_workspace_reset); every call that completes leaves the counters zero again, so one workspace
 * serves any number of calls one after the other. The library keeps no counters of its own: calls that are in flight
 * together (different streams, or graphs replayed side by side) must each have a workspace of their own and then share
 * nothing; two calls in flight on ONE workspace race on everything in it. A call that was aborted midway (a reset
 * device, a killed launch) may leave a counter standing: hb_workspace_reset puts the workspace back in service.
 *
 * Citations "ref:" give the interface of the reference (sharar-project/hibana, paths relative to its tree) that the
 * entry point replaces.
 */
#ifndef HIBANA_HIP_H
#define HIBANA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  HB_OK = 0,
  HB_EINVAL = -1,     /* a shape, alignment or flag the kernels do not take (the Python layer raises ValueError):
                         activations, tile layouts and workspaces must lie on 16-byte boundaries, FP32 / int32 arrays on
                         4-byte ones (any allocator's blocks do; the calls check) */
  HB_ENULL = -2,      /* a required pointer is NULL */
  HB_EWORKSPACE = -3, /* workspace smaller than hb_*_workspace_bytes() says */
  HB_ELAUNCH = -4,    /* the HIP runtime refused a launch (hipGetLastError is left set for the caller) */
  HB_ESCRATCH = -5    /* hb_w3_moe_layer_static: the call needs more scratch than HB_STATIC_SCRATCH_BYTES */
};

/* Library version (major * 1000 + minor). */
int hb_version(void);
const char* hb_error_string(int code);

/* The bytes at a workspace's head that must be zero before its first use (or all of it, if it is smaller). */
#define HB_WORKSPACE_ZERO_BYTES (1u << 20)

/* Bits of a workspace's fault word. HB_FAULT_WAIT: a workgroup of a launch that runs a routed call's fc1 and fc2
 * together waited for its slot's fc1 workgroups longer than the bound allows (about a second) - it has stored nothing,
 * so rows of the call's output are stale. The launch relies on the hardware starting a grid's workgroups in index
 * order; the bound and this bit are what happens should that ever fail. */
enum { HB_FAULT_WAIT = 1 };

/* Zero a workspace's head (its first min(bytes, HB_WORKSPACE_ZERO_BYTES) bytes: the arrival counters and the fault
 * word) with a small kernel on `stream` - capturable, no hipMemset. For a new workspace, and to put one back in
 * service after a fault or an aborted call. workspace == NULL: the library's own scratch (hb_w3_moe_layer_static).
 * No counterpart in the reference (its kernels' split-K counters live in a torch tensor it zeroes at allocation,
 * hibana/kernels/csrc/w3_gemm.cu:230-240). */
int hb_workspace_reset(void* workspace, size_t workspace_bytes, void* stream);

/* Copy a workspace's fault word (0: no fault; HB_FAULT_* bits otherwise; sticky until hb_workspace_reset) to *status
 * (HOST memory) behind the work already enqueued on `stream`. wait != 0: synchronize the stream before returning, so
 * *status is valid on return; wait == 0: only enqueue the copy (*status is valid once the caller has synchronized;
 * pinned host memory keeps the copy asynchronous). workspace == NULL: the library's own scratch. The word means
 * something in the workspaces of the routed calls (hb_w3_moe*, hb_nvfp4_moe, hb_latent_*); other workspaces hold zero
 * there. No counterpart in the reference. */
int hb_workspace_status(const void* workspace, int32_t* status, int wait, void* stream);

#ifndef HB_NO_DEBUG_HOOKS  /* a build with -DHB_NO_DEBUG_HOOKS exports none of hb_tune / hb_debug_*: a serving process cannot race on them */

/* Tuning knobs for experiments and tests; value 0 restores the built-in choice. "w3_ksplit" / "w3_nbw",
 * "moe_fc1_ksplit" / "moe_fc1_nbw", "moe_fc2_ksplit" / "moe_fc2_nbw", "nvfp4_ksplit" / "nvfp4_nbw": K splits and 64-row
 * blocks per workgroup (their product at most 16); "w3_tile" / "nvfp4_tile": 1 forces the MFMA tile kernel, 2 the weight
 * stream; "w3_few" / "nvfp4_few": 2 switches off the stream's body for slots of few rows (W3: at most four, NVFP4: at
 * most eight); "moe_one": 2 switches off the single launch that does one token's fc2 and combine; "moe_fused": 2 runs a
 * routed call's fc1 and fc2 as two launches; "moe_lag": the slots fc2 lags fc1 by in their common launch; "moe_split":
 * 1 gives fc1's slots of at most two rows a two-plane E4M3 form of x (FP8 matrix cores; 4e-4 of the norm); "route_plan": 2 keeps
 * routing and plan in separate launches; "nvfp4_tile_ks": the workgroups that share a tile's K in hb_nvfp4_gemm_ws.
 * Returns HB_EINVAL for an unknown key or a value out of range. The knobs are process-wide relaxed atomics: setting one
 * while another thread launches is a race-free read of either value, not a per-call setting. */
int hb_tune(const char* key, int value);

/* Measurement hook (no counterpart in the reference): `events` are hipEvent_t handles the caller created, taken in
 * (start, stop) pairs: each kernel the next calls launch carries the next pair, and the runtime stamps the two events
 * with that kernel's own begin and end (hipEventElapsedTime(start, stop) is the kernel's duration). A routed call
 * launches plan, fc1 and fc2 (one launch for both when it has more than one row, weight-only) and, when it sums,
 * combine; hb_w3_moe_layer_logits routes inside the plan's launch (up to 4 rows: its workgroup routes them first; up
 * to 8191 pairs: a workgroup a row routes and the last to finish plans) or, beyond that, in a launch of its own ahead
 * of the plan's three. count = 0 switches the hook off. Not for captured graphs. */
int hb_debug_events(void* const* events, int count);

/* Measurement hook (no counterpart in the reference): `buffer` (device, int64, four values a record, `records` of them;
 * NULL or 0 switches it off) receives, per workgroup of the launch that runs a routed call's fc1 and fc2 together (the
 * workgroup's index in the launch's grid is the record's; workgroups past `records` write nothing), if it had rows: its
 * start, the end of its wait for fc1 (fc2 workgroups; else 0) and its end, in ticks of the 100 MHz device clock, and its
 * rows (bit 16: an fc1 workgroup). The hook stays armed until it is switched off: the buffer must outlive that. */
int hb_debug_trace(void* buffer, int64_t records);

/* Measurement hook (no counterpart in the reference): one plain streaming read of `bytes` (a multiple of 16 KB) from
 * `src`, 128-bit loads, sixteen in flight a lane - the read rate this device gives a kernel that does nothing else, to
 * hold a weight stream's rate against. `sink`: at least bytes / 65536 + 1 uint32 (practically never written). */
int hb_debug_stream_read(const void* src, size_t bytes, void* sink, void* stream);

/* Measurement hook (no counterpart in the reference): the W3 weight stream's traffic without its arithmetic - what its
 * request structure alone gets from this device, the ceiling to hold the stream's rate against. `groups` workgroups of
 * four wavefronts each read one block of 53 248 bytes (sixteen 3328-byte chunks, four a wavefront through a two-slot
 * LDS ring of LDS-direct loads) at place table[group] of `src` (places of 53 248 bytes, src_bytes / 53 248 of them; a
 * table value outside is clamped), with a dependent read of the table first, sixteen bytes of `acts` (32 rows of 4 KB) a
 * lane and chunk, the K split's exchange through LDS and one store a lane to `out` (groups x 256 floats). `sink`: at
 * least `groups` uint32 (practically never written). The three sizes are checked against what the kernel touches
 * (acts 131 072 bytes, out groups x 1024, sink groups x 4): HB_EINVAL for a buffer too small. */
int hb_debug_ring_skeleton(const void* src, size_t src_bytes, const int32_t* table, int groups, const void* acts, size_t acts_bytes, float* out,
                           size_t out_bytes, void* sink, size_t sink_bytes, void* stream);

/* Measurement hook (no counterpart in the reference): `blocks` workgroups of eight wavefronts each run `iters` rounds of
 * eight independent BF16 MFMAs (16x16x32) on registers - the rate this device's matrix cores give a kernel that does
 * nothing else, to hold an expert GEMM's rate against. Returns the launch's FLOP, or an HB_E* code (they are negative).
 * `sink`: at least `blocks` floats (practically never written). */
int64_t hb_debug_mfma_rate(int blocks, int iters, void* sink, void* stream);
#endif /* HB_NO_DEBUG_HOOKS */

/* ------------------------------------------------------------------------------------------------------------------
 * W3 format: 3-bit (or 2-bit) codes into an 8-entry E4M3 codebook, one E4M3 scale per 32 weights along K, one FP32
 * multiplier per output row.
 *
 * Reference layout (what checkpoints hold; ref: hibana/kernels/w3.py:75-91):
 *   planes uint32 [rows/32, K/128, bits, 32, 4], scales uint8 [rows/32, K/128, 4, 32], row_scale float [rows].
 * Tile layout (what the kernels stream; built once at load time): blocks of 64 rows x 128 k, 3328 bytes each,
 *   [rows/64][K/128]{ 3 x 64 lanes x 16 B of codes, 16 x 16 B of scales }, see hibana_amd/csrc/w3_layout.hpp.
 * `rows` may stack several matrices (experts) of the same K as long as each has a multiple of 64 rows.
 * ---------------------------------------------------------------------------------------------------------------- */

/* Bytes of the tile layout of a [rows, k] matrix of `bits`-bit tiles (3: blocks of 3328 bytes; 2: of 2304); 0 if
 * rows % 64, k % 128 or bits is neither. */
size_t hb_w3_tiled_bytes(int64_t rows, int k, int bits);

/* Reference layout -> tile layout (load-time repack). bits = 3 or 2: the planes' (the reference streams two planes for a
 * four-level codebook, hibana/kernels/w3.py:12-19,89-91); tile_bits: the tiles' - bits itself (a two-bit matrix keeps
 * its 2.25 bits a weight; hb_w3_gemm serves it), or 3 for two-bit codes widened into three-bit tiles (what the routed
 * experts' kernels read).
 * ref: the layout contract of w3_gemm's operands, hibana/kernels/csrc/w3_gemm.cu:1299-1315 (kernel template P, :113);
 * hook point hibana/weights/w3_checkpoint.py:115-139 (CalibratedWeights._load). */
int hb_w3_repack(const uint32_t* planes, const uint8_t* scales, int64_t rows, int k, int bits, int tile_bits, void* tiled, void* stream);

/* codes uint8 [rows, k] + E4M3 scale bytes uint8 [rows, k/32] -> reference layout (planes, scales).
 * ref: w3._pack_codes_rows, hibana/kernels/w3.py:175-195. */
int hb_w3_pack_codes(const uint8_t* codes, const uint8_t* scale_bytes, int64_t rows, int k, int bits, uint32_t* planes,
                     uint8_t* scales, void* stream);

/* Tile layout (of `bits`-bit tiles) -> codes uint8 [rows, k] and E4M3 scale bytes uint8 [rows, k/32] (either output may be NULL).
 * ref: w3.codes / the byte part of w3.group_scales, hibana/kernels/w3.py:217-236. */
int hb_w3_unpack(const void* tiled, int64_t rows, int k, int bits, uint8_t* codes, uint8_t* scale_bytes, void* stream);

/* Reference layout -> codes / scale bytes, same outputs as hb_w3_unpack (the unpack of a checkpoint tensor as stored).
 * ref: hibana/kernels/w3.py:217-236. */
int hb_w3_unpack_planes(const uint32_t* planes, const uint8_t* scales, int64_t rows, int k, int bits, uint8_t* codes,
                        uint8_t* scale_bytes, void* stream);

/* Tile layout (of `bits`-bit tiles) -> float32 [rows, k]: level[code] * (float(e4m3 scale) * row_scale[row]), both products rounded to
 * FP32 in this order (bit-exact with the reference's unpack). `lut` = the codebook as 8 E4M3 bytes, entry i in byte i.
 * ref: w3.dequantize, hibana/kernels/w3.py:239-242; lut: w3.lut_of, :105-107. */
int hb_w3_dequant(const void* tiled, const float* row_scale, int64_t lut, int64_t rows, int k, int bits, float* out, void* stream);

/* y[m, n] = bf16( row_scale[n] * sum_g scale[n, g] * sum_{k in g} x[m, k] * level[code[n, k]] ), FP32 accumulation,
 * x BF16 [m, k] row-major with row stride k, y BF16 [m, n]. Any m >= 1 (the reference stops at 128 rows).
 * n % 64 == 0, k % 128 == 0. bits: the tiles' (3, or 2 for a matrix repacked at two bits: the weight stream then reads
 * 2.25 bits a weight, as the reference's kernel does for its draft head's copy, hibana/proposers/draft_head.py:106).
 * ref: w3_gemm / w3_gemm_wide, hibana/kernels/csrc/w3_gemm.cu:1299-1331,1385-1413 (called by w3.w3_linear,
 * hibana/kernels/w3.py:340-365), in its weight-only form (BF16 activations are not re-quantized to E4M3). */
int hb_w3_gemm(const void* x, int m, const void* tiled, const float* row_scale, int64_t lut, int n, int k, int bits,
               void* y, void* stream);

/* The reference's activation rounding: x BF16 [m, k] (k % 32 == 0) -> q E4M3 bytes [m, k], scales float32 [m, k / 32]:
 * s = max(amax / 448, 1e-12) per (row, 32-group), q = e4m3(clamp(x / s, -448, 448)), IEEE FP32 divisions.
 * ref: w3.quant_groups, hibana/kernels/w3.py:333-337 (quant_groups_kernel, hibana/kernels/csrc/w3_gemm.cu:291-327), as
 * its torch statement defines it (hibana/kernels/w3_moe.py:187-190): the CUDA kernel multiplies by an approximate
 * reciprocal, whose bits are NVIDIA's. */
int hb_w3_quant_groups(const void* x, int64_t m, int k, void* q, float* scales, void* stream);

/* The per-row form of the activation rounding: x BF16 [m, k] (k % 8 == 0) -> q E4M3 bytes [m, k], scales float32 [m]:
 * s = max(amax of the row / 448, 1e-12), q = e4m3(clamp(x / s, -448, 448)), IEEE FP32 divisions. hb_w3_gemm_e4m3 takes
 * the result with the row's scale repeated over its k / 32 groups.
 * ref: w3.quant_rows, hibana/kernels/w3.py:326-330 (quant_rows_kernel, hibana/kernels/csrc/w3_gemm.cu:244-288, which
 * multiplies by a reciprocal where this divides, as hb_w3_quant_groups does). */
int hb_w3_quant_rows(const void* x, int64_t m, int k, void* q, float* scales, void* stream);

/* hb_w3_gemm on rounded activations, the reference kernel's own arithmetic:
 * y[m, n] = bf16( row_scale[n] * sum_g (x_scale[m, g] * scale[n, g]) * sum_{k in g} xq[m, k] * level[code[n, k]] ),
 * FP8 x FP8 products summed in FP32 a group. xq E4M3 [m, k], x_scale float32 [m, k / 32] as hb_w3_quant_groups makes
 * them. Served by the weight stream at any m (the reference stops at 128 rows).
 * ref: w3_gemm, hibana/kernels/csrc/w3_gemm.cu:105-108,209-210,1299-1331 (w3.w3_linear with E4M3 x, hibana/kernels/
 * w3.py:340-365). */
int hb_w3_gemm_e4m3(const void* xq, const float* x_scale, int m, const void* tiled, const float* row_scale, int64_t lut,
                    int n, int k, int bits, void* y, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Routed experts on W3 weights (gated SiLU when fc1 has 2*inter rows per expert in the reference's fc1_order, ReLU^2
 * when it has inter rows).
 * ---------------------------------------------------------------------------------------------------------------- */
typedef struct hb_w3_experts {
  const void* fc1;        /* tile layout of the stacked fc1 [experts * n1, hidden], n1 = gated ? 2*inter : inter */
  const float* fc1_rows;  /* [experts, n1] */
  const void* fc2;        /* tile layout of the stacked fc2 [experts * hidden_out, inter] */
  const float* fc2_rows;  /* [experts, hidden_out] */
  int64_t fc1_lut, fc2_lut;
  int experts;            /* experts held here (expert parallel: one rank's range) */
  int base;               /* id of the first one */
  int hidden, inter, hidden_out; /* fc1 in-features, intermediate size, fc2 out-features (== hidden for these models) */
  int gated;
} hb_w3_experts;

enum { HB_MOE_SUM = 0, HB_MOE_PAIRS_F32 = 1, HB_MOE_PAIRS_BF16 = 2, HB_MOE_E4M3 = 16 /* flag: or it into a mode */ };

/* Workspace bytes for hb_w3_moe / hb_w3_moe_layer with up to m rows of top-k ids (shared: 1 if a shared expert rides
 * along). */
size_t hb_w3_moe_workspace_bytes(int m, int topk, const hb_w3_experts* routed, int shared);

#ifndef HB_NO_DEBUG_HOOKS
/* Test hook (no counterpart in the reference): where a routed W3 call of this shape keeps its plan in its workspace, so
 * that a test can read the plan back - offsets (HOST, six values): byte offsets of the slot table (int32: slots, distinct
 * experts, kept pairs, ticket, fault word, ..., then from word 16 four words a slot: local expert id or -1 for the
 * shared expert, first sorted position, rows, 0), of the sorted pair list (int32 [pairs + shared rows]), of h, of the
 * pair outputs and of the slots' arrival counters; last, the slot table's capacity in slots. */
int hb_debug_workspace_layout(int m, int topk, const hb_w3_experts* routed, int shared, int64_t* offsets);
#endif

/* Routed sum: out[r] = bf16( fma-chain over the row's slots, in selection order, of weights[r, s] * y[r, s] ),
 * y = fc2_e( act( bf16(fc1_e x_r) ) ) in FP32, h rounded to BF16. ids int32 [m, topk]; an id outside
 * [base, base + experts) adds nothing. mode HB_MOE_SUM: out BF16 [m, hidden_out]; HB_MOE_PAIRS_F32 / _BF16: out is
 * the unsummed pair outputs [m * topk, hidden_out] (rows of dropped pairs are left untouched).
 * With HB_MOE_E4M3 or-ed into mode, x and h go through the reference's activation rounding (hb_w3_quant_groups) before
 * their products, as in the reference kernel (y = fc2_e(Q(act(bf16(fc1_e Q(x_r)))))); without it the weight-only form.
 * ref: w3_moe, hibana/kernels/csrc/w3_gemm.cu:1366-1382 (run<S> :1215-1292; Python hibana/kernels/w3_moe.py:158-179;
 * its torch statement w3_moe.reference, :193-214). */
int hb_w3_moe(const hb_w3_experts* routed, const void* x, const int32_t* ids, const float* weights, int m, int topk,
              int mode, void* out, void* workspace, size_t workspace_bytes, void* stream);

/* The whole MoE layer on 3-bit weights: routed sum + shared expert (a one-expert hb_w3_experts, may be NULL) +
 * combine: out = bf16( bf16(routed) + g * bf16(shared) ), g = sigmoid(x . gate_vec) or 1 when gate_vec is NULL
 * (float32 [hidden]).
 * ref: MoeLayer.__call__, hibana/model/flashnext/moe.py:177-192 (w3_moe with pairs + moe_combine_pairs,
 * hibana/kernels/flashnext_fused.py:530-571). */
int hb_w3_moe_layer(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x,
                    const int32_t* ids, const float* weights, int m, int topk, void* out, void* workspace,
                    size_t workspace_bytes, void* stream);

/* hb_w3_moe_layer for callers that cannot allocate device memory or carry a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the same chain of launches and the same bits, with the plan, the
 * sorted pair list, h and the pair outputs in a device array of HB_STATIC_SCRATCH_BYTES that the library itself holds
 * (one copy on every GPU it runs on, until the process ends). A call whose hb_w3_moe_workspace_bytes(m, topk, routed,
 * shared != NULL) exceeds that returns HB_ESCRATCH and enqueues nothing (the benchmark's verify step - 32 tokens, top-10,
 * 512 experts of 2048 x 512 and a shared one - takes 3.7 MB). It calls no allocator. The array is zero when the library
 * is loaded and every call leaves its head words zero, as with any workspace; everything else a launch of the chain
 * writes before it is read, so nothing is cleared. All calls on one GPU share the array: two calls that overlap on one
 * GPU (different streams, or replays of graphs holding them) race; on one stream they are ordered like any other work.
 * hb_workspace_status(NULL, ...) reads its fault word, hb_workspace_reset(NULL, 0, stream) puts it back in service.
 * No counterpart in the reference (its op allocates its scratch from torch's caching allocator on every call,
 * hibana/kernels/csrc/w3_gemm.cu:1234-1247); for the callers above. */
#define HB_STATIC_SCRATCH_BYTES (8u << 20)
int hb_w3_moe_layer_static(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x,
                           const int32_t* ids, const float* weights, int m, int topk, void* out, void* stream);

/* hb_w3_moe_layer in the reference kernel's own arithmetic: x and h of the routed experts and of the shared expert go
 * through the activation rounding (hb_w3_quant_groups' arithmetic) before their products, as with HB_MOE_E4M3 in
 * hb_w3_moe; the combine is the same. No launch of its own for either rounding: x is rounded by further workgroups of
 * the planning launch, h in fc1's epilogue.
 * ref: as hb_w3_moe_layer, with w3_moe.reference's `quant`, hibana/kernels/w3_moe.py:187-214. */
int hb_w3_moe_layer_e4m3(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x,
                         const int32_t* ids, const float* weights, int m, int topk, void* out, void* workspace,
                         size_t workspace_bytes, void* stream);

/* The same layer from the router's logits (float32 [m, experts_total]): softmax top-k routing as
 * hb_route_softmax_topk, written to ids int32 [m, topk] and weights float32 [m, topk] (caller's buffers), then the
 * chain of hb_w3_moe_layer. Routing and plan are one launch up to 8191 pairs (up to 4 rows the planning workgroup
 * routes them itself; beyond, a workgroup a row routes and the last one to finish plans); one token has no such launch
 * at all: fc1's wavefronts route the row themselves.
 * ref: MoeLayer.__call__ with its route step, hibana/model/flashnext/moe.py:122-144,177-192. */
int hb_w3_moe_layer_logits(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec,
                           const void* x, const float* logits, int experts_total, int m, int topk, int32_t* ids,
                           float* weights, void* out, void* workspace, size_t workspace_bytes, void* stream);

/* hb_w3_moe_layer_logits with the activation rounding of hb_w3_moe_layer_e4m3 (the routing itself reads the FP32
 * logits and is the same).
 * ref: as hb_w3_moe_layer_logits, with w3_moe.reference's `quant`, hibana/kernels/w3_moe.py:187-214. */
int hb_w3_moe_layer_logits_e4m3(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec,
                                const void* x, const float* logits, int experts_total, int m, int topk, int32_t* ids,
                                float* weights, void* out, void* workspace, size_t workspace_bytes, void* stream);

/* The same layer from the router's BF16 logits [m, experts_total] under a budget: the experts are chosen by
 * hb_route_budget's rule (keep, budget, slots / steps, per_request, min_cap as there; slots left over name no expert:
 * id experts_total at weight 0, which the experts skip), written to ids / weights (caller's buffers), then the chain of
 * hb_w3_moe_layer. Two launches ahead of the experts': the rows' candidates, then one workgroup that selects and also
 * plans (up to 8191 pairs; beyond, the plan's own launches follow). Weight-only arithmetic. topk and keep at most
 * HB_ROUTE_CANDIDATES, 20 <= experts_total <= 1024, m a multiple of steps. The same ids, weights and output as
 * hb_route_budget followed by hb_w3_moe_layer, bit for bit.
 * ref: MoeLayer.__call__ with the budgeted branch of its route step, hibana/model/flashnext/moe.py:122-135,177-192. */
int hb_w3_moe_layer_budget(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec,
                           const void* x, const void* logits, int experts_total, int m, int topk, int keep, int budget,
                           const int32_t* slots, int steps, int per_request, int min_cap, int32_t* ids, float* weights,
                           void* out, void* workspace, size_t workspace_bytes, void* stream);

/* out = bf16( bf16(sum over the row's local slots of w * pairs) + g * shared ) from unsummed pair outputs (FP32 or,
 * pairs_bf16 != 0, BF16) [m * topk, h]; shared BF16 [m, h] or NULL; gate_vec float32 [h] or NULL (then g = 1; x
 * unused). ref: moe_combine_pairs, hibana/kernels/flashnext_fused.py:530-571; with shared == NULL it is
 * combine_kernel, hibana/kernels/csrc/w3_gemm.cu:1196-1213. */
int hb_moe_combine_pairs(const void* pairs, int pairs_bf16, const int32_t* ids, const float* weights, const void* shared,
                         const void* x, const float* gate_vec, int e_lo, int e_n, int m, int topk, int h, void* out,
                         void* stream);

/* out BF16 [rows, half] = bf16( bf16(silu(gate)) * up ) from gate_up BF16 [rows, 2 * half]: columns [gate | up]
 * (pairs == 0) or blocks of `pairs` gate columns alternating with their `pairs` up columns (half % pairs == 0; half and
 * pairs even). The experts' fc1 epilogues do this inside their launches; this is the standalone op.
 * ref: ops.silu_and_mul, hibana/kernels/ops.py:86-92. */
int hb_silu_and_mul(const void* gate_up, int64_t rows, int half, int pairs, void* out, void* stream);

/* The same from the FP32 product, rounded once: out = bf16(silu(gate) * up) (shapes and `pairs` as hb_silu_and_mul).
 * ref: silu_mul, hibana/kernels/flashnext_fused.py:624-639. */
int hb_silu_mul(const void* gate_up, int64_t rows, int half, int pairs, void* out, void* stream);

/* x = bf16(relu(x)^2) in place, BF16 [rows, n] with rows `stride` elements apart (n and stride even): the square in FP32
 * with one rounding. ref: relu2_, hibana/model/nemotron/moe.py:316-321 (the expert kernels do it in their epilogues). */
int hb_relu2(void* x, int64_t rows, int n, int64_t stride, void* stream);

/* silu(gate) * up of BF16 [rows, 2 half] (columns as in hb_silu_and_mul) rounded to E4M3 per (row, 32-group) in one
 * launch: q E4M3 [rows, half], scales FP32 [rows, half / 32], bit for bit hb_w3_quant_groups of hb_silu_and_mul's
 * result when `torch_chain` != 0 (silu rounded to BF16, then the BF16 product), else of bf16(silu(gate) * up) from the
 * FP32 product. half % 32 == 0, pairs % 32 == 0.
 * ref: silu_mul_quant_groups, hibana/kernels/flashnext_fused.py:814-853 (caller Mlp.__call__, hibana/model/mlp.py:36-42),
 * with the exact divisions of the quantizer's torch statement. */
int hb_silu_mul_quant_groups(const void* gate_up, int64_t rows, int half, int pairs, int torch_chain, void* q,
                             float* scales, void* stream);

/* Softmax top-k routing: logits float32 [m, e] -> ids int32 [m, k] (descending probability, ties to the lower id),
 * weights float32 [m, k] renormalized over the selection. slots (may be NULL: every row is real): row r is real iff
 * slots[r / steps] != 0; a padded row gets weight 0 in every slot and the id e ("no expert", which the 3-bit experts
 * skip) or, repeat != 0, row 0's first choice.
 * ref: route_topk, hibana/kernels/flashnext_fused.py:278-319. */
int hb_route_softmax_topk(const float* logits, int m, int e, int k, const int32_t* slots, int steps, int repeat, int32_t* ids,
                          float* weights, void* stream);

/* Sigmoid top-k routing of the latent MoE on the fused router|fc1_latent GEMM output: fused FP32 [m, stride], columns
 * 0..e-1 the router logits, e..e+latent-1 the latent projection. s = 1 / (1 + exp(-logit)); ids = the k largest of
 * s + bias[e] in descending order, equal scores to the lower id; weights = s[ids] / (sum of s[ids] + 1e-20) (no
 * routed scaling factor); lat BF16 [m, latent] = the latent columns rounded (latent may be 0). slots (may be NULL):
 * row r is real iff slots[r / steps] != 0; a padded row gets weight 0 and row 0's first choice (repeat != 0) or id e.
 * ref: route_topk / _route_kernel, hibana/model/nemotron/moe.py:75-121. */
int hb_route_sigmoid_topk(const float* fused, int64_t stride, const float* bias, int m, int e, int k, int latent,
                          const int32_t* slots, int steps, int repeat, int32_t* ids, float* weights, void* lat,
                          void* stream);

/* Budgeted top-k: the experts one decode / verify forward reads are chosen for all its rows, under a cap. logits BF16
 * [r, e] contiguous (20 <= e <= 1024) -> ids int32 [r, k], weights FP32 [r, k] (k, keep <= HB_ROUTE_CANDIDATES).
 *   the set: every real row's top `keep`, then the experts with the most softmax probability within the real rows'
 *   top k, summed over the rows (equal sums: the lower expert), until it holds the cap (more only when the guaranteed
 *   experts alone exceed it); the cap is `budget`, or with per_request > 0,
 *   min(budget, max(min_cap, per_request x the real requests)), a request being `steps` consecutive rows;
 *   a real row takes its candidates (its HB_ROUTE_CANDIDATES largest logits, largest first, an exact tie to the lower
 *   expert, -0 equal to +0) that are in the set, in rank order, up to k, at the FP32 softmax over e renormalized over
 *   the ones taken.
 * Slots left over (all of a padded row's; row t is real iff slots == NULL or slots[t / steps] != 0; r % steps == 0)
 * hold id e at weight 0, or with repeat != 0 the row's first candidate (a padded row: row 0's) at weight 0.
 * Two launches, the same bits on every run; nothing is allocated: `workspace` (4-byte aligned, at least
 * hb_route_budget_workspace_bytes(r)) holds the rows' candidates between the launches.
 * ref: route_budget, hibana/kernels/flashnext_fused.py:322-502 (the rule row by row:
 * tests/unit/test_moe_selection.py:19-58); caller MoeLayer.route, hibana/model/flashnext/moe.py:122-135. */
#define HB_ROUTE_CANDIDATES 20
int64_t hb_route_budget_workspace_bytes(int r);
int hb_route_budget(const void* logits, int r, int e, int k, int keep, int budget, const int32_t* slots, int steps,
                    int repeat, int per_request, int min_cap, void* workspace, int64_t workspace_bytes, int32_t* ids,
                    float* weights, void* stream);

/* The latent MoE's budgeted top-k: hb_route_budget's selection on hb_route_sigmoid_topk's ranking. fused FP32
 * [r, stride] (e router logits, then `latent` columns), bias [e] -> ids int32 [r, k], weights FP32 [r, k], lat BF16
 * [r, latent]; k <= 32, e <= 1024. A row's candidates are its top k by sigmoid + bias (equal scores to the lower
 * expert); a candidate adds its renormalized weight s / (sum of the row's k sigmoids) to its expert's score; the set
 * is every real row's top `keep`, then the best-scoring other experts up to the cap (`budget`, or with per_request > 0,
 * min(budget, per_request x the real requests); a budget of 0: the guaranteed experts alone). `fallback` (0: none;
 * at most keep): when the rows' top `keep` alone exceed a cap above 0, each real row is guaranteed only its top
 * `fallback`. A real row takes its candidates in the set in rank order; its weights are the plain sigmoids over
 * (their sum in rank order + 1e-20): a row that keeps all k gets hb_route_sigmoid_topk's weights bit for bit. Slots left
 * over (all of a padded row's) hold the row's first candidate (a padded row: row 0's) at weight 0, or id e when
 * repeat == 0. Two launches; `workspace` (4-byte aligned) of hb_route_budget_sigmoid_workspace_bytes(r, k).
 * ref: route_budget, hibana/model/nemotron/moe.py:124-313; caller NemotronMoe.route / fallback, :453-474. */
int64_t hb_route_budget_sigmoid_workspace_bytes(int r, int k);
int hb_route_budget_sigmoid(const float* fused, int64_t stride, const float* bias, int r, int e, int k, int latent,
                            int keep, int budget, const int32_t* slots, int steps, int repeat, int per_request,
                            int fallback, void* workspace, int64_t workspace_bytes, int32_t* ids, float* weights,
                            void* lat, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * NVFP4 format: E2M1 codes two per byte (element 2i in the low nibble), one E4M3 scale per 16 weights, one FP32
 * global scale. ref: hibana/weights/modelopt.py:57-81,150-156.
 * Tile layout: blocks of 64 rows x 128 k, 4608 bytes each: { 4 x 64 lanes x 16 B of codes, 64 rows x 8 scale bytes }.
 * ---------------------------------------------------------------------------------------------------------------- */
size_t hb_nvfp4_tiled_bytes(int64_t rows, int k);

/* weight uint8 [rows, k/2] + block scales E4M3 uint8 [rows, k/16] (row-major, unswizzled) or, swizzled != 0, in the
 * CUTLASS 128x4 interleave [rows_pad128, (k/16)_pad4] -> tile layout.
 * ref: the operand layout of mm_fp4 at hibana/kernels/ops.py:74-82; swizzle hibana/weights/modelopt.py:130-147. */
int hb_nvfp4_repack(const uint8_t* weight, const uint8_t* scales, int swizzled, int64_t rows, int k, void* tiled,
                    void* stream);

/* Tile layout -> float32 [rows, k]: e2m1 * float(e4m3 scale) * global_scale (two FP32 roundings in this order).
 * ref: unpack_fp4 / Nvfp4Linear.dequantize, hibana/weights/modelopt.py:73-77,150-156. */
int hb_nvfp4_dequant(const void* tiled, float global_scale, int64_t rows, int k, float* out, void* stream);

/* y = bf16( (x Wq^T)_fp32 * global_scale ), Wq = e2m1 * e4m3 (exact in BF16); relu2 != 0 applies
 * bf16(relu(y)^2) on top. x BF16 [m, k], y BF16 [m, n]; n % 64 == 0, k % 128 == 0.
 * ref: ops.nvfp4_linear, hibana/kernels/ops.py:56-83 in its weight-only form, which the reference states as
 * ggml_bf16.matmul(..., "NVFP4"), hibana/kernels/ggml_bf16.py:125-159. */
int hb_nvfp4_gemm(const void* x, int m, const void* tiled, float global_scale, int n, int k, int relu2, void* y,
                  void* stream);

/* The same product with room for partial sums: calls of a few dozen rows (17 .. about 250), too many for the weight
 * stream's sixteen rows a pass over the matrix and too few to fill the device with 128-row tiles, share K among the
 * workgroups of a tile; their partial tiles meet in `workspace` and whichever workgroup of a tile finishes last adds them
 * in one fixed order: the result does not depend on the schedule. hb_nvfp4_gemm_workspace_bytes: what a call of this
 * shape uses (0: none, the call is hb_nvfp4_gemm's); the tiles' arrival counters lie at its head (zero before the first
 * use, see "Workspaces" above). No counterpart in the reference (cuBLASLt / FlashInfer own their workspaces there). */
size_t hb_nvfp4_gemm_workspace_bytes(int m, int n, int k);
int hb_nvfp4_gemm_ws(const void* x, int m, const void* tiled, float global_scale, int n, int k, int relu2, void* y,
                     void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Routed experts on NVFP4 weights (ReLU^2 when fc1 has inter rows per expert, gated SiLU when it has 2*inter rows in
 * the W3 path's fc1_order).
 * ---------------------------------------------------------------------------------------------------------------- */
typedef struct hb_nvfp4_experts {
  const void* fc1;          /* tile layout of the stacked fc1 [experts * n1, hidden], n1 = gated ? 2*inter : inter */
  const float* fc1_scale2;  /* [experts] FP32 scale of each fc1 matrix (the checkpoint's weight_scale_2) */
  const void* fc2;          /* tile layout of the stacked fc2 [experts * hidden_out, inter] */
  const float* fc2_scale2;  /* [experts]; a routed_scaling_factor is folded in here by the caller */
  int experts, base;        /* experts held here and the id of the first one */
  int hidden, inter, hidden_out;
  int gated;
} hb_nvfp4_experts;

size_t hb_nvfp4_moe_workspace_bytes(int m, int topk, const hb_nvfp4_experts* routed);

/* Routed sum on NVFP4 experts, same contract and modes as hb_w3_moe:
 * h = bf16(act(bf16((x up_e^T)_fp32 * s2))), y = (h down_e^T)_fp32 * s2, out[r] = bf16(sum_s weights[r, s] * y[r, s]).
 * ref: B12xExperts.__call__, hibana/kernels/b12x_moe.py:58-68 (caller NemotronMoe.routed,
 * hibana/model/nemotron/moe.py:476-482) in the weight-only form stated by moe_mixer,
 * tests/nemotron_reference.py:568-593. */
int hb_nvfp4_moe(const hb_nvfp4_experts* routed, const void* x, const int32_t* ids, const float* weights, int m,
                 int topk, int mode, void* out, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * The latent-MoE block of a decode / verify call (at most HB_LATENT_MAX_ROWS rows), the native surface of the
 * reference's hibana/kernels/nemotron_moe.py:45-68 (`router`, `block`, `shared_up`, `out`; kernels in
 * hibana/kernels/csrc/nemotron_moe.cu):
 *
 *   fused  = x [router; fc1_latent]^T                    FP32 [m, experts_total + latent]
 *   ids, w = top-k of sigmoid(logits) + bias, w = the plain sigmoids renormalized; lat = bf16(fused[:, experts_total:])
 *   routed = sum_k w_k * down_e(relu(up_e lat)^2)         BF16 [m, latent]
 *   out    = bf16(shared_down(relu(shared_up x)^2) + routed fc2^T)
 *
 * Weight-only arithmetic: activations stay BF16 (the reference's small-call kernels round x, lat and h to NVFP4 for its
 * FP4 tensor cores; its own FP32 statement of the block, NemotronMoe.reference, hibana/model/nemotron/moe.py:521-566,
 * is what these entry points follow). hb_latent_router (two launches: the product; routing and plan) followed by
 * hb_latent_block (four) is six launches where the block through separate operators is nine.
 * ---------------------------------------------------------------------------------------------------------------- */
#define HB_LATENT_MAX_ROWS 16

typedef struct hb_latent_weights {
  const void* gate_fc1;            /* BF16 [experts_total + latent, hidden]: the router's rows, then fc1_latent's */
  const float* bias;               /* [experts_total]: added to the scores for the choice only */
  const void* fc2;                 /* BF16 [hidden, latent] */
  const hb_nvfp4_experts* routed;  /* NVFP4 experts with hidden = hidden_out = latent; NULL when the routed experts
                                      are not NVFP4 (then hb_latent_block is not available) */
  const void* shared_up;           /* tile layout of [shared_inter, hidden], or NULL: no shared expert */
  const void* shared_down;         /* tile layout of [hidden, shared_inter] */
  float shared_up_scale, shared_down_scale;  /* their FP32 scales (weight_scale_2) */
  int experts_total, latent, hidden, shared_inter;
} hb_latent_weights;

/* One workspace serves the four calls of a block; its size depends on (weights, m, topk) only. 0 on invalid input. */
size_t hb_latent_workspace_bytes(const hb_latent_weights* w, int m, int topk);

/* ref: `router`, hibana/kernels/nemotron_moe.py:45-55 (router_kernel, nemotron_moe.cu:496-558). x BF16 [m, hidden] ->
 * fused FP32 [m, experts_total + latent] and lat BF16 [m, latent]; with `route`, ids int32 [m, topk] / weights FP32
 * [m, topk] as hb_route_sigmoid_topk gives them from `fused`, bit for bit (slots / steps: its padded rows; a padded
 * row takes row 0's first choice at weight 0, or `pad_id` when that is >= 0), and the call's plan is left in the
 * workspace for hb_latent_block. Without `route`, ids / weights are not written (and may be NULL). */
int hb_latent_router(const hb_latent_weights* w, const void* x, int m, int topk, const int32_t* slots, int steps,
                     int route, int pad_id, float* fused, int32_t* ids, float* weights, void* lat, void* workspace,
                     size_t workspace_bytes, void* stream);

/* ref: `block`, hibana/kernels/nemotron_moe.py:58-60: the rest of the block after hb_latent_router -> out BF16
 * [m, hidden]. `plan` != 0 when ids are not the router's (the caller routed): the plan is then made here, one more
 * launch. Four launches otherwise: routed fc1 beside the shared expert's up, routed fc2 beside its down, the combine,
 * fc2_latent. */
int hb_latent_block(const hb_latent_weights* w, const void* x, const void* lat, const int32_t* ids,
                    const float* weights, int m, int topk, int plan, void* out, void* workspace,
                    size_t workspace_bytes, void* stream);

/* ref: `shared_up` / `out` as `w3_block` uses them around other routed experts, hibana/kernels/nemotron_moe.py:63-68:
 * hb_latent_shared_up leaves relu(shared_up x)^2 in the workspace; hb_latent_out, given the routed sum BF16
 * [m, latent], writes out = bf16(shared_down(...) + routed fc2^T). Without a shared expert hb_latent_shared_up
 * returns HB_ENULL and hb_latent_out adds nothing. */
int hb_latent_shared_up(const hb_latent_weights* w, const void* x, int m, int topk, void* workspace,
                        size_t workspace_bytes, void* stream);
int hb_latent_out(const hb_latent_weights* w, const void* routed, int m, int topk, void* out, void* workspace,
                  size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HIBANA_HIP_H */
