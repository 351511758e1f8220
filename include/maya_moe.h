/* maya_moe.h - C ABI of the MI355X (gfx950) routed-MoE expert block.
 *
 * The library (libmaya_moe.so) replaces the reference engine's expert-rows operators on one GPU: router top-k, the
 * per-expert grouping of a token batch, the activation quantizers, the fused dequant gate/up GLU mat-vec, the down
 * mat-vec, the weighted combine, and the prefill grouped int8 GEMM.  Each entry point names the reference interface it
 * stands in for (paths relative to the reference tree).
 *
 * Conventions (the reference's operator contract, include/strata/kernels/glm_fast.hpp:496-501, src/ds4/ds4_iq.cuh:60-91,
 * include/strata/kernels/s2_expert_grouped.hpp:36-38):
 *   - every pointer is DEVICE memory unless it says "host"; the caller owns every buffer, scratch included
 *     (maya_moe_workspace_bytes gives the size); no entry point allocates, synchronizes or calls back to the host;
 *   - `stream` is a hipStream_t passed as void*; work is asynchronous and ordered on it; calls on different streams
 *     may overlap as long as they use different workspaces;
 *   - routing results stay on the device: kernels read plans, groups and counts from device memory, so a launch
 *     sequence does not depend on routing and can be captured in a HIP graph;
 *   - a plan slot whose blob address is 0 is skipped (the expert is not resident here; its part is left out);
 *   - weights are raw GGUF rows, row-major, [gate rows | up rows | down rows] per expert (offsets in maya_moe_layout),
 *     aligned to 2 bytes or better;
 *   - return value: 0 ok; > 0 "not covered, nothing launched" (MAYA_E_*); < 0 a HIP error (-hipError_t).
 *     maya_last_error() returns a thread-local message for the last non-zero return.
 */
#ifndef MAYA_MOE_H
#define MAYA_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids of the weight formats (src/ds4/ds4_iq.cuh:27-31) */
#define MAYA_TYPE_Q8_0 8
#define MAYA_TYPE_Q4_K 12
#define MAYA_TYPE_IQ2_XXS 16 /* general kernels only: no stream packing of its own, no prefill GEMM */
#define MAYA_TYPE_IQ1_S 19
#define MAYA_TYPE_IQ2_S 22
#define MAYA_TYPE_IQ1_M 29

/* element types of activations handed in by the caller */
#define MAYA_DT_F32 0
#define MAYA_DT_BF16 1
#define MAYA_DT_F16 2

#define MAYA_OK 0
#define MAYA_E_UNSUPPORTED 1 /* a weight type, dtype or codebook this library has no kernel for */
#define MAYA_E_SHAPE 2       /* a size outside what the kernels assume (not whole blocks, too many tokens, ...) */
#define MAYA_E_ARG 3         /* a null pointer or a workspace that is too small */
#define MAYA_E_NOGPU 4       /* no gfx950 device / the library's device code is not loadable */
#define MAYA_E_BUSY 5        /* maya_moe_layer_decode_shared: the device's side stream is inside another stream's capture */

#define MAYA_MAX_K 16          /* experts per token */
#define MAYA_MAX_TOKENS 16     /* tokens of one decode / verify-window call */
#define MAYA_MAX_EXPERTS 1024  /* router width */

/* One layer's expert geometry: strata::kernels::cpu::NativeFmt (include/strata/kernels/cpu/native_expert.hpp:26-39),
 * iq::Args::tr / tg / td (src/ds4/ds4_iq.cuh:72-84). */
typedef struct maya_moe_layout {
    int32_t gate_type, up_type, down_type; /* ggml ids; gate and up must share the activation format */
    int32_t n_embd, n_ff;                  /* multiples of 256 */
    uint64_t gate_off, up_off, down_off;   /* byte offsets of the three row arrays inside an expert blob */
    int32_t packing;                       /* MAYA_PACK_GGUF or MAYA_PACK_STREAM (maya_moe_repack) */
    int32_t reserved;
} maya_moe_layout;

/* Row packings.  GGUF: the file's own block sequence.  STREAM: the same bytes regrouped so that a wavefront's loads
 * are aligned, contiguous and addressed by position alone.  IQ2_S rows are taken four at a time (a quad; row counts
 * are multiples of 4): with nu = k / 32 sub-blocks a row, the quad's 4 * row_bytes bytes hold, for sub-block u of row
 * r of the quad, the (index word, sign word) pair at byte 8 (4 u + r), the (high-bit byte, scale byte) pair at 32 nu +
 * 2 (4 u + r), and block b's FP16 scale at 40 nu + 2 (4 b + r).  IQ1_S rows likewise in quads: sub-block u's four
 * index bytes at 4 (4 u + r), its qh word at 16 nu + 2 (4 u + r), block b's scale at 24 nu + 2 (4 b + r).  IQ1_M:
 * index bytes and qh words as IQ1_S, then 8 bytes a (block b, row r) at 24 nu + 8 (4 b + r) = the FP16 block scale
 * (gathered from the top nibbles of the block's four scale words) followed by those words' 4 x 12 bits of 3-bit
 * scales.  A Q8_0 row holds its k codes first, then its k / 32 FP16 scales (block b's scale at k + 2 b).  Other types
 * are left as they are.  A row (a quad) keeps its size and its position in the blob and every field keeps its bits, so
 * dequantized values are unchanged.  Stream-packed blobs and the offsets of their three row arrays are 16-byte
 * aligned. */
#define MAYA_PACK_GGUF 0
#define MAYA_PACK_STREAM 1

/* A quantized activation batch in device memory (rows x k): int8 codes, an F32 scale per 32 values (a 256-value
 * Q8_K block's scale is written 8 times, as ds4's xd / hd hold it: src/ds4/ds4_lane_parity.hpp:40-42) and ggml's
 * bsums (the sum of every 16 codes, third_party/ggml/ggml-common.h:371-376). */
typedef struct maya_act {
    int8_t* q;      /* [rows][k] */
    float* d;       /* [rows][k/32] */
    int16_t* bsums; /* [rows][k/16] */
} maya_act;

/* The token / window experts: iq::Args (src/ds4/ds4_iq.cuh:66-87), glmf::MoeDev's plan_ptr / plan_w / skip / cpu_part /
 * cpu_flag (include/strata/kernels/glm_fast.hpp:293-318).  Entry e = token e / k, slot e % k.  Group g = one distinct
 * expert and the entries routed to it; with grp_ptr == NULL the groups are the plan itself (group g = entry g). */
typedef struct maya_moe_args {
    maya_moe_layout layout;
    int32_t n_tokens, k;
    const uint64_t* plan_ptr;  /* [n_tokens*k] blob address of each entry's expert (0: skipped) */
    const float* plan_w;       /* [n_tokens*k] combine weights */
    const uint64_t* grp_ptr;   /* [<= n_tokens*k] or NULL */
    const int32_t* grp_start;  /* [groups+1] */
    const int32_t* grp_ent;    /* [n_tokens*k]; given WITHOUT grp_ptr: only the order in which the entry-by-entry kernels take
                                * the entries (an expert's entries side by side: its rows come from DRAM once), -1 = the end */
    const int32_t* n_groups;   /* device count of groups (NULL: n_tokens*k) */
    const int32_t* skip;       /* NULL or a device flag: non-zero makes every kernel of the call a no-op */
    float limit;               /* SwiGLU clamp; +inf or <= 0: none */
    maya_act x;                /* gate/up input, rows = tokens (maya_quant_act of the hidden state) */
    float* h;                  /* [n_tokens*k][n_ff] SwiGLU output */
    maya_act hq;               /* down input, rows = entries (maya_quant_act of h) */
    float* part;               /* [n_tokens*k][n_embd] each entry's down output (NULL in the fused 1-token form) */
    const float* add;          /* NULL or [n_tokens][n_embd] added to the combined output (shared expert, CPU lane part) */
    const int32_t* add_flag;   /* NULL or a device flag: `add` is added only when it is non-zero */
    const float* add2;         /* NULL or [n_tokens][n_embd] added after `add`, always (glmf::moe_down's sh_out beside its
                                * flagged cpu_part, include/strata/kernels/glm_fast.hpp:499-501) */
    float* out;                /* [n_tokens][n_embd] */
} maya_moe_args;

/* ---- probes: glmf::moe_supported, iq::supported / block_bytes / row_bytes (src/ds4/ds4_iq.cuh:40-52) */
int maya_moe_supported(int ggml_type);
int maya_moe_block_bytes(int ggml_type);
int maya_moe_block_values(int ggml_type);
size_t maya_moe_row_bytes(int ggml_type, int64_t k);
/* fills off/sizes for the contiguous [gate|up|down] blob: native_fmt / native_fmt_mixed
 * (src/kernels/cpu/native_expert.cpp:195-260); returns the blob's bytes (0: unsupported) */
size_t maya_moe_layout_init(maya_moe_layout* l, int gate_type, int up_type, int down_type, int n_embd, int n_ff);

/* One-time regrouping of an expert blob for the streaming kernels, at upload: dst (same size as src, 16-byte aligned)
 * receives src's rows in MAYA_PACK_STREAM order; maya_moe_unpack is the inverse.  `l` describes the GGUF blob; use a copy
 * of it with packing = MAYA_PACK_STREAM for calls on dst.  The reference uploads resident experts into VRAM slots of a pool
 * (include/strata/kernels/glm_fast.hpp:284-300); this is the hook that runs on that copy.  src and dst must not overlap. */
int maya_moe_repack(const maya_moe_layout* l, const void* src, void* dst, void* stream);
int maya_moe_unpack(const maya_moe_layout* l, const void* src, void* dst, void* stream);
/* A layer's expert blobs from its three stacked GGUF tensors, on the device: blob e at dst + e * dst_stride receives
 * [gate rows | up rows | down rows] of expert e - gate_exps / up_exps / down_exps are ffn_{gate,up,down}_exps.weight as the
 * file stores them, [n_expert][rows][row bytes] - in GGUF order (packing MAYA_PACK_GGUF: the concatenation the
 * reference's packer writes on the host, tools/iq_pack.py:510-514, read back as native_expert_layout's blob,
 * src/kernels/cuda/iq_kernels.cu:1077-1101) or already regrouped for the streaming kernels (MAYA_PACK_STREAM: what
 * maya_moe_repack makes of that blob).  `l` describes the GGUF blob (maya_moe_layout_init); dst_stride >= its size. */
int maya_moe_pack_experts(const maya_moe_layout* l, const void* gate_exps, const void* up_exps, const void* down_exps,
                          int n_expert, int packing, void* dst, size_t dst_stride, void* stream);

const char* maya_last_error(void);
/* Device and library identification: "gfx950 ..." (host string, valid until the next call on this thread). */
const char* maya_device_info(void);
/* Loads the device code and uploads the codebooks on the current device; idempotent.  Every other entry point calls it on
 * its first use of a device - and this set-up is the one place that allocates (the codebooks' 24 KB) and copies
 * synchronously: call maya_init() once a device BEFORE the first call made under stream capture (a set-up attempted
 * while the stream is capturing fails with the runtime's error, < 0, and launches nothing). */
int maya_init(void);

/* ---- dequantization to F32, bit-exact with the block formats' reference decode:
 * dequantize_q4_K / dequantize_q8_0 (include/strata/artifact/dequant.hpp:81-85, 162-190), dq_iq2_s / dq_iq1_s /
 * dq_iq1_m + iq_dequant_f32 (src/kernels/cuda/iq_kernels.cu:686-695, 825-855, 1038-1075), iq::decode_values
 * (src/ds4/ds4_iq.cuh:171-175).  w: n_rows rows of k values, row_stride bytes apart (0: the type's own row size). */
int maya_dequant_rows(int ggml_type, const void* w, size_t row_stride, int64_t k, int64_t n_rows, float* out,
                      void* stream);
/* the same for rows in MAYA_PACK_STREAM order */
int maya_dequant_rows_packed(int ggml_type, int packing, const void* w, size_t row_stride, int64_t k, int64_t n_rows,
                             float* out, void* stream);

/* ---- activation quantizers.  act_type = the WEIGHT type whose dot will consume the activation:
 * Q8_K rounding for the 256-value types - quantize_q8_K (src/kernels/cuda/quantize_act.cu:161-207), q8k_quant_kernel
 * (src/ds4/ds4_gguf.cu:299-336), native_quant_act / native_quant_h (src/kernels/cpu/native_expert.cpp:262-268);
 * Q8_0 rounding for Q8_0 weights - the CPU expert path's on x86, ggml-cpu's quantize_row_q8_0 as the reference restates it
 * (quantize_oracle_q8_0, src/kernels/cpu/expert.cpp:92-130): FP16 d = amax / 127, q = nearest-even(x * (127 / amax)); the
 * reference's GPU quantize_q8_0 (include/strata/kernels/quantize_act.hpp:28-31; rint of the double quotient x / d) gives
 * the same scale and differs by one code on the rare value next to a rounding boundary.
 * The contract covers finite inputs: a block that holds a NaN, an infinity or a value whose scaled magnitude passes 2^31 is
 * outside it (the x86 path saturates such lanes to -128, this library clamps them to +-127 and turns NaN into 0).
 * x: rows x k of x_dtype, x_stride elements apart (0: k). */
int maya_quant_act(int act_type, const void* x, int x_dtype, int64_t x_stride, int rows, int64_t k, maya_act out,
                   void* stream);
/* per-32 int8 + F32 scale, the prefill form: quant_act_nat_kernel (src/prefill/moe_fused_rdna4.cu:87-109),
 * q8_quant_kernel (src/ds4/ds4_gguf.cu:219-227), mmq::quantize (src/prefill/moe_mmq.cu:120-157).
 * row_idx: NULL or a gather table (row r reads x[row_idx[r]]). */
int maya_quant_i8x32(const void* x, int x_dtype, int64_t x_stride, const int32_t* row_idx, int rows, int64_t k,
                     int8_t* q, float* d, void* stream);

/* ---- router: strata::kernels::router_top10 (src/kernels/cuda/router_top10.cu:191-224): softmax over all experts in
 * double, stable top-k (strict >, lower index on ties) on the float probabilities, renormalised by max(sum, 2^-14). */
int maya_moe_route_topk(const float* logits, int n_tokens, int n_expert, int k, int32_t* ids, float* weights,
                        void* stream);
/* The sigmoid router of the GLM / DeepSeek-V3 family: strata::kernels::router_sigmoid
 * (include/strata/kernels/router_sigmoid.hpp:8-31, src/kernels/cuda/router_sigmoid.cu:29-74) and the selection of
 * glmf::moe_route (include/strata/kernels/glm_fast.hpp:420-433): p = sigmoid(logits) in float, ids = the stable top-k of
 * p + bias (bias NULL or [n_expert]: it chooses, it does not weigh; ties to the lower index), weights = p / D * w_scale with
 * D = max(sum of the k chosen p, 2^-14) (norm MAYA_ROUTER_NORM_CLAMP = kRouteNormClamp), sum + 1e-20 (MAYA_ROUTER_NORM_HF =
 * kRouteNormHf) or 1 (MAYA_ROUTER_NORM_NONE: norm_topk_prob off).
 * A token with a non-finite logit or score (NaN, +-Inf; a bias counts) is refused as the engine's routers refuse it
 * (route_kernel, src/kernels/cuda/glm_batch.cu:2077-2092; moe_route_kernel, glm_fast.cu:4040, 4136-4141): ids -1, weights 0, so
 * the plans made from them hold no expert for it and a layer gives it the added part alone. */
#define MAYA_ROUTER_NORM_NONE 0
#define MAYA_ROUTER_NORM_CLAMP 1
#define MAYA_ROUTER_NORM_HF 2
int maya_moe_route_sigmoid(const float* logits, const float* bias, int n_tokens, int n_expert, int k, float w_scale, int norm,
                           int32_t* ids, float* weights, void* stream);
/* Route and plan in one launch (router NULL: the softmax router; else see maya_router below): ids, weights and
 * plan_ptr[e] = expert_table[ids[e]] - the routing and look-up of glmf::moe_route (include/strata/kernels/glm_fast.hpp:424-433)
 * without its residency tiers. */
struct maya_router;
int maya_moe_route_plan(const struct maya_router* router, const float* logits, int n_tokens, int n_expert, int k,
                        const uint64_t* expert_table, int32_t* ids, float* weights, uint64_t* plan_ptr, void* stream);
/* The residency tiers of the routed experts, decided on the device per routed expert: glmf::MoeDev's tables
 * (include/strata/kernels/glm_fast.hpp:284-296) and the plan part of moe_route that reads them
 * (src/kernels/cuda/glm_fast.cu:4262-4375).  key = layer * n_expert + expert.  tab is ONE device array: tab[key] != 0 =
 * the expert's blob is in HBM at that address (a hit); else tab[n_keys + key] != 0 = it is in the second tier at that
 * address (pinned host memory mapped to the device, or any memory the device reads): it goes into one of the layer's
 * MAYA_SPARES spare slots (tab[2 n_keys + layer * MAYA_SPARES + j] != 0 = a free HBM slot; the device takes it, clears it
 * and writes tab[key] itself: resident from here on) or, with no spare left or fewer than promote_min counted routes,
 * into the next unused slot of scratch[n_scratch]; fetch_src[e] names its source.  In neither table: plan_ptr[e] = 0 and
 * the miss mask says so (moe_route hands those to the host over its request ring; that ring, its CPU lane, the next
 * layer's prefetch and the disk tier stay the engine's).  masks[4 t + 0..3] = token t's entries (bit i = its i-th) that
 * missed / have a fetch source / were promoted / found no slot (left out: plan_ptr 0).  counts ([n_keys] or NULL) are the
 * routes a key (moe_route's dcnt), halved each time seq ([1] or NULL: the routes so far) reaches a multiple of 4096.
 * The n_tokens rows are planned one after another, as one moe_route call a token of a window. */
#define MAYA_SPARES 3
typedef struct maya_residency {
    uint64_t* tab;             /* [2 * n_keys + n_layers * MAYA_SPARES] */
    int32_t n_keys;            /* n_layers * n_expert */
    int32_t n_layers;
    const uint64_t* scratch;   /* [n_scratch] HBM slots */
    int32_t n_scratch;
    int32_t reserved;
    uint64_t* fetch_src;       /* [n_tokens * k] out */
    uint32_t* counts;          /* [n_keys] or NULL */
    uint32_t* seq;             /* [1] or NULL */
    uint32_t* masks;           /* [n_tokens * 4] out */
} maya_residency;
int maya_moe_route_tiered(const struct maya_router* router, const float* logits, int n_tokens, int layer, int n_expert, int k,
                          const maya_residency* r, int promote_min, int32_t* ids, float* weights, uint64_t* plan_ptr,
                          void* stream);
/* Copies every planned entry with a fetch source into its slot: moe_fetch (glm_fast.hpp:468-469, glm_fast.cu:4688-4704). */
int maya_moe_fetch(const uint64_t* fetch_src, const uint64_t* plan_ptr, int n_entries, size_t blob_bytes, void* stream);
/* The copy of a prefetch list: moe_prefetch (glm_fast.hpp:473-474, glm_fast.cu:4619-4627, 7105-7123) - *pf_n entries (a
 * DEVICE count, read by the kernel; clamped to max_entries) of blob_bytes each from pf_src[i] (HBM or mapped host memory)
 * to pf_dst[i]; a null source or slot is skipped.  n_workgroups: how many workgroups copy (the call is meant for a side
 * stream beside the layer's kernels, and every compute unit it holds is one they wait for); 0 = half the compute units,
 * the reference's default.  Which experts to prefetch, and their slots, stay the engine's decision. */
int maya_moe_prefetch(const uint64_t* pf_src, const uint64_t* pf_dst, const int32_t* pf_n, int max_entries, size_t blob_bytes,
                      int n_workgroups, void* stream);
/* tab[keys[i]] = vals[i], the engine's edits between tokens: tab_update (glm_fast.cu:7745-7754); n_words = the array's
 * length (a key outside it is ignored). */
int maya_moe_tab_update(uint64_t* tab, int n_words, const int32_t* keys, const uint64_t* vals, int n, void* stream);
/* ids -> plan: plan_ptr[e] = expert_table[ids[e]] (0 stays 0: not resident), the plan part of moe_route_kernel
 * (src/kernels/cuda/glm_fast.cu:3998-4545) without its residency tiers. */
int maya_moe_plan(const int32_t* ids, int n_entries, const uint64_t* expert_table, int n_expert, uint64_t* plan_ptr,
                  void* stream);
/* plan -> groups of distinct experts, in first-appearance order, entries of a group ascending:
 * moe_win_group_kernel (src/kernels/cuda/glm_fast.cu:7545-7625), MoeWin (include/strata/kernels/glm_fast.hpp:439-458).
 * grp_ptr / grp_ent: [n_entries]; grp_start: [n_entries+1]; n_groups: [1]. */
int maya_moe_group(const uint64_t* plan_ptr, int n_entries, uint64_t* grp_ptr, int32_t* grp_start, int32_t* grp_ent,
                   int32_t* n_groups, void* stream);

/* A window's routing, plan and groups in ONE launch (the softmax router, up to 256 experts, n_tokens * k <= 256): what
 * maya_moe_route_plan followed by maya_moe_group writes, bit for bit - one workgroup routes the tokens a wave each and
 * groups their plans itself (glmf::moe_route + moe_win_group_kernel, include/strata/kernels/glm_fast.hpp:424-458,
 * src/kernels/cuda/glm_fast.cu:7545-7625).  maya_moe_route_window_ok: 1 when the arguments are covered;
 * maya_moe_layer_decode* and maya_exl3_layer_decode take this launch for windows of up to four tokens (the workgroup
 * routes four tokens at a time: beyond that the separate launches, a workgroup a token, are faster). */
int maya_moe_route_window_ok(const struct maya_router* router, int n_tokens, int n_expert, int k);
int maya_moe_route_window(const struct maya_router* router, const float* logits, int n_tokens, int n_expert, int k,
                          const uint64_t* expert_table, int32_t* ids, float* weights, uint64_t* plan_ptr, uint64_t* grp_ptr,
                          int32_t* grp_start, int32_t* grp_ent, int32_t* n_groups, void* stream);

/* ---- the expert rows.
 * maya_moe_gate_up: h[e][r] = swiglu(gate_r . x[token(e)], up_r . x[token(e)]) for every entry:
 *   glmf::moe_gate_up (include/strata/kernels/glm_fast.hpp:496-498), iq::gate_up (src/ds4/ds4_iq.cuh:88-89),
 *   native_gu_rows_split (src/kernels/cpu/native_expert.cpp:343-393).
 * maya_moe_down: part[e][r] = down_r . hq[e], then out[t] = sum_i plan_w[t*k+i] * part[t*k+i] (+ add[t]) in slot order:
 *   glmf::moe_down (glm_fast.hpp:499-501), iq::down (ds4_iq.cuh:90-91), native_down_rows_split
 *   (native_expert.cpp:395-417), native_moe_combine (src/kernels/cuda/native_moe.cu:36-52). */
int maya_moe_gate_up(const maya_moe_args* a, void* stream);
/* 1 when maya_moe_down, given hq = {NULL, NULL, NULL}, rounds h to the down type's activation format itself for these
 * arguments (native_quant_h's arithmetic, in the kernel's prologue; part may then be NULL), 0 when hq must be given. */
int maya_moe_down_rounds_h(const maya_moe_args* a);
int maya_moe_down(const maya_moe_args* a, void* stream);

/* ---- dense quantized mat-vecs beside the routed block (the shared expert's and the dense layers' projections):
 * glmf::mv / glmf::MvJob (include/strata/kernels/glm_fast.hpp:23-55): y[c][r] = alpha * (W_r . x[c]) + (bias ? bias[r] : 0)
 * for r in [0, n_out), c in [0, ncol).  The same weights meet ncol activations (a verify window's tokens); each column's
 * sum is the single-column call's, bit for bit, and a row's weights are decoded once for up to 4 columns.  The
 * activations are in the weight type's activation format (maya_quant_act: Q8_K for the K- and I-quants, Q8_0 for Q8_0 -
 * the CPU path's contract; the reference's GPU form takes q8_1).  Up to MAYA_MV_MAX_JOBS independent jobs a call; jobs
 * of one weight type share a launch.  n_in a multiple of 256, ncol <= MAYA_MAX_TOKENS. */
#define MAYA_MV_MAX_JOBS 8
typedef struct maya_mv_job {
    const void* w;        /* n_out rows of n_in values of `type`, MAYA_PACK_GGUF or (IQ2_S: n_out a multiple of 4) MAYA_PACK_STREAM */
    int32_t type, packing;
    int32_t n_in, n_out;
    int32_t ncol;
    float alpha;
    maya_act x;           /* [ncol][n_in] quantized activations */
    const float* bias;    /* [n_out] or NULL */
    float* y;             /* column c at y + c * y_stride */
    int64_t y_stride;     /* floats; >= n_out */
} maya_mv_job;
int maya_mv_supported(int type);                                              /* glmf::mv_supported (glm_fast.hpp:52) */
int maya_mv(const maya_mv_job* jobs, int n_jobs, void* stream);               /* glmf::mv / mv_nt (glm_fast.hpp:45-50) */

/* ---- the whole routed layer for a decode step / verify window of n_tokens <= MAYA_MAX_TOKENS tokens:
 * route -> plan -> group -> quantize x -> gate/up -> quantize h -> down -> combine, every step on `stream`, nothing on
 * the host (the sequence of glm_fast_path.cu:2688-2691 and ds4_gguf.cu:1903-1971).
 *   expert_table: [n_expert] device array of blob addresses (0: not resident);
 *   x: [n_tokens][n_embd] of x_dtype; out: [n_tokens][n_embd] F32; ids / weights: [n_tokens][k] results of the router;
 *   logits NULL (here, in maya_moe_prefill_layer and in maya_exl3_layer_decode): the tokens are already routed - ids and
 *   weights are inputs (any router's: maya_moe_route_sigmoid, the engine's own) and the layer starts at the plan;
 *   workspace: maya_moe_workspace_bytes(layout, n_tokens, k) bytes, 256-byte aligned. */
size_t maya_moe_workspace_bytes(const maya_moe_layout* l, int n_tokens, int k);
int maya_moe_layer_decode(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k,
                          const float* logits, const void* x, int x_dtype, int n_tokens, float limit, const float* add,
                          int32_t* ids, float* weights, float* out, void* workspace, size_t workspace_bytes,
                          void* stream);
/* The same layer with the router named: NULL or kind MAYA_ROUTER_SOFTMAX = maya_moe_route_topk's (router_top10),
 * MAYA_ROUTER_SIGMOID = maya_moe_route_sigmoid's with this bias, w_scale and norm - the route of glmf::moe_route
 * (include/strata/kernels/glm_fast.hpp:424-433) in the head's launch. */
#define MAYA_ROUTER_SOFTMAX 0
#define MAYA_ROUTER_SIGMOID 1
typedef struct maya_router {
    int32_t kind;
    int32_t norm;        /* sigmoid: MAYA_ROUTER_NORM_* */
    const float* bias;   /* sigmoid: NULL or [n_expert] */
    float w_scale;       /* sigmoid: routed_scaling_factor */
} maya_router;
int maya_moe_layer_decode_routed(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k,
                                 const maya_router* router, const float* logits, const void* x, int x_dtype, int n_tokens,
                                 float limit, const float* add, int32_t* ids, float* weights, float* out, void* workspace,
                                 size_t workspace_bytes, void* stream);

/* The same layer in its two halves, for a caller that puts work of its own between them or times them apart (the
 * reference's engines call glmf::moe_route / moe_gate_up and moe_down one by one, glm_fast_path.cu:2688-2691):
 *   _begin: route -> plan -> group -> quantize x -> gate/up, h left in the workspace;
 *   _end:   quantize h -> down -> combine, from that workspace.
 * Both take maya_moe_layer_decode_routed's arguments, the same in both calls; _begin followed by _end on one stream
 * launches what that call launches, in the same order, and gives its bits. */
int maya_moe_layer_decode_begin(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k,
                                const maya_router* router, const float* logits, const void* x, int x_dtype, int n_tokens,
                                float limit, const float* add, int32_t* ids, float* weights, float* out, void* workspace,
                                size_t workspace_bytes, void* stream);
int maya_moe_layer_decode_end(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k,
                              const maya_router* router, const float* logits, const void* x, int x_dtype, int n_tokens,
                              float limit, const float* add, int32_t* ids, float* weights, float* out, void* workspace,
                              size_t workspace_bytes, void* stream);

/* The routed layer and the expert EVERY token takes (a shared expert), side by side:
 *   out[t] = shared->add[t] + shared_expert(x[t]) + sum_j weights[t][j] * expert_{ids[t][j]}(x[t]).
 * The reference runs the shared expert's down rows as extra blocks of the routed experts' gate/up launch
 * (include/strata/kernels/glm_fast.hpp:496-501, src/kernels/cuda/glm_fast.cu:4841-4849) so that they cost no time of
 * their own; here the shared expert's launches (quantize x, gate/up, quantize h, down + add) go to a second stream that
 * the library keeps a device (default priority), forked from `stream` by an event when the call starts and joined back
 * before the routed down launch, which adds the routed experts to the shared expert's output.  Every result is the bits
 * of maya_moe_gate_up / maya_moe_down on `shared` followed by maya_moe_layer_decode_routed with add = shared->out.
 *   shared: the stage arguments of the shared expert as maya_moe_gate_up / maya_moe_down take them - k = 1, n_tokens
 *   entries, plan_ptr all its blob, plan_w all 1, its groups (one group of n_tokens entries), its own x / h / hq (NULL
 *   where the down kernel rounds h itself) / part buffers, `add` the layer's residual or NULL, `out` its own
 *   [n_tokens][n_embd] buffer (not the layer's out).
 * The fork and the join are event records and waits, so the call may be captured in a HIP graph (maya_init() first).
 * Every refusal of the stages (status > 0) is found before the fork: such a call has launched nothing on either stream.
 * Calls on one device are serialised on the host by a lock.  The device has ONE such second stream: while `stream` is being
 * captured that second stream belongs to the capture until hipStreamEndCapture, and a call from any other stream (eager,
 * or inside another capture) in between is refused with MAYA_E_BUSY and launches nothing - the open capture is not
 * disturbed and may call again.  After a HIP error (status < 0) `stream` has joined the second stream again when the
 * call returns. */
int maya_moe_layer_decode_shared(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k,
                                 const maya_router* router, const float* logits, const void* x, int x_dtype, int n_tokens,
                                 float limit, const maya_moe_args* shared, int32_t* ids, float* weights, float* out,
                                 void* workspace, size_t workspace_bytes, void* stream);

/* The same layer for callers that cannot allocate or own a workspace (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the workspace is a file-scope device array of MAYA_STATIC_SCRATCH_BYTES inside the
 * library, one copy a device, held until the process ends.  No counterpart in the reference (its callers own every buffer,
 * include/strata/kernels/s2_expert_grouped.hpp:36-38).  The call allocates nothing and sets nothing up: maya_init() must
 * have run on the current device (it fails with MAYA_E_ARG otherwise); a call whose maya_moe_workspace_bytes exceeds
 * MAYA_STATIC_SCRATCH_BYTES fails with MAYA_E_SHAPE and launches nothing (7168 x 2048, k 8: up to 3 tokens).  Every call on a
 * device shares that device's array: calls that overlap on one device (two streams, two threads) race; calls ordered on
 * one stream do not, and nothing has to be cleared between them (every region is written before it is read). */
#define MAYA_STATIC_SCRATCH_BYTES (1u << 20)
int maya_moe_layer_decode_static(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k,
                                 const maya_router* router, const float* logits, const void* x, int x_dtype, int n_tokens,
                                 float limit, const float* add, int32_t* ids, float* weights, float* out, void* stream);

/* ============================================================================================= prefill
 * A prompt chunk's routed experts as a grouped GEMM (the reference's expert_count_kernel / expert_scatter_kernel,
 * src/kernels/cuda/glm_batch.cu:2102-2133, with the host's prefix sum of src/prefill/glm_prefill.cu:3339-3361 done on
 * the device; mmq::quantize / Context::run / run_glu, src/prefill/moe_mmq.cu:120-228; the per-32 int8 activation
 * format of src/prefill/moe_fused_rdna4.cu:87-109 and its requantized H, :620-660).
 * Entry e = t * k + j is token t's j-th expert.  The plan sorts the entries by expert, stably: expert x's rows are
 * bounds[x] .. bounds[x + 1], row r serves entry row_entry[r], entry e sits at row entry_row[e] (-1: its expert is not
 * resident or its id is out of range).  Tiles of at most maya_moe_prefill_tile_rows() rows of one expert are what a
 * workgroup of the GEMM kernels takes; all counts stay on the device, so nothing here synchronises. */
typedef struct maya_prefill_plan {
    int32_t* bounds;      /* [n_expert + 1] */
    int32_t* row_entry;   /* [n_entries] */
    int32_t* entry_row;   /* [n_entries] */
    int32_t* tile_expert; /* [maya_moe_prefill_max_tiles()] */
    int32_t* tile_row0;   /* [maya_moe_prefill_max_tiles()] */
    int32_t* n_tiles;     /* [1] */
} maya_prefill_plan;
/* Rows of activations in the CPU expert path's format for the K-quants, Q8_K (src/kernels/cuda/quantize_act.cu:161-207):
 * int8 codes c = min(127, nearest_int(x * (-127 / max))) with max the signed value at the first largest magnitude of a
 * 256-value block, one F32 scale d = 1 / (-127 / max) per block, and s = d * (the sum of every 32 codes), which the
 * minimums of a Q4_K sub-block multiply.  The reference's two GPU prefill forms round per 32 values instead (q8_1,
 * src/prefill/moe_mmq.cu:120; int8 + F32, src/prefill/moe_fused_rdna4.cu:87-109); this one reproduces the integer
 * sums of the CPU path, which is what its results are checked against. */
typedef struct maya_prefill_act {
    int8_t* q; /* [rows][k], 16-byte aligned */
    float* d;  /* [rows][k / 256] */
    uint16_t* s; /* [rows][k / 256][16] FP16, 16-byte aligned: a block's 8 sub-block code sums as two digits, sum = lo + 64 hi:
                  * the 8 lo (0..63), then the 8 hi (-64..63) */
} maya_prefill_act;

int maya_moe_prefill_tile_rows(void);
int maya_moe_prefill_max_tiles(int n_entries, int n_expert);
/* 1 when the prefill GEMMs take this weight type: Q4_K (either packing; 16-byte aligned matrices) and IQ2_S (the stream
 * packing, rows of a multiple of 512 values); gate and up of one type, down of either (the mixed experts) */
int maya_moe_prefill_supported(int type);
int maya_moe_prefill_plan(const int32_t* ids, int n_entries, const uint64_t* expert_table, int n_expert,
                          const maya_prefill_plan* plan, void* stream);
/* row r = the quantized x[row_entry[r] / k] for the plan's rows (rows past bounds[n_expert] are left alone) */
int maya_moe_prefill_quant(const void* x, int x_dtype, int64_t x_stride, const maya_prefill_plan* plan, int n_entries,
                           int n_expert, int k, int64_t n_embd, maya_prefill_act xq, void* stream);
/* h row r [n_ff] F32 = swiglu(gate_e . x_r, up_e . x_r) (clamped by limit), e the row's expert, and hq = its rounding
 * (both written): int8 MFMA over two planes of the weights (their 4-bit codes times the low and the high 3 bits of
 * their 6-bit sub-block scales) and the activation codes, int32 over a 256-value block - ggml_vec_dot_q4_K_q8_K's
 * integer sums - then the two F32 scales of the block.  Matrix offsets 16-byte aligned (GGUF packing). */
int maya_moe_prefill_gate_up(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, const maya_prefill_plan* plan,
                             int n_entries, maya_prefill_act xq, float limit, float* h, maya_prefill_act hq, void* stream);
/* part row r [n_embd] F32 = down_e . h_r */
int maya_moe_prefill_down(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, const maya_prefill_plan* plan,
                          int n_entries, maya_prefill_act hq, float* part, void* stream);
/* out[t] = sum_j weights[t][j] * part[entry_row[t k + j]] in slot order (+ add[t]), stored as out_dtype */
int maya_moe_prefill_combine(const maya_prefill_plan* plan, const float* weights, const float* part, int n_tokens, int k,
                             int64_t n_embd, const float* add, void* out, int out_dtype, void* stream);
/* route -> plan -> quantize -> gate/up -> down -> combine of one chunk, all on `stream`.  A chunk holds at most 8192 tokens
 * and at most 65535 entries (n_tokens * k: the entries are a grid dimension of the quantizers); a larger call is refused
 * with MAYA_E_SHAPE before anything is launched - 8192 tokens at k = 8 is one entry too many, 8191 fit.  The stage calls
 * (maya_moe_prefill_plan / _quant / _gate_up / _down) share the entry limit. */
size_t maya_moe_prefill_workspace_bytes(const maya_moe_layout* l, int n_tokens, int k, int n_expert);
int maya_moe_prefill_layer(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k, const float* logits,
                           const void* x, int x_dtype, int n_tokens, float limit, const float* add, int32_t* ids,
                           float* weights, void* out, int out_dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ================================================================================================ EXL3
 * EXL3 (exllamav3) trellis weights: a matrix with k inputs and n outputs is `trellis` uint32 [k/16][n/16][4*k2]
 * (16x16 tiles, 16*k2 bytes each, k2 = twice the bits per weight), FP16 `suh` [k] and `svh` [n];
 *   y = H(H(x * suh) W') * svh,   H = the 128-point Sylvester-Hadamard transform over sqrt(128), per 128 values,
 * W' decoded from each tile's 256 16-bit trellis states (include/strata/kernels/exl3.hpp:4-22). */
#define MAYA_TYPE_EXL3 200 /* exl3::kTypeEXL3 (include/strata/kernels/exl3.hpp:32) */

/* One routed expert's blob: exl3::ExpertLayout (include/strata/kernels/exl3.hpp:96-103): for each of gate, up, down the
 * byte offsets of its suh, svh and trellis from the blob base (trellis 4-byte aligned, suh / svh 2-byte), its k2, and
 * the codebook (0 3inst, 1 mcg, 2 mul1). */
typedef struct maya_exl3_layout {
    uint64_t suh[3], svh[3], trellis[3];
    int32_t k2[3];
    int32_t cb;
    int32_t n_embd, n_ff; /* multiples of 128 */
} maya_exl3_layout;

/* exl3::MoeArgs / exl3::WinArgs (include/strata/kernels/exl3.hpp:118-168): the routed experts of n_tokens tokens,
 * entry e = token e / k, slot e % k; groups as in maya_moe_args (NULL grp_ptr: group g = entry g). */
typedef struct maya_exl3_args {
    maya_exl3_layout layout;
    int32_t n_tokens, k;
    const uint64_t* plan_ptr;
    const float* plan_w;
    const uint64_t* grp_ptr;
    const int32_t* grp_start;
    const int32_t* grp_ent;
    const int32_t* n_groups;
    const int32_t* skip;
    float limit;        /* SwiGLU clamp; 0 or +inf: none */
    const float* x;     /* [n_tokens][x_stride] F32 */
    int64_t x_stride;   /* floats between tokens (0: n_embd) */
    float* h;           /* [n_tokens*k][n_ff] */
    float* part;        /* [n_tokens*k][n_embd]: down's per-entry outputs; given to maya_exl3_gate_up it also serves as
                         * scratch for gate/up's partial outputs (the faster, split form); NULL there: the fused form */
    const float* add;   /* NULL or [n_tokens][n_embd] (the CPU lane's part: exl3::MoeArgs::cpu_part / cpu_flag) */
    const int32_t* add_flag;
    const float* add2;  /* NULL or [n_tokens][n_embd] added after `add`, always (exl3::moe_down's sh_out) */
    float* out;         /* [n_tokens][n_embd] */
} maya_exl3_args;

/* Offsets of the nine pieces of an expert blob (suh, svh, trellis of gate, up and down) for n_embd x n_ff experts at k2[3]
 * (gate, up, down) and codebook cb; returns the blob's bytes (0: a shape or bitrate the kernels do not take).
 * MAYA_EXL3_ORDER_SCALES_FIRST: a part is [suh | svh | trellis], every piece on a 16-byte boundary - the order of the reference
 * test's blobs (tests/exl3_test.cu:415-439).  MAYA_EXL3_ORDER_TRELLIS_FIRST: a part is [trellis | suh | svh], every piece a
 * multiple of 256 bytes - the blob the engine assembles from a pack (tools/exl3_pack.py:315-349). */
#define MAYA_EXL3_ORDER_SCALES_FIRST 0
#define MAYA_EXL3_ORDER_TRELLIS_FIRST 1
size_t maya_exl3_layout_init(maya_exl3_layout* l, int n_embd, int n_ff, const int32_t* k2, int cb, int order);
/* A layer's expert blobs assembled on the device from the experts' pieces where the model's files keep them, as the engine
 * assembles them from exl3.txt's rows (tools/exl3_pack.py:315-349, 596-612: per expert and part a trellis, a suh and an svh
 * range of a safetensors file): pieces[9 e + 3 r + {0, 1, 2}] = the address (device memory, or host memory mapped to the
 * device) of expert e's part r's trellis / suh / svh, 0 = leave that piece alone; blob e at dst + e * dst_stride gets each
 * piece at its offset in `l` (sizes from l's shape and bitrates). */
int maya_exl3_pack_experts(const maya_exl3_layout* l, const uint64_t* pieces, int n_expert, void* dst, size_t dst_stride,
                           void* stream);
/* exl3::k2_supported (include/strata/kernels/exl3.hpp:56-58) */
int maya_exl3_supported(int k2, int cb);
/* bytes of a k x n trellis at k2: exl3::trellis_bytes_k2 (exl3.hpp:50-52) */
size_t maya_exl3_trellis_bytes(int64_t k, int64_t n, int k2);
/* the decoded W' [k][n] as FP16 bits, exactly the codebook's values: exl3::reconstruct_inner (exl3.hpp:213-214) */
int maya_exl3_reconstruct_inner(const uint32_t* trellis, int64_t k, int64_t n, int k2, int cb, uint16_t* dst, void* stream);
/* exl3::moe_gate_up / moe_down / win_experts (exl3.hpp:133-169): h = clamped swiglu of the gate and up products;
 * part[e] = the down product of h[e]; out[t] = sum_i plan_w * part in slot order (+ add). */
int maya_exl3_gate_up(const maya_exl3_args* a, void* stream);
int maya_exl3_down(const maya_exl3_args* a, void* stream);
/* route -> plan -> group -> gate/up -> down -> combine for n_tokens <= MAYA_MAX_TOKENS tokens, all on `stream` */
size_t maya_exl3_workspace_bytes(const maya_exl3_layout* l, int n_tokens, int k);
int maya_exl3_layer_decode(const maya_exl3_layout* l, const uint64_t* expert_table, int n_expert, int k, const float* logits,
                           const float* x, int n_tokens, float limit, const float* add, int32_t* ids, float* weights,
                           float* out, void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif
