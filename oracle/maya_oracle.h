/* maya_oracle.h - TEST INFRASTRUCTURE, not product code.
 *
 * A plain-C, CPU restatement of the reference's routed-MoE expert arithmetic, used only as the checker by tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg.  Nothing under the product package may include, link or
 * call it; the product path is the HIP library and fails loudly when that is missing.
 *
 * Every function cites the reference file:line it follows (paths relative to the reference tree).  Built with
 * -ffp-contract=off so each float operation written here is rounded once, as the reference's CPU translation units are
 * (CMakeLists.txt:744-746 for the lane-parity unit; iq_avx2.cpp fuses only where it writes an explicit fmadd).
 *
 * Pinning status (what independent evidence holds each function to the reference):
 *   f16/bf16 conversions ............. exhaustive over all 65536 bit patterns against numpy (tests/test_oracle_formats.py)
 *   Q8_0 / Q4_K dequant .............. reference build oracle/_ref (include/strata/artifact/dequant.hpp:81-85,162-190) bit-exact;
 *                                       brute force over all 6-bit scale/min x nibble values
 *   IQ2_S dequant .................... structure check |w| = d(2ls+1)/8 * {8,25,43}; integer decode identical to the
 *                                       reference build's Fmt32<22>::decode through the row dots below; codebook CRC
 *   IQ1_M dequant .................... integer decode pinned through the reference build's iq256_rows(29,...)
 *   IQ2_XXS dequant .................. an independent numpy decode from the block layout (ggml-common.h:380-384) over every
 *                                       codebook index x sign index x scale, bit for bit; codebook CRC and the reference tree's
 *                                       table; the sign table's rule (bit 7 = parity of the low seven) checked against
 *                                       ksigns_iq2xs when the grids are generated; integer decode through the row dots below
 *   IQ1_S dequant .................... an independent numpy decode written from the block layout and dq_iq1_s's formula
 *                                       (ggml-common.h:425-430, src/kernels/cuda/iq_kernels.cu:825-837), bit for bit over every
 *                                       grid index x 3-bit scale x delta sign and on random blocks; the same values, bit for bit,
 *                                       as the IQ1_M block that carries the IQ1_S block's fields (tests/test_oracle_pins.py)
 *   IQ1_S row dot .................... the IQ1_M dot of that carrier block (itself bit-exact with the reference build's
 *                                       iq256_rows(29, ...)) and the reference build on the carrier, to 1e-6 of the terms'
 *                                       magnitude (only the order of the float sums differs); the float64 dot of the independent
 *                                       decode; block-permutation and block-scale invariants
 *   Q8_K activation quantizer ........ reference build: strata::ds4::par::quant (ds4_lane_parity.cpp:610-637) byte-exact;
 *                                       constructed exact ties
 *   Q8_0 activation quantizer ........ the reference's own x86 quantizer (quantize_oracle_q8_0 behind act_quant_q8_1,
 *                                       src/kernels/cpu/expert.cpp:92-130, compiled where it lies into oracle/_ref/libmaya_ref_q80.so):
 *                                       byte-exact on tests/golden/refbuild_q80_vectors.npz (the reference test's five
 *                                       distributions, both-sign maxima, scales past the FP16 range and in its subnormals) and live
 *                                       where that build exists; an independent float32 numpy closed form incl. exact halves of
 *                                       either sign and zero blocks; ggml's scalar form and the reference's GPU form counted
 *                                       against it (one code apart on < 2e-4 of N(0,1) values)
 *   Q8_0 x Q8_0 row dot .............. the float64 dot of both operands dequantized independently with numpy, 1e-6 of the terms'
 *                                       magnitude; block-permutation and negation invariants (exact where they must be)
 *   row dots IQ2_S/Q4_K/IQ1_M/IQ2_XXS  reference build: strata::kernels::cpu::iq256_rows / iq256_gu_rows, BIT-EXACT
 *                                       (this file restates the 8 int32 lanes and the float steps in their order)
 *   IQ2_S expert in device arithmetic  reference build: strata::ds4::par::gate_up_ref / down_ref, bit-exact
 *   SwiGLU ........................... closed form; exp_portable (ds4_par_exp.h:60-85) bit-exact against the reference build
 *   router top-k ..................... closed forms (all-equal logits, ties), float-p vs double-p cross-check
 *   sigmoid router ................... the reference's host form (router_sigmoid_parity.cpp:36-86, restated in double with a
 *                                       stable sort) on its own four case shapes incl. exact ties, to its tolerance (ids
 *                                       equal, weights 1e-5); closed forms (equal logits, a bias that selects but does not
 *                                       weigh, sum of weights = w_scale); the wrong readings the reference names must differ; non-finite
 *                                       rows refused as tests/hip/glm_handoff.cpp:186-207 expects (ids -1)
 *   combine .......................... closed form
 *   residency plan (mo_plan_tiered) .. worked examples written out by hand from the documented rule (include/strata/kernels/
 *                                       glm_fast.hpp:284-292): hits, spares in order, promotion, scratch, no slot left, a window's
 *                                       later token, promote_min against the counts, the counts' halving; the reference test's
 *                                       expectation for empty tables (miss mask 255, tests/hip/glm_handoff.cpp:118)
 *   EXL3 states / codebook ........... the reference's own golden vectors data/exl3-exllamav3 (13 .bin files made by exllamav3)
 *   EXL3 mat-vec ..................... reference build: exl3_ref.cpp bit-exact; H.H = I; the reference's CPU lane (exl3_cpu.cpp,
 *                                      unrounded weights: a second statement of the product) to 3e-4, golden vectors of whole experts
 *   prompt-chunk rows ................ the pieces above, row by row (the Q8_K quantizer, the Q4_K row dots, SwiGLU, combine):
 *                                       a chunk's row is the CPU path's expert on that row's token
 *   mo_grouped_ref / mo_quant_i8x32 .. helpers of the tests (a double product of dequantized weights x dequantized int8 rows,
 *                                       tests/hip/prefill_fused_parity.cpp:150-175; the per-32 rounding of
 *                                       src/prefill/moe_fused_rdna4.cu:87-109): an independent float64 numpy product; invariants
 */
#ifndef MAYA_ORACLE_H
#define MAYA_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids (src/ds4/ds4_iq.cuh:27-31) */
enum {
    MO_Q8_0 = 8,
    MO_Q4_K = 12,
    MO_IQ2_XXS = 16,
    MO_IQ1_S = 19,
    MO_IQ2_S = 22,
    MO_IQ1_M = 29,
};

#pragma pack(push, 1)
/* third_party/ggml/ggml-common.h:371-376 */
typedef struct {
    float d;
    int8_t qs[256];
    int16_t bsums[16];
} mo_q8k;
/* third_party/ggml/ggml-common.h:252-256 */
typedef struct {
    uint16_t d;
    int8_t qs[32];
} mo_q80;
#pragma pack(pop)

/* ---- scalar conversions (include/strata/artifact/dequant.hpp:33-62) */
float mo_f16_to_f32(uint16_t h);
uint16_t mo_f32_to_f16(float f); /* round to nearest even, as _cvtss_sh / the reference's f16_from_f32 */
float mo_bf16_to_f32(uint16_t h);
uint16_t mo_f32_to_bf16(float f); /* round to nearest even */

/* ---- codebooks expanded from iq_grids.h (third_party/ggml/ggml-common.h:758, 1135) */
const uint64_t* mo_iq2s_grid(void); /* 1024 entries */
const uint64_t* mo_iq1s_grid(void); /* 2048 entries */
const uint64_t* mo_iq2xxs_grid(void); /* 256 entries */
uint32_t mo_crc32(const void* p, size_t n);

/* ---- format geometry (src/ds4/ds4_iq.cuh:47-52) */
int mo_block_values(int type);
int mo_block_bytes(int type);
size_t mo_row_bytes(int type, int64_t k);

/* ---- dequantization: k values of one row (k a multiple of the block) */
int mo_dequant_row(int type, const uint8_t* row, int64_t k, float* out);

/* ---- activation quantizers */
void mo_quant_q8k(const float* x, int64_t k, mo_q8k* out);          /* src/kernels/cuda/quantize_act.cu:161-207 */
void mo_quant_q80(const float* x, int64_t k, mo_q80* out);          /* include/strata/kernels/quantize_act.hpp:28-31 */
void mo_quant_i8x32(const float* x, int64_t k, int8_t* q, float* d); /* src/prefill/moe_fused_rdna4.cu:87-109 */
/* bytes of the activation a weight type's dot takes (Q8_K for the 256-value types, Q8_0 for Q8_0) */
size_t mo_act_bytes(int type, int64_t k);
void mo_quant_act(int type, const float* x, int64_t k, void* out);

/* ---- one row's dot in the ggml CPU contract (src/kernels/cpu/iq_avx2.cpp:225-250, 332-394, 462-514) */
float mo_vec_dot(int type, const uint8_t* row, int64_t k, const void* act);
/* out[t][r] = w_r . act[t] for rows [r0, r1) (iq256_rows) */
void mo_rows(int type, const uint8_t* w, size_t row_bytes, int64_t k, const void* const* act, int nt, float* const* out,
             int r0, int r1);
/* ff[t][r] = swiglu(gate_r . act[t], up_r . act[t]) (native_gu_rows_split, src/kernels/cpu/native_expert.cpp:343-393) */
void mo_gu_rows(int type, const uint8_t* gate, const uint8_t* up, size_t row_bytes, int64_t k, const void* const* act,
                int nt, float* const* ff, int r0, int r1, float limit);
float mo_swiglu(float g, float u, float limit); /* limit = +inf: no clamp */

/* ---- a whole expert, one or several tokens (native_quant_act -> gu rows -> native_quant_h -> down rows):
 * out[t][n_embd].  gate / up / down: the three row arrays of the expert.  nthreads > 1 splits rows (OpenMP). */
void mo_expert(int gu_type, int d_type, const uint8_t* gate, const uint8_t* up, const uint8_t* down, int64_t n_embd,
               int64_t n_ff, const float* x, int nt, float limit, float* out, int nthreads);

/* ---- router (src/kernels/cuda/router_top10.cu:95-186; host form src/kernels/router_top10_parity.cpp:36-60) */
void mo_router_topk(const float* logits, int n_tokens, int n_expert, int k, int32_t* ids, float* weights);
void mo_router_topk_f64(const float* logits, int n_tokens, int n_expert, int k, int32_t* ids, float* weights);
/* ---- the sigmoid router (src/kernels/cuda/router_sigmoid.cu:44-73, moe_route_kernel src/kernels/cuda/glm_fast.cu:4050-4297;
 * host form src/kernels/router_sigmoid_parity.cpp:36-86).  norm: 0 none, 1 / max(sum, 2^-14), 2 / (sum + 1e-20).
 * A row with a non-finite logit or score gets ids -1 and weights 0 (src/kernels/cuda/glm_batch.cu:2077-2092). */
void mo_router_sigmoid(const float* logits, const float* bias, int n_tokens, int n_expert, int k, float w_scale, int norm,
                       int32_t* ids, float* weights);
void mo_router_sigmoid_f64(const float* logits, const float* bias, int n_tokens, int n_expert, int k, float w_scale, int norm,
                           int32_t* ids, float* weights);

/* ---- the residency plan over routed ids (moe_route_kernel's tiers, src/kernels/cuda/glm_fast.cu:4262-4375): tab =
 * [n_keys] HBM | [n_keys] second tier | [n_layers][3] spares, edited in place; see maya_oracle.c */
void mo_plan_tiered(const int32_t* ids, int n_tokens, int layer, int n_expert, int k, uint64_t* tab, int n_keys,
                    const uint64_t* scratch, int n_scratch, uint32_t* counts, uint32_t* seq, int promote_min,
                    uint64_t* plan, uint64_t* fetch_src, uint32_t* masks);

/* ---- combine (src/kernels/cuda/native_moe.cu:36-52): out[c] = sum_i w[i] * parts[i][c] in order i = 0..k-1 */
void mo_combine(const float* parts, const float* w, int k, int64_t n, float* out);

/* ---- the routed layer: route, run the k experts of every token, combine.  blobs[e] = expert e's
 * [gate rows | up rows | down rows].  out[t][n_embd]. */
void mo_moe_layer(int gu_type, int d_type, const uint8_t* const* blobs, int n_expert, int k, int64_t n_embd,
                  int64_t n_ff, const float* logits, const float* x, int n_tokens, float limit, int32_t* ids,
                  float* weights, float* out, int nthreads);

/* ---- device-arithmetic lane (src/ds4/ds4_lane_parity.cpp, src/ds4/ds4_par_exp.h) */
float mo_exp_portable(float y);
float mo_swiglu_portable(float g, float u, float limit); /* limit 0: no clamp */
float mo_row_lanes(int type, const uint8_t* row, int64_t k, const int8_t* q, const float* d32, int lpr);

/* ---- EXL3 (src/kernels/cpu/exl3_ref.cpp:11-94) */
float mo_exl3_decode(uint32_t state, int cb);
void mo_exl3_tile_states(const uint32_t* tile, int k2, uint16_t* st);
void mo_exl3_inner(const uint32_t* trellis, int ld, int k, int n, int k2, int cb, float* w);
void mo_exl3_had128(float* v, size_t n);
void mo_exl3_mv(const float* w, const uint16_t* suh, const uint16_t* svh, int k, int n, const float* x, float* y);

/* ---- synthetic weights: an own Q4_K / Q8_0 encoder for "quantized from N(0, 0.02)" inputs (the reference never
 * quantizes weights itself; oracle and device consume the same bytes, so parity does not depend on the encoder). */
void mo_encode_q4k(const float* x, int64_t k, uint8_t* out);
void mo_encode_q80(const float* x, int64_t k, uint8_t* out);

/* ---- prefill reference: y[r][c] = sum_i W_e[c][i] * (xq[r][i] * xd[r][i/32]) in double, rows sorted by expert */
void mo_grouped_ref(int type, const uint8_t* const* w, const int32_t* bounds, int n_expert, int64_t k, int64_t n,
                    const int8_t* xq, const float* xd, float* y, int nthreads);

#ifdef __cplusplus
}
#endif
#endif
