// ref_shim.cpp - TEST INFRASTRUCTURE: C entry points over the reference's own CPU expert sources, so the tests can hold
// maya_oracle.c to them bit for bit.  This file is the only source of the reference build that lives in this
// repository; everything else is compiled from where it lies in the reference tree (oracle/Makefile, REF=...), the
// result goes to oracle/_ref/ and is never committed.  It exists only in a container that has the reference tree.
#include <cstddef>
#include <cstdint>
#include <cstring>

#include "strata/artifact/dequant.hpp"        // dequantize_q4_K, dequantize_q8_0, fp16_to_fp32
#include "strata/kernels/cpu/exl3_ref.hpp"    // exl3_decode, exl3_tile_states_k2, exl3_inner_k2, exl3_had128, exl3_mv
#include "strata/kernels/cpu/iq_avx2.hpp"     // iq256_rows, iq256_gu_rows
#include "strata/kernels/f16_bits.hpp"        // f16_from_f32
#include "ds4_lane_parity.hpp"                // par::quant, gate_up_ref, down_ref, row_ref
#include "ds4_par_exp.h"                      // exp_portable, swiglu_portable

extern "C" {

float ref_f16_to_f32(uint16_t h) { return strata::fp16_to_fp32(h); }
uint16_t ref_f32_to_f16(float f) { return strata::kernels::f16_from_f32(f); }

void ref_dequant_q4_K(const uint8_t* blk, float* out) { strata::dequantize_q4_K(blk, out); }
void ref_dequant_q8_0(const uint8_t* blk, float* out) { strata::dequantize_q8_0(blk, out); }

int ref_iq256_supported(int type) { return strata::kernels::cpu::iq256_supported(type) ? 1 : 0; }
void ref_iq256_rows(int type, const uint8_t* w, size_t row_bytes, int n, const void* const* act, int nt,
                    float* const* out, int r0, int r1) {
    strata::kernels::cpu::iq256_rows(type, w, row_bytes, n, act, nt, out, r0, r1);
}
void ref_iq256_gu_rows(int type, const uint8_t* blob, size_t gu_row, size_t up_off, int n, const void* const* act,
                       int nt, float* const* ff, int r0, int r1) {
    strata::kernels::cpu::iq256_gu_rows(type, blob, gu_row, up_off, n, act, nt, ff, r0, r1);
}

size_t ref_par_act_bytes(int k) { return strata::ds4::par::act_bytes(k); }
void ref_par_quant(const float* x, int k, void* act) { strata::ds4::par::quant(x, k, act); }
float ref_par_row(int type, const uint8_t* row, int k, const void* act, int lpr) {
    return strata::ds4::par::row_ref(type, row, k, act, lpr);
}
void ref_par_gate_up(int type, const uint8_t* gate, const uint8_t* up, int k, const void* const* act, int nt,
                     float* const* h, int r0, int r1, float limit) {
    strata::ds4::par::gate_up_ref(type, gate, up, k, act, nt, h, r0, r1, limit);
}
void ref_par_down(int type, const uint8_t* down, int k, const void* const* act, int nt, float* const* y, int r0,
                  int r1) {
    strata::ds4::par::down_ref(type, down, k, act, nt, y, r0, r1);
}
float ref_exp_portable(float y) { return strata::ds4::par::exp_portable(y); }
float ref_swiglu_portable(float g, float u, float limit) { return strata::ds4::par::swiglu_portable(g, u, limit); }

float ref_exl3_decode(uint32_t state, int cb) { return strata::kernels::cpu::exl3_decode(state, cb); }
void ref_exl3_tile_states(const uint32_t* tile, int k2, uint16_t* st) {
    strata::kernels::cpu::exl3_tile_states_k2(tile, k2, st);
}
void ref_exl3_inner(const uint32_t* trellis, int ld, int k, int n, int k2, int cb, float* w) {
    strata::kernels::cpu::exl3_inner_k2(trellis, ld, k, n, k2, cb, w);
}
void ref_exl3_had128(float* v, size_t n) { strata::kernels::cpu::exl3_had128(v, n); }
void ref_exl3_mv(const float* w, const uint16_t* suh, const uint16_t* svh, int k, int n, const float* x, float* y) {
    strata::kernels::cpu::exl3_mv(w, suh, svh, k, n, x, y);
}

}  // extern "C"
