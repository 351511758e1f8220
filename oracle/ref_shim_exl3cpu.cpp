// ref_shim_exl3cpu.cpp - TEST INFRASTRUCTURE: a C entry point over the reference's CPU lane for EXL3 experts
// (include/strata/kernels/cpu/exl3_cpu.hpp, src/kernels/cpu/exl3_cpu.cpp: what ds4::exl3_experts,
// src/ds4/ds4_cpu_exl3.hpp:245-394, computes each routed matrix with).  The lane keeps the mul1 codebook's affine form
// WITHOUT the FP16 rounding of the weights and of the rotated input that the device form (and exl3_ref.cpp) has, so it is
// a second, independent statement of an EXL3 mat-vec: the two agree to the FP16 roundings, not to the bit.
// exl3_cpu.cpp and expert_layout.cpp (the CPU feature probe it calls) are compiled where they lie; the vector code in
// them is gated by function-level target attributes, so no file-wide instruction-set option is needed and the library
// loads on any x86-64.
#include <cstdint>
#include <vector>

#include "strata/kernels/cpu/exl3_cpu.hpp"

extern "C" {

// 2 AVX-512, 1 AVX2 + FMA, 0 scalar: the kernel ref_exl3_cpu_mv runs here
int ref_exl3_cpu_tier(void) { return strata::kernels::cpu::exl3_cpu_tier(); }
int ref_exl3_cpu_k2_ok(int k2) { return strata::kernels::cpu::exl3_cpu_k2_ok(k2) ? 1 : 0; }

// y[n] = H(H(x * suh) W') * svh for one mul1 matrix (k, n multiples of 128): exl3_cpu_prepare, then every 128-column band
int ref_exl3_cpu_mv(const uint32_t* trellis, const uint16_t* suh, const uint16_t* svh, int k, int n, int k2, const float* x, float* y) {
    using namespace strata::kernels::cpu;
    if (k <= 0 || n <= 0 || k % 128 || n % 128 || !exl3_cpu_k2_ok(k2) || !exl3_cpu_available()) return 1;
    Exl3Part m;
    m.trellis = trellis, m.suh = suh, m.svh = svh, m.k = k, m.n = n, m.k2 = k2;
    std::vector<float> xh((size_t) k);
    const float xsum = exl3_cpu_prepare(m, x, xh.data());
    for (int c0 = 0; c0 < n; c0 += 128) exl3_cpu_band(m, xh.data(), xsum, c0, y + c0);
    return 0;
}

}  // extern "C"
