// ref_shim_q80.cpp - TEST INFRASTRUCTURE: a C entry point over the reference's x86 Q8_0 activation quantizer, the
// "pinned ggml CPU Q8_0 contract" of src/kernels/cpu/expert.cpp:92-130 (quantize_oracle_q8_0, adapted there from
// llama.cpp's ggml-cpu/arch/x86/quants.c quantize_row_q8_0), reached through its public switch
// (include/strata/kernels/cpu/expert.hpp:98-107).  expert.cpp is compiled where it lies, with the options its own
// CMakeLists.txt gives it (AVX-512 VNNI / VBMI: CMakeLists.txt:1513-1514), into a library of its own
// (oracle/_ref/libmaya_ref_q80.so) so that nothing else has to load AVX-512 code; it runs in the build container only,
// to write tests/golden/refbuild_q80_vectors.npz and to check the CPU checker against it there.
#include <cstdint>
#include <cstring>

#include "strata/kernels/cpu/expert.hpp"

extern "C" {

int ref_q80_max_values(void) { return strata::kernels::cpu::H; }

// x: n floats (a multiple of 32, at most ref_q80_max_values()) -> q[n] codes, scale[n / 32] = the FP16 block scales as F32
int ref_q80_quant(const float* x, int n, int8_t* q, float* scale) {
    using namespace strata::kernels::cpu;
    if (n % QKA != 0 || n > H || n <= 0) return 1;
    static ActQ a;
    expert_set_oracle_q8_0(true);
    act_quant_q8_1(x, n, a);
    std::memcpy(q, a.q, (size_t) n);
    std::memcpy(scale, a.scale, (size_t) (n / QKA) * sizeof(float));
    return 0;
}

}  // extern "C"
