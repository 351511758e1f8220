// maya_probe: what this GPU gives the expert kernels to work with, measured with the kernels' own pieces.
//
// A standalone program (no part of libmaya_moe.so), printing
//   1. the shader clock (clock64 against the 100 MHz wall clock);
//   2. the issue rate of the vector instructions the decode uses, one dependent chain of 8 a wave, 16 waves a CU;
//   3. the LDS pipe's time for the codebook gather (ds_read_b64 at a random index) beside a conflict-free read;
//   4. the memory floor of the two expert kernels: their loads alone - same launch shape, same buffer-resource
//      addressing of the stream-packed quads (load_quad), every quad requested up front, the words folded into one
//      that is never stored - over rotating expert sets larger than the last-level cache;
//   5. the matrix instructions the prefill GEMMs use: time an instruction, alone and with vector instructions between them;
//   6. the prefill GEMM's weight stream alone, in the GEMM's own access pattern.
// The kernels' distances from their rooflines are read against these figures.
//
//   maya_probe [n_embd n_ff]      (default 7168 2048: the north-star expert; k = 8, 64 experts in rotation)
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#include <algorithm>
#include <functional>
#include <vector>

#include "../../include/maya_moe.h"
#include "maya_dev.hpp"
namespace maya {
__device__ __forceinline__ float swiglu(float g, float u, float limit) {
    if (limit > 0.0f && limit < INFINITY) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
    }
    return __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, expf(-g))), u);
}
}  // namespace maya
#include "maya_fast.hpp"
using namespace maya;

#define CK(x)                                                                                     \
    do {                                                                                          \
        hipError_t e_ = (x);                                                                      \
        if (e_ != hipSuccess) {                                                                   \
            printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__);         \
            exit(1);                                                                              \
        }                                                                                         \
    } while (0)

// ---- 1. clocks
__global__ void clock_kernel(long long* out, int iters) {
    const long long c0 = clock64(), w0 = wall_clock64();
    float x = threadIdx.x;
    for (int i = 0; i < iters; ++i) x = x * 1.0001f + 0.5f;
    const long long c1 = clock64(), w1 = wall_clock64();
    if (threadIdx.x == 0 && blockIdx.x == 0) out[0] = c1 - c0, out[1] = w1 - w0, out[2] = (long long) x;
}

// ---- 2. issue rates: 8 independent chains a lane, each instruction depending on its chain's last
#define OPK(NAME, ASM)                                                                                                      \
    __global__ __launch_bounds__(512) void op_##NAME(int* out, int iters) {                                                 \
        int a = threadIdx.x, b = threadIdx.x * 3 + 1, c0 = 1, c1 = 2, c2 = 3, c3 = 4, c4 = 5, c5 = 6, c6 = 7, c7 = 8;        \
        for (int i = 0; i < iters; ++i) {                                                                                   \
            asm volatile(ASM(%0) "\n" ASM(%1) "\n" ASM(%2) "\n" ASM(%3) "\n" ASM(%4) "\n" ASM(%5) "\n" ASM(%6) "\n" ASM(%7) \
                         : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3), "+v"(c4), "+v"(c5), "+v"(c6), "+v"(c7)                   \
                         : "v"(a), "v"(b));                                                                                 \
        }                                                                                                                   \
        if (c0 + c1 + c2 + c3 + c4 + c5 + c6 + c7 == 0x7fffffff) out[0] = 1;                                                \
    }
#define A_XOR(d) "v_xor_b32 " #d ", %8, " #d
#define A_ADD(d) "v_add_u32 " #d ", %8, " #d
#define A_DOT4(d) "v_dot4_i32_i8 " #d ", %8, %9, " #d
#define A_ANDOR(d) "v_and_or_b32 " #d ", %8, %9, " #d
#define A_MUL24(d) "v_mul_i32_i24 " #d ", %8, " #d
#define A_CVT(d) "v_cvt_f32_i32 " #d ", " #d
#define A_FMA(d) "v_fma_f32 " #d ", %8, %9, " #d
#define A_PERM(d) "v_perm_b32 " #d ", %8, %9, " #d
#define A_BFE(d) "v_bfe_u32 " #d ", " #d ", 3, 8"
#define A_LSHL(d) "v_lshlrev_b32 " #d ", 3, " #d
#define A_PKMUL(d) "v_pk_mul_lo_u16 " #d ", %8, " #d
#define A_LSHLADD(d) "v_lshl_add_u32 " #d ", " #d ", 3, %8"
#define A_MULLO(d) "v_mul_lo_u32 " #d ", %8, " #d
OPK(xor, A_XOR) OPK(add, A_ADD) OPK(dot4, A_DOT4) OPK(andor, A_ANDOR) OPK(mul24, A_MUL24) OPK(cvt, A_CVT) OPK(fma, A_FMA) OPK(perm, A_PERM)
OPK(bfe, A_BFE) OPK(lshl, A_LSHL) OPK(pkmul16, A_PKMUL) OPK(lshladd, A_LSHLADD) OPK(mullo32, A_MULLO)

// ---- 3. LDS reads: four chains a lane, the next index taken from the value read
template <int MODE>  // 0: b64 at a random index of 1024 (the IQ2_S codebook gather); 1: b64 conflict-free; 2: b32 random; 3: b64 one address
__global__ __launch_bounds__(512) void lds_kernel(unsigned* out, int iters) {
    __shared__ uint2 tab[1024];
    for (int i = threadIdx.x; i < 1024; i += 512) tab[i] = make_uint2(i * 2654435761u, i * 40503u + 7);
    __syncthreads();
    unsigned a0 = threadIdx.x * 7, a1 = threadIdx.x * 13 + 1, a2 = threadIdx.x * 29 + 5, a3 = threadIdx.x * 31 + 3, acc = 0;
    const unsigned lane = threadIdx.x & 63;
    for (int i = 0; i < iters; ++i) {
        uint2 v0, v1, v2, v3;
        if (MODE == 0) {
            v0 = tab[a0 & 1023], v1 = tab[a1 & 1023], v2 = tab[a2 & 1023], v3 = tab[a3 & 1023];
        } else if (MODE == 1) {
            v0 = tab[lane + (a0 & 960)], v1 = tab[lane + (a1 & 960)], v2 = tab[lane + (a2 & 960)], v3 = tab[lane + (a3 & 960)];
        } else if (MODE == 2) {
            const unsigned* t = (const unsigned*) tab;
            v0.x = t[a0 & 1023], v1.x = t[a1 & 1023], v2.x = t[a2 & 1023], v3.x = t[a3 & 1023];
            v0.y = v1.y = v2.y = v3.y = 1;
        } else {
            v0 = tab[a0 & 0], v1 = tab[(a1 & 0) + 1], v2 = tab[(a2 & 0) + 2], v3 = tab[(a3 & 0) + 3];
        }
        a0 += v0.x, a1 += v1.x, a2 += v2.x, a3 += v3.x;
        acc ^= v0.y ^ v1.y ^ v2.y ^ v3.y;
    }
    if (acc + a0 + a1 + a2 + a3 == 0x12345) out[0] = acc;
}

// ---- 5. matrix instructions: 4 independent accumulators a wave, NV vector instructions (independent xor chains) after each
typedef int pr_v4i __attribute__((ext_vector_type(4)));
typedef int pr_v16i __attribute__((ext_vector_type(16)));
typedef float pr_v4f __attribute__((ext_vector_type(4)));
#define VALU_FILL(NV)                                                                                     \
    if (NV >= 1) asm volatile("v_xor_b32 %0, %1, %0" : "+v"(x0) : "v"(k0));                               \
    if (NV >= 2) asm volatile("v_xor_b32 %0, %1, %0" : "+v"(x1) : "v"(k0));                               \
    if (NV >= 3) asm volatile("v_xor_b32 %0, %1, %0" : "+v"(x2) : "v"(k0));                               \
    if (NV >= 4) asm volatile("v_xor_b32 %0, %1, %0" : "+v"(x3) : "v"(k0));                               \
    if (NV >= 5) asm volatile("v_xor_b32 %0, %1, %0\n v_xor_b32 %2, %1, %2" : "+v"(x0), "+v"(x1) : "v"(k0)); \
    if (NV >= 7) asm volatile("v_xor_b32 %0, %1, %0\n v_xor_b32 %2, %1, %2" : "+v"(x2), "+v"(x3) : "v"(k0));
// KIND 0: v_mfma_i32_16x16x64_i8, 1: v_mfma_i32_32x32x32_i8, 2: v_mfma_f32_16x16x4_f32, 3: v_mfma_i32_16x16x32_i8
template <int KIND, int NV>
__global__ __launch_bounds__(256) void mfma_kernel(int* out, int iters) {
    pr_v4i a = {(int) threadIdx.x, 1, 2, 3}, b = {(int) threadIdx.x * 3, 5, 6, 7};
    int x0 = threadIdx.x, x1 = 1, x2 = 2, x3 = 3, k0 = 0x55;
    int r = 0;
    if constexpr (KIND == 1) {
        pr_v16i c[4] = {};
        for (int i = 0; i < iters; ++i) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(c[j]) : "v"(a), "v"(b));
                VALU_FILL(NV)
            }
        }
        r = c[0][0] + c[1][1] + c[2][2] + c[3][3];
    } else if constexpr (KIND == 2) {
        pr_v4f c[4] = {};
        float fa = threadIdx.x, fb = 1.5f;
        for (int i = 0; i < iters; ++i) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0" : "+v"(c[j]) : "v"(fa), "v"(fb));
                VALU_FILL(NV)
            }
        }
        r = (int) (c[0][0] + c[1][1] + c[2][2] + c[3][3]);
    } else {
        pr_v4i c[4] = {};
        for (int i = 0; i < iters; ++i) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (KIND == 0) asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(c[j]) : "v"(a), "v"(b));
                else asm volatile("v_mfma_i32_16x16x32_i8 %0, %1, %2, %0" : "+v"(c[j]) : "v"(*(long*) &a), "v"(*(long*) &b));
                VALU_FILL(NV)
            }
        }
        r = c[0][0] + c[1][1] + c[2][2] + c[3][3];
    }
    if (r + x0 + x1 + x2 + x3 == 0x7fffffff) out[0] = r;
}

// ---- 6. the prefill GEMM's weight stream alone: waves that sweep 32 Q4_K rows (144-byte blocks) a super-block a step, the
// next step's loads in flight during a token amount of arithmetic, a barrier a step - the GEMM's loop without its arithmetic
typedef unsigned int pr_u4 __attribute__((ext_vector_type(4)));
template <int LDSKB>
__global__ __launch_bounds__(256) void q4k_sweep_kernel(const unsigned char* pool, size_t expert_bytes, int row_bytes, unsigned* sink) {
    __shared__ unsigned char pad[LDSKB * 1024];   // (sets the workgroups a CU: 2 at 56 KB, as the GEMM's)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 31, kh = lane >> 5;
    const unsigned char* row = pool + (size_t) blockIdx.y * expert_bytes + (size_t) (blockIdx.x * 128 + wave * 32 + n) * row_bytes;
    const int steps = row_bytes / 144;
    pr_u4 cur[5], nxt[5];
    auto ld = [&](int st, pr_u4* d) {
        const unsigned char* blk = row + (size_t) st * 144;
        d[0] = *(const pr_u4*) blk;
#pragma unroll
        for (int c = 0; c < 4; ++c) d[1 + c] = *(const pr_u4*) (blk + 16 + 32 * c + 16 * kh);
    };
    ld(0, cur);
    unsigned x = 0;
    for (int s = 0; s < steps; ++s) {
        if (s + 1 < steps) ld(s + 1, nxt);
#pragma unroll
        for (int p = 0; p < 5; ++p) x ^= cur[p].x ^ cur[p].y ^ cur[p].z ^ cur[p].w;
        for (int i = 0; i < 32; ++i) x = x * 1664525u + 1013904223u;
        __syncthreads();
#pragma unroll
        for (int p = 0; p < 5; ++p) cur[p] = nxt[p];
    }
    if (x == 0x12345678u) sink[0] = x, pad[threadIdx.x] = 1;
}

// ---- 4. the expert kernels' loads alone
__device__ __forceinline__ uint32_t fold(const QuadIQ2S& q) {
    return q.is01.x ^ q.is01.y ^ q.is01.z ^ q.is01.w ^ q.is23.x ^ q.is23.y ^ q.is23.z ^ q.is23.w ^ q.hs.x ^ q.hs.y ^ q.d.x ^ q.d.y;
}
// down: grid n_embd / ROWS, 8 waves a workgroup, wave w reads slot w's ROWS rows (all n_ff / 32 sub-blocks: one a lane)
template <int ROWS, int NU>
__global__ __launch_bounds__(512, 2) void down_loads_kernel(maya_moe_args a, uint32_t* sink) {
    constexpr int NQ = ROWS / 4;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint64_t blob = a.plan_ptr[min(wave, a.k - 1)];
    constexpr uint32_t qb = NU / 8 * 82 * 4;
    const uint64_t mat = blob + a.layout.down_off;
    const uint32_t lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) mat);
    const uint32_t hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (mat >> 32));
    const __amdgpu_buffer_rsrc_t rs = weight_rsrc(((uint64_t) hi << 32) | (uint64_t) lo, (uint32_t) (a.layout.n_embd >> 2) * qb);
    const QuadOffs qo = quad_offs<NU>(0u, lane);
    const uint32_t quad0 = (uint32_t) (blockIdx.x * ROWS >> 2) * qb;
    QuadIQ2S ring[NQ];
#pragma unroll
    for (int d = 0; d < NQ; ++d) ring[d] = load_quad(rs, qo, quad0 + (uint32_t) d * qb);
    uint32_t x = 0;
#pragma unroll
    for (int d = 0; d < NQ; ++d) x ^= fold(ring[d]);
    if (x == 0x12345678u) sink[0] = x;
}
// gate/up: grid (n_ff / ROWS, k), NW waves a workgroup, half the lanes on gate and half on up, one sub-block a lane
template <int NW, int ROWS>
__global__ __launch_bounds__(64 * NW, 4) void gate_up_loads_kernel(maya_moe_args a, uint32_t* sink) {
    constexpr int NU = 32 * NW, NQ = ROWS / 4;
    const int t = threadIdx.x;
    const bool is_up = t >= NU;
    const int u = is_up ? t - NU : t;
    const uint64_t blob = a.plan_ptr[blockIdx.y];
    constexpr uint32_t qb = NU / 8 * 82 * 4;
    const __amdgpu_buffer_rsrc_t rs = weight_rsrc(blob + a.layout.gate_off, (uint32_t) (a.layout.down_off - a.layout.gate_off));
    const QuadOffs qo = quad_offs<NU>(is_up ? (uint32_t) (a.layout.up_off - a.layout.gate_off) : 0u, u);
    const uint32_t quad0 = (uint32_t) (blockIdx.x * ROWS >> 2) * qb;
    QuadIQ2S ring[NQ];
#pragma unroll
    for (int d = 0; d < NQ; ++d) ring[d] = load_quad(rs, qo, quad0 + (uint32_t) d * qb);
    uint32_t x = 0;
#pragma unroll
    for (int d = 0; d < NQ; ++d) x ^= fold(ring[d]);
    if (x == 0x12345678u) sink[0] = x;
}
__global__ void fill_kernel(uint32_t* p, size_t n, uint32_t seed) {
    size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t) gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        uint32_t x = (uint32_t) i * 2654435761u + seed;
        x ^= x >> 15, x *= 0x2c1b3c6du, x ^= x >> 12;
        p[i] = x;
    }
}

// median over 5 rounds of `reps` launches, in microseconds a launch
static float time_us(hipStream_t s, int reps, const std::function<void(int)>& f) {
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    for (int i = 0; i < 8; ++i) f(i);
    CK(hipStreamSynchronize(s));
    std::vector<float> t;
    for (int r = 0; r < 5; ++r) {
        CK(hipEventRecord(e0, s));
        for (int i = 0; i < reps; ++i) f(i);
        CK(hipEventRecord(e1, s));
        CK(hipEventSynchronize(e1));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        t.push_back(ms * 1e3f / reps);
    }
    std::sort(t.begin(), t.end());
    CK(hipEventDestroy(e0));
    CK(hipEventDestroy(e1));
    return t[t.size() / 2];
}

int main(int argc, char** argv) {
    const int E = argc > 2 ? atoi(argv[1]) : 7168, FF = argc > 2 ? atoi(argv[2]) : 2048, NE = 64, K = 8, NSETS = NE / K;
    if (E != 7168 || FF != 2048) {
        printf("maya_probe: the load kernels are instantiated for 7168 x 2048 only\n");
        return 2;
    }
    hipStream_t s;
    CK(hipStreamCreate(&s));
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount, simds = 4 * cus;
    printf("device %s, %d CUs\n", prop.gcnArchName, cus);

    long long* dclk;
    CK(hipMalloc(&dclk, 64));
    double shader_mhz = 0;
    {
        int rate = 0;
        CK(hipDeviceGetAttribute(&rate, hipDeviceAttributeWallClockRate, 0));
        long long h[3];
        for (int rep = 0; rep < 3; ++rep) {
            hipLaunchKernelGGL(clock_kernel, dim3(4 * cus), dim3(512), 0, s, dclk, 200000);
            CK(hipStreamSynchronize(s));
            CK(hipMemcpy(h, dclk, 24, hipMemcpyDeviceToHost));
            shader_mhz = (double) h[0] / ((double) h[1] / rate) / 1000.0;
        }
        printf("1. shader clock under a vector-ALU load: %.0f MHz (clock64 against the %d kHz wall clock)\n", shader_mhz, rate);
    }
    {
        printf("2. vector instruction issue, 16 waves a CU, 8 dependent chains a wave (wave-instructions / ns / SIMD; clk an instruction)\n");
        const int iters = 4000, wgs = 8 * cus;
#define RUN_OP(NAME)                                                                                                  \
    {                                                                                                                 \
        const float us = time_us(s, 2, [&](int) { hipLaunchKernelGGL(op_##NAME, dim3(wgs), dim3(512), 0, s, (int*) dclk, iters); }); \
        const double instr = (double) wgs * 8 * iters * 8, rate = instr / (us * 1e3) / simds;                         \
        printf("   %-8s %.2f  (%.1f clk)\n", #NAME, rate, shader_mhz * 1e-3 / rate);                                  \
    }
        RUN_OP(xor) RUN_OP(add) RUN_OP(fma) RUN_OP(dot4) RUN_OP(andor) RUN_OP(mul24) RUN_OP(cvt) RUN_OP(perm) RUN_OP(bfe) RUN_OP(lshl) RUN_OP(pkmul16) RUN_OP(lshladd) RUN_OP(mullo32)
    }
    {
        printf("3. LDS reads, 16 waves a CU, 4 chains a wave (clk a wave-instruction a CU)\n");
        const int iters = 2000, wgs = 4 * cus;
#define RUN_LDS(M, NAME)                                                                                               \
    {                                                                                                                  \
        const float us = time_us(s, 2, [&](int) { hipLaunchKernelGGL(lds_kernel<M>, dim3(wgs), dim3(512), 0, s, (unsigned*) dclk, iters); }); \
        const double instr = (double) wgs * 8 * iters * 4;                                                             \
        printf("   %-34s %.1f\n", NAME, us * 1e3 / (instr / cus) * shader_mhz * 1e-3);                                 \
    }
        RUN_LDS(0, "b64 at a random index of 1024") RUN_LDS(1, "b64 conflict-free") RUN_LDS(2, "b32 at a random index of 1024") RUN_LDS(3, "b64 one address")
    }
    {
        printf("5. matrix instructions, W waves a SIMD, 4 accumulators a wave, NV xor after each (clk a matrix instruction a SIMD)\n");
        printf("   %-28s %8s %8s %8s %8s %8s\n", "", "NV=0", "NV=2", "NV=4", "NV=6", "NV=8");
        const int iters = 2000;
#define RUN_MFMA_1(KIND, NV, W, dst)                                                                                               \
    {                                                                                                                              \
        const float us = time_us(s, 2, [&](int) { hipLaunchKernelGGL((mfma_kernel<KIND, NV>), dim3(W * cus), dim3(256), 0, s, (int*) dclk, iters); }); \
        dst = us * 1e3 / ((double) W * iters * 4) * shader_mhz * 1e-3;                                                             \
    }
#define RUN_MFMA(KIND, W, NAME)                                                                                                    \
    {                                                                                                                              \
        double c0, c2, c4, c6, c8;                                                                                                 \
        RUN_MFMA_1(KIND, 0, W, c0) RUN_MFMA_1(KIND, 2, W, c2) RUN_MFMA_1(KIND, 4, W, c4) RUN_MFMA_1(KIND, 6, W, c6) RUN_MFMA_1(KIND, 8, W, c8) \
        printf("   %-22s W=%d %8.1f %8.1f %8.1f %8.1f %8.1f\n", NAME, W, c0, c2, c4, c6, c8);                                      \
    }
        RUN_MFMA(0, 1, "i32_16x16x64_i8") RUN_MFMA(0, 2, "i32_16x16x64_i8") RUN_MFMA(0, 4, "i32_16x16x64_i8")
        RUN_MFMA(3, 1, "i32_16x16x32_i8") RUN_MFMA(3, 2, "i32_16x16x32_i8")
        RUN_MFMA(1, 1, "i32_32x32x32_i8") RUN_MFMA(1, 2, "i32_32x32x32_i8")
        RUN_MFMA(2, 1, "f32_16x16x4_f32") RUN_MFMA(2, 2, "f32_16x16x4_f32")
    }
    {
        const size_t gr = (size_t) E / 256 * 82, dr = (size_t) FF / 256 * 82;
        const size_t up_off = gr * FF, down_off = 2 * gr * FF, blob = down_off + dr * E;
        uint8_t* pool;
        CK(hipMalloc(&pool, NE * blob));
        hipLaunchKernelGGL(fill_kernel, dim3(4096), dim3(256), 0, s, (uint32_t*) pool, NE * blob / 4, 12345u);
        uint64_t* plans;
        CK(hipMalloc(&plans, NE * 8));
        std::vector<uint64_t> p(NE);
        for (int i = 0; i < NE; ++i) p[i] = (uint64_t) (pool + (size_t) i * blob);
        CK(hipMemcpy(plans, p.data(), NE * 8, hipMemcpyHostToDevice));
        uint32_t* sink;
        CK(hipMalloc(&sink, 64));
        auto args = [&](int set) {
            maya_moe_args a{};
            a.layout.gate_type = a.layout.up_type = a.layout.down_type = MAYA_TYPE_IQ2_S;
            a.layout.n_embd = E, a.layout.n_ff = FF;
            a.layout.gate_off = 0, a.layout.up_off = up_off, a.layout.down_off = down_off, a.layout.packing = MAYA_PACK_STREAM;
            a.n_tokens = 1, a.k = K, a.plan_ptr = plans + set * K;
            return a;
        };
        const double gu_bytes = 2.0 * gr * FF * K, dn_bytes = (double) dr * E * K;
        printf("4. the expert kernels' loads alone, %d sets of %d experts in rotation (%.0f MB a set; gate/up %.1f MB, down %.1f MB a launch)\n", NSETS, K,
               blob * K / 1e6, gu_bytes / 1e6, dn_bytes / 1e6);
        float t = time_us(s, 64, [&](int i) { hipLaunchKernelGGL((gate_up_loads_kernel<7, 16>), dim3(FF / 16, K), dim3(448), 0, s, args(i % NSETS), sink); });
        printf("   gate/up, 16 rows a workgroup (the kernel's shape)  %6.2f us  %.0f GB/s\n", t, gu_bytes / t / 1e3);
        t = time_us(s, 64, [&](int i) { hipLaunchKernelGGL((gate_up_loads_kernel<7, 32>), dim3(FF / 32, K), dim3(448), 0, s, args(i % NSETS), sink); });
        printf("   gate/up, 32 rows a workgroup                       %6.2f us  %.0f GB/s\n", t, gu_bytes / t / 1e3);
        t = time_us(s, 64, [&](int i) { hipLaunchKernelGGL((gate_up_loads_kernel<7, 8>), dim3(FF / 8, K), dim3(448), 0, s, args(i % NSETS), sink); });
        printf("   gate/up, 8 rows a workgroup                        %6.2f us  %.0f GB/s\n", t, gu_bytes / t / 1e3);
        t = time_us(s, 64, [&](int i) { hipLaunchKernelGGL((down_loads_kernel<28, 64>), dim3(E / 28), dim3(512), 0, s, args(i % NSETS), sink); });
        printf("   down, 28 rows a workgroup (the kernel's shape)     %6.2f us  %.0f GB/s\n", t, dn_bytes / t / 1e3);
        t = time_us(s, 64, [&](int i) { hipLaunchKernelGGL((down_loads_kernel<56, 64>), dim3(E / 56), dim3(512), 0, s, args(i % NSETS), sink); });
        printf("   down, 56 rows a workgroup                          %6.2f us  %.0f GB/s\n", t, dn_bytes / t / 1e3);
        {
            // 6: the pool read as 48 "experts" of 4096 Q4_K rows of 7168 values (4032 bytes a row)
            const int rows = 4096, row_bytes = 4032, ne = 48;
            const size_t eb = (size_t) rows * row_bytes;
            if ((size_t) ne * eb <= (size_t) NE * blob) {
                const float tq = time_us(s, 4, [&](int) { hipLaunchKernelGGL(q4k_sweep_kernel<56>, dim3(rows / 128, ne), dim3(256), 0, s, pool, eb, row_bytes, sink); });
                printf("6. the prefill GEMM's weight stream alone (Q4_K rows of 4032 bytes, 32 rows a wave, 144 bytes a row a step, 2 workgroups a CU)\n");
                printf("   %d x %d rows  %8.2f us  %.0f GB/s\n", ne, rows, tq, (double) ne * eb / tq / 1e3);
            }
        }
        t = time_us(s, 16, [&](int i) { CK(hipMemcpyAsync(pool + (size_t) ((i + 1) % NSETS) * K * blob, pool + (size_t) (i % NSETS) * K * blob, (size_t) K * blob, hipMemcpyDeviceToDevice, s)); });
        printf("   for scale: a device copy of one set (%.0f MB read + written)  %6.2f us  %.0f GB/s\n", 2.0 * blob * K / 1e6, t, 2.0 * blob * K / t / 1e3);
    }
    return 0;
}
