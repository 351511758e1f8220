// maya_exl3.hip - EXL3 (exllamav3 trellis) routed experts on gfx950: decode mat-vec kernels and their C ABI.
//
// A workgroup owns 128 output columns (one block of the output Hadamard transform): its 8 waves take one 16-column
// tile each and walk down the k / 16 row tiles.  For a tile a lane decodes 4 consecutive trellis steps - by the tile's
// element order (include/strata/kernels/exl3.hpp:15-16) those are 4 rows of ONE column - and multiplies them with the
// rotated, FP16-rounded activation held in LDS; the rotation H(x * suh) is done by the workgroup itself before the walk
// and the output rotation, the svh scaling, the SwiGLU and the FP32 stores after it.  Several activations (a verify
// window's tokens routed to one expert) share one decode of the weights.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <math.h>
#include <stdint.h>

#include <type_traits>

#include "maya_host.h"
#include "maya_dev.hpp"

namespace maya {

constexpr int kExThreads = 512;

// ---- codebooks: the value of a 16-bit state, as the FP16 bits the format defines (src/kernels/cpu/exl3_ref.cpp:11-27)
template <int CB>
__device__ __forceinline__ __half exl3_value(uint32_t state) {
    if constexpr (CB == 2) {
        // fp16(1024 + bytesum(state * 0x83DCD12D)) * fp16(0x1eee) + fp16(0xc931) in one FP16 FMA
        const uint32_t x = state * 0x83DCD12Du;
        const uint32_t bs = __builtin_amdgcn_sad_u8(x, 0u, 1024u);   // 1024 + the sum of the four bytes
        const __half h = __ushort2half_rn((unsigned short) bs);      // exact: an integer below 2048
        return __hfma(h, __ushort_as_half(0x1eee), __ushort_as_half(0xc931));
    } else {
        uint32_t x = CB == 1 ? state * 0xCBAC1FEDu : state * 89226354u + 64248484u;
        x = (x & 0x8fff8fffu) ^ 0x3b603b60u;
        return __hadd(__ushort_as_half((unsigned short) (x & 0xffffu)), __ushort_as_half((unsigned short) (x >> 16)));
    }
}

// step p's state of a tile whose 4 * k2 words are in t[] (LDS or registers): the 16-bit window that ends at bit
// floor((p + 1) k2 / 2) of the words read MSB-first, around the ring (src/kernels/cpu/exl3_ref.cpp:33-43)
__device__ __forceinline__ uint32_t exl3_state(const uint32_t* t, int k2, int p) {
    const int W = 4 * k2;
    const int e = ((p + 1) * k2) >> 1;            // the window's end bit, 1 .. 128 k2
    const int i1 = (e - 1) >> 5;                  // the word of its last bit
    const int i0 = e < 16 ? W - 1 : (e - 16) >> 5;  // ... of its first bit (before bit 0: the ring's last word)
    const int sh = ((i1 + 1) << 5) - e;
    const uint64_t m = ((uint64_t) t[i0] << 32) | (uint64_t) t[i1];
    return (uint32_t) (m >> sh) & 0xffffu;
}

// tile step p -> (row, column) inside the 16 x 16 tile (src/kernels/cpu/exl3_ref.cpp:52-55)
__device__ __forceinline__ void exl3_rc(int p, int& r, int& c) {
    const int lane = p >> 3, j = p & 7;
    r = (lane & 3) * 2 + (j & 1) + 8 * ((j >> 1) & 1);
    c = (lane >> 2) + 8 * (j >> 2);
}

template <int CB>
__global__ __launch_bounds__(256) void exl3_inner_kernel(const uint32_t* __restrict__ trellis, int64_t k, int64_t n, int k2,
                                                         uint16_t* __restrict__ dst) {
    __shared__ uint32_t t[64];
    const int64_t tiles_n = n >> 4;
    const int64_t tile = blockIdx.x;
    const int W = 4 * k2;
    if ((int) threadIdx.x < W) t[threadIdx.x] = trellis[tile * W + threadIdx.x];
    __syncthreads();
    const int p = threadIdx.x;
    int r, c;
    exl3_rc(p, r, c);
    const __half v = exl3_value<CB>(exl3_state(t, k2, p));
    const int64_t ks = tile / tiles_n, tc = tile % tiles_n;
    dst[(ks * 16 + r) * n + tc * 16 + c] = __half_as_ushort(v);
}

// ---- the blockwise Hadamard transform H / sqrt(128) of one 128-value block inside a wave: lane L holds values L and L + 64.
// Stage h < 64 pairs lane L with lane L ^ h (the lower index adds, the upper takes lower - upper), stage 64 pairs the
// lane's own two values: the butterflies, their order and every rounding are the reference's
// (src/kernels/cpu/exl3_ref.cpp:61-75), so the same bits.
// The partner's value comes through a DPP operand, a swizzle or the half-wave swap (xor_lane), not through __shfl_xor's
// LDS-routed permute: six exchanges a value, each of which was an LDS round trip.
template <int H>
__device__ __forceinline__ void had128_stage(float& v0, float& v1, int lane) {
    const float p0 = xor_lane<H>(v0), p1 = xor_lane<H>(v1);
    const bool upper = (lane & H) != 0;
    v0 = upper ? __fsub_rn(p0, v0) : __fadd_rn(v0, p0);
    v1 = upper ? __fsub_rn(p1, v1) : __fadd_rn(v1, p1);
}
__device__ __forceinline__ void had128_wave(float& v0, float& v1, int lane) {
    had128_stage<1>(v0, v1, lane);
    had128_stage<2>(v0, v1, lane);
    had128_stage<4>(v0, v1, lane);
    had128_stage<8>(v0, v1, lane);
    had128_stage<16>(v0, v1, lane);
    had128_stage<32>(v0, v1, lane);
    const float a = v0, c = v1;
    v0 = __fadd_rn(a, c);
    v1 = __fsub_rn(a, c);
    const float s = 1.0f / sqrtf(128.0f);
    v0 = __fmul_rn(v0, s);
    v1 = __fmul_rn(v1, s);
}

struct ExGroup {
    uint64_t blob;
    int e0, ne;
};
__device__ __forceinline__ bool ex_group_of(const maya_exl3_args& a, int g, ExGroup& r) {
    if (a.skip && *a.skip) return false;
    if (a.grp_ptr) {
        if (g >= *a.n_groups) return false;
        r.blob = a.grp_ptr[g];
        r.e0 = a.grp_start[g];
        r.ne = a.grp_start[g + 1] - r.e0;
    } else {
        if (g >= a.n_tokens * a.k) return false;
        r.blob = a.plan_ptr[g];
        r.e0 = g;
        r.ne = 1;
    }
    return r.blob != 0ull && r.ne > 0;
}
__device__ __forceinline__ int ex_entry_of(const maya_exl3_args& a, const ExGroup& r, int i) {
    return a.grp_ptr ? a.grp_ent[r.e0 + i] : r.e0;
}

// xr = FP16(H(x * suh)) of one activation into LDS; every wave of the workgroup takes blocks of 128 values (`tmp` is not
// used: the transform runs in registers)
// PAIRED (the compile-time walk): inside every 16 rows the word of rows 2q, 2q + 1 and the word of rows 2q + 8, 2q + 9 -
// a lane's four rows - sit side by side (words 2q, 2q + 1), so the walk reads them in one 8-byte LDS read
__device__ __forceinline__ int paired_pos(int i) {
    const int w = (i >> 1) & 7;
    return (i & ~15) | ((w < 4 ? 2 * w : 2 * (w - 4) + 1) << 1) | (i & 1);
}
template <bool PAIRED>
__device__ __forceinline__ void rotate_in(const float* __restrict__ x, const uint16_t* __restrict__ suh, int k, float* tmp,
                                          __half* xr) {
    (void) tmp;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nb = k >> 7;
    // a wave's blocks three at a time: their loads go out together (one block a pass of the loop is one trip to memory a
    // pass: the compiler waits for a pass's loads before it issues the next pass's)
    constexpr int kAtOnce = 3, kWaves = kExThreads / 64;
    for (int b0 = wave; b0 < nb; b0 += kAtOnce * kWaves) {
        float xa[kAtOnce], xb[kAtOnce];
        uint16_t sa[kAtOnce], sb[kAtOnce];
#pragma unroll
        for (int u = 0; u < kAtOnce; ++u) {
            const int b = b0 + u * kWaves;
            const int i0 = (b < nb ? b : b0) * 128 + lane;   // (past the end: the first block again, its result dropped)
            xa[u] = x[i0], xb[u] = x[i0 + 64];
            sa[u] = suh[i0], sb[u] = suh[i0 + 64];
        }
#pragma unroll
        for (int u = 0; u < kAtOnce; ++u) {
            const int b = b0 + u * kWaves;
            if (b < nb) {
                const int i0 = b * 128 + lane;
                float v0 = __fmul_rn(xa[u], f16_bits_to_f32(sa[u])), v1 = __fmul_rn(xb[u], f16_bits_to_f32(sb[u]));
                had128_wave(v0, v1, lane);
                xr[PAIRED ? paired_pos(i0) : i0] = __float2half_rn(v0);
                xr[PAIRED ? paired_pos(i0 + 64) : i0 + 64] = __float2half_rn(v1);
            }
        }
    }
    __syncthreads();
}
// the output rotation of nb blocks of 128 values in LDS, block b by wave b (nb <= 8), in place
__device__ __forceinline__ void had128_out(float* v, int nb) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (wave < nb) {
        float v0 = v[wave * 128 + lane], v1 = v[wave * 128 + lane + 64];
        had128_wave(v0, v1, lane);
        v[wave * 128 + lane] = v0;
        v[wave * 128 + lane + 64] = v1;
    }
    __syncthreads();
}

// One matrix's 16-column tile over all its row tiles for NT activations: returns this lane's partial sums for its column
// (the lane's 4 steps are rows 2q, 2q+1, 2q+8, 2q+9 of column (L >> 3) + 8 (L & 1), q = (L >> 1) & 3)
template <int CB, int NT>
__device__ __forceinline__ void walk_tiles(const uint32_t* __restrict__ trellis, int k, int ld, int tc, int k2, int lane,
                                           uint32_t* wt, const __half* xr, int xr_stride, float (&acc)[NT]) {
    const int W = 4 * k2, q = (lane >> 1) & 3;
    for (int ks = 0; ks < (k >> 4); ++ks) {
        const uint32_t* tile = trellis + ((size_t) ks * ld + tc) * W;
        if (lane < W) wt[lane] = tile[lane];
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0);  // the wave's own LDS writes have landed before any lane reads them
        float w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = __half2float(exl3_value<CB>(exl3_state(wt, k2, 4 * lane + i)));
        __builtin_amdgcn_wave_barrier();
        const int rb = ks * 16 + 2 * q;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const __half* xv = xr + t * xr_stride + rb;
            float s = acc[t];
            s = fmaf(w[0], __half2float(xv[0]), s);
            s = fmaf(w[1], __half2float(xv[1]), s);
            s = fmaf(w[2], __half2float(xv[8]), s);
            s = fmaf(w[3], __half2float(xv[9]), s);
            acc[t] = s;
        }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {  // the 4 lanes of a column: q = bits 1, 2 of the lane
        acc[t] += __shfl_xor(acc[t], 2, 64);
        acc[t] += __shfl_xor(acc[t], 4, 64);
    }
}

// ---- the same walk with the bit rate a compile-time constant (K2 <= 10, the mul1 codebook): no LDS staging of the tile.
// A lane's 4 windows span 16 + 3 K2 / 2 <= 31 bits, so they sit in the two words around the last window's end - two
// dword buffer loads at lane-constant offsets, the tile's address in the scalar offset - and one 64-bit shift puts all
// four into one register, where they are bit-field extracts at compile-time positions.  1024 + the byte sum is an FP16
// whose bit pattern is 0x6400 + the byte sum (one v_sad_u8); values are made two at a time (v_pk_fma_f16) and meet the
// FP16 activation pairs (rows 2q, 2q+1 and 2q+8, 2q+9 are adjacent) in v_dot2_f32_f16.
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
template <int K2> struct Taps {
    static constexpr int end(int i) { return ((i + 1) * K2) / 2; }       // end bit of step i above the lane's 2 L K2
    static constexpr int below(int i) { return end(3) - end(i); }        // how far window i ends before the last one
};
__device__ __forceinline__ h2 as_h2(uint32_t v) {
    union { uint32_t u; h2 h; } c;
    c.u = v;
    return c.h;
}
template <int K2>
__device__ __forceinline__ void tile_values(uint32_t wa, uint32_t wb, int sh, h2& w01, h2& w23) {
    const uint32_t c = __builtin_amdgcn_alignbit(wa, wb, (uint32_t) sh);   // (wa : wb) >> sh, 0 <= sh < 32
    uint32_t prod[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) prod[i] = __builtin_amdgcn_ubfe(c, Taps<K2>::below(i), 16) * 0x83DCD12Du;
    // 0x6400 + the byte sum (at most 1020: no carry out of the half) = the bits of FP16(1024 + byte sum); the pair's second
    // sum lands in the upper half directly (v_sad_hi_u8: (sum << 16) + the third operand), so the pair needs no packing
    const uint32_t p01 = __builtin_amdgcn_sad_hi_u8(prod[1], 0u, __builtin_amdgcn_sad_u8(prod[0], 0u, 0x64006400u));
    const uint32_t p23 = __builtin_amdgcn_sad_hi_u8(prod[3], 0u, __builtin_amdgcn_sad_u8(prod[2], 0u, 0x64006400u));
    const h2 kinv = as_h2(0x1eee1eeeu), kbias = as_h2(0xc931c931u);
    w01 = __builtin_elementwise_fma(as_h2(p01), kinv, kbias);
    w23 = __builtin_elementwise_fma(as_h2(p23), kinv, kbias);
}
template <int K2, int NT>
__device__ __forceinline__ void walk_tiles_fast(const uint32_t* __restrict__ trellis, int k, int ld, int tc, int lane,
                                                const __half* xr, int xr_stride, float (&acc)[NT]) {
    static_assert(K2 >= 2 && K2 <= 10, "the four windows of a lane must fit 32 bits");
    constexpr int W = 4 * K2;
    const int E = 2 * lane * K2 + Taps<K2>::end(3);   // the end bit of the lane's last window: 1 .. 128 K2
    const int ib = (E - 1) >> 5, ia = ib == 0 ? W - 1 : ib - 1;
    const int sh = 32 * (ib + 1) - E;
    const int q = (lane >> 1) & 3, nks = k >> 4;
    const uint64_t base = (uint64_t) trellis;
    const uint32_t b_lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) base);
    const uint32_t b_hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (base >> 32));
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*) (((uint64_t) b_hi << 32) | b_lo), 0,
                                                                         (int) ((uint32_t) nks * ld * W * 4), 0x00020000);
    const uint32_t oa = 4u * ia, ob = 4u * ib, step = (uint32_t) ld * W * 4;
    // (tc comes from the wave's index: uniform, but only readfirstlane tells the compiler so - a divergent scalar offset
    // would turn every load into a loop over the lanes)
    const uint32_t t_off = (uint32_t) __builtin_amdgcn_readfirstlane(tc) * W * 4;
    // A wave's row tiles are ld * W * 4 bytes apart (a 96-byte read every 9 KB at 3 bits a weight): only many reads in
    // flight keep the memory busy, so the walk runs kAhead tiles ahead in a ring of registers.
    constexpr int kAhead = 8;   // (k is a multiple of 128: the row tiles come in eights)
    uint32_t ra[kAhead], rb[kAhead];
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
        ra[i] = __builtin_amdgcn_raw_buffer_load_b32(rs, oa, t_off + (uint32_t) i * step, 0);
        rb[i] = __builtin_amdgcn_raw_buffer_load_b32(rs, ob, t_off + (uint32_t) i * step, 0);
    }
    const uint2* xw = (const uint2*) xr;   // the lane's two pairs of FP16 activations of a row tile (rotate_in<true>'s order)
    const int xs = xr_stride >> 2;
#pragma unroll 1
    for (int ks = 0; ks < nks; ks += kAhead) {
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
            const uint32_t ca = ra[i], cb = rb[i];
            const uint32_t nxt = t_off + (uint32_t) (ks + i + kAhead) * step;   // (past the matrix: the buffer returns 0)
            ra[i] = __builtin_amdgcn_raw_buffer_load_b32(rs, oa, nxt, 0);
            rb[i] = __builtin_amdgcn_raw_buffer_load_b32(rs, ob, nxt, 0);
            h2 w01, w23;
            tile_values<K2>(ca, cb, sh, w01, w23);
            const int rw = (ks + i) * 4 + q;   // rows 2q, 2q + 1 | 2q + 8, 2q + 9 of this row tile
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const uint2 xv = xw[t * xs + rw];
                acc[t] = __builtin_amdgcn_fdot2(w01, as_h2(xv.x), acc[t], false);
                acc[t] = __builtin_amdgcn_fdot2(w23, as_h2(xv.y), acc[t], false);
            }
        }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        acc[t] += __shfl_xor(acc[t], 2, 64);
        acc[t] += __shfl_xor(acc[t], 4, 64);
    }
}
// K2 > 0: the compile-time walk; 0: the general one
template <int CB, int NT, int K2>
__device__ __forceinline__ void walk(const uint32_t* __restrict__ trellis, int k, int ld, int tc, int k2, int lane,
                                     uint32_t* wt, const __half* xr, int xr_stride, float (&acc)[NT]) {
    if constexpr (K2 > 0) walk_tiles_fast<K2, NT>(trellis, k, ld, tc, lane, xr, xr_stride, acc);
    else walk_tiles<CB, NT>(trellis, k, ld, tc, k2, lane, wt, xr, xr_stride, acc);
}

__device__ __forceinline__ float ex_swiglu(float g, float u, float limit) {
    if (limit > 0.0f && limit < INFINITY) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
    }
    return __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, expf(-g))), u);
}

// dynamic LDS: [8 waves x 64 words of tile][NT x 2 x k halves of rotated inputs][NT*2*128 floats of raw outputs]
// grid (n_ff / 128, groups)
template <int CB, int NT, int K2>
__global__ __launch_bounds__(kExThreads) void exl3_gate_up_kernel(maya_exl3_args a) {
    extern __shared__ uint32_t lds[];
    ExGroup gr;
    if (!ex_group_of(a, blockIdx.y, gr)) return;
    const int k = a.layout.n_embd, n = a.layout.n_ff;
    uint32_t* wt = lds + (threadIdx.x >> 6) * 64;
    __half* xr = (__half*) (lds + 8 * 64);                       // [NT][2][k]
    float* tmp = (float*) (xr + (size_t) NT * 2 * k);            // the raw outputs [NT][2][128]
    const uint8_t* blob = (const uint8_t*) gr.blob;
    const int64_t xs = a.x_stride ? a.x_stride : k;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int tc = blockIdx.x * 8 + wave;
    // the group's entries two at a time while two are left (one decode of the weights serves both), else one
    auto chunk = [&](auto ntc, int c0) {
        constexpr int NTC = decltype(ntc)::value;
        int ents[NTC];
#pragma unroll
        for (int t = 0; t < NTC; ++t) ents[t] = ex_entry_of(a, gr, c0 + t);
        __syncthreads();
        for (int t = 0; t < NTC; ++t) {
            const float* x = a.x + (size_t) (ents[t] / a.k) * xs;
            for (int role = 0; role < 2; ++role)
                rotate_in<(K2 > 0)>(x, (const uint16_t*) (blob + a.layout.suh[role]), k, tmp, xr + ((size_t) t * 2 + role) * k);
        }
        float raw[2][NTC];
#pragma unroll
        for (int role = 0; role < 2; ++role) {
            float acc[NTC];
#pragma unroll
            for (int t = 0; t < NTC; ++t) acc[t] = 0.0f;
            walk<CB, NTC, K2>((const uint32_t*) (blob + a.layout.trellis[role]), k, n >> 4, tc, a.layout.k2[role], lane, wt,
                              xr + (size_t) role * k, 2 * k, acc);
#pragma unroll
            for (int t = 0; t < NTC; ++t) raw[role][t] = acc[t];
        }
        __syncthreads();
        // the lane with q = 0 of each column holds the sums: column (L >> 3) + 8 (L & 1) of the wave's tile
        if (((lane >> 1) & 3) == 0) {
            const int col = wave * 16 + (lane >> 3) + 8 * (lane & 1);
#pragma unroll
            for (int t = 0; t < NTC; ++t) {
                tmp[(t * 2 + 0) * 128 + col] = raw[0][t];
                tmp[(t * 2 + 1) * 128 + col] = raw[1][t];
            }
        }
        __syncthreads();
        had128_out(tmp, NTC * 2);
        const uint16_t* svg = (const uint16_t*) (blob + a.layout.svh[0]) + blockIdx.x * 128;
        const uint16_t* svu = (const uint16_t*) (blob + a.layout.svh[1]) + blockIdx.x * 128;
        for (int i = threadIdx.x; i < NTC * 128; i += kExThreads) {
            const int t = i >> 7, c = i & 127;
            const float g = __fmul_rn(tmp[(t * 2 + 0) * 128 + c], f16_bits_to_f32(svg[c]));
            const float u = __fmul_rn(tmp[(t * 2 + 1) * 128 + c], f16_bits_to_f32(svu[c]));
            a.h[(size_t) ents[t] * n + blockIdx.x * 128 + c] = ex_swiglu(g, u, a.limit);
        }
    };
    for (int c0 = 0; c0 < gr.ne;) {
        if (NT >= 2 && gr.ne - c0 >= 2) {
            chunk(std::integral_constant<int, 2>{}, c0);
            c0 += 2;
        } else {
            chunk(std::integral_constant<int, 1>{}, c0);
            c0 += 1;
        }
    }
}

// ---- gate/up split over more workgroups (the compile-time walk only): grid (n_ff / 128, groups, 2 KS), z = role KS + ks.
// A workgroup takes one role (gate or up) and one of KS slices of the rows: it rotates its slice of the input, walks
// its row tiles, rotates the 128 partial sums and scales them - rotation and scaling are linear, so the slices' partial
// outputs simply add - and stores them to P[entry][role][ks][n_ff] (the caller's `part` scratch).  exl3_swiglu_kernel adds the
// slices and applies the SwiGLU.  Twice 2 KS as many, shorter workgroups as the fused kernel: the chip fills evenly.
// dynamic LDS: [NT x k/KS halves of rotated input][NT*128 floats of raw outputs]
template <int NT, int K2>
__global__ __launch_bounds__(kExThreads) void exl3_gu_split_kernel(maya_exl3_args a, int KS) {
    extern __shared__ uint32_t lds[];
    ExGroup gr;
    if (!ex_group_of(a, blockIdx.y, gr)) return;
    const int role = blockIdx.z / KS, ks = blockIdx.z % KS;
    const int k = a.layout.n_embd, n = a.layout.n_ff, kb = k / KS;
    __half* xr = (__half*) lds;                         // [NT][kb]
    float* tmp = (float*) (xr + (size_t) NT * kb);      // the raw outputs [NT][128]
    const uint8_t* blob = (const uint8_t*) gr.blob;
    const int64_t xs = a.x_stride ? a.x_stride : k;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int tc = blockIdx.x * 8 + wave, ld = n >> 4;
    const uint32_t* trellis = (const uint32_t*) (blob + a.layout.trellis[role]) + (size_t) ks * (kb >> 4) * ld * (4 * K2);
    const uint16_t* suh = (const uint16_t*) (blob + a.layout.suh[role]) + (size_t) ks * kb;
    const uint16_t* sv = (const uint16_t*) (blob + a.layout.svh[role]) + blockIdx.x * 128;
    auto chunk = [&](auto ntc, int c0) {
        constexpr int NTC = decltype(ntc)::value;
        int ents[NTC];
#pragma unroll
        for (int t = 0; t < NTC; ++t) ents[t] = ex_entry_of(a, gr, c0 + t);
        __syncthreads();
        for (int t = 0; t < NTC; ++t)
            rotate_in<true>(a.x + (size_t) (ents[t] / a.k) * xs + (size_t) ks * kb, suh, kb, tmp, xr + (size_t) t * kb);
        float acc[NTC];
#pragma unroll
        for (int t = 0; t < NTC; ++t) acc[t] = 0.0f;
        walk_tiles_fast<K2, NTC>(trellis, kb, ld, tc, lane, xr, kb, acc);
        __syncthreads();
        if (((lane >> 1) & 3) == 0) {
            const int col = wave * 16 + (lane >> 3) + 8 * (lane & 1);
#pragma unroll
            for (int t = 0; t < NTC; ++t) tmp[t * 128 + col] = acc[t];
        }
        __syncthreads();
        had128_out(tmp, NTC);
        for (int i = threadIdx.x; i < NTC * 128; i += kExThreads) {
            const int t = i >> 7, c = i & 127;
            a.part[(((size_t) ents[t] * 2 + role) * KS + ks) * n + blockIdx.x * 128 + c] = __fmul_rn(tmp[t * 128 + c], f16_bits_to_f32(sv[c]));
        }
    };
    for (int c0 = 0; c0 < gr.ne;) {
        if (NT >= 2 && gr.ne - c0 >= 2) {
            chunk(std::integral_constant<int, 2>{}, c0);
            c0 += 2;
        } else {
            chunk(std::integral_constant<int, 1>{}, c0);
            c0 += 1;
        }
    }
}
// grid (n_ff / 256, entries): h = the clamped SwiGLU of the slices' sums (slice 0 first)
__global__ __launch_bounds__(256) void exl3_swiglu_kernel(maya_exl3_args a, int KS) {
    if (a.skip && *a.skip) return;
    const int e = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x, n = a.layout.n_ff;
    if (c >= n || a.plan_ptr[e] == 0ull) return;
    const float* pg = a.part + ((size_t) e * 2 + 0) * KS * n + c;
    const float* pu = a.part + ((size_t) e * 2 + 1) * KS * n + c;
    float g = pg[0], u = pu[0];
    for (int s = 1; s < KS; ++s) {
        g = __fadd_rn(g, pg[(size_t) s * n]);
        u = __fadd_rn(u, pu[(size_t) s * n]);
    }
    a.h[(size_t) e * n + c] = ex_swiglu(g, u, a.limit);
}

// grid (n_embd / 128, groups): part[e][columns] = the down product of h[e]
template <int CB, int NT, int K2>
__global__ __launch_bounds__(kExThreads) void exl3_down_kernel(maya_exl3_args a) {
    extern __shared__ uint32_t lds[];
    ExGroup gr;
    if (!ex_group_of(a, blockIdx.y, gr)) return;
    const int k = a.layout.n_ff, n = a.layout.n_embd;
    uint32_t* wt = lds + (threadIdx.x >> 6) * 64;
    __half* xr = (__half*) (lds + 8 * 64);             // [NT][k]
    float* tmp = (float*) (xr + (size_t) NT * k);      // the raw outputs [NT][128]
    const uint8_t* blob = (const uint8_t*) gr.blob;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int tc = blockIdx.x * 8 + wave;
    auto chunk = [&](auto ntc, int c0) {
        constexpr int NTC = decltype(ntc)::value;
        int ents[NTC];
#pragma unroll
        for (int t = 0; t < NTC; ++t) ents[t] = ex_entry_of(a, gr, c0 + t);
        __syncthreads();
        for (int t = 0; t < NTC; ++t)
            rotate_in<(K2 > 0)>(a.h + (size_t) ents[t] * k, (const uint16_t*) (blob + a.layout.suh[2]), k, tmp, xr + (size_t) t * k);
        float acc[NTC];
#pragma unroll
        for (int t = 0; t < NTC; ++t) acc[t] = 0.0f;
        walk<CB, NTC, K2>((const uint32_t*) (blob + a.layout.trellis[2]), k, n >> 4, tc, a.layout.k2[2], lane, wt, xr, k, acc);
        __syncthreads();
        if (((lane >> 1) & 3) == 0) {
            const int col = wave * 16 + (lane >> 3) + 8 * (lane & 1);
#pragma unroll
            for (int t = 0; t < NTC; ++t) tmp[t * 128 + col] = acc[t];
        }
        __syncthreads();
        had128_out(tmp, NTC);
        const uint16_t* sv = (const uint16_t*) (blob + a.layout.svh[2]) + blockIdx.x * 128;
        for (int i = threadIdx.x; i < NTC * 128; i += kExThreads) {
            const int t = i >> 7, c = i & 127;
            a.part[(size_t) ents[t] * n + blockIdx.x * 128 + c] = __fmul_rn(tmp[t * 128 + c], f16_bits_to_f32(sv[c]));
        }
    };
    for (int c0 = 0; c0 < gr.ne;) {
        if (NT >= 2 && gr.ne - c0 >= 2) {
            chunk(std::integral_constant<int, 2>{}, c0);
            c0 += 2;
        } else {
            chunk(std::integral_constant<int, 1>{}, c0);
            c0 += 1;
        }
    }
}

__global__ __launch_bounds__(256) void exl3_combine_kernel(maya_exl3_args a) {
    if (a.skip && *a.skip) return;
    const int t = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x, n = a.layout.n_embd;
    if (c >= n) return;
    float sum = 0.0f;
    bool first = true;
    for (int i = 0; i < a.k; ++i) {
        const int e = t * a.k + i;
        if (a.plan_ptr[e] == 0ull) continue;
        const float p = __fmul_rn(a.part[(size_t) e * n + c], a.plan_w[e]);
        sum = first ? p : __fadd_rn(sum, p);
        first = false;
    }
    if (a.add && (!a.add_flag || *a.add_flag)) sum = __fadd_rn(sum, a.add[(size_t) t * n + c]);
    if (a.add2) sum = __fadd_rn(sum, a.add2[(size_t) t * n + c]);
    a.out[(size_t) t * n + c] = sum;
}

bool exl3_k2_ok(int k2, int cb) {
    return (k2 >= 2 && k2 <= 16 && (k2 & 1) == 0 && cb >= 0 && cb <= 2) || ((k2 == 3 || k2 == 5 || k2 == 7) && cb == 2);
}
int exl3_check(const maya_exl3_args* a) {
    if (!a) return fail(MAYA_E_ARG, "exl3: null args");
    const maya_exl3_layout& l = a->layout;
    for (int r = 0; r < 3; ++r)
        if (!exl3_k2_ok(l.k2[r], l.cb)) return fail(MAYA_E_UNSUPPORTED, "exl3: k2 %d with codebook %d", l.k2[r], l.cb);
    if (l.n_embd <= 0 || l.n_ff <= 0 || l.n_embd % 128 || l.n_ff % 128 || l.n_embd > 16384 || l.n_ff > 16384)
        return fail(MAYA_E_SHAPE, "exl3: n_embd %d / n_ff %d: multiples of 128 up to 16384 wanted", l.n_embd, l.n_ff);
    for (int r = 0; r < 3; ++r)
        if (l.trellis[r] % 4 || l.suh[r] % 2 || l.svh[r] % 2) return fail(MAYA_E_ARG, "exl3: misaligned part offsets");
    if (a->n_tokens < 1 || a->n_tokens > MAYA_MAX_TOKENS || a->k < 1 || a->k > MAYA_MAX_K)
        return fail(MAYA_E_SHAPE, "exl3: n_tokens %d / k %d", a->n_tokens, a->k);
    if (!a->plan_ptr || !a->plan_w) return fail(MAYA_E_ARG, "exl3: null plan");
    if (a->grp_ptr && (!a->grp_start || !a->grp_ent || !a->n_groups)) return fail(MAYA_E_ARG, "exl3: incomplete groups");
    return MAYA_OK;
}

template <int NT>
int launch_exl3_gate_up(const maya_exl3_args& a, const DeviceState& st, hipStream_t s) {
    const int k = a.layout.n_embd;
    const size_t scratch = (size_t) NT * 256 * 4;
    const size_t lds = 8 * 64 * 4 + (size_t) NT * 2 * k * 2 + scratch;
    if (lds > (size_t) st.lds_limit) return fail(MAYA_E_SHAPE, "exl3 gate/up needs %zu bytes of LDS, the device gives %d", lds, st.lds_limit);
    const dim3 grid((unsigned) (a.layout.n_ff / 128), (unsigned) (a.n_tokens * a.k));
#define MAYA_EX(CBV, K2V)                                                                                         \
    {                                                                                                             \
        auto kern = exl3_gate_up_kernel<CBV, NT, K2V>;                                                            \
        if (lds > 65536) MAYA_HIP(hipFuncSetAttribute((const void*) kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds)); \
        hipLaunchKernelGGL(kern, grid, dim3(kExThreads), lds, s, a);                                              \
    }
    // the compile-time walk: mul1, gate and up at one bit rate of at most 5 bits a weight
    const int k2f = a.layout.cb == 2 && a.layout.k2[0] == a.layout.k2[1] && a.layout.k2[0] <= 10 ? a.layout.k2[0] : 0;
    switch (k2f) {
        case 2: MAYA_EX(2, 2) break;
        case 3: MAYA_EX(2, 3) break;
        case 4: MAYA_EX(2, 4) break;
        case 5: MAYA_EX(2, 5) break;
        case 6: MAYA_EX(2, 6) break;
        case 7: MAYA_EX(2, 7) break;
        case 8: MAYA_EX(2, 8) break;
        case 10: MAYA_EX(2, 10) break;
        default:
            if (a.layout.cb == 2) MAYA_EX(2, 0) else if (a.layout.cb == 1) MAYA_EX(1, 0) else MAYA_EX(0, 0)
    }
#undef MAYA_EX
    MAYA_LAUNCHED("exl3_gate_up_kernel");
    return MAYA_OK;
}
// the split gate/up when it applies (mul1, one bit rate <= 5 bits for gate and up, `part` given and large enough for the
// partial outputs): 1 launched, 0 not applicable
template <int NT>
int try_exl3_gu_split(const maya_exl3_args& a, const DeviceState& st, hipStream_t s, int* rc) {
    const maya_exl3_layout& l = a.layout;
    if (l.cb != 2 || l.k2[0] != l.k2[1] || l.k2[0] > 10 || !a.part) return 0;
    const int KS = (l.n_embd % 256 == 0 && l.n_embd >= 4 * l.n_ff) ? 2 : (l.n_embd >= 2 * l.n_ff ? 1 : 0);
    if (KS == 0) return 0;
    const int kb = l.n_embd / KS;
    const size_t lds = (size_t) NT * kb * 2 + (size_t) NT * 128 * 4;
    if (lds > (size_t) st.lds_limit) return 0;
    const dim3 grid((unsigned) (l.n_ff / 128), (unsigned) (a.n_tokens * a.k), (unsigned) (2 * KS));
#define MAYA_EX(K2V)                                                                                              \
    {                                                                                                             \
        auto kern = exl3_gu_split_kernel<NT, K2V>;                                                                \
        if (lds > 65536) {                                                                                        \
            const hipError_t e_ = hipFuncSetAttribute((const void*) kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds); \
            if (e_ != hipSuccess) { *rc = hip_fail(e_, "hipFuncSetAttribute"); return 1; }                        \
        }                                                                                                         \
        hipLaunchKernelGGL(kern, grid, dim3(kExThreads), lds, s, a, KS);                                          \
    }
    switch (l.k2[0]) {
        case 2: MAYA_EX(2) break;
        case 3: MAYA_EX(3) break;
        case 4: MAYA_EX(4) break;
        case 5: MAYA_EX(5) break;
        case 6: MAYA_EX(6) break;
        case 7: MAYA_EX(7) break;
        case 8: MAYA_EX(8) break;
        case 10: MAYA_EX(10) break;
        default: return 0;
    }
#undef MAYA_EX
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { *rc = hip_fail(e, "exl3_gu_split_kernel"); return 1; }
    hipLaunchKernelGGL(exl3_swiglu_kernel, dim3((unsigned) ((l.n_ff + 255) / 256), (unsigned) (a.n_tokens * a.k)), dim3(256), 0, s, a, KS);
    e = hipGetLastError();
    *rc = e != hipSuccess ? hip_fail(e, "exl3_swiglu_kernel") : MAYA_OK;
    return 1;
}

template <int NT>
int launch_exl3_down(const maya_exl3_args& a, const DeviceState& st, hipStream_t s) {
    const int k = a.layout.n_ff;
    const size_t scratch = (size_t) NT * 128 * 4;
    const size_t lds = 8 * 64 * 4 + (size_t) NT * k * 2 + scratch;
    if (lds > (size_t) st.lds_limit) return fail(MAYA_E_SHAPE, "exl3 down needs %zu bytes of LDS, the device gives %d", lds, st.lds_limit);
    const dim3 grid((unsigned) (a.layout.n_embd / 128), (unsigned) (a.n_tokens * a.k));
#define MAYA_EX(CBV, K2V)                                                                                         \
    {                                                                                                             \
        auto kern = exl3_down_kernel<CBV, NT, K2V>;                                                               \
        if (lds > 65536) MAYA_HIP(hipFuncSetAttribute((const void*) kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds)); \
        hipLaunchKernelGGL(kern, grid, dim3(kExThreads), lds, s, a);                                              \
    }
    const int k2f = a.layout.cb == 2 && a.layout.k2[2] <= 10 ? a.layout.k2[2] : 0;
    switch (k2f) {
        case 2: MAYA_EX(2, 2) break;
        case 3: MAYA_EX(2, 3) break;
        case 4: MAYA_EX(2, 4) break;
        case 5: MAYA_EX(2, 5) break;
        case 6: MAYA_EX(2, 6) break;
        case 7: MAYA_EX(2, 7) break;
        case 8: MAYA_EX(2, 8) break;
        case 10: MAYA_EX(2, 10) break;
        default:
            if (a.layout.cb == 2) MAYA_EX(2, 0) else if (a.layout.cb == 1) MAYA_EX(1, 0) else MAYA_EX(0, 0)
    }
#undef MAYA_EX
    MAYA_LAUNCHED("exl3_down_kernel");
    return MAYA_OK;
}

}  // namespace maya

using namespace maya;

extern "C" {

int maya_exl3_supported(int k2, int cb) { return exl3_k2_ok(k2, cb) ? 1 : 0; }

size_t maya_exl3_layout_init(maya_exl3_layout* l, int n_embd, int n_ff, const int32_t* k2, int cb, int order) {
    if (!l || !k2 || n_embd <= 0 || n_ff <= 0 || n_embd % 128 || n_ff % 128 || (order != MAYA_EXL3_ORDER_SCALES_FIRST && order != MAYA_EXL3_ORDER_TRELLIS_FIRST))
        return 0;
    for (int r = 0; r < 3; ++r)
        if (!exl3_k2_ok(k2[r], cb)) return 0;
    *l = maya_exl3_layout{};
    l->cb = cb;
    l->n_embd = n_embd;
    l->n_ff = n_ff;
    // every piece starts on a multiple of `al` bytes: 16 for the compact order, 256 for the engine's assembled blobs
    const size_t al = order == MAYA_EXL3_ORDER_TRELLIS_FIRST ? 256 : 16;
    auto up = [al](size_t n) { return (n + al - 1) / al * al; };
    size_t off = 0;
    for (int r = 0; r < 3; ++r) {
        const int64_t k = r == 2 ? n_ff : n_embd, n = r == 2 ? n_embd : n_ff;
        const size_t tb = maya_exl3_trellis_bytes(k, n, k2[r]);
        l->k2[r] = k2[r];
        if (order == MAYA_EXL3_ORDER_TRELLIS_FIRST) {
            l->trellis[r] = off, off += up(tb);
            l->suh[r] = off, off += up(2 * (size_t) k);
            l->svh[r] = off, off += up(2 * (size_t) n);
        } else {
            l->suh[r] = off, off += up(2 * (size_t) k);
            l->svh[r] = off, off += up(2 * (size_t) n);
            l->trellis[r] = off, off += up(tb);
        }
    }
    return off;
}
size_t maya_exl3_trellis_bytes(int64_t k, int64_t n, int k2) { return (size_t) (k / 16) * (size_t) (n / 16) * 16u * (size_t) k2; }

// nine pieces an expert (the trellis, suh and svh of gate, up and down) copied to their places in the expert's blob:
// grid (blocks, 9, n_expert).  16 bytes a thread where source and destination allow it, else byte by byte.
__global__ __launch_bounds__(256) void exl3_pack_kernel(const uint64_t* __restrict__ pieces, maya_exl3_layout l, uint8_t* __restrict__ dst,
                                                        size_t dst_stride) {
    const int piece = blockIdx.y, r = piece / 3, what = piece % 3, e = blockIdx.z;
    const int64_t k = r == 2 ? l.n_ff : l.n_embd, n = r == 2 ? l.n_embd : l.n_ff;
    const size_t bytes = what == 0 ? (size_t) (k / 16) * (size_t) (n / 16) * 16u * (size_t) l.k2[r] : what == 1 ? 2 * (size_t) k : 2 * (size_t) n;
    const size_t off = what == 0 ? l.trellis[r] : what == 1 ? l.suh[r] : l.svh[r];
    const uint8_t* src = (const uint8_t*) pieces[(size_t) e * 9 + piece];
    uint8_t* d = dst + (size_t) e * dst_stride + off;
    if (src == nullptr) return;
    const size_t stride = (size_t) gridDim.x * 256;
    if ((((uintptr_t) src | (uintptr_t) d) & 15) == 0) {
        const size_t n16 = bytes >> 4;
        for (size_t i = (size_t) blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) ((uint4*) d)[i] = ((const uint4*) src)[i];
        for (size_t i = (n16 << 4) + (size_t) blockIdx.x * 256 + threadIdx.x; i < bytes; i += stride) d[i] = src[i];
    } else {
        for (size_t i = (size_t) blockIdx.x * 256 + threadIdx.x; i < bytes; i += stride) d[i] = src[i];
    }
}

int maya_exl3_pack_experts(const maya_exl3_layout* l, const uint64_t* pieces, int n_expert, void* dst, size_t dst_stride, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!l || !pieces || !dst) return fail(MAYA_E_ARG, "exl3_pack_experts: null pointer");
    if (n_expert <= 0 || n_expert > 65535) return fail(MAYA_E_SHAPE, "exl3_pack_experts: %d experts", n_expert);
    if (l->n_embd <= 0 || l->n_ff <= 0 || l->n_embd % 128 || l->n_ff % 128) return fail(MAYA_E_SHAPE, "exl3_pack_experts: %d x %d", l->n_embd, l->n_ff);
    size_t end = 0;
    for (int r = 0; r < 3; ++r) {
        if (!exl3_k2_ok(l->k2[r], l->cb)) return fail(MAYA_E_UNSUPPORTED, "exl3_pack_experts: k2 %d with codebook %d", l->k2[r], l->cb);
        const int64_t k = r == 2 ? l->n_ff : l->n_embd, n = r == 2 ? l->n_embd : l->n_ff;
        if ((l->trellis[r] & 3) || (l->suh[r] & 1) || (l->svh[r] & 1)) return fail(MAYA_E_ARG, "exl3_pack_experts: a trellis needs 4-byte, suh / svh 2-byte alignment");
        end = end > l->trellis[r] + maya_exl3_trellis_bytes(k, n, l->k2[r]) ? end : l->trellis[r] + maya_exl3_trellis_bytes(k, n, l->k2[r]);
        end = end > l->suh[r] + 2 * (size_t) k ? end : l->suh[r] + 2 * (size_t) k;
        end = end > l->svh[r] + 2 * (size_t) n ? end : l->svh[r] + 2 * (size_t) n;
    }
    if (dst_stride < end) return fail(MAYA_E_ARG, "exl3_pack_experts: blobs of %zu bytes do not fit a stride of %zu", end, dst_stride);
    hipLaunchKernelGGL(exl3_pack_kernel, dim3(64, 9, (unsigned) n_expert), dim3(256), 0, as_stream(stream), pieces, *l, (uint8_t*) dst, dst_stride);
    MAYA_LAUNCHED("exl3_pack_kernel");
    return MAYA_OK;
}

int maya_exl3_reconstruct_inner(const uint32_t* trellis, int64_t k, int64_t n, int k2, int cb, uint16_t* dst, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!exl3_k2_ok(k2, cb)) return fail(MAYA_E_UNSUPPORTED, "exl3: k2 %d with codebook %d", k2, cb);
    if (!trellis || !dst) return fail(MAYA_E_ARG, "exl3 reconstruct: null pointer");
    if (k <= 0 || n <= 0 || k % 16 || n % 16) return fail(MAYA_E_SHAPE, "exl3 reconstruct: k %lld n %lld", (long long) k, (long long) n);
    const dim3 grid((unsigned) ((k / 16) * (n / 16)));
    hipStream_t s = as_stream(stream);
    if (cb == 2) hipLaunchKernelGGL(exl3_inner_kernel<2>, grid, dim3(256), 0, s, trellis, k, n, k2, dst);
    else if (cb == 1) hipLaunchKernelGGL(exl3_inner_kernel<1>, grid, dim3(256), 0, s, trellis, k, n, k2, dst);
    else hipLaunchKernelGGL(exl3_inner_kernel<0>, grid, dim3(256), 0, s, trellis, k, n, k2, dst);
    MAYA_LAUNCHED("exl3_inner_kernel");
    return MAYA_OK;
}

int maya_exl3_gate_up(const maya_exl3_args* a, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (const int rc = exl3_check(a)) return rc;
    if (!a->x || !a->h) return fail(MAYA_E_ARG, "exl3 gate_up: null x or h");
    const int nt = a->grp_ptr && a->n_tokens >= 2 ? 2 : 1;
    int rc = 0;
    if (nt == 2 ? try_exl3_gu_split<2>(*a, *st, as_stream(stream), &rc) : try_exl3_gu_split<1>(*a, *st, as_stream(stream), &rc)) return rc;
    return nt == 2 ? launch_exl3_gate_up<2>(*a, *st, as_stream(stream)) : launch_exl3_gate_up<1>(*a, *st, as_stream(stream));
}

int maya_exl3_down(const maya_exl3_args* a, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (const int rc = exl3_check(a)) return rc;
    if (!a->h || !a->part || !a->out) return fail(MAYA_E_ARG, "exl3 down: null h, part or out");
    const int nt = a->grp_ptr && a->n_tokens >= 2 ? 2 : 1;
    const int rc = nt == 2 ? launch_exl3_down<2>(*a, *st, as_stream(stream)) : launch_exl3_down<1>(*a, *st, as_stream(stream));
    if (rc) return rc;
    const dim3 grid((unsigned) ((a->layout.n_embd + 255) / 256), (unsigned) a->n_tokens);
    hipLaunchKernelGGL(exl3_combine_kernel, grid, dim3(256), 0, as_stream(stream), *a);
    MAYA_LAUNCHED("exl3_combine_kernel");
    return MAYA_OK;
}

struct Exl3Ws {
    uint64_t *plan_ptr, *grp_ptr;
    int32_t *grp_start, *grp_ent, *n_groups;
    float *h, *part;
    size_t bytes;
};
static Exl3Ws exl3_carve(const maya_exl3_layout& l, int n_tokens, int k, uint8_t* base) {
    Exl3Ws w{};
    size_t off = 0;
    const int ne = n_tokens * k;
    auto take = [&](size_t n) {
        uint8_t* p = base ? base + off : nullptr;
        off += (n + 255) & ~(size_t) 255;
        return p;
    };
    w.plan_ptr = (uint64_t*) take(sizeof(uint64_t) * ne);
    w.grp_ptr = (uint64_t*) take(sizeof(uint64_t) * ne);
    w.grp_start = (int32_t*) take(sizeof(int32_t) * (ne + 1));
    w.grp_ent = (int32_t*) take(sizeof(int32_t) * ne);
    w.n_groups = (int32_t*) take(sizeof(int32_t));
    w.h = (float*) take(sizeof(float) * (size_t) ne * l.n_ff);
    w.part = (float*) take(sizeof(float) * (size_t) ne * l.n_embd);
    w.bytes = off;
    return w;
}
size_t maya_exl3_workspace_bytes(const maya_exl3_layout* l, int n_tokens, int k) {
    if (!l || n_tokens < 1 || n_tokens > MAYA_MAX_TOKENS || k < 1 || k > MAYA_MAX_K || l->n_embd <= 0 || l->n_ff <= 0) return 0;
    return exl3_carve(*l, n_tokens, k, nullptr).bytes;
}

int maya_exl3_layer_decode(const maya_exl3_layout* l, const uint64_t* expert_table, int n_expert, int k, const float* logits,
                           const float* x, int n_tokens, float limit, const float* add, int32_t* ids, float* weights,
                           float* out, void* workspace, size_t workspace_bytes, void* stream) {
    if (!l || !expert_table || !x || !ids || !weights || !out || !workspace) return fail(MAYA_E_ARG, "exl3 layer: null pointer");
    if (n_tokens < 1 || n_tokens > MAYA_MAX_TOKENS || k < 1 || k > MAYA_MAX_K) return fail(MAYA_E_SHAPE, "exl3 layer: n_tokens %d / k %d", n_tokens, k);
    if (((uintptr_t) workspace & 255) != 0) return fail(MAYA_E_ARG, "exl3 layer: workspace not 256-byte aligned");
    const Exl3Ws w = exl3_carve(*l, n_tokens, k, (uint8_t*) workspace);
    if (workspace_bytes < w.bytes) return fail(MAYA_E_ARG, "exl3 layer: workspace %zu < %zu bytes", workspace_bytes, w.bytes);
    int rc;
    bool grouped = false;
    if (logits && n_tokens > 1 && n_tokens <= 4 && maya_moe_route_window_ok(nullptr, n_tokens, n_expert, k)) {   // a window of up to four tokens (one pass of the routing workgroup): route, plan and group in one launch
        if ((rc = maya_moe_route_window(nullptr, logits, n_tokens, n_expert, k, expert_table, ids, weights, w.plan_ptr, w.grp_ptr, w.grp_start,
                                        w.grp_ent, w.n_groups, stream)))
            return rc;
        grouped = true;
    } else if (logits) {   // route and plan in one launch; null: ids / weights are given
        if ((rc = maya_moe_route_plan(nullptr, logits, n_tokens, n_expert, k, expert_table, ids, weights, w.plan_ptr, stream))) return rc;
    } else if ((rc = maya_moe_plan(ids, n_tokens * k, expert_table, n_expert, w.plan_ptr, stream))) return rc;
    maya_exl3_args a{};
    a.layout = *l;
    a.n_tokens = n_tokens;
    a.k = k;
    a.plan_ptr = w.plan_ptr;
    a.plan_w = weights;
    if (n_tokens > 1) {
        if (!grouped && (rc = maya_moe_group(w.plan_ptr, n_tokens * k, w.grp_ptr, w.grp_start, w.grp_ent, w.n_groups, stream))) return rc;
        a.grp_ptr = w.grp_ptr;
        a.grp_start = w.grp_start;
        a.grp_ent = w.grp_ent;
        a.n_groups = w.n_groups;
    }
    a.limit = limit;
    a.x = x;
    a.h = w.h;
    a.part = w.part;
    a.add = add;
    a.out = out;
    if ((rc = maya_exl3_gate_up(&a, stream))) return rc;
    return maya_exl3_down(&a, stream);
}

}  // extern "C"
