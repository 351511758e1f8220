// maya_dev.hpp - device-side building blocks shared by the kernels: scalar conversions, unaligned loads, wave64
// reductions and the per-format decoders of a quantized block into int8 codes and integer scales.
//
// One decoded "unit" of a row is the work of one lane for one step.  Every format reduces to
//     w_i = D * s_h * q_i  (- M_j for Q4_K)          q_i an int8 code, s_h an integer scale per 16 or 32 values
// so a unit's contribution to a row sum against an int8 activation (codes y, F32 scale dy per 32) is
//     D * dy * sum_h s_h * dot(q_h, y_h)   [ - Dmin * dy * sum_j m_j * sum(y_j) ]
// with every dot an exact integer (v_dot4_i32_i8).  This is the arithmetic of the reference's exact-decode kernels
// (src/ds4/ds4_iq.cu:178-184, 285-297, 347-361, 426-432; ds4_iq.cuh:7-13) and of its CPU contract
// (src/kernels/cpu/iq_avx2.cpp:225-250, 332-394): exact block integers, F32 scales, no integer division.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace maya {

constexpr int kQ8_0 = 8, kQ4_K = 12, kIQ2_XXS = 16, kIQ1_S = 19, kIQ2_S = 22, kIQ1_M = 29;
constexpr int kWave = 64;

// ------------------------------------------------------------------------------------------------ scalars

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    // exact for every bit pattern (subnormals, infinities): the hardware conversion
    return __half2float(__ushort_as_half((unsigned short) h));
}
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

typedef uint32_t __attribute__((aligned(2))) u32_a2;
typedef uint16_t __attribute__((aligned(1))) u16_a1;
// 4 bytes from a 2-byte aligned address (GGUF blocks are 2-byte aligned: their sizes are not multiples of 4)
__device__ __forceinline__ uint32_t ld32_a2(const uint8_t* p) { return *(const u32_a2*) p; }
__device__ __forceinline__ uint32_t ld16(const uint8_t* p) { return *(const uint16_t*) p; }

__device__ __forceinline__ int dot4(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }
// a . b alone: the three-operand encoding with a literal zero as the addend (the compiler's own choice for
// dot4(a, b, 0) is the two-operand accumulate form behind a v_mov of zero: one instruction more)
__device__ __forceinline__ int dot4_first(int a, int b) {
    int d;
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b));
    return d;
}

// sum over the lanes of an aligned group of `width` lanes (a power of two <= 64); every lane gets the sum
template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int o = WIDTH / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

// ------------------------------------------------------------------------------------------------ codebooks

// Expanded on the host at init (maya_init) into device memory; kernels stage what they need into LDS.
struct Codebooks {
    const uint64_t* iq2s;  // 1024 x 8 magnitudes
    const uint64_t* iq1s;  // 2048 x 8 values -1 / 0 / +1
    const uint64_t* iq2xxs;  // 256 x 8 magnitudes
};

// four sign bits -> 0x01 in the bytes of the set bits (bit i -> byte i); the 16 partial products land on distinct bits
__device__ __forceinline__ uint32_t spread4(uint32_t nib) { return (nib * 0x00204081u) & 0x01010101u; }
// negate the bytes of g that c marks with 0x01 (g's bytes in 1..127): (g ^ 0xff) + 1 per byte, no carry across bytes
__device__ __forceinline__ uint32_t neg_bytes(uint32_t g, uint32_t c) {
    const uint32_t m = (c << 8) - c;  // 0xff in the marked bytes
    return (g ^ m) + c;
}

// ------------------------------------------------------------------------------------------------ decoders
//
// Fmt<TYPE>: kBytes / kValues of a block; kUnit values a lane takes a step; decode(blk, u, cb) fills codes and scales.

// A lane's value of lane ^ 1 (CTRL 0xB1, quad_perm [1,0,3,2]), lane ^ 2 (0x4E, quad_perm [2,3,0,1]) or of lane 7 - (lane & 7)
// in its run of 8 (0x141, row_half_mirror): data-parallel-primitive moves, no LDS traffic.
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) { return __builtin_amdgcn_mov_dpp(v, CTRL, 0xf, 0xf, true); }

// The down kernels' grid is (row blocks, tokens).  A window's tokens that route the same expert read the same rows of it,
// so the workgroups of ONE row block for all the tokens should run at the same time on the same XCD (workgroups go to the
// XCDs in turn by their linear index, x fastest).  With the row blocks a multiple of 8: runs of 8 row blocks x all tokens -
// index -> row block (index / (8 T)) 8 + index % 8, token (index / 8) % T - keep a row block on XCD (row block % 8) for
// every token and its tokens' workgroups within 8 T of each other in launch order.  One token, or row blocks not a
// multiple of 8: the grid as it is.
__device__ __forceinline__ void down_block_of_grid(int& row_block, int& token) {
    row_block = (int) blockIdx.x, token = (int) blockIdx.y;
    if (gridDim.y > 1 && (gridDim.x & 7u) == 0) {
        const unsigned id = blockIdx.y * gridDim.x + blockIdx.x, nt = gridDim.y;
        row_block = (int) ((id / (8u * nt)) * 8u + (id & 7u));
        token = (int) ((id >> 3) % nt);
    }
}

// The value of lane (lane ^ MASK), without address arithmetic: a DPP operand for masks 1, 2 (quad permutes) and 8 (a
// rotation by 8 inside a row of 16 lanes), ds_swizzle for 4 and 16 (an LDS-crossbar exchange inside 32 lanes whose
// pattern is an immediate), the gfx950 half-wave swap for 32.  (__shfl_xor costs four vector instructions of index
// arithmetic per call before its ds_bpermute.)
template <int MASK>
__device__ __forceinline__ float xor_lane(float v) {
    const int i = __float_as_int(v);
    if constexpr (MASK == 1) return __int_as_float(__builtin_amdgcn_update_dpp(0, i, 0xB1, 0xf, 0xf, true));        // quad_perm [1,0,3,2]
    else if constexpr (MASK == 2) return __int_as_float(__builtin_amdgcn_update_dpp(0, i, 0x4E, 0xf, 0xf, true));   // quad_perm [2,3,0,1]
    else if constexpr (MASK == 8) return __int_as_float(__builtin_amdgcn_update_dpp(0, i, 0x128, 0xf, 0xf, true));  // row_ror:8
    else if constexpr (MASK == 4) return __int_as_float(__builtin_amdgcn_ds_swizzle(i, 0x101F));                    // swap 4
    else if constexpr (MASK == 16) return __int_as_float(__builtin_amdgcn_ds_swizzle(i, 0x401F));                   // swap 16
    else {
        static_assert(MASK == 32, "masks inside a wave");
        const auto r = __builtin_amdgcn_permlane32_swap(i, i, false, false);   // r[0] = (lower, lower), r[1] = (upper, upper)
        return __int_as_float((threadIdx.x & 32) ? r[0] : r[1]);
    }
}
// v + the value of lane ^ 32 (both halves get lower + upper, the order __shfl_xor's form adds them in)
__device__ __forceinline__ float add_other_half(float v) {
    const int i = __float_as_int(v);
    const auto r = __builtin_amdgcn_permlane32_swap(i, i, false, false);
    return __int_as_float(r[0]) + __int_as_float(r[1]);
}

// Q8_K rounding of a 256-value block held by 8 consecutive lanes, 32 values a lane: the arithmetic of the reference's
// quantize_q8_K_kernel (src/kernels/cuda/quantize_act.cu:161-207) and codes, bit for bit, 4 codes a word in the order
// of v.  The block's scale comes from the signed value at the FIRST largest magnitude.  Its magnitude is the largest
// magnitude; its sign depends on the order only when the largest positive and the largest negative value share that
// magnitude.  So the common case needs two max3 chains over the raw bits (as signed integers the largest is the
// largest positive value; as unsigned integers the largest is the negative value of the largest magnitude) and three
// lane exchanges; only a wave that holds such a tie scans with indices (index_of(i) = the index of v[i] inside the
// block, ascending in i).  A product never rounds beyond +-127 (|iscale * v| <= 127 (1 + 2^-23)), so the low byte of
// the magic-number sum is the code.
template <typename IndexOf>
__device__ __forceinline__ void q8k_round_lane32(const float (&v)[32], IndexOf index_of, int (&y)[8], float& d) {
    int pb = __float_as_int(v[0]);
    uint32_t nb = __float_as_uint(v[0]);
#pragma unroll
    for (int i = 1; i < 31; i += 2) {
        pb = max(max(pb, __float_as_int(v[i])), __float_as_int(v[i + 1]));
        nb = max(max(nb, __float_as_uint(v[i])), __float_as_uint(v[i + 1]));
    }
    pb = max(pb, __float_as_int(v[31]));
    nb = max(nb, __float_as_uint(v[31]));
    pb = max(pb, dpp_i<0xB1>(pb)), nb = max(nb, (uint32_t) dpp_i<0xB1>((int) nb));
    pb = max(pb, dpp_i<0x4E>(pb)), nb = max(nb, (uint32_t) dpp_i<0x4E>((int) nb));
    pb = max(pb, dpp_i<0x141>(pb)), nb = max(nb, (uint32_t) dpp_i<0x141>((int) nb));
    const int pos = max(pb, 0);                                   // bits of the largest positive value, 0: none
    const int neg = (nb >> 31) ? (int) (nb & 0x7fffffffu) : 0;    // bits of the largest magnitude among the negative ones
    float sv = pos > neg ? __int_as_float(pos) : (neg > pos ? -__int_as_float(neg) : 0.0f);
    if (__any(pos == neg && pos != 0)) {
        float am = 0.0f;
        int ix = 0;
        sv = 0.0f;
#pragma unroll
        for (int i = 0; i < 32; ++i) {   // ascending index inside the lane: a strict > keeps the first
            const float av = fabsf(v[i]);
            if (av > am) am = av, sv = v[i], ix = index_of(i);
        }
#pragma unroll
        for (int o = 1; o < 8; o <<= 1) {
            const float oa = __shfl_xor(am, o, kWave), os = __shfl_xor(sv, o, kWave);
            const int oi = __shfl_xor(ix, o, kWave);
            if (oa > am || (oa == am && oi < ix)) am = oa, sv = os, ix = oi;
        }
    }
    float iscale = 0.0f;
    d = 0.0f;
    if (sv != 0.0f) {
        iscale = __fdiv_rn(-127.0f, sv);
        d = __fdiv_rn(1.0f, iscale);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        uint32_t c[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) c[b] = __float_as_uint(__fadd_rn(__fmul_rn(iscale, v[4 * i + b]), 12582912.0f));
        const uint32_t lo = __builtin_amdgcn_perm(c[1], c[0], 0x0c0c0400u), hi = __builtin_amdgcn_perm(c[3], c[2], 0x0c0c0400u);
        y[i] = (int) __builtin_amdgcn_perm(hi, lo, 0x05040100u);
    }
}

// A table of NWORDS 32-bit words from global memory into LDS by a workgroup of NT threads, in 16-byte pieces: every
// piece a thread moves is REQUESTED before the first one is stored, so the table costs one trip to memory.  (Written as
// a loop "lds[i] = src[i]; i += NT" the compiler waits for each load before it issues the next: one trip a pass, five
// for an 8 KB table on 448 threads.)  The request and the store are separate calls so that a kernel can put its other
// first loads between them.  Source and LDS destination 16-byte aligned.
template <int NWORDS, int NT>
struct TablePieces {
    static_assert(NWORDS % 4 == 0, "whole 16-byte pieces");
    static constexpr int kPieces = NWORDS / 4, kRounds = (kPieces + NT - 1) / NT;
    int4 r[kRounds];
};
template <int NWORDS, int NT>
__device__ __forceinline__ void table_request(const void* src, TablePieces<NWORDS, NT>& t) {
    const int4* s4 = (const int4*) src;
#pragma unroll
    for (int i = 0; i < TablePieces<NWORDS, NT>::kRounds; ++i) {
        const int j = (int) threadIdx.x + i * NT;
        t.r[i] = (i + 1) * NT <= TablePieces<NWORDS, NT>::kPieces || j < TablePieces<NWORDS, NT>::kPieces ? s4[j] : int4{0, 0, 0, 0};
    }
}
template <int NWORDS, int NT, typename Map>
__device__ __forceinline__ void table_store(int* lds, const TablePieces<NWORDS, NT>& t, Map map) {
#pragma unroll
    for (int i = 0; i < TablePieces<NWORDS, NT>::kRounds; ++i) {
        const int j = (int) threadIdx.x + i * NT;
        if ((i + 1) * NT <= TablePieces<NWORDS, NT>::kPieces || j < TablePieces<NWORDS, NT>::kPieces) {
            const int4 v = t.r[i];
            ((int4*) lds)[j] = int4{map(v.x), map(v.y), map(v.z), map(v.w)};
        }
    }
}
template <int NWORDS, int NT>
__device__ __forceinline__ void table_store(int* lds, const TablePieces<NWORDS, NT>& t) {
    table_store(lds, t, [](int v) { return v; });
}

struct Unit32 {
    int q[8];    // 32 int8 codes in value order (the IQ1 types: codes + 9 - delta, see Fmt<kIQ1_S>)
    int s0, s1;  // integer scales of values 0..15 / 16..31
    int dm[4];   // the IQ1 types: delta - 9 of each group of 8 values
};

template <int TYPE> struct Fmt;

template <> struct Fmt<kIQ2_S> {
    static constexpr bool kBiased = false;
    static constexpr int kBytes = 82, kValues = 256, kUnit = 32, kLdsWords = 2048;  // codebook: 1024 x u64
    static constexpr bool kMin = false;
    __device__ static __forceinline__ float scale(const uint8_t* blk) { return f16_bits_to_f32(ld16(blk)) * 0.125f; }
    // third_party/ggml/ggml-common.h:396-402; decode: src/kernels/cuda/iq_kernels.cu:686-695
    __device__ static __forceinline__ void decode_fields(uint32_t i4, uint32_t sg4, uint32_t h, uint32_t sc,
                                                         const uint2* grid, Unit32& u) {
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            const uint32_t idx = ((i4 >> (8 * l)) & 255u) | ((h << (8 - 2 * l)) & 0x300u);
            const uint2 g = grid[idx];
            const uint32_t sb = (sg4 >> (8 * l)) & 255u;
            u.q[2 * l] = (int) neg_bytes(g.x, spread4(sb & 15u));
            u.q[2 * l + 1] = (int) neg_bytes(g.y, spread4(sb >> 4));
        }
        u.s0 = 2 * (int) (sc & 15u) + 1;
        u.s1 = 2 * (int) (sc >> 4) + 1;
    }
    __device__ static __forceinline__ void decode(const uint8_t* blk, int ib, const uint2* grid, Unit32& u) {
        decode_fields(ld32_a2(blk + 2 + 4 * ib), ld32_a2(blk + 34 + 4 * ib), blk[66 + ib], blk[74 + ib], grid, u);
    }
    // the stream packing: rows in quads (rows 4q .. 4q+3); a quad of rows of nu sub-blocks is
    //   [nu][4] (index word, sign word) | [nu][4] (high bits, scales) | [nu/8][4] d      (4 x the row's bytes)
    // quad = the quad's first byte, rq = the row inside it
    __device__ static __forceinline__ void decode_stream(const uint8_t* quad, int nu, int rq, int un, const uint2* grid,
                                                         Unit32& u, float& d) {
        const uint2 is = ((const uint2*) quad)[un * 4 + rq];
        const uint32_t hs = ((const uint16_t*) (quad + 32 * (size_t) nu))[un * 4 + rq];
        d = f16_bits_to_f32(((const uint16_t*) (quad + 40 * (size_t) nu))[(un >> 3) * 4 + rq]) * 0.125f;
        decode_fields(is.x, is.y, hs & 255u, hs >> 8, grid, u);
    }
};

// IQ2_XXS: 66 bytes a 256-value block - d, then 8 bytes a 32-value sub-block: four codebook indices (256 entries), then one
// word of four 7-bit sign indices and a 4-bit scale for all 32 values.  A sign index is seven sign bits; the eighth is
// their parity (ksigns_iq2xs, third_party/ggml/ggml-common.h:513: an even number of negative values a group of 8).
template <> struct Fmt<kIQ2_XXS> {
    static constexpr bool kBiased = false;
    static constexpr int kBytes = 66, kValues = 256, kUnit = 32, kLdsWords = 512;  // codebook: 256 x u64
    static constexpr bool kMin = false;
    __device__ static __forceinline__ float scale(const uint8_t* blk) { return f16_bits_to_f32(ld16(blk)) * 0.125f; }
    __device__ static __forceinline__ uint32_t signs8(uint32_t seven) { return seven | ((uint32_t) (__popc(seven) & 1) << 7); }
    // third_party/ggml/ggml-common.h:380-384; decode: src/kernels/cuda/iq_kernels.cu:661-672
    __device__ static __forceinline__ void decode(const uint8_t* blk, int ib, const uint2* grid, Unit32& u) {
        const uint32_t w0 = ld32_a2(blk + 2 + 8 * ib), aux = ld32_a2(blk + 6 + 8 * ib);
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            const uint2 g = grid[(w0 >> (8 * l)) & 255u];
            const uint32_t sb = signs8((aux >> (7 * l)) & 127u);
            u.q[2 * l] = (int) neg_bytes(g.x, spread4(sb & 15u));
            u.q[2 * l + 1] = (int) neg_bytes(g.y, spread4(sb >> 4));
        }
        u.s0 = u.s1 = 2 * (int) (aux >> 28) + 1;
    }
};

// IQ1_S / IQ1_M: the +-1/8 shift of each grid value rides in the integer dot: codes 8 g +- 1, scale d / 8
// (src/ds4/ds4_iq.cuh:11-13).  Grid bytes are -1 / 0 / +1: 8 g as bytes is (g << 3) per byte, done on the u32 with the
// sign bytes handled by two's complement: 8 * 0xff = 0xf8 (= -8) needs no carry when done per byte via a multiply of the
// separated positive / negative masks.
__device__ __forceinline__ uint32_t iq1_codes(uint32_t g, uint32_t delta_byte) {
    // g bytes in {0xff, 0x00, 0x01}.  pos = bytes equal to 1, neg = bytes equal to 0xff (bit 1 set only there)
    const uint32_t neg = (g >> 1) & 0x01010101u, pos = g & ~(g >> 1) & 0x01010101u;
    // 8 g + delta per byte, delta = +1 (0x01) or -1 (0xff): bytes stay within -9..9, assembled without cross-byte carries
    // as (pos*8) | (neg * 0xf8) then a per-byte add of delta through the carry-free form below
    const uint32_t v = (pos << 3) | ((neg << 8) - (neg << 3));  // 0x08 / 0xf8 / 0x00
    // per-byte add of delta_byte (0x01010101 or 0xffffffff): add the low 7 bits, fix the top bit by xor
    const uint32_t lo = (v & 0x7f7f7f7fu) + (delta_byte & 0x7f7f7f7fu);
    return lo ^ ((v ^ delta_byte) & 0x80808080u);
}

// The IQ1 types: a value is d (2 s + 1) (g + delta / 8) with g in {-1, 0, +1} from the grid and delta = +-1 a group (IQ1_M)
// or a sub-block (IQ1_S), i.e. the int8 code 8 g + delta.  In LDS the grid is kept as t = 8 g + 9 (bytes 1 / 9 / 17:
// stage_codebook), so a looked-up word IS the operand of the dot products and no per-byte arithmetic is needed:
//   sum (8 g + delta) y = sum t y + (delta - 9) sum y,
// the second term from the activations' sums (the Q8_K bsums, and two dot products a group where delta changes inside
// 16 values).
template <> struct Fmt<kIQ1_S> {
    static constexpr int kBytes = 50, kValues = 256, kUnit = 32, kLdsWords = 4096;  // codebook: 2048 x u64
    static constexpr bool kMin = false, kBiased = true;
    __device__ static __forceinline__ float scale(const uint8_t* blk) { return f16_bits_to_f32(ld16(blk)) * 0.125f; }
    // third_party/ggml/ggml-common.h:425-430; decode: src/kernels/cuda/iq_kernels.cu:825-837
    __device__ static __forceinline__ void decode(const uint8_t* blk, int ib, const uint2* grid, Unit32& u) {
        const uint32_t q4 = ld32_a2(blk + 2 + 4 * ib), qh = ld16(blk + 34 + 2 * ib);
        const int dm = (qh & 0x8000u) ? -10 : -8;
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            const uint2 g = grid[((q4 >> (8 * l)) & 255u) | (((qh >> (3 * l)) & 7u) << 8)];
            u.q[2 * l] = (int) g.x;
            u.q[2 * l + 1] = (int) g.y;
            u.dm[l] = dm;
        }
        u.s0 = u.s1 = 2 * (int) ((qh >> 12) & 7u) + 1;
    }
    // the same from a quad of the stream order: the sub-blocks' index words, then their qh words, then the block scales
    __device__ static __forceinline__ void decode_stream(const uint8_t* quad, int nu, int rq, int un, const uint2* grid,
                                                         Unit32& u, float& d) {
        const uint32_t q4 = ((const uint32_t*) quad)[un * 4 + rq];
        const uint32_t qh = ((const uint16_t*) (quad + 16 * (size_t) nu))[un * 4 + rq];
        d = f16_bits_to_f32(((const uint16_t*) (quad + 24 * (size_t) nu))[(un >> 3) * 4 + rq]) * 0.125f;
        const int dm = (qh & 0x8000u) ? -10 : -8;
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            const uint2 g = grid[((q4 >> (8 * l)) & 255u) | (((qh >> (3 * l)) & 7u) << 8)];
            u.q[2 * l] = (int) g.x;
            u.q[2 * l + 1] = (int) g.y;
            u.dm[l] = dm;
        }
        u.s0 = u.s1 = 2 * (int) ((qh >> 12) & 7u) + 1;
    }
};

template <> struct Fmt<kIQ1_M> {
    static constexpr int kBytes = 56, kValues = 256, kUnit = 32, kLdsWords = 4096;
    static constexpr bool kMin = false, kBiased = true;
    // the FP16 super-scale sits in the top nibbles of the four u16 scale words (src/kernels/cpu/iq_avx2.cpp:471-475)
    __device__ static __forceinline__ float scale(const uint8_t* blk) {
        const uint32_t s0 = ld16(blk + 48), s1 = ld16(blk + 50), s2 = ld16(blk + 52), s3 = ld16(blk + 54);
        return f16_bits_to_f32((s0 >> 12) | ((s1 >> 8) & 0x00f0u) | ((s2 >> 4) & 0x0f00u) | (s3 & 0xf000u)) * 0.125f;
    }
    // third_party/ggml/ggml-common.h:433-438; decode: src/kernels/cuda/iq_kernels.cu:839-855
    __device__ static __forceinline__ void decode(const uint8_t* blk, int ib, const uint2* grid, Unit32& u) {
        const uint32_t q4 = ld32_a2(blk + 4 * ib), qh = ld16(blk + 32 + 2 * ib);
        const uint32_t sc = ld16(blk + 48 + 2 * (ib >> 1)) >> (6 * (ib & 1));
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            const uint32_t nib = (qh >> (4 * l)) & 15u;
            const uint2 g = grid[((q4 >> (8 * l)) & 255u) | ((nib & 7u) << 8)];
            u.q[2 * l] = (int) g.x;
            u.q[2 * l + 1] = (int) g.y;
            u.dm[l] = (nib & 8u) ? -10 : -8;
        }
        u.s0 = 2 * (int) (sc & 7u) + 1;
        u.s1 = 2 * (int) ((sc >> 3) & 7u) + 1;
    }
    // the same from a quad of the stream order: index words, qh words, then 8 bytes a (block, row): the block scale, then
    // the sixteen 3-bit scales in order
    __device__ static __forceinline__ void decode_stream(const uint8_t* quad, int nu, int rq, int un, const uint2* grid,
                                                         Unit32& u, float& d) {
        const uint32_t q4 = ((const uint32_t*) quad)[un * 4 + rq];
        const uint32_t qh = ((const uint16_t*) (quad + 16 * (size_t) nu))[un * 4 + rq];
        const uint2 rec = ((const uint2*) (quad + 24 * (size_t) nu))[(un >> 3) * 4 + rq];
        d = f16_bits_to_f32(rec.x & 0xffffu) * 0.125f;
        const uint32_t sc = (uint32_t) ((((uint64_t) rec.y << 32) | (uint64_t) rec.x) >> (16 + 6 * (un & 7)));
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            const uint32_t nib = (qh >> (4 * l)) & 15u;
            const uint2 g = grid[((q4 >> (8 * l)) & 255u) | ((nib & 7u) << 8)];
            u.q[2 * l] = (int) g.x;
            u.q[2 * l + 1] = (int) g.y;
            u.dm[l] = (nib & 8u) ? -10 : -8;
        }
        u.s0 = 2 * (int) (sc & 7u) + 1;
        u.s1 = 2 * (int) ((sc >> 3) & 7u) + 1;
    }
};

template <> struct Fmt<kQ8_0> {
    static constexpr bool kBiased = false;
    static constexpr int kBytes = 34, kValues = 32, kUnit = 32, kLdsWords = 0;
    static constexpr bool kMin = false;
    __device__ static __forceinline__ float scale(const uint8_t* blk) { return f16_bits_to_f32(ld16(blk)); }
    // third_party/ggml/ggml-common.h:252-256; a unit is one block
    __device__ static __forceinline__ void decode(const uint8_t* blk, int, const uint2*, Unit32& u) {
#pragma unroll
        for (int i = 0; i < 8; ++i) u.q[i] = (int) ld32_a2(blk + 2 + 4 * i);
        u.s0 = u.s1 = 1;
    }
};

// Q4_K: a unit is a pair of sub-blocks (64 values) sharing 32 bytes of nibbles
// (third_party/ggml/ggml-common.h:327-338; include/strata/artifact/dequant.hpp:152-190)
struct UnitQ4K {
    int lo[8], hi[8];  // sub-block 2p (low nibbles), 2p+1 (high nibbles)
    int sc0, sc1, m0, m1;
};
__device__ __forceinline__ void q4k_scale_min(const uint8_t* s, int j, int& sc, int& m) {
    if (j < 4) {
        sc = s[j] & 63;
        m = s[j + 4] & 63;
    } else {
        sc = (s[j + 4] & 0x0f) | ((s[j - 4] >> 6) << 4);
        m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
}
template <> struct Fmt<kQ4_K> {
    static constexpr bool kBiased = false;
    static constexpr int kBytes = 144, kValues = 256, kUnit = 64, kLdsWords = 0;
    static constexpr bool kMin = true;
    __device__ static __forceinline__ float scale(const uint8_t* blk) { return f16_bits_to_f32(ld16(blk)); }
    __device__ static __forceinline__ float scale_min(const uint8_t* blk) { return f16_bits_to_f32(ld16(blk + 2)); }
    __device__ static __forceinline__ void decode(const uint8_t* blk, int p, UnitQ4K& u) {
        const uint8_t* q = blk + 16 + 32 * p;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t w = ld32_a2(q + 4 * i);
            u.lo[i] = (int) (w & 0x0f0f0f0fu);
            u.hi[i] = (int) ((w >> 4) & 0x0f0f0f0fu);
        }
        q4k_scale_min(blk + 4, 2 * p, u.sc0, u.m0);
        q4k_scale_min(blk + 4, 2 * p + 1, u.sc1, u.m1);
    }
};

}  // namespace maya
