// maya_fast.cuh - the single-token streaming kernels for IQ2_S experts (the decode layer's hot loops).
//
// Both kernels are HBM-bound streams over raw GGUF rows.  A lane owns the same 32-value sub-block positions of every
// row it touches, so its slice of the int8 activation lives in registers for the whole kernel; a row's quantized bytes
// are fetched with all of the lane's loads in flight at once and the next row is fetched while the current one is
// decoded.  The IQ2_S codebook (8 KiB) and a 256-entry sign-mask table (2 KiB) sit in LDS.
//
// Sign handling without per-byte negation: with m the mask of the negative values (0xff bytes) and g the magnitudes,
//     sum s_i g_i y_i = dot4(g ^ m, y) - dot4(m, y)
// because g ^ 0xff = -g - 1 as int8 and m = -1 there; every term is an exact integer.
#pragma once

#include "maya_dev.cuh"

namespace maya {

typedef const __attribute__((address_space(1))) uint8_t* gptr8;
typedef const __attribute__((address_space(1))) uint16_t* gptr16;
typedef const __attribute__((address_space(1))) uint32_t __attribute__((aligned(2))) * gptr32_a2;
typedef uint32_t __attribute__((ext_vector_type(2))) u32x2;
typedef const __attribute__((address_space(1))) u32x2* gptr64;

__device__ __forceinline__ uint32_t gld32_a2(gptr8 p) { return *(gptr32_a2) p; }
__device__ __forceinline__ uint32_t gld16(gptr8 p) { return *(gptr16) p; }
__device__ __forceinline__ uint32_t gld8(gptr8 p) { return *p; }

struct RawIQ2S {
    uint32_t i4, sg4, hs, d;  // index word, sign word, high bits | scales << 8, FP16 block scale
};

// the lane's KU sub-blocks of one IQ2_S row: sub-block u = sub + LPR j.
// GGUF rows: u sits in block u / 8 at position u % 8 (2-byte aligned fields).  Stream rows: field arrays, aligned.
template <int KU, int LPR, bool STREAM>
__device__ __forceinline__ void load_iq2s(gptr8 row, int sub, RawIQ2S (&raw)[KU]) {
    if constexpr (STREAM) {
        constexpr int NU = KU * LPR;
        gptr64 is = (gptr64) row + sub;
        gptr16 hs = (gptr16) (row + 8 * NU) + sub;
        gptr16 d = (gptr16) (row + 10 * NU) + (sub >> 3);
#pragma unroll
        for (int j = 0; j < KU; ++j) {
            const u32x2 v = is[j * LPR];
            raw[j].i4 = v.x;
            raw[j].sg4 = v.y;
            raw[j].hs = hs[j * LPR];
            raw[j].d = d[j * (LPR / 8)];
        }
    } else {
        gptr8 p = row + (sub >> 3) * 82 + (sub & 7);
        const int ib3 = 3 * (sub & 7);  // the 4-byte fields advance 4 bytes a sub-block: 1 from p, 3 here
#pragma unroll
        for (int j = 0; j < KU; ++j) {
            gptr8 b = p + j * (LPR / 8) * 82;
            raw[j].i4 = gld32_a2(b + 2 + ib3);
            raw[j].sg4 = gld32_a2(b + 34 + ib3);
            raw[j].hs = gld8(b + 66) | (gld8(b + 74) << 8);
            raw[j].d = gld16(b - (sub & 7));
        }
    }
}

// one sub-block against the lane's activation slice: the integer sum with its two 16-value scales applied
__device__ __forceinline__ int dot_iq2s(const RawIQ2S& r, const uint2* __restrict__ grid, const uint2* __restrict__ stab,
                                        const int (&y)[8]) {
    int p0 = 0, n0 = 0, p1 = 0, n1 = 0;
#pragma unroll
    for (int l = 0; l < 4; ++l) {
        // (hs << (8 - 2 l)) & 0x300: the scale bits of hs land above bit 9 and fall to the mask
        const uint32_t idx = ((r.i4 >> (8 * l)) & 255u) | ((r.hs << (8 - 2 * l)) & 0x300u);
        const uint2 g = grid[idx];
        const uint2 m = stab[(r.sg4 >> (8 * l)) & 255u];
        if (l < 2) {
            p0 = dot4((int) (g.x ^ m.x), y[2 * l], p0);
            n0 = dot4((int) m.x, y[2 * l], n0);
            p0 = dot4((int) (g.y ^ m.y), y[2 * l + 1], p0);
            n0 = dot4((int) m.y, y[2 * l + 1], n0);
        } else {
            p1 = dot4((int) (g.x ^ m.x), y[2 * l], p1);
            n1 = dot4((int) m.x, y[2 * l], n1);
            p1 = dot4((int) (g.y ^ m.y), y[2 * l + 1], p1);
            n1 = dot4((int) m.y, y[2 * l + 1], n1);
        }
    }
    const int s0 = 2 * (int) ((r.hs >> 8) & 15u) + 1, s1 = 2 * (int) (r.hs >> 12) + 1;
    return __mul24(s0, p0 - n0) + __mul24(s1, p1 - n1);
}

template <int KU>
__device__ __forceinline__ float row_iq2s(const RawIQ2S (&raw)[KU], const uint2* grid, const uint2* stab,
                                          const int (&y)[KU][8], const float (&dy)[KU]) {
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < KU; ++j) {
        const int isum = dot_iq2s(raw[j], grid, stab, y[j]);
        acc = fmaf(__fmul_rn(f16_bits_to_f32(raw[j].d) * 0.125f, dy[j]), (float) isum, acc);
    }
    return acc;
}

// LDS: [0, 2048) words the codebook, [2048, 2560) the sign masks
__device__ __forceinline__ void stage_iq2s_tables(int* lds, const Codebooks& cb, int nthreads) {
    const int* src = (const int*) cb.iq2s;
    for (int i = threadIdx.x; i < 2048; i += nthreads) lds[i] = src[i];
    for (int i = threadIdx.x; i < 256; i += nthreads) {
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            if (i & (1 << b)) lo |= 0xffu << (8 * b);
            if (i & (16 << b)) hi |= 0xffu << (8 * b);
        }
        lds[2048 + 2 * i] = (int) lo;
        lds[2048 + 2 * i + 1] = (int) hi;
    }
}

constexpr int kFastLdsWords = 2048 + 512;

// the lane's slice of an activation row: units sub + LPR j
template <int KU, int LPR>
__device__ __forceinline__ void load_act_slice(const maya_act& x, int row, int k, int sub, int (&y)[KU][8], float (&dy)[KU]) {
    const int4* q = (const int4*) (x.q + (size_t) row * k);
    const float* d = x.d + (size_t) row * (k >> 5);
#pragma unroll
    for (int j = 0; j < KU; ++j) {
        const int u = sub + LPR * j;
        const int4 a = q[2 * u], b = q[2 * u + 1];
        y[j][0] = a.x, y[j][1] = a.y, y[j][2] = a.z, y[j][3] = a.w;
        y[j][4] = b.x, y[j][5] = b.y, y[j][6] = b.z, y[j][7] = b.w;
        dy[j] = d[u];
    }
}

// ---- gate/up, one token: grid (n_ff / ROWS, k); a wave takes row pairs (gate on lanes 0..31, up on 32..63).
// n_embd = 1024 KU.  YREG: the lane's activation slice in registers (else read from LDS); PF: the next pair's bytes
// are fetched while this one is decoded; MINB: waves a SIMD must hold (bounds the registers).
template <int KU, int ROWS, bool YREG, bool PF, int MINB, bool STREAM>
__global__ __launch_bounds__(512, MINB) void gate_up_iq2s_1tok_kernel(maya_moe_args a, Codebooks cb) {
    __shared__ int lds[kFastLdsWords + (YREG ? 0 : KU * 32 * 9)];
    if (a.skip && *a.skip) return;
    const int e = blockIdx.y;  // entry = plan slot (one token)
    const uint64_t blob = a.plan_ptr[e];
    if (blob == 0ull) return;
    stage_iq2s_tables(lds, cb, 512);
    const uint2* grid = (const uint2*) lds;
    const uint2* stab = (const uint2*) (lds + 2048);
    const int k = a.layout.n_embd, n_ff = a.layout.n_ff;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, sub = lane & 31;
    int y[YREG ? KU : 1][8];
    float dy[YREG ? KU : 1];
    int* ylds = lds + kFastLdsWords;             // [KU*32 units][8 words], then [KU*32] scales
    if constexpr (YREG) {
        load_act_slice<KU, 32>(a.x, 0, k, sub, y, dy);
    } else {
        const int* q = (const int*) a.x.q;
        for (int i = threadIdx.x; i < KU * 256; i += 512) ylds[i] = q[i];
        for (int i = threadIdx.x; i < KU * 32; i += 512) ylds[KU * 256 + i] = __float_as_int(a.x.d[i]);
    }
    const size_t rb = (size_t) (k >> 8) * 82;
    gptr8 base = (gptr8) (blob + (lane < 32 ? a.layout.gate_off : a.layout.up_off));
    const int r0 = blockIdx.x * ROWS + wave, r1 = min(n_ff, (int) (blockIdx.x + 1) * ROWS);
    __syncthreads();
    auto row_sum = [&](const RawIQ2S (&raw)[KU]) {
        if constexpr (YREG) {
            return row_iq2s<KU>(raw, grid, stab, y, dy);
        } else {
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < KU; ++j) {
                const int u = sub + 32 * j;
                const int4 ya = ((const int4*) ylds)[2 * u], yb = ((const int4*) ylds)[2 * u + 1];
                const int yy[8] = {ya.x, ya.y, ya.z, ya.w, yb.x, yb.y, yb.z, yb.w};
                const int isum = dot_iq2s(raw[j], grid, stab, yy);
                acc = fmaf(__fmul_rn(f16_bits_to_f32(raw[j].d) * 0.125f, __int_as_float(ylds[KU * 256 + u])), (float) isum, acc);
            }
            return acc;
        }
    };
    if constexpr (PF) {
        RawIQ2S cur[KU], nxt[KU];
        if (r0 < r1) load_iq2s<KU, 32, STREAM>(base + (size_t) r0 * rb, sub, cur);
        for (int r = r0; r < r1; r += 8) {
            const bool more = r + 8 < r1;
            if (more) load_iq2s<KU, 32, STREAM>(base + (size_t) (r + 8) * rb, sub, nxt);
            float s = row_sum(cur);
            s = group_sum<32>(s);
            const float up = __shfl(s, 32, kWave);
            if (lane == 0) a.h[(size_t) e * n_ff + r] = swiglu(s, up, a.limit);
            if (more) {
#pragma unroll
                for (int j = 0; j < KU; ++j) cur[j] = nxt[j];
            }
        }
    } else {
        for (int r = r0; r < r1; r += 8) {
            RawIQ2S cur[KU];
            load_iq2s<KU, 32, STREAM>(base + (size_t) r * rb, sub, cur);
            float s = row_sum(cur);
            s = group_sum<32>(s);
            const float up = __shfl(s, 32, kWave);
            if (lane == 0) a.h[(size_t) e * n_ff + r] = swiglu(s, up, a.limit);
        }
    }
}

// ---- down + combine, one token: grid (n_embd / ROWS); wave w = plan slot w (k <= 8 slots), two rows a pass (32 lanes a
// row); the slots' partial rows meet in LDS and are summed in slot order.  n_ff = 1024 KU.
template <int KU, int ROWS, bool STREAM>
__global__ __launch_bounds__(512) void down_iq2s_1tok_kernel(maya_moe_args a, Codebooks cb) {
    __shared__ int lds[kFastLdsWords];
    __shared__ float part[8][ROWS];
    if (a.skip && *a.skip) return;
    stage_iq2s_tables(lds, cb, 512);
    const uint2* grid = (const uint2*) lds;
    const uint2* stab = (const uint2*) (lds + 2048);
    const int k = a.layout.n_ff, n_embd = a.layout.n_embd;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, sub = lane & 31, rsub = lane >> 5;
    const int r0 = blockIdx.x * ROWS;
    const uint64_t blob = wave < a.k ? a.plan_ptr[wave] : 0ull;
    __syncthreads();
    if (blob != 0ull) {
        int y[KU][8];
        float dy[KU];
        load_act_slice<KU, 32>(a.hq, wave, k, sub, y, dy);
        const size_t rb = (size_t) (k >> 8) * 82;
        gptr8 base = (gptr8) (blob + a.layout.down_off) + (size_t) (r0 + rsub) * rb;
        RawIQ2S cur[KU], nxt[KU];
        load_iq2s<KU, 32, STREAM>(base, sub, cur);
#pragma unroll 1
        for (int i = 0; i < ROWS; i += 2) {
            const bool more = i + 2 < ROWS;
            if (more) load_iq2s<KU, 32, STREAM>(base + (size_t) (i + 2) * rb, sub, nxt);
            float s = row_iq2s<KU>(cur, grid, stab, y, dy);
            s = group_sum<32>(s);
            if (sub == 0) part[wave][i + rsub] = s;
            if (more) {
#pragma unroll
                for (int j = 0; j < KU; ++j) cur[j] = nxt[j];
            }
        }
    }
    __syncthreads();
    if (threadIdx.x < ROWS) {
        const int c = threadIdx.x;
        float sum = 0.0f;
        bool first = true;
        for (int i = 0; i < a.k; ++i) {
            if (a.plan_ptr[i] == 0ull) continue;
            const float p = __fmul_rn(part[i][c], a.plan_w[i]);
            sum = first ? p : __fadd_rn(sum, p);
            first = false;
        }
        if (a.add && (!a.add_flag || *a.add_flag)) sum = __fadd_rn(sum, a.add[r0 + c]);
        a.out[r0 + c] = sum;
        if (a.part)
            for (int i = 0; i < a.k; ++i)
                if (a.plan_ptr[i] != 0ull) a.part[(size_t) i * n_embd + r0 + c] = part[i][c];
    }
}

}  // namespace maya
