// maya_fast.hpp - the single-token streaming kernels for IQ2_S experts (the decode layer's hot loops).
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

#include "maya_dev.hpp"

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
// GGUF rows: u sits in block u / 8 at position u % 8 (2-byte aligned fields).
template <int KU, int LPR, bool STREAM>
__device__ __forceinline__ void load_iq2s(gptr8 row, int sub, RawIQ2S (&raw)[KU]) {
    static_assert(!STREAM, "the stream packing is read by the position-mapped kernels");
    {
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
template <int NT>
__device__ __forceinline__ void stage_iq2s_tables(int* lds, const Codebooks& cb) {
    TablePieces<2048, NT> t;
    table_request(cb.iq2s, t);
    for (int i = threadIdx.x; i < 256; i += NT) {
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            if (i & (1 << b)) lo |= 0xffu << (8 * b);
            if (i & (16 << b)) hi |= 0xffu << (8 * b);
        }
        lds[2048 + 2 * i] = (int) lo;
        lds[2048 + 2 * i + 1] = (int) hi;
    }
    table_store(lds, t);
}

constexpr int kFastLdsWords = 2048 + 512;

// The position-mapped kernels' form of the second table: per sign byte the two v_perm_b32 selectors that pick, for the
// eight values it covers, each activation code from y (bit clear) or from the negated copy -y (bit set): selector byte i
// of a word = i + 4 * bit i.  LDS: [0, 2048) words the codebook, [2048, 2560) the selectors.
template <int NT>
__device__ __forceinline__ void store_iq2s_selectors(int* lds) {
    for (int j = threadIdx.x; j < 256; j += NT) {
        const int i = j;
        uint32_t lo = 0x03020100u, hi = 0x03020100u;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            if (i & (1 << b)) lo |= 4u << (8 * b);
            if (i & (16 << b)) hi |= 4u << (8 * b);
        }
        lds[2048 + 2 * j] = (int) lo;
        lds[2048 + 2 * j + 1] = (int) hi;
    }
}
template <int NT>
__device__ __forceinline__ void stage_iq2s_tables_sel(int* lds, const Codebooks& cb) {
    TablePieces<2048, NT> t;
    table_request(cb.iq2s, t);
    store_iq2s_selectors<NT>(lds);
    table_store(lds, t);
}

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
    __shared__ __align__(16) int lds[kFastLdsWords + (YREG ? 0 : KU * 32 * 9)];
    if (a.skip && *a.skip) return;
    const int e = blockIdx.y;  // entry = plan slot (one token)
    const uint64_t blob = a.plan_ptr[e];
    if (blob == 0ull) return;
    stage_iq2s_tables<512>(lds, cb);
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
    __shared__ __align__(16) int lds[kFastLdsWords];
    __shared__ float part[8][ROWS];
    if (a.skip && *a.skip) return;
    stage_iq2s_tables<512>(lds, cb);
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
        if (a.add2) sum = __fadd_rn(sum, a.add2[r0 + c]);
        a.out[r0 + c] = sum;
        if (a.part)
            for (int i = 0; i < a.k; ++i)
                if (a.plan_ptr[i] != 0ull) a.part[(size_t) i * n_embd + r0 + c] = part[i][c];
    }
}

// ================================================================================================================
// Position-mapped kernels (stream packing): a lane owns ONE sub-block position of the row (its 32 activation codes
// stay in 8 registers), walks down the rows with a ring of prefetched rows, and every 8 rows a butterfly over the
// lanes turns 8 per-lane values into per-row sums.  Loads of a wave are contiguous 512-byte / 128-byte runs.

// acc[i] = this lane's value for row i of the batch.  On return every lane holds, in acc[0], the sum over its
// 32-lane half of the values of row (lane >> 2) & 7.
__device__ __forceinline__ float reduce8_half(float (&acc)[8], int lane) {
    const bool b4 = lane & 16, b3 = lane & 8, b2 = lane & 4;
    float v4[4], v2[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float send = b4 ? acc[i] : acc[i + 4], keep = b4 ? acc[i + 4] : acc[i];
        v4[i] = keep + xor_lane<16>(send);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const float send = b3 ? v4[i] : v4[i + 2], keep = b3 ? v4[i + 2] : v4[i];
        v2[i] = keep + xor_lane<8>(send);
    }
    const float send = b2 ? v2[0] : v2[1], keep = b2 ? v2[1] : v2[0];
    float v = keep + xor_lane<4>(send);
    v += xor_lane<2>(v);
    v += xor_lane<1>(v);
    return v;
}

typedef uint32_t __attribute__((ext_vector_type(4))) u32x4;

// A lane's share of one quad of rows (4 rows x its sub-block): 12 registers
struct QuadIQ2S {
    u32x4 is01, is23;  // (index word, sign word) of rows 0,1 and 2,3
    u32x2 hs, d;       // four (high bits | scales << 8) halfwords, four FP16 block scales
};
struct QuadOffs {  // byte offsets of the lane's fields inside a quad; quads advance through the scalar offset
    uint32_t is, hs, d;
};
template <int NU>
__device__ __forceinline__ QuadOffs quad_offs(uint32_t mat_off, int u) {
    return QuadOffs{mat_off + 32u * u, mat_off + 32u * NU + 8u * u, mat_off + 40u * NU + 8u * (u >> 3)};
}
// A raw buffer resource over `bytes` of weights at `base`: loads take a per-lane 32-bit offset plus a scalar offset
// (no vector address arithmetic in the row loop), and a load past `bytes` returns zero instead of faulting.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t weight_rsrc(uint64_t base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc((void*) base, 0, (int) bytes, 0x00020000);
}
__device__ __forceinline__ QuadIQ2S load_quad(__amdgpu_buffer_rsrc_t rs, const QuadOffs& o, uint32_t quad_off) {
    QuadIQ2S q;
    q.is01 = __builtin_amdgcn_raw_buffer_load_b128(rs, o.is, quad_off, 0);
    q.is23 = __builtin_amdgcn_raw_buffer_load_b128(rs, o.is + 16u, quad_off, 0);
    q.hs = __builtin_amdgcn_raw_buffer_load_b64(rs, o.hs, quad_off, 0);
    q.d = __builtin_amdgcn_raw_buffer_load_b64(rs, o.d, quad_off, 0);
    return q;
}
template <int R>
__device__ __forceinline__ RawIQ2S quad_row(const QuadIQ2S& q) {
    RawIQ2S r;
    const u32x4 v = R < 2 ? q.is01 : q.is23;
    r.i4 = (R & 1) ? v.z : v.x;
    r.sg4 = (R & 1) ? v.w : v.y;
    const uint32_t h = R < 2 ? q.hs.x : q.hs.y, d = R < 2 ? q.d.x : q.d.y;
    r.hs = (R & 1) ? (h >> 16) : (h & 0xffffu);
    r.d = (R & 1) ? (d >> 16) : (d & 0xffffu);
    return r;
}
// One sub-block against the lane's activation codes y and their negation yn.  The signs go onto the activation, not
// the weight: v_perm_b32 over the pair (-y word, y word) with the sign byte's selector takes -y_i where value i is
// negative, and the codebook word meets it in one dot4 - two instructions per four weights, no xor, no mask term.
// dy8 = the activation scale / 8.
// Z3: the first product of a sum in the three-operand encoding (dot4_first): one instruction less a sum; it pays in
// the down kernel and costs in the gate/up kernels (measured: their register count goes from 57 to 64).
template <bool Z3 = false>
__device__ __forceinline__ float unit_value(const RawIQ2S& r, const uint2* grid, const uint2* ssel, const int (&y)[8],
                                            const int (&yn)[8], float dy8) {
    int t0 = 0, t1 = 0;
#pragma unroll
    for (int l = 0; l < 4; ++l) {
        const uint32_t idx = ((r.i4 >> (8 * l)) & 255u) | ((r.hs << (8 - 2 * l)) & 0x300u);
        const uint2 g = grid[idx];
        const uint2 sl = ssel[(r.sg4 >> (8 * l)) & 255u];
        const int ya = (int) __builtin_amdgcn_perm((uint32_t) yn[2 * l], (uint32_t) y[2 * l], sl.x);
        const int yb = (int) __builtin_amdgcn_perm((uint32_t) yn[2 * l + 1], (uint32_t) y[2 * l + 1], sl.y);
        if (Z3 && l == 0) t0 = dot4_first((int) g.x, ya);
        else if (Z3 && l == 2) t1 = dot4_first((int) g.x, ya);
        else if (l < 2) t0 = dot4((int) g.x, ya, t0);
        else t1 = dot4((int) g.x, ya, t1);
        if (l < 2) t0 = dot4((int) g.y, yb, t0);
        else t1 = dot4((int) g.y, yb, t1);
    }
    const int s0 = 2 * (int) ((r.hs >> 8) & 15u) + 1, s1 = 2 * (int) ((r.hs >> 12) & 15u) + 1;
    const int isum = __mul24(s0, t0) + __mul24(s1, t1);
    return __fmul_rn(__fmul_rn(f16_bits_to_f32(r.d), dy8), (float) isum);
}
// the byte-wise negation of four int8 codes (none is -128)
__device__ __forceinline__ int neg4(int v) {
    const uint32_t x = ~(uint32_t) v;
    return (int) (((x & 0x7f7f7f7fu) + 0x01010101u) ^ (x & 0x80808080u));
}
// the four rows of a quad: acc[B + r] = this lane's value for row r.  Each value is pinned where it is made: without
// that the optimizer sinks all the batch's decodes down to the reduction and keeps every prefetched quad live.
template <int B, bool Z3 = false>
__device__ __forceinline__ void quad_values(const QuadIQ2S& q, const uint2* grid, const uint2* stab, const int (&y)[8],
                                            const int (&yn)[8], float dy8, float (&acc)[8]) {
#define MAYA_ROW(R)                                                              \
    acc[B + R] = unit_value<Z3>(quad_row<R>(q), grid, stab, y, yn, dy8);         \
    asm volatile("" : "+v"(acc[B + R]));                                         \
    __builtin_amdgcn_sched_barrier(0);
    MAYA_ROW(0) MAYA_ROW(1) MAYA_ROW(2) MAYA_ROW(3)
#undef MAYA_ROW
}

// ---- gate/up, one token, n_embd = 1024 NW: a workgroup of NW waves = the 2 * 32 NW sub-block positions of a
// (gate row, up row) pair; grid (n_ff / ROWS, k).  DEPTH rows are in flight per lane.
template <int NW, int ROWS, int DEPTH, int MINW>
__global__ __launch_bounds__(64 * NW, MINW) void gate_up_iq2s_pos_kernel(maya_moe_args a, Codebooks cb) {
    static_assert(ROWS % 8 == 0 && (DEPTH == 1 || DEPTH == 2), "a batch is two quads; the ring holds one or two");
    constexpr int NU = 32 * NW;  // sub-blocks a row
    __shared__ __align__(16) int lds[kFastLdsWords];
    __shared__ float part[2][2 * NW][8];
    if (a.skip && *a.skip) return;
    // (a window's entries in the order of grp_ent where one is given: the entries of an expert side by side; -1 ends it)
    const int e = (a.grp_ent && !a.grp_ptr) ? a.grp_ent[blockIdx.y] : (int) blockIdx.y;
    if (e < 0) return;
    const uint64_t blob = a.plan_ptr[e];
    if (blob == 0ull) return;
    stage_iq2s_tables_sel<64 * NW>(lds, cb);
    const uint2* grid = (const uint2*) lds;
    const uint2* stab = (const uint2*) (lds + 2048);
    const int t = threadIdx.x, lane = t & 63, hw = t >> 5;
    const bool is_up = t >= NU;
    const int u = is_up ? t - NU : t;
    const int tok = e / a.k;   // the entry's token: its activation row
    int y[8];
    {
        const int4* q = (const int4*) (a.x.q + (size_t) tok * (32 * NU));
        const int4 ya = q[2 * u], yb = q[2 * u + 1];
        y[0] = ya.x, y[1] = ya.y, y[2] = ya.z, y[3] = ya.w, y[4] = yb.x, y[5] = yb.y, y[6] = yb.z, y[7] = yb.w;
    }
    int yn[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) yn[i] = neg4(y[i]);
    const float dy8 = a.x.d[(size_t) tok * NU + u] * 0.125f;
    constexpr uint32_t qb = NU / 8 * 82 * 4;  // bytes of a quad of rows
    const int n_ff = a.layout.n_ff, r0 = blockIdx.x * ROWS;
    // one resource over the expert's gate and up rows; the up rows ride in the lane offset
    const __amdgpu_buffer_rsrc_t rs = weight_rsrc(blob + a.layout.gate_off, (uint32_t) (a.layout.down_off - a.layout.gate_off));
    const QuadOffs qo = quad_offs<NU>(is_up ? (uint32_t) (a.layout.up_off - a.layout.gate_off) : 0u, u);
    const uint32_t quad0 = (uint32_t) (r0 >> 2) * qb;
    constexpr int NQ = ROWS / 4;
    QuadIQ2S ring[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) ring[d] = load_quad(rs, qo, quad0 + (uint32_t) d * qb);
    __syncthreads();
    float acc[8];
#pragma unroll 1
    for (int r = 0; r < ROWS; r += 8) {
        const int q = r >> 2;
        {
            const QuadIQ2S cur = ring[0];
            if (q + DEPTH < NQ) ring[0] = load_quad(rs, qo, quad0 + (uint32_t) (q + DEPTH) * qb);
            quad_values<0>(cur, grid, stab, y, yn, dy8, acc);
        }
        {
            const QuadIQ2S cur = ring[1 % DEPTH];
            if (q + 1 + DEPTH < NQ) ring[1 % DEPTH] = load_quad(rs, qo, quad0 + (uint32_t) (q + 1 + DEPTH) * qb);
            quad_values<4>(cur, grid, stab, y, yn, dy8, acc);
        }
        const float v = reduce8_half(acc, lane);
        const int buf = (r >> 3) & 1;
        if ((lane & 3) == 0) part[buf][hw][(lane >> 2) & 7] = v;
        __syncthreads();
        if (t < 8) {
            float g = part[buf][0][t], up = part[buf][NW][t];
#pragma unroll
            for (int w = 1; w < NW; ++w) {
                g += part[buf][w][t];
                up += part[buf][NW + w][t];
            }
            if (r0 + r + t < n_ff) a.h[(size_t) e * n_ff + r0 + r + t] = swiglu(g, up, a.limit);
        }
    }
}

// ---- gate/up, one token, as a stream of tiles: the same arithmetic as gate_up_iq2s_pos_kernel (a row is the same
// sequence of operations, so its bits are the same), but the workgroups stay: as many workgroups as the chip holds at
// once walk the (entry, 8-row block) tiles and request the next tile's first rows while they compute this one's.  A
// workgroup pays the cold start (arguments, plan, tables, first weights: three memory round trips one after the other)
// once instead of once per 16 rows, and no second round of workgroups starts behind the first.
//
// HEAD: the layer's head rides in the same launch, and no workgroup waits for another.  Workgroup 0 is the router: one
// wave routes the token exactly (route_wave_softmax) and writes ids, weights and the plan for the down launch and the
// caller.  Every other workgroup finds out for itself which experts were picked - the order of the k + 1 largest logits
// (route_wave_order_only; the exact router on its first wave in the rare case that this does not settle it) - and rounds
// its lanes' share of x to Q8_K in registers (q8k_round_lane32: a 256-value block is 8 lanes), while the tables are
// staged: the picks cost a workgroup some hundred instructions on one wave, against a launch and two memory round
// trips between a head kernel and this one.
struct LayerHead {
    int32_t* ids;            // [k]
    float* weights;          // [k]
    uint64_t* plan;          // [k]
    float w_scale;           // the sigmoid router's weight scale and normalisation
    int norm;
};
// the head's inputs when it rides in the gate/up launch, and where its results go
struct LayerHeadIn {
    const float* logits;
    const uint64_t* table;
    const void* x;
    const float* bias;   // the sigmoid router's, or NULL
    int n_expert, x_dtype, sigmoid;
    LayerHead out;
};
// The head of a one-token layer inside a gate/up launch whose workgroups are a (gate row, up row) pair's 2 * 32 NW
// positions, grid (row blocks + 1, k): called by every thread once.  The workgroup (last column, 0) is the exact router
// (ids, weights, plan: hd.out); the rest of that column leaves.  Every other workgroup picks the experts on its last
// wave (up lanes only) from the ORDER of the logits - the exact router on the same wave when two of them are too close to
// call - while the waves with gate lanes round their positions' x to Q8_K in registers (a 256-value block is 8 lanes: the
// lane of position u holds the values o0 .. o0 + 15 and o1 .. o1 + 15 of x, o0 < o1 inside one block) and hand codes and
// scale to the up lanes through LDS.  y: the position's 32 codes in that order, d: its block's scale, blob: the expert of
// slot blockIdx.y.  False: the thread has nothing more to do in this launch.
template <int NW>
__device__ __forceinline__ bool head_in_gate_up(const LayerHeadIn& hd, int n_ent, const int32_t* skip, bool is_up, int u, int o0, int o1,
                                                int (&y)[8], float& d, uint64_t& blob) {
    constexpr int NU = 32 * NW;
    __shared__ uint64_t s_blob[MAYA_MAX_K];
    __shared__ float s_lv[256];
    __shared__ uint64_t s_tab[256];
    __shared__ int s_y[9][NU];
    const int t = threadIdx.x, lane = t & 63, ne = hd.n_expert;
    const bool picker = t >= 64 * (NW - 1), sigm = hd.sigmoid != 0;
    float lv[4] = {0.0f, 0.0f, 0.0f, 0.0f}, bv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    uint64_t tab[4] = {0ull, 0ull, 0ull, 0ull};
    if (picker) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int x = 64 * r + lane;
            lv[r] = x < ne ? hd.logits[x] : -INFINITY;
            tab[r] = x < ne ? hd.table[x] : 0ull;
            if (hd.bias) bv[r] = x < ne ? hd.bias[x] : 0.0f;
        }
    }
    if (blockIdx.x == gridDim.x - 1) {   // the router (it looks at no skip flag, like the head kernel)
        if (blockIdx.y != 0 || !picker) return false;
        int id;
        float w;
        uint64_t ptr;
        if (sigm) {
            float pr[4], sc[4];
            const bool fin = sigmoid_scores(lv, bv, hd.bias != nullptr, ne, pr, sc);
            route_wave_sigmoid(pr, sc, fin, tab, ne, n_ent, hd.out.norm, hd.out.w_scale, id, w, ptr);
        } else {
            route_wave_softmax(lv, tab, ne, n_ent, id, w, ptr);
        }
        if (lane < n_ent) {
            hd.out.ids[lane] = id;
            hd.out.weights[lane] = w;
            hd.out.plan[lane] = ptr;
        }
        return false;
    }
    if (skip && *skip) return false;
    if (picker) {
        __builtin_amdgcn_s_setprio(3);   // the workgroup waits for this wave: it goes first on its SIMD
#pragma unroll
        for (int r = 0; r < 4; ++r) s_tab[64 * r + lane] = tab[r];
        int id;
        uint64_t ptr;
        if (sigm) {
            // the scores are the exact router's own keys: any strictly descending order of the picks is its order
            float pr[4], sc[4];
            const bool fin = sigmoid_scores(lv, bv, hd.bias != nullptr, ne, pr, sc);
            if (route_wave_order_only(sc, fin, ne, n_ent, s_lv, 0.0f, INFINITY, id)) {
                ptr = s_tab[lane < n_ent ? id : 0];
            } else {
                float w;
                route_wave_sigmoid(pr, sc, fin, tab, ne, n_ent, hd.out.norm, hd.out.w_scale, id, w, ptr);
            }
        } else if (route_wave_order_only(lv, true, ne, n_ent, s_lv, 1e-6f, 60.0f, id)) {
            ptr = s_tab[lane < n_ent ? id : 0];
        } else {
            float w;
            route_wave_softmax(lv, tab, ne, n_ent, id, w, ptr);
        }
        if (lane < n_ent) s_blob[lane] = ptr;
        __builtin_amdgcn_s_setprio(0);
    }
    float v[32];
    if (!is_up) {
        if (hd.x_dtype == MAYA_DT_F32) {
            const float4 *xa = (const float4*) ((const float*) hd.x + o0), *xb = (const float4*) ((const float*) hd.x + o1);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 lo = xa[i], hi = xb[i];
                v[4 * i] = lo.x, v[4 * i + 1] = lo.y, v[4 * i + 2] = lo.z, v[4 * i + 3] = lo.w;
                v[16 + 4 * i] = hi.x, v[16 + 4 * i + 1] = hi.y, v[16 + 4 * i + 2] = hi.z, v[16 + 4 * i + 3] = hi.w;
            }
        } else {
            const uint4 *xa = (const uint4*) ((const uint16_t*) hd.x + o0), *xb = (const uint4*) ((const uint16_t*) hd.x + o1);
            uint32_t w4[16];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const uint4 lo = xa[i], hi = xb[i];
                w4[4 * i] = lo.x, w4[4 * i + 1] = lo.y, w4[4 * i + 2] = lo.z, w4[4 * i + 3] = lo.w;
                w4[8 + 4 * i] = hi.x, w4[8 + 4 * i + 1] = hi.y, w4[8 + 4 * i + 2] = hi.z, w4[8 + 4 * i + 3] = hi.w;
            }
            if (hd.x_dtype == MAYA_DT_BF16) {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    v[2 * j] = __uint_as_float(w4[j] << 16);
                    v[2 * j + 1] = __uint_as_float(w4[j] & 0xffff0000u);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    v[2 * j] = f16_bits_to_f32((uint16_t) (w4[j] & 0xffffu));
                    v[2 * j + 1] = f16_bits_to_f32((uint16_t) (w4[j] >> 16));
                }
            }
        }
    }
    d = 0.0f;
    // (a wave with a gate lane rounds: the block's 8 lanes are all gate lanes or all up lanes, NU being a multiple of 8)
    if (64 * (t >> 6) < NU) {
        q8k_round_lane32(v, [&](int i) { return i < 16 ? (o0 & 255) + i : (o1 & 255) + i - 16; }, y, d);
        if (!is_up) {
#pragma unroll
            for (int i = 0; i < 8; ++i) s_y[i][u] = y[i];
            s_y[8][u] = __float_as_int(d);
        }
    }
    __syncthreads();
    if (is_up) {
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = s_y[i][u];
        d = __int_as_float(s_y[8][u]);
    }
    const uint64_t bl = s_blob[blockIdx.y];
    const uint32_t lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) bl);
    const uint32_t hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (bl >> 32));
    blob = ((uint64_t) hi << 32) | lo;
    return blob != 0ull;
}

// The leading arguments are what the kernel asks of memory first; as plain pointers and integers at the head of the
// argument list they arrive in scalar registers with the dispatch (a structure passed by value is read from memory
// first).  HEAD: p0 = the logits [n_expert], p1 = the table [n_expert] of blob addresses (0 = absent), p2 = x [n_embd] of
// dtype `mode & 255`, bias = the sigmoid router's (`mode >> 8` = 1: the sigmoid router) or NULL; else p0 = the plan's blob
// addresses (a.plan_ptr), p1 = the codes of x (a.x.q), p2 = their scales (a.x.d).
template <int NW, int MINW, bool HEAD>
__global__ __launch_bounds__(NW > 4 ? 512 : 256, MINW) void gate_up_iq2s_tiles_kernel(const void* __restrict__ p0, const void* __restrict__ p1,
                                                                                      const void* __restrict__ p2,
                                                                                      const uint64_t* __restrict__ iq2s_grid,
                                                                                      const float* __restrict__ bias,
                                                                                      const int32_t* __restrict__ skip, int n_expert,
                                                                                      int mode, int n_ent, maya_moe_args a,
                                                                                      LayerHead hd) {
    constexpr int NU = 32 * NW;  // sub-blocks a row
    __shared__ __align__(16) int lds[kFastLdsWords];
    __shared__ float part[2][2 * NW][8];
    __shared__ uint64_t s_blob[HEAD ? MAYA_MAX_K : 1];
    __shared__ float s_lv[HEAD ? 256 : 1];              // the picker's scratch: the logits, the table
    __shared__ uint64_t s_tab[HEAD ? 256 : 1];
    __shared__ int s_y[HEAD ? 9 : 1][HEAD ? NU : 1];   // a position's codes and scale, from its gate lane to its up lane
    const uint2* grid = (const uint2*) lds;
    const uint2* stab = (const uint2*) (lds + 2048);
    const int t = threadIdx.x, lane = t & 63, hw = t >> 5;
    const bool is_up = t >= NU;
    const int u = is_up ? t - NU : t;
    // (n_ent = a.k: one token, entry = plan slot)
    int y[8];
    float dy8;
    int first_tile = blockIdx.x, tile_step = gridDim.x;
    TablePieces<2048, 64 * NW> tp;   // the codebook: requested early, stored once the other first loads are on their way
    if constexpr (!HEAD) table_request(iq2s_grid, tp);
    if constexpr (HEAD) {
        // The workgroup's last wave holds up rows only; it picks the experts while the gate lanes round x (a gate lane and
        // the up lane of the same position need the same codes: the gate lane rounds, the up lane takes them from LDS).
        const int ne = n_expert;
        const float* logits = (const float*) p0;
        const uint64_t* table = (const uint64_t*) p1;
        const bool picker = t >= 64 * (NW - 1);
        const int x_dtype = mode & 255;
        const bool sigm = (mode >> 8) != 0;
        float lv[4] = {0.0f, 0.0f, 0.0f, 0.0f}, bv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        uint64_t tab[4] = {0ull, 0ull, 0ull, 0ull};
        if (picker) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int e = 64 * r + lane;
                lv[r] = e < ne ? logits[e] : -INFINITY;
                tab[r] = e < ne ? table[e] : 0ull;
                if (bias) bv[r] = e < ne ? bias[e] : 0.0f;
            }
        }
        table_request(iq2s_grid, tp);   // (behind the picker's loads: loads come back in the order they were asked for)
        if (blockIdx.x == 0) {   // the router (it looks at no skip flag, like the head kernel)
            if (!picker) return;
            int id;
            float w;
            uint64_t ptr;
            if (sigm) {
                float p[4], sc[4];
                const bool fin = sigmoid_scores(lv, bv, bias != nullptr, ne, p, sc);
                route_wave_sigmoid(p, sc, fin, tab, ne, n_ent, hd.norm, hd.w_scale, id, w, ptr);
            } else {
                route_wave_softmax(lv, tab, ne, n_ent, id, w, ptr);
            }
            if (lane < n_ent) {
                hd.ids[lane] = id;
                hd.weights[lane] = w;
                hd.plan[lane] = ptr;
            }
            return;
        }
        first_tile = (int) blockIdx.x - 1, tile_step = (int) gridDim.x - 1;
        const int skipv = skip ? *skip : 0;
        if (skipv) return;
        if (picker) {   // (before x is loaded: the values of x then take no registers here)
            __builtin_amdgcn_s_setprio(3);   // the workgroup waits for this wave: it goes first on its SIMD
#pragma unroll
            for (int r = 0; r < 4; ++r) s_tab[64 * r + lane] = tab[r];
            int id;
            uint64_t ptr;
            if (sigm) {
                // the scores are the exact router's own keys: any strictly descending order of the picks is its order
                float p[4], sc[4];
                const bool fin = sigmoid_scores(lv, bv, bias != nullptr, ne, p, sc);
                if (route_wave_order_only(sc, fin, ne, n_ent, s_lv, 0.0f, INFINITY, id)) {
                    ptr = s_tab[lane < n_ent ? id : 0];
                } else {
                    float w;
                    route_wave_sigmoid(p, sc, fin, tab, ne, n_ent, hd.norm, hd.w_scale, id, w, ptr);
                }
            } else if (route_wave_order_only(lv, true, ne, n_ent, s_lv, 1e-6f, 60.0f, id)) {
                ptr = s_tab[lane < n_ent ? id : 0];
            } else {
                float w;
                route_wave_softmax(lv, tab, ne, n_ent, id, w, ptr);
            }
            if (lane < n_ent) s_blob[lane] = ptr;
            __builtin_amdgcn_s_setprio(0);
        }
        float v[32];
        if (!is_up) {
            if (x_dtype == MAYA_DT_F32) {
                const float4* xv = (const float4*) p2 + 8 * u;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float4 q = xv[i];
                    v[4 * i] = q.x, v[4 * i + 1] = q.y, v[4 * i + 2] = q.z, v[4 * i + 3] = q.w;
                }
            } else {
                const uint4* xv = (const uint4*) p2 + 4 * u;
                uint32_t w4[16];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint4 q = xv[i];
                    w4[4 * i] = q.x, w4[4 * i + 1] = q.y, w4[4 * i + 2] = q.z, w4[4 * i + 3] = q.w;
                }
                if (x_dtype == MAYA_DT_BF16) {
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        v[2 * j] = __uint_as_float(w4[j] << 16);
                        v[2 * j + 1] = __uint_as_float(w4[j] & 0xffff0000u);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        v[2 * j] = f16_bits_to_f32((uint16_t) (w4[j] & 0xffffu));
                        v[2 * j + 1] = f16_bits_to_f32((uint16_t) (w4[j] >> 16));
                    }
                }
            }
        }
        store_iq2s_selectors<64 * NW>(lds);
        table_store(lds, tp);
        // (a wave with a gate lane rounds: the block's 8 lanes are all gate lanes or all up lanes, NU being a multiple of 8)
        if (64 * (t >> 6) < NU) {
            float d;
            q8k_round_lane32(v, [&](int i) { return 32 * (lane & 7) + i; }, y, d);
            dy8 = d * 0.125f;
            if (!is_up) {
#pragma unroll
                for (int i = 0; i < 8; ++i) s_y[i][u] = y[i];
                s_y[8][u] = __float_as_int(dy8);
            }
        }
        __syncthreads();
        if (is_up) {
#pragma unroll
            for (int i = 0; i < 8; ++i) y[i] = s_y[i][u];
            dy8 = __int_as_float(s_y[8][u]);
        }
    } else {
        // everything the first tile needs is requested side by side: no load waits on another
        const int skipv = skip ? *skip : 0;
        {
            const int4* q = (const int4*) p1;
            const int4 ya = q[2 * u], yb = q[2 * u + 1];
            y[0] = ya.x, y[1] = ya.y, y[2] = ya.z, y[3] = ya.w, y[4] = yb.x, y[5] = yb.y, y[6] = yb.z, y[7] = yb.w;
        }
        dy8 = ((const float*) p2)[u] * 0.125f;
        if (skipv) return;
    }
    int yn[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) yn[i] = neg4(y[i]);
    constexpr uint32_t qb = NU / 8 * 82 * 4;  // bytes of a quad of rows
    const int n_ff = a.layout.n_ff;
    const int tiles_per_entry = n_ff >> 3, n_tiles = n_ent * tiles_per_entry;
    const uint32_t gu_bytes = (uint32_t) (a.layout.down_off - a.layout.gate_off);
    const QuadOffs qo = quad_offs<NU>(is_up ? (uint32_t) (a.layout.up_off - a.layout.gate_off) : 0u, u);
    // the resource of a tile's expert (an absent expert: an empty resource, whose loads read as zero and touch nothing);
    // the entry is the same for the whole workgroup: its blob address is a scalar load (HEAD: read from LDS and moved to
    // scalar registers)
    auto blob_of = [&](int e) -> uint64_t {
        if constexpr (HEAD) {
            const uint64_t b = s_blob[e];
            const uint32_t lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) b);
            const uint32_t hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (b >> 32));
            return ((uint64_t) hi << 32) | lo;
        } else {
            return ((const uint64_t*) p0)[e];
        }
    };
    int tile = first_tile;
    if (tile >= n_tiles) return;
    int e = tile / tiles_per_entry, rb = tile - e * tiles_per_entry;
    uint64_t blob = blob_of(e);
    __amdgpu_buffer_rsrc_t rs = weight_rsrc(blob ? blob + a.layout.gate_off : 0ull, blob ? gu_bytes : 0u);
    QuadIQ2S ring = load_quad(rs, qo, (uint32_t) (2 * rb) * qb);
    if constexpr (!HEAD) {
        store_iq2s_selectors<64 * NW>(lds);
        table_store(lds, tp);
        __syncthreads();
    }
    float acc[8];
    int buf = 0;
    // The ring is consumed in place: a register pair of the quad is requested again, for the quad after, as soon as its
    // last row is done, so a lane never holds a second copy of a quad (12 registers saved: 8 waves a SIMD).
#define MAYA_TROW(B, R)                                                          \
    acc[B + R] = unit_value(quad_row<R>(ring), grid, stab, y, yn, dy8);          \
    asm volatile("" : "+v"(acc[B + R]));                                         \
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll 1
    for (;;) {
        const uint32_t o1 = (uint32_t) (2 * rb + 1) * qb;
        MAYA_TROW(0, 0) MAYA_TROW(0, 1)
        ring.is01 = __builtin_amdgcn_raw_buffer_load_b128(rs, qo.is, o1, 0);
        MAYA_TROW(0, 2) MAYA_TROW(0, 3)
        ring.is23 = __builtin_amdgcn_raw_buffer_load_b128(rs, qo.is + 16u, o1, 0);
        ring.hs = __builtin_amdgcn_raw_buffer_load_b64(rs, qo.hs, o1, 0);
        ring.d = __builtin_amdgcn_raw_buffer_load_b64(rs, qo.d, o1, 0);
        // the next tile (past the end: the empty resource)
        const int nt = tile + tile_step;
        const bool more = nt < n_tiles;
        const int ne = more ? nt / tiles_per_entry : 0, nrb = nt - ne * tiles_per_entry;
        const uint64_t pblob = blob_of(ne);
        const uint64_t nblob = more ? pblob : 0ull;
        const __amdgpu_buffer_rsrc_t nrs = weight_rsrc(nblob ? nblob + a.layout.gate_off : 0ull, nblob ? gu_bytes : 0u);
        const uint32_t o2 = (uint32_t) (2 * nrb) * qb;
        MAYA_TROW(4, 0) MAYA_TROW(4, 1)
        ring.is01 = __builtin_amdgcn_raw_buffer_load_b128(nrs, qo.is, o2, 0);
        MAYA_TROW(4, 2) MAYA_TROW(4, 3)
        ring.is23 = __builtin_amdgcn_raw_buffer_load_b128(nrs, qo.is + 16u, o2, 0);
        ring.hs = __builtin_amdgcn_raw_buffer_load_b64(nrs, qo.hs, o2, 0);
        ring.d = __builtin_amdgcn_raw_buffer_load_b64(nrs, qo.d, o2, 0);
        const float v = reduce8_half(acc, lane);
        if ((lane & 3) == 0) part[buf][hw][(lane >> 2) & 7] = v;
        const bool present = blob != 0ull;
        __syncthreads();
        if (t < 8) {
            float g = part[buf][0][t], up = part[buf][NW][t];
#pragma unroll
            for (int w = 1; w < NW; ++w) {
                g += part[buf][w][t];
                up += part[buf][NW + w][t];
            }
            if (present) a.h[(size_t) e * n_ff + 8 * rb + t] = swiglu(g, up, a.limit);
        }
        if (!more) break;
        tile = nt, e = ne, rb = nrb, rs = nrs, blob = nblob, buf ^= 1;
    }
#undef MAYA_TROW
}

// ---- down + combine, one token, n_ff = 32 NU <= 2048 (NU sub-blocks a row on the first NU lanes of one wave; NU a
// multiple of 8, the lanes past it idle): wave w = plan slot w, rows in batches of 8; grid (n_embd / ROWS).  The slots' rows
// meet in LDS and are summed in slot order.
template <int ROWS, int DEPTH, int MINW, int NU = 64>
__global__ __launch_bounds__(512, MINW) void down_iq2s_pos_kernel(const uint64_t* __restrict__ plan_ptr, const float* __restrict__ plan_w,
                                                                  const float* __restrict__ h, const uint64_t* __restrict__ iq2s_grid,
                                                                  const int32_t* __restrict__ skip, const int8_t* __restrict__ hq_q, int k,
                                                                  int n_embd, maya_moe_args a, Codebooks cb) {
    // (the leading arguments repeat a.plan_ptr, a.plan_w, a.h, cb.iq2s, a.skip, a.hq.q, a.k, a.layout.n_embd: plain pointers
    // and integers at the head of the argument list arrive in scalar registers with the dispatch, a structure passed by
    // value is read from memory first - and everything the kernel asks of memory at its start hangs on these)
    static_assert(ROWS % 4 == 0 && DEPTH >= 1 && DEPTH <= ROWS / 4, "a batch is two quads (the last may be one); the ring holds DEPTH quads");
    static_assert(NU % 8 == 0 && NU >= 8 && NU <= 64, "whole 256-value blocks on one wave");
    __shared__ __align__(16) int lds[kFastLdsWords];
    __shared__ float part[8][ROWS];
    __shared__ float s_w[8];
    __shared__ int s_on[8];
    const uint2* grid = (const uint2*) lds;
    const uint2* stab = (const uint2*) (lds + 2048);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int bx, by;
    down_block_of_grid(bx, by);
    const int r0 = bx * ROWS;
    const int e0 = by * k;   // the token's first entry; wave w = its slot w
    // Everything the workgroup needs before its weights is requested side by side, ahead of the one barrier: the skip
    // flag, the plan (the wave's slot; the slots' presence and weights for the combine), the slot's h and the tables.
    // A wave past slot k - 1 reads that slot's data and drops it: no branch, and no load waits on another.
    const int skipv = skip ? *skip : 0;
    const int ent = e0 + min(wave, k - 1);
    uint64_t blob = plan_ptr[ent];   // (asked for first: loads come back in order, and the weights' request waits for this one)
    TablePieces<2048, 512> tp;
    table_request(iq2s_grid, tp);
    const int ci = e0 + min((int) threadIdx.x & 7, k - 1);
    const uint64_t c_ptr = plan_ptr[ci];
    const float c_w = plan_w[ci];
    const bool on = NU == 64 || lane < NU;   // (an idle lane reads the last position's data and uses zeros)
    const int pos = on ? lane : NU - 1;
    const bool rounded = hq_q != nullptr;
    int y[8];
    float dy8 = 0.0f;
    float v[32];
    if (rounded) {
        const int4* q = (const int4*) (hq_q + (size_t) ent * (32 * NU));
        const int4 ya = q[2 * pos], yb = q[2 * pos + 1];
        y[0] = ya.x, y[1] = ya.y, y[2] = ya.z, y[3] = ya.w, y[4] = yb.x, y[5] = yb.y, y[6] = yb.z, y[7] = yb.w;
        dy8 = a.hq.d[(size_t) ent * NU + pos] * 0.125f;
    } else {
        const float4* hv = (const float4*) (h + (size_t) ent * (32 * NU) + 32 * pos);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float4 t = hv[i];
            v[4 * i] = t.x, v[4 * i + 1] = t.y, v[4 * i + 2] = t.z, v[4 * i + 3] = t.w;
        }
    }
    if (skipv) return;
    if (wave >= k) blob = 0ull;
    constexpr uint32_t qb = NU / 8 * 82 * 4;
    // the wave's blob address is wave-uniform; readfirstlane (a signed int: widened through uint32_t) moves it to
    // scalar registers for the buffer resource (no blob: an empty resource, whose loads read as zero and touch nothing)
    const uint64_t mat = blob ? blob + a.layout.down_off : 0ull;
    const uint32_t mat_lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) mat);
    const uint32_t mat_hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (mat >> 32));
    const __amdgpu_buffer_rsrc_t rs = weight_rsrc(((uint64_t) mat_hi << 32) | (uint64_t) mat_lo, (mat_lo | mat_hi) != 0u ? (uint32_t) (n_embd >> 2) * qb : 0u);
    const QuadOffs qo = quad_offs<NU>(0u, pos);
    const uint32_t quad0 = (uint32_t) (r0 >> 2) * qb;
    constexpr int NQ = ROWS / 4;
    // the first rows' weights are requested before the tables are stored and h is rounded: one trip to memory for the
    // tables, the plan and h, a second for the weights, and the barrier and the rounding sit under the second
    QuadIQ2S ring[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) ring[d] = load_quad(rs, qo, quad0 + (uint32_t) d * qb);
    store_iq2s_selectors<512>(lds);
    table_store(lds, tp);
    if (threadIdx.x < 8) {
        s_on[threadIdx.x] = (int) threadIdx.x < k && c_ptr != 0ull;
        s_w[threadIdx.x] = c_w;
    }
    __syncthreads();
    if (blob != 0ull) {
        if (rounded) {
            if (!on) {
#pragma unroll
                for (int i = 0; i < 8; ++i) y[i] = 0;
                dy8 = 0.0f;
            }
        } else {
            // no rounded h given: the wave rounds its slot's h to Q8_K itself (quant_q8k_block's arithmetic): a lane holds
            // sub-block `lane`, a 256-value block is 8 lanes; the block's signed maximum is the value at the FIRST largest
            // magnitude - inside a lane the scan keeps the first, between lanes the lower lane wins a tie
            if (!on) {
#pragma unroll
                for (int i = 0; i < 32; ++i) v[i] = 0.0f;
            }
            float d;
            q8k_round_lane32(v, [&](int i) { return 32 * (lane & 7) + i; }, y, d);
            dy8 = on ? d * 0.125f : 0.0f;
        }
        int yn[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) yn[i] = neg4(y[i]);
        float acc[8];
        // (unrolled: the ring's slots are then fixed registers whatever its depth)
#pragma unroll
        for (int r = 0; r < ROWS; r += 8) {
            const int q = r >> 2;
            {
                const QuadIQ2S cur = ring[q % DEPTH];
                if (q + DEPTH < NQ) ring[q % DEPTH] = load_quad(rs, qo, quad0 + (uint32_t) (q + DEPTH) * qb);
                quad_values<0, true>(cur, grid, stab, y, yn, dy8, acc);
            }
            if (q + 1 < NQ) {
                const QuadIQ2S cur = ring[(q + 1) % DEPTH];
                if (q + 1 + DEPTH < NQ) ring[(q + 1) % DEPTH] = load_quad(rs, qo, quad0 + (uint32_t) (q + 1 + DEPTH) * qb);
                quad_values<4, true>(cur, grid, stab, y, yn, dy8, acc);
            } else {
#pragma unroll
                for (int i = 4; i < 8; ++i) acc[i] = 0.0f;   // an odd number of quads: the last batch's second half is empty
            }
            float v = reduce8_half(acc, lane);
            v = add_other_half(v);
            const int rr = r + ((lane >> 2) & 7);
            if ((lane & 35) == 0 && (ROWS % 8 == 0 || rr < ROWS)) part[wave][rr] = v;
        }
    }
    __syncthreads();
    if (threadIdx.x < ROWS) {
        const int c = threadIdx.x;
        float sum = 0.0f;
        bool first = true;
#pragma unroll
        for (int i = 0; i < 8; ++i) {   // the present slots in slot order; the first product starts the sum
            const bool have = s_on[i] != 0;
            const float p = __fmul_rn(part[i][c], s_w[i]);
            const float t = first ? p : __fadd_rn(sum, p);
            sum = have ? t : sum;
            first = first && !have;
        }
        const size_t o = (size_t) by * n_embd + r0 + c;
        if (a.add && (!a.add_flag || *a.add_flag)) sum = __fadd_rn(sum, a.add[o]);
        if (a.add2) sum = __fadd_rn(sum, a.add2[o]);
        a.out[o] = sum;
        if (a.part)
            for (int i = 0; i < a.k; ++i)
                if (s_on[i]) a.part[(size_t) (e0 + i) * n_embd + r0 + c] = part[i][c];
    }
}

}  // namespace maya
