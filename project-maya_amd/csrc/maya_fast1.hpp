// maya_fast1.hpp - position-mapped decode kernels for IQ1_S rows in the stream packing: the skeleton of the IQ2_S ones
// (maya_fast.hpp) with a cheaper unit.  A value is d (2 s + 1) (g + delta / 8), g in {-1, 0, +1} from the 2048-entry
// grid, delta = +-1 a sub-block (third_party/ggml/ggml-common.h:425-430, src/kernels/cuda/iq_kernels.cu:825-837), i.e.
// the int8 code 8 g + delta.  The grid sits in LDS as t = 8 g + 9 (bytes 1 / 9 / 17), so a looked-up word is the operand
// of the dot products as it is, and
//   sum (8 g + delta) y = sum t y + (delta - 9) SY,   SY = the sum of the lane's 32 activation codes (fixed for the kernel):
// four lookups, eight dot products and a multiply-add a sub-block, no sign table and no per-byte arithmetic.
//
// Stream packing of IQ1_S (rows in quads; nu = k / 32 sub-blocks a row; a quad keeps its 4 x row_bytes = 25 nu bytes):
//   the 4 index bytes of sub-block u of row r at 4 (4 u + r); its 16-bit qh word at 16 nu + 2 (4 u + r);
//   block b's FP16 scale at 24 nu + 2 (4 b + r).
// IQ1_M (third_party/ggml/ggml-common.h:433-438, iq_kernels.cu:839-855) differs in three places: delta belongs to a group
// of 8 values (so the correction uses the four sums of 8 codes), a 3-bit scale to 16 values, and the FP16 block scale is
// scattered over the top nibbles of the four 16-bit scale words.  Its stream packing (a quad keeps its 28 nu bytes):
//   index bytes and qh words as above; then 8 bytes a (block b, row r) at 24 nu + 8 (4 b + r): the block scale put
//   together (2 bytes), then the sixteen 3-bit scales in order (6 bytes; sub-block ib's pair at bit 6 ib).
#pragma once

namespace maya {

template <int NT>
__device__ __forceinline__ void stage_iq1s_table(int* lds, const Codebooks& cb) {
    TablePieces<4096, NT> t;
    table_request(cb.iq1s, t);
    table_store(lds, t, [](int w) {
        const uint32_t g = (uint32_t) w;
        const uint32_t neg = (g >> 1) & 0x01010101u, pos = g & ~(g >> 1) & 0x01010101u;
        return (int) (0x09090909u + (pos << 3) - (neg << 3));
    });
}
constexpr int kFast1LdsWords = 4096;

// A lane's share of one quad of rows (4 rows x its sub-block): 8 registers
struct QuadIQ1S {
    u32x4 i4;      // the four index bytes of rows 0..3
    u32x2 qh, d;   // four qh halfwords, four FP16 block scales
};
struct QuadOffs1 {
    uint32_t i4, qh, d;
};
template <int NU>
__device__ __forceinline__ QuadOffs1 quad_offs1(uint32_t mat_off, int u) {
    return QuadOffs1{mat_off + 16u * u, mat_off + 16u * NU + 8u * u, mat_off + 24u * NU + 8u * (u >> 3)};
}
__device__ __forceinline__ QuadIQ1S load_quad1(__amdgpu_buffer_rsrc_t rs, const QuadOffs1& o, uint32_t quad_off) {
    QuadIQ1S q;
    q.i4 = __builtin_amdgcn_raw_buffer_load_b128(rs, o.i4, quad_off, 0);
    q.qh = __builtin_amdgcn_raw_buffer_load_b64(rs, o.qh, quad_off, 0);
    q.d = __builtin_amdgcn_raw_buffer_load_b64(rs, o.d, quad_off, 0);
    return q;
}
// row R of the quad against the lane's activation codes; sy = the sum of the lane's 32 codes
template <int R>
__device__ __forceinline__ float unit1_value(const QuadIQ1S& q, const uint2* grid, const int (&y)[8], int sy, float dy8) {
    const uint32_t i4 = q.i4[R];
    const uint32_t hw = R < 2 ? q.qh.x : q.qh.y, dw = R < 2 ? q.d.x : q.d.y;
    const uint32_t qh = (R & 1) ? (hw >> 16) : (hw & 0xffffu), d = (R & 1) ? (dw >> 16) : (dw & 0xffffu);
    int t = 0;
#pragma unroll
    for (int l = 0; l < 4; ++l) {
        const uint2 g = grid[((i4 >> (8 * l)) & 255u) | (((qh >> (3 * l)) & 7u) << 8)];
        t = dot4((int) g.x, y[2 * l], t);
        t = dot4((int) g.y, y[2 * l + 1], t);
    }
    t += __mul24((qh & 0x8000u) ? -10 : -8, sy);   // (a 24-bit multiply-add: the 32-bit one runs at a quarter of the rate)
    const int isum = __mul24(2 * (int) ((qh >> 12) & 7u) + 1, t);
    return __fmul_rn(__fmul_rn(f16_bits_to_f32(d), dy8), (float) isum);
}
template <int B>
__device__ __forceinline__ void quad1_values(const QuadIQ1S& q, const uint2* grid, const int (&y)[8], int sy, float dy8, float (&acc)[8]) {
#define MAYA_ROW(R)                                              \
    acc[B + R] = unit1_value<R>(q, grid, y, sy, dy8);            \
    asm volatile("" : "+v"(acc[B + R]));                         \
    __builtin_amdgcn_sched_barrier(0);
    MAYA_ROW(0) MAYA_ROW(1) MAYA_ROW(2) MAYA_ROW(3)
#undef MAYA_ROW
}
__device__ __forceinline__ int sum32_codes(const int (&y)[8]) {
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s = dot4(0x01010101, y[i], s);
    return s;
}

// ---- gate/up, n_embd = 1024 NW: a workgroup of NW waves = the 2 * 32 NW sub-block positions of a (gate row, up row) pair;
// grid (n_ff / ROWS, entries); entry e = token e / k, slot e % k.  Rows in batches of 8 (two quads), a quad ahead.
// HEAD (one token): the layer's head rides in this launch (head_in_gate_up) - grid (n_ff / ROWS + 1, k).
template <int NW, int ROWS, int MINW, bool HEAD = false>
__global__ __launch_bounds__(64 * NW, MINW) void gate_up_iq1s_pos_kernel(maya_moe_args a, Codebooks cb, LayerHeadIn hd) {
    static_assert(ROWS % 8 == 0, "a batch is two quads");
    constexpr int NU = 32 * NW;
    __shared__ __align__(16) int lds[kFast1LdsWords];
    __shared__ float part[2][2 * NW][8];
    const int t = threadIdx.x, lane = t & 63, hw = t >> 5;
    const bool is_up = t >= NU;
    const int u = is_up ? t - NU : t;
    const int e = blockIdx.y;
    uint64_t blob;
    int y[8];
    float dy8;
    if constexpr (HEAD) {
        float d;
        if (!head_in_gate_up<NW>(hd, a.k, a.skip, is_up, u, 32 * u, 32 * u + 16, y, d, blob)) return;
        dy8 = d * 0.125f;
    } else {
        if (a.skip && *a.skip) return;
        blob = a.plan_ptr[e];
        if (blob == 0ull) return;
        const int tok = e / a.k;
        const int4* q = (const int4*) (a.x.q + (size_t) tok * (32 * NU));
        const int4 ya = q[2 * u], yb = q[2 * u + 1];
        y[0] = ya.x, y[1] = ya.y, y[2] = ya.z, y[3] = ya.w, y[4] = yb.x, y[5] = yb.y, y[6] = yb.z, y[7] = yb.w;
        dy8 = a.x.d[(size_t) tok * NU + u] * 0.125f;
    }
    stage_iq1s_table<64 * NW>(lds, cb);
    const uint2* grid = (const uint2*) lds;
    const int sy = sum32_codes(y);
    constexpr uint32_t qb = NU / 8 * 50 * 4;  // bytes of a quad of rows
    const int n_ff = a.layout.n_ff, r0 = blockIdx.x * ROWS;
    const __amdgpu_buffer_rsrc_t rs = weight_rsrc(blob + a.layout.gate_off, (uint32_t) (a.layout.down_off - a.layout.gate_off));
    const QuadOffs1 qo = quad_offs1<NU>(is_up ? (uint32_t) (a.layout.up_off - a.layout.gate_off) : 0u, u);
    const uint32_t quad0 = (uint32_t) (r0 >> 2) * qb;
    constexpr int NQ = ROWS / 4;
    QuadIQ1S nxt = load_quad1(rs, qo, quad0);
    __syncthreads();
    float acc[8];
#pragma unroll 1
    for (int r = 0; r < ROWS; r += 8) {
        const int q = r >> 2;
        {
            const QuadIQ1S cur = nxt;
            nxt = load_quad1(rs, qo, quad0 + (uint32_t) (q + 1) * qb);
            quad1_values<0>(cur, grid, y, sy, dy8, acc);
        }
        {
            const QuadIQ1S cur = nxt;
            if (q + 2 < NQ) nxt = load_quad1(rs, qo, quad0 + (uint32_t) (q + 2) * qb);
            quad1_values<4>(cur, grid, y, sy, dy8, acc);
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

// ---- down + combine, n_ff = 2048 (64 sub-blocks a row = one wave): wave w = slot w of token blockIdx.y, rows in batches
// of 8; grid (n_embd / ROWS, tokens).  Without a rounded h (hq.q == NULL) a wave rounds its slot's h to Q8_K itself.  The
// slots' rows meet in LDS and are summed in slot order.
template <int ROWS, int MINW, int NU = 64>
__global__ __launch_bounds__(512, MINW) void down_iq1s_pos_kernel(maya_moe_args a, Codebooks cb) {
    static_assert(ROWS % 8 == 0, "a batch is two quads");
    static_assert(NU % 8 == 0 && NU >= 8 && NU <= 64, "whole 256-value blocks on one wave");
    __shared__ __align__(16) int lds[kFast1LdsWords];
    __shared__ float part[8][ROWS];
    if (a.skip && *a.skip) return;
    stage_iq1s_table<512>(lds, cb);
    const uint2* grid = (const uint2*) lds;
    const int n_embd = a.layout.n_embd;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r0 = blockIdx.x * ROWS;
    const int e0 = blockIdx.y * a.k, ent = e0 + wave;
    const uint64_t blob = wave < a.k ? a.plan_ptr[ent] : 0ull;
    __syncthreads();
    if (blob != 0ull) {
        constexpr uint32_t qb = NU / 8 * 50 * 4;
        const uint64_t mat = blob + a.layout.down_off;
        const uint32_t mat_lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) mat);
        const uint32_t mat_hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (mat >> 32));
        const __amdgpu_buffer_rsrc_t rs = weight_rsrc(((uint64_t) mat_hi << 32) | (uint64_t) mat_lo, (uint32_t) (n_embd >> 2) * qb);
        // (an idle lane - past the row's NU positions - reads the last position's weights again and meets them with zero
        // activations)
        const bool on = NU == 64 || lane < NU;
        const int pos = on ? lane : NU - 1;
        const QuadOffs1 qo = quad_offs1<NU>(0u, pos);
        const uint32_t quad0 = (uint32_t) (r0 >> 2) * qb;
        constexpr int NQ = ROWS / 4;
        QuadIQ1S nxt = load_quad1(rs, qo, quad0);
        int y[8];
        float dy8;
        if (a.hq.q) {
            const int4* q = (const int4*) (a.hq.q + (size_t) ent * (32 * NU));
            const int4 ya = q[2 * pos], yb = q[2 * pos + 1];
            y[0] = ya.x, y[1] = ya.y, y[2] = ya.z, y[3] = ya.w, y[4] = yb.x, y[5] = yb.y, y[6] = yb.z, y[7] = yb.w;
            dy8 = a.hq.d[(size_t) ent * NU + pos] * 0.125f;
        } else {
            const float4* hv = (const float4*) (a.h + (size_t) ent * (32 * NU) + 32 * pos);
            float v[32];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float4 t = hv[i];
                v[4 * i] = t.x, v[4 * i + 1] = t.y, v[4 * i + 2] = t.z, v[4 * i + 3] = t.w;
            }
            if (!on) {
#pragma unroll
                for (int i = 0; i < 32; ++i) v[i] = 0.0f;
            }
            float d;
            q8k_round_lane32(v, [&](int i) { return 32 * (lane & 7) + i; }, y, d);
            dy8 = d * 0.125f;
        }
        if (!on) {
#pragma unroll
            for (int i = 0; i < 8; ++i) y[i] = 0;
            dy8 = 0.0f;
        }
        const int sy = sum32_codes(y);
        float acc[8];
#pragma unroll 1
        for (int r = 0; r < ROWS; r += 8) {
            const int q = r >> 2;
            {
                const QuadIQ1S cur = nxt;
                nxt = load_quad1(rs, qo, quad0 + (uint32_t) (q + 1) * qb);
                quad1_values<0>(cur, grid, y, sy, dy8, acc);
            }
            {
                const QuadIQ1S cur = nxt;
                if (q + 2 < NQ) nxt = load_quad1(rs, qo, quad0 + (uint32_t) (q + 2) * qb);
                quad1_values<4>(cur, grid, y, sy, dy8, acc);
            }
            float v = reduce8_half(acc, lane);
            v = add_other_half(v);
            if ((lane & 35) == 0) part[wave][r + ((lane >> 2) & 7)] = v;
        }
    }
    __syncthreads();
    if (threadIdx.x < ROWS) {
        const int c = threadIdx.x;
        float sum = 0.0f;
        bool first = true;
        for (int i = 0; i < a.k; ++i) {
            if (a.plan_ptr[e0 + i] == 0ull) continue;
            const float p = __fmul_rn(part[i][c], a.plan_w[e0 + i]);
            sum = first ? p : __fadd_rn(sum, p);
            first = false;
        }
        const size_t o = (size_t) blockIdx.y * n_embd + r0 + c;
        if (a.add && (!a.add_flag || *a.add_flag)) sum = __fadd_rn(sum, a.add[o]);
        if (a.add2) sum = __fadd_rn(sum, a.add2[o]);
        a.out[o] = sum;
        if (a.part)
            for (int i = 0; i < a.k; ++i)
                if (a.plan_ptr[e0 + i] != 0ull) a.part[(size_t) (e0 + i) * n_embd + r0 + c] = part[i][c];
    }
}

// ---------------------------------------------------------------------------------------------------- IQ1_M
// A lane's share of one quad of rows: 14 registers
struct QuadIQ1M {
    u32x4 i4;        // the four index bytes of rows 0..3
    u32x2 qh;        // four qh halfwords
    u32x4 sc01, sc23;  // (block scale | 48 bits of 3-bit scales) of rows 0,1 and 2,3
};
struct QuadOffsM {
    uint32_t i4, qh, d;
};
template <int NU>
__device__ __forceinline__ QuadOffsM quad_offsm(uint32_t mat_off, int u) {
    return QuadOffsM{mat_off + 16u * u, mat_off + 16u * NU + 8u * u, mat_off + 24u * NU + 32u * (u >> 3)};
}
__device__ __forceinline__ QuadIQ1M load_quadm(__amdgpu_buffer_rsrc_t rs, const QuadOffsM& o, uint32_t quad_off) {
    QuadIQ1M q;
    q.i4 = __builtin_amdgcn_raw_buffer_load_b128(rs, o.i4, quad_off, 0);
    q.qh = __builtin_amdgcn_raw_buffer_load_b64(rs, o.qh, quad_off, 0);
    q.sc01 = __builtin_amdgcn_raw_buffer_load_b128(rs, o.d, quad_off, 0);
    q.sc23 = __builtin_amdgcn_raw_buffer_load_b128(rs, o.d + 16u, quad_off, 0);
    return q;
}
// row R of the quad against the lane's activation codes; sy8[l] = the sum of the 8 codes of group l, sh = 16 + 6 x the
// lane's sub-block inside its block (where its pair of 3-bit scales sits)
template <int R>
__device__ __forceinline__ float unitm_value(const QuadIQ1M& q, const uint2* grid, const int (&y)[8], const int (&sy8)[4], int sh,
                                             float dy8) {
    const uint32_t i4 = q.i4[R];
    const uint32_t hw = R < 2 ? q.qh.x : q.qh.y;
    const uint32_t qh = (R & 1) ? (hw >> 16) : (hw & 0xffffu);
    const u32x4 sw = R < 2 ? q.sc01 : q.sc23;
    const uint32_t s_lo = (R & 1) ? sw.z : sw.x, s_hi = (R & 1) ? sw.w : sw.y;
    const uint32_t sc = (uint32_t) ((((uint64_t) s_hi << 32) | (uint64_t) s_lo) >> sh);
    int t[2] = {0, 0};
#pragma unroll
    for (int l = 0; l < 4; ++l) {
        const uint32_t nib = (qh >> (4 * l)) & 15u;
        const uint2 g = grid[((i4 >> (8 * l)) & 255u) | ((nib & 7u) << 8)];
        t[l >> 1] = dot4((int) g.x, y[2 * l], t[l >> 1]);
        t[l >> 1] = dot4((int) g.y, y[2 * l + 1], t[l >> 1]);
        t[l >> 1] += __mul24((nib & 8u) ? -10 : -8, sy8[l]);
    }
    const int isum = __mul24(2 * (int) (sc & 7u) + 1, t[0]) + __mul24(2 * (int) ((sc >> 3) & 7u) + 1, t[1]);
    return __fmul_rn(__fmul_rn(f16_bits_to_f32(s_lo & 0xffffu), dy8), (float) isum);
}
template <int B>
__device__ __forceinline__ void quadm_values(const QuadIQ1M& q, const uint2* grid, const int (&y)[8], const int (&sy8)[4], int sh,
                                             float dy8, float (&acc)[8]) {
#define MAYA_ROW(R)                                              \
    acc[B + R] = unitm_value<R>(q, grid, y, sy8, sh, dy8);       \
    asm volatile("" : "+v"(acc[B + R]));                         \
    __builtin_amdgcn_sched_barrier(0);
    MAYA_ROW(0) MAYA_ROW(1) MAYA_ROW(2) MAYA_ROW(3)
#undef MAYA_ROW
}
__device__ __forceinline__ void sums8_codes(const int (&y)[8], int (&sy8)[4]) {
#pragma unroll
    for (int l = 0; l < 4; ++l) sy8[l] = dot4(0x01010101, y[2 * l], dot4(0x01010101, y[2 * l + 1], 0));
}

// ---- gate/up, n_embd = 1024 NW: a workgroup of NW waves = the 2 * 32 NW sub-block positions of a (gate row, up row) pair;
// grid (n_ff / ROWS, entries); entry e = token e / k, slot e % k.  Rows in batches of 8 (two quads), a quad ahead.
template <int NW, int ROWS, int MINW>
__global__ __launch_bounds__(64 * NW, MINW) void gate_up_iq1m_pos_kernel(maya_moe_args a, Codebooks cb) {
    static_assert(ROWS % 8 == 0, "a batch is two quads");
    constexpr int NU = 32 * NW;
    __shared__ __align__(16) int lds[kFast1LdsWords];
    __shared__ float part[2][2 * NW][8];
    if (a.skip && *a.skip) return;
    const int e = blockIdx.y;
    const uint64_t blob = a.plan_ptr[e];
    if (blob == 0ull) return;
    stage_iq1s_table<64 * NW>(lds, cb);
    const uint2* grid = (const uint2*) lds;
    const int t = threadIdx.x, lane = t & 63, hw = t >> 5;
    const bool is_up = t >= NU;
    const int u = is_up ? t - NU : t;
    const int tok = e / a.k;
    int y[8];
    {
        const int4* q = (const int4*) (a.x.q + (size_t) tok * (32 * NU));
        const int4 ya = q[2 * u], yb = q[2 * u + 1];
        y[0] = ya.x, y[1] = ya.y, y[2] = ya.z, y[3] = ya.w, y[4] = yb.x, y[5] = yb.y, y[6] = yb.z, y[7] = yb.w;
    }
    int sy8[4];
    sums8_codes(y, sy8);
    const int sh = 16 + 6 * (u & 7);
    const float dy8 = a.x.d[(size_t) tok * NU + u] * 0.125f;
    constexpr uint32_t qb = NU / 8 * 56 * 4;  // bytes of a quad of rows
    const int n_ff = a.layout.n_ff, r0 = blockIdx.x * ROWS;
    const __amdgpu_buffer_rsrc_t rs = weight_rsrc(blob + a.layout.gate_off, (uint32_t) (a.layout.down_off - a.layout.gate_off));
    const QuadOffsM qo = quad_offsm<NU>(is_up ? (uint32_t) (a.layout.up_off - a.layout.gate_off) : 0u, u);
    const uint32_t quad0 = (uint32_t) (r0 >> 2) * qb;
    constexpr int NQ = ROWS / 4;
    QuadIQ1M nxt = load_quadm(rs, qo, quad0);
    __syncthreads();
    float acc[8];
#pragma unroll 1
    for (int r = 0; r < ROWS; r += 8) {
        const int q = r >> 2;
        {
            const QuadIQ1M cur = nxt;
            nxt = load_quadm(rs, qo, quad0 + (uint32_t) (q + 1) * qb);
            quadm_values<0>(cur, grid, y, sy8, sh, dy8, acc);
        }
        {
            const QuadIQ1M cur = nxt;
            if (q + 2 < NQ) nxt = load_quadm(rs, qo, quad0 + (uint32_t) (q + 2) * qb);
            quadm_values<4>(cur, grid, y, sy8, sh, dy8, acc);
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

// ---- down + combine, n_ff = 2048 (64 sub-blocks a row = one wave): wave w = slot w of token blockIdx.y, rows in batches
// of 8; grid (n_embd / ROWS, tokens).  Without a rounded h (hq.q == NULL) a wave rounds its slot's h to Q8_K itself.  The
// slots' rows meet in LDS and are summed in slot order.
template <int ROWS, int MINW, int NU = 64>
__global__ __launch_bounds__(512, MINW) void down_iq1m_pos_kernel(maya_moe_args a, Codebooks cb) {
    static_assert(ROWS % 8 == 0, "a batch is two quads");
    static_assert(NU % 8 == 0 && NU >= 8 && NU <= 64, "whole 256-value blocks on one wave");
    __shared__ __align__(16) int lds[kFast1LdsWords];
    __shared__ float part[8][ROWS];
    if (a.skip && *a.skip) return;
    stage_iq1s_table<512>(lds, cb);
    const uint2* grid = (const uint2*) lds;
    const int n_embd = a.layout.n_embd;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r0 = blockIdx.x * ROWS;
    const int e0 = blockIdx.y * a.k, ent = e0 + wave;
    const uint64_t blob = wave < a.k ? a.plan_ptr[ent] : 0ull;
    __syncthreads();
    if (blob != 0ull) {
        constexpr uint32_t qb = NU / 8 * 56 * 4;
        const uint64_t mat = blob + a.layout.down_off;
        const uint32_t mat_lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) mat);
        const uint32_t mat_hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (mat >> 32));
        const __amdgpu_buffer_rsrc_t rs = weight_rsrc(((uint64_t) mat_hi << 32) | (uint64_t) mat_lo, (uint32_t) (n_embd >> 2) * qb);
        // (an idle lane - past the row's NU positions - reads the last position's weights again and meets them with zero
        // activations)
        const bool on = NU == 64 || lane < NU;
        const int pos = on ? lane : NU - 1;
        const QuadOffsM qo = quad_offsm<NU>(0u, pos);
        const uint32_t quad0 = (uint32_t) (r0 >> 2) * qb;
        constexpr int NQ = ROWS / 4;
        QuadIQ1M nxt = load_quadm(rs, qo, quad0);
        int y[8];
        float dy8;
        if (a.hq.q) {
            const int4* q = (const int4*) (a.hq.q + (size_t) ent * (32 * NU));
            const int4 ya = q[2 * pos], yb = q[2 * pos + 1];
            y[0] = ya.x, y[1] = ya.y, y[2] = ya.z, y[3] = ya.w, y[4] = yb.x, y[5] = yb.y, y[6] = yb.z, y[7] = yb.w;
            dy8 = a.hq.d[(size_t) ent * NU + pos] * 0.125f;
        } else {
            const float4* hv = (const float4*) (a.h + (size_t) ent * (32 * NU) + 32 * pos);
            float v[32];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float4 t = hv[i];
                v[4 * i] = t.x, v[4 * i + 1] = t.y, v[4 * i + 2] = t.z, v[4 * i + 3] = t.w;
            }
            if (!on) {
#pragma unroll
                for (int i = 0; i < 32; ++i) v[i] = 0.0f;
            }
            float d;
            q8k_round_lane32(v, [&](int i) { return 32 * (lane & 7) + i; }, y, d);
            dy8 = d * 0.125f;
        }
        if (!on) {
#pragma unroll
            for (int i = 0; i < 8; ++i) y[i] = 0;
            dy8 = 0.0f;
        }
        int sy8[4];
        sums8_codes(y, sy8);
        const int sh = 16 + 6 * (lane & 7);
        float acc[8];
#pragma unroll 1
        for (int r = 0; r < ROWS; r += 8) {
            const int q = r >> 2;
            {
                const QuadIQ1M cur = nxt;
                nxt = load_quadm(rs, qo, quad0 + (uint32_t) (q + 1) * qb);
                quadm_values<0>(cur, grid, y, sy8, sh, dy8, acc);
            }
            {
                const QuadIQ1M cur = nxt;
                if (q + 2 < NQ) nxt = load_quadm(rs, qo, quad0 + (uint32_t) (q + 2) * qb);
                quadm_values<4>(cur, grid, y, sy8, sh, dy8, acc);
            }
            float v = reduce8_half(acc, lane);
            v = add_other_half(v);
            if ((lane & 35) == 0) part[wave][r + ((lane >> 2) & 7)] = v;
        }
    }
    __syncthreads();
    if (threadIdx.x < ROWS) {
        const int c = threadIdx.x;
        float sum = 0.0f;
        bool first = true;
        for (int i = 0; i < a.k; ++i) {
            if (a.plan_ptr[e0 + i] == 0ull) continue;
            const float p = __fmul_rn(part[i][c], a.plan_w[e0 + i]);
            sum = first ? p : __fadd_rn(sum, p);
            first = false;
        }
        const size_t o = (size_t) blockIdx.y * n_embd + r0 + c;
        if (a.add && (!a.add_flag || *a.add_flag)) sum = __fadd_rn(sum, a.add[o]);
        if (a.add2) sum = __fadd_rn(sum, a.add2[o]);
        a.out[o] = sum;
        if (a.part)
            for (int i = 0; i < a.k; ++i)
                if (a.plan_ptr[e0 + i] != 0ull) a.part[(size_t) (e0 + i) * n_embd + r0 + c] = part[i][c];
    }
}

}  // namespace maya
