// maya_fastk.hpp - position-mapped decode kernels for Q4_K rows in their own GGUF order (blobs 16-byte aligned): the same
// skeleton as the IQ2_S ones.  A lane owns one 16-byte piece of every block's codes - the low nibbles are 16 values of
// sub-block 2j, the high nibbles 16 values of sub-block 2j + 1 - so its 32 activation codes, their two sums and the
// block's activation scale stay in registers while it walks down the rows; 8 lanes read a block's 128 code bytes as one
// contiguous run and all 8 the block's 16-byte header.  The format is cheap to decode (about 45 vector operations for 18
// bytes), so these kernels are bound by the weight stream.
#pragma once

namespace maya {

// the lane's fixed part: activation codes (low-nibble values, then high-nibble values), their sums, the scale
struct PosQ4K {
    int ylo[4], yhi[4];
    int slo, shi;
    float dx;
    uint32_t o_hdr, o_q;   // byte offsets of the block header and of the lane's piece inside a row
    int sh;                // bit offset of the lane's two sub-blocks' scale bytes in their packed word
    int wsel;              // which packed word (sub-blocks 0-3 or 4-7)
};
// position u of a row: block u >> 3, piece u & 7 (sub-block pair j = piece >> 1, half = piece & 1)
__device__ __forceinline__ void pos_q4k_init(PosQ4K& p, int u, uint32_t mat_off) {
    const int b = u >> 3, piece = u & 7, j = piece >> 1;
    p.o_hdr = mat_off + 144u * b;
    p.o_q = p.o_hdr + 16u + 16u * piece;
    p.wsel = j >> 1;
    p.sh = 16 * (j & 1);
}
__device__ __forceinline__ void pos_q4k_codes(PosQ4K& p, int u, const int8_t* q, const float* d, const int16_t* bsums) {
    const int b = u >> 3, piece = u & 7, j = piece >> 1, half = piece & 1;
    const int v0 = 256 * b + 64 * j + 16 * half;
    const int4 lo = *(const int4*) (q + v0), hi = *(const int4*) (q + v0 + 32);
    p.ylo[0] = lo.x, p.ylo[1] = lo.y, p.ylo[2] = lo.z, p.ylo[3] = lo.w;
    p.yhi[0] = hi.x, p.yhi[1] = hi.y, p.yhi[2] = hi.z, p.yhi[3] = hi.w;
    p.dx = d[v0 >> 5];
    if (bsums) {
        p.slo = bsums[v0 >> 4];
        p.shi = bsums[(v0 + 32) >> 4];
    } else {
        p.slo = dot4(0x01010101, p.ylo[0], dot4(0x01010101, p.ylo[1], dot4(0x01010101, p.ylo[2], dot4(0x01010101, p.ylo[3], 0))));
        p.shi = dot4(0x01010101, p.yhi[0], dot4(0x01010101, p.yhi[1], dot4(0x01010101, p.yhi[2], dot4(0x01010101, p.yhi[3], 0))));
    }
}
// one row's value at this position: dx (d (sc0 t0 + sc1 t1) - dmin (m0 s0 + m1 s1))
__device__ __forceinline__ float pos_q4k_value(const PosQ4K& p, const u32x4 hdr, const u32x4 q) {
    // the 6-bit scales / minimums of the lane's two sub-blocks (get_scale_min_k4: include/strata/artifact/dequant.hpp:162-172)
    const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
    const uint32_t scw = p.wsel ? ((s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u)) : (s0 & 0x3f3f3f3fu);
    const uint32_t mnw = p.wsel ? (((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u)) : (s1 & 0x3f3f3f3fu);
    const uint32_t sc2 = scw >> p.sh, mn2 = mnw >> p.sh;
    int t0 = 0, t1 = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        t0 = dot4((int) (q[i] & 0x0f0f0f0fu), p.ylo[i], t0);
        t1 = dot4((int) ((q[i] >> 4) & 0x0f0f0f0fu), p.yhi[i], t1);
    }
    const int is = __mul24((int) (sc2 & 0xffu), t0) + __mul24((int) ((sc2 >> 8) & 0xffu), t1);
    const int ms = __mul24((int) (mn2 & 0xffu), p.slo) + __mul24((int) ((mn2 >> 8) & 0xffu), p.shi);
    const float d = f16_bits_to_f32((uint16_t) (hdr.x & 0xffffu)), dmin = f16_bits_to_f32((uint16_t) (hdr.x >> 16));
    return __fmul_rn(p.dx, __fsub_rn(__fmul_rn(d, (float) is), __fmul_rn(dmin, (float) ms)));
}

// ---- gate/up: a workgroup of NW waves = the 2 * 32 NW positions of a (gate row, up row) pair of n_embd = 1024 NW values;
// grid (n_ff / ROWS, entries); entry e = token e / k, slot e % k.  Rows in batches of 8, one row ahead in registers.
// AHEAD (8 rows): all of a lane's rows are requested up front - the launches of a few entries, whose workgroups do not fill
// the chip and would otherwise run at the memory's latency a row.
// HEAD (one token): the layer's head rides in this launch (head_in_gate_up) - grid (n_ff / ROWS + 1, k).
template <int NW, int ROWS, int MINW, bool AHEAD = false, bool HEAD = false>
__global__ __launch_bounds__(64 * NW, MINW) void gate_up_q4k_pos_kernel(maya_moe_args a, LayerHeadIn hd) {
    static_assert(ROWS % 8 == 0, "rows come in batches of 8");
    static_assert(!AHEAD || ROWS == 8, "every row up front: one batch");
    constexpr int NU = 32 * NW;
    __shared__ float part[2][2 * NW][8];
    const int t = threadIdx.x, lane = t & 63, hw = t >> 5;
    const bool is_up = t >= NU;
    const int u = is_up ? t - NU : t;
    PosQ4K p;
    pos_q4k_init(p, u, is_up ? (uint32_t) (a.layout.up_off - a.layout.gate_off) : 0u);
    int e;
    uint64_t blob;
    if constexpr (HEAD) {
        // position u holds the block's values v0 .. v0 + 15 (against the low nibbles) and v0 + 32 .. v0 + 47 (the high ones)
        const int v0 = 256 * (u >> 3) + 64 * ((u & 7) >> 1) + 16 * (u & 1);
        int y[8];
        float d;
        e = (int) blockIdx.y;
        if (!head_in_gate_up<NW>(hd, a.k, a.skip, is_up, u, v0, v0 + 32, y, d, blob)) return;
#pragma unroll
        for (int i = 0; i < 4; ++i) p.ylo[i] = y[i], p.yhi[i] = y[4 + i];
        p.dx = d;
        p.slo = dot4(0x01010101, p.ylo[0], dot4(0x01010101, p.ylo[1], dot4(0x01010101, p.ylo[2], dot4(0x01010101, p.ylo[3], 0))));
        p.shi = dot4(0x01010101, p.yhi[0], dot4(0x01010101, p.yhi[1], dot4(0x01010101, p.yhi[2], dot4(0x01010101, p.yhi[3], 0))));
    } else {
        if (a.skip && *a.skip) return;
        // (a window's entries in the order of grp_ent where one is given: the entries of an expert side by side; -1 ends it)
        e = (a.grp_ent && !a.grp_ptr) ? a.grp_ent[blockIdx.y] : (int) blockIdx.y;
        if (e < 0) return;
        blob = a.plan_ptr[e];
        if (blob == 0ull) return;
        const int tok = e / a.k;
        pos_q4k_codes(p, u, a.x.q + (size_t) tok * (32 * NU), a.x.d + (size_t) tok * NU, a.x.bsums + (size_t) tok * (2 * NU));
    }
    constexpr uint32_t rb = NU / 8 * 144;   // bytes of a row
    const int n_ff = a.layout.n_ff, r0 = blockIdx.x * ROWS;
    const __amdgpu_buffer_rsrc_t rs = weight_rsrc(blob + a.layout.gate_off, (uint32_t) (a.layout.down_off - a.layout.gate_off));
    u32x4 hn = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_hdr, (uint32_t) r0 * rb, 0);
    u32x4 qn = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_q, (uint32_t) r0 * rb, 0);
    u32x4 ha[AHEAD ? ROWS : 1], qa[AHEAD ? ROWS : 1];
    if constexpr (AHEAD) {
        ha[0] = hn, qa[0] = qn;
#pragma unroll
        for (int i = 1; i < ROWS; ++i) {
            ha[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_hdr, (uint32_t) (r0 + i) * rb, 0);
            qa[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_q, (uint32_t) (r0 + i) * rb, 0);
        }
    }
    float acc[8];
#pragma unroll 1
    for (int r = 0; r < ROWS; r += 8) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if constexpr (AHEAD) {
                acc[i] = pos_q4k_value(p, ha[i], qa[i]);
            } else {
                const u32x4 hc = hn, qc = qn;
                if (r + i + 1 < ROWS) {
                    hn = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_hdr, (uint32_t) (r0 + r + i + 1) * rb, 0);
                    qn = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_q, (uint32_t) (r0 + r + i + 1) * rb, 0);
                }
                acc[i] = pos_q4k_value(p, hc, qc);
            }
            asm volatile("" : "+v"(acc[i]));
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

// ---- down + combine, n_ff = 32 NU <= 2048 (NU positions a row on the first NU lanes of one wave; NU a multiple of 8, the
// lanes past it idle): wave w = slot w of token blockIdx.y, rows in batches of 8; grid (n_embd / ROWS, tokens).  Without a
// rounded h (hq.q == NULL) a wave rounds its slot's h to Q8_K itself.
// AHEAD: all ROWS rows of the wave are requested before anything else is done (one or two slots on one token: a few
// hundred waves on the whole chip, each with one row in flight, run at the memory's latency a row).
template <int ROWS, int MINW, int NU = 64, bool AHEAD = false>
__global__ __launch_bounds__(512, MINW) void down_q4k_pos_kernel(maya_moe_args a) {
    static_assert(ROWS % 8 == 0, "rows come in batches of 8");
    static_assert(!AHEAD || ROWS == 8, "every row up front: one batch");
    static_assert(NU % 8 == 0 && NU >= 8 && NU <= 64, "whole 256-value blocks on one wave");
    __shared__ float part[8][ROWS];
    if (a.skip && *a.skip) return;
    const int n_embd = a.layout.n_embd;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int bx, by;
    down_block_of_grid(bx, by);
    const int r0 = bx * ROWS;
    const int e0 = by * a.k, ent = e0 + wave;
    const uint64_t blob = wave < a.k ? a.plan_ptr[ent] : 0ull;
    if (blob != 0ull) {
        // (an idle lane reads the last position's weights again and meets them with zero activations)
        const bool on = NU == 64 || lane < NU;
        const int pos = on ? lane : NU - 1;
        PosQ4K p;
        pos_q4k_init(p, pos, 0u);
        // the first row's weights are requested before h is rounded: their latency hides behind that arithmetic
        constexpr uint32_t rb = NU / 8 * 144;
        const uint64_t mat = blob + a.layout.down_off;
        const uint32_t mat_lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) mat);
        const uint32_t mat_hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (mat >> 32));
        const __amdgpu_buffer_rsrc_t rs = weight_rsrc(((uint64_t) mat_hi << 32) | (uint64_t) mat_lo, (uint32_t) n_embd * rb);
        u32x4 hn = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_hdr, (uint32_t) r0 * rb, 0);
        u32x4 qn = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_q, (uint32_t) r0 * rb, 0);
        u32x4 ha[AHEAD ? ROWS : 1], qa[AHEAD ? ROWS : 1];
        if constexpr (AHEAD) {
#pragma unroll
            for (int i = 1; i < ROWS; ++i) {
                ha[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_hdr, (uint32_t) (r0 + i) * rb, 0);
                qa[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_q, (uint32_t) (r0 + i) * rb, 0);
            }
        }
        if (a.hq.q) {
            pos_q4k_codes(p, pos, a.hq.q + (size_t) ent * (32 * NU), a.hq.d + (size_t) ent * NU, a.hq.bsums + (size_t) ent * (2 * NU));
        } else {
            // Q8_K of h in registers (quant_q8k_block's arithmetic): the lane's 32 values are two runs of 16, a block is
            // 8 lanes; the block's signed maximum is the value at the FIRST largest magnitude, so candidates carry their index
            const int piece = pos & 7, j = piece >> 1, half = piece & 1;
            const int v0 = 256 * (pos >> 3) + 64 * j + 16 * half;
            const float* hrow = a.h + (size_t) ent * (32 * NU);
            float v[32];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 lo = *(const float4*) (hrow + v0 + 4 * i), hi = *(const float4*) (hrow + v0 + 32 + 4 * i);
                v[4 * i] = lo.x, v[4 * i + 1] = lo.y, v[4 * i + 2] = lo.z, v[4 * i + 3] = lo.w;
                v[16 + 4 * i] = hi.x, v[16 + 4 * i + 1] = hi.y, v[16 + 4 * i + 2] = hi.z, v[16 + 4 * i + 3] = hi.w;
            }
            if (!on) {
#pragma unroll
                for (int i = 0; i < 32; ++i) v[i] = 0.0f;
            }
            int y[8];
            float d;
            q8k_round_lane32(v, [&](int i) { return 64 * j + 16 * half + (i < 16 ? i : i + 16); }, y, d);
#pragma unroll
            for (int i = 0; i < 4; ++i) p.ylo[i] = y[i], p.yhi[i] = y[4 + i];
            p.dx = d;
            p.slo = dot4(0x01010101, p.ylo[0], dot4(0x01010101, p.ylo[1], dot4(0x01010101, p.ylo[2], dot4(0x01010101, p.ylo[3], 0))));
            p.shi = dot4(0x01010101, p.yhi[0], dot4(0x01010101, p.yhi[1], dot4(0x01010101, p.yhi[2], dot4(0x01010101, p.yhi[3], 0))));
        }
        if (!on) {
#pragma unroll
            for (int i = 0; i < 4; ++i) p.ylo[i] = p.yhi[i] = 0;
            p.slo = p.shi = 0;
            p.dx = 0.0f;
        }
        float acc[8];
        if constexpr (AHEAD) {
            ha[0] = hn, qa[0] = qn;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                acc[i] = pos_q4k_value(p, ha[i], qa[i]);
                asm volatile("" : "+v"(acc[i]));
            }
            float v = reduce8_half(acc, lane);
            v = add_other_half(v);
            if ((lane & 35) == 0) part[wave][(lane >> 2) & 7] = v;
        } else
#pragma unroll 1
        for (int r = 0; r < ROWS; r += 8) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const u32x4 hc = hn, qc = qn;
                if (r + i + 1 < ROWS) {
                    hn = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_hdr, (uint32_t) (r0 + r + i + 1) * rb, 0);
                    qn = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_q, (uint32_t) (r0 + r + i + 1) * rb, 0);
                }
                acc[i] = pos_q4k_value(p, hc, qc);
                asm volatile("" : "+v"(acc[i]));
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
            const float pv = __fmul_rn(part[i][c], a.plan_w[e0 + i]);
            sum = first ? pv : __fadd_rn(sum, pv);
            first = false;
        }
        const size_t o = (size_t) by * n_embd + r0 + c;
        if (a.add && (!a.add_flag || *a.add_flag)) sum = __fadd_rn(sum, a.add[o]);
        if (a.add2) sum = __fadd_rn(sum, a.add2[o]);
        a.out[o] = sum;
        if (a.part)
            for (int i = 0; i < a.k; ++i)
                if (a.plan_ptr[e0 + i] != 0ull) a.part[(size_t) (e0 + i) * n_embd + r0 + c] = part[i][c];
    }
}

}  // namespace maya
