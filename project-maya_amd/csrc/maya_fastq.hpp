// maya_fastq.hpp - position-mapped kernels for Q8_0 rows in the stream packing (a row = its k codes, then its k / 32 FP16
// scales: aligned 16-byte loads; the GGUF order interleaves a 2-byte scale with every 32 codes).  Made for the expert
// every token takes (a shared expert, a dense FFN): the tokens of a group share one read of the weights.  A lane owns
// one 32-value block position; the batch of a step is 8 (row, token) values - 8 / NT rows of NT tokens - so one
// transposing butterfly reduces a step whatever NT is.
#pragma once

namespace maya {

// the group's entries c0 .. c0 + NT - 1 (-1 past its end) and their tokens' codes / scales at block position u
template <int NT>
__device__ __forceinline__ void q80_chunk(const maya_moe_args& a, const GroupRef& gr, int c0, const maya_act& x, bool by_token,
                                          int k, int u, int (&ents)[NT], int (&y)[NT][8], float (&dx)[NT]) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        ents[t] = c0 + t < gr.ne ? entry_of(a, gr, c0 + t) : -1;
        if (ents[t] >= 0) {
            const int row = by_token ? ents[t] / a.k : ents[t];
            const int4* q = (const int4*) (x.q + (size_t) row * k);
            const int4 ya = q[2 * u], yb = q[2 * u + 1];
            y[t][0] = ya.x, y[t][1] = ya.y, y[t][2] = ya.z, y[t][3] = ya.w;
            y[t][4] = yb.x, y[t][5] = yb.y, y[t][6] = yb.z, y[t][7] = yb.w;
            dx[t] = x.d[(size_t) row * (k >> 5) + u];
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) y[t][i] = 0;
            dx[t] = 0.0f;
        }
    }
}
// one row's block at this position against NT tokens: acc[base + t] = d_w d_x[t] * (codes . y[t])
template <int NT>
__device__ __forceinline__ void q80_values(const u32x4 qa, const u32x4 qb, uint32_t dbits, const int (&y)[NT][8],
                                           const float (&dx)[NT], float (&acc)[8], int base) {
    const float dw = f16_bits_to_f32((uint16_t) dbits);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        int s = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            s = dot4((int) qa[i], y[t][i], s);
            s = dot4((int) qb[i], y[t][4 + i], s);
        }
        acc[base + t] = __fmul_rn(__fmul_rn(dw, dx[t]), (float) s);
    }
}

// ---- gate/up: a workgroup of NW waves = the 2 * 32 NW block positions of a (gate row, up row) pair of n_embd = 1024 NW
// values; grid (n_ff / ROWS, groups).  A step takes 8 / NT row pairs for NT tokens.
template <int NW, int NT, int ROWS>
__global__ __launch_bounds__(64 * NW) void gate_up_q80_pos_kernel(maya_moe_args a) {
    constexpr int NU = 32 * NW, R = 8 / NT;
    static_assert(ROWS % R == 0, "whole steps");
    __shared__ float part[2][2 * NW][8];
    GroupRef gr;
    if (!group_of(a, blockIdx.y, gr)) return;
    const int t = threadIdx.x, lane = t & 63, hw = t >> 5;
    const bool is_up = t >= NU;
    const int u = is_up ? t - NU : t;
    const int k = 32 * NU, n_ff = a.layout.n_ff, r0 = blockIdx.x * ROWS;
    constexpr uint32_t rb = NU * 34;   // bytes of a row
    const __amdgpu_buffer_rsrc_t rs = weight_rsrc(gr.blob + a.layout.gate_off, (uint32_t) (a.layout.down_off - a.layout.gate_off));
    const uint32_t mat = is_up ? (uint32_t) (a.layout.up_off - a.layout.gate_off) : 0u;
    const uint32_t oq = mat + 32u * u, od = mat + 32u * NU + 2u * u;
    int step = 0;
    for (int c0 = 0; c0 < gr.ne; c0 += NT) {
        int ents[NT], y[NT][8];
        float dx[NT];
        q80_chunk<NT>(a, gr, c0, a.x, true, k, u, ents, y, dx);
        for (int r = 0; r < ROWS; r += R, ++step) {
            float acc[8];
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                const uint32_t ro = (uint32_t) (r0 + r + rr) * rb;
                const u32x4 qa = __builtin_amdgcn_raw_buffer_load_b128(rs, oq, ro, 0);
                const u32x4 qb = __builtin_amdgcn_raw_buffer_load_b128(rs, oq + 16u, ro, 0);
                const uint32_t db = __builtin_amdgcn_raw_buffer_load_b16(rs, od, ro, 0);
                q80_values<NT>(qa, qb, db, y, dx, acc, rr * NT);
            }
            const float v = reduce8_half(acc, lane);
            const int buf = step & 1;
            if ((lane & 3) == 0) part[buf][hw][(lane >> 2) & 7] = v;
            __syncthreads();
            if (t < 8) {
                float g = part[buf][0][t], up = part[buf][NW][t];
#pragma unroll
                for (int w = 1; w < NW; ++w) {
                    g += part[buf][w][t];
                    up += part[buf][NW + w][t];
                }
                const int rr = t / NT, tk = t % NT;
                if (ents[tk] >= 0 && r0 + r + rr < n_ff) a.h[(size_t) ents[tk] * n_ff + r0 + r + rr] = swiglu(g, up, a.limit);
            }
        }
    }
}

// ---- down, n_ff = 32 NU <= 2048 (NU block positions a row on the first NU lanes of one wave, the lanes past it idle):
// every wave takes its own rows (wg_rows / 8 of them), a step 8 / NT rows for NT entries of the group; writes
// part[entry][row]; grid (n_embd / wg_rows, groups)
template <int NT, int NU = 64>
__global__ __launch_bounds__(512) void down_q80_pos_kernel(maya_moe_args a, int wg_rows) {
    constexpr int R = 8 / NT;
    static_assert(NU % 8 == 0 && NU >= 8 && NU <= 64, "a row on one wave");
    GroupRef gr;
    if (!group_of(a, blockIdx.y, gr)) return;
    const int wave = threadIdx.x >> 6, lane0 = threadIdx.x & 63;
    // (an idle lane reads the last position's weights again and meets them with zero activations)
    const bool on = NU == 64 || lane0 < NU;
    const int lane = on ? lane0 : NU - 1;
    const int n_embd = a.layout.n_embd, k = 32 * NU;
    const int per_wave = wg_rows >> 3, r0 = blockIdx.x * wg_rows + wave * per_wave;
    constexpr uint32_t rb = NU * 34;
    const uint64_t mat = gr.blob + a.layout.down_off;
    const __amdgpu_buffer_rsrc_t rs = weight_rsrc(mat, (uint32_t) n_embd * rb);
    const uint32_t oq = 32u * lane, od = 32u * NU + 2u * lane;
    for (int c0 = 0; c0 < gr.ne; c0 += NT) {
        int ents[NT], y[NT][8];
        float dx[NT];
        q80_chunk<NT>(a, gr, c0, a.hq, false, k, lane, ents, y, dx);
        if (!on) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
#pragma unroll
                for (int i = 0; i < 8; ++i) y[t][i] = 0;
                dx[t] = 0.0f;
            }
        }
        for (int r = 0; r < per_wave; r += R) {
            float acc[8];
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                // (the wave's row offset is uniform, but only readfirstlane tells the compiler so)
                const uint32_t ro = (uint32_t) __builtin_amdgcn_readfirstlane(r0 + r + rr) * rb;
                const u32x4 qa = __builtin_amdgcn_raw_buffer_load_b128(rs, oq, ro, 0);
                const u32x4 qb = __builtin_amdgcn_raw_buffer_load_b128(rs, oq + 16u, ro, 0);
                const uint32_t db = __builtin_amdgcn_raw_buffer_load_b16(rs, od, ro, 0);
                q80_values<NT>(qa, qb, db, y, dx, acc, rr * NT);
            }
            float v = reduce8_half(acc, lane0);
            v = add_other_half(v);
            if ((lane0 & 35) == 0) {
                const int i = (lane0 >> 2) & 7, rr = i / NT, tk = i % NT;
                if (ents[tk] >= 0 && r0 + r + rr < n_embd) a.part[(size_t) ents[tk] * n_embd + r0 + r + rr] = v;
            }
        }
    }
}

}  // namespace maya
