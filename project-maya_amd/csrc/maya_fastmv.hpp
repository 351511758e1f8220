// maya_fastmv.hpp - dense mat-vec jobs on the position-mapped skeleton of the expert kernels: a workgroup of NW waves =
// the 2 * 32 NW positions of a pair of adjacent rows (2 p on the first half of the lanes, 2 p + 1 on the second) of
// n_in = 1024 NW values; a lane keeps its position, so a column's 32 activation codes stay in registers while the lane
// walks down the rows, and a row pair is read in whole contiguous runs.  Q8_0 rows in the stream packing (codes, then
// scales) for up to 8 columns a read of the weights, Q4_K rows (16-byte aligned) one column at a time.
// y[c][r] = alpha * (W_r . x[c]) + bias[r], each operation rounded (glmf::mv, include/strata/kernels/glm_fast.hpp:23-55).
#pragma once

namespace maya {

struct MvPos {
    const uint8_t* w;
    maya_act x;
    const float* bias;
    float* y;
    long long y_stride;
    float alpha;
    int n_out, ncol;
};
__device__ __forceinline__ void mv_store(const MvPos& j, int c, int r, float dot) {
    float v = __fmul_rn(j.alpha, dot);
    if (j.bias) v = __fadd_rn(v, j.bias[r]);
    j.y[(size_t) c * j.y_stride + r] = v;
}

// grid (n_out / (2 ROWS)); a step takes 8 / NT row pairs for NT columns
template <int NW, int NT, int ROWS>
__global__ __launch_bounds__(64 * NW) void mv_q80_pos_kernel(MvPos j) {
    constexpr int NU = 32 * NW, R = 8 / NT, k = 32 * NU;
    static_assert(ROWS % R == 0, "whole steps");
    __shared__ float part[2][2 * NW][8];
    const int t = threadIdx.x, lane = t & 63, hw = t >> 5;
    const bool second = t >= NU;
    const int u = second ? t - NU : t;
    const int p0 = blockIdx.x * ROWS;   // the first row pair
    constexpr uint32_t rb = NU * 34;    // bytes of a row
    const __amdgpu_buffer_rsrc_t rs = weight_rsrc((uint64_t) j.w, (uint32_t) j.n_out * rb);
    const uint32_t mat = second ? rb : 0u;
    const uint32_t oq = mat + 32u * u, od = mat + 32u * NU + 2u * u;
    int step = 0;
    for (int c0 = 0; c0 < j.ncol; c0 += NT) {
        int y[NT][8];
        float dx[NT];
#pragma unroll
        for (int c = 0; c < NT; ++c) {
            if (c0 + c < j.ncol) {
                const int4* q = (const int4*) (j.x.q + (size_t) (c0 + c) * k);
                const int4 ya = q[2 * u], yb = q[2 * u + 1];
                y[c][0] = ya.x, y[c][1] = ya.y, y[c][2] = ya.z, y[c][3] = ya.w;
                y[c][4] = yb.x, y[c][5] = yb.y, y[c][6] = yb.z, y[c][7] = yb.w;
                dx[c] = j.x.d[(size_t) (c0 + c) * NU + u];
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) y[c][i] = 0;
                dx[c] = 0.0f;
            }
        }
        for (int r = 0; r < ROWS; r += R, ++step) {
            float acc[8];
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                const uint32_t ro = (uint32_t) (p0 + r + rr) * (2u * rb);
                const u32x4 qa = __builtin_amdgcn_raw_buffer_load_b128(rs, oq, ro, 0);
                const u32x4 qb = __builtin_amdgcn_raw_buffer_load_b128(rs, oq + 16u, ro, 0);
                const uint32_t db = __builtin_amdgcn_raw_buffer_load_b16(rs, od, ro, 0);
                q80_values<NT>(qa, qb, db, y, dx, acc, rr * NT);
            }
            const float v = reduce8_half(acc, lane);
            const int buf = step & 1;
            if ((lane & 3) == 0) part[buf][hw][(lane >> 2) & 7] = v;
            __syncthreads();
            if (t < 16) {
                const int i = t & 7, half = t >> 3;
                float s = part[buf][half * NW][i];
#pragma unroll
                for (int w = 1; w < NW; ++w) s += part[buf][half * NW + w][i];
                const int rr = i / NT, c = i % NT;
                if (c0 + c < j.ncol) mv_store(j, c0 + c, 2 * (p0 + r + rr) + half, s);
            }
        }
    }
}

// grid (n_out / (2 ROWS), columns); rows in batches of 8 pairs, one pair ahead in registers
template <int NW, int ROWS>
__global__ __launch_bounds__(64 * NW, 8) void mv_q4k_pos_kernel(MvPos j) {
    static_assert(ROWS % 8 == 0, "row pairs come in batches of 8");
    constexpr int NU = 32 * NW;
    __shared__ float part[2][2 * NW][8];
    const int t = threadIdx.x, lane = t & 63, hw = t >> 5;
    const bool second = t >= NU;
    const int u = second ? t - NU : t;
    const int c = blockIdx.y;
    constexpr uint32_t rb = NU / 8 * 144;   // bytes of a row
    PosQ4K p;
    pos_q4k_init(p, u, second ? rb : 0u);
    pos_q4k_codes(p, u, j.x.q + (size_t) c * (32 * NU), j.x.d + (size_t) c * NU, j.x.bsums + (size_t) c * (2 * NU));
    const int p0 = blockIdx.x * ROWS;
    const __amdgpu_buffer_rsrc_t rs = weight_rsrc((uint64_t) j.w, (uint32_t) j.n_out * rb);
    u32x4 hn = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_hdr, (uint32_t) p0 * (2u * rb), 0);
    u32x4 qn = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_q, (uint32_t) p0 * (2u * rb), 0);
    float acc[8];
#pragma unroll 1
    for (int r = 0; r < ROWS; r += 8) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const u32x4 hc = hn, qc = qn;
            if (r + i + 1 < ROWS) {
                hn = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_hdr, (uint32_t) (p0 + r + i + 1) * (2u * rb), 0);
                qn = __builtin_amdgcn_raw_buffer_load_b128(rs, p.o_q, (uint32_t) (p0 + r + i + 1) * (2u * rb), 0);
            }
            acc[i] = pos_q4k_value(p, hc, qc);
            asm volatile("" : "+v"(acc[i]));
        }
        const float v = reduce8_half(acc, lane);
        const int buf = (r >> 3) & 1;
        if ((lane & 3) == 0) part[buf][hw][(lane >> 2) & 7] = v;
        __syncthreads();
        if (t < 16) {
            const int i = t & 7, half = t >> 3;
            float s = part[buf][half * NW][i];
#pragma unroll
            for (int w = 1; w < NW; ++w) s += part[buf][half * NW + w][i];
            mv_store(j, c, 2 * (p0 + r + i) + half, s);
        }
    }
}

}  // namespace maya
