// maya_prefill.hip - a prompt chunk's routed experts on gfx950: the device-side plan (count, scan, stable scatter, tile
// list), the per-32 int8 activation quantizer over the plan's rows, and the grouped GEMM of Q4_K weights with those
// activations on the int8 matrix cores.
//
// The GEMM: a workgroup takes one tile (up to 64 rows of one expert) and a band of weight rows; its 4 waves take 4
// tiles of 16 weight rows each (gate/up: 2 tiles of gate rows and the same features' 2 tiles of up rows, so the SwiGLU
// and the requantization of H per 32 features stay inside the wave).  Per 32 values of the inner dimension one
// v_mfma_i32_16x16x32_i8 gives the exact integer dots of 16 tokens' codes with 16 weight rows' 4-bit codes; the F32
// scales (d * sc of the weight sub-block, the activation block's d) and the minimum's term (dmin * m times the
// activation block's s) are applied per output.  Weights stream from HBM straight into registers (each lane reads its own
// row), activations are staged through LDS a 256-value super-block at a time, double-buffered.
#include <hip/hip_runtime.h>

#include <math.h>
#include <stdint.h>

#include "maya_host.h"

namespace maya {

constexpr int kPfRows = 64;        // rows of a tile
constexpr int kPfMt = kPfRows / 16;
constexpr int kPfRowBytes = 272;   // a staged row of 256 codes: 4 banks' offset a row keeps the 8-byte reads apart
constexpr int kPlanThreads = 1024;
constexpr int kPlanWaves = kPlanThreads / 64;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------------------------------- the plan
// One workgroup: counts per expert and per segment (a wave's contiguous share of the entries), the prefix sums, then
// every wave walks its segment in order so that an expert's rows keep the entries' order.
// dynamic LDS: seg[kPlanWaves][n_expert] counts -> bases, base[n_expert + 1]
__global__ __launch_bounds__(kPlanThreads) void prefill_plan_kernel(const int32_t* __restrict__ ids, int n_entries,
                                                                    const uint64_t* __restrict__ table, int n_expert,
                                                                    maya_prefill_plan p, int max_tiles) {
    extern __shared__ int32_t sm[];
    int32_t* seg = sm;                               // [kPlanWaves][n_expert]
    int32_t* base = sm + kPlanWaves * n_expert;      // [n_expert + 1]
    __shared__ int32_t s_tiles;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    for (int i = tid; i < kPlanWaves * n_expert; i += kPlanThreads) seg[i] = 0;
    if (tid == 0) s_tiles = 0;
    __syncthreads();
    const int per = (((n_entries + kPlanWaves - 1) / kPlanWaves) + 63) & ~63;   // a wave's share, whole chunks of 64
    const int lo = wave * per, hi = min(n_entries, lo + per);
    auto expert_of = [&](int e) {
        const int x = ids[e];
        return (x >= 0 && x < n_expert && table[x] != 0ull) ? x : -1;
    };
    for (int e = lo + lane; e < hi; e += 64) {
        const int x = expert_of(e);
        if (x >= 0) atomicAdd(&seg[wave * n_expert + x], 1);
    }
    __syncthreads();
    // per expert: the segments' counts -> exclusive offsets, the total into base[x + 1]
    for (int x = tid; x < n_expert; x += kPlanThreads) {
        int run = 0;
        for (int w = 0; w < kPlanWaves; ++w) {
            const int c = seg[w * n_expert + x];
            seg[w * n_expert + x] = run;
            run += c;
        }
        base[x + 1] = run;
    }
    __syncthreads();
    if (tid == 0) {
        base[0] = 0;
        for (int x = 0; x < n_expert; ++x) base[x + 1] += base[x];
    }
    __syncthreads();
    for (int x = tid; x <= n_expert; x += kPlanThreads) p.bounds[x] = base[x];
    // tiles: expert x's rows in runs of kPfRows
    for (int x = tid; x < n_expert; x += kPlanThreads) {
        const int r0 = base[x], r1 = base[x + 1];
        const int nt = (r1 - r0 + kPfRows - 1) / kPfRows;
        if (nt > 0) {
            const int t0 = atomicAdd(&s_tiles, nt);
            for (int i = 0; i < nt && t0 + i < max_tiles; ++i) {
                p.tile_expert[t0 + i] = x;
                p.tile_row0[t0 + i] = r0 + i * kPfRows;
            }
        }
    }
    // the stable scatter: 64 entries a step, a lane's rank = the earlier lanes of the step with its expert
    for (int c0 = lo; c0 < hi; c0 += 64) {
        const int e = c0 + lane;
        const int x = e < hi ? expert_of(e) : -1;
        int rank = 0, cnt = 0;
        unsigned long long todo = __ballot(x >= 0);
        while (todo) {
            const int leader = __ffsll((long long) todo) - 1;
            const int lx = __shfl(x, leader, 64);
            const unsigned long long same = __ballot(x == lx);
            if (x == lx) {
                rank = __popcll(same & ((1ull << lane) - 1ull));
                cnt = __popcll(same);
            }
            todo &= ~same;
        }
        if (x >= 0) {
            const int row = base[x] + seg[wave * n_expert + x] + rank;
            p.row_entry[row] = e;
            p.entry_row[e] = row;
        } else if (e < hi) {
            p.entry_row[e] = -1;
        }
        __builtin_amdgcn_wave_barrier();
        if (x >= 0 && rank == cnt - 1) seg[wave * n_expert + x] += cnt;   // one lane an expert: no two write one word
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0);
    }
    __syncthreads();
    if (tid == 0) *p.n_tiles = min(s_tiles, max_tiles);
}

// ------------------------------------------------------------------------------------------ activation quantizer
template <int DT> __device__ __forceinline__ float pf_load(const void* x, int64_t i) {
    if constexpr (DT == MAYA_DT_F32) return ((const float*) x)[i];
    else if constexpr (DT == MAYA_DT_BF16) return __uint_as_float((uint32_t) ((const uint16_t*) x)[i] << 16);
    else return f16_bits_to_f32(((const uint16_t*) x)[i]);
}
__device__ __forceinline__ int pf_rint(float f) { return (int) rintf(f); }

// grid (k / 256, tokens): a token's block is rounded once and written to the rows of all its entries in the plan
template <int DT>
__global__ __launch_bounds__(256) void prefill_quant_kernel(const void* __restrict__ x, int64_t x_stride, maya_prefill_plan p,
                                                            int top_k, int64_t k, maya_prefill_act o) {
    const int t = blockIdx.y;
    const int64_t v = (int64_t) blockIdx.x * 256 + threadIdx.x;
    const float xv = pf_load<DT>(x, (int64_t) t * x_stride + v);
    float am = fabsf(xv);
#pragma unroll
    for (int s = 16; s > 0; s >>= 1) am = fmaxf(am, __shfl_xor(am, s, 64));
    const float inv = am > 0.0f ? __fdiv_rn(127.0f, am) : 0.0f;
    const int c = pf_rint(__fmul_rn(xv, inv));
    int sum = c;
#pragma unroll
    for (int s = 16; s > 0; s >>= 1) sum += __shfl_xor(sum, s, 64);
    const float d = __fdiv_rn(am, 127.0f), ds = __fmul_rn(d, (float) sum);
    for (int j = 0; j < top_k; ++j) {
        const int row = p.entry_row[t * top_k + j];
        if (row < 0) continue;   // an entry of an expert that is not resident
        o.q[(size_t) row * k + v] = (int8_t) c;
        if ((threadIdx.x & 31) == 0) {
            o.d[((size_t) row * k + v) >> 5] = d;
            o.s[((size_t) row * k + v) >> 5] = ds;
        }
    }
}

// ---------------------------------------------------------------------------------------------------- the GEMM
struct PfGemm {
    const uint64_t* table;
    maya_prefill_plan plan;
    uint64_t off[2];       // gate and up (gate/up), down and unused (down): byte offsets of the matrices in a blob
    int64_t k, n;          // inner length, weight rows of one matrix
    int64_t row_bytes;
    maya_prefill_act x;    // the tile rows' activations [rows][k]
    maya_prefill_act h;    // gate/up: the requantized H [rows][n]
    float* part;           // down: [rows][n]
    float limit;
};

struct PfStage {
    uint4 q[4];
    float4 sc;
};
// this thread's share of super-block sb of the tile's activations: 4 chunks of 16 codes, 4 scales (threads 0-127: d,
// 128-255: s)
__device__ __forceinline__ void pf_fetch(const PfGemm& a, int row0, int nrows, int sb, PfStage& st) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = tid + 256 * i, r = c >> 4, col = c & 15;
        st.q[i] = r < nrows ? *(const uint4*) (a.x.q + (size_t) (row0 + r) * a.k + (size_t) sb * 256 + col * 16) : make_uint4(0, 0, 0, 0);
    }
    const int r = (tid & 127) >> 1, half = tid & 1;
    const float* src = (tid < 128 ? a.x.d : a.x.s) + (size_t) (row0 + r) * (a.k >> 5) + sb * 8 + half * 4;
    st.sc = r < nrows ? *(const float4*) src : make_float4(0.f, 0.f, 0.f, 0.f);
}
// LDS of one buffer: codes [kPfRows][kPfRowBytes], d [8][kPfRows], s [8][kPfRows]
constexpr int kPfBufBytes = kPfRows * kPfRowBytes + 2 * 8 * kPfRows * 4;
__device__ __forceinline__ void pf_store(uint8_t* buf, const PfStage& st) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = tid + 256 * i, r = c >> 4, col = c & 15;
        *(uint4*) (buf + r * kPfRowBytes + col * 16) = st.q[i];
    }
    float* sc = (float*) (buf + kPfRows * kPfRowBytes) + (tid < 128 ? 0 : 8 * kPfRows);
    const int r = (tid & 127) >> 1, half = tid & 1;
    sc[(half * 4 + 0) * kPfRows + r] = st.sc.x;
    sc[(half * 4 + 1) * kPfRows + r] = st.sc.y;
    sc[(half * 4 + 2) * kPfRows + r] = st.sc.z;
    sc[(half * 4 + 3) * kPfRows + r] = st.sc.w;
}

// the 8 six-bit scales and 8 six-bit minimums of a Q4_K block's 12 bytes, as bytes of two words each
// (get_scale_min_k4, include/strata/artifact/dequant.hpp:162-172)
__device__ __forceinline__ void q4k_unpack_scales(uint32_t s0, uint32_t s1, uint32_t s2, uint32_t (&sc)[2], uint32_t (&mn)[2]) {
    sc[0] = s0 & 0x3f3f3f3fu;
    mn[0] = s1 & 0x3f3f3f3fu;
    sc[1] = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
    mn[1] = ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u);
}
__device__ __forceinline__ float byte_f32(uint32_t w, int i) { return (float) ((w >> (8 * i)) & 0xffu); }

__device__ __forceinline__ float pf_swiglu(float g, float u, float limit) {
    if (limit > 0.0f && limit < INFINITY) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
    }
    return __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, expf(-g))), u);
}

// one tile of NMT x 16 rows (the row count of the tile is a compile-time bound, so the inner loop is branch-free and
// the compiler can move the LDS reads of a step above the arithmetic of the one before)
template <bool GU, int NMT>
__device__ __forceinline__ void pf_tile(const PfGemm& a, uint8_t (*lds)[kPfBufBytes], int ex, int row0, int nrows) {
    const uint8_t* blob = (const uint8_t*) a.table[ex];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, ln = lane & 15, g = lane >> 4;

    // the 4 weight rows this lane feeds: gate/up: features f0 + ln and f0 + 16 + ln of gate, then of up
    const uint8_t* wrow[4];
    int64_t n0;   // the wave's first feature (gate/up) or output row (down)
    if constexpr (GU) {
        n0 = (int64_t) blockIdx.x * 128 + wave * 32;
#pragma unroll
        for (int t = 0; t < 4; ++t) wrow[t] = blob + a.off[t >> 1] + (size_t) (n0 + 16 * (t & 1) + ln) * a.row_bytes;
    } else {
        n0 = (int64_t) blockIdx.x * 256 + wave * 64;
#pragma unroll
        for (int t = 0; t < 4; ++t) wrow[t] = blob + a.off[0] + (size_t) (n0 + 16 * t + ln) * a.row_bytes;
    }
    const bool wave_on = n0 < a.n;   // (a.n is a multiple of the wave's rows: checked on the host)

    v4f acc[4][NMT];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int m = 0; m < NMT; ++m) acc[t][m] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    const int nsb = (int) (a.k >> 8);
    PfStage st;
    pf_fetch(a, row0, nrows, 0, st);
    pf_store(lds[0], st);
    // Weights run ahead of the arithmetic in registers.  Small tiles (1 or 2 groups of 16 rows) are bound by the weight
    // stream: they keep a whole super-block in flight, and everything a lane needs of a row's 144-byte block (the 16-byte
    // header and its four 8-byte slices of the codes) is requested in one burst, so the block's one or two cache lines are
    // fetched once, not once per slice at different times.
    // Tiles of 3 and 4 row groups have no registers to spare for a second block: their code slices run three slices
    // ahead in a ring of four register sets instead (slice j in set j) and the header a block ahead.
    constexpr bool kBurst = NMT <= 2;
    uint64_t q[4][4], qn[kBurst ? 4 : 1][4];     // [slice j][row tile t]
    uint32_t hdr[4][4], hdrn[kBurst ? 4 : 1][4];
    auto load_q = [&](int sb, int j, uint64_t (&dst)[4]) {
#pragma unroll
        for (int t = 0; t < 4; ++t) dst[t] = *(const uint64_t*) (wrow[t] + (size_t) sb * 144 + 16 + 32 * j + 8 * g);
    };
    auto load_h = [&](int sb, uint32_t (&dh)[4][4]) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint4 h = *(const uint4*) (wrow[t] + (size_t) sb * 144);
            dh[t][0] = h.x, dh[t][1] = h.y, dh[t][2] = h.z, dh[t][3] = h.w;
        }
    };
    auto load_block = [&](int sb, uint64_t (&dq)[4][4], uint32_t (&dh)[4][4]) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint8_t* blk = wrow[t] + (size_t) sb * 144;
            const uint4 h = *(const uint4*) blk;
            dh[t][0] = h.x, dh[t][1] = h.y, dh[t][2] = h.z, dh[t][3] = h.w;
#pragma unroll
            for (int j = 0; j < 4; ++j) dq[j][t] = *(const uint64_t*) (blk + 16 + 32 * j + 8 * g);
        }
    };
    if (wave_on) {
        if constexpr (kBurst) load_block(0, q, hdr);
        else {
            load_h(0, hdr);
            load_q(0, 0, q[0]);
            load_q(0, 1, q[1]);
            load_q(0, 2, q[2]);
        }
    }
    __syncthreads();
    for (int sb = 0; sb < nsb; ++sb) {
        const uint8_t* buf = lds[sb & 1];
        if (sb + 1 < nsb) pf_fetch(a, row0, nrows, sb + 1, st);
        if (wave_on) {
            float d[4], dmin[4];
            uint32_t sc[4][2], mn[4][2];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                d[t] = f16_bits_to_f32((uint16_t) (hdr[t][0] & 0xffffu));
                dmin[t] = f16_bits_to_f32((uint16_t) (hdr[t][0] >> 16));
                q4k_unpack_scales(hdr[t][1], hdr[t][2], hdr[t][3], sc[t], mn[t]);
            }
            if (sb + 1 < nsb) {
                if constexpr (kBurst) load_block(sb + 1, qn, hdrn);
                else load_h(sb + 1, hdr);   // (decoded above: its registers are free)
            }
            const float* sxl = (const float*) (buf + kPfRows * kPfRowBytes);
            const float* ssl = sxl + 8 * kPfRows;
            // the minimums' term, -(dmin m) . s over the 8 sub-blocks, on the matrix cores in F32: A = the tokens' s
            // (row = token, k = sub-block), B = this lane's row's -dmin m, accumulated straight into acc
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                float nb[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) nb[t] = -__fmul_rn(dmin[t], (float) ((mn[t][half] >> (8 * g)) & 0xffu));
#pragma unroll
                for (int m = 0; m < NMT; ++m) {
                    const float sa = ssl[(4 * half + g) * kPfRows + 16 * m + ln];
#pragma unroll
                    for (int t = 0; t < 4; ++t) acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x4f32(sa, nb[t], acc[t][m], 0, 0, 0);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (!kBurst) {   // slice (sb, j) + 3 into the set that slice (sb, j) - 1 has left
                    const int jn = (j + 3) & 3, sbn = sb + ((j + 3) >> 2);
                    if (sbn < nsb) load_q(sbn, jn, q[jn]);
                }
#pragma unroll
                for (int nib = 0; nib < 2; ++nib) {
                    const int blk = 2 * j + nib;
                    long wb[4];
                    float dsc[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        wb[t] = (long) ((q[j][t] >> (4 * nib)) & 0x0f0f0f0f0f0f0f0full);
                        // (the scale word is made opaque here: converted up front for all 8 sub-blocks, the 32 products
                        // would sit in registers for the whole super-block)
                        uint32_t scw = sc[t][blk >> 2];
                        asm volatile("" : "+v"(scw));
                        dsc[t] = __fmul_rn(d[t], byte_f32(scw, blk & 3));
                    }
#pragma unroll
                    for (int m = 0; m < NMT; ++m) {
                        const long xa = *(const long*) (buf + (16 * m + ln) * kPfRowBytes + blk * 32 + 8 * g);
                        const float4 sx = *(const float4*) (sxl + blk * kPfRows + 16 * m + 4 * g);
                        const float sxa[4] = {sx.x, sx.y, sx.z, sx.w};
                        v4i dot[4];
#pragma unroll
                        for (int t = 0; t < 4; ++t) dot[t] = __builtin_amdgcn_mfma_i32_16x16x32_i8(xa, wb[t], v4i{0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                acc[t][m][i] = fmaf(__fmul_rn(dsc[t], sxa[i]), (float) dot[t][i], acc[t][m][i]);
                            // (pinned: left free, the optimizer issues every dot of the super-block first and holds
                            // their 128 results in registers)
                            asm volatile("" : "+v"(acc[t][m]));
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);   // a sub-block's work stays together
                }
            }
            if constexpr (kBurst) {
                if (sb + 1 < nsb) {
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) hdr[t][i] = hdrn[t][i], q[i][t] = qn[i][t];
                    }
                }
            }
        }
        if (sb + 1 < nsb) pf_store(lds[(sb + 1) & 1], st);
        __syncthreads();
    }
    if (!wave_on) return;

    // outputs: lane (ln, g) holds weight row ln of each tile for the tokens 16 m + 4 g + i
#pragma unroll
    for (int m = 0; m < NMT; ++m) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = 16 * m + 4 * g + i;
            const bool on = r < nrows;
            if constexpr (GU) {
                // 32 features of one token: this lane's 2, the 16 lanes of its group
                const float h0 = pf_swiglu(acc[0][m][i], acc[2][m][i], a.limit);
                const float h1 = pf_swiglu(acc[1][m][i], acc[3][m][i], a.limit);
                float am = fmaxf(fabsf(h0), fabsf(h1));
#pragma unroll
                for (int s = 8; s > 0; s >>= 1) am = fmaxf(am, __shfl_xor(am, s, 64));
                const float inv = am > 0.0f ? __fdiv_rn(127.0f, am) : 0.0f;
                const int c0 = pf_rint(__fmul_rn(h0, inv)), c1 = pf_rint(__fmul_rn(h1, inv));
                int sum = c0 + c1;
#pragma unroll
                for (int s = 8; s > 0; s >>= 1) sum += __shfl_xor(sum, s, 64);
                if (on) {
                    int8_t* q = a.h.q + (size_t) (row0 + r) * a.n + n0;
                    q[ln] = (int8_t) c0;
                    q[16 + ln] = (int8_t) c1;
                    if (ln == 0) {
                        const float dd = __fdiv_rn(am, 127.0f);
                        const size_t b = ((size_t) (row0 + r) * a.n + n0) >> 5;
                        a.h.d[b] = dd;
                        a.h.s[b] = __fmul_rn(dd, (float) sum);
                    }
                }
            } else if (on) {
                float* o = a.part + (size_t) (row0 + r) * a.n + n0 + ln;
#pragma unroll
                for (int t = 0; t < 4; ++t) o[16 * t] = acc[t][m][i];
            }
        }
    }
}

// grid (bands of weight rows, tiles at most)
template <bool GU>
__global__ __launch_bounds__(256, 2) void prefill_q4k_kernel(PfGemm a) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2][kPfBufBytes];
    const int tile = blockIdx.y;
    if (tile >= *a.plan.n_tiles) return;
    const int ex = a.plan.tile_expert[tile], row0 = a.plan.tile_row0[tile];
    const int nrows = min(kPfRows, a.plan.bounds[ex + 1] - row0);
    switch ((nrows + 15) >> 4) {
        case 1: pf_tile<GU, 1>(a, lds, ex, row0, nrows); break;
        case 2: pf_tile<GU, 2>(a, lds, ex, row0, nrows); break;
        case 3: pf_tile<GU, 3>(a, lds, ex, row0, nrows); break;
        default: pf_tile<GU, 4>(a, lds, ex, row0, nrows); break;
    }
}

template <int ODT>
__global__ __launch_bounds__(256) void prefill_combine_kernel(const int32_t* __restrict__ entry_row, const float* __restrict__ w,
                                                              const float* __restrict__ part, int k, int64_t n,
                                                              const float* __restrict__ add, void* __restrict__ out) {
    const int t = blockIdx.y;
    const int64_t c = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (c >= n) return;
    float sum = 0.0f;
    bool first = true;
    for (int j = 0; j < k; ++j) {
        const int row = entry_row[t * k + j];
        if (row < 0) continue;
        const float v = __fmul_rn(part[(size_t) row * n + c], w[t * k + j]);
        sum = first ? v : __fadd_rn(sum, v);
        first = false;
    }
    if (add) sum = __fadd_rn(sum, add[(size_t) t * n + c]);
    if constexpr (ODT == MAYA_DT_F32) ((float*) out)[(size_t) t * n + c] = sum;
    else if constexpr (ODT == MAYA_DT_BF16) {
        uint32_t u = __float_as_uint(sum);
        if ((u & 0x7fffffffu) > 0x7f800000u) u |= 0x00400000u;          // NaN stays NaN
        else u += 0x7fffu + ((u >> 16) & 1u);                            // round to nearest even
        ((uint16_t*) out)[(size_t) t * n + c] = (uint16_t) (u >> 16);
    } else ((__half*) out)[(size_t) t * n + c] = __float2half_rn(sum);
}

static bool plan_ok(const maya_prefill_plan* p) {
    return p && p->bounds && p->row_entry && p->entry_row && p->tile_expert && p->tile_row0 && p->n_tiles;
}
static bool act_ok(const maya_prefill_act& a) { return a.q && a.d && a.s && ((uintptr_t) a.q & 15) == 0 && ((uintptr_t) a.d & 15) == 0 && ((uintptr_t) a.s & 15) == 0; }

}  // namespace maya

using namespace maya;

extern "C" {

int maya_moe_prefill_tile_rows(void) { return kPfRows; }
int maya_moe_prefill_max_tiles(int n_entries, int n_expert) {
    if (n_entries <= 0 || n_expert <= 0) return 0;
    return (n_entries + kPfRows - 1) / kPfRows + n_expert;
}
int maya_moe_prefill_supported(int type) { return type == kQ4_K ? 1 : 0; }

int maya_moe_prefill_plan(const int32_t* ids, int n_entries, const uint64_t* expert_table, int n_expert,
                          const maya_prefill_plan* plan, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!ids || !expert_table || !plan_ok(plan)) return fail(MAYA_E_ARG, "prefill_plan: null pointer");
    if (n_entries <= 0 || n_entries > (1 << 20) || n_expert <= 0 || n_expert > MAYA_MAX_EXPERTS)
        return fail(MAYA_E_SHAPE, "prefill_plan: entries %d experts %d", n_entries, n_expert);
    const size_t lds = sizeof(int32_t) * ((size_t) kPlanWaves * n_expert + n_expert + 1);
    if (lds > 65536) MAYA_HIP(hipFuncSetAttribute((const void*) prefill_plan_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
    hipLaunchKernelGGL(prefill_plan_kernel, dim3(1), dim3(kPlanThreads), lds, as_stream(stream), ids, n_entries, expert_table,
                       n_expert, *plan, maya_moe_prefill_max_tiles(n_entries, n_expert));
    MAYA_LAUNCHED("prefill_plan_kernel");
    return MAYA_OK;
}

int maya_moe_prefill_quant(const void* x, int x_dtype, int64_t x_stride, const maya_prefill_plan* plan, int n_entries,
                           int n_expert, int k, int64_t n_embd, maya_prefill_act xq, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (x_dtype < 0 || x_dtype > 2) return fail(MAYA_E_UNSUPPORTED, "prefill_quant: dtype %d", x_dtype);
    if (!x || !plan_ok(plan) || !act_ok(xq)) return fail(MAYA_E_ARG, "prefill_quant: null or misaligned pointer");
    if (n_entries <= 0 || n_entries > 65535 || k <= 0 || n_embd <= 0 || n_embd % 256 || n_expert <= 0)
        return fail(MAYA_E_SHAPE, "prefill_quant: entries %d k %d n_embd %lld", n_entries, k, (long long) n_embd);
    if (x_stride == 0) x_stride = n_embd;
    if (n_entries % k) return fail(MAYA_E_SHAPE, "prefill_quant: %d entries are not whole tokens of %d", n_entries, k);
    const dim3 grid((unsigned) (n_embd / 256), (unsigned) (n_entries / k));
    hipStream_t s = as_stream(stream);
    switch (x_dtype) {
        case MAYA_DT_F32: hipLaunchKernelGGL(prefill_quant_kernel<MAYA_DT_F32>, grid, dim3(256), 0, s, x, x_stride, *plan, k, n_embd, xq); break;
        case MAYA_DT_BF16: hipLaunchKernelGGL(prefill_quant_kernel<MAYA_DT_BF16>, grid, dim3(256), 0, s, x, x_stride, *plan, k, n_embd, xq); break;
        default: hipLaunchKernelGGL(prefill_quant_kernel<MAYA_DT_F16>, grid, dim3(256), 0, s, x, x_stride, *plan, k, n_embd, xq); break;
    }
    MAYA_LAUNCHED("prefill_quant_kernel");
    return MAYA_OK;
}

static int prefill_check(const char* what, const maya_moe_layout* l, const uint64_t* table, int n_expert, const maya_prefill_plan* plan,
                         int n_entries, int type_a, int type_b) {
    if (!l || !table || !plan_ok(plan)) return fail(MAYA_E_ARG, "%s: null pointer", what);
    if (type_a != kQ4_K || type_b != kQ4_K) return fail(MAYA_E_UNSUPPORTED, "%s: weight types %d / %d (Q4_K only)", what, type_a, type_b);
    if (l->packing != MAYA_PACK_GGUF) return fail(MAYA_E_UNSUPPORTED, "%s: GGUF packing only", what);
    if (l->n_embd <= 0 || l->n_ff <= 0 || l->n_embd % 256 || l->n_ff % 256)
        return fail(MAYA_E_SHAPE, "%s: n_embd %d / n_ff %d: multiples of 256 wanted", what, l->n_embd, l->n_ff);
    if ((l->gate_off | l->up_off | l->down_off) & 15) return fail(MAYA_E_ARG, "%s: matrix offsets not 16-byte aligned", what);
    if (n_entries <= 0 || n_entries > 65535 * kPfRows || n_expert <= 0) return fail(MAYA_E_SHAPE, "%s: entries %d experts %d", what, n_entries, n_expert);
    return MAYA_OK;
}

int maya_moe_prefill_gate_up(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, const maya_prefill_plan* plan,
                             int n_entries, maya_prefill_act xq, float limit, maya_prefill_act hq, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (const int rc = prefill_check("prefill_gate_up", l, expert_table, n_expert, plan, n_entries, l ? l->gate_type : 0, l ? l->up_type : 0)) return rc;
    if (!act_ok(xq) || !act_ok(hq)) return fail(MAYA_E_ARG, "prefill_gate_up: null or misaligned activations");
    if (l->n_ff % 128) return fail(MAYA_E_SHAPE, "prefill_gate_up: n_ff %d: a multiple of 128 wanted", l->n_ff);
    PfGemm a{};
    a.table = expert_table;
    a.plan = *plan;
    a.off[0] = l->gate_off;
    a.off[1] = l->up_off;
    a.k = l->n_embd;
    a.n = l->n_ff;
    a.row_bytes = (int64_t) (l->n_embd / 256) * 144;
    a.x = xq;
    a.h = hq;
    a.limit = limit;
    const dim3 grid((unsigned) (l->n_ff / 128), (unsigned) maya_moe_prefill_max_tiles(n_entries, n_expert));
    hipLaunchKernelGGL(prefill_q4k_kernel<true>, grid, dim3(256), 0, as_stream(stream), a);
    MAYA_LAUNCHED("prefill_q4k_kernel<gate_up>");
    return MAYA_OK;
}

int maya_moe_prefill_down(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, const maya_prefill_plan* plan,
                          int n_entries, maya_prefill_act hq, float* part, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (const int rc = prefill_check("prefill_down", l, expert_table, n_expert, plan, n_entries, l ? l->down_type : 0, l ? l->down_type : 0)) return rc;
    if (!act_ok(hq) || !part) return fail(MAYA_E_ARG, "prefill_down: null or misaligned pointer");
    if (l->n_embd % 64) return fail(MAYA_E_SHAPE, "prefill_down: n_embd %d", l->n_embd);
    PfGemm a{};
    a.table = expert_table;
    a.plan = *plan;
    a.off[0] = l->down_off;
    a.k = l->n_ff;
    a.n = l->n_embd;
    a.row_bytes = (int64_t) (l->n_ff / 256) * 144;
    a.x = hq;
    a.part = part;
    const dim3 grid((unsigned) ((l->n_embd + 255) / 256), (unsigned) maya_moe_prefill_max_tiles(n_entries, n_expert));
    hipLaunchKernelGGL(prefill_q4k_kernel<false>, grid, dim3(256), 0, as_stream(stream), a);
    MAYA_LAUNCHED("prefill_q4k_kernel<down>");
    return MAYA_OK;
}

int maya_moe_prefill_combine(const maya_prefill_plan* plan, const float* weights, const float* part, int n_tokens, int k,
                             int64_t n_embd, const float* add, void* out, int out_dtype, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!plan_ok(plan) || !weights || !part || !out) return fail(MAYA_E_ARG, "prefill_combine: null pointer");
    if (out_dtype < 0 || out_dtype > 2) return fail(MAYA_E_UNSUPPORTED, "prefill_combine: dtype %d", out_dtype);
    if (n_tokens <= 0 || n_tokens > 65535 || k <= 0 || n_embd <= 0) return fail(MAYA_E_SHAPE, "prefill_combine: tokens %d k %d", n_tokens, k);
    const dim3 grid((unsigned) ((n_embd + 255) / 256), (unsigned) n_tokens);
    hipStream_t s = as_stream(stream);
    switch (out_dtype) {
        case MAYA_DT_F32: hipLaunchKernelGGL(prefill_combine_kernel<MAYA_DT_F32>, grid, dim3(256), 0, s, plan->entry_row, weights, part, k, n_embd, add, out); break;
        case MAYA_DT_BF16: hipLaunchKernelGGL(prefill_combine_kernel<MAYA_DT_BF16>, grid, dim3(256), 0, s, plan->entry_row, weights, part, k, n_embd, add, out); break;
        default: hipLaunchKernelGGL(prefill_combine_kernel<MAYA_DT_F16>, grid, dim3(256), 0, s, plan->entry_row, weights, part, k, n_embd, add, out); break;
    }
    MAYA_LAUNCHED("prefill_combine_kernel");
    return MAYA_OK;
}

struct PrefillWs {
    maya_prefill_plan plan;
    maya_prefill_act x, h;
    float* part;
    size_t bytes;
};
static PrefillWs prefill_carve(const maya_moe_layout& l, int n_tokens, int k, int n_expert, uint8_t* base) {
    PrefillWs w{};
    size_t off = 0;
    const size_t ne = (size_t) n_tokens * k;
    auto take = [&](size_t n) {
        uint8_t* p = base ? base + off : nullptr;
        off += (n + 255) & ~(size_t) 255;
        return p;
    };
    const size_t mt = (size_t) maya_moe_prefill_max_tiles((int) ne, n_expert);
    w.plan.bounds = (int32_t*) take(4 * ((size_t) n_expert + 1));
    w.plan.row_entry = (int32_t*) take(4 * ne);
    w.plan.entry_row = (int32_t*) take(4 * ne);
    w.plan.tile_expert = (int32_t*) take(4 * mt);
    w.plan.tile_row0 = (int32_t*) take(4 * mt);
    w.plan.n_tiles = (int32_t*) take(4);
    w.x.q = (int8_t*) take(ne * l.n_embd);
    w.x.d = (float*) take(ne * (l.n_embd / 32) * 4);
    w.x.s = (float*) take(ne * (l.n_embd / 32) * 4);
    w.h.q = (int8_t*) take(ne * l.n_ff);
    w.h.d = (float*) take(ne * (l.n_ff / 32) * 4);
    w.h.s = (float*) take(ne * (l.n_ff / 32) * 4);
    w.part = (float*) take(ne * l.n_embd * 4);
    w.bytes = off;
    return w;
}
size_t maya_moe_prefill_workspace_bytes(const maya_moe_layout* l, int n_tokens, int k, int n_expert) {
    if (!l || n_tokens <= 0 || k <= 0 || n_expert <= 0 || l->n_embd <= 0 || l->n_ff <= 0) return 0;
    return prefill_carve(*l, n_tokens, k, n_expert, nullptr).bytes;
}

int maya_moe_prefill_layer(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k, const float* logits,
                           const void* x, int x_dtype, int n_tokens, float limit, const float* add, int32_t* ids,
                           float* weights, void* out, int out_dtype, void* workspace, size_t workspace_bytes, void* stream) {
    if (!l || !expert_table || !logits || !x || !ids || !weights || !out || !workspace) return fail(MAYA_E_ARG, "prefill_layer: null pointer");
    if (n_tokens <= 0 || n_tokens > 8192 || k <= 0 || k > MAYA_MAX_K) return fail(MAYA_E_SHAPE, "prefill_layer: tokens %d k %d", n_tokens, k);
    if (((uintptr_t) workspace & 255) != 0) return fail(MAYA_E_ARG, "prefill_layer: workspace not 256-byte aligned");
    const PrefillWs w = prefill_carve(*l, n_tokens, k, n_expert, (uint8_t*) workspace);
    if (workspace_bytes < w.bytes) return fail(MAYA_E_ARG, "prefill_layer: workspace %zu < %zu bytes", workspace_bytes, w.bytes);
    const int ne = n_tokens * k;
    int rc;
    if ((rc = maya_moe_route_topk(logits, n_tokens, n_expert, k, ids, weights, stream))) return rc;
    if ((rc = maya_moe_prefill_plan(ids, ne, expert_table, n_expert, &w.plan, stream))) return rc;
    if ((rc = maya_moe_prefill_quant(x, x_dtype, 0, &w.plan, ne, n_expert, k, l->n_embd, w.x, stream))) return rc;
    if ((rc = maya_moe_prefill_gate_up(l, expert_table, n_expert, &w.plan, ne, w.x, limit, w.h, stream))) return rc;
    if ((rc = maya_moe_prefill_down(l, expert_table, n_expert, &w.plan, ne, w.h, w.part, stream))) return rc;
    return maya_moe_prefill_combine(&w.plan, weights, w.part, n_tokens, k, l->n_embd, add, out, out_dtype, stream);
}

}  // extern "C"
