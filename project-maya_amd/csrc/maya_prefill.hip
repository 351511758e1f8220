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
                                                                    maya_prefill_plan p, int max_tiles, int with_masks) {
    extern __shared__ __attribute__((aligned(16))) int32_t sm[];
    int32_t* seg = sm;                               // [kPlanWaves][n_expert]
    int32_t* base = sm + kPlanWaves * n_expert;      // [n_expert + 1]
    // (with_masks: [kPlanWaves][n_expert] 64-bit words behind base, 8-byte aligned)
    unsigned long long* mask = with_masks ? (unsigned long long*) (sm + ((kPlanWaves * n_expert + n_expert + 1 + 1) & ~1)) : nullptr;
    __shared__ int32_t s_tiles;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    for (int i = tid; i < kPlanWaves * n_expert; i += kPlanThreads) seg[i] = 0;
    if (mask != nullptr)
        for (int i = tid; i < kPlanWaves * n_expert; i += kPlanThreads) mask[i] = 0ull;
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
    // base[x + 1] = the experts' running total: wave 0, a lane a run of experts, a scan over the lanes between two passes
    if (tid < 64) {
        const int per_lane = (n_expert + 63) >> 6, x0 = tid * per_lane;
        int local = 0;
        for (int i = 0; i < per_lane; ++i)
            if (x0 + i < n_expert) local += base[x0 + i + 1];
        int incl = local;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d, 64);
            if (tid >= d) incl += up;
        }
        int run = incl - local;
        for (int i = 0; i < per_lane; ++i)
            if (x0 + i < n_expert) {
                run += base[x0 + i + 1];
                base[x0 + i + 1] = run;
            }
        if (tid == 0) base[0] = 0;
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
        if (mask != nullptr) {
            // every lane sets its bit in its expert's word; the word then tells each lane how many earlier lanes share its
            // expert (LDS operations of one wave complete in order); the expert's last lane clears the word again
            unsigned long long* mk = mask + (size_t) wave * n_expert;
            if (x >= 0) atomicOr(&mk[x], 1ull << lane);
            __builtin_amdgcn_wave_barrier();
            if (x >= 0) {
                const unsigned long long m = mk[x];
                rank = __popcll(m & ((1ull << lane) - 1ull));
                cnt = __popcll(m);
            }
            __builtin_amdgcn_wave_barrier();
            if (x >= 0 && rank == cnt - 1) mk[x] = 0ull;
        }
        unsigned long long todo = mask != nullptr ? 0ull : __ballot(x >= 0);
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

// Q8_K rows - the activation format of the reference's CPU expert path for the K-quants
// (src/kernels/cuda/quantize_act.cu:161-207) - rounded 32 values a lane, 8 lanes a 256-value block (q8k_round_lane32: no
// LDS, no barrier): the block's signed maximum is the value at the FIRST largest magnitude, iscale = -127 / max,
// c = min(127, nearest_int(iscale x)), d = 1 / iscale; s = the sum of each 32 codes - what the minimums of a Q4_K
// sub-block multiply - as two FP16 digits, sum = lo + 64 hi with lo in 0..63: both are exact in FP16, and so is every
// product with a 6-bit minimum (times 64 for the high digit), which lets an FP16 matrix instruction form the integer
// sum over a block's 8 sub-blocks exactly.
struct PfLane {
    int y[8];      // 32 codes
    float d;
    int sum;
};
template <int DT>
__device__ __forceinline__ void pf_load32(const void* x, int64_t i0, bool on, float (&v)[32]) {
    if (!on) {
#pragma unroll
        for (int i = 0; i < 32; ++i) v[i] = 0.0f;
        return;
    }
    if constexpr (DT == MAYA_DT_F32) {
        const float* p = (const float*) x + i0;
        if (((uintptr_t) p & 15) == 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float4 t = ((const float4*) p)[i];
                v[4 * i] = t.x, v[4 * i + 1] = t.y, v[4 * i + 2] = t.z, v[4 * i + 3] = t.w;
            }
            return;
        }
    } else {
        const uint16_t* p = (const uint16_t*) x + i0;
        if (((uintptr_t) p & 15) == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint4 t = ((const uint4*) p)[i];
                const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if constexpr (DT == MAYA_DT_BF16) {
                        v[8 * i + 2 * j] = __uint_as_float(w[j] << 16);
                        v[8 * i + 2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
                    } else {
                        v[8 * i + 2 * j] = f16_bits_to_f32(w[j] & 0xffffu);
                        v[8 * i + 2 * j + 1] = f16_bits_to_f32(w[j] >> 16);
                    }
                }
            }
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < 32; ++i) v[i] = pf_load<DT>(x, i0 + i);
}
__device__ __forceinline__ PfLane pf_round_lane(const float (&v)[32], int lane) {
    PfLane o;
    q8k_round_lane32(v, [&](int i) { return 32 * (lane & 7) + i; }, o.y, o.d);
    int sum = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) sum = dot4(0x01010101, o.y[i], sum);
    o.sum = sum;
    return o;
}
__device__ __forceinline__ void pf_store_lane(const maya_prefill_act& o, size_t row, int64_t k, int64_t v0, int lane, const PfLane& c) {
    const size_t at = row * (size_t) k + (size_t) v0;
    int4* q = (int4*) (o.q + at);
    q[0] = make_int4(c.y[0], c.y[1], c.y[2], c.y[3]);
    q[1] = make_int4(c.y[4], c.y[5], c.y[6], c.y[7]);
    // (a block's 16 halves: the low digits of its 8 sub-blocks, then the high digits)
    _Float16* sp = (_Float16*) o.s + (at >> 8) * 16 + (lane & 7);
    sp[0] = (_Float16) (float) (c.sum & 63);
    sp[8] = (_Float16) (float) (c.sum >> 6);
    if ((lane & 7) == 0) o.d[at >> 8] = c.d;
}

// grid (k / 8192 rounded up, tokens): a token's values are rounded once and written to the rows of all its entries in the plan
template <int DT>
__global__ __launch_bounds__(256) void prefill_quant_kernel(const void* __restrict__ x, int64_t x_stride, maya_prefill_plan p,
                                                            int top_k, int64_t k, maya_prefill_act o) {
    const int t = blockIdx.y, lane = threadIdx.x & 63;
    const int64_t v0 = ((int64_t) blockIdx.x * 256 + threadIdx.x) * 32;
    const bool on = v0 < k;   // (k is a multiple of 256: the 8 lanes of a block are on or off together)
    float v[32];
    pf_load32<DT>(x, (int64_t) t * x_stride + v0, on, v);
    const PfLane c = pf_round_lane(v, lane);
    if (!on) return;
    for (int j = 0; j < top_k; ++j) {
        const int row = p.entry_row[t * top_k + j];
        if (row < 0) continue;   // an entry of an expert that is not resident
        pf_store_lane(o, (size_t) row, k, v0, lane, c);
    }
}
// grid (k / 8192 rounded up, rows at most): the plan's row blockIdx.y of an F32 matrix (the SwiGLU outputs)
__global__ __launch_bounds__(256) void prefill_quant_rows_kernel(const float* __restrict__ x, maya_prefill_plan p, int n_expert,
                                                                 int64_t k, maya_prefill_act o) {
    const int row = blockIdx.y, lane = threadIdx.x & 63;
    if (row >= p.bounds[n_expert]) return;
    const int64_t v0 = ((int64_t) blockIdx.x * 256 + threadIdx.x) * 32;
    const bool on = v0 < k;
    float v[32];
    pf_load32<MAYA_DT_F32>(x, (int64_t) row * k + v0, on, v);
    const PfLane c = pf_round_lane(v, lane);
    if (on) pf_store_lane(o, (size_t) row, k, v0, lane, c);
}

// ---------------------------------------------------------------------------------------------------- the GEMM
// out[row][n] = sum over 256-value blocks b of (d_w[n][b] d_x[row][b]) * sum_j sc[n][j] (q[n] . c[row])_j  -  the
// minimums' term: ggml_vec_dot_q4_K_q8_K's integer sums, exactly.  The 6-bit sub-block scale is split sc = 8 hi + lo, so
// q sc = 8 (q hi) + (q lo) with both products <= 105: two int8 planes of the weights.  Their products with the codes run
// on the int8 matrix cores and are accumulated in int32 over the whole 256-value block - the sub-block scales never leave
// the integer domain, and the vector ALU converts and scales once per 256 values.
struct PfGemm {
    const uint64_t* table;
    maya_prefill_plan plan;
    uint64_t off[2];       // gate and up (gate/up), down and unused (down): byte offsets of the matrices in a blob
    int64_t k, n;          // inner length, weight rows of one matrix
    int64_t row_bytes;
    maya_prefill_act x;    // the tile rows' activations [rows][k]
    float* out;            // gate/up: the SwiGLU outputs [rows][n] F32; down: part [rows][n]
    float limit;
};

// LDS of one buffer: the codes [kPfRows][256] (16-byte chunk c of row r at position c ^ (r & 15): the 16 rows x 4
// k-groups of a matrix-core operand read then hit distinct banks), s [kPfRows][8], d [kPfRows]
constexpr int kPfPlane = kPfRows * 256;
constexpr int kPfSOff = kPfPlane, kPfDOff = kPfSOff + kPfRows * 32;
constexpr int kPfBufBytes = kPfDOff + kPfRows * 4;
constexpr int kPfDOffNoS = kPfPlane, kPfBufBytesNoS = kPfDOffNoS + kPfRows * 4;   // (a buffer without s: types without minimums)

typedef __attribute__((address_space(3))) void* pf_lptr;
// The tile's activations go from global memory to LDS without passing registers (each lane's 16 bytes land at the
// wave's base + 16 lane): buffer loads whose per-lane offsets are fixed for the tile - the super-block rides in the
// scalar offset - so a copy costs no vector arithmetic.  Rows past the tile's end repeat its last row (their results
// are never stored).
template <int NMT, bool WITH_S = true>
struct PfDma {
    __amdgpu_buffer_rsrc_t rq, rs, rd;
    uint32_t oq[NMT], os, od;
    int wave;
    __device__ __forceinline__ void init(const PfGemm& a, int row0, int nrows, int wave_, int lane) {
        wave = wave_;
        const int last = nrows - 1;
        rq = __builtin_amdgcn_make_buffer_rsrc((void*) (a.x.q + (size_t) row0 * a.k), 0, (int) (nrows * a.k), 0x00020000);
        rs = __builtin_amdgcn_make_buffer_rsrc((void*) (a.x.s + (size_t) row0 * (a.k >> 4)), 0, (int) (nrows * (a.k >> 5) * 4), 0x00020000);
        rd = __builtin_amdgcn_make_buffer_rsrc((void*) (a.x.d + (size_t) row0 * (a.k >> 8)), 0, (int) (nrows * (a.k >> 8) * 4), 0x00020000);
#pragma unroll
        for (int n = 0; n < NMT; ++n) {
            const int r = 4 * (wave + 4 * n) + (lane >> 4), cp = lane & 15;   // rows 4 i .. 4 i + 3, i = wave + 4 n
            oq[n] = (uint32_t) (min(r, last) * (int) a.k + ((cp ^ (r & 15)) * 16));
        }
        os = (uint32_t) (min(32 * wave + (lane >> 1), last) * (int) (a.k >> 5) * 4 + (lane & 1) * 16);
        od = (uint32_t) (min(lane, last) * (int) (a.k >> 8) * 4);
    }
    // super-block sb into the buffer at `buf`
    __device__ __forceinline__ void copy(uint8_t* buf, int sb) const {
#pragma unroll
        for (int n = 0; n < NMT; ++n)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rq, (pf_lptr) (buf + (wave + 4 * n) * 1024), 16, oq[n], sb * 256, 0, 0);
        if (WITH_S && wave < 2 && 32 * wave < 16 * NMT)   // s: 32 rows an instruction, 32 bytes a row
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (pf_lptr) (buf + kPfSOff + wave * 1024), 16, os, sb * 32, 0, 0);
        if (wave == 2) __builtin_amdgcn_raw_ptr_buffer_load_lds(rd, (pf_lptr) (buf + (WITH_S ? kPfDOff : kPfDOffNoS)), 4, od, sb * 4, 0, 0);
    }
};

// the 8 six-bit scales and 8 six-bit minimums of a Q4_K block's 12 bytes, as bytes of two words each
// (get_scale_min_k4, include/strata/artifact/dequant.hpp:162-172)
__device__ __forceinline__ void q4k_unpack_scales(uint32_t s0, uint32_t s1, uint32_t s2, uint32_t (&sc)[2], uint32_t (&mn)[2]) {
    sc[0] = s0 & 0x3f3f3f3fu;
    mn[0] = s1 & 0x3f3f3f3fu;
    sc[1] = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
    mn[1] = ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u);
}

__device__ __forceinline__ float pf_swiglu(float g, float u, float limit) {
    if (limit > 0.0f && limit < INFINITY) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
    }
    return __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, expf(-g))), u);
}

typedef unsigned short pf_u16x2 __attribute__((ext_vector_type(2)));
// four 4-bit codes (one a byte) times a factor <= 7: no byte overflows, so one packed 16-bit multiply does it
__device__ __forceinline__ uint32_t pf_scale_codes(uint32_t w, uint32_t f) {
    const pf_u16x2 ff = {(unsigned short) f, (unsigned short) f};
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(pf_u16x2, w) * ff);
}

// LDS reads of the GEMM loop are written out by hand.  The compiler cannot tell which LDS buffer a direct-to-LDS copy
// fills, so before any LDS read of its own it waits for every copy in flight - here that would be the copy of the
// super-block two ahead, issued moments earlier.  These reads it does not see; each group is followed by pf_lds_wait
// on the registers it filled (the values pass through the wait, so nothing that uses them can move above it).
__device__ __forceinline__ uint32_t pf_lds_addr(const void* p) {
    return (uint32_t) (uintptr_t) (const __attribute__((address_space(3))) void*) p;
}
typedef int pf_i2 __attribute__((ext_vector_type(2)));
template <int OFF> __device__ __forceinline__ pf_i2 pf_lds_b64(uint32_t addr) {
    pf_i2 v;
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
template <int OFF> __device__ __forceinline__ uint32_t pf_lds_u16(uint32_t addr) {
    uint32_t v;
    asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
template <int OFF> __device__ __forceinline__ float pf_lds_f32(uint32_t addr) {
    float v;
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
template <int OFF> __device__ __forceinline__ v4f pf_lds_f32x4(uint32_t addr) {
    v4f v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
template <int OFF> __device__ __forceinline__ v4i pf_lds_i32x4(uint32_t addr) {
    v4i v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
template <int N, typename T> __device__ __forceinline__ void pf_lds_wait(T (&r)[N]) {
    if constexpr (N == 1) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]));
    else if constexpr (N == 2) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]));
    else if constexpr (N == 3) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]));
    else if constexpr (N == 4) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]));
    else if constexpr (N == 6) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]));
    else {
        static_assert(N == 8, "1, 2, 3, 4, 6 or 8 registers");
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
    }
}
// the registers r have landed once at most BUT later LDS reads are outstanding (LDS operations complete in order)
template <int BUT, int N> __device__ __forceinline__ void pf_lds_wait_but(v4i (&r)[N]) {
    static_assert(N == 1 || N == 2, "1 or 2 registers");
    if constexpr (N == 1) asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(r[0]) : "n"(BUT));
    else asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(r[0]), "+v"(r[1]) : "n"(BUT));
}
template <int BUT> __device__ __forceinline__ void pf_lds_wait_tail(v4i& a, v4f (&d)[4]) {
    asm volatile("s_waitcnt lgkmcnt(%5)" : "+v"(a), "+v"(d[0]), "+v"(d[1]), "+v"(d[2]), "+v"(d[3]) : "n"(BUT));
}
// (compile-time loops over the row groups of a tile)
template <int M, int NMT, typename F> __device__ __forceinline__ void pf_for_m(F&& f) {
    if constexpr (M < NMT) {
        f(std::integral_constant<int, M>{});
        pf_for_m<M + 1, NMT>(f);
    }
}

typedef int pf_v16i __attribute__((ext_vector_type(16)));
typedef float pf_v16f __attribute__((ext_vector_type(16)));
typedef _Float16 pf_v8h __attribute__((ext_vector_type(8)));
typedef _Float16 pf_v2h __attribute__((ext_vector_type(2)));

// One tile of NM x 32 rows against the wave's 32 weight rows (gate/up: the gate rows of 16 features, then their up rows;
// down: 32 output rows), on the 32x32 matrix instructions: lane (ln = lane & 31, kh = lane >> 5) holds 16 of a
// sub-block's 32 values of activation row ln (A operand, from LDS) and of weight row ln (B operand, decoded in
// registers), and 16 outputs: weight row ln against the rows 8 b + 4 kh + r (b, r = 0..3) of the 32.  These
// instructions take 32 cycles, and the vector ALU issues about four instructions under each of them; the 16-cycle
// 16x16 forms leave it no slot (measured with a microbenchmark of matrix instructions followed by vector instructions), which is what bounds a
// kernel that has as many vector instructions as this one.
template <bool GU, int NM>
__device__ __forceinline__ void pf_tile(const PfGemm& a, uint8_t* b0, uint8_t* b1, uint8_t* b2, int ex, int row0, int nrows) {
    // (global address space: a generic pointer's loads would count as LDS operations too, and every wait for them
    // would also wait for the copies into LDS behind them)
    typedef const __attribute__((address_space(1))) uint8_t* wptr;
    constexpr int NMT = 2 * NM;   // groups of 16 rows: what the copies into LDS count in
    wptr blob = (wptr) a.table[ex];
    const int tid = threadIdx.x, lane = tid & 63, ln = lane & 31, kh = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    wptr wrow;
    int64_t n0;   // the wave's first feature (gate/up) or output row (down)
    if constexpr (GU) {
        n0 = (int64_t) blockIdx.x * 64 + wave * 16;
        wrow = blob + a.off[ln >> 4] + (size_t) (n0 + (ln & 15)) * a.row_bytes;
    } else {
        n0 = (int64_t) blockIdx.x * 128 + wave * 32;
        wrow = blob + a.off[0] + (size_t) (n0 + ln) * a.row_bytes;
    }
    const bool wave_on = n0 < a.n;   // (a.n is a multiple of the wave's rows: checked on the host)

    pf_v16f acc[NM];
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[m][i] = 0.0f;

    const int nsb = (int) (a.k >> 8);
    // The activations run two super-blocks ahead through three LDS buffers, the weights one ahead in registers.  The
    // buffers are three separate arrays and the loop below is unrolled over them, so that the compiler can tell a read
    // of one from a copy into another (it would otherwise wait for every copy in flight before each LDS read).
    PfDma<NMT> dma;
    dma.init(a, row0, nrows, wave, lane);
    dma.copy(b0, 0);
    if (nsb > 1) dma.copy(b1, 1);
    // the weights of a super-block: the 16-byte header of the lane's row and four 16-byte pieces of its codes, bytes
    // 32 c + 16 kh of the row's 128 (c = 0..3): the low nibbles are 16 values of sub-block 2 c, the high ones of 2 c + 1
    typedef uint32_t w4 __attribute__((ext_vector_type(4)));
    w4 q[4], qn[4], hdr, hdrn;
    auto load_block = [&](int sb, w4 (&dq)[4], w4& dh) {
        wptr blk = wrow + (size_t) sb * 144;
        dh = *(const __attribute__((address_space(1))) w4*) blk;
#pragma unroll
        for (int c = 0; c < 4; ++c) dq[c] = *(const __attribute__((address_space(1))) w4*) (blk + 16 + 32 * c + 16 * kh);
    };
    if (wave_on) load_block(0, q, hdr);
    // a lane's 16 codes of sub-block j: the row's 16-byte chunk 2 j + kh, which sits at that index ^ (the row & 15)
    const int a_base = ln * 256, a_swz = ((ln & 15) ^ kh) << 4;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    auto step = [&](int sb, const uint8_t* buf, uint8_t* buf2) {   // super-block sb from buf; sb + 2 is copied into buf2
        float d = 0.0f, ndmin = 0.0f;
        uint32_t sc[2], mn[2];
        if (wave_on) {
            d = f16_bits_to_f32((uint16_t) (hdr.x & 0xffffu));
            ndmin = -f16_bits_to_f32((uint16_t) (hdr.x >> 16));
            q4k_unpack_scales(hdr.y, hdr.z, hdr.w, sc, mn);
            if (sb + 1 < nsb) load_block(sb + 1, qn, hdrn);
        }
        // (after the weights' loads, so that waiting for everything but these copies covers the weights too)
        if (sb + 2 < nsb) dma.copy(buf2, sb + 2);
        if (wave_on) {
            const uint32_t lbuf = pf_lds_addr(buf);
            // The two plane products of the block, int32: [m][0] = (q lo) . c, [1] = (q hi) . c, a matrix instruction a
            // sub-block and plane, accumulated over the 8 sub-blocks.  The activation operand of sub-block jj + 1 is
            // requested from LDS before the arithmetic of sub-block jj, and the operands of the block's closing stage
            // (the code sums, the block scales) before the last sub-block: a read issued just ahead of its use leaves
            // the wave waiting for LDS eight times a step.
            pf_v16i dot[NM][2];
            v4i xr[2][NM];
            auto read_x = [&](int jj, v4i (&dst)[NM]) {
                const uint32_t at = lbuf + a_base + (a_swz ^ ((2 * jj) << 4));
                pf_for_m<0, NM>([&](auto mc) {
                    constexpr int m = decltype(mc)::value;
                    dst[m] = pf_lds_i32x4<m * 8192>(at);
                });
            };
            v4i sa[NM];
            v4f dxr[NM][4];
            auto read_tail = [&](auto mc) {   // the closing stage's operands of row group m: its code sums and block scales
                constexpr int m = decltype(mc)::value;
                sa[m] = pf_lds_i32x4<kPfSOff + m * 1024>(lbuf + ln * 32 + kh * 16);
                const uint32_t at = lbuf + 16 * kh;
                dxr[m][0] = pf_lds_f32x4<kPfDOff + m * 128>(at);
                dxr[m][1] = pf_lds_f32x4<kPfDOff + m * 128 + 32>(at);
                dxr[m][2] = pf_lds_f32x4<kPfDOff + m * 128 + 64>(at);
                dxr[m][3] = pf_lds_f32x4<kPfDOff + m * 128 + 96>(at);
            };
            read_x(0, xr[0]);
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) {
                const int c = jj >> 1, j = jj & 1;
                if (jj < 7) read_x(jj + 1, xr[(jj + 1) & 1]);
                if (jj == 7) read_tail(std::integral_constant<int, 0>{});
                const uint32_t f = (sc[c >> 1] >> (16 * (c & 1) + 8 * j)) & 0x3fu, flo = f & 7u, fhi = f >> 3;
                v4i wl, wh;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t w = (q[c][i] >> (4 * j)) & 0x0f0f0f0fu;
                    wl[i] = (int) pf_scale_codes(w, flo);
                    wh[i] = (int) pf_scale_codes(w, fhi);
                }
                // this sub-block's operand has landed once only the reads issued after it are outstanding (LDS answers in order)
                if (jj < 7) pf_lds_wait_but<NM>(xr[jj & 1]);
                else pf_lds_wait_but<5>(xr[jj & 1]);
#pragma unroll
                for (int m = 0; m < NM; ++m) {
                    const pf_v16i z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    dot[m][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xr[jj & 1][m], wl, jj ? dot[m][0] : z, 0, 0, 0);
                    dot[m][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xr[jj & 1][m], wh, jj ? dot[m][1] : z, 0, 0, 0);
                }
            }
            // The minimums' integer term sum_j m_j (sum of sub-block j's codes), exactly, from one FP16 matrix instruction:
            // k = 0..7 pairs m_j with the sums' low digits, k = 8..15 pairs 64 m_j with their high digits (every operand
            // and every partial sum an integer below 2^24).
            pf_v8h mb;
            {
                const float mul = kh ? 64.0f : 1.0f;
#pragma unroll
                for (int w = 0; w < 2; ++w)
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        const pf_v2h t = __builtin_bit_cast(pf_v2h, __builtin_amdgcn_cvt_pkrtz(__fmul_rn((float) ((mn[w] >> (16 * i)) & 0xffu), mul),
                                                                                              __fmul_rn((float) ((mn[w] >> (16 * i + 8)) & 0xffu), mul)));
                        mb[4 * w + 2 * i] = t[0], mb[4 * w + 2 * i + 1] = t[1];
                    }
            }
            // once a block: lo + 8 hi = the block's integer sum (< 2^25), then d_x (d_w sum - dmin_w minimums)
            pf_for_m<0, NM>([&](auto mc) {
                constexpr int m = decltype(mc)::value;
                if constexpr (m + 1 < NM) {
                    read_tail(std::integral_constant<int, m + 1>{});
                    pf_lds_wait_tail<5>(sa[m], dxr[m]);
                } else {
                    pf_lds_wait_tail<0>(sa[m], dxr[m]);
                }
                const pf_v16f z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                const pf_v16f mins = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pf_v8h, sa[m]), mb, z, 0, 0, 0);
                // (a lane's outputs 4 b .. 4 b + 3 are the tile's rows 32 m + 8 b + 4 kh + 0..3: blocks of 8 rows past the
                // tile's last row are skipped - most tiles of a skewed routing hold 8 rows or fewer)
                const int nb = (nrows - 32 * m + 7) >> 3;
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    if (b < nb) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int i = 4 * b + r;
                            const float t = fmaf(ndmin, mins[i], __fmul_rn(d, (float) (dot[m][0][i] + 8 * dot[m][1][i])));
                            acc[m][i] = fmaf(dxr[m][b][r], t, acc[m][i]);
                        }
                    }
                }
            });
            if (sb + 1 < nsb) {
                hdr = hdrn;
#pragma unroll
                for (int c = 0; c < 4; ++c) q[c] = qn[c];
            }
        }
        // super-block sb + 1 has landed once only the wave's youngest NMT operations may still be in flight: this
        // iteration's copies (of sb + 2), or - in the last steps, which copy nothing - some of the five weight loads
        // issued above; a wave that holds no weight rows has nothing younger than its last copies then and waits for all
        // (a bare barrier: __syncthreads() would first wait for every memory operation of the wave, these copies included)
        if (sb + 2 < nsb || wave_on) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(NMT) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };
    for (int sb = 0; sb < nsb; sb += 3) {
        step(sb, b0, b2);
        if (sb + 1 < nsb) step(sb + 1, b1, b0);
        if (sb + 2 < nsb) step(sb + 2, b2, b1);
    }
    if (!wave_on) return;

    // outputs: lane (ln, kh) holds weight row ln for the tile's rows 32 m + 8 b + 4 kh + r (i = 4 b + r)
#pragma unroll
    for (int m = 0; m < NM; ++m) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int r = 32 * m + 8 * (i >> 2) + 4 * kh + (i & 3);
            if constexpr (GU) {
                // the up row of a feature sits 16 lanes above its gate row
                const float up = __shfl(acc[m][i], (lane + 16) & 63, kWave);
                if (ln < 16 && r < nrows) a.out[(size_t) (row0 + r) * a.n + n0 + ln] = pf_swiglu(acc[m][i], up, a.limit);
            } else {
                if (r < nrows) a.out[(size_t) (row0 + r) * a.n + n0 + ln] = acc[m][i];
            }
        }
    }
}

#include "maya_prefill_iq2s.hpp"

// grid (bands of weight rows, tiles at most)
template <bool GU>
__global__ __launch_bounds__(256, 2) void prefill_q4k_kernel(PfGemm a) {
    __shared__ __attribute__((aligned(16))) uint8_t b0[kPfBufBytes], b1[kPfBufBytes], b2[kPfBufBytes];
    const int tile = blockIdx.y;
    if (tile >= *a.plan.n_tiles) return;
    const int ex = a.plan.tile_expert[tile], row0 = a.plan.tile_row0[tile];
    const int nrows = min(kPfRows, a.plan.bounds[ex + 1] - row0);
    if (nrows <= 32) pf_tile<GU, 1>(a, b0, b1, b2, ex, row0, nrows);
    else pf_tile<GU, 2>(a, b0, b1, b2, ex, row0, nrows);
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

// the same, four columns a thread (n a multiple of 4, 16-byte aligned rows): the k rows' loads are issued together, the
// sum keeps the slot order
template <int ODT>
__global__ __launch_bounds__(256) void prefill_combine4_kernel(const int32_t* __restrict__ entry_row, const float* __restrict__ w,
                                                               const float* __restrict__ part, int k, int64_t n,
                                                               const float* __restrict__ add, void* __restrict__ out) {
    const int t = blockIdx.y;
    const int64_t c = ((int64_t) blockIdx.x * 256 + threadIdx.x) * 4;
    if (c >= n) return;
    float4 v[MAYA_MAX_K];
    float wj[MAYA_MAX_K];
    bool on[MAYA_MAX_K];
#pragma unroll
    for (int j = 0; j < MAYA_MAX_K; ++j) {
        const int row = j < k ? entry_row[t * k + j] : -1;
        on[j] = row >= 0;
        if (on[j]) {
            v[j] = *(const float4*) (part + (size_t) row * n + c);
            wj[j] = w[t * k + j];
        }
    }
    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    bool first = true;
#pragma unroll
    for (int j = 0; j < MAYA_MAX_K; ++j) {
        if (!on[j]) continue;
        const float p[4] = {__fmul_rn(v[j].x, wj[j]), __fmul_rn(v[j].y, wj[j]), __fmul_rn(v[j].z, wj[j]), __fmul_rn(v[j].w, wj[j])};
#pragma unroll
        for (int i = 0; i < 4; ++i) sum[i] = first ? p[i] : __fadd_rn(sum[i], p[i]);
        first = false;
    }
    if (add) {
        const float4 a = *(const float4*) (add + (size_t) t * n + c);
        sum[0] = __fadd_rn(sum[0], a.x), sum[1] = __fadd_rn(sum[1], a.y), sum[2] = __fadd_rn(sum[2], a.z), sum[3] = __fadd_rn(sum[3], a.w);
    }
    if constexpr (ODT == MAYA_DT_F32) {
        *(float4*) ((float*) out + (size_t) t * n + c) = make_float4(sum[0], sum[1], sum[2], sum[3]);
    } else {
        uint16_t h[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if constexpr (ODT == MAYA_DT_BF16) {
                uint32_t u = __float_as_uint(sum[i]);
                if ((u & 0x7fffffffu) > 0x7f800000u) u |= 0x00400000u;          // NaN stays NaN
                else u += 0x7fffu + ((u >> 16) & 1u);                            // round to nearest even
                h[i] = (uint16_t) (u >> 16);
            } else {
                h[i] = __half_as_ushort(__float2half_rn(sum[i]));
            }
        }
        *(uint2*) ((uint16_t*) out + (size_t) t * n + c) = make_uint2(h[0] | ((uint32_t) h[1] << 16), h[2] | ((uint32_t) h[3] << 16));
    }
}

static bool plan_ok(const maya_prefill_plan* p) {
    return p && p->bounds && p->row_entry && p->entry_row && p->tile_expert && p->tile_row0 && p->n_tiles;
}
static bool act_ok(const maya_prefill_act& a) {
    return a.q && a.d && a.s && (((uintptr_t) a.q | (uintptr_t) a.s) & 15) == 0 && ((uintptr_t) a.d & 3) == 0;
}
template <bool GU>
static int pf_launch(const PfGemm& a, dim3 grid, hipStream_t s) {
    hipLaunchKernelGGL(prefill_q4k_kernel<GU>, grid, dim3(256), 0, s, a);
    return MAYA_OK;
}

}  // namespace maya

using namespace maya;

extern "C" {

int maya_moe_prefill_tile_rows(void) { return kPfRows; }
int maya_moe_prefill_max_tiles(int n_entries, int n_expert) {
    if (n_entries <= 0 || n_expert <= 0) return 0;
    return (n_entries + kPfRows - 1) / kPfRows + n_expert;
}
int maya_moe_prefill_supported(int type) { return type == kQ4_K || type == kIQ2_S ? 1 : 0; }

int maya_moe_prefill_plan(const int32_t* ids, int n_entries, const uint64_t* expert_table, int n_expert,
                          const maya_prefill_plan* plan, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!ids || !expert_table || !plan_ok(plan)) return fail(MAYA_E_ARG, "prefill_plan: null pointer");
    if (n_entries <= 0 || n_entries > (1 << 20) || n_expert <= 0 || n_expert > MAYA_MAX_EXPERTS)
        return fail(MAYA_E_SHAPE, "prefill_plan: entries %d experts %d", n_entries, n_expert);
    // (up to 256 experts: a wave's 64-bit lane masks per expert ride along, 8 bytes x 16 waves an expert)
    const int with_masks = n_expert <= 256;
    size_t lds = sizeof(int32_t) * ((size_t) kPlanWaves * n_expert + n_expert + 1);
    if (with_masks) lds = ((lds + 7) & ~(size_t) 7) + sizeof(unsigned long long) * (size_t) kPlanWaves * n_expert;
    if (lds > 65536) MAYA_HIP(hipFuncSetAttribute((const void*) prefill_plan_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
    hipLaunchKernelGGL(prefill_plan_kernel, dim3(1), dim3(kPlanThreads), lds, as_stream(stream), ids, n_entries, expert_table,
                       n_expert, *plan, maya_moe_prefill_max_tiles(n_entries, n_expert), with_masks);
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
    const dim3 grid((unsigned) ((n_embd + 8191) / 8192), (unsigned) (n_entries / k));
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
                         int n_entries, int type_a, int type_b, int64_t k) {
    if (!l || !table || !plan_ok(plan)) return fail(MAYA_E_ARG, "%s: null pointer", what);
    if (type_a != type_b || (type_a != kQ4_K && type_a != kIQ2_S))
        return fail(MAYA_E_UNSUPPORTED, "%s: weight types %d / %d (Q4_K or IQ2_S, gate and up alike)", what, type_a, type_b);
    if (l->packing != MAYA_PACK_GGUF && l->packing != MAYA_PACK_STREAM) return fail(MAYA_E_UNSUPPORTED, "%s: packing %d", what, l->packing);
    if (type_a == kIQ2_S && l->packing != MAYA_PACK_STREAM)
        return fail(MAYA_E_UNSUPPORTED, "%s: IQ2_S rows are taken in the stream packing (maya_moe_repack)", what);
    if (l->n_embd <= 0 || l->n_ff <= 0 || l->n_embd % 256 || l->n_ff % 256)
        return fail(MAYA_E_SHAPE, "%s: n_embd %d / n_ff %d: multiples of 256 wanted", what, l->n_embd, l->n_ff);
    // (IQ2_S: the 16-byte copies of a quad's index words want quads of a multiple of 16 bytes: 328 bytes a block)
    if (type_a == kIQ2_S && k % 512) return fail(MAYA_E_SHAPE, "%s: IQ2_S rows of %lld values: a multiple of 512 wanted", what, (long long) k);
    if ((l->gate_off | l->up_off | l->down_off) & 15) return fail(MAYA_E_ARG, "%s: matrix offsets not 16-byte aligned", what);
    // (an entry is a row of the second grid dimension in the quantizers' launches)
    if (n_entries <= 0 || n_entries > 65535 || n_expert <= 0) return fail(MAYA_E_SHAPE, "%s: entries %d (1..65535) experts %d", what, n_entries, n_expert);
    return MAYA_OK;
}

int maya_moe_prefill_gate_up(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, const maya_prefill_plan* plan,
                             int n_entries, maya_prefill_act xq, float limit, float* h, maya_prefill_act hq, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (const int rc = prefill_check("prefill_gate_up", l, expert_table, n_expert, plan, n_entries, l ? l->gate_type : 0, l ? l->up_type : 0, l ? l->n_embd : 0)) return rc;
    if (!act_ok(xq) || !act_ok(hq) || !h) return fail(MAYA_E_ARG, "prefill_gate_up: null or misaligned activations");
    PfGemm a{};
    a.table = expert_table;
    a.plan = *plan;
    a.off[0] = l->gate_off;
    a.off[1] = l->up_off;
    a.k = l->n_embd;
    a.n = l->n_ff;
    a.row_bytes = (int64_t) (l->n_embd / 256) * 144;
    a.x = xq;
    a.out = h;
    a.limit = limit;
    const dim3 grid((unsigned) (l->n_ff / 64), (unsigned) maya_moe_prefill_max_tiles(n_entries, n_expert));
    if (l->gate_type == kIQ2_S) {
        hipLaunchKernelGGL(prefill_iq2s_kernel<true>, grid, dim3(256), 0, as_stream(stream), a, st->cb);
        MAYA_LAUNCHED("prefill_iq2s_kernel<gate_up>");
    } else {
        if (const int rc = pf_launch<true>(a, grid, as_stream(stream))) return rc;
        MAYA_LAUNCHED("prefill_q4k_kernel<gate_up>");
    }
    const dim3 qgrid((unsigned) ((l->n_ff + 8191) / 8192), (unsigned) n_entries);
    hipLaunchKernelGGL(prefill_quant_rows_kernel, qgrid, dim3(256), 0, as_stream(stream), (const float*) h, *plan, n_expert, (int64_t) l->n_ff, hq);
    MAYA_LAUNCHED("prefill_quant_rows_kernel");
    return MAYA_OK;
}

int maya_moe_prefill_down(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, const maya_prefill_plan* plan,
                          int n_entries, maya_prefill_act hq, float* part, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (const int rc = prefill_check("prefill_down", l, expert_table, n_expert, plan, n_entries, l ? l->down_type : 0, l ? l->down_type : 0, l ? l->n_ff : 0)) return rc;
    if (!act_ok(hq) || !part) return fail(MAYA_E_ARG, "prefill_down: null or misaligned pointer");
    if (l->n_embd % 32) return fail(MAYA_E_SHAPE, "prefill_down: n_embd %d", l->n_embd);
    PfGemm a{};
    a.table = expert_table;
    a.plan = *plan;
    a.off[0] = l->down_off;
    a.k = l->n_ff;
    a.n = l->n_embd;
    a.row_bytes = (int64_t) (l->n_ff / 256) * 144;
    a.x = hq;
    a.out = part;
    const dim3 grid((unsigned) ((l->n_embd + 127) / 128), (unsigned) maya_moe_prefill_max_tiles(n_entries, n_expert));
    if (l->down_type == kIQ2_S) {
        hipLaunchKernelGGL(prefill_iq2s_kernel<false>, grid, dim3(256), 0, as_stream(stream), a, st->cb);
        MAYA_LAUNCHED("prefill_iq2s_kernel<down>");
    } else {
        if (const int rc = pf_launch<false>(a, grid, as_stream(stream))) return rc;
        MAYA_LAUNCHED("prefill_q4k_kernel<down>");
    }
    return MAYA_OK;
}

int maya_moe_prefill_combine(const maya_prefill_plan* plan, const float* weights, const float* part, int n_tokens, int k,
                             int64_t n_embd, const float* add, void* out, int out_dtype, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!plan_ok(plan) || !weights || !part || !out) return fail(MAYA_E_ARG, "prefill_combine: null pointer");
    if (out_dtype < 0 || out_dtype > 2) return fail(MAYA_E_UNSUPPORTED, "prefill_combine: dtype %d", out_dtype);
    if (n_tokens <= 0 || n_tokens > 65535 || k <= 0 || n_embd <= 0) return fail(MAYA_E_SHAPE, "prefill_combine: tokens %d k %d", n_tokens, k);
    hipStream_t s = as_stream(stream);
    if (n_embd % 4 == 0 && k <= MAYA_MAX_K && (((uintptr_t) part | (uintptr_t) add | (uintptr_t) out) & 15) == 0) {
        const dim3 grid4((unsigned) ((n_embd / 4 + 255) / 256), (unsigned) n_tokens);
        switch (out_dtype) {
            case MAYA_DT_F32: hipLaunchKernelGGL(prefill_combine4_kernel<MAYA_DT_F32>, grid4, dim3(256), 0, s, plan->entry_row, weights, part, k, n_embd, add, out); break;
            case MAYA_DT_BF16: hipLaunchKernelGGL(prefill_combine4_kernel<MAYA_DT_BF16>, grid4, dim3(256), 0, s, plan->entry_row, weights, part, k, n_embd, add, out); break;
            default: hipLaunchKernelGGL(prefill_combine4_kernel<MAYA_DT_F16>, grid4, dim3(256), 0, s, plan->entry_row, weights, part, k, n_embd, add, out); break;
        }
        MAYA_LAUNCHED("prefill_combine4_kernel");
        return MAYA_OK;
    }
    const dim3 grid((unsigned) ((n_embd + 255) / 256), (unsigned) n_tokens);
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
    float *hf, *part;
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
    auto take_act = [&](maya_prefill_act& a, size_t k) {
        a.q = (int8_t*) take(ne * k);
        a.d = (float*) take(ne * (k / 256) * 4);
        a.s = (uint16_t*) take(ne * (k / 32) * 4);
    };
    take_act(w.x, (size_t) l.n_embd);
    take_act(w.h, (size_t) l.n_ff);
    w.hf = (float*) take(ne * l.n_ff * 4);
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
    if (!l || !expert_table || !x || !ids || !weights || !out || !workspace) return fail(MAYA_E_ARG, "prefill_layer: null pointer");
    if (n_tokens <= 0 || n_tokens > 8192 || k <= 0 || k > MAYA_MAX_K || (int64_t) n_tokens * k > 65535)
        return fail(MAYA_E_SHAPE, "prefill_layer: tokens %d k %d (at most 65535 entries a call)", n_tokens, k);
    if (((uintptr_t) workspace & 255) != 0) return fail(MAYA_E_ARG, "prefill_layer: workspace not 256-byte aligned");
    // everything a stage would refuse is refused here, before the first launch ("> 0: not covered, nothing launched")
    {
        DeviceState* st;
        if (const int rc0 = current_state(&st)) return rc0;
        if (n_expert <= 0 || n_expert > MAYA_MAX_EXPERTS || k > n_expert)
            return fail(MAYA_E_SHAPE, "prefill_layer: experts %d (1..%d) k %d", n_expert, MAYA_MAX_EXPERTS, k);
        if (x_dtype < 0 || x_dtype > 2 || out_dtype < 0 || out_dtype > 2) return fail(MAYA_E_UNSUPPORTED, "prefill_layer: dtypes %d / %d", x_dtype, out_dtype);
        maya_prefill_plan probe{};   // (the plan's pointers come from the workspace: only the layout's side is checked here)
        int32_t dummy = 0;
        probe.bounds = probe.row_entry = probe.entry_row = probe.tile_expert = probe.tile_row0 = probe.n_tiles = &dummy;
        if (const int rc0 = prefill_check("prefill_layer", l, expert_table, n_expert, &probe, n_tokens * k, l->gate_type, l->up_type, l->n_embd)) return rc0;
        if (const int rc0 = prefill_check("prefill_layer", l, expert_table, n_expert, &probe, n_tokens * k, l->down_type, l->down_type, l->n_ff)) return rc0;
        if (l->n_embd % 32) return fail(MAYA_E_SHAPE, "prefill_layer: n_embd %d", l->n_embd);
    }
    const PrefillWs w = prefill_carve(*l, n_tokens, k, n_expert, (uint8_t*) workspace);
    if (workspace_bytes < w.bytes) return fail(MAYA_E_ARG, "prefill_layer: workspace %zu < %zu bytes", workspace_bytes, w.bytes);
    const int ne = n_tokens * k;
    int rc;
    if (logits && (rc = maya_moe_route_topk(logits, n_tokens, n_expert, k, ids, weights, stream))) return rc;   // (null: ids / weights are given)
    if ((rc = maya_moe_prefill_plan(ids, ne, expert_table, n_expert, &w.plan, stream))) return rc;
    if ((rc = maya_moe_prefill_quant(x, x_dtype, 0, &w.plan, ne, n_expert, k, l->n_embd, w.x, stream))) return rc;
    if ((rc = maya_moe_prefill_gate_up(l, expert_table, n_expert, &w.plan, ne, w.x, limit, w.hf, w.h, stream))) return rc;
    if ((rc = maya_moe_prefill_down(l, expert_table, n_expert, &w.plan, ne, w.h, w.part, stream))) return rc;
    return maya_moe_prefill_combine(&w.plan, weights, w.part, n_tokens, k, l->n_embd, add, out, out_dtype, stream);
}

}  // extern "C"
