// maya_kernels.hip - gfx950 kernels of the routed-MoE expert block and their C ABI (include/maya_moe.h).
//
// Data layout in HBM: expert weights stay in their GGUF rows (row-major, [gate | up | down] per expert); activations
// are int8 codes with an F32 scale per 32 values (maya_act); routing state (ids, weights, plan, groups) lives in device
// arrays that only kernels read.  All kernels are HBM-bound integer work: a lane streams quantized blocks, expands them to
// int8 codes in registers (codebooks staged in LDS), takes exact v_dot4_i32_i8 sums against the int8 activation held in
// LDS and scales them in F32; rows are reduced across the lanes of a wavefront-64 with shuffles.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <math.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "maya_host.h"
#include "maya_iq_grids.h"

namespace maya {

// ------------------------------------------------------------------------------------------------ host state

thread_local char g_err[512] = "";
int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}
int hip_fail(hipError_t e, const char* what) {
    snprintf(g_err, sizeof g_err, "%s: %s", what, hipGetErrorString(e));
    return -(int) e;
}

constexpr int kMaxDevices = 16;
DeviceState g_dev[kMaxDevices];
std::mutex g_init_mu;

// The scratch of maya_moe_layer_decode_static, the layer call for callers that cannot allocate: a file-scope device array
// in place of the caller's workspace.  Every device the library runs on holds its own copy until the process ends; in host
// code the name is only a handle for hipGetSymbolAddress (done once a device in current_state), never an address to pass on.
static __device__ __align__(256) unsigned char scratch[MAYA_STATIC_SCRATCH_BYTES];

int current_state(DeviceState** out) {
    int dev = 0;
    MAYA_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(MAYA_E_NOGPU, "device ordinal %d outside 0..%d", dev, kMaxDevices - 1);
    DeviceState& s = g_dev[dev];
    if (!s.ready) {
        std::lock_guard<std::mutex> lock(g_init_mu);
        if (!s.ready) {
            hipDeviceProp_t p;
            MAYA_HIP(hipGetDeviceProperties(&p, dev));
            if (strncmp(p.gcnArchName, "gfx950", 6) != 0)
                return fail(MAYA_E_NOGPU, "device %d is %s; this library holds gfx950 code only", dev, p.gcnArchName);
            static const uint8_t m2[4] = {8, 25, 43, 0}, m1[4] = {0xff, 0x00, 0x01, 0};
            uint64_t* host = new uint64_t[1024 + 2048 + 256];
            for (int i = 0; i < 1024; ++i) {
                uint64_t v = 0;
                for (int j = 0; j < 8; ++j) v |= (uint64_t) m2[(maya_iq2s_packed[i] >> (2 * j)) & 3] << (8 * j);
                host[i] = v;
            }
            for (int i = 0; i < 2048; ++i) {
                uint64_t v = 0;
                for (int j = 0; j < 8; ++j) v |= (uint64_t) m1[(maya_iq1s_packed[i] >> (2 * j)) & 3] << (8 * j);
                host[1024 + i] = v;
            }
            for (int i = 0; i < 256; ++i) {
                uint64_t v = 0;
                for (int j = 0; j < 8; ++j) v |= (uint64_t) m2[(maya_iq2xxs_packed[i] >> (2 * j)) & 3] << (8 * j);
                host[1024 + 2048 + i] = v;
            }
            uint64_t* d = nullptr;
            hipError_t e = hipMalloc((void**) &d, sizeof(uint64_t) * (1024 + 2048 + 256));
            if (e == hipSuccess) e = hipMemcpy(d, host, sizeof(uint64_t) * (1024 + 2048 + 256), hipMemcpyHostToDevice);
            delete[] host;
            // (a step that fails gives back what the steps before it made: the next call starts over)
            auto undo = [&](hipError_t err, const char* what) {
                if (s.side_join) (void) hipEventDestroy(s.side_join);
                if (s.side_fork) (void) hipEventDestroy(s.side_fork);
                if (s.side) (void) hipStreamDestroy(s.side);
                s.side_join = s.side_fork = nullptr;
                s.side = nullptr;
                s.static_scratch = nullptr;
                if (d) (void) hipFree(d);
                return hip_fail(err, what);
            };
            if (e != hipSuccess) return undo(e, "codebook upload");
            void* sp = nullptr;
            e = hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch));   // (this device is the current one)
            if (e != hipSuccess || sp == nullptr) return undo(e == hipSuccess ? hipErrorInvalidSymbol : e, "address of the static scratch");
            s.static_scratch = sp;
            if ((e = hipStreamCreateWithFlags(&s.side, hipStreamNonBlocking)) != hipSuccess) return undo(e, "the shared expert's stream");
            if ((e = hipEventCreateWithFlags(&s.side_fork, hipEventDisableTiming)) != hipSuccess ||
                (e = hipEventCreateWithFlags(&s.side_join, hipEventDisableTiming)) != hipSuccess)
                return undo(e, "the shared expert's events");
            s.cb.iq2s = d;
            s.cb.iq1s = d + 1024;
            s.cb.iq2xxs = d + 1024 + 2048;
            s.lds_limit = (int) p.sharedMemPerBlock;
            s.n_cu = p.multiProcessorCount;
            s.ready = true;
        }
    }
    *out = &s;
    return MAYA_OK;
}


// ------------------------------------------------------------------------------------------------ dequantize
//
// One thread a value; the float steps are the reference decode's, each rounded once (no contraction), so the output is
// the block format's value to the bit.

template <int TYPE>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ w, size_t row_stride, int64_t k,
                                                      float* __restrict__ out, Codebooks cb, int packing) {
    const int64_t row = blockIdx.y;
    const int64_t v = (int64_t) blockIdx.x * 256 + threadIdx.x;  // value index in the row
    if (v >= k) return;
    const uint8_t* rp = w + (size_t) row * row_stride;
    float r;
    if constexpr (TYPE == kQ8_0) {
        if (packing == MAYA_PACK_STREAM) {   // a row = its k codes, then its k / 32 scales
            r = __fmul_rn((float) (int8_t) rp[v], f16_bits_to_f32(ld16(rp + k + 2 * (v >> 5))));
        } else {
            const uint8_t* blk = rp + (size_t) (v >> 5) * 34;
            r = __fmul_rn((float) (int8_t) blk[2 + (v & 31)], f16_bits_to_f32(ld16(blk)));
        }
    } else if constexpr (TYPE == kQ4_K) {
        const uint8_t* blk = rp + (size_t) (v >> 8) * 144;
        const int i = (int) (v & 255), j = i >> 5, l = i & 31;
        int sc, m;
        q4k_scale_min(blk + 4, j, sc, m);
        const float d1 = __fmul_rn(f16_bits_to_f32(ld16(blk)), (float) sc);
        const float m1 = __fmul_rn(f16_bits_to_f32(ld16(blk + 2)), (float) m);
        const uint8_t qb = blk[16 + 32 * (j >> 1) + l];
        const int q = (j & 1) ? (qb >> 4) : (qb & 15);
        r = __fsub_rn(__fmul_rn(d1, (float) q), m1);
    } else if constexpr (TYPE == kIQ2_S) {
        const int i = (int) (v & 255), ib = i >> 5, il = (i >> 3) & 3, j = i & 7;
        uint32_t qs, sg, h, sc, dbits;
        if (packing == MAYA_PACK_STREAM) {
            const int64_t nu = k >> 5, un = v >> 5, rq = row & 3;
            const uint8_t* quad = w + (size_t) (row >> 2) * 4 * row_stride;
            qs = quad[8 * (un * 4 + rq) + il];
            sg = quad[8 * (un * 4 + rq) + 4 + il];
            h = quad[32 * nu + 2 * (un * 4 + rq)];
            sc = quad[32 * nu + 2 * (un * 4 + rq) + 1];
            dbits = ld16(quad + 40 * nu + 2 * ((un >> 3) * 4 + rq));
        } else {
            const uint8_t* blk = rp + (size_t) (v >> 8) * 82;
            qs = blk[2 + 4 * ib + il];
            sg = blk[34 + 4 * ib + il];
            h = blk[66 + ib];
            sc = blk[74 + ib];
            dbits = ld16(blk);
        }
        const uint32_t idx = qs | ((h << (8 - 2 * il)) & 0x300u);
        const uint64_t g = cb.iq2s[idx];
        const int ls = (sc >> (4 * (il >> 1))) & 15;
        const float dl = __fmul_rn(__fmul_rn(f16_bits_to_f32(dbits), __fadd_rn(0.5f, (float) ls)), 0.25f);
        const float mag = __fmul_rn(dl, (float) (uint32_t) ((g >> (8 * j)) & 255u));
        r = (sg >> j) & 1 ? -mag : mag;
    } else if constexpr (TYPE == kIQ2_XXS) {
        const int i = (int) (v & 255), ib = i >> 5, il = (i >> 3) & 3, j = i & 7;
        const uint8_t* blk = rp + (size_t) (v >> 8) * 66;
        const uint32_t aux = ld32_a2(blk + 6 + 8 * ib);
        const uint64_t g = cb.iq2xxs[blk[2 + 8 * ib + il]];
        const uint32_t sg = Fmt<kIQ2_XXS>::signs8((aux >> (7 * il)) & 127u);
        const float dl = __fmul_rn(__fmul_rn(f16_bits_to_f32(ld16(blk)), __fadd_rn(0.5f, (float) (aux >> 28))), 0.25f);
        const float mag = __fmul_rn(dl, (float) (uint32_t) ((g >> (8 * j)) & 255u));
        r = (sg >> j) & 1 ? -mag : mag;
    } else if constexpr (TYPE == kIQ1_S) {
        const int i = (int) (v & 255), ib = i >> 5, il = (i >> 3) & 3, j = i & 7;
        uint32_t qs, qh, dbits;
        if (packing == MAYA_PACK_STREAM) {
            const int64_t nu = k >> 5, un = v >> 5, rq = row & 3;
            const uint8_t* quad = w + (size_t) (row >> 2) * 4 * row_stride;
            qs = quad[4 * (un * 4 + rq) + il];
            qh = ld16(quad + 16 * nu + 2 * (un * 4 + rq));
            dbits = ld16(quad + 24 * nu + 2 * ((un >> 3) * 4 + rq));
        } else {
            const uint8_t* blk = rp + (size_t) (v >> 8) * 50;
            qs = blk[2 + 4 * ib + il];
            qh = ld16(blk + 34 + 2 * ib);
            dbits = ld16(blk);
        }
        const uint64_t g = cb.iq1s[qs | (((qh >> (3 * il)) & 7u) << 8)];
        const float dl = __fmul_rn(f16_bits_to_f32(dbits), (float) (2 * (int) ((qh >> 12) & 7u) + 1));
        const float delta = (qh & 0x8000u) ? -0.125f : 0.125f;
        r = __fmul_rn(dl, __fadd_rn((float) (int8_t) ((g >> (8 * j)) & 255u), delta));
    } else {  // IQ1_M
        const int i = (int) (v & 255), ib = i >> 5, il = (i >> 3) & 3, j = i & 7;
        const int ib16 = 2 * ib + (il >> 1);
        uint32_t qs, nib;
        int s;
        float d;
        if (packing == MAYA_PACK_STREAM) {
            const int64_t nu = k >> 5, un = v >> 5, rq = row & 3;
            const uint8_t* quad = w + (size_t) (row >> 2) * 4 * row_stride;
            qs = quad[4 * (un * 4 + rq) + il];
            nib = (quad[16 * nu + 2 * (un * 4 + rq) + (il >> 1)] >> (4 * (il & 1))) & 15u;
            const uint8_t* rec = quad + 24 * nu + 8 * ((un >> 3) * 4 + rq);
            uint64_t r8 = 0;
            for (int b = 0; b < 8; ++b) r8 |= (uint64_t) rec[b] << (8 * b);
            s = (int) ((r8 >> (16 + 3 * ib16)) & 7u);
            d = f16_bits_to_f32((uint32_t) (r8 & 0xffffu));
        } else {
            const uint8_t* blk = rp + (size_t) (v >> 8) * 56;
            qs = blk[4 * ib + il];
            nib = (blk[32 + 2 * ib + (il >> 1)] >> (4 * (il & 1))) & 15u;
            s = (ld16(blk + 48 + 2 * (ib16 >> 2)) >> (3 * (ib16 & 3))) & 7;
            d = Fmt<kIQ1_M>::scale(blk) * 8.0f;  // scale() carries the 1/8 of the integer-code form
        }
        const uint64_t g = cb.iq1s[qs | ((nib & 7u) << 8)];
        const float dl = __fmul_rn(d, (float) (2 * s + 1));
        const float delta = (nib & 8u) ? -0.125f : 0.125f;
        r = __fmul_rn(dl, __fadd_rn((float) (int8_t) ((g >> (8 * j)) & 255u), delta));
    }
    out[(size_t) row * k + v] = r;
}

// ------------------------------------------------------------------------------------------------ stream packing

// IQ2_S rows between the GGUF block sequence and the stream order (rows in quads, fields regrouped); one thread a
// sub-block, grid (k/32 sub-blocks / 256, rows).  DIR 0: GGUF -> stream, 1: stream -> GGUF.  Every byte is written once.
template <int DIR>
__global__ __launch_bounds__(256) void repack_iq2s_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                          int64_t k, int64_t n_rows, size_t src_stride, size_t dst_stride) {
    src += blockIdx.z * src_stride, dst += blockIdx.z * dst_stride;   // blob blockIdx.z of a layer's experts
    const int64_t nu = k >> 5, rb = (k >> 8) * 82;
    const int64_t un = (int64_t) blockIdx.x * 256 + threadIdx.x, row = blockIdx.y;
    if (un >= nu) return;
    const int64_t b = un >> 3, rq = row & 3;
    const int ib = (int) (un & 7);
    const uint8_t* gs = src + row * rb + b * 82;              // GGUF side when DIR == 0
    uint8_t* gd = dst + row * rb + b * 82;                    // GGUF side when DIR == 1
    const uint8_t* qs = src + (row >> 2) * 4 * rb;            // stream side (the quad) when DIR == 1
    uint8_t* qd = dst + (row >> 2) * 4 * rb;                  // stream side when DIR == 0
    const int64_t o_is = 8 * (un * 4 + rq), o_hs = 32 * nu + 2 * (un * 4 + rq), o_d = 40 * nu + 2 * (b * 4 + rq);
    if (DIR == 0) {
        for (int i = 0; i < 4; ++i) qd[o_is + i] = gs[2 + 4 * ib + i];
        for (int i = 0; i < 4; ++i) qd[o_is + 4 + i] = gs[34 + 4 * ib + i];
        qd[o_hs] = gs[66 + ib];
        qd[o_hs + 1] = gs[74 + ib];
        if (ib == 0) {
            qd[o_d] = gs[0];
            qd[o_d + 1] = gs[1];
        }
    } else {
        for (int i = 0; i < 4; ++i) gd[2 + 4 * ib + i] = qs[o_is + i];
        for (int i = 0; i < 4; ++i) gd[34 + 4 * ib + i] = qs[o_is + 4 + i];
        gd[66 + ib] = qs[o_hs];
        gd[74 + ib] = qs[o_hs + 1];
        if (ib == 0) {
            gd[0] = qs[o_d];
            gd[1] = qs[o_d + 1];
        }
    }
}

// IQ1_S rows between the GGUF block sequence and the stream order (rows in quads: the sub-blocks' index words, then their
// qh words, then the block scales); one thread a sub-block, grid (k/32 sub-blocks / 256, rows).  DIR as above.
template <int DIR>
__global__ __launch_bounds__(256) void repack_iq1s_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                          int64_t k, int64_t n_rows, size_t src_stride, size_t dst_stride) {
    src += blockIdx.z * src_stride, dst += blockIdx.z * dst_stride;   // blob blockIdx.z of a layer's experts
    const int64_t nu = k >> 5, rb = (k >> 8) * 50;
    const int64_t un = (int64_t) blockIdx.x * 256 + threadIdx.x, row = blockIdx.y;
    if (un >= nu) return;
    const int64_t b = un >> 3, rq = row & 3;
    const int ib = (int) (un & 7);
    const uint8_t* g = (DIR == 0 ? src : dst) + row * rb + b * 50;          // the GGUF block
    const uint8_t* q = (DIR == 0 ? dst : src) + (row >> 2) * 4 * rb;        // the quad
    const int64_t o_i = 4 * (un * 4 + rq), o_h = 16 * nu + 2 * (un * 4 + rq), o_d = 24 * nu + 2 * (b * 4 + rq);
    uint8_t* gw = (uint8_t*) g;
    uint8_t* qw = (uint8_t*) q;
    if (DIR == 0) {
        for (int i = 0; i < 4; ++i) qw[o_i + i] = g[2 + 4 * ib + i];
        qw[o_h] = g[34 + 2 * ib], qw[o_h + 1] = g[35 + 2 * ib];
        if (ib == 0) qw[o_d] = g[0], qw[o_d + 1] = g[1];
    } else {
        for (int i = 0; i < 4; ++i) gw[2 + 4 * ib + i] = q[o_i + i];
        gw[34 + 2 * ib] = q[o_h], gw[35 + 2 * ib] = q[o_h + 1];
        if (ib == 0) gw[0] = q[o_d], gw[1] = q[o_d + 1];
    }
}

// IQ1_M rows likewise (quads: index words, qh words, then 8 bytes a (block, row): the block scale gathered from the top
// nibbles of the four scale words, and their 4 x 12 bits of 3-bit scales in order); one thread a sub-block.
template <int DIR>
__global__ __launch_bounds__(256) void repack_iq1m_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                          int64_t k, int64_t n_rows, size_t src_stride, size_t dst_stride) {
    src += blockIdx.z * src_stride, dst += blockIdx.z * dst_stride;   // blob blockIdx.z of a layer's experts
    const int64_t nu = k >> 5, rb = (k >> 8) * 56;
    const int64_t un = (int64_t) blockIdx.x * 256 + threadIdx.x, row = blockIdx.y;
    if (un >= nu) return;
    const int64_t b = un >> 3, rq = row & 3;
    const int ib = (int) (un & 7);
    const uint8_t* g = (DIR == 0 ? src : dst) + row * rb + b * 56;          // the GGUF block
    const uint8_t* q = (DIR == 0 ? dst : src) + (row >> 2) * 4 * rb;        // the quad
    const int64_t o_i = 4 * (un * 4 + rq), o_h = 16 * nu + 2 * (un * 4 + rq), o_s = 24 * nu + 8 * (b * 4 + rq);
    uint8_t* gw = (uint8_t*) g;
    uint8_t* qw = (uint8_t*) q;
    if (DIR == 0) {
        for (int i = 0; i < 4; ++i) qw[o_i + i] = g[4 * ib + i];
        qw[o_h] = g[32 + 2 * ib], qw[o_h + 1] = g[33 + 2 * ib];
        if (ib == 0) {
            uint64_t w[4];
            for (int i = 0; i < 4; ++i) w[i] = (uint64_t) ld16(g + 48 + 2 * i);
            const uint64_t d = (w[0] >> 12) | ((w[1] >> 8) & 0xf0u) | ((w[2] >> 4) & 0xf00u) | (w[3] & 0xf000u);
            const uint64_t rec = d | ((w[0] & 0xfffu) << 16) | ((w[1] & 0xfffu) << 28) | ((w[2] & 0xfffu) << 40) | ((w[3] & 0xfffu) << 52);
            for (int i = 0; i < 8; ++i) qw[o_s + i] = (uint8_t) (rec >> (8 * i));
        }
    } else {
        for (int i = 0; i < 4; ++i) gw[4 * ib + i] = q[o_i + i];
        gw[32 + 2 * ib] = q[o_h], gw[33 + 2 * ib] = q[o_h + 1];
        if (ib == 0) {
            uint64_t rec = 0;
            for (int i = 0; i < 8; ++i) rec |= (uint64_t) q[o_s + i] << (8 * i);
            const uint32_t d = (uint32_t) (rec & 0xffffu);
            for (int i = 0; i < 4; ++i) {
                const uint32_t w = (uint32_t) ((rec >> (16 + 12 * i)) & 0xfffu) | (((d >> (4 * i)) & 0xfu) << 12);
                gw[48 + 2 * i] = (uint8_t) w, gw[49 + 2 * i] = (uint8_t) (w >> 8);
            }
        }
    }
}

// Q8_0 rows between the GGUF block sequence (2-byte scale, 32 codes, ...) and the stream order (the row's codes, then its
// scales); one thread a block, grid (k/32 blocks / 256, rows).  DIR 0: GGUF -> stream, 1: stream -> GGUF.
template <int DIR>
__global__ __launch_bounds__(256) void repack_q80_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int64_t k,
                                                         int64_t n_rows, size_t src_stride, size_t dst_stride) {
    src += blockIdx.z * src_stride, dst += blockIdx.z * dst_stride;
    const int64_t nb = k >> 5, rb = nb * 34;
    const int64_t b = (int64_t) blockIdx.x * 256 + threadIdx.x, row = blockIdx.y;
    if (b >= nb || row >= n_rows) return;
    const uint16_t* g = (const uint16_t*) ((DIR == 0 ? src : dst) + row * rb + b * 34);          // the GGUF block
    const uint16_t* sq = (const uint16_t*) ((DIR == 0 ? dst : src) + row * rb + b * 32);         // the stream codes
    const uint16_t* sd = (const uint16_t*) ((DIR == 0 ? dst : src) + row * rb + k + b * 2);      // the stream scale
    if constexpr (DIR == 0) {
        *(uint16_t*) sd = g[0];
#pragma unroll
        for (int i = 0; i < 16; ++i) ((uint16_t*) sq)[i] = g[1 + i];
    } else {
        ((uint16_t*) g)[0] = *sd;
#pragma unroll
        for (int i = 0; i < 16; ++i) ((uint16_t*) g)[1 + i] = sq[i];
    }
}

// n bytes of blob blockIdx.z, 16 at a time where both sides are aligned
__global__ __launch_bounds__(256) void copy_bytes_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, size_t n,
                                                         size_t src_stride, size_t dst_stride) {
    src += blockIdx.z * src_stride, dst += blockIdx.z * dst_stride;
    const size_t i0 = (size_t) blockIdx.x * 256 + threadIdx.x, step = (size_t) gridDim.x * 256;
    if ((((uintptr_t) src | (uintptr_t) dst) & 15) == 0) {
        const size_t n16 = n >> 4;
        for (size_t i = i0; i < n16; i += step) ((uint4*) dst)[i] = ((const uint4*) src)[i];
        for (size_t i = (n16 << 4) + i0; i < n; i += step) dst[i] = src[i];
    } else {
        for (size_t i = i0; i < n; i += step) dst[i] = src[i];
    }
}

// ------------------------------------------------------------------------------------------------ activation quantizers

template <int DT> __device__ __forceinline__ float load_x(const void* x, int64_t i) {
    if constexpr (DT == MAYA_DT_F32) return ((const float*) x)[i];
    else if constexpr (DT == MAYA_DT_BF16) return bf16_bits_to_f32(((const uint16_t*) x)[i]);
    else return f16_bits_to_f32(((const uint16_t*) x)[i]);
}

// ggml's nearest_int: the magic-number round (ties to even) of a product already rounded to F32
__device__ __forceinline__ int nearest_int(float f) {
    const float v = __fadd_rn(f, 12582912.0f);
    return (__float_as_int(v) & 0x007fffff) - 0x00400000;
}

// Q8_K: one workgroup of 256 threads a 256-value block (src/kernels/cuda/quantize_act.cu:161-207).  The block's signed
// maximum is the value at the FIRST largest magnitude: the reduction keeps (|x|, index) and prefers the lower index.
// One 256-value block by the first 256 threads of a workgroup (j = the thread's value, active = j < 256); `sm` is
// 256 + 8 words of LDS.  EVERY thread of the workgroup calls it (it holds a workgroup barrier); whole waves are active
// or idle.
__device__ __forceinline__ void quant_q8k_block(float xv, int j, bool active, int* sm, const maya_act& out, size_t base) {
    float am = fabsf(xv);
    int ix = j;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float oa = __shfl_xor(am, o, kWave);
        const int oi = __shfl_xor(ix, o, kWave);
        if (oa > am || (oa == am && oi < ix)) {
            am = oa;
            ix = oi;
        }
    }
    float* s_x = (float*) sm;
    float* s_am = (float*) (sm + 256);
    int* s_ix = sm + 260;
    if (active) {
        s_x[j] = xv;
        if ((j & 63) == 0) {
            s_am[j >> 6] = am;
            s_ix[j >> 6] = ix;
        }
    }
    __syncthreads();
    if (!active) return;
    am = s_am[0];
    ix = s_ix[0];
#pragma unroll
    for (int w = 1; w < 4; ++w)
        if (s_am[w] > am) {  // later waves hold higher indices: only a strictly larger magnitude replaces
            am = s_am[w];
            ix = s_ix[w];
        }
    int q = 0;
    float d = 0.0f;
    if (am > 0.0f) {
        const float iscale = __fdiv_rn(-127.0f, s_x[ix]);
        q = min(127, nearest_int(__fmul_rn(iscale, xv)));
        d = __fdiv_rn(1.0f, iscale);
    }
    out.q[base + j] = (int8_t) q;
    int s = q;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) s += __shfl_xor(s, o, kWave);
    if ((j & 15) == 0) out.bsums[(base >> 4) + (j >> 4)] = (int16_t) s;
    if (j < 8) out.d[(base >> 5) + j] = d;
}

template <int DT>
__global__ __launch_bounds__(256) void quant_q8k_kernel(const void* __restrict__ x, int64_t x_stride, int64_t k,
                                                        maya_act out) {
    __shared__ int sm[264];
    const int row = blockIdx.y, b = blockIdx.x, j = threadIdx.x;
    const float xv = load_x<DT>(x, (int64_t) row * x_stride + (int64_t) b * 256 + j);
    quant_q8k_block(xv, j, true, sm, out, (size_t) row * k + (size_t) b * 256);
}

// Q8_0: 32-value blocks in the CPU expert path's rounding on x86 (ggml-cpu's quantize_row_q8_0 as the reference restates
// it, src/kernels/cpu/expert.cpp:92-130): d = amax / 127 kept as FP16 (65504 when larger), q = nearest-even(x * (127 / amax))
// with the product rounded to F32 first.  256 threads = 8 blocks.
template <int DT>
__global__ __launch_bounds__(256) void quant_q80_kernel(const void* __restrict__ x, int64_t x_stride, int64_t k,
                                                        maya_act out) {
    const int row = blockIdx.y, j = threadIdx.x;
    const int64_t v = (int64_t) blockIdx.x * 256 + j;
    const float xv = load_x<DT>(x, (int64_t) row * x_stride + v);
    float am = fabsf(xv);
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) am = fmaxf(am, __shfl_xor(am, o, kWave));
    const float d0 = __fdiv_rn(am, 127.0f);
    const bool big = d0 > 65504.0f;
    const float d = big ? 65504.0f : d0;
    const float inv = am == 0.0f ? 0.0f : big ? __fdiv_rn(1.0f, 65504.0f) : __fdiv_rn(127.0f, am);
    const int q = max(-128, min(127, (int) rintf(__fmul_rn(xv, inv))));
    const size_t base = (size_t) row * k + v;
    out.q[base] = (int8_t) q;
    int s = q;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) s += __shfl_xor(s, o, kWave);
    if ((j & 15) == 0) out.bsums[base >> 4] = (int16_t) s;
    if ((j & 31) == 0) out.d[base >> 5] = __half2float(__float2half_rn(d));
}

// per-32 int8 with an F32 scale: c = rint(x * (127 / amax)), d = amax / 127 (src/prefill/moe_fused_rdna4.cu:87-109)
template <int DT>
__global__ __launch_bounds__(256) void quant_i8x32_kernel(const void* __restrict__ x, int64_t x_stride,
                                                          const int32_t* __restrict__ row_idx, int64_t k,
                                                          int8_t* __restrict__ q, float* __restrict__ d) {
    const int row = blockIdx.y, j = threadIdx.x;
    const int64_t v = (int64_t) blockIdx.x * 256 + j;
    const int64_t src = row_idx ? row_idx[row] : row;
    const float xv = load_x<DT>(x, src * x_stride + v);
    float am = fabsf(xv);
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) am = fmaxf(am, __shfl_xor(am, o, kWave));
    const float inv = am > 0.0f ? __fdiv_rn(127.0f, am) : 0.0f;
    q[(size_t) row * k + v] = (int8_t) nearest_int(__fmul_rn(xv, inv));
    if ((j & 31) == 0) d[((size_t) row * k + v) >> 5] = __fdiv_rn(am, 127.0f);
}

// ------------------------------------------------------------------------------------------------ router

// One workgroup a token (src/kernels/cuda/router_top10.cu:68-187): the maximum (exact in any order), the exponentials in
// double in parallel, their sum ascending on one thread, p = (float)(ex * inv) with inv a float, the k largest p in the
// order k rounds of a strict-> arg-max with the lower index on ties would pick them, renormalisation by
// max(sum, 2^-14) in double.
struct alignas(16) RouterLds {
    double ex[MAYA_MAX_EXPERTS];
    float p[MAYA_MAX_EXPERTS];
    float rv[8];
    int ri[8];
    double sum;
    float w[MAYA_MAX_K];
    int id[MAYA_MAX_K];
    // (more than 256 experts) the threads' best keys, the k-th largest of them, the keys at or above it
    unsigned long long lb[256], thr, cand[MAYA_MAX_K * (MAYA_MAX_EXPERTS / 256)];
    int nc;
};
// The largest of a wave's values, in every lane's scalar copy: exchanges inside the rows of 16 lanes (lane ^ 1, lane ^ 2,
// the half-row and row mirrors), then lane 15 of a row to the next row and lane 31 to the upper half; lane 63 has it.
__device__ __forceinline__ int wave_max_i32(int v) {
    v = max(v, dpp_i<0xB1>(v));
    v = max(v, dpp_i<0x4E>(v));
    v = max(v, dpp_i<0x141>(v));
    v = max(v, dpp_i<0x140>(v));
    v = max(v, __builtin_amdgcn_update_dpp(v, v, 0x142, 0xa, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(v, v, 0x143, 0xc, 0xf, false));
    return __builtin_amdgcn_readlane(v, 63);
}

// Up to 256 experts, ONE wave, sm.ex filled: lane L keeps experts L, L + 64, L + 128, L + 192 in registers from the sum
// to the weights, so nothing but the result touches LDS and no workgroup barrier sits on the path.
//  * the sum: ascending, one add after the other (the reference's order).  The chain of dependent double adds is the
//    critical path, so every add takes its operand from a lane by v_readlane, eight fetched ahead; all lanes carry the sum.
//  * the k largest: k rounds of the reference's strict-> arg-max with the lower index on ties
//    (src/kernels/cuda/router_top10.cu:140-176).  Probabilities are non-negative, so their bit patterns order like the
//    values as signed integers and -1 marks "taken" or "no such expert"; a round is a 4-way maximum a lane, the wave
//    maximum, and the first lane (lowest expert: lower register first, then lower lane) that holds it.
//  * renormalisation: the k weights summed in slot order in double, one division a lane.
// (the token's exponentials already 4 a lane in ex; the wave's lane i < k returns slot i: its expert and weight.  `tab`:
// the residency table's entries of the lane's four experts, NULL when no plan is wanted; the slot's blob address then
// comes back in my_ptr - read from the chosen expert's lane, no second trip to memory.)
__device__ __forceinline__ void route_narrow_regs(int n_expert, int k, const double (&ex)[4], const uint64_t* tab, int& my_id,
                                                  float& my_weight, uint64_t& my_ptr) {
    const int lane = threadIdx.x & 63;
    int lo[4], hi[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        lo[r] = __double2loint(ex[r]);
        hi[r] = __double2hiint(ex[r]);
    }
    double sum = 0.0;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (64 * r < n_expert) {
#pragma unroll
            for (int j0 = 0; j0 < 64; j0 += 8) {
                int sl[8], sh[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    sl[j] = __builtin_amdgcn_readlane(lo[r], j0 + j);
                    sh[j] = __builtin_amdgcn_readlane(hi[r], j0 + j);
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) sum += __hiloint2double(sh[j], sl[j]);
            }
        }
    }
    const float inv = (float) (1.0 / sum);
    int key[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) key[r] = 64 * r + lane < n_expert ? __float_as_int((float) (ex[r] * (double) inv)) : -1;
    int id = 0, my_w = 0;
    uint64_t ptr = 0ull;
    for (int i = 0; i < k; ++i) {
        const int top = wave_max_i32(max(max(key[0], key[1]), max(key[2], key[3])));
        unsigned long long b = __ballot(key[0] == top);
        int r = 0;
        if (b == 0ull) b = __ballot(key[1] == top), r = 1;
        if (b == 0ull) b = __ballot(key[2] == top), r = 2;
        if (b == 0ull) b = __ballot(key[3] == top), r = 3;
        const int at = __builtin_amdgcn_readfirstlane(__builtin_ctzll(b));
#pragma unroll
        for (int q = 0; q < 4; ++q) key[q] = (q == r && lane == at) ? -1 : key[q];
        if (lane == i) id = 64 * r + at, my_w = top;
        if (tab) {
            const uint64_t tq = r == 0 ? tab[0] : r == 1 ? tab[1] : r == 2 ? tab[2] : tab[3];
            const uint32_t plo = (uint32_t) __builtin_amdgcn_readlane((int) (uint32_t) tq, at);
            const uint32_t phi = (uint32_t) __builtin_amdgcn_readlane((int) (uint32_t) (tq >> 32), at);
            if (lane == i) ptr = ((uint64_t) phi << 32) | plo;
        }
    }
    double s = 0.0;
    for (int i = 0; i < k; ++i) s += (double) __int_as_float(__builtin_amdgcn_readlane(my_w, i));
    const double sc = fmax(s, 6.103515625e-05);
    my_id = id;
    my_weight = (float) ((double) __int_as_float(my_w) / sc);
    my_ptr = ptr;
}
__device__ __forceinline__ void route_narrow(int n_expert, int k, RouterLds& sm) {
    const int lane = threadIdx.x;
    double ex[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int e = 64 * r + lane;
        ex[r] = e < n_expert ? sm.ex[e] : 0.0;   // (+0.0 past the end: adding it changes nothing)
    }
    int id;
    float w;
    uint64_t ptr;
    route_narrow_regs(n_expert, k, ex, nullptr, id, w, ptr);
    if (lane < k) {
        sm.id[lane] = id;
        sm.w[lane] = w;
    }
}

// The k largest of n_expert 64-bit keys (a value's ordered bits above the complemented index, so "beats" is one unsigned
// compare and equal values rank by the lower index) into sm.id / sm.w (= sm.p of the expert), 256 threads.  Ranking every
// expert against every other grows with the square.  The k-th largest of the threads' best keys is a lower bound of the
// k-th largest key overall (those are k different experts), so only keys at or above it can be among the k largest, and
// every key that beats one of them is at or above it too: the few candidates (at most k threads' experts) are ranked
// among themselves.
__device__ __forceinline__ void topk_by_keys(const unsigned long long* key, int n_expert, int k, RouterLds& sm) {
    const int tid = threadIdx.x;
    unsigned long long best = 0ull;
    for (int e = tid; e < n_expert; e += 256) best = key[e] > best ? key[e] : best;
    sm.lb[tid] = best;
    if (tid == 0) sm.nc = 0;
    __syncthreads();
    int rank = 0;
    for (int j = 0; j < 256; j += 2) {
        const ulonglong2 kj = *(const ulonglong2*) (sm.lb + j);
        rank += kj.x > best ? 1 : 0;
        rank += kj.y > best ? 1 : 0;
    }
    if (rank == k - 1) sm.thr = best;
    __syncthreads();
    const unsigned long long thr = sm.thr;
    for (int e = tid; e < n_expert; e += 256)
        if (key[e] >= thr) sm.cand[atomicAdd(&sm.nc, 1)] = key[e];
    __syncthreads();
    const int nc = sm.nc;
    if (tid < nc) {
        const unsigned long long kc = sm.cand[tid];
        int r = 0;
        for (int j = 0; j < nc; ++j) r += sm.cand[j] > kc ? 1 : 0;
        if (r < k) {
            const int e = (int) (0xffffffffu - (unsigned) (kc & 0xffffffffull));
            sm.id[r] = e;
            sm.w[r] = sm.p[e];
        }
    }
}

// NTH threads (256, or a workgroup of 512 with up to 256 experts); on return sm.id / sm.w hold the token's k experts and
// renormalised weights
template <int NTH = 256>
__device__ __forceinline__ void route_token(const float* __restrict__ l, int n_expert, int k, RouterLds& sm) {
    const int tid = threadIdx.x;
    float mx = -INFINITY;
    for (int e = tid; e < n_expert; e += NTH) mx = fmaxf(mx, l[e]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, kWave));
    if ((tid & 63) == 0) sm.rv[tid >> 6] = mx;
    __syncthreads();
    mx = sm.rv[0];
#pragma unroll
    for (int w = 1; w < NTH / 64; ++w) mx = fmaxf(mx, sm.rv[w]);   // (the maximum is exact in any order)
    __syncthreads();
    for (int e = tid; e < n_expert; e += NTH) sm.ex[e] = exp((double) l[e] - (double) mx);
    __syncthreads();
    if (n_expert <= 256 || NTH != 256) {   // (wider workgroups are only given up to 256 experts)
        if (tid < 64) route_narrow(n_expert, k, sm);
        __syncthreads();
        return;
    }
    if (tid < 64) {
        // ascending, one add after the other (the reference's order).  The chain of dependent double adds is the router's
        // critical path, so nothing else may sit on it: the first wave pulls the values into registers (lane L holds
        // experts L, L + 64, ...), then every add takes its operand from a lane by v_readlane (scalar registers, no
        // memory wait); all lanes carry the same sum.
        double sum = 0.0;
        for (int r0 = 0; r0 < n_expert; r0 += 256) {
            int lo[4], hi[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int e = r0 + 64 * r + tid;
                const double v = e < n_expert ? sm.ex[e] : 0.0;   // (+0.0 past the end: adding it changes nothing)
                lo[r] = __double2loint(v);
                hi[r] = __double2hiint(v);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (r0 + 64 * r < n_expert) {
#pragma unroll
                    for (int j0 = 0; j0 < 64; j0 += 8) {   // eight operands fetched ahead of the eight adds that use them
                        int sl[8], sh[8];
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            sl[j] = __builtin_amdgcn_readlane(lo[r], j0 + j);
                            sh[j] = __builtin_amdgcn_readlane(hi[r], j0 + j);
                        }
#pragma unroll
                        for (int j = 0; j < 8; ++j) sum += __hiloint2double(sh[j], sl[j]);
                    }
                }
            }
        }
        if (tid == 0) sm.sum = sum;
    }
    __syncthreads();
    const float inv = (float) (1.0 / sm.sum);
    for (int e = tid; e < n_expert; e += 256) sm.p[e] = (float) (sm.ex[e] * (double) inv);
    __syncthreads();
    // More than 256 experts: the k largest by rank.  Expert e's rank = the experts that beat it (a larger probability -
    // they are non-negative, so their bit patterns order like the values - or an equal one at a lower index): exactly
    // the order in which k rounds of a strict-> arg-max with the lower index on ties would pick them
    // (src/kernels/cuda/router_top10.cu:140-176).  64-bit keys, probability bits above the complemented index, make
    // "beats" one unsigned compare; they take the place of the exponentials, which are no longer needed.
    unsigned long long* key = (unsigned long long*) sm.ex;
    for (int e = tid; e < n_expert; e += 256)
        key[e] = ((unsigned long long) __float_as_uint(sm.p[e]) << 32) | (unsigned long long) (0xffffffffu - (unsigned) e);
    __syncthreads();
    topk_by_keys(key, n_expert, k, sm);
    __syncthreads();
    if (tid < 64) {
        // renormalisation: the sum of the k weights in slot order in double, one division a lane
        double s = 0.0;
        for (int i = 0; i < k; ++i) s += (double) sm.w[i];
        const double sc = fmax(s, 6.103515625e-05);
        __builtin_amdgcn_wave_barrier();
        if (tid < k) sm.w[tid] = (float) ((double) sm.w[tid] / sc);
    }
    __syncthreads();
}

// ---- the sigmoid router of the GLM / DeepSeek-V3 family (src/kernels/cuda/router_sigmoid.cu:44-73; moe_route_kernel,
// src/kernels/cuda/glm_fast.cu:4050-4056, 4214, 4297): p = 1 / (1 + expf(-logit)) in float, the selection score p + bias
// (the bias chooses, it does not weigh), stable top-k, the chosen p summed in rank order in double,
// w = (float)((double) p * inv * w_scale) with inv a float: 1 / max(sum, 2^-14) (norm 1), 1 / (sum + 1e-20) (norm 2), 1.
struct RouterSpec {
    const float* bias;   // [n_expert] or null (sigmoid only)
    float w_scale;
    int kind;            // MAYA_ROUTER_SOFTMAX, MAYA_ROUTER_SIGMOID
    int norm;
};
// a float's bits as a signed integer that orders like the float (no -0.0 arises: p > 0 and p + bias = 0 rounds to +0.0)
__device__ __forceinline__ int float_order_key(float v) {
    const int b = __float_as_int(v);
    return b >= 0 ? b : b ^ 0x7fffffff;
}
// one wave, up to 256 experts, sm.p and the scores (sm.ex's storage, as floats) filled; on return lane i < k holds slot i
__device__ __forceinline__ void sigmoid_narrow(int n_expert, int k, const RouterSpec& r, RouterLds& sm) {
    const int lane = threadIdx.x;
    const float* sel = (const float*) sm.ex;
    constexpr int kNone = (int) 0x80000000;   // below every key: a taken expert, or none at this index
    int key[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) key[q] = 64 * q + lane < n_expert ? float_order_key(sel[64 * q + lane]) : kNone;
    int my_id = 0;
    for (int i = 0; i < k; ++i) {
        const int top = wave_max_i32(max(max(key[0], key[1]), max(key[2], key[3])));
        unsigned long long b = __ballot(key[0] == top);
        int q = 0;
        if (b == 0ull) b = __ballot(key[1] == top), q = 1;
        if (b == 0ull) b = __ballot(key[2] == top), q = 2;
        if (b == 0ull) b = __ballot(key[3] == top), q = 3;
        const int at = __builtin_ctzll(b);
#pragma unroll
        for (int j = 0; j < 4; ++j) key[j] = (j == q && lane == at) ? kNone : key[j];
        if (lane == i) my_id = 64 * q + at;
    }
    if (lane < k) sm.id[lane] = my_id;
}
// NTH threads (as route_token); on return sm.id / sm.w hold the token's k experts and weights
template <int NTH = 256>
__device__ __forceinline__ void route_token_sigmoid(const float* __restrict__ l, int n_expert, int k, const RouterSpec& r, RouterLds& sm) {
    const int tid = threadIdx.x;
    float* sel = (float*) sm.ex;
    int bad = 0;
    for (int e = tid; e < n_expert; e += NTH) {
        const float le = l[e];
        const float p = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf(-le)));
        const float sc = r.bias ? __fadd_rn(p, r.bias[e]) : p;
        sm.p[e] = p;
        sel[e] = sc;
        bad |= !isfinite(le) || !isfinite(sc);
    }
    // a row with a non-finite logit or score is refused: no routes (the engine's routers,
    // src/kernels/cuda/glm_batch.cu:2077-2092, glm_fast.cu:4040); it is still ranked below, its picks unused
    bad = __syncthreads_or(bad);
    if (n_expert <= 256 || NTH != 256) {
        if (tid < 64) sigmoid_narrow(n_expert, k, r, sm);
    } else {
        // (the scores' ordered bits, offset to unsigned, above the complemented index; the keys take the scores' place)
        float v[MAYA_MAX_EXPERTS / 256];
#pragma unroll
        for (int i = 0; i < MAYA_MAX_EXPERTS / 256; ++i) v[i] = tid + 256 * i < n_expert ? sel[tid + 256 * i] : 0.0f;
        __syncthreads();
        unsigned long long* key = (unsigned long long*) sm.ex;
#pragma unroll
        for (int i = 0; i < MAYA_MAX_EXPERTS / 256; ++i) {
            const int e = tid + 256 * i;
            if (e < n_expert)
                key[e] = ((unsigned long long) ((unsigned) float_order_key(v[i]) ^ 0x80000000u) << 32) | (unsigned long long) (0xffffffffu - (unsigned) e);
        }
        __syncthreads();
        topk_by_keys(key, n_expert, k, sm);
    }
    __syncthreads();
    if (tid < 64) {
        const float p = tid < k ? sm.p[sm.id[tid]] : 0.0f;
        double s = 0.0;
        for (int i = 0; i < k; ++i) s += (double) __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), i));
        const float inv = (float) (r.norm == 0 ? 1.0 : r.norm == 2 ? 1.0 / (s + 1e-20) : 1.0 / fmax(s, 6.103515625e-05));
        if (tid < k) {
            sm.w[tid] = bad ? 0.0f : (float) ((double) p * (double) inv * (double) r.w_scale);
            if (bad) sm.id[tid] = -1;
        }
    }
    __syncthreads();
}
template <int NTH = 256>
__device__ __forceinline__ void route_any(const float* __restrict__ l, int n_expert, int k, const RouterSpec& r, RouterLds& sm) {
    if (r.kind == MAYA_ROUTER_SIGMOID) route_token_sigmoid<NTH>(l, n_expert, k, r, sm);
    else route_token<NTH>(l, n_expert, k, sm);
}

// The softmax router on ONE wave, nothing but registers (up to 256 experts, 4 a lane: lane L holds experts L, L + 64, ...;
// lv = -inf and tab = 0 past the end): the maximum, the exponentials, then route_narrow_regs.  Lane i < k returns slot i.
__device__ __forceinline__ void route_wave_softmax(const float (&lv)[4], const uint64_t (&tab)[4], int n_expert, int k, int& id,
                                                   float& w, uint64_t& ptr) {
    const int lane = threadIdx.x & 63;
    float mx = fmaxf(fmaxf(lv[0], lv[1]), fmaxf(lv[2], lv[3]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, kWave));
    double ex[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) ex[r] = 64 * r + lane < n_expert ? exp((double) lv[r] - (double) mx) : 0.0;
    route_narrow_regs(n_expert, k, ex, tab, id, w, ptr);
}

// Which k experts the softmax router picks, and in which order, WITHOUT the probabilities: p = exp(l - max) / sum grows
// with the logit, so the k largest logits in descending order are the k largest probabilities in descending order as long
// as rounding cannot merge or reorder two of them.  Two logits more than 1e-6 apart give probabilities whose ratio
// exceeds 1 + 1e-6, far beyond the 2^-24 relative rounding of a float, and a probability within e^-60 of the largest
// is a normal float.  So: every logit finite, each pick more than 1e-6 above the next, the k-th more than 1e-6 above
// everything not picked, and all of that within 60 of the first - then the picks and their order are the exact router's.
// Anything else (ties, near ties, the sub-normal range, NaN / Inf) returns false and the caller runs the exact router.
//
// A round must be short (k + 1 of them run one after the other on one wave while its workgroup waits), so a key is one
// word that names its expert: the logit's ordered bits with the low byte replaced by 255 - index.  The largest key of
// the wave IS the pick, with no search for the lane that holds it.  The 8 bits given up make picks inside one
// 256-ulp bucket come out in index order: the check below therefore compares the picks' TRUE logits (a wrong order
// shows as a negative gap), and holds the k-th pick against the upper end of the (k + 1)-th pick's bucket, above which
// nothing unpicked can lie.  One wave, k < n_expert <= 256, k + 1 <= 64; s_lv [256] floats of LDS scratch; lane i < k
// gets slot i's expert.
// (The sigmoid router picks by the score p + bias itself, so its keys ARE the exact router's: margin 0 - any strictly
// descending order is the router's - and no range to keep; `fin` then says that no logit and no score is non-finite.)
__device__ __forceinline__ bool route_wave_order_only(const float (&lv)[4], bool fin, int n_expert, int k, float* s_lv, float margin,
                                                      float range, int& my_id) {
    const int lane = threadIdx.x & 63;
    constexpr int kNone = (int) 0x80000000;
    int k0, k1, k2, k3;
    {
        int key[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int e = 64 * r + lane;
            const bool have = e < n_expert;
            key[r] = have ? (int) (((uint32_t) float_order_key(lv[r]) & 0xffffff00u) | (uint32_t) (255 - e)) : kNone;
            fin = fin && (!have || isfinite(lv[r]));
            s_lv[e] = lv[r];
        }
        k0 = key[0], k1 = key[1], k2 = key[2], k3 = key[3];
    }
    int my_key = kNone;
    for (int i = 0; i <= k; ++i) {
        const int top = wave_max_i32(max(max(k0, k1), max(k2, k3)));
        k0 = k0 == top ? kNone : k0;
        k1 = k1 == top ? kNone : k1;
        k2 = k2 == top ? kNone : k2;
        k3 = k3 == top ? kNone : k3;
        my_key = lane == i ? top : my_key;
    }
    const int id = 255 - (my_key & 255);
    const float val = lane <= k ? s_lv[id] : 0.0f;
    const int ub_key = my_key | 255;
    const float ub = __int_as_float(ub_key >= 0 ? ub_key : ub_key ^ 0x7fffffff);   // the bucket's upper end
    const float nxt = __shfl_down(lane == k ? ub : val, 1, kWave);
    const float first = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(val), 0));
    const bool apart = lane >= k || (val - nxt > margin && first - nxt <= range);
    my_id = id;
    return __all(fin && apart) != 0;
}

// The sigmoid router on ONE wave, nothing but registers (route_token_sigmoid's arithmetic; up to 256 experts, 4 a lane:
// lv / bv / tab of experts L, L + 64, ...; bv all zero without a bias).  sc: the lane's four scores p + bias as the
// caller already made them with sigmoid_scores (the same instructions, so the same bits).  Lane i < k returns slot i; a
// row with a non-finite logit or score returns id -1, weight 0, no blob.
__device__ __forceinline__ bool sigmoid_scores(const float (&lv)[4], const float (&bv)[4], bool has_bias, int n_expert, float (&p)[4],
                                               float (&sc)[4]) {
    const int lane = threadIdx.x & 63;
    bool fin = true;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const bool have = 64 * r + lane < n_expert;
        const float le = have ? lv[r] : 0.0f;
        p[r] = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf(-le)));
        sc[r] = has_bias ? __fadd_rn(p[r], bv[r]) : p[r];
        fin = fin && (!have || (isfinite(le) && isfinite(sc[r])));
    }
    return fin;
}
__device__ __forceinline__ void route_wave_sigmoid(const float (&p)[4], const float (&sc)[4], bool fin, const uint64_t (&tab)[4], int n_expert,
                                                   int k, int norm, float w_scale, int& my_id, float& my_w, uint64_t& my_ptr) {
    const int lane = threadIdx.x & 63;
    constexpr int kNone = (int) 0x80000000;
    const bool bad = __any(!fin) != 0;
    // (named copies: a select among array elements invites the compiler to index the array in memory)
    const uint64_t t0 = tab[0], t1 = tab[1], t2 = tab[2], t3 = tab[3];
    const float p0 = p[0], p1 = p[1], p2 = p[2], p3 = p[3];
    int k0 = lane < n_expert ? float_order_key(sc[0]) : kNone, k1 = 64 + lane < n_expert ? float_order_key(sc[1]) : kNone;
    int k2 = 128 + lane < n_expert ? float_order_key(sc[2]) : kNone, k3 = 192 + lane < n_expert ? float_order_key(sc[3]) : kNone;
    int id = 0;
    float pw = 0.0f;
    uint64_t ptr = 0ull;
    for (int i = 0; i < k; ++i) {
        const int top = wave_max_i32(max(max(k0, k1), max(k2, k3)));
        unsigned long long b = __ballot(k0 == top);
        int q = 0;
        if (b == 0ull) b = __ballot(k1 == top), q = 1;
        if (b == 0ull) b = __ballot(k2 == top), q = 2;
        if (b == 0ull) b = __ballot(k3 == top), q = 3;
        const int at = __builtin_amdgcn_readfirstlane(__builtin_ctzll(b));
        const bool hit = lane == at;
        k0 = hit && q == 0 ? kNone : k0;
        k1 = hit && q == 1 ? kNone : k1;
        k2 = hit && q == 2 ? kNone : k2;
        k3 = hit && q == 3 ? kNone : k3;
        const float pq = q == 0 ? p0 : q == 1 ? p1 : q == 2 ? p2 : p3;
        const uint64_t tq = q == 0 ? t0 : q == 1 ? t1 : q == 2 ? t2 : t3;
        const float pv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(pq), at));
        const uint32_t plo = (uint32_t) __builtin_amdgcn_readlane((int) (uint32_t) tq, at);
        const uint32_t phi = (uint32_t) __builtin_amdgcn_readlane((int) (uint32_t) (tq >> 32), at);
        if (lane == i) id = 64 * q + at, pw = pv, ptr = ((uint64_t) phi << 32) | plo;
    }
    double s = 0.0;
    for (int i = 0; i < k; ++i) s += (double) __int_as_float(__builtin_amdgcn_readlane(__float_as_int(pw), i));
    const float inv = (float) (norm == 0 ? 1.0 : norm == 2 ? 1.0 / (s + 1e-20) : 1.0 / fmax(s, 6.103515625e-05));
    my_id = bad ? -1 : id;
    my_w = bad ? 0.0f : (float) ((double) pw * (double) inv * (double) w_scale);
    my_ptr = bad ? 0ull : ptr;
}

__global__ __launch_bounds__(256) void router_kernel(const float* __restrict__ logits, int n_expert, int k, RouterSpec r,
                                                     int32_t* __restrict__ ids, float* __restrict__ weights) {
    __shared__ RouterLds sm;
    const int t = blockIdx.x;
    route_any(logits + (size_t) t * n_expert, n_expert, k, r, sm);
    if (threadIdx.x < k) {
        ids[(size_t) t * k + threadIdx.x] = sm.id[threadIdx.x];
        weights[(size_t) t * k + threadIdx.x] = sm.w[threadIdx.x];
    }
}

// The layer's head in one launch, grid (1 + n_embd / 256, n_tokens): workgroup 0 of a token routes it, writes its
// plan slots (blob addresses from the residency table); the other workgroups round one 256-value block of the hidden
// state each to Q8_K.
template <int DT>
__global__ __launch_bounds__(256) void layer_head_kernel(const float* __restrict__ logits, int n_expert, int k, RouterSpec rs,
                                                         const uint64_t* __restrict__ table, int32_t* __restrict__ ids,
                                                         float* __restrict__ weights, uint64_t* __restrict__ plan,
                                                         const void* __restrict__ x, int64_t n_embd, maya_act xq) {
    __shared__ RouterLds sm;
    __shared__ int qs[264];
    __shared__ uint64_t s_table[MAYA_MAX_EXPERTS];
    const int t = blockIdx.y;
    if (blockIdx.x == 0) {
        // the residency table rides along in registers while the token is routed: the plan's look-up then costs no second
        // trip to memory after the ids are known
        uint64_t tab[MAYA_MAX_EXPERTS / 256];
#pragma unroll
        for (int i = 0; i < MAYA_MAX_EXPERTS / 256; ++i) {
            const int e = threadIdx.x + 256 * i;
            tab[i] = e < n_expert ? table[e] : 0ull;
        }
        route_any(logits + (size_t) t * n_expert, n_expert, k, rs, sm);
#pragma unroll
        for (int i = 0; i < MAYA_MAX_EXPERTS / 256; ++i) s_table[threadIdx.x + 256 * i] = tab[i];
        __syncthreads();
        if (threadIdx.x < k) {
            const int id = sm.id[threadIdx.x];
            ids[(size_t) t * k + threadIdx.x] = id;
            weights[(size_t) t * k + threadIdx.x] = sm.w[threadIdx.x];
            plan[(size_t) t * k + threadIdx.x] = (id >= 0 && id < n_expert) ? s_table[id] : 0ull;
        }
    } else {
        const int b = blockIdx.x - 1, j = threadIdx.x;
        const float xv = load_x<DT>(x, (int64_t) t * n_embd + (int64_t) b * 256 + j);
        quant_q8k_block(xv, j, true, qs, xq, (size_t) t * n_embd + (size_t) b * 256);
    }
}

__global__ void plan_kernel(const int32_t* __restrict__ ids, int n, const uint64_t* __restrict__ table, int n_expert,
                            uint64_t* __restrict__ plan) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    const int id = ids[e];
    plan[e] = (id >= 0 && id < n_expert) ? table[id] : 0ull;
}

// Groups of distinct experts in first-appearance order, a group's entries ascending (what the reference's one-thread
// grouping produces, src/kernels/cuda/glm_fast.cu:7545-7590).  n <= 256 entries: one workgroup, entry e's thread finds the
// first entry with its blob (its group's leader); leaders are ranked by a prefix count; members are ranked inside their
// group the same way.  Entries with a null blob belong to no group.
struct GroupLds {
    uint64_t ptr[256];
    int leader[256];   // the first entry with the same blob, -1 for a null blob
    int gidx[256];     // leader entry -> group index
    int count[256];    // group -> entries
    int start[257];
    int ng;
};
// 256 threads, g.ptr[0 .. n) filled (and a barrier passed); thread e = entry e
__device__ __forceinline__ void group_entries(GroupLds& g, int n, uint64_t* __restrict__ grp_ptr, int32_t* __restrict__ grp_start,
                                              int32_t* __restrict__ grp_ent, int32_t* __restrict__ n_groups) {
    const int e = threadIdx.x;
    if (n <= 64) {
        // Up to 64 entries: one wave, registers only.  A lane learns which lanes hold its blob (n reads of a lane's value),
        // and everything else is a count of bits: its group's leader (the first such lane), its rank in the group, the
        // groups before its own (leaders below its leader), the entries before its group (lanes whose leader is below its
        // own).  The same groups, order and members as the general form below, value for value.
        if (e >= 64) return;
        const uint64_t ptr = e < n ? g.ptr[e] : 0ull;
        const uint32_t plo = (uint32_t) ptr, phi = (uint32_t) (ptr >> 32);
        unsigned long long same = 0ull;
        for (int f = 0; f < n; ++f) {
            const uint32_t flo = (uint32_t) __builtin_amdgcn_readlane((int) plo, f), fhi = (uint32_t) __builtin_amdgcn_readlane((int) phi, f);
            if (flo == plo && fhi == phi) same |= 1ull << f;
        }
        const bool valid = ptr != 0ull;
        if (!valid) same = 0ull;
        const int leader = valid ? __builtin_ctzll(same) : -1;
        const unsigned long long below = (1ull << e) - 1ull;
        const int rank = __popcll(same & below);
        const unsigned long long leaders = __ballot(leader == e);
        const int gi = valid ? __popcll(leaders & ((1ull << leader) - 1ull)) : -1;
        const int ng = __popcll(leaders);
        int start = 0;
        for (int f = 0; f < n; ++f) {
            const int lf = __builtin_amdgcn_readlane(leader, f);
            start += (lf >= 0 && lf < leader) ? 1 : 0;
        }
        const int total = __popcll(__ballot(valid));
        if (leader == e) {
            grp_ptr[gi] = ptr;
            grp_start[gi] = start;
        }
        if (e == 0) {
            grp_start[ng] = total;
            *n_groups = ng;
        }
        if (valid) grp_ent[start + rank] = e;
        if (e >= total && e < n) grp_ent[e] = -1;
        return;
    }
    g.count[e] = 0;
    int leader = -1;
    if (e < n && g.ptr[e] != 0ull) {
        leader = e;
        for (int f = 0; f < e; ++f)
            if (g.ptr[f] == g.ptr[e]) {
                leader = f;
                break;
            }
    }
    g.leader[e] = leader;
    __syncthreads();
    if (leader == e) {
        int gi = 0;
        for (int f = 0; f < e; ++f) gi += g.leader[f] == f;
        g.gidx[e] = gi;
    }
    __syncthreads();
    int rank = 0, gi = -1;
    if (leader >= 0) {
        gi = g.gidx[leader];
        for (int f = 0; f < e; ++f) rank += g.leader[f] == leader;
        atomicAdd(&g.count[gi], 1);
        if (leader == e) grp_ptr[gi] = g.ptr[e];
    }
    __syncthreads();
    if (e == 0) {
        int ng = 0, acc = 0;
        for (int f = 0; f < n; ++f) ng += g.leader[f] == f;
        for (int i = 0; i < ng; ++i) {
            g.start[i] = acc;
            acc += g.count[i];
        }
        g.start[ng] = acc;
        *n_groups = ng;
        g.ng = ng;
    }
    __syncthreads();
    const int ng = g.ng;
    if (e <= ng) grp_start[e] = g.start[e];
    if (gi >= 0) grp_ent[g.start[gi] + rank] = e;
    // (past the grouped entries: -1, so that grp_ent read as a list of length n says where it ends)
    if (e >= g.start[ng] && e < n) grp_ent[e] = -1;
}
__global__ __launch_bounds__(256) void group_kernel(const uint64_t* __restrict__ plan, int n,
                                                    uint64_t* __restrict__ grp_ptr, int32_t* __restrict__ grp_start,
                                                    int32_t* __restrict__ grp_ent, int32_t* __restrict__ n_groups) {
    __shared__ GroupLds g;
    const int e = threadIdx.x;
    g.ptr[e] = e < n ? plan[e] : 0ull;
    __syncthreads();
    group_entries(g, n, grp_ptr, grp_start, grp_ent, n_groups);
}

// A window's head in ONE launch (2 ... 16 tokens, the softmax router, up to 256 experts), grid (1 + n_embd / 256, tokens):
// workgroup (0, 0) routes every token - a wave a token, the token's experts 4 a lane, nothing but registers: the
// maximum, the exponentials, then route_narrow_regs - writes ids / weights / plan and groups the plan itself
// (group_kernel's arithmetic), so a window needs no grouping launch; the workgroups (b >= 1, t) round x like
// layer_head_kernel's.  x NULL: routing only, grid (1, 1).
template <int DT>
__global__ __launch_bounds__(256) void window_head_kernel(const float* __restrict__ logits, int n_expert, int k, int n_tokens,
                                                          const uint64_t* __restrict__ table, int32_t* __restrict__ ids,
                                                          float* __restrict__ weights, uint64_t* __restrict__ plan,
                                                          uint64_t* __restrict__ grp_ptr, int32_t* __restrict__ grp_start,
                                                          int32_t* __restrict__ grp_ent, int32_t* __restrict__ n_groups,
                                                          const void* __restrict__ x, int64_t n_embd, maya_act xq) {
    __shared__ GroupLds g;
    __shared__ int qs[264];
    if (blockIdx.x == 0) {
        if (blockIdx.y != 0) return;
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
        for (int t = wave; t < n_tokens; t += 4) {
            const float* l = logits + (size_t) t * n_expert;
            float lv[4];
            uint64_t tab[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int e = 64 * r + lane;
                lv[r] = e < n_expert ? l[e] : -INFINITY;
                tab[r] = e < n_expert ? table[e] : 0ull;
            }
            int id;
            float w;
            uint64_t ptr;
            route_wave_softmax(lv, tab, n_expert, k, id, w, ptr);
            if (lane < k) {
                ids[(size_t) t * k + lane] = id;
                weights[(size_t) t * k + lane] = w;
                plan[(size_t) t * k + lane] = ptr;
                g.ptr[t * k + lane] = ptr;
            }
        }
        const int n = n_tokens * k;
        if ((int) threadIdx.x >= n) g.ptr[threadIdx.x] = 0ull;
        __syncthreads();
        group_entries(g, n, grp_ptr, grp_start, grp_ent, n_groups);
    } else {
        const int t = blockIdx.y, b = blockIdx.x - 1, j = threadIdx.x;
        const float xv = load_x<DT>(x, (int64_t) t * n_embd + (int64_t) b * 256 + j);
        quant_q8k_block(xv, j, true, qs, xq, (size_t) t * n_embd + (size_t) b * 256);
    }
}

// ------------------------------------------------------------------------------------------------ expert rows

// the types whose stream packing groups rows in quads
__host__ __device__ constexpr bool quad_packed(int t) { return t == kIQ2_S || t == kIQ1_S || t == kIQ1_M; }

// LDS view of up to NT staged activation rows of k values
struct ActLds {
    const int* q;          // [NT][k/4]
    const float* d;        // [NT][k/32]
    const int* bs2;        // [NT][k/32] pairs of int16 bsums as one word (Q4_K only)
    int kq, kd;            // strides in words: k/4, k/32
};

// One row against NT activations: the lanes of an aligned group of LPR lanes share the row's units; acc[t] holds this
// lane's part.  `sub` = lane index inside the group.
template <int TYPE, int NT, int LPR>
__device__ __forceinline__ void row_dot(const uint8_t* __restrict__ row, int k, int sub, const ActLds& a,
                                        const uint2* __restrict__ grid, float (&acc)[NT], bool stream_packed, int rq) {
    if constexpr (TYPE == kQ4_K) {
        const int np = k >> 6;
        for (int p = sub; p < np; p += LPR) {
            const uint8_t* blk = row + (size_t) (p >> 2) * 144;
            UnitQ4K u;
            Fmt<kQ4_K>::decode(blk, p & 3, u);
            const float D = Fmt<kQ4_K>::scale(blk), Dm = Fmt<kQ4_K>::scale_min(blk);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const int* y = a.q + t * a.kq + p * 16;
                int lo = 0, hi = 0;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    lo = dot4(u.lo[i], y[i], lo);
                    hi = dot4(u.hi[i], y[8 + i], hi);
                }
                const int b0 = a.bs2[t * a.kd + 2 * p], b1 = a.bs2[t * a.kd + 2 * p + 1];
                // (24-bit multiplies throughout: the operands are sums of at most 32 products of bytes, and the 32-bit
                // integer multiply runs at a quarter of the rate)
                const int ms = __mul24(u.m0, (int) (short) (b0 & 0xffff) + (b0 >> 16)) +
                               __mul24(u.m1, (int) (short) (b1 & 0xffff) + (b1 >> 16));
                const float dy = a.d[t * a.kd + 2 * p];
                acc[t] = fmaf(__fmul_rn(dy, D), (float) (__mul24(u.sc0, lo) + __mul24(u.sc1, hi)), acc[t]);
                acc[t] = fmaf(-__fmul_rn(dy, Dm), (float) ms, acc[t]);
            }
        }
    } else {
        const int nu = k >> 5;
        for (int un = sub; un < nu; un += LPR) {
            const uint8_t* blk;
            int ib;
            if constexpr (TYPE == kQ8_0) {
                blk = row + (size_t) un * 34;
                ib = 0;
            } else {
                blk = row + (size_t) (un >> 3) * Fmt<TYPE>::kBytes;
                ib = un & 7;
            }
            Unit32 u;
            float D;
            if (quad_packed(TYPE) && stream_packed) {
                if constexpr (quad_packed(TYPE)) Fmt<TYPE>::decode_stream(row, nu, rq, un, grid, u, D);
            } else if (TYPE == kQ8_0 && stream_packed) {   // the row's codes, then its scales
                const int* c = (const int*) (row + 32 * (size_t) un);
#pragma unroll
                for (int i = 0; i < 8; ++i) u.q[i] = c[i];
                u.s0 = u.s1 = 1;
                D = f16_bits_to_f32(ld16(row + k + 2 * (size_t) un));
            } else {
                Fmt<TYPE>::decode(blk, ib, grid, u);
                D = Fmt<TYPE>::scale(blk);
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const int* y = a.q + t * a.kq + un * 8;
                int lo = 0, hi = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    lo = dot4(u.q[i], y[i], lo);
                    hi = dot4(u.q[4 + i], y[4 + i], hi);
                }
                if constexpr (Fmt<TYPE>::kBiased) {
                    // the table holds codes + 9 - delta: + (delta - 9) x (the activations' sums), 16 values a half
                    const int bs = a.bs2[t * a.kd + un];
                    const int s_lo = (int) (short) (bs & 0xffff), s_hi = bs >> 16;
                    if constexpr (TYPE == kIQ1_S) {   // one delta a sub-block
                        lo += __mul24(u.dm[0], s_lo);
                        hi += __mul24(u.dm[0], s_hi);
                    } else {                          // one a group of 8: the first group's sum, the second's by difference
                        const int a0 = dot4(0x01010101, y[0], dot4(0x01010101, y[1], 0));
                        const int a1 = dot4(0x01010101, y[4], dot4(0x01010101, y[5], 0));
                        lo += __mul24(u.dm[0], a0) + __mul24(u.dm[1], s_lo - a0);
                        hi += __mul24(u.dm[2], a1) + __mul24(u.dm[3], s_hi - a1);
                    }
                }
                acc[t] = fmaf(__fmul_rn(D, a.d[t * a.kd + un]), (float) (__mul24(u.s0, lo) + __mul24(u.s1, hi)), acc[t]);
            }
        }
    }
}

template <int TYPE> __device__ __forceinline__ const uint64_t* codebook_of(const Codebooks& cb) {
    if constexpr (TYPE == kIQ2_S) return cb.iq2s;
    else if constexpr (TYPE == kIQ1_S || TYPE == kIQ1_M) return cb.iq1s;
    else if constexpr (TYPE == kIQ2_XXS) return cb.iq2xxs;
    else return nullptr;
}

// a type's codebook into LDS; the IQ1 grid (bytes -1 / 0 / +1) as 8 g + 9 (see Fmt<kIQ1_S>)
template <int TYPE, int NT>
__device__ __forceinline__ void stage_codebook(int* lds, const Codebooks& cb) {
    constexpr int n = Fmt<TYPE>::kLdsWords;
    if constexpr (n > 0) {
        TablePieces<n, NT> t;
        table_request(codebook_of<TYPE>(cb), t);
        table_store(lds, t, [](int w) {
            uint32_t g = (uint32_t) w;
            if constexpr (Fmt<TYPE>::kBiased) {
                const uint32_t neg = (g >> 1) & 0x01010101u, pos = g & ~(g >> 1) & 0x01010101u;
                g = 0x09090909u + (pos << 3) - (neg << 3);
            }
            return (int) g;
        });
    }
}

// stage the codebook (once) and NT activation rows into LDS; rows[t] = the activation row of staged slot t (-1: none)
template <int TYPE, int NT>
__device__ __forceinline__ void stage_act(int* lds_act, int k, const maya_act& src, const int (&rows)[NT], bool want_bs) {
    const int kq = k >> 2, kd = k >> 5;
    int* q = lds_act;
    float* d = (float*) (lds_act + NT * kq);
    int* bs = lds_act + NT * kq + NT * kd;
    for (int t = 0; t < NT; ++t) {
        if (rows[t] < 0) continue;
        const int* sq = (const int*) (src.q + (size_t) rows[t] * k);
        const float* sd = src.d + (size_t) rows[t] * kd;
        for (int i = threadIdx.x; i < kq; i += blockDim.x) q[t * kq + i] = sq[i];
        for (int i = threadIdx.x; i < kd; i += blockDim.x) d[t * kd + i] = sd[i];
        if (want_bs) {
            const int* sb = (const int*) (src.bsums + (size_t) rows[t] * (k >> 4));
            for (int i = threadIdx.x; i < kd; i += blockDim.x) bs[t * kd + i] = sb[i];
        }
    }
}

struct GroupRef {
    uint64_t blob;
    int e0, ne;          // entries [e0, e0 + ne) of grp_ent (or the single entry e0 when grp_ent is null)
};
__device__ __forceinline__ bool group_of(const maya_moe_args& a, int g, GroupRef& r) {
    if (a.skip && *a.skip) return false;
    const int total = a.n_tokens * a.k;
    if (a.grp_ptr) {
        if (g >= *a.n_groups) return false;
        r.blob = a.grp_ptr[g];
        r.e0 = a.grp_start[g];
        r.ne = a.grp_start[g + 1] - r.e0;
    } else {
        if (g >= total) return false;
        r.blob = a.plan_ptr[g];
        r.e0 = g;
        r.ne = 1;
    }
    return r.blob != 0ull && r.ne > 0;
}
__device__ __forceinline__ int entry_of(const maya_moe_args& a, const GroupRef& r, int i) {
    return a.grp_ptr ? a.grp_ent[r.e0 + i] : r.e0;
}

__device__ __forceinline__ float swiglu(float g, float u, float limit) {
    if (limit > 0.0f && limit < INFINITY) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
    }
    return __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, expf(-g))), u);
}

constexpr int kGuThreads = 512, kGuRows = 32;   // a workgroup: 8 waves, at most 32 gate + 32 up rows
constexpr int kDnThreads = 512, kDnRows = 64;   // 8 waves x 2 rows a pass, at most 4 passes
// rows a workgroup takes (a multiple of `unit`, at most `most`): fewer when the call has few entries - a shared expert,
// a single token - so that the grid still covers the chip
inline int rows_per_wg(int n_rows, int entries, int unit, int most) {
    int r = most;
    while (r > unit && (long long) ((n_rows + r - 1) / r) * entries < 1024) r >>= 1;
    return r < unit ? unit : r;
}

// grid (n_ff / kGuRows, groups): wave w takes row pairs w, w + 8, ...: lanes 0..31 the gate row, 32..63 the up row
template <int TG, int TU, int NT>
__global__ __launch_bounds__(kGuThreads) void gate_up_kernel(maya_moe_args a, Codebooks cb, int wg_rows) {
    extern __shared__ __align__(16) int lds[];
    GroupRef gr;
    if (!group_of(a, blockIdx.y, gr)) return;
    const int k = a.layout.n_embd, n_ff = a.layout.n_ff;
    // the codebooks of the gate and of the up type (one copy when they share it)
    constexpr int cbg = Fmt<TG>::kLdsWords, cbu = Fmt<TG>::kLdsWords == Fmt<TU>::kLdsWords ? 0 : Fmt<TU>::kLdsWords;
    constexpr int cbw = cbg + cbu;
    stage_codebook<TG, kGuThreads>(lds, cb);
    if constexpr (cbu > 0) stage_codebook<TU, kGuThreads>(lds + cbg, cb);
    const uint2* grid_g = (const uint2*) lds;
    const uint2* grid_u = (const uint2*) (lds + (cbu > 0 ? cbg : 0));
    int* lds_act = lds + cbw;
    const int kq = k >> 2, kd = k >> 5;
    ActLds al{lds_act, (const float*) (lds_act + NT * kq), lds_act + NT * kq + NT * kd, kq, kd};
    const uint8_t* blob = (const uint8_t*) gr.blob;
    const size_t grow = (size_t) (k / Fmt<TG>::kValues) * Fmt<TG>::kBytes, urow = (size_t) (k / Fmt<TU>::kValues) * Fmt<TU>::kBytes;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, sub = lane & 31;
    const bool is_up = lane >= 32;
    const bool packed = a.layout.packing == MAYA_PACK_STREAM;
    for (int c0 = 0; c0 < gr.ne; c0 += NT) {
        int ents[NT], rows[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            ents[t] = c0 + t < gr.ne ? entry_of(a, gr, c0 + t) : -1;
            rows[t] = ents[t] >= 0 ? ents[t] / a.k : -1;
        }
        __syncthreads();
        stage_act<TG, NT>(lds_act, k, a.x, rows, Fmt<TG>::kMin || Fmt<TU>::kMin || Fmt<TG>::kBiased || Fmt<TU>::kBiased);
        __syncthreads();
        for (int r = blockIdx.x * wg_rows + wave; r < min(n_ff, (int) (blockIdx.x + 1) * wg_rows); r += kGuThreads / 64) {
            float acc[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[t] = 0.0f;
            // (stream packing: the row's quad and its place in it; the GGUF packing: the row itself)
            // (only IQ2_S rows have a stream order; the other types' rows stay where GGUF puts them)
            // (IQ2_S rows are packed in quads, Q8_0 rows one by one)
            const bool qg = packed && quad_packed(TG), qu = packed && quad_packed(TU);
            const bool pg = packed && (quad_packed(TG) || TG == kQ8_0), pu = packed && (quad_packed(TU) || TU == kQ8_0);
            const int rq = r & 3;
            if constexpr (TG == TU) {
                const uint8_t* row = blob + (is_up ? a.layout.up_off : a.layout.gate_off) + (size_t) (qg ? (r & ~3) : r) * grow;
                row_dot<TG, NT, 32>(row, k, sub, al, grid_g, acc, pg, rq);
            } else {
                if (!is_up) row_dot<TG, NT, 32>(blob + a.layout.gate_off + (size_t) (qg ? (r & ~3) : r) * grow, k, sub, al, grid_g, acc, pg, rq);
                else row_dot<TU, NT, 32>(blob + a.layout.up_off + (size_t) (qu ? (r & ~3) : r) * urow, k, sub, al, grid_u, acc, pu, rq);
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const float s = group_sum<32>(acc[t]);
                const float up = __shfl(s, 32, kWave);
                if (lane == 0 && ents[t] >= 0) a.h[(size_t) ents[t] * n_ff + r] = swiglu(s, up, a.limit);
            }
        }
    }
}

// grid (n_embd / kDnRows, groups): a wave takes 2 rows a pass, 32 lanes a row (the single-token kernel's split of a
// row over lanes, so a window's rows get the token path's bits)
template <int TD, int NT>
__global__ __launch_bounds__(kDnThreads) void down_kernel(maya_moe_args a, Codebooks cb, int wg_rows) {
    extern __shared__ __align__(16) int lds[];
    GroupRef gr;
    if (!group_of(a, blockIdx.y, gr)) return;
    const int k = a.layout.n_ff, n_embd = a.layout.n_embd;
    constexpr int cbw = Fmt<TD>::kLdsWords;
    stage_codebook<TD, kDnThreads>(lds, cb);
    const uint2* grid = (const uint2*) lds;
    int* lds_act = lds + cbw;
    const int kq = k >> 2, kd = k >> 5;
    ActLds al{lds_act, (const float*) (lds_act + NT * kq), lds_act + NT * kq + NT * kd, kq, kd};
    const uint8_t* base = (const uint8_t*) gr.blob + a.layout.down_off;
    const size_t drow = (size_t) (k / Fmt<TD>::kValues) * Fmt<TD>::kBytes;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, sub = lane & 31, rsub = lane >> 5;
    const bool quads = a.layout.packing == MAYA_PACK_STREAM && quad_packed(TD);
    const bool packed = a.layout.packing == MAYA_PACK_STREAM && (quad_packed(TD) || TD == kQ8_0);
    for (int c0 = 0; c0 < gr.ne; c0 += NT) {
        int ents[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) ents[t] = c0 + t < gr.ne ? entry_of(a, gr, c0 + t) : -1;
        __syncthreads();
        stage_act<TD, NT>(lds_act, k, a.hq, ents, Fmt<TD>::kMin || Fmt<TD>::kBiased);
        __syncthreads();
        const int r_end = min(n_embd, (int) (blockIdx.x + 1) * wg_rows);
        for (int r = blockIdx.x * wg_rows + wave * 2 + rsub; r < r_end; r += (kDnThreads / 64) * 2) {
            float acc[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[t] = 0.0f;
            row_dot<TD, NT, 32>(base + (size_t) (quads ? (r & ~3) : r) * drow, k, sub, al, grid, acc, packed, r & 3);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const float s = group_sum<32>(acc[t]);
                if (sub == 0 && ents[t] >= 0) a.part[(size_t) ents[t] * n_embd + r] = s;
            }
        }
    }
}

// out[t][c] = sum_i w[t*k+i] * part[t*k+i][c] in slot order, each product and sum rounded (native_moe.cu:36-52);
// skipped slots (null blob) are left out; + add[t][c] when given and flagged
__global__ __launch_bounds__(256) void combine_kernel(maya_moe_args a) {
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

// ---- dense mat-vec jobs (glmf::mv, include/strata/kernels/glm_fast.hpp:23-55): the down kernel's row split - a wave
// takes 2 rows a pass, 32 lanes a row, the activations staged in LDS, NT columns sharing one decode of a row - without
// plan or groups; grid (rows / wg_rows, jobs).  y = alpha * dot + bias, each operation rounded.
struct MvJobDev {
    const uint8_t* w;
    maya_act x;
    const float* bias;
    float* y;
    long long y_stride;
    float alpha;
    int n_in, n_out, ncol, packing;
};
struct MvBatch {
    MvJobDev job[MAYA_MV_MAX_JOBS];
};
template <int T, int NT>
__global__ __launch_bounds__(kDnThreads) void mv_kernel(MvBatch b, Codebooks cb, int wg_rows) {
    extern __shared__ __align__(16) int lds[];
    const MvJobDev& j = b.job[blockIdx.y];
    const int k = j.n_in, n_out = j.n_out;
    if ((int) blockIdx.x * wg_rows >= n_out) return;
    constexpr int cbw = Fmt<T>::kLdsWords;
    stage_codebook<T, kDnThreads>(lds, cb);
    const uint2* grid = (const uint2*) lds;
    int* lds_act = lds + cbw;
    const int kq = k >> 2, kd = k >> 5;
    ActLds al{lds_act, (const float*) (lds_act + NT * kq), lds_act + NT * kq + NT * kd, kq, kd};
    const size_t drow = (size_t) (k / Fmt<T>::kValues) * Fmt<T>::kBytes;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, sub = lane & 31, rsub = lane >> 5;
    const bool quads = j.packing == MAYA_PACK_STREAM && quad_packed(T);
    const bool packed = j.packing == MAYA_PACK_STREAM && (quad_packed(T) || T == kQ8_0);
    for (int c0 = 0; c0 < j.ncol; c0 += NT) {
        int cols[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) cols[t] = c0 + t < j.ncol ? c0 + t : -1;
        __syncthreads();
        stage_act<T, NT>(lds_act, k, j.x, cols, Fmt<T>::kMin || Fmt<T>::kBiased);
        __syncthreads();
        const int r_end = min(n_out, (int) (blockIdx.x + 1) * wg_rows);
        for (int r = blockIdx.x * wg_rows + wave * 2 + rsub; r < r_end; r += (kDnThreads / 64) * 2) {
            float acc[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[t] = 0.0f;
            row_dot<T, NT, 32>(j.w + (size_t) (quads ? (r & ~3) : r) * drow, k, sub, al, grid, acc, packed, r & 3);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const float sum = group_sum<32>(acc[t]);
                if (sub == 0 && cols[t] >= 0) {
                    float v = __fmul_rn(j.alpha, sum);
                    if (j.bias) v = __fadd_rn(v, j.bias[r]);
                    j.y[(size_t) cols[t] * j.y_stride + r] = v;
                }
            }
        }
    }
}

}  // namespace maya

#include "maya_fast.hpp"
#include "maya_fast1.hpp"
#include "maya_fastk.hpp"
#include "maya_fastq.hpp"
#include "maya_fastmv.hpp"
#include "maya_tiers.hpp"

namespace maya {

// ------------------------------------------------------------------------------------------------ host launchers

bool type_ok(int t) { return t == kQ8_0 || t == kQ4_K || t == kIQ2_XXS || t == kIQ1_S || t == kIQ2_S || t == kIQ1_M; }
bool q8k_act(int t) { return t != kQ8_0; }
int block_bytes(int t) {
    switch (t) {
        case kQ8_0: return 34;
        case kQ4_K: return 144;
        case kIQ1_S: return 50;
        case kIQ2_S: return 82;
        case kIQ1_M: return 56;
        case kIQ2_XXS: return 66;
        default: return 0;
    }
}
int block_values(int t) { return t == kQ8_0 ? 32 : (type_ok(t) ? 256 : 0); }
int codebook_words(int t) { return t == kIQ2_S ? 2048 : (t == kIQ1_S || t == kIQ1_M) ? 4096 : t == kIQ2_XXS ? 512 : 0; }
size_t act_lds_bytes(int k, int nt) { return (size_t) nt * ((size_t) k + (size_t) (k / 32) * 8); }

int check_layout(const maya_moe_layout& l) {
    if (!type_ok(l.gate_type) || !type_ok(l.up_type) || !type_ok(l.down_type))
        return fail(MAYA_E_UNSUPPORTED, "expert types %d/%d/%d: no kernel", l.gate_type, l.up_type, l.down_type);
    if (q8k_act(l.gate_type) != q8k_act(l.up_type))
        return fail(MAYA_E_UNSUPPORTED, "gate type %d and up type %d quantize their activation differently", l.gate_type,
                    l.up_type);
    if (l.n_embd <= 0 || l.n_ff <= 0 || l.n_embd % 256 || l.n_ff % 256)
        return fail(MAYA_E_SHAPE, "n_embd %d / n_ff %d: multiples of 256 wanted", l.n_embd, l.n_ff);
    if (l.packing != MAYA_PACK_GGUF && l.packing != MAYA_PACK_STREAM) return fail(MAYA_E_UNSUPPORTED, "packing %d", l.packing);
    if (l.packing == MAYA_PACK_STREAM && (l.gate_off % 16 || l.up_off % 16 || l.down_off % 16))
        return fail(MAYA_E_ARG, "stream packing wants 16-byte aligned row arrays");
    if (l.n_embd > 16384 || l.n_ff > 16384) return fail(MAYA_E_SHAPE, "n_embd %d / n_ff %d past 16384", l.n_embd, l.n_ff);
    return MAYA_OK;
}
int check_args(const maya_moe_args* a) {
    if (!a) return fail(MAYA_E_ARG, "null args");
    if (const int rc = check_layout(a->layout)) return rc;
    if (a->n_tokens < 1 || a->n_tokens > MAYA_MAX_TOKENS || a->k < 1 || a->k > MAYA_MAX_K)
        return fail(MAYA_E_SHAPE, "n_tokens %d / k %d outside 1..%d / 1..%d", a->n_tokens, a->k, MAYA_MAX_TOKENS, MAYA_MAX_K);
    if (!a->plan_ptr || !a->plan_w) return fail(MAYA_E_ARG, "null plan");
    if (a->grp_ptr && (!a->grp_start || !a->grp_ent || !a->n_groups)) return fail(MAYA_E_ARG, "incomplete groups");
    return MAYA_OK;
}

template <int TG, int TU>
int launch_gate_up_t(const maya_moe_args& a, const DeviceState& st, hipStream_t s) {
    const int nt = a.grp_ptr ? (a.n_tokens >= 4 ? 4 : a.n_tokens >= 2 ? 2 : 1) : 1;
    const int cbw = codebook_words(TG) + (codebook_words(TG) == codebook_words(TU) ? 0 : codebook_words(TU));
    const size_t lds = (size_t) cbw * 4 + act_lds_bytes(a.layout.n_embd, nt);
    if (lds > (size_t) st.lds_limit) return fail(MAYA_E_SHAPE, "gate/up needs %zu bytes of LDS, the device gives %d", lds, st.lds_limit);
    const int wr = rows_per_wg(a.layout.n_ff, a.n_tokens * a.k, 8, kGuRows);
    const dim3 grid((unsigned) ((a.layout.n_ff + wr - 1) / wr), (unsigned) (a.n_tokens * a.k));
    if (nt == 4) hipLaunchKernelGGL((gate_up_kernel<TG, TU, 4>), grid, dim3(kGuThreads), lds, s, a, st.cb, wr);
    else if (nt == 2) hipLaunchKernelGGL((gate_up_kernel<TG, TU, 2>), grid, dim3(kGuThreads), lds, s, a, st.cb, wr);
    else hipLaunchKernelGGL((gate_up_kernel<TG, TU, 1>), grid, dim3(kGuThreads), lds, s, a, st.cb, wr);
    MAYA_LAUNCHED("gate_up_kernel");
    return MAYA_OK;
}
template <int TD>
int launch_down_t(const maya_moe_args& a, const DeviceState& st, hipStream_t s) {
    const int nt = a.grp_ptr ? (a.n_tokens >= 4 ? 4 : a.n_tokens >= 2 ? 2 : 1) : 1;
    const size_t lds = (size_t) codebook_words(TD) * 4 + act_lds_bytes(a.layout.n_ff, nt);
    if (lds > (size_t) st.lds_limit) return fail(MAYA_E_SHAPE, "down needs %zu bytes of LDS, the device gives %d", lds, st.lds_limit);
    const int wr = rows_per_wg(a.layout.n_embd, a.n_tokens * a.k, 16, kDnRows);
    const dim3 grid((unsigned) ((a.layout.n_embd + wr - 1) / wr), (unsigned) (a.n_tokens * a.k));
    if (nt == 4) hipLaunchKernelGGL((down_kernel<TD, 4>), grid, dim3(kDnThreads), lds, s, a, st.cb, wr);
    else if (nt == 2) hipLaunchKernelGGL((down_kernel<TD, 2>), grid, dim3(kDnThreads), lds, s, a, st.cb, wr);
    else hipLaunchKernelGGL((down_kernel<TD, 1>), grid, dim3(kDnThreads), lds, s, a, st.cb, wr);
    MAYA_LAUNCHED("down_kernel");
    return MAYA_OK;
}

bool fast_1tok(const maya_moe_args& a) { return a.n_tokens == 1 && a.grp_ptr == nullptr; }

int launch_gate_up_iq2s_gguf(const maya_moe_args& a, const DeviceState& st, hipStream_t s) {
    constexpr int kRows = 32;
    const dim3 grid((unsigned) (a.layout.n_ff / kRows), (unsigned) a.k);
#define MAYA_KU(N) case N: hipLaunchKernelGGL((gate_up_iq2s_1tok_kernel<N, kRows, true, false, 4, false>), grid, dim3(512), 0, s, a, st.cb); break;
    switch (a.layout.n_embd / 1024) {
        MAYA_KU(1) MAYA_KU(2) MAYA_KU(3) MAYA_KU(4) MAYA_KU(5) MAYA_KU(6) MAYA_KU(7) MAYA_KU(8)
    }
#undef MAYA_KU
    MAYA_LAUNCHED("gate_up_iq2s_1tok_kernel");
    return MAYA_OK;
}
// the position-mapped kernels: gate/up 16 rows a workgroup at the 6 waves a SIMD its registers allow; down 16 rows at 7
// waves a SIMD (8 spill), or n_embd / 256 rows for the wide rows
template <int NW>
int launch_gate_up_iq2s_pos(const maya_moe_args& a, const DeviceState& st, hipStream_t s) {
    constexpr int kRows = 16;
    const dim3 grid((unsigned) (a.layout.n_ff / kRows), (unsigned) (a.n_tokens * a.k));   // an entry a column of the grid
    hipLaunchKernelGGL((gate_up_iq2s_pos_kernel<NW, kRows, 1, 8>), grid, dim3(64 * NW), 0, s, a, st.cb);
    MAYA_LAUNCHED("gate_up_iq2s_pos_kernel");
    return MAYA_OK;
}
// One token: the tile-streaming form, launched with the workgroups the chip holds at once (asked of the runtime once a
// shape), at most three a compute unit: measured on 7168 x 2048, top-8, 768 workgroups 18.5 us, 1024 (all resident, two
// tiles each) 20.1 us, 512 20.4 us, 256 24.1 us - a workgroup's cold start is paid per workgroup, latency hiding per wave.
// The kernel is compiled for 6 waves a SIMD - three workgroups of up to 8 waves a compute unit, what is launched - not 8:
// with the head's prologue in it the kernel needs 73-77 registers, and at 64 it spilled 36 bytes a lane to scratch
// memory: 6.8 MB written and read back a launch, 2.1 us of the layer.  Windows keep gate_up_iq2s_pos_kernel: the tile
// stream with the resident workgroups shared out among the tokens (a token's codes in a workgroup's registers) was built
// and is slower there (configs[2]: 260 us against 234).
template <int NW>
int launch_gate_up_iq2s_tiles(const maya_moe_args& a, const DeviceState& st, hipStream_t s, const LayerHeadIn* hd = nullptr) {
    static int per_cu = 0;
    if (per_cu == 0) {
        int n = 0, m = 0;
        MAYA_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gate_up_iq2s_tiles_kernel<NW, 6, false>, 64 * NW, 0));
        MAYA_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&m, gate_up_iq2s_tiles_kernel<NW, 6, true>, 64 * NW, 0));
        n = m < n ? m : n;
        per_cu = n > 3 ? 3 : n > 0 ? n : 1;
    }
    const int n_tiles = a.k * (a.layout.n_ff / 8);
    const int wgs = per_cu * st.n_cu;
    const unsigned walkers = (unsigned) (wgs < n_tiles ? wgs : n_tiles);
    if (hd) {   // workgroup 0 routes, the others walk the tiles
        hipLaunchKernelGGL((gate_up_iq2s_tiles_kernel<NW, 6, true>), dim3(walkers + 1), dim3(64 * NW), 0, s, (const void*) hd->logits,
                           (const void*) hd->table, hd->x, st.cb.iq2s, hd->bias, a.skip, hd->n_expert, hd->x_dtype | (hd->sigmoid << 8), a.k, a,
                           hd->out);
    } else {
        hipLaunchKernelGGL((gate_up_iq2s_tiles_kernel<NW, 6, false>), dim3(walkers), dim3(64 * NW), 0, s, (const void*) a.plan_ptr,
                           (const void*) a.x.q, (const void*) a.x.d, st.cb.iq2s, (const float*) nullptr, a.skip, 0, 0, a.k, a, LayerHead{});
    }
    MAYA_LAUNCHED("gate_up_iq2s_tiles_kernel");
    return MAYA_OK;
}
// The single-token layer whose head rides in the gate/up launch (gate_up_iq2s_tiles_kernel<.., true>,
// gate_up_q4k_pos_kernel<.., true>): either router over up to 256 experts with more experts than slots, x aligned for
// 16-byte loads, IQ2_S, Q4_K or IQ1_S gate/up rows in the stream packing's shapes.  (IQ1_M keeps its head launch: its
// gate/up kernel with the head in it was 6.3 us slower a launch than without, more than the 4.8 us head launch it replaces;
// IQ1_S gains 1.4 us a layer, Q4_K 0.6, and the one-expert Q4_K layer of few workgroups 2.7 of 16.)
bool gate_up_q4k_pos_ok(const maya_moe_args& a);
bool gate_up_iq1s_pos_ok(const maya_moe_args& a);
static bool layer_head_in_gate_up_ok(const maya_moe_args& a, const RouterSpec& rs, const float* logits, int n_expert, const void* x,
                                     int x_dtype) {
    const maya_moe_layout& l = a.layout;
    if (!(logits && a.n_tokens == 1 && n_expert <= 256 && a.k < n_expert && x_dtype >= 0 && x_dtype <= 2 && ((uintptr_t) x & 15) == 0))
        return false;
    if (l.gate_type == kQ4_K) return gate_up_q4k_pos_ok(a);
    if (l.gate_type == kIQ1_S) return gate_up_iq1s_pos_ok(a);
    return l.gate_type == kIQ2_S && l.up_type == kIQ2_S && l.packing == MAYA_PACK_STREAM && l.n_ff % 16 == 0 && l.n_embd % 1024 == 0 &&
           l.n_embd >= 2048 && l.n_embd <= 8192;
}
static int launch_layer_gate_up_iq2s(const maya_moe_args& a, const LayerHeadIn& hd, const DeviceState& st, hipStream_t s) {
    switch (a.layout.n_embd / 1024) {
        case 2: return launch_gate_up_iq2s_tiles<2>(a, st, s, &hd);
        case 3: return launch_gate_up_iq2s_tiles<3>(a, st, s, &hd);
        case 4: return launch_gate_up_iq2s_tiles<4>(a, st, s, &hd);
        case 5: return launch_gate_up_iq2s_tiles<5>(a, st, s, &hd);
        case 6: return launch_gate_up_iq2s_tiles<6>(a, st, s, &hd);
        case 7: return launch_gate_up_iq2s_tiles<7>(a, st, s, &hd);
        default: return launch_gate_up_iq2s_tiles<8>(a, st, s, &hd);
    }
}
// the rows the position-mapped down kernels take on one wave: n_ff = 1024, 1536 or 2048
static bool down_pos_nff_ok(int n_ff) { return n_ff == 1024 || n_ff == 1536 || n_ff == 2048; }
int launch_down_iq2s_pos(const maya_moe_args& a, const DeviceState& st, hipStream_t s) {
    // One quad of rows in flight a wave: with 2, 4 or all 7 of a wave's quads requested ahead the 7168 x 2048 launch took
    // 12.6, 14.0 and 15.9 us against 11.9.
    // Rows a workgroup: n_embd / 256 for the wide rows (20 ... 32: one workgroup a compute unit on a single token, every
    // SIMD the same number of rows, and half as many waves rounding h as with 16), else 16.
    const int n_embd = a.layout.n_embd;
    const int wide = n_embd % 1024 == 0 && n_embd >= 5120 && n_embd <= 8192 ? n_embd / 256 : 16;
#define MAYA_DN_HEAD a.plan_ptr, a.plan_w, a.h, st.cb.iq2s, a.skip, a.hq.q, a.k, a.layout.n_embd
#define MAYA_ROWS(R, MINW)                                                                                             \
    {                                                                                                                  \
        const dim3 grid((unsigned) (n_embd / R), (unsigned) a.n_tokens);                                               \
        if (a.layout.n_ff == 1024) hipLaunchKernelGGL((down_iq2s_pos_kernel<R, 1, MINW, 32>), grid, dim3(512), 0, s, MAYA_DN_HEAD, a, st.cb);      \
        else if (a.layout.n_ff == 1536) hipLaunchKernelGGL((down_iq2s_pos_kernel<R, 1, MINW, 48>), grid, dim3(512), 0, s, MAYA_DN_HEAD, a, st.cb); \
        else hipLaunchKernelGGL((down_iq2s_pos_kernel<R, 1, MINW>), grid, dim3(512), 0, s, MAYA_DN_HEAD, a, st.cb);                  \
    }
    switch (wide) {
        case 20: MAYA_ROWS(20, 4) break;
        case 24: MAYA_ROWS(24, 4) break;
        case 28: MAYA_ROWS(28, 4) break;
        case 32: MAYA_ROWS(32, 4) break;
        default: MAYA_ROWS(16, 7) break;
    }
#undef MAYA_DN_HEAD
#undef MAYA_ROWS
    MAYA_LAUNCHED("down_iq2s_pos_kernel");
    return MAYA_OK;
}
int launch_down_iq2s_gguf(const maya_moe_args& a, const DeviceState& st, hipStream_t s) {
    constexpr int kRows = 14;
    const dim3 grid((unsigned) (a.layout.n_embd / kRows));
#define MAYA_KU(N) case N: hipLaunchKernelGGL((down_iq2s_1tok_kernel<N, kRows, false>), grid, dim3(512), 0, s, a, st.cb); break;
    switch (a.layout.n_ff / 1024) {
        MAYA_KU(1) MAYA_KU(2) MAYA_KU(3) MAYA_KU(4)
    }
#undef MAYA_KU
    MAYA_LAUNCHED("down_iq2s_1tok_kernel");
    return MAYA_OK;
}

// single-token IQ2_S gate/up: 1 launched, 0 no specialised kernel for this shape (the caller takes the general one)
int try_gate_up_iq2s_1tok(const maya_moe_args& a, const DeviceState& st, hipStream_t s, int* rc) {
    const maya_moe_layout& l = a.layout;
    if (l.packing != MAYA_PACK_STREAM && !fast_1tok(a)) return 0;
    // (the position-mapped kernels take the entries of several tokens one by one, whether grouped or not: every entry
    // is computed as its token alone would compute it)
    if (l.packing == MAYA_PACK_STREAM) {
        if (l.n_ff % 16 != 0) return 0;
        if (a.n_tokens == 1) {
            switch (l.n_embd / 1024 * (l.n_embd % 1024 == 0)) {
                case 2: *rc = launch_gate_up_iq2s_tiles<2>(a, st, s); return 1;
                case 3: *rc = launch_gate_up_iq2s_tiles<3>(a, st, s); return 1;
                case 4: *rc = launch_gate_up_iq2s_tiles<4>(a, st, s); return 1;
                case 5: *rc = launch_gate_up_iq2s_tiles<5>(a, st, s); return 1;
                case 6: *rc = launch_gate_up_iq2s_tiles<6>(a, st, s); return 1;
                case 7: *rc = launch_gate_up_iq2s_tiles<7>(a, st, s); return 1;
                case 8: *rc = launch_gate_up_iq2s_tiles<8>(a, st, s); return 1;
                default: return 0;
            }
        }
        switch (l.n_embd / 1024 * (l.n_embd % 1024 == 0)) {
            case 2: *rc = launch_gate_up_iq2s_pos<2>(a, st, s); return 1;
            case 3: *rc = launch_gate_up_iq2s_pos<3>(a, st, s); return 1;
            case 4: *rc = launch_gate_up_iq2s_pos<4>(a, st, s); return 1;
            case 5: *rc = launch_gate_up_iq2s_pos<5>(a, st, s); return 1;
            case 6: *rc = launch_gate_up_iq2s_pos<6>(a, st, s); return 1;
            case 7: *rc = launch_gate_up_iq2s_pos<7>(a, st, s); return 1;
            case 8: *rc = launch_gate_up_iq2s_pos<8>(a, st, s); return 1;
            default: return 0;
        }
    }
    if (l.n_embd % 1024 != 0 || l.n_embd > 8192 || l.n_ff % 32 != 0) return 0;
    *rc = launch_gate_up_iq2s_gguf(a, st, s);
    return 1;
}
// ---- IQ1_S / IQ1_M in the stream packing: the position-mapped kernels
bool gate_up_iq1s_pos_ok(const maya_moe_args& a) {
    const maya_moe_layout& l = a.layout;
    if (!((l.gate_type == kIQ1_S || l.gate_type == kIQ1_M) && l.up_type == l.gate_type && l.packing == MAYA_PACK_STREAM)) return false;
    if (l.n_embd % 1024 != 0 || l.n_ff % 16 != 0 || ((l.gate_off | l.up_off | l.down_off) & 15)) return false;
    const int nw = l.n_embd / 1024;
    return nw >= 2 && nw <= 8;
}
bool down_iq1s_pos_ok(const maya_moe_args& a) {
    const maya_moe_layout& l = a.layout;
    return (l.down_type == kIQ1_S || l.down_type == kIQ1_M) && l.packing == MAYA_PACK_STREAM && a.k <= 8 &&
           (l.n_ff == 1024 || l.n_ff == 1536 || l.n_ff == 2048) && l.n_embd % 16 == 0 && (l.down_off & 15) == 0;
}
int launch_gate_up_iq1s_pos(const maya_moe_args& a, const DeviceState& st, hipStream_t s, const LayerHeadIn* hd = nullptr) {
    // (IQ1_S with the head in the launch: one more column, whose first workgroup is the router)
    const dim3 grid((unsigned) (a.layout.n_ff / 16) + (hd ? 1u : 0u), (unsigned) (a.n_tokens * a.k));
    if (a.layout.gate_type == kIQ1_M) {
        if (hd) return fail(MAYA_E_UNSUPPORTED, "gate_up: the IQ1_M rows take no head in their launch");
        switch (a.layout.n_embd / 1024) {
            case 2: hipLaunchKernelGGL((gate_up_iq1m_pos_kernel<2, 16, 8>), grid, dim3(128), 0, s, a, st.cb); break;
            case 3: hipLaunchKernelGGL((gate_up_iq1m_pos_kernel<3, 16, 8>), grid, dim3(192), 0, s, a, st.cb); break;
            case 5: hipLaunchKernelGGL((gate_up_iq1m_pos_kernel<5, 16, 8>), grid, dim3(320), 0, s, a, st.cb); break;
            case 4: hipLaunchKernelGGL((gate_up_iq1m_pos_kernel<4, 16, 8>), grid, dim3(256), 0, s, a, st.cb); break;
            case 6: hipLaunchKernelGGL((gate_up_iq1m_pos_kernel<6, 16, 8>), grid, dim3(384), 0, s, a, st.cb); break;
            case 7: hipLaunchKernelGGL((gate_up_iq1m_pos_kernel<7, 16, 8>), grid, dim3(448), 0, s, a, st.cb); break;
            default: hipLaunchKernelGGL((gate_up_iq1m_pos_kernel<8, 16, 8>), grid, dim3(512), 0, s, a, st.cb); break;
        }
        MAYA_LAUNCHED("gate_up_iq1m_pos_kernel");
        return MAYA_OK;
    }
    const LayerHeadIn h = hd ? *hd : LayerHeadIn{};
#define MAYA_IQ1(NWV)                                                                                                          \
    if (hd) hipLaunchKernelGGL((gate_up_iq1s_pos_kernel<NWV, 16, 6, true>), grid, dim3(64 * NWV), 0, s, a, st.cb, h);             \
    else hipLaunchKernelGGL((gate_up_iq1s_pos_kernel<NWV, 16, 8>), grid, dim3(64 * NWV), 0, s, a, st.cb, h);
    switch (a.layout.n_embd / 1024) {
        case 2: MAYA_IQ1(2) break;
        case 3: MAYA_IQ1(3) break;
        case 4: MAYA_IQ1(4) break;
        case 5: MAYA_IQ1(5) break;
        case 6: MAYA_IQ1(6) break;
        case 7: MAYA_IQ1(7) break;
        default: MAYA_IQ1(8) break;
    }
#undef MAYA_IQ1
    MAYA_LAUNCHED("gate_up_iq1s_pos_kernel");
    return MAYA_OK;
}
int launch_down_iq1s_pos(const maya_moe_args& a, const DeviceState& st, hipStream_t s) {
    // 32 rows a workgroup for the wide rows (half as many waves rounding h, as in the IQ2_S kernel), else 16
    const bool wide = a.layout.n_embd >= 5120 && a.layout.n_embd % 32 == 0;
    const dim3 grid((unsigned) (a.layout.n_embd / (wide ? 32 : 16)), (unsigned) a.n_tokens);
#define MAYA_D1(NUV)                                                                                                     \
    if (wide) {                                                                                                          \
        if (a.layout.down_type == kIQ1_M) hipLaunchKernelGGL((down_iq1m_pos_kernel<32, 7, NUV>), grid, dim3(512), 0, s, a, st.cb); \
        else hipLaunchKernelGGL((down_iq1s_pos_kernel<32, 7, NUV>), grid, dim3(512), 0, s, a, st.cb);                    \
    } else if (a.layout.down_type == kIQ1_M) hipLaunchKernelGGL((down_iq1m_pos_kernel<16, 7, NUV>), grid, dim3(512), 0, s, a, st.cb); \
    else hipLaunchKernelGGL((down_iq1s_pos_kernel<16, 7, NUV>), grid, dim3(512), 0, s, a, st.cb);
    if (a.layout.n_ff == 1024) { MAYA_D1(32) } else if (a.layout.n_ff == 1536) { MAYA_D1(48) } else { MAYA_D1(64) }
#undef MAYA_D1
    MAYA_LAUNCHED("down_iq1s_pos_kernel");
    return MAYA_OK;
}

// whether try_down_iq2s_1tok would take the position-mapped kernel, which can round h to Q8_K itself (hq.q == NULL)
bool down_rounds_h(const maya_moe_args& a) {
    const maya_moe_layout& l = a.layout;
    if (down_iq1s_pos_ok(a)) return true;
    if (l.down_type == kQ4_K) return l.packing == MAYA_PACK_STREAM && a.k <= 8 && down_pos_nff_ok(l.n_ff) && l.n_embd % 16 == 0 && (l.down_off & 15) == 0;
    return l.down_type == kIQ2_S && a.k <= 8 && l.packing == MAYA_PACK_STREAM && down_pos_nff_ok(l.n_ff) && l.n_embd % 16 == 0;
}
int try_down_iq2s_1tok(const maya_moe_args& a, const DeviceState& st, hipStream_t s, int* rc) {
    const maya_moe_layout& l = a.layout;
    if (a.k > 8) return 0;
    if (l.packing != MAYA_PACK_STREAM && !fast_1tok(a)) return 0;
    if (l.packing == MAYA_PACK_STREAM) {
        if (!down_pos_nff_ok(l.n_ff) || l.n_embd % 16 != 0) return 0;
        *rc = launch_down_iq2s_pos(a, st, s);
        return 1;
    }
    if (l.n_ff % 1024 != 0 || l.n_ff > 4096 || l.n_embd % 14 != 0) return 0;
    *rc = launch_down_iq2s_gguf(a, st, s);
    return 1;
}

// ---- Q4_K in the stream packing (its own GGUF order, blobs 16-byte aligned): the position-mapped kernels
bool gate_up_q4k_pos_ok(const maya_moe_args& a) {
    const maya_moe_layout& l = a.layout;
    if (!(l.gate_type == kQ4_K && l.up_type == kQ4_K && l.packing == MAYA_PACK_STREAM)) return false;
    if (l.n_embd % 1024 != 0 || l.n_ff % 16 != 0 || ((l.gate_off | l.up_off | l.down_off) & 15)) return false;
    const int nw = l.n_embd / 1024;
    return nw >= 2 && nw <= 8;
}
bool down_q4k_pos_ok(const maya_moe_args& a) {
    const maya_moe_layout& l = a.layout;
    return l.down_type == kQ4_K && l.packing == MAYA_PACK_STREAM && a.k <= 8 && down_pos_nff_ok(l.n_ff) && l.n_embd % 16 == 0 &&
           (l.down_off & 15) == 0;
}
int launch_gate_up_q4k_pos(const maya_moe_args& a, hipStream_t s, const LayerHeadIn* hd = nullptr) {
    // 16 rows a workgroup, 8 - all requested up front - when the call has so few entries that 16 would leave compute units idle
    const bool small = (long long) (a.layout.n_ff / 16) * a.n_tokens * a.k < 512;
    const int rows = small ? 8 : 16;
    // (with the head in the launch: one more column, whose first workgroup is the router)
    const dim3 grid((unsigned) (a.layout.n_ff / rows) + (hd ? 1u : 0u), (unsigned) (a.n_tokens * a.k));
    const LayerHeadIn h = hd ? *hd : LayerHeadIn{};
#define MAYA_Q4(NWV)                                                                                                       \
    if (hd && small) hipLaunchKernelGGL((gate_up_q4k_pos_kernel<NWV, 8, 4, true, true>), grid, dim3(64 * NWV), 0, s, a, h);   \
    else if (hd) hipLaunchKernelGGL((gate_up_q4k_pos_kernel<NWV, 16, 6, false, true>), grid, dim3(64 * NWV), 0, s, a, h);     \
    else if (small) hipLaunchKernelGGL((gate_up_q4k_pos_kernel<NWV, 8, 4, true>), grid, dim3(64 * NWV), 0, s, a, h);          \
    else hipLaunchKernelGGL((gate_up_q4k_pos_kernel<NWV, 16, 8>), grid, dim3(64 * NWV), 0, s, a, h);
    switch (a.layout.n_embd / 1024) {
        case 2: MAYA_Q4(2) break;
        case 3: MAYA_Q4(3) break;
        case 4: MAYA_Q4(4) break;
        case 5: MAYA_Q4(5) break;
        case 6: MAYA_Q4(6) break;
        case 7: MAYA_Q4(7) break;
        default: MAYA_Q4(8) break;
    }
#undef MAYA_Q4
    MAYA_LAUNCHED("gate_up_q4k_pos_kernel");
    return MAYA_OK;
}
int launch_down_q4k_pos(const maya_moe_args& a, hipStream_t s) {
    // Rows a workgroup: 32 when that still leaves two workgroups a compute unit (half as many waves rounding h); 8 for
    // one or two slots on few tokens (more, shorter waves: the rows of one expert alone are latency-bound); else 16.
    // A workgroup has one wave a slot.
    const int n_embd = a.layout.n_embd;
    const int rows = (long long) (n_embd / 32) * a.n_tokens >= 512 && n_embd % 32 == 0 ? 32
                     : a.k <= 2 && (long long) (n_embd / 16) * a.n_tokens < 1024 && n_embd % 8 == 0 ? 8 : 16;
    const dim3 grid((unsigned) (n_embd / rows), (unsigned) a.n_tokens), block(64u * (unsigned) a.k);
#define MAYA_ROWS(R)                                                                                              \
    if (a.layout.n_ff == 1024) hipLaunchKernelGGL((down_q4k_pos_kernel<R, 8, 32>), grid, block, 0, s, a);          \
    else if (a.layout.n_ff == 1536) hipLaunchKernelGGL((down_q4k_pos_kernel<R, 8, 48>), grid, block, 0, s, a);     \
    else hipLaunchKernelGGL((down_q4k_pos_kernel<R, 8>), grid, block, 0, s, a);
    if (rows == 32) { MAYA_ROWS(32) }
    else if (rows == 8) {
        // every row of a wave requested up front (128 registers)
        if (a.layout.n_ff == 1024) hipLaunchKernelGGL((down_q4k_pos_kernel<8, 4, 32, true>), grid, block, 0, s, a);
        else if (a.layout.n_ff == 1536) hipLaunchKernelGGL((down_q4k_pos_kernel<8, 4, 48, true>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((down_q4k_pos_kernel<8, 4, 64, true>), grid, block, 0, s, a);
    }
    else { MAYA_ROWS(16) }
#undef MAYA_ROWS
    MAYA_LAUNCHED("down_q4k_pos_kernel");
    return MAYA_OK;
}
// ---- Q8_0 in the stream packing: the position-mapped kernels for the shapes they take
bool gate_up_q80_pos_ok(const maya_moe_args& a) {
    const maya_moe_layout& l = a.layout;
    if (!(l.gate_type == kQ8_0 && l.up_type == kQ8_0 && l.packing == MAYA_PACK_STREAM)) return false;
    if (l.n_embd % 1024 != 0 || l.n_ff % 8 != 0 || ((l.gate_off | l.up_off | l.down_off) & 15)) return false;
    const int nw = l.n_embd / 1024;
    return nw >= 2 && nw <= 8;
}
bool down_q80_pos_ok(const maya_moe_args& a) {
    const maya_moe_layout& l = a.layout;
    return l.down_type == kQ8_0 && l.packing == MAYA_PACK_STREAM && down_pos_nff_ok(l.n_ff) && l.n_embd % 64 == 0 && (l.down_off & 15) == 0;
}
// tokens of a group served by one read of the weights: as many as the call can have in a group, rounded up to 1, 2, 4, 8
inline int q80_group_tokens(const maya_moe_args& a) {
    if (!a.grp_ptr) return 1;
    return a.n_tokens >= 5 ? 8 : a.n_tokens >= 3 ? 4 : a.n_tokens >= 2 ? 2 : 1;
}
int launch_gate_up_q80_pos(const maya_moe_args& a, hipStream_t s) {
    const int nt = q80_group_tokens(a);
    const dim3 grid((unsigned) (a.layout.n_ff / 8), (unsigned) (a.n_tokens * a.k));
#define MAYA_Q8(NWV)                                                                                              \
    switch (nt) {                                                                                                 \
        case 8: hipLaunchKernelGGL((gate_up_q80_pos_kernel<NWV, 8, 8>), grid, dim3(64 * NWV), 0, s, a); break;  \
        case 4: hipLaunchKernelGGL((gate_up_q80_pos_kernel<NWV, 4, 8>), grid, dim3(64 * NWV), 0, s, a); break;  \
        case 2: hipLaunchKernelGGL((gate_up_q80_pos_kernel<NWV, 2, 8>), grid, dim3(64 * NWV), 0, s, a); break;  \
        default: hipLaunchKernelGGL((gate_up_q80_pos_kernel<NWV, 1, 8>), grid, dim3(64 * NWV), 0, s, a); break; \
    }
    switch (a.layout.n_embd / 1024) {
        case 2: MAYA_Q8(2) break;
        case 3: MAYA_Q8(3) break;
        case 4: MAYA_Q8(4) break;
        case 5: MAYA_Q8(5) break;
        case 6: MAYA_Q8(6) break;
        case 7: MAYA_Q8(7) break;
        default: MAYA_Q8(8) break;
    }
#undef MAYA_Q8
    MAYA_LAUNCHED("gate_up_q80_pos_kernel");
    return MAYA_OK;
}
int launch_down_q80_pos(const maya_moe_args& a, hipStream_t s) {
    const int nt = q80_group_tokens(a);
    // a wave takes per_wave rows, a multiple of the 8 / nt rows of a step: 8 (64 rows a workgroup) unless the call has so
    // few entries that the grid would not cover the chip
    const int step = 8 / nt;
    int per_wave = 8;
    while (per_wave > step && (long long) (a.layout.n_embd / (per_wave * 8)) * a.n_tokens * a.k < 1024) per_wave >>= 1;
    const int wg_rows = per_wave * 8;
    const dim3 grid((unsigned) ((a.layout.n_embd + wg_rows - 1) / wg_rows), (unsigned) (a.n_tokens * a.k));
#define MAYA_DQ(NUV)                                                                                                    \
    switch (nt) {                                                                                                       \
        case 8: hipLaunchKernelGGL((down_q80_pos_kernel<8, NUV>), grid, dim3(512), 0, s, a, wg_rows); break;        \
        case 4: hipLaunchKernelGGL((down_q80_pos_kernel<4, NUV>), grid, dim3(512), 0, s, a, wg_rows); break;        \
        case 2: hipLaunchKernelGGL((down_q80_pos_kernel<2, NUV>), grid, dim3(512), 0, s, a, wg_rows); break;        \
        default: hipLaunchKernelGGL((down_q80_pos_kernel<1, NUV>), grid, dim3(512), 0, s, a, wg_rows); break;       \
    }
    if (a.layout.n_ff == 1024) { MAYA_DQ(32) } else if (a.layout.n_ff == 1536) { MAYA_DQ(48) } else { MAYA_DQ(64) }
#undef MAYA_DQ
    MAYA_LAUNCHED("down_q80_pos_kernel");
    return MAYA_OK;
}

// whether the gate/up (down) call is served entry by entry (no use for the groups of a window)
// the shapes the IQ2_S streaming kernels take (what try_gate_up_iq2s_1tok / try_down_iq2s_1tok launch on)
static bool gate_up_iq2s_fast_ok(const maya_moe_args& a) {
    const maya_moe_layout& l = a.layout;
    if (l.packing == MAYA_PACK_STREAM) return l.n_ff % 16 == 0 && l.n_embd % 1024 == 0 && l.n_embd >= 2048 && l.n_embd <= 8192;
    return fast_1tok(a) && l.n_embd % 1024 == 0 && l.n_embd <= 8192 && l.n_ff % 32 == 0;
}
static bool down_iq2s_fast_ok(const maya_moe_args& a) {
    const maya_moe_layout& l = a.layout;
    if (a.k > 8) return false;
    if (l.packing == MAYA_PACK_STREAM) return down_pos_nff_ok(l.n_ff) && l.n_embd % 16 == 0;
    return fast_1tok(a) && l.n_ff % 1024 == 0 && l.n_ff <= 4096 && l.n_embd % 14 == 0;
}
// Everything maya_moe_gate_up / maya_moe_down / maya_quant_act refuse (status > 0), asked without launching anything:
// the calls themselves ask first, and a caller that forks a stream before them (maya_moe_layer_decode_shared) asks before
// the fork, so that its own "> 0: nothing launched" holds.
static int gate_up_refusal(const maya_moe_args* a, const DeviceState& st) {
    if (const int rc = check_args(a)) return rc;
    if (!a->x.q || !a->x.d || !a->x.bsums || !a->h) return fail(MAYA_E_ARG, "gate_up: null activation or h");
    const int tg = a->layout.gate_type, tu = a->layout.up_type;
    const bool pair = (tg == tu) || (tg == kIQ2_S && tu == kIQ1_M) || (tg == kIQ1_M && tu == kIQ2_S) || (tg == kIQ2_S && tu == kQ4_K) ||
                      (tg == kIQ1_S && tu == kIQ1_M) || (tg == kIQ1_M && tu == kIQ1_S);
    if (!pair) return fail(MAYA_E_UNSUPPORTED, "gate_up: no kernel for gate type %d with up type %d", tg, tu);
    const bool pos = (tg == kIQ2_S && tu == kIQ2_S && gate_up_iq2s_fast_ok(*a)) || gate_up_q4k_pos_ok(*a) || gate_up_iq1s_pos_ok(*a) ||
                     gate_up_q80_pos_ok(*a);
    if (!pos) {   // the general kernel: its activation tile and codebooks must fit the device's LDS
        const int nt = a->grp_ptr ? (a->n_tokens >= 4 ? 4 : a->n_tokens >= 2 ? 2 : 1) : 1;
        const int cbw = codebook_words(tg) + (codebook_words(tg) == codebook_words(tu) ? 0 : codebook_words(tu));
        const size_t lds = (size_t) cbw * 4 + act_lds_bytes(a->layout.n_embd, nt);
        if (lds > (size_t) st.lds_limit) return fail(MAYA_E_SHAPE, "gate/up needs %zu bytes of LDS, the device gives %d", lds, st.lds_limit);
    }
    return MAYA_OK;
}
static int quant_act_refusal(int act_type, const void* x, int x_dtype, int rows, int64_t k, const maya_act& out) {
    if (!type_ok(act_type)) return fail(MAYA_E_UNSUPPORTED, "quant_act: weight type %d", act_type);
    if (x_dtype < 0 || x_dtype > 2) return fail(MAYA_E_UNSUPPORTED, "quant_act: dtype %d", x_dtype);
    if (!x || !out.q || !out.d || !out.bsums) return fail(MAYA_E_ARG, "quant_act: null pointer");
    if (rows <= 0 || rows > 65535 || k <= 0 || k % 256) return fail(MAYA_E_SHAPE, "quant_act: rows %d k %lld", rows, (long long) k);
    return MAYA_OK;
}

static bool down_self_rounding(const maya_moe_args& a) { return !a.hq.q && !a.hq.d && !a.hq.bsums && a.h && a.out && down_rounds_h(a); }
static int down_refusal(const maya_moe_args* a, const DeviceState& st) {
    if (const int rc = check_args(a)) return rc;
    if (down_self_rounding(*a)) return MAYA_OK;
    if (!a->hq.q || !a->hq.d || !a->hq.bsums || !a->part || !a->out) return fail(MAYA_E_ARG, "down: null activation, part or out");
    const bool pos = (a->layout.down_type == kIQ2_S && down_iq2s_fast_ok(*a)) || down_q4k_pos_ok(*a) || down_iq1s_pos_ok(*a) ||
                     down_q80_pos_ok(*a);
    if (!pos) {
        const int nt = a->grp_ptr ? (a->n_tokens >= 4 ? 4 : a->n_tokens >= 2 ? 2 : 1) : 1;
        const size_t lds = (size_t) codebook_words(a->layout.down_type) * 4 + act_lds_bytes(a->layout.n_ff, nt);
        if (lds > (size_t) st.lds_limit) return fail(MAYA_E_SHAPE, "down needs %zu bytes of LDS, the device gives %d", lds, st.lds_limit);
    }
    return MAYA_OK;
}

bool gate_up_by_entries(const maya_moe_args& a) {
    const maya_moe_layout& l = a.layout;
    if (gate_up_q4k_pos_ok(a) || gate_up_iq1s_pos_ok(a)) return true;
    if (!(l.gate_type == kIQ2_S && l.up_type == kIQ2_S && l.packing == MAYA_PACK_STREAM) || l.n_ff % 16 != 0 || l.n_embd % 1024 != 0) return false;
    const int nw = l.n_embd / 1024;
    return nw == 4 || nw == 6 || nw == 7 || nw == 8;
}
bool down_by_entries(const maya_moe_args& a) { return down_q4k_pos_ok(a) || down_rounds_h(a); }

template <int T>
int launch_mv_t(const MvBatch& b, int n, int max_in, int max_out, int max_col, const DeviceState& st, hipStream_t s) {
    int nt = max_col >= 4 ? 4 : max_col >= 2 ? 2 : 1;
    while (nt > 1 && (size_t) codebook_words(T) * 4 + act_lds_bytes(max_in, nt) > (size_t) st.lds_limit) nt >>= 1;   // long rows: fewer columns a pass
    const size_t lds = (size_t) codebook_words(T) * 4 + act_lds_bytes(max_in, nt);
    if (lds > (size_t) st.lds_limit) return fail(MAYA_E_SHAPE, "mv needs %zu bytes of LDS, the device gives %d", lds, st.lds_limit);
    const int wr = rows_per_wg(max_out, n, 16, kDnRows);
    const dim3 grid((unsigned) ((max_out + wr - 1) / wr), (unsigned) n);
    if (nt == 4) hipLaunchKernelGGL((mv_kernel<T, 4>), grid, dim3(kDnThreads), lds, s, b, st.cb, wr);
    else if (nt == 2) hipLaunchKernelGGL((mv_kernel<T, 2>), grid, dim3(kDnThreads), lds, s, b, st.cb, wr);
    else hipLaunchKernelGGL((mv_kernel<T, 1>), grid, dim3(kDnThreads), lds, s, b, st.cb, wr);
    MAYA_LAUNCHED("mv_kernel");
    return MAYA_OK;
}

}  // namespace maya

using namespace maya;

// ================================================================================================= C ABI

extern "C" {

const char* maya_last_error(void) { return g_err; }

int maya_init(void) {
    DeviceState* st;
    return current_state(&st);
}

const char* maya_device_info(void) {
    static thread_local char buf[256];
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&p, dev) != hipSuccess) {
        snprintf(buf, sizeof buf, "no device");
        return buf;
    }
    snprintf(buf, sizeof buf, "%s %s cus=%d lds=%zu clock_khz=%d mem_clock_khz=%d bus_bits=%d", p.gcnArchName, p.name,
             p.multiProcessorCount, p.sharedMemPerBlock, p.clockRate, p.memoryClockRate, p.memoryBusWidth);
    return buf;
}

int maya_moe_supported(int t) { return type_ok(t) ? 1 : 0; }
int maya_moe_block_bytes(int t) { return block_bytes(t); }
int maya_moe_block_values(int t) { return block_values(t); }
size_t maya_moe_row_bytes(int t, int64_t k) {
    return type_ok(t) && k % block_values(t) == 0 ? (size_t) (k / block_values(t)) * (size_t) block_bytes(t) : 0;
}
size_t maya_moe_layout_init(maya_moe_layout* l, int gate_type, int up_type, int down_type, int n_embd, int n_ff) {
    if (!l) return 0;
    l->gate_type = gate_type;
    l->up_type = up_type;
    l->down_type = down_type;
    l->n_embd = n_embd;
    l->n_ff = n_ff;
    l->gate_off = l->up_off = l->down_off = 0;
    l->packing = MAYA_PACK_GGUF;
    l->reserved = 0;
    if (check_layout(*l) != MAYA_OK) return 0;
    l->up_off = maya_moe_row_bytes(gate_type, n_embd) * (size_t) n_ff;
    l->down_off = l->up_off + maya_moe_row_bytes(up_type, n_embd) * (size_t) n_ff;
    return l->down_off + maya_moe_row_bytes(down_type, n_ff) * (size_t) n_embd;
}

// dir 0: the blobs' GGUF row arrays -> stream order, 1: back, 2: a plain copy.  role i of blob b is read at
// src[i] + b * src_stride[i] and written at dst[i] + b * dst_stride.
static int repack_impl(const maya_moe_layout* l, const uint8_t* const (&src)[3], const size_t (&src_stride)[3], uint8_t* const (&dst)[3],
                       size_t dst_stride, int n_blobs, void* stream, int dir) {
    hipStream_t s = as_stream(stream);
    const struct { int type; int64_t k, rows; } roles[3] = {
        {l->gate_type, l->n_embd, l->n_ff}, {l->up_type, l->n_embd, l->n_ff}, {l->down_type, l->n_ff, l->n_embd}};
    for (int i = 0; i < 3; ++i) {
        const auto& r = roles[i];
        const uint8_t* sp = src[i];
        uint8_t* dp = dst[i];
        const size_t ss = src_stride[i], ds = dst_stride;
        const dim3 grid((unsigned) (((r.k >> 5) + 255) / 256), (unsigned) r.rows, (unsigned) n_blobs);
        if (dir == 2 || !(quad_packed(r.type) || r.type == kQ8_0)) {
            const size_t n = maya_moe_row_bytes(r.type, r.k) * (size_t) r.rows;
            hipLaunchKernelGGL(copy_bytes_kernel, dim3(256, 1, (unsigned) n_blobs), dim3(256), 0, s, sp, dp, n, ss, ds);
        } else if (r.type == kIQ2_S) {
            if (dir == 0) hipLaunchKernelGGL(repack_iq2s_kernel<0>, grid, dim3(256), 0, s, sp, dp, r.k, r.rows, ss, ds);
            else hipLaunchKernelGGL(repack_iq2s_kernel<1>, grid, dim3(256), 0, s, sp, dp, r.k, r.rows, ss, ds);
        } else if (r.type == kIQ1_S) {
            if (dir == 0) hipLaunchKernelGGL(repack_iq1s_kernel<0>, grid, dim3(256), 0, s, sp, dp, r.k, r.rows, ss, ds);
            else hipLaunchKernelGGL(repack_iq1s_kernel<1>, grid, dim3(256), 0, s, sp, dp, r.k, r.rows, ss, ds);
        } else if (r.type == kIQ1_M) {
            if (dir == 0) hipLaunchKernelGGL(repack_iq1m_kernel<0>, grid, dim3(256), 0, s, sp, dp, r.k, r.rows, ss, ds);
            else hipLaunchKernelGGL(repack_iq1m_kernel<1>, grid, dim3(256), 0, s, sp, dp, r.k, r.rows, ss, ds);
        } else {
            if (dir == 0) hipLaunchKernelGGL(repack_q80_kernel<0>, grid, dim3(256), 0, s, sp, dp, r.k, r.rows, ss, ds);
            else hipLaunchKernelGGL(repack_q80_kernel<1>, grid, dim3(256), 0, s, sp, dp, r.k, r.rows, ss, ds);
        }
        MAYA_LAUNCHED("repack kernel");
    }
    return MAYA_OK;
}
static int repack_blob(const maya_moe_layout* l, const void* src, void* dst, void* stream, int dir) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!l || !src || !dst) return fail(MAYA_E_ARG, "repack: null pointer");
    if (const int rc = check_layout(*l)) return rc;
    if (l->packing != MAYA_PACK_GGUF) return fail(MAYA_E_ARG, "repack: the layout must describe the GGUF blob");
    const uint8_t* sp = (const uint8_t*) src;
    uint8_t* dp = (uint8_t*) dst;
    const uint8_t* const srcs[3] = {sp + l->gate_off, sp + l->up_off, sp + l->down_off};
    uint8_t* const dsts[3] = {dp + l->gate_off, dp + l->up_off, dp + l->down_off};
    const size_t strides[3] = {0, 0, 0};
    return repack_impl(l, srcs, strides, dsts, 0, 1, stream, dir);
}
int maya_moe_repack(const maya_moe_layout* l, const void* src, void* dst, void* stream) { return repack_blob(l, src, dst, stream, 0); }
int maya_moe_unpack(const maya_moe_layout* l, const void* src, void* dst, void* stream) { return repack_blob(l, src, dst, stream, 1); }

int maya_moe_pack_experts(const maya_moe_layout* l, const void* gate_exps, const void* up_exps, const void* down_exps, int n_expert,
                          int packing, void* dst, size_t dst_stride, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!l || !gate_exps || !up_exps || !down_exps || !dst) return fail(MAYA_E_ARG, "pack_experts: null pointer");
    if (const int rc = check_layout(*l)) return rc;
    if (l->packing != MAYA_PACK_GGUF) return fail(MAYA_E_ARG, "pack_experts: the layout must describe the GGUF blob");
    if (packing != MAYA_PACK_GGUF && packing != MAYA_PACK_STREAM) return fail(MAYA_E_UNSUPPORTED, "pack_experts: packing %d", packing);
    if (n_expert <= 0 || n_expert > 65535) return fail(MAYA_E_SHAPE, "pack_experts: %d experts", n_expert);
    const size_t gb = maya_moe_row_bytes(l->gate_type, l->n_embd) * (size_t) l->n_ff, ub = maya_moe_row_bytes(l->up_type, l->n_embd) * (size_t) l->n_ff;
    const size_t db = maya_moe_row_bytes(l->down_type, l->n_ff) * (size_t) l->n_embd;
    if (dst_stride < l->down_off + db) return fail(MAYA_E_SHAPE, "pack_experts: blobs %zu bytes apart hold %zu", dst_stride, (size_t) (l->down_off + db));
    if (packing == MAYA_PACK_STREAM && ((((uintptr_t) dst | dst_stride | l->gate_off | l->up_off | l->down_off) & 15) ||
                                        ((l->n_ff | l->n_embd) & 3)))
        return fail(MAYA_E_ARG, "pack_experts: stream packing wants 16-byte aligned blobs and row arrays, rows in fours");
    uint8_t* dp = (uint8_t*) dst;
    const uint8_t* const srcs[3] = {(const uint8_t*) gate_exps, (const uint8_t*) up_exps, (const uint8_t*) down_exps};
    uint8_t* const dsts[3] = {dp + l->gate_off, dp + l->up_off, dp + l->down_off};
    const size_t strides[3] = {gb, ub, db};
    return repack_impl(l, srcs, strides, dsts, dst_stride, n_expert, stream, packing == MAYA_PACK_STREAM ? 0 : 2);
}

int maya_dequant_rows(int t, const void* w, size_t row_stride, int64_t k, int64_t n_rows, float* out, void* stream) {
    return maya_dequant_rows_packed(t, MAYA_PACK_GGUF, w, row_stride, k, n_rows, out, stream);
}

int maya_dequant_rows_packed(int t, int packing, const void* w, size_t row_stride, int64_t k, int64_t n_rows, float* out,
                             void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!type_ok(t)) return fail(MAYA_E_UNSUPPORTED, "dequant: type %d", t);
    if (packing != MAYA_PACK_GGUF && packing != MAYA_PACK_STREAM) return fail(MAYA_E_UNSUPPORTED, "dequant: packing %d", packing);
    if (!w || !out) return fail(MAYA_E_ARG, "dequant: null pointer");
    if (k <= 0 || k % block_values(t) || n_rows <= 0 || n_rows > 65535 || (packing == MAYA_PACK_STREAM && n_rows % 4))
        return fail(MAYA_E_SHAPE, "dequant: k %lld rows %lld", (long long) k, (long long) n_rows);
    if (row_stride == 0) row_stride = maya_moe_row_bytes(t, k);
    const dim3 grid((unsigned) ((k + 255) / 256), (unsigned) n_rows);
    const uint8_t* wb = (const uint8_t*) w;
    hipStream_t s = as_stream(stream);
    switch (t) {
        case kQ8_0: hipLaunchKernelGGL(dequant_kernel<kQ8_0>, grid, dim3(256), 0, s, wb, row_stride, k, out, st->cb, packing); break;
        case kQ4_K: hipLaunchKernelGGL(dequant_kernel<kQ4_K>, grid, dim3(256), 0, s, wb, row_stride, k, out, st->cb, packing); break;
        case kIQ2_S: hipLaunchKernelGGL(dequant_kernel<kIQ2_S>, grid, dim3(256), 0, s, wb, row_stride, k, out, st->cb, packing); break;
        case kIQ1_S: hipLaunchKernelGGL(dequant_kernel<kIQ1_S>, grid, dim3(256), 0, s, wb, row_stride, k, out, st->cb, packing); break;
        case kIQ2_XXS: hipLaunchKernelGGL(dequant_kernel<kIQ2_XXS>, grid, dim3(256), 0, s, wb, row_stride, k, out, st->cb, packing); break;
        default: hipLaunchKernelGGL(dequant_kernel<kIQ1_M>, grid, dim3(256), 0, s, wb, row_stride, k, out, st->cb, packing); break;
    }
    MAYA_LAUNCHED("dequant_kernel");
    return MAYA_OK;
}

int maya_quant_act(int act_type, const void* x, int x_dtype, int64_t x_stride, int rows, int64_t k, maya_act out,
                   void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (const int rc = quant_act_refusal(act_type, x, x_dtype, rows, k, out)) return rc;
    if (x_stride == 0) x_stride = k;
    const dim3 grid((unsigned) (k / 256), (unsigned) rows);
    hipStream_t s = as_stream(stream);
#define MAYA_Q(KERNEL)                                                                                              \
    switch (x_dtype) {                                                                                              \
        case MAYA_DT_F32: hipLaunchKernelGGL(KERNEL<MAYA_DT_F32>, grid, dim3(256), 0, s, x, x_stride, k, out); break;   \
        case MAYA_DT_BF16: hipLaunchKernelGGL(KERNEL<MAYA_DT_BF16>, grid, dim3(256), 0, s, x, x_stride, k, out); break; \
        default: hipLaunchKernelGGL(KERNEL<MAYA_DT_F16>, grid, dim3(256), 0, s, x, x_stride, k, out); break;            \
    }
    if (q8k_act(act_type)) {
        MAYA_Q(quant_q8k_kernel)
    } else {
        MAYA_Q(quant_q80_kernel)
    }
#undef MAYA_Q
    MAYA_LAUNCHED("quant_act kernel");
    return MAYA_OK;
}

int maya_quant_i8x32(const void* x, int x_dtype, int64_t x_stride, const int32_t* row_idx, int rows, int64_t k, int8_t* q,
                     float* d, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (x_dtype < 0 || x_dtype > 2) return fail(MAYA_E_UNSUPPORTED, "quant_i8x32: dtype %d", x_dtype);
    if (!x || !q || !d) return fail(MAYA_E_ARG, "quant_i8x32: null pointer");
    if (rows <= 0 || rows > 65535 || k <= 0 || k % 256) return fail(MAYA_E_SHAPE, "quant_i8x32: rows %d k %lld", rows, (long long) k);
    if (x_stride == 0) x_stride = k;
    const dim3 grid((unsigned) (k / 256), (unsigned) rows);
    hipStream_t s = as_stream(stream);
    switch (x_dtype) {
        case MAYA_DT_F32: hipLaunchKernelGGL(quant_i8x32_kernel<MAYA_DT_F32>, grid, dim3(256), 0, s, x, x_stride, row_idx, k, q, d); break;
        case MAYA_DT_BF16: hipLaunchKernelGGL(quant_i8x32_kernel<MAYA_DT_BF16>, grid, dim3(256), 0, s, x, x_stride, row_idx, k, q, d); break;
        default: hipLaunchKernelGGL(quant_i8x32_kernel<MAYA_DT_F16>, grid, dim3(256), 0, s, x, x_stride, row_idx, k, q, d); break;
    }
    MAYA_LAUNCHED("quant_i8x32_kernel");
    return MAYA_OK;
}

static int route_impl(const char* what, const float* logits, int n_tokens, int n_expert, int k, const RouterSpec& r, int32_t* ids,
                      float* weights, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!logits || !ids || !weights) return fail(MAYA_E_ARG, "%s: null pointer", what);
    if (n_tokens <= 0 || n_tokens > 65535 || n_expert <= 0 || n_expert > MAYA_MAX_EXPERTS || k <= 0 || k > MAYA_MAX_K || k > n_expert)
        return fail(MAYA_E_SHAPE, "%s: tokens %d experts %d k %d (limits %d experts, k %d)", what, n_tokens, n_expert, k,
                    MAYA_MAX_EXPERTS, MAYA_MAX_K);
    hipLaunchKernelGGL(router_kernel, dim3((unsigned) n_tokens), dim3(256), 0, as_stream(stream), logits, n_expert, k, r, ids, weights);
    MAYA_LAUNCHED("router_kernel");
    return MAYA_OK;
}
static bool router_spec(const maya_router* r, RouterSpec& s) {
    s = RouterSpec{nullptr, 1.0f, MAYA_ROUTER_SOFTMAX, 1};
    if (!r) return true;
    if (r->kind != MAYA_ROUTER_SOFTMAX && r->kind != MAYA_ROUTER_SIGMOID) return false;
    if (r->kind == MAYA_ROUTER_SIGMOID) {
        if (r->norm < 0 || r->norm > 2) return false;
        s = RouterSpec{r->bias, r->w_scale, MAYA_ROUTER_SIGMOID, r->norm};
    }
    return true;
}
int maya_moe_route_topk(const float* logits, int n_tokens, int n_expert, int k, int32_t* ids, float* weights,
                        void* stream) {
    return route_impl("route_topk", logits, n_tokens, n_expert, k, RouterSpec{nullptr, 1.0f, MAYA_ROUTER_SOFTMAX, 1}, ids, weights, stream);
}
int maya_moe_route_sigmoid(const float* logits, const float* bias, int n_tokens, int n_expert, int k, float w_scale, int norm,
                           int32_t* ids, float* weights, void* stream) {
    if (norm < 0 || norm > 2) return fail(MAYA_E_UNSUPPORTED, "route_sigmoid: normalisation %d", norm);
    return route_impl("route_sigmoid", logits, n_tokens, n_expert, k, RouterSpec{bias, w_scale, MAYA_ROUTER_SIGMOID, norm}, ids, weights, stream);
}

int maya_moe_route_plan(const maya_router* router, const float* logits, int n_tokens, int n_expert, int k, const uint64_t* expert_table,
                        int32_t* ids, float* weights, uint64_t* plan_ptr, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    RouterSpec rs;
    if (!router_spec(router, rs)) return fail(MAYA_E_UNSUPPORTED, "route_plan: router kind %d / normalisation %d", router->kind, router->norm);
    if (!logits || !expert_table || !ids || !weights || !plan_ptr) return fail(MAYA_E_ARG, "route_plan: null pointer");
    if (n_tokens <= 0 || n_tokens > 65535 || n_expert <= 0 || n_expert > MAYA_MAX_EXPERTS || k <= 0 || k > MAYA_MAX_K || k > n_expert)
        return fail(MAYA_E_SHAPE, "route_plan: tokens %d experts %d k %d (limits %d experts, k %d)", n_tokens, n_expert, k, MAYA_MAX_EXPERTS, MAYA_MAX_K);
    // (the layer head's routing workgroup alone: no activation blocks)
    hipLaunchKernelGGL(layer_head_kernel<MAYA_DT_F32>, dim3(1, (unsigned) n_tokens), dim3(256), 0, as_stream(stream), logits, n_expert, k, rs,
                       expert_table, ids, weights, plan_ptr, nullptr, (int64_t) 0, maya_act{nullptr, nullptr, nullptr});
    MAYA_LAUNCHED("layer_head_kernel");
    return MAYA_OK;
}

int maya_moe_route_window_ok(const maya_router* router, int n_tokens, int n_expert, int k) {
    return (!router || router->kind == MAYA_ROUTER_SOFTMAX) && n_tokens >= 1 && n_tokens <= MAYA_MAX_TOKENS && n_expert >= 1 && n_expert <= 256 &&
           k >= 1 && k <= MAYA_MAX_K && k <= n_expert && n_tokens * k <= 256;
}
int maya_moe_route_window(const maya_router* router, const float* logits, int n_tokens, int n_expert, int k, const uint64_t* expert_table,
                          int32_t* ids, float* weights, uint64_t* plan_ptr, uint64_t* grp_ptr, int32_t* grp_start, int32_t* grp_ent,
                          int32_t* n_groups, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!logits || !expert_table || !ids || !weights || !plan_ptr || !grp_ptr || !grp_start || !grp_ent || !n_groups)
        return fail(MAYA_E_ARG, "route_window: null pointer");
    if (!maya_moe_route_window_ok(router, n_tokens, n_expert, k))
        return fail(MAYA_E_UNSUPPORTED, "route_window: the softmax router, up to 256 experts and 256 entries (tokens %d experts %d k %d)", n_tokens, n_expert, k);
    hipLaunchKernelGGL(window_head_kernel<MAYA_DT_F32>, dim3(1, 1), dim3(256), 0, as_stream(stream), logits, n_expert, k, n_tokens, expert_table, ids,
                       weights, plan_ptr, grp_ptr, grp_start, grp_ent, n_groups, nullptr, (int64_t) 0, maya_act{nullptr, nullptr, nullptr});
    MAYA_LAUNCHED("window_head_kernel");
    return MAYA_OK;
}

int maya_moe_route_tiered(const maya_router* router, const float* logits, int n_tokens, int layer, int n_expert, int k,
                          const maya_residency* r, int promote_min, int32_t* ids, float* weights, uint64_t* plan_ptr, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    RouterSpec rs;
    if (!router_spec(router, rs)) return fail(MAYA_E_UNSUPPORTED, "route_tiered: router kind %d / normalisation %d", router->kind, router->norm);
    if (!logits || !r || !r->tab || !r->fetch_src || !r->masks || !ids || !weights || !plan_ptr || (r->n_scratch > 0 && !r->scratch))
        return fail(MAYA_E_ARG, "route_tiered: null pointer");
    if (n_tokens <= 0 || n_tokens > 256 || n_expert <= 0 || n_expert > MAYA_MAX_EXPERTS || k <= 0 || k > MAYA_MAX_K || k > n_expert)
        return fail(MAYA_E_SHAPE, "route_tiered: tokens %d experts %d k %d (limits 256 tokens, %d experts, k %d)", n_tokens, n_expert, k,
                    MAYA_MAX_EXPERTS, MAYA_MAX_K);
    if (r->n_layers <= 0 || layer < 0 || layer >= r->n_layers || r->n_scratch < 0 || (int64_t) r->n_layers * n_expert != (int64_t) r->n_keys)
        return fail(MAYA_E_SHAPE, "route_tiered: layer %d of %d, %d keys for %d experts a layer, %d scratch slots", layer, r->n_layers,
                    r->n_keys, n_expert, r->n_scratch);
    const Tiers tr{r->tab, r->scratch, r->fetch_src, r->counts, r->seq, r->masks, r->n_keys, r->n_scratch};
    if (n_tokens > 1 && n_tokens * k <= 256) {
        // a window: the tokens routed side by side, then one workgroup plans their entries in order
        hipLaunchKernelGGL(router_kernel, dim3((unsigned) n_tokens), dim3(256), 0, as_stream(stream), logits, n_expert, k, rs, ids, weights);
        MAYA_LAUNCHED("router_kernel");
        hipLaunchKernelGGL(plan_tiered_kernel, dim3(1), dim3(256), 0, as_stream(stream), (const int32_t*) ids, n_tokens, n_expert, k, layer, tr,
                           promote_min, plan_ptr);
        MAYA_LAUNCHED("plan_tiered_kernel");
        return MAYA_OK;
    }
    hipLaunchKernelGGL(route_tiered_kernel, dim3(1), dim3(256), 0, as_stream(stream), logits, n_tokens, n_expert, k, rs, layer, tr,
                       promote_min, ids, weights, plan_ptr);
    MAYA_LAUNCHED("route_tiered_kernel");
    return MAYA_OK;
}

int maya_moe_fetch(const uint64_t* fetch_src, const uint64_t* plan_ptr, int n_entries, size_t blob_bytes, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!fetch_src || !plan_ptr) return fail(MAYA_E_ARG, "fetch: null pointer");
    if (n_entries <= 0 || n_entries > 65535 || blob_bytes == 0) return fail(MAYA_E_SHAPE, "fetch: %d entries of %zu bytes", n_entries, blob_bytes);
    // (slices of at least 64 KB, at most 256 of them a blob: an entry with nothing to fetch costs its workgroups a load)
    const unsigned slices = (unsigned) std::min<size_t>(256, (blob_bytes + 65535) / 65536);
    hipLaunchKernelGGL(fetch_kernel, dim3(slices, (unsigned) n_entries), dim3(256), 0, as_stream(stream), fetch_src, plan_ptr, blob_bytes);
    MAYA_LAUNCHED("fetch_kernel");
    return MAYA_OK;
}

int maya_moe_prefetch(const uint64_t* pf_src, const uint64_t* pf_dst, const int32_t* pf_n, int max_entries, size_t blob_bytes,
                      int n_workgroups, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!pf_src || !pf_dst || !pf_n) return fail(MAYA_E_ARG, "prefetch: null pointer");
    if (max_entries <= 0 || max_entries > 65535 || blob_bytes == 0 || n_workgroups < 0 || n_workgroups > 65535)
        return fail(MAYA_E_SHAPE, "prefetch: up to %d entries of %zu bytes by %d workgroups", max_entries, blob_bytes, n_workgroups);
    // (0: half the compute units, the reference's default)
    const unsigned wgs = n_workgroups > 0 ? (unsigned) n_workgroups : (unsigned) std::max(1, st->n_cu / 2);
    hipLaunchKernelGGL(prefetch_kernel, dim3(wgs), dim3(256), 0, as_stream(stream), pf_src, pf_dst, pf_n, max_entries, blob_bytes);
    MAYA_LAUNCHED("prefetch_kernel");
    return MAYA_OK;
}

int maya_moe_tab_update(uint64_t* tab, int n_words, const int32_t* keys, const uint64_t* vals, int n, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (n == 0) return MAYA_OK;
    if (!tab || !keys || !vals) return fail(MAYA_E_ARG, "tab_update: null pointer");
    if (n < 0 || n_words <= 0) return fail(MAYA_E_SHAPE, "tab_update: %d edits of %d words", n, n_words);
    hipLaunchKernelGGL(tab_update_kernel, dim3((unsigned) ((n + 255) / 256)), dim3(256), 0, as_stream(stream), tab, keys, vals, n, n_words);
    MAYA_LAUNCHED("tab_update_kernel");
    return MAYA_OK;
}

int maya_moe_plan(const int32_t* ids, int n_entries, const uint64_t* expert_table, int n_expert, uint64_t* plan_ptr,
                  void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!ids || !expert_table || !plan_ptr) return fail(MAYA_E_ARG, "plan: null pointer");
    if (n_entries <= 0 || n_expert <= 0) return fail(MAYA_E_SHAPE, "plan: entries %d experts %d", n_entries, n_expert);
    hipLaunchKernelGGL(plan_kernel, dim3((unsigned) ((n_entries + 255) / 256)), dim3(256), 0, as_stream(stream), ids, n_entries,
                       expert_table, n_expert, plan_ptr);
    MAYA_LAUNCHED("plan_kernel");
    return MAYA_OK;
}

int maya_moe_group(const uint64_t* plan_ptr, int n_entries, uint64_t* grp_ptr, int32_t* grp_start, int32_t* grp_ent,
                   int32_t* n_groups, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!plan_ptr || !grp_ptr || !grp_start || !grp_ent || !n_groups) return fail(MAYA_E_ARG, "group: null pointer");
    if (n_entries <= 0 || n_entries > 256) return fail(MAYA_E_SHAPE, "group: %d entries outside 1..256", n_entries);
    hipLaunchKernelGGL(group_kernel, dim3(1), dim3(256), 0, as_stream(stream), plan_ptr, n_entries, grp_ptr, grp_start, grp_ent, n_groups);
    MAYA_LAUNCHED("group_kernel");
    return MAYA_OK;
}

int maya_moe_gate_up(const maya_moe_args* a, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (const int rc = gate_up_refusal(a, *st)) return rc;
    hipStream_t s = as_stream(stream);
    const int tg = a->layout.gate_type, tu = a->layout.up_type;
    if (tg == kIQ2_S && tu == kIQ2_S) {
        int rc = 0;
        if (try_gate_up_iq2s_1tok(*a, *st, s, &rc)) return rc;
    }
    if (gate_up_q4k_pos_ok(*a)) return launch_gate_up_q4k_pos(*a, s);
    if (gate_up_iq1s_pos_ok(*a)) return launch_gate_up_iq1s_pos(*a, *st, s);
    if (gate_up_q80_pos_ok(*a)) return launch_gate_up_q80_pos(*a, s);
#define MAYA_GU(TG, TU) if (tg == TG && tu == TU) return launch_gate_up_t<TG, TU>(*a, *st, s);
    MAYA_GU(kIQ2_S, kIQ2_S)
    MAYA_GU(kQ4_K, kQ4_K)
    MAYA_GU(kQ8_0, kQ8_0)
    MAYA_GU(kIQ1_S, kIQ1_S)
    MAYA_GU(kIQ1_M, kIQ1_M)
    MAYA_GU(kIQ2_XXS, kIQ2_XXS)
    MAYA_GU(kIQ2_S, kIQ1_M)
    MAYA_GU(kIQ1_M, kIQ2_S)
    MAYA_GU(kIQ2_S, kQ4_K)
    MAYA_GU(kIQ1_S, kIQ1_M)
    MAYA_GU(kIQ1_M, kIQ1_S)
#undef MAYA_GU
    return fail(MAYA_E_UNSUPPORTED, "gate_up: no kernel for gate type %d with up type %d", tg, tu);
}

int maya_moe_down_rounds_h(const maya_moe_args* a) { return a && down_rounds_h(*a) ? 1 : 0; }

int maya_moe_down(const maya_moe_args* a, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (const int rc = down_refusal(a, *st)) return rc;
    if (down_self_rounding(*a)) {
        int rc = 0;   // the kernel rounds h itself
        if (a->layout.down_type == kQ4_K) return launch_down_q4k_pos(*a, as_stream(stream));
        if (a->layout.down_type == kIQ1_S || a->layout.down_type == kIQ1_M) return launch_down_iq1s_pos(*a, *st, as_stream(stream));
        if (try_down_iq2s_1tok(*a, *st, as_stream(stream), &rc)) return rc;
    }
    if (!a->hq.q || !a->hq.d || !a->hq.bsums || !a->part || !a->out) return fail(MAYA_E_ARG, "down: null activation, part or out");
    hipStream_t s = as_stream(stream);
    if (a->layout.down_type == kIQ2_S) {
        int rc = 0;
        if (try_down_iq2s_1tok(*a, *st, s, &rc)) return rc;
    }
    if (down_q4k_pos_ok(*a)) return launch_down_q4k_pos(*a, s);
    if (down_iq1s_pos_ok(*a)) return launch_down_iq1s_pos(*a, *st, s);
    if (down_q80_pos_ok(*a)) {
        if (const int rc = launch_down_q80_pos(*a, s)) return rc;
        const dim3 cgrid((unsigned) ((a->layout.n_embd + 255) / 256), (unsigned) a->n_tokens);
        hipLaunchKernelGGL(combine_kernel, cgrid, dim3(256), 0, s, *a);
        MAYA_LAUNCHED("combine_kernel");
        return MAYA_OK;
    }
    int rc;
    switch (a->layout.down_type) {
        case kIQ2_S: rc = launch_down_t<kIQ2_S>(*a, *st, s); break;
        case kQ4_K: rc = launch_down_t<kQ4_K>(*a, *st, s); break;
        case kQ8_0: rc = launch_down_t<kQ8_0>(*a, *st, s); break;
        case kIQ1_S: rc = launch_down_t<kIQ1_S>(*a, *st, s); break;
        case kIQ2_XXS: rc = launch_down_t<kIQ2_XXS>(*a, *st, s); break;
        default: rc = launch_down_t<kIQ1_M>(*a, *st, s); break;
    }
    if (rc) return rc;
    const dim3 grid((unsigned) ((a->layout.n_embd + 255) / 256), (unsigned) a->n_tokens);
    hipLaunchKernelGGL(combine_kernel, grid, dim3(256), 0, s, *a);
    MAYA_LAUNCHED("combine_kernel");
    return MAYA_OK;
}

}  // extern "C"

namespace maya {
// rows of 1024 NW values (NW 2 .. 8) in whole groups of 16 row pairs; Q8_0 in the stream packing, Q4_K 16-byte aligned
static bool mv_pos_ok(const maya_mv_job& j) {
    const int nw = j.n_in / 1024;
    if (j.n_in % 1024 || nw < 2 || nw > 8 || j.n_out % 32 || ((uintptr_t) j.w & 15)) return false;
    if ((size_t) j.n_out * maya_moe_row_bytes(j.type, j.n_in) >= (1ull << 32)) return false;   // (32-bit buffer offsets)
    if (j.type == kQ8_0) return j.packing == MAYA_PACK_STREAM;
    return j.type == kQ4_K;
}
template <int NW>
static void launch_mv_pos_nw(const maya_mv_job& j, hipStream_t s) {
    const MvPos a{(const uint8_t*) j.w, j.x, j.bias, j.y, (long long) j.y_stride, j.alpha, j.n_out, j.ncol};
    // 16 row pairs a workgroup when that still gives two workgroups a compute unit, else 8
    const bool big = j.n_out / 32 >= 512;
    if (j.type == kQ4_K) {
        if (big) hipLaunchKernelGGL((mv_q4k_pos_kernel<NW, 16>), dim3((unsigned) (j.n_out / 32), (unsigned) j.ncol), dim3(64 * NW), 0, s, a);
        else hipLaunchKernelGGL((mv_q4k_pos_kernel<NW, 8>), dim3((unsigned) (j.n_out / 16), (unsigned) j.ncol), dim3(64 * NW), 0, s, a);
    } else {
        const unsigned g16 = (unsigned) (j.n_out / 32), g8 = (unsigned) (j.n_out / 16);
        if (j.ncol == 1) {
            if (big) hipLaunchKernelGGL((mv_q80_pos_kernel<NW, 1, 16>), dim3(g16), dim3(64 * NW), 0, s, a);
            else hipLaunchKernelGGL((mv_q80_pos_kernel<NW, 1, 8>), dim3(g8), dim3(64 * NW), 0, s, a);
        } else if (j.ncol == 2) {
            if (big) hipLaunchKernelGGL((mv_q80_pos_kernel<NW, 2, 16>), dim3(g16), dim3(64 * NW), 0, s, a);
            else hipLaunchKernelGGL((mv_q80_pos_kernel<NW, 2, 8>), dim3(g8), dim3(64 * NW), 0, s, a);
        } else if (j.ncol <= 4) {
            if (big) hipLaunchKernelGGL((mv_q80_pos_kernel<NW, 4, 16>), dim3(g16), dim3(64 * NW), 0, s, a);
            else hipLaunchKernelGGL((mv_q80_pos_kernel<NW, 4, 8>), dim3(g8), dim3(64 * NW), 0, s, a);
        } else {
            if (big) hipLaunchKernelGGL((mv_q80_pos_kernel<NW, 8, 16>), dim3(g16), dim3(64 * NW), 0, s, a);
            else hipLaunchKernelGGL((mv_q80_pos_kernel<NW, 8, 8>), dim3(g8), dim3(64 * NW), 0, s, a);
        }
    }
}
static void launch_mv_pos(const maya_mv_job& j, hipStream_t s) {
    switch (j.n_in / 1024) {
        case 2: launch_mv_pos_nw<2>(j, s); break;
        case 3: launch_mv_pos_nw<3>(j, s); break;
        case 4: launch_mv_pos_nw<4>(j, s); break;
        case 5: launch_mv_pos_nw<5>(j, s); break;
        case 6: launch_mv_pos_nw<6>(j, s); break;
        case 7: launch_mv_pos_nw<7>(j, s); break;
        default: launch_mv_pos_nw<8>(j, s); break;
    }
}
}  // namespace maya

extern "C" {

int maya_mv_supported(int type) { return type_ok(type) ? 1 : 0; }

int maya_mv(const maya_mv_job* jobs, int n_jobs, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!jobs || n_jobs < 1 || n_jobs > MAYA_MV_MAX_JOBS) return fail(MAYA_E_ARG, "mv: %d jobs outside 1..%d", n_jobs, MAYA_MV_MAX_JOBS);
    for (int i = 0; i < n_jobs; ++i) {   // nothing is launched unless every job is covered
        const maya_mv_job& j = jobs[i];
        if (!type_ok(j.type)) return fail(MAYA_E_UNSUPPORTED, "mv: job %d: weight type %d is not covered", i, j.type);
        if (j.packing != MAYA_PACK_GGUF && j.packing != MAYA_PACK_STREAM) return fail(MAYA_E_ARG, "mv: job %d: packing %d", i, j.packing);
        if (j.n_in < 256 || j.n_in % 256 || j.n_in > 16384 || j.n_out < 1)
            return fail(MAYA_E_SHAPE, "mv: job %d: n_in %d (a multiple of 256 up to 16384) / n_out %d", i, j.n_in, j.n_out);
        if (j.ncol < 1 || j.ncol > MAYA_MAX_TOKENS) return fail(MAYA_E_SHAPE, "mv: job %d: ncol %d outside 1..%d", i, j.ncol, MAYA_MAX_TOKENS);
        if (j.packing == MAYA_PACK_STREAM && quad_packed(j.type) && j.n_out % 4)
            return fail(MAYA_E_SHAPE, "mv: job %d: stream-packed IQ2_S / IQ1_S / IQ1_M rows come in quads, n_out %d", i, j.n_out);
        if (j.packing == MAYA_PACK_STREAM && ((uintptr_t) j.w & 15)) return fail(MAYA_E_ARG, "mv: job %d: stream-packed weights must be 16-byte aligned", i);
        if (!j.w || !j.x.q || !j.x.d || (q8k_act(j.type) && !j.x.bsums) || !j.y) return fail(MAYA_E_ARG, "mv: job %d: null pointer", i);
        if (j.y_stride < j.n_out && j.ncol > 1) return fail(MAYA_E_ARG, "mv: job %d: y_stride %lld below n_out %d", i, (long long) j.y_stride, j.n_out);
    }
    // the position-mapped kernels take the jobs whose shape they cover, a launch each; the others go by type
    bool fast[MAYA_MV_MAX_JOBS];
    for (int i = 0; i < n_jobs; ++i) {
        fast[i] = mv_pos_ok(jobs[i]);
        if (fast[i]) launch_mv_pos(jobs[i], as_stream(stream));
    }
    static const int kTypes[] = {kQ8_0, kQ4_K, kIQ2_XXS, kIQ1_S, kIQ2_S, kIQ1_M};
    for (const int t : kTypes) {
        MvBatch b{};
        int n = 0, max_in = 0, max_out = 0, max_col = 0;
        for (int i = 0; i < n_jobs; ++i) {
            const maya_mv_job& j = jobs[i];
            if (j.type != t || fast[i]) continue;
            b.job[n++] = MvJobDev{(const uint8_t*) j.w, j.x, j.bias, j.y, (long long) j.y_stride, j.alpha, j.n_in, j.n_out, j.ncol, j.packing};
            max_in = j.n_in > max_in ? j.n_in : max_in;
            max_out = j.n_out > max_out ? j.n_out : max_out;
            max_col = j.ncol > max_col ? j.ncol : max_col;
        }
        if (n == 0) continue;
        int rc;
        switch (t) {
            case kQ8_0: rc = launch_mv_t<kQ8_0>(b, n, max_in, max_out, max_col, *st, as_stream(stream)); break;
            case kQ4_K: rc = launch_mv_t<kQ4_K>(b, n, max_in, max_out, max_col, *st, as_stream(stream)); break;
            case kIQ1_S: rc = launch_mv_t<kIQ1_S>(b, n, max_in, max_out, max_col, *st, as_stream(stream)); break;
            case kIQ2_S: rc = launch_mv_t<kIQ2_S>(b, n, max_in, max_out, max_col, *st, as_stream(stream)); break;
            case kIQ2_XXS: rc = launch_mv_t<kIQ2_XXS>(b, n, max_in, max_out, max_col, *st, as_stream(stream)); break;
            default: rc = launch_mv_t<kIQ1_M>(b, n, max_in, max_out, max_col, *st, as_stream(stream)); break;
        }
        if (rc) return rc;
    }
    return MAYA_OK;
}

// Windows of up to this many tokens take window_head_kernel: its one workgroup routes four tokens at a time, so four tokens
// cost one router's time and save the grouping launch (configs[4], 4 tokens: 172.9 -> 171.3 us), eight cost two and lose
// more than the launch saves (configs[2], 8 tokens: 256.0 -> 261.8 us, A/B on one box).
constexpr int kWindowHeadTokens = 4;

// workspace carve-up of maya_moe_layer_decode (every region 256-byte aligned)
struct LayerWs {
    uint64_t *plan_ptr, *grp_ptr;
    int32_t *grp_start, *grp_ent, *n_groups;
    maya_act x, hq;
    float *h, *part;
    size_t bytes;
};
static LayerWs carve(const maya_moe_layout& l, int n_tokens, int k, uint8_t* base) {
    LayerWs w{};
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
    w.x.q = (int8_t*) take((size_t) n_tokens * l.n_embd);
    w.x.d = (float*) take(sizeof(float) * (size_t) n_tokens * (l.n_embd / 32));
    w.x.bsums = (int16_t*) take(sizeof(int16_t) * (size_t) n_tokens * (l.n_embd / 16));
    w.hq.q = (int8_t*) take((size_t) ne * l.n_ff);
    w.hq.d = (float*) take(sizeof(float) * (size_t) ne * (l.n_ff / 32));
    w.hq.bsums = (int16_t*) take(sizeof(int16_t) * (size_t) ne * (l.n_ff / 16));
    w.h = (float*) take(sizeof(float) * (size_t) ne * l.n_ff);
    w.part = (float*) take(sizeof(float) * (size_t) ne * l.n_embd);
    w.bytes = off;
    return w;
}

size_t maya_moe_workspace_bytes(const maya_moe_layout* l, int n_tokens, int k) {
    if (!l || check_layout(*l) != MAYA_OK || n_tokens < 1 || n_tokens > MAYA_MAX_TOKENS || k < 1 || k > MAYA_MAX_K) return 0;
    return carve(*l, n_tokens, k, nullptr).bytes;
}

int maya_moe_layer_decode(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k, const float* logits,
                          const void* x, int x_dtype, int n_tokens, float limit, const float* add, int32_t* ids,
                          float* weights, float* out, void* workspace, size_t workspace_bytes, void* stream) {
    return maya_moe_layer_decode_routed(l, expert_table, n_expert, k, nullptr, logits, x, x_dtype, n_tokens, limit, add, ids, weights,
                                        out, workspace, workspace_bytes, stream);
}
}  // extern "C"

// The layer's launches.  `join`: an event the down launch waits for (the shared expert's output, which `add` then points
// at), *joined set once the stream waits for it.
// The routed layer's refusals (status > 0) and its stage arguments over the carved workspace, without launching anything.
static int layer_setup(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k, const maya_router* router,
                       const float* logits, const void* x, int x_dtype, int n_tokens, float limit, const float* add, int32_t* ids,
                       float* weights, float* out, void* workspace, size_t workspace_bytes, const DeviceState& st, RouterSpec& rs,
                       LayerWs& w, maya_moe_args& a) {
    if (!l) return fail(MAYA_E_ARG, "layer_decode: null layout");
    if (!router_spec(router, rs)) return fail(MAYA_E_UNSUPPORTED, "layer_decode: router kind %d / normalisation %d", router->kind, router->norm);
    if (const int rc = check_layout(*l)) return rc;
    if (!expert_table || !x || !ids || !weights || !out || !workspace) return fail(MAYA_E_ARG, "layer_decode: null pointer");
    if (n_tokens < 1 || n_tokens > MAYA_MAX_TOKENS || k < 1 || k > MAYA_MAX_K)
        return fail(MAYA_E_SHAPE, "layer_decode: n_tokens %d / k %d", n_tokens, k);
    if (((uintptr_t) workspace & 255) != 0) return fail(MAYA_E_ARG, "layer_decode: workspace not 256-byte aligned");
    w = carve(*l, n_tokens, k, (uint8_t*) workspace);
    if (workspace_bytes < w.bytes) return fail(MAYA_E_ARG, "layer_decode: workspace %zu < %zu bytes", workspace_bytes, w.bytes);
    if (logits && k > n_expert) return fail(MAYA_E_SHAPE, "layer_decode: k %d > n_expert %d", k, n_expert);
    if (logits && n_expert > MAYA_MAX_EXPERTS) return fail(MAYA_E_SHAPE, "layer_decode: %d experts, the routers take %d", n_expert, MAYA_MAX_EXPERTS);
    if (const int rc = quant_act_refusal(l->gate_type, x, x_dtype, n_tokens, l->n_embd, w.x)) return rc;
    a = maya_moe_args{};
    a.layout = *l;
    a.n_tokens = n_tokens;
    a.k = k;
    a.plan_ptr = w.plan_ptr;
    a.plan_w = weights;
    a.limit = limit;
    a.x = w.x;
    a.h = w.h;
    a.hq = w.hq;
    a.part = w.part;
    a.add = add;
    a.out = out;
    // (the stage calls' own refusals, on the arguments they will get: grouped beyond one token unless both stages take
    // the entries one by one)
    maya_moe_args probe = a;
    if (n_tokens > 1) {
        probe.grp_ent = w.grp_ent;
        if (!(gate_up_by_entries(a) && down_by_entries(a))) probe.grp_ptr = w.grp_ptr, probe.grp_start = w.grp_start, probe.n_groups = w.n_groups;
    }
    if (const int rc = gate_up_refusal(&probe, st)) return rc;
    if (down_rounds_h(probe)) probe.hq = maya_act{nullptr, nullptr, nullptr}, probe.part = nullptr;
    return down_refusal(&probe, st);
}

enum { kLayerWhole = 0, kLayerBegin = 1, kLayerEnd = 2 };
static int layer_decode_core(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k, const maya_router* router,
                             const float* logits, const void* x, int x_dtype, int n_tokens, float limit, const float* add,
                             int32_t* ids, float* weights, float* out, void* workspace, size_t workspace_bytes, void* stream,
                             hipEvent_t join, bool* joined, int phase = kLayerWhole) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    RouterSpec rs;
    LayerWs w;
    maya_moe_args a;
    const bool head = phase != kLayerEnd, tail = phase != kLayerBegin;
    if (const int rc0 = layer_setup(l, expert_table, n_expert, k, router, logits, x, x_dtype, n_tokens, limit, add, ids, weights, out,
                                    workspace, workspace_bytes, *st, rs, w, a))
        return rc0;
    int rc;
    bool grouped = !head, gate_up_done = !head;
    if (!head) {
        // (the second half of a call made in two: the plan, the groups and h are in the workspace)
    } else if (layer_head_in_gate_up_ok(a, rs, logits, n_expert, x, x_dtype)) {
        // one token of IQ2_S, Q4_K or IQ1_S experts: route, plan, Q8_K of x and gate/up in one launch
        const LayerHeadIn hd{logits, expert_table, x, rs.bias, n_expert, x_dtype, rs.kind == MAYA_ROUTER_SIGMOID ? 1 : 0,
                             LayerHead{ids, weights, w.plan_ptr, rs.w_scale, rs.norm}};
        hipStream_t s = as_stream(stream);
        if ((rc = l->gate_type == kQ4_K   ? launch_gate_up_q4k_pos(a, s, &hd)
                  : l->gate_type == kIQ2_S ? launch_layer_gate_up_iq2s(a, hd, *st, s)
                                           : launch_gate_up_iq1s_pos(a, *st, s, &hd)))
            return rc;
        gate_up_done = true;
    } else if (logits && q8k_act(l->gate_type) && n_expert <= MAYA_MAX_EXPERTS && x_dtype >= 0 && x_dtype <= 2 && n_tokens > 1 &&
        n_tokens <= kWindowHeadTokens && maya_moe_route_window_ok(router, n_tokens, n_expert, k)) {
        // a window, one launch: route every token, plan, group, Q8_K of x
        const dim3 grid((unsigned) (1 + l->n_embd / 256), (unsigned) n_tokens);
        hipStream_t s = as_stream(stream);
        switch (x_dtype) {
            case MAYA_DT_F32: hipLaunchKernelGGL(window_head_kernel<MAYA_DT_F32>, grid, dim3(256), 0, s, logits, n_expert, k, n_tokens, expert_table, ids, weights, w.plan_ptr, w.grp_ptr, w.grp_start, w.grp_ent, w.n_groups, x, (int64_t) l->n_embd, w.x); break;
            case MAYA_DT_BF16: hipLaunchKernelGGL(window_head_kernel<MAYA_DT_BF16>, grid, dim3(256), 0, s, logits, n_expert, k, n_tokens, expert_table, ids, weights, w.plan_ptr, w.grp_ptr, w.grp_start, w.grp_ent, w.n_groups, x, (int64_t) l->n_embd, w.x); break;
            default: hipLaunchKernelGGL(window_head_kernel<MAYA_DT_F16>, grid, dim3(256), 0, s, logits, n_expert, k, n_tokens, expert_table, ids, weights, w.plan_ptr, w.grp_ptr, w.grp_start, w.grp_ent, w.n_groups, x, (int64_t) l->n_embd, w.x); break;
        }
        MAYA_LAUNCHED("window_head_kernel");
        grouped = true;
    } else if (logits && q8k_act(l->gate_type) && n_expert <= MAYA_MAX_EXPERTS && x_dtype >= 0 && x_dtype <= 2) {
        // one launch: route, plan, Q8_K of x
        const dim3 grid((unsigned) (1 + l->n_embd / 256), (unsigned) n_tokens);
        hipStream_t s = as_stream(stream);
        switch (x_dtype) {
            case MAYA_DT_F32: hipLaunchKernelGGL(layer_head_kernel<MAYA_DT_F32>, grid, dim3(256), 0, s, logits, n_expert, k, rs, expert_table, ids, weights, w.plan_ptr, x, (int64_t) l->n_embd, w.x); break;
            case MAYA_DT_BF16: hipLaunchKernelGGL(layer_head_kernel<MAYA_DT_BF16>, grid, dim3(256), 0, s, logits, n_expert, k, rs, expert_table, ids, weights, w.plan_ptr, x, (int64_t) l->n_embd, w.x); break;
            default: hipLaunchKernelGGL(layer_head_kernel<MAYA_DT_F16>, grid, dim3(256), 0, s, logits, n_expert, k, rs, expert_table, ids, weights, w.plan_ptr, x, (int64_t) l->n_embd, w.x); break;
        }
        MAYA_LAUNCHED("layer_head_kernel");
    } else {
        if (logits && n_expert <= MAYA_MAX_EXPERTS) {
            if ((rc = maya_moe_route_plan(router, logits, n_tokens, n_expert, k, expert_table, ids, weights, w.plan_ptr, stream))) return rc;
        } else {
            if (logits && (rc = route_impl("layer_decode", logits, n_tokens, n_expert, k, rs, ids, weights, stream))) return rc;   // (null: ids / weights are given)
            if ((rc = maya_moe_plan(ids, n_tokens * k, expert_table, n_expert, w.plan_ptr, stream))) return rc;
        }
        if ((rc = maya_quant_act(l->gate_type, x, x_dtype, 0, n_tokens, l->n_embd, w.x, stream))) return rc;
    }
    if (n_tokens > 1) {
        if (!grouped && (rc = maya_moe_group(w.plan_ptr, n_tokens * k, w.grp_ptr, w.grp_start, w.grp_ent, w.n_groups, stream))) return rc;
        if (gate_up_by_entries(a) && down_by_entries(a)) {
            // The entry-by-entry kernels take no groups, only the ORDER of the entries: those of one expert side by side,
            // so that they run at the same time on the same XCD (an entry's row block b always lands on XCD b % 8) and
            // the expert's rows come from DRAM once and from that XCD's L2 for the other tokens.
            a.grp_ent = w.grp_ent;
        } else {
            a.grp_ptr = w.grp_ptr;
            a.grp_start = w.grp_start;
            a.grp_ent = w.grp_ent;
            a.n_groups = w.n_groups;
        }
    }
    if (!gate_up_done && (rc = maya_moe_gate_up(&a, stream))) return rc;
    if (!tail) return MAYA_OK;
    if (down_rounds_h(a)) {
        a.hq = maya_act{nullptr, nullptr, nullptr};
        a.part = nullptr;
    } else {
        if ((rc = maya_quant_act(l->down_type, w.h, MAYA_DT_F32, 0, n_tokens * k, l->n_ff, w.hq, stream))) return rc;
    }
    if (join) {
        MAYA_HIP(hipStreamWaitEvent(as_stream(stream), join, 0));
        *joined = true;
    }
    return maya_moe_down(&a, stream);
}

extern "C" {

int maya_moe_layer_decode_routed(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k, const maya_router* router,
                                 const float* logits, const void* x, int x_dtype, int n_tokens, float limit, const float* add,
                                 int32_t* ids, float* weights, float* out, void* workspace, size_t workspace_bytes, void* stream) {
    return layer_decode_core(l, expert_table, n_expert, k, router, logits, x, x_dtype, n_tokens, limit, add, ids, weights, out, workspace,
                             workspace_bytes, stream, nullptr, nullptr);
}

int maya_moe_layer_decode_begin(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k, const maya_router* router,
                                const float* logits, const void* x, int x_dtype, int n_tokens, float limit, const float* add,
                                int32_t* ids, float* weights, float* out, void* workspace, size_t workspace_bytes, void* stream) {
    return layer_decode_core(l, expert_table, n_expert, k, router, logits, x, x_dtype, n_tokens, limit, add, ids, weights, out, workspace,
                             workspace_bytes, stream, nullptr, nullptr, kLayerBegin);
}
int maya_moe_layer_decode_end(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k, const maya_router* router,
                              const float* logits, const void* x, int x_dtype, int n_tokens, float limit, const float* add,
                              int32_t* ids, float* weights, float* out, void* workspace, size_t workspace_bytes, void* stream) {
    return layer_decode_core(l, expert_table, n_expert, k, router, logits, x, x_dtype, n_tokens, limit, add, ids, weights, out, workspace,
                             workspace_bytes, stream, nullptr, nullptr, kLayerEnd);
}

int maya_moe_layer_decode_shared(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k, const maya_router* router,
                                 const float* logits, const void* x, int x_dtype, int n_tokens, float limit, const maya_moe_args* shared,
                                 int32_t* ids, float* weights, float* out, void* workspace, size_t workspace_bytes, void* stream) {
    DeviceState* st;
    if (const int rc = current_state(&st)) return rc;
    if (!l || !shared || !x) return fail(MAYA_E_ARG, "layer_decode_shared: null pointer");
    if (const int rc = check_layout(shared->layout)) return rc;
    if (shared->k != 1 || shared->n_tokens != n_tokens || shared->layout.n_embd != l->n_embd)
        return fail(MAYA_E_SHAPE, "layer_decode_shared: the shared expert's arguments hold %d tokens x %d slots of %lld values, the layer %d tokens of %lld",
                    shared->n_tokens, shared->k, (long long) shared->layout.n_embd, n_tokens, (long long) l->n_embd);
    if (!shared->x.q || !shared->x.d || !shared->h || !shared->out || !shared->plan_ptr || !shared->plan_w)
        return fail(MAYA_E_ARG, "layer_decode_shared: the shared expert's arguments lack a buffer (x, h, out, plan)");
    if (shared->out == out) return fail(MAYA_E_ARG, "layer_decode_shared: the shared expert's out is the layer's out");
    // Everything the stage calls below could refuse is asked BEFORE the fork, so that a status > 0 means nothing was launched
    // on either stream.
    if (const int rc = quant_act_refusal(shared->layout.gate_type, x, x_dtype, n_tokens, shared->layout.n_embd, shared->x)) return rc;
    if (const int rc = gate_up_refusal(shared, *st)) return rc;
    if (shared->hq.q)
        if (const int rc = quant_act_refusal(shared->layout.down_type, shared->h, MAYA_DT_F32, n_tokens, shared->layout.n_ff, shared->hq)) return rc;
    if (const int rc = down_refusal(shared, *st)) return rc;
    {
        RouterSpec rs;
        LayerWs w;
        maya_moe_args a;
        if (const int rc = layer_setup(l, expert_table, n_expert, k, router, logits, x, x_dtype, n_tokens, limit, shared->out, ids, weights,
                                       out, workspace, workspace_bytes, *st, rs, w, a))
            return rc;
    }
    // one call at a time a device: the side stream and its two events are the device's
    std::lock_guard<std::mutex> lock(st->side_mu);
    hipStream_t s = as_stream(stream);
    {   // A side stream that an earlier call left inside a capture that has not ended belongs to that capture's graph until
        // hipStreamEndCapture: work forked onto it from another stream (eager, or another capture) would land in the wrong
        // graph or break the open capture.  The same capture calling again (a graph of several layers) is fine.
        hipStreamCaptureStatus side_st = hipStreamCaptureStatusNone, mine_st = hipStreamCaptureStatusNone;
        unsigned long long side_id = 0, mine_id = 0;
        MAYA_HIP(hipStreamGetCaptureInfo(st->side, &side_st, &side_id));
        MAYA_HIP(hipStreamGetCaptureInfo(s, &mine_st, &mine_id));
        if (side_st != hipStreamCaptureStatusNone && !(mine_st == hipStreamCaptureStatusActive && mine_id == side_id))
            return fail(MAYA_E_BUSY, "layer_decode_shared: the device's side stream is inside another stream's capture; end that capture first");
    }
    MAYA_HIP(hipEventRecord(st->side_fork, s));
    MAYA_HIP(hipStreamWaitEvent(st->side, st->side_fork, 0));
    // the shared expert beside the routed experts' head and gate/up launches: quantize x, gate/up, quantize h, down + add
    int rc = maya_quant_act(shared->layout.gate_type, x, x_dtype, 0, n_tokens, shared->layout.n_embd, shared->x, st->side);
    if (!rc) rc = maya_moe_gate_up(shared, st->side);
    if (!rc && shared->hq.q)   // (no hq: a down kernel that rounds h itself, as in maya_moe_down)
        rc = maya_quant_act(shared->layout.down_type, shared->h, MAYA_DT_F32, 0, n_tokens, shared->layout.n_ff, shared->hq, st->side);
    if (!rc) rc = maya_moe_down(shared, st->side);
    // (whatever happened, the side stream joins the caller's again: a capture must not end with it forked)
    bool joined = false;
    hipError_t e = hipEventRecord(st->side_join, st->side);
    if (e == hipSuccess && !rc)
        rc = layer_decode_core(l, expert_table, n_expert, k, router, logits, x, x_dtype, n_tokens, limit, shared->out, ids, weights, out,
                               workspace, workspace_bytes, stream, st->side_join, &joined);
    if (e == hipSuccess && !joined) e = hipStreamWaitEvent(s, st->side_join, 0);
    if (e != hipSuccess && !rc) rc = hip_fail(e, "layer_decode_shared: joining the shared expert's stream");
    return rc;
}

int maya_moe_layer_decode_static(const maya_moe_layout* l, const uint64_t* expert_table, int n_expert, int k, const maya_router* router,
                                 const float* logits, const void* x, int x_dtype, int n_tokens, float limit, const float* add,
                                 int32_t* ids, float* weights, float* out, void* stream) {
    // No lazy set-up here: the first use of a device uploads the codebooks (an allocation and a synchronous copy), which
    // this entry point must not do - maya_init() does, once, outside any capture.
    int dev = 0;
    MAYA_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices || !g_dev[dev].ready || !g_dev[dev].static_scratch)
        return fail(MAYA_E_ARG, "layer_decode_static: call maya_init() on device %d first (this entry point sets nothing up)", dev);
    const size_t need = maya_moe_workspace_bytes(l, n_tokens, k);
    if (need == 0) return fail(MAYA_E_SHAPE, "layer_decode_static: layout, n_tokens %d or k %d not covered", n_tokens, k);
    if (need > (size_t) MAYA_STATIC_SCRATCH_BYTES)
        return fail(MAYA_E_SHAPE, "layer_decode_static: this call needs %zu bytes of scratch, the static buffer holds %zu (use maya_moe_layer_decode_routed with a workspace)",
                    need, (size_t) MAYA_STATIC_SCRATCH_BYTES);
    return maya_moe_layer_decode_routed(l, expert_table, n_expert, k, router, logits, x, x_dtype, n_tokens, limit, add, ids, weights, out,
                                        g_dev[dev].static_scratch, (size_t) MAYA_STATIC_SCRATCH_BYTES, stream);
}

}  // extern "C"
