/* maya_oracle.c - TEST INFRASTRUCTURE (see maya_oracle.h): a CPU restatement of the reference's routed-MoE expert
 * arithmetic.  Build: gcc -O2 -ffp-contract=off -fopenmp (oracle/Makefile).  Not linked into the product library. */
#include "maya_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "iq_grids.h"

/* ------------------------------------------------------------------------------------------------ conversions */

/* include/strata/artifact/dequant.hpp:33-55 (fp16_to_fp32): exact, subnormals and infinities included */
float mo_f16_to_f32(uint16_t h) {
    const uint32_t s = (uint32_t) (h & 0x8000u) << 16, e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    uint32_t b;
    float f;
    if (e == 0) {
        f = (float) m * 5.9604644775390625e-8f; /* m * 2^-24, exact */
        memcpy(&b, &f, 4);
        b |= s;
    } else if (e == 31) {
        b = s | 0x7f800000u | (m << 13);
    } else {
        b = s | ((e + 112u) << 23) | (m << 13);
    }
    memcpy(&f, &b, 4);
    return f;
}

/* round-to-nearest-even F32 -> F16 (the rounding of _cvtss_sh and of src/kernels f16_bits.hpp's f16_from_f32) */
uint16_t mo_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) return (uint16_t) (sign | 0x7c00u | (ax > 0x7f800000u ? 0x200u | ((ax >> 13) & 0x3ffu) : 0u));
    if (ax >= 0x477ff000u) return (uint16_t) (sign | 0x7c00u); /* rounds to >= 65520: infinity */
    if (ax < 0x33000001u) return (uint16_t) sign;             /* <= 2^-25: rounds to zero (2^-25 itself ties to even 0) */
    int e = (int) (ax >> 23) - 127;
    uint32_t m = (ax & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int shift;                                 /* bits dropped */
    uint32_t base;
    if (e < -14) { /* subnormal half: value = m * 2^(e-23), unit 2^-24 */
        shift = -e - 1;                        /* 13 + (-14 - e) */
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t) (e + 15) << 10;
        m &= 0x7fffffu;
    }
    uint32_t q = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) ++q;
    return (uint16_t) (sign | (base + q)); /* a carry out of the mantissa bumps the exponent, as it must */
}

float mo_bf16_to_f32(uint16_t h) {
    const uint32_t b = (uint32_t) h << 16;
    float f;
    memcpy(&f, &b, 4);
    return f;
}

uint16_t mo_f32_to_bf16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t) ((x >> 16) | 0x40u);
    x += 0x7fffu + ((x >> 16) & 1u);
    return (uint16_t) (x >> 16);
}

/* ------------------------------------------------------------------------------------------------- codebooks */

static uint64_t g_iq2s[1024], g_iq1s[2048], g_iq2xxs[256];
static int g_grids_ready = 0;

static void grids_init(void) {
    if (g_grids_ready) return;
#pragma omp critical(mo_grids)
    {
        if (!g_grids_ready) {
            static const uint8_t m2[4] = {8, 25, 43, 0}, m1[4] = {0xff, 0x00, 0x01, 0};
            for (int i = 0; i < 1024; ++i) {
                uint64_t v = 0;
                for (int j = 0; j < 8; ++j) v |= (uint64_t) m2[(maya_iq2s_packed[i] >> (2 * j)) & 3] << (8 * j);
                g_iq2s[i] = v;
            }
            for (int i = 0; i < 2048; ++i) {
                uint64_t v = 0;
                for (int j = 0; j < 8; ++j) v |= (uint64_t) m1[(maya_iq1s_packed[i] >> (2 * j)) & 3] << (8 * j);
                g_iq1s[i] = v;
            }
            for (int i = 0; i < 256; ++i) {
                uint64_t v = 0;
                for (int j = 0; j < 8; ++j) v |= (uint64_t) m2[(maya_iq2xxs_packed[i] >> (2 * j)) & 3] << (8 * j);
                g_iq2xxs[i] = v;
            }
            g_grids_ready = 1;
        }
    }
}
const uint64_t* mo_iq2s_grid(void) {
    grids_init();
    return g_iq2s;
}
const uint64_t* mo_iq1s_grid(void) {
    grids_init();
    return g_iq1s;
}
const uint64_t* mo_iq2xxs_grid(void) {
    grids_init();
    return g_iq2xxs;
}
/* ksigns_iq2xs (third_party/ggml/ggml-common.h:513): seven sign bits and, in bit 7, their parity - an even number of
 * negative values in every group of 8 */
static inline uint8_t ksigns7(uint32_t i) { return (uint8_t) (i | ((uint32_t) (__builtin_popcount(i) & 1) << 7)); }

uint32_t mo_crc32(const void* p, size_t n) {
    const uint8_t* b = (const uint8_t*) p;
    uint32_t c = 0xffffffffu;
    for (size_t i = 0; i < n; ++i) {
        c ^= b[i];
        for (int k = 0; k < 8; ++k) c = (c >> 1) ^ (0xedb88320u & (0u - (c & 1u)));
    }
    return ~c;
}

/* -------------------------------------------------------------------------------------------------- geometry */

int mo_block_values(int type) { return type == MO_Q8_0 ? 32 : 256; }
int mo_block_bytes(int type) {
    switch (type) {
        case MO_Q8_0: return 34;
        case MO_Q4_K: return 144;
        case MO_IQ1_S: return 50;
        case MO_IQ2_S: return 82;
        case MO_IQ1_M: return 56;
        case MO_IQ2_XXS: return 66;
        default: return 0;
    }
}
size_t mo_row_bytes(int type, int64_t k) { return (size_t) (k / mo_block_values(type)) * (size_t) mo_block_bytes(type); }

static inline uint16_t rd16(const uint8_t* p) { return (uint16_t) (p[0] | (p[1] << 8)); }
static inline uint32_t rd32(const uint8_t* p) { return (uint32_t) rd16(p) | ((uint32_t) rd16(p + 2) << 16); }

/* Q4_K 6-bit scale / min of sub-block j (include/strata/artifact/dequant.hpp:152-160, get_scale_min_k4) */
static inline void q4k_scale_min(int j, const uint8_t* q, int* sc, int* m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (q[j + 4] & 0x0f) | ((q[j - 4] >> 6) << 4);
        *m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}

/* IQ1_M: the f16 super-scale scattered over the top nibbles of the four u16 scale words (iq_avx2.cpp:471-475) */
static inline uint16_t iq1m_dbits(const uint8_t* blk) {
    const uint16_t s0 = rd16(blk + 48), s1 = rd16(blk + 50), s2 = rd16(blk + 52), s3 = rd16(blk + 54);
    return (uint16_t) ((s0 >> 12) | ((s1 >> 8) & 0x00f0) | ((s2 >> 4) & 0x0f00) | (s3 & 0xf000));
}

/* ------------------------------------------------------------------------------------------------ dequantize */

/* include/strata/artifact/dequant.hpp:81-85 */
static void dq_q8_0(const uint8_t* blk, float* out) {
    const float d = mo_f16_to_f32(rd16(blk));
    for (int j = 0; j < 32; ++j) out[j] = (float) (int8_t) blk[2 + j] * d;
}
/* include/strata/artifact/dequant.hpp:162-190; canonical form: every operation rounded once (d*sc, dmin*m, d1*q, - m1) */
static void dq_q4_K(const uint8_t* blk, float* out) {
    const float d = mo_f16_to_f32(rd16(blk)), mn = mo_f16_to_f32(rd16(blk + 2));
    const uint8_t* scales = blk + 4;
    const uint8_t* q = blk + 16;
    int is = 0;
    for (int j = 0; j < 256; j += 64) {
        int sc, m;
        q4k_scale_min(is, scales, &sc, &m);
        const float d1 = d * (float) sc, m1 = mn * (float) m;
        q4k_scale_min(is + 1, scales, &sc, &m);
        const float d2 = d * (float) sc, m2 = mn * (float) m;
        for (int l = 0; l < 32; ++l) {
            const float p = d1 * (float) (q[l] & 0x0f);
            out[j + l] = p - m1;
        }
        for (int l = 0; l < 32; ++l) {
            const float p = d2 * (float) (q[l] >> 4);
            out[j + 32 + l] = p - m2;
        }
        q += 32;
        is += 2;
    }
}
/* src/kernels/cuda/iq_kernels.cu:686-695 (dq_iq2_s): d*(0.5f+ls)*0.25f, then * grid byte * sign */
static void dq_iq2_s(const uint8_t* blk, float* out) {
    const uint64_t* grid = mo_iq2s_grid();
    const float d = mo_f16_to_f32(rd16(blk));
    const uint8_t *qs = blk + 2, *signs = blk + 34, *qh = blk + 66, *scales = blk + 74;
    for (int ib = 0; ib < 8; ++ib) {
        for (int il = 0; il < 4; ++il) {
            const int idx = qs[4 * ib + il] | ((qh[ib] << (8 - 2 * il)) & 0x300);
            const uint64_t g = grid[idx];
            const uint8_t sg = signs[4 * ib + il];
            const int ls = (scales[ib] >> (4 * (il / 2))) & 0x0f;
            const float dl = d * (0.5f + (float) ls) * 0.25f;
            for (int j = 0; j < 8; ++j) {
                const float v = dl * (float) ((g >> (8 * j)) & 255u);
                out[32 * ib + 8 * il + j] = (sg >> j) & 1 ? -v : v;
            }
        }
    }
}
/* src/kernels/cuda/iq_kernels.cu:661-672 (dq_iq2_xxs); block third_party/ggml/ggml-common.h:380-384: d, then 8 bytes a
 * 32-value sub-block - four codebook indices, then four 7-bit sign indices and a 4-bit scale in one word */
static void dq_iq2_xxs(const uint8_t* blk, float* out) {
    const uint64_t* grid = mo_iq2xxs_grid();
    const float d = mo_f16_to_f32(rd16(blk));
    for (int ib = 0; ib < 8; ++ib) {
        const uint8_t* q = blk + 2 + 8 * ib;
        const uint32_t aux = rd32(q + 4);
        const float dl = d * (0.5f + (float) (aux >> 28)) * 0.25f;
        for (int il = 0; il < 4; ++il) {
            const uint64_t g = grid[q[il]];
            const uint8_t sg = ksigns7((aux >> (7 * il)) & 127u);
            for (int j = 0; j < 8; ++j) {
                const float v = dl * (float) ((g >> (8 * j)) & 255u);
                out[32 * ib + 8 * il + j] = (sg >> j) & 1 ? -v : v;
            }
        }
    }
}
/* src/kernels/cuda/iq_kernels.cu:825-837 (dq_iq1_s): d*(2s+1) * (grid + delta), delta = -+0.125 by qh bit 15 */
static void dq_iq1_s(const uint8_t* blk, float* out) {
    const uint64_t* grid = mo_iq1s_grid();
    const float d = mo_f16_to_f32(rd16(blk));
    const uint8_t* qs = blk + 2;
    for (int ib = 0; ib < 8; ++ib) {
        const uint16_t qh = rd16(blk + 34 + 2 * ib);
        const float dl = d * (float) (2 * ((qh >> 12) & 7) + 1);
        const float delta = (qh & 0x8000) ? -0.125f : 0.125f;
        for (int il = 0; il < 4; ++il) {
            const uint64_t g = grid[qs[4 * ib + il] | (((qh >> (3 * il)) & 7) << 8)];
            for (int j = 0; j < 8; ++j) out[32 * ib + 8 * il + j] = dl * ((float) (int8_t) ((g >> (8 * j)) & 255u) + delta);
        }
    }
}
/* src/kernels/cuda/iq_kernels.cu:839-855 (dq_iq1_m) */
static void dq_iq1_m(const uint8_t* blk, float* out) {
    const uint64_t* grid = mo_iq1s_grid();
    const float d = mo_f16_to_f32(iq1m_dbits(blk));
    const uint8_t *qs = blk, *qh = blk + 32;
    for (int ib = 0; ib < 8; ++ib) {
        for (int il = 0; il < 4; ++il) {
            const int nib = (qh[2 * ib + il / 2] >> (4 * (il % 2))) & 0x0f;
            const int ib16 = 2 * ib + il / 2;
            const int s = (rd16(blk + 48 + 2 * (ib16 / 4)) >> (3 * (ib16 % 4))) & 7;
            const float dl = d * (float) (2 * s + 1);
            const float delta = (nib & 8) ? -0.125f : 0.125f;
            const uint64_t g = grid[qs[4 * ib + il] | ((nib & 7) << 8)];
            for (int j = 0; j < 8; ++j) out[32 * ib + 8 * il + j] = dl * ((float) (int8_t) ((g >> (8 * j)) & 255u) + delta);
        }
    }
}

int mo_dequant_row(int type, const uint8_t* row, int64_t k, float* out) {
    const int bv = mo_block_values(type), bb = mo_block_bytes(type);
    if (bb == 0 || k % bv) return 1;
    for (int64_t b = 0; b < k / bv; ++b) {
        const uint8_t* blk = row + (size_t) b * bb;
        float* o = out + b * bv;
        switch (type) {
            case MO_Q8_0: dq_q8_0(blk, o); break;
            case MO_Q4_K: dq_q4_K(blk, o); break;
            case MO_IQ2_S: dq_iq2_s(blk, o); break;
            case MO_IQ1_S: dq_iq1_s(blk, o); break;
            case MO_IQ1_M: dq_iq1_m(blk, o); break;
            case MO_IQ2_XXS: dq_iq2_xxs(blk, o); break;
            default: return 1;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------- activation quantizers */

/* ggml's nearest_int (src/kernels/cuda/quantize_act.cu:172-177): the magic-number round, ties to even */
static inline int nearest_int(float fval) {
    const float val = fval + 12582912.0f;
    int i;
    memcpy(&i, &val, 4);
    return (i & 0x007fffff) - 0x00400000;
}

/* src/kernels/cuda/quantize_act.cu:179-207; host form src/ds4/ds4_lane_parity.cpp:610-637 */
void mo_quant_q8k(const float* x, int64_t k, mo_q8k* out) {
    for (int64_t b = 0; b < k / 256; ++b) {
        const float* xb = x + b * 256;
        mo_q8k* o = out + b;
        float max = 0.0f, amax = 0.0f;
        for (int j = 0; j < 256; ++j) {
            const float ax = fabsf(xb[j]);
            if (ax > amax) {
                amax = ax;
                max = xb[j];
            }
        }
        if (amax == 0.0f) {
            memset(o, 0, sizeof *o);
            continue;
        }
        const float iscale = -127.0f / max;
        for (int j = 0; j < 256; ++j) {
            const float p = iscale * xb[j]; /* rounded to F32 before the magic add (-ffp-contract=off) */
            const int v = nearest_int(p);
            o->qs[j] = (int8_t) (v < 127 ? v : 127);
        }
        for (int j = 0; j < 16; ++j) {
            int sum = 0;
            for (int i = 0; i < 16; ++i) sum += o->qs[16 * j + i];
            o->bsums[j] = (int16_t) sum;
        }
        o->d = 1.0f / iscale;
    }
}

/* The Q8_0 activation rounding of the CPU expert path on x86, ggml-cpu's quantize_row_q8_0 (arch/x86/quants.c) as the
 * reference restates it in quantize_oracle_q8_0 (src/kernels/cpu/expert.cpp:92-130, "the pinned ggml CPU Q8_0 contract":
 * FP16-rounded scales and x86 nearest-even codes, include/strata/kernels/cpu/expert.hpp:55-57):
 *   d = amax / 127 (65504 when that is larger: the FP16 scale stays finite), stored as FP16 (nearest even);
 *   q = nearest-even(x * (127 / amax)), the product rounded to F32 first; an all-zero block is all zeros.
 * Two other statements of this quantizer exist and differ from it on values next to a rounding boundary: ggml's scalar
 * quantize_row_q8_0_ref (roundf(x * (1 / d)): halves away from zero) and the reference's GPU quantize_q8_0
 * (src/kernels/cuda/quantize_act.cu:47-78: rint of the double quotient x / d); tests/test_oracle_pins.py counts how often. */
void mo_quant_q80(const float* x, int64_t k, mo_q80* out) {
    for (int64_t b = 0; b < k / 32; ++b) {
        const float* xb = x + b * 32;
        float amax = 0.0f;
        for (int j = 0; j < 32; ++j) {
            const float ax = fabsf(xb[j]);
            if (ax > amax) amax = ax;
        }
        const int big = amax / 127.0f > 65504.0f;
        const float d = big ? 65504.0f : amax / 127.0f;
        const float inv = amax == 0.0f ? 0.0f : big ? 1.0f / 65504.0f : 127.0f / amax;
        out[b].d = mo_f32_to_f16(d);
        for (int j = 0; j < 32; ++j) {
            float r = nearbyintf(xb[j] * inv); /* the default rounding mode: to nearest, ties to even */
            r = r > 127.0f ? 127.0f : r < -128.0f ? -128.0f : r;
            out[b].qs[j] = (int8_t) r;
        }
    }
}

/* src/prefill/moe_fused_rdna4.cu:87-109: c = rint(x * (127 / amax)), d = amax / 127 */
void mo_quant_i8x32(const float* x, int64_t k, int8_t* q, float* d) {
    for (int64_t b = 0; b < k / 32; ++b) {
        const float* xb = x + b * 32;
        float amax = 0.0f;
        for (int j = 0; j < 32; ++j) {
            const float ax = fabsf(xb[j]);
            if (ax > amax) amax = ax;
        }
        const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
        for (int j = 0; j < 32; ++j) q[b * 32 + j] = (int8_t) nearest_int(xb[j] * inv);
        d[b] = amax / 127.0f;
    }
}

size_t mo_act_bytes(int type, int64_t k) {
    return type == MO_Q8_0 ? (size_t) (k / 32) * sizeof(mo_q80) : (size_t) (k / 256) * sizeof(mo_q8k);
}
void mo_quant_act(int type, const float* x, int64_t k, void* out) {
    if (type == MO_Q8_0) mo_quant_q80(x, k, (mo_q80*) out);
    else mo_quant_q8k(x, k, (mo_q8k*) out);
}

/* ---------------------------------------------------------------------------------------------- the row dots */

/* ggml's hsum_float_8 (src/kernels/cpu/iq_avx2.cpp:111-117): (hi128 + lo128), + movehl, + movehdup */
static inline float hsum8(const float* x) {
    const float r0 = x[4] + x[0], r1 = x[5] + x[1], r2 = x[6] + x[2], r3 = x[7] + x[3];
    const float a = r0 + r2, b = r1 + r3;
    return a + b;
}

/* IQ2_S x Q8_K (iq_avx2.cpp:160-176 Fmt32<22>::decode, 225-250 row_dot): int32 lane n of a 32-value chunk holds values
 * 4n..4n+3 times the chunk's half scale; one fmadd a block with d_w * d_x; K = 0.125 after hsum */
static float dot_iq2_s(const uint8_t* row, int nb, const mo_q8k* y) {
    const uint64_t* grid = mo_iq2s_grid();
    float accf[8] = {0};
    for (int i = 0; i < nb; ++i) {
        const uint8_t* blk = row + (size_t) i * 82;
        int32_t acci[8] = {0};
        for (int c = 0; c < 8; ++c) { /* chunk c = 2j + half: values 32c .. 32c+31 */
            const uint8_t h = blk[66 + c], sb = blk[74 + c];
            const int sca = 2 * (sb & 15) + 1, scb = 2 * (sb >> 4) + 1;
            for (int l = 0; l < 4; ++l) {
                const uint64_t g = grid[blk[2 + 4 * c + l] | ((h << (8 - 2 * l)) & 0x300)];
                const uint8_t sg = blk[34 + 4 * c + l];
                const int8_t* q8 = y[i].qs + 32 * c + 8 * l;
                for (int hf = 0; hf < 2; ++hf) { /* lane n = 2l + hf */
                    int s = 0;
                    for (int j = 4 * hf; j < 4 * hf + 4; ++j) {
                        const int m = (int) ((g >> (8 * j)) & 255u);
                        s += m * ((sg >> j) & 1 ? -(int) q8[j] : (int) q8[j]);
                    }
                    acci[2 * l + hf] += s * (l < 2 ? sca : scb);
                }
            }
        }
        const float dd = mo_f16_to_f32(rd16(blk)) * y[i].d;
        for (int n = 0; n < 8; ++n) accf[n] = fmaf(dd, (float) acci[n], accf[n]);
    }
    return 0.125f * hsum8(accf);
}

/* IQ2_XXS x Q8_K (iq_avx2.cpp:130-141 Fmt32<16>::decode, 225-250 row_dot): as IQ2_S with one scale a 32-value chunk */
static float dot_iq2_xxs(const uint8_t* row, int nb, const mo_q8k* y) {
    const uint64_t* grid = mo_iq2xxs_grid();
    float accf[8] = {0};
    for (int i = 0; i < nb; ++i) {
        const uint8_t* blk = row + (size_t) i * 66;
        int32_t acci[8] = {0};
        for (int c = 0; c < 8; ++c) {
            const uint8_t* q = blk + 2 + 8 * c;
            const uint32_t aux = rd32(q + 4);
            const int sc = 2 * (int) (aux >> 28) + 1;
            for (int l = 0; l < 4; ++l) {
                const uint64_t g = grid[q[l]];
                const uint8_t sg = ksigns7((aux >> (7 * l)) & 127u);
                const int8_t* q8 = y[i].qs + 32 * c + 8 * l;
                for (int hf = 0; hf < 2; ++hf) { /* lane n = 2l + hf */
                    int s = 0;
                    for (int j = 4 * hf; j < 4 * hf + 4; ++j) {
                        const int m = (int) ((g >> (8 * j)) & 255u);
                        s += m * ((sg >> j) & 1 ? -(int) q8[j] : (int) q8[j]);
                    }
                    acci[2 * l + hf] += s * sc;
                }
            }
        }
        const float dd = mo_f16_to_f32(rd16(blk)) * y[i].d;
        for (int n = 0; n < 8; ++n) accf[n] = fmaf(dd, (float) acci[n], accf[n]);
    }
    return 0.125f * hsum8(accf);
}

/* Q4_K x Q8_K (iq_avx2.cpp:319-394 k_scales + row_dot_k<12>) */
static float dot_q4_K(const uint8_t* row, int nb, const mo_q8k* y) {
    float accf[8] = {0}, accm[4] = {0};
    for (int i = 0; i < nb; ++i) {
        const uint8_t* blk = row + (size_t) i * 144;
        int sc[8], mn[8];
        for (int j = 0; j < 8; ++j) q4k_scale_min(j, blk + 4, &sc[j], &mn[j]);
        int32_t acci[8] = {0};
        for (int j = 0; j < 4; ++j) {
            const uint8_t* q = blk + 16 + 32 * j;
            const int8_t *yl = y[i].qs + 64 * j, *yh = yl + 32;
            for (int n = 0; n < 8; ++n) {
                int lo = 0, hi = 0;
                for (int v = 4 * n; v < 4 * n + 4; ++v) {
                    lo += (q[v] & 0x0f) * yl[v];
                    hi += (q[v] >> 4) * yh[v];
                }
                acci[n] += lo * sc[2 * j] + hi * sc[2 * j + 1];
            }
        }
        const float dx = mo_f16_to_f32(rd16(blk)), mx = mo_f16_to_f32(rd16(blk + 2));
        const float d = y[i].d * dx, dmin = -y[i].d * mx;
        for (int n = 0; n < 8; ++n) accf[n] = fmaf(d, (float) acci[n], accf[n]);
        for (int n = 0; n < 4; ++n) { /* madd(mins, hadd(bsums)): lane n = sub-blocks 2n, 2n+1 */
            const int p = mn[2 * n] * (y[i].bsums[4 * n] + y[i].bsums[4 * n + 1]) +
                          mn[2 * n + 1] * (y[i].bsums[4 * n + 2] + y[i].bsums[4 * n + 3]);
            accm[n] = fmaf(dmin, (float) p, accm[n]);
        }
    }
    const float a0 = accm[0] + accm[2], a1 = accm[1] + accm[3];
    const float am = a0 + a1;
    return hsum8(accf) + am;
}

/* IQ1_M x Q8_K (iq_avx2.cpp:462-514 row_dot_iq1m): two float accumulators (values, deltas), int32 lane n = values
 * 4n..4n+3 of both 32-value chunks of each 64-value step, summed over the block; result = fma(1/8, hsum(delta), hsum(acc)) */
static float dot_iq1_m(const uint8_t* row, int nb, const mo_q8k* y) {
    const uint64_t* grid = mo_iq1s_grid();
    float accf[8] = {0}, deltaf[8] = {0};
    for (int i = 0; i < nb; ++i) {
        const uint8_t* blk = row + (size_t) i * 56;
        const float dx = mo_f16_to_f32(iq1m_dbits(blk));
        int32_t acc[8] = {0}, del[8] = {0};
        for (int j = 0; j < 4; ++j) {
            const uint8_t *qs = blk + 8 * j, *qh = blk + 32 + 4 * j;
            const unsigned sc = rd16(blk + 48 + 2 * j);
            for (int c = 0; c < 2; ++c) { /* chunk c of the step: values 64j + 32c .. */
                const int8_t* a = y[i].qs + 64 * j + 32 * c;
                for (int il = 0; il < 4; ++il) {
                    const int nib = (qh[2 * c + il / 2] >> (4 * (il % 2))) & 0x0f;
                    const uint64_t g = grid[qs[4 * c + il] | ((nib & 7) << 8)];
                    const int s = 2 * (int) ((sc >> (6 * c + 3 * (il / 2))) & 7) + 1;
                    const int dsg = (nib & 8) ? -1 : 1;
                    for (int hf = 0; hf < 2; ++hf) {
                        int sv = 0, sd = 0;
                        for (int v = 4 * hf; v < 4 * hf + 4; ++v) {
                            sv += (int) (int8_t) ((g >> (8 * v)) & 255u) * a[8 * il + v];
                            sd += dsg * a[8 * il + v];
                        }
                        acc[2 * il + hf] += s * sv;
                        del[2 * il + hf] += s * sd;
                    }
                }
            }
        }
        const float d = dx * y[i].d;
        for (int n = 0; n < 8; ++n) {
            accf[n] = fmaf(d, (float) acc[n], accf[n]);
            deltaf[n] = fmaf(d, (float) del[n], deltaf[n]);
        }
    }
    return fmaf(0.125f, hsum8(deltaf), hsum8(accf));
}

/* IQ1_S x Q8_K: ggml's generic form (no ggml-free twin in the reference tree; pinned through the IQ1_M carrier, see the header);
 * per block sumf += d * y.d * (sumi + IQ1S_DELTA * sumi1), following the decode of iq_kernels.cu:825-837 */
static float dot_iq1_s(const uint8_t* row, int nb, const mo_q8k* y) {
    const uint64_t* grid = mo_iq1s_grid();
    float sumf = 0.0f;
    for (int i = 0; i < nb; ++i) {
        const uint8_t* blk = row + (size_t) i * 50;
        int sumi = 0, sumi1 = 0;
        for (int ib = 0; ib < 8; ++ib) {
            const uint16_t qh = rd16(blk + 34 + 2 * ib);
            const int ls = 2 * ((qh >> 12) & 7) + 1, delta = (qh & 0x8000) ? -1 : 1;
            int lsum = 0;
            for (int l = 0; l < 4; ++l) {
                const uint64_t g = grid[blk[2 + 4 * ib + l] | (((qh >> (3 * l)) & 7) << 8)];
                for (int j = 0; j < 8; ++j) lsum += (int) (int8_t) ((g >> (8 * j)) & 255u) * y[i].qs[32 * ib + 8 * l + j];
            }
            sumi += ls * lsum;
            sumi1 += ls * delta * (y[i].bsums[2 * ib] + y[i].bsums[2 * ib + 1]);
        }
        sumf += mo_f16_to_f32(rd16(blk)) * y[i].d * ((float) sumi + 0.125f * (float) sumi1);
    }
    return sumf;
}

/* Q8_0 x Q8_0: ggml's generic form: sumf += sumi * (d_w * d_y) per 32 (pinned by an independent float64 product) */
static float dot_q8_0(const uint8_t* row, int nb, const mo_q80* y) {
    float sumf = 0.0f;
    for (int i = 0; i < nb; ++i) {
        const uint8_t* blk = row + (size_t) i * 34;
        int sumi = 0;
        for (int j = 0; j < 32; ++j) sumi += (int) (int8_t) blk[2 + j] * y[i].qs[j];
        sumf += (float) sumi * (mo_f16_to_f32(rd16(blk)) * mo_f16_to_f32(y[i].d));
    }
    return sumf;
}

float mo_vec_dot(int type, const uint8_t* row, int64_t k, const void* act) {
    switch (type) {
        case MO_Q8_0: return dot_q8_0(row, (int) (k / 32), (const mo_q80*) act);
        case MO_Q4_K: return dot_q4_K(row, (int) (k / 256), (const mo_q8k*) act);
        case MO_IQ2_S: return dot_iq2_s(row, (int) (k / 256), (const mo_q8k*) act);
        case MO_IQ1_S: return dot_iq1_s(row, (int) (k / 256), (const mo_q8k*) act);
        case MO_IQ1_M: return dot_iq1_m(row, (int) (k / 256), (const mo_q8k*) act);
        case MO_IQ2_XXS: return dot_iq2_xxs(row, (int) (k / 256), (const mo_q8k*) act);
        default: return NAN;
    }
}

void mo_rows(int type, const uint8_t* w, size_t row_bytes, int64_t k, const void* const* act, int nt, float* const* out,
             int r0, int r1) {
    for (int r = r0; r < r1; ++r)
        for (int t = 0; t < nt; ++t) out[t][r] = mo_vec_dot(type, w + (size_t) r * row_bytes, k, act[t]);
}

/* src/kernels/cpu/native_expert.cpp:364-371: clamp only under a finite limit, (g / (1 + exp(-g))) * u in F32 */
float mo_swiglu(float g, float u, float limit) {
    if (limit != INFINITY) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
    }
    return (g / (1.0f + expf(-g))) * u;
}

void mo_gu_rows(int type, const uint8_t* gate, const uint8_t* up, size_t row_bytes, int64_t k, const void* const* act,
                int nt, float* const* ff, int r0, int r1, float limit) {
    for (int r = r0; r < r1; ++r)
        for (int t = 0; t < nt; ++t) {
            const float g = mo_vec_dot(type, gate + (size_t) r * row_bytes, k, act[t]);
            const float u = mo_vec_dot(type, up + (size_t) r * row_bytes, k, act[t]);
            ff[t][r] = mo_swiglu(g, u, limit);
        }
}

/* native_quant_act -> native_gu_rows_split -> native_quant_h -> native_down_rows_split
 * (src/kernels/cpu/native_expert.cpp:262-268, 343-417); rows split over threads as ExpertPool::run_split_multi_native
 * (include/strata/kernels/cpu/pool.hpp:120-131): gate/up rows, barrier, quantize h, down rows */
void mo_expert(int gu_type, int d_type, const uint8_t* gate, const uint8_t* up, const uint8_t* down, int64_t n_embd,
               int64_t n_ff, const float* x, int nt, float limit, float* out, int nthreads) {
    const size_t ab = mo_act_bytes(gu_type, n_embd), hb = mo_act_bytes(d_type, n_ff);
    const size_t gr = mo_row_bytes(gu_type, n_embd), dr = mo_row_bytes(d_type, n_ff);
    uint8_t* act = (uint8_t*) malloc(ab * (size_t) nt);
    uint8_t* hq = (uint8_t*) malloc(hb * (size_t) nt);
    float* h = (float*) malloc(sizeof(float) * (size_t) n_ff * (size_t) nt);
    const void* actp[64];
    const void* hqp[64];
    float* hp[64];
    float* op[64];
    for (int t = 0; t < nt; ++t) {
        mo_quant_act(gu_type, x + (size_t) t * n_embd, n_embd, act + ab * t);
        actp[t] = act + ab * t;
        hqp[t] = hq + hb * t;
        hp[t] = h + (size_t) t * n_ff;
        op[t] = out + (size_t) t * n_embd;
    }
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int c = 0; c < (int) (n_ff / 32); ++c)
        mo_gu_rows(gu_type, gate, up, gr, n_embd, actp, nt, hp, 32 * c, 32 * c + 32, limit);
    for (int t = 0; t < nt; ++t) mo_quant_act(d_type, hp[t], n_ff, hq + hb * t);
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int c = 0; c < (int) (n_embd / 32); ++c) mo_rows(d_type, down, dr, n_ff, hqp, nt, op, 32 * c, 32 * c + 32);
    free(act);
    free(hq);
    free(h);
}

/* --------------------------------------------------------------------------------------------------- router */

/* src/kernels/cuda/router_top10.cu:95-186: softmax over all experts in double, p as float, k rounds of arg-max with a
 * strict > (lowest index on a tie), renormalise by max(sum, 2^-14) in double */
static void router_impl(const float* logits, int n_tokens, int n_expert, int k, int32_t* ids, float* weights, int f64) {
    double* ex = (double*) malloc(sizeof(double) * (size_t) n_expert);
    double* pd = (double*) malloc(sizeof(double) * (size_t) n_expert);
    float* p = (float*) malloc(sizeof(float) * (size_t) n_expert);
    uint8_t* taken = (uint8_t*) malloc((size_t) n_expert);
    for (int t = 0; t < n_tokens; ++t) {
        const float* l = logits + (size_t) t * n_expert;
        float mx = -INFINITY;
        for (int e = 0; e < n_expert; ++e) mx = fmaxf(mx, l[e]);
        double sum = 0.0;
        for (int e = 0; e < n_expert; ++e) {
            ex[e] = exp((double) l[e] - (double) mx);
            sum += ex[e];
        }
        const float inv = (float) (1.0 / sum);
        for (int e = 0; e < n_expert; ++e) {
            pd[e] = f64 ? ex[e] / sum : 0.0; /* the parity test's host form selects on the double p */
            p[e] = f64 ? (float) pd[e] : (float) (ex[e] * inv);
            taken[e] = 0;
        }
        for (int i = 0; i < k; ++i) {
            int bi = -1;
            for (int e = 0; e < n_expert; ++e) {
                if (taken[e]) continue;
                if (bi < 0 || (f64 ? pd[e] > pd[bi] : p[e] > p[bi])) bi = e;
            }
            if (bi < 0) bi = 0;
            taken[bi] = 1;
            ids[(size_t) t * k + i] = bi;
            weights[(size_t) t * k + i] = p[bi];
        }
        double s = 0.0;
        for (int i = 0; i < k; ++i) s += (double) weights[(size_t) t * k + i];
        const double sc = fmax(s, 6.103515625e-05);
        for (int i = 0; i < k; ++i) weights[(size_t) t * k + i] = (float) ((double) weights[(size_t) t * k + i] / sc);
    }
    free(ex);
    free(pd);
    free(p);
    free(taken);
}
void mo_router_topk(const float* logits, int n_tokens, int n_expert, int k, int32_t* ids, float* weights) {
    router_impl(logits, n_tokens, n_expert, k, ids, weights, 0);
}
void mo_router_topk_f64(const float* logits, int n_tokens, int n_expert, int k, int32_t* ids, float* weights) {
    router_impl(logits, n_tokens, n_expert, k, ids, weights, 1);
}

/* The sigmoid router of the GLM / DeepSeek-V3 family (noaux_tc): p = sigmoid(logit), the bias enters the SELECTION only,
 * stable top-k (ties to the lower index), w = p / max(sum, 2^-14) * w_scale (norm 1; norm 2: / (sum + 1e-20); norm 0: no
 * division).  f64 = 0: the device arithmetic of src/kernels/cuda/router_sigmoid.cu:44-73 and moe_route_kernel
 * (src/kernels/cuda/glm_fast.cu:4050-4056, 4214, 4297): p and p + bias in float, rank = the experts that beat e (a larger
 * score, or an equal one at a lower index), the selected p summed in rank order in double, inv a float,
 * w = (float)((double) p * inv * w_scale).  f64 = 1: the host form of src/kernels/router_sigmoid_parity.cpp:36-86
 * (double sigmoid and scores, stable sort). */
static void router_sigmoid_impl(const float* logits, const float* bias, int n_tokens, int n_expert, int k, float w_scale, int norm,
                                int32_t* ids, float* weights, int f64) {
    double* pd = (double*) malloc(sizeof(double) * (size_t) n_expert);
    double* sd = (double*) malloc(sizeof(double) * (size_t) n_expert);
    float* p = (float*) malloc(sizeof(float) * (size_t) n_expert);
    float* sel = (float*) malloc(sizeof(float) * (size_t) n_expert);
    for (int t = 0; t < n_tokens; ++t) {
        const float* l = logits + (size_t) t * n_expert;
        for (int e = 0; e < n_expert; ++e) {
            p[e] = 1.0f / (1.0f + expf(-l[e]));
            sel[e] = bias ? p[e] + bias[e] : p[e];
            pd[e] = 1.0 / (1.0 + exp(-(double) l[e]));
            sd[e] = bias ? pd[e] + (double) bias[e] : pd[e];
        }
        /* a row with a non-finite logit or selection score is refused: no routes (ids -1, weights 0), as the engine's
         * routers do (route_kernel src/kernels/cuda/glm_batch.cu:2077-2092; moe_route_kernel glm_fast.cu:4040) */
        int bad = 0;
        for (int e = 0; e < n_expert; ++e) bad |= !isfinite(l[e]) || !isfinite(sel[e]);
        if (bad) {
            for (int i = 0; i < k; ++i) {
                ids[(size_t) t * k + i] = -1;
                weights[(size_t) t * k + i] = 0.0f;
            }
            continue;
        }
        for (int e = 0; e < n_expert; ++e) {
            int rank = 0;
            for (int f = 0; f < n_expert; ++f) {
                if (f64) rank += (sd[f] > sd[e]) || (f < e && sd[f] == sd[e]);
                else rank += (sel[f] > sel[e]) || (f < e && sel[f] == sel[e]);
            }
            if (rank < k) ids[(size_t) t * k + rank] = e;
        }
        double sum = 0.0;
        for (int i = 0; i < k; ++i) sum += f64 ? pd[ids[(size_t) t * k + i]] : (double) p[ids[(size_t) t * k + i]];
        const double invd = norm == 0 ? 1.0 : norm == 2 ? 1.0 / (sum + 1e-20) : 1.0 / fmax(sum, 6.103515625e-05);
        const float inv = (float) invd;
        for (int i = 0; i < k; ++i) {
            const int e = ids[(size_t) t * k + i];
            weights[(size_t) t * k + i] = f64 ? (float) (pd[e] * invd * (double) w_scale) : (float) ((double) p[e] * inv * w_scale);
        }
    }
    free(pd);
    free(sd);
    free(p);
    free(sel);
}
void mo_router_sigmoid(const float* logits, const float* bias, int n_tokens, int n_expert, int k, float w_scale, int norm,
                       int32_t* ids, float* weights) {
    router_sigmoid_impl(logits, bias, n_tokens, n_expert, k, w_scale, norm, ids, weights, 0);
}
void mo_router_sigmoid_f64(const float* logits, const float* bias, int n_tokens, int n_expert, int k, float w_scale, int norm,
                           int32_t* ids, float* weights) {
    router_sigmoid_impl(logits, bias, n_tokens, n_expert, k, w_scale, norm, ids, weights, 1);
}

/* The residency plan of moe_route_kernel (src/kernels/cuda/glm_fast.cu:4262-4375; the tables: include/strata/kernels/
 * glm_fast.hpp:284-296) over already routed ids, the device-side tiers only: a hit in tab; else a second-tier source in
 * rtab = tab + n_keys: the layer's next free spare (it becomes resident: tab[key] written, the spare cleared) when
 * promote_min <= 1 or the key's count reaches it, else the next unused scratch slot, else left out (the "full" mask); in
 * neither table: a null entry and the miss mask.  counts ([n_keys] or NULL): ++ per routed key, all halved before a
 * route when (seq + 1) % 4096 == 0 (glm_fast.cu:4032-4034, 4175); seq ([1] or NULL) counts the routes.  Tokens in order;
 * masks[4 t + 0..3] = miss, fetch, promoted, full.  A refused row (ids -1) plans nothing. */
void mo_plan_tiered(const int32_t* ids, int n_tokens, int layer, int n_expert, int k, uint64_t* tab, int n_keys,
                    const uint64_t* scratch, int n_scratch, uint32_t* counts, uint32_t* seq, int promote_min,
                    uint64_t* plan, uint64_t* fetch_src, uint32_t* masks) {
    uint64_t* rtab = tab + n_keys;
    uint64_t* spares = tab + 2 * (size_t) n_keys + (size_t) layer * 3;
    int next_spare = 0, next_scratch = 0;
    for (int t = 0; t < n_tokens; ++t) {
        if (counts && seq && ((*seq + 1u) & 4095u) == 0u)
            for (int i = 0; i < n_keys; ++i) counts[i] >>= 1;
        uint32_t cnt[64];
        for (int i = 0; i < k; ++i) {
            const int id = ids[(size_t) t * k + i];
            cnt[i] = (id >= 0 && counts) ? ++counts[(size_t) layer * n_expert + id] : 0u;
        }
        uint32_t miss = 0, fetch = 0, promo = 0, full = 0;
        for (int i = 0; i < k; ++i) {
            const int id = ids[(size_t) t * k + i];
            uint64_t ptr = 0, src = 0;
            if (id >= 0) {
                const size_t key = (size_t) layer * n_expert + id;
                ptr = tab[key];
                if (ptr == 0) {
                    src = rtab[key];
                    if (src == 0) {
                        miss |= 1u << i;
                    } else {
                        while (next_spare < 3 && spares[next_spare] == 0) ++next_spare;
                        if (next_spare < 3 && (promote_min <= 1 || cnt[i] >= (uint32_t) promote_min)) {
                            ptr = spares[next_spare];
                            spares[next_spare] = 0;
                            tab[key] = ptr;
                            promo |= 1u << i;
                        } else if (next_scratch < n_scratch) {
                            ptr = scratch[next_scratch++];
                        } else {
                            full |= 1u << i;
                            src = 0;
                        }
                        if (src != 0) fetch |= 1u << i;
                    }
                }
            }
            plan[(size_t) t * k + i] = ptr;
            fetch_src[(size_t) t * k + i] = src;
        }
        masks[4 * t + 0] = miss;
        masks[4 * t + 1] = fetch;
        masks[4 * t + 2] = promo;
        masks[4 * t + 3] = full;
        if (seq) *seq += 1u;
    }
}

/* src/kernels/cuda/native_moe.cu:36-52: sum = parts[0]*w[0]; sum += parts[i]*w[i] ... (each product and add rounded) */
void mo_combine(const float* parts, const float* w, int k, int64_t n, float* out) {
    for (int64_t c = 0; c < n; ++c) {
        float sum = parts[c] * w[0];
        for (int i = 1; i < k; ++i) {
            const float p = parts[(size_t) i * n + c] * w[i];
            sum = sum + p;
        }
        out[c] = sum;
    }
}

void mo_moe_layer(int gu_type, int d_type, const uint8_t* const* blobs, int n_expert, int k, int64_t n_embd,
                  int64_t n_ff, const float* logits, const float* x, int n_tokens, float limit, int32_t* ids,
                  float* weights, float* out, int nthreads) {
    const size_t gr = mo_row_bytes(gu_type, n_embd), dr = mo_row_bytes(d_type, n_ff);
    const size_t up_off = gr * (size_t) n_ff, down_off = 2 * up_off;
    (void) dr;
    mo_router_topk(logits, n_tokens, n_expert, k, ids, weights);
    float* parts = (float*) malloc(sizeof(float) * (size_t) k * (size_t) n_embd);
    for (int t = 0; t < n_tokens; ++t) {
        for (int i = 0; i < k; ++i) {
            const uint8_t* b = blobs[ids[(size_t) t * k + i]];
            mo_expert(gu_type, d_type, b, b + up_off, b + down_off, n_embd, n_ff, x + (size_t) t * n_embd, 1, limit,
                      parts + (size_t) i * n_embd, nthreads);
        }
        mo_combine(parts, weights + (size_t) t * k, k, n_embd, out + (size_t) t * n_embd);
    }
    free(parts);
}

/* ------------------------------------------------------------------------------------ device-arithmetic lane */

/* src/ds4/ds4_par_exp.h:60-85 */
float mo_exp_portable(float y) {
    if (!(y < 89.0f)) return y != y ? y : INFINITY;
    if (y < -87.0f) return 0.0f;
    const float t = fmaf(y, 1.44269504088896341f, 12582912.0f);
    const float n = t - 12582912.0f;
    float r = fmaf(n, -0.693359375f, y);
    r = fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    const float r2 = r * r;
    p = fmaf(p, r2, r);
    p = p + 1.0f;
    const int ni = (int) n;
    uint32_t b;
    float s;
    if (ni > 127) {
        b = (uint32_t) (127 + 127) << 23;
        memcpy(&s, &b, 4);
        return (p * s) * 2.0f;
    }
    b = (uint32_t) (ni + 127) << 23;
    memcpy(&s, &b, 4);
    return p * s;
}
/* src/ds4/ds4_par_exp.h:76-83 */
float mo_swiglu_portable(float g, float u, float limit) {
    if (limit > 0.0f) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
    }
    return (g / (1.0f + mo_exp_portable(-g))) * u;
}

/* src/ds4/ds4_lane_parity.cpp:180-245 (decode, sub_dot, rows_scalar, lanes_tree) for IQ2_S: sub-block kb goes to lane
 * kb mod lpr, acc = fma(dx, d * (s0 lo + s1 hi), acc) with d = f16 * 0.125, lanes folded l += l + o for o = lpr/2 .. 1 */
float mo_row_lanes(int type, const uint8_t* row, int64_t k, const int8_t* q, const float* d32, int lpr) {
    if (type != MO_IQ2_S) return NAN;
    const uint64_t* grid = mo_iq2s_grid();
    float acc[32] = {0};
    for (int kb = 0; kb < (int) (k / 32); ++kb) {
        const uint8_t* b = row + (size_t) (kb >> 3) * 82;
        const int ib = kb & 7;
        const uint32_t i4 = rd32(b + 2 + 4 * ib), sg4 = rd32(b + 34 + 4 * ib), h = b[66 + ib], sc = b[74 + ib];
        int lo = 0, hi = 0;
        for (int l = 0; l < 4; ++l) {
            const uint64_t g = grid[((i4 >> (8 * l)) & 255u) | ((h << (8 - 2 * l)) & 0x300u)];
            const uint32_t sg = (sg4 >> (8 * l)) & 255u;
            int s = 0;
            for (int j = 0; j < 8; ++j) {
                const int m = (int) ((g >> (8 * j)) & 255u);
                s += ((sg >> j) & 1u ? -m : m) * (int) q[32 * kb + 8 * l + j];
            }
            if (l < 2) lo += s;
            else hi += s;
        }
        const int s0 = 2 * (int) (sc & 15) + 1, s1 = 2 * (int) (sc >> 4) + 1;
        const float d = mo_f16_to_f32(rd16(b)) * 0.125f;
        const float v = d * (float) (s0 * lo + s1 * hi);
        const int lane = kb & (lpr - 1);
        acc[lane] = fmaf(d32[kb], v, acc[lane]);
    }
    for (int o = lpr / 2; o > 0; o >>= 1)
        for (int l = 0; l < o; ++l) acc[l] = acc[l] + acc[l + o];
    return acc[0];
}

/* ----------------------------------------------------------------------------------------------------- EXL3 */

/* src/kernels/cpu/exl3_ref.cpp:11-27 */
float mo_exl3_decode(uint32_t state, int cb) {
    if (cb == 2) {
        const uint32_t x = state * 0x83DCD12Du;
        const float h = (float) (1024u + (x & 0xffu) + ((x >> 8) & 0xffu) + ((x >> 16) & 0xffu) + (x >> 24));
        return mo_f16_to_f32(mo_f32_to_f16(fmaf(h, mo_f16_to_f32(0x1eee), mo_f16_to_f32(0xc931))));
    }
    uint32_t x = cb == 1 ? state * 0xCBAC1FEDu : state * 89226354u + 64248484u;
    x = (x & 0x8fff8fffu) ^ 0x3b603b60u;
    return mo_f16_to_f32(mo_f32_to_f16(mo_f16_to_f32((uint16_t) (x & 0xffffu)) + mo_f16_to_f32((uint16_t) (x >> 16))));
}

/* src/kernels/cpu/exl3_ref.cpp:33-43: step p's state = the 16-bit window ending at bit floor((p+1) k2 / 2) of the
 * tile's 4 k2 words read MSB-first, around the ring */
void mo_exl3_tile_states(const uint32_t* t, int k2, uint16_t* st) {
    const int W = 4 * k2;
    for (int p = 0; p < 256; ++p) {
        const int b1 = ((p + 1) * k2) / 2 + 128 * k2;
        const int i1 = (b1 - 1) >> 5, i0 = (b1 - 16) >> 5;
        const int sh = ((i1 + 1) << 5) - b1;
        const uint64_t m = ((uint64_t) t[i0 % W] << 32) | (uint64_t) t[i1 % W];
        st[p] = (uint16_t) ((m >> sh) & 0xffffu);
    }
}

/* src/kernels/cpu/exl3_ref.cpp:45-59 */
void mo_exl3_inner(const uint32_t* trellis, int ld, int k, int n, int k2, int cb, float* w) {
    const int W = 4 * k2;
    uint16_t st[256];
    for (int ks = 0; ks < k / 16; ++ks)
        for (int tc = 0; tc < n / 16; ++tc) {
            mo_exl3_tile_states(trellis + ((size_t) ks * ld + tc) * W, k2, st);
            for (int p = 0; p < 256; ++p) {
                const int lane = p >> 3, j = p & 7;
                const int r = ks * 16 + (lane & 3) * 2 + (j & 1) + 8 * ((j >> 1) & 1);
                const int c = tc * 16 + (lane >> 2) + 8 * (j >> 2);
                w[(size_t) r * n + c] = mo_exl3_decode(st[p], cb);
            }
        }
}

/* src/kernels/cpu/exl3_ref.cpp:61-75 */
void mo_exl3_had128(float* v, size_t n) {
    const float s = 1.0f / sqrtf(128.0f);
    for (size_t b = 0; b < n; b += 128) {
        float* x = v + b;
        for (int h = 1; h < 128; h <<= 1)
            for (int i = 0; i < 128; i += 2 * h)
                for (int j = i; j < i + h; ++j) {
                    const float a = x[j], c = x[j + h];
                    x[j] = a + c;
                    x[j + h] = a - c;
                }
        for (int i = 0; i < 128; ++i) x[i] *= s;
    }
}

/* src/kernels/cpu/exl3_ref.cpp:77-94 */
void mo_exl3_mv(const float* w, const uint16_t* suh, const uint16_t* svh, int k, int n, const float* x, float* y) {
    float* xh = (float*) malloc(sizeof(float) * (size_t) k);
    double* acc = (double*) calloc((size_t) n, sizeof(double));
    for (int i = 0; i < k; ++i) xh[i] = x[i] * mo_f16_to_f32(suh[i]);
    mo_exl3_had128(xh, (size_t) k);
    for (int i = 0; i < k; ++i) xh[i] = mo_f16_to_f32(mo_f32_to_f16(xh[i]));
    for (int r = 0; r < k; ++r) {
        const double xv = xh[r];
        const float* row = w + (size_t) r * n;
        for (int c = 0; c < n; ++c) acc[c] += xv * row[c];
    }
    for (int c = 0; c < n; ++c) y[c] = (float) acc[c];
    mo_exl3_had128(y, (size_t) n);
    for (int c = 0; c < n; ++c) y[c] *= mo_f16_to_f32(svh[c]);
    free(xh);
    free(acc);
}

/* --------------------------------------------------------------------------------------- synthetic encoders */

/* An own Q4_K encoder (not the reference's: it has none).  Per 32-value sub-block: min/max affine fit with a
 * non-negative offset, 6-bit scales against the super-block's largest scale and largest offset. */
void mo_encode_q4k(const float* x, int64_t k, uint8_t* out) {
    for (int64_t b = 0; b < k / 256; ++b) {
        const float* xb = x + b * 256;
        uint8_t* blk = out + (size_t) b * 144;
        float sc[8], mn[8], maxsc = 0.0f, maxmn = 0.0f;
        for (int j = 0; j < 8; ++j) {
            float lo = xb[32 * j], hi = lo;
            for (int i = 1; i < 32; ++i) {
                const float v = xb[32 * j + i];
                if (v < lo) lo = v;
                if (v > hi) hi = v;
            }
            if (lo > 0.0f) lo = 0.0f;
            sc[j] = (hi - lo) / 15.0f;
            mn[j] = -lo;
            if (sc[j] > maxsc) maxsc = sc[j];
            if (mn[j] > maxmn) maxmn = mn[j];
        }
        const uint16_t dh = mo_f32_to_f16(maxsc / 63.0f), mh = mo_f32_to_f16(maxmn / 63.0f);
        const float d = mo_f16_to_f32(dh), dm = mo_f16_to_f32(mh);
        int ls[8], lm[8];
        for (int j = 0; j < 8; ++j) {
            ls[j] = d > 0.0f ? (int) lrintf(sc[j] / d) : 0;
            lm[j] = dm > 0.0f ? (int) lrintf(mn[j] / dm) : 0;
            if (ls[j] > 63) ls[j] = 63;
            if (lm[j] > 63) lm[j] = 63;
        }
        blk[0] = (uint8_t) (dh & 255);
        blk[1] = (uint8_t) (dh >> 8);
        blk[2] = (uint8_t) (mh & 255);
        blk[3] = (uint8_t) (mh >> 8);
        uint8_t* s = blk + 4;
        memset(s, 0, 12);
        for (int j = 0; j < 8; ++j) {
            if (j < 4) {
                s[j] |= (uint8_t) ls[j];
                s[j + 4] |= (uint8_t) lm[j];
            } else {
                s[j + 4] |= (uint8_t) ((ls[j] & 0x0f) | ((lm[j] & 0x0f) << 4));
                s[j - 4] |= (uint8_t) ((ls[j] >> 4) << 6);
                s[j] |= (uint8_t) ((lm[j] >> 4) << 6);
            }
        }
        for (int j = 0; j < 8; ++j) {
            const float dj = d * (float) ls[j], mj = dm * (float) lm[j];
            for (int i = 0; i < 32; ++i) {
                int q = dj > 0.0f ? (int) lrintf((xb[32 * j + i] + mj) / dj) : 0;
                if (q < 0) q = 0;
                if (q > 15) q = 15;
                uint8_t* dst = blk + 16 + 32 * (j / 2) + i;
                if (j & 1) *dst = (uint8_t) ((*dst & 0x0f) | (q << 4));
                else *dst = (uint8_t) q;
            }
        }
    }
}

void mo_encode_q80(const float* x, int64_t k, uint8_t* out) { mo_quant_q80(x, k, (mo_q80*) out); }

/* ------------------------------------------------------------------------------------------ prefill reference */

/* tests/hip/prefill_fused_parity.cpp:150-175: the double product of dequantized weights and dequantized int8 rows */
void mo_grouped_ref(int type, const uint8_t* const* w, const int32_t* bounds, int n_expert, int64_t k, int64_t n,
                    const int8_t* xq, const float* xd, float* y, int nthreads) {
    const size_t rb = mo_row_bytes(type, k);
    if (nthreads < 1) nthreads = 1;
    for (int e = 0; e < n_expert; ++e) {
        const int r0 = bounds[e], r1 = bounds[e + 1];
        if (r1 <= r0) continue;
#pragma omp parallel num_threads(nthreads)
        {
            float* wf = (float*) malloc(sizeof(float) * (size_t) k);
#pragma omp for schedule(static)
            for (int64_t c = 0; c < n; ++c) {
                mo_dequant_row(type, w[e] + (size_t) c * rb, k, wf);
                for (int r = r0; r < r1; ++r) {
                    double s = 0.0;
                    const int8_t* q = xq + (size_t) r * k;
                    const float* d = xd + (size_t) r * (k / 32);
                    for (int64_t i = 0; i < k; ++i) s += (double) wf[i] * ((double) q[i] * (double) d[i / 32]);
                    y[(size_t) r * n + c] = (float) s;
                }
            }
            free(wf);
        }
    }
}
