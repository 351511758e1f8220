// maya_prefill_iq2s.hpp - the prompt chunk's grouped GEMM on IQ2_S rows in the stream packing (included by
// maya_prefill.hip inside namespace maya; the skeleton - tiles, the activations' copies, the barriers - is pf_tile's).
// out[row][n] = 1/8 sum over blocks b of (d_w[n][b] d_x[row][b]) * sum over the block's 16-value groups j of (2 ls_j +
// 1) (w_j . c_j), w = the grid magnitudes with their signs: the integer sums of the CPU path's IQ2_S x Q8_K row dot
// (src/kernels/cpu/iq_avx2.cpp:160-176, 225-250).  The scale belongs to 16 values and (2 ls + 1) x 43 does not fit
// int8, so a 32-deep matrix instruction takes ONE group: a lane (row ln, k-group kg) decodes grid entry kg of a sub-
// block - 8 signed bytes (the grid's magnitudes and a sign-mask table sit in LDS), its whole operand - and the two
// groups of a sub-block come from two instructions whose operands are zero in the lanes of the other group (kg < 2:
// values 0..15, kg >= 2: 16..31).  The vector ALU then adds (2 ls + 1) x the group's sums to the block's int32 sums:
// two multiply-adds an output a sub-block.  Weights go global -> LDS without registers, one super-block ahead: per
// tile of 16 rows (4 quads) the 8 sub-blocks' index + sign words (1024 bytes: one 16-byte copy a lane) and their qh /
// scale bytes (256 bytes: one 4-byte copy a lane), each lane's source chosen so that LDS holds [sub-block][quad][row]:
// the 16 rows of a read then sit in 16 different bank pairs.  The block scales (2 bytes a row a block) come through a
// register.

constexpr int kIqTileBytes = 1280, kIqWaveBytes = 2 * kIqTileBytes, kIqBufBytes = 4 * kIqWaveBytes;

template <bool GU, int NMT>
__device__ __forceinline__ void pf_tile_iq2s(const PfGemm& a, uint8_t* b0, uint8_t* b1, uint8_t* b2, uint8_t* w0, uint8_t* w1,
                                             uint32_t grid_lds, int ex, int row0, int nrows) {
    typedef const __attribute__((address_space(1))) uint8_t* wptr;
    const uint64_t blob = a.table[ex];
    const int tid = threadIdx.x, lane = tid & 63, ln = lane & 15, kg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nsb = (int) (a.k >> 8), nu = nsb * 8;
    const uint32_t qb = 4u * (uint32_t) nsb * 82u;   // bytes of a quad of rows

    int64_t n0;   // the wave's first feature (gate/up) or output row (down)
    uint64_t base[2];   // the first quad of each of the wave's two tiles
    if constexpr (GU) {
        n0 = (int64_t) blockIdx.x * 64 + wave * 16;
#pragma unroll
        for (int t = 0; t < 2; ++t) base[t] = blob + a.off[t] + (uint64_t) (n0 >> 2) * qb;
    } else {
        n0 = (int64_t) blockIdx.x * 128 + wave * 32;
#pragma unroll
        for (int t = 0; t < 2; ++t) base[t] = blob + a.off[0] + (uint64_t) ((n0 + 16 * t) >> 2) * qb;
    }
    const bool wave_on = n0 < a.n;   // (a.n is a multiple of the wave's rows: checked on the host)

    v4f acc[2][NMT];
    v4i isum[2][NMT];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int m = 0; m < NMT; ++m) acc[t][m] = v4f{0.0f, 0.0f, 0.0f, 0.0f}, isum[t][m] = v4i{0, 0, 0, 0};

    PfDma<NMT, false> dma;
    dma.init(a, row0, nrows, wave, lane);
    // the weights' copies: lane L fills LDS piece L = [sub-block L >> 3][quad (L >> 1) & 3][row pair L & 1]
    __amdgpu_buffer_rsrc_t wr[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const uint32_t lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) base[t]);
        const uint32_t hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (base[t] >> 32));
        wr[t] = __builtin_amdgcn_make_buffer_rsrc((void*) (((uint64_t) hi << 32) | lo), 0, (int) (4u * qb), 0x00020000);
    }
    const uint32_t cu = (uint32_t) (lane >> 3), cq = (uint32_t) ((lane >> 1) & 3), cp = (uint32_t) (lane & 1);
    const uint32_t oi = cq * qb + 8u * (4u * cu + 2u * cp), oh = cq * qb + 32u * (uint32_t) nu + 2u * (4u * cu + 2u * cp);
    auto wcopy = [&](uint8_t* wbuf, int sb) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            uint8_t* dst = wbuf + wave * kIqWaveBytes + t * kIqTileBytes;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(wr[t], (pf_lptr) dst, 16, oi, sb * 256, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(wr[t], (pf_lptr) (dst + 1024), 4, oh, sb * 64, 0, 0);
        }
    };
    // the block scale of the lane's row: 2 bytes at 40 nu + 2 (4 b + r) of its quad
    wptr dp[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) dp[t] = (wptr) base[t] + (size_t) (ln >> 2) * qb + 40u * (uint32_t) nu + 2u * (uint32_t) (ln & 3);
    uint32_t dh[2] = {0u, 0u}, dhn[2] = {0u, 0u};
    auto load_d = [&](int sb, uint32_t (&o)[2]) {
#pragma unroll
        for (int t = 0; t < 2; ++t) o[t] = *(const __attribute__((address_space(1))) uint16_t*) (dp[t] + 8 * sb);
    };

    dma.copy(b0, 0);
    if (nsb > 1) dma.copy(b1, 1);
    if (wave_on) {
        wcopy(w0, 0);
        load_d(0, dh);
    }
    // lane constants of the decode: the entry's byte and its two high bits, the group masks, the activations' place
    const uint32_t sh8 = 8u * (uint32_t) kg, sh2 = 2u * (uint32_t) kg;
    const uint32_t m0 = kg < 2 ? 0xffffffffu : 0u, m1 = ~m0;
    const uint32_t w_rd = (uint32_t) (wave * kIqWaveBytes + (ln >> 2) * 32 + (ln & 3) * 8);
    const uint32_t h_rd = (uint32_t) (wave * kIqWaveBytes + 1024 + (ln >> 2) * 8 + (ln & 3) * 2);
    const int a_base = ln * 256 + 8 * (kg & 1), a_swz = (ln ^ (kg >> 1)) << 4;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    auto step = [&](int sb, const uint8_t* buf, uint8_t* buf2, const uint8_t* wbuf, uint8_t* wbuf2) {
        const bool more = sb + 2 < nsb;
        if (wave_on && sb + 1 < nsb) {
            load_d(sb + 1, dhn);
            wcopy(wbuf2, sb + 1);
        }
        // (after the weights' copies, so that waiting for everything but these copies covers the weights too)
        if (more) dma.copy(buf2, sb + 2);
        if (wave_on) {
            const uint32_t lbuf = pf_lds_addr(buf), lw = pf_lds_addr(wbuf);
#pragma unroll 1
            for (int u = 0; u < 8; ++u) {
                // the activations' 8 codes of this lane's k-group: chunk 2 u + (kg >> 1) of the row, its half kg & 1
                pf_i2 xr[NMT];
                {
                    const uint32_t at = lbuf + a_base + (a_swz ^ (32 * u));
                    pf_for_m<0, NMT>([&](auto mc) {
                        constexpr int m = decltype(mc)::value;
                        xr[m] = pf_lds_b64<m * 4096>(at);
                    });
                }
                pf_i2 iw[2];
                uint32_t hs[2];
                iw[0] = pf_lds_b64<0>(lw + w_rd + 128 * u);
                iw[1] = pf_lds_b64<kIqTileBytes>(lw + w_rd + 128 * u);
                hs[0] = pf_lds_u16<0>(lw + h_rd + 32 * u);
                hs[1] = pf_lds_u16<kIqTileBytes>(lw + h_rd + 32 * u);
                pf_lds_wait(iw);
                pf_lds_wait(hs);
                pf_i2 gr[2];
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const uint32_t idx = __builtin_amdgcn_ubfe((uint32_t) iw[t].x, sh8, 8u), hi2 = __builtin_amdgcn_ubfe(hs[t], sh2, 2u);
                    const uint32_t ga = grid_lds + ((idx | (hi2 << 8)) << 3);
                    gr[t] = pf_lds_b64<0>(ga);
                }
                // the signs: the entry's sign byte -> 0xff in the bytes of its set bits (a 256-entry table beside the grid)
                pf_i2 sm[2];
                int s0[2], s1[2];
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const uint32_t sbyte = __builtin_amdgcn_ubfe((uint32_t) iw[t].y, sh8, 8u);
                    sm[t] = pf_lds_b64<8192>(grid_lds + (sbyte << 3));
                    const uint32_t sc = hs[t] >> 8;
                    s0[t] = (int) (2u * (sc & 15u) + 1u);
                    s1[t] = (int) (2u * (sc >> 4) + 1u);
                }
                pf_lds_wait(gr);
                pf_lds_wait(sm);
                pf_lds_wait(xr);
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    // the marked bytes negated: (g ^ 0xff) + 1 a byte, no carry (no magnitude is 0)
                    const uint32_t ma = (uint32_t) sm[t].x, mb = (uint32_t) sm[t].y;
                    const uint32_t wa = ((uint32_t) gr[t].x ^ ma) + (ma & 0x01010101u), wb = ((uint32_t) gr[t].y ^ mb) + (mb & 0x01010101u);
                    const long o0 = (long) (((uint64_t) (wb & m0) << 32) | (uint64_t) (wa & m0));
                    const long o1 = (long) (((uint64_t) (wb & m1) << 32) | (uint64_t) (wa & m1));
#pragma unroll
                    for (int m = 0; m < NMT; ++m) {
                        const long xa = (long) (((uint64_t) (uint32_t) xr[m].y << 32) | (uint64_t) (uint32_t) xr[m].x);
                        const v4i z = {0, 0, 0, 0};
                        const v4i d0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(xa, o0, z, 0, 0, 0);
                        const v4i d1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(xa, o1, z, 0, 0, 0);
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                        {   // two 24-bit multiply-adds (kept apart: joined, the compiler makes two multiplies and a 3-way add)
                            int v = __mul24(s0[t], d0[i]) + isum[t][m][i];
                            asm("" : "+v"(v));
                            isum[t][m][i] = __mul24(s1[t], d1[i]) + v;
                        }
                    }
                }
            }
            // once a block: the integer sums times the two block scales
            v4f dxr[NMT];
            pf_for_m<0, NMT>([&](auto mc) {
                constexpr int m = decltype(mc)::value;
                dxr[m] = pf_lds_f32x4<kPfDOffNoS + m * 64>(lbuf + 16 * kg);
            });
            float d[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) d[t] = f16_bits_to_f32((uint16_t) dh[t]);
            pf_lds_wait(dxr);
#pragma unroll
            for (int m = 0; m < NMT; ++m) {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        acc[t][m][i] = fmaf(__fmul_rn(dxr[m][i], d[t]), (float) isum[t][m][i], acc[t][m][i]);
                        isum[t][m][i] = 0;
                    }
                }
            }
            dh[0] = dhn[0], dh[1] = dhn[1];
        }
        // super-block sb + 1 (activations and weights) has landed once only this iteration's activation copies (of
        // sb + 2) may still be in flight; without such copies everything must have landed
        if (more) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(NMT) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };
    for (int sb = 0; sb < nsb; sb += 6) {
        step(sb, b0, b2, w0, w1);
        if (sb + 1 < nsb) step(sb + 1, b1, b0, w1, w0);
        if (sb + 2 < nsb) step(sb + 2, b2, b1, w0, w1);
        if (sb + 3 < nsb) step(sb + 3, b0, b2, w1, w0);
        if (sb + 4 < nsb) step(sb + 4, b1, b0, w0, w1);
        if (sb + 5 < nsb) step(sb + 5, b2, b1, w1, w0);
    }
    if (!wave_on) return;

    // outputs: lane (ln, kg) holds weight row ln of each tile for the tokens 16 m + 4 kg + i
#pragma unroll
    for (int m = 0; m < NMT; ++m) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = 16 * m + 4 * kg + i;
            if (r >= nrows) continue;
            float* o = a.out + (size_t) (row0 + r) * a.n + n0 + ln;
            const float v0 = __fmul_rn(acc[0][m][i], 0.125f), v1 = __fmul_rn(acc[1][m][i], 0.125f);
            if constexpr (GU) o[0] = pf_swiglu(v0, v1, a.limit);
            else o[0] = v0, o[16] = v1;
        }
    }
}

// grid (bands of weight rows, tiles at most)
template <bool GU>
__global__ __launch_bounds__(256, 2) void prefill_iq2s_kernel(PfGemm a, Codebooks cb) {
    __shared__ __attribute__((aligned(16))) uint8_t b0[kPfBufBytesNoS], b1[kPfBufBytesNoS], b2[kPfBufBytesNoS];
    __shared__ __attribute__((aligned(16))) uint8_t w0[kIqBufBytes], w1[kIqBufBytes];
    __shared__ __attribute__((aligned(16))) uint64_t grid[1024 + 256];   // the magnitudes, then the sign masks
    const int tile = blockIdx.y;
    if (tile >= *a.plan.n_tiles) return;
    for (int i = threadIdx.x; i < 1024; i += 256) grid[i] = cb.iq2s[i];
    {
        uint64_t m = 0ull;
#pragma unroll
        for (int b = 0; b < 8; ++b)
            if (threadIdx.x & (1 << b)) m |= 0xffull << (8 * b);
        grid[1024 + threadIdx.x] = m;
    }
    const int ex = a.plan.tile_expert[tile], row0 = a.plan.tile_row0[tile];
    const int nrows = min(kPfRows, a.plan.bounds[ex + 1] - row0);
    const uint32_t gl = pf_lds_addr(grid);
    switch ((nrows + 15) >> 4) {
        case 1: pf_tile_iq2s<GU, 1>(a, b0, b1, b2, w0, w1, gl, ex, row0, nrows); break;
        case 2: pf_tile_iq2s<GU, 2>(a, b0, b1, b2, w0, w1, gl, ex, row0, nrows); break;
        case 3: pf_tile_iq2s<GU, 3>(a, b0, b1, b2, w0, w1, gl, ex, row0, nrows); break;
        default: pf_tile_iq2s<GU, 4>(a, b0, b1, b2, w0, w1, gl, ex, row0, nrows); break;
    }
}
