// The routed experts' residency tiers, decided on the device per routed expert: the tables of glmf::MoeDev
// (include/strata/kernels/glm_fast.hpp:284-296) and the plan part of moe_route_kernel that reads them
// (src/kernels/cuda/glm_fast.cu:4262-4375), the fetch of moe_fetch_kernel (glm_fast.cu:4688-4704) and tab_update
// (glm_fast.cu:7745-7754).  The request ring to the host, the CPU lane, the prefetch of the next layer and the disk tier
// stay the engine's (the prefetch LIST's copy is here: prefetch_kernel): an expert in neither table is reported in the miss mask and left out of the plan.
#pragma once

namespace maya {

struct Tiers {
    uint64_t* tab;             // [n_keys] HBM address | [n_keys] second-tier address | [n_layers][MAYA_SPARES] free HBM slots
    const uint64_t* scratch;   // [n_scratch] HBM slots for fetched experts that are not promoted
    uint64_t* fetch_src;       // [n_tokens * k] out
    uint32_t* counts;          // [n_keys] or null
    uint32_t* seq;             // [1] or null: the routes so far (the counts halve when it reaches a multiple of 4096)
    uint32_t* masks;           // [n_tokens][4] out: miss, fetch, promoted, no slot left
    int n_keys, n_scratch;
};

template <typename T> __device__ __forceinline__ T tier_load(const T* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One workgroup of 256; the tokens one after another (a window's tokens take the spares and the scratch slots in order,
// as one moe_route call a token does).
__global__ __launch_bounds__(256) void route_tiered_kernel(const float* __restrict__ logits, int n_tokens, int n_expert, int k,
                                                           RouterSpec rs, int layer, Tiers r, int promote_min,
                                                           int32_t* __restrict__ ids, float* __restrict__ weights,
                                                           uint64_t* __restrict__ plan) {
    __shared__ RouterLds sm;
    __shared__ uint64_t s_tab[MAYA_MAX_K], s_rtab[MAYA_MAX_K];
    __shared__ uint32_t s_cnt[MAYA_MAX_K];
    const int tid = threadIdx.x;
    uint64_t* const rtab = r.tab + r.n_keys;
    uint64_t* const spares = r.tab + 2 * (size_t) r.n_keys + (size_t) layer * MAYA_SPARES;
    int next_spare = 0, next_scratch = 0;   // (thread 0's)
    for (int t = 0; t < n_tokens; ++t) {
        // (words an earlier token of this launch may have written are read past the CU's cache)
        if (r.counts != nullptr && r.seq != nullptr && ((tier_load(r.seq) + 1u) & 4095u) == 0u) {
            for (int i = tid; i < r.n_keys; i += 256) r.counts[i] = tier_load(r.counts + i) >> 1;
            __threadfence();
        }
        route_any(logits + (size_t) t * n_expert, n_expert, k, rs, sm);
        // a thread an entry: its count and its two table words (a route's keys are distinct)
        if (tid < k) {
            const int id = sm.id[tid];
            if (id >= 0) {
                const size_t key = (size_t) layer * n_expert + id;
                s_cnt[tid] = r.counts != nullptr ? atomicAdd(r.counts + key, 1u) + 1u : 0u;
                s_tab[tid] = tier_load(r.tab + key);
                s_rtab[tid] = tier_load(rtab + key);
            } else {
                s_cnt[tid] = 0u, s_tab[tid] = 0ull, s_rtab[tid] = 0ull;
            }
        }
        __syncthreads();
        if (tid == 0) {
            uint32_t miss = 0u, fetch = 0u, promo = 0u, full = 0u;
            for (int i = 0; i < k; ++i) {
                const int id = sm.id[i];
                uint64_t ptr = s_tab[i], src = 0ull;
                if (id >= 0 && ptr == 0ull) {
                    src = s_rtab[i];
                    if (src == 0ull) {
                        miss |= 1u << i;   // in neither tier: the engine's to provide
                    } else {
                        while (next_spare < MAYA_SPARES && tier_load(spares + next_spare) == 0ull) ++next_spare;
                        if (next_spare < MAYA_SPARES && (promote_min <= 1 || s_cnt[i] >= (uint32_t) promote_min)) {
                            ptr = tier_load(spares + next_spare);
                            spares[next_spare] = 0ull;
                            r.tab[(size_t) layer * n_expert + id] = ptr;   // resident from here on
                            promo |= 1u << i;
                        } else if (next_scratch < r.n_scratch) {
                            ptr = r.scratch[next_scratch++];
                        } else {
                            full |= 1u << i;   // left out
                            src = 0ull;
                        }
                        if (src != 0ull) fetch |= 1u << i;
                    }
                }
                ids[(size_t) t * k + i] = id;
                weights[(size_t) t * k + i] = sm.w[i];
                plan[(size_t) t * k + i] = ptr;
                r.fetch_src[(size_t) t * k + i] = src;
            }
            r.masks[4 * t + 0] = miss;
            r.masks[4 * t + 1] = fetch;
            r.masks[4 * t + 2] = promo;
            r.masks[4 * t + 3] = full;
            if (r.seq != nullptr) *r.seq = tier_load(r.seq) + 1u;
        }
        // (the next token reads the table words and the counter this one wrote)
        __threadfence();
        __syncthreads();
    }
}

// The same plan over already routed ids, for a window of tokens (n = n_tokens * k <= 256 entries): one workgroup, a thread
// an entry fetches its table words, thread 0 then walks the entries in order out of LDS (a promotion is carried to the
// later entries of the same expert), and every thread writes its entry's results.  The counts stay per token (a token
// after a halving must see halved counts): one round of atomics a token, only when counts are kept.
__global__ __launch_bounds__(256) void plan_tiered_kernel(const int32_t* __restrict__ ids, int n_tokens, int n_expert, int k, int layer,
                                                          Tiers r, int promote_min, uint64_t* __restrict__ plan) {
    __shared__ uint64_t s_tab[256], s_rtab[256], s_plan[256], s_src[256];
    __shared__ uint32_t s_cnt[256], s_mask[256][4];
    __shared__ int s_id[256];
    const int tid = threadIdx.x, n = n_tokens * k;
    uint64_t* const rtab = r.tab + r.n_keys;
    uint64_t* const spares = r.tab + 2 * (size_t) r.n_keys + (size_t) layer * MAYA_SPARES;
    const int id = tid < n ? ids[tid] : -1;
    const size_t key = (size_t) layer * n_expert + (id >= 0 ? id : 0);
    if (tid < n) {
        s_id[tid] = id;
        s_tab[tid] = id >= 0 ? tier_load(r.tab + key) : 0ull;
        s_rtab[tid] = id >= 0 ? tier_load(rtab + key) : 0ull;
        s_cnt[tid] = 0u;
    }
    if (r.counts != nullptr) {
        const uint32_t seq0 = r.seq != nullptr ? tier_load(r.seq) : 1u;
        for (int t = 0; t < n_tokens; ++t) {
            if (r.seq != nullptr && ((seq0 + (uint32_t) t + 1u) & 4095u) == 0u) {
                for (int i = tid; i < r.n_keys; i += 256) r.counts[i] = tier_load(r.counts + i) >> 1;
                __threadfence();
                __syncthreads();
            }
            if (tid >= t * k && tid < (t + 1) * k && id >= 0) s_cnt[tid] = atomicAdd(r.counts + key, 1u) + 1u;
            __threadfence();
            __syncthreads();
        }
    }
    __syncthreads();
    if (tid == 0) {
        int next_spare = 0, next_scratch = 0;
        uint64_t sp[MAYA_SPARES];
        for (int j = 0; j < MAYA_SPARES; ++j) sp[j] = tier_load(spares + j);
        for (int t = 0; t < n_tokens; ++t) {
            uint32_t miss = 0u, fetch = 0u, promo = 0u, full = 0u;
            for (int i = 0; i < k; ++i) {
                const int e = t * k + i, eid = s_id[e];
                uint64_t ptr = s_tab[e], src = 0ull;
                if (eid >= 0 && ptr == 0ull) {
                    src = s_rtab[e];
                    if (src == 0ull) {
                        miss |= 1u << i;
                    } else {
                        while (next_spare < MAYA_SPARES && sp[next_spare] == 0ull) ++next_spare;
                        if (next_spare < MAYA_SPARES && (promote_min <= 1 || s_cnt[e] >= (uint32_t) promote_min)) {
                            ptr = sp[next_spare];
                            sp[next_spare] = 0ull;
                            spares[next_spare] = 0ull;
                            r.tab[(size_t) layer * n_expert + eid] = ptr;
                            for (int f = e + 1; f < n; ++f)
                                if (s_id[f] == eid) s_tab[f] = ptr;   // resident for the window's later tokens
                            promo |= 1u << i;
                        } else if (next_scratch < r.n_scratch) {
                            ptr = r.scratch[next_scratch++];
                        } else {
                            full |= 1u << i;
                            src = 0ull;
                        }
                        if (src != 0ull) fetch |= 1u << i;
                    }
                }
                s_plan[e] = ptr;
                s_src[e] = src;
            }
            s_mask[t][0] = miss, s_mask[t][1] = fetch, s_mask[t][2] = promo, s_mask[t][3] = full;
        }
        if (r.seq != nullptr) *r.seq = tier_load(r.seq) + (uint32_t) n_tokens;
    }
    __syncthreads();
    if (tid < n) {
        plan[tid] = s_plan[tid];
        r.fetch_src[tid] = s_src[tid];
    }
    if (tid < 4 * n_tokens) r.masks[tid] = s_mask[tid >> 2][tid & 3];
}

// grid (slices, entries): entry blockIdx.y's blob from its source into its slot, 16 bytes a lane where both are aligned
__global__ __launch_bounds__(256) void fetch_kernel(const uint64_t* __restrict__ fetch_src, const uint64_t* __restrict__ plan, size_t n) {
    const uint8_t* src = (const uint8_t*) fetch_src[blockIdx.y];
    uint8_t* dst = (uint8_t*) plan[blockIdx.y];
    if (src == nullptr || dst == nullptr) return;
    const size_t i0 = (size_t) blockIdx.x * 256 + threadIdx.x, step = (size_t) gridDim.x * 256;
    if ((((uintptr_t) src | (uintptr_t) dst) & 15) == 0) {
        const size_t n16 = n >> 4;
        for (size_t i = i0; i < n16; i += step) ((uint4*) dst)[i] = ((const uint4*) src)[i];
        for (size_t i = (n16 << 4) + i0; i < n; i += step) dst[i] = src[i];
    } else {
        for (size_t i = i0; i < n; i += step) dst[i] = src[i];
    }
}

// The prefetch list's copy (moe_prefetch_kernel, glm_fast.cu:4619-4627): *n_list entries - the count is the device's, read
// here - of n bytes each from src[i] to dst[i], by however many workgroups the caller grants (it runs beside the main
// stream's kernels: every compute unit it holds is one they wait for).  Entry after entry, the workgroups striding
// through each; a null source or slot is skipped.
__global__ __launch_bounds__(256) void prefetch_kernel(const uint64_t* __restrict__ src_list, const uint64_t* __restrict__ dst_list,
                                                       const int32_t* __restrict__ n_list, int max_entries, size_t n) {
    const int cnt = min(max(*n_list, 0), max_entries);
    const size_t i0 = (size_t) blockIdx.x * 256 + threadIdx.x, step = (size_t) gridDim.x * 256;
    for (int e = 0; e < cnt; ++e) {
        const uint8_t* src = (const uint8_t*) src_list[e];
        uint8_t* dst = (uint8_t*) dst_list[e];
        if (src == nullptr || dst == nullptr) continue;
        if ((((uintptr_t) src | (uintptr_t) dst) & 15) == 0) {
            const size_t n16 = n >> 4;
            for (size_t i = i0; i < n16; i += step) ((uint4*) dst)[i] = ((const uint4*) src)[i];
            for (size_t i = (n16 << 4) + i0; i < n; i += step) dst[i] = src[i];
        } else {
            for (size_t i = i0; i < n; i += step) dst[i] = src[i];
        }
    }
}

__global__ void tab_update_kernel(uint64_t* __restrict__ tab, const int32_t* __restrict__ keys, const uint64_t* __restrict__ vals, int n,
                                  int n_words) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && keys[i] >= 0 && keys[i] < n_words) tab[keys[i]] = vals[i];
}

}  // namespace maya
