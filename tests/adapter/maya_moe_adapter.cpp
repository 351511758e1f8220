// maya_moe_adapter.cpp - what a maintainer of the reference engine adds to forward its routed-expert operators to
// libmaya_moe.so (include/maya_moe.h).  It defines, with the reference's own signatures, the entry points the engines call:
//
//   strata::ds4::gguf::moe_gate_up / moe_down / win_experts   (src/ds4/ds4_gguf.cuh:95-99; F32 x and h at the boundary)
//   strata::kernels::glmf::moe_gate_up / moe_down             (include/strata/kernels/glm_fast.hpp:496-501)
//   strata::kernels::exl3::moe_gate_up / moe_down / win_experts (include/strata/kernels/exl3.hpp:133-169)
//   the probes and switches beside them (moe_supported, iq::supported, set_skip, launch_errors)
//
// It is compiled in place of src/kernels/cuda/glm_fast.cu's / src/ds4/ds4_gguf.cu's / src/kernels/cuda/exl3.cu's definitions
// of those symbols in the reference's HIP build (which force-includes include/strata/hip_compat/cuda_runtime.h, so
// cudaStream_t below is hipStream_t).  tests/test_abi_compiles.py syntax-checks this file against the reference's headers.
#include "maya_moe.h"

#include <atomic>
#include <cstdio>
#include <mutex>
#include <unordered_map>

#include "strata/kernels/exl3.hpp"
#include "strata/kernels/glm_fast.hpp"
#include "ds4_gguf.cuh"
#include "ds4_iq.cuh"

namespace maya_adapter {

std::atomic<int> g_launch_errors{0};
thread_local const int* g_skip = nullptr;   // glmf::set_skip's / exl3::set_skip's thread-local flag (glm_fast.hpp:72-75)

// The reference's three error styles (printed + counted; "not covered, nothing launched"; a HIP error) from one status code.
inline bool ok(int rc, const char* what) {
    if (rc == MAYA_OK) return true;
    if (rc < 0) {
        g_launch_errors.fetch_add(1, std::memory_order_relaxed);
        std::fprintf(stderr, "%s: %s\n", what, maya_last_error());
    }
    return false;   // rc > 0: not covered, nothing launched - the caller takes its other path
}

// ---- per-stream scratch, as exl3::prepare / ds4 gguf's scratch(s) keep it (include/strata/kernels/exl3.hpp:88-92):
// allocated once a stream, before a graph capture; the library itself never allocates.
constexpr int kMaxTok = MAYA_MAX_TOKENS, kK = 8, kMaxEmbd = 8192, kMaxFf = 4096;
struct Scratch {
    maya_act x{}, hq{};
    float *h = nullptr, *part = nullptr;
    unsigned long long* grp_ptr = nullptr;
    int *grp_start = nullptr, *grp_ent = nullptr, *n_groups = nullptr;
};
inline Scratch* scratch(cudaStream_t s) {
    static std::mutex mu;
    static std::unordered_map<cudaStream_t, Scratch> map;
    std::lock_guard<std::mutex> lock(mu);
    auto it = map.find(s);
    if (it != map.end()) return &it->second;
    Scratch sc;
    const size_t ent = (size_t) kMaxTok * kK;
    auto dev = [](size_t n) {
        void* p = nullptr;
        return cudaMalloc(&p, n) == cudaSuccess ? p : nullptr;
    };
    sc.x = maya_act{(int8_t*) dev((size_t) kMaxTok * kMaxEmbd), (float*) dev(sizeof(float) * kMaxTok * (kMaxEmbd / 32)),
                    (int16_t*) dev(sizeof(int16_t) * kMaxTok * (kMaxEmbd / 16))};
    sc.hq = maya_act{(int8_t*) dev(ent * kMaxFf), (float*) dev(sizeof(float) * ent * (kMaxFf / 32)),
                     (int16_t*) dev(sizeof(int16_t) * ent * (kMaxFf / 16))};
    sc.h = (float*) dev(sizeof(float) * ent * kMaxFf);
    sc.part = (float*) dev(sizeof(float) * ent * kMaxEmbd);
    sc.grp_ptr = (unsigned long long*) dev(sizeof(unsigned long long) * ent);
    sc.grp_start = (int*) dev(sizeof(int) * (ent + 1));
    sc.grp_ent = (int*) dev(sizeof(int) * ent);
    sc.n_groups = (int*) dev(sizeof(int));
    if (!sc.x.q || !sc.x.d || !sc.x.bsums || !sc.hq.q || !sc.hq.d || !sc.hq.bsums || !sc.h || !sc.part || !sc.grp_ptr ||
        !sc.grp_start || !sc.grp_ent || !sc.n_groups)
        return nullptr;
    return &map.emplace(s, sc).first->second;
}

// A GGUF expert layer's geometry from the engine's layout record (ds4_gguf.cuh:39-45: role r's rows at trellis[r], its
// ggml type in gg_type[r]).  The blobs are the file's own rows (MAYA_PACK_GGUF); an engine that regroups its slots with
// maya_moe_repack at upload passes MAYA_PACK_STREAM here instead.
inline bool gguf_layout(const strata::kernels::exl3::ExpertLayout& lay, int n_embd, int n_ff, int packing, maya_moe_layout* l) {
    namespace g = strata::ds4::gguf;
    if (maya_moe_layout_init(l, g::expert_type(lay, 0), g::expert_type(lay, 1), g::expert_type(lay, 2), n_embd, n_ff) == 0) return false;
    l->gate_off = lay.trellis[0];
    l->up_off = lay.trellis[1];
    l->down_off = lay.trellis[2];
    l->packing = packing;
    return true;
}

// One token's (T = 1) or a window's routed experts through the library: Q8_K of x, gate / up + SwiGLU, Q8_K of h (in the
// down kernel's prologue where it can), down, the weighted sum in plan order + the CPU lane's flagged part + sh_out.
inline bool run_gguf(const strata::kernels::exl3::ExpertLayout& lay, const unsigned long long* plan_ptr, const float* plan_w,
                     const float* cpu_part, const int* cpu_flag, int T, int k, int n_embd, int n_ff, float limit, const float* x,
                     size_t x_stride, float* h, const float* sh_out, float* out, bool gate_up, bool down, cudaStream_t s) {
    Scratch* sc = scratch(s);
    maya_moe_args a{};
    if (!sc || T > kMaxTok || k > kK || n_embd > kMaxEmbd || n_ff > kMaxFf || !gguf_layout(lay, n_embd, n_ff, MAYA_PACK_GGUF, &a.layout))
        return false;
    a.n_tokens = T;
    a.k = k;
    a.plan_ptr = (const uint64_t*) plan_ptr;
    a.plan_w = plan_w;
    a.skip = g_skip;
    a.limit = limit;
    a.x = sc->x;
    a.h = h;
    a.hq = sc->hq;
    a.part = sc->part;
    a.add = cpu_part;
    a.add_flag = cpu_flag;
    a.add2 = sh_out;
    a.out = out;
    if (T > 1) {   // a window: each distinct expert's rows read once for the tokens it serves (glmf::moe_win_group's groups)
        if (!ok(maya_moe_group(a.plan_ptr, T * k, (uint64_t*) sc->grp_ptr, sc->grp_start, sc->grp_ent, sc->n_groups, s), "moe_group")) return false;
        a.grp_ptr = (const uint64_t*) sc->grp_ptr;
        a.grp_start = sc->grp_start;
        a.grp_ent = sc->grp_ent;
        a.n_groups = sc->n_groups;
    }
    if (gate_up) {
        if (!ok(maya_quant_act(a.layout.gate_type, x, MAYA_DT_F32, (int64_t) x_stride, T, n_embd, sc->x, s), "quant_act(x)")) return false;
        if (!ok(maya_moe_gate_up(&a, s), "moe_gate_up")) return false;
    }
    if (down) {
        if (maya_moe_down_rounds_h(&a)) {
            a.hq = maya_act{nullptr, nullptr, nullptr};
            a.part = nullptr;
        } else if (!ok(maya_quant_act(a.layout.down_type, h, MAYA_DT_F32, 0, T * k, n_ff, sc->hq, s), "quant_act(h)")) {
            return false;
        }
        if (!ok(maya_moe_down(&a, s), "moe_down")) return false;
    }
    return true;
}

// glmf's activation buffers are opaque to its callers (`const void* xq`, `void* hq`: block_q8_1 in the reference).  Here
// they hold the library's activation rows instead - the engine sizes them with act_bytes / hq_bytes and fills xq with
// quant_x below where it called its q8_1 quantizer (glm_fast_path.cu:2688-2691) - Q8_K rounding, the CPU expert path's.
inline size_t act_bytes(int rows, int k) { return (size_t) rows * ((size_t) k + 4 * (size_t) (k / 32) + 2 * (size_t) (k / 16)); }
inline maya_act act_view(const void* p, int rows, int k) {
    int8_t* q = (int8_t*) p;
    float* d = (float*) (q + (size_t) rows * k);
    return maya_act{q, d, (int16_t*) (d + (size_t) rows * (k / 32))};
}
inline size_t hq_bytes(int entries, int n_ff) { return sizeof(float) * (size_t) entries * n_ff + act_bytes(entries, n_ff); }
inline bool quant_x(int gu_type, const float* x, int rows, int k, void* xq, cudaStream_t s) {
    return ok(maya_quant_act(gu_type, x, MAYA_DT_F32, 0, rows, k, act_view(xq, rows, k), s), "quant_x");
}

}  // namespace maya_adapter

// ================================================================================ ds4 GGUF experts (F32 x, F32 h)
namespace strata::ds4::gguf {
bool prepare(cudaStream_t s) { return maya_init() == MAYA_OK && maya_adapter::scratch(s) != nullptr; }
int launch_errors() { return maya_adapter::g_launch_errors.load(std::memory_order_relaxed); }
bool expert_type_ok(int type) { return maya_moe_supported(type) != 0; }

void moe_gate_up(const x3::MoeArgs& a, const float* x, float* h, cudaStream_t s) {
    maya_adapter::run_gguf(a.lay, a.plan_ptr, a.plan_w, nullptr, nullptr, 1, a.k, a.n_embd, a.n_ff, a.limit, x, 0, h, nullptr, nullptr,
                           true, false, s);
}
void moe_down(const x3::MoeArgs& a, const float* h, const float* sh_out, float* out, cudaStream_t s) {
    maya_adapter::run_gguf(a.lay, a.plan_ptr, a.plan_w, a.cpu_part, a.cpu_flag, 1, a.k, a.n_embd, a.n_ff, a.limit, nullptr, 0,
                           const_cast<float*>(h), sh_out, out, false, true, s);
}
bool win_experts(const x3::WinArgs& a, cudaStream_t s) {
    if (a.out_stride != 0 && a.out_stride != (size_t) a.n_embd) return false;   // (the library writes dense [T][n_embd] rows)
    if (a.cpu_part && a.cpu_stride != 0 && a.cpu_stride != (size_t) a.n_embd) return false;
    return maya_adapter::run_gguf(a.lay, a.plan_ptr, a.plan_w, a.cpu_part, a.cpu_flag, a.T, a.k, a.n_embd, a.n_ff, a.limit, a.x,
                                  a.x_stride, a.h, a.sh_out, a.out, true, true, s);
}
}  // namespace strata::ds4::gguf

namespace strata::ds4::iq {
bool supported(int type) { return maya_moe_supported(type) != 0; }
bool expert_supported(int type) { return maya_moe_supported(type) != 0; }
bool down_supported(int type) { return maya_moe_supported(type) != 0; }
int block_bytes(int type) { return maya_moe_block_bytes(type); }
}  // namespace strata::ds4::iq

// ================================================================================ glm5 fast path (MoeDev plans)
namespace strata::kernels::glmf {
bool moe_supported(int type) { return maya_moe_supported(type) != 0; }
int launch_errors() { return maya_adapter::g_launch_errors.load(std::memory_order_relaxed); }
void set_skip(const int* flag) { maya_adapter::g_skip = flag; }

static bool glmf_args(int gu_type, int d_type, const MoeDev& d, int k, int n_embd, int n_ff, size_t down_off, float limit,
                      const void* xq, void* hq, maya_moe_args* a) {
    *a = maya_moe_args{};
    if (maya_moe_layout_init(&a->layout, gu_type, gu_type, d_type, n_embd, n_ff) == 0) return false;
    if (down_off) a->layout.down_off = down_off;   // [gate | up | down]: the same offsets the engine's blobs have
    a->n_tokens = 1;
    a->k = k;
    a->plan_ptr = (const uint64_t*) d.plan_ptr;   // 0 = an expert the GPU does not compute (glm_fast.hpp:297)
    a->plan_w = d.plan_w;
    a->skip = d.skip ? d.skip : maya_adapter::g_skip;
    a->limit = limit;
    if (xq) a->x = maya_adapter::act_view(xq, 1, n_embd);
    a->h = (float*) hq;   // hq = [h F32 k x n_ff | its Q8_K rows]: maya_adapter::hq_bytes(k, n_ff)
    a->hq = maya_adapter::act_view((const char*) hq + sizeof(float) * (size_t) k * n_ff, k, n_ff);
    return true;
}

void moe_gate_up(int gu_type, const MoeDev& d, int k, int n_embd, int n_ff, float limit, const void* xq, void* hq, const void* sh_down,
                 int sh_type, const void* sh_hq, int n_ff_sh, float* sh_out, cudaStream_t s) {
    maya_moe_args a;
    if (!glmf_args(gu_type, gu_type, d, k, n_embd, n_ff, 0, limit, xq, hq, &a)) {
        std::fprintf(stderr, "moe_gate_up: type %d with %d x %d not covered\n", gu_type, n_embd, n_ff);
        maya_adapter::g_launch_errors.fetch_add(1, std::memory_order_relaxed);
        return;
    }
    if (!maya_adapter::ok(maya_moe_gate_up(&a, s), "moe_gate_up")) return;
    if (sh_down && sh_out) {   // the shared expert's down rows over its rounded h (glm_fast.cu:4841-4849): one mat-vec job
        maya_mv_job j{};
        j.w = sh_down;
        j.type = sh_type;
        j.packing = MAYA_PACK_GGUF;
        j.n_in = n_ff_sh;
        j.n_out = n_embd;
        j.ncol = 1;
        j.alpha = 1.0f;
        j.x = maya_adapter::act_view(sh_hq, 1, n_ff_sh);
        j.y = sh_out;
        j.y_stride = n_embd;
        maya_adapter::ok(maya_mv(&j, 1, s), "moe_gate_up (shared down rows)");
    }
}
void moe_down(int d_type, const MoeDev& d, int k, int n_embd, int n_ff, size_t down_off, const void* hq, const float* sh_out, float* out,
              cudaStream_t s) {
    maya_moe_args a;
    // (the gate / up type only sizes the first two row arrays: down_off is given, so any 256-value type serves here)
    if (!glmf_args(d_type, d_type, d, k, n_embd, n_ff, down_off, 0.0f, nullptr, const_cast<void*>(hq), &a)) {
        std::fprintf(stderr, "moe_down: type %d with %d x %d not covered\n", d_type, n_embd, n_ff);
        maya_adapter::g_launch_errors.fetch_add(1, std::memory_order_relaxed);
        return;
    }
    a.add = d.cpu_part;
    a.add_flag = d.cpu_flag;
    a.add2 = sh_out;
    a.out = out;
    if (maya_moe_down_rounds_h(&a)) {
        a.hq = maya_act{nullptr, nullptr, nullptr};
    } else {
        if (!maya_adapter::ok(maya_quant_act(d_type, a.h, MAYA_DT_F32, 0, k, n_ff, a.hq, s), "quant_act(h)")) return;
        maya_adapter::Scratch* sc = maya_adapter::scratch(s);
        if (!sc) return;
        a.part = sc->part;
    }
    maya_adapter::ok(maya_moe_down(&a, s), "moe_down");
}
}  // namespace strata::kernels::glmf

// ================================================================================ EXL3
namespace strata::kernels::exl3 {
int launch_errors() { return maya_adapter::g_launch_errors.load(std::memory_order_relaxed); }
void set_skip(const int* flag) { maya_adapter::g_skip = flag; }
bool k2_supported(int k2, int cb) { return maya_exl3_supported(k2, cb) != 0; }
bool prepare(cudaStream_t s) { return maya_init() == MAYA_OK && maya_adapter::scratch(s) != nullptr; }

static bool exl3_args(const ExpertLayout& lay, int T, int k, int n_embd, int n_ff, float limit, maya_exl3_args* a) {
    *a = maya_exl3_args{};
    if (lay.fmt != 0) return false;   // a GGUF expert layer: strata::ds4::gguf's entry points above
    for (int r = 0; r < 3; ++r) {
        a->layout.suh[r] = lay.suh[r];
        a->layout.svh[r] = lay.svh[r];
        a->layout.trellis[r] = lay.trellis[r];
        a->layout.k2[r] = lay.k2[r];
    }
    a->layout.cb = lay.cb;
    a->layout.n_embd = n_embd;
    a->layout.n_ff = n_ff;
    a->n_tokens = T;
    a->k = k;
    a->skip = maya_adapter::g_skip;
    a->limit = limit;
    return true;
}
void moe_gate_up(const MoeArgs& a, const float* x, float* h, cudaStream_t s) {
    maya_exl3_args m;
    maya_adapter::Scratch* sc = maya_adapter::scratch(s);
    if (!sc || a.mix.n > 0 || !exl3_args(a.lay, 1, a.k, a.n_embd, a.n_ff, a.limit, &m)) return;   // (mixed-K layers: not covered)
    m.plan_ptr = (const uint64_t*) a.plan_ptr;
    m.plan_w = a.plan_w;
    m.x = x;
    m.h = h;
    m.part = sc->part;   // scratch of the split gate / up form
    maya_adapter::ok(maya_exl3_gate_up(&m, s), "exl3::moe_gate_up");
}
void moe_down(const MoeArgs& a, const float* h, const float* sh_out, float* out, cudaStream_t s) {
    maya_exl3_args m;
    maya_adapter::Scratch* sc = maya_adapter::scratch(s);
    if (!sc || a.mix.n > 0 || !exl3_args(a.lay, 1, a.k, a.n_embd, a.n_ff, a.limit, &m)) return;
    m.plan_ptr = (const uint64_t*) a.plan_ptr;
    m.plan_w = a.plan_w;
    m.h = const_cast<float*>(h);
    m.part = sc->part;
    m.add = a.cpu_part;
    m.add_flag = a.cpu_flag;
    m.add2 = sh_out;
    m.out = out;
    maya_adapter::ok(maya_exl3_down(&m, s), "exl3::moe_down");
}
bool win_experts(const WinArgs& a, cudaStream_t s) {
    maya_exl3_args m;
    if (a.mix.n > 0 || !exl3_args(a.lay, a.T, a.k, a.n_embd, a.n_ff, a.limit, &m)) return false;
    if ((a.out_stride != 0 && a.out_stride != (size_t) a.n_embd) || a.wait_ptr) return false;   // (the device-side wait stays the engine's)
    m.plan_ptr = (const uint64_t*) a.plan_ptr;
    m.plan_w = a.plan_w;
    m.grp_ptr = (const uint64_t*) a.grp_ptr;   // glmf::moe_win_group's groups, or maya_moe_group's: the same arrays
    m.grp_start = a.grp_start;
    m.grp_ent = a.grp_ent;
    m.n_groups = a.n_groups;
    m.x = a.x;
    m.x_stride = (int64_t) a.x_stride;
    m.h = a.h;
    m.part = a.part;
    m.add = a.cpu_part;
    m.add_flag = a.cpu_flag;
    m.add2 = a.sh_out;
    m.out = a.out;
    return maya_adapter::ok(maya_exl3_gate_up(&m, s), "exl3::win_experts (gate/up)") &&
           maya_adapter::ok(maya_exl3_down(&m, s), "exl3::win_experts (down)");
}
}  // namespace strata::kernels::exl3

// Every definition above must BE the function the reference's headers declare, not an overload beside it: taking the
// address of a name with two candidates does not compile.
namespace maya_adapter_check {
[[maybe_unused]] auto* c01 = &strata::ds4::gguf::moe_gate_up;
[[maybe_unused]] auto* c02 = &strata::ds4::gguf::moe_down;
[[maybe_unused]] auto* c03 = &strata::ds4::gguf::win_experts;
[[maybe_unused]] auto* c04 = &strata::ds4::gguf::prepare;
[[maybe_unused]] auto* c05 = &strata::ds4::gguf::launch_errors;
[[maybe_unused]] auto* c06 = &strata::ds4::gguf::expert_type_ok;
[[maybe_unused]] auto* c07 = &strata::ds4::iq::supported;
[[maybe_unused]] auto* c08 = &strata::ds4::iq::expert_supported;
[[maybe_unused]] auto* c09 = &strata::ds4::iq::down_supported;
[[maybe_unused]] auto* c10 = &strata::ds4::iq::block_bytes;
[[maybe_unused]] auto* c11 = &strata::kernels::glmf::moe_gate_up;
[[maybe_unused]] auto* c12 = &strata::kernels::glmf::moe_down;
[[maybe_unused]] auto* c13 = &strata::kernels::glmf::moe_supported;
[[maybe_unused]] auto* c14 = &strata::kernels::glmf::set_skip;
[[maybe_unused]] auto* c15 = &strata::kernels::glmf::launch_errors;
[[maybe_unused]] auto* c16 = &strata::kernels::exl3::moe_gate_up;
[[maybe_unused]] auto* c17 = &strata::kernels::exl3::moe_down;
[[maybe_unused]] auto* c18 = &strata::kernels::exl3::win_experts;
[[maybe_unused]] auto* c19 = &strata::kernels::exl3::k2_supported;
[[maybe_unused]] auto* c20 = &strata::kernels::exl3::prepare;
[[maybe_unused]] auto* c21 = &strata::kernels::exl3::set_skip;
[[maybe_unused]] auto* c22 = &strata::kernels::exl3::launch_errors;
}  // namespace maya_adapter_check
