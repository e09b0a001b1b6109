// The grouped GEMM kernels (csrc/grouped_gemm.hip, the source the library is built from) compiled for the host and run
// under an emulation of a gfx950 workgroup: one coroutine per lane (shim/hip/hip_runtime.h), the matrix instruction,
// the transposing LDS read and the direct global -> LDS copy modelled by their lane layouts.  Both loops of the kernel
// (eight and four wavefronts per tile) run the C entry points on small problems whose sums are exact in fp32, so
// that every output must equal the reference product bit for bit, and
//   * every global address a copy reads is checked against the operand it belongs to (what would fault a GPU),
//   * copies land either at once or as late as the kernel's own waits allow (both legal on the hardware): a read
//     that comes before its wait, or a copy that overwrites a half still being read, gives wrong results in one of the
//     two modes.
// The model of the three instructions is itself checked by the eight-wave loop, whose results on the GPU are pinned
// by the GPU tests: if a lane layout here were wrong, that loop would fail here.
// Output: "ok: N cases"; any mismatch or stray address prints the case and ends with status 1.
#include <hip/hip_runtime.h>

#include <map>
#include <random>
#include <string>
#include <type_traits>

#include "shim/ck_gemm_prims_emulated.h"

#ifndef CK_GEMM_SOURCE  // (another copy of the kernel source can be named on the compiler's command line)
#define CK_GEMM_SOURCE "../../kernel-hyperdrive_amd/csrc/grouped_gemm.hip"
#endif
#include CK_GEMM_SOURCE

// ---- problems -----------------------------------------------------------------------------------------------------------
namespace {
typedef __bf16 bf16;

struct Buffer {  // device memory: every byte outside is outside every operand
    std::vector<char> bytes;
    template <typename T>
    T* as() { return reinterpret_cast<T*>(bytes.data()); }
    size_t size() const { return bytes.size(); }
};
Buffer make(size_t nbytes, const char* name) {
    Buffer b;
    b.bytes.assign(nbytes, 0);
    return b;
}
void expose(std::initializer_list<std::pair<Buffer*, const char*>> buffers) {
    emu::g_regions.clear();
    for (auto& [b, name] : buffers) emu::g_regions.push_back({b->bytes.data(), b->bytes.data() + b->size(), name});
}

// values whose products and sums are exact in fp32: multiples of 1/2 (activations) and of 1/4 (weights), small
template <typename S = bf16>
void fill(Buffer& b, std::mt19937& rng, int scale_quarters) {
    S* v = b.as<S>();
    for (size_t i = 0; i < b.size() / 2; ++i) v[i] = (S)(((int)(rng() % 9) - 4) * 0.25f * scale_quarters);
}
float f(bf16 v) { return (float)v; }
float f(_Float16 v) { return (float)v; }

struct Routing {
    std::vector<int64_t> sorted_scattered, offsets;
    int T, k, E, slots;
};
Routing route(std::mt19937& rng, int T, int k, int E, int empty_expert) {
    Routing r{{}, {}, T, k, E, T * k};
    std::vector<std::pair<int, int>> chosen;  // (expert, position t * k + j)
    for (int t = 0; t < T; ++t) {
        std::vector<int> experts;
        while ((int)experts.size() < k) {
            const int e = (int)(rng() % E);
            if (e != empty_expert && std::find(experts.begin(), experts.end(), e) == experts.end()) experts.push_back(e);
        }
        for (int j = 0; j < k; ++j) chosen.push_back({experts[j], t * k + j});
    }
    std::stable_sort(chosen.begin(), chosen.end(), [](auto& a, auto& b) { return a.first < b.first; });
    r.offsets.assign(E, 0);
    for (auto& c : chosen) {
        r.sorted_scattered.push_back(c.second);
        for (int e = c.first; e < E; ++e) ++r.offsets[e];
    }
    return r;
}
int expert_of(const Routing& r, int slot) {
    int e = 0;
    while (r.offsets[e] <= slot) ++e;
    return e;
}

int g_cases = 0;

// out[out_row(i)] = X[in_row(i)] @ W[e(i)], W as the view [E, K, N] of [E, N, K] (k contiguous) or [E, K, N] (n contiguous)
template <typename S = bf16>
void scatter2scatter_case(std::mt19937& rng, int T, int k, int E, int K, int N, bool w_k_contiguous, bool x_grouped, bool y_grouped,
                          bool split, int waves, bool late, int empty_expert, bool with_bias = false) {
    const int dtype = sizeof(S) == 2 && std::is_same<S, bf16>::value ? CK_BF16 : CK_F16;
    char text[200];
    std::snprintf(text, sizeof text, "scatter2scatter %s T=%d k=%d E=%d K=%d N=%d %s %s%s%s%s waves=%d copies %s",
                  dtype == CK_BF16 ? "bf16" : "fp16", T, k, E, K, N, w_k_contiguous ? "NT" : "NN", x_grouped ? "grouped-in " : "gather-in ",
                  y_grouped ? "grouped-out" : "scatter-out", split ? " split-tail" : "", with_bias ? " bias" : "", waves,
                  late ? "late" : "at once");
    emu::g_case = text;
    emu::g_late_copies = late;
    const Routing r = route(rng, T, k, E, empty_expert);
    const int fan_out = x_grouped ? 1 : k;
    const int x_rows = x_grouped ? r.slots : T;
    Buffer X = make((size_t)x_rows * K * 2, "X"), W = make((size_t)E * K * N * 2, "W"), out = make((size_t)r.slots * N * 2, "out");
    fill<S>(X, rng, 2);
    fill<S>(W, rng, 1);
    Buffer bias = make((size_t)E * N * 2, "bias");
    fill<S>(bias, rng, 3);
    for (size_t i = 0; i < out.size() / 2; ++i) out.as<S>()[i] = (S)-777.f;
    Buffer idx = make(r.slots * 8, "idx"), off = make(E * 8, "offsets");
    std::memcpy(idx.bytes.data(), r.sorted_scattered.data(), r.slots * 8);
    std::memcpy(off.bytes.data(), r.offsets.data(), E * 8);
    const int64_t ws_bytes = split ? ck_scatter2scatter_workspace_size(r.slots, K, N, E, dtype) : 0;
    if (split && ws_bytes == 0) emu::die("the case is meant to have a tail to split");
    Buffer ws = make((size_t)std::max<int64_t>(ws_bytes, 16), "workspace");
    expose({{&X, "X"}, {&W, "W"}});
    const int64_t se = (int64_t)K * N, sk = w_k_contiguous ? 1 : N, sn = w_k_contiguous ? K : 1;
    const int status = ck_scatter2scatter_ws(X.as<void>(), K, W.as<void>(), se, sk, sn, idx.as<int64_t>(), off.as<int64_t>(),
                                             out.as<void>(), N, r.slots, K, N, E, fan_out, x_grouped, y_grouped,
                                             with_bias ? bias.as<void>() : nullptr, dtype, waves, split ? ws.as<void>() : nullptr,
                                             ws_bytes, nullptr);
    if (status != CK_OK) emu::die("status " + std::to_string(status));
    const S *x = X.as<S>(), *w = W.as<S>(), *o = out.as<S>(), *bv = bias.as<S>();
    for (int i = 0; i < r.slots; ++i) {
        const int e = expert_of(r, i);
        const int64_t in_row = x_grouped ? i : r.sorted_scattered[i] / fan_out, out_row = y_grouped ? i : r.sorted_scattered[i];
        for (int n = 0; n < N; ++n) {
            float sum = with_bias ? f(bv[(int64_t)e * N + n]) : 0.f;  // the bias joins the fp32 sum before its one rounding
            for (int kk = 0; kk < K; ++kk) sum += f(x[in_row * K + kk]) * f(w[e * se + kk * sk + n * sn]);
            const S expected = (S)sum;
            if (std::memcmp(&expected, &o[out_row * N + n], 2) != 0) {
                std::snprintf(text, sizeof text, "slot %d (expert %d) column %d: %g, expected %g", i, e, n, f(o[out_row * N + n]), f(expected));
                emu::die(text);
            }
        }
    }
    ++g_cases;
}

// DW[e] = X_e^T DY_e, DW as the view [E, K, N] of [E, N, K] (the parameter's layout) or plain [E, K, N]
void group_bwd_w_case(std::mt19937& rng, int T, int k, int E, int K, int N, bool k_contiguous, int waves, bool late, int empty_expert) {
    char text[200];
    std::snprintf(text, sizeof text, "group_bwd_W T=%d k=%d E=%d K=%d N=%d %s waves=%d copies %s", T, k, E, K, N,
                  k_contiguous ? "k-contiguous" : "n-contiguous", waves, late ? "late" : "at once");
    emu::g_case = text;
    emu::g_late_copies = late;
    const Routing r = route(rng, T, k, E, empty_expert);
    Buffer X = make((size_t)r.slots * K * 2, "X"), DY = make((size_t)r.slots * N * 2, "DY"), DW = make((size_t)E * K * N * 2, "DW");
    fill(X, rng, 2);
    fill(DY, rng, 1);
    for (size_t i = 0; i < DW.size() / 2; ++i) DW.as<bf16>()[i] = (bf16)-777.f;
    Buffer off = make(E * 8, "offsets");
    std::memcpy(off.bytes.data(), r.offsets.data(), E * 8);
    expose({{&X, "X"}, {&DY, "DY"}});
    const int64_t se = (int64_t)K * N, sk = k_contiguous ? 1 : N, sn = k_contiguous ? K : 1;
    const int status = ck_group_bwd_W(DY.as<void>(), N, X.as<void>(), K, off.as<int64_t>(), DW.as<void>(), se, sk, sn, r.slots, K, N, E,
                                      CK_BF16, waves, nullptr);
    if (status != CK_OK) emu::die("status " + std::to_string(status));
    const bf16 *x = X.as<bf16>(), *dy = DY.as<bf16>(), *dw = DW.as<bf16>();
    for (int e = 0; e < E; ++e) {
        const int begin = e == 0 ? 0 : (int)r.offsets[e - 1], end = (int)r.offsets[e];
        for (int kk = 0; kk < K; ++kk)
            for (int n = 0; n < N; ++n) {
                float sum = 0.f;
                for (int m = begin; m < end; ++m) sum += f(x[(int64_t)m * K + kk]) * f(dy[(int64_t)m * N + n]);
                const bf16 expected = (bf16)sum;
                if (std::memcmp(&expected, &dw[e * se + kk * sk + n * sn], 2) != 0) {
                    std::snprintf(text, sizeof text, "expert %d (%d rows) k %d n %d: %g, expected %g", e, end - begin, kk, n,
                                  f(dw[e * se + kk * sk + n * sn]), f(expected));
                    emu::die(text);
                }
            }
    }
    ++g_cases;
}

bool within_ulps(bf16 got, float expected, int ulps) {
    const float e = f((bf16)expected);
    const float step = std::ldexp(1.0f, std::max(std::ilogb(std::max(std::fabs(e), 1e-30f)), -126) - 7);
    return std::fabs(f(got) - e) <= ulps * step;
}

// h = X[gathered] @ W_fc[e] (exact), act = up * silu(gate) from the rounded h; then, with h given, d_h from DY @ W_proj[e]
void glu_case(std::mt19937& rng, int T, int k, int E, int K, int I, int waves, bool late) {
    char text[200];
    std::snprintf(text, sizeof text, "scatter2scatter + SwiGLU T=%d k=%d E=%d K=%d I=%d waves=%d copies %s", T, k, E, K, I, waves,
                  late ? "late" : "at once");
    emu::g_case = text;
    emu::g_late_copies = late;
    const Routing r = route(rng, T, k, E, -1);
    Buffer X = make((size_t)T * K * 2, "X"), W = make((size_t)E * 2 * I * K * 2, "W_fc"), h = make((size_t)r.slots * 2 * I * 2, "h"),
           act = make((size_t)r.slots * I * 2, "act");
    fill(X, rng, 2);
    fill(W, rng, 1);
    Buffer idx = make(r.slots * 8, "idx"), off = make(E * 8, "offsets");
    std::memcpy(idx.bytes.data(), r.sorted_scattered.data(), r.slots * 8);
    std::memcpy(off.bytes.data(), r.offsets.data(), E * 8);
    expose({{&X, "X"}, {&W, "W_fc"}});
    // W_fc is [E, 2I, K]; the kernel takes the view [E, K, 2I]
    int status = ck_scatter2scatter_glu(X.as<void>(), K, W.as<void>(), (int64_t)2 * I * K, 1, K, idx.as<int64_t>(), off.as<int64_t>(),
                                        h.as<void>(), 2 * I, act.as<void>(), I, r.slots, K, I, E, k, 0, CK_BF16, waves, nullptr);
    if (status != CK_OK) emu::die("status " + std::to_string(status));
    const bf16 *x = X.as<bf16>(), *w = W.as<bf16>(), *hh = h.as<bf16>(), *a = act.as<bf16>();
    for (int i = 0; i < r.slots; ++i) {
        const int e = expert_of(r, i);
        const int64_t in_row = r.sorted_scattered[i] / k;
        for (int n = 0; n < 2 * I; ++n) {
            float sum = 0.f;
            for (int kk = 0; kk < K; ++kk) sum += f(x[in_row * K + kk]) * f(w[((int64_t)e * 2 * I + n) * K + kk]);
            const bf16 expected = (bf16)sum;
            if (std::memcmp(&expected, &hh[(int64_t)i * 2 * I + n], 2) != 0) emu::die("h differs at slot " + std::to_string(i) + " column " + std::to_string(n));
        }
        for (int c = 0; c < I; ++c) {
            const float u = f(hh[(int64_t)i * 2 * I + c]), g = f(hh[(int64_t)i * 2 * I + I + c]);
            if (!within_ulps(a[(int64_t)i * I + c], u * g * (1.0f / (1.0f + std::exp(-g))), 1)) emu::die("act differs at slot " + std::to_string(i) + " column " + std::to_string(c));
        }
    }
    // backward: DY [slots, H] grouped, W_proj [E, H, I] read as [E, K = H, N = I]
    const int H = K;
    Buffer DY = make((size_t)r.slots * H * 2, "DY"), Wp = make((size_t)E * H * I * 2, "W_proj"), dh = make((size_t)r.slots * 2 * I * 2, "d_h");
    fill(DY, rng, 1);
    fill(Wp, rng, 1);
    expose({{&DY, "DY"}, {&Wp, "W_proj"}});
    status = ck_scatter2scatter_glu_bwd(DY.as<void>(), H, Wp.as<void>(), (int64_t)H * I, I, 1, off.as<int64_t>(), h.as<void>(), 2 * I,
                                        dh.as<void>(), 2 * I, r.slots, H, I, E, CK_BF16, waves, nullptr);
    if (status != CK_OK) emu::die("status " + std::to_string(status));
    const bf16 *dy = DY.as<bf16>(), *wp = Wp.as<bf16>(), *d = dh.as<bf16>();
    for (int i = 0; i < r.slots; ++i) {
        const int e = expert_of(r, i);
        for (int c = 0; c < I; ++c) {
            float sum = 0.f;
            for (int kk = 0; kk < H; ++kk) sum += f(dy[(int64_t)i * H + kk]) * f(wp[((int64_t)e * H + kk) * I + c]);
            const float d_act = f((bf16)sum), u = f(hh[(int64_t)i * 2 * I + c]), g = f(hh[(int64_t)i * 2 * I + I + c]);
            const float sg = 1.0f / (1.0f + std::exp(-g)), gs = g * sg;
            if (!within_ulps(d[(int64_t)i * 2 * I + c], d_act * gs, 1) || !within_ulps(d[(int64_t)i * 2 * I + I + c], d_act * u * (sg + gs * (1.0f - sg)), 1))
                emu::die("d_h differs at slot " + std::to_string(i) + " column " + std::to_string(c));
        }
    }
    ++g_cases;
}
}  // namespace

int main(int argc, char** argv) {
    // arguments: "8" or "4" (one loop only), "--lax-waits" (every wait on the copies eight short: the results must differ),
    // "--random N [--seed S]" (N random cases per loop instead of the fixed list)
    std::string only;
    int random_cases = 0;
    unsigned random_seed = 1;
    for (int i = 1; i < argc; ++i) {
        if (std::string(argv[i]) == "--lax-waits") emu::g_lax_waits = 8;
        else if (std::string(argv[i]) == "--random" && i + 1 < argc) random_cases = std::atoi(argv[++i]);
        else if (std::string(argv[i]) == "--seed" && i + 1 < argc) random_seed = (unsigned)std::atoi(argv[++i]);
        else only = argv[i];
    }
    emu::g_after_block = [] {
        for (int l = 0; l < emu::g_threads; ++l)
            if (!emu::g_pending[l].empty()) {
                if (emu::g_lax_waits) emu::g_pending[l].clear();
                else emu::die("a workgroup ended with copies still under way");
            }
    };
    std::mt19937 rng(2024);
    if (random_cases > 0) {
        // "--random N": N cases of random shape, layout, routing and copy timing per loop (for a longer soak than the fixed list)
        rng.seed(random_seed);
        for (int c = 0; c < random_cases; ++c) {
            const int E = 1 + (int)(rng() % 5), k = 1 + (int)(rng() % std::min(E, 3)), T = 1 + (int)(rng() % 400);
            const int K = 8 * (1 + (int)(rng() % 80)), N = 8 * (1 + (int)(rng() % 70));
            const bool late = rng() % 2, kc = rng() % 2, xg = rng() % 2, yg = rng() % 2;
            const int empty = E > k && rng() % 3 == 0 ? (int)(rng() % E) : -1;
            for (int waves : {8, 4}) {
                if (!only.empty() && only != std::to_string(waves)) continue;
                if (rng() % 2)
                    scatter2scatter_case(rng, T, k, E, K, N, kc, xg, yg, false, waves, late, empty);
                else
                    group_bwd_w_case(rng, T, k, E, K, N, kc, waves, late, empty);
            }
        }
        std::printf("ok: %d random cases\n", g_cases);
        return 0;
    }
    for (int waves : {8, 4}) {
        if (!only.empty() && only != std::to_string(waves)) continue;
        // Copies that land as late as the kernel's waits allow: contractions of 2, 3 (odd: the last tile outside the
        // pipeline) and 5 tiles plus a partial one; row tiles with an empty upper half; a column tile with an empty upper
        // half; an expert without rows; the tail split along the contraction; both weight-gradient layouts; the fused
        // SwiGLU epilogues.
        scatter2scatter_case(rng, 150, 2, 3, 128, 256, true, false, true, false, waves, true, -1);
        scatter2scatter_case(rng, 40, 1, 2, 192, 136, false, true, false, false, waves, true, -1);
        scatter2scatter_case(rng, 70, 2, 4, 320 + 24, 264, true, true, true, false, waves, true, 2);
        scatter2scatter_case(rng, 30, 1, 2, 4096, 128, false, true, true, true, waves, true, -1);
        scatter2scatter_case(rng, 30, 1, 2, 4096 + 64, 72, true, false, false, true, waves, true, -1);
        group_bwd_w_case(rng, 200, 1, 2, 256, 256, true, waves, true, -1);
        group_bwd_w_case(rng, 90, 2, 3, 136, 264, false, waves, true, 1);
        glu_case(rng, 40, 2, 2, 192, 128, waves, true);
        if (emu::g_lax_waits) continue;
        // fp16 storage; a per-expert bias, whole tiles and split tail (a product with a bias takes the eight-wave loop
        // whichever is asked for)
        scatter2scatter_case<_Float16>(rng, 70, 2, 3, 192 + 8, 264, true, false, false, false, waves, true, -1);
        scatter2scatter_case(rng, 70, 2, 3, 256, 136, true, false, true, false, waves, true, 1, true);
        scatter2scatter_case(rng, 30, 1, 2, 4096, 128, false, true, true, true, waves, true, -1, true);
        // Copies that land at once (a copy that overwrites a half too early would show here)
        scatter2scatter_case(rng, 150, 2, 3, 320, 256, true, false, true, false, waves, false, -1);
        scatter2scatter_case(rng, 40, 1, 2, 192, 136, false, true, false, false, waves, false, -1);
        group_bwd_w_case(rng, 300, 1, 2, 136, 264, true, waves, false, -1);
        glu_case(rng, 40, 2, 2, 256, 128, waves, false);
    }
    std::printf("ok: %d cases, %lld lane switches\n", g_cases, emu::g_switches);
    return 0;
}
