// A caller that cannot allocate: a chain of products through maize_hip_gemm_bf16_noalloc, captured once into a HIP
// graph on the caller's own stream and replayed with new inputs.  Every product in the chain passes partial tiles
// and ticket counters through the library's fixed per-GPU scratch array; every replay must reproduce, bit for bit,
// what the same calls give when launched eagerly on the same inputs -- the kernels return their counters to zero
// themselves, and nothing on the path allocates, synchronises or records a memset node.  (The reference has no
// counterpart: its main() only prints PTX, src/main.rs:75-89.)  Prints one JSON line; exit code 0 when all replays
// match.
//
//   maize_graph_replay [rounds]       (default 6)
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "maize_hip.h"

#define HIP_OK(call) do { hipError_t e_ = (call); if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_)); return 2; } } while (0)
#define MZ_OK(call) do { int32_t r_ = (call); if (r_ != MAIZE_OK) { fprintf(stderr, "%s: %s\n", #call, maize_hip_last_error()); return 2; } } while (0)

struct Product {
    uint32_t m, n, k, layout;
    uint16_t *a, *b, *c;
    maize_gemm_desc_t desc;
    std::string kernel;
};

int main(int argc, char** argv) {
    const int rounds = argc > 1 ? atoi(argv[1]) : 6;
    maize_ctx_t* ctx = nullptr;
    MZ_OK(maize_hip_ctx_create(0, &ctx));
    // a few-row product in K ranges, the same against N x K weights, 64 rows in four row groups (the slab's workgroups
    // share the additions), 128-row tiles cut over K with the reduce pass behind them, a ragged product (24 columns past the last whole tile column) whose edge tiles
    // are split, and a plain one that needs no scratch
    std::vector<Product> ps = {{16, 14336, 4096, MAIZE_LAYOUT_NN, nullptr, nullptr, nullptr, {}, ""}, {16, 4096, 4096, MAIZE_LAYOUT_NT, nullptr, nullptr, nullptr, {}, ""},
                               {64, 14336, 4096, MAIZE_LAYOUT_NN, nullptr, nullptr, nullptr, {}, ""}, {100, 2048, 4096, MAIZE_LAYOUT_NN, nullptr, nullptr, nullptr, {}, ""},
                               {4000, 4120, 512, MAIZE_LAYOUT_NN, nullptr, nullptr, nullptr, {}, ""}, {512, 512, 512, MAIZE_LAYOUT_NN, nullptr, nullptr, nullptr, {}, ""}};
    int with_scratch = 0;
    for (Product& p : ps) {
        MZ_OK(maize_hip_malloc(ctx, (size_t)p.m * p.k * 2, (void**)&p.a));
        MZ_OK(maize_hip_malloc(ctx, (size_t)p.k * p.n * 2, (void**)&p.b));
        MZ_OK(maize_hip_malloc(ctx, (size_t)p.m * p.n * 2, (void**)&p.c));
        std::memset(&p.desc, 0, sizeof p.desc);
        p.desc.a = {p.a, p.m, p.k};
        p.desc.b = p.layout == MAIZE_LAYOUT_NN ? maize_matrix_t{p.b, p.k, p.n} : maize_matrix_t{p.b, p.n, p.k};
        p.desc.c = {p.c, p.m, p.n};
        p.desc.layout = p.layout;
        p.desc.batch = 1;
        maize_gemm_plan_t plan;
        MZ_OK(maize_hip_gemm_plan(&p.desc, nullptr, 256, &plan));
        char name[96];
        MZ_OK(maize_hip_gemm_select(ctx, &p.desc, name, sizeof name));
        p.kernel = name;
        with_scratch += plan.workspace_bytes > 0;
        if (plan.workspace_bytes > MAIZE_NOALLOC_MAX_WORKSPACE_BYTES) { fprintf(stderr, "%s needs too much scratch\n", name); return 2; }
    }
    auto fill = [&](uint64_t seed) -> int {
        for (size_t i = 0; i < ps.size(); ++i) {
            Product& p = ps[i];
            std::vector<uint16_t> a((size_t)p.m * p.k), b((size_t)p.k * p.n);
            maize_fill_uniform_bf16(a.data(), a.size(), seed * 1000 + 2 * i, 0);
            maize_fill_uniform_bf16(b.data(), b.size(), seed * 1000 + 2 * i + 1, 0);
            MZ_OK(maize_hip_memcpy_h2d(ctx, p.a, a.data(), a.size() * 2));
            MZ_OK(maize_hip_memcpy_h2d(ctx, p.b, b.data(), b.size() * 2));
            std::vector<uint16_t> nan((size_t)p.m * p.n, 0x7FC0);                    // C starts as NaN: every element must be written
            MZ_OK(maize_hip_memcpy_h2d(ctx, p.c, nan.data(), nan.size() * 2));
        }
        return 0;
    };
    auto launch_all = [&](hipStream_t s) -> int {
        for (Product& p : ps) MZ_OK(maize_hip_gemm_bf16_noalloc(ctx, &p.desc, (void*)s));
        return 0;
    };
    auto download = [&](std::vector<std::vector<uint16_t>>& out) -> int {
        out.resize(ps.size());
        for (size_t i = 0; i < ps.size(); ++i) {
            out[i].resize((size_t)ps[i].m * ps[i].n);
            MZ_OK(maize_hip_memcpy_d2h(ctx, out[i].data(), ps[i].c, out[i].size() * 2));
        }
        return 0;
    };
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));                                               // default priority
    // eager results for three sets of inputs
    std::vector<std::vector<std::vector<uint16_t>>> want(4);
    for (uint64_t seed = 1; seed <= 3; ++seed) {
        if (fill(seed)) return 2;
        if (launch_all(stream)) return 2;
        HIP_OK(hipStreamSynchronize(stream));
        if (download(want[seed])) return 2;
    }
    // capture the chain once
    hipGraph_t graph;
    hipGraphExec_t exec;
    HIP_OK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
    if (launch_all(stream)) return 2;
    HIP_OK(hipStreamEndCapture(stream, &graph));
    size_t nodes = 0;
    HIP_OK(hipGraphGetNodes(graph, nullptr, &nodes));
    HIP_OK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    // replay with new inputs, eager work of the same kind in between
    uint64_t mismatches = 0;
    const uint64_t order[6] = {1, 2, 3, 2, 1, 3};
    for (int r = 0; r < rounds; ++r) {
        const uint64_t seed = order[r % 6];
        if (fill(seed)) return 2;
        HIP_OK(hipGraphLaunch(exec, stream));
        HIP_OK(hipStreamSynchronize(stream));
        std::vector<std::vector<uint16_t>> got;
        if (download(got)) return 2;
        for (size_t i = 0; i < ps.size(); ++i)
            for (size_t e = 0; e < got[i].size(); ++e) mismatches += got[i][e] != want[seed][i][e];
        if (r == 2) {                                                                // shares the scratch array with the graph's kernels
            if (launch_all(stream)) return 2;
            HIP_OK(hipStreamSynchronize(stream));
        }
    }
    // what capture buys a launch-bound chain
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    float ms_graph = 0, ms_eager = 0;
    const int reps = 50;
    HIP_OK(hipGraphLaunch(exec, stream));
    HIP_OK(hipEventRecord(e0, stream));
    for (int i = 0; i < reps; ++i) HIP_OK(hipGraphLaunch(exec, stream));
    HIP_OK(hipEventRecord(e1, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipEventElapsedTime(&ms_graph, e0, e1));
    if (launch_all(stream)) return 2;
    HIP_OK(hipEventRecord(e0, stream));
    for (int i = 0; i < reps; ++i) if (launch_all(stream)) return 2;
    HIP_OK(hipEventRecord(e1, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipEventElapsedTime(&ms_eager, e0, e1));
    std::string names;
    for (const Product& p : ps) names += (names.empty() ? "\"" : ", \"") + p.kernel + "\"";
    printf("{\"products\": %zu, \"with_scratch\": %d, \"graph_nodes\": %zu, \"rounds\": %d, \"mismatches\": %llu, \"us_per_chain_graph\": %.1f, "
           "\"us_per_chain_eager\": %.1f, \"kernels\": [%s]}\n",
           ps.size(), with_scratch, nodes, rounds, (unsigned long long)mismatches, ms_graph / reps * 1e3, ms_eager / reps * 1e3, names.c_str());
    HIP_OK(hipGraphExecDestroy(exec));
    HIP_OK(hipGraphDestroy(graph));
    HIP_OK(hipStreamDestroy(stream));
    for (Product& p : ps) { maize_hip_free(ctx, p.a); maize_hip_free(ctx, p.b); maize_hip_free(ctx, p.c); }
    maize_hip_ctx_destroy(ctx);
    return mismatches == 0 ? 0 : 3;
}
