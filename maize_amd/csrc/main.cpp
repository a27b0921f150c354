// C++ twin of the reference's src/main.rs on the AMD launch path.
//
// The reference's test_inner() (src/main.rs:31-90) builds the pipelined BF16 GEMM kernel for
// 4096 x 4096 operands and prints the PTX; it cannot launch it and the kernel has no C operand.
// This program keeps the same steps -- declare the kernel, fix its launch bounds, compile for a
// target, describe A and B as GlobalMatrix -- and then launches on an MI355X, twice: through the
// dispatcher (gemm_smem_multibuffer), through the explicit builder chain, and as a kernel described in the
// reference's tile vocabulary (panels, groups, ring, MMA op) -- once as the reference's caller has it, with the panels and
// the two-stage ring of the 256-row kernels, once with 128-row panels of A on a ring of three stages -- and checks that all
// agree bit for bit.  Output: one JSON line with the kernels chosen and checksums of C.
//
//   maize_gemm_example [M N K]        (default 4096 4096 4096, like src/main.rs:47-48)
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "maize_tile.hpp"

using namespace maize;

int main(int argc, char** argv) {
    uint32_t M = 4096, N = 4096, K = 4096;
    if (argc == 4) { M = (uint32_t)atoi(argv[1]); N = (uint32_t)atoi(argv[2]); K = (uint32_t)atoi(argv[3]); }
    try {
        Ctx ctx(0);
        std::vector<BF16> a((size_t)M * K), b((size_t)K * N);
        maize_fill_uniform_bf16((uint16_t*)a.data(), a.size(), 0x5EED0001ull, 0);
        maize_fill_uniform_bf16((uint16_t*)b.data(), b.size(), 0x5EED0002ull, 0);
        BF16* da = ctx.malloc<BF16>(a.size());
        BF16* db = ctx.malloc<BF16>(b.size());
        BF16* dc = ctx.malloc<BF16>((size_t)M * N);
        BF16* dc2 = ctx.malloc<BF16>((size_t)M * N);
        ctx.upload(da, a);
        ctx.upload(db, b);

        const Matrix amat = Matrix::make(da, M, K);           // Matrix::new(amat, arows, acols), src/main.rs:47
        const Matrix bmat = Matrix::make(db, K, N);           // src/main.rs:48
        const Matrix cmat = Matrix::make(dc, M, N);           // the C operand the reference never had

        // 1. dispatcher path
        gemm_smem_multibuffer(ctx, amat, bmat, cmat);
        ctx.sync();
        const std::string chosen = ctx.select(gemm_desc(amat, bmat, cmat));

        // 2. builder chain, any-shape kernel, hand-packed parameter block (gen.ptx:12-19 prefix + C)
        LoadedKernel k = new_hip_kernel("maize_gemm_bf16_wave32").with_launch_bounds_2d({256, 1}).finalize().compile(Gfx::Gfx950, ctx);
        maize_gemm_args_t args;
        std::memset(&args, 0, sizeof args);
        args.a = da; args.arows = M; args.acols = K;
        args.b = db; args.brows = K; args.bcols = N;
        args.c = dc2; args.crows = M; args.ccols = N;
        args.batch = 1; args.layout = MAIZE_LAYOUT_NN;
        const uint32_t grid[3] = {(N + 63) / 64, (M + 63) / 64, 1};
        k.launch(grid, args);
        ctx.sync();

        // 3. the kernel described in the reference's tile vocabulary, in the order of src/main.rs:32-73
        BF16* dc3 = ctx.malloc<BF16>((size_t)M * N);
        TracedKernel kernel = new_hip_kernel();
        kernel.with_launch_bounds_2d({256, 1});
        auto pipe_shared = kernel.alloc_aligned_shared<TilePair<Tile<BF16_256x64>, Tile<BF16_64x256>>, 2>(1024);
        const BlockX a_panel_group{kernel.cx()};
        const BlockY b_panel_group{kernel.cx()};
        const Wave wave{kernel.cx()};
        const auto a_iter = collective_aligned_row_panel_iter<256>(amat, a_panel_group);     // (bulk panels, ragged epilogue panel)
        const auto b_iter = collective_aligned_col_panel_iter<256>(bmat, b_panel_group);
        a_iter.first.for_every_value([&](const RowPanel<256>& a_panel) {
            b_iter.first.for_every_value([&](const ColPanel<256>& b_panel) {
                Accum ret = gemm_smem_multibuffer(Gfx950MfmaBf16F32_16x16x32{}, KTile<64>{}, a_panel, b_panel, pipe_shared, wave, 16);
                ret.store(Matrix::make(dc3, M, N));                                          // where the reference traps on a zero sum
            });
        });
        LoadedGemm described = kernel.finalize().compile(Gfx::Gfx950, ctx);
        described.launch();
        ctx.sync();

        // 4. the same mainloop with the ring depth and the panel height as parameters ([TilePair; PIPE], gemm/mod.rs:37-45):
        //    128-row panels of A, three ring stages
        BF16* dc4 = ctx.malloc<BF16>((size_t)M * N);
        TracedKernel kernel3 = new_hip_kernel();
        kernel3.with_launch_bounds_2d({256, 1});
        auto ring3 = kernel3.alloc_aligned_shared<TilePair<Tile<BF16_128x64>, Tile<BF16_64x256>>, 3>(1024);
        const BlockX a_group3{kernel3.cx()};
        const BlockY b_group3{kernel3.cx()};
        const Wave wave3{kernel3.cx()};
        const auto a_iter3 = collective_aligned_row_panel_iter<128>(amat, a_group3);
        const auto b_iter3 = collective_aligned_col_panel_iter<256>(bmat, b_group3);
        a_iter3.first.for_every_value([&](const RowPanel<128>& a_panel) {
            b_iter3.first.for_every_value([&](const ColPanel<256>& b_panel) {
                gemm_smem_multibuffer(Gfx950MfmaBf16F32_16x16x32{}, KTile<64>{}, a_panel, b_panel, ring3, wave3, 16).store(Matrix::make(dc4, M, N));
            });
        });
        LoadedGemm described3 = kernel3.finalize().compile(Gfx::Gfx950, ctx);
        described3.launch();
        ctx.sync();

        // 5. ... 128-row panels of A against 128-column panels of B, four ring stages: the 128 x 128 tile kernels (whole K
        //    tiles of 64 only: a description no kernel of the family runs is refused, not replaced)
        BF16* dc5 = ctx.malloc<BF16>((size_t)M * N);
        std::string described5_name = "refused";
        {
            TracedKernel kernel5 = new_hip_kernel();
            kernel5.with_launch_bounds_2d({256, 1});
            auto ring5 = kernel5.alloc_aligned_shared<TilePair<Tile<BF16_128x64>, Tile<BF16_64x128>>, 4>(1024);
            const BlockX a_group5{kernel5.cx()};
            const BlockY b_group5{kernel5.cx()};
            const Wave wave5{kernel5.cx()};
            const auto a_iter5 = collective_aligned_row_panel_iter<128>(amat, a_group5);
            const auto b_iter5 = collective_aligned_col_panel_iter<128>(bmat, b_group5);
            a_iter5.first.for_every_value([&](const RowPanel<128>& a_panel) {
                b_iter5.first.for_every_value([&](const ColPanel<128>& b_panel) {
                    gemm_smem_multibuffer(Gfx950MfmaBf16F32_16x16x32{}, KTile<64>{}, a_panel, b_panel, ring5, wave5, 16).store(Matrix::make(dc5, M, N));
                });
            });
            try {
                LoadedGemm described5 = kernel5.finalize().compile(Gfx::Gfx950, ctx);
                described5.launch();
                ctx.sync();
                described5_name = described5.kernel_name();
            } catch (const std::invalid_argument&) {
            }
        }

        const std::vector<BF16> c1 = ctx.download(dc, (size_t)M * N), c2 = ctx.download(dc2, (size_t)M * N), c3 = ctx.download(dc3, (size_t)M * N),
                                c4 = ctx.download(dc4, (size_t)M * N), c5 = ctx.download(dc5, (size_t)M * N);
        uint64_t sum = 0, x = 0, diff = 0, diff3 = 0, diff4 = 0, diff5 = 0;
        for (size_t i = 0; i < c1.size(); ++i) {
            sum += c1[i].bits;
            x ^= (uint64_t)c1[i].bits << (i % 48);
            diff += c1[i].bits != c2[i].bits;
            diff3 += c1[i].bits != c3[i].bits;
            diff4 += c1[i].bits != c4[i].bits;
            if (described5_name != "refused") diff5 += c1[i].bits != c5[i].bits;
        }
        printf("{\"M\": %u, \"N\": %u, \"K\": %u, \"kernel\": \"%s\", \"described_kernel\": \"%s\", \"described_128_rows_3_stages\": \"%s\", \"ragged_rows\": %u, \"ragged_cols\": %u, "
               "\"sum\": %" PRIu64 ", \"xor\": %" PRIu64 ", \"mismatch_vs_any_shape_kernel\": %" PRIu64 ", \"mismatch_vs_described_kernel\": %" PRIu64
               ", \"mismatch_vs_described_128_rows_3_stages\": %" PRIu64 ", \"described_128_by_128_4_stages\": \"%s\", \"mismatch_vs_described_128_by_128_4_stages\": %" PRIu64 "}\n",
               M, N, K, chosen.c_str(), described.kernel_name().c_str(), described3.kernel_name().c_str(), a_iter.second.extent, b_iter.second.extent, sum, x, diff, diff3, diff4,
               described5_name.c_str(), diff5);
        ctx.free(da); ctx.free(db); ctx.free(dc); ctx.free(dc2); ctx.free(dc3); ctx.free(dc4); ctx.free(dc5);
        return (diff == 0 && diff3 == 0 && diff4 == 0 && diff5 == 0) ? 0 : 3;
    } catch (const Error& e) {
        fprintf(stderr, "maize error: %s\n", e.what());
        return 2;
    }
}
