// maize_tile.hpp -- header-only C++ mirror of the reference's host-side surface for the BF16
// GEMM path, on top of the C ABI in maize_hip.h.
//
// The reference is a Rust workspace; this image carries no Rust toolchain, so the host side
// above the C ABI is written in C++ with the reference's names and argument meaning:
//
//   GlobalMatrix<T>                       src/main.rs:20-27 (struct_reflect!, #[repr(align(16))])
//   Matrix::new(ptr, nrows, ncols)        crates/maize_tile/src/gmem/matrix.rs:6-19
//   KTile<N>                              crates/maize_tile/src/gemm/mod.rs:35
//   new_hip_kernel(name)                  new_ptx_kernel, crates/maize_core/src/codegen/mod.rs:50
//     .with_launch_bounds_2d({x, y})      crates/maize_core/src/codegen/calling_convention.rs:66-78
//     .finalize().compile(Gfx::Gfx950)    crates/maize_core/src/codegen/typed_func.rs:740-826, SM enum target_cpu/cuda.rs:3-53
//   gemm_smem_multibuffer(ctx, a, b, c)   sm80_gemm_smem_multibuffer, crates/maize_tile/src/gemm/mod.rs:37-90
//
// Where the reference panics at trace time (typed_func.rs:200,668; gmem_tile.rs:59-62), this
// mirror throws maize::Error carrying the C ABI's status code and message.
#pragma once
#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "maize_hip.h"

namespace maize {

struct Error : std::runtime_error {
    int32_t code;
    Error(int32_t c, const std::string& m) : std::runtime_error("[" + std::to_string(c) + "] " + m), code(c) {}
};
inline void check(int32_t rc) {
    if (rc != MAIZE_OK) throw Error(rc, maize_hip_last_error());
}

struct BF16 {  // 2-byte, u16-backed (crates/maize_core/src/ty/sized.rs:62-68)
    uint16_t bits;
    static BF16 from_f32(float x) { return BF16{maize_bf16_from_f32(x)}; }
    float to_f32() const { return maize_bf16_to_f32(bits); }
};
static_assert(sizeof(BF16) == 2, "BF16 is two bytes");

// The kernel-side descriptor and its host twin are the same 16 bytes.
template <class T>
struct alignas(16) GlobalMatrix {
    T* ptr;
    uint32_t nrows;
    uint32_t ncols;
    maize_matrix_t realize() const { maize_matrix_t m; m.ptr = (void*)ptr; m.nrows = nrows; m.ncols = ncols; return m; }
};
static_assert(sizeof(GlobalMatrix<BF16>) == 16 && alignof(GlobalMatrix<BF16>) == 16, "GlobalMatrix layout");

enum class Gfx { Gfx950 };                 // compile targets: this library carries one
enum class Layout : uint32_t { NN = MAIZE_LAYOUT_NN, NT = MAIZE_LAYOUT_NT };
template <uint32_t K_TILE> struct KTile { static constexpr uint32_t value = K_TILE; };

class Ctx {
  public:
    explicit Ctx(int32_t device = 0) { check(maize_hip_ctx_create(device, &h_)); }
    ~Ctx() { if (h_) maize_hip_ctx_destroy(h_); }
    Ctx(const Ctx&) = delete;
    Ctx& operator=(const Ctx&) = delete;
    maize_ctx_t* handle() const { return h_; }

    template <class T> T* malloc(size_t count) { void* p = nullptr; check(maize_hip_malloc(h_, count * sizeof(T), &p)); return (T*)p; }
    void free(void* p) { check(maize_hip_free(h_, p)); }
    template <class T> void upload(T* dst, const std::vector<T>& src) { check(maize_hip_memcpy_h2d(h_, dst, src.data(), src.size() * sizeof(T))); }
    template <class T> std::vector<T> download(const T* src, size_t count) {
        std::vector<T> out(count);
        check(maize_hip_memcpy_d2h(h_, out.data(), src, count * sizeof(T)));
        return out;
    }
    void sync(void* stream = nullptr) { check(maize_hip_sync(h_, stream)); }
    std::string select(const maize_gemm_desc_t& d) { char buf[128]; check(maize_hip_gemm_select(h_, &d, buf, sizeof buf)); return buf; }

  private:
    maize_ctx_t* h_ = nullptr;
};

// A device matrix view: row-major, leading dimension == ncols.
struct Matrix {
    GlobalMatrix<BF16> g;
    static Matrix make(BF16* ptr, uint32_t nrows, uint32_t ncols) { return Matrix{GlobalMatrix<BF16>{ptr, nrows, ncols}}; }
};

inline maize_gemm_desc_t gemm_desc(const Matrix& a, const Matrix& b, const Matrix& c, Layout layout = Layout::NN,
                                   uint32_t batch = 1, uint64_t stride_a = 0, uint64_t stride_b = 0, uint64_t stride_c = 0) {
    maize_gemm_desc_t d;
    std::memset(&d, 0, sizeof d);
    d.a = a.g.realize(); d.b = b.g.realize(); d.c = c.g.realize();
    d.layout = (uint32_t)layout; d.batch = batch;
    d.stride_a = stride_a; d.stride_b = stride_b; d.stride_c = stride_c;
    return d;
}

// C = A.B through the dispatcher: the reference's mainloop entry, carried through to a launch.
// The extended descriptor: leading dimensions (0 = ncols), element type of C, C = alpha * A.B + beta * C.
inline maize_gemm_ex_desc_t gemm_ex_desc(const maize_gemm_desc_t& d, uint32_t lda = 0, uint32_t ldb = 0, uint32_t ldc = 0,
                                         maize_out_type_t out = MAIZE_OUT_BF16, float alpha = 1.0f, float beta = 0.0f,
                                         maize_in_type_t in = MAIZE_IN_BF16) {
    maize_gemm_ex_desc_t x{};
    x.gemm = d;
    x.lda = lda; x.ldb = ldb; x.ldc = ldc;
    x.out_type = out;
    x.alpha = alpha; x.beta = beta;
    x.in_type = in;            // half, the 8-bit E4M3 / E5M2 (one byte per element), fp32 or fp64; the Matrix views then wrap pointers to elements of that size
    return x;
}

// Kernel choice and launch geometry for a descriptor; needs no device.
inline maize_gemm_plan_t gemm_plan(const maize_gemm_desc_t& d, uint32_t compute_units = 256, const char* kernel = nullptr) {
    maize_gemm_plan_t p;
    check(maize_hip_gemm_plan(&d, kernel, compute_units, &p));
    return p;
}

inline void gemm_smem_multibuffer(Ctx& ctx, const Matrix& a, const Matrix& b, const Matrix& c, Layout layout = Layout::NN,
                                  void* stream = nullptr) {
    const maize_gemm_desc_t d = gemm_desc(a, b, c, layout);
    check(maize_hip_gemm_bf16(ctx.handle(), &d, stream));
}

inline void gemm_smem_multibuffer(Ctx& ctx, const maize_gemm_ex_desc_t& x, void* stream = nullptr, const char* kernel = nullptr) {
    check(maize_hip_gemm_bf16_ex(ctx.handle(), &x, kernel, stream));
}

// ---- the tile vocabulary ---------------------------------------------------------------------------
// The reference's caller *traces* its kernel (src/main.rs:31-90): shared-memory ring, Matrix, row / column panels over
// groups of blocks, sm80_gemm_smem_multibuffer per panel pair.  Here the kernels are hand-written, so the same calls
// *describe* one: small host-side types with the reference's names, checked against what the kernels implement --
// at compile time where the reference's trait bounds would refuse (tile types, K tile, ring depth), by exceptions
// where it panics at trace time -- and resolved by finalize().compile() to the launch maize_hip_gemm_bf16_ex makes.
//
//   Tile<T>, TilePair<TA, TB>, tile types    crates/maize_tile/src/lib.rs:87-108,231-265, pair.rs:3-8
//   RowPanel / ColPanel / PanelIterLooper    crates/maize_tile/src/gmem/row_panel.rs:10-161, col_panel.rs:10-158
//   BlockX / BlockY / Wave (was Warp)        crates/maize_tile/src/group/by_block.rs:10-75, warp.rs:10-37
//   SyncMMAOp catalogue                      crates/maize_tile/src/mma/mod.rs:19-99, sm80.rs, sm80_derived.rs:5-28, sm89.rs
//   gemm_smem_multibuffer(mma, KTile, ...)   crates/maize_tile/src/gemm/mod.rs:37-90
enum class Swizzle { None, KC16, KN32, KN16 };   // KC16: 128-byte rows along K, 16-byte chunk ^ ((row >> 1) & 7); KN32: row-major K x N, 32-byte granule ^ (row % 4 + 4 bit3(row)); KN16: row-major K x N of 8-bit elements, 16-byte chunk ^ (row % 8 + 8 bit4(row))
#define MAIZE_TILE_TY(name, rows, cols, bytes, swz) \
    struct name { static constexpr uint32_t ROWS = rows, COLS = cols, ELEM_BYTES = bytes; static constexpr Swizzle SWIZZLE = swz; };
MAIZE_TILE_TY(BF16_16x16, 16, 16, 2, Swizzle::None)      // the reference's tile (lib.rs:98-108); no kernel here takes it
MAIZE_TILE_TY(BF16_256x64, 256, 64, 2, Swizzle::KC16)    // A stage; B stage when B is stored N x K
MAIZE_TILE_TY(BF16_64x256, 64, 256, 2, Swizzle::KN32)    // B stage of a row-major K x N B
MAIZE_TILE_TY(F16_256x64, 256, 64, 2, Swizzle::KC16)
MAIZE_TILE_TY(F16_64x256, 64, 256, 2, Swizzle::KN32)
MAIZE_TILE_TY(F8_256x128, 256, 128, 1, Swizzle::KC16)    // 8-bit operands: 128 elements of K per 128-byte row
MAIZE_TILE_TY(F8_128x256, 128, 256, 1, Swizzle::KN16)    // B stage of a row-major K x N 8-bit B (read back by ds_read_b64_tr_b8)
MAIZE_TILE_TY(BF16_128x64, 128, 64, 2, Swizzle::KC16)    // A stages of the 128 x 256 tile kernels (the B stages are the ones above)
MAIZE_TILE_TY(F16_128x64, 128, 64, 2, Swizzle::KC16)
MAIZE_TILE_TY(F8_128x128, 128, 128, 1, Swizzle::KC16)
MAIZE_TILE_TY(BF16_64x128, 64, 128, 2, Swizzle::KN32)    // B stage of the 128 x 128 tile kernels for a row-major K x N B (stored N x K: BF16_128x64, like their A stage)
MAIZE_TILE_TY(F16_64x128, 64, 128, 2, Swizzle::KN32)
MAIZE_TILE_TY(F8_128x128_KN, 128, 128, 1, Swizzle::KN16) // ... for a row-major K x N 8-bit B (stored N x K: F8_128x128)
#undef MAIZE_TILE_TY
template <class T> struct Tile { using Ty = T; static constexpr size_t SIZE = (size_t)T::ROWS * T::COLS * T::ELEM_BYTES; };
template <class TA, class TB> struct TilePair { using A = TA; using B = TB; static constexpr size_t SIZE = TA::SIZE + TB::SIZE; };
template <class Pair, size_t PIPE> struct SharedRing {   // [TilePair; PIPE] in LDS (src/main.rs:42-44)
    using PairT = Pair;
    static constexpr size_t DEPTH = PIPE, SIZE = Pair::SIZE * PIPE;
    static_assert(SIZE <= 160 * 1024, "a compute unit has 160 KiB of LDS");
    uint32_t align;
};

// The MMA catalogue: one matrix instruction as an operation on wave fragments, D = A.B + C.  FRAG_*: 32-bit registers
// per lane; K_TILE: elements of K per ring stage of the kernels built on it.
enum class Family { MT256, WAVE32, MT128 };
#define MAIZE_MMA(name, m, n, k, in, fa, fb, fc, mnem, fam, ktile) \
    struct name { static constexpr uint32_t M = m, N = n, K = k, FRAG_A = fa, FRAG_B = fb, FRAG_C = fc, K_TILE = ktile; \
                  static constexpr maize_in_type_t IN_TYPE = in; static constexpr Family FAMILY = fam; \
                  static constexpr const char* NAME = #name; static constexpr const char* MNEMONIC = mnem; };
MAIZE_MMA(Gfx950MfmaBf16F32_16x16x32, 16, 16, 32, MAIZE_IN_BF16, 4, 4, 4, "v_mfma_f32_16x16x32_bf16", Family::MT256, 64)
MAIZE_MMA(Gfx950MfmaBf16F32_32x32x16, 32, 32, 16, MAIZE_IN_BF16, 4, 4, 16, "v_mfma_f32_32x32x16_bf16", Family::WAVE32, 16)
MAIZE_MMA(Gfx950MfmaF16F32_16x16x32, 16, 16, 32, MAIZE_IN_F16, 4, 4, 4, "v_mfma_f32_16x16x32_f16", Family::MT256, 64)
MAIZE_MMA(Gfx950MfmaE4M3F32_16x16x128, 16, 16, 128, MAIZE_IN_E4M3, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", Family::MT256, 128)
MAIZE_MMA(Gfx950MfmaE5M2F32_16x16x128, 16, 16, 128, MAIZE_IN_E5M2, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", Family::MT256, 128)
MAIZE_MMA(Gfx950MfmaE4M3E5M2F32_16x16x128, 16, 16, 128, MAIZE_IN_E4M3_E5M2, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", Family::MT256, 128)
MAIZE_MMA(Gfx950MfmaE5M2E4M3F32_16x16x128, 16, 16, 128, MAIZE_IN_E5M2_E4M3, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", Family::MT256, 128)
MAIZE_MMA(Gfx950MfmaF32F32_16x16x4, 16, 16, 4, MAIZE_IN_F32, 1, 1, 4, "v_mfma_f32_16x16x4_f32", Family::MT128, 32)
MAIZE_MMA(Gfx950MfmaF64F64_16x16x4, 16, 16, 4, MAIZE_IN_F64, 2, 2, 8, "v_mfma_f64_16x16x4_f64", Family::MT128, 16)
#undef MAIZE_MMA

class TracedKernel;
// Groups (Group, group/mod.rs:19-29).  BlockX shares out row panels, BlockY column panels; both are realised by one
// persistent 1-D grid whose workgroup g computes tiles g, g + grid, ... of an XCD-aware list (walk()).
inline uint32_t xcd_run(uint32_t pid, uint32_t total) {
    const uint32_t per = (total + 7u) / 8u, tall = (total % 8u) ? (total % 8u) : 8u, xcd = pid % 8u, local = pid / 8u;
    return xcd < tall ? xcd * per + local : tall * per + (xcd - tall) * (per - 1u) + local;
}
inline std::pair<uint32_t, uint32_t> tile_of(uint32_t idx, uint32_t tm, uint32_t tn, uint32_t group_rows = 4) {
    const uint32_t first = idx / (group_rows * tn) * group_rows, gsz = (tm - first) < group_rows ? (tm - first) : group_rows;
    const uint32_t in = idx % (group_rows * tn);
    return {first + in % gsz, in / gsz};
}
template <int AXIS> struct Block {
    TracedKernel* kernel;
    // Panel index of every tile workgroup `pid` of a grid of `grid` computes, and the number of panels (index_size()).
    std::pair<std::vector<uint32_t>, uint32_t> index_size(uint32_t pid, uint32_t tm, uint32_t tn, uint32_t grid) const {
        std::vector<uint32_t> walk;
        for (uint32_t i = pid; i < tm * tn; i += grid) { const auto t = tile_of(xcd_run(i, tm * tn), tm, tn); walk.push_back(AXIS == 0 ? t.first : t.second); }
        return {walk, AXIS == 0 ? tm : tn};
    }
};
using BlockX = Block<0>;
using BlockY = Block<1>;
struct Wave {                              // the 64-lane wavefront: the group that issues one cooperative copy (was Warp, 32 lanes)
    TracedKernel* kernel;
    static constexpr uint32_t const_size() { return 64; }
};

// Panels: N rows (columns) x the whole other extent.  `extent` is the window: N for bulk panels, the remainder for the
// ragged epilogue panel, which the reference's caller throws away (src/main.rs:56-57) and the kernels here compute.
template <uint32_t N> struct RowPanel { Matrix matrix; uint32_t extent; bool ragged; static constexpr uint32_t WINDOW = N;
    uint32_t row_size() const { return extent; } uint32_t col_size() const { return matrix.g.ncols; } };
template <uint32_t N> struct ColPanel { Matrix matrix; uint32_t extent; bool ragged; static constexpr uint32_t WINDOW = N;
    uint32_t row_size() const { return matrix.g.nrows; } uint32_t col_size() const { return extent; } };
template <class Panel> struct PanelIterLooper {
    Panel panel; uint32_t count;
    template <class F> void for_every_value(F&& body) const { body(panel); }   // once, like the reference's looper at trace time
};
template <uint32_t N, class Group>
std::pair<PanelIterLooper<RowPanel<N>>, RowPanel<N>> collective_aligned_row_panel_iter(const Matrix& m, Group) {
    return {PanelIterLooper<RowPanel<N>>{RowPanel<N>{m, N, false}, m.g.nrows / N}, RowPanel<N>{m, m.g.nrows % N, true}};
}
template <uint32_t N, class Group>
std::pair<PanelIterLooper<ColPanel<N>>, ColPanel<N>> collective_aligned_col_panel_iter(const Matrix& m, Group) {
    return {PanelIterLooper<ColPanel<N>>{ColPanel<N>{m, N, false}, m.g.ncols / N}, ColPanel<N>{m, m.g.ncols % N, true}};
}

// panel_rows, pipe, panel_cols: the panel height of A, the ring depth and the panel width of B as described (pipe 0: the description has no ring)
struct TracedOp { Matrix a, b, c; bool nt; maize_in_type_t in; Family family; bool stored; maize_out_type_t out; float alpha, beta; uint32_t panel_rows, pipe, panel_cols = 256; };
// The kernel that a description of the mainloop (panel height of A, ring depth) names for `x`; empty when the
// dispatcher's own choice already is of that family.  A description is honoured wherever a kernel of its family accepts
// the descriptor -- also where the dispatcher by itself would take another family -- and refused where none does.
inline std::string described_kernel(const maize_gemm_ex_desc_t& x, bool nt, uint32_t panel_rows, uint32_t pipe, uint32_t cus, uint32_t panel_cols = 256) {
    maize_gemm_plan_t plan;
    check(maize_hip_gemm_ex_plan(&x, nullptr, cus, &plan));
    const std::string chosen = plan.kernel;
    static const char* const tags[] = {"bf16", "f16", "e4m3", "e5m2", "e4m3e5m2", "e5m2e4m3"};
    if ((uint32_t)x.in_type > (uint32_t)MAIZE_IN_E5M2_E4M3) throw std::invalid_argument("no macro-tile kernel for this operand type");
    const std::string base = std::string("maize_gemm_") + tags[(int)x.in_type] + "_mt256_" + (nt ? "nt" : "nn");
    std::vector<std::string> names;
    const bool is_h = chosen.find("_h128") != std::string::npos, is_r3 = chosen.find("_h128r3") != std::string::npos;
    const bool is_q = chosen.find("_t128_") != std::string::npos;
    if (panel_cols == 128) {                      // 128 x 128 tiles
        names = {std::string("maize_gemm_") + tags[(int)x.in_type] + "_t128_" + (nt ? "nt" : "nn")};
        if (chosen == names[0]) return "";
    } else if (panel_rows == 256) {
        if (!is_h && !is_q) return "";            // a 256-row kernel, a split of one, or a few-row kernel: the dispatcher's
        names = {base, base + "_ktail", base + "_gen", base + "_ktail_gen"};
    } else {
        if (pipe == 3 ? is_r3 : (is_h && !is_r3)) return "";
        const std::string tag = pipe == 3 ? "_h128r3" : "_h128";
        names = {base + tag, base + tag + "_gen"};
    }
    for (const std::string& n : names)
        if (maize_hip_gemm_ex_plan(&x, n.c_str(), cus, &plan) == MAIZE_OK) return n;
    throw std::invalid_argument("no kernel with " + std::to_string(panel_rows) + "-row panels of A on " + std::to_string(pipe) + " ring stages runs this product");
}
class LoadedGemm {
  public:
    LoadedGemm(Ctx& ctx, const maize_gemm_ex_desc_t& x, const TracedOp& op) : ctx_(ctx), x_(x) {
        uint32_t cus = 256;
        maize_device_info_t info;
        if (maize_hip_device_info(ctx.handle(), &info) == MAIZE_OK) cus = info.compute_units;
        if (op.family == Family::WAVE32) forced_ = "maize_gemm_bf16_wave32";
        else if (op.family == Family::MT256 && op.pipe) forced_ = described_kernel(x_, op.nt, op.panel_rows, op.pipe, cus, op.panel_cols);
        check(maize_hip_gemm_ex_plan(&x_, forced(), cus, &plan_));
    }
    std::string kernel_name() const { return plan_.kernel; }
    const maize_gemm_plan_t& plan() const { return plan_; }
    void launch(void* stream = nullptr) { check(maize_hip_gemm_bf16_ex(ctx_.handle(), &x_, forced(), stream)); }
  private:
    const char* forced() const { return forced_.empty() ? nullptr : forced_.c_str(); }
    Ctx& ctx_; maize_gemm_ex_desc_t x_; std::string forced_; maize_gemm_plan_t plan_;
};
class PreLoadGemm {
  public:
    explicit PreLoadGemm(const TracedOp& op) : op_(op) {}
    LoadedGemm compile(Gfx target, Ctx& ctx) const {
        if (target != Gfx::Gfx950) throw std::invalid_argument("only Gfx::Gfx950 code is carried");
        maize_gemm_desc_t d;
        std::memset(&d, 0, sizeof d);
        d.a = op_.a.g.realize(); d.b = op_.b.g.realize(); d.c = op_.c.g.realize();
        d.layout = op_.nt ? MAIZE_LAYOUT_NT : MAIZE_LAYOUT_NN; d.batch = 1;
        maize_gemm_ex_desc_t x{};
        x.gemm = d; x.out_type = op_.out; x.alpha = op_.alpha; x.beta = op_.beta; x.in_type = op_.in;
        return LoadedGemm(ctx, x, op_);
    }
  private:
    TracedOp op_;
};
class TracedKernel {                       // new_hip_kernel() without a name: the kernel being described
  public:
    TracedKernel& with_launch_bounds_2d(std::pair<uint32_t, uint32_t> xy) {
        const uint64_t t = (uint64_t)xy.first * xy.second;
        if (t != 256 && t != 512) throw std::invalid_argument("the GEMM kernels run 4 wavefronts (256 threads; the skinny kernels 8)");
        bounds_ = true;
        return *this;
    }
    template <class Pair, size_t PIPE> SharedRing<Pair, PIPE> alloc_aligned_shared(uint32_t align) { return SharedRing<Pair, PIPE>{align}; }
    TracedKernel* cx() { return this; }
    PreLoadGemm finalize() const {
        if (!bounds_) throw std::invalid_argument("launch bounds not set");
        if (ops_.size() != 1 || !ops_[0].stored) throw std::invalid_argument("the trace must hold exactly one stored GEMM");
        return PreLoadGemm(ops_[0]);
    }
    std::vector<TracedOp> ops_;
  private:
    bool bounds_ = false;
};
class Accum {                              // the accumulator fragments of one panel pair; store() names the C they go to
  public:
    Accum(TracedKernel* k, const TracedOp& op) : k_(k), op_(op) {}
    void store(const Matrix& c, maize_out_type_t out = MAIZE_OUT_SAME, float alpha = 1.0f, float beta = 0.0f) {
        const uint32_t n = op_.nt ? op_.b.g.nrows : op_.b.g.ncols;
        if (c.g.nrows != op_.a.g.nrows || c.g.ncols != n) throw std::invalid_argument("C does not have the shape the panels describe");
        op_.c = c; op_.out = out; op_.alpha = alpha; op_.beta = beta; op_.stored = true;
        k_->ops_.push_back(op_);
    }
  private:
    TracedKernel* k_; TracedOp op_;
};
template <class Panel> struct is_row_panel : std::false_type {};
template <uint32_t N> struct is_row_panel<RowPanel<N>> : std::true_type {};
// sm80_gemm_smem_multibuffer(&mma, KTile::<K>, a_panel, b_panel, smem, cp_group, cp_size), gemm/mod.rs:37-90.  A B stored
// N x K hands in row panels of B; a K x N B column panels.
template <class MMA, uint32_t K_TILE, uint32_t NA, class BPanel, class Pair, size_t PIPE>
Accum gemm_smem_multibuffer(const MMA&, KTile<K_TILE>, const RowPanel<NA>& a, const BPanel& b, const SharedRing<Pair, PIPE>&, Wave cp_group, uint8_t cp_size) {
    constexpr bool NT = is_row_panel<BPanel>::value;
    static_assert(MMA::FAMILY == Family::MT256, "a shared-memory ring goes with the macro-tile kernels' instructions");
    static_assert(K_TILE == MMA::K_TILE, "KTile does not match the K a ring stage of this instruction's kernels holds");
    // Generic in the ring depth and the panel height like the reference's mainloop ([TilePair; PIPE], KTile<N>,
    // gemm/mod.rs:37-45), within what kernels exist: 256- or 128-row panels of A on two stages, 128-row panels also on
    // three (a 128 x 256 tile's stage is 48 KiB; three fit the 160 KiB of LDS).
    // ... and 128 x 128 tiles (128-row panels of A against 128-column panels of B) on a ring of four 32 KiB stages, 16-bit or 8-bit operands.
    constexpr uint32_t NB = BPanel::WINDOW;
    constexpr bool QUARTER = NA == 128 && NB == 128;
    static_assert(QUARTER ? PIPE == 4 : (PIPE == 2 || PIPE == 3), "the macro-tile kernels run a ring of two or three stages, the 128 x 128 tile kernels one of four");
    static_assert((NA == 256 || NA == 128) && (NB == 256 || QUARTER), "the macro-tile kernels take panels of 256 or 128 rows (A) and 256 columns (B), or 128 rows and 128 columns");
    static_assert(PIPE != 3 || NA == 128, "three ring stages fit the LDS with 128-row panels of A only");
    using TA = typename Pair::A::Ty; using TB = typename Pair::B::Ty;
    constexpr uint32_t ES = MMA::K_TILE == 128 ? 1 : 2;
    static_assert(TA::ROWS == NA && TA::COLS == MMA::K_TILE && TA::ELEM_BYTES == ES && TA::SWIZZLE == Swizzle::KC16, "A stage: panel rows x K_TILE, K-contiguous");
    static_assert(NT ? (TB::ROWS == NB && TB::COLS == MMA::K_TILE && TB::ELEM_BYTES == ES && TB::SWIZZLE == Swizzle::KC16)
                     : (TB::ROWS == MMA::K_TILE && TB::COLS == NB && TB::ELEM_BYTES == ES && TB::SWIZZLE == (ES == 2 ? Swizzle::KN32 : Swizzle::KN16)), "B stage does not match how B is stored");
    if (cp_size != 16) throw std::invalid_argument("direct-to-LDS copies are 16 bytes per lane");
    const uint32_t ka = a.col_size(), kb = NT ? b.matrix.g.ncols : b.matrix.g.nrows;
    if (ka != kb) throw std::invalid_argument("inner dimensions differ");
    return Accum(cp_group.kernel, TracedOp{a.matrix, b.matrix, Matrix{}, NT, MMA::IN_TYPE, MMA::FAMILY, false, MAIZE_OUT_SAME, 1.0f, 0.0f, NA, (uint32_t)PIPE, NB});
}
inline TracedKernel new_hip_kernel() { return TracedKernel(); }

// ---- builder chain: kernel name -> launch bounds -> finalize -> compile(target) -> launch ------
class LoadedKernel {
  public:
    LoadedKernel(maize_module_t* m, maize_kernel_t* k, uint32_t bx, uint32_t by) : mod_(m), k_(k) { block_[0] = bx; block_[1] = by; block_[2] = 1; }
    LoadedKernel(LoadedKernel&& o) noexcept : mod_(o.mod_), k_(o.k_) { std::memcpy(block_, o.block_, sizeof block_); o.mod_ = nullptr; o.k_ = nullptr; }
    LoadedKernel(const LoadedKernel&) = delete;
    ~LoadedKernel() { if (k_) maize_hip_kernel_release(k_); if (mod_) maize_hip_module_unload(mod_); }
    template <class Args>
    void launch(const uint32_t (&grid)[3], const Args& args, uint32_t lds_bytes = 0, void* stream = nullptr) {
        check(maize_hip_launch(k_, grid, block_, lds_bytes, stream, &args, sizeof(Args)));
    }
  private:
    maize_module_t* mod_;
    maize_kernel_t* k_;
    uint32_t block_[3];
};

class PreLoadKernel {
  public:
    PreLoadKernel(std::string name, uint32_t bx, uint32_t by) : name_(std::move(name)), bx_(bx), by_(by) {}
    LoadedKernel compile(Gfx target, Ctx& ctx) {
        if (target != Gfx::Gfx950) throw std::invalid_argument("only Gfx::Gfx950 code is carried");
        const void* co = nullptr; size_t n = 0;
        check(maize_hip_embedded_code_object(&co, &n));
        maize_module_t* m = nullptr; maize_kernel_t* k = nullptr;
        check(maize_hip_module_load(ctx.handle(), co, n, &m));
        const int32_t rc = maize_hip_kernel_get(m, name_.c_str(), &k);
        if (rc != MAIZE_OK) { const std::string msg = maize_hip_last_error(); maize_hip_module_unload(m); throw Error(rc, msg); }
        return LoadedKernel(m, k, bx_, by_);
    }
  private:
    std::string name_;
    uint32_t bx_, by_;
};

class HipKernel {
  public:
    explicit HipKernel(std::string name) : name_(std::move(name)) {}
    HipKernel& with_launch_bounds_2d(std::pair<uint32_t, uint32_t> xy) {
        if ((uint64_t)xy.first * xy.second == 0 || (uint64_t)xy.first * xy.second > 1024) throw std::invalid_argument("block must have 1..1024 threads");
        bx_ = xy.first; by_ = xy.second;
        return *this;
    }
    HipKernel& with_launch_bounds_1d(uint32_t x) { return with_launch_bounds_2d({x, 1}); }
    PreLoadKernel finalize() const {
        if (bx_ == 0) throw std::invalid_argument("launch bounds not set");
        return PreLoadKernel(name_, bx_, by_);
    }
  private:
    std::string name_;
    uint32_t bx_ = 0, by_ = 0;
};
inline HipKernel new_hip_kernel(const std::string& name) { return HipKernel(name); }

}  // namespace maize
