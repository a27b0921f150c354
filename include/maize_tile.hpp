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
