// Backward of the shared SwiGLU MLP  y = (silu(x Wg^T) * (x Wu^T)) Wd^T  for gfx950.
//
// The forward keeps only silu(a) * b unless it was asked to keep the gate and up products a, b as well
// (fmoe_mlp_gate_up_save); without them they are recomputed here (two launches of the forward's own NT GEMM).  The SwiGLU gradient is the fused
// elementwise kernel of fmoe_backward.hip (it also rebuilds h = silu(a) * b for dWd).  The remaining products are
// plain GEMMs in layouts the forward never needs (A B and A^T B); they go to rocBLAS, which is loaded on first use so
// that the forward path carries no dependency on it:
//     dh  = dy Wd              [T,H][H,I]
//     dWd = dy^T h             [T,H]^T [T,I]
//     dx  = da Wg + db Wu      [T,I][I,H] twice, the second accumulating
//     dWg = da^T x, dWu = db^T x
#include <dlfcn.h>
#include <rocblas/rocblas.h>

#include <mutex>

#include "fmoe_common.h"

namespace fmoe {

int launch_swiglu_backward(const void* dc, const void* a, const void* b, void* da, void* db, void* h, int64_t rows, int cols,
                           int64_t da_stride, int64_t db_stride, int dtype, hipStream_t stream);

namespace {

struct RocblasApi {
    decltype(&rocblas_create_handle) create_handle = nullptr;
    decltype(&rocblas_set_stream) set_stream = nullptr;
    decltype(&rocblas_gemm_ex) gemm_ex = nullptr;
    rocblas_handle handle[64] = {};
    std::mutex lock;
    bool tried = false;
};

RocblasApi& api() {
    static RocblasApi a;
    return a;
}

// Caller holds api().lock.
int rocblas_for_device(rocblas_handle* out) {
    RocblasApi& r = api();
    if (!r.tried) {
        r.tried = true;
        void* lib = nullptr;
        for (const char* name : {"librocblas.so.5", "librocblas.so", "/opt/rocm/lib/librocblas.so"}) {
            lib = dlopen(name, RTLD_NOW | RTLD_GLOBAL);
            if (lib) break;
        }
        if (lib) {
            r.create_handle = (decltype(r.create_handle))dlsym(lib, "rocblas_create_handle");
            r.set_stream = (decltype(r.set_stream))dlsym(lib, "rocblas_set_stream");
            r.gemm_ex = (decltype(r.gemm_ex))dlsym(lib, "rocblas_gemm_ex");
        }
    }
    FMOE_REQUIRE(r.create_handle && r.set_stream && r.gemm_ex, FMOE_ERR_LIBRARY,
                 "rocBLAS (librocblas.so) could not be loaded: %s", dlerror() ? dlerror() : "missing symbols");
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    FMOE_REQUIRE(e == hipSuccess && dev >= 0 && dev < 64, FMOE_ERR_LIBRARY, "no current HIP device for rocBLAS");
    if (!r.handle[dev]) {
        const rocblas_status st = r.create_handle(&r.handle[dev]);
        FMOE_REQUIRE(st == rocblas_status_success, FMOE_ERR_LIBRARY, "rocblas_create_handle failed (%d)", (int)st);
    }
    *out = r.handle[dev];
    return FMOE_OK;
}

constexpr int kNN = kBlasNN, kTN = kBlasTN;

struct MlpBwdPlan {
    size_t off_a, off_b, off_dh, off_h, off_dab, bytes;
};

MlpBwdPlan plan_mlp_backward(int64_t T_, int I, int dtype) {
    MlpBwdPlan p;
    const size_t ti = (size_t)T_ * I * dtype_size(dtype);
    size_t o = 0;
    auto take = [&](size_t n) { const size_t at = o; o = round_up(o + n, 256); return at; };
    p.off_a = take(ti);
    p.off_b = take(ti);
    p.off_dh = take(ti);
    p.off_h = take(ti);
    p.off_dab = take(2 * ti);
    p.bytes = o;
    return p;
}

}  // namespace

// Row-major product through the column-major library: C^T = B^T A^T, where a row-major [r,c] array is the
// column-major [c,r] one.  fp32 accumulation; A, B and C have the element type `dtype`.
int blas_gemm(int layout, int M, int N, int K, const void* A, int lda, const void* B, int ldb, void* C, int ldc, float beta,
              int dtype, hipStream_t stream) {
    std::lock_guard<std::mutex> guard(api().lock);
    rocblas_handle h = nullptr;
    if (int rc = rocblas_for_device(&h)) return rc;
    FMOE_REQUIRE(api().set_stream(h, stream) == rocblas_status_success, FMOE_ERR_LIBRARY, "rocblas_set_stream failed");
    const rocblas_datatype dt = dtype == FMOE_F32 ? rocblas_datatype_f32_r : (dtype == FMOE_BF16 ? rocblas_datatype_bf16_r : rocblas_datatype_f16_r);
    const float alpha = 1.0f;
    const rocblas_status st = api().gemm_ex(h, rocblas_operation_none, layout == kBlasNN ? rocblas_operation_none : rocblas_operation_transpose,
                                            N, M, K, &alpha, B, dt, ldb, A, dt, lda, &beta, C, dt, ldc, C, dt, ldc,
                                            rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
    FMOE_REQUIRE(st == rocblas_status_success, FMOE_ERR_LIBRARY, "rocblas_gemm_ex failed (%d)", (int)st);
    return FMOE_OK;
}

}  // namespace fmoe

extern "C" size_t fmoe_mlp_backward_workspace_bytes(int64_t num_tokens, int hidden, int intermediate, int dtype) {
    if (num_tokens <= 0 || hidden <= 0 || intermediate <= 0 || !fmoe::dtype_ok(dtype)) return 0;
    return fmoe::plan_mlp_backward(num_tokens, intermediate, dtype).bytes;
}

extern "C" int fmoe_mlp_backward(const void* dy, const void* x, const void* gate_w, const void* up_w, const void* down_w,
                                 const void* saved_products, int64_t num_tokens, int hidden, int intermediate, int dtype, void* dx, void* dgate_w, void* dup_w,
                                 void* ddown_w, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace fmoe;
    clear_error();
    FMOE_REQUIRE(dtype_ok(dtype), FMOE_ERR_BAD_DTYPE, "fmoe_mlp_backward: unknown dtype %d", dtype);
    FMOE_REQUIRE(num_tokens > 0 && hidden > 0 && intermediate > 0, FMOE_ERR_BAD_SHAPE, "fmoe_mlp_backward: bad shape T=%lld H=%d I=%d",
                 (long long)num_tokens, hidden, intermediate);
    FMOE_REQUIRE(num_tokens < (1ll << 31), FMOE_ERR_UNSUPPORTED, "fmoe_mlp_backward: T=%lld >= 2^31", (long long)num_tokens);
    const int vec = (int)(16 / dtype_size(dtype));
    FMOE_REQUIRE(hidden % vec == 0 && intermediate % vec == 0, FMOE_ERR_ALIGNMENT,
                 "fmoe_mlp_backward: hidden=%d and intermediate=%d must be multiples of %d (16-byte rows)", hidden, intermediate, vec);
    FMOE_REQUIRE(dy && x && gate_w && up_w && down_w && dx && dgate_w && dup_w && ddown_w, FMOE_ERR_NULL_POINTER,
                 "fmoe_mlp_backward: null tensor pointer");
    const MlpBwdPlan p = plan_mlp_backward(num_tokens, intermediate, dtype);
    FMOE_REQUIRE(workspace && workspace_bytes >= p.bytes && aligned16(workspace), FMOE_ERR_WORKSPACE,
                 "fmoe_mlp_backward: workspace of %zu bytes needed, %zu given", p.bytes, workspace_bytes);
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    void *a = ws + p.off_a, *b = ws + p.off_b, *dh = ws + p.off_dh, *h = ws + p.off_h;
    char* dab = ws + p.off_dab;
    const int T_ = (int)num_tokens, H = hidden, I = intermediate;
    const size_t elt = dtype_size(dtype);

    int rc = FMOE_OK;
    if (saved_products != nullptr) {
        // the forward kept a = x Wg^T and b = x Wu^T (fmoe_mlp_gate_up_save): planes [0] and [1] of a [2, T, I] buffer
        a = const_cast<void*>(saved_products);
        b = (char*)a + (size_t)num_tokens * I * elt;
    } else {
        // recompute them with the forward's NT kernel ("down" form: out[T,N] = act[T,K] W[N,K]^T)
        rc = fmoe_mlp_down(x, gate_w, num_tokens, I, H, dtype, nullptr, a, stream);
        if (rc) return rc;
        rc = fmoe_mlp_down(x, up_w, num_tokens, I, H, dtype, nullptr, b, stream);
        if (rc) return rc;
    }

    rc = blas_gemm(kNN, T_, I, H, dy, H, down_w, I, dh, I, 0.0f, dtype, s);                        // dh = dy Wd
    if (rc) return rc;
    // da and db side by side: one [T, 2I] matrix [da | db], so that products over both are single library calls
    char* db = dab + (size_t)I * elt;
    const int I2 = 2 * I;
    rc = launch_swiglu_backward(dh, a, b, dab, db, h, num_tokens, I, I2, I2, dtype, s);
    if (rc) return rc;
    rc = blas_gemm(kTN, H, I, T_, dy, H, h, I, ddown_w, I, 0.0f, dtype, s);                         // dWd = dy^T h
    if (rc) return rc;
    const size_t w_bytes = (size_t)I * H * elt;
    rc = blas_gemm(kNN, T_, H, I, dab, I2, gate_w, H, dx, H, 0.0f, dtype, s);                       // dx = da Wg
    if (rc) return rc;
    rc = blas_gemm(kNN, T_, H, I, db, I2, up_w, H, dx, H, 1.0f, dtype, s);                          //    + db Wu
    if (rc) return rc;
    // the two weight gradients are one [2I, H] product when the caller's buffers follow each other: one 74 us kernel at
    // T = I = 4096, H = 1024 instead of two of 49 us
    if ((char*)dup_w == (char*)dgate_w + w_bytes) return blas_gemm(kTN, I2, H, T_, dab, I2, x, H, dgate_w, H, 0.0f, dtype, s);
    rc = blas_gemm(kTN, I, H, T_, dab, I2, x, H, dgate_w, H, 0.0f, dtype, s);                       // dWg = da^T x
    if (rc) return rc;
    return blas_gemm(kTN, I, H, T_, db, I2, x, H, dup_w, H, 0.0f, dtype, s);                        // dWu = db^T x
}
