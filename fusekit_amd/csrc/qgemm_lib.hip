// Multi-row quantised matmul for LARGE row counts (prompt passes of several hundred rows):
// dequantise the matrix once to bf16, w = T(s * q + b) (one rounding per weight element: the
// arithmetic of the reference's multi-row kernels, which fill tiles of dequantised bf16 weights,
// src/codegen/msl.rs:2318-2440, and of this library's own form from 65 rows up), and hand the
// plain bf16 x bf16 -> fp32 product to rocBLAS; the epilogue kernel of the split-k path then
// applies bias / residual / SwiGLU to the fp32 sums and rounds once.
//
// From about 512 rows the matrix product itself dominates and a tuned library GEMM (≈ 0.9 PFLOP/s
// at 512 x 9728 x 2560, 1.1 at 1024 rows) beats the fused kernel, whose weight fragments are
// unpacked by every block that uses them (0.35 PFLOP/s).  Below that the int4 stream and the
// launch count matter more and the fused kernel is used.  rocBLAS is opened with dlopen on first
// use: the decode path never touches it, and a box without it keeps the fused kernel.
// Only direct calls take this route (fk_qgemm, fk_qgemm_swiglu); the dispatch families
// fusekit_qgemm* stay kernel nodes of a hipGraph.
#include <dlfcn.h>

#include <mutex>

#include "fk_device.hpp"
#include "fk_host.hpp"
#include "gemv_kernel.hpp"

namespace fk {

namespace {

// ---- the few rocBLAS declarations used (rocblas/rocblas.h; values from internal/rocblas-types.h) ----
typedef struct _rocblas_handle* rb_handle;
enum { rb_status_success = 0 };
enum { rb_op_none = 111, rb_op_transpose = 112 };
enum { rb_f32_r = 151, rb_bf16_r = 168 };
enum { rb_algo_standard = 0 };
enum { rb_atomics_not_allowed = 0 };
typedef int (*rb_create_handle_t)(rb_handle*);
typedef int (*rb_set_stream_t)(rb_handle, hipStream_t);
typedef int (*rb_set_atomics_mode_t)(rb_handle, int);
typedef int (*rb_gemm_sb_ex_t)(rb_handle, int, int, int, int, int, const void*, const void*, int, int, int64_t, const void*, int, int,
                               int64_t, const void*, const void*, int, int, int64_t, void*, int, int, int64_t, int, int, int, int32_t,
                               uint32_t);
typedef int (*rb_gemm_ex_t)(rb_handle, int, int, int, int, int, const void*, const void*, int, int, const void*, int, int,
                            const void*, const void*, int, int, void*, int, int, int, int, int32_t, uint32_t);

struct RocblasApi {
    bool tried = false, ok = false;
    rb_handle handle = nullptr;
    rb_set_stream_t set_stream = nullptr;
    rb_gemm_ex_t gemm_ex = nullptr;
    rb_gemm_sb_ex_t gemm_sb_ex = nullptr;
    std::mutex mu;  // one handle, one stream binding at a time
};
RocblasApi g_rb;
// row count from which direct calls take this route (0: never): below it the fused kernel's tile form is the faster
// one on the 4B-class projections (passes of 256 / 512 / 768 rows: +16 / +3..9 / +7 % prompt rate), from 1024 rows this route
uint32_t g_library_rows = 1024;

bool rocblas_ready() {
    if (g_rb.tried) return g_rb.ok;
    g_rb.tried = true;
    void* lib = dlopen("librocblas.so.5", RTLD_NOW | RTLD_LOCAL);
    if (!lib) lib = dlopen("librocblas.so", RTLD_NOW | RTLD_LOCAL);
    if (!lib) return false;
    auto create = reinterpret_cast<rb_create_handle_t>(dlsym(lib, "rocblas_create_handle"));
    auto atomics = reinterpret_cast<rb_set_atomics_mode_t>(dlsym(lib, "rocblas_set_atomics_mode"));
    g_rb.set_stream = reinterpret_cast<rb_set_stream_t>(dlsym(lib, "rocblas_set_stream"));
    g_rb.gemm_ex = reinterpret_cast<rb_gemm_ex_t>(dlsym(lib, "rocblas_gemm_ex"));
    g_rb.gemm_sb_ex = reinterpret_cast<rb_gemm_sb_ex_t>(dlsym(lib, "rocblas_gemm_strided_batched_ex"));
    if (!create || !atomics || !g_rb.set_stream || !g_rb.gemm_ex || !g_rb.gemm_sb_ex) return false;
    if (create(&g_rb.handle) != rb_status_success) return false;
    if (atomics(g_rb.handle, rb_atomics_not_allowed) != rb_status_success) return false;  // same bits on every run
    g_rb.ok = true;
    return true;
}

struct DequantArgs {
    const uint32_t* w;    // packed codes, one word = 8 int4 or 4 int8 codes
    const uint16_t* sc;
    const uint16_t* bi;
    uint16_t* out;        // bf16 [N, K]
    size_t words;
    uint32_t wpr;         // words per row
    uint32_t gpr;         // groups per row
    uint32_t wshift;      // log2(words per group)
};

// One thread per packed word: consecutive lanes read consecutive words and write consecutive
// 16-byte (int4) or 8-byte (int8) pieces of bf16, so loads and stores are whole cache lines.
template <bool Q4>
__global__ __launch_bounds__(256) void dequant_bf16_kernel(const DequantArgs a) {
    for (size_t p = (size_t)blockIdx.x * 256 + threadIdx.x; p < a.words; p += (size_t)gridDim.x * 256) {
        const size_t row = p / a.wpr;
        const uint32_t g = (uint32_t)(p - row * a.wpr) >> a.wshift;
        const float s = bf16_bits_to_f32(a.sc[row * a.gpr + g]), b = bf16_bits_to_f32(a.bi[row * a.gpr + g]);
        const uint32_t w = a.w[p];
        auto dq = [&](uint32_t code) { return fmaf((float)code, s, b); };
        if constexpr (Q4) {
            const uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;  // even / odd codes of the word
            *reinterpret_cast<uint4*>(a.out + p * 8u) =
                make_uint4(pack_bf16(dq(lo & 0xffu), dq(hi & 0xffu)), pack_bf16(dq((lo >> 8) & 0xffu), dq((hi >> 8) & 0xffu)),
                           pack_bf16(dq((lo >> 16) & 0xffu), dq((hi >> 16) & 0xffu)), pack_bf16(dq(lo >> 24), dq(hi >> 24)));
        } else {
            *reinterpret_cast<uint2*>(a.out + p * 4u) =
                make_uint2(pack_bf16(dq(w & 0xffu), dq((w >> 8) & 0xffu)), pack_bf16(dq((w >> 16) & 0xffu), dq(w >> 24)));
        }
    }
}

fk_status plan_dequant(const DeviceFacts* dev, const fk_weight* W, uint16_t* out, Launch* l) {
    DequantArgs a;
    const uint32_t per_word = W->bits == 4 ? 8u : 4u;
    a.w = reinterpret_cast<const uint32_t*>(W->w);
    a.sc = W->scales;
    a.bi = W->biases;
    a.out = out;
    a.wpr = W->k / per_word;
    a.words = (size_t)W->n * a.wpr;
    a.gpr = W->k / W->group;
    a.wshift = (W->group == 128 ? 7u : 6u) - (W->bits == 4 ? 3u : 2u);
    size_t blocks = (a.words + 255) / 256;
    if (blocks > (size_t)dev->cus * 32) blocks = (size_t)dev->cus * 32;
    l->func = W->bits == 4 ? reinterpret_cast<const void*>(&dequant_bf16_kernel<true>) : reinterpret_cast<const void*>(&dequant_bf16_kernel<false>);
    l->grid = dim3((uint32_t)blocks, 1, 1);
    l->block = dim3(256, 1, 1);
    l->shmem = 0;
    l->set_args(a);
    return FK_OK;
}

// P[m, N] (fp32, row-major) = x[m, K] . Wb[N, K]^T.  In the library's column-major terms:
// P^T (N x m, ld N) = op(A) . B with A = Wb seen as K x N (ld K), transposed, and B = x seen as K x m (ld K).
// With y set the library rounds T(sums (+ res)) itself (fp32 accumulate, one rounding) and p is unused.
fk_status library_product(const uint16_t* wb, const uint16_t* x, uint32_t m, uint32_t n, uint32_t k, float* p, uint16_t* y,
                          const uint16_t* res, hipStream_t s) {
    std::lock_guard<std::mutex> lk(g_rb.mu);
    if (g_rb.set_stream(g_rb.handle, s) != rb_status_success) return set_error(FK_ERR_HIP, "rocblas_set_stream failed");
    const float alpha = 1.0f, beta = (y && res) ? 1.0f : 0.0f;
    int st;
    if (y)
        st = g_rb.gemm_ex(g_rb.handle, rb_op_transpose, rb_op_none, (int)n, (int)m, (int)k, &alpha, wb, rb_bf16_r, (int)k, x, rb_bf16_r,
                          (int)k, &beta, res ? res : y, rb_bf16_r, (int)n, y, rb_bf16_r, (int)n, rb_f32_r, rb_algo_standard, 0, 0);
    else
        st = g_rb.gemm_ex(g_rb.handle, rb_op_transpose, rb_op_none, (int)n, (int)m, (int)k, &alpha, wb, rb_bf16_r, (int)k, x, rb_bf16_r,
                          (int)k, &beta, p, rb_f32_r, (int)n, p, rb_f32_r, (int)n, rb_f32_r, rb_algo_standard, 0, 0);
    if (st != rb_status_success) return set_error(FK_ERR_HIP, "rocblas_gemm_ex failed with status " + std::to_string(st));
    return FK_OK;
}

// Few output tiles and a deep k (the down projection: N = 2560, K = 9728): without atomics the
// library cannot split k itself and leaves most CUs idle (108 us whatever the row count up to
// 2048).  The k range is cut into `split` slices run as ONE strided-batched call, each into its
// own fp32 buffer; the epilogue kernel adds them in slice order.
uint32_t library_split(uint32_t m, uint32_t n, uint32_t k) {
    const uint32_t tiles = ((n + 255u) / 256u) * ((m + 255u) / 256u);
    if (tiles > 48u || k < 4096u) return 1;  // (9728 x 2560 at 512 rows: two slices 61 us, one 42 us)
    uint32_t want = (256u + tiles - 1u) / tiles;
    if (want > 8u) want = 8u;
    if (want > k / 1024u) want = k / 1024u;
    for (uint32_t sp = want; sp > 1u; --sp)
        if (k % (sp * 64u) == 0) return sp;
    return 1;
}

fk_status library_product_split(const uint16_t* wb, const uint16_t* x, uint32_t m, uint32_t n, uint32_t k, uint32_t split, float* p,
                                hipStream_t s) {
    std::lock_guard<std::mutex> lk(g_rb.mu);
    if (g_rb.set_stream(g_rb.handle, s) != rb_status_success) return set_error(FK_ERR_HIP, "rocblas_set_stream failed");
    const float alpha = 1.0f, beta = 0.0f;
    const uint32_t ks = k / split;
    const int st = g_rb.gemm_sb_ex(g_rb.handle, rb_op_transpose, rb_op_none, (int)n, (int)m, (int)ks, &alpha, wb, rb_bf16_r, (int)k, (int64_t)ks,
                                   x, rb_bf16_r, (int)k, (int64_t)ks, &beta, p, rb_f32_r, (int)n, (int64_t)m * n, p, rb_f32_r, (int)n,
                                   (int64_t)m * n, (int)split, rb_f32_r, rb_algo_standard, 0, 0);
    if (st != rb_status_success) return set_error(FK_ERR_HIP, "rocblas_gemm_strided_batched_ex failed with status " + std::to_string(st));
    return FK_OK;
}

bool shape_ok(const fk_weight* W, uint32_t m) {
    if (!W || !W->w || m == 0 || W->n == 0 || W->k == 0) return false;
    if ((uint64_t)m * W->n > 0x7fffffffull || W->n > 0x7fffffffu || W->k > 0x7fffffffu) return false;
    if (W->bits == 16) return W->k % 8u == 0;  // dense bf16 rows, 16-byte aligned
    const uint32_t vpl = W->bits == 4 ? 32u : 16u;
    return (W->bits == 4 || W->bits == 8) && W->scales && W->biases && (W->group == 64 || W->group == 128) &&
           W->k % W->group == 0 && W->k % vpl == 0;
}

}  // namespace

// SwiGLU of gate / up sums the library already rounded to T (every variant starts from T(acc_g), T(acc_u)):
// 16 bytes per lane and operand, 240 MB instead of 400 MB for a 4096 x 9728 pair.
struct SwigluRowsArgs {
    const uint4* g;
    const uint4* u;
    uint4* out;
    size_t n8;   // elements / 8
    int variant;
};
__global__ __launch_bounds__(256) void swiglu_rows_kernel(const SwigluRowsArgs a) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < a.n8; i += (size_t)gridDim.x * 256) {
        const uint4 g = a.g[i], u = a.u[i];
        const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            o[j] = swiglu_bits(bf16_lo(gw[j]), bf16_lo(uw[j]), a.variant, 1.0f) |
                   (swiglu_bits(bf16_hi(gw[j]), bf16_hi(uw[j]), a.variant, 1.0f) << 16);
        a.out[i] = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// An MLX-affine matrix as bf16 [n, k], every element T(code * scale + bias): the values the library route of the
// multi-row matmul works on.  A caller with memory to spare keeps the result and passes it as a dense weight.
fk_status run_dequantize_bf16(const fk_weight* W, uint16_t* out, hipStream_t s) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!W || !W->w || !W->scales || !W->biases || !out) return set_error(FK_ERR_INVALID, "dequantize: null tensor");
    if ((W->bits != 4 && W->bits != 8) || (W->group != 64 && W->group != 128) || W->k % W->group || W->n == 0)
        return set_error(FK_ERR_UNSUPPORTED, "dequantize: bits must be 4 or 8, group 64 or 128 dividing k");
    Launch l;
    FK_TRY(plan_dequant(dev, W, out, &l));
    return run_launch(l, s);
}

void set_gemm_library_rows(uint32_t rows) { g_library_rows = rows; }

bool qgemm_takes_library(uint32_t m) {
    if (g_library_rows == 0 || m < g_library_rows) return false;
    std::lock_guard<std::mutex> lk(g_rb.mu);
    return rocblas_ready();
}

bool gemm_library_available() {
    std::lock_guard<std::mutex> lk(g_rb.mu);
    return rocblas_ready();
}

size_t qgemm_library_sums_bytes(uint32_t m, uint32_t n, uint32_t k) {
    return (size_t)library_split(m, n, k) * m * n * sizeof(float);  // one fp32 buffer per k slice
}

size_t qgemm_library_workspace_bytes(uint32_t m, uint32_t n, uint32_t k) {
    return qgemm_library_sums_bytes(m, n, k) + (size_t)n * k * 2u;  // the sums, then the dequantised matrix
}

// workspace: [(m x N) fp32 sums per matrix or k slice][N x K bf16 dequantised matrix, reused by the second matrix in stream order]
fk_status run_qgemm_library(const fk_weight* W0, const fk_weight* W1, const uint16_t* x, uint32_t m, const uint16_t* bias,
                            const uint16_t* res, int variant, uint16_t* y, void* workspace, hipStream_t s) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!shape_ok(W0, m) || (W1 && !shape_ok(W1, m))) return set_error(FK_ERR_UNSUPPORTED, "qgemm (library route): shape not supported");
    const size_t sums = (size_t)m * W0->n;
    const uint32_t split = W1 ? 1u : library_split(m, W0->n, W0->k);
    float* p0 = static_cast<float*>(workspace);
    float* p1 = W1 ? p0 + sums : nullptr;
    uint16_t* scratch = reinterpret_cast<uint16_t*>(p0 + (W1 ? 2u : split) * sums);
    Launch l;
    // a dense bf16 matrix is used where it lies; a quantised one is dequantised into the workspace
    auto bf16_rows = [&](const fk_weight* W, const uint16_t** out) -> fk_status {
        if (W->bits == 16) {
            *out = static_cast<const uint16_t*>(W->w);
            return FK_OK;
        }
        FK_TRY(plan_dequant(dev, W, scratch, &l));
        FK_TRY(run_launch(l, s));
        *out = scratch;
        return FK_OK;
    };
    const uint16_t* wb = nullptr;
    FK_TRY(bf16_rows(W0, &wb));
    if (split > 1) {
        FK_TRY(library_product_split(wb, x, m, W0->n, W0->k, split, p0, s));
        Launch reduce;
        plan_qgemm_epilogue(p0, nullptr, bias, res, y, m, W0->n, split, 0, &reduce);
        return run_launch(reduce, s);
    }
    if (!W1 && !bias)  // nothing left for an epilogue kernel but the rounding (and the residual)
        return library_product(wb, x, m, W0->n, W0->k, nullptr, y, res, s);
    if (W1 && m >= 2048 && sums % 8 == 0 && ((uintptr_t)y & 15u) == 0) {
        // Large passes (measured on one box: 4096 rows +4 %, 512 rows -2 %, so from 2048 rows): gate and up rounded
        // to T by the library into the two halves of the sums area, then one pass over bf16
        uint16_t* gb = reinterpret_cast<uint16_t*>(p0);
        uint16_t* ub = reinterpret_cast<uint16_t*>(p1);
        FK_TRY(library_product(wb, x, m, W0->n, W0->k, nullptr, gb, nullptr, s));
        FK_TRY(bf16_rows(W1, &wb));  // reuses the scratch: the first product is ahead of it in stream order
        FK_TRY(library_product(wb, x, m, W1->n, W1->k, nullptr, ub, nullptr, s));
        SwigluRowsArgs a{reinterpret_cast<const uint4*>(gb), reinterpret_cast<const uint4*>(ub), reinterpret_cast<uint4*>(y),
                         sums / 8, variant};
        size_t blocks = (a.n8 + 255) / 256;
        if (blocks > (size_t)dev->cus * 16) blocks = (size_t)dev->cus * 16;
        l.func = reinterpret_cast<const void*>(&swiglu_rows_kernel);
        l.grid = dim3((uint32_t)blocks, 1, 1);
        l.block = dim3(256, 1, 1);
        l.shmem = 0;
        l.then.clear();
        l.set_args(a);
        return run_launch(l, s);
    }
    FK_TRY(library_product(wb, x, m, W0->n, W0->k, p0, nullptr, nullptr, s));
    if (W1) {
        FK_TRY(bf16_rows(W1, &wb));  // reuses the scratch: the first product is ahead of it in stream order
        FK_TRY(library_product(wb, x, m, W1->n, W1->k, p1, nullptr, nullptr, s));
    }
    Launch reduce;
    plan_qgemm_epilogue(p0, p1, bias, res, y, m, W0->n, 1, variant, &reduce);
    return run_launch(reduce, s);
}

}  // namespace fk
