// extern "C" surface of libfusekit_hip.so: error state, device memory and the
// operator launches.  Declarations and reference citations live in
// include/fusekit_hip.h.
#include <math.h>

#include <mutex>

#include "fk_host.hpp"
#include "xcd_layer.hpp"

namespace fk {

static thread_local std::string t_last_error;

fk_status set_error(fk_status code, const std::string& msg) {
    t_last_error = msg;
    return code;
}

fk_status hip_error(hipError_t e, const char* what) {
    return set_error(FK_ERR_HIP, std::string(what) + ": " + hipGetErrorString(e));
}

fk_status device_facts(const DeviceFacts** out) {
    static DeviceFacts facts;
    static fk_status status = FK_OK;
    static std::string message;
    static std::once_flag once;
    std::call_once(once, [] {
        int n = 0;
        hipError_t e = hipGetDeviceCount(&n);
        if (e != hipSuccess || n == 0) {
            status = FK_ERR_HIP;
            message = "no HIP device available (this library has no CPU path)";
            return;
        }
        e = hipGetDeviceProperties(&facts.prop, 0);
        if (e != hipSuccess) {
            status = FK_ERR_HIP;
            message = std::string("hipGetDeviceProperties: ") + hipGetErrorString(e);
            return;
        }
        facts.cus = facts.prop.multiProcessorCount;
        facts.max_dyn_lds = (int)facts.prop.sharedMemPerBlock;
        int optin = 0;
        if (hipDeviceGetAttribute(&optin, hipDeviceAttributeSharedMemPerBlockOptin, 0) == hipSuccess &&
            optin > facts.max_dyn_lds)
            facts.max_dyn_lds = optin;
    });
    if (status != FK_OK) return set_error(status, message);
    *out = &facts;
    return FK_OK;
}

fk_status run_launch(const Launch& l, hipStream_t s) {
    if (!l.func) return FK_OK;  // an empty launch (a planner that needed fewer kernels than its caller offers)
    void* params[kMaxKernelParams];
    const_cast<Launch&>(l).params(params);
    FK_HIP(hipLaunchKernel(l.func, l.grid, l.block, params, l.shmem, s));
    for (const Launch& f : l.then) FK_TRY(run_launch(f, s));
    return FK_OK;
}

}  // namespace fk

using namespace fk;

extern "C" {

const char* fk_last_error(void) { return t_last_error.c_str(); }
const char* fk_version(void) { return "fusekit-hip 0.1.0 (gfx950)"; }

fk_status fk_device_props_get(fk_device_props* out) {
    if (!out) return set_error(FK_ERR_INVALID, "null out");
    const DeviceFacts* d;
    FK_TRY(device_facts(&d));
    memset(out, 0, sizeof(*out));
    strncpy(out->name, d->prop.name, sizeof(out->name) - 1);
    strncpy(out->arch, d->prop.gcnArchName, sizeof(out->arch) - 1);
    out->compute_units = d->cus;
    out->wavefront = d->prop.warpSize;
    out->lds_bytes_per_block = d->max_dyn_lds;
    out->l2_bytes = d->prop.l2CacheSize;
    out->hbm_bytes = d->prop.totalGlobalMem;
    out->clock_khz = d->prop.clockRate;
    return FK_OK;
}

fk_status fk_target_describe(fk_target* out) {
    if (!out) return set_error(FK_ERR_INVALID, "null out");
    memset(out, 0, sizeof(*out));
    // published MI355X (gfx950, CDNA4) figures
    strncpy(out->arch, "gfx950", sizeof(out->arch) - 1);
    out->compute_units = 256;
    out->xcds = 8;
    out->wave_size = 64;
    out->simds_per_cu = 4;
    out->vgprs_per_lane = 512;
    out->lds_bytes_per_cu = 160 * 1024;
    out->workgroup_threads = 256;
    out->gemm_min_rows = 2;
    out->gemm_rows_per_pass = 128;
    out->hbm_bytes = 288ull << 30;
    out->hbm_peak_bytes_per_s = 8.0e12;
    out->mfma_bf16_peak_flops = 2.5e15;
    const DeviceFacts* d;
    if (device_facts(&d) == FK_OK) {
        out->from_device = 1;
        strncpy(out->arch, d->prop.gcnArchName, sizeof(out->arch) - 1);
        out->compute_units = (uint32_t)d->cus;
        out->wave_size = (uint32_t)d->prop.warpSize;
        out->lds_bytes_per_cu = (uint32_t)d->prop.maxSharedMemoryPerMultiProcessor;
        out->hbm_bytes = d->prop.totalGlobalMem;
    } else {
        set_error(FK_OK, "");
    }
    return FK_OK;
}

fk_status fk_alloc(size_t nbytes, void** dptr) {
    if (!dptr || nbytes == 0) return set_error(FK_ERR_INVALID, "fk_alloc: null out pointer or zero size");
    const DeviceFacts* d;
    FK_TRY(device_facts(&d));
    FK_HIP(hipMalloc(dptr, nbytes));
    return FK_OK;
}

fk_status fk_mem_info(size_t* free_bytes, size_t* total_bytes) {
    if (!free_bytes || !total_bytes) return set_error(FK_ERR_INVALID, "fk_mem_info: null out pointer");
    const DeviceFacts* d;
    FK_TRY(device_facts(&d));
    FK_HIP(hipMemGetInfo(free_bytes, total_bytes));
    return FK_OK;
}

fk_status fk_free(void* dptr) {
    if (!dptr) return FK_OK;
    FK_HIP(hipFree(dptr));
    return FK_OK;
}

fk_status fk_upload(void* dptr, const void* host, size_t nbytes) {
    if (!dptr || !host) return set_error(FK_ERR_INVALID, "fk_upload: null pointer");
    FK_HIP(hipMemcpy(dptr, host, nbytes, hipMemcpyHostToDevice));
    return FK_OK;
}

fk_status fk_download(void* host, const void* dptr, size_t nbytes) {
    if (!dptr || !host) return set_error(FK_ERR_INVALID, "fk_download: null pointer");
    FK_HIP(hipMemcpy(host, dptr, nbytes, hipMemcpyDeviceToHost));
    return FK_OK;
}

fk_status fk_stream_create(fk_stream* out) {
    if (!out) return set_error(FK_ERR_INVALID, "null out");
    const DeviceFacts* d;
    FK_TRY(device_facts(&d));
    hipStream_t s;
    FK_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *out = s;
    return FK_OK;
}
fk_status fk_stream_destroy(fk_stream s) {
    if (s) FK_HIP(hipStreamDestroy((hipStream_t)s));
    return FK_OK;
}
fk_status fk_stream_sync(fk_stream s) {
    FK_HIP(hipStreamSynchronize((hipStream_t)s));
    return FK_OK;
}

fk_status fk_event_create(fk_event* out) {
    if (!out) return set_error(FK_ERR_INVALID, "null out");
    const DeviceFacts* d;
    FK_TRY(device_facts(&d));
    hipEvent_t e;
    FK_HIP(hipEventCreate(&e));
    *out = e;
    return FK_OK;
}
fk_status fk_event_destroy(fk_event e) {
    if (e) FK_HIP(hipEventDestroy((hipEvent_t)e));
    return FK_OK;
}
fk_status fk_event_record(fk_event e, fk_stream s) {
    if (!e) return set_error(FK_ERR_INVALID, "null event");
    FK_HIP(hipEventRecord((hipEvent_t)e, (hipStream_t)s));
    return FK_OK;
}
fk_status fk_event_elapsed_ms(fk_event start, fk_event stop, float* ms) {
    if (!start || !stop || !ms) return set_error(FK_ERR_INVALID, "null event or out pointer");
    FK_HIP(hipEventSynchronize((hipEvent_t)stop));
    FK_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return FK_OK;
}

fk_status fk_set_qgemm_wide(int enabled) {
    set_qgemm_wide(enabled != 0);
    return FK_OK;
}

fk_status fk_set_gemm_library_rows(uint32_t rows) {
    set_gemm_library_rows(rows);
    return FK_OK;
}

fk_status fk_set_gemv_policy(uint32_t rows_per_tile, uint32_t grid_blocks) {
    g_gemv_policy.rows_per_tile = rows_per_tile;
    g_gemv_policy.grid_blocks = grid_blocks;
    return FK_OK;
}

int fk_gemv_form(uint32_t n, uint32_t k, uint32_t bits, uint32_t group) { return gemv_rows_batch(n, k, bits, group) ? 1 : 0; }

fk_status fk_set_gemv_flat_only(int flat_only) {
    g_gemv_policy.flat_only = flat_only != 0;
    return FK_OK;
}

fk_status fk_qgemv(const fk_weight* W, const uint16_t* x, const uint16_t* bias, uint16_t* y, fk_stream s) {
    GemvRequest rq;
    rq.mats[0] = W;
    rq.bias[0] = bias;
    rq.y[0] = y;
    rq.x = x;
    Launch l;
    FK_TRY(plan_gemv(rq, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_linear_residual(const fk_weight* W, const uint16_t* x, const uint16_t* res, const uint16_t* res2,
                             uint16_t* y, fk_stream s) {
    if (!res) return set_error(FK_ERR_INVALID, "fk_linear_residual: null residual");
    GemvRequest rq;
    rq.mats[0] = W;
    rq.y[0] = y;
    rq.x = x;
    rq.res = res;
    rq.res2 = res2;
    Launch l;
    FK_TRY(plan_gemv(rq, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_rmsnorm_qkv(const uint16_t* x, const uint16_t* norm_w, float eps, const fk_weight* Wq,
                         const fk_weight* Wk, const fk_weight* Wv, const uint16_t* bq, const uint16_t* bk,
                         const uint16_t* bv, uint16_t* q, uint16_t* k, uint16_t* v, fk_stream s) {
    GemvRequest rq;
    rq.n_mats = 3;
    rq.mats[0] = Wq; rq.mats[1] = Wk; rq.mats[2] = Wv;
    rq.bias[0] = bq; rq.bias[1] = bk; rq.bias[2] = bv;
    rq.y[0] = q; rq.y[1] = k; rq.y[2] = v;
    rq.x = x;
    rq.norm_w = norm_w;
    rq.eps = eps;
    Launch l;
    FK_TRY(plan_gemv(rq, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_rmsnorm_qkv_rows(const uint16_t* x, uint32_t rows, uint32_t x_row_stride, const uint16_t* norm_w, float eps,
                              const fk_weight* Wq, const fk_weight* Wk, const fk_weight* Wv, uint16_t* q,
                              uint32_t q_row_stride, uint16_t* k, uint32_t k_row_stride, uint16_t* v, uint32_t v_row_stride,
                              fk_stream s) {
    if (!Wq) return set_error(FK_ERR_INVALID, "fk_rmsnorm_qkv_rows: null Wq");
    if (!Wk && Wv) return set_error(FK_ERR_INVALID, "fk_rmsnorm_qkv_rows: Wv without Wk");
    WideSeg segs[3] = {{Wq, q, q_row_stride}, {Wk, k, k_row_stride}, {Wv, v, v_row_stride}};
    Launch l;
    FK_TRY(plan_qgemm_wide_fan(x, x_row_stride, rows, norm_w, eps, segs, Wv ? 3u : (Wk ? 2u : 1u), &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_gateup_swiglu_rows(const uint16_t* x, uint32_t rows, const uint16_t* norm_w, float eps, const fk_weight* Wg,
                                const fk_weight* Wu, int variant, uint16_t* out, fk_stream s) {
    if (!Wg || !Wu || !x || !out) return set_error(FK_ERR_INVALID, "fk_gateup_swiglu_rows: null weight, input or output");
    if (variant < 0 || variant > 2) return set_error(FK_ERR_INVALID, "fk_gateup_swiglu_rows: variant must be 0, 1 or 2");
    if (Wg->n != Wu->n || Wg->k != Wu->k || Wg->group != Wu->group || Wg->bits != Wu->bits)
        return set_error(FK_ERR_INVALID, "fk_gateup_swiglu_rows: gate and up need the same shape, bits and group size");
    if (rows < 2 || rows > 8 || Wg->group != 64 || (Wg->bits != 4 && Wg->bits != 8))
        return set_error(FK_ERR_UNSUPPORTED, "fk_gateup_swiglu_rows: 2..8 rows, 4- or 8-bit weights, group size 64");
    Launch l;
    FK_TRY(plan_qgemm_wide(Wg, Wu, x, rows, nullptr, nullptr, variant, out, &l, norm_w, eps));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_gateup_swiglu(const uint16_t* x, const uint16_t* norm_w, float eps, const fk_weight* Wg,
                           const fk_weight* Wu, int variant, uint16_t* out, fk_stream s) {
    if (variant < 0 || variant > 2) return set_error(FK_ERR_INVALID, "fk_gateup_swiglu: variant must be 0, 1 or 2");
    GemvRequest rq;
    rq.swiglu = true;
    rq.swiglu_variant = variant;
    rq.mats[0] = Wg; rq.mats[1] = Wu;
    rq.y[0] = out;
    rq.x = x;
    rq.norm_w = norm_w;
    rq.eps = eps;
    Launch l;
    FK_TRY(plan_gemv(rq, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_routed_qmv_swiglu(const uint16_t* x, uint32_t n_x_rows, const fk_weight* Wg, const fk_weight* Wu,
                               uint32_t n_experts, const uint32_t* row_idx, const uint32_t* expert_idx,
                               const uint16_t* route_weight, uint32_t n_routes, uint16_t* out0, fk_stream s) {
    if (!Wg || !Wu) return set_error(FK_ERR_INVALID, "fk_routed_qmv_swiglu: null weight");
    Launch l;
    FK_TRY(plan_routed_gemv(x, n_x_rows, Wg, Wu, n_experts, row_idx, expert_idx, route_weight, n_routes, out0, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_routed_qmv_swiglu_shared(const uint16_t* x, const fk_weight* Wg, const fk_weight* Wu, uint32_t n_experts,
                                      const uint32_t* expert_idx, const uint16_t* route_weight, uint32_t n_routes,
                                      uint16_t* out0, const fk_weight* Sg, const fk_weight* Su, uint16_t* shared_out,
                                      fk_stream s) {
    if (!Wg || !Wu || !Sg || !Su) return set_error(FK_ERR_INVALID, "fk_routed_qmv_swiglu_shared: null weight");
    Launch l;
    FK_TRY(plan_routed_gemv(x, 1, Wg, Wu, n_experts, nullptr, expert_idx, route_weight, n_routes, out0, &l, Sg, Su, shared_out));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_routed_qmv_swiglu_routing(const uint16_t* x, const fk_weight* Wg, const fk_weight* Wu, uint32_t n_experts,
                                       const uint16_t* logits, const uint16_t* scale, uint32_t top_k, int apply_weight,
                                       uint32_t* idx_out, uint16_t* weight_out, uint16_t* out0, const fk_weight* Sg,
                                       const fk_weight* Su, uint16_t* shared_out, fk_stream s) {
    if (!Wg || !Wu) return set_error(FK_ERR_INVALID, "fk_routed_qmv_swiglu_routing: null weight");
    if ((Sg != nullptr) != (Su != nullptr)) return set_error(FK_ERR_INVALID, "fk_routed_qmv_swiglu_routing: shared gate and up come together");
    RouteInKernel rk;
    rk.logits = logits; rk.scale = scale; rk.idx_out = idx_out; rk.weight_out = weight_out; rk.apply_weight = apply_weight != 0;
    Launch l;
    FK_TRY(plan_routed_gemv(x, 1, Wg, Wu, n_experts, nullptr, nullptr, nullptr, top_k, out0, &l, Sg, Su, shared_out, &rk));
    return run_launch(l, (hipStream_t)s);
}

size_t fk_routed_reduce_workspace_bytes(uint32_t n_tokens, uint32_t top_k, uint32_t out_dim) {
    return routed_reduce_workspace_bytes(n_tokens, top_k, out_dim, 0, 0);
}

size_t fk_routed_reduce_workspace_bytes_shared(uint32_t n_tokens, uint32_t top_k, uint32_t out_dim, uint32_t shared_k,
                                               uint32_t group) {
    return routed_reduce_workspace_bytes(n_tokens, top_k, out_dim, shared_k, group);
}

fk_status fk_routed_qmv_reduce(const uint16_t* h, uint32_t n_h_rows, const fk_weight* Wd, uint32_t n_experts,
                               const uint32_t* row_idx, const uint32_t* expert_idx, const uint16_t* route_weight,
                               const uint16_t* shared_x, const fk_weight* W_shared, const uint16_t* residual_extra,
                               uint32_t n_tokens, uint32_t top_k, uint16_t* out, void* workspace, fk_stream s) {
    if (!workspace) return set_error(FK_ERR_INVALID, "fk_routed_qmv_reduce: null workspace");
    Launch l;
    FK_TRY(plan_routed_reduce_chain(h, n_h_rows, Wd, n_experts, row_idx, expert_idx, route_weight, shared_x, W_shared,
                                    residual_extra, n_tokens, top_k, out, static_cast<uint16_t*>(workspace), &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_route_order(const uint32_t* expert_idx, uint32_t n_routes, uint32_t n_experts, uint32_t* order, fk_stream s) {
    Launch l;
    FK_TRY(plan_route_order(expert_idx, n_routes, n_experts, order, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_routed_qmv_swiglu_ordered(const uint16_t* x, uint32_t n_x_rows, const fk_weight* Wg, const fk_weight* Wu,
                                       uint32_t n_experts, const uint32_t* row_idx, const uint32_t* expert_idx,
                                       const uint16_t* route_weight, uint32_t n_routes, const uint32_t* order,
                                       uint16_t* out0, fk_stream s) {
    if (!Wg || !Wu) return set_error(FK_ERR_INVALID, "fk_routed_qmv_swiglu_ordered: null weight");
    Launch l;   // no order array: the launch ranks its routes itself
    FK_TRY(plan_routed_gemv(x, n_x_rows, Wg, Wu, n_experts, row_idx, expert_idx, route_weight, n_routes, out0, &l, nullptr,
                            nullptr, nullptr, nullptr, order ? order : kOrderInKernel));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_routed_qmv_reduce_ordered(const uint16_t* h, uint32_t n_h_rows, const fk_weight* Wd, uint32_t n_experts,
                                       const uint32_t* row_idx, const uint32_t* expert_idx, const uint16_t* route_weight,
                                       const uint16_t* shared_x, const fk_weight* W_shared, const uint16_t* residual_extra,
                                       uint32_t n_tokens, uint32_t top_k, const uint32_t* order, uint16_t* out, void* workspace,
                                       fk_stream s) {
    if (!workspace) return set_error(FK_ERR_INVALID, "fk_routed_qmv_reduce_ordered: null workspace");
    Launch l;
    FK_TRY(plan_routed_reduce_chain(h, n_h_rows, Wd, n_experts, row_idx, expert_idx, route_weight, shared_x, W_shared,
                                    residual_extra, n_tokens, top_k, out, static_cast<uint16_t*>(workspace), &l,
                                    order ? order : kOrderInKernel));
    return run_launch(l, (hipStream_t)s);
}

void fk_set_routed_fused_reduce(int on) { set_routed_fused_reduce(on != 0); }

int fk_gemm_library_available(void) { return gemm_library_available() ? 1 : 0; }

fk_status fk_dequantize_bf16(const fk_weight* W, uint16_t* out, fk_stream s) { return run_dequantize_bf16(W, out, (hipStream_t)s); }

fk_status fk_qgemm_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, uint32_t group, size_t* bytes) {
    if (!bytes) return set_error(FK_ERR_INVALID, "fk_qgemm_workspace_bytes: null output");
    return qgemm_workspace_bytes(m, n, k, group, bytes);
}

fk_status fk_qgemm(const fk_weight* W, const uint16_t* x, uint32_t m, const uint16_t* bias, const uint16_t* residual,
                   uint16_t* y, void* workspace, fk_stream s) {
    if (W && W->bits == 16) {  // dense bf16 weights: the plain library GEMM with this library's epilogue
        if (!x || !y || !workspace) return set_error(FK_ERR_INVALID, "fk_qgemm: null activation, output or workspace");
        if (!gemm_library_available()) return set_error(FK_ERR_UNSUPPORTED, "fk_qgemm: bf16 weights need rocBLAS (librocblas.so.5 not found)");
        return run_qgemm_library(W, nullptr, x, m, bias, residual, 0, y, workspace, (hipStream_t)s);
    }
    Launch main, reduce;
    FK_TRY(plan_qgemm(W, x, m, bias, residual, y, workspace, &main, &reduce));  // validates the arguments for both routes
    if (qgemm_takes_library(m)) return run_qgemm_library(W, nullptr, x, m, bias, residual, 0, y, workspace, (hipStream_t)s);
    FK_TRY(run_launch(main, (hipStream_t)s));
    return run_launch(reduce, (hipStream_t)s);
}

fk_status fk_qgemm_fanout(const fk_weight* const* W, uint32_t n_mats, const uint16_t* x, uint32_t m,
                          const uint16_t* const* bias, uint16_t* const* y, void* workspace, fk_stream s) {
    if (!W || !y || n_mats < 1 || n_mats > 3) return set_error(FK_ERR_INVALID, "fk_qgemm_fanout: one to three matrices");
    bool fused = false;
    if (n_mats > 1 && W[0] && W[0]->bits != 16 && !qgemm_takes_library(m)) {
        Launch main, reduce;
        FK_TRY(plan_qgemm_fanout(W, n_mats, x, m, bias, y, workspace, &main, &reduce, &fused));
        if (fused) {
            FK_TRY(run_launch(main, (hipStream_t)s));
            return run_launch(reduce, (hipStream_t)s);
        }
    }
    for (uint32_t i = 0; i < n_mats; ++i)   // one by one, in stream order (they share the workspace)
        FK_TRY(fk_qgemm(W[i], x, m, bias ? bias[i] : nullptr, nullptr, y[i], workspace, s));
    return FK_OK;
}

fk_status fk_qgemm_swiglu(const fk_weight* Wg, const fk_weight* Wu, const uint16_t* x, uint32_t m, int variant,
                          uint16_t* out, void* workspace, fk_stream s) {
    if (Wg && Wu && Wg->bits == 16 && Wu->bits == 16) {
        if (!x || !out || !workspace) return set_error(FK_ERR_INVALID, "fk_qgemm_swiglu: null activation, output or workspace");
        if (Wg->n != Wu->n || Wg->k != Wu->k) return set_error(FK_ERR_INVALID, "fk_qgemm_swiglu: gate and up need the same shape");
        if (variant < 0 || variant > 2) return set_error(FK_ERR_INVALID, "fk_qgemm_swiglu: variant must be 0, 1 or 2");
        if (!gemm_library_available()) return set_error(FK_ERR_UNSUPPORTED, "fk_qgemm_swiglu: bf16 weights need rocBLAS (librocblas.so.5 not found)");
        return run_qgemm_library(Wg, Wu, x, m, nullptr, nullptr, variant, out, workspace, (hipStream_t)s);
    }
    Launch gate, up, reduce;
    FK_TRY(plan_qgemm_swiglu(Wg, Wu, x, m, variant, out, workspace, &gate, &up, &reduce));
    if (qgemm_takes_library(m)) return run_qgemm_library(Wg, Wu, x, m, nullptr, nullptr, variant, out, workspace, (hipStream_t)s);
    FK_TRY(run_launch(gate, (hipStream_t)s));
    FK_TRY(run_launch(up, (hipStream_t)s));
    return run_launch(reduce, (hipStream_t)s);
}

fk_status fk_final_rmsnorm_lm_head(const uint16_t* x, const uint16_t* norm_w, float eps, const fk_weight* W,
                                   uint16_t* logits, fk_stream s) {
    if (!norm_w) return set_error(FK_ERR_INVALID, "fk_final_rmsnorm_lm_head: null norm weight");
    GemvRequest rq;
    rq.mats[0] = W;
    rq.y[0] = logits;
    rq.x = x;
    rq.norm_w = norm_w;
    rq.eps = eps;
    Launch l;
    FK_TRY(plan_gemv(rq, &l));
    return run_launch(l, (hipStream_t)s);
}

static_assert(FK_HEAD_ARGMAX_WORKSPACE_BYTES == kHeadArgmaxWorkspaceBytes, "header and kernel disagree");

fk_status fk_final_rmsnorm_lm_head_argmax(const uint16_t* x, const uint16_t* norm_w, float eps, const fk_weight* W,
                                          uint16_t* logits, uint32_t* next_token, uint32_t* history,
                                          uint32_t* hist_counter, uint32_t hist_capacity, void* workspace,
                                          fk_stream s) {
    if (!norm_w) return set_error(FK_ERR_INVALID, "fk_final_rmsnorm_lm_head_argmax: null norm weight");
    HeadArgmax am;
    am.next_token = next_token;
    am.history = history;
    am.hist_counter = hist_counter;
    am.hist_capacity = hist_capacity;
    am.workspace = workspace;
    GemvRequest rq;
    rq.mats[0] = W;
    rq.y[0] = logits;
    rq.x = x;
    rq.norm_w = norm_w;
    rq.eps = eps;
    rq.argmax = &am;
    Launch l;
    FK_TRY(plan_gemv(rq, &l));
    return run_launch(l, (hipStream_t)s);
}

static float theta_log2(float theta) { return (float)log2((double)theta); }

fk_status fk_rope_q_decode(uint16_t* q, const uint16_t* q_norm, uint32_t n_heads, uint32_t head_dim,
                           uint32_t rope_dims, float theta, float eps, const uint32_t* d_offset, uint32_t offset,
                           fk_stream s) {
    RopeArgs a;
    memset(&a, 0, sizeof(a));
    a.q = q; a.q_norm = q_norm;
    a.n_q = n_heads; a.head_dim = head_dim; a.rope_dims = rope_dims;
    a.offset_ptr = d_offset; a.offset_imm = offset;
    a.eps = eps; a.base_log2 = theta_log2(theta);
    a.rope_on = rope_dims ? 1u : 0u;
    a.capacity = 1;
    Launch l;
    FK_TRY(plan_rope_store(a, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_rope_kv_cache_store_decode(const uint16_t* k, const uint16_t* v, const uint16_t* k_norm, uint32_t n_kv,
                                        uint32_t k_dim, uint32_t v_dim, uint32_t rope_dims, float theta, float eps,
                                        const uint32_t* d_offset, uint32_t offset, const uint32_t* d_write_offset,
                                        uint32_t write_offset, uint32_t capacity, uint16_t* cache_k,
                                        uint16_t* cache_v, fk_stream s) {
    RopeArgs a;
    memset(&a, 0, sizeof(a));
    a.k = k; a.v = v; a.k_norm = k_norm;
    a.n_kv = n_kv; a.k_dim = k_dim; a.v_dim = v_dim; a.rope_dims = rope_dims;
    a.offset_ptr = d_offset; a.offset_imm = offset;
    a.write_offset_ptr = d_write_offset; a.write_offset_imm = write_offset; a.use_write_imm = 1;
    a.capacity = capacity;
    a.cache_k = cache_k; a.cache_v = cache_v;
    a.eps = eps; a.base_log2 = theta_log2(theta);
    a.rope_on = rope_dims ? 1u : 0u;
    Launch l;
    FK_TRY(plan_rope_store(a, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_kv_cache_store_split_decode(uint16_t* q, uint32_t n_heads, uint32_t q0_dim, uint32_t q1_dim,
                                         const uint16_t* k0, uint32_t k0_stride, const uint16_t* k1, uint32_t k1_heads,
                                         const uint16_t* v, uint32_t v_stride, uint32_t n_kv, uint32_t k0_dim,
                                         uint32_t k1_dim, uint32_t v_dim, uint32_t rope_dims, int traditional,
                                         float theta, const uint32_t* d_offset, uint32_t offset,
                                         const uint32_t* d_write_offset, uint32_t write_offset, uint32_t capacity,
                                         uint16_t* cache_k, uint16_t* cache_v, fk_stream s) {
    SplitStoreArgs a;
    memset(&a, 0, sizeof(a));
    a.q = q; a.n_heads = n_heads; a.q0_dim = q0_dim; a.q1_dim = q1_dim;
    a.k0 = k0; a.k0_stride = k0_stride; a.k1 = k1; a.k1_heads = k1_heads; a.v = v; a.v_stride = v_stride;
    a.n_kv = n_kv; a.k0_dim = k0_dim; a.k1_dim = k1_dim; a.v_dim = v_dim;
    a.rope_dims = rope_dims; a.traditional = traditional ? 1u : 0u;
    a.base_log2 = rope_dims ? theta_log2(theta) : 0.f;
    a.offset_ptr = d_offset; a.offset_imm = offset;
    a.write_offset_ptr = d_write_offset; a.write_offset_imm = write_offset; a.use_write_imm = 1;
    a.capacity = capacity;
    a.cache_k = cache_k; a.cache_v = cache_v;
    Launch l;
    FK_TRY(plan_split_rope_store(a, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_kv_cache_store_split_rows(uint16_t* q, uint32_t n_heads, uint32_t q0_dim, uint32_t q1_dim, const uint16_t* k0,
                                       uint32_t k0_stride, uint32_t k0_row_stride, const uint16_t* k1, uint32_t k1_heads,
                                       uint32_t k1_row_stride, const uint16_t* v, uint32_t v_stride, uint32_t v_row_stride,
                                       uint32_t n_kv, uint32_t k0_dim, uint32_t k1_dim, uint32_t v_dim, uint32_t rope_dims,
                                       int traditional, float theta, uint32_t rows, uint32_t offset, uint32_t capacity,
                                       uint16_t* cache_k, uint16_t* cache_v, fk_stream s) {
    if (rows == 0) return set_error(FK_ERR_INVALID, "fk_kv_cache_store_split_rows: no rows");
    SplitStoreArgs a;
    memset(&a, 0, sizeof(a));
    a.q = q; a.n_heads = n_heads; a.q0_dim = q0_dim; a.q1_dim = q1_dim;
    a.k0 = k0; a.k0_stride = k0_stride; a.k1 = k1; a.k1_heads = k1_heads; a.v = v; a.v_stride = v_stride;
    a.n_kv = n_kv; a.k0_dim = k0_dim; a.k1_dim = k1_dim; a.v_dim = v_dim;
    a.rope_dims = rope_dims; a.traditional = traditional ? 1u : 0u;
    a.base_log2 = rope_dims ? theta_log2(theta) : 0.f;
    a.offset_imm = offset; a.write_offset_imm = offset; a.use_write_imm = 1;
    a.capacity = capacity;
    a.cache_k = cache_k; a.cache_v = cache_v;
    a.rows = rows; a.k0_row_stride = k0_row_stride; a.k1_row_stride = k1_row_stride; a.v_row_stride = v_row_stride;
    Launch l;
    FK_TRY(plan_split_rope_store(a, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_softmax_topk_route(const uint16_t* logits, const uint16_t* scale, int scale_per_route, uint32_t rows,
                                uint32_t row_n, uint32_t top_k, uint32_t* idx, uint16_t* weight, fk_stream s) {
    Launch l;
    FK_TRY(plan_softmax_topk_route(logits, scale, scale_per_route != 0, rows, row_n, top_k, idx, weight, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_moe_router(const uint16_t* x, const uint16_t* norm_w, float eps, const uint16_t* w, const uint16_t* scale,
                        uint32_t hidden, uint32_t experts, uint32_t top_k, uint16_t* xn, uint16_t* logits, uint32_t* idx,
                        uint16_t* weight, uint32_t* workspace, uint32_t rows, fk_stream s) {
    Launch l;
    FK_TRY(plan_moe_router(x, norm_w, eps, w, scale, hidden, experts, top_k, xn, logits, idx, weight, workspace, &l, rows));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_qkv_rope_store_decode(uint16_t* q, const uint16_t* k, const uint16_t* v, const uint16_t* q_norm,
                                   const uint16_t* k_norm, uint32_t n_heads, uint32_t n_kv, uint32_t head_dim,
                                   uint32_t rope_dims, float theta, float eps, const uint32_t* d_offset,
                                   uint32_t offset, uint32_t capacity, uint16_t* cache_k, uint16_t* cache_v,
                                   fk_stream s) {
    RopeArgs a;
    memset(&a, 0, sizeof(a));
    a.q = q; a.k = k; a.v = v; a.q_norm = q_norm; a.k_norm = k_norm;
    a.n_q = n_heads; a.n_kv = n_kv; a.head_dim = head_dim; a.k_dim = head_dim; a.v_dim = head_dim;
    a.rope_dims = rope_dims;
    a.offset_ptr = d_offset; a.offset_imm = offset;
    a.capacity = capacity;
    a.cache_k = cache_k; a.cache_v = cache_v;
    a.eps = eps; a.base_log2 = theta_log2(theta);
    a.rope_on = rope_dims ? 1u : 0u;
    Launch l;
    FK_TRY(plan_rope_store(a, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_kv_cache_store_quant(const uint16_t* k, const uint16_t* v, const uint16_t* k_norm, uint32_t n_kv,
                                  uint32_t head_dim, uint32_t rope_dims, float theta, float eps, const uint32_t* d_offset,
                                  uint32_t offset, uint32_t rows, uint32_t capacity, uint32_t bits, uint32_t group,
                                  const fk_kv_quant_cache* cache_k, const fk_kv_quant_cache* cache_v, fk_stream s) {
    if (!cache_k || !cache_v) return set_error(FK_ERR_INVALID, "fk_kv_cache_store_quant: null cache");
    KvQuantStore a;
    memset(&a, 0, sizeof(a));
    a.k = k; a.v = v; a.k_norm = k_norm;
    a.ck_packed = cache_k->packed; a.ck_scales = cache_k->scales; a.ck_biases = cache_k->biases;
    a.cv_packed = cache_v->packed; a.cv_scales = cache_v->scales; a.cv_biases = cache_v->biases;
    a.offset_ptr = d_offset; a.offset_imm = offset;
    a.n_kv = n_kv; a.dim = head_dim; a.rope_dims = rope_dims; a.capacity = capacity; a.bits = bits; a.group = group;
    a.rows = rows;
    a.eps = eps; a.base_log2 = theta_log2(theta);
    Launch l;
    FK_TRY(plan_kv_store_quant(a, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_kv_cache_dequant(const fk_kv_quant_cache* cache, uint32_t n_kv, uint32_t dim, uint32_t capacity, uint32_t bits,
                              uint32_t group, uint32_t rows, uint16_t* out, uint32_t out_capacity, fk_stream s) {
    if (!cache) return set_error(FK_ERR_INVALID, "fk_kv_cache_dequant: null cache");
    Launch l;
    FK_TRY(plan_kv_dequant(cache->packed, cache->scales, cache->biases, n_kv, dim, capacity, bits, group, rows, out, out_capacity, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_sdpa_decode_quant(const uint16_t* q, const fk_kv_quant_cache* cache_k, const fk_kv_quant_cache* cache_v,
                               uint16_t* out, const uint32_t* d_kv_len, uint32_t kv_len, uint32_t max_len, uint32_t rows,
                               uint32_t n_heads, uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim, uint32_t capacity,
                               uint32_t bits, uint32_t group, float scale, float* partials, uint32_t* counters,
                               fk_stream s) {
    if (!cache_k || !cache_v || !cache_k->packed || !cache_v->packed)
        return set_error(FK_ERR_INVALID, "fk_sdpa_decode_quant: null cache");
    KvQuant qz;
    qz.k_scales = cache_k->scales; qz.k_biases = cache_k->biases;
    qz.v_scales = cache_v->scales; qz.v_biases = cache_v->biases;
    qz.bits = bits; qz.group = group;
    if (bits != 4 && bits != 8) return set_error(FK_ERR_UNSUPPORTED, "fk_sdpa_decode_quant: bits must be 4 or 8");
    Launch l;
    FK_TRY(plan_sdpa_decode(q, reinterpret_cast<const uint16_t*>(cache_k->packed),
                            reinterpret_cast<const uint16_t*>(cache_v->packed), out, d_kv_len, kv_len, max_len, n_heads,
                            n_kv, qk_dim, v_dim, capacity, scale, partials, counters, &l, rows ? rows : 1, &qz));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_rmsnorm_rows(const uint16_t* x, const uint16_t* w, float eps, uint32_t rows, uint32_t hidden, uint16_t* y,
                          fk_stream s) {
    Launch l;
    FK_TRY(plan_rmsnorm_rows(x, w, eps, rows, hidden, y, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_embed_lookup_rows(const fk_weight* E, const uint32_t* d_tokens, uint32_t rows, float out_scale, uint16_t* x,
                               fk_stream s) {
    if (!d_tokens) return set_error(FK_ERR_INVALID, "fk_embed_lookup_rows: null token array");
    Launch l;
    FK_TRY(plan_embed(E, d_tokens, 0, out_scale, x, &l, rows));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_qkv_rope_store_rows(uint16_t* q, const uint16_t* k, const uint16_t* v, const uint16_t* q_norm,
                                 const uint16_t* k_norm, uint32_t n_heads, uint32_t n_kv, uint32_t head_dim,
                                 uint32_t rope_dims, float theta, float eps, uint32_t rows, uint32_t offset,
                                 uint32_t capacity, uint16_t* cache_k, uint16_t* cache_v, const float* rope_tab,
                                 fk_stream s) {
    if (rows == 0) return set_error(FK_ERR_INVALID, "fk_qkv_rope_store_rows: zero rows");
    RopeArgs a;
    memset(&a, 0, sizeof(a));
    a.q = q; a.k = k; a.v = v; a.q_norm = q_norm; a.k_norm = k_norm;
    a.n_q = n_heads; a.n_kv = n_kv; a.head_dim = head_dim; a.k_dim = head_dim; a.v_dim = head_dim;
    a.rope_dims = rope_dims;
    a.offset_imm = offset;
    a.capacity = capacity;
    a.cache_k = cache_k; a.cache_v = cache_v;
    a.eps = eps; a.base_log2 = theta_log2(theta);
    a.rope_on = rope_dims ? 1u : 0u;
    a.rows = rows;
    a.rope_tab = rope_dims ? rope_tab : nullptr;
    Launch l;
    FK_TRY(plan_rope_store(a, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_rope_table_rows(float* tab, uint32_t rope_dims, float theta, uint32_t offset, uint32_t rows, fk_stream s) {
    Launch l;
    FK_TRY(plan_rope_table(tab, rope_dims, theta_log2(theta), offset, rows, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_sdpa_decode_rows(const uint16_t* q, const uint16_t* cache_k, const uint16_t* cache_v, uint16_t* out,
                              uint32_t rows, uint32_t kv_len, uint32_t n_heads, uint32_t n_kv, uint32_t qk_dim,
                              uint32_t v_dim, uint32_t capacity, float scale, float* partials, uint32_t* counters,
                              fk_stream s) {
    if (rows == 0 || kv_len == 0) return set_error(FK_ERR_INVALID, "fk_sdpa_decode_rows: zero rows or kv length");
    Launch l;
    FK_TRY(plan_sdpa_decode(q, cache_k, cache_v, out, nullptr, kv_len, kv_len + rows - 1, n_heads, n_kv, qk_dim, v_dim,
                            capacity, scale, partials, counters, &l, rows));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_sdpa_prefill(const uint16_t* q, const uint16_t* cache_k, const uint16_t* cache_v, uint16_t* out,
                          uint32_t rows, uint32_t kv_len, uint32_t n_heads, uint32_t n_kv, uint32_t head_dim,
                          uint32_t capacity, float scale, fk_stream s) {
    Launch l;
    FK_TRY(plan_sdpa_prefill(q, cache_k, cache_v, out, rows, kv_len, n_heads, n_kv, head_dim, capacity, scale, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_sdpa_workspace_bytes(uint32_t n_heads, uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim, uint32_t max_len,
                                  size_t* partial_bytes, size_t* counter_bytes) {
    if (!partial_bytes || !counter_bytes || max_len == 0 || qk_dim < 8 || v_dim < 8)
        return set_error(FK_ERR_INVALID, "sdpa workspace: bad argument");
    return sdpa_workspace_bytes(n_heads, n_kv, qk_dim, v_dim, max_len, partial_bytes, counter_bytes);
}

fk_status fk_sdpa_decode(const uint16_t* q, const uint16_t* cache_k, const uint16_t* cache_v, uint16_t* out,
                         const uint32_t* d_kv_len, uint32_t kv_len, uint32_t max_len, uint32_t n_heads,
                         uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim, uint32_t capacity, float scale,
                         float* partials, uint32_t* counters, fk_stream s) {
    Launch l;
    FK_TRY(plan_sdpa_decode(q, cache_k, cache_v, out, d_kv_len, kv_len, max_len, n_heads, n_kv, qk_dim, v_dim,
                            capacity, scale, partials, counters, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_embed_lookup_decode(const fk_weight* E, const uint32_t* d_token, uint32_t token, float out_scale,
                                 uint16_t* x, fk_stream s) {
    Launch l;
    FK_TRY(plan_embed(E, d_token, token, out_scale, x, &l));
    return run_launch(l, (hipStream_t)s);
}

static_assert(FK_ARGMAX_WORKSPACE_BYTES == kArgmaxWorkspaceBytes, "header and kernel disagree");

fk_status fk_argmax_logits_decode(const uint16_t* logits, uint32_t n, uint32_t* next_token, uint32_t* history,
                                  uint32_t* hist_counter, uint32_t hist_capacity, void* workspace, fk_stream s) {
    Launch l;
    FK_TRY(plan_argmax(logits, n, next_token, history, hist_counter, hist_capacity, workspace, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_step_init(uint32_t* step_counter, uint32_t* offset, uint32_t* kv_len, fk_stream s) {
    Launch l;
    FK_TRY(plan_step_init(step_counter, offset, kv_len, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_step_init_rope(uint32_t* step_counter, uint32_t* offset, uint32_t* kv_len, float* rope_tab,
                            uint32_t rope_dims, float theta, fk_stream s) {
    if (!rope_tab) return set_error(FK_ERR_INVALID, "fk_step_init_rope: null table");
    Launch l;
    FK_TRY(plan_step_init(step_counter, offset, kv_len, &l, rope_tab, rope_dims, theta_log2(theta)));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_rope_store_sdpa_decode(const uint16_t* q, const uint16_t* k, const uint16_t* v, const uint16_t* q_norm,
                                    const uint16_t* k_norm, uint16_t* cache_k, uint16_t* cache_v, uint16_t* out,
                                    const uint32_t* d_kv_len, uint32_t kv_len, uint32_t max_len, uint32_t n_heads,
                                    uint32_t n_kv, uint32_t head_dim, uint32_t rope_dims, float theta, float eps,
                                    uint32_t capacity, float scale, const float* rope_tab, float* partials,
                                    uint32_t* counters, fk_stream s) {
    SdpaFusion f;
    f.k_new = k; f.v_new = v; f.q_norm = q_norm; f.k_norm = k_norm;
    f.rope_dims = rope_dims; f.eps = eps; f.base_log2 = theta_log2(theta); f.rope_tab = rope_tab;
    Launch l;
    FK_TRY(plan_sdpa_decode(q, cache_k, cache_v, out, d_kv_len, kv_len, max_len, n_heads, n_kv, head_dim, head_dim,
                            capacity, scale, partials, counters, &l, 1, nullptr, &f));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_split_store_sdpa_decode(const uint16_t* q, uint32_t n_heads, uint32_t q0_dim, uint32_t q1_dim,
                                     const uint16_t* k0, uint32_t k0_stride, const uint16_t* k1, uint32_t k1_heads,
                                     const uint16_t* v, uint32_t v_stride, uint32_t n_kv, uint32_t v_dim, uint32_t rope_dims,
                                     int traditional, float theta, const float* rope_tab, uint16_t* cache_k,
                                     uint16_t* cache_v, uint16_t* out, const uint32_t* d_kv_len, uint32_t kv_len,
                                     uint32_t max_len, uint32_t capacity, float scale, float* partials, uint32_t* counters,
                                     fk_stream s) {
    SdpaFusion f;
    f.k_new = k0; f.k1_new = k1; f.v_new = v;
    f.q0_dim = q0_dim; f.k0_stride = k0_stride; f.v_stride = v_stride; f.k1_heads = k1_heads;
    f.traditional = traditional ? 1u : 0u;
    f.rope_dims = rope_dims; f.base_log2 = rope_dims ? theta_log2(theta) : 0.f; f.rope_tab = rope_tab;
    if (q0_dim == 0 || q1_dim == 0) return set_error(FK_ERR_INVALID, "fk_split_store_sdpa_decode: both head parts must be non-empty");
    Launch l;
    FK_TRY(plan_sdpa_decode(q, cache_k, cache_v, out, d_kv_len, kv_len, max_len, n_heads, n_kv, q0_dim + q1_dim, v_dim,
                            capacity, scale, partials, counters, &l, 1, nullptr, &f));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_copy(void* dst, const void* src, size_t nbytes, fk_stream s) {
    Launch l;
    FK_TRY(plan_copy(dst, src, nbytes, &l));
    return run_launch(l, (hipStream_t)s);
}

size_t fk_read_reduce_out_bytes(void) { return (size_t)256 * 8 * 8; }

fk_status fk_read_reduce(const void* src, size_t nbytes, void* out, size_t out_bytes, fk_stream s) {
    Launch l;
    FK_TRY(plan_read_reduce(src, nbytes, out, out_bytes, 0, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_fill_u32(void* dptr, uint32_t value, size_t count, fk_stream s) {
    Launch l;
    FK_TRY(plan_fill_u32(dptr, value, count, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_quantize_affine(const float* d_w, size_t n, size_t k, uint32_t bits, uint32_t group,
                             uint32_t* d_packed, uint16_t* d_scales, uint16_t* d_biases, fk_stream s) {
    Launch l;
    FK_TRY(plan_quantize(d_w, n, k, bits, group, d_packed, d_scales, d_biases, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_synth_fill(void* dptr, size_t count, uint64_t seed, float mean, float std, uint32_t kind, uint32_t bound,
                        fk_stream s) {
    Launch l;
    FK_TRY(plan_synth(dptr, count, seed, mean, std, kind, bound, &l));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_synth_fill_exact(void* dptr, size_t count, uint64_t seed, float mean, float std, uint32_t kind,
                              size_t row_len, float tau, size_t loud_rows, float loud_gain, fk_stream s) {
    if (kind != 3 && kind != 4) return set_error(FK_ERR_INVALID, "synth_fill_exact: kind must be 3 (fp32) or 4 (bf16)");
    Launch l;
    FK_TRY(plan_synth(dptr, count, seed, mean, std, kind, 0, &l, row_len, tau, loud_rows, loud_gain));
    return run_launch(l, (hipStream_t)s);
}

fk_status fk_xcd_layer_supported(uint32_t hidden, uint32_t inter, uint32_t n_heads, uint32_t n_kv, uint32_t head_dim,
                                 uint32_t capacity, uint32_t bits, uint32_t group) {
    return xcd_layer_supported(XcdLayerShape{hidden, inter, n_heads, n_kv, head_dim, capacity, bits, group});
}

fk_status fk_xcd_workspace_bytes(uint32_t n_heads, uint32_t head_dim, size_t* control_bytes, size_t* attention_partial_bytes) {
    if (!control_bytes || !attention_partial_bytes) return set_error(FK_ERR_INVALID, "fk_xcd_workspace_bytes: null out");
    XcdLayerShape s{};
    s.n_heads = n_heads;
    s.head_dim = head_dim;
    *control_bytes = xcd_workspace_bytes();
    *attention_partial_bytes = xcd_attn_partials_bytes(s);
    return FK_OK;
}

size_t fk_xcd_sum_row_bytes(uint32_t hidden) { return xcd_sum_row_bytes(hidden); }

fk_status fk_xcd_moe_supported(uint32_t hidden, uint32_t inter, uint32_t shared_inter, uint32_t experts, uint32_t top_k,
                               uint32_t bits, uint32_t group) {
    return xcd_moe_supported(XcdMoeShape{hidden, inter, shared_inter, experts, top_k, bits, group});
}

fk_status fk_xcd_mla_supported(uint32_t hidden, uint32_t n_heads, uint32_t rank, uint32_t rope_dim, uint32_t nope_dim,
                               uint32_t v_dim, uint32_t capacity, uint32_t bits, uint32_t group) {
    return xcd_mla_supported(XcdMlaShape{hidden, n_heads, rank, rope_dim, nope_dim, v_dim, capacity, bits, group});
}

fk_status fk_xcd_mla_workspace_bytes(uint32_t n_heads, uint32_t rank, uint32_t rope_dim, uint32_t v_dim, size_t* latent_bytes,
                                     size_t* attention_partial_bytes) {
    if (!latent_bytes || !attention_partial_bytes) return set_error(FK_ERR_INVALID, "fk_xcd_mla_workspace_bytes: null out");
    XcdMlaShape s{};
    s.n_heads = n_heads;
    s.rank = rank;
    s.rope_dim = rope_dim;
    s.v_dim = v_dim;
    *latent_bytes = xcd_mla_latent_bytes(s);
    *attention_partial_bytes = xcd_mla_partials_bytes(s);
    return FK_OK;
}

size_t fk_xcd_moe_scratch_bytes(uint32_t inter) {
    XcdMoeShape s{};
    s.inter = inter;
    return xcd_moe_scratch_bytes(s);
}

fk_status fk_xcd_kslice_meta(const uint16_t* src, uint32_t n, uint32_t groups, uint16_t* dst, fk_stream s) {
    return xcd_kslice_meta(src, n, groups, dst, (hipStream_t)s);
}

fk_status fk_xcd_check(void* workspace, fk_stream s) {
    if (!workspace) return set_error(FK_ERR_INVALID, "fk_xcd_check: null workspace");
    FK_HIP(hipStreamSynchronize((hipStream_t)s));
    return xcd_check_control(workspace);
}

}  // extern "C"
