// Host-side plumbing shared by the launch planners and the C ABI: the Launch
// descriptor every planner fills (so a kernel can be launched directly or added
// to a hipGraph as a kernel node), error reporting and cached device facts.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <string>
#include <vector>

#include "../../include/fusekit_hip.h"

namespace fk {

struct Launch {
    const void* func = nullptr;
    dim3 grid{1, 1, 1}, block{1, 1, 1};
    uint32_t shmem = 0;
    size_t args_size = 0;
    alignas(16) unsigned char args[896];
    // Kernels that complete the same operation and must run after this one, in
    // order (a split-k reduction, a routed reduction).  run_launch and the graph
    // builder treat the chain as one unit.
    std::vector<Launch> then;

    // Kernel parameters AHEAD of the argument block (at most kMaxLead, 8 bytes or less each): what a kernel needs for
    // its very first requests.  Leading scalar parameters can be handed to a wave in registers at its launch (kernel
    // argument preload), a by-value block cannot: its fields arrive with a load, one trip to memory into the kernel.
    static constexpr int kMaxLead = 4;
    uint32_t n_lead = 0;
    uint64_t lead[kMaxLead] = {0, 0, 0, 0};

    template <typename T>
    void set_args(const T& a) {
        static_assert(sizeof(T) <= sizeof(args), "argument block too large");
        memcpy(args, &a, sizeof(T));
        args_size = sizeof(T);
    }
    template <typename T>
    void add_lead(T v) {
        static_assert(sizeof(T) <= 8, "a leading parameter is a pointer or a scalar");
        uint64_t w = 0;
        memcpy(&w, &v, sizeof(T));
        lead[n_lead++] = w;
    }
    // The kernelParams array of this launch (kMaxLead + 1 entries at most); valid while the Launch is.
    void params(void** out) {
        for (uint32_t i = 0; i < n_lead; ++i) out[i] = &lead[i];
        out[n_lead] = args;
    }
};
constexpr int kMaxKernelParams = Launch::kMaxLead + 1;

struct DeviceFacts {
    int cus = 0;
    int max_dyn_lds = 0;
    hipDeviceProp_t prop;
};

// Fails with FK_ERR_HIP (message set) when no device is usable.
fk_status device_facts(const DeviceFacts** out);

fk_status set_error(fk_status code, const std::string& msg);
fk_status hip_error(hipError_t e, const char* what);
fk_status run_launch(const Launch& l, hipStream_t s);

#define FK_HIP(call)                                            \
    do {                                                        \
        hipError_t _e = (call);                                 \
        if (_e != hipSuccess) return ::fk::hip_error(_e, #call); \
    } while (0)

#define FK_TRY(call)                  \
    do {                              \
        fk_status _s = (call);        \
        if (_s != FK_OK) return _s;   \
    } while (0)

// ---- planners (one per kernel family); each validates shapes on the host ----
struct GemvPolicy {
    uint32_t rows_per_tile = 0, grid_blocks = 0;
    bool flat_only = false;  // never pick the row-group form
};
extern GemvPolicy g_gemv_policy;
// Column blocks per batch (3, 4 or 5) of the row-group GEMV form for one [n, k] matrix without bias or residual, or
// 0 when the shape stays on the flat form.
uint32_t gemv_rows_batch(uint32_t n, uint32_t k, uint32_t bits, uint32_t group);
// When non-zero, plan_gemv on this thread sizes its tiles for exactly this many
// blocks (the persistent whole-token kernel plans every phase for its own grid).
extern thread_local uint32_t t_gemv_grid_override;

// Greedy selection fused into the GEMV that produces the logits (row-group form only): the launch writes y as usual
// and also the index of its largest bf16 output, lowest index on ties, like plan_argmax.  `workspace` holds
// kHeadArgmaxWorkspaceBytes, zero before the first launch.
struct HeadArgmax {
    uint32_t* next_token = nullptr;
    uint32_t* history = nullptr;  // optional, with hist_counter: history[(*hist_counter)++] = token
    uint32_t* hist_counter = nullptr;
    uint32_t hist_capacity = 0;
    void* workspace = nullptr;
};
constexpr uint32_t kHeadArgmaxMaxBlocks = 4096;
constexpr size_t kHeadArgmaxWorkspaceBytes = 8 + 8 * (size_t)kHeadArgmaxMaxBlocks;

struct GemvRequest {
    const fk_weight* mats[3] = {nullptr, nullptr, nullptr};
    const uint16_t* bias[3] = {nullptr, nullptr, nullptr};
    uint16_t* y[3] = {nullptr, nullptr, nullptr};
    int n_mats = 1;
    bool swiglu = false;  // mats[0] = gate, mats[1] = up, y[0] = out
    int swiglu_variant = 0;
    const uint16_t* x = nullptr;
    const uint16_t* norm_w = nullptr;
    float eps = 0.f;
    const uint16_t* res = nullptr;
    const uint16_t* res2 = nullptr;
    const HeadArgmax* argmax = nullptr;  // FK_ERR_UNSUPPORTED when the shape does not take the row-group form
};
fk_status plan_gemv(const GemvRequest& rq, Launch* out);

// Mixture-of-experts routed projections (w_b non-null: gate/up pair with SwiGLU).
// Routing inside the routed launch (one token): logits bf16 [n_experts], one bf16 scale; the launch ranks them
// per wave and writes the chosen experts and weights (bf16 [n_routes]) for the kernels that follow.
struct RouteInKernel {
    const uint16_t* logits = nullptr;
    const uint16_t* scale = nullptr;
    uint32_t* idx_out = nullptr;
    uint16_t* weight_out = nullptr;
    bool apply_weight = false;   // multiply this launch's outputs by the route weight (else a later kernel does)
};
fk_status plan_routed_gemv(const uint16_t* x, uint32_t n_x_rows, const fk_weight* w_a, const fk_weight* w_b,
                           uint32_t n_experts, const uint32_t* row_idx, const uint32_t* expert_idx,
                           const uint16_t* route_weight, uint32_t n_routes, uint16_t* y, Launch* out,
                           const fk_weight* sh_a = nullptr, const fk_weight* sh_b = nullptr, uint16_t* sh_y = nullptr,
                           const RouteInKernel* rk = nullptr, const uint32_t* order = nullptr);
// order[position] = route: the routes sorted by expert (stable), for the `order` argument of the routed launches.
// kOrderInKernel in place of an array: every wave of the launch ranks the routes itself (up to 64 routes); the value
// is a tag and is never dereferenced.
static const uint32_t* const kOrderInKernel = reinterpret_cast<const uint32_t*>(uintptr_t(1));
fk_status plan_route_order(const uint32_t* expert_idx, uint32_t n_routes, uint32_t n_experts, uint32_t* order, Launch* out);
// Routed down projection + weighted reduction (+ shared expert + residual): one fused launch for one token
// of int4 weights, else routed GEMV -> shared GEMV -> ordered reduction chained in out->then (`parts`,
// (routes + tokens) * O bf16, is only touched by the chain).
fk_status plan_routed_reduce_chain(const uint16_t* h, uint32_t n_h_rows, const fk_weight* Wd, uint32_t n_experts,
                                   const uint32_t* row_idx, const uint32_t* expert_idx, const uint16_t* route_weight,
                                   const uint16_t* shared_x, const fk_weight* W_shared, const uint16_t* residual,
                                   uint32_t n_tokens, uint32_t top_k, uint16_t* out_ptr, uint16_t* parts, Launch* out,
                                   const uint32_t* order = nullptr);
void set_routed_fused_reduce(bool on);
// partial rows ((routes + tokens) * O bf16, rounded up to 256 bytes); with a shared expert and several tokens
// the multi-row matmul's workspace follows them
size_t routed_parts_bytes(uint32_t n_tokens, uint32_t top_k, uint32_t out_dim);
size_t routed_reduce_workspace_bytes(uint32_t n_tokens, uint32_t top_k, uint32_t out_dim, uint32_t shared_k, uint32_t group);
fk_status plan_route_reduce(const uint16_t* parts, const uint16_t* route_weight, const uint16_t* residual,
                            uint16_t* out_ptr, uint32_t n_tokens, uint32_t top_k, uint32_t O, bool has_shared,
                            Launch* out);

// Multi-row quantised matmul on the matrix cores (main kernel(s) + split-k reduction).
fk_status qgemm_workspace_bytes(uint32_t M, uint32_t N, uint32_t K, uint32_t group, size_t* bytes);
fk_status plan_qgemm(const fk_weight* W, const uint16_t* x, uint32_t M, const uint16_t* bias, const uint16_t* res,
                     uint16_t* y, void* workspace, Launch* main, Launch* reduce);
fk_status plan_qgemm_fanout(const fk_weight* const* W, uint32_t n_mats, const uint16_t* x, uint32_t M,
                            const uint16_t* const* bias, uint16_t* const* y, void* workspace, Launch* main, Launch* reduce,
                            bool* fused);
fk_status plan_qgemm_swiglu(const fk_weight* Wg, const fk_weight* Wu, const uint16_t* x, uint32_t M, int variant,
                            uint16_t* out, void* workspace, Launch* gate, Launch* up, Launch* reduce);

// Large row counts, direct calls only: dequantise to bf16 once, library GEMM, the same epilogue.
void set_gemm_library_rows(uint32_t rows);  // 0: never
fk_status run_dequantize_bf16(const fk_weight* W, uint16_t* out, hipStream_t s);
bool qgemm_takes_library(uint32_t m);
// 2..10 activation rows at group size 64 run the shared-stream kernel (qgemm_wide.hip): one launch, epilogue
// included.  plan_qgemm / plan_qgemm_swiglu then leave their other launches empty (func == nullptr), which
// run_launch and the graph builder skip.
bool qgemm_takes_wide(uint32_t M, uint32_t group);
void set_qgemm_wide(bool on);
struct WideSeg {
    const fk_weight* W;
    uint16_t* y;
    uint32_t y_stride;   // elements between the rows of y
};
fk_status plan_qgemm_wide_fan(const uint16_t* x, uint32_t x_stride, uint32_t M, const uint16_t* norm_w, float eps,
                              const WideSeg* segs, uint32_t n_seg, Launch* out);
fk_status plan_qgemm_wide(const fk_weight* W0, const fk_weight* W1, const uint16_t* x, uint32_t M, const uint16_t* bias,
                          const uint16_t* res, int variant, uint16_t* y, Launch* out, const uint16_t* norm_w = nullptr,
                          float eps = 0.f);
bool gemm_library_available();
size_t qgemm_library_sums_bytes(uint32_t m, uint32_t n, uint32_t k);
size_t qgemm_library_workspace_bytes(uint32_t m, uint32_t n, uint32_t k);
void plan_qgemm_epilogue(const float* p0, const float* p1, const uint16_t* bias, const uint16_t* res, uint16_t* y,
                         uint32_t M, uint32_t N, uint32_t ksplit, int variant, Launch* out);
fk_status run_qgemm_library(const fk_weight* W0, const fk_weight* W1, const uint16_t* x, uint32_t m, const uint16_t* bias,
                            const uint16_t* res, int variant, uint16_t* y, void* workspace, hipStream_t s);

// RoPE / per-head RMSNorm / KV-cache store (one wave per head).
struct RopeArgs {
    uint16_t* q;             // [n_q, head_dim] in place, or null
    const uint16_t* k;       // [n_kv, k_dim] or null
    const uint16_t* v;       // [n_kv, v_dim] or null
    const uint16_t* q_norm;  // [head_dim] or null
    const uint16_t* k_norm;  // [k_dim] or null
    uint16_t* cache_k;       // [n_kv, capacity, k_dim]
    uint16_t* cache_v;       // [n_kv, capacity, v_dim]
    const uint32_t* offset_ptr;        // rotary position (device) or null -> offset_imm
    const uint32_t* write_offset_ptr;  // cache row before the modulo, or null
    uint32_t offset_imm, write_offset_imm;
    uint32_t use_write_imm;  // with a null write_offset_ptr: 1 = write_offset_imm, 0 = same as offset
    uint32_t n_q, n_kv, head_dim, k_dim, v_dim, rope_dims, capacity;
    float eps, base_log2;
    uint32_t rope_on;  // 0: plain store of K (no rotation)
    uint32_t rows;     // active token rows (0 = 1): row r is position offset + r and reads q/k/v row r
    const float* rope_tab;  // optional [rows][rope_dims/2] (cos, sin) as plan_rope_table fills it, for position offset + r
};
fk_status plan_rope_store(const RopeArgs& in, Launch* out);
// (cos, sin) of every rotary pair at positions offset .. offset + rows - 1: the values the
// rope/store kernel would compute itself, filled once per prompt pass for all layers and heads.
fk_status plan_rope_table(float* tab, uint32_t rope_dims, float base_log2, uint32_t offset, uint32_t rows, Launch* out);

// Cache store of a key given as two parts [K0 | K1] with K1 rotated while written, plus the same
// rotation of the query's second part in place (mla.hip).
struct SplitStoreArgs {
    uint16_t* q;             // packed [n_heads, q0_dim + q1_dim]; Q1 rotated in place; null with n_heads = 0
    const uint16_t* k0;      // n_kv rows of k0_dim, k0_stride elements apart
    const uint16_t* k1;      // [k1_heads, k1_dim], k1_heads = 1 (shared) or n_kv
    const uint16_t* v;       // n_kv rows of v_dim, v_stride elements apart
    uint16_t* cache_k;       // [n_kv, capacity, k0_dim + k1_dim]
    uint16_t* cache_v;       // [n_kv, capacity, v_dim]
    const uint32_t* offset_ptr;        // rotary position (device) or null -> offset_imm
    const uint32_t* write_offset_ptr;  // cache row before the modulo, or null
    uint32_t offset_imm, write_offset_imm;
    uint32_t use_write_imm;  // with a null write_offset_ptr: 1 = write_offset_imm, 0 = the position
    uint32_t n_heads, q0_dim, q1_dim;
    uint32_t n_kv, k0_dim, k1_dim, v_dim, k0_stride, v_stride, k1_heads;
    uint32_t rope_dims, traditional, capacity;
    float base_log2;
    // several active token rows (0 = 1): row r is position offset + r; its q row follows the previous one, its
    // K0 / K1 / V rows start k0_row_stride / k1_row_stride / v_row_stride elements after the previous row's
    uint32_t rows, k0_row_stride, k1_row_stride, v_row_stride;
};
fk_status plan_split_rope_store(const SplitStoreArgs& a, Launch* out);
fk_status plan_softmax_topk_route(const uint16_t* logits, const uint16_t* scale, bool scale_per_route, uint32_t rows,
                                  uint32_t row_n, uint32_t top_k, uint32_t* idx, uint16_t* weight, Launch* out);

// RMSNorm + router projection (bf16 [experts, hidden]) + softmax top-k route in one launch; xn (normalised
// row) and logits are optional outputs; workspace: (experts + 1) words, zero before the first launch.
fk_status plan_moe_router(const uint16_t* x, const uint16_t* norm_w, float eps, const uint16_t* w, const uint16_t* scale,
                          uint32_t hidden, uint32_t experts, uint32_t top_k, uint16_t* xn, uint16_t* logits, uint32_t* idx,
                          uint16_t* weight, uint32_t* workspace, Launch* out, uint32_t rows = 1);

// Quantised KV cache (mlx-lm QuantizedKVCache layout): packed uint32 [n_kv, capacity, dim*bits/32],
// scales / biases bf16 [n_kv, capacity, dim/group].
struct KvQuant {
    const uint16_t* k_scales = nullptr;
    const uint16_t* k_biases = nullptr;
    const uint16_t* v_scales = nullptr;
    const uint16_t* v_biases = nullptr;
    uint32_t bits = 0, group = 64;  // bits 0: plain bf16 cache
};
struct KvQuantStore {
    const uint16_t* k;       // [rows, n_kv, dim] raw projection output
    const uint16_t* v;
    const uint16_t* k_norm;  // [dim] or null
    uint32_t* ck_packed; uint16_t* ck_scales; uint16_t* ck_biases;
    uint32_t* cv_packed; uint16_t* cv_scales; uint16_t* cv_biases;
    const uint32_t* offset_ptr;        // position of row 0 (device) or null -> offset_imm
    const uint32_t* write_offset_ptr;  // cache row of row 0 before the modulo, or null -> the position
    uint32_t offset_imm;
    uint32_t n_kv, dim, rope_dims, capacity, bits, group, rows;
    float eps, base_log2;
};
fk_status plan_kv_store_quant(const KvQuantStore& in, Launch* out);
// rows [0, rows) of a quantised cache as bf16 [n_kv, out_capacity, dim] (operand of the prefill attention)
fk_status plan_kv_dequant(const uint32_t* packed, const uint16_t* scales, const uint16_t* biases, uint32_t n_kv, uint32_t dim,
                          uint32_t capacity, uint32_t bits, uint32_t group, uint32_t rows, uint16_t* out, uint32_t out_capacity,
                          Launch* l);
// RoPE (+ head norm) of q and the new k row, the cache append and the attention in one launch:
// q / k_new / v_new are the raw projection outputs; the cache pointers of plan_sdpa_decode are
// the cache the rows are appended to.
struct SdpaFusion {
    const uint16_t* k_new = nullptr;
    const uint16_t* v_new = nullptr;
    const uint16_t* q_norm = nullptr;  // [qk_dim] or null
    const uint16_t* k_norm = nullptr;
    uint32_t rope_dims = 0;
    float eps = 1e-6f, base_log2 = 0.f;
    const float* rope_tab = nullptr;   // (cos, sin) per pair at this token's position, or null
    // heads as two parts (q0_dim != 0): q = [Q0 | Q1], new key = [k_new rows k0_stride apart | k1_new], rope_dims
    // counted from the start of the second part, v_new rows v_stride apart; no head norm
    const uint16_t* k1_new = nullptr;
    uint32_t q0_dim = 0, k0_stride = 0, v_stride = 0, k1_heads = 1, traditional = 0;
};
uint32_t sdpa_chunk_len(uint32_t qk_dim, uint32_t v_dim, bool fused);
fk_status sdpa_workspace_bytes(uint32_t n_heads, uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim, uint32_t max_len,
                               size_t* partial_bytes, size_t* counter_bytes);
fk_status plan_sdpa_decode(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint16_t* out,
                           const uint32_t* kv_len_ptr, uint32_t kv_len_imm, uint32_t max_len, uint32_t n_heads,
                           uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim, uint32_t capacity, float scale,
                           float* partials, uint32_t* counters, Launch* out_launch, uint32_t rows = 1,
                           const KvQuant* quant = nullptr, const SdpaFusion* fusion = nullptr);
// Causal attention of a group of rows on the matrix cores (head dimension 64 or 128, bf16 cache):
// kv_len counts the rows of the group, row r sees the first kv_len - rows + r + 1 positions.  With
// kv_len_ptr the count is read on the device at run time (clamped to rows .. capacity).
fk_status plan_sdpa_prefill(const uint16_t* q, const uint16_t* cache_k, const uint16_t* cache_v, uint16_t* out,
                            uint32_t rows, uint32_t kv_len, uint32_t n_heads, uint32_t n_kv, uint32_t head_dim,
                            uint32_t capacity, float scale, Launch* out_launch, const uint32_t* kv_len_ptr = nullptr);
fk_status plan_embed(const fk_weight* E, const uint32_t* token_ptr, uint32_t token_imm, float out_scale,
                     uint16_t* x, Launch* out, uint32_t rows = 1);
fk_status plan_rmsnorm_rows(const uint16_t* x, const uint16_t* w, float eps, uint32_t rows, uint32_t hidden, uint16_t* y,
                            Launch* out);
// workspace: 8 bytes (counter, zeroed once) + 8 bytes per block (<= 160 blocks)
constexpr size_t kArgmaxWorkspaceBytes = 8 + 8 * 160;
fk_status plan_argmax(const uint16_t* logits, uint32_t n, uint32_t* next_token, uint32_t* history,
                      uint32_t* hist_counter, uint32_t hist_capacity, void* workspace, Launch* out);
fk_status plan_step_init(uint32_t* step_counter, uint32_t* offset, uint32_t* kv_len, Launch* out,
                         float* rope_tab = nullptr, uint32_t rope_dims = 0, float base_log2 = 0.f);
fk_status plan_fill_u32(void* p, uint32_t value, size_t count, Launch* out);
fk_status plan_copy(void* dst, const void* src, size_t nbytes, Launch* out);
fk_status plan_read_reduce(const void* src, size_t nbytes, void* out, size_t out_bytes, uint32_t blocks_per_cu, Launch* l);
fk_status plan_quantize(const float* w, size_t n, size_t k, uint32_t bits, uint32_t group, uint32_t* packed,
                        uint16_t* scales, uint16_t* biases, Launch* out);
fk_status plan_synth(void* out_ptr, size_t count, uint64_t seed, float mean, float std, uint32_t kind, uint32_t bound,
                     Launch* out, uint64_t row_len = 0, float tau = 0.f, uint64_t loud_rows = 0, float loud_gain = 1.f);

}  // namespace fk
