/*
 * fusekit_hip.h -- C ABI of the MI355X (gfx950) decode backend for FuseKit.
 *
 * This is the boundary a FuseKit maintainer binds from Rust (`extern "C"` in an
 * FFI crate) in place of the Metal runtime.  Two groups of entry points:
 *
 *  1. Operator launches: one per hot-path FusionKind.  Plain device pointers,
 *     sizes and a HIP stream (NULL = default stream).  Each replaces the Metal
 *     kernel text one reference emitter produces; the emitter is cited.
 *  2. Dispatcher: the replacement of the pyo3 module
 *     `_fusekit_runtime_native` (reference python_runtime/src/lib.rs:1939-1971):
 *     device allocations, named dispatch, hipGraph build / update / replay and
 *     the native per-token decode loop.
 *
 * Conventions: every call returns fk_status (0 = ok); fk_last_error() gives the
 * message of the last failure on the calling thread.  Activations are bfloat16
 * bit patterns (uint16_t).  All pointers named d_* or documented "device" must
 * be device memory; the library never dereferences them on the host.  Nothing
 * here falls back to a CPU path: without a HIP device every compute call fails
 * with FK_ERR_HIP.
 */
#ifndef FUSEKIT_HIP_H
#define FUSEKIT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

typedef int fk_status;
enum {
    FK_OK = 0,
    FK_ERR_INVALID = 1,     /* bad handle / id / range / name / null buffer (PyValueError in lib.rs:1977-1985) */
    FK_ERR_IO = 2,          /* PyIOError */
    FK_ERR_NOT_FOUND = 3,   /* PyFileNotFoundError */
    FK_ERR_HIP = 4,         /* a HIP runtime call failed or no device */
    FK_ERR_UNSUPPORTED = 5  /* shape / option outside what the kernels admit */
};

typedef void *fk_stream; /* hipStream_t; NULL = default stream */

/* One [n, k] weight matrix.  bits 4 / 8: MLX-affine, `w` = packed uint32
 * [n, k*bits/32] (value j of a word at bit j*bits), scales/biases bf16
 * [n, k/group] (reference src/fusion/ir.rs:236-242).  bits 16: dense bf16
 * [n, k], scales/biases NULL, group ignored. */
typedef struct fk_weight {
    const void *w;
    const uint16_t *scales;
    const uint16_t *biases;
    uint32_t n, k;
    uint32_t bits, group;
} fk_weight;

const char *fk_last_error(void);
/* reference python_runtime/src/lib.rs:1880 `version` */
const char *fk_version(void);

/* ---- device memory (replaces alloc_uniform lib.rs:1658 and the no-copy wraps
 *      of unified memory lib.rs:417-427; MI355X has no unified memory) ---- */
typedef struct fk_device_props {
    char name[128];
    char arch[32];
    int compute_units;
    int wavefront;
    int lds_bytes_per_block;
    int l2_bytes;
    uint64_t hbm_bytes;
    int clock_khz;
} fk_device_props;

fk_status fk_device_props_get(fk_device_props *out);
/* Device memory (hipMalloc).  The reference's buffers carry a storage mode (shared / private); here every
 * buffer is device-private HBM and the host reaches it through fk_upload / fk_download only, so there is no
 * memory-kind argument. */
fk_status fk_alloc(size_t nbytes, void **dptr);
fk_status fk_free(void *dptr);
/* Free and total device memory in bytes (what `peak_gb` of the bench driver is taken from; scripts/bench.py:148). */
fk_status fk_mem_info(size_t *free_bytes, size_t *total_bytes);
fk_status fk_upload(void *dptr, const void *host, size_t nbytes);
fk_status fk_download(void *host, const void *dptr, size_t nbytes);
fk_status fk_fill_u32(void *dptr, uint32_t value, size_t count, fk_stream s);
/* Device-to-device copy by a plain kernel (pointers and size multiples of 16 bytes):
 * moves buffers inside a stream / graph and is the known-traffic kernel against
 * which hardware byte counters are calibrated. */
fk_status fk_copy(void *dst, const void *src, size_t nbytes, fk_stream s);
/* Measurement aid with no counterpart in the reference: reads nbytes (a multiple of 16, 16-byte aligned) with
 * plain 16-byte-per-lane loads (every workgroup walks its own contiguous span, 1 KiB per wave instruction, eight requests in flight per lane) and
 * keeps only the XOR of what it read, one 64-bit word per workgroup in `out` (fk_read_reduce_out_bytes() bytes).
 * Over a buffer larger than the 256 MB last-level cache its rate is what a read-only streaming kernel gets from
 * HBM on the device at hand: the bench prices the GEMVs against the published 8 TB/s and against this.  Also the
 * dispatch family `fusekit_read_reduce` (slots: src, out; parameter blocks_per_cu, default 4). */
fk_status fk_read_reduce(const void *src, size_t nbytes, void *out, size_t out_bytes, fk_stream s);
size_t fk_read_reduce_out_bytes(void);
fk_status fk_stream_create(fk_stream *out);
fk_status fk_stream_destroy(fk_stream s);
fk_status fk_stream_sync(fk_stream s);

/* GPU timing on the stream the work was launched on (hipEvent pairs); the
 * reference reports GPU seconds from command-buffer timestamps
 * (python_runtime/src/lib.rs:745-760). */
typedef void *fk_event;
fk_status fk_event_create(fk_event *out);
fk_status fk_event_destroy(fk_event e);
fk_status fk_event_record(fk_event e, fk_stream s);
fk_status fk_event_elapsed_ms(fk_event start, fk_event stop, float *ms); /* waits for `stop` */

/* ---- target description and launch geometry ---------------------------
 * T1  The gfx950 entry of the reference's ChipModel / Budgets table
 *     (src/target/mod.rs:17-200): what a code generator needs to know about the
 *     machine, plus the policy thresholds this library applies itself.  Without a
 *     visible GPU the published MI355X figures are returned and from_device is 0. */
typedef struct fk_target {
    char arch[32];                  /* "gfx950..." */
    uint32_t from_device;           /* 1: read from the running GPU, 0: published MI355X figures */
    uint32_t compute_units;         /* 256 */
    uint32_t xcds;                  /* 8 accelerator dies, one L2 each */
    uint32_t wave_size;             /* 64 (the reference's simd_width) */
    uint32_t simds_per_cu;          /* 4 */
    uint32_t vgprs_per_lane;        /* 512 per SIMD lane, shared by the resident waves (regs_per_thread budget) */
    uint32_t lds_bytes_per_cu;      /* 163840 (smem_per_threadgroup ceiling) */
    uint32_t workgroup_threads;     /* 256: threadgroup size every kernel here uses (4 waves) */
    uint32_t gemm_min_rows;         /* active rows from which the matrix-core path is taken (the reference: 8,
                                       src/target/mod.rs:162-171; here 2 -- one weight pass serves 32 rows) */
    uint32_t gemm_rows_per_pass;    /* 128: activation rows one block of the multi-row matmul serves */
    uint64_t hbm_bytes;
    double hbm_peak_bytes_per_s;    /* 8.0e12, published */
    double mfma_bf16_peak_flops;    /* 2.5e15 dense, published */
} fk_target;
fk_status fk_target_describe(fk_target *out);

/* (T2 fk_plan_geometry is declared with the dispatcher below.) */

/* ---- operator launches ------------------------------------------------ */

/* K1  y = T(x @ dequant(W)^T (+ bias)).  Replaces the qGEMV inner loop
 *     src/codegen/kernels/mod.rs:2553-3201 and fusekit_qmv_fast_impl
 *     src/codegen/msl.rs:310-440. */
fk_status fk_qgemv(const fk_weight *W, const uint16_t *x, const uint16_t *bias, uint16_t *y, fk_stream s);

/* K1r y = T(acc + res); with res2: T(float(y) + res2).  Replaces
 *     src/codegen/kernels/linear_residual.rs:17-388. */
fk_status fk_linear_residual(const fk_weight *W, const uint16_t *x, const uint16_t *res, const uint16_t *res2,
                             uint16_t *y, fk_stream s);

/* K2  RMSNorm -> Q,K,V projections (+ bf16 bias).  Replaces
 *     src/codegen/kernels/rmsnorm_qkv.rs:53-736 (non-sink variant).
 *     norm_w may be NULL: x is then consumed as is (QmvFanout,
 *     src/codegen/kernels/qmv_fanout.rs). */
fk_status fk_rmsnorm_qkv(const uint16_t *x, const uint16_t *norm_w, float eps, const fk_weight *Wq,
                         const fk_weight *Wk, const fk_weight *Wv, const uint16_t *bq, const uint16_t *bk,
                         const uint16_t *bv, uint16_t *q, uint16_t *k, uint16_t *v, fk_stream s);

/* K2 for 2..8 token rows (the reference compiles the same emitter with active_m = N for its prefill_mN variants,
 *     src/commands/patch.rs:112-150, src/codegen/kernels/rmsnorm_qkv.rs:53-736): x [rows, x_row_stride], outputs
 *     [rows, *_row_stride]; ONE launch streams the one to three matrices once for all rows (Wk, Wv may be NULL from
 *     the end; 4- or 8-bit, group 64, no bias) and applies the norm while the rows are staged (norm_w NULL: none).
 *     Row strides let the outputs be column blocks of a wider row.  Dispatch family fusekit_rmsnorm_qkv with the
 *     parameter rows (and x_row_stride, q_ / k_ / v_row_stride). */
fk_status fk_rmsnorm_qkv_rows(const uint16_t *x, uint32_t rows, uint32_t x_row_stride, const uint16_t *norm_w, float eps,
                              const fk_weight *Wq, const fk_weight *Wk, const fk_weight *Wv, uint16_t *q,
                              uint32_t q_row_stride, uint16_t *k, uint32_t k_row_stride, uint16_t *v, uint32_t v_row_stride,
                              fk_stream s);

/* K3a (RMSNorm ->) gate/up projections -> SwiGLU.  variant 0: every op in T
 *     (src/codegen/kernels/rmsnorm_gateup_swiglu.rs:236-257); 1: fp32 sigmoid,
 *     one round (src/codegen/msl.rs:1286-1294); 2: rounded sigmoid and gate
 *     (src/codegen/msl.rs:2441-2449).  norm_w NULL = QmvSwiglu
 *     (src/codegen/kernels/qmv_swiglu.rs:20-246). */
fk_status fk_gateup_swiglu(const uint16_t *x, const uint16_t *norm_w, float eps, const fk_weight *Wg,
                           const fk_weight *Wu, int variant, uint16_t *out, fk_stream s);
/* K3a for 2..8 token rows (the emitter compiled with active_m = N, src/codegen/kernels/rmsnorm_gateup_swiglu.rs:20-330,
 *     src/commands/patch.rs:112-150): x [rows, hidden], out [rows, inter]; ONE launch streams the pair once for all rows
 *     and applies the norm while the rows are staged (norm_w NULL: none); 4- or 8-bit, group 64.  Dispatch family
 *     fusekit_rmsnorm_gateup_swiglu with the parameter rows. */
fk_status fk_gateup_swiglu_rows(const uint16_t *x, uint32_t rows, const uint16_t *norm_w, float eps, const fk_weight *Wg,
                                const fk_weight *Wu, int variant, uint16_t *out, fk_stream s);

/* M1  routed gate/up + SwiGLU over expert-stacked weights.  Replaces
 *     src/codegen/kernels/routed_qmv_swiglu.rs:20-450 (slots x, gate w/s/b, up w/s/b,
 *     row_idx, expert_idx, [route_weight], out0).  Wg / Wu describe ONE expert's
 *     matrix [n, k]; their pointers are the bases of tensors stacked [E, n, ...].
 *     Route r reads activation row min(row_idx[r], n_x_rows-1) (row_idx NULL: row r)
 *     and expert min(expert_idx[r], n_experts-1);
 *     out0[r, o] = T(((sigmoid(g) * g) * u) * route_weight[r]) with g, u = T(acc)
 *     (route_weight NULL: factor 1). */
fk_status fk_routed_qmv_swiglu(const uint16_t *x, uint32_t n_x_rows, const fk_weight *Wg, const fk_weight *Wu,
                               uint32_t n_experts, const uint32_t *row_idx, const uint32_t *expert_idx,
                               const uint16_t *route_weight, uint32_t n_routes, uint16_t *out0, fk_stream s);
/* Several tokens whose routes share experts: `order` [n_routes] lists the routes in the order they are served
 * (fk_route_order: sorted by expert, stable).  Inputs, outputs and arithmetic per route are those of
 * fk_routed_qmv_swiglu (a route gets a multiple of eight blocks, so its tiles -- and the order in which a row's
 * partial sums are added -- may differ from the listed launch's: equal to rounding-edge flips); routes of one
 * expert sit next to each other in the grid and their blocks share an XCD, so an expert's slice is streamed
 * from HBM once instead of once per route (the
 * reference's kernels serve routes as listed, src/codegen/kernels/routed_qmv_swiglu.rs:104-160: row_idx /
 * expert_idx per route).  Dispatch families fusekit_routed_qmv_swiglu / fusekit_routed_qmv_reduce take the same
 * array as a last slot with the parameter has_order = 1; fusekit_route_order (slots expert_idx, order;
 * parameters routes, experts) writes it.  order = NULL (families: parameter expert_order = 1, no slot): up to 64
 * routes, every wave of the launch ranks the routes by (expert, route) itself -- the same order without an array
 * and without the launch that writes one (one graph node less per layer; more than 64 routes: FK_ERR_UNSUPPORTED). */
fk_status fk_route_order(const uint32_t *expert_idx, uint32_t n_routes, uint32_t n_experts, uint32_t *order, fk_stream s);
fk_status fk_routed_qmv_swiglu_ordered(const uint16_t *x, uint32_t n_x_rows, const fk_weight *Wg, const fk_weight *Wu,
                                       uint32_t n_experts, const uint32_t *row_idx, const uint32_t *expert_idx,
                                       const uint16_t *route_weight, uint32_t n_routes, const uint32_t *order,
                                       uint16_t *out0, fk_stream s);
/* fk_routed_qmv_reduce with the routed down projections served in `order` (several tokens); the weighted sums
 * stay in slot order per token (src/codegen/kernels/routed_qmv_reduce.rs:240, 315-322). */
fk_status fk_routed_qmv_reduce_ordered(const uint16_t *h, uint32_t n_h_rows, const fk_weight *Wd, uint32_t n_experts,
                                       const uint32_t *row_idx, const uint32_t *expert_idx, const uint16_t *route_weight,
                                       const uint16_t *shared_x, const fk_weight *W_shared, const uint16_t *residual_extra,
                                       uint32_t n_tokens, uint32_t top_k, const uint32_t *order, uint16_t *out,
                                       void *workspace, fk_stream s);
/* The same launch with the block's SHARED experts riding along (one token): Sg / Su [n_shared * O, K] are
 * read as n_shared further routes -- row block j into shared_out [j * O ..) -- unweighted, with the same SwiGLU
 * (the reference runs them as a separate qmv_swiglu launch, src/codegen/kernels/qmv_swiglu.rs:20-246; the
 * arithmetic per output is that kernel's).  Every route reads the one activation row x [K]. */
fk_status fk_routed_qmv_swiglu_shared(const uint16_t *x, const fk_weight *Wg, const fk_weight *Wu, uint32_t n_experts,
                                      const uint32_t *expert_idx, const uint16_t *route_weight, uint32_t n_routes,
                                      uint16_t *out0, const fk_weight *Sg, const fk_weight *Su, uint16_t *shared_out,
                                      fk_stream s);
/* The routed (and optionally shared: Sg / Su / shared_out, or all three NULL) gate/up launch ROUTING FOR ITSELF,
 * one token: instead of expert indices it takes the router logits (bf16 [n_experts]) and the bf16 scale; every
 * wave evaluates fk_softmax_topk_route's arithmetic on them and the block of route r serves the r-th winner.
 * idx_out u32 [top_k] / weight_out bf16 [top_k] are written for the kernels that follow (fk_routed_qmv_reduce);
 * apply_weight != 0 multiplies this launch's outputs by the route weight as route_weight does above.  With
 * fk_moe_router(top_k = 0), which then only publishes logits, no kernel of the block waits on another block. */
fk_status fk_routed_qmv_swiglu_routing(const uint16_t *x, const fk_weight *Wg, const fk_weight *Wu, uint32_t n_experts,
                                       const uint16_t *logits, const uint16_t *scale, uint32_t top_k, int apply_weight,
                                       uint32_t *idx_out, uint16_t *weight_out, uint16_t *out0, const fk_weight *Sg,
                                       const fk_weight *Su, uint16_t *shared_out, fk_stream s);

/* M2  routed down projection + weighted reduction (+ shared expert + residual).
 *     Replaces src/codegen/kernels/routed_qmv_reduce.rs:14-460.  h is [n_h_rows, k]
 *     (M1's out0); route r = tok * top_k + slot reads row min(row_idx[r], n_h_rows-1)
 *     (row_idx NULL: row r).  out[tok, o] = T(sum_slot rw * T(dot) [+ T(shared dot)]
 *     [+ residual_extra[tok, o]]) in slot order, fp32; route_weight NULL means the
 *     input was pre-weighted (rw = 1).  W_shared / shared_x (both or neither; then
 *     n_tokens must be 1, as routed_qmv_reduce.rs:80) add the shared expert's down
 *     projection of shared_x.  workspace: fk_routed_reduce_workspace_bytes() bytes. */
size_t fk_routed_reduce_workspace_bytes(uint32_t n_tokens, uint32_t top_k, uint32_t out_dim);
/* With a shared expert and SEVERAL tokens the shared rows go through the multi-row matmul, whose workspace
 * follows the partial rows: size the buffer with this query (shared_k = the shared expert's input width). */
size_t fk_routed_reduce_workspace_bytes_shared(uint32_t n_tokens, uint32_t top_k, uint32_t out_dim, uint32_t shared_k,
                                               uint32_t group);
fk_status fk_routed_qmv_reduce(const uint16_t *h, uint32_t n_h_rows, const fk_weight *Wd, uint32_t n_experts,
                               const uint32_t *row_idx, const uint32_t *expert_idx, const uint16_t *route_weight,
                               const uint16_t *shared_x, const fk_weight *W_shared, const uint16_t *residual_extra,
                               uint32_t n_tokens, uint32_t top_k, uint16_t *out, void *workspace, fk_stream s);
/* One token of int4 weights takes ONE launch (a wave per output row walks every route and the shared
 * expert and adds them in slot order; the workspace is then not touched); other shapes take three
 * (routed GEMV, shared GEMV, ordered reduction).  fk_set_routed_fused_reduce(0) forces the three. */
void fk_set_routed_fused_reduce(int on);

/* G   multi-row quantised matmul on the matrix cores: y[m, N] = T(x[m, K] @ dequant(W)^T
 *     (+ bias[N]) (+ residual[m, N])), fp32 accumulate, one round.  Replaces the
 *     reference's qMM-T / NAX tile path (src/codegen/msl.rs:2318-2440, 3821-4330;
 *     admission src/codegen/kernels/mod.rs:1442-1475) and its small-M shared-stream
 *     GEMVs (fusekit_qmv_wide_impl, src/codegen/msl.rs:461-546).  Any m >= 1; bits 4
 *     or 8, group 64 or 128; bits 16 (dense bf16 rows, k a multiple of 8): the plain
 *     library GEMM (rocBLAS) with the same epilogue, direct calls only.  workspace: fk_qgemm_workspace_bytes() bytes of device
 *     memory (fp32 split-k partial sums; from fk_set_gemm_library_rows() rows up the fp32
 *     sums and the matrix dequantised to bf16, N*K*2 bytes; group 0 = dense bf16 weights: the
 *     fp32 sums only); the SwiGLU pair needs twice that.
 *     fk_qgemm_swiglu: out[m, N] = SwiGLU(x @ Wg^T, x @ Wu^T) with the rounding variant
 *     as in fk_gateup_swiglu (the reference's qMM epilogue is variant 2,
 *     src/codegen/msl.rs:2441-2449). */
fk_status fk_qgemm_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, uint32_t group, size_t *bytes);
fk_status fk_qgemm(const fk_weight *W, const uint16_t *x, uint32_t m, const uint16_t *bias,
                   const uint16_t *residual, uint16_t *y, void *workspace, fk_stream s);
fk_status fk_qgemm_swiglu(const fk_weight *Wg, const fk_weight *Wu, const uint16_t *x, uint32_t m, int variant,
                          uint16_t *out, void *workspace, fk_stream s);
/*     fk_qgemm_fanout: one to three matrices over the SAME activation rows, y[i][m, N_i] = T(x @ W[i]^T (+ bias[i])) -- the
 *     q / k / v projections of a prompt pass, which the reference dispatches one after the other (qMM per projection,
 *     python/fusekit_runtime/dispatch.py prefill variants).  Same results as fk_qgemm per matrix (same kernel
 *     arithmetic).  From 65 rows, below the fk_set_gemm_library_rows() threshold, with equal K, bits and group size
 *     and every N_i a multiple of 4, the matrices run as ONE launch of the fused kernel whose blocks along N run
 *     through them in turn (the narrow k and v projections alone leave most of the device idle); otherwise the
 *     call is fk_qgemm per matrix.  bias: null or an array of n_mats pointers (each may be null).
 *     workspace: fk_qgemm_workspace_bytes(m, N_0 + N_1 + N_2, k, group) bytes. */
fk_status fk_qgemm_fanout(const fk_weight *const *W, uint32_t n_mats, const uint16_t *x, uint32_t m,
                          const uint16_t *const *bias, uint16_t *const *y, void *workspace, fk_stream s);

/* H   final RMSNorm + vocabulary GEMV, logits in T.  Replaces
 *     src/codegen/kernels/final_rmsnorm_lm_head.rs:144-629. */
fk_status fk_final_rmsnorm_lm_head(const uint16_t *x, const uint16_t *norm_w, float eps, const fk_weight *W,
                                   uint16_t *logits, fk_stream s);
/* H+A the same launch also selects the greedy token: next_token = index of the largest bf16 logit, lowest
 *     index on ties, NaN never wins, and optionally history[(*hist_counter)++] = token, exactly as
 *     fk_argmax_logits_decode over the logits it writes.  Replaces the reference's direct head
 *     (`<head kernel>_argmax` + `_argmax_finalize`, src/codegen/msl.rs:1674-1890, enabled per
 *     python/fusekit_runtime/dispatch.py:1846-1866 and bound at 3458-3505) -- as ONE launch whose last block
 *     finishes the selection; unlike the reference's form the logits are still written (300 KB beside a matrix
 *     of hundreds of MB).  Only for matrices that fk_gemv_form reports as row-group form; anything else
 *     FK_ERR_UNSUPPORTED (the caller keeps the two launches).  Workspace: FK_HEAD_ARGMAX_WORKSPACE_BYTES,
 *     zeroed once; launches that share a workspace must not overlap. */
#define FK_HEAD_ARGMAX_WORKSPACE_BYTES 32776
fk_status fk_final_rmsnorm_lm_head_argmax(const uint16_t *x, const uint16_t *norm_w, float eps, const fk_weight *W,
                                          uint16_t *logits, uint32_t *next_token, uint32_t *history,
                                          uint32_t *hist_counter, uint32_t hist_capacity, void *workspace,
                                          fk_stream s);

/* Q0  MLX-affine quantiser on the device: w fp32 [n, k] -> packed uint32
 *     [n, k*bits/32], scales / biases bf16 [n, k/group].  Arithmetic of the
 *     reference's restatement of mx.quantize,
 *     src/codegen/kernels/rope_kv_cache_store_decode_quant.rs:208-221; integer
 *     codes are bit-exact against the CPU statement of the same formula. */
fk_status fk_quantize_affine(const float *d_w, size_t n, size_t k, uint32_t bits, uint32_t group,
                             uint32_t *d_packed, uint16_t *d_scales, uint16_t *d_biases, fk_stream s);

/* Seeded synthetic data written straight into HBM (random-init models for
 * `fusekit bench` without a checkpoint): element i depends only on (seed, i).
 * kind 0: fp32 N(mean, std^2); 1: bf16 N(mean, std^2); 2: uint32 uniform in [0, bound). */
fk_status fk_synth_fill(void *dptr, size_t count, uint64_t seed, float mean, float std, uint32_t kind,
                        uint32_t bound, fk_stream s);
/* The same for values a host can reproduce bit for bit (parity tests build the very model on the
 * CPU): kind 3 fp32, kind 4 bf16; value = fma(std, z, mean) with z a sum of eight 16-bit uniform
 * integers, centred and scaled to unit variance (integer arithmetic and single IEEE operations
 * only).  With row_len and tau non-zero every row of row_len elements is multiplied by
 * (1 + (u & 7) / 8) * 2^(u >> 3), u = floor(8 * tau * z_row): row norms spread like a log-normal;
 * row j of the first loud_rows rows is multiplied by loud_gain * 2^-j instead.  Either gives a tied embedding / LM
 * head the peaked logits of a trained model (a random one is near-uniform over the vocabulary).  Like
 * fk_synth_fill this has no counterpart in the reference, which loads real checkpoints. */
fk_status fk_synth_fill_exact(void *dptr, size_t count, uint64_t seed, float mean, float std, uint32_t kind,
                              size_t row_len, float tau, size_t loud_rows, float loud_gain, fk_stream s);

/* Per-token scalars (rotary position, cache row, KV length) come either from a
 * device scalar `d_*` (so a captured hipGraph can be replayed while a step
 * kernel advances them, as the reference binds `layer_offset` / `layer_kv_len`
 * uniform buffers, src/codegen/kernels/mod.rs:5531-5577) or, when that pointer
 * is NULL, from the immediate value next to it. */

/* R   half-split RoPE on q [n_heads, head_dim] in place; pair (d, d+rope_dims/2),
 *     inv = exp2(-(d/half)*log2(theta)), angle = pos*inv.  Replaces
 *     src/codegen/kernels/rope_q_decode.rs:24-125.  q_norm != NULL first applies
 *     the per-head RMSNorm T(w*T(x*r)) (q side of
 *     src/codegen/kernels/rmsnorm_rope_qgate_decode.rs:84-136, without the gate). */
fk_status fk_rope_q_decode(uint16_t *q, const uint16_t *q_norm, uint32_t n_heads, uint32_t head_dim,
                           uint32_t rope_dims, float theta, float eps, const uint32_t *d_offset,
                           uint32_t offset, fk_stream s);

/* R   RoPE(K) -> cache_k[kh, write_offset % capacity, :], V copied likewise;
 *     caches [n_kv, capacity, dim].  Replaces
 *     src/codegen/kernels/rope_kv_cache_store_decode.rs:21-143; with k_norm the
 *     per-head RMSNorm variant src/codegen/kernels/rmsnorm_rope_kv_cache_store_decode.rs:11-176;
 *     rope_dims == 0 stores K unrotated (src/codegen/kernels/kv_cache_store_decode.rs,
 *     k_dim may differ from v_dim). */
fk_status fk_rope_kv_cache_store_decode(const uint16_t *k, const uint16_t *v, const uint16_t *k_norm,
                                        uint32_t n_kv, uint32_t k_dim, uint32_t v_dim, uint32_t rope_dims,
                                        float theta, float eps, const uint32_t *d_offset, uint32_t offset,
                                        const uint32_t *d_write_offset, uint32_t write_offset,
                                        uint32_t capacity, uint16_t *cache_k, uint16_t *cache_v, fk_stream s);

/* R   the two above in ONE launch (MI355X addition: halves the launch count of
 *     the rope/store stage; same arithmetic). */
fk_status fk_qkv_rope_store_decode(uint16_t *q, const uint16_t *k, const uint16_t *v, const uint16_t *q_norm,
                                   const uint16_t *k_norm, uint32_t n_heads, uint32_t n_kv, uint32_t head_dim,
                                   uint32_t rope_dims, float theta, float eps, const uint32_t *d_offset,
                                   uint32_t offset, uint32_t capacity, uint16_t *cache_k, uint16_t *cache_v,
                                   fk_stream s);

/* K4  GQA SDPA for one query token over the bf16 cache, fp32 softmax, split-K
 *     with an in-kernel ordered merge.  Replaces
 *     src/codegen/kernels/sdpa_decode.rs:133-408 (online body :1064-1211,
 *     partial/combine :717-1046).  `max_len` bounds kv_len for this launch (it
 *     sizes the split; use the cache capacity when replaying a graph).
 *     Workspace sizes from fk_sdpa_workspace_bytes; `counters` must be zero
 *     before the first launch (the kernel leaves them zero). */
fk_status fk_sdpa_workspace_bytes(uint32_t n_heads, uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim,
                                  uint32_t max_len, size_t *partial_bytes, size_t *counter_bytes);
fk_status fk_sdpa_decode(const uint16_t *q, const uint16_t *cache_k, const uint16_t *cache_v, uint16_t *out,
                         const uint32_t *d_kv_len, uint32_t kv_len, uint32_t max_len, uint32_t n_heads,
                         uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim, uint32_t capacity, float scale,
                         float *partials, uint32_t *counters, fk_stream s);

/*     The same attention for callers that cannot allocate device memory (code under hipGraph capture,
 *     tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference: the
 *     split-K workspace (partial rows + arrival counters) is a device array inside the library,
 *     fk_sdpa_static_scratch_bytes() = 9 MiB per GPU for the life of the process, found once per device
 *     with hipGetSymbolAddress.  The call allocates nothing; problems whose workspace
 *     (fk_sdpa_workspace_bytes) does not fit are refused with FK_ERR_UNSUPPORTED.  All calls on one GPU
 *     share the array: calls that overlap on one GPU race and must be serialised by the caller. */
size_t fk_sdpa_static_scratch_bytes(void);
fk_status fk_sdpa_decode_static(const uint16_t *q, const uint16_t *cache_k, const uint16_t *cache_v, uint16_t *out,
                                const uint32_t *d_kv_len, uint32_t kv_len, uint32_t max_len, uint32_t n_heads,
                                uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim, uint32_t capacity, float scale,
                                fk_stream s);

/* ---- quantised KV cache (mlx-lm QuantizedKVCache: kv_bits = 4 | 8) ----------------
 * Layout: packed uint32 [n_kv, capacity, dim*bits/32], scales / biases bf16
 * [n_kv, capacity, dim/group] (src/codegen/kernels/sdpa_decode_quant.rs:10-17).
 * fk_kv_cache_store_quant replaces src/codegen/kernels/rope_kv_cache_store_decode_quant.rs:
 * rows of new K (RoPE, optional head norm, kept in fp32) and V are quantised per group and
 * written at cache rows (offset + r) % capacity.  fk_sdpa_decode_quant replaces
 * sdpa_decode_quant.rs: attention with k = code * scale + bias evaluated in fp32; split,
 * workspace and counters exactly as fk_sdpa_decode; `rows` > 1 as fk_sdpa_decode_rows. */
typedef struct fk_kv_quant_cache {
    uint32_t *packed;
    uint16_t *scales;
    uint16_t *biases;
} fk_kv_quant_cache;
fk_status fk_kv_cache_store_quant(const uint16_t *k, const uint16_t *v, const uint16_t *k_norm, uint32_t n_kv,
                                  uint32_t head_dim, uint32_t rope_dims, float theta, float eps,
                                  const uint32_t *d_offset, uint32_t offset, uint32_t rows, uint32_t capacity,
                                  uint32_t bits, uint32_t group, const fk_kv_quant_cache *cache_k,
                                  const fk_kv_quant_cache *cache_v, fk_stream s);
/* Rows [0, rows) of every head of a quantised cache as bf16 [n_kv, out_capacity, dim], T(code * scale + bias):
 * the operand form of fk_sdpa_prefill, so that a prompt pass over a quantised cache runs the matrix-core
 * attention on the dequantised prefix (an MI355X addition; the reference's prefill variants keep a bf16 cache). */
fk_status fk_kv_cache_dequant(const fk_kv_quant_cache *cache, uint32_t n_kv, uint32_t dim, uint32_t capacity,
                              uint32_t bits, uint32_t group, uint32_t rows, uint16_t *out, uint32_t out_capacity,
                              fk_stream s);
fk_status fk_sdpa_decode_quant(const uint16_t *q, const fk_kv_quant_cache *cache_k, const fk_kv_quant_cache *cache_v,
                               uint16_t *out, const uint32_t *d_kv_len, uint32_t kv_len, uint32_t max_len,
                               uint32_t rows, uint32_t n_heads, uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim,
                               uint32_t capacity, uint32_t bits, uint32_t group, float scale, float *partials,
                               uint32_t *counters, fk_stream s);

/* ---- mixture-of-experts decoder with low-rank (MLA-style) keys: the glue around M1 / M2 / K4 ----
 * fk_kv_cache_store_split_decode replaces the split-key form of KvCacheStoreDecode
 * (src/codegen/kernels/kv_cache_store_decode.rs:84-352; attrs src/fusion/ir.rs:343-357): cache K row =
 * [K0 | K1]; K0 has n_kv heads, K1 has k1_heads = n_kv heads or 1 head shared by all; the first rope_dims
 * of K1 are rotated at `offset` while written (traditional != 0: pairs (2i, 2i+1), else (i, i + rope_dims/2)).
 * K0 / V head rows start k0_stride / v_stride elements apart, so both may point into one packed
 * [n_kv, k0_dim + v_dim] projection output (the reference's kv_transpose_split).  With n_heads > 0 the
 * query's second part -- Q1 of the packed rows q [n_heads, q0_dim + q1_dim] -- gets the same rotation in
 * place, rounded to bf16; the reference rotates Q1 inside its attention kernel and keeps fp32 there
 * (src/codegen/kernels/sdpa_decode.rs:592-660), a difference of at most one bf16 rounding per rotated
 * query element.  Offsets as in fk_rope_kv_cache_store_decode. */
fk_status fk_kv_cache_store_split_decode(uint16_t *q, uint32_t n_heads, uint32_t q0_dim, uint32_t q1_dim,
                                         const uint16_t *k0, uint32_t k0_stride, const uint16_t *k1, uint32_t k1_heads,
                                         const uint16_t *v, uint32_t v_stride, uint32_t n_kv, uint32_t k0_dim,
                                         uint32_t k1_dim, uint32_t v_dim, uint32_t rope_dims, int traditional,
                                         float theta, const uint32_t *d_offset, uint32_t offset,
                                         const uint32_t *d_write_offset, uint32_t write_offset, uint32_t capacity,
                                         uint16_t *cache_k, uint16_t *cache_v, fk_stream s);
/* Row form (several active token rows, row r at position offset + r, as the other _rows entry points): q is
 * [rows, n_heads, q0_dim + q1_dim]; the K0 / K1 / V rows of token r start k0_row_stride / k1_row_stride /
 * v_row_stride elements after those of token r - 1 (packed projection outputs [rows, n_kv, k0_dim + v_dim] and
 * [rows, kv_lora_rank + k1_dim] are addressed without copies). */
fk_status fk_kv_cache_store_split_rows(uint16_t *q, uint32_t n_heads, uint32_t q0_dim, uint32_t q1_dim, const uint16_t *k0,
                                       uint32_t k0_stride, uint32_t k0_row_stride, const uint16_t *k1, uint32_t k1_heads,
                                       uint32_t k1_row_stride, const uint16_t *v, uint32_t v_stride, uint32_t v_row_stride,
                                       uint32_t n_kv, uint32_t k0_dim, uint32_t k1_dim, uint32_t v_dim, uint32_t rope_dims,
                                       int traditional, float theta, uint32_t rows, uint32_t offset, uint32_t capacity,
                                       uint16_t *cache_k, uint16_t *cache_v, fk_stream s);
/* The split-key store and the attention of a layer in ONE launch (one token): what fk_kv_cache_store_split_decode
 * followed by fk_sdpa_decode computes, bit for bit.  Every block rotates its query heads itself (q is only
 * read), the block whose range holds the new position assembles [K0 | rope(K1)], uses it and the new V row in
 * place of the cache row and appends both to the caches.  kv_len counts the new token (its position is
 * kv_len - 1).  rope_tab (may be NULL): (cos, sin) per rotary pair at that position as fk_step_init_rope fills
 * it for rope_dims.  Workspace as fk_sdpa_decode (fk_sdpa_workspace_bytes). */
fk_status fk_split_store_sdpa_decode(const uint16_t *q, uint32_t n_heads, uint32_t q0_dim, uint32_t q1_dim,
                                     const uint16_t *k0, uint32_t k0_stride, const uint16_t *k1, uint32_t k1_heads,
                                     const uint16_t *v, uint32_t v_stride, uint32_t n_kv, uint32_t v_dim,
                                     uint32_t rope_dims, int traditional, float theta, const float *rope_tab,
                                     uint16_t *cache_k, uint16_t *cache_v, uint16_t *out, const uint32_t *d_kv_len,
                                     uint32_t kv_len, uint32_t max_len, uint32_t capacity, float scale,
                                     float *partials, uint32_t *counters, fk_stream s);
/* fk_softmax_topk_route replaces the router kernel SoftmaxTopKRoute (src/codegen/kernels/single.rs:2615-2760;
 * matcher src/fusion/general.rs:6768-6880): per row softmax over row_n bf16 logits, probabilities rounded
 * to bf16 BEFORE the ordering, the top_k largest in descending order with ties to the lower index;
 * idx u32 [rows, top_k], weight bf16 [rows, top_k] = T(prob * scale).  scale: one bf16 value
 * (scale_per_route = 0) or bf16 [rows, top_k].  row_n a power of two <= 256, top_k < row_n and <= 32
 * (the reference's admission); anything else FK_ERR_UNSUPPORTED. */
fk_status fk_softmax_topk_route(const uint16_t *logits, const uint16_t *scale, int scale_per_route, uint32_t rows,
                                uint32_t row_n, uint32_t top_k, uint32_t *idx, uint16_t *weight, fk_stream s);

/* fk_moe_router: RMSNorm of one hidden row (norm_w may be NULL: x as it is), the router projection with
 * bf16 weights w [experts, hidden] and fk_softmax_topk_route with one scale, as ONE launch (one wave per
 * expert; the wave that finishes last routes).
 * The reference runs these as three kernels (norm: src/codegen/kernels/mod.rs:4424-4516; linear: K1;
 * SoftmaxTopKRoute: src/codegen/kernels/single.rs:2615-2760); the arithmetic here is their composition
 * with the same roundings (normalised row and logits rounded to bf16).  xn [hidden] and logits [experts]
 * are optional outputs (NULL to skip).  hidden a multiple of 512 up to 4096; experts / top_k as above.
 * top_k = 0: no routing here -- the logits (then required) are the output, for a consumer that routes itself
 * (fk_routed_qmv_swiglu_routing); scale, idx, weight and workspace may then be NULL.
 * rows token rows at once: x / xn [rows, hidden], logits [rows, experts], idx / weight [rows, top_k].
 * workspace: rows * (experts + 1) 32-bit words, zero before the first launch, left zeroed by every launch;
 * launches that share it must not overlap. */
fk_status fk_moe_router(const uint16_t *x, const uint16_t *norm_w, float eps, const uint16_t *w, const uint16_t *scale,
                        uint32_t hidden, uint32_t experts, uint32_t top_k, uint16_t *xn, uint16_t *logits,
                        uint32_t *idx, uint16_t *weight, uint32_t *workspace, uint32_t rows, fk_stream s);

/* ---- several active token rows (multi-token verification, chunked prefill) ----
 * The reference compiles such variants with active_m > 1 (src/target/mod.rs:170-200,
 * variants `prefill_mN`, src/patch.rs:103-150; causal attention
 * src/codegen/kernels/sdpa_prefill.rs:1-30).  Row r of a group is the token at position
 * offset + r.  The projections of a group run through fk_qgemm / fk_qgemm_swiglu on rows that
 * fk_rmsnorm_rows normalised; the functions below are the row forms of E, R and K4. */
fk_status fk_rmsnorm_rows(const uint16_t *x, const uint16_t *w, float eps, uint32_t rows, uint32_t hidden,
                          uint16_t *y, fk_stream s);
fk_status fk_embed_lookup_rows(const fk_weight *E, const uint32_t *d_tokens, uint32_t rows, float out_scale,
                               uint16_t *x, fk_stream s);
/* q [rows, n_heads, head_dim] in place; k, v [rows, n_kv, head_dim] -> cache rows (offset + r) % capacity.
 * rope_tab (may be NULL): [rows][rope_dims/2] (cos, sin) pairs for positions offset .. offset + rows - 1 as
 * fk_rope_table_rows fills them -- the very values the kernel computes without it, so the results are
 * bit-identical; a prompt pass fills the table once and every layer reuses it. */
fk_status fk_rope_table_rows(float *tab, uint32_t rope_dims, float theta, uint32_t offset, uint32_t rows, fk_stream s);
fk_status fk_qkv_rope_store_rows(uint16_t *q, const uint16_t *k, const uint16_t *v, const uint16_t *q_norm,
                                 const uint16_t *k_norm, uint32_t n_heads, uint32_t n_kv, uint32_t head_dim,
                                 uint32_t rope_dims, float theta, float eps, uint32_t rows, uint32_t offset,
                                 uint32_t capacity, uint16_t *cache_k, uint16_t *cache_v, const float *rope_tab,
                                 fk_stream s);
/* Row r attends to the first kv_len + r cache positions (causal inside the group); q and out are
 * [rows, n_heads, dim].  Workspace: rows times the sizes of fk_sdpa_workspace_bytes(max_len =
 * kv_len + rows - 1); counters zero before the first launch. */
fk_status fk_sdpa_decode_rows(const uint16_t *q, const uint16_t *cache_k, const uint16_t *cache_v, uint16_t *out,
                              uint32_t rows, uint32_t kv_len, uint32_t n_heads, uint32_t n_kv, uint32_t qk_dim,
                              uint32_t v_dim, uint32_t capacity, float scale, float *partials, uint32_t *counters,
                              fk_stream s);
/* Causal attention of a group of rows on the matrix cores.  Replaces
 * src/codegen/kernels/sdpa_prefill.rs:1-205 with its buffer contract (:11-21): q and out
 * [rows, n_heads, head_dim]; caches [n_kv, capacity, head_dim]; `kv_len` = positions in the cache
 * INCLUDING the rows of this group (prior + rows); row r sits at position (kv_len - rows) + r and
 * sees positions 0 .. that one.  fp32 scores and softmax (probabilities enter the second product
 * as bf16), one rounding of the output.  No workspace; kv_len is bounded by the capacity only (the
 * reference: 4096).  head_dim 64 or 128, bf16 cache; other shapes and the quantised cache go
 * through fk_sdpa_decode_rows / fk_sdpa_decode_quant. */
fk_status fk_sdpa_prefill(const uint16_t *q, const uint16_t *cache_k, const uint16_t *cache_v, uint16_t *out,
                          uint32_t rows, uint32_t kv_len, uint32_t n_heads, uint32_t n_kv, uint32_t head_dim,
                          uint32_t capacity, float scale, fk_stream s);

/* E   x = T(embed[token] * out_scale), dense bf16 or MLX-affine table.  Replaces
 *     src/codegen/kernels/embed_lookup_decode.rs:17-108. */
fk_status fk_embed_lookup_decode(const fk_weight *E, const uint32_t *d_token, uint32_t token, float out_scale,
                                 uint16_t *x, fk_stream s);

/* A   greedy argmax over bf16 logits, lowest index wins ties, NaN never wins;
 *     optionally appends the token to history[(*hist_counter)++].  Replaces
 *     src/codegen/kernels/argmax_logits_{decode,scan,finalize}.rs.  Workspace:
 *     FK_ARGMAX_WORKSPACE_BYTES, zeroed once. */
#define FK_ARGMAX_WORKSPACE_BYTES 1288
fk_status fk_argmax_logits_decode(const uint16_t *logits, uint32_t n, uint32_t *next_token, uint32_t *history,
                                  uint32_t *hist_counter, uint32_t hist_capacity, void *workspace, fk_stream s);

/* U   offset = step_counter++ ; kv_len = offset + 1.  Replaces fusekit_step_init
 *     (src/codegen/kernels/mod.rs:542-563). */
fk_status fk_step_init(uint32_t *step_counter, uint32_t *offset, uint32_t *kv_len, fk_stream s);
/*     The same, and fills `rope_tab` (2 * (rope_dims / 2) floats: cos, sin of every rotary pair at
 *     position `offset`, the values rope_q_decode.rs:93-114 computes per head) once for all layers of
 *     the token; fk_rope_store_sdpa_decode reads it. */
fk_status fk_step_init_rope(uint32_t *step_counter, uint32_t *offset, uint32_t *kv_len, float *rope_tab,
                            uint32_t rope_dims, float theta, fk_stream s);

/* R+H+A in one launch: head norm + RoPE of q and of the new k row, the append of the new k / v rows
 *     to the cache at row kv_len - 1, and the attention of fk_sdpa_decode over kv_len rows.  Same
 *     arithmetic and rounding points as fk_qkv_rope_store_decode followed by fk_sdpa_decode (the
 *     rotated q is used from on-chip memory and not written back); replaces the dispatch pair
 *     rope_q_decode.rs / rope_kv_cache_store_decode.rs + sdpa_decode.rs of one layer.  q_norm and
 *     k_norm come together or not at all; rope_tab from fk_step_init_rope or NULL (computed in place). */
fk_status fk_rope_store_sdpa_decode(const uint16_t *q, const uint16_t *k, const uint16_t *v, const uint16_t *q_norm,
                                    const uint16_t *k_norm, uint16_t *cache_k, uint16_t *cache_v, uint16_t *out,
                                    const uint32_t *d_kv_len, uint32_t kv_len, uint32_t max_len, uint32_t n_heads,
                                    uint32_t n_kv, uint32_t head_dim, uint32_t rope_dims, float theta, float eps,
                                    uint32_t capacity, float scale, const float *rope_tab, float *partials,
                                    uint32_t *counters, fk_stream s);

/* ---- XCD-resident layer: a decoder layer as TWO launches -------------------------------------
 *
 * Dispatch families `fusekit_xcd_attn_block` (replaces, for one layer, the dispatches
 * rmsnorm_qkv.rs + rope_q_decode.rs / rope_kv_cache_store_decode.rs (or their head-norm forms) +
 * sdpa_decode.rs + linear_residual.rs of the attention half) and `fusekit_xcd_mlp_block` (replaces
 * rmsnorm_gateup_swiglu.rs + linear_residual.rs of the MLP half); `fusekit_xcd_reduce` finishes the last
 * layer's output row for final_rmsnorm_lm_head.rs.  Same arithmetic and rounding points per output
 * (fp32 accumulation, one rounding to bf16 after the residual is added); the K dimension of o_proj and
 * down_proj is summed as 8 slices, one per XCD, whose fp32 sums are added as 64-bit fixed-point integers
 * (2^-32 units, memory-side atomic adds) into a "sum row": integer addition is associative, so the result
 * does not depend on the order of arrival.  A sum row holds fk_xcd_sum_row_bytes(hidden) bytes; element e
 * of the vector sits at index ((((t >> 6) * 4 + ((e & 7) >> 1)) * 64 + (t & 63)) << 1) | (e & 1), t = e >> 3.
 * Three rows rotate through the launches of a token: a launch reads one (the previous launch's), adds into
 * the second and clears the third (the one the launch after it adds into); the row the first launch of a
 * token adds into must hold zeros (fusekit_xcd_reduce clears it at the end of the previous token; zero all
 * three once after allocation, and again after a launch has reported an error -- the dispatcher does that
 * for the rows bound to a graph).  One contribution must be finite and below 2^27 in magnitude; a launch that
 * meets another clamps it and raises a word of the control block, reported as FK_ERR_HIP by the next check
 * (resolution: 2^-32 per contribution).  Slot orders are documented at the planners
 * (fusekit_amd/csrc/dispatcher.hip).  Requires 8 KV heads (one per XCD), 1 / 2 / 4 / 8 query heads per KV
 * head, head_dim 64 or 128, hidden <= 4096, and a shape whose workgroups fit two per CU (LDS and registers:
 * answered from the shape where possible, else by the device's occupancy query); other layers use the
 * per-dispatch families.  Parameter token_launch on the dispatches of a run: 1 -- fk_build_graph executes the
 * whole run attention, MLP, attention, ... as ONE kernel node (device-wide barriers between the phases; every
 * layer then needs its own q / k / v rows); 2 -- each attention dispatch and the MLP dispatch behind it as one
 * node where both take their one-pass flavour.  Both are off by default: on this part a kernel boundary costs
 * less than the barrier that replaces it.
 *
 * EXCLUSIVE USE OF THE DEVICE.  A launch of these families is 512 workgroups that wait for one another inside
 * the launch, so all of them must be resident at once, two per CU of all 256 CUs, dealt to the XCDs round-robin.
 * Nothing else may run on the device while such a launch runs: no kernel of another stream, process or graph
 * branch.  fk_build_graph refuses a graph in which any other node is not ordered before or after such a
 * launch.  A launch that cannot make progress does not hang: every wait is bounded (parameter spin_limit),
 * gives up, and the error is reported by fk_xcd_check / by the dispatcher call that executed the graph;
 * the results of that token are then invalid -- decode it again (the retry rewrites the cache rows). */
fk_status fk_xcd_layer_supported(uint32_t hidden, uint32_t inter, uint32_t n_heads, uint32_t n_kv, uint32_t head_dim,
                                 uint32_t capacity, uint32_t bits, uint32_t group);
/* Bytes of the control block (arrival words, abort / overflow words, placement words; zero it once) and of the
 * attention partial rows. */
fk_status fk_xcd_workspace_bytes(uint32_t n_heads, uint32_t head_dim, size_t *control_bytes, size_t *attention_partial_bytes);
/* Bytes of one sum row of a hidden-wide vector (0 for hidden == 0). */
size_t fk_xcd_sum_row_bytes(uint32_t hidden);
/* The expert block of a mixture-of-experts layer as ONE such launch, dispatch family `fusekit_xcd_moe_block`: replaces,
 * for one layer and one token, the router (an RMSNorm, a bf16 linear layer and SoftmaxTopKRoute,
 * src/codegen/kernels/single.rs:2615-2760), routed_qmv_swiglu.rs (with the shared expert's gate / up pair) and
 * routed_qmv_reduce.rs (with the shared expert's down_proj).  The cut is BY ROUTE: XCD u < top_k serves the u-th winner
 * of the ranking -- its 64 workgroups form the 64 router logits, hand them over inside the XCD, every wave ranks them,
 * then the expert's gate / up rows, SwiGLU, a second hand-over, and the expert's down_proj over the whole intermediate
 * width.  A route's full dot product is formed, rounded to bf16 and weighted inside one XCD, as the reference's
 * reduction does it (routed_qmv_reduce.rs:236-322).  The shared expert, n = shared_inter / inter times as wide as a
 * routed one, is n more units of the same size on the next XCDs (gate / up rows [h inter, (h+1) inter) and the K-slice
 * of the shared down_proj they feed); their partial dot products are added unrounded into a second sum row.  Outputs:
 * the two sum rows -- x = T((f32(row) + T(f32(shared row))) + residual) is the reference's result with its additions in
 * its order, the weighted routes being added exactly, in 64-bit fixed point, where the reference adds them one by one
 * in fp32; fusekit_xcd_reduce with six slots forms it -- and the logits, the routes and their weights for the host.
 * Slot order at the planner (fusekit_amd/csrc/dispatcher.hip).  Requires 4-bit weights, at most 64 experts,
 * top_k + n <= 8, widths that are multiples of 128 and give every workgroup whole rows (inter % 64 == 0,
 * hidden % 64 == 0), tiles of at most 1536 16-byte chunks and 768 quantisation groups; other layers use the
 * per-dispatch families.  The exclusive-use rule below applies. */
fk_status fk_xcd_moe_supported(uint32_t hidden, uint32_t inter, uint32_t shared_inter, uint32_t experts, uint32_t top_k,
                               uint32_t bits, uint32_t group);
/* Bytes of the launch's scratch slot: per-XCD copies of the router logits and the SwiGLU rows of the eight units. */
size_t fk_xcd_moe_scratch_bytes(uint32_t inter);
/* The attention half of a layer with low-rank keys as ONE such launch, dispatch family `fusekit_xcd_mla_block`:
 * replaces, for one layer and one token, the two rmsnorm_qkv.rs launches (norm + q / kv_a, latent norm + kv_b), the
 * split-key cache store with its rotations, sdpa_decode.rs and linear_residual.rs (o_proj).  n_heads / 8 heads per XCD;
 * every XCD forms the whole kv_a row itself (its own copy in the `kva` slot), so the latent norm and kv_b need no
 * exchange between XCDs; o_proj is cut along K by XCD as in fusekit_xcd_attn_block and added into a sum row.  The input
 * is a plain row or the two rows of the previous layer's fusekit_xcd_moe_block (x = T((f32(row) + T(f32(shared row))) +
 * residual)).  Same arithmetic and rounding points per output as the launches it replaces.  Requires 4-bit weights,
 * 8 .. 32 heads in multiples of 8, hidden a multiple of 256 up to 4096, a latent width that is a multiple of 128;
 * slot order at the planner (fusekit_amd/csrc/dispatcher.hip).  The exclusive-use rule below applies. */
fk_status fk_xcd_mla_supported(uint32_t hidden, uint32_t n_heads, uint32_t rank, uint32_t rope_dim, uint32_t nope_dim,
                               uint32_t v_dim, uint32_t capacity, uint32_t bits, uint32_t group);
/* Bytes of that family's `kva` slot (eight copies of the latent row) and of its attention partial rows. */
fk_status fk_xcd_mla_workspace_bytes(uint32_t n_heads, uint32_t rank, uint32_t rope_dim, uint32_t v_dim, size_t *latent_bytes,
                                     size_t *attention_partial_bytes);
/* The o_proj and down_proj slots of the two families take their scales and biases re-laid out per K-slice:
 * dst[(h * n + r) * (groups / 8) + g] = src[r * groups + h * (groups / 8) + g] for the [n, groups] array of a
 * matrix (same size as the source).  An XCD then reads its slice of every row as one contiguous stream; in the
 * MLX layout its 16..38 bytes of every row drag whole 128-byte lines into all eight L2s.  Done once per matrix
 * at load time; the weights themselves stay in the MLX layout (src/fusion/ir.rs:236-242). */
fk_status fk_xcd_kslice_meta(const uint16_t *src, uint32_t n, uint32_t groups, uint16_t *dst, fk_stream s);
/* Synchronises the stream and reports (FK_ERR_HIP, control block reset to zeros) whether a launch gave up on a
 * hand-over wait, met a contribution outside the sum rows' range, or ran two workgroups in one (XCD, slot).  The
 * dispatcher does the same check after every execution of a graph that holds such launches -- synchronous,
 * range, per-node profile, decode chunks, and in fk_wait_pending for the asynchronous pair -- and zeroes the
 * graph's sum rows when it fails. */
fk_status fk_xcd_check(void *workspace, fk_stream s);

/* ---- dispatcher: replaces `_fusekit_runtime_native` ------------------------
 *
 * A dispatch names a kernel family by prefix ("fusekit_rmsnorm_qkv_f12" ->
 * family "fusekit_rmsnorm_qkv"; names follow kernel_function_name,
 * src/codegen/kernels/mod.rs:5578-5583), lists its buffers as (pointer, bytes)
 * in slot order and carries key/value parameters (dims, eps, theta, bits ...)
 * in place of the constants the reference bakes into kernel text.  Slot order
 * per family ([..] optional; quantised weights add their scales then biases):
 *   fusekit_step_init                 step_counter, offset, kv_len
 *   fusekit_embed_lookup_decode       token, table [, scales, biases], x
 *       {bits=16, hidden, vocab, group=64, output_scale=1}
 *   fusekit_rmsnorm_qkv | fusekit_qmv_fanout(has_norm=0)
 *       x, [norm_w], W_q, W_k, W_v, [s_q, s_k, s_v, b_q, b_k, b_v], [bias_q, bias_k, bias_v], q, k, v
 *       {bits=4, group=64, hidden, n_q, n_kv, eps, has_norm=1, has_bias=0}
 *   fusekit_rope_q_decode             Q, offset            {n_heads, head_dim, rope_dims, theta}
 *   fusekit_rmsnorm_rope_q_decode     Q, q_weight, offset  {+ eps}
 *   fusekit_rope_kv_cache_store_decode | fusekit_kv_cache_store_decode (no rotation)
 *       K, V, cache_k, cache_v, offset, write_offset   {n_kv, head_dim, v_dim, rope_dims, theta, capacity}
 *   fusekit_rmsnorm_rope_kv_cache_store_decode
 *       K, V, k_weight, cache_k, cache_v, offset, write_offset   {+ eps}
 *   fusekit_qkv_rope_store_decode     Q, K, V, [q_weight, k_weight], cache_k, cache_v, offset
 *       {n_heads, n_kv, head_dim, rope_dims, theta, capacity, eps, has_norm=0}
 *   fusekit_sdpa_decode               Q, K, V, kv_len, out, partials, counters
 *       {n_heads, n_kv, head_dim | qk_dim, v_dim, capacity, max_len=capacity, scale=1/sqrt(qk_dim)}
 *   fusekit_linear_residual           x, W [, scales, biases], residual, [residual_extra], y
 *       {bits=4, group=64, m (= K), n, has_extra=0}
 *   fusekit_rmsnorm_gateup_swiglu | fusekit_qmv_swiglu(has_norm=0)
 *       x, [norm_w], W_gate, W_up, [s_g, s_u, b_g, b_u], out   {bits, group, hidden, inter, eps, variant=0, has_norm=1}
 *   fusekit_final_rmsnorm_lm_head     x, norm_w, W [, scales, biases], logits   {bits=16, group, hidden, vocab, eps}
 *   fusekit_final_rmsnorm_lm_head_argmax   x, norm_w, W [, scales, biases], logits, next_tok, workspace
 *                                     [, history, hist_counter]   {bits=16, group, hidden, vocab, eps}
 *   fusekit_qgemv                     x, W [, scales, biases], [bias], y        {bits, group, m, n, has_bias=0}
 *   fusekit_argmax_logits_decode      logits, next_tok, workspace [, history, hist_counter]   {vocab}
 * Read/write slots per family follow the reference's table
 * (python/fusekit_runtime/dispatch.py:100-190); graph edges are derived from
 * them on overlapping byte ranges (RAW, WAW, WAR). */
typedef uint64_t fk_handle;
typedef struct fk_arg { void *ptr; size_t nbytes; } fk_arg;
typedef struct fk_param { const char *key; double value; } fk_param;
typedef struct fk_dispatch {
    const char *kernel;
    const fk_arg *args;
    uint32_t n_args;
    const fk_param *params;
    uint32_t n_params;
} fk_dispatch;
typedef struct fk_binding_update { uint32_t cmd_idx, slot; void *ptr; size_t nbytes; } fk_binding_update;

/* Device scalars of the per-token protocol (python_runtime/src/lib.rs:1299-1303,
 * src/codegen/kernels/mod.rs:544-577): `token` is read by the embedding lookup
 * and written by the argmax (token_id_in aliases next_token_out). */
typedef struct fk_decode_uniforms {
    uint32_t *token;
    uint32_t *step_counter;
    uint32_t *hist_counter;
    uint32_t *history;
    uint32_t hist_capacity;
} fk_decode_uniforms;

/* load_dispatcher (lib.rs:116-169).  The kernels are compiled into the library:
 * `code_object_path` may be NULL or "builtin"; a path is only checked to exist.
 * `task_graph_path` (may be NULL) is parsed: version must be 2
 * (src/runtime/plan.rs:175-180) and every task's kernel must name a family of
 * this library (lib.rs:412-415), else FK_ERR_INVALID. */
fk_status fk_load_dispatcher(const char *code_object_path, const char *task_graph_path, fk_handle *out);
/* kernel_names (lib.rs:223) */
fk_status fk_kernel_names(fk_handle h, const char *const **names, size_t *n);
fk_status fk_dispatcher_stream(fk_handle h, fk_stream *out);
/* dispatch_kernel (lib.rs:398) / dispatch_batch (lib.rs:1723): launch and wait, GPU seconds out */
fk_status fk_dispatch_kernel(fk_handle h, const fk_dispatch *d, double *gpu_seconds);
fk_status fk_dispatch_batch(fk_handle h, const fk_dispatch *list, size_t n, double *gpu_seconds);
/* T2  Launch geometry and slot access of one dispatch, as the planners decide it: what the
 *     reference computes in kernel_threadgroup_for / kernel_grid_threads_impl and records per
 *     task in task_graph.json (src/codegen/kernels/mod.rs:5694, 6218; task_graph_json.rs
 *     grid_threads / threadgroup).  A dispatch may expand to up to FK_MAX_TASK_KERNELS kernels
 *     that run back to back (a split-k or routed reduction).  slot_access[i]: bit 0 = the
 *     kernels read slot i, bit 1 = they write it (the hazard mask of
 *     python/fusekit_runtime/dispatch.py:36-100 is derived from these). */
#define FK_MAX_TASK_KERNELS 4
#define FK_MAX_TASK_SLOTS 32
typedef struct fk_launch_geometry {
    uint32_t n_kernels;
    uint32_t grid[FK_MAX_TASK_KERNELS][3];        /* workgroups per axis */
    uint32_t threadgroup[FK_MAX_TASK_KERNELS][3]; /* threads per workgroup */
    uint32_t lds_bytes[FK_MAX_TASK_KERNELS];
    uint32_t n_slots;
    uint8_t slot_access[FK_MAX_TASK_SLOTS];
} fk_launch_geometry;
fk_status fk_plan_geometry(fk_handle h, const fk_dispatch *d, fk_launch_geometry *out);

/* build_icb (lib.rs:461): pre-encode the list as one hipGraph.  `barriers`
 * NULL = edges from the read/write tables; barriers[i] != 0 additionally makes
 * command i wait for every earlier command. */
fk_status fk_build_graph(fk_handle h, const fk_dispatch *list, size_t n, const uint8_t *barriers,
                         uint32_t *graph_id);
/* Decode pipeline as a graph.  persistent = 0: one node per task, executed in list order (fk_build_graph with
 * every barrier set): the launches of a decode pipeline each fill the GPU, and a graph that forks anywhere -- the
 * step counter beside the embedding lookup is enough -- is replayed through several hardware queues, which
 * measured about 70 us more per replay than the same nodes as a chain.  persistent = 1: the task list must be the canonical dense decode
 * pipeline (step_init, embed_lookup_decode, L x [rmsnorm_qkv, rope / KV-store
 * task(s), sdpa_decode, linear_residual, rmsnorm_gateup_swiglu, linear_residual],
 * final_rmsnorm_lm_head, argmax_logits_decode with history); it is run by ONE
 * persistent kernel per token whose phases are separated by grid barriers and
 * which prefetches the next phase's weights across them -- the working form of
 * what the reference sketches as emit_megakernel (src/codegen/persistent.rs:57-75)
 * and the LayerBlock experiment (src/fusion/layer_block.rs).  Same arithmetic.
 * Otherwise FK_ERR_UNSUPPORTED.  spin_limit bounds every barrier wait in polls
 * (0 = default); a wait that exceeds it sets an abort flag, all waves still
 * drain, and the launching call returns FK_ERR_HIP. */
fk_status fk_build_decode_graph(fk_handle h, const fk_dispatch *list, size_t n, int persistent,
                                uint32_t spin_limit, uint32_t *graph_id);
fk_status fk_graph_launch_shape(fk_handle h, uint32_t graph_id, uint32_t *persistent, uint32_t *grid,
                                uint32_t *lds_bytes);
/* Persistent graphs only: duration of every phase of the LAST launch, seconds
 * (embed, then per layer qkv / attention / o_proj / gate-up / down, LM head,
 * argmax scan, argmax final) -- the per-kernel profile of the one-kernel form,
 * what profile_icb_commands (lib.rs:823) gives for the task-per-kernel form. */
fk_status fk_graph_phase_trace(fk_handle h, uint32_t graph_id, double *seconds, uint32_t cap, uint32_t *n);
fk_status fk_graph_info(fk_handle h, uint32_t graph_id, uint32_t *n_nodes, uint32_t *n_edges);
fk_status fk_graph_node_deps(fk_handle h, uint32_t graph_id, uint32_t node, uint32_t *deps, uint32_t cap,
                             uint32_t *n);
/* update_icb_bindings (lib.rs:575): patch buffers (KV-cache growth) without a rebuild */
fk_status fk_update_graph_bindings(fk_handle h, uint32_t graph_id, const fk_binding_update *ups, size_t n);
/* execute_icb (lib.rs:719), execute_icb_range (lib.rs:770), profile_icb_commands (lib.rs:823) */
fk_status fk_execute_graph(fk_handle h, uint32_t graph_id, double *gpu_seconds);
fk_status fk_execute_graph_repeat(fk_handle h, uint32_t graph_id, uint32_t count, double *gpu_seconds);
fk_status fk_execute_graph_range(fk_handle h, uint32_t graph_id, uint32_t start, uint32_t end,
                                 double *gpu_seconds);
fk_status fk_profile_graph_nodes(fk_handle h, uint32_t graph_id, double *per_node_seconds, size_t n);
/* submit_icb_async (lib.rs:660) + wait_pending_icb (lib.rs:702): one launch in flight */
fk_status fk_submit_graph_async(fk_handle h, uint32_t graph_id);
fk_status fk_wait_pending(fk_handle h, double *gpu_seconds);
/* decode_chunk_gpu_chain (lib.rs:1277-1420): seed step_counter = start_offset,
 * hist_counter = 0, token = seed_token; replay the graph `count` times back to
 * back; wait for the last; copy history[0..count) out. */
fk_status fk_decode_chunk(fk_handle h, uint32_t graph_id, const fk_decode_uniforms *u, uint32_t start_offset,
                          uint32_t seed_token, uint32_t count, uint32_t *out_tokens, double *gpu_seconds);
/* decode_chunk_host_loop (lib.rs:1131-1257): per step the host writes
 * token = tokens_in[i] and step_counter = start_offset + i, replays the graph,
 * waits and reads the next token back into out_next[i].  Used to feed a prompt
 * (forced tokens) through the decode graph. */
fk_status fk_decode_chunk_host_loop(fk_handle h, uint32_t graph_id, const fk_decode_uniforms *u,
                                    uint32_t start_offset, const uint32_t *tokens_in, uint32_t count,
                                    uint32_t *out_next, double *gpu_seconds);

/* Launch-geometry overrides for experiments (0 = library policy): rows per
 * tile and grid blocks of the streaming GEMV.  Process-wide. */
fk_status fk_set_gemv_policy(uint32_t rows_per_tile, uint32_t grid_blocks);
/* The streaming GEMV has two kernel forms: the flat stream (any K that is a multiple of 64, fused epilogues, up to
 * three matrices) and the row-group form (sixteen lanes per row, one accumulator per lane; a single matrix without
 * bias or residual whose rows are whole 256-byte blocks, group size 64, K <= 10240, at least eight rows per
 * compute unit pair).  fk_gemv_form answers which one a plain fk_qgemv / fk_final_rmsnorm_lm_head over an
 * [n, k] matrix would run: 1 = row-group, 0 = flat.  fk_set_gemv_flat_only(1) keeps every launch planned from then
 * on on the flat form (measurements, tests); 0 restores the library's choice.  Process-wide. */
int fk_gemv_form(uint32_t n, uint32_t k, uint32_t bits, uint32_t group);
fk_status fk_set_gemv_flat_only(int flat_only);
/* Row count from which fk_qgemm / fk_qgemm_swiglu dequantise the matrix to bf16 once and hand the
 * product to rocBLAS (opened on first use; absent: the fused kernel is kept).  Default 1024 (below it the fused
 * kernel's LDS-tiled form is the faster one on the benchmark model's projections); 0 = never.
 * Set it BEFORE sizing workspaces: fk_qgemm_workspace_bytes covers the route that will be taken. */
fk_status fk_set_gemm_library_rows(uint32_t rows);
/* 2..10 activation rows at group size 64 run fk_qgemm / fk_qgemm_swiglu as ONE launch that streams the weights
 * once for all rows and includes the epilogue (the reference's small-M kernels: src/codegen/msl.rs:462-546,
 * :1307-1485, policy src/codegen/kernels/mod.rs:164-186).  fk_set_qgemm_wide(0) sends those row counts through
 * the split-k kernel + reduction instead (measurements, tests); 1 restores the default.  Process-wide; takes
 * effect for launches planned afterwards. */
fk_status fk_set_qgemm_wide(int enabled);
/* An MLX-affine matrix (bits 4 / 8, group 64 / 128) as dense bf16 [n, k], every element T(code * scale + bias):
 * the values the library route of fk_qgemm multiplies with.  With 288 GB of HBM a runtime may keep the bf16 copy
 * of a model's projections resident for its prompt passes and hand it to fk_qgemm as a bits-16 weight, which
 * then skips the per-pass dequantisation; the results are the library route's, bit for bit.  No counterpart in
 * the reference (its qMM dequantises inside the kernel, src/codegen/msl.rs:2318-2440). */
fk_status fk_dequantize_bf16(const fk_weight *W, uint16_t *out, fk_stream s);
/* 1 when the GEMM library (rocBLAS, loaded at first use) is present: bits-16 weights and the route from
 * fk_set_gemm_library_rows rows up need it. */
int fk_gemm_library_available(void);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* FUSEKIT_HIP_H */
