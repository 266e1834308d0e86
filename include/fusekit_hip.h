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
fk_status fk_alloc(size_t nbytes, void **dptr);
fk_status fk_free(void *dptr);
fk_status fk_upload(void *dptr, const void *host, size_t nbytes);
fk_status fk_download(void *host, const void *dptr, size_t nbytes);
fk_status fk_fill_u32(void *dptr, uint32_t value, size_t count, fk_stream s);
fk_status fk_stream_create(fk_stream *out);
fk_status fk_stream_destroy(fk_stream s);
fk_status fk_stream_sync(fk_stream s);

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

/* K3a (RMSNorm ->) gate/up projections -> SwiGLU.  variant 0: every op in T
 *     (src/codegen/kernels/rmsnorm_gateup_swiglu.rs:236-257); 1: fp32 sigmoid,
 *     one round (src/codegen/msl.rs:1286-1294); 2: rounded sigmoid and gate
 *     (src/codegen/msl.rs:2441-2449).  norm_w NULL = QmvSwiglu
 *     (src/codegen/kernels/qmv_swiglu.rs:20-246). */
fk_status fk_gateup_swiglu(const uint16_t *x, const uint16_t *norm_w, float eps, const fk_weight *Wg,
                           const fk_weight *Wu, int variant, uint16_t *out, fk_stream s);

/* H   final RMSNorm + vocabulary GEMV, logits in T.  Replaces
 *     src/codegen/kernels/final_rmsnorm_lm_head.rs:144-629. */
fk_status fk_final_rmsnorm_lm_head(const uint16_t *x, const uint16_t *norm_w, float eps, const fk_weight *W,
                                   uint16_t *logits, fk_stream s);

/* Launch-geometry overrides for experiments (0 = library policy): rows per
 * tile and grid blocks of the streaming GEMV.  Process-wide. */
fk_status fk_set_gemv_policy(uint32_t rows_per_tile, uint32_t grid_blocks);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* FUSEKIT_HIP_H */
