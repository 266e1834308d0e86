// XCD-resident decoder layer for gfx950: a layer runs as TWO launches whose inner dependencies never
// leave an XCD.
//
// An MI355X is 8 XCDs of 32 CUs, each with its own L2; the workgroups of a launch are dealt to the XCDs
// round-robin (workgroups i and i + 8 share an XCD; which one is read from the hardware).
// Data written with ordinary stores by one CU is visible to every CU of the SAME XCD as soon as the
// store has been acknowledged (it sits in their common L2), provided the reader bypasses its own L1
// (an `sc1` load); across XCDs it only becomes visible through memory.  A kernel boundary or a
// device-wide barrier therefore costs 2-3 us, a hand-over inside one XCD 0.8 us.
//
// The layer is cut so that every hand-over but two stays inside an XCD:
//
//   attention launch   x = T(sum of the previous launch's 8 partial rows + residual); RMSNorm;
//                      XCD h: q / k / v rows of KV head h  ->  head norm + RoPE + cache append +
//                      attention of KV head h (its G query heads, S key ranges)  ->  merge  ->
//                      o_proj restricted to the K-slice of those heads, ALL output rows: fp32 partial
//                      row h of 8.
//   MLP launch         x1 = T(sum of the 8 o_proj partial rows + residual); RMSNorm;
//                      XCD h: gate / up rows [h I/8, (h+1) I/8) + SwiGLU  ->  down_proj restricted to
//                      that K-slice, ALL output rows: fp32 partial row h of 8.
//
// The sum over the 8 partial rows is taken in a fixed order by the NEXT launch (the kernel boundary makes
// them visible), so results do not depend on timing.  Every block issues the weight loads of BOTH of its
// projections when it starts; the hand-overs only gate arithmetic.
//
// Hand-over protocol inside an XCD: block (xcd, slot) owns one 32-bit flag word.  It reads the word when
// it starts (base), and publishes base + k with an ordinary store after the stores of stage k have been
// acknowledged; a waiting block polls the 64 words of its XCD with one L1-bypassing load per lane until
// all have reached base + k.  Words only grow, so no launch has to reset anything; every wait is bounded
// (spin limit -> abort word, reported by the host).
#pragma once
#include "fk_host.hpp"
#include "gemv_kernel.hpp"
#include "sdpa_kernel.hpp"

namespace fk {

constexpr uint32_t kXcds = 8;
constexpr uint32_t kXcdSlots = 64;                  // blocks per XCD: 2 per CU
constexpr uint32_t kXcdGrid = kXcds * kXcdSlots;    // 512 blocks of 256 threads
constexpr uint32_t kXcdMaxRanges = 16;              // key ranges merged per query head

// Control words of the protocol, one allocation per decoder (fk_xcd_workspace_bytes):
//   flags[8][64]   uint32   arrival word of block (xcd, slot)
//   ssq[8][64]     float    per-block sums of squares of the rows a block reduced
//   abort          uint32   set when a wait ran into the spin limit
struct XcdControl {
    uint32_t flags[kXcds * kXcdSlots];
    float ssq[kXcds * kXcdSlots];
    uint32_t abort_flag;
    uint32_t pad[63];
};

// One projection restricted to a row block and a K-slice: rows [row0, row0 + rows) of a [n, K] matrix,
// chunks [col0, col0 + cs) of each row's cpr 16-byte chunks.
struct XcdMat {
    const uint4* w;
    const uint16_t* sc;
    const uint16_t* bi;
    uint32_t cpr;      // chunks per full row
    uint32_t gshift;   // chunk index >> gshift = quantisation group
};

// The input of a launch: hidden = T(sum_j partial[j][i] + residual[i]) (n_partials = 0: the residual alone),
// written to x_out (one copy per XCD) and RMS-normalised with norm_w for the projections.
struct XcdInput {
    const float* partials;      // [8][hidden] or null
    const uint16_t* residual;   // [hidden] (stride 0) or one copy per XCD (stride hidden)
    uint32_t residual_stride;
    uint16_t* x_out;            // [8][hidden]
    const uint16_t* norm_w;
    float eps;
    uint32_t hidden;
    uint32_t rows_per_block;    // hidden rows one block reduces (ceil(hidden / 64))
};

struct XcdMlpArgs {
    XcdInput in;
    XcdMat gate, up, down;
    uint32_t inter;             // intermediate size; XCD h owns [h * inter / 8, (h + 1) * inter / 8)
    uint32_t gu_rows;           // gate (and up) rows per block
    uint32_t down_rows;         // down_proj output rows per block
    uint32_t down_cs;           // chunks of one XCD's K-slice of a down_proj row
    int swiglu_variant;
    uint16_t* mid;              // [inter] bf16, every XCD touches only its slice
    float* out_partials;        // [8][hidden] fp32
    XcdControl* ctl;
    uint32_t spin_limit;
    uint32_t cs_max, work_floats;  // LDS layout: chunks of the longest staged vector, floats of the work area
};

struct XcdAttnArgs {
    XcdInput in;
    XcdMat wq, wk, wv, wo;
    uint32_t q_rows, kv_rows;   // rows of q / of k (= of v) one XCD owns: G * head_dim, head_dim
    uint32_t qkv_tile_rows;     // rows per block tile of the q / k / v projections
    uint32_t q_tiles, kv_tiles; // tiles of the q part, of the k part (= of the v part)
    uint32_t o_rows;            // o_proj output rows per block
    uint32_t o_cs;              // chunks of one XCD's K-slice of an o_proj row
    uint16_t* q;                // [n_heads * head_dim] raw projection outputs (every XCD its heads)
    uint16_t* k;                // [n_kv * head_dim]
    uint16_t* v;
    SdpaArgs sdpa;              // attention of one KV head per XCD: n_splits ranges x G heads = 64 blocks
    float* out_partials;        // [8][hidden] fp32
    XcdControl* ctl;
    uint32_t spin_limit;
    uint32_t cs_max, work_floats, att_elems;  // LDS layout (att_elems: bf16 elements of the merged attention rows)
};

// x = T(sum of 8 partial rows + residual): the last layer's output for the LM head.
struct XcdReduceArgs {
    const float* partials;
    const uint16_t* residual;   // one copy per XCD: copy 0 is read
    uint16_t* x;
    uint32_t hidden;
};

struct XcdLayerShape {
    uint32_t hidden, inter, n_heads, n_kv, head_dim, capacity, bits, group;
};

// Can this layer shape run XCD-resident?  (8 KV heads, group of 1 / 2 / 4 / 8 query heads, slices that are
// whole quantisation groups, tiles that fit the per-thread load budget.)  Sets an error message if not.
fk_status xcd_layer_supported(const XcdLayerShape& s);
size_t xcd_workspace_bytes();
size_t xcd_attn_partials_bytes(const XcdLayerShape& s);

struct XcdAttnRequest {
    XcdLayerShape shape;
    const float* partials_in;        // previous MLP launch's partial rows, or null (first layer)
    const uint16_t* residual;
    uint32_t residual_stride;
    uint16_t* x_out;
    const uint16_t* norm_w;
    float eps;
    const fk_weight *wq, *wk, *wv, *wo;
    uint16_t *q, *k, *v;
    const uint16_t *q_norm, *k_norm;
    uint16_t *cache_k, *cache_v;
    const uint32_t* kv_len;
    const float* rope_tab;
    float theta;
    float* att_partials;
    float* out_partials;
    void* workspace;
    uint32_t spin_limit;
};
fk_status plan_xcd_attn(const XcdAttnRequest& rq, Launch* out);

struct XcdMlpRequest {
    XcdLayerShape shape;
    const float* partials_in;
    const uint16_t* residual;
    uint32_t residual_stride;
    uint16_t* x_out;
    const uint16_t* norm_w;
    float eps;
    const fk_weight *wgate, *wup, *wdown;
    int swiglu_variant;
    uint16_t* mid;
    float* out_partials;
    void* workspace;
    uint32_t spin_limit;
};
fk_status plan_xcd_mlp(const XcdMlpRequest& rq, Launch* out);
fk_status plan_xcd_reduce(const float* partials, const uint16_t* residual, uint16_t* x, uint32_t hidden, Launch* out);

}  // namespace fk
