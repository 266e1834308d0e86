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
//   attention launch   x = T(sum row of the previous launch + residual); RMSNorm;
//                      XCD h: q / k / v rows of KV head h  ->  head norm + RoPE + cache append +
//                      attention of KV head h (its G query heads, S key ranges)  ->  merge  ->
//                      o_proj restricted to the K-slice of those heads, ALL output rows, each added
//                      into the launch's sum row.
//   MLP launch         x1 = T(sum row of the attention launch + residual); RMSNorm;
//                      XCD h: gate / up rows [h I/8, (h+1) I/8) + SwiGLU  ->  down_proj restricted to
//                      that K-slice, ALL output rows, each added into the launch's sum row.
//
// The sum row: every output element receives eight contributions, one per XCD.  They are added as 64-bit
// fixed-point integers (2^-32 units) with memory-side atomic adds -- integer addition is associative, so the
// row does not depend on the order of arrival, and a contribution of magnitude >= 2^-8 is carried exactly.
// The NEXT launch reads the finished row behind the kernel boundary: every block takes the whole row (20 KB at
// hidden 2560), adds the residual, and has the vector and its sum of squares without waiting for any other
// block.  Three rows rotate: a launch reads one, adds into the second and clears the third for the launch
// after it.  Every block requests the weights of BOTH of its projections when it starts; the hand-overs only
// gate arithmetic.
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
//   abort          uint32   set when a wait ran into the spin limit
//   arrivals       uint32   device-wide barrier of the whole-token launch: XCD leaders arrived (memory-side adds)
//   release[8]     uint32   ... and the word each XCD's leader releases its XCD with
//   overflow       uint32   set when a contribution to a sum row was not finite or lay beyond the fixed-point range
//   placement[8]   uint64   one word per XCD, each in a 256-byte line of its own: every block of a launch flips bit
//                           `slot` of its XCD's word when it ends (a memory-side xor that returns nothing).  With one
//                           block per (XCD, slot) all 64 bits of a word flip together, so between launches every word
//                           is all zeros or all ones; anything else means two blocks shared a slot and the host
//                           reports it.  (Two blocks in one slot also leave some slot of another XCD empty, whose
//                           arrival word then never advances: the hand-over waits of that XCD give up and the launch
//                           already reports through the abort word.  The placement words name the cause.)
struct XcdPlacement {
    unsigned long long bits;
    uint32_t pad[62];
};
struct XcdControl {
    uint32_t flags[kXcds * kXcdSlots];
    uint32_t abort_flag;
    uint32_t arrivals;
    uint32_t release[kXcds];
    uint32_t overflow;
    uint32_t pad[53];
    XcdPlacement placement[kXcds];
};
static_assert(sizeof(XcdControl) == 2304 + 8 * 256, "control block layout");

// A sum row: hidden 64-bit fixed-point sums (value * 2^32), padded to whole 512-element sections.  Inside a
// section the elements are permuted so that the control wave of a block, whose lane l takes the eight
// elements 8 (l + 64 i) .. + 7 in step i, reads 1 KiB contiguous per instruction: element e sits at
// xcd_sum_index(e).
constexpr float kXcdSumScale = 4294967296.0f;
constexpr float kXcdSumInv = 1.0f / 4294967296.0f;
// Range of one contribution: |v| < 2^27, so that eight of them (one per XCD) stay far inside 64 bits.  A contribution
// at or beyond it, or one that is not finite, is clamped and raises XcdControl::overflow, which the host reports as
// an error (the reference's bf16 row would carry such a value on; a row of fixed-point sums cannot).  Resolution:
// 2^-32 per contribution, i.e. below half a bf16 step of any result of magnitude >= 2^-24.
constexpr float kXcdSumLimit = 134217728.0f;
__host__ __device__ inline uint32_t xcd_sum_index(uint32_t e) {
    const uint32_t t = e >> 3;
    return (((((t >> 6) * 4u + ((e & 7u) >> 1)) * 64u + (t & 63u)) << 1) | (e & 1u));
}
inline uint32_t xcd_sum_row_elems(uint32_t hidden) { return (hidden + 511u) / 512u * 512u; }

// One projection restricted to a row block and a K-slice: rows [row0, row0 + rows) of a [n, K] matrix,
// chunks [col0, col0 + cs) of each row's cpr 16-byte chunks.
struct XcdMat {
    const uint4* w;
    const uint16_t* sc;   // o_proj / down_proj: the per-XCD re-laid-out copies (fk_xcd_kslice_meta)
    const uint16_t* bi;
    uint32_t rows;     // rows of the matrix
    uint32_t cpr;      // chunks per full row
    uint32_t gshift;   // chunk index >> gshift = quantisation group
};

// The input of a launch: x[i] = T(f32(sums[i]) + residual[i]) (sums null: the residual alone), written to x_out
// by workgroup 0 and RMS-normalised with norm_w for the projections; f32(s) = fma(f32(low word), 2^-32,
// f32(high word)).
struct XcdInput {
    const long long* sums;      // sum row of the previous launch, or null
    const uint16_t* residual;   // [hidden]
    uint16_t* x_out;            // [hidden]
    long long* clear;           // sum row this launch zeroes (the one the launch after it adds into), or null
    const uint16_t* norm_w;
    float eps;
    uint32_t hidden;
    uint32_t row_elems;         // elements of a (padded) sum row
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
    long long* out_sums;        // sum row the down_proj outputs are added into
    XcdControl* ctl;
    uint32_t spin_limit;
    uint32_t cs_max, work_floats;  // LDS layout: chunks of the longest staged vector, floats of the work area
    uint32_t mark_placement;       // every block flips its bit of its XCD's placement word when it ends
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
    long long* out_sums;        // sum row the o_proj outputs are added into
    XcdControl* ctl;
    uint32_t spin_limit;
    uint32_t cs_max, work_floats, att_elems;  // LDS layout (att_elems: bf16 elements of the merged attention rows)
    uint32_t mark_placement;
};

// Every layer of a token in ONE launch: the attention and MLP phases of the two kernels above, layer after layer,
// with a device-wide barrier where the separate launches have a kernel boundary.  The per-layer argument blocks
// (exactly what the separate launches take) sit in device memory.
struct XcdTokenArgs {
    const XcdAttnArgs* attn;   // [n_layers]
    const XcdMlpArgs* mlp;     // [n_layers]
    uint32_t n_layers;
    XcdControl* ctl;
    uint32_t spin_limit;
    uint32_t xres_off;         // LDS offset (16-byte units) of the block's copy of the residual row
    uint32_t mark_placement;
};

// A whole layer in one launch: the attention phase, a device-wide barrier, the MLP phase (xcd_layer_kernel).  The two
// blocks are those of the stand-alone launches, by value.
struct XcdLayerArgs {
    XcdAttnArgs attn;
    XcdMlpArgs mlp;
    uint32_t xres_off;         // LDS offset (16-byte units) of the block's copy of the residual row
    uint32_t mark_placement;
};

// ---- the expert block of a mixture-of-experts layer as ONE launch ----------------------------------------------
// router + routed gate / up + shared gate / up + routed down + shared down + weighted sum, cut BY ROUTE: XCD u < top_k
// serves the u-th winner of the ranking entirely (its expert's gate / up rows, then its down_proj rows over the whole
// intermediate width).  A route's FULL dot product is therefore formed, rounded to T and weighted inside one XCD,
// exactly as the reference's reduction does it (routed_qmv_reduce.rs:236-322); only the final sum over the routes
// crosses XCDs, through the sum row.  The shared expert (width n_shared x an expert's) is n_shared more units of the
// same size on the following XCDs: unit h takes its gate / up rows [h I, (h+1) I) and the K-slice of the shared
// down_proj that those rows feed; its partial dot products go UNROUNDED into a second sum row, whose finished element
// is the shared expert's full dot product -- rounded to T where the row is read.  Every XCD streams the same bytes.
//   every XCD      x1 = T(sum row + residual); RMSNorm; staged
//   XCD u < top_k  block `slot` forms router logit `slot` (bf16 router row . normalised x) -> hand-over -> every wave
//                  ranks the 64 logits (softmax, top-k) and takes winner u: expert e, weight w
//   every unit     gate / up rows [slot I/64, (slot+1) I/64) of the unit, SwiGLU -> hand-over
//                  -> down_proj rows [slot H/64, ..) over the unit's intermediate row:
//                  routed: w * T(dot) into the sum row; shared: the partial dot into the second sum row
// What reads the rows forms x2 = T((f32(row) + T(f32(second row))) + residual): the reference's order of additions.
struct XcdMoeArgs {
    XcdInput in;
    const uint16_t* router_w;      // bf16 [experts, hidden]
    const uint16_t* route_scale;   // one bf16 value
    XcdMat gate, up, down;         // expert stacks: [experts * inter, hidden] twice, [experts * hidden, inter]
    XcdMat sgate, sup, sdown;      // shared expert: [shared_inter, hidden] twice, [hidden, shared_inter]
    uint32_t experts, top_k, n_shared, inter;
    uint32_t gu_rows;              // gate (and up) rows per block: inter / 64
    uint32_t down_rows;            // down_proj rows per block: hidden / 64
    int swiglu_variant;
    uint32_t* logits_xcd;          // [8][64] fp32 bits of the bf16 logits, every XCD its own copy
    uint16_t* mid;                 // [8][inter]: the SwiGLU row of every unit
    uint16_t* logits_out;          // [experts] bf16, or null   } what the host reads back; written by one block
    uint32_t* idx_out;             // [top_k] or null            }
    uint16_t* weight_out;          // [top_k] or null            }
    long long* out_sums;           // the routes' weighted outputs
    long long* out_sums2;          // the shared expert's dot products
    XcdControl* ctl;
    uint32_t spin_limit;
    uint32_t cs_max, work_floats;
    uint32_t mark_placement;
};

struct XcdMoeShape {
    uint32_t hidden, inter, shared_inter, experts, top_k, bits, group;
};
fk_status xcd_moe_supported(const XcdMoeShape& s);
size_t xcd_moe_scratch_bytes(const XcdMoeShape& s);   // logits_xcd + mid
struct XcdMoeRequest {
    XcdMoeShape shape;
    const long long* sums_in;
    const uint16_t* residual;
    uint16_t* x_out;
    long long* clear;
    const uint16_t* norm_w;
    float eps;
    const uint16_t* router_w;
    const uint16_t* route_scale;
    const fk_weight *gate, *up, *down, *sgate, *sup, *sdown;
    int swiglu_variant;
    uint16_t* logits_out;
    uint32_t* idx_out;
    uint16_t* weight_out;
    void* scratch;
    long long* out_sums;
    long long* out_sums2;
    void* workspace;
    uint32_t spin_limit;
    bool mark_placement;
};
fk_status plan_xcd_moe(const XcdMoeRequest& rq, Launch* out);

// ---- the attention half of a layer with low-rank keys as ONE launch -------------------------------------------
// (q = [q_nope | q_pe] per head from q_proj; kv_a -> [latent | k_pe]; RMSNorm(latent) -> kv_b -> per head [k_nope | v];
// K = [k_nope | rope(k_pe)], the rotated k_pe shared by all heads; n_heads / 8 heads per XCD.)
//   every XCD   x = T((f32(row) + T(f32(second row))) + residual) -- the rows of the previous layer's expert launch --
//               or a plain row; RMSNorm; staged
//   XCD u       q rows of its heads AND the whole kv_a row (every XCD forms the latent row itself: no hand-over
//               between XCDs; its copy lies in its own part of `kva`)  -> hand-over
//               -> latent RMSNorm, kv_b rows of its heads -> hand-over
//               -> rotation of q_pe / k_pe, cache append, attention: block = (head of the XCD, key range) -> hand-over
//               -> merge of the ranges -> o_proj restricted to the K-slice of its heads, all output rows, added into
//               the launch's sum row
struct XcdMlaArgs {
    XcdInput in;                // in.sums: the routes' row of the previous expert launch, or null
    const long long* sums2;     // the shared expert's row (with in.sums), or null
    long long* clear2;          // a second row this launch zeroes, or null
    XcdMat wq, wa, wb, wo;      // q_proj, kv_a_proj, kv_b_proj, o_proj (o_proj: per-XCD re-laid-out scales / biases)
    const uint16_t* a_norm;     // [rank] latent norm weight
    uint32_t hl;                // heads per XCD
    uint32_t q_rows;            // q rows of one XCD: hl * (nope + rope)
    uint32_t a_rows;            // rank + rope
    uint32_t rank;
    uint32_t b_total;           // kv_b rows of one XCD: hl * (nope + v)
    uint32_t tile_rows;         // rows per block tile of the q / kv_a projections
    uint32_t q_tiles, a_tiles;
    uint32_t b_rows;            // kv_b rows per block
    uint32_t o_rows, o_cs;      // o_proj output rows per block, chunks of one XCD's K-slice of an o_proj row
    uint16_t* q;                // [2][n_heads * (nope + rope)]: raw projection outputs, then the rows with q_pe rotated
    uint16_t* kva;              // [8][rank + rope]: every XCD's own copy of the latent row
    uint16_t* kvb;              // [n_heads * (nope + v)]
    SdpaArgs sdpa;              // geometry of the attention phase and the split-head parameters of the rotations
    long long* out_sums;
    XcdControl* ctl;
    uint32_t spin_limit;
    uint32_t cs_max, work_floats, att_elems;
    uint32_t mark_placement;
};

struct XcdMlaShape {
    uint32_t hidden, n_heads, rank, rope_dim, nope_dim, v_dim, capacity, bits, group;
};
fk_status xcd_mla_supported(const XcdMlaShape& s);
size_t xcd_mla_partials_bytes(const XcdMlaShape& s);
size_t xcd_mla_latent_bytes(const XcdMlaShape& s);   // the `kva` slot
struct XcdMlaRequest {
    XcdMlaShape shape;
    const long long* sums_in;
    const long long* sums2_in;
    const uint16_t* residual;
    uint16_t* x_out;
    long long* clear;
    long long* clear2;
    const uint16_t* norm_w;
    float eps;
    const fk_weight *wq, *wa, *wb, *wo;
    const uint16_t* a_norm;
    uint16_t *q, *kva, *kvb;
    uint16_t *cache_k, *cache_v;
    const uint32_t* kv_len;
    const float* rope_tab;
    float theta, scale;
    bool traditional;
    float* att_partials;
    long long* out_sums;
    void* workspace;
    uint32_t spin_limit;
    bool mark_placement;
};
fk_status plan_xcd_mla(const XcdMlaRequest& rq, Launch* out);

// x = T(f32(sums) + residual): the last layer's output for the LM head.  `clear` (may be the row read, or null)
// is zeroed element by element behind the read: the row the next token's first launch adds into.
struct XcdReduceArgs {
    const long long* sums;
    const uint16_t* residual;
    uint16_t* x;
    long long* clear;
    uint32_t hidden;
    // with a second row (the shared expert's of the expert launch): x = T((f32(sums) + T(f32(sums2))) + residual)
    const long long* sums2;
    long long* clear2;
    long long* clear3;   // one more row to zero, or null
};

struct XcdLayerShape {
    uint32_t hidden, inter, n_heads, n_kv, head_dim, capacity, bits, group;
};

// Can this layer shape run XCD-resident?  (8 KV heads, group of 1 / 2 / 4 / 8 query heads, slices that are
// whole quantisation groups, tiles that fit the per-thread load budget.)  Sets an error message if not.
fk_status xcd_layer_supported(const XcdLayerShape& s);
size_t xcd_workspace_bytes();
// Reads the control block after the launches that use it have completed (the caller has synchronised).  FK_OK when
// nothing was raised; otherwise the block is reset to zeros and FK_ERR_HIP says which of the three it was: a hand-over
// wait that gave up, a sum-row contribution outside the fixed-point range, two blocks of a launch in one slot.  After
// an error the sum rows the launches added into hold partial sums and the cache rows of the token's position may hold
// values built from unfinished rows: the caller zeroes the sum rows and decodes that token again (which rewrites the
// cache rows).
fk_status xcd_check_control(void* workspace);
size_t xcd_sum_row_bytes(uint32_t hidden);
// Scales (or biases) [n, groups] -> [8][n][groups / 8]: what the o_proj / down_proj slots of the launches take.
fk_status xcd_kslice_meta(const uint16_t* src, uint32_t n, uint32_t groups, uint16_t* dst, hipStream_t stream);
size_t xcd_attn_partials_bytes(const XcdLayerShape& s);

struct XcdAttnRequest {
    XcdLayerShape shape;
    const long long* sums_in;        // previous MLP launch's sum row, or null (first layer)
    const uint16_t* residual;
    uint16_t* x_out;
    long long* clear;
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
    long long* out_sums;
    void* workspace;
    uint32_t spin_limit;
    bool mark_placement;
    bool for_token = false;   // the block is meant for the whole-token launch (which runs the flavour with the pass loop)
};
fk_status plan_xcd_attn(const XcdAttnRequest& rq, Launch* out);

struct XcdMlpRequest {
    XcdLayerShape shape;
    const long long* sums_in;
    const uint16_t* residual;
    uint16_t* x_out;
    long long* clear;
    const uint16_t* norm_w;
    float eps;
    const fk_weight *wgate, *wup, *wdown;
    int swiglu_variant;
    uint16_t* mid;
    long long* out_sums;
    void* workspace;
    uint32_t spin_limit;
    bool mark_placement;
    bool for_token;   // the block is meant for the whole-token launch (its gate / up passes are shallower)
};
fk_status plan_xcd_mlp(const XcdMlpRequest& rq, Launch* out);
// One launch for an attention launch and the MLP launch that follows it (both as planned by plan_xcd_attn /
// plan_xcd_mlp in their one-pass flavours, the MLP launch reading the sum row the attention launch adds into and the
// row it writes as x_out): attention phase, device-wide barrier, MLP phase.  The MLP phase's first weight requests go
// out in front of the barrier.
fk_status plan_xcd_layer(const Launch& attn, const Launch& mlp, Launch* out);
// One launch for a run of alternating attention / MLP launches (as planned by plan_xcd_attn / plan_xcd_mlp, same
// weight kind): `d_attn` / `d_mlp` are device copies of their argument blocks.  Requirements beyond the separate
// launches': every layer has its own q / k / v rows (a block reads them with ordinary loads, and inside one launch
// a line of the previous layer's row may still sit in its L1).
fk_status plan_xcd_token(const XcdAttnArgs* h_attn, const XcdMlpArgs* h_mlp, uint32_t n_layers, uint32_t bits,
                         const XcdAttnArgs* d_attn, const XcdMlpArgs* d_mlp, uint32_t attn_lds, uint32_t mlp_lds, Launch* out);
fk_status plan_xcd_reduce(const long long* sums, const uint16_t* residual, uint16_t* x, long long* clear, uint32_t hidden,
                          Launch* out, const long long* sums2 = nullptr, long long* clear2 = nullptr, long long* clear3 = nullptr);

}  // namespace fk
