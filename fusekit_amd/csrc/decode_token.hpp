// Whole-token persistent decode kernel: arguments shared by device and host.
#pragma once
#include "fk_host.hpp"
#include "gemv_kernel.hpp"
#include "sdpa_kernel.hpp"

namespace fk {

struct TokenArgs {
    // Per layer four GEMV phases (qkv, o_proj, gate/up, down), then the LM head:
    // gemv[4 * n_layers + 1], sdpa[n_layers]; both arrays live in device memory.
    const GemvArgs* gemv;
    const SdpaArgs* sdpa;
    uint32_t n_layers;
    // embedding lookup (dense bf16 table) into x0
    const uint16_t* embed;
    uint16_t* x0;
    uint32_t hidden, vocab;
    float embed_scale;
    // rotary table of this token, filled in the first phase: (cos, sin) per pair
    float* rope_tab;
    uint32_t rope_dims;
    float rope_base_log2;
    // per-token protocol (python_runtime/src/lib.rs:1299-1303, kernels/mod.rs:544-577)
    uint32_t* token;         // in: token to embed; out: greedy next token
    uint32_t* step_counter;  // offset = step_counter++ ; kv_len = offset + 1
    uint32_t* offset;
    uint32_t* kv_len;
    uint32_t* history;
    uint32_t* hist_counter;
    uint32_t hist_capacity;
    // argmax over the logits the LM head phase wrote
    const uint16_t* logits;
    unsigned long long* argmax_partial;  // [grid]
    // grid barrier: monotonic two-level arrival counters, the released-epoch flag,
    // the epoch at launch start and an abort flag (set when a wait exceeds
    // spin_limit polls; every later wait then returns at once, so all waves drain)
    unsigned long long* bar_groups;   // one arrival counter per group of blocks, 128 bytes apart
    unsigned long long* bar_counter;  // arrivals of whole groups
    unsigned long long* bar_flag;     // last barrier every block may pass
    unsigned long long* bar_base;     // barriers passed when the launch starts
    uint32_t* abort_flag;
    uint32_t spin_limit;
    // optional: block 0 stamps the constant-rate clock (100 MHz) after every barrier,
    // trace[0] at entry; the per-phase profile of the last launch (null = off)
    unsigned long long* trace;
    uint32_t trace_capacity;
};

struct TokenKernelSpec {
    int kind;  // WKind of the layer projections
    int gt;    // query heads per kv head tile (2, 4 or 8)
    uint32_t lds_bytes;
    TokenArgs args;
};

fk_status token_kernel_max_grid(int kind, int gt, uint32_t lds_bytes, uint32_t* grid);
fk_status plan_token_kernel(const TokenKernelSpec& spec, uint32_t grid, Launch* out);

}  // namespace fk
