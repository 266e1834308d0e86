// fk_sdpa_decode for callers that cannot allocate device memory (code under hipGraph capture, tight serving
// loops, harnesses that forbid hipMalloc): the split-K workspace of the attention kernel -- partial (m, l, o)
// rows and the arrival counters -- lives in a file-scope device array instead of caller-provided buffers.
//
// Every GPU the library runs on holds its own copy of the array (kStaticScratchBytes, until the process ends)
// at its own address; the address is looked up once per device with hipGetSymbolAddress and kept.  All calls
// on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two threads) race on the
// partial rows and counters and must be serialised by the caller.
#include <mutex>

#include "fk_host.hpp"

namespace {

constexpr size_t kCounterBytes = 4096;                      // 1024 arrival counters
constexpr size_t kStaticScratchBytes = 9u * 1024u * 1024u;  // counters + partial rows: 32 heads x 128 dims up to 32768 positions
constexpr int kMaxDevices = 64;

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

std::mutex g_mu;
void* g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` per device ordinal, set on first use

// The device address of this GPU's copy of the array.  In host code `scratch` is only a handle for the
// symbol: the address a kernel may use comes from hipGetSymbolAddress, with the device current.
fk_status scratch_address(void** out) {
    int dev = -1;
    FK_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fk::set_error(FK_ERR_UNSUPPORTED, "fk_sdpa_decode_static: device ordinal out of range");
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        FK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fk::set_error(FK_ERR_HIP, "fk_sdpa_decode_static: the scratch symbol has no device address");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return FK_OK;
}

}  // namespace

extern "C" {

size_t fk_sdpa_static_scratch_bytes(void) { return kStaticScratchBytes; }

fk_status fk_sdpa_decode_static(const uint16_t* q, const uint16_t* cache_k, const uint16_t* cache_v, uint16_t* out,
                                const uint32_t* d_kv_len, uint32_t kv_len, uint32_t max_len, uint32_t n_heads,
                                uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim, uint32_t capacity, float scale,
                                fk_stream s) {
    using namespace fk;
    size_t pb = 0, cb = 0;
    FK_TRY(sdpa_workspace_bytes(n_heads, n_kv, qk_dim, v_dim, max_len ? max_len : 1, &pb, &cb));
    if (cb > kCounterBytes || pb > kStaticScratchBytes - kCounterBytes)
        return set_error(FK_ERR_UNSUPPORTED,
                         "fk_sdpa_decode_static: this problem needs " + std::to_string(pb + cb) +
                             " bytes of split-K workspace, the static scratch holds " +
                             std::to_string(kStaticScratchBytes - kCounterBytes) + " + " + std::to_string(kCounterBytes) +
                             "; use fk_sdpa_decode with a caller-provided workspace");
    void* base = nullptr;
    FK_TRY(scratch_address(&base));
    uint32_t* counters = reinterpret_cast<uint32_t*>(base);
    float* partials = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(base) + kCounterBytes);
    Launch attention, clear;
    FK_TRY(plan_sdpa_decode(q, cache_k, cache_v, out, d_kv_len, kv_len, max_len, n_heads, n_kv, qk_dim, v_dim, capacity,
                            scale, partials, counters, &attention));
    // The counters must be zero when the launch starts; the array keeps whatever the last call left (zero after
    // a complete launch, anything after one that was cut short).  A fill kernel, not a memset: a caller may be
    // capturing this stream into a graph.
    FK_TRY(plan_fill_u32(counters, 0u, kCounterBytes / 4, &clear));
    FK_TRY(run_launch(clear, (hipStream_t)s));
    return run_launch(attention, (hipStream_t)s);
}

}  // extern "C"
