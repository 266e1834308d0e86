// Host-side plumbing shared by the launch planners and the C ABI: the Launch
// descriptor every planner fills (so a kernel can be launched directly or added
// to a hipGraph as a kernel node), error reporting and cached device facts.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <string>

#include "../../include/fusekit_hip.h"

namespace fk {

struct Launch {
    const void* func = nullptr;
    dim3 grid{1, 1, 1}, block{1, 1, 1};
    uint32_t shmem = 0;
    size_t args_size = 0;
    alignas(16) unsigned char args[640];

    template <typename T>
    void set_args(const T& a) {
        static_assert(sizeof(T) <= sizeof(args), "argument block too large");
        memcpy(args, &a, sizeof(T));
        args_size = sizeof(T);
    }
};

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
};
extern GemvPolicy g_gemv_policy;

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
};
fk_status plan_gemv(const GemvRequest& rq, Launch* out);

}  // namespace fk
