// Shared host/device declarations of the HIP layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <stdexcept>
#include <string>

#include "../../include/cldnn_hip.h"

namespace chip {

// ----------------------------------------------------------------------------- errors
struct error : std::runtime_error {
    cldnn_hip_status status;
    error(cldnn_hip_status s, const std::string& m) : std::runtime_error(m), status(s) {}
};

void set_last_error(const std::string& m);

#define CHIP_CHECK(expr)                                                                              \
    do {                                                                                              \
        hipError_t e_ = (expr);                                                                       \
        if (e_ != hipSuccess)                                                                         \
            throw ::chip::error(CLDNN_HIP_DEVICE_ERROR, std::string(#expr) + ": " + hipGetErrorString(e_)); \
    } while (0)

#define CHIP_REQUIRE(cond, status, msg)                      \
    do {                                                     \
        if (!(cond)) throw ::chip::error((status), (msg));   \
    } while (0)

// ----------------------------------------------------------------------------- tensor addressing
// element index of (b, f, y, x) = off + b*pb + (f / fsv)*pf + y*py + x*px + (f % fsv)
// (fsv == 1 for the plain formats; padding is folded into off)
struct Pitch {
    int64_t off, pb, pf, py, px;
    int32_t fsv;
    int32_t fs_count;  // feature slices physically present (padded feature count / fsv)
    __host__ __device__ int64_t at(int b, int f, int y, int x) const
    {
        return off + (int64_t)b * pb + (int64_t)(f / fsv) * pf + (int64_t)y * py + (int64_t)x * px + (f % fsv);
    }
};

Pitch make_pitch(const cldnn_hip_tensor& t);
size_t dtype_size(int dt);
size_t tensor_elems(const cldnn_hip_tensor& t);

// ----------------------------------------------------------------------------- epilogue description
enum { MODE_Q = 0, MODE_FINT = 1, MODE_NAT = 2 };

struct Epilogue {
    const void* bias;        // int32 or float, [ofm_padded]
    const float* wqf;        // nullptr when absent
    const float* calib;      // nullptr when absent
    const float* eltw_calib; // nullptr when absent
    int32_t mode;
    int32_t bias_dt;         // CLDNN_HIP_I32 / F32 / NO_TYPE
    int32_t bias_after;      // f32 bias added after dequantisation
    int32_t oqf_on;
    float iqf, oqf;
    int32_t act;
    float act_m, act_n;
    int32_t fused;
    int32_t ncs_on;
    float ncs;
    int32_t eltw_act;
    float eltw_m, eltw_n;
    int32_t out_dt, eltw_dt, in_dt;
    int32_t round_even;
    int32_t fc;              // quantized fully_connected form (see cldnn_hip_conv_desc.fully_connected)
    int32_t conv_sat;        // fused form: 1 / 2 = the rounded convolution result is saturated to s8 / u8 before the sum
    int32_t split_f;         // > 0: features from here on take act2 (two convolutions of one input in one launch)
    int32_t act2;
    float act2_m, act2_n;
};

}  // namespace chip
