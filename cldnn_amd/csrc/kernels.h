// Host-side launchers of the device kernels.
#pragma once
#include "common.h"

namespace chip {

struct ConvProblem {
    int B, IFM, IH, IW, OFM, OH, OW, FY, FX;
    int sy, sx, dy, dx, py, px, groups;
    int esy, esx;
    int in_dt, w_dt, out_dt, eltw_dt;
    cldnn_hip_tensor in_t, out_t, eltw_t;
    Pitch in_p, out_p, eltw_p;
};

// ---- layout-agnostic kernels (kernels_ref.hip)
void launch_conv_ref(hipStream_t s, const ConvProblem& p, const Epilogue& epi, const void* in, const void* w,
                     const void* eltw, void* out, int* acc_out);
void launch_eltwise(hipStream_t s, const cldnn_hip_eltwise_desc& d, const void* const* inputs, const float* calib, void* dst);
void launch_pooling(hipStream_t s, const cldnn_hip_pooling_desc& d, const void* in, void* out);
void launch_reorder(hipStream_t s, const cldnn_hip_tensor& st, const void* src, const cldnn_hip_tensor& dt, void* dst);
// src copied into dst with its element (0, 0, 0, 0) at (ob, of, oy, ox): one input of a concatenation
void launch_copy_region(hipStream_t s, const cldnn_hip_tensor& st, const void* src, const cldnn_hip_tensor& dt, void* dst, int ob, int of,
                        int oy, int ox);
// dst = act(a [+ b]); quantized: round((a + b) * (calib[f] or oqf)) saturated to char before the activation
void launch_pointwise(hipStream_t s, const cldnn_hip_tensor& at, const void* a, const cldnn_hip_tensor* bt, const void* b,
                      const cldnn_hip_tensor& dt, void* dst, int quantized, const float* calib, float oqf, int act, float m,
                      float n);

// ---- implicit-GEMM int8 MFMA kernel on fs_b_yx_fsv16 (conv_mfma*.hip)
struct TileConfig {
    const char* name;
    int tile_pixels;  // BM: output pixels per workgroup
    int tile_ofm;     // BN: output features per workgroup (multiple of 64)
    int wave_pixels;  // pixels per wave (4 waves: (BM / wave_pixels) * (BN / 64) == 4)
    int kgroups = 1;  // groups of four waves that split K inside the workgroup (direct-activation kernel)
};
int tile_config_count();
const TileConfig& tile_config(int i);

// Pre-packed weights and launch geometry of one convolution for the MFMA kernel.
struct MfmaPlan {
    int tile;            // row of the tile table
    int stream;          // 1: streaming kernel (no LDS), 0: LDS-staged tile kernel
    int bdir;            // 1: direct-activation tile kernel (weights through LDS, activations into registers)
    int stem;            // 1: first-layer row (b_fs_yx_fsv4 input, streaming kernel)
    int by_features;     // 1: accelerator dies split the feature tiles (weights larger than activations)
    int wsl;             // 1: weights-stationary persistent kernel (weight tile resident in LDS)
    int wsl_depth;       // its activation look-ahead in K-steps
    int wsl_parts;       // pixel-range partitions per feature tile (multiple of 8)
    int wsl_tpp;         // pixel tiles per partition
    int gemv;            // 1: few pixels, long K: 16-feature fragments, waves split K (no LDS in the loop)
    int gemv_waves;      // its waves per workgroup
    int halo;            // 1: nine-tap stride-1 kernel with both operands staged in LDS by direct loads (conv_halo_kernel.h)
    int halo_patch_len;  // its patch length in positions per slice (multiple of 64)
    int halo_parts;      // its workgroups per feature tile (multiple of 8)
    int halo_ptiles;     // its position tiles (positions count the input's border)
    int halo_pl;         // its patch wave-loads per wave and requesting step
    int block;           // threads per workgroup
    int checked;         // 1: taps bounds-checked per load, 0: input carries a sufficient zero border
    int tap_minor;       // K order: 1 = (group of 4 slices, tap), taps innermost; 0 = (tap, slice)
    int cb;              // input feature slices of 16
    int kchunks;         // FY*FX*cb
    int ksteps;          // ceil(kchunks / 4)
    int ofm_tiles;       // ceil(OFM / tile_ofm)
    int mtiles;          // ceil(M / tile_pixels)
    int64_t m_total;     // B*OH*OW
    int grid;
    int lds_bytes;
    size_t packed_bytes; // device bytes of the packed weight stream
    size_t ktab_bytes;
};
// table lookup: row of the tile table for a problem
int mfma_choose(const ConvProblem& p, int cus);
MfmaPlan mfma_plan(const ConvProblem& p, int tile, int cus);
// host-side packing: weights [OFM][IFM][FY][FX] s8 -> MFMA operand stream, ktab -> per-kchunk tap table
void mfma_pack_weights(const ConvProblem& p, const MfmaPlan& plan, const int8_t* w, int8_t* packed, int32_t* ktab);
struct MfmaBuffers {
    const int8_t* packed;
    const int32_t* ktab;
    void* gather = nullptr;  // small-batch kernel with a filter wider than one tap: mfma_gather_bytes() of scratch
};
size_t mfma_gather_bytes(const ConvProblem& p, const MfmaPlan& pl);  // 0 when the plan needs no scratch
// The same scratch without an allocation: a fixed-size array inside the loaded code object, one copy per device.
// mfma_static_scratch returns its device address on `device`, which must be the current device.
size_t mfma_static_scratch_bytes();
void* mfma_static_scratch(int device);
// parameters of the short epilogue (int8 output, float requantisation)
struct FastEpi {
    int32_t has_wqf;      // multiply by wqf[f] and iqf
    int32_t act;          // CLDNN_HIP_ACT_NONE / RELU / CLAMP
    float act_m, act_n;
    int32_t relu_folded;  // relu with non-negative scales: folded into the final clamp
    int32_t fused;
    int32_t eltw_act;     // NONE / RELU / CLAMP
    float eltw_m, eltw_n;
    int32_t has_ecal;
    int32_t eltw_relu_folded;  // residual relu with non-negative scales: folded into the final clamp
    int32_t eltw_u8;
    float lo, hi;         // saturation bounds of the output type
    float iqf;
    int32_t iqf_one;      // iqf == 1: the multiplication is left out (x * 1.0f == x)
    int32_t clamp_folded; // clamp{m, n} with 0 <= m <= n, factors >= 0 and n * factor inside the output range: the result
                          // needs no second clamp and rounds like a non-negative number
    int32_t conv_sat;     // fused: the rounded convolution result is limited to [conv_lo, conv_hi] before the sum
    float conv_lo, conv_hi;
    int32_t fc;           // the fully_connected form: float bias after the dequantisation, conversion to char keeps the low byte
    // two convolutions of one input in one launch: a 16-feature group with at most split_valid features from its start
    // to the end of the output belongs to the second one and clamps from lo2 instead of lo (0 for a folded relu, the
    // type's lower bound without activation).  split_valid == 0: one convolution.
    int32_t split_valid;
    float lo2;
};
// true (and *out filled) when the short epilogue reproduces the long one bit for bit
bool mfma_fast_epilogue(const ConvProblem& p, const Epilogue& e, const float* calib, const float* ecal, const float* wqf,
                        FastEpi* out);
// acc_init: per-feature int32 start value of the accumulators, padded to ofm_tiles * tile_ofm.
// fast == nullptr selects the long epilogue; raw != nullptr dumps the int32 accumulators instead.
void launch_conv_mfma(hipStream_t s, const ConvProblem& p, const MfmaPlan& plan, const MfmaBuffers& wb,
                      const int32_t* acc_init, const Epilogue& epi, const FastEpi* fast, const void* in, const void* eltw,
                      void* out, int32_t* raw);

// ---- depthwise bandwidth kernel on fs_b_yx_fsv16 (conv_dw.hip)
struct DwPlan {
    int grid, block;
    size_t packed_bytes;
    size_t mask_bytes;  // masked weight dwords of the 3x3 kernel
};
DwPlan dw_plan(const ConvProblem& p);
void dw_pack_weights(const ConvProblem& p, const int8_t* w, int8_t* packed);
void dw_mask_weights(const ConvProblem& p, const int8_t* w, int32_t* masked);
bool dw_fast_applies(const ConvProblem& p, bool fast_epilogue);
bool conv_border_covers(const ConvProblem& p);
void launch_conv_dw(hipStream_t s, const ConvProblem& p, const DwPlan& plan, const int8_t* packed, const int32_t* masked,
                    const int32_t* acc_init, const Epilogue& epi, const FastEpi* fast, const void* in, const void* eltw,
                    void* out, int32_t* raw);

}  // namespace chip
