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
void launch_reorder(hipStream_t s, const cldnn_hip_tensor& st, const void* src, const cldnn_hip_tensor& dt, void* dst);

// ---- implicit-GEMM int8 MFMA kernel on fs_b_yx_fsv16 (conv_mfma.hip)
struct TileConfig {
    const char* name;
    int tile_pixels;  // BM: output pixels per workgroup
    int tile_ofm;     // BN: output features per workgroup (multiple of 64)
    int wave_pixels;  // pixels per wave (4 waves: (BM / wave_pixels) * (BN / 64) == 4)
};
int tile_config_count();
const TileConfig& tile_config(int i);

// Pre-packed weights of one convolution for the MFMA kernel.
struct MfmaPlan {
    int tile;            // row of the tile table
    int cb;              // input feature slices of 16 (per group)
    int kchunks;         // FY*FX*cb
    int ksteps;          // ceil(kchunks / 4)
    int ofm_tiles;       // ceil(OFM / tile_ofm)
    int64_t m_total;     // B*OH*OW
    int grid;
    int lds_bytes;
    size_t packed_bytes; // device bytes of the packed weight stream
    size_t ktab_bytes;
};
MfmaPlan mfma_plan(const ConvProblem& p, int tile);
// host-side packing: weights [OFM][IFM][FY][FX] s8 -> MFMA operand stream, ktab -> per-kchunk tap table
void mfma_pack_weights(const ConvProblem& p, const MfmaPlan& plan, const int8_t* w, int8_t* packed, int32_t* ktab);
struct MfmaBuffers {
    const int8_t* packed;
    const int32_t* ktab;
};
enum { EPI_GENERIC = 0, EPI_RAW = 1, EPI_FAST = 2 };
// true when the short epilogue (convert, scale, clamp, round) reproduces the generic one bit for bit
bool mfma_fast_epilogue_ok(const ConvProblem& p, const Epilogue& e, const float* calib_host, const float* ecal_host,
                           const float* wqf_host, int ofm);
// acc_init: per-feature int32 start value of the accumulators, padded to ofm_tiles * tile_ofm
void launch_conv_mfma(hipStream_t s, const ConvProblem& p, const MfmaPlan& plan, const MfmaBuffers& wb,
                      const int32_t* acc_init, const Epilogue& epi, int epi_kind, const void* in, const void* eltw,
                      void* out, int32_t* raw);

// ---- depthwise bandwidth kernel on fs_b_yx_fsv16 (conv_dw.hip)
struct DwPlan {
    int grid, block;
    size_t packed_bytes;
};
DwPlan dw_plan(const ConvProblem& p);
void dw_pack_weights(const ConvProblem& p, const int8_t* w, int8_t* packed);
void launch_conv_dw(hipStream_t s, const ConvProblem& p, const DwPlan& plan, const int8_t* packed, const int32_t* acc_init,
                    const Epilogue& epi, const void* in, const void* eltw, void* out, int32_t* raw);

}  // namespace chip
