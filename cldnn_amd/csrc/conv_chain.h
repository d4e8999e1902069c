// Host-side interface of the convolution chain kernel (conv_chain.hip): two or three quantized convolutions in one
// launch, each stage feeding the next from registers.
#pragma once
#include <string>

#include "kernels.h"

namespace chip {

// what the chain needs to know about one stage (all of it lives in the stage's convolution object)
struct ChainStageIn {
    const ConvProblem* p;
    const Epilogue* epi;       // device pointers of the per-feature vectors inside
    const FastEpi* fe;
    bool fast;                 // the short int8 epilogue applies
    const int32_t* acc_init;   // device
    // a depthwise first stage (3x3, masked weights of the stand-alone depthwise kernel): device pointers, else nullptr
    const int32_t* dw_wmask = nullptr;
};

struct ChainPlan {
    int stages;
    int dw;                    // 1: the first stage is a depthwise 3x3 on the vector ALU (granules of 64 pixels), the LDS
                               // image holds the units and vectors of the later stages only
    int nt;                    // 16-pixel fragments per wave and granule
    int depth;                 // activation look-ahead of stage 0 in K-steps
    int ksteps0;               // K-steps of stage 0 (padded to a multiple of depth)
    int sp[3];                 // 64-feature spans per stage
    int epi[3];                // epilogue kind per stage
    int unit0[3], kstride[3];  // LDS image: first 4 KB unit and units per span of every stage
    int vec0[3];               // first dword of every stage's per-feature vectors behind the weights
    int units;
    int lds_bytes;
    int grid;
    int granules;
    int64_t m_total;
    char name[96];
};

// empty string: the chain can run and *out is filled; otherwise the reason why not
std::string chain_plan(const ChainStageIn* st, int n, int cus, ChainPlan* out);
size_t chain_packed_bytes(const ChainPlan& pl);
// host copies of one stage's per-feature vectors, OFM entries each (nullptr: absent)
struct ChainVectors {
    const int32_t* acc_init;
    const float* calib;
    const float* eltw_calib;
    const float* wqf;
};
// w[k]: dense host weights of stage k, [ofm][ifm][fy][fx].  The image is what a workgroup copies into LDS: the weight
// units of all stages, then their per-feature vectors.
void chain_pack_weights(const ChainStageIn* st, const ChainPlan& pl, int cus, const int8_t* const* w, const ChainVectors* vec,
                        int8_t* packed);
// outs[k] == nullptr: stage k's result is not written; eltws[k]: residual operand of a fused stage
void launch_conv_chain(hipStream_t s, const ChainStageIn* st, const ChainPlan& pl, const void* packed_dev, const void* in,
                       void* const* outs, const void* const* eltws);

}  // namespace chip
