"""MI355X-native implementation of clDNN's quantized convolution hot path.

cldnn_amd.hip    -- ctypes binding of the thin C-ABI HIP layer (libcldnn_hip.so)
cldnn_amd/csrc   -- HIP kernels and the C-ABI itself
"""
