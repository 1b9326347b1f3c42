"""MI355X (gfx950) implementation of mimir's quantized-matmul decode path.

mimir_amd.capi binds the C ABI (include/mimir_mi355x.h); mimir_amd.build
compiles the HIP sources under mimir_amd/csrc; mimir_amd.mimfile reads .mim
model files.
"""
