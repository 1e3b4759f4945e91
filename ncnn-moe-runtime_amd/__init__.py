"""MI355X-native generation sampler for the ncnn-MoE-Runtime Session/BatchScheduler sampling path.

The product is the C-ABI library built from csrc/ (see include/ncnn_moe_hip_sampler.h); this package
holds the build recipe, a ctypes binding used by the tests and the benchmark, and the seeded
workload generator for the benchmark configurations.
"""
