"""MI355X-native stochastic-computing convolution path (LFSR streams, AND/OR/popcount
convolution with partial binary accumulation, surrogate backward).

``geo_amd.capi``              - Python callers of the C ABI (include/geo_sc.h)
``geo_amd.utils_functional``  - conv2d_generic / quantize with the reference's signatures
``geo_amd.utils_class``       - Conv2d_Add_Partial and the fixed-point batch norms
"""
__all__ = ["capi", "utils_functional", "utils_class", "workloads"]
