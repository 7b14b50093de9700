"""MI355X-native execution backend for the Tile contraction hot path.

hipkernels -- ctypes view of the kernel library C ABI (include/pml_hip.h)
"""
