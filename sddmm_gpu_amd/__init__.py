"""MI355X-native SDDMM engine: host-side mirror of the C ABI in include/sddmm.h."""
