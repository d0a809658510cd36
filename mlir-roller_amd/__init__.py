"""MI355X-native Roller fp32 GEMM: rTile policy on the host, hand-written gfx950 MFMA kernel
template JIT-compiled through hiprtc, driven over the C ABI of libroller_hip.so."""
