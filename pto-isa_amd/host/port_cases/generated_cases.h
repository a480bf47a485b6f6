// The case list that the reference's build generates for kernels/manual/common/flash_atten/fa_performance_kernel.cpp
// (its last lines instantiate LaunchTFA once per case: TFA_FOR_EACH_CASE(INSTANTIATE_TFA)); this is the list used when
// that source is compiled against include/pto for gfx950 (pto-isa_amd/build.py: build_ported).
//   M(S0, HEAD, S1, CUBE_S0, CUBE_S1, TILE_S1, QK_PRELOAD, CAUSAL_MASK)
// One workgroup plays the Cube core and the Vec core of a block in program order, so a case either has
// TILE_S1 == CUBE_S1 (the Vec side then never asks for a score tile of which the Cube side has produced only a part) or
// fits its whole key range into the preload (S1 <= QK_PRELOAD * TILE_S1).
#pragma once
#define TFA_FOR_EACH_CASE(M)                      \
    M(128, 128, 1024, 128, 128, 256, 4, false)    \
    M(256, 128, 2048, 128, 128, 128, 4, false)    \
    M(256, 128, 1024, 128, 128, 128, 4, true)     \
    M(512, 128, 2048, 128, 128, 128, 2, true)
