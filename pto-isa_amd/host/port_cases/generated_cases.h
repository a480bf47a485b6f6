// The case list that the reference's build generates for kernels/manual/common/flash_atten/fa_performance_kernel.cpp
// (its last lines instantiate LaunchTFA once per case: TFA_FOR_EACH_CASE(INSTANTIATE_TFA)); this is the list used when
// that source is compiled against include/pto for gfx950 (pto-isa_amd/build.py: build_ported).
//   M(S0, HEAD, S1, CUBE_S0, CUBE_S1, TILE_S1, QK_PRELOAD, CAUSAL_MASK)
// The first four are the reference generator's defaults (scripts/gen_data.py:192-199: CUBE_S1 = 128, TILE_S1 = 256,
// QK_PRELOAD = 4) at S1 = 1024, 2048 and 8192; the others vary the tile width, the preload and the mask.
#pragma once
#define TFA_FOR_EACH_CASE(M)                      \
    M(128, 128, 1024, 128, 128, 256, 4, false)    \
    M(128, 128, 2048, 128, 128, 256, 4, false)    \
    M(128, 128, 8192, 128, 128, 256, 4, false)    \
    M(512, 128, 2048, 128, 128, 256, 4, false)    \
    M(256, 128, 2048, 128, 128, 256, 2, true)     \
    M(256, 128, 2048, 128, 128, 128, 4, false)    \
    M(256, 128, 1024, 128, 128, 128, 4, true)     \
    M(512, 128, 2048, 128, 128, 128, 2, true)
