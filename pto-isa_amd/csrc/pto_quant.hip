// Block-scaled quantisation of fp32 to MXFP8 for MI355X: e4m3 elements, one e8m0 scale per 32 consecutive elements, the
// operand format of pto_gemm_mxfp8 (A [m, k] with its scales [m, k / 32], B [n, k] likewise).
//
// Mirrors TQUANT<QuantType::MXFP8> of the reference (include/pto/npu/a5/TQuant.hpp:262-322 TQuant_MXFP8: the absolute
// maximum of every group :35-126, the shared exponent and the reciprocal scale :128-180, the scaled conversion :182-224)
// and its generator (tests/npu/a5/src/st/testcase/tquant/gen_data.py:43-57, :27-33):
//   E = biased fp32 exponent of the group's largest |x|;  e8m0 = E - 8;  q = e4m3(clip(x * 2^(127 - e8m0), +-448)),
// round to nearest even.  A group with an infinity or a NaN gets e8m0 = 0xff and NaN -> NaN, +-inf -> +-448, finite -> +-0;
// a group whose maximum is below 2^-119 (a zero group included) gets e8m0 = 0 and the factor 2^127.
//
// The reference quantises one Vec tile in its unified buffer with vector-register loops.  Here the matrix is a stream:
// a lane loads 16 bytes (four fp32) so that a wave's load instruction covers 1 KiB of consecutive addresses, a group of 32
// is eight neighbouring lanes whose maxima are combined with three lane moves, a lane converts its four values with the
// hardware conversion (two per v_cvt_pk_fp8_f32, round to nearest even) and stores 4 bytes, the first lane of every
// eight stores the scale byte.  Eight loads per lane are in flight before the first use; no LDS, no barrier.
#include <hip/hip_runtime.h>

#include "common.hpp"

namespace {

constexpr int kQuantThreads = 256, kQuantSteps = 8, kQuantPerStep = kQuantThreads * 4, kQuantTile = kQuantPerStep * kQuantSteps;

typedef float f32x4 __attribute__((ext_vector_type(4)));

// largest value among the eight lanes of a group (lanes 8g .. 8g + 7 of a row of 16)
__device__ inline uint32_t MaxOverEight(uint32_t v)
{
    uint32_t o = (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xf, 0xf, true); // quad_perm [1,0,3,2]
    v = v > o ? v : o;
    o = (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xf, 0xf, true); // quad_perm [2,3,0,1]
    v = v > o ? v : o;
    o = (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x141, 0xf, 0xf, true); // row_half_mirror: lane i <-> 7 - i of its eight
    return v > o ? v : o;
}

__device__ inline uint32_t QuantFour(f32x4 x, uint8_t &scaleByte)
{
    uint32_t a = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t u = __float_as_uint(x[j]) & 0x7fffffffu;
        a = u > a ? u : a; // as integers: a NaN is above every number
    }
    const uint32_t E = MaxOverEight(a) >> 23;
    if (E == 255u) { // wave-divergent and rare
        scaleByte = 0xffu;
        uint32_t out = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t u = __float_as_uint(x[j]), mag = u & 0x7fffffffu;
            const uint32_t code = ((u >> 24) & 0x80u) | (mag > 0x7f800000u ? 0x7fu : mag == 0x7f800000u ? 0x7eu : 0u);
            out |= code << (8 * j);
        }
        return out;
    }
    const uint32_t se = E < 8u ? 0u : E - 8u;
    scaleByte = (uint8_t)se;
    const float scale = __uint_as_float((254u - se) << 23);
    float y[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
        y[j] = __builtin_fminf(__builtin_fmaxf(x[j] * scale, -448.0f), 448.0f);
    int packed = 0;
    packed = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], packed, false);
    packed = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], packed, true);
    return (uint32_t)packed;
}

// kTail: the last, partial tile (n is a multiple of 32, so groups and lanes are whole)
template <bool kTail>
__global__ __launch_bounds__(kQuantThreads) void QuantMxFp8(uint8_t *q, uint8_t *e8m0, const float *src, size_t n, size_t firstTile)
{
    const size_t base = (firstTile + blockIdx.x) * (size_t)kQuantTile + 4 * threadIdx.x;
    f32x4 x[kQuantSteps];
#pragma unroll
    for (int i = 0; i < kQuantSteps; ++i) {
        const size_t at = base + (size_t)i * kQuantPerStep;
        if (!kTail || at < n)
            x[i] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src + at));
        else
            x[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int i = 0; i < kQuantSteps; ++i) {
        const size_t at = base + (size_t)i * kQuantPerStep;
        uint8_t scaleByte;
        const uint32_t four = QuantFour(x[i], scaleByte); // every lane takes part in the lane moves
        if (!kTail || at < n) {
            __builtin_nontemporal_store(four, reinterpret_cast<uint32_t *>(q + at));
            if ((threadIdx.x & 7) == 0)
                e8m0[at >> 5] = scaleByte;
        }
    }
}

} // namespace

extern "C" int pto_quant_mxfp8_f32(void *stream, uint8_t *q, uint8_t *scale, const float *src, size_t rows, size_t cols)
{
    if (rows == 0 || cols == 0)
        return PTO_OK;
    if (!q || !scale || !src)
        return PTO_ERR_BAD_ARG;
    if (cols % 32 || reinterpret_cast<uintptr_t>(src) % 16 || reinterpret_cast<uintptr_t>(q) % 4)
        return PTO_ERR_UNSUPPORTED; // whole groups; 16-byte loads and 4-byte stores at their natural alignment
    if (rows > ((size_t)1 << 62) / cols)
        return PTO_ERR_UNSUPPORTED;
    const size_t n = rows * cols, full = n / kQuantTile, tail = n % kQuantTile;
    hipStream_t st = static_cast<hipStream_t>(stream);
    constexpr size_t kMaxBlocks = 1u << 30;
    for (size_t t0 = 0; t0 < full; t0 += kMaxBlocks) {
        const size_t nb = full - t0 < kMaxBlocks ? full - t0 : kMaxBlocks;
        QuantMxFp8<false><<<dim3((unsigned)nb), dim3(kQuantThreads), 0, st>>>(q, scale, src, n, t0);
    }
    if (tail)
        QuantMxFp8<true><<<dim3(1), dim3(kQuantThreads), 0, st>>>(q, scale, src, n, full);
    return pto_amd::check_launch();
}
