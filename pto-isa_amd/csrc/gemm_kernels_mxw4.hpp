// MXFP8 GEMM tile of 256 x BN (BN = 192 or 128) on four wavefronts: the four-wave fp16 kernel of gemm_kernels_w4.hpp with
// 8-bit operands.  A K-step is the same 128 bytes per operand row (128 k instead of 64), so copies, LDS images and fragment
// reads are byte for byte those of the fp16 kernel; what differs:
//   * one v_mfma_scale_f32_16x16x128_f8f6f4 (8 passes) per 16 x 16 block and step instead of two v_mfma_f32_16x16x32_f16
//     (4 passes each).  Its operand registers hold, for lane group g = lane / 16, bytes 16 g .. + 15 of the row's first 64
//     k and bytes 64 + 16 g .. + 15 of its second 64 k: exactly the two reads of the fp16 kernel;
//   * the block scales (one e8m0 byte per row and 32 k = per lane and MFMA exactly one byte).  The MFMAs of four steps
//     (512 k = 16 scale bytes of a row) take theirs from one register per block row / column: byte j = the scale of the
//     lane's k block g in step j (op_sel selects j).  These registers are made for 16 steps (64 scale bytes of a row) at
//     once: lane group g loads bytes 16 g .. + 15 of the 64 straight from memory (one instruction and one cache line per
//     row for 16 steps), transposes its 4 x 4 bytes (register u = byte u of each k-block quadruple: what lane group u
//     needs) and the four lane groups exchange register u of group g with register g of group u (two
//     v_permlane32_swap, two v_permlane16_swap).  One block row / column per step: load at the start of the step,
//     permutes and swaps behind its barrier, into the set of the next 16 steps;
//   * four B stages (96 + 64 KiB = the whole LDS at BN = 192), which makes the step's second barrier unnecessary: a
//     stage is overwritten two steps after its last read, with the barrier of the step in between.
// Steps come in groups of four (B stage, A slot and scale byte repeat): k % 512 == 0.
// MXFP4 (format 4, two e2m1 per byte): a K-step of 128 bytes is 256 k = two MFMAs (4 passes each, 16-byte operands: lane group
// g holds bytes 16 g .. + 15 of the MFMA's 64) and eight scale blocks per row, so a scale register lasts two steps (the MFMA of
// step j % 2 and half kk selects byte 2 (j % 2) + kk), the 64 scale bytes of a row eight steps, and two block rows / columns
// are loaded per step: k % 1024 == 0.
#pragma once
#include "gemm_kernels_w4.hpp"

PTO_DEVICE_CODE_BEGIN
namespace {

// acc block BLK += first x second (both 16 rows x 128 k bytes) with their scales, scale byte SEL of either register
template <int BLK, int SEL, int FMT_FIRST, int FMT_SECOND>
PTO_DEV void MxW4Mfma(i32x8 first, i32x8 second, uint32_t scaleFirst, uint32_t scaleSecond)
{
#define X(b, r0, r1, r2, r3)                                                                                                          \
    if constexpr (BLK == b)                                                                                                           \
        asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[" #r0 ":" #r3 "], %0, %1, a[" #r0 ":" #r3 "], %2, %3 op_sel:[%4,%4,0] "       \
                     "op_sel_hi:[%5,%5,0] cbsz:%6 blgp:%7" ::"v"(first),                                                              \
                     "v"(second), "v"(scaleFirst), "v"(scaleSecond), "n"(SEL & 1), "n"(SEL >> 1), "n"(FMT_FIRST), "n"(FMT_SECOND)    \
                     : "a" #r0, "a" #r1, "a" #r2, "a" #r3);
    PTO_W4_ACC_BLOCKS(X)
#undef X
}

// the same with 4-bit operands: 16 rows x 128 k = 64 bytes per row, 16 per lane
template <int BLK, int SEL>
PTO_DEV void MxW4MfmaFp4(u32x4 first, u32x4 second, uint32_t scaleFirst, uint32_t scaleSecond)
{
#define X(b, r0, r1, r2, r3)                                                                                                          \
    if constexpr (BLK == b)                                                                                                           \
        asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[" #r0 ":" #r3 "], %0, %1, a[" #r0 ":" #r3 "], %2, %3 op_sel:[%4,%4,0] "       \
                     "op_sel_hi:[%5,%5,0] cbsz:4 blgp:4" ::"v"(first),                                                                \
                     "v"(second), "v"(scaleFirst), "v"(scaleSecond), "n"(SEL & 1), "n"(SEL >> 1)                                      \
                     : "a" #r0, "a" #r1, "a" #r2, "a" #r3);
    PTO_W4_ACC_BLOCKS(X)
#undef X
}

// 16 bytes per lane from memory as assembly (counted by the kernel's own waits); use the result only behind such a wait
PTO_DEV u32x4 MxW4Load16(const char *base, uint32_t voff)
{
    u32x4 r;
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(r) : "v"(voff), "s"(base) : "memory");
    return r;
}

// (the compiler does not see that the load above is still on its way: a value is used only behind one of these)
PTO_DEV void MxW4Pin(u32x4 &x) { asm volatile("" : "+v"(x)); }
PTO_DEV void MxW4WaitLoads(u32x4 &x) { asm volatile("s_waitcnt vmcnt(0)" : "+v"(x)::"memory"); }

// w = the 16 scale bytes that this lane's group g loaded (bytes 16 g .. + 15 of the 64 of its row) -> out[u] = bytes g, 4 + g,
// 8 + g, 12 + g of the 16 bytes that group u loaded: the scales of the lane's k block in the four MFMA rounds of quarter u
// In four parts, each a few instructions between two MFMAs; w is worked on in place and holds out[0 .. 3] after part 3.
template <int PART>
PTO_DEV void MxW4ScaleSpreadPart(u32x4 &w)
{
    if constexpr (PART == 0) { // bytes transposed within the lane: register u = byte u of w[0], w[1], w[2], w[3], in two rounds
        const uint32_t t0 = __builtin_amdgcn_perm(w[1], w[0], 0x05010400u), t1 = __builtin_amdgcn_perm(w[1], w[0], 0x07030602u);
        const uint32_t t2 = __builtin_amdgcn_perm(w[3], w[2], 0x05010400u), t3 = __builtin_amdgcn_perm(w[3], w[2], 0x07030602u);
        w = u32x4{t0, t1, t2, t3};
    } else if constexpr (PART == 1) {
        const uint32_t p0 = __builtin_amdgcn_perm(w[2], w[0], 0x05040100u), p1 = __builtin_amdgcn_perm(w[2], w[0], 0x07060302u);
        const uint32_t p2 = __builtin_amdgcn_perm(w[3], w[1], 0x05040100u), p3 = __builtin_amdgcn_perm(w[3], w[1], 0x07060302u);
        w = u32x4{p0, p1, p2, p3};
    } else if constexpr (PART == 2) { // registers transposed against lane groups: (register u of group g) <-> (register g of group u)
        const auto a = __builtin_amdgcn_permlane32_swap(w[0], w[2], false, false), b = __builtin_amdgcn_permlane32_swap(w[1], w[3], false, false);
        w = u32x4{a[0], b[0], a[1], b[1]};
    } else {
        const auto c = __builtin_amdgcn_permlane16_swap(w[0], w[1], false, false), d = __builtin_amdgcn_permlane16_swap(w[2], w[3], false, false);
        w = u32x4{c[0], c[1], d[0], d[1]};
    }
}

PTO_DEV void MxW4ScaleSpread(u32x4 w, uint32_t (&out)[4])
{
    MxW4ScaleSpreadPart<0>(w);
    MxW4ScaleSpreadPart<1>(w);
    MxW4ScaleSpreadPart<2>(w);
    MxW4ScaleSpreadPart<3>(w);
    out[0] = w[0];
    out[1] = w[1];
    out[2] = w[2];
    out[3] = w[3];
}

// Issue slots of a K-step: slot = 4 nb + mb (nb: 16-column block, outer; mb: 16-row block of the wave's 64 rows).
template <int NNB, int NCOPY>
struct MxW4Sched {
    static constexpr int kPD = 2, kSlots = 4 * NNB, kBarrier = 4 * (NNB - kPD) - 1;
    // the eight A reads of the next step
    static constexpr int aReadSlot(int q) { return NNB >= 10 ? 4 * (q + 1) + 3 : 4 * (q / 2 + 1) + 2 + q % 2; }
    static constexpr int copySlot(int j) { return 2 + j * (kSlots - 6) / NCOPY; }
    static constexpr int aReadAt(int idx)
    {
        for (int q = 0; q < 8; ++q)
            if (aReadSlot(q) == idx)
                return q;
        return -1;
    }
    static constexpr int copyAt(int idx)
    {
        for (int j = 0; j < NCOPY; ++j)
            if (copySlot(j) == idx)
                return j;
        return -1;
    }
    static constexpr int aReadsIn(int lo, int hi) // A reads at slots in [lo, hi]
    {
        int n = 0;
        for (int q = 0; q < 8; ++q)
            if (aReadSlot(q) >= lo && aReadSlot(q) <= hi)
                ++n;
        return n;
    }
    static constexpr int copiesBefore(int idx) // copies of this step issued at slots < idx
    {
        int n = 0;
        for (int j = 0; j < NCOPY; ++j)
            if (copySlot(j) < idx)
                ++n;
        return n;
    }
    static constexpr bool distinct()
    {
        for (int q = 1; q < 8; ++q)
            if (aReadSlot(q) <= aReadSlot(q - 1))
                return false;
        for (int j = 1; j < NCOPY; ++j)
            if (copySlot(j) <= copySlot(j - 1) + 1) // the LDS address of copy j is set one slot before it
                return false;
        return true;
    }
    static_assert(aReadSlot(7) < kBarrier && copySlot(NCOPY - 1) < kSlots && copySlot(0) >= 2 && distinct(), "order of the step");
    static_assert(kBarrier + 8 < kSlots, "two scale rows are spread in the slots behind the barrier");
};

// accumulators = (A .* scales)[row0 .. + 256, :] x (B .* scales)[col0 .. + BN, :]^T over the whole K extent (k elements, four
// K-steps of 128 bytes per row at a time); block (mb, nb) of this wave's 64 rows in accumulator block (BN / 16) mb + nb.
// FMT: 0 = e4m3, 1 = e5m2, 4 = e2m1 (both operands then).
template <int FMT_A, int FMT_B, int BN>
AICORE inline __attribute__((always_inline)) void MxW4TileCompute(__gm__ const uint8_t *src0, __gm__ const uint8_t *src1,
                                                                  __gm__ const uint8_t *scale0, __gm__ const uint8_t *scale1, int k,
                                                                  int row0, int col0)
{
    constexpr int NMB = 4, NNB = BN / 16, NBUF = 4, BSTAGES = 4, NA = 8, NCB = BN / 32, NCOPY = NA + NCB;
    using S = MxW4Sched<NNB, NCOPY>;
    constexpr bool FP4 = FMT_A == 4;
    static_assert((FMT_A == 4) == (FMT_B == 4), "fp4 with fp4");
    // steps that a scale register (16 scale bytes of a row) lasts, steps that the 64 bytes loaded at once last, and block rows /
    // columns loaded in each of these
    constexpr int PD = S::kPD, kScales = NMB + NNB, kGroupSteps = FP4 ? 2 : 4, kSuperSteps = 4 * kGroupSteps;
    constexpr int kScaleLoads = (kScales + kSuperSteps - 1) / kSuperSteps;
    constexpr uint32_t kStepBytes = 128, kBBytes = kStepBytes * BN, kASlot = 64 * kStepBytes, kABase = BSTAGES * kBBytes;
    static_assert(BN % 32 == 0 && kABase + 8 * kASlot <= 160 * 1024, "tile width");
    using std::integral_constant;

    const int wave = hw::wave();
    const uint32_t lane = (uint32_t)hw::lane();
    const uint32_t ldsBase = (uint32_t)(uintptr_t)hw::lds_base();
    const int64_t ld = FP4 ? k / 2 : k; // bytes between rows of A and between columns of B
    const int kLoop = (int)(ld / 128), supers = (kLoop + kSuperSteps - 1) / kSuperSteps;
    const char *aWave = reinterpret_cast<const char *>(src0) + ((int64_t)row0 + 64 * wave) * ld;
    const char *bPanel = reinterpret_cast<const char *>(src1) + (int64_t)col0 * ld;
    auto chunkOf = [](uint32_t q) { return q; };
    const uint32_t posEven = (lane % 8) ^ (lane / 16);
    const uint32_t aCopyOff[2] = {(lane / 8) * (uint32_t)ld + chunkOf(posEven) * 16u, (lane / 8) * (uint32_t)ld + chunkOf(posEven ^ 4u) * 16u};
    const uint32_t bCopyOff = (uint32_t)(8 * wave + lane / 8) * (uint32_t)ld + chunkOf((lane % 8) ^ ((4 * wave + lane / 16) % 8)) * 16u;
    const uint32_t aLdsWave = ldsBase + kABase + (uint32_t)wave * (2 * kASlot), bLdsWave = ldsBase + (uint32_t)wave * 1024u;
    uint32_t aAddr[2][2], bAddr[2][BSTAGES];
    {
        const uint32_t r = lane % 16, pos = (lane / 16) ^ detail::mat_swz<128>(r);
        const uint32_t off = r * 128u + pos * 16u;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            aAddr[0][s] = aLdsWave + s * kASlot + off;
            aAddr[1][s] = aAddr[0][s] ^ 64u;
        }
#pragma unroll
        for (int s = 0; s < BSTAGES; ++s) {
            bAddr[0][s] = ldsBase + s * kBBytes + off;
            bAddr[1][s] = bAddr[0][s] ^ 64u;
        }
    }
    const char *aBase[NA], *bBase[NCB];
#pragma unroll
    for (int t = 0; t < NA; ++t)
        aBase[t] = detail::uniform_ptr(aWave + (int64_t)(8 * t) * ld);
#pragma unroll
    for (int t = 0; t < NCB; ++t)
        bBase[t] = detail::uniform_ptr(bPanel + (int64_t)(32 * t) * ld);
    // scales: scale row i < NMB is block row i of this wave (row 16 i + lane % 16), i >= NMB block column i - NMB of the tile;
    // k / 32 bytes between rows, 64 bytes per kSuperSteps steps of which lane group g loads bytes 16 g .. + 15 (the last 16 of
    // the row where that is past its end: scales of steps beyond K)
    const uint32_t ldScale = (uint32_t)(k / 32);
    const char *saWave = detail::uniform_ptr(reinterpret_cast<const char *>(scale0) + ((int64_t)row0 + 64 * wave) * ldScale);
    const char *sbPanel = detail::uniform_ptr(reinterpret_cast<const char *>(scale1) + (int64_t)col0 * ldScale);
    const uint32_t scaleRowOff = (lane % 16) * ldScale;
    auto scaleLoad = [&](auto iTag, int super) __attribute__((always_inline)) {
        constexpr int i = decltype(iTag)::value;
        const uint32_t chunk = (uint32_t)super * 64u + (lane / 16) * 16u;
        const uint32_t voff = scaleRowOff + (uint32_t)((i < NMB ? i : i - NMB) * 16) * ldScale + (chunk < ldScale - 16u ? chunk : ldScale - 16u);
        return MxW4Load16(i < NMB ? saWave : sbPanel, voff);
    };

    uint32_t voffA[2], voffB;
    auto setLds = [&](uint32_t waveBase, auto immTag) __attribute__((always_inline)) {
        asm volatile("s_add_u32 m0, %0, %1" ::"s"(waveBase), "n"(decltype(immTag)::value) : "memory", "scc");
    };
    auto copyAsm = [&](uint32_t voff, const char *base) __attribute__((always_inline)) {
        asm volatile("global_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(base) : "memory");
    };
    struct Pair { // the two 16-byte halves of a 32-byte operand
        f16x8 h[2];
    };
    Pair aF[2][NMB], bF[NBUF];
    uint32_t sc[kScales][4], scNext[kScales][4] = {}; // scales of the current kSuperSteps steps and of the next, a register per quarter
    u32x4 raw[kScaleLoads];
    auto readA = [&](auto setTag, auto qTag) __attribute__((always_inline)) {
        constexpr int set = decltype(setTag)::value, q = decltype(qTag)::value, mb = q / 2, kk = q % 2;
        aF[set][mb].h[kk] = W4LdsRead16<mb * 2048>(aAddr[kk][set]);
    };
    auto readB = [&](auto stageTag, auto nbTag, auto kkTag) __attribute__((always_inline)) {
        constexpr int stage = decltype(stageTag)::value, nb = decltype(nbTag)::value, kk = decltype(kkTag)::value;
        bF[nb % NBUF].h[kk] = W4LdsRead16<nb * 2048>(bAddr[kk][stage]);
    };
    auto operand = [](const Pair &p) {
        const u32x4 lo = __builtin_bit_cast(u32x4, p.h[0]), hi = __builtin_bit_cast(u32x4, p.h[1]);
        return i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
    };
    auto clampStep = [&](int s) { return s < kLoop ? s : kLoop - 1; };

    // ---- prologue: the scales of the first four steps, A and B of steps 0 and 1 ----
    __builtin_amdgcn_s_barrier(); // every wave is done with the LDS of the tile before
    u32x4 first[kScales]; // all in flight at once, picked apart behind the wait for step 0 below
    W4For<0, kScales>([&](auto iTag) __attribute__((always_inline)) { first[decltype(iTag)::value] = scaleLoad(iTag, 0); });
    W4For<0, 2>([&](auto sTag) __attribute__((always_inline)) {
        constexpr int s = decltype(sTag)::value;
        const uint32_t kOff = (uint32_t)clampStep(s) * kStepBytes;
        W4For<0, NCOPY>([&](auto jTag) __attribute__((always_inline)) {
            constexpr int j = decltype(jTag)::value;
            if constexpr (j < NA)
                setLds(aLdsWave, integral_constant<int, s * kASlot + j * 1024>());
            else
                setLds(bLdsWave, integral_constant<int, s * kBBytes + (j - NA) * 4096>());
            asm volatile("s_nop 0" ::: "memory");
            if constexpr (j < NA)
                copyAsm(aCopyOff[j % 2] + kOff, aBase[j]);
            else
                copyAsm(bCopyOff + kOff, bBase[j - NA]);
        });
    });
    hw::wait_vm<NCOPY>();
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    W4For<0, kScales>([&](auto iTag) __attribute__((always_inline)) {
        constexpr int i = decltype(iTag)::value;
        MxW4Pin(first[i]); // (older than the copies waited for above)
        MxW4ScaleSpread(first[i], sc[i]);
    });
    __builtin_amdgcn_sched_barrier(0);
    W4For<0, NA>([&](auto qTag) __attribute__((always_inline)) { readA(integral_constant<int, 0>(), qTag); });
    W4For<0, 2 * PD>([&](auto fTag) __attribute__((always_inline)) {
        constexpr int f = decltype(fTag)::value;
        readB(integral_constant<int, 0>(), integral_constant<int, f / 2>(), integral_constant<int, f % 2>());
    });

    // ---- K-step `it`, number t = it % kSuperSteps of its scale period: B stage t % 4, A register set and LDS slot t % 2, scale
    // register t / kGroupSteps, byte t % kGroupSteps (fp4: two bytes).  The copies of A of step it + 2 go to this step's A slot,
    // those of B to the stage of step it - 2; scale rows kScaleLoads t .. of the next period are loaded at the start of the step
    // and spread over the lane groups behind its barrier.
    auto step = [&](auto tTag, int it, int super) __attribute__((always_inline)) {
        constexpr int t = decltype(tTag)::value, j = t % 4, s = j, par = j % 2, sNext = (j + 1) % BSTAGES, sCopy = (j + 2) % BSTAGES;
        constexpr int quarter = t / kGroupSteps, jj = t % kGroupSteps, left = kScales - kScaleLoads * t;
        constexpr int nLoads = left < 0 ? 0 : (left < kScaleLoads ? left : kScaleLoads);
        const uint32_t kOff = (uint32_t)clampStep(it + 2) * kStepBytes;
        const int nextSuper = super + 1 < supers ? super + 1 : supers - 1;
        W4For<0, S::kSlots>([&](auto idxTag) __attribute__((always_inline)) {
            constexpr int idx = decltype(idxTag)::value, nb = idx / NMB, mb = idx % NMB;
            if constexpr (idx == 0) { // (older than every copy of this step)
                W4For<0, nLoads>([&](auto uTag) __attribute__((always_inline)) {
                    constexpr int u = decltype(uTag)::value;
                    raw[u] = scaleLoad(integral_constant<int, kScaleLoads * t + u>(), nextSuper);
                });
            }
            if constexpr (idx == 1) {
                voffA[0] = aCopyOff[0] + kOff;
                voffA[1] = aCopyOff[1] + kOff;
                voffB = bCopyOff + kOff;
            }
            if constexpr (idx == S::kBarrier) {
                // this wave's copies of the step before have landed (and this step's scale rows, which are older than its copies)
                hw::wait_vm<S::copiesBefore(S::kBarrier)>();
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (idx > S::kBarrier && idx <= S::kBarrier + 4 * nLoads) { // a part of the spreading of a loaded scale row
                constexpr int u = (idx - S::kBarrier - 1) / 4, part = (idx - S::kBarrier - 1) % 4;
                if constexpr (part == 0)
                    MxW4Pin(raw[u]); // (not before the wait above)
                MxW4ScaleSpreadPart<part>(raw[u]);
                if constexpr (part == 3) {
                    scNext[kScaleLoads * t + u][0] = raw[u][0];
                    scNext[kScaleLoads * t + u][1] = raw[u][1];
                    scNext[kScaleLoads * t + u][2] = raw[u][2];
                    scNext[kScaleLoads * t + u][3] = raw[u][3];
                }
            }
            if constexpr (mb < 2) { // half mb of the B operand of block column nb + PD
                constexpr int g = nb + PD;
                if constexpr (g < NNB)
                    readB(integral_constant<int, s>(), integral_constant<int, g>(), integral_constant<int, mb>());
                else
                    readB(integral_constant<int, sNext>(), integral_constant<int, g - NNB>(), integral_constant<int, mb>());
            }
            if constexpr (S::aReadAt(idx) >= 0) {
                if constexpr (S::aReadAt(idx) == 0) // this wave's A copies of the step before have landed
                    hw::wait_vm<NCB + nLoads + S::copiesBefore(idx)>();
                readA(integral_constant<int, par ^ 1>(), integral_constant<int, S::aReadAt(idx)>());
            }
            if constexpr (S::copyAt(idx) >= 0) {
                constexpr int c = S::copyAt(idx);
                if constexpr (c < NA)
                    copyAsm(voffA[c % 2], aBase[c]);
                else
                    copyAsm(voffB, bBase[c - NA]);
            }
            if constexpr (S::copyAt(idx + 1) >= 0) {
                constexpr int c = S::copyAt(idx + 1);
                if constexpr (c < NA)
                    setLds(aLdsWave, integral_constant<int, par * kASlot + c * 1024>());
                else
                    setLds(bLdsWave, integral_constant<int, sCopy * kBBytes + (c - NA) * 4096>());
            }
            if constexpr (mb == 0) { // both halves of block column nb have arrived; what was read after them may be under way
                constexpr int lo = 4 * (nb - PD) + 1;
                asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(2 * (PD - 1) + 1 + (lo > 0 ? S::aReadsIn(lo, idx) : 0)) : "memory");
            }
            if constexpr (FP4) {
                MxW4MfmaFp4<mb * NNB + nb, 2 * jj>(__builtin_bit_cast(u32x4, bF[nb % NBUF].h[0]), __builtin_bit_cast(u32x4, aF[par][mb].h[0]),
                                                   sc[NMB + nb][quarter], sc[mb][quarter]);
                MxW4MfmaFp4<mb * NNB + nb, 2 * jj + 1>(__builtin_bit_cast(u32x4, bF[nb % NBUF].h[1]),
                                                       __builtin_bit_cast(u32x4, aF[par][mb].h[1]), sc[NMB + nb][quarter], sc[mb][quarter]);
            } else {
                MxW4Mfma<mb * NNB + nb, jj, FMT_B, FMT_A>(operand(bF[nb % NBUF]), operand(aF[par][mb]), sc[NMB + nb][quarter],
                                                          sc[mb][quarter]);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    for (int super = 0; super < supers; ++super) {
        const int it0 = super * kSuperSteps;
        W4For<0, kSuperSteps / 4>([&](auto qTag) __attribute__((always_inline)) {
            constexpr int q = decltype(qTag)::value;
            if (it0 + 4 * q < kLoop) { // (K is whole groups of four steps, not whole scale periods)
                step(integral_constant<int, 4 * q>(), it0 + 4 * q, super);
                step(integral_constant<int, 4 * q + 1>(), it0 + 4 * q + 1, super);
                step(integral_constant<int, 4 * q + 2>(), it0 + 4 * q + 2, super);
                step(integral_constant<int, 4 * q + 3>(), it0 + 4 * q + 3, super);
            }
        });
#pragma unroll
        for (int i = 0; i < kScales; ++i)
#pragma unroll
            for (int u = 0; u < 4; ++u)
                sc[i][u] = scNext[i][u];
    }
    hw::wait_vm0(); // the copies issued past the end of K
    // the last MFMAs have written their accumulators
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
}

// this wave's accumulator blocks to C (row-major, n elements between rows; fp32, or bf16 rounded to nearest even)
template <typename OutT, int BN>
AICORE inline __attribute__((always_inline)) void MxW4StoreTile(OutT *out, int64_t n, int row0, int col0)
{
    constexpr int NNB = BN / 16;
    const uint32_t lane = (uint32_t)hw::lane();
    OutT *cWave = out + ((int64_t)row0 + 64 * hw::wave() + lane % 16) * n + col0 + 4 * (lane / 16);
    W4For<0, 4 * NNB>([&](auto idxTag) __attribute__((always_inline)) {
        constexpr int idx = decltype(idxTag)::value, mb = idx / NNB, nb = idx % NNB;
        const detail::AccFrag v = W4ReadAcc<idx>();
        OutT *dst = cWave + (int64_t)(16 * mb) * n + 16 * nb;
        if constexpr (std::is_same_v<OutT, float>) {
            *reinterpret_cast<detail::AccFrag *>(dst) = v;
        } else {
            const uint32_t lo = (uint32_t)detail::f32_to_bf16_bits_rne(v.x) | ((uint32_t)detail::f32_to_bf16_bits_rne(v.y) << 16);
            const uint32_t hi = (uint32_t)detail::f32_to_bf16_bits_rne(v.z) | ((uint32_t)detail::f32_to_bf16_bits_rne(v.w) << 16);
            typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
            *reinterpret_cast<u32x2 *>(dst) = u32x2{lo, hi};
        }
    });
}

// One 256 x BN tile of C per workgroup; the last tile row / column is moved back to end with the matrix.
template <int FMT_A, int FMT_B, typename OutT, int BN, int GROUP_M>
__global__ __launch_bounds__(kBlockThreads, 1) AICORE
    void GemmMxW4(__gm__ OutT *out, __gm__ const uint8_t *src0, __gm__ const uint8_t *src1, __gm__ const uint8_t *scale0,
                  __gm__ const uint8_t *scale1, int m, int n, int k)
{
    constexpr int TM = 256;
    const int tilesM = (m + TM - 1) / TM, tilesN = (n + BN - 1) / BN;
    int tm, tn;
    TileOfId<GROUP_M>(RegroupXcd((int)get_block_idx(), tilesM * tilesN), tilesM, tilesN, tm, tn);
    const int r = tm * TM, c = tn * BN;
    const int row0 = __builtin_amdgcn_readfirstlane(r + TM <= m ? r : m - TM);
    const int col0 = __builtin_amdgcn_readfirstlane(c + BN <= n ? c : n - BN);
    W4ZeroAcc<4 * BN / 16>();
    MxW4TileCompute<FMT_A, FMT_B, BN>(src0, src1, scale0, scale1, k, row0, col0);
    MxW4StoreTile<OutT, BN>(out, n, row0, col0);
}

} // namespace
PTO_DEVICE_CODE_END

namespace {
template <int FMT_A, int FMT_B, typename OutT, int BN>
int launch_gemm_mxw4(hipStream_t st, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *sa, const uint8_t *sb, int m, int n, int k)
{
    // (n % 4: a lane stores four consecutive elements of a row, 16 or 8 bytes, at once)
    if (m < 256 || n < BN || n % 4 || k % (FMT_A == 4 ? 1024 : 512) || k <= 0)
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = 4 * 128 * BN + 4 * 2 * 64 * 128; // four B stages + two A slots per wave
    auto kernel = GemmMxW4<FMT_A, FMT_B, OutT, BN, 4>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int tiles = ((m + 255) / 256) * ((n + BN - 1) / BN);
    kernel<<<dim3((unsigned)tiles), dim3(kBlockThreads), lds, st>>>(reinterpret_cast<OutT *>(c), a, b, sa, sb, m, n, k);
    return pto_amd::check_launch();
}
} // namespace
