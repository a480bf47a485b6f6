// fp16 x fp16 -> fp32 GEMM tile of 256 x BN or 192 x BN (BN = 256, 192 or 128) on four wavefronts, wave grid 4 x 1, one wave
// per SIMD, NMB = 4 or 3 row blocks of 16 = 64 or 48 rows x BN of C per wave; K-steps of 64 on v_mfma_f32_16x16x32_f16.
// (What follows is written for NMB = 4; with three row blocks a wave copies 48 rows in six instructions and a slot is
// 3 f + mb.)
//
// A wave's 64 rows of A are used by no other wave: each wave copies them into a ring of its own in the LDS (two slots of
// 8 KiB) and reads its fragments back from there, so A needs no workgroup barrier, only the wave's own counters.  B
// (BN / 8 KiB per step) goes through a ring of three stages shared by the four waves.  Every copy is a 1 KiB asynchronous
// global -> LDS instruction of eight whole 128-byte lines (a lane's eight halves of an A fragment cannot be loaded
// straight from memory at speed: the sixteen rows of a fragment are sixteen different lines for four consecutive lanes).
//
// A K-step is 8 BN / 16 MFMAs (B fragment f = (BN / 16) kk + nb outer, the four row blocks mb inner), written slot by slot,
// slot = 4 f + mb:
//   slot 4 f:     B fragment f + 4 is read (a rolling set of eight fragment registers), then the wait for fragment f;
//   slot 4 g + 1: for eight values of g, one A fragment of the next step is read into the other of two register sets;
//   slot 4 g + 2, 4 g + 3: for 8 + BN / 32 values of g, the LDS address of a copy (M0), then the copy: A of two steps
//                 ahead (eight copies), then B of two steps ahead;
//   barrier 1 (before the first read of the next step's stage): B of the next step has landed for every wave;
//   barrier 2 (behind the wait for the last B fragment): this step's stage is dead for every wave and may be overwritten.
// No slot holds more than three instructions besides its MFMA: with one wave per SIMD every further one delays the MFMA
// behind it.
// The MFMA takes the B fragment as its first operand and the A fragment as its second: a 16 x 16 accumulator block holds
// C transposed, lane l owns row l % 16 and the four consecutive columns 4 (l / 16) .. + 3, one 16-byte store per block.
#pragma once
#include "gemm_kernels.hpp"

PTO_DEVICE_CODE_BEGIN
namespace {

template <int FIRST, int LAST, typename F>
__device__ __attribute__((always_inline)) inline void W4For(F &&f)
{
    if constexpr (FIRST < LAST) {
        f(std::integral_constant<int, FIRST>());
        W4For<FIRST + 1, LAST>(f);
    }
}

// 16 bytes per lane from the LDS as assembly: the reads stay in flight under waits that the kernel places itself.  The
// result may be used only behind such a wait.
template <int IMM>
PTO_DEV f16x8 W4LdsRead16(uint32_t addr)
{
    f16x8 r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(IMM));
    return r;
}

// Accumulator block b of a wave (16 x 16 of C, four values per lane) lives in the accumulation registers a[4 b : 4 b + 3]
// and only there: the instructions that touch it name the registers themselves, and the compiler is told only that they
// are overwritten.  As operands of the compiler's own allocation a block gets different registers in different parts of
// a kernel of this size, with moves between them at the head of the K loop, behind MFMAs whose wait states the compiler
// does not know.  The kernel uses fewer than 256 ordinary registers, so the compiler has no use of its own for
// accumulation registers (checked in the build: no v_accvgpr instruction outside these helpers).
#define PTO_W4_ACC_BLOCKS(X) \
    X(0, 0, 1, 2, 3) X(1, 4, 5, 6, 7) X(2, 8, 9, 10, 11) X(3, 12, 13, 14, 15) \
    X(4, 16, 17, 18, 19) X(5, 20, 21, 22, 23) X(6, 24, 25, 26, 27) X(7, 28, 29, 30, 31) \
    X(8, 32, 33, 34, 35) X(9, 36, 37, 38, 39) X(10, 40, 41, 42, 43) X(11, 44, 45, 46, 47) \
    X(12, 48, 49, 50, 51) X(13, 52, 53, 54, 55) X(14, 56, 57, 58, 59) X(15, 60, 61, 62, 63) \
    X(16, 64, 65, 66, 67) X(17, 68, 69, 70, 71) X(18, 72, 73, 74, 75) X(19, 76, 77, 78, 79) \
    X(20, 80, 81, 82, 83) X(21, 84, 85, 86, 87) X(22, 88, 89, 90, 91) X(23, 92, 93, 94, 95) \
    X(24, 96, 97, 98, 99) X(25, 100, 101, 102, 103) X(26, 104, 105, 106, 107) X(27, 108, 109, 110, 111) \
    X(28, 112, 113, 114, 115) X(29, 116, 117, 118, 119) X(30, 120, 121, 122, 123) X(31, 124, 125, 126, 127) \
    X(32, 128, 129, 130, 131) X(33, 132, 133, 134, 135) X(34, 136, 137, 138, 139) X(35, 140, 141, 142, 143) \
    X(36, 144, 145, 146, 147) X(37, 148, 149, 150, 151) X(38, 152, 153, 154, 155) X(39, 156, 157, 158, 159) \
    X(40, 160, 161, 162, 163) X(41, 164, 165, 166, 167) X(42, 168, 169, 170, 171) X(43, 172, 173, 174, 175) \
    X(44, 176, 177, 178, 179) X(45, 180, 181, 182, 183) X(46, 184, 185, 186, 187) X(47, 188, 189, 190, 191) \
    X(48, 192, 193, 194, 195) X(49, 196, 197, 198, 199) X(50, 200, 201, 202, 203) X(51, 204, 205, 206, 207) \
    X(52, 208, 209, 210, 211) X(53, 212, 213, 214, 215) X(54, 216, 217, 218, 219) X(55, 220, 221, 222, 223) \
    X(56, 224, 225, 226, 227) X(57, 228, 229, 230, 231) X(58, 232, 233, 234, 235) X(59, 236, 237, 238, 239) \
    X(60, 240, 241, 242, 243) X(61, 244, 245, 246, 247) X(62, 248, 249, 250, 251) X(63, 252, 253, 254, 255)
template <int BLK>
PTO_DEV void W4Mfma(f16x8 first, f16x8 second)
{
#define X(b, r0, r1, r2, r3)  \
    if constexpr (BLK == b) \
        asm volatile("v_mfma_f32_16x16x32_f16 a[" #r0 ":" #r3 "], %0, %1, a[" #r0 ":" #r3 "]" ::"v"(first), "v"(second) : "a" #r0, "a" #r1, "a" #r2, "a" #r3);
    PTO_W4_ACC_BLOCKS(X)
#undef X
}
template <int BLOCKS>
PTO_DEV void W4ZeroAcc()
{
#define X(b, r0, r1, r2, r3)                                                                                                             \
    if constexpr (b < BLOCKS)                                                                                                            \
        asm volatile("v_accvgpr_write_b32 a" #r0 ", 0\n\tv_accvgpr_write_b32 a" #r1 ", 0\n\tv_accvgpr_write_b32 a" #r2 ", 0\n\tv_accvgpr_write_b32 a" #r3 ", 0" :: \
                     : "a" #r0, "a" #r1, "a" #r2, "a" #r3);
    PTO_W4_ACC_BLOCKS(X)
#undef X
}
// (only behind the wait states that follow the last MFMA)
template <int BLK>
PTO_DEV detail::AccFrag W4ReadAcc()
{
    detail::AccFrag v;
#define X(b, r0, r1, r2, r3)  \
    if constexpr (BLK == b) \
        asm volatile("v_accvgpr_read_b32 %0, a" #r0 "\n\tv_accvgpr_read_b32 %1, a" #r1 "\n\tv_accvgpr_read_b32 %2, a" #r2 "\n\tv_accvgpr_read_b32 %3, a" #r3 : "=v"(v.x), "=v"(v.y), "=v"(v.z), "=v"(v.w));
    PTO_W4_ACC_BLOCKS(X)
#undef X
    return v;
}

// Issue slots of a K-step for NFRAG B fragments and NMB row blocks per wave (see the head of the file; slot = NMB f + mb).
template <int NFRAG, int NCOPY, int NMB>
struct W4Sched {
    static constexpr int kPD = 4, kSlots = NMB * NFRAG, kAReads = 2 * NMB;
    static constexpr int kBarrier1 = NMB * (NFRAG - kPD) - 1, kBarrier2 = NMB * (NFRAG - 1) + 1;
    static constexpr int aReadSlot(int q) { return NMB * (NFRAG / 4 + q * (NFRAG / 2) / kAReads) + 1; }
    static constexpr int copySlot(int j) { return NMB * (j * NFRAG / NCOPY) + NMB - 1; }
    static constexpr int aReadAt(int idx) // the A read issued at slot idx, or -1
    {
        for (int q = 0; q < kAReads; ++q)
            if (aReadSlot(q) == idx)
                return q;
        return -1;
    }
    static constexpr int copyAt(int idx) // the copy issued at slot idx, or -1
    {
        for (int j = 0; j < NCOPY; ++j)
            if (copySlot(j) == idx)
                return j;
        return -1;
    }
    static constexpr int aReadsIn(int lo, int hi) // A reads at slots in (lo, hi)
    {
        int n = 0;
        for (int q = 0; q < kAReads; ++q)
            if (aReadSlot(q) > lo && aReadSlot(q) < hi)
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
    static constexpr bool distinct() // no two A reads and no two copies in one slot
    {
        for (int q = 1; q < kAReads; ++q)
            if (aReadSlot(q) == aReadSlot(q - 1))
                return false;
        for (int j = 1; j < NCOPY; ++j)
            if (copySlot(j) == copySlot(j - 1))
                return false;
        return true;
    }
    static_assert(NFRAG >= NCOPY && aReadSlot(kAReads - 1) < kBarrier1 && copySlot(NCOPY - 1) < kSlots && distinct(), "order of the step");
};

constexpr int kW4Group = 6; // K-steps of 64 come in groups of six (three B stages x two A slots)

// accumulators += A[row0 .. + 256, 64 kFirst .. 64 (kFirst + kLoop)) x B[col0 .. + BN, the same k]^T, block (mb, nb) of this
// wave's 64 rows in accumulator block (BN / 16) mb + nb.  TAIL == 0: kLoop is a positive multiple of kW4Group, a loop of
// groups of six steps; TAIL > 0: exactly kLoop == TAIL steps in straight-line code (the steps that a K extent leaves over
// after its whole groups: conditions around single steps of the loop would make the compiler join register
// assignments of fragments that are still on their way from the LDS).
template <int BN, int TAIL, int NMB>
AICORE inline __attribute__((always_inline)) void W4Pass(__gm__ const half *src0, __gm__ const half *src1, int k, int row0, int col0, int kFirst,
                                                         int kLoop)
{
    constexpr int BK = 64, NNB = BN / 16, NBUF = 8, BSTAGES = 3, NA = 2 * NMB; // NA: A copies (of eight rows) and A fragments per step
    constexpr int NFRAG = 2 * NNB, NM = NFRAG * NMB, NCB = BN / 32, NCOPY = NA + NCB;
    using S = W4Sched<NFRAG, NCOPY, NMB>;
    constexpr int PD = S::kPD;
    constexpr uint32_t kBBytes = BK * BN * sizeof(half), kASlot = 16 * NMB * BK * sizeof(half), kABase = BSTAGES * kBBytes;
    static_assert((NMB == 3 || NMB == 4) && BN % 32 == 0 && BN <= 256 && kABase + 8 * kASlot <= 160 * 1024, "tile shape");

    const int wave = hw::wave();
    const uint32_t lane = (uint32_t)hw::lane();
    const uint32_t ldsBase = (uint32_t)(uintptr_t)hw::lds_base();
    const int64_t ld = (int64_t)k * 2; // bytes between rows of A and between columns of B
    // A: this wave's 64 rows.  Copy t takes rows 8 t .. 8 t + 7: lane l copies the 16-byte chunk (l % 8) ^ swz(row) of row
    // 8 t + l / 8 to position l % 8 of that row's LDS image (swz(r) = (r / 2) % 8 as in a Mat tile: 4 t + l / 16).
    const char *aWave = reinterpret_cast<const char *>(src0 + ((int64_t)row0 + 16 * NMB * wave) * k + (int64_t)kFirst * BK);
    const char *bPanel = reinterpret_cast<const char *>(src1 + (int64_t)col0 * k + (int64_t)kFirst * BK);
    const uint32_t chunkEven = (lane % 8) ^ (lane / 16);
    const uint32_t aCopyOff[2] = {(lane / 8) * (uint32_t)ld + chunkEven * 16u, (lane / 8) * (uint32_t)ld + (chunkEven ^ 4u) * 16u};
    // B: copy j of wave w takes columns 32 j + 8 w .. + 7 of the stage, the image of a Mat tile of BN columns of 64 k
    const uint32_t bCopyOff = (uint32_t)(8 * wave + lane / 8) * (uint32_t)ld + (((lane % 8) ^ ((4 * wave + lane / 16) % 8)) * 16u);
    const uint32_t aLdsWave = ldsBase + kABase + (uint32_t)wave * (2 * kASlot), bLdsWave = ldsBase + (uint32_t)wave * 1024u;
    // fragment reads: lane l holds row l % 16 of a 16-row block and the k group l / 16
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
    // a copy in two halves: the LDS address (M0), and one slot later the copy itself; bases per copy in scalar registers,
    // the K offset of the step in the lane offsets
    const char *aBase[NA], *bBase[NCB];
#pragma unroll
    for (int t = 0; t < NA; ++t)
        aBase[t] = detail::uniform_ptr(aWave + (int64_t)(8 * t) * ld);
#pragma unroll
    for (int t = 0; t < NCB; ++t)
        bBase[t] = detail::uniform_ptr(bPanel + (int64_t)(32 * t) * ld);
    uint32_t voffA[2], voffB;
    auto setLds = [&](uint32_t waveBase, auto immTag) __attribute__((always_inline)) {
        asm volatile("s_add_u32 m0, %0, %1" ::"s"(waveBase), "n"(decltype(immTag)::value) : "memory", "scc");
    };
    auto copyAsm = [&](uint32_t voff, const char *base) __attribute__((always_inline)) {
        asm volatile("global_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(base) : "memory");
    };
    f16x8 aF[2][NMB][2], bF[NBUF];
    auto readA = [&](auto setTag, auto qTag) __attribute__((always_inline)) { // A register set p comes from LDS slot p
        constexpr int set = decltype(setTag)::value, q = decltype(qTag)::value, mb = q / 2, kk = q % 2;
        aF[set][mb][kk] = W4LdsRead16<mb * 2048>(aAddr[kk][set]);
    };
    auto readB = [&](auto bufTag, auto stageTag, auto fragTag) __attribute__((always_inline)) {
        constexpr int buf = decltype(bufTag)::value, stage = decltype(stageTag)::value, f = decltype(fragTag)::value;
        bF[buf] = W4LdsRead16<(f % NNB) * 2048>(bAddr[f / NNB][stage]);
    };
    auto clampStep = [&](int s) { return s < kLoop ? s : kLoop - 1; };
    using std::integral_constant;

    // Every wave is done with the LDS of the tile before.  Then A and B of steps 0 and 1 in flight (copies with wait
    // states between M0 and its use); when step 0 has landed, its A fragments and its first PD B fragments.
    __builtin_amdgcn_s_barrier();
    W4For<0, 2>([&](auto sTag) __attribute__((always_inline)) {
        constexpr int s = decltype(sTag)::value;
        const uint32_t kOff = (uint32_t)clampStep(s) * (BK * 2);
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
    W4For<0, NA>([&](auto qTag) __attribute__((always_inline)) { readA(integral_constant<int, 0>(), qTag); });
    W4For<0, PD>([&](auto fTag) __attribute__((always_inline)) {
        readB(integral_constant<int, decltype(fTag)::value % NBUF>(), integral_constant<int, 0>(), fTag);
    });

    // K-step `it`: B stage it % 3, A register set and LDS slot it % 2: the A fragments of step it + 1 come from the other
    // slot into the other set, the copies of A of step it + 2 go to this step's slot (read during the step before), those
    // of B of step it + 2 to the stage of step it - 1.
    auto step = [&](auto stageTag, auto parTag, int it) __attribute__((always_inline)) {
        constexpr int s = decltype(stageTag)::value, par = decltype(parTag)::value;
        constexpr int sNext = (s + 1) % BSTAGES, sCopy = (s + 2) % BSTAGES;
        const uint32_t kOff = (uint32_t)clampStep(it + 2) * (BK * 2);
        W4For<0, NM>([&](auto idxTag) __attribute__((always_inline)) {
            constexpr int idx = decltype(idxTag)::value, f = idx / NMB, mb = idx % NMB, kk = f / NNB, nb = f % NNB;
            if constexpr (idx == 1) {
                voffA[0] = aCopyOff[0] + kOff;
                voffA[1] = aCopyOff[1] + kOff;
                voffB = bCopyOff + kOff;
            }
            if constexpr (idx == S::kBarrier1) {
                hw::wait_vm<S::copiesBefore(S::kBarrier1)>(); // this wave's copies of the step before have landed
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (mb == 0) {
                constexpr int g = f + PD;
                if constexpr (g < NFRAG)
                    readB(integral_constant<int, g % NBUF>(), stageTag, integral_constant<int, g>());
                else
                    readB(integral_constant<int, g % NBUF>(), integral_constant<int, sNext>(), integral_constant<int, g - NFRAG>());
            }
            if constexpr (S::aReadAt(idx) >= 0) {
                if constexpr (S::aReadAt(idx) == 0)
                    hw::wait_vm<NCB + S::copiesBefore(idx)>(); // this wave's A copies of the step before have landed
                readA(integral_constant<int, par ^ 1>(), integral_constant<int, S::aReadAt(idx)>());
            }
            if constexpr (S::copyAt(idx + 1) >= 0) {
                constexpr int j = S::copyAt(idx + 1);
                if constexpr (j < NA)
                    setLds(aLdsWave, integral_constant<int, par * kASlot + j * 1024>());
                else
                    setLds(bLdsWave, integral_constant<int, sCopy * kBBytes + (j - NA) * 4096>());
            }
            if constexpr (S::copyAt(idx) >= 0) {
                constexpr int j = S::copyAt(idx);
                if constexpr (j < NA)
                    copyAsm(voffA[j % 2], aBase[j]);
                else
                    copyAsm(voffB, bBase[j - NA]);
            }
            if constexpr (mb == 0) // B fragment f has arrived; the reads issued after it may be under way
                asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(PD + S::aReadsIn(NMB * (f - PD), NMB * f)) : "memory");
            if constexpr (idx == S::kBarrier2) {
                __builtin_amdgcn_s_barrier(); // every wave has the last B fragment of this step: the stage is dead
                __builtin_amdgcn_sched_barrier(0);
            }
            W4Mfma<mb * NNB + nb>(bF[f % NBUF], aF[par][mb][kk]);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    if constexpr (TAIL == 0) {
        for (int it = 0; it < kLoop; it += 6) { // B stages x A slots repeat every six steps
            step(integral_constant<int, 0>(), integral_constant<int, 0>(), it);
            step(integral_constant<int, 1>(), integral_constant<int, 1>(), it + 1);
            step(integral_constant<int, 2>(), integral_constant<int, 0>(), it + 2);
            step(integral_constant<int, 0>(), integral_constant<int, 1>(), it + 3);
            step(integral_constant<int, 1>(), integral_constant<int, 0>(), it + 4);
            step(integral_constant<int, 2>(), integral_constant<int, 1>(), it + 5);
        }
    } else {
        W4For<0, TAIL>([&](auto itTag) __attribute__((always_inline)) {
            constexpr int it = decltype(itTag)::value;
            step(integral_constant<int, it % 3>(), integral_constant<int, it % 2>(), it);
        });
    }
    hw::wait_vm0(); // the copies issued past the end of K
    // the last MFMAs have written their accumulators
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
}

// accumulators = A[row0 .. + 64 NMB, :] x B[col0 .. + BN, :]^T over the whole K extent (k % 128 == 0, k >= 128)
template <int BN, int NMB>
AICORE inline __attribute__((always_inline)) void W4TileCompute(__gm__ const half *src0, __gm__ const half *src1, int k, int row0, int col0)
{
    const int steps = k / 64, whole = steps / kW4Group * kW4Group, left = steps - whole;
    W4ZeroAcc<NMB * BN / 16>();
    if (whole > 0)
        W4Pass<BN, 0, NMB>(src0, src1, k, row0, col0, 0, whole);
    if (left == 2)
        W4Pass<BN, 2, NMB>(src0, src1, k, row0, col0, whole, 2);
    else if (left == 4)
        W4Pass<BN, 4, NMB>(src0, src1, k, row0, col0, whole, 4);
}

// this wave's accumulator blocks to C (row-major, n floats between rows)
template <int BN, int NMB>
AICORE inline __attribute__((always_inline)) void W4StoreTile(float *out, int64_t n, int row0, int col0)
{
    constexpr int NNB = BN / 16;
    const uint32_t lane = (uint32_t)hw::lane();
    float *cWave = out + ((int64_t)row0 + 16 * NMB * hw::wave() + lane % 16) * n + col0 + 4 * (lane / 16);
    W4For<0, NMB * NNB>([&](auto idxTag) __attribute__((always_inline)) {
        constexpr int idx = decltype(idxTag)::value, mb = idx / NNB, nb = idx % NNB;
        *reinterpret_cast<detail::AccFrag *>(cWave + (int64_t)(16 * mb) * n + 16 * nb) = W4ReadAcc<idx>();
    });
}

// One 64 NMB x BN tile of C per workgroup.  Where the tile height does not divide m (BN does not divide n) the last tile
// row (column) is moved back so that it ends with the matrix: it computes some rows (columns) of its neighbour a second
// time and stores the same values.
template <int BN, int GROUP_M, int NMB>
__global__ __launch_bounds__(kBlockThreads, 1) AICORE
    void GemmF16F32W4(__gm__ float *out, __gm__ const half *src0, __gm__ const half *src1, int m, int n, int k)
{
    constexpr int TM = 64 * NMB;
    const int tilesM = (m + TM - 1) / TM, tilesN = (n + BN - 1) / BN;
    int tm, tn;
    TileOfId<GROUP_M>(RegroupXcd((int)get_block_idx(), tilesM * tilesN), tilesM, tilesN, tm, tn);
    const int r = tm * TM, c = tn * BN;
    const int row0 = __builtin_amdgcn_readfirstlane(r + TM <= m ? r : m - TM);
    const int col0 = __builtin_amdgcn_readfirstlane(c + BN <= n ? c : n - BN);
    W4TileCompute<BN, NMB>(src0, src1, k, row0, col0);
    W4StoreTile<BN, NMB>(out, n, row0, col0);
}

} // namespace
PTO_DEVICE_CODE_END

namespace {
// NMB row blocks of 16 per wave: tiles of 256 (NMB = 4) or 192 (NMB = 3) rows
template <int BN, int NMB = 4>
int launch_gemm_w4(hipStream_t st, float *c, const half *a, const half *b, int m, int n, int k)
{
    constexpr int TM = 64 * NMB;
    // (n % 4: the accumulator blocks are stored 16 bytes at a time)
    if (m < TM || n < BN || n % 4 || k % 128 || k < 128)
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = 3 * 64 * BN * (int)sizeof(half) + 4 * 2 * (16 * NMB) * 64 * (int)sizeof(half); // three B stages + two A slots per wave
    auto kernel = GemmF16F32W4<BN, 4, NMB>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int tiles = ((m + TM - 1) / TM) * ((n + BN - 1) / BN);
    kernel<<<dim3((unsigned)tiles), dim3(kBlockThreads), lds, st>>>(c, a, b, m, n, k);
    return pto_amd::check_launch();
}
} // namespace
