// The Cube / Vec communication-slot handshake of the reference (include/pto/npu/a2a3/custom/TSyncCVID.hpp:33-75): with
// more blocks than physical core groups a Cube core and its Vec cores agree on a slot of the FIFO workspace at run time.
// Here the two roles are one workgroup: the slot is the block index.
#pragma once
#include <pto/pto-inst.hpp>

namespace pto {
constexpr int kCvMaxCores = 25;
constexpr int kCvCommSlotBytes = 512;
enum CVSyncMode : uint16_t { CUBE_ALL_SYNC = 0, VEC_SUB_SYNC = 1, CV_CORE_SYNC = 2 };
constexpr uint16_t CV_COMM_CTRL = 6;

PTO_DEV uint16_t _getFFTSMsg(CVSyncMode mode, uint16_t flag_id, uint16_t base_const = 0x1)
{
    return (uint16_t)((base_const & 0xf) + ((mode & 0x3) << 4) + ((flag_id & 0xf) << 8));
}

template <int CV_COMM_SLOT_BYTES = kCvCommSlotBytes, int CV_MAX_CORES = kCvMaxCores>
PTO_DEV int TSYNC_CVID(int blockId, uint8_t *cv_comm_buf)
{
    (void)cv_comm_buf;
    return blockId;
}
} // namespace pto
