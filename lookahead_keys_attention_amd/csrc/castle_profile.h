// Per-kernel HIP-event timing hooks (see castle_profile.hip).
#pragma once
#include <hip/hip_runtime.h>

namespace castle {

// kernel slots reported by castle_profile_read
enum ProfSlot {
  kSlotPrep = 0, kSlotScan = 1, kSlotAttn = 2,
  kSlotDelta = 3, kSlotBwdKey = 4, kSlotBwdQuery = 5,
  kSlotDecodeStream = 6, kSlotDecodeFinish = 7,
};

// Records an event pair around the enclosed launch when profiling is enabled.
class ProfScope {
 public:
  ProfScope(int slot, hipStream_t stream);
  ~ProfScope();
  ProfScope(const ProfScope&) = delete;
  ProfScope& operator=(const ProfScope&) = delete;

 private:
  hipStream_t stream_;
  int index_;
};

int profile_enable(int on);
int profile_read(int* slots, float* ms, int max_records);

}  // namespace castle
