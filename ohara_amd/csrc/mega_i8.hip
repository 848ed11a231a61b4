// The polled builds of the persistent decode kernel over an int8 KV cache (ohara/modules/kv_cache.py:15-32, 94-118),
// compiled apart from the bf16 builds so that the two sets build in parallel.
#include "mega_kernel.h"

namespace ohara_mega {

int mega_launch_i8(const MegaArgs& a, int D, int G, int mode, size_t smem, int n_workgroups, hipStream_t st) {
  if (mode != 1 && mode != 2) return OHARA_ESIZE;
  if (a.prof && D == 128 && G == 1) {  // the builds with the phase stamps
    static ResidencySlot p1, p2;
    return mode == 1 ? mega_launch(decode_mega_kernel<128, 1, 1, true, true>, p1, a, smem, n_workgroups, st)
                     : mega_launch(decode_mega_kernel<128, 1, 2, true, true>, p2, a, smem, n_workgroups, st);
  }
#define OHARA_MEGA_I8(DD, GG)                                                                            \
  do {                                                                                                   \
    static ResidencySlot s1, s2;                                                                         \
    return mode == 1 ? mega_launch(decode_mega_kernel<DD, GG, 1, true>, s1, a, smem, n_workgroups, st)   \
                     : mega_launch(decode_mega_kernel<DD, GG, 2, true>, s2, a, smem, n_workgroups, st);  \
  } while (0)
  if (D == 128 && G == 1) OHARA_MEGA_I8(128, 1);
  if (D == 128 && G == 2) OHARA_MEGA_I8(128, 2);
  if (D == 128 && G == 4) OHARA_MEGA_I8(128, 4);
  if (D == 64 && G == 1) OHARA_MEGA_I8(64, 1);
  if (D == 64 && G == 2) OHARA_MEGA_I8(64, 2);
  if (D == 64 && G == 4) OHARA_MEGA_I8(64, 4);
#undef OHARA_MEGA_I8
  return OHARA_ESIZE;
}

}  // namespace ohara_mega
