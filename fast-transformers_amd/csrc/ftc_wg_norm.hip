// Workgroup scan, fused attention form (feature map, key-length mask and normaliser inside
// the scan): instantiations and launcher.
#include "ftc_wg_kernel.h"

namespace ftc {
namespace mfma {

bool scan_wg_norm_covers(int D, int F) { return (D == 32 || D == 64) && (F == 32 || F == 64); }

void launch_scan_wg_norm(int D, int F, const dim3 grid, void *workspace, const ScanArgs &args,
                         hipStream_t stream) {
#define FTC_LAUNCH(DD, FF)                                                             \
    hipLaunchKernelGGL((scan_wg_kernel<DD, FF, true>), grid, dim3(512), 0, stream,     \
                       (uint32_t *)workspace, args)
    if (D == 64 && F == 64) FTC_LAUNCH(64, 64);
    else if (D == 64 && F == 32) FTC_LAUNCH(64, 32);
    else if (D == 32 && F == 64) FTC_LAUNCH(32, 64);
    else FTC_LAUNCH(32, 32);
#undef FTC_LAUNCH
}

}  // namespace mfma
}  // namespace ftc
