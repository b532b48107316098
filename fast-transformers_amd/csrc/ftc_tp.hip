// Chain-parallel scan (ftc_tp_kernel.h): launcher.
#include "ftc_tp_kernel.h"

namespace ftc {
namespace mfma {

void launch_scan_tp(void *ws, const ScanArgs &args, hipStream_t stream) {
    // args.waves_per_scan counts chains, args.total_waves chains of all scans of the launch
    hipLaunchKernelGGL(scan_tp_kernel, dim3((unsigned)args.total_waves), dim3(512), 0, stream,
                       (uint32_t *)ws, args);
}

}  // namespace mfma
}  // namespace ftc
