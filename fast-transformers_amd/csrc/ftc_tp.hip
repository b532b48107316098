// Chain-parallel scan (ftc_tp_kernel.h): launcher.
#include "ftc_tp_kernel.h"

namespace ftc {
namespace mfma {

void launch_scan_tp(void *ws, const ScanArgs &args, hipStream_t stream) {
    // args.waves_per_scan counts the workgroups of one block of 64 output columns of one scan,
    // args.total_waves those of all blocks of all scans of the launch
    const dim3 grid((unsigned)args.total_waves), block(512);
    if (args.tp_d <= 32)
        hipLaunchKernelGGL((scan_tp_kernel<1, 1>), grid, block, 0, stream, (uint32_t *)ws, args);
    else if (args.tp_d <= 64)
        hipLaunchKernelGGL((scan_tp_kernel<1, 2>), grid, block, 0, stream, (uint32_t *)ws, args);
    else if (args.tp_d <= 96)
        hipLaunchKernelGGL((scan_tp_kernel<2, 1>), grid, block, 0, stream, (uint32_t *)ws, args);
    else
        hipLaunchKernelGGL((scan_tp_kernel<2, 2>), grid, block, 0, stream, (uint32_t *)ws, args);
}

}  // namespace mfma
}  // namespace ftc
