// Chain-parallel scan on the fp16 matrix path (ftc_tph_kernel.h): launcher.
#include "ftc_tph_kernel.h"

namespace ftc {
namespace mfma {

void launch_scan_tph(void *ws, const ScanArgs &args, bool mixed, hipStream_t stream) {
    // (grid as for launch_scan_tp)
    const dim3 grid((unsigned)args.total_waves), block(768);
    if (mixed) {
        if (args.tp_d <= 32)
            hipLaunchKernelGGL((scan_tph_kernel<1, true>), grid, block, 0, stream, (uint32_t *)ws, args);
        else
            hipLaunchKernelGGL((scan_tph_kernel<2, true>), grid, block, 0, stream, (uint32_t *)ws, args);
    } else if (args.tp_d <= 32) {
        hipLaunchKernelGGL((scan_tph_kernel<1, false>), grid, block, 0, stream, (uint32_t *)ws, args);
    } else {
        hipLaunchKernelGGL((scan_tph_kernel<2, false>), grid, block, 0, stream, (uint32_t *)ws, args);
    }
}

}  // namespace mfma
}  // namespace ftc
