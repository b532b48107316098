// Workgroup scan, all-fp32 rows: instantiations and launcher.
#include "ftc_wg_kernel.h"

namespace ftc {
namespace mfma {

bool scan_wg_covers(int D, int F) {
    return (D == 64 && (F == 64 || F == 128)) || (D == 32 && (F == 32 || F == 64 || F == 128));
}

void launch_scan_wg_norm(int D, int F, const dim3 grid, void *workspace, const ScanArgs &args,
                         hipStream_t stream);

void launch_scan_wg_ffff(int D, int F, bool norm, void *workspace, const ScanArgs &args,
                         hipStream_t stream) {
    // args.waves_per_scan / args.total_waves count units; a workgroup carries several
    const unsigned ns = (unsigned)scan_wg_units_per_block(F, norm);
    const unsigned nscans = (unsigned)(args.total_waves / args.waves_per_scan);
    const unsigned blocks_per_scan = ((unsigned)args.waves_per_scan + ns - 1) / ns;
    const dim3 grid(nscans * blocks_per_scan), block(512);
    if (norm) return launch_scan_wg_norm(D, F, grid, workspace, args, stream);
#define FTC_LAUNCH(DD, FF)                                                           \
    hipLaunchKernelGGL((scan_wg_kernel<DD, FF, false>), grid, block, 0, stream,      \
                       (uint32_t *)workspace, args)
    if (D == 64 && F == 64) FTC_LAUNCH(64, 64);
    else if (D == 64 && F == 128) FTC_LAUNCH(64, 128);
    else if (D == 32 && F == 32) FTC_LAUNCH(32, 32);
    else if (D == 32 && F == 64) FTC_LAUNCH(32, 64);
    else FTC_LAUNCH(32, 128);
#undef FTC_LAUNCH
}

}  // namespace mfma
}  // namespace ftc
