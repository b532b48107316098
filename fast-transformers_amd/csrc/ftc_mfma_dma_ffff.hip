// Instantiations of the LDS-fed MFMA scan kernel for (a, b, v, out) = (fp32, fp32, fp32, fp32);
// see ftc_mfma_dma_kernel.h.
#include "ftc_mfma_dma_kernel.h"

namespace ftc {
namespace mfma {
#define FTC_INSTANTIATE(DD, FF) \
    template __global__ void scan_dma_kernel<DD, FF, float, float, float, float>(uint32_t *, ScanArgs)
FTC_INSTANTIATE(64, 64);
FTC_INSTANTIATE(32, 128);
FTC_INSTANTIATE(32, 32);
FTC_INSTANTIATE(32, 64);
FTC_INSTANTIATE(64, 32);
#undef FTC_INSTANTIATE

void launch_scan_dma_ffff(int D, int F, void *ws, const ScanArgs &args, hipStream_t stream) {
    launch_scan_dma<float, float, float, float>(D, F, ws, args, stream);
}
}  // namespace mfma
}  // namespace ftc
