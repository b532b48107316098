// MFMA scan kernels for one combination of element types (a, b, v, out) =
// (fp32, bf16, bf16, bf16); see ftc_mfma_kernel.h.
#include "ftc_mfma_kernel.h"

namespace ftc {
namespace mfma {
void launch_scan_fbbb(int D, int F, void *ws, const ScanArgs &args, hipStream_t stream) {
    launch_scan<float, bf16_t, bf16_t, bf16_t>(D, F, ws, args, stream);
}
}  // namespace mfma
}  // namespace ftc
