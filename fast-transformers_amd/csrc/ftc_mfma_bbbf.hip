// MFMA scan kernels for one combination of element types (a, b, v, out) =
// (bf16, bf16, bf16, fp32); see ftc_mfma_kernel.h.
#include "ftc_mfma_kernel.h"

namespace ftc {
namespace mfma {
void launch_scan_bbbf(int D, int F, void *ws, const ScanArgs &args, hipStream_t stream) {
    launch_scan<bf16_t, bf16_t, bf16_t, float>(D, F, ws, args, stream);
}
}  // namespace mfma
}  // namespace ftc
