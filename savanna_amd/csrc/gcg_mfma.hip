// placeholder until the MFMA kernels land
#include "gcg_common.h"
namespace gcg {
bool mfma_supported(int, const Dims &) { return false; }
int mfma_fwd_launch(int, const void *, const void *, const void *, const void *, void *, void *, void *, const Dims &, hipStream_t) { return (int)hipErrorNotSupported; }
size_t mfma_bwd_workspace(const Dims &) { return 0; }
int mfma_bwd_launch(int, const void *, const void *, const void *, const void *, const void *, void *, void *, void *, void *, void *, const Dims &, hipStream_t) { return (int)hipErrorNotSupported; }
}
