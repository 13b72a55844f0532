// placeholder until the MFMA kernels land
#include "hstu_device.h"
namespace hstu {
bool mfma_supported(const KArgs&, const char** name) { *name = nullptr; return false; }
hipError_t launch_mfma(const KArgs&, hipStream_t) { return hipErrorNotSupported; }
}
