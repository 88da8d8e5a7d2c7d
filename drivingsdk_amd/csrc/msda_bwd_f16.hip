// The backward's first kernel for f16_t (see msda_bwd_kernel.h; one translation unit per dtype).
#include "msda_bwd_kernel.h"

namespace mxd {

hipError_t launch_backward_f16(const KArgs& a, bool scatter, hipStream_t stream) { return launch_dtype<f16_t>(a, scatter, stream); }

}  // namespace mxd
