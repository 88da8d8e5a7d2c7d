// The backward's first kernel for float (see msda_bwd_kernel.h; one translation unit per dtype).
#include "msda_bwd_kernel.h"

namespace mxd {

hipError_t launch_backward_f32(const KArgs& a, bool scatter, hipStream_t stream) { return launch_dtype<float>(a, scatter, stream); }

}  // namespace mxd
