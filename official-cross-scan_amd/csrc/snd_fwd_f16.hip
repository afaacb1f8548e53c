// Forward kernel instantiation for f16 inputs.
#include "snd_fwd_kernel.h"
namespace snd {
int launch_fwd_f16(const snd_fwd_params &p, hipStream_t stream) { return launch_fwd_t<f16_t>(p, stream); }
}  // namespace snd
