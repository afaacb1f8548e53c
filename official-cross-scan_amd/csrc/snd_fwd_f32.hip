// Forward kernel instantiation for f32 inputs.
#include "snd_fwd_kernel.h"
namespace snd {
int launch_fwd_f32(const snd_fwd_params &p, hipStream_t stream) { return launch_fwd_t<float>(p, stream); }
}  // namespace snd
