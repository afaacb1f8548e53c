// Backward kernel instantiation for f16 inputs.
#include "snd_bwd_kernel.h"
namespace snd {
int launch_bwd_f16(const snd_bwd_params &p, hipStream_t stream) { return launch_bwd_t<f16_t>(p, stream); }
int configure_bwd_f16() { return configure_bwd_t<f16_t>(); }
}  // namespace snd
