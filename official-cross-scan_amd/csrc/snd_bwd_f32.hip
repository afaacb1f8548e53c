// Backward kernel instantiation for f32 inputs.
#include "snd_bwd_kernel.h"
namespace snd {
int launch_bwd_f32(const snd_bwd_params &p, hipStream_t stream) { return launch_bwd_t<float>(p, stream); }
int configure_bwd_f32() { return configure_bwd_t<float>(); }
}  // namespace snd
