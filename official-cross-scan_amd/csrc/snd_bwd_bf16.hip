// Backward kernel instantiation for bf16 inputs.
#include "snd_bwd_kernel.h"
namespace snd {
int launch_bwd_bf16(const snd_bwd_params &p, hipStream_t stream) { return launch_bwd_t<bf16_t>(p, stream); }
int configure_bwd_bf16() { return configure_bwd_t<bf16_t>(); }
}  // namespace snd
