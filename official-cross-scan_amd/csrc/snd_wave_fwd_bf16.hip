// Row-segment wavefront forward (1-4 states per channel): instantiations for bf16_t inputs.
#include "snd_wave_fwd_kernel.h"
namespace snd {
int launch_wave_fwd_bf16(const snd_fwd_params &p, float *group_ws, hipStream_t stream) { return launch_wave_fwd_t<bf16_t>(p, group_ws, stream); }
}  // namespace snd
