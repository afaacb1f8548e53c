// Row-segment wavefront forward (1-4 states per channel): instantiations for float inputs.
#include "snd_wave_fwd_kernel.h"
namespace snd {
int launch_wave_fwd_f32(const snd_fwd_params &p, float *group_ws, hipStream_t stream) { return launch_wave_fwd_t<float>(p, group_ws, stream); }
}  // namespace snd
