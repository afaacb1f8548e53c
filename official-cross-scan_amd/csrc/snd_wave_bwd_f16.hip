// Row-segment wavefront backward (1-4 states per channel): instantiations for f16_t inputs.
#include "snd_wave_bwd_kernel.h"
namespace snd {
int launch_wave_bwd_f16(const snd_bwd_params &p, float *group_ws, hipStream_t stream) { return launch_wave_bwd_t<f16_t>(p, group_ws, stream); }
}  // namespace snd
