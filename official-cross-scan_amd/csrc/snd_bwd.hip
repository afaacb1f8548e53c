#include "snd_device.h"
namespace snd {
int launch_bwd(const snd_bwd_params &p, hipStream_t stream) { (void)p; (void)stream; return SND_ERR_LAUNCH; }
}
