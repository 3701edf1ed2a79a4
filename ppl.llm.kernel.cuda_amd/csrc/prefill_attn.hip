// placeholder until the MFMA tile lands
#include "launch_params.h"
namespace pmxhip {
int launch_prefill(const PrefillLaunch&, hipStream_t) { return 1; }
}
