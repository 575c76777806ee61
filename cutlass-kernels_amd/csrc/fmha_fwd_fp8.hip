// FMHA forward, fp8 e4m3 operands -- placeholder until the f8f6f4 kernel lands.
#include "fmha_common.h"
namespace cfk {
bool plan_fmha_fp8(int, int, int, int, int, FmhaPlan *) { return false; }
hipError_t launch_fmha_fp8(const FmhaArgs &, int, hipStream_t) { return hipErrorNotSupported; }
}  // namespace cfk
