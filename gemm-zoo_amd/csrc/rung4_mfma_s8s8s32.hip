// MFMA rung, s8s8s32 instantiation (one translation unit per type bundle keeps the build parallel).
#include "rung4_mfma.hpp"

namespace gz {
template int launch_mfma<GZ_S8S8S32>(const GemmArgs<GZ_S8S8S32>&, int, hipStream_t);
}  // namespace gz
