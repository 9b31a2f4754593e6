// MFMA rung, f16f16f16 instantiation (one translation unit per type bundle keeps the build parallel).
#include "rung4_mfma.hpp"

namespace gz {
template int launch_mfma<GZ_F16F16F16>(const GemmArgs<GZ_F16F16F16>&, int, hipStream_t);
}  // namespace gz
