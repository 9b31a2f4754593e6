// MFMA rung, e4m3e4m3f16 instantiation (one translation unit per type bundle keeps the build parallel).
#include "rung4_mfma.hpp"

namespace gz {
template int launch_mfma<GZ_E4M3E4M3F16>(const GemmArgs<GZ_E4M3E4M3F16>&, int, hipStream_t);
}  // namespace gz
