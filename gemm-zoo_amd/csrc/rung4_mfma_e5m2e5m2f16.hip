// MFMA rung, e5m2e5m2f16 instantiation (one translation unit per type bundle keeps the build parallel).
#include "rung4_mfma.hpp"

namespace gz {
template int launch_mfma<GZ_E5M2E5M2F16>(const GemmArgs<GZ_E5M2E5M2F16>&, int, hipStream_t);
}  // namespace gz
