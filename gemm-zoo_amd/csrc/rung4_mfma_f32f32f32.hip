// MFMA rung, f32f32f32 instantiation (one translation unit per type bundle keeps the build parallel).
#include "rung4_mfma.hpp"

namespace gz {
template int launch_mfma<GZ_F32F32F32>(const GemmArgs<GZ_F32F32F32>&, int, hipStream_t);
}  // namespace gz
