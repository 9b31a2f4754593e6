// MFMA rung, bf16bf16bf16 instantiation (one translation unit per type bundle keeps the build parallel).
#include "rung4_mfma.hpp"

namespace gz {
template int launch_mfma<GZ_BF16BF16BF16>(const GemmArgs<GZ_BF16BF16BF16>&, int, hipStream_t);
}  // namespace gz
