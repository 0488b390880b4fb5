// Kernel instantiations for flagcxBfloat16 (all ops, k = 1..8 and runtime k).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsBF16() { return makeSets<flagcxBfloat16, false>(); }
}  // namespace fx
