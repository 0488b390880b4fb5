// Kernel instantiations for flagcxUint8 (all ops, k = 1..8 and runtime k).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsU8() { return makeSets<flagcxUint8, true>(); }
}  // namespace fx
