// Kernel instantiations for flagcxUint32 (all ops, k = 1..8 and runtime k).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsU32() { return makeSets<flagcxUint32, true>(); }
}  // namespace fx
