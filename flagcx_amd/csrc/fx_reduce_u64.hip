// Kernel instantiations for flagcxUint64 (all ops, k = 1..8 and runtime k).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsU64() { return makeSets<flagcxUint64, true>(); }
}  // namespace fx
