// Kernel instantiations for flagcxInt8 (all ops, k = 1..8 and runtime k).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsI8() { return makeSets<flagcxInt8, true>(); }
}  // namespace fx
