// Kernel instantiations for flagcxInt32 (all ops, k = 1..8 and runtime k).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsI32() { return makeSets<flagcxInt32, false>(); }
}  // namespace fx
