// Kernel instantiations for flagcxInt64 (all ops, k = 1..8 and runtime k).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsI64() { return makeSets<flagcxInt64, true>(); }
}  // namespace fx
