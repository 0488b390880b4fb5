// Kernel instantiations for flagcxFloat64 (all ops, k = 1..8 and runtime k).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsF64() { return makeSets<flagcxFloat64, true>(); }
}  // namespace fx
