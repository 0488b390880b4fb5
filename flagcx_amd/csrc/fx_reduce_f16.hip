// Kernel instantiations for flagcxFloat16 (all ops, k = 1..8 and runtime k).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsF16() { return makeSets<flagcxFloat16, false>(); }
}  // namespace fx
