// Kernel instantiations for flagcxFloat32 (all ops, k = 1..8 and runtime k).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsF32() { return makeSets<flagcxFloat32, false>(); }
}  // namespace fx
