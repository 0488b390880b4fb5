// Kernel instantiations for the byte mover (copy slices, pack, unpack).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsCopy() {
  static const KernelSet sets[3] = {makeCopySet<1>(), makeCopySet<2>(), makeCopySet<4>()};
  return sets;
}
}  // namespace fx
