// Kernel instantiations for the 16-bit types folded in the element type itself
// (RedElem: sum, max, min; k = 1..8 and runtime k).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsElem() {
  static const KernelSet sets[6] = {makeSet<RedElem<flagcxFloat16, flagcxSum>, true>(),  makeSet<RedElem<flagcxFloat16, flagcxMax>, true>(),
                                    makeSet<RedElem<flagcxFloat16, flagcxMin>, true>(),  makeSet<RedElem<flagcxBfloat16, flagcxSum>, true>(),
                                    makeSet<RedElem<flagcxBfloat16, flagcxMax>, true>(), makeSet<RedElem<flagcxBfloat16, flagcxMin>, true>()};
  return sets;
}
}  // namespace fx
