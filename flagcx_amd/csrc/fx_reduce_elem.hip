// Kernel instantiations for the 16-bit types folded in the element type itself
// (RedElem: sum, max, min; k = 1..8 and runtime k).
#include "fx_launch.hpp"
namespace fx {
const KernelSet *kernelSetsElem() {
  static const KernelSet sets[6] = {makeSet<RedElem<flagcxFloat16, flagcxSum>>(),  makeSet<RedElem<flagcxFloat16, flagcxMax>>(),
                                    makeSet<RedElem<flagcxFloat16, flagcxMin>>(),  makeSet<RedElem<flagcxBfloat16, flagcxSum>>(),
                                    makeSet<RedElem<flagcxBfloat16, flagcxMax>>(), makeSet<RedElem<flagcxBfloat16, flagcxMin>>()};
  return sets;
}
}  // namespace fx
