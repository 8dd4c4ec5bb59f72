// One fifth of the executor's kernels: the two element types 2 * MSCCLX_KERNEL_GROUP and
// 2 * MSCCLX_KERNEL_GROUP + 1 (mscclx_dtype), every reduction, every variant.  Compiled five times
// (build.py) so that the translation units build in parallel.
#include "exec_device.h"

#ifndef MSCCLX_KERNEL_GROUP
#error "compile with -DMSCCLX_KERNEL_GROUP=0..4"
#endif
#define MSCCLX_PASTE2(a, b) a##b
#define MSCCLX_PASTE(a, b) MSCCLX_PASTE2(a, b)

namespace mscclx {

kernel_fn MSCCLX_PASTE(pick_kernel_group_, MSCCLX_KERNEL_GROUP)(int dtype, int op, bool ll, int fold, bool ragged) {
  static_assert(2 * MSCCLX_KERNEL_GROUP + 1 < MSCCLX_NUM_DTYPES, "two element types per group");
  if (dtype == 2 * MSCCLX_KERNEL_GROUP) return pick_op<2 * MSCCLX_KERNEL_GROUP>(op, ll, fold, ragged);
  if (dtype == 2 * MSCCLX_KERNEL_GROUP + 1) return pick_op<2 * MSCCLX_KERNEL_GROUP + 1>(op, ll, fold, ragged);
  return nullptr;
}

}  // namespace mscclx
