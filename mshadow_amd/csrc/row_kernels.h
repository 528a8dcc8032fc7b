/*
 * The library's float instances of the row scatter / gather kernel
 * (mshadow/hip/kernels/rows_by_index.h, which holds the algorithm for every element type).
 */
#ifndef MSHADOW_AMD_CSRC_ROW_KERNELS_H_
#define MSHADOW_AMD_CSRC_ROW_KERNELS_H_

#include <mshadow/hip/kernels/rows_by_index.h>

namespace mshadow_hipk {
using mshadow::hip::kFill;
using mshadow::hip::kTakeBlock;
using mshadow::hip::kTakeGrad;
using mshadow::hip::kTakeGradSorted;
using mshadow::hip::RowsByIndexKernel;
}  // namespace mshadow_hipk
#endif  // MSHADOW_AMD_CSRC_ROW_KERNELS_H_
