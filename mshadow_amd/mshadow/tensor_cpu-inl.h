/*! \file tensor_cpu-inl.h  public include name kept for callers; everything comes with tensor.h */
#ifndef MSHADOW_TENSOR_CPU_INL_H_
#define MSHADOW_TENSOR_CPU_INL_H_
#include "./tensor.h"
#endif  // MSHADOW_TENSOR_CPU_INL_H_
