/*! \file expr_scalar-inl.h  public include name kept for callers; everything comes with tensor.h */
#ifndef MSHADOW_EXPR_SCALAR_INL_H_
#define MSHADOW_EXPR_SCALAR_INL_H_
#include "./tensor.h"
#endif  // MSHADOW_EXPR_SCALAR_INL_H_
