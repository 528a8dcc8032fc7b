/*! \file expr_engine-inl.h  public include name kept for callers; see expr/plan.h,
 *  expr/traits.h and expr/engine.h */
#ifndef MSHADOW_EXPR_ENGINE_INL_H_
#define MSHADOW_EXPR_ENGINE_INL_H_
#include "./tensor.h"
#endif  // MSHADOW_EXPR_ENGINE_INL_H_
