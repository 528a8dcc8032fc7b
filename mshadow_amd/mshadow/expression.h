/*! \file expression.h  public include name kept for callers; the nodes live in expr/nodes.h */
#ifndef MSHADOW_EXPRESSION_H_
#define MSHADOW_EXPRESSION_H_
#include "./expr/nodes.h"
#endif  // MSHADOW_EXPRESSION_H_
