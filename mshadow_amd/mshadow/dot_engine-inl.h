/*! \file dot_engine-inl.h  public include name kept for callers; see dot_engine.h */
#ifndef MSHADOW_DOT_ENGINE_INL_H_
#define MSHADOW_DOT_ENGINE_INL_H_
#include "./dot_engine.h"
#endif  // MSHADOW_DOT_ENGINE_INL_H_
