/*! \file implicit_gemm.h  include name kept for callers; the code lives under ../ext/ */
#include "../extension.h"
