/*! \file unpack_patch2col.h  include name kept for callers; the code lives under ../ext/ */
#include "../extension.h"
