/*! \file broadcast_with_axis.h  include name kept for callers; the code lives under ../ext/ */
#include "../extension.h"
