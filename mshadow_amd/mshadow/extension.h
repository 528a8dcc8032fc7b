/*! \file extension.h  the expression extensions this backend provides */
#ifndef MSHADOW_EXTENSION_H_
#define MSHADOW_EXTENSION_H_
#include "./tensor.h"
#include "./ext/reduceto1d.h"
#include "./ext/pooling.h"
#include "./ext/patches.h"
#include "./ext/shaping.h"
#include "./ext/channels.h"
#include "./ext/axes.h"
#include "./ext/indexing.h"
#include "./ext/complex.h"
#include "./ext/implicit_gemm.h"
#endif  // MSHADOW_EXTENSION_H_
