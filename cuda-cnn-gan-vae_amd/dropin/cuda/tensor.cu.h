// Drop-in for the reference's cuda/tensor.cu.h: the four tensor classes on top of the C ABI of libmi355tensor.so.
// The include guards are the reference's own, so a translation unit that sees these headers first skips the CUDA ones.
#ifndef TENSOR_CU_H
#define TENSOR_CU_H

#include "ctensor.cu.h"
#include "ctensormath.cu.h"
#include "ctensorconv.cu.h"
#include "ctensorapplyfunc.cu.h"

#endif
