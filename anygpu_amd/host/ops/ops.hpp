// Umbrella header of the operator layer (the reference's srcs/ops/ops.hpp role).
#ifndef __OPS__
#define __OPS__

#include "binary_ops.hpp"
#include "math_ops.hpp"
#include "mm_ops.hpp"
#include "norm_ops.hpp"
#include "shape_ops.hpp"
#include "softmax_ops.hpp"
#include "transp_ops.hpp"
#include "causal_conv1d.hpp"

#endif  // __OPS__
