from .base import (BinaryOperation, CreationOperation, Operation, ReduceOperation, ShapeOp,
                   UnaryOperation, AxisOp, ensure_tensor)
from .binary import add, div, matmul, mul, pow, sub
from .comparison import (equal, greater, greater_equal, less, less_equal, logical_and,
                         logical_not, logical_or, not_equal)
from .control_flow import where
from .convolution import conv2d, conv2d_transpose
from .creation import (arange, constant, full, full_like, gaussian, normal, ones, ones_like, tril,
                       triu, uniform, zeros, zeros_like)
from .extra import (atanh, chunk, flip, floor, is_inf, is_nan, log1p, logical_xor, minmax, outer, split,
                    trunc, unbind)
from .pooling import avg_pool2d, max_pool2d
from .reduction import (argmax, argmin, mean, reduce_max, reduce_min, reduce_sum)
from .unary import (abs, cast, cos, erf, exp, gelu, log, logsoftmax, neg, relu, rsqrt, sigmoid,
                    silu, sin, softmax, sqrt, tanh)
from .utils import call_custom_kernel
from .view import (broadcast_to, concatenate, flatten, gather, moveaxis, pad, permute, reshape,
                   scatter, slice_tensor, slice_update, squeeze, stack, swap_axes, take, transpose,
                   unsqueeze)
