"""nabla_amd: an MI355X-native execution backend behind Nabla's tensor API.

The public names follow nabla/__init__.py for the path this package covers:
tensors, the Operation plugin classes, the op functions of the MLP /
transformer / CNN / LoRA examples, ``grad`` / ``value_and_grad`` / ``vjp`` /
``compile``, ``realize_all`` and ``call_custom_kernel``.
"""
from . import config
from .core import (CPU, GRAPH, Accelerator, Device, DType, OpNode, PyTreeDef, Tensor, TensorImpl,
                   Trace, default_device, default_dtype, defaults, defaults_like, get_cache_stats,
                   is_tensor, realize_all, register_pytree_node, set_seed, tensor_leaves, trace,
                   tree_flatten, tree_leaves, tree_map, tree_structure, tree_unflatten)
from .core.backward import backward, backward_on_trace
from .ops import *  # noqa: F401,F403
from .ops import (BinaryOperation, CreationOperation, Operation, ReduceOperation,
                  UnaryOperation, call_custom_kernel)
from .ops.reduction import reduce_max as max, reduce_min as min, reduce_sum as sum  # noqa: A001
from .transforms import (CompilationStats, CompiledFunction, compile, grad, jacfwd, jacrev, jvp,
                         value_and_grad, vjp, vmap)
from . import nn  # noqa: E402
from . import testing  # noqa: E402
from . import workloads  # noqa: E402

__version__ = "0.1.0"
