from .context import (Accelerator, CPU, Device, default_device, default_dtype, defaults,
                      defaults_like)
from .dtype import DType
from .engine import GRAPH, get_cache_stats, set_seed
from .pytree import (PyTreeDef, is_tensor, register_pytree_node, tensor_leaves, tree_flatten,
                     tree_leaves, tree_map, tree_structure, tree_unflatten)
from .tensor import Tensor, TensorImpl, realize_all
from .tracing import OpNode, Trace, trace
