"""Host-side mirror of the reference's front end (tensor -> graph -> kernel AST
-> backend registry).  It produces the ASTs a backend's `compile_ast` receives
and drives any registered backend through the reference's own interface."""

from .ast import AstNode, DType, F32, F64, I32, I64, BOOL, VarDecl
from .device import (DeviceError, EclatDevice, cache_stats, clear_cache,
                     clear_default_device, get_default_device, get_default_device_kind,
                     has_default_device, register_backend, registered_backends,
                     set_device, set_device_str)
from .executor import ExecutionError, execute_graph
from .expr import Expr
from .graph import GraphNode, GraphOp
from .lowerer import Lowerer, all_fusions, lower_graph
from .tensor import Tensor, realize_many
from .view import View
from . import nn
from . import layers, optim
from .config import exact_mode
