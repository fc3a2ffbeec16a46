"""Python surface of the auto-tensorize path, re-exported flat as the reference does
(python/tvm/auto_tensorize/__init__.py:1-6)."""
from .hw_abstraction import *            # noqa: F401,F403
from .hw_abstraction import compute_dag_from_tensors, register_abstraction, ComputeDAG  # noqa: F401
from .hw_abs_dag import *                # noqa: F401,F403
from .hw_abs_dag import register_hw_abs_dag, query_hw_abs_dag  # noqa: F401
from .intrin_match import *              # noqa: F401,F403
from .compute_transform import *         # noqa: F401,F403
from .policy import all_fit, first_fit, best_fit, choose_one  # noqa: F401
from .lowering import lower_main_op, LoweredOp, NoKernelError  # noqa: F401
from .schedule import *                  # noqa: F401,F403
from .measure import MeasureOptions, evaluate_params, MAX_FLOAT  # noqa: F401
from .target import MI355X, get_device_arch  # noqa: F401
from .runtime import build, array, context, Module, NDArray  # noqa: F401
from .auto_tensorize import (AutoTensorizeResult, auto_tensorize, auto_tensorize_compute,  # noqa: F401
                             auto_tensorize_schedule, auto_tensorize_v4, get_schedule)
from .network import (AutoScheduleMultiGraphDispatch, AutoTensorizeContext, SubGraph, evaluate_graph,  # noqa: F401
                      NETWORKS, bert_base, mi_lstm, mobilenet_v1, resnet18, resnet50, shufflenet)
