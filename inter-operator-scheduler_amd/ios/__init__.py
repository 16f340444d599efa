"""
ios: inter-operator scheduler for CNN inference on AMD Instinct MI355X.

Public surface (same names as reference python/ios/__init__.py:1-9): graph construction
(``placeholder, conv2d, pool2d, identity, relu, activation, multiply, addition, element, sequential``,
``Graph``, ``Block``, ``reset_name``), the schedule search ``optimize``, the cost models, the runtime
bindings ``ios_runtime`` and the model zoo ``models``.
"""
from .ir import Graph, Block
from .cost_model import CostModel, IOSCostModel, RandomCostModel, AnalyticCostModel
from .models.common import placeholder, reset_name
from .models.common import conv2d, pool2d, identity, relu, activation, multiply, addition, element, sequential
from .models.common import sigmoid, tanh, sep_conv, relu_sep_conv, relu_conv
from .optimizer import optimize, graph_dp_summary
from .contrib import ios_runtime
from .visualizer import draw
from . import models

__version__ = "0.1.dev0"
