"""
ctypes bindings of the MI355X runtime library ``libios_runtime.so``.

``graph_latency``, ``block_latency``, ``stage_latency`` and ``graph_inference`` keep the signatures and
return values of reference python/ios/contrib/ios_runtime.py:26-135.  Differences: inputs and weights are
converted to C-contiguous float32 before they cross the boundary (the reference passes the raw buffer of
whatever array it is given), and a failing library call raises ``RuntimeError`` with the library's message
instead of terminating the process.

``Session`` exposes the library's persistent-session extension: the graph is planned once, weights stay
resident on the device and the forward pass can be run, timed and profiled repeatedly.
"""
import ctypes
import json
import os
from typing import List, Optional

import numpy as np

from ios.ir import Block, Conv, Graph, Node
from .ctypes_utils import (as_f32, c_float_array, c_int, c_ndarray_list, c_string, c_string_list,
                           get_nodes_by_type)

cur_dir = os.path.dirname(os.path.abspath(os.path.realpath(__file__)))

# Search order: an explicit override, the in-tree build directory next to the package, then the
# locations the reference glue looks at relative to this file.
libname_list = [
    '../../csrc/build/libios_runtime.so',
    'libios_runtime.so',
    '../libios_runtime.so',
    '../../libios_runtime.so',
    '../build/libios_runtime.so',
    '../../build/libios_runtime.so',
    '../../../build/libios_runtime.so',
]
lib = None


def _declare(handle):
    f32p = ctypes.POINTER(ctypes.c_float)
    i, s, vp = ctypes.c_int, ctypes.c_char_p, ctypes.c_void_p
    latency_args = [s, i, i, i, i, i, f32p, f32p]
    handle.graph_latency.argtypes = latency_args
    handle.block_latency.argtypes = latency_args
    handle.stage_latency.argtypes = [s, s, i, i, i, i, i, f32p, f32p]
    handle.graph_inference.argtypes = [s, i, vp, i, ctypes.POINTER(s), ctypes.POINTER(vp),
                                       ctypes.POINTER(vp), vp]
    handle.graph_inference_no_alloc.argtypes = handle.graph_inference.argtypes
    for name in ('graph_latency', 'block_latency', 'stage_latency', 'graph_inference', 'graph_inference_no_alloc'):
        getattr(handle, name).restype = i
    handle.ios_last_error.restype = s
    handle.ios_last_error.argtypes = []
    handle.ios_set_option.argtypes = [s, s]
    handle.ios_set_option.restype = i
    handle.ios_device_info.argtypes = [ctypes.c_char_p, i]
    handle.ios_device_info.restype = i
    handle.ios_conv_variant_names.argtypes = [ctypes.c_char_p, i]
    handle.ios_conv_variant_names.restype = i
    handle.ios_plan_describe.argtypes = [s, i, ctypes.c_char_p, i]
    handle.ios_plan_describe.restype = i
    handle.ios_plan_arena_bytes.argtypes = [s, i]
    handle.ios_plan_arena_bytes.restype = ctypes.c_longlong
    handle.ios_device_free_bytes.argtypes = []
    handle.ios_device_free_bytes.restype = ctypes.c_longlong
    handle.ios_session_create.argtypes = [s, i]
    handle.ios_session_create.restype = vp
    handle.ios_session_destroy.argtypes = [vp]
    handle.ios_session_destroy.restype = None
    handle.ios_session_set_conv_weights.argtypes = [vp, i, ctypes.POINTER(s), ctypes.POINTER(vp),
                                                    ctypes.POINTER(vp)]
    handle.ios_session_set_input.argtypes = [vp, vp]
    handle.ios_session_run.argtypes = [vp]
    handle.ios_session_enqueue.argtypes = [vp]
    handle.ios_session_synchronize.argtypes = [vp]
    handle.ios_session_get_output.argtypes = [vp, vp]
    handle.ios_session_get_tensor.argtypes = [vp, s, vp]
    handle.ios_session_measure.argtypes = [vp, i, i, i, i, f32p, f32p]
    handle.ios_session_num_ops.argtypes = [vp]
    handle.ios_session_describe.argtypes = [vp, ctypes.c_char_p, i]
    handle.ios_session_profile_ops.argtypes = [vp, i, i, f32p]
    handle.ios_session_describe_launches.argtypes = [vp, ctypes.c_char_p, i]
    handle.ios_session_profile_launches.argtypes = [vp, i, i, f32p, i]
    for name in ('ios_session_set_conv_weights', 'ios_session_set_input', 'ios_session_run',
                 'ios_session_get_output', 'ios_session_get_tensor', 'ios_session_measure', 'ios_session_enqueue', 'ios_session_synchronize',
                 'ios_session_num_ops', 'ios_session_describe', 'ios_session_profile_ops',
                 'ios_session_describe_launches', 'ios_session_profile_launches'):
        getattr(handle, name).restype = i
    return handle


def load_ios_library():
    candidates = []
    if os.environ.get('IOS_RUNTIME_LIB'):
        candidates.append(os.environ['IOS_RUNTIME_LIB'])
    candidates += [os.path.join(cur_dir, name) for name in libname_list]
    for path in candidates:
        if os.path.exists(path):
            return _declare(ctypes.cdll.LoadLibrary(path))
    raise FileNotFoundError('IOS Backend library not found')


def get_lib():
    global lib
    if lib is None:
        lib = load_ios_library()
    return lib


def _check(status, what):
    if status != 0:
        message = get_lib().ios_last_error()
        raise RuntimeError(f'{what} failed: {message.decode() if message else "unknown error"}')


def set_option(key: str, value) -> None:
    """Set a runtime option, e.g. ``set_option('executor', 'graph')``; unknown keys raise RuntimeError."""
    _check(get_lib().ios_set_option(c_string(key), c_string(str(value))), f'ios_set_option({key})')


def device_info() -> dict:
    buf = ctypes.create_string_buffer(4096)
    _check(get_lib().ios_device_info(buf, len(buf)), 'ios_device_info')
    return json.loads(buf.value.decode())


def device_free_bytes() -> int:
    """Free device memory in bytes (hipMemGetInfo)."""
    free = get_lib().ios_device_free_bytes()
    if free < 0:
        _check(1, 'ios_device_free_bytes')
    return int(free)


def conv_variant_names() -> List[str]:
    """Names of the convolution kernel configurations of this build, in index order (needs no GPU)."""
    handle = get_lib()
    cap = 1 << 14
    while True:
        buf = ctypes.create_string_buffer(cap)
        need = handle.ios_conv_variant_names(buf, c_int(cap))
        if need < cap:
            return json.loads(buf.value.decode())
        cap = need + 1


def plan_describe(graph: Graph, batch_size=1) -> List[dict]:
    """Device operations the library would launch for ``graph`` (host-only planning, needs no GPU)."""
    handle = get_lib()
    doc = c_string(json.dumps(graph.export_config()))
    cap = 1 << 16
    while True:
        buf = ctypes.create_string_buffer(cap)
        need = handle.ios_plan_describe(doc, c_int(batch_size), buf, c_int(cap))
        if need < 0:
            _check(1, 'ios_plan_describe')
        if need < cap:
            return json.loads(buf.value.decode())
        cap = need + 1


def plan_arena_bytes(graph: Graph, batch_size=1) -> int:
    """Device memory the library lays out for ``graph`` at ``batch_size`` (host-only planning, needs no GPU)."""
    need = get_lib().ios_plan_arena_bytes(c_string(json.dumps(graph.export_config())), c_int(batch_size))
    if need < 0:
        _check(1, 'ios_plan_arena_bytes')
    return int(need)


def _latency_call(fn_name, documents, batch_size, warmup, number, repeat, num_stages, profile_stage):
    handle = get_lib()
    results = c_float_array(repeat)
    stage_results = c_float_array(max(1, repeat * num_stages))
    status = getattr(handle, fn_name)(*[c_string(d) for d in documents], c_int(batch_size), c_int(warmup),
                                      c_int(number), c_int(repeat), c_int(1 if profile_stage else 0),
                                      results, stage_results)
    _check(status, fn_name)
    if profile_stage:
        return [float(v) for v in results], [float(v) for v in stage_results][:repeat * num_stages]
    return [float(v) for v in results]


def graph_latency(graph: Graph, batch_size=1, warmup=2, number=6, repeat=6, profile_stage=False):
    """
    Latency of ``graph`` under its schedule in milliseconds, one value per repeat (each the mean of
    ``number`` forward passes).  With ``profile_stage`` also returns the per-stage latencies as a flat list
    of ``repeat * num_stages`` values in row-major (repeat, stage) order.
    """
    num_stages = sum(len(b.stages) for b in graph.blocks)
    return _latency_call('graph_latency', [json.dumps(graph.export_config())], batch_size, warmup, number,
                         repeat, num_stages, profile_stage)


def block_latency(block: Block, batch_size, warmup, number, repeat, profile_stage=False):
    return _latency_call('block_latency', [json.dumps(block.export_config())], batch_size, warmup, number,
                         repeat, len(block.stages), profile_stage)


def stage_documents(stage: List[List[Node]]):
    """JSON documents for one stage: the groups' operator configs and the shapes of external producers."""
    inside = {node.name for group in stage for node in group}
    producers = {}
    for group in stage:
        for node in group:
            for term in node.inputs:
                for value in term:
                    if value.node.name not in inside:
                        producers.setdefault(value.node.name, list(value.node.output_shape))
    return (json.dumps([[node.export_config() for node in group] for group in stage]),
            json.dumps(producers))


def stage_latency(stage: List[List[Node]], batch_size, warmup, number, repeat, profile_stage=False):
    """Latency of one stage (groups of operators run concurrently) with synthetic inputs, in ms per repeat."""
    stage_json, input_json = stage_documents(stage)
    return _latency_call('stage_latency', [stage_json, input_json], batch_size, warmup, number, repeat, 1,
                         profile_stage)


def _weight_lists(graph: Graph):
    convs: List[Conv] = list(get_nodes_by_type(graph.nodes(), Conv))
    for conv in convs:
        if conv.weight is None or conv.bias is None:
            raise ValueError(f'convolution {conv.name} has no weights; call graph.init_weights() first')
    names = [conv.name for conv in convs]
    weights = [as_f32(conv.weight) for conv in convs]
    biases = [as_f32(conv.bias) for conv in convs]
    return names, weights, biases


def graph_inference(graph: Graph, batch_size, input: np.ndarray, no_alloc=False):
    """
    Run ``graph`` on ``input`` (batch, C, H, W) with the weights stored in its Conv operators.  ``no_alloc`` calls the
    library's variant that lays all device buffers out in its static scratch array and allocates nothing.
    """
    handle = get_lib()
    x = as_f32(input)
    expected = (batch_size, *graph.enter_node.output_shape)
    if tuple(x.shape) != tuple(expected):
        raise ValueError(f'input has shape {x.shape}, expected {expected}')
    output = np.empty(shape=(batch_size, *graph.blocks[-1].exit_node.output_shape), dtype=np.float32)
    names, weights, biases = _weight_lists(graph)
    name_array = c_string_list(names)
    entry = handle.graph_inference_no_alloc if no_alloc else handle.graph_inference
    status = entry(c_string(json.dumps(graph.export_config())), c_int(batch_size),
                                    x.ctypes.data_as(ctypes.c_void_p), c_int(len(names)),
                                    ctypes.cast(name_array, ctypes.POINTER(ctypes.c_char_p)),
                                    ctypes.cast(c_ndarray_list(weights), ctypes.POINTER(ctypes.c_void_p)),
                                    ctypes.cast(c_ndarray_list(biases), ctypes.POINTER(ctypes.c_void_p)),
                                    output.ctypes.data_as(ctypes.c_void_p))
    _check(status, 'graph_inference_no_alloc' if no_alloc else 'graph_inference')
    return output


class Session:
    """A planned graph that stays on the device: upload weights once, then run / measure / profile."""

    def __init__(self, graph: Graph, batch_size: int):
        self._lib = get_lib()
        self.graph, self.batch_size = graph, batch_size
        self._handle = self._lib.ios_session_create(c_string(json.dumps(graph.export_config())), c_int(batch_size))
        if not self._handle:
            _check(1, 'ios_session_create')
        self.output_shape = (batch_size, *graph.blocks[-1].exit_node.output_shape)

    def close(self):
        if self._handle:
            self._lib.ios_session_destroy(self._handle)
            self._handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def load_weights(self):
        names, weights, biases = _weight_lists(self.graph)
        name_array = c_string_list(names)
        _check(self._lib.ios_session_set_conv_weights(
            self._handle, c_int(len(names)), ctypes.cast(name_array, ctypes.POINTER(ctypes.c_char_p)),
            ctypes.cast(c_ndarray_list(weights), ctypes.POINTER(ctypes.c_void_p)),
            ctypes.cast(c_ndarray_list(biases), ctypes.POINTER(ctypes.c_void_p))), 'ios_session_set_conv_weights')

    def set_input(self, x: np.ndarray):
        x = as_f32(x)
        expected = (self.batch_size, *self.graph.enter_node.output_shape)
        if tuple(x.shape) != tuple(expected):
            raise ValueError(f'input has shape {x.shape}, expected {expected}')
        _check(self._lib.ios_session_set_input(self._handle, x.ctypes.data_as(ctypes.c_void_p)),
               'ios_session_set_input')

    def run(self):
        _check(self._lib.ios_session_run(self._handle), 'ios_session_run')

    def enqueue(self):
        """Queue one forward pass behind the earlier ones without waiting (see ``synchronize``)."""
        _check(self._lib.ios_session_enqueue(self._handle), 'ios_session_enqueue')

    def synchronize(self):
        _check(self._lib.ios_session_synchronize(self._handle), 'ios_session_synchronize')

    def output(self) -> np.ndarray:
        out = np.empty(self.output_shape, dtype=np.float32)
        _check(self._lib.ios_session_get_output(self._handle, out.ctypes.data_as(ctypes.c_void_p)),
               'ios_session_get_output')
        return out

    def tensor(self, node: Node) -> np.ndarray:
        """Output of any operator of the graph after ``run`` (dense copy, shape (batch, C, H, W))."""
        out = np.empty((self.batch_size, *node.output_shape), dtype=np.float32)
        _check(self._lib.ios_session_get_tensor(self._handle, c_string(node.name),
                                                out.ctypes.data_as(ctypes.c_void_p)), 'ios_session_get_tensor')
        return out

    def measure(self, warmup=2, number=6, repeat=6, profile_stage=False):
        num_stages = sum(len(b.stages) for b in self.graph.blocks)
        results = c_float_array(repeat)
        stage_results = c_float_array(max(1, repeat * num_stages))
        _check(self._lib.ios_session_measure(self._handle, c_int(warmup), c_int(number), c_int(repeat),
                                             c_int(1 if profile_stage else 0), results, stage_results),
               'ios_session_measure')
        if profile_stage:
            return [float(v) for v in results], [float(v) for v in stage_results][:repeat * num_stages]
        return [float(v) for v in results]

    def describe(self) -> List[dict]:
        """One record per device operation: name, kind, kernel variant, stage, group, flops, bytes."""
        cap = 1 << 16
        while True:
            buf = ctypes.create_string_buffer(cap)
            need = self._lib.ios_session_describe(self._handle, buf, c_int(cap))
            if need < 0:
                _check(1, 'ios_session_describe')
            if need < cap:
                return json.loads(buf.value.decode())
            cap = need + 1

    def launches(self) -> List[dict]:
        """The kernel launches of one pass under the executor in force: kernel name, stage, operations, flops, bytes."""
        cap = 1 << 16
        while True:
            buf = ctypes.create_string_buffer(cap)
            need = self._lib.ios_session_describe_launches(self._handle, buf, c_int(cap))
            if need < 0:
                _check(1, 'ios_session_describe_launches')
            if need < cap:
                return json.loads(buf.value.decode())
            cap = need + 1

    def profile_launches(self, warmup=2, repeat=10) -> List[float]:
        """Mean milliseconds of every launch of the pass (see ``launches``) issued back to back, HIP-event timed."""
        n = len(self.launches())
        out = c_float_array(max(1, n))
        _check(self._lib.ios_session_profile_launches(self._handle, c_int(warmup), c_int(repeat), out, c_int(n)),
               'ios_session_profile_launches')
        return [float(v) for v in out][:n]

    def profile_ops(self, warmup=2, repeat=10) -> List[float]:
        """Mean milliseconds of every device operation run alone on one stream, HIP-event timed."""
        n = self._lib.ios_session_num_ops(self._handle)
        out = c_float_array(max(1, n))
        _check(self._lib.ios_session_profile_ops(self._handle, c_int(warmup), c_int(repeat), out),
               'ios_session_profile_ops')
        return [float(v) for v in out][:n]
