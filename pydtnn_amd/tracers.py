"""Event tracing with the reference's event vocabulary.

Event types and values follow pydtnn/tracers/events.py:24-70: an event is ``(type, value)`` with
``value = layer.id * EVENTS + kind`` to open a region and ``0`` to close the innermost open region of that
type.  Three tracers share the call surface of pydtnn/tracers/tracer.py:55-106 (``emit_event``,
``emit_nevent``, ``define_event_types``, enable / disable):

* ``NullTracer``     tracing off (the default of a Model);
* ``SimpleTracer``   host-side timing per event, written as the reference's ';'-separated table
                     (pydtnn/tracers/simple_tracer.py:46-84); because kernels run asynchronously the device is
                     synchronised when a region opens and closes, so the times are those of the GPU work inside;
* ``RoctxTracer``    opens / closes a roctx range named like the reference's event, so that
                     ``rocprofv3 --marker-trace`` shows layers and operations around the kernels it traces.
"""
import atexit
import ctypes
from collections import defaultdict
from timeit import default_timer as timer

PYDTNN_MDL_EVENT = 60000001
_MDL_NAMES = ("FORWARD", "BACKWARD", "ALLREDUCE_DW", "WAIT_DW", "UPDATE_DW")
PYDTNN_MDL_EVENTS = len(_MDL_NAMES)

PYDTNN_OPS_EVENT = 60000002
_OPS_NAMES = (
    "ALLREDUCE_DW", "BACKWARD_CONVGEMM", "BACKWARD_CUBLAS_MATMUL_DW", "BACKWARD_CUBLAS_MATMUL_DX",
    "BACKWARD_CUBLAS_MATVEC_DB", "BACKWARD_CUDNN_DB", "BACKWARD_CUDNN_DW", "BACKWARD_CUDNN_DX",
    "BACKWARD_DECONV_GEMM", "BACKWARD_ELTW_SUM", "BACKWARD_IM2COL", "BACKWARD_RESHAPE_DW", "BACKWARD_RESHAPE_DX",
    "BACKWARD_SPLIT", "BACKWARD_SUM_BIASES", "BACKWARD_TRANSPOSE_DY", "BACKWARD_TRANSPOSE_W", "COMP_DW_MATMUL",
    "COMP_DX_COL2IM", "COMP_DX_MATMUL", "FORWARD_DEPTHWISE_CONV", "FORWARD_POINTWISE_CONV", "FORWARD_CONCAT",
    "FORWARD_CONVGEMM", "FORWARD_CONVWINOGRAD", "FORWARD_CUBLAS_MATMUL", "FORWARD_CUDNN",
    "FORWARD_CUDNN_SUM_BIASES", "FORWARD_ELTW_SUM", "FORWARD_IM2COL", "FORWARD_MATMUL", "FORWARD_REPLICATE",
    "FORWARD_RESHAPE_W", "FORWARD_RESHAPE_Y", "FORWARD_SUM_BIASES", "FORWARD_TRANSPOSE_Y")
PYDTNN_OPS_EVENTS = len(_OPS_NAMES)

for _i, _n in enumerate(_MDL_NAMES, 1):
    globals()["PYDTNN_MDL_" + _n] = _i
for _i, _n in enumerate(_OPS_NAMES, 1):
    globals()["PYDTNN_OPS_" + _n] = _i


class NullTracer:
    def define_event_types(self, model):
        pass

    def emit_event(self, evt_type, evt_val, stream=None):
        pass

    def emit_nevent(self, evt_types, evt_vals, stream=None):
        pass


class Tracer:
    """Common part: event names per model, switching on and off (pydtnn/tracers/tracer.py:60-131)."""

    def __init__(self, tracing=True):
        self.event_names = {PYDTNN_MDL_EVENT: {0: "End"}, PYDTNN_OPS_EVENT: {0: "End"}}
        self.type_names = {PYDTNN_MDL_EVENT: "Model", PYDTNN_OPS_EVENT: "Operations"}
        self.tracing = False
        if tracing:
            self.enable_tracing()

    def enable_tracing(self):
        self.tracing = True

    def disable_tracing(self):
        self.tracing = False

    def define_event_types(self, model):
        if not self.tracing:
            return
        for layer in model.get_all_layers():
            for val, name in enumerate(_MDL_NAMES, 1):
                self.event_names[PYDTNN_MDL_EVENT][layer.id * PYDTNN_MDL_EVENTS + val] = \
                    f"{layer.canonical_name_with_id}_{name.lower()}"
            for val, name in enumerate(_OPS_NAMES, 1):
                self.event_names[PYDTNN_OPS_EVENT][layer.id * PYDTNN_OPS_EVENTS + val] = \
                    f"{layer.id:03}_{layer.canonical_name}_{name.lower()}"

    def name_of(self, evt_type, evt_val):
        return self.event_names.get(evt_type, {}).get(evt_val, f"{evt_type}:{evt_val}")

    def emit_event(self, evt_type, evt_val, stream=None):
        if self.tracing:
            self._emit_event(evt_type, evt_val)

    def emit_nevent(self, evt_types, evt_vals, stream=None):
        # several regions opened at once, or closed in reverse order (simple_tracer.py:60-66)
        pairs = list(zip(evt_types, evt_vals))
        if evt_vals[0] == 0:
            pairs.reverse()
        for evt_type, evt_val in pairs:
            self.emit_event(evt_type, evt_val)

    def _emit_event(self, evt_type, evt_val):
        raise NotImplementedError


def _device_sync():
    import torch
    if torch.cuda.is_available():
        torch.cuda.synchronize()


class SimpleTracer(Tracer):
    def __init__(self, tracing=True, output_filename="simple_tracer.csv", sync=None):
        self.output_filename = output_filename
        self.sync = sync if sync is not None else _device_sync
        self.events = defaultdict(lambda: defaultdict(lambda: [0, []]))
        self.pending_events = []
        self._registered = False
        super().__init__(tracing)

    def enable_tracing(self):
        super().enable_tracing()
        if not self._registered:
            atexit.register(self.write_output)
            self._registered = True

    def _emit_event(self, evt_type, evt_val):
        self.sync()
        if evt_val != 0:
            self.pending_events.append((evt_type, evt_val, timer()))
            return
        toc = timer()
        if not self.pending_events:
            raise ValueError("Received an 'End' event but there are no pending events!")
        if self.pending_events[-1][0] != evt_type:
            raise ValueError("Received an 'End' event for a different event type than expected!")
        _type, _val, tic = self.pending_events.pop()
        self.events[_type][_val][0] += 1
        self.events[_type][_val][1].append(toc - tic)

    def write_output(self):
        if not self.events:
            return
        with open(self.output_filename, "w") as f:
            f.write("Event type;Event value;Event name;Calls;Total time;Median of times\n")
            for evt_type, events in self.events.items():
                for value, (calls, times) in events.items():
                    times = sorted(times)
                    if not times:   # an event that was opened and never closed has no duration to report
                        continue
                    f.write(f"{self.type_names[evt_type]};{value};{self.name_of(evt_type, value)};{calls};"
                            f"{sum(times)};{times[len(times) // 2]}\n")


class RoctxTracer(Tracer):
    """Ranges for rocprofv3's marker trace.  Needs libroctx64 (part of ROCm); raises OSError without it."""

    def __init__(self, tracing=True, library="libroctx64.so"):
        self._lib = ctypes.CDLL(library)
        self._lib.roctxRangePushA.argtypes = [ctypes.c_char_p]
        self._lib.roctxRangePushA.restype = ctypes.c_int
        self._lib.roctxRangePop.restype = ctypes.c_int
        self._open = []
        super().__init__(tracing)

    def _emit_event(self, evt_type, evt_val):
        if evt_val != 0:
            self._open.append(evt_type)
            self._lib.roctxRangePushA(self.name_of(evt_type, evt_val).encode())
            return
        if not self._open or self._open[-1] != evt_type:
            raise ValueError("Received an 'End' event that does not close the innermost open region!")
        self._open.pop()
        self._lib.roctxRangePop()
