"""Python mirror of lc0's Network / NetworkComputation interface
(src/neural/network.h:43-126) on top of the C ABI in include/lc0mi.h.

Method names and meanings are the reference's: AddInput, ComputeBlocking,
GetBatchSize, GetQVal, GetDVal, GetPVal, GetMVal; errors surface as
BackendError (the reference throws lczero::Exception). The library is the only
compute path: if liblc0mi.so is missing or no GPU is present, construction
fails; nothing falls back to the CPU.
"""
import ctypes as C
import os
from collections import namedtuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

InputPlane = namedtuple("InputPlane", ["mask", "value"])
NetworkCapabilities = namedtuple("NetworkCapabilities", ["input_format", "output_format", "moves_left"])
KernelTime = namedtuple("KernelTime", ["name", "ms", "launches", "flops", "bytes"])


class BackendError(RuntimeError):
    pass


def library_path():
    return os.path.join(_HERE, "liblc0mi.so")


def load_library():
    """Loads liblc0mi.so (built in-tree by lc0_amd/build.py); never builds it."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = library_path()
    if not os.path.exists(path):
        raise BackendError("%s is missing: build it with `python -m lc0_amd.build`" % path)
    lib = C.CDLL(path)
    vp, ci, cf = C.c_void_p, C.c_int, C.c_float
    lib.lc0mi_net_create_from_buffer.argtypes = [vp, C.c_size_t, C.c_char_p, C.POINTER(vp)]
    lib.lc0mi_net_create_from_file.argtypes = [C.c_char_p, C.c_char_p, C.POINTER(vp)]
    lib.lc0mi_net_destroy.argtypes = [vp]
    lib.lc0mi_net_destroy.restype = None
    lib.lc0mi_net_caps.argtypes = [vp, C.POINTER(ci), C.POINTER(ci), C.POINTER(ci)]
    lib.lc0mi_net_hints.argtypes = [vp] + [C.POINTER(ci)] * 5
    lib.lc0mi_comp_create.argtypes = [vp, C.POINTER(vp)]
    lib.lc0mi_comp_destroy.argtypes = [vp]
    lib.lc0mi_comp_destroy.restype = None
    lib.lc0mi_comp_add_input.argtypes = [vp, vp, vp]
    lib.lc0mi_comp_add_inputs.argtypes = [vp, ci, vp, vp]
    lib.lc0mi_comp_compute_blocking.argtypes = [vp]
    lib.lc0mi_comp_batch_size.argtypes = [vp]
    for name in ("lc0mi_comp_q", "lc0mi_comp_d", "lc0mi_comp_m"):
        getattr(lib, name).argtypes = [vp, ci]
        getattr(lib, name).restype = cf
    lib.lc0mi_comp_p.argtypes = [vp, ci, ci]
    lib.lc0mi_comp_p.restype = cf
    lib.lc0mi_comp_policy_row.argtypes = [vp, ci]
    lib.lc0mi_comp_policy_row.restype = C.POINTER(cf)
    lib.lc0mi_comp_add_legal_moves.argtypes = [vp, ci, vp]
    lib.lc0mi_comp_set_policy_softmax_temperature.argtypes = [vp, cf]
    lib.lc0mi_comp_legal_policy.argtypes = [vp, ci, C.POINTER(ci)]
    lib.lc0mi_comp_legal_policy.restype = C.POINTER(cf)
    lib.lc0mi_last_error.restype = C.c_char_p
    lib.lc0mi_net_set_profiling.argtypes = [vp, ci]
    lib.lc0mi_net_take_profile.argtypes = [vp, C.c_char_p, ci]
    lib.lc0mi_net_time_resident_forward.argtypes = [vp, ci, ci, C.POINTER(C.c_double)]
    lib.lc0mi_net_calibrate_fp8.argtypes = [vp, ci, vp, vp]
    lib.lc0mi_net_fp8_scales.argtypes = [vp, vp, ci]
    lib.lc0mi_weights_list.argtypes = [vp, C.c_size_t, C.c_char_p, ci]
    lib.lc0mi_weights_tensor.argtypes = [vp, C.c_size_t, C.c_char_p, vp, C.c_longlong]
    lib.lc0mi_weights_tensor.restype = C.c_longlong
    for name, typ in (("lc0mi_attn_policy_map", C.c_int16), ("lc0mi_conv_policy_map", C.c_int16),
                      ("lc0mi_pos_encoding", cf)):
        getattr(lib, name).argtypes = [C.POINTER(ci)]
        getattr(lib, name).restype = C.POINTER(typ)
    _LIB = lib
    return lib


def _check(rc):
    if rc != 0:
        raise BackendError(load_library().lc0mi_last_error().decode(errors="replace"))


def _table(fn_name, dtype):
    lib = load_library()
    n = C.c_int(0)
    ptr = getattr(lib, fn_name)(C.byref(n))
    return np.ctypeslib.as_array(ptr, (n.value,)).astype(dtype).copy()


def decoded_weights(data):
    """What the library reads from serialized (raw or gzip) pblczero.Net bytes, without a GPU:
    (format dict, {tensor name: float32 array}); heads resolved, batch norm folded."""
    lib = load_library()
    data = bytes(data)
    need = lib.lc0mi_weights_list(data, len(data), None, 0)
    if need < 0:
        raise BackendError(lib.lc0mi_last_error().decode(errors="replace"))
    buf = C.create_string_buffer(need)
    lib.lc0mi_weights_list(data, len(data), buf, need)
    lines = buf.value.decode().splitlines()
    fmt = {k: int(v) for k, v in (kv.split("=") for kv in lines[0].split()[1:])}
    tensors = {}
    for line in lines[1:]:
        name, count = line.split()
        arr = np.zeros(int(count), np.float32)
        got = lib.lc0mi_weights_tensor(data, len(data), name.encode(), arr.ctypes.data, arr.size)
        if got != arr.size:
            raise BackendError("tensor %s: expected %d elements, got %d" % (name, arr.size, got))
        tensors[name] = arr
    return fmt, tensors


def attn_policy_map():
    return _table("lc0mi_attn_policy_map", np.int16)


def conv_policy_map():
    return _table("lc0mi_conv_policy_map", np.int16)


def pos_encoding():
    return _table("lc0mi_pos_encoding", np.float32).reshape(64, 64)


class Network:
    """lczero::Network built by the mi355x factory from a weights file or buffer."""

    def __init__(self, weights, options=""):
        lib = load_library()
        self._h = C.c_void_p()
        opts = options.encode() if isinstance(options, str) else options
        if isinstance(weights, (bytes, bytearray, memoryview)):
            buf = bytes(weights)
            _check(lib.lc0mi_net_create_from_buffer(buf, len(buf), opts, C.byref(self._h)))
        else:
            _check(lib.lc0mi_net_create_from_file(os.fspath(weights).encode(), opts, C.byref(self._h)))

    def close(self):
        if getattr(self, "_h", None):
            load_library().lc0mi_net_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def GetCapabilities(self):
        a, b, c = C.c_int(), C.c_int(), C.c_int()
        _check(load_library().lc0mi_net_caps(self._h, C.byref(a), C.byref(b), C.byref(c)))
        return NetworkCapabilities(a.value, b.value, c.value)

    def _hints(self):
        v = [C.c_int() for _ in range(5)]
        _check(load_library().lc0mi_net_hints(self._h, *[C.byref(x) for x in v]))
        return [x.value for x in v]

    def GetMiniBatchSize(self):
        return self._hints()[0]

    def GetPreferredBatchStep(self):
        return self._hints()[1]

    def GetMaxBatchSize(self):
        return self._hints()[2]

    def GetThreads(self):
        return self._hints()[3]

    def IsCpu(self):
        return bool(self._hints()[4])

    def NewComputation(self):
        return NetworkComputation(self)

    # measurement hooks
    def SetProfiling(self, on):
        _check(load_library().lc0mi_net_set_profiling(self._h, int(bool(on))))

    def TakeProfile(self):
        lib = load_library()
        buf = C.create_string_buffer(1 << 16)
        lib.lc0mi_net_take_profile(self._h, buf, len(buf))
        out = []
        for line in buf.value.decode().splitlines():
            name, ms, n, fl, by = line.split()
            out.append(KernelTime(name, float(ms), int(n), float(fl), float(by)))
        return out

    def CalibrateFp8(self, masks, values):
        """precision=fp8: activation scales from these positions (uint64 [n,112], float32 [n,112])."""
        import numpy as np
        masks = np.ascontiguousarray(masks, np.uint64)
        values = np.ascontiguousarray(values, np.float32)
        if masks.shape != values.shape or masks.ndim != 2 or masks.shape[1] != 112:
            raise BackendError("masks and values must both be [n, 112]")
        _check(load_library().lc0mi_net_calibrate_fp8(self._h, masks.shape[0], masks.ctypes.data, values.ctypes.data))

    def Fp8Scales(self):
        """precision=fp8: float32 [layers, 7], the activation scales of the operands of Q/K/V, attention output,
        FFN1, FFN2 and of smolgen's first dense, second dense and generator layers (1 where unused)."""
        import numpy as np
        lib = load_library()
        n = lib.lc0mi_net_fp8_scales(self._h, None, 0)
        if n < 0:
            raise BackendError(lib.lc0mi_last_error().decode())
        out = np.zeros(n, np.float32)
        lib.lc0mi_net_fp8_scales(self._h, out.ctypes.data, n)
        return out.reshape(-1, 7)

    def TimeResidentForward(self, batch, iters):
        ms = C.c_double()
        _check(load_library().lc0mi_net_time_resident_forward(self._h, batch, iters, C.byref(ms)))
        return ms.value


class NetworkComputation:
    """lczero::NetworkComputation: fill with AddInput, ComputeBlocking, read."""

    def __init__(self, network):
        self._net = network  # keeps the network alive
        self._h = C.c_void_p()
        _check(load_library().lc0mi_comp_create(network._h, C.byref(self._h)))

    def close(self):
        if getattr(self, "_h", None):
            load_library().lc0mi_comp_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def AddInput(self, planes):
        """planes: sequence of 112 InputPlane(mask, value)."""
        if len(planes) != 112:
            raise BackendError("AddInput expects exactly 112 input planes, got %d." % len(planes))
        masks = np.array([p[0] for p in planes], dtype=np.uint64)
        values = np.array([p[1] for p in planes], dtype=np.float32)
        _check(load_library().lc0mi_comp_add_input(self._h, masks.ctypes.data, values.ctypes.data))

    def AddInputs(self, masks, values):
        """Bulk AddInput: masks u64[n,112], values f32[n,112]."""
        masks = np.ascontiguousarray(masks, dtype=np.uint64)
        values = np.ascontiguousarray(values, dtype=np.float32)
        if masks.ndim != 2 or masks.shape[1] != 112 or values.shape != masks.shape:
            raise BackendError("AddInputs expects [n,112] masks and values.")
        _check(load_library().lc0mi_comp_add_inputs(self._h, masks.shape[0], masks.ctypes.data,
                                                    values.ctypes.data))

    def ComputeBlocking(self):
        _check(load_library().lc0mi_comp_compute_blocking(self._h))

    def GetBatchSize(self):
        return load_library().lc0mi_comp_batch_size(self._h)

    def _get(self, fn, *args):
        v = fn(self._h, *args)
        if v != v:  # NaN marks an error
            raise BackendError(load_library().lc0mi_last_error().decode(errors="replace"))
        return v

    def GetQVal(self, sample):
        return self._get(load_library().lc0mi_comp_q, sample)

    def GetDVal(self, sample):
        return self._get(load_library().lc0mi_comp_d, sample)

    def GetMVal(self, sample):
        return self._get(load_library().lc0mi_comp_m, sample)

    def GetPVal(self, sample, move_id):
        return self._get(load_library().lc0mi_comp_p, sample, move_id)

    def GetPolicyRow(self, sample):
        ptr = load_library().lc0mi_comp_policy_row(self._h, sample)
        if not ptr:
            raise BackendError(load_library().lc0mi_last_error().decode(errors="replace"))
        return np.ctypeslib.as_array(ptr, (1858,)).copy()

    def AddLegalMoves(self, move_ids):
        """Policy indices (0..1857) of the legal moves of the input added last. Once used, every input
        needs its list; the policy then comes from GetLegalPolicy (softmax over these moves, computed on
        the device as lc0's search wrapper does on the host) and the raw logits are not downloaded."""
        ids = np.ascontiguousarray(move_ids, dtype=np.uint16)
        if ids.ndim != 1:
            raise BackendError("AddLegalMoves expects a one-dimensional list of move ids.")
        _check(load_library().lc0mi_comp_add_legal_moves(self._h, ids.shape[0], ids.ctypes.data))

    def SetPolicySoftmaxTemperature(self, temperature):
        _check(load_library().lc0mi_comp_set_policy_softmax_temperature(self._h, float(temperature)))

    def GetLegalPolicy(self, sample):
        n = C.c_int(0)
        ptr = load_library().lc0mi_comp_legal_policy(self._h, sample, C.byref(n))
        if not ptr:
            raise BackendError(load_library().lc0mi_last_error().decode(errors="replace"))
        if n.value == 0:
            return np.zeros(0, np.float32)
        return np.ctypeslib.as_array(ptr, (n.value,)).copy()

    def results(self):
        """All outputs as arrays: dict(policy [n,1858], q [n], d [n], m [n])."""
        n = self.GetBatchSize()
        return dict(policy=np.stack([self.GetPolicyRow(i) for i in range(n)]) if n else np.zeros((0, 1858), np.float32),
                    q=np.array([self.GetQVal(i) for i in range(n)], np.float32),
                    d=np.array([self.GetDVal(i) for i in range(n)], np.float32),
                    m=np.array([self.GetMVal(i) for i in range(n)], np.float32))
