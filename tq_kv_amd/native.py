"""Python face of the engine library (csrc/tq_engine.h; csrc/host_engine.cpp and csrc/engine/*.cpp):
configuration, weights, models, the cache, the step function, sampling and the generation loop
live behind C handles; the classes of this package hold a handle and turn status codes into
exceptions.  The library is host code only and is built with the host compiler at first use; it
reaches the GPU through the HIP runtime and the kernel library beside it."""
import ctypes
import json

import numpy as np

from .csrc import build as _build

_LIB = None
(OK, ERR_ARGUMENT, ERR_FULL, ERR_STATE, ERR_RANGE, ERR_STEP, ERR_CONFIG, ERR_WEIGHTS, ERR_WEIGHT_FILE, ERR_DEVICE, ERR_KERNEL,
 ERR_GENERATION, ERR_PART) = 0, -1, -2, -3, -4, -5, -6, -7, -8, -9, -10, -11, -12
NO_LIST = -100
MAX_GROUPS = 16
META_SIZE = 12 + 12 + 2 * MAX_GROUPS
(META_TOTAL, META_TOKENS, META_WANT, META_LAST, META_ALL_DECODE, META_PRUNE_LAST, META_MAX_NEW, META_MAX_END,
 META_GROUPS) = range(9)
META_OFFSETS = 12
META_WIDTHS = META_OFFSETS + 12 + MAX_GROUPS
F32, BF16, I32 = 0, 1, 2
STEP_ARRAYS = ("tokens", "tok_seq", "tok_pos", "seq_slot", "seq_start", "seq_new", "cu", "want_rows", "last_rows", "want_in_last",
               "last_seq", "last_pos")
_I32P = ctypes.POINTER(ctypes.c_int32)


# ---- exceptions: one per kind of status ---------------------------------------------------------------
class EngineLibraryError(RuntimeError, ValueError):
    """A bad argument, or anything else the library refuses."""


class StepError(ValueError):
    """A step the engine cannot run (no sequence, a slot twice, an empty prompt, a token outside
    the vocabulary, more positions than the model has)."""


class CacheFull(RuntimeError):
    """No free slot, or not enough free pages; nothing was changed."""


class ConfigError(ValueError):
    """A config.json that cannot be used: missing key, wrong type, bad combination."""


class WeightFileError(ValueError):
    """A folder or safetensors file that cannot be read."""


class WeightError(ValueError):
    """Missing tensors, unexpected tensors or wrong shapes; lists all of them."""

    def __init__(self, message, detail=None):
        super().__init__(message)
        detail = detail or {}
        self.missing = list(detail.get("missing", []))
        self.unexpected = list(detail.get("unexpected", []))
        self.wrong_shape = [(n, tuple(got), tuple(want)) for n, got, want in detail.get("wrong_shape", [])]
        self.wrong_kind = [tuple(e) for e in detail.get("wrong_kind", [])]


class GenerationError(ValueError):
    """Requests the loop cannot serve."""


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments, or the kernel library is missing."""


class DeviceError(RuntimeError):
    """The GPU runtime or a library on it failed."""


class PartError(RuntimeError):
    """A part registered from Python failed (its own exception is the cause)."""


class tqe_tensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("dtype", ctypes.c_int32), ("ndim", ctypes.c_int32), ("shape", ctypes.c_int64 * 6),
                ("row_stride", ctypes.c_int64)]


class tqe_step_view(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("n_seqs", "n_tokens", "n_want", "n_last", "all_decode", "prune_last", "max_new", "max_end",
                                              "act_dtype", "n_groups")] + [
        ("host", _I32P * 12), ("dev", ctypes.c_void_p * 12), ("sizes", ctypes.c_int32 * 12),
        ("table_host", _I32P * MAX_GROUPS), ("table_dev", ctypes.c_void_p * MAX_GROUPS), ("table_width", ctypes.c_int32 * MAX_GROUPS),
        ("entry_group", ctypes.c_int32), ("entry_writes", ctypes.c_int32), ("entry_window", ctypes.c_int32), ("last_rows_only", ctypes.c_int32),
        ("stream", ctypes.c_void_p)]


class tqe_generation_params(ctypes.Structure):
    _fields_ = [("max_tokens", ctypes.c_int32), ("temperature", ctypes.c_float), ("top_p", ctypes.c_float), ("top_k", ctypes.c_int32),
                ("repeat_penalty", ctypes.c_float), ("seed", ctypes.c_uint64)]


PART_CREATE = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int,
                               ctypes.POINTER(ctypes.c_void_p))
PART_DESTROY = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_void_p)
PART_DESCRIBE = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p)       # returns the address of a C string
PART_LOAD = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_char_p),
                             ctypes.POINTER(tqe_tensor))
PART_CALL = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p, ctypes.POINTER(tqe_step_view), ctypes.c_int,
                             ctypes.POINTER(tqe_tensor))
PART_ERROR = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_void_p)


class tqe_part_callbacks(ctypes.Structure):
    _fields_ = [("create", PART_CREATE), ("destroy", PART_DESTROY), ("describe", PART_DESCRIBE), ("load", PART_LOAD), ("call", PART_CALL),
                ("last_error", PART_ERROR)]


ON_TOKENS = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_int, _I32P, _I32P)
LOOP_OPEN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, _I32P)
LOOP_CLOSE = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_int)
LOOP_STEP = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_int, _I32P, _I32P, _I32P, _I32P)
LOOP_BATCH = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_int, _I32P)
LOOP_SAMPLE = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_int, _I32P, _I32P)
LOOP_DRAW = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_int, _I32P, _I32P)
LOOP_AHEAD = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_int, _I32P, ctypes.c_int, _I32P)
LOOP_READ = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, _I32P)
INIT_FILL = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_uint64, ctypes.c_int64, ctypes.c_int64,
                             ctypes.POINTER(ctypes.c_float))
TRACE_PUSH = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_char_p)
TRACE_POP = ctypes.CFUNCTYPE(ctypes.c_int)


class tqe_loop_callbacks(ctypes.Structure):
    _fields_ = [("open", LOOP_OPEN), ("close", LOOP_CLOSE), ("step", LOOP_STEP), ("new_batch", LOOP_BATCH), ("sample", LOOP_SAMPLE),
                ("last_error", PART_ERROR), ("max_tokens", ctypes.c_longlong), ("max_positions", ctypes.c_longlong),
                ("max_slots", ctypes.c_int32), ("holds_pages", ctypes.c_int32), ("draw", LOOP_DRAW), ("step_ahead", LOOP_AHEAD),
                ("read", LOOP_READ)]


_KERNEL_BUILDER_TYPE = ctypes.CFUNCTYPE(ctypes.c_void_p)
_KERNEL_PATH = None


def _build_kernels():
    """What the engine library calls when it needs the kernel library and finds none: compile it (progress lines on
    standard error) and say where it is."""
    global _KERNEL_PATH
    try:
        _KERNEL_PATH = CString(_build.ensure_built())
        return _KERNEL_PATH.address
    except BaseException as e:          # nothing may escape into the library; the caller sees it once the library has returned
        _pending_exception.append(e)
        return None


_KERNEL_BUILDER = _KERNEL_BUILDER_TYPE(_build_kernels)


def library():
    global _LIB
    if _LIB is None:
        path = _build.ensure_host_built()
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise EngineLibraryError("cannot load the engine library %s: %s" % (path, e))
        P, I, L, S = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong, ctypes.c_char_p
        U64, I64 = ctypes.c_uint64, ctypes.c_int64
        T = ctypes.POINTER(tqe_tensor)
        text = ("tqe_last_error", "tqe_last_error_detail", "tqe_last_warning", "tqe_kernel_library", "tqe_known_architectures")
        for name in text:
            getattr(lib, name).restype = S
            getattr(lib, name).argtypes = []
        for name, args in (("tqe_known_parts", [S]), ("tqe_config_parse", [S]), ("tqe_config_spec", [S]), ("tqe_read_config", [S]),
                           ("tqe_stop_token_ids", [S]), ("tqe_model_describe", [P]), ("tqe_folder_describe", [P]), ("tqe_part_describe", [P]),
                           ("tqe_store_describe", [P]), ("tqe_engine_describe", [P])):
            getattr(lib, name).restype = S
            getattr(lib, name).argtypes = args
        for name, args in (("tqe_cache_new", [I, I, _I32P, _I32P]), ("tqe_batch_new", [I, I, _I32P, I]),
                           ("tqe_model_load", [S, I, I, I]), ("tqe_model_random", [S, U64, I, I]), ("tqe_model_new", [S, I, I]),
                           ("tqe_model_from_spec", [S, I, I]), ("tqe_folder_open", [S]), ("tqe_part_new", [S, S, I, I]),
                           ("tqe_store_new", [S, _I32P, I, L, I, I, I]), ("tqe_store_cache", [P]),
                           ("tqe_stepctx_new", [P, I, _I32P, _I32P, _I32P, _I32P, _I32P, I, P]), ("tqe_engine_new", [P, L, I, I]),
                           ("tqe_engine_cache", [P]), ("tqe_sampler_new", [ctypes.POINTER(tqe_generation_params), I, _I32P, I, P])):
            getattr(lib, name).restype = P
            getattr(lib, name).argtypes = args
        for name in ("tqe_cache_free", "tqe_batch_free", "tqe_model_free", "tqe_folder_free", "tqe_part_free", "tqe_store_free",
                     "tqe_stepctx_free", "tqe_engine_free", "tqe_sampler_free"):
            getattr(lib, name).restype = None
            getattr(lib, name).argtypes = [P]
        for name, args in (
                ("tqe_abi_version", []), ("tqe_page_size", []),
                ("tqe_cache_acquire", [P, _I32P]), ("tqe_cache_release", [P, I]), ("tqe_cache_length", [P, I]), ("tqe_cache_is_held", [P, I]),
                ("tqe_cache_counts", [P, I, _I32P, _I32P]), ("tqe_cache_reserve", [P, I, _I32P, _I32P]),
                ("tqe_cache_commit", [P, I, _I32P, _I32P]), ("tqe_cache_trim", [P, I, _I32P]), ("tqe_cache_pages", [P, I, I, _I32P, I]),
                ("tqe_cache_check", [P]), ("tqe_check_step", [P, I, _I32P, _I32P, _I32P, I, I]),
                ("tqe_plan_step", [P, I, _I32P, _I32P, _I32P, _I32P, _I32P, _I32P, I, _I32P, I, _I32P]),
                ("tqe_plan_batches", [I, _I32P, I, L, I, I, _I32P]), ("tqe_prompt_steps", [I, _I32P, I, _I32P, I]),
                ("tqe_batch_accept", [P, I, I]), ("tqe_batch_goes_on", [P, I]), ("tqe_batch_emitted", [P, I]), ("tqe_batch_ended", [P, I]),
                ("tqe_set_kernel_library", [S]), ("tqe_policy_set", [S, I]), ("tqe_policy_get", [S]), ("tqe_trace_enable", [I]),
                ("tqe_trace_enabled", []), ("tqe_register_part", [S, S, ctypes.POINTER(tqe_part_callbacks), P]),
                ("tqe_register_init", [S, INIT_FILL, P]),
                ("tqe_model_set_tensor", [P, S, T, I, P]), ("tqe_model_finish", [P, I, P]), ("tqe_model_randomize", [P, U64, P]),
                ("tqe_model_tensor", [P, S, T]), ("tqe_model_tune_library", [P, I, P]), ("tqe_model_set_stop_tokens", [P, I, _I32P]),
                ("tqe_write_random_folder", [S, S, U64, I]), ("tqe_random_stream", [U64, S, I64, I64, ctypes.POINTER(ctypes.c_float)]),
                ("tqe_random_stream_of_key", [U64, I64, I64, ctypes.POINTER(ctypes.c_float)]), ("tqe_check_weights", [P, S, I]), ("tqe_write_safetensors", [S, S, ctypes.POINTER(P), S]),
                ("tqe_part_set_tensor", [P, S, T, I, P]), ("tqe_part_finish", [P, P]), ("tqe_part_tensor", [P, S, T]),
                ("tqe_part_call", [P, S, P, P, I, I, T, P]), ("tqe_store_acquire", [P, _I32P, P]),
                ("tqe_stepctx_view", [P, ctypes.POINTER(tqe_step_view)]),
                ("tqe_engine_open", [P, _I32P, P]), ("tqe_engine_close", [P, I]),
                ("tqe_step", [P, I, _I32P, _I32P, _I32P, _I32P, _I32P, P, P, I, ctypes.POINTER(P), P]),
                ("tqe_generate", [P, I, _I32P, _I32P, ctypes.POINTER(tqe_generation_params), _I32P, I, I, I, ON_TOKENS, P, _I32P, _I32P, P]),
                ("tqe_generate_with", [ctypes.POINTER(tqe_loop_callbacks), P, I, _I32P, _I32P, ctypes.POINTER(tqe_generation_params), _I32P, I, I,
                                       I, ON_TOKENS, P, _I32P, _I32P]),
                ("tqe_sampler_sample", [P, P, I, _I32P, _I32P])):
            getattr(lib, name).restype = I
            getattr(lib, name).argtypes = args
        lib.tqe_tensor_key.restype = U64
        lib.tqe_tensor_key.argtypes = [U64, S]
        lib.tqe_draw_uniform.restype = ctypes.c_float
        lib.tqe_draw_uniform.argtypes = [U64, U64, U64]
        lib.tqe_generation_defaults.restype = None
        lib.tqe_generation_defaults.argtypes = [ctypes.POINTER(tqe_generation_params)]
        lib.tqe_trace_sink.restype = None
        lib.tqe_trace_sink.argtypes = [TRACE_PUSH, TRACE_POP]
        lib.tqe_trace_push.restype = None
        lib.tqe_trace_push.argtypes = [S]
        lib.tqe_trace_pop.restype = None
        lib.tqe_trace_pop.argtypes = []
        lib.tqe_set_kernel_builder.restype = None
        lib.tqe_set_kernel_builder.argtypes = [_KERNEL_BUILDER_TYPE]
        lib.tqe_set_kernel_builder(_KERNEL_BUILDER)
        _LIB = lib
    return _LIB


def library_path():
    library()
    return _LIB._name


def _message():
    return library().tqe_last_error().decode("utf-8", "replace")


_pending_exception = []          # a Python exception raised inside a callback, to be raised again once the library has returned


def _raise(status):
    """The exception of a status code."""
    if _pending_exception:
        exc = _pending_exception.pop()
        del _pending_exception[:]
        raise exc
    msg = _message()
    if status == ERR_FULL:
        raise CacheFull(msg)
    if status == ERR_STATE:
        raise AssertionError(msg)
    if status == ERR_RANGE:
        raise IndexError(msg)
    if status == ERR_STEP:
        raise StepError(msg)
    if status == ERR_CONFIG:
        raise ConfigError(msg)
    if status == ERR_WEIGHTS:
        detail = library().tqe_last_error_detail().decode("utf-8", "replace")
        raise WeightError(msg, json.loads(detail) if detail else None)
    if status == ERR_WEIGHT_FILE:
        raise WeightFileError(msg)
    if status == ERR_GENERATION:
        raise GenerationError(msg)
    if status == ERR_KERNEL:
        raise KernelError(msg)
    if status == ERR_DEVICE:
        raise DeviceError(msg)
    if status == ERR_PART:
        raise PartError(msg)
    raise EngineLibraryError(msg)


def check(status):
    if status != OK:
        _raise(status)


def handle(value):
    """A handle the library made, or the exception of why it did not."""
    if not value:
        _raise(library().tqe_last_status())
    return value


def text(value):
    """A string the library returned (JSON as a rule), or the exception of why it did not."""
    if value is None:
        _raise(library().tqe_last_status())
    return value.decode("utf-8", "replace")


def parsed(value):
    return json.loads(text(value))


def warn_if_any():
    """Passes on a warning the last model call left (tensors a folder holds that the model does not use)."""
    w = library().tqe_last_warning()
    if w:
        import warnings
        warnings.warn(w.decode("utf-8", "replace"))


def _ptr(a):
    return a.ctypes.data_as(_I32P) if a is not None else None


def _i32(values):
    return np.ascontiguousarray(values, dtype=np.int32)


def enc(s):
    return s.encode("utf-8") if isinstance(s, str) else s


class CString:
    """A C string a callback can return the address of; it lives as long as this object does."""

    def __init__(self, text=b""):
        self.set(text)

    def set(self, text):
        self.buf = ctypes.create_string_buffer(enc(text))
        return self.address

    @property
    def address(self):
        return ctypes.addressof(self.buf)


def page_size():
    return int(library().tqe_page_size())


# ---- tensors across the boundary ---------------------------------------------------------------------
def _torch():
    import torch
    return torch


def dtype_code(dtype):
    torch = _torch()
    if dtype in (torch.float32, "float32", "fp32"):
        return F32
    if dtype in (torch.bfloat16, "bfloat16", "bf16"):
        return BF16
    if dtype in (torch.int32, "int32"):
        return I32
    raise ValueError("dtype must be bfloat16, float32 or int32, got %r" % (dtype,))


def torch_dtype(code):
    torch = _torch()
    return {F32: torch.float32, BF16: torch.bfloat16, I32: torch.int32}[int(code)]


def c_tensor(t, row_stride=0):
    """The library's view of a torch tensor (contiguous, float32 / bfloat16 / int32, at most 6 dimensions), or of None."""
    out = tqe_tensor()
    if t is None:
        return out
    if not t.is_contiguous():
        raise ValueError("a tensor handed to the engine must be contiguous")
    if t.dim() > 6:
        raise ValueError("a tensor handed to the engine has at most 6 dimensions, got %d" % t.dim())
    out.data = t.data_ptr()
    out.dtype = dtype_code(t.dtype)
    out.ndim = t.dim()
    for i, s in enumerate(t.shape):
        out.shape[i] = int(s)
    out.row_stride = row_stride
    return out


class _Memory:
    """Device memory of the library's, for torch to view (the CUDA array interface)."""

    def __init__(self, ptr, shape, strides, typestr):
        self.__cuda_array_interface__ = {"shape": tuple(shape), "typestr": typestr, "data": (int(ptr), False), "version": 2, "strides": strides}


def view(ptr, dtype, shape, on_gpu=True, row_stride=0, keep=None):
    """A torch tensor over memory the library owns (no copy).  keep: an object that must outlive the view."""
    torch = _torch()
    shape = tuple(int(s) for s in shape)
    dt = torch_dtype(dtype) if not isinstance(dtype, torch.dtype) else dtype
    numel = 1
    for s in shape:
        numel *= s
    if numel == 0 or not ptr:
        return torch.empty(shape, dtype=dt, device="cuda" if on_gpu else "cpu")
    item = 2 if dt == torch.bfloat16 else 4
    strides = None
    if row_stride and len(shape) > 1:
        # strides in bytes: the first dimension row_stride values apart, the others packed
        packed = [1] * len(shape)
        for i in range(len(shape) - 2, -1, -1):
            packed[i] = packed[i + 1] * shape[i + 1]
        packed[0] = row_stride
        strides = tuple(x * item for x in packed)
    if on_gpu:
        typestr = "<i2" if dt == torch.bfloat16 else ("<f4" if dt == torch.float32 else "<i4")
        t = torch.as_tensor(_Memory(ptr, shape, strides, typestr), device="cuda")
        if dt == torch.bfloat16:
            t = t.view(torch.bfloat16)
    else:
        span = numel if strides is None else (shape[0] - 1) * row_stride + numel // shape[0]
        buf = (ctypes.c_char * (span * item)).from_address(int(ptr))
        flat = torch.frombuffer(buf, dtype=dt, count=span)
        t = flat.reshape(shape) if strides is None else flat.as_strided(shape, [x // item for x in strides])
    if keep is not None:
        t._tq_keep = keep
    return t


def view_of(ct, on_gpu=True, keep=None):
    """view() of a tqe_tensor the library filled in; None for an absent one."""
    if not ct.data:
        return None
    return view(ct.data, ct.dtype, [ct.shape[i] for i in range(ct.ndim)], on_gpu, int(ct.row_stride), keep)


def current_stream():
    """The stream torch is working on (what every call into the engine is ordered on), or None without a GPU."""
    torch = _torch()
    if not torch.cuda.is_available():
        return None
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


# ---- the bookkeeping of a cache ----------------------------------------------------------------------
class NativeCache:
    """A tqe_cache_t: max_slots slots, one page pool per group (pages, window or 0).  handle: one the
    library already has (an engine's or a store's), which is then not freed here."""

    def __init__(self, max_slots, groups, handle=None):
        self._lib = library()
        self.n_groups = len(groups)
        self.max_slots = int(max_slots)
        self._owned = handle is None
        if handle is None:
            pages = _i32([p for p, _ in groups])
            windows = _i32([w or 0 for _, w in groups])
            handle = self._lib.tqe_cache_new(self.max_slots, self.n_groups, _ptr(pages), _ptr(windows))
            if not handle:
                _raise(self._lib.tqe_last_status())
        self.handle = handle

    def __del__(self):
        handle, self.handle = getattr(self, "handle", None), None
        if handle and getattr(self, "_owned", False) and self._lib is not None:
            self._lib.tqe_cache_free(handle)

    def acquire(self):
        slot = ctypes.c_int32(-1)
        status = self._lib.tqe_cache_acquire(self.handle, ctypes.byref(slot))
        if status != OK:
            _raise(status)
        return slot.value

    def release(self, slot):
        status = self._lib.tqe_cache_release(self.handle, int(slot))
        if status != OK:
            _raise(status)

    def length(self, slot):
        n = self._lib.tqe_cache_length(self.handle, int(slot))
        if n < 0:
            _raise(n)
        return n

    def is_held(self, slot):
        return bool(self._lib.tqe_cache_is_held(self.handle, int(slot)))

    def counts(self, group):
        """(free, total) slots (group -1) or pages of a group."""
        free, total = ctypes.c_int32(0), ctypes.c_int32(0)
        status = self._lib.tqe_cache_counts(self.handle, int(group), ctypes.byref(free), ctypes.byref(total))
        if status != OK:
            _raise(status)
        return free.value, total.value

    def _items(self, items):
        return _i32([s for s, _ in items]), _i32([n for _, n in items])

    def reserve(self, items):
        slots, counts = self._items(items)
        status = self._lib.tqe_cache_reserve(self.handle, len(items), _ptr(slots), _ptr(counts))
        if status != OK:
            _raise(status)

    def commit(self, items):
        slots, counts = self._items(items)
        status = self._lib.tqe_cache_commit(self.handle, len(items), _ptr(slots), _ptr(counts))
        if status != OK:
            _raise(status)

    def trim(self, slots):
        """Give back what was reserved for these slots and never committed."""
        slots = _i32(list(slots))
        status = self._lib.tqe_cache_trim(self.handle, len(slots), _ptr(slots))
        if status != OK:
            _raise(status)

    def pages(self, group, slot):
        """The slot's page list in the group (-1 where given back), or None if it has none."""
        n = self._lib.tqe_cache_pages(self.handle, int(group), int(slot), None, 0)
        if n == NO_LIST:
            return None
        if n < 0:
            _raise(n)
        out = np.empty(max(n, 1), dtype=np.int32)
        self._lib.tqe_cache_pages(self.handle, int(group), int(slot), _ptr(out), n)
        return out[:n].tolist()

    def check(self):
        status = self._lib.tqe_cache_check(self.handle)
        if status != OK:
            _raise(status)

    def check_step(self, slots, n_new, tokens, vocab_size, max_positions):
        """Raises StepError unless the step can run (tqe_check_step).  tokens: int32 array of all the
        step's tokens, or None where the host does not know them."""
        status = self._lib.tqe_check_step(self.handle, len(slots), _ptr(slots), _ptr(n_new), _ptr(tokens), int(vocab_size), int(max_positions))
        if status != OK:
            _raise(status)


def plan_step(cache, slots, starts, n_new, tokens, want_counts, want_idx, width_step, out=None):
    """The packed arrays of one step (tqe_plan_step).  cache: a NativeCache or None (then starts
    must be given).  out: an int32 numpy array to fill (grown copies are the caller's business), or
    None for a new one.  Returns (packed array, meta array)."""
    lib = library()
    handle = cache.handle if cache is not None else None
    n = len(slots)
    meta = np.zeros(META_SIZE, dtype=np.int32)
    args = (handle, n, _ptr(slots), _ptr(starts), _ptr(n_new), _ptr(tokens), _ptr(want_counts), _ptr(want_idx), int(width_step))
    if out is None:
        status = lib.tqe_plan_step(*args, None, 0, _ptr(meta))
        if status != OK:
            _raise(status)
        out = np.empty(int(meta[META_TOTAL]), dtype=np.int32)
    status = lib.tqe_plan_step(*args, _ptr(out), out.shape[0], _ptr(meta))
    if status != OK:
        _raise(status)
    return out[:int(meta[META_TOTAL])], meta


# ---- the generation loop's decisions ----------------------------------------------------------
TOKEN_FEED, TOKEN_LAST, TOKEN_STOP, TOKEN_DROPPED = 0, 1, 2, 3


def plan_batches(prompt_lens, max_new, max_tokens, max_batch, holds_pages=True):
    """tqe_plan_batches: lists of request indices, one list per batch.  CacheFull where one request
    alone does not fit."""
    lens = np.ascontiguousarray(prompt_lens, dtype=np.int32)
    batch_of = np.zeros(len(lens), dtype=np.int32)
    n = library().tqe_plan_batches(len(lens), _ptr(lens), int(max_new), int(max_tokens), int(max_batch), 1 if holds_pages else 0,
                                   _ptr(batch_of))
    if n < 0:
        _raise(n)
    batches = [[] for _ in range(n)]
    for i, b in enumerate(batch_of.tolist()):
        batches[b].append(i)
    return batches


def prompt_steps(lens, max_step_tokens):
    """tqe_prompt_steps: steps, each a list of (prompt, begin, end)."""
    lens = np.ascontiguousarray(lens, dtype=np.int32)
    n = library().tqe_prompt_steps(len(lens), _ptr(lens), int(max_step_tokens), None, 0)
    if n < 0:
        _raise(n)
    pieces = np.zeros((max(n, 1), 4), dtype=np.int32)
    n = library().tqe_prompt_steps(len(lens), _ptr(lens), int(max_step_tokens), _ptr(pieces), len(pieces))
    if n < 0:
        _raise(n)
    steps = []
    for i, begin, end, step in pieces[:n].tolist():
        while len(steps) <= step:
            steps.append([])
        steps[step].append((i, begin, end))
    return steps


class BatchProgress:
    """tqe_batch_t: how many tokens each request of a batch has emitted, which have ended, and
    what becomes of a drawn token."""

    def __init__(self, n_requests, max_new, stop_ids):
        # a stop id is a token id: nothing negative, nothing beyond the library's int32
        stop = np.ascontiguousarray(sorted(set(int(t) for t in stop_ids if 0 <= int(t) < 2 ** 31)), dtype=np.int32)
        self._lib = library()
        self.handle = self._lib.tqe_batch_new(int(n_requests), int(max_new), _ptr(stop) if len(stop) else None, len(stop))
        if not self.handle:
            _raise(self._lib.tqe_last_status())

    def __del__(self):
        if getattr(self, "handle", None):
            self._lib.tqe_batch_free(self.handle)
            self.handle = None

    def accept(self, row, token):
        token = int(token)
        if not -2 ** 31 <= token < 2 ** 31:
            token = -1                       # no stop id is negative
        status = self._lib.tqe_batch_accept(self.handle, int(row), token)
        if status < 0:
            _raise(status)
        return status

    def goes_on(self, row):
        return bool(self._lib.tqe_batch_goes_on(self.handle, int(row)))

    def emitted(self, row):
        n = self._lib.tqe_batch_emitted(self.handle, int(row))
        if n < 0:
            _raise(n)
        return n

    def ended(self, row):
        return bool(self._lib.tqe_batch_ended(self.handle, int(row)))
