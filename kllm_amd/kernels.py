"""Python side of the kernel library: loads ``libkllm_hip.so`` and wraps each
entry point so that it takes torch tensors.

There is no fallback: if the library cannot be found, built or loaded, the
first call raises.  Every wrapper checks device, dtype and contiguity of its
tensors (the library itself checks the sizes) and launches on torch's current
stream, so the launches order with torch's own work and are recorded by a HIP
graph capture.
"""

from __future__ import annotations

import ctypes
import functools
import struct
import threading
from ctypes import c_char_p, c_double, c_float, c_int, c_long, c_void_p

import torch

DT_F32, DT_BF16 = 0, 1
GEMM_PLAIN, GEMM_TILED_F32, GEMM_MFMA_BF16, GEMM_SKINNY_BF16, GEMM_GEMV, GEMM_GEMV_LDS, GEMM_MFMA_F32 = 0, 1, 2, 3, 4, 5, 6
GEMV_BEST_ROWS = 0         # rows up to which they beat the MFMA kernels in bfloat16: none (a step at 1.1B sizes, one token: 1.036 against 0.963 ms)
ABI_VERSION = 8


class KernelError(RuntimeError):
    """The kernel library refused a call or a launch failed."""


_lib = None
_lib_path = None
_lock = threading.Lock()


def limit(name: str) -> int:
    """A size limit of the kernels, asked of the library (so that the host's choice of a
    kernel and the kernel's own checks cannot drift apart): ``gemv_max_rows``,
    ``gemv_normed_max_rows``, ``gemv_normed_max_parts``, ``fused_linear_max_parts``."""
    v = _limits.get(name)
    if v is None:
        v = _limits[name] = int(getattr(library(), "kllm_" + name)())
    return v


_limits = {}


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return DT_F32
    if dtype == torch.bfloat16:
        return DT_BF16
    raise KernelError(f"dtype {dtype} is not a storage type of the kernels")


def library():
    """The loaded library; builds it on the first call if nothing is built."""
    global _lib, _lib_path
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        import os
        path = os.environ.get("KLLM_AMD_LIBRARY")
        if not path:
            from .csrc.build import ensure_built
            path = ensure_built()
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load the kernel library {path}: {e}") from None
        lib.kllm_abi_version.restype = c_int
        if lib.kllm_abi_version() != ABI_VERSION:
            raise KernelError(
                f"{path} has ABI version {lib.kllm_abi_version()}, this package needs "
                f"{ABI_VERSION}: rebuild it (python -m kllm_amd.csrc.build)")
        _declare(lib)
        _lib, _lib_path = lib, path
    return _lib


def library_path():
    library()
    return _lib_path


def _declare(lib):
    P, I, L, F, D = c_void_p, c_int, c_long, c_float, c_double
    sigs = {
        "kllm_last_error": [c_char_p, I],
        "kllm_device_info": [I, c_char_p, I],
        "kllm_embed": [P, P, P, P, P, I, I, I, I, P],
        "kllm_add_rmsnorm": [P, P, I, I, L, P, P, I, P, I, I, F, I, P],
        "kllm_rope_tables": [P, P, P, I, I, D, P],
        "kllm_rope_append": [P, I, I, L, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, I, P],
        "kllm_silu_mul": [P, I, I, L, P, I, I, I, I, P],
        "kllm_gemm": [P, P, P, I, I, I, I, I, I, I, P],
        "kllm_sum_splits": [P, I, L, P, I, P],
        "kllm_gemm_swiglu": [P, P, P, I, I, I, I, I, P],
        "kllm_gemv_plain": [P, P, P, I, I, I, I, P, P],
        "kllm_gemv_swiglu": [P, P, P, I, I, I, I, I, P, P],
        "kllm_gemv_rope_append": [P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, P, P],
        "kllm_gemv_resid": [P, P, P, P, I, I, I, I, P],
        "kllm_gemv_resid_parts": [I],
        "kllm_fused_linear": [P, I, P, P, I, I, I, I, P],
        "kllm_fused_linear_resid_parts": [I, I],
        "kllm_fused_linear_passes": [I, I, I],
        "kllm_fused_linear_tile": [P, P, I, I, I, I, I, I, I, P],
        "kllm_command_op": [c_char_p],
        "kllm_command_nargs": [I],
        "kllm_run_commands": [P, L, P, P],
        "kllm_fused_linear_max_parts": [],
        "kllm_attn_generic": [P, P, P, P, P, P, I, I, I, I, I, I, I, F, I, P],
        "kllm_sample": [P, P, P, P, I, I, P],
        "kllm_attn_decode_slices": [I, I, I, I, I, I],
        "kllm_device_cus": [],
        "kllm_device_xcds": [],
        "kllm_gemm_decode_tile_cols": [I, I, I],
        "kllm_gemv_max_rows": [],
        "kllm_gemv_normed_max_rows": [],
        "kllm_gemv_normed_max_parts": [],
        "kllm_attn_f32_fits": [I, I],
        "kllm_calibrate_copy": [P, P, L, P],
        "kllm_calibrate_read": [P, L, P, P],
        "kllm_calibrate_read_workgroups": [],
        "kllm_calibrate_mfma": [I, I, P, P, P],
        "kllm_attn_decode": [P, P, P, L, P, P, P, P, I, I, I, I, I, I, I, F, I, I, P, I, P],
        "kllm_attn_prefill": [P, P, P, P, I, P, P, P, I, I, I, I, I, I, F, L, I, P, L, I, I, I, P],
        "kllm_attn_prefill_slices": [I, I, I],
    }
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_int
    lib.kllm_fused_linear_lds_bytes.argtypes = [I, I, I]
    lib.kllm_fused_linear_lds_bytes.restype = L
    lib.kllm_fused_linear_tiled_elements.argtypes = [I, I, I]
    lib.kllm_fused_linear_tiled_elements.restype = L


# Entry points that launch work on a stream (and can be recorded into a command buffer), and
# which of their arguments are pointers to structures that travel with the command.
LAUNCHING = ("kllm_embed", "kllm_add_rmsnorm", "kllm_rope_tables", "kllm_rope_append", "kllm_silu_mul",
             "kllm_sum_splits", "kllm_gemm", "kllm_gemm_swiglu", "kllm_gemv_plain", "kllm_gemv_swiglu",
             "kllm_gemv_resid", "kllm_gemv_rope_append", "kllm_fused_linear", "kllm_attn_generic",
             "kllm_attn_decode", "kllm_attn_prefill", "kllm_sample")
DYNAMIC_ARGS = {"kllm_attn_prefill": (15, 16)}     # arguments that may be a StepValue
STRUCT_ARGS = {"kllm_gemv_plain": (7,), "kllm_gemv_swiglu": (8,), "kllm_gemv_rope_append": (17,),
               "kllm_fused_linear": (2,)}


def _check(rc: int, what: str):
    if rc == 0:
        return
    buf = ctypes.create_string_buffer(512)
    library().kllm_last_error(buf, 512)
    raise KernelError(f"{what}: {buf.value.decode(errors='replace')} (code {rc})")


_scoped = threading.local()


def _stream() -> int:
    s = getattr(_scoped, "stream", None)
    return s if s is not None else torch.cuda.current_stream().cuda_stream


class stream_scope:
    """Within the scope every launch of this thread goes to the stream that was
    current when the scope was entered, looked up once instead of once per
    launch (a step is a few hundred launches, and the lookup costs as much as
    a launch).  The caller must not switch streams inside the scope.

    With ``record`` the launches are not made one by one: each wrapper writes its entry
    point and arguments into a command buffer, and the library runs the buffer in one call
    (``kllm_run_commands``) when it holds ``chunk`` commands, when ``flush_recorded`` is
    called, and when the scope ends.  Work that reaches the stream by another way (torch
    operations, a part that launches for itself) must come after ``flush_recorded()``, and
    code that is not written for recording runs inside ``direct_launches()``."""

    def __init__(self, record: bool = False, chunk: int = 32, keep: bool = False):
        self._record, self._chunk, self._keep = record, chunk, keep
        self.recorder = None

    def __enter__(self):
        self._outer = (getattr(_scoped, "stream", None), getattr(_scoped, "recorder", None))
        _scoped.stream = torch.cuda.current_stream().cuda_stream
        self.recorder = _scoped.recorder = _Recorder(_scoped.stream, self._chunk, self._keep) if self._record else None
        return self

    def __exit__(self, exc_type, *exc):
        rec = _scoped.recorder
        _scoped.stream, _scoped.recorder = self._outer
        if rec is not None and exc_type is None:
            rec.flush()                      # after an error what was recorded is dropped
        return False

    def plan(self):
        """After the scope (opened with ``keep``): everything it ran, as a ``CommandPlan`` that
        runs the same launches again, or None if something in the scope was launched past the
        recording (such a step cannot be repeated from its commands alone)."""
        rec = self.recorder
        if rec is None or not rec.keep or rec.bypassed or not rec.kept:
            return None
        return CommandPlan(b"".join(rec.kept), rec.patches, rec.launched)


class StepValue(int):
    """A number that a part worked out on the host from a step's positions (how many keys its
    queries read, say) and hands to a kernel wrapper: it carries its name, so that a recorded
    step can be run again with this step's value in its place."""

    def __new__(cls, value, name):
        self = super().__new__(cls, value)
        self.name = name
        return self


class CommandPlan:
    """The launches of a step as they were recorded, ready to run again with one call of the
    library: the commands' bytes, and where the step's own values (``StepValue``) go in them."""

    def __init__(self, data: bytes, patches, count: int):
        self.size = len(data)
        self.buf = bytearray(data)
        self.cbuf = (ctypes.c_char * self.size).from_buffer(self.buf)
        self.patches = list(patches)         # (byte offset, name)
        self.count = count

    def run(self, values, stream=None):
        for off, name in self.patches:
            _PATCH.pack_into(self.buf, off, int(values[name]))
        failed = c_int(-1)
        rc = library().kllm_run_commands(self.cbuf, self.size // 8, ctypes.byref(failed),
                                         _stream() if stream is None else stream)
        if rc:
            buf = ctypes.create_string_buffer(512)
            library().kllm_last_error(buf, 512)
            raise KernelError(f"recorded step: {buf.value.decode(errors='replace')} (code {rc}; command "
                              f"{failed.value} of {self.count}, the ones before it have run)")


_PATCH = struct.Struct("<q")


class _Op:
    __slots__ = ("name", "index", "nargs", "pack", "size", "structs", "dynamic", "fn")


_op_table = None


def _ops():
    """name -> how to record a call of that entry point; built once from the signatures."""
    global _op_table
    if _op_table is None:
        lib = library()
        table = {}
        for name in LAUNCHING:
            fn = getattr(lib, name)
            op = _Op()
            op.name, op.fn = name, fn
            op.index = lib.kllm_command_op(name.encode())
            if op.index < 0 or lib.kllm_command_nargs(op.index) != len(fn.argtypes):
                raise KernelError(f"{name} cannot be recorded: the library knows it as command {op.index} with "
                                  f"{lib.kllm_command_nargs(op.index)} arguments, the host has {len(fn.argtypes)}")
            fmt, op.structs = "<Q", []
            for i, t in enumerate(fn.argtypes):
                if t is c_float:
                    fmt += "f4x"
                elif t is c_double:
                    fmt += "d"
                elif t is c_void_p:
                    fmt += "Q"
                else:
                    fmt += "q"
                if i in STRUCT_ARGS.get(name, ()):
                    op.structs.append(i)
            op.nargs = len(fn.argtypes)
            op.dynamic = DYNAMIC_ARGS.get(name, ())
            op.pack = struct.Struct(fmt)
            op.size = op.pack.size
            table[name] = op
        _op_table = table
    return _op_table


class _Recorder:
    """A step's launches as a buffer of commands (the layout is the library's, see
    csrc/executor.hpp) and the call that runs them."""

    def __init__(self, stream, chunk, keep=False):
        self.stream, self.chunk, self.keep = stream, chunk, keep
        self.kept, self.patches, self.kept_bytes = [], [], 0    # keep: all commands that ran, and where StepValues sit
        self.bypassed = False                                   # something was launched past the recording
        self.cap = 1 << 15
        self.buf = bytearray(self.cap)
        self.cbuf = (ctypes.c_char * self.cap).from_buffer(self.buf)
        self.at = 0                 # bytes used
        self.names = []             # what each command is, for error texts
        self.ops = _ops()
        self.run = library().kllm_run_commands
        self.launched = 0
        self.copy = None            # a RecordedRun that takes a copy of every command added, or None

    def _room(self, need):
        if self.at + need > self.cap:
            self.flush()
            if need > self.cap:
                del self.cbuf
                self.cap = max(2 * self.cap, need)
                self.buf = bytearray(self.cap)
                self.cbuf = (ctypes.c_char * self.cap).from_buffer(self.buf)

    def add(self, name, what, args):
        op = self.ops[name]
        if op.structs:
            # structs travel behind the arguments; the argument is their offset in words from the
            # command's first word
            args = list(args)
            payload = [(i, bytes(args[i])) for i in op.structs if args[i] is not None]
            total = op.size + sum(-(-len(b) // 8) * 8 for _, b in payload)
            self._room(total)
            at = self.at + op.size
            for i in op.structs:
                args[i] = 0
            for i, b in payload:
                self.buf[at:at + len(b)] = b
                args[i] = (at - self.at) // 8
                at += -(-len(b) // 8) * 8
        else:
            total = op.size
            self._room(total)
        op.pack.pack_into(self.buf, self.at, op.index | (op.nargs << 16) | ((total // 8) << 32), *args)
        copy = self.copy
        if self.keep and op.dynamic:
            for i in op.dynamic:
                if type(args[i]) is StepValue:
                    self.patches.append((self.kept_bytes + self.at + 8 + 8 * i, args[i].name))
                    if copy is not None:
                        copy.patches.append((len(copy.data) + 8 + 8 * i, args[i].name))
        if copy is not None:
            copy.data += self.buf[self.at:self.at + total]
            copy.names.append(what)
        self.at += total
        self.names.append(what)
        if len(self.names) >= self.chunk:
            self.flush()

    def add_commands(self, data, names, patches=()):
        """Commands that are written already (``data``: their bytes in the buffer's layout,
        ``names``: what each is, ``patches``: (byte offset in data, name) of the step's values
        in them), behind what was recorded so far."""
        self._room(len(data))
        self.buf[self.at:self.at + len(data)] = data
        if self.keep:
            self.patches.extend((self.kept_bytes + self.at + off, name) for off, name in patches)
        self.at += len(data)
        self.names.extend(names)
        if len(self.names) >= self.chunk:
            self.flush()

    def flush(self):
        if not self.names:
            return
        failed = c_int(-1)
        rc = self.run(self.cbuf, self.at // 8, ctypes.byref(failed), self.stream)
        if self.keep:
            self.kept.append(bytes(self.buf[:self.at]))
            self.kept_bytes += self.at
        names, self.names, self.at = self.names, [], 0
        self.launched += len(names)
        if rc:
            what = names[failed.value] if 0 <= failed.value < len(names) else "run_commands"
            buf = ctypes.create_string_buffer(512)
            library().kllm_last_error(buf, 512)
            raise KernelError(f"{what}: {buf.value.decode(errors='replace')} (code {rc}; command {failed.value} "
                              f"of {len(names)} recorded, the ones before it have run)")


class RecordedRun:
    """A copy of the commands that a stretch of a recording scope added (see ``copy_recorded``):
    their bytes, what each is, and where the step's values (``StepValue``) sit in them."""

    def __init__(self):
        self.data, self.names, self.patches = bytearray(), [], []


class copy_recorded:
    """Inside, every command that this thread records is also copied into ``self.run`` (a
    ``RecordedRun``); ``self.run`` is None outside a recording scope, and ``whole`` is False
    afterwards if something inside was launched past the recording."""

    def __enter__(self):
        self._rec = getattr(_scoped, "recorder", None)
        self.run, self.whole = None, False
        if self._rec is not None and self._rec.copy is None:
            self.run = self._rec.copy = RecordedRun()
            self._bypassed = self._rec.bypassed
            self._rec.bypassed = False
        return self

    def __exit__(self, *exc):
        if self.run is not None:
            self._rec.copy = None
            self.whole = not self._rec.bypassed and getattr(_scoped, "recorder", None) is self._rec
            self._rec.bypassed = self._rec.bypassed or self._bypassed
        return False


def add_recorded(data, names, patches=()):
    """Add commands that are written already to this thread's recording (``RecordedRun``'s
    fields, possibly changed)."""
    _scoped.recorder.add_commands(data, names, patches)


def flush_recorded():
    """Run what this thread has recorded so far (nothing to do outside a recording scope):
    call it before anything else is given to the stream."""
    rec = getattr(_scoped, "recorder", None)
    if rec is not None:
        rec.flush()


def bypass_recorded():
    """``flush_recorded`` for work that a repeat of the recorded commands would not repeat (a
    torch operation, a library call): the step is marked as not repeatable from its commands."""
    rec = getattr(_scoped, "recorder", None)
    if rec is not None:
        rec.flush()
        rec.bypassed = True


def recording() -> bool:
    return getattr(_scoped, "recorder", None) is not None


class direct_launches:
    """Inside, launches of this thread are made at once even in a recording scope (what was
    recorded before runs first): for code that puts work on the stream by other ways."""

    def __enter__(self):
        self._rec = getattr(_scoped, "recorder", None)
        if self._rec is not None:
            self._rec.flush()
            self._rec.bypassed = True
            _scoped.recorder = None
        return self

    def __exit__(self, *exc):
        if self._rec is not None:
            _scoped.recorder = self._rec
        return False


def _launch(name, what, *args):
    """Call the entry point ``name`` with ``args`` (pointers and numbers; a ctypes structure
    stands for a pointer to it), or record the call if this thread is recording."""
    rec = getattr(_scoped, "recorder", None)
    if rec is not None:
        rec.add(name, what, args)
        return
    fn = getattr(library(), name)
    if name in STRUCT_ARGS:
        args = [ctypes.byref(a) if isinstance(a, ctypes.Structure) else a for a in args]
    _check(fn(*args), what)


def _ptr(t, name, dtype=None, allow_none=False):
    if t is None:
        if allow_none:
            return 0            # a null pointer, for ctypes and in a recorded command alike
        raise KernelError(f"{name}: tensor is missing")
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on {t.device}, the kernels run on the GPU only")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: dtype {t.dtype}, expected {dtype}")
    return t.data_ptr()


def device_info(device: int = 0) -> str:
    buf = ctypes.create_string_buffer(256)
    _check(library().kllm_device_info(device, buf, 256), "device_info")
    return buf.value.decode()


# ----------------------------------------------------------------------------- wrappers

def calibrate_copy(dst, src):
    """dst = src with a plain copy kernel (for measuring the box's copy bandwidth)."""
    if dst.numel() * dst.element_size() != src.numel() * src.element_size():
        raise KernelError("calibrate_copy: sizes differ")
    _check(library().kllm_calibrate_copy(_ptr(dst, "copy dst"), _ptr(src, "copy src"),
                                         src.numel() * src.element_size(), _stream()), "calibrate_copy")


def calibrate_read(src, sink):
    """Read all of src with a plain streaming kernel (for measuring the box's read bandwidth);
    sink: float32, one element per workgroup (calibrate_read_workgroups())."""
    if sink.numel() < calibrate_read_workgroups():
        raise KernelError("calibrate_read: the sink is too short")
    _check(library().kllm_calibrate_read(_ptr(src, "read src"), src.numel() * src.element_size(),
                                         _ptr(sink, "read sink", torch.float32), _stream()), "calibrate_read")


def calibrate_read_workgroups() -> int:
    return int(library().kllm_calibrate_read_workgroups())


def calibrate_mfma(dtype_code_, iters, sink) -> float:
    """Launch the MFMA loop; returns the floating-point operations of the launch."""
    flops = c_double(0.0)
    _check(library().kllm_calibrate_mfma(int(dtype_code_), int(iters), _ptr(sink, "mfma sink", torch.float32),
                                         ctypes.byref(flops), _stream()), "calibrate_mfma")
    return flops.value


def embed(out, table, ids, from_sampled=None, sampled=None):
    """out [n, d] = table[ids]; where ``from_sampled[t] >= 0`` the id is
    ``sampled[from_sampled[t]]``, a token id still on the device."""
    n, d = out.shape
    if ids.numel() < n or table.shape[1] != d:
        raise KernelError(f"embed: out {tuple(out.shape)}, table {tuple(table.shape)}, "
                          f"{ids.numel()} ids do not fit")
    if (from_sampled is None) != (sampled is None) or (from_sampled is not None and from_sampled.numel() < n):
        raise KernelError("embed: from_sampled and sampled go together, one entry per token")
    _launch("kllm_embed", "embed", _ptr(out, "embed out", torch.float32), _ptr(table, "embed table"),
        _ptr(ids, "embed ids", torch.int32), _ptr(from_sampled, "embed from", torch.int32, True),
        _ptr(sampled, "embed sampled", torch.int32, True), n, d, table.shape[0], dtype_code(table.dtype),
        _stream())


def add_rmsnorm(x, delta=None, weight=None, out=None, rows=None, eps=0.0, write_x=None):
    """x [N, d] float32 in place; delta [nsplit, N, d] or [N, d]; out [n, d]."""
    d = x.shape[-1]
    if rows is not None:
        n = rows.numel()
        write_x = False
    else:
        n = x.shape[0]
        if write_x is None:
            write_x = delta is not None
    nsplit, stride, ddt = 1, 0, DT_F32
    if delta is not None:
        if delta.dim() == 3:
            nsplit, stride = delta.shape[0], delta.shape[1] * delta.shape[2]
        if delta.shape[-1] != d or delta.shape[-2] != x.shape[0]:
            raise KernelError(f"add_rmsnorm: delta {tuple(delta.shape)} does not fit x {tuple(x.shape)}")
        ddt = dtype_code(delta.dtype)
    if out is not None:
        if tuple(out.shape) != (n, d) or weight is None or weight.numel() != d:
            raise KernelError("add_rmsnorm: output or weight shape does not fit")
    _launch("kllm_add_rmsnorm", "add_rmsnorm", _ptr(x, "add_rmsnorm x", torch.float32), _ptr(delta, "add_rmsnorm delta", None, True), ddt,
        nsplit, stride, _ptr(weight, "add_rmsnorm weight", torch.float32, True),
        _ptr(out, "add_rmsnorm out", None, True),
        dtype_code(out.dtype) if out is not None else DT_F32,
        _ptr(rows, "add_rmsnorm rows", torch.int32, True), n, d, float(eps), int(bool(write_x)),
        _stream())


def rope_tables(cos, sin, positions, head_dim, theta):
    n = positions.numel()
    if tuple(cos.shape) != (n, head_dim // 2) or tuple(sin.shape) != (n, head_dim // 2):
        raise KernelError("rope_tables: table shapes do not fit")
    _launch("kllm_rope_tables", "rope_tables", _ptr(cos, "rope cos", torch.float32), _ptr(sin, "rope sin", torch.float32),
        _ptr(positions, "rope positions", torch.int32), n, head_dim, float(theta), _stream())


def rope_append(qkv, q_out, cos, sin, cache, positions, span_of_token, block_table, page_size,
                n_heads, n_kv_heads, head_dim, rotary_dim=None, interleaved=False):
    """qkv [nsplit, n, cols] or [n, cols]; cache [pages, 2, KV, page_size*hd] or None.
    ``rotary_dim`` (default: the head) elements of every head are rotated, in pairs
    (j, j + rotary_dim/2) or, ``interleaved``, (2j, 2j + 1); cos and sin are [n, rotary_dim/2]."""
    rot = head_dim if rotary_dim is None else int(rotary_dim)
    n = q_out.shape[0]
    nsplit, stride = 1, 0
    if qkv.dim() == 3:
        nsplit, stride = qkv.shape[0], qkv.shape[1] * qkv.shape[2]
    cols = n_heads * head_dim + (2 * n_kv_heads * head_dim if cache is not None else 0)
    if qkv.shape[-1] != cols or qkv.shape[-2] != n or q_out.shape[1] != n_heads * head_dim:
        raise KernelError(f"rope_append: qkv {tuple(qkv.shape)} does not fit {n} x {cols}")
    max_pages = 0
    if cache is not None:
        if tuple(cache.shape[1:]) != (2, n_kv_heads, page_size * head_dim) or cache.dtype != q_out.dtype:
            raise KernelError(f"rope_append: cache {tuple(cache.shape)} {cache.dtype} does not fit")
        max_pages = block_table.shape[1]
        if positions.numel() < n or span_of_token.numel() < n:
            raise KernelError("rope_append: index arrays are too short")
    if cos is not None and (tuple(cos.shape) != (n, rot // 2) or tuple(sin.shape) != tuple(cos.shape)):
        raise KernelError("rope_append: cos/sin shapes do not fit")
    _launch("kllm_rope_append", "rope_append", _ptr(qkv, "rope_append qkv"), dtype_code(qkv.dtype), nsplit, stride,
        _ptr(q_out, "rope_append q_out"), _ptr(cos, "rope_append cos", torch.float32, True),
        _ptr(sin, "rope_append sin", torch.float32, True), _ptr(cache, "rope_append cache", None, True),
        _ptr(positions, "rope_append positions", torch.int32, True),
        _ptr(span_of_token, "rope_append span_of_token", torch.int32, True),
        _ptr(block_table, "rope_append block_table", torch.int32, True), max_pages, page_size, n,
        n_heads, n_kv_heads, head_dim, rot, int(bool(interleaved)), dtype_code(q_out.dtype), _stream())


ACT_SILU, ACT_GELU_TANH = 0, 1
ACTIVATIONS = {"silu": ACT_SILU, "swish": ACT_SILU, "gelu_tanh": ACT_GELU_TANH, "gelu_pytorch_tanh": ACT_GELU_TANH}


def silu_mul(gu, out, act=ACT_SILU):
    """out [n, f] = act(gu[:, :f]) * gu[:, f:] (the gate of a gated feed-forward)."""
    n, f = out.shape
    nsplit, stride = 1, 0
    if gu.dim() == 3:
        nsplit, stride = gu.shape[0], gu.shape[1] * gu.shape[2]
    if gu.shape[-1] != 2 * f or gu.shape[-2] != n:
        raise KernelError(f"silu_mul: input {tuple(gu.shape)} does not fit output {tuple(out.shape)}")
    _launch("kllm_silu_mul", "silu_mul", _ptr(gu, "silu_mul in"), dtype_code(gu.dtype), nsplit, stride, _ptr(out, "silu_mul out"),
        dtype_code(out.dtype), n, f, int(act), _stream())


class _NormedInput(ctypes.Structure):
    _fields_ = [("x", c_void_p), ("weight", c_void_p), ("ss", c_void_p), ("parts", c_int), ("eps", c_float)]


class NormedInput:
    """The input of a product as the RMS norm of a residual stream, made by the product's
    kernel while it stages X: ``x`` [n, k] float32 (the stream, already holding what was
    added), the norm's ``weight`` [k] and ``eps``, and ``ss`` [n, parts rounded up to 4]
    float32, the partial sums of squares of x's rows that a residual product left."""

    def __init__(self, x, weight, ss, parts, eps):
        self.x, self.weight, self.ss, self.parts, self.eps = x, weight, ss, int(parts), float(eps)

    @property
    def shape(self):
        return self.x.shape

    def struct(self, n, k):
        stride = -(-self.parts // 4) * 4
        if (tuple(self.x.shape) != (n, k) or self.weight.numel() != k or tuple(self.ss.shape) != (n, stride)
                or not 1 <= self.parts <= limit("gemv_normed_max_parts")):
            raise KernelError(f"normed input: stream {tuple(self.x.shape)}, weight {tuple(self.weight.shape)}, sums of "
                              f"squares {tuple(self.ss.shape)} do not fit {n} x {k} with {self.parts} parts")
        return _NormedInput(_ptr(self.x, "normed x", torch.float32), _ptr(self.weight, "normed weight", torch.float32),
                            _ptr(self.ss, "normed ss", torch.float32), self.parts, self.eps)


def _x_and_norm(x, dtype):
    """(pointer of x or 0, struct or None, n, k) for an input that is a tensor or a NormedInput."""
    if isinstance(x, NormedInput):
        n, k = x.shape
        st = x.struct(n, k)
        return 0, st, n, k
    n, k = x.shape
    if x.dtype != dtype:
        raise KernelError(f"input dtype {x.dtype}, weights {dtype}")
    return _ptr(x, "x"), None, n, k


def normed_max_rows() -> int:
    """Rows that the small-batch kernels normalise while they stage their input."""
    return limit("gemv_normed_max_rows")


def resid_parts(n, m, k, dtype, best=True):
    """Partial sums of squares per row that a residual product of these sizes
    leaves (one per workgroup of eight rows of W), or 0 if the small-batch
    kernel with that epilogue does not take them (``best``: or is not the
    faster choice)."""
    if not (gemv_fits(n, m, k, dtype, best) and n <= normed_max_rows()):
        return 0
    parts = library().kllm_gemv_resid_parts(m)
    return parts if parts <= limit("gemv_normed_max_parts") else 0


def linear_resid(x, w, resid, ss):
    """resid [n, m] float32 += x . w^T in place; ss [n, parts rounded up to 4] receives the
    partial sums of squares of resid's new rows (parts = resid_parts(...), returned)."""
    n, k = x.shape
    m = w.shape[0]
    parts = resid_parts(n, m, k, x.dtype, best=False)
    stride = -(-parts // 4) * 4
    if (parts == 0 or tuple(resid.shape) != (n, m) or tuple(ss.shape) != (n, stride) or w.shape[1] != k
            or w.dtype != x.dtype):
        raise KernelError(f"linear_resid: x {tuple(x.shape)}, w {tuple(w.shape)}, resid {tuple(resid.shape)}, "
                          f"ss {tuple(ss.shape)} do not fit ({parts} parts)")
    _launch("kllm_gemv_resid", "gemv_resid", _ptr(x, "resid x"), _ptr(w, "resid w"), _ptr(resid, "resid", torch.float32),
        _ptr(ss, "resid ss", torch.float32), n, m, k, dtype_code(x.dtype), _stream())
    return parts


def gemm(x, w, y, algo, nsplit=1):
    """y [nsplit, n, m] (or [n, m]) = x [n, k] . w [m, k]^T."""
    n, k = x.shape
    m = w.shape[0]
    if w.shape[1] != k or x.dtype != w.dtype:
        raise KernelError(f"gemm: x {tuple(x.shape)} {x.dtype} and w {tuple(w.shape)} {w.dtype} do not fit")
    want = (nsplit, n, m) if y.dim() == 3 else (n, m)
    if tuple(y.shape) != want or (y.dim() == 2 and nsplit != 1):
        raise KernelError(f"gemm: output {tuple(y.shape)} does not fit {want}")
    if algo == GEMM_GEMV_LDS:
        if nsplit != 1:
            raise KernelError("gemm: the LDS gemv does not split K")
        _launch("kllm_gemv_plain", "gemv_plain", _ptr(x, "gemv x"), _ptr(w, "gemv w"), _ptr(y, "gemv y", torch.float32), n, m, k,
            dtype_code(x.dtype), None, _stream())
        return
    _launch("kllm_gemm", "gemm", _ptr(x, "gemm x"), _ptr(w, "gemm w"), _ptr(y, "gemm y"), n, m, k, dtype_code(x.dtype),
        dtype_code(y.dtype), algo, nsplit, _stream())


def gemv_fits(n, m, k, dtype, best=True) -> bool:
    """Whether the fused small-batch products take these sizes and, with
    ``best``, are the faster choice: always in float32 (which has no MFMA
    kernel for decode batches), up to GEMV_BEST_ROWS rows in bfloat16."""
    v = 4 if dtype == torch.float32 else 8
    most = limit("gemv_max_rows") if dtype == torch.float32 or not best else GEMV_BEST_ROWS
    return n <= most and m % 2 == 0 and k % v == 0


def gemm_swiglu(x, w_gate_up, h, act=ACT_SILU):
    """h [n, f] = silu(x . gate^T) * (x . up^T) on the MFMA tiles (any n; float32 with 32-bit MFMA)."""
    n, k = x.shape
    f = h.shape[1]
    if tuple(w_gate_up.shape) != (2 * f, k) or h.shape[0] != n or x.dtype != w_gate_up.dtype or h.dtype != x.dtype:
        raise KernelError("gemm_swiglu: shapes or dtypes do not fit")
    _launch("kllm_gemm_swiglu", "gemm_swiglu", _ptr(x, "gemm x"), _ptr(w_gate_up, "gemm w"), _ptr(h, "gemm h"), n, f, k,
                                      dtype_code(x.dtype), int(act), _stream())


def gemv_swiglu(x, w_gate_up, h, act=ACT_SILU):
    """h [n, f] = act(x . gate^T) * (x . up^T); w_gate_up is [2f, k], gate rows first.  x
    is a tensor or a NormedInput."""
    xp, st, n, k = _x_and_norm(x, w_gate_up.dtype)
    f = h.shape[1]
    if tuple(w_gate_up.shape) != (2 * f, k) or h.shape[0] != n or h.dtype != w_gate_up.dtype:
        raise KernelError("gemv_swiglu: shapes or dtypes do not fit")
    _launch("kllm_gemv_swiglu", "gemv_swiglu", xp, _ptr(w_gate_up, "gemv w"), _ptr(h, "gemv h"), n, f, k,
                                      dtype_code(w_gate_up.dtype), int(act), st, _stream())


def gemv_rope_append(x, w_qkv, q_out, cos, sin, cache, positions, span_of_token, block_table, page_size,
                     n_heads, n_kv_heads, head_dim):
    """q, k, v projections of up to 8 rows (x a tensor or a NormedInput), rotation, q_out and
    the cache append in one launch."""
    xp, st, n, k = _x_and_norm(x, w_qkv.dtype)
    rows = n_heads * head_dim + (2 * n_kv_heads * head_dim if cache is not None else 0)
    if (tuple(w_qkv.shape) != (rows, k) or tuple(q_out.shape) != (n, n_heads * head_dim)
            or q_out.dtype != w_qkv.dtype):
        raise KernelError("gemv_rope_append: shapes or dtypes do not fit")
    max_pages = 0
    if cache is not None:
        if tuple(cache.shape[1:]) != (2, n_kv_heads, page_size * head_dim) or cache.dtype != w_qkv.dtype:
            raise KernelError(f"gemv_rope_append: cache {tuple(cache.shape)} {cache.dtype} does not fit")
        max_pages = block_table.shape[1]
        if positions.numel() < n or span_of_token.numel() < n:
            raise KernelError("gemv_rope_append: index arrays are too short")
    if cos is not None and (tuple(cos.shape) != (n, head_dim // 2) or tuple(sin.shape) != tuple(cos.shape)):
        raise KernelError("gemv_rope_append: cos/sin shapes do not fit")
    _launch("kllm_gemv_rope_append", "gemv_rope_append", xp, _ptr(w_qkv, "gemv w"), _ptr(q_out, "gemv q_out"),
        _ptr(cos, "gemv cos", torch.float32, True), _ptr(sin, "gemv sin", torch.float32, True),
        _ptr(cache, "gemv cache", None, True), _ptr(positions, "gemv positions", torch.int32, True),
        _ptr(span_of_token, "gemv span_of_token", torch.int32, True),
        _ptr(block_table, "gemv block_table", torch.int32, True), max_pages, page_size, n, n_heads,
        n_kv_heads, head_dim, k, dtype_code(w_qkv.dtype), st, _stream())


class _LinearOut(ctypes.Structure):
    _fields_ = [("y", c_void_p), ("cos_t", c_void_p), ("sin_t", c_void_p), ("cache", c_void_p),
                ("positions", c_void_p), ("span_of_token", c_void_p), ("block_table", c_void_p),
                ("kind", c_int), ("nsplit", c_int), ("max_pages", c_int), ("page_size", c_int),
                ("H", c_int), ("KV", c_int), ("hd", c_int), ("act", c_int),
                ("resid", c_void_p), ("norm_w", c_void_p), ("ss_out", c_void_p), ("ss_in", c_void_p),
                ("ss_parts", c_int), ("eps", c_float), ("tiled", c_int)]


FUSED_LINEAR_MAX_ROWS = 32
FUSED_LINEAR_LDS = 160 * 1024
LINEAR_PARTS, LINEAR_RESID, LINEAR_SWIGLU, LINEAR_ROPE = 0, 1, 2, 3


# Rows up to which the decode-batch kernel beats the split-K kernel plus a separate
# elementwise launch (measured at widths 2048 -> 2560 and 2048 -> 11264).
FUSED_NORM_BEST_ROWS = 32      # rows up to which a residual product and a consumer that scales its rows replace the norm kernel
FUSED_ROPE_BEST_ROWS = 32      # (17 tokens at 1.1B sizes: 1.59 -> 1.55 ms a step against the tiled product and a rotation kernel)
FUSED_SWIGLU_BEST_ROWS = 32    # (both at 32 against 16, a step at 1.1B sizes: 17 tokens 1.51 -> 1.41 ms, 32 tokens 1.70 -> 1.62; at 8B sizes 17 tokens 5.50 -> 5.19)


@functools.lru_cache(maxsize=4096)
def fused_tiles_per_wg(n, m, k) -> int:
    """Tiles of 16 rows of W that one workgroup of the decode-batch kernel takes, one after
    the other, with the rows of X staged once: from 9 rows of X on against large weights two
    (16 rows, 4,096 -> 2 x 14,336 with the gate: 58.8 us against 66.1; 4,096 -> 6,144 with the
    rotation: 18.1 against 22.4), or up to four if that brings the workgroups down to one
    round of the chip (2,048 -> 2 x 5,632, 704 tiles: a step of 9 / 12 / 16 tokens at 1.1B sizes
    1.271 / 1.297 / 1.379 ms with two, 1.254 / 1.272 / 1.353 with three), one otherwise."""
    if n <= 8 or m * k < 20_000_000:
        return 1
    tiles, t = -(-m // 16), 2
    while t < 4 and -(-tiles // t) > device_cus():
        t += 1
    return t


@functools.lru_cache(maxsize=4096)
def fused_linear_fits(n, k, nsplit=1) -> bool:
    """Whether the decode-batch products take n rows of K: bfloat16 only, K a
    multiple of 8, and all rows of a workgroup's slice of K in LDS."""
    if n < 1 or n > FUSED_LINEAR_MAX_ROWS or k % 8:
        return False
    return 0 < library().kllm_fused_linear_lds_bytes(int(n), int(k), int(nsplit)) <= FUSED_LINEAR_LDS


# Passes over K up to which the decode-batch kernel is taken where the rows do not fit into LDS at
# once, and the rows up to which that pays (a step at 1.1B sizes, 16 tokens: 1.284 -> 1.237 ms; at 8B
# sizes 8 tokens 4.41 -> 4.08, 16 tokens 5.61 -> 4.75; from 17 rows on, two tiles of rows, the
# tiled product and a kernel behind it are as fast or faster: 1.1B sizes, 24 tokens 1.47 against
# 1.48 ms, 32 tokens 1.59 against 1.66; 8B sizes, 24 tokens 5.71 against 6.48).
FUSED_LINEAR_BEST_PASSES = 4
FUSED_LINEAR_PASSES_BEST_ROWS = 16


@functools.lru_cache(maxsize=4096)
def fused_linear_passes(n, k, nsplit=1) -> int:
    """Passes over K in which the decode-batch products take n rows: 1 where all rows of a
    workgroup's slice of K fit into LDS (``fused_linear_fits``); more, with one tile to a
    workgroup, where they do not; 0 if the kernel does not take the sizes."""
    if n < 1 or n > FUSED_LINEAR_MAX_ROWS or k % 8:
        return 0
    return int(library().kllm_fused_linear_passes(int(n), int(k), int(nsplit)))


def fused_linear_tiles(n, m, k) -> int:
    """Tiles per workgroup with which the decode-batch kernel is taken for n rows against
    w [m, k] (``fused_tiles_per_wg`` where the rows fit into LDS at once, one where they go in
    a few passes over K), or 0 where it is not taken."""
    passes = fused_linear_passes(n, k)
    if passes == 0 or (passes > 1 and (passes > FUSED_LINEAR_BEST_PASSES or n > FUSED_LINEAR_PASSES_BEST_ROWS)):
        return 0
    return fused_tiles_per_wg(n, m, k) if passes == 1 else 1


class TiledWeights:
    """A copy of a weight matrix [m, k] in the order the decode-batch kernel's lanes read it, for
    one output kind (LINEAR_PARTS serves LINEAR_RESID too; LINEAR_ROPE is made for the heads it
    will be called with).  ``fused_linear`` takes it in place of the matrix."""

    def __init__(self, data, kind, m, k, heads=None):
        self.data, self.kind, self.shape, self.heads = data, kind, (m, k), heads
        self.dtype = data.dtype


def fused_linear_tile(w, kind, rope=None):
    """The tiled copy of ``w`` [m, k] (bfloat16, k a multiple of 8) for ``kind``; ``rope`` as
    for ``fused_linear`` (its heads and whether a cache is written decide the rows' order)."""
    m, k = w.shape
    if w.dtype != torch.bfloat16 or k % 8:
        raise KernelError("fused_linear_tile: bfloat16 weights with K a multiple of 8 only")
    base = LINEAR_PARTS if kind == LINEAR_RESID else kind
    count = library().kllm_fused_linear_tiled_elements(base, m, k)
    if count <= 0:
        raise KernelError(f"fused_linear_tile: sizes {m} x {k} are not taken")
    out = torch.empty(count, dtype=torch.bfloat16, device=w.device)
    heads = (0, 0, 0, 0)
    if base == LINEAR_ROPE:
        if rope is None:
            raise KernelError("fused_linear_tile: the rope kind needs its heads")
        heads = (rope.heads, rope.kv_heads, rope.head_dim, int(rope.cache is not None))
    _check(library().kllm_fused_linear_tile(_ptr(w, "tile w"), _ptr(out, "tile out"), base, m, k, *heads, _stream()),
           "fused_linear_tile")
    return TiledWeights(out, base, m, k, heads)


class ScaledRows:
    """The input of a decode batch's product as a residual product (LINEAR_RESID) left it:
    ``xw`` [n, k] bfloat16, the residual stream's rows times the norm's weight, and ``ss``
    [n, parts rounded up to 4] float32, partial sums of squares of the stream's rows.  The
    consuming product multiplies its sums by rsqrt(sum of a row's ss / k + eps)."""

    def __init__(self, xw, ss, parts, eps):
        self.xw, self.ss, self.parts, self.eps = xw, ss, int(parts), float(eps)

    @property
    def shape(self):
        return self.xw.shape


@functools.lru_cache(maxsize=4096)
def fused_resid_parts(n, m, k, tiles_per_wg=1) -> int:
    """Partial sums of squares per row that a LINEAR_RESID product of these sizes leaves, or 0
    if the decode-batch kernel does not take them."""
    passes = fused_linear_passes(n, k)
    if passes == 0 or (passes > 1 and tiles_per_wg != 1):
        return 0
    parts = library().kllm_fused_linear_resid_parts(int(m), int(tiles_per_wg))
    return parts if 0 < parts <= limit("fused_linear_max_parts") else 0


class Rope:
    """What the rotate-and-append epilogue needs beside the product."""

    def __init__(self, cos, sin, cache, positions, span_of_token, block_table, page_size, heads, kv_heads,
                 head_dim):
        self.cos, self.sin, self.cache = cos, sin, cache
        self.positions, self.span_of_token, self.block_table = positions, span_of_token, block_table
        self.page_size, self.heads, self.kv_heads, self.head_dim = page_size, heads, kv_heads, head_dim


def fused_linear(w, y, kind, x, nsplit=1, tiles_per_wg=1, rope=None, act=ACT_SILU, resid=None, norm_weight=None,
                 ss_out=None):
    """One launch for a decode batch's product of x [n, k] (bfloat16; a view
    with a row stride is taken) with w [m, k], and the step after it, by
    ``kind``: LINEAR_PARTS y float32 [nsplit, n, m]; LINEAR_SWIGLU y bfloat16
    [n, m/2]; LINEAR_ROPE y = q_out with ``rope`` describing rotation and
    cache; LINEAR_RESID adds the product to ``resid`` [n, m] float32 in place, writes
    y bfloat16 [n, m] = the new rows times ``norm_weight`` [m] and leaves partial sums of
    squares of the new rows in ``ss_out`` [n, fused_resid_parts rounded up to 4].  ``x`` may
    be a ``ScaledRows`` (SWIGLU and ROPE): what a LINEAR_RESID product left, see there."""
    m, k = w.shape
    lo = _LinearOut()
    if w.dtype != torch.bfloat16:
        raise KernelError("fused_linear: bfloat16 weights only")
    if isinstance(w, TiledWeights):
        if w.kind != (LINEAR_PARTS if kind == LINEAR_RESID else kind):
            raise KernelError(f"fused_linear: the tiled weights were made for output kind {w.kind}, not {kind}")
        if kind == LINEAR_ROPE and (rope is None or w.heads != (rope.heads, rope.kv_heads, rope.head_dim,
                                                                 int(rope.cache is not None))):
            raise KernelError("fused_linear: the tiled weights were made for other heads")
        lo.tiled, w = 1, w.data
    if isinstance(x, ScaledRows):
        sr, x = x, x.xw
        stride = -(-sr.parts // 4) * 4
        if kind not in (LINEAR_SWIGLU, LINEAR_ROPE) or tuple(sr.ss.shape) != (x.shape[0], stride):
            raise KernelError(f"fused_linear: row scales {tuple(sr.ss.shape)} of {sr.parts} parts do not fit "
                              f"{x.shape[0]} rows, or the output kind {kind} takes none")
        lo.ss_in, lo.ss_parts, lo.eps = _ptr(sr.ss, "fused_linear ss", torch.float32), sr.parts, sr.eps
    n = x.shape[0]
    lo.kind, lo.nsplit, lo.act = kind, nsplit, int(act)
    if x.dim() != 2 or x.shape[1] != k or x.dtype != torch.bfloat16 or x.stride(1) != 1 or not x.is_cuda:
        raise KernelError(f"fused_linear: x {tuple(x.shape)} {x.dtype} does not fit w {tuple(w.shape)}")
    x_ptr, x_stride = x.data_ptr(), (x.stride(0) if n > 1 else k)
    if kind == LINEAR_PARTS:
        want, dt = (nsplit, n, m), torch.float32
    elif kind == LINEAR_RESID:
        want, dt = (n, m), torch.bfloat16
        parts = library().kllm_fused_linear_resid_parts(int(m), int(tiles_per_wg))
        if (resid is None or norm_weight is None or ss_out is None or tuple(resid.shape) != (n, m)
                or norm_weight.numel() != m or tuple(ss_out.shape) != (n, -(-parts // 4) * 4)):
            raise KernelError(f"fused_linear: the residual epilogue needs resid [{n}, {m}], the norm's weight [{m}] "
                              f"and ss_out [{n}, {-(-parts // 4) * 4}]")
        lo.resid = _ptr(resid, "fused_linear resid", torch.float32)
        lo.norm_w = _ptr(norm_weight, "fused_linear norm weight", torch.float32)
        lo.ss_out = _ptr(ss_out, "fused_linear ss_out", torch.float32)
    elif kind == LINEAR_SWIGLU:
        want, dt = (n, m // 2), torch.bfloat16
    elif kind == LINEAR_ROPE:
        if rope is None:
            raise KernelError("fused_linear: the rope epilogue needs its description")
        want, dt = (n, rope.heads * rope.head_dim), torch.bfloat16
        half = rope.head_dim // 2
        if rope.cos is not None and (tuple(rope.cos.shape) != (n, half) or tuple(rope.sin.shape) != (n, half)):
            raise KernelError("fused_linear: cos/sin shapes do not fit")
        lo.cos_t = _ptr(rope.cos, "fused_linear cos", torch.float32, True)
        lo.sin_t = _ptr(rope.sin, "fused_linear sin", torch.float32, True)
        if rope.cache is not None:
            if (tuple(rope.cache.shape[1:]) != (2, rope.kv_heads, rope.page_size * rope.head_dim)
                    or rope.cache.dtype != torch.bfloat16):
                raise KernelError(f"fused_linear: cache {tuple(rope.cache.shape)} {rope.cache.dtype} does not fit")
            if rope.positions.numel() < n or rope.span_of_token.numel() < n:
                raise KernelError("fused_linear: index arrays are too short")
            lo.cache = _ptr(rope.cache, "fused_linear cache")
            lo.positions = _ptr(rope.positions, "fused_linear positions", torch.int32)
            lo.span_of_token = _ptr(rope.span_of_token, "fused_linear span_of_token", torch.int32)
            lo.block_table = _ptr(rope.block_table, "fused_linear block_table", torch.int32)
            lo.max_pages = rope.block_table.shape[1]
        lo.page_size, lo.H, lo.KV, lo.hd = rope.page_size, rope.heads, rope.kv_heads, rope.head_dim
    else:
        raise KernelError(f"fused_linear: unknown output kind {kind}")
    if tuple(y.shape) != want or y.dtype != dt:
        raise KernelError(f"fused_linear: output {tuple(y.shape)} {y.dtype}, expected {want} {dt}")
    lo.y = _ptr(y, "fused_linear y")
    _launch("kllm_fused_linear", "fused_linear", x_ptr, x_stride, lo, _ptr(w, "fused_linear w"), n, m, k,
                                       tiles_per_wg, _stream())


def sum_splits(parts, out):
    """out [n, m] = parts [nsplit, n, m] summed over the first axis."""
    nsplit = parts.shape[0]
    if tuple(parts.shape[1:]) != tuple(out.shape):
        raise KernelError("sum_splits: shapes do not fit")
    _launch("kllm_sum_splits", "sum_splits", _ptr(parts, "sum_splits in", torch.float32), nsplit, out.numel(),
                                     _ptr(out, "sum_splits out"), dtype_code(out.dtype), _stream())


def attn_generic(q, out, cache, positions, span_of_token, block_table, page_size, n_heads,
                 n_kv_heads, head_dim, window, scale):
    n = q.shape[0]
    if (tuple(q.shape) != (n, n_heads * head_dim) or tuple(out.shape) != tuple(q.shape)
            or q.dtype != cache.dtype or out.dtype != q.dtype):
        raise KernelError("attn_generic: q/out shapes or dtypes do not fit")
    if tuple(cache.shape[1:]) != (2, n_kv_heads, page_size * head_dim):
        raise KernelError(f"attn_generic: cache {tuple(cache.shape)} does not fit")
    if positions.numel() < n or span_of_token.numel() < n:
        raise KernelError("attn_generic: index arrays are too short")
    _launch("kllm_attn_generic", "attn_generic", _ptr(q, "attn q"), _ptr(out, "attn out"), _ptr(cache, "attn cache"),
        _ptr(positions, "attn positions", torch.int32),
        _ptr(span_of_token, "attn span_of_token", torch.int32),
        _ptr(block_table, "attn block_table", torch.int32), block_table.shape[1], page_size, n,
        n_heads, n_kv_heads, head_dim, int(window), float(scale), dtype_code(q.dtype), _stream())


GENERIC_MAX_PAGE_SIZE = 256     # pages of the kernel that takes every size
DECODE_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 192, 256)


@functools.lru_cache(maxsize=4096)
def attn_decode_slices(n, n_kv_heads, n_heads, head_dim, dtype=torch.bfloat16, max_keys=0) -> int:
    """Slices of keys for a decode batch of n tokens; ``max_keys`` bounds the keys of the
    longest request (block-table width x page size, or the window), 0 if unknown."""
    return library().kllm_attn_decode_slices(n, n_kv_heads, n_heads, int(head_dim), dtype_code(dtype),
                                             int(max_keys))


def attn_f32_fits(head_dim, page_size) -> bool:
    """Sizes the float32 attention on the matrix cores takes; the rest goes to
    the generic kernel."""
    return bool(library().kllm_attn_f32_fits(int(head_dim), int(page_size)))


@functools.lru_cache(maxsize=4096)
def gemm_decode_tile_cols(n, m, k) -> int:
    """Columns of the tiles that the MFMA kernel gives a decode batch of these sizes."""
    return int(library().kllm_gemm_decode_tile_cols(int(n), int(m), int(k)))


_cus = None


def device_cus() -> int:
    """Compute units of the current device; the choice of kernels and of
    slices of K scales with it."""
    global _cus
    if _cus is None:
        _cus = int(library().kllm_device_cus())
    return _cus


GEMM_TILE_ROWS = 128           # rows of X in a tile of the prompt products (256 where those fill the chip)
PREFILL_HEAD_DIMS = (32, 64, 96, 128, 192, 256)
PREFILL_QUERY_BLOCK = 128      # tokens of one request that a workgroup of the prompt kernel takes


def attn_prefill_slices(n_tiles, n_heads, head_dim, dtype=torch.bfloat16) -> int:
    """Workgroups that share out the keys of a block and head in ``attn_prefill`` (1: none):
    more where few blocks of a large head would leave CUs idle; the library says."""
    if dtype != torch.bfloat16:
        return 1
    return int(library().kllm_attn_prefill_slices(int(n_tiles), int(n_heads), int(head_dim)))


def attn_prefill(q, out, cache, query_tiles, n_tiles, span_start, span_pos, block_table, page_size,
                 n_heads, n_kv_heads, head_dim, window, scale, keys_total=0, keys_longest=0, part=None,
                 nslices=None):
    """query_tiles [n_tiles, 2] int32: (first token row, span) of each block of up to
    PREFILL_QUERY_BLOCK consecutive tokens of one span.  ``keys_total`` and
    ``keys_longest``: how many keys the blocks read, all together and the longest block
    alone, if the caller knows (the kernel is chosen by them).  ``part``: float32 room for the
    slices' partial results where ``attn_prefill_slices`` says more than one (rows of q x heads
    x slices x (head_dim + 2)); made here if the caller brings none.  ``nslices``: 1 to do
    without slices, or what ``attn_prefill_slices`` says (the default)."""
    n = q.shape[0]
    if nslices is None:
        nslices = attn_prefill_slices(n_tiles, n_heads, head_dim, q.dtype)
    need = n * n_heads * nslices * (head_dim + 2) if nslices > 1 else 0
    if nslices > 1 and part is None:
        part = torch.empty(need, dtype=torch.float32, device=q.device)
    if nslices > 1 and (part.dtype != torch.float32 or part.numel() < need):
        raise KernelError(f"attn_prefill: {nslices} slices need {need} floats of room, {part.numel()} {part.dtype} given")
    if (tuple(q.shape) != (n, n_heads * head_dim) or tuple(out.shape) != tuple(q.shape)
            or q.dtype != cache.dtype or out.dtype != q.dtype):
        raise KernelError("attn_prefill: q/out shapes or dtypes do not fit")
    if tuple(cache.shape[1:]) != (2, n_kv_heads, page_size * head_dim):
        raise KernelError(f"attn_prefill: cache {tuple(cache.shape)} does not fit")
    if query_tiles.numel() < 2 * n_tiles:
        raise KernelError("attn_prefill: tile list is too short")
    _launch("kllm_attn_prefill", "attn_prefill", _ptr(q, "attn q"), _ptr(out, "attn out"), _ptr(cache, "attn cache"),
        _ptr(query_tiles, "attn query_tiles", torch.int32), n_tiles,
        _ptr(span_start, "attn span_start", torch.int32), _ptr(span_pos, "attn span_pos", torch.int32),
        _ptr(block_table, "attn block_table", torch.int32), block_table.shape[1], page_size,
        n_heads, n_kv_heads, head_dim, int(window), float(scale),
        keys_total if type(keys_total) is StepValue else int(keys_total),
        keys_longest if type(keys_longest) is StepValue else int(keys_longest),
        _ptr(part, "attn part", torch.float32, True) if nslices > 1 else 0, need, nslices, n,
        dtype_code(q.dtype), _stream())


def attn_decode(q, out, part, cache, positions, span_of_token, block_table, page_size, n_heads,
                n_kv_heads, head_dim, window, scale, nslices, token_list=None, n_listed=0):
    n = q.shape[0]
    if (tuple(q.shape) != (n, n_heads * head_dim) or tuple(out.shape) != tuple(q.shape)
            or q.dtype != cache.dtype or out.dtype != q.dtype):
        raise KernelError("attn_decode: q/out shapes or dtypes do not fit")
    if tuple(cache.shape[1:]) != (2, n_kv_heads, page_size * head_dim):
        raise KernelError(f"attn_decode: cache {tuple(cache.shape)} does not fit")
    if positions.numel() < n or span_of_token.numel() < n:
        raise KernelError("attn_decode: index arrays are too short")
    _launch("kllm_attn_decode", "attn_decode", _ptr(q, "attn q"), _ptr(out, "attn out"), _ptr(part, "attn part", torch.float32),
        part.numel(), _ptr(cache, "attn cache"), _ptr(positions, "attn positions", torch.int32),
        _ptr(span_of_token, "attn span_of_token", torch.int32),
        _ptr(block_table, "attn block_table", torch.int32), block_table.shape[1], page_size, n,
        n_heads, n_kv_heads, head_dim, int(window), float(scale), int(nslices), dtype_code(q.dtype),
        _ptr(token_list, "attn token_list", torch.int32, True), int(n_listed), _stream())


def sample(out, logits, temperature=None, uniform=None):
    rows, vocab = logits.shape
    if out.numel() < rows:
        raise KernelError("sample: output is too short")
    _launch("kllm_sample", "sample", _ptr(out, "sample out", torch.int32), _ptr(logits, "sample logits", torch.float32),
        _ptr(temperature, "sample temperature", torch.float32, True),
        _ptr(uniform, "sample uniform", torch.float32, True), rows, vocab, _stream())
