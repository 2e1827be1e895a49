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
ABI_VERSION = 13


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
        "kllm_embed": [P, P, P, P, P, I, I, I, I, F, P, P],
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
        "kllm_attn_generic": [P, P, P, P, P, P, I, I, I, I, I, I, I, I, I, I, F, P, I, I, P],
        "kllm_norm_residual": [P, P, I, L, P, P, P, I, I, I, F, P, P, I, P, P, I, I, F, P, P, P, I, L, P, P, F, F, P],
        "kllm_rope_tables_freq": [P, P, P, P, I, I, D, P],
        "kllm_qkv_norm_append": [P, I, L, P, P, P, I, I, I, F, P, P, P, P, P, I, I, I, I, I, I, I, I, P, P, P],
        "kllm_gate_bias": [P, I, L, P, P, I, I, I, I, F, F, P],
        "kllm_moe_tile_rows": [],
        "kllm_moe_route": [P, I, L, P, I, I, I, P, P, I, I, I, F, I, I, P, P],
        "kllm_moe_plan": [P, I, I, I, I, P, P, P],
        "kllm_moe_expert": [P, P, P, P, P, I, I, I, I, I, I, I, F, F, I, P],
        "kllm_moe_expert_rows": [P, P, P, P, I, I, I, I, I, I, I, F, F, I, P],
        "kllm_moe_combine": [P, P, P, P, P, I, L, P, I, I, I, I, I, P, P],
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
        "kllm_attn_decode": [P, P, P, L, P, P, P, P, I, I, I, I, I, I, I, I, I, I, F, P, I, I, P, I, P],
        "kllm_attn_prefill": [P, P, P, P, I, P, P, P, I, I, I, I, I, I, I, I, I, F, P, L, I, P, L, I, I, I, P],
        "kllm_attn_prefill_slices": [I, I, I],
        "kllm_gemm_act": [P, P, P, I, I, I, I, I, P, P],
        "kllm_add_sinusoid": [P, P, I, I, D, P],
        "kllm_unary_act": [P, I, L, I, P, I, I, I, I, P, P],
        "kllm_group_norm_add": [P, P, I, L, P, I, L, P, F, P, P, I, P, I, I, I, F, I, P],
        "kllm_qk_norm_append": [P, I, L, P, P, P, P, F, F, I, P, P, P, P, P, I, I, I, I, I, I, I, I, P, P, I, I, P],
        "kllm_delta_prep": [P, I, L, P, P, P, P, I, L, F, F, P, P, I, I, I, I, I, P],
        "kllm_delta_scan_max_dim": [],
        "kllm_delta_scan": [P, P, P, P, P, P, I, I, I, I, P],
        "kllm_delta_out": [P, P, P, F, P, I, I, I, I, P],
        "kllm_conv_state_update": [P, I, L, I, I, I, P, P, L, I, P, P, P, I, P],
        "kllm_gated_delta_prep": [P, I, L, P, I, P, L, P, P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, F, I, P, I, L, I, P, I, L,
                                  I, I, P, P],
        "kllm_gated_delta_max_dim": [],
        "kllm_gated_delta_scan": [P, P, P, P, P, P, L, P, P, P, I, I, I, I, I, P, P],
        "kllm_linear_recurrence_prep": [P, I, L, P, P, P, I, P, L, P, P, P, P, P, P, P, P, P, P, P, I, I, I, P],
        "kllm_linear_recurrence_scan": [P, P, P, I, L, P, P, L, P, P, P, P, I, I, I, P],
        "kllm_scaled_sum": [P, P, I, L, F, P, I, L, F, L, P],
        "kllm_normed_sum": [P, P, I, L, F, P, P, I, L, F, P, I, I, F, P],
        "kllm_latent_max_row": [],
        "kllm_latent_kv_append": [P, I, L, P, F, P, P, P, P, P, P, I, I, I, I, I, I, L, P],
        "kllm_latent_norm": [P, I, L, L, P, F, P, I, I, I, P],
        "kllm_latent_query": [P, I, L, P, P, P, P, I, I, I, I, I, I, I, P],
        "kllm_attn_latent": [P, P, P, P, P, P, I, I, I, I, I, I, F, I, I, P, L, I, P],
        "kllm_latent_out": [P, P, P, I, L, L, P, I, I, I, I, I, P],
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
             "kllm_attn_decode", "kllm_attn_prefill", "kllm_sample", "kllm_gemm_act", "kllm_add_sinusoid", "kllm_unary_act",
             "kllm_group_norm_add", "kllm_qk_norm_append", "kllm_delta_prep", "kllm_delta_scan", "kllm_delta_out",
             "kllm_norm_residual", "kllm_rope_tables_freq", "kllm_qkv_norm_append", "kllm_gate_bias", "kllm_moe_route",
             "kllm_moe_plan", "kllm_moe_expert", "kllm_moe_expert_rows", "kllm_moe_combine",
             "kllm_conv_state_update", "kllm_gated_delta_prep", "kllm_gated_delta_scan", "kllm_linear_recurrence_prep",
             "kllm_linear_recurrence_scan", "kllm_latent_kv_append", "kllm_latent_norm", "kllm_latent_query", "kllm_attn_latent",
             "kllm_latent_out", "kllm_scaled_sum", "kllm_normed_sum")
DYNAMIC_ARGS = {"kllm_attn_prefill": (19, 20)}     # arguments that may be a StepValue
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


def embed(out, table, ids, from_sampled=None, sampled=None, scale=1.0, copy=None):
    """out [n, d] = scale * table[ids]; where ``from_sampled[t] >= 0`` the id is
    ``sampled[from_sampled[t]]``, a token id still on the device.  ``copy`` [n, d] in the
    table's dtype receives the same rows."""
    n, d = out.shape
    if copy is not None and (tuple(copy.shape) != (n, d) or copy.dtype != table.dtype):
        raise KernelError("embed: the copy of the rows does not fit")
    if ids.numel() < n or table.shape[1] != d:
        raise KernelError(f"embed: out {tuple(out.shape)}, table {tuple(table.shape)}, "
                          f"{ids.numel()} ids do not fit")
    if (from_sampled is None) != (sampled is None) or (from_sampled is not None and from_sampled.numel() < n):
        raise KernelError("embed: from_sampled and sampled go together, one entry per token")
    _launch("kllm_embed", "embed", _ptr(out, "embed out", torch.float32), _ptr(table, "embed table"),
        _ptr(ids, "embed ids", torch.int32), _ptr(from_sampled, "embed from", torch.int32, True),
        _ptr(sampled, "embed sampled", torch.int32, True), n, d, table.shape[0], dtype_code(table.dtype),
        float(scale), _ptr(copy, "embed copy", None, True), _stream())


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


FUSED_LINEAR_UNARY = 16    # LINEAR_PARTS with act = this + an activation without a gate: see fused_linear


def fused_linear(w, y, kind, x, nsplit=1, tiles_per_wg=1, rope=None, act=ACT_SILU, resid=None, norm_weight=None,
                 ss_out=None, unary=None):
    """One launch for a decode batch's product of x [n, k] (bfloat16; a view
    with a row stride is taken) with w [m, k], and the step after it, by
    ``kind``: LINEAR_PARTS y float32 [nsplit, n, m]; LINEAR_SWIGLU y bfloat16
    [n, m/2]; LINEAR_ROPE y = q_out with ``rope`` describing rotation and
    cache; LINEAR_RESID adds the product to ``resid`` [n, m] float32 in place, writes
    y bfloat16 [n, m] = the new rows times ``norm_weight`` [m] and leaves partial sums of
    squares of the new rows in ``ss_out`` [n, fused_resid_parts rounded up to 4].  ``x`` may
    be a ``ScaledRows`` (SWIGLU and ROPE): what a LINEAR_RESID product left, see there.
    LINEAR_PARTS with ``unary`` = (activation without a gate, its float32 constants or None):
    y bfloat16 [n, m] = activation(sums), one slice."""
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
    if kind == LINEAR_PARTS and unary is not None:
        code, params = unary
        if nsplit != 1 or (code == ACT_XIELU and (params is None or params.numel() != 2)):
            raise KernelError("fused_linear: an activation on the sums takes one slice, and xielu its two constants")
        want, dt = (n, m), torch.bfloat16
        lo.act = FUSED_LINEAR_UNARY + int(code)
        lo.norm_w = _ptr(params, "fused_linear activation constants", torch.float32, True)
    elif kind == LINEAR_PARTS:
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


def _slopes(slopes, n_heads, who):
    """Pointer of the per-head slopes of a distance bias (float32 [heads]), or null for none."""
    if slopes is not None and slopes.numel() != n_heads:
        raise KernelError(f"{who}: {slopes.numel()} slopes for {n_heads} heads")
    return _ptr(slopes, who + " slopes", torch.float32, True)


def paged_cache_fits(cache, n_kv_heads, page_size, head_dim, value_dim):
    """Whether ``cache`` is a pool of pages for keys of ``head_dim`` and values of ``value_dim``:
    [pages, 2, KV, page_size * head_dim] where the two are equal, or flat pages of
    KV * page_size * (head_dim + value_dim) elements (keys [KV][slot][head_dim], then values
    [KV][value_dim][slot]: the same place for every element where the widths are equal)."""
    if cache.dim() == 4:
        return head_dim == value_dim and tuple(cache.shape[1:]) == (2, n_kv_heads, page_size * head_dim)
    return cache.dim() == 2 and cache.shape[1] == n_kv_heads * page_size * (head_dim + value_dim)


def attn_generic(q, out, cache, positions, span_of_token, block_table, page_size, n_heads,
                 n_kv_heads, head_dim, window, scale, slopes=None, value_dim=None, chunk=0, sink=False, keep_first=0):
    """``keep_first`` > 0: the first keep_first positions of a request stay readable behind the
    window.  ``slopes`` (here and in the other attention wrappers): float32 [heads] or None; slopes[h]
    times the distance from the query to the key is taken off head h's scaled scores.
    ``value_dim``: width of a value (default: the key's); ``chunk`` > 0: the query at position p
    reads no key before p - p % chunk; ``sink``: the softmax's denominator has one more term,
    exp(0)."""
    n = q.shape[0]
    vd = head_dim if value_dim is None else int(value_dim)
    if (tuple(q.shape) != (n, n_heads * head_dim) or tuple(out.shape) != (n, n_heads * vd)
            or q.dtype != cache.dtype or out.dtype != q.dtype):
        raise KernelError("attn_generic: q/out shapes or dtypes do not fit")
    if not paged_cache_fits(cache, n_kv_heads, page_size, head_dim, vd):
        raise KernelError(f"attn_generic: cache {tuple(cache.shape)} does not fit")
    if positions.numel() < n or span_of_token.numel() < n:
        raise KernelError("attn_generic: index arrays are too short")
    _launch("kllm_attn_generic", "attn_generic", _ptr(q, "attn q"), _ptr(out, "attn out"), _ptr(cache, "attn cache"),
        _ptr(positions, "attn positions", torch.int32),
        _ptr(span_of_token, "attn span_of_token", torch.int32),
        _ptr(block_table, "attn block_table", torch.int32), block_table.shape[1], page_size, n,
        n_heads, n_kv_heads, head_dim, vd, int(window), int(chunk), int(bool(sink)), float(scale),
        _slopes(slopes, n_heads, "attn_generic"), dtype_code(q.dtype), int(keep_first), _stream())


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
                 nslices=None, slopes=None, chunk=0, sink=False, keep_first=0):
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
        n_heads, n_kv_heads, head_dim, int(window), int(chunk), int(bool(sink)), int(keep_first), float(scale),
        _slopes(slopes, n_heads, "attn_prefill"),
        keys_total if type(keys_total) is StepValue else int(keys_total),
        keys_longest if type(keys_longest) is StepValue else int(keys_longest),
        _ptr(part, "attn part", torch.float32, True) if nslices > 1 else 0, need, nslices, n,
        dtype_code(q.dtype), _stream())


def attn_decode(q, out, part, cache, positions, span_of_token, block_table, page_size, n_heads,
                n_kv_heads, head_dim, window, scale, nslices, token_list=None, n_listed=0, slopes=None, chunk=0,
                sink=False, keep_first=0):
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
        n_heads, n_kv_heads, head_dim, int(window), int(chunk), int(bool(sink)), int(keep_first), float(scale),
        _slopes(slopes, n_heads, "attn_decode"),
        int(nslices), dtype_code(q.dtype),
        _ptr(token_list, "attn token_list", torch.int32, True), int(n_listed), _stream())


def sample(out, logits, temperature=None, uniform=None):
    rows, vocab = logits.shape
    if out.numel() < rows:
        raise KernelError("sample: output is too short")
    _launch("kllm_sample", "sample", _ptr(out, "sample out", torch.int32), _ptr(logits, "sample logits", torch.float32),
        _ptr(temperature, "sample temperature", torch.float32, True),
        _ptr(uniform, "sample uniform", torch.float32, True), rows, vocab, _stream())


# ----------------------------------------------------------------------------- steps of other layer designs

def add_sinusoid(x, positions, base=10000.0):
    """x [n, d] float32 += the sinusoidal position vector: channel 2i gets sin, 2i + 1 cos of
    positions[t] * base^(-2i/d)."""
    n, d = x.shape
    if positions.numel() < n:
        raise KernelError("add_sinusoid: positions are too short")
    _launch("kllm_add_sinusoid", "add_sinusoid", _ptr(x, "add_sinusoid x", torch.float32),
            _ptr(positions, "add_sinusoid positions", torch.int32), n, d, float(base), _stream())


ACT_XIELU, ACT_TANH, ACT_RELU_SQ, ACT_IDENTITY, ACT_SIGMOID = 2, 3, 4, 5, 6
UNARY_ACTIVATIONS = dict(ACTIVATIONS, xielu=ACT_XIELU, tanh=ACT_TANH, relu2=ACT_RELU_SQ, identity=ACT_IDENTITY,
                         sigmoid=ACT_SIGMOID)


def _splits(t, n, cols, who):
    """(nsplit, stride) of float32 sums [nsplit, n, cols] or [n, cols]."""
    if t.dtype != torch.float32 or t.shape[-1] != cols or t.shape[-2] != n or t.dim() not in (2, 3):
        raise KernelError(f"{who}: sums {tuple(t.shape)} {t.dtype} do not fit {n} x {cols} float32")
    return (t.shape[0], n * cols) if t.dim() == 3 else (1, 0)


def unary_act(sums, out, act, params=None, first_column=0):
    """out [n, f] = act(sums summed over their slices); ``params``: float32 [2], the learned
    constants of an activation that has them.  With ``first_column`` the f columns from there
    of wider sums are taken."""
    n, f = out.shape
    cols = sums.shape[-1]
    nsplit, stride = _splits(sums, n, cols, "unary_act")
    if first_column < 0 or first_column + f > cols or (first_column == 0 and cols != f):
        raise KernelError(f"unary_act: columns {first_column} .. {first_column + f} of {cols}")
    if act == ACT_XIELU and (params is None or params.numel() != 2):
        raise KernelError("unary_act: xielu needs its two constants")
    _launch("kllm_unary_act", "unary_act", _ptr(sums, "unary_act in", torch.float32) + 4 * int(first_column), nsplit,
            stride, cols, _ptr(out, "unary_act out"), dtype_code(out.dtype), n, f, int(act),
            _ptr(params, "unary_act params", torch.float32, True), _stream())


def gemm_act(x, w, h, act, params=None):
    """h [n, m] = act(x . w^T) on the MFMA tiles, the activation (one without a gate) in the
    product's epilogue; h in the dtype of x and w."""
    n, k = x.shape
    m = w.shape[0]
    if w.shape[1] != k or x.dtype != w.dtype or tuple(h.shape) != (n, m) or h.dtype != x.dtype:
        raise KernelError(f"gemm_act: x {tuple(x.shape)}, w {tuple(w.shape)}, h {tuple(h.shape)} do not fit")
    if act == ACT_XIELU and (params is None or params.numel() != 2):
        raise KernelError("gemm_act: xielu needs its two constants")
    _launch("kllm_gemm_act", "gemm_act", _ptr(x, "gemm_act x"), _ptr(w, "gemm_act w"), _ptr(h, "gemm_act h"), n, m, k,
            dtype_code(x.dtype), int(act), _ptr(params, "gemm_act params", torch.float32, True), _stream())


def group_norm_add(x, deltas=(), bias=None, mult=1.0, weight=None, out=None, rows=None, groups=1, eps=0.0,
                   write_x=None):
    """x [N, d] float32; v = x + mult * (the deltas' slices summed + bias), written back to x
    (unless ``rows`` selects rows to read); out [n, d] = v normalised in ``groups`` groups of
    channels, times weight.  ``deltas``: up to two float32 tensors [N, d] or [nsplit, N, d]."""
    N, d = x.shape
    deltas = [t for t in deltas if t is not None]
    if len(deltas) > 2:
        raise KernelError("group_norm_add: at most two sums")
    n = rows.numel() if rows is not None else N
    if write_x is None:
        write_x = rows is None and (bool(deltas) or bias is not None)
    if out is not None and (tuple(out.shape) != (n, d) or weight is None or weight.numel() != d):
        raise KernelError("group_norm_add: output or weight shape does not fit")
    if bias is not None and bias.numel() != d:
        raise KernelError("group_norm_add: bias does not fit")
    args = []
    for t in deltas + [None] * (2 - len(deltas)):
        if t is None:
            args += [0, 0, 0]
        else:
            ns, st = _splits(t, N, d, "group_norm_add")
            args += [_ptr(t, "group_norm_add delta", torch.float32), ns, st]
    _launch("kllm_group_norm_add", "group_norm_add", _ptr(x, "group_norm_add x", torch.float32), *args,
            _ptr(bias, "group_norm_add bias", torch.float32, True), float(mult),
            _ptr(weight, "group_norm_add weight", torch.float32, True), _ptr(out, "group_norm_add out", None, True),
            dtype_code(out.dtype) if out is not None else DT_F32, _ptr(rows, "group_norm_add rows", torch.int32, True),
            n, d, int(groups), float(eps), int(bool(write_x)), _stream())


def qk_norm_append(qk, q_out, cache, positions, span_of_token, block_table, page_size, n_heads, n_kv_heads,
                   head_dim, q_bias=None, k_bias=None, q_weight=None, k_weight=None, eps=0.0, temp_coef=0.0,
                   temp_every=0, value_dim=0, cos=None, sin=None, rotary_dim=0, interleaved=False):
    """qk: float32 sums [nsplit, n, (H + KV) * hd + KV * value_dim] of the query, key and value
    products.  Adds the biases, normalises the whole query row and the whole key row (RMS, times
    their weights), turns the first ``rotary_dim`` elements of every head (cos, sin [n, rotary_dim /
    2]), scales the query by 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1), writes q_out and
    appends to the pages.  ``value_dim`` 0: the values are the keys (the normalised key is cached
    as the key, the key before its norm as the value)."""
    n = q_out.shape[0]
    qd, kd = n_heads * head_dim, n_kv_heads * head_dim
    nsplit, stride = _splits(qk, n, qd + kd + n_kv_heads * value_dim, "qk_norm_append")
    rot = int(rotary_dim) if cos is not None else 0
    if cos is not None and (tuple(cos.shape) != (n, rot // 2) or tuple(sin.shape) != tuple(cos.shape)):
        raise KernelError("qk_norm_append: cos/sin shapes do not fit")
    if q_out.shape[1] != qd:
        raise KernelError("qk_norm_append: q_out does not fit")
    for t, size in ((q_bias, qd), (k_bias, kd), (q_weight, qd), (k_weight, kd)):
        if t is not None and t.numel() != size:
            raise KernelError("qk_norm_append: a bias or norm weight does not fit")
    max_pages = 0
    if cache is not None:
        if (not paged_cache_fits(cache, n_kv_heads, page_size, head_dim, value_dim or head_dim)
                or cache.dtype != q_out.dtype):
            raise KernelError(f"qk_norm_append: cache {tuple(cache.shape)} {cache.dtype} does not fit")
        max_pages = block_table.shape[1]
        if span_of_token.numel() < n:
            raise KernelError("qk_norm_append: index arrays are too short")
    if positions.numel() < n:
        raise KernelError("qk_norm_append: index arrays are too short")
    F32 = torch.float32
    _launch("kllm_qk_norm_append", "qk_norm_append", _ptr(qk, "qk_norm_append qk", F32), nsplit, stride,
            _ptr(q_bias, "qk_norm_append q bias", F32, True), _ptr(k_bias, "qk_norm_append k bias", F32, True),
            _ptr(q_weight, "qk_norm_append q weight", F32, True), _ptr(k_weight, "qk_norm_append k weight", F32, True),
            float(eps), float(temp_coef), int(temp_every), _ptr(q_out, "qk_norm_append q_out"),
            _ptr(cache, "qk_norm_append cache", None, True), _ptr(positions, "qk_norm_append positions", torch.int32),
            _ptr(span_of_token, "qk_norm_append span_of_token", torch.int32, True),
            _ptr(block_table, "qk_norm_append block_table", torch.int32, True), max_pages, page_size, n,
            n_heads, n_kv_heads, head_dim, dtype_code(q_out.dtype), int(value_dim),
            _ptr(cos, "qk_norm_append cos", F32, True), _ptr(sin, "qk_norm_append sin", F32, True), rot,
            1 if interleaved else 0, _stream())


DELTA_SCAN_FIELDS = 6      # per token and head the recurrence reads r, k, v, w, u, a*u


def delta_scan_max_dim() -> int:
    return limit("delta_scan_max_dim")


def delta_prep(proj, a_bias, w2, w0, decay_scale, key_eps, scan_in, gate, heads, head_dim, low=None):
    """proj: float32 sums [nsplit, n, 5*H*hd + L] of the products r | k | v | g | a | w1; writes
    what the recurrence reads, scan_in [H, n, 6, hd], and gate [n, H*hd] = sigmoid(g).  ``low``:
    float32 sums [slices, n, H*hd] of w2 . tanh(w1 part) where a matrix kernel made them (the
    kernel then leaves that product alone)."""
    n, HD = gate.shape
    L = w2.shape[1]
    nsplit, stride = _splits(proj, n, 5 * HD + L, "delta_prep")
    low_ns, low_st = _splits(low, n, HD, "delta_prep low") if low is not None else (0, 0)
    if (HD != heads * head_dim or tuple(scan_in.shape) != (heads, n, DELTA_SCAN_FIELDS, head_dim)
            or w2.shape[0] != HD or a_bias.numel() != HD or w0.numel() != HD):
        raise KernelError("delta_prep: shapes do not fit")
    F32 = torch.float32
    _launch("kllm_delta_prep", "delta_prep", _ptr(proj, "delta_prep proj", F32), nsplit, stride,
            _ptr(a_bias, "delta_prep a bias", F32), _ptr(w2, "delta_prep w2"), _ptr(w0, "delta_prep w0", F32),
            _ptr(low, "delta_prep low", F32, True), low_ns, low_st, float(decay_scale), float(key_eps), _ptr(scan_in, "delta_prep scan_in", F32),
            _ptr(gate, "delta_prep gate", F32), n, heads, head_dim, L, dtype_code(w2.dtype), _stream())


def delta_scan(scan_in, o_out, state, slots, span_start, span_pos, n_spans):
    """The recurrence, each request through its state: scan_in [H, n, 6, hd], o_out [n, H*hd], state
    [slots, H, hd, hd] float32 (started from zero where a span's position is 0)."""
    H, n, _, hd = scan_in.shape
    if (tuple(o_out.shape) != (n, H * hd) or tuple(state.shape[1:]) != (H, hd, hd) or state.dtype != torch.float32
            or slots.numel() < n_spans or span_start.numel() < n_spans + 1 or span_pos.numel() < n_spans):
        raise KernelError("delta_scan: shapes do not fit")
    F32, I32 = torch.float32, torch.int32
    _launch("kllm_delta_scan", "delta_scan", _ptr(scan_in, "delta_scan in", F32), _ptr(o_out, "delta_scan out", F32),
            _ptr(state, "delta_scan state", F32), _ptr(slots, "delta_scan slots", I32),
            _ptr(span_start, "delta_scan span_start", I32), _ptr(span_pos, "delta_scan span_pos", I32),
            int(n_spans), n, H, hd, _stream())


def delta_out(o, gate, weight, eps, out, heads, head_dim):
    """out [n, H*hd] = each head of o divided by its root mean square, times weight, times gate."""
    n = o.shape[0]
    if (tuple(o.shape) != (n, heads * head_dim) or tuple(gate.shape) != tuple(o.shape)
            or tuple(out.shape) != tuple(o.shape) or weight.numel() != heads * head_dim):
        raise KernelError("delta_out: shapes do not fit")
    F32 = torch.float32
    _launch("kllm_delta_out", "delta_out", _ptr(o, "delta_out o", F32), _ptr(gate, "delta_out gate", F32),
            _ptr(weight, "delta_out weight", F32), float(eps), _ptr(out, "delta_out out"), n, heads, head_dim,
            dtype_code(out.dtype), _stream())


# ----------------------------------------------------------------------------- norm behind the sub-layer, rotation then unit norm, routed experts

class NormedPair:
    """What two sub-layers that ran side by side leave for the norm behind them: ``scale_a *
    weight_a * N(a) + scale_b * weight_b * N(b)``, each of the float32 sums ``a`` and ``b`` ([n, d] or
    [slices, n, d]) normed over the row (with the eps of the norm that takes the pair)."""

    def __init__(self, a, scale_a, weight_a, b, scale_b, weight_b):
        self.a, self.scale_a, self.weight_a, self.b, self.scale_b, self.weight_b = a, float(scale_a), weight_a, b, float(scale_b), weight_b


class ChosenSums:
    """What a routed feed-forward leaves for the norm behind it to add up: per token the weighted
    sum over its choices of ``y`` [n * top, d] (float32), or of ``xin`` [n, d] where the chosen
    expert is an identity (``idx`` >= ``experts``), plus the slices of ``shared`` (or None), each
    token's times ``shared_scale`` [n] (or None: one)."""

    def __init__(self, y, xin, idx, wgt, experts, shared=None, shared_scale=None):
        self.y, self.xin, self.idx, self.wgt, self.experts, self.shared = y, xin, idx, wgt, int(experts), shared
        self.shared_scale = shared_scale


def norm_residual(x, weight, delta=None, bias=None, out=None, eps=0.0, mult=1.0, next_weight=None, delta_scale=None):
    """x [n, d] float32 in place.  With ``delta`` (float32 [n, d] or [nsplit, n, d], or a
    ``ChosenSums``; ``bias`` [d] is added to it): x += mult * weight * N(delta + bias); without: x =
    weight * N(x), where N divides a row by sqrt(mean of its squares + eps).  ``out`` [n, d]
    receives the new x in its own dtype, or, with ``next_weight`` [d], next_weight * N(new x): the
    norm in front of the next sub-layer.  ``delta_scale`` [n]: a factor per row on delta."""
    n, d = x.shape
    chosen = pair = None
    if isinstance(delta, ChosenSums):
        chosen, delta = delta, delta.shared
        delta_scale = chosen.shared_scale if delta_scale is None else delta_scale
        top = chosen.idx.shape[1]
        if (tuple(chosen.y.shape) != (n * top, d) or tuple(chosen.xin.shape) != (n, d)
                or tuple(chosen.wgt.shape) != (n, top)):
            raise KernelError("norm_residual: the chosen experts' sums do not fit")
    elif isinstance(delta, NormedPair):
        pair, delta = delta, delta.a
        pair_nb, pair_stride = _splits(pair.b, n, d, "norm_residual pair")
        if pair.weight_a.numel() != d or pair.weight_b.numel() != d:
            raise KernelError("norm_residual: the pair's weights do not fit")
    nsplit, stride = (1, 0) if delta is None else _splits(delta, n, d, "norm_residual")
    if weight.numel() != d or (bias is not None and bias.numel() != d) or (out is not None and tuple(out.shape) != (n, d)):
        raise KernelError("norm_residual: weight, bias or output does not fit")
    if (next_weight is not None and (next_weight.numel() != d or out is None)) or (
            delta_scale is not None and (delta_scale.numel() != n or delta is None)):
        raise KernelError("norm_residual: the next norm's weight or the rows' factors do not fit")
    F32 = torch.float32
    _launch("kllm_norm_residual", "norm_residual", _ptr(x, "norm_residual x", F32),
            _ptr(delta, "norm_residual delta", F32, True), nsplit, stride, _ptr(bias, "norm_residual bias", F32, True),
            _ptr(weight, "norm_residual weight", F32), _ptr(out, "norm_residual out", None, True),
            dtype_code(out.dtype) if out is not None else DT_F32, n, d, float(eps),
            _ptr(chosen.y, "norm_residual y", F32) if chosen else 0, _ptr(chosen.xin, "norm_residual xin") if chosen else 0,
            dtype_code(chosen.xin.dtype) if chosen else DT_F32,
            _ptr(chosen.idx, "norm_residual idx", torch.int32) if chosen else 0,
            _ptr(chosen.wgt, "norm_residual wgt", F32) if chosen else 0, chosen.idx.shape[1] if chosen else 0,
            chosen.experts if chosen else 0, float(mult), _ptr(next_weight, "norm_residual next weight", F32, True),
            _ptr(delta_scale, "norm_residual delta scale", F32, True),
            _ptr(pair.b, "norm_residual pair b", F32) if pair else 0, pair_nb if pair else 0, pair_stride if pair else 0,
            _ptr(pair.weight_a, "norm_residual pair weight", F32) if pair else 0,
            _ptr(pair.weight_b, "norm_residual pair weight", F32) if pair else 0, pair.scale_a if pair else 0.0,
            pair.scale_b if pair else 0.0, _stream())


def rope_tables_freq(cos, sin, positions, freq, factor=1.0):
    """cos, sin [n, half] = factor * cos/sin(positions[t] * freq[i]); freq: float64 [half]."""
    n, half = cos.shape
    if tuple(sin.shape) != (n, half) or freq.numel() != half or positions.numel() < n:
        raise KernelError("rope_tables_freq: table shapes do not fit")
    _launch("kllm_rope_tables_freq", "rope_tables_freq", _ptr(cos, "rope cos", torch.float32),
            _ptr(sin, "rope sin", torch.float32), _ptr(positions, "rope positions", torch.int32),
            _ptr(freq, "rope freq", torch.float64), n, half, float(factor), _stream())


def qkv_norm_append(qkv, q_out, cache, positions, span_of_token, block_table, page_size, n_heads, n_kv_heads,
                    head_dim, value_dim, bias=None, cos=None, sin=None, rotary_dim=0, interleaved=True,
                    unit_norm=True, eps=0.0, q_weight=None, k_weight=None):
    """qkv: float32 sums [nsplit, n, (H + KV) * head_dim + KV * value_dim].  Adds ``bias``, rotates the
    first ``rotary_dim`` elements of every query and key head (cos, sin [n, rotary_dim / 2]),
    divides every query and key head by its root mean square (``unit_norm``), writes q_out and
    appends keys and values to the pages.  With ``q_weight`` and ``k_weight`` (float32 [head_dim], shared
    by the heads) the norm stands in front of the rotation and has these weights."""
    n = q_out.shape[0]
    cols = (n_heads + n_kv_heads) * head_dim + n_kv_heads * value_dim
    nsplit, stride = _splits(qkv, n, cols, "qkv_norm_append")
    if q_out.shape[1] != n_heads * head_dim or (bias is not None and bias.numel() != cols):
        raise KernelError("qkv_norm_append: q_out or bias does not fit")
    if not paged_cache_fits(cache, n_kv_heads, page_size, head_dim, value_dim) or cache.dtype != q_out.dtype:
        raise KernelError(f"qkv_norm_append: cache {tuple(cache.shape)} {cache.dtype} does not fit")
    if positions.numel() < n or span_of_token.numel() < n:
        raise KernelError("qkv_norm_append: index arrays are too short")
    rot = int(rotary_dim) if cos is not None else 0
    if cos is not None and (tuple(cos.shape) != (n, rot // 2) or tuple(sin.shape) != tuple(cos.shape)):
        raise KernelError("qkv_norm_append: cos/sin shapes do not fit")
    if (q_weight is None) != (k_weight is None) or (q_weight is not None and (q_weight.numel() != head_dim
                                                                              or k_weight.numel() != head_dim)):
        raise KernelError("qkv_norm_append: the norms' weights do not fit")
    F32 = torch.float32
    _launch("kllm_qkv_norm_append", "qkv_norm_append", _ptr(qkv, "qkv_norm_append qkv", F32), nsplit, stride,
            _ptr(bias, "qkv_norm_append bias", F32, True), _ptr(cos, "qkv_norm_append cos", F32, True),
            _ptr(sin, "qkv_norm_append sin", F32, True), rot, int(bool(interleaved)), int(bool(unit_norm)), float(eps),
            _ptr(q_out, "qkv_norm_append q_out"), _ptr(cache, "qkv_norm_append cache"),
            _ptr(positions, "qkv_norm_append positions", torch.int32),
            _ptr(span_of_token, "qkv_norm_append span_of_token", torch.int32),
            _ptr(block_table, "qkv_norm_append block_table", torch.int32), block_table.shape[1], page_size, n,
            n_heads, n_kv_heads, head_dim, value_dim, dtype_code(q_out.dtype),
            _ptr(q_weight, "qkv_norm_append q weight", F32, True), _ptr(k_weight, "qkv_norm_append k weight", F32, True),
            _stream())


GATE_CLAMPED_SWISH = 4     # g' = min(g, limit), u' = clamp(u, -limit, limit): g' sigmoid(alpha g') (u' + 1)
GATES = dict(ACTIVATIONS, clamped_swish=GATE_CLAMPED_SWISH)


def gate_bias(gu, out, act=ACT_SILU, bias=None, limit=0.0, alpha=1.0):
    """out [n, f] = gated(gu[:, :f] + bias[:f], gu[:, f:] + bias[f:]); gu float32 sums [nsplit, n, 2f]."""
    n, f = out.shape
    nsplit, stride = _splits(gu, n, 2 * f, "gate_bias")
    if bias is not None and bias.numel() != 2 * f:
        raise KernelError("gate_bias: bias does not fit")
    _launch("kllm_gate_bias", "gate_bias", _ptr(gu, "gate_bias in", torch.float32), nsplit, stride,
            _ptr(bias, "gate_bias bias", torch.float32, True), _ptr(out, "gate_bias out"), dtype_code(out.dtype), n, f,
            int(act), float(limit), float(alpha), _stream())


def moe_tile_rows() -> int:
    return limit("moe_tile_rows")


def moe_max_tiles(entries, experts, tile_rows=None) -> int:
    """Tiles of ``tile_rows`` rows that always hold ``entries`` (token, choice) pairs of ``experts`` experts."""
    return -(-entries // (tile_rows or moe_tile_rows())) + experts


def moe_best_tile_rows(entries, experts) -> int:
    """Rows of a tile for this many entries: the large tiles (twice ``moe_tile_rows()``, as many
    columns) from where an expert's share fills one, the small ones below."""
    small = moe_tile_rows()
    return 2 * small if entries >= 2 * small * experts else small


MOE_MAX_GROUPS = 64      # groups of experts a router may choose among


def moe_route(z, correction, idx, wgt, experts=None, scoring="softmax", groups=1, keep_groups=1, scale=1.0,
              renormalize=True, shared_gate=None):
    """z: float32 sums [nsplit, n, cols] of the router, the first ``experts`` (default: all) of a row
    the experts'; idx int32, wgt float32 [n, top].  ``scoring``: "softmax" or "sigmoid";
    ``groups`` > 1: only experts of the ``keep_groups`` best of that many equal groups of
    neighbours are chosen; the weights are the chosen scores, divided by their sum if
    ``renormalize``, times ``scale``.  ``shared_gate`` [n] receives the logistic function of the
    sum behind the experts' (column ``experts``)."""
    n, top = idx.shape
    cols = z.shape[-1]
    R = cols if experts is None else int(experts)
    nsplit, stride = _splits(z, n, cols, "moe_route")
    if scoring not in ("softmax", "sigmoid"):
        raise KernelError(f"moe_route: scoring {scoring!r} is not built (softmax, sigmoid)")
    if (tuple(wgt.shape) != (n, top) or (correction is not None and correction.numel() != R)
            or cols < R + (1 if shared_gate is not None else 0)
            or (shared_gate is not None and shared_gate.numel() != n)):
        raise KernelError("moe_route: outputs or correction do not fit")
    _launch("kllm_moe_route", "moe_route", _ptr(z, "moe_route z", torch.float32), nsplit, stride,
            _ptr(correction, "moe_route correction", torch.float32, True), n, R, top,
            _ptr(idx, "moe_route idx", torch.int32), _ptr(wgt, "moe_route wgt", torch.float32),
            0 if scoring == "softmax" else 1, int(groups), int(keep_groups), float(scale), 1 if renormalize else 0,
            cols, _ptr(shared_gate, "moe_route shared gate", torch.float32, True), _stream())


def moe_plan(idx, experts, sorted_entries, tiles, tile_rows=None):
    entries = idx.numel()
    tile_rows = int(tile_rows or moe_tile_rows())
    if sorted_entries.numel() < entries or tiles.dim() != 2 or tiles.shape[1] != 3:
        raise KernelError("moe_plan: outputs do not fit")
    _launch("kllm_moe_plan", "moe_plan", _ptr(idx, "moe_plan idx", torch.int32), entries, int(experts), tiles.shape[0],
            tile_rows, _ptr(sorted_entries, "moe_plan sorted", torch.int32), _ptr(tiles, "moe_plan tiles", torch.int32), _stream())


def moe_expert(x, w, out, sorted_entries, tiles, top, mode, act=ACT_SILU, limit=0.0, alpha=1.0, tile_rows=None):
    """mode 0: x [tokens, k], w [E, 2m, k] -> out [tokens * top, m] gated, in x's dtype;
    mode 1: x [tokens * top, k], w [E, m, k] -> out [tokens * top, m] float32."""
    k = x.shape[1]
    m = out.shape[1]
    if (w.dim() != 3 or w.shape[2] != k or w.shape[1] != (2 * m if mode == 0 else m) or w.dtype != x.dtype
            or out.dtype != (x.dtype if mode == 0 else torch.float32)
            or out.shape[0] != (x.shape[0] * top if mode == 0 else x.shape[0]) or sorted_entries.numel() < out.shape[0]):
        raise KernelError(f"moe_expert: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
    _launch("kllm_moe_expert", "moe_expert", _ptr(x, "moe_expert x"), _ptr(w, "moe_expert w"), _ptr(out, "moe_expert out"),
            _ptr(sorted_entries, "moe_expert sorted", torch.int32), _ptr(tiles, "moe_expert tiles", torch.int32),
            tiles.shape[0], int(tile_rows or moe_tile_rows()), int(top), m, k, int(mode), int(act), float(limit),
            float(alpha), dtype_code(x.dtype), _stream())


MOE_ROWS_BEST_ENTRIES = 16     # (token, choice) pairs up to which the entry-by-entry products beat the tiles


def moe_expert_rows(x, w, out, idx, experts, mode, act=ACT_SILU, limit=0.0, alpha=1.0):
    """``moe_expert`` entry by entry, without a plan: idx int32 [tokens, top] names each entry's
    expert; entries of experts from ``experts`` on are skipped."""
    k, m, top = x.shape[1], out.shape[1], idx.shape[1]
    entries = idx.numel()
    if (w.dim() != 3 or w.shape[2] != k or w.shape[1] != (2 * m if mode == 0 else m) or w.dtype != x.dtype
            or out.dtype != (x.dtype if mode == 0 else torch.float32) or out.shape[0] != entries
            or x.shape[0] != (entries // top if mode == 0 else entries)):
        raise KernelError(f"moe_expert_rows: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
    _launch("kllm_moe_expert_rows", "moe_expert_rows", _ptr(x, "moe_expert_rows x"), _ptr(w, "moe_expert_rows w"),
            _ptr(out, "moe_expert_rows out"), _ptr(idx, "moe_expert_rows idx", torch.int32), entries, int(experts), top,
            m, k, int(mode), int(act), float(limit), float(alpha), dtype_code(x.dtype), _stream())


def moe_combine(y, xin, idx, wgt, out, experts, shared=None, shared_scale=None):
    """out [n, d] float32 = sum over choices of wgt * (idx < experts ? y[token * top + choice] : xin[token])
    + the slices of ``shared`` (float32 [n, d] or [ns, n, d]), each token's times ``shared_scale`` [n]."""
    n, d = out.shape
    top = idx.shape[1]
    ns, stride = (0, 0)
    if shared is not None:
        ns, stride = _splits(shared, n, d, "moe_combine")
    if tuple(y.shape) != (n * top, d) or tuple(xin.shape) != (n, d) or tuple(wgt.shape) != (n, top):
        raise KernelError("moe_combine: shapes do not fit")
    _launch("kllm_moe_combine", "moe_combine", _ptr(y, "moe_combine y", torch.float32), _ptr(xin, "moe_combine x"),
            _ptr(idx, "moe_combine idx", torch.int32), _ptr(wgt, "moe_combine wgt", torch.float32),
            _ptr(shared, "moe_combine shared", torch.float32, True), ns, stride,
            _ptr(out, "moe_combine out", torch.float32), n, d, top, int(experts), dtype_code(xin.dtype),
            _ptr(shared_scale if shared is not None else None, "moe_combine shared scale", torch.float32, True), _stream())


# ----------------------------------------------------------------------------- recurrent mixers with a short convolution

def _field(state, offset, who):
    """Address of a field of the per-slot state: ``state`` [slots, floats] float32, the field
    ``offset`` floats into a slot.  Returns (address in slot 0, floats per slot)."""
    if state.dim() != 2 or state.dtype != torch.float32 or not 0 <= offset <= state.shape[1]:
        raise KernelError(f"{who}: state {tuple(state.shape)} {state.dtype}, field at {offset}")
    return _ptr(state, who + " state", torch.float32) + 4 * int(offset), int(state.shape[1])


def conv_state_update(proj, col0, channels, taps, state, offset, slots, span_start, span_pos, n_spans, in_bias=None):
    """The convolution's field of the state ([channels, taps - 1] per slot, ``offset`` floats into
    it) takes the inputs of every span's last taps - 1 positions: columns col0 .. col0 + channels
    of the float32 sums ``proj`` [nsplit, n, cols] (plus ``in_bias`` [channels]); where a span is
    shorter, the entries it had move up (zeros where the span starts at position 0)."""
    n, cols = proj.shape[-2], proj.shape[-1]
    nsplit, stride = _splits(proj, n, cols, "conv_state_update")
    if taps <= 1:
        return
    addr, per_slot = _field(state, offset, "conv_state_update")
    if (offset + channels * (taps - 1) > per_slot or col0 + channels > cols or slots.numel() < n_spans
            or span_start.numel() < n_spans + 1 or (in_bias is not None and in_bias.numel() != channels)):
        raise KernelError("conv_state_update: sizes do not fit")
    I32 = torch.int32
    _launch("kllm_conv_state_update", "conv_state_update", _ptr(proj, "conv proj", torch.float32), nsplit, stride, cols,
            int(col0), int(channels), _ptr(in_bias, "conv bias", torch.float32, True), addr, per_slot, int(taps),
            _ptr(slots, "conv slots", I32), _ptr(span_start, "conv span_start", I32), _ptr(span_pos, "conv span_pos", I32),
            int(n_spans), _stream())


def gated_delta_max_dim() -> int:
    return limit("gated_delta_max_dim")


def gated_delta_prep(proj, conv_w, taps, state, conv_offset, a_log, dt_bias, span_of_token, slots, span_start, span_pos,
                     qn, kn, vv, gb, gate, heads, kv_heads, dim, vdim, unit_eps=1e-6, a_sums=None, decays=None,
                     gate_sums=None, gate_sigmoid=False, low_sums=None):
    """proj: float32 sums [nsplit, n, 2 G dk + 2 H dv + 2 H (or more)] of q | k | v | b | a | gate.
    Convolution (conv_w [2 G dk + H dv, taps], its earlier inputs from the state's field at
    ``conv_offset``) and SiLU of q, k, v; q and k to unit vectors per head, q times dk^-1/2; gb [n, 2,
    H] = (exp(-exp(a_log) softplus(a + dt_bias)), sigmoid(b)); gate [n, H dv] = silu (``gate_sigmoid``:
    the logistic function) of the gate's sums.  With ``a_sums`` (float32 sums [slices, n, H dk]) the
    decay has one number per head and key channel (dt_bias [H dk]), written to ``decays`` [n, H dk],
    and proj has no a columns; with ``gate_sums`` ([slices, n, H dv]) proj has no gate columns.
    ``low_sums`` ([slices, n, H dk + H dv]) is both in one: the decays' sums, then the gates'."""
    n = qn.shape[0]
    QK, HV = kv_heads * dim, heads * vdim
    C = 2 * QK + HV
    cols = proj.shape[-1]
    nsplit, stride = _splits(proj, n, cols, "gated_delta_prep")
    addr, per_slot = _field(state, conv_offset, "gated_delta_prep")
    F32, I32 = torch.float32, torch.int32
    a_ptr = g_ptr = a_row = g_row = 0
    if low_sums is not None:
        if a_sums is not None or gate_sums is not None:
            raise KernelError("gated_delta_prep: the decays' and gates' sums come together or apart")
        a_row = g_row = heads * dim + HV
        a_ns, a_st = g_ns, g_st = _splits(low_sums, n, a_row, "gated_delta_prep low")
        a_ptr = _ptr(low_sums, "gated_delta low sums", F32)
        g_ptr = a_ptr + 4 * heads * dim
        a_sums = gate_sums = low_sums
    else:
        a_ns, a_st = _splits(a_sums, n, heads * dim, "gated_delta_prep a") if a_sums is not None else (0, 0)
        g_ns, g_st = _splits(gate_sums, n, HV, "gated_delta_prep gate") if gate_sums is not None else (0, 0)
        a_ptr, a_row = _ptr(a_sums, "gated_delta a sums", F32, True), heads * dim
        g_ptr, g_row = _ptr(gate_sums, "gated_delta gate sums", F32, True), HV
    need = C + (heads if a_sums is not None else 2 * heads) + (0 if gate_sums is not None else HV)
    if (tuple(conv_w.shape) != (C, taps) or a_log.numel() != heads or cols < need
            or dt_bias.numel() != (heads * dim if a_sums is not None else heads)
            or (a_sums is None) != (decays is None) or (decays is not None and tuple(decays.shape) != (n, heads * dim))
            or tuple(qn.shape) != (n, QK) or tuple(kn.shape) != (n, QK) or tuple(vv.shape) != (n, HV)
            or tuple(gb.shape) != (n, 2, heads) or tuple(gate.shape) != (n, HV)
            or conv_offset + C * (taps - 1) > per_slot or span_of_token.numel() < n):
        raise KernelError("gated_delta_prep: shapes do not fit")
    _launch("kllm_gated_delta_prep", "gated_delta_prep", _ptr(proj, "gated_delta proj", F32), nsplit, stride,
            _ptr(conv_w, "gated_delta conv", F32), int(taps), addr, per_slot, _ptr(a_log, "gated_delta A", F32),
            _ptr(dt_bias, "gated_delta dt", F32), _ptr(span_of_token, "gated_delta span_of_token", I32),
            _ptr(slots, "gated_delta slots", I32), _ptr(span_start, "gated_delta span_start", I32),
            _ptr(span_pos, "gated_delta span_pos", I32), _ptr(qn, "gated_delta qn", F32), _ptr(kn, "gated_delta kn", F32),
            _ptr(vv, "gated_delta v", F32), _ptr(gb, "gated_delta gb", F32), _ptr(gate, "gated_delta gate", F32), n,
            int(heads), int(kv_heads), int(dim), int(vdim), float(unit_eps), int(cols),
            a_ptr, a_ns, a_st, a_row, g_ptr, g_ns, g_st, g_row, 1 if gate_sigmoid else 0, _ptr(decays, "gated_delta decays", F32, True), _stream())


def gated_delta_scan(qn, kn, vv, gb, o_out, state, offset, slots, span_start, span_pos, n_spans, heads, kv_heads, dim,
                     vdim, decays=None):
    """S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, each request through its state
    ([heads, dim, vdim] float32 at ``offset`` floats into its slot; zero where a span's position is 0).
    ``decays`` [n, heads * dim]: g has one number per head and key channel (a row of S each)."""
    n = qn.shape[0]
    addr, per_slot = _field(state, offset, "gated_delta_scan")
    if (tuple(o_out.shape) != (n, heads * vdim) or tuple(vv.shape) != (n, heads * vdim)
            or tuple(qn.shape) != (n, kv_heads * dim) or tuple(kn.shape) != tuple(qn.shape)
            or tuple(gb.shape) != (n, 2, heads) or offset + heads * dim * vdim > per_slot
            or (decays is not None and tuple(decays.shape) != (n, heads * dim))
            or slots.numel() < n_spans or span_start.numel() < n_spans + 1 or span_pos.numel() < n_spans):
        raise KernelError("gated_delta_scan: shapes do not fit")
    F32, I32 = torch.float32, torch.int32
    _launch("kllm_gated_delta_scan", "gated_delta_scan", _ptr(qn, "gated_delta qn", F32), _ptr(kn, "gated_delta kn", F32),
            _ptr(vv, "gated_delta v", F32), _ptr(gb, "gated_delta gb", F32), _ptr(o_out, "gated_delta o", F32), addr,
            per_slot, _ptr(slots, "gated_delta slots", I32), _ptr(span_start, "gated_delta span_start", I32),
            _ptr(span_pos, "gated_delta span_pos", I32), int(n_spans), int(heads), int(kv_heads), int(dim), int(vdim),
            _ptr(decays, "gated_delta decays", F32, True), _stream())


def linear_recurrence_prep(proj, x_bias, conv_w, conv_b, taps, state, conv_offset, wr_t, wi_t, br, bi, rate,
                           span_of_token, slots, span_start, span_pos, a_out, b_out, blocks):
    """proj: float32 sums [nsplit, n, 2 W] of y | x.  u = conv(x + x_bias) + conv_b; gates r, i =
    sigmoid(block-diagonal products of u + biases), the matrices given [blocks, in, out]; a_out =
    exp(-rate r), b_out = sqrt(1 - a^2) i u, both [n, W]."""
    n, W = a_out.shape
    nsplit, stride = _splits(proj, n, 2 * W, "linear_recurrence_prep")
    addr, per_slot = _field(state, conv_offset, "linear_recurrence_prep")
    bs = W // blocks
    F32, I32 = torch.float32, torch.int32
    if (W % blocks or tuple(wr_t.shape) != (blocks, bs, bs) or tuple(wi_t.shape) != (blocks, bs, bs)
            or tuple(conv_w.shape) != (W, taps) or any(t.numel() != W for t in (x_bias, conv_b, br, bi, rate))
            or tuple(b_out.shape) != (n, W) or conv_offset + W * (taps - 1) > per_slot or span_of_token.numel() < n):
        raise KernelError("linear_recurrence_prep: shapes do not fit")
    _launch("kllm_linear_recurrence_prep", "linear_recurrence_prep", _ptr(proj, "recurrence proj", F32), nsplit, stride,
            _ptr(x_bias, "recurrence x bias", F32), _ptr(conv_w, "recurrence conv", F32),
            _ptr(conv_b, "recurrence conv bias", F32), int(taps), addr, per_slot, _ptr(wr_t, "recurrence gate r", F32),
            _ptr(wi_t, "recurrence gate i", F32), _ptr(br, "recurrence gate r bias", F32),
            _ptr(bi, "recurrence gate i bias", F32), _ptr(rate, "recurrence rate", F32),
            _ptr(span_of_token, "recurrence span_of_token", I32), _ptr(slots, "recurrence slots", I32),
            _ptr(span_start, "recurrence span_start", I32), _ptr(span_pos, "recurrence span_pos", I32),
            _ptr(a_out, "recurrence a", F32), _ptr(b_out, "recurrence b", F32), n, W, int(blocks), _stream())


def linear_recurrence_scan(a_in, b_in, proj, y_bias, state, offset, slots, span_start, span_pos, n_spans, out):
    """S <- a S + b along every span (state [W] float32 at ``offset`` floats into the slot); out
    [n, W] = S * gelu_tanh(y + y_bias), y the first W columns of the sums ``proj`` [nsplit, n, 2 W]."""
    n, W = a_in.shape
    nsplit, stride = _splits(proj, n, 2 * W, "linear_recurrence_scan")
    addr, per_slot = _field(state, offset, "linear_recurrence_scan")
    if (tuple(b_in.shape) != (n, W) or tuple(out.shape) != (n, W) or y_bias.numel() != W or offset + W > per_slot
            or slots.numel() < n_spans or span_start.numel() < n_spans + 1 or span_pos.numel() < n_spans):
        raise KernelError("linear_recurrence_scan: shapes do not fit")
    F32, I32 = torch.float32, torch.int32
    _launch("kllm_linear_recurrence_scan", "linear_recurrence_scan", _ptr(a_in, "recurrence a", F32),
            _ptr(b_in, "recurrence b", F32), _ptr(proj, "recurrence proj", F32), nsplit, stride,
            _ptr(y_bias, "recurrence y bias", F32), addr, per_slot, _ptr(slots, "recurrence slots", I32),
            _ptr(span_start, "recurrence span_start", I32), _ptr(span_pos, "recurrence span_pos", I32),
            _ptr(out, "recurrence out"), int(n_spans), W, dtype_code(out.dtype), _stream())


def scaled_sum(out, a, scale_a, b, scale_b):
    """out [n, d] float32 = scale_a * a + scale_b * b; a and b are float32 sums [n, d] or [slices, n, d]."""
    n, d = out.shape
    na, sa = _splits(a, n, d, "scaled_sum")
    nb, sb = _splits(b, n, d, "scaled_sum")
    F32 = torch.float32
    _launch("kllm_scaled_sum", "scaled_sum", _ptr(out, "scaled_sum out", F32), _ptr(a, "scaled_sum a", F32), na, sa,
            float(scale_a), _ptr(b, "scaled_sum b", F32), nb, sb, float(scale_b), n * d, _stream())


def normed_sum(out, a, scale_a, weight_a, b, scale_b, weight_b, eps):
    """out [n, d] float32 = scale_a * weight_a * N(a) + scale_b * weight_b * N(b), row by row; a and b
    are float32 sums [n, d] or [slices, n, d], N(v) = v / sqrt(mean(v^2) + eps)."""
    n, d = out.shape
    na, sa = _splits(a, n, d, "normed_sum")
    nb, sb = _splits(b, n, d, "normed_sum")
    if weight_a.numel() != d or weight_b.numel() != d:
        raise KernelError("normed_sum: the norms' weights do not fit")
    F32 = torch.float32
    _launch("kllm_normed_sum", "normed_sum", _ptr(out, "normed_sum out", F32), _ptr(a, "normed_sum a", F32), na, sa,
            float(scale_a), _ptr(weight_a, "normed_sum weight a", F32), _ptr(b, "normed_sum b", F32), nb, sb,
            float(scale_b), _ptr(weight_b, "normed_sum weight b", F32), n, d, float(eps), _stream())


# ----------------------------------------------------------------------------- attention through low-rank latents

def latent_max_row() -> int:
    return limit("latent_max_row")


def _columns(sums, first_column, width, who):
    """(address, nsplit, slice stride, row stride) of ``width`` columns from ``first_column`` of float32
    sums [n, cols] or [nsplit, n, cols]."""
    n, cols = sums.shape[-2], sums.shape[-1]
    nsplit, stride = _splits(sums, n, cols, who)
    if first_column < 0 or first_column + width > cols:
        raise KernelError(f"{who}: columns {first_column} .. {first_column + width} of {cols}")
    return _ptr(sums, who + " sums", torch.float32) + 4 * int(first_column), nsplit, stride, cols


def latent_kv_append(sums, first_column, weight, eps, cos, sin, cache, positions, span_of_token, block_table, page_size,
                     rank, rot_dim):
    """Columns first_column .. + rank + rot_dim of the float32 sums: the first ``rank`` through an RMS
    norm with ``weight``, the rest rotated (halves paired; cos, sin [n, rot_dim / 2]); the row is
    appended to the pages (``cache`` [pages, page_size * (rank + rot_dim) + rank * page_size]: a
    page's rows, then the normalised part once more as [rank][slot])."""
    n = cos.shape[0]
    row = rank + rot_dim
    addr, nsplit, stride, cols = _columns(sums, first_column, row, "latent_kv_append")
    if (sums.shape[-2] != n or cache.dim() != 2 or cache.shape[1] != page_size * (row + rank) or weight.numel() != rank
            or tuple(cos.shape) != (n, rot_dim // 2) or tuple(sin.shape) != tuple(cos.shape)
            or positions.numel() < n or span_of_token.numel() < n):
        raise KernelError("latent_kv_append: shapes do not fit")
    F32, I32 = torch.float32, torch.int32
    _launch("kllm_latent_kv_append", "latent_kv_append", addr, nsplit, stride,
            _ptr(weight, "latent norm", F32), float(eps), _ptr(cos, "latent cos", F32), _ptr(sin, "latent sin", F32),
            _ptr(cache, "latent cache"), _ptr(positions, "latent positions", I32),
            _ptr(span_of_token, "latent span_of_token", I32), _ptr(block_table, "latent block_table", I32),
            block_table.shape[1], int(page_size), n, int(rank), int(rot_dim), dtype_code(cache.dtype), cols, _stream())


def latent_norm(sums, first_column, weight, eps, out):
    """out [n, r] = RMS norm with ``weight`` of columns first_column .. + r of the float32 sums."""
    n, r = out.shape
    addr, nsplit, stride, cols = _columns(sums, first_column, r, "latent_norm")
    if sums.shape[-2] != n or weight.numel() != r:
        raise KernelError("latent_norm: shapes do not fit")
    _launch("kllm_latent_norm", "latent_norm", addr, nsplit, stride, cols, _ptr(weight, "latent norm", torch.float32),
            float(eps), _ptr(out, "latent_norm out"), n, r, dtype_code(out.dtype), _stream())


def latent_query(q, w_uk, cos, sin, out, heads, dim, rot_dim, rank, transposed=False):
    """q: float32 sums [nsplit, n, H (dim + rot_dim)], a head laid out [dim | rot_dim].  out [n, H
    (rank + rot_dim)]: per head the first dim folded through w_uk ([H dim, rank]: sum_i q_i w[i, :]),
    then the rotated rest.  ``transposed``: w_uk is given head by head as [H rank, dim] (bfloat16,
    dim in steps of 32): the product runs on the matrix cores."""
    n = out.shape[0]
    nsplit, stride = _splits(q, n, heads * (dim + rot_dim), "latent_query")
    if (tuple(out.shape) != (n, heads * (rank + rot_dim))
            or tuple(w_uk.shape) != ((heads * rank, dim) if transposed else (heads * dim, rank))
            or w_uk.dtype != out.dtype or tuple(cos.shape) != (n, rot_dim // 2) or tuple(sin.shape) != tuple(cos.shape)):
        raise KernelError("latent_query: shapes do not fit")
    F32 = torch.float32
    _launch("kllm_latent_query", "latent_query", _ptr(q, "latent q", F32), nsplit, stride, _ptr(w_uk, "latent w_uk"),
            _ptr(cos, "latent cos", F32), _ptr(sin, "latent sin", F32), _ptr(out, "latent q out"), n, int(heads),
            int(dim), int(rot_dim), int(rank), dtype_code(out.dtype), int(bool(transposed)), _stream())


LATENT_BLOCK_FROM = 64      # tokens of a step from which four tokens share a workgroup and its tiles of keys


def attn_latent_slices(n, heads, rank, dtype=torch.bfloat16) -> int:
    """Workgroups that share out the keys of a token and 16 heads (their results are merged in
    the same call): as many as bring a step's workgroups to about two a CU, for steps of few
    tokens; 1 where the kernel on the matrix cores does not run; 0 for steps of many tokens: there
    a workgroup takes four tokens, whose keys pass through LDS once for the four.  Does not depend on any context
    length, so a recorded step can be replayed as contexts grow."""
    if dtype != torch.bfloat16 or rank % 16 or rank > 512:
        return 1
    if n >= LATENT_BLOCK_FROM:
        return 0
    groups = n * ((heads + 15) // 16)
    slices = 1
    while slices < 32 and groups * slices * 2 <= 2 * device_cus():
        slices *= 2
    return slices


def attn_latent(q, out, cache, positions, span_of_token, block_table, page_size, heads, row, rank, scale, plain=False,
                part=None, nslices=1):
    """Causal attention of q [n, H row] over cached rows of ``row`` elements whose first ``rank``
    are also the values (a page: its rows, then the first ``rank`` elements once more as
    [rank][slot]): out [n, H rank].  ``plain``: the kernel for every size, also where the one on
    the matrix cores fits."""
    n = q.shape[0]
    if (tuple(q.shape) != (n, heads * row) or tuple(out.shape) != (n, heads * rank) or q.dtype != cache.dtype
            or out.dtype != q.dtype or cache.dim() != 2 or cache.shape[1] != page_size * (row + rank)
            or positions.numel() < n or span_of_token.numel() < n):
        raise KernelError("attn_latent: shapes or dtypes do not fit")
    I32 = torch.int32
    _launch("kllm_attn_latent", "attn_latent", _ptr(q, "attn_latent q"), _ptr(out, "attn_latent out"),
            _ptr(cache, "attn_latent cache"), _ptr(positions, "attn_latent positions", I32),
            _ptr(span_of_token, "attn_latent span_of_token", I32), _ptr(block_table, "attn_latent block_table", I32),
            block_table.shape[1], int(page_size), n, int(heads), int(row), int(rank), float(scale), dtype_code(q.dtype),
            int(bool(plain)), _ptr(part, "attn_latent part", torch.float32, True) if nslices > 1 else 0,
            part.numel() if nslices > 1 else 0, int(nslices), _stream())


def latent_out(attended, w_uv, out, heads, vdim, rank, gate=None, gate_column=0):
    """out [n, H vdim] = per head w_uv ([H vdim, rank]) times attended [n, H rank], times sigmoid of
    columns gate_column .. + H vdim of the float32 sums ``gate`` (None: no gate)."""
    n = out.shape[0]
    addr, nsplit, stride, cols = _columns(gate, gate_column, heads * vdim, "latent_out") if gate is not None else (0, 0, 0, 0)
    if (tuple(attended.shape) != (n, heads * rank) or tuple(out.shape) != (n, heads * vdim)
            or tuple(w_uv.shape) != (heads * vdim, rank) or w_uv.dtype != out.dtype or attended.dtype != out.dtype
            or (gate is not None and gate.shape[-2] != n)):
        raise KernelError("latent_out: shapes or dtypes do not fit")
    _launch("kllm_latent_out", "latent_out", _ptr(attended, "latent attended"), _ptr(w_uv, "latent w_uv"),
            addr, nsplit, stride, cols, _ptr(out, "latent out"), n, int(heads), int(vdim), int(rank),
            dtype_code(out.dtype), _stream())
