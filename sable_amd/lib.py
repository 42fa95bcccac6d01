"""ctypes loader of libexacta_hip.so (built in-tree by `make -C sable_amd/csrc` / __graft_entry__.build()).

The library is the product; nothing here falls back to a CPU path: a missing library raises, and on a
box without an MI355X every device entry point returns EXH_E_DEVICE, which surfaces as DeviceError.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libexacta_hip.so")

OK, E_PARAM, E_DIVZERO, E_SHAPE, E_EXHAUSTED, E_REJECT, E_MALFORMED, E_DEVICE, E_NOMEM = 0, -1, -2, -3, -4, -5, -6, -7, -8


class ExactaError(Exception):
    """The root of the library's errors (the reference's exacta-error, src/conditions.lisp)."""

    def __init__(self, status, message):
        super().__init__(f"{message} (status {status})")
        self.status = status
        self.message = message


class InvalidParameter(ExactaError): pass
class FieldDivisionByZero(ExactaError, ZeroDivisionError): pass
class MessageShapeError(ExactaError): pass
class TranscriptExhausted(ExactaError): pass
class VerificationFailure(ExactaError): pass
class DeviceError(ExactaError): pass


class MalformedProof(ExactaError):
    @property
    def reason(self):
        return self.message.split(": ", 1)[-1]


_ERRORS = {E_PARAM: InvalidParameter, E_DIVZERO: FieldDivisionByZero, E_SHAPE: MessageShapeError,
           E_EXHAUSTED: TranscriptExhausted, E_REJECT: VerificationFailure, E_MALFORMED: MalformedProof,
           E_DEVICE: DeviceError, E_NOMEM: DeviceError}

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with `make -C sable_amd/csrc` "
                              "(or __graft_entry__.build()); there is no CPU fallback")
        _lib = C.CDLL(LIB_PATH)
        _lib.exh_last_error.restype = C.c_char_p
        _lib.exh_table_device_ptr.restype = C.c_void_p
        _lib.exh_table_device_ptr.argtypes = [C.c_uint64]
    return _lib


def check(status):
    if status == OK:
        return
    message = load().exh_last_error().decode(errors="replace")
    raise _ERRORS.get(status, ExactaError)(status, message)


_initialised = False


def init(device=0):
    """exh_init once per process; raises DeviceError when no gfx950 GPU is usable."""
    global _initialised
    if not _initialised:
        check(load().exh_init(device))
        _initialised = True
