"""Status codes of the engine, as exceptions.

The codes and their meanings are those of the reference's ``hfc_status``
(src/hfc.h:12-22); a failed call raises ``EngineError`` with one of them, and the
command line reports it as ``@done status=error code=... msg=...``
(src/ops.c:1066-1071).
"""

ENOMEM = "ENOMEM"      # allocation failure: pages or state slots ran out
EINVAL = "EINVAL"      # bad argument or option
EIO = "EIO"            # a system call failed
EFORMAT = "EFORMAT"    # malformed input file
ERANGE = "ERANGE"      # size or offset out of range
ENOTSUP = "ENOTSUP"    # valid but not implemented
ECANCEL = "ECANCEL"    # request cancelled or timed out

CODES = (ENOMEM, EINVAL, EIO, EFORMAT, ERANGE, ENOTSUP, ECANCEL)


class EngineError(Exception):
    """An error with a status code; ``str()`` is the message alone."""

    def __init__(self, code, msg):
        assert code in CODES, code
        super().__init__(msg)
        self.code = code
        self.msg = msg


def fail(code, msg):
    raise EngineError(code, msg)
