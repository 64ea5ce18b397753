"""The wire protocol: records in on stdin, event lines out on stdout.

Events are ``@name key=value ...``; a value is quoted when it is empty or holds a
space, a quote, a backslash, ``=`` or a control character, with the escapes \\\" \\\\ \\n
\\r \\t \\xHH (src/proto.c:111-167). Records end with a separator byte and are capped in
size; an oversize record is skipped and the stream stays in sync (src/proto.c:51-99).
"""
from ..status import ERANGE, EngineError


def quote(v):
    v = str(v)
    need = v == "" or any(ord(c) <= 0x20 or c in '"\\=' or ord(c) == 0x7f for c in v)
    if not need:
        return v
    out = ['"']
    for c in v:
        if c in '"\\':
            out.append("\\" + c)
        elif c == "\n":
            out.append("\\n")
        elif c == "\r":
            out.append("\\r")
        elif c == "\t":
            out.append("\\t")
        elif ord(c) < 0x20 or ord(c) == 0x7f:
            out.append(f"\\x{ord(c):02x}")
        else:
            out.append(c)
    out.append('"')
    return "".join(out)


class Out:
    """Event writer with a sticky error: once a write fails, later writes are dropped and
    the loops above end (src/proto.c:105-109)."""

    def __init__(self, stream):
        self.stream = stream
        self.err = False

    def raw(self, data):
        if self.err:
            return
        try:
            self.stream.write(data)
            self.stream.flush()
        except (OSError, ValueError):
            self.err = True

    def event(self, event_name, /, **pairs):
        self.raw("@" + event_name + "".join(f" {k}={quote(v)}" for k, v in pairs.items()) + "\n")


class Reader:
    """Records from a binary stream, ended by ``sep``; ``next()`` returns bytes, None at the
    end of input, or raises ERANGE for a record beyond ``cap`` after skipping it."""

    def __init__(self, stream, sep, cap):
        self.stream, self.sep, self.cap = stream, bytes([sep]), cap
        self.buf = b""
        self.eof = False

    def next(self):
        skipped = False
        while True:
            i = self.buf.find(self.sep)
            if i >= 0:
                rec, self.buf = self.buf[:i], self.buf[i + 1:]
                if skipped or len(rec) > self.cap:
                    raise EngineError(ERANGE, f"record exceeds --max-record ({self.cap} bytes)")
                return rec
            if len(self.buf) > self.cap:
                self.buf, skipped = b"", True
            if self.eof:
                rec, self.buf = self.buf, b""
                if skipped:
                    raise EngineError(ERANGE, f"record exceeds --max-record ({self.cap} bytes)")
                return rec if rec else None
            chunk = self.stream.read1(1 << 16) if hasattr(self.stream, "read1") else self.stream.read(1 << 16)
            if not chunk:
                self.eof = True
            else:
                self.buf += chunk
