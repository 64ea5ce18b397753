"""The option table: one table drives the command line, the settings file and
per-request option lines, layered ``defaults < settings file < command line < request``.

Names, kinds, ranges, defaults and meanings are the reference's where it has them
(src/opts.c:30-111); syntax is ``--name value``, ``--name=value``, booleans ``--name`` /
``--no-name`` / ``--name=false`` (src/opts.c:272-311); sizes take K M G T suffixes,
1024-based (src/opts.c:142-166). Session options are refused inside a request
(src/opts.c:297-300). Options of the reference that concern its tokenizer, its CPU
threads or its GGUF files do not exist here; the ones marked "ours" are new.
"""
from dataclasses import dataclass

from ..status import EINVAL, EIO, ERANGE, EngineError, fail

STR, INT, U64, SIZE, DBL, BOOL, ENUM, BYTE = "str", "int", "u64", "size", "dbl", "bool", "enum", "byte"
SESSION, REQUEST = "session", "request"


@dataclass(frozen=True)
class OptDef:
    name: str
    kind: str
    scope: str
    default: object
    lo: float = None
    hi: float = None
    choices: tuple = ()
    help: str = ""


DEFS = (
    OptDef("settings", STR, SESSION, None, help="settings file (key = value lines)"),
    OptDef("stdin-mode", ENUM, SESSION, "prompts", choices=("prompts", "args", "none"), help="prompts | args | none"),
    OptDef("record-sep", BYTE, SESSION, 0x1e, help="record separator byte (RS, 0x1e, 30, or a char)"),
    OptDef("ctx-max", SIZE, SESSION, 32768, help="maximum context tokens of a request"),
    OptDef("max-record", SIZE, SESSION, 64 << 20, help="largest accepted prompt or request line"),
    OptDef("batch", INT, SESSION, 64, 1, 4096, help="tokens per step (prompt portions and decoded tokens together)"),
    OptDef("log-level", ENUM, SESSION, "info", choices=("error", "warn", "info", "debug"),
           help="error | warn | info | debug"),
    OptDef("dtype", ENUM, SESSION, "bfloat16", choices=("bfloat16", "float32", "bf16", "fp32"),
           help="ours: compute precision"),
    OptDef("page-size", INT, SESSION, 16, 1, 1024, help="ours: tokens per cache page"),
    OptDef("kv-tokens", SIZE, SESSION, 0, help="ours: tokens the cache pools hold, 0 = ctx-max x max-seqs "
                                                "within free memory"),
    OptDef("max-seqs", INT, SESSION, 64, 1, 4096, help="ours: most sequences decoded together"),
    OptDef("window", INT, SESSION, None, 0, 1 << 30, help="ours: sliding window in tokens for the layers that config.json "
                                                        "lets have one, instead of config.json's (0 = none)"),

    OptDef("op", STR, REQUEST, "generate", help="generate | bench | echo"),
    OptDef("model", STR, REQUEST, None, help="model folder (config.json + model.safetensors)"),
    OptDef("random-weights", U64, REQUEST, None, help="ours: with --op bench, take only config.json from --model "
                                                      "and make random weights from this seed"),
    OptDef("id", STR, REQUEST, "", help="request id echoed in the response"),
    OptDef("prompt-ids", STR, REQUEST, None, help="prompt as token ids, space or comma separated; several "
                                                  "prompts separated by ';' are decoded together (ours)"),
    OptDef("n", INT, REQUEST, 1, 1, 64, help="completions decoded together from one prompt (seeds seed, seed+1, ...)"),
    OptDef("temp", DBL, REQUEST, 0.8, 0, 5, help="sampling temperature, 0 = greedy"),
    OptDef("top-k", INT, REQUEST, 40, 0, 1000000, help="top-k, 0 = off"),
    OptDef("top-p", DBL, REQUEST, 0.95, 0, 1, help="top-p"),
    OptDef("min-p", DBL, REQUEST, 0.05, 0, 1, help="min-p"),
    OptDef("seed", U64, REQUEST, 0, help="RNG seed (deterministic)"),
    OptDef("max-tokens", INT, REQUEST, 512, 1, 1 << 24, help="maximum new tokens"),
    OptDef("logprobs", INT, REQUEST, 0, 0, 100, help="top-N logprobs per token, 0 = off"),
    OptDef("eos-ids", STR, REQUEST, None, help="ours: end-of-sequence token ids (default: config.json's)"),
    OptDef("timeout", DBL, REQUEST, 0.0, 0, 1e7, help="per-request time limit in seconds, 0 = none"),
    OptDef("profile", BOOL, REQUEST, False, help="report per-kernel time of the request (@profile events)"),
    OptDef("bench-prompt", INT, REQUEST, 256, 1, 32768, help="bench: prompt tokens to prefill"),
    OptDef("bench-gen", INT, REQUEST, 32, 1, 4096, help="bench: tokens to decode"),
    OptDef("bench-batch", INT, REQUEST, 1, 1, 4096, help="ours: bench: sequences decoded together"),
    OptDef("probe-reps", INT, REQUEST, 1, 1, 32, help="bench: repetitions, the median is reported"),
)
BY_NAME = {d.name: d for d in DEFS}
BYTE_NAMES = {"NUL": 0, "EOT": 4, "LF": 10, "FF": 12, "FS": 28, "GS": 29, "RS": 30, "US": 31}


def defaults():
    return {d.name: d.default for d in DEFS}


def parse_size(s):
    """Digits with an optional K M G T suffix (optionally followed by B or iB), 1024-based."""
    i = 0
    while i < len(s) and s[i].isdigit():
        i += 1
    if i == 0:
        raise ValueError
    v, rest = int(s[:i]), s[i:]
    if rest:
        mult = {"K": 1 << 10, "M": 1 << 20, "G": 1 << 30, "T": 1 << 40}.get(rest[0].upper())
        if mult is None or rest[1:] not in ("", "B", "b", "iB", "ib"):
            raise ValueError
        v *= mult
    if v >= 1 << 64:
        raise OverflowError
    return v


def parse_bool(s):
    if s in ("1", "true", "yes", "on"):
        return True
    if s in ("0", "false", "no", "off"):
        return False
    raise ValueError


def parse_byte(s):
    if s in BYTE_NAMES:
        return BYTE_NAMES[s]
    if len(s) == 1 and not s.isdigit():
        return ord(s) & 0xff
    v = int(s, 0)
    if not 0 <= v <= 255:
        raise ValueError
    return v


def set_value(opts, d, val):
    try:
        if d.kind == STR:
            v = val
        elif d.kind == INT:
            v = int(val, 10)
        elif d.kind == U64:
            v = int(val, 0)
            if not 0 <= v < 1 << 64:
                raise ValueError
        elif d.kind == SIZE:
            v = parse_size(val)
        elif d.kind == DBL:
            v = float(val)
            if v != v:
                raise ValueError
        elif d.kind == BOOL:
            v = parse_bool(val)
        elif d.kind == BYTE:
            v = parse_byte(val)
        else:
            if val not in d.choices:
                fail(EINVAL, f"option '--{d.name}': '{val}' is not one of {', '.join(d.choices)}")
            v = val
    except OverflowError:
        fail(ERANGE, f"option '--{d.name}': value '{val}' is too large")
    except ValueError:
        fail(EINVAL, f"option '--{d.name}': bad value '{val}'")
    if d.kind in (INT, DBL) and d.lo is not None and not d.lo <= v <= d.hi:
        fail(EINVAL, f"option '--{d.name}': {val} is outside {d.lo:g}..{d.hi:g}")
    opts[d.name] = v


def apply(opts, argv, request=False):
    """Applies option words to ``opts`` in place (src/opts.c:272-311)."""
    i = 0
    while i < len(argv):
        a = argv[i]
        if len(a) < 3 or not a.startswith("--"):
            fail(EINVAL, f"unexpected argument '{a}' (options start with --)")
        name, eq, val = a[2:].partition("=")
        val = val if eq else None
        d, negate = BY_NAME.get(name), False
        if d is None and name.startswith("no-") and len(name) > 3:
            d = BY_NAME.get(name[3:])
            if d is not None and d.kind == BOOL and val is None:
                negate = True
            else:
                d = None
        if d is None:
            fail(EINVAL, f"unknown option '--{name}'")
        if request and d.scope == SESSION:
            fail(EINVAL, f"option '--{d.name}' can only be set at startup, not per request")
        if d.kind == BOOL and val is None:
            val = "0" if negate else "1"
        elif val is None:
            if i + 1 >= len(argv):
                fail(EINVAL, f"option '--{d.name}' needs a value")
            i += 1
            val = argv[i]
        set_value(opts, d, val)
        i += 1
    return opts


def load_settings(opts, path):
    """``key = value`` lines, ``#`` comments (src/opts.c:313-358)."""
    try:
        with open(path, encoding="utf-8") as f:
            lines = f.read().splitlines()
    except OSError as e:
        fail(EIO, f"cannot read settings file {path}: {e.strerror}")
    for n, line in enumerate(lines, 1):
        line = line.strip()
        if not line or line.startswith("#"):
            continue
        key, eq, val = line.partition("=")
        key, val = key.strip().lstrip("-"), val.strip()
        if not eq or key not in BY_NAME:
            fail(EINVAL, f"{path}:{n}: unknown setting '{key}'")
        try:
            set_value(opts, BY_NAME[key], val)
        except EngineError as e:
            fail(e.code, f"{path}:{n}: {e.msg}")
    return opts


def shell_split(line):
    """POSIX-style word splitting without any expansion (src/opts.c:372-442): single quotes
    are literal; double quotes allow \\\" \\\\ \\n \\t; outside quotes a backslash escapes
    the next character."""
    words, cur, have, i, n = [], [], False, 0, len(line)
    while i < n:
        c = line[i]
        if c in " \t\r\n":
            if have:
                words.append("".join(cur))
                cur, have = [], False
            i += 1
        elif c == "'":
            j = line.find("'", i + 1)
            if j < 0:
                fail(EINVAL, "unterminated single quote")
            cur.append(line[i + 1:j])
            have, i = True, j + 1
        elif c == '"':
            i += 1
            have = True
            while True:
                if i >= n:
                    fail(EINVAL, "unterminated double quote")
                c = line[i]
                if c == '"':
                    i += 1
                    break
                if c == "\\" and i + 1 < n and line[i + 1] in '"\\nt':
                    cur.append({"n": "\n", "t": "\t"}.get(line[i + 1], line[i + 1]))
                    i += 2
                else:
                    cur.append(c)
                    i += 1
        elif c == "\\":
            if i + 1 >= n:
                fail(EINVAL, "trailing backslash")
            cur.append(line[i + 1])
            have, i = True, i + 2
        else:
            cur.append(c)
            have, i = True, i + 1
    if have:
        words.append("".join(cur))
    return words


def usage():
    lines = ["options (S = startup only):"]
    for d in DEFS:
        dflt = "" if d.default in (None, "") else f" [{d.default}]"
        lines.append(f"  --{d.name:<16}{'S ' if d.scope == SESSION else '  '}{d.help}{dflt}")
    return "\n".join(lines)
