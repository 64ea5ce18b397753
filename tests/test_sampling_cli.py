"""The sampler's host part, the option table and the wire protocol (no GPU)."""
import io

import numpy as np
import pytest

import plain
from hf_cpu_amd.cli import opts as O
from hf_cpu_amd.cli.proto import Out, Reader, quote
from host_draw import order_on_host, pick, pick_rows
from hf_cpu_amd.sampling import Rng, SamplerParams
from hf_cpu_amd.status import EngineError


def test_rng_is_the_plain_one():
    for seed in (0, 1, 7, 2 ** 63 + 5):
        a, b = Rng(seed), plain.Rng(seed)
        assert [a.uniform() for _ in range(50)] == [b.uniform() for _ in range(50)]


@pytest.mark.parametrize("params", [(0.8, 40, 0.95, 0.05), (1.0, 0, 1.0, 0.0), (0.3, 5, 0.5, 0.0),
                                    (2.0, 0, 0.9, 0.2), (5.0, 1000, 1.0, 0.0)])
def test_pick_follows_the_plain_pipeline(params):
    rng = np.random.default_rng(0)
    temp, top_k, top_p, min_p = params
    for trial in range(30):
        logits = (rng.standard_normal(300) * 3).astype(np.float32)
        logits[5] = logits[200]                     # a tie: ordered by id
        ids, vals = order_on_host(logits, top_k)
        a = pick(ids, vals, SamplerParams(temp, top_k, top_p, min_p), Rng(trial))
        b = plain.sample(logits, temp, top_k, top_p, min_p, plain.Rng(trial))
        assert a == b


@pytest.mark.parametrize("params", [(0.8, 40, 0.95, 0.05), (0.3, 5, 0.5, 0.0), (2.0, 64, 0.9, 0.2), (1.0, 7, 1.0, 0.0)])
def test_rows_drawn_together_are_drawn_as_alone(params):
    """Many rows of one step in one call: each row's token is what the plain sampler draws for
    that row with that row's generator, whatever the other rows hold (a row that keeps one
    candidate beside rows that keep all of them)."""
    rng = np.random.default_rng(1)
    temp, top_k, top_p, min_p = params
    logits = (rng.standard_normal((17, 500)) * 3).astype(np.float32)
    logits[3, 100] = 40.0                           # one candidate takes all the mass
    logits[4] = 0.25                                # all equal
    logits[5, 7] = logits[5, 300] = logits[5].max() + 1
    cands = [order_on_host(r, top_k) for r in logits]
    got = pick_rows(np.stack([c[0] for c in cands]), np.stack([c[1] for c in cands]),
                    SamplerParams(temp, top_k, top_p, min_p), [Rng(100 + i) for i in range(17)])
    want = [plain.sample(logits[i], temp, top_k, top_p, min_p, plain.Rng(100 + i)) for i in range(17)]
    assert got == want


def test_option_layers_and_syntax(tmp_path):
    o = O.defaults()
    assert (o["temp"], o["top-k"], o["top-p"], o["min-p"], o["max-tokens"], o["batch"], o["ctx-max"], o["n"]) == \
        (0.8, 40, 0.95, 0.05, 512, 64, 32768, 1)                                     # src/opts.c:84-111
    O.apply(o, ["--temp", "0", "--top-k=7", "--ctx-max", "4K", "--profile", "--seed", "0x10"])
    assert (o["temp"], o["top-k"], o["ctx-max"], o["profile"], o["seed"]) == (0.0, 7, 4096, True, 16)
    O.apply(o, ["--no-profile"])
    assert o["profile"] is False
    O.apply(o, ["--profile=true", "--record-sep", "LF"])
    assert o["profile"] is True and o["record-sep"] == 10
    for bad, word in ((["--bogus"], "unknown option"), (["--temp"], "needs a value"), (["--temp", "9"], "outside"),
                      (["--batch", "0"], "outside"), (["--top-k", "x"], "bad value"), (["stray"], "unexpected"),
                      (["--no-temp"], "unknown option"), (["--stdin-mode", "maybe"], "not one of")):
        with pytest.raises(EngineError, match=word):
            O.apply(O.defaults(), bad)
    with pytest.raises(EngineError, match="only be set at startup"):             # src/opts.c:297-300
        O.apply(O.defaults(), ["--batch", "8"], request=True)
    f = tmp_path / "s.conf"
    f.write_text("# comment\ntemp = 0.1\nmax-tokens = 9\n")
    s = O.load_settings(O.defaults(), str(f))
    assert s["temp"] == 0.1 and s["max-tokens"] == 9
    O.apply(s, ["--temp", "0.2"])                    # the command line wins over the settings file
    assert s["temp"] == 0.2
    f.write_text("nonsense = 1\n")
    with pytest.raises(EngineError, match="s.conf:1"):
        O.load_settings(O.defaults(), str(f))
    assert O.parse_size("10") == 10 and O.parse_size("2M") == 2 << 20 and O.parse_size("1GiB") == 1 << 30
    with pytest.raises(ValueError):
        O.parse_size("1X")


def test_shell_split_without_expansion():
    assert O.shell_split("--a 'x y' \"p\\\"q\\n\" b\\ c $HOME *") == ["--a", "x y", 'p"q\n', "b c", "$HOME", "*"]
    assert O.shell_split("  ") == [] and O.shell_split("''") == [""]
    with pytest.raises(EngineError):
        O.shell_split("'open")


def test_event_quoting_and_records():
    assert quote("plain") == "plain" and quote("") == '""' and quote("a b") == '"a b"'
    assert quote('q"\\\n\x01=') == '"q\\"\\\\\\n\\x01="'
    buf = io.StringIO()
    Out(buf).event("token", pos=0, id=17)
    assert buf.getvalue() == "@token pos=0 id=17\n"
    r = Reader(io.BytesIO(b"one\x1etwo\x1e" + b"x" * 50 + b"\x1elast"), 0x1e, 10)
    assert r.next() == b"one" and r.next() == b"two"
    with pytest.raises(EngineError) as e:
        r.next()
    assert e.value.code == "ERANGE"
    assert r.next() == b"last" and r.next() is None            # the stream stayed in sync
    assert Reader(io.BytesIO(b""), 0x1e, 10).next() is None


def test_sticky_output_error():
    class Closed:
        def write(self, s):
            raise OSError("closed")

        def flush(self):
            pass
    o = Out(Closed())
    o.event("x")
    assert o.err
    o.event("y")
