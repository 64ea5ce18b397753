"""Each kernel alone against a plain reference, at sizes other than the engine's."""
import math
import types

import numpy as np
import pytest
import torch

import plain
from helpers import bf16_round

pytestmark = pytest.mark.gpu


def dev(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dtype).cuda()


def ints(a):
    return torch.tensor(np.asarray(a, dtype=np.int32), dtype=torch.int32, device="cuda")


def rounded(a, dtype):
    """What the kernel is given after the cast to ``dtype``, as float64."""
    a = np.asarray(a, dtype=np.float32)
    return (bf16_round(a) if dtype == torch.bfloat16 else a).astype(np.float64)


DTYPES = [torch.float32, torch.bfloat16]


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(ops32, dtype):
    rng = np.random.default_rng(0)
    table = rng.standard_normal((37, 50)).astype(np.float32)
    toks = [0, 36, 5, 5, 17]
    out = torch.empty((5, 50), dtype=torch.float32, device="cuda")
    ops32.embed(dev(table, dtype), ints(toks), out)
    assert np.array_equal(out.cpu().numpy(), rounded(table, dtype)[toks].astype(np.float32))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [5, 64, 100, 1000, 3584])
def test_rmsnorm(ops32, dtype, width):
    rng = np.random.default_rng(width)
    x = (rng.standard_normal((7, width)) * 3).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(width)).astype(np.float32)
    out = torch.empty((7, width), dtype=dtype, device="cuda")
    ops32.rmsnorm(dev(x), dev(w), 1e-5, out)
    want = plain.rmsnorm(x.astype(np.float64), w.astype(np.float64), 1e-5)
    tol = 1e-5 if dtype == torch.float32 else 0.02
    assert np.max(np.abs(out.float().cpu().numpy() - want)) <= tol * np.max(np.abs(want))
    rows = [6, 0, 3]
    out2 = torch.empty((3, width), dtype=dtype, device="cuda")
    ops32.rmsnorm(dev(x), dev(w), 1e-5, out2, ints(rows))
    assert torch.equal(out2, out[rows])


def test_rmsnorm_reference_vector(ops32):
    """x = {1..5}, w = {1, 1, 2, 2, 0.5}, eps 1e-6 -> x * w / sqrt(11 + 1e-6)
    (the reference's tests/test_kern.c:242-248)."""
    x = np.array([[1, 2, 3, 4, 5]], dtype=np.float32)
    w = np.array([1, 1, 2, 2, 0.5], dtype=np.float32)
    out = torch.empty((1, 5), dtype=torch.float32, device="cuda")
    ops32.rmsnorm(dev(x), dev(w), 1e-6, out)
    want = x[0] * w / math.sqrt(11 + 1e-6)
    assert np.max(np.abs(out.cpu().numpy()[0] - want)) < 1e-5


@pytest.mark.parametrize("adt,wdt,odt", [(torch.float32, torch.float32, torch.float32),
                                         (torch.bfloat16, torch.bfloat16, torch.bfloat16),
                                         (torch.bfloat16, torch.bfloat16, torch.float32),
                                         (torch.bfloat16, torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("M,N,K", [(1, 7, 5), (3, 100, 33), (64, 64, 64), (65, 130, 257), (200, 48, 1000),
                                   (8, 512, 3584), (257, 1000, 96)])
def test_gemm(ops32, adt, wdt, odt, M, N, K):
    rng = np.random.default_rng(M * 1000 + N + K)
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) / math.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    want = rounded(a, adt) @ rounded(w, wdt).T + b
    out = torch.empty((M, N), dtype=odt, device="cuda")
    ops32.gemm(dev(a, adt), dev(w, wdt), out, bias=dev(b))
    tol = 2e-5 if odt == torch.float32 else 0.02
    got = out.float().cpu().numpy()
    assert np.max(np.abs(got - want)) <= tol * max(1.0, np.max(np.abs(want)))
    if odt == torch.float32:       # accumulate into the residual sum, through a strided view
        wide = torch.zeros((M, N + 3), dtype=torch.float32, device="cuda")
        res = rng.standard_normal((M, N)).astype(np.float32)
        wide[:, :N] = dev(res)
        ops32.gemm(dev(a, adt), dev(w, wdt), wide[:, :N], accumulate=True)
        got = wide[:, :N].cpu().numpy()
        assert np.max(np.abs(got - (want - b + res))) <= tol * max(1.0, np.max(np.abs(want)))
        assert float(wide[:, N:].abs().max()) == 0.0


@pytest.mark.parametrize("N,K", [(100, 333), (1000, 3584), (37, 18944)])
def test_fp32_rows_do_not_depend_on_the_batch(ops32, N, K):
    """The 32-bit product sums every output in ascending k whatever the number of rows (few rows
    take a kernel of their own): a row gives the same bits alone, among 7, 20, 50 and 200 rows."""
    rng = np.random.default_rng(N + K)
    a = rng.standard_normal((200, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) / math.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    da, dw, db = dev(a), dev(w), dev(b)
    whole = torch.empty((200, N), dtype=torch.float32, device="cuda")
    ops32.gemm(da, dw, whole, bias=db)
    want = a.astype(np.float64) @ w.astype(np.float64).T + b
    assert np.max(np.abs(whole.cpu().numpy() - want)) <= 2e-5 * max(1.0, np.max(np.abs(want)))
    for M in (1, 7, 20, 50, 64):
        part = torch.empty((M, N), dtype=torch.float32, device="cuda")
        ops32.gemm(da[:M], dw, part, bias=db)
        assert torch.equal(part, whole[:M]), f"{M} rows differ from the same rows among 200"


@pytest.mark.parametrize("M,N,K", [(1, 256, 512), (8, 4608, 3584), (8, 3584, 18944), (33, 200, 1000),
                                   (64, 1000, 4096), (65, 129, 72), (200, 333, 264), (500, 1100, 1024),
                                   (2048, 512, 3584), (2048, 4608, 1024), (1000, 8200, 512), (700, 5408, 640),
                                   (2048, 3584, 1024), (1024, 8192, 64), (2048, 3584, 64), (512, 4096, 128), (1800, 3600, 2176),
                                   (64, 4608, 3584), (48, 3584, 18944), (33, 37888, 256), (40, 1024, 8192),
                                   (150, 4608, 3584), (300, 3584, 4736), (1900, 4624, 192), (50, 33024, 320), (64, 65536, 64),
                                   (100, 3584, 18944), (128, 4096, 8192), (65, 37888, 1024),      # the stream kernel's tiles of 128 rows
                                   (400, 3584, 18944), (256, 4608, 3584), (700, 3584, 3584),      # 256-row tiles, K cut into parts
                                   (200, 3584, 18944), (250, 3584, 3584), (192, 896, 4864)])      # one row of 256 x 128 tiles, parts by cost
def test_gemm_on_matrix_cores(ops16, M, N, K):
    """bf16 x bf16 with K a multiple of 8 runs on the matrix cores (K split for small M; tiles of
    256 rows loaded straight into LDS for long prompts and wide outputs, with edges in M and N
    and as few as one or two steps of K, K cut in two where the output is narrow, tiles of 192 columns where they fill the CUs better; for 33 to 64 rows one stream of tile-and-K units cut
    evenly over the CUs, with runs shorter and longer than a tile's K; K split also for prompt
    portions of a few hundred rows whose output has few tiles): against fp64 on the rounded operands, against the
    plain kernel on the same operands, in the three output modes, with operands that are views
    of wider buffers."""
    rng = np.random.default_rng(M + N + K)
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) / math.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    want = rounded(a, torch.bfloat16) @ rounded(w, torch.bfloat16).T
    wide_a = torch.zeros((M, K + 16), dtype=torch.bfloat16, device="cuda")
    wide_a[:, 8:K + 8] = dev(a, torch.bfloat16)
    ta, tw, tb = wide_a[:, 8:K + 8], dev(w, torch.bfloat16), dev(b)
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    ops16.gemm(ta, tw, out, bias=tb)
    scale = max(1.0, float(np.max(np.abs(want))))
    assert np.max(np.abs(out.cpu().numpy() - (want + b))) <= 2e-5 * scale
    plain_out = torch.empty_like(out)
    ops16.force_plain_gemm = True
    try:
        ops16.gemm(ta, tw, plain_out, bias=tb)
    finally:
        ops16.force_plain_gemm = False
    assert float((out - plain_out).abs().max()) <= 2e-5 * scale
    o16 = torch.empty((M, N + 8), dtype=torch.bfloat16, device="cuda")[:, :N]
    ops16.gemm(ta, tw, o16)
    assert np.max(np.abs(o16.float().cpu().numpy() - want)) <= 0.01 * scale
    res = rng.standard_normal((M, N)).astype(np.float32)
    acc = dev(res)
    ops16.gemm(ta, tw, acc, accumulate=True)
    assert np.max(np.abs(acc.cpu().numpy() - (want + res))) <= 2e-5 * scale


@pytest.mark.parametrize("M,E,F", [(1, 256, 352), (8, 256, 352), (64, 256, 352), (100, 256, 352), (300, 256, 352),
                                   (1500, 192, 16416), (600, 320, 4512), (48, 192, 16512), (64, 128, 18944)])
def test_gemm_with_gate_up_epilogue(ops16, M, E, F):
    """Gate and up rows interleaved in blocks of 32; the product's last step forms silu(gate) * up:
    directly in the tile's epilogue (large M) or when the split K is added up (small M)."""
    rng = np.random.default_rng(M)
    x = rng.standard_normal((M, E)).astype(np.float32)
    wg = (rng.standard_normal((F, E)) / 16).astype(np.float32)
    wu = (rng.standard_normal((F, E)) / 16).astype(np.float32)
    tg, tu = dev(wg, torch.bfloat16), dev(wu, torch.bfloat16)
    assert ops16.can_fuse_swiglu(tg, tu)
    w = ops16.interleave_gate_up(tg, tu)
    assert torch.equal(w[:32], tg[:32]) and torch.equal(w[32:64], tu[:32]) and torch.equal(w[64:96], tg[32:64])
    out = torch.empty((M, F), dtype=torch.bfloat16, device="cuda")
    ops16.gemm(dev(x, torch.bfloat16), w, out, swiglu=True)
    xr = rounded(x, torch.bfloat16)
    want = plain.silu(xr @ rounded(wg, torch.bfloat16).T) * (xr @ rounded(wu, torch.bfloat16).T)
    assert np.max(np.abs(out.float().cpu().numpy() - want)) <= 0.01 * max(1.0, np.max(np.abs(want)))


@pytest.mark.parametrize("M,K,E", [(5, 4096, 512), (40, 8192, 1024)])
def test_deferred_products_are_finished_by_the_next_kernel(ops16, M, K, E):
    """A product with few rows and a long K leaves partial sums (for 40 rows: the planes of the
    streamed product); the norm that follows adds them into the residual stream and norms the
    result; rope_store does the same for q, k and v."""
    ops16.fuse_rows = False        # the chain of separate kernels (few rows otherwise take products that finish their outputs)
    try:
        _deferred_products(ops16, M, K, E)
    finally:
        ops16.fuse_rows = True


def _deferred_products(ops16, M, K, E):
    rng = np.random.default_rng(0)
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((E, K)) / 64).astype(np.float32)
    b = rng.standard_normal(E).astype(np.float32)
    x0 = rng.standard_normal((M, E)).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(E)).astype(np.float32)
    x = dev(x0)
    ops16.gemm(dev(a, torch.bfloat16), dev(w, torch.bfloat16), x, bias=dev(b), accumulate=True, defer=True)
    assert ops16._pending is not None and ops16._pending.splits > 1, "the case was meant to split K"
    h = torch.empty((M, E), dtype=torch.bfloat16, device="cuda")
    ops16.rmsnorm(x, dev(g), 1e-6, h)
    assert ops16._pending is None
    x_want = x0 + rounded(a, torch.bfloat16) @ rounded(w, torch.bfloat16).T + b
    assert np.max(np.abs(x.cpu().numpy() - x_want)) < 1e-4
    assert np.max(np.abs(h.float().cpu().numpy() - plain.rmsnorm(x_want, g, 1e-6))) < 0.03
    # the same product, settled explicitly
    x2 = dev(x0)
    ops16.gemm(dev(a, torch.bfloat16), dev(w, torch.bfloat16), x2, bias=dev(b), accumulate=True, defer=True)
    ops16.settle(x2)
    assert float((x2 - x).abs().max()) < 1e-5          # the same sums in another order
    # q, k, v: H = 2, G = 1, D = 64 -> width 256
    H, G, D = 2, 1, 64
    wq = (rng.standard_normal(((H + 2 * G) * D, K)) / 64).astype(np.float32)
    bq = rng.standard_normal((H + 2 * G) * D).astype(np.float32)
    qkv = torch.zeros((M, (H + 2 * G) * D), dtype=torch.bfloat16, device="cuda")
    ops16.gemm(dev(a, torch.bfloat16), dev(wq, torch.bfloat16), qkv, bias=dev(bq), defer=True)
    assert ops16._pending is not None
    rows = (M + 3 + 3) // 4 * 4
    cache = FakeCache(group=0, k=torch.zeros((rows, G * D), dtype=torch.bfloat16, device="cuda"),
                      v=torch.zeros((rows, G * D), dtype=torch.bfloat16, device="cuda"), page_tokens=4)
    positions = [int(p) for p in rng.integers(0, 200, M)]
    slot_map = [int(p) for p in rng.permutation(M + 3)[:M]]
    i = np.arange(D // 2, dtype=np.float64)
    inv_freq = dev((1e4 ** (-2.0 * i / D)).astype(np.float32))
    ops16.rope_store(qkv, ints(positions), inv_freq, D, H, G, D, cache, ints(slot_map))
    assert ops16._pending is None
    full = rounded(a, torch.bfloat16) @ rounded(wq, torch.bfloat16).T + bq
    q_want = plain.rope(full[:, :H * D].reshape(M, H, D), positions, D, 1e4).reshape(M, H * D)
    k_want = plain.rope(full[:, H * D:(H + G) * D].reshape(M, G, D), positions, D, 1e4).reshape(M, G * D)
    assert np.max(np.abs(qkv[:, :H * D].float().cpu().numpy() - q_want)) < 0.05
    assert np.max(np.abs(cache.k.float().cpu().numpy()[slot_map] - k_want)) < 0.05
    vc = from_value_layout(cache.v.float().cpu().numpy(), 4)
    assert np.max(np.abs(vc[slot_map] - full[:, (H + G) * D:])) < 0.05


@pytest.mark.parametrize("M,K,E,N", [(1, 256, 128, 1000), (5, 4096, 896, 1152), (8, 18944, 3584, 4608), (16, 3584, 3584, 4100),
                                     (11, 640, 2176, 77), (16, 1536, 8960, 333),
                                     (17, 3584, 3584, 4608), (32, 18944, 3584, 37888), (24, 896, 896, 1152), (29, 256, 8960, 77),
                                     (32, 1024, 40000, 2100)])
def test_products_of_few_rows_that_finish_their_outputs(ops16, M, K, E, N):
    """Up to 32 rows (from 17 on the kernel holds two tiles of 16 rows, and the shares of the sums of squares are
    laid out for 32): a product into the residual stream waits for the norm that follows; one kernel then does product,
    residual sum, the sums of squares and x * weight, and the product that reads the norm's output scales its sums
    (``Ops.rmsnorm(..., lazy=True)``). Against the same in float64: the residual stream, the product behind the
    norm (into fp32, into bf16, and as the 32-bit plane that the rotation of queries and keys takes), gate and up
    with the activation, and the norm's output made whole when something else asks for it."""
    ops16.rows_always = True       # (left to itself, Ops sends a long K at 17 rows and more to other kernels: they are quicker)
    try:
        _products_of_few_rows(ops16, M, K, E, N)
    finally:
        ops16.rows_always = False


def _products_of_few_rows(ops16, M, K, E, N):
    rng = np.random.default_rng(M + K)
    bf = torch.bfloat16
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((E, K)) / math.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(E).astype(np.float32)
    x0 = rng.standard_normal((M, E)).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(E)).astype(np.float32)
    w2 = (rng.standard_normal((N, E)) / math.sqrt(E)).astype(np.float32)
    b2 = rng.standard_normal(N).astype(np.float32)
    x_want = x0 + rounded(a, bf) @ rounded(w, bf).T + b
    h_want = plain.rmsnorm(x_want, g, 1e-5)
    out_want = h_want @ rounded(w2, bf).T + b2

    def lazily():
        x, h = dev(x0), torch.empty((M, E), dtype=bf, device="cuda")
        ops16.gemm(dev(a, bf), dev(w, bf), x, bias=dev(b), accumulate=True, defer=True)
        assert ops16._lazy is not None and ops16._pending is None
        ops16.rmsnorm(x, dev(g), 1e-5, h, lazy=True)
        assert ops16._lazy is None and h.data_ptr() in ops16._scaled
        return x, h
    x, h = lazily()
    assert np.max(np.abs(x.cpu().numpy() - x_want)) < 2e-5 * max(1.0, np.max(np.abs(x_want)))
    scale = np.max(np.abs(out_want))
    for odt, tol in ((torch.float32, 6e-3), (bf, 1.2e-2)):
        out = torch.empty((M, N), dtype=odt, device="cuda")
        ops16.gemm(h, dev(w2, bf), out, bias=dev(b2))
        assert np.max(np.abs(out.float().cpu().numpy() - out_want)) < tol * scale, str(odt)
    if N % 8 == 0:                                         # deferred: a 32-bit plane for the kernel that follows
        out = torch.empty((M, N), dtype=bf, device="cuda")
        ops16.gemm(h, dev(w2, bf), out, bias=dev(b2), defer=True)
        assert ops16._pending is not None and ops16._pending.splits == 1
        ops16.settle()
        assert np.max(np.abs(out.float().cpu().numpy() - out_want)) < 1.2e-2 * scale
    # the norm's output made whole: what the plain norm kernel gives
    ops16.settle(h)
    assert h.data_ptr() not in ops16._scaled
    assert np.max(np.abs(h.float().cpu().numpy() - h_want)) < 0.02 * np.max(np.abs(h_want))
    # without the norm: the product alone (settled), the same residual stream bit for bit
    x2 = dev(x0)
    ops16.gemm(dev(a, bf), dev(w, bf), x2, bias=dev(b), accumulate=True, defer=True)
    ops16.settle(x2)
    assert torch.equal(x2, x)
    # gate and up with the activation, from the lazy norm's output
    F = (N + 31) // 32 * 32
    wg, wu = ((rng.standard_normal((F, E)) / math.sqrt(E)).astype(np.float32) for _ in range(2))
    x, h = lazily()
    assert ops16.can_fuse_swiglu(dev(wg, bf), dev(wu, bf))
    act = torch.empty((M, F), dtype=bf, device="cuda")
    ops16.gemm(h, ops16.interleave_gate_up(dev(wg, bf), dev(wu, bf)), act, swiglu=True)
    gt, up = h_want @ rounded(wg, bf).T, h_want @ rounded(wu, bf).T
    act_want = plain.silu(gt) * up
    assert np.max(np.abs(act.float().cpu().numpy() - act_want)) < 1.5e-2 * max(1.0, np.max(np.abs(act_want)))
    # the same calls with the fusion off give the same values within bf16's rounding
    ops16.fuse_rows = False
    try:
        x3, h3 = dev(x0), torch.empty((M, E), dtype=bf, device="cuda")
        ops16.gemm(dev(a, bf), dev(w, bf), x3, bias=dev(b), accumulate=True, defer=True)
        ops16.rmsnorm(x3, dev(g), 1e-5, h3, lazy=True)
        assert h3.data_ptr() not in ops16._scaled
        assert float((x3 - x).abs().max()) < 2e-5 * max(1.0, np.max(np.abs(x_want)))
    finally:
        ops16.fuse_rows = True


def test_products_with_a_weight_matrix_beyond_four_gigabytes(ops16):
    """300,000 rows of 8,192 bf16 weights are 4.9 GB: byte offsets from the matrix's start no longer fit 32 bits.
    Every product kernel (1, 8, 24, 64, 128, 300 and 2,048 rows of activations) against the library's product on
    slices of the columns, among them the last ones and those around the 2 GB and 4 GB marks."""
    bf = torch.bfloat16
    N, K = 300000, 8192
    g = torch.Generator(device="cuda").manual_seed(1)
    w = torch.empty((N, K), device="cuda", dtype=bf)
    for i in range(0, N, 50000):
        w[i:i + 50000] = (torch.randn((min(50000, N - i), K), device="cuda", generator=g) * 0.02).to(bf)
    for M in (1, 8, 24, 64, 128, 300, 2048):
        a = torch.randn((M, K), device="cuda", generator=g).to(bf)
        out = torch.empty((M, N), device="cuda", dtype=torch.float32)
        ops16.gemm(a, w, out)
        ops16.settle()
        for c0 in (0, 131072 - 64, 262144 - 100, N - 5000):
            ref = a.float() @ w[c0:c0 + 5000].float().T
            err = float((out[:, c0:c0 + 5000] - ref).abs().max() / ref.abs().max())
            assert err < 2e-5, f"{M} rows, columns from {c0}: {err:.2e}"
    del w, out
    torch.cuda.empty_cache()


def test_gemm_matches_library_product(ops32):
    """The kernel against the library's fp32 matrix product on the same operands."""
    torch.manual_seed(0)
    a = torch.randn(70, 300, device="cuda")
    w = torch.randn(90, 300, device="cuda")
    out = torch.empty(70, 90, device="cuda")
    ops32.gemm(a, w, out)
    ref = (a.double() @ w.double().T).float()
    assert float((out - ref).abs().max()) < 1e-3


class FakeCache(types.SimpleNamespace):
    pass


class FakeStep:
    """Step inputs for a kernel alone: tokens of one request are consecutive in the batch."""

    def __init__(self, positions, token_slot, block_table, slot_map):
        self.positions, self.token_slot = positions, token_slot
        self._g = types.SimpleNamespace(block_table=block_table, slot_map=slot_map)
        slots, pos = token_slot.cpu().tolist(), positions.cpu().tolist()
        starts = [0] + [i for i in range(1, len(slots)) if slots[i] != slots[i - 1]] + [len(slots)]
        self.q_start = ints(starts)
        self.n_seqs = len(starts) - 1
        self.max_q_len = max(b - a for a, b in zip(starts, starts[1:]))
        self.max_seq_len = max(pos) + 1

    def group(self, i):
        return self._g


def to_value_layout(rows, page):
    """[n_pages * page, width] by token -> the cache's value layout: each page transposed."""
    n, w = rows.shape
    return np.ascontiguousarray(rows.reshape(n // page, page, w).transpose(0, 2, 1)).reshape(n, w)


def from_value_layout(rows, page):
    n, w = rows.shape
    return np.ascontiguousarray(rows.reshape(n // page, w, page).transpose(0, 2, 1)).reshape(n, w)


def paged_setup(rng, lengths, G, D, page, dtype, n_pages=None, shuffle=True):
    """Random keys and values for requests of the given lengths, scattered over pages in a
    random order. Returns (k [list of [n, G, D]], v, cache, block_table)."""
    blocks = [-(-n // page) for n in lengths]
    n_pages = n_pages or sum(blocks) + 3
    perm = rng.permutation(n_pages) if shuffle else np.arange(n_pages)
    max_blocks = max(blocks) + 2
    table = np.zeros((len(lengths), max_blocks), np.int32)
    kc = np.full((n_pages * page, G * D), 1e4, np.float32)     # stale rows hold large values
    vc = np.full((n_pages * page, G * D), -1e4, np.float32)
    ks, vs, at = [], [], 0
    for s, n in enumerate(lengths):
        k = rng.standard_normal((n, G, D)).astype(np.float32)
        v = rng.standard_normal((n, G, D)).astype(np.float32)
        for b in range(blocks[s]):
            pg = perm[at]
            at += 1
            table[s, b] = pg
            rows = slice(b * page, min((b + 1) * page, n))
            cnt = rows.stop - rows.start
            kc[pg * page:pg * page + cnt] = k[rows].reshape(cnt, G * D)
            vc[pg * page:pg * page + cnt] = v[rows].reshape(cnt, G * D)
        ks.append(k)
        vs.append(v)
    vc = to_value_layout(vc, page)
    cache = FakeCache(group=0, k=dev(kc, dtype), v=dev(vc, dtype), page_tokens=page, window=0)
    return ks, vs, cache, ints(table)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,page,window", [(4, 2, 16, 16, 0), (3, 1, 32, 8, 20), (8, 8, 64, 16, 0),
                                               (14, 2, 64, 32, 0), (6, 2, 128, 16, 70), (5, 5, 48, 4, 0),
                                               (2, 1, 256, 64, 0)])
def test_paged_attention(ops32, dtype, H, G, D, page, window):
    """Queries at the last positions of each request (a prompt portion of several tokens for
    some, a single token for others) against attention over whole sequences."""
    rng = np.random.default_rng(H * 100 + D + page)
    lengths = [1, 5, 64, 130, 203]
    q_lens = [1, 3, 64, 1, 17]
    ks, vs, cache, table = paged_setup(rng, lengths, G, D, page, dtype)
    qs, positions, slots, wants = [], [], [], []
    for s, (n, ql) in enumerate(zip(lengths, q_lens)):
        q_full = rng.standard_normal((n, H, D)).astype(np.float32)
        full = plain.attention(rounded(q_full, dtype), rounded(ks[s], dtype), rounded(vs[s], dtype), window)
        qs.append(q_full[n - ql:])
        wants.append(full[n - ql:])
        positions += list(range(n - ql, n))
        slots += [s] * ql
    q = np.concatenate(qs).reshape(-1, H * D)
    want = np.concatenate(wants).reshape(-1, H * D)
    T = q.shape[0]
    qpad = torch.zeros((T, H * D + 2 * G * D), dtype=dtype, device="cuda")    # q inside wider rows
    qpad[:, :H * D] = dev(q, dtype)
    out = torch.empty((T, H * D), dtype=dtype, device="cuda")
    step = FakeStep(ints(positions), ints(slots), table, None)
    ops32.paged_attention(qpad[:, :H * D], H, G, D, cache, step, window, 1.0 / math.sqrt(D), out)
    tol = 2e-5 if dtype == torch.float32 else 0.02
    err = np.max(np.abs(out.float().cpu().numpy() - want))
    assert err <= tol, f"max |diff| {err:.3e}"
    if dtype == torch.bfloat16:          # the plain kernel on the same inputs
        other = torch.empty_like(out)
        ops32.force_plain_attention = True
        try:
            ops32.paged_attention(qpad[:, :H * D], H, G, D, cache, step, window, 1.0 / math.sqrt(D), other)
        finally:
            ops32.force_plain_attention = False
        assert np.max(np.abs(other.float().cpu().numpy() - want)) <= tol


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,page,window", [(6, 2, 32, 8, 0), (4, 4, 48, 16, 30), (28, 4, 128, 16, 0)])
def test_paged_attention_with_score_slopes(ops32, dtype, H, G, D, page, window):
    """The hook for position encodings that enter the scores: slope_h * (j - p) added to the score of key j
    for the query at p, against attention written out in float64 (also for a shape that would otherwise run on
    the matrix cores)."""
    rng = np.random.default_rng(H + D)
    lengths, q_lens = [1, 77, 300], [1, 40, 2]
    slopes = (2.0 ** -(1 + 6 * np.arange(H) / H)).astype(np.float32)
    ks, vs, cache, table = paged_setup(rng, lengths, G, D, page, dtype)
    qs, positions, slots, wants = [], [], [], []
    for s, (n, ql) in enumerate(zip(lengths, q_lens)):
        q_tail = rounded(rng.standard_normal((ql, H, D)).astype(np.float32), dtype).astype(np.float64)
        k64, v64 = rounded(ks[s], dtype).astype(np.float64), rounded(vs[s], dtype).astype(np.float64)
        want = np.empty((ql, H, D))
        for i in range(ql):
            p = n - ql + i
            lo = max(0, p - window + 1) if window else 0
            for h in range(H):
                sc = k64[lo:p + 1, h // (H // G)] @ q_tail[i, h] / math.sqrt(D) + slopes[h] * (np.arange(lo, p + 1) - p)
                e = np.exp(sc - sc.max())
                want[i, h] = (e / e.sum()) @ v64[lo:p + 1, h // (H // G)]
        qs.append(q_tail)
        wants.append(want)
        positions += list(range(n - ql, n))
        slots += [s] * ql
    q = np.concatenate(qs).reshape(-1, H * D)
    want = np.concatenate(wants).reshape(-1, H * D)
    out = torch.empty((q.shape[0], H * D), dtype=dtype, device="cuda")
    step = FakeStep(ints(positions), ints(slots), table, None)
    ops32.paged_attention(dev(q, dtype), H, G, D, cache, step, window, 1.0 / math.sqrt(D), out, slopes=dev(slopes))
    err = np.max(np.abs(out.float().cpu().numpy() - want))
    assert err <= (2e-5 if dtype == torch.float32 else 0.02), f"max |diff| {err:.3e}"
    none = torch.empty_like(out)                                    # and the slopes do matter
    ops32.paged_attention(dev(q, dtype), H, G, D, cache, step, window, 1.0 / math.sqrt(D), none)
    assert np.max(np.abs(none.float().cpu().numpy() - want)) > 0.05
    from hf_cpu_amd.status import EngineError
    with pytest.raises(EngineError, match="slopes"):
        ops32.paged_attention(dev(q, dtype), H, G, D, cache, step, window, 1.0 / math.sqrt(D), out, slopes=dev(slopes[:-1]))


@pytest.mark.parametrize("H,G,D,page,window,lengths,q_lens", [
    (28, 4, 128, 16, 0, [2100, 700, 64, 1500], [1, 1, 1, 1]),          # decode: keys cut into chunks
    (28, 4, 128, 16, 0, [600], [600]),                                   # one prompt, whole
    (14, 2, 64, 16, 300, [1000, 333], [1, 40]),                          # window shorter than the context
    (8, 1, 96, 8, 0, [257, 31], [9, 31]),                                # one key/value head, 8 query heads
    (32, 1, 32, 4, 0, [70], [3]),                                        # 32 heads on one key/value head
    (28, 4, 128, 16, 0, [700, 90, 333, 64], [100, 90, 17, 1]),           # portions of several prompts beside a decoded token
    (12, 4, 64, 8, 50, [400, 130], [130, 130]),                          # portions longer than the window
    (6, 2, 96, 32, 0, [300], [37]),                                      # pages of 32 tokens
    (28, 4, 128, 16, 0, [1200], [1200]),                                 # one prompt whose 300 blocks are all resident: long tiles beside short ones
    (28, 4, 128, 16, 0, [1100], [1000]),                                 # the same for a portion late in a prompt
    # pages of more than 32 tokens: a block of 32 keys is part of a page, and the prompt kernel addresses them otherwise
    (28, 4, 128, 64, 0, [2100, 700, 64, 1500], [1, 1, 1, 1]),
    (28, 4, 128, 128, 0, [600], [600]),
    (14, 2, 64, 64, 300, [1000, 333], [1, 40]),                          # the window begins inside a page
    (12, 4, 64, 128, 50, [400, 130], [130, 130]),
    (28, 4, 128, 64, 0, [700, 90, 333, 64], [100, 90, 17, 1]),
    (8, 1, 96, 128, 81, [657, 31], [9, 31]),
    (28, 4, 128, 128, 0, [1100], [1000]),
])
def test_paged_attention_on_matrix_cores(ops16, H, G, D, page, window, lengths, q_lens):
    """bf16 with head_dim a multiple of 32: long contexts (many key blocks, split into chunks when
    there are few queries), groups of 7, 8 and 32 query heads, tiles that end inside a request."""
    rng = np.random.default_rng(H + D + len(lengths))
    dtype = torch.bfloat16
    ks, vs, cache, table = paged_setup(rng, lengths, G, D, page, dtype)
    qs, positions, slots, wants = [], [], [], []
    for s, (n, ql) in enumerate(zip(lengths, q_lens)):
        q_tail = rng.standard_normal((ql, H, D)).astype(np.float32)
        q_full = np.zeros((n, H, D), np.float32)
        q_full[n - ql:] = q_tail
        full = plain.attention(rounded(q_full, dtype)[n - ql:] if False else rounded(q_full, dtype),
                               rounded(ks[s], dtype), rounded(vs[s], dtype), window)
        qs.append(q_tail)
        wants.append(full[n - ql:])
        positions += list(range(n - ql, n))
        slots += [s] * ql
    q = np.concatenate(qs).reshape(-1, H * D)
    want = np.concatenate(wants).reshape(-1, H * D)
    out = torch.empty((q.shape[0], H * D), dtype=dtype, device="cuda")
    step = FakeStep(ints(positions), ints(slots), table, None)
    ops16.paged_attention(dev(q, dtype), H, G, D, cache, step, window, 1.0 / math.sqrt(D), out)
    err = np.max(np.abs(out.float().cpu().numpy() - want))
    assert err <= 0.02, f"max |diff| {err:.3e}"


def tail_attention(q_tail, k, v, window, rows=None):
    """Attention of the last queries of a sequence only (float64): q_tail [ql, H, D] stands at
    positions n-ql .. n-1 of k, v [n, G, D]; key j is visible to position p iff j <= p and,
    with a window W, p - j < W. The mask is built per query, so that long sequences stay cheap.
    ``rows``: only these queries are computed (the others stay zero)."""
    ql, H, D = q_tail.shape
    n, G, _ = k.shape
    out = np.zeros((ql, H, D))
    k64, v64 = k.astype(np.float64), v.astype(np.float64)
    for i in (range(ql) if rows is None else rows):
        p = n - ql + i
        lo = max(0, p - window + 1) if window else 0
        for h in range(H):
            g = h // (H // G)
            s = k64[lo:p + 1, g] @ q_tail[i, h].astype(np.float64) / math.sqrt(D)
            e = np.exp(s - s.max())
            out[i, h] = (e / e.sum()) @ v64[lo:p + 1, g]
    return out


@pytest.mark.parametrize("H,G,D,page,window,lengths,q_lens", [
    (28, 4, 128, 16, 0, [40000, 9000, 17], [1, 1, 1]),       # more pages than one window of page ids holds
    (8, 2, 64, 16, 0, [20000], [200]),                         # a portion late in a long prompt: few blocks, keys in chunks
    (8, 2, 64, 16, 0, [12000], [2100]),                        # the same with enough tokens for the kernel that shares keys through LDS (keys in chunks too)
    (28, 4, 32, 16, 0, [12000], [2100]),                       # and with enough blocks that each walks all its keys, through several windows of page ids
    (4, 4, 32, 8, 5000, [30000, 4999, 5001], [3, 1, 2]),       # a window far into a long sequence
    (14, 2, 64, 16, 0, [100000], [1]),                         # more chunks of keys than one merge pass takes
])
def test_paged_attention_long_contexts(ops16, H, G, D, page, window, lengths, q_lens):
    """Tens of thousands of keys: the last queries against float64 attention over the same
    rounded inputs. In each request one far key is made to matter: its dot product with the
    first query head stands out, so that a chunk that is skipped or read twice shows."""
    rng = np.random.default_rng(H + D + len(lengths))
    dtype = torch.bfloat16
    ks, vs, cache, table = paged_setup(rng, lengths, G, D, page, dtype)
    qs, positions, slots, wants = [], [], [], []
    kc = cache.k.float().cpu().numpy()
    for s, (n, ql) in enumerate(zip(lengths, q_lens)):
        q_tail = rng.standard_normal((ql, H, D)).astype(np.float32)
        lo = max(0, n - ql - window + 1) if window else 0
        far = lo + (n - ql - lo) // 3                         # visible to every query of the tail
        if n > 100:
            ks[s][far, 0] = 11.0 * math.sqrt(D) * q_tail[0, 0] / np.dot(q_tail[0, 0], q_tail[0, 0])   # score 11
            row = int(table[s, far // page].item()) * page + far % page
            kc[row, :D] = ks[s][far, 0]
        wants.append(tail_attention(rounded(q_tail, dtype), rounded(ks[s], dtype), rounded(vs[s], dtype), window))
        qs.append(q_tail)
        positions += list(range(n - ql, n))
        slots += [s] * ql
    cache = FakeCache(group=0, k=dev(kc, dtype), v=cache.v, page_tokens=page, window=0)
    q = np.concatenate(qs).reshape(-1, H * D)
    want = np.concatenate(wants).reshape(-1, H * D)
    out = torch.empty((q.shape[0], H * D), dtype=dtype, device="cuda")
    step = FakeStep(ints(positions), ints(slots), table, None)
    ops16.paged_attention(dev(q, dtype), H, G, D, cache, step, window, 1.0 / math.sqrt(D), out)
    err = np.max(np.abs(out.float().cpu().numpy() - want))
    assert err <= 0.02, f"max |diff| {err:.3e}"
    other = torch.empty_like(out)
    ops16.force_plain_attention = True
    try:
        ops16.paged_attention(dev(q, dtype), H, G, D, cache, step, window, 1.0 / math.sqrt(D), other)
    finally:
        ops16.force_plain_attention = False
    assert np.max(np.abs(other.float().cpu().numpy() - want)) <= 0.02


@pytest.mark.parametrize("H,G,D,page,window,n,ql,cut", [
    (8, 2, 64, 64, 0, 40000, 1, False),          # a decoded token whose one walk needs two windows of page ids
    (8, 2, 64, 128, 0, 70000, 1, False),
    (4, 4, 32, 64, 0, 40000, 900, False),        # a portion late in a prompt, every block walking all its keys
    (4, 4, 32, 128, 0, 70000, 900, False),
    (4, 2, 32, 64, 36000, 76109, 3, False),      # the window's first key lies inside a page: one page more than the keys fill
    (4, 4, 32, 64, 36000, 76941, 900, False),
    (8, 2, 64, 64, 0, 40000, 1, True),           # the same contexts with the keys cut into chunks
    (4, 4, 32, 128, 0, 70000, 900, True),
    (4, 2, 32, 64, 36000, 76109, 3, True),
])
def test_paged_attention_large_pages_long_walks(ops16, H, G, D, page, window, n, ql, cut):
    """Pages of 64 and 128 tokens with more keys in one walk than one window of page ids covers (511 pages
    when a walk may begin inside a page). Without ``cut`` the attention workspace is too small for partial
    results, so the kernels do not cut the keys into chunks and one wave (or block) walks them all. A far
    key in the first window and one in the second are made to matter."""
    rng = np.random.default_rng(H + D + page + n)
    dtype = torch.bfloat16
    ks, vs, cache, table = paged_setup(rng, [n], G, D, page, dtype)
    q_tail = rng.standard_normal((ql, H, D)).astype(np.float32)
    lo = max(0, n - ql - window + 1) if window else 0
    if window:
        assert (lo // 32 * 32) % page >= 32                       # the walk begins inside a page
    assert n - ql - lo > 511 * page
    kc = cache.k.float().cpu().numpy()
    for j, (far, score) in enumerate(((lo + 300, 12.0), (lo + 511 * page + 700, 13.0))):
        ks[0][far, 0] = score * math.sqrt(D) * q_tail[j % ql, 0] / np.dot(q_tail[j % ql, 0], q_tail[j % ql, 0])
        kc[int(table[0, far // page].item()) * page + far % page, :D] = ks[0][far, 0]
    cache = FakeCache(group=0, k=dev(kc, dtype), v=cache.v, page_tokens=page, window=0)
    rows = sorted({0, 1, ql // 2, ql - 2, ql - 1} & set(range(ql)))
    want = tail_attention(rounded(q_tail, dtype), rounded(ks[0], dtype), rounded(vs[0], dtype), window, rows)[rows]
    q = dev(q_tail.reshape(ql, H * D), dtype)
    out = torch.empty((ql, H * D), dtype=dtype, device="cuda")
    step = FakeStep(ints(list(range(n - ql, n))), ints([0] * ql), table, None)
    whole = ops16.attn_workspace
    if not cut:
        ops16.attn_workspace = whole[:256]
    try:
        ops16.paged_attention(q, H, G, D, cache, step, window, 1.0 / math.sqrt(D), out)
    finally:
        ops16.attn_workspace = whole
    got = out.float().cpu().numpy().reshape(ql, H, D)[rows]
    err = np.max(np.abs(got - want))
    assert err <= 0.02, f"max |diff| {err:.3e}"
    assert np.max(np.abs(want[0, 0])) > 0.3                        # the far keys carry weight


@pytest.mark.parametrize("H,G,D,page,window,rot,lengths", [
    (28, 4, 128, 16, 0, True, [2100, 700, 64, 1500, 1, 17, 16, 33]),      # the 7B shape: keys in chunks, new keys at a page's first and last row
    (14, 2, 64, 16, 0, True, [300, 2049, 5]),
    (6, 2, 96, 8, 40, True, [100, 41, 40, 39, 7]),                         # a window; three fragments a half head
    (3, 1, 32, 8, 0, True, [130, 9]),
    (8, 8, 64, 64, 0, False, [200, 65, 64]),                               # no rotation; pages of 64
    (28, 4, 128, 128, 300, True, [5000, 129, 128]),
    (14, 2, 64, 16, 0, True, [40000, 12]),                                 # more pages than one window of page ids
])
def test_decoded_tokens_rotated_stored_and_attended_in_one_kernel(ops16, H, G, D, page, window, rot, lengths):
    """Decoded tokens whose q, k and v are still the 32-bit plane a product left: ``rope_store`` waits and
    ``paged_attention`` does rotation, the store of the new key and value, and attention in one kernel. Against float64
    attention over the whole sequences (queries and keys rotated by the plain implementation), and against the two
    kernels one after the other on the same plane: the same attention output within bf16's rounding, the same cache."""
    from hf_cpu_amd.kernels.ops import Pending
    rng = np.random.default_rng(H + D + len(lengths))
    bf = torch.bfloat16
    theta = 1e6
    S = len(lengths)
    ks, vs, cache, table = paged_setup(rng, lengths, G, D, page, bf)
    raw = rng.standard_normal((S, (H + 2 * G) * D)).astype(np.float32)
    positions = [n - 1 for n in lengths]
    slot_rows = [int(table[s, (n - 1) // page].item()) * page + (n - 1) % page for s, n in enumerate(lengths)]
    half = D // 2
    inv = (theta ** (-2.0 * np.arange(half, dtype=np.float64) / D)).astype(np.float32)
    # what the step should compute, in float64 on the values as they are rounded: the new key replaces the last row
    wants = []
    for s, n in enumerate(lengths):
        q = raw[s, :H * D].reshape(1, H, D).astype(np.float64)
        k_new = raw[s, H * D:(H + G) * D].reshape(1, G, D).astype(np.float64)
        v_new = raw[s, (H + G) * D:].reshape(1, G, D).astype(np.float64)
        if rot:
            q, k_new = plain.rope(q, [n - 1], D, theta), plain.rope(k_new, [n - 1], D, theta)
        k_all = np.concatenate([rounded(ks[s][:n - 1], bf), rounded(k_new, bf)])
        v_all = np.concatenate([rounded(vs[s][:n - 1], bf), rounded(v_new, bf)])
        wants.append(tail_attention(rounded(q, bf), k_all, v_all, window)[0])
    want = np.stack(wants).reshape(S, H * D)
    step = FakeStep(ints(positions), ints(list(range(S))), table, ints(slot_rows))
    outs, caches = [], []
    for fused in (True, False):
        c = FakeCache(group=0, k=cache.k.clone(), v=cache.v.clone(), page_tokens=page, window=0)
        qkv = torch.zeros((S, (H + 2 * G) * D), dtype=bf, device="cuda")
        ops16.workspace[:raw.size * 4].view(torch.float32).copy_(dev(raw).view(-1))
        ops16._pending = Pending(qkv, 1, None, False)
        ops16.fuse_rows = fused
        try:
            ops16.rope_store(qkv, step.positions, dev(inv) if rot else None, D if rot else 0, H, G, D, c, step.group(0).slot_map)
            assert (ops16._lazy_rope is not None) == fused
            out = torch.empty((S, H * D), dtype=bf, device="cuda")
            ops16.paged_attention(qkv, H, G, D, c, step, window, 1.0 / math.sqrt(D), out)
            assert ops16._lazy_rope is None and ops16._pending is None
        finally:
            ops16.fuse_rows = True
        outs.append(out.float().cpu().numpy())
        caches.append((c.k.float().cpu().numpy(), c.v.float().cpu().numpy()))
    for name, got in zip(("one kernel", "two kernels"), outs):
        err = np.max(np.abs(got - want))
        assert err <= 0.02, f"{name}: max |diff| {err:.3e}"
    assert np.max(np.abs(outs[0] - outs[1])) <= 0.02
    for a, b in zip(caches[0], caches[1]):                 # the same rows written, to a rounding of the rotation
        assert np.max(np.abs(a - b)) <= 0.04 and np.mean(a != b) < 1e-3
    k_rows = caches[0][0][slot_rows]
    assert np.max(np.abs(k_rows - np.stack([w for w in (rounded(plain.rope(raw[s, H * D:(H + G) * D].reshape(1, G, D).astype(np.float64), [lengths[s] - 1], D, theta) if rot else raw[s, H * D:(H + G) * D].reshape(1, G, D), bf).reshape(G * D) for s in range(S))]))) <= 0.04


def test_attention_special_cases(ops32):
    """A single query at position 0 returns value row 0 exactly; equal scores (zero query)
    return the mean of the visible value rows (softmax of equal numbers)."""
    rng = np.random.default_rng(1)
    H, G, D, page = 2, 1, 32, 8
    ks, vs, cache, table = paged_setup(rng, [1, 40], G, D, page, torch.float32)
    q = np.zeros((2, H * D), np.float32)
    q[0] = rng.standard_normal(H * D)
    out = torch.empty((2, H * D), dtype=torch.float32, device="cuda")
    step = FakeStep(ints([0, 39]), ints([0, 1]), table, None)
    ops32.paged_attention(dev(q), H, G, D, cache, step, 0, 1.0, out)
    got = out.cpu().numpy()
    assert np.array_equal(got[0].reshape(H, D), np.repeat(vs[0][0], H, axis=0))
    assert np.max(np.abs(got[1].reshape(H, D) - vs[1].mean(axis=0))) < 1e-6
    ops32.paged_attention(dev(q), H, G, D, cache, step, 10, 1.0, out)     # window of 10: mean of the last 10
    assert np.max(np.abs(out.cpu().numpy()[1].reshape(H, D) - vs[1][30:].mean(axis=0))) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,rot", [(4, 2, 16, 16), (3, 1, 32, 32), (5, 5, 48, 32), (2, 1, 128, 128)])
def test_rope_store(ops32, dtype, H, G, D, rot):
    rng = np.random.default_rng(D + rot)
    T, base = 9, 1e4 if D < 100 else 1e6
    positions = [0, 1, 2, 77, 500, 4095, 3, 30000, 17]
    qkv = rng.standard_normal((T, (H + 2 * G) * D)).astype(np.float32)
    slot_map = [4, 0, 11, 7, 2, 9, 1, 3, 10]
    t_qkv = dev(qkv, dtype)
    cache = FakeCache(group=0, k=torch.zeros((12, G * D), dtype=dtype, device="cuda"),
                      v=torch.zeros((12, G * D), dtype=dtype, device="cuda"), page_tokens=4)
    i = np.arange(rot // 2, dtype=np.float64)
    inv_freq = dev((base ** (-2.0 * i / rot)).astype(np.float32))
    ops32.rope_store(t_qkv, ints(positions), inv_freq, rot, H, G, D, cache, ints(slot_map))
    src = rounded(qkv, dtype)
    q_want = plain.rope(src[:, :H * D].reshape(T, H, D), positions, rot, base).reshape(T, H * D)
    k_want = plain.rope(src[:, H * D:(H + G) * D].reshape(T, G, D), positions, rot, base).reshape(T, G * D)
    v_want = src[:, (H + G) * D:]
    # the angle is an fp32 product: at position 30000 it is off by up to 30000 * 2^-24 rad
    tol = 4e-3 if dtype == torch.float32 else 0.03
    got = t_qkv.float().cpu().numpy()
    assert np.max(np.abs(got[:, :H * D] - q_want)) <= tol
    small = [t for t, p in enumerate(positions) if p < 100]
    assert np.max(np.abs(got[small, :H * D] - q_want[small])) <= (1e-5 if dtype == torch.float32 else 0.03)
    kc, vc = cache.k.float().cpu().numpy(), from_value_layout(cache.v.float().cpu().numpy(), 4)
    assert np.max(np.abs(kc[slot_map] - k_want)) <= tol
    assert np.array_equal(vc[slot_map], v_want.astype(np.float32))
    assert np.array_equal(got[0, :H * D], src[0, :H * D].astype(np.float32)), "position 0 is the identity"
    unused = [r for r in range(12) if r not in slot_map]
    assert float(cache.k[unused].abs().max()) == 0.0


@pytest.mark.parametrize("H,G,D,rot,page,T", [(4, 2, 16, 16, 8, 547), (28, 4, 128, 128, 16, 700), (5, 5, 48, 32, 8, 521),
                                              (3, 1, 64, 64, 4, 520), (2, 2, 32, 32, 16, 576)])
def test_rope_store_for_prompt_portions(ops16, H, G, D, rot, page, T):
    """bf16 with many tokens takes a kernel of its own (8 tokens per block, 16 bytes per lane,
    values through LDS): the result must be, bit for bit, what the kernel for few tokens gives:
    token runs that fill cache rows in order (aligned to 8 and not), scattered rows, a last
    block of fewer than 8 tokens, a part of the head that is not rotated, without a cache."""
    rng = np.random.default_rng(T + D)
    dtype = torch.bfloat16
    qkv = rng.standard_normal((T, (H + 2 * G) * D)).astype(np.float32)
    positions = [int(p) for p in np.concatenate([np.arange(100, 100 + T - 9), rng.integers(0, 30000, 9)])]
    n_rows = (T + 40) // page * page + page
    rows = list(range(16, 16 + 24)) + list(range(43, 43 + 11))          # a run aligned to 8, then one that is not
    rest = [r for r in rng.permutation(n_rows) if r not in rows]
    slot_map = (rows + [int(r) for r in rest])[:T]
    i = np.arange(rot // 2, dtype=np.float64)
    inv_freq = dev((1e4 ** (-2.0 * i / rot)).astype(np.float32))

    def run(tokens):
        t_qkv = dev(qkv[tokens], dtype)
        cache = FakeCache(group=0, k=torch.zeros((n_rows, G * D), dtype=dtype, device="cuda"),
                          v=torch.zeros((n_rows, G * D), dtype=dtype, device="cuda"), page_tokens=page)
        ops16.rope_store(t_qkv, ints([positions[t] for t in tokens]), inv_freq, rot, H, G, D, cache,
                         ints([slot_map[t] for t in tokens]))
        return t_qkv, cache
    all_q, all_c = run(list(range(T)))
    few_q = torch.empty_like(all_q)
    few_c = FakeCache(k=torch.zeros_like(all_c.k), v=torch.zeros_like(all_c.v))
    for a in range(0, T, 7):                                            # 7 tokens at a time: the other kernel
        toks = list(range(a, min(a + 7, T)))
        q, c = run(toks)
        few_q[toks] = q
        for t in toks:
            r = slot_map[t]
            few_c.k[r] = c.k[r]
        pages = sorted({slot_map[t] // page for t in toks})
        for pg in pages:
            blk = slice(pg * page, (pg + 1) * page)
            few_c.v[blk] = torch.where(c.v[blk] != 0, c.v[blk], few_c.v[blk])
    assert torch.equal(all_q, few_q) and torch.equal(all_c.k, few_c.k) and torch.equal(all_c.v, few_c.v)
    src = rounded(qkv, dtype)                                           # and both are right
    k_want = plain.rope(src[:, H * D:(H + G) * D].reshape(T, G, D), positions, rot, 1e4).reshape(T, G * D)
    assert np.max(np.abs(all_c.k.float().cpu().numpy()[slot_map] - k_want)) <= 0.03
    vc = from_value_layout(all_c.v.float().cpu().numpy(), page)
    assert np.array_equal(vc[slot_map], src[:, (H + G) * D:].astype(np.float32))
    no_cache = dev(qkv, dtype)                                          # without a cache: keys are rotated in place
    ops16.rope_store(no_cache, ints(positions), inv_freq, rot, H, G, D, FakeCache(group=0, k=None, v=None, page_tokens=page), None)
    assert torch.equal(no_cache[:, :H * D], all_q[:, :H * D])
    assert np.max(np.abs(no_cache[:, H * D:(H + G) * D].float().cpu().numpy() - k_want)) <= 0.03
    assert torch.equal(no_cache[:, (H + G) * D:], dev(qkv, dtype)[:, (H + G) * D:])


def test_rope_relative_position(ops32):
    """<rope(q, p + s), rope(k, p' + s)> does not depend on the shift s: only distances count.
    A wrong sign or a wrong pairing breaks this."""
    rng = np.random.default_rng(5)
    H, G, D = 1, 1, 64
    qkv = rng.standard_normal((1, 3 * D)).astype(np.float32)
    i = np.arange(D // 2, dtype=np.float64)
    inv_freq = dev((1e4 ** (-2.0 * i / D)).astype(np.float32))
    dots = []
    for shift in (0, 5, 100):
        rows = torch.cat([dev(qkv), dev(qkv)])
        cache = FakeCache(group=0, k=torch.zeros((2, D), device="cuda"), v=torch.zeros((2, D), device="cuda"),
                          page_tokens=2)
        ops32.rope_store(rows, ints([9 + shift, 2 + shift]), inv_freq, D, H, G, D, cache, ints([0, 1]))
        dots.append(float((rows[0, :D].double() * cache.k[1].double()).sum()))
    assert abs(dots[0] - dots[1]) < 1e-4 and abs(dots[0] - dots[2]) < 1e-4
    want = float((plain.rope(qkv[:, :D].reshape(1, 1, D).astype(np.float64), [9], D, 1e4) *
                  plain.rope(qkv[:, D:2 * D].reshape(1, 1, D).astype(np.float64), [2], D, 1e4)).sum())
    assert abs(dots[0] - want) < 1e-4


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu(ops32, dtype):
    rng = np.random.default_rng(3)
    gu = (rng.standard_normal((5, 2 * 177)) * 3).astype(np.float32)
    out = torch.empty((5, 177), dtype=dtype, device="cuda")
    ops32.swiglu(dev(gu, dtype), out)
    src = rounded(gu, dtype)
    want = plain.silu(src[:, :177]) * src[:, 177:]
    tol = 1e-5 if dtype == torch.float32 else 0.02
    assert np.max(np.abs(out.float().cpu().numpy() - want)) <= tol * np.max(np.abs(want))
    one = torch.empty((1, 2), dtype=torch.float32, device="cuda")
    ops32.swiglu(dev(np.array([[0.0, 1.0, 5.0, 1.0]], np.float32)), one)     # silu(0) = 0, silu(1) = 0.7310585786
    assert float(one[0, 0]) == 0.0 and abs(float(one[0, 1]) - 0.7310585786) < 1e-6


def test_argmax_and_topk(ops32):
    rng = np.random.default_rng(8)
    logits = rng.standard_normal((6, 1000)).astype(np.float32)
    logits[1, 17] = logits[1, 900] = 9.0        # a tie: the lower id wins
    logits[2, :] = 0.5                          # all equal
    logits[3, 999] = 50.0
    t = dev(logits)
    assert ops32.argmax(t).cpu().tolist() == [int(np.argmax(r)) for r in logits]
    assert ops32.argmax(t).cpu().tolist()[1:4] == [17, 0, 999]
    ids, vals, stats = ops32.topk(t, 40)
    for r in range(6):
        order = sorted(range(1000), key=lambda i: (-logits[r, i], i))[:40]
        assert ids[r].cpu().tolist() == order
        assert np.array_equal(vals[r].cpu().numpy(), logits[r, order])
        mx = logits[r].max()
        lse = np.log(np.sum(np.exp(logits[r].astype(np.float64) - mx)))
        assert float(stats[r, 0]) == mx and abs(float(stats[r, 1]) - lse) < 1e-5
    big_np = rng.standard_normal((3, 152064)).astype(np.float32)
    big_np[1, ::7] = 2.5                        # thousands of ties around the cut
    big_np[2] = np.round(big_np[2] * 4) / 4     # few distinct values, negative ones among them
    big_np[2, 5] = -np.inf
    big = dev(big_np)
    assert ops32.argmax(big).cpu().tolist() == big.argmax(dim=1).cpu().tolist()
    for k in (1, 2, 40, 333, 1024):             # the ordered best-k at other k, with ties across the cut
        ids, vals, stats = ops32.topk(big, k)
        for r in range(3):
            order = np.lexsort((np.arange(152064), -big_np[r]))[:k]
            assert np.array_equal(ids[r].cpu().numpy(), order), f"k={k} row {r}"
            assert np.array_equal(vals[r].cpu().numpy(), big_np[r, order])
    zeros_np = np.round(rng.standard_normal((2, 5000)).astype(np.float32) * 0.3)     # 0.0, -0.0 and a few +-1: the cut
    zeros_np[1] = np.minimum(zeros_np[1], 0.0)                                       # falls among zeros of either sign,
    for k in (1, 40, 1024):                                                          # which are one value: ids decide
        ids, vals, _ = ops32.topk(dev(zeros_np), k)
        for r in range(2):
            order = np.argsort(-zeros_np[r], kind="stable")[:k]
            assert np.array_equal(ids[r].cpu().numpy(), order), f"signed zeros, k={k} row {r}"
            assert np.array_equal(vals[r].cpu().numpy(), zeros_np[r, order])
    small = rng.standard_normal((2, 37)).astype(np.float32)     # fewer ids than threads; k = all of them
    ids, vals, stats = ops32.topk(dev(small), 37)
    assert ids.cpu().tolist() == [list(np.lexsort((np.arange(37), -r))) for r in small]
    _, _, stats = ops32.topk(dev(small), 0)
    assert abs(float(stats[1, 1]) - np.log(np.sum(np.exp(small[1].astype(np.float64) - small[1].max())))) < 1e-5


@pytest.mark.parametrize("V", [5, 1000, 1025, 4096, 152064])
def test_order_rows(ops32, V):
    """A whole row in order (logit descending, id ascending) against numpy's stable sort: random
    logits with many ties (values drawn from a few hundred numbers), signed zeros, huge and tiny
    values; all rows, and a choice of rows."""
    rng = np.random.default_rng(V)
    R = 5
    pool = np.concatenate([rng.standard_normal(300).astype(np.float32) * 7, np.array([0.0, -0.0, 1e30, -1e30, 1e-40, -1e-40], np.float32)])
    logits = pool[rng.integers(0, len(pool), (R, V))]
    logits[1] = rng.standard_normal(V).astype(np.float32)            # a row without ties
    logits[2] = 3.25                                                  # a row of equal values: ids in order
    dev_logits = torch.from_numpy(logits).cuda()
    for chosen in (None, [3, 0]):
        rows = None if chosen is None else torch.tensor(chosen, dtype=torch.int32, device="cuda")
        ids, vals = (t.cpu().numpy() for t in ops32.order_rows(dev_logits, rows))
        for j, r in enumerate(range(R) if chosen is None else chosen):
            want = np.argsort(-logits[r], kind="stable")            # 0.0 and -0.0 are a tie here as in the kernel
            assert np.array_equal(ids[j], want), f"row {r}: first difference at {int(np.argmax(ids[j] != want))}"
            assert np.array_equal(vals[j], logits[r][want])           # == : the kernel returns 0.0 for -0.0


@pytest.mark.parametrize("V", [1, 7, 1000, 4097, 152064])
def test_draw_rows(ops32, V):
    """The device's draw over a whole ordered row against the plain sampler (tests/plain.py, from the row's
    logits, with its own ordering and its own exponential) with the same uniform numbers: the same token,
    row for row; at the largest sizes, where the plain sampler's scalar loops take seconds a row, eight rows
    against it and all of them against its vectorised stand-in in tests/host_draw.py. The rows differ in
    temperature, in each cut being on or off, and in how peaked they are (a peaked row ends the
    top-p cut within a few candidates, a flat one takes it far into the row: past several of the
    kernel's pieces); uniform numbers include 0 and the largest below 1."""
    from hf_cpu_amd.sampling import SamplerParams
    from host_draw import pick
    rng = np.random.default_rng(V + 1)

    class Fixed:
        def __init__(self, u):
            self.u = u

        def uniform(self):
            return self.u

    cases = []
    for temp in (0.05, 0.8, 1.0, 4.5):
        for top_k in (0, 3, 2000):
            for top_p in (0.0, 0.3, 0.95, 1.0):
                for min_p in (0.0, 0.05, 0.9):
                    cases.append((temp, top_k, top_p, min_p))
    rng.shuffle(cases)
    cases = cases[:96]
    R = len(cases)
    logits = rng.standard_normal((R, V)).astype(np.float32) * rng.choice([0.01, 1.0, 6.0], (R, 1)).astype(np.float32)
    logits[::5] = np.round(logits[::5] * 2) / 2                          # rows with many ties
    us = rng.integers(0, 1 << 24, R).astype(np.float32) / np.float32(1 << 24)
    us[:4] = [0.0, (2.0 ** 24 - 1) / 2.0 ** 24, 0.5, 2.0 ** -24]
    ids, vals = ops32.order_rows(torch.from_numpy(logits).cuda())
    host_ids, host_vals = ids.cpu().numpy(), vals.cpu().numpy()
    numbers = np.array([(t, tp, mp, u) for (t, _, tp, mp), u in zip(cases, us)], dtype=np.float32)
    cuts = np.array([k if 0 < k < V else V for _, k, _, _ in cases], dtype=np.int32)
    got = ops32.draw_rows(ids, vals, torch.from_numpy(numbers).cuda(), torch.from_numpy(cuts).cuda()).cpu().numpy()
    by_plain = range(R) if V <= 1000 else range(0, R, 12)
    for r, (temp, top_k, top_p, min_p) in enumerate(cases):
        what = f"row {r}: temp {temp} top_k {top_k} top_p {top_p} min_p {min_p} u {us[r]}"
        if r in by_plain:
            assert int(got[r]) == plain.sample(logits[r], temp, top_k, top_p, min_p, Fixed(us[r])), what
        want = pick(host_ids[r, :cuts[r]], host_vals[r, :cuts[r]], SamplerParams(temp, top_k, top_p, min_p), Fixed(us[r]))
        assert int(got[r]) == want, what


def test_sampler_with_rows_of_every_kind_in_one_step(ops32):
    """One call of the sampler for rows that take every one of its paths (greedy, the best-k
    kernel, the whole vocabulary with top-k off, a top-k beyond the best-k kernel's 1024, greedy
    with log-probabilities) gives each row what the plain sampler gives it alone, and moves each
    request's generator on by one draw (two calls in a row are compared)."""
    from hf_cpu_amd.sampling import Rng, Sampler, SamplerParams
    rng = np.random.default_rng(77)
    V = 3001
    kinds = [(0.0, 40, 0.95, 0.05), (0.8, 40, 0.95, 0.05), (1.3, 0, 1.0, 0.0), (0.7, 2000, 0.9, 0.0), (0.0, 0, 1.0, 0.0),
             (2.0, 0, 0.5, 0.02), (0.9, 1, 1.0, 0.0), (1.0, 1024, 1.0, 0.0), (1.0, 1025, 1.0, 0.0)]
    wants = [(SamplerParams(*k), Rng(100 + i), 2 if i == 4 else 0) for i, k in enumerate(kinds)]
    theirs = [plain.Rng(100 + i) for i in range(len(kinds))]
    sampler = Sampler(ops32)
    for call in range(2):
        logits = (rng.standard_normal((len(kinds), V)) * 3).astype(np.float32)
        got = sampler.sample(torch.from_numpy(logits).cuda(), wants)
        for i, k in enumerate(kinds):
            assert got[i].token == plain.sample(logits[i], *k, theirs[i]), f"call {call}, row {i}: {k}"
        assert [t for t, _ in got[4].top] == [int(t) for t in np.argsort(-logits[4], kind="stable")[:2]]


@pytest.mark.parametrize("greedy", [True, False])
def test_sampling_starts_without_waiting_for_the_stream(ops32, greedy):
    """``sample_start`` only enqueues: with a long piece of work on the stream before it (the step that the
    scheduler has just enqueued), it returns while that work still runs, for greedy rows and for rows drawn
    from their best k with the reference's defaults (the rows' numbers travel from pinned memory; from
    pageable memory the copy would make the host wait for the whole stream). The tokens are the plain
    sampler's all the same."""
    from hf_cpu_amd.sampling import Rng, Sampler, SamplerParams
    rng = np.random.default_rng(5)
    V, R = 4099, 6
    params = (0.0, 40, 0.95, 0.05) if greedy else (0.8, 40, 0.95, 0.05)
    sampler = Sampler(ops32)
    big = torch.randn((4096, 4096), device="cuda")
    junk = torch.empty_like(big)
    for trial in range(3):                      # the first trial also allocates the pinned buffers
        logits = (rng.standard_normal((R, V)) * 3).astype(np.float32)
        dl = torch.from_numpy(logits).cuda()
        wants = [(SamplerParams(*params), Rng(50 + trial * R + i), 0) for i in range(R)]
        torch.cuda.synchronize()
        for _ in range(60):                     # about a quarter of a second of fp32 products
            torch.mm(big, big, out=junk)
        busy = torch.cuda.Event()
        busy.record()
        started = sampler.sample_start(dl, wants)
        still_running = not busy.query()
        assert started.device_tokens is not None
        if trial:
            assert still_running, "sample_start waited for the work enqueued before it"
        got = [c.token for c in started.finish()]
        theirs = [plain.Rng(50 + trial * R + i) for i in range(R)]
        assert got == [plain.sample(logits[i], *params, theirs[i]) for i in range(R)]


def test_kernels_refuse_what_they_cannot_do(ops32):
    from hf_cpu_amd.status import EngineError
    with pytest.raises(EngineError, match="head_dim"):
        cache = FakeCache(group=0, k=torch.zeros((16, 512), device="cuda"), v=torch.zeros((16, 512), device="cuda"),
                          page_tokens=16, window=0)
        step = FakeStep(ints([0]), ints([0]), ints(np.zeros((1, 4))), None)
        ops32.paged_attention(torch.zeros((1, 512), device="cuda"), 1, 1, 512, cache, step, 0, 1.0,
                              torch.zeros((1, 512), device="cuda"))
    with pytest.raises(EngineError, match="shapes"):
        ops32.gemm(torch.zeros((2, 3), device="cuda"), torch.zeros((4, 5), device="cuda"),
                   torch.zeros((2, 4), device="cuda"))
    with pytest.raises(EngineError, match="multiple"):
        cache = FakeCache(group=0, k=torch.zeros((16, 32), device="cuda"), v=torch.zeros((16, 32), device="cuda"),
                          page_tokens=16, window=0)
        step = FakeStep(ints([0]), ints([0]), ints(np.zeros((1, 4))), None)
        ops32.paged_attention(torch.zeros((1, 48), device="cuda"), 3, 2, 16, cache, step, 0, 1.0,
                              torch.zeros((1, 48), device="cuda"))


def test_probes_of_the_device_peaks(ops16):
    """The bench's yardsticks: a streaming read, a copy, the matrix cores on random and on zero operands.
    Sanity of the numbers, not their size: a read faster than the published peak or a burn slower with zeros
    than with random operands would mean a broken probe."""
    from hf_cpu_amd.probe import measure_peaks
    p = measure_peaks(ops16, read_bytes=256 << 20, reps=3, mfma_iters=1 << 12)
    assert 1000 < p["hbm_copy_GBps"] and 1000 < p["hbm_read_GBps"] < 8000
    assert 200 < p["mfma_bf16_TFLOPs"] <= p["mfma_bf16_zero_TFLOPs"] * 1.05 < 2700


@pytest.mark.parametrize("M,N,K", [(1, 4608, 3584), (8, 3584, 18944), (3, 2016, 896), (9, 37888, 3584), (16, 1000, 1024),
                                   (17, 4608, 3584), (32, 3584, 3584), (8, 152064, 3584), (5, 33, 8192), (32, 40, 16384),
                                   (7, 37888, 3584), (2, 3584, 3584), (8, 9000, 1024), (4, 70000, 128), (6, 65530, 192),
                                   (12, 3584, 18944), (16, 4608, 3584), (13, 70000, 128)])
def test_products_of_few_rows_streamed_wave_by_wave(ops16, M, N, K):
    """The product for up to 16 rows in which every wave streams a run of the weights by itself (gemm_wave.hip),
    and the tiled product that takes more rows, against a float64 product of the same bf16 operands: widths that are no multiple of the 32-column tiles (the last tile repeats its last row), runs of
    a few units and of hundreds, tiles that one wave covers whole, that the waves of one block share and that
    several blocks share, results stored, accumulated and left for the next kernel; and the same bits
    twice (no wave's sum depends on another's timing)."""
    torch.manual_seed(M + N)
    a = (torch.randn((M, K), device="cuda") * 0.5).bfloat16()
    w = (torch.randn((N, K), device="cuda") / K ** 0.5).bfloat16()
    bias = torch.randn((N,), device="cuda")
    want = a.double() @ w.double().T
    out = torch.empty((M, N), device="cuda")
    ops16.gemm(a, w, out, bias=bias)
    err = ((out.double() - (want + bias.double())).abs().max() / want.abs().max()).item()
    assert err < 1e-5, f"stored: {err:.3e}"
    again = torch.empty_like(out)
    ops16.gemm(a, w, again, bias=bias)
    assert torch.equal(out, again)
    x = torch.randn((M, N), device="cuda")
    x0 = x.clone()
    ops16.gemm(a, w, x, accumulate=True, defer=True)            # left as planes; settle adds them up
    ops16.settle()
    err = ((x.double() - (x0.double() + want)).abs().max() / want.abs().max()).item()
    assert err < 1e-5, f"accumulated: {err:.3e}"
    o16 = torch.empty((M, N), device="cuda", dtype=torch.bfloat16)
    ops16.gemm(a, w, o16)
    err = ((o16.double() - want).abs().max() / want.abs().max()).item()
    assert err < 1e-2, f"bf16 output: {err:.3e}"
