"""Each kernel of libvla_seq_gfx950.so alone against the float64 reference of its equation
(tests/lusadra_oracle.py): row-wise stream layers, the paged sliding-window key attention and the
gated linear recurrence.  Inputs are float32 unless a test says otherwise, so the comparison bar is
float32 rounding; shapes include sizes that are not multiples of the wave (64), of a block or of
each other, and values that a typical model makes equal (heads = kv heads, window 1, one head).

Where random inputs would hide an off-by-one, the inputs are built so that one key decides the
result: a query and one key share a long vector, so that key takes all the softmax weight when
it is visible and the result is far from it when it is not."""
import math

import pytest
import torch

from tests import lusadra_oracle as R

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def ops():
    from vllm_legacy_amd import _seq_ops
    return _seq_ops


def close(got, want, tol=2e-5):
    got, want = got.detach().cpu().to(R.F), want.to(R.F)
    err = float((got - want).abs().max() / max(1.0, float(want.abs().max())))
    assert err <= tol, err


# ------------------------------------------------------------------------------ stream layers


@pytest.mark.parametrize("width", [2, 30, 64, 257, 2500])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_positions(width, dtype):
    g = torch.Generator().manual_seed(width)
    table = torch.randn(50, width, generator=g).to(dtype)
    ids = torch.randint(0, 50, (9, ), generator=g)
    pos = torch.tensor([0, 1, 2, 3, 63, 64, 999, 4095, 70000])
    i2 = torch.arange(0, width, 2, dtype=torch.float32)
    inv = torch.pow(torch.tensor(10000.0), -i2 / width)
    out = torch.empty(9, width, dtype=torch.float32, device=DEV)
    ops().embed_positions(out, table.to(DEV), ids.to(DEV), pos.to(DEV), inv.to(DEV))
    close(out, table[ids].to(R.F) + R.sinusoid(pos, width), 1e-5)


@pytest.mark.parametrize("width", [1, 48, 256, 1000, 2304])
@pytest.mark.parametrize("adds", [(False, False), (True, False), (False, True), (True, True)])
def test_scalar_rms_norm(width, adds):
    g = torch.Generator().manual_seed(width)
    x = torch.randn(5, width, generator=g) * 3
    rows = torch.randn(5, width, generator=g) if adds[0] else None
    row = torch.randn(width, generator=g) if adds[1] else None
    gain = torch.tensor([1.3])
    xs = x.clone().to(DEV)
    out = torch.empty(5, width, dtype=torch.float32, device=DEV)
    ops().scalar_rms_norm(out, xs, gain.to(DEV), 1e-5, None if rows is None else rows.to(DEV),
                          None if row is None else row.to(DEV))
    want_x = x.to(R.F) + (0 if rows is None else rows.to(R.F)) + (0 if row is None else row.to(R.F))
    close(xs, want_x, 1e-6)
    close(out, R.scalar_rms_norm(want_x, 1.3, 1e-5))


@pytest.mark.parametrize("features", [1, 40, 256, 1100, 2100])
def test_poly_norm_on_strided_rows(features):
    g = torch.Generator().manual_seed(features)
    wide = torch.randn(4, features + 13, generator=g).to(DEV) * 2
    z = wide[:, 5:5 + features]
    coef = torch.tensor([0.7, -0.4, 0.25, 0.1])
    dst = torch.zeros(4, features + 3, dtype=torch.float32, device=DEV)
    ops().poly_norm(dst[:, 3:], z, coef.to(DEV), 1e-5)
    close(dst[:, 3:], R.poly_norm(z.cpu().to(R.F), coef, 1e-5))
    assert float(dst[:, :3].abs().max()) == 0.0


def test_poly_norm_bf16_rounds_only_at_the_ends():
    g = torch.Generator().manual_seed(1)
    z = (torch.randn(3, 300, generator=g) * 2).bfloat16().to(DEV)
    coef = torch.tensor([0.5, 0.3, 0.2, 0.0])
    out = torch.empty_like(z)
    ops().poly_norm(out, z, coef.to(DEV), 1e-5)
    want = R.poly_norm(z.cpu().to(R.F), coef, 1e-5)
    assert torch.equal(out.cpu(), want.to(torch.float32).bfloat16()) or \
        float((out.cpu().to(R.F) - want).abs().max()) <= 2.0**-8 * float(want.abs().max())


@pytest.mark.parametrize("H,V", [(1, 1), (2, 16), (3, 64), (2, 100), (1, 300)])
def test_gated_head_rms_norm(H, V):
    g = torch.Generator().manual_seed(H * V)
    o = torch.randn(6, H, V, generator=g)
    w = torch.randn(V, generator=g)
    gate = torch.randn(6, H * V + 4, generator=g).to(DEV)[:, 4:]
    out = torch.empty(6, H * V, dtype=torch.float32, device=DEV)
    ops().gated_head_rms_norm(out, o.to(DEV), w.to(DEV), gate, 1e-5, 0.9)
    close(out, R.gated_head_norm(o.to(R.F), w.to(R.F), gate.cpu().to(R.F), 1e-5, 0.9))


def test_residual_add():
    x = torch.randn(1000).to(DEV)
    y = torch.randn(1000).bfloat16().to(DEV)
    want = x.cpu() + y.cpu().float()
    ops().residual_add(x, y)
    assert torch.equal(x.cpu(), want)


# ------------------------------------------------------------------------------ window attention


class PagedKeys:
    """A key cache whose block table is a random permutation, filled through the product's write
    kernel; `attend` runs the product kernel for rows lo..hi-1 of the sequence."""

    def __init__(self, G, D, block_size, max_tokens, dtype=torch.float32, seed=0, spare=3):
        nb = (max_tokens + block_size - 1) // block_size + spare
        g = torch.Generator().manual_seed(seed)
        self.table = torch.randperm(nb, generator=g)[:nb - spare].to(torch.int32)
        self.bs, self.G, self.D = block_size, G, D
        # stale data everywhere: nothing may depend on a block being clean
        self.cache = (torch.randn(nb, block_size, G, D, generator=g) * 50).to(dtype).to(DEV)

    def attend(self, q, k, gate, lo, hi, H, window, scale, slopes, coef=0.0, every=1.0, out_scale=1.0,
               kernel="auto"):
        """kernel: "auto" (rows, picked per shape: matrix cores for 16-bit rows), "grouped" (rows, no
        matrix cores), "simple" (one wave per row and head), "tiles" (runs of rows on the matrix
        cores, 16-bit only)."""
        n = hi - lo
        pos = torch.arange(lo, hi)
        slots = (self.table[pos // self.bs].long() * self.bs + pos % self.bs).to(DEV)
        ops().key_cache_write(self.cache, k[lo:hi].to(DEV), slots)
        out = torch.empty(n, H * self.D, dtype=q.dtype, device=DEV)
        sl = None if slopes is None else torch.tensor(slopes, dtype=torch.float32, device=DEV)
        if kernel == "tiles":
            i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)      # noqa: E731
            ops().window_attention_tiles(out, q[lo:hi].to(DEV), None if gate is None else gate[lo:hi].to(DEV),
                                         self.cache, self.table[None].contiguous().to(DEV), i32([0, n]), i32([lo]), n,
                                         sl, H, window, scale, coef, every, out_scale)
            return out.cpu()
        ops().set_window_kernel({"simple": 1, "grouped": 2}.get(kernel, 0))
        try:
            self._rows(out, q, gate, lo, hi, pos, sl, H, window, scale, coef, every, out_scale)
        finally:
            ops().set_window_kernel(0)
        return out.cpu()

    def _rows(self, out, q, gate, lo, hi, pos, slopes_t, H, window, scale, coef, every, out_scale):
        n = hi - lo
        ops().window_attention(out, q[lo:hi].to(DEV), None if gate is None else gate[lo:hi].to(DEV), self.cache,
                               self.table[None].contiguous().to(DEV), torch.zeros(n, dtype=torch.int32, device=DEV),
                               pos.to(DEV), slopes_t, H, window, scale, coef, every, out_scale)


CASES = [  # H, G, D, window, block, n
    (6, 2, 48, 7, 8, 40),
    (3, 3, 80, 70, 16, 150),     # two key tiles per query
    (5, 1, 256, 33, 32, 70),
    (4, 4, 16, 1, 4, 12),        # a window of one: every token sees itself only
    (2, 1, 64, 0, 16, 90),       # no window: everything before
    (1, 1, 20, 64, 64, 130),     # window = one tile exactly
    (7, 7, 8, 65, 16, 140),
]


@pytest.mark.parametrize("kernel", ["auto", "simple"])
@pytest.mark.parametrize("H,G,D,window,bs,n", CASES)
def test_window_attention_whole_portions_and_single_tokens(H, G, D, window, bs, n, kernel):
    g = torch.Generator().manual_seed(n)
    q, k = torch.randn(n, H * D, generator=g), torch.randn(n, G * D, generator=g)
    gate = torch.randn(n, H * D, generator=g)
    slopes, scale, coef, every = R.head_slopes(H), D**-0.5, 0.4, 3
    want = R.windowed_key_attention(q.to(R.F), k.to(R.F), torch.arange(n), H, G, D, window, scale, coef, every, slopes)
    want = want * torch.sigmoid(gate.to(R.F)) * 0.6
    cuts = {"whole": [n], "portions": [2, 3, bs, bs + 1, 1, 1, 2, 17], "tokens": [1] * n}
    for name, sizes in cuts.items():
        pk = PagedKeys(G, D, bs, n, seed=len(name))
        got, lo = [], 0
        i = 0
        while lo < n:
            step = min(sizes[i % len(sizes)], n - lo)
            got.append(pk.attend(q, k, gate, lo, lo + step, H, window, scale, slopes, coef, every, 0.6, kernel))
            lo += step
            i += 1
        close(torch.cat(got), want, 3e-5)


TILE_CASES = [  # H, G, D, window, block, n
    (6, 2, 32, 7, 8, 70),
    (3, 3, 96, 70, 16, 150),
    (16, 2, 128, 33, 32, 100),    # eight query heads per KV head: two chunks of four
    (4, 4, 64, 1, 4, 40),
    (2, 1, 64, 0, 16, 90),
    (5, 1, 128, 64, 16, 130),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("H,G,D,window,bs,n", TILE_CASES)
def test_window_attention_tiles(H, G, D, window, bs, n, dtype):
    """The matrix-core kernel on whole prompts and on portions that start anywhere (a tile's first
    row in the middle of a page and of a window).  Inputs are 16-bit; the bar is the output's own
    rounding (scores and weights are fp32 inside)."""
    g = torch.Generator().manual_seed(n + H)
    q, k = torch.randn(n, H * D, generator=g).to(dtype), torch.randn(n, G * D, generator=g).to(dtype)
    gate = torch.randn(n, H * D, generator=g).to(dtype)
    slopes, scale, coef, every = R.head_slopes(H), D**-0.5, 0.4, 3
    want = R.windowed_key_attention(q.to(R.F), k.to(R.F), torch.arange(n), H, G, D, window, scale, coef, every, slopes)
    want = want * torch.sigmoid(gate.to(R.F)) * 0.6
    ulp = 2.0**-8 if dtype == torch.bfloat16 else 2.0**-11
    # whole, portions (tiles), single rows on the matrix cores (auto) and off them (grouped)
    for sizes, kernel in (([n], "tiles"), ([5, 33, 2, 40, 31, 32, 64], "tiles"), ([1], "auto"), ([1], "grouped"),
                          ([7, 1, 1], "auto")):
        pk = PagedKeys(G, D, bs, n, dtype=dtype, seed=len(sizes))
        got, lo, i = [], 0, 0
        while lo < n:
            step = min(sizes[i % len(sizes)], n - lo)
            got.append(pk.attend(q, k, gate, lo, lo + step, H, window, scale, slopes, coef, every, 0.6, kernel))
            lo += step
            i += 1
        close(torch.cat(got).float(), want, 1.5 * ulp)


def test_window_attention_tiles_batch_matches_rows():
    """Several sequences with contexts in one tiled launch against the row kernel on the same
    cache: the two kernels differ by rounding only."""
    H, G, D, bs, window = 8, 2, 64, 16, 37
    lens, ctx = [70, 33, 5, 1], [10, 0, 64, 90]
    g = torch.Generator().manual_seed(11)
    total = [c + n for c, n in zip(ctx, lens)]
    nb = sum((t + bs - 1) // bs for t in total)
    perm = torch.randperm(nb, generator=g).tolist()
    tables, at = [], 0
    for t in total:
        cnt = (t + bs - 1) // bs
        tables.append(perm[at:at + cnt])
        at += cnt
    cache = torch.randn(nb, bs, G, D, generator=g).bfloat16().to(DEV)
    T = sum(lens)
    q = torch.randn(T, H * D, generator=g).bfloat16().to(DEV)
    bt = torch.zeros(4, max(len(t) for t in tables), dtype=torch.int32)
    for b, t in enumerate(tables):
        bt[b, :len(t)] = torch.tensor(t, dtype=torch.int32)
    starts = [0]
    for n in lens:
        starts.append(starts[-1] + n)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)      # noqa: E731
    pos = torch.cat([torch.arange(c, c + n) for c, n in zip(ctx, lens)]).to(DEV)
    tseq = torch.cat([torch.full((n, ), b, dtype=torch.int32) for b, n in enumerate(lens)]).to(DEV)
    slopes = torch.tensor(R.head_slopes(H), dtype=torch.float32, device=DEV)
    a, b_ = torch.empty_like(q), torch.empty_like(q)
    ops().window_attention_tiles(a, q, None, cache, bt.to(DEV), i32(starts), i32(ctx), max(lens), slopes, H, window,
                                 D**-0.5, 0.3, 16.0)
    ops().window_attention(b_, q, None, cache, bt.to(DEV), tseq, pos, slopes, H, window, D**-0.5, 0.3, 16.0)
    close(a.float(), b_.cpu().float(), 2.0**-7)
    c_ = torch.empty_like(q)
    ops().set_window_kernel(2)
    try:
        ops().window_attention(c_, q, None, cache, bt.to(DEV), tseq, pos, slopes, H, window, D**-0.5, 0.3, 16.0)
    finally:
        ops().set_window_kernel(0)
    close(b_.float(), c_.cpu().float(), 2.0**-7)


def test_window_attention_without_bias_temperature_or_gate_in_bf16():
    H, G, D, n = 4, 2, 32, 50
    g = torch.Generator().manual_seed(5)
    q, k = torch.randn(n, H * D, generator=g).bfloat16(), torch.randn(n, G * D, generator=g).bfloat16()
    pk = PagedKeys(G, D, 16, n, dtype=torch.bfloat16)
    got = pk.attend(q, k, None, 0, n, H, 9, 0.2, None)
    want = R.windowed_key_attention(q.to(R.F), k.to(R.F), torch.arange(n), H, G, D, 9, 0.2, 0.0, 1.0, [0.0] * H)
    close(got.float(), want, 2.0**-8)


@pytest.mark.parametrize("window,bs", [(5, 4), (16, 16), (17, 16), (32, 16), (33, 8), (64, 16), (65, 8), (100, 32)])
@pytest.mark.parametrize("decode", [False, True, "tiles", "heads"])
def test_window_edge_decides_the_result(window, bs, decode):
    """Query i and key j share a long vector.  j = i - window + 1 is the last key inside: the
    result is that key.  j = i - window is the first outside: the result is far from it.  i is
    placed so that j falls on the first slot of a page, the last slot of a page, and position 0."""
    H, G, D = 2, 1, 32
    dt = torch.bfloat16 if decode in ("tiles", "heads") else torch.float32
    n = 3 * window + 2 * bs + 3
    scale = D**-0.5
    for inside in (True, False):
        dist = window - 1 if inside else window
        for j in sorted({0, bs, 2 * bs - 1, n - 1 - dist}):
            i = j + dist
            if i >= n:
                continue
            g = torch.Generator().manual_seed(i * 7 + j)
            q, k = torch.randn(n, H * D, generator=g) * 0.1, torch.randn(n, G * D, generator=g) * 0.1
            u = torch.nn.functional.normalize(torch.randn(D, generator=g), dim=0)
            big = math.sqrt((60.0 + window) / scale)        # score big^2 * scale outweighs any bias
            k[j] = u * big
            q[i] = (u * big).repeat(H)
            q, k = q.to(dt), k.to(dt)
            pk = PagedKeys(G, D, bs, n, dtype=dt, seed=j)
            if decode == "tiles":
                cut = max(1, i - 3)         # the portion's first tile starts three rows before i
                pk.attend(q, k, None, 0, cut, H, window, scale, R.head_slopes(H), kernel="tiles")
                out = pk.attend(q, k, None, cut, n, H, window, scale, R.head_slopes(H), kernel="tiles")[i - cut].float()
                k = k.float()
            elif decode == "heads":         # 16-bit single rows: the matrix-core row kernel
                pk.attend(q, k, None, 0, i, H, window, scale, R.head_slopes(H), kernel="tiles")
                out = pk.attend(q, k, None, i, i + 1, H, window, scale, R.head_slopes(H))[0].float()
                k = k.float()
            elif decode:
                pk.attend(q, k, None, 0, i, H, window, scale, R.head_slopes(H))
                out = pk.attend(q, k, None, i, i + 1, H, window, scale, R.head_slopes(H))[0]
            else:
                out = pk.attend(q, k, None, 0, n, H, window, scale, R.head_slopes(H))[i]
            for h in range(H):
                d = float((out[h * D:(h + 1) * D] - k[j]).norm() / k[j].norm())
                assert (d < (1e-2 if decode in ("tiles", "heads") else 1e-3)) if inside else (d > 0.5), (inside, i, j, h, d)


def test_query_temperature_steps_at_multiples_of_its_period():
    """With one key per query visible besides itself the softmax weight exposes the temperature:
    positions every-2 and every-1 differ (floor((p + 1) / every) goes 0 -> 1)."""
    H, G, D, every, coef = 1, 1, 8, 6, 0.8
    n = 2 * every + 2
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(n, D, generator=g), torch.randn(n, D, generator=g)
    pk = PagedKeys(G, D, 4, n)
    got = pk.attend(q, k, None, 0, n, H, 2, 0.5, None, coef, every)
    want = R.windowed_key_attention(q.to(R.F), k.to(R.F), torch.arange(n), H, G, D, 2, 0.5, coef, every, [0.0])
    close(got, want, 3e-5)
    plain = R.windowed_key_attention(q.to(R.F), k.to(R.F), torch.arange(n), H, G, D, 2, 0.5, 0.0, every, [0.0])
    assert torch.allclose(want[:every - 1], plain[:every - 1]) and not torch.allclose(want[every - 1], plain[every - 1])


def test_window_attention_batch_of_unequal_sequences():
    """Three sequences in one launch (a decode token, a portion that continues a context, a whole
    prompt) against each alone."""
    H, G, D, bs, window = 4, 2, 40, 8, 11
    lens, ctx = [30, 45, 19], [29, 20, 0]
    g = torch.Generator().manual_seed(3)
    seqs = [(torch.randn(n, H * D, generator=g), torch.randn(n, G * D, generator=g)) for n in lens]
    nb = sum((n + bs - 1) // bs for n in lens) + 2
    perm = torch.randperm(nb, generator=g).tolist()
    tables, at = [], 0
    for n in lens:
        c = (n + bs - 1) // bs
        tables.append(perm[at:at + c])
        at += c
    cache = (torch.randn(nb, bs, G, D, generator=g) * 30).to(DEV)
    slopes = torch.tensor(R.head_slopes(H), dtype=torch.float32, device=DEV)

    def slots(b, lo, hi):
        p = torch.arange(lo, hi)
        return (torch.tensor(tables[b])[p // bs] * bs + p % bs).long()

    for b, c in enumerate(ctx):          # contexts first, one sequence at a time
        if c:
            ops().key_cache_write(cache, seqs[b][1][:c].to(DEV), slots(b, 0, c).to(DEV))
    qs = torch.cat([seqs[b][0][ctx[b]:] for b in range(3)]).to(DEV)
    ks = torch.cat([seqs[b][1][ctx[b]:] for b in range(3)]).to(DEV)
    sl = torch.cat([slots(b, ctx[b], lens[b]) for b in range(3)]).to(DEV)
    pos = torch.cat([torch.arange(ctx[b], lens[b]) for b in range(3)]).to(DEV)
    tseq = torch.cat([torch.full((lens[b] - ctx[b], ), b, dtype=torch.int32) for b in range(3)]).to(DEV)
    bt = torch.zeros(3, max(len(t) for t in tables), dtype=torch.int32)
    for b, t in enumerate(tables):
        bt[b, :len(t)] = torch.tensor(t, dtype=torch.int32)
    ops().key_cache_write(cache, ks, sl)
    out = torch.empty_like(qs)
    ops().window_attention(out, qs, None, cache, bt.to(DEV), tseq, pos, slopes, H, window, D**-0.5)
    at = 0
    for b in range(3):
        q, k = seqs[b]
        want = R.windowed_key_attention(q.to(R.F), k.to(R.F), torch.arange(lens[b]), H, G, D, window, D**-0.5, 0.0,
                                        1.0, R.head_slopes(H))[ctx[b]:]
        close(out[at:at + lens[b] - ctx[b]], want, 3e-5)
        at += lens[b] - ctx[b]


# ------------------------------------------------------------------------------ linear recurrence


@pytest.mark.parametrize("n", [7, 45, 512, 530])       # few tokens: one thread per (token, channel); many: rows of W2 in registers
@pytest.mark.parametrize("C,rank,dtype", [(8, 1, torch.float32), (96, 4, torch.float32), (300, 16, torch.float32),
                                          (64, 8, torch.bfloat16), (40, 32, torch.float32), (70, 33, torch.float32)])
def test_gla_log_decay(C, rank, dtype, n):
    g = torch.Generator().manual_seed(C)
    y = (torch.randn(n, rank + 2, generator=g) * 3).to(dtype).to(DEV)[:, 1:1 + rank]
    w2 = torch.randn(C, rank, generator=g).to(dtype)
    bias = torch.randn(C, generator=g) * 4          # both tails of the sigmoid
    out = torch.empty(n, C, dtype=torch.float32, device=DEV)
    ops().gla_log_decay(out, y, w2.to(DEV), bias.to(DEV), 1 / 5.0)
    close(out, R.log_decay(y.cpu().to(R.F), w2.to(R.F), bias.to(R.F), 5.0), 1e-5)
    assert bool((out <= 0).all())


SCAN_KERNEL = {"mode": 0}      # 0: picked per shape (the blocked walk where it fits); 1: token by token


@pytest.fixture(params=[0, 1], ids=["blocked", "token-by-token"])
def scan_kernel(request):
    SCAN_KERNEL["mode"] = request.param
    yield request.param
    SCAN_KERNEL["mode"] = 0


def run_scan(q, k, v, ln_a, state, starts, ctx, slots, H, D, V, q_scale):
    T = q.shape[0]
    o = torch.empty(T, H, V, dtype=torch.float32, device=DEV)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)      # noqa: E731
    ops().set_scan_kernel(SCAN_KERNEL["mode"])
    try:
        ops().gla_scan(o, q.to(DEV), k.to(DEV), v.to(DEV), ln_a.to(DEV), state, i32(starts), i32(ctx), i32(slots),
                       q_scale)
    finally:
        ops().set_scan_kernel(0)
    return o.cpu()


SCAN = [(2, 8, 16), (3, 32, 64), (1, 5, 7), (2, 64, 128), (2, 100, 40), (1, 16, 300), (2, 1, 1), (1, 130, 64)]


@pytest.mark.parametrize("H,D,V", SCAN)
def test_gla_scan_whole_portions_and_single_tokens(H, D, V, scan_kernel):
    n = 57
    g = torch.Generator().manual_seed(H * D + V)
    q, k, v = torch.randn(n, H * D, generator=g), torch.randn(n, H * D, generator=g), torch.randn(n, H * V, generator=g)
    ln_a = -torch.rand(n, H * D, generator=g) * 0.3
    want, want_state = R.gated_linear_attention(q.to(R.F) * 0.37, k.to(R.F), v.to(R.F), ln_a.to(R.F), H, D, V)
    for sizes in ([n], [2, 5, 1, 1, 19, 3, 16, 17], [1] * n):
        state = torch.full((3, H, D, V), 7.0, device=DEV)     # stale: the sequence starts at context 0
        got, lo, i = [], 0, 0
        while lo < n:
            step = min(sizes[i % len(sizes)], n - lo)
            got.append(run_scan(q[lo:lo + step], k[lo:lo + step], v[lo:lo + step], ln_a[lo:lo + step], state,
                                [0, step], [lo], [1], H, D, V, 0.37))
            lo += step
            i += 1
        close(torch.cat(got), want, 2e-5)
        close(state[1], want_state, 2e-5)
        assert float((state[0] - 7).abs().max()) == 0 and float((state[2] - 7).abs().max()) == 0


def test_gla_scan_batch_with_slots_used_again(scan_kernel):
    """Four sequences of unequal length in one launch, two of them continuing; then the slot of a
    finished one goes to a new sequence, which must not see what the slot held."""
    H, D, V = 2, 12, 20
    g = torch.Generator().manual_seed(9)
    lens = [9, 1, 34, 5]

    def mk(n):
        return (torch.randn(n, H * D, generator=g), torch.randn(n, H * D, generator=g),
                torch.randn(n, H * V, generator=g), -torch.rand(n, H * D, generator=g) * 0.2)
    seqs = [mk(n + 6) for n in lens]
    state = torch.randn(4, H, D, V, generator=g).to(DEV)
    slots = [2, 0, 3, 1]
    ctx = [6, 0, 6, 0]
    for b in (0, 2):                      # contexts of the continuing ones
        q, k, v, a = (t[:6] for t in seqs[b])
        run_scan(q, k, v, a, state, [0, 6], [0], [slots[b]], H, D, V, 1.0)
    parts = [[t[ctx[b]:ctx[b] + lens[b]] for t in seqs[b]] for b in range(4)]
    starts = [0]
    for n in lens:
        starts.append(starts[-1] + n)
    o = run_scan(*(torch.cat([p[i] for p in parts]) for i in range(4)), state, starts, ctx, slots, H, D, V, 1.0)
    for b in range(4):
        q, k, v, a = (t[:ctx[b] + lens[b]].to(R.F) for t in seqs[b])
        want, st = R.gated_linear_attention(q, k, v, a, H, D, V)
        close(o[starts[b]:starts[b + 1]], want[ctx[b]:], 2e-5)
        close(state[slots[b]], st, 2e-5)
    q, k, v, a = mk(4)                    # a new sequence takes slot 3 over
    o = run_scan(q, k, v, a, state, [0, 4], [0], [3], H, D, V, 1.0)
    close(o, R.gated_linear_attention(q.to(R.F), k.to(R.F), v.to(R.F), a.to(R.F), H, D, V)[0], 2e-5)


@pytest.mark.parametrize("decode", [False, True])
def test_gla_carries_a_far_token(decode, scan_kernel):
    """One channel never decays and holds a key at token 3 only; 600 tokens later a query on
    that channel returns token 3's value, through one launch or through 600."""
    H, D, V, n = 1, 8, 16, 604
    g = torch.Generator().manual_seed(2)
    q, k, v = torch.zeros(n, D), torch.randn(n, D, generator=g) * 0.1, torch.randn(n, V, generator=g)
    ln_a = torch.full((n, D), -0.05)
    ln_a[:, 5] = 0.0
    k[:, 5] = 0.0
    k[3, 5] = 2.0
    q[n - 1, 5] = 1.0
    state = torch.zeros(1, H, D, V, device=DEV)
    if decode:
        for t in range(n):
            o = run_scan(q[t:t + 1], k[t:t + 1], v[t:t + 1], ln_a[t:t + 1], state, [0, 1], [t], [0], H, D, V, 1.0)
        last = o[0, 0]
    else:
        last = run_scan(q, k, v, ln_a, state, [0, n], [0], [0], H, D, V, 1.0)[n - 1, 0]
    close(last, 2.0 * v[3], 1e-5)


@pytest.mark.parametrize("piece_rows", [8, 32])
def test_recurrent_layer_cuts_long_runs_into_pieces(piece_rows, monkeypatch):
    """The layer as the model calls it: runs of at least two pieces are walked piece-parallel
    (zero-state walks, a matrix product for the missing start state, a chain over the pieces'
    states), next to a short run and a single row, with one cut sequence continuing a context.
    Everything must equal the one long walk."""
    from vllm_legacy_amd.attention.batch import SequenceBatch
    from vllm_legacy_amd.attention.recurrent import GatedLinearRecurrence
    monkeypatch.setattr(GatedLinearRecurrence, "PIECE_ROWS", piece_rows)
    H, D, V, rank, tau, eps = 2, 12, 20, 3, 5.0, 1e-5
    layer = GatedLinearRecurrence(H, D, V, tau, eps)
    g = torch.Generator().manual_seed(piece_rows)
    lens, ctx = [5 * piece_rows + 3, 3, 2 * piece_rows, 1], [0, 4, 7, 9]
    slots = [2, 0, 3, 1]
    state = torch.randn(GatedLinearRecurrence.get_state_shape(4, H, D, V), generator=g).to(DEV)
    w2, bias = torch.randn(H * D, rank, generator=g) * 0.5, torch.randn(H * D, generator=g) + 2
    norm_w = torch.randn(V, generator=g)

    def mk(n):
        return [torch.randn(n, w, generator=g) for w in (H * D, H * D, H * V, H * V, rank)]     # q k v gate y
    seqs = [mk(c + n) for c, n in zip(ctx, lens)]

    def run(batch_lens, batch_ctx, batch_slots, parts):
        b = SequenceBatch.build(batch_lens, batch_ctx, [[0] * 64] * len(batch_lens), batch_slots, 16, DEV)
        q, k, v, gate, y = (torch.cat([p[i] for p in parts]).to(DEV) for i in range(5))
        out = torch.empty(q.shape[0], H * V, device=DEV)
        layer(out, q, k, v, gate, y, w2.to(DEV), bias.to(DEV), norm_w.to(DEV), state, b, 0.8)
        return out.cpu()

    for b_, c in enumerate(ctx):              # contexts, one sequence at a time
        if c:
            run([c], [0], [slots[b_]], [[t[:c] for t in seqs[b_]]])
    got = run(lens, ctx, slots, [[t[c:] for t in s] for s, c in zip(seqs, ctx)])
    at = 0
    for b_, (c, n) in enumerate(zip(ctx, lens)):
        q, k, v, gate, y = (t.to(R.F) for t in seqs[b_])
        ln_a = R.log_decay(y, w2.to(R.F), bias.to(R.F), tau)
        o, st = R.gated_linear_attention(q * D**-0.5, k, v, ln_a, H, D, V)
        want = R.gated_head_norm(o, norm_w.to(R.F), gate, eps, 0.8)[c:]
        close(got[at:at + n], want, 3e-5)
        close(state[slots[b_]], st, 3e-5)
        at += n


@pytest.mark.parametrize("features,offset", [(40, 0), (256, 4), (1100, 8), (4100, 0), (5632, 4), (300, 3), (302, 0)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_poly_norm_16bit_rows_aligned_or_not(features, offset, dtype):
    """Rows inside a wider matrix: offsets that are multiples of four values take the four-wide
    kernel (rows longer than the 4096 values a workgroup keeps in registers included), others
    and lengths that are not multiples of four the element-wise one."""
    g = torch.Generator().manual_seed(features + offset)
    width = (features + offset + 7) // 4 * 4
    wide = (torch.randn(3, width, generator=g) * 1.5).to(dtype).to(DEV)
    z = wide[:, offset:offset + features]
    coef = torch.tensor([0.6, 0.3, -0.2, 0.05])
    dst = torch.zeros(3, width, dtype=dtype, device=DEV)
    ops().poly_norm(dst[:, offset:offset + features], z, coef.to(DEV), 1e-5)
    want = R.poly_norm(z.cpu().to(R.F), coef, 1e-5)
    ulp = 2.0**-8 if dtype == torch.bfloat16 else 2.0**-11
    close(dst[:, offset:offset + features].float(), want, 1.1 * ulp)
    assert float(dst[:, :offset].float().abs().max() if offset else 0.0) == 0.0
    assert float(dst[:, offset + features:].float().abs().max()) == 0.0
