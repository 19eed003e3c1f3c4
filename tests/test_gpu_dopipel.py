"""Dopipel through the framework -- registry, checkpoint loader, cache manager, model runner,
scheduler, sampler -- and its mechanisms one by one, against the float64 reference of
tests/dopipel_oracle.py on small random models and inputs.

Mechanisms alone: the residual update with both norms; the input convolution and its state across
cuts; rotary attention over paged key / value caches (rotated values, head gate, partial rotation,
both pair layouts, a window, a far key that carries the whole output, page borders); the minGRU walk,
short and in pieces; activations; the router (correction, ties aside), the grouped expert
products and the combine with identity and shared experts.
Whole models: prompts whole, in portions down to two tokens and token by token; mixed batches with
pages and slots used again; long decoding; long prompts; a batch does not change a request; greedy
generation through LLMEngine; the trace replayer as a program.  The float32 bar is float32
rounding through the stack (1e-4 of the logits' spread) and is the one that finds faults of
cutting, batching and reuse: both number formats run the same code paths except the matrix-core
kernels, which the bfloat16 runs cover with a looser bar (widths of 64 average little rounding
noise out: nine rows in ten within 0.2 of the logits' spread, 0.05 on average)."""
import json
import os
import subprocess
import sys

import pytest
import torch

from tests import dopipel_oracle as R

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F = R.F
BAR = {torch.float32: 1e-4, torch.bfloat16: 0.2}
MEAN_BAR = {torch.float32: 1e-4, torch.bfloat16: 0.05}


def configs():
    A, M, D, E = R.attention_layer, R.mingru_layer, R.dense_mlp, R.moe_mlp
    return {
        "plain": R.make_config([M(48, D(96)), A(4, 2, 16, mlp=E()), A(4, 2, 16, mlp=D(80)), M(40, E(5, 2, 2, 24, 0))],
                               loop=(1, 3, 2)),
        # sizes that are neither equal nor powers of two; one KV head, vdim != dim, part of a head
        # rotated, a feed-forward missing, one expert chosen, no identity or shared expert, a loop
        # that runs once and starts late
        "odd": R.make_config([A(3, 1, 24, vdim=12, rot_dims=8, base=300.0, scale=0.3, mlp=None),
                              M(50, E(3, 0, 1, 20, 0)), A(6, 3, 8, vdim=20, mlp=D(52))],
                             vocab=131, width=40, taps=2, loop=(2, 3, 1)),
        # kv heads = heads, every routed expert chosen, one tap, a single real expert, three passes
        "equal": R.make_config([A(2, 2, 16, mlp=E(1, 2, 3, 16, 8)), M(64, D(64))], taps=1, loop=(0, 2, 3)),
        # more taps than some requests have tokens, no loop
        "taps": R.make_config([M(32, D(48)), A(2, 1, 32, mlp=E(4, 1, 2, 16, 16))], width=48, taps=6),
        # head sizes for the matrix-core kernels: multiples of 32, groups larger than a chunk
        "mfma": R.make_config([A(10, 2, 32, vdim=64, mlp=D(64)), A(2, 1, 96, vdim=64, mlp=E(6, 1, 2, 32, 32)),
                               A(4, 4, 64, vdim=32, rot_dims=32, mlp=None)], width=128, loop=(0, 2, 2)),
    }


class Served:
    """A checkpoint on disk, loaded through the registry, with the engine's cache manager and
    model runner around it."""

    def __init__(self, tmp_path, name, dtype, num_blocks=64, block_size=4, num_slots=3, seed=0):
        from vllm_legacy_amd.engine.cache_manager import CacheManager
        from vllm_legacy_amd.engine.model_runner import ModelRunner
        from vllm_legacy_amd.model.registry import load_model
        self.cfg = configs()[name]
        self.W = R.make_weights(self.cfg, seed=seed)
        self.folder = R.write_checkpoint(str(tmp_path / name), self.cfg, self.W)
        self.dtype = dtype
        self.model = load_model(self.folder, dtype, DEV)
        self.cache = CacheManager(num_blocks, block_size, num_slots)
        self.runner = ModelRunner(self.model, self.cache, DEV)
        self.done = {}

    def step(self, entries):
        """entries: [(id, tokens)]; logits of every token come back per id."""
        batch, want = [], []
        for sid, tokens in entries:
            if not self.cache.is_live(sid):
                self.cache.admit(sid)
                self.done[sid] = 0
            self.cache.grow(sid, self.done[sid] + len(tokens))
            batch.append((sid, list(tokens), self.done[sid]))
            want.append(list(range(len(tokens))))
        logits = self.runner.execute(batch, want).cpu()
        out, at = {}, 0
        for sid, tokens in entries:
            out[sid] = logits[at:at + len(tokens)]
            at += len(tokens)
            self.done[sid] += len(tokens)
        return out

    def end(self, sid):
        self.cache.free(sid)
        del self.done[sid]

    def reference(self, tokens):
        return R.forward(tokens, self.cfg, self.W)

    def check(self, got, tokens, what=""):
        within(logit_error(got, self.reference(tokens)), self.dtype, what)


def logit_error(got, want):
    return R.row_errors(got, want) / R.spread(want.to(F))


def within(err, dtype, what=""):
    # in bfloat16 a router's close call can go the other way than in the float64 reference and move
    # that token's logits: one row in ten may be out; float32 rows must all be in
    worst = float(err.max()) if dtype == torch.float32 else float(torch.quantile(err, 0.9))
    assert worst <= BAR[dtype] and float(err.mean()) <= MEAN_BAR[dtype], (what, float(err.max()), float(err.mean()))


def tokens_of(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n, ), generator=g).tolist()


def rnd(shape, seed, std=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * std


# ------------------------------------------------------------------------------------------------
# mechanisms alone

def make_batch(query_lens, context_lens, block_size, tables=None, slots=None):
    from vllm_legacy_amd.attention.batch import SequenceBatch
    B = len(query_lens)
    if tables is None:
        tables, at = [], 0
        for q, c in zip(query_lens, context_lens):
            n = (q + c + block_size - 1) // block_size
            tables.append(list(range(at, at + n)))
            at += n
    return SequenceBatch.build(query_lens, context_lens, tables, slots or list(range(B)), block_size, DEV)


@pytest.mark.parametrize("width", [40, 256, 2500])
def test_residual_update_with_both_norms(width):
    from vllm_legacy_amd import _seq_ops as ops
    T, eps = 5, 1e-5
    x, y = rnd((T, width), 0), rnd((T, width), 1, 3.0)
    bias, post, ls, row, pre = (rnd((width, ), s) for s in range(2, 7))
    for ydt in (torch.float32, torch.bfloat16):
        yy = y.to(ydt)
        want_x = x.to(F) + R.rms_norm(yy.to(F) + bias, post.to(F), eps) * ls + row
        want_h = R.rms_norm(want_x, pre.to(F), eps)
        gx = x.to(DEV).clone()
        out = torch.empty((T, width), dtype=torch.float32, device=DEV)
        ops.residual_norms(gx, yy.to(DEV), bias.to(DEV), post.to(DEV), ls.to(DEV), row.to(DEV), out, pre.to(DEV), eps)
        assert float((gx.cpu() - want_x).abs().max()) <= 1e-5 and float((out.cpu() - want_h).abs().max()) <= 1e-5
    # the parts alone: only a norm; only the update
    gx = x.to(DEV).clone()
    out = torch.empty((T, width), dtype=torch.bfloat16, device=DEV)
    ops.residual_norms(gx, out=out, pre_weight=pre.to(DEV), eps=eps)
    assert torch.equal(gx.cpu(), x)
    assert float((out.float().cpu() - R.rms_norm(x.to(F), pre.to(F), eps)).abs().max()) <= 0.05
    ops.residual_norms(gx, y.to(DEV), None, post.to(DEV), None, None, None, None, eps)
    assert float((gx.cpu() - (x.to(F) + R.rms_norm(y.to(F), post.to(F), eps))).abs().max()) <= 1e-5


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_input_convolution_across_cuts_and_slots(taps):
    """Two sequences cut into steps of unequal sizes (shorter than the taps too), slots swapped
    against the batch order, a slot used again by a new sequence."""
    from vllm_legacy_amd.layers import CausalConvMix
    W = 70
    conv = CausalConvMix(W, taps, DEV)
    w = rnd((W, taps), 0, 0.5)
    conv.weight.data = w.to(DEV)
    state = torch.full(CausalConvMix.get_state_shape(3, W, taps), 7.0, device=DEV)     # stale values
    ha, hb, hc = rnd((23, W), 1), rnd((9, W), 2), rnd((4, W), 3)
    want = {k: R.input_convolution(h.to(F), w.to(F)) for k, h in (("a", ha), ("b", hb), ("c", hc))}
    got = {"a": [], "b": [], "c": []}
    at = {"a": 0, "b": 0, "c": 0}
    src = {"a": ha, "b": hb, "c": hc}
    slot = {"a": 2, "b": 0, "c": 0}          # c starts in b's slot after b has ended
    for step in ([("a", 1), ("b", 2)], [("b", 1), ("a", 2)], [("a", 9), ("b", 6)], [("c", 1), ("a", 1)],
                 [("a", 10), ("c", 3)]):
        batch = make_batch([n for _, n in step], [at[k] for k, _ in step], 4, slots=[slot[k] for k, _ in step])
        h = torch.cat([src[k][at[k]:at[k] + n] for k, n in step]).to(DEV)
        out = conv(h, state, batch, torch.float32).cpu()
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n])
            o += n
            at[k] += n
    for k in got:
        assert float((torch.cat(got[k]) - want[k]).abs().max()) <= 1e-5, k


def attention_spec(H, G, D, V, rot_dims, base=10000.0, layout="interleaved", scale=None):
    return {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": D**-0.5 if scale is None else scale,
            "rot": {"dims": rot_dims, "base": base, "layout": layout}}


def run_attention(spec, q, k, v, gate, cuts, dtype, block_size=4, window=0, shuffle_pages=True):
    """One sequence through RotaryKVAttention in steps of the given sizes; pages in a scrambled
    order.  Returns [n, H, V] fp32 on the CPU."""
    from vllm_legacy_amd.attention.backends.rotary_kv import RotaryKVAttention
    H, G, D, V = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    n = q.shape[0]
    layer = RotaryKVAttention(H, G, D, V, spec["scale"], spec["rot"]["dims"], spec["rot"]["base"],
                              spec["rot"]["layout"] == "interleaved", True, window, DEV)
    pages = (n + block_size - 1) // block_size
    order = torch.randperm(pages + 3, generator=torch.Generator().manual_seed(1)).tolist() if shuffle_pages \
        else list(range(pages + 3))
    ks, vs = RotaryKVAttention.get_cache_shapes(pages + 3, block_size, G, D, V)
    kc = torch.full(ks, float("nan"), dtype=dtype, device=DEV)      # a read of an unwritten place shows
    vc = torch.full(vs, float("nan"), dtype=dtype, device=DEV)
    outs, at = [], 0
    for c in cuts:
        c = min(c, n - at)
        if c <= 0:
            break
        batch = make_batch([c], [at], block_size, tables=[order[:pages]])
        qq = q[at:at + c].reshape(c, H * D).to(dtype).to(DEV).clone()
        kk = k[at:at + c].reshape(c, G * D).to(dtype).to(DEV)
        vv = v[at:at + c].reshape(c, G * V).to(dtype).to(DEV)
        gg = None if gate is None else gate[at:at + c].to(dtype).to(DEV)
        out = torch.empty((c, H * V), dtype=dtype, device=DEV)
        layer(out, qq, kk, vv, gg, kc, vc, batch)
        outs.append(out.float().cpu().view(c, H, V))
        at += c
    assert at == n
    return torch.cat(outs)


ATTN_SHAPES = [
    # H, G, D, V, rot_dims, layout
    (4, 2, 16, 16, 16, "interleaved"),
    (3, 1, 24, 12, 8, "interleaved"),
    (6, 3, 8, 20, 8, "halves"),
    (2, 2, 40, 6, 0, "interleaved"),
    (10, 2, 32, 64, 32, "interleaved"),
    (2, 1, 96, 64, 64, "interleaved"),
    (8, 1, 64, 32, 32, "halves"),
    (5, 5, 128, 128, 64, "interleaved"),
    (2, 1, 32, 96, 32, "halves"),
]


@pytest.mark.parametrize("shape", ATTN_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotary_attention_prompt_portions_and_decoding(shape, dtype):
    H, G, D, V, rot, layout = shape
    spec = attention_spec(H, G, D, V, rot, 500.0, layout)
    n = 75
    q, k, v, gate = rnd((n, H, D), 0), rnd((n, G, D), 1), rnd((n, G, V), 2), rnd((n, H), 3, 2.0)
    if dtype == torch.bfloat16:
        q, k, v, gate = (t.to(dtype).float() for t in (q, k, v, gate))
    want = R.attention_core(q.to(F), k.to(F), v.to(F), gate.to(F), spec)
    bar = 2e-5 if dtype == torch.float32 else 0.06
    for cuts in ([n], [2, 3, 4, 5, 1, 7, 2] * 5, [40] + [1] * 35, [33, 35, 7], [1] * n):
        got = run_attention(spec, q, k, v, gate, cuts, dtype)
        assert float((got - want).abs().max()) <= bar * float(want.abs().max()), (cuts[:3], float((got - want).abs().max()))


def test_plain_and_matrix_core_kernels_agree():
    """bfloat16 through the kernel every dtype can take and through the matrix-core kernels."""
    from vllm_legacy_amd import _seq_ops as ops
    H, G, D, V = 8, 2, 96, 64
    spec = attention_spec(H, G, D, V, 64, 1000.0)
    n = 101
    q, k, v, gate = (t.to(torch.bfloat16).float() for t in (rnd((n, H, D), 0), rnd((n, G, D), 1), rnd((n, G, V), 2), rnd((n, H), 3)))
    fast = run_attention(spec, q, k, v, gate, [60, 3] + [1] * 38, torch.bfloat16)
    ops.set_kv_attention_kernel(1)
    try:
        plain = run_attention(spec, q, k, v, gate, [60, 3] + [1] * 38, torch.bfloat16)
    finally:
        ops.set_kv_attention_kernel(0)
    assert float((fast - plain).abs().max()) <= 0.03 * float(plain.abs().max())
    assert not torch.equal(fast, plain)          # two kernels did run


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dim", [16, 64])
def test_a_far_key_carries_the_output(dtype, dim):
    """Queries near the end all look for one key hundreds of tokens back: its value must make up the
    output, in a prompt, in portions and in decoding.  The key is built so that, once both are
    rotated, it lines up with the queries."""
    H, G, D, V, n, far = 2, 1, dim, dim, 330, 5
    spec = attention_spec(H, G, D, V, D, 10000.0)
    q, k, v = rnd((n, H, D), 0, 0.3), rnd((n, G, D), 1, 0.3), rnd((n, G, V), 2)
    ang = R.pair_angles(torch.arange(n), D // 2, 10000.0, D)
    target = rnd((1, 1, D), 3).to(F)
    target = 6.0 * target / target.norm() * D**0.25
    # rotated key at `far` = target; rotated queries of the last tokens = target
    k[far] = R.rotate_pairs(target, -ang[far:far + 1])[0].float()
    for i in range(n - 40, n):
        q[i] = R.rotate_pairs(target.expand(1, H, D), -ang[i:i + 1])[0].float()
    v[far] = 0.0
    v[far, 0, 0] = 50.0
    if dtype == torch.bfloat16:
        q, k, v = (t.to(dtype).float() for t in (q, k, v))
    want = R.attention_core(q.to(F), k.to(F), v.to(F), None, spec)
    # the far key matters: without it the outputs are elsewhere
    v2 = v.clone()
    v2[far] = 0.0
    assert float((R.attention_core(q.to(F), k.to(F), v2.to(F), None, spec)[-40:] - want[-40:]).norm(dim=-1).min()) > 5.0
    bar = 2e-5 if dtype == torch.float32 else 0.06
    for cuts in ([n], [n - 40] + [1] * 40, [100, 3, 190, 2, 35]):
        got = run_attention(spec, q, k, v, None, cuts, dtype, block_size=16)
        assert float((got - want).abs().max()) <= bar * float(want.abs().max()), cuts[:2]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 5, 16, 37])
def test_window_edges(dtype, window):
    """With a window, the key just inside it counts and the one just outside does not: every key
    gets its own large value, so a window that is one token off moves the output."""
    H, G, D, V, n = 4, 2, 32, 32, 90
    spec = attention_spec(H, G, D, V, D, 100.0)
    q, k, v = rnd((n, H, D), 0), rnd((n, G, D), 1), rnd((n, G, V), 2)
    v += (torch.arange(n).float() % 7)[:, None, None] * 3.0
    if dtype == torch.bfloat16:
        q, k, v = (t.to(dtype).float() for t in (q, k, v))
    want = R.attention_core(q.to(F), k.to(F), v.to(F), None, spec, window)
    off = R.attention_core(q.to(F), k.to(F), v.to(F), None, spec, window + 1)
    assert float((want - off).abs().max()) > 0.3
    bar = 2e-5 if dtype == torch.float32 else 0.06
    for cuts in ([n], [50] + [1] * 40, [7, 2, 31, 1, 49]):
        got = run_attention(spec, q, k, v, None, cuts, dtype, window=window)
        assert float((got - want).abs().max()) <= bar * float(want.abs().max()), cuts[:2]


@pytest.mark.parametrize("channels", [50, 256, 700])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mingru_walk_short_long_and_cut(channels, dtype):
    """Runs below and above the length from which the walk goes in pieces, cut in several ways, two
    sequences in a batch with swapped slots; stale slots."""
    from vllm_legacy_amd.attention.recurrent import MinGRURecurrence
    layer = MinGRURecurrence(channels)
    na, nb = 600, 281
    pre = {k: [rnd((n, channels), s + i, 2.0).to(dtype) for i in range(3)] for k, n, s in (("a", na, 0), ("b", nb, 10))}
    want = {k: R.mingru_core(*(t.to(F) for t in pre[k])) for k in pre}
    plans = [
        [[("a", na)], [("b", nb)]],
        [[("a", 300), ("b", 1)], [("b", 280), ("a", 255)], [("a", 45)]],
        [[("b", 2), ("a", 511)], [("a", 1), ("b", 3)], [("a", 88), ("b", 276)]],
    ]
    bar = 1e-5 if dtype == torch.float32 else 0.03
    for plan in plans:
        state = torch.full(MinGRURecurrence.get_state_shape(3, channels), 9.0, device=DEV)
        slot, at, got = {"a": 2, "b": 1}, {"a": 0, "b": 0}, {"a": [], "b": []}
        for step in plan:
            batch = make_batch([n for _, n in step], [at[k] for k, _ in step], 16, slots=[slot[k] for k, _ in step])
            zp, up, gp = (torch.cat([pre[k][i][at[k]:at[k] + n] for k, n in step]).to(DEV) for i in range(3))
            out = torch.empty_like(zp)
            layer(out, zp, up, gp, state, batch)
            o = 0
            for k, n in step:
                got[k].append(out[o:o + n].float().cpu())
                o += n
                at[k] += n
        for k in got:
            g = torch.cat(got[k])
            assert float((g - want[k]).abs().max()) <= bar * max(1.0, float(want[k].abs().max())), (k, plan[0])


@pytest.mark.parametrize("act", ["relu", "relu2", "silu", "gelu_tanh"])
def test_activations(act):
    import math
    from vllm_legacy_amd.layers import GatedActivation
    z = rnd((6, 2 * 37), 0, 2.0)
    g, u = z[:, :37].to(F), z[:, 37:].to(F)
    f = {"relu": torch.relu, "relu2": lambda t: torch.relu(t)**2, "silu": lambda t: t * torch.sigmoid(t),
         "gelu_tanh": lambda t: 0.5 * t * (1 + torch.tanh(math.sqrt(2 / math.pi) * (t + 0.044715 * t**3)))}[act]
    got = GatedActivation(act)(z.to(DEV)).cpu()
    assert float((got - f(g) * u).abs().max()) <= 1e-5
    got = GatedActivation(act, gated=False)(z.to(DEV)).cpu()
    assert float((got - f(z.to(F))).abs().max()) <= 1e-5
    # 16-bit rows of a multiple of eight values take the vector form
    zb = rnd((5, 2 * 72), 1, 2.0).to(torch.bfloat16)
    got = GatedActivation(act)(zb.to(DEV)).float().cpu()
    want = f(zb[:, :72].to(F)) * zb[:, 72:].to(F)
    assert float((got - want).abs().max()) <= 0.02 * float(want.abs().max())


MOE_SHAPES = [
    # width, experts, identity, top, ff, shared_ff
    (64, 6, 1, 2, 24, 32),
    (40, 3, 0, 1, 20, 0),
    (64, 1, 2, 3, 16, 8),
    (96, 10, 3, 2, 48, 80),
    (72, 5, 3, 4, 130, 0),
    (50, 4, 1, 2, 9, 7),       # sizes the matrix-core product does not take: the plain one runs
    (72, 2, 0, 1, 40, 0),      # multiples of 8 but not of 16: the narrower matrix-core product
    (64, 2, 0, 2, 48, 16),     # two experts, both chosen: long runs of tiles of one expert
]


@pytest.mark.parametrize("shape", MOE_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routed_experts(shape, dtype):
    from vllm_legacy_amd.routed_experts import RoutedExperts
    W, E, I, top, ff, sff = shape
    mlp = R.moe_mlp(E, I, top, ff, sff)
    cfg = R.make_config([R.mingru_layer(8, mlp)], width=W)
    t = R.sub(R.make_weights(cfg, seed=3), "l0.mlp.")
    layer = RoutedExperts(W, E, I, top, ff, sff, dtype=dtype, device=DEV)
    layer.set_weights(t)
    for T in (1, 2, 33, 150, 300):
        h = rnd((T, W), T).to(dtype)
        tt = {k: v.to(F) for k, v in t.items()}
        want = R.moe_ff(h.to(F), tt, mlp)
        idx, w = R.route(h.to(F), tt, top)
        from vllm_legacy_amd import _seq_ops as ops
        ge, gw, _ = ops.moe_route(h.to(DEV), layer.router.data, layer.correction.data, None, top)
        # a token whose choice is clear must get the reference's experts, in its order of scores
        s = torch.softmax(h.to(F) @ tt["router"].T, -1) + tt["correction"]
        srt = torch.sort(s, -1, descending=True).values
        clear = (srt[:, :top] - srt[:, 1:top + 1]).min(-1).values > 1e-3 if top < E + I else torch.ones(T, dtype=torch.bool)
        assert torch.equal(torch.sort(ge.cpu()[clear].long(), -1).values, torch.sort(idx[clear], -1).values)
        got = layer(h.to(DEV)).cpu()
        if T == 150:        # the same step with the router's logits from a matrix product
            layer.ROUTE_PRODUCT_MIN_TOKENS = 100
            other = layer(h.to(DEV)).cpu()
            del layer.ROUTE_PRODUCT_MIN_TOKENS
            assert float(((other - got).abs().max(-1).values / want.abs().max())[clear].max()) <= 1e-5
        bar = 2e-5 if dtype == torch.float32 else 0.03
        err = (got - want).abs().max(-1).values / want.abs().max()
        assert float(err[clear].max()) <= bar, (T, float(err[clear].max()))


@pytest.mark.parametrize("shape", [(64, 2, 0, 2, 64, 16), (128, 5, 1, 2, 64, 0), (64, 3, 0, 1, 48, 0)])
@pytest.mark.parametrize("form", [1, 2])
def test_grouped_products_in_every_form(shape, form):
    """The 16-bit expert products in the form for decode steps and in the forms for prompts (runs of
    tiles of one expert; through LDS where the inner size is a multiple of 64)."""
    from vllm_legacy_amd import _seq_ops as ops
    from vllm_legacy_amd.routed_experts import RoutedExperts
    W, E, I, top, ff, sff = shape
    mlp = R.moe_mlp(E, I, top, ff, sff)
    cfg = R.make_config([R.mingru_layer(8, mlp)], width=W)
    t = R.sub(R.make_weights(cfg, seed=5), "l0.mlp.")
    layer = RoutedExperts(W, E, I, top, ff, sff, dtype=torch.bfloat16, device=DEV)
    layer.set_weights(t)
    tt = {k: v.to(F) for k, v in t.items()}
    ops.set_grouped_linear_form(form)
    try:
        for T in (3, 70, 333):
            h = rnd((T, W), T).to(torch.bfloat16)
            want = R.moe_ff(h.to(F), tt, mlp)
            s = torch.softmax(h.to(F) @ tt["router"].T, -1) + tt["correction"]
            srt = torch.sort(s, -1, descending=True).values
            clear = (srt[:, :top] - srt[:, 1:top + 1]).min(-1).values > 1e-3 if top < E + I else torch.ones(T, dtype=torch.bool)
            got = layer(h.to(DEV)).cpu()
            err = (got - want).abs().max(-1).values / want.abs().max()
            assert float(err[clear].max()) <= 0.03, (T, float(err[clear].max()))
    finally:
        ops.set_grouped_linear_form(0)


# ------------------------------------------------------------------------------------------------
# whole models

@pytest.mark.parametrize("name", list(configs()))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_whole_prompt_portions_and_decoding_agree_with_the_reference(tmp_path, name, dtype):
    s = Served(tmp_path, name, dtype)
    n = 70 if name == "mfma" else 41
    toks = tokens_of(s.cfg, n, 1)
    want = s.reference(toks)

    def run(sizes, sid):
        got, lo, i = [], 0, 0
        while lo < n:
            c = min(sizes[i % len(sizes)], n - lo)
            got.append(s.step([(sid, toks[lo:lo + c])])[sid])
            lo += c
            i += 1
        s.end(sid)
        return torch.cat(got)

    for sid, sizes in (("whole", [n]), ("portions", [2, 3, 4, 5, 1, 7, 2]), ("prefill+decode", [n - 12] + [1] * 12),
                       ("long portions", [33, 40, 5]), ("tokens", [1])):
        within(logit_error(run(sizes, sid), want), dtype, sid)


@pytest.mark.parametrize("name", ["plain", "odd"])
def test_layer_by_layer_against_the_reference(tmp_path, name):
    """The residual stream after every layer run, float32."""
    s = Served(tmp_path, name, torch.float32)
    toks = tokens_of(s.cfg, 17, 4)
    taps = []
    R.forward(toks, s.cfg, s.W, taps)
    s.cache.admit("a")
    s.cache.grow("a", 17)
    batch = make_batch([17], [0], 4, tables=[s.cache.block_table("a")], slots=[s.cache.state_slot("a")])
    got = []
    with torch.inference_mode():
        s.model(torch.tensor(toks, device=DEV), batch.positions, s.runner.caches, batch,
                tap=lambda run, x: got.append(x.detach().cpu().clone()))
    assert len(got) == len(taps) == len(s.model.runs)
    for run, (a, b) in enumerate(zip(got, taps)):
        assert float((a.to(F) - b).abs().max() / b.abs().max()) <= 2e-5, run


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixed_batches_with_pages_and_slots_used_again(tmp_path, dtype):
    """Three slots, a pool that cannot hold all five requests at once: requests end, their
    pages and slots go to later ones; every step mixes portions and single tokens."""
    s = Served(tmp_path, "plain", dtype, num_blocks=30, block_size=4, num_slots=3)
    reqs = {k: tokens_of(s.cfg, n, i) for i, (k, n) in enumerate([("a", 45), ("b", 9), ("c", 30), ("d", 38), ("e", 2)])}
    plan = [
        [("a", 5), ("b", 2)],
        [("a", 16), ("b", 1), ("c", 2)],
        [("b", 1), ("c", 7), ("a", 1)],
        [("a", 9), ("b", 5), ("c", 1)],          # b ends here (9 tokens)
        [("d", 3), ("a", 1), ("c", 13)],         # d takes b's slot and pages
        [("d", 1), ("a", 13), ("c", 7)],         # a and c end
        [("d", 30), ("e", 1)],
        [("e", 1), ("d", 1)],
        [("d", 3)],
    ]
    got = {k: [] for k in reqs}
    at = {k: 0 for k in reqs}
    used_slots = {}
    for step in plan:
        entries = [(k, reqs[k][at[k]:at[k] + n]) for k, n in step]
        out = s.step(entries)
        for k, n in step:
            used_slots.setdefault(k, s.cache.state_slot(k))
            got[k].append(out[k])
            at[k] += n
            if at[k] == len(reqs[k]):
                s.end(k)
    assert at == {k: len(v) for k, v in reqs.items()}
    assert used_slots["d"] == used_slots["b"] and len(set(used_slots.values())) == 3
    for k in reqs:
        s.check(torch.cat(got[k]), reqs[k], k)


def test_long_decoding_over_many_pages(tmp_path):
    s = Served(tmp_path, "taps", torch.float32, num_blocks=80, block_size=4)
    toks = tokens_of(s.cfg, 200, 8)
    got = [s.step([("a", toks[:3])])["a"]]
    for t in range(3, 200):
        got.append(s.step([("a", toks[t:t + 1])])["a"])
    s.check(torch.cat(got), toks)


def test_long_prompts_walk_the_recurrence_in_pieces(tmp_path):
    """Prompts long enough for the recurrent layers to walk them in pieces, whole and in large
    portions beside a decoding request; then decoding goes on from the state the pieces left."""
    s = Served(tmp_path, "taps", torch.float32, num_blocks=100, block_size=16)
    a, b = tokens_of(s.cfg, 300, 5), tokens_of(s.cfg, 560, 6)
    got_a = [s.step([("a", a[:290])])["a"]] + [s.step([("a", a[t:t + 1])])["a"] for t in range(290, 300)]
    s.check(torch.cat(got_a), a, "whole + decode")
    s.end("a")
    got_b = [s.step([("b", b[:257])])["b"], s.step([("b", b[257:554]), ("a", a[:3])])["b"]]
    got_b += [s.step([("b", b[t:t + 1])])["b"] for t in range(554, 560)]
    s.check(torch.cat(got_b), b, "portions + decode")


def test_a_batch_does_not_change_a_request(tmp_path):
    """The same request alone and beside two others: equal beyond rounding (float32)."""
    s = Served(tmp_path, "odd", torch.float32)
    a, b, c = (tokens_of(s.cfg, n, i) for i, n in enumerate((33, 12, 50)))
    alone = torch.cat([s.step([("a", a[:20])])["a"], s.step([("a", a[20:])])["a"]])
    s.end("a")
    s.step([("c", c[:41])])
    first = s.step([("b", b[:5]), ("a", a[:20]), ("c", c[41:42])])["a"]
    second = s.step([("c", c[42:43]), ("a", a[20:]), ("b", b[5:])])["a"]
    both = torch.cat([first, second])
    assert float(logit_error(both, alone).max()) <= 1e-5


def greedy_reference(s, prompt, n):
    """(tokens, how clear each choice was): a choice closer than the bar is a tie."""
    toks, margins = list(prompt), []
    for _ in range(n):
        last = s.reference(toks)[-1]
        top = torch.topk(last, 2).values
        margins.append(float(top[0] - top[1]))
        toks.append(int(torch.argmax(last)))
    return toks[len(prompt):], margins


@pytest.mark.parametrize("num_blocks,preempt", [(64, False), (9, True)])
def test_greedy_generation_through_the_engine(tmp_path, num_blocks, preempt):
    from vllm_legacy_amd.engine import EngineConfig, LLMEngine, SamplingParams
    s = Served(tmp_path, "plain", torch.float32)
    engine = LLMEngine(s.model, EngineConfig(block_size=4, num_blocks=num_blocks, max_num_seqs=3,
                                             max_num_batched_tokens=7), DEV)
    prompts = [tokens_of(s.cfg, n, 20 + n) for n in (11, 3, 6, 1)]
    outs = engine.generate(prompts, SamplingParams(max_tokens=8))
    assert (engine.scheduler.num_preemptions > 0) == preempt
    assert engine.cache.free_blocks == num_blocks and engine.cache.free_slots == 3
    for p, o in zip(prompts, outs):
        want, margins = greedy_reference(s, p, 8)
        assert o.finished and o.finish_reason == "length" and len(o.token_ids) == 8
        for t, (a, b, m) in enumerate(zip(o.token_ids, want, margins)):
            if m < 1e-3:
                break                      # a tie within rounding: what follows may differ
            assert a == b, (t, a, b)


def test_generation_from_a_folder_and_the_command_line(tmp_path):
    """LLMEngine.from_pretrained picks the model class by config.json; the command line prints the
    same greedy tokens."""
    from vllm_legacy_amd.engine import EngineConfig, LLMEngine, SamplingParams
    s = Served(tmp_path, "equal", torch.float32)
    engine = LLMEngine.from_pretrained(s.folder, torch.float32, EngineConfig(block_size=4, num_blocks=40, max_num_seqs=2), DEV)
    assert type(engine.runner.model).__name__ == "DopipelForCausalLM"
    p = tokens_of(s.cfg, 7, 3)
    first = engine.generate([p], SamplingParams(max_tokens=6))[0].token_ids
    out = engine.generate([p], SamplingParams(max_tokens=6, stop_token_ids=[first[2]]))[0]
    assert out.finish_reason == "stop" and out.token_ids == first[:first.index(first[2]) + 1]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-m", "vllm_legacy_amd.engine.cli", "generate", "--model", s.folder, "--dtype",
                        "float32", "--prompt", ",".join(map(str, p)), "--max-tokens", "6", "--num-blocks", "64"],
                       cwd=root, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert json.loads(r.stdout.strip().splitlines()[-1])["token_ids"] == first


def test_trace_replayer_as_a_program(tmp_path):
    """bin/trace_run fed four steps (two requests, a portion beside a single token, a request that
    ends and whose id comes back as a new request) writes the logits the reference gives."""
    s = Served(tmp_path, "odd", torch.float32)
    a, b = tokens_of(s.cfg, 9, 1), tokens_of(s.cfg, 4, 2)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:6], "want": [0, 5]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[6:7], "want": []}, {"id": "b", "tokens": b[:3], "want": [2]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[3:], "want": [0]}, {"id": "a", "tokens": a[7:], "want": [1]}], "end": ["a", "b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": b, "want": [3]}], "end": ["a"]},
    ]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", s.folder, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(x) for x in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
    import numpy as np
    ra, rb = s.reference(a), s.reference(b)
    V = s.cfg["vocab"]
    want = {0: ra[[0, 5]], 1: rb[[2]], 2: torch.stack([rb[3], ra[8]]), 3: rb[[3]]}
    for n, w in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, V))
        assert got.shape == w.shape and float(logit_error(got, w).max()) <= 1e-4, n
