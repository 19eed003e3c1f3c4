"""Lusadra: a decoder-only stack of parallel layers over an fp32 residual stream.

  x = embed[token] + sinusoid(position)
  layers `loop.start .. loop.stop - 1` run `loop.times` passes with the same weights; every pass
  has its own cache and state ("layer runs"); before pass t its first layer adds the embedding
  output again (t > 0) and the row t of `loop.step`
  layer:  h = g * x / rms(x);   x += mixer(h) + ff(h)           (one norm, two readers)
  mixer:  left_scale * windowed key attention(h) + right_scale * gated linear attention(h)
  ff:     W_down PolyNorm(W_up h)                                (absent when mlp is null)
  logits = head (g_final * x / rms(x))

All sizes and per-model constants come from config.json; a layer entry carries its own mixer
sizes, so layers of one model may differ.  The nine projections that read h are one matrix
product, and so are the three that write x (their inputs are laid side by side in one buffer by
the kernels that produce them, already multiplied by left_scale / right_scale); matrix products go
to the vendor library, everything else runs on libvla_seq_gfx950.so.  The residual stream, norms,
attention scores and weights, decays and the recurrent state are fp32 whatever `dtype` is;
`dtype` is the type of weights, projections and activations (bfloat16 to serve, float32 for an
all-fp32 run).
"""
import json
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn as nn

from vllm_legacy_amd import _seq_ops as ops
from vllm_legacy_amd.attention.backends.windowed_keys import WindowedKeyAttention, geometric_slopes
from vllm_legacy_amd.attention.batch import SequenceBatch
from vllm_legacy_amd.attention.recurrent import GatedLinearRecurrence
from vllm_legacy_amd.layers import PolyNorm, ScalarRMSNorm, SinusoidalEmbedding


@dataclass
class WindowedSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int
    scale: float
    temp_coef: float
    temp_every: float


@dataclass
class RecurrentSpec:
    heads: int
    dim: int
    vdim: int
    tau: float


@dataclass
class LayerSpec:
    left: WindowedSpec
    right: RecurrentSpec
    left_scale: float
    right_scale: float
    ff: int            # 0: no feed-forward


@dataclass
class LusadraConfig:
    vocab: int
    width: int
    eps: float
    layers: List[LayerSpec]
    loop_start: int
    loop_stop: int
    loop_times: int
    architecture: str = "Lusadra"
    raw: Dict = field(default_factory=dict, repr=False)

    @staticmethod
    def from_dict(d: Dict) -> "LusadraConfig":
        layers = []
        for i, entry in enumerate(d["layers"]):
            if entry.get("type") != "parallel":
                raise ValueError(f"layer {i}: unknown layer type {entry.get('type')!r}")
            m = entry["mixer"]
            le, ri = m["left"], m["right"]
            if le.get("vdim", le["dim"]) != le["dim"]:
                raise ValueError(f"layer {i}: values are the keys, so vdim must equal dim")
            temp = le.get("q_temp") or {}
            left = WindowedSpec(int(le["heads"]), int(le.get("kv_heads", le["heads"])), int(le["dim"]),
                                int(le.get("vdim", le["dim"])), int((le.get("mask") or {}).get("size", 0)),
                                float(le["scale"]), float(temp.get("coef", 0.0)),
                                float(temp.get("every", 1.0)))
            right = RecurrentSpec(int(ri["heads"]), int(ri["dim"]), int(ri["vdim"]), float(ri["tau"]))
            mlp = entry.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            layers.append(LayerSpec(left, right, float(m["left_scale"]), float(m["right_scale"]),
                                    0 if mlp is None else int(mlp["ff"])))
        loop = d.get("loop") or {"start": 0, "stop": 0, "times": 1}
        cfg = LusadraConfig(int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]), layers,
                            int(loop["start"]), int(loop["stop"]), int(loop["times"]),
                            d.get("architecture", "Lusadra"), d)
        if not (0 <= cfg.loop_start <= cfg.loop_stop <= len(layers)) or cfg.loop_times < 1:
            raise ValueError("loop: need 0 <= start <= stop <= number of layers and times >= 1")
        return cfg

    @staticmethod
    def from_json(path: str) -> "LusadraConfig":
        with open(path) as f:
            return LusadraConfig.from_dict(json.load(f))

    def layer_runs(self) -> List[Tuple[int, Optional[int]]]:
        """(layer, pass) in execution order; pass is the number of the pass this run opens, None
        for a run that opens none."""
        runs: List[Tuple[int, Optional[int]]] = [(i, None) for i in range(self.loop_start)]
        if self.loop_stop > self.loop_start:
            for t in range(self.loop_times):
                for i in range(self.loop_start, self.loop_stop):
                    runs.append((i, t if i == self.loop_start else None))
        runs += [(i, None) for i in range(self.loop_stop, len(self.layers))]
        return runs


class LusadraLayer(nn.Module):

    def __init__(self, cfg: LusadraConfig, spec: LayerSpec, dtype, device, generator=None):
        super().__init__()
        self.spec, self.dtype, W = spec, dtype, cfg.width
        le, ri = spec.left, spec.right
        self.norm1 = ScalarRMSNorm(cfg.eps, device)
        self.attn = WindowedKeyAttention(le.heads, le.kv_heads, le.dim, le.scale, le.window,
                                         geometric_slopes(le.heads), le.temp_coef, le.temp_every, device)
        self.recur = GatedLinearRecurrence(ri.heads, ri.dim, ri.vdim, ri.tau, cfg.eps)
        self.act = PolyNorm(cfg.eps, device) if spec.ff else None
        self.rank = 0   # set with the weights (the low-rank width is a tensor's shape)
        # column ranges of the merged input projection and of the merged output projection's input
        self.in_names = ["mix.left.q", "mix.left.k", "mix.left.g", "mix.right.q", "mix.right.k",
                         "mix.right.v", "mix.right.g", "mix.right.a1"] + (["mlp.up"] if spec.ff else [])
        self.out_names = ["mix.left.o", "mix.right.o"] + (["mlp.down"] if spec.ff else [])
        self.out_widths = [le.heads * le.vdim, ri.heads * ri.vdim] + ([spec.ff] if spec.ff else [])
        self.w_in = nn.Parameter(torch.empty(0, dtype=dtype, device=device), requires_grad=False)
        self.w_out = nn.Parameter(torch.empty(0, dtype=dtype, device=device), requires_grad=False)
        self.w_a2 = nn.Parameter(torch.empty(0, dtype=dtype, device=device), requires_grad=False)
        self.b_a2 = nn.Parameter(torch.zeros(ri.heads * ri.dim, dtype=torch.float32, device=device),
                                 requires_grad=False)
        self.recur_norm = nn.Parameter(torch.ones(ri.vdim, dtype=torch.float32, device=device),
                                       requires_grad=False)
        self.in_widths: List[int] = []
        if generator is not None:
            self._random_init(W, 16, device, generator)

    def in_shapes(self, width: int, rank: int) -> List[Tuple[int, int]]:
        le, ri = self.spec.left, self.spec.right
        rows = [le.heads * le.dim, le.kv_heads * le.dim, le.heads * le.vdim, ri.heads * ri.dim,
                ri.heads * ri.dim, ri.heads * ri.vdim, ri.heads * ri.vdim, rank]
        if self.spec.ff:
            rows.append(self.spec.ff)
        return [(r, width) for r in rows]

    def set_weights(self, t: Dict[str, torch.Tensor], width: int) -> None:
        """t: this layer's tensors by their names without the layer prefix."""
        dev, dt = self.w_in.device, self.dtype
        rank = t["mix.right.a1"].shape[0]
        for name, shape in zip(self.in_names, self.in_shapes(width, rank)):
            if tuple(t[name].shape) != shape:
                raise ValueError(f"{name}: shape {tuple(t[name].shape)}, expected {shape}")
        for name, k in zip(self.out_names, self.out_widths):
            if tuple(t[name].shape) != (width, k):
                raise ValueError(f"{name}: shape {tuple(t[name].shape)}, expected {(width, k)}")
        self.rank = rank
        self.in_widths = [t[n].shape[0] for n in self.in_names]
        self.w_in.data = torch.cat([t[n].to(dt) for n in self.in_names], 0).to(dev).contiguous()
        self.w_out.data = torch.cat([t[n].to(dt) for n in self.out_names], 1).to(dev).contiguous()
        ri = self.spec.right
        if tuple(t["mix.right.a2"].shape) != (ri.heads * ri.dim, rank):
            raise ValueError("mix.right.a2: shape does not fit heads * dim x rank")
        self.w_a2.data = t["mix.right.a2"].to(dt).to(dev).contiguous()
        self.b_a2.data = t["mix.right.a2.b"].float().to(dev).contiguous()
        self.recur_norm.data = t["mix.right.norm"].float().to(dev).contiguous()
        self.norm1.weight.data = t["norm1"].float().reshape(()).to(dev)
        if self.act is not None:
            self.act.weight.data = t["mlp.act"].float().to(dev).contiguous()

    def _random_init(self, width: int, rank: int, device, g) -> None:
        def rnd(shape, std):
            return torch.randn(shape, generator=g, dtype=torch.float32) * std
        t = {}
        for name, shape in zip(self.in_names, self.in_shapes(width, rank)):
            t[name] = rnd(shape, width**-0.5)
        for name, k in zip(self.out_names, self.out_widths):
            t[name] = rnd((width, k), 0.5 * k**-0.5)
        ri = self.spec.right
        t["mix.right.a2"] = rnd((ri.heads * ri.dim, rank), rank**-0.5)
        t["mix.right.a2.b"] = rnd((ri.heads * ri.dim, ), 1.0) + 2.0
        t["mix.right.norm"] = 1.0 + rnd((ri.vdim, ), 0.1)
        t["norm1"] = torch.tensor(1.0)
        t["mlp.act"] = torch.tensor([0.6, 0.3, 0.1, 0.0])
        self.set_weights(t, width)

    def forward(self, x: torch.Tensor, batch: SequenceBatch, key_cache: torch.Tensor,
                state: torch.Tensor, add_rows: Optional[torch.Tensor] = None,
                add_row: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x: fp32 [T, width], updated in place."""
        h = self.norm1(x, self.dtype, add_rows, add_row)
        proj = torch.matmul(h, self.w_in.t())
        ql, kl, gl, qr, kr, vr, gr, y, *up = proj.split(self.in_widths, dim=1)
        mixed = torch.empty((x.shape[0], sum(self.out_widths)), dtype=self.dtype, device=x.device)
        a, r, *f = mixed.split(self.out_widths, dim=1)
        self.attn(a, ql, kl, gl, key_cache, batch, self.spec.left_scale)
        self.recur(r, qr, kr, vr, gr, y, self.w_a2.data, self.b_a2.data, self.recur_norm.data, state,
                   batch, self.spec.right_scale)
        if self.act is not None:
            self.act(up[0], f[0])
        if self.dtype == torch.float32:
            x.addmm_(mixed, self.w_out.t())
        else:   # 16-bit operands, fp32 accumulator written as fp32: the sum never rounds to 16 bits
            ops.residual_add(x, torch.mm(mixed, self.w_out.t(), out_dtype=torch.float32))
        return x


class LusadraForCausalLM(nn.Module):
    """The stack and its per-run caches' shapes.  `seed` fills random weights (benchmarks, tests);
    load_weights installs a checkpoint's."""

    architecture = "Lusadra"

    def __init__(self, cfg: LusadraConfig, dtype=torch.bfloat16, device="cuda", seed: Optional[int] = None):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        g = None if seed is None else torch.Generator().manual_seed(seed)
        self.embed = SinusoidalEmbedding(cfg.vocab, cfg.width, dtype, device)
        self.layers = nn.ModuleList([LusadraLayer(cfg, s, dtype, device, g) for s in cfg.layers])
        self.loop_step = nn.Parameter(torch.zeros((cfg.loop_times, cfg.width), dtype=torch.float32,
                                                  device=device), requires_grad=False)
        self.final_norm = ScalarRMSNorm(cfg.eps, device)
        self.head = nn.Parameter(torch.zeros((cfg.vocab, cfg.width), dtype=dtype, device=device),
                                 requires_grad=False)
        self.runs = cfg.layer_runs()
        if g is not None:
            self.embed.weight.data = torch.randn((cfg.vocab, cfg.width), generator=g).to(dtype).to(device)
            self.head.data = (torch.randn((cfg.vocab, cfg.width), generator=g) * cfg.width**-0.5).to(dtype).to(device)
            self.loop_step.data = (torch.randn((cfg.loop_times, cfg.width), generator=g) * 0.1).to(device)

    # ------------------------------------------------------------------ caches
    def cache_spec(self) -> List[Dict[str, Tuple[int, ...]]]:
        """Per layer run: the key cache's (kv_heads, dim) and the recurrent state's
        (heads, dim, vdim); the engine's cache manager turns them into tensors."""
        out = []
        for i, _ in self.runs:
            s = self.cfg.layers[i]
            out.append({"keys": (s.left.kv_heads, s.left.dim),
                        "state": (s.right.heads, s.right.dim, s.right.vdim)})
        return out

    def allocate_caches(self, num_blocks: int, block_size: int, num_slots: int):
        dev = self.head.device
        caches = []
        for spec in self.cache_spec():
            keys = torch.zeros(WindowedKeyAttention.get_cache_shape(num_blocks, block_size, *spec["keys"]),
                               dtype=self.dtype, device=dev)
            # (the recurrent layer adds its scratch slots behind the sequences' own)
            state = torch.zeros(GatedLinearRecurrence.get_state_shape(num_slots, *spec["state"]),
                                dtype=torch.float32, device=dev)
            caches.append((keys, state))
        return caches

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, caches, batch: SequenceBatch,
                tap=None) -> torch.Tensor:
        """Returns the fp32 residual stream [T, width] after the last layer.  tap(run, x) is
        called after every layer run (tests, layer-by-layer comparison)."""
        x = self.embed(input_ids, positions)
        x0 = x.clone() if self.cfg.loop_times > 1 and self.cfg.loop_stop > self.cfg.loop_start else None
        for run, (i, opens) in enumerate(self.runs):
            keys, state = caches[run]
            add_rows = x0 if (opens is not None and opens > 0) else None
            add_row = self.loop_step.data[opens] if opens is not None else None
            x = self.layers[i](x, batch, keys, state, add_rows, add_row)
            if tap is not None:
                tap(run, x)
        return x

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """hidden: the rows of the stream whose logits are wanted -> fp32 [n, vocab]."""
        h = self.final_norm(hidden.contiguous(), self.dtype)
        if self.dtype == torch.float32:
            return torch.mm(h, self.head.t())
        return torch.mm(h, self.head.t(), out_dtype=torch.float32)

    # ------------------------------------------------------------------ weights
    def load_weights(self, tensors: Dict[str, torch.Tensor]) -> int:
        cfg, dev = self.cfg, self.head.device
        used = 0
        for i, layer in enumerate(self.layers):
            prefix = f"l{i}."
            mine = {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}
            layer.set_weights(mine, cfg.width)
            used += len(mine)
        for name, shape in (("embed", (cfg.vocab, cfg.width)), ("head", (cfg.vocab, cfg.width))):
            if tuple(tensors[name].shape) != shape:
                raise ValueError(f"{name}: shape {tuple(tensors[name].shape)}, expected {shape}")
        self.embed.weight.data = tensors["embed"].to(self.dtype).to(dev).contiguous()
        self.head.data = tensors["head"].to(self.dtype).to(dev).contiguous()
        self.final_norm.weight.data = tensors["final.norm"].float().reshape(()).to(dev)
        used += 3
        if "loop.step" in tensors:
            self.loop_step.data = tensors["loop.step"].float().to(dev).contiguous()
            used += 1
        return used
