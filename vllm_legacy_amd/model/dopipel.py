"""Dopipel: a decoder-only stack over an fp32 residual stream whose sublayers are normed on both
sides, with rotary attention layers and minGRU layers in any order and dense or mixture-of-experts
feed-forwards.

  x = embed[token]                                    (x0: this embedding output)
  layers `loop.start .. loop.stop - 1` run `loop.times` passes with the same weights; every pass
  has its own caches and states ("layer runs"); a pass t opens with x <- W_in [x; x0] + step[t]
  layer:  h = N1(x);  h <- h + conv(h)                (causal, `taps` taps per channel)
          x += ls1 * N1b(mixer(h));   x += ls2 * N2b(ff(N2(x)))
          N(u) = u / rms(u) * w, every norm with its own weight
  mixer 'attention': q, k, v (with biases) from h; rotary q, k; values rotated by their position,
          the head's output turned back by the query's; causal softmax; each head times
          sigmoid(W_g h)_head; output projection with bias
  mixer 'mingru':  S_t = (1 - z) S_(t-1) + z c, z = sigmoid(W_z h + b), c from W_x h + b;
          output W_o (S_t * silu(W_g h))
  ff 'dense':  W_down (relu(W_gate h) * W_up h)
  ff 'moe':    top experts of a softmax router (scores + correction choose, scores weigh), experts
          W_down relu(W_up h)^2, identity experts, a shared expert times sigmoid(w_sg . h)
  logits = head N_final(x)

All sizes and per-model constants come from config.json; a layer entry carries its own mixer and
feed-forward sizes.  The projections that read h are one matrix product per sublayer; matrix
products go to the vendor library, everything else runs on libvla_seq_gfx950.so.  The residual
stream, norms, angles, attention scores and weights, routers, gates of the recurrence and its state
are fp32 whatever `dtype` is; `dtype` is the type of weights, projections and activations
(bfloat16 to serve, float32 for an all-fp32 run).  The residual update that closes a sublayer and
the norm that opens the next one are one launch, across layers too.
"""
import json
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn as nn

from vllm_legacy_amd import _seq_ops as ops
from vllm_legacy_amd.attention.backends.rotary_kv import RotaryKVAttention
from vllm_legacy_amd.attention.batch import SequenceBatch
from vllm_legacy_amd.attention.recurrent import MinGRURecurrence
from vllm_legacy_amd.layers import CausalConvMix, GatedActivation
from vllm_legacy_amd.routed_experts import RoutedExperts, mm_f32


@dataclass
class AttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float
    interleaved: bool = True
    window: int = 0


@dataclass
class MinGRUSpec:
    width: int


@dataclass
class MlpSpec:
    kind: str                   # dense | moe
    ff: int = 0                 # dense: hidden size; moe: an expert's
    experts: int = 0
    identity: int = 0
    top: int = 0
    shared_ff: int = 0
    act: str = "relu"


@dataclass
class LayerSpec:
    type: str                   # attention | mingru
    mixer: object
    mlp: Optional[MlpSpec]


@dataclass
class DopipelConfig:
    vocab: int
    width: int
    eps: float
    taps: int                   # 0: no input convolution
    layers: List[LayerSpec]
    loop_start: int
    loop_stop: int
    loop_times: int
    architecture: str = "Dopipel"
    raw: Dict = field(default_factory=dict, repr=False)

    @staticmethod
    def from_dict(d: Dict) -> "DopipelConfig":
        layers = []
        for i, entry in enumerate(d["layers"]):
            kind, m = entry.get("type"), entry.get("mixer") or {}
            if kind == "attention":
                rot = m.get("rot") or {}
                dim = int(m["dim"])
                layout = rot.get("layout", "interleaved")
                if layout not in ("interleaved", "halves"):
                    raise ValueError(f"layer {i}: unknown rotary layout {layout!r}")
                mixer = AttentionSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), dim,
                                      int(m.get("vdim", dim)), float(m.get("scale", dim**-0.5)),
                                      int(rot.get("dims", dim)) if rot else 0, float(rot.get("base", 10000.0)),
                                      layout == "interleaved", int((m.get("mask") or {}).get("size", 0)))
                if mixer.heads % mixer.kv_heads or mixer.rot_dims % 2 or mixer.rot_dims > dim or mixer.vdim % 2:
                    raise ValueError(f"layer {i}: heads / kv_heads / rot.dims / vdim do not fit")
            elif kind == "mingru":
                mixer = MinGRUSpec(int(m["width"]))
            else:
                raise ValueError(f"layer {i}: unknown layer type {kind!r}")
            mlp = entry.get("mlp")
            if mlp is None:
                spec = None
            elif mlp.get("kind") == "dense":
                spec = MlpSpec("dense", int(mlp["ff"]), act=mlp.get("act", "relu"))
            elif mlp.get("kind") == "moe":
                r = mlp["router"]
                shared = mlp.get("shared") or {}
                spec = MlpSpec("moe", int(mlp["expert"]["ff"]), int(r["experts"]), int(r.get("identity", 0)),
                               int(r["top"]), int(shared.get("ff", 0)), mlp.get("act", "relu2"))
                if spec.top < 1 or spec.top > spec.experts + spec.identity:
                    raise ValueError(f"layer {i}: router.top does not fit the number of experts")
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            layers.append(LayerSpec(kind, mixer, spec))
        loop = d.get("loop") or {"start": 0, "stop": 0, "times": 1}
        cfg = DopipelConfig(int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]),
                            int((d.get("canon") or {}).get("taps", 0)), layers, int(loop["start"]),
                            int(loop["stop"]), int(loop["times"]), d.get("architecture", "Dopipel"), d)
        if not (0 <= cfg.loop_start <= cfg.loop_stop <= len(layers)) or cfg.loop_times < 1:
            raise ValueError("loop: need 0 <= start <= stop <= number of layers and times >= 1")
        return cfg

    @staticmethod
    def from_json(path: str) -> "DopipelConfig":
        with open(path) as f:
            return DopipelConfig.from_dict(json.load(f))

    @property
    def loops(self) -> bool:
        return self.loop_stop > self.loop_start

    def layer_runs(self) -> List[Tuple[int, Optional[int]]]:
        """(layer, pass) in execution order; pass is the number of the pass this run opens, None
        for a run that opens none."""
        runs: List[Tuple[int, Optional[int]]] = [(i, None) for i in range(self.loop_start)]
        if self.loops:
            for t in range(self.loop_times):
                for i in range(self.loop_start, self.loop_stop):
                    runs.append((i, t if i == self.loop_start else None))
        runs += [(i, None) for i in range(self.loop_stop, len(self.layers))]
        return runs


@dataclass
class Pending:
    """A sublayer's result that is not in the stream yet: x += ls * N(y + bias)."""
    y: torch.Tensor
    bias: Optional[torch.Tensor]
    norm: torch.Tensor
    scale: torch.Tensor


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


class DopipelLayer(nn.Module):

    def __init__(self, cfg: DopipelConfig, spec: LayerSpec, dtype, device):
        super().__init__()
        self.spec, self.dtype, self.eps, W = spec, dtype, cfg.eps, cfg.width

        def vec(n=W):
            return nn.Parameter(torch.ones(n, dtype=torch.float32, device=device), requires_grad=False)

        def mat(rows, cols, dt=dtype):
            return nn.Parameter(torch.zeros((rows, cols), dtype=dt, device=device), requires_grad=False)

        self.norm1, self.norm1b, self.norm2, self.norm2b = vec(), vec(), vec(), vec()
        self.ls1, self.ls2 = vec(), vec()
        self.conv = CausalConvMix(W, cfg.taps, device) if cfg.taps else None
        m = spec.mixer
        if spec.type == "attention":
            self.attn = RotaryKVAttention(m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.rot_dims, m.rot_base,
                                          m.interleaved, True, m.window, device)
            self.in_names = ["mix.q", "mix.k", "mix.v", "mix.g"]
            self.in_widths = [m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim, m.heads]
            self.in_bias = [True, True, True, False]
            self.mixed = m.heads * m.vdim
            self.out_bias = vec()
        else:
            self.recur = MinGRURecurrence(m.width)
            self.in_names = ["mix.z", "mix.x", "mix.g"]
            self.in_widths = [m.width] * 3
            self.in_bias = [True, True, False]
            self.mixed = m.width
            self.out_bias = None
        # the merged input projection's rows are padded to a multiple of 8 so that every row of its
        # result starts 16-byte aligned
        rows = _pad8(sum(self.in_widths))
        self.pad = rows - sum(self.in_widths)
        self.w_in, self.b_in = mat(rows, W), nn.Parameter(torch.zeros(rows, dtype=dtype, device=device),
                                                          requires_grad=False)
        self.w_out = mat(W, self.mixed)
        mlp = spec.mlp
        if mlp is None:
            self.ff = None
        elif mlp.kind == "dense":
            self.w_gate_up, self.w_down = mat(2 * mlp.ff, W), mat(W, mlp.ff)
            self.act = GatedActivation(mlp.act)
        else:
            self.experts = RoutedExperts(W, mlp.experts, mlp.identity, mlp.top, mlp.ff, mlp.shared_ff, mlp.act,
                                         dtype=dtype, device=device)

    # ------------------------------------------------------------------ weights
    def tensor_shapes(self, cfg: DopipelConfig) -> Dict[str, Tuple[int, ...]]:
        """Checkpoint names (without the layer prefix) and shapes of this layer's tensors."""
        W, mlp = cfg.width, self.spec.mlp
        t: Dict[str, Tuple[int, ...]] = {n: (W, ) for n in ("norm1", "norm2", "norm1b", "norm2b", "ls1", "ls2")}
        if cfg.taps:
            t["canon1"] = (W, cfg.taps)
        for name, n, b in zip(self.in_names, self.in_widths, self.in_bias):
            t[name] = (n, W)
            if b:
                t[name + ".b"] = (n, )
        t["mix.o"] = (W, self.mixed)
        if self.out_bias is not None:
            t["mix.o.b"] = (W, )
        if mlp is not None and mlp.kind == "dense":
            t.update({"mlp.gate": (mlp.ff, W), "mlp.up": (mlp.ff, W), "mlp.down": (W, mlp.ff)})
        elif mlp is not None:
            for e in range(mlp.experts):
                t[f"mlp.e{e}.up"], t[f"mlp.e{e}.down"] = (mlp.ff, W), (W, mlp.ff)
            t["mlp.router"] = (mlp.experts + mlp.identity, W)
            t["mlp.correction"] = (mlp.experts + mlp.identity, )
            if mlp.shared_ff:
                t.update({"mlp.shared.up": (mlp.shared_ff, W), "mlp.shared.down": (W, mlp.shared_ff),
                          "mlp.shared.sg": (1, W)})
        return t

    def set_weights(self, t: Dict[str, torch.Tensor], cfg: DopipelConfig) -> None:
        """t: this layer's tensors by their names without the layer prefix."""
        dev, dt = self.w_in.device, self.dtype
        for name, shape in self.tensor_shapes(cfg).items():
            if name not in t:
                if name == "mlp.correction":        # a router without a correction chooses by its scores
                    continue
                raise KeyError(f"tensor {name} is missing")
            if tuple(t[name].shape) != shape:
                raise ValueError(f"{name}: shape {tuple(t[name].shape)}, expected {shape}")

        def f32(name):
            return t[name].float().to(dev).contiguous()

        for nm in ("norm1", "norm2", "norm1b", "norm2b", "ls1", "ls2"):
            getattr(self, nm).data = f32(nm)
        if self.conv is not None:
            self.conv.weight.data = f32("canon1")
        W = cfg.width
        parts = [t[n].to(dt) for n in self.in_names] + [torch.zeros((self.pad, W), dtype=dt)]
        bias = [t[n + ".b"].to(dt) if b else torch.zeros(w, dtype=dt)
                for n, w, b in zip(self.in_names, self.in_widths, self.in_bias)] + [torch.zeros(self.pad, dtype=dt)]
        self.w_in.data = torch.cat(parts, 0).to(dev).contiguous()
        self.b_in.data = torch.cat(bias, 0).to(dev).contiguous()
        self.w_out.data = t["mix.o"].to(dt).to(dev).contiguous()
        if self.out_bias is not None:
            self.out_bias.data = f32("mix.o.b")
        mlp = self.spec.mlp
        if mlp is not None and mlp.kind == "dense":
            self.w_gate_up.data = torch.cat([t["mlp.gate"], t["mlp.up"]], 0).to(dt).to(dev).contiguous()
            self.w_down.data = t["mlp.down"].to(dt).to(dev).contiguous()
        elif mlp is not None:
            self.experts.set_weights({k[4:]: v for k, v in t.items() if k.startswith("mlp.")})

    # ------------------------------------------------------------------ caches
    def cache_shapes(self, cfg: DopipelConfig, num_blocks: int, block_size: int, num_slots: int):
        """name -> (shape, dtype) of what one run of this layer keeps between steps."""
        m = self.spec.mixer
        out = {}
        if self.conv is not None and cfg.taps > 1:
            out["conv"] = (CausalConvMix.get_state_shape(num_slots, cfg.width, cfg.taps), torch.float32)
        if self.spec.type == "attention":
            ks, vs = RotaryKVAttention.get_cache_shapes(num_blocks, block_size, m.kv_heads, m.dim, m.vdim)
            out["keys"], out["values"] = (ks, self.dtype), (vs, self.dtype)
        else:
            out["state"] = (MinGRURecurrence.get_state_shape(num_slots, m.width), torch.float32)
        return out

    # ------------------------------------------------------------------ forward
    def forward(self, x: torch.Tensor, batch: SequenceBatch, cache: Dict[str, torch.Tensor],
                pending: Optional[Pending], add_row: Optional[torch.Tensor] = None) -> Pending:
        """x: fp32 [T, width], updated in place except for the last sublayer's result, which comes
        back as Pending (the next norm's launch adds it)."""
        T, dev = x.shape[0], x.device
        h32 = torch.empty_like(x)
        _apply(x, pending, add_row, h32, self.norm1.data, self.eps)
        if self.conv is not None:
            h = self.conv(h32, cache.get("conv"), batch, self.dtype)
        else:
            h = h32 if self.dtype == torch.float32 else h32.to(self.dtype)
        proj = torch.addmm(self.b_in.data, h, self.w_in.data.t())
        mixed = torch.empty((T, self.mixed), dtype=self.dtype, device=dev)
        if self.spec.type == "attention":
            q, k, v, g = proj.split(self.in_widths + [self.pad], dim=1)[:4]
            self.attn(mixed, q, k, v, g, cache["keys"], cache["values"], batch)
        else:
            zp, up, gp = proj.split(self.in_widths + [self.pad], dim=1)[:3]
            self.recur(mixed, zp, up, gp, cache["state"], batch)
        pending = Pending(mm_f32(mixed, self.w_out.data), None if self.out_bias is None else self.out_bias.data,
                          self.norm1b.data, self.ls1.data)
        mlp = self.spec.mlp
        if mlp is None:
            return pending
        h2 = torch.empty((T, x.shape[1]), dtype=self.dtype, device=dev)
        _apply(x, pending, None, h2, self.norm2.data, self.eps)
        if mlp.kind == "dense":
            y = mm_f32(self.act(torch.mm(h2, self.w_gate_up.data.t())), self.w_down.data)
        else:
            y = self.experts(h2)
        return Pending(y, None, self.norm2b.data, self.ls2.data)


def _apply(x: torch.Tensor, pending: Optional[Pending], add_row: Optional[torch.Tensor],
           out: Optional[torch.Tensor], pre_weight: Optional[torch.Tensor], eps: float) -> None:
    """One launch: the pending sublayer result into the stream, a row added, the next norm."""
    if pending is None and add_row is None and out is None:
        return
    if pending is None:
        ops.residual_norms(x, add_row=add_row, out=out, pre_weight=pre_weight, eps=eps)
    else:
        ops.residual_norms(x, pending.y, pending.bias, pending.norm, pending.scale, add_row, out, pre_weight, eps)


class DopipelForCausalLM(nn.Module):
    """The stack and its per-run caches.  `seed` fills random weights (benchmarks); load_weights
    installs a checkpoint's."""

    architecture = "Dopipel"

    def __init__(self, cfg: DopipelConfig, dtype=torch.bfloat16, device="cuda", seed: Optional[int] = None):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        W = cfg.width
        self.embed = nn.Parameter(torch.zeros((cfg.vocab, W), dtype=dtype, device=device), requires_grad=False)
        self.layers = nn.ModuleList([DopipelLayer(cfg, s, dtype, device) for s in cfg.layers])
        self.loop_in = nn.Parameter(torch.zeros((W, 2 * W), dtype=dtype, device=device), requires_grad=False)
        self.loop_step = nn.Parameter(torch.zeros((cfg.loop_times, W), dtype=torch.float32, device=device),
                                      requires_grad=False)
        self.final_norm = nn.Parameter(torch.ones(W, dtype=torch.float32, device=device), requires_grad=False)
        self.head = nn.Parameter(torch.zeros((cfg.vocab, W), dtype=dtype, device=device), requires_grad=False)
        self.runs = cfg.layer_runs()
        if seed is not None:
            self.load_weights(self.random_weights(seed))

    # ------------------------------------------------------------------ caches
    def cache_spec(self) -> List[Dict[str, Tuple[int, ...]]]:
        """Per layer run: the shapes of its caches for one block of one token and one slot."""
        return [{k: v[0] for k, v in self.layers[i].cache_shapes(self.cfg, 1, 1, 1).items()} for i, _ in self.runs]

    def allocate_caches(self, num_blocks: int, block_size: int, num_slots: int):
        dev = self.head.device
        return [{name: torch.zeros(shape, dtype=dt, device=dev)
                 for name, (shape, dt) in self.layers[i].cache_shapes(self.cfg, num_blocks, block_size,
                                                                      num_slots).items()}
                for i, _ in self.runs]

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, caches, batch: SequenceBatch,
                tap=None) -> torch.Tensor:
        """Returns the fp32 residual stream [T, width] after the last layer.  tap(run, x) is
        called after every layer run (tests, layer-by-layer comparison)."""
        cfg = self.cfg
        x = torch.empty((input_ids.numel(), cfg.width), dtype=torch.float32, device=self.head.device)
        ops.embed_positions(x, self.embed.data, input_ids, positions, None)
        x0 = x.clone() if cfg.loops else None
        pending: Optional[Pending] = None
        for run, (i, opens) in enumerate(self.runs):
            add_row = None
            if opens is not None:
                _apply(x, pending, None, None, None, cfg.eps)
                pending = None
                both = torch.empty((x.shape[0], 2 * cfg.width), dtype=self.dtype, device=x.device)
                ops.concat_cast(both, x, x0)
                x = mm_f32(both, self.loop_in.data)
                add_row = self.loop_step.data[opens]
            pending = self.layers[i](x, batch, caches[run], pending, add_row)
            if tap is not None:
                _apply(x, pending, None, None, None, cfg.eps)
                pending = None
                tap(run, x)
        _apply(x, pending, None, None, None, cfg.eps)
        return x

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """hidden: the rows of the stream whose logits are wanted -> fp32 [n, vocab]."""
        x = hidden.contiguous()
        h = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        ops.residual_norms(x, out=h, pre_weight=self.final_norm.data, eps=self.cfg.eps)
        return mm_f32(h, self.head.data)

    # ------------------------------------------------------------------ weights
    def tensor_shapes(self) -> Dict[str, Tuple[int, ...]]:
        cfg = self.cfg
        t = {"embed": (cfg.vocab, cfg.width), "head": (cfg.vocab, cfg.width), "final.norm": (cfg.width, )}
        if cfg.loops:
            t["loop.in"], t["loop.step"] = (cfg.width, 2 * cfg.width), (cfg.loop_times, cfg.width)
        for i, layer in enumerate(self.layers):
            t.update({f"l{i}.{k}": v for k, v in layer.tensor_shapes(cfg).items()})
        return t

    def load_weights(self, tensors: Dict[str, torch.Tensor]) -> int:
        cfg, dev = self.cfg, self.head.device
        used = 0
        for i, layer in enumerate(self.layers):
            prefix = f"l{i}."
            mine = {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}
            layer.set_weights(mine, cfg)
            used += len(layer.tensor_shapes(cfg))
        for name, shape in (("embed", (cfg.vocab, cfg.width)), ("head", (cfg.vocab, cfg.width)),
                            ("final.norm", (cfg.width, ))):
            if tuple(tensors[name].shape) != shape:
                raise ValueError(f"{name}: shape {tuple(tensors[name].shape)}, expected {shape}")
        self.embed.data = tensors["embed"].to(self.dtype).to(dev).contiguous()
        self.head.data = tensors["head"].to(self.dtype).to(dev).contiguous()
        self.final_norm.data = tensors["final.norm"].float().to(dev).contiguous()
        used += 3
        if cfg.loops:
            for name, shape in (("loop.in", (cfg.width, 2 * cfg.width)), ("loop.step", (cfg.loop_times, cfg.width))):
                if tuple(tensors[name].shape) != shape:
                    raise ValueError(f"{name}: shape {tuple(tensors[name].shape)}, expected {shape}")
            self.loop_in.data = tensors["loop.in"].to(self.dtype).to(dev).contiguous()
            self.loop_step.data = tensors["loop.step"].float().to(dev).contiguous()
            used += 2
        return used

    def random_weights(self, seed: int) -> Dict[str, torch.Tensor]:
        """Tensors of every checkpoint name: projections ~ N(0, 1 / fan_in), norms and layer scales
        near 1 and 1/2, small biases."""
        g = torch.Generator().manual_seed(seed)
        out = {}
        for name, shape in self.tensor_shapes().items():
            last = name.rsplit(".", 1)[-1]
            if len(shape) == 1 or last in ("step", "canon1"):
                base = 1.0 if "norm" in name else (0.5 if last in ("ls1", "ls2") else 0.0)
                t = base + 0.1 * torch.randn(shape, generator=g)
            elif name == "embed":
                t = torch.randn(shape, generator=g)
            else:
                t = torch.randn(shape, generator=g) * shape[-1]**-0.5
            out[name] = t.to(torch.bfloat16)
        return out
