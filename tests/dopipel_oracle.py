"""Slow reference of the Dopipel design in float64 on the CPU, one function per mechanism, written
from the equations and sharing no code with vllm_legacy_amd.  Also the helpers that make small
random models (config dict + tensors under their checkpoint names) and write them as a
checkpoint folder.

Notation: x[t] the stream at token t (position p_t, counted from 0 in its sequence), W y a linear
map stored [out, in].  Every function takes one whole sequence from its first token.
"""
import json
import math
import os
import struct

import torch

F = torch.float64


def rms_norm(u, w, eps):
    """u / sqrt(mean(u^2) + eps) * w over the last axis."""
    return u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps) * w


def input_convolution(h, w):
    """h [n, C], w [C, taps]: h_t + sum_j w[:, j] h_(t - taps + 1 + j), zeros before the start."""
    n, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def pair_angles(positions, pairs, base, span):
    """angle[p, i] = p * base^(-2 i / span), formed in float32 like positions and angles are."""
    i = torch.arange(pairs, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / span).to(torch.float32)
    return (positions.to(torch.float32)[:, None] * f[None, :]).to(F)


def rotate_pairs(u, angle, layout="interleaved"):
    """u [n, heads, 2 m]; pair i is (2i, 2i + 1) when interleaved, (i, i + m) in halves.  The pair
    (a, b) turns to (a cos - b sin, b cos + a sin)."""
    out = u.clone()
    m = angle.shape[1]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    if layout == "interleaved":
        a, b = u[..., 0:2 * m:2], u[..., 1:2 * m:2]
        out[..., 0:2 * m:2] = a * c - b * s
        out[..., 1:2 * m:2] = b * c + a * s
    else:
        a, b = u[..., :m], u[..., m:2 * m]
        out[..., :m] = a * c - b * s
        out[..., m:2 * m] = b * c + a * s
    return out


def attention_core(q, k, v, gate_logits, spec, window=0):
    """q [n, H, D], k [n, G, D], v [n, G, V] before any rotation, gate_logits [n, H] or None, of one
    sequence from its first token.  Returns [n, H, V] after the gate."""
    n = q.shape[0]
    H, G, V = spec["heads"], spec["kv_heads"], spec["vdim"]
    rot = spec["rot"]
    layout = rot.get("layout", "interleaved")
    pos = torch.arange(n)
    if rot["dims"]:
        ang = pair_angles(pos, rot["dims"] // 2, rot["base"], rot["dims"])
        q, k = rotate_pairs(q, ang, layout), rotate_pairs(k, ang, layout)
    vang = pair_angles(pos, V // 2, rot["base"], V)
    v = rotate_pairs(v, vang, layout)
    out = torch.zeros(n, H, V, dtype=F)
    for a in range(n):
        lo = max(0, a - window + 1) if window else 0
        for hh in range(H):
            g = hh // (H // G)
            s = (k[lo:a + 1, g] @ q[a, hh]) * spec["scale"]
            out[a, hh] = torch.softmax(s, 0) @ v[lo:a + 1, g]
    out = rotate_pairs(out, -vang, layout)
    if gate_logits is not None:
        out = out * torch.sigmoid(gate_logits)[:, :, None]
    return out


def rotary_attention(h, t, spec):
    """The attention mixer on its input h [n, width]; t: this layer's mixer tensors by short name."""
    n = h.shape[0]
    H, G, D, V = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    q = (h @ t["q"].T + t["q.b"]).view(n, H, D)
    k = (h @ t["k"].T + t["k.b"]).view(n, G, D)
    v = (h @ t["v"].T + t["v.b"]).view(n, G, V)
    out = attention_core(q, k, v, h @ t["g"].T, spec)
    return out.reshape(n, H * V) @ t["o"].T + t["o.b"]


def mingru_core(zp, up, gp):
    """Pre-activations [n, R] of one sequence from its first token -> gated outputs [n, R]."""
    z = torch.sigmoid(zp)
    cand = torch.where(up >= 0, up + 0.5, torch.sigmoid(up))
    S = torch.zeros(zp.shape[1], dtype=F)
    out = torch.zeros_like(zp)
    for i in range(zp.shape[0]):
        S = (1 - z[i]) * S + z[i] * cand[i]
        out[i] = S * gp[i] * torch.sigmoid(gp[i])
    return out


def mingru(h, t):
    """Gated recurrence whose gates read only the current token."""
    return mingru_core(h @ t["z"].T + t["z.b"], h @ t["x"].T + t["x.b"], h @ t["g"].T) @ t["o"].T


def dense_ff(h, t):
    return (torch.relu(h @ t["gate"].T) * (h @ t["up"].T)) @ t["down"].T


def expert(h, up, down):
    return (torch.relu(h @ up.T)**2) @ down.T


def route(h, t, top):
    """Returns per token the chosen experts and their weights."""
    s = torch.softmax(h @ t["router"].T, -1)
    choice = s + t["correction"]
    idx = torch.topk(choice, top, dim=-1).indices
    w = torch.gather(s, 1, idx)
    return idx, w / (w.sum(-1, keepdim=True) + 1e-20)


def moe_ff(h, t, mlp):
    E, ident, top = mlp["router"]["experts"], mlp["router"]["identity"], mlp["router"]["top"]
    idx, w = route(h, t, top)
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e, we in zip(idx[i].tolist(), w[i]):
            if e >= E:
                out[i] += we * h[i]
            else:
                out[i] += we * expert(h[i:i + 1], t[f"e{e}.up"], t[f"e{e}.down"])[0]
    if mlp.get("shared"):
        sg = torch.sigmoid(h @ t["shared.sg"].T)            # [n, 1]
        out = out + sg * expert(h, t["shared.up"], t["shared.down"])
    return out


def sub(W, prefix):
    return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}


def layer(x, i, cfg, W):
    spec, eps = cfg["layers"][i], cfg["norm"]["eps"]
    t = sub(W, f"l{i}.")
    h = rms_norm(x, t["norm1"], eps)
    if "canon1" in t:
        h = input_convolution(h, t["canon1"])
    if spec["type"] == "attention":
        y = rotary_attention(h, sub(t, "mix."), spec["mixer"])
    elif spec["type"] == "mingru":
        y = mingru(h, sub(t, "mix."))
    else:
        raise ValueError(spec["type"])
    x = x + rms_norm(y, t["norm1b"], eps) * t["ls1"]
    if spec.get("mlp") is not None:
        h = rms_norm(x, t["norm2"], eps)
        mlp = spec["mlp"]
        y = dense_ff(h, sub(t, "mlp.")) if mlp["kind"] == "dense" else moe_ff(h, sub(t, "mlp."), mlp)
        x = x + rms_norm(y, t["norm2b"], eps) * t["ls2"]
    return x


def forward(tokens, cfg, W, taps=None):
    """Logits [n, vocab] of one sequence; taps (a list) collects the stream after every layer run."""
    W = {k: (v.to(F) if v.is_floating_point() else v) for k, v in W.items()}
    x = W["embed"][torch.as_tensor(tokens)]
    x0 = x.clone()
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    n_layers = len(cfg["layers"])

    def run(i, x):
        x = layer(x, i, cfg, W)
        if taps is not None:
            taps.append(x.clone())
        return x

    for i in range(loop["start"]):
        x = run(i, x)
    if loop["stop"] > loop["start"]:
        for t in range(loop["times"]):
            x = torch.cat([x, x0], -1) @ W["loop.in"].T + W["loop.step"][t]
            for i in range(loop["start"], loop["stop"]):
                x = run(i, x)
    for i in range(loop["stop"], n_layers):
        x = run(i, x)
    return rms_norm(x, W["final.norm"], cfg["norm"]["eps"]) @ W["head"].T


# ------------------------------------------------------------------------------------------------
# small random models

def attention_layer(heads=4, kv_heads=2, dim=16, vdim=None, rot_dims=None, base=10000.0, scale=None,
                    mlp=None):
    vdim = dim if vdim is None else vdim
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                      "rot": {"base": base, "dims": dim if rot_dims is None else rot_dims},
                      "scale": dim**-0.5 if scale is None else scale},
            "mlp": mlp}


def mingru_layer(width=48, mlp=None):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": mlp}


def dense_mlp(ff=96):
    return {"kind": "dense", "ff": ff}


def moe_mlp(experts=6, identity=1, top=2, ff=24, shared_ff=32):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top}}
    if shared_ff:
        m["shared"] = {"ff": shared_ff}
    return m


def make_config(layers, vocab=97, width=64, taps=3, eps=1e-5, loop=None):
    cfg = {"architecture": "Dopipel", "vocab": vocab, "width": width, "canon": {"taps": taps},
           "norm": {"eps": eps}, "layers": layers}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg, seed=0, router_scale=4.0):
    g = torch.Generator().manual_seed(seed)
    Wd, V = cfg["width"], cfg["vocab"]

    def rnd(shape, std):
        return (torch.randn(shape, generator=g) * std).to(torch.bfloat16)

    def lin(out, inp, gain=1.0):
        return rnd((out, inp), gain * inp**-0.5)

    W = {"embed": rnd((V, Wd), 1.0), "head": lin(V, Wd), "final.norm": 1.0 + rnd((Wd, ), 0.1)}
    loop = cfg.get("loop")
    if loop:
        W["loop.in"] = lin(Wd, 2 * Wd, 1.4)
        W["loop.step"] = rnd((loop["times"], Wd), 0.3)
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        for nm in ("norm1", "norm2", "norm1b", "norm2b"):
            W[p + nm] = 1.0 + rnd((Wd, ), 0.1)
        W[p + "ls1"] = 0.5 + rnd((Wd, ), 0.1)
        W[p + "ls2"] = 0.5 + rnd((Wd, ), 0.1)
        W[p + "canon1"] = rnd((Wd, cfg["canon"]["taps"]), 0.3)
        m = spec["mixer"]
        if spec["type"] == "attention":
            H, G, D, Vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            W[p + "mix.q"], W[p + "mix.q.b"] = lin(H * D, Wd, 2.0), rnd((H * D, ), 0.3)
            W[p + "mix.k"], W[p + "mix.k.b"] = lin(G * D, Wd, 2.0), rnd((G * D, ), 0.3)
            W[p + "mix.v"], W[p + "mix.v.b"] = lin(G * Vd, Wd), rnd((G * Vd, ), 0.3)
            W[p + "mix.g"] = lin(H, Wd, 2.0)
            W[p + "mix.o"], W[p + "mix.o.b"] = lin(Wd, H * Vd), rnd((Wd, ), 0.3)
        else:
            R = m["width"]
            W[p + "mix.z"], W[p + "mix.z.b"] = lin(R, Wd, 2.0), rnd((R, ), 0.5)
            W[p + "mix.x"], W[p + "mix.x.b"] = lin(R, Wd, 2.0), rnd((R, ), 0.5)
            W[p + "mix.g"] = lin(R, Wd, 2.0)
            W[p + "mix.o"] = lin(Wd, R)
        mlp = spec.get("mlp")
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            W[p + "mlp.gate"], W[p + "mlp.up"] = lin(mlp["ff"], Wd, 1.5), lin(mlp["ff"], Wd, 1.5)
            W[p + "mlp.down"] = lin(Wd, mlp["ff"])
        else:
            r, ff = mlp["router"], mlp["expert"]["ff"]
            for e in range(r["experts"]):
                W[p + f"mlp.e{e}.up"], W[p + f"mlp.e{e}.down"] = lin(ff, Wd, 1.5), lin(Wd, ff)
            n = r["experts"] + r["identity"]
            W[p + "mlp.router"] = lin(n, Wd, router_scale)
            W[p + "mlp.correction"] = rnd((n, ), 0.05)
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                W[p + "mlp.shared.up"], W[p + "mlp.shared.down"] = lin(sf, Wd, 1.5), lin(Wd, sf)
                W[p + "mlp.shared.sg"] = lin(1, Wd, 2.0)
    return W


_ST = {torch.bfloat16: "BF16", torch.float32: "F32", torch.int32: "I32"}


def write_checkpoint(folder, cfg, W):
    """config.json + model.safetensors (8-byte length, JSON header, raw little-endian data)."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, at = {}, [], 0
    for name, t in W.items():
        t = t.contiguous()
        raw = t.view(torch.uint8).numpy().tobytes() if t.numel() else b""
        header[name] = {"dtype": _ST[t.dtype], "shape": list(t.shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)
    return folder


def spread(logits):
    """Root mean square of the logits around their mean over the vocabulary, averaged over rows."""
    c = logits - logits.mean(-1, keepdim=True)
    return float(torch.sqrt((c * c).mean(-1)).mean())


def row_errors(got, want):
    """Per row: rms over the vocabulary of the difference with its mean taken off."""
    d = got.to(F) - want.to(F)
    d = d - d.mean(-1, keepdim=True)
    return torch.sqrt((d * d).mean(-1))
