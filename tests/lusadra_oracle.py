"""Slow reference of the Lusadra design in float64 on the CPU, one function per mechanism, written
from the equations and sharing no code with vllm_legacy_amd.  Also the helpers that make small
random models (config dict + tensors under their checkpoint names) and write them as a
checkpoint folder.

Notation: x[t] the stream at token t (position p_t), W y a linear map stored [out, in].
"""
import json
import math
import os
import struct

import torch

F = torch.float64


def rms_unit(u, eps):
    """u / sqrt(mean(u^2) + eps) over the last axis."""
    return u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps)


def sinusoid(positions, width):
    """pe[p, 2i] = sin(p w_i), pe[p, 2i+1] = cos(p w_i), w_i = 10000^(-2i/width); the angle is
    formed in float32 as the design computes positions and angles in 32 bits."""
    i2 = torch.arange(0, width, 2, dtype=torch.float32)
    w = torch.pow(torch.tensor(10000.0, dtype=torch.float32), -i2 / width)
    ang = (positions.to(torch.float32)[:, None] * w[None, :]).to(F)
    pe = torch.zeros(len(positions), width, dtype=F)
    pe[:, 0::2] = torch.sin(ang)
    pe[:, 1::2] = torch.cos(ang)[:, :pe[:, 1::2].shape[1]]
    return pe


def scalar_rms_norm(x, gain, eps):
    return rms_unit(x, eps) * gain


def poly_norm(z, coef, eps):
    a, b, c, e = [float(v) for v in coef]
    return a * rms_unit(z, eps) + b * rms_unit(z**2, eps) + c * rms_unit(z**3, eps) + e


def head_slopes(H):
    return [2.0**(-8.0 * (h + 1) / H) for h in range(H)]


def windowed_key_attention(q, k, positions, H, G, D, window, scale, temp_coef, temp_every, slopes):
    """q [n, H*D], k [n, G*D] of one sequence whose tokens sit at `positions` (consecutive);
    values are the keys.  Returns [n, H*D] before any gate."""
    n = q.shape[0]
    q, k = q.view(n, H, D), k.view(n, G, D)
    out = torch.zeros(n, H, D, dtype=F)
    for a in range(n):
        p = int(positions[a])
        temp = 1.0 + temp_coef * math.log(math.floor((p + 1) / temp_every) + 1.0) if temp_coef else 1.0
        for h in range(H):
            kk = k[:, h // (H // G)]
            js = [b for b in range(n) if 0 <= p - int(positions[b]) and (window <= 0 or p - int(positions[b]) < window)]
            s = torch.stack([(q[a, h] * temp) @ kk[b] * scale - slopes[h] * (p - int(positions[b])) for b in js])
            w = torch.softmax(s, 0)
            out[a, h] = (w[:, None] * kk[js]).sum(0)
    return out.reshape(n, H * D)


def log_decay(y, w2, bias, tau):
    """ln(sigmoid(z)^(1/tau)), z = W2 y + b."""
    z = y @ w2.T + bias
    return torch.nn.functional.logsigmoid(z) / tau


def gated_linear_attention(q, k, v, ln_a, H, D, V, state=None):
    """S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head; q already scaled.
    Returns (o [n, H, V], final state [H, D, V])."""
    n = q.shape[0]
    q, k, v, a = q.view(n, H, D), k.view(n, H, D), v.view(n, H, V), torch.exp(ln_a).view(n, H, D)
    S = torch.zeros(H, D, V, dtype=F) if state is None else state.clone()
    o = torch.zeros(n, H, V, dtype=F)
    for t in range(n):
        S = a[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return o, S


def gated_head_norm(o, weight, gate, eps, scale=1.0):
    """o [n, H, V] -> [n, H*V]: unit RMS per head times weight, times silu(gate)."""
    n = o.shape[0]
    y = (rms_unit(o, eps) * weight).reshape(n, -1)
    return y * gate * torch.sigmoid(gate) * scale


# ------------------------------------------------------------------------------------ model


def layer_forward(cfg, W, i, x, positions):
    L, eps = cfg["layers"][i], cfg["norm"]["eps"]
    m, p = L["mixer"], f"l{i}."
    h = scalar_rms_norm(x, W[p + "norm1"], eps)
    le, ri = m["left"], m["right"]
    H, G, D = le["heads"], le["kv_heads"], le["dim"]
    att = windowed_key_attention(h @ W[p + "mix.left.q"].T, h @ W[p + "mix.left.k"].T, positions, H, G, D,
                                 le["mask"]["size"], le["scale"], le["q_temp"]["coef"], le["q_temp"]["every"],
                                 head_slopes(H))
    left = (att * torch.sigmoid(h @ W[p + "mix.left.g"].T)) @ W[p + "mix.left.o"].T
    Hr, Dr, Vr = ri["heads"], ri["dim"], ri["vdim"]
    ln_a = log_decay(h @ W[p + "mix.right.a1"].T, W[p + "mix.right.a2"], W[p + "mix.right.a2.b"], ri["tau"])
    o, _ = gated_linear_attention((h @ W[p + "mix.right.q"].T) * Dr**-0.5, h @ W[p + "mix.right.k"].T,
                                  h @ W[p + "mix.right.v"].T, ln_a, Hr, Dr, Vr)
    right = gated_head_norm(o, W[p + "mix.right.norm"], h @ W[p + "mix.right.g"].T, eps) @ W[p + "mix.right.o"].T
    y = m["left_scale"] * left + m["right_scale"] * right
    if L["mlp"] is not None:
        y = y + poly_norm(h @ W[p + "mlp.up"].T, W[p + "mlp.act"], eps) @ W[p + "mlp.down"].T
    return x + y


def model_forward(cfg, W, tokens, taps=None):
    """Logits [n, vocab] of one whole sequence (float64).  W: tensors by checkpoint name."""
    W = {k: v.to(F) for k, v in W.items()}
    n = len(tokens)
    positions = torch.arange(n)
    x = W["embed"][torch.as_tensor(tokens)] + sinusoid(positions, cfg["width"])
    x0 = x.clone()
    lp = cfg["loop"]
    order = [(i, None) for i in range(lp["start"])]
    for t in range(lp["times"]):
        order += [(i, t if i == lp["start"] else None) for i in range(lp["start"], lp["stop"])]
    order += [(i, None) for i in range(lp["stop"], len(cfg["layers"]))]
    for i, t in order:
        if t is not None:
            if t > 0:
                x = x + x0
            x = x + W["loop.step"][t]
        x = layer_forward(cfg, W, i, x, positions)
        if taps is not None:
            taps.append(x.clone())
    return scalar_rms_norm(x, W["final.norm"], cfg["norm"]["eps"]) @ W["head"].T


# ------------------------------------------------------------------------------------ models


def make_config(vocab=97, width=64, layers=2, heads=2, kv_heads=1, dim=16, window=5, temp_coef=0.25,
                temp_every=4, r_heads=2, r_dim=8, r_vdim=16, tau=4.0, ff=48, loop=(0, 0, 1), eps=1e-5,
                left_scale=0.7, right_scale=1.1, scale=None, per_layer=None):
    """per_layer: optional list of dicts overriding the keyword sizes for each layer (ff None: no
    feed-forward)."""
    out = []
    for i in range(layers):
        o = dict(heads=heads, kv_heads=kv_heads, dim=dim, window=window, r_heads=r_heads, r_dim=r_dim,
                 r_vdim=r_vdim, ff=ff, tau=tau)
        if per_layer:
            o.update(per_layer[i])
        out.append({
            "type": "parallel",
            "mixer": {
                "left": {"heads": o["heads"], "kv_heads": o["kv_heads"], "dim": o["dim"], "vdim": o["dim"],
                         "mask": {"size": o["window"]}, "q_temp": {"coef": temp_coef, "every": temp_every},
                         "scale": scale if scale is not None else o["dim"]**-0.5},
                "right": {"heads": o["r_heads"], "dim": o["r_dim"], "vdim": o["r_vdim"], "tau": o["tau"]},
                "left_scale": left_scale, "right_scale": right_scale},
            "mlp": None if o["ff"] is None else {"kind": "dense", "ff": o["ff"]}})
    return {"architecture": "Lusadra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": out,
            "loop": {"start": loop[0], "stop": loop[1], "times": loop[2]}}


def make_weights(cfg, seed=0, rank=4, dtype=torch.bfloat16):
    """Random tensors under the checkpoint names, rounded to `dtype` (so the framework and the
    oracle start from identical values)."""
    g = torch.Generator().manual_seed(seed)
    W, width = {}, cfg["width"]

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(shape or (1, ), generator=g) * std + mean).to(dtype)

    W["embed"] = rnd(cfg["vocab"], width)
    W["head"] = rnd(cfg["vocab"], width, std=width**-0.5)
    W["final.norm"] = rnd(std=0.1, mean=1.0).reshape(())
    W["loop.step"] = rnd(cfg["loop"]["times"], width, std=0.3)
    for i, L in enumerate(cfg["layers"]):
        p, le, ri = f"l{i}.", L["mixer"]["left"], L["mixer"]["right"]
        W[p + "norm1"] = rnd(std=0.1, mean=1.0).reshape(())
        s = width**-0.5
        W[p + "mix.left.q"] = rnd(le["heads"] * le["dim"], width, std=2 * s)
        W[p + "mix.left.k"] = rnd(le["kv_heads"] * le["dim"], width, std=2 * s)
        W[p + "mix.left.g"] = rnd(le["heads"] * le["dim"], width, std=s)
        W[p + "mix.left.o"] = rnd(width, le["heads"] * le["dim"], std=(le["heads"] * le["dim"])**-0.5)
        W[p + "mix.right.q"] = rnd(ri["heads"] * ri["dim"], width, std=s)
        W[p + "mix.right.k"] = rnd(ri["heads"] * ri["dim"], width, std=s)
        W[p + "mix.right.v"] = rnd(ri["heads"] * ri["vdim"], width, std=s)
        W[p + "mix.right.g"] = rnd(ri["heads"] * ri["vdim"], width, std=s)
        W[p + "mix.right.o"] = rnd(width, ri["heads"] * ri["vdim"], std=(ri["heads"] * ri["vdim"])**-0.5)
        W[p + "mix.right.norm"] = rnd(ri["vdim"], std=0.2, mean=1.0)
        W[p + "mix.right.a1"] = rnd(rank, width, std=s)
        W[p + "mix.right.a2"] = rnd(ri["heads"] * ri["dim"], rank, std=rank**-0.5)
        W[p + "mix.right.a2.b"] = rnd(ri["heads"] * ri["dim"], std=1.0, mean=2.0)
        if L["mlp"] is not None:
            W[p + "mlp.up"] = rnd(L["mlp"]["ff"], width, std=s)
            W[p + "mlp.down"] = rnd(width, L["mlp"]["ff"], std=L["mlp"]["ff"]**-0.5)
            W[p + "mlp.act"] = torch.tensor([0.5, 0.3, 0.2, 0.1]).to(dtype) + rnd(4, std=0.05)
    return W


_ST = {torch.bfloat16: "BF16", torch.float32: "F32", torch.float16: "F16", torch.int32: "I32"}


def write_checkpoint(folder, cfg, W):
    """config.json + model.safetensors (8-byte header length, JSON header, raw data)."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, at = {}, [], 0
    for name, t in W.items():
        t = t.contiguous()
        raw = t.view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes()
        header[name] = {"dtype": _ST[t.dtype], "shape": list(t.shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    h = json.dumps(header).encode()
    h += b" " * (-len(h) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(h)))
        f.write(h)
        for b in blobs:
            f.write(b)
    return folder


def logit_error(got, want):
    """Per row: rms over the vocabulary of the difference with its mean taken off, relative to
    the rms of the expected logits."""
    got, want = got.to(F), want.to(F)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    scale = (want - want.mean(-1, keepdim=True)).pow(2).mean().sqrt()
    return (d.pow(2).mean(-1).sqrt() / scale)
