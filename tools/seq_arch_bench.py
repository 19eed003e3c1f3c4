"""Prefill and decode throughput of the Lusadra stack beside the Llama stack at equal size, and
each of its kernels beside the like kernel of the Llama stack against its roofline.

Run through `python bench.py --arch lusadra [--arch-size 2k|4k]` (one GPU, random weights, bf16).
Prints one JSON line.  `end_to_end`: tokens/s of a prompt step (one sequence of --arch-prompt
tokens) and of a decode step (--arch-batch sequences at --arch-context tokens) of four layers plus
logits, both stacks.  `kernels`: microseconds per launch, the time its algorithmic bytes or
arithmetic would take at the part's peaks, and the ratio (1.0 = on the roofline).
"""
import json
import time

import torch

HBM = 8.0e12          # B/s
MFMA_BF16 = 2.5e15    # dense bf16 flop/s
FMA_F32 = 157.3e12    # vector fp32 flop/s


def timed(fn, iters=20, warm=3):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e-3 / iters


SIZES = {
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, window=1024, r_heads=16, r_dim=64, r_vdim=128, ff=5632),
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, window=1024, r_heads=32, r_dim=64, r_vdim=128, ff=11008),
}


def lusadra_config(s, layers, vocab):
    layer = {"type": "parallel",
             "mixer": {"left": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["dim"],
                                "mask": {"size": s["window"]}, "q_temp": {"coef": 0.25, "every": 512},
                                "scale": s["dim"]**-0.5},
                       "right": {"heads": s["r_heads"], "dim": s["r_dim"], "vdim": s["r_vdim"], "tau": 8.0},
                       "left_scale": 0.5, "right_scale": 0.5},
             "mlp": {"kind": "dense", "ff": s["ff"]}}
    return {"architecture": "Lusadra", "vocab": vocab, "width": s["width"], "norm": {"eps": 1e-5},
            "layers": [layer] * layers, "loop": {"start": 0, "stop": 0, "times": 1}}


def record(out, name, seconds, nbytes=0.0, flops=0.0, peak=MFMA_BF16, note=""):
    roof = max(nbytes / HBM, flops / peak)
    out[name] = {"us": round(seconds * 1e6, 2), "roofline_us": round(roof * 1e6, 2),
                 "of_roofline": round(roof / seconds, 4), "bound": "hbm" if nbytes / HBM >= flops / peak else "flops"}
    if note:
        out[name]["note"] = note


def run(args):
    from vllm_legacy_amd import _custom_ops as cops
    from vllm_legacy_amd import _seq_ops as sops
    from vllm_legacy_amd.attention.backends.gfx950_paged import Gfx950PagedAttentionMetadata
    from vllm_legacy_amd.attention.batch import SequenceBatch
    from vllm_legacy_amd.attention.ops.paged_attn import PagedAttention
    from vllm_legacy_amd.model.llama_decode import LlamaConfig, LlamaDecodeModel
    from vllm_legacy_amd.model.lusadra import LusadraConfig, LusadraForCausalLM

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    dt = torch.bfloat16
    s = SIZES[args.arch_size]
    layers, vocab, BS = 4, 32000, 16
    P, B, C = args.arch_prompt, args.arch_batch, args.arch_context
    e2e, kern = {}, {}
    g = torch.Generator(device=dev).manual_seed(0)

    # ------------------------------------------------------------------ Lusadra, whole steps
    model = LusadraForCausalLM(LusadraConfig.from_dict(lusadra_config(s, layers, vocab)), dt, dev, seed=0)
    nblk = max(B * (C // BS + 1), P // BS + 1) + 4
    caches = model.allocate_caches(nblk, BS, B)
    for keys, state in caches:
        keys.normal_(0, 1.0, generator=g)
        state.normal_(0, 0.1, generator=g)
    per = C // BS + 1
    tables = torch.randperm(nblk - 4, generator=g, device=dev)[:B * per].view(B, per).tolist()
    pre = SequenceBatch.build([P], [0], [list(range(P // BS + 1))], [0], BS, dev)
    dec = SequenceBatch.build([1] * B, [C - 1] * B, tables, list(range(B)), BS, dev)
    ids_p = torch.randint(0, vocab, (P, ), generator=g, device=dev)
    ids_d = torch.randint(0, vocab, (B, ), generator=g, device=dev)

    @torch.inference_mode()
    def lus_prefill():
        x = model(ids_p, pre.positions, caches, pre)
        return model.compute_logits(x[-1:])

    @torch.inference_mode()
    def lus_decode():
        x = model(ids_d, dec.positions, caches, dec)
        return model.compute_logits(x)

    t = timed(lus_prefill, 8, 6)
    e2e["lusadra_prefill_tokens_per_s"] = round(P / t, 1)
    t = timed(lus_decode, 20, 3)
    e2e["lusadra_decode_tokens_per_s"] = round(B / t, 1)
    e2e["lusadra_decode_ms_per_step"] = round(t * 1e3, 3)

    # ------------------------------------------------------------------ Lusadra, kernel by kernel
    H, G, D, W = s["heads"], s["kv_heads"], s["dim"], s["window"]
    Hr, Dr, Vr, ff, width = s["r_heads"], s["r_dim"], s["r_vdim"], s["ff"], s["width"]
    lay = model.layers[0]
    keys, state = caches[0]
    with torch.inference_mode():
        for tag, batch, T in (("prefill", pre, P), ("decode", dec, B)):
            q = torch.randn(T, H * D, device=dev, dtype=dt)
            k = torch.randn(T, G * D, device=dev, dtype=dt)
            gate = torch.randn(T, H * D, device=dev, dtype=dt)
            out = torch.empty_like(q)
            if tag == "prefill":     # runs of rows: the tiled kernel, as the layer picks it
                sec = timed(lambda: sops.window_attention_tiles(out, q, gate, keys, batch.block_tables,
                                                                batch.query_start_loc, batch.context_lens,
                                                                batch.max_query_len, lay.attn.slopes, H, W, D**-0.5,
                                                                0.25, 512.0, 0.5), 5)
            else:
                sec = timed(lambda: sops.window_attention(out, q, gate, keys, batch.block_tables, batch.token_seq,
                                                          batch.positions, lay.attn.slopes, H, W, D**-0.5, 0.25, 512.0,
                                                          0.5), 20)
            if tag == "prefill":
                pairs = sum(min(W, p + 1) for p in range(T))
                record(kern, "lusadra.window_attention.prefill", sec, flops=4.0 * pairs * H * D,
                       nbytes=2.0 * T * (2 * H + G) * D * 2)
            else:
                record(kern, "lusadra.window_attention.decode", sec, nbytes=2.0 * B * G * min(W, C) * D + 3 * 2.0 * B * H * D)
            sec = timed(lambda: sops.key_cache_write(keys, k, batch.slot_mapping))
            record(kern, f"lusadra.key_cache_write.{tag}", sec, nbytes=2 * 2.0 * T * G * D)
            qr = torch.randn(T, Hr * Dr, device=dev, dtype=dt)
            kr = torch.randn(T, Hr * Dr, device=dev, dtype=dt)
            vr = torch.randn(T, Hr * Vr, device=dev, dtype=dt)
            ld = -torch.rand(T, Hr * Dr, device=dev) * 0.1
            o = torch.empty(T, Hr, Vr, device=dev)
            sec = timed(lambda: sops.gla_scan(o, qr, kr, vr, ld, state, batch.query_start_loc, batch.context_lens,
                                              batch.state_slots, Dr**-0.5, batch.max_query_len),
                        5 if tag == "prefill" else 20)
            nseq = batch.num_seqs
            record(kern, f"lusadra.gla_scan.{tag}", sec, peak=FMA_F32, flops=4.0 * T * Hr * Dr * Vr,
                   nbytes=T * (2.0 * (2 * Hr * Dr + Hr * Vr) + 4.0 * Hr * Dr + 4.0 * Hr * Vr) + 8.0 * nseq * Hr * Dr * Vr,
                   note="a recurrence: the walk over a sequence's tokens is serial")
            y = torch.randn(T, lay.rank, device=dev, dtype=dt)
            og2 = torch.empty(T, Hr * Vr, device=dev, dtype=dt)
            # the layer as the model calls it: log decays, the walk (long runs in pieces), norm + gate
            sec = timed(lambda: lay.recur(og2, qr, kr, vr, vr, y, lay.w_a2.data, lay.b_a2.data, lay.recur_norm.data,
                                          state, batch, 0.5), 5 if tag == "prefill" else 20)
            record(kern, f"lusadra.recurrent_layer.{tag}", sec, peak=FMA_F32, flops=4.0 * T * Hr * Dr * Vr,
                   nbytes=T * (2.0 * (2 * Hr * Dr + 3 * Hr * Vr) + 2.0 * lay.rank) + 8.0 * nseq * Hr * Dr * Vr,
                   note="log decays + walk + gated norm; runs of 512 rows and more are walked in pieces of 256")
            sec = timed(lambda: sops.gla_log_decay(ld, y, lay.w_a2.data, lay.b_a2.data, 1 / 8.0))
            record(kern, f"lusadra.gla_log_decay.{tag}", sec, nbytes=4.0 * T * Hr * Dr + 2.0 * T * lay.rank)
            og = torch.empty(T, Hr * Vr, device=dev, dtype=dt)
            sec = timed(lambda: sops.gated_head_rms_norm(og, o, lay.recur_norm.data, vr, 1e-5, 0.5))
            record(kern, f"lusadra.gated_head_rms_norm.{tag}", sec, nbytes=T * Hr * Vr * (4.0 + 2 + 2))
            z = torch.randn(T, ff, device=dev, dtype=dt)
            zo = torch.empty_like(z)
            sec = timed(lambda: sops.poly_norm(zo, z, lay.act.weight.data, 1e-5))
            record(kern, f"lusadra.poly_norm.{tag}", sec, nbytes=2 * 2.0 * T * ff)
            x = torch.randn(T, width, device=dev)
            h = torch.empty(T, width, device=dev, dtype=dt)
            sec = timed(lambda: sops.scalar_rms_norm(h, x, lay.norm1.weight.data.view(1), 1e-5))
            record(kern, f"lusadra.scalar_rms_norm.{tag}", sec, nbytes=T * width * (4.0 + 2))
            yb = torch.randn(T, width, device=dev)
            sec = timed(lambda: sops.residual_add(x, yb))
            record(kern, f"lusadra.residual_add.{tag}", sec, nbytes=T * width * 12.0)
    del model, caches
    torch.cuda.empty_cache()

    # ------------------------------------------------------------------ Llama stack at equal size
    cfg = LlamaConfig(hidden_size=width, intermediate_size=ff, num_hidden_layers=layers, num_attention_heads=H,
                      num_key_value_heads=G, head_dim=D, vocab_size=vocab, max_position_embeddings=max(C, P) + 16)
    llama = LlamaDecodeModel(cfg, quant="none", kv_cache_dtype="auto", device=dev, dtype=dt)
    nblk = max(B * (C // BS), P // BS + 1) + 8
    shape = llama.kv_cache_shape(nblk, BS)
    kv = [torch.randn(shape, device=dev, dtype=dt) * 0.1 for _ in range(layers)]
    bt = torch.randperm(nblk, generator=g, device=dev)[:B * (C // BS)].to(torch.int32).view(B, C // BS).contiguous()
    seq_lens = torch.full((B, ), C, dtype=torch.int32, device=dev)
    pos_d = torch.full((B, ), C - 1, dtype=torch.int64, device=dev)
    slots_d = bt[:, (C - 1) // BS].to(torch.int64) * BS + (C - 1) % BS
    meta_d = Gfx950PagedAttentionMetadata(
        num_prefills=0, num_prefill_tokens=0, num_decode_tokens=B, slot_mapping=slots_d, seq_lens=None,
        seq_lens_tensor=seq_lens, max_query_len=None, max_prefill_seq_len=0, max_decode_seq_len=C,
        query_start_loc=None, seq_start_loc=None, use_cuda_graph=False, context_lens_tensor=None, block_tables=bt)
    pos_p = torch.arange(P, dtype=torch.int64, device=dev)
    cu = torch.tensor([0, P], dtype=torch.int32, device=dev)
    meta_p = Gfx950PagedAttentionMetadata(
        num_prefills=1, num_prefill_tokens=P, num_decode_tokens=0, slot_mapping=pos_p.clone(), seq_lens=[P],
        seq_lens_tensor=torch.tensor([P], dtype=torch.int32, device=dev), max_query_len=P, max_prefill_seq_len=P,
        max_decode_seq_len=0, query_start_loc=cu, seq_start_loc=cu, use_cuda_graph=False,
        context_lens_tensor=torch.zeros(1, dtype=torch.int32, device=dev),
        block_tables=torch.empty((1, 0), dtype=torch.int32, device=dev))

    @torch.inference_mode()
    def llama_prefill():
        hdn = llama(ids_p, pos_p, kv, meta_p)
        return llama.compute_logits(hdn[-1:])

    @torch.inference_mode()
    def llama_decode():
        hdn = llama(ids_d, pos_d, kv, meta_d)
        return llama.compute_logits(hdn)

    t = timed(llama_prefill, 8, 6)
    e2e["llama_prefill_tokens_per_s"] = round(P / t, 1)
    t = timed(llama_decode, 20, 3)
    e2e["llama_decode_tokens_per_s"] = round(B / t, 1)
    e2e["llama_decode_ms_per_step"] = round(t * 1e3, 3)

    with torch.inference_mode():
        kc, vc = PagedAttention.split_kv_cache(kv[0], G, D)
        q = torch.randn(B, H, D, device=dev, dtype=dt)
        sec = timed(lambda: PagedAttention.forward_decode(q, kc, vc, bt, seq_lens, C, "auto", G, D**-0.5, None, 1.0))
        record(kern, "llama.paged_attention.decode", sec, nbytes=2 * 2.0 * B * G * C * D + 2 * 2.0 * B * H * D)
        qp = torch.randn(P, H, D, device=dev, dtype=dt)
        kp = torch.randn(P, G, D, device=dev, dtype=dt)
        vp = torch.randn(P, G, D, device=dev, dtype=dt)
        op = torch.empty_like(qp)
        sec = timed(lambda: cops.prefill_attention(op, qp, kp, vp, cu, P, D**-0.5, None), 5)
        record(kern, "llama.prefill_attention.prefill", sec, flops=4.0 * (P * (P + 1) / 2) * H * D,
               nbytes=2.0 * P * (2 * H + 2 * G) * D)
        for tag, T in (("prefill", P), ("decode", B)):
            x = torch.randn(T, width, device=dev, dtype=dt)
            res = torch.randn(T, width, device=dev, dtype=dt)
            w = torch.ones(width, device=dev, dtype=dt)
            sec = timed(lambda: cops.fused_add_rms_norm(x, res, w, 1e-5))
            record(kern, f"llama.fused_add_rms_norm.{tag}", sec, nbytes=T * width * 8.0)
            gu = torch.randn(T, 2 * ff, device=dev, dtype=dt)
            a = torch.empty(T, ff, device=dev, dtype=dt)
            sec = timed(lambda: cops.silu_and_mul(a, gu))
            record(kern, f"llama.silu_and_mul.{tag}", sec, nbytes=T * ff * 6.0)
            kk = torch.randn(T, G, D, device=dev, dtype=dt)
            vv = torch.randn(T, G, D, device=dev, dtype=dt)
            sl = slots_d if tag == "decode" else pos_p
            sec = timed(lambda: cops.reshape_and_cache(kk, vv, kc, vc, sl, "auto", 1.0))
            record(kern, f"llama.reshape_and_cache.{tag}", sec, nbytes=2 * 2 * 2.0 * T * G * D)

    print(json.dumps({"metric": "prefill and decode tokens/s, Lusadra beside Llama at equal size (4 layers, bf16, random weights)",
                      "size": args.arch_size, "shape": s, "prompt_tokens": P, "decode_batch": B, "decode_context": C,
                      "end_to_end": e2e, "kernels": kern, "peaks": {"hbm_Bps": HBM, "mfma_bf16": MFMA_BF16, "fma_f32": FMA_F32},
                      "time": time.strftime("%Y-%m-%d %H:%M:%S")}))
