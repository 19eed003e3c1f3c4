"""Prefill and decode throughput of Dopipel stacks beside the Llama stack at equal size, and each
of Dopipel's kernels beside the like kernel of the closest existing model against its roofline.

Run through `python bench.py --arch dopipel [--arch-size 2k|4k]` (one GPU, random weights, bf16).
Prints one JSON line.  `end_to_end`: tokens/s of a prompt step (one sequence of --arch-prompt
tokens) and of a decode step (--arch-batch sequences at --arch-context tokens) of four layers plus
logits: Dopipel with attention layers and dense feed-forwards (the Llama stack's shape), Dopipel
with minGRU / attention layers and dense / mixture-of-experts feed-forwards, and the Llama stack.
`kernels`: microseconds per launch, the time its algorithmic bytes or arithmetic would take at the
part's peaks, and the ratio (1.0 = on the roofline).  The like kernels: Llama's prompt and paged
decode attention, cache write, fused add + norm and activation; Lusadra's recurrence walk.
"""
import json
import time

import torch

from tools.seq_arch_bench import FMA_F32, HBM, MFMA_BF16, record, timed

SIZES = {
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, ff=5632, gru=2048, experts=16, identity=1, top=2,
               expert_ff=1408, shared_ff=1408, taps=4),
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, ff=11008, gru=4096, experts=32, identity=2, top=4,
               expert_ff=1408, shared_ff=2816, taps=4),
}


def dopipel_config(s, kinds, vocab):
    """kinds: per layer (mixer, feed-forward) out of attention | mingru and dense | moe."""
    attn = {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["dim"],
            "rot": {"base": 10000.0, "dims": s["dim"]}, "scale": s["dim"]**-0.5}
    dense = {"kind": "dense", "ff": s["ff"]}
    moe = {"kind": "moe", "expert": {"ff": s["expert_ff"]}, "shared": {"ff": s["shared_ff"]},
           "router": {"experts": s["experts"], "identity": s["identity"], "top": s["top"]}}
    layers = [{"type": m, "mixer": attn if m == "attention" else {"width": s["gru"]}, "mlp": dense if f == "dense" else moe}
              for m, f in kinds]
    return {"architecture": "Dopipel", "vocab": vocab, "width": s["width"], "norm": {"eps": 1e-5},
            "canon": {"taps": s["taps"]}, "layers": layers}


def run(args):
    from vllm_legacy_amd import _custom_ops as cops
    from vllm_legacy_amd import _seq_ops as sops
    from vllm_legacy_amd.attention.backends.gfx950_paged import Gfx950PagedAttentionMetadata
    from vllm_legacy_amd.attention.batch import SequenceBatch
    from vllm_legacy_amd.attention.ops.paged_attn import PagedAttention
    from vllm_legacy_amd.model.dopipel import DopipelConfig, DopipelForCausalLM
    from vllm_legacy_amd.model.llama_decode import LlamaConfig, LlamaDecodeModel

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    dt = torch.bfloat16
    s = SIZES[args.arch_size]
    layers, vocab, BS = 4, 32000, 16
    P, B, C = args.arch_prompt, args.arch_batch, args.arch_context
    e2e, kern = {}, {}
    g = torch.Generator(device=dev).manual_seed(0)
    nblk = max(B * (C // BS + 1), P // BS + 1) + 4
    per = C // BS + 1
    tables = torch.randperm(nblk - 4, generator=g, device=dev)[:B * per].view(B, per).tolist()
    pre = SequenceBatch.build([P], [0], [list(range(P // BS + 1))], [0], BS, dev)
    dec = SequenceBatch.build([1] * B, [C - 1] * B, tables, list(range(B)), BS, dev)
    ids_p = torch.randint(0, vocab, (P, ), generator=g, device=dev)
    ids_d = torch.randint(0, vocab, (B, ), generator=g, device=dev)

    stacks = {"dopipel_attention_dense": [("attention", "dense")] * 4,
              "dopipel_mixed": [("mingru", "dense"), ("attention", "moe"), ("attention", "dense"), ("mingru", "moe")]}
    model = caches = None
    for name, kinds in stacks.items():
        del model, caches
        torch.cuda.empty_cache()
        model = DopipelForCausalLM(DopipelConfig.from_dict(dopipel_config(s, kinds, vocab)), dt, dev, seed=0)
        caches = model.allocate_caches(nblk, BS, B)
        for c in caches:
            for k, t in c.items():
                t.normal_(0, 1.0 if k in ("keys", "values") else 0.1, generator=g)

        @torch.inference_mode()
        def prefill():
            x = model(ids_p, pre.positions, caches, pre)
            return model.compute_logits(x[-1:])

        @torch.inference_mode()
        def decode():
            x = model(ids_d, dec.positions, caches, dec)
            return model.compute_logits(x)

        t = timed(prefill, 8, 6)
        e2e[f"{name}_prefill_tokens_per_s"] = round(P / t, 1)
        t = timed(decode, 20, 3)
        e2e[f"{name}_decode_tokens_per_s"] = round(B / t, 1)
        e2e[f"{name}_decode_ms_per_step"] = round(t * 1e3, 3)

    # ------------------------------------------------------------------ kernel by kernel (the mixed stack)
    H, G, D, width, ff, R = s["heads"], s["kv_heads"], s["dim"], s["width"], s["ff"], s["gru"]
    attn = model.layers[1].attn
    keys, values, conv_state = caches[1]["keys"], caches[1]["values"], caches[1]["conv"]
    gru_state = caches[0]["state"]
    moe = model.layers[1].experts
    E, top, eff = s["experts"], s["top"], s["expert_ff"]
    with torch.inference_mode():
        for tag, batch, T in (("prefill", pre, P), ("decode", dec, B)):
            it = 5 if tag == "prefill" else 20
            q = torch.randn(T, H * D, device=dev, dtype=dt)
            k = torch.randn(T, G * D, device=dev, dtype=dt)
            v = torch.randn(T, G * D, device=dev, dtype=dt)
            gate = torch.randn(T, H, device=dev, dtype=dt)
            out = torch.empty_like(q)
            if tag == "prefill":
                sec = timed(lambda: sops.kv_attention_tiles(out, q, gate, keys, values, batch.block_tables,
                                                            batch.query_start_loc, batch.context_lens,
                                                            batch.max_query_len, attn.value_inv_freq, True, H, 0,
                                                            D**-0.5), it)
                record(kern, "dopipel.kv_attention.prefill", sec, flops=4.0 * (T * (T + 1) / 2) * H * D,
                       nbytes=2.0 * T * (2 * H + 2 * G) * D)
            else:
                sec = timed(lambda: sops.kv_attention(out, q, gate, keys, values, batch.block_tables, batch.token_seq,
                                                      batch.positions, attn.value_inv_freq, True, H, 0, D**-0.5), it)
                record(kern, "dopipel.kv_attention.decode", sec, nbytes=2 * 2.0 * B * G * C * D + 2 * 2.0 * B * H * D)
            sec = timed(lambda: sops.rotary_kv_write(q, k, v, keys, values, batch.positions, batch.slot_mapping,
                                                     attn.inv_freq, attn.value_inv_freq, H, D, True), it)
            record(kern, f"dopipel.rotary_kv_write.{tag}", sec, nbytes=2.0 * T * (2 * H + 4 * G) * D,
                   note="rotates the queries in place and writes rotated keys and values")
            x = torch.randn(T, width, device=dev)
            y = torch.randn(T, width, device=dev)
            h = torch.empty(T, width, device=dev, dtype=dt)
            w = torch.ones(width, device=dev)
            sec = timed(lambda: sops.residual_norms(x, y, None, w, w, None, h, w, 1e-5), it)
            record(kern, f"dopipel.residual_norms.{tag}", sec, nbytes=T * width * (4.0 + 4 + 4 + 2),
                   note="norm of the sublayer's result, layer scale, fp32 residual update and the next norm")
            h32 = torch.randn(T, width, device=dev)
            cw = torch.randn(width, s["taps"], device=dev)
            sec = timed(lambda: sops.causal_conv(h, h32, cw, conv_state, batch.query_start_loc, batch.context_lens,
                                                 batch.state_slots, batch.token_seq), it)
            record(kern, f"dopipel.causal_conv.{tag}", sec,
                   nbytes=T * width * (4.0 + 2) + batch.num_seqs * (s["taps"] - 1) * width * 8.0)
            zp, up, gp = (torch.randn(T, R, device=dev, dtype=dt) for _ in range(3))
            og = torch.empty(T, R, device=dev, dtype=dt)
            sec = timed(lambda: sops.mingru_scan(og, zp, up, gp, gru_state, batch.query_start_loc, batch.context_lens,
                                                 batch.state_slots, batch.max_query_len), it)
            record(kern, f"dopipel.mingru_scan.{tag}", sec, nbytes=T * R * 2.0 * 4 + batch.num_seqs * R * 8.0,
                   note="gates, candidate, walk and output gate in one pass; long runs are walked in pieces")
            gu = torch.randn(T, 2 * ff, device=dev, dtype=dt)
            a = torch.empty(T, ff, device=dev, dtype=dt)
            sec = timed(lambda: sops.gated_act(a, gu[:, :ff], gu[:, ff:], "relu"), it)
            record(kern, f"dopipel.gated_act.{tag}", sec, nbytes=T * ff * 6.0)
            hh = torch.randn(T, width, device=dev, dtype=dt)
            def route():        # as the layer routes: many tokens take their logits from one fp32 product
                logits = torch.mm(hh.float(), moe.router_rows().t()) if T >= moe.ROUTE_PRODUCT_MIN_TOKENS else None
                return sops.moe_route(hh, moe.router.data, moe.correction.data, moe.shared_gate.data, top, logits)

            sec = timed(route, it)
            record(kern, f"dopipel.moe_route.{tag}", sec, nbytes=T * width * 2.0 + (E + s["identity"] + 1) * width * 4.0,
                   note="prompt: cast + fp32 product + choice kernel; decode: one kernel")
            experts, weights, sg = sops.moe_route(hh, moe.router.data, moe.correction.data, moe.shared_gate.data, top)
            sec = timed(lambda: sops.moe_plan(experts, E), it)
            record(kern, f"dopipel.moe_plan.{tag}", sec, nbytes=T * top * 12.0, note="one workgroup")
            pair_row, row_token, tile_expert = sops.moe_plan(experts, E)
            rows = row_token.numel()
            routed = int((experts < E).sum())
            u = torch.empty(rows, eff, device=dev, dtype=dt)
            sec = timed(lambda: sops.grouped_linear(u, hh, row_token, moe.w_up.data, tile_expert, "relu2"), it)
            used = min(E, routed)
            record(kern, f"dopipel.grouped_linear_up.{tag}", sec, flops=2.0 * routed * width * eff,
                   nbytes=2.0 * (used * eff * width + routed * (width + eff)))
            yy = torch.empty(rows, width, device=dev)
            sec = timed(lambda: sops.grouped_linear(yy, u, None, moe.w_down.data, tile_expert), it)
            record(kern, f"dopipel.grouped_linear_down.{tag}", sec, flops=2.0 * routed * width * eff,
                   nbytes=2.0 * (used * eff * width + routed * eff) + 4.0 * routed * width)
            sy = torch.randn(T, width, device=dev)
            oo = torch.empty(T, width, device=dev)
            sec = timed(lambda: sops.moe_combine(oo, yy, pair_row, weights, hh, sy, sg), it)
            record(kern, f"dopipel.moe_combine.{tag}", sec, nbytes=T * width * (4.0 * top + 2 + 4 + 4))
    del model, caches
    torch.cuda.empty_cache()

    # ------------------------------------------------------------------ Lusadra's walk (the like recurrence)
    with torch.inference_mode():
        Hr, Dr, Vr = H, 64, 128
        state = torch.randn(B + 64, Hr, Dr, Vr, device=dev) * 0.1
        for tag, batch, T in (("prefill", pre, P), ("decode", dec, B)):
            qr = torch.randn(T, Hr * Dr, device=dev, dtype=dt)
            kr = torch.randn(T, Hr * Dr, device=dev, dtype=dt)
            vr = torch.randn(T, Hr * Vr, device=dev, dtype=dt)
            ld = -torch.rand(T, Hr * Dr, device=dev) * 0.1
            o = torch.empty(T, Hr, Vr, device=dev)
            sec = timed(lambda: sops.gla_scan(o, qr, kr, vr, ld, state, batch.query_start_loc, batch.context_lens,
                                              batch.state_slots, Dr**-0.5, batch.max_query_len), 5 if tag == "prefill" else 20)
            record(kern, f"lusadra.gla_scan.{tag}", sec, peak=FMA_F32, flops=4.0 * T * Hr * Dr * Vr,
                   nbytes=T * (2.0 * (2 * Hr * Dr + Hr * Vr) + 4.0 * Hr * Dr + 4.0 * Hr * Vr) + 8.0 * batch.num_seqs * Hr * Dr * Vr)
        del state

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

    print(json.dumps({"metric": "prefill and decode tokens/s, Dopipel beside Llama at equal size (4 layers, bf16, random weights)",
                      "size": args.arch_size, "shape": s, "prompt_tokens": P, "decode_batch": B, "decode_context": C,
                      "end_to_end": e2e, "kernels": kern, "peaks": {"hbm_Bps": HBM, "mfma_bf16": MFMA_BF16, "fma_f32": FMA_F32},
                      "time": time.strftime("%Y-%m-%d %H:%M:%S")}))
