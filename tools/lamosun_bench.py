"""Prefill and decode throughput of a Lamosun stack beside the Dopipel stack (the closest existing
model: attention and recurrent layers, dense and mixture-of-experts feed-forwards over an fp32
stream) at equal size, and each of Lamosun's kernels beside the like kernel of Dopipel or Lusadra
against its roofline.

Run through `python bench.py --arch lamosun [--arch-size 2k|4k]` (one GPU, random weights, bf16).
Prints one JSON line.  `end_to_end`: tokens/s of a prompt step (one sequence of --arch-prompt
tokens) and of a decode step (--arch-batch sequences at --arch-context tokens) of four layers plus
logits: Lamosun (real-gated recurrence / latent attention / latent attention / delta rule with dense
/ experts / dense / experts) and Dopipel (minGRU / attention / attention / minGRU with the same
feed-forwards).  `kernels`: microseconds per launch, the time its algorithmic bytes or arithmetic
would take at the part's peaks, and the ratio (1.0 = on the roofline).
"""
import json
import time

import torch

from tools.dopipel_bench import dopipel_config
from tools.seq_arch_bench import FMA_F32, HBM, MFMA_BF16, record, timed

SIZES = {
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, ff=5632, gru=2048, experts=16, identity=0, top=2,
               expert_ff=1408, shared_ff=0, taps=4, rot_dim=64, kv_rank=512, q_rank=1536, blocks=16, delta_kv_heads=8,
               side=64),
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, ff=11008, gru=4096, experts=32, identity=0, top=4,
               expert_ff=1408, shared_ff=0, taps=4, rot_dim=64, kv_rank=512, q_rank=1536, blocks=32, delta_kv_heads=16,
               side=64),
}


def lamosun_config(s, kinds, vocab):
    """kinds: per layer (mixer, feed-forward) out of delta | rglru | latent_attention and dense | moe."""
    mixers = {
        "latent_attention": {"heads": s["heads"], "dim": s["dim"], "rot_dim": s["rot_dim"], "vdim": s["dim"],
                             "kv_rank": s["kv_rank"], "q_rank": s["q_rank"], "scale": (s["dim"] + s["rot_dim"])**-0.5,
                             "rot": {"base": 10000.0, "dims": s["rot_dim"],
                                     "scaling": {"factor": 40.0, "original": 4096, "fast": 32.0, "slow": 1.0}}},
        "delta": {"heads": s["heads"], "kv_heads": s["delta_kv_heads"], "dim": s["dim"], "vdim": s["dim"], "conv": s["taps"]},
        "rglru": {"width": s["gru"], "blocks": s["blocks"], "conv": s["taps"]},
    }
    dense = {"kind": "dense", "ff": s["ff"]}
    moe = {"kind": "moe", "expert": {"ff": s["expert_ff"]}, "router": {"experts": s["experts"], "top": s["top"]}}
    layers = [{"type": m, "mixer": mixers[m], "mlp": dense if f == "dense" else moe} for m, f in kinds]
    return {"architecture": "Lamosun", "vocab": vocab, "width": s["width"], "norm": {"eps": 1e-5}, "postln_alpha": 2.0,
            "embedding": {"scale": s["width"]**0.5}, "token_side": {"dim": s["side"]}, "logit_softcap": 30.0,
            "layers": layers}


def run(args):
    from vllm_legacy_amd import _seq_ops as sops
    from vllm_legacy_amd.attention.batch import SequenceBatch
    from vllm_legacy_amd.model.dopipel import DopipelConfig, DopipelForCausalLM
    from vllm_legacy_amd.model.lamosun import LamosunConfig, LamosunForCausalLM

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    dt = torch.bfloat16
    s = SIZES[args.arch_size]
    vocab, BS = 32000, 16
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

    def whole_steps(name, model, caches):
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

    def fill(caches):
        for c in caches:
            for k, t in c.items():
                t.normal_(0, 1.0 if k in ("keys", "values", "latent") else 0.1, generator=g)

    # ------------------------------------------------------------------ Dopipel: whole steps and the like kernels
    kinds = [("mingru", "dense"), ("attention", "moe"), ("attention", "dense"), ("mingru", "moe")]
    model = DopipelForCausalLM(DopipelConfig.from_dict(dopipel_config(dict(s, shared_ff=0), kinds, vocab)), dt, dev, seed=0)
    caches = model.allocate_caches(nblk, BS, B)
    fill(caches)
    whole_steps("dopipel", model, caches)
    H, G, D, width, ff, R = s["heads"], s["kv_heads"], s["dim"], s["width"], s["ff"], s["gru"]
    E, top, eff = s["experts"], s["top"], s["expert_ff"]
    with torch.inference_mode():
        attn, moe = model.layers[1].attn, model.layers[1].experts
        keys, values, conv_state, gru_state = caches[1]["keys"], caches[1]["values"], caches[1]["conv"], caches[0]["state"]
        for tag, batch, T in (("prefill", pre, P), ("decode", dec, B)):
            it = 5 if tag == "prefill" else 20
            q = torch.randn(T, H * D, device=dev, dtype=dt)
            k = torch.randn(T, G * D, device=dev, dtype=dt)
            v = torch.randn(T, G * D, device=dev, dtype=dt)
            out = torch.empty_like(q)
            if tag == "prefill":
                sec = timed(lambda: sops.kv_attention_tiles(out, q, None, keys, values, batch.block_tables,
                                                            batch.query_start_loc, batch.context_lens,
                                                            batch.max_query_len, attn.value_inv_freq, True, H, 0,
                                                            D**-0.5), it)
                record(kern, "dopipel.kv_attention.prefill", sec, flops=4.0 * (T * (T + 1) / 2) * H * D,
                       nbytes=2.0 * T * (2 * H + 2 * G) * D)
            else:
                sec = timed(lambda: sops.kv_attention(out, q, None, keys, values, batch.block_tables, batch.token_seq,
                                                      batch.positions, attn.value_inv_freq, True, H, 0, D**-0.5), it)
                record(kern, "dopipel.kv_attention.decode", sec, nbytes=2 * 2.0 * B * G * C * D + 2 * 2.0 * B * H * D)
            sec = timed(lambda: sops.rotary_kv_write(q, k, v, keys, values, batch.positions, batch.slot_mapping,
                                                     attn.inv_freq, attn.value_inv_freq, H, D, True), it)
            record(kern, f"dopipel.rotary_kv_write.{tag}", sec, nbytes=2.0 * T * (2 * H + 4 * G) * D)
            x = torch.randn(T, width, device=dev)
            y = torch.randn(T, width, device=dev)
            h = torch.empty(T, width, device=dev, dtype=dt)
            w = torch.ones(width, device=dev)
            sec = timed(lambda: sops.residual_norms(x, y, None, w, w, None, h, w, 1e-5), it)
            record(kern, f"dopipel.residual_norms.{tag}", sec, nbytes=T * width * (4.0 + 4 + 4 + 2))
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
            record(kern, f"dopipel.mingru_scan.{tag}", sec, nbytes=T * R * 2.0 * 4 + batch.num_seqs * R * 8.0)
            hh = torch.randn(T, width, device=dev, dtype=dt)
            experts, weights, _ = sops.moe_route(hh, moe.router.data, moe.correction.data, None, top)
            pair_row, row_token, tile_expert = sops.moe_plan(experts, E)
            rows, routed, used = row_token.numel(), T * top, min(E, T * top)
            u = torch.empty(rows, eff, device=dev, dtype=dt)
            sec = timed(lambda: sops.grouped_linear(u, hh, row_token, moe.w_up.data, tile_expert, "relu2"), it)
            record(kern, f"dopipel.grouped_linear_up.{tag}", sec, flops=2.0 * routed * width * eff,
                   nbytes=2.0 * (used * eff * width + routed * (width + eff)))
    del model, caches
    torch.cuda.empty_cache()

    # ------------------------------------------------------------------ Lusadra's walk (the like matrix recurrence)
    with torch.inference_mode():
        Dr, Vr = 128, 128
        state = torch.randn(B + 64, H, Dr, Vr, device=dev) * 0.1
        for tag, batch, T in (("prefill", pre, P), ("decode", dec, B)):
            qr = torch.randn(T, H * Dr, device=dev, dtype=dt)
            kr = torch.randn(T, H * Dr, device=dev, dtype=dt)
            vr = torch.randn(T, H * Vr, device=dev, dtype=dt)
            ld = -torch.rand(T, H * Dr, device=dev) * 0.1
            o = torch.empty(T, H, Vr, device=dev)
            sec = timed(lambda: sops.gla_scan(o, qr, kr, vr, ld, state, batch.query_start_loc, batch.context_lens,
                                              batch.state_slots, Dr**-0.5, batch.max_query_len), 5 if tag == "prefill" else 20)
            record(kern, f"lusadra.gla_scan.{tag}", sec, peak=FMA_F32, flops=4.0 * T * H * Dr * Vr,
                   nbytes=T * (2.0 * (2 * H * Dr + H * Vr) + 4.0 * H * Dr + 4.0 * H * Vr) + 8.0 * batch.num_seqs * H * Dr * Vr,
                   note="token by token, no cut into pieces")
        del state

    # ------------------------------------------------------------------ Lamosun: whole steps and its kernels
    kinds = [("rglru", "dense"), ("latent_attention", "moe"), ("latent_attention", "dense"), ("delta", "moe")]
    model = LamosunForCausalLM(LamosunConfig.from_dict(lamosun_config(s, kinds, vocab)), dt, dev, seed=0)
    caches = model.allocate_caches(nblk, BS, B)
    fill(caches)
    whole_steps("lamosun", model, caches)
    Rr, Cr, Gd = s["rot_dim"], s["kv_rank"], s["delta_kv_heads"]
    Wl = Cr + Rr
    with torch.inference_mode():
        attn, moe = model.layers[1].attn, model.layers[1].experts
        latent = caches[1]["latent"]
        lru, lru_conv = model.layers[0].lru, model.layers[0].conv
        rule, rule_conv = model.layers[3].rule, model.layers[3].conv
        for tag, batch, T in (("prefill", pre, P), ("decode", dec, B)):
            it = 5 if tag == "prefill" else 20
            q_lat = torch.randn(H, T, Cr, device=dev, dtype=dt).transpose(0, 1)
            q = torch.randn(T, H * (D + Rr), device=dev, dtype=dt)
            q_rot = q.view(T, H, D + Rr)[:, :, D:]
            o_lat = torch.empty(H, T, Cr, device=dev, dtype=dt).transpose(0, 1)
            sec = timed(lambda: sops.latent_attention_tiles(o_lat, q_lat, q_rot, latent, batch.block_tables,
                                                            batch.query_start_loc, batch.context_lens,
                                                            batch.max_query_len, attn.scale, attn.key_splits(batch)), it)
            if tag == "prefill":
                record(kern, "lamosun.latent_attention.prefill", sec, flops=2.0 * (T * (T + 1) / 2) * H * (Wl + Cr),
                       nbytes=2.0 * T * (H * (Wl + Cr) + Wl),
                       note="every head scores the cached latent itself: rank + rot numbers per key and rank per value")
            else:
                record(kern, "lamosun.latent_attention.decode", sec, flops=2.0 * B * C * H * (Wl + Cr),
                       nbytes=2.0 * B * C * Wl + 2.0 * B * H * (Wl + Cr),
                       note="the cache row of a key is read once for all heads")
            kv = torch.randn(T, Wl, device=dev, dtype=dt)
            sec = timed(lambda: sops.latent_rotary_write(q, D + Rr, D, H, kv, attn.latent_norm.data, 1e-5, latent,
                                                         batch.positions, batch.slot_mapping, attn.inv_freq,
                                                         attn.magnitude, Rr), it)
            record(kern, f"lamosun.latent_rotary_write.{tag}", sec, nbytes=2.0 * T * (2 * H * Rr + 2 * Wl),
                   note="norms the latent, rotates the shared key part and the queries' rotated parts, writes the cache row")
            x = torch.randn(T, width, device=dev)
            y = torch.randn(T, width, device=dev)
            h = torch.empty(T, width, device=dev, dtype=dt)
            w = torch.ones(width, device=dev)
            sec = timed(lambda: sops.post_norm(x, y, w, 2.0, 1e-5, h), it)
            record(kern, f"lamosun.post_norm.{tag}", sec, nbytes=T * width * (4.0 + 4 + 4 + 2),
                   note="sum, norm, fp32 stream and its 16-bit copy")
            sec = timed(lambda: sops.residual_norms(x, y, None, w, None, None, h, None, 1e-5), it)
            record(kern, f"lamosun.side_update.{tag}", sec, nbytes=T * width * (4.0 + 4 + 4 + 2))
            proj = torch.randn(T, 2 * R, device=dev)
            u = torch.empty(T, R, device=dev)
            sec = timed(lambda: lru_conv(u, proj[:, R:], caches[0]["conv"], batch), it)
            record(kern, f"lamosun.short_conv.{tag}", sec,
                   nbytes=T * R * 8.0 + batch.num_seqs * (s["taps"] - 1) * R * 8.0, note="fp32 in and out")
            bw = R // s["blocks"]
            gates = torch.randn(s["blocks"], T, 2 * bw, device=dev)
            og = torch.empty(T, R, device=dev, dtype=dt)
            sec = timed(lambda: sops.rglru_scan(og, gates, u, proj[:, :R], lru.rate.data, caches[0]["state"],
                                                batch.query_start_loc, batch.context_lens, batch.state_slots,
                                                batch.max_query_len), it)
            record(kern, f"lamosun.rglru_scan.{tag}", sec, nbytes=T * R * (4.0 * 4 + 2) + batch.num_seqs * R * 8.0,
                   note="fp32 gates, branch and recurrent input; long runs are walked in pieces")
            sec = timed(lambda: torch.baddbmm(lru.gate_bias.data, u.view(T, s["blocks"], bw).transpose(0, 1),
                                              lru.gate_weight.data), it)
            record(kern, f"lamosun.rglru_gates_product.{tag}", sec, peak=FMA_F32, flops=4.0 * T * R * bw,
                   nbytes=T * R * 12.0 + 8.0 * R * bw, note="vendor batched product in fp32")
            HV, GD = H * D, Gd * D
            cin = torch.randn(T, 2 * GD + 2 * HV + 2 * H, device=dev)
            qkv = torch.empty(T, 2 * GD + HV, device=dev)
            sec = timed(lambda: rule_conv(qkv, cin[:, :2 * GD + HV], caches[3]["conv"], batch), it)
            record(kern, f"lamosun.short_conv_silu.{tag}", sec,
                   nbytes=T * (2 * GD + HV) * 8.0 + batch.num_seqs * (s["taps"] - 1) * (2 * GD + HV) * 8.0)
            mixed = torch.empty(T, HV, device=dev, dtype=dt)
            qd, kd, vd = qkv.split([GD, GD, HV], dim=1)
            gt, bt, dtp = cin[:, 2 * GD + HV:].split([HV, H, H], dim=1)
            sec = timed(lambda: rule(mixed, qd, kd, vd, gt, bt, dtp, caches[3]["state"], batch), it)
            record(kern, f"lamosun.delta_rule_scan.{tag}", sec, peak=FMA_F32, flops=6.0 * T * H * D * D,
                   nbytes=T * (4.0 * (2 * GD + 2 * HV + 2 * H) + 2.0 * HV) + 8.0 * batch.num_seqs * H * D * D,
                   note="token by token: unit norms, gates, state update, read-out, head norm and output gate")
            hh = torch.randn(T, width, device=dev, dtype=dt)
            sec = timed(lambda: moe(hh), it)
            routed, used = T * top, min(E, T * top)
            record(kern, f"lamosun.gated_experts.{tag}", sec, flops=6.0 * routed * width * eff,
                   nbytes=2.0 * (3 * used * eff * width + routed * width) + 4.0 * T * width,
                   note="route, plan, gate | up product, activation, down product, combine")
            experts, weights, _ = sops.moe_route(hh, moe.router.data, None, None, top, None, moe.router_bias.data)
            pair_row, row_token, tile_expert = sops.moe_plan(experts, E)
            rows = row_token.numel()
            both = torch.empty(rows, 2 * eff, device=dev, dtype=dt)
            sec = timed(lambda: sops.grouped_linear(both, hh, row_token, moe.w_up.data, tile_expert), it)
            record(kern, f"lamosun.grouped_linear_gate_up.{tag}", sec, flops=4.0 * routed * width * eff,
                   nbytes=2.0 * (2 * used * eff * width + routed * (width + 2 * eff)))
            side = model.layers[0].side
            sec = timed(lambda: side(x, h, model.side_embed.data, ids_p if tag == "prefill" else ids_d), it)
            record(kern, f"lamosun.token_side_input.{tag}", sec,
                   nbytes=T * width * (2.0 + 4 + 4 + 2) + 2.0 * 2 * width * s["side"],
                   note="two thin products, the gated lookup and the stream update")
    del model, caches
    torch.cuda.empty_cache()

    print(json.dumps({"metric": "prefill and decode tokens/s, Lamosun beside Dopipel at equal size (4 layers, bf16, random weights)",
                      "size": args.arch_size, "shape": s, "prompt_tokens": P, "decode_batch": B, "decode_context": C,
                      "end_to_end": e2e, "kernels": kern, "peaks": {"hbm_Bps": HBM, "mfma_bf16": MFMA_BF16, "fma_f32": FMA_F32},
                      "time": time.strftime("%Y-%m-%d %H:%M:%S")}))
