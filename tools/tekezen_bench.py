"""Prefill and decode throughput of a Tekezen stack beside the Dopipel stack (the closest existing
model: rotary attention over key and value caches, dense and mixture-of-experts feed-forwards with
a shared expert over an fp32 stream) at equal size, and each of Tekezen's kernels beside the like
kernel of Dopipel or Lamosun against its roofline.

Run through `python bench.py --arch tekezen [--arch-size 2k|4k]` (one GPU, random weights, bf16).
Prints one JSON line.  `end_to_end`: tokens/s of a prompt step (one sequence of --arch-prompt
tokens) and of a decode step (--arch-batch sequences at --arch-context tokens) of four layers plus
logits: Tekezen (attention / latent attention / attention / latent attention with dense / experts
/ experts / dense) and Dopipel (four attention layers with the same feed-forwards).  `kernels`:
microseconds per launch, the time its algorithmic bytes or arithmetic would take at the part's
peaks, and the ratio (1.0 = on the roofline).  A windowed kernel is priced for the keys its window
lets it see.
"""
import json
import time

import torch

from tools.dopipel_bench import dopipel_config
from tools.seq_arch_bench import HBM, MFMA_BF16, FMA_F32, record, timed

SIZES = {
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, ff=5632, gru=2048, experts=16, identity=0, top=2,
               expert_ff=1408, shared_ff=1408, taps=4, rot_dim=64, kv_rank=512, window=1024, keep_first=4,
               latent_window=2048, softcap=30.0),
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, ff=11008, gru=4096, experts=32, identity=0, top=4,
               expert_ff=1408, shared_ff=2816, taps=4, rot_dim=64, kv_rank=512, window=1024, keep_first=4,
               latent_window=2048, softcap=30.0),
}


def tekezen_config(s, kinds, vocab):
    """kinds: per layer (mixer, feed-forward) out of attention | latent_attention and dense | moe."""
    mixers = {
        "attention": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["dim"],
                      "mask": {"size": s["window"], "keep_first": s["keep_first"]}, "scale": s["dim"]**-0.5,
                      "softcap": s["softcap"], "v_mix": True,
                      "rot": {"base": 100000.0, "dims": s["dim"] // 2, "scaling": {"factor": 4.0}}},
        "latent_attention": {"heads": s["heads"], "dim": s["dim"], "rot_dim": s["rot_dim"], "vdim": s["dim"],
                             "kv_rank": s["kv_rank"], "scale": (s["dim"] + s["rot_dim"])**-0.5,
                             "mask": {"size": s["latent_window"]},
                             "rot": {"base": 10000.0, "dims": s["rot_dim"],
                                     "scaling": {"factor": 40.0, "original": 4096, "fast": 32.0, "slow": 1.0}}},
    }
    dense = {"kind": "dense", "ff": s["ff"], "limit": 7.0}
    moe = {"kind": "moe", "expert": {"ff": s["expert_ff"], "limit": 7.0}, "shared": {"ff": s["shared_ff"], "limit": 7.0},
           "router": {"experts": s["experts"], "top": s["top"]}}
    layers = [{"type": m, "mixer": mixers[m], "mlp": dense if f == "dense" else moe} for m, f in kinds]
    return {"architecture": "Tekezen", "vocab": vocab, "width": s["width"], "norm": {"eps": 1e-5},
            "embedding": {"bigram": {"buckets": 65521, "mul_prev": 92821, "mul_cur": 1000003}}, "layers": layers}


def run(args):
    from vllm_legacy_amd import _seq_ops as sops
    from vllm_legacy_amd.attention.batch import SequenceBatch
    from vllm_legacy_amd.model.dopipel import DopipelConfig, DopipelForCausalLM
    from vllm_legacy_amd.model.tekezen import TekezenConfig, TekezenForCausalLM

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
                if t.is_floating_point():
                    t.normal_(0, 1.0 if k in ("keys", "values", "latent") else 0.1, generator=g)

    H, G, D, width, ff = s["heads"], s["kv_heads"], s["dim"], s["width"], s["ff"]
    E, top, eff, sff = s["experts"], s["top"], s["expert_ff"], s["shared_ff"]
    Rr, Cr = s["rot_dim"], s["kv_rank"]
    Wl = Cr + Rr
    win, keep, lwin = s["window"], s["keep_first"], s["latent_window"]

    def seen(T, ctx, window, kept=0):
        """(query, key) pairs a step of T rows after ctx cached tokens computes, per sequence."""
        if not window:
            return sum(p + 1 for p in range(ctx, ctx + T))
        return sum(min(p + 1, window) + min(kept, max(p + 1 - window, 0)) for p in range(ctx, ctx + T))

    # ------------------------------------------------------------------ Dopipel: whole steps and the like kernels
    kinds = [("attention", "dense"), ("attention", "moe"), ("attention", "moe"), ("attention", "dense")]
    model = DopipelForCausalLM(DopipelConfig.from_dict(dopipel_config(s, kinds, vocab)), dt, dev, seed=0)
    caches = model.allocate_caches(nblk, BS, B)
    fill(caches)
    whole_steps("dopipel", model, caches)
    with torch.inference_mode():
        attn, moe = model.layers[1].attn, model.layers[1].experts
        keys, values = caches[1]["keys"], caches[1]["values"]
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
                record(kern, "dopipel.kv_attention.prefill", sec, flops=4.0 * seen(T, 0, 0) * H * D,
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
            z = torch.randn(T, 2 * ff, device=dev, dtype=dt)
            a = torch.empty(T, ff, device=dev, dtype=dt)
            sec = timed(lambda: sops.gated_act(a, z[:, :ff], z[:, ff:], "relu"), it)
            record(kern, f"dopipel.gated_act.{tag}", sec, nbytes=2.0 * T * 3 * ff)
            hh = torch.randn(T, width, device=dev, dtype=dt)
            sec = timed(lambda: moe(hh), it)
            routed, used = T * top, min(E, T * top)
            record(kern, f"dopipel.experts.{tag}", sec, flops=4.0 * routed * width * eff + 4.0 * T * width * sff,
                   nbytes=2.0 * (2 * used * eff * width + 2 * sff * width + routed * width) + 4.0 * T * width,
                   note="route, plan, up product with its activation, down product, shared expert, combine")
    del model, caches
    torch.cuda.empty_cache()

    # ------------------------------------------------------------------ Lamosun's latent attention (no window)
    from vllm_legacy_amd.attention.backends.latent_kv import LatentKVAttention
    with torch.inference_mode():
        plain = LatentKVAttention(H, D, Rr, D, Cr, (D + Rr)**-0.5, Rr, 10000.0, None, 1e-5, dt, dev)
        latent = torch.randn(LatentKVAttention.get_cache_shape(nblk, BS, Cr, Rr), device=dev, dtype=dt)
        for tag, batch, T in (("prefill", pre, P), ("decode", dec, B)):
            it = 5 if tag == "prefill" else 20
            q_lat = torch.randn(H, T, Cr, device=dev, dtype=dt).transpose(0, 1)
            q = torch.randn(T, H * (D + Rr), device=dev, dtype=dt)
            q_rot = q.view(T, H, D + Rr)[:, :, D:]
            o_lat = torch.empty(H, T, Cr, device=dev, dtype=dt).transpose(0, 1)
            sec = timed(lambda: sops.latent_attention_tiles(o_lat, q_lat, q_rot, latent, batch.block_tables,
                                                            batch.query_start_loc, batch.context_lens,
                                                            batch.max_query_len, plain.scale, plain.key_splits(batch)), it)
            pairs = seen(T, 0, 0) if tag == "prefill" else seen(1, C - 1, 0) * B
            record(kern, f"lamosun.latent_attention.{tag}", sec, flops=2.0 * pairs * H * (Wl + Cr),
                   nbytes=2.0 * T * H * (Wl + Cr) + 2.0 * (T if tag == "prefill" else B * C) * Wl)
            kv = torch.randn(T, Wl, device=dev, dtype=dt)
            sec = timed(lambda: sops.latent_rotary_write(q, D + Rr, D, H, kv, plain.latent_norm.data, 1e-5, latent,
                                                         batch.positions, batch.slot_mapping, plain.inv_freq,
                                                         plain.magnitude, Rr), it)
            record(kern, f"lamosun.latent_rotary_write.{tag}", sec, nbytes=2.0 * T * (2 * H * Rr + 2 * Wl))
            xs = torch.empty(T, width, device=dev)
            table = torch.randn(vocab, width, device=dev, dtype=dt)
            ids = ids_p if tag == "prefill" else ids_d
            sec = timed(lambda: sops.embed_scaled(xs, table, ids, 2.0), it)
            record(kern, f"lamosun.embed_scaled.{tag}", sec, nbytes=T * width * (2.0 + 4))
        del plain, latent, table

    # ------------------------------------------------------------------ Tekezen: whole steps and its kernels
    kinds = [("attention", "dense"), ("latent_attention", "moe"), ("attention", "moe"), ("latent_attention", "dense")]
    model = TekezenForCausalLM(TekezenConfig.from_dict(tekezen_config(s, kinds, vocab)), dt, dev, seed=0)
    caches = model.allocate_caches(nblk, BS, B)
    fill(caches)
    whole_steps("tekezen", model, caches)
    with torch.inference_mode():
        attn, lat, moe = model.layers[2].attn, model.layers[1].attn, model.layers[1].experts
        keys, values, latent = caches[2]["keys"], caches[2]["values"], caches[1]["latent"]
        blend = model.layers[2].v_blend.data
        for tag, batch, T in (("prefill", pre, P), ("decode", dec, B)):
            it = 5 if tag == "prefill" else 20
            ctx, seqs, per_seq = (0, 1, T) if tag == "prefill" else (C - 1, B, 1)
            q = torch.randn(T, H * D, device=dev, dtype=dt)
            k = torch.randn(T, G * D, device=dev, dtype=dt)
            v = torch.randn(T, G * D, device=dev, dtype=dt)
            vo = torch.randn(T, G * D, device=dev, dtype=dt)
            out = torch.empty_like(q)
            pairs = seen(per_seq, ctx, win, keep) * seqs
            if tag == "prefill":
                sec = timed(lambda: sops.kv_attention_tiles(out, q, None, keys, values, batch.block_tables,
                                                            batch.query_start_loc, batch.context_lens,
                                                            batch.max_query_len, None, False, H, win, attn.scale, keep,
                                                            attn.softcap), it)
                record(kern, "tekezen.kv_attention.prefill", sec, flops=4.0 * pairs * H * D,
                       nbytes=2.0 * T * (2 * H + 2 * G) * D, note="window, kept first tokens, capped scores")
            else:
                sec = timed(lambda: sops.kv_attention(out, q, None, keys, values, batch.block_tables, batch.token_seq,
                                                      batch.positions, None, False, H, win, attn.scale, keep,
                                                      attn.softcap), it)
                record(kern, "tekezen.kv_attention.decode", sec, nbytes=2 * 2.0 * G * pairs * D + 2 * 2.0 * B * H * D,
                       note="reads the window and the kept tokens only")
            sec = timed(lambda: sops.rotary_kv_write(q, k, v, keys, values, batch.positions, batch.slot_mapping,
                                                     attn.inv_freq, None, H, attn.rot_dims, False, attn.q_norm.data,
                                                     attn.k_norm.data, 1e-5, vo, blend), it)
            record(kern, f"tekezen.rotary_kv_write.{tag}", sec, nbytes=2.0 * T * (2 * H + 5 * G) * D + 4.0 * (H + G) * D,
                   note="row norms, rotation, value blend and cache write in one launch")
            q_lat = torch.randn(H, T, Cr, device=dev, dtype=dt).transpose(0, 1)
            ql = torch.randn(T, H * (D + Rr), device=dev, dtype=dt)
            q_rot = ql.view(T, H, D + Rr)[:, :, D:]
            gate = torch.randn(T, H, device=dev, dtype=dt)
            o_lat = torch.empty(H, T, Cr, device=dev, dtype=dt).transpose(0, 1)
            sec = timed(lambda: sops.latent_attention_tiles(o_lat, q_lat, q_rot, latent, batch.block_tables,
                                                            batch.query_start_loc, batch.context_lens,
                                                            batch.max_query_len, lat.scale, lat.key_splits(batch), lwin,
                                                            gate), it)
            lpairs = seen(per_seq, ctx, lwin) * seqs
            record(kern, f"tekezen.latent_attention.{tag}", sec, flops=2.0 * lpairs * H * (Wl + Cr),
                   nbytes=2.0 * T * H * (Wl + Cr) + 2.0 * (T if tag == "prefill" else lpairs) * Wl,
                   note="window and head gates")
            kv = torch.randn(T, Wl, device=dev, dtype=dt)
            sec = timed(lambda: sops.latent_rotary_write(ql, D + Rr, D, H, kv, lat.latent_norm.data, 1e-5, latent,
                                                         batch.positions, batch.slot_mapping, lat.inv_freq, lat.magnitude,
                                                         Rr, False), it)
            record(kern, f"tekezen.latent_rotary_write.{tag}", sec, nbytes=2.0 * T * (2 * H * Rr + 2 * Wl))
            x = torch.randn(T, width, device=dev)
            y = torch.randn(T, width, device=dev)
            h = torch.empty(T, width, device=dev, dtype=dt)
            w = torch.ones(width, device=dev)
            sec = timed(lambda: sops.residual_norms(x, y, None, w, None, None, h, None, 1e-5), it)
            record(kern, f"tekezen.stream_update.{tag}", sec, nbytes=T * width * (4.0 + 4 + 4 + 2),
                   note="norm of the sublayer's output, fp32 stream and its 16-bit copy")
            z = torch.randn(T, 2 * ff, device=dev, dtype=dt)
            a = torch.empty(T, ff, device=dev, dtype=dt)
            sec = timed(lambda: sops.clamped_glu(a, z[:, :ff], z[:, ff:], 7.0, 1.702, 1.0), it)
            record(kern, f"tekezen.clamped_glu.{tag}", sec, nbytes=2.0 * T * 3 * ff)
            ids = ids_p if tag == "prefill" else ids_d
            xs = torch.empty(T, width, device=dev)
            sec = timed(lambda: sops.pair_hash_embed(xs, model.embed.weight.data, model.embed.pair_weight.data, ids,
                                                     caches[4]["last_token"], batch.query_start_loc, batch.context_lens,
                                                     batch.state_slots, batch.token_seq, 92821, 1000003), it)
            record(kern, f"tekezen.pair_hash_embed.{tag}", sec, nbytes=T * width * (2.0 + 2 + 4),
                   note="two table rows per token, and the launch that keeps every sequence's last token")
            hh = torch.randn(T, width, device=dev, dtype=dt)
            sec = timed(lambda: moe(hh), it)
            routed, used = T * top, min(E, T * top)
            record(kern, f"tekezen.experts.{tag}", sec, flops=6.0 * routed * width * eff + 6.0 * T * width * sff,
                   nbytes=2.0 * (3 * used * eff * width + 3 * sff * width + routed * width) + 4.0 * T * width,
                   note="route, plan, gate | up product, activation, down product, gated shared expert, combine")
    del model, caches
    torch.cuda.empty_cache()

    print(json.dumps({"metric": "prefill and decode tokens/s, Tekezen beside Dopipel at equal size (4 layers, bf16, random weights)",
                      "size": args.arch_size, "shape": s, "prompt_tokens": P, "decode_batch": B, "decode_context": C,
                      "end_to_end": e2e, "kernels": kern, "peaks": {"hbm_Bps": HBM, "mfma_bf16": MFMA_BF16, "fma_f32": FMA_F32},
                      "time": time.strftime("%Y-%m-%d %H:%M:%S")}))
