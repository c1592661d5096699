"""Tekezen through the framework -- registry, checkpoint loader, cache manager, model runner,
scheduler, sampler -- and its mechanisms one by one, against the float64 reference of
tests/tekezen_oracle.py on small random models and inputs.

Mechanisms alone: the hashed pair embedding and its state across cuts and reused slots; the
clamped gated activation around its limits; the stream update with a norm weight stored around
zero; the row norms, rotation and value blend that the cache write does; attention with a window,
kept first tokens and a score cap (random inputs in many sizes and cuts; one planted key just
inside and just outside the window, just inside and just outside the kept tokens, at page borders,
in prompts and in decoding; the plain kernel against the matrix-core kernels); latent attention
with a window, a gate and rotate-half pairs (the same, plus keys shared out to several
workgroups); the experts with their shared expert.
Whole models: prompts whole, in portions down to two tokens and token by token; mixed batches with
pages and slots used again; long decoding; a batch does not change a request; greedy generation
through LLMEngine and the command line; the trace replayer as a program.  The float32 bar is
float32 rounding through the stack and is the one that finds faults of cutting, batching and
reuse: both number formats run the same code paths except the matrix-core kernels, which the
bfloat16 runs cover with a looser bar."""
import json
import os
import subprocess
import sys

import pytest
import torch

from tests import tekezen_oracle as R

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F = R.F
BAR = {torch.float32: 1e-4, torch.bfloat16: 0.2}
MEAN_BAR = {torch.float32: 1e-4, torch.bfloat16: 0.06}
YARN = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}


def configs():
    A, L, M, E = R.attention_layer, R.latent_layer, R.dense_mlp, R.moe_mlp
    return {
        "plain": R.make_config([
            A(4, 2, 16, window=9, keep_first=3, rot_dims=8, factor=2.0, softcap=12.0, v_mix=True, mlp=M(96)),
            L(4, 16, 8, 16, 24, window=13, scaling=YARN, mlp=E(6, 2, 24, 2.0, 16, 1.0)),
            A(4, 2, 16, window=9, keep_first=3, rot_dims=8, factor=2.0, softcap=12.0, v_mix=True, mlp=E(5, 3, 16, 1.5, 8, 3.0)),
            L(2, 8, 8, 24, 16, window=6, mlp=M(80, 0.7))]),
        # sizes that are neither equal nor powers of two; one key head, vdim != dim, a layer that does
        # not blend between two that do, a feed-forward missing, one expert chosen, no shared expert,
        # no cap, more kept tokens than the window is long, the whole head rotated, a latent layer first
        "odd": R.make_config([
            L(3, 12, 6, 20, 10, window=4, scale=0.4, base=300.0, scaling=YARN, mlp=E(3, 1, 20)),
            A(3, 1, 12, vdim=20, window=3, keep_first=5, base=77.0, v_mix=True, mlp=None),
            A(6, 3, 10, vdim=14, window=30, keep_first=1, rot_dims=4, factor=3.0, softcap=5.0, mlp=M(52, 1.0)),
            A(2, 1, 12, vdim=20, window=7, rot_dims=12, softcap=50.0, v_mix=True, mlp=E(4, 4, 6, 0.9, 10, 2.0))],
            vocab=131, width=40, buckets=29, mul_prev=7, mul_cur=1),
        # key heads = heads, every expert chosen, no windows at all, nobody blends, no rotated part
        # in the latent layer, one bucket, a multiplier of zero
        "equal": R.make_config([A(2, 2, 16, mlp=E(3, 3, 16, 2.0, 16, 2.0)), L(2, 16, 0, 16, 16, mlp=M(64)),
                                A(4, 4, 8, rot_dims=0, softcap=8.0, mlp=None)], buckets=1, mul_prev=0, mul_cur=3),
        # a window of one token; a window longer than any request; kept tokens without a cap (dense
        # feed-forwards only: behind a window that sees everything, one close call of a router in
        # bfloat16 would move every later token)
        "edges": R.make_config([A(2, 1, 8, window=1, keep_first=2, v_mix=True, mlp=M(24)),
                                L(2, 8, 4, 8, 12, window=1, mlp=None),
                                A(2, 1, 8, window=500, keep_first=4, factor=8.0, v_mix=True, mlp=M(20, 3.0)),
                                L(3, 8, 4, 8, 12, window=500, scaling=YARN, mlp=M(24))], width=48, buckets=997,
                               mul_prev=1000003, mul_cur=999983),
        # nothing a multiple of four: widths, ranks, head sizes, vocabulary, feed-forward sizes
        "ragged": R.make_config([
            A(3, 3, 10, vdim=14, window=11, keep_first=2, rot_dims=6, factor=2.5, softcap=9.0, mlp=E(5, 2, 18, 2.0, 6, 1.0)),
            L(3, 10, 6, 14, 18, window=7, scaling=YARN, mlp=M(50)),
            A(1, 1, 22, vdim=42, window=5, keep_first=1, rot_dims=2, v_mix=True, mlp=E(4, 4, 6, 1.0)),
            A(6, 1, 6, vdim=42, window=30, rot_dims=6, v_mix=True, mlp=None)],
            vocab=101, width=50, buckets=11, mul_prev=2, mul_cur=9),
        # sizes for the matrix-core kernels: multiples of 32, many heads
        "mfma": R.make_config([
            A(8, 2, 32, vdim=64, window=20, keep_first=4, rot_dims=16, factor=2.0, softcap=15.0, v_mix=True, mlp=M(64)),
            L(10, 32, 32, 32, 64, window=24, scaling=YARN, mlp=E(6, 2, 32, 2.0, 32, 1.0)),
            A(4, 4, 64, vdim=32, window=40, keep_first=70, softcap=30.0, mlp=None),
            L(3, 64, 16, 32, 96, window=70, mlp=None),
            A(4, 2, 32, vdim=64, window=33, v_mix=True, mlp=M(64))], width=128),
    }


class Served:
    """A checkpoint on disk, loaded through the registry, with the engine's cache manager and
    model runner around it."""

    def __init__(self, tmp_path, name, dtype, num_blocks=64, block_size=4, num_slots=3, seed=0):
        from vllm_legacy_amd.engine.cache_manager import CacheManager
        from vllm_legacy_amd.engine.model_runner import ModelRunner
        from vllm_legacy_amd.model.registry import load_model
        self.cfg = configs()[name]
        self.W = R.random_tensors(self.cfg, seed)
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
        return R.forward(self.cfg, self.W, tokens)

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


def make_batch(query_lens, context_lens, block_size=4, tables=None, slots=None):
    from vllm_legacy_amd.attention.batch import SequenceBatch
    if tables is None:
        tables, at = [], 0
        for n, c in zip(query_lens, context_lens):
            need = (n + c + block_size - 1) // block_size
            tables.append(list(range(at, at + need)))
            at += need
    slots = list(range(len(query_lens))) if slots is None else slots
    return SequenceBatch.build(query_lens, context_lens, tables, slots, block_size, DEV)


def close(got, want, tol, what=""):
    err = float((got.detach().cpu().to(F) - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err <= tol, (what, err)


# ----------------------------------------------------------------------------- row-wise layers
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pair_hash_embedding_cut_anywhere_with_slots_used_again(dtype):
    """Three sequences in steps of unequal sizes; the slots hold another sequence's last token when
    a new one starts; the first token of a sequence takes the table's last row whatever the slot
    holds."""
    from vllm_legacy_amd.layers import PairHashEmbedding
    vocab, W, buckets, mp, mc = 41, 24, 13, 1000003, 17
    emb = PairHashEmbedding(vocab, W, buckets, mp, mc, dtype, DEV)
    table, pair = rnd((vocab, W), 1).to(dtype), rnd((buckets + 1, W), 2).to(dtype)
    emb.weight.data, emb.pair_weight.data = table.to(DEV), pair.to(DEV)
    seqs = {k: tokens_of({"vocab": vocab}, n, s) for k, n, s in (("a", 11, 0), ("b", 1, 1), ("c", 6, 2), ("d", 5, 3))}
    want = {k: R.embedding(v, table.to(F), pair.to(F), {"buckets": buckets, "mul_prev": mp, "mul_cur": mc})
            for k, v in seqs.items()}
    state = torch.full((2, ), 7, dtype=torch.int64, device=DEV)
    slot = {"a": 1, "b": 0, "c": 0, "d": 1}            # c takes b's slot, d takes a's
    plan = [[("a", 2), ("b", 1)], [("c", 1), ("a", 1)], [("a", 8), ("c", 3)], [("c", 2), ("d", 4)], [("d", 1)]]
    at, got = {k: 0 for k in seqs}, {k: [] for k in seqs}
    for step in plan:
        batch = make_batch([n for _, n in step], [at[k] for k, _ in step], 4, slots=[slot[k] for k, _ in step])
        ids = torch.tensor(sum((seqs[k][at[k]:at[k] + n] for k, n in step), []), dtype=torch.int64, device=DEV)
        out = emb(ids, state, batch).cpu()
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n])
            o += n
            at[k] += n
    for k in seqs:
        assert at[k] == len(seqs[k])
        close(torch.cat(got[k]), want[k], 1e-6, k)
    assert state.tolist() == [seqs["c"][-1], seqs["d"][-1]]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("features,limit", [(24, 2.0), (50, 0.6), (1030, 7.0)])
def test_clamped_gated_activation(dtype, features, limit):
    """Values on both sides of +limit and -limit; aligned rows (eight values per access) and rows
    that are not."""
    from vllm_legacy_amd.layers import GatedActivation
    z = rnd((7, 2 * features), 1, 1.5 * limit).to(dtype)
    z[0, :4] = torch.tensor([limit, -limit, 1.01 * limit, -1.01 * limit]).to(dtype)
    z[0, features:features + 4] = torch.tensor([1.01 * limit, -1.01 * limit, limit, -limit]).to(dtype)
    want = R.clamped_glu(z[:, :features].to(F), z[:, features:].to(F), limit)
    assert float(want.abs().max()) <= limit * (limit + 1) + 1e-9
    got = GatedActivation("clamped_glu", True, limit, R.GLU_ALPHA, R.GLU_SHIFT)(z.to(DEV))
    close(got, want, 2e-6 if dtype == torch.float32 else 6e-3)
    if features % 8:            # a view whose rows start where eight-value accesses cannot
        got = GatedActivation("clamped_glu", True, limit)(z.to(DEV)[:, 1:2 * features - 1])
        close(got, R.clamped_glu(z[:, 1:features].to(F), z[:, features:2 * features - 1].to(F), limit),
              2e-6 if dtype == torch.float32 else 6e-3)
    with pytest.raises(ValueError):
        GatedActivation("clamped_glu", True, 0.0)


@pytest.mark.parametrize("width", [40, 256, 2500])
def test_stream_update_with_a_weight_stored_around_zero(width):
    from vllm_legacy_amd import _seq_ops as ops
    x, y, w = rnd((5, width), 1), rnd((5, width), 2, 3.0), 0.3 * rnd((width, ), 3)
    want = x.to(F) + R.stream_norm(y.to(F), w.to(F), 1e-5)
    xs, h = x.to(DEV).clone(), torch.empty((5, width), dtype=torch.bfloat16, device=DEV)
    ops.residual_norms(xs, y.to(DEV), None, (1.0 + w).to(DEV), None, None, h, None, 1e-5)
    close(xs, want, 2e-6)
    assert torch.equal(h, xs.to(torch.bfloat16))


# ----------------------------------------------------------------------------- attention over keys and values
def attention_spec(H, G, D, V, rot_dims, base=500.0, factor=1.0, scale=None, softcap=0.0, window=0, keep_first=0):
    return {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": D**-0.5 if scale is None else scale,
            "softcap": softcap, "rot": {"dims": rot_dims, "base": base, "scaling": {"factor": factor}},
            "mask": {"size": window, "keep_first": keep_first}}


def attention_reference(spec, q, k, v, q_norm=None, k_norm=None, eps=1e-5, v_other=None, lam=None):
    """q [n, H, D], k [n, G, D], v [n, G, V] as the projections give them -> ([n, H, V], rotated
    keys, cached values)."""
    n, (H, G, D, V) = q.shape[0], (spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"])
    pos = torch.arange(n)
    f = R.plain_frequencies(spec["rot"]["dims"], spec["rot"]["base"]) / spec["rot"]["scaling"]["factor"] \
        if spec["rot"]["dims"] else torch.zeros(0, dtype=F)
    q, k, v = q.to(F), k.to(F), v.to(F)
    if q_norm is not None:
        q = R.rms_norm(q.reshape(n, H * D), q_norm.to(F), eps).view(n, H, D)
        k = R.rms_norm(k.reshape(n, G * D), k_norm.to(F), eps).view(n, G, D)
    q, k = R.rotate_half(q, pos, f), R.rotate_half(k, pos, f)
    if v_other is not None:
        v = (1.0 - lam) * v + lam * v_other.to(F)
    out = R.attention_core(q, k, v, spec["scale"], spec["softcap"], spec["mask"]["size"], spec["mask"]["keep_first"])
    return out, k, v


def run_attention(spec, q, k, v, cuts, dtype, block_size=4, norms=None, v_other=None, lam=None, shuffle_pages=True,
                  caches_out=None):
    """One sequence through RotaryKVAttention in steps of the given sizes; pages in a scrambled
    order.  Returns [n, H, V] fp32 on the CPU."""
    from vllm_legacy_amd.attention.backends.rotary_kv import RotaryKVAttention
    H, G, D, V = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    n = q.shape[0]
    layer = RotaryKVAttention(H, G, D, V, spec["scale"], spec["rot"]["dims"], spec["rot"]["base"], False, False,
                              spec["mask"]["size"] or None, DEV, keep_first=spec["mask"]["keep_first"],
                              softcap=spec["softcap"], freq_scale=spec["rot"]["scaling"]["factor"],
                              norm_rows=norms is not None, norm_eps=1e-5)
    if norms is not None:
        layer.q_norm.data, layer.k_norm.data = norms[0].float().to(DEV), norms[1].float().to(DEV)
    blend = None if lam is None else torch.tensor([lam], dtype=torch.float32, device=DEV)
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
        vo = None if v_other is None else v_other[at:at + c].reshape(c, G * V).to(dtype).to(DEV)
        out = torch.empty((c, H * V), dtype=dtype, device=DEV)
        layer(out, qq, kk, vv, None, kc, vc, batch, vo, blend)
        outs.append(out.float().cpu().view(c, H, V))
        at += c
    assert at == n
    if caches_out is not None:
        rows = torch.tensor([order[j // block_size] * block_size + j % block_size for j in range(n)])
        caches_out.append(kc.view(-1, G, D)[rows.to(DEV)].float().cpu())
        caches_out.append(vc.view(-1, G, V)[rows.to(DEV)].float().cpu())
    return torch.cat(outs)


ATTN_SHAPES = [
    # H, G, D, V, rot_dims, window, keep_first, softcap, factor
    (4, 2, 16, 16, 8, 9, 3, 10.0, 2.0),
    (3, 1, 24, 12, 24, 5, 0, 0.0, 1.0),
    (6, 3, 8, 20, 4, 70, 2, 4.0, 3.0),
    (2, 2, 40, 6, 0, 1, 1, 25.0, 1.0),
    (2, 1, 12, 12, 12, 3, 9, 0.0, 5.0),
    (10, 2, 32, 64, 16, 20, 4, 12.0, 2.0),
    (2, 1, 96, 64, 64, 33, 0, 8.0, 1.0),
    (8, 1, 64, 32, 32, 64, 6, 0.0, 4.0),
    (5, 5, 128, 128, 64, 17, 40, 30.0, 2.0),
    (4, 2, 32, 96, 32, 0, 0, 6.0, 1.0),
    (6, 2, 64, 32, 16, 60, 5, 18.0, 3.0),
    (4, 1, 32, 32, 16, 10, 3, 0.0, 1.0),
]


@pytest.mark.parametrize("shape", ATTN_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_prompt_portions_and_decoding(shape, dtype):
    """Random inputs large enough for the cap to bend the scores; every key has a value level of its
    own, so a window or a kept token that is one off moves the output."""
    H, G, D, V, rot, window, keep, cap, factor = shape
    spec = attention_spec(H, G, D, V, rot, 500.0, factor, None, cap, window, keep)
    n = 75
    q, k, v = rnd((n, H, D), 0, 1.7), rnd((n, G, D), 1, 1.7), rnd((n, G, V), 2)
    v += (torch.arange(n).float() % 7)[:, None, None] * 3.0
    if dtype == torch.bfloat16:
        q, k, v = (t.to(dtype).float() for t in (q, k, v))
    want, _, _ = attention_reference(spec, q, k, v)
    if window:
        for other in (dict(window=window + 1), dict(keep_first=keep + 1))[:2 if window < 40 else 1]:
            off, _, _ = attention_reference(attention_spec(H, G, D, V, rot, 500.0, factor, None, cap,
                                                           other.get("window", window), other.get("keep_first", keep)), q, k, v)
            assert float((want - off).abs().max()) > 0.05
    bar = 3e-5 if dtype == torch.float32 else 0.06
    for cuts in ([n], [2, 3, 4, 5, 1, 7, 2] * 5, [40] + [1] * 35, [33, 35, 7], [1] * n):
        got = run_attention(spec, q, k, v, cuts, dtype)
        assert float((got - want).abs().max()) <= bar * float(want.abs().max()), (cuts[:3], float((got - want).abs().max()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 2, 16, 24, 8), (3, 3, 12, 12, 12), (4, 1, 64, 32, 32)])
def test_row_norms_rotation_and_value_blend_in_the_cache(dtype, shape):
    """The whole query row and the whole key row are normed (not head by head) before they are
    rotated; the cache holds the rotated keys and the blended values."""
    H, G, D, V, rot = shape
    spec = attention_spec(H, G, D, V, rot, 300.0, 2.0, 0.3, 9.0, 6, 2)
    n = 29
    q, k, v, vo = rnd((n, H, D), 0, 3.0), rnd((n, G, D), 1, 0.2), rnd((n, G, V), 2), rnd((n, G, V), 3, 2.0)
    q[:, 0] *= 4.0               # heads of unequal size: a norm per head would give something else
    k[:, -1] *= 5.0
    norms = (1 + 0.3 * rnd((H * D, ), 4), 1 + 0.3 * rnd((G * D, ), 5))
    if dtype == torch.bfloat16:
        q, k, v, vo = (t.to(dtype).float() for t in (q, k, v, vo))
    want, want_k, want_v = attention_reference(spec, q, k, v, norms[0], norms[1], 1e-5, vo, 0.3)
    bar = 3e-5 if dtype == torch.float32 else 0.06
    for cuts in ([n], [5, 1, 1, 9, 2, 11], [1] * n):
        caches = []
        got = run_attention(spec, q, k, v, cuts, dtype, norms=norms, v_other=vo, lam=0.3, caches_out=caches)
        assert float((got - want).abs().max()) <= bar * float(want.abs().max()), cuts[:3]
        close(caches[0], want_k, 1e-5 if dtype == torch.float32 else 1e-2, "keys")
        close(caches[1], want_v, 1e-5 if dtype == torch.float32 else 1e-2, "values")


def planted(spec, n, rows, key, dtype, seed=0):
    """Random q, k, v in which the queries `rows` and the key `key` share one large coordinate that
    is not rotated, and the key's value is a level nobody else has: if the key is visible it takes
    the whole weight, if not the output stays with the others."""
    H, G, D, V = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    q, k, v = rnd((n, H, D), seed, 0.3), rnd((n, G, D), seed + 1, 0.3), rnd((n, G, V), seed + 2)
    big = (60.0 / spec["scale"])**0.5
    q[rows, :, D - 1] = big
    k[key, :, D - 1] = big
    v[key] = 40.0
    if dtype == torch.bfloat16:
        q, k, v = (t.to(dtype).float() for t in (q, k, v))
    return q, k, v


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dim,block_size", [(16, 4), (64, 16)])
@pytest.mark.parametrize("case", ["window_in", "window_out", "first_in", "first_out", "far_first", "page_edge"])
def test_one_key_at_the_edges_of_window_and_kept_tokens(dtype, dim, block_size, case):
    """A key exactly window - 1 back (seen) and window back (not seen); the last kept token (seen
    from hundreds of tokens on) and the one after it (not); the sequence's first token; a key on a
    page's last place seen from the next page's first.  In a prompt, in portions and in decoded
    rows; 16-bit runs take the matrix-core kernels at dim 64."""
    window, keep, n = 37, 5, 300
    spec = attention_spec(4, 2, dim, dim, dim // 2, 200.0, 2.0, None, 50.0, window, keep)
    rows = list(range(n - 20, n))
    # window_in: the last row sees the key at exactly window - 1 back; window_out: the rows up to
    # n - 11 see it (the last of them at window - 1 back), the rows from n - 10 on do not
    key, seen = {"window_in": (n - window, True), "window_out": (n - window - 10, None),
                 "first_in": (keep - 1, True), "first_out": (keep, False), "far_first": (0, True),
                 "page_edge": (n - 20 - (n - 20) % block_size - 1, None)}[case]
    q, k, v = planted(spec, n, rows, key, dtype)
    want, _, _ = attention_reference(spec, q, k, v)
    level = want[rows].mean(-1)           # ~40 where the key is seen, ~0 where it is not
    for i, r in enumerate(rows):
        vis = key <= r and (r - key < window or key < keep)
        assert (float(level[i].min()) > 35.0) == vis and (float(level[i].max()) < 5.0) == (not vis), (case, r)
    if seen is not None:
        assert all((float(level[i].min()) > 35.0) == seen for i in range(len(rows)))
    else:
        assert 0 < sum(float(level[i].min()) > 35.0 for i in range(len(rows))) < len(rows) or case == "page_edge"
    bar = 3e-5 if dtype == torch.float32 else 0.06
    for cuts in ([n], [n - 20] + [1] * 20, [100, 3, 170, 2, 25], [n - 30, 17, 2, 2] + [1] * 9):
        got = run_attention(spec, q, k, v, cuts, dtype, block_size=block_size)
        assert float((got - want).abs().max()) <= bar * float(want.abs().max()), (case, cuts[:2])


def test_plain_and_matrix_core_kernels_agree():
    """bfloat16 through the kernel every dtype can take and through the matrix-core kernels."""
    from vllm_legacy_amd import _seq_ops as ops
    spec = attention_spec(8, 2, 96, 64, 64, 1000.0, 2.0, None, 9.0, 45, 3)
    n = 131
    q, k, v = (t.to(torch.bfloat16).float() for t in (rnd((n, 8, 96), 0, 1.5), rnd((n, 2, 96), 1, 1.5), rnd((n, 2, 64), 2)))
    fast = run_attention(spec, q, k, v, [90, 3] + [1] * 38, torch.bfloat16)
    ops.set_kv_attention_kernel(1)
    try:
        plain = run_attention(spec, q, k, v, [90, 3] + [1] * 38, torch.bfloat16)
    finally:
        ops.set_kv_attention_kernel(0)
    assert float((fast - plain).abs().max()) <= 0.03 * float(plain.abs().max())
    assert not torch.equal(fast, plain)          # two kernels did run


# ----------------------------------------------------------------------------- latent attention
def latent_layer_of(shape, dtype, scaling, window, seed=0, base=700.0):
    from vllm_legacy_amd.attention.backends.latent_kv import LatentKVAttention
    H, D, Rr, V, C = shape
    attn = LatentKVAttention(H, D, Rr, V, C, (D + Rr)**-0.5, Rr, base, scaling, 1e-5, dtype, DEV, interleaved=False,
                             window=window or None)
    uk, uv, nw = rnd((H * D, C), seed + 1, C**-0.5), rnd((H * V, C), seed + 2, C**-0.5), 1 + 0.2 * rnd((C, ), seed + 3)
    uk, uv = uk.to(torch.bfloat16), uv.to(torch.bfloat16)
    attn.set_weights(uk, uv, nw)
    return attn, uk.to(F), uv.to(F), nw.to(F)


def latent_reference(shape, q, kv, gate, uk, uv, nw, scaling, window, base=700.0):
    """q [n, H (D + R)], kv [n, C + R], gate [n, H] -> ([n, H V], cache rows [n, C + R])."""
    H, D, Rr, V, C = shape
    n = q.shape[0]
    pos = torch.arange(n)
    f, mag = R.yarn_frequencies({"dims": Rr, "base": base, "scaling": scaling}) if Rr else (torch.zeros(0, dtype=F), 1.0)
    q3, kv = q.to(F).view(n, H, D + Rr), kv.to(F)
    c = R.rms_norm(kv[:, :C], nw, 1e-5)
    k_rot = R.rotate_half(kv[:, C:].view(n, 1, Rr), pos, f, mag)
    keys = torch.cat([(c @ uk.T).view(n, H, D), k_rot.expand(n, H, Rr)], -1)
    qq = torch.cat([q3[..., :D], R.rotate_half(q3[..., D:], pos, f, mag)], -1)
    o = R.attention_core(qq, keys, (c @ uv.T).view(n, H, V), (D + Rr)**-0.5, 0.0, window)
    if gate is not None:
        o = o * torch.sigmoid(gate.to(F))[:, :, None]
    return o.reshape(n, H * V), torch.cat([c, k_rot[:, 0]], -1)


def run_latent(attn, shape, q, kv, gate, cuts, dtype, block_size=4, cache_out=None):
    from vllm_legacy_amd.attention.backends.latent_kv import LatentKVAttention
    H, D, Rr, V, C = shape
    n = q.shape[0]
    pages = (n + block_size - 1) // block_size
    order = torch.randperm(pages + 3, generator=torch.Generator().manual_seed(2)).tolist()
    cache = torch.full(LatentKVAttention.get_cache_shape(pages + 3, block_size, C, Rr), float("nan"), dtype=dtype, device=DEV)
    outs, at = [], 0
    for c in cuts:
        c = min(c, n - at)
        if c <= 0:
            break
        batch = make_batch([c], [at], block_size, tables=[order[:pages]])
        gg = None if gate is None else gate[at:at + c].to(dtype).to(DEV)
        outs.append(attn(q[at:at + c].to(dtype).to(DEV).clone(), kv[at:at + c].to(dtype).to(DEV), cache, batch, gg).float().cpu())
        at += c
    assert at == n
    if cache_out is not None:
        rows = torch.tensor([order[j // block_size] * block_size + j % block_size for j in range(n)])
        cache_out.append(cache.view(-1, C + Rr)[rows.to(DEV)].float().cpu())
    return torch.cat(outs)


LATENT_SHAPES = [
    # H, D, R, V, C, window, scaling
    (4, 16, 8, 16, 24, 13, YARN),
    (3, 12, 6, 20, 10, 4, None),
    (2, 16, 0, 16, 16, 30, None),
    (5, 8, 12, 6, 18, 1, YARN),
    (2, 24, 4, 24, 40, 0, YARN),
    (10, 32, 32, 32, 64, 24, YARN),
    (3, 64, 16, 32, 96, 70, None),
    (40, 16, 16, 16, 32, 9, YARN),
    (4, 32, 48, 64, 128, 0, None),
]


@pytest.mark.parametrize("shape", LATENT_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_attention_prompt_portions_and_decoding(shape, dtype):
    *sizes, window, scaling = shape
    attn, uk, uv, nw = latent_layer_of(sizes, dtype, scaling, window)
    H, D, Rr, V, C = sizes
    n = 75
    q, kv, gate = rnd((n, H * (D + Rr)), 5, 1.5), rnd((n, C + Rr), 6, 1.5), rnd((n, H), 7, 2.0)
    if dtype == torch.bfloat16:
        q, kv, gate = (t.to(dtype).float() for t in (q, kv, gate))
    want, rows = latent_reference(sizes, q, kv, gate, uk, uv, nw, scaling, window)
    if window:
        off, _ = latent_reference(sizes, q, kv, gate, uk, uv, nw, scaling, window + 1)
        assert float((want - off).abs().max()) > 0.01
    bar = 3e-5 if dtype == torch.float32 else 0.06
    for cuts in ([n], [2, 3, 4, 5, 1, 7, 2] * 5, [40] + [1] * 35, [1] * n):
        cache = []
        got = run_latent(attn, sizes, q, kv, gate, cuts, dtype, cache_out=cache)
        assert float((got - want).abs().max()) <= bar * float(want.abs().max()), (cuts[:3], float((got - want).abs().max()))
        close(cache[0], rows, 1e-5 if dtype == torch.float32 else 1e-2, "cache rows")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape,block_size", [((4, 16, 8, 16, 24), 4), ((4, 32, 16, 32, 64), 16)])
@pytest.mark.parametrize("back", ["inside", "outside", "own_page_edge"])
def test_one_latent_key_at_the_window_edge(dtype, shape, block_size, back):
    """Head 1's last queries ask, through W_uk, for the latent of one key: exactly window - 1 back
    from some of them and window back from the others (or on a page's last place), in a prompt, in
    portions, in decoded rows, and with the keys shared out to two workgroups."""
    H, D, Rr, V, C = shape
    window, n = 290, 620
    attn, uk, uv, nw = latent_layer_of(shape, dtype, YARN, window, seed=5)
    first = n - 20
    key = {"inside": first - window + 1, "outside": first - window + 10,
           "own_page_edge": first - first % block_size - 1}[back]
    q, kv = rnd((n, H * (D + Rr)), 9, 0.3), rnd((n, C + Rr), 10)
    ask = rnd((D, ), 11)
    lat = (uk.view(H, D, C)[1].T @ ask.to(F)).float()
    unit = lat / lat.norm()
    kv[:, :C] -= (kv[:, :C] @ unit)[:, None] * unit[None, :]      # nobody else answers that question
    kv[key, :C] = 6.0 * unit * C**0.5
    q.view(n, H, D + Rr)[first:, 1, :D] = 30.0 * ask / ask.norm()
    if dtype == torch.bfloat16:
        q, kv = q.to(dtype).float(), kv.to(dtype).float()
    want, _ = latent_reference(shape, q, kv, None, uk, uv, nw, YARN, window)
    alone, _ = latent_reference(shape, q[key:key + 1], kv[key:key + 1], None, uk, uv, nw, YARN, window)
    own = alone.view(H, V)[1]
    hits = [float((want[r].view(H, V)[1] - own).abs().max()) < 0.05 * float(own.abs().max()) for r in range(first, n)]
    assert hits == [r - key < window for r in range(first, n)] and (back != "outside" or (any(hits) and not all(hits)))
    bar = 3e-5 if dtype == torch.float32 else 0.06
    for cuts, splits in (([n], None), ([first] + [1] * 20, None), ([first] + [1] * 20, 2), ([300, 3, 290, 2, 25], None)):
        if splits:
            attn.key_splits = lambda batch, s=splits: s if batch.max_seq_len > 512 else 1
        got = run_latent(attn, shape, q, kv, None, cuts, dtype, block_size=block_size)
        assert float((got - want).abs().max()) <= bar * float(want.abs().max()), (back, cuts[:2], splits)


def test_plain_and_matrix_core_latent_kernels_agree():
    from vllm_legacy_amd import _seq_ops as ops
    shape = (6, 32, 16, 32, 96)
    attn, uk, uv, nw = latent_layer_of(shape, torch.bfloat16, YARN, 50)
    n = 131
    q, kv, gate = (t.to(torch.bfloat16).float() for t in (rnd((n, 6 * 48), 0), rnd((n, 112), 1), rnd((n, 6), 2)))
    fast = run_latent(attn, shape, q, kv, gate, [90, 3] + [1] * 38, torch.bfloat16)
    ops.set_latent_attention_kernel(1)
    try:
        plain = run_latent(attn, shape, q, kv, gate, [90, 3] + [1] * 38, torch.bfloat16)
    finally:
        ops.set_latent_attention_kernel(0)
    assert float((fast - plain).abs().max()) <= 0.03 * float(plain.abs().max())
    assert not torch.equal(fast, plain)


# ----------------------------------------------------------------------------- feed-forward
@pytest.mark.parametrize("shape", [(64, 6, 2, 24, 16), (40, 3, 1, 20, 0), (128, 5, 5, 64, 32), (96, 12, 3, 32, 40)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [3, 300])
def test_experts_with_clamped_activation_and_shared_expert(shape, dtype, rows):
    from vllm_legacy_amd.routed_experts import RoutedExperts
    W, E, top, ff, sff = shape
    moe = RoutedExperts(W, E, 0, top, ff, sff, "clamped_glu", dtype=dtype, device=DEV, gated=True, act_limit=1.2,
                        act_alpha=R.GLU_ALPHA, act_shift=R.GLU_SHIFT, shared_gated=True, shared_limit=0.5)
    t = {"router": rnd((E, W), 1, 3 * W**-0.5)}
    names = [f"e{e}." for e in range(E)] + (["shared."] if sff else [])
    for i, p in enumerate(names):
        f = sff if p == "shared." else ff
        t[p + "gate"], t[p + "up"], t[p + "down"] = rnd((f, W), 10 + i, 2 * W**-0.5), rnd((f, W), 40 + i, 2 * W**-0.5), rnd((W, f), 70 + i, f**-0.5)
    t = {k: v.to(torch.bfloat16) for k, v in t.items()}
    moe.set_weights(t)
    h = rnd((rows, W), 3).to(dtype)
    spec = {"router": {"experts": E, "top": top}, "expert": {"limit": 1.2}}
    if sff:
        spec["shared"] = {"limit": 0.5}
    want = R.routed_ff(h.to(F), {k: v.to(F) for k, v in t.items()}, spec)
    got = moe(h.to(DEV)).cpu()
    err = (got.to(F) - want).abs().amax(1) / want.abs().max()
    if dtype == torch.float32:
        assert float(err.max()) <= 2e-5
    else:       # a close call of the router may go the other way for a few rows
        assert float(torch.quantile(err, 0.9)) <= 3e-2


# ----------------------------------------------------------------------------- whole models
@pytest.mark.parametrize("name", list(configs()))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_whole_prompt_portions_and_decoding_agree_with_the_reference(tmp_path, name, dtype):
    s = Served(tmp_path, name, dtype)
    n = 90 if name == "mfma" else 41
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


@pytest.mark.parametrize("name", ["plain", "odd", "equal", "edges", "ragged"])
def test_layer_by_layer_against_the_reference(tmp_path, name):
    """The stream after every layer, float32."""
    s = Served(tmp_path, name, torch.float32)
    toks = tokens_of(s.cfg, 17, 4)
    taps = []
    R.forward(s.cfg, s.W, toks, taps)
    s.cache.admit("a")
    s.cache.grow("a", 17)
    batch = make_batch([17], [0], 4, tables=[s.cache.block_table("a")], slots=[s.cache.state_slot("a")])
    got = []
    with torch.inference_mode():
        s.model(torch.tensor(toks, device=DEV), batch.positions, s.runner.caches, batch,
                tap=lambda i, x: got.append(x.detach().cpu().clone()))
    assert len(got) == len(taps) == len(s.cfg["layers"])
    for i, (a, b) in enumerate(zip(got, taps)):
        assert float((a.to(F) - b).abs().max() / b.abs().max()) <= 2e-5, i


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


@pytest.mark.parametrize("name", ["plain", "edges"])
def test_long_decoding_over_many_pages(tmp_path, name):
    """The windows pass over decoded tokens many times; kept tokens stay in sight."""
    s = Served(tmp_path, name, torch.float32, num_blocks=80, block_size=4)
    toks = tokens_of(s.cfg, 200, 8)
    got = [s.step([("a", toks[:3])])["a"]]
    for t in range(3, 200):
        got.append(s.step([("a", toks[t:t + 1])])["a"])
    s.check(torch.cat(got), toks)


def test_long_prompts_beside_a_decoding_request(tmp_path):
    """Prompts of several hundred tokens (windows and kept tokens far apart), whole and in large
    portions beside a decoding request, in bfloat16 on the matrix cores."""
    s = Served(tmp_path, "mfma", torch.bfloat16, num_blocks=100, block_size=16)
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
    assert type(engine.runner.model).__name__ == "TekezenForCausalLM"
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
