"""Lamosun through the framework -- registry, checkpoint loader, cache manager, model runner,
scheduler, sampler -- and its mechanisms one by one, against the float64 reference of
tests/lamosun_oracle.py on small random models and inputs.

Mechanisms alone: the norm after the sum; plain row norms; the short convolution with bias and
activation and its state across cuts and reused slots; the gated delta rule (shared key heads, a
write that is read hundreds of tokens later, cuts, slots used again); the real-gated recurrence
short, in pieces and cut; latent attention (the cache rows, a far key that carries the whole
output, keys at page borders, prompts in portions and decoding); gated experts with a router bias;
the token's side input; embedding scale and logit cap.
Whole models: prompts whole, in portions down to two tokens and token by token; mixed batches with
pages and slots used again; long decoding; long prompts; a batch does not change a request; greedy
generation through LLMEngine and the command line; the trace replayer as a program.  The float32
bar is float32 rounding through the stack (1e-4 of the logits' spread) and is the one that finds
faults of cutting, batching and reuse: both number formats run the same code paths except the
matrix-core kernels, which the bfloat16 runs cover with a looser bar."""
import json
import os
import subprocess
import sys

import pytest
import torch

from tests import lamosun_oracle as R

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F = R.F
BAR = {torch.float32: 1e-4, torch.bfloat16: 0.2}
MEAN_BAR = {torch.float32: 1e-4, torch.bfloat16: 0.06}
YARN = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}


def configs():
    A, D, G, M, E = R.latent_layer, R.delta_layer, R.rglru_layer, R.dense_mlp, R.moe_mlp
    return {
        "plain": R.make_config([D(4, 2, 16, mlp=E(6, 2, 24)), A(4, 16, 8, 16, 24, 20, scaling=YARN, mlp=M(96)),
                                G(48, 3, mlp=E(5, 3, 16)), D(2, 2, 16, vdim=24, mlp=M(80))]),
        # sizes that are neither equal nor powers of two; one key head, vdim != dim, no side input,
        # no cap, alpha 1, a feed-forward missing, one expert chosen, one block, two taps
        "odd": R.make_config([G(50, 1, conv=2, mlp=None), A(3, 12, 6, 20, 10, 14, scale=0.4, base=300.0, mlp=E(3, 1, 20)),
                              D(6, 1, 12, vdim=20, conv=2, mlp=M(52))], vocab=131, width=40, alpha=1.0, embed_scale=1.0,
                             side_dim=0, softcap=0),
        # key heads = heads, every expert chosen, one tap, blocks = width, no rotated part
        "equal": R.make_config([D(2, 2, 16, conv=1, mlp=E(3, 3, 16)), G(32, 32, conv=1, mlp=M(64)),
                                A(2, 16, 0, 16, 16, 16, mlp=None)], side_dim=4),
        # more taps than some requests have tokens
        "taps": R.make_config([G(32, 2, conv=6, mlp=M(48)), D(2, 1, 32, conv=7, mlp=E(4, 2, 16)),
                               A(2, 32, 16, 32, 32, 24, scaling=YARN, mlp=None)], width=48),
        # nothing a multiple of eight: widths, ranks, head sizes, vocabulary, the side input's size
        "ragged": R.make_config([A(3, 10, 6, 14, 10, 18, scaling=YARN, mlp=E(5, 2, 18)), D(3, 3, 12, vdim=10, conv=3, mlp=M(50)),
                                 G(30, 3, conv=5, mlp=E(4, 4, 6))], vocab=101, width=44, side_dim=5),
        # sizes for the matrix-core kernels: multiples of 32, many heads
        "mfma": R.make_config([A(10, 32, 32, 32, 64, 48, scaling=YARN, mlp=M(64)), D(4, 2, 32, vdim=64, mlp=E(6, 2, 32)),
                               A(3, 64, 64, 32, 96, 64, mlp=None)], width=128),
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
@pytest.mark.parametrize("width", [40, 256, 2500])
def test_norm_after_the_sum(width):
    from vllm_legacy_amd import _seq_ops as ops
    x, y, w = rnd((5, width), 1), rnd((5, width), 2, 3.0), 1 + 0.3 * rnd((width, ), 3)
    want = R.rms_norm(1.7 * x.to(F) + y.to(F), w.to(F), 1e-5)
    for ydt in (torch.float32, torch.bfloat16):
        xs, h = x.to(DEV).clone(), torch.empty((5, width), dtype=torch.bfloat16, device=DEV)
        ops.post_norm(xs, y.to(ydt).to(DEV), w.to(DEV), 1.7, 1e-5, h)
        close(xs, want, 2e-6 if ydt == torch.float32 else 2e-2)
        assert torch.equal(h, xs.to(torch.bfloat16))
    out = torch.empty((5, width), dtype=torch.float32, device=DEV)
    ops.rms_norm_rows(out, x.to(DEV), w.to(DEV), 1e-5)
    close(out, R.rms_norm(x.to(F), w.to(F), 1e-5), 2e-6)
    # a plain copy of the stream in another dtype, and the logit cap
    ops.residual_norms(xs, out=h)
    assert torch.equal(h, xs.to(torch.bfloat16))
    z = (8 * x).to(DEV).contiguous()
    ops.softcap(z, 5.0)
    close(z, 5.0 * torch.tanh(8 * x.to(F) / 5.0), 2e-6)


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
@pytest.mark.parametrize("act,bias", [("silu", False), ("none", True)])
def test_short_convolution_across_cuts_and_slots(taps, act, bias):
    from vllm_legacy_amd.layers import ShortConv
    C = 70
    conv = ShortConv(C, taps, bias, act, DEV)
    conv.weight.data = rnd((C, taps), 1, 0.5).to(DEV)
    if bias:
        conv.bias.data = rnd((C, ), 2).to(DEV)
    state = torch.full(ShortConv.get_state_shape(3, C, taps), 7.0, device=DEV)     # stale slots
    seqs = {"a": rnd((23, C), 3), "b": rnd((9, C), 4), "c": rnd((2, C), 5)}

    def want(u):
        z = R.short_convolution(u.to(F), conv.weight.data.cpu().to(F), conv.bias.data.cpu().to(F) if bias else None)
        return R.silu(z) if act == "silu" else z

    # steps: (sequence, rows, slot); b ends and c takes its slot
    plan = [[("a", 5, 0), ("b", 1, 2)], [("b", 8, 2), ("a", 1, 0)], [("a", 2, 0), ("c", 1, 2)], [("c", 1, 2), ("a", 15, 0)]]
    at, got = {k: 0 for k in seqs}, {k: [] for k in seqs}
    for step in plan:
        u = torch.cat([seqs[k][at[k]:at[k] + n] for k, n, _ in step]).to(DEV)
        # the input is a slice of a wider matrix, as in the models
        wide = torch.zeros((u.shape[0], C + 9), device=DEV)
        wide[:, 4:4 + C] = u
        batch = make_batch([n for _, n, _ in step], [at[k] for k, _, _ in step], slots=[s for _, _, s in step])
        out = torch.empty((u.shape[0], C), dtype=torch.float32, device=DEV)
        conv(out, wide[:, 4:4 + C], state, batch)
        lo = 0
        for k, n, _ in step:
            got[k].append(out[lo:lo + n].cpu())
            lo += n
            at[k] += n
    for k in seqs:
        close(torch.cat(got[k]), want(seqs[k]), 2e-6, k)


# ----------------------------------------------------------------------------- gated delta rule
def run_delta(H, G, D, V, rows, cuts, seed=0, craft=None):
    """rows tokens of one sequence through the kernel in portions `cuts`, beside a second sequence;
    returns (got [rows, H, V], want)."""
    from vllm_legacy_amd.attention.recurrent import GatedDeltaRule
    rule = GatedDeltaRule(H, G, D, V, 1e-5, DEV)
    rule.a_log.data, rule.dt_bias.data = rnd((H, ), seed + 1, 0.5).to(DEV), rnd((H, ), seed + 2, 0.5).to(DEV)
    rule.norm_weight.data = (1 + 0.2 * rnd((V, ), seed + 3)).to(DEV)
    q, k, v, g = rnd((rows, G * D), seed + 4), rnd((rows, G * D), seed + 5), rnd((rows, H * V), seed + 6), rnd((rows, H * V), seed + 7)
    beta, dt = rnd((rows, H), seed + 8, 2.0), rnd((rows, H), seed + 9, 2.0) - 3.0
    if craft is not None:
        craft(q, k, v, beta, dt)
    other = 5
    state = torch.full(GatedDeltaRule.get_state_shape(3, H, D, V), 3.0, device=DEV)        # stale slots
    got, lo = [], 0
    for i, n in enumerate(cuts):
        batch = make_batch([other, n], [i * other, lo], slots=[0, 2])

        def both(t, seed2):
            return torch.cat([rnd((other, t.shape[1]), seed2 + i), t[lo:lo + n]]).to(DEV)

        out = torch.empty((other + n, H * V), dtype=torch.float32, device=DEV)
        rule(out, both(q, 50), both(k, 60), both(v, 70), both(g, 80), both(beta, 90), both(dt, 100), state, batch)
        got.append(out[other:].cpu())
        lo += n
    assert lo == rows
    qn = q.to(F).view(rows, G, D)
    kn = k.to(F).view(rows, G, D)
    qn = qn / torch.sqrt((qn * qn).sum(-1, keepdim=True) + 1e-6) * D**-0.5
    kn = kn / torch.sqrt((kn * kn).sum(-1, keepdim=True) + 1e-6)
    decay = torch.exp(-torch.exp(rule.a_log.data.cpu().to(F)) * R.softplus(dt.to(F) + rule.dt_bias.data.cpu().to(F)))
    o = torch.stack([R.delta_rule(qn[:, h // (H // G)], kn[:, h // (H // G)], v.to(F).view(rows, H, V)[:, h],
                                  torch.sigmoid(beta.to(F))[:, h], decay[:, h]) for h in range(H)], 1)
    want = R.rms_norm(o, rule.norm_weight.data.cpu().to(F), 1e-5) * R.silu(g.to(F)).view(rows, H, V)
    return torch.cat(got).view(rows, H, V), want


@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (3, 1, 24, 40), (2, 2, 128, 128), (1, 1, 200, 72), (5, 5, 8, 12)])
@pytest.mark.parametrize("kernel", [0, 1, 2])
def test_delta_rule_whole_cut_and_token_by_token(shape, kernel):
    """kernel 0: as a step picks it; 1: every run on the kernel for short runs; 2: every run staged."""
    from vllm_legacy_amd import _seq_ops as ops
    rows = 45
    ops.set_delta_kernel(kernel)
    try:
        for cuts in ([rows], [2, 17, 3, 23], [1] * rows):
            got, want = run_delta(*shape, rows, cuts)
            close(got, want, 3e-5, (shape, cuts[:3]))
    finally:
        ops.set_delta_kernel(0)


def test_delta_rule_reads_a_write_from_hundreds_of_tokens_back():
    """Token 3 writes a value along a key no later token touches; decays are near one; token 400
    asks for it with that key.  What it reads is that value, whatever came between."""
    H, G, D, V, rows = 2, 1, 32, 32, 420

    def craft(q, k, v, beta, dt):
        k[:, 0] = 0.0               # nobody else writes along the first axis
        q[:, 0] = 0.0
        k[3] = 0.0
        k[3, 0] = 5.0
        v[3] = 40.0 * torch.sign(v[3])
        beta[3] = 9.0
        q[400] = 0.0
        q[400, 0] = 5.0
        dt[:] = -9.0                # decay close to one

    got, want = run_delta(H, G, D, V, rows, [390, 5, 5, 1, 19], craft=craft)
    assert float(want[400].abs().max()) > 0.5
    close(got[400], want[400], 3e-5)
    close(got, want, 1e-4)


# ----------------------------------------------------------------------------- real-gated recurrence
@pytest.mark.parametrize("channels,blocks", [(48, 3), (256, 1), (700, 700), (640, 5)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_real_gated_recurrence_short_long_and_cut(channels, blocks, dtype):
    from vllm_legacy_amd.attention.recurrent import RealGatedLRU
    lru = RealGatedLRU(channels, blocks, 8.0, DEV)
    bw = channels // blocks
    ra, ri = rnd((blocks, bw, bw), 1, bw**-0.5), rnd((blocks, bw, bw), 2, bw**-0.5)
    rab, rib, lam = rnd((blocks, bw), 3), rnd((blocks, bw), 4), rnd((channels, ), 5) - 2.0
    lru.set_weights(ra, rab, ri, rib, lam)
    n = 600
    u, y = rnd((n, channels), 6), rnd((n, channels), 7)
    ub = u.to(F).view(n, blocks, bw)
    r = torch.sigmoid(torch.einsum("boi,nbi->nbo", ra.to(F), ub) + rab.to(F)).reshape(n, channels)
    i = torch.sigmoid(torch.einsum("boi,nbi->nbo", ri.to(F), ub) + rib.to(F)).reshape(n, channels)
    want = R.rglru_recurrence(u.to(F), r, i, lam.to(F)) * R.gelu_tanh(y.to(F))
    state = torch.full(RealGatedLRU.get_state_shape(2, channels), 5.0, device=DEV)
    for cuts in ([n], [3, 1, 300, 2, 294], [257, 343]):
        got, lo = [], 0
        for c in cuts:
            out = torch.empty((c, channels), dtype=dtype, device=DEV)
            lru(out, u[lo:lo + c].to(DEV).contiguous(), y[lo:lo + c].to(DEV), state, make_batch([c], [lo], slots=[1]))
            got.append(out.float().cpu())
            lo += c
        close(torch.cat(got), want, 2e-5 if dtype == torch.float32 else 1e-2, cuts)


# ----------------------------------------------------------------------------- latent attention
LATENT_SHAPES = [(4, 16, 8, 16, 24), (3, 12, 6, 20, 10), (2, 16, 0, 16, 16), (10, 32, 32, 32, 64), (16, 64, 64, 32, 128),
                 (40, 32, 32, 16, 96), (5, 32, 0, 32, 32), (2, 64, 16, 64, 512), (64, 32, 48, 32, 160)]


def latent_layer_of(shape, dtype, scaling=None, seed=0):
    from vllm_legacy_amd.attention.backends.latent_kv import LatentKVAttention
    H, D, Rr, V, C = shape
    attn = LatentKVAttention(H, D, Rr, V, C, 0.3, Rr, 500.0, scaling, 1e-5, dtype, DEV)
    uk, uv, nw = rnd((H * D, C), seed + 1, C**-0.5), rnd((H * V, C), seed + 2, C**-0.5), 1 + 0.2 * rnd((C, ), seed + 3)
    attn.set_weights(uk, uv, nw)
    return attn, uk.to(dtype).to(F), uv.to(dtype).to(F), nw.to(F)


def latent_reference(shape, q, kv, uk, uv, nw, scaling):
    H, D, Rr, V, C = shape
    n = q.shape[0]
    rot = {"dims": Rr, "base": 500.0, **({"scaling": scaling} if scaling else {})}
    pos = torch.arange(n)
    q3 = q.to(F).view(n, H, D + Rr)
    c = R.rms_norm(kv.to(F)[:, :C], nw, 1e-5)
    k_rot = R.rotate_interleaved(kv.to(F)[:, None, C:], pos, rot)[:, 0] if Rr else torch.zeros(n, 0, dtype=F)
    q_rot = R.rotate_interleaved(q3[..., D:], pos, rot) if Rr else torch.zeros(n, H, 0, dtype=F)
    q_lat = torch.einsum("nhd,hdc->nhc", q3[..., :D], uk.view(H, D, C))
    o = R.latent_attention_core(q_lat, q_rot, c, k_rot, 0.3)
    return torch.einsum("nhc,hvc->nhv", o, uv.view(H, V, C)).reshape(n, H * V), c, k_rot


@pytest.fixture
def plain_kernels():
    """Keeps latent attention off the matrix cores for one test."""
    from vllm_legacy_amd import _seq_ops as ops
    ops.set_latent_attention_kernel(1)
    yield
    ops.set_latent_attention_kernel(0)


@pytest.mark.parametrize("shape", [s for s in LATENT_SHAPES if s[4] % 32 == 0 and s[2] % 16 == 0])
def test_latent_attention_without_the_matrix_cores(shape, plain_kernels):
    test_latent_attention_prompt_portions_and_decoding(shape, torch.bfloat16)


@pytest.mark.parametrize("shape", LATENT_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_attention_prompt_portions_and_decoding(shape, dtype):
    from vllm_legacy_amd.attention.backends.latent_kv import LatentKVAttention
    H, D, Rr, V, C = shape
    scaling = YARN if Rr else None
    attn, uk, uv, nw = latent_layer_of(shape, dtype, scaling)
    n = 75
    q, kv = rnd((n, H * (D + Rr)), 7).to(dtype), rnd((n, C + Rr), 8).to(dtype)
    want, c, k_rot = latent_reference(shape, q, kv, uk, uv, nw, scaling)
    table = [5, 2, 9, 0, 7, 11, 3, 1, 12, 4, 13, 6, 8, 10, 14, 15, 16, 17, 18][:(n + 3) // 4]      # pages out of order
    cache = torch.zeros(LatentKVAttention.get_cache_shape(20, 4, C, Rr), dtype=dtype, device=DEV)
    for cuts in ([n], [2, 33, 1, 1, 30, 3, 5], [40] + [1] * 35):
        cache.fill_(9.0)
        got, lo = [], 0
        for m in cuts:
            batch = make_batch([m], [lo], tables=[table])
            got.append(attn(q[lo:lo + m].to(DEV).clone(), kv[lo:lo + m].to(DEV), cache, batch).float().cpu())
            lo += m
        tol = 3e-5 if dtype == torch.float32 else 4e-2
        close(torch.cat(got), want, tol, cuts[:3])
    # what the cache holds: the normed latent and the rotated shared key part, page by page
    rows = torch.cat([cache[b] for b in table]).float().cpu()[:n]
    close(rows[:, :C], c, 2e-6 if dtype == torch.float32 else 1e-2)
    if Rr:
        close(rows[:, C:], k_rot, 2e-6 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("far", [0, 3, 4, 255, 256, 300])
def test_latent_attention_a_far_key_carries_the_output(dtype, far):
    """One key hundreds of positions back, at a page's first or last place or the very first of the
    sequence, scores far above the rest for the last queries (in a prompt's portion and decoded
    alone): their output is that key's value."""
    from vllm_legacy_amd.attention.backends.latent_kv import LatentKVAttention
    shape = (4, 32, 32, 32, 64)
    H, D, Rr, V, C = shape
    attn, uk, uv, nw = latent_layer_of(shape, dtype, None, seed=5)
    n = 520
    q, kv = rnd((n, H * (D + Rr)), 9, 0.3), rnd((n, C + Rr), 10)
    # the far key's latent is large along what head 1's query, through W_uk, asks for
    ask = rnd((D, ), 11)
    lat = (uk.view(H, D, C)[1].T @ ask.to(F)).float()
    kv[far, :C] = 6.0 * lat / lat.norm() * C**0.5
    q3 = q.view(n, H, D + Rr)
    q3[500:, 1, :D] = 8.0 * ask / ask.norm()
    q, kv = q.to(dtype), kv.to(dtype)
    want, _, _ = latent_reference(shape, q, kv, uk, uv, nw, None)
    cache = torch.zeros(LatentKVAttention.get_cache_shape(40, 16, C, Rr), dtype=dtype, device=DEV)
    table = list(range(39, 39 - 33, -1))
    got, lo = [], 0
    for m in [257, 250] + [1] * 13:
        batch = make_batch([m], [lo], block_size=16, tables=[table])
        got.append(attn(q[lo:lo + m].to(DEV).clone(), kv[lo:lo + m].to(DEV), cache, batch).float().cpu())
        lo += m
    got = torch.cat(got)
    alone = latent_reference(shape, q[far:far + 1], kv[far:far + 1], uk, uv, nw, None)[0]   # the key's own value
    assert float((want[505].view(H, V)[1] - alone.view(H, V)[1]).abs().max()) < 0.05 * float(alone.abs().max())
    close(got[500:], want[500:], 3e-5 if dtype == torch.float32 else 4e-2)
    close(got, want, 3e-5 if dtype == torch.float32 else 6e-2)


# ----------------------------------------------------------------------------- feed-forwards, side input
@pytest.mark.parametrize("shape", [(64, 6, 2, 24), (40, 3, 1, 20), (128, 5, 5, 64), (96, 12, 3, 32)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [3, 300])
def test_gated_experts_with_a_router_bias(shape, dtype, rows):
    from vllm_legacy_amd.routed_experts import RoutedExperts
    W, E, top, ff = shape
    moe = RoutedExperts(W, E, 0, top, ff, 0, "silu", dtype=dtype, device=DEV, gated=True, router_bias=True)
    t = {"router": rnd((E, W), 1, W**-0.5), "router.b": rnd((E, ), 2, 2.0)}     # the bias decides many choices
    for e in range(E):
        t[f"e{e}.gate"], t[f"e{e}.up"], t[f"e{e}.down"] = rnd((ff, W), 10 + e, W**-0.5), rnd((ff, W), 30 + e, W**-0.5), rnd((W, ff), 50 + e, ff**-0.5)
    t = {k: v.to(torch.bfloat16) for k, v in t.items()}
    moe.set_weights(t)
    h = rnd((rows, W), 3).to(dtype)
    want = R.routed_ff(h.to(F), {k: v.to(F) for k, v in t.items()}, {"router": {"experts": E, "top": top}})
    got = moe(h.to(DEV)).cpu()
    err = (got.to(F) - want).abs().amax(1) / want.abs().max()
    if dtype == torch.float32:
        assert float(err.max()) <= 2e-5
    else:       # a close call of the router may go the other way for a few rows
        assert float(torch.quantile(err, 0.9)) <= 3e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_side_input_and_scaled_embedding(dtype):
    from vllm_legacy_amd import _seq_ops as ops
    from vllm_legacy_amd.layers import TokenGatedInput
    W, dim, layers, vocab, n = 72, 6, 3, 31, 9
    table = rnd((vocab, layers * dim), 1).to(dtype)
    ids = torch.randint(0, vocab, (n, ), generator=torch.Generator().manual_seed(2))
    x = rnd((n, W), 3)
    for layer in range(layers):
        side = TokenGatedInput(W, dim, layer * dim, 1e-5, "gelu_tanh", dtype, DEV)
        t = {"gate": rnd((dim, W), 4 + layer, W**-0.5).to(dtype), "proj": rnd((W, dim), 8 + layer).to(dtype),
             "norm": 1 + 0.2 * rnd((W, ), 12)}
        side.gate.data, side.proj.data, side.weight.data = t["gate"].to(DEV), t["proj"].to(DEV), t["norm"].to(DEV)
        xs = x.to(DEV).clone()
        h = xs.to(dtype)
        want = R.token_side_input(h.cpu().to(F), table.to(F)[ids][:, layer * dim:(layer + 1) * dim],
                                  {k: v.to(F) for k, v in t.items()}, 1e-5) - h.cpu().to(F) + x.to(F)
        side(xs, h, table.to(DEV), ids.to(DEV))
        close(xs, want, 3e-6 if dtype == torch.float32 else 2e-2, layer)
        assert torch.equal(h, xs.to(dtype))
    emb = torch.empty((n, layers * dim), dtype=torch.float32, device=DEV)
    ops.embed_scaled(emb, table.to(DEV), ids.to(DEV), 2.5)
    close(emb, table.to(F)[ids] * 2.5, 1e-6)


# ----------------------------------------------------------------------------- whole models
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


@pytest.mark.parametrize("name", ["plain", "odd", "equal", "ragged"])
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
    assert type(engine.runner.model).__name__ == "LamosunForCausalLM"
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
